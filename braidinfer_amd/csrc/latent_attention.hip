// Attention through a latent: per token the cache keeps one row, the normed latent c (R elements) followed
// by a rotated key part shared by all heads (DR elements).  A head's key is W_uk c beside that part and its
// value W_uv c, so with the query's unrotated part taken through W_uk^T first,
//     score = (W_uk^T q_u) . c + q_r . k_r,        output = W_uv (sum_j p_j c_j),
// which is attention of all heads over ONE row per token: keys [c | k_r] (R + DR wide), values c (R wide).
// The attention itself is the kernels of `pooled_attention.hip` with one kv head; this file prepares their
// operands (`prepare`) and multiplies head by head (`head_linear`: the products with W_uk^T and W_uv).
//
// `prepare`, a workgroup per token:
//   * c = rms_norm(dkv[0:R]) * weight and k_r = rotate(dkv[R:R+DR]) into the token's cache page: the key row
//     [c | k_r], and c once more transposed ([channel][row]) where those kernels read their values;
//   * per head, the query's unrotated part (the products' type) into `q_plain` [T, H, D] and its rotated part
//     into `q_wide` [T, H, R + DR] at offset R (the first R elements are the product's that follows).
// Rotation: elements 2i and 2i + 1 of the first `rot` elements of a rotated part are a pair turned by the
// token's angle i (cos and sin come as tables [T, rot / 2], with any factor on them already in); elements
// from `rot` on pass unchanged.  Sums, norms and angles are float in both precisions.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const float* __restrict__ q, size_t q_stride, const float* __restrict__ dkv, size_t dkv_stride,
    const float* __restrict__ c_weight, float eps, const float* __restrict__ cs, const float* __restrict__ sn,
    const int* __restrict__ pos, const int* __restrict__ seq_of_token, const int* __restrict__ slots,
    const int* __restrict__ block_table, int table_stride, T* __restrict__ cache, T* __restrict__ q_plain,
    T* __restrict__ q_wide, int H, int D, int DR, int R, int rot, int page) {
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int half = rot >> 1;
    const float* ct = cs + (size_t)t * half;
    const float* st = sn + (size_t)t * half;
    // queries: every head's plain part as it is, its rotated part turned
    const float* qr = q + (size_t)t * q_stride;
    const int per = D + DR, wide = R + DR;
    for (int i = tid; i < H * D; i += 256) {
        const int hh = i / D, j = i - hh * D;
        q_plain[(size_t)t * H * D + i] = from_f32<T>(qr[hh * per + j]);
    }
    for (int i = tid; i < H * DR; i += 256) {
        const int hh = i / DR, j = i - hh * DR;
        const float* src = qr + hh * per + D;
        float v = src[j];
        if (j < rot) {
            const int p = j >> 1;
            const float other = src[j ^ 1];
            v = (j & 1) ? v * ct[p] + other * st[p] : v * ct[p] - other * st[p];
        }
        q_wide[((size_t)t * H + hh) * wide + R + j] = from_f32<T>(v);
    }
    if (!dkv) return;                       // a layer that reads another layer's rows
    const int slot = slots[seq_of_token[t]];
    if (slot < 0) return;                   // padding: nothing is kept
    const float* xr = dkv + (size_t)t * dkv_stride;
    float ss = 0.f;
    for (int i = tid; i < R; i += 256) { const float v = xr[i]; ss += v * v; }
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)R + eps);
    const int p = pos[t];
    const int pg = block_table[(size_t)slot * table_stride + p / page], row = p % page;
    T* krow = cache + (size_t)pg * page * (wide + R) + (size_t)row * wide;
    T* vcol = cache + (size_t)pg * page * (wide + R) + (size_t)page * wide + row;
    for (int i = tid; i < R; i += 256) {
        const T c = from_f32<T>(xr[i] * inv * c_weight[i]);
        krow[i] = c;
        vcol[(size_t)i * page] = c;
    }
    for (int j = tid; j < DR; j += 256) {
        float v = xr[R + j];
        if (j < rot) {
            const int pr = j >> 1;
            const float other = xr[R + (j ^ 1)];
            v = (j & 1) ? v * ct[pr] + other * st[pr] : v * ct[pr] - other * st[pr];
        }
        krow[R + j] = from_f32<T>(v);
    }
}

// q float [T, >= H (D + DR)] rows `q_stride` apart; dkv float [T, >= R + DR] rows `dkv_stride` apart, or null for a
// layer that keeps nothing itself; cache [pages][page (R + DR) keys, then R x page values] of the products' type;
// q_plain [T, H, D], q_wide [T, H, R + DR].
extern "C" int br_latent_prepare(const float* q, size_t q_stride, const float* dkv, size_t dkv_stride, const float* c_weight,
                                 float eps, const float* cs, const float* sn, const int* pos, const int* seq_of_token,
                                 const int* slots, const int* block_table, int table_stride, void* cache, void* q_plain,
                                 void* q_wide, int is_bf16, int T, int H, int D, int DR, int R, int rot, int page, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || D <= 0 || DR < 0 || R <= 0 || rot < 0 || rot > DR || rot % 2 || page <= 0 || q_stride < (size_t)H * (D + DR) ||
        (rot > 0 && (!cs || !sn)) || (dkv && (dkv_stride < (size_t)(R + DR) || !c_weight || !cache || !block_table)))
        return BR_BAD_ARG;
    if (is_bf16) latent_prepare_kernel<bf16><<<T, 256, 0, s>>>(q, q_stride, dkv, dkv_stride, c_weight, eps, cs, sn, pos, seq_of_token,
        slots, block_table, table_stride, (bf16*)cache, (bf16*)q_plain, (bf16*)q_wide, H, D, DR, R, rot, page);
    else latent_prepare_kernel<float><<<T, 256, 0, s>>>(q, q_stride, dkv, dkv_stride, c_weight, eps, cs, sn, pos, seq_of_token,
        slots, block_table, table_stride, (float*)cache, (float*)q_plain, (float*)q_wide, H, D, DR, R, rot, page);
    return br_check_launch();
}

// ------------------------------------------------------- a product head by head -----
// out[t, h, n] = sum_k a[t, h, k] * w[h, n, k]: every head's rows through a matrix of its own, all heads in one
// launch (the products with W_uk^T and W_uv around the attention).  a and out are [T, H, .] views: rows `lda` /
// `ldo` elements apart, heads `a_hs` / `o_hs` apart; w is [H, N, K] dense.
//
// bfloat16 on the matrix cores: a wave owns 32 outputs n x 32 tokens t and walks k 16 at a time with
// v_mfma_f32_32x32x16_bf16, the weight rows as the first operand (so a lane ends with four neighbouring n of one
// token in four neighbouring registers), both operands straight from memory 16 bytes a lane; four waves a
// workgroup side by side along n.  grid (ceil(T / 32), ceil(N / 128), H).  K in steps of 8, rows and heads of a
// at multiples of 16 bytes.
__global__ __launch_bounds__(256) void head_linear_bf16_kernel(const bf16* __restrict__ a, size_t lda, size_t a_hs,
                                                               const bf16* __restrict__ w, bf16* __restrict__ out, size_t ldo,
                                                               size_t o_hs, int T, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, g = lane >> 5;
    const int t0 = blockIdx.x * 32, n0 = blockIdx.y * 128 + wave * 32, h = blockIdx.z;
    if (n0 >= N) return;
    const int t = t0 + c, nrow = n0 + c;
    const bf16* wrow = w + ((size_t)h * N + (nrow < N ? nrow : N - 1)) * K;
    const bf16* arow = a + (size_t)(t < T ? t : T - 1) * lda + (size_t)h * a_hs;
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    bf16x8 zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
        const int k = k0 + 8 * g;
        const bf16x8 wf = (k < K && nrow < N) ? *(const bf16x8*)(wrow + k) : zero;
        const bf16x8 af = (k < K && t < T) ? *(const bf16x8*)(arow + k) : zero;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, af, acc, 0, 0, 0);
    }
    if (t >= T) return;
    bf16* orow = out + (size_t)t * ldo + (size_t)h * o_hs;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int n = n0 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (n < N) orow[n] = (bf16)acc[r];
    }
}

// Any type and alignment: a thread an output, float sums in ascending k.
template <typename T>
__global__ __launch_bounds__(256) void head_linear_plain_kernel(const T* __restrict__ a, size_t lda, size_t a_hs,
                                                                const T* __restrict__ w, T* __restrict__ out, size_t ldo,
                                                                size_t o_hs, int n_tok, int H, int N, int K) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)n_tok * H * N) return;
    const int n = (int)(i % N), h = (int)((i / N) % H);
    const size_t t = i / ((size_t)N * H);
    const T* ar = a + t * lda + (size_t)h * a_hs;
    const T* wr = w + ((size_t)h * N + n) * K;
    float s = 0.f;
    for (int k = 0; k < K; ++k) s = fmaf(to_f32<T>(ar[k]), to_f32<T>(wr[k]), s);
    out[t * ldo + (size_t)h * o_hs + n] = from_f32<T>(s);
}

extern "C" int br_head_linear(const void* a, size_t lda, size_t a_hs, const void* w, void* out, size_t ldo, size_t o_hs,
                              int is_bf16, int T, int H, int N, int K, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || N <= 0 || K <= 0 || H > 65535 || (N + 127) / 128 > 65535) return BR_BAD_ARG;
    if (is_bf16 && K % 8 == 0 && lda % 8 == 0 && a_hs % 8 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0) {
        dim3 grid((T + 31) / 32, (N + 127) / 128, H);
        head_linear_bf16_kernel<<<grid, 256, 0, s>>>((const bf16*)a, lda, a_hs, (const bf16*)w, (bf16*)out, ldo, o_hs, T, N, K);
        return br_check_launch();
    }
    const size_t n = (size_t)T * H * N;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (is_bf16) head_linear_plain_kernel<bf16><<<blocks, 256, 0, s>>>((const bf16*)a, lda, a_hs, (const bf16*)w, (bf16*)out, ldo, o_hs, T, H, N, K);
    else head_linear_plain_kernel<float><<<blocks, 256, 0, s>>>((const float*)a, lda, a_hs, (const float*)w, (float*)out, ldo, o_hs, T, H, N, K);
    return br_check_launch();
}
