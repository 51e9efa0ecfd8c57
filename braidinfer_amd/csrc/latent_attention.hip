// Attention through a latent: per token the cache keeps one row, the normed latent c (R elements) followed
// by a rotated key part shared by all heads (DR elements).  A head's key is W_uk c beside that part and its
// value W_uv c, so with the query's unrotated part taken through W_uk^T first,
//     score = (W_uk^T q_u) . c + q_r . k_r,        output = W_uv (sum_j p_j c_j),
// which is attention of all heads over ONE row per token: keys [c | k_r] (R + DR wide), values c (R wide).
// The products with W_uk^T and W_uv are the library's matrix products head by head, the attention itself is
// the kernels of `pooled_attention.hip` with one kv head; this file prepares their operands.
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
