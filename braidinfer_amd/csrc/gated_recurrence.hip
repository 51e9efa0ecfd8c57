// A gated linear recurrence per head, state in float: for a head with d query channels and e
// value channels,
//     S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T      (S is d x e, starts at zero)
//     o_t = S_t^T q_t
// with the forget gate f_t in (lower, 1) per channel deciding what stays and what is written
// (no key, no further scale).  The columns of S never meet: column c follows
// S[:, c] <- f * S[:, c] + (1 - f) * v[c], so the work is cut by (sequence, head, 64 columns).
//
// Three kernels: `gates` turns the projections' float sums into q = silu(.) and
// f = lower + (1 - lower) * sigmoid(. + bias) in place (parallel over tokens), `scan` walks a
// sequence's new tokens in order from the state its slot holds and leaves the state behind,
// `head_norm` is the RMS norm of every head's output over its e channels.
#include "common.h"

// ---------------------------------------------------------------------- gates ------
// rows [T, 2 * hd + he]: q | f | v (hd = heads * d); q and f are rewritten.
__global__ void glr_gates_kernel(float* __restrict__ rows, const float* __restrict__ f_bias,
                                 const float* __restrict__ lower, int hd, int width, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / (2 * (size_t)hd);
    const int c = (int)(i - t * 2 * (size_t)hd);
    float* r = rows + t * width;
    const float z = r[c];
    if (c < hd) r[c] = z / (1.0f + expf(-z));
    else {
        const int k = c - hd;
        const float lo = lower ? lower[k] : 0.f;
        const float g = 1.0f / (1.0f + expf(-(z + (f_bias ? f_bias[k] : 0.f))));
        r[c] = lo + (1.0f - lo) * g;
    }
}

extern "C" int br_glr_gates(float* rows, const float* f_bias, const float* lower, int T, int hd, int width,
                            hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (hd <= 0 || width < 2 * hd) return BR_BAD_ARG;
    const size_t n = (size_t)T * 2 * hd;
    glr_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(rows, f_bias, lower, hd, width, n);
    return br_check_launch();
}

// ----------------------------------------------------------------------- scan ------
// grid (sequences, heads, ceil(e / 64)), 256 threads: thread (c, g) owns column c of the
// workgroup's 64 and the rows g, g + 4, g + 8, ... of S, RPT of them in registers.  The four
// row groups' shares of o_t[c] are added in group order through LDS.
template <int RPT>
__global__ __launch_bounds__(256) void glr_scan_kernel(
    const float* __restrict__ rows, float* __restrict__ o, float* __restrict__ state,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots, int H, int d, int e, int width,
    size_t slot_stride) {
    __shared__ float part[2][4][64];
    const int s = blockIdx.x, h = blockIdx.y;
    const int cl = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int c = blockIdx.z * 64 + cl;
    const int slot = slots[s];
    if (slot < 0) return;
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const bool live = c < e;
    float* S = state + (size_t)slot * slot_stride + ((size_t)h * d) * e;
    float st[RPT];
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
        const int r = g + 4 * k;
        st[k] = (live && r < d) ? S[(size_t)r * e + c] : 0.f;
    }
    const int hd = H * d;
    for (int t = t0; t < t1; ++t) {
        const float* row = rows + (size_t)t * width;
        const float* qr = row + h * d;
        const float* fr = row + hd + h * d;
        const float vc = live ? row[2 * hd + h * e + c] : 0.f;
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < RPT; ++k) {
            const int r = g + 4 * k;
            if (r < d) {
                const float f = fr[r];
                st[k] = fmaf(f, st[k], (1.0f - f) * vc);
                sum = fmaf(st[k], qr[r], sum);
            }
        }
        float (*pt)[64] = part[(t - t0) & 1];
        pt[g][cl] = sum;
        __syncthreads();
        if (g == 0 && live)
            o[(size_t)t * H * e + h * e + c] = ((pt[0][cl] + pt[1][cl]) + pt[2][cl]) + pt[3][cl];
    }
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
        const int r = g + 4 * k;
        if (live && r < d) S[(size_t)r * e + c] = st[k];
    }
}

// `slot_stride`: floats from one slot's state to the next (at least H * d * e).
extern "C" int br_glr_scan(const float* rows, float* o, float* state, const int* cu_seqlens, const int* slots,
                           int B, int H, int d, int e, int width, size_t slot_stride, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (H <= 0 || H > 65535 || d <= 0 || e <= 0 || d > 512 || width < 2 * H * d + H * e ||
        slot_stride < (size_t)H * d * e)
        return BR_BAD_ARG;
    dim3 grid(B, H, (e + 63) / 64);
    const int rpt = (d + 3) / 4;
#define GLR_SCAN(R) glr_scan_kernel<R><<<grid, 256, 0, s>>>(rows, o, state, cu_seqlens, slots, H, d, e, width, slot_stride)
    if (rpt <= 8) GLR_SCAN(8);
    else if (rpt <= 16) GLR_SCAN(16);
    else if (rpt <= 32) GLR_SCAN(32);
    else if (rpt <= 64) GLR_SCAN(64);
    else GLR_SCAN(128);
#undef GLR_SCAN
    return br_check_launch();
}

// ------------------------------------------------------------------ head norm ------
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w, one wave per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void glr_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                           T* __restrict__ y, int e, float eps) {
    const size_t base = ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * e;
    float ss = 0.f;
    for (int i = threadIdx.x; i < e; i += 64) { const float v = o[base + i]; ss += v * v; }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)e + eps);
    for (int i = threadIdx.x; i < e; i += 64) y[base + i] = from_f32<T>(o[base + i] * inv * (w ? w[i] : 1.0f));
}

extern "C" int br_glr_head_norm(const float* o, const float* w, void* y, int y_is_bf16, int T, int H, int e,
                                float eps, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || H > 65535 || e <= 0) return BR_BAD_ARG;
    dim3 grid(T, H);
    if (y_is_bf16) glr_head_norm_kernel<bf16><<<grid, 64, 0, s>>>(o, w, (bf16*)y, e, eps);
    else glr_head_norm_kernel<float><<<grid, 64, 0, s>>>(o, w, (float*)y, e, eps);
    return br_check_launch();
}
