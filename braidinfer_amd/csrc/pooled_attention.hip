// Attention over a sliding window plus pooled blocks of the tokens that left it, over the
// paged cache, in float arithmetic for both storage types.
//
// A query at position p of its sequence sees the tokens lo..p, lo = max(0, p - size + 1),
// and one pooled key and value for every block b of `pool` tokens that lies wholly before
// the window: b * pool + pool - 1 <= p - size.  Pooled rows live in a cache unit of their
// own with one row per block (the means of the block's keys and of its values as the
// token cache holds them); both kinds of key share one softmax, which may carry a sink: a
// key of score 0 without a value, i.e. one added to the denominator.
//
// Three kernels: `prepare` (bias, per-head RMS norm of queries and keys, rotation of the
// first `rd` elements in (i, i + rd/2) pairs, value mixing with another layer's values,
// cache write), `pool` (the means of the blocks that the step completed) and `attend`.
// Keys and values of a page: [kv_head][token][dk] and, behind the keys of all heads,
// [kv_head][token][dv].
//
// The sums of `attend` run over the seen blocks in ascending order and then over the window's
// tokens in ascending position, 64 at a time, so the chunking depends on (p, size, pool) only:
// whole prompts, portions and single tokens give the same bits.
#include "common.h"

#define MAX_EPL 8   // head widths up to 64 * MAX_EPL

// ------------------------------------------------------------------- prepare -------
// qkv [T, nq*dk + nkv*dk + nkv*dv] float (the product's float sums), one wave per (token, head).
// vf_role: 0 none, 1 this layer's values are written to `v_first`, 2 values become
// (1 - lambda) v + lambda v_first.  Tokens of padding sequences (slot < 0) store nothing.
template <typename T>
__global__ __launch_bounds__(64) void pwa_prepare_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ qn_w,
    const float* __restrict__ kn_w, float eps, const float* __restrict__ cs, const float* __restrict__ sn,
    int rd, const int* __restrict__ pos, const int* __restrict__ seq_of_token,
    const int* __restrict__ slots, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ q_out, T* __restrict__ storage, float* __restrict__ v_first,
    const float* __restrict__ lambda, int vf_role, int nq, int nkv, int dk, int dv, int page,
    int write_cache) {
    extern __shared__ float row[];          // [max(dk, dv)]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int width = nq * dk + nkv * dk + nkv * dv;
    const bool is_q = h < nq, is_k = !is_q && h < nq + nkv;
    const int kvh = is_q ? 0 : (is_k ? h - nq : h - nq - nkv);
    const int n = (is_q || is_k) ? dk : dv;
    const int col0 = is_q ? h * dk : (is_k ? nq * dk + kvh * dk : nq * dk + nkv * dk + kvh * dv);
    const float* src = qkv + (size_t)t * width + col0;
    const int slot = slots[seq_of_token[t]];
    const int p = pos[t];
    T* dst = nullptr;
    if (is_q) dst = q_out + ((size_t)t * nq + h) * dk;
    else if (write_cache && slot >= 0) {
        const size_t page_elems = (size_t)nkv * page * (dk + dv);
        const int pg = block_table[(size_t)slot * table_stride + p / page];
        T* pb = storage + (size_t)pg * page_elems;
        dst = is_k ? pb + ((size_t)kvh * page + (p % page)) * dk
                   : pb + (size_t)nkv * page * dk + ((size_t)kvh * page + (p % page)) * dv;
    }
    float v[MAX_EPL];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        v[j] = 0.f;
        if (i < n) {
            v[j] = src[i] + (bias ? bias[col0 + i] : 0.f);
            ss += v[j] * v[j];
        }
    }
    if (is_q || is_k) {
        const float* nw = is_q ? qn_w : kn_w;
        if (nw) {
            const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dk + eps);
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < n) v[j] = v[j] * inv * nw[i];
            }
        }
        if (rd > 0) {
            const int half = rd >> 1;
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < n) row[i] = v[j];
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < rd) {
                    const int f = i < half ? i : i - half;
                    const float c = cs[(size_t)t * half + f], s = sn[(size_t)t * half + f];
                    v[j] = i < half ? row[i] * c - row[i + half] * s : row[i] * c + row[i - half] * s;
                }
            }
        }
    } else if (vf_role) {
        float* vf = v_first + (size_t)t * nkv * dv + (size_t)kvh * dv;
        const float lam = vf_role == 2 ? lambda[0] : 0.f;
#pragma unroll
        for (int j = 0; j < MAX_EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < n) {
                if (vf_role == 1) vf[i] = v[j];
                else v[j] = (1.0f - lam) * v[j] + lam * vf[i];
            }
        }
    }
    if (dst) {
#pragma unroll
        for (int j = 0; j < MAX_EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < n) dst[i] = from_f32<T>(v[j]);
        }
    }
}

extern "C" int br_pwa_prepare(const float* qkv, const float* bias, const float* qn_w, const float* kn_w, float eps,
                              const float* cs, const float* sn, int rd, const int* pos, const int* seq_of_token,
                              const int* slots, const int* block_table, int table_stride, void* q_out,
                              void* storage, int is_bf16, float* v_first, const float* lambda, int vf_role,
                              int T, int nq, int nkv, int dk, int dv, int page, int write_cache, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || nq % nkv || dk <= 0 || dv <= 0 || dk > 64 * MAX_EPL || dv > 64 * MAX_EPL ||
        rd < 0 || rd > dk || (rd & 1) || page <= 0 || nq + 2 * nkv > 65535 || (rd > 0 && (!cs || !sn)) ||
        (vf_role && !v_first) || (vf_role == 2 && !lambda) || vf_role < 0 || vf_role > 2)
        return BR_BAD_ARG;
    dim3 grid(T, nq + 2 * nkv);
    const size_t lds = (size_t)(dk > dv ? dk : dv) * sizeof(float);
    if (is_bf16)
        pwa_prepare_kernel<bf16><<<grid, 64, lds, s>>>(qkv, bias, qn_w, kn_w, eps, cs, sn, rd, pos, seq_of_token, slots,
                                                       block_table, table_stride, (bf16*)q_out, (bf16*)storage, v_first,
                                                       lambda, vf_role, nq, nkv, dk, dv, page, write_cache);
    else
        pwa_prepare_kernel<float><<<grid, 64, lds, s>>>(qkv, bias, qn_w, kn_w, eps, cs, sn, rd, pos, seq_of_token, slots,
                                                        block_table, table_stride, (float*)q_out, (float*)storage,
                                                        v_first, lambda, vf_role, nq, nkv, dk, dv, page, write_cache);
    return br_check_launch();
}

// ---------------------------------------------------------------------- pool -------
// For sequence s with n new tokens ending at length L: the blocks b with
// start <= b * pool + pool - 1 < L (start = L - n) are complete after this step; their means go
// into row b of the pooled unit.  Block floor(start / pool) + blockIdx.y is this workgroup's;
// the grid's second size is max_new / pool + 1.
template <typename T>
__global__ __launch_bounds__(64) void pwa_pool_kernel(
    const T* __restrict__ storage, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ pooled, const int* __restrict__ pooled_table, int pooled_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ ctx_lens, const int* __restrict__ slots,
    int nkv, int dk, int dv, int page, int pool) {
    const int s = blockIdx.x, kvh = blockIdx.z, lane = threadIdx.x;
    const int slot = slots[s];
    if (slot < 0) return;
    const int end = ctx_lens[s];
    const int start = end - (cu_seqlens[s + 1] - cu_seqlens[s]);
    const int b = start / pool + blockIdx.y;
    if ((long long)b * pool + pool > end) return;
    const size_t page_elems = (size_t)nkv * page * (dk + dv);
    const int* bt = block_table + (size_t)slot * table_stride;
    const int ppg = pooled_table[(size_t)slot * pooled_stride + b / page];
    T* pk = pooled + (size_t)ppg * page_elems + ((size_t)kvh * page + (b % page)) * dk;
    T* pv = pooled + (size_t)ppg * page_elems + (size_t)nkv * page * dk + ((size_t)kvh * page + (b % page)) * dv;
    const float inv = 1.0f / (float)pool;
    for (int i = lane; i < dk + dv; i += 64) {
        const bool key = i < dk;
        float acc = 0.f;
        for (int r = 0; r < pool; ++r) {
            const int j = b * pool + r;
            const T* pb = storage + (size_t)bt[j / page] * page_elems;
            acc += key ? to_f32<T>(pb[((size_t)kvh * page + (j % page)) * dk + i])
                       : to_f32<T>(pb[(size_t)nkv * page * dk + ((size_t)kvh * page + (j % page)) * dv + (i - dk)]);
        }
        if (key) pk[i] = from_f32<T>(acc * inv);
        else pv[i - dk] = from_f32<T>(acc * inv);
    }
}

extern "C" int br_pwa_pool(const void* storage, const int* block_table, int table_stride, void* pooled,
                           const int* pooled_table, int pooled_stride, const int* cu_seqlens, const int* ctx_lens,
                           const int* slots, int is_bf16, int B, int max_new, int nkv, int dk, int dv, int page,
                           int pool, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (nkv <= 0 || nkv > 65535 || dk <= 0 || dv <= 0 || page <= 0 || pool <= 0 || max_new <= 0) return BR_BAD_ARG;
    const int per_seq = max_new / pool + 1;
    if (per_seq > 65535) return BR_TOO_LARGE;
    dim3 grid(B, per_seq, nkv);
    if (is_bf16)
        pwa_pool_kernel<bf16><<<grid, 64, 0, s>>>((const bf16*)storage, block_table, table_stride, (bf16*)pooled, pooled_table,
                                                  pooled_stride, cu_seqlens, ctx_lens, slots, nkv, dk, dv, page, pool);
    else
        pwa_pool_kernel<float><<<grid, 64, 0, s>>>((const float*)storage, block_table, table_stride, (float*)pooled,
                                                   pooled_table, pooled_stride, cu_seqlens, ctx_lens, slots, nkv, dk, dv,
                                                   page, pool);
    return br_check_launch();
}

// -------------------------------------------------------------------- attend -------
// One wave per (query token, query head).  Key c of a query: pooled row c for c < nb, the token
// lo + c - nb after that.  Online softmax (m' = max(m, s), corr = exp(m - m'), l = l corr + sum w,
// acc = acc corr + w v); a sink starts it at m = 0, l = 1 instead of m = -inf, l = 0.
template <typename T>
__global__ __launch_bounds__(64) void pwa_attend_kernel(
    const T* __restrict__ q, T* __restrict__ out, const int* __restrict__ pos,
    const int* __restrict__ seq_of_token, const int* __restrict__ slots,
    const int* __restrict__ block_table, int table_stride, const T* __restrict__ storage,
    const int* __restrict__ pooled_table, int pooled_stride, const T* __restrict__ pooled,
    int nq, int nkv, int dk, int dv, int page, int size, int pool, float scale, int sink) {
    extern __shared__ float lds[];
    float* qs = lds;            // [dk]
    float* ps = lds + dk;       // [64]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (nq / nkv);
    T* o = out + ((size_t)t * nq + h) * dv;
    const int slot = slots[seq_of_token[t]];
    if (slot < 0) {
        for (int d = lane; d < dv; d += 64) o[d] = from_f32<T>(0.f);
        return;
    }
    const T* qr = q + ((size_t)t * nq + h) * dk;
    for (int d = lane; d < dk; d += 64) qs[d] = to_f32<T>(qr[d]);
    __syncthreads();
    const int p = pos[t];
    const int lo = (size > 0 && p - size + 1 > 0) ? p - size + 1 : 0;
    int nb = 0;
    if (pool > 0 && size > 0 && p - size - pool + 1 >= 0) nb = (p - size - pool + 1) / pool + 1;
    const int total = nb + (p - lo + 1);
    const int* bt = block_table + (size_t)slot * table_stride;
    const int* pt = pooled_table ? pooled_table + (size_t)slot * pooled_stride : nullptr;
    const size_t page_elems = (size_t)nkv * page * (dk + dv);
    const size_t k_off = (size_t)kvh * page * dk, v_off = (size_t)nkv * page * dk + (size_t)kvh * page * dv;

    float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
    float acc[MAX_EPL];
#pragma unroll
    for (int i = 0; i < MAX_EPL; ++i) acc[i] = 0.f;

    for (int c0 = 0; c0 < total; c0 += 64) {
        const int c = c0 + lane;
        float s = -INFINITY;
        if (c < total) {
            const bool pl = c < nb;
            const int j = pl ? c : lo + (c - nb);
            const T* base = pl ? pooled + (size_t)pt[j / page] * page_elems : storage + (size_t)bt[j / page] * page_elems;
            const T* kr = base + k_off + (size_t)(j % page) * dk;
            float dot = 0.f;
            for (int d = 0; d < dk; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = expf(m - m_new);          // exp(-inf) = 0 on the first chunk without a sink
        const float w = (c < total) ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(w);
        __syncthreads();
        ps[lane] = w;
        __syncthreads();
        const int nk = (total - c0) < 64 ? (total - c0) : 64;
#pragma unroll
        for (int i = 0; i < MAX_EPL; ++i) acc[i] *= corr;
        for (int jj = 0; jj < nk; ++jj) {
            const int cc = c0 + jj;
            const bool pl = cc < nb;
            const int j = pl ? cc : lo + (cc - nb);
            const T* base = pl ? pooled + (size_t)pt[j / page] * page_elems : storage + (size_t)bt[j / page] * page_elems;
            const T* vr = base + v_off + (size_t)(j % page) * dv;
            const float pw = ps[jj];
#pragma unroll
            for (int i = 0; i < MAX_EPL; ++i) {
                const int d = lane + 64 * i;
                if (d < dv) acc[i] = fmaf(pw, to_f32<T>(vr[d]), acc[i]);
            }
        }
        m = m_new;
    }
#pragma unroll
    for (int i = 0; i < MAX_EPL; ++i) {
        const int d = lane + 64 * i;
        if (d < dv) o[d] = from_f32<T>(acc[i] / l);
    }
}

extern "C" int br_pwa_attend(const void* q, void* out, int is_bf16, const int* pos, const int* seq_of_token,
                             const int* slots, const int* block_table, int table_stride, const void* storage,
                             const int* pooled_table, int pooled_stride, const void* pooled, int T, int nq, int nkv,
                             int dk, int dv, int page, int size, int pool, float scale, int sink, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || nq % nkv || dk <= 0 || dv <= 0 || dk > 64 * MAX_EPL || dv > 64 * MAX_EPL || page <= 0 ||
        size < 0 || pool < 0 || nq > 65535 || (pool > 0 && size > 0 && (!pooled_table || !pooled)))
        return BR_BAD_ARG;
    dim3 grid(T, nq);
    const size_t lds = (size_t)(dk + 64) * sizeof(float);
    if (is_bf16)
        pwa_attend_kernel<bf16><<<grid, 64, lds, s>>>((const bf16*)q, (bf16*)out, pos, seq_of_token, slots, block_table,
                                                      table_stride, (const bf16*)storage, pooled_table, pooled_stride,
                                                      (const bf16*)pooled, nq, nkv, dk, dv, page, size, pool, scale, sink);
    else
        pwa_attend_kernel<float><<<grid, 64, lds, s>>>((const float*)q, (float*)out, pos, seq_of_token, slots, block_table,
                                                       table_stride, (const float*)storage, pooled_table, pooled_stride,
                                                       (const float*)pooled, nq, nkv, dk, dv, page, size, pool, scale, sink);
    return br_check_launch();
}
