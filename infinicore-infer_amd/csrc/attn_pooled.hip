// Attention over a window of tokens plus one mean key and value for every block of tokens that lies wholly before
// the window, with weights sigmoid(score + bias[head]) that are NOT normalised over the keys:
//   query at position i sees token j when 0 <= i - j < window, and block b (positions b*P .. b*P + P - 1) when
//   b*P + P - 1 <= i - window;   out_i = sum_seen sigmoid(scale * q_i . k + bias[h]) * v.
// window 0: every earlier token and no block.  P 0: no blocks.
//
//   * rotation of adjacent pairs (2i, 2i+1) of the first rot_dims entries of every query and key head by the angle
//     position * f_i, fused with the write of keys and values into the paged cache,
//   * the means of the blocks that a step completes, read back from the token cache and written to a paged
//     cache of their own (one row per block),
//   * the attention itself: a general kernel (one wave per token and head, any sizes, float32 or bfloat16), a
//     split-key kernel for single tokens and a matrix-core kernel for prompt portions (bfloat16).
// Angles, scores, weights and sums are float32.
//
// Cache layout of one layer: K plane [pages, kv_heads, page_size, key_dim], V plane [.., value_dim]; the block
// means lie in planes of the same layout with a block table of their own (row b of a request is its block b).
#include "common.h"

constexpr int kPoolMaxDim = 512;

// cos and sin of position * f, f given as the float32 rounding of its float64 value and what the rounding left: the
// float32 product plus a small rest (the product's own rounding error from an fma, and position * the second
// part), to second order in the rest.
__device__ __forceinline__ void pair_angle(float p, float f_hi, float f_lo, float& cs, float& sn) {
    const float ang = p * f_hi;
    const float rest = fmaf(p, f_hi, -ang) + p * f_lo;
    const float s0 = sinf(ang), c0 = cosf(ang), half = 0.5f * rest * rest;
    sn = (s0 - half * s0) + rest * c0;
    cs = (c0 - half * c0) - rest * s0;
}

__device__ __forceinline__ long long cache_row(const int* table, int item, int page_size, int nkvh, int kvh) {
    return ((long long)table[item / page_size] * nkvh + kvh) * page_size + item % page_size;
}

// ---------------------------------------------------------------------------------------------
// rows[t] = [q (nh * dk) | k (nkvh * dk) | v (nkvh * dv) | ..]: rotated q -> q_out[t], rotated k and v -> cache at slots[t].
// grid (T, nh + nkvh), one wave a head.  freq: float32 [2, rot_dims / 2].
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
rope_pairs_store_kernel(const T* __restrict__ rows, int row_stride, const int* __restrict__ positions,
                        const float* __restrict__ freq, int rot_dims, T* __restrict__ q_out, T* __restrict__ kcache,
                        T* __restrict__ vcache, const int* __restrict__ slots, int nh, int nkvh, int dk, int dv, int page_size) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const float p = (float)positions[t];
    const bool is_q = hh < nh;
    const int g = is_q ? hh : hh - nh;
    const T* src = rows + (size_t)t * row_stride + (is_q ? (size_t)g * dk : (size_t)nh * dk + (size_t)g * dk);
    T* dst;
    long long crow = 0;
    if (is_q) {
        dst = q_out + ((size_t)t * nh + g) * dk;
    } else {
        const int slot = slots[t];
        crow = ((long long)(slot / page_size) * nkvh + g) * page_size + slot % page_size;
        dst = kcache + crow * dk;
    }
    const int half = rot_dims / 2;
    for (int d = lane; d < dk; d += 64) {
        float o;
        if (d < rot_dims) {
            const int i = d >> 1;
            float cs, sn;
            pair_angle(p, freq[i], freq[half + i], cs, sn);
            const float u = to_f32(src[2 * i]), v = to_f32(src[2 * i + 1]);
            o = (d & 1) ? (v * cs + u * sn) : (u * cs - v * sn);
        } else {
            o = to_f32(src[d]);
        }
        dst[d] = from_f32<T>(o);
    }
    if (!is_q) {
        const T* vs = rows + (size_t)t * row_stride + (size_t)nh * dk + (size_t)nkvh * dk + (size_t)g * dv;
        T* vd = vcache + crow * dv;
        for (int d = lane; d < dv; d += 64) vd[d] = vs[d];
    }
}

IC_EXPORT int ic_rope_pairs_store(const void* rows, int row_stride, int dtype, const int* positions, const float* freq,
                                  int rot_dims, void* q_out, void* kcache, void* vcache, const int* slots, int T, int nh,
                                  int nkvh, int dk, int dv, int page_size, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh < 0 || dk <= 0 || dv <= 0 || rot_dims < 0 || rot_dims > dk || (rot_dims & 1) || page_size <= 0 ||
        (rot_dims > 0 && freq == nullptr))
        return IC_ERR_ARG;
    const int kv = slots ? nkvh : 0;
    if (nh + kv > 65535) return IC_ERR_ARG;
    dim3 grid((unsigned)T, (unsigned)(nh + kv)), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(rope_pairs_store_kernel<float>, grid, block, 0, stream, (const float*)rows, row_stride, positions,
                           freq, rot_dims, (float*)q_out, (float*)kcache, (float*)vcache, slots, nh, nkvh, dk, dv, page_size);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(rope_pairs_store_kernel<bf16>, grid, block, 0, stream, (const bf16*)rows, row_stride, positions,
                           freq, rot_dims, (bf16*)q_out, (bf16*)kcache, (bf16*)vcache, slots, nh, nkvh, dk, dv, page_size);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The mean key and value of every block that this step completes: a token at position p with (p + 1) % P == 0
// ends block b = (p + 1) / P - 1; its P keys and values are read back from the token cache (as the cache holds
// them) and their means go to row b of the request's block-mean cache.  grid (T, nkvh).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
pool_blocks_kernel(const T* __restrict__ kcache, const T* __restrict__ vcache, T* __restrict__ kpool, T* __restrict__ vpool,
                   const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ pool_tables, int pt_stride,
                   const int* __restrict__ token_req, const int* __restrict__ positions, int P, int nkvh, int dk, int dv,
                   int page_size) {
    const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
    const int p = positions[t];
    if ((p + 1) % P != 0) return;
    const int b = (p + 1) / P - 1;
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const int* pt = pool_tables + (size_t)token_req[t] * pt_stride;
    const long long orow = cache_row(pt, b, page_size, nkvh, g);
    const float inv = 1.0f / (float)P;
    for (int d = lane; d < dk + dv; d += 64) {
        const bool key = d < dk;
        const int c = key ? d : d - dk, w = key ? dk : dv;
        const T* plane = key ? kcache : vcache;
        float s = 0.f;
        for (int j = 0; j < P; ++j) s += to_f32(plane[cache_row(bt, b * P + j, page_size, nkvh, g) * w + c]);
        (key ? kpool : vpool)[orow * w + c] = from_f32<T>(s * inv);
    }
}

IC_EXPORT int ic_pool_blocks(const void* kcache, const void* vcache, void* kpool, void* vpool, int dtype,
                             const int* block_tables, int bt_stride, const int* pool_tables, int pt_stride,
                             const int* token_req, const int* positions, int T, int P, int nkvh, int dk, int dv,
                             int page_size, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (P <= 0 || nkvh <= 0 || nkvh > 65535 || dk <= 0 || dv <= 0 || page_size <= 0) return IC_ERR_ARG;
    dim3 grid((unsigned)T, (unsigned)nkvh), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(pool_blocks_kernel<float>, grid, block, 0, stream, (const float*)kcache, (const float*)vcache,
                           (float*)kpool, (float*)vpool, block_tables, bt_stride, pool_tables, pt_stride, token_req, positions,
                           P, nkvh, dk, dv, page_size);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(pool_blocks_kernel<bf16>, grid, block, 0, stream, (const bf16*)kcache, (const bf16*)vcache,
                           (bf16*)kpool, (bf16*)vpool, block_tables, bt_stride, pool_tables, pt_stride, token_req, positions,
                           P, nkvh, dk, dv, page_size);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// What a query at position pos sees: blocks 0 .. nb - 1, then tokens lo .. pos.
struct PooledSpan { int nb, lo, total; };
__device__ __forceinline__ PooledSpan pooled_span(int pos, int window, int P) {
    PooledSpan s;
    s.lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    s.nb = (window > 0 && P > 0) ? s.lo / P : 0;          // block b is seen when (b + 1) * P <= pos - window + 1
    s.total = s.nb + (pos - s.lo + 1);
    return s;
}

__device__ __forceinline__ float sigmoid_acc(float z) { return 1.0f / (1.0f + expf(-z)); }

// ---------------------------------------------------------------------------------------------
// The general kernel: one wave per (token, head), the seen items 64 at a time, a lane an item for the scores and
// a lane a column for the sums.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
attn_pooled_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                           const T* __restrict__ kcache, const T* __restrict__ vcache, const T* __restrict__ kpool,
                           const T* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride,
                           const int* __restrict__ pool_tables, int pt_stride, const int* __restrict__ token_req,
                           const int* __restrict__ positions, const float* __restrict__ bias, int nh, int nkvh, int dk, int dv,
                           int page_size, float scale, int window, int P) {
    __shared__ float qs[kPoolMaxDim];
    __shared__ float ps[64];
    __shared__ const T* vrow[64];

    const int h = blockIdx.x % nh, t = blockIdx.x / nh, lane = threadIdx.x;
    const int kvh = h / (nh / nkvh);
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const int* pt = pool_tables ? pool_tables + (size_t)token_req[t] * pt_stride : nullptr;
    const T* qp = q + (size_t)t * q_stride + (size_t)h * dk;
    for (int d = lane; d < dk; d += 64) qs[d] = to_f32(qp[d]);
    __syncthreads();
    const PooledSpan span = pooled_span(pos, window, pt ? P : 0);
    const float hb = bias ? bias[h] : 0.f;
    const int nd = (dv + 63) / 64;
    float acc[kPoolMaxDim / 64];
#pragma unroll
    for (int i = 0; i < kPoolMaxDim / 64; ++i) acc[i] = 0.f;

    for (int ib = 0; ib < span.total; ib += 64) {
        const int idx = ib + lane;
        float p = 0.f;
        const T* vp = vcache;
        if (idx < span.total) {
            const bool pooled = idx < span.nb;
            const long long rowi = pooled ? cache_row(pt, idx, page_size, nkvh, kvh)
                                          : cache_row(bt, span.lo + (idx - span.nb), page_size, nkvh, kvh);
            const T* kp = (pooled ? kpool : kcache) + rowi * dk;
            vp = (pooled ? vpool : vcache) + rowi * dv;
            float dot = 0.f;
            for (int d = 0; d < dk; ++d) dot += qs[d] * to_f32(kp[d]);
            p = sigmoid_acc(dot * scale + hb);
        }
        __syncthreads();
        ps[lane] = p;
        vrow[lane] = vp;
        __syncthreads();
        const int nk = (span.total - ib < 64) ? span.total - ib : 64;
#pragma unroll
        for (int i = 0; i < kPoolMaxDim / 64; ++i) {
            if (i < nd) {
                const int d = lane + 64 * i;
                if (d < dv) {
                    float a = acc[i];
                    for (int kk = 0; kk < nk; ++kk) a += ps[kk] * to_f32(vrow[kk][d]);
                    acc[i] = a;
                }
            }
        }
    }
    T* op = out + (size_t)t * out_stride + (size_t)h * dv;
#pragma unroll
    for (int i = 0; i < kPoolMaxDim / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < dv) op[d] = from_f32<T>(acc[i]);
    }
}

IC_EXPORT int ic_attn_pooled_generic(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache,
                                     const void* vcache, const void* kpool, const void* vpool, const int* block_tables,
                                     int bt_stride, const int* pool_tables, int pt_stride, const int* token_req,
                                     const int* positions, const float* bias, int T, int nh, int nkvh, int dk, int dv,
                                     int page_size, float scale, int window, int P, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dk <= 0 || dv <= 0 || dk > kPoolMaxDim || dv > kPoolMaxDim || page_size <= 0 ||
        window < 0 || P < 0)
        return IC_ERR_ARG;
    if (P > 0 && window > 0 && (pool_tables == nullptr || kpool == nullptr || vpool == nullptr)) return IC_ERR_ARG;
    if ((long long)T * nh > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(T * nh)), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(attn_pooled_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride, (float*)out,
                           out_stride, (const float*)kcache, (const float*)vcache, (const float*)kpool, (const float*)vpool,
                           block_tables, bt_stride, pool_tables, pt_stride, token_req, positions, bias, nh, nkvh, dk, dv,
                           page_size, scale, window, P);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(attn_pooled_generic_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out,
                           out_stride, (const bf16*)kcache, (const bf16*)vcache, (const bf16*)kpool, (const bf16*)vpool,
                           block_tables, bt_stride, pool_tables, pt_stride, token_req, positions, bias, nh, nkvh, dk, dv,
                           page_size, scale, window, P);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
