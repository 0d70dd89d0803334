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
// The mean key and value of every block that this step completes.  A request's portion at positions p0 .. p0 + n - 1
// completes the blocks b = p0 / P, p0 / P + 1, .. with (b + 1) P <= p0 + n; their P keys and values are read back from
// the token cache (as the cache holds them) and their means go to row b of the request's block-mean cache.
// grid (most blocks a request can complete, kv heads, requests); req_rows: first token row of every request, then T.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
pool_blocks_kernel(const T* __restrict__ kcache, const T* __restrict__ vcache, T* __restrict__ kpool, T* __restrict__ vpool,
                   const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ pool_tables, int pt_stride,
                   const int* __restrict__ req_rows, const int* __restrict__ positions, int P, int nkvh, int dk, int dv,
                   int page_size) {
    // a thread a column; the block's rows eight at a time, so that eight loads are in flight
    const int r = blockIdx.z, g = blockIdx.y;
    const int row0 = req_rows[r], n = req_rows[r + 1] - row0;
    if (n <= 0) return;
    const int p0 = positions[row0];
    const int b = p0 / P + (int)blockIdx.x;
    if ((long long)(b + 1) * P > (long long)p0 + n) return;
    const int* bt = block_tables + (size_t)r * bt_stride;
    const int* pt = pool_tables + (size_t)r * pt_stride;
    const long long orow = cache_row(pt, b, page_size, nkvh, g);
    for (int d = threadIdx.x; d < dk + dv; d += 256) {
        const bool key = d < dk;
        const int c = key ? d : d - dk, w = key ? dk : dv;
        const T* plane = key ? kcache : vcache;
        float s = 0.f;
        for (int j0 = 0; j0 < P; j0 += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = min(j0 + u, P - 1);
                v[u] = to_f32(plane[cache_row(bt, b * P + j, page_size, nkvh, g) * w + c]);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) s += (j0 + u < P) ? v[u] : 0.f;
        }
        (key ? kpool : vpool)[orow * w + c] = from_f32<T>(s / (float)P);
    }
}

IC_EXPORT int ic_pool_blocks(const void* kcache, const void* vcache, void* kpool, void* vpool, int dtype,
                             const int* block_tables, int bt_stride, const int* pool_tables, int pt_stride,
                             const int* req_rows, const int* positions, int n_requests, int most_blocks, int P, int nkvh,
                             int dk, int dv, int page_size, hipStream_t stream) {
    if (n_requests <= 0 || most_blocks <= 0) return IC_OK;
    if (P <= 0 || nkvh <= 0 || nkvh > 65535 || n_requests > 65535 || dk <= 0 || dv <= 0 || page_size <= 0) return IC_ERR_ARG;
    dim3 grid((unsigned)most_blocks, (unsigned)nkvh, (unsigned)n_requests), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(pool_blocks_kernel<float>, grid, block, 0, stream, (const float*)kcache, (const float*)vcache,
                           (float*)kpool, (float*)vpool, block_tables, bt_stride, pool_tables, pt_stride, req_rows, positions,
                           P, nkvh, dk, dv, page_size);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(pool_blocks_kernel<bf16>, grid, block, 0, stream, (const bf16*)kcache, (const bf16*)vcache,
                           (bf16*)kpool, (bf16*)vpool, block_tables, bt_stride, pool_tables, pt_stride, req_rows, positions,
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

// =============================================================================================
// Single new tokens, split over what a token sees so that few requests fill the chip.
//
// Pass 1, grid (splits, kv heads, tokens), 256 threads: the seen items of a token are numbered 0 .. total - 1 (the
// blocks, then the window's tokens); a block streams its share once and serves every query head of the kv head, four
// at a time.  DK / VEC lanes share an item (VEC = 16 bytes of elements), so a wave reads whole rows; the same lanes
// read the value row in 16-byte pieces.  The weights are not normalised, so shares simply add up: lane groups,
// waves, and (pass 2) splits.  With one split pass 1 writes the result itself.
// =============================================================================================
template <typename T> struct PoolVec;
template <> struct PoolVec<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const uint4 v = load_stream16(p);
        o[0] = __uint_as_float(v.x); o[1] = __uint_as_float(v.y); o[2] = __uint_as_float(v.z); o[3] = __uint_as_float(v.w);
    }
    __device__ static float sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
};
template <> struct PoolVec<bf16> {
    static constexpr int N = 8;
    __device__ static void load(const bf16* p, float* o) {
        const uint4 v = load_stream16(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    // the hardware's exp2 and reciprocal (each good to an ulp): for results that are rounded to bfloat16
    __device__ static float sigmoid(float z) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z)); }
};

constexpr int kPdHeads = 4;      // query heads served per walk

template <typename T, int DK, int DV>
__global__ void __launch_bounds__(256)
attn_pooled_decode_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ kcache, const T* __restrict__ vcache,
                          const T* __restrict__ kpool, const T* __restrict__ vpool, const int* __restrict__ block_tables,
                          int bt_stride, const int* __restrict__ pool_tables, int pt_stride, const int* __restrict__ tok_list,
                          const int* __restrict__ token_req, const int* __restrict__ positions, const float* __restrict__ bias,
                          float* __restrict__ parts, T* __restrict__ out, int out_stride, int nh, int nkvh, int page_size,
                          float scale, int window, int P, int n_tok, int nsplit) {
    constexpr int VEC = PoolVec<T>::N;
    constexpr int LPK = DK / VEC;                   // lanes that share an item
    constexpr int KPW = 64 / LPK;                   // items a wave takes at a time
    constexpr int VP = DV / VEC;                    // 16-byte pieces of a value row
    constexpr int NP = (VP + LPK - 1) / LPK;        // pieces a lane takes
    static_assert(LPK <= 64 && 64 % LPK == 0 && DV % VEC == 0, "rows in whole 16-byte pieces");
    __shared__ float qs[kPdHeads][DK];
    __shared__ float red[4][kPdHeads][DV];

    const int split = blockIdx.x, kvh = blockIdx.y, ti = blockIdx.z;
    const int t = tok_list ? tok_list[ti] : ti;
    const int G = nh / nkvh;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane % LPK, grp = lane / LPK;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const int* pt = pool_tables ? pool_tables + (size_t)token_req[t] * pt_stride : nullptr;
    const PooledSpan span = pooled_span(pos, window, pt ? P : 0);
    const int per = (span.total + nsplit - 1) / nsplit;
    const int i0 = split * per, i1 = min(span.total, i0 + per);

    for (int g0 = 0; g0 < G; g0 += kPdHeads) {
        const int gq = min(kPdHeads, G - g0);
        __syncthreads();
        for (int i = tid; i < gq * DK; i += 256) {
            const int g = i / DK, d = i - g * DK;
            qs[g][d] = to_f32(q[(size_t)t * q_stride + (size_t)(kvh * G + g0 + g) * DK + d]);
        }
        __syncthreads();
        float qr[kPdHeads][VEC], hb[kPdHeads], acc[kPdHeads][NP][VEC];
#pragma unroll
        for (int g = 0; g < kPdHeads; ++g) {
            hb[g] = (bias && g < gq) ? bias[kvh * G + g0 + g] : 0.f;
#pragma unroll
            for (int j = 0; j < VEC; ++j) qr[g][j] = g < gq ? qs[g][sub * VEC + j] : 0.f;
#pragma unroll
            for (int n = 0; n < NP; ++n)
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[g][n][j] = 0.f;
        }
        for (int it = i0 + wave * KPW + grp; it < i1; it += 4 * KPW) {
            const bool pooled = it < span.nb;
            const long long rowi = pooled ? cache_row(pt, it, page_size, nkvh, kvh)
                                          : cache_row(bt, span.lo + (it - span.nb), page_size, nkvh, kvh);
            float kf[VEC], vf[NP][VEC];
            PoolVec<T>::load((pooled ? kpool : kcache) + rowi * DK + sub * VEC, kf);
#pragma unroll
            for (int n = 0; n < NP; ++n) {
                const int piece = sub + n * LPK;
                if (piece < VP) PoolVec<T>::load((pooled ? vpool : vcache) + rowi * DV + piece * VEC, vf[n]);
                else
#pragma unroll
                    for (int j = 0; j < VEC; ++j) vf[n][j] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < kPdHeads; ++g) {
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < VEC; ++j) d += kf[j] * qr[g][j];
                d = group_sum<LPK>(d);
                const float p = PoolVec<T>::sigmoid(d * scale + hb[g]);
#pragma unroll
                for (int n = 0; n < NP; ++n)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[g][n][j] += p * vf[n][j];
            }
        }
        // lanes with the same place in their group hold shares of the same columns
#pragma unroll
        for (int g = 0; g < kPdHeads; ++g)
#pragma unroll
            for (int n = 0; n < NP; ++n)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float v = acc[g][n][j];
#pragma unroll
                    for (int o = LPK; o < 64; o <<= 1) v += __shfl_xor(v, o, kWave);
                    acc[g][n][j] = v;
                }
        if (grp == 0) {
#pragma unroll
            for (int g = 0; g < kPdHeads; ++g)
#pragma unroll
                for (int n = 0; n < NP; ++n) {
                    const int piece = sub + n * LPK;
                    if (piece < VP)
#pragma unroll
                        for (int j = 0; j < VEC; ++j) red[wave][g][piece * VEC + j] = acc[g][n][j];
                }
        }
        __syncthreads();
        for (int i = tid; i < gq * DV; i += 256) {
            const int g = i / DV, d = i - g * DV;
            const float v = red[0][g][d] + red[1][g][d] + red[2][g][d] + red[3][g][d];
            const int h = kvh * G + g0 + g;
            if (nsplit == 1) out[(size_t)t * out_stride + (size_t)h * DV + d] = from_f32<T>(v);
            else parts[(((size_t)split * n_tok + ti) * nh + h) * DV + d] = v;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
attn_pooled_merge_kernel(const float* __restrict__ parts, const int* __restrict__ tok_list, T* __restrict__ out, int out_stride,
                         int n_tok, int width, int nsplit) {
    const int ti = blockIdx.x, t = tok_list ? tok_list[ti] : ti;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x) {
        float v = 0.f;
        for (int s = 0; s < nsplit; ++s) v += parts[((size_t)s * n_tok + ti) * width + i];
        out[(size_t)t * out_stride + i] = from_f32<T>(v);
    }
}

IC_EXPORT int ic_attn_pooled_decode_supported(int dtype, int dk, int dv) {
    return (dtype == IC_F32 || dtype == IC_BF16) && (dk == 64 || dk == 128) && (dv == 64 || dv == 128);
}

IC_EXPORT int ic_attn_pooled_decode(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache,
                                    const void* vcache, const void* kpool, const void* vpool, const int* block_tables,
                                    int bt_stride, const int* pool_tables, int pt_stride, const int* tok_list,
                                    const int* token_req, const int* positions, const float* bias, float* parts, int n_tok,
                                    int nh, int nkvh, int dk, int dv, int page_size, float scale, int window, int P, int nsplit,
                                    hipStream_t stream) {
    if (n_tok <= 0) return IC_OK;
    if (!ic_attn_pooled_decode_supported(dtype, dk, dv)) return IC_ERR_UNSUPPORTED;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || window < 0 || P < 0 || nsplit < 1 || nsplit > 64 || nkvh > 65535 ||
        n_tok > 65535 || (nsplit > 1 && parts == nullptr))
        return IC_ERR_ARG;
    if (P > 0 && window > 0 && (pool_tables == nullptr || kpool == nullptr || vpool == nullptr)) return IC_ERR_ARG;
    dim3 grid((unsigned)nsplit, (unsigned)nkvh, (unsigned)n_tok), block(256);
#define IC_PD(TT, K, V)                                                                                                 \
    hipLaunchKernelGGL((attn_pooled_decode_kernel<TT, K, V>), grid, block, 0, stream, (const TT*)q, q_stride,             \
                       (const TT*)kcache, (const TT*)vcache, (const TT*)kpool, (const TT*)vpool, block_tables, bt_stride, \
                       pool_tables, pt_stride, tok_list, token_req, positions, bias, parts, (TT*)out, out_stride, nh, nkvh, \
                       page_size, scale, window, P, n_tok, nsplit)
#define IC_PD_T(TT)                                                                                                     \
    do {                                                                                                                \
        if (dk == 64 && dv == 64) IC_PD(TT, 64, 64);                                                                    \
        else if (dk == 64) IC_PD(TT, 64, 128);                                                                          \
        else if (dv == 64) IC_PD(TT, 128, 64);                                                                          \
        else IC_PD(TT, 128, 128);                                                                                       \
    } while (0)
    if (dtype == IC_F32) IC_PD_T(float); else IC_PD_T(bf16);
#undef IC_PD_T
#undef IC_PD
    int st = ic_launch_status();
    if (st != IC_OK || nsplit == 1) return st;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(attn_pooled_merge_kernel<float>, dim3(n_tok, (nh * dv + 255) / 256), dim3(256), 0, stream, parts, tok_list, (float*)out,
                           out_stride, n_tok, nh * dv, nsplit);
    else
        hipLaunchKernelGGL(attn_pooled_merge_kernel<bf16>, dim3(n_tok, (nh * dv + 255) / 256), dim3(256), 0, stream, parts, tok_list, (bf16*)out,
                           out_stride, n_tok, nh * dv, nsplit);
    return ic_launch_status();
}

// =============================================================================================
// Prompt portions on the matrix cores (bfloat16; key and value sizes 32, 64, 128).
//
// Grid (query tiles * heads), tile-major, 256 threads.  A tile is up to 128 consecutive tokens of one request (int4:
// request row, first token row, rows, first position); wave w owns rows 32w..32w+31.  What the tile may see is walked 64
// items at a time: first the blocks' means that its last row sees, then the tokens from the first row's window to the
// last row.  A step's keys and values pass through LDS as padded rows.  S^T = K Q^T with v_mfma_f32_32x32x16_bf16: a lane
// holds 32 items of ONE query, so the mask and the sigmoid need no cross-lane step and the weights are already the B
// operand of O^T = V^T P^T, whose A operand comes out of LDS through the transposing read.  Operand layout (lane l,
// h = l/32): A[i = l%32][k = 8h..8h+7], B[k = 8h..8h+7][j = l%32], D[i = 8(r/4) + 4h + r%4][j = l%32].
// An item outside the run a step walks is replaced by the last one inside when it is loaded, and masked.
// =============================================================================================
typedef __bf16 pl_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pl_v16f __attribute__((ext_vector_type(16)));
typedef float pl_v8f __attribute__((ext_vector_type(8)));
typedef short pl_v4s __attribute__((ext_vector_type(4)));
typedef unsigned pl_v4u __attribute__((ext_vector_type(4)));

constexpr int kPlRows = 128;
constexpr int kPlItems = 64;

template <int DK, int DV>
__global__ void __launch_bounds__(256, 2)
attn_pooled_prefill_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                           const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                           const uint16_t* __restrict__ kpool, const uint16_t* __restrict__ vpool,
                           const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ pool_tables, int pt_stride,
                           const int4* __restrict__ tiles, const float* __restrict__ bias, int nh, int nkvh, int page_size,
                           float scale, int window, int P) {
    constexpr int NC = DK / 16, ND = DV / 32, PK = DK + 8, PV = DV + 8, KCH = DK / 8, VCH = DV / 8;
    constexpr int NLK = kPlItems * KCH / 256, NLV = kPlItems * VCH / 256;
    static_assert(DK % 32 == 0 && DV % 32 == 0, "a step's rows split evenly over the block");
    __shared__ __attribute__((aligned(16))) uint16_t Ks[kPlItems * PK];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[kPlItems * PV];

    const int slot = (int)blockIdx.x;
    const int h = slot % nh;
    const int4 tile = tiles[slot / nh];
    const int req = tile.x, row0 = tile.y, n_rows = tile.z, pos0 = tile.w;
    const int kvh = h / (nh / nkvh);
    const int* bt = block_tables + (size_t)req * bt_stride;
    const int* pt = pool_tables ? pool_tables + (size_t)req * pt_stride : nullptr;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const bool wave_ok = 32 * wave < n_rows;
    const int my_row = min(32 * wave + lq, n_rows - 1);
    const int qpos = pos0 + my_row;
    const PooledSpan mine = pooled_span(qpos, window, pt ? P : 0);
    const int last_pos = pos0 + n_rows - 1;
    const int lo_min = pooled_span(pos0, window, 0).lo;
    const int nb_max = pooled_span(last_pos, window, pt ? P : 0).nb;
    const int block_steps = (nb_max + kPlItems - 1) / kPlItems;
    const int n_steps = block_steps + (last_pos - lo_min + kPlItems) / kPlItems;
    const float hb = bias ? bias[h] : 0.f;

    pl_bf16x8 qf[NC];
    {
        const uint16_t* qp = q + (size_t)(row0 + my_row) * q_stride + (size_t)h * DK + 8 * half;
#pragma unroll
        for (int c = 0; c < NC; ++c) qf[c] = *reinterpret_cast<const pl_bf16x8*>(qp + 16 * c);
    }
    pl_v16f oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    const int vrow = 4 * half + ((lane & 15) >> 2);
    const int vcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    for (int s = 0; s < n_steps; ++s) {
        const bool pooled = s < block_steps;
        const int base = pooled ? kPlItems * s : lo_min + kPlItems * (s - block_steps);
        const int hi = pooled ? nb_max - 1 : last_pos;
        const uint16_t* kplane = pooled ? kpool : kcache;
        const uint16_t* vplane = pooled ? vpool : vcache;
        const int* table = pooled ? pt : bt;
        __syncthreads();                                   // the step before has been read
#pragma unroll
        for (int i = 0; i < NLK; ++i) {
            const int idx = tid + i * 256, kk = idx / KCH, c = idx - kk * KCH;
            const long long rowi = cache_row(table, min(base + kk, hi), page_size, nkvh, kvh);
            *reinterpret_cast<pl_v4u*>(Ks + kk * PK + c * 8) = *reinterpret_cast<const pl_v4u*>(kplane + rowi * DK + c * 8);
        }
#pragma unroll
        for (int i = 0; i < NLV; ++i) {
            const int idx = tid + i * 256, kk = idx / VCH, c = idx - kk * VCH;
            const long long rowi = cache_row(table, min(base + kk, hi), page_size, nkvh, kvh);
            *reinterpret_cast<pl_v4u*>(Vs + kk * PV + c * 8) = *reinterpret_cast<const pl_v4u*>(vplane + rowi * DV + c * 8);
        }
        __syncthreads();
        if (!wave_ok) continue;
        pl_v16f sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[tt][r] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const pl_bf16x8 a = *reinterpret_cast<const pl_bf16x8*>(Ks + (32 * tt + lq) * PK + 16 * c + 8 * half);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[c], sacc[tt], 0, 0, 0);
            }
        }
        // weights: sigmoid(scale s + bias) where this lane's query sees the item, else nothing
        const int lim_lo = pooled ? 0 : mine.lo, lim_hi = pooled ? mine.nb - 1 : qpos;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int item = base + 32 * tt + 8 * (r >> 2) + 4 * half + (r & 3);
                const float z = fmaf(sacc[tt][r], scale, hb);
                const float p = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
                sacc[tt][r] = (item >= lim_lo && item <= lim_hi) ? p : 0.f;
            }
#pragma unroll
        for (int kc = 0; kc < 4; ++kc) {
            const int tt = kc >> 1, r0 = 8 * (kc & 1);
            pl_v8f pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = sacc[tt][r0 + e];
            const pl_bf16x8 b = __builtin_convertvector(pf, pl_bf16x8);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const uint16_t* vp = Vs + (16 * kc + vrow) * PV + 32 * dt + vcol;
                const pl_v4s lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_v4s __attribute__((address_space(3)))*)vp);
                const pl_v4s hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_v4s __attribute__((address_space(3)))*)(vp + 8 * PV));
                const pl_bf16x8 a = __builtin_bit_cast(pl_bf16x8, __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, oacc[dt], 0, 0, 0);
            }
        }
    }
    if (32 * wave + lq < n_rows) {
        uint16_t* op = out + (size_t)(row0 + my_row) * out_stride + (size_t)h * DV;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                uint2 v;
                v.x = (uint32_t)f32_to_bf16_bits(oacc[dt][4 * r4]) | ((uint32_t)f32_to_bf16_bits(oacc[dt][4 * r4 + 1]) << 16);
                v.y = (uint32_t)f32_to_bf16_bits(oacc[dt][4 * r4 + 2]) | ((uint32_t)f32_to_bf16_bits(oacc[dt][4 * r4 + 3]) << 16);
                *reinterpret_cast<uint2*>(op + 32 * dt + 8 * r4 + 4 * half) = v;
            }
    }
}

IC_EXPORT int ic_attn_pooled_prefill_supported(int dtype, int dk, int dv) {
    auto ok = [](int d) { return d == 32 || d == 64 || d == 128; };
    return dtype == IC_BF16 && ok(dk) && ok(dv);
}

IC_EXPORT int ic_attn_pooled_prefill(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache,
                                     const void* vcache, const void* kpool, const void* vpool, const int* block_tables,
                                     int bt_stride, const int* pool_tables, int pt_stride, const int* tiles, int n_tiles,
                                     const float* bias, int nh, int nkvh, int dk, int dv, int page_size, float scale,
                                     int window, int P, hipStream_t stream) {
    if (n_tiles <= 0) return IC_OK;
    if (!ic_attn_pooled_prefill_supported(dtype, dk, dv)) return IC_ERR_UNSUPPORTED;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || window < 0 || P < 0 || (q_stride % 8) || (out_stride % 4) ||
        ((uintptr_t)q % 16) || ((uintptr_t)out % 8) || (long long)n_tiles * nh > 0x7fffffffLL)
        return IC_ERR_ARG;
    if (P > 0 && window > 0 && (pool_tables == nullptr || kpool == nullptr || vpool == nullptr)) return IC_ERR_ARG;
    dim3 grid((unsigned)(n_tiles * nh)), block(256);
#define IC_PP(K, V)                                                                                                     \
    hipLaunchKernelGGL((attn_pooled_prefill_kernel<K, V>), grid, block, 0, stream, (const uint16_t*)q, q_stride,          \
                       (uint16_t*)out, out_stride, (const uint16_t*)kcache, (const uint16_t*)vcache, (const uint16_t*)kpool, \
                       (const uint16_t*)vpool, block_tables, bt_stride, pool_tables, pt_stride, (const int4*)tiles, bias, nh, \
                       nkvh, page_size, scale, window, P)
#define IC_PP_V(K)                                                                                                      \
    do {                                                                                                                \
        if (dv == 32) IC_PP(K, 32); else if (dv == 64) IC_PP(K, 64); else IC_PP(K, 128);                                 \
    } while (0)
    if (dk == 32) IC_PP_V(32); else if (dk == 64) IC_PP_V(64); else IC_PP_V(128);
#undef IC_PP_V
#undef IC_PP
    return ic_launch_status();
}
