// Row kernels of decoders that normalise a sublayer's OUTPUT before it joins the residual stream
// (x += norm(f(x))) and whose sublayers read the stream itself:
//   * embedding gather with a sinusoidal position vector added,
//   * x += rmsnorm(y + bias) * w, with the stream's copy in the compute dtype written along,
//   * bias, query/key norm (per head or over the whole row), value mixing with an earlier layer's
//     values and the write of keys and values into the paged cache, in one pass over a token's
//     projected row,
//   * element-wise activations of a dense feed-forward.
// The residual stream is float32; every norm, sum of squares, angle and mix is float32.
//
// Cache layout of one layer: K plane [num_pages, n_kv_heads, page_size, key_dim], V plane
// [num_pages, n_kv_heads, page_size, value_dim].
#include "common.h"

// 16 bytes of a row as float32 values.
template <typename T> struct RowPack;
template <> struct RowPack<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
    __device__ static void store(float* p, const float* o) { *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]); }
};
template <> struct RowPack<bf16> {
    static constexpr int N = 8;
    __device__ static void load(const bf16* p, float* o) {
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        const v4u v = *reinterpret_cast<const v4u*>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(v[i] << 16); o[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u); }
    }
    __device__ static void store(bf16* p, const float* o) {
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        v4u v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (uint32_t)f32_to_bf16_bits(o[2 * i]) | ((uint32_t)f32_to_bf16_bits(o[2 * i + 1]) << 16);
        *reinterpret_cast<v4u*>(p) = v;
    }
};
// N (4 or 8) float32 values from a 16-byte aligned address, 16 bytes a load.
template <int N> __device__ __forceinline__ void load_floats(const float* p, float* o) {
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
        const float4 v = *reinterpret_cast<const float4*>(p + 4 * i);
        o[4 * i] = v.x; o[4 * i + 1] = v.y; o[4 * i + 2] = v.z; o[4 * i + 3] = v.w;
    }
}

// ---------------------------------------------------------------------------------------------
// x[t, 2i] = table[tok, 2i] * scale + sin(p f_i), x[t, 2i+1] = table[tok, 2i+1] * scale + cos(p f_i);
// f_i comes as two float32 tables of n = ceil(d/2) entries made by the host from the float64 value: freq[i] its
// rounding and freq[n + i] what the rounding left.  The angle is the float32 product p * freq[i] plus a small
// rest (the product's own rounding error, from an fma, and p * freq[n + i]); sine and cosine of the sum follow
// from those of the product to second order in the rest, so that far positions keep float32 accuracy.
// copy (nullable): x rounded to the compute dtype.
// ---------------------------------------------------------------------------------------------
template <typename TW, typename TC>
__global__ void embed_sinusoid_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                      const TW* __restrict__ table, const float* __restrict__ freq,
                                      float* __restrict__ x, TC* __restrict__ copy, int d, float scale) {
    const int t = blockIdx.x;
    const TW* row = table + (size_t)tokens[t] * d;
    const float p = (float)positions[t];
    float* o = x + (size_t)t * d;
    const int n = (d + 1) / 2;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float f = freq[i];
        const float ang = p * f;
        const float rest = fmaf(p, f, -ang) + p * freq[n + i];
        const float sn = sinf(ang), cs = cosf(ang), half = 0.5f * rest * rest;
        const float a = to_f32(row[2 * i]) * scale + ((sn - half * sn) + rest * cs);
        o[2 * i] = a;
        if (copy) copy[(size_t)t * d + 2 * i] = from_f32<TC>(a);
        if (2 * i + 1 < d) {                              // an odd width ends on a sine
            const float b = to_f32(row[2 * i + 1]) * scale + ((cs - half * cs) - rest * sn);
            o[2 * i + 1] = b;
            if (copy) copy[(size_t)t * d + 2 * i + 1] = from_f32<TC>(b);
        }
    }
}

IC_EXPORT int ic_embed_sinusoid(const int* tokens, const int* positions, const void* table, int table_dtype,
                                const float* freq, float* x, void* copy, int copy_dtype, int T, int d, float scale,
                                hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    dim3 grid(T), block(256);
    if (table_dtype == IC_F32 && (copy == nullptr || copy_dtype == IC_F32))
        hipLaunchKernelGGL((embed_sinusoid_kernel<float, float>), grid, block, 0, stream, tokens, positions,
                           (const float*)table, freq, x, (float*)copy, d, scale);
    else if (table_dtype == IC_BF16 && (copy == nullptr || copy_dtype == IC_BF16))
        hipLaunchKernelGGL((embed_sinusoid_kernel<bf16, bf16>), grid, block, 0, stream, tokens, positions,
                           (const bf16*)table, freq, x, (bf16*)copy, d, scale);
    else if (table_dtype == IC_F32 && copy_dtype == IC_BF16)
        hipLaunchKernelGGL((embed_sinusoid_kernel<float, bf16>), grid, block, 0, stream, tokens, positions,
                           (const float*)table, freq, x, (bf16*)copy, d, scale);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// x[t] += (y[t] + bias) * rsqrt(mean((y[t] + bias)^2) + eps) * w;  copy[t] = x[t] in the compute dtype.
// One block per row; the row is read twice (the second time from cache).
// ---------------------------------------------------------------------------------------------
template <typename TY, typename TC>
__global__ void __launch_bounds__(256)
norm_into_stream_kernel(const TY* __restrict__ y, const float* __restrict__ bias, const float* __restrict__ w,
                        float* __restrict__ x, TC* __restrict__ copy, int d, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const TY* yr = y + (size_t)t * d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = to_f32(yr[i]) + (bias ? bias[i] : 0.f);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float* xr = x + (size_t)t * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = to_f32(yr[i]) + (bias ? bias[i] : 0.f);
        const float s = xr[i] + v * r * w[i];
        xr[i] = s;
        if (copy) copy[(size_t)t * d + i] = from_f32<TC>(s);
    }
}

IC_EXPORT int ic_norm_into_stream(const void* y, int y_dtype, const float* bias, const float* w, float* x, void* copy,
                                  int copy_dtype, int T, int d, float eps, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    dim3 grid(T), block(256);
    if (y_dtype == IC_F32 && (copy == nullptr || copy_dtype == IC_F32))
        hipLaunchKernelGGL((norm_into_stream_kernel<float, float>), grid, block, 0, stream, (const float*)y, bias, w, x,
                           (float*)copy, d, eps);
    else if (y_dtype == IC_BF16 && (copy == nullptr || copy_dtype == IC_BF16))
        hipLaunchKernelGGL((norm_into_stream_kernel<bf16, bf16>), grid, block, 0, stream, (const bf16*)y, bias, w, x,
                           (bf16*)copy, d, eps);
    else if (y_dtype == IC_F32 && copy_dtype == IC_BF16)
        hipLaunchKernelGGL((norm_into_stream_kernel<float, bf16>), grid, block, 0, stream, (const float*)y, bias, w, x,
                           (bf16*)copy, d, eps);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// One token's projected row [q (nh * dk) | k (nkvh * dk) | v (nkvh * dv) | ...] of row_stride elements:
//   q <- norm(q + bq) -> q_out[t] (compute dtype, row stride nh * dk)
//   k <- norm(k + bk) -> K plane at slots[t]
//   v <- v + bv; mix_mode 1: v_keep[t] = v (float32, for later layers of this step);
//                mix_mode 2: v = (1 - lambda) v + lambda v_keep[t]        -> V plane at slots[t]
// norm_mode 0: none; 1: every head's dk entries to unit root mean square, times w[dk] (shared by the heads; qw and kw both
// null: no weight);
// 2: the whole of q (or k) to unit root mean square, times w[nh * dk] (or w[nkvh * dk]).
// One wave per (token, head of q, k or v); head sizes up to 512.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_store_kernel(const T* __restrict__ rows, int row_stride, const float* __restrict__ bias,
                     const float* __restrict__ qw, const float* __restrict__ kw, int norm_mode, float eps,
                     int mix_mode, const float* __restrict__ lambda, float* __restrict__ v_keep,
                     T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache,
                     const int* __restrict__ slots, int nh, int nkvh, int dk, int dv, int page_size) {
    // Grid (tokens, ceil(heads / 4)): one wave per head of q, k or v; a lane holds up to 8 of the head's entries.
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (head >= nh + 2 * nkvh) return;
    const int nq = nh * dk, nk = nkvh * dk, nv = nkvh * dv;
    const T* src = rows + (size_t)t * row_stride;
    const int slot = slots ? slots[t] : -1;
    const int pg = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - pg * page_size : 0;
    float val[8];
    if (head < nh + nkvh) {                               // a head of q or k
        const bool is_q = head < nh;
        const int base = head * dk;                       // k follows q in the row
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int e = lane + 64 * j;
            val[j] = e < dk ? to_f32(src[base + e]) + (bias ? bias[base + e] : 0.f) : 0.f;
        }
        const float* w = is_q ? qw : kw;
        if (norm_mode == 1) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += val[j] * val[j];
            const float r = 1.0f / sqrtf(wave_sum(ss) / (float)dk + eps);
#pragma unroll
            for (int j = 0; j < 8; ++j) { const int e = lane + 64 * j; if (e < dk) val[j] = val[j] * r * (w ? w[e] : 1.f); }
        } else if (norm_mode == 2) {                      // the sum runs over the whole of q (or k), which every wave reads
            const int p0 = is_q ? 0 : nq, pn = is_q ? nq : nk;
            float ss = 0.f;
            for (int i = lane; i < pn; i += 64) { const float v = to_f32(src[p0 + i]) + (bias ? bias[p0 + i] : 0.f); ss += v * v; }
            const float r = 1.0f / sqrtf(wave_sum(ss) / (float)pn + eps);
#pragma unroll
            for (int j = 0; j < 8; ++j) { const int e = lane + 64 * j; if (e < dk) val[j] = val[j] * r * w[base - p0 + e]; }
        }
        T* dst = nullptr;
        if (is_q) dst = q_out + (size_t)t * nq + base;
        else if (slot >= 0 && kcache) dst = kcache + (((size_t)pg * nkvh + (head - nh)) * page_size + off) * dk;
        if (dst) {
#pragma unroll
            for (int j = 0; j < 8; ++j) { const int e = lane + 64 * j; if (e < dk) dst[e] = from_f32<T>(val[j]); }
        }
        return;
    }
    const int vh = head - nh - nkvh, base = nq + nk + vh * dv;
    const float lam = (mix_mode == 2) ? lambda[0] : 0.f;
    T* dst = (slot >= 0 && vcache) ? vcache + (((size_t)pg * nkvh + vh) * page_size + off) * dv : nullptr;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int e = lane + 64 * j;
        if (e >= dv) continue;
        float v = to_f32(src[base + e]) + (bias ? bias[base + e] : 0.f);
        float* keep = v_keep + (size_t)t * nv + vh * dv + e;
        if (mix_mode == 1) *keep = v;
        else if (mix_mode == 2) v = (1.0f - lam) * v + lam * *keep;
        if (dst) dst[e] = from_f32<T>(v);
    }
}

// The same work 16 bytes a lane, for head sizes whose 16-byte pieces are a power of two per head (LPH lanes share a head of
// q or k, LPV lanes a head of v) and rows that start on 16-byte boundaries.  Grid (tokens, ceil(items / 256)); an item is one
// 16-byte piece of the row [q | k | v].  norm_mode 0 or 1 (1: the lanes of a head sum their squares among themselves; the whole-row
// norm has a kernel of its own below).  A wave never straddles q/k and v pieces (the launcher pads the q/k pieces to whole waves).
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_store_vec_kernel(const T* __restrict__ rows, int row_stride, const float* __restrict__ bias,
                         const float* __restrict__ qw, const float* __restrict__ kw, int norm_mode, float eps,
                         int mix_mode, const float* __restrict__ lambda, float* __restrict__ v_keep,
                         T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache,
                         const int* __restrict__ slots, int nh, int nkvh, int dk, int dv, int page_size, int qk_items_padded) {
    constexpr int N = RowPack<T>::N;
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int item = blockIdx.y * 256 + threadIdx.x;
    const int nq = nh * dk, nk = nkvh * dk, nv = nkvh * dv;
    const int lph = dk / N, lpv = dv / N;
    const T* src = rows + (size_t)t * row_stride;
    const int slot = slots ? slots[t] : -1;
    const int pg = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - pg * page_size : 0;
    float val[N];
    if (item < qk_items_padded) {                         // (wave-uniform) pieces of q and k
        const bool live = item < (nq + nk) / N;
        const int e0 = live ? item * N : 0;               // first entry of the piece in [q | k]
        const int head = e0 / dk, j0 = e0 - head * dk;
        const bool is_q = head < nh;
        RowPack<T>::load(src + e0, val);
        if (bias) {
            float b[N];
            load_floats<N>(bias + e0, b);
#pragma unroll
            for (int i = 0; i < N; ++i) val[i] += b[i];
        }
        if (norm_mode == 1) {
            float wv[N];
            if (qw) load_floats<N>((is_q ? qw : kw) + j0, wv);        // no weights: the heads are brought to unit root mean square, no more
            else
#pragma unroll
                for (int i = 0; i < N; ++i) wv[i] = 1.f;
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < N; ++i) ss += val[i] * val[i];
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, kWave);       // lph is a power of two and divides 64
            const float r = 1.0f / sqrtf(ss / (float)dk + eps);
#pragma unroll
            for (int i = 0; i < N; ++i) val[i] = val[i] * r * wv[i];
        }
        if (!live) return;
        if (is_q) RowPack<T>::store(q_out + (size_t)t * nq + e0, val);
        else if (slot >= 0 && kcache)
            RowPack<T>::store(kcache + (((size_t)pg * nkvh + (head - nh)) * page_size + off) * dk + j0, val);
        return;
    }
    const int vi = item - qk_items_padded;
    if (vi >= nv / N) return;
    const int e0 = vi * N, vh = e0 / dv, j0 = e0 - vh * dv;
    RowPack<T>::load(src + nq + nk + e0, val);
    if (bias) {
        float b[N];
        load_floats<N>(bias + nq + nk + e0, b);
#pragma unroll
        for (int i = 0; i < N; ++i) val[i] += b[i];
    }
    float* keep = v_keep + (size_t)t * nv + e0;
    if (mix_mode == 1) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) reinterpret_cast<float4*>(keep)[i] = make_float4(val[4 * i], val[4 * i + 1], val[4 * i + 2], val[4 * i + 3]);
    } else if (mix_mode == 2) {
        const float lam = lambda[0];
        float kv[N];
        load_floats<N>(keep, kv);
#pragma unroll
        for (int i = 0; i < N; ++i) val[i] = (1.0f - lam) * val[i] + lam * kv[i];
    }
    if (slot >= 0 && vcache) RowPack<T>::store(vcache + (((size_t)pg * nkvh + vh) * page_size + off) * dv + j0, val);
    (void)lpv;
}

// norm_mode 2, 16 bytes a lane: one block per token (256 threads, or 1024 for rows of more than 512 pieces).  The sums of squares over the whole of q and of k are formed once
// (first pass), then the row is read again (from cache), scaled and stored; the values follow.
template <typename T>
__global__ void __launch_bounds__(1024)
qk_norm_store_whole_kernel(const T* __restrict__ rows, int row_stride, const float* __restrict__ bias,
                           const float* __restrict__ qw, const float* __restrict__ kw, float eps,
                           int mix_mode, const float* __restrict__ lambda, float* __restrict__ v_keep,
                           T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache,
                           const int* __restrict__ slots, int nh, int nkvh, int dk, int dv, int page_size) {
    constexpr int N = RowPack<T>::N;
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int nq = nh * dk, nk = nkvh * dk, nv = nkvh * dv;
    const T* src = rows + (size_t)t * row_stride;
    const int slot = slots ? slots[t] : -1;
    const int pg = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - pg * page_size : 0;
    const int qk_items = (nq + nk) / N;
    float sq = 0.f, sk = 0.f;
    for (int item = tid; item < qk_items; item += blockDim.x) {
        float v[N], b[N];
        RowPack<T>::load(src + item * N, v);
        if (bias) load_floats<N>(bias + item * N, b);
        float s2 = 0.f;
#pragma unroll
        for (int e = 0; e < N; ++e) { const float z = v[e] + (bias ? b[e] : 0.f); s2 += z * z; }
        if (item * N < nq) sq += s2; else sk += s2;
    }
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    const float rq = 1.0f / sqrtf(sq / (float)nq + eps), rk = 1.0f / sqrtf(sk / (float)nk + eps);
    for (int item = tid; item < qk_items; item += blockDim.x) {
        const int e0 = item * N;
        const bool is_q = e0 < nq;
        float v[N], b[N], wv[N];
        RowPack<T>::load(src + e0, v);
        if (bias) load_floats<N>(bias + e0, b);
        load_floats<N>(is_q ? qw + e0 : kw + (e0 - nq), wv);
        const float r = is_q ? rq : rk;
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = (v[e] + (bias ? b[e] : 0.f)) * r * wv[e];
        if (is_q) RowPack<T>::store(q_out + (size_t)t * nq + e0, v);
        else if (slot >= 0 && kcache) {
            const int kh = (e0 - nq) / dk, j0 = (e0 - nq) - kh * dk;
            RowPack<T>::store(kcache + (((size_t)pg * nkvh + kh) * page_size + off) * dk + j0, v);
        }
    }
    const float lam = (mix_mode == 2) ? lambda[0] : 0.f;
    for (int vi = tid; vi < nv / N; vi += blockDim.x) {
        const int e0 = vi * N, vh = e0 / dv, j0 = e0 - vh * dv;
        float v[N], b[N], kv[N];
        RowPack<T>::load(src + nq + nk + e0, v);
        if (bias) load_floats<N>(bias + nq + nk + e0, b);
        float* keep = v_keep + (size_t)t * nv + e0;
        if (mix_mode == 2) load_floats<N>(keep, kv);
#pragma unroll
        for (int e = 0; e < N; ++e) {
            v[e] += bias ? b[e] : 0.f;
            if (mix_mode == 2) v[e] = (1.0f - lam) * v[e] + lam * kv[e];
        }
        if (mix_mode == 1) {
#pragma unroll
            for (int i = 0; i < N / 4; ++i) reinterpret_cast<float4*>(keep)[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
        }
        if (slot >= 0 && vcache) RowPack<T>::store(vcache + (((size_t)pg * nkvh + vh) * page_size + off) * dv + j0, v);
    }
}

IC_EXPORT int ic_qk_norm_store(const void* rows, int row_stride, int dtype, const float* bias, const float* qw,
                               const float* kw, int norm_mode, float eps, int mix_mode, const float* lambda,
                               float* v_keep, void* q_out, void* kcache, void* vcache, const int* slots, int T, int nh,
                               int nkvh, int dk, int dv, int page_size, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || dk <= 0 || dv <= 0 || page_size <= 0 || norm_mode < 0 || norm_mode > 2 || mix_mode < 0 ||
        mix_mode > 2)
        return IC_ERR_ARG;
    if ((qw == nullptr) != (kw == nullptr)) return IC_ERR_ARG;
    if (norm_mode == 2 && qw == nullptr) return IC_ERR_ARG;       // the per-head norm (1) may come without weights
    if (mix_mode != 0 && v_keep == nullptr) return IC_ERR_ARG;
    if (mix_mode == 2 && lambda == nullptr) return IC_ERR_ARG;
    const long long n = (long long)(nh + nkvh) * dk + (long long)nkvh * dv;
    if (row_stride < n) return IC_ERR_ARG;
    if (dk > 512 || dv > 512) return IC_ERR_TOO_LARGE;
    const size_t lds = 0;
    {
        // 16 bytes a lane where the sizes allow it: pieces per head of q/k a power of two that divides 64, values in whole pieces,
        // rows, outputs and cache rows on 16-byte boundaries
        const int pack = dtype == IC_F32 ? 4 : 8;
        const int lph = dk % pack == 0 ? dk / pack : 0;
        const bool pow2 = lph > 0 && lph <= 64 && (lph & (lph - 1)) == 0;
        const uintptr_t ptrs = (uintptr_t)rows | (uintptr_t)q_out | (uintptr_t)kcache | (uintptr_t)vcache | (uintptr_t)bias |
                               (uintptr_t)qw | (uintptr_t)kw | (uintptr_t)v_keep;
        if ((dtype == IC_F32 || dtype == IC_BF16) && pow2 && dv % pack == 0 && row_stride % pack == 0 && (ptrs & 15) == 0) {
            if (norm_mode == 2) {
                const int threads = ((long long)(nh + nkvh) * dk / pack > 512) ? 1024 : 256;
                if (dtype == IC_F32)
                    hipLaunchKernelGGL(qk_norm_store_whole_kernel<float>, dim3(T), dim3(threads), 0, stream, (const float*)rows, row_stride,
                                       bias, qw, kw, eps, mix_mode, lambda, v_keep, (float*)q_out, (float*)kcache, (float*)vcache, slots,
                                       nh, nkvh, dk, dv, page_size);
                else
                    hipLaunchKernelGGL(qk_norm_store_whole_kernel<bf16>, dim3(T), dim3(threads), 0, stream, (const bf16*)rows, row_stride,
                                       bias, qw, kw, eps, mix_mode, lambda, v_keep, (bf16*)q_out, (bf16*)kcache, (bf16*)vcache, slots, nh,
                                       nkvh, dk, dv, page_size);
                return ic_launch_status();
            }
            const int qk_items = (int)(((long long)(nh + nkvh) * dk) / pack);
            const int qk_padded = (qk_items + 63) / 64 * 64;
            const int items = qk_padded + nkvh * dv / pack;
            dim3 vgrid(T, (items + 255) / 256), vblock(256);
            if (dtype == IC_F32)
                hipLaunchKernelGGL(qk_norm_store_vec_kernel<float>, vgrid, vblock, 0, stream, (const float*)rows, row_stride, bias, qw,
                                   kw, norm_mode, eps, mix_mode, lambda, v_keep, (float*)q_out, (float*)kcache, (float*)vcache, slots,
                                   nh, nkvh, dk, dv, page_size, qk_padded);
            else
                hipLaunchKernelGGL(qk_norm_store_vec_kernel<bf16>, vgrid, vblock, 0, stream, (const bf16*)rows, row_stride, bias, qw, kw,
                                   norm_mode, eps, mix_mode, lambda, v_keep, (bf16*)q_out, (bf16*)kcache, (bf16*)vcache, slots, nh,
                                   nkvh, dk, dv, page_size, qk_padded);
            return ic_launch_status();
        }
    }
    dim3 grid(T, (nh + 2 * nkvh + 3) / 4), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(qk_norm_store_kernel<float>, grid, block, lds, stream, (const float*)rows, row_stride, bias, qw,
                           kw, norm_mode, eps, mix_mode, lambda, v_keep, (float*)q_out, (float*)kcache, (float*)vcache,
                           slots, nh, nkvh, dk, dv, page_size);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(qk_norm_store_kernel<bf16>, grid, block, lds, stream, (const bf16*)rows, row_stride, bias, qw, kw,
                           norm_mode, eps, mix_mode, lambda, v_keep, (bf16*)q_out, (bf16*)kcache, (bf16*)vcache, slots, nh,
                           nkvh, dk, dv, page_size);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Element-wise activations of a dense feed-forward.  kind 0: relu(z)^2; 1: gelu_tanh(z); 2: silu(z).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float act_apply(float z, int kind) {
    if (kind == 0) { const float r = fmaxf(z, 0.f); return r * r; }
    if (kind == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return z / (1.0f + expf(-z));
}

template <typename T>
__global__ void activation_kernel(const T* __restrict__ in, T* __restrict__ out, long long n, int kind) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = from_f32<T>(act_apply(to_f32(in[i]), kind));
}

// 16 bytes a thread (n a multiple of the pack, both pointers on 16-byte boundaries).
template <typename T>
__global__ void activation_vec_kernel(const T* __restrict__ in, T* __restrict__ out, long long n_packs, int kind) {
    constexpr int N = RowPack<T>::N;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n_packs; i += stride) {
        float v[N];
        RowPack<T>::load(in + i * N, v);
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = act_apply(v[e], kind);
        RowPack<T>::store(out + i * N, v);
    }
}

IC_EXPORT int ic_activation(const void* in, void* out, int dtype, long long n, int kind, hipStream_t stream) {
    if (n <= 0) return IC_OK;
    if (kind < 0 || kind > 2) return IC_ERR_ARG;
    const int pack = dtype == IC_F32 ? 4 : 8;
    if ((dtype == IC_F32 || dtype == IC_BF16) && n % pack == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
        const long long np = n / pack;
        long long vb = (np + 255) / 256;
        if (vb > 8192) vb = 8192;
        if (dtype == IC_F32)
            hipLaunchKernelGGL(activation_vec_kernel<float>, dim3((unsigned)vb), dim3(256), 0, stream, (const float*)in, (float*)out, np, kind);
        else
            hipLaunchKernelGGL(activation_vec_kernel<bf16>, dim3((unsigned)vb), dim3(256), 0, stream, (const bf16*)in, (bf16*)out, np, kind);
        return ic_launch_status();
    }
    long long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    dim3 grid((unsigned)blocks), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(activation_kernel<float>, grid, block, 0, stream, (const float*)in, (float*)out, n, kind);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(activation_kernel<bf16>, grid, block, 0, stream, (const bf16*)in, (bf16*)out, n, kind);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// A sublayer's result behind a gate made from the sublayer's input:
//   v = y[t] * sigmoid(g[t] + gb);  x[t] += v * rsqrt(mean(v^2) + eps) * w;  copy[t] = x[t] in the compute dtype.
// g null: no gate (the kernel is then the plain norm into the stream).  One block per row.
// ---------------------------------------------------------------------------------------------
constexpr int kGnKeep = 16;       // gated values a thread keeps between the two passes (rows up to 256 * 16 wide)
constexpr int kGnPieces = 4;      // the same in 16-byte pieces of the row (rows up to 256 * 4 pieces wide)

// sigmoid for a gate: float32 rows divide and call expf; rows that are rounded to bfloat16 take the hardware's exp2 and
// reciprocal (each good to an ulp)
template <typename T> __device__ __forceinline__ float gate_sigmoid(float z);
template <> __device__ __forceinline__ float gate_sigmoid<float>(float z) { return 1.0f / (1.0f + expf(-z)); }
template <> __device__ __forceinline__ float gate_sigmoid<bf16>(float z) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
}

template <typename TY, typename TC>
__global__ void __launch_bounds__(256)
gated_norm_into_stream_kernel(const TY* __restrict__ y, const TY* __restrict__ g, int g_stride, const float* __restrict__ gb,
                              const float* __restrict__ w, float* __restrict__ x, TC* __restrict__ copy, int d, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const TY* yr = y + (size_t)t * d;
    const TY* gr = g ? g + (size_t)t * g_stride : nullptr;
    auto gated = [&](int i) {
        float v = to_f32(yr[i]);
        if (gr) v *= gate_sigmoid<TY>(to_f32(gr[i]) + (gb ? gb[i] : 0.f));
        return v;
    };
    float keep[kGnKeep];
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < kGnKeep; ++n) {
        const int i = threadIdx.x + n * 256;
        keep[n] = i < d ? gated(i) : 0.f;
        ss += keep[n] * keep[n];
    }
    for (int i = threadIdx.x + kGnKeep * 256; i < d; i += 256) {
        const float v = gated(i);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float* xr = x + (size_t)t * d;
#pragma unroll
    for (int n = 0; n < kGnKeep; ++n) {
        const int i = threadIdx.x + n * 256;
        if (i < d) {
            const float s = xr[i] + keep[n] * r * w[i];
            xr[i] = s;
            if (copy) copy[(size_t)t * d + i] = from_f32<TC>(s);
        }
    }
    for (int i = threadIdx.x + kGnKeep * 256; i < d; i += 256) {
        const float s = xr[i] + gated(i) * r * w[i];
        xr[i] = s;
        if (copy) copy[(size_t)t * d + i] = from_f32<TC>(s);
    }
}

// The same for rows made of whole 16-byte pieces (d, the gate's stride and every address a multiple of a piece): a thread
// a piece, every access 16 bytes.
template <typename TY>
__global__ void __launch_bounds__(256)
gated_norm_into_stream_vec_kernel(const TY* __restrict__ y, const TY* __restrict__ g, int g_stride, const float* __restrict__ gb,
                                  const float* __restrict__ w, float* __restrict__ x, TY* __restrict__ copy, int d, float eps) {
    constexpr int N = RowPack<TY>::N;
    __shared__ float red[16];
    const int t = blockIdx.x, pieces = d / N;
    const TY* yr = y + (size_t)t * d;
    const TY* gr = g ? g + (size_t)t * g_stride : nullptr;
    auto gated = [&](int c, float* v) {
        RowPack<TY>::load(yr + c * N, v);
        if (gr) {
            float z[N], bz[N];
            RowPack<TY>::load(gr + c * N, z);
            if (gb) load_floats<N>(gb + c * N, bz);
#pragma unroll
            for (int j = 0; j < N; ++j) v[j] *= gate_sigmoid<TY>(z[j] + (gb ? bz[j] : 0.f));
        }
    };
    float keep[kGnPieces][N];
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < kGnPieces; ++n) {
        const int c = threadIdx.x + n * 256;
        if (c < pieces) {
            gated(c, keep[n]);
#pragma unroll
            for (int j = 0; j < N; ++j) ss += keep[n][j] * keep[n][j];
        }
    }
    for (int c = threadIdx.x + kGnPieces * 256; c < pieces; c += 256) {
        float v[N];
        gated(c, v);
#pragma unroll
        for (int j = 0; j < N; ++j) ss += v[j] * v[j];
    }
    ss = block_sum(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float* xr = x + (size_t)t * d;
    auto into = [&](int c, const float* v) {
        float xs[N], ws[N];
        load_floats<N>(xr + c * N, xs);
        load_floats<N>(w + c * N, ws);
#pragma unroll
        for (int j = 0; j < N; ++j) xs[j] += v[j] * r * ws[j];
#pragma unroll
        for (int j = 0; j < N / 4; ++j)
            *reinterpret_cast<float4*>(xr + c * N + 4 * j) = make_float4(xs[4 * j], xs[4 * j + 1], xs[4 * j + 2], xs[4 * j + 3]);
        if (copy) RowPack<TY>::store(copy + (size_t)t * d + c * N, xs);
    };
#pragma unroll
    for (int n = 0; n < kGnPieces; ++n) {
        const int c = threadIdx.x + n * 256;
        if (c < pieces) into(c, keep[n]);
    }
    for (int c = threadIdx.x + kGnPieces * 256; c < pieces; c += 256) {
        float v[N];
        gated(c, v);
        into(c, v);
    }
}

IC_EXPORT int ic_gated_norm_into_stream(const void* y, const void* g, int g_stride, int y_dtype, const float* gb, const float* w,
                                        float* x, void* copy, int copy_dtype, int T, int d, float eps, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    dim3 grid(T), block(256);
    const int piece = y_dtype == IC_BF16 ? 8 : 4;
    const auto aligned = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = d % piece == 0 && (g == nullptr || g_stride % piece == 0) && aligned(y) && aligned(g) && aligned(gb) && aligned(w) &&
                     aligned(x) && aligned(copy) && (copy == nullptr || copy_dtype == y_dtype);
    if (vec && y_dtype == IC_F32)
        hipLaunchKernelGGL(gated_norm_into_stream_vec_kernel<float>, grid, block, 0, stream, (const float*)y, (const float*)g, g_stride,
                           gb, w, x, (float*)copy, d, eps);
    else if (vec && y_dtype == IC_BF16)
        hipLaunchKernelGGL(gated_norm_into_stream_vec_kernel<bf16>, grid, block, 0, stream, (const bf16*)y, (const bf16*)g, g_stride,
                           gb, w, x, (bf16*)copy, d, eps);
    else if (y_dtype == IC_F32 && (copy == nullptr || copy_dtype == IC_F32))
        hipLaunchKernelGGL((gated_norm_into_stream_kernel<float, float>), grid, block, 0, stream, (const float*)y, (const float*)g,
                           g_stride, gb, w, x, (float*)copy, d, eps);
    else if (y_dtype == IC_BF16 && (copy == nullptr || copy_dtype == IC_BF16))
        hipLaunchKernelGGL((gated_norm_into_stream_kernel<bf16, bf16>), grid, block, 0, stream, (const bf16*)y, (const bf16*)g,
                           g_stride, gb, w, x, (bf16*)copy, d, eps);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[t, j] = gelu_tanh(z[t, j]) * table[tokens[t], col0 + j], j < n: a gate made from the stream on a slice of the
// token's row of a second embedding table.  gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
token_gate_kernel(const T* __restrict__ z, int z_stride, const T* __restrict__ table, int table_stride, const int* __restrict__ tokens,
                  int col0, int n, T* __restrict__ out, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = (int)(i / n), j = (int)(i - (long long)t * n);
    const float v = to_f32(z[(size_t)t * z_stride + j]);
    const float ge = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    out[i] = from_f32<T>(ge * to_f32(table[(size_t)tokens[t] * table_stride + col0 + j]));
}

IC_EXPORT int ic_token_gate(const void* z, int z_stride, const void* table, int table_stride, int dtype, const int* tokens,
                            int col0, int n, void* out, int T, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (n <= 0 || col0 < 0 || col0 + n > table_stride) return IC_ERR_ARG;
    const long long total = (long long)T * n;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(token_gate_kernel<float>, grid, block, 0, stream, (const float*)z, z_stride, (const float*)table,
                           table_stride, tokens, col0, n, (float*)out, total);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(token_gate_kernel<bf16>, grid, block, 0, stream, (const bf16*)z, z_stride, (const bf16*)table,
                           table_stride, tokens, col0, n, (bf16*)out, total);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
