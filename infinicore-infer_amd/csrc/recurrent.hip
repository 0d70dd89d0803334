// Mixers that carry a fixed-size state per sequence instead of a cache of keys: a short causal convolution
// per channel, a gated diagonal linear recurrence, a state-space recurrence with a matrix state per head, the
// gated norm in groups that follows it, and a product with one small weight matrix per block of columns.
//
// A step's tokens are rows 0..T-1; request r owns rows req_start[r] .. req_start[r+1]-1 and the state slot
// state_slots[r].  State lives in float32, [slots, state_stride] floats, a part of a mixer's state at an offset.
// Everything that enters a recurrence is float32.
#include "common.h"

constexpr int kConvMaxTaps = 8;

__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---- causal convolution per channel -----------------------------------------------------------------------
// in(t, c) = xin[t, c] + in_bias[c]; out(t, c) = act(b[c] + sum_k w[c, k] in(t - (taps-1-k), c)); inputs before
// the step's first row come from the state (the last taps-1 inputs, oldest first), zeros for a new sequence.
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ xin, int xin_stride, const float* __restrict__ in_bias,
                   const float* __restrict__ w, const float* __restrict__ b, int taps, int C,
                   float* __restrict__ out, T* __restrict__ out_copy, int copy_stride, int act,
                   const float* __restrict__ state, long long state_stride,
                   const int* __restrict__ token_req, const int* __restrict__ req_start,
                   const int* __restrict__ state_slots) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (c >= C) return;
    const int r = token_req[t];
    const int start = req_start[r];
    const float* st = state + (long long)state_slots[r] * state_stride;
    const float ib = in_bias ? in_bias[c] : 0.f;
    float acc = b ? b[c] : 0.f;
    for (int k = 0; k < taps; ++k) {
        const int src = t - (taps - 1 - k);
        float v;
        if (src >= start) v = to_f32(xin[(size_t)src * xin_stride + c]) + ib;
        else v = st[(size_t)(taps - 1 - (start - src)) * C + c];
        acc += w[(size_t)c * taps + k] * v;
    }
    if (act == 1) acc = silu_f(acc);
    out[(size_t)t * C + c] = acc;
    if (out_copy) out_copy[(size_t)t * copy_stride + c] = from_f32<T>(acc);
}

// The state after the step: the last taps-1 of (old state, the step's inputs).  One thread per (request, channel).
template <typename T>
__global__ void __launch_bounds__(256)
conv_state_kernel(const T* __restrict__ xin, int xin_stride, const float* __restrict__ in_bias, int taps, int C,
                  float* __restrict__ state, long long state_stride, const int* __restrict__ req_start,
                  const int* __restrict__ state_slots) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
    if (c >= C) return;
    const int start = req_start[r], n = req_start[r + 1] - start;
    float* st = state + (long long)state_slots[r] * state_stride;
    const float ib = in_bias ? in_bias[c] : 0.f;
    float nv[kConvMaxTaps];
    for (int k = 0; k < taps - 1; ++k) {
        const int i = n + k;                      // index into (old state, inputs)
        nv[k] = i < taps - 1 ? st[(size_t)i * C + c]
                             : to_f32(xin[(size_t)(start + i - (taps - 1)) * xin_stride + c]) + ib;
    }
    for (int k = 0; k < taps - 1; ++k) st[(size_t)k * C + c] = nv[k];
}

IC_EXPORT int ic_causal_conv(const void* xin, int xin_stride, int dtype, const float* in_bias, const float* w,
                             const float* b, int taps, int C, float* out, void* out_copy, int copy_stride, int act,
                             float* state, long long state_stride, const int* token_req, const int* req_start,
                             const int* state_slots, int T, int R, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (taps < 1 || taps > kConvMaxTaps || C <= 0 || R <= 0 || !state || !req_start || !state_slots) return IC_ERR_ARG;
    dim3 grid((C + 255) / 256, T), sgrid((C + 255) / 256, R), block(256);
    if (dtype == IC_F32) {
        hipLaunchKernelGGL(causal_conv_kernel<float>, grid, block, 0, stream, (const float*)xin, xin_stride, in_bias, w, b,
                           taps, C, out, (float*)out_copy, copy_stride, act, state, state_stride, token_req, req_start,
                           state_slots);
        if (taps > 1)
            hipLaunchKernelGGL(conv_state_kernel<float>, sgrid, block, 0, stream, (const float*)xin, xin_stride, in_bias,
                               taps, C, state, state_stride, req_start, state_slots);
    } else if (dtype == IC_BF16) {
        hipLaunchKernelGGL(causal_conv_kernel<bf16>, grid, block, 0, stream, (const bf16*)xin, xin_stride, in_bias, w, b,
                           taps, C, out, (bf16*)out_copy, copy_stride, act, state, state_stride, token_req, req_start,
                           state_slots);
        if (taps > 1)
            hipLaunchKernelGGL(conv_state_kernel<bf16>, sgrid, block, 0, stream, (const bf16*)xin, xin_stride, in_bias,
                               taps, C, state, state_stride, req_start, state_slots);
    } else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---- gated diagonal linear recurrence -------------------------------------------------------------------------
// Channel c lies in block c / bw; its gate pre-activations are gates[t, (c / bw) * 2 bw + c % bw] (recurrence
// gate) and the same + bw (input gate), biases laid out alike.  With r, i their sigmoids:
//     log a = decay[c] * r,  S <- exp(log a) S + sqrt(1 - exp(2 log a)) * i * u,  out = S * gelu_tanh(yb + y_bias).
// decay[c] = -8 softplus(lam[c]), made once when the weights are loaded.
//
// Both recurrences of this file are linear in the state, S_end = A S_begin + S_local, so a long portion is cut into
// chunks that run side by side: pass 1 (mode 1) runs every chunk from a zero state and leaves (S_local, A); a small
// kernel walks a request's chunks in order and replaces S_local by the state the chunk really starts from (and
// writes the request's new state); pass 2 (mode 2) runs every chunk again from there and writes the results.
// mode 0 is the single pass from and to the request's state (few tokens).
template <typename T>
__global__ void __launch_bounds__(128)
rglru_scan_kernel(const float* __restrict__ gates, const float* __restrict__ gate_bias, const float* __restrict__ u,
                  const T* __restrict__ yb, int yb_stride, const float* __restrict__ y_bias,
                  const float* __restrict__ decay, int width, int bw, T* __restrict__ out,
                  float* __restrict__ state, long long state_stride, const int* __restrict__ req_start,
                  const int* __restrict__ state_slots, int mode, int chunk_len, int max_chunks,
                  float* __restrict__ scr_s, float* __restrict__ scr_a) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y, ck = blockIdx.z;
    if (c >= width) return;
    const int req_end = req_start[r + 1];
    const int begin = req_start[r] + (mode ? ck * chunk_len : 0);
    const int end = mode ? min(req_end, begin + chunk_len) : req_end;
    if (begin >= req_end) return;
    const int g0 = (c / bw) * 2 * bw + c % bw;
    const float br = gate_bias[g0], bi = gate_bias[g0 + bw], dc = decay[c], yb0 = y_bias ? y_bias[c] : 0.f;
    float* st = state + (long long)state_slots[r] * state_stride;
    const size_t si = ((size_t)r * max_chunks + ck) * width + c;
    float S = mode == 0 ? st[c] : mode == 2 ? scr_s[si] : 0.f;
    float a_total = 1.f;
#pragma unroll 4
    for (int t = begin; t < end; ++t) {
        const float* g = gates + (size_t)t * 2 * width;
        const float rg = sigmoid_f(g[g0] + br), ig = sigmoid_f(g[g0 + bw] + bi);
        const float la = dc * rg;
        const float a = expf(la);
        S = a * S + sqrtf(-expm1f(2.0f * la)) * ig * u[(size_t)t * width + c];
        a_total *= a;
        if (mode != 1)
            out[(size_t)t * width + c] = from_f32<T>(S * gelu_tanh_f(to_f32(yb[(size_t)t * yb_stride + c]) + yb0));
    }
    if (mode == 0) st[c] = S;
    if (mode == 1) { scr_s[si] = S; scr_a[si] = a_total; }
}

// scr_s[r, k, e] <- the state chunk k of request r starts from; state <- the state after the last chunk.
// `per`: state elements per factor (scr_a holds one factor per `per` elements: per channel, or per head).
__global__ void __launch_bounds__(256)
chunk_states_kernel(float* __restrict__ scr_s, const float* __restrict__ scr_a, int n_state, int per, int chunk_len,
                    int max_chunks, float* __restrict__ state, long long state_stride,
                    const int* __restrict__ req_start, const int* __restrict__ state_slots) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
    if (e >= n_state) return;
    const int n = req_start[r + 1] - req_start[r];
    const int chunks = (n + chunk_len - 1) / chunk_len;
    float* st = state + (long long)state_slots[r] * state_stride;
    float S = st[e];
    for (int k = 0; k < chunks; ++k) {
        const size_t i = ((size_t)r * max_chunks + k) * n_state + e;
        const float local = scr_s[i];
        scr_s[i] = S;
        S = scr_a[((size_t)r * max_chunks + k) * (n_state / per) + e / per] * S + local;
    }
    st[e] = S;
}

IC_EXPORT int ic_rglru_scan(const float* gates, const float* gate_bias, const float* u, const void* yb, int yb_stride,
                            int dtype, const float* y_bias, const float* decay, int width, int bw, void* out,
                            float* state, long long state_stride, const int* req_start, const int* state_slots, int R,
                            int chunk_len, int max_chunks, float* scr_s, float* scr_a, hipStream_t stream) {
    if (R <= 0) return IC_OK;
    if (width <= 0 || bw <= 0 || width % bw || !state) return IC_ERR_ARG;
    const bool chunked = chunk_len > 0 && max_chunks > 1;
    if (chunked && (!scr_s || !scr_a || max_chunks > 65535)) return IC_ERR_ARG;
    dim3 block(128);
    for (int pass = 0; pass < (chunked ? 3 : 1); ++pass) {
        const int mode = chunked ? (pass == 0 ? 1 : 2) : 0;
        if (chunked && pass == 1) {
            hipLaunchKernelGGL(chunk_states_kernel, dim3((width + 255) / 256, R), dim3(256), 0, stream, scr_s, scr_a, width, 1,
                               chunk_len, max_chunks, state, state_stride, req_start, state_slots);
            continue;
        }
        dim3 grid((width + 127) / 128, R, chunked ? max_chunks : 1);
        if (dtype == IC_F32)
            hipLaunchKernelGGL(rglru_scan_kernel<float>, grid, block, 0, stream, gates, gate_bias, u, (const float*)yb, yb_stride,
                               y_bias, decay, width, bw, (float*)out, state, state_stride, req_start, state_slots, mode,
                               chunk_len, max_chunks, scr_s, scr_a);
        else if (dtype == IC_BF16)
            hipLaunchKernelGGL(rglru_scan_kernel<bf16>, grid, block, 0, stream, gates, gate_bias, u, (const bf16*)yb, yb_stride,
                               y_bias, decay, width, bw, (bf16*)out, state, state_stride, req_start, state_slots, mode,
                               chunk_len, max_chunks, scr_s, scr_a);
        else
            return IC_ERR_UNSUPPORTED;
    }
    return ic_launch_status();
}

// ---- state-space recurrence with a matrix state per head ---------------------------------------------------------
// xbc [T, x_stride >= inner + 2 G N] (float32, or the step's compute dtype; in_act 1: silu on the way in) holds x
// (heads x P), then B (G x N), then C (G x N) of every token.  Per head h with group g = h / (heads / G),
// dt = softplus(dt_raw + dt_bias[h]):
//     S <- exp(neg_a[h] dt) S + dt B_g x_h^T   (S is N x P),   y_h = S^T C_g + D[h] x_h.
// Without step sizes (dt_raw null) the decay is fixed per head and every step is one: S <- neg_a[h] S + B_g x_h^T
// (neg_a then holds the decay itself): linear attention with keys B, values x and queries C.  D null: no skip term.
// One block per (head, request, chunk).  Thread (grp, p) keeps column p of a run of NI rows of S in registers;
// a token's B, C and x pass through LDS, the next token's are loaded while this one is computed.
template <typename T, int NI, bool FULL>       // FULL: every thread owns exactly NI rows (N = NI * groups): no guards, 16-byte LDS reads
__global__ void __launch_bounds__(256)
ssm_scan_kernel(const void* __restrict__ xbc, int x_stride, int x_f32, int in_act, const T* __restrict__ dt_raw, int dt_stride,
                const float* __restrict__ dt_bias, const float* __restrict__ neg_a, const float* __restrict__ Dw,
                int heads, int P, int N, int G, float* __restrict__ y, float* __restrict__ state,
                long long state_stride, const int* __restrict__ req_start, const int* __restrict__ state_slots,
                int mode, int chunk_len, int max_chunks, float* __restrict__ scr_s, float* __restrict__ scr_a) {
    extern __shared__ float lds[];
    const int h = blockIdx.x, r = blockIdx.y, ck = blockIdx.z, tid = threadIdx.x;
    const int req_end = req_start[r + 1];
    const int begin = req_start[r] + (mode ? ck * chunk_len : 0);
    const int end = mode ? min(req_end, begin + chunk_len) : req_end;
    if (begin >= req_end) return;
    const int g = h / (heads / G), inner = heads * P;
    const int ngrp = 256 / P, ni = (N + ngrp - 1) / ngrp;       // P <= 256, ni <= NI
    const int grp = tid / P, p = tid % P, n0 = grp * ni;
    const bool active = grp < ngrp;
    const int bufsz = 2 * N + P;                                 // B, C, x of one token; <= 1024
    float* buf0 = lds;
    float* buf1 = lds + bufsz;
    float* part = lds + 2 * bufsz;                               // ngrp * P
    float* st = state + (long long)state_slots[r] * state_stride + (size_t)h * N * P;
    float* sc = scr_s + (((size_t)r * max_chunks + ck) * heads + h) * N * P;
    float s[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int n = n0 + i;
        const bool ok = active && i < ni && n < N;
        s[i] = !ok ? 0.f : mode == 0 ? st[n * P + p] : mode == 2 ? sc[n * P + p] : 0.f;
    }
    const float db = dt_bias ? dt_bias[h] : 0.f, na = neg_a[h], dw = Dw ? Dw[h] : 0.f;
    // a token's inputs as they lie in memory: float32, or the step's compute dtype (a projection's own rows), with silu on the way in
    auto ldx = [&](size_t i) -> float {
        const float v = x_f32 ? reinterpret_cast<const float*>(xbc)[i] : to_f32(reinterpret_cast<const T*>(xbc)[i]);
        return in_act ? silu_f(v) : v;
    };
    const int off_b = inner + g * N, off_c = inner + G * N + g * N, off_x = h * P;
    auto src = [&](int e) { return e < N ? off_b + e : e < 2 * N ? off_c + (e - N) : off_x + (e - 2 * N); };
    float pre[4];
    {
        const size_t row = (size_t)begin * x_stride;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int e = tid + 256 * k;
            if (e < bufsz) buf0[e] = ldx(row + src(e));
        }
    }
    float dt_next = dt_raw ? to_f32(dt_raw[(size_t)begin * dt_stride + h]) : 0.f;
    float a_total = 1.f;
    __syncthreads();
    for (int t = begin; t < end; ++t) {
        float* cur = ((t - begin) & 1) ? buf1 : buf0;
        float* nxt = ((t - begin) & 1) ? buf0 : buf1;
        const float dt = dt_raw ? softplus_f(dt_next + db) : 1.f;       // no step sizes: a fixed decay per head, steps of one
        const bool more = t + 1 < end;
        if (more) {
            const size_t row = (size_t)(t + 1) * x_stride;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int e = tid + 256 * k;
                if (e < bufsz) pre[k] = ldx(row + src(e));
            }
            if (dt_raw) dt_next = to_f32(dt_raw[(size_t)(t + 1) * dt_stride + h]);
        }
        const float da = dt_raw ? expf(na * dt) : na;
        a_total *= da;
        const float* Bs = cur;
        const float* Cs = cur + N;
        const float* xs = cur + 2 * N;
        if (active) {
            const float dx = dt * xs[p];
            float acc = 0.f;
            if (FULL) {
#pragma unroll
                for (int i = 0; i < NI; i += 4) {
                    const float4 b4 = *reinterpret_cast<const float4*>(Bs + n0 + i);
                    const float4 c4 = *reinterpret_cast<const float4*>(Cs + n0 + i);
                    s[i] = da * s[i] + b4.x * dx;
                    s[i + 1] = da * s[i + 1] + b4.y * dx;
                    s[i + 2] = da * s[i + 2] + b4.z * dx;
                    s[i + 3] = da * s[i + 3] + b4.w * dx;
                    acc += s[i] * c4.x + s[i + 1] * c4.y + s[i + 2] * c4.z + s[i + 3] * c4.w;
                }
            } else {
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const int n = n0 + i;
                    if (i < ni && n < N) {
                        s[i] = da * s[i] + Bs[n] * dx;
                        acc += s[i] * Cs[n];
                    }
                }
            }
            if (mode != 1) part[grp * P + p] = acc;
        }
        __syncthreads();
        if (mode != 1 && tid < P) {
            float acc = dw * xs[tid];
            for (int q = 0; q < ngrp; ++q) acc += part[q * P + tid];
            y[(size_t)t * inner + h * P + tid] = acc;
        }
        if (more) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int e = tid + 256 * k;
                if (e < bufsz) nxt[e] = pre[k];
            }
        }
        __syncthreads();
    }
    if (mode == 2) return;
    float* dst = mode == 0 ? st : sc;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int n = n0 + i;
        if (active && i < ni && n < N) dst[n * P + p] = s[i];
    }
    if (mode == 1 && tid == 0) scr_a[((size_t)r * max_chunks + ck) * heads + h] = a_total;
}

template <typename T>
static int ssm_launch(int ni, dim3 grid, size_t lds, hipStream_t stream, const void* xbc, int x_stride, int x_f32, int in_act,
                      const void* dt_raw, int dt_stride,
                      const float* dt_bias, const float* neg_a, const float* Dw, int heads, int P, int N, int G, float* y,
                      float* state, long long state_stride, const int* req_start, const int* state_slots, int mode,
                      int chunk_len, int max_chunks, float* scr_s, float* scr_a) {
    const bool full = N % 4 == 0 && P % 4 == 0 && 256 % P == 0 && (256 / P) * ni == N;      // (multiples of 4 keep the LDS rows 16-byte aligned)
#define IC_SSM(NI)                                                                                                      \
    do {                                                                                                                \
    if (full && ni == NI)                                                                                               \
        hipLaunchKernelGGL((ssm_scan_kernel<T, NI, true>), grid, dim3(256), lds, stream, xbc, x_stride, x_f32, in_act, (const T*)dt_raw, dt_stride, \
                           dt_bias, neg_a, Dw, heads, P, N, G, y, state, state_stride, req_start, state_slots, mode,     \
                           chunk_len, max_chunks, scr_s, scr_a);                                                         \
    else                                                                                                                \
        hipLaunchKernelGGL((ssm_scan_kernel<T, NI, false>), grid, dim3(256), lds, stream, xbc, x_stride, x_f32, in_act, (const T*)dt_raw, dt_stride, \
                           dt_bias, neg_a, Dw, heads, P, N, G, y, state, state_stride, req_start, state_slots, mode,     \
                           chunk_len, max_chunks, scr_s, scr_a);                                                         \
    } while (0)
    if (ni <= 8) IC_SSM(8);
    else if (ni <= 16) IC_SSM(16);
    else if (ni <= 32) IC_SSM(32);
    else if (ni <= 64) IC_SSM(64);
    else if (ni <= 128) IC_SSM(128);
    else return IC_ERR_TOO_LARGE;
#undef IC_SSM
    return IC_OK;
}

IC_EXPORT int ic_ssm_scan(const void* xbc, int x_stride, int x_dtype, int in_act, const void* dt_raw, int dt_stride, int dtype, const float* dt_bias,
                          const float* neg_a, const float* Dw, int heads, int P, int N, int G, float* y, float* state,
                          long long state_stride, const int* req_start, const int* state_slots, int R, int chunk_len,
                          int max_chunks, float* scr_s, float* scr_a, hipStream_t stream) {
    if (R <= 0) return IC_OK;
    if (heads <= 0 || P <= 0 || P > 256 || N <= 0 || G <= 0 || heads % G || !state || !xbc || !neg_a) return IC_ERR_ARG;
    if (x_stride < heads * P + 2 * G * N || (x_dtype != IC_F32 && x_dtype != dtype)) return IC_ERR_ARG;
    if (2 * N + P > 1024) return IC_ERR_TOO_LARGE;
    const int x_f32 = x_dtype == IC_F32;
    const bool chunked = chunk_len > 0 && max_chunks > 1;
    if (chunked && (!scr_s || !scr_a || max_chunks > 65535)) return IC_ERR_ARG;
    const int ngrp = 256 / P, ni = (N + ngrp - 1) / ngrp;
    const size_t lds = ((size_t)2 * (2 * N + P) + (size_t)ngrp * P) * sizeof(float);
    for (int pass = 0; pass < (chunked ? 3 : 1); ++pass) {
        const int mode = chunked ? (pass == 0 ? 1 : 2) : 0;
        if (chunked && pass == 1) {
            const int n_state = heads * N * P;
            hipLaunchKernelGGL(chunk_states_kernel, dim3((n_state + 255) / 256, R), dim3(256), 0, stream, scr_s, scr_a, n_state,
                               N * P, chunk_len, max_chunks, state, state_stride, req_start, state_slots);
            continue;
        }
        dim3 grid(heads, R, chunked ? max_chunks : 1);
        int st;
        if (dtype == IC_F32)
            st = ssm_launch<float>(ni, grid, lds, stream, xbc, x_stride, x_f32, in_act, dt_raw, dt_stride, dt_bias, neg_a, Dw, heads, P, N, G, y, state,
                                   state_stride, req_start, state_slots, mode, chunk_len, max_chunks, scr_s, scr_a);
        else if (dtype == IC_BF16)
            st = ssm_launch<bf16>(ni, grid, lds, stream, xbc, x_stride, x_f32, in_act, dt_raw, dt_stride, dt_bias, neg_a, Dw, heads, P, N, G, y, state,
                                  state_stride, req_start, state_slots, mode, chunk_len, max_chunks, scr_s, scr_a);
        else
            return IC_ERR_UNSUPPORTED;
        if (st != IC_OK) return st;
    }
    return ic_launch_status();
}

// ---- gate and RMS norm in groups --------------------------------------------------------------------------------------
// mode 0: v = y * silu(z); every group of `gs` columns is divided by its own root mean square; times w (the gate before
// the norm).  mode 1: y's groups are divided by their root mean square, times w, times sigmoid(z) (the gate after it).
// One block per (token, group).
template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_stride, const float* __restrict__ w,
                        int inner, int gs, float eps, T* __restrict__ out, int mode) {
    extern __shared__ float v_row[];          // gs floats
    __shared__ float red[8];
    const int t = blockIdx.x, c0 = blockIdx.y * gs;
    float ss = 0.f;
    for (int j = threadIdx.x; j < gs; j += blockDim.x) {
        float v = y[(size_t)t * inner + c0 + j];
        if (mode == 0) v *= silu_f(to_f32(z[(size_t)t * z_stride + c0 + j]));
        v_row[j] = v;
        ss += v * v;
    }
    const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)gs + eps);
    for (int j = threadIdx.x; j < gs; j += blockDim.x) {
        float v = v_row[j] * r * w[c0 + j];
        if (mode == 1) v *= sigmoid_f(to_f32(z[(size_t)t * z_stride + c0 + j]));
        out[(size_t)t * inner + c0 + j] = from_f32<T>(v);
    }
}

IC_EXPORT int ic_gated_group_norm(const float* y, const void* z, int z_stride, int dtype, const float* w, int inner,
                                  int groups, float eps, void* out, int T, int mode, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (inner <= 0 || groups <= 0 || inner % groups || inner / groups > 16128 || mode < 0 || mode > 1) return IC_ERR_ARG;
    const int gs = inner / groups;
    dim3 grid(T, groups), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, gs * sizeof(float), stream, y, (const float*)z,
                           z_stride, w, inner, gs, eps, (float*)out, mode);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(gated_group_norm_kernel<bf16>, grid, block, gs * sizeof(float), stream, y, (const bf16*)z,
                           z_stride, w, inner, gs, eps, (bf16*)out, mode);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---- a product with one weight matrix per block of columns --------------------------------------------------------------
// C[m, b * c_step + n] = sum_k A[m, b * a_step + k] W[b, n, k]  (b < B, n < N, k < K; W contiguous [B, N, K]),
// optionally times sigmoid(gate[m, b * c_step + n]).  float32 accumulation on the vector units; tiles of BM x 64
// results per block of 256 threads, 16 k at a time through LDS.
template <typename T, typename TC, int BM>
__global__ void __launch_bounds__(256)
blocked_product_kernel(const T* __restrict__ A, int lda, int a_step, const T* __restrict__ W, TC* __restrict__ C,
                       int ldc, int c_step, const T* __restrict__ gate, int gate_stride, int M, int N, int K) {
    constexpr int BN = 64, BK = 16, RM = BM / 16;
    __shared__ float As[BK][BM + 1];
    __shared__ float Ws[BK][BN + 1];
    const int b = blockIdx.z, m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const T* Ab = A + (size_t)b * a_step;
    const T* Wb = W + (size_t)b * N * K;
    float acc[RM][4];
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int e = threadIdx.x; e < BM * BK; e += 256) {
            const int m = e / BK, k = e % BK;
            As[k][m] = (m0 + m < M && k0 + k < K) ? to_f32(Ab[(size_t)(m0 + m) * lda + k0 + k]) : 0.f;
        }
        for (int e = threadIdx.x; e < BN * BK; e += 256) {
            const int n = e / BK, k = e % BK;
            Ws[k][n] = (n0 + n < N && k0 + k < K) ? to_f32(Wb[(size_t)(n0 + n) * K + k0 + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[RM], w[4];
#pragma unroll
            for (int i = 0; i < RM; ++i) a[i] = As[k][ty * RM + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * w[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        const int m = m0 + ty * RM + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (gate) v *= sigmoid_f(to_f32(gate[(size_t)m * gate_stride + (size_t)b * c_step + n]));
            C[(size_t)m * ldc + (size_t)b * c_step + n] = from_f32<TC>(v);
        }
    }
}

// Up to 8 rows: nothing is tiled, the weights stream through once.  Eight lanes share a column and read its
// weight row 16 bytes a lane (one cache line a round); the rows of A wait in LDS as floats.
template <typename T, typename TC, int MT>
__global__ void __launch_bounds__(256)
blocked_product_rows_kernel(const T* __restrict__ A, int lda, int a_step, const T* __restrict__ W, TC* __restrict__ C,
                            int ldc, int c_step, const T* __restrict__ gate, int gate_stride, int M, int N, int K) {
    constexpr int VEC = 16 / sizeof(T);
    extern __shared__ float a_rows[];         // MT * K
    const int b = blockIdx.y, n = blockIdx.x * 32 + threadIdx.x / 8, sub = threadIdx.x % 8;
    for (int e = threadIdx.x; e < MT * K; e += 256) {
        const int mm = e / K, k = e % K;
        a_rows[e] = mm < M ? to_f32(A[(size_t)mm * lda + (size_t)b * a_step + k]) : 0.f;
    }
    __syncthreads();
    float acc[MT];
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) acc[mm] = 0.f;
    const T* wrow = W + ((size_t)b * N + (n < N ? n : 0)) * K;
#pragma unroll 4
    for (int ch = sub; ch < K / VEC; ch += 8) {
        alignas(16) T wv[VEC];
        *reinterpret_cast<uint4*>(wv) = load_stream16(wrow + ch * VEC);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            const float wf = to_f32(wv[v]);
#pragma unroll
            for (int mm = 0; mm < MT; ++mm) acc[mm] += a_rows[mm * K + ch * VEC + v] * wf;
        }
    }
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) {
        float v = acc[mm];
        v += __shfl_xor(v, 4, kWave);
        v += __shfl_xor(v, 2, kWave);
        v += __shfl_xor(v, 1, kWave);
        if (sub == 0 && n < N && mm < M) {
            if (gate) v *= sigmoid_f(to_f32(gate[(size_t)mm * gate_stride + (size_t)b * c_step + n]));
            C[(size_t)mm * ldc + (size_t)b * c_step + n] = from_f32<TC>(v);
        }
    }
}

// More than 8 rows in bfloat16 on the matrix cores: a wave owns 32 rows x 32 columns and computes them transposed,
// C^T = W A^T with v_mfma_f32_32x32x16_bf16, so that both operands are 16 bytes a lane of a row as it lies in memory
// (A operand: weight row l % 32, values 8h..8h+7 of the step; B operand: row l % 32 of A, the same values) and nothing
// passes LDS.  Accumulator r of a lane is column 8(r / 4) + 4h + r % 4 of its row.
typedef __bf16 bp_bf16x8 __attribute__((ext_vector_type(8)));
typedef float bp_v16f __attribute__((ext_vector_type(16)));

template <typename TC>
__global__ void __launch_bounds__(256)
blocked_product_mfma_kernel(const bf16* __restrict__ A, int lda, int a_step, const bf16* __restrict__ W, TC* __restrict__ C,
                            int ldc, int c_step, const bf16* __restrict__ gate, int gate_stride, int M, int N, int K) {
    const int b = blockIdx.z, wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lq = lane & 31, half = lane >> 5;
    const int m0 = blockIdx.y * 64 + 32 * (wave >> 1), n0 = blockIdx.x * 64 + 32 * (wave & 1);
    if (m0 >= M || n0 >= N) return;
    const int m = m0 + lq, n = n0 + lq;
    const bf16* ap = A + (size_t)(m < M ? m : M - 1) * lda + (size_t)b * a_step + 8 * half;
    const bf16* wp = W + ((size_t)b * N + (n < N ? n : N - 1)) * K + 8 * half;
    bp_v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    int k0 = 0;
    for (; k0 + 64 <= K; k0 += 64) {              // four steps' loads in flight together
        bp_bf16x8 wv[4], av[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wv[i] = *reinterpret_cast<const bp_bf16x8*>(wp + k0 + 16 * i);
            av[i] = *reinterpret_cast<const bp_bf16x8*>(ap + k0 + 16 * i);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv[i], av[i], acc, 0, 0, 0);
    }
    for (; k0 < K; k0 += 16) {
        const bp_bf16x8 wv = *reinterpret_cast<const bp_bf16x8*>(wp + k0);
        const bp_bf16x8 av = *reinterpret_cast<const bp_bf16x8*>(ap + k0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv, av, acc, 0, 0, 0);
    }
    if (m >= M) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int nn = n0 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (nn < N) {
            float v = acc[r];
            if (gate) v *= sigmoid_f(to_f32(gate[(size_t)m * gate_stride + (size_t)b * c_step + nn]));
            C[(size_t)m * ldc + (size_t)b * c_step + nn] = from_f32<TC>(v);
        }
    }
}

template <typename T> struct bp_is_bf16 { static constexpr bool value = false; };
template <> struct bp_is_bf16<bf16> { static constexpr bool value = true; };

template <typename T, typename TC>
static void blocked_product_launch(const void* A, int lda, int a_step, const void* W, void* C, int ldc, int c_step,
                                   const void* gate, int gate_stride, int M, int N, int K, int B, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    if (M <= 8 && K % VEC == 0 && (size_t)8 * K * sizeof(float) <= 48 * 1024 && ((uintptr_t)W % 16) == 0) {
        dim3 grid((N + 31) / 32, B);
#define IC_ROWS(MT)                                                                                                   \
    hipLaunchKernelGGL((blocked_product_rows_kernel<T, TC, MT>), grid, dim3(256), (size_t)MT * K * sizeof(float), stream, \
                       (const T*)A, lda, a_step, (const T*)W, (TC*)C, ldc, c_step, (const T*)gate, gate_stride, M, N, K)
        if (M == 1) IC_ROWS(1); else if (M == 2) IC_ROWS(2); else if (M <= 4) IC_ROWS(4); else IC_ROWS(8);
#undef IC_ROWS
        return;
    }
    if constexpr (bp_is_bf16<T>::value) {
        if (M > 8 && K % 16 == 0 && lda % 8 == 0 && a_step % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0) {
            dim3 grid((N + 63) / 64, (M + 63) / 64, B);
            hipLaunchKernelGGL((blocked_product_mfma_kernel<TC>), grid, dim3(256), 0, stream, (const bf16*)A, lda, a_step,
                               (const bf16*)W, (TC*)C, ldc, c_step, (const bf16*)gate, gate_stride, M, N, K);
            return;
        }
    }
    // 16-row tiles for few rows, and wherever 64-row tiles would be fewer blocks than the chip has compute units
    if (M <= 16 || (long long)((N + 63) / 64) * ((M + 63) / 64) * B < 256) {
        dim3 grid((N + 63) / 64, (M + 15) / 16, B);
        hipLaunchKernelGGL((blocked_product_kernel<T, TC, 16>), grid, dim3(256), 0, stream, (const T*)A, lda, a_step,
                           (const T*)W, (TC*)C, ldc, c_step, (const T*)gate, gate_stride, M, N, K);
    } else {
        dim3 grid((N + 63) / 64, (M + 63) / 64, B);
        hipLaunchKernelGGL((blocked_product_kernel<T, TC, 64>), grid, dim3(256), 0, stream, (const T*)A, lda, a_step,
                           (const T*)W, (TC*)C, ldc, c_step, (const T*)gate, gate_stride, M, N, K);
    }
}

IC_EXPORT int ic_blocked_product(const void* A, int lda, int a_step, const void* W, int dtype, void* C, int c_dtype,
                                 int ldc, int c_step, const void* gate, int gate_stride, int M, int N, int K, int B,
                                 hipStream_t stream) {
    if (M <= 0) return IC_OK;
    if (N <= 0 || K <= 0 || B <= 0 || B > 65535 || (M + 15) / 16 > 65535) return IC_ERR_ARG;
    if (dtype == IC_F32 && c_dtype == IC_F32)
        blocked_product_launch<float, float>(A, lda, a_step, W, C, ldc, c_step, gate, gate_stride, M, N, K, B, stream);
    else if (dtype == IC_BF16 && c_dtype == IC_BF16)
        blocked_product_launch<bf16, bf16>(A, lda, a_step, W, C, ldc, c_step, gate, gate_stride, M, N, K, B, stream);
    else if (dtype == IC_BF16 && c_dtype == IC_F32)
        blocked_product_launch<bf16, float>(A, lda, a_step, W, C, ldc, c_step, gate, gate_stride, M, N, K, B, stream);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
