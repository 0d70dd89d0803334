// Attention over the paged cache for mixers whose keys and values have different sizes per head and
// whose queries see a SPAN of the keys: the last `window` keys (window 0: all earlier keys) plus the
// first `keep_first` keys of the sequence, which are never dropped.  Query at position i sees key j when
//     j <= i  and  (window == 0  or  i - j < window  or  j < keep_first).
// `sink` adds one term to the softmax's denominator that has no value, exp(0) or, with `sinks` (one float32
// per head, a learned number), exp(sinks[h]):
//     p_j = exp(s_j) / (exp(sink_h) + sum_j exp(s_j)).
// `softcap` c > 0 bounds the scaled score before the softmax: s <- c tanh(s / c).  The sink is neither scaled nor capped.
// `gate` (nullable): the result is multiplied element by element with sigmoid(gate[t, h * dv + d]).
// Scores, the running softmax and the sums are float32.
//
// Cache layout of one layer: K plane [num_pages, n_kv_heads, page_size, dk], V plane [.., dv].
//
// This file holds the general kernel (any sizes, float32 or bfloat16), which is also the yardstick of
// the others, a split-key kernel for single new tokens and a matrix-core kernel for prompt portions
// (key and value sizes 32, 64 or 128 each).
#include "common.h"

constexpr int kSpanMaxDim = 512;

// The visible keys of a query at `pos` as two runs: [0, n_kept) and [lo, pos].
struct SpanRuns {
    int n_kept;   // keys 0 .. n_kept-1 (the kept first keys that lie before the window)
    int lo;       // first key of the window
    int total;    // number of visible keys
};
__device__ __forceinline__ SpanRuns span_runs(int pos, int window, int keep_first) {
    SpanRuns r;
    r.lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    r.n_kept = keep_first < r.lo ? keep_first : r.lo;
    if (r.n_kept < 0) r.n_kept = 0;
    r.total = r.n_kept + (pos - r.lo + 1);
    return r;
}
__device__ __forceinline__ int span_key(const SpanRuns& r, int i) { return i < r.n_kept ? i : r.lo + (i - r.n_kept); }

// One wave per (token, head): walks the visible keys 64 at a time.
template <typename T>
__global__ void __launch_bounds__(64)
attn_span_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                         const T* __restrict__ gate, int gate_stride,
                         const T* __restrict__ kcache, const T* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ token_req, const int* __restrict__ positions,
                         int nh, int nkvh, int dk, int dv, int page_size, float scale, int window, int keep_first,
                         int sink, const float* __restrict__ sinks, float softcap) {
    __shared__ float qs[kSpanMaxDim];
    __shared__ float ps[64];
    __shared__ long long vrow[64];

    const int h = blockIdx.x % nh, t = blockIdx.x / nh, lane = threadIdx.x;
    const int kvh = h / (nh / nkvh);
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const T* qp = q + (size_t)t * q_stride + (size_t)h * dk;
    for (int d = lane; d < dk; d += 64) qs[d] = to_f32(qp[d]);
    __syncthreads();

    const SpanRuns runs = span_runs(pos, window, keep_first);
    const int nd = (dv + 63) / 64;
    float acc[kSpanMaxDim / 64];
#pragma unroll
    for (int i = 0; i < kSpanMaxDim / 64; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;

    for (int ib = 0; ib < runs.total; ib += 64) {
        const int idx = ib + lane;
        const bool valid = idx < runs.total;
        float s = -INFINITY;
        long long vbase = 0;
        if (valid) {
            const int key = span_key(runs, idx);
            const int pg = bt[key / page_size];
            const int off = key % page_size;
            const long long rowi = ((long long)pg * nkvh + kvh) * page_size + off;
            vbase = rowi * dv;
            const T* kp = kcache + rowi * dk;
            float dot = 0.f;
            for (int d = 0; d < dk; ++d) dot += qs[d] * to_f32(kp[d]);
            s = dot * scale;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        }
        const float m_new = fmaxf(m, wave_max(s));       // lane 0 of every chunk is valid: m_new is finite
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);               // exp(-inf) = 0 on the first chunk
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        vrow[lane] = vbase;
        __syncthreads();
        const int nk = (runs.total - ib < 64) ? runs.total - ib : 64;
#pragma unroll
        for (int i = 0; i < kSpanMaxDim / 64; ++i) {
            if (i < nd) {
                const int d = lane + 64 * i;
                float a = acc[i] * corr;
                if (d < dv)
                    for (int kk = 0; kk < nk; ++kk) a += ps[kk] * to_f32(vcache[vrow[kk] + d]);
                acc[i] = a;
            }
        }
    }
    if (sink) {                                           // the term exp(sink - m) joins the denominator
        const float sv = sinks ? sinks[h] : 0.f;
        const float m_new = fmaxf(m, sv);
        const float corr = expf(m - m_new);
        l = l * corr + expf(sv - m_new);
#pragma unroll
        for (int i = 0; i < kSpanMaxDim / 64; ++i) acc[i] *= corr;
    }
    T* op = out + (size_t)t * out_stride + (size_t)h * dv;
    const T* gp = gate ? gate + (size_t)t * gate_stride + (size_t)h * dv : nullptr;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < kSpanMaxDim / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < dv) {
            float o = acc[i] * inv;
            if (gp) o *= 1.0f / (1.0f + expf(-to_f32(gp[d])));
            op[d] = from_f32<T>(o);
        }
    }
}

IC_EXPORT int ic_attn_span_generic(const void* q, int q_stride, void* out, int out_stride, const void* gate,
                                   int gate_stride, int dtype, const void* kcache, const void* vcache,
                                   const int* block_tables, int bt_stride, const int* token_req, const int* positions,
                                   int T, int nh, int nkvh, int dk, int dv, int page_size, float scale, int window,
                                   int keep_first, int sink, const float* sinks, float softcap, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dk <= 0 || dk > kSpanMaxDim || dv <= 0 || dv > kSpanMaxDim ||
        page_size <= 0 || window < 0 || keep_first < 0)
        return IC_ERR_ARG;
    if ((long long)T * nh > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(T * nh)), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(attn_span_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride, (float*)out,
                           out_stride, (const float*)gate, gate_stride, (const float*)kcache, (const float*)vcache,
                           block_tables, bt_stride, token_req, positions, nh, nkvh, dk, dv, page_size, scale, window,
                           keep_first, sink, sinks, softcap);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(attn_span_generic_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out,
                           out_stride, (const bf16*)gate, gate_stride, (const bf16*)kcache, (const bf16*)vcache,
                           block_tables, bt_stride, token_req, positions, nh, nkvh, dk, dv, page_size, scale, window,
                           keep_first, sink, sinks, softcap);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// =============================================================================================
// Single new tokens (decoding), split over the visible keys so that few requests fill the chip.
//
// Pass 1, grid (splits, kv heads, tokens), 256 threads: the visible keys of a token are numbered
// 0 .. total-1 (the kept first keys, then the window); a block streams its share once and serves
// every query head of the kv head, GQ (1, 2 or 4) at a time.  DK/VEC lanes share a key (VEC = 16 bytes of
// elements), so a wave reads whole contiguous rows; the same lanes read the value row in pieces
// of 16 bytes (a lane takes pieces sub, sub + LPK, .. when values are wider than keys, and none
// when its piece lies beyond a narrower value row).  Every lane keeps a float32 running softmax
// (base 2) for its keys; they are merged across the lane groups, the waves and, in pass 2, the
// splits, where the sink joins the denominator and the gate is applied.
// =============================================================================================
constexpr int kSdThreads = 256;
constexpr int kSdWaves = 4;
constexpr int kSdUnroll = 4;    // keys a lane group has in flight
constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct SpanVec;
template <> struct SpanVec<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const uint4 v = load_stream16(p);
        o[0] = __uint_as_float(v.x); o[1] = __uint_as_float(v.y); o[2] = __uint_as_float(v.z); o[3] = __uint_as_float(v.w);
    }
};
template <> struct SpanVec<bf16> {
    static constexpr int N = 8;
    __device__ static void load(const bf16* p, float* o) {
        const uint4 v = load_stream16(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
};

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T, int DK, int DV, int GQ>
__global__ void __launch_bounds__(kSdThreads)
attn_span_decode_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ kcache, const T* __restrict__ vcache,
                        const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tok_list,
                        const int* __restrict__ token_req, const int* __restrict__ positions,
                        float* __restrict__ part_acc, float* __restrict__ part_ml, int nh, int nkvh, int page_size,
                        float scale, int window, int keep_first, int nsplit, int sink, const float* __restrict__ sinks,
                        float softcap, T* __restrict__ final_out, int out_stride, const T* __restrict__ gate, int gate_stride) {
    constexpr int VEC = SpanVec<T>::N;
    constexpr int LPK = DK / VEC;                  // lanes per key
    constexpr int LPV = DV / VEC;                  // 16-byte pieces of a value row
    constexpr int KPW = 64 / LPK;                  // keys per wave per step
    constexpr int NVS = (LPV + LPK - 1) / LPK;     // value pieces per lane
    static_assert(DK % VEC == 0 && DV % VEC == 0 && 64 % LPK == 0 && LPK <= 64, "sizes must split a wave evenly");

    __shared__ float sm_acc[kSdWaves][GQ][DV];
    __shared__ float sm_ml[kSdWaves][GQ][2];

    const int split = blockIdx.x, kvh = blockIdx.y, n = blockIdx.z;
    const int t = tok_list ? tok_list[n] : n;
    const int g = nh / nkvh;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const SpanRuns runs = span_runs(pos, window, keep_first);
    const int per = (runs.total + nsplit - 1) / nsplit;
    const int lo = split * per;
    int hi = lo + per;
    if (hi > runs.total) hi = runs.total;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPK, grp = lane / LPK;
    // scores in units of log 2; with a cap c the query carries scale / c and the score becomes (c log2 e) tanh(.)
    const float qscale = softcap > 0.f ? scale / softcap : scale * kLog2e;
    const float cap2 = softcap * kLog2e;

    for (int h0 = 0; h0 < g; h0 += GQ) {
        float qv[GQ][VEC], acc[GQ][NVS * VEC], m[GQ], l[GQ];
#pragma unroll
        for (int j = 0; j < GQ; ++j) {
            m[j] = -INFINITY; l[j] = 0.f;
            const int hh = (h0 + j < g) ? h0 + j : g - 1;
            SpanVec<T>::load(q + (size_t)t * q_stride + (size_t)(kvh * g + hh) * DK + sub * VEC, qv[j]);
#pragma unroll
            for (int i = 0; i < VEC; ++i) qv[j][i] *= qscale;
#pragma unroll
            for (int i = 0; i < NVS * VEC; ++i) acc[j][i] = 0.f;
        }
        // The page ids of an iteration's keys are looked up one iteration ahead: an iteration then waits for one trip to
        // memory (its rows), not for two in a row (page id, then row).
        constexpr int STEP = kSdUnroll * KPW * kSdWaves;
        int keyn[kSdUnroll], pgn[kSdUnroll];
        auto look = [&](int ib) {
#pragma unroll
            for (int u = 0; u < kSdUnroll; ++u) {
                const int idx = ib + u * KPW * kSdWaves;
                keyn[u] = span_key(runs, idx < hi ? idx : hi - 1);         // a stand-in key that is a real one
                pgn[u] = bt[keyn[u] / page_size];
            }
        };
        const int ib0 = lo + wave * KPW + grp;
        if (lo < hi) look(ib0);
        for (int ib = ib0; ib - grp - wave * KPW < hi; ib += STEP) {
            float kf[kSdUnroll][VEC], vf[kSdUnroll][NVS * VEC];
            bool ok[kSdUnroll];
#pragma unroll
            for (int u = 0; u < kSdUnroll; ++u) {
                ok[u] = ib + u * KPW * kSdWaves < hi;
                const size_t rowi = ((size_t)pgn[u] * nkvh + kvh) * page_size + (keyn[u] % page_size);
                SpanVec<T>::load(kcache + rowi * DK + sub * VEC, kf[u]);
#pragma unroll
                for (int s = 0; s < NVS; ++s) {
                    if (sub + s * LPK < LPV) SpanVec<T>::load(vcache + rowi * DV + (sub + s * LPK) * VEC, vf[u] + s * VEC);
                    else
#pragma unroll
                        for (int i = 0; i < VEC; ++i) vf[u][s * VEC + i] = 0.f;
                }
            }
            if (ib + STEP - grp - wave * KPW < hi) look(ib + STEP);
#pragma unroll
            for (int j = 0; j < GQ; ++j) {
                float s[kSdUnroll];
                float mx = m[j];
#pragma unroll
                for (int u = 0; u < kSdUnroll; ++u) {
                    float d = 0.f;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) d += qv[j][i] * kf[u][i];
                    d = group_sum<LPK>(d);                  // over the lanes that share the key (DPP steps inside a row of 16 lanes)
                    if (softcap > 0.f) d = cap2 * tanhf(d);
                    s[u] = ok[u] ? d : -INFINITY;
                    mx = fmaxf(mx, s[u]);
                }
                if (mx == -INFINITY) continue;          // this lane group has seen no key yet
                const float corr = __builtin_amdgcn_exp2f(m[j] - mx);
                float lsum = l[j] * corr;
#pragma unroll
                for (int i = 0; i < NVS * VEC; ++i) acc[j][i] *= corr;
#pragma unroll
                for (int u = 0; u < kSdUnroll; ++u) {
                    const float p = __builtin_amdgcn_exp2f(s[u] - mx);      // 0 for a stand-in key
                    lsum += p;
#pragma unroll
                    for (int i = 0; i < NVS * VEC; ++i) acc[j][i] += p * vf[u][i];
                }
                l[j] = lsum;
                m[j] = mx;
            }
        }
        // merge the lane groups of the wave (lanes with the same `sub`)
#pragma unroll
        for (int j = 0; j < GQ; ++j) {
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) {
                const float mb = __shfl_xor(m[j], o, kWave);
                const float lb = __shfl_xor(l[j], o, kWave);
                const float mn = fmaxf(m[j], mb);
                const float ca = (mn == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m[j] - mn);
                const float cb = (mn == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mb - mn);
                l[j] = l[j] * ca + lb * cb;
#pragma unroll
                for (int i = 0; i < NVS * VEC; ++i) acc[j][i] = acc[j][i] * ca + __shfl_xor(acc[j][i], o, kWave) * cb;
                m[j] = mn;
            }
        }
        __syncthreads();                                // LDS free from the previous chunk of heads
        if (grp == 0) {
#pragma unroll
            for (int j = 0; j < GQ; ++j) {
#pragma unroll
                for (int s = 0; s < NVS; ++s)
                    if (sub + s * LPK < LPV)
#pragma unroll
                        for (int i = 0; i < VEC; ++i) sm_acc[wave][j][(sub + s * LPK) * VEC + i] = acc[j][s * VEC + i];
                if (sub == 0) { sm_ml[wave][j][0] = m[j]; sm_ml[wave][j][1] = l[j]; }
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < GQ * DV; idx += kSdThreads) {
            const int j = idx / DV, d = idx - j * DV;
            if (h0 + j >= g) continue;
            float mm = -INFINITY;
            for (int w = 0; w < kSdWaves; ++w) mm = fmaxf(mm, sm_ml[w][j][0]);
            float a = 0.f, ll = 0.f;
            if (mm != -INFINITY) {
                for (int w = 0; w < kSdWaves; ++w) {
                    const float c = __builtin_amdgcn_exp2f(sm_ml[w][j][0] - mm);
                    a += sm_acc[w][j][d] * c;
                    ll += sm_ml[w][j][1] * c;
                }
            }
            const int h = kvh * g + h0 + j;
            if (final_out) {                            // a single split: this is the result, no second pass
                if (sink) {
                    const float sv = sinks ? sinks[h] * kLog2e : 0.f;
                    const float mf = fmaxf(mm, sv), c = __builtin_amdgcn_exp2f(mm - mf);
                    a *= c;
                    ll = ll * c + __builtin_amdgcn_exp2f(sv - mf);
                }
                float o = a / ll;
                if (gate) o *= sigmoid_f(to_f32(gate[(size_t)t * gate_stride + (size_t)h * DV + d]));
                final_out[(size_t)t * out_stride + (size_t)h * DV + d] = from_f32<T>(o);
                continue;
            }
            const size_t pidx = ((size_t)n * nh + h) * nsplit + split;
            part_acc[pidx * DV + d] = a;
            if (d == 0) { part_ml[pidx * 2] = mm; part_ml[pidx * 2 + 1] = ll; }      // the maximum in units of log 2
        }
    }
}

// Pass 2, grid (tokens * heads), one thread per value entry: merges the splits, lets the sink join, applies the gate.
template <typename T>
__global__ void attn_span_reduce_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                                        const int* __restrict__ tok_list, T* __restrict__ out, int out_stride,
                                        const T* __restrict__ gate, int gate_stride, int nh, int dv, int nsplit, int sink,
                                        const float* __restrict__ sinks) {
    const int n = blockIdx.x / nh, h = blockIdx.x % nh;
    const int t = tok_list ? tok_list[n] : n;
    const size_t base = ((size_t)n * nh + h) * nsplit;
    const float sv = (sink && sinks) ? sinks[h] * kLog2e : 0.f;      // in units of log 2, as the partial maxima
    float mm = sink ? sv : -INFINITY;
    for (int s = 0; s < nsplit; ++s) mm = fmaxf(mm, part_ml[(base + s) * 2]);
    float den = sink ? __builtin_amdgcn_exp2f(sv - mm) : 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float ms = part_ml[(base + s) * 2];
        if (ms != -INFINITY) den += part_ml[(base + s) * 2 + 1] * __builtin_amdgcn_exp2f(ms - mm);
    }
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float ms = part_ml[(base + s) * 2];
            if (ms != -INFINITY) a += part_acc[(base + s) * dv + d] * __builtin_amdgcn_exp2f(ms - mm);
        }
        float o = a / den;
        if (gate) o *= sigmoid_f(to_f32(gate[(size_t)t * gate_stride + (size_t)h * dv + d]));
        out[(size_t)t * out_stride + (size_t)h * dv + d] = from_f32<T>(o);
    }
}

static bool span_dim_ok(int d) { return d == 32 || d == 64 || d == 128; }

IC_EXPORT int ic_attn_span_decode_supported(int dtype, int dk, int dv) {
    return (dtype == IC_F32 || dtype == IC_BF16) && span_dim_ok(dk) && span_dim_ok(dv);
}

// How many ways to split the visible keys of n_rows single tokens (<= 32): enough blocks for the chip, at least 128 keys a split.
IC_EXPORT int ic_attn_span_decode_splits(int n_rows, int n_kv_heads, int max_keys, int compute_units) {
    if (n_rows <= 0 || n_kv_heads <= 0) return 1;
    long long blocks = (long long)n_rows * n_kv_heads;
    int want = (int)((2LL * compute_units + blocks - 1) / blocks);
    int most = (max_keys + 127) / 128;
    if (want > most) want = most;
    if (want > 32) want = 32;
    return want < 1 ? 1 : want;
}

template <typename T, int DK, int DV>
static int span_decode_launch(const void* q, int q_stride, void* out, int out_stride, const void* gate, int gate_stride,
                              const void* kcache, const void* vcache, const int* block_tables, int bt_stride,
                              const int* tok_list, const int* token_req, const int* positions, float* part_acc,
                              float* part_ml, int n_tok, int nh, int nkvh, int page_size, float scale, int window,
                              int keep_first, int sink, const float* sinks, float softcap, int nsplit, hipStream_t stream) {
    dim3 grid(nsplit, nkvh, n_tok), block(kSdThreads);
    const int g = nh / nkvh;
#define IC_SPAN_GQ(GQ)                                                                                                          \
    hipLaunchKernelGGL((attn_span_decode_kernel<T, DK, DV, GQ>), grid, block, 0, stream, (const T*)q, q_stride, (const T*)kcache, \
                       (const T*)vcache, block_tables, bt_stride, tok_list, token_req, positions, part_acc, part_ml, nh, nkvh,   \
                       page_size, scale, window, keep_first, nsplit, sink, sinks, softcap,                                       \
                       nsplit == 1 ? (T*)out : (T*)nullptr, out_stride,                                                          \
                       (const T*)gate, gate_stride)
    if (g == 1) IC_SPAN_GQ(1);                      // query heads served per walk over the keys: no more than there are
    else if (g == 2) IC_SPAN_GQ(2);
    else IC_SPAN_GQ(4);
#undef IC_SPAN_GQ
    int st = ic_launch_status();
    if (st != IC_OK || nsplit == 1) return st;
    hipLaunchKernelGGL(attn_span_reduce_kernel<T>, dim3((unsigned)(n_tok * nh)), dim3(DV < 64 ? 64 : DV), 0, stream, part_acc,
                       part_ml, tok_list, (T*)out, out_stride, (const T*)gate, gate_stride, nh, DV, nsplit, sink, sinks);
    return ic_launch_status();
}

template <typename T>
static int span_decode_dims(int dk, int dv, const void* q, int q_stride, void* out, int out_stride, const void* gate,
                            int gate_stride, const void* kcache, const void* vcache, const int* block_tables, int bt_stride,
                            const int* tok_list, const int* token_req, const int* positions, float* part_acc, float* part_ml,
                            int n_tok, int nh, int nkvh, int page_size, float scale, int window, int keep_first, int sink,
                            const float* sinks, float softcap, int nsplit, hipStream_t stream) {
#define IC_SPAN_DEC(K, V)                                                                                                   \
    if (dk == K && dv == V)                                                                                                 \
        return span_decode_launch<T, K, V>(q, q_stride, out, out_stride, gate, gate_stride, kcache, vcache, block_tables,   \
                                           bt_stride, tok_list, token_req, positions, part_acc, part_ml, n_tok, nh, nkvh,   \
                                           page_size, scale, window, keep_first, sink, sinks, softcap, nsplit, stream);
    IC_SPAN_DEC(32, 32) IC_SPAN_DEC(32, 64) IC_SPAN_DEC(32, 128)
    IC_SPAN_DEC(64, 32) IC_SPAN_DEC(64, 64) IC_SPAN_DEC(64, 128)
    IC_SPAN_DEC(128, 32) IC_SPAN_DEC(128, 64) IC_SPAN_DEC(128, 128)
#undef IC_SPAN_DEC
    return IC_ERR_UNSUPPORTED;
}

// tok_list (nullable): the rows that are single tokens, int32 [n_tok].  part_acc: float32 [n_tok, nh, nsplit, dv]; part_ml: [n_tok, nh, nsplit, 2].
IC_EXPORT int ic_attn_span_decode(const void* q, int q_stride, void* out, int out_stride, const void* gate, int gate_stride,
                                  int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride,
                                  const int* tok_list, const int* token_req, const int* positions, float* part_acc,
                                  float* part_ml, int n_tok, int nh, int nkvh, int dk, int dv, int page_size, float scale,
                                  int window, int keep_first, int sink, const float* sinks, float softcap, int nsplit,
                                  hipStream_t stream) {
    if (n_tok <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || window < 0 || keep_first < 0 || nsplit < 1 || nsplit > 32)
        return IC_ERR_ARG;
    if (nkvh > 65535 || n_tok > 65535) return IC_ERR_ARG;
    if (nsplit > 1 && (part_acc == nullptr || part_ml == nullptr)) return IC_ERR_ARG;
    if (!ic_attn_span_decode_supported(dtype, dk, dv)) return IC_ERR_UNSUPPORTED;
    if (dtype == IC_F32)
        return span_decode_dims<float>(dk, dv, q, q_stride, out, out_stride, gate, gate_stride, kcache, vcache, block_tables,
                                       bt_stride, tok_list, token_req, positions, part_acc, part_ml, n_tok, nh, nkvh, page_size,
                                       scale, window, keep_first, sink, sinks, softcap, nsplit, stream);
    return span_decode_dims<bf16>(dk, dv, q, q_stride, out, out_stride, gate, gate_stride, kcache, vcache, block_tables,
                                  bt_stride, tok_list, token_req, positions, part_acc, part_ml, n_tok, nh, nkvh, page_size,
                                  scale, window, keep_first, sink, sinks, softcap, nsplit, stream);
}

// =============================================================================================
// Prompt portions on the matrix cores (bfloat16 operands, float32 accumulation and softmax).
//
// Grid (query tiles * heads), tile-major, 256 threads.  A tile is up to 128 consecutive tokens of one
// request (int4: request row, first token row, rows, first position); wave w owns rows 32w..32w+31.
// The keys the tile may see are walked 64 at a time, first the kept first keys (when they lie before
// the window of the tile's first row), then the window up to the tile's last row.  A step's keys and
// values come through LDS as padded rows; the next step's are on their way into registers meanwhile.
// Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: a lane then holds 32
// keys of ONE query, the running softmax needs one cross-lane step, and the probabilities are
// already laid out as the B operand of O^T = V^T P^T.  The V^T operand is read with
// ds_read_b64_tr_b16, which transposes 16-bit elements across the 16 lanes of a group on the way out
// of LDS.  Operand layout (lane l, h = l/32): A[i = l%32][k = 8h..8h+7], B[k = 8h..8h+7][j = l%32],
// D[i = 8(r/4) + 4h + r%4][j = l%32] for the 16 accumulators r.
//
// A key outside the run a step walks is replaced by the nearest one inside when it is loaded (its
// page may have been given back, or not be written yet) and its score is masked.
// =============================================================================================
typedef __bf16 sp_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sp_v16f __attribute__((ext_vector_type(16)));
typedef float sp_v8f __attribute__((ext_vector_type(8)));
typedef short sp_v4s __attribute__((ext_vector_type(4)));
typedef unsigned sp_v4u __attribute__((ext_vector_type(4)));

constexpr int kSpRows = 128;      // query rows per block
constexpr int kSpKeys = 64;       // keys per step

template <int DK, int DV>
__global__ void __launch_bounds__(256, 2)
attn_span_prefill_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                         const uint16_t* __restrict__ gate, int gate_stride,
                         const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride, const int4* __restrict__ tiles,
                         int nh, int nkvh, int page_shift, float scale_log2e, int window, int keep_first, int sink,
                         const float* __restrict__ sinks, float cap_in) {
    // cap_in > 0: a raw score s becomes tanh(s * cap_in) (cap_in = scale / cap) and scale_log2e holds cap * log2 e
    constexpr int NC = DK / 16;           // 16-wide chunks of the key size
    constexpr int ND = DV / 32;           // 32-row tiles of O^T
    constexpr int PK = DK + 8;            // padded row pitches in LDS (elements)
    constexpr int PV = DV + 8;
    constexpr int KCH = DK / 8, VCH = DV / 8;              // 16-byte chunks of a row
    constexpr int NLK = kSpKeys * KCH / 256, NLV = kSpKeys * VCH / 256;     // loads per thread and step
    static_assert(DK % 32 == 0 && DV % 32 == 0, "a step's rows split evenly over the block");

    // two stages: a step is computed from one while the next step's rows are written into the other (one barrier a step)
    __shared__ __attribute__((aligned(16))) uint16_t Ks0[kSpKeys * PK];
    __shared__ __attribute__((aligned(16))) uint16_t Vs0[kSpKeys * PV];
    __shared__ __attribute__((aligned(16))) uint16_t Ks1[kSpKeys * PK];
    __shared__ __attribute__((aligned(16))) uint16_t Vs1[kSpKeys * PV];

    const int slot = (int)blockIdx.x;
    const int h = slot % nh;
    const int4 tile = tiles[slot / nh];
    const int req = tile.x, row0 = tile.y, n_rows = tile.z, pos0 = tile.w;
    const int kvh = h / (nh / nkvh);
    const int* bt = block_tables + (size_t)req * bt_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int page_size = 1 << page_shift, page_mask = page_size - 1;      // pages are a power of two here

    const int my_row = 32 * wave + lq;
    const bool row_ok = my_row < n_rows;
    const int qpos = pos0 + my_row;
    const bool wave_ok = 32 * wave < n_rows;
    const int wave_first = pos0 + 32 * wave;
    const int wave_last = pos0 + ((32 * wave + 31 < n_rows - 1) ? 32 * wave + 31 : n_rows - 1);
    const int last_key = pos0 + n_rows - 1;
    int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    int n_kept = keep_first;                           // keys 0 .. n_kept-1 are walked as a run of their own
    if (window == 0 || n_kept >= first_key) { n_kept = 0; if (keep_first >= first_key) first_key = 0; }
    const int kept_steps = (n_kept + kSpKeys - 1) / kSpKeys;
    const int win_kb0 = (first_key / kSpKeys) * kSpKeys;
    const int n_steps = kept_steps + (last_key - win_kb0) / kSpKeys + 1;

    // step -> (first key of the 64, the run's first and last key)
    auto step_of = [&](int s, int& kb, int& klo, int& khi) {
        if (s < kept_steps) { kb = s * kSpKeys; klo = 0; khi = n_kept - 1; }
        else { kb = win_kb0 + (s - kept_steps) * kSpKeys; klo = first_key; khi = last_key; }
    };

    sp_bf16x8 qf[NC];
    {
        const uint16_t* qp = q + (size_t)(row0 + (row_ok ? my_row : 0)) * q_stride + (size_t)h * DK + 8 * half;
#pragma unroll
        for (int c = 0; c < NC; ++c) qf[c] = *reinterpret_cast<const sp_bf16x8*>(qp + 16 * c);      // rows beyond the tile read row 0 and are never written
    }
    sp_v16f oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    const size_t khead = (size_t)kvh * page_size * DK, vhead = (size_t)kvh * page_size * DV;
    sp_v4u kreg0[NLK], vreg0[NLV], kreg1[NLK], vreg1[NLV];     // two steps' keys and values on their way: a load has two steps' time to arrive
    int pgk[NLK], pgv[NLV];                            // page ids of the keys this thread fetches next: looked up a step ahead of the
                                                       // fetch, so a step waits for one trip to memory, not for two in a row
    auto key_of = [&](int s, int kk) -> int {
        int kb, klo, khi;
        step_of(s, kb, klo, khi);
        int key = kb + kk;
        key = key < klo ? klo : key;
        return key > khi ? khi : key;
    };
    auto lookup = [&](int s) {
#pragma unroll
        for (int i = 0; i < NLK; ++i) pgk[i] = bt[key_of(s, (tid + i * 256) / KCH) >> page_shift];
#pragma unroll
        for (int i = 0; i < NLV; ++i) pgv[i] = bt[key_of(s, (tid + i * 256) / VCH) >> page_shift];
    };
    auto fetch = [&](int s, sp_v4u* kreg, sp_v4u* vreg) {
#pragma unroll
        for (int i = 0; i < NLK; ++i) {
            const int idx = tid + i * 256, kk = idx / KCH, c = idx - kk * KCH;
            const int key = key_of(s, kk);
            const size_t rowi = (((size_t)pgk[i] * nkvh) << page_shift) + (key & page_mask);
            kreg[i] = *reinterpret_cast<const sp_v4u*>(kcache + khead + rowi * DK + c * 8);
        }
#pragma unroll
        for (int i = 0; i < NLV; ++i) {
            const int idx = tid + i * 256, kk = idx / VCH, c = idx - kk * VCH;
            const int key = key_of(s, kk);
            const size_t rowi = (((size_t)pgv[i] * nkvh) << page_shift) + (key & page_mask);
            vreg[i] = *reinterpret_cast<const sp_v4u*>(vcache + vhead + rowi * DV + c * 8);
        }
    };
    auto stash = [&](const sp_v4u* kreg, const sp_v4u* vreg, uint16_t* Ks, uint16_t* Vs) {
#pragma unroll
        for (int i = 0; i < NLK; ++i) {
            const int idx = tid + i * 256, kk = idx / KCH, c = idx - kk * KCH;
            *reinterpret_cast<sp_v4u*>(Ks + kk * PK + c * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < NLV; ++i) {
            const int idx = tid + i * 256, kk = idx / VCH, c = idx - kk * VCH;
            *reinterpret_cast<sp_v4u*>(Vs + kk * PV + c * 8) = vreg[i];
        }
    };

    // where this lane reads V^T: rows 4 half + (l % 16) / 4 of a 16-key chunk (and 8 rows on), dims 32 dt + 16 (l / 16 % 2) + 4 (l % 4) ..+3
    const int vrow = 4 * half + ((lane & 15) >> 2);
    const int vcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    // Step s is fetched into registers three steps ahead and written to LDS one step ahead; its page ids are looked up a step before the fetch.
    lookup(0);
    fetch(0, kreg0, vreg0);
    if (n_steps > 1) { lookup(1); fetch(1, kreg1, vreg1); }
    stash(kreg0, vreg0, Ks0, Vs0);
    if (n_steps > 2) { lookup(2); fetch(2, kreg0, vreg0); }
    if (n_steps > 3) lookup(3);
    auto compute = [&](int s, const uint16_t* Ks, const uint16_t* Vs) {
        int kb, klo, khi;
        step_of(s, kb, klo, khi);
        if (!wave_ok || kb > wave_last) return;            // nothing this wave may see
        const bool kept_run = s < kept_steps;
        if (!kept_run && window > 0 && kb + kSpKeys - 1 < wave_first - window + 1 && kb >= keep_first) return;   // all before this wave's windows, none kept

        // ---- S^T = K Q^T : two tiles of 32 keys ----------------------------------
        sp_v16f sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[tt][r] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const sp_bf16x8 a = *reinterpret_cast<const sp_bf16x8*>(Ks + (32 * tt + lq) * PK + 16 * c + 8 * half);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[c], sacc[tt], 0, 0, 0);
            }
        }
        if (cap_in > 0.f) {                                // tanh(z) = 1 - 2 / (1 + e^(2z)): finite for every z
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float e = __builtin_amdgcn_exp2f(sacc[tt][r] * (2.f * kLog2e * cap_in));
                    sacc[tt][r] = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e);
                }
        }
        // ---- mask: the run's bounds, the diagonal, the window and the kept first keys --------
        const bool all_seen = kb >= klo && kb + kSpKeys - 1 <= khi && kb + kSpKeys - 1 <= wave_first
                              && (window == 0 || wave_last - kb < window || kb + kSpKeys - 1 < keep_first);
        if (!all_seen) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 32 * tt + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool seen = key >= klo && key <= khi && key <= qpos
                                      && (window == 0 || qpos - key < window || key < keep_first);
                    if (!seen) sacc[tt][r] = -INFINITY;
                }
        }
        // ---- running softmax, base 2: p = 2^(s c - m c) ---------------------------------
        float mloc = sacc[0][0];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sacc[tt][r]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
        const float m_new = fmaxf(m, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float mc = m_use * scale_log2e;
        const float corr = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m * scale_log2e - mc);
        float rs = 0.f;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sacc[tt][r], scale_log2e, -mc));
                sacc[tt][r] = p;
                rs += p;
            }
        rs += __shfl_xor(rs, 32, kWave);
        l = l * corr + rs;
        m = m_new;
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= corr;

        // ---- O^T += V^T P^T : four chunks of 16 keys ------------------------------------------
#pragma unroll
        for (int kc = 0; kc < 4; ++kc) {
            const int tt = kc >> 1, r0 = 8 * (kc & 1);
            sp_v8f pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = sacc[tt][r0 + e];
            const sp_bf16x8 b = __builtin_convertvector(pf, sp_bf16x8);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const uint16_t* vp = Vs + (16 * kc + vrow) * PV + 32 * dt + vcol;
                const sp_v4s lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((sp_v4s __attribute__((address_space(3)))*)vp);
                const sp_v4s hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((sp_v4s __attribute__((address_space(3)))*)(vp + 8 * PV));
                const sp_bf16x8 a = __builtin_bit_cast(sp_bf16x8, __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, oacc[dt], 0, 0, 0);
            }
        }
    };
    for (int s = 0; s < n_steps; s += 2) {
        __syncthreads();                                   // stage 0 holds step s; stage 1 has been read
        if (s + 1 < n_steps) stash(kreg1, vreg1, Ks1, Vs1);
        if (s + 3 < n_steps) fetch(s + 3, kreg1, vreg1);
        if (s + 4 < n_steps) lookup(s + 4);
        compute(s, Ks0, Vs0);
        if (s + 1 >= n_steps) break;
        __syncthreads();                                   // stage 1 holds step s + 1; stage 0 has been read
        if (s + 2 < n_steps) stash(kreg0, vreg0, Ks0, Vs0);
        if (s + 4 < n_steps) fetch(s + 4, kreg0, vreg0);
        if (s + 5 < n_steps) lookup(s + 5);
        compute(s + 1, Ks1, Vs1);
    }

    if (!row_ok) return;
    if (sink) {                                            // exp(sink - m) joins the denominator
        const float sv = sinks ? sinks[h] * kLog2e : 0.f;
        const float mc = (m == -INFINITY) ? sv : m * scale_log2e;
        const float mf = fmaxf(mc, sv);
        const float corr = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - mf);
        l = l * corr + __builtin_amdgcn_exp2f(sv - mf);
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= corr;
    }
    const float inv = 1.0f / l;
    uint16_t* op = out + (size_t)(row0 + my_row) * out_stride + (size_t)h * DV;
    const uint16_t* gp = gate ? gate + (size_t)(row0 + my_row) * gate_stride + (size_t)h * DV : nullptr;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = 32 * dt + 8 * r4 + 4 * half;     // dims d .. d+3 are accumulators 4 r4 .. 4 r4 + 3
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = oacc[dt][4 * r4 + e] * inv;
            if (gp) {
                const uint2 gv = *reinterpret_cast<const uint2*>(gp + d);
                o[0] *= sigmoid_f(__uint_as_float(gv.x << 16)); o[1] *= sigmoid_f(__uint_as_float(gv.x & 0xffff0000u));
                o[2] *= sigmoid_f(__uint_as_float(gv.y << 16)); o[3] *= sigmoid_f(__uint_as_float(gv.y & 0xffff0000u));
            }
            uint2 w;
            w.x = (uint32_t)f32_to_bf16_bits(o[0]) | ((uint32_t)f32_to_bf16_bits(o[1]) << 16);
            w.y = (uint32_t)f32_to_bf16_bits(o[2]) | ((uint32_t)f32_to_bf16_bits(o[3]) << 16);
            *reinterpret_cast<uint2*>(op + d) = w;
        }
}

IC_EXPORT int ic_attn_span_prefill_supported(int dtype, int dk, int dv) {
    return dtype == IC_BF16 && span_dim_ok(dk) && span_dim_ok(dv);
}

// tiles: int32 [n_tiles, 4] = (request row, first token row, rows <= 128, first position).  Pages of a power of two.  Strides in elements; q rows, out rows and
// gate rows must start on 16-, 8- and 8-byte boundaries.  scale > 0.
IC_EXPORT int ic_attn_span_prefill(const void* q, int q_stride, void* out, int out_stride, const void* gate, int gate_stride,
                                   int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride,
                                   const int* tiles, int n_tiles, int nh, int nkvh, int dk, int dv, int page_size, float scale,
                                   int window, int keep_first, int sink, const float* sinks, float softcap, hipStream_t stream) {
    if (n_tiles <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || window < 0 || keep_first < 0 || !(scale > 0.f)) return IC_ERR_ARG;
    if (!ic_attn_span_prefill_supported(dtype, dk, dv) || (page_size & (page_size - 1))) return IC_ERR_UNSUPPORTED;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    if ((q_stride & 7) || (out_stride & 3) || (gate && (gate_stride & 3)) || ((uintptr_t)q & 15) || ((uintptr_t)out & 7) ||
        ((uintptr_t)gate & 7) || ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15))
        return IC_ERR_ARG;
    if ((long long)n_tiles * nh > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(n_tiles * nh)), block(256);
    const float c = softcap > 0.f ? softcap * kLog2e : scale * kLog2e;
    const float cap_in = softcap > 0.f ? scale / softcap : 0.f;
#define IC_SPAN_PRE(K, V)                                                                                                     \
    if (dk == K && dv == V) {                                                                                                 \
        hipLaunchKernelGGL((attn_span_prefill_kernel<K, V>), grid, block, 0, stream, (const uint16_t*)q, q_stride,            \
                           (uint16_t*)out, out_stride, (const uint16_t*)gate, gate_stride, (const uint16_t*)kcache,           \
                           (const uint16_t*)vcache, block_tables, bt_stride, (const int4*)tiles, nh, nkvh, page_shift, c,      \
                           window, keep_first, sink, sinks, cap_in);                                                          \
        return ic_launch_status();                                                                                            \
    }
    IC_SPAN_PRE(32, 32) IC_SPAN_PRE(32, 64) IC_SPAN_PRE(32, 128)
    IC_SPAN_PRE(64, 32) IC_SPAN_PRE(64, 64) IC_SPAN_PRE(64, 128)
    IC_SPAN_PRE(128, 32) IC_SPAN_PRE(128, 64) IC_SPAN_PRE(128, 128)
#undef IC_SPAN_PRE
    return IC_ERR_UNSUPPORTED;
}
