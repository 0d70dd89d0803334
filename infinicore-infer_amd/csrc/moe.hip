// A feed-forward of routed experts.  A token's router logits z[E] (float32) give scores s = sigmoid(z) (or, for
// another design, a softmax over the experts); the `top` experts with the largest scores are chosen (the lower
// index wins a tie), their weights are the scores, optionally renormalised over the chosen ones.  A (token,
// choice) pair is numbered token * top + choice.
//
//   * ic_moe_route: scores, choice and weights of every token,
//   * ic_moe_sort: the pairs in expert order (stable): offsets[E + 1], order[n] (sorted place -> pair),
//     place[n] (pair -> sorted place),
//   * ic_moe_gather: the sorted pairs' input rows, each multiplied by its weight (a design whose weight is on the
//     expert's INPUT) or as they are,
//   * ic_moe_expert_product: for few rows, the product of every sorted row with its own expert's matrix, the
//     weights streamed once per expert and chunk of rows; with the gated unit silu(gate) * up in its epilogue,
//   * ic_moe_combine: a token's result is the sum of its pairs' rows (times the weight when it is on the
//     OUTPUT), plus an optional row of a shared expert.
// For many rows the products between gather and combine are library products over each expert's run of rows.
#include "common.h"

constexpr int kMoeMaxExperts = 1024;
constexpr int kMoeMaxTop = 16;

// ---------------------------------------------------------------------------------------------
// One thread a token.  mode 0: s = sigmoid(z); mode 1: s = softmax(z) over all experts.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ z, int z_stride, int T, int E, int top, int mode, int renorm,
                 int* __restrict__ ids, float* __restrict__ weights) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    const float* zr = z + (size_t)t * z_stride;
    float zmax = -INFINITY, den = 1.f;
    if (mode == 1) {
        for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, zr[e]);
        den = 0.f;
        for (int e = 0; e < E; ++e) den += expf(zr[e] - zmax);
    }
    int chosen[kMoeMaxTop];
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bz = -INFINITY;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
            if (!taken && (best < 0 || zr[e] > bz)) { best = e; bz = zr[e]; }     // both score functions grow with z
        }
        chosen[k] = best;
        const float s = mode == 1 ? expf(bz - zmax) / den : 1.0f / (1.0f + expf(-bz));
        ids[(size_t)t * top + k] = best;
        weights[(size_t)t * top + k] = s;
        total += s;
    }
    if (renorm)
        for (int k = 0; k < top; ++k) weights[(size_t)t * top + k] /= total;
}

IC_EXPORT int ic_moe_route(const float* z, int z_stride, int T, int E, int top, int mode, int renorm, int* ids,
                           float* weights, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (E <= 0 || E > kMoeMaxExperts || top <= 0 || top > kMoeMaxTop || top > E || z_stride < E || (mode != 0 && mode != 1))
        return IC_ERR_ARG;
    hipLaunchKernelGGL(moe_route_kernel, dim3((T + 255) / 256), dim3(256), 0, stream, z, z_stride, T, E, top, mode, renorm,
                       ids, weights);
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Block e takes the pairs in 256 contiguous runs, a thread a run: it counts its run's pairs of experts below e and of e
// itself, the counts meet in LDS (the pairs below e are the expert's offset, the pairs of e in the runs before a thread's
// are where its own begin), and a second walk over the run hands e's pairs their places in order of appearance.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
moe_sort_kernel(const int* __restrict__ ids, int n, int E, int* __restrict__ offsets, int* __restrict__ order,
                int* __restrict__ place) {
    __shared__ int below_s[256], mine_s[256];
    const int e = blockIdx.x, tid = threadIdx.x;
    const int run = (n + 255) / 256;
    const int lo = min(n, tid * run), hi = min(n, lo + run);
    int below = 0, mine = 0;
    for (int i = lo; i < hi; ++i) {
        const int id = ids[i];
        below += id < e;
        mine += id == e;
    }
    below_s[tid] = below;
    mine_s[tid] = mine;
    __syncthreads();
    int total_below = 0, before = 0, total_mine = 0;
    for (int j = 0; j < 256; ++j) {
        total_below += below_s[j];
        before += j < tid ? mine_s[j] : 0;
        total_mine += mine_s[j];
    }
    if (tid == 0) {
        offsets[e] = total_below;
        if (e == E - 1) offsets[E] = total_below + total_mine;
    }
    int at = total_below + before;
    for (int i = lo; i < hi; ++i)
        if (ids[i] == e) {
            order[at] = i;
            place[i] = at;
            ++at;
        }
}

IC_EXPORT int ic_moe_sort(const int* ids, int n, int E, int* offsets, int* order, int* place, hipStream_t stream) {
    if (E <= 0 || E > kMoeMaxExperts || n < 0) return IC_ERR_ARG;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(E), dim3(256), 0, stream, ids, n, E, offsets, order, place);
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[s] = h[order[s] / top] * (weights[order[s]] or 1), rounded to the rows' dtype.  grid (n).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
moe_gather_kernel(const T* __restrict__ h, int h_stride, const int* __restrict__ order, const float* __restrict__ weights,
                  int top, int d, T* __restrict__ out) {
    const int s = blockIdx.x, pair = order[s];
    const float w = weights ? weights[pair] : 1.f;
    const T* src = h + (size_t)(pair / top) * h_stride;
    T* dst = out + (size_t)s * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = from_f32<T>(to_f32(src[i]) * w);
}

IC_EXPORT int ic_moe_gather(const void* h, int h_stride, int dtype, const int* order, const float* weights, int n, int top,
                            int d, void* out, hipStream_t stream) {
    if (n <= 0) return IC_OK;
    if (top <= 0 || d <= 0) return IC_ERR_ARG;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(moe_gather_kernel<float>, dim3(n), dim3(256), 0, stream, (const float*)h, h_stride, order, weights,
                           top, d, (float*)out);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(moe_gather_kernel<bf16>, dim3(n), dim3(256), 0, stream, (const bf16*)h, h_stride, order, weights, top,
                           d, (bf16*)out);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Few rows: out[s, c] = a[s, :] . W_e[c, :] for the sorted rows s of expert e = blockIdx.y (GLU: out[s, c] =
// silu(a . W_e[c]) * (a . W_e[N + c]), W_e holding the gate rows, then the up rows).  Rows are taken RC at a time
// into LDS (float32; RC = 8, or fewer where 8 rows of K floats exceed 64 KB); a wave owns columns blockIdx.x * cols_per_block + wave, + waves, ..; its lanes stride
// over K in 16-byte pieces of the weight row, so a weight row is read once per chunk of rows.
// ---------------------------------------------------------------------------------------------

template <typename T> struct MoeVec;
template <> struct MoeVec<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct MoeVec<bf16> {
    static constexpr int N = 8;
    __device__ static void load(const bf16* p, float* o) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
};

template <typename T, bool GLU, bool VEC, int kMoeRC>
__global__ void __launch_bounds__(256)
moe_expert_product_kernel(const T* __restrict__ a, int a_stride, const T* __restrict__ w, long long w_expert_stride,
                          const int* __restrict__ offsets, T* __restrict__ out, int out_stride, int N, int K,
                          int cols_per_block) {
    extern __shared__ float rows_lds[];            // [kMoeRC][K]
    const int e = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int r0 = offsets[e], r1 = offsets[e + 1];
    if (r0 >= r1) return;
    const T* we = w + (size_t)e * w_expert_stride;
    const int c0 = blockIdx.x * cols_per_block;
    const int c1 = min(N, c0 + cols_per_block);
    for (int rb = r0; rb < r1; rb += kMoeRC) {
        const int nr = min(kMoeRC, r1 - rb);
        __syncthreads();
        for (int i = threadIdx.x; i < kMoeRC * K; i += blockDim.x) {
            const int r = i / K, k = i - r * K;
            rows_lds[i] = r < nr ? to_f32(a[(size_t)(rb + r) * a_stride + k]) : 0.f;
        }
        __syncthreads();
        for (int c = c0 + wave; c < c1; c += waves) {
            float acc[kMoeRC], acc2[kMoeRC];
#pragma unroll
            for (int r = 0; r < kMoeRC; ++r) { acc[r] = 0.f; acc2[r] = 0.f; }
            const T* w1 = we + (size_t)c * K;
            const T* w2 = we + (size_t)(N + c) * K;
            if (VEC) {
                constexpr int V = MoeVec<T>::N;
                for (int k = lane * V; k < K; k += 64 * V) {
                    float x[V], y[V];
                    MoeVec<T>::load(w1 + k, x);
                    if (GLU) MoeVec<T>::load(w2 + k, y);
#pragma unroll
                    for (int r = 0; r < kMoeRC; ++r) {
                        const float* ar = rows_lds + r * K + k;
#pragma unroll
                        for (int j = 0; j < V; ++j) {
                            acc[r] += ar[j] * x[j];
                            if (GLU) acc2[r] += ar[j] * y[j];
                        }
                    }
                }
            } else {
                for (int k = lane; k < K; k += 64) {
                    const float x = to_f32(w1[k]), y = GLU ? to_f32(w2[k]) : 0.f;
#pragma unroll
                    for (int r = 0; r < kMoeRC; ++r) {
                        acc[r] += rows_lds[r * K + k] * x;
                        if (GLU) acc2[r] += rows_lds[r * K + k] * y;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < kMoeRC; ++r) {
                acc[r] = wave_sum(acc[r]);
                if (GLU) acc2[r] = wave_sum(acc2[r]);
            }
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < kMoeRC; ++r) {
                    if (r < nr) {
                        float v = acc[r];
                        if (GLU) {
                            // the gate and up products are rounded to the rows' dtype first, as a product kernel followed
                            // by the gated unit's kernel would leave them
                            const float g = to_f32(from_f32<T>(acc[r])), u = to_f32(from_f32<T>(acc2[r]));
                            v = u * (g / (1.0f + expf(-g)));
                        }
                        out[(size_t)(rb + r) * out_stride + c] = from_f32<T>(v);
                    }
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// The same product on the matrix cores (bfloat16, N a multiple of 16, K of 32).  Grid (N / 16, experts), four waves:
// a block owns 16 output columns of one expert (with GLU: 16 gate rows and the matching 16 up rows); its waves take
// the k-steps of 32 in turn, so that together they read 256 consecutive bytes of every weight row at a time.  Lane
// (r = l % 16, kq = l / 16) loads 16 bytes W[c0 + r][k0 + 8 kq ..] and the matching 16 bytes of token row r of the
// chunk, and feeds them to one v_mfma_f32_16x16x32_bf16 as A and B operands (D[i = 4 (l / 16) + e][j = l % 16]:
// column c0 + i of token row j).  The waves' sums meet in LDS.  An expert's rows are taken 32 at a time (two tiles of 16 per
// pass over the weights; the second only where the expert has that many rows); the token
// rows are few and come out of the caches, the weights are streamed with loads the caches do not keep.
// ---------------------------------------------------------------------------------------------
typedef __bf16 moe_v8b __attribute__((ext_vector_type(8)));
typedef float moe_v4f __attribute__((ext_vector_type(4)));

template <bool GLU>
__global__ void __launch_bounds__(256)
moe_expert_product_mfma_kernel(const uint16_t* __restrict__ a, int a_stride, const uint16_t* __restrict__ w,
                               long long w_expert_stride, const int* __restrict__ offsets, uint16_t* __restrict__ out,
                               int out_stride, int N, int K) {
    constexpr int NW = GLU ? 2 : 1;                       // weight rows per column: gate and up, or one
    constexpr int MT = 2;                                 // tiles of 16 token rows per pass over the weights
    __shared__ float sums[4][MT][NW][16][17];
    const int e = blockIdx.y, c0 = blockIdx.x * 16;
    const int r0 = offsets[e], r1 = offsets[e + 1];
    if (r0 >= r1) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    const uint16_t* w1 = w + (size_t)e * w_expert_stride + (size_t)(c0 + r) * K + 8 * kq;
    const uint16_t* w2 = w1 + (size_t)N * K;
    const int steps = K / 32;
    for (int rb = r0; rb < r1; rb += 16 * MT) {
        const bool two = rb + 16 < r1;                    // the same for the whole block
        const uint16_t* ar[MT];
        bool row_ok[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = rb + 16 * m + r;
            row_ok[m] = row < r1;
            ar[m] = a + (size_t)(row_ok[m] ? row : r1 - 1) * a_stride + 8 * kq;
        }
        moe_v4f acc[MT][NW];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NW; ++n) acc[m][n] = moe_v4f{0.f, 0.f, 0.f, 0.f};
        for (int s = wave; s < steps; s += 4) {
            uint4 wv[NW];
            wv[0] = load_stream16(w1 + 32 * s);
            if (GLU) wv[NW - 1] = load_stream16(w2 + 32 * s);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m == 0 || two) {
                    uint4 xa = *reinterpret_cast<const uint4*>(ar[m] + 32 * s);
                    if (!row_ok[m]) xa = uint4{0u, 0u, 0u, 0u};
#pragma unroll
                    for (int n = 0; n < NW; ++n)
                        acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_v8b, wv[n]), __builtin_bit_cast(moe_v8b, xa),
                                                                           acc[m][n], 0, 0, 0);
                }
            }
        }
        __syncthreads();                                   // the pass before has been summed
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NW; ++n)
#pragma unroll
                for (int i = 0; i < 4; ++i) sums[wave][m][n][4 * kq + i][r] = acc[m][n][i];
        __syncthreads();
        const int col = tid >> 4, j = tid & 15;            // 256 threads: 16 columns x 16 token rows
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = rb + 16 * m + j;
            if (row < r1) {
                float v = sums[0][m][0][col][j] + sums[1][m][0][col][j] + sums[2][m][0][col][j] + sums[3][m][0][col][j];
                if (GLU) {
                    const float u2 = sums[0][m][NW - 1][col][j] + sums[1][m][NW - 1][col][j] + sums[2][m][NW - 1][col][j] + sums[3][m][NW - 1][col][j];
                    // gate and up are rounded to bfloat16 first, as a product kernel followed by the gated unit's kernel leaves them
                    const float g = bf16_bits_to_f32(f32_to_bf16_bits(v)), u = bf16_bits_to_f32(f32_to_bf16_bits(u2));
                    v = u * (g / (1.0f + expf(-g)));
                }
                out[(size_t)row * out_stride + c0 + col] = f32_to_bf16_bits(v);
            }
        }
    }
}

IC_EXPORT int ic_moe_expert_product(const void* a, int a_stride, const void* w, long long w_expert_stride, int dtype,
                                    const int* offsets, void* out, int out_stride, int E, int N, int K, int glu,
                                    int compute_units, hipStream_t stream) {
    if (E <= 0 || E > 65535 || N <= 0 || K <= 0) return IC_ERR_ARG;
    if (dtype == IC_BF16 && N % 16 == 0 && K % 32 == 0 && (w_expert_stride % 8) == 0 && (a_stride % 8) == 0 &&
        ((uintptr_t)w % 16) == 0 && ((uintptr_t)a % 16) == 0 && N / 16 <= 0x7fffffff / 2) {
        dim3 grid((unsigned)(N / 16), (unsigned)E), block(256);
        if (glu)
            hipLaunchKernelGGL(moe_expert_product_mfma_kernel<true>, grid, block, 0, stream, (const uint16_t*)a, a_stride,
                               (const uint16_t*)w, w_expert_stride, offsets, (uint16_t*)out, out_stride, N, K);
        else
            hipLaunchKernelGGL(moe_expert_product_mfma_kernel<false>, grid, block, 0, stream, (const uint16_t*)a, a_stride,
                               (const uint16_t*)w, w_expert_stride, offsets, (uint16_t*)out, out_stride, N, K);
        return ic_launch_status();
    }
    int rc = 8;
    while (rc > 1 && (size_t)rc * K * sizeof(float) > 64 * 1024) rc >>= 1;
    const size_t lds = (size_t)rc * K * sizeof(float);
    if (lds > 64 * 1024) return IC_ERR_TOO_LARGE;
    // blocks per expert so that all experts' blocks fill the chip about twice
    int per = (2 * (compute_units > 0 ? compute_units : 256) + E - 1) / E;
    int cols = (N + per - 1) / per;
    if (cols < 4) cols = 4;
    const int bx = (N + cols - 1) / cols;
    const bool vec16 = dtype == IC_F32 ? (K % 4 == 0 && (w_expert_stride % 4) == 0 && ((uintptr_t)w % 16) == 0)
                                       : (K % 8 == 0 && (w_expert_stride % 8) == 0 && ((uintptr_t)w % 16) == 0);
    dim3 grid((unsigned)bx, (unsigned)E), block(256);
#define IC_MOE_LAUNCH(TT, G, V, R)                                                                                       \
    hipLaunchKernelGGL((moe_expert_product_kernel<TT, G, V, R>), grid, block, lds, stream, (const TT*)a, a_stride,        \
                       (const TT*)w, w_expert_stride, offsets, (TT*)out, out_stride, N, K, cols)
#define IC_MOE_RC(TT, G, V)                                                                                              \
    do {                                                                                                                 \
        if (rc == 8) IC_MOE_LAUNCH(TT, G, V, 8);                                                                         \
        else if (rc == 4) IC_MOE_LAUNCH(TT, G, V, 4);                                                                    \
        else if (rc == 2) IC_MOE_LAUNCH(TT, G, V, 2);                                                                    \
        else IC_MOE_LAUNCH(TT, G, V, 1);                                                                                 \
    } while (0)
    if (dtype == IC_F32) {
        if (glu) { if (vec16) IC_MOE_RC(float, true, true); else IC_MOE_RC(float, true, false); }
        else { if (vec16) IC_MOE_RC(float, false, true); else IC_MOE_RC(float, false, false); }
    } else if (dtype == IC_BF16) {
        if (glu) { if (vec16) IC_MOE_RC(bf16, true, true); else IC_MOE_RC(bf16, true, false); }
        else { if (vec16) IC_MOE_RC(bf16, false, true); else IC_MOE_RC(bf16, false, false); }
    } else {
        return IC_ERR_UNSUPPORTED;
    }
#undef IC_MOE_RC
#undef IC_MOE_LAUNCH
    return ic_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[t] = sum_k y[place[t * top + k]] * (weights[t * top + k] or 1) + shared[t].  grid (T, blocks over the columns), a
// thread 16 bytes of columns (one column where rows are not made of whole 16-byte pieces): the pairs' places are read
// once, then the top + 1 loads of a piece are in flight together.
// ---------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ void moe_store(T* p, const float* o);
template <> __device__ __forceinline__ void moe_store<float>(float* p, const float* o) {
    *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
template <> __device__ __forceinline__ void moe_store<bf16>(bf16* p, const float* o) {
    uint4 v;
    v.x = (uint32_t)f32_to_bf16_bits(o[0]) | ((uint32_t)f32_to_bf16_bits(o[1]) << 16);
    v.y = (uint32_t)f32_to_bf16_bits(o[2]) | ((uint32_t)f32_to_bf16_bits(o[3]) << 16);
    v.z = (uint32_t)f32_to_bf16_bits(o[4]) | ((uint32_t)f32_to_bf16_bits(o[5]) << 16);
    v.w = (uint32_t)f32_to_bf16_bits(o[6]) | ((uint32_t)f32_to_bf16_bits(o[7]) << 16);
    *reinterpret_cast<uint4*>(p) = v;
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const T* __restrict__ y, int y_stride, const int* __restrict__ place, const float* __restrict__ weights,
                   const T* __restrict__ shared, int shared_stride, int top, int d, T* __restrict__ out, int out_stride) {
    constexpr int V = VEC ? MoeVec<T>::N : 1;
    const int t = blockIdx.x, i = (blockIdx.y * 256 + threadIdx.x) * V;
    if (i >= d) return;
    float s[V];
    if (VEC) {
        if (shared) MoeVec<T>::load(shared + (size_t)t * shared_stride + i, s);
        else
#pragma unroll
            for (int j = 0; j < V; ++j) s[j] = 0.f;
    } else {
        s[0] = shared ? to_f32(shared[(size_t)t * shared_stride + i]) : 0.f;
    }
    for (int k = 0; k < top; ++k) {
        const int pair = t * top + k;
        const float w = weights ? weights[pair] : 1.f;
        const T* row = y + (size_t)place[pair] * y_stride + i;
        if (VEC) {
            float v[V];
            MoeVec<T>::load(row, v);
#pragma unroll
            for (int j = 0; j < V; ++j) s[j] += v[j] * w;
        } else {
            s[0] += to_f32(row[0]) * w;
        }
    }
    if (VEC) moe_store<T>(out + (size_t)t * out_stride + i, s);
    else out[(size_t)t * out_stride + i] = from_f32<T>(s[0]);
}

IC_EXPORT int ic_moe_combine(const void* y, int y_stride, int dtype, const int* place, const float* weights,
                             const void* shared, int shared_stride, int T, int top, int d, void* out, int out_stride,
                             hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (top <= 0 || top > kMoeMaxTop || d <= 0 || (dtype != IC_F32 && dtype != IC_BF16)) return IC_ERR_ARG;
    const int V = dtype == IC_F32 ? 4 : 8;
    const bool vec = d % V == 0 && y_stride % V == 0 && out_stride % V == 0 && (!shared || shared_stride % V == 0) &&
                     ((uintptr_t)y % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)shared % 16) == 0;
    const int per = 256 * (vec ? V : 1);
    dim3 grid((unsigned)T, (unsigned)((d + per - 1) / per)), block(256);
    if (grid.y > 65535) return IC_ERR_ARG;
#define IC_MC(TT, VV)                                                                                                   \
    hipLaunchKernelGGL((moe_combine_kernel<TT, VV>), grid, block, 0, stream, (const TT*)y, y_stride, place, weights,      \
                       (const TT*)shared, shared_stride, top, d, (TT*)out, out_stride)
    if (dtype == IC_F32) { if (vec) IC_MC(float, true); else IC_MC(float, false); }
    else { if (vec) IC_MC(bf16, true); else IC_MC(bf16, false); }
#undef IC_MC
    return ic_launch_status();
}
