// Register-tiled kernels for the dense signature (every word up to depth N over D letters).
//
// Work decomposition.  The update S <- S (x) exp(dx) of a word only reads the word's own prefixes, so
// the sub-trie below any prefix u evolves on its own once the chain S(u_1), S(u_1 u_2), .. S(u) is
// known.  A lane owns one prefix u of length P: it keeps the P chain values (recomputed redundantly by
// every lane that shares them) and the whole sub-trie below u (levels P+1..N, sum_k D^k values) in
// registers.  All letters below u are compile-time constants, so every state access is a fixed
// register and the increment of the step is the same for all lanes of the unit: there is no
// inter-lane traffic and no barrier inside the time loop.  One "unit" = one (path, window); its D^P
// lanes fill ceil(D^P / 64) wavefronts of one workgroup, which stages a tile of increments in LDS.
//
// Horner form of one step for target level m (every node is one FMA):
//     tmp_j[w a] = S_j[w a] + (tmp_{j-1}[w] / (m - j + 1)) * dx[a],   j = 1..m-1,   tmp_0 = 1
//     S_m[w a]  += tmp_{m-1}[w] * dx[a]
// evaluated depth-first below the lane's prefix, targets descending so lower levels are still old.
//
// Backward.  With A_t = S_{0,t} and H_t = dL/dS_{0,t}: a reverse sweep rolls A back with exp(-dx_t)
// (levels < N only: the top level of A is never read), back-propagates through the Horner chains of the
// step (which yields H_{t-1} and dL/d(dx_t)), and keeps the top level of H equal to the upstream
// gradient.  Adjoint values of the shared chain nodes stay lane-private partial sums (everything they
// feed is linear in them), so the only cross-lane operation is the final sum of D numbers per step.
#include <type_traits>

#include "dense.hpp"

namespace psig {

namespace {

// compile-time loop: f(std::integral_constant<int, I>) for I in [Begin, End)
template <int Begin, int End, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (Begin < End) {
        f(std::integral_constant<int, Begin>{});
        static_for<Begin + 1, End>(f);
    }
}

constexpr int ipow(int b, int e) { return e <= 0 ? 1 : b * ipow(b, e - 1); }
// number of sub-trie values in levels 1..k below a prefix
constexpr int trie_size(int D, int k) { return k <= 0 ? 0 : ipow(D, k) + trie_size(D, k - 1); }

template <typename T>
__device__ __forceinline__ constexpr T rcp(int k) { return T(1) / T(k); }

template <typename T>
__device__ __forceinline__ T fmad(T a, T b, T c);
template <>
__device__ __forceinline__ float fmad<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <>
__device__ __forceinline__ double fmad<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }

// ---------------------------------------------------------------------------------------------
// one Chen step on a lane's state: chain a[1..P] and sub-trie levels P+1..TOP (TOP <= N)
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int P, int M, int J, bool NEG>
struct StepDescend {
    // children (level J > P) of a node whose scaled value is ps; idx0 = index of the first child within level J
    template <int SUB>
    static __device__ __forceinline__ void run(T ps, int idx0, T (&sub)[SUB], const T (&dx)[D]) {
        constexpr int off = trie_size(D, J - P - 1);
#pragma unroll
        for (int a = 0; a < D; ++a) {
            const T inc = NEG ? -dx[a] : dx[a];
            if constexpr (J == M) {
                sub[off + idx0 + a] = fmad<T>(ps, inc, sub[off + idx0 + a]);
            } else {
                const T tmp = fmad<T>(ps, inc, sub[off + idx0 + a]);
                StepDescend<T, D, P, M, J + 1, NEG>::template run<SUB>(tmp * rcp<T>(M - J), (idx0 + a) * D, sub, dx);
            }
        }
    }
};

template <typename T, int D, int P, int M, bool NEG>
struct StepTargets {
    template <int SUB>
    static __device__ __forceinline__ void run(T (&a)[P + 1], T (&sub)[SUB], const T (&dx)[D], const T (&dxp)[P]) {
        T ps = rcp<T>(M);
        constexpr int JP = (M - 1 < P) ? (M - 1) : P;
#pragma unroll
        for (int j = 1; j <= JP; ++j) {
            const T tmp = fmad<T>(ps, NEG ? -dxp[j - 1] : dxp[j - 1], a[j]);
            ps = tmp * rcp<T>(M - j);
        }
        if constexpr (M <= P) {
            a[M] = fmad<T>(ps, NEG ? -dxp[M - 1] : dxp[M - 1], a[M]);
        } else {
            StepDescend<T, D, P, M, P + 1, NEG>::template run<SUB>(ps, 0, sub, dx);
        }
        if constexpr (M > 1) StepTargets<T, D, P, M - 1, NEG>::template run<SUB>(a, sub, dx, dxp);
    }
};

// ---------------------------------------------------------------------------------------------
// adjoint of one Chen step
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int P, int M, int J>
struct AdjDescend {
    // returns the adjoint of the scaled parent value ps
    template <int ASUB, int HSUB>
    static __device__ __forceinline__ T run(T ps, int idx0, const T (&asub)[ASUB], T (&hsub)[HSUB], const T (&dx)[D],
                                            T (&gdx)[D]) {
        constexpr int off = trie_size(D, J - P - 1);
        T gps = T(0);
#pragma unroll
        for (int a = 0; a < D; ++a) {
            T g;
            if constexpr (J == M) {
                g = hsub[off + idx0 + a];
            } else {
                const T tmp = fmad<T>(ps, dx[a], asub[off + idx0 + a]);
                g = AdjDescend<T, D, P, M, J + 1>::template run<ASUB, HSUB>(tmp * rcp<T>(M - J), (idx0 + a) * D, asub,
                                                                            hsub, dx, gdx) *
                    rcp<T>(M - J);
                hsub[off + idx0 + a] += g;
            }
            gdx[a] = fmad<T>(g, ps, gdx[a]);
            gps = fmad<T>(g, dx[a], gps);
        }
        return gps;
    }
};

template <typename T, int D, int N, int P, int M>
struct AdjTargets {
    // targets ascending: the seed of target M (adjoint of level M) is only changed by targets above M
    template <int ASUB, int HSUB>
    static __device__ __forceinline__ void run(const T (&a)[P + 1], const T (&asub)[ASUB], T (&hc)[P + 1],
                                               T (&hsub)[HSUB], const T (&dx)[D], const T (&dxp)[P], T (&gdx)[D],
                                               T (&gpre)[P]) {
        constexpr int JP = (M - 1 < P) ? (M - 1) : P;
        T ps[P + 2];
        ps[1] = rcp<T>(M);
#pragma unroll
        for (int j = 1; j <= JP; ++j) {
            const T tmp = fmad<T>(ps[j], dxp[j - 1], a[j]);
            ps[j + 1] = tmp * rcp<T>(M - j);
        }
        T g;
        constexpr int JS = (M <= P) ? M : P;  // chain level where the walk back starts
        if constexpr (M <= P) {
            g = hc[M];
        } else {
            g = AdjDescend<T, D, P, M, P + 1>::template run<ASUB, HSUB>(ps[P + 1], 0, asub, hsub, dx, gdx) *
                rcp<T>(M - P);
            hc[P] += g;
        }
#pragma unroll
        for (int j = JS; j >= 1; --j) {
            gpre[j - 1] = fmad<T>(g, ps[j], gpre[j - 1]);
            if (j > 1) {
                g = g * dxp[j - 1] * rcp<T>(M - j + 1);
                hc[j - 1] += g;
            }
        }
        if constexpr (M < N) AdjTargets<T, D, N, P, M + 1>::template run<ASUB, HSUB>(a, asub, hc, hsub, dx, dxp, gdx, gpre);
    }
};

// ---------------------------------------------------------------------------------------------
// wave-wide sum; the total is valid in lane 63
// ---------------------------------------------------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add_c(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}

__device__ __forceinline__ float wave_total(float v) {
    v = dpp_add_c<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add_c<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add_c<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add_c<0x140, 0xF>(v);  // row_mirror: every lane now holds the sum of its row of 16
    v = dpp_add_c<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add_c<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ double wave_total(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

struct Span {
    int64_t start, steps;
};

__device__ __forceinline__ Span unit_span(const SigShape &shape, int64_t w) {
    int64_t start = 0, end = shape.L;
    if (shape.windows) {
        start = shape.windows[2 * w];
        end = shape.windows[2 * w + 1];
        start = start < 0 ? 0 : (start > shape.L ? shape.L : start);
        end = end < 0 ? 0 : (end > shape.L ? shape.L : end);
    }
    int64_t steps = end - start - 1;
    return {start, steps < 0 ? 0 : steps};
}

constexpr int kTile = 64;  // increments staged in LDS at a time

template <int D, int N, int P>
struct Geometry {
    static constexpr int kLanes = ipow(D, P);
    static constexpr int kWaves = (kLanes + kWave - 1) / kWave;
    static constexpr int kBlock = kWaves * kWave;
    static constexpr int kFwdSub = trie_size(D, N - P);      // sub-trie levels P+1..N
    static constexpr int kASub = trie_size(D, N - 1 - P);    // levels P+1..N-1
    static __host__ __device__ constexpr int64_t level_off(int k) {  // first column of level k in the dense layout
        int64_t o = 0, w = 1;
        for (int i = 1; i < k; ++i) {
            w *= D;
            o += w;
        }
        return o;
    }
    static constexpr int64_t kSigSize = level_off(N + 1);
};

// letters of the lane's prefix, most significant first
template <int D, int P>
__device__ __forceinline__ void prefix_letters(int pu, int (&u)[P]) {
#pragma unroll
    for (int j = P - 1; j >= 0; --j) {
        u[j] = pu % D;
        pu /= D;
    }
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int N, int P>
__global__ void __launch_bounds__((Geometry<D, N, P>::kBlock))
    dense_forward_kernel(const T *__restrict__ path, T *__restrict__ sig, SigShape shape) {
    using G = Geometry<D, N, P>;
    __shared__ T sdx[kTile * D];
    const int pu = threadIdx.x;
    const bool active = pu < G::kLanes;
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);

    const int64_t row = blockIdx.x;
    const int64_t b = row / shape.W, w = row - b * shape.W;
    const Span span = unit_span(shape, w);
    const T *x = path + (b * shape.L + span.start) * D;

    T a[P + 1];
    T sub[G::kFwdSub];
#pragma unroll
    for (int j = 0; j <= P; ++j) a[j] = T(0);
#pragma unroll
    for (int i = 0; i < G::kFwdSub; ++i) sub[i] = T(0);

    for (int64_t t0 = 0; t0 < span.steps; t0 += kTile) {
        const int nt = (int)((span.steps - t0) < kTile ? (span.steps - t0) : kTile);
        const T *xw = x + t0 * D;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * D; idx += G::kBlock) sdx[idx] = xw[idx + D] - xw[idx];
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            T dx[D], dxp[P];
#pragma unroll
            for (int k = 0; k < D; ++k) dx[k] = sdx[tt * D + k];
#pragma unroll
            for (int j = 0; j < P; ++j) dxp[j] = sdx[tt * D + u[j]];
            StepTargets<T, D, P, N, false>::template run<G::kFwdSub>(a, sub, dx, dxp);
        }
    }

    if (!active) return;
    T *out = sig + row * G::kSigSize;
    // chain values are written by the lane whose remaining prefix letters are all zero
    {
        int rest = 1;  // D^(P-j)
#pragma unroll
        for (int j = P; j >= 1; --j) {
            if (pu % rest == 0) out[G::level_off(j) + pu / rest] = a[j];
            rest *= D;
        }
    }
    static_for<1, N - P + 1>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        constexpr int width = ipow(D, k);
        constexpr int off = trie_size(D, k - 1);
        T *dst = out + G::level_off(P + k) + (int64_t)pu * width;
#pragma unroll
        for (int i = 0; i < width; ++i) dst[i] = sub[off + i];
    });
}

// ---------------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int N, int P, bool ACCUMULATE>
__global__ void __launch_bounds__((Geometry<D, N, P>::kBlock))
    dense_backward_kernel(const T *__restrict__ path, const T *__restrict__ sig, const T *__restrict__ grad_sig,
                          T *__restrict__ grad_inc, SigShape shape) {
    using G = Geometry<D, N, P>;
    __shared__ T sdx[kTile * D];
    __shared__ T sg[G::kWaves][kTile * D];
    const int pu = threadIdx.x;
    const int lane = pu & (kWave - 1);
    const int wave = pu / kWave;
    const bool active = pu < G::kLanes;
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);

    const int64_t row = blockIdx.x;
    const int64_t b = row / shape.W, w = row - b * shape.W;
    const Span span = unit_span(shape, w);
    const T *x = path + (b * shape.L + span.start) * D;
    T *ginc = grad_inc + (b * (shape.L - 1) + span.start) * D;
    const T *srow = sig + row * G::kSigSize;
    const T *grow = grad_sig + row * G::kSigSize;

    // A: signature at the right end (levels < N).  H: upstream gradient; chain entries are lane-private
    // partial sums, so only the lane whose remaining prefix letters are zero starts from the gradient.
    T a[P + 1], hc[P + 1];
    constexpr int kAS = G::kASub > 0 ? G::kASub : 1;
    T asub[kAS];
    T hsub[G::kFwdSub];
    a[0] = T(1);
    hc[0] = T(0);
    {
        int rest = 1;
#pragma unroll
        for (int j = P; j >= 1; --j) {
            const int64_t col = G::level_off(j) + pu / rest;
            a[j] = (active && j < N) ? srow[col] : T(0);
            hc[j] = (active && pu % rest == 0) ? grow[col] : T(0);
            rest *= D;
        }
    }
    static_for<1, N - P + 1>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        constexpr int width = ipow(D, k);
        constexpr int off = trie_size(D, k - 1);
        const int64_t col = G::level_off(P + k) + (int64_t)pu * width;
#pragma unroll
        for (int i = 0; i < width; ++i) {
            hsub[off + i] = active ? grow[col + i] : T(0);
            if constexpr (k < N - P) asub[off + i] = active ? srow[col + i] : T(0);
        }
    });

    const int64_t ntiles = (span.steps + kTile - 1) / kTile;
    for (int64_t ti = ntiles - 1; ti >= 0; --ti) {
        const int64_t t0 = ti * kTile;
        const int nt = (int)((span.steps - t0) < kTile ? (span.steps - t0) : kTile);
        const T *xw = x + t0 * D;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * D; idx += G::kBlock) sdx[idx] = xw[idx + D] - xw[idx];
        __syncthreads();
        for (int tt = nt - 1; tt >= 0; --tt) {
            T dx[D], dxp[P];
#pragma unroll
            for (int k = 0; k < D; ++k) dx[k] = sdx[tt * D + k];
#pragma unroll
            for (int j = 0; j < P; ++j) dxp[j] = sdx[tt * D + u[j]];
            // A_t = A_{t+1} (x) exp(-dx_t), levels < N
            if constexpr (N > 1) StepTargets<T, D, P, N - 1, true>::template run<kAS>(a, asub, dx, dxp);
            T gdx[D], gpre[P];
#pragma unroll
            for (int k = 0; k < D; ++k) gdx[k] = T(0);
#pragma unroll
            for (int j = 0; j < P; ++j) gpre[j] = T(0);
            AdjTargets<T, D, N, P, 1>::template run<kAS, G::kFwdSub>(a, asub, hc, hsub, dx, dxp, gdx, gpre);
            // letter a collects the sub-trie sums and the chain positions whose letter is a
#pragma unroll
            for (int k = 0; k < D; ++k) {
                T v = gdx[k];
#pragma unroll
                for (int j = 0; j < P; ++j) v += (u[j] == k) ? gpre[j] : T(0);
                v = wave_total(v);
                if (lane == kWave - 1) sg[wave][tt * D + k] = v;
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * D; idx += G::kBlock) {
            T v = sg[0][idx];
#pragma unroll
            for (int q = 1; q < G::kWaves; ++q) v += sg[q][idx];
            if constexpr (ACCUMULATE) {
                atomicAdd(&ginc[t0 * D + idx], v);
            } else {
                ginc[t0 * D + idx] = v;
            }
        }
    }
}

// table of compiled shapes
struct Variant {
    int d, depth;
};
constexpr Variant kVariants[] = {{4, 6}, {8, 4}, {6, 5}, {4, 4}, {3, 5}, {2, 8}};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <typename T, int D, int N, int P>
hipError_t run_forward(const T *path, T *sig, const SigShape &shape, hipStream_t stream) {
    using G = Geometry<D, N, P>;
    const int64_t rows = shape.B * shape.W;
    hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P>), dim3((unsigned)rows), dim3(G::kBlock), 0, stream, path, sig,
                       shape);
    return hipGetLastError();
}

template <typename T, int D, int N, int P>
hipError_t run_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, const SigShape &shape,
                        hipStream_t stream) {
    using G = Geometry<D, N, P>;
    const int64_t rows = shape.B * shape.W;
    if (shape.windows) {
        hipError_t e = launch_fill_zero<T>(grad_inc, shape.B * (shape.L - 1) * shape.d, stream);
        if (e != hipSuccess) return e;
        if (rows == 0) return hipSuccess;
        hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, true>), dim3((unsigned)rows), dim3(G::kBlock), 0, stream,
                           path, sig, grad_sig, grad_inc, shape);
    } else {
        hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, false>), dim3((unsigned)rows), dim3(G::kBlock), 0, stream,
                           path, sig, grad_sig, grad_inc, shape);
    }
    return hipGetLastError();
}

}  // namespace

DenseChoice dense_choice(size_t, int64_t d, int depth, bool all_dense, const int64_t *, int64_t B, int64_t, int64_t W,
                         bool) {
    DenseChoice dc{false, -1, 1, 0, 0};
    if (!all_dense) return dc;
    if (B * W >= (int64_t(1) << 31)) return dc;
    for (int i = 0; i < kNumVariants; ++i) {
        if (kVariants[i].d == d && kVariants[i].depth == depth) {
            dc.usable = true;
            dc.variant = i;
            return dc;
        }
    }
    return dc;
}

#define PSIG_DISPATCH(CALL)                      \
    switch (dc.variant) {                        \
        case 0: return CALL(4, 6, 3);            \
        case 1: return CALL(8, 4, 2);            \
        case 2: return CALL(6, 5, 3);            \
        case 3: return CALL(4, 4, 2);            \
        case 4: return CALL(3, 5, 3);            \
        case 5: return CALL(2, 8, 5);            \
        default: return hipErrorNotSupported;    \
    }

template <typename T>
hipError_t launch_dense_forward(const T *path, T *sig, const SigShape &shape, const LevelPlan &, const int64_t *,
                                const DenseChoice &dc, void *, hipStream_t stream) {
#define PSIG_FWD(D, N, P) run_forward<T, D, N, P>(path, sig, shape, stream)
    PSIG_DISPATCH(PSIG_FWD)
#undef PSIG_FWD
}

template <typename T>
hipError_t launch_dense_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, const SigShape &shape,
                                 const LevelPlan &, const int64_t *, const DenseChoice &dc, void *,
                                 hipStream_t stream) {
#define PSIG_BWD(D, N, P) run_backward<T, D, N, P>(path, sig, grad_sig, grad_inc, shape, stream)
    PSIG_DISPATCH(PSIG_BWD)
#undef PSIG_BWD
}

#define PSIG_INSTANTIATE(T)                                                                                  \
    template hipError_t launch_dense_forward<T>(const T *, T *, const SigShape &, const LevelPlan &,         \
                                                const int64_t *, const DenseChoice &, void *, hipStream_t);  \
    template hipError_t launch_dense_backward<T>(const T *, const T *, const T *, T *, const SigShape &,     \
                                                 const LevelPlan &, const int64_t *, const DenseChoice &,    \
                                                 void *, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

}  // namespace psig
