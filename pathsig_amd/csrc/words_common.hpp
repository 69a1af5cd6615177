// Device helpers shared by the per-word signature kernels (lanes on words, and lanes on paths).
#pragma once

#include "common.hpp"

namespace psig {
namespace {

template <typename T>
__device__ __forceinline__ T fma_t(T a, T b, T c);
template <>
__device__ __forceinline__ float fma_t<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <>
__device__ __forceinline__ double fma_t<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ int find_level(const LevelPlan &plan, int64_t blk) {
    int deg = 1;
    while (deg < plan.depth && blk >= plan.block_begin[deg + 1]) ++deg;
    return deg;
}

struct WindowSpan {
    int64_t start, steps;
};

__device__ __forceinline__ WindowSpan window_span(const SigShape &shape, int64_t w) {
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

template <int DEG>
__device__ __forceinline__ void decode_letters(uint64_t code, uint64_t d, int (&l)[DEG]) {
#pragma unroll
    for (int pos = DEG - 1; pos >= 0; --pos) {
        const uint64_t q = code / d;
        l[pos] = (int)(code - q * d);
        code = q;
    }
}

// The letters of a word's step at every scale the chain asks for: dq[j][q - 1] = dl[j] / q, q <= DEG - j
// (position j + 1 is divided by m - j for target level m).  With them every chain node is one FMA, as in the
// register-tiled kernels, instead of an FMA and two multiplies.
template <typename T, int DEG>
__device__ __forceinline__ void scale_letters(const T (&dl)[DEG], T (&dq)[DEG][DEG]) {
#pragma unroll
    for (int j = 0; j < DEG; ++j) {
        dq[j][0] = dl[j];
#pragma unroll
        for (int q = 2; q <= DEG - j; ++q) dq[j][q - 1] = dl[j] * Recip<T>::of(q);
    }
}

// one forward Horner/Chen step on the chain p[0..TOP]; FORWARD = false rolls the step back (increment negated)
template <typename T, int DEG, int TOP, bool FORWARD>
__device__ __forceinline__ void chain_step(T (&p)[DEG + 1], const T (&dq)[DEG][DEG]) {
#pragma unroll
    for (int m = TOP; m >= 1; --m) {
        T tmp = T(1);
#pragma unroll
        for (int j = 1; j < m; ++j) {
            const T inc = FORWARD ? dq[j - 1][m - j] : -dq[j - 1][m - j];  // dl[j - 1] / (m - j + 1)
            tmp = j == 1 ? p[1] + inc : fma_t<T>(tmp, inc, p[j]);
        }
        const T inc = FORWARD ? dq[m - 1][0] : -dq[m - 1][0];
        p[m] = m == 1 ? p[1] + inc : fma_t<T>(tmp, inc, p[m]);
    }
}

// Adjoint of one Chen step on the chain.  p is the chain before the step (levels < DEG are read), h the
// adjoint of the chain after the step; on return h is the adjoint before the step and gl[k] holds the
// step's dL/d(dl[k]).  Targets ascend, so h[m] is still the adjoint after the step when target m reads it.
template <typename T, int DEG>
__device__ __forceinline__ void chain_step_adjoint(const T (&p)[DEG + 1], T (&h)[DEG + 1], const T (&dl)[DEG],
                                                   const T (&dq)[DEG][DEG], T (&gl)[DEG]) {
#pragma unroll
    for (int k = 0; k < DEG; ++k) gl[k] = T(0);
#pragma unroll
    for (int m = 1; m <= DEG; ++m) {
        // t[j] = Horner value after position j for target m (t[0] = 1)
        T t[DEG + 1];
        t[0] = T(1);
#pragma unroll
        for (int j = 1; j < m; ++j) t[j] = j == 1 ? p[1] + dq[0][m - 1] : fma_t<T>(t[j - 1], dq[j - 1][m - j], p[j]);
        T gt = h[m];
#pragma unroll
        for (int j = m; j >= 1; --j) {
            // node j: value p[j] + t[j - 1] * dl[j - 1] / q with q = m - j + 1
            const T gts = j == m ? gt : gt * Recip<T>::of(m - j + 1);
            gl[j - 1] = j == 1 ? gl[0] + gts : fma_t<T>(gts, t[j - 1], gl[j - 1]);
            if (j > 1) {
                gt = gts * dl[j - 1];
                h[j - 1] += gt;
            }
        }
    }
}

}  // namespace
}  // namespace psig
