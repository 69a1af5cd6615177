// Signature <-> log-signature on the hybrid layout (levels below `depth` dense, top level dense or
// a list of words).  One workgroup owns one row (one path, or one window of one path) and walks the
// levels itself, so the whole conversion is one launch per direction.
//
// Forward (reference: src/pathsig/forward/sig_kernels.cu:161-241): with X = S - 1,
//     P_1(w) = S(w),  P_m(w) = sum_{k=m-1}^{n-1} P_{m-1}(w_1..w_k) * S(w_{k+1}..w_n),
//     log S(w) = sum_m (-1)^(m+1)/m * P_m(w).
// Level n reads the P rows of the levels below it, so levels go up with a workgroup barrier between.
// Backward (reference: src/pathsig/backward/sig_backward_kernels.cu:381-477) is the adjoint, levels
// going down; the P adjoint of the lower levels lives in the caller's workspace.
#include "common.hpp"

namespace psig {

namespace {

constexpr int kLogBlock = 512;

template <typename T>
__device__ __forceinline__ T alt_coeff(int m) {
    const T r = T(1) / T(m);
    return (m & 1) ? r : -r;
}

struct HybridPlan {
    int depth;
    int64_t d;
    int64_t size[kMaxDepth + 1];
    int64_t off[kMaxDepth + 1];
    int64_t total;     // S of the hybrid layout
    int64_t lower;     // columns of the levels below `depth`
    int top_is_list;   // top level takes its codes from top_words
};

template <typename T, int DEG>
__device__ void logsig_forward_level(const T *__restrict__ s, T *P, T *__restrict__ lg, const HybridPlan &hp,
                                     const int64_t *__restrict__ top_words) {
    const int depth = hp.depth;
    const uint64_t d = (uint64_t)hp.d;
    const bool listed = (DEG == depth) && hp.top_is_list;
    for (int64_t i = threadIdx.x; i < hp.size[DEG]; i += kLogBlock) {
        const uint64_t code = listed ? (uint64_t)top_words[i] : (uint64_t)i;
        // dense column of every proper prefix, value of every proper suffix
        uint64_t pidx[DEG + 1];
        T sufv[DEG + 1];
        {
            uint64_t div = 1;  // d^(DEG-k)
#pragma unroll
            for (int k = 1; k < DEG; ++k) div *= d;
            uint64_t lo = 0, width = 1;
#pragma unroll
            for (int k = 1; k < DEG; ++k) {
                width *= d;
                pidx[k] = lo + code / div;  // first k letters
                sufv[k] = s[lo + code % width];  // last k letters
                lo += width;
                div /= d;
            }
        }
        const uint64_t own = (uint64_t)(hp.off[DEG] + i);
        const T sw = s[own];
        sufv[DEG] = sw;
        T *Pw = P + own * (uint64_t)depth;
        Pw[0] = sw;
        T acc = sw;
#pragma unroll
        for (int m = 2; m <= DEG; ++m) {
            T pv = T(0);
#pragma unroll
            for (int k = m - 1; k < DEG; ++k) pv += P[pidx[k] * (uint64_t)depth + (uint64_t)(m - 2)] * sufv[DEG - k];
            acc += alt_coeff<T>(m) * pv;
            Pw[m - 1] = pv;
        }
        for (int m = DEG + 1; m <= depth; ++m) Pw[m - 1] = T(0);
        lg[own] = acc;
    }
}

template <typename T>
__global__ void __launch_bounds__(kLogBlock) logsig_forward_kernel(const T *__restrict__ sig, T *__restrict__ logsig,
                                                                   T *P, HybridPlan hp,
                                                                   const int64_t *__restrict__ top_words) {
    const int64_t row = blockIdx.x;
    const T *s = sig + row * hp.total;
    T *lg = logsig + row * hp.total;
    T *Pr = P + row * hp.total * hp.depth;
    for (int deg = 1; deg <= hp.depth; ++deg) {
        switch (deg) {
#define PSIG_CASE(N) \
    case N: logsig_forward_level<T, N>(s, Pr, lg, hp, top_words); break;
            PSIG_CASE(1) PSIG_CASE(2) PSIG_CASE(3) PSIG_CASE(4) PSIG_CASE(5) PSIG_CASE(6)
            PSIG_CASE(7) PSIG_CASE(8) PSIG_CASE(9) PSIG_CASE(10) PSIG_CASE(11) PSIG_CASE(12)
#undef PSIG_CASE
            default: break;
        }
        __threadfence_block();
        __syncthreads();
    }
}

// Accumulators of the adjoint.  Short words collect contributions from every longer word, so the
// columns below `lds_cols` (whole levels) live in LDS, where the adds are cheap; the rest are global.
template <typename T>
struct AdjointSink {
    T *gs;         // global: gradient w.r.t. the signature, one row
    T *gP;         // global: adjoint of the power cache, rows of `depth`, levels below the top
    T *lds_gs;     // LDS copies of the first lds_cols columns
    T *lds_gP;
    int64_t lds_cols;
    int depth;
    __device__ __forceinline__ void add_gs(uint64_t col, T v) {
        if ((int64_t)col < lds_cols) atomicAdd(&lds_gs[col], v);
        else atomicAdd(&gs[col], v);
    }
    __device__ __forceinline__ void add_gP(uint64_t col, int m_index, T v) {
        if ((int64_t)col < lds_cols) atomicAdd(&lds_gP[col * depth + m_index], v);
        else atomicAdd(&gP[col * depth + m_index], v);
    }
    __device__ __forceinline__ T read_gP(uint64_t col, int m_index) const {
        return ((int64_t)col < lds_cols) ? lds_gP[col * depth + m_index] : gP[col * depth + m_index];
    }
};

template <typename T, int DEG>
__device__ void logsig_backward_level(const T *__restrict__ s, const T *__restrict__ P, const T *__restrict__ gl,
                                      AdjointSink<T> &sink, const HybridPlan &hp,
                                      const int64_t *__restrict__ top_words) {
    const int depth = hp.depth;
    const uint64_t d = (uint64_t)hp.d;
    const bool top = (DEG == depth);
    const bool listed = top && hp.top_is_list;
    for (int64_t i = threadIdx.x; i < hp.size[DEG]; i += kLogBlock) {
        const uint64_t code = listed ? (uint64_t)top_words[i] : (uint64_t)i;
        uint64_t pidx[DEG + 1], sidx[DEG + 1];
        {
            uint64_t div = 1;
#pragma unroll
            for (int k = 1; k < DEG; ++k) div *= d;
            uint64_t lo = 0, width = 1;
#pragma unroll
            for (int k = 1; k < DEG; ++k) {
                width *= d;
                pidx[k] = lo + code / div;
                sidx[k] = lo + code % width;
                lo += width;
                div /= d;
            }
        }
        const uint64_t own = (uint64_t)(hp.off[DEG] + i);
        const T g = gl[own];
        T gPv[DEG];
#pragma unroll
        for (int m = 1; m <= DEG; ++m) {
            // a top-level word is nobody's prefix: nothing has been accumulated for it
            const T acc = top ? T(0) : sink.read_gP(own, m - 1);
            gPv[m - 1] = alt_coeff<T>(m) * g + acc;
        }
        sink.add_gs(own, gPv[0]);
#pragma unroll
        for (int m = 2; m <= DEG; ++m) {
#pragma unroll
            for (int k = m - 1; k < DEG; ++k) {
                const uint64_t pi = pidx[k], si = sidx[DEG - k];
                sink.add_gP(pi, m - 2, gPv[m - 1] * s[si]);
                sink.add_gs(si, gPv[m - 1] * P[pi * (uint64_t)depth + (uint64_t)(m - 2)]);
            }
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kLogBlock) logsig_backward_kernel(const T *__restrict__ sig, const T *__restrict__ P,
                                                                    const T *__restrict__ grad_logsig, T *grad_sig,
                                                                    T *gradP, HybridPlan hp,
                                                                    const int64_t *__restrict__ top_words,
                                                                    int64_t lds_cols) {
    extern __shared__ __align__(16) unsigned char logsig_smem[];
    const int64_t row = blockIdx.x;
    const T *s = sig + row * hp.total;
    const T *Pr = P + row * hp.total * hp.depth;
    const T *gl = grad_logsig + row * hp.total;
    AdjointSink<T> sink;
    sink.gs = grad_sig + row * hp.total;
    sink.gP = gradP + row * hp.lower * hp.depth;
    sink.lds_gs = reinterpret_cast<T *>(logsig_smem);
    sink.lds_gP = sink.lds_gs + lds_cols;
    sink.lds_cols = lds_cols;
    sink.depth = hp.depth;
    for (int64_t i = threadIdx.x; i < hp.total; i += kLogBlock) sink.gs[i] = T(0);
    for (int64_t i = threadIdx.x; i < hp.lower * hp.depth; i += kLogBlock) sink.gP[i] = T(0);
    for (int64_t i = threadIdx.x; i < lds_cols * (hp.depth + 1); i += kLogBlock) sink.lds_gs[i] = T(0);
    __threadfence_block();
    __syncthreads();
    for (int deg = hp.depth; deg >= 1; --deg) {
        switch (deg) {
#define PSIG_CASE(N) \
    case N: logsig_backward_level<T, N>(s, Pr, gl, sink, hp, top_words); break;
            PSIG_CASE(1) PSIG_CASE(2) PSIG_CASE(3) PSIG_CASE(4) PSIG_CASE(5) PSIG_CASE(6)
            PSIG_CASE(7) PSIG_CASE(8) PSIG_CASE(9) PSIG_CASE(10) PSIG_CASE(11) PSIG_CASE(12)
#undef PSIG_CASE
            default: break;
        }
        __threadfence_block();
        __syncthreads();
    }
    for (int64_t i = threadIdx.x; i < lds_cols; i += kLogBlock) sink.gs[i] = sink.lds_gs[i];
}

// largest number of whole low levels whose accumulators (1 + depth values per column) fit `budget` bytes
int64_t lds_columns(int64_t d, int depth, size_t elem, size_t budget) {
    int64_t cols = 0, width = 1;
    for (int k = 1; k < depth; ++k) {
        width *= d;
        if ((size_t)(cols + width) * (size_t)(depth + 1) * elem > budget) break;
        cols += width;
    }
    return cols;
}

HybridPlan make_hybrid(int64_t d, int depth, int64_t top_size, const int64_t *top_words) {
    HybridPlan hp{};
    hp.depth = depth;
    hp.d = d;
    int64_t off = 0, width = 1;
    for (int k = 1; k <= depth; ++k) {
        width *= d;
        hp.size[k] = (k == depth) ? top_size : width;
        hp.off[k] = off;
        if (k == depth) {
            hp.lower = off;
            hp.top_is_list = (top_size != width && top_words != nullptr) ? 1 : 0;
        }
        off += hp.size[k];
    }
    hp.total = off;
    return hp;
}

}  // namespace

template <typename T>
hipError_t launch_logsig_forward(const T *sig, T *logsig, T *P, int64_t rows, int64_t d, int depth, int64_t top_size,
                                 const int64_t *top_words, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    const HybridPlan hp = make_hybrid(d, depth, top_size, top_words);
    hipLaunchKernelGGL(logsig_forward_kernel<T>, dim3((unsigned)rows), dim3(kLogBlock), 0, stream, sig, logsig, P, hp,
                       top_words);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_logsig_backward(const T *sig, const T *P, const T *grad_logsig, T *grad_sig, T *gradP, int64_t rows,
                                  int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                                  hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    const HybridPlan hp = make_hybrid(d, depth, top_size, top_words);
    const int64_t lds_cols = lds_columns(d, depth, sizeof(T), 32 * 1024);
    const size_t lds_bytes = (size_t)lds_cols * (size_t)(depth + 1) * sizeof(T);
    hipLaunchKernelGGL(logsig_backward_kernel<T>, dim3((unsigned)rows), dim3(kLogBlock), lds_bytes, stream, sig, P,
                       grad_logsig, grad_sig, gradP, hp, top_words, lds_cols);
    return hipGetLastError();
}

#define PSIG_INSTANTIATE(T)                                                                                       \
    template hipError_t launch_logsig_forward<T>(const T *, T *, T *, int64_t, int64_t, int, int64_t,             \
                                                 const int64_t *, hipStream_t);                                   \
    template hipError_t launch_logsig_backward<T>(const T *, const T *, const T *, T *, T *, int64_t, int64_t, int, \
                                                  int64_t, const int64_t *, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

}  // namespace psig
