// Signature <-> log-signature on the hybrid layout (levels below `depth` dense, top level dense or
// a list of words).  One workgroup owns one row (one path, or one window of one path) and walks the
// levels itself, so the whole conversion is one launch per direction.
//
// The reference (src/pathsig/forward/sig_kernels.cu:161-241) sums the series of log(1 + X), X = S - 1:
//     P_1(w) = S(w),  P_m(w) = sum_{k=m-1}^{n-1} P_{m-1}(w_1..w_k) * S(w_{k+1}..w_n),
//     log S(w) = sum_m (-1)^(m+1)/m * P_m(w).
// The powers of X grow like exp|x| and cancel in the alternating sum, which costs that series most of the
// digits of fp32 on long or deep inputs.  The values are therefore computed by inverting the exponential
// instead, with powers of the (much smaller) log-signature L itself and the coefficients 1/k! :
//     Q_1(w) = L(w),  Q_k(w) = sum_{j=k-1}^{n-1} Q_{k-1}(w_1..w_j) * L(w_{j+1}..w_n),
//     L(w) = S(w) - sum_{k=2}^{n} Q_k(w) / k! .
// Same recursion shape, same cost, same cache layout (row idx, entry k - 1); the cache of this form is what
// the adjoint below reads.  The power cache P of the reference is still produced, by a second pass of the
// same kernel, for the entry point that returns it.
//
// Backward (reference: src/pathsig/backward/sig_backward_kernels.cu:381-477, the adjoint of the P form) is
// the adjoint of the Q form, levels going down.  With lam(w) = dLoss/dL(w), a_k(w) = dLoss/dQ_k(w), f_k = 1/k!
// and g the upstream gradient,
//     lam(w) = g(w) + a_1(w) + sum_{u} sum_{k=2}^{|u|+1} a_k(u w) Q_{k-1}(u),
//     a_k(w) = -[k >= 2] f_k lam(w) + sum_{v, |wv| <= depth} a_{k+1}(w v) L(v),
//     dLoss/dS(w) = lam(w);  for top-level words lam = g and a_k = -f_k g.
// Two forms:
//   * gather form (used whenever a dense copy of the top-level gradient fits the workspace): every sum over
//     v (or u) of a fixed length is a matrix-vector product over a dense level, so each output has one owner
//     and nothing is atomic;
//   * scatter form (any size): every word pushes its terms to its prefixes and suffixes with atomics.
#include <cmath>
#include <cstdlib>

#include "common.hpp"

namespace psig {

namespace {

constexpr int kLogBlock = 512;  // threads of a block at most; the kernels take their stride from blockDim.x

// Threads per row (a row is one block).  A few rows get the largest block: the time of one row is all there is.
// With many rows of a small layout most of 512 threads would idle through every pass while few rows fit a CU, so
// the block shrinks with the layout and more rows run side by side.
inline int logsig_block(int64_t columns, int64_t rows) {
    if (rows <= 256 || columns > 2048) return kLogBlock;
    return columns > 512 ? 256 : columns > 128 ? 128 : 64;
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

// 1/k! for the exponential series
template <typename T>
__device__ __forceinline__ constexpr T inv_factorial(int k) {
    T r = T(1);
    for (int i = 2; i <= k; ++i) r /= T(i);
    return r;
}

// Dense columns (level offsets included) of every proper prefix and suffix of a word of DEG letters: pidx[k] its
// first k letters, sidx[k] its last k letters, k = 1 .. DEG - 1.  One division per letter: the first k letters are
// the first k + 1 without the last, and the last k are what the first DEG - k leave of the word.  IDX is uint32_t
// when the codes of the level and the cache columns fit 32 bits (a 64-bit division by a run-time divisor is a
// hundred instructions, and there would be 2 (DEG - 1) of them per word).
template <typename IDX, int DEG>
__device__ __forceinline__ void word_splits(IDX code, IDX d, IDX (&pidx)[DEG + 1], IDX (&sidx)[DEG + 1]) {
    IDX first[DEG + 1];
    first[DEG] = code;
#pragma unroll
    for (int k = DEG - 1; k >= 1; --k) first[k] = first[k + 1] / d;
    IDX lo = 0, width = 1;
#pragma unroll
    for (int k = 1; k < DEG; ++k) {
        width *= d;
        pidx[k] = lo + first[k];
        sidx[k] = lo + (code - first[DEG - k] * width);
        lo += width;
    }
}

// One level of one row.  STABLE: C is the cache of the Q form (entry k - 1 of a row holds Q_k; entry 0 the
// log-signature itself), the right factors are log-signature values of the levels below, read from lg, and
// lg receives the level.  Otherwise C is the power cache P of the reference, the right factors are signature
// values, and lg is not touched.
template <typename T, int DEG, bool STABLE, typename IDX>
__device__ void logsig_forward_level(const T *__restrict__ s, T *C, T *lg, const HybridPlan &hp,
                                     const int64_t *__restrict__ top_words) {
    const int depth = hp.depth;
    const IDX d = (IDX)hp.d;
    const bool listed = (DEG == depth) && hp.top_is_list;
    const T *right = STABLE ? lg : s;
    // the blocks of one row (gridDim.y of them) share the words of the level
    for (int64_t i = (int64_t)blockIdx.y * (int)blockDim.x + threadIdx.x; i < hp.size[DEG]; i += (int64_t)gridDim.y * (int)blockDim.x) {
        const IDX code = listed ? (IDX)top_words[i] : (IDX)i;
        // dense column of every proper prefix, right factor of every proper suffix
        IDX pidx[DEG + 1], sidx[DEG + 1];
        T sufv[DEG + 1];
        word_splits<IDX, DEG>(code, d, pidx, sidx);
#pragma unroll
        for (int k = 1; k < DEG; ++k) sufv[k] = right[sidx[k]];
        const IDX own = (IDX)(hp.off[DEG] + i);
        const T sw = s[own];
        T *Cw = C + own * (IDX)depth;
        // the Q form never reads the cache rows of the top level (nothing is longer than a top-level word), so
        // they are not written: for many rows the cache is most of what this kernel moves
        const bool keep_row = !STABLE || DEG < depth;
        T acc = sw;
        T qc = T(0);  // -sum_{m=2}^{DEG} Q_m(w) / (m + 1)!
#pragma unroll
        for (int m = 2; m <= DEG; ++m) {
            T pv = T(0);
#pragma unroll
            for (int k = m - 1; k < DEG; ++k) pv += C[pidx[k] * (IDX)depth + (IDX)(m - 2)] * sufv[DEG - k];
            if constexpr (STABLE) {
                acc -= inv_factorial<T>(m) * pv;
                qc -= inv_factorial<T>(m + 1) * pv;
            }
            if (keep_row) Cw[m - 1] = pv;
        }
        if constexpr (STABLE) {
            if (keep_row) {
                // entry |w| of the row, which no product reads: Qc(w) = -sum_{m=1}^{|w|} Q_m(w) / (m + 1)!, the
                // weight with which w enters the top-level sums of the adjoint as a prefix
                Cw[0] = acc;
                Cw[DEG] = qc - inv_factorial<T>(2) * acc;
                for (int m = DEG + 2; m <= depth; ++m) Cw[m - 1] = T(0);
            }
            lg[own] = acc;
        } else {
            for (int m = DEG + 1; m <= depth; ++m) Cw[m - 1] = T(0);
            Cw[0] = sw;
        }
    }
}

// Levels first..last of one row per blockIdx.x.  Several levels need one block per row (gridDim.y == 1: the
// barrier between levels is a workgroup barrier); a single level may be shared by gridDim.y blocks.
// IDX: type of the column arithmetic (word_splits).
template <typename T, bool STABLE, typename IDX>
__global__ void __launch_bounds__(kLogBlock) logsig_forward_kernel(const T *__restrict__ sig, T *logsig, T *C,
                                                                   HybridPlan hp,
                                                                   const int64_t *__restrict__ top_words, int first,
                                                                   int last) {
    const int64_t row = blockIdx.x;
    const T *s = sig + row * hp.total;
    T *lg = logsig + row * hp.total;
    T *Cr = C + row * hp.total * hp.depth;
    for (int deg = first; deg <= last; ++deg) {
        switch (deg) {
#define PSIG_CASE(N) \
    case N: logsig_forward_level<T, N, STABLE, IDX>(s, Cr, lg, hp, top_words); break;
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
    __device__ __forceinline__ T read_gs(uint64_t col) const { return ((int64_t)col < lds_cols) ? lds_gs[col] : gs[col]; }
    __device__ __forceinline__ void set_gs(uint64_t col, T v) {
        if ((int64_t)col < lds_cols) lds_gs[col] = v;
        else gs[col] = v;
    }
};

// lgrow: the log-signature row; C: the cache row of the Q form.  When a level is processed, everything the
// longer words push to it has arrived (levels go down with a barrier between them): the accumulated gradient
// of a word holds its suffix-type sums and entry k - 1 of its cache adjoint holds sum_v a_{k+1}(w v) L(v).
template <typename T, int DEG>
__device__ void logsig_backward_level(const T *__restrict__ lgrow, const T *__restrict__ C, const T *__restrict__ gl,
                                      AdjointSink<T> &sink, const HybridPlan &hp,
                                      const int64_t *__restrict__ top_words) {
    const int depth = hp.depth;
    const uint64_t d = (uint64_t)hp.d;
    const bool top = (DEG == depth);
    const bool listed = top && hp.top_is_list;
    for (int64_t i = threadIdx.x; i < hp.size[DEG]; i += (int)blockDim.x) {
        const uint64_t code = listed ? (uint64_t)top_words[i] : (uint64_t)i;
        uint64_t pidx[DEG + 1], sidx[DEG + 1];
        word_splits<uint64_t, DEG>(code, d, pidx, sidx);
        const uint64_t own = (uint64_t)(hp.off[DEG] + i);
        // a top-level word is nobody's prefix or suffix: nothing has been accumulated for it
        T lam = gl[own];
        if (!top) lam += sink.read_gP(own, 0) + sink.read_gs(own);
        T av[DEG];
#pragma unroll
        for (int k = 2; k <= DEG; ++k) av[k - 1] = (top ? T(0) : sink.read_gP(own, k - 1)) - inv_factorial<T>(k) * lam;
        sink.set_gs(own, lam);
#pragma unroll
        for (int k = 2; k <= DEG; ++k) {
#pragma unroll
            for (int j = k - 1; j < DEG; ++j) {
                const uint64_t pi = pidx[j], si = sidx[DEG - j];
                sink.add_gP(pi, k - 2, av[k - 1] * lgrow[si]);
                sink.add_gs(si, av[k - 1] * C[pi * (uint64_t)depth + (uint64_t)(k - 2)]);
            }
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kLogBlock) logsig_backward_kernel(const T *__restrict__ logsig,
                                                                    const T *__restrict__ cache,
                                                                    const T *__restrict__ grad_logsig, T *grad_sig,
                                                                    T *gradP, HybridPlan hp,
                                                                    const int64_t *__restrict__ top_words,
                                                                    int64_t lds_cols) {
    extern __shared__ __align__(16) unsigned char logsig_smem[];
    const int64_t row = blockIdx.x;
    const T *s = logsig + row * hp.total;
    const T *Pr = cache + row * hp.total * hp.depth;
    const T *gl = grad_logsig + row * hp.total;
    AdjointSink<T> sink;
    sink.gs = grad_sig + row * hp.total;
    sink.gP = gradP + row * hp.lower * hp.depth;
    sink.lds_gs = reinterpret_cast<T *>(logsig_smem);
    sink.lds_gP = sink.lds_gs + lds_cols;
    sink.lds_cols = lds_cols;
    sink.depth = hp.depth;
    for (int64_t i = threadIdx.x; i < hp.total; i += (int)blockDim.x) sink.gs[i] = T(0);
    for (int64_t i = threadIdx.x; i < hp.lower * hp.depth; i += (int)blockDim.x) sink.gP[i] = T(0);
    for (int64_t i = threadIdx.x; i < lds_cols * (hp.depth + 1); i += (int)blockDim.x) sink.lds_gs[i] = T(0);
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
    for (int64_t i = threadIdx.x; i < lds_cols; i += (int)blockDim.x) sink.gs[i] = sink.lds_gs[i];
}

// ---------------------------------------------------------------------------------------------
// gather form of the adjoint
// ---------------------------------------------------------------------------------------------
// use(i, load(i)) for i = threadIdx.x, threadIdx.x + blockDim.x, .. below count, with the loads of K rounds issued
// before the first value is used: a loop that loads and uses one element per round waits for memory in every
// round.  (The loads are unconditional, at a clamped index, so that the compiler can count them.)
template <int K, typename Load, typename Use>
__device__ __forceinline__ void batched_rounds(int64_t count, Load &&load, Use &&use) {
    using V = decltype(load(int64_t(0)));
    for (int64_t base = threadIdx.x; base < count; base += (int64_t)K * (int)blockDim.x) {
        V v[K];
#pragma unroll
        for (int r = 0; r < K; ++r) {
            const int64_t i = base + (int64_t)r * (int)blockDim.x;
            v[r] = load(i < count ? i : count - 1);
        }
#pragma unroll
        for (int r = 0; r < K; ++r) {
            const int64_t i = base + (int64_t)r * (int)blockDim.x;
            if (i < count) use(i, v[r]);
        }
    }
}

// A batch of matrix-vector products by all threads of the block:
//     out[b][o] = sum_{k < nk} sum_{m < nm} A[b*ab + o*so + k*sk + m*sm] * B[b*bb + k*sb + m*sn]
// for b < nb, o < no; store(b, o, value) runs once per output, in one thread.  When there are fewer outputs
// than threads the k range is split over `parts` threads per output and the partial sums meet in LDS
// (`red`, one element per thread).  Lanes run along whichever of o and k is contiguous in A.  Ends with a
// block barrier that also orders the stores in global memory for the next call.
// When k is the contiguous index, nm = 1 and there are outputs enough to occupy the block that way, up to 64
// consecutive lanes of a wave share an output instead, whatever the number of outputs: their loads are coalesced
// (a thread that walks a row of its own makes every load of the wave touch 64 cache lines: measured 19 µs against
// 7 for the same 128 KB), and the partial sums of eight outputs at a time meet through wave shuffles.
struct MatvecShape {
    int64_t nb, no, nk, nm;   // batch, outputs, reduction length, inner terms
    int64_t ab, so, sk, sm;   // strides of A
    int64_t bb, sb, sn;       // strides of B
};

// Counts fit 32 bits (the caller's layouts are bounded by the workspace limits); the operands are walked with
// pointers that advance by a constant, so the inner loop is two loads, one multiply-add and two pointer steps.
template <typename T, typename Store>
__device__ void block_matvec(const T *A, const T *B, const MatvecShape &sh, T *red, Store &&store) {
    const int no = (int)sh.no, nk = (int)sh.nk, nm = (int)sh.nm;
    const int outputs = (int)sh.nb * no;
    int parts = 1;
    while (parts * 2 * outputs <= (int)blockDim.x && parts * 2 <= nk) parts *= 2;
    const int slots = (int)blockDim.x / parts;  // outputs worked on at once; >= outputs whenever parts > 1
    const bool k_fast = sh.sk < sh.so;
    const int tid = threadIdx.x;
    if (k_fast && nm == 1 && (int)blockDim.x % kWave == 0) {
        int lanes = 1;  // lanes of a wave that share an output
        while (lanes * 2 <= kWave && lanes * 2 <= nk) lanes *= 2;
        constexpr int kAtOnce = 8;
        const int per_pass = (int)blockDim.x / lanes;  // outputs of one pass of the block
        if (lanes >= 4 && outputs >= per_pass) {
            const int at = tid % lanes, oloc = tid / lanes;
            const int64_t astep = (int64_t)lanes * sh.sk, bstep = (int64_t)lanes * sh.sb;
            for (int o0 = 0; o0 < outputs; o0 += per_pass * kAtOnce) {
                T acc[kAtOnce];
                int bi[kAtOnce], o[kAtOnce];
#pragma unroll
                for (int r = 0; r < kAtOnce; ++r) {
                    const int oo = o0 + r * per_pass + oloc;
                    const bool have = oo < outputs;
                    bi[r] = have ? (sh.nb == 1 ? 0 : oo / no) : -1;
                    o[r] = have ? oo - bi[r] * no : 0;
                    acc[r] = T(0);
                }
                if (nk <= lanes) {
                    // one term per lane: the loads of the eight outputs are in flight together
                    T av[kAtOnce], bv[kAtOnce];
#pragma unroll
                    for (int r = 0; r < kAtOnce; ++r) {
                        const bool have = bi[r] >= 0 && at < nk;
                        const int b = have ? bi[r] : 0;
                        av[r] = have ? A[(int64_t)b * sh.ab + (int64_t)o[r] * sh.so + (int64_t)at * sh.sk] : T(0);
                        bv[r] = have ? B[(int64_t)b * sh.bb + (int64_t)at * sh.sb] : T(0);
                    }
#pragma unroll
                    for (int r = 0; r < kAtOnce; ++r) acc[r] = av[r] * bv[r];
                } else {
#pragma unroll
                    for (int r = 0; r < kAtOnce; ++r) {
                        if (bi[r] < 0) continue;
                        const T *ap = A + (int64_t)bi[r] * sh.ab + (int64_t)o[r] * sh.so + (int64_t)at * sh.sk;
                        const T *bp = B + (int64_t)bi[r] * sh.bb + (int64_t)at * sh.sb;
                        T sum = T(0);
#pragma unroll 8
                        for (int k = at; k < nk; k += lanes) {
                            sum += *ap * *bp;
                            ap += astep;
                            bp += bstep;
                        }
                        acc[r] = sum;
                    }
                }
                for (int off = lanes / 2; off >= 1; off /= 2) {
#pragma unroll
                    for (int r = 0; r < kAtOnce; ++r) acc[r] += __shfl_xor(acc[r], off);
                }
                if (at == 0) {
#pragma unroll
                    for (int r = 0; r < kAtOnce; ++r)
                        if (bi[r] >= 0) store((int64_t)bi[r], (int64_t)o[r], acc[r]);
                }
            }
            __threadfence_block();
            __syncthreads();
            return;
        }
    }
    const int part = k_fast ? tid % parts : tid / slots;
    const int oloc = k_fast ? tid / parts : tid % slots;
    const int64_t astep = (int64_t)parts * sh.sk, bstep = (int64_t)parts * sh.sb;
    for (int o0 = 0; o0 < outputs; o0 += slots) {
        const int oo = o0 + oloc;
        const int bi = oo / no, o = oo - bi * no;
        T acc = T(0);
        if (oo < outputs) {
            const T *ap = A + (int64_t)bi * sh.ab + (int64_t)o * sh.so + (int64_t)part * sh.sk;
            const T *bp = B + (int64_t)bi * sh.bb + (int64_t)part * sh.sb;
            if (nm == 1) {
#pragma unroll 8
                for (int k = part; k < nk; k += parts) {
                    acc += *ap * *bp;
                    ap += astep;
                    bp += bstep;
                }
            } else {
                for (int k = part; k < nk; k += parts) {
                    const T *am = ap, *bm = bp;
                    for (int m = 0; m < nm; ++m) {
                        acc += *am * *bm;
                        am += sh.sm;
                        bm += sh.sn;
                    }
                    ap += astep;
                    bp += bstep;
                }
            }
        }
        if (parts > 1) {
            red[tid] = acc;
            __syncthreads();
            if (part == 0 && oo < outputs) {
                T total = T(0);
                for (int q = 0; q < parts; ++q) total += red[k_fast ? oloc * parts + q : q * slots + oloc];
                store((int64_t)bi, (int64_t)o, total);
            }
            __syncthreads();
        } else if (oo < outputs) {
            store((int64_t)bi, (int64_t)o, acc);
        }
    }
    __threadfence_block();
    __syncthreads();
}

// Top-level part of the gather form, one block per (row, split, side): with the top-level gradient g as a
// d^j x d^(N-j) matrix, side 0 computes R(u) = sum_v g(uv) L(v) for the prefixes u of length j, side 1
// computes T(v) = sum_u g(uv) Qc(u) for the suffixes v of length N - j, where
// Qc(u) = -sum_{k=2}^{|u|+1} Q_{k-1}(u) / k! is entry |u| of u's cache row (the forward puts it there).  R goes to its own workspace array, T
// initialises the gradient.
template <typename T>
__global__ void __launch_bounds__(kLogBlock) logsig_gather_top_kernel(const T *__restrict__ logsig,
                                                                      const T *__restrict__ cache,
                                                                      const T *__restrict__ gtop_all, T *grad_sig,
                                                                      T *R_all, HybridPlan hp, int64_t top_dense,
                                                                      const T *__restrict__ grad_logsig) {
    __shared__ T red[kLogBlock];
    const int N = hp.depth;
    const int64_t row = blockIdx.x;
    const int j = (int)blockIdx.y + 1, i = N - j;
    const bool suffix_side = blockIdx.z == 1;
    {
        // the gradient of a top-level word is its upstream gradient: every block of the row copies a slice
        const int64_t slices = 2 * (int64_t)gridDim.y, slice = 2 * (int64_t)blockIdx.y + blockIdx.z;
        const int64_t per = (hp.size[N] + slices - 1) / slices;
        const int64_t from = slice * per, to = from + per < hp.size[N] ? from + per : hp.size[N];
        const T *gl = grad_logsig + row * hp.total + hp.off[N];
        T *gs = grad_sig + row * hp.total + hp.off[N];
        if (from < to)
            batched_rounds<4>(to - from, [&](int64_t e) { return gl[from + e]; }, [&](int64_t e, T v) { gs[from + e] = v; });
    }
    const T *lgs = logsig + row * hp.total;
    const T *gtop = gtop_all + row * top_dense;
    int64_t wi = 1, wj = 1;
    for (int k = 0; k < i; ++k) wi *= hp.d;
    for (int k = 0; k < j; ++k) wj *= hp.d;
    if (!suffix_side) {
        T *R = R_all + row * hp.lower + hp.off[j];
        block_matvec<T>(gtop, lgs + hp.off[i], MatvecShape{1, wj, wi, 1, 0, wi, 1, 0, 0, 1, 0}, red,
                        [&](int64_t, int64_t o, T r) { R[o] = r; });
    } else {
        T *gsi = grad_sig + row * hp.total + hp.off[i];
        block_matvec<T>(gtop, cache + (row * hp.total + hp.off[j]) * N + j, MatvecShape{1, wi, wj, 1, 0, 1, wi, 0, 0, N, 0}, red,
                        [&](int64_t, int64_t o, T r) { gsi[o] = r; });
    }
}

// The same products for many rows of a small layout, one block per row: the row's top-level gradient is built
// once in LDS as a dense d^N array (a listed top level is scattered into it, repeated words adding up) and all
// 2 (N - 1) products read it from there.  With thousands of rows the launch over (row, split, side) above is
// bound by reading each row's dense gradient 2 (N - 1) times from L2, and needs that array in memory first.
template <typename T>
__global__ void __launch_bounds__(kLogBlock) logsig_gather_top_rows_kernel(
    const T *__restrict__ logsig, const T *__restrict__ cache, const T *__restrict__ grad_logsig, T *grad_sig,
    T *R_all, HybridPlan hp, const int64_t *__restrict__ top_words, int64_t top_dense) {
    extern __shared__ __align__(16) unsigned char top_smem[];
    __shared__ T red[kLogBlock];
    T *gtop = reinterpret_cast<T *>(top_smem);
    const int N = hp.depth;
    const int64_t row = blockIdx.x;
    const T *lgs = logsig + row * hp.total;
    const T *gl = grad_logsig + row * hp.total + hp.off[N];
    if (hp.size[N] != top_dense) {  // a listed top level (possibly empty)
        for (int64_t i = threadIdx.x; i < top_dense; i += (int)blockDim.x) gtop[i] = T(0);
        __syncthreads();
        for (int64_t i = threadIdx.x; i < hp.size[N]; i += (int)blockDim.x) atomicAdd(&gtop[top_words[i]], gl[i]);
    } else {
        for (int64_t i = threadIdx.x; i < top_dense; i += (int)blockDim.x) gtop[i] = gl[i];
    }
    __syncthreads();
    int64_t wj = 1, wi = top_dense;
    for (int j = 1; j < N; ++j) {
        wj *= hp.d;
        wi /= hp.d;
        const int i = N - j;
        T *R = R_all + row * hp.lower + hp.off[j];
        block_matvec<T>(gtop, lgs + hp.off[i], MatvecShape{1, wj, wi, 1, 0, wi, 1, 0, 0, 1, 0}, red,
                        [&](int64_t, int64_t o, T r) { R[o] = r; });
        T *gsi = grad_sig + row * hp.total + hp.off[i];
        block_matvec<T>(gtop, cache + (row * hp.total + hp.off[j]) * N + j, MatvecShape{1, wi, wj, 1, 0, 1, wi, 0, 0, N, 0}, red,
                        [&](int64_t, int64_t o, T r) { gsi[o] = r; });
    }
}

// Levels below the top, one block per row, going down.  `a` ([lower columns][depth]) holds a_k: in LDS when the
// launch provides room for it (A_IN_LDS; the kernel is a chain of short dependent passes over `a`, so their
// latency is what it costs), else in the workspace.  `R` ([lower columns], workspace) are the top-level sums of
// logsig_gather_top_kernel, which has also stored the top-level part of the gradient in grad_sig.
// STAGED (with A_IN_LDS): everything else the passes read or update is brought to LDS in one burst of loads at the
// start (the gradient of the levels below the top with the upstream gradient already added, the log-signature and
// the cache rows of the levels 1 .. depth - 2), so that no pass waits for memory; the gradient goes back to memory
// at the end.  For calls of a few hundred rows at most, where a row's latency is all there is.
template <typename T, bool A_IN_LDS, bool STAGED = false>
__global__ void __launch_bounds__(kLogBlock) logsig_gather_kernel(const T *__restrict__ logsig,
                                                                  const T *__restrict__ cache,
                                                                  const T *__restrict__ grad_logsig, T *grad_sig,
                                                                  T *a_all, const T *__restrict__ R_all, HybridPlan hp,
                                                                  bool copy_top) {
    extern __shared__ __align__(16) unsigned char gather_smem[];
    __shared__ T red[kLogBlock];
    const int N = hp.depth;
    const int64_t row = blockIdx.x;
    const T *lgs = logsig + row * hp.total;
    const T *Cr = cache + row * hp.total * N;
    const T *gl = grad_logsig + row * hp.total;
    T *gs = grad_sig + row * hp.total;
    // the address space of `a` is fixed at compile time, so that its loads are LDS loads and not generic ones
    static_assert(A_IN_LDS || !STAGED, "the staged form keeps `a` in LDS too");
    T *a;
    if constexpr (A_IN_LDS) a = reinterpret_cast<T *>(gather_smem);
    else a = a_all + row * hp.lower * N;
    const T *R = R_all + row * hp.lower;
    const int64_t few = N >= 2 ? hp.off[N - 1] : 0;  // columns of the levels 1 .. N - 2
    const T *lgsp, *Crp;
    T *gsp;
    if constexpr (STAGED) {
        T *gs_l = a + hp.lower * N, *lgs_l = gs_l + hp.lower, *C_l = lgs_l + few;
        batched_rounds<4>(few, [&](int64_t i) { return lgs[i]; }, [&](int64_t i, T v) { lgs_l[i] = v; });
        batched_rounds<8>(few * N, [&](int64_t i) { return Cr[i]; }, [&](int64_t i, T v) { C_l[i] = v; });
        batched_rounds<8>(hp.lower, [&](int64_t i) { return gs[i] + gl[i]; }, [&](int64_t i, T v) { gs_l[i] = v; });
        lgsp = lgs_l;
        Crp = C_l;
        gsp = gs_l;
    } else {
        lgsp = lgs;
        Crp = Cr;
        gsp = gs;
    }
    int64_t width[kMaxDepth + 1];  // d^k
    width[0] = 1;
    for (int k = 1; k <= N; ++k) width[k] = width[k - 1] * hp.d;

    // a_k(w) starts from its top-level part, sum_v a_{k+1}(w v) L(v) = -f_{k+1} R(w); the top-level columns
    // of the gradient are g
    __shared__ T invf[kMaxDepth + 2];  // 1 / k!
    if (threadIdx.x == 0) {
        invf[0] = invf[1] = T(1);
        for (int k = 2; k <= N + 1; ++k) invf[k] = invf[k - 1] / T(k);
    }
    __syncthreads();
    batched_rounds<8>(hp.lower, [&](int64_t col) { return R[col]; }, [&](int64_t col, T r) {
        int n = 1;  // level of the column
        while (n < N - 1 && col >= hp.off[n + 1]) ++n;
        for (int m = 1; m <= N; ++m) a[col * N + m - 1] = m <= n ? -invf[m + 1] * r : T(0);
    });
    // (the launch over (row, split, side) has copied the top-level part already)
    if (copy_top)
        batched_rounds<8>(hp.size[N], [&](int64_t i) { return gl[hp.off[N] + i]; },
                          [&](int64_t i, T v) { gs[hp.off[N] + i] = v; });
    __threadfence_block();
    __syncthreads();

    const int BLK = (int)blockDim.x, tid = (int)threadIdx.x;
    for (int n = N - 1; n >= 1; --n) {
        T *an = a + hp.off[n] * N;
        T *gsn = gsp + hp.off[n];
        const int wn = (int)width[n];
        const int levels = N - 1 - n;  // levels between this one and the top
        if (levels > 0) {
            const int longest = (int)width[levels];
            // a_k(w) += sum_v a_{k+1}(w v) L(v), v over all those levels at once, k = 1..n (output = (k, w)).
            // When there are fewer outputs than threads, `parts` consecutive lanes of a wave share an output (lanes
            // along v, which is contiguous in a) and their partial sums meet through wave shuffles.
            {
                const int outputs = n * wn;
                int parts = 1;
                while (parts * 2 * outputs <= BLK && parts * 2 <= longest && parts * 2 <= kWave) parts *= 2;
                const int slots = BLK / parts, part = tid % parts, oloc = tid / parts;
                for (int o0 = 0; o0 < outputs; o0 += slots) {
                    const int oo = o0 + oloc;
                    const int bi = oo / wn, o = oo - bi * wn;
                    T acc = T(0);
                    if (oo < outputs) {
                        for (int i = 1; i <= levels; ++i) {
                            const int wi = (int)width[i];
                            const T *ap = a + (hp.off[n + i] + (int64_t)o * wi + part) * N + 1 + bi;
                            const T *bp = lgsp + hp.off[i] + part;
                            for (int k = part; k < wi; k += parts) {
                                acc += *ap * *bp;
                                ap += (int64_t)parts * N;
                                bp += parts;
                            }
                        }
                    }
                    for (int off = parts / 2; off >= 1; off /= 2) acc += __shfl_xor(acc, off);
                    if (part == 0 && oo < outputs) an[o * N + bi] += acc;
                }
            }
            // gradient(w) += sum_u sum_{k=2}^{|u|+1} a_k(u w) Q_{k-1}(u), u over the same levels (output = w; lanes
            // along w, which is contiguous in a; the parts of an output split the range of u)
            {
                int parts = 1;
                while (parts * 2 * wn <= BLK && parts * 2 <= longest) parts *= 2;
                const int slots = BLK / parts, part = tid / slots, oloc = tid % slots;
                for (int o0 = 0; o0 < wn; o0 += slots) {
                    const int o = o0 + oloc;
                    T acc = T(0);
                    if (o < wn) {
                        for (int j = 1; j <= levels; ++j) {
                            const int wj = (int)width[j];
                            const T *ap = a + (hp.off[n + j] + (int64_t)part * wn + o) * N + 1;
                            const T *bp = Crp + (hp.off[j] + part) * N;
                            for (int k = part; k < wj; k += parts) {
                                for (int m = 0; m < j; ++m) acc += ap[m] * bp[m];
                                ap += (int64_t)parts * wn * N;
                                bp += (int64_t)parts * N;
                            }
                        }
                    }
                    if (parts > 1) {
                        // the parts of an output are `slots` threads apart: those inside a wave meet through
                        // shuffles, the waves' sums in LDS
                        int left = parts, stride = slots;  // partial sums still apart, and by how many threads
                        if (slots < kWave && BLK % kWave == 0) {
                            for (int off = kWave / 2; off >= slots; off /= 2) acc += __shfl_xor(acc, off);
                            const int in_wave = kWave / slots < parts ? kWave / slots : parts;
                            left = parts / in_wave;
                            stride = kWave;
                        }
                        if (left > 1) {
                            red[tid] = acc;
                            __syncthreads();
                            if (part == 0 && o < wn) {
                                T total = T(0);
                                for (int q = 0; q < left; ++q) total += red[q * stride + oloc];
                                gsn[o] += total;
                            }
                            __syncthreads();
                        } else if (part == 0 && o < wn) {
                            gsn[o] += acc;
                        }
                    } else if (o < wn) {
                        gsn[o] += acc;
                    }
                }
            }
            __threadfence_block();
            __syncthreads();
        }
        // lam(w) = g(w) + a_1(w) + the sums above is the gradient of the word; a_k(w) -= lam(w) / k! for k >= 2
        for (int i = tid; i < wn; i += BLK) {
            const T lam = (STAGED ? T(0) : gl[hp.off[n] + i]) + an[i * N] + gsn[i];
            gsn[i] = lam;
            for (int k = 2; k <= n; ++k) an[i * N + k - 1] -= invf[k] * lam;
        }
        __threadfence_block();
        __syncthreads();
    }
    if constexpr (STAGED)
        for (int64_t i = threadIdx.x; i < hp.lower; i += (int)blockDim.x) gs[i] = gsp[i];
}

// dense[row][code of word e] += grad_logsig[row][top column e]; dense must be zero on entry
template <typename T>
__global__ void scatter_top_kernel(const T *__restrict__ grad_logsig, T *__restrict__ dense, HybridPlan hp,
                                   const int64_t *__restrict__ top_words, int64_t rows, int64_t top_dense) {
    // grid: x over the listed words, y over the rows
    const int64_t listed = hp.size[hp.depth];
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < listed; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t to = top_words[e], from = hp.off[hp.depth] + e;
        for (int64_t row = blockIdx.y; row < rows; row += gridDim.y)
            atomicAdd(&dense[row * top_dense + to], grad_logsig[row * hp.total + from]);
    }
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

namespace {
// one pass over all levels of all rows: the top level only reads the cache rows of the levels below it, so when
// it is large it gets a launch of its own, with its words dealt out to several blocks per row
template <typename T, bool STABLE, typename IDX>
hipError_t forward_pass_as(const T *sig, T *logsig, T *C, const HybridPlan &hp, int64_t rows, int64_t top_size,
                           const int64_t *top_words, hipStream_t stream) {
    const int depth = hp.depth;
    const int blk = logsig_block(hp.total, rows);
    int64_t slices = (top_size + 4 * blk - 1) / (4 * blk);
    if (slices > 16) slices = 16;
    if (depth < 2 || slices < 2) {
        hipLaunchKernelGGL((logsig_forward_kernel<T, STABLE, IDX>), dim3((unsigned)rows), dim3(blk), 0, stream, sig,
                           logsig, C, hp, top_words, 1, depth);
        return hipGetLastError();
    }
    hipLaunchKernelGGL((logsig_forward_kernel<T, STABLE, IDX>), dim3((unsigned)rows), dim3(blk), 0, stream, sig, logsig,
                       C, hp, top_words, 1, depth - 1);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((logsig_forward_kernel<T, STABLE, IDX>), dim3((unsigned)rows, (unsigned)slices), dim3(blk), 0,
                       stream, sig, logsig, C, hp, top_words, depth, depth);
    return hipGetLastError();
}

template <typename T, bool STABLE>
hipError_t forward_pass(const T *sig, T *logsig, T *C, const HybridPlan &hp, int64_t rows, int64_t top_size,
                        const int64_t *top_words, hipStream_t stream) {
    // 32-bit column arithmetic when every word code (below d^depth) and every cache column of a row fit
    const double codes = std::pow((double)hp.d, (double)hp.depth);
    const bool narrow = codes < 4294967296.0 && (double)hp.total * (double)hp.depth < 4294967296.0;
    if (narrow) return forward_pass_as<T, STABLE, uint32_t>(sig, logsig, C, hp, rows, top_size, top_words, stream);
    return forward_pass_as<T, STABLE, uint64_t>(sig, logsig, C, hp, rows, top_size, top_words, stream);
}
}  // namespace

// logsig and `cache` (the Q form) are always written; `powers` (the P cache of the reference), when not null,
// is written by a second pass and may be the same buffer as `cache`, which it then replaces.
template <typename T>
hipError_t launch_logsig_forward(const T *sig, T *logsig, T *cache, T *powers, int64_t rows, int64_t d, int depth,
                                 int64_t top_size, const int64_t *top_words, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    const HybridPlan hp = make_hybrid(d, depth, top_size, top_words);
    hipError_t e = forward_pass<T, true>(sig, logsig, cache, hp, rows, top_size, top_words, stream);
    if (e != hipSuccess || powers == nullptr) return e;
    return forward_pass<T, false>(sig, logsig, powers, hp, rows, top_size, top_words, stream);
}

// Workspace of the adjoint in elements of T: [a: rows x lower x depth][R, Q: rows x lower each][dense top gradient:
// rows x d^depth, only for a listed top level].  gather = false (scatter form) needs the first part only.
LogsigBackwardPlan logsig_backward_plan(size_t elem, int64_t rows, int64_t d, int depth, int64_t top_size) {
    LogsigBackwardPlan lp{};
    int64_t lower = 0, width = 1;
    for (int k = 1; k < depth; ++k) {
        width *= d;
        lower += width;
    }
    width *= d;  // d^depth (the caller has checked that it fits)
    lp.a_elems = rows * lower * depth;
    lp.q_elems = 0;
    lp.top_elems = 0;
    lp.top_dense = width;
    lp.gather = false;
    const bool forced_scatter = options().logsig_scatter != 0;
    const bool listed = top_size != width;
    // the dense copy of the top-level gradient must stay modest: 1 GiB
    const bool fits = (double)rows * (double)width * (double)elem <= 1073741824.0;
    // the gather form counts its products in 32 bits
    const bool small = (double)width * (double)depth < 2e9;
    if (depth >= 2 && !forced_scatter && (!listed || fits) && small && rows > 0) {
        lp.gather = true;
        lp.q_elems = rows * lower;  // R
        lp.top_elems = listed ? rows * width : 0;
    }
    return lp;
}

// logsig and cache are the outputs of launch_logsig_forward for the same signature
template <typename T>
hipError_t launch_logsig_backward(const T *logsig, const T *cache, const T *grad_logsig, T *grad_sig, T *workspace,
                                  int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                                  hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    const HybridPlan hp = make_hybrid(d, depth, top_size, top_words);
    const LogsigBackwardPlan lp = logsig_backward_plan(sizeof(T), rows, d, depth, top_size);
    const int blk = logsig_block(hp.total, rows);
    T *gradP = workspace;
    if (lp.gather) {
        T *R = gradP + lp.a_elems;
        hipError_t e = hipSuccess;
        // top-level products: with many rows of a small layout one block per row with the row's dense top-level
        // gradient in LDS; else one block per (row, split, side) over a dense copy of that gradient in memory
        const size_t top_bytes = (size_t)lp.top_dense * sizeof(T);
        bool copy_top = true;  // the lower-level kernel copies the top-level part of the gradient
        if (rows >= 256 && top_bytes <= 64 * 1024) {
            if (top_bytes > 32 * 1024) {
                e = allow_dynamic_lds<logsig_gather_top_rows_kernel<T>>(top_bytes);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(logsig_gather_top_rows_kernel<T>, dim3((unsigned)rows), dim3(blk), top_bytes, stream,
                               logsig, cache, grad_logsig, grad_sig, R, hp, top_words, lp.top_dense);
        } else {
            copy_top = false;  // (the launch over (row, split, side) does)
            const T *gtop = grad_logsig + hp.off[depth];
            int64_t top_stride = hp.total;  // dense top level: read in place, row stride of the gradient
            if (lp.top_elems > 0) {
                T *dense = R + lp.q_elems;
                e = launch_fill_zero<T>(dense, lp.top_elems, stream);
                if (e != hipSuccess) return e;
                const int64_t n = rows * top_size;
                if (n > 0) {
                    hipLaunchKernelGGL(scatter_top_kernel<T>, columns_by_rows_grid(top_size, rows), dim3(256), 0, stream,
                                       grad_logsig, dense, hp, top_words, rows, lp.top_dense);
                    e = hipGetLastError();
                    if (e != hipSuccess) return e;
                }
                gtop = dense;
                top_stride = lp.top_dense;
            }
            hipLaunchKernelGGL(logsig_gather_top_kernel<T>, dim3((unsigned)rows, (unsigned)(depth - 1), 2),
                               dim3(kLogBlock), 0, stream, logsig, cache, gtop, grad_sig, R, hp, top_stride,
                               grad_logsig);
        }
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        // the adjoint of the cache goes to LDS when a block's share of it fits beside the static arrays
        const size_t a_bytes = (size_t)hp.lower * (size_t)depth * sizeof(T);
        const bool a_in_lds = a_bytes <= 144 * 1024;
        const int64_t few = depth >= 2 ? hp.off[depth - 1] : 0;
        const size_t staged_bytes = a_bytes + (size_t)(hp.lower + few * (1 + depth)) * sizeof(T);
        if (a_in_lds && rows <= 512 && staged_bytes <= 150 * 1024) {
            if (staged_bytes > 32 * 1024) {
                e = allow_dynamic_lds<logsig_gather_kernel<T, true, true>>(staged_bytes);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL((logsig_gather_kernel<T, true, true>), dim3((unsigned)rows), dim3(blk), staged_bytes,
                               stream, logsig, cache, grad_logsig, grad_sig, gradP, (const T *)R, hp, copy_top);
        } else if (a_in_lds) {
            if (a_bytes > 32 * 1024) {
                e = allow_dynamic_lds<logsig_gather_kernel<T, true>>(a_bytes);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL((logsig_gather_kernel<T, true>), dim3((unsigned)rows), dim3(blk), a_bytes, stream,
                               logsig, cache, grad_logsig, grad_sig, gradP, (const T *)R, hp, copy_top);
        } else {
            hipLaunchKernelGGL((logsig_gather_kernel<T, false>), dim3((unsigned)rows), dim3(blk), 0, stream, logsig,
                               cache, grad_logsig, grad_sig, gradP, (const T *)R, hp, copy_top);
        }
        return hipGetLastError();
    }
    const int64_t lds_cols = lds_columns(d, depth, sizeof(T), 32 * 1024);
    const size_t lds_bytes = (size_t)lds_cols * (size_t)(depth + 1) * sizeof(T);
    hipLaunchKernelGGL(logsig_backward_kernel<T>, dim3((unsigned)rows), dim3(blk), lds_bytes, stream, logsig, cache,
                       grad_logsig, grad_sig, gradP, hp, top_words, lds_cols);
    return hipGetLastError();
}

#define PSIG_INSTANTIATE(T)                                                                                       \
    template hipError_t launch_logsig_forward<T>(const T *, T *, T *, T *, int64_t, int64_t, int, int64_t,        \
                                                 const int64_t *, hipStream_t);                                   \
    template hipError_t launch_logsig_backward<T>(const T *, const T *, const T *, T *, T *, int64_t, int64_t, int, \
                                                  int64_t, const int64_t *, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

}  // namespace psig
