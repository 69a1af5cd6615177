// General signature kernels: one lane per requested word, any path dimension, any depth <= 12,
// any word projection, any windows.  These are the kernels every call can fall back to; the
// register-tiled dense kernels in dense_kernels.hip take over for the shapes they are built for.
//
// A lane that owns the word w = (w_1..w_n) carries the signature values of the prefixes of w
// (a chain of n+1 numbers) and sweeps the window once.  Per increment it evaluates, for every
// target level m = n..1, the Horner chain
//     s_1 = 1/m,  tmp_j = p_j + s_j * dx[w_j],  s_{j+1} = tmp_j / (m - j),   p_m += s_m * dx[w_m]
// which is S <- S (x) exp(dx) restricted to the chain (reference: src/pathsig/forward/sig_kernels.cu:129-154).
// The backward lane carries the chain rolled back with exp(-dx) and the adjoint of the chain, and
// back-propagates through the same Horner chains; this needs O(n^2) work per increment
// (the reference assembles prefix x segment x suffix products in O(n^3),
// src/pathsig/backward/sig_backward_kernels.cu:204-253).  Increments of a tile of time steps are
// staged once per block in LDS; per-letter gradient sums are collected in LDS and flushed to the
// per-increment accumulator with one atomic per (step, letter) per block.
#include "common.hpp"
#include "words_common.hpp"

namespace psig {

namespace {

constexpr int kBlock = 256;

template <typename T, int DEG>
__device__ void forward_body(const T *__restrict__ path, T *__restrict__ sig, const SigShape &shape,
                             const LevelPlan &plan, const int64_t *__restrict__ codes, int64_t row, int64_t blk_in_level,
                             int tile, T *sdx) {
    const int tid = threadIdx.x;
    const int64_t d = shape.d;
    const int64_t word_idx = blk_in_level * kBlock + tid;
    const bool active = word_idx < plan.size[DEG];
    uint64_t code = 0;
    if (active) code = plan.code_off[DEG] >= 0 ? (uint64_t)codes[plan.code_off[DEG] + word_idx] : (uint64_t)word_idx;
    int l[DEG];
    decode_letters<DEG>(code, (uint64_t)d, l);

    const int64_t b = row / shape.W, w = row - b * shape.W;
    const WindowSpan span = window_span(shape, w);
    const T *x = path + (b * shape.L + span.start) * d;

    T p[DEG + 1];
    p[0] = T(1);
#pragma unroll
    for (int k = 1; k <= DEG; ++k) p[k] = T(0);

    for (int64_t t0 = 0; t0 < span.steps; t0 += tile) {
        const int nt = (int)((span.steps - t0) < tile ? (span.steps - t0) : tile);
        const T *xw = x + t0 * d;
        __syncthreads();
        for (int64_t idx = tid; idx < (int64_t)nt * d; idx += kBlock) sdx[idx] = xw[idx + d] - xw[idx];
        __syncthreads();
        if (active) {
            for (int tt = 0; tt < nt; ++tt) {
                const T *dxr = sdx + (int64_t)tt * d;
                T dl[DEG];
#pragma unroll
                for (int k = 0; k < DEG; ++k) dl[k] = dxr[l[k]];
                T dq[DEG][DEG];
                scale_letters<T, DEG>(dl, dq);
                chain_step<T, DEG, DEG, true>(p, dq);
            }
        }
    }
    if (active) {
        sig[row * plan.sig_size + plan.out_off[DEG] + word_idx] = p[DEG];
        if (plan.keep && plan.keep_off[DEG] >= 0) {
            T *kept = (T *)plan.keep + row * plan.keep_size + plan.keep_off[DEG] + word_idx * (DEG - 1);
#pragma unroll
            for (int k = 1; k < DEG; ++k) kept[k - 1] = p[k];
        }
    }
}

template <typename T, int MAXDEG>
__global__ void __launch_bounds__(kBlock) words_forward_kernel(const T *__restrict__ path, T *__restrict__ sig,
                                                               SigShape shape, LevelPlan plan,
                                                               const int64_t *__restrict__ codes, int tile) {
    extern __shared__ __align__(16) unsigned char smem[];
    T *sdx = reinterpret_cast<T *>(smem);
    const int64_t per_row = plan.block_begin[plan.depth + 1];
    const int64_t row = (int64_t)blockIdx.x / per_row;
    const int64_t blk = (int64_t)blockIdx.x - row * per_row;
    const int deg = find_level(plan, blk);
    const int64_t bl = blk - plan.block_begin[deg];
    switch (deg) {
#define PSIG_CASE(N)                                                                                  \
    case N:                                                                                           \
        if constexpr (N <= MAXDEG) forward_body<T, N>(path, sig, shape, plan, codes, row, bl, tile, sdx); \
        break;
        PSIG_CASE(1) PSIG_CASE(2) PSIG_CASE(3) PSIG_CASE(4) PSIG_CASE(5) PSIG_CASE(6)
        PSIG_CASE(7) PSIG_CASE(8) PSIG_CASE(9) PSIG_CASE(10) PSIG_CASE(11) PSIG_CASE(12)
#undef PSIG_CASE
        default: break;
    }
}

// The backward runs one wave per block.  For path dimensions up to kSortedMax the per-letter sums of an
// increment go through a list that is built once per block: the (lane, position) pairs of the wave's
// words sorted by letter.  Every step each lane drops its per-position gradients into LDS, then adds up
// DEG consecutive entries of the sorted list (mostly one letter, so mostly one LDS add per lane).
constexpr int kBwdBlock = kWave;
constexpr int kSortedMax = 64;

template <typename T, int DEG>
__device__ void backward_body(const T *__restrict__ path, const T *__restrict__ sig, const T *__restrict__ grad_sig,
                              double *__restrict__ grad_inc, const SigShape &shape, const LevelPlan &plan,
                              const int64_t *__restrict__ codes, int64_t row, int64_t blk_in_level, int tile, T *sdx,
                              T *sacc, T *sval, int *sorder, int *scnt) {
    const int lane = threadIdx.x;
    const int64_t d = shape.d;
    const int64_t word_idx = blk_in_level * kBwdBlock + lane;
    const bool active = word_idx < plan.size[DEG];
    uint64_t code = 0;
    if (active) code = plan.code_off[DEG] >= 0 ? (uint64_t)codes[plan.code_off[DEG] + word_idx] : (uint64_t)word_idx;
    int l[DEG];
    decode_letters<DEG>(code, (uint64_t)d, l);
    const bool sorted = d <= kSortedMax;

    // entries of the sorted list this lane adds up: source slot in sval, letter
    int src[DEG], let[DEG];
    if (sorted) {
        for (int i = lane; i < (int)d; i += kBwdBlock) scnt[i] = 0;
        __syncthreads();
        int pos[DEG];
#pragma unroll
        for (int k = 0; k < DEG; ++k) pos[k] = atomicAdd(&scnt[l[k]], 1);
        __syncthreads();
        if (lane == 0) {
            int run = 0;
            for (int a = 0; a < (int)d; ++a) {
                const int c = scnt[a];
                scnt[a] = run;
                run += c;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < DEG; ++k) sorder[scnt[l[k]] + pos[k]] = (l[k] << 16) | (k * kBwdBlock + lane);
        __syncthreads();
#pragma unroll
        for (int e = 0; e < DEG; ++e) {
            const int o = sorder[lane * DEG + e];
            src[e] = o & 0xffff;
            let[e] = o >> 16;
        }
    }
    // Usual case: the DEG consecutive entries of every lane cover at most two letters.  Then a lane needs
    // two sums (entries of its first letter, the rest) and at most two LDS adds per step, without branches
    // inside the entry loop.
    T first_mask[DEG];
    int changes = 0;
#pragma unroll
    for (int e = 0; e < DEG; ++e) {
        if (e > 0 && sorted && let[e] != let[e - 1]) ++changes;
        first_mask[e] = (sorted && let[e] == let[0]) ? T(1) : T(0);
    }
    const bool two_runs = sorted && __all(changes <= 1);

    const int64_t b = row / shape.W, w = row - b * shape.W;
    const WindowSpan span = window_span(shape, w);
    const T *x = path + (b * shape.L + span.start) * d;
    double *ginc = grad_inc + (b * (shape.L - 1) + span.start) * d;
    const T *srow = sig + row * plan.sig_size;

    // chain of prefix values at the right end of the window (levels < DEG)
    T p[DEG + 1];
    p[0] = T(1);
#pragma unroll
    for (int k = 1; k <= DEG; ++k) p[k] = T(0);
    if (plan.from_saved[DEG]) {
        if (active) {
            uint64_t off = 0, width = (uint64_t)d, pref = 0;
#pragma unroll
            for (int k = 1; k < DEG; ++k) {
                pref = pref * (uint64_t)d + (uint64_t)l[k - 1];
                p[k] = srow[off + pref];
                off += width;
                width *= (uint64_t)d;
            }
        }
    } else if (DEG > 1 && plan.keep && plan.keep_off[DEG] >= 0) {
        // the forward of this call kept the chain
        if (active) {
            const T *kept = (const T *)plan.keep + row * plan.keep_size + plan.keep_off[DEG] + word_idx * (DEG - 1);
#pragma unroll
            for (int k = 1; k < DEG; ++k) p[k] = kept[k - 1];
        }
    } else if (DEG > 1) {
        for (int64_t t0 = 0; t0 < span.steps; t0 += tile) {
            const int nt = (int)((span.steps - t0) < tile ? (span.steps - t0) : tile);
            const T *xw = x + t0 * d;
            __syncthreads();
            for (int64_t idx = lane; idx < (int64_t)nt * d; idx += kBwdBlock) sdx[idx] = xw[idx + d] - xw[idx];
            __syncthreads();
            for (int tt = 0; tt < nt; ++tt) {
                const T *dxr = sdx + (int64_t)tt * d;
                T dl[DEG];
#pragma unroll
                for (int k = 0; k < DEG; ++k) dl[k] = dxr[l[k]];
                T dq[DEG][DEG];
                scale_letters<T, DEG>(dl, dq);
                chain_step<T, DEG, DEG - 1, true>(p, dq);
            }
        }
    }

    // adjoint of the chain: h[k] = dL/dS(w_1..w_k) as far as this word contributes
    T h[DEG + 1];
#pragma unroll
    for (int k = 0; k <= DEG; ++k) h[k] = T(0);
    h[DEG] = active ? grad_sig[row * plan.sig_size + plan.out_off[DEG] + word_idx] : T(0);

    const int64_t ntiles = (span.steps + tile - 1) / tile;
    for (int64_t ti = ntiles - 1; ti >= 0; --ti) {
        const int64_t t0 = ti * tile;
        const int nt = (int)((span.steps - t0) < tile ? (span.steps - t0) : tile);
        const T *xw = x + t0 * d;
        __syncthreads();
        for (int64_t idx = lane; idx < (int64_t)nt * d; idx += kBwdBlock) {
            sdx[idx] = xw[idx + d] - xw[idx];
            sacc[idx] = T(0);
        }
        __syncthreads();
        for (int tt = nt - 1; tt >= 0; --tt) {
            const T *dxr = sdx + (int64_t)tt * d;
            T *acc = sacc + (int64_t)tt * d;
            T dl[DEG];
#pragma unroll
            for (int k = 0; k < DEG; ++k) dl[k] = dxr[l[k]];
            // S_t = S_{t+1} (x) exp(-dx_t) on the chain (levels < DEG are all the adjoint needs)
            T dq[DEG][DEG];
            scale_letters<T, DEG>(dl, dq);
            chain_step<T, DEG, DEG - 1, false>(p, dq);
            T gl[DEG];
            chain_step_adjoint<T, DEG>(p, h, dl, dq, gl);
            if (sorted) {
                T *val = sval + (tt & 1) * (DEG * kBwdBlock);  // two buffers: one barrier per step is enough
#pragma unroll
                for (int k = 0; k < DEG; ++k) val[k * kBwdBlock + lane] = gl[k];
                __syncthreads();
                if (two_runs) {
                    T total = T(0), head = T(0);
#pragma unroll
                    for (int e = 0; e < DEG; ++e) {
                        const T v = val[src[e]];
                        total += v;
                        head = fma_t<T>(first_mask[e], v, head);
                    }
                    const T tail = total - head;
                    if (head != T(0)) atomicAdd(&acc[let[0]], head);
                    if (tail != T(0)) atomicAdd(&acc[let[DEG - 1]], tail);
                } else {
                    T run = T(0);
#pragma unroll
                    for (int e = 0; e < DEG; ++e) {
                        run += val[src[e]];
                        const bool last = (e == DEG - 1) || (let[e + 1 < DEG ? e + 1 : e] != let[e]);
                        if (last) {
                            if (run != T(0)) atomicAdd(&acc[let[e]], run);
                            run = T(0);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int k = 0; k < DEG; ++k)
                    if (gl[k] != T(0)) atomicAdd(&acc[l[k]], gl[k]);
            }
        }
        __syncthreads();
        for (int64_t idx = lane; idx < (int64_t)nt * d; idx += kBwdBlock) {
            const T v = sacc[idx];
            // one term per block of words: summed in fp64, because a dense level of millions of words adds tens of
            // thousands of them to one cell (fp32 there: 2e-5 to 3e-5 of the largest gradient lost at (8,8))
            if (v != T(0)) atomicAdd(&ginc[t0 * d + idx], (double)v);
        }
    }
}

// MAXDEG bounds the word lengths compiled into one kernel: the register budget of a kernel is that of its
// longest chain, so shallow signatures get a kernel with more waves per SIMD.
template <typename T, int MAXDEG>
__global__ void __launch_bounds__(kBwdBlock) words_backward_kernel(const T *__restrict__ path, const T *__restrict__ sig,
                                                                   const T *__restrict__ grad_sig,
                                                                   double *__restrict__ grad_inc, SigShape shape,
                                                                   LevelPlan plan, const int64_t *__restrict__ codes,
                                                                   int tile) {
    extern __shared__ __align__(16) unsigned char smem[];
    T *sdx = reinterpret_cast<T *>(smem);
    T *sacc = sdx + (int64_t)tile * shape.d;
    T *sval = sacc + (int64_t)tile * shape.d;
    int *sorder = reinterpret_cast<int *>(sval + 2 * plan.depth * kBwdBlock);
    int *scnt = sorder + plan.depth * kBwdBlock;
    const int64_t per_row = plan.block_begin[plan.depth + 1];
    const int64_t row = (int64_t)blockIdx.x / per_row;
    const int64_t blk = (int64_t)blockIdx.x - row * per_row;
    const int deg = find_level(plan, blk);
    const int64_t bl = blk - plan.block_begin[deg];
    switch (deg) {
#define PSIG_CASE(N)                                                                                              \
    case N:                                                                                                       \
        if constexpr (N <= MAXDEG)                                                                                \
            backward_body<T, N>(path, sig, grad_sig, grad_inc, shape, plan, codes, row, bl, tile, sdx, sacc, sval, \
                                sorder, scnt);                                                                    \
        break;
        PSIG_CASE(1) PSIG_CASE(2) PSIG_CASE(3) PSIG_CASE(4) PSIG_CASE(5) PSIG_CASE(6)
        PSIG_CASE(7) PSIG_CASE(8) PSIG_CASE(9) PSIG_CASE(10) PSIG_CASE(11) PSIG_CASE(12)
#undef PSIG_CASE
        default: break;
    }
}

template <typename T>
__global__ void fill_zero_kernel(T *__restrict__ ptr, int64_t n) {
    zero_span<T>(ptr, n, (int64_t)blockIdx.x * blockDim.x + threadIdx.x, (int64_t)gridDim.x * blockDim.x);
}

// dL/dx[t] = dL/d(dx[t-1]) - dL/d(dx[t]) with one-sided ends
// (reference: src/pathsig/backward/sig_backward_kernels.cu:347-377; 64-bit indices here)
// (TI: type of the per-increment sums, fp64 behind the word-per-lane backward)
// Grid: x over the L * d values of a path, y over the paths (no division by L * d; the one by d is a 32-bit
// division when L * d fits 31 bits, and 64-bit divisions are a hundred instructions each).
template <typename TI, typename T>
__global__ void increments_to_path_kernel(const TI *__restrict__ ginc, T *__restrict__ gpath, int64_t B, int64_t L,
                                          int64_t d) {
    const int64_t per_path = L * d;
    const bool narrow = per_path < (int64_t(1) << 31);
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < per_path; j += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = narrow ? (int64_t)((uint32_t)j / (uint32_t)d) : j / d;
        const int64_t a = j - t * d;
        for (int64_t b = blockIdx.y; b < B; b += gridDim.y) {
            const TI *g = ginc + b * (L - 1) * d + a;
            const TI left = t > 0 ? g[(t - 1) * d] : TI(0);
            const TI right = t < L - 1 ? g[t * d] : TI(0);
            gpath[b * per_path + j] = (T)(left - right);
        }
    }
}

// Column j of the projected layout <-> its column in the dense layout (same rule as the forward
// kernels: dense levels map to themselves, listed levels go through their codes).
struct ColumnMap {
    int depth;
    int64_t out_off[kMaxDepth + 2];    // first projected column of level k; [depth+1] = projected size
    int64_t code_off[kMaxDepth + 1];   // offset into the code array, < 0 for dense levels
    int64_t dense_off[kMaxDepth + 1];  // first dense column of level k
    int64_t dense_size;
};

__device__ __forceinline__ int64_t dense_column(const ColumnMap &m, const int64_t *__restrict__ codes, int64_t col) {
    int k = 1;
    while (k < m.depth && col >= m.out_off[k + 1]) ++k;
    const int64_t j = col - m.out_off[k];
    const int64_t code = m.code_off[k] >= 0 ? codes[m.code_off[k] + j] : j;
    return m.dense_off[k] + code;
}

template <typename T>
__global__ void gather_columns_kernel(const T *__restrict__ dense, T *__restrict__ out, ColumnMap m,
                                      const int64_t *__restrict__ codes, int64_t rows) {
    // grid: x over the projected columns, y over the rows (a thread looks its column up once)
    const int64_t width = m.out_off[m.depth + 1];
    for (int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; col < width; col += (int64_t)gridDim.x * blockDim.x) {
        const int64_t from = dense_column(m, codes, col);
        for (int64_t row = blockIdx.y; row < rows; row += gridDim.y) out[row * width + col] = dense[row * m.dense_size + from];
    }
}

// dense must be zero on entry; repeated columns add up
template <typename T>
__global__ void scatter_columns_kernel(const T *__restrict__ grad, T *__restrict__ dense, ColumnMap m,
                                       const int64_t *__restrict__ codes, int64_t rows) {
    const int64_t width = m.out_off[m.depth + 1];
    for (int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; col < width; col += (int64_t)gridDim.x * blockDim.x) {
        const int64_t to = dense_column(m, codes, col);
        for (int64_t row = blockIdx.y; row < rows; row += gridDim.y)
            atomicAdd(&dense[row * m.dense_size + to], grad[row * width + col]);
    }
}

ColumnMap make_column_map(const LevelPlan &plan, int64_t d) {
    ColumnMap m{};
    m.depth = plan.depth;
    int64_t off = 0, width = 1;
    for (int k = 1; k <= plan.depth; ++k) {
        width *= d;
        m.out_off[k] = plan.out_off[k];
        m.code_off[k] = plan.code_off[k];
        m.dense_off[k] = off;
        off += width;
    }
    m.out_off[plan.depth + 1] = plan.sig_size;
    m.dense_size = off;
    return m;
}

// number of increments staged per tile so that `arrays` LDS arrays of tile * d elements fit `budget` bytes
int pick_tile(int64_t d, size_t elem, int64_t max_steps, int arrays, int64_t budget) {
    int64_t tile = budget / arrays / (int64_t)(d * elem);
    if (tile < 1) tile = 1;
    if (tile > 128) tile = 128;
    if (tile > max_steps) tile = max_steps;
    return (int)(tile < 1 ? 1 : tile);
}

}  // namespace

template <typename T>
hipError_t launch_words_forward(const T *path, T *sig, const SigShape &shape, const LevelPlan &plan,
                                const int64_t *codes, hipStream_t stream) {
    const int64_t per_row = plan.block_begin[plan.depth + 1];
    const int64_t blocks = per_row * shape.B * shape.W;
    if (blocks == 0) return hipSuccess;
    const int tile = pick_tile(shape.d, sizeof(T), shape.L - 1, 1, 16384);
    const size_t lds = (size_t)tile * shape.d * sizeof(T);
#define PSIG_LAUNCH(MAXDEG)                                                                                    \
    hipLaunchKernelGGL((words_forward_kernel<T, MAXDEG>), dim3((unsigned)blocks), dim3(kBlock), lds, stream, path, sig, \
                       shape, plan, codes, tile)
    if (plan.depth <= 4) PSIG_LAUNCH(4);
    else if (plan.depth <= 8) PSIG_LAUNCH(8);
    else PSIG_LAUNCH(12);
#undef PSIG_LAUNCH
    return hipGetLastError();
}

template <typename T>
hipError_t launch_words_backward(const T *path, const T *sig, const T *grad_sig, double *grad_inc, const SigShape &shape,
                                 const LevelPlan &plan_in, const int64_t *codes, hipStream_t stream) {
    // same levels, blocks of one wave
    LevelPlan plan = plan_in;
    int64_t per_row = 0;
    for (int k = 1; k <= plan.depth; ++k) {
        plan.block_begin[k] = per_row;
        per_row += (plan.size[k] + kBwdBlock - 1) / kBwdBlock;
    }
    plan.block_begin[plan.depth + 1] = per_row;
    const int64_t blocks = per_row * shape.B * shape.W;
    if (blocks == 0) return hipSuccess;
    if (blocks >= (int64_t(1) << 31)) return hipErrorInvalidValue;
    // one wave per block: a small tile keeps many blocks resident on a CU
    const int tile = pick_tile(shape.d, sizeof(T), shape.L - 1, 2, 4096);
    const size_t lds = (size_t)2 * tile * shape.d * sizeof(T) + (size_t)2 * plan.depth * kBwdBlock * sizeof(T) +
                       (size_t)plan.depth * kBwdBlock * sizeof(int) + (size_t)(kSortedMax + 1) * sizeof(int);
#define PSIG_LAUNCH(MAXDEG)                                                                                       \
    hipLaunchKernelGGL((words_backward_kernel<T, MAXDEG>), dim3((unsigned)blocks), dim3(kBwdBlock), lds, stream, path, \
                       sig, grad_sig, grad_inc, shape, plan, codes, tile)
    if (plan.depth <= 3) PSIG_LAUNCH(3);
    else if (plan.depth <= 4) PSIG_LAUNCH(4);
    else if (plan.depth <= 6) PSIG_LAUNCH(6);
    else if (plan.depth <= 8) PSIG_LAUNCH(8);
    else PSIG_LAUNCH(12);
#undef PSIG_LAUNCH
    return hipGetLastError();
}

template <typename T>
hipError_t launch_fill_zero(T *ptr, int64_t n, hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n / (16 / (int64_t)sizeof(T)) + 255) / 256 + 1;  // one thread per 16-byte piece
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_zero_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, ptr, n);
    return hipGetLastError();
}

template <typename TI, typename T>
hipError_t launch_increments_to_path(const TI *grad_inc, T *grad_path, int64_t B, int64_t L, int64_t d,
                                     hipStream_t stream) {
    const int64_t n = B * L * d;
    if (n <= 0) return hipSuccess;
    const dim3 grid = columns_by_rows_grid(L * d, B);
    hipLaunchKernelGGL((increments_to_path_kernel<TI, T>), grid, dim3(256), 0, stream, grad_inc, grad_path, B, L, d);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_gather_columns(const T *dense, T *out, const LevelPlan &plan, int64_t d, const int64_t *codes,
                                 int64_t rows, hipStream_t stream) {
    const int64_t n = rows * plan.sig_size;
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(gather_columns_kernel<T>, columns_by_rows_grid(plan.sig_size, rows), dim3(256), 0, stream, dense, out,
                       make_column_map(plan, d), codes, rows);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_scatter_columns(const T *grad, T *dense, const LevelPlan &plan, int64_t d, const int64_t *codes,
                                  int64_t rows, hipStream_t stream) {
    const int64_t n = rows * plan.sig_size;
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(scatter_columns_kernel<T>, columns_by_rows_grid(plan.sig_size, rows), dim3(256), 0, stream, grad, dense,
                       make_column_map(plan, d), codes, rows);
    return hipGetLastError();
}

#define PSIG_INSTANTIATE(T)                                                                                         \
    template hipError_t launch_gather_columns<T>(const T *, T *, const LevelPlan &, int64_t, const int64_t *,       \
                                                 int64_t, hipStream_t);                                             \
    template hipError_t launch_scatter_columns<T>(const T *, T *, const LevelPlan &, int64_t, const int64_t *,      \
                                                  int64_t, hipStream_t);                                            \
    template hipError_t launch_words_forward<T>(const T *, T *, const SigShape &, const LevelPlan &, const int64_t *, \
                                                hipStream_t);                                                       \
    template hipError_t launch_words_backward<T>(const T *, const T *, const T *, double *, const SigShape &,       \
                                                 const LevelPlan &, const int64_t *, hipStream_t);                  \
    template hipError_t launch_fill_zero<T>(T *, int64_t, hipStream_t);                                             \
    template hipError_t launch_increments_to_path<T, T>(const T *, T *, int64_t, int64_t, int64_t, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE
template hipError_t launch_increments_to_path<double, float>(const double *, float *, int64_t, int64_t, int64_t,
                                                               hipStream_t);

}  // namespace psig
