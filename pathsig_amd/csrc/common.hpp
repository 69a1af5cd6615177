// Shared declarations of libpathsig_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "pathsig_hip.h"

namespace psig {

constexpr int kMaxDepth = PATHSIG_MAX_DEPTH;
constexpr int kWave = 64;

// Per-level output plan of one signature call, passed to kernels by value.
// Level k has size[k] words whose first output column is out_off[k]; their codes start at
// code_off[k] in the encoded-word array, or the level is dense (code == column index) when
// code_off[k] < 0.  block_begin[k] is the first block (within one row of blocks) that works on
// level k; block_begin[depth + 1] is the number of blocks per row.
struct LevelPlan {
    int depth;
    int from_saved[kMaxDepth + 1];  // backward: prefixes of level k can be read from the saved signature
    int64_t size[kMaxDepth + 1];
    int64_t out_off[kMaxDepth + 1];
    int64_t code_off[kMaxDepth + 1];
    int64_t block_begin[kMaxDepth + 2];
    int64_t sig_size;
    // What a forward can keep for the backward of the same call: the prefix values S(w_1..w_k), k < |w|, of
    // the words of every level whose prefixes are not all in the saved signature (from_saved == 0), which the
    // backward would otherwise recompute with a forward sweep.  Row layout: keep_off[level] + word * (level - 1)
    // + (k - 1); keep_off is -1 for levels that keep nothing, keep_size the elements per row.
    int64_t keep_off[kMaxDepth + 1];
    int64_t keep_size;
    void *keep;  // device buffer [rows, keep_size] of the call's element type, or nullptr (nothing kept)
};

// Geometry of one signature call.
struct SigShape {
    int64_t B, L, d, W;  // W = 1 and windows == nullptr when no windows are given
    const int32_t *windows;
};

void set_error(const char *fmt, ...);

// Tuning switches of the library (pathsig_set_option).  Their initial values come from the environment, read
// once when the first call needs them; nothing on a call's path reads the environment.
struct Options {
    int64_t chunks;          // forced number of time chunks of the register-tiled kernels (0: chosen per call)
    int64_t letter_bounds;   // embedded projections leave out top-level words by letter bounds (default 1)
    int64_t logsig_scatter;  // log-signature adjoint in its scatter form even where the gather form fits (default 0)
    int64_t batch_tile;      // cap on the increments per tile of the lanes-on-paths backward (0: no cap)
    int64_t embed_share;     // a projection runs on the register-tiled kernels when its top level keeps at least
                             // 1/embed_share of the dense one (0: never; -1: the library's own rule)
    int64_t tiled;           // 0: every call takes the per-word kernels, whatever its shape (default 1)
    int64_t deep_fp64;       // 1 (default): fp32 backward calls of depth 9 and more run their sweep in fp64 (see
                             // backward_in_fp64 in api.hip); 0: in fp32 like every other call
    int64_t grouped;         // 1 (default): a keeping fp32 forward hands the chunk products over by groups of four
                             // chunks where that is compiled (DenseChoice::grouped); 0: one scan over all chunks
};
const Options &options();

#if defined(__HIPCC__)
// Wave-wide sum of one value per lane; the total is valid in lane 63 only.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add_c(float v) {
    // lanes outside ROW_MASK, and lanes whose source lane is invalid, add zero
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

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, which on
// this hardware means waiting for every outstanding global load, including prefetches that are meant to
// stay in flight across the barrier.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// the same lane moves for a double: both halves go through the DPP move, then one fp64 add
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_add_c(double v) {
    const long long bits = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(bits & 0xffffffffll), CTRL, ROW_MASK, 0xF, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(bits >> 32), CTRL, ROW_MASK, 0xF, false);
    const long long moved = ((long long)hi << 32) | (long long)(unsigned)lo;
    return v + __builtin_bit_cast(double, moved);
}

__device__ __forceinline__ double wave_total(double v) {
    v = dpp_add_c<0xB1, 0xF>(v);
    v = dpp_add_c<0x4E, 0xF>(v);
    v = dpp_add_c<0x141, 0xF>(v);
    v = dpp_add_c<0x140, 0xF>(v);
    v = dpp_add_c<0x142, 0xA>(v);
    v = dpp_add_c<0x143, 0xC>(v);
    return v;
}
#endif

#if defined(__HIPCC__)
// A kernel that asks for more dynamic LDS than the default limit needs that limit raised first.  Done once per
// kernel and device (the table belongs to the kernel: it is a template argument, not a function argument, since
// kernels of one signature share a pointer type), and again only when a call asks for more than any before it.
template <auto Kernel>
hipError_t allow_dynamic_lds(size_t bytes) {
    static std::atomic<size_t> allowed[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && allowed[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes);
    if (e == hipSuccess && tracked) allowed[dev].store(bytes, std::memory_order_release);
    return e;
}
#endif

template <typename T>
struct Recip {
    // 1/k for k = 1..12 as compile-time constants of type T
    __host__ __device__ static constexpr T of(int k) { return T(1) / T(k); }
};

// Launchers implemented in the kernel translation units.  Each returns hipSuccess or the launch error.
template <typename T>
hipError_t launch_words_forward(const T *path, T *sig, const SigShape &shape, const LevelPlan &plan,
                                const int64_t *codes, hipStream_t stream);
// (its per-increment sums are fp64 whatever T is: one term per block of words and cell)
template <typename T>
hipError_t launch_words_backward(const T *path, const T *sig, const T *grad_sig, double *grad_inc,
                                 const SigShape &shape, const LevelPlan &plan, const int64_t *codes, hipStream_t stream);
// backward with lanes on paths (batch_kernels.hip): same contract as launch_words_backward; usable for
// batches of at least a dozen paths of moderate dimension
bool batch_backward_usable(size_t elem, int64_t B, int64_t d, int64_t W);
// (ACC: type of the per-increment sums, T or, for fp32 calls where batch_wide_sums says so, double)
bool batch_wide_sums(size_t elem, const LevelPlan &plan);
template <typename T, typename ACC>
hipError_t launch_batch_backward(const T *path, const T *sig, const T *grad_sig, ACC *grad_inc, const SigShape &shape,
                                 const LevelPlan &plan, const int64_t *codes, hipStream_t stream);
template <typename T>
hipError_t launch_fill_zero(T *ptr, int64_t n, hipStream_t stream);
// Grid of the kernels that run x over the columns of a row (256 threads to a block, a thread per column while
// that keeps x below 2^16) and y over the rows, in strides of gridDim.y once the grid holds enough blocks to fill
// the device several times: no thread divides an element index by the row length.
inline dim3 columns_by_rows_grid(int64_t columns, int64_t rows) {
    int64_t x = (columns + 255) / 256;
    x = x < 1 ? 1 : (x > 65535 ? 65535 : x);
    int64_t y = rows < 1 ? 1 : rows;
    if (x * y > 16384) y = 16384 / x < 1 ? 1 : 16384 / x;
    if (y > 65535) y = 65535;
    return dim3((unsigned)x, (unsigned)y);
}
// ptr[0..n) = 0 by the threads tid, tid + stride, ..: 16-byte stores between the first and the last 16-byte
// boundary of the buffer, single elements before and after
template <typename T>
__device__ __forceinline__ void zero_span(T *__restrict__ ptr, int64_t n, int64_t tid, int64_t stride) {
    constexpr int VW = 16 / (int)sizeof(T);
    typedef T V __attribute__((ext_vector_type(VW)));
    int64_t head = (int64_t)(((16 - ((uintptr_t)ptr & 15)) & 15) / sizeof(T));
    if (head > n) head = n;
    const int64_t vecs = (n - head) / VW;
    const int64_t tail_from = head + vecs * VW;
    V *v = reinterpret_cast<V *>(ptr + head);
    V zero;
#pragma unroll
    for (int k = 0; k < VW; ++k) zero[k] = T(0);
    for (int64_t i = tid; i < vecs; i += stride) v[i] = zero;
    if (tid < head) ptr[tid] = T(0);
    if (tid < n - tail_from) ptr[tail_from + tid] = T(0);
}
// projected layout <- dense layout (gather) and dense layout += projected layout (scatter; dense zeroed before)
template <typename T>
hipError_t launch_gather_columns(const T *dense, T *out, const LevelPlan &plan, int64_t d, const int64_t *codes,
                                 int64_t rows, hipStream_t stream);
template <typename T>
hipError_t launch_scatter_columns(const T *grad, T *dense, const LevelPlan &plan, int64_t d, const int64_t *codes,
                                  int64_t rows, hipStream_t stream);
template <typename TI, typename T>
hipError_t launch_increments_to_path(const TI *grad_inc, T *grad_path, int64_t B, int64_t L, int64_t d,
                                     hipStream_t stream);
// sig -> logsig and the cache its adjoint reads; `powers`, when not null, also receives the power cache of the
// reference (it may be the same buffer as `cache`, which it then replaces)
template <typename T>
hipError_t launch_logsig_forward(const T *sig, T *logsig, T *cache, T *powers, int64_t rows, int64_t d, int depth,
                                 int64_t top_size, const int64_t *top_words, hipStream_t stream);
// workspace of the log-signature adjoint, in elements of the floating type (see logsig_kernels.hip)
struct LogsigBackwardPlan {
    bool gather;
    int64_t a_elems, q_elems, top_elems, top_dense;
};
LogsigBackwardPlan logsig_backward_plan(size_t elem, int64_t rows, int64_t d, int depth, int64_t top_size);
template <typename T>
hipError_t launch_logsig_backward(const T *logsig, const T *cache, const T *grad_logsig, T *grad_sig, T *workspace,
                                  int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                                  hipStream_t stream);

}  // namespace psig
