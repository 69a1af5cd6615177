// Shared declarations of libpathsig_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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
};

// Geometry of one signature call.
struct SigShape {
    int64_t B, L, d, W;  // W = 1 and windows == nullptr when no windows are given
    const int32_t *windows;
};

void set_error(const char *fmt, ...);

template <typename T>
struct Recip {
    // 1/k for k = 1..12 as compile-time constants of type T
    __host__ __device__ static constexpr T of(int k) { return T(1) / T(k); }
};

// Launchers implemented in the kernel translation units.  Each returns hipSuccess or the launch error.
template <typename T>
hipError_t launch_words_forward(const T *path, T *sig, const SigShape &shape, const LevelPlan &plan,
                                const int64_t *codes, hipStream_t stream);
template <typename T>
hipError_t launch_words_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, const SigShape &shape,
                                 const LevelPlan &plan, const int64_t *codes, hipStream_t stream);
template <typename T>
hipError_t launch_fill_zero(T *ptr, int64_t n, hipStream_t stream);
template <typename T>
hipError_t launch_increments_to_path(const T *grad_inc, T *grad_path, int64_t B, int64_t L, int64_t d,
                                     hipStream_t stream);
template <typename T>
hipError_t launch_logsig_forward(const T *sig, T *logsig, T *P, int64_t rows, int64_t d, int depth, int64_t top_size,
                                 const int64_t *top_words, hipStream_t stream);
template <typename T>
hipError_t launch_logsig_backward(const T *sig, const T *P, const T *grad_logsig, T *grad_sig, T *gradP, int64_t rows,
                                  int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                                  hipStream_t stream);

}  // namespace psig
