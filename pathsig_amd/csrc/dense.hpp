// Register-tiled kernels for the dense (all words) signature at selected (path dimension, depth).
#pragma once

#include "common.hpp"

namespace psig {

struct DenseChoice {
    bool usable;                // a register-tiled kernel exists for this call
    int variant;                // index into the table of compiled shapes
    int chunks;                 // time chunks per (path, window)
    size_t forward_workspace;   // bytes of scratch the forward needs
    size_t backward_workspace;  // bytes of scratch the backward needs beyond the increment accumulator
};

DenseChoice dense_choice(size_t elem, int64_t d, int depth, bool all_dense, const int64_t *level_sizes, int64_t B,
                         int64_t L, int64_t W, bool windowed);

template <typename T>
hipError_t launch_dense_forward(const T *path, T *sig, const SigShape &shape, const LevelPlan &plan,
                                const int64_t *codes, const DenseChoice &dc, void *workspace, hipStream_t stream);
template <typename T>
hipError_t launch_dense_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, const SigShape &shape,
                                 const LevelPlan &plan, const int64_t *codes, const DenseChoice &dc, void *workspace,
                                 hipStream_t stream);

}  // namespace psig
