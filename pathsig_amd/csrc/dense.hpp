// Register-tiled kernels for the dense (all words) signature at selected (path dimension, depth).
#pragma once

#include "common.hpp"

namespace psig {

struct DenseChoice {
    bool usable;                // a register-tiled kernel exists for this call
    bool embed;                 // the call is a word projection that is computed densely and then gathered
    bool bounded;               // embed: the sweeps leave out top-level words by the letter bounds of the word list
    bool resweep;               // embed with a shape that is not cut into time chunks: the backward needs the dense
                                // signature, which the forward keeps or the backward computes again
    int variant;                // index into the table of compiled shapes
    int fwd_chunks;             // time chunks per (path, window) in the forward
    int bwd_chunks;             // ... and in the backward (at least 2 when embedding: no dense signature is saved)
    size_t dense_bytes;         // embed: bytes of one dense [rows, S] buffer
    size_t forward_workspace;   // bytes of scratch the forward needs (including the dense buffer)
    size_t backward_workspace;  // bytes of scratch the backward needs beyond the increment accumulator
    size_t keep_bytes;          // bytes the forward can keep for the backward: the prefix and suffix products of the
                                // chunk signatures below the top level, or (resweep) the dense signature (0: none)
    bool grouped;               // the kept products are those within groups of four chunks plus those of whole groups
                                // (four arrays: [rows, chunks, low] twice, then [rows, chunks / 4, low] twice)
};

DenseChoice dense_choice(size_t elem, int64_t d, int depth, bool all_dense, const int64_t *level_sizes, int64_t B,
                         int64_t L, int64_t W, bool windowed);

// `sig` / `grad_sig` are dense-layout rows; `workspace` is the part of the scratch after any dense buffer.
// top_codes / top_count: the word list of the top level (device memory), read only when dc.bounded.
// keep (optional, dc.keep_bytes bytes): receives, per time chunk, the signature of the row up to the chunk's right
// edge and that of the rest of the row, below the top level; passing the same buffer as `kept` to the backward of
// the same call saves it the launches that recompute them.
template <typename T>
hipError_t launch_dense_forward(const T *path, T *sig, const SigShape &shape, const DenseChoice &dc,
                                const int64_t *top_codes, int64_t top_count, T *keep, void *workspace,
                                hipStream_t stream);
// The backward fills grad_inc ([B, L-1, d] increment gradients), or, for time-chunked calls without windows,
// writes grad_path ([B, L, d]) itself and reports that in *wrote_path.
// prepared: prepare_dense_backward has run for this call (grad_inc is zero, the letter bounds of a bounded call
// are at the head of `workspace`).
template <typename T>
hipError_t launch_dense_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, T *grad_path,
                                 bool *wrote_path, const SigShape &shape, const DenseChoice &dc,
                                 const int64_t *top_codes, int64_t top_count, const T *kept, void *workspace,
                                 bool prepared, hipStream_t stream);
// One launch in front of the backward of an embedded projection, in place of three: clears zero[0..count) (the
// per-increment sums and the dense gradient buffer behind them) and, for a bounded call, computes the letter
// bounds into bounds_at (the head of the workspace that launch_dense_backward will be given).
template <typename T>
hipError_t prepare_dense_backward(const DenseChoice &dc, T *zero, int64_t count, const int64_t *top_codes,
                                  int64_t top_count, void *bounds_at, hipStream_t stream);

// The compiled shapes are dealt to kDenseGroups translation units (shape index modulo kDenseGroups); these are the
// launch sequences of one group.  `bounds`: device array of letter bounds, or nullptr.
constexpr int kDenseGroups = 8;
template <int GROUP, typename T>
hipError_t launch_dense_forward_group(const T *path, T *sig, const SigShape &shape, const DenseChoice &dc,
                                      const int *bounds, T *keep, void *workspace, hipStream_t stream);
template <int GROUP, typename T>
hipError_t launch_dense_backward_group(const T *path, const T *sig, const T *grad_sig, T *grad_inc, T *grad_path,
                                       bool *wrote_path, const SigShape &shape, const DenseChoice &dc,
                                       const int *bounds, const T *kept, void *workspace, bool inc_cleared,
                                       hipStream_t stream);

// measurement hook: events around the reverse-sweep kernel of the last backward call (profile_bracket marks
// the begin and the end of that kernel on its stream; a no-op while the hook is off)
void profile_enable(bool on);
void profile_bracket(bool begin, hipStream_t stream);
float profile_sweep_ms();

}  // namespace psig
