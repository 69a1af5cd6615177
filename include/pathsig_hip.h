/*
 * C ABI of libpathsig_hip.so: signature / log-signature operators for AMD MI355X (gfx950).
 *
 * The four compute entry points are what a host binding of the reference's four operators calls
 * (schemas in src/pathsig/bindings.cpp:9-63 of tobiasny12/pathsig).  All pointers are raw device or
 * host addresses, all sizes are plain integers, nothing here depends on torch.
 *
 * Conventions
 *   - dtype: PATHSIG_F32 or PATHSIG_F64; every floating buffer of one call has that type.
 *   - device buffers are dense row-major and must not overlap; the library never allocates, frees,
 *     or synchronises: scratch memory is passed in as `workspace` (size from the matching
 *     *_workspace function; contents need not be initialised) and all work is enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL is the default stream).
 *   - level_sizes is a HOST array with depth+1 entries (entry 0 unused) or NULL for the dense
 *     signature.  A level whose size equals d^k is dense (all words, lexicographic); any other level
 *     takes its words from encoded_words, a DEVICE int64 array with the base-d codes (first letter
 *     most significant) of the non-dense levels concatenated in level order.
 *   - windows is a DEVICE int32 array of W [start, end) pairs over point indices, or NULL.  Windows
 *     are clamped to [0, L]; a window with fewer than two points yields zeros.
 *   - return value: PATHSIG_OK or a negative error code; pathsig_last_error() gives the message of
 *     the last failure on the calling thread.
 */
#ifndef PATHSIG_HIP_H
#define PATHSIG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PATHSIG_F32 0
#define PATHSIG_F64 1

#define PATHSIG_OK 0
#define PATHSIG_ERR_ARGUMENT (-1)    /* null pointer, bad dtype, depth outside 1..12, L < 2, ... */
#define PATHSIG_ERR_UNSUPPORTED (-2) /* a size the kernels cannot handle */
#define PATHSIG_ERR_WORKSPACE (-3)   /* workspace missing or too small */
#define PATHSIG_ERR_LAUNCH (-4)      /* the HIP runtime rejected a launch */

#define PATHSIG_MAX_DEPTH 12

/* Library ABI version (bumped when a signature below changes). */
int pathsig_abi_version(void);

/* Message of the last error on this thread ("" if none). */
const char *pathsig_last_error(void);

/*
 * Signature forward.  Replaces computeSignature (src/pathsig/forward/sig_launch.cu:75-225, op
 * `pathsig::compute_signature`, src/pathsig/bindings.cpp:9-20).
 *   path [B, L, d] -> sig [B, S] (windows == NULL) or [B, W, S];  S = sum of the level sizes.
 */
size_t pathsig_sig_forward_workspace(int dtype, int64_t B, int64_t L, int64_t d, int depth,
                                     const int64_t *level_sizes, int64_t W);
int pathsig_sig_forward(const void *path, void *sig, int dtype, int64_t B, int64_t L, int64_t d, int depth,
                        const int64_t *level_sizes, const int64_t *encoded_words, int64_t n_encoded,
                        const int32_t *windows, int64_t W, void *workspace, size_t workspace_bytes,
                        void *stream);

/*
 * Signature backward: dL/dpath from dL/dsig.  Replaces signature_backward
 * (src/pathsig/backward/sig_backward_launch.cu:83-303, op `pathsig::signature_backward`,
 * src/pathsig/bindings.cpp:23-36).  `sig` is the forward output for the same arguments.
 *   path [B, L, d], sig and grad_sig [B, (W,) S] -> grad_path [B, L, d].
 * Gradients of overlapping windows add.
 */
size_t pathsig_sig_backward_workspace(int dtype, int64_t B, int64_t L, int64_t d, int depth,
                                      const int64_t *level_sizes, int64_t W);
int pathsig_sig_backward(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                         int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                         const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * Signature backward that allocates nothing.  No counterpart in the reference: it is for callers that cannot
 * call hipMalloc or bring a workspace -- code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  Same arguments and results as pathsig_sig_backward, without `workspace`: the scratch is a fixed
 * array of PATHSIG_STATIC_SCRATCH_BYTES that lives in the library's device image (every GPU the library runs on
 * holds one until the process ends).  A call that needs more (pathsig_sig_backward_workspace tells) fails with
 * PATHSIG_ERR_WORKSPACE and launches nothing.  All calls on one GPU share that array: calls that overlap on one
 * GPU (two streams, two threads) race; serialise them or use the entry point with a workspace.  The first call on
 * a device looks the array's address up (hipGetSymbolAddress); make that call outside a graph capture.
 */
#define PATHSIG_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
int pathsig_sig_backward_noalloc(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                                 int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                                 const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                                 void *stream);

/*
 * The same pair with a hand-over from the forward to the backward of one call (no counterpart in the
 * reference, whose backward receives the path and the signature only and recomputes what it needs).
 * On long paths the register-tiled kernels cut every row into time chunks; the backward starts every chunk
 * from the signature of the row up to the chunk's right edge and from the signature of the rest of the row,
 * both below the top level (products of the chunks' own signatures).  The forward can write those two
 * arrays into `chunks`, and a backward that is given the same buffer skips the two launches that would
 * recompute them.  (PATHSIG_F32 rows of eight and more chunks, a multiple of four, keep the factors of those
 * products instead: every chunk's products with its neighbours inside its group of four chunks, and the products
 * of the groups to the left and to the right of every group; the backward multiplies them as it starts a chunk.
 * See the "grouped" option.)  The per-word kernels hand over, in the same buffer, the
 * prefix values of the words whose prefixes are not all part of the signature (the backward otherwise
 * rebuilds them with a forward sweep, as src/pathsig/backward/sig_backward_kernels.cu:134-157 does).
 * A word projection that is computed through a register-tiled shape which is swept in one piece (depth 2,
 * shapes with more than 1024 lanes per row) hands over its dense signature, which the backward otherwise
 * sweeps again.
 * pathsig_sig_chunks_bytes() returns the size of that buffer for a call, or 0 when the call has nothing to
 * hand over (then use the plain entry points).  All other arguments are as above; `chunks == NULL` makes
 * both functions identical to the plain ones.
 */
size_t pathsig_sig_chunks_bytes(int dtype, int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                                int64_t W);
int pathsig_sig_forward_keep(const void *path, void *sig, int dtype, int64_t B, int64_t L, int64_t d, int depth,
                             const int64_t *level_sizes, const int64_t *encoded_words, int64_t n_encoded,
                             const int32_t *windows, int64_t W, void *chunks, size_t chunks_bytes, void *workspace,
                             size_t workspace_bytes, void *stream);
int pathsig_sig_backward_kept(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                              int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                              const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                              const void *chunks, size_t chunks_bytes, void *workspace, size_t workspace_bytes,
                              void *stream);

/*
 * Signature -> log-signature on the hybrid layout (levels 1..depth-1 dense, level `depth` with
 * `top_size` columns whose codes are `top_words`, a DEVICE int64 array, or NULL when the top level
 * is dense).  Replaces sig_to_logsig (src/pathsig/forward/sig_launch.cu:230-339, op
 * `pathsig::sig_to_logsig`, src/pathsig/bindings.cpp:39-49).
 *   sig [rows, S] -> logsig [rows, S] and the power cache P [rows, S * depth] with
 *   P[idx * depth + (m - 1)] = level-|w| part of (S - 1)^(x)m at word idx, 0 for m > |w|
 *   (the layout and contents of src/pathsig/forward/sig_kernels.cu:184,215-216,237).
 * Every element of logsig and P is written.  The values of logsig do not come from summing the powers in P
 * (that alternating sum loses most digits of fp32 on long or deep inputs) but from inverting the exponential
 * series with powers of the log-signature itself; P is filled by a second pass for callers that read it.
 */
int pathsig_logsig_forward(const void *sig, void *logsig, void *P, int dtype, int64_t rows, int64_t d, int depth,
                           int64_t top_size, const int64_t *top_words, void *stream);

/*
 * Adjoint of the above: dL/dsig from dL/dlogsig.  Replaces logsig_backward
 * (src/pathsig/backward/sig_backward_launch.cu:307-460, op `pathsig::logsig_backward`,
 * src/pathsig/bindings.cpp:52-63).
 *   sig, grad_logsig [rows, S] -> grad_sig [rows, S].
 * P is accepted for the reference's argument list and not read (it may be NULL): the adjoint rebuilds the
 * log-signature and the cache it needs from sig inside `workspace`.
 */
size_t pathsig_logsig_backward_workspace(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size);
int pathsig_logsig_backward(const void *sig, const void *P, const void *grad_logsig, void *grad_sig, int dtype,
                            int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                            void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same pair with a hand-over from the forward to the backward (no counterpart in the reference).  The
 * forward writes, instead of P, the cache its own adjoint reads: cache [rows, S * depth] with
 * cache[idx * depth + (k - 1)] = level-|w| part of (log S)^(x)k at word idx (entry 0 is the log-signature
 * itself) for the words below the top level; entry |w| of such a row holds -sum_{m<=|w|} (log S)^(x)m (w) / (m+1)!
 * (the weight of w as a prefix in the adjoint's top-level sums), later entries 0; the rows of top-level words are
 * not written (the adjoint never reads them).  The backward takes that cache and the log-signature and skips rebuilding them.
 */
int pathsig_logsig_forward_keep(const void *sig, void *logsig, void *cache, int dtype, int64_t rows, int64_t d,
                                int depth, int64_t top_size, const int64_t *top_words, void *stream);
size_t pathsig_logsig_backward_kept_workspace(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size);
int pathsig_logsig_backward_kept(const void *logsig, const void *cache, const void *grad_logsig, void *grad_sig,
                                 int dtype, int64_t rows, int64_t d, int depth, int64_t top_size,
                                 const int64_t *top_words, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Tuning switches (no counterpart in the reference, whose two heuristics are hard-coded:
 * src/pathsig/forward/sig_launch.cu:23-27, src/pathsig/backward/sig_backward_launch.cu:171).  They are process
 * wide and meant for tests and measurements; the defaults need no call.  Initial values come from the environment
 * variables named below, which are read once, when the first call of the process needs them.
 *   "chunks"          forced number of time chunks per row of the register-tiled kernels, 0 = chosen per call
 *                     (PATHSIG_CHUNKS)
 *   "letter_bounds"   1 = embedded projections leave out unwanted top-level words (PATHSIG_NO_LETTER_BOUNDS sets 0)
 *   "logsig_scatter"  1 = the log-signature adjoint always takes its scatter form (PATHSIG_LOGSIG_SCATTER=1)
 *   "batch_tile"      cap on the increments per tile of the lanes-on-paths backward, 0 = none (PATHSIG_BATCH_TILE)
 *   "embed_share"     which word projections run on the register-tiled kernels (dense sweep + gather of the
 *                     wanted columns) instead of the per-word kernels: -1 = the library's rule (top level keeps
 *                     1/8 of the dense one, or the dense sweep is estimated cheaper), 0 = none, n > 0 = those whose
 *                     top level keeps at least 1/n of the dense one (PATHSIG_EMBED_SHARE)
 *   "tiled"           0 = every call takes the per-word kernels, whatever its shape (PATHSIG_NO_TILED sets 0)
 *   "deep_fp64"       1 (default) = a PATHSIG_F32 backward of depth 9 or more runs in fp64 on copies of the path
 *                     and of grad_sig (its workspace holds them), sweeps the signature again in fp64 and rounds the
 *                     path gradient at the end, unless it is a dense call of depth 9 cut into four time chunks or
 *                     more; 0 = in fp32 like any other call, two to three times as fast and off by up to 3.5e-5 of
 *                     the largest gradient at depth 12 (PATHSIG_NO_DEEP_FP64 sets 0)
 *   "grouped"         1 (default) = a keeping PATHSIG_F32 forward whose rows are cut into eight or more time chunks,
 *                     a multiple of four, keeps the chunk products by groups of four chunks (products within the
 *                     groups and products of whole groups; pathsig_sig_chunks_bytes says how much), where the
 *                     shape is compiled for it; 0 = products over all chunks of a row (PATHSIG_NO_GROUPED sets 0)
 * Returns PATHSIG_ERR_ARGUMENT for an unknown name or a value out of range.
 */
int pathsig_set_option(const char *name, int64_t value);

/*
 * Measurement hook (no counterpart in the reference).  While enabled, every signature backward call brackets
 * its reverse-sweep kernel (register-tiled, or per-word for general projections) with HIP events on the
 * launch stream.
 * pathsig_profile_sweep_ms() waits for the events of the last such call and returns the kernel's
 * duration in milliseconds (a negative value if there was none).  It is the only entry point that
 * synchronises with the device; the hook is off by default and is not thread safe.
 */
int pathsig_profile_enable(int on);
float pathsig_profile_sweep_ms(void);

#ifdef __cplusplus
}
#endif
#endif /* PATHSIG_HIP_H */
