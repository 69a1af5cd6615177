// extern "C" entry points of libpathsig_hip.so: argument checks, level plans, kernel selection.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <mutex>

#include "common.hpp"
#include "dense.hpp"

// Scratch of the entry point that allocates nothing (pathsig_sig_backward_noalloc).  Every GPU that loads the
// library holds its own copy of this array, at its own address, until the process ends.  In host code the name
// below is only a handle for hipGetSymbolAddress: the address that kernels and fills receive is the one that
// call returns for the current device (static_scratch_of_current_device).
static __device__ __align__(256) unsigned char scratch[PATHSIG_STATIC_SCRATCH_BYTES];

namespace psig {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

namespace {
int64_t env_int(const char *name, int64_t fallback) {
    const char *v = getenv(name);
    return (v && *v) ? atoll(v) : fallback;
}

// Plain integers behind relaxed atomics: a setter on one thread and a call on another see whole values.
struct OptionCells {
    std::atomic<int64_t> chunks, letter_bounds, logsig_scatter, batch_tile, embed_share, tiled, deep_fp64, grouped;
    OptionCells()
        : chunks(env_int("PATHSIG_CHUNKS", 0)),
          letter_bounds(getenv("PATHSIG_NO_LETTER_BOUNDS") ? 0 : 1),
          logsig_scatter(env_int("PATHSIG_LOGSIG_SCATTER", 0) == 1 ? 1 : 0),
          batch_tile(env_int("PATHSIG_BATCH_TILE", 0)),
          embed_share(env_int("PATHSIG_EMBED_SHARE", -1)),
          tiled(getenv("PATHSIG_NO_TILED") ? 0 : 1),
          deep_fp64(getenv("PATHSIG_NO_DEEP_FP64") ? 0 : 1),
          grouped(getenv("PATHSIG_NO_GROUPED") ? 0 : 1) {}
};
OptionCells &option_cells() {
    static OptionCells cells;  // the environment is read here, once
    return cells;
}
}  // namespace

const Options &options() {
    thread_local Options snapshot;
    OptionCells &c = option_cells();
    snapshot.chunks = c.chunks.load(std::memory_order_relaxed);
    snapshot.letter_bounds = c.letter_bounds.load(std::memory_order_relaxed);
    snapshot.logsig_scatter = c.logsig_scatter.load(std::memory_order_relaxed);
    snapshot.batch_tile = c.batch_tile.load(std::memory_order_relaxed);
    snapshot.embed_share = c.embed_share.load(std::memory_order_relaxed);
    snapshot.tiled = c.tiled.load(std::memory_order_relaxed);
    snapshot.deep_fp64 = c.deep_fp64.load(std::memory_order_relaxed);
    snapshot.grouped = c.grouped.load(std::memory_order_relaxed);
    return snapshot;
}

namespace {

constexpr int kWordsBlock = 256;

size_t elem_size(int dtype) { return dtype == PATHSIG_F64 ? sizeof(double) : sizeof(float); }

size_t align_up(size_t n, size_t a = 256) { return (n + a - 1) / a * a; }

// d^k with overflow detection (returns -1 when it does not fit 62 bits)
int64_t checked_pow(int64_t d, int k) {
    int64_t r = 1;
    for (int i = 0; i < k; ++i) {
        if (r > (int64_t(1) << 62) / d) return -1;
        r *= d;
    }
    return r;
}

int check_common(int dtype, int64_t B, int64_t L, int64_t d, int depth) {
    if (dtype != PATHSIG_F32 && dtype != PATHSIG_F64) {
        set_error("dtype must be PATHSIG_F32 or PATHSIG_F64 (got %d)", dtype);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (depth < 1 || depth > kMaxDepth) {
        set_error("depth must be in [1,12] (got %d)", depth);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (B < 0 || d < 1) {
        set_error("path must be [B,L,d] with B >= 0 and d >= 1 (got B=%lld d=%lld)", (long long)B, (long long)d);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (L < 2) {
        set_error("path must have at least 2 time steps (got %lld)", (long long)L);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (d * (int64_t)elem_size(dtype) > 8192) {
        set_error("path dimension %lld is beyond what the kernels stage in LDS", (long long)d);
        return PATHSIG_ERR_UNSUPPORTED;
    }
    return PATHSIG_OK;
}

// Builds the per-level plan; returns PATHSIG_OK or an error.  *all_dense is set when every level is full.
int build_plan(int64_t d, int depth, const int64_t *level_sizes, int64_t n_encoded, bool have_codes, LevelPlan *plan,
               bool *all_dense) {
    std::memset(plan, 0, sizeof(*plan));
    plan->depth = depth;
    int64_t out = 0, enc = 0, blocks = 0;
    bool saved_ok = true;  // every level so far is dense: prefixes can be read from the saved signature
    *all_dense = true;
    for (int k = 1; k <= depth; ++k) {
        const int64_t width = checked_pow(d, k);
        int64_t size = width;
        if (level_sizes) size = level_sizes[k];
        if (size < 0) {
            set_error("level_sizes[%d] is negative", k);
            return PATHSIG_ERR_ARGUMENT;
        }
        if (!level_sizes && width < 0) {
            set_error("d^%d does not fit 64 bits", k);
            return PATHSIG_ERR_UNSUPPORTED;
        }
        const bool dense = (size == width);
        plan->size[k] = size;
        plan->out_off[k] = out;
        plan->code_off[k] = dense ? -1 : enc;
        plan->from_saved[k] = saved_ok ? 1 : 0;
        plan->block_begin[k] = blocks;
        if (!dense) {
            enc += size;
            *all_dense = false;
            saved_ok = false;
        }
        out += size;
        blocks += (size + kWordsBlock - 1) / kWordsBlock;
    }
    plan->block_begin[depth + 1] = blocks;
    plan->sig_size = out;
    int64_t keep = 0;
    for (int k = 1; k <= depth; ++k) {
        plan->keep_off[k] = -1;
        if (k > 1 && !plan->from_saved[k] && plan->size[k] > 0) {
            plan->keep_off[k] = keep;
            keep += plan->size[k] * (k - 1);
        }
    }
    plan->keep_size = keep;
    plan->keep = nullptr;
    if (enc > 0 && !have_codes) {
        set_error("encoded_words is NULL but %lld word codes are needed", (long long)enc);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (enc > n_encoded) {
        set_error("encoded_words holds %lld codes but the level sizes need %lld", (long long)n_encoded, (long long)enc);
        return PATHSIG_ERR_ARGUMENT;
    }
    return PATHSIG_OK;
}

int check_grid(const LevelPlan &plan, int64_t rows) {
    const int64_t per_row = plan.block_begin[plan.depth + 1];
    if (per_row > 0 && rows > (int64_t(1) << 31) / per_row - 1) {
        set_error("problem too large for one launch (%lld blocks per row x %lld rows)", (long long)per_row,
                  (long long)rows);
        return PATHSIG_ERR_UNSUPPORTED;
    }
    return PATHSIG_OK;
}

int launch_failed(hipError_t e, const char *what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return PATHSIG_ERR_LAUNCH;
}

template <typename T>
int sig_forward_t(const void *path, void *sig, int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                  const int64_t *codes, int64_t n_encoded, const int32_t *windows, int64_t W, void *keep,
                  size_t keep_bytes, void *workspace, size_t workspace_bytes, hipStream_t stream) {
    LevelPlan plan;
    bool all_dense;
    int rc = build_plan(d, depth, level_sizes, n_encoded, codes != nullptr, &plan, &all_dense);
    if (rc != PATHSIG_OK) return rc;
    SigShape shape{B, L, d, windows ? W : 1, windows};
    if (B == 0 || shape.W == 0 || plan.sig_size == 0) return PATHSIG_OK;
    rc = check_grid(plan, B * shape.W);
    if (rc != PATHSIG_OK) return rc;
    const DenseChoice dc = dense_choice(sizeof(T), d, depth, all_dense, level_sizes, B, L, shape.W, windows != nullptr);
    const size_t keep_need = dc.usable ? dc.keep_bytes : (size_t)(B * shape.W * plan.keep_size) * sizeof(T);
    if (keep && (keep_need == 0 || keep_bytes < keep_need)) {
        set_error("chunk buffer: this call keeps %zu bytes, got %zu", keep_need, keep_bytes);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (dc.usable) {
        if (workspace_bytes < dc.forward_workspace || (dc.forward_workspace && !workspace)) {
            set_error("workspace too small: need %zu bytes, got %zu", dc.forward_workspace, workspace_bytes);
            return PATHSIG_ERR_WORKSPACE;
        }
        // a dense call writes straight into sig; an embedded projection goes through a dense buffer (the buffer kept
        // for the backward when that is the dense signature itself)
        const bool keep_dense = dc.embed && dc.resweep && keep;
        T *dense = keep_dense ? (T *)keep : dc.embed ? (T *)workspace : (T *)sig;
        void *rest = (unsigned char *)workspace + dc.dense_bytes;
        const int64_t *top_codes = plan.code_off[depth] >= 0 ? codes + plan.code_off[depth] : nullptr;
        hipError_t e = launch_dense_forward<T>((const T *)path, dense, shape, dc, top_codes, plan.size[depth],
                                               dc.resweep ? (T *)nullptr : (T *)keep, rest, stream);
        if (e != hipSuccess) return launch_failed(e, "dense forward launch");
        if (dc.embed) {
            e = launch_gather_columns<T>(dense, (T *)sig, plan, d, codes, B * shape.W, stream);
            if (e != hipSuccess) return launch_failed(e, "gather launch");
        }
        return PATHSIG_OK;
    }
    plan.keep = keep;  // the per-word forward leaves the prefix values its backward would recompute
    hipError_t e = launch_words_forward<T>((const T *)path, (T *)sig, shape, plan, codes, stream);
    if (e != hipSuccess) return launch_failed(e, "forward launch");
    return PATHSIG_OK;
}

// bytes of the per-increment sums dL/d(dx): of the call's type, fp64 behind the word-per-lane backward
size_t inc_buffer_bytes(size_t elem, int64_t B, int64_t L, int64_t d, bool words_kernel) {
    return align_up((size_t)(B * (L - 1) * d) * (words_kernel ? sizeof(double) : elem));
}

template <typename T>
int sig_backward_t(const void *path, const void *sig, const void *grad_sig, void *grad_path, int64_t B, int64_t L,
                   int64_t d, int depth, const int64_t *level_sizes, const int64_t *codes, int64_t n_encoded,
                   const int32_t *windows, int64_t W, const void *kept, size_t kept_bytes, void *workspace,
                   size_t workspace_bytes, hipStream_t stream) {
    LevelPlan plan;
    bool all_dense;
    int rc = build_plan(d, depth, level_sizes, n_encoded, codes != nullptr, &plan, &all_dense);
    if (rc != PATHSIG_OK) return rc;
    SigShape shape{B, L, d, windows ? W : 1, windows};
    if (B == 0) return PATHSIG_OK;
    rc = check_grid(plan, B * shape.W);
    if (rc != PATHSIG_OK) return rc;
    const DenseChoice dc = dense_choice(sizeof(T), d, depth, all_dense, level_sizes, B, L, shape.W, windows != nullptr);
    const size_t keep_need = dc.usable ? dc.keep_bytes : (size_t)(B * shape.W * plan.keep_size) * sizeof(T);
    // The layout of what a forward keeps follows from the choice of kernels, which the tuning switches can change
    // between the two calls.  A buffer of another size than this call would have kept comes from a forward that
    // chose differently and is refused (every such choice keeps a different number of bytes: prefix values per
    // word, two rows of products per chunk, or the dense signature).
    if (kept && (keep_need == 0 || kept_bytes != keep_need)) {
        set_error("chunk buffer: the forward of this call keeps %zu bytes, got %zu (made under other options?)", keep_need,
                  kept_bytes);
        return PATHSIG_ERR_ARGUMENT;
    }
    plan.keep = const_cast<void *>(kept);
    const bool words_kernel = !dc.usable && !batch_backward_usable(sizeof(T), B, d, shape.W);
    const bool batch_wide = !dc.usable && !words_kernel && batch_wide_sums(sizeof(T), plan);
    const size_t inc_bytes = inc_buffer_bytes(sizeof(T), B, L, d, words_kernel || batch_wide);
    const size_t need = inc_bytes + (dc.usable ? dc.backward_workspace : 0);
    if (!workspace || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return PATHSIG_ERR_WORKSPACE;
    }
    T *ginc = (T *)workspace;
    hipError_t e;
    if (dc.usable) {
        unsigned char *extra = (unsigned char *)workspace + inc_bytes;
        const T *gdense = (const T *)grad_sig;
        const T *sdense = (const T *)sig;
        const int64_t *top_codes = plan.code_off[depth] >= 0 ? codes + plan.code_off[depth] : nullptr;
        size_t used = 0;
        bool prepared = false;
        if (dc.embed) {
            // upstream gradient scattered into a zeroed dense buffer.  The time-chunked backward rebuilds what it
            // reads of the dense signature; a shape that is swept in one piece reads the dense signature, which the
            // forward kept or which is swept again here
            // (one launch clears the increment sums and the dense buffer behind them and, for a bounded call,
            // computes the letter bounds where the backward looks for them: the head of its workspace)
            T *buf = (T *)extra;
            used = (dc.resweep ? 2 : 1) * dc.dense_bytes;
            e = prepare_dense_backward<T>(dc, ginc, (int64_t)((inc_bytes + dc.dense_bytes) / sizeof(T)), top_codes,
                                          plan.size[depth], extra + used, stream);
            if (e != hipSuccess) return launch_failed(e, "fill launch");
            prepared = true;
            e = launch_scatter_columns<T>((const T *)grad_sig, buf, plan, d, codes, B * shape.W, stream);
            if (e != hipSuccess) return launch_failed(e, "scatter launch");
            gdense = buf;
            sdense = nullptr;
            if (dc.resweep) {
                if (kept) {
                    sdense = (const T *)kept;
                } else {
                    T *again = (T *)(extra + dc.dense_bytes);
                    e = launch_dense_forward<T>((const T *)path, again, shape, dc, top_codes, plan.size[depth],
                                                (T *)nullptr, extra + 2 * dc.dense_bytes, stream);
                    if (e != hipSuccess) return launch_failed(e, "dense forward launch");
                    sdense = again;
                }
            }
        }
        bool wrote_path = false;
        e = launch_dense_backward<T>((const T *)path, sdense, gdense, ginc, (T *)grad_path, &wrote_path, shape, dc,
                                     top_codes, plan.size[depth], dc.resweep ? (const T *)nullptr : (const T *)kept,
                                     extra + used, prepared, stream);
        if (e != hipSuccess) return launch_failed(e, "dense backward launch");
        if (wrote_path) return PATHSIG_OK;
    } else if (words_kernel || batch_wide) {
        // lanes on words, or lanes on paths with a great many words: the per-increment sums are kept in fp64 (one
        // term per block of words and cell)
        double *ginc64 = (double *)workspace;
        e = launch_fill_zero<double>(ginc64, B * (L - 1) * d, stream);
        if (e != hipSuccess) return launch_failed(e, "fill launch");
        if (shape.W > 0 && plan.sig_size > 0) {
            profile_bracket(true, stream);
            if (words_kernel)
                e = launch_words_backward<T>((const T *)path, (const T *)sig, (const T *)grad_sig, ginc64, shape, plan,
                                             codes, stream);
            else
                e = launch_batch_backward<T, double>((const T *)path, (const T *)sig, (const T *)grad_sig, ginc64, shape,
                                                     plan, codes, stream);
            profile_bracket(false, stream);
            if (e != hipSuccess) return launch_failed(e, "backward launch");
        }
        e = launch_increments_to_path<double, T>(ginc64, (T *)grad_path, B, L, d, stream);
        if (e != hipSuccess) return launch_failed(e, "path-gradient launch");
        return PATHSIG_OK;
    } else {
        e = launch_fill_zero<T>(ginc, B * (L - 1) * d, stream);
        if (e != hipSuccess) return launch_failed(e, "fill launch");
        if (shape.W > 0 && plan.sig_size > 0) {
            profile_bracket(true, stream);
            e = launch_batch_backward<T, T>((const T *)path, (const T *)sig, (const T *)grad_sig, ginc, shape, plan, codes,
                                            stream);
            profile_bracket(false, stream);
            if (e != hipSuccess) return launch_failed(e, "backward launch");
        }
    }
    e = launch_increments_to_path<T, T>(ginc, (T *)grad_path, B, L, d, stream);
    if (e != hipSuccess) return launch_failed(e, "path-gradient launch");
    return PATHSIG_OK;
}

// Deep fp32 calls.  The reverse sweep rebuilds the signature of every earlier time by multiplying with exp(-dx_t),
// and the gradient of a top-level coefficient sums thousands of terms of mixed sign: from depth 9 on, fp32 rounding
// in those two places passes 1e-5 of the largest gradient (over a span of increments of size one, swept in one
// piece: 1.0e-5 to 1.5e-5 at depth 9, up to 3.5e-5 at depth 12).  Such a backward runs in fp64 on copies of the
// path and of the upstream gradient, sweeps the signature again in fp64 (rolled back over such a span, the rounding
// of the fp32 signature alone shows as 1.4e-5 in the gradient at depth 10) and rounds the path gradient at the end;
// the forward call stays in fp32.  Exempt: dense calls of depth 9 that are cut into four time chunks or more, which
// stay below 1e-5 in fp32.
__global__ void __launch_bounds__(256) widen_kernel(const float *__restrict__ src, double *__restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}
__global__ void __launch_bounds__(256) narrow_kernel(const double *__restrict__ src, float *__restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dst[i] = (float)src[i];
}
unsigned convert_blocks(int64_t n) { return (unsigned)std::min<int64_t>((n + 255) / 256, 16384); }

bool backward_in_fp64(int dtype, int depth, const DenseChoice &dc) {
    if (dtype != PATHSIG_F32 || depth < 9 || options().deep_fp64 == 0) return false;
    return depth >= 10 || !(dc.usable && !dc.embed && dc.bwd_chunks >= 4);
}

struct DeepLayout {
    size_t path_bytes, sig_bytes, total;  // two buffers of each size, then the workspace of the fp64 call
};
DeepLayout deep_layout(int64_t B, int64_t L, int64_t d, int64_t rows, int64_t sig_size, size_t inner) {
    DeepLayout lay;
    lay.path_bytes = align_up((size_t)(B * L * d) * sizeof(double));
    lay.sig_bytes = align_up((size_t)(rows * sig_size) * sizeof(double));
    lay.total = 2 * lay.path_bytes + 2 * lay.sig_bytes + inner;
    return lay;
}

// Wide alphabets at depth 3.  The register-tiled kernels exist for every alphabet up to 64 letters; from 65 to 112
// letters they exist for every eighth size (72, 80, .. 112).  A dense depth-3 call over d letters in that range
// runs as the call over the next of these sizes D on a copy of the path with D - d constant coordinates: every
// coefficient of a word that uses one of them is exactly zero, the others are the coefficients wanted, and the
// gradient with respect to the added coordinates is dropped.  (The per-word kernels, which such calls took before,
// run the backward of d = 100 at 0.4 TFLOP/s.)
int64_t wide_pad_dim(size_t elem, int64_t d, int depth, bool all_dense, int64_t B, int64_t L, int64_t W, bool windowed) {
    if (depth != 3 || !all_dense || d <= 64 || d > 112 || options().tiled == 0) return 0;
    const int64_t D = (d + 7) / 8 * 8;
    if (D == d) return 0;  // compiled as it is
    return dense_choice(elem, D, depth, true, nullptr, B, L, W, windowed).usable ? D : 0;
}

// index of dense-layout column `col` of a depth-3 signature over d letters in the layout over D letters
__device__ __forceinline__ int64_t wide_column(int64_t col, int64_t d, int64_t D) {
    if (col < d) return col;
    col -= d;
    if (col < d * d) {
        const int64_t a = col / d;
        return D + a * D + (col - a * d);
    }
    col -= d * d;
    const int64_t ab = col / d, c = col - ab * d, a = ab / d, b = ab - a * d;
    return D + D * D + (a * D + b) * D + c;
}

// the first `count` values of every row: narrow[row][i] <-> wide[row][map(i)]; TO_WIDE copies narrow -> wide (the
// rest of `wide` is cleared before where it is read), else wide -> narrow
template <typename T, bool TO_WIDE, bool SIGNATURE>
__global__ void __launch_bounds__(256) wide_copy_kernel(T *__restrict__ narrow, T *__restrict__ wide, int64_t rows,
                                                        int64_t count, int64_t narrow_stride, int64_t wide_stride,
                                                        int64_t d, int64_t D) {
    const int64_t total = rows * count;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / count, col = i - row * count;
        // a path row is one point: the letters keep their places; a signature row is mapped level by level
        const int64_t at = row * wide_stride + (SIGNATURE ? wide_column(col, d, D) : col);
        if (TO_WIDE) wide[at] = narrow[row * narrow_stride + col];
        else narrow[row * narrow_stride + col] = wide[at];
    }
}

template <typename T, bool TO_WIDE, bool SIGNATURE>
hipError_t launch_wide_copy(const T *narrow, const T *wide, int64_t rows, int64_t count, int64_t narrow_stride,
                            int64_t wide_stride, int64_t d, int64_t D, hipStream_t stream) {
    if (rows * count == 0) return hipSuccess;
    hipLaunchKernelGGL((wide_copy_kernel<T, TO_WIDE, SIGNATURE>), dim3(convert_blocks(rows * count)), dim3(256), 0, stream,
                       const_cast<T *>(narrow), const_cast<T *>(wide), rows, count, narrow_stride, wide_stride, d, D);
    return hipGetLastError();
}

struct WideLayout {
    size_t path_bytes, sig_bytes;  // of the copies over D letters
    int64_t sig_size, wide_sig_size;
};
WideLayout wide_layout(size_t elem, int64_t B, int64_t L, int64_t d, int64_t D, int64_t rows) {
    WideLayout lay;
    lay.sig_size = d + d * d + d * d * d;
    lay.wide_sig_size = D + D * D + D * D * D;
    lay.path_bytes = align_up((size_t)(B * L * D) * elem);
    lay.sig_bytes = align_up((size_t)(rows * lay.wide_sig_size) * elem);
    return lay;
}

template <typename T>
int wide_forward(const void *path, void *sig, int64_t B, int64_t L, int64_t d, int64_t D, const int32_t *windows,
                 int64_t W, void *workspace, size_t workspace_bytes, hipStream_t stream) {
    const int64_t rows = B * (windows ? W : 1);
    const WideLayout lay = wide_layout(sizeof(T), B, L, d, D, rows);
    const size_t inner = pathsig_sig_forward_workspace(sizeof(T) == 8 ? PATHSIG_F64 : PATHSIG_F32, B, L, D, 3, nullptr,
                                                       windows ? W : 0);
    const size_t need = lay.path_bytes + lay.sig_bytes + inner;
    if (!workspace || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return PATHSIG_ERR_WORKSPACE;
    }
    unsigned char *at = (unsigned char *)workspace;
    T *wide_path = (T *)at, *wide_sig = (T *)(at + lay.path_bytes);
    hipError_t e = launch_fill_zero<T>(wide_path, B * L * D, stream);
    if (e == hipSuccess) e = launch_wide_copy<T, true, false>((const T *)path, wide_path, B * L, d, d, D, d, D, stream);
    if (e != hipSuccess) return launch_failed(e, "wide path launch");
    const int rc = sig_forward_t<T>(wide_path, wide_sig, B, L, D, 3, nullptr, nullptr, 0, windows, W, nullptr, 0,
                                    at + lay.path_bytes + lay.sig_bytes, inner, stream);
    if (rc != PATHSIG_OK) return rc;
    e = launch_wide_copy<T, false, true>((const T *)sig, wide_sig, rows, lay.sig_size, lay.sig_size, lay.wide_sig_size, d,
                                         D, stream);
    if (e != hipSuccess) return launch_failed(e, "wide gather launch");
    return PATHSIG_OK;
}

size_t wide_backward_bytes(size_t elem, int64_t B, int64_t L, int64_t d, int64_t D, int64_t W) {
    const WideLayout lay = wide_layout(elem, B, L, d, D, B * (W > 0 ? W : 1));
    return 2 * lay.path_bytes + 2 * lay.sig_bytes +
           pathsig_sig_backward_workspace(elem == 8 ? PATHSIG_F64 : PATHSIG_F32, B, L, D, 3, nullptr, W);
}

template <typename T>
int wide_backward(const void *path, const void *sig, const void *grad_sig, void *grad_path, int64_t B, int64_t L,
                  int64_t d, int64_t D, const int32_t *windows, int64_t W, void *workspace, size_t workspace_bytes,
                  hipStream_t stream) {
    const int64_t rows = B * (windows ? W : 1);
    const WideLayout lay = wide_layout(sizeof(T), B, L, d, D, rows);
    const size_t need = wide_backward_bytes(sizeof(T), B, L, d, D, windows ? W : 0);
    if (!workspace || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return PATHSIG_ERR_WORKSPACE;
    }
    unsigned char *at = (unsigned char *)workspace;
    T *wide_path = (T *)at, *wide_gpath = (T *)(at + lay.path_bytes);
    T *wide_sig = (T *)(at + 2 * lay.path_bytes), *wide_grad = (T *)(at + 2 * lay.path_bytes + lay.sig_bytes);
    void *inner_ws = at + 2 * lay.path_bytes + 2 * lay.sig_bytes;
    // (the coefficients of the words that use an added letter are zero in the signature, and their upstream
    // gradient is taken as zero: they are no outputs of the call)
    // Of the signature the reverse sweep reads the levels below the top one (its state at the right end): the first
    // two levels are copied into a cleared buffer.
    hipError_t e = launch_fill_zero<T>(wide_path, B * L * D, stream);
    if (e == hipSuccess) e = launch_fill_zero<T>(wide_sig, 2 * (int64_t)(lay.sig_bytes / sizeof(T)), stream);
    if (e == hipSuccess) e = launch_wide_copy<T, true, false>((const T *)path, wide_path, B * L, d, d, D, d, D, stream);
    if (e == hipSuccess)
        e = launch_wide_copy<T, true, true>((const T *)sig, wide_sig, rows, d + d * d, lay.sig_size, lay.wide_sig_size, d,
                                            D, stream);
    if (e == hipSuccess)
        e = launch_wide_copy<T, true, true>((const T *)grad_sig, wide_grad, rows, lay.sig_size, lay.sig_size,
                                            lay.wide_sig_size, d, D, stream);
    if (e != hipSuccess) return launch_failed(e, "wide scatter launch");
    const int rc = sig_backward_t<T>(wide_path, wide_sig, wide_grad, wide_gpath, B, L, D, 3, nullptr, nullptr, 0, windows, W,
                                     nullptr, 0, inner_ws, need - 2 * lay.path_bytes - 2 * lay.sig_bytes, stream);
    if (rc != PATHSIG_OK) return rc;
    e = launch_wide_copy<T, false, false>((const T *)grad_path, wide_gpath, B * L, d, d, D, d, D, stream);
    if (e != hipSuccess) return launch_failed(e, "wide gradient launch");
    return PATHSIG_OK;
}

int check_logsig(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size) {
    if (dtype != PATHSIG_F32 && dtype != PATHSIG_F64) {
        set_error("dtype must be PATHSIG_F32 or PATHSIG_F64 (got %d)", dtype);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (depth < 1 || depth > kMaxDepth) {
        set_error("depth must be in [1,12] (got %d)", depth);
        return PATHSIG_ERR_ARGUMENT;
    }
    if (d < 1 || rows < 0 || top_size < 0) {
        set_error("d must be >= 1, rows and top_size >= 0");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (checked_pow(d, depth) < 0) {
        set_error("d^depth does not fit 64 bits");
        return PATHSIG_ERR_UNSUPPORTED;
    }
    if (rows >= (int64_t(1) << 31)) {
        set_error("too many rows for one launch");
        return PATHSIG_ERR_UNSUPPORTED;
    }
    return PATHSIG_OK;
}

size_t logsig_backward_bytes(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size) {
    const LogsigBackwardPlan lp = logsig_backward_plan(elem_size(dtype), rows, d, depth, top_size);
    return (size_t)(lp.a_elems + lp.q_elems + lp.top_elems) * elem_size(dtype);
}

}  // namespace
}  // namespace psig

using namespace psig;

extern "C" {

int pathsig_abi_version(void) { return 3; }

const char *pathsig_last_error(void) { return g_error; }

int pathsig_profile_enable(int on) {
    profile_enable(on != 0);
    return PATHSIG_OK;
}

float pathsig_profile_sweep_ms(void) { return profile_sweep_ms(); }

int pathsig_set_option(const char *name, int64_t value) {
    if (!name) {
        set_error("option name is NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (!strcmp(name, "chunks") && value >= 0 && value <= 1024) {
        option_cells().chunks.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "letter_bounds") && (value == 0 || value == 1)) {
        option_cells().letter_bounds.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "logsig_scatter") && (value == 0 || value == 1)) {
        option_cells().logsig_scatter.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "batch_tile") && value >= 0) {
        option_cells().batch_tile.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "embed_share") && value >= -1) {
        option_cells().embed_share.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "tiled") && (value == 0 || value == 1)) {
        option_cells().tiled.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "deep_fp64") && (value == 0 || value == 1)) {
        option_cells().deep_fp64.store(value, std::memory_order_relaxed);
    } else if (!strcmp(name, "grouped") && (value == 0 || value == 1)) {
        option_cells().grouped.store(value, std::memory_order_relaxed);
    } else {
        set_error("unknown option or value out of range: %s = %lld", name, (long long)value);
        return PATHSIG_ERR_ARGUMENT;
    }
    return PATHSIG_OK;
}

size_t pathsig_sig_forward_workspace(int dtype, int64_t B, int64_t L, int64_t d, int depth,
                                     const int64_t *level_sizes, int64_t W) {
    if (check_common(dtype, B, L, d, depth) != PATHSIG_OK) return 0;
    LevelPlan plan;
    bool all_dense;
    if (build_plan(d, depth, level_sizes, INT64_MAX, true, &plan, &all_dense) != PATHSIG_OK) return 0;
    if (const int64_t D = wide_pad_dim(elem_size(dtype), d, depth, all_dense, B, L, W > 0 ? W : 1, W > 0)) {
        const WideLayout lay = wide_layout(elem_size(dtype), B, L, d, D, B * (W > 0 ? W : 1));
        return lay.path_bytes + lay.sig_bytes + pathsig_sig_forward_workspace(dtype, B, L, D, depth, nullptr, W);
    }
    const DenseChoice dc =
        dense_choice(elem_size(dtype), d, depth, all_dense, level_sizes, B, L, W > 0 ? W : 1, W > 0);
    return dc.usable ? dc.forward_workspace : 0;
}

size_t pathsig_sig_chunks_bytes(int dtype, int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                                int64_t W) {
    if (check_common(dtype, B, L, d, depth) != PATHSIG_OK) return 0;
    LevelPlan plan;
    bool all_dense;
    if (build_plan(d, depth, level_sizes, INT64_MAX, true, &plan, &all_dense) != PATHSIG_OK) return 0;
    const DenseChoice dc =
        dense_choice(elem_size(dtype), d, depth, all_dense, level_sizes, B, L, W > 0 ? W : 1, W > 0);
    if (dc.usable) return dc.keep_bytes;
    return (size_t)(B * (W > 0 ? W : 1) * plan.keep_size) * elem_size(dtype);
}

int pathsig_sig_forward(const void *path, void *sig, int dtype, int64_t B, int64_t L, int64_t d, int depth,
                        const int64_t *level_sizes, const int64_t *encoded_words, int64_t n_encoded,
                        const int32_t *windows, int64_t W, void *workspace, size_t workspace_bytes, void *stream) {
    return pathsig_sig_forward_keep(path, sig, dtype, B, L, d, depth, level_sizes, encoded_words, n_encoded, windows,
                                    W, nullptr, 0, workspace, workspace_bytes, stream);
}

int pathsig_sig_forward_keep(const void *path, void *sig, int dtype, int64_t B, int64_t L, int64_t d, int depth,
                             const int64_t *level_sizes, const int64_t *encoded_words, int64_t n_encoded,
                             const int32_t *windows, int64_t W, void *chunks, size_t chunks_bytes, void *workspace,
                             size_t workspace_bytes, void *stream) {
    int rc = check_common(dtype, B, L, d, depth);
    if (rc != PATHSIG_OK) return rc;
    if (B > 0 && (!path || !sig)) {
        set_error("path and sig must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (windows && W < 0) {
        set_error("W must be >= 0");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (depth == 3 && d > 64 && B > 0 && (!windows || W > 0)) {
        LevelPlan plan;
        bool all_dense;
        rc = build_plan(d, depth, level_sizes, n_encoded, encoded_words != nullptr, &plan, &all_dense);
        if (rc != PATHSIG_OK) return rc;
        if (const int64_t D = wide_pad_dim(elem_size(dtype), d, depth, all_dense, B, L, windows ? W : 1, windows != nullptr)) {
            if (chunks && chunks_bytes > 0) {
                set_error("chunk buffer: this call keeps 0 bytes, got %zu", chunks_bytes);
                return PATHSIG_ERR_ARGUMENT;
            }
            if (dtype == PATHSIG_F32)
                return wide_forward<float>(path, sig, B, L, d, D, windows, W, workspace, workspace_bytes,
                                           (hipStream_t)stream);
            return wide_forward<double>(path, sig, B, L, d, D, windows, W, workspace, workspace_bytes,
                                        (hipStream_t)stream);
        }
    }
    if (dtype == PATHSIG_F32)
        return sig_forward_t<float>(path, sig, B, L, d, depth, level_sizes, encoded_words, n_encoded, windows, W,
                                    chunks, chunks_bytes, workspace, workspace_bytes, (hipStream_t)stream);
    return sig_forward_t<double>(path, sig, B, L, d, depth, level_sizes, encoded_words, n_encoded, windows, W, chunks,
                                 chunks_bytes, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t pathsig_sig_backward_workspace(int dtype, int64_t B, int64_t L, int64_t d, int depth,
                                      const int64_t *level_sizes, int64_t W) {
    if (check_common(dtype, B, L, d, depth) != PATHSIG_OK) return 0;
    LevelPlan plan;
    bool all_dense;
    if (build_plan(d, depth, level_sizes, INT64_MAX, true, &plan, &all_dense) != PATHSIG_OK) return 0;
    const DenseChoice dc =
        dense_choice(elem_size(dtype), d, depth, all_dense, level_sizes, B, L, W > 0 ? W : 1, W > 0);
    if (const int64_t D = wide_pad_dim(elem_size(dtype), d, depth, all_dense, B, L, W > 0 ? W : 1, W > 0))
        return wide_backward_bytes(elem_size(dtype), B, L, d, D, W);
    if (backward_in_fp64(dtype, depth, dc)) {
        const size_t inner = std::max(pathsig_sig_backward_workspace(PATHSIG_F64, B, L, d, depth, level_sizes, W),
                                      pathsig_sig_forward_workspace(PATHSIG_F64, B, L, d, depth, level_sizes, W));
        return deep_layout(B, L, d, B * (W > 0 ? W : 1), plan.sig_size, inner).total;
    }
    const bool words_kernel = !dc.usable && !batch_backward_usable(elem_size(dtype), B, d, W > 0 ? W : 1);
    const bool batch_wide = !dc.usable && !words_kernel && batch_wide_sums(elem_size(dtype), plan);
    return inc_buffer_bytes(elem_size(dtype), B, L, d, words_kernel || batch_wide) +
           (dc.usable ? dc.backward_workspace : 0) + 256;
}

int pathsig_sig_backward(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                         int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                         const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                         void *workspace, size_t workspace_bytes, void *stream) {
    return pathsig_sig_backward_kept(path, sig, grad_sig, grad_path, dtype, B, L, d, depth, level_sizes, encoded_words,
                                     n_encoded, windows, W, nullptr, 0, workspace, workspace_bytes, stream);
}

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return launch_failed(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) {
        set_error("device index %d is beyond the %d devices the static scratch is tracked for", dev, kMaxDevices);
        return PATHSIG_ERR_UNSUPPORTED;
    }
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) return launch_failed(e, "hipGetSymbolAddress(scratch)");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return PATHSIG_OK;
}
}  // namespace

int pathsig_sig_backward_noalloc(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                                 int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                                 const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                                 void *stream) {
    int rc = check_common(dtype, B, L, d, depth);
    if (rc != PATHSIG_OK) return rc;
    const size_t need = pathsig_sig_backward_workspace(dtype, B, L, d, depth, level_sizes, windows ? W : 0);
    if (need > (size_t)PATHSIG_STATIC_SCRATCH_BYTES) {
        set_error("this call needs %zu bytes of scratch; the static buffer of pathsig_sig_backward_noalloc holds %zu "
                  "(use pathsig_sig_backward with a workspace of your own)", need, (size_t)PATHSIG_STATIC_SCRATCH_BYTES);
        return PATHSIG_ERR_WORKSPACE;
    }
    void *ws = nullptr;
    rc = static_scratch_of_current_device(&ws);
    if (rc != PATHSIG_OK) return rc;
    // the backward clears every part of its workspace that has to start from zero
    return pathsig_sig_backward(path, sig, grad_sig, grad_path, dtype, B, L, d, depth, level_sizes, encoded_words,
                                n_encoded, windows, W, ws, (size_t)PATHSIG_STATIC_SCRATCH_BYTES, stream);
}

int pathsig_sig_backward_kept(const void *path, const void *sig, const void *grad_sig, void *grad_path, int dtype,
                              int64_t B, int64_t L, int64_t d, int depth, const int64_t *level_sizes,
                              const int64_t *encoded_words, int64_t n_encoded, const int32_t *windows, int64_t W,
                              const void *chunks, size_t chunks_bytes, void *workspace, size_t workspace_bytes,
                              void *stream) {
    int rc = check_common(dtype, B, L, d, depth);
    if (rc != PATHSIG_OK) return rc;
    if (B > 0 && (!path || !grad_path)) {
        set_error("path and grad_path must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (windows && W < 0) {
        set_error("W must be >= 0");
        return PATHSIG_ERR_ARGUMENT;
    }
    if (B > 0 && (!windows || W > 0) && (!sig || !grad_sig)) {
        // an empty signature (every level of size zero) is the one case with nothing to read behind them
        bool empty = level_sizes != nullptr;
        for (int k = 1; empty && k <= depth; ++k) empty = level_sizes[k] == 0;
        if (!empty) {
            set_error("sig and grad_sig must not be NULL");
            return PATHSIG_ERR_ARGUMENT;
        }
    }
    if (depth == 3 && d > 64 && B > 0 && (!windows || W > 0) && sig && grad_sig) {
        LevelPlan plan;
        bool all_dense;
        rc = build_plan(d, depth, level_sizes, n_encoded, encoded_words != nullptr, &plan, &all_dense);
        if (rc != PATHSIG_OK) return rc;
        if (const int64_t D = wide_pad_dim(elem_size(dtype), d, depth, all_dense, B, L, windows ? W : 1, windows != nullptr)) {
            if (chunks && chunks_bytes > 0) {
                set_error("chunk buffer: the forward of this call keeps 0 bytes, got %zu", chunks_bytes);
                return PATHSIG_ERR_ARGUMENT;
            }
            if (dtype == PATHSIG_F32)
                return wide_backward<float>(path, sig, grad_sig, grad_path, B, L, d, D, windows, W, workspace,
                                            workspace_bytes, (hipStream_t)stream);
            return wide_backward<double>(path, sig, grad_sig, grad_path, B, L, d, D, windows, W, workspace,
                                         workspace_bytes, (hipStream_t)stream);
        }
    }
    if (dtype == PATHSIG_F32 && depth >= 9 && B > 0) {
        LevelPlan plan;
        bool all_dense;
        rc = build_plan(d, depth, level_sizes, n_encoded, encoded_words != nullptr, &plan, &all_dense);
        if (rc != PATHSIG_OK) return rc;
        const int64_t rows = B * (windows ? W : 1);
        const DenseChoice dc =
            dense_choice(sizeof(float), d, depth, all_dense, level_sizes, B, L, windows ? W : 1, windows != nullptr);
        if (backward_in_fp64(dtype, depth, dc)) {
            // (the fp32 signature of the call, rounded, is no state to roll back from: the signature is swept again
            // in fp64; what a keeping forward left is in fp32 and stays unused)
            const size_t inner =
                std::max(pathsig_sig_backward_workspace(PATHSIG_F64, B, L, d, depth, level_sizes, windows ? W : 0),
                         pathsig_sig_forward_workspace(PATHSIG_F64, B, L, d, depth, level_sizes, windows ? W : 0));
            const DeepLayout lay = deep_layout(B, L, d, rows, plan.sig_size, inner);
            if (!workspace || workspace_bytes < lay.total) {
                set_error("workspace too small: need %zu bytes, got %zu", lay.total, workspace_bytes);
                return PATHSIG_ERR_WORKSPACE;
            }
            hipStream_t st = (hipStream_t)stream;
            unsigned char *at = (unsigned char *)workspace;
            double *path64 = (double *)at, *gpath64 = (double *)(at + lay.path_bytes);
            double *sig64 = (double *)(at + 2 * lay.path_bytes);
            double *grad64 = (double *)(at + 2 * lay.path_bytes + lay.sig_bytes);
            void *inner_ws = at + 2 * lay.path_bytes + 2 * lay.sig_bytes;
            const int64_t points = B * L * d, coefficients = rows * plan.sig_size;
            hipLaunchKernelGGL(widen_kernel, dim3(convert_blocks(points)), dim3(256), 0, st, (const float *)path, path64,
                               points);
            const bool have_sig = sig && grad_sig && coefficients > 0;
            if (have_sig)
                hipLaunchKernelGGL(widen_kernel, dim3(convert_blocks(coefficients)), dim3(256), 0, st,
                                   (const float *)grad_sig, grad64, coefficients);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return launch_failed(e, "conversion launch");
            if (have_sig) {
                rc = sig_forward_t<double>(path64, sig64, B, L, d, depth, level_sizes, encoded_words, n_encoded, windows,
                                           W, nullptr, 0, inner_ws, inner, st);
                if (rc != PATHSIG_OK) return rc;
            }
            rc = sig_backward_t<double>(path64, have_sig ? sig64 : nullptr, have_sig ? grad64 : nullptr, gpath64, B, L, d,
                                        depth, level_sizes, encoded_words, n_encoded, windows, W, nullptr, 0, inner_ws,
                                        inner, st);
            if (rc != PATHSIG_OK) return rc;
            hipLaunchKernelGGL(narrow_kernel, dim3(convert_blocks(points)), dim3(256), 0, st, (const double *)gpath64,
                               (float *)grad_path, points);
            e = hipGetLastError();
            if (e != hipSuccess) return launch_failed(e, "conversion launch");
            return PATHSIG_OK;
        }
    }
    if (dtype == PATHSIG_F32)
        return sig_backward_t<float>(path, sig, grad_sig, grad_path, B, L, d, depth, level_sizes, encoded_words,
                                     n_encoded, windows, W, chunks, chunks_bytes, workspace, workspace_bytes,
                                     (hipStream_t)stream);
    return sig_backward_t<double>(path, sig, grad_sig, grad_path, B, L, d, depth, level_sizes, encoded_words,
                                  n_encoded, windows, W, chunks, chunks_bytes, workspace, workspace_bytes,
                                  (hipStream_t)stream);
}

namespace {
int check_logsig_call(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words) {
    int rc = check_logsig(dtype, rows, d, depth, top_size);
    if (rc != PATHSIG_OK) return rc;
    if (rows > 0 && top_size != checked_pow(d, depth) && top_size > 0 && !top_words) {
        set_error("top_words is NULL but the top level is not dense");
        return PATHSIG_ERR_ARGUMENT;
    }
    return PATHSIG_OK;
}

// columns of the hybrid layout
int64_t hybrid_size(int64_t d, int depth, int64_t top_size) {
    int64_t lower = 0, width = 1;
    for (int k = 1; k < depth; ++k) {
        width *= d;
        lower += width;
    }
    return lower + top_size;
}

int logsig_forward_any(const void *sig, void *logsig, void *cache, void *powers, int dtype, int64_t rows, int64_t d,
                       int depth, int64_t top_size, const int64_t *top_words, hipStream_t stream) {
    hipError_t e;
    if (dtype == PATHSIG_F32)
        e = launch_logsig_forward<float>((const float *)sig, (float *)logsig, (float *)cache, (float *)powers, rows, d,
                                         depth, top_size, top_words, stream);
    else
        e = launch_logsig_forward<double>((const double *)sig, (double *)logsig, (double *)cache, (double *)powers, rows,
                                          d, depth, top_size, top_words, stream);
    if (e != hipSuccess) return launch_failed(e, "logsig forward launch");
    return PATHSIG_OK;
}

int logsig_backward_any(const void *logsig, const void *cache, const void *grad_logsig, void *grad_sig, int dtype,
                        int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words, void *workspace,
                        hipStream_t stream) {
    hipError_t e;
    if (dtype == PATHSIG_F32)
        e = launch_logsig_backward<float>((const float *)logsig, (const float *)cache, (const float *)grad_logsig,
                                          (float *)grad_sig, (float *)workspace, rows, d, depth, top_size, top_words,
                                          stream);
    else
        e = launch_logsig_backward<double>((const double *)logsig, (const double *)cache, (const double *)grad_logsig,
                                           (double *)grad_sig, (double *)workspace, rows, d, depth, top_size, top_words,
                                           stream);
    if (e != hipSuccess) return launch_failed(e, "logsig backward launch");
    return PATHSIG_OK;
}
}  // namespace

int pathsig_logsig_forward(const void *sig, void *logsig, void *P, int dtype, int64_t rows, int64_t d, int depth,
                           int64_t top_size, const int64_t *top_words, void *stream) {
    int rc = check_logsig_call(dtype, rows, d, depth, top_size, top_words);
    if (rc != PATHSIG_OK) return rc;
    if (rows == 0) return PATHSIG_OK;
    if (!sig || !logsig || !P) {
        set_error("sig, logsig and P must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    // P first serves as the cache of the pass that computes the values, then receives the powers
    return logsig_forward_any(sig, logsig, P, P, dtype, rows, d, depth, top_size, top_words, (hipStream_t)stream);
}

int pathsig_logsig_forward_keep(const void *sig, void *logsig, void *cache, int dtype, int64_t rows, int64_t d,
                                int depth, int64_t top_size, const int64_t *top_words, void *stream) {
    int rc = check_logsig_call(dtype, rows, d, depth, top_size, top_words);
    if (rc != PATHSIG_OK) return rc;
    if (rows == 0) return PATHSIG_OK;
    if (!sig || !logsig || !cache) {
        set_error("sig, logsig and cache must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    return logsig_forward_any(sig, logsig, cache, nullptr, dtype, rows, d, depth, top_size, top_words,
                              (hipStream_t)stream);
}

size_t pathsig_logsig_backward_kept_workspace(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size) {
    if (check_logsig(dtype, rows, d, depth, top_size) != PATHSIG_OK) return 0;
    return logsig_backward_bytes(dtype, rows, d, depth, top_size) + 256;
}

size_t pathsig_logsig_backward_workspace(int dtype, int64_t rows, int64_t d, int depth, int64_t top_size) {
    if (check_logsig(dtype, rows, d, depth, top_size) != PATHSIG_OK) return 0;
    // the log-signature and its cache are rebuilt in front of the adjoint's own scratch
    const size_t S = (size_t)hybrid_size(d, depth, top_size);
    const size_t rebuilt = align_up((size_t)rows * S * elem_size(dtype)) + align_up((size_t)rows * S * depth * elem_size(dtype));
    return rebuilt + logsig_backward_bytes(dtype, rows, d, depth, top_size) + 256;
}

int pathsig_logsig_backward(const void *sig, const void *P, const void *grad_logsig, void *grad_sig, int dtype,
                            int64_t rows, int64_t d, int depth, int64_t top_size, const int64_t *top_words,
                            void *workspace, size_t workspace_bytes, void *stream) {
    (void)P;  // the adjoint works from the cache of the Q form, which it rebuilds from sig
    int rc = check_logsig_call(dtype, rows, d, depth, top_size, top_words);
    if (rc != PATHSIG_OK) return rc;
    if (rows == 0) return PATHSIG_OK;
    if (!sig || !grad_logsig || !grad_sig) {
        set_error("sig, grad_logsig and grad_sig must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    const size_t S = (size_t)hybrid_size(d, depth, top_size);
    const size_t lg_bytes = align_up((size_t)rows * S * elem_size(dtype));
    const size_t cache_bytes = align_up((size_t)rows * S * depth * elem_size(dtype));
    const size_t need = lg_bytes + cache_bytes + logsig_backward_bytes(dtype, rows, d, depth, top_size);
    if (!workspace || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return PATHSIG_ERR_WORKSPACE;
    }
    unsigned char *ws = (unsigned char *)workspace;
    void *lg = ws, *cache = ws + lg_bytes, *rest = ws + lg_bytes + cache_bytes;
    rc = logsig_forward_any(sig, lg, cache, nullptr, dtype, rows, d, depth, top_size, top_words, (hipStream_t)stream);
    if (rc != PATHSIG_OK) return rc;
    return logsig_backward_any(lg, cache, grad_logsig, grad_sig, dtype, rows, d, depth, top_size, top_words, rest,
                               (hipStream_t)stream);
}

int pathsig_logsig_backward_kept(const void *logsig, const void *cache, const void *grad_logsig, void *grad_sig,
                                 int dtype, int64_t rows, int64_t d, int depth, int64_t top_size,
                                 const int64_t *top_words, void *workspace, size_t workspace_bytes, void *stream) {
    int rc = check_logsig_call(dtype, rows, d, depth, top_size, top_words);
    if (rc != PATHSIG_OK) return rc;
    if (rows == 0) return PATHSIG_OK;
    if (!logsig || !cache || !grad_logsig || !grad_sig) {
        set_error("logsig, cache, grad_logsig and grad_sig must not be NULL");
        return PATHSIG_ERR_ARGUMENT;
    }
    const size_t need = logsig_backward_bytes(dtype, rows, d, depth, top_size);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return PATHSIG_ERR_WORKSPACE;
    }
    return logsig_backward_any(logsig, cache, grad_logsig, grad_sig, dtype, rows, d, depth, top_size, top_words,
                               workspace, (hipStream_t)stream);
}

}  // extern "C"
