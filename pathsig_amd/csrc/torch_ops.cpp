// Registration of the `pathsig` operators with the torch dispatcher, in C++.
//
// Schemas are those of the reference (`src/pathsig/bindings.cpp:9-63`); argument checks, output shapes and
// the autograd formulas follow `src/pathsig/ops.py:59-297`.  Each device implementation makes its inputs
// contiguous, allocates outputs and scratch with torch (so they are stream-ordered) and hands raw pointers
// plus the current HIP stream to the C ABI declared in pathsig_hip.h.  The autograd nodes are C++ too, so a
// forward + backward step runs without entering the Python interpreter (which costs several times the GPU
// time of small workloads when the same registration is done from Python).
#include <ATen/ATen.h>
#include <ATen/core/dispatch/Dispatcher.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/autograd.h>
#include <torch/library.h>

#include <limits>
#include <tuple>
#include <vector>

#include "pathsig_hip.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

int dtype_code(const Tensor &t, const char *what) {
    if (t.scalar_type() == at::kFloat) return PATHSIG_F32;
    if (t.scalar_type() == at::kDouble) return PATHSIG_F64;
    TORCH_CHECK(false, what, " must be float32 or float64");
}

void *ptr(const Tensor &t) { return t.defined() && t.numel() > 0 ? t.data_ptr() : nullptr; }

void check_rc(int rc) { TORCH_CHECK(rc == PATHSIG_OK, "pathsig: ", pathsig_last_error(), " (error ", rc, ")"); }

void *stream_of(const Tensor &t) { return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

Tensor scratch(size_t nbytes, const Tensor &like) {
    if (nbytes == 0) return Tensor();
    return at::empty({(int64_t)nbytes}, like.options().dtype(at::kByte));
}

void check_words_arg(const Tensor &encoded_words) {
    TORCH_CHECK(encoded_words.is_cuda(), "encoded_words must be CUDA");
    TORCH_CHECK(encoded_words.scalar_type() == at::kLong, "encoded_words must be int64");
    TORCH_CHECK(encoded_words.dim() == 1, "encoded_words must be 1D");
}

Tensor windows_arg(const Tensor &windows) {
    TORCH_CHECK(windows.is_cuda(), "windows must be CUDA");
    TORCH_CHECK(windows.dim() == 2 && windows.size(1) == 2, "windows must be [W,2]");
    TORCH_CHECK(windows.scalar_type() == at::kInt || windows.scalar_type() == at::kLong,
                "windows must be int32 or int64");
    return windows.to(at::kInt).contiguous();
}

// sum of d^k for k = 1..depth (the dense signature size); fails instead of overflowing
int64_t dense_size(int64_t d, int64_t first, int64_t last) {
    int64_t total = 0, width = 1;
    for (int64_t k = 1; k <= last; ++k) {
        TORCH_CHECK(d == 0 || width <= std::numeric_limits<int64_t>::max() / (d > 0 ? d : 1),
                    "d^depth does not fit 64 bits");
        width *= d;
        if (k >= first) {
            TORCH_CHECK(total <= std::numeric_limits<int64_t>::max() - width, "signature size does not fit 64 bits");
            total += width;
        }
    }
    return total;
}

// arguments shared by the signature forward and backward
struct SigCall {
    Tensor path, words, win;
    int dt;
    int64_t B, L, d, depth, W, sig_size;
    const int64_t *sizes;  // host
    int64_t n_words;
};

SigCall sig_call(const Tensor &path_in, int64_t depth, bool alt, const Tensor &encoded_words,
                 at::IntArrayRef level_sizes, bool use_windows, const Tensor &windows) {
    SigCall c;
    TORCH_CHECK(path_in.is_cuda(), "path must be CUDA");
    TORCH_CHECK(path_in.dim() == 3, "path must be [B,T,d]");
    c.dt = dtype_code(path_in, "path");
    TORCH_CHECK(depth >= 1 && depth <= PATHSIG_MAX_DEPTH, "depth must be in [1,12]");
    c.depth = depth;
    c.path = path_in.contiguous();
    c.B = c.path.size(0);
    c.L = c.path.size(1);
    c.d = c.path.size(2);
    TORCH_CHECK(c.L >= 2, "path must have at least 2 time steps");
    c.sizes = nullptr;
    c.n_words = 0;
    if (alt) {
        check_words_arg(encoded_words);
        TORCH_CHECK((int64_t)level_sizes.size() >= depth + 1, "level_sizes must cover at least depth + 1 entries");
        c.words = encoded_words.contiguous();
        c.n_words = c.words.numel();
        c.sizes = level_sizes.data();
        c.sig_size = 0;
        for (int64_t k = 1; k <= depth; ++k) c.sig_size += level_sizes[k];
    } else {
        c.sig_size = dense_size(c.d, 1, depth);
    }
    c.W = 0;
    if (use_windows) {
        c.win = windows_arg(windows);
        c.W = c.win.size(0);
    }
    return c;
}

std::tuple<Tensor, Tensor> sig_forward(const Tensor &path_in, int64_t depth, bool alt, const Tensor &encoded_words,
                                       at::IntArrayRef level_sizes, bool use_windows, const Tensor &windows,
                                       bool keep) {
    const SigCall c = sig_call(path_in, depth, alt, encoded_words, level_sizes, use_windows, windows);
    c10::DeviceGuard guard(c.path.device());
    Tensor out = use_windows ? at::empty({c.B, c.W, c.sig_size}, c.path.options())
                             : at::empty({c.B, c.sig_size}, c.path.options());
    Tensor chunks;
    size_t chunk_bytes = 0;
    if (keep) {
        chunk_bytes = pathsig_sig_chunks_bytes(c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes, c.W);
        chunks = at::empty({(int64_t)(chunk_bytes / c.path.element_size())}, c.path.options());
    }
    const size_t ws_bytes = pathsig_sig_forward_workspace(c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes, c.W);
    Tensor ws = scratch(ws_bytes, c.path);
    check_rc(pathsig_sig_forward_keep(ptr(c.path), ptr(out), c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes,
                                      (const int64_t *)ptr(c.words), c.n_words,
                                      use_windows ? (const int32_t *)ptr(c.win) : nullptr, c.W, ptr(chunks),
                                      chunk_bytes, ptr(ws), ws_bytes, stream_of(c.path)));
    return {out, chunks};
}

Tensor sig_backward(const Tensor &path_in, const Tensor &signature_in, const Tensor &grad_signature_in,
                    const Tensor &chunks_in, int64_t depth, bool alt, const Tensor &encoded_words,
                    at::IntArrayRef level_sizes, bool use_windows, const Tensor &windows) {
    TORCH_CHECK(path_in.is_cuda(), "path must be CUDA");
    TORCH_CHECK(path_in.dim() == 3, "path must be [B,T,d]");
    dtype_code(path_in, "path");
    TORCH_CHECK(signature_in.is_cuda(), "signature must be CUDA");
    TORCH_CHECK(grad_signature_in.is_cuda(), "grad_signature must be CUDA");
    TORCH_CHECK(signature_in.scalar_type() == path_in.scalar_type(), "signature must have same dtype as path");
    TORCH_CHECK(grad_signature_in.scalar_type() == path_in.scalar_type(),
                "grad_signature must have same dtype as path");
    const SigCall c = sig_call(path_in, depth, alt, encoded_words, level_sizes, use_windows, windows);
    Tensor sig = signature_in.contiguous();
    Tensor grad = grad_signature_in.contiguous();
    TORCH_CHECK(sig.dim() == 2 || sig.dim() == 3, "signature must be [B,S] or [B,W,S]");
    TORCH_CHECK(sig.sizes() == grad.sizes(), "grad_signature must match signature shape");
    TORCH_CHECK(sig.size(0) == c.B, "signature batch size must match path");
    TORCH_CHECK(sig.size(-1) == c.sig_size, "signature size does not match depth / projection");
    if (use_windows) {
        TORCH_CHECK(sig.dim() == 3 && sig.size(1) == c.W, "windows.size(0) must match signature num_windows");
    } else {
        TORCH_CHECK(sig.dim() == 2, "signature must be [B,S] when no windows are used");
    }
    Tensor chunks;
    if (chunks_in.defined() && chunks_in.numel() > 0) {
        TORCH_CHECK(chunks_in.is_cuda() && chunks_in.scalar_type() == path_in.scalar_type(),
                    "chunks must be a CUDA tensor of the path's dtype");
        chunks = chunks_in.contiguous();
        // kept under other tuning switches than the ones in force now (its size tells): the backward recomputes
        const size_t now = pathsig_sig_chunks_bytes(c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes, c.W);
        if ((size_t)chunks.numel() * chunks.element_size() != now) chunks = Tensor();
    }
    c10::DeviceGuard guard(c.path.device());
    Tensor out = at::empty_like(c.path);
    const size_t ws_bytes = pathsig_sig_backward_workspace(c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes, c.W);
    Tensor ws = scratch(ws_bytes, c.path);
    check_rc(pathsig_sig_backward_kept(
        ptr(c.path), ptr(sig), ptr(grad), ptr(out), c.dt, c.B, c.L, c.d, (int)c.depth, c.sizes,
        (const int64_t *)ptr(c.words), c.n_words, use_windows ? (const int32_t *)ptr(c.win) : nullptr, c.W, ptr(chunks),
        chunks.defined() ? (size_t)chunks.numel() * chunks.element_size() : 0, ptr(ws), ws_bytes, stream_of(c.path)));
    return out;
}

// ---- device implementations (dispatch key CUDA == HIP on ROCm builds) ------------------------------------
Tensor compute_signature_hip(const Tensor &path, int64_t depth, bool alt, const Tensor &words,
                             at::IntArrayRef level_sizes, bool use_windows, const Tensor &windows) {
    return std::get<0>(sig_forward(path, depth, alt, words, level_sizes, use_windows, windows, false));
}

std::tuple<Tensor, Tensor> compute_signature_keep_hip(const Tensor &path, int64_t depth, bool alt, const Tensor &words,
                                                      at::IntArrayRef level_sizes, bool use_windows,
                                                      const Tensor &windows) {
    return sig_forward(path, depth, alt, words, level_sizes, use_windows, windows, true);
}

Tensor signature_backward_hip(const Tensor &path, const Tensor &sig, const Tensor &grad, int64_t depth, bool alt,
                              const Tensor &words, at::IntArrayRef level_sizes, bool use_windows,
                              const Tensor &windows) {
    return sig_backward(path, sig, grad, Tensor(), depth, alt, words, level_sizes, use_windows, windows);
}

Tensor signature_backward_kept_hip(const Tensor &path, const Tensor &sig, const Tensor &grad, const Tensor &chunks,
                                   int64_t depth, bool alt, const Tensor &words, at::IntArrayRef level_sizes,
                                   bool use_windows, const Tensor &windows) {
    return sig_backward(path, sig, grad, chunks, depth, alt, words, level_sizes, use_windows, windows);
}

// size of the top level of the hybrid layout (levels below `depth` dense, level `depth` as given)
int64_t hybrid_top(const Tensor &signature, int64_t depth, int64_t d, bool alt, at::IntArrayRef level_sizes) {
    const int64_t lower = dense_size(d, 1, depth - 1);
    int64_t top;
    if (alt) {
        TORCH_CHECK((int64_t)level_sizes.size() >= depth + 1, "level_sizes must have entries up to depth");
        top = level_sizes[depth];
    } else {
        top = dense_size(d, depth, depth);
    }
    TORCH_CHECK(signature.size(-1) == lower + top, "signature size does not match the hybrid layout");
    return top;
}

// arguments shared by the log-signature operators: the hybrid-layout tensor `like` fixes rows and columns
struct LogCall {
    Tensor words;
    int dt;
    int64_t depth, d, top, S, rows;
};

LogCall log_call(const Tensor &like, const char *what, int64_t depth, int64_t d, bool alt, const Tensor &encoded_words,
                 at::IntArrayRef level_sizes) {
    LogCall c;
    TORCH_CHECK(like.is_cuda(), what, " must be CUDA");
    c.dt = dtype_code(like, what);
    TORCH_CHECK(depth >= 1 && depth <= PATHSIG_MAX_DEPTH, "depth must be in [1,12]");
    TORCH_CHECK(d >= 1, "d must be >= 1");
    TORCH_CHECK(like.dim() == 2 || like.dim() == 3, what, " must be [B,S] or [B,W,S]");
    c.depth = depth;
    c.d = d;
    if (alt) {
        check_words_arg(encoded_words);
        c.words = encoded_words.contiguous();
    }
    c.top = hybrid_top(like, depth, d, alt, level_sizes);
    if (c.words.defined() && c.top != dense_size(d, depth, depth)) {
        TORCH_CHECK(c.words.numel() >= c.top, "encoded_words is shorter than the top level");
    }
    c.S = like.size(-1);
    c.rows = c.S > 0 ? like.numel() / c.S : 0;
    return c;
}

std::vector<int64_t> cache_shape_of(const Tensor &sig, int64_t depth) {
    std::vector<int64_t> shape(sig.sizes().begin(), sig.sizes().end());
    shape.back() = sig.size(-1) * depth;
    return shape;
}

// keep: the second output is the cache the adjoint reads (powers of the log-signature) instead of the power
// cache of the reference
std::tuple<Tensor, Tensor> logsig_forward(const Tensor &signature_in, int64_t depth, int64_t d, bool alt,
                                          const Tensor &encoded_words, at::IntArrayRef level_sizes, bool keep) {
    const LogCall c = log_call(signature_in, "signature", depth, d, alt, encoded_words, level_sizes);
    Tensor sig = signature_in.contiguous();
    c10::DeviceGuard guard(sig.device());
    Tensor logsig = at::empty_like(sig);
    Tensor cache = at::empty(cache_shape_of(sig, depth), sig.options());
    if (keep)
        check_rc(pathsig_logsig_forward_keep(ptr(sig), ptr(logsig), ptr(cache), c.dt, c.rows, d, (int)depth, c.top,
                                             (const int64_t *)ptr(c.words), stream_of(sig)));
    else
        check_rc(pathsig_logsig_forward(ptr(sig), ptr(logsig), ptr(cache), c.dt, c.rows, d, (int)depth, c.top,
                                        (const int64_t *)ptr(c.words), stream_of(sig)));
    return {logsig, cache};
}

std::tuple<Tensor, Tensor> sig_to_logsig_hip(const Tensor &signature_in, int64_t depth, int64_t d, bool alt,
                                             const Tensor &encoded_words, at::IntArrayRef level_sizes) {
    return logsig_forward(signature_in, depth, d, alt, encoded_words, level_sizes, false);
}

std::tuple<Tensor, Tensor> sig_to_logsig_keep_hip(const Tensor &signature_in, int64_t depth, int64_t d, bool alt,
                                                  const Tensor &encoded_words, at::IntArrayRef level_sizes) {
    return logsig_forward(signature_in, depth, d, alt, encoded_words, level_sizes, true);
}

// first_in is the signature (kept == false; cache_in is then the reference's P, which is only checked for its
// shape) or the log-signature of the keeping forward (kept == true; cache_in is its cache)
Tensor logsig_backward_any(const Tensor &first_in, const Tensor &cache_in, const Tensor &grad_logsig_in, int64_t depth,
                           bool alt, const Tensor &encoded_words, at::IntArrayRef level_sizes, bool kept) {
    const char *first_name = kept ? "logsig" : "sig";
    TORCH_CHECK(cache_in.is_cuda(), kept ? "cache" : "P", " must be CUDA");
    TORCH_CHECK(grad_logsig_in.is_cuda(), "grad_logsig must be CUDA");
    TORCH_CHECK((int64_t)level_sizes.size() > depth && depth >= 1, "level_sizes must have entries up to depth");
    const int64_t d = level_sizes[1];  // the path dimension is read off the (always dense) first level
    TORCH_CHECK(d >= 1, "level_sizes[1] must be >= 1 (infers path_dim)");
    const LogCall c = log_call(first_in, first_name, depth, d, alt, encoded_words, level_sizes);
    TORCH_CHECK(cache_in.scalar_type() == first_in.scalar_type(), "P must have same dtype as sig");
    TORCH_CHECK(grad_logsig_in.scalar_type() == first_in.scalar_type(), "grad_logsig must have same dtype as sig");
    Tensor first = first_in.contiguous();
    Tensor cache = cache_in.contiguous();
    Tensor grad = grad_logsig_in.contiguous();
    TORCH_CHECK(first.sizes() == grad.sizes(), "grad_logsig must match sig shape");
    TORCH_CHECK(cache.sizes() == at::IntArrayRef(cache_shape_of(first, depth)), "P must be [..., S*depth]");
    c10::DeviceGuard guard(first.device());
    Tensor out = at::empty_like(first);
    if (kept) {
        const size_t ws_bytes = pathsig_logsig_backward_kept_workspace(c.dt, c.rows, d, (int)depth, c.top);
        Tensor ws = scratch(ws_bytes, first);
        check_rc(pathsig_logsig_backward_kept(ptr(first), ptr(cache), ptr(grad), ptr(out), c.dt, c.rows, d, (int)depth,
                                              c.top, (const int64_t *)ptr(c.words), ptr(ws), ws_bytes,
                                              stream_of(first)));
    } else {
        const size_t ws_bytes = pathsig_logsig_backward_workspace(c.dt, c.rows, d, (int)depth, c.top);
        Tensor ws = scratch(ws_bytes, first);
        check_rc(pathsig_logsig_backward(ptr(first), ptr(cache), ptr(grad), ptr(out), c.dt, c.rows, d, (int)depth, c.top,
                                         (const int64_t *)ptr(c.words), ptr(ws), ws_bytes, stream_of(first)));
    }
    return out;
}

Tensor logsig_backward_hip(const Tensor &signature_in, const Tensor &P_in, const Tensor &grad_logsig_in, int64_t depth,
                           bool alt, const Tensor &encoded_words, at::IntArrayRef level_sizes) {
    return logsig_backward_any(signature_in, P_in, grad_logsig_in, depth, alt, encoded_words, level_sizes, false);
}

Tensor logsig_backward_kept_hip(const Tensor &logsig_in, const Tensor &cache_in, const Tensor &grad_logsig_in,
                                int64_t depth, bool alt, const Tensor &encoded_words, at::IntArrayRef level_sizes) {
    return logsig_backward_any(logsig_in, cache_in, grad_logsig_in, depth, alt, encoded_words, level_sizes, true);
}

// ---- autograd (`src/pathsig/ops.py:231-297`) ---------------------------------------------------------------
template <typename Signature>
auto typed_op(const char *name) {
    return c10::Dispatcher::singleton().findSchemaOrThrow(name, "").typed<Signature>();
}

using SigForward = Tensor(const Tensor &, int64_t, bool, const Tensor &, at::IntArrayRef, bool, const Tensor &);
using SigForwardKeep = std::tuple<Tensor, Tensor>(const Tensor &, int64_t, bool, const Tensor &, at::IntArrayRef, bool,
                                                  const Tensor &);
using SigBackward = Tensor(const Tensor &, const Tensor &, const Tensor &, int64_t, bool, const Tensor &,
                           at::IntArrayRef, bool, const Tensor &);
using SigBackwardKept = Tensor(const Tensor &, const Tensor &, const Tensor &, const Tensor &, int64_t, bool,
                               const Tensor &, at::IntArrayRef, bool, const Tensor &);
using LogForward = std::tuple<Tensor, Tensor>(const Tensor &, int64_t, int64_t, bool, const Tensor &, at::IntArrayRef);
using LogBackward = Tensor(const Tensor &, const Tensor &, const Tensor &, int64_t, bool, const Tensor &,
                           at::IntArrayRef);

// saves (path, output, windows, encoded_words); only the path gets a gradient
struct SignatureFunction : public torch::autograd::Function<SignatureFunction> {
    static Tensor forward(AutogradContext *ctx, const Tensor &path, int64_t depth, bool alt, const Tensor &words,
                          std::vector<int64_t> level_sizes, bool use_windows, const Tensor &windows) {
        at::AutoDispatchBelowADInplaceOrView below;
        static auto op = typed_op<SigForward>("pathsig::compute_signature");
        Tensor out = op.call(path, depth, alt, words, level_sizes, use_windows, windows);
        ctx->save_for_backward({path, out, windows, words});
        ctx->saved_data["depth"] = depth;
        ctx->saved_data["alt"] = alt;
        ctx->saved_data["level_sizes"] = level_sizes;
        ctx->saved_data["use_windows"] = use_windows;
        return out;
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        Tensor grad_path;
        if (ctx->needs_input_grad(0) && grads[0].defined()) {
            static auto op = typed_op<SigBackward>("pathsig::signature_backward");
            grad_path = op.call(saved[0], saved[1], grads[0], ctx->saved_data["depth"].toInt(),
                                ctx->saved_data["alt"].toBool(), saved[3], ctx->saved_data["level_sizes"].toIntVector(),
                                ctx->saved_data["use_windows"].toBool(), saved[2]);
        }
        return {grad_path, Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

// the same with the chunk signatures handed from the forward to the backward
struct SignatureKeepFunction : public torch::autograd::Function<SignatureKeepFunction> {
    static variable_list forward(AutogradContext *ctx, const Tensor &path, int64_t depth, bool alt, const Tensor &words,
                                 std::vector<int64_t> level_sizes, bool use_windows, const Tensor &windows) {
        at::AutoDispatchBelowADInplaceOrView below;
        static auto op = typed_op<SigForwardKeep>("pathsig::compute_signature_keep");
        auto [out, chunks] = op.call(path, depth, alt, words, level_sizes, use_windows, windows);
        ctx->save_for_backward({path, out, chunks, windows, words});
        ctx->saved_data["depth"] = depth;
        ctx->saved_data["alt"] = alt;
        ctx->saved_data["level_sizes"] = level_sizes;
        ctx->saved_data["use_windows"] = use_windows;
        ctx->set_materialize_grads(false);
        ctx->mark_non_differentiable({chunks});
        return {out, chunks};
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        Tensor grad_path;
        if (ctx->needs_input_grad(0) && grads[0].defined()) {
            static auto op = typed_op<SigBackwardKept>("pathsig::signature_backward_kept");
            grad_path = op.call(saved[0], saved[1], grads[0], saved[2], ctx->saved_data["depth"].toInt(),
                                ctx->saved_data["alt"].toBool(), saved[4], ctx->saved_data["level_sizes"].toIntVector(),
                                ctx->saved_data["use_windows"].toBool(), saved[3]);
        }
        return {grad_path, Tensor(), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

// saves (signature, power cache, encoded_words); the gradient of the cache is ignored
struct LogSignatureFunction : public torch::autograd::Function<LogSignatureFunction> {
    static variable_list forward(AutogradContext *ctx, const Tensor &signature, int64_t depth, int64_t d, bool alt,
                                 const Tensor &words, std::vector<int64_t> level_sizes) {
        at::AutoDispatchBelowADInplaceOrView below;
        static auto op = typed_op<LogForward>("pathsig::sig_to_logsig");
        auto [logsig, cache] = op.call(signature, depth, d, alt, words, level_sizes);
        ctx->save_for_backward({signature, cache, words});
        ctx->saved_data["depth"] = depth;
        ctx->saved_data["alt"] = alt;
        ctx->saved_data["level_sizes"] = level_sizes;
        ctx->set_materialize_grads(false);
        return {logsig, cache};
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        Tensor grad_sig;
        if (ctx->needs_input_grad(0) && grads[0].defined()) {
            static auto op = typed_op<LogBackward>("pathsig::logsig_backward");
            grad_sig = op.call(saved[0], saved[1], grads[0], ctx->saved_data["depth"].toInt(),
                               ctx->saved_data["alt"].toBool(), saved[2], ctx->saved_data["level_sizes"].toIntVector());
        }
        return {grad_sig, Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

// the same with the log-signature and its own cache handed to the backward (saves them instead of the signature)
struct LogSignatureKeepFunction : public torch::autograd::Function<LogSignatureKeepFunction> {
    static variable_list forward(AutogradContext *ctx, const Tensor &signature, int64_t depth, int64_t d, bool alt,
                                 const Tensor &words, std::vector<int64_t> level_sizes) {
        at::AutoDispatchBelowADInplaceOrView below;
        static auto op = typed_op<LogForward>("pathsig::sig_to_logsig_keep");
        auto [logsig, cache] = op.call(signature, depth, d, alt, words, level_sizes);
        ctx->save_for_backward({logsig, cache, words});
        ctx->saved_data["depth"] = depth;
        ctx->saved_data["alt"] = alt;
        ctx->saved_data["level_sizes"] = level_sizes;
        ctx->set_materialize_grads(false);
        ctx->mark_non_differentiable({cache});
        return {logsig, cache};
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        Tensor grad_sig;
        if (ctx->needs_input_grad(0) && grads[0].defined()) {
            static auto op = typed_op<LogBackward>("pathsig::logsig_backward_kept");
            grad_sig = op.call(saved[0], saved[1], grads[0], ctx->saved_data["depth"].toInt(),
                               ctx->saved_data["alt"].toBool(), saved[2], ctx->saved_data["level_sizes"].toIntVector());
        }
        return {grad_sig, Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

Tensor compute_signature_autograd(const Tensor &path, int64_t depth, bool alt, const Tensor &words,
                                  at::IntArrayRef level_sizes, bool use_windows, const Tensor &windows) {
    return SignatureFunction::apply(path, depth, alt, words, level_sizes.vec(), use_windows, windows);
}

std::tuple<Tensor, Tensor> compute_signature_keep_autograd(const Tensor &path, int64_t depth, bool alt,
                                                           const Tensor &words, at::IntArrayRef level_sizes,
                                                           bool use_windows, const Tensor &windows) {
    auto out = SignatureKeepFunction::apply(path, depth, alt, words, level_sizes.vec(), use_windows, windows);
    return {out[0], out[1]};
}

std::tuple<Tensor, Tensor> sig_to_logsig_autograd(const Tensor &signature, int64_t depth, int64_t d, bool alt,
                                                  const Tensor &words, at::IntArrayRef level_sizes) {
    auto out = LogSignatureFunction::apply(signature, depth, d, alt, words, level_sizes.vec());
    return {out[0], out[1]};
}

std::tuple<Tensor, Tensor> sig_to_logsig_keep_autograd(const Tensor &signature, int64_t depth, int64_t d, bool alt,
                                                       const Tensor &words, at::IntArrayRef level_sizes) {
    auto out = LogSignatureKeepFunction::apply(signature, depth, d, alt, words, level_sizes.vec());
    return {out[0], out[1]};
}

}  // namespace

TORCH_LIBRARY(pathsig, m) {
    const std::vector<at::Tag> pt2{at::Tag::pt2_compliant_tag};
    m.def("compute_signature(Tensor path_in, int depth, bool alternative_projection, Tensor encoded_words, "
          "int[] level_sizes, bool use_windows, Tensor windows) -> Tensor", pt2);
    m.def("signature_backward(Tensor path_in, Tensor signature_in, Tensor grad_signature_in, int depth, "
          "bool alternative_projection, Tensor encoded_words, int[] level_sizes, bool use_windows, Tensor windows) "
          "-> Tensor", pt2);
    m.def("sig_to_logsig(Tensor signature_in, int depth, int d, bool alternative_projection, Tensor encoded_words, "
          "int[] level_sizes) -> (Tensor, Tensor)", pt2);
    m.def("logsig_backward(Tensor signature_in, Tensor P_in, Tensor grad_logsig_in, int depth, "
          "bool alternative_projection, Tensor encoded_words, int[] level_sizes) -> Tensor", pt2);
    // not in the reference: the forward also returns the signatures of its time chunks below the top level (an
    // empty tensor when the call is not time-chunked); the backward that receives them does not recompute them
    m.def("compute_signature_keep(Tensor path_in, int depth, bool alternative_projection, Tensor encoded_words, "
          "int[] level_sizes, bool use_windows, Tensor windows) -> (Tensor, Tensor)", pt2);
    m.def("signature_backward_kept(Tensor path_in, Tensor signature_in, Tensor grad_signature_in, Tensor chunks, "
          "int depth, bool alternative_projection, Tensor encoded_words, int[] level_sizes, bool use_windows, "
          "Tensor windows) -> Tensor", pt2);
    // not in the reference: the second output is the cache of the adjoint (powers of the log-signature), and the
    // backward takes the log-signature and that cache instead of the signature and the power cache
    m.def("sig_to_logsig_keep(Tensor signature_in, int depth, int d, bool alternative_projection, "
          "Tensor encoded_words, int[] level_sizes) -> (Tensor, Tensor)", pt2);
    m.def("logsig_backward_kept(Tensor logsig_in, Tensor cache_in, Tensor grad_logsig_in, int depth, "
          "bool alternative_projection, Tensor encoded_words, int[] level_sizes) -> Tensor", pt2);
}

TORCH_LIBRARY_IMPL(pathsig, CUDA, m) {
    m.impl("compute_signature", &compute_signature_hip);
    m.impl("signature_backward", &signature_backward_hip);
    m.impl("sig_to_logsig", &sig_to_logsig_hip);
    m.impl("logsig_backward", &logsig_backward_hip);
    m.impl("compute_signature_keep", &compute_signature_keep_hip);
    m.impl("signature_backward_kept", &signature_backward_kept_hip);
    m.impl("sig_to_logsig_keep", &sig_to_logsig_keep_hip);
    m.impl("logsig_backward_kept", &logsig_backward_kept_hip);
}

TORCH_LIBRARY_IMPL(pathsig, Autograd, m) {
    m.impl("compute_signature", &compute_signature_autograd);
    m.impl("sig_to_logsig", &sig_to_logsig_autograd);
    m.impl("compute_signature_keep", &compute_signature_keep_autograd);
    m.impl("sig_to_logsig_keep", &sig_to_logsig_keep_autograd);
}
