"""The four operators of the torch library namespace `pathsig`, backed by libpathsig_hip.so.

Schemas are those of the reference (`src/pathsig/bindings.cpp:9-63`); shape inference for fake/meta
tensors and the autograd formulas follow `src/pathsig/ops.py:59-297`.  The device implementation
makes its inputs contiguous, allocates outputs and scratch with torch (so they are stream-ordered),
and hands raw pointers plus the current HIP stream to the C ABI declared in include/pathsig_hip.h.
"""
from __future__ import annotations

import ctypes
import os
from typing import Sequence

import torch
from torch import Tensor

from . import _load

__all__ = ["compute_signature", "sig_to_logsig", "signature_backward", "logsig_backward"]

_F32, _F64 = 0, 1

# The C++ registration (csrc/torch_ops.cpp: schemas, device implementations and autograd nodes) is used when
# it is built; otherwise the same is registered from Python below.  Shape inference for fake tensors is
# registered from Python in both cases.
_NATIVE_OPS = _load.load_torch_ops()
_library = torch.library.Library("pathsig", "FRAGMENT" if _NATIVE_OPS else "DEF")
_PT2 = (torch.Tag.pt2_compliant_tag,)


def _define_schemas() -> None:
    _library.define(
        "compute_signature(Tensor path_in, int depth, bool alternative_projection, Tensor encoded_words, "
        "int[] level_sizes, bool use_windows, Tensor windows) -> Tensor", tags=_PT2)
    _library.define(
        "signature_backward(Tensor path_in, Tensor signature_in, Tensor grad_signature_in, int depth, "
        "bool alternative_projection, Tensor encoded_words, int[] level_sizes, bool use_windows, Tensor windows) -> Tensor",
        tags=_PT2)
    _library.define(
        "sig_to_logsig(Tensor signature_in, int depth, int d, bool alternative_projection, Tensor encoded_words, "
        "int[] level_sizes) -> (Tensor, Tensor)", tags=_PT2)
    # The same signature pair with a hand-over from the forward to the backward (not in the reference): the forward
    # also returns the signatures of its time chunks below the top level (an empty tensor when the call is not
    # time-chunked), and the backward that receives them skips the launch that would recompute them.
    _library.define(
        "compute_signature_keep(Tensor path_in, int depth, bool alternative_projection, Tensor encoded_words, "
        "int[] level_sizes, bool use_windows, Tensor windows) -> (Tensor, Tensor)", tags=_PT2)
    _library.define(
        "signature_backward_kept(Tensor path_in, Tensor signature_in, Tensor grad_signature_in, Tensor chunks, int depth, "
        "bool alternative_projection, Tensor encoded_words, int[] level_sizes, bool use_windows, Tensor windows) -> Tensor",
        tags=_PT2)
    _library.define(
        "logsig_backward(Tensor signature_in, Tensor P_in, Tensor grad_logsig_in, int depth, "
        "bool alternative_projection, Tensor encoded_words, int[] level_sizes) -> Tensor", tags=_PT2)


if not _NATIVE_OPS:
    _define_schemas()


# ------------------------------------------------------------------------------------------------
# helpers for the device implementations
# ------------------------------------------------------------------------------------------------
def _fail(rc: int) -> None:
    msg = _load.lib().pathsig_last_error().decode("utf-8", "replace")
    raise RuntimeError(f"pathsig: {msg} (error {rc})")


def _dtype_code(t: Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.float64:
        return _F64
    raise RuntimeError("path must be float32 or float64")


def _ptr(t: Tensor | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None or t.numel() == 0 else t.data_ptr())


def _host_i64(values: Sequence[int]):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


# handle of the current stream without building a torch.cuda.Stream object (about 2 us less per call)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device) -> ctypes.c_void_p:
    if _raw_stream is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _scratch(nbytes: int, device: torch.device) -> Tensor | None:
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes > 0 else None


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_words_arg(encoded_words: Tensor) -> None:
    _require(encoded_words.is_cuda, "encoded_words must be CUDA")
    _require(encoded_words.dtype == torch.int64, "encoded_words must be int64")
    _require(encoded_words.dim() == 1, "encoded_words must be 1D")


def _windows_arg(windows: Tensor) -> Tensor:
    _require(windows.is_cuda, "windows must be CUDA")
    _require(windows.dim() == 2 and windows.size(1) == 2, "windows must be [W,2]")
    _require(windows.dtype in (torch.int32, torch.int64), "windows must be int32 or int64")
    return windows.to(torch.int32).contiguous()


# ------------------------------------------------------------------------------------------------
# device implementations (dispatch key CUDA == HIP on ROCm builds)
# ------------------------------------------------------------------------------------------------
def _chunks_numel(path: Tensor, depth: int, alternative_projection: bool, level_sizes, W: int) -> int:
    """Elements of the chunk buffer a forward on `path` can hand to its backward (0: nothing to hand over)."""
    B, L, d = (int(n) for n in path.shape)
    sizes_host = _host_i64(level_sizes) if alternative_projection else None
    nbytes = _load.lib().pathsig_sig_chunks_bytes(_dtype_code(path), B, L, d, int(depth), sizes_host, int(W))
    return int(nbytes) // path.element_size()


def _sig_forward(path_in, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows, keep):
    _require(path_in.is_cuda, "path must be CUDA")
    _require(path_in.dim() == 3, "path must be [B,T,d]")
    dt = _dtype_code(path_in)
    depth = int(depth)
    _require(1 <= depth <= 12, "depth must be in [1,12]")
    path = path_in.contiguous()
    B, L, d = path.shape
    _require(L >= 2, "path must have at least 2 time steps")
    sizes_host = None
    words = None
    if alternative_projection:
        _check_words_arg(encoded_words)
        _require(len(level_sizes) >= depth + 1, "level_sizes must cover at least depth + 1 entries")
        words = encoded_words.contiguous()
        sizes_host = _host_i64(level_sizes)
        sig_size = int(sum(level_sizes[1:depth + 1]))
    else:
        sig_size = sum(d ** k for k in range(1, depth + 1))
    win = _windows_arg(windows) if use_windows else None
    W = int(win.size(0)) if win is not None else 0
    out = torch.empty((B, W, sig_size) if use_windows else (B, sig_size), dtype=path.dtype, device=path.device)
    lib = _load.lib()
    chunks = None
    with torch.cuda.device(path.device):
        if keep:
            n_keep = lib.pathsig_sig_chunks_bytes(dt, B, L, d, depth, sizes_host, W) // path.element_size()
            chunks = torch.empty(n_keep, dtype=path.dtype, device=path.device)
        ws_bytes = lib.pathsig_sig_forward_workspace(dt, B, L, d, depth, sizes_host, W)
        ws = _scratch(ws_bytes, path.device)
        rc = lib.pathsig_sig_forward_keep(
            _ptr(path), _ptr(out), dt, B, L, d, depth, sizes_host, _ptr(words), 0 if words is None else words.numel(),
            _ptr(win) if use_windows else None, W, _ptr(chunks), 0 if chunks is None else chunks.numel() * chunks.element_size(),
            _ptr(ws), ws_bytes, _stream(path.device))
    if rc != 0:
        _fail(rc)
    return out, chunks


def _compute_signature_hip(path_in, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows):
    return _sig_forward(path_in, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows,
                        keep=False)[0]


def _compute_signature_keep_hip(path_in, depth, alternative_projection, encoded_words, level_sizes, use_windows,
                                windows):
    return _sig_forward(path_in, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows,
                        keep=True)


def _sig_backward(path_in, signature_in, grad_signature_in, chunks, depth, alternative_projection, encoded_words,
                  level_sizes, use_windows, windows):
    _require(path_in.is_cuda, "path must be CUDA")
    _require(path_in.dim() == 3, "path must be [B,T,d]")
    dt = _dtype_code(path_in)
    _require(signature_in.is_cuda, "signature must be CUDA")
    _require(grad_signature_in.is_cuda, "grad_signature must be CUDA")
    _require(signature_in.dtype == path_in.dtype, "signature must have same dtype as path")
    _require(grad_signature_in.dtype == path_in.dtype, "grad_signature must have same dtype as path")
    depth = int(depth)
    _require(1 <= depth <= 12, "depth must be in [1,12]")
    path = path_in.contiguous()
    sig = signature_in.contiguous()
    grad = grad_signature_in.contiguous()
    B, L, d = path.shape
    _require(L >= 2, "path must have at least 2 time steps")
    _require(sig.dim() in (2, 3), "signature must be [B,S] or [B,W,S]")
    _require(sig.shape == grad.shape, "grad_signature must match signature shape")
    _require(sig.size(0) == B, "signature batch size must match path")
    sizes_host = None
    words = None
    if alternative_projection:
        _check_words_arg(encoded_words)
        _require(len(level_sizes) >= depth + 1, "level_sizes must cover at least depth + 1 entries")
        words = encoded_words.contiguous()
        sizes_host = _host_i64(level_sizes)
        sig_size = int(sum(level_sizes[1:depth + 1]))
    else:
        sig_size = sum(d ** k for k in range(1, depth + 1))
    _require(sig.size(-1) == sig_size, "signature size does not match depth / projection")
    win = None
    W = 0
    if use_windows:
        win = _windows_arg(windows)
        W = int(win.size(0))
        _require(sig.dim() == 3 and sig.size(1) == W, "windows.size(0) must match signature num_windows")
    else:
        _require(sig.dim() == 2, "signature must be [B,S] when no windows are used")
    out = torch.empty_like(path)
    lib = _load.lib()
    if chunks is not None and chunks.numel() > 0:
        _require(chunks.is_cuda and chunks.dtype == path.dtype, "chunks must be a CUDA tensor of the path's dtype")
        chunks = chunks.contiguous()
    else:
        chunks = None
    with torch.cuda.device(path.device):
        ws_bytes = lib.pathsig_sig_backward_workspace(dt, B, L, d, depth, sizes_host, W)
        ws = _scratch(ws_bytes, path.device)
        rc = lib.pathsig_sig_backward_kept(
            _ptr(path), _ptr(sig), _ptr(grad), _ptr(out), dt, B, L, d, depth, sizes_host, _ptr(words),
            0 if words is None else words.numel(), _ptr(win) if use_windows else None, W, _ptr(chunks),
            0 if chunks is None else chunks.numel() * chunks.element_size(), _ptr(ws), ws_bytes, _stream(path.device))
    if rc != 0:
        _fail(rc)
    return out


def _signature_backward_hip(path_in, signature_in, grad_signature_in, depth, alternative_projection, encoded_words,
                            level_sizes, use_windows, windows):
    return _sig_backward(path_in, signature_in, grad_signature_in, None, depth, alternative_projection, encoded_words,
                         level_sizes, use_windows, windows)


def _signature_backward_kept_hip(path_in, signature_in, grad_signature_in, chunks, depth, alternative_projection,
                                 encoded_words, level_sizes, use_windows, windows):
    return _sig_backward(path_in, signature_in, grad_signature_in, chunks, depth, alternative_projection, encoded_words,
                         level_sizes, use_windows, windows)


def _hybrid_top(signature: Tensor, depth: int, d: int, alternative_projection: bool, level_sizes):
    """Size of the top level of the hybrid layout and whether it is a word list."""
    lower = sum(d ** k for k in range(1, depth))
    if alternative_projection:
        _require(len(level_sizes) >= depth + 1, "level_sizes must have entries up to depth")
        top = int(level_sizes[depth])
    else:
        top = d ** depth
    _require(signature.size(-1) == lower + top, "signature size does not match the hybrid layout")
    return top


def _sig_to_logsig_hip(signature_in, depth, d, alternative_projection, encoded_words, level_sizes):
    _require(signature_in.is_cuda, "signature must be CUDA")
    dt = _dtype_code(signature_in)
    depth, d = int(depth), int(d)
    _require(1 <= depth <= 12, "depth must be in [1,12]")
    _require(d >= 1, "d must be >= 1")
    _require(signature_in.dim() in (2, 3), "signature must be [B,S] or [B,W,S]")
    sig = signature_in.contiguous()
    words = None
    if alternative_projection:
        _check_words_arg(encoded_words)
        words = encoded_words.contiguous()
    top = _hybrid_top(sig, depth, d, alternative_projection, level_sizes)
    if words is not None and top != d ** depth:
        _require(words.numel() >= top, "encoded_words is shorter than the top level")
    S = sig.size(-1)
    rows = sig.numel() // S if S > 0 else 0
    logsig = torch.empty_like(sig)
    P = torch.empty(*sig.shape[:-1], S * depth, dtype=sig.dtype, device=sig.device)
    lib = _load.lib()
    with torch.cuda.device(sig.device):
        rc = lib.pathsig_logsig_forward(_ptr(sig), _ptr(logsig), _ptr(P), dt, rows, d, depth, top, _ptr(words),
                                        _stream(sig.device))
    if rc != 0:
        _fail(rc)
    return logsig, P


def _logsig_backward_hip(signature_in, P_in, grad_logsig_in, depth, alternative_projection, encoded_words, level_sizes):
    _require(signature_in.is_cuda, "sig must be CUDA")
    _require(P_in.is_cuda, "P must be CUDA")
    _require(grad_logsig_in.is_cuda, "grad_logsig must be CUDA")
    dt = _dtype_code(signature_in)
    _require(P_in.dtype == signature_in.dtype, "P must have same dtype as sig")
    _require(grad_logsig_in.dtype == signature_in.dtype, "grad_logsig must have same dtype as sig")
    depth = int(depth)
    _require(1 <= depth <= 12, "depth must be in [1,12]")
    _require(len(level_sizes) > depth, "level_sizes must have entries up to depth")
    d = int(level_sizes[1])  # the path dimension is read off the (always dense) first level
    _require(d >= 1, "level_sizes[1] must be >= 1 (infers path_dim)")
    sig = signature_in.contiguous()
    P = P_in.contiguous()
    grad = grad_logsig_in.contiguous()
    _require(sig.dim() in (2, 3), "sig must be [B,S] or [B,W,S]")
    _require(sig.shape == grad.shape, "grad_logsig must match sig shape")
    S = sig.size(-1)
    _require(P.shape == (*sig.shape[:-1], S * depth), "P must be [..., S*depth]")
    words = None
    if alternative_projection:
        _check_words_arg(encoded_words)
        words = encoded_words.contiguous()
    top = _hybrid_top(sig, depth, d, alternative_projection, level_sizes)
    if words is not None and top != d ** depth:
        _require(words.numel() >= top, "encoded_words is shorter than the top level")
    rows = sig.numel() // S if S > 0 else 0
    out = torch.empty_like(sig)
    lib = _load.lib()
    with torch.cuda.device(sig.device):
        ws_bytes = lib.pathsig_logsig_backward_workspace(dt, rows, d, depth, top)
        ws = _scratch(ws_bytes, sig.device)
        rc = lib.pathsig_logsig_backward(_ptr(sig), _ptr(P), _ptr(grad), _ptr(out), dt, rows, d, depth, top,
                                         _ptr(words), _ptr(ws), ws_bytes, _stream(sig.device))
    if rc != 0:
        _fail(rc)
    return out


# ------------------------------------------------------------------------------------------------
# python-level wrappers (same names and argument order as `src/pathsig/ops.py:44-56,87-98,127-149,182-194`)
# ------------------------------------------------------------------------------------------------
def compute_signature(path: Tensor, depth: int, alternative_projection: bool, encoded_words: Tensor,
                      level_sizes: list[int], use_windows: bool, windows: Tensor) -> Tensor:
    """(Windowed / projected) signature of a batch of paths.

    When a gradient will be asked for, the forward also keeps what its backward would otherwise recompute
    (the signatures of the time chunks of long paths); the values returned are the same either way."""
    if torch.is_grad_enabled() and path.requires_grad and not os.environ.get("PATHSIG_NO_KEEP"):
        return torch.ops.pathsig.compute_signature_keep.default(
            path, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows)[0]
    return torch.ops.pathsig.compute_signature.default(
        path, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows)


def sig_to_logsig(signature: Tensor, depth: int, d: int, alternative_projection: bool, encoded_words: Tensor,
                  level_sizes: list[int]) -> tuple[Tensor, Tensor]:
    """Signature in the hybrid layout -> (log-signature, power cache)."""
    return torch.ops.pathsig.sig_to_logsig.default(
        signature, depth, d, alternative_projection, encoded_words, level_sizes)


def signature_backward(path: Tensor, signature: Tensor, grad_signature: Tensor, depth: int,
                       alternative_projection: bool, encoded_words: Tensor, level_sizes: list[int],
                       use_windows: bool, windows: Tensor) -> Tensor:
    """dL/dpath from dL/dsignature."""
    return torch.ops.pathsig.signature_backward.default(
        path, signature, grad_signature, depth, alternative_projection, encoded_words, level_sizes, use_windows,
        windows)


def logsig_backward(signature: Tensor, P_arr: Tensor, grad_logsig: Tensor, depth: int, alternative_projection: bool,
                    encoded_words: Tensor, level_sizes: list[int]) -> Tensor:
    """dL/dsignature from dL/dlogsignature, using the power cache of the forward."""
    return torch.ops.pathsig.logsig_backward.default(
        signature, P_arr, grad_logsig, depth, alternative_projection, encoded_words, level_sizes)


# ------------------------------------------------------------------------------------------------
# shape inference for fake / meta tensors
# ------------------------------------------------------------------------------------------------
def _on_device(t: Tensor) -> bool:
    return t.device.type in ("cuda", "meta")


def _path_dims(path: Tensor) -> tuple[int, int, int]:
    torch._check(_on_device(path), lambda: "path must be a CUDA tensor")
    torch._check(path.dtype in (torch.float32, torch.float64), lambda: "path must be float32 or float64")
    torch._check(path.dim() == 3, lambda: "path must have shape (B, L, d)")
    B, L, d = path.shape
    torch._check(L >= 2, lambda: "path length must be at least 2")
    return B, L, d


def _windows_ok(windows: Tensor) -> None:
    torch._check(_on_device(windows), lambda: "windows must be a CUDA tensor")
    torch._check(windows.dtype in (torch.int32, torch.int64), lambda: "windows must be int32 or int64")
    torch._check(windows.dim() == 2, lambda: "windows must have shape (num_windows, 2)")
    torch._check(windows.size(1) == 2, lambda: "windows must have shape (num_windows, 2)")


def _projection_ok(encoded_words: Tensor, level_sizes, depth: int) -> None:
    torch._check(_on_device(encoded_words), lambda: "encoded_words must be a CUDA tensor")
    torch._check(encoded_words.dtype == torch.int64, lambda: "encoded_words must be int64")
    torch._check(encoded_words.dim() == 1, lambda: "encoded_words must be 1D")
    torch._check(isinstance(level_sizes, (list, tuple)), lambda: "level_sizes must be a list/tuple")
    torch._check(len(level_sizes) >= depth + 1, lambda: "level_sizes must cover at least depth + 1 entries")


def _depth_ok(depth) -> int:
    depth = int(depth)
    torch._check(1 <= depth <= 12, lambda: "depth must satisfy 1 <= depth <= 12")
    return depth


@torch.library.register_fake("pathsig::compute_signature", lib=_library)
def _compute_signature_fake(path, depth, alternative_projection, encoded_words, level_sizes, use_windows, windows):
    B, _, d = _path_dims(path)
    depth = _depth_ok(depth)
    if use_windows:
        _windows_ok(windows)
    if alternative_projection:
        _projection_ok(encoded_words, level_sizes, depth)
        size = int(sum(level_sizes[1:depth + 1]))
    else:
        size = int(sum(d ** k for k in range(1, depth + 1)))
    shape = (B, windows.size(0), size) if use_windows else (B, size)
    return torch.empty(shape, device=path.device, dtype=path.dtype)


@torch.library.register_fake("pathsig::compute_signature_keep", lib=_library)
def _compute_signature_keep_fake(path, depth, alternative_projection, encoded_words, level_sizes, use_windows,
                                 windows):
    out = _compute_signature_fake(path, depth, alternative_projection, encoded_words, level_sizes, use_windows,
                                  windows)
    n_keep = _chunks_numel(path, depth, alternative_projection, level_sizes, windows.size(0) if use_windows else 0)
    return out, torch.empty((n_keep,), device=path.device, dtype=path.dtype)


@torch.library.register_fake("pathsig::signature_backward_kept", lib=_library)
def _signature_backward_kept_fake(path, signature, grad_signature, chunks, depth, alternative_projection,
                                  encoded_words, level_sizes, use_windows, windows):
    torch._check(_on_device(chunks))
    torch._check(chunks.dim() == 1)
    return _signature_backward_fake(path, signature, grad_signature, depth, alternative_projection, encoded_words,
                                    level_sizes, use_windows, windows)


@torch.library.register_fake("pathsig::sig_to_logsig", lib=_library)
def _sig_to_logsig_fake(signature, depth, d, alternative_projection, encoded_words, level_sizes):
    torch._check(_on_device(signature), lambda: "signature must be a CUDA tensor")
    torch._check(signature.dtype in (torch.float32, torch.float64), lambda: "signature must be float32 or float64")
    depth = _depth_ok(depth)
    torch._check(int(d) >= 1, lambda: "path dimension d must be >= 1")
    torch._check(signature.dim() in (2, 3), lambda: "signature must be 2D or 3D")
    if alternative_projection:
        _projection_ok(encoded_words, level_sizes, depth)
    cache_shape = (*signature.shape[:-1], signature.shape[-1] * depth)
    return torch.empty_like(signature), torch.empty(cache_shape, device=signature.device, dtype=signature.dtype)


@torch.library.register_fake("pathsig::signature_backward", lib=_library)
def _signature_backward_fake(path, signature, grad_signature, depth, alternative_projection, encoded_words,
                             level_sizes, use_windows, windows):
    _path_dims(path)
    torch._check(_on_device(signature))
    torch._check(_on_device(grad_signature))
    torch._check(signature.dtype == path.dtype, lambda: "signature must have same dtype as path")
    torch._check(grad_signature.dtype == path.dtype, lambda: "grad_signature must have same dtype as path")
    torch._check(grad_signature.shape == signature.shape)
    depth = _depth_ok(depth)
    if use_windows:
        _windows_ok(windows)
        torch._check(signature.dim() == 3)
        torch._check(windows.size(0) == signature.size(1))
    else:
        torch._check(signature.dim() == 2)
    if alternative_projection:
        _projection_ok(encoded_words, level_sizes, depth)
    return torch.empty_like(path)


@torch.library.register_fake("pathsig::logsig_backward", lib=_library)
def _logsig_backward_fake(signature, P_arr, grad_logsig, depth, alternative_projection, encoded_words, level_sizes):
    for t in (signature, P_arr, grad_logsig):
        torch._check(_on_device(t))
    torch._check(signature.dtype in (torch.float32, torch.float64), lambda: "signature must be float32 or float64")
    torch._check(signature.dtype == grad_logsig.dtype, lambda: "signature must have same dtype as grad_logsig")
    torch._check(grad_logsig.dtype == P_arr.dtype, lambda: "grad_logsig must have same dtype as P_arr")
    depth = _depth_ok(depth)
    torch._check(grad_logsig.shape == signature.shape)
    torch._check(signature.dim() in (2, 3))
    torch._check(P_arr.dim() == signature.dim())
    torch._check(tuple(P_arr.shape[:-1]) == tuple(signature.shape[:-1]))
    torch._check(P_arr.size(-1) == signature.size(-1) * depth)
    if alternative_projection:
        _projection_ok(encoded_words, level_sizes, depth)
    return torch.empty_like(signature)


# ------------------------------------------------------------------------------------------------
# autograd
# ------------------------------------------------------------------------------------------------
def _save_for_signature(ctx, inputs, output):
    path, depth, alt, encoded_words, level_sizes, use_windows, windows = inputs
    ctx.save_for_backward(path, output, windows, encoded_words)
    ctx.depth, ctx.alt, ctx.level_sizes, ctx.use_windows = int(depth), bool(alt), level_sizes, bool(use_windows)


def _signature_vjp(ctx, grad_out):
    path, signature, windows, encoded_words = ctx.saved_tensors
    grad_path = None
    if ctx.needs_input_grad[0]:
        grad_path = torch.ops.pathsig.signature_backward.default(
            path, signature, grad_out, ctx.depth, ctx.alt, encoded_words, ctx.level_sizes, ctx.use_windows, windows)
    return grad_path, None, None, None, None, None, None




def _save_for_signature_keep(ctx, inputs, output):
    path, depth, alt, encoded_words, level_sizes, use_windows, windows = inputs
    signature, chunks = output
    ctx.save_for_backward(path, signature, chunks, windows, encoded_words)
    ctx.depth, ctx.alt, ctx.level_sizes, ctx.use_windows = int(depth), bool(alt), level_sizes, bool(use_windows)


def _signature_keep_vjp(ctx, grad_out, grad_chunks):
    path, signature, chunks, windows, encoded_words = ctx.saved_tensors
    grad_path = None
    if ctx.needs_input_grad[0]:
        grad_path = torch.ops.pathsig.signature_backward_kept.default(
            path, signature, grad_out, chunks, ctx.depth, ctx.alt, encoded_words, ctx.level_sizes, ctx.use_windows,
            windows)
    return grad_path, None, None, None, None, None, None




def _save_for_logsig(ctx, inputs, output):
    signature, depth, d, alt, encoded_words, level_sizes = inputs
    _, cache = output
    ctx.save_for_backward(signature, cache, encoded_words)
    ctx.depth, ctx.d, ctx.alt, ctx.level_sizes = int(depth), int(d), bool(alt), level_sizes


def _logsig_vjp(ctx, grad_logsig, grad_cache):
    signature, cache, encoded_words = ctx.saved_tensors
    grad_sig = None
    if ctx.needs_input_grad[0]:
        grad_sig = torch.ops.pathsig.logsig_backward.default(
            signature, cache, grad_logsig, ctx.depth, ctx.alt, encoded_words, ctx.level_sizes)
    return grad_sig, None, None, None, None, None


if not _NATIVE_OPS:
    for _name, _impl in (("compute_signature", _compute_signature_hip),
                         ("compute_signature_keep", _compute_signature_keep_hip),
                         ("signature_backward", _signature_backward_hip),
                         ("signature_backward_kept", _signature_backward_kept_hip),
                         ("sig_to_logsig", _sig_to_logsig_hip),
                         ("logsig_backward", _logsig_backward_hip)):
        _library.impl(_name, _impl, "CUDA")
    torch.library.register_autograd("pathsig::compute_signature", _signature_vjp, setup_context=_save_for_signature,
                                    lib=_library)
    torch.library.register_autograd("pathsig::compute_signature_keep", _signature_keep_vjp,
                                    setup_context=_save_for_signature_keep, lib=_library)
    torch.library.register_autograd("pathsig::sig_to_logsig", _logsig_vjp, setup_context=_save_for_logsig,
                                    lib=_library)
