"""Python side of the operators of the torch library namespace `pathsig`.

The operators themselves (schemas of `src/pathsig/bindings.cpp:9-63`, device implementations over the C ABI of
libpathsig_hip.so, autograd formulas of `src/pathsig/ops.py:231-297`) are registered in C++ by
libpathsig_torch.so.  Here: the wrappers with the reference's names and argument order
(`src/pathsig/ops.py:44-56,87-98,127-149,182-194`) and the shape inference for fake / meta tensors
(`src/pathsig/ops.py:59-84,101-123,152-179,197-227`).
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

# The operators (schemas, device implementations, autograd nodes) are registered in C++ by libpathsig_torch.so
# (csrc/torch_ops.cpp); this module adds the shape inference for fake / meta tensors and the Python wrappers.
_load.load_torch_ops()
_library = torch.library.Library("pathsig", "FRAGMENT")


def _dtype_code(t: Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.float64:
        return _F64
    raise RuntimeError("path must be float32 or float64")


def _host_i64(values: Sequence[int]):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


def _chunks_numel(path: Tensor, depth: int, alternative_projection: bool, level_sizes, W: int) -> int:
    """Elements of the chunk buffer a forward on `path` can hand to its backward (0: nothing to hand over)."""
    B, L, d = (int(n) for n in path.shape)
    sizes_host = _host_i64(level_sizes) if alternative_projection else None
    nbytes = _load.lib().pathsig_sig_chunks_bytes(_dtype_code(path), B, L, d, int(depth), sizes_host, int(W))
    return int(nbytes) // path.element_size()


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
    """Signature in the hybrid layout -> (log-signature, P_arr).

    The second output is the power cache of the reference (`src/pathsig/ops.py:87-98`, layout of
    `sig_kernels.cu:184,215-216`), with or without a gradient: a caller may read it or hand it to
    `logsig_backward`."""
    return torch.ops.pathsig.sig_to_logsig.default(
        signature, depth, d, alternative_projection, encoded_words, level_sizes)


def _logsig_of(signature: Tensor, depth: int, d: int, alternative_projection: bool, encoded_words: Tensor,
               level_sizes: list[int]) -> Tensor:
    """Log-signature alone, for the `LogSignature` module, which never shows the cache to its caller: when a
    gradient will be asked for, the forward keeps the cache its own adjoint reads (powers of the log-signature)
    in place of the reference's power cache, so the backward need not rebuild it."""
    if torch.is_grad_enabled() and signature.requires_grad and not os.environ.get("PATHSIG_NO_KEEP"):
        return torch.ops.pathsig.sig_to_logsig_keep.default(
            signature, depth, d, alternative_projection, encoded_words, level_sizes)[0]
    return torch.ops.pathsig.sig_to_logsig.default(
        signature, depth, d, alternative_projection, encoded_words, level_sizes)[0]


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


@torch.library.register_fake("pathsig::sig_to_logsig_keep", lib=_library)
def _sig_to_logsig_keep_fake(signature, depth, d, alternative_projection, encoded_words, level_sizes):
    return _sig_to_logsig_fake(signature, depth, d, alternative_projection, encoded_words, level_sizes)


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


@torch.library.register_fake("pathsig::logsig_backward_kept", lib=_library)
def _logsig_backward_kept_fake(logsig, cache, grad_logsig, depth, alternative_projection, encoded_words, level_sizes):
    return _logsig_backward_fake(logsig, cache, grad_logsig, depth, alternative_projection, encoded_words, level_sizes)
