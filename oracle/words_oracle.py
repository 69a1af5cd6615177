"""ctypes front-end of oracle/liboracle_words.so (the per-word C restatement in oracle/ref_words.c).

Test infrastructure only.  Tensors are CPU torch tensors (fp64 or fp32); arguments mirror the four
reference ops (`src/pathsig/bindings.cpp:9-63`).
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import build as _build

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _build.LIB.is_file():
            _build.build()
        _lib = ctypes.CDLL(str(_build.LIB))
    return _lib


def _suf(t: torch.Tensor) -> str:
    if t.dtype == torch.float64:
        return "_f64"
    if t.dtype == torch.float32:
        return "_f32"
    raise TypeError("fp32 / fp64 only")


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i64(vals: Optional[Sequence[int]]):
    if vals is None:
        return None
    return torch.tensor(list(vals), dtype=torch.int64)


def _win(windows):
    if windows is None:
        return None, 0
    w = torch.as_tensor(windows).to(torch.int32).contiguous()
    return w, int(w.shape[0])


def sig_forward(path, depth, level_sizes=None, codes=None, windows=None) -> torch.Tensor:
    path = path.contiguous()
    B, L, d = path.shape
    ls, cd = _i64(level_sizes), _i64(codes if level_sizes is not None else None)
    S = sum(level_sizes[1:depth + 1]) if level_sizes is not None else sum(d ** k for k in range(1, depth + 1))
    w, W = _win(windows)
    out = torch.empty((B, W, S) if w is not None else (B, S), dtype=path.dtype)
    rc = getattr(lib(), "ow_sig_forward" + _suf(path))(
        _p(path), _p(out), ctypes.c_int64(B), ctypes.c_int64(L), ctypes.c_int64(d), ctypes.c_int(depth),
        _p(ls), _p(cd), _p(w), ctypes.c_int64(W))
    assert rc == 0
    return out


def sig_backward(path, sig, grad_sig, depth, level_sizes=None, codes=None, windows=None) -> torch.Tensor:
    path, sig, grad_sig = path.contiguous(), sig.contiguous(), grad_sig.contiguous()
    B, L, d = path.shape
    ls, cd = _i64(level_sizes), _i64(codes if level_sizes is not None else None)
    w, W = _win(windows)
    out = torch.empty_like(path)
    rc = getattr(lib(), "ow_sig_backward" + _suf(path))(
        _p(path), _p(sig), _p(grad_sig), _p(out), ctypes.c_int64(B), ctypes.c_int64(L), ctypes.c_int64(d),
        ctypes.c_int(depth), _p(ls), _p(cd), _p(w), ctypes.c_int64(W))
    assert rc == 0
    return out


def logsig_forward(sig, depth, d, top_size=None, top_codes=None):
    sig = sig.contiguous()
    S = sig.shape[-1]
    rows = sig.numel() // S
    top = d ** depth if top_size is None else int(top_size)
    tc = _i64(top_codes) if (top_codes is not None and top != d ** depth) else None
    logsig = torch.empty_like(sig)
    P = torch.empty(*sig.shape[:-1], S * depth, dtype=sig.dtype)
    rc = getattr(lib(), "ow_logsig_forward" + _suf(sig))(
        _p(sig), _p(P), _p(logsig), ctypes.c_int64(rows), ctypes.c_int64(d), ctypes.c_int(depth),
        ctypes.c_int64(top), _p(tc))
    assert rc == 0
    return logsig, P


def logsig_backward(sig, P, grad_logsig, depth, d, top_size=None, top_codes=None) -> torch.Tensor:
    sig, P, grad_logsig = sig.contiguous(), P.contiguous(), grad_logsig.contiguous()
    S = sig.shape[-1]
    rows = sig.numel() // S
    top = d ** depth if top_size is None else int(top_size)
    tc = _i64(top_codes) if (top_codes is not None and top != d ** depth) else None
    gsig = torch.empty_like(sig)
    rc = getattr(lib(), "ow_logsig_backward" + _suf(sig))(
        _p(sig), _p(P), _p(grad_logsig), _p(gsig), ctypes.c_int64(rows), ctypes.c_int64(d), ctypes.c_int(depth),
        ctypes.c_int64(top), _p(tc))
    assert rc == 0
    return gsig
