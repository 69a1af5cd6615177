"""Loads libpathsig_hip.so (the hand-written HIP kernels behind a C ABI) and declares its entry points.

Counterpart of the reference loader `src/pathsig/_load.py:12-45`, with two differences: the library is
a plain C-ABI object opened with ctypes instead of a torch extension, and the PyTorch build must be a
ROCm one (`torch.version.hip`), where the reference insists on `torch.version.cuda`.
There is no fallback: if the library is missing, importing the package fails.
"""
from __future__ import annotations

import ctypes
import pathlib
import threading

import torch

_LIB_NAME = "libpathsig_hip.so"
_ABI_VERSION = 3
_lock = threading.Lock()
_lib: ctypes.CDLL | None = None

_I64 = ctypes.c_int64
_INT = ctypes.c_int
_PTR = ctypes.c_void_p
_SIZE = ctypes.c_size_t


def _declare(lib: ctypes.CDLL) -> None:
    lib.pathsig_abi_version.restype = _INT
    lib.pathsig_abi_version.argtypes = []
    lib.pathsig_last_error.restype = ctypes.c_char_p
    lib.pathsig_last_error.argtypes = []

    lib.pathsig_set_option.restype = _INT
    lib.pathsig_set_option.argtypes = [ctypes.c_char_p, _I64]
    lib.pathsig_profile_enable.restype = _INT
    lib.pathsig_profile_enable.argtypes = [_INT]
    lib.pathsig_profile_sweep_ms.restype = ctypes.c_float
    lib.pathsig_profile_sweep_ms.argtypes = []

    lib.pathsig_sig_forward_workspace.restype = _SIZE
    lib.pathsig_sig_forward_workspace.argtypes = [_INT, _I64, _I64, _I64, _INT, _PTR, _I64]
    lib.pathsig_sig_forward.restype = _INT
    lib.pathsig_sig_forward.argtypes = [_PTR, _PTR, _INT, _I64, _I64, _I64, _INT, _PTR, _PTR, _I64, _PTR, _I64,
                                        _PTR, _SIZE, _PTR]
    lib.pathsig_sig_backward_workspace.restype = _SIZE
    lib.pathsig_sig_backward_workspace.argtypes = [_INT, _I64, _I64, _I64, _INT, _PTR, _I64]
    lib.pathsig_sig_backward.restype = _INT
    lib.pathsig_sig_backward.argtypes = [_PTR, _PTR, _PTR, _PTR, _INT, _I64, _I64, _I64, _INT, _PTR, _PTR, _I64,
                                         _PTR, _I64, _PTR, _SIZE, _PTR]
    lib.pathsig_sig_backward_noalloc.restype = _INT
    lib.pathsig_sig_backward_noalloc.argtypes = [_PTR, _PTR, _PTR, _PTR, _INT, _I64, _I64, _I64, _INT, _PTR, _PTR, _I64,
                                                 _PTR, _I64, _PTR]
    lib.pathsig_sig_chunks_bytes.restype = _SIZE
    lib.pathsig_sig_chunks_bytes.argtypes = [_INT, _I64, _I64, _I64, _INT, _PTR, _I64]
    lib.pathsig_sig_forward_keep.restype = _INT
    lib.pathsig_sig_forward_keep.argtypes = [_PTR, _PTR, _INT, _I64, _I64, _I64, _INT, _PTR, _PTR, _I64, _PTR, _I64,
                                             _PTR, _SIZE, _PTR, _SIZE, _PTR]
    lib.pathsig_sig_backward_kept.restype = _INT
    lib.pathsig_sig_backward_kept.argtypes = [_PTR, _PTR, _PTR, _PTR, _INT, _I64, _I64, _I64, _INT, _PTR, _PTR, _I64,
                                              _PTR, _I64, _PTR, _SIZE, _PTR, _SIZE, _PTR]
    lib.pathsig_logsig_forward.restype = _INT
    lib.pathsig_logsig_forward.argtypes = [_PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _I64, _PTR, _PTR]
    lib.pathsig_logsig_backward_workspace.restype = _SIZE
    lib.pathsig_logsig_backward_workspace.argtypes = [_INT, _I64, _I64, _INT, _I64]
    lib.pathsig_logsig_backward.restype = _INT
    lib.pathsig_logsig_backward.argtypes = [_PTR, _PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _I64, _PTR, _PTR, _SIZE,
                                            _PTR]
    lib.pathsig_logsig_forward_keep.restype = _INT
    lib.pathsig_logsig_forward_keep.argtypes = [_PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _I64, _PTR, _PTR]
    lib.pathsig_logsig_backward_kept_workspace.restype = _SIZE
    lib.pathsig_logsig_backward_kept_workspace.argtypes = [_INT, _I64, _I64, _INT, _I64]
    lib.pathsig_logsig_backward_kept.restype = _INT
    lib.pathsig_logsig_backward_kept.argtypes = [_PTR, _PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _I64, _PTR, _PTR,
                                                 _SIZE, _PTR]


def library_path() -> pathlib.Path:
    return pathlib.Path(__file__).resolve().parent / _LIB_NAME


def ensure_loaded() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if torch.version.hip is None:
        raise RuntimeError("pathsig_amd needs a ROCm build of PyTorch (torch.version.hip is None).")
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not path.is_file():
            raise RuntimeError(
                f"Could not find the native kernel library {path}. Build it with "
                "`python pathsig_amd/build_ext.py` (needs hipcc); there is no fallback implementation.")
        lib = ctypes.CDLL(str(path))
        _declare(lib)
        got = lib.pathsig_abi_version()
        if got != _ABI_VERSION:
            raise RuntimeError(f"{path} has ABI version {got}, this package needs {_ABI_VERSION}; rebuild it.")
        _lib = lib
        return lib


def lib() -> ctypes.CDLL:
    return ensure_loaded()


_TORCH_LIB_NAME = "libpathsig_torch.so"
_torch_ops_loaded = False


def load_torch_ops() -> None:
    """Loads the C++ registration of the operators (schemas, device implementations, autograd nodes).

    There is no second registration: a missing or stale library is an error."""
    global _torch_ops_loaded
    if _torch_ops_loaded:
        return
    ensure_loaded()
    path = pathlib.Path(__file__).resolve().parent / _TORCH_LIB_NAME
    if not path.is_file():
        raise RuntimeError(
            f"Could not find the operator library {path}. Build it with `python pathsig_amd/build_ext.py` "
            "(needs g++ and the torch headers).")
    try:
        torch.ops.load_library(str(path))
    except OSError as exc:  # built against another torch or an older libpathsig_hip.so
        raise RuntimeError(f"{path} could not be loaded ({exc}); rebuild it with "
                           "`python pathsig_amd/build_ext.py`.") from exc
    _torch_ops_loaded = True


def set_option(name: str, value: int) -> None:
    """Process-wide tuning switch of the kernel library (see `pathsig_set_option` in include/pathsig_hip.h)."""
    rc = lib().pathsig_set_option(name.encode(), int(value))
    if rc != 0:
        raise ValueError(lib().pathsig_last_error().decode("utf-8", "replace"))
