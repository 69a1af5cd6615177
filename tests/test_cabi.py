"""The C ABI without a GPU: the library loads, exports every function that include/pathsig_hip.h declares,
and rejects bad arguments with its error codes before anything is launched."""
from __future__ import annotations

import ctypes
import pathlib
import re

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "pathsig_hip.h"


@pytest.fixture(scope="module")
def lib():
    from pathsig_amd import _load
    return _load.lib()


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(pathsig_[a-z_]+)\s*\(", text)))


def test_header_functions_are_exported(lib):
    names = declared_functions()
    assert {"pathsig_sig_forward", "pathsig_sig_backward", "pathsig_logsig_forward", "pathsig_logsig_backward",
            "pathsig_sig_forward_workspace", "pathsig_sig_backward_workspace", "pathsig_logsig_backward_workspace",
            "pathsig_sig_chunks_bytes", "pathsig_sig_forward_keep", "pathsig_sig_backward_kept",
            "pathsig_logsig_forward_keep", "pathsig_logsig_backward_kept", "pathsig_logsig_backward_kept_workspace",
            "pathsig_last_error", "pathsig_abi_version"} <= set(names)
    for name in names:
        assert hasattr(lib, name), name
    assert lib.pathsig_abi_version() == 3


def _fwd(lib, dtype=0, B=2, L=5, d=3, depth=3, path=1, sig=1, sizes=None):
    arr = None if sizes is None else (ctypes.c_int64 * len(sizes))(*sizes)
    return lib.pathsig_sig_forward(ctypes.c_void_p(path), ctypes.c_void_p(sig), dtype, B, L, d, depth, arr, None, 0,
                                   None, 0, None, 0, None)


def test_argument_errors_have_codes_and_messages(lib):
    ERR_ARG, ERR_UNSUPPORTED, ERR_WORKSPACE = -1, -2, -3
    assert _fwd(lib, depth=0) == ERR_ARG and b"depth" in lib.pathsig_last_error()
    assert _fwd(lib, depth=13) == ERR_ARG
    assert _fwd(lib, dtype=7) == ERR_ARG and b"dtype" in lib.pathsig_last_error()
    assert _fwd(lib, L=1) == ERR_ARG and b"2 time steps" in lib.pathsig_last_error()
    assert _fwd(lib, d=0) == ERR_ARG
    assert _fwd(lib, path=0) == ERR_ARG and b"NULL" in lib.pathsig_last_error()
    assert _fwd(lib, d=5000) == ERR_UNSUPPORTED
    # a projection whose level sizes need codes, but no code array
    assert _fwd(lib, sizes=[0, 3, 2, 0]) == ERR_ARG and b"encoded_words" in lib.pathsig_last_error()
    assert _fwd(lib, sizes=[0, 3, -1, 0]) == ERR_ARG
    # backward without its workspace
    rc = lib.pathsig_sig_backward(ctypes.c_void_p(1), ctypes.c_void_p(1), ctypes.c_void_p(1), ctypes.c_void_p(1), 0,
                                  2, 5, 3, 3, None, None, 0, None, 0, None, 0, None)
    assert rc == ERR_WORKSPACE and b"workspace" in lib.pathsig_last_error()
    # backward with a NULL signature or upstream gradient (a kernel would dereference them)
    ws = ctypes.c_void_p(1)
    for sig_ptr, grad_ptr in ((0, 1), (1, 0)):
        rc = lib.pathsig_sig_backward(ctypes.c_void_p(1), ctypes.c_void_p(sig_ptr), ctypes.c_void_p(grad_ptr),
                                      ctypes.c_void_p(1), 0, 2, 5, 3, 3, None, None, 0, None, 0, ws, 1 << 20, None)
        assert rc == ERR_ARG and b"sig and grad_sig" in lib.pathsig_last_error()
    # log-signature entry points
    assert lib.pathsig_logsig_forward(None, None, None, 0, 4, 3, 3, 27, None, None) == ERR_ARG
    assert lib.pathsig_logsig_forward(ctypes.c_void_p(1), ctypes.c_void_p(1), ctypes.c_void_p(1), 0, 4, 3, 3, 5, None,
                                      None) == ERR_ARG  # listed top level without its codes
    assert lib.pathsig_logsig_forward(ctypes.c_void_p(1), ctypes.c_void_p(1), ctypes.c_void_p(1), 0, 4, 3, 0, 0, None,
                                      None) == ERR_ARG
    assert lib.pathsig_logsig_forward_keep(ctypes.c_void_p(1), ctypes.c_void_p(1), None, 0, 4, 3, 3, 27, None,
                                           None) == ERR_ARG and b"cache" in lib.pathsig_last_error()
    assert lib.pathsig_logsig_backward_kept(ctypes.c_void_p(1), ctypes.c_void_p(1), ctypes.c_void_p(1),
                                            ctypes.c_void_p(1), 0, 4, 3, 3, 27, None, None, 0, None) == ERR_WORKSPACE
    # the plain adjoint rebuilds the log-signature and its cache in the workspace: it asks for more than the kept one
    assert lib.pathsig_logsig_backward_workspace(0, 4, 3, 3, 27) >= \
        lib.pathsig_logsig_backward_kept_workspace(0, 4, 3, 3, 27) + 4 * 39 * 4 * 4
    # empty batches are a no-op
    assert _fwd(lib, B=0, path=0, sig=0) == 0
    assert lib.pathsig_logsig_forward(None, None, None, 0, 0, 3, 3, 27, None, None) == 0


def test_workspace_sizes(lib):
    # general kernels: the forward needs none, the backward one increment accumulator
    assert lib.pathsig_sig_forward_workspace(0, 4, 100, 120, 3, None, 0) == 0
    need = lib.pathsig_sig_backward_workspace(0, 4, 100, 120, 3, None, 0)
    assert need >= 4 * 99 * 120 * 4
    assert lib.pathsig_sig_backward_workspace(1, 4, 100, 120, 3, None, 0) >= 4 * 99 * 120 * 8
    # 65 letters at depth 3 run as 72 letters on copies: of the path and the signature in the forward, of the path
    # (twice), the signature and its gradient in the backward
    wide_sig, wide_path = 4 * (72 + 72 ** 2 + 72 ** 3) * 4, 4 * 100 * 72 * 4
    assert lib.pathsig_sig_forward_workspace(0, 4, 100, 65, 3, None, 0) >= wide_sig + wide_path
    assert lib.pathsig_sig_backward_workspace(0, 4, 100, 65, 3, None, 0) >= 2 * wide_sig + 2 * wide_path
    assert lib.pathsig_sig_forward_workspace(0, 4, 100, 72, 3, None, 0) == 0     # compiled as it is, one piece
    # a long path on a tiled shape is cut into chunks, which need scratch in the forward too
    assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 4, 6, None, 0) > 0
    assert lib.pathsig_sig_forward_workspace(0, 4096, 64, 4, 6, None, 0) == 0
    assert lib.pathsig_logsig_backward_workspace(0, 10, 3, 4, 81) >= 10 * (3 + 9 + 27) * 4 * 4
    # bad arguments give 0
    assert lib.pathsig_sig_forward_workspace(0, 4, 1, 5, 3, None, 0) == 0


def test_sparse_projections_take_the_dense_kernels_when_that_is_cheaper(lib):
    """A projection with a few words: the per-word kernels sweep the path one increment after the other, so on a
    long path the dense kernels + a gather win as long as the dense signature is small; the forward then needs a
    dense buffer as workspace.  (Host-side decision only; nothing is launched.)"""
    import ctypes
    def sizes(d, depth, top, low=3):
        return (ctypes.c_int64 * (depth + 1))(0, *([low] * (depth - 1)), top)
    dense = 4 * 128 * sum(4 ** k for k in range(1, 7))          # one fp32 dense row per path, d = 4, depth 6
    assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 4, 6, sizes(4, 6, 10), 0) >= dense
    assert lib.pathsig_sig_forward_workspace(0, 128, 20, 4, 6, sizes(4, 6, 10), 0) == 0      # short path: per word
    assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 6, 6, sizes(6, 6, 10), 0) == 0    # 56 k coefficients: per word
    assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 65, 3, sizes(65, 3, 10), 0) == 0  # no compiled shape
    try:
        assert lib.pathsig_set_option(b"embed_share", 0) == 0
        assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 4, 6, sizes(4, 6, 10), 0) == 0
        assert lib.pathsig_set_option(b"embed_share", 10 ** 9) == 0
        assert lib.pathsig_sig_forward_workspace(0, 128, 20, 4, 6, sizes(4, 6, 10), 0) >= dense
        assert lib.pathsig_set_option(b"tiled", 0) == 0                  # no tiled kernels at all: no dense buffer
        assert lib.pathsig_sig_forward_workspace(0, 128, 1024, 4, 6, sizes(4, 6, 10), 0) == 0
        assert lib.pathsig_set_option(b"tiled", 2) != 0
    finally:
        assert lib.pathsig_set_option(b"embed_share", -1) == 0
        assert lib.pathsig_set_option(b"tiled", 1) == 0
