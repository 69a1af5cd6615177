"""The C ABI called directly on a GPU: ctypes, raw device pointers, a raw stream handle, caller-provided workspaces
(no torch operator in between), against the CPU checkers.  Covers the four entry points that replace the
reference's launchers and the two keeping pairs."""
from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import tensor_oracle as TO
from tests.helpers import brownian_path, randn, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float64: 1e-12, torch.float32: 1e-5}


def _p(t):
    return ctypes.c_void_p(0 if t is None or t.numel() == 0 else t.data_ptr())


def _bytes(n):
    return torch.empty(max(int(n), 1), dtype=torch.uint8, device=DEV)


@pytest.fixture(scope="module")
def lib():
    from pathsig_amd import _load
    return _load.lib()


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("case", ["dense_chunked", "windows", "words"])
def test_signature_entry_points(lib, dtype, case):
    code = 0 if dtype == torch.float32 else 1
    sizes = codes = windows = None
    if case == "dense_chunked":
        B, L, d, depth = 3, 200, 4, 6          # a register-tiled shape, cut into time chunks
    elif case == "windows":
        B, L, d, depth = 4, 30, 3, 4
        windows = [(0, 30), (4, 9), (4, 9), (29, 30), (10, 25)]
    else:
        B, L, d, depth = 3, 12, 5, 3
        sizes, codes = [0, 5, 3, 4], [7, 24, 0, 31, 124, 31, 5]   # levels 2 and 3 listed, one word repeated
    path = brownian_path(B, L, d, seed=21) * 1.5
    want = TO.compute_signature(path, depth, sizes, codes, windows)
    G = randn(tuple(want.shape), seed=22)
    want_grad = TO.signature_vjp(path, G, depth, sizes, codes, windows)

    x = path.to(dtype).to(DEV)
    g = G.to(dtype).to(DEV)
    win = None if windows is None else torch.tensor(windows, dtype=torch.int32, device=DEV)
    W = 0 if win is None else win.shape[0]
    host_sizes = None if sizes is None else (ctypes.c_int64 * len(sizes))(*sizes)
    words = None if codes is None else torch.tensor(codes, dtype=torch.int64, device=DEV)
    n_words = 0 if words is None else words.numel()
    stream = torch.cuda.Stream()
    handle = ctypes.c_void_p(stream.cuda_stream)
    stream.wait_stream(torch.cuda.current_stream())

    sig = torch.full(tuple(want.shape), float("nan"), dtype=dtype, device=DEV)
    fws_bytes = lib.pathsig_sig_forward_workspace(code, B, L, d, depth, host_sizes, W)
    fws = _bytes(fws_bytes)
    rc = lib.pathsig_sig_forward(_p(x), _p(sig), code, B, L, d, depth, host_sizes, _p(words), n_words, _p(win), W,
                                 _p(fws), fws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()
    grad = torch.full_like(x, float("nan"))
    bws_bytes = lib.pathsig_sig_backward_workspace(code, B, L, d, depth, host_sizes, W)
    bws = _bytes(bws_bytes)
    rc = lib.pathsig_sig_backward(_p(x), _p(sig), _p(g), _p(grad), code, B, L, d, depth, host_sizes, _p(words), n_words,
                                  _p(win), W, _p(bws), bws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()

    # the keeping pair on the same inputs
    keep_bytes = lib.pathsig_sig_chunks_bytes(code, B, L, d, depth, host_sizes, W)
    keep = _bytes(keep_bytes)
    sig_k = torch.full_like(sig, float("nan"))
    grad_k = torch.full_like(x, float("nan"))
    rc = lib.pathsig_sig_forward_keep(_p(x), _p(sig_k), code, B, L, d, depth, host_sizes, _p(words), n_words, _p(win), W,
                                      _p(keep) if keep_bytes else None, keep_bytes, _p(fws), fws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()
    rc = lib.pathsig_sig_backward_kept(_p(x), _p(sig_k), _p(g), _p(grad_k), code, B, L, d, depth, host_sizes, _p(words),
                                       n_words, _p(win), W, _p(keep) if keep_bytes else None, keep_bytes, _p(bws),
                                       bws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()
    stream.synchronize()
    if case == "dense_chunked":
        assert keep_bytes > 0
        # a buffer of another size than this call keeps (one made under other tuning switches) is refused
        for wrong in (keep_bytes - 256, keep_bytes + 256):
            rc = lib.pathsig_sig_backward_kept(_p(x), _p(sig_k), _p(g), _p(grad_k), code, B, L, d, depth, host_sizes,
                                               _p(words), n_words, _p(win), W, _p(keep), wrong, _p(bws), bws_bytes, handle)
            assert rc != 0 and b"chunk buffer" in lib.pathsig_last_error()
        stream.synchronize()
    assert rel_err(sig, want) < TOL[dtype] and rel_err(grad, want_grad) < TOL[dtype]
    assert torch.equal(sig_k, sig) and rel_err(grad_k, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_logsignature_entry_points(lib, dtype):
    code = 0 if dtype == torch.float32 else 1
    d, depth, rows = 3, 4, 5
    top = [5, 80, 17, 17, 2, 44]
    dense = TO.signature(brownian_path(rows, 11, d, seed=23) * 1.5, depth)
    hyb = dense[:, TO.hybrid_columns(d, depth, len(top), top)]
    want_log, want_P = TO.sig_to_logsig(hyb, depth, d, len(top), top)
    want_cache = TO.logsig_power_cache(want_log, depth, d, len(top), top)
    G = randn(tuple(hyb.shape), seed=24)
    want_grad = TO.logsig_vjp(hyb, G, depth, d, len(top), top)

    sig = hyb.to(dtype).to(DEV)
    g = G.to(dtype).to(DEV)
    words = torch.tensor(top, dtype=torch.int64, device=DEV)
    S = hyb.shape[1]
    handle = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    logsig = torch.full_like(sig, float("nan"))
    P = torch.full((rows, S * depth), float("nan"), dtype=dtype, device=DEV)
    rc = lib.pathsig_logsig_forward(_p(sig), _p(logsig), _p(P), code, rows, d, depth, len(top), _p(words), handle)
    assert rc == 0, lib.pathsig_last_error()
    ws_bytes = lib.pathsig_logsig_backward_workspace(code, rows, d, depth, len(top))
    ws = _bytes(ws_bytes)
    grad = torch.full_like(sig, float("nan"))
    rc = lib.pathsig_logsig_backward(_p(sig), _p(P), _p(g), _p(grad), code, rows, d, depth, len(top), _p(words), _p(ws),
                                     ws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()
    # the keeping pair
    logsig_k = torch.full_like(sig, float("nan"))
    cache = torch.full_like(P, float("nan"))
    rc = lib.pathsig_logsig_forward_keep(_p(sig), _p(logsig_k), _p(cache), code, rows, d, depth, len(top), _p(words),
                                         handle)
    assert rc == 0, lib.pathsig_last_error()
    kws_bytes = lib.pathsig_logsig_backward_kept_workspace(code, rows, d, depth, len(top))
    kws = _bytes(kws_bytes)
    grad_k = torch.full_like(sig, float("nan"))
    rc = lib.pathsig_logsig_backward_kept(_p(logsig_k), _p(cache), _p(g), _p(grad_k), code, rows, d, depth, len(top),
                                          _p(words), _p(kws), kws_bytes, handle)
    assert rc == 0, lib.pathsig_last_error()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert rel_err(logsig, want_log) < tol and rel_err(P, want_P) < tol and rel_err(grad, want_grad) < tol
    low = (hyb.shape[-1] - len(top)) * depth          # the cache rows of the top-level words are not written
    assert torch.isnan(cache[:, low:]).all()
    assert torch.equal(logsig_k, logsig) and rel_err(cache[:, :low], want_cache[:, :low]) < tol
    assert rel_err(grad_k, want_grad) < tol
