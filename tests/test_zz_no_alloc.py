"""The signature backward that allocates nothing (`pathsig_sig_backward_noalloc`), called through the C ABI with
raw device pointers, against `pathsig_sig_backward` with a caller-provided workspace: same inputs, two calls in a
row (the second one smaller, so stale contents of the shared static scratch would show), fp32 1e-5 / fp64 1e-12
with the metric of the other parity tests, plus the size limit, plus the two properties the entry point exists for:
free device memory does not move across a call, and a call can be captured into a HIP graph and replayed."""
from __future__ import annotations

import ctypes

import pytest
import torch

from tests.helpers import brownian_path, randn, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float64: 1e-12, torch.float32: 1e-5}
STATIC_BYTES = 64 * 1024 * 1024


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _both(lib, dtype, B, L, d, depth, windows=None, sizes=None, codes=None):
    code = 0 if dtype == torch.float32 else 1
    path = brownian_path(B, L, d, seed=5 + B).to(dtype).to(DEV)
    win = None if windows is None else torch.tensor(windows, dtype=torch.int32, device=DEV)
    W = 0 if win is None else win.shape[0]
    S = sum(sizes[1:]) if sizes else sum(d ** k for k in range(1, depth + 1))
    host_sizes = None if sizes is None else (ctypes.c_int64 * len(sizes))(*sizes)
    words = None if codes is None else torch.tensor(codes, dtype=torch.int64, device=DEV)
    n_words = 0 if words is None else words.numel()
    sig = torch.empty((B, W, S) if W else (B, S), dtype=dtype, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    fws_bytes = lib.pathsig_sig_forward_workspace(code, B, L, d, depth, host_sizes, W)
    fws = torch.empty(max(fws_bytes, 1), dtype=torch.uint8, device=DEV)
    rc = lib.pathsig_sig_forward(_p(path), _p(sig), code, B, L, d, depth, host_sizes, _p(words), n_words, _p(win), W,
                                 _p(fws), fws_bytes, stream)
    assert rc == 0, lib.pathsig_last_error()
    grad_sig = randn(tuple(sig.shape), seed=9).to(dtype).to(DEV)
    ws_bytes = lib.pathsig_sig_backward_workspace(code, B, L, d, depth, host_sizes, W)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    want = torch.full_like(path, float("nan"))
    rc = lib.pathsig_sig_backward(_p(path), _p(sig), _p(grad_sig), _p(want), code, B, L, d, depth, host_sizes,
                                  _p(words), n_words, _p(win), W, _p(ws), ws_bytes, stream)
    assert rc == 0, lib.pathsig_last_error()
    got = torch.full_like(path, float("nan"))
    rc = lib.pathsig_sig_backward_noalloc(_p(path), _p(sig), _p(grad_sig), _p(got), code, B, L, d, depth, host_sizes,
                                          _p(words), n_words, _p(win), W, stream)
    torch.cuda.synchronize()
    return rc, ws_bytes, got, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_noalloc_backward_matches_the_workspace_one(dtype):
    from pathsig_amd import _load
    lib = _load.lib()
    # two calls in a row on the same GPU: the time-chunked register-tiled path (scratch: chunk signatures, edge
    # products, path-gradient cells), then a smaller one through the per-word kernels with overlapping windows
    # (scratch: the increment-gradient accumulator, which must start from zero)
    cases = [dict(B=6, L=300, d=4, depth=6),
             dict(B=3, L=40, d=5, depth=3, windows=[(0, 40), (5, 30), (5, 30), (38, 40)]),
             dict(B=2, L=9, d=3, depth=3, sizes=[0, 3, 2, 3], codes=[1, 7, 26, 0, 13])]
    for case in cases:
        rc, ws_bytes, got, want = _both(lib, dtype, **case)
        assert rc == 0, lib.pathsig_last_error()
        assert 0 < ws_bytes <= STATIC_BYTES
        assert torch.isfinite(got).all() and rel_err(got, want) < TOL[dtype], case


def _call_pair(lib, path, sig, grad_sig, B, L, d, depth):
    """(noalloc closure, workspace closure) on fixed device tensors; each returns the library's status code."""
    got, want = torch.full_like(path, float("nan")), torch.full_like(path, float("nan"))
    ws_bytes = lib.pathsig_sig_backward_workspace(0, B, L, d, depth, None, 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)

    def noalloc():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return lib.pathsig_sig_backward_noalloc(_p(path), _p(sig), _p(grad_sig), _p(got), 0, B, L, d, depth, None, None,
                                                0, None, 0, stream)

    def with_workspace():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return lib.pathsig_sig_backward(_p(path), _p(sig), _p(grad_sig), _p(want), 0, B, L, d, depth, None, None, 0,
                                        None, 0, _p(ws), ws_bytes, stream)

    return noalloc, with_workspace, got, want


def test_noalloc_backward_leaves_free_memory_alone_and_can_be_captured():
    import pathsig_amd as ps
    from pathsig_amd import _load
    lib = _load.lib()
    B, L, d, depth = 6, 300, 4, 6
    path = brownian_path(B, L, d, seed=11).float().to(DEV)
    sig = ps.Signature(depth=depth)(path)
    grad_sig = randn(tuple(sig.shape), seed=12).float().to(DEV)
    noalloc, with_workspace, got, want = _call_pair(lib, path, sig, grad_sig, B, L, d, depth)
    assert noalloc() == 0, lib.pathsig_last_error()     # warm-up: the scratch address is looked up once per device
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        assert noalloc() == 0, lib.pathsig_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    # captured once, replayed on new inputs, with eager work and synchronisations between the replays
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = noalloc()
    assert rc == 0, lib.pathsig_last_error()
    for replay in range(3):
        path.copy_(brownian_path(B, L, d, seed=20 + replay).float())
        sig.copy_(ps.Signature(depth=depth)(path))
        grad_sig.copy_(randn(tuple(sig.shape), seed=30 + replay).float())
        got.fill_(float("nan"))
        graph.replay()
        assert with_workspace() == 0, lib.pathsig_last_error()
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and rel_err(got, want) < 1e-6, replay


def test_noalloc_backward_rejects_what_does_not_fit():
    from pathsig_amd import _load
    lib = _load.lib()
    # 2048 paths of 4096 points need twice the static scratch for their increment gradients alone: the call must
    # fail before any launch
    B, L, d, depth = 2048, 4096, 4, 6
    assert lib.pathsig_sig_backward_workspace(0, B, L, d, depth, None, 0) > STATIC_BYTES
    dummy = torch.zeros(16, device=DEV)
    rc = lib.pathsig_sig_backward_noalloc(_p(dummy), _p(dummy), _p(dummy), _p(dummy), 0, B, L, d, depth, None, None, 0,
                                          None, 0, None)
    assert rc == -3 and b"static buffer" in lib.pathsig_last_error()
