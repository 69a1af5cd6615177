"""The five benchmark configurations at their full sizes.

The CPU checkers cannot sweep these sizes in seconds, so each configuration is checked (a) against the
per-word C checker on the first paths of the batch (paths are independent), and (b) through properties
that do not depend on the size: Chen's identity between the two halves of the path, windows equal to
slices, linearity of the backward in the upstream gradient, and the adjoint identity
<G, J h> = <J^T G, h> against a forward finite difference.

Both dtypes.  Besides the global metric max|d| / max(1, max|ref|) (1e-5 fp32, 1e-12 fp64), every level is held
to a relative bound of its own, max|d_k| / max|ref_k|: the inputs are Brownian with unit variance at the end of
the path, so the coefficients of level k fall off like 1/k! and the global metric alone would let a
percent-sized error through in the top levels.  Bounds: LEVEL_TOL below; gradients max|d| / max|ref|."""
from __future__ import annotations

import pytest
import torch

import bench
from oracle import tensor_oracle as TO
from oracle import words_oracle as WO
from tests.helpers import level_rel_errs, rel_err, strict_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}
# per-level and gradient bounds, relative to the largest entry of the level (of the gradient)
LEVEL_TOL = {torch.float32: 2e-5, torch.float64: 2e-12}
BOTH = pytest.mark.parametrize("dtype", [torch.float32, torch.float64])


def _dense_sizes(d, depth):
    return [d ** k for k in range(1, depth + 1)]


def _check(out, want, sizes, dtype, what=""):
    assert rel_err(out, want) < TOL[dtype], what
    errs = level_rel_errs(out, want, sizes)
    assert max(errs) < LEVEL_TOL[dtype], (what, errs)


def _ops_args(mod):
    return (mod.depth, mod.alternative_projection, mod._encoded_words, mod._level_sizes, mod.use_windows, mod._windows)


@BOTH
def test_c1_forward_full_size(dtype):
    wl = bench.make_workload("c1", dtype, 1)
    out = wl["mod"](wl["x"])
    want = WO.sig_forward(wl["path_cpu"], 4)
    assert out.shape == (32, 4680)
    _check(out, want, _dense_sizes(8, 4), dtype)


@BOTH
def test_c2_full_size_subset_and_properties(dtype):
    wl = bench.make_workload("c2", dtype, 2)
    mod, x, G, path = wl["mod"], wl["x"], wl["G"], wl["path_cpu"]
    xg = x.clone().requires_grad_(True)
    out = mod(xg)
    (grad,) = torch.autograd.grad(out, xg, G)
    assert out.shape == (128, 5460) and grad.shape == (128, 1024, 4)
    sub = 3
    want = WO.sig_forward(path[:sub], 6)
    _check(out[:sub], want, _dense_sizes(4, 6), dtype)
    want_grad = WO.sig_backward(path[:sub], want, G[:sub].double().cpu(), 6)
    assert rel_err(grad[:sub], want_grad) < TOL[dtype]
    assert strict_rel_err(grad[:sub], want_grad) < LEVEL_TOL[dtype]
    if dtype != torch.float32:
        return  # the properties below run in fp64 from the fp32 workload
    # Chen: signature of the whole path = product of the signatures of its halves (fp64 on the GPU)
    x64 = path.to(DEV)
    whole = mod(x64)
    left = TO.split_levels(mod(x64[:, :513]).cpu(), 4, 6)
    right = TO.split_levels(mod(x64[:, 512:]).cpu(), 4, 6)
    prod = torch.cat(TO.tensor_product_levels(left, right, 6), dim=-1)
    assert rel_err(whole, prod) < 1e-12
    # the backward is linear in the upstream gradient
    G64 = G.double()
    H64 = torch.randn_like(G64)
    gb = lambda g: torch.ops.pathsig.signature_backward(x64, whole, g, *_ops_args(mod))
    assert rel_err(gb(2.0 * G64 - 0.5 * H64), 2.0 * gb(G64) - 0.5 * gb(H64)) < 1e-12
    # adjoint identity against a directional finite difference of the forward
    h = torch.randn_like(x64)
    eps = 1e-6
    fd = (mod(x64 + eps * h) - mod(x64 - eps * h)) / (2 * eps)
    lhs = (fd * G64).sum()
    rhs = (gb(G64) * h).sum()
    assert abs(float(lhs - rhs)) < 1e-6 * max(1.0, abs(float(lhs)))


@BOTH
def test_c3_windows_full_size(dtype):
    wl = bench.make_workload("c3", dtype, 3)
    mod, x, G, path = wl["mod"], wl["x"], wl["G"], wl["path_cpu"]
    xg = x.clone().requires_grad_(True)
    out = mod(xg)
    (grad,) = torch.autograd.grad(out, xg, G)
    assert out.shape == (64, 63, 9330)
    wins = wl["windows"].tolist()
    # windows are slices: a few windows of a few paths against the checker
    for w in (0, 17, 62):
        s, e = wins[w]
        want = WO.sig_forward(path[:2, s:e], 5)
        _check(out[:2, w], want, _dense_sizes(6, 5), dtype, f"window {w}")
    sub = 1
    sig_sub = WO.sig_forward(path[:sub], 5, windows=wins)
    _check(out[:sub], sig_sub, _dense_sizes(6, 5), dtype)
    want_grad = WO.sig_backward(path[:sub], sig_sub, G[:sub].double().cpu(), 5, windows=wins)
    assert rel_err(grad[:sub], want_grad) < TOL[dtype]
    assert strict_rel_err(grad[:sub], want_grad) < LEVEL_TOL[dtype]
    if dtype != torch.float32:
        return
    # overlapping windows: gradients add (sum of per-window backward calls == one windowed call), fp64
    x64 = path[:4].to(DEV)
    G64 = G[:4].double()
    full = torch.ops.pathsig.signature_backward(x64, mod(x64), G64, *_ops_args(mod))
    import pathsig_amd as ps
    acc = torch.zeros_like(x64)
    for w in (0, 1, 2):
        one = ps.Signature(depth=5, windows=wl["windows"][w:w + 1].to(DEV))
        acc += torch.ops.pathsig.signature_backward(x64, one(x64), G64[:, w:w + 1].contiguous(), *_ops_args(one))
    three = ps.Signature(depth=5, windows=wl["windows"][:3].to(DEV))
    got = torch.ops.pathsig.signature_backward(x64, three(x64), G64[:, :3].contiguous(), *_ops_args(three))
    assert rel_err(got, acc) < 1e-12
    assert torch.isfinite(full).all()


@BOTH
def test_c4_word_projection_full_size(dtype):
    wl = bench.make_workload("c4", dtype, 4)
    mod, x, G, path, proj = wl["mod"], wl["x"], wl["G"], wl["path_cpu"], wl["proj"]
    assert proj.level_sizes == [0, 16, 256, 484, 513, 548, 503] and wl["nodes"] == 10835
    xg = x.clone().requires_grad_(True)
    out = mod(xg)
    (grad,) = torch.autograd.grad(out, xg, G)
    assert out.shape == (256, 2320)
    sub = 2
    want = WO.sig_forward(path[:sub], 6, proj.level_sizes, proj._codes)
    _check(out[:sub], want, proj.level_sizes[1:], dtype)
    want_grad = WO.sig_backward(path[:sub], want, G[:sub].double().cpu(), 6, proj.level_sizes, proj._codes)
    assert rel_err(grad[:sub], want_grad) < TOL[dtype]
    assert strict_rel_err(grad[:sub], want_grad) < LEVEL_TOL[dtype]
    # levels 1 and 2 are full: they equal the depth-2 dense signature
    import pathsig_amd as ps
    assert rel_err(out[:, :272], ps.Signature(depth=2)(x)) < TOL[dtype]


@BOTH
def test_c5_logsignature_lyndon_full_size(dtype):
    tol = TOL[dtype]
    wl = bench.make_workload("c5", dtype, 5)
    mod, x, G, path, proj = wl["mod"], wl["x"], wl["G"], wl["path_cpu"], wl["proj"]
    xg = x.clone().requires_grad_(True)
    out = mod(xg)
    (grad,) = torch.autograd.grad(out, xg, G)
    assert out.shape == (128, 7764)
    # first path through the per-word checker: hybrid signature -> log -> projection's coordinates
    d, depth, sub = 8, 5, 1
    top_codes, top = mod._top_words.cpu().tolist(), mod._ext_level_sizes[depth]
    sig = WO.sig_forward(path[:sub], depth, mod._ext_level_sizes, top_codes)
    logsig, P = WO.logsig_forward(sig, depth, d, top, top_codes)
    idx = mod._indices_from_sig.cpu()
    assert rel_err(out[:sub], logsig[:, idx]) < tol
    errs = level_rel_errs(out[:sub], logsig[:, idx], proj.level_sizes[1:])
    assert max(errs) < LEVEL_TOL[dtype], errs
    g_hyb = torch.zeros_like(sig).index_add_(1, idx, G[:sub].double().cpu())
    g_sig = WO.logsig_backward(sig, P, g_hyb, depth, d, top, top_codes)
    want_grad = WO.sig_backward(path[:sub], sig, g_sig, depth, mod._ext_level_sizes, top_codes)
    assert rel_err(grad[:sub], want_grad) < tol
    assert strict_rel_err(grad[:sub], want_grad) < LEVEL_TOL[dtype]
    # level 1 of a log-signature is the total increment
    assert rel_err(out[:, :8], (path[:, -1] - path[:, 0])) < tol
