"""Parity of the HIP kernels (through the torch ops, i.e. through the C ABI) with the CPU checkers.

Tolerances (max|got-want| / max(1, max|want|), the metric of the reference's `tests/test_sig.py:88-91`):
fp64 1e-12, fp32 1e-5, as the build target states.  Index and layout checks are exact.
"""
from __future__ import annotations

import random

import pytest
import torch

from oracle import tensor_oracle as TO
from tests.helpers import brownian_path, randn, random_word_set, rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float64: 1e-12, torch.float32: 1e-5}
DEV = "cuda"


@pytest.fixture(scope="module")
def ps():
    import pathsig_amd
    return pathsig_amd


def _empty_i64():
    return torch.empty(0, dtype=torch.int64, device=DEV)


def _run_sig(ps, path_cpu, depth, dtype, projection=None, windows=None, G=None):
    """Forward (+ backward when G is given) on the GPU; returns CPU tensors."""
    x = path_cpu.to(dtype).to(DEV).requires_grad_(G is not None)
    win = None if windows is None else torch.tensor(windows, dtype=torch.int64, device=DEV)
    mod = ps.Signature(depth=depth, projection=projection, windows=win)
    out = mod(x)
    grad = None
    if G is not None:
        (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
        grad = grad.cpu()
    return out.detach().cpu(), grad


def _plan(projection):
    if projection is None:
        return None, None
    return projection.level_sizes, projection._codes


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,L,B", [
    (2, 1, 5, 3), (2, 2, 9, 2), (3, 3, 17, 4), (2, 6, 33, 3), (4, 4, 20, 5), (5, 3, 12, 2), (3, 5, 40, 2),
    (7, 2, 6, 3), (2, 8, 11, 2), (2, 12, 6, 1), (33, 2, 7, 2), (4, 6, 24, 2), (6, 4, 2, 3),
])
def test_dense_forward_backward(ps, dtype, d, depth, L, B):
    # large increments on purpose; at depth 12 they are kept a little smaller: with increments of size 1.5 the
    # gradient of a level-12 coefficient sums thousands of terms of mixed sign up to 700 in size, and fp32
    # rounding alone reaches 1e-5 of that
    path = brownian_path(B, L, d, seed=100 + d * 13 + depth) * (3.0 if depth < 10 else 2.0)
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=7)
    got, grad = _run_sig(ps, path, depth, dtype, G=G)
    assert got.shape == want.shape
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_windows(ps, dtype):
    d, depth, L, B = 3, 4, 30, 3
    path = brownian_path(B, L, d, seed=21) * 2.0
    wins = [(0, 30), (3, 5), (2, 19), (15, 30), (4, 6), (10, 12), (0, 2), (28, 30), (5, 25), (5, 25)]
    want = TO.compute_signature(path, depth, windows=wins)
    G = randn(tuple(want.shape), seed=22)
    got, grad = _run_sig(ps, path, depth, dtype, windows=wins, G=G)
    assert got.shape == (B, len(wins), TO.dense_size(d, depth))
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth, windows=wins)
    assert rel_err(grad, want_grad) < TOL[dtype]


def test_degenerate_windows_give_zero(ps):
    d, depth = 2, 3
    path = brownian_path(2, 10, d, seed=23)
    wins = [(4, 5), (6, 6), (0, 10)]
    got, grad = _run_sig(ps, path, depth, torch.float64, windows=wins,
                         G=torch.ones(2, 3, TO.dense_size(d, depth), dtype=torch.float64))
    assert got[:, 0].abs().max() == 0 and got[:, 1].abs().max() == 0
    assert rel_err(got[:, 2], TO.signature(path, depth)) < 1e-12
    assert torch.isfinite(grad).all()


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("route", ["share", "dense"])
@pytest.mark.parametrize("kind", ["words", "lyndon", "gap", "all_words", "full_levels"])
def test_projections(ps, set_option, dtype, kind, route):
    """route "share": a projection runs on the register-tiled kernels only when its top level keeps 1/8 of the
    dense one (the others exercise the per-word kernels); "dense": whenever a compiled shape exists."""
    set_option("embed_share", 8 if route == "share" else 10 ** 9)
    d, depth, L, B = 3, 4, 15, 3
    if kind == "words":
        proj = ps.projections.words(random_word_set(d, 1, 4, 40, seed=5), depth=depth, path_dim=d)
    elif kind == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
    elif kind == "gap":
        proj = ps.projections.words([(1,), (0, 1, 2), (2, 2, 1), (1, 0, 0, 2), (1, 0, 0, 2)], depth=depth, path_dim=d)
    elif kind == "all_words":
        import itertools
        words = [w for n in range(1, depth + 1) for w in itertools.product(range(d), repeat=n)]
        proj = ps.projections.words(words, depth=depth, path_dim=d)
        assert proj._codes == []
    else:
        proj = ps.projections.words(random_word_set(d, 3, 4, 20, seed=6), depth=depth, path_dim=d, full_levels=(1, 2))
    sizes, codes = _plan(proj)
    path = brownian_path(B, L, d, seed=31) * 2.0
    want = TO.compute_signature(path, depth, sizes, codes)
    G = randn(tuple(want.shape), seed=32)
    got, grad = _run_sig(ps, path, depth, dtype, projection=proj, G=G)
    assert got.shape == (B, proj.sig_size)
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth, sizes, codes)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("route", ["share", "dense"])
@pytest.mark.parametrize("B", [3, 20])
def test_anisotropic_projection(ps, set_option, dtype, B, route):
    """Weighted-degree truncation (`projections.py:132-223`): signature and log-signature through the projection,
    for a small batch (lanes on words) and a larger one (lanes on paths)."""
    set_option("embed_share", 8 if route == "share" else 10 ** 9)
    d, depth, L = 4, 5, 16
    proj = ps.projections.anisotropic([1.0, 1.5, 2.0, 3.0], weight_threshold=5.0, depth=depth, path_dim=d)
    assert 0 < proj.sig_size < TO.dense_size(d, depth)
    sizes, codes = _plan(proj)
    path = brownian_path(B, L, d, seed=81) * 1.5
    want = TO.compute_signature(path, depth, sizes, codes)
    G = randn(tuple(want.shape), seed=82)
    got, grad = _run_sig(ps, path, depth, dtype, projection=proj, G=G)
    assert got.shape == (B, proj.sig_size)
    assert rel_err(got, want) < TOL[dtype]
    assert rel_err(grad, TO.signature_vjp(path, G, depth, sizes, codes)) < TOL[dtype]
    # the log-signature in the projection's coordinates equals the gather of the dense log-signature
    cols = torch.tensor(TO.projection_columns(d, depth, sizes, codes))
    x = path.to(dtype).to(DEV)
    out = ps.LogSignature(depth=depth, projection=proj)(x)
    assert rel_err(out, TO.logsignature(path, depth).index_select(-1, cols)) < TOL[dtype]


@pytest.mark.parametrize("route", ["share", "dense"])
def test_projection_with_windows(ps, set_option, route):
    set_option("embed_share", 8 if route == "share" else 10 ** 9)
    d, depth, L, B = 4, 3, 20, 2
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    wins = [(0, 10), (5, 20), (7, 9)]
    path = brownian_path(B, L, d, seed=33)
    sizes, codes = _plan(proj)
    want = TO.compute_signature(path, depth, sizes, codes, wins)
    G = randn(tuple(want.shape), seed=34)
    got, grad = _run_sig(ps, path, depth, torch.float64, projection=proj, windows=wins, G=G)
    assert rel_err(got, want) < 1e-12
    assert rel_err(grad, TO.signature_vjp(path, G, depth, sizes, codes, wins)) < 1e-12


# Batches of a dozen paths or more take the backward kernels that put lanes on paths (groups of 16 or 32
# paths per word); the cases cover both group sizes, ragged last groups, dense and listed levels, prefixes
# read from the saved signature and prefixes rebuilt by a forward sweep, long words and wide alphabets.
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("case", [
    dict(d=3, depth=4, L=15, B=13, kind="words"),
    dict(d=3, depth=4, L=40, B=37, kind="gap"),
    dict(d=66, depth=3, L=9, B=16, kind="dense"),       # no register-tiled shape: all levels dense, per word
    dict(d=16, depth=6, L=19, B=33, kind="c4"),
    dict(d=2, depth=12, L=9, B=17, kind="long"),
    dict(d=7, depth=5, L=70, B=24, kind="full_low"),
    dict(d=70, depth=2, L=11, B=29, kind="dense"),      # wider than any register-tiled shape
    dict(d=3, depth=7, L=12, B=50, kind="dups"),
])
def test_projection_backward_lanes_on_paths(ps, set_option, dtype, case):
    set_option("embed_share", 8)    # sparse projections stay on the per-word kernels, whatever the path length
    d, depth, L, B, kind = case["d"], case["depth"], case["L"], case["B"], case["kind"]
    if kind == "words":
        proj = ps.projections.words(random_word_set(d, 1, depth, 45, seed=51), depth=depth, path_dim=d)
    elif kind == "gap":
        proj = ps.projections.words([(1,), (0, 1, 2), (2, 2, 1), (1, 0, 0, 2), (1, 0, 0, 2)], depth=depth, path_dim=d)
    elif kind == "dense":
        proj = None
    elif kind == "c4":
        proj = ps.projections.words(random_word_set(d, 3, 6, 150, seed=52), depth=depth, path_dim=d,
                                    full_levels=(1, 2))
    elif kind == "long":
        proj = ps.projections.words(random_word_set(d, 9, 12, 40, seed=53), depth=depth, path_dim=d,
                                    full_levels=(1, 2, 3))
    elif kind == "full_low":
        proj = ps.projections.words(random_word_set(d, 4, 5, 90, seed=54), depth=depth, path_dim=d,
                                    full_levels=(1, 2, 3))
    else:
        words = random_word_set(d, 2, 7, 30, seed=55)
        proj = ps.projections.words(sorted(words + words[:9], key=len), depth=depth, path_dim=d)
    sizes, codes = _plan(proj)
    path = brownian_path(B, L, d, seed=56) * 1.5
    big = d ** depth > 200_000  # the level-tensor checker would need the dense top level: per-word checker
    if big:
        from oracle import words_oracle as WO
        want = WO.sig_forward(path, depth, sizes, codes)
    else:
        want = TO.compute_signature(path, depth, sizes, codes)
    G = randn(tuple(want.shape), seed=57)
    got, grad = _run_sig(ps, path, depth, dtype, projection=proj, G=G)
    assert rel_err(got, want) < TOL[dtype]
    if big:
        want_grad = WO.sig_backward(path, want, G, depth, sizes, codes)
    else:
        want_grad = TO.signature_vjp(path, G, depth, sizes, codes)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_projection_backward_lanes_on_paths_windows(ps, set_option, dtype):
    set_option("embed_share", 8)
    d, depth, L, B = 4, 5, 30, 19
    proj = ps.projections.words(random_word_set(d, 2, 5, 60, seed=61), depth=depth, path_dim=d, full_levels=(1,))
    wins = [(0, 30), (3, 5), (2, 19), (15, 30), (4, 6), (0, 2), (28, 30), (5, 25), (5, 25), (7, 8), (40, 50)]
    sizes, codes = _plan(proj)
    path = brownian_path(B, L, d, seed=62) * 2.0
    want = TO.compute_signature(path, depth, sizes, codes, wins)
    G = randn(tuple(want.shape), seed=63)
    got, grad = _run_sig(ps, path, depth, dtype, projection=proj, windows=wins, G=G)
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth, sizes, codes, wins)
    assert rel_err(grad, want_grad) < TOL[dtype]


# ------------------------------------------------------------------------------------------------
# log-signature
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", [(2, 1), (2, 5), (3, 4), (4, 3), (5, 2)])
def test_logsignature_dense(ps, dtype, d, depth):
    B, L = 3, 14
    path = brownian_path(B, L, d, seed=41) * 2.0
    want = TO.logsignature(path, depth)
    G = randn(tuple(want.shape), seed=42)
    x = path.to(dtype).to(DEV).requires_grad_(True)
    out = ps.LogSignature(depth=depth)(x)
    (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
    assert rel_err(out.detach(), want) < TOL[dtype]
    xr = path.clone().requires_grad_(True)
    (want_grad,) = torch.autograd.grad(TO.logsignature(xr, depth), xr, G)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,windows", [(3, 4, None), (2, 5, None), (4, 3, [(0, 9), (4, 14), (6, 8)])])
def test_logsignature_lyndon(ps, dtype, d, depth, windows):
    B, L = 3, 14
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    path = brownian_path(B, L, d, seed=43) * 2.0
    offs = TO.dense_level_offsets(d, depth)
    cols = []
    it = iter(proj._codes)
    for k in range(1, depth + 1):
        if proj.level_sizes[k] == d ** k:
            cols += list(range(offs[k], offs[k + 1]))
        else:
            cols += [offs[k] + next(it) for _ in range(proj.level_sizes[k])]
    cols = torch.tensor(cols)

    def ref(x):
        return TO.logsignature(x, depth, windows).index_select(-1, cols)

    want = ref(path)
    G = randn(tuple(want.shape), seed=44)
    x = path.to(dtype).to(DEV).requires_grad_(True)
    win = None if windows is None else torch.tensor(windows, dtype=torch.int32, device=DEV)
    out = ps.LogSignature(depth=depth, projection=proj, windows=win)(x)
    assert out.shape == want.shape
    (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
    assert rel_err(out.detach(), want) < TOL[dtype]
    xr = path.clone().requires_grad_(True)
    (want_grad,) = torch.autograd.grad(ref(xr), xr, G)
    assert rel_err(grad, want_grad) < TOL[dtype]


def test_sig_to_logsig_cache_layout(ps):
    """P[idx*depth + m-1] as the reference lays it out (`sig_kernels.cu:184,215-216`), every entry written."""
    d, depth, B = 3, 4, 2
    top = [5, 80, 17, 17, 2]
    path = brownian_path(B, 9, d, seed=45)
    dense = TO.signature(path, depth)
    cols = TO.hybrid_columns(d, depth, len(top), top)
    hyb = dense[:, cols]
    want_log, want_P = TO.sig_to_logsig(hyb, depth, d, len(top), top)
    sizes = [0] + [d ** k for k in range(1, depth)] + [len(top)]
    words = torch.tensor(top, dtype=torch.int64, device=DEV)
    logsig, P = torch.ops.pathsig.sig_to_logsig(hyb.to(DEV), depth, d, True, words, sizes)
    assert P.shape == (B, len(cols) * depth)
    assert rel_err(logsig, want_log) < 1e-12
    assert rel_err(P, want_P) < 1e-12
    g = randn(tuple(hyb.shape), seed=46)
    got = torch.ops.pathsig.logsig_backward(hyb.to(DEV), P, g.to(DEV), depth, True, words, sizes)
    assert rel_err(got, TO.logsig_vjp(hyb, g, depth, d, len(top), top)) < 1e-12


def test_public_sig_to_logsig_returns_the_power_cache_with_a_gradient_too(ps):
    """`ops.sig_to_logsig` (`src/pathsig/ops.py:87-98`) returns the reference's P_arr whether or not its input
    asks for a gradient, and the gradient through it agrees with the checker's adjoint."""
    from pathsig_amd import ops
    d, depth, B = 3, 4, 2
    top = [5, 80, 17, 17, 2]
    path = brownian_path(B, 9, d, seed=45)
    cols = TO.hybrid_columns(d, depth, len(top), top)
    hyb = TO.signature(path, depth)[:, cols]
    want_log, want_P = TO.sig_to_logsig(hyb, depth, d, len(top), top)
    sizes = [0] + [d ** k for k in range(1, depth)] + [len(top)]
    words = torch.tensor(top, dtype=torch.int64, device=DEV)
    sg = hyb.to(DEV).requires_grad_(True)
    logsig, P = ops.sig_to_logsig(sg, depth, d, True, words, sizes)
    assert rel_err(logsig, want_log) < 1e-12
    assert rel_err(P, want_P) < 1e-12
    g = randn(tuple(hyb.shape), seed=46)
    (got,) = torch.autograd.grad(logsig, sg, g.to(DEV))
    assert rel_err(got, TO.logsig_vjp(hyb, g, depth, d, len(top), top)) < 1e-12
    again = ops.logsig_backward(sg.detach(), P.detach(), g.to(DEV), depth, True, words, sizes)
    assert rel_err(again, got) < 1e-12


def test_sig_to_logsig_keep_cache(ps):
    """The keeping forward returns the same log-signature and, as its cache, the tensor powers of that
    log-signature for the words below the top level (entry k - 1 of a word's row: its coefficient in L^(x)k;
    the adjoint never reads the rows of top-level words, which are left unwritten); the kept backward agrees
    with the checker's adjoint."""
    d, depth, B = 3, 4, 2
    top = [5, 80, 17, 17, 2]
    path = brownian_path(B, 9, d, seed=45) * 1.5
    dense = TO.signature(path, depth)
    cols = TO.hybrid_columns(d, depth, len(top), top)
    hyb = dense[:, cols]
    want_log, _ = TO.sig_to_logsig(hyb, depth, d, len(top), top)
    want_cache = TO.logsig_power_cache(want_log, depth, d, len(top), top)
    sizes = [0] + [d ** k for k in range(1, depth)] + [len(top)]
    words = torch.tensor(top, dtype=torch.int64, device=DEV)
    logsig, cache = torch.ops.pathsig.sig_to_logsig_keep(hyb.to(DEV), depth, d, True, words, sizes)
    assert cache.shape == (B, len(cols) * depth)
    assert rel_err(logsig, want_log) < 1e-12
    low = (len(cols) - len(top)) * depth       # the rows of the top level are not part of the hand-over
    assert rel_err(cache[:, :low], want_cache[:, :low]) < 1e-12
    g = randn(tuple(hyb.shape), seed=46)
    got = torch.ops.pathsig.logsig_backward_kept(logsig, cache, g.to(DEV), depth, True, words, sizes)
    assert rel_err(got, TO.logsig_vjp(hyb, g, depth, d, len(top), top)) < 1e-12
    checks = ("test_schema", "test_faketensor", "test_autograd_registration")
    sg = hyb.to(DEV).requires_grad_(True)
    torch.library.opcheck(torch.ops.pathsig.sig_to_logsig_keep.default, (sg, depth, d, True, words, sizes),
                          test_utils=checks)
    torch.library.opcheck(torch.ops.pathsig.logsig_backward_kept.default,
                          (logsig, cache, g.to(DEV), depth, True, words, sizes), test_utils=checks)


@pytest.mark.parametrize("form", ["gather", "scatter"])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,top", [
    (3, 4, [5, 80, 17, 17, 2]),      # listed top level, unsorted, with a repeated word
    (2, 6, None),                      # dense top level
    (5, 2, [24, 0, 7]),
    (4, 5, "lyndon"),
    (7, 3, []),                        # empty top level
    (8, 5, "lyndon"),                  # the size of the benchmark configuration
    (9, 5, None),                      # odd alphabet, dense top level of 59049 words
])
def test_logsig_adjoint_both_forms(ps, set_option, form, dtype, d, depth, top):
    """The adjoint op against the checker, in its gather form and (forced) in its scatter form."""
    set_option("logsig_scatter", 1 if form == "scatter" else 0)
    B = 5
    if top == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
        top = list(proj._codes[-proj.level_sizes[depth]:])
    path = brownian_path(B, 11, d, seed=71) * 1.5
    dense = TO.signature(path, depth)
    n_top = d ** depth if top is None else len(top)
    cols = TO.hybrid_columns(d, depth, n_top, top)
    hyb = dense[:, cols]
    sizes = [0] + [d ** k for k in range(1, depth)] + [n_top]
    words = torch.tensor([] if top is None else top, dtype=torch.int64, device=DEV)
    alt = top is not None
    logsig, P = torch.ops.pathsig.sig_to_logsig(hyb.to(dtype).to(DEV), depth, d, alt, words, sizes)
    g = randn(tuple(hyb.shape), seed=72)
    got = torch.ops.pathsig.logsig_backward(hyb.to(dtype).to(DEV), P, g.to(dtype).to(DEV), depth, alt, words, sizes)
    want = TO.logsig_vjp(hyb, g, depth, d, n_top, top)
    assert rel_err(got, want) < TOL[dtype]
    # the pair that hands the log-signature and its cache over instead of rebuilding them
    logsig_k, cache = torch.ops.pathsig.sig_to_logsig_keep(hyb.to(dtype).to(DEV), depth, d, alt, words, sizes)
    assert torch.equal(logsig_k, logsig)
    got_k = torch.ops.pathsig.logsig_backward_kept(logsig_k, cache, g.to(dtype).to(DEV), depth, alt, words, sizes)
    assert rel_err(got_k, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,top", [
    (3, 4, [5, 80, 17, 17, 2]),      # listed top level, unsorted, with a repeated word
    (2, 6, None),                      # dense top level
    (4, 5, "lyndon"),
    (7, 3, []),                        # empty top level
    (6, 5, "lyndon"),                  # 7776 dense top-level words: 30 KB (fp32), 61 KB (fp64) of LDS per row
])
def test_logsig_adjoint_many_rows(ps, dtype, d, depth, top):
    """From 256 rows on, a layout whose dense top level fits 64 KB takes the top-level products of the adjoint
    from the row's gradient staged in LDS (one block per row); same checks as for a few rows."""
    rows = 300
    if top == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
        top = list(proj._codes[-proj.level_sizes[depth]:])
    path = brownian_path(rows, 7, d, seed=77) * 1.5
    dense = TO.signature(path, depth)
    n_top = d ** depth if top is None else len(top)
    cols = TO.hybrid_columns(d, depth, n_top, top)
    hyb = dense[:, cols]
    sizes = [0] + [d ** k for k in range(1, depth)] + [n_top]
    words = torch.tensor([] if top is None else top, dtype=torch.int64, device=DEV)
    alt = top is not None
    g = randn(tuple(hyb.shape), seed=78)
    logsig, cache = torch.ops.pathsig.sig_to_logsig_keep(hyb.to(dtype).to(DEV), depth, d, alt, words, sizes)
    got = torch.ops.pathsig.logsig_backward_kept(logsig, cache, g.to(dtype).to(DEV), depth, alt, words, sizes)
    sub = slice(0, rows, 7)
    want = TO.logsig_vjp(hyb[sub], g[sub], depth, d, n_top, top)
    assert rel_err(got[sub], want) < TOL[dtype]
    # the same rows a few at a time take the other kernel; both must agree closely
    few = torch.ops.pathsig.logsig_backward_kept(logsig[:40].contiguous(), cache[:40].contiguous(),
                                                 g[:40].to(dtype).to(DEV), depth, alt, words, sizes)
    assert rel_err(got[:40], few) < TOL[dtype] * 0.1


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,L,scale,kind", [
    (2, 7, 3, 2.0, "lyndon"), (2, 8, 3, 2.0, "lyndon"), (2, 8, 65, 2.0, "dense"), (2, 8, 130, 2.0, "dense"),
    (2, 8, 130, 2.0, "lyndon"), (3, 6, 2, 2.0, "dense"), (3, 6, 200, 2.0, "dense"), (3, 7, 40, 2.0, "lyndon"),
    (3, 8, 100, 3.0, "lyndon"), (2, 10, 50, 2.0, "lyndon"), (2, 12, 30, 2.0, "lyndon"), (3, 9, 20, 1.0, "lyndon"),
])
def test_logsignature_deep_and_long(ps, dtype, d, depth, L, scale, kind):
    """Regimes where the powers of S - 1 reach 1e5 .. 1e7 while the log-signature stays O(10): summing the
    alternating series of the reference in fp32 is off by 1e-4 .. 1e-3 there (its literal fp32 restatement in
    oracle/ref_words.c shows the same), the inverted exponential series holds the fp32 tolerance.  Depths follow
    the sweep of the reference's `tests/test_logsig.py:138-146` (depth 2..12 at d = 3, fp32 at 1e-5 / 1e-4)."""
    B = 2
    proj = ps.projections.lyndon(depth=depth, path_dim=d) if kind == "lyndon" else None
    path = brownian_path(B, L, d, seed=300 + depth) * scale
    cols = None if proj is None else torch.tensor(TO.projection_columns(d, depth, proj.level_sizes, proj._codes))
    # the checker sees the inputs of the call, rounded to its type
    xr = path.to(dtype).double().requires_grad_(True)
    # checker: the logarithm by inverting the exponential (the alternating series of the reference, summed in
    # fp64, is itself off by 1e-11 in these regimes; tests/test_oracle_math.py pins both against extended precision)
    full = TO.logsignature(xr, depth, method="inverse_exp")
    ref = full if cols is None else full.index_select(-1, cols)
    G = randn(tuple(ref.shape), seed=301).to(dtype)
    (ref_grad,) = torch.autograd.grad(ref, xr, G.double())
    x = path.to(dtype).to(DEV).requires_grad_(True)
    out = ps.LogSignature(depth=depth, projection=proj)(x)
    (grad,) = torch.autograd.grad(out, x, G.to(DEV))
    assert rel_err(out, ref.detach()) < TOL[dtype]
    # One case sits on the fp32 bound: 200 increments at d = 3, depth 6, where the gradient of the logarithm is a
    # difference of terms a hundred times its size.  Measured 1.19e-5; 7.9e-6 with the signature part in fp64,
    # 1.14e-5 with the logarithm part in fp64, 3e-8 with both; the fp32 signature tensor that crosses the operator
    # boundary alone costs 1.0e-6 (checker evaluated on the rounded signature).  The reference's own suite allows
    # 1e-3 for fp32 log-signature gradients below depth 10 (`tests/test_logsig.py:29-30`).
    on_the_bound = dtype == torch.float32 and (d, depth, L) == (3, 6, 200)
    assert rel_err(grad, ref_grad) < (2e-5 if on_the_bound else TOL[dtype])


# ------------------------------------------------------------------------------------------------
# behaviour at the operator boundary
# ------------------------------------------------------------------------------------------------
def test_errors(ps):
    x = torch.zeros(2, 5, 3, device=DEV)
    with pytest.raises(ValueError):
        ps.Signature(depth=0)
    with pytest.raises(ValueError):
        ps.Signature(depth=13)
    with pytest.raises(TypeError):
        ps.Signature(depth=2, windows=torch.zeros(3, 2, dtype=torch.int64))
    with pytest.raises(TypeError):
        ps.Signature(depth=2, windows=torch.zeros(3, 3, dtype=torch.int64, device=DEV))
    with pytest.raises(RuntimeError):
        ps.Signature(depth=2)(torch.zeros(2, 1, 3, device=DEV))
    with pytest.raises(RuntimeError):
        ps.Signature(depth=2)(torch.zeros(2, 5, 3, device=DEV, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        ps.Signature(depth=2)(torch.zeros(5, 3, device=DEV))
    assert ps.Signature(depth=2)(x).shape == (2, 12)


# The regimes the reference's own suite sweeps (`tests/test_sig.py:135-152`): depths 7..12, path dimensions
# up to 100, batches up to 512; and the window / no-projection combinations of LogSignature
# (`tests/test_windows.py:62-93`).
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,L,B", [
    (2, 7, 12, 3), (2, 9, 10, 2), (2, 10, 8, 20), (2, 11, 7, 2), (3, 7, 9, 2), (100, 2, 6, 3), (64, 2, 9, 40),
    (30, 3, 7, 2), (31, 2, 5, 16), (3, 3, 10, 512), (2, 4, 50, 512),
])
def test_reference_test_regimes(ps, dtype, d, depth, L, B):
    path = brownian_path(B, L, d, seed=300 + d + depth) * 1.5
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=301)
    got, grad = _run_sig(ps, path, depth, dtype, G=G)
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", [(3, 4), (2, 6), (8, 2)])
def test_logsignature_windows_without_projection(ps, dtype, d, depth):
    B, L = 4, 21
    wins = [(0, 21), (3, 9), (10, 12), (5, 6), (8, 21)]
    path = brownian_path(B, L, d, seed=310)
    want = TO.logsignature(path, depth, wins)
    G = randn(tuple(want.shape), seed=311)
    x = path.to(dtype).to(DEV).requires_grad_(True)
    win = torch.tensor(wins, dtype=torch.int64, device=DEV)
    out = ps.LogSignature(depth=depth, windows=win)(x)
    assert out.shape == want.shape
    (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
    assert rel_err(out.detach(), want) < TOL[dtype]
    xr = path.clone().requires_grad_(True)
    (want_grad,) = torch.autograd.grad(TO.logsignature(xr, depth, wins), xr, G)
    assert rel_err(grad, want_grad) < TOL[dtype]


def test_opcheck_and_compile(ps):
    """The four ops pass torch's operator checks (schema, fake tensors, autograd registration), as their
    `pt2_compliant_tag` promises (`bindings.cpp:19`), and the modules trace under torch.compile."""
    d, depth, B, L = 3, 3, 4, 9
    x = brownian_path(B, L, d, seed=320).to(DEV)
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    win = torch.tensor([[0, 5], [2, 9]], dtype=torch.int32, device=DEV)
    empty_w = torch.empty(0, dtype=torch.int64, device=DEV)
    empty_win = torch.empty((0, 2), dtype=torch.int32, device=DEV)
    checks = ("test_schema", "test_faketensor", "test_autograd_registration")
    xg = x.clone().requires_grad_(True)
    torch.library.opcheck(torch.ops.pathsig.compute_signature.default, (xg, depth, False, empty_w, [], False, empty_win),
                          test_utils=checks)
    torch.library.opcheck(torch.ops.pathsig.compute_signature.default,
                          (xg, depth, True, proj.encoded_words, list(proj.level_sizes), True, win), test_utils=checks)
    sig = ps.Signature(depth=depth)(x)
    g = torch.randn_like(sig)
    torch.library.opcheck(torch.ops.pathsig.signature_backward.default,
                          (x, sig, g, depth, False, empty_w, [], False, empty_win), test_utils=checks)
    # the log-signature ops always get the level sizes of the hybrid layout (`modules.py:113-120`)
    full = [0] + [d ** k for k in range(1, depth + 1)]
    sg = sig.clone().requires_grad_(True)
    torch.library.opcheck(torch.ops.pathsig.sig_to_logsig.default, (sg, depth, d, False, empty_w, full), test_utils=checks)
    logsig, P = torch.ops.pathsig.sig_to_logsig(sig, depth, d, False, empty_w, full)
    torch.library.opcheck(torch.ops.pathsig.logsig_backward.default,
                          (sig, P, torch.randn_like(sig), depth, False, empty_w, full), test_utils=checks)
    mod = ps.LogSignature(depth=depth, projection=proj)
    compiled = torch.compile(mod, fullgraph=True, backend="aot_eager")
    xc = x.clone().requires_grad_(True)
    out = compiled(xc)
    want = mod(x)
    assert rel_err(out, want) < 1e-12
    (gc,) = torch.autograd.grad(out, xc, torch.ones_like(out))
    xe = x.clone().requires_grad_(True)
    (ge,) = torch.autograd.grad(mod(xe), xe, torch.ones_like(want))
    assert rel_err(gc, ge) < 1e-12


def test_long_path_fp32_stays_accurate(ps):
    """The reverse reconstruction S_t = S_{t+1} (x) exp(-dx_t) runs in the input precision; time chunks keep
    its drift bounded on long paths."""
    d, depth, B, L = 4, 6, 3, 8192
    path = brownian_path(B, L, d, seed=330) * 2.0
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=331)
    got, grad = _run_sig(ps, path, depth, torch.float32, G=G)
    assert rel_err(got, want) < 1e-5
    assert rel_err(grad, TO.signature_vjp(path, G, depth)) < 1e-5


def test_graph_capture_and_replay(ps):
    """The library only enqueues kernels on the caller's stream (no allocation, no synchronisation, no memset
    nodes), so forward + backward can be captured in a graph; every replay is checked against eager results."""
    d, depth, B, L = 4, 4, 16, 40
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    words = ps.projections.words(random_word_set(d, 2, 4, 30, seed=341), depth=depth, path_dim=d, full_levels=(1,))
    # dense kernels, the log-signature chain, and the per-word kernels (batch of 16: lanes on paths)
    mods = [ps.Signature(depth=depth), ps.LogSignature(depth=depth, projection=proj),
            ps.Signature(depth=depth, projection=words)]
    inputs = [brownian_path(B, L, d, seed=340 + i).to(torch.float32).to(DEV) for i in range(3)]
    for mod in mods:
        static_x = inputs[0].clone().requires_grad_(True)
        static_g = torch.ones_like(mod(static_x.detach()))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):  # warm-up on the capture stream
                (gw,) = torch.autograd.grad(mod(static_x), static_x, static_g)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = mod(static_x)
            (static_grad,) = torch.autograd.grad(static_out, static_x, static_g)
        for x in inputs + inputs[:1]:
            with torch.no_grad():
                static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            xe = x.clone().requires_grad_(True)
            want = mod(xe)
            (want_grad,) = torch.autograd.grad(want, xe, torch.ones_like(want))
            assert rel_err(static_out, want) < 1e-6
            assert rel_err(static_grad, want_grad) < 1e-5


def test_non_contiguous_and_empty_batch(ps):
    d, depth = 3, 3
    base = brownian_path(2, 8, 2 * d, seed=51)
    view = base.to(DEV)[:, :, ::2]
    got = ps.Signature(depth=depth)(view)
    assert rel_err(got, TO.signature(base[:, :, ::2].contiguous(), depth)) < 1e-12
    empty = ps.Signature(depth=depth)(torch.zeros(0, 8, d, device=DEV, dtype=torch.float64))
    assert empty.shape == (0, TO.dense_size(d, depth))


def test_state_dict_buffers(ps):
    proj = ps.projections.lyndon(depth=3, path_dim=3)
    win = torch.tensor([[0, 4], [2, 6]], device=DEV)
    sd = ps.Signature(depth=3, projection=proj, windows=win).state_dict()
    assert set(sd) == {"_windows", "_encoded_words"} and sd["_windows"].dtype == torch.int32
    assert ps.Signature(depth=3).state_dict() == {}
    sd = ps.LogSignature(depth=3, projection=proj).state_dict()
    assert set(sd) == {"_encoded_words", "_top_words", "_indices_from_sig"}
    assert ps.LogSignature(depth=3).state_dict() == {}


def test_gradcheck(ps):
    torch.manual_seed(0)
    x = torch.randn(2, 6, 2, dtype=torch.float64, device=DEV, requires_grad=True)
    # the per-word backward kernels add the contributions of their blocks (levels, windows) with float atomics,
    # as the reference does (`sig_backward_kernels.cu:317`), so repeated backward passes may differ in the last bits
    nd = dict(atol=1e-5, rtol=1e-3, nondet_tol=1e-12)
    assert torch.autograd.gradcheck(ps.Signature(depth=3), (x,), **nd)
    assert torch.autograd.gradcheck(ps.LogSignature(depth=3), (x,), **nd)
    proj = ps.projections.lyndon(depth=3, path_dim=2)
    win = torch.tensor([[0, 4], [2, 6], [1, 3]], device=DEV)
    assert torch.autograd.gradcheck(ps.LogSignature(depth=3, projection=proj, windows=win), (x,), **nd)


# ------------------------------------------------------------------------------------------------
# shapes served by the register-tiled dense kernels (forward, backward, windows, long paths)
# ------------------------------------------------------------------------------------------------
TILED = [(4, 6), (8, 4), (6, 5), (4, 4), (3, 5), (2, 8), (3, 6), (4, 5), (5, 4), (5, 5), (5, 6), (6, 4), (7, 4), (7, 5),
         (2, 2), (5, 2), (8, 2), (2, 3), (3, 3), (6, 3), (7, 3), (8, 3), (2, 4), (3, 4), (2, 5), (2, 6),
         (9, 2), (13, 2), (16, 2), (9, 3), (11, 3), (16, 3), (9, 4), (10, 4), (2, 7), (3, 7), (4, 7), (3, 8), (2, 9), (2, 10),
         (17, 2), (32, 2), (17, 3), (27, 3), (32, 3), (33, 2), (50, 2), (64, 2),
         (2, 11), (3, 9), (2, 12)]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", TILED)
def test_tiled_shapes(ps, dtype, d, depth):
    B, L = 3, 150  # more than one LDS tile of increments, not a multiple of the tile
    path = brownian_path(B, L, d, seed=200 + d + depth)
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=61)
    got, grad = _run_sig(ps, path, depth, dtype, G=G)
    assert rel_err(got, want) < TOL[dtype]
    assert rel_err(grad, TO.signature_vjp(path, G, depth)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", [(4, 6), (6, 5), (8, 4)])
def test_tiled_shapes_with_windows(ps, dtype, d, depth):
    B, L = 2, 100
    path = brownian_path(B, L, d, seed=300 + d)
    wins = [(0, 100), (0, 64), (32, 96), (64, 100), (10, 12), (50, 50), (3, 80), (3, 80)]
    want = TO.compute_signature(path, depth, windows=wins)
    G = randn(tuple(want.shape), seed=62)
    got, grad = _run_sig(ps, path, depth, dtype, windows=wins, G=G)
    assert rel_err(got, want) < TOL[dtype]
    want_grad = TO.signature_vjp(path, G, depth, windows=wins)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("chunks", ["2", "5", "16"])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", TILED)
def test_tiled_shapes_time_chunked(ps, set_option, chunks, dtype, d, depth):
    """Long paths are cut into time chunks whose signatures are multiplied back together (Chen);
    The "chunks" option forces the chunk count so that small inputs exercise that path too."""
    set_option("chunks", int(chunks))
    B, L = 2, 150
    path = brownian_path(B, L, d, seed=400 + d + depth)
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=63)
    got, grad = _run_sig(ps, path, depth, dtype, G=G)
    assert rel_err(got, want) < TOL[dtype]
    assert rel_err(grad, TO.signature_vjp(path, G, depth)) < TOL[dtype]


@pytest.mark.parametrize("L", [2, 3, 5, 67])
@pytest.mark.parametrize("d,depth", TILED)
def test_tiled_shapes_more_chunks_than_increments(ps, set_option, d, depth, L):
    """Chunks without increments, one-increment chunks, and chunks longer than a tile of the reverse sweep:
    the backward writes the path gradient chunk by chunk and must leave no point untouched."""
    set_option("chunks", 4)
    B = 3
    path = brownian_path(B, L, d, seed=450 + d + depth + L)
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=65)
    for dtype in (torch.float64, torch.float32):
        x = path.to(dtype).to(DEV).requires_grad_(True)
        out = ps.Signature(depth=depth)(x)
        # a poisoned gradient buffer would show cells that the kernels never write
        (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
        assert torch.isfinite(grad).all()
        assert rel_err(out, want) < TOL[dtype]
        assert rel_err(grad, TO.signature_vjp(path, G, depth)) < TOL[dtype]


@pytest.mark.parametrize("d,depth", [(4, 6), (6, 5)])
def test_tiled_shapes_time_chunked_windows(ps, set_option, d, depth):
    set_option("chunks", 4)
    B, L = 2, 100
    path = brownian_path(B, L, d, seed=500 + d)
    wins = [(0, 100), (0, 64), (32, 96), (64, 100), (10, 12), (50, 50), (3, 80), (97, 100)]  # some shorter than the chunk count
    want = TO.compute_signature(path, depth, windows=wins)
    G = randn(tuple(want.shape), seed=64)
    got, grad = _run_sig(ps, path, depth, torch.float64, windows=wins, G=G)
    assert rel_err(got, want) < 1e-12
    assert rel_err(grad, TO.signature_vjp(path, G, depth, windows=wins)) < 1e-12


# ------------------------------------------------------------------------------------------------
# word projections that are computed through the dense kernels and gathered (top level kept >= 1/8)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,kind", [(4, 4, "lyndon"), (3, 5, "lyndon"), (4, 4, "words"), (3, 5, "dups")])
def test_projection_through_dense_kernels(ps, dtype, d, depth, kind):
    B, L = 3, 70
    if kind == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
    elif kind == "words":
        words = random_word_set(d, 1, depth - 1, 30, seed=9) + [w for w in random_word_set(d, depth, depth, 80, seed=10)]
        proj = ps.projections.words(words, depth=depth, path_dim=d)
    else:  # repeated words: their gradients must add up
        top = random_word_set(d, depth, depth, 40, seed=11)
        proj = ps.projections.words([(0,), (2,), (0,), (1, 1), (1, 1)] + top + top[:7], depth=depth, path_dim=d)
    sizes, codes = _plan(proj)
    assert sizes[depth] * 8 >= d ** depth
    path = brownian_path(B, L, d, seed=71)
    wins = [(0, 70), (5, 40), (33, 35)]
    for windows in (None, wins):
        want = TO.compute_signature(path, depth, sizes, codes, windows)
        G = randn(tuple(want.shape), seed=72)
        got, grad = _run_sig(ps, path, depth, dtype, projection=proj, windows=windows, G=G)
        assert rel_err(got, want) < TOL[dtype]
        want_grad = TO.signature_vjp(path, G, depth, sizes, codes, windows)
        assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,kind", [(3, 2, "lyndon"), (16, 2, "lyndon"), (20, 2, "dups"), (6, 6, "lyndon"),
                                          (11, 4, "lyndon"), (9, 5, "words")])
def test_projection_through_shapes_swept_in_one_piece(ps, dtype, d, depth, kind):
    """The shapes whose units take several blocks are never cut into time chunks, so the backward of a projection
    computed through them reads the dense signature: kept by the forward (the modules) or swept again (the
    stateless pair of operators).  Both must agree with the checker, with and without windows.  (Depth 2, whose
    chunk signatures are plain sums of increments, rides along.)"""
    B, L = 2, 9
    if kind == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
    elif kind == "dups":
        top = random_word_set(d, depth, depth, 120, seed=21)
        proj = ps.projections.words([(3,), (0,), (3,)] + top + top[:9], depth=depth, path_dim=d)
    else:
        top = random_word_set(d, depth, depth, d ** depth // 6, seed=22)
        proj = ps.projections.words(random_word_set(d, 1, depth - 1, 50, seed=23) + top, depth=depth, path_dim=d)
    sizes, codes = _plan(proj)
    assert sizes[depth] * 8 >= d ** depth
    path = brownian_path(B, L, d, seed=75) * 1.5
    for windows in (None, [(0, 9), (2, 7), (4, 5), (6, 6), (2, 7)]):
        want = TO.compute_signature(path, depth, sizes, codes, windows)
        G = randn(tuple(want.shape), seed=76)
        want_grad = TO.signature_vjp(path, G, depth, sizes, codes, windows)
        got, grad = _run_sig(ps, path, depth, dtype, projection=proj, windows=windows, G=G)   # keeping pair
        assert rel_err(got, want) < TOL[dtype]
        assert rel_err(grad, want_grad) < TOL[dtype]
        x = path.to(dtype).to(DEV)
        win = None if windows is None else torch.tensor(windows, dtype=torch.int64, device=DEV)
        mod = ps.Signature(depth=depth, projection=proj, windows=win)
        args = (mod.depth, mod.alternative_projection, mod._encoded_words, mod._level_sizes, mod.use_windows,
                mod._windows)
        sig = torch.ops.pathsig.compute_signature(x, *args)
        sig_k, kept = torch.ops.pathsig.compute_signature_keep(x, *args)
        rows = B * (1 if windows is None else len(windows))
        if depth > 2:  # units of several blocks: the dense signature is what is kept (depth 2 is time-chunked)
            assert kept.numel() == rows * TO.dense_size(d, depth)
        assert torch.equal(sig, sig_k)
        g2 = torch.ops.pathsig.signature_backward(x, sig, G.to(dtype).to(DEV), *args)            # sweeps again
        assert rel_err(g2.cpu(), want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_logsignature_lyndon_through_dense_kernels(ps, dtype):
    d, depth, B, L = 4, 4, 3, 60
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    path = brownian_path(B, L, d, seed=73)
    cols = torch.tensor(TO.projection_columns(d, depth, proj.level_sizes, proj._codes))
    want = TO.logsignature(path, depth).index_select(-1, cols)
    G = randn(tuple(want.shape), seed=74)
    x = path.to(dtype).to(DEV).requires_grad_(True)
    out = ps.LogSignature(depth=depth, projection=proj)(x)
    (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
    assert rel_err(out.detach(), want) < TOL[dtype]
    xr = path.clone().requires_grad_(True)
    (want_grad,) = torch.autograd.grad(TO.logsignature(xr, depth).index_select(-1, cols), xr, G)
    assert rel_err(grad, want_grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("kind", ["irregular", "lyndon"])
def test_projection_through_dense_kernels_with_letter_bounds(ps, set_option, dtype, kind):
    """d = 8, depth 5: the sweeps leave out the top-level words whose later letters fall below the
    smallest one used after the same first letter.  The word list has a different bound per first letter,
    one first letter without words, and unordered, repeated words; the run without bounds must agree."""
    import itertools
    d, depth, B, L = 8, 5, 2, 45
    if kind == "lyndon":
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
    else:
        least = {0: 0, 1: 3, 2: 8, 3: 1, 5: 6, 6: 7, 7: 2}   # first letter -> smallest later letter (4: no words)
        rng = random.Random(12)
        top = []
        for first, lo in least.items():
            if lo >= d:
                continue
            tails = list(itertools.product(range(lo, d), repeat=depth - 1))
            keep = tails if first == 0 else rng.sample(tails, min(len(tails), 300))
            top += [(first,) + t for t in keep]
            top.append((first,) + (lo,) * (depth - 1))       # the bound is attained
        rng.shuffle(top)
        top += top[:5]
        proj = ps.projections.words(top, depth=depth, path_dim=d, full_levels=(1, 2, 3, 4))
    sizes, codes = _plan(proj)
    assert sizes[depth] * 8 >= d ** depth and sizes[depth] < d ** depth
    path = brownian_path(B, L, d, seed=91) * 1.5
    for windows in (None, [(0, 45), (7, 30), (20, 22)]):
        want = TO.compute_signature(path, depth, sizes, codes, windows)
        G = randn(tuple(want.shape), seed=92)
        got, grad = _run_sig(ps, path, depth, dtype, projection=proj, windows=windows, G=G)
        assert rel_err(got, want) < TOL[dtype]
        assert rel_err(grad, TO.signature_vjp(path, G, depth, sizes, codes, windows)) < TOL[dtype]
        set_option("letter_bounds", 0)
        plain, plain_grad = _run_sig(ps, path, depth, dtype, projection=proj, windows=windows, G=G)
        set_option("letter_bounds", 1)
        assert rel_err(got, plain) < TOL[dtype] and rel_err(grad, plain_grad) < TOL[dtype]


@pytest.mark.parametrize("d,depth", [(2, 7), (3, 5), (3, 6), (3, 7), (4, 5), (4, 7), (5, 4), (5, 5), (6, 4), (6, 5),
                                     (7, 4), (8, 4), (8, 5), (12, 4), (16, 4)])
@pytest.mark.parametrize("chunks", [8, 12])
def test_grouped_handover_across_shapes(ps, set_option, d, depth, chunks):
    """fp32 rows of eight and more time chunks in whole groups of four: the keeping forward hands the chunk products
    over by groups where the shape is compiled for it (the modules take the keeping pair).  Signature and gradient
    against the checker, with chunks of unequal length and with windows, and against the run with the switch off."""
    set_option("chunks", chunks)
    B, L = 2, 16 * chunks + 5
    path = brownian_path(B, L, d, seed=97) * (1.2 if depth < 7 else 0.8)
    for windows in (None, [(0, L), (4, L - 3), (L // 3, L // 3 + 2)]):
        want = TO.compute_signature(path, depth, windows=windows)
        G = randn(tuple(want.shape), seed=98)
        want_grad = TO.signature_vjp(path, G, depth, windows=windows)
        got, grad = _run_sig(ps, path, depth, torch.float32, windows=windows, G=G)
        assert rel_err(got, want) < TOL[torch.float32]
        assert rel_err(grad, want_grad) < TOL[torch.float32]
        set_option("grouped", 0)
        plain, plain_grad = _run_sig(ps, path, depth, torch.float32, windows=windows, G=G)
        set_option("grouped", 1)
        assert torch.equal(got, plain) and rel_err(grad, plain_grad) < TOL[torch.float32]


@pytest.mark.parametrize("d,depth", [(8, 5), (8, 4)])
@pytest.mark.parametrize("chunks", [2, 3, 5])
def test_letter_bounds_in_one_wave_blocks(ps, set_option, d, depth, chunks):
    """fp32 sweeps with letter bounds run one wave to a block (the blocks of a first letter together in the grid,
    the per-increment sums of a unit's waves added in memory): Lyndon projection at forced chunk counts, chunks of
    unequal length, with and without windows, against the checker and against the run without bounds."""
    set_option("chunks", chunks)
    B, L = 3, 16 * chunks + 7
    proj = ps.projections.lyndon(depth=depth, path_dim=d)
    sizes, codes = _plan(proj)
    path = brownian_path(B, L, d, seed=95) * 1.2
    for windows in (None, [(0, L), (3, L - 2), (L // 2, L // 2 + 1)]):
        want = TO.compute_signature(path, depth, sizes, codes, windows)
        G = randn(tuple(want.shape), seed=96)
        got, grad = _run_sig(ps, path, depth, torch.float32, projection=proj, windows=windows, G=G)
        assert rel_err(got, want) < TOL[torch.float32]
        assert rel_err(grad, TO.signature_vjp(path, G, depth, sizes, codes, windows)) < TOL[torch.float32]
        set_option("letter_bounds", 0)
        plain, plain_grad = _run_sig(ps, path, depth, torch.float32, projection=proj, windows=windows, G=G)
        set_option("letter_bounds", 1)
        assert rel_err(got, plain) < TOL[torch.float32] and rel_err(grad, plain_grad) < TOL[torch.float32]


# ------------------------------------------------------------------------------------------------
# hand-over of the time-chunk signatures from the forward to the backward of one call
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("case", ["dense", "windows", "lyndon", "not_chunked", "per_word", "words_few_paths",
                                  "words_many_paths", "words_windows", "groups_of_four", "three_groups",
                                  "groups_windows", "groups_off"])
def test_forward_keeps_chunk_signatures_for_backward(ps, set_option, dtype, case):
    """`compute_signature_keep` / `signature_backward_kept` (what the modules use when a gradient is wanted)
    against the reference's pair `compute_signature` / `signature_backward`: same signature, same dL/dpath.
    Kept are the time-chunk signatures of the register-tiled kernels, or, on the per-word kernels, the prefix
    values of the words whose prefixes are not in the saved signature (both backward kernels read them: lanes
    on words for a few paths, lanes on paths for a dozen and more); the buffer is empty when neither applies."""
    import ctypes
    from pathsig_amd import _load
    set_option("embed_share", 8)    # the words_* cases are about the per-word kernels
    depth, kw, chunked = 4, {}, True
    if case == "dense":
        d, B, L = 4, 5, 300
        set_option("chunks", 5)
    elif case == "windows":
        d, B, L = 4, 3, 200
        kw["windows"] = [(0, 200), (10, 150), (40, 42), (7, 7)]
        set_option("chunks", 4)
    elif case == "lyndon":
        d, depth, B, L = 8, 5, 2, 90
        kw["projection"] = ps.projections.lyndon(depth=depth, path_dim=d, full_levels=(1, 2, 3, 4))
        set_option("chunks", 3)
    elif case in ("groups_of_four", "groups_off"):
        d, depth, B, L = 4, 6, 3, 400       # fp32, a multiple of four chunks, eight and more: products within groups
        set_option("chunks", 16)            # of four from the forward sweep, products of whole groups from a scan
        if case == "groups_off":
            set_option("grouped", 0)
    elif case == "three_groups":
        d, B, L = 4, 5, 333
        set_option("chunks", 12)
    elif case == "groups_windows":
        d, B, L = 4, 3, 200
        kw["windows"] = [(0, 200), (10, 150), (40, 42), (7, 7), (3, 199)]
        set_option("chunks", 8)
    elif case == "not_chunked":
        d, B, L, chunked = 4, 3000, 20, False
    elif case == "per_word":
        d, B, L, chunked = 17, 3, 40, False         # no register-tiled shape for d = 17: per-word kernels, all dense
    else:
        d, depth, L = 5, 5, 60
        B = 3 if case == "words_few_paths" else 20
        words = random_word_set(d, 1, depth, 70, seed=403)
        kw["projection"] = ps.projections.words(words, depth=depth, path_dim=d)
        if case == "words_windows":
            kw["windows"] = [(0, 60), (5, 31), (20, 21), (9, 9)]
    path = brownian_path(B, L, d, seed=401) * 1.5
    x = path.to(dtype).to(DEV)
    wins = kw.get("windows")
    mod = ps.Signature(depth=depth, projection=kw.get("projection"),
                       windows=None if wins is None else torch.tensor(wins, dtype=torch.int64, device=DEV))
    args = (mod.depth, mod.alternative_projection, mod._encoded_words, mod._level_sizes, mod.use_windows, mod._windows)
    sig = torch.ops.pathsig.compute_signature(x, *args)
    G = randn(tuple(sig.shape), seed=402).to(dtype).to(DEV)
    grad = torch.ops.pathsig.signature_backward(x, sig, G, *args)
    sig_k, chunks = torch.ops.pathsig.compute_signature_keep(x, *args)
    assert (chunks.numel() > 0) == chunked
    sizes = None if not mod.alternative_projection else (ctypes.c_int64 * len(mod._level_sizes))(*mod._level_sizes)
    assert chunks.numel() * chunks.element_size() == _load.lib().pathsig_sig_chunks_bytes(
        0 if dtype == torch.float32 else 1, B, L, d, depth, sizes, 0 if wins is None else len(wins))
    grad_k = torch.ops.pathsig.signature_backward_kept(x, sig_k, G, chunks, *args)
    assert torch.equal(sig_k, sig)
    # two runs of the per-word backward differ by the order of their float atomics (a few 1e-6 of the largest
    # gradient in fp32 at 83521 words); the register-tiled backward is deterministic without windows
    close = TOL[dtype] * (0.5 if case == "per_word" else 0.1)
    assert rel_err(grad_k, grad) < close
    # the module takes the keeping pair when a gradient is wanted
    xg = x.clone().requires_grad_(True)
    out = mod(xg)
    assert out.grad_fn is not None and "keep" in out.grad_fn.name().lower()
    (grad_m,) = torch.autograd.grad(out, xg, G)
    assert torch.equal(out.detach(), sig) and rel_err(grad_m, grad) < close
    # a chunk buffer of another size than the call keeps now (kept under other tuning switches) is left unread:
    # the backward recomputes what it needs
    if chunked:
        again = torch.ops.pathsig.signature_backward_kept(x, sig, G, chunks[:-1], *args)
        assert rel_err(again, grad) < close
    if case == "dense":
        set_option("chunks", 10)
        assert chunks.numel() * chunks.element_size() != _load.lib().pathsig_sig_chunks_bytes(
            0 if dtype == torch.float32 else 1, B, L, d, depth, sizes, 0)
        again = torch.ops.pathsig.signature_backward_kept(x, sig, G, chunks, *args)
        assert rel_err(again, grad) < TOL[dtype]
        set_option("chunks", 5)
    if case == "groups_of_four" and dtype == torch.float32:
        # kept by groups, read back with the switch off: another size than the call would keep now, so left unread
        set_option("grouped", 0)
        assert chunks.numel() * chunks.element_size() > _load.lib().pathsig_sig_chunks_bytes(0, B, L, d, depth, sizes, 0)
        again = torch.ops.pathsig.signature_backward_kept(x, sig, G, chunks, *args)
        assert rel_err(again, grad) < TOL[dtype]
        set_option("grouped", 1)
    checks = ("test_schema", "test_faketensor", "test_autograd_registration")
    if case in ("dense", "per_word") and dtype == torch.float64:
        torch.library.opcheck(torch.ops.pathsig.compute_signature_keep.default, (xg, *args), test_utils=checks)
        torch.library.opcheck(torch.ops.pathsig.signature_backward_kept.default, (x, sig, G, chunks, *args),
                              test_utils=checks)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("chunks", [None, "4"])
def test_shape_with_two_prefix_lengths(ps, set_option, dtype, chunks):
    """(d, depth) = (8, 4) is compiled with lanes on prefixes of length 2 and of length 3; small batches take the
    longer prefix (the other tests of this shape), a batch that fills the GPU takes the shorter one."""
    if chunks:
        set_option("chunks", int(chunks))
    d, depth, B, L = 8, 4, 200, 100
    path = brownian_path(B, L, d, seed=501)
    for windows in (None, [(0, 100), (10, 90), (50, 52)]):
        want = TO.compute_signature(path, depth, windows=windows)
        G = randn(tuple(want.shape), seed=502)
        got, grad = _run_sig(ps, path, depth, dtype, windows=windows, G=G)
        assert rel_err(got, want) < TOL[dtype]
        assert rel_err(grad, TO.signature_vjp(path, G, depth, windows=windows)) < TOL[dtype]


@pytest.mark.parametrize("d,depth", [(4, 6), (6, 5)])
def test_many_long_rows_fp32_one_chunk(ps, d, depth):
    """2048 rows of 4096 points in fp32: with that many rows the register-tiled kernels fill the GPU without
    cutting the paths into time chunks, so the uncompensated forward accumulation and the reverse reconstruction
    S_t = S_{t+1} (x) exp(-dx_t) both run over all 4095 increments in one piece.  Two of the paths against the
    per-word C checker in fp64, level by level."""
    from oracle import words_oracle as WO
    from tests.helpers import level_rel_errs, strict_rel_err
    B, L, sub = 2048, 4096, 2
    head = brownian_path(sub, L, d, seed=77)
    rest = brownian_path(8, L, d, seed=78).repeat(B // 8, 1, 1)[:B - sub]
    x = torch.cat([head, rest]).float().to(DEV).requires_grad_(True)
    out = ps.Signature(depth=depth)(x)
    want = WO.sig_forward(head, depth)
    G_head = randn(tuple(want.shape), seed=79)
    G = torch.cat([G_head, randn((8, want.shape[1]), seed=80).repeat(B // 8, 1)[:B - sub]]).float().to(DEV)
    (grad,) = torch.autograd.grad(out, x, G)
    assert rel_err(out[:sub], want) < 1e-5
    errs = level_rel_errs(out[:sub], want, [d ** k for k in range(1, depth + 1)])
    assert max(errs) < 2e-5, errs
    want_grad = WO.sig_backward(head, want, G_head, depth)
    assert rel_err(grad[:sub], want_grad) < 1e-5
    assert strict_rel_err(grad[:sub], want_grad) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", [(6, 6), (7, 6), (8, 6), (11, 4), (16, 4), (9, 5), (12, 5), (33, 3), (47, 3), (64, 3),
                                     (3, 10), (4, 8), (5, 7), (6, 7), (7, 7), (4, 9), (3, 11), (3, 12), (5, 8), (9, 6),
                                     (13, 5), (16, 5), (17, 4), (25, 4), (32, 4)])
def test_shapes_whose_units_take_several_blocks(ps, dtype, d, depth):
    """d^6 for d >= 6, d^4 for d >= 11, d^5 for d >= 9: a row's lanes (one per prefix) do not fit one block; the
    unit is spread over two to twenty-one blocks, swept in one piece, and the per-increment sums of the backward
    meet in memory.  With and without windows (overlapping ones included)."""
    B, L = 2, 8
    path = brownian_path(B, L, d, seed=500 + d) * 2.0
    for windows in (None, [(0, 8), (2, 7), (3, 4), (5, 5)]):
        want = TO.compute_signature(path, depth, None, None, windows)
        G = randn(tuple(want.shape), seed=501)
        got, grad = _run_sig(ps, path, depth, dtype, windows=windows, G=G)
        assert rel_err(got, want) < TOL[dtype]
        assert rel_err(grad, TO.signature_vjp(path, G, depth, None, None, windows)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth", [(8, 7), (4, 10), (4, 11), (5, 9), (6, 8), (7, 8), (12, 6)])
def test_largest_compiled_shapes(ps, dtype, d, depth):
    """Rows of 1.4 to 6.7 million coefficients, units of 120 to 1840 waves: one short path each."""
    path = brownian_path(1, 4, d, seed=700 + d) * 1.5
    want = TO.signature(path, depth)
    G = randn(tuple(want.shape), seed=701)
    got, grad = _run_sig(ps, path, depth, dtype, G=G)
    assert rel_err(got, want) < TOL[dtype]
    assert rel_err(grad, TO.signature_vjp(path, G, depth)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,B", [(4, 6, 2), (8, 4, 3), (2, 8, 70), (16, 3, 5), (3, 5, 130), (20, 2, 9)])
def test_per_word_kernels_on_shapes_that_have_a_tiled_kernel(ps, set_option, dtype, d, depth, B):
    """With the tiled kernels switched off the same dense calls run on the per-word kernels (lanes on words for few
    paths, lanes on paths for many): both families must agree with the checker, and with each other to rounding."""
    L = 12
    path = brownian_path(B, L, d, seed=900 + d)
    for windows in (None, [(0, 12), (3, 9), (4, 5), (7, 7)]):
        want = TO.compute_signature(path, depth, None, None, windows)
        G = randn(tuple(want.shape), seed=901)
        want_grad = TO.signature_vjp(path, G, depth, None, None, windows)
        results = []
        for tiled in (0, 1):
            set_option("tiled", tiled)
            got, grad = _run_sig(ps, path, depth, dtype, windows=windows, G=G)
            assert rel_err(got, want) < TOL[dtype] and rel_err(grad, want_grad) < TOL[dtype], f"tiled={tiled}"
            results.append((got, grad))
        assert rel_err(results[0][0], results[1][0]) < TOL[dtype]
        assert rel_err(results[0][1], results[1][1]) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,B,L", [(9, 4, 64, 150), (12, 4, 64, 150), (13, 4, 64, 150), (15, 4, 64, 150),
                                         (9, 5, 12, 150), (12, 5, 12, 150), (13, 5, 12, 150), (15, 5, 12, 40),
                                         (9, 6, 6, 40), (12, 6, 2, 24),
                                         (16, 4, 64, 40), (17, 4, 64, 40), (20, 4, 32, 40), (23, 4, 32, 40),
                                         (29, 4, 16, 24), (32, 4, 16, 24), (16, 5, 8, 24),
                                         (28, 3, 256, 40), (33, 3, 256, 24), (47, 3, 128, 24)])
def test_wide_alphabets_with_enough_rows_for_the_short_prefix(ps, dtype, d, depth, B, L):
    """d = 28..48 at depth 3, 9..32 at depth 4, 9..16 at depth 5 and 9..12 at depth 6 are compiled twice: lanes on prefixes of length
    depth - 2 (68 to 240 values per lane, taken in fp32 when the rows fill the device; from d = 16 on the children
    of a prefix are split between several lanes, the last of which may hold fewer: 17 = 6 + 6 + 5, 23 = 5 x 4 + 3,
    29 = 7 x 4 + 1) and of length depth - 1 (fp64 from d = 12 on, few rows).  Enough rows here for the first kind; the
    checker runs on two of them."""
    path = brownian_path(B, L, d, seed=800 + d + depth)
    x = path.to(dtype).to(DEV).requires_grad_(True)
    out = ps.Signature(depth=depth)(x)
    G = randn(tuple(out.shape), seed=801)
    (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
    idx = torch.tensor([0, B - 1])
    want = TO.signature(path[idx], depth)
    assert rel_err(out.detach().cpu()[idx], want) < TOL[dtype]
    assert rel_err(grad.cpu()[idx], TO.signature_vjp(path[idx], G[idx], depth)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("d,depth,B", [(16, 4, 40), (17, 4, 40), (32, 3, 64), (15, 5, 6)])
def test_projection_and_windows_through_split_children(ps, dtype, d, depth, B):
    """Enough rows for the variants whose lanes split the children of a prefix: dense and Lyndon-projected, with
    overlapping and degenerate windows, through the modules (forward keeps the dense signature) and through the
    stateless pair of operators (the backward sweeps again).  The checker runs on two paths."""
    L = 12
    windows = [(0, 12), (2, 9), (5, 6), (7, 7), (3, 11)]
    path = brownian_path(B, L, d, seed=820 + d) * 1.5
    idx = torch.tensor([0, B - 1])
    for proj in (None, ps.projections.lyndon(depth=depth, path_dim=d)):
        sizes, codes = _plan(proj)
        x = path.to(dtype).to(DEV).requires_grad_(True)
        win = torch.tensor(windows, dtype=torch.int64, device=DEV)
        mod = ps.Signature(depth=depth, projection=proj, windows=win)
        out = mod(x)
        G = randn(tuple(out.shape), seed=821)
        (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
        want = TO.compute_signature(path[idx], depth, sizes, codes, windows)
        want_grad = TO.signature_vjp(path[idx], G[idx], depth, sizes, codes, windows)
        assert rel_err(out.detach().cpu()[idx], want) < TOL[dtype]
        assert rel_err(grad.cpu()[idx], want_grad) < TOL[dtype]
        args = (mod.depth, mod.alternative_projection, mod._encoded_words, mod._level_sizes, mod.use_windows,
                mod._windows)
        with torch.no_grad():
            sig = torch.ops.pathsig.compute_signature(x, *args)
            g2 = torch.ops.pathsig.signature_backward(x, sig, G.to(dtype).to(DEV), *args)
        assert torch.equal(sig, out.detach())
        assert rel_err(g2.cpu()[idx], want_grad) < TOL[dtype]


@pytest.mark.parametrize("d,depth,windows", [(2, 12, None), (3, 10, [(0, 8), (2, 7), (3, 4)]), (4, 9, None)])
def test_deep_fp32_backward_runs_in_fp64_unless_switched_off(ps, set_option, d, depth, windows):
    """Option "deep_fp64": from depth 9 on an fp32 backward sweeps in fp64 and holds 1e-5 over increments of size
    one; switched off it is the plain fp32 sweep, within the 1e-4 the reference's own suite allows there
    (`tests/test_sig.py:26-34`), and the two differ."""
    path = brownian_path(2, 8, d, seed=900 + d) * 2.0
    want = TO.compute_signature(path, depth, None, None, windows)
    G = randn(tuple(want.shape), seed=901)
    want_grad = TO.signature_vjp(path, G, depth, None, None, windows)
    grads = {}
    for on in (1, 0):
        set_option("deep_fp64", on)
        got, grads[on] = _run_sig(ps, path, depth, torch.float32, windows=windows, G=G)
        assert rel_err(got, want) < TOL[torch.float32]
    assert rel_err(grads[1], want_grad) < TOL[torch.float32]
    assert rel_err(grads[0], want_grad) < 1e-4
    assert not torch.equal(grads[0], grads[1])


@pytest.mark.parametrize("d,depth,B", [(100, 3, 2), (8, 8, 1), (8, 8, 16)])
def test_fp32_gradient_on_dense_levels_of_a_million_words(ps, d, depth, B):
    """Shapes without a tiled kernel whose top level has 10^6 to 10^7 words: the per-word kernels add one term per
    block of words to every (increment, letter) cell, tens of thousands of terms of mixed sign.  Summed in fp64 the
    fp32 gradient stays within 5e-6 of the fp64 one (in fp32 it was off by up to 3.5e-5)."""
    path = brownian_path(B, 6 if depth == 8 else 10, d, seed=2000)
    res = {}
    for dtype in (torch.float64, torch.float32):
        x = path.to(dtype).to(DEV).requires_grad_(True)
        out = ps.Signature(depth=depth)(x)
        G = randn(tuple(out.shape), seed=3)
        (g,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
        res[dtype] = (out.detach().cpu().double(), g.cpu().double())
    assert rel_err(res[torch.float32][0], res[torch.float64][0]) < 1e-6
    assert rel_err(res[torch.float32][1], res[torch.float64][1]) < 5e-6
