"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py with the fp64
level-tensor checker) against the per-word C restatement, the planner, and -- on a GPU -- the kernels."""
from __future__ import annotations

import pathlib

import numpy as np
import pytest
import torch

from oracle import tensor_oracle as TO
from oracle import words_oracle as WO
from tests.helpers import level_rel_errs, rel_err

GOLD = pathlib.Path(__file__).resolve().parent / "golden"


def load(name):
    z = np.load(GOLD / f"{name}.npz", allow_pickle=False)
    return {k: (torch.from_numpy(z[k]) if z[k].ndim else int(z[k])) for k in z.files}


def test_words_oracle_reproduces_fixtures():
    f = load("c1_small")
    assert rel_err(WO.sig_forward(f["path"], f["depth"]), f["sig"]) < 1e-13
    f = load("c2_small")
    sig = WO.sig_forward(f["path"], f["depth"])
    assert rel_err(sig, f["sig"]) < 1e-13
    assert rel_err(WO.sig_backward(f["path"], sig, f["grad_out"], f["depth"]), f["grad_path"]) < 1e-12
    f = load("c3_small")
    wins = f["windows"].tolist()
    sig = WO.sig_forward(f["path"], f["depth"], windows=wins)
    assert rel_err(sig, f["sig"]) < 1e-13
    assert rel_err(WO.sig_backward(f["path"], sig, f["grad_out"], f["depth"], windows=wins), f["grad_path"]) < 1e-12
    f = load("c4_small")
    ls, codes = f["level_sizes"].tolist(), f["codes"].tolist()
    sig = WO.sig_forward(f["path"], f["depth"], ls, codes)
    assert rel_err(sig, f["sig"]) < 1e-13
    assert rel_err(WO.sig_backward(f["path"], sig, f["grad_out"], f["depth"], ls, codes), f["grad_path"]) < 1e-12


def test_words_oracle_logsig_reproduces_fixture():
    f = load("c5_small")
    d, depth = 4, f["depth"]
    ls, codes = f["level_sizes"].tolist(), f["codes"].tolist()
    skipped = sum(ls[k] for k in range(1, depth) if ls[k] != d ** k)
    top_codes, top = codes[skipped:], ls[depth]
    hyb_sizes = [0] + [d ** k for k in range(1, depth)] + [top]
    sig = WO.sig_forward(f["path"], depth, hyb_sizes, top_codes)
    logsig, P = WO.logsig_forward(sig, depth, d, top, top_codes)
    # pick the projection's coordinates out of the hybrid layout
    from pathsig_amd.projections import projections
    proj = projections.lyndon(depth=depth, path_dim=d)
    assert proj.level_sizes == ls and proj._codes == codes
    idx = torch.tensor(proj._logsig_index_list())
    assert rel_err(logsig[:, idx], f["logsig"]) < 1e-13
    g_hyb = torch.zeros_like(sig).index_add_(1, idx, f["grad_out"])
    g_sig = WO.logsig_backward(sig, P, g_hyb, depth, d, top, top_codes)
    g_path = WO.sig_backward(f["path"], sig, g_sig, depth, hyb_sizes, top_codes)
    assert rel_err(g_path, f["grad_path"]) < 1e-12


def test_planner_reproduces_lyndon_fixtures():
    from pathsig_amd.projections import projections
    f = load("lyndon_plans")
    for d, n in [(2, 6), (3, 5), (4, 4), (8, 5)]:
        p = projections.lyndon(depth=n, path_dim=d)
        assert p.level_sizes == f[f"sizes_{d}_{n}"].tolist()
        assert p._codes == f[f"codes_{d}_{n}"].tolist()
        assert p._logsig_index_list() == f[f"logsig_idx_{d}_{n}"].tolist()
    # the sizes the benchmark definition states for d = 8, depth 5
    assert f["sizes_8_5"].tolist() == [0, 8, 28, 168, 1008, 6552]


def test_fixture_c4_word_list_matches_codes():
    from pathsig_amd.projections import projections
    f = load("c4_small")
    flat, lens = f["words_flat"].tolist(), f["word_lengths"].tolist()
    words, pos = [], 0
    for n in lens:
        words.append(tuple(flat[pos:pos + n]))
        pos += n
    p = projections.words(words, depth=f["depth"], path_dim=16, full_levels=(1, 2))
    assert p.level_sizes == f["level_sizes"].tolist() and p._codes == f["codes"].tolist()


# ------------------------------------------------------------------------------------------------
# GPU: the kernels against the same fixtures (fp64 1e-12, fp32 1e-5 of the build target)
# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-12), (torch.float32, 1e-5)])
def test_kernels_reproduce_fixtures(dtype, tol):
    import pathsig_amd as ps
    dev = "cuda"
    gtol = tol * (10 if dtype == torch.float32 else 1)

    def levels_ok(out, want, sizes):
        # every level relative to its own largest coefficient (twice the global bound)
        errs = level_rel_errs(out, want, sizes)
        assert max(errs) < 2 * tol, errs

    def dense_sizes(f):
        return [f["path"].shape[2] ** k for k in range(1, f["depth"] + 1)]

    def run(mod, f):
        x = f["path"].to(dtype).to(dev).requires_grad_("grad_out" in f)
        out = mod(x)
        grad = None
        if "grad_out" in f:
            (grad,) = torch.autograd.grad(out, x, f["grad_out"].to(dtype).to(dev))
        return out.detach(), grad

    f = load("c1_small")
    out, _ = run(ps.Signature(depth=f["depth"]), f)
    assert rel_err(out, f["sig"]) < tol
    levels_ok(out, f["sig"], dense_sizes(f))
    f = load("c2_small")
    out, grad = run(ps.Signature(depth=f["depth"]), f)
    assert rel_err(out, f["sig"]) < tol and rel_err(grad, f["grad_path"]) < gtol
    levels_ok(out, f["sig"], dense_sizes(f))
    f = load("c3_small")
    out, grad = run(ps.Signature(depth=f["depth"], windows=f["windows"].to(dev)), f)
    assert rel_err(out, f["sig"]) < tol and rel_err(grad, f["grad_path"]) < gtol
    levels_ok(out, f["sig"], dense_sizes(f))
    f = load("c4_small")
    flat, lens = f["words_flat"].tolist(), f["word_lengths"].tolist()
    words, pos = [], 0
    for n in lens:
        words.append(tuple(flat[pos:pos + n]))
        pos += n
    proj = ps.projections.words(words, depth=f["depth"], path_dim=16, full_levels=(1, 2))
    out, grad = run(ps.Signature(depth=f["depth"], projection=proj), f)
    assert rel_err(out, f["sig"]) < tol and rel_err(grad, f["grad_path"]) < gtol
    levels_ok(out, f["sig"], proj.level_sizes[1:])
    f = load("c5_small")
    proj = ps.projections.lyndon(depth=f["depth"], path_dim=4)
    out, grad = run(ps.LogSignature(depth=f["depth"], projection=proj), f)
    assert rel_err(out, f["logsig"]) < tol and rel_err(grad, f["grad_path"]) < gtol
