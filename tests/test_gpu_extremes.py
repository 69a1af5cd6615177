"""Sizes at the edges of what the launches assume: very long paths, very many rows, more (path group, window) pairs
than a grid's second dimension holds, tens of thousands of listed words.  fp64 against the checker on a subset of
the batch, fp32 against fp64."""
from __future__ import annotations

import random

import pytest
import torch

from oracle import tensor_oracle as TO
from tests.helpers import brownian_path, randn, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ps():
    import pathsig_amd
    return pathsig_amd


def _run(ps, x, depth, proj, windows, dtype, G=None):
    xg = x.to(dtype).to(DEV).requires_grad_(True)
    win = None if windows is None else torch.tensor(windows, dtype=torch.int64, device=DEV)
    out = ps.Signature(depth=depth, projection=proj, windows=win)(xg)
    if G is None:
        G = randn(tuple(out.shape), seed=5)
    (grad,) = torch.autograd.grad(out, xg, G.to(dtype).to(DEV))
    return out.detach().cpu(), grad.cpu(), G


def _check(ps, d, depth, B, L, proj=None, windows=None, subset=2):
    x = brownian_path(B, L, d, seed=7)
    o64, g64, G = _run(ps, x, depth, proj, windows, torch.float64)
    o32, g32, _ = _run(ps, x, depth, proj, windows, torch.float32, G)
    assert rel_err(o32, o64) < 1e-5 and rel_err(g32, g64) < 1e-5
    idx = torch.linspace(0, B - 1, subset).long().unique()
    sizes, codes = (None, None) if proj is None else (proj.level_sizes, proj._codes)
    want = TO.compute_signature(x[idx], depth, sizes, codes, windows)
    want_grad = TO.signature_vjp(x[idx], G[idx].double(), depth, sizes, codes, windows)
    assert rel_err(o64[idx], want) < 1e-12 and rel_err(g64[idx], want_grad) < 1e-12


@pytest.mark.parametrize("d,depth,L", [(3, 3, 20001), (70, 2, 6001)])
def test_very_long_path(ps, d, depth, L):
    """One path of thousands of increments: tiled shape cut into time chunks, and the per-word kernels."""
    _check(ps, d, depth, 1, L, subset=1)


@pytest.mark.parametrize("d,depth,B,L", [(4, 3, 70000, 3), (2, 2, 300000, 2), (66, 2, 20000, 3)])
def test_very_many_rows(ps, d, depth, B, L):
    _check(ps, d, depth, B, L, subset=3)


def test_more_group_window_pairs_than_a_grid_dimension(ps):
    """2200 paths are 138 groups of sixteen lanes; with 600 windows that is more than the 65535 blocks that the
    second grid dimension of the lanes-on-paths backward can hold: the call must take another kernel, not fail."""
    few = ps.projections.words([(1,), (7,), (5, 60), (65, 0), (3, 3)], depth=2, path_dim=66)
    wins = [(i, i + 5) for i in range(600)]
    _check(ps, 66, 2, 2200, 700, proj=few, windows=wins)


@pytest.mark.parametrize("B", [4, 40])
def test_tens_of_thousands_of_words(ps, B):
    rng = random.Random(3)
    words = sorted({tuple(rng.randrange(66) for _ in range(rng.randint(1, 3))) for _ in range(60000)}, key=len)
    proj = ps.projections.words(words, depth=3, path_dim=66)
    _check(ps, 66, 3, B, 20, proj=proj, subset=1)
