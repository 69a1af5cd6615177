"""Writes the committed fixtures tests/golden/*.npz with OUR OWN CPU checker (oracle/tensor_oracle.py, fp64).

The reference holds no stored vectors (its tests compare against third-party packages that are not
available here), so these fixtures pin regressions of the checker and of the kernels against each other;
the checker itself is pinned to mathematics in tests/test_oracle_math.py.  Reduced-size versions of the
five benchmark configurations, generated with the same seeding rule as the benchmark
(increments seed 1000+i, upstream gradient seed 2000+i).

    python tests/golden/make_fixtures.py
"""
from __future__ import annotations

import math
import pathlib
import sys

import numpy as np
import torch

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import tensor_oracle as TO  # noqa: E402
from pathsig_amd.projections import projections  # noqa: E402
from tests.helpers import random_word_set  # noqa: E402

HERE = pathlib.Path(__file__).resolve().parent


def brownian(B, L, d, seed):
    g = torch.Generator().manual_seed(seed)
    dx = torch.randn(B, L - 1, d, dtype=torch.float64, generator=g) / math.sqrt(L)
    return torch.cat([torch.zeros(B, 1, d, dtype=torch.float64), torch.cumsum(dx, dim=1)], dim=1)


def upstream(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, dtype=torch.float64, generator=g)


def save(name, **arrays):
    np.savez_compressed(HERE / f"{name}.npz", **{k: np.asarray(v) for k, v in arrays.items()})
    print("wrote", name, {k: np.asarray(v).shape for k, v in arrays.items()})


def main():
    # c1-like: depth 4, d = 8, forward only
    x = brownian(3, 24, 8, 1001)
    save("c1_small", path=x.numpy(), depth=4, sig=TO.signature(x, 4).numpy())

    # c2-like: depth 6, d = 4, forward + backward
    x = brownian(3, 40, 4, 1002)
    sig = TO.signature(x, 6)
    G = upstream(sig.shape, 2002)
    save("c2_small", path=x.numpy(), depth=6, sig=sig.numpy(), grad_out=G.numpy(),
         grad_path=TO.signature_vjp(x, G, 6).numpy())

    # c3-like: windows of 16 points with stride 8, depth 5, d = 6
    x = brownian(1, 48, 6, 1003)
    wins = [[8 * i, 8 * i + 16] for i in range(5)]
    sig = TO.compute_signature(x, 5, windows=wins)
    G = upstream(sig.shape, 2003)
    save("c3_small", path=x.numpy(), depth=5, windows=np.array(wins, dtype=np.int64), sig=sig.numpy(),
         grad_out=G.numpy(), grad_path=TO.signature_vjp(x, G, 5, windows=wins).numpy())

    # c4-like: d = 16, depth 4 (dense depth 6 does not fit a CPU checker), levels 1-2 full + 200 words of length 3..4
    words = random_word_set(16, 3, 4, 200, seed=20240)
    proj = projections.words(words, depth=4, path_dim=16, full_levels=(1, 2))
    x = brownian(2, 20, 16, 1004)
    sig = TO.compute_signature(x, 4, proj.level_sizes, proj._codes)
    G = upstream(sig.shape, 2004)
    save("c4_small", path=x.numpy(), depth=4, level_sizes=np.array(proj.level_sizes, dtype=np.int64),
         codes=np.array(proj._codes, dtype=np.int64), words_flat=np.array([a for w in words for a in w]),
         word_lengths=np.array([len(w) for w in words]), sig=sig.numpy(), grad_out=G.numpy(),
         grad_path=TO.signature_vjp(x, G, 4, proj.level_sizes, proj._codes).numpy())

    # c5-like: log-signature with Lyndon projection, d = 4, depth 5
    proj = projections.lyndon(depth=5, path_dim=4)
    x = brownian(2, 30, 4, 1005)
    cols = torch.tensor(TO.projection_columns(4, 5, proj.level_sizes, proj._codes))
    xr = x.clone().requires_grad_(True)
    out = TO.logsignature(xr, 5).index_select(-1, cols)
    G = upstream(out.shape, 2005)
    (g,) = torch.autograd.grad(out, xr, G)
    save("c5_small", path=x.numpy(), depth=5, level_sizes=np.array(proj.level_sizes, dtype=np.int64),
         codes=np.array(proj._codes, dtype=np.int64), logsig=out.detach().numpy(), grad_out=G.numpy(),
         grad_path=g.numpy())

    # planner outputs: Lyndon code lists and the benchmark's word set for config 4
    lyn = {}
    for d, n in [(2, 6), (3, 5), (4, 4), (8, 5)]:
        p = projections.lyndon(depth=n, path_dim=d)
        lyn[f"sizes_{d}_{n}"] = np.array(p.level_sizes, dtype=np.int64)
        lyn[f"codes_{d}_{n}"] = np.array(p._codes, dtype=np.int64)
        lyn[f"logsig_idx_{d}_{n}"] = np.array(p._logsig_index_list(), dtype=np.int64)
    save("lyndon_plans", **lyn)


if __name__ == "__main__":
    main()
