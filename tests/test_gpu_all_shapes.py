"""Every shape that has a register-tiled kernel, with few rows and with many rows (a shape compiled twice takes a
different variant then), random windows, both dtypes: the tiled kernels against the per-word kernels on the same
call (option "tiled" = 0).  The two families share no code below the entry points."""
from __future__ import annotations

import random

import pytest
import torch

from tests.helpers import brownian_path, randn, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _compiled_shapes():
    shapes = [(d, n) for d in range(2, 9) for n in range(2, 8)]
    shapes += [(d, n) for d in range(9, 13) for n in range(2, 7)] + [(d, n) for d in range(13, 17) for n in range(2, 6)]
    shapes += [(d, n) for d in range(17, 33) for n in range(2, 5)] + [(d, n) for d in range(33, 65) for n in (2, 3)]
    shapes += [(2, 8), (2, 9), (2, 10), (2, 11), (2, 12), (3, 8), (3, 9), (3, 10), (3, 11), (3, 12), (4, 8), (4, 9), (4, 10),
               (4, 11), (5, 8), (5, 9), (6, 8), (7, 8)]
    return shapes


@pytest.mark.parametrize("part", range(8))
def test_tiled_and_per_word_kernels_agree_on_every_compiled_shape(set_option, part):
    import pathsig_amd as ps
    shapes = _compiled_shapes()
    assert len(shapes) == 208
    rng = random.Random(100 + part)
    for d, n in shapes[part::8]:
        size = sum(d ** k for k in range(1, n + 1))
        for many in (False, True):
            if many and size > 1200000:
                continue
            B = rng.choice([1, 2, 3]) if not many else max(4, min(600, int(3e7 / size / 8)))
            L = rng.choice([2, 3, 6, 11]) if size > 100000 else rng.choice([2, 5, 19, 40])
            windows = None
            if rng.random() < 0.5 and size * B < 2e6:
                starts = [rng.randint(0, L - 1) for _ in range(rng.randint(1, 3))]
                windows = [(s, rng.randint(s, L)) for s in starts]
            for dtype in (torch.float32, torch.float64):
                path = brownian_path(B, L, d, seed=rng.randint(0, 10 ** 6))
                win = None if windows is None else torch.tensor(windows, dtype=torch.int64, device=DEV)
                results, G = [], None
                for tiled in (1, 0):
                    set_option("tiled", tiled)
                    x = path.to(dtype).to(DEV).requires_grad_(True)
                    out = ps.Signature(depth=n, windows=win)(x)
                    if G is None:
                        G = randn(tuple(out.shape), seed=3).to(dtype).to(DEV)
                    (grad,) = torch.autograd.grad(out, x, G)
                    results.append((out.detach().cpu(), grad.cpu()))
                tol = 2e-5 if dtype == torch.float32 else 1e-11
                what = f"d={d} depth={n} B={B} L={L} {dtype} windows={windows}"
                assert rel_err(results[0][0], results[1][0]) < tol, what
                assert rel_err(results[0][1], results[1][1]) < tol, what
