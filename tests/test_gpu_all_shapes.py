"""Every shape that has a register-tiled kernel, both dtypes.

* against the per-word kernels on the same call (option "tiled" = 0; the two families share no code below the
  entry points), with few rows and with many rows (a shape compiled twice takes a different variant then) and
  random windows;
* against the CPU checker (`oracle.tensor_oracle`, fp64) on a tiny case per shape, and for the shapes that are
  compiled twice also on a batch large enough for the variant with the shorter prefix, checked on three of its rows
  (rows are independent);
* the widest alphabets of the reference's own sweep, (65, 3) and (100, 3) at L = 10
  (`tests/test_sig.py:145-152`), against the CPU checker."""
from __future__ import annotations

import random

import pytest
import torch

from oracle import tensor_oracle as TO
from tests.helpers import brownian_path, randn, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _compiled_shapes():
    shapes = [(d, n) for d in range(2, 9) for n in range(2, 8)]
    shapes += [(d, n) for d in range(9, 13) for n in range(2, 7)] + [(d, n) for d in range(13, 17) for n in range(2, 6)]
    shapes += [(d, n) for d in range(17, 33) for n in range(2, 5)] + [(d, n) for d in range(33, 65) for n in (2, 3)]
    shapes += [(72, 3), (80, 3), (88, 3), (96, 3), (104, 3), (112, 3)]
    shapes += [(2, 8), (2, 9), (2, 10), (2, 11), (2, 12), (3, 8), (3, 9), (3, 10), (3, 11), (3, 12), (4, 8), (4, 9), (4, 10),
               (4, 11), (5, 8), (5, 9), (6, 8), (7, 8)]
    return shapes


@pytest.mark.parametrize("part", range(8))
def test_tiled_and_per_word_kernels_agree_on_every_compiled_shape(set_option, part):
    import pathsig_amd as ps
    shapes = _compiled_shapes()
    assert len(shapes) == 214
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


def _first_variant_rows(d, n):
    """Rows from which a shape that is compiled twice runs on its first entry (the shorter prefix), for paths of
    fewer than 33 points; None for a shape compiled once.  Follows the table of compiled shapes and the row rule of
    `dense_choice` in `pathsig_amd/csrc/dense_kernels.hip` (a wave for every SIMD: rows x waves per row >= 1024)."""
    short_prefix = None
    if n == 4 and 8 <= d <= 32:
        short_prefix = 2
    elif n == 5 and 9 <= d <= 16:
        short_prefix = 3
    elif n == 6 and 9 <= d <= 12:
        short_prefix = 4
    elif n == 3 and 28 <= d <= 48:
        short_prefix = 1
    if short_prefix is None:
        return None
    waves = min(16, -(-d ** short_prefix // 64))
    return -(-1024 // waves)


def _against_oracle(ps, d, n, B, L, seed, rows, what):
    path = brownian_path(B, L, d, seed=seed)
    for dtype, tol in ((torch.float32, 1e-5), (torch.float64, 1e-12)):
        x = path.to(dtype).to(DEV).requires_grad_(True)
        out = ps.Signature(depth=n)(x)
        gen = torch.Generator(device=DEV).manual_seed(seed + 1)
        G = torch.randn(out.shape, dtype=dtype, device=DEV, generator=gen)
        (grad,) = torch.autograd.grad(out, x, G)
        index = torch.tensor(rows, device=DEV)
        # the checker sees the rounded inputs of the call, in fp64
        sub = path.to(dtype).double()[rows]
        want = TO.signature(sub, n)
        assert rel_err(out.detach()[index], want) < tol, f"{what} {dtype} signature"
        want_grad = TO.signature_vjp(sub, G[index].double().cpu(), n)
        assert rel_err(grad[index], want_grad) < tol, f"{what} {dtype} gradient"
        del out, G, grad, x


@pytest.mark.parametrize("part", range(8))
def test_every_compiled_shape_against_the_oracle(part):
    import pathsig_amd as ps
    shapes = _compiled_shapes()
    rng = random.Random(300 + part)
    for d, n in shapes[part::8]:
        B, L = rng.choice([1, 2]), rng.choice([2, 3, 4])
        _against_oracle(ps, d, n, B, L, rng.randint(0, 10 ** 6), list(range(B)), f"d={d} depth={n} B={B} L={L}")
        many = _first_variant_rows(d, n)
        if many is not None:
            B = many + rng.randint(0, 3)
            _against_oracle(ps, d, n, B, 3, rng.randint(0, 10 ** 6), [0, B // 2, B - 1],
                            f"d={d} depth={n} B={B} L=3 (rows 0, {B // 2}, {B - 1})")
            torch.cuda.empty_cache()


@pytest.mark.parametrize("d", [65, 79, 81, 100, 111])
def test_widest_alphabets_of_the_reference_sweep_against_the_oracle(d):
    """Alphabets between the compiled sizes 64, 72, 80, .. 112 run as the next compiled size on a path with constant
    extra coordinates."""
    import pathsig_amd as ps
    _against_oracle(ps, d, 3, 2, 10, 77 + d, [0, 1], f"d={d} depth=3 B=2 L=10")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_padded_wide_alphabet_with_windows_and_both_kernel_families(set_option, dtype):
    import pathsig_amd as ps
    d, B, L = 70, 3, 12
    path = brownian_path(B, L, d, seed=41)
    windows = [(0, 12), (2, 9), (5, 6), (7, 7)]
    want = TO.compute_signature(path, 3, None, None, windows)
    G = randn(tuple(want.shape), seed=42)
    want_grad = TO.signature_vjp(path, G, 3, None, None, windows)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    win = torch.tensor(windows, dtype=torch.int64, device=DEV)
    for tiled in (1, 0):
        set_option("tiled", tiled)
        x = path.to(dtype).to(DEV).requires_grad_(True)
        out = ps.Signature(depth=3, windows=win)(x)
        (grad,) = torch.autograd.grad(out, x, G.to(dtype).to(DEV))
        assert rel_err(out, want) < tol and rel_err(grad, want_grad) < tol, tiled
