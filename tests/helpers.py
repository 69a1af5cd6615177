"""Shared input builders for the tests (seeded on the CPU so the checker and the GPU see the same bits)."""
from __future__ import annotations

import itertools
import math
import random

import torch


def brownian_path(B, L, d, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    dx = torch.randn(B, L - 1, d, dtype=torch.float64, generator=g) / math.sqrt(L)
    x = torch.cat([torch.zeros(B, 1, d, dtype=torch.float64), torch.cumsum(dx, dim=1)], dim=1)
    return x.to(dtype)


def randn(shape, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, dtype=torch.float64, generator=g).to(dtype)


def rel_err(a, b):
    """max|a-b| / max(1, max|b|): the parity metric of the reference tests (`tests/test_sig.py:88-91`)."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / max(1.0, float(b.abs().max())))


def strict_rel_err(a, b):
    """max|a-b| / max|b| (no floor of 1 in the denominator: small quantities are held to the same relative bound)."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    scale = float(b.abs().max())
    return float((a - b).abs().max() / scale) if scale > 0 else float((a - b).abs().max())


def level_rel_errs(got, want, level_sizes):
    """Per level k: max|got_k - want_k| / max|want_k| over the columns of that level (the last axis holds the levels
    one after the other with the given sizes).  The global metric divides by the largest coefficient of all, which
    on Brownian inputs sits in level 1 or 2 and hides the high levels, whose coefficients are 1e-3 .. 1e-6."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    errs, off = [], 0
    for size in level_sizes:
        if size > 0:
            errs.append(strict_rel_err(got[..., off:off + size], want[..., off:off + size]))
        off += size
    assert off == want.shape[-1]
    return errs


def all_words(d, n):
    return list(itertools.product(range(d), repeat=n))


def code_of(word, d):
    c = 0
    for a in word:
        c = c * d + a
    return c


def random_word_set(d, lo, hi, count, seed):
    """`count` distinct words with lengths uniform in lo..hi, stably sorted by length."""
    rng = random.Random(seed)
    seen, words = set(), []
    while len(words) < count:
        n = rng.randint(lo, hi)
        w = tuple(rng.randrange(d) for _ in range(n))
        if w in seen:
            continue
        seen.add(w)
        words.append(w)
    words.sort(key=len)
    return words
