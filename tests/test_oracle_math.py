"""Pins the CPU checkers (oracle/tensor_oracle.py and the per-word C restatement oracle/ref_words.c)
to facts that do not depend on either of them: closed forms, brute-force iterated sums, algebraic
identities of the signature, finite differences.  A dropped term, a wrong factorial, a transposed
tensor product or a wrong word index fails at least one of these."""
from __future__ import annotations

import itertools
import math

import pytest
import torch

from oracle import tensor_oracle as TO
from oracle import words_oracle as WO
from tests.helpers import all_words, brownian_path, code_of, randn, random_word_set

torch.set_default_dtype(torch.float64)


def sig_by_iterated_sums(path, depth):
    """Definition of the signature of a piecewise-linear path, written without any recurrence:
    S(w) = sum over non-decreasing segment choices t_1<=...<=t_n of prod dx_{t_j}[w_j] / prod (run length)!"""
    L, d = path.shape
    dx = (path[1:] - path[:-1]).tolist()
    out = {}
    for n in range(1, depth + 1):
        for w in all_words(d, n):
            tot = 0.0
            for ts in itertools.combinations_with_replacement(range(L - 1), n):
                term = 1.0
                for j, t in enumerate(ts):
                    term *= dx[t][w[j]]
                runs = [len(list(g)) for _, g in itertools.groupby(ts)]
                for r in runs:
                    term /= math.factorial(r)
                tot += term
            out[w] = tot
    return out


def as_dict(flat, d, depth):
    offs = TO.dense_level_offsets(d, depth)
    return {w: float(flat[offs[n] + code_of(w, d)]) for n in range(1, depth + 1) for w in all_words(d, n)}


def shuffles(u, v):
    if not u:
        return [tuple(v)]
    if not v:
        return [tuple(u)]
    return [(u[0],) + s for s in shuffles(u[1:], v)] + [(v[0],) + s for s in shuffles(u, v[1:])]


BOTH = [("tensor", lambda p, n: TO.signature(p, n)), ("words", lambda p, n: WO.sig_forward(p, n))]


@pytest.mark.parametrize("name,fn", BOTH)
def test_single_segment_is_tensor_exponential(name, fn):
    d, depth = 3, 5
    path = torch.zeros(1, 2, d)
    v = torch.tensor([0.7, -1.3, 0.4])
    path[0, 0] = torch.tensor([0.2, 0.1, -0.5])
    path[0, 1] = path[0, 0] + v
    got = as_dict(fn(path, depth)[0], d, depth)
    for w, val in got.items():
        want = math.prod(float(v[a]) for a in w) / math.factorial(len(w))
        assert abs(val - want) < 1e-15 * max(1, abs(want)) + 1e-16


@pytest.mark.parametrize("name,fn", BOTH)
def test_matches_iterated_sums(name, fn):
    d, depth, L = 2, 4, 5
    path = randn((1, L, d), seed=3)
    want = sig_by_iterated_sums(path[0], depth)
    got = as_dict(fn(path, depth)[0], d, depth)
    for w in want:
        assert abs(got[w] - want[w]) < 1e-13, w


@pytest.mark.parametrize("name,fn", BOTH)
def test_matches_iterated_sums_three_letters(name, fn):
    d, depth, L = 3, 3, 4
    path = randn((1, L, d), seed=4)
    want = sig_by_iterated_sums(path[0], depth)
    got = as_dict(fn(path, depth)[0], d, depth)
    for w in want:
        assert abs(got[w] - want[w]) < 1e-13, w


@pytest.mark.parametrize("name,fn", BOTH)
def test_chen_identity(name, fn):
    d, depth, L = 3, 4, 9
    path = randn((2, L, d), seed=5)
    whole = fn(path, depth)
    for m in (1, 4, 7):
        left = TO.split_levels(fn(path[:, :m + 1], depth), d, depth)
        right = TO.split_levels(fn(path[:, m:], depth), d, depth)
        prod = torch.cat(TO.tensor_product_levels(left, right, depth), dim=-1)
        assert (prod - whole).abs().max() < 1e-13


@pytest.mark.parametrize("name,fn", BOTH)
def test_shuffle_identity_and_level_one(name, fn):
    d, depth, L = 3, 4, 8
    path = randn((1, L, d), seed=6)
    S = as_dict(fn(path, depth)[0], d, depth)
    for a in range(d):
        assert abs(S[(a,)] - float(path[0, -1, a] - path[0, 0, a])) < 1e-14
    for u, v in [((0,), (1,)), ((0, 1), (2,)), ((2, 0), (1, 1)), ((0,), (0, 0, 1)), ((1,), (1,))]:
        lhs = S[u] * S[v]
        rhs = sum(S[w] for w in shuffles(u, v))
        assert abs(lhs - rhs) < 1e-13, (u, v)


@pytest.mark.parametrize("name,fn", BOTH)
def test_invariances(name, fn):
    d, depth, L = 2, 5, 7
    path = randn((1, L, d), seed=7)
    base = fn(path, depth)
    assert (fn(path + 3.25, depth) - base).abs().max() < 1e-13  # translation
    doubled = path.repeat_interleave(2, dim=1)  # repeated points add zero increments
    assert (fn(doubled, depth) - base).abs().max() < 1e-13
    rev = fn(path.flip(1), depth)  # time reversal gives the tensor inverse
    one = TO.tensor_product_levels(TO.split_levels(base, d, depth), TO.split_levels(rev, d, depth), depth)
    assert torch.cat(one, dim=-1).abs().max() < 1e-13


def test_projection_layout_is_gather_of_dense():
    d, depth = 3, 4
    path = randn((2, 6, d), seed=8)
    dense = TO.signature(path, depth)
    words = random_word_set(d, 1, 4, 25, seed=1)
    sizes = [0] * (depth + 1)
    codes = []
    for w in words:
        sizes[len(w)] += 1
        codes.append(code_of(w, d))
    sizes[2] = d ** 2  # also exercise a full level in the middle
    codes = [c for c, w in zip(codes, words) if len(w) != 2]
    offs = TO.dense_level_offsets(d, depth)
    want_cols = []
    it = iter(codes)
    for k in range(1, depth + 1):
        if sizes[k] == d ** k:
            want_cols += [offs[k] + c for c in range(d ** k)]
        else:
            want_cols += [offs[k] + next(it) for _ in range(sizes[k])]
    want = dense[:, want_cols]
    assert torch.equal(TO.compute_signature(path, depth, sizes, codes), want)
    got = WO.sig_forward(path, depth, sizes, codes)
    assert (got - want).abs().max() < 1e-14


def test_windows_are_slices():
    d, depth = 2, 4
    path = randn((3, 12, d), seed=9)
    wins = [(0, 12), (3, 5), (2, 9), (5, 12), (4, 6), (1, 4)]
    got_t = TO.compute_signature(path, depth, windows=wins)
    got_w = WO.sig_forward(path, depth, windows=wins)
    for i, (s, e) in enumerate(wins):
        want = TO.signature(path[:, s:e], depth)
        assert torch.equal(got_t[:, i], want)
        assert (got_w[:, i] - want).abs().max() < 1e-14


# ------------------------------------------------------------------------------------------------
# log-signature
# ------------------------------------------------------------------------------------------------
def tensor_exp_levels(X, depth):
    """exp(X) = sum X^(x)k / k! for X without a level-0 term (independent of the log code)."""
    out = [x.clone() for x in X]
    power = [x.clone() for x in X]
    for k in range(2, depth + 1):
        power = TO.tensor_product_levels(power, X, depth, a0=0.0, b0=0.0)
        out = [o + p / math.factorial(k) for o, p in zip(out, power)]
    return out


def test_log_then_exp_is_identity():
    d, depth = 3, 5
    S = TO.split_levels(TO.signature(randn((2, 7, d), seed=10), depth), d, depth)
    back = tensor_exp_levels(TO.tensor_log_levels(S, depth), depth)
    for a, b in zip(S, back):
        assert (a - b).abs().max() < 1e-13


def test_inverse_exp_log_is_the_same_function():
    """`tensor_log_levels_inverse_exp`: exp of it is S (independent exponential), it equals the alternating series
    on a well-conditioned input, and on an ill-conditioned one (powers of S - 1 up to 1e6) it is the series
    summed in extended precision that it agrees with, not the series summed in fp64."""
    import numpy as np

    d, depth = 3, 5
    S = TO.split_levels(TO.signature(randn((2, 7, d), seed=10), depth), d, depth)
    L = TO.tensor_log_levels_inverse_exp(S, depth)
    for a, b in zip(S, tensor_exp_levels(L, depth)):
        assert (a - b).abs().max() < 1e-13
    for a, b in zip(L, TO.tensor_log_levels(S, depth)):
        assert (a - b).abs().max() < 1e-13

    d, depth = 2, 8
    sig = TO.signature(brownian_path(2, 130, d, seed=5) * 2.0, depth)
    S = TO.split_levels(sig, d, depth)
    series = torch.cat(TO.tensor_log_levels(S, depth), dim=-1)
    inverse = torch.cat(TO.tensor_log_levels_inverse_exp(S, depth), dim=-1)
    # the alternating series in x87 extended precision (64-bit mantissa), level tensors as numpy arrays
    ld = np.longdouble
    if np.finfo(ld).eps > 1e-18:
        pytest.skip("no extended precision on this platform")
    Sn = [x.numpy().astype(ld) for x in S]
    powers = [list(Sn)]
    for m in range(2, depth + 1):
        prev, cur = powers[-1], []
        for n in range(1, depth + 1):
            acc = np.zeros_like(Sn[n - 1])
            for k in range(m - 1, n):
                acc = acc + (prev[k - 1][:, :, None] * Sn[n - k - 1][:, None, :]).reshape(acc.shape[0], -1)
            cur.append(acc)
        powers.append(cur)
    exact = np.concatenate([sum(ld((-1.0) ** (m + 1)) / ld(m) * powers[m - 1][n - 1] for m in range(1, n + 1))
                            for n in range(1, depth + 1)], axis=1).astype(np.float64)
    scale = max(1.0, float(np.abs(exact).max()))
    assert max(float(np.abs(p).max()) for pw in powers for p in pw) > 1e5      # the input is ill conditioned
    err_inverse = np.abs(inverse.numpy() - exact).max() / scale
    err_series = np.abs(series.numpy() - exact).max() / scale
    assert err_inverse < 1e-13
    assert err_series > 10 * err_inverse and err_series > 5e-13                # the fp64 series is the one off


def test_log_closed_forms_and_lie_property():
    d, depth = 3, 4
    path = randn((1, 6, d), seed=11)
    S = as_dict(TO.signature(path, depth)[0], d, depth)
    lg = as_dict(TO.logsignature(path, depth)[0], d, depth)
    for a in range(d):
        assert abs(lg[(a,)] - S[(a,)]) < 1e-14
        for b in range(d):
            assert abs(lg[(a, b)] - 0.5 * (S[(a, b)] - S[(b, a)])) < 1e-14
    # a Lie element is orthogonal to every shuffle product of two non-empty words
    for u, v in [((0,), (1,)), ((0, 1), (2,)), ((0,), (0,)), ((2, 0), (1, 1)), ((1,), (0, 2, 2))]:
        assert abs(sum(lg[w] for w in shuffles(u, v))) < 1e-13, (u, v)
    # one segment: the log-signature is the increment itself
    seg = torch.zeros(1, 2, d)
    seg[0, 1] = torch.tensor([0.3, -0.8, 1.1])
    flat = TO.logsignature(seg, depth)[0]
    assert (flat[:d] - seg[0, 1]).abs().max() < 1e-15 and flat[d:].abs().max() < 1e-15


@pytest.mark.parametrize("d,depth,top", [(2, 4, None), (3, 3, None), (3, 4, "lyndon"), (2, 5, "some")])
def test_words_logsig_matches_tensor_logsig(d, depth, top):
    from pathsig_amd.projections import lyndon_codes
    path = randn((2, 6, d), seed=12)
    dense = TO.signature(path, depth)
    if top is None:
        top_codes, top_size = None, d ** depth
    elif top == "lyndon":
        top_codes = lyndon_codes(d, depth)
        top_size = len(top_codes)
    else:
        top_codes = [5, 0, 31, 12, 12, 7]
        top_size = len(top_codes)
    cols = TO.hybrid_columns(d, depth, top_size, top_codes)
    hyb = dense[:, cols]
    want_log = TO.logsignature(path, depth)[:, cols]
    lt, Pt = TO.sig_to_logsig(hyb, depth, d, top_size, top_codes)
    lw, Pw = WO.logsig_forward(hyb, depth, d, top_size, top_codes)
    assert (lt - want_log).abs().max() < 1e-13
    assert (lw - want_log).abs().max() < 1e-13
    assert (Pw - Pt).abs().max() < 1e-13
    # P cache layout: P_1 is the signature itself, entries above the word length are zero
    P3 = Pw.reshape(2, len(cols), depth)
    assert torch.equal(P3[:, :, 0], hyb)
    assert P3[:, :d, 1:].abs().max() == 0
    # adjoint
    g = randn(tuple(hyb.shape), seed=13)
    gt = TO.logsig_vjp(hyb, g, depth, d, top_size, top_codes)
    gw = WO.logsig_backward(hyb, Pw, g, depth, d, top_size, top_codes)
    assert (gw - gt).abs().max() < 1e-12


def _word_of(col, d, depth):
    """Letters of the word at dense column `col` (levels one after the other, words in base-d order)."""
    for n in range(1, depth + 1):
        if col < d ** n:
            return tuple((col // d ** (n - 1 - i)) % d for i in range(n))
        col -= d ** n
    raise AssertionError("column beyond the last level")


def _power_by_cuts(logs, w, k):
    """(L^(x)k)(w) from the definition: the sum over the ways to cut w into k non-empty consecutive pieces of the
    product of L on the pieces."""
    n, total = len(w), 0.0
    for cuts in itertools.combinations(range(1, n), k - 1):
        edges = (0,) + cuts + (n,)
        term = 1.0
        for a, b in zip(edges[:-1], edges[1:]):
            term *= logs[w[a:b]]
        total += term
    return total


@pytest.mark.parametrize("d,depth,top", [(2, 4, None), (3, 3, None), (3, 4, "lyndon"), (2, 5, "some")])
def test_logsig_power_cache_against_powers_from_the_definition(d, depth, top):
    """`logsig_power_cache` against tensor powers written out word by word (sums over the cuts of the word), of
    a logarithm computed another way than the one the cache is usually built from (level by level from
    exp(L) = S, not the alternating series)."""
    from pathsig_amd.projections import lyndon_codes
    path = randn((2, 5, d), seed=21) * 0.7
    if top is None:
        top_codes, top_size = None, d ** depth
    elif top == "lyndon":
        top_codes = lyndon_codes(d, depth)
        top_size = len(top_codes)
    else:
        top_codes = [5, 0, 31, 12, 12, 7]
        top_size = len(top_codes)
    cols = TO.hybrid_columns(d, depth, top_size, top_codes)
    dense_log = TO.logsignature(path, depth, method="inverse_exp")
    got = TO.logsig_power_cache(dense_log[:, cols], depth, d, top_size, top_codes).reshape(2, len(cols), depth)
    for row in range(2):
        logs = {_word_of(c, d, depth): float(dense_log[row, c]) for c in range(dense_log.shape[1])}
        for idx, col in enumerate(cols):
            w = _word_of(col, d, depth)
            powers = [_power_by_cuts(logs, w, k) for k in range(1, len(w) + 1)]
            want = powers + [0.0] * (depth - len(w))
            if len(w) < depth:
                # the weight with which w enters the top-level sums of the adjoint as a prefix
                want[len(w)] = -sum(powers[m - 1] / math.factorial(m + 1) for m in range(1, len(w) + 1))
            for k in range(depth):
                assert abs(float(got[row, idx, k]) - want[k]) < 1e-13, (row, w, k)


# ------------------------------------------------------------------------------------------------
# gradients
# ------------------------------------------------------------------------------------------------
def test_tensor_vjp_matches_finite_differences():
    d, depth = 2, 3
    path = randn((1, 5, d), seed=14)
    G = randn((1, TO.dense_size(d, depth)), seed=15)
    g = TO.signature_vjp(path, G, depth)
    eps = 1e-6
    for t in range(5):
        for a in range(d):
            hi, lo = path.clone(), path.clone()
            hi[0, t, a] += eps
            lo[0, t, a] -= eps
            fd = float(((TO.signature(hi, depth) - TO.signature(lo, depth)) * G).sum() / (2 * eps))
            assert abs(fd - float(g[0, t, a])) < 1e-8


@pytest.mark.parametrize("case", ["dense", "windows", "words", "lyndon", "gap"])
def test_words_backward_matches_autograd(case):
    from pathsig_amd.projections import projections
    d, depth, L = 3, 4, 9
    path = randn((2, L, d), seed=16)
    level_sizes = codes = wins = None
    if case == "windows":
        wins = [(0, 9), (2, 6), (4, 9), (3, 5), (0, 4)]
    elif case == "words":
        p = projections.words(random_word_set(d, 1, 4, 30, seed=2), depth=depth, path_dim=d)
        level_sizes, codes = p.level_sizes, p._codes
    elif case == "lyndon":
        p = projections.lyndon(depth=depth, path_dim=d)
        level_sizes, codes = p.level_sizes, p._codes
    elif case == "gap":  # an empty level below requested ones
        p = projections.words([(0,), (2,), (0, 1, 2), (2, 2, 1), (1, 0, 0, 2)], depth=depth, path_dim=d)
        level_sizes, codes = p.level_sizes, p._codes
    sig = TO.compute_signature(path, depth, level_sizes, codes, wins)
    sig_w = WO.sig_forward(path, depth, level_sizes, codes, wins)
    assert (sig - sig_w).abs().max() < 1e-13
    G = randn(tuple(sig.shape), seed=17)
    want = TO.signature_vjp(path, G, depth, level_sizes, codes, wins)
    got = WO.sig_backward(path, sig_w, G, depth, level_sizes, codes, wins)
    assert (got - want).abs().max() < 1e-12


def test_fp32_words_oracle_close_to_fp64():
    d, depth = 4, 4
    path = brownian_path(3, 64, d, seed=18)
    want = TO.signature(path, depth)
    got = WO.sig_forward(path.float(), depth)
    assert (got.double() - want).abs().max() < 1e-6
