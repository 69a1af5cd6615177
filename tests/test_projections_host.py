"""Planner behaviour on the host: orderings, sizes, error types.  Restates, without a GPU, what the
reference's `tests/test_projections.py:327-353` and the planner source pin, plus independent checks
of the Lyndon enumeration (definition by rotations, Witt's formula)."""
from __future__ import annotations

import itertools

import pytest

from pathsig_amd.projections import (AnisotropicProjection, LyndonProjection, WordsProjection, lyndon_codes,
                                     projections)
from tests.helpers import code_of


def is_lyndon(w):
    return all(w < w[i:] + w[:i] for i in range(1, len(w)))


def mobius(n):
    res, p, m = 1, 2, n
    while p * p <= m:
        if m % p == 0:
            m //= p
            if m % p == 0:
                return 0
            res = -res
        p += 1
    return -res if m > 1 else res


def witt(d, n):
    return sum(mobius(k) * d ** (n // k) for k in range(1, n + 1) if n % k == 0) // n


@pytest.mark.parametrize("d,n", [(2, 1), (2, 5), (3, 4), (4, 3), (5, 2), (2, 8), (3, 6)])
def test_lyndon_words_by_definition(d, n):
    want = [code_of(w, d) for w in itertools.product(range(d), repeat=n) if is_lyndon(w)]
    assert lyndon_codes(d, n) == want  # itertools.product is lexicographic == ascending code
    assert len(want) == witt(d, n)


def test_lyndon_counts_of_the_benchmark_projection():
    p = projections.lyndon(5, 8)
    assert p.level_sizes == [0, 8, 28, 168, 1008, 6552]
    assert [witt(8, n) for n in range(1, 6)] == [8, 28, 168, 1008, 6552]
    assert p.sig_size == 7764 and len(p._codes) == 7756
    assert len(p._logsig_index_list()) == 7764
    # levels below the top map to dense offsets + code, the top level to a plain range
    offs = [0, 8, 72, 584, 4680]
    idx = p._logsig_index_list()
    assert idx[:8] == list(range(8))
    assert idx[8:36] == [offs[1] + c for c in p._codes[:28]]
    assert idx[-6552:] == list(range(4680, 4680 + 6552))


def test_lyndon_full_levels():
    p = projections.lyndon(depth=4, path_dim=3, full_levels=(2, 4))
    assert p.level_sizes == [0, 3, 9, witt(3, 3), 81]
    assert p._codes == lyndon_codes(3, 3)
    assert isinstance(p, LyndonProjection)


def test_words_order_is_kept_and_complete_levels_become_dense():
    d, depth = 3, 3
    words = [(2,), (0,), (1, 1), (0, 2), (2, 2, 1), (0, 0, 0)]
    p = projections.words(words, depth=depth, path_dim=d)
    assert isinstance(p, WordsProjection)
    assert p.level_sizes == [0, 2, 2, 2]
    assert p._codes == [2, 0, 4, 2, 25, 0]
    # every word of levels 1 and 2 listed (in any order): those levels turn dense and lose their codes
    allw = [w for n in (1, 2) for w in itertools.product(range(d), repeat=n)]
    p = projections.words(list(reversed(allw[:3])) + list(reversed(allw[3:])) + [(1, 0, 2)], depth=depth, path_dim=d)
    assert p.level_sizes == [0, 3, 9, 1] and p._codes == [code_of((1, 0, 2), d)]
    assert p.sig_size == 13


def test_words_validation():
    with pytest.raises(ValueError, match="letter"):
        projections.words([(0, 3)], depth=2, path_dim=3)
    with pytest.raises(ValueError, match="non-decreasing"):
        projections.words([(0, 1), (2,)], depth=2, path_dim=3)
    with pytest.raises(ValueError, match="full"):
        projections.words([(0,), (1, 1)], depth=2, path_dim=3, full_levels=[1])
    # a word longer than the depth ends the list
    p = projections.words([(0,), (1, 1), (0, 1, 2), (2, 2)], depth=2, path_dim=3)
    assert p.level_sizes == [0, 1, 1] and p._codes == [0, 4]
    p = projections.words([(0, 1)], depth=3, path_dim=4, full_levels=(1, 3))
    assert p.level_sizes == [0, 4, 1, 64] and p.sig_size == 69


def test_input_limits():
    with pytest.raises(ValueError, match="path_dim"):
        projections.lyndon(depth=2, path_dim=1)
    with pytest.raises(ValueError, match="depth"):
        projections.lyndon(depth=13, path_dim=2)
    with pytest.raises(ValueError, match="depth"):
        projections.lyndon(depth=0, path_dim=2)
    with pytest.raises(ValueError, match="full_levels"):
        projections.lyndon(depth=3, path_dim=2, full_levels=(4,))
    # letters of a word share 64 bits: depth 12 allows 5 bits per letter
    projections.words([], depth=12, path_dim=32)
    with pytest.raises(ValueError, match="Maximum path_dim"):
        projections.words([], depth=12, path_dim=33)
    # codes must fit int64 where that is stricter than the bit rule
    projections.words([], depth=4, path_dim=55108)
    with pytest.raises(ValueError, match="55108"):
        projections.words([], depth=4, path_dim=55109)
    with pytest.raises(ValueError, match="234"):
        projections.words([], depth=8, path_dim=235)
    # depth 1 is held to the depth-2 limit
    with pytest.raises(ValueError, match="3037000499"):
        projections.words([], depth=1, path_dim=3037000500)


def test_anisotropic():
    p = projections.anisotropic([1.0, 2.0, 3.0], weight_threshold=4.0, depth=3, path_dim=3)
    assert isinstance(p, AnisotropicProjection)
    # level 1: all three letters (dense); level 2: pairs with weight <= 4; level 3: triples with weight <= 4
    lvl2 = [code_of((a, b), 3) for a in range(3) for b in range(3) if [1, 2, 3][a] + [1, 2, 3][b] <= 4]
    lvl3 = [code_of(w, 3) for w in itertools.product(range(3), repeat=3) if sum([1, 2, 3][a] for a in w) <= 4]
    assert p.level_sizes == [0, 3, len(lvl2), len(lvl3)]
    assert p._codes == lvl2 + lvl3
    # a letter above the threshold drops out of level 1, which then stores codes
    p = projections.anisotropic([1.0, 5.0], weight_threshold=2.0, depth=2, path_dim=2)
    assert p.level_sizes == [0, 1, 1] and p._codes == [0, 0]
    # an emptied level stops the growth; a full level requested on top of it stays dense
    p = projections.anisotropic([1.0, 1.0], weight_threshold=1.5, depth=3, path_dim=2, full_levels=(3,))
    assert p.level_sizes == [0, 2, 0, 8] and p._codes == []
    with pytest.raises(ValueError, match="weight_threshold"):
        projections.anisotropic([1.0, 1.0], weight_threshold=0.0, depth=2, path_dim=2)
    with pytest.raises(ValueError, match="length"):
        projections.anisotropic([1.0], weight_threshold=1.0, depth=2, path_dim=2)
    with pytest.raises(ValueError, match="non-negative"):
        projections.anisotropic([1.0, -1.0], weight_threshold=1.0, depth=2, path_dim=2)
    with pytest.raises(ValueError, match="At least one"):
        projections.anisotropic([3.0, 4.0], weight_threshold=1.0, depth=2, path_dim=2)


def test_sig_size_and_logsig_index_length():
    for d, depth in [(2, 3), (3, 4), (4, 2)]:
        p = projections.lyndon(depth=depth, path_dim=d)
        assert p.sig_size == sum(p.level_sizes[1:])
        assert len(p._logsig_index_list()) == p.sig_size
