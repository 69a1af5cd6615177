"""Word projections: host-side plans that say which signature coefficients an operator computes.

A plan is the pair (`encoded_words`, `level_sizes`):

* `level_sizes[k]` (k = 1..depth, entry 0 unused) is the number of output columns of level k;
* a level with `level_sizes[k] == path_dim**k` is *full*: its columns are all words of length k in
  lexicographic order and no codes are stored for it;
* for every other level the columns follow `encoded_words`, the base-`path_dim` codes (first letter
  most significant) of the chosen words, concatenated over the non-full levels only.

Behaviour follows the reference planner `src/pathsig/projections.py:8-298` (same class names,
properties, validation limits, orderings and error types).  The integer work happens on the host
with Python ints; the device tensor is only materialised when `encoded_words` is first read, so a
plan can be built and inspected on a machine without a GPU.
"""
from __future__ import annotations

from typing import Iterable, List, Optional, Sequence, Tuple, Union

import torch

_MAX_DEPTH = 12
_WORD_BITS = 64
# largest path_dim whose depth-n codes fit a signed 64-bit integer, for the depths where this is
# stricter than the bits-per-letter rule (`src/pathsig/projections.py:69-74`)
_INT64_BASE_LIMIT = {2: 3037000499, 4: 55108, 8: 234}


class Projection:
    """Common behaviour of all projections (`src/pathsig/projections.py:8-74`)."""

    depth: int
    path_dim: int
    _codes: List[int]
    _level_sizes: List[int]
    _device_codes: Optional[torch.Tensor] = None

    # -- plan accessors ---------------------------------------------------------------------
    @property
    def encoded_words(self) -> torch.Tensor:
        """1-D int64 device tensor with the codes of the non-full levels."""
        if self._device_codes is None:
            self._device_codes = torch.tensor(self._codes, dtype=torch.int64, device="cuda")
        return self._device_codes

    @property
    def level_sizes(self) -> List[int]:
        return self._level_sizes

    @property
    def sig_size(self) -> int:
        return sum(self._level_sizes[1:self.depth + 1])

    def _logsig_index_list(self) -> List[int]:
        """Columns of the hybrid signature layout (levels below `depth` dense, level `depth` as in
        this plan) that make up the projected log-signature (`src/pathsig/projections.py:26-50`)."""
        picked: List[int] = []
        dense_off = 0
        code_off = 0
        width = 1
        for k in range(1, self.depth):
            width *= self.path_dim
            size = self._level_sizes[k]
            if size == width:
                picked.extend(range(dense_off, dense_off + width))
            else:
                picked.extend(dense_off + c for c in self._codes[code_off:code_off + size])
                code_off += size
            dense_off += width
        picked.extend(range(dense_off, dense_off + self._level_sizes[self.depth]))
        return picked

    def logsig_indices(self) -> torch.Tensor:
        return torch.tensor(self._logsig_index_list(), dtype=torch.int64, device=self.encoded_words.device)

    # -- validation -------------------------------------------------------------------------
    @staticmethod
    def _validate_inputs(d: int, depth: int, full_levels, max_depth: int = _MAX_DEPTH,
                         word_bits: int = _WORD_BITS) -> None:
        if d <= 1:
            raise ValueError(f"path_dim must be >= 2 (got {d}).")
        if depth < 1 or depth > max_depth:
            raise ValueError(f"depth must satisfy 1 <= depth <= {max_depth} (got {depth}).")
        if full_levels and (min(full_levels) < 1 or max(full_levels) > depth):
            raise ValueError("full_levels entries must satisfy 1 <= level <= depth.")
        # letters of a word share one 64-bit register on the device; depth 1 is held to the depth-2 rule
        eff = max(depth, 2)
        letter_bits = word_bits // eff
        if (d - 1).bit_length() > letter_bits:
            raise ValueError(f"Maximum path_dim for depth={depth} is {1 << letter_bits}, but got path_dim={d}.")
        limit = _INT64_BASE_LIMIT.get(eff)
        if limit is not None and d > limit:
            raise ValueError(f"Maximum path_dim for depth={depth} is {limit}, but got path_dim={d}.")

    def _drop_codes_of_complete_levels(self, codes: List[int], sizes: List[int]) -> None:
        """A level that lists every word is emitted as a full level, in lexicographic order."""
        pos = 0
        for k in range(1, self.depth + 1):
            if sizes[k] == self.path_dim ** k:
                del codes[pos:pos + sizes[k]]
            else:
                pos += sizes[k]


class WordsProjection(Projection):
    """Projection onto an explicit list of words (`src/pathsig/projections.py:76-130`)."""

    def __init__(self, words: Iterable[Iterable[int]], depth: int, path_dim: int,
                 full_levels: Iterable[int] = ()) -> None:
        self.path_dim = int(path_dim)
        self.depth = int(depth)
        self._full_levels = {int(k) for k in full_levels}
        self._validate_inputs(self.path_dim, self.depth, self._full_levels)
        self._codes, self._level_sizes = self._plan(words)

    def _plan(self, words) -> Tuple[List[int], List[int]]:
        d = self.path_dim
        codes: List[int] = []
        sizes = [0] * (self.depth + 1)
        longest = 0
        for word in words:
            code = length = 0
            for letter in word:
                if letter < 0 or letter >= d:
                    raise ValueError(
                        "Invalid letter encountered in a word, ensure all letters satisfy 0 <= letter < d.")
                code = code * d + letter
                length += 1
            if length < longest:
                raise ValueError("Words must be non-decreasing in length.")
            if length > self.depth:
                break  # words past the truncation depth end the list
            longest = length
            codes.append(code)
            sizes[length] += 1
        self._drop_codes_of_complete_levels(codes, sizes)
        for k in self._full_levels:
            if sizes[k] > 0:
                raise ValueError(
                    f"Degree {k} is marked as full, but explicit words were also provided for that level.")
            sizes[k] = d ** k
        return codes, sizes


class AnisotropicProjection(Projection):
    """Words whose summed letter weights stay within a threshold
    (`src/pathsig/projections.py:132-223`)."""

    def __init__(self, weights: Union[Sequence[float], torch.Tensor], weight_threshold: float, depth: int,
                 path_dim: int, full_levels: Iterable[int] = ()) -> None:
        self.path_dim = int(path_dim)
        self.depth = int(depth)
        self._full_levels = {int(k) for k in full_levels}
        self._validate_inputs(self.path_dim, self.depth, self._full_levels)
        self.weight_threshold = float(weight_threshold)
        if self.weight_threshold <= 0.0:
            raise ValueError("weight_threshold must be > 0.")
        if isinstance(weights, torch.Tensor):
            listed = weights.detach().to(device="cpu").flatten().tolist()
        else:
            listed = list(weights)
        if len(listed) != self.path_dim:
            raise ValueError(f"weights must have length == path_dim ({self.path_dim}), got {len(listed)}.")
        self.weights = [float(v) for v in listed]
        if any(v < 0.0 for v in self.weights):
            raise ValueError("weights must be non-negative.")
        self._codes, self._level_sizes = self._plan()

    def _plan(self) -> Tuple[List[int], List[int]]:
        d, thr, wts = self.path_dim, self.weight_threshold, self.weights
        sizes = [0] * (self.depth + 1)
        # breadth-first growth: level k extends every kept word of level k-1, letters ascending;
        # weights are accumulated in float in exactly this order
        frontier = [(a, wts[a]) for a in range(d) if wts[a] <= thr]
        if not frontier:
            raise ValueError("At least one weight must be <= weight_threshold.")
        codes = [c for c, _ in frontier]
        sizes[1] = len(frontier)
        for k in range(2, self.depth + 1):
            grown = []
            for code, weight in frontier:
                for a in range(d):
                    total = weight + wts[a]
                    if total <= thr:
                        grown.append((code * d + a, total))
            sizes[k] = len(grown)
            codes.extend(c for c, _ in grown)
            frontier = grown
            if not grown:
                break
        pos = 0
        for k in range(1, self.depth + 1):
            size = sizes[k]
            if size == 0 and k in self._full_levels:
                sizes[k] = d ** k
            elif k in self._full_levels or size == d ** k:
                del codes[pos:pos + size]
                sizes[k] = d ** k
            else:
                pos += size
        return codes, sizes


class LyndonProjection(Projection):
    """Lyndon words of every length up to `depth` (`src/pathsig/projections.py:225-272`)."""

    def __init__(self, depth: int, path_dim: int, full_levels: Iterable[int] = ()) -> None:
        self.depth = int(depth)
        self.path_dim = int(path_dim)
        self._full_levels = {int(k) for k in full_levels}
        self._validate_inputs(self.path_dim, self.depth, self._full_levels)
        self._codes, self._level_sizes = self._plan()

    def _plan(self) -> Tuple[List[int], List[int]]:
        d = self.path_dim
        sizes = [0] * (self.depth + 1)
        sizes[1] = d  # every letter is a Lyndon word: level 1 is always full
        codes: List[int] = []
        for k in range(2, self.depth + 1):
            if k in self._full_levels:
                sizes[k] = d ** k
            else:
                level = lyndon_codes(d, k)
                sizes[k] = len(level)
                codes.extend(level)
        return codes, sizes


def lyndon_codes(d: int, n: int) -> List[int]:
    """Codes of the Lyndon words of length exactly n over d letters, ascending (Duval's generation;
    same output order as `src/pathsig/projections.py:253-272`)."""
    out: List[int] = []
    word = [-1]
    while word:
        word[-1] += 1
        period = len(word)
        if period == n:
            code = 0
            for letter in word:
                code = code * d + letter
            out.append(code)
        while len(word) < n:  # periodic extension
            word.append(word[len(word) - period])
        while word and word[-1] == d - 1:
            word.pop()
    return out


class projections:
    """Factory namespace: `projections.words(...)`, `.anisotropic(...)`, `.lyndon(...)`
    (`src/pathsig/projections.py:274-298`)."""

    @staticmethod
    def words(words: Iterable[Iterable[int]], depth: int, path_dim: int,
              full_levels: Iterable[int] = ()) -> WordsProjection:
        return WordsProjection(words, depth, path_dim, full_levels)

    @staticmethod
    def anisotropic(weights: Union[Sequence[float], torch.Tensor], weight_threshold: float, depth: int,
                    path_dim: int, full_levels: Iterable[int] = ()) -> AnisotropicProjection:
        return AnisotropicProjection(weights, weight_threshold, depth, path_dim, full_levels)

    @staticmethod
    def lyndon(depth: int, path_dim: int, full_levels: Iterable[int] = ()) -> LyndonProjection:
        return LyndonProjection(depth, path_dim, full_levels)
