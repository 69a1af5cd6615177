"""`Signature` and `LogSignature` modules (keyword-only constructors, same buffers and persistence
flags as the reference `src/pathsig/modules.py:45-135`, so state_dicts are interchangeable)."""
from __future__ import annotations

import torch
from torch import nn

from .ops import _logsig_of, compute_signature

_DEVICE = "cuda"


def _checked_depth(depth: int) -> int:
    if depth < 1 or depth > 12:
        raise ValueError("depth must satisfy 1 <= depth <= 12.")
    return depth


def _no_tensor(dtype: torch.dtype, shape=(0,)) -> torch.Tensor:
    return torch.empty(shape, dtype=dtype, device=_DEVICE)


def _window_buffer(windows):
    """(use_windows, int32 [W,2] buffer).  Windows are half-open [start, end) over point indices."""
    if windows is None:
        return False, _no_tensor(torch.int32, (0, 2))
    if windows.device.type != "cuda":
        raise TypeError("windows must be a CUDA tensor.")
    if windows.dim() != 2 or windows.size(1) != 2:
        raise TypeError("windows must have shape [num_windows, 2].")
    if windows.dtype not in (torch.int32, torch.int64):
        raise TypeError("windows must have dtype int32 or int64.")
    return True, windows.contiguous().to(dtype=torch.int32)


def _projection_words(projection):
    if projection is None:
        return False, None
    words = projection.encoded_words
    if words.device.type != "cuda" or words.dtype != torch.int64 or words.dim() != 1:
        raise TypeError("projection.encoded_words must be a 1D CUDA int64 tensor.")
    return True, words.contiguous()


class Signature(nn.Module):
    """Truncated signature of a batch of paths (B, L, d) -> (B, S) or, with windows, (B, W, S)."""

    def __init__(self, *, depth: int, projection=None, windows=None):
        super().__init__()
        self.depth = _checked_depth(depth)
        self.projection = projection
        self.alternative_projection, words = _projection_words(projection)
        self.use_windows, win = _window_buffer(windows)
        self.register_buffer("_windows", win, persistent=self.use_windows)
        self.register_buffer("_encoded_words", words if self.alternative_projection else _no_tensor(torch.int64),
                             persistent=self.alternative_projection)
        self._level_sizes = projection.level_sizes if self.alternative_projection else []

    def forward(self, path: torch.Tensor) -> torch.Tensor:
        return compute_signature(path, self.depth, self.alternative_projection, self._encoded_words,
                                 self._level_sizes, self.use_windows, self._windows)


class LogSignature(nn.Module):
    """Truncated log-signature.  With a projection the signature is computed in a hybrid layout
    (levels below `depth` dense, level `depth` as projected), converted, and the projection's
    coordinates are selected from it."""

    def __init__(self, *, depth: int, projection=None, windows=None):
        super().__init__()
        self.depth = _checked_depth(depth)
        self.projection = projection
        self.alternative_projection, words = _projection_words(projection)
        self.use_windows, win = _window_buffer(windows)
        self.register_buffer("_windows", win, persistent=self.use_windows)

        if not self.alternative_projection:
            for name in ("_encoded_words", "_top_words", "_indices_from_sig"):
                self.register_buffer(name, _no_tensor(torch.int64), persistent=False)
            self._level_sizes: list[int] = []
            self._ext_level_sizes: list[int] = []
            return

        self.register_buffer("_encoded_words", words, persistent=True)
        self._level_sizes = projection.level_sizes
        d = self._path_dim = int(projection.path_dim)
        # codes of the non-dense levels below `depth` come first in the stored list; skip them
        skipped = sum(self._level_sizes[k] for k in range(1, self.depth) if self._level_sizes[k] != d ** k)
        self.register_buffer("_top_words", words[skipped:], persistent=True)
        self._ext_level_sizes = [0] + [d ** k for k in range(1, self.depth)] + [int(self._level_sizes[self.depth])]
        picked = projection.logsig_indices()
        self.register_buffer("_indices_from_sig", picked.to(device=_DEVICE, dtype=torch.int64).contiguous(),
                             persistent=True)

    def forward(self, path: torch.Tensor) -> torch.Tensor:
        if self.alternative_projection:
            d = self._path_dim
            sizes = self._ext_level_sizes
        else:
            d = int(path.shape[-1])
            sizes = [0] + [d ** k for k in range(1, self.depth + 1)]
        top_words = self._top_words
        sig = compute_signature(path, self.depth, self.alternative_projection, top_words, sizes, self.use_windows,
                                self._windows)
        logsig = _logsig_of(sig, self.depth, d, self.alternative_projection, top_words, sizes)
        if not self.alternative_projection:
            return logsig
        return logsig.index_select(dim=-1, index=self._indices_from_sig.to(logsig.device))
