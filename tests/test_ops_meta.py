"""Operator registration checked without a GPU: schemas equal to the reference's, and output shapes inferred for
meta tensors (`src/pathsig/ops.py:59-84,101-123,152-179,197-227`)."""
from __future__ import annotations

import os
import subprocess
import sys

import pytest
import torch

import pathsig_amd  # noqa: F401  (registers the ops)
from pathsig_amd import ops

REFERENCE_SCHEMAS = {
    "compute_signature": "pathsig::compute_signature(Tensor path_in, int depth, bool alternative_projection, "
                         "Tensor encoded_words, int[] level_sizes, bool use_windows, Tensor windows) -> Tensor",
    "signature_backward": "pathsig::signature_backward(Tensor path_in, Tensor signature_in, Tensor grad_signature_in, "
                          "int depth, bool alternative_projection, Tensor encoded_words, int[] level_sizes, "
                          "bool use_windows, Tensor windows) -> Tensor",
    "sig_to_logsig": "pathsig::sig_to_logsig(Tensor signature_in, int depth, int d, bool alternative_projection, "
                     "Tensor encoded_words, int[] level_sizes) -> (Tensor, Tensor)",
    "logsig_backward": "pathsig::logsig_backward(Tensor signature_in, Tensor P_in, Tensor grad_logsig_in, int depth, "
                       "bool alternative_projection, Tensor encoded_words, int[] level_sizes) -> Tensor",
}


def test_schemas_are_the_reference_ones():
    """`src/pathsig/bindings.cpp:9-63`, verbatim, with the pt2 tag."""
    for name, schema in REFERENCE_SCHEMAS.items():
        op = getattr(torch.ops.pathsig, name).default
        assert str(op._schema) == schema
        assert torch.Tag.pt2_compliant_tag in op.tags


def _meta(*shape, dtype=torch.float32):
    return torch.empty(*shape, dtype=dtype, device="meta")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_meta_shapes(dtype):
    B, L, d, depth = 5, 40, 3, 4
    path = _meta(B, L, d, dtype=dtype)
    no_words, no_win = _meta(0, dtype=torch.int64), _meta(0, 2, dtype=torch.int32)
    S = sum(d ** k for k in range(1, depth + 1))
    sig = torch.ops.pathsig.compute_signature(path, depth, False, no_words, [], False, no_win)
    assert sig.shape == (B, S) and sig.dtype == dtype and sig.device.type == "meta"
    win = _meta(7, 2, dtype=torch.int64)
    sizes = [0, 3, 4, 0, 6]
    words = _meta(10, dtype=torch.int64)
    sig_w = torch.ops.pathsig.compute_signature(path, depth, True, words, sizes, True, win)
    assert sig_w.shape == (B, 7, 13)
    grad = torch.ops.pathsig.signature_backward(path, sig_w, sig_w, depth, True, words, sizes, True, win)
    assert grad.shape == path.shape and grad.dtype == dtype
    full = [0] + [d ** k for k in range(1, depth + 1)]
    logsig, cache = torch.ops.pathsig.sig_to_logsig(sig, depth, d, False, no_words, full)
    assert logsig.shape == sig.shape and cache.shape == (B, S * depth)
    assert torch.ops.pathsig.logsig_backward(sig, cache, logsig, depth, False, no_words, full).shape == sig.shape
    # the keeping pair: same signature shape, plus a flat buffer whose size the library reports
    sig_k, chunks = torch.ops.pathsig.compute_signature_keep(path, depth, False, no_words, [], False, no_win)
    assert sig_k.shape == sig.shape and chunks.dim() == 1 and chunks.dtype == dtype
    assert chunks.numel() == ops._chunks_numel(path, depth, False, [], 0)
    grad_k = torch.ops.pathsig.signature_backward_kept(path, sig, sig, chunks, depth, False, no_words, [], False, no_win)
    assert grad_k.shape == path.shape


def test_chunk_buffer_size_follows_the_library():
    """Long paths at a register-tiled shape are cut into time chunks (a buffer to hand over); other calls are not."""
    long_dense = _meta(128, 1024, 4)
    assert ops._chunks_numel(long_dense, 6, False, [], 0) % (128 * (4 + 16 + 64 + 256 + 1024)) == 0
    assert ops._chunks_numel(long_dense, 6, False, [], 0) > 0
    assert ops._chunks_numel(_meta(128, 1024, 17), 4, False, [], 0) == 0     # no tiled shape for d = 17
    assert ops._chunks_numel(_meta(4096, 20, 4), 6, False, [], 0) == 0       # short paths, many rows: one chunk


def test_missing_operator_library_is_an_error(tmp_path):
    """There is one registration (C++): a package copy without libpathsig_torch.so refuses to import."""
    import shutil
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = tmp_path / "pathsig_amd"
    shutil.copytree(os.path.join(root, "pathsig_amd"), pkg, ignore=shutil.ignore_patterns("csrc", "__pycache__", "libpathsig_torch.so"))
    res = subprocess.run([sys.executable, "-c", "import pathsig_amd"], capture_output=True, text=True, timeout=300,
                         cwd=str(tmp_path))
    assert res.returncode != 0 and "libpathsig_torch.so" in res.stderr
