"""CPU checker for the signature / log-signature path, written as level-tensor algebra in torch.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; it is used by the
test-suite, by the smoke check and by the CPU-baseline leg of the benchmark.

The reference (a CUDA-only extension) evaluates every requested word on its own thread
(`src/pathsig/forward/sig_kernels.cu:79-157`).  This module restates the same mathematics in the
dense level-tensor form so that it can run on a CPU in fp64 and be differentiated by autograd:

* `signature_levels`   S <- S (x) exp(dx) per increment, Horner form
                       (same recurrence as `sig_kernels.cu:139-152`, all words of a level at once);
* `windowed`           a window [s, e) is the signature of `path[:, s:e]`
                       (`sig_kernels.cu:116-126`, `tests/test_windows.py:41-44`);
* `project`            column j of a non-full level is the dense entry `level_offset + code_j`
                       (`forward/sig_launch.cu:171-206`, `tests/test_projections.py:13-37`);
* `tensor_log_levels`  log(1 + X) = sum_m (-1)^(m+1)/m X^(x)m with P_m = P_{m-1} (x) X
                       (`sig_kernels.cu:221-240`);
* `sig_to_logsig`      logsig and the P cache in the "dense below the top level" layout
                       (`src/pathsig/modules.py:98-135`, `sig_kernels.cu:184,215-216`);
* `logsig_power_cache` tensor powers of the log-signature in the same layout (what the keeping forward of the
                       HIP library hands to its adjoint; not in the reference).

Pinned by tests/test_oracle_math.py (closed forms, brute-force iterated sums, Chen, shuffle
products, exp/log round trip, Lie property, finite differences) and cross-checked against the
literal per-word restatement in oracle/ref_words.c.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


# ----------------------------------------------------------------------------------------------
# layout helpers
# ----------------------------------------------------------------------------------------------
def dense_level_offsets(d: int, depth: int) -> List[int]:
    """offsets[k] = index of the first level-k coefficient in the dense layout (k = 1..depth)."""
    offs = [0] * (depth + 2)
    acc = 0
    for k in range(1, depth + 1):
        offs[k] = acc
        acc += d ** k
    offs[depth + 1] = acc
    return offs


def dense_size(d: int, depth: int) -> int:
    return sum(d ** k for k in range(1, depth + 1))


def projection_columns(d: int, depth: int, level_sizes: Sequence[int], codes: Sequence[int]) -> List[int]:
    """Dense-layout column of every projected output column (`forward/sig_launch.cu:171-206`)."""
    cols: List[int] = []
    off_codes = 0
    offs = dense_level_offsets(d, depth)
    for k in range(1, depth + 1):
        size = int(level_sizes[k])
        if size == d ** k:
            cols.extend(range(offs[k], offs[k] + size))
        elif size > 0:
            cols.extend(offs[k] + int(c) for c in codes[off_codes:off_codes + size])
            off_codes += size
    return cols


# ----------------------------------------------------------------------------------------------
# signature
# ----------------------------------------------------------------------------------------------
def signature_levels(path: torch.Tensor, depth: int) -> List[torch.Tensor]:
    """Dense truncated signature, one tensor (B, d**k) per level k = 1..depth.

    Horner step for target level m (A1 of the reference, `sig_kernels.cu:139-152`):
        h_1 = dx / m ;  h_j = (S_{j-1} + h_{j-1}) (x) dx / (m - j + 1) ;  S_m <- S_m + h_m
    with all S on the right-hand side taken before the step.
    """
    B, L, d = path.shape
    dx_all = path[:, 1:, :] - path[:, :-1, :]
    S = [torch.zeros(B, d ** k, dtype=path.dtype) for k in range(1, depth + 1)]
    for t in range(L - 1):
        dx = dx_all[:, t, :]
        new = []
        for m in range(1, depth + 1):
            h = dx / m
            for j in range(2, m + 1):
                h = ((S[j - 2] + h).unsqueeze(2) * (dx / (m - j + 1)).unsqueeze(1)).reshape(B, -1)
            new.append(S[m - 1] + h)
        S = new
    return S


def signature(path: torch.Tensor, depth: int) -> torch.Tensor:
    """Dense signature in the reference's output layout: [level 1 | level 2 | ... ]."""
    return torch.cat(signature_levels(path, depth), dim=1)


def windowed(path: torch.Tensor, depth: int, windows: Sequence[Sequence[int]]) -> torch.Tensor:
    """(B, W, S): the signature of `path[:, s:e]` for every window [s, e)."""
    outs = []
    for s, e in windows:
        s, e = int(s), int(e)
        if e - s < 2:
            outs.append(torch.zeros(path.shape[0], dense_size(path.shape[2], depth), dtype=path.dtype))
        else:
            outs.append(signature(path[:, s:e, :], depth))
    return torch.stack(outs, dim=1)


def project(sig_dense: torch.Tensor, d: int, depth: int, level_sizes, codes) -> torch.Tensor:
    cols = torch.tensor(projection_columns(d, depth, level_sizes, codes), dtype=torch.int64)
    return sig_dense.index_select(-1, cols)


def compute_signature(path, depth, level_sizes=None, codes=None, windows=None) -> torch.Tensor:
    """Counterpart of the op `pathsig::compute_signature` (`src/pathsig/bindings.cpp:9-20`)."""
    d = path.shape[2]
    out = windowed(path, depth, windows) if windows is not None else signature(path, depth)
    if level_sizes is not None:
        out = project(out, d, depth, level_sizes, codes if codes is not None else [])
    return out


# ----------------------------------------------------------------------------------------------
# tensor algebra (used for the log and by the tests)
# ----------------------------------------------------------------------------------------------
def split_levels(flat: torch.Tensor, d: int, depth: int) -> List[torch.Tensor]:
    offs = dense_level_offsets(d, depth)
    return [flat[..., offs[k]:offs[k + 1]] for k in range(1, depth + 1)]


def tensor_product_levels(A: List[torch.Tensor], B: List[torch.Tensor], depth: int,
                          a0: float = 1.0, b0: float = 1.0) -> List[torch.Tensor]:
    """Truncated product of a0 + A and b0 + B (lists over levels 1..depth); returns levels 1..depth."""
    out = []
    for m in range(1, depth + 1):
        acc = a0 * B[m - 1] + b0 * A[m - 1]
        for k in range(1, m):
            lead = A[k - 1].shape[:-1]
            acc = acc + (A[k - 1].unsqueeze(-1) * B[m - k - 1].unsqueeze(-2)).reshape(*lead, -1)
        out.append(acc)
    return out


def tensor_log_powers(S: List[torch.Tensor], depth: int) -> List[List[torch.Tensor]]:
    """P[m-1][k-1] = level k of X^(x)m for X = S - 1 (`sig_kernels.cu:221-238`)."""
    P = [list(S)]
    for m in range(2, depth + 1):
        prev = P[-1]
        cur = []
        for n in range(1, depth + 1):
            lead = S[0].shape[:-1]
            acc = torch.zeros_like(S[n - 1])
            # X has no level-0 term and X^(x)(m-1) vanishes below level m-1
            for k in range(m - 1, n):
                acc = acc + (prev[k - 1].unsqueeze(-1) * S[n - k - 1].unsqueeze(-2)).reshape(*lead, -1)
            cur.append(acc)
        P.append(cur)
    return P


def tensor_log_levels(S: List[torch.Tensor], depth: int) -> List[torch.Tensor]:
    P = tensor_log_powers(S, depth)
    out = []
    for n in range(1, depth + 1):
        acc = torch.zeros_like(S[n - 1])
        for m in range(1, n + 1):
            acc = acc + ((-1.0) ** (m + 1) / m) * P[m - 1][n - 1]
        out.append(acc)
    return out


def tensor_log_levels_inverse_exp(S: List[torch.Tensor], depth: int) -> List[torch.Tensor]:
    """The same logarithm from exp(L) = S, level by level:  L_n = S_n - sum_{k=2}^{n} (L^(x)k)_n / k!  (the k-th
    power at level n only involves L_1 .. L_{n-1}).

    Not the reference's formula (that is `tensor_log_levels`), but the same function of S, and the one to check
    against where the alternating series is ill conditioned: the powers of X = S - 1 grow like exp|x| and cancel,
    which costs the series about log10(max|X^(x)m|) digits even in fp64 (1e-11 at depth 12), while the powers of
    L stay small and come with 1/k!.  Pinned by exp(L) = S with an independent exponential, by agreement with the
    series where that is well conditioned, and against the series summed in extended precision where it is not
    (tests/test_oracle_math.py)."""
    L: List[torch.Tensor] = []
    for n in range(1, depth + 1):
        acc = S[n - 1]
        if n >= 2:
            known = L + [torch.zeros_like(S[k - 1]) for k in range(n, depth + 1)]
            power = known
            fact = 1.0
            for k in range(2, n + 1):
                power = tensor_product_levels(power, known, n, a0=0.0, b0=0.0)
                fact *= k
                acc = acc - power[n - 1] / fact
        L.append(acc)
    return L


def logsignature(path: torch.Tensor, depth: int, windows=None, method: str = "series") -> torch.Tensor:
    """Dense log-signature (no projection), same layout as the signature.  method: "series" (the reference's
    alternating series) or "inverse_exp" (see `tensor_log_levels_inverse_exp`)."""
    d = path.shape[2]
    sig = windowed(path, depth, windows) if windows is not None else signature(path, depth)
    log_fn = tensor_log_levels if method == "series" else tensor_log_levels_inverse_exp
    return torch.cat(log_fn(split_levels(sig, d, depth), depth), dim=-1)


def hybrid_columns(d: int, depth: int, top_size: int, top_codes: Optional[Sequence[int]]) -> List[int]:
    """Dense column of every column of the hybrid layout: levels < depth dense, top level as given
    (`src/pathsig/modules.py:98-108`)."""
    offs = dense_level_offsets(d, depth)
    cols = list(range(0, offs[depth]))
    if top_codes is None or top_size == d ** depth:
        cols.extend(range(offs[depth], offs[depth] + top_size))
    else:
        cols.extend(offs[depth] + int(c) for c in top_codes[:top_size])
    return cols


def sig_to_logsig(sig_hybrid: torch.Tensor, depth: int, d: int, top_size: Optional[int] = None,
                  top_codes: Optional[Sequence[int]] = None):
    """Counterpart of the op `pathsig::sig_to_logsig` on the hybrid layout.

    Returns (logsig, P_arr) with P_arr[..., idx * depth + (m - 1)] = P_m(word idx), zero for m above the
    word's length (`sig_kernels.cu:184,215-216,237`).  Differentiable w.r.t. `sig_hybrid`.
    """
    offs = dense_level_offsets(d, depth)
    if top_size is None:
        top_size = d ** depth
    cols = hybrid_columns(d, depth, top_size, top_codes)
    lead = sig_hybrid.shape[:-1]
    low = offs[depth]
    # Dense layout with the lower levels copied and the top level left at zero: a level-`depth` word is
    # the prefix or suffix of no other word, so only P_1 of the top level needs the top coefficients,
    # and P_1 is the coefficient itself.  Columns may repeat (the planner does not de-duplicate).
    dense = torch.cat([sig_hybrid[..., :low], torch.zeros(*lead, d ** depth, dtype=sig_hybrid.dtype)], dim=-1)
    S = split_levels(dense, d, depth)
    P = tensor_log_powers(S, depth)
    logd = torch.cat(tensor_log_levels(S, depth), dim=-1)
    colt = torch.tensor(cols, dtype=torch.int64)
    top_only = torch.cat([torch.zeros(*lead, low, dtype=sig_hybrid.dtype), sig_hybrid[..., low:]], dim=-1)
    logsig = logd.index_select(-1, colt) + top_only
    Pm = [torch.cat(P[m - 1], dim=-1).index_select(-1, colt) for m in range(1, depth + 1)]
    Pm[0] = Pm[0] + top_only
    P_arr = torch.stack(Pm, dim=-1).reshape(*lead, -1)
    return logsig, P_arr


def logsig_power_cache(logsig_hybrid: torch.Tensor, depth: int, d: int, top_size: Optional[int] = None,
                       top_codes: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Cache of the keeping forward (`pathsig_logsig_forward_keep`; no counterpart in the reference): with
    L = log S, cache[..., idx * depth + (k - 1)] = level-|w| part of L^(x)k at word idx (entry 0 is L itself),
    zero for k above the word's length, except that a word w below the top level carries in entry |w|
    (k = |w| + 1) the sum -sum_{m=1}^{|w|} (L^(x)m)(w) / (m + 1)!, the weight with which w enters the top-level
    sums of the adjoint as a prefix.  Built here from plain truncated tensor products of L.  (The library leaves
    the rows of top-level words unwritten; here they hold the powers.)"""
    import math
    offs = dense_level_offsets(d, depth)
    if top_size is None:
        top_size = d ** depth
    cols = hybrid_columns(d, depth, top_size, top_codes)
    lead = logsig_hybrid.shape[:-1]
    low = offs[depth]
    # the top level of L enters no product that stays within `depth` letters
    dense = torch.cat([logsig_hybrid[..., :low], torch.zeros(*lead, d ** depth, dtype=logsig_hybrid.dtype)], dim=-1)
    L = split_levels(dense, d, depth)
    powers = [L]
    for _ in range(2, depth + 1):
        powers.append(tensor_product_levels(powers[-1], L, depth, a0=0.0, b0=0.0))
    colt = torch.tensor(cols, dtype=torch.int64)
    Q = [torch.cat(pw, dim=-1).index_select(-1, colt) for pw in powers]
    Q[0] = logsig_hybrid
    out = torch.stack(Q, dim=-1).clone()                       # [..., S, depth]
    for n in range(1, depth):                                   # words of length n < depth: entry n
        lo, hi = offs[n], offs[n + 1]
        out[..., lo:hi, n] = -sum(Q[m - 1][..., lo:hi] / math.factorial(m + 1) for m in range(1, n + 1))
    return out.reshape(*lead, -1)


# ----------------------------------------------------------------------------------------------
# gradients by autograd (the adjoint the reference codes by hand in
# `backward/sig_backward_kernels.cu:61-343,347-377,381-477`)
# ----------------------------------------------------------------------------------------------
def signature_vjp(path, grad_out, depth, level_sizes=None, codes=None, windows=None) -> torch.Tensor:
    x = path.detach().clone().requires_grad_(True)
    out = compute_signature(x, depth, level_sizes, codes, windows)
    (g,) = torch.autograd.grad(out, x, grad_out)
    return g


def logsig_vjp(sig_hybrid, grad_logsig, depth, d, top_size=None, top_codes=None) -> torch.Tensor:
    s = sig_hybrid.detach().clone().requires_grad_(True)
    logsig, _ = sig_to_logsig(s, depth, d, top_size, top_codes)
    (g,) = torch.autograd.grad(logsig, s, grad_logsig)
    return g
