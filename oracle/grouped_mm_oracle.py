"""CPU oracle for grouped_mm: TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, what the reference's forward path computes
so that the HIP kernels can be checked against it.  It is never imported by the
product package: only tests, the smoke check and the benchmark's CPU-baseline
leg use it.

What it follows (reference citations, relative to the reference tree):

* ``upper_bound``        -> ``grouped_mm_bf16/kernels.py:162-172``
  (first g with offs[g] > idx, i.e. searchsorted(offs, idx, right=True)).
* ``grouped_mm_2d3d``    -> ``kernels.py:304-419`` (row ownership) and the
  reference test's per-group loop ``tests/test_grouped_mm.py:56-66``.
* ``grouped_mm_3d3d``    -> ``kernels.py:197-245`` / ``tests/test_grouped_mm.py:27``.
* ``grouped_mm_2d2d``    -> ``kernels.py:248-301`` (K segment per group, exact
  zeros for an empty group) / ``tests/test_grouped_mm.py:93-105``.
* ``grouped_mm_3d2d``    -> ``kernels.py:475-521`` / ``tests/test_grouped_mm.py:133-144``.
* ``grouped_mm``         -> dispatch on operand rank, ``api.py:191-214``, with
  the K==0 -> zeros short-cut of ``api.py:192-212``.

Arithmetic: every product is formed from fp32 copies of the operands with one
``torch.matmul`` per group (fp32 accumulate) and rounded once, to nearest even,
to the output dtype.  Elements that no group owns (rows / columns at or beyond
``offs[-1]``) are left at ``fill`` (NaN by default) so a test can tell "not
written" from "written".

How each function is pinned (see tests/test_oracle.py): against torch's own CPU
``torch.nn.functional.grouped_mm`` (a library routine, bit-equal on aligned
shapes), against a brute-force fp64 triple loop written in C
(oracle/oracle_bruteforce.c), against the committed golden vectors in
tests/golden/, and through invariants (group permutation, group splitting,
3D*3D == uniform 2D*3D, sum over groups of 2D*2D == A@B).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch


# --------------------------------------------------------------------------- #
# integer part: the group lookup
# --------------------------------------------------------------------------- #
def upper_bound(offs: Sequence[int], idx: int) -> int:
    """First g with offs[g] > idx; len(offs) if there is none.

    Follows the fixed-depth binary search of kernels.py:162-172 (low/high/mid,
    `go_left = idx < offs[mid]`), written as an ordinary loop.
    """
    lo, hi = 0, len(offs)
    while lo < hi:
        mid = (lo + hi) // 2
        if idx < int(offs[mid]):
            hi = mid
        else:
            lo = mid + 1
    return lo


def group_ranges(offs: Sequence[int]) -> List[tuple]:
    """[(start_g, end_g)] with start_0 = 0 and start_g = offs[g-1]."""
    out = []
    start = 0
    for e in offs:
        e = int(e)
        out.append((start, e))
        start = e
    return out


# --------------------------------------------------------------------------- #
# floating-point part
# --------------------------------------------------------------------------- #
def _mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.matmul(a.to(torch.float32), b.to(torch.float32))


def _empty(shape, out_dtype, fill) -> torch.Tensor:
    return torch.full(shape, fill, dtype=out_dtype)


def grouped_mm_2d3d(a, b, offs, out_dtype=None, fill=float("nan")) -> torch.Tensor:
    """out[s_g:e_g] = A[s_g:e_g] @ B[g] for every non-empty group."""
    out_dtype = out_dtype or a.dtype
    out = _empty((a.shape[0], b.shape[2]), out_dtype, fill)
    for g, (s, e) in enumerate(group_ranges(offs.tolist())):
        if e > s:
            out[s:e] = _mm(a[s:e], b[g]).to(out_dtype)
    return out


def grouped_mm_3d3d(a, b, out_dtype=None) -> torch.Tensor:
    """out[g] = A[g] @ B[g]."""
    out_dtype = out_dtype or a.dtype
    out = torch.empty((a.shape[0], a.shape[1], b.shape[2]), dtype=out_dtype)
    for g in range(a.shape[0]):
        out[g] = _mm(a[g], b[g]).to(out_dtype)
    return out


def grouped_mm_2d2d(a, b, offs, out_dtype=None) -> torch.Tensor:
    """out[g] = A[:, s_g:e_g] @ B[s_g:e_g, :]; exact zeros for an empty group."""
    out_dtype = out_dtype or a.dtype
    G = offs.numel()
    out = torch.zeros((G, a.shape[0], b.shape[1]), dtype=out_dtype)
    for g, (s, e) in enumerate(group_ranges(offs.tolist())):
        if e > s:
            out[g] = _mm(a[:, s:e], b[s:e, :]).to(out_dtype)
    return out


def grouped_mm_3d2d(a, b, offs, out_dtype=None, fill=float("nan")) -> torch.Tensor:
    """out[:, s_g:e_g] = A[g] @ B[:, s_g:e_g] for every non-empty group."""
    out_dtype = out_dtype or a.dtype
    out = _empty((a.shape[1], b.shape[1]), out_dtype, fill)
    for g, (s, e) in enumerate(group_ranges(offs.tolist())):
        if e > s:
            out[:, s:e] = _mm(a[g], b[:, s:e]).to(out_dtype)
    return out


def grouped_mm(a, b, offs: Optional[torch.Tensor] = None, out_dtype=None,
               fill=float("nan")) -> torch.Tensor:
    """Rank dispatch of api.py:191-214 (no validation: the oracle trusts its caller)."""
    a = a.detach().cpu()
    b = b.detach().cpu()
    if offs is not None:
        offs = offs.detach().cpu()
    a2, b2 = a.dim() == 2, b.dim() == 2
    if not a2 and not b2:
        return grouped_mm_3d3d(a, b, out_dtype)
    if a2 and b2:
        return grouped_mm_2d2d(a, b, offs, out_dtype)
    if a2:
        return grouped_mm_2d3d(a, b, offs, out_dtype, fill)
    return grouped_mm_3d2d(a, b, offs, out_dtype, fill)


# --------------------------------------------------------------------------- #
# comparison helper: the graded tolerance
# --------------------------------------------------------------------------- #
RTOL = 1.6e-2


def atol_for_k(k: int) -> float:
    """atol = 1e-2 * sqrt(K / 64), K = contraction length of the compared elements."""
    return 1e-2 * math.sqrt(max(int(k), 0) / 64.0)


def assert_close(actual: torch.Tensor, expected: torch.Tensor, k: int, what: str = "") -> None:
    """Compare where the oracle wrote a value; NaN in `expected` means "unowned"."""
    actual = actual.detach().cpu().to(torch.float32)
    expected = expected.detach().cpu().to(torch.float32)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    owned = ~torch.isnan(expected)
    torch.testing.assert_close(actual[owned], expected[owned], rtol=RTOL, atol=atol_for_k(k),
                               msg=lambda m: f"{what}: {m}")


def assert_close_grouped(actual: torch.Tensor, expected: torch.Tensor, a, b, offs, what: str = "") -> None:
    """`assert_close` with K taken per element: the contraction length of the element's own group.
    Only the K-grouped variant (2-D x 2-D) has groups with different K; the others use the shared K."""
    if a.dim() == 2 and b.dim() == 2:
        for g, (s, e) in enumerate(group_ranges(offs.tolist())):
            assert_close(actual[g], expected[g], e - s, what=f"{what} group {g} (K={e - s})")
    else:
        assert_close(actual, expected, a.shape[-1], what=what)
