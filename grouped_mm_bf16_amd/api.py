"""Public entry point: ``grouped_mm(mat_a, mat_b, offs=None, bias=None, out_dtype=None)``.

Host layer of the MI355X grouped matrix multiply.  It reproduces the rule set of
the reference's ``grouped_mm_bf16/api.py`` (same checks, same order, same
``RuntimeError`` texts) so that callers can switch without changes, and hands
the arithmetic to hand-written gfx950 kernels through the launchers in
``kernels.py``.  There is no CPU or eager fallback: without the HIP library the
call raises.

Reference behaviour followed (paths relative to the reference tree):

* rule order and messages ......... ``api.py:61-122``
* row-/column-major stride test ... ``api.py:31-51``
* out_dtype must equal a.dtype .... ``api.py:54-58``
* output shapes and G checks ...... ``api.py:125-154`` (ROCm branch)
* short-cuts (numel==0, K==0) ..... ``api.py:188-212``
* rank dispatch ................... ``api.py:191-214``
* autograd backward ............... ``api.py:216-272`` (built here by composing
  the four forward variants on transposed views)
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import kernels as _k

_FLOAT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


class Checked(NamedTuple):
    """Outcome of the rule set: which operands are 2-D and the output dtype."""

    a_is_2d: bool
    b_is_2d: bool
    out_dtype: torch.dtype


def is_row_major(mat) -> bool:
    """True for a row-major matrix, False for a column-major one, else raise.

    Only the last two dimensions count; a batch stride is unconstrained and no
    alignment is asked for (reference ``api.py:31-51``).
    """
    nd = mat.dim()
    if nd not in (2, 3):
        raise RuntimeError(f"mat must be 2D or 3D, got dim={nd}")
    rows, cols = mat.size(nd - 2), mat.size(nd - 1)
    s_row, s_col = mat.stride(nd - 2), mat.stride(nd - 1)
    if s_col == 1 and s_row >= max(1, cols):
        return True
    if s_row == 1 and s_col >= max(1, rows):
        return False
    raise RuntimeError(
        f"Invalid strides/sizes, got {tuple(mat.stride())} for strides and {tuple(mat.size())} for sizes"
    )


def resolve_out_dtype(mat_a, out_dtype: Optional[torch.dtype]) -> torch.dtype:
    chosen = mat_a.dtype if out_dtype is None else out_dtype
    if chosen != mat_a.dtype:
        raise RuntimeError("Grouped gemm output dtype must match `mat_a` dtype")
    return chosen


def validate_inputs(mat_a, mat_b, offs, bias, out_dtype) -> Checked:
    """Every rule of reference ``api.py:61-122``, in that order."""
    for name, mat in (("mat_a", mat_a), ("mat_b", mat_b)):
        if mat.dtype not in _FLOAT_DTYPES:
            raise RuntimeError(
                f"Expected {name} to be Float32, BFloat16 or Float16 matrix, got {mat.dtype}"
            )
    for name, mat in (("mat_a", mat_a), ("mat_b", mat_b)):
        if mat.dim() not in (2, 3):
            raise RuntimeError(f"{name} has to be 2 or 3d")
    if mat_a.dtype != mat_b.dtype:
        raise RuntimeError("mat_a and mat_b must have the same dtype")

    a_is_2d, b_is_2d = mat_a.dim() == 2, mat_b.dim() == 2
    k_of_b = mat_b.size(0) if (a_is_2d and b_is_2d) else mat_b.size(-2)
    if mat_a.size(-1) != k_of_b:
        raise RuntimeError("contraction dimension of mat_a and mat_b must match")

    if not (mat_a.is_cuda and mat_b.is_cuda):
        raise RuntimeError("grouped_mm_bf16 is GPU-only (CUDA/HIP); CPU tensors are not supported")
    if mat_a.device != mat_b.device:
        raise RuntimeError("mat_a and mat_b must be on the same device")

    is_row_major(mat_a)
    is_row_major(mat_b)

    needs_offs = a_is_2d or b_is_2d
    if (offs is not None) != needs_offs:
        raise RuntimeError(
            "Have to provide offsets if there is a 2d matrix, or no offset if both matrices are 3d"
        )
    if offs is not None:
        if not offs.is_cuda:
            raise RuntimeError("offs must be a CUDA/HIP tensor (CPU offs are not supported)")
        if offs.device != mat_a.device:
            raise RuntimeError("offs must be on the same device as inputs")
        if offs.dim() != 1:
            raise RuntimeError("offs has to be 1D")
        if offs.dtype != torch.int32:
            raise RuntimeError("Offsets have to be int32")
        if offs.numel() >= 1024:
            raise RuntimeError("Can't process more than 1024 groups")

    if bias is not None:
        raise RuntimeError("Bias not supported yet")

    return Checked(a_is_2d, b_is_2d, resolve_out_dtype(mat_a, out_dtype))


def output_shape(mat_a, mat_b, offs) -> tuple:
    """Output size per variant with the group-count checks of reference ``api.py:134-149``."""
    a_is_2d, b_is_2d = mat_a.dim() == 2, mat_b.dim() == 2
    if a_is_2d and b_is_2d:
        return (offs.size(0), mat_a.size(0), mat_b.size(1))
    if a_is_2d:
        if offs.size(0) != mat_b.size(0):
            raise RuntimeError("matrix batch sizes have to match")
        return (mat_a.size(0), mat_b.size(-1))
    if b_is_2d:
        if offs.size(0) != mat_a.size(0):
            raise RuntimeError("matrix batch sizes have to match")
        return (mat_a.size(1), mat_b.size(1))
    if mat_a.size(0) != mat_b.size(0):
        raise RuntimeError("batched dimension has to match")
    return (mat_a.size(0), mat_a.size(1), mat_b.size(-1))


def create_output(mat_a, mat_b, offs, out_dtype) -> torch.Tensor:
    """Contiguous, uninitialised output (reference ``api.py:153-154``)."""
    return torch.empty(output_shape(mat_a, mat_b, offs), device=mat_a.device, dtype=out_dtype)


def _forward(mat_a, mat_b, offs, out: torch.Tensor) -> torch.Tensor:
    """Short-cuts and rank dispatch of reference ``api.py:188-214``."""
    if out.numel() == 0:
        return out
    if mat_a.size(-1) == 0:
        return out.zero_()
    a_is_2d, b_is_2d = mat_a.dim() == 2, mat_b.dim() == 2
    if not a_is_2d and not b_is_2d:
        _k.grouped_mm_3d3d(mat_a, mat_b, out)
    elif a_is_2d and b_is_2d:
        _k.grouped_mm_2d2d(mat_a, mat_b, offs, out)
    elif a_is_2d:
        _k.grouped_mm_2d3d(mat_a, mat_b, offs, out)
    else:
        _k.grouped_mm_3d2d(mat_a, mat_b, offs, out)
    return out


def _t(x: torch.Tensor) -> torch.Tensor:
    return x.transpose(-2, -1)


class _GroupedMM(torch.autograd.Function):
    """Forward = validate, allocate, launch.  Backward = the same four forward
    variants applied to transposed views (column-major operands are first-class
    in the kernels' load path), replacing the eight bespoke backward kernels of
    reference ``kernels.py:720-1390``:

    =========  =============================  =============================
    forward    grad_a                         grad_b
    =========  =============================  =============================
    2D x 3D    2d3d(dC, B^T, offs)            2d2d(A^T, dC, offs)
    3D x 3D    3d3d(dC, B^T)                  3d3d(A^T, dC)
    2D x 2D    3d2d(dC, B^T, offs)            2d3d(A^T, dC, offs)
    3D x 2D    2d2d(dC, B^T, offs)            3d2d(A^T, dC, offs)
    =========  =============================  =============================
    """

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs, bias, out_dtype):
        checked = validate_inputs(mat_a, mat_b, offs, bias, out_dtype)
        out = create_output(mat_a, mat_b, offs, checked.out_dtype)
        ctx.has_offs = offs is not None
        ctx.save_for_backward(
            mat_a, mat_b,
            offs if offs is not None else torch.empty((), device=mat_a.device, dtype=torch.int32),
        )
        return _forward(mat_a, mat_b, offs, out)

    @staticmethod
    def backward(ctx, grad_out):
        mat_a, mat_b, offs = ctx.saved_tensors
        offs = offs if ctx.has_offs else None
        need_a, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if grad_out.numel() == 0 or mat_a.size(-1) == 0:
            return (torch.zeros_like(mat_a) if need_a else None,
                    torch.zeros_like(mat_b) if need_b else None, None, None, None)
        try:
            is_row_major(grad_out)
        except RuntimeError:
            grad_out = grad_out.contiguous()

        a_is_2d, b_is_2d = mat_a.dim() == 2, mat_b.dim() == 2
        grad_a = grad_b = None
        if need_a:
            # Elements of a jagged operand that no group owns get a zero gradient.
            jagged_a = (a_is_2d and not b_is_2d) or (a_is_2d and b_is_2d)
            grad_a = (torch.zeros if jagged_a else torch.empty)(
                mat_a.shape, device=mat_a.device, dtype=mat_a.dtype)
            if not a_is_2d and not b_is_2d:
                _k.grouped_mm_3d3d(grad_out, _t(mat_b), grad_a)
            elif a_is_2d and not b_is_2d:
                _k.grouped_mm_2d3d(grad_out, _t(mat_b), offs, grad_a)
            elif a_is_2d and b_is_2d:
                _k.grouped_mm_3d2d(grad_out, _t(mat_b), offs, grad_a)
            else:
                _k.grouped_mm_2d2d(grad_out, _t(mat_b), offs, grad_a)
        if need_b:
            jagged_b = b_is_2d
            grad_b = (torch.zeros if jagged_b else torch.empty)(
                mat_b.shape, device=mat_b.device, dtype=mat_b.dtype)
            if not a_is_2d and not b_is_2d:
                _k.grouped_mm_3d3d(_t(mat_a), grad_out, grad_b)
            elif a_is_2d and not b_is_2d:
                _k.grouped_mm_2d2d(_t(mat_a), grad_out, offs, grad_b)
            elif a_is_2d and b_is_2d:
                _k.grouped_mm_2d3d(_t(mat_a), grad_out, offs, grad_b)
            else:
                _k.grouped_mm_3d2d(_t(mat_a), grad_out, offs, grad_b)
        return grad_a, grad_b, None, None, None


def grouped_mm(
    mat_a: torch.Tensor,
    mat_b: torch.Tensor,
    offs: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """``torch.nn.functional.grouped_mm`` semantics on MI355X (reference ``api.py:275-287``).

    =======  ================  ==============  ===============  ===============
    variant  mat_a             mat_b           offs (int32)     result
    =======  ================  ==============  ===============  ===============
    2D x 3D  ``[M_total, K]``  ``[G, K, N]``   ends along M     ``[M_total, N]``
    3D x 3D  ``[G, M, K]``     ``[G, K, N]``   must be None     ``[G, M, N]``
    2D x 2D  ``[M, K_total]``  ``[K_total,N]`` ends along K     ``[G, M, N]``
    3D x 2D  ``[G, M, K]``     ``[K,N_total]`` ends along N     ``[M, N_total]``
    =======  ================  ==============  ===============  ===============

    Rows / columns at or beyond ``offs[-1]`` are left uninitialised, as in the
    reference.  ``bias`` is rejected and ``out_dtype`` must equal the input dtype.
    """
    return _GroupedMM.apply(mat_a, mat_b, offs, bias, out_dtype)
