"""Launchers: the same four names and argument meaning as the forward launchers
of the reference (``grouped_mm_bf16/kernels.py:524-717``) -- each writes into a
caller-allocated ``out`` and returns None -- but they hand raw pointers, sizes
and strides to the gfx950 kernels behind the C ABI instead of JIT-compiling
Triton.  ``out.dtype`` selects the epilogue (input dtype or float32), as the
reference's ``OUT_DTYPE=_as_tl_dtype(out.dtype)`` does.

The launch itself is registered as the torch custom op
``grouped_mm_bf16_amd::launch`` (mutating ``out``) so that it is visible to
torch's dispatcher and tracing; it runs on the current stream of the operands'
device and never synchronises.
"""
from __future__ import annotations

import contextlib
from typing import Optional

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16, torch.float32: _lib.DT_F32}

V_2D3D, V_3D3D, V_2D2D, V_3D2D = 0, 1, 2, 3


def _dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError(f"Unsupported dtype: {dtype}") from None


def _require_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("grouped_mm_bf16 is GPU-only (CUDA/HIP); CPU tensors are not supported")


# One workspace per (device, stream): launches on one stream run one after the other, so they can share it;
# launches on different streams may overlap and must not.  Allocated on first use and kept (the library leaves
# the arrival counters at its head zero after every launch).
_workspaces: dict = {}


def workspace(device: torch.device, stream: int):
    """(pointer, bytes) of the split workspace for launches on `stream` of `device`, or (None, 0) when none
    can be had: inside a stream capture no new workspace is allocated (a captured allocation would belong to
    the graph's memory pool), so a stream first used under capture launches without one."""
    key = (device.index, stream)
    ws = _workspaces.get(key)
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            return None, 0
        nbytes = _lib.load().gmm_workspace_bytes()
        if nbytes <= 0:
            return None, 0
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws.data_ptr(), ws.numel()


def _launch_now(variant: int, a: torch.Tensor, b: torch.Tensor, offs: Optional[torch.Tensor],
                out: torch.Tensor) -> None:
    lib = _lib.load()
    _require_gpu(a, b, offs, out)
    in_dt, out_dt = _dtype_code(a.dtype), _dtype_code(out.dtype)
    # the device guard costs microseconds; only switch when the tensors live on another device
    guard = torch.cuda.device(a.device) if a.device.index != torch.cuda.current_device() else contextlib.nullcontext()
    with guard:
        stream = torch.cuda.current_stream().cuda_stream
        pa, pb, po = a.data_ptr(), b.data_ptr(), out.data_ptr()
        poffs = offs.data_ptr() if offs is not None else None
        ws, ws_bytes = workspace(a.device, stream)
        if variant == V_2D3D:
            rc = lib.gmm_2d3d(pa, pb, po, poffs, offs.numel(), a.size(0), b.size(2), a.size(1),
                              a.stride(0), a.stride(1), b.stride(0), b.stride(1), b.stride(2),
                              out.stride(0), out.stride(1), in_dt, out_dt, ws, ws_bytes, stream)
        elif variant == V_3D3D:
            rc = lib.gmm_3d3d(pa, pb, po, a.size(0), a.size(1), b.size(2), a.size(2),
                              a.stride(0), a.stride(1), a.stride(2), b.stride(0), b.stride(1), b.stride(2),
                              out.stride(0), out.stride(1), out.stride(2), in_dt, out_dt, ws, ws_bytes, stream)
        elif variant == V_2D2D:
            rc = lib.gmm_2d2d(pa, pb, po, poffs, offs.numel(), a.size(0), b.size(1), a.size(1),
                              a.stride(0), a.stride(1), b.stride(0), b.stride(1),
                              out.stride(0), out.stride(1), out.stride(2), in_dt, out_dt, ws, ws_bytes, stream)
        elif variant == V_3D2D:
            rc = lib.gmm_3d2d(pa, pb, po, poffs, offs.numel(), a.size(1), b.size(1), a.size(2),
                              a.stride(0), a.stride(1), a.stride(2), b.stride(0), b.stride(1),
                              out.stride(0), out.stride(1), in_dt, out_dt, ws, ws_bytes, stream)
        else:
            raise RuntimeError(f"unknown variant {variant}")
    _lib.check(rc, "grouped_mm launch")


# The launch as a torch custom op (mutates `out`), for callers that trace or compile.  Eager calls skip
# the dispatcher, which costs more than the kernel for small products.
_launch_op = torch.library.custom_op("grouped_mm_bf16_amd::launch", mutates_args=("out",))(_launch_now)


@_launch_op.register_fake
def _launch_fake(variant, a, b, offs, out) -> None:
    """Shape propagation under FakeTensor: the op returns nothing and only fills `out`."""
    return None


def _launch(variant: int, a: torch.Tensor, b: torch.Tensor, offs: Optional[torch.Tensor], out: torch.Tensor) -> None:
    if torch.compiler.is_compiling():
        _launch_op(variant, a, b, offs, out)
    else:
        _launch_now(variant, a, b, offs, out)


def grouped_mm_3d3d(mat_a: torch.Tensor, mat_b: torch.Tensor, out: torch.Tensor) -> None:
    """out[g] = mat_a[g] @ mat_b[g]  (reference ``kernels.py:524-550``)."""
    if mat_a.size(0) != mat_b.size(0):
        raise RuntimeError("batched dimension has to match")
    _launch(V_3D3D, mat_a, mat_b, None, out)


def grouped_mm_2d2d(mat_a: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor, out: torch.Tensor) -> None:
    """out[g] = mat_a[:, s_g:e_g] @ mat_b[s_g:e_g, :], zeros for an empty group
    (reference ``kernels.py:553-580``)."""
    _launch(V_2D2D, mat_a, mat_b, offs, out)


def grouped_mm_2d3d(mat_a: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor, out: torch.Tensor) -> None:
    """out[s_g:e_g] = mat_a[s_g:e_g] @ mat_b[g]  (reference ``kernels.py:583-686``)."""
    if offs.numel() != mat_b.size(0):
        raise RuntimeError("matrix batch sizes have to match")
    if mat_a.size(0) == 0 or mat_b.size(2) == 0:
        return
    _launch(V_2D3D, mat_a, mat_b, offs, out)


def grouped_mm_3d2d(mat_a: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor, out: torch.Tensor) -> None:
    """out[:, s_g:e_g] = mat_a[g] @ mat_b[:, s_g:e_g]  (reference ``kernels.py:689-717``)."""
    if offs.numel() != mat_a.size(0):
        raise RuntimeError("matrix batch sizes have to match")
    _launch(V_3D2D, mat_a, mat_b, offs, out)


# ---- test / tuning hooks ---------------------------------------------------- #
@contextlib.contextmanager
def forced_path(path: str):
    """Force a kernel family ("auto", "generic" or "mfma") inside the block.

    The reference's tests force tile sizes through environment variables
    (``tests/test_grouped_mm.py:388-394``); this is the equivalent hook here.
    """
    code = {"auto": _lib.PATH_AUTO, "generic": _lib.PATH_GENERIC, "mfma": _lib.PATH_MFMA}[path]
    lib = _lib.load()
    prev = lib.gmm_set_path(code)
    try:
        yield
    finally:
        lib.gmm_set_path(prev)


@contextlib.contextmanager
def forced_mfma_config(config: int):
    lib = _lib.load()
    prev = lib.gmm_set_mfma_config(config)
    try:
        yield
    finally:
        lib.gmm_set_mfma_config(prev)


@contextlib.contextmanager
def forced_tile_heights(tall: int, shrt: int):
    """Force the tile heights of the assembly tile (tall 256 / 128, short 64 / 0; -1 = automatic)."""
    lib = _lib.load()
    prev = lib.gmm_set_tile_heights(tall, shrt)   # ((tall + 1) << 16) | (short + 1) of the previous setting
    try:
        yield
    finally:
        lib.gmm_set_tile_heights((prev >> 16) - 1, (prev & 0xffff) - 1)


@contextlib.contextmanager
def tail_split(on: bool):
    """Inside the block launches do (True) or do not (False) cut the tiles of a sparse last round along the
    contraction.  A cut tile adds its fp32 partial sums in a fixed order, so results are reproducible either
    way, but they differ in the last bit from the uncut tile's: tests that compare two launches bit for bit
    across different tile lists switch the split off."""
    lib = _lib.load()
    prev = lib.gmm_set_tail_split(1 if on else 0)
    try:
        yield
    finally:
        lib.gmm_set_tail_split(prev)


def last_path() -> str:
    """Kernel family used by this thread's last launch: "generic", "mfma" or "none"."""
    return {0: "none", _lib.PATH_GENERIC: "generic", _lib.PATH_MFMA: "mfma"}[_lib.load().gmm_last_path()]
