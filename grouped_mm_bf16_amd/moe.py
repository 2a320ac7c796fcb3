"""The mixture-of-experts step around the grouped product, entirely on the device:

    routing (top-k, weights, stable sort by expert -> offs)  ->  up projection with the token gather done
    by the tile's own copies  ->  SiLU / SwiGLU  ->  down projection  ->  weighted un-permute.

The reference ships the grouped product only; its benchmark prepares rows that are already sorted by expert
and gets ``offs`` from ``bincount(...).cumsum(0)`` with a host round trip (``bench/bench_2d3d.py:124-149``).
Here no count ever reaches the host: the kernels read ``offs`` from device memory, and every buffer is sized
by ``tokens * top_k``, which the host knows.

Forward only (inference); the functions take and return plain tensors.  Each one is also registered as a
torch custom op (``grouped_mm_bf16_amd::moe_route``, ``gathered``, ``swiglu``, ``activation``, ``combine``) and
dispatches to it while a model around it is being traced or compiled.
"""
from __future__ import annotations

import contextlib
from typing import NamedTuple

import torch

from . import _lib, kernels
from .kernels import _dtype_code, _require_gpu, grouped_mm_2d3d

ACTIVATIONS = {"silu": 0, "swiglu": 1}


class Routing(NamedTuple):
    """What :func:`moe_route` returns; S = tokens * top_k slots, slot t * top_k + j is choice j of token t."""
    offs: torch.Tensor          # int32 [E]  end offset of each expert's rows (what grouped_mm takes)
    slot_expert: torch.Tensor   # int32 [S]  expert of each slot
    slot_weight: torch.Tensor   # float32 [S] combine weight of each slot
    row_token: torch.Tensor     # int32 [S]  token whose activations row r of the sorted matrix holds
    token_rows: torch.Tensor    # int32 [S]  row of each slot (inverse permutation)


def _guard(t: torch.Tensor):
    return torch.cuda.device(t.device) if t.device.index != torch.cuda.current_device() else contextlib.nullcontext()


def _route_packed_now(router_logits: torch.Tensor, top_k: int, renormalize: bool) -> torch.Tensor:
    """The five routing results in one int32 buffer [E + 4 S] (offs, slot_expert, slot_weight bits, row_token,
    token_rows): one allocation for results and workspace (each allocation costs microseconds of host time)."""
    _require_gpu(router_logits)
    if router_logits.dim() != 2:
        raise RuntimeError("router_logits has to be 2D [tokens, experts]")
    if router_logits.size(0) and router_logits.stride(1) != 1:
        raise RuntimeError("router_logits must be contiguous along the experts")
    T, E = router_logits.shape
    if not 1 <= top_k <= min(E, 32):
        raise RuntimeError(f"top_k must be in [1, min(experts, 32)], got {top_k} for {E} experts")
    if E > 1023:
        raise RuntimeError("Can't process more than 1024 groups")
    lib = _lib.load()
    dev, S = router_logits.device, T * top_k
    ws_bytes = lib.gmm_moe_route_workspace_bytes(T, E, top_k)
    if ws_bytes < 0:
        raise RuntimeError("moe_route: sizes out of range")
    buf = torch.empty(E + 4 * S + ws_bytes // 4, device=dev, dtype=torch.int32)
    base, ws = buf.data_ptr(), buf[E + 4 * S:]
    with _guard(router_logits):
        rc = lib.gmm_moe_route(router_logits.data_ptr(), router_logits.stride(0) if T else E,
                               _dtype_code(router_logits.dtype), T, E, top_k, int(bool(renormalize)),
                               base, base + 4 * E, base + 4 * (E + S), base + 4 * (E + 2 * S), base + 4 * (E + 3 * S),
                               ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "moe_route")
    return buf[:E + 4 * S]


_route_op = torch.library.custom_op("grouped_mm_bf16_amd::moe_route", mutates_args=())(_route_packed_now)


@_route_op.register_fake
def _route_fake(router_logits, top_k, renormalize):
    T, E = router_logits.shape
    return router_logits.new_empty(E + 4 * T * top_k, dtype=torch.int32)


def moe_route(router_logits: torch.Tensor, top_k: int, renormalize: bool = True) -> Routing:
    """Top-k routing and the stable sort of the slots by expert.

    router_logits [T, E] (bf16, fp16 or fp32, last dimension contiguous).  Ties go to the lower expert index;
    weights are the softmax over the chosen logits (``renormalize``) or the chosen entries of the softmax
    over all experts.
    """
    impl = _route_op if torch.compiler.is_compiling() else _route_packed_now
    buf = impl(router_logits, top_k, bool(renormalize))
    E, S = router_logits.size(1), router_logits.size(0) * top_k
    parts = torch.split(buf, [E, S, S, S, S])
    return Routing(parts[0], parts[1], parts[2].view(torch.float32), parts[3], parts[4])


def _check_out(out: torch.Tensor, shape, like: torch.Tensor, what: str) -> None:
    """A caller-supplied output must be exactly what the call computes: the kernels write through a raw pointer."""
    if tuple(out.shape) != tuple(shape) or out.dtype != like.dtype or out.device != like.device:
        raise RuntimeError(f"{what}: out has to be {tuple(shape)} {like.dtype} on {like.device}, "
                           f"got {tuple(out.shape)} {out.dtype} on {out.device}")
    if out.dim() != 2 or (out.numel() and (out.stride(1) != 1 or out.stride(0) < out.size(1))):
        raise RuntimeError(f"{what}: out has to be row-major, got strides {tuple(out.stride())}")


def _no_out_when_compiling(out, what: str) -> None:
    if out is not None:
        raise RuntimeError(f"{what}: out= is not available under torch.compile (the traced ops allocate their results)")


def grouped_mm_gathered(a: torch.Tensor, row_index: torch.Tensor, b: torch.Tensor, offs: torch.Tensor,
                        out: torch.Tensor | None = None) -> torch.Tensor:
    """``grouped_mm(a[row_index], b, offs=offs)`` without materialising ``a[row_index]``.

    a [R_src, K], row_index int32 [M_total], b [G, K, N], offs int32 [G]; returns [M_total, N] in a's dtype.
    An index outside [0, R_src) reads a row of zeros.
    """
    if torch.compiler.is_compiling():
        _no_out_when_compiling(out, "grouped_mm_gathered")
        return _gathered_op(a, row_index, b, offs)
    return _gathered_now(a, row_index, b, offs, out)


def _gathered_now(a: torch.Tensor, row_index: torch.Tensor, b: torch.Tensor, offs: torch.Tensor,
                  out: torch.Tensor | None = None) -> torch.Tensor:
    _require_gpu(a, row_index, b, offs)
    if a.dim() != 2 or b.dim() != 3:
        raise RuntimeError("grouped_mm_gathered takes a 2D first and a 3D second operand")
    if a.dtype != b.dtype:
        raise RuntimeError("mat_a and mat_b must have the same dtype")
    if a.size(1) != b.size(1):
        raise RuntimeError("contraction dimension of mat_a and mat_b must match")
    if row_index.dtype != torch.int32 or row_index.dim() != 1 or not row_index.is_contiguous():
        raise RuntimeError("row_index has to be a contiguous 1D int32 tensor")
    if offs.dtype != torch.int32 or offs.dim() != 1 or not offs.is_contiguous():
        raise RuntimeError("Offsets have to be int32")
    if offs.numel() != b.size(0):
        raise RuntimeError("matrix batch sizes have to match")
    M, N = row_index.numel(), b.size(2)
    if out is None:
        out = torch.empty(M, N, device=a.device, dtype=a.dtype)
    else:
        _check_out(out, (M, N), a, "grouped_mm_gathered")
    if M == 0 or N == 0:
        return out
    if a.size(1) == 0:
        return out.zero_()
    lib = _lib.load()
    with _guard(a):
        stream = torch.cuda.current_stream().cuda_stream
        ws, ws_bytes = kernels.workspace(a.device, stream)
        rc = lib.gmm_2d3d_gather(a.data_ptr(), row_index.data_ptr(), b.data_ptr(), out.data_ptr(), offs.data_ptr(),
                                 offs.numel(), a.size(0), M, N, a.size(1), a.stride(0), a.stride(1),
                                 b.stride(0), b.stride(1), b.stride(2), out.stride(0), out.stride(1),
                                 _dtype_code(a.dtype), _dtype_code(out.dtype), ws, ws_bytes, stream)
    _lib.check(rc, "grouped_mm_gathered launch")
    return out


def _gathered_functional(a: torch.Tensor, row_index: torch.Tensor, b: torch.Tensor, offs: torch.Tensor) -> torch.Tensor:
    return _gathered_now(a, row_index, b, offs)


# The functions of this module as torch custom ops (functional: they allocate their result), for callers that
# trace or compile a model around them.  Eager calls skip the dispatcher.
_gathered_op = torch.library.custom_op("grouped_mm_bf16_amd::gathered", mutates_args=())(_gathered_functional)


@_gathered_op.register_fake
def _gathered_fake(a, row_index, b, offs):
    return a.new_empty(row_index.numel(), b.size(2))


def interleave_gate_up(w_up: torch.Tensor) -> torch.Tensor:
    """[E, H, 2I] with all gate columns first, then all partner ("up") columns  ->  the layout the fused SwiGLU
    epilogue wants: in every block of 128 columns, 64 gate columns followed by their 64 partners.  I must be a
    multiple of 64.  Done once, when the weights are loaded."""
    E, H, N = w_up.shape
    inner = N // 2
    if N % 128:
        raise RuntimeError("interleave_gate_up needs an inner size that is a multiple of 64")
    g = w_up[..., :inner].reshape(E, H, inner // 64, 1, 64)
    u = w_up[..., inner:].reshape(E, H, inner // 64, 1, 64)
    return torch.cat([g, u], dim=3).reshape(E, H, N).contiguous()


def grouped_mm_swiglu(a: torch.Tensor, row_index: torch.Tensor | None, b: torch.Tensor, offs: torch.Tensor,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """``swiglu(grouped_mm(a[row_index], b, offs))`` in one kernel, for ``b`` in the layout of
    :func:`interleave_gate_up`; the [M_total, N] intermediate is never written.  Returns [M_total, N / 2].
    Raises if the operands do not qualify for the fast path (see ``gmm_2d3d_swiglu`` in the C header)."""
    if torch.compiler.is_compiling():
        _no_out_when_compiling(out, "grouped_mm_swiglu")
        return _swiglu_op(a, row_index, b, offs)
    return _swiglu_now(a, row_index, b, offs, out)


def _swiglu_now(a: torch.Tensor, row_index: torch.Tensor | None, b: torch.Tensor, offs: torch.Tensor,
                out: torch.Tensor | None = None) -> torch.Tensor:
    _require_gpu(a, row_index, b, offs)
    if a.dim() != 2 or b.dim() != 3 or a.dtype != b.dtype or a.size(1) != b.size(1):
        raise RuntimeError("grouped_mm_swiglu takes a [R, K] and b [G, K, N] of one dtype")
    if row_index is not None and (row_index.dtype != torch.int32 or row_index.dim() != 1 or not row_index.is_contiguous()):
        raise RuntimeError("row_index has to be a contiguous 1D int32 tensor")
    if offs.dtype != torch.int32 or offs.dim() != 1 or offs.numel() != b.size(0) or not offs.is_contiguous():
        raise RuntimeError("offs has to be int32 [G]")
    M = row_index.numel() if row_index is not None else a.size(0)
    N = b.size(2)
    if out is None:
        out = torch.empty(M, N // 2, device=a.device, dtype=a.dtype)
    else:
        _check_out(out, (M, N // 2), a, "grouped_mm_swiglu")
    lib = _lib.load()
    with _guard(a):
        rc = lib.gmm_2d3d_swiglu(a.data_ptr(), row_index.data_ptr() if row_index is not None else None, b.data_ptr(),
                                 out.data_ptr(), offs.data_ptr(), offs.numel(), a.size(0), M, N, a.size(1),
                                 a.stride(0), a.stride(1), b.stride(0), b.stride(1), b.stride(2), out.stride(0), out.stride(1),
                                 _dtype_code(a.dtype), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "grouped_mm_swiglu launch")
    return out


def _swiglu_functional(a: torch.Tensor, row_index: torch.Tensor | None, b: torch.Tensor, offs: torch.Tensor) -> torch.Tensor:
    return _swiglu_now(a, row_index, b, offs)


_swiglu_op = torch.library.custom_op("grouped_mm_bf16_amd::swiglu", mutates_args=())(_swiglu_functional)


@_swiglu_op.register_fake
def _swiglu_fake(a, row_index, b, offs):
    return a.new_empty(row_index.numel() if row_index is not None else a.size(0), b.size(2) // 2)


def moe_activation(h: torch.Tensor, kind: str = "swiglu", out: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(h)`` or, for "swiglu", ``silu(h[:, :I]) * h[:, I:]`` with I = h.size(1) // 2 (fp32 arithmetic,
    one rounding).  h [R, I or 2I], bf16 or fp16, row-major."""
    if torch.compiler.is_compiling():
        _no_out_when_compiling(out, "moe_activation")
        return _activation_op(h, kind)
    return _activation_now(h, kind, out)


def _activation_now(h: torch.Tensor, kind: str = "swiglu", out: torch.Tensor | None = None) -> torch.Tensor:
    _require_gpu(h)
    if kind not in ACTIVATIONS:
        raise RuntimeError(f"unknown activation {kind!r}; have {sorted(ACTIVATIONS)}")
    code = ACTIVATIONS[kind]
    if h.dim() != 2 or (h.numel() and h.stride(1) != 1):
        raise RuntimeError("moe_activation takes a row-major 2D tensor")
    if code and h.size(1) % 2:
        raise RuntimeError("swiglu needs an even number of columns")
    inner = h.size(1) // 2 if code else h.size(1)
    if out is None:
        out = torch.empty(h.size(0), inner, device=h.device, dtype=h.dtype)
    else:
        _check_out(out, (h.size(0), inner), h, "moe_activation")
    lib = _lib.load()
    with _guard(h):
        rc = lib.gmm_moe_activation(h.data_ptr(), out.data_ptr(), h.size(0), inner, h.stride(0) if h.size(0) else inner,
                                    out.stride(0) if h.size(0) else inner, code, _dtype_code(h.dtype),
                                    torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "moe_activation")
    return out


def _activation_functional(h: torch.Tensor, kind: str) -> torch.Tensor:
    return _activation_now(h, kind)


_activation_op = torch.library.custom_op("grouped_mm_bf16_amd::activation", mutates_args=())(_activation_functional)


@_activation_op.register_fake
def _activation_fake(h, kind):
    return h.new_empty(h.size(0), h.size(1) // 2 if ACTIVATIONS.get(kind) else h.size(1))


def moe_combine(y: torch.Tensor, routing: Routing, tokens: int, top_k: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = sum_j slot_weight[t, j] * y[token_rows[t, j]] in fp32, rounded once.  y [S, H] row-major."""
    if torch.compiler.is_compiling():
        _no_out_when_compiling(out, "moe_combine")
        return _combine_op(y, routing.token_rows, routing.slot_weight, tokens, top_k)
    return _combine_now(y, routing.token_rows, routing.slot_weight, tokens, top_k, out)


def _combine_now(y: torch.Tensor, token_rows: torch.Tensor, slot_weight: torch.Tensor, tokens: int, top_k: int,
                 out: torch.Tensor | None = None) -> torch.Tensor:
    _require_gpu(y)
    if y.dim() != 2 or (y.numel() and y.stride(1) != 1):
        raise RuntimeError("moe_combine takes a row-major 2D tensor")
    H = y.size(1)
    slots = tokens * top_k
    for name, t, dt in (("token_rows", token_rows, torch.int32), ("slot_weight", slot_weight, torch.float32)):
        if t.dtype != dt or t.numel() != slots or not t.is_contiguous() or t.device != y.device:
            raise RuntimeError(f"moe_combine: routing.{name} has to be a contiguous {dt} tensor of tokens * top_k = {slots} "
                               f"elements on {y.device}, got {t.numel()} of {t.dtype} on {t.device}")
    if out is None:
        out = torch.empty(tokens, H, device=y.device, dtype=y.dtype)
    else:
        _check_out(out, (tokens, H), y, "moe_combine")
    lib = _lib.load()
    with _guard(y):
        rc = lib.gmm_moe_combine(y.data_ptr(), token_rows.data_ptr(), slot_weight.data_ptr(), out.data_ptr(),
                                 tokens, top_k, H, y.size(0), y.stride(0) if y.size(0) else H, out.stride(0) if tokens else H,
                                 _dtype_code(y.dtype), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "moe_combine")
    return out


def _combine_functional(y: torch.Tensor, token_rows: torch.Tensor, slot_weight: torch.Tensor, tokens: int, top_k: int) -> torch.Tensor:
    return _combine_now(y, token_rows, slot_weight, tokens, top_k)


_combine_op = torch.library.custom_op("grouped_mm_bf16_amd::combine", mutates_args=())(_combine_functional)


@_combine_op.register_fake
def _combine_fake(y, token_rows, slot_weight, tokens, top_k):
    return y.new_empty(tokens, y.size(1))


def moe_forward(x: torch.Tensor, router_logits: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, top_k: int,
                activation: str = "swiglu", renormalize: bool = True, interleaved: bool = False) -> torch.Tensor:
    """One mixture-of-experts feed-forward layer.

    x [T, H]; router_logits [T, E]; w_up [E, H, I] ("silu") or [E, H, 2I] ("swiglu": gate columns first, then
    up columns); w_down [E, I, H].  Returns [T, H] in x's dtype:
    ``sum_j weight[t, j] * (act(x[t] @ w_up[e_tj]) @ w_down[e_tj])``.
    Intermediate results are rounded to x's dtype after each of the three stages, as separate layers would.

    ``interleaved`` ("swiglu" only): ``w_up`` is in the layout of :func:`interleave_gate_up`; the activation then
    runs inside the up projection's epilogue on the fp32 products (one rounding less, no [S, 2I] intermediate).
    """
    if x.dim() != 2 or router_logits.dim() != 2 or x.size(0) != router_logits.size(0):
        raise RuntimeError("x [T, H] and router_logits [T, E] must agree on T")
    if w_up.dim() != 3 or w_down.dim() != 3 or w_up.size(0) != router_logits.size(1) or w_down.size(0) != w_up.size(0):
        raise RuntimeError("w_up [E, H, I or 2I] and w_down [E, I, H] must agree with router_logits on E")
    if activation not in ACTIVATIONS:
        raise RuntimeError(f"unknown activation {activation!r}; have {sorted(ACTIVATIONS)}")
    inner = w_up.size(2) // 2 if ACTIVATIONS[activation] else w_up.size(2)
    if w_up.size(1) != x.size(1) or w_down.size(1) != inner or w_down.size(2) != x.size(1):
        raise RuntimeError("weight shapes do not chain: x [T, H], w_up [E, H, I or 2I], w_down [E, I, H]")
    T = x.size(0)
    routing = moe_route(router_logits, top_k, renormalize)
    if interleaved:
        if activation != "swiglu":
            raise RuntimeError("interleaved weights go with the swiglu activation")
        act = grouped_mm_swiglu(x, routing.row_token, w_up, routing.offs)
    else:
        h = grouped_mm_gathered(x, routing.row_token, w_up, routing.offs)
        act = moe_activation(h, activation)
        del h
    y = torch.empty(act.size(0), w_down.size(2), device=x.device, dtype=x.dtype)
    grouped_mm_2d3d(act, w_down, routing.offs, y)   # rows are already sorted by expert
    del act
    return moe_combine(y, routing, T, top_k)

