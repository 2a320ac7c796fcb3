"""CPU oracle for the mixture-of-experts step around grouped_mm: TEST INFRASTRUCTURE ONLY.

Never imported by the product package; only tests, the smoke check and the benchmark's CPU leg use it.

The reference holds no code for this step.  What it does hold is the recipe its benchmark uses to prepare
a 2D x 3D problem: expert indices per (token, choice) -> ``bincount`` -> ``cumsum`` -> int32 ``offs``, rows
sorted by expert (``bench/bench_2d3d.py:124-149``).  This module restates that recipe with torch's CPU
library routines and adds the layer arithmetic around it:

* ``route``           top-k by a stable descending sort (ties: lower expert first), softmax weights, stable
                      sort of the slots by expert, ``offs = bincount.cumsum`` (the benchmark's recipe).
* ``activation``      silu / swiglu in fp32, one rounding.
* ``moe_forward``     gather -> grouped_mm oracle (up) -> activation -> grouped_mm oracle (down) -> weighted
                      sum per token; rounded to the input dtype after each stage, as the device path does.
* ``moe_dense``       a separate formulation that pins the above: one token at a time, experts found by
                      repeated arg-max with masking, fp64 arithmetic, no sort, no offs, no intermediate rounding.

How each function is pinned (tests/test_moe_oracle.py): ``route`` against a pure-Python selection and
placement loop and against permutation invariants; ``moe_forward`` against ``moe_dense`` (tightly with
fp32 inputs, where the intermediate roundings vanish) and against hand-computed one-expert cases that
reduce to two plain matrix products.
"""
from __future__ import annotations

from typing import NamedTuple

import torch

from . import grouped_mm_oracle as gmm


class Routing(NamedTuple):
    offs: torch.Tensor          # int32 [E]
    slot_expert: torch.Tensor   # int32 [T * k]
    slot_weight: torch.Tensor   # float32 [T * k]
    row_token: torch.Tensor     # int32 [T * k]
    token_rows: torch.Tensor    # int32 [T * k]


def route(logits: torch.Tensor, top_k: int, renormalize: bool = True) -> Routing:
    T, E = logits.shape
    lf = logits.float()
    order = torch.sort(lf, dim=-1, descending=True, stable=True)
    chosen = order.indices[:, :top_k]                                   # [T, k], descending, ties -> lower index
    probs = torch.softmax(lf, dim=-1)
    # a row whose maximum is infinite (a +inf logit, or every logit -inf): the softmax's limit, all weight in
    # equal shares on the entries that equal the maximum (torch.softmax itself returns NaN there)
    top = lf.max(dim=-1, keepdim=True).values
    at_top = (lf == top).float()
    probs = torch.where(torch.isinf(top), at_top / at_top.sum(dim=-1, keepdim=True), probs)
    w = torch.gather(probs, 1, chosen)
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    flat = chosen.reshape(-1)
    perm = torch.sort(flat, stable=True).indices                        # rows: slots sorted by expert, stably
    token_rows = torch.empty_like(perm)
    token_rows[perm] = torch.arange(perm.numel())
    counts = torch.bincount(flat, minlength=E)
    offs = counts.cumsum(0).to(torch.int32)                             # bench/bench_2d3d.py:136-138
    return Routing(offs, flat.to(torch.int32), w.reshape(-1).float(), (perm // top_k).to(torch.int32),
                   token_rows.to(torch.int32))


def activation(h: torch.Tensor, kind: str) -> torch.Tensor:
    hf = h.float()
    if kind == "silu":
        return torch.nn.functional.silu(hf).to(h.dtype)
    if kind == "swiglu":
        inner = h.shape[-1] // 2
        return (torch.nn.functional.silu(hf[..., :inner]) * hf[..., inner:]).to(h.dtype)
    raise ValueError(kind)


def interleave_gate_up(w_up: torch.Tensor) -> torch.Tensor:
    """Columns [gate_0..gate_{I-1} | up_0..up_{I-1}] -> per block of 128: 64 gates, then their 64 partners
    (written with index arithmetic, not with the reshape the package uses)."""
    n = w_up.shape[-1]
    inner = n // 2
    idx = torch.empty(n, dtype=torch.long)
    for c in range(n):
        blk, within = divmod(c, 128)
        idx[c] = blk * 64 + within if within < 64 else inner + blk * 64 + (within - 64)
    return w_up[..., idx]


def combine(y: torch.Tensor, r: Routing, tokens: int, top_k: int) -> torch.Tensor:
    rows = r.token_rows.long().reshape(tokens, top_k)
    w = r.slot_weight.reshape(tokens, top_k)
    acc = torch.zeros(tokens, y.shape[1], dtype=torch.float32)
    for j in range(top_k):                                              # in the order of j, fp32
        acc += w[:, j:j + 1] * y[rows[:, j]].float()
    return acc.to(y.dtype)


def moe_forward(x, logits, w_up, w_down, top_k: int, kind: str = "swiglu", renormalize: bool = True,
                routing: Routing | None = None, fused: bool = False) -> torch.Tensor:
    """w_up always in the plain [gate | up] layout.  fused: the activation sees the fp32 products (what the
    fused epilogue does); else the products are rounded to the input dtype first (separate kernels)."""
    r = routing if routing is not None else route(logits, top_k, renormalize)
    xs = x[r.row_token.long()]
    if fused:
        act = activation(gmm.grouped_mm(xs, w_up, r.offs, out_dtype=torch.float32), kind).to(x.dtype)
    else:
        act = activation(gmm.grouped_mm(xs, w_up, r.offs), kind)
    y = gmm.grouped_mm(act, w_down, r.offs)
    return combine(y, r, x.shape[0], top_k)


def moe_dense(x, logits, w_up, w_down, top_k: int, kind: str = "swiglu", renormalize: bool = True) -> torch.Tensor:
    """Token by token in fp64 (small sizes only)."""
    T, E = logits.shape
    out = torch.zeros(T, w_down.shape[2], dtype=torch.float64)
    for t in range(T):
        v = logits[t].double().tolist()
        left = list(range(E))
        picked = []
        for _ in range(top_k):
            best = left[0]
            for e in left[1:]:
                if v[e] > v[best]:
                    best = e
            picked.append(best)
            left.remove(best)
        m = max(v)
        ex = [pow(2.718281828459045, vi - m) for vi in v]
        den = sum(ex[e] for e in picked) if renormalize else sum(ex)
        for e in picked:
            h = x[t].double() @ w_up[e].double()
            if kind == "swiglu":
                inner = h.numel() // 2
                g, u = h[:inner], h[inner:]
                a = g / (1 + torch.exp(-g)) * u
            else:
                a = h / (1 + torch.exp(-h))
            out[t] += (ex[e] / den) * (a @ w_down[e].double())
    return out
