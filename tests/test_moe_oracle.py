"""Pins oracle/moe_oracle.py (CPU only): routing against a pure-Python selection and placement loop and
its invariants; the layer arithmetic against the token-by-token fp64 formulation and against cases that
reduce to two plain matrix products."""
import math

import pytest
import torch

from oracle import moe_oracle as moe


def py_route(logits, k):
    """Selection and placement with Python lists only: no sort of tensors, no bincount."""
    T, E = len(logits), len(logits[0])
    slot_expert = []
    for t in range(T):
        ranked = sorted(range(E), key=lambda e: (-logits[t][e], e))
        slot_expert += ranked[:k]
    rows = sorted(range(T * k), key=lambda s: (slot_expert[s], s))
    token_rows = [0] * (T * k)
    for r, s in enumerate(rows):
        token_rows[s] = r
    counts = [0] * E
    for e in slot_expert:
        counts[e] += 1
    offs, run = [], 0
    for c in counts:
        run += c
        offs.append(run)
    return offs, slot_expert, [s // k for s in rows], token_rows


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (5, 3, 3), (37, 8, 2), (64, 128, 8), (200, 17, 5)])
@pytest.mark.parametrize("ties", [False, True])
def test_route_matches_python_lists(T, E, k, ties):
    gen = torch.Generator().manual_seed(T * 1000 + E * 10 + k)
    logits = torch.randn(T, E, generator=gen)
    if ties:
        logits = (logits * 2).round() / 2   # many equal values: ties must go to the lower expert index
    r = moe.route(logits, k)
    offs, slot_expert, row_token, token_rows = py_route(logits.tolist(), k)
    assert r.offs.tolist() == offs
    assert r.slot_expert.tolist() == slot_expert
    assert r.row_token.tolist() == row_token
    assert r.token_rows.tolist() == token_rows
    assert r.offs.dtype == r.slot_expert.dtype == r.row_token.dtype == r.token_rows.dtype == torch.int32


def test_route_invariants_and_weights():
    gen = torch.Generator().manual_seed(5)
    T, E, k = 300, 16, 4
    logits = torch.randn(T, E, generator=gen)
    r = moe.route(logits, k, renormalize=True)
    S = T * k
    assert sorted(r.token_rows.tolist()) == list(range(S))
    assert (r.row_token[r.token_rows.long()] == torch.arange(S) // k).all()
    row_expert = torch.empty(S, dtype=torch.int32)
    row_expert[r.token_rows.long()] = r.slot_expert
    assert (row_expert[1:] >= row_expert[:-1]).all()
    assert int(r.offs[-1]) == S
    # within one expert the rows keep the slot order (stable)
    inv = torch.empty(S, dtype=torch.long)
    inv[r.token_rows.long()] = torch.arange(S)
    for e in range(E):
        lo, hi = (0 if e == 0 else int(r.offs[e - 1])), int(r.offs[e])
        assert (inv[lo:hi][1:] > inv[lo:hi][:-1]).all()
    w = r.slot_weight.reshape(T, k)
    assert torch.allclose(w.sum(-1), torch.ones(T), atol=1e-6)
    assert (w[:, 1:] <= w[:, :-1] + 1e-7).all()   # choices come in descending order
    # closed form of the weights
    t = 11
    v = logits[t].double()
    chosen = r.slot_expert.reshape(T, k)[t].long()
    want = torch.exp(v[chosen]) / torch.exp(v[chosen]).sum()
    assert torch.allclose(w[t].double(), want, atol=1e-6)
    full = moe.route(logits, k, renormalize=False).slot_weight.reshape(T, k)
    want = torch.exp(v[chosen]) / torch.exp(v).sum()
    assert torch.allclose(full[t].double(), want, atol=1e-6)


def test_activation_known_values():
    h = torch.tensor([[0.0, 1.0, -1.0, 30.0, 2.0, 3.0, 4.0, 5.0]])
    s = moe.activation(h, "silu")
    assert s[0, 0] == 0 and abs(float(s[0, 1]) - 1 / (1 + math.exp(-1))) < 1e-6
    assert abs(float(s[0, 2]) + 1 / (1 + math.exp(1))) < 1e-6 and abs(float(s[0, 3]) - 30.0) < 1e-5
    g = moe.activation(h, "swiglu")   # gate columns first: silu(h[:4]) * h[4:]
    assert g.shape == (1, 4)
    assert torch.allclose(g, s[:, :4] * h[:, 4:])


@pytest.mark.parametrize("kind", ["silu", "swiglu"])
@pytest.mark.parametrize("renorm", [True, False])
def test_forward_matches_the_token_by_token_formulation(kind, renorm):
    gen = torch.Generator().manual_seed(9)
    T, H, I, E, k = 23, 24, 40, 5, 2
    x = torch.randn(T, H, generator=gen)
    logits = torch.randn(T, E, generator=gen)
    w_up = torch.randn(E, H, 2 * I if kind == "swiglu" else I, generator=gen) * 0.2
    w_down = torch.randn(E, I, H, generator=gen) * 0.2
    got = moe.moe_forward(x, logits, w_up, w_down, k, kind, renorm)
    want = moe.moe_dense(x, logits, w_up, w_down, k, kind, renorm)
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-4)
    # bf16: same routing (logits kept in fp32), results agree to the roundings of three stages
    got16 = moe.moe_forward(x.bfloat16(), logits, w_up.bfloat16(), w_down.bfloat16(), k, kind, renorm)
    want16 = moe.moe_dense(x.bfloat16(), logits, w_up.bfloat16(), w_down.bfloat16(), k, kind, renorm)
    assert torch.allclose(got16.double(), want16, rtol=3e-2, atol=3e-2)


def test_one_expert_reduces_to_two_products():
    gen = torch.Generator().manual_seed(10)
    x = torch.randn(9, 16, generator=gen)
    w_up, w_down = torch.randn(1, 16, 24, generator=gen), torch.randn(1, 24, 16, generator=gen)
    got = moe.moe_forward(x, torch.zeros(9, 1), w_up, w_down, 1, "silu")
    want = torch.nn.functional.silu(x @ w_up[0]) @ w_down[0]
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_permuting_experts_permutes_nothing_a_caller_sees():
    """Relabelling the experts (logit columns and weight slabs together) leaves the layer's output alone."""
    gen = torch.Generator().manual_seed(12)
    T, H, I, E, k = 31, 16, 24, 6, 3
    x, logits = torch.randn(T, H, generator=gen), torch.randn(T, E, generator=gen)
    w_up, w_down = torch.randn(E, H, 2 * I, generator=gen) * 0.2, torch.randn(E, I, H, generator=gen) * 0.2
    p = torch.randperm(E, generator=gen)
    a = moe.moe_forward(x, logits, w_up, w_down, k)
    b = moe.moe_forward(x, logits[:, p], w_up[p], w_down[p], k)
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-5)


def test_interleaved_layout_and_fused_rounding():
    """The gate/partner interleave: block b of 128 columns = gate columns 64 b .. 64 b + 63, then their
    partners; the package's reshape and the oracle's index arithmetic agree, and swiglu on the interleaved
    product, taken block by block, equals swiglu on the plain one."""
    from grouped_mm_bf16_amd.moe import interleave_gate_up
    w = torch.arange(2 * 3 * 256, dtype=torch.float32).reshape(2, 3, 256)   # I = 128: columns 0..127 gates, 128..255 partners
    il = moe.interleave_gate_up(w)
    assert torch.equal(il, interleave_gate_up(w))
    assert il[0, 0, :64].tolist() == list(range(0, 64)) and il[0, 0, 64:128].tolist() == list(range(128, 192))
    assert il[0, 0, 128:192].tolist() == list(range(64, 128)) and il[0, 0, 192:].tolist() == list(range(192, 256))
    gen = torch.Generator().manual_seed(3)
    h = torch.randn(5, 256, generator=gen)
    hi = moe.interleave_gate_up(h)
    blocks = hi.reshape(5, 2, 2, 64)
    fused = (torch.nn.functional.silu(blocks[:, :, 0]) * blocks[:, :, 1]).reshape(5, 128)
    assert torch.equal(fused, moe.activation(h, "swiglu"))
    # fused flag: same layer, one rounding less; with fp32 inputs the two coincide and match the dense formulation
    x, logits = torch.randn(9, 16, generator=gen), torch.randn(9, 4, generator=gen)
    w_up, w_down = torch.randn(4, 16, 128, generator=gen) * 0.2, torch.randn(4, 64, 16, generator=gen) * 0.2
    a = moe.moe_forward(x, logits, w_up, w_down, 2, fused=True)
    assert torch.allclose(a, moe.moe_forward(x, logits, w_up, w_down, 2), rtol=1e-6, atol=1e-6)
    assert torch.allclose(a.double(), moe.moe_dense(x, logits, w_up, w_down, 2), rtol=1e-4, atol=1e-4)
