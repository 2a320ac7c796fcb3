"""Argument rules of the MoE step's host layer, checked on the CPU: a caller-supplied ``out`` (the kernels
write through a raw pointer with no extent) and the routing tensors must be exactly what the call computes.
The device check is switched off so that plain CPU tensors reach the rules; every case must raise before
anything is launched."""
import pytest
import torch

from grouped_mm_bf16_amd import moe


@pytest.fixture(autouse=True)
def no_device_check(monkeypatch):
    monkeypatch.setattr(moe, "_require_gpu", lambda *tensors: None)


def bf(*shape):
    return torch.zeros(*shape, dtype=torch.bfloat16)


def i32(n):
    return torch.zeros(n, dtype=torch.int32)


BAD_OUTS = [
    ("shape", lambda r, c: bf(r, c + 8)),
    ("rows", lambda r, c: bf(r - 1, c)),
    ("dtype", lambda r, c: torch.zeros(r, c, dtype=torch.float16)),
    ("column-major", lambda r, c: bf(c, r).t()),
    ("strided columns", lambda r, c: bf(r, 2 * c)[:, ::2]),
    ("rank", lambda r, c: bf(1, r, c)),
]


@pytest.mark.parametrize("what,make", BAD_OUTS)
def test_gathered_rejects_a_wrong_out(what, make):
    with pytest.raises(RuntimeError, match="out has to be"):
        moe.grouped_mm_gathered(bf(40, 64), i32(24), bf(3, 64, 48), i32(3), out=make(24, 48))


@pytest.mark.parametrize("what,make", BAD_OUTS)
def test_swiglu_rejects_a_wrong_out(what, make):
    with pytest.raises(RuntimeError, match="out has to be"):
        moe.grouped_mm_swiglu(bf(40, 64), i32(24), bf(3, 64, 256), i32(3), out=make(24, 128))


@pytest.mark.parametrize("what,make", BAD_OUTS)
def test_activation_rejects_a_wrong_out(what, make):
    with pytest.raises(RuntimeError, match="out has to be"):
        moe.moe_activation(bf(24, 256), "swiglu", out=make(24, 128))


@pytest.mark.parametrize("what,make", BAD_OUTS)
def test_combine_rejects_a_wrong_out(what, make):
    r = moe.Routing(i32(4), i32(16), torch.zeros(16), i32(16), i32(16))
    with pytest.raises(RuntimeError, match="out has to be"):
        moe.moe_combine(bf(16, 64), r, 8, 2, out=make(8, 64))


@pytest.mark.parametrize("tokens,top_k", [(8, 3), (9, 2), (4, 2)])
def test_combine_rejects_routing_that_disagrees_with_tokens_and_top_k(tokens, top_k):
    r = moe.Routing(i32(4), i32(16), torch.zeros(16), i32(16), i32(16))
    with pytest.raises(RuntimeError, match="tokens \\* top_k"):
        moe.moe_combine(bf(16, 64), r, tokens, top_k)


def test_combine_rejects_routing_of_the_wrong_type():
    r = moe.Routing(i32(4), i32(16), torch.zeros(16, dtype=torch.float64), i32(16), i32(16))
    with pytest.raises(RuntimeError, match="slot_weight"):
        moe.moe_combine(bf(16, 64), r, 8, 2)
    r = moe.Routing(i32(4), i32(16), torch.zeros(16), i32(16), torch.zeros(32, dtype=torch.int32)[::2])
    with pytest.raises(RuntimeError, match="token_rows"):
        moe.moe_combine(bf(16, 64), r, 8, 2)


def test_strided_offsets_are_rejected():
    offs = torch.zeros(6, dtype=torch.int32)[::2]
    with pytest.raises(RuntimeError, match="Offsets have to be int32"):
        moe.grouped_mm_gathered(bf(40, 64), i32(24), bf(3, 64, 48), offs)
    with pytest.raises(RuntimeError, match="offs has to be int32"):
        moe.grouped_mm_swiglu(bf(40, 64), i32(24), bf(3, 64, 256), offs)
