"""The boundary as callers see it, on a real MI355X: the torch custom op that carries the launch, the
benchmark command line, views with padded leading dimensions / storage offsets, and G == 0."""
import re

import pytest
import torch

from grouped_mm_bf16_amd import bench_2d3d, grouped_mm
from grouped_mm_bf16_amd import kernels as K_
from oracle import grouped_mm_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def offs_of(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def rnd(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def _case(gen):
    sizes = [77, 0, 1, 130, 64, 200]
    a, b = rnd(gen, sum(sizes), 136), rnd(gen, len(sizes), 136, 264, scale=0.1)
    return a, b, offs_of(sizes)


# ------------------------------------------------------------------ torch custom op
def test_custom_op_matches_the_direct_launch_bit_for_bit():
    """`grouped_mm_bf16_amd::launch` (reference boundary: the four launchers of kernels.py:524-717 behind one
    op): called through torch.ops it must do exactly what the eager shortcut does."""
    gen = torch.Generator().manual_seed(61)
    a, b, offs = _case(gen)
    ad, bd, od = a.to(DEV), b.to(DEV), offs.to(DEV)
    direct = torch.full((a.shape[0], 264), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_._launch_now(K_.V_2D3D, ad, bd, od, direct)
    via_op = torch.full_like(direct, float("nan"))
    assert torch.ops.grouped_mm_bf16_amd.launch(K_.V_2D3D, ad, bd, od, via_op) is None
    torch.cuda.synchronize()
    assert torch.equal(direct.view(torch.int16), via_op.view(torch.int16))
    assert K_.last_path() == "mfma"
    want = oracle.grouped_mm(a, b, offs)
    oracle.assert_close(via_op.cpu(), want, 136)
    # 3D x 3D: the optional offs argument is None
    a3, b3 = rnd(gen, 3, 72, 136).to(DEV), rnd(gen, 3, 136, 264, scale=0.1).to(DEV)
    o1, o2 = (torch.empty(3, 72, 264, device=DEV, dtype=torch.bfloat16) for _ in range(2))
    K_._launch_now(K_.V_3D3D, a3, b3, None, o1)
    torch.ops.grouped_mm_bf16_amd.launch(K_.V_3D3D, a3, b3, None, o2)
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))


def test_custom_op_passes_opcheck():
    gen = torch.Generator().manual_seed(62)
    a, b, offs = _case(gen)
    out = torch.empty(a.shape[0], 264, device=DEV, dtype=torch.bfloat16)
    torch.library.opcheck(torch.ops.grouped_mm_bf16_amd.launch.default,
                          (K_.V_2D3D, a.to(DEV), b.to(DEV), offs.to(DEV), out),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("variant", ["2d3d", "3d3d"])
def test_compiled_graph_goes_through_the_custom_op(variant):
    """torch.compile(fullgraph=True): tracing reaches the launch through the registered op (no graph break),
    and the compiled function returns what eager returns, bit for bit, forward and backward."""
    gen = torch.Generator().manual_seed(63)
    if variant == "2d3d":
        a, b, offs = _case(gen)
    else:
        a, b, offs = rnd(gen, 3, 72, 136), rnd(gen, 3, 136, 264, scale=0.1), None
    od = None if offs is None else offs.to(DEV)

    def run(fn):
        ad, bd = a.to(DEV).requires_grad_(), b.to(DEV).requires_grad_()
        out = fn(ad, bd, od)
        rows = slice(None) if offs is None else slice(0, int(offs[-1]))
        out[rows].float().square().sum().backward()
        torch.cuda.synchronize()
        return out.detach()[rows], ad.grad, bd.grad

    eager = run(lambda x, y, o: grouped_mm(x, y, offs=o))
    torch._dynamo.reset()
    compiled_fn = torch.compile(lambda x, y, o: grouped_mm(x, y, offs=o), backend="aot_eager", fullgraph=True)
    compiled = run(compiled_fn)
    for e, c in zip(eager, compiled):
        assert torch.equal(e.view(torch.int16), c.view(torch.int16))
    want = oracle.grouped_mm(a, b, offs)
    oracle.assert_close(compiled[0].cpu(), want if offs is None else want[:int(offs[-1])], 136)


# ------------------------------------------------------------------ benchmark command line
def test_bench_cli_prints_forward_and_backward_lines(capsys):
    """Flags and output of the reference's bench/bench_2d3d.py:73-218 on a small problem."""
    bench_2d3d.main(["--experts", "4", "--batch-size", "256", "--active-experts-per-token", "2",
                     "--embedding-size", "128", "--output-features", "264", "--dtype", "bf16",
                     "--iters", "3", "--warmup", "1", "--mode", "both", "--seed", "1"])
    lines = [l for l in capsys.readouterr().out.splitlines() if l.strip()]
    assert len(lines) == 2
    fwd = re.match(r"\s*(\w+)\s+forward\s+([\d.]+) ms\s+([\d.]+) TFLOPs\s+\(experts=4, total_routed_tokens=512, ", lines[0])
    bwd = re.match(r"\s*(\w+)\s+backward\s+([\d.]+) ms\s+([\d.]+) TFLOPs\s+\(experts=4, total_routed_tokens=512, ", lines[1])
    assert fwd and bwd, lines
    assert float(fwd.group(2)) > 0 and float(bwd.group(2)) > 0
    assert "family=mfma" in lines[0] and "backward=both" in lines[1]
    # uniform load, one gradient, the generic family
    bench_2d3d.main(["--experts", "3", "--tokens-per-expert", "40", "--embedding-size", "33", "--output-features", "29",
                     "--iters", "2", "--warmup", "1", "--mode", "backward", "--backward", "da", "--impl", "generic"])
    lines = [l for l in capsys.readouterr().out.splitlines() if l.strip()]
    assert len(lines) == 1 and "total_routed_tokens=120" in lines[0] and "backward=da" in lines[0]


# ------------------------------------------------------------------ views: padded leading dimensions, offsets
@pytest.mark.parametrize("a_col", [False, True])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
def test_padded_views_on_the_assembly_tile(variant, a_col, b_col):
    """Operands that are slices of wider tensors (leading dimension larger than the extent, storage
    offset), with the storage ending at the view's last element: the tile must not depend on what lies
    around the view."""
    gen = torch.Generator().manual_seed(64)
    sizes = [77, 0, 1, 130, 64, 200]
    tot, G = sum(sizes), len(sizes)
    offs = offs_of(sizes)
    if variant == "2d3d":
        a, b, fn = rnd(gen, tot, 136), rnd(gen, G, 136, 264, scale=0.1), K_.grouped_mm_2d3d
    elif variant == "3d3d":
        a, b, fn, offs = rnd(gen, 3, 304, 136), rnd(gen, 3, 136, 264, scale=0.1), K_.grouped_mm_3d3d, None
    elif variant == "2d2d":
        a, b, fn = rnd(gen, 264, tot), rnd(gen, tot, 272, scale=0.1), K_.grouped_mm_2d2d
    else:
        a, b, fn = rnd(gen, G, 264, 136), rnd(gen, 136, tot, scale=0.1), K_.grouped_mm_3d2d

    def padded_view(x, col):
        """A view of `x`'s values whose rows (columns if `col`) are 24 elements apart from the extent, at a
        storage offset of 16 elements, in a buffer that ends with the view's last element; all padding is NaN."""
        y = x.transpose(-2, -1) if col else x
        r, c = y.shape[-2], y.shape[-1]
        ld = c + 24
        batch = y.shape[:-2]
        per = r * ld
        n = 16 + (int(torch.tensor(batch).prod()) if batch else 1) * per - 24   # ends at the last element
        buf = torch.full((n,), float("nan"), device=DEV, dtype=x.dtype)
        v = torch.as_strided(buf, (*batch, r, c), (*[per] * len(batch), ld, 1), 16)
        v.copy_(y)
        return v.transpose(-2, -1) if col else v

    ad, bd = padded_view(a, a_col), padded_view(b, b_col)
    shape = oracle.grouped_mm(a, b, offs).shape
    out = torch.full(shape, float("nan"), device=DEV, dtype=torch.bfloat16)
    with K_.forced_path("mfma"):
        if offs is None:
            fn(ad, bd, out)
        else:
            fn(ad, bd, offs.to(DEV), out)
        torch.cuda.synchronize()
    want = oracle.grouped_mm(a, b, offs)
    got = out.cpu()
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs"
    oracle.assert_close_grouped(got, want, a, b, offs)


# ------------------------------------------------------------------ no groups at all
def test_zero_groups_write_nothing():
    """offs.numel() == 0: the reference launches and no row finds an owner (kernels.py:162-172, :335-360);
    here the launch is skipped and the output is left as it was."""
    a = torch.randn(16, 64, device=DEV, dtype=torch.bfloat16)
    b = torch.randn(0, 64, 48, device=DEV, dtype=torch.bfloat16)
    offs = torch.zeros(0, device=DEV, dtype=torch.int32)
    out = torch.full((16, 48), 7.0, device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(a, b, offs, out)
    torch.cuda.synchronize()
    assert (out == 7).all()
    res = grouped_mm(a, b, offs=offs)
    assert res.shape == (16, 48)
    a3 = torch.randn(0, 16, 64, device=DEV, dtype=torch.bfloat16)
    b2 = torch.randn(64, 40, device=DEV, dtype=torch.bfloat16)
    out = torch.full((16, 40), 7.0, device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_3d2d(a3, b2, offs, out)
    torch.cuda.synchronize()
    assert (out == 7).all()
    # K-grouped: the output has G == 0 slabs, i.e. no elements
    assert grouped_mm(a, torch.randn(64, 24, device=DEV, dtype=torch.bfloat16), offs=offs).shape == (0, 16, 24)
