"""Backward of grouped_mm on a real MI355X: every gradient is one of the four forward variants on
transposed views (grouped_mm_bf16_amd/api.py), so these tests drive the kernels with column-major
operands, with the upstream gradient as an operand and with jagged contractions that start at odd k.

The matrix restates the reference's backward tests (reference tests/test_grouped_mm.py: :243/:265 3Dx3D,
:289/:320 2Dx3D with empty groups, :405-525 the four boundary lists in fp32 and bf16, :527/:592 3Dx2D,
:560/:627 2Dx2D, :661-747 the 1023-group cases) with the reference's tolerances, and adds aligned shapes
that take the assembly tile, where each gradient is also held to the forward bar (rtol 1.6e-2,
atol 1e-2 * sqrt(K / 64), K = contraction length of that gradient's product).
"""
import pytest
import torch

from grouped_mm_bf16_amd import grouped_mm
from grouped_mm_bf16_amd import kernels as K_
from oracle import grouped_mm_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def offs_of(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def rnd(gen, *shape, dtype=torch.float32, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def loop_reference(variant, a, b, offs):
    """The per-group product written with stock torch ops in fp32 (what the reference's tests differentiate)."""
    rng = oracle.group_ranges(offs.tolist()) if offs is not None else None
    if variant == "2d3d":
        parts = [a[s:e] @ b[g] for g, (s, e) in enumerate(rng)]
        tail = a.shape[0] - rng[-1][1]
        if tail:   # rows past the last offset belong to nobody: they produce nothing and get no gradient
            parts.append(a.new_zeros(tail, b.shape[2]) + 0.0 * a[rng[-1][1]:, :1])
        return torch.cat(parts)
    if variant == "3d3d":
        return torch.bmm(a, b)
    if variant == "2d2d":
        return torch.stack([a[:, s:e] @ b[s:e] for (s, e) in rng])
    parts = [a[g] @ b[:, s:e] for g, (s, e) in enumerate(rng)]
    tail = b.shape[1] - rng[-1][1]
    if tail:
        parts.append(b.new_zeros(a.shape[1], tail) + 0.0 * b[:1, rng[-1][1]:])
    return torch.cat(parts, dim=1)


def make_case(variant, sizes, d1, d2, dtype, gen, scale_b=1.0, extra=0):
    """Operands of one variant; `sizes` run along the jagged dimension, `extra` unowned elements follow."""
    G, tot = len(sizes), sum(sizes) + extra
    offs = offs_of(sizes)
    if variant == "2d3d":
        return rnd(gen, tot, d1, dtype=dtype), rnd(gen, G, d1, d2, dtype=dtype, scale=scale_b), offs
    if variant == "3d3d":
        return rnd(gen, G, d2, d1, dtype=dtype), rnd(gen, G, d1, sizes[0], dtype=dtype, scale=scale_b), None
    if variant == "2d2d":
        return rnd(gen, d1, tot, dtype=dtype), rnd(gen, tot, d2, dtype=dtype, scale=scale_b), offs
    return rnd(gen, G, d1, d2, dtype=dtype), rnd(gen, d2, tot, dtype=dtype, scale=scale_b), offs


class LaunchLog:
    """Records (variant code, kernel family) of every launch inside the block."""

    def __enter__(self):
        self.calls, self._orig = [], K_._launch_now

        def logged(variant, a, b, offs, out):
            self._orig(variant, a, b, offs, out)
            self.calls.append((variant, K_.last_path()))
        K_._launch_now = logged
        return self

    def __exit__(self, *exc):
        K_._launch_now = self._orig


def run_both(variant, a, b, offs, layout=(False, False), grad_out=None, gen=None):
    """Forward + backward through grouped_mm on the GPU and through the fp32 loop on the host.
    Returns (out, grad_a, grad_b) of each and the launch log of the GPU side."""
    ad, bd = a.to(DEV), b.to(DEV)
    if layout[0]:
        ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
    if layout[1]:
        bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
    ad.requires_grad_()
    bd.requires_grad_()
    with LaunchLog() as log:
        out = grouped_mm(ad, bd, offs=None if offs is None else offs.to(DEV))
        if grad_out is None:
            grad_out = rnd(gen, *out.shape).to(out.dtype)
        out.backward(grad_out.to(DEV))
        torch.cuda.synchronize()
    ar, br = a.float().clone().requires_grad_(), b.float().clone().requires_grad_()
    ref = loop_reference(variant, ar, br, offs)
    # unowned rows / columns of the upstream gradient must not matter (they may hold anything)
    ref.backward(torch.nan_to_num(grad_out.float(), nan=0.0))
    return (out.detach().cpu(), ad.grad.cpu(), bd.grad.cpu()), (ref.detach(), ar.grad, br.grad), log.calls


def grad_contractions(variant, a, b, offs):
    """Contraction length of the products that give grad_a and grad_b (per group where it differs)."""
    if variant == "2d3d":      # dA = dC @ B^T over N; dB[g] = A_g^T @ dC_g over the group's rows
        return b.shape[2], "rows"
    if variant == "3d3d":
        return b.shape[2], a.shape[1]
    if variant == "2d2d":      # dA[:, k] = dC[g(k)] @ B[k]^T over N; dB[k] = A[:, k]^T dC[g(k)] over M
        return b.shape[1], a.shape[0]
    return "cols", a.shape[1]  # 3d2d: dA[g] = dC[:, cols_g] @ B[:, cols_g]^T over the group's columns; dB over M


def assert_grads_forward_bar(variant, got, want, a, b, offs):
    """Each gradient within rtol 1.6e-2 / atol 1e-2 sqrt(K / 64) of the fp32 loop's gradient rounded to the
    operand dtype, K taken per group where the contraction is the jagged dimension."""
    ka, kb = grad_contractions(variant, a, b, offs)
    dt = got[1].dtype
    rng = oracle.group_ranges(offs.tolist()) if offs is not None else None
    if kb == "rows":
        for g, (s, e) in enumerate(rng):
            oracle.assert_close(got[2][g], want[2][g].to(dt), e - s, what=f"grad_b group {g}")
    else:
        oracle.assert_close(got[2], want[2].to(dt), kb, what="grad_b")
    if ka == "cols":
        for g, (s, e) in enumerate(rng):
            oracle.assert_close(got[1][g], want[1][g].to(dt), e - s, what=f"grad_a group {g}")
    else:
        oracle.assert_close(got[1], want[1].to(dt), ka, what="grad_a")


# ------------------------------------------------------------------ the reference's matrix, its tolerances
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 4e-2)])
def test_3d3d_backward_reference_shapes(dtype, tol):
    gen = torch.Generator().manual_seed(0)
    a, b = rnd(gen, 3, 17, 19, dtype=dtype), rnd(gen, 3, 19, 23, dtype=dtype)
    got, want, _ = run_both("3d3d", a, b, None, gen=gen)
    for x, y in zip(got, want):
        torch.testing.assert_close(x.float(), y, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype,tol_a,tol_b", [(torch.float32, 3e-4, 5e-4), (torch.bfloat16, 5e-2, 5e-2)])
def test_2d3d_backward_with_empty_groups(dtype, tol_a, tol_b):
    gen = torch.Generator().manual_seed(1)
    a, b, offs = make_case("2d3d", [0, 7, 1, 13, 0, 11], 29, 31, dtype, gen)
    got, want, _ = run_both("2d3d", a, b, offs, gen=gen)
    torch.testing.assert_close(got[1].float(), want[1], rtol=tol_a, atol=tol_a)
    torch.testing.assert_close(got[2].float(), want[2], rtol=tol_b, atol=tol_b)
    assert (got[2][0] == 0).all() and (got[2][4] == 0).all()      # empty groups: exact zero slabs


BWD_BOUNDARY_LISTS = [[32, 1, 30], [31, 1, 31], [11, 90, 7], [0, 3, 0, 0, 5, 0, 1, 0, 9]]


@pytest.mark.parametrize("sizes", BWD_BOUNDARY_LISTS)
@pytest.mark.parametrize("seed", [0, 1])
def test_2d3d_backward_boundary_lists_fp32(sizes, seed):
    gen = torch.Generator().manual_seed(seed)
    a, b, offs = make_case("2d3d", sizes, 41, 37, torch.float32, gen)
    got, want, _ = run_both("2d3d", a, b, offs, gen=gen)
    torch.testing.assert_close(got[0], want[0], rtol=3e-4, atol=3e-4)
    torch.testing.assert_close(got[1], want[1], rtol=6e-4, atol=6e-4)
    torch.testing.assert_close(got[2], want[2], rtol=8e-4, atol=8e-4)


@pytest.mark.parametrize("sizes", BWD_BOUNDARY_LISTS)
def test_2d3d_backward_boundary_lists_bf16(sizes):
    gen = torch.Generator().manual_seed(2)
    a, b, offs = make_case("2d3d", sizes, 41, 37, torch.bfloat16, gen)
    got, want, _ = run_both("2d3d", a, b, offs, gen=gen)
    torch.testing.assert_close(got[1].float(), want[1], rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(got[2].float(), want[2], rtol=1e-1, atol=6e-1)
    assert_grads_forward_bar("2d3d", got, want, a, b, offs)


@pytest.mark.parametrize("variant,d1,d2", [("3d2d", 23, 17), ("2d2d", 19, 21)])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 6e-4), (torch.bfloat16, 6e-2)])
def test_3d2d_and_2d2d_backward_reference_shapes(variant, d1, d2, dtype, tol):
    gen = torch.Generator().manual_seed(3)
    a, b, offs = make_case(variant, [7, 0, 1, 13, 11], d1, d2, dtype, gen)
    got, want, _ = run_both(variant, a, b, offs, gen=gen)
    for x, y in zip(got, want):
        torch.testing.assert_close(x.float(), y, rtol=tol, atol=tol)
    if dtype == torch.bfloat16:
        assert_grads_forward_bar(variant, got, want, a, b, offs)


@pytest.mark.parametrize("variant", ["2d3d", "3d2d", "2d2d"])
def test_1023_groups_forward_and_backward_fp32(variant):
    """G = 1023, sizes alternate 1, 0 with a trailing empty group."""
    gen = torch.Generator().manual_seed(4)
    sizes = [1 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    d1, d2 = {"2d3d": (8, 8), "3d2d": (4, 8), "2d2d": (4, 8)}[variant]
    a, b, offs = make_case(variant, sizes, d1, d2, torch.float32, gen)
    got, want, _ = run_both(variant, a, b, offs, gen=gen)
    torch.testing.assert_close(got[0], want[0], rtol=3e-4, atol=3e-4)
    torch.testing.assert_close(got[1], want[1], rtol=6e-4, atol=6e-4)
    torch.testing.assert_close(got[2], want[2], rtol=8e-4, atol=8e-4)


# ------------------------------------------------------------------ the assembly tile as a backward
ALIGNED = {  # variant -> (sizes along the jagged dimension, d1, d2): every extent a multiple of 8
    "2d3d": ([77, 0, 1, 130, 64, 200], 136, 264),
    "3d3d": ([272, 272, 272], 136, 304),
    "2d2d": ([77, 0, 1, 130, 64, 200], 264, 272),
    "3d2d": ([77, 0, 1, 130, 64, 200], 264, 136),
}


@pytest.mark.parametrize("layout", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_on_the_assembly_tile(variant, layout, dtype):
    """bf16 / fp16 with aligned extents: the forward and both gradient launches take the MFMA family (the
    gradients through transposed views, with jagged contractions starting at odd k)."""
    gen = torch.Generator().manual_seed(5)
    sizes, d1, d2 = ALIGNED[variant]
    extra = 0 if variant == "3d3d" else 8 - sum(sizes) % 8   # pad the jagged extent to a multiple of 8
    a, b, offs = make_case(variant, sizes, d1, d2, dtype, gen, scale_b=0.1, extra=extra)
    got, want, calls = run_both(variant, a, b, offs, layout=layout, gen=gen)
    assert len(calls) == 3 and all(path == "mfma" for _, path in calls), calls
    assert_grads_forward_bar(variant, got, want, a, b, offs)
    tot = sum(sizes)
    owned = {"2d3d": (slice(0, tot),), "3d2d": (slice(None), slice(0, tot))}.get(variant, (slice(None),))
    oracle.assert_close_grouped(got[0][owned], want[0][owned].to(dtype), a, b, offs, what="forward")
    # what no group owns gets an exactly zero gradient
    if variant == "2d3d":
        assert (got[1][tot:] == 0).all() and (got[2][1] == 0).all()
    if variant == "2d2d":
        assert (got[1][:, tot:] == 0).all() and (got[2][tot:] == 0).all()
    if variant == "3d2d":
        assert (got[2][:, tot:] == 0).all() and (got[1][1] == 0).all()


@pytest.mark.parametrize("variant", ["2d3d", "3d2d"])
def test_unowned_upstream_gradient_does_not_leak(variant):
    """Rows / columns of grad_out past the last offset are NaN: no gradient element may see them."""
    gen = torch.Generator().manual_seed(6)
    sizes, d1, d2 = ALIGNED[variant]
    tot = sum(sizes)
    a, b, offs = make_case(variant, sizes, d1, d2, torch.bfloat16, gen, scale_b=0.1, extra=8 + 8 - tot % 8)
    shape = (a.shape[0], b.shape[2]) if variant == "2d3d" else (a.shape[1], b.shape[1])
    grad_out = rnd(gen, *shape).to(torch.bfloat16)
    if variant == "2d3d":
        grad_out[tot:] = float("nan")
    else:
        grad_out[:, tot:] = float("nan")
    got, want, calls = run_both(variant, a, b, offs, grad_out=grad_out)
    assert all(path == "mfma" for _, path in calls), calls
    assert torch.isfinite(got[1].float()).all() and torch.isfinite(got[2].float()).all()
    assert_grads_forward_bar(variant, got, want, a, b, offs)


def test_1023_groups_backward_bf16_mfma():
    """The alternating pattern with 8-row groups so that every launch of the backward is on the MFMA family."""
    gen = torch.Generator().manual_seed(7)
    sizes = [8 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    a, b, offs = make_case("2d3d", sizes, 64, 16, torch.bfloat16, gen)
    got, want, calls = run_both("2d3d", a, b, offs, gen=gen)
    assert len(calls) == 3 and all(path == "mfma" for _, path in calls), calls
    assert_grads_forward_bar("2d3d", got, want, a, b, offs)
    assert (got[2][1::2] == 0).all()
