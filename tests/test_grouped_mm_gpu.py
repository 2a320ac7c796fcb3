"""Parity of the HIP path with the CPU oracle, on a real MI355X.

Shapes, size lists and tolerances restate the reference's own test matrix
(reference tests/test_grouped_mm.py: :19 3Dx3D, :32 2Dx3D, :70 2Dx2D, :109 3Dx2D,
:356-370 the seven boundary lists, :661-747 the 1023-group cases) and add the
benchmark workloads.  Tolerance: rtol 1.6e-2, atol 1e-2 * sqrt(K / 64) against
the fp32 oracle; which elements are written is checked exactly (NaN poisoning).
"""
import json
import os

import numpy as np
import pytest
import torch

from grouped_mm_bf16_amd import grouped_mm
from grouped_mm_bf16_amd import kernels as K_
from oracle import grouped_mm_oracle as oracle

pytestmark = pytest.mark.gpu

DEV = "cuda"


def offs_of(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def rnd(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def run_poisoned(variant_fn, a, b, offs, shape, dtype):
    """Launch into a NaN-filled output so unwritten elements stay visible."""
    out = torch.full(shape, float("nan"), device=DEV, dtype=dtype)
    if offs is None:
        variant_fn(a.to(DEV), b.to(DEV), out)
    else:
        variant_fn(a.to(DEV), b.to(DEV), offs.to(DEV), out)
    torch.cuda.synchronize()
    return out.cpu()


def check(out, a, b, offs, k=None, path=None, what=""):
    """Oracle comparison with exact ownership.  The tolerance uses the contraction length of each
    element's own group (`k`, when given, must be that length: it is only asserted, never trusted)."""
    want = oracle.grouped_mm(a, b, offs, out_dtype=out.dtype)
    got = out.cpu()
    # structure: exactly the owned elements are written
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs " + what
    if k is not None and not (a.dim() == 2 and b.dim() == 2):
        assert k == a.shape[-1]
    oracle.assert_close_grouped(got, want, a, b, offs, what=what)
    if path is not None:
        assert K_.last_path() == path


# ------------------------------------------------------------------ golden fixtures
@pytest.mark.parametrize("name,a_shape,b_shape", [
    ("2d3d", (32, 64), (6, 64, 48)), ("3d3d", (4, 32, 64), (4, 64, 48)),
    ("2d2d", (16, 32), (32, 24)), ("3d2d", (5, 32, 48), (48, 32)),
])
@pytest.mark.parametrize("path", ["mfma", "generic"])
def test_golden_vectors(golden_dir, name, a_shape, b_shape, path):
    z = np.load(os.path.join(golden_dir, "small_cases.npz"))
    bits = lambda arr, shape: torch.from_numpy(arr.astype(np.int16)).view(torch.bfloat16).reshape(shape)
    a, b = bits(z[f"a_{name}"], a_shape), bits(z[f"b_{name}"], b_shape)
    offs = torch.from_numpy(z[f"offs_{name}"]) if f"offs_{name}" in z else None
    with K_.forced_path(path):
        got = grouped_mm(a.to(DEV), b.to(DEV), offs=None if offs is None else offs.to(DEV)).cpu()
    want = bits(z[f"out_{name}"], got.shape)
    own = ~torch.isnan(oracle.grouped_mm(a, b, offs).float())
    oracle.assert_close(got[own], want[own], a.shape[-1])
    assert K_.last_path() == path


# ------------------------------------------------------------------ the reference's basic cases
@pytest.mark.parametrize("path", ["auto", "generic"])
def test_3d3d_bf16(path):
    gen = torch.Generator().manual_seed(0)
    a, b = rnd(gen, 4, 32, 64), rnd(gen, 4, 64, 48)
    with K_.forced_path(path):
        out = run_poisoned(K_.grouped_mm_3d3d, a, b, None, (4, 32, 48), torch.bfloat16)
    check(out, a, b, None, 64)


@pytest.mark.parametrize("path", ["auto", "generic"])
def test_2d3d_bf16_with_empty_groups(path):
    gen = torch.Generator().manual_seed(1)
    sizes = [0, 7, 1, 13, 0, 11]
    a, b = rnd(gen, 32, 32), rnd(gen, 6, 32, 40)
    with K_.forced_path(path):
        out = run_poisoned(K_.grouped_mm_2d3d, a, b, offs_of(sizes), (32, 40), torch.bfloat16)
    check(out, a, b, offs_of(sizes), 32)


@pytest.mark.parametrize("path", ["auto", "generic"])
def test_2d2d_bf16_empty_group_is_zero(path):
    gen = torch.Generator().manual_seed(2)
    sizes = [7, 0, 1, 13, 11]
    a, b = rnd(gen, 16, 32), rnd(gen, 32, 24)
    with K_.forced_path(path):
        out = run_poisoned(K_.grouped_mm_2d2d, a, b, offs_of(sizes), (5, 16, 24), torch.bfloat16)
    check(out, a, b, offs_of(sizes))
    assert (out[1] == 0).all() and not torch.isnan(out.float()).any()


@pytest.mark.parametrize("path", ["auto", "generic"])
def test_3d2d_bf16(path):
    gen = torch.Generator().manual_seed(3)
    sizes = [7, 0, 1, 13, 11]
    a, b = rnd(gen, 5, 32, 48), rnd(gen, 48, 32)
    with K_.forced_path(path):
        out = run_poisoned(K_.grouped_mm_3d2d, a, b, offs_of(sizes), (32, 32), torch.bfloat16)
    check(out, a, b, offs_of(sizes), 48)


BOUNDARY_LISTS = [
    [32, 32, 32], [10, 10, 10, 2], [31, 1, 31], [40, 30, 10, 7], [32, 16, 0, 0, 0],
    [1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0], [5, 0, 7, 0, 3, 9],
]


@pytest.mark.parametrize("sizes", BOUNDARY_LISTS)
def test_2d3d_boundary_lists_unaligned_shapes(sizes):
    """K = 33, N = 29: no 16-byte alignment anywhere, so the generic family runs."""
    gen = torch.Generator().manual_seed(sum(sizes))
    m = sum(sizes)
    a, b = rnd(gen, m, 33), rnd(gen, len(sizes), 33, 29)
    out = run_poisoned(K_.grouped_mm_2d3d, a, b, offs_of(sizes), (m, 29), torch.bfloat16)
    check(out, a, b, offs_of(sizes), 33, path="generic")


@pytest.mark.parametrize("sizes", BOUNDARY_LISTS + [[300, 0, 1, 255, 256, 257, 33], [256, 256], [257, 255, 512]])
@pytest.mark.parametrize("b_col", [False, True])
def test_2d3d_boundary_lists_mfma(sizes, b_col):
    """Same lists on aligned K / N so that the MFMA family and its 256-row tiles run."""
    gen = torch.Generator().manual_seed(sum(sizes) + 1)
    m = sum(sizes)
    a, b = rnd(gen, m, 72), rnd(gen, len(sizes), 72, 264)
    bd = b.to(DEV)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((m, 264), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(a.to(DEV), bd, offs_of(sizes).to(DEV), out)
    check(out, a, b, offs_of(sizes), 72, path="mfma")


SMALL_GROUPS = [1, 15, 16, 17, 31, 33, 0, 1, 1, 63, 64, 65, 127, 129, 2]


@pytest.mark.parametrize("tall,shrt", [(-1, -1), (256, 64), (256, 0), (128, 64), (128, 0)])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("K,N", [(72, 264), (2048, 768)])
def test_small_groups_on_every_tile_height(K, N, b_col, tall, shrt):
    """Groups of 1, 15, 16, 17, 31, 33 ... rows (what a fine-grained expert layer produces): each row is owned
    by exactly its group whatever heights the tiles have, and rows of neighbouring groups inside one tile's
    extent are neither read into the product nor written."""
    gen = torch.Generator().manual_seed(K + N)
    sizes = SMALL_GROUPS
    m = sum(sizes)
    a, b = rnd(gen, m + 5, K), rnd(gen, len(sizes), K, N, scale=0.05)
    a[m:] = float("nan")                       # rows past offs[-1]: never part of any product
    bd = b.to(DEV)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((m + 5, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    with K_.forced_tile_heights(tall, shrt):
        K_.grouped_mm_2d3d(a.to(DEV), bd, offs_of(sizes).to(DEV), out)
        torch.cuda.synchronize()
    check(out, a, b, offs_of(sizes), K, path="mfma")


def test_output_larger_than_4_gib():
    """70000 x 32768 bf16 output (4.6 GB): every tile's address arithmetic must be 64-bit up to the tile's
    origin.  Rows on both sides of the 2 GiB and 4 GiB marks and of the group boundaries against the oracle."""
    gen = torch.Generator().manual_seed(17)
    sizes = [30000, 5, 39995]
    m, K, N = sum(sizes), 64, 32768
    a, b = rnd(gen, m, K), rnd(gen, len(sizes), K, N, scale=0.1)
    offs = offs_of(sizes)
    out = torch.empty(m, N, device=DEV, dtype=torch.bfloat16)
    out[::997].fill_(float("nan"))
    K_.grouped_mm_2d3d(a.to(DEV), b.to(DEV), offs.to(DEV), out)
    torch.cuda.synchronize()
    assert K_.last_path() == "mfma"
    marks = [0, 255, 256, 29999, 30000, 30004, 30005, 32767, 32768, 32769, 65535, 65536, 65537, m - 257, m - 1]
    rows = sorted(set(marks + list(range(0, m, 997))))
    got = out[rows].cpu()
    grp = torch.searchsorted(offs.long(), torch.tensor(rows), right=True)
    for g in range(len(sizes)):
        sel = (grp == g).nonzero().flatten()
        if len(sel):
            want = (a[[rows[i] for i in sel]].float() @ b[g].float()).to(torch.bfloat16)
            oracle.assert_close(got[sel], want, K, what=f"group {g}")
    del out


def test_rows_past_the_last_offset_are_not_written():
    gen = torch.Generator().manual_seed(5)
    a, b = rnd(gen, 40, 64), rnd(gen, 2, 64, 48)
    offs = offs_of([9, 14])  # rows 23..39 belong to nobody
    for path in ("mfma", "generic"):
        with K_.forced_path(path):
            out = run_poisoned(K_.grouped_mm_2d3d, a, b, offs, (40, 48), torch.bfloat16)
        check(out, a, b, offs, 64, path=path)
        assert torch.isnan(out[23:].float()).all()


def test_launch_replays_from_a_captured_graph():
    """The launcher allocates nothing and never synchronises, so it can be captured; every replay must
    give what the eager launch gives on the same inputs (new contents, same buffers)."""
    gen = torch.Generator().manual_seed(41)
    sizes = [130, 0, 257, 64, 61]
    m, offs = sum(sizes), offs_of(sizes).to(DEV)
    a_s = torch.zeros(m, 192, device=DEV, dtype=torch.bfloat16)
    b_s = torch.zeros(len(sizes), 192, 264, device=DEV, dtype=torch.bfloat16)
    out_s = torch.zeros(m, 264, device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(a_s, b_s, offs, out_s)        # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            K_.grouped_mm_2d3d(a_s, b_s, offs, out_s)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        a, b = rnd(gen, m, 192), rnd(gen, len(sizes), 192, 264)
        a_s.copy_(a.to(DEV))
        b_s.copy_(b.to(DEV))
        out_s.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        replayed = out_s.clone()
        eager = torch.full_like(out_s, float("nan"))
        K_.grouped_mm_2d3d(a_s, b_s, offs, eager)
        torch.cuda.synchronize()
        assert torch.equal(replayed.view(torch.int16), eager.view(torch.int16)), f"replay {rep} differs from eager"
        check(replayed, a, b, offs.cpu(), 192)


# ------------------------------------------------------------------ operand layouts
@pytest.mark.parametrize("a_col", [False, True])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
def test_all_layouts_all_variants_mfma(variant, a_col, b_col):
    gen = torch.Generator().manual_seed(17)
    sizes = [77, 0, 1, 130, 64, 200]  # sum 472
    offs = offs_of(sizes)
    G = len(sizes)
    if variant == "2d3d":
        a, b, shape, k, fn = rnd(gen, 472, 136), rnd(gen, G, 136, 264), (472, 264), 136, K_.grouped_mm_2d3d
    elif variant == "3d3d":
        a, b, shape, k, fn, offs = rnd(gen, 3, 304, 136), rnd(gen, 3, 136, 264), (3, 304, 264), 136, K_.grouped_mm_3d3d, None
    elif variant == "2d2d":
        a, b, shape, k, fn = rnd(gen, 264, 472), rnd(gen, 472, 272), (G, 264, 272), 200, K_.grouped_mm_2d2d
    else:
        a, b, shape, k, fn = rnd(gen, G, 264, 136), rnd(gen, 136, 472), (264, 472), 136, K_.grouped_mm_3d2d
    ad, bd = a.to(DEV), b.to(DEV)
    if a_col:
        ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
    if b_col:
        bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
    out = torch.full(shape, float("nan"), device=DEV, dtype=torch.bfloat16)
    if offs is None:
        fn(ad, bd, out)
    else:
        fn(ad, bd, offs.to(DEV), out)
    check(out, a, b, offs, k, path="mfma")


@pytest.mark.parametrize("tall,shrt", [(256, 64), (256, 0), (128, 64), (128, 0)])
@pytest.mark.parametrize("b_col", [False, True])
def test_tile_heights_agree_bit_for_bit(tall, shrt, b_col):
    """Groups whose remainders fall in every height class (1..64, 65..128, 129..255 rows): each forced
    choice of tile heights gives the oracle's result, and all choices give the same bits (the order of
    the K loop does not depend on the tile height)."""
    gen = torch.Generator().manual_seed(29)
    sizes = [256 + 1, 64, 65, 128, 129, 512 + 200, 0, 255, 3 * 256, 63]
    m = sum(sizes)
    a, b = rnd(gen, m, 328), rnd(gen, len(sizes), 328, 264, scale=0.05)
    ad, bd, offs = a.to(DEV), b.to(DEV), offs_of(sizes)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    outs = []
    for heights in ((tall, shrt), (256, 0)):
        out = torch.full((m, 264), float("nan"), device=DEV, dtype=torch.bfloat16)
        with K_.forced_tile_heights(*heights):
            K_.grouped_mm_2d3d(ad, bd, offs.to(DEV), out)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    check(outs[0], a, b, offs, 328, path="mfma")
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


@pytest.mark.parametrize("a_col", [False, True])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                               (torch.float16, torch.float16), (torch.float16, torch.float32)])
@pytest.mark.parametrize("sizes", [[77, 0, 1, 330, 64, 200], [8, 16, 256, 512, 24], [3, 5, 7, 9, 300, 1, 600]])
def test_3d2d_on_the_assembly_tile(sizes, in_dtype, out_dtype, a_col, b_col):
    """Jagged columns: group boundaries inside a 16-byte chunk of the output go out as element stores;
    nothing outside a group's columns (and nothing past the last offset) is written."""
    gen = torch.Generator().manual_seed(31 + len(sizes))
    G, n_total = len(sizes), sum(sizes)
    extra = 16 + (-n_total % 8)   # columns past the last offset belong to nobody; the total is a multiple of 8
    a, b = rnd(gen, G, 328, 200, dtype=in_dtype), rnd(gen, 200, n_total + extra, scale=0.05, dtype=in_dtype)
    offs = offs_of(sizes)
    ad, bd = a.to(DEV), b.to(DEV)
    if a_col:
        ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
    if b_col:
        bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
    out = torch.full((328, n_total + extra), float("nan"), device=DEV, dtype=out_dtype)
    K_.grouped_mm_3d2d(ad, bd, offs.to(DEV), out)
    torch.cuda.synchronize()
    assert K_.last_path() == "mfma" and K_._lib.load().gmm_last_mfma_config() == 1
    got = out.cpu()
    assert torch.isnan(got[:, n_total:].float()).all()
    want = oracle.grouped_mm(a, b, offs, out_dtype=out_dtype)
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs"
    oracle.assert_close(got, want, 200)


def test_row_major_and_column_major_b_agree_bit_for_bit():
    gen = torch.Generator().manual_seed(19)
    a, b = rnd(gen, 4, 256, 512).to(DEV), rnd(gen, 4, 512, 256, scale=0.02).to(DEV)
    b_col = b.transpose(1, 2).contiguous().transpose(1, 2)
    assert torch.equal(grouped_mm(a, b).view(torch.int16), grouped_mm(a, b_col).view(torch.int16))


def test_mfma_rate_diagnostic_runs():
    """The register-only MFMA loops behind `bench.py --workload mfma_only` (a bench-only library of their own):
    argument checks and one launch per MFMA shape."""
    import ctypes
    import bench
    lib = bench.load_diag()
    frags = torch.randn(64, 8).to(torch.bfloat16).to(DEV)
    out = torch.full((512 * 256 * 2,), float("nan"), device=DEV)
    blocks = ctypes.c_int32(0)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.gmm_diag_mfma_rate(None, 16, out.data_ptr(), out.numel() * 4, 1, 10, 0, ctypes.addressof(blocks), stream) != 0
    assert lib.gmm_diag_mfma_rate(frags.data_ptr(), frags.numel() * 2, out.data_ptr(), 16, 1, 10, 0, ctypes.addressof(blocks), stream) != 0
    assert lib.gmm_diag_mfma_rate(frags.data_ptr(), frags.numel() * 2, out.data_ptr(), out.numel() * 4, 1, 10, 2,
                                  ctypes.addressof(blocks), stream) != 0
    for shape in (0, 1):
        out.fill_(float("nan"))
        assert lib.gmm_diag_mfma_rate(frags.data_ptr(), frags.numel() * 2, out.data_ptr(), out.numel() * 4, 2, 10, shape,
                                      ctypes.addressof(blocks), stream) == 0
        torch.cuda.synchronize()
        n = blocks.value * 256
        assert blocks.value > 0 and torch.isfinite(out[:n]).all() and torch.isnan(out[n:]).all()


@pytest.mark.parametrize("a_col", [False, True])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-4), (torch.bfloat16, None)])
def test_generic_family_on_the_matrix_cores(variant, a_col, b_col, dtype, tol):
    """Problems with at least one 128 x 128 tile that the 16-bit MFMA tile does not take (fp32 operands;
    bf16 with odd extents): the stride-generic kernel built on v_mfma_f32_32x32x2_f32."""
    gen = torch.Generator().manual_seed(53)
    sizes = [77, 0, 1, 331, 64, 200]  # sum 673
    offs = offs_of(sizes)
    G = len(sizes)
    if variant == "2d3d":
        a, b, shape, k, fn = rnd(gen, 673, 203, dtype=dtype), rnd(gen, G, 203, 261, dtype=dtype, scale=0.1), (673, 261), 203, K_.grouped_mm_2d3d
    elif variant == "3d3d":
        a, b, shape, k, fn, offs = rnd(gen, 3, 301, 203, dtype=dtype), rnd(gen, 3, 203, 261, dtype=dtype, scale=0.1), (3, 301, 261), 203, K_.grouped_mm_3d3d, None
    elif variant == "2d2d":
        a, b, shape, k, fn = rnd(gen, 261, 673, dtype=dtype), rnd(gen, 673, 269, dtype=dtype, scale=0.1), (G, 261, 269), 331, K_.grouped_mm_2d2d
    else:
        a, b, shape, k, fn = rnd(gen, G, 261, 203, dtype=dtype), rnd(gen, 203, 673, dtype=dtype, scale=0.1), (261, 673), 203, K_.grouped_mm_3d2d
    ad, bd = a.to(DEV), b.to(DEV)
    if a_col:
        ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
    if b_col:
        bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
    out = torch.full(shape, float("nan"), device=DEV, dtype=dtype)
    if offs is None:
        fn(ad, bd, out)
    else:
        fn(ad, bd, offs.to(DEV), out)
    torch.cuda.synchronize()
    assert K_.last_path() == "generic"
    want = oracle.grouped_mm(a, b, offs, out_dtype=dtype)
    got = out.cpu()
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs"
    if tol is None:
        oracle.assert_close_grouped(got, want, a, b, offs)
    else:
        owned = ~torch.isnan(want)
        torch.testing.assert_close(got[owned], want[owned], rtol=tol, atol=tol)


# ------------------------------------------------------------------ seeded random sweep
def _random_case(rng):
    variant = ["2d3d", "3d3d", "2d2d", "3d2d"][int(rng.integers(0, 4))]
    G = int(rng.integers(1, 9))
    # group sizes around the tile heights (0, 1, 63..65, 127..129, 255..257, a few hundred)
    pool = [0, 0, 1, 2, 7, 8, 9, 31, 63, 64, 65, 100, 127, 128, 129, 191, 192, 193, 255, 256, 257, 300, 511, 513]
    sizes = [int(pool[int(rng.integers(0, len(pool)))]) for _ in range(G)]
    if sum(sizes) == 0:
        sizes[0] = 8
    mult8 = lambda x: max(8, (x + 7) // 8 * 8)
    d1 = mult8(int(rng.integers(8, 400)))
    d2 = mult8(int(rng.integers(8, 600)))
    return variant, sizes, d1, d2


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_all_variants(seed):
    """Random variant / group sizes / extents / layouts / element and output types, MFMA family, against
    the oracle with exact ownership."""
    rng = np.random.default_rng(1000 + seed)
    gen = torch.Generator().manual_seed(2000 + seed)
    for _ in range(4):
        variant, sizes, d1, d2 = _random_case(rng)
        G, tot = len(sizes), sum(sizes)
        tot8 = tot + (-tot % 8)           # the jagged extent, padded so that strides stay multiples of 8
        dt = [torch.bfloat16, torch.float16][int(rng.integers(0, 2))]
        out_dt = [dt, torch.float32][int(rng.integers(0, 2))]
        a_col, b_col = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        offs = offs_of(sizes)
        if variant == "2d3d":
            a, b, shape, k, fn = rnd(gen, tot8, d1, dtype=dt), rnd(gen, G, d1, d2, dtype=dt, scale=0.1), (tot8, d2), d1, K_.grouped_mm_2d3d
        elif variant == "3d3d":
            a, b, shape, k, fn, offs = rnd(gen, G, d2, d1, dtype=dt), rnd(gen, G, d1, 264, dtype=dt, scale=0.1), (G, d2, 264), d1, K_.grouped_mm_3d3d, None
        elif variant == "2d2d":
            a, b, shape, k, fn = rnd(gen, d1, tot8, dtype=dt), rnd(gen, tot8, d2, dtype=dt, scale=0.1), (G, d1, d2), max(sizes), K_.grouped_mm_2d2d
        else:
            a, b, shape, k, fn = rnd(gen, G, d1, d2, dtype=dt), rnd(gen, d2, tot8, dtype=dt, scale=0.1), (d1, tot8), d2, K_.grouped_mm_3d2d
        ad, bd = a.to(DEV), b.to(DEV)
        if a_col:
            ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
        if b_col:
            bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
        out = torch.full(shape, float("nan"), device=DEV, dtype=out_dt)
        what = f"{variant} sizes={sizes} d1={d1} d2={d2} {dt} -> {out_dt} a_col={a_col} b_col={b_col}"
        with K_.forced_path("mfma"):
            if offs is None:
                fn(ad, bd, out)
            else:
                fn(ad, bd, offs.to(DEV), out)
            torch.cuda.synchronize()
        want = oracle.grouped_mm(a, b, offs, out_dtype=out_dt)
        got = out.cpu()
        assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs: " + what
        oracle.assert_close_grouped(got, want, a, b, offs, what=what)


# ------------------------------------------------------------------ dtypes
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-4), (torch.float16, 2e-2)])
def test_fp32_and_fp16_inputs(dtype, tol):
    gen = torch.Generator().manual_seed(23)
    sizes = [0, 7, 1, 13, 0, 11]
    a, b = rnd(gen, 32, 29, dtype=dtype), rnd(gen, 6, 29, 31, dtype=dtype)
    got = grouped_mm(a.to(DEV), b.to(DEV), offs=offs_of(sizes).to(DEV)).cpu()
    assert got.dtype == dtype and K_.last_path() == "generic"
    want = oracle.grouped_mm(a, b, offs_of(sizes))
    torch.testing.assert_close(got, want, rtol=tol, atol=tol)


@pytest.mark.parametrize("a_col", [False, True])
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_fp16_inputs_on_the_assembly_tile(variant, a_col, b_col, out_dtype):
    """fp16 inputs take the same tile with the fp16 MFMA; fp16 or fp32 out."""
    gen = torch.Generator().manual_seed(43)
    sizes = [77, 0, 1, 330, 64, 200]  # sum 672
    offs = offs_of(sizes)
    G, h = len(sizes), torch.float16
    if variant == "2d3d":
        a, b, shape, k, fn = rnd(gen, 672, 200, dtype=h), rnd(gen, G, 200, 264, dtype=h), (672, 264), 200, K_.grouped_mm_2d3d
    elif variant == "3d3d":
        a, b, shape, k, fn, offs = rnd(gen, 3, 304, 200, dtype=h), rnd(gen, 3, 200, 264, dtype=h), (3, 304, 264), 200, K_.grouped_mm_3d3d, None
    elif variant == "2d2d":
        a, b, shape, k, fn = rnd(gen, 264, 672, dtype=h), rnd(gen, 672, 272, dtype=h), (G, 264, 272), 330, K_.grouped_mm_2d2d
    else:
        a, b, shape, k, fn = rnd(gen, G, 264, 200, dtype=h), rnd(gen, 200, 672, dtype=h), (264, 672), 200, K_.grouped_mm_3d2d
    ad, bd = a.to(DEV), b.to(DEV)
    if a_col:
        ad = ad.transpose(-2, -1).contiguous().transpose(-2, -1)
    if b_col:
        bd = bd.transpose(-2, -1).contiguous().transpose(-2, -1)
    out = torch.full(shape, float("nan"), device=DEV, dtype=out_dtype)
    if offs is None:
        fn(ad, bd, out)
    else:
        fn(ad, bd, offs.to(DEV), out)
    torch.cuda.synchronize()
    assert K_.last_path() == "mfma" and K_._lib.load().gmm_last_mfma_config() == 1
    want = oracle.grouped_mm(a, b, offs, out_dtype=out_dtype)
    got = out.cpu()
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs"
    # fp16 keeps 11 bits: one rounding of the fp32 sum, and the sum itself in another order than the oracle's
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-3, atol=2e-2 if out_dtype == torch.float16 else 2e-3)


@pytest.mark.parametrize("variant", ["2d3d", "3d2d", "2d2d"])
def test_1023_groups_fp32(variant):
    """G = 1023, sizes alternate 1, 0 with a trailing empty group (reference tests :661-747)."""
    gen = torch.Generator().manual_seed(29)
    sizes = [1 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    tot, offs = sum(sizes), offs_of(sizes)
    if variant == "2d3d":
        a, b = rnd(gen, tot, 8, dtype=torch.float32), rnd(gen, 1023, 8, 8, dtype=torch.float32)
    elif variant == "3d2d":
        a, b = rnd(gen, 1023, 4, 8, dtype=torch.float32), rnd(gen, 8, tot, dtype=torch.float32)
    else:
        a, b = rnd(gen, 4, tot, dtype=torch.float32), rnd(gen, tot, 8, dtype=torch.float32)
    got = grouped_mm(a.to(DEV), b.to(DEV), offs=offs.to(DEV)).cpu()
    want = oracle.grouped_mm(a, b, offs)
    torch.testing.assert_close(got, want, rtol=3e-4, atol=3e-4)


def test_1023_groups_bf16_mfma():
    gen = torch.Generator().manual_seed(31)
    sizes = [3 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    tot, offs = sum(sizes), offs_of(sizes)
    a, b = rnd(gen, tot, 64), rnd(gen, 1023, 64, 16)
    with K_.forced_path("mfma"):
        out = run_poisoned(K_.grouped_mm_2d3d, a, b, offs, (tot, 16), torch.bfloat16)
    check(out, a, b, offs, 64, path="mfma")


def test_1023_groups_bf16_mfma_3d2d_and_2d2d():
    """The alternating 3 / 0 pattern of the reference's 1023-group cases on the MFMA family: every
    group boundary of 3D x 2D lies inside a 16-byte chunk of the output."""
    gen = torch.Generator().manual_seed(33)
    sizes = [3 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    tot, offs = sum(sizes), offs_of(sizes)          # 1533 columns; pad the total to a multiple of 8
    n_total = tot + (-tot % 8)
    a, b = rnd(gen, 1023, 16, 64), rnd(gen, 64, n_total)
    out = run_poisoned(K_.grouped_mm_3d2d, a, b, offs, (16, n_total), torch.bfloat16)
    check(out, a, b, offs, 64, path="mfma")
    k_total = tot + (-tot % 8)
    a2, b2 = rnd(gen, 16, k_total), rnd(gen, k_total, 24)
    with K_.forced_path("mfma"):
        out2 = run_poisoned(K_.grouped_mm_2d2d, a2, b2, offs, (1023, 16, 24), torch.bfloat16)
    check(out2, a2, b2, offs, path="mfma")


def test_fp32_epilogue_for_bf16_inputs_through_the_launcher():
    """The public function keeps the reference's dtype rule; the launcher honours out.dtype."""
    gen = torch.Generator().manual_seed(37)
    sizes = [40, 0, 88]
    a, b = rnd(gen, 64, 128), rnd(gen, 128, 72)
    out = run_poisoned(K_.grouped_mm_2d2d, a, b, offs_of(sizes), (3, 64, 72), torch.float32)
    want = oracle.grouped_mm(a, b, offs_of(sizes), out_dtype=torch.float32)
    torch.testing.assert_close(out, want, rtol=1e-4, atol=1e-4)
    with pytest.raises(RuntimeError, match="output dtype must match"):
        grouped_mm(a.to(DEV), b.to(DEV), offs=offs_of(sizes).to(DEV), out_dtype=torch.float32)


def test_non_finite_values_stay_inside_their_group():
    """Elements of a neighbouring group must never enter a product, not even multiplied by zero:
    poison one group's rows / k range with NaN and Inf and check every other group is untouched."""
    gen = torch.Generator().manual_seed(53)
    sizes = [13, 70, 0, 131, 58]  # odd boundaries: k ranges start inside 16-byte chunks
    offs, tot = offs_of(sizes), sum(sizes)
    rng = oracle.group_ranges(offs.tolist())
    # 2D x 2D (jagged contraction), row-major A (K contiguous) and row-major B
    a, b = rnd(gen, 264, tot), rnd(gen, tot, 272)
    s, e = rng[1]
    a[:, s:e] = float("nan")
    b[s:e, :] = float("inf")
    for path, cfg in (("mfma", 1), ("mfma", 0), ("generic", -1)):
        with K_.forced_path(path), K_.forced_mfma_config(cfg):
            out = run_poisoned(K_.grouped_mm_2d2d, a, b, offs, (len(sizes), 264, 272), torch.float32)
        want = oracle.grouped_mm(a, b, offs, out_dtype=torch.float32)
        for g in (0, 2, 3, 4):
            assert torch.isfinite(out[g]).all(), (path, cfg, g)
            torch.testing.assert_close(out[g], want[g], rtol=1.6e-2, atol=1e-2 * (131 / 64) ** 0.5)
        assert not torch.isfinite(out[1]).any()
    # 2D x 3D (jagged rows): a poisoned group poisons only its own rows
    a, b = rnd(gen, tot, 64), rnd(gen, len(sizes), 64, 48)
    a[s:e] = float("nan")
    out = run_poisoned(K_.grouped_mm_2d3d, a, b, offs, (tot, 48), torch.bfloat16)
    assert torch.isnan(out[s:e].float()).all()
    keep = torch.ones(tot, dtype=torch.bool)
    keep[s:e] = False
    assert torch.isfinite(out[keep].float()).all()


# ------------------------------------------------------------------ host rules on real tensors
def test_rules_on_gpu_tensors_and_shortcuts():
    a = torch.randn(8, 16, device=DEV, dtype=torch.bfloat16)
    b = torch.randn(2, 16, 8, device=DEV, dtype=torch.bfloat16)
    offs = torch.tensor([3, 8], device=DEV, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="Bias not supported yet"):
        grouped_mm(a, b, offs=offs, bias=torch.zeros(8, device=DEV))
    with pytest.raises(RuntimeError, match="CPU offs are not supported"):
        grouped_mm(a, b, offs=offs.cpu())
    with pytest.raises(RuntimeError, match="Have to provide offsets"):
        grouped_mm(a, b)
    with pytest.raises(RuntimeError, match="matrix batch sizes have to match"):
        grouped_mm(a, b, offs=torch.tensor([3, 5, 8], device=DEV, dtype=torch.int32))
    # K == 0 gives zeros, an empty output comes back empty (reference api.py:188-212)
    z = grouped_mm(a[:, :0], b[:, :0, :], offs=offs)
    assert z.shape == (8, 8) and (z == 0).all()
    e = grouped_mm(a[:0], b, offs=torch.zeros(2, device=DEV, dtype=torch.int32))
    assert e.shape == (0, 8)
    # positional and keyword call styles
    assert torch.equal(grouped_mm(a, b, offs), grouped_mm(mat_a=a, mat_b=b, offs=offs))


def test_runs_on_the_current_stream_without_sync():
    gen = torch.Generator().manual_seed(41)
    a, b = rnd(gen, 512, 256).to(DEV), rnd(gen, 4, 256, 256).to(DEV)
    offs = offs_of([100, 0, 300, 112]).to(DEV)
    ref = grouped_mm(a, b, offs=offs)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        got = grouped_mm(a, b, offs=offs)
    s.synchronize()
    assert torch.equal(got, ref)


# ------------------------------------------------------------------ backward (composition of forwards)
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
def test_backward_fp32_matches_autograd_of_the_loop(variant):
    gen = torch.Generator().manual_seed(43)
    sizes = [0, 7, 1, 13, 0, 11]
    G, tot, offs = len(sizes), sum(sizes), offs_of(sizes)
    f32 = torch.float32
    if variant == "2d3d":
        a, b = rnd(gen, tot, 29, dtype=f32), rnd(gen, G, 29, 31, dtype=f32)
    elif variant == "3d3d":
        a, b, offs = rnd(gen, 3, 17, 19, dtype=f32), rnd(gen, 3, 19, 23, dtype=f32), None
    elif variant == "2d2d":
        a, b = rnd(gen, 19, tot, dtype=f32), rnd(gen, tot, 21, dtype=f32)
    else:
        a, b = rnd(gen, G, 23, 17, dtype=f32), rnd(gen, 17, tot, dtype=f32)
    ad, bd = a.to(DEV).requires_grad_(), b.to(DEV).requires_grad_()
    out = grouped_mm(ad, bd, offs=None if offs is None else offs.to(DEV))
    w = torch.randn(out.shape, generator=gen)
    (out * w.to(DEV)).sum().backward()

    ar, br = a.clone().requires_grad_(), b.clone().requires_grad_()
    rng = oracle.group_ranges(offs.tolist()) if offs is not None else None
    if variant == "2d3d":
        ref = torch.cat([ar[s:e] @ br[g] for g, (s, e) in enumerate(rng)])
    elif variant == "3d3d":
        ref = torch.bmm(ar, br)
    elif variant == "2d2d":
        ref = torch.stack([ar[:, s:e] @ br[s:e] for (s, e) in rng])
    else:
        ref = torch.cat([ar[g] @ br[:, s:e] for g, (s, e) in enumerate(rng)], dim=1)
    (ref * w).sum().backward()
    torch.testing.assert_close(out.detach().cpu(), ref.detach(), rtol=3e-4, atol=3e-4)
    torch.testing.assert_close(ad.grad.cpu(), ar.grad, rtol=8e-4, atol=8e-4)
    torch.testing.assert_close(bd.grad.cpu(), br.grad, rtol=8e-4, atol=8e-4)


# ------------------------------------------------------------------ benchmark workloads, full size
def _sizes(golden_dir, key):
    with open(os.path.join(golden_dir, "group_sizes.json")) as f:
        return json.load(f)[key]


def _full_check_2d3d(out, a, b, offs_list, k, chunk=2048):
    """The whole output against the oracle, group by group and in row chunks (bounded host memory)."""
    got = out.cpu()
    for g, (s, e) in enumerate(oracle.group_ranges(offs_list)):
        if e == s:
            continue
        bg = b[g].float()
        for r0 in range(s, e, chunk):
            r1 = min(e, r0 + chunk)
            want = (a[r0:r1].float() @ bg).to(out.dtype)
            oracle.assert_close(got[r0:r1], want, k, what=f"rows {r0}:{r1} group {g}")


def test_mixtral_up_projection_full_size(golden_dir):
    sizes = _sizes(golden_dir, "mixtral_top2_g8")
    offs = offs_of(sizes)
    gen = torch.Generator().manual_seed(1)
    a = rnd(gen, 16384, 4096)
    b = rnd(torch.Generator().manual_seed(2), 8, 4096, 14336, scale=0.02)
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.full((16384, 14336), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(ad, bd, offs.to(DEV), out)
    assert K_.last_path() == "mfma"
    assert not torch.isnan(out.float()).any()
    _full_check_2d3d(out, a, b, offs.tolist(), 4096)     # every element, 1.9 TFLOP on the host
    # size-independent properties: splitting every group in two (same weights) must reproduce the same
    # rows bit for bit
    halves, idx = [], []
    for g, s in enumerate(sizes):
        halves += [s // 2, s - s // 2]
        idx += [g, g]
    # (with no tile cut along K: the two launches have different tile lists, and a cut tile adds its partial
    # sums in another order than an uncut one)
    with K_.tail_split(False):
        out2 = grouped_mm(ad, bd[idx], offs=offs_of(halves).to(DEV))
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    # linearity in A: f(2a) == 2 f(a) exactly in bf16 (power-of-two scaling)
    out3 = grouped_mm(ad * 2, bd, offs=offs.to(DEV))
    assert torch.equal((out * 2).view(torch.int16), out3.view(torch.int16))
    # against the generic family on a band that crosses a group boundary
    with K_.forced_path("generic"):
        ref_band = grouped_mm(ad[4700:4900], bd[:2], offs=torch.tensor([112, 200], dtype=torch.int32, device=DEV))
    oracle.assert_close(out[4700:4900].cpu(), ref_band.cpu(), 4096)


def test_mixtral_up_projection_full_size_column_major_weights(golden_dir):
    """The weights as a linear layer stores them, [G, N, K] viewed transposed (B contiguous along K): whole
    output against the oracle, and the same bits as the row-major launch (same K order)."""
    sizes = _sizes(golden_dir, "mixtral_top2_g8")
    offs = offs_of(sizes)
    a = rnd(torch.Generator().manual_seed(1), 16384, 4096)
    b = rnd(torch.Generator().manual_seed(2), 8, 4096, 14336, scale=0.02)
    ad, bd = a.to(DEV), b.to(DEV)
    b_nk = bd.transpose(1, 2).contiguous()           # [8, 14336, 4096]
    out = torch.full((16384, 14336), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(ad, b_nk.transpose(1, 2), offs.to(DEV), out)
    assert K_.last_path() == "mfma" and K_._lib.load().gmm_last_mfma_config() == 1
    assert not torch.isnan(out.float()).any()
    _full_check_2d3d(out, a, b, offs.tolist(), 4096)
    ref = torch.empty_like(out)
    K_.grouped_mm_2d3d(ad, bd, offs.to(DEV), ref)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("b_col", [False, True])
def test_fine_grained_moe_full_size(golden_dir, b_col):
    sizes = _sizes(golden_dir, "fine_grained_top8_g128")
    offs = offs_of(sizes)
    a = rnd(torch.Generator().manual_seed(1), 32768, 2048)
    b = rnd(torch.Generator().manual_seed(2), 128, 2048, 768, scale=0.02)
    bd = b.to(DEV)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((32768, 768), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(a.to(DEV), bd, offs.to(DEV), out)
    assert K_.last_path() == "mfma"
    want = oracle.grouped_mm(a, b, offs)  # 0.1 TFLOP: a few seconds on the host
    assert not torch.isnan(out.float()).any()
    oracle.assert_close(out.cpu(), want, 2048)


@pytest.mark.parametrize("b_col", [False, True])
def test_batched_3d3d_full_size(b_col):
    a = rnd(torch.Generator().manual_seed(1), 32, 1024, 1024)
    b = rnd(torch.Generator().manual_seed(2), 32, 1024, 4096, scale=0.02)
    bd = b.to(DEV)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((32, 1024, 4096), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_3d3d(a.to(DEV), bd, out)
    assert K_.last_path() == "mfma"
    got = out.cpu()
    for g in range(32):                                   # every batch, every element
        want = (a[g].float() @ b[g].float()).to(torch.bfloat16)
        oracle.assert_close(got[g], want, 1024, what=f"batch {g}")


def test_k_grouped_weight_gradient_full_size(golden_dir):
    sizes = _sizes(golden_dir, "mixtral_top2_g8")
    offs = offs_of(sizes)
    a = rnd(torch.Generator().manual_seed(1), 4096, 16384)
    b = rnd(torch.Generator().manual_seed(2), 16384, 14336)
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.full((8, 4096, 14336), float("nan"), device=DEV, dtype=torch.float32)
    K_.grouped_mm_2d2d(ad, bd, offs.to(DEV), out)
    assert K_.last_path() == "mfma"
    assert not torch.isnan(out).any()
    total = torch.zeros(4096, 14336)
    for g, (s, e) in enumerate(oracle.group_ranges(offs.tolist())):   # every group, every element
        got = out[g].cpu()
        want = a[:, s:e].float() @ b[s:e].float()
        oracle.assert_close(got, want, e - s, what=f"group {g}")
        total += got
    # the groups partition K: their sum is the plain product
    torch.testing.assert_close(total, a.float() @ b.float(), rtol=1.6e-2, atol=1e-2 * (16384 / 64) ** 0.5)
