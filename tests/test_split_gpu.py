"""Tiles of a sparse last round cut along the contraction (the split workspace): parity with the oracle on
every variant and layout, exact ownership, run-to-run identical bits, and the down projection at full size.

The reference launches one program per tile (reference kernels.py:636-659) and has no such path; what must
hold is the reference's own bar for the result (tests/test_grouped_mm.py tolerances) whether or not a tile was
cut, and that cutting never changes which elements are written."""
import json
import os

import pytest
import torch

from grouped_mm_bf16_amd import _lib, grouped_mm, moe
from grouped_mm_bf16_amd import kernels as K_
from oracle import grouped_mm_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def offs_of(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def rnd(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def as_layout(t, col_major):
    """Same values, column-major storage in the last two dimensions."""
    return t.transpose(-2, -1).contiguous().transpose(-2, -1) if col_major else t


def launch(variant, a, b, offs, out):
    fn = {"2d3d": K_.grouped_mm_2d3d, "3d3d": K_.grouped_mm_3d3d, "2d2d": K_.grouped_mm_2d2d, "3d2d": K_.grouped_mm_3d2d}[variant]
    if offs is None:
        fn(a, b, out)
    else:
        fn(a, b, offs, out)


def n_parts_expected(sizes, jag, M, N, K, tall=256, shrt=64, align=1):
    """How many parts the launch cuts its last round into, from the host mirror of the tile list."""
    import numpy as np
    lib = _lib.load()
    offs = np.cumsum(sizes).astype(np.int32) if jag else np.zeros(1, np.int32)
    cus = torch.cuda.get_device_properties(0).multi_processor_count // 8 * 8
    parts = (lib.gmm_workspace_bytes() - 4096) // 262144
    n = lib.gmm_host_tile_list3(offs.ctypes.data, len(sizes), jag, M, N, K, tall, shrt, 256, align, 1, cus, parts, 0, None, 0)
    rec = np.zeros((n, 12), np.int32)
    lib.gmm_host_tile_list3(offs.ctypes.data, len(sizes), jag, M, N, K, tall, shrt, 256, align, 1, cus, parts, 0, rec.ctypes.data, n)
    return int((rec[:, 11] > 1).sum())


CASES = {   # variant -> (sizes, a shape, b shape, out shape): few tiles, long contraction
    "2d3d": ([300, 0, 1, 255, 257, 33], (846, 6144), (6, 6144, 520), (846, 520)),
    "3d3d": (None, (3, 304, 6144), (3, 6144, 520), (3, 304, 520)),
    "3d2d": ([129, 0, 127, 700, 4], (5, 336, 6152), (6152, 960), (336, 960)),
}


@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "3d2d"])
@pytest.mark.parametrize("a_col,b_col", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("dtype,out_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                            (torch.bfloat16, torch.float32), (torch.float16, torch.float32)])
def test_split_tiles_match_the_oracle(variant, a_col, b_col, dtype, out_dtype):
    sizes, sa, sb, so = CASES[variant]
    if variant == "2d3d" and a_col:
        sizes = [s // 8 * 8 for s in sizes]           # a column-major A wants aligned row ranges
        sa, so = (sum(sizes), sa[1]), (sum(sizes), so[1])
    gen = torch.Generator().manual_seed(11)
    a, b = rnd(gen, *sa, dtype=dtype), rnd(gen, *sb, dtype=dtype, scale=0.05)
    offs = None if sizes is None else offs_of(sizes)
    ad, bd = as_layout(a.to(DEV), a_col), as_layout(b.to(DEV), b_col)
    outs = []
    for on in (True, False, True):
        out = torch.full(so, float("nan"), device=DEV, dtype=out_dtype)
        with K_.tail_split(on), K_.forced_path("mfma"):
            launch(variant, ad, bd, None if offs is None else offs.to(DEV), out)
        torch.cuda.synchronize()
        assert K_.last_path() == "mfma"
        outs.append(out.cpu())
    want = oracle.grouped_mm(a, b, offs, out_dtype=out_dtype)
    for got in outs:
        assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), "ownership differs"
        oracle.assert_close_grouped(got, want, a, b, offs)
    # the same launch gives the same bits (the partial sums are added in a fixed order) ...
    assert torch.equal(outs[0].view(torch.int16 if out_dtype != torch.float32 else torch.int32),
                       outs[2].view(torch.int16 if out_dtype != torch.float32 else torch.int32))
    # ... and the launch did cut tiles: its fp32 output differs from the uncut one's in some last bits
    jag = {"2d3d": 1, "3d3d": 0, "3d2d": 2}[variant]
    M, N = (so[-2], so[-1])
    expect = n_parts_expected(sizes if sizes is not None else [0] * sa[0], jag, M if jag != 1 else sum(sizes),
                              N if jag != 2 else sum(sizes), sa[-1], tall=256 if a_col else 128, shrt=0 if a_col else 64,
                              align=8 if (jag == 2 or (jag == 1 and a_col)) else 1)
    assert expect > 0, "this case is meant to be cut"
    if out_dtype == torch.float32:
        assert not torch.equal(outs[0][~torch.isnan(outs[0])], outs[1][~torch.isnan(outs[1])])


def test_jagged_contraction_is_never_cut():
    gen = torch.Generator().manual_seed(12)
    sizes = [3000, 0, 3144]
    a, b = rnd(gen, 300, 6144), rnd(gen, 6144, 520, scale=0.05)
    outs = []
    for on in (True, False):
        out = torch.full((3, 300, 520), float("nan"), device=DEV, dtype=torch.float32)
        with K_.tail_split(on):
            K_.grouped_mm_2d2d(a.to(DEV), b.to(DEV), offs_of(sizes).to(DEV), out)
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])
    oracle.assert_close_grouped(outs[0], oracle.grouped_mm(a, b, offs_of(sizes), out_dtype=torch.float32), a, b, offs_of(sizes))


def test_gathered_rows_with_split():
    """The token gather of the MoE up projection with tiles cut along K: bit-equal to the product of the
    materialised rows (same tile list, same cuts)."""
    gen = torch.Generator().manual_seed(13)
    sizes = [300, 0, 1, 255, 257, 33]
    x = rnd(gen, 500, 6144).to(DEV)
    idx = torch.randint(0, 500, (sum(sizes),), generator=gen, dtype=torch.int32).to(DEV)
    b = rnd(gen, 6, 6144, 520, scale=0.05).to(DEV)
    offs = offs_of(sizes).to(DEV)
    got = moe.grouped_mm_gathered(x, idx, b, offs)
    want = torch.empty_like(got)
    K_.grouped_mm_2d3d(x[idx.long()].contiguous(), b, offs, want)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    oracle.assert_close(got.cpu(), oracle.grouped_mm(x[idx.long()].cpu(), b.cpu(), offs.cpu()), 6144)


def test_workspace_is_left_clean_and_small_workspaces_are_honoured():
    """Direct calls through the C ABI: the header of the workspace is zero after every launch; a workspace
    with room for two parts per tile still cuts; one below the minimum (or none) launches uncut."""
    lib = _lib.load()
    gen = torch.Generator().manual_seed(14)
    a, b = rnd(gen, 300, 8192).to(DEV), rnd(gen, 8192, 512, scale=0.05).to(DEV)       # 4 tiles, 128 K tiles
    want = (a.float() @ b.float())
    stream = torch.cuda.current_stream().cuda_stream
    results = {}
    for slots in (0, 1, 12, 32):
        ws = torch.zeros(4096 + slots * 262144, dtype=torch.uint8, device=DEV)
        out = torch.empty(1, 300, 512, device=DEV, dtype=torch.float32)
        for _ in range(3):
            rc = lib.gmm_3d3d(a.data_ptr(), b.data_ptr(), out.data_ptr(), 1, 300, 512, 8192, 0, 8192, 1, 0, 512, 1,
                              300 * 512, 512, 1, _lib.DT_BF16, _lib.DT_F32, ws.data_ptr(), ws.numel(), stream)
            assert rc == 0
        torch.cuda.synchronize()
        assert int(ws[:4096].view(torch.int32).abs().sum()) == 0, "arrival / ticket counters must be back at zero"
        torch.testing.assert_close(out[0], want, rtol=1.6e-2, atol=0.12)
        results[slots] = out.cpu()
    rc = lib.gmm_3d3d(a.data_ptr(), b.data_ptr(), out.data_ptr(), 1, 300, 512, 8192, 0, 8192, 1, 0, 512, 1,
                      300 * 512, 512, 1, _lib.DT_BF16, _lib.DT_F32, None, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), results[0]) and torch.equal(results[0], results[1])   # too small: not cut
    assert not torch.equal(results[12], results[0]) and not torch.equal(results[32], results[12])  # 2 parts, 3 parts


def test_down_projection_full_size(golden_dir):
    """16384 x 14336 -> 4096 with the skewed Mixtral group sizes: the last round (64 tiles on 256 compute
    units) is cut; whole output against the oracle, ownership by NaN poisoning, identical bits twice."""
    with open(os.path.join(golden_dir, "group_sizes.json")) as f:
        sizes = json.load(f)["mixtral_top2_g8"]
    offs = offs_of(sizes)
    a = rnd(torch.Generator().manual_seed(1), 16384, 14336)
    b = rnd(torch.Generator().manual_seed(2), 8, 14336, 4096, scale=0.02)
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.full((16384, 4096), float("nan"), device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(ad, bd, offs.to(DEV), out)
    assert K_.last_path() == "mfma"
    got = out.cpu()
    assert not torch.isnan(got.float()).any()
    for g, (s, e) in enumerate(oracle.group_ranges(offs.tolist())):
        want = (a[s:e].float() @ b[g].float()).to(torch.bfloat16)
        oracle.assert_close(got[s:e], want, 14336, what=f"group {g}")
    out2 = torch.empty_like(out)
    K_.grouped_mm_2d3d(ad, bd, offs.to(DEV), out2)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    with K_.tail_split(False):
        out3 = grouped_mm(ad, bd, offs=offs.to(DEV))
    oracle.assert_close(out3.cpu(), got, 14336)
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert n_parts_expected(sizes, 1, 16384, 4096, 14336) == 256
        assert not torch.equal(out3.view(torch.int16), out.view(torch.int16))
