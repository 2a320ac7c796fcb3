"""Pins the CPU oracle (oracle/) before anything is checked against it.

Each check is chosen so that a plausible mistake in the oracle -- a wrong group
start, an off-by-one in the ownership search, a transposed operand, a missing
zero fill -- fails at least one of them:

* committed golden vectors made with torch's own CPU grouped_mm;
* torch's CPU ``torch.nn.functional.grouped_mm`` on fresh seeded inputs;
* an element-wise fp64 brute force written in C (different formulation);
* ``torch.searchsorted(right=True)`` for the ownership search;
* invariants the mathematics fixes.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bruteforce
from oracle import grouped_mm_oracle as oracle


def _from_bits(arr, shape):
    return torch.from_numpy(arr.astype(np.int16)).view(torch.bfloat16).reshape(shape)


def _offs(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def _rand(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


# ---------------------------------------------------------------- golden vectors
@pytest.mark.parametrize("name,a_shape,b_shape", [
    ("2d3d", (32, 64), (6, 64, 48)),
    ("3d3d", (4, 32, 64), (4, 64, 48)),
    ("2d2d", (16, 32), (32, 24)),
    ("3d2d", (5, 32, 48), (48, 32)),
])
def test_oracle_reproduces_golden_vectors(golden_dir, name, a_shape, b_shape):
    z = np.load(os.path.join(golden_dir, "small_cases.npz"))
    a = _from_bits(z[f"a_{name}"], a_shape)
    b = _from_bits(z[f"b_{name}"], b_shape)
    offs = torch.from_numpy(z[f"offs_{name}"]) if f"offs_{name}" in z else None
    got = oracle.grouped_mm(a, b, offs)
    want = _from_bits(z[f"out_{name}"], got.shape)
    owned = ~torch.isnan(got.float())
    # bf16 results of the same fp32 sums: identical bits wherever a group owns the element
    assert torch.equal(got[owned].view(torch.int16), want[owned].view(torch.int16))
    if name in ("2d2d",):
        assert owned.all()
        assert (got[1] == 0).all()  # the empty group is an all-zero slab


def test_group_size_fixtures_match_their_recipes(golden_dir):
    import json
    with open(os.path.join(golden_dir, "group_sizes.json")) as f:
        sizes = json.load(f)
    assert sizes["readme_2d3d"] == [0, 7, 1, 13, 0, 11]
    mix = sizes["mixtral_top2_g8"]
    assert len(mix) == 8 and sum(mix) == 16384 and mix[0] == max(mix)
    fine = sizes["fine_grained_top8_g128"]
    assert len(fine) == 128 and sum(fine) == 32768
    assert fine.count(0) > 0 and fine.count(1) > 0  # "includes empty and 1-row groups"


# ---------------------------------------------------------------- library cross-check
def _same_up_to_one_ulp(got, want):
    """torch's CPU grouped_mm sums in another order than one fp32 matmul, so a sum
    that sits on a rounding boundary may land on the neighbouring bf16 value: allow
    one unit in the last place on a handful of elements, nothing more."""
    g, w = got.view(torch.int16).to(torch.int32), want.view(torch.int16).to(torch.int32)
    diff = (g - w).abs()
    assert int(diff.max()) <= 1
    assert int((diff > 0).sum()) <= max(1, got.numel() // 500)


@pytest.mark.parametrize("seed", [0, 1])
def test_oracle_equals_torch_cpu_grouped_mm(seed):
    gen = torch.Generator().manual_seed(seed)
    sizes = [16, 0, 8, 40, 0, 24]
    offs = _offs(sizes)
    a, b = _rand(gen, 88, 128), _rand(gen, 6, 128, 64)
    _same_up_to_one_ulp(oracle.grouped_mm(a, b, offs), F.grouped_mm(a, b, offs=offs))
    a, b = _rand(gen, 3, 24, 64), _rand(gen, 3, 64, 40)
    _same_up_to_one_ulp(oracle.grouped_mm(a, b), F.grouped_mm(a, b))
    a, b = _rand(gen, 24, 88), _rand(gen, 88, 40)
    _same_up_to_one_ulp(oracle.grouped_mm(a, b, offs), F.grouped_mm(a, b, offs=offs))
    a, b = _rand(gen, 6, 24, 64), _rand(gen, 64, 88)
    _same_up_to_one_ulp(oracle.grouped_mm(a, b, offs), F.grouped_mm(a, b, offs=offs))


def test_oracle_column_major_b_equals_row_major_b():
    gen = torch.Generator().manual_seed(5)
    a = _rand(gen, 4, 16, 32)
    b = _rand(gen, 4, 32, 24)
    b_col = b.transpose(-2, -1).contiguous().transpose(-2, -1)
    assert not b_col.is_contiguous()
    assert torch.equal(oracle.grouped_mm(a, b).view(torch.int16), oracle.grouped_mm(a, b_col).view(torch.int16))


# ---------------------------------------------------------------- brute force (C, fp64)
@pytest.mark.parametrize("variant", ["2d3d", "3d3d", "2d2d", "3d2d"])
@pytest.mark.parametrize("sizes", [[0, 7, 1, 13, 0, 11], [5, 0, 7, 0, 3, 9], [1, 0, 1, 0, 1, 0]])
def test_oracle_matches_fp64_bruteforce(variant, sizes):
    gen = torch.Generator().manual_seed(len(sizes) + sum(sizes))
    G, tot = len(sizes), sum(sizes)
    offs = _offs(sizes)
    if variant == "2d3d":
        a, b = _rand(gen, tot, 33), _rand(gen, G, 33, 29)
    elif variant == "3d3d":
        a, b, offs = _rand(gen, G, 17, 19), _rand(gen, G, 19, 23), None
    elif variant == "2d2d":
        a, b = _rand(gen, 19, tot), _rand(gen, tot, 21)
    else:
        a, b = _rand(gen, G, 23, 17), _rand(gen, 17, tot)
    got = oracle.grouped_mm(a, b, offs, out_dtype=torch.float32)
    want = bruteforce.grouped_mm_f64(a, b, offs)
    assert torch.equal(torch.isnan(got), torch.isnan(want))  # same ownership
    m = ~torch.isnan(want)
    torch.testing.assert_close(got[m].double(), want[m], rtol=1e-5, atol=1e-5)


def test_bruteforce_2d3d_by_hand():
    # one row per group, identity-like B: the result can be read off by eye
    a = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
    b = torch.stack([torch.eye(2), 2 * torch.eye(2), torch.tensor([[0.0, 1.0], [1.0, 0.0]])])
    offs = torch.tensor([1, 2, 3], dtype=torch.int32)
    want = torch.tensor([[1.0, 2.0], [6.0, 8.0], [6.0, 5.0]], dtype=torch.float64)
    assert torch.equal(bruteforce.grouped_mm_f64(a, b, offs), want)
    assert torch.equal(oracle.grouped_mm(a, b, offs).double(), want)


# ---------------------------------------------------------------- ownership search
def test_upper_bound_matches_searchsorted_right():
    rng = np.random.default_rng(0)
    for _ in range(50):
        G = int(rng.integers(1, 40))
        sizes = rng.integers(0, 5, size=G)
        offs = np.cumsum(sizes).astype(np.int32)
        idx = torch.arange(0, int(offs[-1]) + 3)
        want = torch.searchsorted(torch.from_numpy(offs), idx.to(torch.int32), right=True).tolist()
        assert [oracle.upper_bound(offs, int(i)) for i in idx] == want
        assert [bruteforce.upper_bound(offs, int(i)) for i in idx] == want


def test_upper_bound_1023_groups_alternating():
    sizes = [1 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    offs = np.cumsum(sizes).astype(np.int32)
    for i in range(int(offs[-1])):
        g = oracle.upper_bound(offs, i)
        assert sizes[g] == 1 and offs[g] == i + 1
    assert oracle.upper_bound(offs, int(offs[-1])) == 1023


# ---------------------------------------------------------------- rounding
def test_c_bf16_rounding_matches_torch():
    xs = torch.tensor([0.0, 1.0, 1.00390625, 1.01171875, -3.14159, 65504.0, 1e-40, float("inf"), 3.3895314e38])
    for x in xs.tolist():
        want = torch.tensor(x, dtype=torch.float32).to(torch.bfloat16).view(torch.int16).item() & 0xFFFF
        assert bruteforce.f32_to_bf16_bits(x) == want
    assert bruteforce.f32_to_bf16_bits(float("nan")) & 0x7FC0 == 0x7FC0


# ---------------------------------------------------------------- invariants
def test_permuting_groups_permutes_rows():
    gen = torch.Generator().manual_seed(7)
    sizes = [3, 0, 5, 2]
    a, b = _rand(gen, 10, 16), _rand(gen, 4, 16, 8)
    out = oracle.grouped_mm(a, b, _offs(sizes))
    perm = [2, 0, 3, 1]
    starts = [0, 3, 3, 8]
    rows = torch.cat([torch.arange(starts[g], starts[g] + sizes[g]) for g in perm])
    out_p = oracle.grouped_mm(a[rows], b[perm], _offs([sizes[g] for g in perm]))
    assert torch.equal(out_p.view(torch.int16), out[rows].view(torch.int16))


def test_splitting_a_group_changes_nothing():
    gen = torch.Generator().manual_seed(8)
    a, b = _rand(gen, 12, 16), _rand(gen, 2, 16, 8)
    whole = oracle.grouped_mm(a, b, _offs([7, 5]))
    split = oracle.grouped_mm(a, b[[0, 0, 1]], _offs([3, 4, 5]))
    assert torch.equal(whole.view(torch.int16), split.view(torch.int16))


def test_3d3d_is_2d3d_with_uniform_groups():
    gen = torch.Generator().manual_seed(9)
    a, b = _rand(gen, 3, 5, 16), _rand(gen, 3, 16, 8)
    flat = oracle.grouped_mm(a.reshape(15, 16), b, _offs([5, 5, 5]))
    assert torch.equal(oracle.grouped_mm(a, b).reshape(15, 8).view(torch.int16), flat.view(torch.int16))


def test_2d2d_groups_sum_to_plain_matmul_and_empty_is_zero():
    gen = torch.Generator().manual_seed(10)
    a, b = _rand(gen, 6, 20), _rand(gen, 20, 7)
    out = oracle.grouped_mm(a, b, _offs([4, 0, 9, 7]), out_dtype=torch.float32)
    assert (out[1] == 0).all()
    torch.testing.assert_close(out.sum(0), a.float() @ b.float(), rtol=1e-5, atol=1e-5)


def test_3d2d_is_columnwise_2d3d_transposed():
    # (A[g] @ B[:, cols])^T == B[:, cols]^T @ A[g]^T : 3D x 2D is 2D x 3D on transposes
    gen = torch.Generator().manual_seed(11)
    sizes = [4, 0, 3, 5]
    a, b = _rand(gen, 4, 6, 16), _rand(gen, 16, 12)
    out = oracle.grouped_mm(a, b, _offs(sizes), out_dtype=torch.float32)
    out_t = oracle.grouped_mm(b.t().contiguous(), a.transpose(1, 2).contiguous(), _offs(sizes), out_dtype=torch.float32)
    torch.testing.assert_close(out, out_t.t(), rtol=1e-6, atol=1e-6)


def test_unowned_elements_are_left_alone():
    gen = torch.Generator().manual_seed(12)
    a, b = _rand(gen, 10, 16), _rand(gen, 2, 16, 8)
    out = oracle.grouped_mm(a, b, _offs([3, 4]))  # rows 7..9 belong to nobody
    assert torch.isnan(out[7:].float()).all() and not torch.isnan(out[:7].float()).any()
