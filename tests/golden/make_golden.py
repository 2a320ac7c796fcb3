"""Writes the committed fixtures of tests/golden/ with stock torch on the CPU.

    python tests/golden/make_golden.py

* group_sizes.json -- the group-size lists of the benchmark workloads, from the
  seeded recipes (so they do not depend on RNG drift between torch builds).
* small_cases.npz  -- inputs (bf16 bit patterns) and expected outputs for one
  small case per variant, with the size lists the reference's tests use
  (tests/test_grouped_mm.py:23, :37, :75, :114 of the reference).  Expected
  outputs come from torch's own CPU ``torch.nn.functional.grouped_mm`` (a
  library routine), not from this repository's oracle, so they pin the oracle.
Nothing here imports the reference or this repository's kernels.
"""
import json
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def mixtral_sizes():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(8192, 8, generator=g)
    logits[:, 0] += 1.0
    idx = torch.topk(logits, 2, dim=1).indices.reshape(-1)
    return torch.bincount(idx, minlength=8).tolist()


def fine_grained_sizes():
    g = torch.Generator().manual_seed(0)
    pop = 3.0 * torch.randn(128, generator=g)
    u = torch.rand(4096, 128, generator=g)
    gumbel = -torch.log(-torch.log(u))
    idx = torch.topk(pop + gumbel, 8, dim=1).indices.reshape(-1)
    return torch.bincount(idx, minlength=128).tolist()


def bits(t):
    return t.contiguous().view(torch.int16).numpy().astype(np.uint16)


def main():
    sizes = {
        "readme_2d3d": [0, 7, 1, 13, 0, 11],
        "mixtral_top2_g8": mixtral_sizes(),
        "fine_grained_top8_g128": fine_grained_sizes(),
    }
    assert sum(sizes["mixtral_top2_g8"]) == 16384
    assert sum(sizes["fine_grained_top8_g128"]) == 32768
    with open(os.path.join(HERE, "group_sizes.json"), "w") as f:
        json.dump(sizes, f, indent=1)

    out = {}
    gen = torch.Generator().manual_seed(1234)

    def rnd(*shape):
        return torch.randn(*shape, generator=gen).to(torch.bfloat16)

    # 2D x 3D, README shape
    offs = torch.tensor(sizes["readme_2d3d"]).cumsum(0).to(torch.int32)
    a, b = rnd(32, 64), rnd(6, 64, 48)
    out.update(a_2d3d=bits(a), b_2d3d=bits(b), offs_2d3d=offs.numpy(), out_2d3d=bits(F.grouped_mm(a, b, offs=offs)))
    # 3D x 3D
    a, b = rnd(4, 32, 64), rnd(4, 64, 48)
    out.update(a_3d3d=bits(a), b_3d3d=bits(b), out_3d3d=bits(F.grouped_mm(a, b)))
    # 2D x 2D, jagged contraction with an empty group
    offs = torch.tensor([7, 0, 1, 13, 11]).cumsum(0).to(torch.int32)
    a, b = rnd(16, 32), rnd(32, 24)
    out.update(a_2d2d=bits(a), b_2d2d=bits(b), offs_2d2d=offs.numpy(), out_2d2d=bits(F.grouped_mm(a, b, offs=offs)))
    # 3D x 2D, jagged columns with an empty group
    a, b = rnd(5, 32, 48), rnd(48, 32)
    out.update(a_3d2d=bits(a), b_3d2d=bits(b), offs_3d2d=offs.numpy(), out_3d2d=bits(F.grouped_mm(a, b, offs=offs)))
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), **out)
    print({k: len(v) for k, v in sizes.items()}, sizes["mixtral_top2_g8"])


if __name__ == "__main__":
    main()
