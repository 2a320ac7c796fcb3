"""The tile scheduler (csrc/gmm_sched.h), run on the host exactly as the kernels
run it on the device: every element a group owns is covered by exactly one tile
of that group, nothing else is covered, and the XCD renumbering is a permutation."""
import ctypes

import numpy as np
import pytest

from grouped_mm_bf16_amd import _lib

NONE, ROWS, COLS, CONTRACTION = 0, 1, 2, 3


def tile_list(sizes, jag, M, N, K, bm, bn, align=1, remap=0, num_wg=256):
    lib = _lib.load()
    offs = np.cumsum(sizes).astype(np.int32) if jag != NONE else np.zeros(1, np.int32)
    G = len(sizes)
    n = lib.gmm_host_tile_list(offs.ctypes.data, G, jag, M, N, K, bm, bn, align, remap, num_wg, None, 0)
    assert n >= 0
    rec = np.zeros((max(n, 1), 9), np.int32)
    n2 = lib.gmm_host_tile_list(offs.ctypes.data, G, jag, M, N, K, bm, bn, align, remap, num_wg, rec.ctypes.data, n)
    assert n2 == n
    return rec[:n]


def coverage(rec, G, M, N, bm, bn, per_group_out):
    """count[g or 0, m, n] = number of tiles that store element (m, n)."""
    cnt = np.zeros((G if per_group_out else 1, M, N), np.int32)
    for g, m0, n0, m_lo, m_hi, n_lo, n_hi, _, _ in rec:
        r0, r1 = max(m0, m_lo), min(m0 + bm, m_hi)
        c0, c1 = max(n0, n_lo), min(n0 + bn, n_hi)
        if r1 > r0 and c1 > c0:
            cnt[g if per_group_out else 0, r0:r1, c0:c1] += 1
    return cnt


SIZE_LISTS = [
    [0, 7, 1, 13, 0, 11], [32, 32, 32], [10, 10, 10, 2], [31, 1, 31], [40, 30, 10, 7],
    [32, 16, 0, 0, 0], [1, 0] * 6, [5, 0, 7, 0, 3, 9], [300, 0, 1, 255, 256, 257, 33], [0, 0, 0],
]


@pytest.mark.parametrize("sizes", SIZE_LISTS)
@pytest.mark.parametrize("bm,align", [(32, 1), (256, 1), (32, 8), (256, 8), (16, 8)])
def test_jagged_rows_exact_cover(sizes, bm, align):
    M, N = sum(sizes), 70
    if M == 0:
        assert len(tile_list(sizes, ROWS, 0, N, 16, bm, 64, align)) == 0
        return
    rec = tile_list(sizes, ROWS, M, N, 16, bm, 64, align)
    cnt = coverage(rec, len(sizes), M, N, bm, 64, False)
    assert (cnt == 1).all()
    offs = np.cumsum(sizes)
    for g, m0, n0, m_lo, m_hi, *_ in rec:
        assert sizes[g] > 0 and m_hi == offs[g] and m_lo == offs[g] - sizes[g]
        assert m0 % align == 0 and m0 + bm > m_lo and m0 < m_hi  # no tile is pure waste
        assert n0 % 64 == 0


@pytest.mark.parametrize("sizes", SIZE_LISTS)
@pytest.mark.parametrize("bn,align", [(64, 1), (256, 8)])
def test_jagged_columns_exact_cover(sizes, bn, align):
    M, N = 50, sum(sizes)
    if N == 0:
        return
    rec = tile_list(sizes, COLS, M, N, 16, 32, bn, align)
    assert (coverage(rec, len(sizes), M, N, 32, bn, False) == 1).all()
    assert all(sizes[r[0]] > 0 for r in rec)


@pytest.mark.parametrize("sizes", SIZE_LISTS)
def test_jagged_contraction_covers_every_group_including_empty(sizes):
    M, N, K = 70, 90, sum(sizes)
    rec = tile_list(sizes, CONTRACTION, M, N, K, 64, 64)
    cnt = coverage(rec, len(sizes), M, N, 64, 64, True)
    assert (cnt == 1).all()  # also the empty groups: they must be zero-filled
    offs = np.cumsum(sizes)
    for r in rec:
        assert r[7] == offs[r[0]] - sizes[r[0]] and r[8] == offs[r[0]]


def test_batched_grid():
    rec = tile_list([0] * 5, NONE, 100, 130, 16, 64, 64)
    assert len(rec) == 5 * 2 * 3
    assert (coverage(rec, 5, 100, 130, 64, 64, True) == 1).all()


def test_1023_groups_alternating():
    sizes = [1 if i % 2 == 0 else 0 for i in range(1023)]
    sizes[-1] = 0
    M = sum(sizes)
    rec = tile_list(sizes, ROWS, M, 8, 8, 256, 256)
    assert len(rec) == M and (coverage(rec, 1023, M, 8, 256, 256, False) == 1).all()
    assert sorted(r[0] for r in rec) == [g for g in range(1023) if sizes[g]]


@pytest.mark.parametrize("total_like", [[5000], [256 * 3], [1], [255, 300, 7, 1000]])
def test_xcd_renumbering_is_a_permutation(total_like):
    sizes = total_like
    plain = tile_list(sizes, ROWS, sum(sizes), 512, 16, 16, 64, 1, remap=0)
    remap = tile_list(sizes, ROWS, sum(sizes), 512, 16, 16, 64, 1, remap=1, num_wg=256)
    assert len(plain) == len(remap)
    key = lambda r: tuple(r)
    assert sorted(map(key, plain)) == sorted(map(key, remap))
    # workgroups of one XCD (ids equal mod 8) get consecutive tiles of the plain order
    order = {key(r): i for i, r in enumerate(plain)}
    span = remap[:256]
    for x in range(8):
        ids = [order[key(r)] for r in span[x::8]]
        assert ids == list(range(ids[0], ids[0] + len(ids)))


def test_malformed_offsets_never_leave_the_tensor():
    lib = _lib.load()
    offs = np.array([5, 3, 100, -4, 20], np.int32)  # decreasing, too large, negative
    rec = np.zeros((64, 9), np.int32)
    n = lib.gmm_host_tile_list(offs.ctypes.data, 5, ROWS, 20, 8, 8, 16, 16, 1, 0, 8, rec.ctypes.data, 64)
    assert 0 <= n <= 64
    for g, m0, n0, m_lo, m_hi, *_ in rec[:n]:
        assert 0 <= m_lo <= m_hi <= 20 and 0 <= m0 < 20


def test_random_lists_exact_cover():
    rng = np.random.default_rng(1)
    for _ in range(60):
        G = int(rng.integers(1, 30))
        sizes = (rng.integers(0, 80, size=G) * (rng.random(G) > 0.3)).astype(int).tolist()
        if sum(sizes) == 0:
            continue
        bm = int(rng.choice([16, 32, 64, 256]))
        align = int(rng.choice([1, 8]))
        rec = tile_list(sizes, ROWS, sum(sizes), 40, 8, bm, 32, align, remap=int(rng.integers(0, 2)), num_wg=16)
        assert (coverage(rec, G, sum(sizes), 40, bm, 32, False) == 1).all()


# ---------------------------------------------------------------- two tile heights (assembly tile)
def tile_list2(sizes, jag, M, N, K, tall, shrt, align=1, remap=0, num_wg=256):
    lib = _lib.load()
    offs = np.cumsum(sizes).astype(np.int32) if jag != NONE else np.zeros(1, np.int32)
    G = len(sizes)
    n = lib.gmm_host_tile_list2(offs.ctypes.data, G, jag, M, N, K, tall, shrt, 256, align, remap, num_wg, None, 0)
    assert n >= 0
    rec = np.zeros((max(n, 1), 10), np.int32)
    assert lib.gmm_host_tile_list2(offs.ctypes.data, G, jag, M, N, K, tall, shrt, 256, align, remap, num_wg,
                                   rec.ctypes.data, n) == n
    return rec[:n]


def coverage2(rec, G, M, N, per_group_out):
    cnt = np.zeros((G if per_group_out else 1, M, N), np.int32)
    for g, m0, n0, m_lo, m_hi, n_lo, n_hi, _, _, rows in rec:
        r0, r1 = max(m0, m_lo), min(m0 + rows, m_hi)
        c0, c1 = max(n0, n_lo), min(n0 + 256, n_hi)
        assert r1 > r0 and c1 > c0, "a tile that stores nothing"
        cnt[g if per_group_out else 0, r0:r1, c0:c1] += 1
    return cnt


@pytest.mark.parametrize("sizes", SIZE_LISTS + [[4812, 1663, 1610, 1663, 1656, 1682, 1633, 1665], [129, 128, 127, 65, 64, 63, 1]])
@pytest.mark.parametrize("tall,shrt,align", [(256, 64, 1), (128, 64, 1), (256, 0, 1), (256, 0, 8), (256, 64, 8)])
def test_two_heights_jagged_rows_exact_cover(sizes, tall, shrt, align):
    M, N = sum(sizes), 300
    if M == 0:
        return
    rec = tile_list2(sizes, ROWS, M, N, 16, tall, shrt, align, remap=1, num_wg=16)
    assert (coverage2(rec, len(sizes), M, N, False) == 1).all()
    heights = set(int(r[9]) for r in rec)
    assert heights <= {tall, 2 * shrt, shrt}
    # tall tiles come first in the launch order when ids are not renumbered
    plain = tile_list2(sizes, ROWS, M, N, 16, tall, shrt, align)
    hs = [int(r[9]) for r in plain]
    assert hs == sorted(hs, reverse=True)
    # a remainder that fits one short tile never pays for a tall tile
    if shrt and align == 1:
        for g, sz in enumerate(sizes):
            rem = sz % tall
            mine = [r for r in plain if r[0] == g and r[2] == 0]
            if 0 < rem <= shrt:
                assert sorted(int(r[9]) for r in mine) == [shrt] + [tall] * (sz // tall)
            elif tall == 4 * shrt and 0 < rem <= 2 * shrt:
                assert sorted(int(r[9]) for r in mine) == [2 * shrt] + [tall] * (sz // tall)
            else:
                assert all(r[9] == tall for r in mine)


@pytest.mark.parametrize("sizes", SIZE_LISTS + [[129, 128, 127, 65, 64, 63, 1, 700]])
@pytest.mark.parametrize("tall,shrt,align", [(256, 64, 8), (128, 64, 8), (256, 0, 8), (256, 64, 1)])
def test_two_heights_jagged_columns_exact_cover(sizes, tall, shrt, align):
    """3D x 2D on the assembly tile: rows are split by height, every group has its own tile columns, and
    tile columns start at multiples of `align` elements."""
    N, M = sum(sizes), 330
    if N == 0:
        return
    rec = tile_list2(sizes, COLS, M, N, 16, tall, shrt, align, remap=1, num_wg=16)
    assert (coverage2(rec, len(sizes), M, N, False) == 1).all()
    for g, m0, n0, m_lo, m_hi, n_lo, n_hi, _, _, rows in rec:
        assert n0 % align == 0 and n0 <= max(n_lo, n0) and (m_lo, m_hi) == (0, M)
        assert rows in (tall, 2 * shrt, shrt)


@pytest.mark.parametrize("tall,shrt", [(256, 64), (128, 64), (256, 0)])
def test_two_heights_contraction_and_batched(tall, shrt):
    sizes = [7, 0, 1, 13, 11]
    rec = tile_list2(sizes, CONTRACTION, 330, 300, sum(sizes), tall, shrt)
    assert (coverage2(rec, 5, 330, 300, True) == 1).all()  # also the empty group
    offs = np.cumsum(sizes)
    for r in rec:
        assert r[7] == offs[r[0]] - sizes[r[0]] and r[8] == offs[r[0]]
    rec = tile_list2([0] * 5, NONE, 330, 300, 16, tall, shrt)
    assert (coverage2(rec, 5, 330, 300, True) == 1).all()


def test_two_heights_fine_grained_fixture(golden_dir):
    import json, os
    with open(os.path.join(golden_dir, "group_sizes.json")) as f:
        sizes = json.load(f)["fine_grained_top8_g128"]
    rec = tile_list2(sizes, ROWS, 32768, 768, 2048, 128, 64, remap=1, num_wg=256)
    assert (coverage2(rec, 128, 32768, 768, False) == 1).all()
    rows_paid = sum(int(r[9]) for r in rec if r[2] == 0)
    assert rows_paid < 1.2 * 32768  # 256-row tiles alone pay for 54784 rows here


# ---------------------------------------------------------------- last round cut along K (split workspace)
def tile_list3(sizes, jag, M, N, K, tall, shrt, max_parts, align=1, remap=1, num_wg=256, group_major=0):
    lib = _lib.load()
    offs = np.cumsum(sizes).astype(np.int32) if jag != NONE else np.zeros(1, np.int32)
    G = len(sizes)
    n = lib.gmm_host_tile_list3(offs.ctypes.data, G, jag, M, N, K, tall, shrt, 256, align, remap, num_wg, max_parts, group_major, None, 0)
    assert n >= 0
    rec = np.zeros((max(n, 1), 12), np.int32)
    assert lib.gmm_host_tile_list3(offs.ctypes.data, G, jag, M, N, K, tall, shrt, 256, align, remap, num_wg, max_parts,
                                   group_major, rec.ctypes.data, n) == n
    return rec[:n]


def k_coverage(rec, K):
    """Per output tile (group, m0, n0, rows): the K ranges of its records must partition [0, K) in part order."""
    by_tile = {}
    for r in rec:
        by_tile.setdefault((int(r[0]), int(r[1]), int(r[2]), int(r[9])), []).append((int(r[10]), int(r[7]), int(r[8]), int(r[11])))
    n_split = 0
    for key, parts in by_tile.items():
        parts.sort()
        assert [p[0] for p in parts] == list(range(len(parts))), key
        assert all(p[3] == len(parts) for p in parts), key
        assert parts[0][1] == 0 and parts[-1][2] == K, key
        for (_, _, hi, _), (_, lo, _, _) in zip(parts, parts[1:]):
            assert hi == lo and lo % 64 == 0
        assert all(hi - lo >= 24 * 64 or len(parts) == 1 for _, lo, hi, _ in parts)
        n_split += len(parts) > 1
    return by_tile, n_split


MIXTRAL = [4812, 1663, 1610, 1663, 1656, 1682, 1633, 1665]


def test_down_projection_tail_is_cut_four_ways():
    """16384 x 14336 -> 4096 on 256 workgroups: 1008 tall + 80 remainder tiles = 4 rounds + 64 tiles; the 64
    tiles of the fifth round become 256 parts of 56 K tiles each: one part per workgroup (five parts each would
    be 320, a second turn for 64 of them)."""
    whole = tile_list3(MIXTRAL, ROWS, 16384, 4096, 14336, 256, 64, 0)
    assert len(whole) == 1088 and (whole[:, 11] == 1).all()
    rec = tile_list3(MIXTRAL, ROWS, 16384, 4096, 14336, 256, 64, 512)
    assert len(rec) == 1024 + 4 * 64
    by_tile, n_split = k_coverage(rec, 14336)
    assert len(by_tile) == 1088 and n_split == 64
    assert (rec[:1024, 11] == 1).all() and (rec[1024:, 11] == 4).all()
    # without the K ranges the list is the unsplit one: same tiles, same owners
    assert (coverage2(whole[:, :10], 8, 16384, 4096, False) == 1).all()
    first_parts = rec[rec[:, 10] == 0][:, :10]
    assert (coverage2(first_parts, 8, 16384, 4096, False) == 1).all()
    # the parts come in ticket order: K part 0 of every tile of the round, then K part 1, ...
    assert (rec[1024:, 10] == np.repeat(np.arange(4), 64)).all()
    # a workspace too small for four parts per tile allows fewer
    rec = tile_list3(MIXTRAL, ROWS, 16384, 4096, 14336, 256, 64, 128)
    assert len(rec) == 1024 + 2 * 64


def test_up_projection_is_left_alone():
    """16384 x 4096 -> 14336: the last round holds 224 of 256 tiles; cutting them would cost more than it saves.
    Nor is a thinly filled last round of tiles with 64 K tiles cut: a part costs about 20 K tiles beyond its own
    (measured: 56 such tiles cut four ways take as long as uncut)."""
    rec = tile_list3(MIXTRAL, ROWS, 16384, 14336, 4096, 256, 64, 512)
    assert len(rec) == 3808 and (rec[:, 11] == 1).all()
    sizes = [256 * r for r in (20, 7, 6, 6, 6, 7, 6, 7)]          # 65 tile rows: 14 rounds + 56 tiles
    rec = tile_list3(sizes, ROWS, sum(sizes), 14336, 4096, 256, 64, 512)
    assert len(rec) == 65 * 56 and (rec[:, 11] == 1).all()
    rec = tile_list3(sizes, ROWS, sum(sizes), 14336, 8192, 256, 64, 512)   # twice the contraction: cut four ways
    assert len(rec) == 64 * 56 + 4 * 56 and set(rec[:, 11].tolist()) == {1, 4}


@pytest.mark.parametrize("jag,sizes,M,N", [(ROWS, [300, 0, 1, 255, 256, 257, 33], 1102, 700), (COLS, [129, 128, 127, 700], 330, 1084),
                                           (NONE, [0] * 3, 330, 300)])
@pytest.mark.parametrize("K", [1024, 1096, 4096, 16384])
@pytest.mark.parametrize("num_wg,max_parts", [(256, 512), (64, 128), (16, 32), (8, 5)])
def test_split_lists_cover_every_element_and_every_k(jag, sizes, M, N, K, num_wg, max_parts):
    rec = tile_list3(sizes, jag, M, N, K, 256, 64, max_parts, align=8 if jag == COLS else 1, num_wg=num_wg)
    by_tile, _ = k_coverage(rec, K)
    first_parts = rec[rec[:, 10] == 0][:, :10]
    G = len(sizes)
    assert (coverage2(first_parts, G, M, N, jag == NONE) == 1).all()
    unsplit = tile_list2(sizes, jag, M, N, K, 256, 64, align=8 if jag == COLS else 1, remap=1, num_wg=num_wg)
    assert len(by_tile) == len(unsplit)
    nparts = set(int(r[11]) for r in rec)
    assert len(nparts - {1}) <= 1 and max(nparts) <= 8
    if max(nparts) > 1:
        n_parts_total = int((rec[:, 11] > 1).sum())
        assert n_parts_total <= max_parts and len(rec) == len(unsplit) + n_parts_total - n_parts_total // max(nparts)


def test_contraction_jagged_lists_are_never_split():
    rec = tile_list3([4000, 5000, 7384], CONTRACTION, 330, 300, 16384, 256, 64, 512)
    assert (rec[:, 11] == 1).all()


@pytest.mark.parametrize("sizes", SIZE_LISTS + [MIXTRAL, [129, 128, 127, 65, 64, 63, 1]])
@pytest.mark.parametrize("tall,remap", [(256, 0), (128, 0), (128, 1)])
def test_group_major_order_covers_the_same_tiles(sizes, tall, remap):
    """Group by group: the same tiles as the tall-first order, every group's remainder tiles right after its
    tall tiles, groups in order."""
    M, N = sum(sizes), 600
    if M == 0:
        return
    a = tile_list3(sizes, ROWS, M, N, 64, tall, 64, 0, remap=remap, num_wg=16, group_major=1)
    b = tile_list3(sizes, ROWS, M, N, 64, tall, 64, 0, remap=remap, num_wg=16, group_major=0)
    assert sorted(map(tuple, a.tolist())) == sorted(map(tuple, b.tolist()))
    assert (coverage2(a[:, :10], len(sizes), M, N, False) == 1).all()
    if not remap:
        groups = [int(r[0]) for r in a]
        assert groups == sorted(groups)
        for g in set(groups):
            hs = [int(r[9]) for r in a if r[0] == g]
            assert hs == sorted(hs, reverse=True)


def test_fine_grained_fixture_group_major_with_split(golden_dir):
    import json, os
    with open(os.path.join(golden_dir, "group_sizes.json")) as f:
        sizes = json.load(f)["fine_grained_top8_g128"]
    rec = tile_list3(sizes, ROWS, 32768, 768, 2048, 128, 64, 512, group_major=1)
    assert (rec[:, 11] == 1).all()          # 32 K tiles: too short a contraction to cut
    assert (coverage2(rec[:, :10], 128, 32768, 768, False) == 1).all()


def fabric_floor_bytes(rec, K, num_wg=256, esz=2):
    """Bytes the launch order must pull through the fabric if an XCD's L2 keeps an operand panel exactly as long
    as the round that uses it: tiles are dealt round by round, workgroup w runs on XCD w % 8, and the tiles of
    one XCD in one round share every A row panel (group, first row) and B column panel (group, first column)
    they have in common.  Records in launch order, as gmm_host_tile_list2/3 return them."""
    total = 0
    for r0 in range(0, len(rec), num_wg):
        span = rec[r0:r0 + num_wg]
        for x in range(8):
            mine = span[x::8]
            a_panels = {(int(t[0]), int(t[1])): min(int(t[1]) + int(t[9]), int(t[4])) - max(int(t[1]), int(t[3])) for t in mine}
            b_panels = {(int(t[0]), int(t[2])): min(int(t[2]) + 256, int(t[6])) - max(int(t[2]), int(t[5])) for t in mine}
            total += (sum(a_panels.values()) + sum(b_panels.values())) * K * esz
    return total


def test_fabric_traffic_floor_of_the_mixtral_launch_order():
    """What the 8 x 4 blocks per XCD must fetch past the L2s on the benchmark's headline workload: 3.47 GB of
    operand panels for 1.07 GB of operands (every XCD reads all eight A panels of its band; a B panel is read by
    one XCD per band of its group; a 2 MB panel outlives no round in a 4 MB L2).  The FETCH_SIZE counter reads
    3.86 GB per launch on the device: 1.11 times this floor.  Without the XCD renumbering (a round's tiles dealt to the XCDs one by one)
    every XCD touches every panel of the round: 2.6 times as much."""
    def order(remap):
        # device order: tile ids 0 .. n - 1 in launch order after the renumbering, workgroup w takes id w of a round
        return tile_list3(MIXTRAL, ROWS, 16384, 14336, 4096, 256, 64, 0, remap=remap)
    blocked, plain = fabric_floor_bytes(order(1), 4096), fabric_floor_bytes(order(0), 4096)
    operands = (16384 * 4096 + 8 * 4096 * 14336) * 2
    assert 3.4e9 < blocked < 3.55e9, blocked
    assert plain > 2.4 * blocked
    assert blocked > 2.5 * operands
