"""Brute-force checks of the integer schedule functions (CPU)."""
import itertools
import numpy as np

import pytest

from oracle import schedule as S


@pytest.mark.parametrize("n_wg,xcds", [(8, 8), (64, 8), (100, 8), (3584, 8), (1024, 8), (7, 8), (1, 8), (305, 8), (96, 4)])
def test_chiplet_transform_is_bijection(n_wg, xcds):
    out = sorted(S.chiplet_transform(p, n_wg, xcds) for p in range(n_wg))
    assert out == list(range(n_wg))


@pytest.mark.parametrize("n_wg,xcds,chunk", [(64, 8, 4), (3584, 8, 64), (1024, 8, 64), (100, 8, 3), (8, 8, 1), (5, 8, 1),
                                             (256, 8, 32), (257, 8, 32), (1000, 8, 7), (17, 4, 2)])
def test_chiplet_transform_chunked_is_bijection(n_wg, xcds, chunk):
    out = sorted(S.chiplet_transform_chunked(p, n_wg, xcds, chunk) for p in range(n_wg))
    assert out == list(range(n_wg))


def test_chunked_gives_each_xcd_contiguous_chunks():
    # workgroup p runs on XCD p % 8; inside the chunked region an XCD's tiles come in runs of `chunk`
    n, x, c = 1024, 8, 16
    per_xcd = {}
    for p in range(n):
        per_xcd.setdefault(p % x, []).append(S.chiplet_transform_chunked(p, n, x, c))
    for xcd, tiles in per_xcd.items():
        for i in range(0, len(tiles) - c + 1, c):
            run = tiles[i:i + c]
            assert run == list(range(run[0], run[0] + c))


@pytest.mark.parametrize("tm,tn,gm", [(32, 112, 8), (4, 4, 8), (5, 7, 2), (1, 9, 8), (9, 1, 4), (13, 3, 8), (8, 8, 1)])
def test_group_m_swizzle_is_bijection(tm, tn, gm):
    seen = {S.tile_coords(t, tm, tn, gm) for t in range(tm * tn)}
    assert seen == set(itertools.product(range(tm), range(tn)))


def test_group_m_walks_columns_inside_a_group():
    assert [S.tile_coords(t, 4, 3, 2) for t in range(6)] == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2)]


@pytest.mark.parametrize("tiles,grid,ipt", [(64, 256, 112), (300, 256, 7), (5, 8, 3), (3, 7, 1), (10, 4, 5), (256, 256, 9),
                                            (1, 256, 100), (2, 256, 5)])
def test_streamk_covers_every_iteration_once(tiles, grid, ipt):
    sk_tiles = S.streamk_partition(tiles, grid)
    full = tiles - sk_tiles
    covered = {}
    publishers = {}
    for pid in range(grid):
        segs = S.streamk_segments(pid, grid, tiles, sk_tiles, ipt)
        n_publish = 0
        for tile, k0, k1, is_start in segs:
            assert full <= tile < tiles and 0 <= k0 < k1 <= ipt
            assert is_start == (k0 == 0)
            for k in range(k0, k1):
                assert (tile, k) not in covered
                covered[(tile, k)] = pid
            if not is_start:
                n_publish += 1
                publishers.setdefault(tile, []).append(pid)
        assert n_publish <= 1        # a workgroup owns one partial slot: only its first segment may be a non-start
        if n_publish:
            assert not segs[0][3]
    assert set(covered) == {(t, k) for t in range(full, tiles) for k in range(ipt)}
    # the owner of a tile (k = 0) is followed by its publishers in ascending, consecutive pid order
    for tile, pubs in publishers.items():
        owner = covered[(tile, 0)]
        assert pubs == list(range(owner + 1, owner + 1 + len(pubs)))


@pytest.mark.parametrize("tiles,grid,ipt", [(64, 256, 112), (300, 256, 7), (5, 8, 3), (3, 7, 1), (10, 4, 5), (256, 256, 9),
                                            (1, 256, 100), (2, 256, 5), (16, 200, 32)])
def test_streamk_last_owner_walk_waits_only_for_started_workgroups(tiles, grid, ipt):
    """The library's walk of the Stream-K range: every iteration once; a workgroup publishes at most one
    partial and does so before anything else; the owner of a tile holds its last iteration and waits
    exactly for the workgroups that hold the rest, all with lower ids (started earlier by the hardware),
    each of which publishes that tile."""
    sk_tiles = S.streamk_partition(tiles, grid)
    if sk_tiles == 0:
        sk_tiles = min(tiles, 1)       # (the host would take the whole-tile path; exercise the walk anyway)
    full = tiles - sk_tiles
    covered, publishes, owners = {}, {}, {}
    for wg in range(grid):
        walk = S.streamk_walk_last_owner(wg, grid, tiles, sk_tiles, ipt)
        kinds = [w[3] for w in walk]
        assert kinds.count("publish") <= 1 and (kinds.count("publish") == 0 or kinds[0] == "publish")
        for tile, k0, k1, kind, waits in walk:
            assert full <= tile < tiles and 0 <= k0 < k1 <= ipt
            for k in range(k0, k1):
                assert (tile, k) not in covered
                covered[(tile, k)] = wg
            if kind == "publish":
                assert k1 < ipt
                publishes[(tile, wg)] = (k0, k1)
            else:
                assert k1 == ipt
                owners[tile] = (wg, k0, waits)
    assert set(covered) == {(t, k) for t in range(full, tiles) for k in range(ipt)}
    for tile, (wg, k0, waits) in owners.items():
        assert all(w < wg for w in waits) and waits == list(range(wg - 1, wg - 1 - len(waits), -1))
        need = k0
        for w in waits:                      # nearest first: each partial ends where the previous began
            a, b = publishes[(tile, w)]
            assert b == need
            need = a
        assert need == 0
    assert len(owners) == sk_tiles


@pytest.mark.parametrize("tiles,xcds,cpx,grid", [(3584, 8, 1, 256), (1024, 8, 4, 256), (100, 8, 8, 256), (7, 8, 8, 256),
                                                 (513, 8, 4, 304), (64, 8, 8, 512)])
def test_work_stealing_queues_partition_the_tiles(tiles, xcds, cpx, grid):
    seen = {}
    for pid in range(grid):
        ctr, first, bound = S.ws_slot_range(pid, tiles, xcds, cpx)
        assert 0 <= ctr < xcds * cpx
        if ctr in seen:
            assert seen[ctr] == (first, bound)
        seen[ctr] = (first, bound)
    if grid >= xcds * cpx:
        covered = sorted(t for first, bound in seen.values() for t in range(first, first + bound))
        assert covered == list(range(tiles))


def test_grouped_tile_table():
    offsets = [0, 300, 300, 1000, 1024]  # expert 1 is empty
    bm, tn = 256, 3
    seen = set()
    t = 0
    while True:
        r = S.grouped_tile_lookup(t, offsets, bm, tn)
        if r is None:
            break
        seen.add(r)
        t += 1
    want = {(0, mb, nb) for mb in range(2) for nb in range(tn)} | {(2, mb, nb) for mb in range(3) for nb in range(tn)} | \
           {(3, 0, nb) for nb in range(tn)}
    assert seen == want and t == len(want)
    assert t <= (S.cdiv(1024, bm) + 4) * tn   # the launch grid bound


@pytest.mark.parametrize("small_rows", [1, 32, 64, 100, 255])
def test_grouped_two_launches_cover_every_row_once(small_rows):
    """Whatever the threshold, the two launches' row blocks partition every expert's rows, phase 2
    only ever holds blocks of at most small_rows rows in total per expert, and both tables stay
    inside the bounds the host sizes its grids with."""
    rng = np.random.default_rng(small_rows)
    for _ in range(50):
        counts = [int(c) for c in rng.choice([0, 1, 5, 31, 32, 33, 64, 65, 100, 255, 256, 257, 300, 511, 512, 1030], size=rng.integers(1, 9))]
        offsets = [0] + list(np.cumsum(counts))
        big, bm2 = 256, 32
        b1 = S.grouped_two_launch_blocks(offsets, 1, big, small_rows, big)
        b2 = S.grouped_two_launch_blocks(offsets, 2, big, small_rows, bm2)
        for e, c in enumerate(counts):
            rows = sorted(r for (ee, a, b) in b1 + b2 if ee == e for r in range(a, b))
            assert rows == list(range(offsets[e], offsets[e + 1]))
            left = sum(b - a for (ee, a, b) in b2 if ee == e)
            assert left == (c % big if 0 < c % big <= small_rows else 0)
        assert all(0 < b - a <= big for _, a, b in b1) and all(0 < b - a <= bm2 for _, a, b in b2)
        assert len(b1) <= S.cdiv(offsets[-1], big) + len(counts)
        assert len(b2) <= len(counts) * S.cdiv(small_rows, bm2)


def test_grouped_split_verdicts():
    """Hand-priced cases on 256 compute units, 8 experts of (14336, 4096) weights: 56 column tiles of
    256, 112 of 128; a round of tall tiles costs 4, a round of short tiles 3.  Routed counts with five
    remainders of at most 27 rows: 37 blocks = 9 rounds (36) against 32 blocks = 7 rounds + 560 short
    tiles = 3 rounds (28 + 9 = 37): one launch.  Remainders of 60 rows on four experts: 36 blocks = 8
    rounds (32) against 7 rounds + 896 short tiles = 4 rounds (40): one launch.  Equal counts: nothing
    short, one launch.  One big expert and two single rows: 34 blocks = 8 rounds (32) against 7 rounds +
    224 short tiles = 1 round (31): split."""
    def verdict(counts):
        return S.grouped_split_pays([0] + list(np.cumsum(counts)), 256, 64, 32, 56, 112, 256, 256)
    assert verdict([1051, 1035, 1034, 1029, 997, 1019, 991, 1036]) is False
    assert verdict([1084, 964] * 4) is False
    assert verdict([1024] * 8) is False
    assert verdict([8190, 1, 1, 0, 0, 0, 0, 0]) is True
