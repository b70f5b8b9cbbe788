"""TileGroup planner: known answers derived by hand from the reference's rules, the
loop-form oracle, and brute-force invariants (reference tileccl_v2/tile_group.py)."""

import itertools
import math

import pytest
import torch

from oracle import planning as ref
from tileccl_amd.v2 import (
    build_group_table,
    build_tile_group_plan,
    build_tile_groups,
    split_groups_at_row_boundaries,
    split_groups_at_row_shards,
)

FP16_TILE = 128 * 128 * 2


# ---- closed-form known answers ---------------------------------------------------------------
def test_plumbing_config_is_one_group():
    # 512x512: 16 tiles, p0 = ceil(262144/32768) = 8; the only wave (4 tile rows) holds 16 >= 8.
    plan = build_tile_group_plan(512, 512, FP16_TILE)
    assert plan.groups == [(0, 512, 16)]
    assert plan.group_table.tolist() == [0] * 16
    assert plan.group_table.dtype == torch.int32 and plan.group_table.device.type == "cpu"
    assert plan.p0_min_tiles == 8
    assert (plan.max_rb, plan.max_cb, plan.max_group_elems) == (4, 4, 262144)
    assert plan.n_groups == 1


@pytest.mark.parametrize("M,n", [(8192, 8), (4096, 4), (16384, 16)])
def test_headline_shapes_one_group_per_swizzle_wave(M, n):
    # N = 4096 -> 32 tile columns; one wave = 8 tile rows = 256 tiles >= p0 = 8.
    plan = build_tile_group_plan(M, 4096, FP16_TILE)
    assert plan.n_groups == n
    assert plan.groups == [(1024 * k, 1024 * (k + 1), 256) for k in range(n)]
    table = plan.group_table.tolist()
    assert table == [t // 256 for t in range(n * 256)]
    assert (plan.max_rb, plan.max_cb, plan.max_group_elems) == (8, 32, 1024 * 4096)
    assert plan.min_group_tiles == plan.max_group_tiles == 256 and plan.avg_group_tiles == 256.0
    assert plan.row_starts() == [1024 * k for k in range(n)]
    assert plan.row_ends() == [1024 * (k + 1) for k in range(n)]
    assert plan.tile_counts() == [256] * n


def test_block_m_256():
    # 256x128 fp16 tiles: p0 = ceil(262144/65536) = 4; wave = 8 tile rows = 2048 rows, 256 tiles.
    plan = build_tile_group_plan(8192, 4096, 256 * 128 * 2, block_m=256)
    assert plan.p0_min_tiles == 4
    assert plan.groups == [(2048 * k, 2048 * (k + 1), 256) for k in range(4)]


def test_tail_wave_is_folded_into_last_group():
    # M=2560 -> 20 tile rows, N=128 -> 1 col.  Waves of 8,8,4 tiles; g_min=8: groups close at
    # 8 and 16, the 4 left over join the last one whose row_end becomes M.
    assert build_tile_groups(2560, 128, FP16_TILE) == [(0, 1024, 8), (1024, 2560, 12)]


def test_row_end_may_exceed_M():
    # M=1000 -> 8 tile rows; the single wave closes at 8*128 = 1024 > M.
    plan = build_tile_group_plan(1000, 512, FP16_TILE)
    assert plan.groups == [(0, 1024, 32)]
    assert plan.row_ends() == [1000]
    assert plan.max_group_elems == 1024 * 512  # unclamped on purpose


def test_max_groups_merge():
    # 133120 rows = 1040 tile rows = 130 waves of 256 tiles -> merge factor ceil(130/64) = 3 -> 44 groups.
    groups = build_tile_groups(133120, 4096, FP16_TILE)
    assert len(groups) == 44
    assert groups[0] == (0, 3072, 768)
    assert groups[-1] == (132096, 133120, 256)
    assert sum(g[2] for g in groups) == 1040 * 32


def test_target_group_tiles_widens_groups():
    groups = build_tile_groups(8192, 4096, FP16_TILE, target_group_tiles=512)
    assert groups == [(2048 * k, 2048 * (k + 1), 512) for k in range(4)]
    # a target below the saturation floor changes nothing
    assert build_tile_groups(8192, 4096, FP16_TILE, target_group_tiles=1) == build_tile_groups(8192, 4096, FP16_TILE)


def test_nothing_ever_closes():
    # 2 tiles < p0 = 8: the whole output is one group.
    assert build_tile_groups(128, 256, FP16_TILE) == [(0, 128, 2)]


def test_swizzle_with_short_last_band():
    # 12 tile rows, 2 cols, group_m=8: ids 0-15 walk rows 0-7 (col 0 then 1); ids 16-23 walk rows 8-11.
    groups = [(r * 128, (r + 1) * 128, 2) for r in range(12)]  # one group per tile row -> table == tile_m
    table = build_group_table(12 * 128, 256, groups).tolist()
    assert table[:16] == [t % 8 for t in range(16)]
    assert table[16:] == [8 + (t - 16) % 4 for t in range(16, 24)]


def test_unmatched_tiles_default_to_group_zero():
    table = build_group_table(512, 128, [(128, 256, 1)]).tolist()
    assert table == [0, 0, 0, 0]
    table = build_group_table(512, 128, [(0, 128, 1), (256, 384, 1)]).tolist()
    assert table == [0, 0, 1, 0]


def test_first_matching_group_wins_on_overlap():
    table = build_group_table(256, 128, [(0, 256, 2), (128, 256, 1)]).tolist()
    assert table == [0, 0]


# ---- splits --------------------------------------------------------------------------------------
def test_split_aligned_boundary_changes_nothing():
    groups = build_tile_groups(8192, 4096, FP16_TILE)
    assert split_groups_at_row_boundaries(8192, 4096, groups, [4096]) == groups


def test_split_inside_a_group_recounts_tiles():
    out = split_groups_at_row_boundaries(2048, 256, [(0, 2048, 32)], [768])
    assert out == [(0, 768, 12), (768, 2048, 20)]
    # ragged piece: 100 rows still cost one tile row
    assert split_groups_at_row_boundaries(1024, 128, [(0, 1024, 8)], [100]) == [(0, 100, 1), (100, 1024, 8)]


def test_split_clamps_and_drops_empty():
    assert split_groups_at_row_boundaries(1000, 128, [(0, 1024, 8), (1000, 1100, 1)], []) == [(0, 1000, 8)]
    # boundaries outside (0, M) are ignored
    assert split_groups_at_row_boundaries(512, 128, [(0, 512, 4)], [0, 512, 9999, -5]) == [(0, 512, 4)]


def test_split_at_row_shards():
    groups = [(0, 4096, 64)]
    assert split_groups_at_row_shards(4096, 256, groups, num_shards=4) == [
        (1024 * k, 1024 * (k + 1), 16) for k in range(4)
    ]
    with pytest.raises(ValueError, match="num_shards must be positive"):
        split_groups_at_row_shards(4096, 256, groups, num_shards=0)
    with pytest.raises(ValueError, match=r"M=1000 must be divisible by num_shards=3"):
        split_groups_at_row_shards(1000, 256, groups, num_shards=3)


def test_plan_with_owner_split():
    plan = build_tile_group_plan(8192, 4096, FP16_TILE, row_split_boundaries=[4096])
    assert plan.n_groups == 8  # waves already end on the owner border
    plan = build_tile_group_plan(2048, 256, FP16_TILE, row_split_boundaries=[512])
    # groups before the split: waves of 16 tiles -> [(0,1024,16),(1024,2048,16)]; cut at 512
    assert plan.groups == [(0, 512, 8), (512, 1024, 8), (1024, 2048, 16)]
    assert plan.group_table.tolist() == ref.group_table(2048, 256, plan.groups)
    # None means "no boundaries" (reference tile_group.py:269), the same as an empty sequence
    assert build_tile_group_plan(2048, 256, FP16_TILE, row_split_boundaries=None).groups == \
        build_tile_group_plan(2048, 256, FP16_TILE).groups == [(0, 1024, 16), (1024, 2048, 16)]


# ---- validation ------------------------------------------------------------------------------------
@pytest.mark.parametrize(
    "kwargs,msg",
    [
        (dict(M=0, N=1, tile_bytes=1), "M and N must be positive"),
        (dict(M=1, N=-1, tile_bytes=1), "M and N must be positive"),
        (dict(M=1, N=1, tile_bytes=0), "tile_bytes must be positive"),
        (dict(M=1, N=1, tile_bytes=1, block_m=0), "block_m, block_n, and group_m must be positive"),
        (dict(M=1, N=1, tile_bytes=1, group_m=0), "block_m, block_n, and group_m must be positive"),
        (dict(M=1, N=1, tile_bytes=1, max_groups=0), "max_groups must be positive"),
    ],
)
def test_validation(kwargs, msg):
    M, N, tb = kwargs.pop("M"), kwargs.pop("N"), kwargs.pop("tile_bytes")
    with pytest.raises(ValueError, match=msg):
        build_tile_groups(M, N, tb, **kwargs)


# ---- product == loop-form oracle, and invariants, over a sweep -----------------------------------------
SWEEP = list(
    itertools.product(
        [1, 100, 128, 129, 1000, 1024, 2560, 4096, 5000],  # M
        [8, 128, 200, 512, 4096],  # N
        [(128, 128), (256, 128), (64, 64)],  # block
        [1, 3, 8],  # group_m
        [None, 5, 40],  # target
    )
)


@pytest.mark.parametrize("M,N,block,group_m,target", SWEEP[:: max(1, len(SWEEP) // 160)])
def test_against_loop_oracle_and_invariants(M, N, block, group_m, target):
    bm, bn = block
    tile_bytes = bm * bn * 2
    kw = dict(target_group_tiles=target, block_m=bm, block_n=bn, group_m=group_m, max_groups=7)
    groups = build_tile_groups(M, N, tile_bytes, **kw)
    assert groups == ref.tile_groups(M, N, tile_bytes, **kw)

    tile_rows, tile_cols = math.ceil(M / bm), math.ceil(N / bn)
    # groups tile [0, M) contiguously and account for every tile exactly once
    assert groups[0][0] == 0
    for (_, hi, _), (lo, _, _) in zip(groups, groups[1:]):
        assert hi == lo
    assert min(groups[-1][1], M) == M
    assert sum(g[2] for g in groups) == tile_rows * tile_cols
    assert len(groups) <= 7

    table = build_group_table(M, N, groups, block_m=bm, block_n=bn, group_m=group_m).tolist()
    assert table == ref.group_table(M, N, groups, bm, bn, group_m)
    # every tile sits in the group that contains its first row; counts per group match
    for t, gid in enumerate(table):
        tm, _ = ref.swizzle(t, tile_rows, tile_cols, group_m)
        lo, hi, _ = groups[gid]
        assert lo <= tm * bm < hi
    for gid, (lo, hi, tiles) in enumerate(groups):
        assert table.count(gid) == tiles

    cut = (M // 2 // 8) * 8
    if cut:
        pieces = split_groups_at_row_boundaries(M, N, groups, [cut], block_m=bm, block_n=bn)
        assert pieces == ref.split_at_boundaries(M, N, groups, [cut], bm, bn)
        assert all(not (lo < cut < hi) for lo, hi, _ in pieces)


def test_table_is_monotone_for_wave_aligned_groups():
    plan = build_tile_group_plan(16384, 4096, FP16_TILE)
    t = plan.group_table.tolist()
    assert t == sorted(t)
