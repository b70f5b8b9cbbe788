"""TileGroup planner: which output tiles travel together, and in which order they appear.

Host-side contract consumed by the fused GEMM+collective kernels.  Mirrors the
reference planner's public surface (``/root/reference/tileccl_v2/tile_group.py``):

* ``build_tile_groups``             -> reference ``tile_group.py:87-153``
* ``split_groups_at_row_boundaries``-> reference ``tile_group.py:156-184``
* ``split_groups_at_row_shards``    -> reference ``tile_group.py:187-211``
* ``build_group_table``             -> reference ``tile_group.py:214-241``
* ``build_tile_group_plan`` / ``TileGroupPlan`` -> reference ``tile_group.py:27-84, 244-301``

A TileGroup is ``(row_start, row_end, tile_count)``: a band of output rows whose tiles
are signalled as one unit.  Two rules shape the bands:

P0 (saturation)  a group must carry at least ``ceil(tau_min_bytes / tile_bytes)`` tiles
                 so one transfer is large enough to saturate the link;
P1 (alignment)   group borders sit on the borders of the GEMM's swizzle waves
                 (``group_m`` tile rows), so a group completes when a contiguous run
                 of tile ids has completed.

The group table maps a *tile id in the persistent GEMM's swizzled order* to its group id;
the swizzle is the one used by the GEMM kernel (``tile_m`` runs fastest inside a band of
``group_m`` tile rows; reference ``tileccl/kernels/gemm.py:118-123``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Sequence

import numpy as np
import torch

DEFAULT_BLOCK_M = 128
DEFAULT_BLOCK_N = 128
DEFAULT_GROUP_M = 8
DEFAULT_TAU_MIN_BYTES = 262144

TileGroup = tuple[int, int, int]


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


@dataclass(frozen=True)
class TileGroupPlan:
    """Everything a fused kernel needs to know about the TileGroups of one output."""

    M: int
    N: int
    tile_bytes: int
    target_group_tiles: int | None
    max_groups: int
    groups: list[TileGroup]
    group_table: torch.Tensor
    block_m: int = DEFAULT_BLOCK_M
    block_n: int = DEFAULT_BLOCK_N
    group_m: int = DEFAULT_GROUP_M
    tau_min_bytes: int = DEFAULT_TAU_MIN_BYTES
    p0_min_tiles: int = 1

    # -- scalar summaries ----------------------------------------------------
    n_groups = property(lambda self: len(self.groups))
    # largest number of tile rows any group spans (row_end not clamped to M), and tile columns of the output
    max_rb = property(lambda self: max(_cdiv(end - first, self.block_m) for first, end, _ in self.groups))
    max_cb = property(lambda self: _cdiv(self.N, self.block_n))
    # largest group payload in elements; row_end is not clamped to M
    max_group_elems = property(lambda self: max((end - first) * self.N for first, end, _ in self.groups))
    min_group_tiles = property(lambda self: min(self.tile_counts()))
    max_group_tiles = property(lambda self: max(self.tile_counts()))
    avg_group_tiles = property(lambda self: sum(self.tile_counts()) / len(self.groups))

    # -- per-group vectors (what the kernels take) ----------------------------
    def row_starts(self) -> "list[int]":
        return [first for first, _, _ in self.groups]

    def row_ends(self) -> "list[int]":
        return [min(end, self.M) for _, end, _ in self.groups]

    def tile_counts(self) -> "list[int]":
        return [tiles for _, _, tiles in self.groups]


def _check_geometry(M, N, tile_bytes, block_m, block_n, group_m, max_groups) -> None:
    if M <= 0 or N <= 0:
        raise ValueError("M and N must be positive")
    if tile_bytes <= 0:
        raise ValueError("tile_bytes must be positive")
    if block_m <= 0 or block_n <= 0 or group_m <= 0:
        raise ValueError("block_m, block_n, and group_m must be positive")
    if max_groups <= 0:
        raise ValueError("max_groups must be positive")


def build_tile_groups(M: int, N: int, tile_bytes: int, *, target_group_tiles: "int | None" = None, max_groups: int = 64,
                      block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N, group_m: int = DEFAULT_GROUP_M,
                      tau_min_bytes: int = DEFAULT_TAU_MIN_BYTES) -> "list[TileGroup]":
    """Cut ``[0, M)`` into wave-aligned row bands of at least ``g_min`` tiles each.

    Walks the swizzle waves in order, closing a band as soon as it holds enough tiles.
    Tiles left over after the last closed band are folded into it (its ``row_end``
    becomes ``M``); if nothing was ever closed the whole output is one band.  More than
    ``max_groups`` bands are merged ``ceil(n / max_groups)`` neighbours at a time.
    """
    _check_geometry(M, N, tile_bytes, block_m, block_n, group_m, max_groups)

    tile_rows = _cdiv(M, block_m)
    tile_cols = _cdiv(N, block_n)
    saturation_tiles = max(1, _cdiv(tau_min_bytes, tile_bytes))
    g_min = max(saturation_tiles, target_group_tiles or saturation_tiles)

    bands: list[TileGroup] = []
    band_first_row = 0  # in tile rows
    pending = 0
    for wave_first in range(0, tile_rows, group_m):
        wave_last = min(wave_first + group_m, tile_rows)
        pending += (wave_last - wave_first) * tile_cols
        if pending >= g_min:
            bands.append((band_first_row * block_m, wave_last * block_m, pending))
            band_first_row, pending = wave_last, 0

    if pending:
        if bands:
            lo, _, n = bands.pop()
            bands.append((lo, M, n + pending))
        else:
            bands.append((0, M, pending))

    if len(bands) > max_groups:
        stride = _cdiv(len(bands), max_groups)
        runs = [bands[i:i + stride] for i in range(0, len(bands), stride)]
        bands = [(run[0][0], min(run[-1][1], M), sum(tiles for _, _, tiles in run)) for run in runs]
    return bands


def split_groups_at_row_boundaries(M: int, N: int, groups: "Sequence[TileGroup]", row_boundaries: "Sequence[int]", *,
                                   block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N) -> "list[TileGroup]":
    """Cut every band at each interior boundary so no band straddles two row owners.

    Tile counts of the pieces are recomputed from their row extent
    (``ceil(rows / block_m) * tile_cols``); bands are first clamped to ``M`` and empty
    ones dropped.
    """
    tile_cols = _cdiv(N, block_n)
    cuts = sorted({b for b in row_boundaries if 0 < b < M})
    pieces: list[TileGroup] = []
    for lo, hi, _ in groups:
        hi = min(hi, M)
        if lo >= hi:
            continue
        edges = [lo, *(c for c in cuts if lo < c < hi), hi]
        for a, b in zip(edges[:-1], edges[1:]):
            pieces.append((a, b, _cdiv(b - a, block_m) * tile_cols))
    return pieces


def split_groups_at_row_shards(M: int, N: int, groups: "Sequence[TileGroup]", *, num_shards: int,
                               block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N) -> "list[TileGroup]":
    """Cut bands at the borders of ``num_shards`` equal row shards."""
    if num_shards <= 0:
        raise ValueError("num_shards must be positive")
    if M % num_shards:
        raise ValueError(f"M={M} must be divisible by num_shards={num_shards}")
    borders = range(M // num_shards, M, M // num_shards)
    return split_groups_at_row_boundaries(M, N, groups, borders, block_m=block_m, block_n=block_n)


def swizzled_tile_rows(tile_rows: int, tile_cols: int, group_m: int) -> np.ndarray:
    """``tile_m`` of every tile id in the persistent GEMM's swizzled launch order.

    Inside a band of ``group_m`` tile rows (fewer in the last band) consecutive ids walk
    down the rows first, then step to the next tile column
    (reference ``tileccl/kernels/gemm.py:118-123``).
    """
    ids = np.arange(tile_rows * tile_cols, dtype=np.int64)
    per_band = group_m * tile_cols
    first = (ids // per_band) * group_m
    height = np.minimum(tile_rows - first, group_m)
    return first + (ids % per_band) % height


def swizzled_tile_cols(tile_rows: int, tile_cols: int, group_m: int) -> np.ndarray:
    """``tile_n`` of every tile id in the swizzled order (companion of ``swizzled_tile_rows``)."""
    ids = np.arange(tile_rows * tile_cols, dtype=np.int64)
    per_band = group_m * tile_cols
    first = (ids // per_band) * group_m
    height = np.minimum(tile_rows - first, group_m)
    return (ids % per_band) // height


def build_group_table(M: int, N: int, groups: "Sequence[TileGroup]", *, block_m: int = DEFAULT_BLOCK_M,
                      block_n: int = DEFAULT_BLOCK_N, group_m: int = DEFAULT_GROUP_M) -> torch.Tensor:
    """``int32[total_tiles]`` on the CPU: swizzled tile id -> group id.

    A tile belongs to the first group whose ``[row_start, row_end)`` contains the tile's
    first row; tiles matched by no group keep id 0.
    """
    tile_rows = _cdiv(M, block_m)
    tile_cols = _cdiv(N, block_n)
    first_row = swizzled_tile_rows(tile_rows, tile_cols, group_m) * block_m
    table = np.zeros(tile_rows * tile_cols, dtype=np.int32)
    # Paint from the last group to the first so the earliest match wins.
    for gid in range(len(groups) - 1, -1, -1):
        lo, hi, _ = groups[gid]
        table[(first_row >= lo) & (first_row < hi)] = gid
    return torch.from_numpy(table)


def build_tile_group_plan(M: int, N: int, tile_bytes: int, *, target_group_tiles: "int | None" = None, max_groups: int = 64,
                          block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N, group_m: int = DEFAULT_GROUP_M,
                          tau_min_bytes: int = DEFAULT_TAU_MIN_BYTES,
                          row_split_boundaries: "Iterable[int] | None" = ()) -> TileGroupPlan:
    """Groups (optionally cut at owner boundaries) plus their swizzle table, as one plan."""
    tiling = dict(block_m=block_m, block_n=block_n)
    sizing = dict(target_group_tiles=target_group_tiles, max_groups=max_groups, tau_min_bytes=tau_min_bytes)
    groups = build_tile_groups(M, N, tile_bytes, group_m=group_m, **tiling, **sizing)
    cuts = list(row_split_boundaries or ())  # None: no boundaries, as the reference accepts (tile_group.py:269)
    if cuts:
        groups = split_groups_at_row_boundaries(M, N, groups, cuts, **tiling)
    table = build_group_table(M, N, groups, group_m=group_m, **tiling)
    return TileGroupPlan(M=M, N=N, tile_bytes=tile_bytes, groups=groups, group_table=table, group_m=group_m,
                         p0_min_tiles=max(1, _cdiv(tau_min_bytes, tile_bytes)), **tiling, **sizing)
