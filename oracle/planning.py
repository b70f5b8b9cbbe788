"""Loop-form restatement of the reference TileGroup planner (test infrastructure only).

Written the slow, literal way -- one tile or one row at a time -- so that it shares no
structure with the vectorised product code in ``tileccl_amd/v2/tile_group.py``.

Follows
    build_tile_groups               /root/reference/tileccl_v2/tile_group.py:87-153
    split_groups_at_row_boundaries  /root/reference/tileccl_v2/tile_group.py:156-184
    build_group_table               /root/reference/tileccl_v2/tile_group.py:214-241
    swizzle                         /root/reference/tileccl/kernels/gemm.py:118-123
    TileGroupPlan properties        /root/reference/tileccl_v2/tile_group.py:44-84
    CollectiveSpec                  /root/reference/tileccl_v2/collective_spec.py:37-72
    WGPlan properties               /root/reference/tileccl_v2/wg.py:21-51
"""

from __future__ import annotations

import math


def tile_groups(M, N, tile_bytes, target_group_tiles=None, max_groups=64, block_m=128, block_n=128,
                group_m=8, tau_min_bytes=262144):
    """List of (row_start, row_end, tiles); see tile_group.py:114-153."""
    tile_rows = math.ceil(M / block_m)
    tile_cols = math.ceil(N / block_n)
    p0 = max(1, math.ceil(tau_min_bytes / tile_bytes))  # :116
    need = max(p0, target_group_tiles or p0)  # :117

    # wave borders in tile rows: 0, group_m, 2*group_m, ..., tile_rows  (:119-121)
    borders = [0]
    while borders[-1] < tile_rows:
        borders.append(min(borders[-1] + group_m, tile_rows))

    out = []
    open_from = 0
    have = 0
    for lo, hi in zip(borders, borders[1:]):
        have += (hi - lo) * tile_cols
        if have >= need:  # :128
            out.append((open_from * block_m, hi * block_m, have))
            open_from = hi
            have = 0
    if have > 0:  # :136-141
        if out:
            start, _, tiles = out[-1]
            out[-1] = (start, M, tiles + have)
        else:
            out.append((0, M, have))
    if len(out) > max_groups:  # :143-151
        k = math.ceil(len(out) / max_groups)
        merged = []
        i = 0
        while i < len(out):
            part = out[i:i + k]
            merged.append((part[0][0], min(part[-1][1], M), sum(p[2] for p in part)))
            i += k
        out = merged
    return out


def split_at_boundaries(M, N, groups, boundaries, block_m=128, block_n=128):
    """tile_group.py:166-184: walk each group row range and cut at every interior boundary."""
    tile_cols = math.ceil(N / block_n)
    cuts = sorted(set([0, M] + [b for b in boundaries if 0 < b < M]))
    out = []
    for start, raw_end, _ in groups:
        end = min(raw_end, M)
        pos = start
        while pos < end:
            nxt = min(b for b in cuts if b > pos)
            stop = min(end, nxt)
            out.append((pos, stop, math.ceil((stop - pos) / block_m) * tile_cols))
            pos = stop
    return out


def swizzle(tile_id, tile_rows, tile_cols, group_m):
    """(tile_m, tile_n) of a tile id; kernels/gemm.py:118-123."""
    per_band = group_m * tile_cols
    band = tile_id // per_band
    first = band * group_m
    height = min(tile_rows - first, group_m)
    return first + (tile_id % per_band) % height, (tile_id % per_band) // height


def group_table(M, N, groups, block_m=128, block_n=128, group_m=8):
    """tile id -> group id list; tile_group.py:223-241 (first containing group, default 0)."""
    tile_rows = math.ceil(M / block_m)
    tile_cols = math.ceil(N / block_n)
    table = []
    for t in range(tile_rows * tile_cols):
        tm, _ = swizzle(t, tile_rows, tile_cols, group_m)
        row = tm * block_m
        gid = 0
        for i, (lo, hi, _) in enumerate(groups):
            if lo <= row < hi:
                gid = i
                break
        table.append(gid)
    return table


def plan_summary(M, N, groups, block_m=128, block_n=128):
    """max_rb, max_cb, max_group_elems, row_ends (clamped); tile_group.py:47-84."""
    return {
        "max_rb": max(math.ceil((hi - lo) / block_m) for lo, hi, _ in groups),
        "max_cb": math.ceil(N / block_n),
        "max_group_elems": max((hi - lo) * N for lo, hi, _ in groups),
        "row_starts": [g[0] for g in groups],
        "row_ends": [min(g[1], M) for g in groups],
        "tile_counts": [g[2] for g in groups],
    }


def row_owner(row, M, world_size):
    """collective_spec.py:51-58."""
    return row // (M // world_size)


def owner_boundaries(M, world_size):
    """collective_spec.py:44-49 (reduce-scatter only)."""
    return [(M // world_size) * r for r in range(1, world_size)]


def wg_numbers(total_sms, num_comm_wgs, max_group_elems, copy_elems, reduce_elems=None, packed=4):
    """wg.py:21-51."""
    copy_tasks = math.ceil(max_group_elems / copy_elems)
    reduce_tasks = 0 if reduce_elems is None else math.ceil(max_group_elems / reduce_elems)
    return {
        "num_comp_wgs": total_sms - num_comm_wgs,
        "grid": (total_sms,),
        "copy_qwords": copy_elems // packed,
        "copy_tasks_per_group": copy_tasks,
        "reduce_tasks_per_group": reduce_tasks,
        "tasks_per_group": copy_tasks if reduce_elems is None else max(copy_tasks, reduce_tasks),
    }
