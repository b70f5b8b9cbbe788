"""CollectiveSpec / transport / WG plan: closed forms and every error branch
(reference tileccl_v2/collective_spec.py, transport.py, wg.py)."""

import pytest

from oracle import planning as ref
from tileccl_amd.v2 import (
    CollectiveKind,
    CommMode,
    all_gather_spec,
    build_p2p_transport_plan,
    build_tile_group_plan,
    build_wg_plan,
    normalize_comm_mode,
    reduce_scatter_spec,
)


def test_reduce_scatter_spec_owners():
    spec = reduce_scatter_spec(world_size=2)
    assert spec.kind is CollectiveKind.REDUCE_SCATTER and spec.requires_row_owner_split
    assert spec.shard_rows(8192) == 4096
    assert spec.row_split_boundaries(8192) == [4096] == ref.owner_boundaries(8192, 2)
    assert [spec.owner_for_row(r, 8192) for r in (0, 4095, 4096, 8191)] == [0, 0, 1, 1]
    spec4 = reduce_scatter_spec(world_size=4)
    assert spec4.row_split_boundaries(16384) == [4096, 8192, 12288]
    assert all(spec4.owner_for_row(r, 16384) == ref.row_owner(r, 16384, 4) for r in range(0, 16384, 777))


def test_all_gather_spec_has_no_owners():
    spec = all_gather_spec(world_size=2)
    assert not spec.requires_row_owner_split
    assert spec.row_split_boundaries(8192) == []
    spec.validate_tile_groups(8192, [(0, 8192, 1)])  # nothing to check
    with pytest.raises(ValueError, match="all_gather does not have row owners"):
        spec.owner_for_row(0, 8192)


def test_spec_errors():
    spec = reduce_scatter_spec(world_size=3)
    with pytest.raises(ValueError, match=r"M=8192 must be divisible by world_size=3"):
        spec.shard_rows(8192)
    spec = reduce_scatter_spec(world_size=2)
    with pytest.raises(ValueError, match=r"row=8192 outside \[0, 8192\)"):
        spec.owner_for_row(8192, 8192)
    with pytest.raises(ValueError, match=r"row=-1 outside"):
        spec.owner_for_row(-1, 8192)
    with pytest.raises(ValueError, match="world_size must be positive"):
        reduce_scatter_spec(world_size=0).shard_rows(8)
    with pytest.raises(ValueError, match="invalid TileGroup rows 5-5"):
        spec.validate_tile_groups(8192, [(5, 5, 0)])
    with pytest.raises(ValueError, match="TileGroup rows 0-8192 cross row owner boundary"):
        spec.validate_tile_groups(8192, [(0, 8192, 2048)])


def test_validate_accepts_split_plan():
    spec = reduce_scatter_spec(world_size=2)
    plan = build_tile_group_plan(8192, 4096, 32768, row_split_boundaries=spec.row_split_boundaries(8192))
    spec.validate_tile_groups(8192, plan.groups)
    plan = build_tile_group_plan(16384, 4096, 32768, row_split_boundaries=spec.row_split_boundaries(16384))
    assert plan.n_groups == 16
    spec.validate_tile_groups(16384, plan.groups)


def test_transport_plan():
    t = build_p2p_transport_plan(comm_mode="push", copy_elems=16384)
    assert t.push_mode and t.comm_mode is CommMode.PUSH
    assert t.copy_qwords == 4096 and t.packed_values_per_word == 4 and t.reduce_elems is None
    t = build_p2p_transport_plan(comm_mode=CommMode.PULL, copy_elems=8192, reduce_elems=4096)
    assert not t.push_mode and t.copy_qwords == 2048
    assert normalize_comm_mode("pull") is CommMode.PULL and normalize_comm_mode(CommMode.PUSH) is CommMode.PUSH
    with pytest.raises(ValueError, match=r"unknown comm_mode='shove'; expected one of push, pull"):
        normalize_comm_mode("shove")
    for kw, msg in [
        (dict(comm_mode="push", copy_elems=0), "copy_elems must be positive"),
        (dict(comm_mode="push", copy_elems=4, reduce_elems=0), "reduce_elems must be positive"),
        (dict(comm_mode="push", copy_elems=4, packed_values_per_word=0), "packed_values_per_word must be positive"),
    ]:
        with pytest.raises(ValueError, match=msg):
            build_p2p_transport_plan(**kw)


def test_wg_plan_numbers():
    plan = build_tile_group_plan(8192, 4096, 32768)
    t = build_p2p_transport_plan(comm_mode="push", copy_elems=16384)
    wg = t.build_wg_plan(total_sms=256, num_comm_wgs=51, max_group_elems=plan.max_group_elems)
    want = ref.wg_numbers(256, 51, 1024 * 4096, 16384)
    assert wg.num_comp_wgs == 205 == want["num_comp_wgs"]
    assert wg.total_wgs == 256 and wg.grid == (256,) == want["grid"]
    assert wg.copy_qwords == 4096 == want["copy_qwords"]
    assert wg.copy_tasks_per_group == 256 == want["copy_tasks_per_group"]
    assert wg.reduce_tasks_per_group == 0 and wg.tasks_per_group == 256
    wg = build_wg_plan(total_sms=256, num_comm_wgs=32, max_group_elems=1000 * 4, copy_elems=16, reduce_elems=12)
    want = ref.wg_numbers(256, 32, 4000, 16, 12)
    assert (wg.copy_tasks_per_group, wg.reduce_tasks_per_group, wg.tasks_per_group) == (250, 334, 334)
    assert wg.tasks_per_group == want["tasks_per_group"]


@pytest.mark.parametrize(
    "kw,msg",
    [
        (dict(total_sms=0), "total_sms must be positive"),
        (dict(num_comm_wgs=-1), "num_comm_wgs must be non-negative"),
        (dict(num_comm_wgs=256), "num_comm_wgs=256 leaves no compute WGs"),
        (dict(max_group_elems=0), "max_group_elems must be positive"),
        (dict(copy_elems=0), "copy_elems must be positive"),
        (dict(packed_values_per_word=0), "packed_values_per_word must be positive"),
        (dict(copy_elems=6), "copy_elems must be divisible by packed_values_per_word"),
        (dict(max_group_elems=1022), "max_group_elems must be divisible by packed_values_per_word"),
        (dict(reduce_elems=-4), "reduce_elems must be positive"),
    ],
)
def test_wg_plan_errors(kw, msg):
    base = dict(total_sms=256, num_comm_wgs=16, max_group_elems=4096, copy_elems=16)
    base.update(kw)
    with pytest.raises(ValueError, match=msg):
        build_wg_plan(**base)
