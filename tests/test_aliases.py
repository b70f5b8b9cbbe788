"""The reference's import lines resolve to this package after ``tileccl_amd.install_aliases()``.

The statements below are the ones the reference's callers open with: README.md:128,141-151 (the
minimal usage and the TileGroup planning example), tests/test_gemm_allscatter_smoke.py:9,20 and
examples/benchmark_patterns.py:19-26.
"""

from __future__ import annotations

import subprocess
import sys
import textwrap
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture()
def aliased():
    import tileccl_amd
    from tileccl_amd import aliases

    tileccl_amd.install_aliases()
    yield
    aliases.remove_aliases()


def test_not_aliased_until_asked():
    from tileccl_amd import aliases

    aliases.remove_aliases()
    with pytest.raises(ModuleNotFoundError):
        import tileccl  # noqa: F401
    with pytest.raises(ModuleNotFoundError):
        import tileccl_v2  # noqa: F401


def test_readme_planning_example(aliased):
    from tileccl_v2 import build_p2p_transport_plan, build_tile_group_plan, reduce_scatter_spec

    spec = reduce_scatter_spec(world_size=2)
    plan = build_tile_group_plan(8192, 4096, 128 * 128 * 2)
    transport = build_p2p_transport_plan(comm_mode="push", copy_elems=16384)
    assert str(spec.kind.value) == "reduce_scatter" and spec.requires_row_owner_split
    assert plan.n_groups == 8
    assert transport.push_mode is True
    assert transport.copy_qwords == 4096


def test_aliases_are_the_same_modules(aliased):
    import tileccl
    import tileccl.ops
    import tileccl.patterns
    import tileccl.patterns.contracts
    import tileccl_v2
    import tileccl_v2.cost_model
    import tileccl_v2.runtime.timeline
    import tileccl_v2.tile_group

    import tileccl_amd
    import tileccl_amd.ops
    import tileccl_amd.patterns.contracts
    import tileccl_amd.v2.cost_model
    import tileccl_amd.v2.runtime.timeline
    import tileccl_amd.v2.tile_group

    assert tileccl is tileccl_amd and tileccl_v2 is tileccl_amd.v2
    assert tileccl.ops is tileccl_amd.ops
    assert tileccl.patterns.contracts is tileccl_amd.patterns.contracts
    assert tileccl_v2.tile_group is tileccl_amd.v2.tile_group
    assert tileccl_v2.cost_model.TileCostModel is tileccl_amd.v2.cost_model.TileCostModel
    assert tileccl_v2.runtime.timeline.TimelineRecorder is tileccl_amd.v2.runtime.timeline.TimelineRecorder
    assert callable(tileccl.init) and callable(tileccl.init_local) and callable(tileccl.ops.gemm_allscatter)


def test_the_callers_from_imports(aliased):
    from tileccl.memory.symmetric_heap import SymmetricHeap
    from tileccl.ops import build_gemm_allscatter_plan
    from tileccl.patterns import BulkSyncPattern, FusedSequentialPattern, ProducerConsumerPattern, WGSpecializedPattern
    from tileccl_v2 import (CollectiveSpec, CommMode, P2PTransportPlan, SymmetricHeap as HeapV2, TileCostModel, TileGroupPlan,
                            TileGroupSignalState, TimelineRecorder, WGPlan, all_gather_spec, allocate_tile_group_signals,
                            build_group_table, build_tile_groups, build_wg_plan, normalize_comm_mode,
                            split_groups_at_row_boundaries, split_groups_at_row_shards)

    import tileccl_amd.memory.symmetric_heap as real

    assert SymmetricHeap is real.SymmetricHeap
    for name in (build_gemm_allscatter_plan, BulkSyncPattern, FusedSequentialPattern, ProducerConsumerPattern, WGSpecializedPattern,
                 CollectiveSpec, CommMode, P2PTransportPlan, HeapV2, TileCostModel, TileGroupPlan, TileGroupSignalState,
                 TimelineRecorder, WGPlan, all_gather_spec, allocate_tile_group_signals, build_group_table, build_tile_groups,
                 build_wg_plan, normalize_comm_mode, split_groups_at_row_boundaries, split_groups_at_row_shards):
        assert name is not None


def test_names_outside_the_reference_stay_unresolved(aliased):
    with pytest.raises(ModuleNotFoundError):
        import tileccl.csrc  # noqa: F401
    with pytest.raises(ModuleNotFoundError):
        import tileccl.v2  # noqa: F401
    with pytest.raises(ModuleNotFoundError):
        import tileccl.no_such_module  # noqa: F401


def test_refuses_to_shadow_an_installed_package(tmp_path):
    """In a fresh interpreter with a real `tileccl` on the path, the call raises unless forced."""
    pkg = tmp_path / "tileccl"
    pkg.mkdir()
    (pkg / "__init__.py").write_text("MARK = 'someone else'\n")
    script = textwrap.dedent(f"""
        import sys
        sys.path[:0] = [{str(tmp_path)!r}, {str(ROOT)!r}]
        import tileccl_amd
        try:
            tileccl_amd.install_aliases()
        except ImportError as exc:
            print("refused:", "installed" in str(exc))
        tileccl_amd.install_aliases(force=True)
        import tileccl
        print("forced:", tileccl is tileccl_amd)
    """)
    out = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, check=True).stdout
    assert "refused: True" in out and "forced: True" in out


@pytest.mark.gpu
def test_readme_minimal_usage_under_the_reference_names(aliased):
    """README.md:125-137 and tests/test_gemm_allscatter_smoke.py:19-40 as a caller of the reference writes them."""
    import torch

    import tileccl
    from tileccl.memory.symmetric_heap import SymmetricHeap

    ctx = tileccl.init(heap_size=64 * 1024 * 1024)
    try:
        A = ctx.randn(256, 128, dtype=torch.float16)
        B = ctx.randn(128, 256, dtype=torch.float16)
        C = ctx.zeros(256, 256, dtype=torch.float16)
        tileccl.ops.gemm_allscatter(A, B, C, ctx=ctx)
        torch.cuda.synchronize()
        assert torch.allclose(C, torch.matmul(A.float(), B.float()).half(), rtol=1e-2, atol=1e-1)
    finally:
        ctx.heap.cleanup()

    heaps = SymmetricHeap.create_all(size=64 * 1024 * 1024, world_size=1)
    try:
        ctx = tileccl.init(backend="hip", rank=0, world_size=1, heap=heaps[0], force_backend=True)
        a = torch.randn(128, 64, device=ctx.device, dtype=torch.float16)
        b = torch.randn(64, 128, device=ctx.device, dtype=torch.float16)
        c = torch.zeros(128, 128, device=ctx.device, dtype=torch.float16)
        tileccl.ops.gemm_allscatter(a, b, c, ctx=ctx, pattern="bulk_sync")
        torch.cuda.synchronize()
        assert torch.allclose(c, torch.matmul(a.float(), b.float()).half(), rtol=1e-2, atol=1e-1)
    finally:
        for heap in heaps:
            heap.cleanup()
