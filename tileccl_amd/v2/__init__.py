"""Planning layer and fused operations with the surface of the reference's ``tileccl_v2``.

Re-exports follow ``/root/reference/tileccl_v2/__init__.py:10-59``; the fused operations
(``FusedGemmAllGather``, ``FusedGemmReduceScatter``) and ``choose_target_group_tiles`` are
additions of this build.  Importing the planning names needs no GPU.
"""

from tileccl_amd.v2.collective_spec import CollectiveKind, CollectiveSpec, all_gather_spec, reduce_scatter_spec
from tileccl_amd.v2.cost_model import (
    CalibrationPoint,
    CostModelCalibrator,
    HardwareProfile,
    Interconnect,
    PipelineCost,
    TileCost,
    TileCostModel,
    choose_target_group_tiles,
)
from tileccl_amd.v2.tile_group import (
    TileGroup,
    TileGroupPlan,
    build_group_table,
    build_tile_group_plan,
    build_tile_groups,
    split_groups_at_row_boundaries,
    split_groups_at_row_shards,
)
from tileccl_amd.v2.transport import CommMode, P2PTransportPlan, build_p2p_transport_plan, normalize_comm_mode
from tileccl_amd.v2.wg import WGPlan, build_wg_plan

__version__ = "2.3.0-mi355x"

_DEVICE_NAMES = {
    "SymmetricHeap": "tileccl_amd.v2.heap",
    "TileGroupSignalState": "tileccl_amd.v2.signal",
    "allocate_tile_group_signals": "tileccl_amd.v2.signal",
    "FusedGemmAllGather": "tileccl_amd.v2.fused",
    "FusedGemmReduceScatter": "tileccl_amd.v2.fused",
    "translate_ptr": "tileccl_amd.v2.ipc",
    "tile_signal": "tileccl_amd.v2.ipc",
    "tile_signal_add": "tileccl_amd.v2.ipc",
    "tile_wait": "tileccl_amd.v2.ipc",
    "tile_poll": "tileccl_amd.v2.ipc",
    "tile_try_wait": "tileccl_amd.v2.ipc",
    "tile_try_poll": "tileccl_amd.v2.ipc",
    "tile_wait_ge": "tileccl_amd.v2.ipc",
    "TimelineEvent": "tileccl_amd.v2.runtime.timeline",
    "TimelineRecorder": "tileccl_amd.v2.runtime.timeline",
}


def __getattr__(name: str):
    # Names that pull in torch device code are resolved on first use.
    if name in _DEVICE_NAMES:
        import importlib

        return getattr(importlib.import_module(_DEVICE_NAMES[name]), name)
    raise AttributeError(f"module 'tileccl_amd.v2' has no attribute {name!r}")


__all__ = [
    "CalibrationPoint",
    "CollectiveKind",
    "CollectiveSpec",
    "CommMode",
    "CostModelCalibrator",
    "HardwareProfile",
    "Interconnect",
    "P2PTransportPlan",
    "PipelineCost",
    "TileCost",
    "TileCostModel",
    "TileGroup",
    "TileGroupPlan",
    "WGPlan",
    "all_gather_spec",
    "build_group_table",
    "build_p2p_transport_plan",
    "build_tile_group_plan",
    "build_tile_groups",
    "build_wg_plan",
    "choose_target_group_tiles",
    "normalize_comm_mode",
    "reduce_scatter_spec",
    "split_groups_at_row_boundaries",
    "split_groups_at_row_shards",
    *sorted(_DEVICE_NAMES),
]
