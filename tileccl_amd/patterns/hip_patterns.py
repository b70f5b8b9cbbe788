"""The three GEMM + all-scatter schedules, each one call into ``tccl_gemm_allscatter``.

Reference launch sites replaced: ``BulkSyncPattern.execute`` (patterns/bulk_sync.py:66-156),
``WGSpecializedPattern.execute`` (patterns/wg_specialized.py:130-204).  ``TileGroupPattern``
has no in-tree reference kernel; it follows the planning contract of ``tileccl_v2``.
"""

from __future__ import annotations

import ctypes as C
from typing import Any

import torch

from tileccl_amd import _launch, _lib
from tileccl_amd.patterns import Pattern
from tileccl_amd.patterns.runtime import resolve_dual_role_scheduler
from tileccl_amd.v2.tile_group import TileGroupPlan, build_tile_group_plan


class _HipAllScatterPattern(Pattern):
    """Shared marshalling: resolve the contract, build descriptors, launch."""

    variant = _lib.S0_BULK

    def __init__(
        self,
        ctx: Any,
        BLOCK_M: int = 128,
        BLOCK_N: int = 128,
        BLOCK_K: int = 64,
        NUM_SMS: int = 0,
        COMPUTE_SMS: int = 0,
        COMM_SMS: int = 0,
        GROUP_M: int = 8,
    ) -> None:
        super().__init__(ctx)
        if BLOCK_K != 64:
            raise ValueError(f"BLOCK_K={BLOCK_K}: the MFMA kernel consumes K in steps of 64")
        if BLOCK_M % 128 or BLOCK_N % 128 or BLOCK_M <= 0 or BLOCK_N <= 0:
            raise ValueError(f"BLOCK_M x BLOCK_N = {BLOCK_M} x {BLOCK_N} must be multiples of 128")
        self.BLOCK_M, self.BLOCK_N, self.BLOCK_K, self.GROUP_M = BLOCK_M, BLOCK_N, BLOCK_K, GROUP_M
        self.NUM_SMS, self.COMPUTE_SMS, self.COMM_SMS = NUM_SMS, COMPUTE_SMS, COMM_SMS
        # Signal words are cut from the heap, which never gives memory back, and a pattern named
        # by a string is instantiated anew on every call (ops._resolve_pattern_impl, as in the
        # reference, ops.py:1289-1296): they are therefore kept with the context, next to its
        # workspaces, and shared by every pattern instance of the same kind and tiling.
        cache = getattr(ctx, "_workspace_cache", None)
        self._sync: dict[tuple, _launch.SyncWords] = cache if isinstance(cache, dict) else {}

    # -- hooks -------------------------------------------------------------------------
    def _sync_words(self, M: int, N: int, C_out: torch.Tensor) -> _launch.SyncWords | None:
        return None

    def _wg_split(self) -> tuple[int, int]:
        """(GEMM workgroups or 0 for the library default, communication workgroups or 0)."""
        return self.NUM_SMS, 0

    # -- execution ---------------------------------------------------------------------
    def execute(self, A, B, C_out, **kwargs: Any) -> None:
        spec = self.resolve_execution(
            A,
            B,
            C_out,
            spec=kwargs.get("spec"),
            full_N=kwargs.get("full_N"),
            b_layout=kwargs.get("b_layout"),
            c_layout=kwargs.get("c_layout"),
            storage_kind=kwargs.get("storage_kind", "symmetric"),
        )
        heap = self.ctx.require_heap()
        if spec.world_size > 1 and not heap.owns_tensor(C_out):
            raise ValueError(
                "C must live in the symmetric heap when world_size > 1: the scatter writes it at the "
                "same offset in every peer's slice"
            )
        compute_wgs, comm_wgs = self._wg_split()
        gemm = _launch.gemm_desc(
            A, B, C_out, block_m=self.BLOCK_M, block_n=self.BLOCK_N, group_m=self.GROUP_M, num_wgs=compute_wgs
        )
        scatter = _lib.ScatterDesc(
            spec.scatter_src_col_offset, spec.scatter_cols, spec.scatter_dst_leading_dim, spec.scatter_dst_col_offset
        )
        view = _launch.heap_view(self.ctx.heap_bases, spec.rank, spec.world_size)
        transport = _launch.transport_desc(_lib.DIR_PUSH, self._copy_elems(), None, comm_wgs)
        words = self._sync_words(spec.M, spec.local_N, C_out)
        sync = None
        if words is not None:
            variant = "s1" if self.variant == _lib.S1_TILE else "s2"
            words.next_epoch(variant)
            sync = words.desc(variant)
        rc = _lib.load().tccl_gemm_allscatter(
            C.byref(gemm),
            C.byref(scatter),
            C.byref(view),
            C.byref(sync) if sync is not None else None,
            C.byref(transport),
            self.variant,
            _launch.stream_ptr(),
        )
        _lib.check(rc, f"tccl_gemm_allscatter[{self.name}]")
        self._last_sync = words

    def _copy_elems(self) -> int:
        return 16384

    def check_faults(self) -> None:
        """Synchronise and raise if the last launch's communication role timed out."""
        words = getattr(self, "_last_sync", None)
        if words is not None:
            words.raise_if_faulted()


class BulkSyncPattern(_HipAllScatterPattern):
    """S0: persistent GEMM kernel, then a scatter kernel, ordered by the stream.

    The reference puts a device-wide synchronize between the two kernels
    (bulk_sync.py:127); stream order gives the same dependency without stalling the host.
    """

    name = "bulk_sync"
    variant = _lib.S0_BULK


class WGSpecializedPattern(_HipAllScatterPattern):
    """S1: one launch; GEMM workgroups signal each tile, communication workgroups drain them."""

    name = "wg_specialized"
    variant = _lib.S1_TILE
    _COMM_SM_FRACTION = 0.2

    def _wg_split(self) -> tuple[int, int]:
        if self.COMPUTE_SMS > 0 or self.COMM_SMS > 0:
            units = self.ctx.backend.get_device_properties().compute_units
            split = resolve_dual_role_scheduler(
                units, compute_sms=self.COMPUTE_SMS, comm_sms=self.COMM_SMS, comm_sm_fraction=self._COMM_SM_FRACTION
            )
            return split.compute_sms, split.comm_sms
        # Default: communication workgroups share CUs with the GEMM workgroups instead of
        # taking CUs away from them (LDS and registers of gfx950 allow three workgroups per CU).
        return 0, 0

    def _sync_words(self, M: int, N: int, C_out: torch.Tensor) -> _launch.SyncWords:
        tiles = -(-M // self.BLOCK_M) * -(-N // self.BLOCK_N)
        key = ("tileccl_amd.sync", "locks", tiles)
        words = self._sync.get(key)
        if words is None:
            heap = self.ctx.require_heap()
            locks = heap.allocate_tensor((tiles,), torch.int32)
            locks.zero_()
            words = self._sync[key] = _launch.SyncWords(locks=locks)
        return words


class FusedSequentialPattern(WGSpecializedPattern):
    """Reference name kept (patterns/fused_sequential.py); runs the S1 schedule."""

    name = "fused_sequential"


class ProducerConsumerPattern(WGSpecializedPattern):
    """Reference name kept (patterns/producer_consumer.py); runs the S1 schedule."""

    name = "producer_consumer"


class TileGroupPattern(_HipAllScatterPattern):
    """S2: one launch; tiles count into per-TileGroup counters, whole groups are moved."""

    name = "tile_group"
    variant = _lib.S2_TILEGROUP

    def __init__(self, ctx: Any, *args: Any, target_group_tiles: int | None = None, copy_elems: int = 16384,
                 tau_min_bytes: int = 262144, max_groups: int = 64, **kwargs: Any) -> None:
        super().__init__(ctx, *args, **kwargs)
        self.target_group_tiles = target_group_tiles
        self.copy_elems = copy_elems
        self.tau_min_bytes = tau_min_bytes
        self.max_groups = max_groups
        self.last_plan: TileGroupPlan | None = None

    def _copy_elems(self) -> int:
        return self.copy_elems

    def _wg_split(self) -> tuple[int, int]:
        return self.COMPUTE_SMS, self.COMM_SMS

    def plan_for(self, M: int, N: int, elem_bytes: int) -> TileGroupPlan:
        return build_tile_group_plan(
            M,
            N,
            self.BLOCK_M * self.BLOCK_N * elem_bytes,
            target_group_tiles=self.target_group_tiles,
            max_groups=self.max_groups,
            block_m=self.BLOCK_M,
            block_n=self.BLOCK_N,
            group_m=self.GROUP_M,
            tau_min_bytes=self.tau_min_bytes,
        )

    def _sync_words(self, M: int, N: int, C_out: torch.Tensor) -> _launch.SyncWords:
        key = ("tileccl_amd.sync", "groups", M, N, C_out.element_size(), self.BLOCK_M, self.BLOCK_N, self.GROUP_M,
               self.target_group_tiles, self.tau_min_bytes, self.max_groups)
        words = self._sync.get(key)
        if words is None:
            plan = self.plan_for(M, N, C_out.element_size())
            heap = self.ctx.require_heap()
            counter = heap.allocate_tensor((plan.n_groups,), torch.int32)
            barrier = heap.allocate_tensor((plan.n_groups,), torch.int32)
            counter.zero_()
            barrier.zero_()
            words = self._sync[key] = _launch.SyncWords(
                counter=counter, barrier=barrier, plan=_launch.DevicePlan.upload(plan)
            )
            words.host_plan = plan
        self.last_plan = words.host_plan
        return words
