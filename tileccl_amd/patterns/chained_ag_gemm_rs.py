"""AllGather -> GEMM -> scatter as one call into ``tccl_chained_ag_gemm_rs``.

Host side of ``ChainedAGGemmRSPattern`` (``/root/reference/tileccl/patterns/chained_ag_gemm_rs.py:40-200``):
every rank holds an ``(M, K_shard)`` column shard of the input; the pattern gathers the
shards into an ``(M, K)`` workspace (column block ``p`` from rank ``p``), multiplies by the full
weight ``W (K, N)`` and stores the ``(M, N)`` result into every peer's output as well as its own.

Stages on MI355X, by ``schedule``: ``"bulk_sync"`` is three launches (gather copy, GEMM
kernel, copy to the peers).  ``"wg_specialized"`` (per tile) and ``"tile_group"`` (per
TileGroup; the default) are one launch on the 256 x 256 tile: the K loops read every
rank's shard where it lies (the shards are resident inputs at the same offset of every
slice), the gathered workspace is filled on the side by the same launch's background
transfer, and the stores to the peers leave from the GEMM epilogue, so neither the gather
nor the scatter is waited for.  Shapes the large tile does not take (small outputs, shards
that are not whole 64-element K steps) run the gather as a bulk launch ahead of the fused
GEMM + scatter launch.

The reference kernel addresses the workspace rows with the column stride
(``gathered_ptr + offs_m * stride_gk``, :298 and :353), so its rows overlap; the result
meant by its docstring, ``concat_k(shards) @ W``, is what is computed here.
"""

from __future__ import annotations

import ctypes as C
from typing import Any

import torch

from tileccl_amd import _launch, _lib
from tileccl_amd.patterns.hip_patterns import BulkSyncPattern, TileGroupPattern, WGSpecializedPattern

_SCHEDULES = {"bulk_sync": BulkSyncPattern, "wg_specialized": WGSpecializedPattern, "tile_group": TileGroupPattern}


class ChainedAGGemmRSPattern:
    """Three stages, gather -> GEMM -> scatter, for column-sharded inputs.

    Arguments as in the reference (:40-75).  The ``*_SMS`` arguments are accepted for
    signature parity; the launch geometry follows the library defaults, because the stages
    are not separate workgroup roles here (see the module docstring).
    """

    name: str = "chained_ag_gemm_rs"

    def __init__(
        self,
        ctx: Any,
        BLOCK_M: int = 128,
        BLOCK_N: int = 128,
        BLOCK_K: int = 64,
        GATHER_SMS: int = 0,
        COMPUTE_SMS: int = 0,
        SCATTER_SMS: int = 0,
        schedule: str = "tile_group",
    ) -> None:
        if schedule not in _SCHEDULES:
            raise ValueError(f"unknown schedule {schedule!r}; choose from {sorted(_SCHEDULES)}")
        self.ctx = ctx
        self.BLOCK_M, self.BLOCK_N, self.BLOCK_K = BLOCK_M, BLOCK_N, BLOCK_K
        self.GATHER_SMS, self.COMPUTE_SMS, self.SCATTER_SMS = GATHER_SMS, COMPUTE_SMS, SCATTER_SMS
        self.schedule = schedule
        # The GEMM + scatter stages reuse the all-scatter pattern's plan and signal words.
        self._stage = _SCHEDULES[schedule](ctx, BLOCK_M=BLOCK_M, BLOCK_N=BLOCK_N, BLOCK_K=BLOCK_K)
        self._last_sync: _launch.SyncWords | None = None

    def execute(
        self,
        input_shard: torch.Tensor,
        W: torch.Tensor,
        output: torch.Tensor,
        gathered_workspace: torch.Tensor | None = None,
    ) -> torch.Tensor:
        M, K_shard = input_shard.shape
        K, N = W.shape
        world_size = self.ctx.world_size
        if K_shard * world_size != K:
            raise ValueError(
                f"input_shard columns ({K_shard}) * world_size ({world_size}) != W rows ({K})"
            )
        if tuple(output.shape) != (M, N):
            raise ValueError(f"output shape {tuple(output.shape)} must be (M, N) = ({M}, {N})")
        heap = self.ctx.require_heap()
        if world_size > 1:
            for name, t in (("input_shard", input_shard), ("output", output)):
                if not heap.owns_tensor(t):
                    raise ValueError(
                        f"{name} must live in the symmetric heap when world_size > 1: peers address it "
                        "at the same offset in their slices"
                    )
        if gathered_workspace is None:
            gathered_workspace = self.ctx.workspace(
                "chained_ag_gemm_rs.gathered_input", M, K, dtype=input_shard.dtype
            )
        elif tuple(gathered_workspace.shape) != (M, K) or gathered_workspace.dtype != input_shard.dtype:
            raise ValueError(f"gathered_workspace must be ({M}, {K}) of {input_shard.dtype}")

        gemm = _launch.gemm_desc(
            gathered_workspace, W, output, block_m=self.BLOCK_M, block_n=self.BLOCK_N, group_m=self._stage.GROUP_M
        )
        view = _launch.heap_view(self.ctx.heap_bases, self.ctx.rank, world_size)
        compute_wgs, comm_wgs = self._stage._wg_split()
        gemm.num_wgs = compute_wgs
        transport = _launch.transport_desc(_lib.DIR_PUSH, self._stage._copy_elems(), None, comm_wgs)
        words = self._stage._sync_words(M, N, output)
        sync = None
        if words is not None:
            variant = "s1" if self._stage.variant == _lib.S1_TILE else "s2"
            words.next_epoch(variant)
            sync = words.desc(variant)
        rc = _lib.load().tccl_chained_ag_gemm_rs(
            C.byref(gemm),
            _launch.ptr(input_shard),
            _launch._row_major(input_shard, "input_shard"),
            K_shard,
            C.byref(view),
            C.byref(sync) if sync is not None else None,
            C.byref(transport),
            self._stage.variant,
            _launch.stream_ptr(),
        )
        _lib.check(rc, f"tccl_chained_ag_gemm_rs[{self.schedule}]")
        self._last_sync = words
        return output

    def check_faults(self) -> None:
        """Synchronise and raise if a bounded device-side wait of the last launch expired."""
        if self._last_sync is not None:
            self._last_sync.raise_if_faulted()
