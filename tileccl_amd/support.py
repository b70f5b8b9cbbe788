"""What this build supports, as a structure (``tileccl.describe_runtime_support``).

Same shape as ``/root/reference/tileccl/support.py:29-88`` (``SupportStatus``,
``RuntimeSupportMatrix.to_dict()`` with its ``context / ops / contracts / execution_paths /
collectives / memory`` sections), filled for the surface built here: the three GEMM +
collective operations on hand-written HIP kernels, one process, ranks emulated as slices of
one device arena, plus the stand-alone collectives in their direct-write / peer-read form.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Literal

SupportState = Literal["supported", "partial", "unsupported"]


@dataclass(frozen=True, slots=True)
class SupportStatus:
    state: SupportState
    detail: str

    @property
    def supported(self) -> bool:
        return self.state == "supported"

    def to_dict(self) -> dict[str, str]:
        return {"state": self.state, "detail": self.detail}


@dataclass(frozen=True, slots=True)
class RuntimeSupportMatrix:
    backend: str
    device: str
    rank: int
    world_size: int
    has_heap: bool
    heap_mode: str | None
    transport_strategy: str | None
    runtime_surface: dict[str, object] = field(default_factory=dict)
    ops: dict[str, SupportStatus] = field(default_factory=dict)
    contracts: dict[str, SupportStatus] = field(default_factory=dict)
    execution_paths: dict[str, SupportStatus] = field(default_factory=dict)
    collectives: dict[str, SupportStatus] = field(default_factory=dict)
    memory: dict[str, SupportStatus] = field(default_factory=dict)

    def to_dict(self) -> dict[str, object]:
        section = lambda d: {name: status.to_dict() for name, status in d.items()}  # noqa: E731
        return {
            "context": {
                "backend": self.backend,
                "device": self.device,
                "rank": self.rank,
                "world_size": self.world_size,
                "has_heap": self.has_heap,
                "heap_mode": self.heap_mode,
                "transport_strategy": self.transport_strategy,
            },
            "runtime_surface": self.runtime_surface,
            "ops": section(self.ops),
            "contracts": section(self.contracts),
            "execution_paths": section(self.execution_paths),
            "collectives": section(self.collectives),
            "memory": section(self.memory),
        }


def describe_runtime_support(ctx=None) -> RuntimeSupportMatrix:
    import tileccl_amd

    ctx = ctx if ctx is not None else tileccl_amd.current_context()
    heap = ctx.heap
    has_heap = heap is not None
    yes = lambda detail: SupportStatus("supported", detail)  # noqa: E731
    no = lambda detail: SupportStatus("unsupported", detail)  # noqa: E731
    needs_heap = "supported" if has_heap or ctx.world_size == 1 else "partial"
    peer = "peers are slices of one device arena (single process); a multi-GPU heap is not built"
    fused = "bulk (S0), per-tile (S1) and TileGroup (S2) schedules on HIP kernels; fp16 / bf16, fp8 e4m3 on the 256 x 256 tile"
    return RuntimeSupportMatrix(
        backend=ctx.backend_name,
        device=ctx.device,
        rank=ctx.rank,
        world_size=ctx.world_size,
        has_heap=has_heap,
        heap_mode=heap.mode if has_heap else None,
        transport_strategy=heap.transport_strategy if has_heap else None,
        runtime_surface={"process_model": "single_process", "kernel_language": "HIP (gfx950)", "abi": "libtileccl_hip.so"},
        ops={
            "gemm_allscatter": SupportStatus(needs_heap, fused + "; " + peer),
            "gemm_allgather": SupportStatus(needs_heap, "column shards through the all-scatter launch; row blocks through tileccl_v2-style FusedGemmAllGather"),
            "gemm_reducescatter": SupportStatus(needs_heap, "column shards: per-owner GEMM + fp32 row reduce; row shards through FusedGemmReduceScatter"),
            "chained_ag_gemm_rs": SupportStatus(needs_heap, "gather launch, then GEMM with the scatter from its epilogue"),
        },
        contracts={
            "full/full": yes("default public contract"),
            "shard/shard": yes("gemm_allscatter_sharded"),
            "mixed layouts": yes("staged through a heap workspace (GemmAllScatterMixedLayoutPlan)"),
        },
        execution_paths={
            "bulk_sync": yes("two stream-ordered launches"),
            "wg_specialized": yes("one launch, per-tile locks (also as fused_sequential / producer_consumer)"),
            "tile_group": yes("one launch, per-TileGroup counters"),
        },
        collectives={
            "allreduce": SupportStatus(needs_heap, "in place (fp16 / bf16 / fp32): reduce-scatter of the caller's chunk, then direct write to every rank"),
            "allgather": SupportStatus(needs_heap, "direct write of the caller's block into every rank's output"),
            "broadcast": SupportStatus(needs_heap, "direct write by the root"),
            "scatter": SupportStatus(needs_heap, "direct write by the root, one chunk per rank"),
            "reduce_scatter": SupportStatus(needs_heap, "peer reads, fp32 accumulate; fp16 / bf16 output, fp32 from fp32 tensors"),
        },
        memory={
            "symmetric_heap": yes("bump allocator over one hipMalloc arena cut into world_size slices") if has_heap
            else SupportStatus("partial", "no heap attached to this context"),
            "multiprocess_heap": no("IPC / peer-mapped heaps across processes or GPUs are not built"),
        },
    )
