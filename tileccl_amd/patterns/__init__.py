"""Overlap patterns for GEMM + all-scatter, backed by hand-written HIP kernels.

Mirrors the plug-in seam of ``/root/reference/tileccl/patterns/__init__.py:52-169``: a
``Pattern`` holds a context and implements ``execute(A, B, C, **kwargs)`` where ``spec`` (a
``PatternExecutionSpec``) or the layout hints describe the call.

==================  =======  ==========================================================
class               variant  reference counterpart
==================  =======  ==========================================================
BulkSyncPattern     S0       patterns/bulk_sync.py (GEMM kernel, then scatter kernel)
WGSpecializedPattern S1      patterns/wg_specialized.py (one launch, per-tile locks)
TileGroupPattern    S2       the TileGroup proof kernels (README.md:66-84), contract in
                             tileccl_v2/{tile_group,signal,transport,wg}.py
==================  =======  ==========================================================

``FusedSequentialPattern`` and ``ProducerConsumerPattern`` name two further schedules of
the reference (patterns/fused_sequential.py, producer_consumer.py) that produce the same
result as S1; here they are thin subclasses of ``WGSpecializedPattern`` so that the
reference's pattern names keep working.
"""

from __future__ import annotations

import abc
import time
from typing import Any, Dict

from tileccl_amd.patterns.contracts import (
    PatternExecutionSpec,
    PatternTensorSpec,
    resolve_pattern_execution,
)


class Pattern(abc.ABC):
    """Base class: a strategy for overlapping the GEMM with the scatter of its output."""

    name: str = "base"

    def __init__(self, ctx: Any) -> None:
        self.ctx = ctx

    @abc.abstractmethod
    def execute(self, A, B, C, **kwargs: Any) -> None:
        """Compute ``C = A @ B`` and store this rank's column block into every peer's ``C``."""

    def benchmark(self, A, B, C, warmup: int = 10, iters: int = 100, **execute_kwargs: Any) -> Dict[str, Any]:
        """Wall-clock statistics over ``iters`` synchronised calls (reference :96-140)."""
        import torch

        for _ in range(warmup):
            self.execute(A, B, C, **execute_kwargs)
        torch.cuda.synchronize()
        samples = []
        for _ in range(iters):
            t0 = time.perf_counter()
            self.execute(A, B, C, **execute_kwargs)
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) * 1e3)
        return {
            "pattern": self.name,
            "mean_ms": sum(samples) / len(samples),
            "min_ms": min(samples),
            "max_ms": max(samples),
            "iters": iters,
        }

    def resolve_execution(
        self,
        A,
        B,
        C,
        *,
        spec: PatternExecutionSpec | None = None,
        full_N: int | None = None,
        b_layout: str | None = None,
        c_layout: str | None = None,
        storage_kind: str = "symmetric",
    ) -> PatternExecutionSpec:
        if spec is not None:
            return spec
        return resolve_pattern_execution(
            A,
            B,
            C,
            rank=self.ctx.rank,
            world_size=self.ctx.world_size,
            full_N=full_N,
            b_layout=b_layout,
            c_layout=c_layout,
            storage_kind=storage_kind,
        )


def _require_device_remote_access_runtime(self, *, operation: str) -> None:
    """The reference's guard against transports whose memory a device kernel cannot reach
    (patterns/__init__.py:171-185).  Every heap of this build is a slice of one device arena,
    reachable by plain loads and stores, so there is nothing to refuse; a heap is still required."""
    self.ctx.require_heap()


Pattern.require_device_remote_access_runtime = _require_device_remote_access_runtime

from tileccl_amd.patterns.hip_patterns import (  # noqa: E402
    BulkSyncPattern,
    FusedSequentialPattern,
    ProducerConsumerPattern,
    TileGroupPattern,
    WGSpecializedPattern,
)

from tileccl_amd.patterns.auto_select import auto_select, benchmark_all_patterns  # noqa: E402

__all__ = [
    "Pattern",
    "auto_select",
    "benchmark_all_patterns",
    "BulkSyncPattern",
    "FusedSequentialPattern",
    "ProducerConsumerPattern",
    "WGSpecializedPattern",
    "TileGroupPattern",
    "PatternExecutionSpec",
    "PatternTensorSpec",
    "resolve_pattern_execution",
]
