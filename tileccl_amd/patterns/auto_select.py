"""Pattern selection and the all-patterns benchmark table.

Mirrors ``/root/reference/tileccl/patterns/auto_select.py``: ``auto_select(op, M, N, K,
world_size, hw_info=None, ctx=None)`` returns a pattern class (or an instance bound to ``ctx``)
and ``benchmark_all_patterns`` times every pattern on one problem.

Two policies.  ``"mi355x"`` (default) is what the measurements on this hardware say: the
TileGroup schedule beat the per-tile and the bulk schedule at every configuration measured
(1.16x-1.37x over bulk), so it is chosen whenever there is a peer; without one the plain
GEMM runs (nothing to move).  ``"reference"`` reproduces the
reference's decision tree (auto_select.py:128-188), whose thresholds come from H100 / MI300X
observations, for callers that want the identical choice.
"""

from __future__ import annotations

from typing import Any, Dict, List, Optional

_SUPPORTED_OPS = {"gemm_allscatter", "gemm_allgather", "gemm_reducescatter"}


def _detect_hardware_info() -> tuple[int, float]:
    """(compute units, link GB/s) of the current device; the reference's conservative
    defaults (auto_select.py:23-38) when no device can be queried."""
    try:
        from tileccl_amd.backends import get_backend

        props = get_backend().get_device_properties()
        units = props.compute_units if props.compute_units > 0 else 132
        return units, 300.0
    except Exception:
        return 132, 300.0


def reference_choice(M: int, N: int, K: int, world_size: int, sm_count: int, bw_gb_s: float) -> str:
    """Name of the pattern the reference's heuristic picks (auto_select.py:128-188)."""
    n_per_rank = N // max(world_size, 1)
    total_tiles_128 = ((M + 127) // 128) * ((n_per_rank + 127) // 128)
    flops = 2 * M * n_per_rank * K
    scatter_bytes = M * n_per_rank * 2  # the reference assumes fp16 here
    compute_intensity = flops / max(scatter_bytes, 1)
    bw_scale = bw_gb_s / 300.0 if bw_gb_s > 0 else 1.0
    if M < 256:
        return "bulk_sync"
    if n_per_rank < 1024 and K > int(12288 * bw_scale):
        return "fused_sequential"
    if n_per_rank < 2048 and K > int(6144 * bw_scale):
        return "producer_consumer"
    if total_tiles_128 >= sm_count and K > int(4096 * bw_scale):
        return "wg_specialized"
    if N > 4096 and K > int(8192 * bw_scale):
        return "wg_specialized"
    if compute_intensity > 256 and total_tiles_128 > 16:
        return "fused_sequential"
    return "bulk_sync"


def measured_choice(M: int, N: int, K: int, world_size: int) -> str:
    """Choice by what was measured on MI355X (see the module docstring)."""
    del M, N, K
    return "tile_group" if world_size > 1 else "bulk_sync"


def auto_select(
    op: str,
    M: int,
    N: int,
    K: int,
    world_size: int,
    hw_info: Optional[Any] = None,
    ctx: Optional[Any] = None,
    policy: str = "mi355x",
):
    """Pattern instance bound to ``ctx``, or the pattern class when ``ctx`` is None."""
    from tileccl_amd.patterns.hip_patterns import (
        BulkSyncPattern,
        FusedSequentialPattern,
        ProducerConsumerPattern,
        TileGroupPattern,
        WGSpecializedPattern,
    )

    if op not in _SUPPORTED_OPS:
        raise ValueError(
            f"Unsupported operation {op!r}.  "
            f"Supported operations: {sorted(_SUPPORTED_OPS)}"
        )
    if policy == "reference":
        if hw_info is not None:
            sm_count = getattr(hw_info, "compute_units", 132)
            bw = getattr(hw_info, "link_bandwidth_gbps", 300.0)
        else:
            sm_count, bw = _detect_hardware_info()
        name = reference_choice(M, N, K, world_size, sm_count, bw)
    elif policy == "mi355x":
        name = measured_choice(M, N, K, world_size)
    else:
        raise ValueError(f"unknown policy {policy!r}; choose 'mi355x' or 'reference'")
    cls = {
        "bulk_sync": BulkSyncPattern,
        "fused_sequential": FusedSequentialPattern,
        "producer_consumer": ProducerConsumerPattern,
        "wg_specialized": WGSpecializedPattern,
        "tile_group": TileGroupPattern,
    }[name]
    return cls(ctx) if ctx is not None else cls


def benchmark_all_patterns(
    A,
    B,
    C,
    ctx: Any,
    warmup: int = 10,
    iters: int = 100,
    *,
    spec: Any | None = None,
    full_N: int | None = None,
    b_layout: str | None = None,
    c_layout: str | None = None,
) -> Dict[str, Any]:
    """Time every pattern on one problem; result dict as the reference's (auto_select.py:194-308)."""
    from tileccl_amd.ops import build_gemm_allscatter_plan
    from tileccl_amd.patterns.hip_patterns import (
        BulkSyncPattern,
        FusedSequentialPattern,
        ProducerConsumerPattern,
        TileGroupPattern,
        WGSpecializedPattern,
    )

    execution = spec
    if execution is None:
        execution = build_gemm_allscatter_plan(
            A, B, C, ctx=ctx, full_N=full_N, b_layout=b_layout, c_layout=c_layout
        ).execution
    results: List[Dict[str, Any]] = []
    for cls in (BulkSyncPattern, FusedSequentialPattern, ProducerConsumerPattern, WGSpecializedPattern, TileGroupPattern):
        plan = build_gemm_allscatter_plan(
            A,
            B,
            C,
            ctx=ctx,
            full_N=execution.full_N,
            b_layout=execution.rhs_layout,
            c_layout=execution.output_layout,
            pattern=cls,
        )
        try:
            results.append(plan.pattern_impl.benchmark(A, B, C, warmup=warmup, iters=iters, spec=plan.execution))
        except Exception as e:  # a failing pattern is recorded, the others still run
            results.append({
                "pattern": plan.pattern_name,
                "mean_ms": float("inf"),
                "min_ms": float("inf"),
                "max_ms": float("inf"),
                "iters": 0,
                "error": str(e),
            })
    results.sort(key=lambda r: r["mean_ms"])
    return {
        "results": results,
        "best": results[0]["pattern"] if results else "none",
        "M": execution.M,
        "N": execution.full_N,
        "K": execution.K,
        "local_N": execution.local_N,
        "layout_mode": execution.output_layout,
        "world_size": ctx.world_size,
    }
