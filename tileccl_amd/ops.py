"""High-level GEMM + all-scatter entry points.

Mirrors the ``gemm_allscatter`` part of ``/root/reference/tileccl/ops.py``:
``GemmAllScatterContract`` (:96-125), ``GemmAllScatterPlan`` (:128-194),
``GemmAllScatterMixedLayoutPlan`` (:197-279), ``build_gemm_allscatter_plan`` (:702-807),
``gemm_allscatter`` (:810-857), ``gemm_allscatter_sharded`` (:860-888),
``_resolve_pattern_impl`` (:1261-1303), ``_resolve_public_layout_contract`` (:1306-1325),
``_resolve_gemm_allscatter_contract`` (:1328-1404).  The reference's other ops
(all-reduce, stand-alone collectives, host-staged pipelines) are not part of this path.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Literal

import tileccl_amd
from tileccl_amd.patterns import (
    BulkSyncPattern,
    FusedSequentialPattern,
    Pattern,
    ProducerConsumerPattern,
    TileGroupPattern,
    WGSpecializedPattern,
)
from tileccl_amd.patterns.contracts import PatternExecutionSpec, resolve_pattern_execution

__all__ = [
    "gemm_allgather",
    "gemm_reducescatter",
    "allgather",
    "allreduce",
    "reduce_scatter",
    "allgather_gemm_reducescatter",
    "build_allgather_plan",
    "build_allreduce_plan",
    "build_reduce_scatter_plan",
    "build_gemm_allgather_plan",
    "build_gemm_reducescatter_plan",
    "build_allgather_gemm_reducescatter_plan",
    "AllGatherPlan",
    "AllReducePlan",
    "ReduceScatterPlan",
    "GemmAllGatherPlan",
    "GemmReduceScatterPlan",
    "AllGatherGemmReduceScatterPlan",
    "AllGatherGemmReduceScatterContract",
    "gemm_allscatter",
    "gemm_allscatter_sharded",
    "build_gemm_allscatter_plan",
    "GemmAllScatterPlan",
    "GemmAllScatterMixedLayoutPlan",
    "GemmAllScatterContract",
]

from tileccl_amd.ops_collective import gemm_allgather, gemm_reducescatter  # noqa: E402  (re-exported)
from tileccl_amd.ops_plans import (  # noqa: E402  (re-exported)
    AllGatherGemmReduceScatterContract,
    AllGatherGemmReduceScatterPlan,
    AllGatherPlan,
    AllReducePlan,
    GemmAllGatherPlan,
    GemmReduceScatterPlan,
    ReduceScatterPlan,
    allgather,
    allgather_gemm_reducescatter,
    allreduce,
    build_allgather_gemm_reducescatter_plan,
    build_allgather_plan,
    build_allreduce_plan,
    build_gemm_allgather_plan,
    build_gemm_reducescatter_plan,
    build_reduce_scatter_plan,
    reduce_scatter,
)

PatternLike = str | type[Pattern] | Pattern | None
LayoutKind = Literal["full", "shard"]

# Reference aliases (ops.py:74-83) plus the names of the three measured variants.
_PATTERN_ALIASES: dict[str, type[Pattern] | None] = {
    "auto": None,
    "bulk_sync": BulkSyncPattern,
    "fused_sequential": FusedSequentialPattern,
    "fused_seq": FusedSequentialPattern,
    "producer_consumer": ProducerConsumerPattern,
    "pc": ProducerConsumerPattern,
    "wg_specialized": WGSpecializedPattern,
    "wg_spec": WGSpecializedPattern,
    "tile_group": TileGroupPattern,
    "s0": BulkSyncPattern,
    "s1": WGSpecializedPattern,
    "s2": TileGroupPattern,
}


@dataclass(frozen=True, slots=True)
class GemmAllScatterContract:
    """What the caller asked for, after validation: shapes, layouts, rank."""

    M: int
    K: int
    full_N: int
    rhs_cols: int
    output_cols: int
    rank: int
    world_size: int
    rhs_layout: LayoutKind
    output_layout: LayoutKind
    storage_kind: str = "symmetric"

    def to_dict(self) -> dict[str, object]:
        return {name: getattr(self, name) for name in self.__slots__}


def _ctx_dict(ctx) -> dict[str, object]:
    return {"rank": ctx.rank, "world_size": ctx.world_size, "backend": ctx.backend_name, "device": ctx.device}


@dataclass(frozen=True, slots=True)
class GemmAllScatterPlan:
    """A validated contract bound to a pattern instance; ``execute`` may be called repeatedly."""

    ctx: "tileccl_amd.TileCCLContext"
    execution: PatternExecutionSpec
    pattern_name: str
    pattern_impl: Pattern = field(repr=False)
    storage_kind: str = "symmetric"

    def validate_tensors(self, A: Any, B: Any, C: Any) -> None:
        fresh = resolve_pattern_execution(
            A,
            B,
            C,
            rank=self.ctx.rank,
            world_size=self.ctx.world_size,
            full_N=self.execution.full_N,
            b_layout=self.execution.rhs_layout,
            c_layout=self.execution.output_layout,
            storage_kind=self.storage_kind,
        )
        if fresh != self.execution:
            raise ValueError(
                "Tensor contract no longer matches this GemmAllScatterPlan. "
                "Build a new plan for tensors with different logical or physical layout."
            )

    def execute(self, A: Any, B: Any, C: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(A, B, C)
        self.pattern_impl.execute(A, B, C, spec=self.execution)
        return C

    def to_dict(self) -> dict[str, object]:
        return {
            "op": "gemm_allscatter",
            "pattern": self.pattern_name,
            "ctx": _ctx_dict(self.ctx),
            "storage_kind": self.storage_kind,
            "execution": self.execution.to_dict(),
        }


@dataclass(frozen=True, slots=True)
class GemmAllScatterMixedLayoutPlan:
    """``B`` full, ``C`` shard: run full/full into a heap workspace, then copy the rank's block out."""

    ctx: "tileccl_amd.TileCCLContext"
    contract: GemmAllScatterContract
    pattern_name: str
    direct_plan: GemmAllScatterPlan = field(repr=False)
    materialization: str = "full_to_shard"
    storage_kind: str = "symmetric"

    def validate_tensors(self, A: Any, B: Any, C: Any) -> None:
        fresh = _resolve_gemm_allscatter_contract(
            A,
            B,
            C,
            ctx=self.ctx,
            full_N=self.contract.full_N,
            b_layout=self.contract.rhs_layout,
            c_layout=self.contract.output_layout,
            storage_kind=self.storage_kind,
        )
        if fresh != self.contract:
            raise ValueError(
                "Tensor contract no longer matches this mixed-layout GemmAllScatter plan. "
                "Build a new plan for tensors with different logical or physical layout."
            )

    def execute(self, A: Any, B: Any, C: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(A, B, C)
        if self.materialization != "full_to_shard":
            raise RuntimeError(f"Unsupported mixed-layout materialization {self.materialization!r}")
        k = self.contract
        if k.world_size == 1:
            self.direct_plan.execute(A, B, C, validate=False)
            return C
        full = self.ctx.workspace("gemm_allscatter.full_output", k.M, k.full_N, dtype=C.dtype)
        self.direct_plan.execute(A, B, full, validate=False)
        first = k.rank * k.output_cols
        C.copy_(full[:, first : first + k.output_cols])
        return C

    def to_dict(self) -> dict[str, object]:
        return {
            "op": "gemm_allscatter",
            "materialization": self.materialization,
            "pattern": self.pattern_name,
            "ctx": _ctx_dict(self.ctx),
            "storage_kind": self.storage_kind,
            "public_contract": self.contract.to_dict(),
            "direct_plan": self.direct_plan.to_dict(),
        }


class _ShapeOnly:
    """Stand-in for a tensor when only its 2-D shape matters to contract resolution."""

    def __init__(self, shape: tuple[int, int]) -> None:
        self.shape = shape
        self.ndim = len(shape)


def _implied_full_N(cols: int, layout: str, world_size: int) -> int:
    return cols if layout == "full" or world_size == 1 else cols * world_size


def _resolve_public_layout_contract(*, b_layout: str | None, c_layout: str | None) -> tuple[str, str]:
    """No hints means full/full; a single hint is an error (reference ops.py:1306-1325)."""
    if b_layout is None and c_layout is None:
        return "full", "full"
    if (b_layout is None) != (c_layout is None):
        raise ValueError(
            "b_layout and c_layout must be specified together. "
            "Use gemm_allscatter(...) for the default full/full public contract, "
            "or gemm_allscatter_sharded(...) for the shard/shard expert contract."
        )
    return b_layout, c_layout  # type: ignore[return-value]


def _resolve_gemm_allscatter_contract(
    A: Any, B: Any, C: Any, *, ctx, full_N: int | None, b_layout: str, c_layout: str, storage_kind: str
) -> GemmAllScatterContract:
    ctx.require_heap()
    if A.ndim != 2 or B.ndim != 2 or C.ndim != 2:
        raise ValueError(
            f"gemm_allscatter expects 2-D tensors: got A.ndim={A.ndim}, B.ndim={B.ndim}, C.ndim={C.ndim}"
        )
    if any(str(t.device) != ctx.device for t in (A, B, C)):
        raise ValueError(
            "gemm_allscatter tensors must all reside on the context device "
            f"{ctx.device}, got A={A.device}, B={B.device}, C={C.device}"
        )
    M, K = int(A.shape[0]), int(A.shape[1])
    b_rows, b_cols = int(B.shape[0]), int(B.shape[1])
    c_rows, c_cols = int(C.shape[0]), int(C.shape[1])
    if b_rows != K:
        raise ValueError(f"B.shape[0] must equal A.shape[1]: got {b_rows} vs {K}")
    if c_rows != M:
        raise ValueError(f"C.shape[0] must equal A.shape[0]: got {c_rows} vs {M}")

    ws = ctx.world_size
    if full_N is None:
        implied = {_implied_full_N(b_cols, b_layout, ws), _implied_full_N(c_cols, c_layout, ws)}
        if len(implied) != 1:
            raise ValueError(f"Provided layout hints disagree on full_N: resolved candidates={sorted(implied)}")
        N = implied.pop()
    else:
        N = int(full_N)
    if N <= 0:
        raise ValueError(f"full_N must be positive, got {N}")
    if N % ws != 0:
        raise ValueError(f"full_N must be divisible by world_size: {N} % {ws} != 0")

    shard = N if ws == 1 else N // ws
    want_b = N if b_layout == "full" else shard
    want_c = N if c_layout == "full" else shard
    if b_cols != want_b:
        raise ValueError(f"B layout={b_layout!r} expects {want_b} columns, got {b_cols}")
    if c_cols != want_c:
        raise ValueError(f"C layout={c_layout!r} expects {want_c} columns, got {c_cols}")
    return GemmAllScatterContract(
        M=M,
        K=K,
        full_N=N,
        rhs_cols=b_cols,
        output_cols=c_cols,
        rank=ctx.rank,
        world_size=ws,
        rhs_layout=b_layout,  # type: ignore[arg-type]
        output_layout=c_layout,  # type: ignore[arg-type]
        storage_kind=storage_kind,
    )


def _auto_pattern(ctx, execution: PatternExecutionSpec, hw_info: object | None = None) -> Pattern:
    """``pattern="auto"``: the selection engine, as in the reference (ops.py:1283-1292)."""
    from tileccl_amd.patterns.auto_select import auto_select

    return auto_select(
        "gemm_allscatter", M=execution.M, N=execution.full_N, K=execution.K,
        world_size=execution.world_size, hw_info=hw_info, ctx=ctx,
    )


def _resolve_pattern_impl(*, pattern: PatternLike, ctx, execution: PatternExecutionSpec, hw_info: object | None) -> Pattern:
    if isinstance(pattern, Pattern):
        owner = getattr(pattern, "ctx", None)
        if owner is not None:
            if getattr(owner, "rank", ctx.rank) != ctx.rank:
                raise ValueError(
                    "Pattern instance rank does not match the provided context: "
                    f"{getattr(owner, 'rank', None)} != {ctx.rank}"
                )
            if getattr(owner, "world_size", ctx.world_size) != ctx.world_size:
                raise ValueError(
                    "Pattern instance world_size does not match the provided context: "
                    f"{getattr(owner, 'world_size', None)} != {ctx.world_size}"
                )
        return pattern
    if pattern is None or pattern == "auto":
        return _auto_pattern(ctx, execution, hw_info)
    if isinstance(pattern, str):
        cls = _PATTERN_ALIASES.get(pattern)
        if cls is None:
            raise ValueError(f"Unknown pattern {pattern!r}. Supported: {sorted(_PATTERN_ALIASES)}")
        return cls(ctx)
    if isinstance(pattern, type) and issubclass(pattern, Pattern):
        return pattern(ctx)
    raise TypeError("pattern must be a pattern name, Pattern subclass, Pattern instance, or 'auto'")


def build_gemm_allscatter_plan(
    A: Any,
    B: Any,
    C: Any,
    *,
    ctx=None,
    full_N: int | None = None,
    b_layout: str | None = None,
    c_layout: str | None = None,
    pattern: PatternLike = "auto",
    hw_info: object | None = None,
    storage_kind: str = "symmetric",
) -> GemmAllScatterPlan | GemmAllScatterMixedLayoutPlan:
    """Resolve the contract once and bind it to a pattern."""
    ctx = ctx if ctx is not None else tileccl_amd.current_context()
    b_kind, c_kind = _resolve_public_layout_contract(b_layout=b_layout, c_layout=c_layout)
    contract = _resolve_gemm_allscatter_contract(
        A, B, C, ctx=ctx, full_N=full_N, b_layout=b_kind, c_layout=c_kind, storage_kind=storage_kind
    )

    def direct(c_like: Any, b_kind_: str, c_kind_: str) -> GemmAllScatterPlan:
        execution = resolve_pattern_execution(
            A,
            B,
            c_like,
            rank=ctx.rank,
            world_size=ctx.world_size,
            full_N=contract.full_N,
            b_layout=b_kind_,
            c_layout=c_kind_,
            storage_kind=storage_kind,
        )
        impl = _resolve_pattern_impl(pattern=pattern, ctx=ctx, execution=execution, hw_info=hw_info)
        return GemmAllScatterPlan(
            ctx=ctx, execution=execution, pattern_name=impl.name, pattern_impl=impl, storage_kind=storage_kind
        )

    if contract.rhs_layout == "full" and contract.output_layout == "shard":
        inner = direct(_ShapeOnly((contract.M, contract.full_N)), "full", "full")
        return GemmAllScatterMixedLayoutPlan(
            ctx=ctx,
            contract=contract,
            pattern_name=inner.pattern_name,
            direct_plan=inner,
            materialization="full_to_shard",
            storage_kind=storage_kind,
        )
    if contract.rhs_layout != contract.output_layout:
        raise ValueError(
            "Mixed multi-rank layout wrapper is only implemented for b_layout='full', "
            "c_layout='shard' right now. "
            "The inverse shard/full case is intentionally still rejected because "
            "current gemm_allscatter shard/shard execution does not define a stable "
            "local-shard ownership contract for assembling a full output; that path "
            "belongs to a future gemm_allgather-style API. "
            f"Got b_layout={contract.rhs_layout!r}, c_layout={contract.output_layout!r}."
        )
    return direct(C, contract.rhs_layout, contract.output_layout)


def gemm_allscatter(
    A: Any,
    B: Any,
    C: Any,
    *,
    ctx=None,
    full_N: int | None = None,
    b_layout: str | None = None,
    c_layout: str | None = None,
    pattern: PatternLike = "auto",
    hw_info: object | None = None,
    storage_kind: str = "symmetric",
) -> Any:
    """``C = A @ B`` on this rank, then this rank's column block lands in every peer's ``C``."""
    plan = build_gemm_allscatter_plan(
        A,
        B,
        C,
        ctx=ctx,
        full_N=full_N,
        b_layout=b_layout,
        c_layout=c_layout,
        pattern=pattern,
        hw_info=hw_info,
        storage_kind=storage_kind,
    )
    return plan.execute(A, B, C, validate=False)


def gemm_allscatter_sharded(
    A: Any,
    B_shard: Any,
    C_shard: Any,
    *,
    full_N: int,
    ctx=None,
    pattern: PatternLike = "auto",
    hw_info: object | None = None,
    storage_kind: str = "symmetric",
) -> Any:
    """shard/shard contract: ``B_shard (K, N/ws)``, ``C_shard (M, N/ws)``; ``full_N`` is mandatory."""
    plan = build_gemm_allscatter_plan(
        A,
        B_shard,
        C_shard,
        ctx=ctx,
        full_N=full_N,
        b_layout="shard",
        c_layout="shard",
        pattern=pattern,
        hw_info=hw_info,
        storage_kind=storage_kind,
    )
    return plan.execute(A, B_shard, C_shard, validate=False)
