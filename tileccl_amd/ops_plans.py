"""The remaining public entries of ``tileccl.ops``: the stand-alone collectives, the chained
AllGather -> GEMM -> scatter op, and the reusable plan objects of all of them.

Names, argument order, ``validate`` semantics and error texts follow
``/root/reference/tileccl/ops.py`` (collectives ``:1083-1258`` with their contracts
``:1908-2062``; GEMM + collective plans ``:305-368, 636-700, 891-1080``; the chained op
``:2189-2375``).  What a plan *does* is this package's: the collectives are the launchers of
``tileccl_amd.primitives`` (direct-write copies, fp32-accumulating reductions), the GEMM ops are
the fused launches of ``tileccl_amd.ops_collective`` and the chained op is
``ChainedAGGemmRSPattern``; the reference's host-staged ``torch.mm`` + collective pipelines have
no counterpart.  A plan only holds the shapes it was resolved for and the context.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass, fields
from typing import Any

import tileccl_amd
from tileccl_amd import ops_collective as _fused
from tileccl_amd import primitives as _prim


def _shape(t: Any) -> "tuple[int, ...]":
    return tuple(int(d) for d in t.shape)


def _context(ctx):
    return ctx if ctx is not None else tileccl_amd.current_context()


def _on_heap_device(what: str, ctx, *tensors: Any, label: str = "tensors") -> None:
    first = tensors[0]
    if len(tensors) == 2 and tensors[0].device != tensors[1].device:
        raise ValueError(f"{what} expects src/output on the same device, got {tensors[0].device} vs {tensors[1].device}")
    if str(first.device) != ctx.device:
        raise ValueError(f"{what} {label} must reside on the attached heap device {ctx.device}, got {first.device}")


def _contiguous(what: str, **named: Any) -> None:
    for name, t in named.items():
        if not t.is_contiguous():
            raise ValueError(f"{what} currently requires {name} to be contiguous")


def _still_matches(what: str, seen: dict, expected: dict) -> None:
    """``expected`` holds what a plan was resolved for (``None``: nothing to compare)."""
    for key, want in expected.items():
        if want is not None and seen[key] != want:
            raise ValueError(f"{what} {key} no longer matches the plan: {seen[key]} != {want}")


class _PlanMixin:
    def to_dict(self) -> "dict[str, object]":
        """Everything but the context object itself, for logs and docs."""
        out = {f.name: getattr(self, f.name) for f in fields(self) if f.name not in ("ctx", "contract")}
        ctx = self.ctx
        out["context"] = {"rank": ctx.rank, "world_size": ctx.world_size, "backend": ctx.backend_name, "device": ctx.device}
        if hasattr(self, "contract"):
            out["contract"] = self.contract.to_dict() if hasattr(self.contract, "to_dict") else asdict(self.contract)
        return out


# ------------------------------------------------------------------------- stand-alone collectives
def _allgather_block(src: Any, output: Any, *, ctx, expected: "dict | None" = None) -> int:
    _on_heap_device("allgather", ctx, src, output)
    _contiguous("allgather", src=src, output=output)
    _fused._require_on_heap(src, ctx=ctx, name="src")
    _fused._require_on_heap(output, ctx=ctx, name="output")
    block = int(src.numel())
    if int(output.numel()) != block * ctx.world_size:
        raise ValueError(f"allgather output.numel must equal src.numel * world_size: {output.numel()} != {block} * {ctx.world_size}")
    _still_matches("allgather", {"src shape": _shape(src), "output shape": _shape(output), "src.numel": block}, expected or {})
    return block


@dataclass(frozen=True)
class AllGatherPlan(_PlanMixin):
    ctx: Any
    input_shape: "tuple[int, ...]"
    output_shape: "tuple[int, ...]"
    block_size: int
    storage_kind: str = "symmetric"

    def validate_tensors(self, src: Any, output: Any) -> None:
        _allgather_block(src, output, ctx=self.ctx, expected={"src shape": self.input_shape, "output shape": self.output_shape,
                                                              "src.numel": self.block_size})

    def execute(self, src: Any, output: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(src, output)
        _prim.allgather(src, output, self.ctx.require_heap())
        return output


def build_allgather_plan(src: Any, output: Any, *, ctx=None, storage_kind: str = "symmetric") -> AllGatherPlan:
    ctx = _context(ctx)
    return AllGatherPlan(ctx, _shape(src), _shape(output), _allgather_block(src, output, ctx=ctx), storage_kind)


def allgather(src: Any, output: Any, *, ctx=None, storage_kind: str = "symmetric") -> Any:
    """Every rank contributes ``src`` and ends with all ranks' blocks, in rank order, in ``output``."""
    return build_allgather_plan(src, output, ctx=ctx, storage_kind=storage_kind).execute(src, output, validate=False)


def _allreduce_block(tensor: Any, *, ctx, op: str, expected: "dict | None" = None) -> int:
    if op != "sum":
        raise ValueError(f"allreduce currently supports only op='sum', got {op!r}")
    _on_heap_device("allreduce", ctx, tensor, label="tensor")
    if not tensor.is_contiguous():
        raise ValueError("allreduce currently requires the tensor to be contiguous")
    _fused._require_on_heap(tensor, ctx=ctx, name="tensor")
    _still_matches("allreduce", {"tensor shape": _shape(tensor), "tensor.numel": int(tensor.numel())}, expected or {})
    return int(tensor.numel())


@dataclass(frozen=True)
class AllReducePlan(_PlanMixin):
    ctx: Any
    tensor_shape: "tuple[int, ...]"
    block_size: int
    op: str = "sum"
    storage_kind: str = "symmetric"

    def validate_tensors(self, tensor: Any) -> None:
        _allreduce_block(tensor, ctx=self.ctx, op=self.op, expected={"tensor shape": self.tensor_shape, "tensor.numel": self.block_size})

    def execute(self, tensor: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(tensor)
        _prim.allreduce(tensor, self.ctx.require_heap(), self.op)
        return tensor


def build_allreduce_plan(tensor: Any, *, ctx=None, op: str = "sum", storage_kind: str = "symmetric") -> AllReducePlan:
    ctx = _context(ctx)
    return AllReducePlan(ctx, _shape(tensor), _allreduce_block(tensor, ctx=ctx, op=op), op, storage_kind)


def allreduce(tensor: Any, *, ctx=None, op: str = "sum", storage_kind: str = "symmetric") -> Any:
    """In place: once every rank has called, ``tensor`` holds the sum over the ranks."""
    return build_allreduce_plan(tensor, ctx=ctx, op=op, storage_kind=storage_kind).execute(tensor, validate=False)


def _reduce_scatter_block(src: Any, output: Any, *, ctx, expected: "dict | None" = None) -> int:
    _on_heap_device("reduce_scatter", ctx, src, output)
    _contiguous("reduce_scatter", src=src, output=output)
    _fused._require_on_heap(src, ctx=ctx, name="src")
    _fused._require_on_heap(output, ctx=ctx, name="output")
    block = int(output.numel())
    if int(src.numel()) != block * ctx.world_size:
        raise ValueError(f"reduce_scatter src.numel must equal output.numel * world_size: {src.numel()} != {block} * {ctx.world_size}")
    _still_matches("reduce_scatter", {"src shape": _shape(src), "output shape": _shape(output), "output.numel": block}, expected or {})
    return block


@dataclass(frozen=True)
class ReduceScatterPlan(_PlanMixin):
    ctx: Any
    input_shape: "tuple[int, ...]"
    output_shape: "tuple[int, ...]"
    block_size: int
    implementation: str = "device"
    storage_kind: str = "symmetric"

    def validate_tensors(self, src: Any, output: Any) -> None:
        _reduce_scatter_block(src, output, ctx=self.ctx, expected={"src shape": self.input_shape, "output shape": self.output_shape,
                                                                   "output.numel": self.block_size})

    def execute(self, src: Any, output: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(src, output)
        _prim.reduce_scatter(src, output, self.ctx.require_heap(), "sum", self.implementation)
        return output


def build_reduce_scatter_plan(src: Any, output: Any, *, ctx=None, implementation: str = "auto",
                              storage_kind: str = "symmetric") -> ReduceScatterPlan:
    ctx = _context(ctx)
    ctx.require_heap()
    if implementation not in {"auto", "reference", "device"}:
        raise ValueError(f"implementation must be one of {{'auto', 'reference', 'device'}}, got {implementation!r}")
    # The reference picks a host restatement for single-process heaps; here every choice runs the device kernel.
    return ReduceScatterPlan(ctx, _shape(src), _shape(output), _reduce_scatter_block(src, output, ctx=ctx), "device", storage_kind)


def reduce_scatter(src: Any, output: Any, *, ctx=None, implementation: str = "auto", storage_kind: str = "symmetric") -> Any:
    """``output`` = the sum over ranks of block ``rank`` of their ``src``."""
    plan = build_reduce_scatter_plan(src, output, ctx=ctx, implementation=implementation, storage_kind=storage_kind)
    return plan.execute(src, output, validate=False)


# ------------------------------------------------------------------------- GEMM + collective plans
_STALE = "Tensor contract no longer matches this {name}. Build a new plan for tensors with different logical shapes or dtypes."


@dataclass(frozen=True)
class GemmAllGatherPlan(_PlanMixin):
    ctx: Any
    contract: "_fused.GemmAllGatherContract"
    materialization: str = "fused_gemm_allscatter_launch"
    pack_layout: str = "rank_major_column_shards"
    storage_kind: str = "symmetric"
    variant: str = "s2"

    def validate_tensors(self, A: Any, B_shard: Any, C: Any) -> None:
        if _fused.resolve_gemm_allgather_contract(A, B_shard, C, ctx=self.ctx, storage_kind=self.storage_kind) != self.contract:
            raise ValueError(_STALE.format(name="GemmAllGatherPlan"))

    def execute(self, A: Any, B_shard: Any, C: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(A, B_shard, C)
        return _fused.gemm_allgather(A, B_shard, C, ctx=self.ctx, storage_kind=self.storage_kind, variant=self.variant)


def build_gemm_allgather_plan(A: Any, B_shard: Any, C: Any, *, ctx=None, storage_kind: str = "symmetric",
                              variant: str = "s2") -> GemmAllGatherPlan:
    ctx = _context(ctx)
    contract = _fused.resolve_gemm_allgather_contract(A, B_shard, C, ctx=ctx, storage_kind=storage_kind)
    return GemmAllGatherPlan(ctx, contract, storage_kind=storage_kind, variant=variant)


@dataclass(frozen=True)
class GemmReduceScatterPlan(_PlanMixin):
    ctx: Any
    contract: "_fused.GemmReduceScatterContract"
    implementation: str = "device"
    materialization: str = "fused_gemm_reducescatter_launch"
    pack_layout: str = "rank_major_column_shards"
    storage_kind: str = "symmetric"
    variant: str = "s2"

    def validate_tensors(self, A: Any, B: Any, C: Any) -> None:
        if _fused.resolve_gemm_reducescatter_contract(A, B, C, ctx=self.ctx, storage_kind=self.storage_kind) != self.contract:
            raise ValueError(_STALE.format(name="GemmReduceScatterPlan"))

    def execute(self, A: Any, B: Any, C: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(A, B, C)
        return _fused.gemm_reducescatter(A, B, C, ctx=self.ctx, implementation=self.implementation,
                                         storage_kind=self.storage_kind, variant=self.variant)


def build_gemm_reducescatter_plan(A: Any, B: Any, C: Any, *, ctx=None, implementation: str = "auto",
                                  storage_kind: str = "symmetric", variant: str = "s2") -> GemmReduceScatterPlan:
    ctx = _context(ctx)
    if implementation not in {"auto", "reference", "device"}:
        raise ValueError(f"implementation must be one of {{'auto', 'reference', 'device'}}, got {implementation!r}")
    contract = _fused.resolve_gemm_reducescatter_contract(A, B, C, ctx=ctx, storage_kind=storage_kind)
    return GemmReduceScatterPlan(ctx, contract, "device", storage_kind=storage_kind, variant=variant)


# ------------------------------------------------------------------------- AllGather -> GEMM -> scatter
@dataclass(frozen=True)
class AllGatherGemmReduceScatterContract:
    M: int
    K: int
    N: int
    K_shard: int
    N_shard: int
    rank: int
    world_size: int
    storage_kind: str = "symmetric"

    def to_dict(self) -> "dict[str, object]":
        return asdict(self)


def _resolve_chained_contract(input_shard: Any, W: Any, output: Any, *, ctx, storage_kind: str) -> AllGatherGemmReduceScatterContract:
    if input_shard.ndim != 2 or W.ndim != 2 or output.ndim != 2:
        raise ValueError("allgather_gemm_reducescatter expects 2-D tensors: "
                         f"got input_shard.ndim={input_shard.ndim}, W.ndim={W.ndim}, output.ndim={output.ndim}")
    (M, K_shard), (K, N), (out_M, out_N) = _shape(input_shard), _shape(W), _shape(output)
    if out_M != M:
        raise ValueError(f"output rows ({out_M}) must equal input_shard rows ({M})")
    if out_N != N:
        raise ValueError(f"output columns ({out_N}) must equal W columns ({N})")
    if K_shard * ctx.world_size != K:
        raise ValueError(f"input_shard columns ({K_shard}) * world_size ({ctx.world_size}) must equal W rows ({K})")
    n_shard = N // ctx.world_size if N % ctx.world_size == 0 else N
    return AllGatherGemmReduceScatterContract(M, K, N, K_shard, n_shard, ctx.rank, ctx.world_size, storage_kind)


@dataclass(frozen=True)
class AllGatherGemmReduceScatterPlan(_PlanMixin):
    ctx: Any
    contract: AllGatherGemmReduceScatterContract
    schedule: str = "tile_group"
    storage_kind: str = "symmetric"

    def validate_tensors(self, input_shard: Any, W: Any, output: Any) -> None:
        if _resolve_chained_contract(input_shard, W, output, ctx=self.ctx, storage_kind=self.storage_kind) != self.contract:
            raise ValueError(_STALE.format(name="AllGatherGemmReduceScatterPlan"))

    def execute(self, input_shard: Any, W: Any, output: Any, *, validate: bool = True) -> Any:
        if validate:
            self.validate_tensors(input_shard, W, output)
        from tileccl_amd.patterns.chained_ag_gemm_rs import ChainedAGGemmRSPattern

        cache = self.ctx.__dict__.setdefault("_chained_patterns", {})
        if self.schedule not in cache:
            cache[self.schedule] = ChainedAGGemmRSPattern(self.ctx, schedule=self.schedule)
        return cache[self.schedule].execute(input_shard, W, output)


def build_allgather_gemm_reducescatter_plan(input_shard: Any, W: Any, output: Any, *, ctx=None, storage_kind: str = "symmetric",
                                            schedule: str = "tile_group") -> AllGatherGemmReduceScatterPlan:
    ctx = _context(ctx)
    ctx.require_heap()
    contract = _resolve_chained_contract(input_shard, W, output, ctx=ctx, storage_kind=storage_kind)
    return AllGatherGemmReduceScatterPlan(ctx, contract, schedule, storage_kind)


def allgather_gemm_reducescatter(input_shard: Any, W: Any, output: Any, *, ctx=None, storage_kind: str = "symmetric") -> Any:
    """Gather the ranks' column shards of the input, multiply by ``W``, write the product to every rank's ``output``."""
    plan = build_allgather_gemm_reducescatter_plan(input_shard, W, output, ctx=ctx, storage_kind=storage_kind)
    return plan.execute(input_shard, W, output, validate=False)
