"""``gemm_allgather`` and ``gemm_reducescatter`` with column shards, on the HIP kernels.

The reference keeps these two ops "intentionally conservative": a local ``torch.mm`` into a
heap workspace, then the stand-alone collective (``/root/reference/tileccl/ops.py:891-1080``,
contracts ``:1406-1549``).  Here the same contracts run on this package's kernels:

* ``gemm_allgather(A, B_shard, C)``: the GEMM writes this rank's column block of the full
  ``C`` in place (``ldc = N``) and that block is placed at the same columns of every peer's
  ``C``: exactly the all-scatter launch, in any of its three variants (S2 by default).
* ``gemm_reducescatter(A, B, C_shard)``: the partial ``A @ B`` is produced in the
  rank-major column-shard layout of the reference (``(world, M, N/world)``: block ``q`` holds
  the columns rank ``q`` owns), which turns the column reduce-scatter into the row
  reduce-scatter of ``tile_reduce_scatter`` (primitives/collectives.py:730-783); the
  reduction accumulates in fp32 and rounds once.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any

import torch

import tileccl_amd
from tileccl_amd import _launch, _lib
from tileccl_amd.patterns import BulkSyncPattern, Pattern, TileGroupPattern, WGSpecializedPattern
from tileccl_amd.patterns.contracts import PatternExecutionSpec, PatternTensorSpec

_VARIANT_PATTERNS = {"s0": BulkSyncPattern, "s1": WGSpecializedPattern, "s2": TileGroupPattern}


def _require_on_heap(t: Any, *, ctx, name: str) -> None:
    if not ctx.require_heap().owns_tensor(t):
        raise ValueError(f"{name} must reside in the attached symmetric heap for the current public contract.")


def _common_checks(op: str, names: tuple[str, str, str], A: Any, B: Any, Cx: Any, *, ctx, collective: str) -> None:
    a, b, c = names
    ctx.require_heap()
    if A.ndim != 2 or B.ndim != 2 or Cx.ndim != 2:
        raise ValueError(f"{op} expects 2-D tensors: got {a}.ndim={A.ndim}, {b}.ndim={B.ndim}, {c}.ndim={Cx.ndim}")
    if any(str(t.device) != ctx.device for t in (A, B, Cx)):
        raise ValueError(
            f"{op} tensors must all reside on the context device "
            f"{ctx.device}, got {a}={A.device}, {b}={B.device}, {c}={Cx.device}"
        )
    if not Cx.is_contiguous():
        raise ValueError(
            f"{op} currently requires C to be contiguous so the {collective} output contract stays well-defined."
        )
    _require_on_heap(Cx, ctx=ctx, name="C")
    if A.dtype != B.dtype or B.dtype != Cx.dtype:
        listed = ", ".join(n for n in names[:-1]) + f", and {names[-1]}"
        raise ValueError(
            f"{op} currently requires {listed} to share one dtype: got {a}={A.dtype}, {b}={B.dtype}, {c}={Cx.dtype}"
        )
    if not (A.is_floating_point() and B.is_floating_point() and Cx.is_floating_point()):
        raise ValueError(f"{op} currently requires floating-point tensors.")


@dataclass(frozen=True, slots=True)
class GemmAllGatherContract:
    """Reference ``GemmAllGatherContract`` (ops.py:283-306)."""

    M: int
    K: int
    full_N: int
    shard_cols: int
    rank: int
    world_size: int
    storage_kind: str = "symmetric"

    def to_dict(self) -> dict[str, object]:
        return {f: getattr(self, f) for f in self.__slots__}


@dataclass(frozen=True, slots=True)
class GemmReduceScatterContract:
    """Reference ``GemmReduceScatterContract`` (ops.py:497-520)."""

    M: int
    K: int
    full_N: int
    output_cols: int
    rank: int
    world_size: int
    storage_kind: str = "symmetric"

    def to_dict(self) -> dict[str, object]:
        return {f: getattr(self, f) for f in self.__slots__}


def resolve_gemm_allgather_contract(A: Any, B_shard: Any, Cx: Any, *, ctx, storage_kind: str = "symmetric") -> GemmAllGatherContract:
    """Validation of ops.py:1477-1549, same messages."""
    _common_checks("gemm_allgather", ("A", "B_shard", "C"), A, B_shard, Cx, ctx=ctx, collective="allgather")
    M, K = int(A.shape[0]), int(A.shape[1])
    b_k, shard_cols = int(B_shard.shape[0]), int(B_shard.shape[1])
    c_m, full_N = int(Cx.shape[0]), int(Cx.shape[1])
    if b_k != K:
        raise ValueError(f"B_shard.shape[0] must equal A.shape[1]: got {b_k} vs {K}")
    if c_m != M:
        raise ValueError(f"C.shape[0] must equal A.shape[0]: got {c_m} vs {M}")
    if full_N <= 0:
        raise ValueError(f"C.shape[1] must be positive, got {full_N}")
    ws = ctx.world_size
    if full_N % ws != 0:
        raise ValueError(f"gemm_allgather requires C.shape[1] to be divisible by world_size: {full_N} % {ws} != 0")
    expected = full_N if ws == 1 else full_N // ws
    if shard_cols != expected:
        raise ValueError(
            f"gemm_allgather RHS shard columns must match the rank-local shard width: expected {expected}, got {shard_cols}"
        )
    return GemmAllGatherContract(M, K, full_N, shard_cols, ctx.rank, ws, storage_kind)


def resolve_gemm_reducescatter_contract(A: Any, B: Any, Cx: Any, *, ctx, storage_kind: str = "symmetric") -> GemmReduceScatterContract:
    """Validation of ops.py:1406-1474, same messages."""
    _common_checks("gemm_reducescatter", ("A", "B", "C"), A, B, Cx, ctx=ctx, collective="reduce_scatter")
    M, K = int(A.shape[0]), int(A.shape[1])
    b_k, full_N = int(B.shape[0]), int(B.shape[1])
    c_m, c_cols = int(Cx.shape[0]), int(Cx.shape[1])
    if b_k != K:
        raise ValueError(f"B.shape[0] must equal A.shape[1]: got {b_k} vs {K}")
    if c_m != M:
        raise ValueError(f"C.shape[0] must equal A.shape[0]: got {c_m} vs {M}")
    if full_N <= 0:
        raise ValueError(f"B.shape[1] must be positive, got {full_N}")
    ws = ctx.world_size
    if full_N % ws != 0:
        raise ValueError(f"gemm_reducescatter requires B.shape[1] to be divisible by world_size: {full_N} % {ws} != 0")
    expected = full_N if ws == 1 else full_N // ws
    if c_cols != expected:
        raise ValueError(
            f"gemm_reducescatter output columns must match the rank-local shard width: expected {expected}, got {c_cols}"
        )
    return GemmReduceScatterContract(M, K, full_N, c_cols, ctx.rank, ws, storage_kind)


def _pattern_for(ctx, variant: str | Pattern) -> Pattern:
    if isinstance(variant, Pattern):
        return variant
    if variant not in _VARIANT_PATTERNS:
        raise ValueError(f"unknown variant {variant!r}; expected one of {sorted(_VARIANT_PATTERNS)}")
    cache = ctx.__dict__.setdefault("_collective_patterns", {})
    if variant not in cache:
        cache[variant] = _VARIANT_PATTERNS[variant](ctx)
    return cache[variant]


def gemm_allgather(A: Any, B_shard: Any, Cx: Any, *, ctx=None, storage_kind: str = "symmetric",
                   variant: str | Pattern = "s2") -> Any:
    """``C[:, rank's columns] = A @ B_shard`` on every rank, each block landing in every rank's ``C``.

    ``variant`` (not in the reference signature) picks the schedule: ``"s0"`` bulk, ``"s1"``
    tile by tile, ``"s2"`` TileGroup (default), or a ``Pattern`` instance.
    """
    ctx = ctx if ctx is not None else tileccl_amd.current_context()
    k = resolve_gemm_allgather_contract(A, B_shard, Cx, ctx=ctx, storage_kind=storage_kind)
    lo = k.rank * k.shard_cols if k.world_size > 1 else 0
    block = Cx[:, lo:lo + k.shard_cols]  # the GEMM's output: this rank's columns of the full C
    shape = (k.M, k.full_N)
    spec = PatternExecutionSpec(
        M=k.M, K=k.K, full_N=k.full_N, local_N=k.shard_cols, rank=k.rank, world_size=k.world_size,
        rhs=PatternTensorSpec((k.K, k.full_N), (k.K, k.shard_cols), k.rank, k.world_size, "shard", storage_kind),
        output=PatternTensorSpec(shape, shape, k.rank, k.world_size, "full", storage_kind),
        # relative to the block: all of its columns go to the same columns of the peer's C
        scatter_src_col_offset=0, scatter_cols=k.shard_cols, scatter_dst_leading_dim=k.full_N, scatter_dst_col_offset=0,
    )
    pattern = _pattern_for(ctx, variant)
    pattern.execute(A, B_shard, block, spec=spec)
    return Cx


def _reduce_scatter_words(ctx, world: int, M: int, cols: int):
    """Signal words and TileGroup plan of the fused column-shard reduce-scatter, kept per shape
    on the context.  Every rank allocates them in the same order, so a peer's words sit at the
    same offset of its slice."""
    from tileccl_amd.v2.tile_group import build_tile_group_plan

    cache = ctx.__dict__.setdefault("_reduce_scatter_words", {})
    key = (world, M, cols)
    if key not in cache:
        plan = build_tile_group_plan(world * M, cols, 128 * 128 * 4, row_split_boundaries=[M * q for q in range(1, world)])
        heap = ctx.require_heap()
        words = {name: heap.allocate_tensor((n,), torch.int32) for name, n in
                 (("counter", plan.n_groups), ("barrier", plan.n_groups), ("locks", int(plan.group_table.numel())))}
        for t in words.values():
            t.zero_()
        cache[key] = _launch.SyncWords(plan=_launch.DevicePlan.upload(plan), host_plan=plan, **words)
    return cache[key]


def gemm_reducescatter(A: Any, B: Any, Cx: Any, *, ctx=None, implementation: str = "auto",
                       storage_kind: str = "symmetric", emulate_peer: bool = False, variant: str = "s2",
                       own_rows_in_registers: bool = True, peers_resident: bool = True) -> Any:
    """``C = (sum over ranks of A_rank @ B)[:, this rank's columns]``.

    The partial products live in the context workspace ``"gemm_reducescatter.partial"`` of
    shape ``(world, M, N/world)``, fp32, at the same offset of every rank's slice; block
    ``q`` is ``A @ B[:, q's columns]`` (the reference's rank-major column-shard layout,
    ops.py:315,646).  Stacked, the blocks are the row shards of a ``(world*M, N/world)``
    matrix, so the operation is one launch of the fused GEMM -> ReduceScatter kernel: the
    GEMM produces row block ``q`` from ``B``'s column block ``q``, block ``rank`` is reduced
    with the peers' partials as its tiles finish, and (``own_rows_in_registers``, the default)
    that block never leaves the accumulators as a partial, so its part of the workspace is not
    written.  ``variant`` picks the schedule (``"s0"`` bulk, ``"s1"`` tile by tile, ``"s2"``
    TileGroup).  ``emulate_peer`` (single-GPU emulation) also writes the other ranks' outputs
    into their slices.

    Precondition (``peers_resident=True``, the default): every other rank has already produced
    its partials FOR THESE INPUTS -- its call has run to completion -- before this rank's call
    is issued.  The launch then does not look at the peers' signal words at all and sums
    whatever their workspaces hold; the first call on a fresh context, or a call made after
    only some ranks have run with new inputs, returns sums over stale or zero partials (its own
    block of the workspace is what the ranks after it read).  That is the arrangement of this
    single-process build, whose ranks run one after another, and the reason the default is on:
    all ranks run once to produce, then once more to reduce.  With ``peers_resident=False`` the
    launch waits (bounded) for each peer's words to reach this launch's number and raises the
    fault word if a producer is missing: the mode for ranks that really run side by side and
    have made the same number of calls.
    ``implementation`` is accepted for signature parity; there is one implementation here.
    When ``M`` is not a multiple of the 128-row plan tile, one GEMM per column block and the
    bulk reduction run instead.
    """
    if implementation not in ("auto", "device", "hip"):
        raise ValueError(f"unsupported gemm_reducescatter implementation {implementation!r}")
    if variant not in _launch.VARIANTS:
        raise ValueError(f"unknown variant {variant!r}; expected one of {sorted(_launch.VARIANTS)}")
    ctx = ctx if ctx is not None else tileccl_amd.current_context()
    k = resolve_gemm_reducescatter_contract(A, B, Cx, ctx=ctx, storage_kind=storage_kind)
    lib = _lib.load()
    stream = _launch.stream_ptr()
    if k.world_size == 1:
        _lib.check(lib.tccl_gemm(C.byref(_launch.gemm_desc(A, B, Cx)), stream), "tccl_gemm")
        return Cx
    partial = ctx.workspace("gemm_reducescatter.partial", k.world_size, k.M, k.output_cols, dtype=torch.float32)
    tall = partial.view(k.world_size * k.M, k.output_cols)  # row block q = the shard rank q owns
    view = _launch.heap_view(ctx.heap_bases, k.rank, k.world_size)
    transport = _launch.transport_desc(_lib.DIR_PULL, 16384, 16384, 0)
    if k.M % 128 == 0:
        words = _reduce_scatter_words(ctx, k.world_size, k.M, k.output_cols)
        gemm = _launch.gemm_desc(A, B, tall, column_shards=k.world_size,
                                 flags=_lib.GEMM_OWN_ROWS_IN_REGISTERS if own_rows_in_registers else 0)
        if variant != "s0":
            words.next_epoch(variant)
        sync = words.desc(variant)
        mode = (_lib.RS_PEERS_RESIDENT if peers_resident else 0) | (_lib.RS_EMULATE_PEERS if emulate_peer else 0)
        rc = lib.tccl_gemm_reducescatter(
            C.byref(gemm), _launch.ptr(Cx), _launch.dtype_code(Cx.dtype), int(Cx.stride(0)), C.byref(view), C.byref(sync),
            C.byref(transport), mode, _launch.VARIANTS[variant], stream,
        )
        _lib.check(rc, f"tccl_gemm_reducescatter[{variant}]")
        ctx.__dict__["_reduce_scatter_last_words"] = words
        return Cx
    for q in range(k.world_size):
        cols = B[:, q * k.output_cols:(q + 1) * k.output_cols]
        _lib.check(lib.tccl_gemm(C.byref(_launch.gemm_desc(A, cols, partial[q])), stream), "tccl_gemm")
    rc = lib.tccl_reduce_rows(
        _launch.ptr(tall), _launch.dtype_code(tall.dtype), int(tall.stride(0)), _launch.ptr(Cx), _launch.dtype_code(Cx.dtype),
        int(Cx.stride(0)), int(tall.shape[0]), int(tall.shape[1]), C.byref(view), C.byref(transport), int(emulate_peer), stream,
    )
    _lib.check(rc, "tccl_reduce_rows")
    return Cx
