"""Shape / layout contract of a GEMM + all-scatter call, resolved once on the host.

Mirrors ``/root/reference/tileccl/patterns/contracts.py``: ``PatternTensorSpec`` (:19-44),
``PatternExecutionSpec`` (:47-90) and ``resolve_pattern_execution`` (:93-230) with its
layout inference (:233-326).  The four ``scatter_*`` integers are what the kernels consume:
columns ``[scatter_src_col_offset, +scatter_cols)`` of the local ``C`` are written to every
peer at ``row * scatter_dst_leading_dim + scatter_dst_col_offset + (col - src_offset)``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

TensorLayout = Literal["full", "shard"]

_LAYOUTS = ("full", "shard")


@dataclass(frozen=True, slots=True)
class PatternTensorSpec:
    """Logical (full) versus physical (local) shape of one operand."""

    full_shape: tuple[int, int]
    local_shape: tuple[int, int]
    rank: int
    world_size: int
    layout_kind: TensorLayout
    storage_kind: str = "symmetric"

    @property
    def cols(self) -> int:
        return self.local_shape[1]

    def to_dict(self) -> dict[str, object]:
        return {
            "full_shape": list(self.full_shape),
            "local_shape": list(self.local_shape),
            "rank": self.rank,
            "world_size": self.world_size,
            "layout_kind": self.layout_kind,
            "storage_kind": self.storage_kind,
        }


@dataclass(frozen=True, slots=True)
class PatternExecutionSpec:
    """Everything a pattern needs to run one call without re-inspecting tensor shapes."""

    M: int
    K: int
    full_N: int
    local_N: int
    rank: int
    world_size: int
    rhs: PatternTensorSpec
    output: PatternTensorSpec
    scatter_src_col_offset: int
    scatter_cols: int
    scatter_dst_leading_dim: int
    scatter_dst_col_offset: int

    @property
    def rhs_layout(self) -> TensorLayout:
        return self.rhs.layout_kind

    @property
    def output_layout(self) -> TensorLayout:
        return self.output.layout_kind

    def to_dict(self) -> dict[str, object]:
        return {
            "M": self.M,
            "K": self.K,
            "full_N": self.full_N,
            "local_N": self.local_N,
            "rank": self.rank,
            "world_size": self.world_size,
            "rhs": self.rhs.to_dict(),
            "output": self.output.to_dict(),
            "scatter": {
                "src_col_offset": self.scatter_src_col_offset,
                "cols": self.scatter_cols,
                "dst_leading_dim": self.scatter_dst_leading_dim,
                "dst_col_offset": self.scatter_dst_col_offset,
            },
        }


def _checked_layout(layout: str | None, name: str) -> TensorLayout | None:
    if layout is not None and layout not in _LAYOUTS:
        raise ValueError(f"{name} must be one of {sorted(_LAYOUTS)}, got {layout!r}")
    return layout  # type: ignore[return-value]


def _implied_full_N(cols: int, layout: TensorLayout, world_size: int) -> int:
    """Full width a tensor of ``cols`` columns implies under ``layout``."""
    return cols if layout == "full" or world_size == 1 else cols * world_size


def _infer_full_N(b_cols, c_cols, world_size, full_N, b_layout, c_layout) -> int:
    if full_N is not None:
        return int(full_N)
    implied = {
        _implied_full_N(cols, layout, world_size)
        for cols, layout in ((b_cols, b_layout), (c_cols, c_layout))
        if layout is not None
    }
    if len(implied) > 1:
        raise ValueError(f"Provided layout hints disagree on full_N: resolved candidates={sorted(implied)}")
    if implied:
        return implied.pop()
    if world_size == 1:
        return max(b_cols, c_cols)
    wide, narrow = max(b_cols, c_cols), min(b_cols, c_cols)
    if wide != narrow and wide == narrow * world_size:
        return wide
    raise ValueError(
        "Ambiguous multi-rank pattern contract. Pass full_N together with "
        "explicit b_layout/c_layout, or use tileccl.ops.gemm_allscatter(...)."
    )


def _infer_layout(cols, full_N, shard_N, explicit, name, world_size) -> TensorLayout:
    if explicit is not None:
        want = full_N if explicit == "full" else shard_N
        if cols != want:
            raise ValueError(f"{name} layout={explicit!r} expects {want} columns, got {cols}")
        return explicit
    if world_size == 1:
        if cols != full_N:
            raise ValueError(f"{name} expects {full_N} columns, got {cols}")
        return "full"
    fits = [kind for kind, width in (("full", full_N), ("shard", shard_N)) if cols == width]
    if len(fits) == 1:
        return fits[0]  # type: ignore[return-value]
    if not fits:
        raise ValueError(f"Cannot infer {name} layout from cols={cols}, full_N={full_N}, shard_N={shard_N}")
    raise ValueError(f"Ambiguous {name} layout for cols={cols}. Pass explicit {name.lower()}_layout.")


def resolve_pattern_execution(
    A,
    B,
    C,
    *,
    rank: int,
    world_size: int,
    full_N: int | None = None,
    b_layout: TensorLayout | None = None,
    c_layout: TensorLayout | None = None,
    storage_kind: str = "symmetric",
) -> PatternExecutionSpec:
    """Validate ``A (M,K)``, ``B (K,N*)``, ``C (M,N*)`` and derive the scatter placement.

    Multi-rank calls must be full/full (``N* = N``) or shard/shard (``N* = N / world_size``,
    with ``full_N`` given or implied); mixed layouts are rejected here and handled by the
    host wrapper in ``tileccl_amd.ops``.
    """
    if A.ndim != 2 or B.ndim != 2 or C.ndim != 2:
        raise ValueError(
            f"Pattern tensors must all be 2-D: got A.ndim={A.ndim}, B.ndim={B.ndim}, C.ndim={C.ndim}"
        )
    if world_size < 1:
        raise ValueError(f"world_size must be >= 1, got {world_size}")
    if not 0 <= rank < world_size:
        raise ValueError(f"rank={rank} out of range for world_size={world_size}")

    M, K = int(A.shape[0]), int(A.shape[1])
    b_rows, b_cols = int(B.shape[0]), int(B.shape[1])
    c_rows, c_cols = int(C.shape[0]), int(C.shape[1])
    if b_rows != K:
        raise ValueError(f"B.shape[0] must equal A.shape[1]: got {b_rows} vs {K}")
    if c_rows != M:
        raise ValueError(f"C.shape[0] must equal A.shape[0]: got {c_rows} vs {M}")

    b_hint = _checked_layout(b_layout, "b_layout")
    c_hint = _checked_layout(c_layout, "c_layout")
    N = _infer_full_N(b_cols, c_cols, world_size, full_N, b_hint, c_hint)
    if N <= 0:
        raise ValueError(f"full_N must be positive, got {N}")
    if N % world_size != 0:
        raise ValueError(f"full_N must be divisible by world_size: {N} % {world_size} != 0")

    shard_N = N if world_size == 1 else N // world_size
    b_kind = _infer_layout(b_cols, N, shard_N, b_hint, "B", world_size)
    c_kind = _infer_layout(c_cols, N, shard_N, c_hint, "C", world_size)
    if world_size > 1 and b_kind != c_kind:
        raise ValueError(
            "Mixed multi-rank layouts are not implemented yet: "
            f"B uses {b_kind!r}, C uses {c_kind!r}. "
            "Use matching full/full or shard/shard tensors, or call a "
            "higher-level host wrapper that materializes the intermediate layout."
        )

    local_N = N if b_kind == "full" else shard_N
    if b_cols != local_N:
        raise ValueError(f"B shape/layout mismatch: layout={b_kind!r} expects {local_N} columns, got {b_cols}")
    if c_cols != local_N:
        raise ValueError(f"C shape/layout mismatch: layout={c_kind!r} expects {local_N} columns, got {c_cols}")

    def spec(rows: int, cols: int, kind: TensorLayout) -> PatternTensorSpec:
        return PatternTensorSpec((rows, N), (rows, cols), rank, world_size, kind, storage_kind)

    if c_kind == "full":
        # Each rank contributes its own N/world_size column block of the full output.
        lone = world_size == 1
        cols, src, dst, ld = (N, 0, 0, N) if lone else (shard_N, rank * shard_N, rank * shard_N, N)
    else:
        cols, src, dst, ld = c_cols, 0, 0, c_cols

    return PatternExecutionSpec(
        M=M,
        K=K,
        full_N=N,
        local_N=b_cols,
        rank=rank,
        world_size=world_size,
        rhs=spec(K, b_cols, b_kind),
        output=spec(M, c_cols, c_kind),
        scatter_src_col_offset=src,
        scatter_cols=cols,
        scatter_dst_leading_dim=ld,
        scatter_dst_col_offset=dst,
    )
