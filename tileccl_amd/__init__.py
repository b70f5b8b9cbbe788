"""tileccl_amd -- the fused GEMM + collective hot path of TileCCL, rebuilt for MI355X.

The host surface follows ``/root/reference/tileccl/__init__.py``: ``init`` (:251-318),
``init_local`` (:321-356), ``TileCCLContext`` (:36-222) with the heap-backed tensor
factories ``empty / zeros / randn / workspace`` (:141-178), ``heap_bases`` (:78-85),
``barrier`` (:122-127), and the process-global context behind ``current_context`` (:228-237).
Behind it, device work is done by hand-written HIP kernels in ``libtileccl_hip.so``.

One GPU only: ranks of a world larger than one are emulated as slices of a single device
allocation, so every context reports device ``cuda:0``.
"""

from __future__ import annotations

__version__ = "0.1.0"

import importlib
import os
from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Optional

if TYPE_CHECKING:
    import torch

    from tileccl_amd.backends.hip import HIPBackend
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

_NO_HEAP = (
    "No SymmetricHeap is attached to this TileCCLContext. "
    "Pass heap=... or heap_size=... to tileccl.init(), call "
    "tileccl.init_local(...), or attach an existing heap via "
    "ctx.attach_heap(heap)."
)


def _normalize_shape(size: tuple[object, ...]) -> tuple[int, ...]:
    """``*size`` or a single tuple/list -> tuple of non-negative ints (reference :432-444)."""
    dims = size[0] if len(size) == 1 and isinstance(size[0], (tuple, list)) else size
    try:
        shape = tuple(int(d) for d in dims)
    except TypeError as exc:
        raise TypeError(f"Invalid shape specification: {size!r}") from exc
    if any(d < 0 for d in shape):
        raise ValueError(f"Shape dimensions must be non-negative, got {shape}")
    return shape


@dataclass
class TileCCLContext:
    """Rank, world size, device, backend and (optionally) the symmetric heap of one rank."""

    rank: int
    world_size: int
    device: str
    backend_name: str
    backend: "HIPBackend" = field(repr=False)
    topology: Optional[object] = field(default=None, repr=False)
    heap: Optional["SymmetricHeap"] = field(default=None, repr=False)
    _workspace_cache: dict = field(default_factory=dict, init=False, repr=False)

    # -- heap plumbing ---------------------------------------------------------------
    @property
    def has_heap(self) -> bool:
        return self.heap is not None

    def require_heap(self) -> "SymmetricHeap":
        if self.heap is None:
            raise RuntimeError(_NO_HEAP)
        return self.heap

    @property
    def heap_bases(self) -> "torch.Tensor":
        return self.require_heap().get_heap_bases()

    def attach_heap(self, heap: "SymmetricHeap") -> "TileCCLContext":
        if heap.rank != self.rank:
            raise ValueError(f"Heap rank {heap.rank} does not match context rank {self.rank}")
        if heap.world_size != self.world_size:
            raise ValueError(
                "Heap world_size does not match context world_size: "
                f"{heap.world_size} != {self.world_size}"
            )
        heap_backend = getattr(heap, "_backend_name", self.backend_name)
        if heap_backend != self.backend_name:
            raise ValueError(
                f"Heap backend does not match context backend: {heap_backend!r} != {self.backend_name!r}"
            )
        self.heap = heap
        self._workspace_cache.clear()
        return self

    def barrier(self) -> None:
        if self.heap is not None:
            self.heap.barrier()
        else:
            self.backend.synchronize()

    # -- tensor factories ------------------------------------------------------------
    def allocate_tensor(self, shape: tuple[int, ...], dtype: "torch.dtype") -> "torch.Tensor":
        return self.require_heap().allocate_tensor(shape, dtype)

    def is_symmetric(self, tensor: "torch.Tensor") -> bool:
        return self.require_heap().is_symmetric(tensor)

    def as_symmetric(self, tensor: "torch.Tensor") -> "torch.Tensor":
        return self.require_heap().as_symmetric(tensor)

    def empty(self, *size: int, dtype: "torch.dtype") -> "torch.Tensor":
        return self.allocate_tensor(_normalize_shape(size), dtype)

    def zeros(self, *size: int, dtype: "torch.dtype") -> "torch.Tensor":
        t = self.allocate_tensor(_normalize_shape(size), dtype)
        t.zero_()
        return t

    def randn(self, *size: int, dtype: "torch.dtype") -> "torch.Tensor":
        """Heap tensor filled from the device's normal generator."""
        t = self.allocate_tensor(_normalize_shape(size), dtype)
        t.normal_()
        return t

    def workspace(self, name: str, *size: int, dtype: "torch.dtype", zero: bool = False) -> "torch.Tensor":
        """Heap scratch tensor reused across calls, keyed by ``(name, shape, dtype)``."""
        shape = _normalize_shape(size)
        key = (name, shape, str(dtype))
        t = self._workspace_cache.get(key)
        if t is None:
            t = self._workspace_cache[key] = self.allocate_tensor(shape, dtype)
        if zero:
            t.zero_()
        return t

    # -- pattern choice and support report (reference __init__.py:180-206) ---------------
    def auto_select_pattern(self, op: str, M: int, N: int, K: int, *, hw_info: object | None = None):
        """The pattern ``auto_select`` picks for this problem, bound to this context."""
        from tileccl_amd.patterns.auto_select import auto_select

        return auto_select(op, M=M, N=N, K=K, world_size=self.world_size, hw_info=hw_info, ctx=self)

    def support_matrix(self):
        from tileccl_amd.support import describe_runtime_support

        return describe_runtime_support(self)

    # -- introspection ---------------------------------------------------------------
    def heap_metadata(self) -> dict[str, object]:
        return self.require_heap().metadata()

    def runtime_metadata(self) -> dict[str, object]:
        return {
            "rank": self.rank,
            "world_size": self.world_size,
            "device": self.device,
            "backend": self.backend_name,
            "has_heap": self.has_heap,
            "heap": self.heap_metadata() if self.has_heap else None,
        }


_ctx: Optional[TileCCLContext] = None


def _get_ctx() -> TileCCLContext:
    if _ctx is None:
        raise RuntimeError("TileCCL has not been initialised. Call tileccl.init() first.")
    return _ctx


def _detect_backend() -> str:
    """Only HIP exists in this build; anything else is an installation problem."""
    try:
        import torch

        if getattr(torch.version, "hip", None) is not None:
            return "hip"
    except ImportError:
        pass
    raise RuntimeError(
        "Cannot auto-detect GPU backend. tileccl_amd needs PyTorch built for ROCm (torch.version.hip)."
    )


def _checked_backend(backend: str) -> str:
    if backend == "auto":
        backend = _detect_backend()
    if backend not in ("cuda", "hip"):
        raise ValueError(f"Unsupported backend: {backend!r}. Use 'cuda', 'hip', or 'auto'.")
    if backend == "cuda":
        raise RuntimeError("Backend 'cuda' is not available: this build targets HIP (MI355X) only.")
    return backend


def _env_or_dist(var: str, dist_getter: str, default: int) -> int:
    value = os.environ.get(var)
    if value is not None:
        return int(value)
    try:
        import torch.distributed as dist

        if dist.is_initialized():
            return getattr(dist, dist_getter)()
    except Exception:
        pass
    return default


def _build_context(*, backend_name: str, rank: int, world_size: int, force_backend: bool = False) -> TileCCLContext:
    from tileccl_amd.backends import get_backend

    return TileCCLContext(
        rank=rank,
        world_size=world_size,
        device="cuda:0",  # emulated ranks share the one GPU
        backend_name=backend_name,
        backend=get_backend(backend_name, force=force_backend),
    )


def _create_heap_for_context(ctx: TileCCLContext, heap_size: int) -> "SymmetricHeap":
    if heap_size <= 0:
        raise ValueError(f"heap_size must be positive, got {heap_size}")
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    if ctx.world_size == 1:
        return SymmetricHeap(size=heap_size, rank=ctx.rank, world_size=1, backend=ctx.backend_name)
    raise RuntimeError(
        "Automatic heap creation for world_size > 1 is not possible from a single rank on one GPU. "
        "For single-process multi-rank emulation use tileccl.init_local(...); "
        "otherwise create the heaps with SymmetricHeap.create_all(...) and attach one via heap=..."
    )


def init(
    backend: str = "auto",
    rank: int | None = None,
    world_size: int | None = None,
    *,
    heap: "SymmetricHeap | None" = None,
    heap_size: int | None = None,
    force_backend: bool = False,
) -> TileCCLContext:
    """Create the process-global context; attach ``heap`` or a new heap of ``heap_size`` bytes."""
    global _ctx
    backend = _checked_backend(backend)
    if rank is None:
        rank = _env_or_dist("RANK", "get_rank", 0)
    if world_size is None:
        world_size = _env_or_dist("WORLD_SIZE", "get_world_size", 1)
    if heap is not None and heap_size is not None:
        raise ValueError("Pass at most one of heap=... and heap_size=...")
    ctx = _build_context(backend_name=backend, rank=rank, world_size=world_size, force_backend=force_backend)
    if heap is not None:
        ctx.attach_heap(heap)
    elif heap_size is not None:
        ctx.attach_heap(_create_heap_for_context(ctx, heap_size))
    _ctx = ctx
    return ctx


def init_local(
    world_size: int, heap_size: int, *, backend: str = "auto", force_backend: bool = False
) -> list[TileCCLContext]:
    """One context per emulated rank, their heaps being slices of one device arena."""
    if world_size < 1:
        raise ValueError(f"world_size must be >= 1, got {world_size}")
    if heap_size <= 0:
        raise ValueError(f"heap_size must be positive, got {heap_size}")
    backend = _checked_backend(backend)
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    heaps = SymmetricHeap.create_all(size=heap_size, world_size=world_size, backend=backend)
    contexts = []
    for rank, heap in enumerate(heaps):
        ctx = _build_context(
            backend_name=backend, rank=rank, world_size=world_size, force_backend=force_backend and rank == 0
        )
        contexts.append(ctx.attach_heap(heap))
    return contexts


def describe_runtime_support(ctx: "TileCCLContext | None" = None):
    """The structured support matrix of this build (reference tileccl/__init__.py:240-244)."""
    from tileccl_amd.support import describe_runtime_support as _describe

    return _describe(ctx)


def get_rank() -> int:
    return _get_ctx().rank


def get_world_size() -> int:
    return _get_ctx().world_size


def current_context() -> TileCCLContext:
    return _get_ctx()


def install_aliases(force: bool = False) -> None:
    """Make the reference's import names (``tileccl``, ``tileccl.ops``, ``tileccl_v2`` ...) resolve to this package."""
    from tileccl_amd import aliases

    aliases.install_aliases(force=force)


_LAZY = {"ops": "tileccl_amd.ops", "patterns": "tileccl_amd.patterns", "v2": "tileccl_amd.v2"}


def __getattr__(name: str):
    if name in _LAZY:
        return importlib.import_module(_LAZY[name])
    if name in ("SymmetricHeap", "Tile"):
        from tileccl_amd.memory.symmetric_heap import SymmetricHeap

        return SymmetricHeap
    raise AttributeError(f"module 'tileccl_amd' has no attribute {name!r}")


__all__ = [
    "__version__",
    "init",
    "init_local",
    "get_rank",
    "get_world_size",
    "current_context",
    "describe_runtime_support",
    "install_aliases",
    "TileCCLContext",
    "Tile",
    "SymmetricHeap",
    "patterns",
    "ops",
    "v2",
]
