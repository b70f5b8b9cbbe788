"""Symmetric heap with the reference's v1 surface, on one GPU.

Public surface mirrored from ``/root/reference/tileccl/memory/symmetric_heap.py``:
``SymmetricHeap(size, rank, world_size)`` (:145), ``create_all`` (:239), ``allocate_tensor``
(:892), ``get_heap_bases`` (:929), ``local_base/size/rank/world_size/bytes_allocated/
bytes_free/mode/transport_strategy`` (:940-978), ``get_peer_buffer`` (:980), ``owns_tensor/
is_symmetric/import_external_tensor/as_symmetric`` (:1215-1229), ``translate/get_offset``
(:1233-1253), ``barrier`` (:1257), ``cleanup`` (:1266, idempotent), context-manager use.

What differs by design: all ranks are slices of one device allocation (``Arena``), so
``mode`` is always ``"single_process"``, the transport is ``"local_only"`` (one rank) or
``"peer_access"`` (several), every heap reports device ``cuda:0``, and a lone heap with
``world_size > 1`` cannot be built -- a second process or GPU does not exist here; use
``create_all`` / ``tileccl_amd.init_local``.
"""

from __future__ import annotations

import logging
import math

import torch

from tileccl_amd.memory.arena import DEVICE, Arena
from tileccl_amd.memory.bump import BumpAllocator

logger = logging.getLogger(__name__)


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class SymmetricHeap:
    """Rank ``rank``'s slice of the arena plus a bump allocator over it."""

    _BUMP_POLICY = "align_start"

    def __init__(
        self,
        size: int,
        rank: int,
        world_size: int,
        backend: str = "auto",
        *,
        allocator_type: str = "torch_bump",
        _arena: Arena | None = None,
    ) -> None:
        self._cleaned_up = True  # until construction succeeds, cleanup() is a no-op
        if size <= 0:
            raise ValueError(f"Heap size must be positive, got {size}")
        if rank < 0 or rank >= world_size:
            raise ValueError(f"rank={rank} out of range for world_size={world_size}")
        if world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {world_size}")
        if backend not in ("auto", "hip"):
            raise ValueError(f"Unsupported backend: {backend!r}. This build is HIP-only.")
        if allocator_type != "torch_bump":
            raise ValueError(f"Unknown allocator_type {allocator_type!r}; only 'torch_bump' exists")
        if _arena is None:
            if world_size != 1:
                raise RuntimeError(
                    "A stand-alone SymmetricHeap with world_size > 1 needs a second process, which "
                    "this single-GPU build does not have. Use SymmetricHeap.create_all(...) or "
                    "tileccl_amd.init_local(...) to get one heap per emulated rank."
                )
            _arena = Arena(size, 1)
        self._arena = _arena.acquire()
        self._size = int(size)
        self._rank = int(rank)
        self._world_size = int(world_size)
        self._backend_name = "hip"
        self._device = torch.device(DEVICE)
        self._buffer: torch.Tensor | None = self._arena.slice(rank)
        self._local_ptr = self._arena.bases[rank]
        self._bump = BumpAllocator(self._size, policy=self._BUMP_POLICY)
        self._mode = "single_process"
        self._transport_strategy = "local_only" if world_size == 1 else "peer_access"
        self._cleaned_up = False

    # ------------------------------------------------------------------ construction
    @classmethod
    def create_all(
        cls, size: int, world_size: int, backend: str = "auto", *, allocator_type: str = "torch_bump"
    ) -> list["SymmetricHeap"]:
        """One heap per emulated rank, all slices of a single arena."""
        if size <= 0:
            raise ValueError(f"Heap size must be positive, got {size}")
        if world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {world_size}")
        arena = Arena(size, world_size)
        return [
            cls(size, rank, world_size, backend, allocator_type=allocator_type, _arena=arena)
            for rank in range(world_size)
        ]

    # ------------------------------------------------------------------ allocation
    def _require_live(self) -> torch.Tensor:
        if self._buffer is None:
            raise RuntimeError("SymmetricHeap has been cleaned up")
        return self._buffer

    def allocate_tensor(self, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """View of ``shape``/``dtype`` into this slice; the start is 256-byte aligned."""
        buffer = self._require_live()
        shape = tuple(int(d) for d in shape)
        nbytes = math.prod(shape) * _element_size(dtype)
        start = self._bump.reserve(nbytes)
        return buffer.narrow(0, start, nbytes).view(dtype).reshape(shape)

    # ------------------------------------------------------------------ queries
    def get_heap_bases(self) -> torch.Tensor:
        if self._buffer is None or self._arena.heap_bases is None:
            raise RuntimeError("Heap bases not initialized.")
        return self._arena.heap_bases

    @property
    def local_base(self) -> int:
        return self._local_ptr

    @property
    def size(self) -> int:
        return self._size

    @property
    def rank(self) -> int:
        return self._rank

    @property
    def world_size(self) -> int:
        return self._world_size

    @property
    def device(self) -> torch.device:
        return self._device

    @property
    def bytes_allocated(self) -> int:
        return self._bump.offset

    @property
    def bytes_free(self) -> int:
        return self._bump.bytes_free

    @property
    def mode(self) -> str:
        return self._mode

    @property
    def transport_strategy(self) -> str:
        return self._transport_strategy

    @property
    def allocator_name(self) -> str:
        return "torch_bump"

    def _check_rank(self, rank: int, label: str = "rank") -> None:
        if rank < 0 or rank >= self._world_size:
            raise ValueError(f"{label}={rank} out of range for world_size={self._world_size}")

    def get_peer_buffer(self, rank: int) -> torch.Tensor:
        """The uint8 tensor backing ``rank``'s slice (host-side reference paths, diagnostics)."""
        self._require_live()
        self._check_rank(rank)
        return self._arena.slice(rank)

    def owns_tensor(self, tensor: torch.Tensor) -> bool:
        if self._buffer is None or tensor.device != self._device:
            return False
        if tensor.numel() == 0:
            return True
        return self._local_ptr <= int(tensor.data_ptr()) < self._local_ptr + self._size

    is_symmetric = owns_tensor

    def import_external_tensor(self, tensor: torch.Tensor) -> torch.Tensor:
        """Copy a contiguous device tensor into the heap."""
        self._require_live()
        if tensor.device != self._device:
            raise ValueError(
                "import_external_tensor requires the tensor to already be on the "
                f"allocator device {self._device}, got {tensor.device}"
            )
        if not tensor.is_contiguous():
            raise ValueError(
                "import_external_tensor requires a contiguous tensor. Call .contiguous() before importing."
            )
        inside = self.allocate_tensor(tuple(tensor.shape), tensor.dtype)
        inside.copy_(tensor)
        return inside

    as_symmetric = import_external_tensor

    def peer_view(self, tensor: torch.Tensor, rank: int) -> torch.Tensor:
        """The tensor at the same slice offset in ``rank``'s slice (what a peer would see)."""
        self._check_rank(rank)
        offset = self.get_offset(int(tensor.data_ptr()))
        nbytes = tensor.numel() * tensor.element_size()
        if not tensor.is_contiguous():
            raise ValueError("peer_view needs a contiguous tensor")
        return self._arena.slice(rank).narrow(0, offset, nbytes).view(tensor.dtype).reshape(tensor.shape)

    # ------------------------------------------------------------------ translation
    def get_offset(self, ptr: int) -> int:
        offset = ptr - self._local_ptr
        if offset < 0 or offset >= self._size:
            raise ValueError(
                f"Pointer 0x{ptr:x} is outside the heap "
                f"[0x{self._local_ptr:x}, 0x{self._local_ptr + self._size:x})"
            )
        return offset

    def translate(self, local_ptr: int, to_rank: int) -> int:
        """Host-side twin of the device ``translate_ptr``."""
        self._check_rank(to_rank, "to_rank")
        return self._arena.bases[to_rank] + self.get_offset(local_ptr)

    # ------------------------------------------------------------------ sync / teardown
    def barrier(self) -> None:
        torch.cuda.synchronize()

    def metadata(self) -> dict[str, object]:
        return {
            "size": self._size,
            "rank": self._rank,
            "world_size": self._world_size,
            "mode": self._mode,
            "transport_strategy": self._transport_strategy,
            "allocator": self.allocator_name,
            "bytes_allocated": self.bytes_allocated,
            "bytes_free": self.bytes_free,
            "device": str(self._device),
        }

    def cleanup(self) -> None:
        if self._cleaned_up:
            return
        self._cleaned_up = True
        self._buffer = None
        self._local_ptr = 0
        self._bump.reset()
        arena, self._arena = self._arena, None
        arena.release()

    def __enter__(self) -> "SymmetricHeap":
        return self

    def __exit__(self, *exc: object) -> None:
        self.cleanup()

    def __del__(self) -> None:
        try:
            self.cleanup()
        except Exception:
            pass

    def __repr__(self) -> str:
        return (
            f"SymmetricHeap(size={self._size}, rank={self._rank}, world_size={self._world_size}, "
            f"mode={self._mode!r})"
        )
