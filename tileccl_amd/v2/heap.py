"""Symmetric heap with the reference's v2 surface (``/root/reference/tileccl_v2/heap.py:88-388``).

Same arena-slice design as ``tileccl_amd.memory.symmetric_heap``; what the v2 API adds or
changes is kept: ``allocate_tensor`` defaults to fp16, rejects empty / non-positive shapes
and rounds the *size* up to 256 bytes (heap.py:302-332), ``allocate_signal_buffer`` returns
zeroed int32 words (:334-341), ``reset_allocator`` rewinds the bump pointer (:343),
``local_ptr`` / ``bytes_used`` names (:283, :348).
"""

from __future__ import annotations

import torch

from tileccl_amd.memory.symmetric_heap import SymmetricHeap as _SliceHeap
from tileccl_amd.memory.symmetric_heap import _element_size


class SymmetricHeap(_SliceHeap):
    _BUMP_POLICY = "round_size"

    def __init__(self, size: int, rank: int, world_size: int, *, _arena=None, group=None) -> None:
        del group  # process groups only matter for multi-process IPC, which does not exist here
        super().__init__(size, rank, world_size, _arena=_arena)

    @classmethod
    def create_all(cls, size: int, world_size: int) -> list["SymmetricHeap"]:
        from tileccl_amd.memory.arena import Arena

        if size <= 0:
            raise ValueError(f"Heap size must be positive, got {size}")
        if world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {world_size}")
        arena = Arena(size, world_size)
        return [cls(size, rank, world_size, _arena=arena) for rank in range(world_size)]

    def allocate_tensor(self, shape: tuple[int, ...], dtype: torch.dtype = torch.float16) -> torch.Tensor:
        if not shape:
            raise ValueError("shape must be non-empty")
        if not all(isinstance(s, int) and s > 0 for s in shape):
            raise ValueError(f"All shape dimensions must be positive integers, got {shape}")
        buffer = self._require_live()
        count = 1
        for s in shape:
            count *= s
        nbytes = count * _element_size(dtype)
        start = self._bump.reserve(nbytes)
        return buffer.narrow(0, start, nbytes).view(dtype).reshape(shape)

    def allocate_signal_buffer(self, n_tiles: int) -> torch.Tensor:
        words = self.allocate_tensor((n_tiles,), dtype=torch.int32)
        words.zero_()
        return words

    def reset_allocator(self) -> None:
        self._bump.reset()

    @property
    def local_ptr(self) -> int:
        return self._local_ptr

    @property
    def bytes_used(self) -> int:
        return self._bump.offset
