"""CPU model of the symmetric heap: a sliced uint8 arena with the reference's bump rules.

Test infrastructure only.  Follows
    v1 allocation (align the start offset to 256, exact size)
        /root/reference/tileccl/memory/allocators.py:574-607
    v2 allocation (round the size up to 256)
        /root/reference/tileccl_v2/heap.py:302-332
    pointer translation   base[to] + (ptr - base[from])
        /root/reference/tileccl/memory/translation.py:39-99
"""

from __future__ import annotations

import numpy as np
import torch


class CpuHeap:
    """``world`` slices of ``size`` bytes in one numpy arena; slice ``r`` starts at ``r*size``."""

    def __init__(self, size: int, world: int, policy: str = "v2") -> None:
        self.size, self.world, self.policy = size, world, policy
        self.arena = np.zeros(size * world, dtype=np.uint8)
        self.bases = [r * size for r in range(world)]
        self.offsets = [0] * world

    def alloc(self, rank: int, shape, dtype: torch.dtype) -> tuple[int, torch.Tensor]:
        """(offset inside the slice, tensor view) -- same arithmetic as the reference allocators."""
        esz = torch.empty((), dtype=dtype).element_size()
        nbytes = int(np.prod(shape)) * esz
        off = self.offsets[rank]
        if self.policy == "v1":
            start = (off + 255) // 256 * 256
            if start + nbytes > self.size:
                raise RuntimeError("heap exhausted")
            self.offsets[rank] = start + nbytes
        else:
            padded = (nbytes + 255) // 256 * 256
            if off + padded > self.size:
                raise RuntimeError("heap exhausted")
            start = off
            self.offsets[rank] = off + padded
        return start, self.view(rank, start, shape, dtype)

    def view(self, rank: int, offset: int, shape, dtype: torch.dtype) -> torch.Tensor:
        esz = torch.empty((), dtype=dtype).element_size()
        nbytes = int(np.prod(shape)) * esz
        lo = self.bases[rank] + offset
        raw = torch.from_numpy(self.arena[lo:lo + nbytes])
        return raw.view(dtype).reshape(tuple(shape))

    def translate(self, ptr: int, from_rank: int, to_rank: int) -> int:
        return self.bases[to_rank] + (ptr - self.bases[from_rank])
