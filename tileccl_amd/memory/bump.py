"""Bump allocation arithmetic of the symmetric heap, free of any device dependency.

Two policies exist in the reference and both are kept:

* ``"align_start"`` -- round the *start offset* up to the alignment and take exactly the
  bytes asked for (``/root/reference/tileccl/memory/allocators.py:574-607``);
* ``"round_size"``  -- round the *size* up to the alignment, so every start is aligned as
  a consequence (``/root/reference/tileccl_v2/heap.py:302-332``).

Nothing is ever freed; ``reset`` rewinds to offset 0.
"""

from __future__ import annotations

ALIGNMENT = 256


def round_up(value: int, alignment: int = ALIGNMENT) -> int:
    return -(-value // alignment) * alignment


class BumpAllocator:
    def __init__(self, size: int, *, policy: str, alignment: int = ALIGNMENT) -> None:
        if size <= 0:
            raise ValueError(f"Heap size must be positive, got {size}")
        if policy not in ("align_start", "round_size"):
            raise ValueError(f"unknown bump policy {policy!r}")
        self.size = int(size)
        self.policy = policy
        self.alignment = int(alignment)
        self.offset = 0
        self.records: list[tuple[int, int]] = []  # (start, nbytes)

    @property
    def bytes_free(self) -> int:
        return self.size - self.offset

    def reserve(self, nbytes: int) -> int:
        """Start offset of a new ``nbytes`` block; raises ``RuntimeError`` when it does not fit."""
        if self.policy == "align_start":
            start = round_up(self.offset, self.alignment)
            if start + nbytes > self.size:
                raise RuntimeError(
                    "Symmetric heap exhausted via allocator torch_bump: "
                    f"requested {nbytes} bytes at offset 0x{start:x}, heap size is {self.size} bytes "
                    f"({self.size - start} bytes remaining)"
                )
            self.offset = start + nbytes
        else:
            padded = round_up(nbytes, self.alignment)
            if self.offset + padded > self.size:
                raise RuntimeError(
                    f"SymmetricHeap OOM: need {padded} bytes but only "
                    f"{self.size - self.offset} remaining "
                    f"(total={self.size}, used={self.offset})"
                )
            start = self.offset
            self.offset += padded
        self.records.append((start, nbytes))
        return start

    def reset(self) -> None:
        self.offset = 0
        self.records.clear()
