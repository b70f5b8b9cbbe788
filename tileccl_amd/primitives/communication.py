"""Block put / get between heap slices.

The reference's ``tile_put`` / ``tile_get`` are device functions that move one tile through
registers after translating one of the two pointers into a peer's address space
(``/root/reference/tileccl/primitives/communication.py:133-225``).  Here the same movement is
a host call on whole contiguous tensors: ``tccl_copy_block`` reads the block in one slice and
writes it into one or several others with the bulk copy kernel (16 bytes per lane and access,
eight loads in flight).  Addresses are symmetric: a tensor of the calling rank names the same
offset in every slice.
"""

from __future__ import annotations

import torch

from tileccl_amd import _launch, _lib


def _check_block(name: str, t: torch.Tensor, heap) -> None:
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if not heap.owns_tensor(t):
        raise ValueError(f"{name} must reside in the provided SymmetricHeap for rank {heap.rank}")


def copy_block(dst: torch.Tensor, src: torch.Tensor, heap, *, src_rank: int, dst_ranks) -> None:
    """``dst`` (as seen by every rank of ``dst_ranks``) = ``src`` (as seen by ``src_rank``).

    Both tensors are the calling rank's; ``dst_ranks`` is an iterable of ranks.  Byte counts
    must be multiples of 16 (heap allocations start on 256-byte boundaries).
    """
    _check_block("dst", dst, heap)
    _check_block("src", src, heap)
    nbytes = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != nbytes:
        raise ValueError(f"dst and src must hold the same number of bytes: {dst.numel() * dst.element_size()} != {nbytes}")
    mask = 0
    for label, ranks in (("dst_rank", dst_ranks), ("src_rank", (src_rank,))):
        for r in ranks:
            if not 0 <= int(r) < heap.world_size:
                raise ValueError(f"{label}={int(r)} out of range for world_size={heap.world_size}")
            if label == "dst_rank":
                mask |= 1 << int(r)
    if nbytes == 0 or mask == 0:
        return
    view = _launch.heap_view(heap.get_heap_bases(), heap.rank, heap.world_size)
    rc = _lib.load().tccl_copy_block(
        _launch.ptr(dst), mask, _launch.ptr(src), int(src_rank), 1, nbytes, nbytes, nbytes, _launch.byref(view),
        _launch.stream_ptr(),
    )
    _lib.check(rc, "tccl_copy_block")


def put(src: torch.Tensor, dst: torch.Tensor, heap, dst_rank: int) -> None:
    """Push: the caller's ``src`` lands in ``dst`` of rank ``dst_rank`` (tile_put, :133-177)."""
    copy_block(dst, src, heap, src_rank=heap.rank, dst_ranks=(dst_rank,))


def get(dst: torch.Tensor, src: torch.Tensor, heap, from_rank: int) -> None:
    """Pull: ``src`` of rank ``from_rank`` lands in the caller's ``dst`` (tile_get, :180-225)."""
    copy_block(dst, src, heap, src_rank=from_rank, dst_ranks=(heap.rank,))
