"""Stand-alone collectives on symmetric-heap tensors: host launchers.

Counterparts of the reference's host launchers ``allreduce / allgather / broadcast / scatter /
reduce_scatter`` (``/root/reference/tileccl/primitives/collectives.py:1882-2478``) with the
same argument order, contracts and messages.  The data movement is the reference's
direct-write / peer-read form (``tile_allgather`` :613-663, ``tile_scatter`` :671-727,
``tile_reduce_scatter`` :730-783, ``tile_broadcast`` :791-836) on this package's bulk copy and
reduce kernels; its chunked and staged multi-process variants (:840-1592) are scheduling of
the same movement and have no counterpart here.

What differs, on purpose:

* Reductions accumulate in fp32 (the owner's chunk first, then the other ranks ascending) and
  round once; the reference adds in the tensor dtype.  Outputs are fp16 or bf16, or fp32 for
  fp32 tensors.
* Blocks move in 16-byte units: a rank's block must be a multiple of 16 bytes (8 elements for
  the reductions).  The reference's one-program kernels take any power-of-two block.
* ``allreduce`` is the reduce-scatter of the caller's chunk followed by its direct write into
  every rank's tensor.  A rank reads and overwrites only its own chunk index on every rank,
  so the calls of different ranks do not conflict in whatever order they run; a tensor is
  complete once every rank's call has finished.

Every call is asynchronous on torch's current stream.
"""

from __future__ import annotations

import weakref

import torch

from tileccl_amd import _launch, _lib
from tileccl_amd.primitives.communication import copy_block

MAX_COLLECTIVE_WORLD_SIZE = _lib.MAX_WORLD

_REDUCE_IN = (torch.float16, torch.bfloat16, torch.float32)
_REDUCE_OUT = (torch.float16, torch.bfloat16)


def _validate_world_size(world_size: int) -> None:
    if world_size > MAX_COLLECTIVE_WORLD_SIZE:
        raise ValueError(f"world_size={world_size} exceeds maximum supported ({MAX_COLLECTIVE_WORLD_SIZE}).")


def _validate_root(root: int, *, world_size: int) -> None:
    if root < 0 or root >= world_size:
        raise ValueError(f"root={root} out of range [0, {world_size})")


def _pair_block(collective: str, *, tensor: torch.Tensor, output: torch.Tensor, world_size: int) -> int:
    """The numel contract of a tensor/output pair (reference :1702-1730); returns the block size."""
    if collective == "allgather":
        block = int(tensor.numel())
        if int(output.numel()) != world_size * block:
            raise ValueError(
                f"allgather output.numel must equal tensor.numel * world_size: {output.numel()} != {block} * {world_size}"
            )
        return block
    block = int(output.numel())
    if int(tensor.numel()) != world_size * block:
        raise ValueError(
            f"{collective} tensor.numel must equal output.numel * world_size: {tensor.numel()} != {block} * {world_size}"
        )
    return block


def _same_device(collective: str, tensor: torch.Tensor, output: torch.Tensor) -> None:
    if tensor.device != output.device:
        raise ValueError(f"{collective} expects tensor/output on the same device, got {tensor.device} vs {output.device}")


def _contiguous(collective: str, t: torch.Tensor, name: str) -> None:
    if not t.is_contiguous():
        raise ValueError(f"{collective} currently requires {name} to be contiguous")


def _on_heap(t: torch.Tensor, heap, name: str) -> None:
    if not heap.owns_tensor(t):
        raise ValueError(f"{name} must reside in the provided SymmetricHeap for rank {heap.rank}")


def _whole_units(collective: str, block: int, element_size: int, *, reduce: bool = False) -> None:
    if (block * element_size) % 16 or (reduce and block % 8):
        need = "8 elements" if reduce else "16 bytes"
        raise ValueError(f"{collective}: a rank's block of {block} elements is not a multiple of {need}")


def allgather(tensor: torch.Tensor, output: torch.Tensor, heap) -> None:
    """Every rank ends with ``[tensor_rank0 | tensor_rank1 | ...]`` in ``output``.

    Direct write (reference :628-630): the caller's block goes into block ``rank`` of every
    rank's ``output``, its own included, in one launch.
    """
    world = heap.world_size
    _validate_world_size(world)
    block = _pair_block("allgather", tensor=tensor, output=output, world_size=world)
    _same_device("allgather", tensor, output)
    _contiguous("allgather", tensor, "tensor")
    _contiguous("allgather", output, "output")
    _on_heap(tensor, heap, "tensor")
    _on_heap(output, heap, "output")
    if tensor.dtype != output.dtype:
        raise ValueError(f"allgather expects one dtype, got tensor={tensor.dtype}, output={output.dtype}")
    if block == 0:
        return
    _whole_units("allgather", block, tensor.element_size())
    mine = output.reshape(-1)[heap.rank * block : (heap.rank + 1) * block]
    copy_block(mine, tensor.reshape(-1), heap, src_rank=heap.rank, dst_ranks=range(world))


def broadcast(tensor: torch.Tensor, heap, root: int = 0) -> None:
    """After the root's call every rank's ``tensor`` holds the root's data; other ranks' calls do nothing."""
    world = heap.world_size
    _validate_world_size(world)
    _validate_root(root, world_size=world)
    _contiguous("broadcast", tensor, "tensor")
    _on_heap(tensor, heap, "tensor")
    if heap.rank != root or tensor.numel() == 0:
        return
    _whole_units("broadcast", int(tensor.numel()), tensor.element_size())
    flat = tensor.reshape(-1)
    copy_block(flat, flat, heap, src_rank=root, dst_ranks=[r for r in range(world) if r != root])


def scatter(tensor: torch.Tensor, output: torch.Tensor, heap, *, root: int = 0) -> None:
    """Rank ``i`` receives chunk ``i`` of the root's ``tensor`` in its ``output``; only the root works."""
    world = heap.world_size
    _validate_world_size(world)
    _validate_root(root, world_size=world)
    block = _pair_block("scatter", tensor=tensor, output=output, world_size=world)
    _same_device("scatter", tensor, output)
    _contiguous("scatter", tensor, "tensor")
    _contiguous("scatter", output, "output")
    _on_heap(tensor, heap, "tensor")
    _on_heap(output, heap, "output")
    if tensor.dtype != output.dtype:
        raise ValueError(f"scatter expects one dtype, got tensor={tensor.dtype}, output={output.dtype}")
    if heap.rank != root or block == 0:
        return
    _whole_units("scatter", block, tensor.element_size())
    flat, out = tensor.reshape(-1), output.reshape(-1)
    for r in range(world):
        copy_block(out, flat[r * block : (r + 1) * block], heap, src_rank=root, dst_ranks=(r,))


def _reduce_chunk(collective: str, tensor: torch.Tensor, out: torch.Tensor, heap, block: int) -> None:
    """out = sum over ranks of chunk ``heap.rank`` of their ``tensor`` (peer reads, fp32 accumulate)."""
    if tensor.dtype not in _REDUCE_IN:
        raise ValueError(f"{collective} supports fp16, bf16 and fp32 tensors, got {tensor.dtype}")
    if out.dtype not in _REDUCE_OUT and not (out.dtype == torch.float32 and tensor.dtype == torch.float32):
        raise ValueError(f"{collective} writes fp16 or bf16 (fp32 for fp32 tensors), got {out.dtype} from {tensor.dtype}")
    _whole_units(collective, block, tensor.element_size(), reduce=True)
    view = _launch.heap_view(heap.get_heap_bases(), heap.rank, heap.world_size)
    rc = _lib.load().tccl_reduce_rows(
        _launch.ptr(tensor), _launch.dtype_code(tensor.dtype), block, _launch.ptr(out), _launch.dtype_code(out.dtype), block,
        heap.world_size, block, _launch.byref(view), None, 0, _launch.stream_ptr(),
    )
    _lib.check(rc, f"tccl_reduce_rows[{collective}]")


def reduce_scatter(tensor: torch.Tensor, output: torch.Tensor, heap, op: str = "sum", implementation: str = "auto") -> None:
    """``output`` = sum over ranks of chunk ``rank`` of their ``tensor`` (peer reads).

    ``implementation``: the reference chooses between a host restatement and its device
    kernel; here every value runs the device kernel.
    """
    if op != "sum":
        raise ValueError(f"Only op='sum' is currently supported, got {op!r}")
    if implementation not in {"auto", "reference", "device"}:
        raise ValueError(f"implementation must be one of {{'auto', 'reference', 'device'}}, got {implementation!r}")
    world = heap.world_size
    _validate_world_size(world)
    block = _pair_block("reduce_scatter", tensor=tensor, output=output, world_size=world)
    _same_device("reduce_scatter", tensor, output)
    _contiguous("reduce_scatter", tensor, "tensor")
    _contiguous("reduce_scatter", output, "output")
    _on_heap(tensor, heap, "tensor")
    _on_heap(output, heap, "output")
    if block == 0:
        return
    _reduce_chunk("reduce_scatter", tensor, output, heap, block)


_STAGING: "weakref.WeakKeyDictionary" = weakref.WeakKeyDictionary()  # heap -> {(block, dtype): tensor}


def _staging(heap, block: int, dtype: torch.dtype) -> torch.Tensor:
    """One reduced chunk per (block, dtype), allocated from the heap on first use (the
    reference caches its all-reduce workspace the same way, :2792-2838).  Ranks that call in
    the same order get the same offset, like every symmetric allocation."""
    cache = _STAGING.setdefault(heap, {})
    key = (block, str(dtype))
    if key not in cache:
        cache[key] = heap.allocate_tensor((block,), dtype)
    return cache[key]


def allreduce(tensor: torch.Tensor, heap, op: str = "sum") -> None:
    """In place: once every rank has called, every rank's ``tensor`` holds the sum over ranks."""
    if op != "sum":
        raise ValueError(f"Only op='sum' is currently supported, got {op!r}")
    world = heap.world_size
    _validate_world_size(world)
    _contiguous("allreduce", tensor, "tensor")
    _on_heap(tensor, heap, "tensor")
    numel = int(tensor.numel())
    if world == 1 or numel == 0:
        return  # local identity (reference :2563-2583)
    if tensor.dtype not in _REDUCE_IN:
        raise ValueError(f"allreduce supports fp16, bf16 and fp32 tensors, got {tensor.dtype}")
    if numel % world:
        raise ValueError(f"allreduce tensor.numel={numel} must be divisible by world_size={world}")
    block = numel // world
    _whole_units("allreduce", block, tensor.element_size(), reduce=True)
    flat = tensor.reshape(-1)
    stage = _staging(heap, block, tensor.dtype)
    _reduce_chunk("allreduce", flat, stage, heap, block)
    copy_block(flat[heap.rank * block : (heap.rank + 1) * block], stage, heap, src_rank=heap.rank, dst_ranks=range(world))
