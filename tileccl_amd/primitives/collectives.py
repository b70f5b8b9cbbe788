"""Stand-alone collectives on symmetric-heap tensors: host launchers.

Counterparts of the reference's host launchers ``allreduce / allgather / broadcast / scatter /
reduce_scatter`` (``/root/reference/tileccl/primitives/collectives.py:1882-2478``) with the
same argument order, contracts and messages.  The data movement is the reference's
direct-write / peer-read form (``tile_allgather`` :613-663, ``tile_scatter`` :671-727,
``tile_reduce_scatter`` :730-783, ``tile_broadcast`` :791-836) on this package's bulk copy and
reduce kernels.  Its staged peer-read kernels (:840-1592: snapshot a chunk into a slot,
publish an epoch, read the peers' slots, acknowledge) are the ``*_staged`` functions below,
all roles of a call in one launch.

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


# ---------------------------------------------------------------------------------------------
# The staged peer-read collectives (reference :840-1592; launchers :1882-2478).
#
# A rank's role waits, inside the kernel, for its peers' roles of the same call, so the roles
# cannot run one call after the other as the collectives above do.  With the ranks emulated as
# slices of one arena, one launch carries all of them ((rank, slot) -> workgroup); a process
# that owns a single rank of a real multi-GPU job would pass ``ranks=(heap.rank,)``.

STAGED_MIN_CHUNK_BYTES = 16 << 10      # a workgroup's chunk: 4 x 16 bytes per thread ...
STAGED_MAX_CHUNK_BYTES = 64 << 10      # ... to 16 x 16 bytes
STAGED_RESIDENT_WORKGROUPS = 1024      # world x slots must be resident at once (4 workgroups on each of 256 CUs)
STAGED_MAX_PIPELINE_SLOTS = 256        # workgroups per rank
_DEFAULT_SPIN_NS = 0                   # the library's default bound on a wait
_BYTES_AS = {1: torch.float8_e4m3fn, 2: torch.float16, 4: torch.float32}  # a library dtype of each element size


class _StagedWorkspace:
    """Staging rows and the two words per slot, at one offset in every rank's slice, plus the
    epoch counter of the calls that used them (reference ``_AllReduceWorkspace``, :2813-2838)."""

    def __init__(self, heaps, dtype: torch.dtype, chunk_elems: int, slots: int, segments: int) -> None:
        self.staging = [h.allocate_tensor((slots, segments, chunk_elems), dtype) for h in heaps]
        self.published = [h.allocate_tensor((slots,), torch.int32) for h in heaps]
        self.consumed = [h.allocate_tensor((slots,), torch.int32) for h in heaps]
        for group in (self.staging, self.published, self.consumed):
            offsets = {h.get_offset(int(t.data_ptr())) for h, t in zip(heaps, group)}
            if len(offsets) != 1:
                raise RuntimeError("staged collective: the ranks' heaps have diverged, no common workspace offset")
        for t in self.published + self.consumed:
            t.zero_()
        self.fault = torch.zeros(1, dtype=torch.int64, device=self.staging[0].device)
        self.next_epoch = 1

    def reserve_epoch_range(self, chunks: int) -> int:
        if self.next_epoch + chunks >= 2**31 - 1:  # start over: no role is in flight between calls on one stream
            for t in self.published + self.consumed:
                t.zero_()
            self.next_epoch = 1
        base, self.next_epoch = self.next_epoch, self.next_epoch + chunks
        return base


_STAGED: "weakref.WeakKeyDictionary" = weakref.WeakKeyDictionary()  # heap of rank 0 -> {(dtype, chunk, slots, segments): workspace}


def resolve_staged_execution(numel: int, element_size: int, world: int, *, chunk_elems: int | None = None,
                             pipeline_slots: int | None = None) -> tuple[int, int, int]:
    """(chunk_elems, chunks, pipeline_slots) for a block of ``numel`` elements: as many slots as
    stay resident, at most 256 per rank, and the smallest chunk of 16 / 32 / 64 KiB that gives
    every slot work (measured for the all-reduce on two and four ranks, 1 MiB to 256 MiB: more
    slots always won; 16 KiB chunks are quickest while the slots outnumber them, 64 KiB chunks
    from there on).  The reference's policy (:2586-2597, :1802-1880) picks 256..4096 elements and
    at most 8 or 16 programs for its target; the contract is the same."""
    per_unit = 16 // element_size
    slot_cap = max(1, min(STAGED_MAX_PIPELINE_SLOTS, STAGED_RESIDENT_WORKGROUPS // world))
    if chunk_elems is None:
        chunk_bytes = STAGED_MIN_CHUNK_BYTES
        while chunk_bytes < STAGED_MAX_CHUNK_BYTES and numel * element_size > chunk_bytes * slot_cap:
            chunk_bytes *= 2
        chunk_elems = min(chunk_bytes // element_size, -(-numel // per_unit) * per_unit)
    if chunk_elems <= 0 or chunk_elems % per_unit:
        raise ValueError(f"staged collective: chunk_elems={chunk_elems} must be a positive multiple of {per_unit}")
    chunks = -(-numel // chunk_elems)
    if pipeline_slots is None:
        pipeline_slots = min(chunks, slot_cap)
    if pipeline_slots < 1:
        raise ValueError(f"staged collective: pipeline_slots={pipeline_slots} must be at least 1")
    return chunk_elems, chunks, min(pipeline_slots, chunks)


def _one_per_rank(name: str, what: str, tensors, heaps) -> None:
    world = len(heaps)
    if len(tensors) != world or any(h.world_size != world or h.rank != r for r, h in enumerate(heaps)):
        raise ValueError(f"{name} expects one {what} and one heap per rank, in rank order")
    first = tensors[0]
    for r, (t, h) in enumerate(zip(tensors, heaps)):
        _contiguous(name, t, f"{what}s[{r}]")
        _on_heap(t, h, f"{what}s[{r}]")
        if t.dtype != first.dtype or t.shape != first.shape:
            raise ValueError(f"{name} expects one dtype and shape on every rank")
    if len({h.get_offset(int(t.data_ptr())) for t, h in zip(tensors, heaps)}) != 1:
        raise ValueError(f"{name} expects the {what} at the same heap offset on every rank")


def _staged(name: str, op: int, srcs, dsts, heaps, block: int, *, root: int = 0, chunk_elems=None, pipeline_slots=None,
            ranks=None, spin_limit_ns: int = _DEFAULT_SPIN_NS) -> torch.Tensor:
    """One launch of ``tccl_collective_staged`` with the roles of ``ranks`` (default: every rank).
    Returns the workspace's fault word (int64[1] on the device): non-zero after a wait ran into
    ``spin_limit_ns``, which is what happens when a role that the others wait for is left out."""
    world = len(heaps)
    first = dsts[0]
    carried = tuple(range(world)) if ranks is None else tuple(int(r) for r in ranks)
    for r in carried:
        _validate_root(r, world_size=world)
    if world == 1 or block == 0 or not carried:
        return torch.zeros(1, dtype=torch.int64, device=first.device)
    esz = first.element_size()
    _whole_units(name, block, esz)
    chunk_elems, chunks, slots = resolve_staged_execution(block, esz, world, chunk_elems=chunk_elems, pipeline_slots=pipeline_slots)
    segments = world if op in (_lib.STAGED_REDUCE_SCATTER, _lib.STAGED_SCATTER) else 1
    cache = _STAGED.setdefault(heaps[0], {})
    key = (str(first.dtype), chunk_elems, slots, segments)
    if key not in cache:
        cache[key] = _StagedWorkspace(heaps, first.dtype, chunk_elems, slots, segments)
    ws = cache[key]
    base_epoch = ws.reserve_epoch_range(chunks)
    ws.fault.zero_()
    view = _launch.heap_view(heaps[0].get_heap_bases(), 0, world)
    mask = 0
    for r in carried:
        mask |= 1 << r
    reduces = op in (_lib.STAGED_ALLREDUCE, _lib.STAGED_REDUCE_SCATTER)
    code = _launch.dtype_code(first.dtype if reduces else _BYTES_AS.get(esz, first.dtype))  # copies move bytes
    rc = _lib.load().tccl_collective_staged(
        op, _launch.ptr(srcs[0]) if srcs is not None else None, _launch.ptr(dsts[0]), code, block,
        _launch.ptr(ws.staging[0]), _launch.ptr(ws.published[0]), _launch.ptr(ws.consumed[0]), chunk_elems, slots, base_epoch, mask,
        int(root), _launch.byref(view), _launch.ptr(ws.fault), int(spin_limit_ns), _launch.stream_ptr(),
    )
    _lib.check(rc, f"tccl_collective_staged[{name}]")
    return ws.fault


def allreduce_staged(tensors, heaps, op: str = "sum", **how) -> torch.Tensor:
    """In place on every rank's tensor, in one launch: each ends with the sum over ranks (the ranks'
    values added in ascending rank order in fp32, one rounding: the same bits everywhere).
    ``tensors[r]`` is rank ``r``'s tensor in ``heaps[r]``, all at one heap offset.  Keywords
    ``chunk_elems``, ``pipeline_slots``, ``ranks``, ``spin_limit_ns``: see ``_staged``."""
    if op != "sum":
        raise ValueError(f"Only op='sum' is currently supported, got {op!r}")
    _validate_world_size(len(heaps))
    _one_per_rank("allreduce_staged", "tensor", tensors, heaps)
    if tensors[0].dtype not in _REDUCE_IN:
        raise ValueError(f"allreduce_staged supports fp16, bf16 and fp32 tensors, got {tensors[0].dtype}")
    return _staged("allreduce_staged", _lib.STAGED_ALLREDUCE, None, tensors, heaps, int(tensors[0].numel()), **how)


def allgather_staged(tensors, outputs, heaps, **how) -> torch.Tensor:
    """Every rank's ``output`` ends with ``[tensor_rank0 | tensor_rank1 | ...]`` (reference :1129-1215)."""
    world = len(heaps)
    _validate_world_size(world)
    _one_per_rank("allgather_staged", "tensor", tensors, heaps)
    _one_per_rank("allgather_staged", "output", outputs, heaps)
    block = _pair_block("allgather", tensor=tensors[0], output=outputs[0], world_size=world)
    if tensors[0].dtype != outputs[0].dtype:
        raise ValueError(f"allgather expects one dtype, got tensor={tensors[0].dtype}, output={outputs[0].dtype}")
    if world == 1 and block:
        outputs[0].reshape(-1).copy_(tensors[0].reshape(-1))
    return _staged("allgather_staged", _lib.STAGED_ALLGATHER, tensors, outputs, heaps, block, **how)


def reduce_scatter_staged(tensors, outputs, heaps, op: str = "sum", **how) -> torch.Tensor:
    """Rank ``r``'s ``output`` = its own chunk ``r`` plus the other ranks' chunk ``r`` in ascending rank
    (fp32 accumulation, one rounding; reference :1276-1366 and tile_reduce_scatter's order :766-781)."""
    if op != "sum":
        raise ValueError(f"Only op='sum' is currently supported, got {op!r}")
    world = len(heaps)
    _validate_world_size(world)
    _one_per_rank("reduce_scatter_staged", "tensor", tensors, heaps)
    _one_per_rank("reduce_scatter_staged", "output", outputs, heaps)
    block = _pair_block("reduce_scatter", tensor=tensors[0], output=outputs[0], world_size=world)
    if tensors[0].dtype not in _REDUCE_IN or outputs[0].dtype != tensors[0].dtype:
        raise ValueError(f"reduce_scatter_staged supports fp16, bf16 and fp32, output of the tensor's type; got "
                         f"{tensors[0].dtype} -> {outputs[0].dtype}")
    if world == 1 and block:
        outputs[0].reshape(-1).copy_(tensors[0].reshape(-1))
    return _staged("reduce_scatter_staged", _lib.STAGED_REDUCE_SCATTER, tensors, outputs, heaps, block, **how)


def broadcast_staged(tensors, heaps, root: int = 0, **how) -> torch.Tensor:
    """Every rank's tensor ends with the root's (reference :1391-1486)."""
    world = len(heaps)
    _validate_world_size(world)
    _validate_root(root, world_size=world)
    _one_per_rank("broadcast_staged", "tensor", tensors, heaps)
    return _staged("broadcast_staged", _lib.STAGED_BROADCAST, None, tensors, heaps, int(tensors[0].numel()), root=root, **how)


def scatter_staged(tensors, outputs, heaps, *, root: int = 0, **how) -> torch.Tensor:
    """Rank ``i``'s ``output`` receives chunk ``i`` of the root's ``tensor`` (reference :1489-1592)."""
    world = len(heaps)
    _validate_world_size(world)
    _validate_root(root, world_size=world)
    _one_per_rank("scatter_staged", "tensor", tensors, heaps)
    _one_per_rank("scatter_staged", "output", outputs, heaps)
    block = _pair_block("scatter", tensor=tensors[0], output=outputs[0], world_size=world)
    if tensors[0].dtype != outputs[0].dtype:
        raise ValueError(f"scatter expects one dtype, got tensor={tensors[0].dtype}, output={outputs[0].dtype}")
    if world == 1 and block:
        outputs[0].reshape(-1).copy_(tensors[0].reshape(-1))
    return _staged("scatter_staged", _lib.STAGED_SCATTER, tensors, outputs, heaps, block, root=root, **how)
