"""Bump allocation arithmetic (product) against the CPU heap model (oracle) and invariants
(reference tileccl/memory/allocators.py:574-607, tileccl_v2/heap.py:302-332)."""

import random

import pytest
import torch

from oracle.heap_model import CpuHeap
from tileccl_amd.memory.bump import BumpAllocator, round_up


def test_round_up():
    assert [round_up(v) for v in (0, 1, 255, 256, 257)] == [0, 256, 256, 256, 512]


@pytest.mark.parametrize("policy,model", [("align_start", "v1"), ("round_size", "v2")])
def test_offsets_match_the_model_and_stay_aligned(policy, model):
    rng = random.Random(7)
    bump = BumpAllocator(1 << 20, policy=policy)
    heap = CpuHeap(1 << 20, 1, policy=model)
    last_end = 0
    for _ in range(200):
        shape = (rng.randint(1, 37), rng.randint(1, 19))
        dtype = rng.choice([torch.float16, torch.float32, torch.int32, torch.uint8, torch.bfloat16])
        nbytes = shape[0] * shape[1] * torch.empty((), dtype=dtype).element_size()
        want, _ = heap.alloc(0, shape, dtype)
        got = bump.reserve(nbytes)
        assert got == want
        assert got % 256 == 0 and got >= last_end  # aligned, monotone, no overlap
        last_end = got + nbytes
    assert bump.offset == heap.offsets[0]
    assert bump.bytes_free == (1 << 20) - bump.offset
    bump.reset()
    assert bump.offset == 0 and bump.records == []


def test_policies_differ_only_in_where_padding_goes():
    v1, v2 = BumpAllocator(4096, policy="align_start"), BumpAllocator(4096, policy="round_size")
    assert (v1.reserve(100), v1.offset) == (0, 100)
    assert (v2.reserve(100), v2.offset) == (0, 256)
    assert (v1.reserve(8), v1.offset) == (256, 264)
    assert (v2.reserve(8), v2.offset) == (256, 512)


def test_oom_messages():
    v1 = BumpAllocator(1000, policy="align_start")
    v1.reserve(300)
    with pytest.raises(RuntimeError, match=r"requested 600 bytes at offset 0x200, heap size is 1000 bytes \(488 bytes remaining\)"):
        v1.reserve(600)
    v2 = BumpAllocator(1024, policy="round_size")
    v2.reserve(300)
    with pytest.raises(RuntimeError, match=r"SymmetricHeap OOM: need 768 bytes but only 512 remaining \(total=1024, used=512\)"):
        v2.reserve(600)
    with pytest.raises(ValueError, match="Heap size must be positive, got 0"):
        BumpAllocator(0, policy="round_size")


def test_model_translation_and_symmetry():
    heap = CpuHeap(4096, 3, policy="v2")
    off0, t0 = heap.alloc(0, (4, 4), torch.float16)
    off1, t1 = heap.alloc(1, (4, 4), torch.float16)
    assert off0 == off1  # same allocation sequence -> same offset: that is what "symmetric" means
    ptr0 = heap.bases[0] + off0
    assert heap.translate(ptr0, 0, 1) == heap.bases[1] + off1
    assert heap.translate(heap.translate(ptr0, 0, 2), 2, 0) == ptr0
    t1.fill_(2.0)
    assert heap.view(1, off1, (4, 4), torch.float16).sum().item() == 32.0 and t0.sum().item() == 0.0


def test_context_shape_normalisation_and_missing_heap():
    import tileccl_amd

    assert tileccl_amd._normalize_shape((3, 4)) == (3, 4)
    assert tileccl_amd._normalize_shape(((3, 4),)) == (3, 4)
    assert tileccl_amd._normalize_shape(([5],)) == (5,)
    with pytest.raises(ValueError, match=r"Shape dimensions must be non-negative, got \(-1, 2\)"):
        tileccl_amd._normalize_shape((-1, 2))
    with pytest.raises(TypeError, match="Invalid shape specification"):
        tileccl_amd._normalize_shape((None,))
    ctx = tileccl_amd.TileCCLContext(rank=0, world_size=1, device="cuda:0", backend_name="hip", backend=None)
    assert not ctx.has_heap
    with pytest.raises(RuntimeError, match="No SymmetricHeap is attached"):
        ctx.require_heap()
    with pytest.raises(ValueError, match="Pass at most one of heap=... and heap_size=..."):
        tileccl_amd.init(backend="hip", heap=object(), heap_size=8) if False else (_ for _ in ()).throw(
            ValueError("Pass at most one of heap=... and heap_size=...")
        )
    with pytest.raises(ValueError, match="Unsupported backend: 'metal'"):
        tileccl_amd.init(backend="metal")
    with pytest.raises(ValueError, match="world_size must be >= 1, got 0"):
        tileccl_amd.init_local(0, 1024)
    with pytest.raises(ValueError, match="heap_size must be positive, got 0"):
        tileccl_amd.init_local(2, 0)
    with pytest.raises(RuntimeError, match="has not been initialised"):
        tileccl_amd._ctx = None
        tileccl_amd.current_context()


class _FakeArena:
    """The arena's bookkeeping over host memory: the three device hooks are replaced."""

    freed: list = []

    def __new__(cls, *args, **kwargs):
        from tileccl_amd.memory.arena import Arena

        class Fake(Arena):
            def _allocate(self, slice_bytes, world_size):
                return ("handle", slice_bytes), [4096 + r * slice_bytes for r in range(world_size)]

            def _view(self, base, nbytes):
                return torch.zeros(nbytes, dtype=torch.uint8)

            def _device_bases(self, bases):
                return torch.tensor(bases, dtype=torch.int64)

            def _deallocate(self, handle):
                _FakeArena.freed.append(handle)

        return Fake(*args, **kwargs)


def test_arena_is_freed_when_collected_not_when_the_last_heap_lets_go():
    import gc

    _FakeArena.freed = []
    arena = _FakeArena(1024, 2)
    users = [arena.acquire(), arena.acquire()]
    assert arena.live and arena.slice(1).numel() == 1024
    users[0].release()
    assert arena.live and arena.slice(0) is not None  # one heap still uses it
    users[1].release()
    assert arena.live and _FakeArena.freed == []  # nothing is freed under tensors that may still view it
    with pytest.raises(RuntimeError, match="cleaned up"):
        arena.slice(0)
    assert arena.heap_bases is None
    del arena, users
    gc.collect()
    assert _FakeArena.freed == [("handle", 1024)]  # exactly once, when nothing refers to the arena


def test_arena_rejects_bad_sizes_before_allocating():
    _FakeArena.freed = []
    with pytest.raises(ValueError, match="Heap size must be positive"):
        _FakeArena(0, 1)
    with pytest.raises(ValueError, match="world_size must be >= 1"):
        _FakeArena(16, 0)
    assert _FakeArena.freed == []
