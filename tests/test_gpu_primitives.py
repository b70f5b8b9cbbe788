"""The stand-alone collectives and block put / get on the GPU, against the CPU oracle.

Ranks are emulated as slices of one arena and call one after the other, as the reference's
single-process heaps do (primitives/collectives.py:2513-2546).  Copies are compared byte for
byte; reductions bit for bit with the oracle (fp32 accumulate, owner first) and within one
rounding of the reference's own restatement (ascending ranks in the tensor dtype)."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import bits, into_heap, seeded

pytestmark = pytest.mark.gpu


def heaps_of(world, size=64 << 20):
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    return SymmetricHeap.create_all(size=size, world_size=world)


def close(heaps):
    for h in heaps:
        h.cleanup()


@pytest.mark.parametrize("world,block,dtype", [(2, 4096, torch.float16), (3, 40, torch.float32), (4, 1 << 20, torch.bfloat16),
                                               (8, 8, torch.float16), (2, 16, torch.int8)])
def test_allgather_every_rank_gets_the_concatenation(lib, world, block, dtype):
    from tileccl_amd.primitives import allgather

    heaps = heaps_of(world, 128 << 20)
    try:
        if dtype == torch.int8:
            cpu = [torch.randint(-128, 127, (block,), dtype=torch.int8, generator=torch.Generator().manual_seed(r)) for r in range(world)]
        else:
            cpu = [seeded((block,), r, dtype) for r in range(world)]
        ins = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        outs = [h.allocate_tensor((world * block,), dtype) for h in heaps]
        for o in outs:
            o.fill_(0)
        # after rank 0's call alone: block 0 everywhere, the rest untouched
        allgather(ins[0], outs[0], heaps[0])
        torch.cuda.synchronize()
        for o in outs:
            assert torch.equal(o[:block].cpu(), cpu[0]) and not o[block:].any()
        for r in range(1, world):
            allgather(ins[r], outs[r], heaps[r])
        torch.cuda.synchronize()
        want = oracle.allgather(cpu)
        for r in range(world):
            assert torch.equal(outs[r].cpu(), want[r])
    finally:
        close(heaps)


@pytest.mark.parametrize("world,root", [(2, 0), (2, 1), (4, 2)])
def test_broadcast_from_root_only(lib, world, root):
    from tileccl_amd.primitives import broadcast

    heaps = heaps_of(world)
    try:
        cpu = [seeded((3, 1000, 8), 10 + r) for r in range(world)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        for r in range(world):
            if r != root:
                broadcast(ts[r], heaps[r], root)  # a non-root call moves nothing
        torch.cuda.synchronize()
        for r in range(world):
            assert torch.equal(ts[r].cpu(), cpu[r])
        broadcast(ts[root], heaps[root], root)
        torch.cuda.synchronize()
        want = oracle.broadcast(cpu, root)
        for r in range(world):
            assert torch.equal(bits(ts[r]).cpu(), bits(want[r]))
    finally:
        close(heaps)


@pytest.mark.parametrize("world,root,block", [(2, 1, 2048), (3, 0, 24), (8, 5, 4096)])
def test_scatter_chunks_to_their_ranks(lib, world, root, block):
    from tileccl_amd.primitives import scatter

    heaps = heaps_of(world)
    try:
        cpu = [seeded((world * block,), 20 + r, torch.bfloat16) for r in range(world)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        outs = [h.allocate_tensor((block,), torch.bfloat16) for h in heaps]
        for o in outs:
            o.fill_(0)
        for r in range(world):
            scatter(ts[r], outs[r], heaps[r], root=root)
        torch.cuda.synchronize()
        want = oracle.scatter(cpu[root], world)
        for r in range(world):
            assert torch.equal(bits(outs[r]).cpu(), bits(want[r]))
            assert torch.equal(ts[r].cpu(), cpu[r])  # sources untouched
    finally:
        close(heaps)


@pytest.mark.parametrize("world,block,dtype,odtype", [
    (2, 4096, torch.float16, torch.float16), (2, 1 << 18, torch.float32, torch.float16), (3, 72, torch.bfloat16, torch.bfloat16),
    (4, 2048, torch.float32, torch.bfloat16), (8, 8, torch.float16, torch.float16),
    (2, 4096, torch.float32, torch.float32), (3, 1 << 16, torch.float32, torch.float32),
])
def test_reduce_scatter_matches_the_oracle_bit_for_bit(lib, world, block, dtype, odtype):
    from tileccl_amd.primitives import reduce_scatter

    heaps = heaps_of(world)
    try:
        cpu = [seeded((world, block), 30 + r, dtype) for r in range(world)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        outs = [h.allocate_tensor((block,), odtype) for h in heaps]
        for r in range(world):
            reduce_scatter(ts[r], outs[r], heaps[r])
        torch.cuda.synchronize()
        want = oracle.reduce_scatter(cpu, odtype)
        for r in range(world):
            assert torch.equal(bits(outs[r]).cpu(), bits(want[r]))
            # the reference's restatement: ascending ranks, tensor dtype (:2536-2545)
            plain = cpu[0].reshape(world, -1)[r].clone()
            for p in range(1, world):
                plain = plain + cpu[p].reshape(world, -1)[r]
            assert torch.allclose(outs[r].cpu().float(), plain.float().to(odtype).float(),
                                  rtol=2 ** -7 if odtype == torch.bfloat16 else 2 ** -9, atol=1e-2)
    finally:
        close(heaps)


@pytest.mark.parametrize("world,numel,dtype", [(2, 1 << 16, torch.float16), (4, 4096, torch.bfloat16), (3, 3 * 8, torch.float16),
                                               (2, 1 << 20, torch.float32)])
def test_allreduce_in_place_any_call_order(lib, world, numel, dtype):
    from tileccl_amd.primitives import allreduce

    heaps = heaps_of(world)
    try:
        cpu = [seeded((numel,), 40 + r, dtype) for r in range(world)]
        want = oracle.allreduce(cpu)
        for order in (range(world), reversed(range(world))):
            ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
            for r in order:
                allreduce(ts[r], heaps[r])
            torch.cuda.synchronize()
            for r in range(world):
                assert torch.equal(bits(ts[r]).cpu(), bits(want[r]))
        # world 1: the local identity
        solo = heaps_of(1)
        try:
            t = into_heap(solo[0], cpu[0])
            allreduce(t, solo[0])
            torch.cuda.synchronize()
            assert torch.equal(t.cpu(), cpu[0])
        finally:
            close(solo)
    finally:
        close(heaps)


@pytest.mark.parametrize("world,numel,dtype,chunk,slots", [
    (2, 1 << 16, torch.float16, None, None),      # two chunks of 64 KiB, a slot each
    (2, 1 << 20, torch.bfloat16, 4096, 4),        # 256 chunks through 4 slots: every slot reused 64 times
    (3, 40 * 8, torch.float16, 64, 2),            # ragged: five chunks, the last one short, odd count over two slots
    (4, 1 << 18, torch.float32, None, None),
    (8, 3 * 4096 + 8, torch.float16, 4096, None), # last chunk of one unit
    (2, 8, torch.float16, None, None),            # one 16-byte unit
])
def test_staged_allreduce_all_roles_in_one_launch(lib, world, numel, dtype, chunk, slots):
    """Bit-exact against the oracle on every rank, on two calls in a row over the same workspace
    (the second with the first's results as input: epochs continue, slots are reused)."""
    from tileccl_amd.primitives import allreduce_staged

    heaps = heaps_of(world)
    try:
        cpu = [seeded((numel,), 70 + r, dtype) for r in range(world)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        for _ in range(2):
            want = oracle.allreduce_staged(cpu)
            fault = allreduce_staged(ts, heaps, chunk_elems=chunk, pipeline_slots=slots)
            torch.cuda.synchronize()
            assert int(fault.item()) == 0
            for r in range(world):
                assert torch.equal(bits(ts[r]).cpu(), bits(want[r])), r
            cpu = [(w * 0.25).to(dtype) for w in want]  # keep the values in range for the second call
            for t, c in zip(ts, cpu):
                t.copy_(c)
        if world == 2:  # two addends commute: the same bits as the reduce-scatter based all-reduce
            assert torch.equal(bits(oracle.allreduce_staged(cpu)[0]), bits(oracle.allreduce(cpu)[0]))
    finally:
        close(heaps)


STAGED_CASES = [
    # world, block, dtype, chunk_elems, pipeline_slots
    (2, 1 << 16, torch.float16, None, None),
    (2, 1 << 19, torch.bfloat16, 4096, 4),       # 128 chunks through 4 slots
    (3, 40 * 8, torch.float16, 64, 2),           # five chunks, the last one short
    (4, 3 * 4096 + 4, torch.float32, 4096, None),
    (8, 4096, torch.float16, 1024, 3),
    (2, 16, torch.int8, None, None),             # copies move bytes of any 1 / 2 / 4-byte type
]
REDUCING = [c for c in STAGED_CASES if c[2] != torch.int8]


def staged_inputs(world, shape, dtype, seed):
    if dtype == torch.int8:
        g = torch.Generator().manual_seed(seed)
        return [torch.randint(-128, 127, shape, generator=g, dtype=torch.int8) for _ in range(world)]
    return [seeded(shape, seed + r, dtype) for r in range(world)]


def raw(t):
    return t.contiguous().view(torch.uint8)


@pytest.mark.parametrize("world,block,dtype,chunk,slots", STAGED_CASES)
def test_staged_allgather(lib, world, block, dtype, chunk, slots):
    from tileccl_amd.primitives import allgather_staged

    heaps = heaps_of(world)
    try:
        for call in range(2):  # the second call reuses the workspace: epochs continue
            cpu = staged_inputs(world, (block,), dtype, 100 + 10 * call)
            ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
            outs = [h.allocate_tensor((world * block,), dtype) for h in heaps]
            for o in outs:
                raw(o).zero_()
            fault = allgather_staged(ts, outs, heaps, chunk_elems=chunk, pipeline_slots=slots)
            torch.cuda.synchronize()
            assert int(fault.item()) == 0
            want = oracle.allgather(cpu)
            for r in range(world):
                assert torch.equal(raw(outs[r]).cpu(), raw(want[r])), (call, r)
    finally:
        close(heaps)


@pytest.mark.parametrize("world,block,dtype,chunk,slots", REDUCING)
def test_staged_reduce_scatter(lib, world, block, dtype, chunk, slots):
    from tileccl_amd.primitives import reduce_scatter_staged

    heaps = heaps_of(world)
    try:
        for call in range(2):
            cpu = staged_inputs(world, (world * block,), dtype, 200 + 10 * call)
            ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
            outs = [h.allocate_tensor((block,), dtype) for h in heaps]
            for o in outs:
                o.zero_()
            fault = reduce_scatter_staged(ts, outs, heaps, chunk_elems=chunk, pipeline_slots=slots)
            torch.cuda.synchronize()
            assert int(fault.item()) == 0
            want = oracle.reduce_scatter(cpu, dtype)  # the owner's chunk first, then the other ranks ascending
            for r in range(world):
                assert torch.equal(raw(outs[r]).cpu(), raw(want[r])), (call, r)
                assert torch.equal(raw(ts[r]).cpu(), raw(cpu[r]))  # inputs untouched
    finally:
        close(heaps)


@pytest.mark.parametrize("world,block,dtype,chunk,slots", STAGED_CASES)
def test_staged_broadcast_and_scatter(lib, world, block, dtype, chunk, slots):
    from tileccl_amd.primitives import broadcast_staged, scatter_staged

    heaps = heaps_of(world)
    try:
        for root in (0, world - 1):
            cpu = staged_inputs(world, (block,), dtype, 300 + root)
            ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
            fault = broadcast_staged(ts, heaps, root=root, chunk_elems=chunk, pipeline_slots=slots)
            torch.cuda.synchronize()
            assert int(fault.item()) == 0
            for r, w in enumerate(oracle.broadcast(cpu, root)):
                assert torch.equal(raw(ts[r]).cpu(), raw(w)), (root, r)

            full = staged_inputs(world, (world * block,), dtype, 400 + root)
            srcs = [into_heap(h, c) for h, c in zip(heaps, full)]
            outs = [h.allocate_tensor((block,), dtype) for h in heaps]
            for o in outs:
                raw(o).zero_()
            fault = scatter_staged(srcs, outs, heaps, root=root, chunk_elems=chunk, pipeline_slots=slots)
            torch.cuda.synchronize()
            assert int(fault.item()) == 0
            for r, w in enumerate(oracle.scatter(full[root], world)):
                assert torch.equal(raw(outs[r]).cpu(), raw(w)), (root, r)
    finally:
        close(heaps)


@pytest.mark.parametrize("seed", [21, 22])
def test_staged_collectives_random_sizes(lib, seed):
    """Seeded random worlds, block sizes, chunk sizes and slot counts through the five staged
    collectives, several calls on one set of heaps (workspaces and epochs are reused)."""
    import random

    from tileccl_amd import primitives as prim

    rng = random.Random(seed)
    for _ in range(12):
        world = rng.choice([2, 3, 4, 5, 8])
        heaps = heaps_of(world, 32 << 20)
        try:
            for call in range(6):
                dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
                per_unit = 16 // (2 if dtype != torch.float32 else 4)
                block = per_unit * rng.randint(1, 3000)
                chunk = rng.choice([None, per_unit * rng.randint(1, 400)])
                slots = rng.choice([None, rng.randint(1, 9)])
                how = dict(chunk_elems=chunk, pipeline_slots=slots)
                op = rng.choice(["allreduce", "allgather", "reduce_scatter", "broadcast", "scatter"])
                root = rng.randrange(world)
                tag = (seed, world, call, op, dtype, block, chunk, slots, root)
                if op == "allreduce":
                    cpu = [seeded((block,), 7 * call + r, dtype) for r in range(world)]
                    ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
                    fault = prim.allreduce_staged(ts, heaps, **how)
                    want, got = oracle.allreduce_staged(cpu), ts
                    # The reference adds in the tensor dtype, own values first (a different order on every rank):
                    # this build's bits (checked exactly below) stay within rounding of what it would leave.
                    bound = oracle.rounding_bound(cpu, world - 1)
                    for r, theirs in enumerate(oracle.allreduce_staged_reference_order(cpu)):
                        assert torch.all((want[r].float() - theirs.float()).abs() <= bound), (tag, r)
                elif op == "allgather":
                    cpu = [seeded((block,), 7 * call + r, dtype) for r in range(world)]
                    ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
                    got = [h.allocate_tensor((world * block,), dtype) for h in heaps]
                    fault = prim.allgather_staged(ts, got, heaps, **how)
                    want = oracle.allgather(cpu)
                elif op == "reduce_scatter":
                    cpu = [seeded((world * block,), 7 * call + r, dtype) for r in range(world)]
                    ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
                    got = [h.allocate_tensor((block,), dtype) for h in heaps]
                    fault = prim.reduce_scatter_staged(ts, got, heaps, **how)
                    want = oracle.reduce_scatter(cpu, dtype)
                elif op == "broadcast":
                    cpu = [seeded((block,), 7 * call + r, dtype) for r in range(world)]
                    got = [into_heap(h, c) for h, c in zip(heaps, cpu)]
                    fault = prim.broadcast_staged(got, heaps, root=root, **how)
                    want = oracle.broadcast(cpu, root)
                else:
                    cpu = [seeded((world * block,), 7 * call + r, dtype) for r in range(world)]
                    ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
                    got = [h.allocate_tensor((block,), dtype) for h in heaps]
                    fault = prim.scatter_staged(ts, got, heaps, root=root, **how)
                    want = oracle.scatter(cpu[root], world)
                torch.cuda.synchronize()
                assert int(fault.item()) == 0, tag
                for r in range(world):
                    assert torch.equal(raw(got[r]).cpu(), raw(want[r])), (tag, r)
        finally:
            close(heaps)


def test_staged_collectives_world_one_and_contracts(lib):
    from tileccl_amd.primitives import allgather_staged, broadcast_staged, reduce_scatter_staged, scatter_staged

    solo = heaps_of(1)
    try:
        t = into_heap(solo[0], seeded((64,), 1))
        o = solo[0].allocate_tensor((64,), torch.float16)
        for fn in (allgather_staged, reduce_scatter_staged, scatter_staged):
            o.zero_()
            fn([t], [o], solo)
            torch.cuda.synchronize()
            assert torch.equal(o, t)
        broadcast_staged([t], solo)
    finally:
        close(solo)
    heaps = heaps_of(2)
    try:
        a = [h.allocate_tensor((64,), torch.float16) for h in heaps]
        b = [h.allocate_tensor((128,), torch.float16) for h in heaps]
        with pytest.raises(ValueError, match="allgather output.numel must equal"):
            allgather_staged(b, a, heaps)
        with pytest.raises(ValueError, match="root=2 out of range"):
            broadcast_staged(a, heaps, root=2)
        with pytest.raises(ValueError, match="reduce_scatter tensor.numel must equal"):
            reduce_scatter_staged(a, b, heaps)
        with pytest.raises(ValueError, match="Only op='sum'"):
            reduce_scatter_staged(b, a, heaps, op="max")
        with pytest.raises(ValueError, match="one output and one heap per rank"):
            scatter_staged(b, a[:1], heaps)
    finally:
        close(heaps)


def test_staged_allreduce_integer_valued_sums_are_exact(lib):
    """A check that does not go through the oracle: small integers add exactly in every order and type."""
    from tileccl_amd.primitives import allreduce_staged

    world, numel = 4, 5 * 4096
    heaps = heaps_of(world)
    try:
        g = torch.Generator().manual_seed(5)
        cpu = [torch.randint(-60, 60, (numel,), generator=g).to(torch.float16) for _ in range(world)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        allreduce_staged(ts, heaps, chunk_elems=4096, pipeline_slots=3)
        torch.cuda.synchronize()
        total = sum(c.long() for c in cpu)
        for t in ts:
            assert torch.equal(t.cpu().long(), total)
    finally:
        close(heaps)


def test_staged_allreduce_missing_role_times_out_and_reports(lib):
    """Only rank 0's role is launched: its wait for rank 1's epoch runs into the (tiny) bound,
    the fault word is raised, the kernel exits, and rank 0's tensor is left as it was."""
    from tileccl_amd.primitives import allreduce_staged

    heaps = heaps_of(2)
    try:
        cpu = [seeded((4096,), 90 + r, torch.float16) for r in range(2)]
        ts = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        fault = allreduce_staged(ts, heaps, ranks=(0,), spin_limit_ns=200_000)
        torch.cuda.synchronize()
        assert int(fault.item()) != 0
        assert torch.equal(bits(ts[0]).cpu(), bits(cpu[0]))
        assert torch.equal(bits(ts[1]).cpu(), bits(cpu[1]))
    finally:
        close(heaps)


def test_staged_allreduce_contracts(lib):
    from tileccl_amd.primitives import allreduce_staged

    heaps = heaps_of(2)
    try:
        a = [h.allocate_tensor((64,), torch.float16) for h in heaps]
        with pytest.raises(ValueError, match="Only op='sum'"):
            allreduce_staged(a, heaps, op="max")
        with pytest.raises(ValueError, match="one tensor and one heap per rank"):
            allreduce_staged(a[:1], heaps)
        with pytest.raises(ValueError, match="chunk_elems=12 must be a positive multiple of 8"):
            allreduce_staged(a, heaps, chunk_elems=12)
        extra = heaps[1].allocate_tensor((64,), torch.float16)  # rank 1's heap is now one allocation ahead
        b = [heaps[0].allocate_tensor((64,), torch.float16), heaps[1].allocate_tensor((64,), torch.float16)]
        with pytest.raises(ValueError, match="same heap offset"):
            allreduce_staged(b, heaps)
        del extra
        ints = [h.allocate_tensor((64,), torch.int32) for h in heaps]
        with pytest.raises(ValueError):
            allreduce_staged(ints, heaps)
    finally:
        close(heaps)


def test_put_and_get_move_one_block(lib):
    from tileccl_amd.primitives import copy_block, get, put

    heaps = heaps_of(3)
    try:
        cpu = [seeded((4, 256), 50 + r) for r in range(3)]
        a = [into_heap(h, c) for h, c in zip(heaps, cpu)]
        b = [h.allocate_tensor((4, 256), torch.float16) for h in heaps]
        for t in b:
            t.fill_(0)
        put(a[0], b[0], heaps[0], dst_rank=2)  # rank 0's a -> rank 2's b
        torch.cuda.synchronize()
        assert torch.equal(b[2].cpu(), cpu[0]) and not b[0].any() and not b[1].any()
        get(b[1], a[1], heaps[1], from_rank=2)  # rank 2's a -> rank 1's b
        torch.cuda.synchronize()
        assert torch.equal(b[1].cpu(), cpu[2])
        copy_block(b[0], a[0], heaps[0], src_rank=1, dst_ranks=(0, 1, 2))  # rank 1's a -> everyone's b
        torch.cuda.synchronize()
        for t in b:
            assert torch.equal(t.cpu(), cpu[1])
        for t, c in zip(a, cpu):
            assert torch.equal(t.cpu(), c)
    finally:
        close(heaps)


def test_contracts_raise_before_any_launch(lib):
    from tileccl_amd import primitives as P

    heaps = heaps_of(2)
    try:
        h = heaps[0]
        t = h.allocate_tensor((64,), torch.float16)
        o = h.allocate_tensor((128,), torch.float16)
        with pytest.raises(ValueError, match=r"allgather output.numel must equal tensor.numel \* world_size: 64 != 64 \* 2"):
            P.allgather(t, t, h)
        with pytest.raises(ValueError, match=r"scatter tensor.numel must equal output.numel \* world_size: 64 != 128 \* 2"):
            P.scatter(t, o, h)
        with pytest.raises(ValueError, match=r"root=2 out of range \[0, 2\)"):
            P.broadcast(t, h, root=2)
        with pytest.raises(ValueError, match="Only op='sum' is currently supported, got 'max'"):
            P.reduce_scatter(o, t, h, op="max")
        with pytest.raises(ValueError, match="implementation must be one of"):
            P.reduce_scatter(o, t, h, implementation="fast")
        with pytest.raises(ValueError, match="output must reside in the provided SymmetricHeap for rank 0"):
            P.allgather(t, torch.zeros(128, dtype=torch.float16, device="cuda"), h)
        with pytest.raises(ValueError, match="allgather currently requires tensor to be contiguous"):
            P.allgather(o.view(64, 2)[:, 0], o, h)
        with pytest.raises(ValueError, match="not a multiple of 16 bytes"):
            P.allgather(t[:4], t[:8], h)
        with pytest.raises(ValueError, match="allreduce supports fp16, bf16 and fp32"):
            P.allreduce(h.allocate_tensor((64,), torch.int32), h)
        with pytest.raises(ValueError, match="writes fp16 or bf16"):
            P.reduce_scatter(o, h.allocate_tensor((64,), torch.float32), h)
        with pytest.raises(ValueError, match="dst_rank=5 out of range"):
            P.put(t, t, h, dst_rank=5)
    finally:
        close(heaps)


def test_copy_block_pitched_rectangle_through_the_c_abi(lib):
    """Rows with different pitches on the two sides, a column offset, and two targets: only the
    rectangle changes, byte for byte."""
    import ctypes as C

    from tileccl_amd import _launch, _lib

    heaps = heaps_of(3)
    try:
        g = torch.Generator().manual_seed(7)
        src_cpu = [torch.randint(0, 255, (64, 256), dtype=torch.uint8, generator=g) for _ in range(3)]
        src = [into_heap(h, c) for h, c in zip(heaps, src_cpu)]
        dst = [h.allocate_tensor((64, 512), torch.uint8) for h in heaps]
        for t in dst:
            t.fill_(7)
        rows, row_bytes, r0, sc0, dc0 = 37, 160, 5, 48, 96
        view = _launch.heap_view(heaps[1].get_heap_bases(), 1, 3)  # called by rank 1
        rc = lib.tccl_copy_block(
            dst[1][r0:, dc0:].data_ptr(), 0b101, src[1][r0:, sc0:].data_ptr(), 2, rows, row_bytes, 256, 512,
            C.byref(view), _launch.stream_ptr(),
        )
        _lib.check(rc, "tccl_copy_block")
        torch.cuda.synchronize()
        want = torch.full((64, 512), 7, dtype=torch.uint8)
        want[r0:r0 + rows, dc0:dc0 + row_bytes] = src_cpu[2][r0:r0 + rows, sc0:sc0 + row_bytes]  # read in slice 2
        assert torch.equal(dst[0].cpu(), want) and torch.equal(dst[2].cpu(), want)
        assert torch.all(dst[1] == 7)  # the caller's own slice was not a target
    finally:
        close(heaps)
