"""Two emulated ranks that wait on words the other rank's launch really wrote.

Everywhere else a resident peer's words are preset (``mark_peers_ready``).  Here rank 1's
launch runs first and publishes its own ``locks`` / ``counter``; rank 0's launch then has to
find them through the heap, with the thresholds of its own launch number.  A second round
checks the other side of the rule: flags left behind by launch 1 must not satisfy launch 2
(rank 0 alone at launch 2 gives up; after rank 1's launch 2 it sees the new bytes).  Every
device-side wait is bounded, so a wrong threshold raises instead of hanging."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu

M, N, K = 1024, 768, 256
SHORT_NS = 200_000


def inputs(heap, seed):
    A_cpu, B_cpu = seeded((M, K), seed), seeded((K, N), seed + 1, scale=K**-0.5)
    return A_cpu, B_cpu, into_heap(heap, A_cpu), into_heap(heap, B_cpu)


def expect_timeout(op):
    with pytest.raises(RuntimeError, match="gave up waiting"):
        op.check_faults()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro", [128, 256])
def test_allgather_pull_follows_the_peers_own_launch(lib, variant, macro):
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        puller = FusedGemmAllGather(heaps[0], M, N, torch.float16, directions="pull", macro_tile=macro)
        pusher = FusedGemmAllGather(heaps[1], M, N, torch.float16, directions="push", macro_tile=macro)
        A0_cpu, B0_cpu, A0, B0 = inputs(heaps[0], 0)
        for o in (puller, pusher):
            o.out.zero_()

        def round_trip(seed):
            A1_cpu, B1_cpu, A1, B1 = inputs(heaps[1], seed)
            pusher(A1, B1, variant)  # publishes rank 1's words; nothing to wait for
            pusher.check_faults()
            block = pusher.out[M:].clone()
            assert_gemm_close(block, A1_cpu.float() @ B1_cpu.float(), tight=0.004)
            assert torch.equal(bits(puller.out[M:]), bits(block))  # the push has delivered it already ...
            puller.out[M:].zero_()  # ... so it is wiped: what is there afterwards, the pull has brought
            puller(A0, B0, variant)
            puller.check_faults()
            assert torch.equal(bits(puller.out[M:]), bits(block))
            assert_gemm_close(puller.out[:M], A0_cpu.float() @ B0_cpu.float(), tight=0.004)
            assert torch.count_nonzero(pusher.out[:M]).item() == 0  # rank 0 pushes nothing
            return block

        first = round_trip(10)
        # Launch 2 of rank 0 alone: rank 1's words still say "launch 1".
        puller.words.spin_limit_ns = SHORT_NS
        puller.out[M:].zero_()
        puller(A0, B0, variant)
        expect_timeout(puller)
        puller.words.spin_limit_ns = pusher.words.spin_limit_ns
        # Both ranks back in step; rank 1 has new inputs, and the new bytes must arrive.
        puller.words.reset()
        pusher.words.reset()
        second = round_trip(20)
        assert not torch.equal(bits(first), bits(second))
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro,own_rows", [(128, False), (256, False), (256, True)])
def test_reduce_scatter_waits_for_the_peers_published_partial(lib, variant, macro, own_rows):
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        kw = dict(emulate_peer=False, macro_tile=macro, own_rows_in_registers=own_rows)
        mine = FusedGemmReduceScatter(heaps[0], M, N, **kw)
        peer = FusedGemmReduceScatter(heaps[1], M, N, spin_limit_ns=SHORT_NS, **kw)
        A0_cpu, B0_cpu, A0, B0 = inputs(heaps[0], 0)

        def round_trip(seed):
            A1_cpu, B1_cpu, A1, B1 = inputs(heaps[1], seed)
            # Rank 1 stores and publishes its partial, then waits for rank 0's partial of its own
            # rows, which does not exist yet: the bounded wait expires, the partial is complete.
            peer(A1, B1, variant)
            expect_timeout(peer)
            assert_gemm_close(peer.partial, A1_cpu.float() @ B1_cpu.float(), tight=1e-3)
            # Reference bytes: rank 0's bulk variant (no waiting, whole partial stored).
            mine.out.zero_()
            mine(A0, B0, "s0")
            mine.check_faults()
            want = oracle.reduce_rows([mine.partial.cpu(), peer.partial.cpu()], 0, torch.float16)
            assert torch.equal(bits(mine.out).cpu(), bits(want))
            mine.out.zero_()
            mine(A0, B0, variant)  # waits on rank 1's locks / counters of the launch above
            mine.check_faults()
            assert torch.equal(bits(mine.out).cpu(), bits(want))
            return want

        first = round_trip(10)
        # Launch 2 of rank 0 alone must not accept rank 1's launch-1 flags.
        mine.words.spin_limit_ns = SHORT_NS
        mine(A0, B0, variant)
        expect_timeout(mine)
        mine.words.spin_limit_ns = 2_000_000_000
        mine.words.reset()
        peer.words.reset()
        second = round_trip(20)
        assert not torch.equal(bits(first), bits(second))
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("macro", [128, 256])
def test_tile_flags_carry_the_launch_number(lib, macro):
    """Two tile-by-tile launches in a row: after launch e every lock holds e, nothing older and
    nothing consumed, so a reader of launch e+1 cannot mistake them for its own."""
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="push", macro_tile=macro) for h in heaps]
        _, _, A, B = inputs(heaps[0], 0)
        for e in (1, 2, 3):
            ops[0](A, B, "s1")
            ops[0].check_faults()
            assert ops[0].words.lock_epoch == e
            assert ops[0].locks.tolist() == [e] * ops[0].locks.numel()
        assert ops[0].words.epoch == 0 and ops[0].signals.counter.tolist() == [0] * ops[0].plan.n_groups
    finally:
        for h in heaps:
            h.cleanup()
