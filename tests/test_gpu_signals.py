"""Device signal primitives, one launch each (reference tileccl/sync/primitives.py:357-500,
tileccl_v2/ipc.py:137-254), and the host-forced time-out of a fused launch."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def heap(lib):
    from tileccl_amd.v2 import SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    yield heaps[0]
    for h in heaps:
        h.cleanup()


def test_signal_wait_poll_semantics(heap):
    from tileccl_amd.v2 import ipc

    w = heap.allocate_signal_buffer(8)
    assert ipc.tile_try_wait(w, 3, MAX_SPINS=16) == 0  # nothing signalled: bounded, returns 0
    ipc.tile_signal(w, 3)
    assert w.tolist() == [0, 0, 0, 1, 0, 0, 0, 0]
    assert ipc.tile_try_poll(w, 3) == 1 and w[3].item() == 1  # poll observes, does not consume
    assert ipc.tile_try_wait(w, 3) == 1 and w[3].item() == 0  # wait consumes 1 -> 0
    assert ipc.tile_try_wait(w, 3, MAX_SPINS=4) == 0  # consumed
    ipc.tile_signal(w, 3)
    ipc.tile_signal(w, 3)  # signalling twice is still "1"
    assert w[3].item() == 1
    ipc.tile_poll(w, 3)  # set: returns, flag untouched
    assert w[3].item() == 1
    ipc.tile_wait(w, 3)  # consumes
    assert w[3].item() == 0
    with pytest.raises(RuntimeError, match=r"tile_wait: locks\[3\] was not signalled within 8 probes"):
        ipc.tile_wait(w, 3, max_spins=8)
    with pytest.raises(RuntimeError, match="tile_poll"):
        ipc.tile_poll(w, 3, max_spins=8)


def test_counter_semantics(heap):
    from tileccl_amd.v2 import ipc

    w = heap.allocate_signal_buffer(8)
    assert ipc.tile_signal_add(w, 5, 7) == 0 and ipc.tile_signal_add(w, 5, 2) == 7
    assert w[5].item() == 9
    assert ipc.tile_wait_ge(w, 5, 9) == 1 and w[5].item() == 9  # reading does not modify
    assert ipc.tile_wait_ge(w, 5, 10, spin_limit_ns=100_000) == 0  # host-chosen bound expires


def test_translate_ptr_host(heap):
    from tileccl_amd.v2 import ipc

    bases = heap.get_heap_bases()
    t = heap.allocate_tensor((16,))
    assert ipc.translate_ptr(t.data_ptr(), 0, 1, bases) == heap.translate(t.data_ptr(), 1)
    assert ipc.translate_ptr(ipc.translate_ptr(t.data_ptr(), 0, 1, bases), 1, 0, bases) == t.data_ptr()


@pytest.mark.parametrize("macro", [128, 256])
def test_fused_launch_times_out_cleanly_when_a_peer_never_signals(lib, macro):
    """Pull from a peer whose counters stay at zero: every communication workgroup gives up
    after the (tiny, host-set) spin limit, the kernel ends normally and the host raises."""
    from tests.gpu_util import into_heap, seeded
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        op = FusedGemmAllGather(heaps[0], 256, 256, torch.float16, directions="pull", spin_limit_ns=200_000,
                                macro_tile=macro)
        FusedGemmAllGather(heaps[1], 256, 256, torch.float16)  # same allocation sequence on the peer
        A, B = into_heap(heaps[0], seeded((256, 64), 0)), into_heap(heaps[0], seeded((64, 256), 1))
        op(A, B, "s2")
        with pytest.raises(RuntimeError, match="gave up waiting"):
            op.check_faults()
        # the GEMM part is unaffected
        ref = A.float().cpu() @ B.float().cpu()
        assert torch.allclose(op.out[:256].float().cpu(), ref, rtol=1e-2, atol=1e-1)
        # once the peer is marked ready the same launch succeeds
        op.mark_peers_ready()
        op(A, B, "s2")
        op.check_faults()
    finally:
        for h in heaps:
            h.cleanup()
