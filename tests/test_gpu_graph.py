"""The fused launches recorded into a HIP graph: every replay must equal the eager result.

A recorded launch replays with frozen arguments, so the TileGroup epoch cannot advance; the
counters are cleared by fill kernels recorded ahead of the launch instead.  Replays are
interleaved with eager work and synchronisations, and the inputs change between replays."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, seeded

pytestmark = pytest.mark.gpu


def _heaps(world=2, size=256 << 20):
    from tileccl_amd.v2 import SymmetricHeap

    return SymmetricHeap.create_all(size, world)


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("macro_tile", [128, 256])
def test_allgather_graph_replays_equal_eager(lib, variant, macro_tile):
    from tileccl_amd.v2.fused import FusedGemmAllGather

    M, N, K = 1024, 1024, 256
    heaps = _heaps()
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="both", macro_tile=macro_tile) for h in heaps]
        A = heaps[0].allocate_tensor((M, K), torch.float16)
        B = heaps[0].allocate_tensor((K, N), torch.float16)
        op = ops[0]
        op.mark_peers_ready()
        inputs = [(seeded((M, K), s), seeded((K, N), s + 1, scale=K**-0.5), seeded((M, N), s + 2)) for s in (0, 10, 20, 30)]

        def load(i):
            a, b, peer = inputs[i]
            A.copy_(a)
            B.copy_(b)
            ops[1].out[M:].copy_(peer)  # the peer's resident block, pulled by rank 0
            op.out.zero_()
            ops[1].out[:M].zero_()

        def check(i):
            torch.cuda.synchronize()
            a, b, peer = inputs[i]
            assert_gemm_close(op.out[:M], a.float() @ b.float(), tight=0.004)
            assert torch.equal(op.out[M:].cpu(), peer)  # pulled, byte for byte
            assert torch.equal(bits(ops[1].out[:M]), bits(op.out[:M]))  # pushed, byte for byte

        load(0)
        op(A, B, variant)  # eager warm-up (also the first-launch set-up of the library)
        op.check_faults()
        check(0)
        eager = op.out.clone()

        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            load(0)
            with torch.cuda.graph(graph, stream=side):
                op(A, B, variant)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for i in (1, 2, 3):
            load(i)
            graph.replay()
            check(i)
            op.check_faults()
            scratch = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")  # eager work in between
            torch.cuda.synchronize()
            assert scratch.isfinite().all()
        # back to the first inputs: the replay reproduces the eager bytes, and eager launches still work
        load(0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(op.out), bits(eager))
        load(1)
        op(A, B, variant)
        op.check_faults()
        check(1)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
def test_reducescatter_graph_replays_equal_eager(lib, variant):
    from tileccl_amd.v2.fused import FusedGemmReduceScatter

    M, N, K = 1024, 512, 128
    heaps = _heaps()
    try:
        ops = [FusedGemmReduceScatter(h, M, N, macro_tile=256, own_rows_in_registers=True) for h in heaps]
        A = heaps[0].allocate_tensor((M, K), torch.float16)
        B = heaps[0].allocate_tensor((K, N), torch.float16)
        op = ops[0]
        op.mark_peers_ready()
        inputs = [(seeded((M, K), s), seeded((K, N), s + 1, scale=K**-0.5), seeded((M, N), s + 2, torch.float32)) for s in (0, 10, 20)]

        def load(i):
            a, b, peer = inputs[i]
            A.copy_(a)
            B.copy_(b)
            ops[1].partial.copy_(peer)
            op.out.zero_()
            ops[1].out.zero_()

        def check(i):
            torch.cuda.synchronize()
            a, b, peer = inputs[i]
            mine = oracle.gemm(a, b, torch.float32)
            for owner in (0, 1):
                want = oracle.reduce_rows([mine, peer], owner, torch.float16)
                assert_gemm_close(ops[owner].out, want.float(), tight=0.01)

        load(0)
        op(A, B, variant)
        op.check_faults()
        check(0)
        eager = [o.out.clone() for o in ops]
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            load(0)
            with torch.cuda.graph(graph, stream=side):
                op(A, B, variant)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for i in (1, 2, 0):
            load(i)
            graph.replay()
            check(i)
            op.check_faults()
            torch.cuda.synchronize()
        for o, e in zip(ops, eager):
            assert torch.equal(bits(o.out), bits(e))
    finally:
        for h in heaps:
            h.cleanup()
