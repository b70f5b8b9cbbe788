"""Two emulated ranks whose launches run at the same time, on two streams, each waiting inside its
kernel for signal words that the other one writes while both are running.

Each launch is held to 100 workgroups (one per CU), so the two fit on the 256 CUs side by side;
nothing is preset with ``mark_peers_ready`` and nothing is emulated on a peer's behalf.  This is as
close to two GPUs as one GPU gets: a wrong threshold, a missed write-through or a stale flag shows
as a bounded wait that expires (an error from ``check_faults``) or as wrong bytes, never as a hang.

Two streams do not always run side by side: the runtime spreads its streams over a few hardware
queues, and two streams on one queue run their kernels one after the other (measured here: the
third and fourth stream of torch's pool did, the others did not).  The tests therefore first look
for a pair of streams on which a one-lane kernel that waits (20 ms at most) is released by a
kernel launched after it on the other stream, and skip if there is none."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu

import ctypes as C

WGS = 100
SPIN_NS = 300_000_000


@pytest.fixture(scope="module")
def streams(lib):
    from tileccl_amd import _launch

    pool = [torch.cuda.Stream() for _ in range(8)]
    word = torch.zeros(1, dtype=torch.int32, device="cuda")
    seen = torch.zeros(2, dtype=torch.int32, device="cuda")
    for first in pool:
        for second in pool:
            if first is second:
                continue
            word.zero_()
            seen.zero_()
            torch.cuda.synchronize()
            for a, b in ((first, second), (second, first)):  # either may be the one that waits
                rc = lib.tccl_prim_wait_ge(_launch.ptr(word), 0, 1, 20_000_000, _launch.ptr(seen), C.c_void_p(a.cuda_stream))
                assert rc == 0
                rc = lib.tccl_prim_signal_add(_launch.ptr(word), 0, 1, _launch.ptr(seen[1:]), C.c_void_p(b.cuda_stream))
                assert rc == 0
                torch.cuda.synchronize()
                if int(seen[0].item()) != 1:
                    break
                word.zero_()
                seen.zero_()
            else:
                return [first, second]
    pytest.skip("no two streams of this process run kernels side by side")



def both_at_once(ops, operands, variant, streams):
    """Rank 1's launch, then rank 0's, each on its own stream, with no host wait in between."""
    torch.cuda.synchronize()
    for rank in (1, 0):
        with torch.cuda.stream(streams[rank]):
            ops[rank](*operands[rank], variant)
    for s in streams:
        s.synchronize()
    for op in ops:
        op.check_faults()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro,M,N,K", [(256, 4096, 2048, 512), (128, 1024, 1024, 256)])
def test_all_gather_both_ranks_pull_while_the_other_produces(lib, streams, variant, macro, M, N, K):
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(256 << 20, 2)
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="pull", macro_tile=macro, num_gemm_wgs=WGS,
                                  spin_limit_ns=SPIN_NS) for h in heaps]
        for launch in range(3):  # launch numbers stay in step on both ranks; inputs change every time
            cpu = [(seeded((M, K), 10 * launch + r), seeded((K, N), 10 * launch + 5 + r, scale=K**-0.5)) for r in range(2)]
            operands = [(into_heap(heaps[r], cpu[r][0]), into_heap(heaps[r], cpu[r][1])) for r in range(2)]
            for op in ops:
                op.out.zero_()
            both_at_once(ops, operands, variant, streams)
            blocks = [ops[r].out[r * M:(r + 1) * M] for r in range(2)]  # what each rank computed itself
            for r in range(2):
                assert_gemm_close(blocks[r], cpu[r][0].float() @ cpu[r][1].float(), tight=0.004)
                other = 1 - r
                assert torch.equal(bits(ops[r].out[other * M:(other + 1) * M]), bits(blocks[other])), (launch, r)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro,own_rows,M,N,K", [(256, False, 4096, 2048, 512), (256, True, 4096, 2048, 512),
                                                  (128, False, 1024, 1024, 256)])
def test_reduce_scatter_each_rank_reduces_its_rows_from_the_others_live_partial(lib, streams, variant, macro, own_rows, M, N, K):
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    heaps = SymmetricHeap.create_all(256 << 20, 2)
    try:
        make = lambda h, **kw: FusedGemmReduceScatter(h, M, N, emulate_peer=False, macro_tile=macro, num_gemm_wgs=WGS,  # noqa: E731
                                                      spin_limit_ns=SPIN_NS, **kw)
        ops = [make(h, own_rows_in_registers=own_rows) for h in heaps]
        for launch in range(2):
            cpu = [(seeded((M, K), 20 * launch + r), seeded((K, N), 20 * launch + 5 + r, scale=K**-0.5)) for r in range(2)]
            operands = [(into_heap(heaps[r], cpu[r][0]), into_heap(heaps[r], cpu[r][1])) for r in range(2)]
            for op in ops:
                op.out.zero_()
            both_at_once(ops, operands, variant, streams)
            got = [op.out.clone() for op in ops]
            # The partials as plain GEMM launches store them (with own_rows the owned rows never reach
            # memory as a partial): same kernel, same k order, same bits.
            from tileccl_amd import _launch, _lib

            partials = []
            for r in range(2):
                full = torch.empty(M, N, dtype=torch.float32, device="cuda")
                d = _launch.gemm_desc(*operands[r], full, macro_tile=macro)
                _lib.check(_lib.load().tccl_gemm(C.byref(d), _launch.stream_ptr()), "tccl_gemm")
                torch.cuda.synchronize()
                assert_gemm_close(full, cpu[r][0].float() @ cpu[r][1].float(), tight=1e-3)
                partials.append(full.cpu())
            for r in range(2):
                want = oracle.reduce_rows(partials, r, torch.float16)
                assert torch.equal(bits(got[r]).cpu(), bits(want)), (launch, r)
    finally:
        for h in heaps:
            h.cleanup()
