"""AllGather -> GEMM -> scatter (``ChainedAGGemmRSPattern``) on the HIP kernels against the CPU
oracle: the gathered input is bit-exact, the product is within the GEMM tolerance, and every
peer's output holds the computing rank's bytes."""

import ctypes as C

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, seeded

pytestmark = pytest.mark.gpu

SCHEDULES = ["bulk_sync", "wg_specialized", "tile_group"]


def contexts(world, heap_bytes=256 << 20):
    import tileccl_amd as tileccl

    return tileccl.init_local(world_size=world, heap_size=heap_bytes)


def put(ctx, cpu):
    t = ctx.zeros(*cpu.shape, dtype=cpu.dtype)
    t.copy_(cpu)
    return t


@pytest.mark.parametrize("schedule", SCHEDULES)
@pytest.mark.parametrize("world,M,Ks,N,dtype", [
    (1, 256, 64, 256, torch.float16),      # one rank: the gather is a plain copy, nothing is scattered
    (2, 512, 128, 512, torch.float16),
    (3, 300, 72, 264, torch.float16),      # ragged rows, K_shard not a multiple of the K step
    (2, 4096, 512, 4096, torch.bfloat16),  # large-tile kernel: the one-launch schedules read the shards in place
    (3, 2048, 192, 4096, torch.float16),   # the same with three shards of three K steps each, odd step count
    (2, 2048, 96, 4096, torch.float16),    # large-tile kernel, shards that are not whole K steps: gathered first
])
def test_chained_matches_the_oracle(lib, schedule, world, M, Ks, N, dtype):
    from tileccl_amd.patterns.chained_ag_gemm_rs import ChainedAGGemmRSPattern

    ctxs = contexts(world)
    try:
        K = Ks * world
        shards_cpu = [seeded((M, Ks), 10 + p, dtype) for p in range(world)]
        W_cpu = seeded((K, N), 1, dtype, scale=K**-0.5)
        shards = [put(c, s) for c, s in zip(ctxs, shards_cpu)]
        Ws = [put(c, W_cpu) for c in ctxs]
        outs = [c.zeros(M, N, dtype=dtype) for c in ctxs]
        rank = world - 1
        pattern = ChainedAGGemmRSPattern(ctxs[rank], schedule=schedule)
        got = pattern.execute(shards[rank], Ws[rank], outs[rank])
        pattern.check_faults()
        torch.cuda.synchronize()
        assert got is outs[rank]
        gathered = ctxs[rank].workspace("chained_ag_gemm_rs.gathered_input", M, K, dtype=dtype)
        want_gathered = oracle.gather_cols(shards_cpu)
        assert torch.equal(bits(gathered).cpu(), bits(want_gathered))
        assert_gemm_close(outs[rank], want_gathered.float() @ W_cpu.float(), tight=0.004 if dtype == torch.float16 else 0.032)
        for q in range(world):  # the scatter stage: every peer holds the computing rank's bytes
            assert torch.equal(bits(outs[q]), bits(outs[rank])), q
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_gather_cols_alone_with_a_padded_workspace(lib):
    """tccl_gather_cols through the C ABI: leading dimensions larger than the rows, three ranks."""
    from tileccl_amd import _launch, _lib

    world, M, Ks = 3, 130, 40
    ctxs = contexts(world, 64 << 20)
    try:
        shards_cpu = [seeded((M, Ks + 8), 20 + p) for p in range(world)]  # rows padded by 8 elements
        shards = [put(c, s) for c, s in zip(ctxs, shards_cpu)]
        for rank in range(world):
            gathered = ctxs[rank].zeros(M, world * Ks + 16, dtype=torch.float16)
            gathered.fill_(-7.0)
            view = _launch.heap_view(ctxs[rank].heap_bases, rank, world)
            rc = _lib.load().tccl_gather_cols(
                _launch.ptr(gathered), gathered.stride(0), _launch.ptr(shards[rank]), shards[rank].stride(0), M, Ks, 2,
                C.byref(view), None, _launch.stream_ptr(),
            )
            _lib.check(rc, "tccl_gather_cols")
            torch.cuda.synchronize()
            want = oracle.gather_cols([s[:, :Ks] for s in shards_cpu])
            assert torch.equal(bits(gathered[:, : world * Ks]).cpu(), bits(want))
            assert torch.all(gathered[:, world * Ks:] == -7.0)  # the padding is left alone
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_argument_errors(lib):
    from tileccl_amd.patterns.chained_ag_gemm_rs import ChainedAGGemmRSPattern

    ctxs = contexts(2, 64 << 20)
    try:
        shard = ctxs[0].zeros(128, 64, dtype=torch.float16)
        W = ctxs[0].zeros(192, 128, dtype=torch.float16)
        out = ctxs[0].zeros(128, 128, dtype=torch.float16)
        with pytest.raises(ValueError, match=r"input_shard columns \(64\) \* world_size \(2\) != W rows \(192\)"):
            ChainedAGGemmRSPattern(ctxs[0]).execute(shard, W, out)
        with pytest.raises(ValueError, match="unknown schedule"):
            ChainedAGGemmRSPattern(ctxs[0], schedule="ring")
        off_heap = torch.zeros(128, 64, dtype=torch.float16, device="cuda")
        W2 = ctxs[0].zeros(128, 128, dtype=torch.float16)
        with pytest.raises(ValueError, match="input_shard must live in the symmetric heap"):
            ChainedAGGemmRSPattern(ctxs[0]).execute(off_heap, W2, out)
    finally:
        for c in ctxs:
            c.heap.cleanup()
