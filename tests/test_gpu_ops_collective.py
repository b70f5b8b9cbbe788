"""``tileccl.ops.gemm_allgather`` / ``gemm_reducescatter`` (column shards) on the HIP kernels,
against the CPU oracle; world size 2 and 3 emulated as slices of one arena."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, seeded

pytestmark = pytest.mark.gpu


def contexts(world, heap_bytes=128 << 20):
    import tileccl_amd as tileccl

    return tileccl.init_local(world_size=world, heap_size=heap_bytes)


def put(ctx, cpu):
    t = ctx.zeros(*cpu.shape, dtype=cpu.dtype)
    t.copy_(cpu)
    return t


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("world,M,N,K", [(2, 512, 512, 256), (3, 300, 768, 72), (2, 4096, 4096, 512)])
def test_gemm_allgather_column_shards(lib, variant, world, M, N, K):
    import tileccl_amd as tileccl

    ctxs = contexts(world, 256 << 20)
    try:
        Ns = N // world
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        As = [put(c, A_cpu) for c in ctxs]
        Bs = [put(c, B_cpu[:, r * Ns:(r + 1) * Ns].contiguous()) for r, c in enumerate(ctxs)]
        Cs = [c.zeros(M, N, dtype=torch.float16) for c in ctxs]
        for r, c in enumerate(ctxs):
            out = tileccl.ops.gemm_allgather(As[r], Bs[r], Cs[r], ctx=c, variant=variant)
            assert out is Cs[r]
        torch.cuda.synchronize()
        # every rank holds the same full product, bit for bit
        for r in range(1, world):
            assert torch.equal(bits(Cs[0]), bits(Cs[r]))
        assert_gemm_close(Cs[0], A_cpu.float() @ B_cpu.float(), tight=0.004)
        # each column block is the bytes its owner's GEMM produced: compare with the oracle per block
        for r in range(world):
            want = oracle.gemm(A_cpu, B_cpu[:, r * Ns:(r + 1) * Ns], torch.float16)
            assert (Cs[0][:, r * Ns:(r + 1) * Ns].cpu().float() - want.float()).abs().max().item() <= 0.004
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
def test_gemm_reducescatter_without_the_resident_peers_promise(lib, variant):
    """``peers_resident=False``: the launch waits for the peers' words instead of trusting that their partials are
    there.  On a fresh context rank 0 runs first and finds no producer: its bounded wait expires and the fault word is
    raised (with the promise it would have summed zeros silently).  Rank 1, run after it, finds rank 0's words at the
    same launch number and its output is the sum of both partials."""
    import tileccl_amd as tileccl
    from tileccl_amd import ops_collective

    world, M, N, K = 2, 512, 1024, 128
    ctxs = contexts(world, 256 << 20)
    try:
        Ns = N // world
        A_cpu = [seeded((M, K), 10 + r) for r in range(world)]
        B_cpu = seeded((K, N), 1, scale=K**-0.5)
        As = [put(c, A_cpu[r]) for r, c in enumerate(ctxs)]
        Bs = [put(c, B_cpu) for c in ctxs]
        Cs = [c.zeros(M, Ns, dtype=torch.float16) for c in ctxs]
        words = [ops_collective._reduce_scatter_words(c, world, M, Ns) for c in ctxs]
        for w in words:
            w.spin_limit_ns = 300_000
        tileccl.ops.gemm_reducescatter(As[0], Bs[0], Cs[0], ctx=ctxs[0], variant=variant, peers_resident=False)
        torch.cuda.synchronize()
        with pytest.raises(RuntimeError, match="gave up waiting"):
            words[0].raise_if_faulted()
        tileccl.ops.gemm_reducescatter(As[1], Bs[1], Cs[1], ctx=ctxs[1], variant=variant, peers_resident=False)
        torch.cuda.synchronize()
        words[1].raise_if_faulted()
        full = sum(a.float() @ B_cpu.float() for a in A_cpu)
        assert_gemm_close(Cs[1], full[:, Ns:], tight=0.006)
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("world,M,N,K", [(2, 512, 512, 256), (2, 200, 272, 72), (3, 256, 768, 128), (2, 2048, 4096, 512),
                                         (3, 768, 1536, 192)])
def test_gemm_reducescatter_column_shards(lib, variant, world, M, N, K):
    """One fused launch per rank (GEMM over the stacked column blocks + reduction of the own
    block), M = 200 being the shape that falls back to one GEMM per block plus the bulk
    reduction.  First with every partial stored, so that the oracle can reduce the very
    partials the GPU produced (bit-exact for two ranks); then in the default mode, where the
    own block's partial stays in the accumulators: same output bytes."""
    import tileccl_amd as tileccl

    ctxs = contexts(world, 256 << 20)
    try:
        Ns = N // world
        A_cpu = [seeded((M, K), 10 + r) for r in range(world)]
        B_cpu = seeded((K, N), 1, scale=K**-0.5)
        As = [put(c, A_cpu[r]) for r, c in enumerate(ctxs)]
        Bs = [put(c, B_cpu) for c in ctxs]
        Cs = [c.zeros(M, Ns, dtype=torch.float16) for c in ctxs]
        # Emulation: a rank's partial is resident once its op has run, so run the round twice;
        # after the second round every rank has reduced over final partials.
        for _ in range(2):
            for r, c in enumerate(ctxs):
                out = tileccl.ops.gemm_reducescatter(As[r], Bs[r], Cs[r], ctx=c, variant=variant, own_rows_in_registers=False)
                assert out is Cs[r]
        torch.cuda.synchronize()
        full = sum(a.float() @ B_cpu.float() for a in A_cpu)
        partials = [c.workspace("gemm_reducescatter.partial", world, M, Ns, dtype=torch.float32).cpu() for c in ctxs]
        stored = [t.clone() for t in Cs]
        for r in range(world):
            assert_gemm_close(Cs[r], full[:, r * Ns:(r + 1) * Ns], tight=0.006)
            for q in range(world):  # block q of rank r's workspace is A_r @ B[:, q's columns]
                assert_gemm_close(partials[r][q], A_cpu[r].float() @ B_cpu[:, q * Ns:(q + 1) * Ns].float(), tight=1e-3)
            # bit-exact against the oracle's reduction of the partials the GPU produced
            tall = [p.reshape(world * M, Ns) for p in partials]
            want = oracle.reduce_rows(tall, r, torch.float16)
            if world == 2:
                assert torch.equal(bits(Cs[r]).cpu(), bits(want))
            else:
                assert (Cs[r].cpu().float() - want.float()).abs().max().item() <= 0.002
        # Default mode: the own block's partial is never stored; the peers' blocks are.
        for r, c in enumerate(ctxs):
            c.workspace("gemm_reducescatter.partial", world, M, Ns, dtype=torch.float32)[r].fill_(-3.0)
            Cs[r].zero_()
        for r, c in enumerate(ctxs):
            tileccl.ops.gemm_reducescatter(As[r], Bs[r], Cs[r], ctx=c, variant=variant)
        torch.cuda.synchronize()
        fused = M % 128 == 0 and variant != "s0"
        for r, c in enumerate(ctxs):
            assert torch.equal(bits(Cs[r]), bits(stored[r])), r
            mine = c.workspace("gemm_reducescatter.partial", world, M, Ns, dtype=torch.float32)
            # the large-tile kernel (chosen from 128 tiles of 256 x 256 on) is the one that keeps rows in registers
            macro = M % 256 == 0 and -(-world * M // 256) * -(-Ns // 256) * 2 >= 256
            if fused and macro:
                assert torch.all(mine[r] == -3.0), r
            for q in range(world):
                if q != r:
                    assert torch.equal(mine[q].cpu(), partials[r][q]), (r, q)
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_contract_errors(lib):
    import tileccl_amd as tileccl

    ctxs = contexts(2, 16 << 20)
    try:
        c = ctxs[0]
        A, B, Cf = c.zeros(128, 64, dtype=torch.float16), c.zeros(64, 128, dtype=torch.float16), c.zeros(128, 256, dtype=torch.float16)
        with pytest.raises(ValueError, match=r"gemm_allgather expects 2-D tensors: got A.ndim=1"):
            tileccl.ops.gemm_allgather(A[0], B, Cf, ctx=c)
        with pytest.raises(ValueError, match="RHS shard columns must match the rank-local shard width: expected 128, got 64"):
            tileccl.ops.gemm_allgather(A, B[:, :64].contiguous(), Cf, ctx=c)
        with pytest.raises(ValueError, match=r"requires C.shape\[1\] to be divisible by world_size: 255 % 2 != 0"):
            tileccl.ops.gemm_allgather(A, B, c.zeros(128, 255, dtype=torch.float16), ctx=c)
        with pytest.raises(ValueError, match="share one dtype"):
            tileccl.ops.gemm_allgather(A, B, c.zeros(128, 256, dtype=torch.bfloat16), ctx=c)
        with pytest.raises(ValueError, match="C must reside in the attached symmetric heap"):
            tileccl.ops.gemm_allgather(A, B, torch.zeros(128, 256, dtype=torch.float16, device="cuda"), ctx=c)
        with pytest.raises(ValueError, match="unknown variant 's7'"):
            tileccl.ops.gemm_allgather(A, B, Cf, ctx=c, variant="s7")
        Bf = c.zeros(64, 256, dtype=torch.float16)
        with pytest.raises(ValueError, match="output columns must match the rank-local shard width: expected 128, got 256"):
            tileccl.ops.gemm_reducescatter(A, Bf, Cf, ctx=c)
        with pytest.raises(ValueError, match=r"B.shape\[0\] must equal A.shape\[1\]: got 32 vs 64"):
            tileccl.ops.gemm_reducescatter(A, Bf[:32], c.zeros(128, 128, dtype=torch.float16), ctx=c)
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_ops_level_collectives_and_their_plans(lib):
    """tileccl.ops.allgather / allreduce / reduce_scatter (reference ops.py:1083-1258): the same results
    as the launchers underneath, plans that can be executed again, and validation that notices a tensor
    the plan was not built for."""
    import tileccl_amd as tileccl

    world, block = 3, 2048
    ctxs = contexts(world, 64 << 20)
    try:
        cpu = [seeded((block,), 50 + r) for r in range(world)]
        srcs = [put(c, t) for c, t in zip(ctxs, cpu)]
        outs = [c.zeros(world * block, dtype=torch.float16) for c in ctxs]
        for r, c in enumerate(ctxs):
            assert tileccl.ops.allgather(srcs[r], outs[r], ctx=c) is outs[r]
        torch.cuda.synchronize()
        for r, want in enumerate(oracle.allgather(cpu)):
            assert torch.equal(bits(outs[r]).cpu(), bits(want))

        wide = [seeded((world * block,), 60 + r) for r in range(world)]
        ins = [put(c, t) for c, t in zip(ctxs, wide)]
        shards = [c.zeros(block, dtype=torch.float16) for c in ctxs]
        plans = [tileccl.ops.build_reduce_scatter_plan(ins[r], shards[r], ctx=c) for r, c in enumerate(ctxs)]
        assert plans[0].to_dict()["block_size"] == block and plans[0].to_dict()["context"]["world_size"] == world
        for _ in range(2):  # a plan is reusable
            for r, plan in enumerate(plans):
                plan.execute(ins[r], shards[r])
        torch.cuda.synchronize()
        for r, want in enumerate(oracle.reduce_scatter(wide, torch.float16)):
            assert torch.equal(bits(shards[r]).cpu(), bits(want))
        with pytest.raises(ValueError, match="reduce_scatter src shape no longer matches the plan"):
            plans[0].execute(ins[0].reshape(world, block), shards[0])
        with pytest.raises(ValueError, match="reduce_scatter src.numel must equal output.numel \\* world_size"):
            tileccl.ops.reduce_scatter(srcs[0], shards[0], ctx=ctxs[0])
        with pytest.raises(ValueError, match="implementation must be one of"):
            tileccl.ops.reduce_scatter(ins[0], shards[0], ctx=ctxs[0], implementation="fast")

        xs = [put(c, t) for c, t in zip(ctxs, wide)]
        for r, c in enumerate(ctxs):
            assert tileccl.ops.allreduce(xs[r], ctx=c) is xs[r]
        torch.cuda.synchronize()
        for r, want in enumerate(oracle.allreduce(wide)):
            assert torch.equal(bits(xs[r]).cpu(), bits(want))
        with pytest.raises(ValueError, match="allreduce currently supports only op='sum'"):
            tileccl.ops.allreduce(xs[0], ctx=ctxs[0], op="max")
        with pytest.raises(ValueError, match="must reside in the attached symmetric heap"):
            tileccl.ops.allreduce(torch.zeros(block, dtype=torch.float16, device="cuda"), ctx=ctxs[0])
        with pytest.raises(ValueError, match="allgather currently requires src to be contiguous"):
            tileccl.ops.allgather(ins[0][::2], outs[0], ctx=ctxs[0])
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_ops_level_gemm_plans_and_the_chained_op(lib):
    """build_gemm_allgather_plan / build_gemm_reducescatter_plan / allgather_gemm_reducescatter
    (reference ops.py:891-1080, 2315-2375) on the fused launches."""
    import tileccl_amd as tileccl

    world, M, N, K = 2, 512, 512, 128
    ctxs = contexts(world, 128 << 20)
    try:
        Ns = N // world
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        As = [put(c, A_cpu) for c in ctxs]
        Bsh = [put(c, B_cpu[:, r * Ns:(r + 1) * Ns].contiguous()) for r, c in enumerate(ctxs)]
        Cs = [c.zeros(M, N, dtype=torch.float16) for c in ctxs]
        plans = [tileccl.ops.build_gemm_allgather_plan(As[r], Bsh[r], Cs[r], ctx=c) for r, c in enumerate(ctxs)]
        assert plans[1].to_dict()["contract"]["shard_cols"] == Ns
        for r, plan in enumerate(plans):
            assert plan.execute(As[r], Bsh[r], Cs[r]) is Cs[r]
        torch.cuda.synchronize()
        assert torch.equal(bits(Cs[0]), bits(Cs[1]))
        assert_gemm_close(Cs[0], A_cpu.float() @ B_cpu.float(), tight=0.004)
        small = [c.zeros(256, N, dtype=torch.float16) for c in ctxs]  # on every rank: the slices stay in step
        with pytest.raises(ValueError, match="Tensor contract no longer matches this GemmAllGatherPlan"):
            plans[0].execute(As[0][:256], Bsh[0], small[0])

        Bs = [put(c, B_cpu) for c in ctxs]
        shard_out = [c.zeros(M, Ns, dtype=torch.float16) for c in ctxs]
        rs = [tileccl.ops.build_gemm_reducescatter_plan(As[r], Bs[r], shard_out[r], ctx=c) for r, c in enumerate(ctxs)]
        for _ in range(2):
            for r, plan in enumerate(rs):
                plan.execute(As[r], Bs[r], shard_out[r])
        torch.cuda.synchronize()
        full = world * (A_cpu.float() @ B_cpu.float())
        for r in range(world):
            assert_gemm_close(shard_out[r], full[:, r * Ns:(r + 1) * Ns], tight=0.008)

        Ks = K // world
        shards_cpu = [seeded((M, Ks), 30 + p) for p in range(world)]
        shards = [put(c, s) for c, s in zip(ctxs, shards_cpu)]
        outs = [c.zeros(M, N, dtype=torch.float16) for c in ctxs]
        got = tileccl.ops.allgather_gemm_reducescatter(shards[1], Bs[1], outs[1], ctx=ctxs[1])
        torch.cuda.synchronize()
        assert got is outs[1]
        assert_gemm_close(outs[1], oracle.gather_cols(shards_cpu).float() @ B_cpu.float(), tight=0.004)
        with pytest.raises(ValueError, match=r"input_shard columns \(64\) \* world_size \(2\) must equal W rows \(192\)"):
            tileccl.ops.allgather_gemm_reducescatter(shards[0], ctxs[0].zeros(192, N, dtype=torch.float16), outs[0], ctx=ctxs[0])
        with pytest.raises(ValueError, match=r"output rows \(256\) must equal input_shard rows \(512\)"):
            tileccl.ops.allgather_gemm_reducescatter(shards[0], Bs[0], small[0], ctx=ctxs[0])
    finally:
        for c in ctxs:
            c.heap.cleanup()
