"""B handed over k-major -- the `.t()` view of an (N, K) tensor, a linear layer's weight layout,
which the reference's stride-taking kernels accept (kernels/gemm.py:139-151) -- through every fused
operation.  The order in which k is summed does not depend on B's layout, so every output byte of
every rank must equal the row-major run's (which the other test files hold to the oracle)."""

import pytest
import torch

from tests.gpu_util import bits, into_heap, seeded

pytestmark = pytest.mark.gpu

F8 = torch.float8_e4m3fn


def weight_view(heap, B_cpu, pad=0):
    """B in `heap` as the transposed view of an (N, K + pad) tensor."""
    K, N = B_cpu.shape
    backing = heap.allocate_tensor((N, K + pad), B_cpu.dtype)
    backing.view(torch.int8 if B_cpu.element_size() == 1 else torch.int16).zero_()
    view = backing[:, :K].t()
    view.copy_(B_cpu)
    assert view.stride() == (1, K + pad) or K == 1
    return view


def both_layouts(heap, B_cpu, pad=0):
    return [into_heap(heap, B_cpu), weight_view(heap, B_cpu, pad)]


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("macro,M,N,K,pad", [(128, 512, 512, 256, 0), (256, 512, 512, 256, 8), (256, 1024, 1280, 200, 0),
                                             (0, 4096, 4096, 1024, 0)])
def test_allgather(lib, variant, macro, M, N, K, pad):
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(512 << 20, 2)
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="both", macro_tile=macro) for h in heaps]
        A = into_heap(heaps[0], seeded((M, K), 0))
        peer_block = seeded((M, N), 2)
        seen = []
        for B in both_layouts(heaps[0], seeded((K, N), 1, scale=K**-0.5), pad):
            for o in ops:
                o.out.zero_()
            ops[1].out[M:].copy_(peer_block)
            ops[0].mark_peers_ready()
            ops[0](A, B, variant)
            ops[0].check_faults()
            torch.cuda.synchronize()
            seen.append([bits(o.out).clone() for o in ops])
        assert seen[0][0].count_nonzero().item() > 0
        for r in range(2):
            assert torch.equal(seen[0][r], seen[1][r]), r
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("macro,own_rows,in_dtype,partial_dtype", [
    (128, False, torch.float16, torch.float32),
    (256, False, torch.bfloat16, torch.bfloat16),
    (256, True, torch.float16, torch.float32),
    (256, True, F8, torch.bfloat16),
    (256, False, F8, torch.bfloat16),
])
def test_reduce_scatter(lib, variant, macro, own_rows, in_dtype, partial_dtype):
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    M, N, K = 1024, 768, 320
    out_dtype = torch.float16 if partial_dtype == torch.float32 else torch.bfloat16
    heaps = SymmetricHeap.create_all(128 << 20, 2)
    try:
        ops = [FusedGemmReduceScatter(h, M, N, partial_dtype=partial_dtype, out_dtype=out_dtype, macro_tile=macro,
                                      own_rows_in_registers=own_rows) for h in heaps]
        if in_dtype == F8:
            A_cpu = (seeded((M, K), 0, torch.float32) * 64).clamp(-448, 448).to(F8)
            B_cpu = (seeded((K, N), 1, torch.float32) * 64).clamp(-448, 448).to(F8)
            scales = dict(scale_a=1 / 64, scale_b=K**-0.5 / 64)
        else:
            A_cpu, B_cpu = seeded((M, K), 0, in_dtype), seeded((K, N), 1, in_dtype, scale=K**-0.5)
            scales = {}
        A = into_heap(heaps[0], A_cpu)
        peer = seeded((M, N), 2, partial_dtype)
        seen = []
        for B in both_layouts(heaps[0], B_cpu, 16):
            ops[1].partial.copy_(peer)
            ops[0].partial.zero_()
            for o in ops:
                o.out.zero_()
            ops[0].mark_peers_ready()
            ops[0](A, B, variant, **scales)
            ops[0].check_faults()
            torch.cuda.synchronize()
            seen.append([bits(o.out).clone() for o in ops] + [bits(ops[0].partial).clone()])
        assert seen[0][0].count_nonzero().item() > 0 and seen[0][1].count_nonzero().item() > 0
        for a, b in zip(*seen):
            assert torch.equal(a, b)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 272, 80), (512, 768, 512)])
def test_fp8_gemm(lib, M, N, K):
    import ctypes as C

    from tileccl_amd import _launch, _lib

    A = (seeded((M, K), 0, torch.float32) * 64).clamp(-448, 448).to(F8).cuda()
    B_cpu = (seeded((K, N), 1, torch.float32) * 64).clamp(-448, 448).to(F8)
    backing = torch.zeros(N, K + 16, dtype=torch.int8, device="cuda").view(F8)
    backing[:, :K].view(torch.int8).copy_(B_cpu.t().contiguous().view(torch.int8))
    outs = []
    for B in (B_cpu.cuda(), backing[:, :K].t()):
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        desc = _launch.gemm_desc(A, B, out, alpha=2.0**-12)
        _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")
        torch.cuda.synchronize()
        outs.append(out)
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(bits(outs[0]), bits(outs[1]))


@pytest.mark.parametrize("pattern", ["bulk_sync", "wg_specialized", "tile_group"])
def test_ops_gemm_allscatter_with_a_weight_view(lib, pattern):
    """tileccl.ops.gemm_allscatter(x, W.t(), out): the public op, two ranks, every rank's C compared."""
    import tileccl_amd as tileccl

    M, K, N = 512, 192, 1024
    ctxs = tileccl.init_local(world_size=2, heap_size=128 << 20)
    try:
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        seen = []
        for layout in ("kn", "nk"):
            Cs = [c.zeros(M, N, dtype=torch.float16) for c in ctxs]
            for c, out in zip(ctxs, Cs):
                A = c.as_symmetric(A_cpu.cuda())
                B = c.as_symmetric(B_cpu.cuda()) if layout == "kn" else weight_view(c.heap, B_cpu)
                tileccl.ops.gemm_allscatter(A, B, out, ctx=c, pattern=pattern)
            torch.cuda.synchronize()
            seen.append([bits(t).clone() for t in Cs])
        assert seen[0][0].count_nonzero().item() > 0
        for a, b in zip(*seen):
            assert torch.equal(a, b)
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("variant", ["s0", "s2"])
@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (200, 272, 72), (2048, 4096, 512)])
def test_ops_gemm_reducescatter_column_shards(lib, variant, M, N, K):
    """The column-shard reduce-scatter (B's columns are split over the ranks): k-major B has w * N/w rows."""
    import tileccl_amd as tileccl

    ctxs = tileccl.init_local(world_size=2, heap_size=256 << 20)
    try:
        A_cpu = [seeded((M, K), 10 + r) for r in range(2)]
        B_cpu = seeded((K, N), 1, scale=K**-0.5)
        As = [c.as_symmetric(a.cuda()) for c, a in zip(ctxs, A_cpu)]
        seen = []
        for layout in ("kn", "nk"):
            Bs = [c.as_symmetric(B_cpu.cuda()) if layout == "kn" else weight_view(c.heap, B_cpu, 8) for c in ctxs]
            Cs = [c.zeros(M, N // 2, dtype=torch.float16) for c in ctxs]
            for _ in range(2):  # a rank's partial is resident once its op has run: second round reduces final partials
                for r, c in enumerate(ctxs):
                    tileccl.ops.gemm_reducescatter(As[r], Bs[r], Cs[r], ctx=c, variant=variant)
            torch.cuda.synchronize()
            seen.append([bits(t).clone() for t in Cs])
        assert seen[0][0].count_nonzero().item() > 0
        for a, b in zip(*seen):
            assert torch.equal(a, b)
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("schedule", ["bulk_sync", "tile_group"])
def test_chained_pattern_with_a_weight_view(lib, schedule):
    """ChainedAGGemmRSPattern: with k-major W the shards are gathered first (the in-place read of the
    shards is built for row-major W); same bytes."""
    import tileccl_amd as tileccl
    from tileccl_amd.patterns.chained_ag_gemm_rs import ChainedAGGemmRSPattern

    world, M, Ks, N = 2, 4096, 512, 4096
    ctxs = tileccl.init_local(world_size=world, heap_size=256 << 20)
    try:
        shards = [c.as_symmetric(seeded((M, Ks), 10 + p).cuda()) for p, c in enumerate(ctxs)]
        W_cpu = seeded((Ks * world, N), 1, scale=(Ks * world) ** -0.5)
        # Everything is allocated before the first execute(): the pattern takes its workspace from
        # rank 1's heap alone, after which the two allocators no longer hand out equal offsets.
        Ws = {"kn": [c.as_symmetric(W_cpu.cuda()) for c in ctxs], "nk": [weight_view(c.heap, W_cpu) for c in ctxs]}
        outs = {layout: [c.zeros(M, N, dtype=torch.float16) for c in ctxs] for layout in Ws}
        pattern = ChainedAGGemmRSPattern(ctxs[1], schedule=schedule)
        seen = []
        for layout in ("kn", "nk"):
            pattern.execute(shards[1], Ws[layout][1], outs[layout][1])
            pattern.check_faults()
            torch.cuda.synchronize()
            seen.append([bits(t).clone() for t in outs[layout]])
        assert seen[0][1].count_nonzero().item() > 0
        for a, b in zip(*seen):
            assert torch.equal(a, b)
    finally:
        for c in ctxs:
            c.heap.cleanup()
