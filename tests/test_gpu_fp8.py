"""fp8 (OCP e4m3) GEMM and GEMM -> ReduceScatter on gfx950's 32x32x64 fp8 MFMA.

Inputs follow the fp8 recipe of benchmark configuration 4: N(0,1) samples divided by a per-tensor fp32 scale,
clipped to +-448 and rounded to e4m3; the scales' product multiplies the accumulator.
Products of two e4m3 values are exact in fp32, so the GPU result differs from the oracle
(dequantise, fp32 matmul) only by fp32 summation order and the output rounding; the stated
tolerance for fp8 is rtol 5e-2, and a tight absolute bound rules out layout mistakes."""

import ctypes as C

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu

F8 = torch.float8_e4m3fn


def quantise(shape, seed, std=1.0):
    """(e4m3 tensor, dequantisation scale) for x ~ N(0, std^2): stored value = clip(x / scale, +-448),
    with the scale chosen so that one standard deviation is stored as 64."""
    x = seeded(shape, seed, torch.float32, scale=std)
    scale = std / 64
    return (x / scale).clamp(-448.0, 448.0).to(F8), scale


def run_gemm(lib, A_cpu, B_cpu, out_dtype, alpha=1.0, **kw):
    from tileccl_amd import _launch, _lib

    A, B = A_cpu.cuda(), B_cpu.cuda()
    out = torch.full((A.shape[0], B.shape[1]), float("nan"), dtype=out_dtype, device="cuda")
    desc = _launch.gemm_desc(A, B, out, alpha=alpha, **kw)
    _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (256, 256, 64), (512, 768, 512), (300, 272, 80), (1, 16, 16),
                                   (1024, 4096, 1024)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_fp8_gemm_matches_dequantised_matmul(lib, M, N, K, out_dtype):
    A, sa = quantise((M, K), 0)
    B, sb = quantise((K, N), 1, K**-0.5)
    got = run_gemm(lib, A, B, out_dtype, alpha=sa * sb)
    ref32 = (A.float() @ B.float()) * (sa * sb)
    assert not torch.isnan(got.float()).any()
    tight = {torch.float32: 1e-3, torch.float16: 0.004, torch.bfloat16: 0.032}[out_dtype]
    assert_gemm_close(got, ref32, rtol=5e-2, atol=1e-1, tight=tight)
    want = oracle.gemm(A, B, out_dtype, alpha=sa * sb)
    assert (got.cpu().float() - want.float()).abs().max().item() <= tight


def test_fp8_exact_small_integers(lib):
    """Integer-valued e4m3 inputs: every product and partial sum is exact, so is the result."""
    g = torch.Generator().manual_seed(7)
    A = torch.randint(-3, 4, (256, 320), generator=g).float().to(F8)
    B = torch.randint(-3, 4, (320, 512), generator=g).float().to(F8)
    got = run_gemm(lib, A, B, torch.float32)
    assert torch.equal(got.cpu(), A.float() @ B.float())


def test_fp8_needs_the_large_tile_kernel(lib):
    from tileccl_amd import _launch, _lib

    A, B = torch.zeros(256, 64, dtype=F8, device="cuda"), torch.zeros(64, 256, dtype=F8, device="cuda")
    out = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="fp8 inputs need the 256x256 kernel"):
        d = _launch.gemm_desc(A, B, out, macro_tile=128)
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="K=72 must be a multiple of 16"):  # the C ABI takes whole 16-byte vectors
        d = _launch.gemm_desc(A, B, out)
        d.K = 72
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    # the launch helper packs such operands (K zero-filled to 80): same bits as the padded operands passed directly
    A72, sa = quantise((256, 72), 40)
    B72, sb = quantise((72, 256), 41, 72**-0.5)
    A80, B80 = torch.zeros(256, 80, dtype=F8), torch.zeros(80, 256, dtype=F8)
    A80.view(torch.uint8)[:, :72], B80.view(torch.uint8)[:72] = A72.view(torch.uint8), B72.view(torch.uint8)
    got72, got80 = run_gemm(lib, A72, B72, torch.bfloat16, alpha=sa * sb), run_gemm(lib, A80, B80, torch.bfloat16, alpha=sa * sb)
    assert torch.equal(got72.view(torch.int16), got80.view(torch.int16))
    assert_gemm_close(got72, (A72.float() @ B72.float()) * (sa * sb), rtol=5e-2, atol=1e-1, tight=0.032)


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
def test_fp8_reduce_scatter_two_ranks(lib, variant):
    """The fp8 ReduceScatter configuration at a small size: bf16 partial, resident bf16 peer
    partial, fp32 reduction, bf16 output; the reduction is bit-exact against the oracle run
    on the partial the GPU produced."""
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    M, N, K = 1024, 512, 256
    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        ops = [FusedGemmReduceScatter(h, M, N, partial_dtype=torch.bfloat16, out_dtype=torch.bfloat16) for h in heaps]
        op = ops[0]
        A_cpu, sa = quantise((M, K), 0)
        B_cpu, sb = quantise((K, N), 1, K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        peer = seeded((M, N), 2, torch.bfloat16)
        ops[1].partial.copy_(peer)
        for o in ops:
            o.out.zero_()
        op.mark_peers_ready()
        op(A, B, variant, scale_a=sa, scale_b=sb)
        op.check_faults()
        assert_gemm_close(op.partial, (A_cpu.float() @ B_cpu.float()) * (sa * sb), rtol=5e-2, tight=0.032)
        partials = [op.partial.cpu(), peer]
        for owner in (0, 1):
            want = oracle.reduce_rows(partials, owner, torch.bfloat16)
            assert torch.equal(bits(ops[owner].out).cpu(), bits(want)), f"owner {owner}"
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s0", "s1", "s2"])
@pytest.mark.parametrize("directions", ["both", "pull"])
def test_fp8_allgather_two_ranks(lib, variant, directions):
    """GEMM-output AllGather with e4m3 inputs and a bf16 output: the fp8 K loop carries the
    background pull of S2 (a few pieces per wavefront inside the K loop, the rest after the
    last tile).  The product is held to the fp8 tolerance, everything moved is bit-exact."""
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    M, N, K = 1024, 512, 512
    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.bfloat16, directions=directions) for h in heaps]
        op = ops[0]
        A_cpu, sa = quantise((M, K), 0)
        B_cpu, sb = quantise((K, N), 1, K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        block = seeded((M, N), 2, torch.bfloat16)
        for o in ops:
            o.out.zero_()
        ops[1].out[M:].copy_(block)
        op.mark_peers_ready()
        op(A, B, variant, scale_a=sa, scale_b=sb)
        op.check_faults()
        mine = op.out[:M].clone()
        assert_gemm_close(mine, (A_cpu.float() @ B_cpu.float()) * (sa * sb), rtol=5e-2, tight=0.032)
        if directions == "both":
            assert torch.equal(bits(op.peer_out(1)[:M]), bits(mine))
        else:
            assert torch.count_nonzero(op.peer_out(1)[:M]).item() == 0  # nothing pushed
        assert torch.equal(bits(op.out[M:]).cpu(), bits(block))  # the pulled block
        assert torch.equal(bits(op.peer_out(1)[M:]).cpu(), bits(block))  # the peer's own block is untouched
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("own_rows", [False, True])
def test_baseline_config_4_properties(lib, own_rows):
    """16384x2048 @ 2048x4096 e4m3 with per-tensor scales, resident bf16 peer partial: the three
    variants agree byte for byte, the reduction equals the oracle on slabs of both owners, the
    partial matches the dequantised matmul on a slab, counters match the plan; with the owned
    rows kept in registers (what the benchmark runs) the outputs are the same bytes."""
    from tests.test_gpu_reducescatter import check_full_size_config
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    M, N, K = 16384, 4096, 2048
    heaps = SymmetricHeap.create_all(1 << 30, 2)
    try:
        kw = dict(partial_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
        ops = [FusedGemmReduceScatter(h, M, N, **kw) for h in heaps]
        kept_ops = [FusedGemmReduceScatter(h, M, N, own_rows_in_registers=True, **kw) for h in heaps] if own_rows else None
        op = ops[0]
        assert op.plan.n_groups == 16 and op.shard_rows == 8192
        A_cpu, sa = quantise((M, K), 0)
        B_cpu, sb = quantise((K, N), 1, K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        peer_cpu = seeded((M, N), 2, torch.bfloat16)  # the peer's partial: bf16 N(0, 1), seeded on the CPU

        def gemm_ref(partial):
            rows = slice(8100, 8228)
            ref = (A_cpu[rows].float() @ B_cpu.float()) * (sa * sb)
            assert_gemm_close(partial[rows], ref, rtol=5e-2, tight=0.032)

        check_full_size_config(heaps, ops, kept_ops, A, B, 8192, torch.bfloat16, gemm_ref, peer_cpu, scale_a=sa, scale_b=sb)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("world,M", [(2, 1024), (3, 768)])
def test_fp8_own_rows_kept_in_registers_give_the_same_bytes(lib, variant, world, M):
    """fp8 inputs with the owned rows' partial kept in the accumulators: with two ranks the other
    owner's rows are reduced from the accumulators as well (the stored, rounded partial enters the
    sum), with three they are reduced by reading the stored partial back.  Outputs equal the oracle's reduction of the partials a plain
    run stored, bit for bit (three ranks: order-sensitive magnitudes); the owned rows of
    `partial` are never written, the other rows are."""
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    N, K = 528, 512  # e4m3 rows of B must be multiples of 16 bytes
    A_cpu, sa = quantise((M, K), 0)
    B_cpu, sb = quantise((K, N), 1, K**-0.5)
    peers_cpu = {p: seeded((M, N), 10 + p, torch.bfloat16) * (1000.0 if world == 3 else 1.0) for p in range(1, world)}

    def run(flag):
        heaps = SymmetricHeap.create_all(64 << 20, world)
        try:
            ops = [FusedGemmReduceScatter(h, M, N, partial_dtype=torch.bfloat16, out_dtype=torch.bfloat16,
                                          tau_min_bytes=1, group_m=1, own_rows_in_registers=flag) for h in heaps]
            A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
            for p in range(1, world):
                ops[p].partial.copy_(peers_cpu[p])
            for o in ops:
                o.out.zero_()
            ops[0].partial.fill_(-3.0)
            ops[0].mark_peers_ready()
            ops[0](A, B, variant, scale_a=sa, scale_b=sb)
            ops[0].check_faults()
            return ops[0].partial.cpu(), [o.out.cpu() for o in ops]
        finally:
            for h in heaps:
                h.cleanup()

    plain_partial, plain_outs = run(False)
    kept_partial, kept_outs = run(True)
    assert_gemm_close(plain_partial, (A_cpu.float() @ B_cpu.float()) * (sa * sb), rtol=5e-2, tight=0.032)
    shard = M // world
    partials = [plain_partial] + [peers_cpu[p] for p in range(1, world)]
    for owner in range(world):
        want = oracle.reduce_rows(partials, owner, torch.bfloat16)
        assert torch.equal(bits(plain_outs[owner]), bits(want)), owner
        assert torch.equal(bits(kept_outs[owner]), bits(want)), owner
    assert torch.all(kept_partial[:shard] == -3.0)  # never stored
    assert torch.equal(bits(kept_partial[shard:]), bits(plain_partial[shard:]))
