"""The MFMA GEMM through the C ABI against the CPU oracle (fp32 matmul, one rounding).

Tolerance: the reference's own (rtol 1e-2, atol 1e-1; tests/test_gemm_allscatter_smoke.py:39-40)
plus a tight absolute bound that a wrong operand layout or a dropped K step cannot meet."""

import ctypes as C

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, seeded

pytestmark = pytest.mark.gpu


def k_major(B_cpu, pad=0):
    """B on the device as the transposed view of an (N, K + pad) tensor: element (k, n) at n * (K + pad) + k."""
    K, N = B_cpu.shape
    backing = torch.zeros(N, K + pad, dtype=B_cpu.dtype, device="cuda")
    backing[:, :K] = B_cpu.t().cuda()
    return backing[:, :K].t()


def run_gemm(lib, A_cpu, B_cpu, out_dtype, b_kmajor=False, b_pad=0, **kw):
    from tileccl_amd import _launch, _lib

    A, B = A_cpu.cuda(), (k_major(B_cpu, b_pad) if b_kmajor else B_cpu.cuda())
    out = torch.full((A.shape[0], B.shape[1]), float("nan"), dtype=out_dtype, device="cuda")
    desc = _launch.gemm_desc(A, B, out, **kw)
    _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")
    torch.cuda.synchronize()
    return out


SHAPES = [
    (128, 128, 64),  # the reference smoke test's single tile, one K step
    (128, 64, 128),  # reference smoke shape (M, K, N) = (128, 64, 128)
    (256, 384, 512),
    (200, 136, 72),  # ragged M, N and a K tail
    (1, 8, 8),
    (130, 8, 264),
    (512, 512, 256),  # benchmark configuration 0
    (1024, 4096, 1024),
]


# macro_tile: 128 = the 128 x 128 kernel, 256 = the large-tile kernel (0 would pick by size)
MACRO = [128, 256]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("macro", MACRO)
def test_gemm_matches_fp32_matmul(lib, M, N, K, dtype, macro):
    A = seeded((M, K), 0, dtype)
    B = seeded((K, N), 1, dtype, scale=K**-0.5)
    got = run_gemm(lib, A, B, dtype, macro_tile=macro)
    ref32 = A.float() @ B.float()
    assert not torch.isnan(got.float()).any()
    # one rounding of an O(1) value: half an ulp of fp16 (2^-11 rel.) / bf16 (2^-8 rel.) at |x| < 8
    assert_gemm_close(got, ref32, tight=0.004 if dtype == torch.float16 else 0.032)
    # the oracle rounds the same fp32 sum once; accumulation order may differ by an fp32 ulp,
    # which can flip a rounding, so allow one output ulp against it
    want = oracle.gemm(A, B, dtype)
    assert (got.cpu().float() - want.float()).abs().max().item() <= (0.004 if dtype == torch.float16 else 0.032)


@pytest.mark.parametrize("M,N,K", SHAPES + [(512, 520, 1000)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("macro", MACRO)
def test_k_major_B_gives_the_bits_of_row_major_B(lib, M, N, K, dtype, macro):
    """B handed over as the `.t()` view of an (N, K) tensor (a linear layer's weight): the k order of
    the sums does not depend on the layout, so the result is bit-identical to the row-major run;
    with a padded pitch too (ldb = K + 8)."""
    A = seeded((M, K), 0, dtype)
    B = seeded((K, N), 1, dtype, scale=K**-0.5)
    want = run_gemm(lib, A, B, dtype, macro_tile=macro)
    assert_gemm_close(want, A.float() @ B.float(), tight=0.004 if dtype == torch.float16 else 0.032)
    for pad in (0, 8):
        got = run_gemm(lib, A, B, dtype, b_kmajor=True, b_pad=pad, macro_tile=macro)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), pad
    got32 = run_gemm(lib, A, B, torch.float32, b_kmajor=True, macro_tile=macro)
    assert torch.equal(got32, run_gemm(lib, A, B, torch.float32, macro_tile=macro))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("macro", MACRO)
def test_fp32_output_keeps_the_accumulator(lib, dtype, macro):
    A, B = seeded((384, 256), 3, dtype), seeded((256, 640), 4, dtype, scale=1 / 16)
    got = run_gemm(lib, A, B, torch.float32, macro_tile=macro)
    ref32 = A.float() @ B.float()
    assert (got.cpu() - ref32).abs().max().item() < 1e-4  # only the fp32 summation order differs


@pytest.mark.parametrize("macro", MACRO)
def test_alpha_and_plan_tile_256(lib, macro):
    A, B = seeded((512, 128), 5), seeded((128, 384), 6, scale=128**-0.5)
    ref32 = 0.5 * (A.float() @ B.float())
    assert_gemm_close(run_gemm(lib, A, B, torch.float16, alpha=0.5, macro_tile=macro), ref32, tight=0.004)
    assert_gemm_close(run_gemm(lib, A, B, torch.float16, alpha=0.5, block_m=256, group_m=3, macro_tile=macro), ref32, tight=0.004)
    assert_gemm_close(
        run_gemm(lib, A, B, torch.float16, alpha=0.5, block_m=256, block_n=256, num_wgs=7, macro_tile=macro), ref32, tight=0.004
    )


@pytest.mark.parametrize("macro", MACRO)
def test_exact_small_integers(lib, macro):
    """Integer-valued inputs whose products and sums are exact in fp16/fp32: bit-exact result."""
    g = torch.Generator().manual_seed(7)
    A = torch.randint(-3, 4, (256, 192), generator=g).half()
    B = torch.randint(-3, 4, (192, 256), generator=g).half()
    got = run_gemm(lib, A, B, torch.float16, macro_tile=macro)
    assert torch.equal(got.cpu(), (A.float() @ B.float()).half())


@pytest.mark.parametrize("macro", MACRO)
def test_rows_beyond_M_and_cols_beyond_N_are_untouched(lib, macro):
    from tileccl_amd import _launch, _lib

    A, B = seeded((100, 64), 8).cuda(), seeded((64, 72), 9).cuda()
    backing = torch.full((128, 128), 7.0, dtype=torch.float16, device="cuda")
    out = backing[:100, :72]  # ldc = 128
    desc = _launch.gemm_desc(A, B, out, macro_tile=macro)
    _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")
    torch.cuda.synchronize()
    assert torch.all(backing[100:] == 7.0) and torch.all(backing[:, 72:] == 7.0)
    assert_gemm_close(out, A.float().cpu() @ B.float().cpu())


def test_unsupported_layouts_fail_loudly(lib):
    from tileccl_amd import _launch, _lib

    A, B = seeded((128, 64), 0).cuda(), seeded((64, 128), 1).cuda()
    out = torch.empty(128, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError, match="contiguous rows"):
        _launch.gemm_desc(A, torch.empty(64, 256, dtype=torch.float16, device="cuda")[:, ::2], out)
    with pytest.raises(ValueError, match="contiguous rows"):
        _launch.gemm_desc(A.t().contiguous().t(), B, out)
    with pytest.raises(ValueError, match="leading dimension smaller"):
        d = _launch.gemm_desc(A, B, out)
        d.flags |= _lib.GEMM_B_KMAJOR  # row-major pitch (128) read as a k-major one is fine; K = 64 <= 128
        d.ldb = 32
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="K=60 must be a multiple of 8"):
        d = _launch.gemm_desc(A[:, :60].contiguous(), B[:60].contiguous(), out)
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="N=100 must be a multiple of 8"):
        d = _launch.gemm_desc(A, B[:, :100].contiguous(), out[:, :100].contiguous())
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="must be a multiple of 128x128"):
        d = _launch.gemm_desc(A, B, out, block_m=64)
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="macro_tile=64 must be 0, 128 or 256"):
        d = _launch.gemm_desc(A, B, out, macro_tile=64)
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="no kernel for in_dtype"):
        d = _launch.gemm_desc(A, B, torch.empty(128, 128, dtype=torch.bfloat16, device="cuda"))
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")


@pytest.mark.parametrize("macro", MACRO)
def test_every_length_of_the_k_loop(lib, macro):
    """K from one chunk to a dozen steps, ragged tails included: the staged K loops (three or five stages of 32 k on
    the 128 tile, two of 64 k on the large tile) leave through each of their exits, and the look-ahead loads past K
    never reach a sum."""
    for K in (8, 24, 32, 40, 64, 96, 104, 128, 136, 160, 168, 192, 200, 224, 256, 296, 320, 352, 384, 776):
        A, B = seeded((256, K), 10 + K), seeded((K, 136), 11 + K, scale=K**-0.5)
        got = run_gemm(lib, A, B, torch.float16, macro_tile=macro)
        assert_gemm_close(got, A.float() @ B.float(), tight=0.004)
        # integer-valued operands: every partial sum is exact, so the result is exact whatever the step structure
        g = torch.Generator().manual_seed(K)
        Ai = torch.randint(-2, 3, (130, K), generator=g).half()
        Bi = torch.randint(-2, 3, (K, 72), generator=g).half()
        want = (Ai.float() @ Bi.float()).half()
        assert torch.equal(run_gemm(lib, Ai, Bi, torch.float16, macro_tile=macro).cpu(), want), K
