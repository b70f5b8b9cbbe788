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
    with pytest.raises(ValueError, match="contiguous rows"):  # the output is written in place, never packed
        _launch.gemm_desc(A, B, torch.empty(128, 256, dtype=torch.float16, device="cuda")[:, ::2])
    with pytest.raises(ValueError, match="leading dimension smaller"):
        d = _launch.gemm_desc(A, B, out)
        d.flags |= _lib.GEMM_B_KMAJOR  # row-major pitch (128) read as a k-major one is fine; K = 64 <= 128
        d.ldb = 32
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="K=60 must be a multiple of 8"):  # the C ABI itself takes whole vectors only
        d = _launch.gemm_desc(A, B, out)
        d.K = 60
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="16-byte boundaries"):
        d = _launch.gemm_desc(A, B, out)
        d.A += 2
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="N=100 must be a multiple of 8"):
        d = _launch.gemm_desc(A, B[:, :100].contiguous(), out[:, :100].contiguous())
        _lib.check(lib.tccl_gemm(C.byref(d), None), "tccl_gemm")
    with pytest.raises(ValueError, match="does not fit"):
        _lib.check(lib.tccl_pack_matrix(A.data_ptr(), 64, 1, 128, 64, out.data_ptr(), 32, 128, 64, 2, None), "tccl_pack_matrix")
    with pytest.raises(ValueError, match="elem_bytes=3"):
        _lib.check(lib.tccl_pack_matrix(A.data_ptr(), 64, 1, 128, 64, out.data_ptr(), 64, 128, 64, 3, None), "tccl_pack_matrix")
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


@pytest.mark.parametrize("macro", MACRO)
def test_operands_with_any_strides(lib, macro):
    """The reference's GEMM addresses A and B with whatever strides the tensors have
    (/root/reference/tileccl/kernels/gemm.py:63-66,139-151).  Layouts the MFMA kernels cannot read in place are
    packed by `tccl_pack_matrix` first: the result must be the bits of the same GEMM on contiguous copies, and a
    K that is no whole vector (zero-filled up to one) must meet the fp32 matmul like any other."""
    from tileccl_amd import _launch, _lib

    def gemm(A, B, shape):
        out = torch.full(shape, float("nan"), dtype=torch.float16, device="cuda")
        desc = _launch.gemm_desc(A, B, out, macro_tile=macro)
        _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")
        torch.cuda.synchronize()
        return out.cpu()

    M, N, K = 200, 136, 104
    A_cpu, B_cpu = seeded((M, K), 20), seeded((K, N), 21, scale=K**-0.5)
    want = gemm(A_cpu.cuda(), B_cpu.cuda(), (M, N))
    assert_gemm_close(want.cuda(), A_cpu.float() @ B_cpu.float(), tight=0.004)

    wide_a = torch.zeros(M, 2 * K + 3, dtype=torch.float16, device="cuda")
    wide_a[:, 3::2] = A_cpu.cuda()
    wide_b = torch.zeros(3 * K, N + 5, dtype=torch.float16, device="cuda")
    wide_b[::3, 5:] = B_cpu.cuda()
    both_b = torch.zeros(2 * N, 2 * K, dtype=torch.float16, device="cuda")
    both_b[::2, ::2] = B_cpu.t().cuda()
    shifted_a = torch.cat([torch.zeros(1, dtype=torch.float16), A_cpu.reshape(-1)]).cuda()
    layouts = {
        "A transposed view": (A_cpu.t().contiguous().cuda().t(), B_cpu.cuda()),
        "A every other column, odd offset": (wide_a[:, 3::2], B_cpu.cuda()),
        "A rows off the 16-byte grid": (shifted_a[1:].view(M, K), B_cpu.cuda()),
        "B every third row, columns off the grid": (A_cpu.cuda(), wide_b[::3, 5:]),
        "B strided both ways": (A_cpu.cuda(), both_b[::2, ::2].t()),
        "both": (A_cpu.t().contiguous().cuda().t(), both_b[::2, ::2].t()),
    }
    for name, (A, B) in layouts.items():
        assert torch.equal(A.cpu(), A_cpu) and torch.equal(B.cpu(), B_cpu), name
        got = gemm(A, B, (M, N))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), name

    # a broadcast operand (stride 0) and a K that is no multiple of 8
    row = seeded((1, K), 22).cuda()
    got = gemm(row.expand(M, K), B_cpu.cuda(), (M, N))
    assert torch.equal(got.view(torch.int16), gemm(row.expand(M, K).contiguous(), B_cpu.cuda(), (M, N)).view(torch.int16))
    for k_odd in (1, 7, 60, 101):
        A_odd, B_odd = seeded((M, k_odd), 23 + k_odd), seeded((k_odd, N), 24 + k_odd, scale=k_odd**-0.5)
        got = gemm(A_odd.cuda(), B_odd.cuda(), (M, N))
        assert_gemm_close(got.cuda(), A_odd.float() @ B_odd.float(), tight=0.004)
        k8 = (k_odd + 7) // 8 * 8
        A_pad, B_pad = torch.zeros(M, k8, dtype=torch.float16), torch.zeros(k8, N, dtype=torch.float16)
        A_pad[:, :k_odd], B_pad[:k_odd] = A_odd, B_odd
        assert torch.equal(got.view(torch.int16), gemm(A_pad.cuda(), B_pad.cuda(), (M, N)).view(torch.int16))
        got_t = gemm(A_odd.cuda(), k_major(B_odd), (M, N))  # k-major B with an odd K is packed as well
        assert torch.equal(got_t.view(torch.int16), got.view(torch.int16))


def test_pack_matrix_moves_every_element_once(lib):
    """`tccl_pack_matrix` against index arithmetic on the host: 1-, 2- and 4-byte elements, both stride orders,
    ragged patch edges, zero fill beyond the source, and a destination pitch wider than its rows."""
    from tileccl_amd import _launch, _lib

    g = torch.Generator().manual_seed(5)
    for dtype, rows, cols, sr, sc, drows, dcols, ld in [
        (torch.uint8, 70, 129, 300, 2, 70, 144, 144),
        (torch.uint8, 65, 64, 1, 65, 128, 64, 80),
        (torch.int16, 200, 104, 1, 200, 200, 104, 104),
        (torch.int16, 1, 1, 1, 1, 3, 9, 16),
        (torch.int32, 130, 67, 67, 1, 131, 72, 72),
        (torch.int32, 64, 64, 0, 1, 64, 64, 64),
    ]:
        span = (rows - 1) * sr + (cols - 1) * sc + 1
        backing = torch.randint(1, 100, (span,), generator=g).to(dtype).cuda()
        src = torch.as_strided(backing, (rows, cols), (sr, sc))
        dst = torch.full((drows, ld), 77, dtype=dtype, device="cuda")
        rc = lib.tccl_pack_matrix(src.data_ptr(), sr, sc, rows, cols, dst.data_ptr(), ld, drows, dcols,
                                  src.element_size(), _launch.stream_ptr())
        _lib.check(rc, "tccl_pack_matrix")
        torch.cuda.synchronize()
        want = torch.full((drows, ld), 77, dtype=dtype)
        want[:, :dcols] = 0
        want[:rows, :cols] = src.cpu()
        assert torch.equal(dst.cpu(), want), (dtype, rows, cols, sr, sc)


def test_packed_operands_outlive_their_descriptor_only(lib):
    """A packed operand belongs to the descriptor it was packed for: a second descriptor built while the first is
    alive gets a buffer of its own (both launches then read what they were given), and the buffer is taken up again
    once the descriptor that held it is gone."""
    from tileccl_amd import _launch, _lib

    M, N, K = 128, 128, 64
    A1, A2 = seeded((K, M), 30).cuda().t(), seeded((K, M), 31).cuda().t()  # transposed views: packed
    B = seeded((K, N), 32, scale=K**-0.5).cuda()
    out1 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    out2 = torch.zeros_like(out1)
    d1 = _launch.gemm_desc(A1, B, out1)
    d2 = _launch.gemm_desc(A2, B, out2)
    assert d1.A != d2.A and d1.A != A1.data_ptr() and d1.B == B.data_ptr()
    for d in (d1, d2):
        _lib.check(lib.tccl_gemm(C.byref(d), _launch.stream_ptr()), "tccl_gemm")
    torch.cuda.synchronize()
    assert_gemm_close(out1, A1.float().cpu() @ B.float().cpu(), tight=0.004)
    assert_gemm_close(out2, A2.float().cpu() @ B.float().cpu(), tight=0.004)
    first = d2.A
    del d, d1, d2
    d3 = _launch.gemm_desc(A1, B, out1)
    assert d3.A == first  # the most recently released buffer of that shape
