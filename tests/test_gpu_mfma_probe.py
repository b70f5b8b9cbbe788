"""``tccl_mfma_rate_probe``: the MFMA-only loop that bench.py prices the K loops against.

Its arithmetic is checked (all-one operands make every accumulator a count of products), its argument
checks, and that the rate it reports is a plausible one for the part."""

import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["f16_32x32x16", "f16_16x16x32", "bf16_16x16x32", "f8_16x16x128", "f8_32x32x64"])
def test_probe_counts_products(lib, kind):
    from tileccl_amd import _launch, _lib
    from tileccl_amd.v2.calibrate import PROBE_KINDS

    code, step_k, dtype = PROBE_KINDS[kind]
    ones = torch.ones(1 << 16, device="cuda").to(dtype)
    wgs, steps = 3, 5
    sink = torch.zeros(wgs * 512, dtype=torch.float32, device="cuda")
    rc = lib.tccl_mfma_rate_probe(code, _launch.ptr(ones), ones.numel() * ones.element_size(), _launch.ptr(ones),
                                  ones.numel() * ones.element_size(), _launch.ptr(sink), steps, wgs, _launch.stream_ptr())
    _lib.check(rc, "tccl_mfma_rate_probe")
    torch.cuda.synchronize()
    # every accumulator element is steps * step_k products of 1 * 1; a lane adds up two elements of each of its
    # 32 blocks of 16 x 16 (8 patches of 32 x 32)
    blocks = 8 if kind.endswith(("32x32x16", "32x32x64")) else 32
    assert torch.all(sink == float(2 * blocks * steps * step_k)), (kind, sink[:4].tolist())


def test_probe_rejects_bad_arguments(lib):
    from tileccl_amd import _launch, _lib

    buf = torch.zeros(1024, dtype=torch.float16, device="cuda")
    sink = torch.zeros(512, dtype=torch.float32, device="cuda")
    ok = (_launch.ptr(buf), 2048, _launch.ptr(buf), 2048, _launch.ptr(sink), 1, 1, None)
    for bad in [(9,) + ok, (1, None) + ok[1:], (1, ok[0], 40) + ok[2:], (1,) + ok[:5] + (-1, 1, None), (1,) + ok[:6] + (0, None)]:
        with pytest.raises(ValueError):
            _lib.check(lib.tccl_mfma_rate_probe(*bad), "tccl_mfma_rate_probe")


def test_sustained_rate_is_plausible_and_depends_on_the_data(lib):
    from tileccl_amd.v2.calibrate import mfma_sustained_tflops

    g = torch.Generator().manual_seed(0)
    a = torch.randn(1 << 22, generator=g).half().cuda()
    b = (torch.randn(1 << 22, generator=g) / 32).half().cuda()
    zeros = torch.zeros(1 << 22, dtype=torch.float16, device="cuda")
    data = mfma_sustained_tflops("f16_16x16x32", a, b)
    idle = mfma_sustained_tflops("f16_16x16x32", zeros, zeros)
    assert 500.0 < data["tflops"] < 2600.0 and 500.0 < idle["tflops"] < 2600.0
    assert idle["tflops"] > data["tflops"]  # all-zero operands toggle nothing: the pipes run faster on them
