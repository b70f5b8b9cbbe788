"""Measure the machine the cost model describes, and refit it ("Phase0 calibration").

The reference ships the fitting half (``CostModelCalibrator``, tileccl_v2/cost_model.py:445-593)
and leaves the measuring half to scripts outside the tree (README.md "Phase0 calibration").
Here both halves run through the C ABI: peer transfers of growing size are timed with HIP
events on the launch stream, the points go through ``CostModelCalibrator``, the GEMM rate is
measured on the shape in question, and the fitted ``HardwareProfile`` feeds
``choose_target_group_tiles`` / ``build_tile_group_plan``.

On one GPU a "peer" is another slice of the same HBM, so the fitted link is HBM-to-HBM copy;
on real xGMI the same procedure fits the link.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Sequence

import torch

from tileccl_amd import _launch, _lib
from tileccl_amd.v2.cost_model import (
    CalibrationPoint,
    CostModelCalibrator,
    HardwareProfile,
    Interconnect,
    TileCostModel,
    choose_target_group_tiles,
)
from tileccl_amd.v2.heap import SymmetricHeap

DEFAULT_ROWS = (1, 4, 16, 64, 256, 1024, 4096)  # x 4096 fp16 columns: 8 KiB .. 32 MiB


def _per_launch_us(launch, iters: int, warmup: int) -> float:
    for _ in range(warmup):
        launch()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        launch()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e3 / iters


def measure_transfers(heap: SymmetricHeap, rows: Sequence[int] = DEFAULT_ROWS, cols: int = 4096,
                      dtype: torch.dtype = torch.float16, iters: int = 50, warmup: int = 5) -> list[CalibrationPoint]:
    """Time a push of ``rows x cols`` elements into every peer's slice, per payload size.

    The transfer is the stand-alone row-block exchange (``tccl_exchange_rows``, push only):
    the same copy loop the fused kernels' communication role runs.
    """
    if heap.world_size < 2:
        raise ValueError("calibration needs at least one peer slice (world_size >= 2)")
    lib = _lib.load()
    view = _launch.heap_view(heap.get_heap_bases(), heap.rank, heap.world_size)
    transport = _launch.transport_desc(_lib.DIR_PUSH, 16384, None, 0)
    name = {torch.float16: "float16", torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    points = []
    for r in rows:
        out = heap.allocate_tensor((heap.world_size * r, cols), dtype)
        out.zero_()

        def launch(out=out, r=r):
            rc = lib.tccl_exchange_rows(_launch.ptr(out), r, cols, int(out.stride(0)), out.element_size(), C.byref(view),
                                        C.byref(transport), _launch.stream_ptr())
            _lib.check(rc, "tccl_exchange_rows")

        points.append(CalibrationPoint(tile_M=r, tile_N=cols, dtype=name, measured_comm_us=_per_launch_us(launch, iters, warmup)))
    return points


def measure_gemm_tflops(M: int, N: int, K: int, dtype: torch.dtype = torch.float16, iters: int = 30, warmup: int = 5) -> float:
    """Achieved TFLOP/s of ``tccl_gemm`` on one shape (device-resident operands)."""
    lib = _lib.load()
    A = torch.randn(M, K, device="cuda").to(dtype)
    B = (torch.randn(K, N, device="cuda") * K**-0.5).to(dtype)
    out = torch.empty(M, N, dtype=dtype, device="cuda")
    desc = _launch.gemm_desc(A, B, out)
    us = _per_launch_us(lambda: _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm"), iters, warmup)
    return 2.0 * M * N * K / us / 1e6


@dataclass(frozen=True)
class Calibration:
    points: tuple[CalibrationPoint, ...]
    profile: HardwareProfile
    gemm_tflops: float
    tau_min_bytes: int  # smallest payload that reaches half of the fitted bandwidth

    def model(self) -> TileCostModel:
        return TileCostModel(self.profile)

    def in_launch_profile(self) -> HardwareProfile:
        """The fitted link as a transfer inside a fused launch sees it.

        The measured points are stand-alone launches, so their latency term is dominated by
        the launch itself (the fit's floor, ~7 us here); a TileGroup moved by a launch that is
        already running pays only what exceeds that floor.  Bandwidth is unchanged.
        """
        p = self.profile
        alpha = max(p.alpha_us - p.min_comm_us, 0.05)
        return HardwareProfile(alpha_us=alpha, beta_us_per_byte=p.beta_us_per_byte, gemm_tflops_fp16=p.gemm_tflops_fp16,
                               gemm_efficiency=p.gemm_efficiency, min_comm_us=0.0, name=f"{p.name}, inside a launch")

    def target_group_tiles(self, M: int, N: int, K: int, *, in_launch: bool = True, **kwargs) -> int:
        """``target_group_tiles`` for ``build_tile_group_plan``; ``in_launch`` prices a group's
        transfer without the launch latency (the fused S1 / S2 kernels), otherwise as a
        stand-alone launch per group."""
        if not in_launch:
            kwargs.setdefault("tau_min_bytes", self.tau_min_bytes)
            return choose_target_group_tiles(self.model(), M, N, K, **kwargs)
        prof = self.in_launch_profile()
        kwargs.setdefault("tau_min_bytes", max(int(prof.alpha_us / prof.beta_us_per_byte), 1))
        return choose_target_group_tiles(TileCostModel(prof), M, N, K, **kwargs)


def calibrate(heap: SymmetricHeap, *, gemm_shape: tuple[int, int, int] = (4096, 4096, 1024),
              rows: Sequence[int] = DEFAULT_ROWS, peak_tflops: float = 2500.0) -> Calibration:
    """Measure transfers and the GEMM, fit ``alpha + bytes * beta`` with a latency floor.

    ``tau_min_bytes`` follows from the fit: a transfer reaches half of the asymptotic
    bandwidth when ``bytes * beta == alpha``, i.e. at ``alpha / beta`` bytes.
    """
    points = measure_transfers(heap, rows)
    tflops = measure_gemm_tflops(*gemm_shape)
    base = HardwareProfile.from_interconnect(Interconnect.HBM_MI355X)
    base = HardwareProfile(alpha_us=base.alpha_us, beta_us_per_byte=base.beta_us_per_byte, gemm_tflops_fp16=peak_tflops,
                           gemm_efficiency=min(1.0, tflops / peak_tflops), name="MI355X, peers in one HBM")
    profile = CostModelCalibrator.calibrate_from_measurements(points, base, two_regime=True)
    tau = int(profile.alpha_us / profile.beta_us_per_byte) if profile.beta_us_per_byte > 0 else 0
    return Calibration(tuple(points), profile, tflops, max(tau, 1))


# ---- what the matrix pipes sustain by themselves ------------------------------------------------------
PROBE_KINDS = {
    # name: (kind code of include/tileccl_hip.h, k per tile step, element type of the operands)
    "f16_32x32x16": (0, 64, torch.float16),
    "f16_16x16x32": (1, 64, torch.float16),
    "bf16_16x16x32": (2, 64, torch.bfloat16),
    "f8_16x16x128": (3, 128, torch.float8_e4m3fn),
    "f8_32x32x64": (4, 128, torch.float8_e4m3fn),
}


def mfma_sustained_tflops(kind: str, a_like: torch.Tensor, b_like: torch.Tensor, *, workgroups: int | None = None,
                          steps: tuple[int, int] = (64, 576), iters: int = 20, warmup: int = 5) -> dict:
    """TFLOP/s of a loop of nothing but MFMAs (``tccl_mfma_rate_probe``) on operand registers filled from ``a_like``
    (row operands) and ``b_like`` (column operands): the bound that the data and the instruction shape set for any K
    loop, whatever feeds it.  Two loop lengths are timed and the difference is taken, so that the launch and the
    operand loads drop out."""
    code, step_k, dtype = PROBE_KINDS[kind]
    if a_like.dtype != dtype or b_like.dtype != dtype:
        raise ValueError(f"{kind} takes {dtype} operands, got {a_like.dtype} and {b_like.dtype}")
    lib = _lib.load()
    if workgroups is None:
        workgroups = torch.cuda.get_device_properties(a_like.device).multi_processor_count
    a_like, b_like = a_like.contiguous(), b_like.contiguous()
    nbytes = [t.numel() * t.element_size() // 32 * 32 for t in (a_like, b_like)]
    sink = torch.empty(workgroups * 512, dtype=torch.float32, device=a_like.device)

    def launch(n):
        rc = lib.tccl_mfma_rate_probe(code, _launch.ptr(a_like), nbytes[0], _launch.ptr(b_like), nbytes[1], _launch.ptr(sink), n,
                                      workgroups, _launch.stream_ptr())
        _lib.check(rc, "tccl_mfma_rate_probe")

    us = [_per_launch_us(lambda n=n: launch(n), iters, warmup) for n in steps]
    per_step = (us[1] - us[0]) / (steps[1] - steps[0])
    flop = 2.0 * 256 * 256 * step_k * workgroups
    return {"kind": kind, "us_per_step": per_step, "tflops": flop / per_step / 1e6, "launch_us": us, "steps": list(steps),
            "workgroups": workgroups}
