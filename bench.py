"""Headline benchmark: fused GEMM + AllGather (TileGroup variant S2) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--variant s2] [--variants s0,s1,s2] [--workload c1]

A step is one pass of the hot path over one synthetic batch: the local GEMM
``4096x1024 @ 1024x4096`` fp16 (fp32 accumulate) whose output is gathered with an emulated
peer into ``8192x4096`` per slice, both transfer directions running through the one HBM
(BASELINE config 1, the reference's "8192x4096x1024" row).  Inputs are resident in the
symmetric heap before the timed region.  Prints ONE JSON line.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0}
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of
# this script scaled by what the same counters read for the bulk copy kernel of known size
# (profiles/fused256_kernel_c1_s2_counters.md).  Known only for the default configuration.
MEASURED_TRAFFIC_BYTES = {("c1", "s2", 0): int(175.8 * 2**20)}

WORKLOADS = {
    # name: (local M, N, K, block_m)
    "c1": (4096, 4096, 1024, 128),
    "c2": (8192, 4096, 1024, 128),
    "c2_256": (8192, 4096, 1024, 256),
}


def seeded(shape, seed, scale=1.0):
    import torch

    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).half()


def time_variant(op, A, B, variant, steps, warmup):
    """(wall ms per step, HIP-event ms per launch) over exactly `steps` back-to-back launches.

    The events are recorded on the stream the kernels are launched on (torch's current
    stream), one before the first launch and one after the last.
    """
    import torch

    for _ in range(warmup):
        op(A, B, variant)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        op(A, B, variant)
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    op.check_faults()
    return wall_ms, start.elapsed_time(stop) / steps


def cpu_baseline(A_cpu, B_cpu, peer_cpu, iters=3):
    """The oracle's restatement of the same operation on the host cores (reported, not a target)."""
    import torch

    from oracle import collectives as oracle

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    M, N = A_cpu.shape[0], B_cpu.shape[1]
    outs = [torch.zeros(2 * M, N, dtype=torch.float16) for _ in range(2)]
    outs[1][M:] = peer_cpu
    best = float("inf")
    for _ in range(iters):
        t0 = time.perf_counter()
        oracle.gemm_allgather(A_cpu, B_cpu, outs, 0)
        best = min(best, time.perf_counter() - t0)
    return best, cores


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--variant", default="s2", choices=["s0", "s1", "s2"], help="the variant `value` reports")
    ap.add_argument("--variants", default="s0,s1,s2", help="variants to time (the reported one is always included)")
    ap.add_argument("--macro-tile", type=int, default=0, choices=[0, 128, 256],
                    help="GEMM tile: 0 lets the library choose, 128 / 256 force a kernel")
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: peer ranks are emulated as slices of one HBM arena, "
              "so --gpus must be 1", file=sys.stderr)
        return 2

    import torch

    from tileccl_amd import _lib
    from tileccl_amd.backends import get_backend
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    _lib.load()
    props = get_backend().get_device_properties()
    M, N, K, block_m = WORKLOADS[args.workload]
    A_cpu, B_cpu, peer_cpu = seeded((M, K), 0), seeded((K, N), 1, K**-0.5), seeded((M, N), 2)

    heaps = SymmetricHeap.create_all(1 << 30, 2)
    ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="both", block_m=block_m, macro_tile=args.macro_tile)
           for h in heaps]
    op = ops[0]
    A, B = heaps[0].allocate_tensor((M, K)), heaps[0].allocate_tensor((K, N))
    A.copy_(A_cpu)
    B.copy_(B_cpu)
    for o in ops:
        o.out.zero_()
    ops[1].out[M:].copy_(peer_cpu)
    op.mark_peers_ready()

    flop = 2.0 * M * N * K
    esz = 2
    copy_bytes = 4.0 * M * N * esz  # push: read + write own block; pull: read + write the peer's block
    results = {}
    wanted = [v for v in ("s0", "s1", "s2") if v in args.variants.split(",") or v == args.variant]
    for variant in wanted:
        wall, mean = time_variant(op, A, B, variant, args.steps, args.warmup)
        results[variant] = {"wall_ms": wall, "event_ms_mean": mean, "tflops": flop / (mean * 1e-3) / 1e12,
                            "wall_tflops": flop / (wall * 1e-3) / 1e12}
    # parity spot-check inside the bench: moved bytes are exact
    assert torch.equal(op.peer_out(1)[:M], op.out[:M]) and torch.equal(op.out[M:].cpu(), peer_cpu)

    # GEMM alone (no communication role) for the phase split
    import ctypes as C

    from tileccl_amd import _launch

    desc = _launch.gemm_desc(A, B, op.local_block, block_m=block_m, macro_tile=args.macro_tile)
    lib = _lib.load()

    class _GemmOnly:
        def __call__(self, *_):
            _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")

        def check_faults(self):
            pass

    _, gemm_mean = time_variant(_GemmOnly(), A, B, "s0", args.steps, args.warmup)

    chosen = results[args.variant]
    tflops = chosen["tflops"]  # per launch, HIP events on the launch stream
    line = {
        "metric": "fused GEMM+AllGather ms & TFLOP/s (MFMA util), 8192x4096x1024 fp16, 1 GPU",
        "value": round(chosen["wall_tflops"], 2),  # whole timed region, host gaps included
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(chosen["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: GEMM-output AllGather, local {M}x{K} @ {K}x{N} fp16 -> {2 * M}x{N} per slice, "
                        f"2 emulated heap slices, tiles {block_m}x128, variant {args.variant.upper()}, push+pull",
            "tile_groups": op.plan.n_groups,
            "device": props.name,
            "compute_units": props.compute_units,
        },
        "variants_ms": {v: round(r["event_ms_mean"], 5) for v, r in results.items()},
        "variants_tflops": {v: round(r["tflops"], 2) for v, r in results.items()},
        "mfma_util": {v: round(r["tflops"] / PEAK_TFLOPS["f16"], 4) for v, r in results.items()},
        "gemm_only_ms": round(gemm_mean, 5),
        "gemm_only_tflops": round(flop / (gemm_mean * 1e-3) / 1e12, 2),
        "roofline": {
            "bound": "mfma",
            "achieved": round(tflops, 2),
            "peak": PEAK_TFLOPS["f16"],
            "unit": "TFLOP/s",
            "frac": round(tflops / PEAK_TFLOPS["f16"], 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, args.variant, args.macro_tile)),
            "kernel_ms": round(chosen["event_ms_mean"], 5),
        },
    }
    if "s0" in results and "s2" in results:
        line["s2_vs_s0_speedup"] = round(results["s0"]["event_ms_mean"] / results["s2"]["event_ms_mean"], 4)
    if "s0" in results:
        phase_ms = results["s0"]["event_ms_mean"] - gemm_mean
        line["copy_phase"] = {
            "bytes": copy_bytes,
            "s0_phase_ms": round(phase_ms, 5),
            "s0_phase_gbs": round(copy_bytes / (phase_ms * 1e-3) / 1e9, 1),
            "peak_gbs": PEAK_HBM_GBS,
        }
    if not args.no_cpu:
        secs, cores = cpu_baseline(A_cpu, B_cpu, peer_cpu)
        line["cpu_baseline"] = {
            "value": round(flop / secs / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": cores,
            "kind": "port",
            "sample": f"the full {args.workload} operation (torch CPU fp32 matmul + block copies), best of 3",
            "ms": round(secs * 1e3, 2),
        }
    for h in heaps:
        h.cleanup()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
