"""Headline benchmark: fused GEMM + AllGather (TileGroup variant S2) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--variant s2] [--variants s0,s1,s2] [--workload c1]

A step is one pass of the hot path over one synthetic batch.  The default workload is the
local GEMM ``4096x1024 @ 1024x4096`` fp16 (fp32 accumulate) whose output is gathered with
an emulated peer into ``8192x4096`` per slice, both transfer directions running through the
one HBM (benchmark configuration 1, the reference's "8192x4096x1024" row).  The other
configurations can be timed with ``--workload`` (c2: the larger all-gather; c3: GEMM ->
ReduceScatter with fp32 partials; c4: the fp8 ReduceScatter; ch1: the chained
gather -> GEMM -> scatter over column shards).  Inputs are resident in the
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

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f8": 5000.0}
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of
# this script scaled by what the same counters read for the bulk copy kernel of known size
# (profiles/fused256_kernel_<workload>_s2_counters.md).  Known only for the default tile choice.
MEASURED_TRAFFIC_BYTES = {("c1", "s2", 0): int(176.2 * 2**20), ("c2", "s2", 0): int(352.0 * 2**20),
                          ("c3", "s2", 0): int(447.9 * 2**20), ("c4", "s2", 0): int(513.3 * 2**20)}

WORKLOADS = {
    # name: kind, local M, N, K, block_m, input type
    "c1": ("ag", 4096, 4096, 1024, 128, "f16"),
    "c2": ("ag", 8192, 4096, 1024, 128, "f16"),
    "c2_256": ("ag", 8192, 4096, 1024, 256, "f16"),
    "c3": ("rs", 8192, 4096, 2048, 128, "f16"),
    "c4": ("rs", 16384, 4096, 2048, 128, "f8"),
    # gather -> GEMM -> scatter over column shards of the input (K = 2 shards of 1024)
    "ch1": ("ch", 4096, 4096, 2048, 128, "f16"),
}
METRIC = "fused GEMM+AllGather ms & TFLOP/s (MFMA util), 8192x4096x1024 fp16, 1 GPU"


def seeded(shape, seed, scale=1.0, dtype=None):
    import torch

    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype or torch.float16)


def quantised(shape, seed, std):
    """fp8 recipe: N(0, std^2) samples over a per-tensor scale (one sigma stored as 64), clipped to +-448."""
    import torch

    scale = std / 64
    x = seeded(shape, seed, std, torch.float32)
    return (x / scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn), scale


SETTLE_SECONDS = 0.05


def time_variant(run, variant, steps, warmup):
    """(wall ms per step, HIP-event ms per launch) over exactly `steps` back-to-back launches.

    The events are recorded on the stream the kernels are launched on (torch's current
    stream), one before the first launch and one after the last.

    Warm-up is `warmup` launches and at least SETTLE_SECONDS of them: the part lowers its clocks
    within milliseconds of idling (the host work between two variants is enough) and takes
    tens of milliseconds of load to raise them again (traced: the same GEMM 37 us right after
    an idle gap, 33 us 40 ms later), so a count alone would time each variant at a different
    point of that ramp.
    """
    import gc

    import torch

    # As timeit does: a full collection of the interpreter's cyclic garbage takes tens of
    # milliseconds with torch loaded, during which nothing is enqueued and the GPU idles.
    gc.collect()
    gc.disable()
    try:
        done, t_warm = 0, time.perf_counter()
        while done < warmup or time.perf_counter() - t_warm < SETTLE_SECONDS:
            for _ in range(20 if done >= warmup else warmup):
                run(variant)
            done += 20 if done >= warmup else warmup
            torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for _ in range(steps):
            run(variant)
        stop.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    finally:
        gc.enable()
    return wall_ms, start.elapsed_time(stop) / steps


def launch_spread(run, variant, launches=100):
    """min / median / mean of single launches, each between its own pair of HIP events, taken
    back to back right after a timed region (so at settled clocks)."""
    import statistics

    import torch

    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    for a, b in pairs:
        a.record()
        run(variant)
        b.record()
    torch.cuda.synchronize()
    us = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
    return {"launches": launches, "min": round(us[0], 2), "median": round(statistics.median(us), 2),
            "mean": round(statistics.fmean(us), 2), "max": round(us[-1], 2),
            "note": "an event pair per launch adds 2-3 us of event handling to each interval; ms_per_step has one pair around all steps"}


class Workload:
    """One benchmark configuration: heap slices, resident inputs, the fused operation."""

    def __init__(self, name, macro_tile, group_tiles=None, b_layout="kn"):
        import torch

        from tileccl_amd.v2 import FusedGemmAllGather, FusedGemmReduceScatter, SymmetricHeap

        self.name = name
        self.b_layout = b_layout
        self.kind, self.M, self.N, self.K, self.block_m, self.in_type = WORKLOADS[name]
        M, N, K = self.M, self.N, self.K
        self.group_tiles, self.calibration = self.resolve_group_tiles(group_tiles)
        self.scales = (1.0, 1.0)
        if self.in_type == "f8":
            self.A_cpu, sa = quantised((M, K), 0, 1.0)
            self.B_cpu, sb = quantised((K, N), 1, K**-0.5)
            self.scales = (sa, sb)
        else:
            self.A_cpu, self.B_cpu = seeded((M, K), 0), seeded((K, N), 1, K**-0.5)
        self.heaps = SymmetricHeap.create_all(2 << 30, 2)
        common = dict(block_m=self.block_m, macro_tile=macro_tile, target_group_tiles=self.group_tiles)
        if self.kind == "ag":
            self.peer_cpu = seeded((M, N), 2)
            self.ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="both", **common) for h in self.heaps]
            for o in self.ops:
                o.out.zero_()
            self.ops[1].out[M:].copy_(self.peer_cpu)
            self.exchange_bytes = 4.0 * M * N * 2  # push: read + write own block; pull: read + write the peer's
            # The same operation with only the push emulated (what one rank of a real pair does itself:
            # the peer's block arrives by the peer's push, without work on this side).
            self.push_only = FusedGemmAllGather(self.heaps[0], M, N, torch.float16, directions="push", **common)
            FusedGemmAllGather(self.heaps[1], M, N, torch.float16, directions="push", **common)  # same offsets in the peer slice
        else:
            pdt = torch.bfloat16 if self.in_type == "f8" else torch.float32
            odt = torch.bfloat16 if self.in_type == "f8" else torch.float16
            self.peer_cpu = seeded((M, N), 2, 1.0, pdt)
            # S1 / S2 keep the partial of the rows a rank owns in the accumulators (S0, two kernels, cannot)
            self.ops = [FusedGemmReduceScatter(h, M, N, partial_dtype=pdt, out_dtype=odt, own_rows_in_registers=True, **common)
                        for h in self.heaps]
            self.ops[1].partial.copy_(self.peer_cpu)
            psz = self.peer_cpu.element_size()
            # What one rank of a real pair does itself: its own rows' reduction; the peer reduces its rows.
            alone = [FusedGemmReduceScatter(h, M, N, partial_dtype=pdt, out_dtype=odt, own_rows_in_registers=True,
                                            emulate_peer=False, **common) for h in self.heaps]
            alone[1].partial.copy_(self.peer_cpu)
            self.push_only = alone[0]
            self.exchange_bytes = 2.0 * M * N * psz + M * N * 2  # both partials read once, every output row written once
        self.op = self.ops[0]
        self.A = self.heaps[0].allocate_tensor((M, K), self.A_cpu.dtype)
        if b_layout == "nk":  # the same B held as an (N, K) tensor, handed over as its `.t()` view
            self.B = self.heaps[0].allocate_tensor((N, K), self.B_cpu.dtype).t()
        else:
            self.B = self.heaps[0].allocate_tensor((K, N), self.B_cpu.dtype)
        self.A.copy_(self.A_cpu)
        self.B.copy_(self.B_cpu)
        self.op.mark_peers_ready()
        self.flop = 2.0 * M * N * K
        self.own_out = {}

    def resolve_group_tiles(self, group_tiles):
        """`--group-tiles`: None keeps the planner's own rule (groups of at least tau_min bytes),
        an integer is passed through, "auto" measures this machine and asks the cost model
        (calibrate -> choose_target_group_tiles, the reference's "Phase0 calibration")."""
        if group_tiles in (None, "default"):
            return None, None
        if group_tiles != "auto":
            return int(group_tiles), None
        from tileccl_amd.v2 import SymmetricHeap
        from tileccl_amd.v2.calibrate import calibrate

        heaps = SymmetricHeap.create_all(256 << 20, 2)  # its own slices: the workload's offsets stay symmetric
        try:
            cal = calibrate(heaps[0], gemm_shape=(self.M, self.N, self.K))
        finally:
            for h in heaps:
                h.cleanup()
        # the element type of what travels: the fp16 output block, or the partial of a reduce-scatter
        dtype = "float16" if self.kind == "ag" else ("bfloat16" if self.in_type == "f8" else "float32")
        tiles = cal.target_group_tiles(self.M, self.N, self.K, block_m=self.block_m, dtype=dtype)
        return tiles, {"alpha_us": round(cal.profile.alpha_us, 3), "gbytes_per_s": round(1e-3 / cal.profile.beta_us_per_byte, 1),
                       "launch_floor_us": round(cal.profile.min_comm_us, 3), "gemm_tflops": round(cal.gemm_tflops, 1),
                       "in_launch_alpha_us": round(cal.in_launch_profile().alpha_us, 3), "target_group_tiles": tiles}

    def run(self, variant):
        self.op(self.A, self.B, variant, scale_a=self.scales[0], scale_b=self.scales[1])

    def run_one_direction(self, variant):
        self.push_only(self.A, self.B, variant, scale_a=self.scales[0], scale_b=self.scales[1])

    @property
    def one_direction_note(self):
        if self.kind == "ag":
            return ("push direction only (the own block read once and written to the peer); "
                    "value and roofline above emulate both directions")
        return ("this rank's share only: the partial of the rows it does not own is stored, its own rows are reduced; "
                "value and roofline above also run the peer's reduction")

    def after_variant(self, variant):
        """Keep what the variant left in the first rows of rank 0's output shard (compared in spot_check)."""
        if self.kind == "rs":
            self.own_out[variant] = self.op.out[:256].clone().view(__import__("torch").int16)

    def describe(self, variant):
        M, N, K = self.M, self.N, self.K
        if self.kind == "ag":
            return (f"{self.name}: GEMM-output AllGather, local {M}x{K} @ {K}x{N} fp16 -> {2 * M}x{N} per slice, "
                    f"2 emulated heap slices, tiles {self.block_m}x128, variant {variant.upper()}, push+pull")
        what = "e4m3 inputs, bf16 partials and output" if self.in_type == "f8" else "fp16 inputs, fp32 partials, fp16 output"
        return (f"{self.name}: GEMM -> ReduceScatter, local {M}x{K} @ {K}x{N} ({what}), resident peer partial, "
                f"2 emulated heap slices (both owners' reductions run), tiles {self.block_m}x128, variant {variant.upper()}"
                + ("" if variant == "s0" else ", reductions fed from the accumulators"))

    def spot_check(self):
        """Parity inside the bench: moved bytes are exact / the reduction matches the oracle on a slab."""
        import torch

        from oracle import collectives as oracle

        M = self.M
        if self.kind == "ag":
            assert torch.equal(self.op.peer_out(1)[:M], self.op.out[:M]) and torch.equal(self.op.out[M:].cpu(), self.peer_cpu)
            return
        # The first 256 rows of owner 1's shard (rank 0 always stores its partial of rows it does
        # not own), handed to the oracle as the owner-0 half of a 512-row problem, owner's addend first.
        half = M // 2
        pad = torch.zeros(256, self.N, dtype=self.peer_cpu.dtype)
        slabs = [torch.cat([self.peer_cpu[half:half + 256], pad]), torch.cat([self.op.partial[half:half + 256].cpu(), pad])]
        want = oracle.reduce_rows(slabs, 0, self.op.out.dtype)
        assert torch.equal(self.ops[1].out[:256].cpu().view(torch.int16), want.view(torch.int16))
        # The rows rank 0 owns: the in-register variants never store that partial, so it cannot be
        # handed to the oracle; every variant timed must have produced the same bytes.
        outs = list(self.own_out.values())
        assert all(torch.equal(o, outs[0]) for o in outs[1:])

    def gemm_only(self):
        import ctypes as C

        from tileccl_amd import _launch, _lib

        target = self.op.local_block if self.kind == "ag" else self.op.partial
        desc = _launch.gemm_desc(self.A, self.B, target, block_m=self.block_m, macro_tile=self.op.macro_tile,
                                 alpha=self.scales[0] * self.scales[1])
        lib = _lib.load()
        return lambda _variant: _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")

    def device_trace(self, variant, macro_tile):
        """One traced launch of `variant` on an operation of its own (stamps cost about 1 us per launch, so
        the timed operation carries none): per TileGroup, when its last tile was published and when the
        transfers that depend on it were finished, in us from the launch's first stamp."""
        import torch

        from tileccl_amd.v2 import FusedGemmAllGather, FusedGemmReduceScatter
        from tileccl_amd.v2.runtime import TimelineRecorder

        common = dict(block_m=self.block_m, macro_tile=macro_tile, target_group_tiles=self.group_tiles, trace=True)
        if self.kind == "ag":
            ops = [FusedGemmAllGather(h, self.M, self.N, torch.float16, directions="both", **common) for h in self.heaps]
            ops[1].out[self.M:].copy_(self.peer_cpu)
        else:
            ops = [FusedGemmReduceScatter(h, self.M, self.N, partial_dtype=self.op.partial.dtype, out_dtype=self.op.out.dtype,
                                          own_rows_in_registers=True, **common) for h in self.heaps]
            ops[1].partial.copy_(self.peer_cpu)
        op = ops[0]
        op.mark_peers_ready()
        for _ in range(3):  # the last launch's stamps are the ones read
            for t in (op.signals.trace_start_clock, op.signals.trace_ready_clock, op.signals.trace_done_clock):
                t.zero_()
            op(self.A, self.B, variant, scale_a=self.scales[0], scale_b=self.scales[1])
        op.check_faults()
        rec = TimelineRecorder(benchmark=self.describe(variant), path_name=variant,
                               metadata={"workload": self.name, "tile_groups": op.plan.n_groups})
        rec.record_signal_state(op.signals, op.plan, rank=0)
        spans = {e.name: e for e in rec.events}
        us = lambda name, end: round((spans[name].end_ms if end else spans[name].start_ms) * 1e3, 2) if name in spans else None  # noqa: E731
        table = {"rows": [list(g[:2]) for g in op.plan.groups],
                 "ready_us": [us(f"group {g} produce", True) for g in range(op.plan.n_groups)],
                 "done_us": [us(f"group {g} transfer", True) for g in range(op.plan.n_groups)]}
        return rec, table

    def s0_host_sync(self):
        """S0 as the reference issues it (patterns/bulk_sync.py:120-135): the GEMM kernel, a device-wide
        synchronize on the host, then the exchange kernel.  All-gather workloads only."""
        import ctypes as C

        import torch

        from tileccl_amd import _launch, _lib

        if self.kind != "ag":
            return None
        gemm, op, lib = self.gemm_only(), self.op, _lib.load()
        view = _launch.heap_view(op.heap.get_heap_bases(), op.rank, op.world_size)
        transport = _launch.transport_desc(op.directions, op.transport.copy_elems, op.transport.reduce_elems, op.num_comm_wgs)

        def run(_variant):
            gemm(_variant)
            torch.cuda.synchronize()
            rc = lib.tccl_exchange_rows(_launch.ptr(op.out), self.M, self.N, int(op.out.stride(0)), op.out.element_size(),
                                        C.byref(view), C.byref(transport), _launch.stream_ptr())
            _lib.check(rc, "tccl_exchange_rows")

        return run

    def library_gemm(self):
        """The same GEMM by torch.matmul (the vendor's GEMM library), for context: B row-major as the
        configurations hold it, and B k-major, the layout that library is fastest with.  16-bit inputs only."""
        import torch

        if self.in_type == "f8":
            return None
        A = self.A.clone()
        B_kn = self.B.clone() if self.b_layout == "kn" else self.B.t().contiguous().t().contiguous()
        B_nk = B_kn.t().contiguous()
        out = torch.empty(self.M, self.N, dtype=A.dtype, device=A.device)
        return {"kn": lambda _v: torch.matmul(A, B_kn, out=out), "nk": lambda _v: torch.matmul(A, B_nk.t(), out=out)}

    def mfma_sustained(self):
        """What the matrix pipes sustain on THIS workload's operand values with nothing else running: a loop of the
        K loop's MFMA instruction on registers filled from A (row operands) and B (column operands), and the same
        loop on all-zero registers (tccl_mfma_rate_probe; TFLOP/s from the difference of two loop lengths)."""
        import torch

        from tileccl_amd.v2.calibrate import mfma_sustained_tflops

        kind = "f8_16x16x128" if self.in_type == "f8" else "f16_16x16x32"
        a, b = self.A.reshape(-1), (self.B if self.b_layout == "kn" else self.B.t()).reshape(-1)
        on_data = mfma_sustained_tflops(kind, a, b)
        zeros = torch.zeros(1 << 22, dtype=a.dtype, device=a.device) if self.in_type != "f8" else \
            torch.zeros(1 << 22, dtype=torch.uint8, device=a.device).view(a.dtype)
        on_zeros = mfma_sustained_tflops(kind, zeros, zeros)
        return {"instruction": kind, "tflops": round(on_data["tflops"], 1), "us_per_tile_step": round(on_data["us_per_step"], 4),
                "on_zero_operands_tflops": round(on_zeros["tflops"], 1),
                "note": "MFMAs only (operands loaded once into registers, no LDS or memory access in the loop), one workgroup of "
                        "8 wavefronts per CU, operand registers filled from this workload's A and B; measured in this run"}

    def live_pair(self, steps=100, warmup=20, wgs=128):
        """Both ranks of the pair for real, at the same time: two launches on two streams, `wgs` workgroups each (they fit
        side by side on the CUs), nothing preset and nothing emulated on a peer's behalf.  Each rank waits inside its
        kernel for the words the other one is writing.  us per pair of launches, all-gather workloads only."""
        import ctypes as C

        import torch

        from tileccl_amd import _launch, _lib
        from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

        if self.kind != "ag":
            return None
        lib = _lib.load()
        pool = [torch.cuda.Stream() for _ in range(8)]
        word = torch.zeros(1, dtype=torch.int32, device="cuda")
        seen = torch.zeros(2, dtype=torch.int32, device="cuda")

        def side_by_side(a, b):
            """A one-lane kernel that waits (20 ms at most) on `a` is released by a kernel launched after it on `b`."""
            for x, y in ((a, b), (b, a)):
                word.zero_()
                seen.zero_()
                torch.cuda.synchronize()
                lib.tccl_prim_wait_ge(_launch.ptr(word), 0, 1, 20_000_000, _launch.ptr(seen), C.c_void_p(x.cuda_stream))
                lib.tccl_prim_signal_add(_launch.ptr(word), 0, 1, _launch.ptr(seen[1:]), C.c_void_p(y.cuda_stream))
                torch.cuda.synchronize()
                if int(seen[0].item()) != 1:
                    return False
            return True

        streams = next(([a, b] for a in pool for b in pool if a is not b and side_by_side(a, b)), None)
        if streams is None:
            return {"us_per_pair": None, "reason": "no two streams of this process ran kernels side by side"}
        M, N, K = self.M, self.N, self.K
        heaps = SymmetricHeap.create_all(1 << 30, 2)
        result = {}
        try:
            operands = []
            for r, h in enumerate(heaps):
                A, B = h.allocate_tensor((M, K), torch.float16), h.allocate_tensor((K, N), torch.float16)
                A.copy_(seeded((M, K), 10 + r))
                B.copy_(seeded((K, N), 15 + r, K**-0.5))
                operands.append((A, B))
            for directions, variants in (("push", ("s0", "s1", "s2")), ("pull", ("s1", "s2"))):
                ops = [FusedGemmAllGather(h, M, N, torch.float16, directions=directions, block_m=self.block_m, num_gemm_wgs=wgs,
                                          macro_tile=self.op.macro_tile, target_group_tiles=self.group_tiles,
                                          spin_limit_ns=300_000_000) for h in heaps]

                def step(variant):
                    for rank in (1, 0):
                        with torch.cuda.stream(streams[rank]):
                            ops[rank](*operands[rank], variant)

                for variant in variants:
                    for _ in range(warmup):
                        step(variant)
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(steps):
                        step(variant)
                    torch.cuda.synchronize()
                    result[f"{variant}_{directions}"] = round((time.perf_counter() - t0) / steps * 1e6, 2)
                    for op in ops:
                        op.check_faults()
                assert torch.equal(ops[0].out[M:], ops[1].out[M:]) and torch.equal(ops[0].out[:M], ops[1].out[:M])
        finally:
            for h in heaps:
                h.cleanup()
        return {"us_per_pair": result, "workgroups_per_rank": wgs,
                "s0_vs_s2_pull": round(result["s0_push"] / result["s2_pull"], 4),
                "s0_vs_s2_push": round(result["s0_push"] / result["s2_push"], 4),
                "note": "two ranks' launches at the same time on two streams, each on half of the CUs, host wall time per pair; "
                        "S0 = GEMM then bulk push per rank; pull = each rank fetches the other's block as its TileGroups "
                        "(S2) / tiles (S1) are published, i.e. not before the peer's K loops have produced them"}

    def cpu_baseline(self, iters=3):
        """The oracle's restatement of the same operation on the host cores (reported, not a target)."""
        import torch

        from oracle import collectives as oracle

        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        M, N = self.M, self.N
        best = float("inf")
        for _ in range(iters):
            t0 = time.perf_counter()
            if self.kind == "ag":
                outs = [torch.zeros(2 * M, N, dtype=torch.float16) for _ in range(2)]
                outs[1][M:] = self.peer_cpu
                oracle.gemm_allgather(self.A_cpu, self.B_cpu, outs, 0)
            else:
                partial = oracle.gemm(self.A_cpu, self.B_cpu, self.peer_cpu.dtype, alpha=self.scales[0] * self.scales[1])
                for owner in (0, 1):
                    oracle.reduce_rows([partial, self.peer_cpu], owner, self.op.out.dtype)
            best = min(best, time.perf_counter() - t0)
        return best, cores

    def close(self):
        for h in self.heaps:
            h.cleanup()


class ChainedWorkload:
    """AllGather -> GEMM -> scatter (ChainedAGGemmRSPattern) with the interface of Workload."""

    SCHEDULES = {"s0": "bulk_sync", "s1": "wg_specialized", "s2": "tile_group"}

    def __init__(self, name, macro_tile):
        import torch

        import tileccl_amd as tileccl
        from tileccl_amd.patterns.chained_ag_gemm_rs import ChainedAGGemmRSPattern

        self.name = name
        self.kind, self.M, self.N, self.K, self.block_m, self.in_type = WORKLOADS[name]
        M, N, K = self.M, self.N, self.K
        self.ctxs = tileccl.init_local(world_size=2, heap_size=1 << 30)
        ks = K // 2
        self.shards_cpu = [seeded((M, ks), 10 + p) for p in range(2)]
        self.W_cpu = seeded((K, N), 1, K**-0.5)
        self.shards, self.outs = [], []
        for c, sc in zip(self.ctxs, self.shards_cpu):
            t = c.zeros(M, ks, dtype=torch.float16)
            t.copy_(sc)
            self.shards.append(t)
            self.outs.append(c.zeros(M, N, dtype=torch.float16))
        self.W = self.ctxs[0].zeros(K, N, dtype=torch.float16)
        self.W.copy_(self.W_cpu)
        self.patterns = {v: ChainedAGGemmRSPattern(self.ctxs[0], schedule=sch) for v, sch in self.SCHEDULES.items()}
        self.last = None
        self.macro_tile = macro_tile
        self.flop = 2.0 * M * N * K
        # gather: both shards read, the gathered input written; scatter: the output read and written once more
        self.exchange_bytes = 2.0 * M * K * 2 + 2.0 * M * N * 2

    # main() reads these through `w.op`
    @property
    def op(self):
        return self

    @property
    def plan(self):
        return self.patterns["s2"]._stage.last_plan

    def check_faults(self):
        if self.last is not None:
            self.last.check_faults()

    def run(self, variant):
        self.last = self.patterns[variant]
        self.last.execute(self.shards[0], self.W, self.outs[0])

    def describe(self, variant):
        M, N, K = self.M, self.N, self.K
        return (f"{self.name}: AllGather -> GEMM -> scatter, 2 column shards {M}x{K // 2} fp16 -> {M}x{K} @ {K}x{N}, "
                f"output stored to both emulated heap slices, schedule {self.SCHEDULES[variant]}")

    def spot_check(self):
        import torch

        from oracle import collectives as oracle

        M, K = self.M, self.K
        gathered = self.ctxs[0].workspace("chained_ag_gemm_rs.gathered_input", M, K, dtype=torch.float16)
        assert torch.equal(gathered.cpu().view(torch.int16), oracle.gather_cols(self.shards_cpu).view(torch.int16))
        assert torch.equal(self.outs[0].view(torch.int16), self.outs[1].view(torch.int16))
        want = oracle.gather_cols([s[:256] for s in self.shards_cpu]).float() @ self.W_cpu.float()
        assert torch.allclose(self.outs[0][:256].float().cpu(), want, rtol=1e-2, atol=1e-1)

    def gemm_only(self):
        import ctypes as C

        import torch

        from tileccl_amd import _launch, _lib

        gathered = self.ctxs[0].workspace("chained_ag_gemm_rs.gathered_input", self.M, self.K, dtype=torch.float16)
        desc = _launch.gemm_desc(gathered, self.W, self.outs[0], block_m=self.block_m, macro_tile=self.macro_tile)
        lib = _lib.load()
        return lambda _variant: _lib.check(lib.tccl_gemm(C.byref(desc), _launch.stream_ptr()), "tccl_gemm")

    def cpu_baseline(self, iters=3):
        import torch

        from oracle import collectives as oracle

        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        best = float("inf")
        for _ in range(iters):
            outs = [torch.zeros(self.M, self.N, dtype=torch.float16) for _ in range(2)]
            t0 = time.perf_counter()
            oracle.chained_ag_gemm_rs(self.shards_cpu, self.W_cpu, outs, 0)
            best = min(best, time.perf_counter() - t0)
        return best, cores

    def close(self):
        for c in self.ctxs:
            c.heap.cleanup()


def probe_mfma_table(repeats=3):
    """Every instruction shape of tccl_mfma_rate_probe on all-zero and on normally distributed operands (row operands
    N(0, 1), column operands N(0, 1/1024): the distributions of the benchmark's A and B), `repeats` measurements each."""
    import torch

    from tileccl_amd.v2.calibrate import PROBE_KINDS, mfma_sustained_tflops

    g = torch.Generator().manual_seed(0)
    n = 1 << 24
    rows, cols = torch.randn(n, generator=g), torch.randn(n, generator=g) / 32
    table = {}
    for kind, (_code, _k, dtype) in PROBE_KINDS.items():
        if dtype == torch.float8_e4m3fn:  # the fp8 recipe of the benchmark: one sigma stored as 64
            a, b = (rows * 64).clamp(-448, 448).to(dtype).cuda(), (cols * 32 * 64).clamp(-448, 448).to(dtype).cuda()
            zeros = torch.zeros(n, dtype=torch.uint8, device="cuda").view(dtype)
        else:
            a, b = rows.to(dtype).cuda(), cols.to(dtype).cuda()
            zeros = torch.zeros(n, dtype=dtype, device="cuda")
        peak = PEAK_TFLOPS["f8" if dtype == torch.float8_e4m3fn else "f16"]
        for name, (x, y) in (("zeros", (zeros, zeros)), ("normal", (a, b))):
            runs = [mfma_sustained_tflops(kind, x, y) for _ in range(repeats)]
            best = max(runs, key=lambda r: r["tflops"])
            table[f"{kind} {name}"] = {"tflops": round(best["tflops"], 1), "us_per_tile_step": round(best["us_per_step"], 4),
                                       "of_published_peak": round(best["tflops"] / peak, 4),
                                       "launch_us": [round(u, 2) for u in best["launch_us"]], "steps": best["steps"]}
    return {"probe": "tccl_mfma_rate_probe", "workgroups": runs[0]["workgroups"], "table": table}


def probe_copy_table(steps=50):
    """What a copy (every byte read once and written once) reaches on this part, by four different kernels: the
    library's `tccl_copy_block` (the loops S0's exchange phase runs), torch's tensor copy (the runtime's
    device-to-device copy), a torch elementwise kernel (`add(src, 0)`), and `tccl_exchange_rows` at c1's shape
    (S0's exchange phase itself, both emulated ranks' blocks).  GB/s counts bytes read plus bytes written."""
    import ctypes as C

    import torch

    from tileccl_amd import _launch, _lib
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap
    from tileccl_amd.primitives import communication

    lib = _lib.load()
    table = {}
    heaps = SymmetricHeap.create_all(size=1536 << 20, world_size=2)
    try:
        h = heaps[0]
        for mib in (32, 64, 512):
            n = mib << 20
            src, dst = h.allocate_tensor((n // 2,), torch.float16), h.allocate_tensor((n // 2,), torch.float16)
            src.normal_()
            runs = {
                "tccl_copy_block": lambda _v, src=src, dst=dst: communication.copy_block(dst, src, h, src_rank=0, dst_ranks=(0,)),
                "torch copy_": lambda _v, src=src, dst=dst: dst.copy_(src),
                "torch add(src, 0)": lambda _v, src=src, dst=dst: torch.add(src, 0, out=dst),
            }
            for name, run in runs.items():
                _, ms = time_variant(run, "copy", steps, 5)
                assert torch.equal(dst, src), name
                table[f"{name} {mib} MiB"] = {"us": round(ms * 1e3, 2), "gbs": round(2 * n / (ms * 1e-3) / 1e9, 1)}
        M, N = WORKLOADS["c1"][1], WORKLOADS["c1"][2]
        outs = [hp.allocate_tensor((2 * M, N), torch.float16) for hp in heaps]
        for r, o in enumerate(outs):
            o[r * M:(r + 1) * M].normal_()
        views = [_launch.heap_view(hp.get_heap_bases(), r, 2) for r, hp in enumerate(heaps)]
        transport = _launch.transport_desc(_lib.DIR_PUSH | _lib.DIR_PULL, 16384, None, 0)

        def exchange(_v):
            rc = lib.tccl_exchange_rows(_launch.ptr(outs[0]), M, N, N, 2, C.byref(views[0]), C.byref(transport), _launch.stream_ptr())
            _lib.check(rc, "tccl_exchange_rows")

        _, ms = time_variant(exchange, "copy", steps, 5)
        moved = 2 * M * N * 2  # this rank's block pushed, the peer's block pulled
        table["tccl_exchange_rows c1 (2 x 32 MiB moved)"] = {"us": round(ms * 1e3, 2), "gbs": round(2 * moved / (ms * 1e-3) / 1e9, 1)}
    finally:
        for hp in heaps:
            hp.cleanup()
    return {"probe": "copy", "peak_gbs": PEAK_HBM_GBS, "table": table}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--variant", default="s2", choices=["s0", "s1", "s2"], help="the variant `value` reports")
    ap.add_argument("--variants", default="s0,s1,s2", help="variants to time (the reported one is always included)")
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--macro-tile", type=int, default=0, choices=[0, 128, 256],
                    help="GEMM tile: 0 lets the library choose, 128 / 256 force a kernel")
    ap.add_argument("--timeline", default=None, metavar="PATH",
                    help="also run one traced launch of the reported variant and write its per-TileGroup timeline "
                         "(tileccl.timeline.v1 JSON) to PATH; the bench line then carries `device_trace`")
    ap.add_argument("--group-tiles", default="default",
                    help="tiles per TileGroup: 'default' (the planner's rule), 'auto' (calibrate this machine and ask the "
                         "cost model), or a number")
    ap.add_argument("--b-layout", default="kn", choices=["kn", "nk"],
                    help="B in memory: 'kn' = (K, N) row-major (the configurations' layout), 'nk' = an (N, K) tensor passed "
                         "as its .t() view (a linear layer's weight)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-live-pair", action="store_true", help="skip the two-live-ranks leg (all-gather workloads)")
    ap.add_argument("--probe-copy", action="store_true",
                    help="only time stand-alone copies (the library's copy loops, torch's copy and an elementwise "
                         "kernel, S0's exchange phase at c1's shape) and print the table as one JSON line")
    ap.add_argument("--probe-mfma", action="store_true",
                    help="only run the MFMA-rate probe (every instruction shape, on zeros and on normally distributed "
                         "operands) and print its table as one JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: peer ranks are emulated as slices of one HBM arena, "
              "so --gpus must be 1", file=sys.stderr)
        return 2

    from tileccl_amd import _lib
    from tileccl_amd.backends import get_backend

    _lib.load()
    if args.probe_mfma:
        print(json.dumps(probe_mfma_table()))
        return 0
    if args.probe_copy:
        print(json.dumps(probe_copy_table()))
        return 0
    props = get_backend().get_device_properties()
    if WORKLOADS[args.workload][0] == "ch":
        w = ChainedWorkload(args.workload, args.macro_tile)
    else:
        w = Workload(args.workload, args.macro_tile, args.group_tiles, args.b_layout)

    results = {}
    wanted = [v for v in ("s0", "s1", "s2") if v in args.variants.split(",") or v == args.variant]
    for variant in wanted:
        wall, mean = time_variant(w.run, variant, args.steps, args.warmup)
        w.op.check_faults()
        if hasattr(w, "after_variant"):
            w.after_variant(variant)
        results[variant] = {"wall_ms": wall, "event_ms_mean": mean, "tflops": w.flop / (mean * 1e-3) / 1e12,
                            "wall_tflops": w.flop / (wall * 1e-3) / 1e12}
        if variant == args.variant:
            spread = launch_spread(w.run, variant)
    w.spot_check()
    push_only = None
    if getattr(w, "push_only", None) is not None:
        w.push_only.mark_peers_ready()
        _, mean = time_variant(w.run_one_direction, args.variant, args.steps, args.warmup)
        w.push_only.check_faults()
        push_only = {"variant": args.variant, "ms": round(mean, 5), "tflops": round(w.flop / (mean * 1e-3) / 1e12, 2),
                     "note": w.one_direction_note}
    _, gemm_mean = time_variant(w.gemm_only(), "s0", args.steps, args.warmup)  # GEMM alone, for the phase split

    library = None
    if getattr(w, "library_gemm", None) and w.library_gemm():
        library = {"note": "torch.matmul (vendor GEMM library) on the same operands, for context: B row-major / B k-major"}
        for layout, run in w.library_gemm().items():
            _, ms = time_variant(run, "s0", args.steps, args.warmup)
            library[f"b_{layout}_ms"] = round(ms, 5)
            library[f"b_{layout}_tflops"] = round(w.flop / (ms * 1e-3) / 1e12, 2)

    peak = PEAK_TFLOPS[w.in_type]
    chosen = results[args.variant]
    tflops = chosen["tflops"]  # per launch, HIP events on the launch stream
    line = {
        "metric": METRIC if args.workload == "c1" else f"fused GEMM+collective TFLOP/s, workload {args.workload}, 1 GPU",
        "value": round(chosen["wall_tflops"], 2),  # whole timed region, host gaps included
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_min_seconds": SETTLE_SECONDS,  # untimed launches continue until this much time has passed
        "ms_per_step": round(chosen["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.in_type,
        "data": "synthetic",
        "config": {
            "workload": w.describe(args.variant),
            "tile_groups": w.op.plan.n_groups,
            "group_tiles": w.op.plan.tile_counts()[0],
            "device": props.name,
            "compute_units": props.compute_units,
        },
        "variants_ms": {v: round(r["event_ms_mean"], 5) for v, r in results.items()},
        "variants_tflops": {v: round(r["tflops"], 2) for v, r in results.items()},
        "mfma_util": {v: round(r["tflops"] / peak, 4) for v, r in results.items()},
        "per_launch_us": spread,  # the reported variant, one event pair per launch
        "gemm_only_ms": round(gemm_mean, 5),
        "gemm_only_tflops": round(w.flop / (gemm_mean * 1e-3) / 1e12, 2),
        "roofline": {
            "bound": "mfma",
            "achieved": round(tflops, 2),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(tflops / peak, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, args.variant, args.macro_tile))
            if args.group_tiles == "default" and args.b_layout == "kn" else None,
            "kernel_ms": round(chosen["event_ms_mean"], 5),
        },
    }
    if getattr(w, "mfma_sustained", None):
        sustained = w.mfma_sustained()
        line["roofline"]["sustained_peak"] = sustained["tflops"]  # beside `peak`, never instead of it
        line["roofline"]["frac_of_sustained"] = round(tflops / sustained["tflops"], 4)
        line["mfma_sustained"] = sustained
        line["gemm_only_frac_of_sustained"] = round(line["gemm_only_tflops"] / sustained["tflops"], 4)
    if getattr(w, "calibration", None):
        line["config"]["calibration"] = w.calibration
    if args.b_layout != "kn":
        line["config"]["b_layout"] = "B held as (N, K), passed as its .t() view"
    if push_only is not None:
        line["one_direction"] = push_only
    if library is not None:
        line["library_gemm"] = library
    if "s0" in results and "s2" in results:
        line["s2_vs_s0_speedup"] = round(results["s0"]["event_ms_mean"] / results["s2"]["event_ms_mean"], 4)
    if args.timeline and getattr(w, "device_trace", None):
        recorder, table = w.device_trace(args.variant, args.macro_tile)
        recorder.write_json(args.timeline)
        line["device_trace"] = table
    if "s0" in results and getattr(w, "s0_host_sync", None) and w.s0_host_sync():
        _, ms = time_variant(w.s0_host_sync(), "s0", args.steps, args.warmup)
        line["s0_host_sync"] = {
            "ms": round(ms, 5),
            "note": "S0 with the reference's host-side device synchronize between the GEMM and the exchange kernel "
                    "(variants_ms.s0 orders the two kernels by the stream alone)",
        }
    if "s0" in results:
        phase_ms = results["s0"]["event_ms_mean"] - gemm_mean
        line["exchange_phase"] = {
            "bytes": w.exchange_bytes,
            "s0_phase_ms": round(phase_ms, 5),
            "s0_phase_gbs": round(w.exchange_bytes / (phase_ms * 1e-3) / 1e9, 1),
            "peak_gbs": PEAK_HBM_GBS,
        }
    if not args.no_live_pair and getattr(w, "live_pair", None):
        pair = w.live_pair()
        if pair is not None:
            line["live_pair"] = pair
    if not args.no_cpu:
        secs, cores = w.cpu_baseline()
        line["cpu_baseline"] = {
            "value": round(w.flop / secs / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": cores,
            "kind": "port",
            "sample": f"the full {args.workload} operation (torch CPU fp32 matmul + block copies / fp32 sums), best of 3",
            "ms": round(secs * 1e3, 2),
        }
    w.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
