"""alpha-beta transfer model + peak-rate GEMM model, used to size TileGroups.

Same public surface and arithmetic as ``/root/reference/tileccl_v2/cost_model.py``:

* transfer time  ``max(min_comm_us, alpha_us + bytes * beta_us_per_byte)``   (ref :222-236)
* GEMM time      ``2*M*N*K / (tflops * efficiency * 1e6)`` microseconds     (ref :238-256)
* pipeline       ``seq_one + (n - 1) * max(comm, compute)``                  (ref :318-322)
* calibration    ordinary least squares on (bytes, microseconds) points, and a
                 two-regime fit that takes the fastest point as a latency floor (ref :445-593)

Added for this build (the reference ships A100/H100 presets only, ref :96-125): MI355X
profiles for one xGMI link and for the single-GPU emulation where the "link" is HBM, and
``choose_target_group_tiles``, the rule that turns the model into a TileGroup size (the
reference's own rule lives in scripts that are not part of its tree).
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from enum import Enum, auto
from typing import Optional, Sequence

DTYPE_BYTES = {
    "float16": 2,
    "bfloat16": 2,
    "float32": 4,
    "float64": 8,
    "int8": 1,
    "int32": 4,
    "float8_e4m3": 1,
}


def _nbytes(rows: int, cols: int, dtype: str) -> int:
    return rows * cols * DTYPE_BYTES.get(dtype, 2)


class Interconnect(Enum):
    PCIE_GEN4 = auto()
    PCIE_GEN5 = auto()
    NVLINK_3 = auto()
    NVLINK_4 = auto()
    CUSTOM = auto()
    XGMI_MI355X = auto()  # one point-to-point xGMI link between two MI355X
    HBM_MI355X = auto()  # peer emulated as a slice of the same HBM (single GPU)


# (alpha_us, GB/s, peak fp16 TFLOP/s, efficiency, name)
_PRESETS = {
    Interconnect.PCIE_GEN4: (5.0, 25.0, 312.0, 0.6, "PCIe Gen4 (A100)"),
    Interconnect.PCIE_GEN5: (3.0, 50.0, 989.0, 0.65, "PCIe Gen5 (H100)"),
    Interconnect.NVLINK_3: (1.5, 300.0, 312.0, 0.7, "NVLink 3.0 (A100)"),
    Interconnect.NVLINK_4: (1.0, 450.0, 989.0, 0.75, "NVLink 4.0 (H100)"),
    Interconnect.XGMI_MI355X: (2.0, 153.0, 2500.0, 0.6, "xGMI link (MI355X)"),
    Interconnect.HBM_MI355X: (2.0, 4000.0, 2500.0, 0.6, "HBM3E slice copy (MI355X)"),
}


@dataclass(frozen=True)
class HardwareProfile:
    """Link latency/bandwidth and GEMM rate of one machine."""

    alpha_us: float
    beta_us_per_byte: float
    gemm_tflops_fp16: float
    gemm_efficiency: float = 0.7
    min_comm_us: float = 0.0
    name: str = "custom"

    @property
    def bandwidth_gb_s(self) -> float:
        if self.beta_us_per_byte <= 0:
            return float("inf")
        return 1.0 / (self.beta_us_per_byte * 1e-6) / 1e9

    @classmethod
    def from_interconnect(cls, interconnect: Interconnect) -> "HardwareProfile":
        if interconnect == Interconnect.CUSTOM:
            raise ValueError("Use HardwareProfile() directly for custom parameters")
        alpha, gb_s, tflops, eff, name = _PRESETS[interconnect]
        return cls(
            alpha_us=alpha,
            beta_us_per_byte=1e6 / (gb_s * 1e9),
            gemm_tflops_fp16=tflops,
            gemm_efficiency=eff,
            name=name,
        )


@dataclass
class TileCost:
    comm_us: float
    compute_us: float
    tile_bytes: int
    overlap_possible: bool = True

    @property
    def sequential_us(self) -> float:
        return self.comm_us + self.compute_us

    @property
    def overlapped_us(self) -> float:
        return max(self.comm_us, self.compute_us)

    @property
    def compute_bound(self) -> bool:
        return self.compute_us >= self.comm_us


@dataclass
class PipelineCost:
    tile_costs: list[TileCost]
    sequential_us: float
    pipelined_us: float
    overlap_ratio: float
    bottleneck: str

    @property
    def speedup(self) -> float:
        return 1.0 if self.pipelined_us <= 0 else self.sequential_us / self.pipelined_us

    def summary(self) -> str:
        return (
            f"Pipeline: {len(self.tile_costs)} tiles, "
            f"seq={self.sequential_us:.1f}µs, pipe={self.pipelined_us:.1f}µs, "
            f"speedup={self.speedup:.2f}x, overlap={self.overlap_ratio:.1%}, "
            f"bottleneck={self.bottleneck}"
        )


class TileCostModel:
    """Per-tile and per-pipeline predictions from a ``HardwareProfile``."""

    def __init__(self, profile: HardwareProfile) -> None:
        self.profile = profile

    def _transfer_us(self, nbytes: float) -> float:
        p = self.profile
        return max(p.min_comm_us, p.alpha_us + nbytes * p.beta_us_per_byte)

    def tile_comm_time(self, tile_M: int, tile_N: int, dtype: str = "float16") -> float:
        return self._transfer_us(_nbytes(tile_M, tile_N, dtype))

    def tile_compute_time(self, tile_M: int, tile_N: int, tile_K: int, dtype: str = "float16") -> float:
        rate = self.profile.gemm_tflops_fp16 * self.profile.gemm_efficiency
        if rate <= 0:
            return float("inf")
        return 2.0 * tile_M * tile_N * tile_K / (rate * 1e6)

    def tile_cost(self, tile_M: int, tile_N: int, tile_K: int, dtype: str = "float16") -> TileCost:
        return TileCost(
            comm_us=self.tile_comm_time(tile_M, tile_N, dtype),
            compute_us=self.tile_compute_time(tile_M, tile_N, tile_K, dtype),
            tile_bytes=_nbytes(tile_M, tile_N, dtype),
        )

    def pipeline_cost(
        self,
        n_tiles: int,
        tile_M: int,
        tile_N: int,
        tile_K: int,
        dtype: str = "float16",
        n_chunks: int = 1,
    ) -> PipelineCost:
        """Cost of ``n_tiles`` identical stages; the first pays comm+compute, the rest overlap.

        With ``n_chunks > 1`` a tile's transfer is split into chunks that each pay
        ``alpha`` (no latency floor is applied to the chunks).
        """
        one = self.tile_cost(tile_M, tile_N, tile_K, dtype)
        if n_chunks > 1:
            per_chunk = self.profile.alpha_us + (one.tile_bytes // n_chunks) * self.profile.beta_us_per_byte
            one = TileCost(comm_us=per_chunk * n_chunks, compute_us=one.compute_us, tile_bytes=one.tile_bytes)

        sequential = one.sequential_us * n_tiles
        pipelined = one.sequential_us + max(n_tiles - 1, 0) * one.overlapped_us
        return PipelineCost(
            tile_costs=[one] * n_tiles,
            sequential_us=sequential,
            pipelined_us=pipelined,
            overlap_ratio=(1.0 - pipelined / sequential) if sequential > 0 else 0.0,
            bottleneck="compute" if one.compute_bound else "comm",
        )

    def optimal_tile_size(
        self,
        M: int,
        N: int,
        K: int,
        dtype: str = "float16",
        candidates: Optional[Sequence[int]] = None,
    ) -> tuple[int, Optional[PipelineCost]]:
        """Square tile edge (from ``candidates``) with the smallest pipelined time."""
        sizes = [32, 64, 128, 256, 512] if candidates is None else list(candidates)
        best_size, best = sizes[0], None
        for edge in sizes:
            if edge > M or edge > N:
                continue
            cost = self.pipeline_cost(
                n_tiles=math.ceil(M / edge) * math.ceil(N / edge),
                tile_M=edge,
                tile_N=edge,
                tile_K=K,
                dtype=dtype,
            )
            if best is None or cost.pipelined_us < best.pipelined_us:
                best_size, best = edge, cost
        return best_size, best

    def allreduce_cost(self, M: int, N: int, K: int, world_size: int, tile_size: int = 128,
                       dtype: str = "float16") -> "dict[str, PipelineCost]":
        """All-reduce of an ``M x N`` output priced as its two halves (reference
        ``tileccl_v2/cost_model.py:381-432``): a reduce-scatter and an all-gather, each a pipeline of the
        ``(world_size - 1)`` transfers of a rank's row shard, tile by tile; ``total`` adds the two
        (no overlap between the halves is assumed)."""
        shard_tiles = math.ceil((M // world_size) / tile_size) * math.ceil(N / tile_size)
        halves = {
            name: self.pipeline_cost(n_tiles=shard_tiles * (world_size - 1), tile_M=tile_size, tile_N=tile_size, tile_K=K, dtype=dtype)
            for name in ("reduce_scatter", "allgather")
        }
        sequential = sum(h.sequential_us for h in halves.values())
        pipelined = sum(h.pipelined_us for h in halves.values())
        halves["total"] = PipelineCost(
            tile_costs=[c for h in list(halves.values()) for c in h.tile_costs],
            sequential_us=sequential,
            pipelined_us=pipelined,
            overlap_ratio=(1.0 - pipelined / sequential) if sequential > 0 else 0.0,
            bottleneck=halves["reduce_scatter"].bottleneck,
        )
        return halves

    # -- TileGroup sizing ---------------------------------------------------
    def group_pipeline_us(
        self, n_groups: int, group_tiles: int, tile_M: int, tile_N: int, K: int, dtype: str, parallel_tiles: int
    ) -> float:
        """Predicted time when tiles are produced ``parallel_tiles`` at a time and moved per group.

        A group's compute time is the time of its tile waves; its transfer is one message of
        ``group_tiles`` tiles.  Groups pipeline like stages: the first pays both, later ones the
        larger of the two.
        """
        # ``parallel_tiles`` tiles run side by side, each at 1/parallel_tiles of the machine
        # rate, so one wave of tiles lasts parallel_tiles single-tile times.
        waves = math.ceil(group_tiles / max(parallel_tiles, 1))
        compute = waves * max(parallel_tiles, 1) * self.tile_compute_time(tile_M, tile_N, K, dtype)
        comm = self._transfer_us(group_tiles * _nbytes(tile_M, tile_N, dtype))
        return compute + comm + max(n_groups - 1, 0) * max(compute, comm)


def choose_target_group_tiles(
    model: TileCostModel,
    M: int,
    N: int,
    K: int,
    *,
    block_m: int = 128,
    block_n: int = 128,
    group_m: int = 8,
    dtype: str = "float16",
    parallel_tiles: int = 256,
    tau_min_bytes: int = 262144,
    max_groups: int = 64,
) -> int:
    """Pick ``target_group_tiles`` for ``build_tile_group_plan`` from the cost model.

    Candidates are whole numbers of swizzle waves (``group_m * tile_cols`` tiles), because
    the planner only closes groups on wave borders.  Each candidate is scored with
    ``TileCostModel.group_pipeline_us`` and the fastest wins; ties go to the larger group
    (fewer signals).  Candidates below the saturation size ``ceil(tau_min_bytes/tile_bytes)``
    are skipped, as are ones that would need more than ``max_groups`` groups.
    """
    tile_rows = math.ceil(M / block_m)
    tile_cols = math.ceil(N / block_n)
    wave_tiles = group_m * tile_cols
    n_waves = math.ceil(tile_rows / group_m)
    floor_tiles = max(1, math.ceil(tau_min_bytes / _nbytes(block_m, block_n, dtype)))

    best_tiles, best_us = wave_tiles * n_waves, float("inf")
    for waves_per_group in range(1, n_waves + 1):
        tiles = waves_per_group * wave_tiles
        n_groups = math.ceil(n_waves / waves_per_group)
        if tiles < floor_tiles or n_groups > max_groups:
            continue
        us = model.group_pipeline_us(n_groups, tiles, block_m, block_n, K, dtype, parallel_tiles)
        if us <= best_us:
            best_tiles, best_us = tiles, us
    return best_tiles


@dataclass
class CalibrationPoint:
    """One measured transfer: a ``tile_M x tile_N`` payload of ``dtype`` took ``measured_comm_us``."""

    tile_M: int
    tile_N: int
    dtype: str
    measured_comm_us: float
    measured_compute_us: Optional[float] = None

    @property
    def nbytes(self) -> int:
        return _nbytes(self.tile_M, self.tile_N, self.dtype)


class CostModelCalibrator:
    """Fit ``alpha``/``beta`` (and optionally a latency floor) to measured transfers."""

    @staticmethod
    def calibrate_comm(points: Sequence[CalibrationPoint], min_bytes_threshold: int = 0) -> tuple[float, float]:
        """Least-squares line through (bytes, us); negative coefficients clamp to 0."""
        if len(points) < 2:
            raise ValueError("Need at least 2 calibration points")
        kept = [p for p in points if p.nbytes >= min_bytes_threshold]
        if len(kept) < 2:
            raise ValueError(
                f"Need at least 2 points with bytes >= {min_bytes_threshold}, got {len(kept)}"
            )
        n = len(kept)
        sx = sy = sxy = sxx = 0.0
        for p in kept:
            x, y = p.nbytes, p.measured_comm_us
            sx += x
            sy += y
            sxy += x * y
            sxx += x * x
        det = n * sxx - sx * sx
        if abs(det) < 1e-12:
            raise ValueError("Degenerate calibration data (all same size)")
        beta = (n * sxy - sx * sy) / det
        alpha = (sy - beta * sx) / n
        return max(0.0, alpha), max(0.0, beta)

    @staticmethod
    def calibrate_two_regime(points: Sequence[CalibrationPoint]) -> tuple[float, float, float]:
        """``(alpha, beta, floor)``: floor = fastest point; line fitted to larger, slower points.

        Falls back to the two largest payloads when fewer than two points lie in the
        bandwidth regime.
        """
        if len(points) < 3:
            raise ValueError("Need at least 3 calibration points for two-regime fit")
        by_size = sorted(points, key=lambda p: p.nbytes)
        knee = min(range(len(by_size)), key=lambda i: by_size[i].measured_comm_us)
        floor_us, knee_bytes = by_size[knee].measured_comm_us, by_size[knee].nbytes
        bandwidth_side = [p for p in by_size if p.nbytes > knee_bytes and p.measured_comm_us > floor_us]
        fit_on = bandwidth_side if len(bandwidth_side) >= 2 else by_size[-2:]
        alpha, beta = CostModelCalibrator.calibrate_comm(fit_on)
        return alpha, beta, floor_us

    @staticmethod
    def calibrate_from_measurements(
        points: Sequence[CalibrationPoint],
        base_profile: HardwareProfile,
        two_regime: bool = False,
    ) -> HardwareProfile:
        """New profile with fitted link terms and ``base_profile``'s GEMM terms."""
        if two_regime:
            alpha, beta, floor_us = CostModelCalibrator.calibrate_two_regime(points)
        else:
            alpha, beta = CostModelCalibrator.calibrate_comm(points)
            floor_us = 0.0
        return HardwareProfile(
            alpha_us=alpha,
            beta_us_per_byte=beta,
            gemm_tflops_fp16=base_profile.gemm_tflops_fp16,
            gemm_efficiency=base_profile.gemm_efficiency,
            min_comm_us=floor_us,
            name=f"{base_profile.name} (calibrated)",
        )
