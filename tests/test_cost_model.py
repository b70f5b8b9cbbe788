"""Cost model: closed-form floats and exact recovery of synthetic link parameters
(reference tileccl_v2/cost_model.py)."""

import math

import pytest

from tileccl_amd.v2 import (
    CalibrationPoint,
    CostModelCalibrator,
    HardwareProfile,
    Interconnect,
    TileCostModel,
    build_tile_group_plan,
    choose_target_group_tiles,
)


def test_presets_and_bandwidth():
    p = HardwareProfile.from_interconnect(Interconnect.NVLINK_4)
    assert (p.alpha_us, p.gemm_tflops_fp16, p.gemm_efficiency, p.name) == (1.0, 989.0, 0.75, "NVLink 4.0 (H100)")
    assert p.beta_us_per_byte == pytest.approx(1e6 / 450e9)
    assert p.bandwidth_gb_s == pytest.approx(450.0)
    assert HardwareProfile(1.0, 0.0, 100.0).bandwidth_gb_s == math.inf
    with pytest.raises(ValueError, match="Use HardwareProfile\\(\\) directly"):
        HardwareProfile.from_interconnect(Interconnect.CUSTOM)
    mi = HardwareProfile.from_interconnect(Interconnect.XGMI_MI355X)
    assert mi.bandwidth_gb_s == pytest.approx(153.0) and mi.gemm_tflops_fp16 == 2500.0


def test_tile_costs_closed_form():
    m = TileCostModel(HardwareProfile.from_interconnect(Interconnect.NVLINK_4))
    assert m.tile_comm_time(128, 128) == pytest.approx(1.0 + 32768 / 450e3)  # 1.0728 us
    assert m.tile_comm_time(128, 128, "float32") == pytest.approx(1.0 + 65536 / 450e3)
    assert m.tile_comm_time(128, 128, "no-such-dtype") == m.tile_comm_time(128, 128)  # unknown -> 2 bytes
    assert m.tile_compute_time(128, 128, 1024) == pytest.approx(2 * 128 * 128 * 1024 / (989 * 0.75e6))
    c = m.tile_cost(128, 128, 1024)
    assert c.tile_bytes == 32768
    assert c.sequential_us == pytest.approx(c.comm_us + c.compute_us)
    assert c.overlapped_us == max(c.comm_us, c.compute_us)
    assert c.compute_bound == (c.compute_us >= c.comm_us)
    floor = TileCostModel(HardwareProfile(1.0, 1e-6, 100.0, min_comm_us=37.0))
    assert floor.tile_comm_time(8, 8) == 37.0
    assert TileCostModel(HardwareProfile(1.0, 1e-6, 0.0)).tile_compute_time(1, 1, 1) == math.inf


def test_pipeline_cost():
    m = TileCostModel(HardwareProfile(alpha_us=2.0, beta_us_per_byte=1e-4, gemm_tflops_fp16=1.0, gemm_efficiency=1.0))
    one = m.tile_cost(16, 16, 16)  # comm = 2 + 512e-4 = 2.0512 ; compute = 8192/1e6
    p = m.pipeline_cost(10, 16, 16, 16)
    assert p.sequential_us == pytest.approx(10 * one.sequential_us)
    assert p.pipelined_us == pytest.approx(one.sequential_us + 9 * one.overlapped_us)
    assert p.overlap_ratio == pytest.approx(1 - p.pipelined_us / p.sequential_us)
    assert p.bottleneck == "comm" and len(p.tile_costs) == 10
    assert p.speedup == pytest.approx(p.sequential_us / p.pipelined_us)
    assert "10 tiles" in p.summary() and "bottleneck=comm" in p.summary()
    assert m.pipeline_cost(1, 16, 16, 16).pipelined_us == pytest.approx(one.sequential_us)
    # chunking pays alpha per chunk
    p4 = m.pipeline_cost(3, 16, 16, 16, n_chunks=4)
    assert p4.tile_costs[0].comm_us == pytest.approx(4 * (2.0 + 128 * 1e-4))


def test_optimal_tile_size():
    m = TileCostModel(HardwareProfile.from_interconnect(Interconnect.NVLINK_4))
    size, cost = m.optimal_tile_size(4096, 4096, 1024)
    brute = {}
    for s in (32, 64, 128, 256, 512):
        brute[s] = m.pipeline_cost((4096 // s) ** 2, s, s, 1024).pipelined_us
    assert size == min(brute, key=brute.get) and cost.pipelined_us == pytest.approx(brute[size])
    size, cost = m.optimal_tile_size(16, 16, 16)  # nothing fits
    assert size == 32 and cost is None


def test_calibration_recovers_linear_law():
    alpha, beta = 3.5, 2.0e-5
    pts = [CalibrationPoint(n, n, "float16", alpha + beta * n * n * 2) for n in (64, 128, 256, 512, 1024)]
    a, b = CostModelCalibrator.calibrate_comm(pts)
    assert a == pytest.approx(alpha, rel=1e-9) and b == pytest.approx(beta, rel=1e-9)
    a, b = CostModelCalibrator.calibrate_comm(pts, min_bytes_threshold=128 * 128 * 2)
    assert a == pytest.approx(alpha) and b == pytest.approx(beta)
    with pytest.raises(ValueError, match="Need at least 2 calibration points"):
        CostModelCalibrator.calibrate_comm(pts[:1])
    with pytest.raises(ValueError, match=r"Need at least 2 points with bytes >= 99999999, got 0"):
        CostModelCalibrator.calibrate_comm(pts, min_bytes_threshold=99999999)
    with pytest.raises(ValueError, match="Degenerate calibration data"):
        CostModelCalibrator.calibrate_comm([pts[0], pts[0]])
    # negative intercept clamps to zero
    a, b = CostModelCalibrator.calibrate_comm([CalibrationPoint(1, 50, "int8", 0.0), CalibrationPoint(1, 100, "int8", 10.0)])
    assert a == 0.0 and b == pytest.approx(0.2)


def test_two_regime_fit():
    # floor at 2 MiB (40 us), then a bandwidth line above it
    alpha, beta = 5.0, 1e-5
    sizes = [256, 512, 1024, 2048, 4096, 8192]
    us = [60.0, 50.0, 40.0] + [alpha + beta * s * s * 2 for s in sizes[3:]]
    pts = [CalibrationPoint(s, s, "float16", t) for s, t in zip(sizes, us)]
    a, b, floor = CostModelCalibrator.calibrate_two_regime(pts)
    assert floor == 40.0 and a == pytest.approx(alpha) and b == pytest.approx(beta)
    prof = CostModelCalibrator.calibrate_from_measurements(
        pts, HardwareProfile.from_interconnect(Interconnect.NVLINK_4), two_regime=True
    )
    assert prof.min_comm_us == 40.0 and prof.name == "NVLink 4.0 (H100) (calibrated)" and prof.gemm_tflops_fp16 == 989.0
    with pytest.raises(ValueError, match="Need at least 3 calibration points"):
        CostModelCalibrator.calibrate_two_regime(pts[:2])
    # minimum at the largest point: falls back to the two largest payloads
    falling = [CalibrationPoint(s, s, "float16", 100.0 - i) for i, s in enumerate(sizes)]
    a, b, floor = CostModelCalibrator.calibrate_two_regime(falling)
    assert floor == 95.0 and b == 0.0
    plain = CostModelCalibrator.calibrate_from_measurements(pts[3:], HardwareProfile(1, 1, 1.0))
    assert plain.min_comm_us == 0.0 and plain.alpha_us == pytest.approx(alpha)


def test_choose_target_group_tiles_feeds_the_planner():
    model = TileCostModel(HardwareProfile.from_interconnect(Interconnect.HBM_MI355X))
    tiles = choose_target_group_tiles(model, 8192, 4096, 1024)
    assert tiles % 256 == 0 and 256 <= tiles <= 2048  # whole swizzle waves
    plan = build_tile_group_plan(8192, 4096, 32768, target_group_tiles=tiles)
    assert all(t >= tiles for t in plan.tile_counts()[:-1])
    # a slow link with a large start-up cost prefers fewer, larger groups than a fast one
    slow = TileCostModel(HardwareProfile(alpha_us=500.0, beta_us_per_byte=1e-6, gemm_tflops_fp16=2500.0))
    fast = TileCostModel(HardwareProfile(alpha_us=0.1, beta_us_per_byte=1e-7, gemm_tflops_fp16=2500.0))
    assert choose_target_group_tiles(slow, 16384, 4096, 1024) >= choose_target_group_tiles(fast, 16384, 4096, 1024)


def test_group_size_rule_prices_a_group_inside_a_launch_without_the_launch():
    """Calibration points are stand-alone launches: ~7 us of latency that a TileGroup moved by a
    running kernel does not pay.  Priced with it, one huge group wins (fewest launches); priced
    without it, groups stay as small as the saturation floor allows, so that they pipeline."""
    from tileccl_amd.v2.calibrate import Calibration
    from tileccl_amd.v2.cost_model import HardwareProfile

    prof = HardwareProfile(alpha_us=7.6, beta_us_per_byte=1e6 / 7.0e12, gemm_tflops_fp16=2500.0, gemm_efficiency=0.4,
                           min_comm_us=7.2, name="measured")
    cal = Calibration((), prof, 1000.0, int(7.6 / prof.beta_us_per_byte))
    inside = cal.in_launch_profile()
    assert inside.alpha_us == pytest.approx(0.4) and inside.min_comm_us == 0.0
    assert inside.beta_us_per_byte == prof.beta_us_per_byte
    # 8192 x 4096, 128 x 128 tiles: 8 swizzle waves of 256 tiles
    assert cal.target_group_tiles(8192, 4096, 1024, in_launch=False) == 2048
    assert cal.target_group_tiles(8192, 4096, 1024) == 256
    assert cal.target_group_tiles(8192, 4096, 1024, block_m=256) == 256
    # a link with real latency (xGMI-like: 2 us, 150 GB/s) asks for larger groups
    slow = HardwareProfile(alpha_us=9.2, beta_us_per_byte=1e6 / 150e9, gemm_tflops_fp16=2500.0, gemm_efficiency=0.4,
                           min_comm_us=7.2, name="link")
    assert Calibration((), slow, 1000.0, 1).target_group_tiles(8192, 4096, 1024) >= 256


def test_allreduce_cost_is_two_pipelines_of_the_shard_transfers():
    """M = 1024 rows over 4 ranks, 128-tiles: a shard is 2 x 4 = 8 tiles, each half moves 3 shards = 24 tiles.
    With alpha = 1 us, 1 GB/s... chosen so that a tile's transfer (32 KiB) and compute are round numbers."""
    from tileccl_amd.v2.cost_model import HardwareProfile, TileCostModel

    profile = HardwareProfile(alpha_us=1.0, beta_us_per_byte=1.0 / 32768, gemm_tflops_fp16=1.0, gemm_efficiency=1.0, name="toy")
    model = TileCostModel(profile)
    one = model.tile_cost(128, 128, 512, "float16")
    assert one.comm_us == pytest.approx(2.0)  # 1 us + 32768 B at 32768 B/us
    cost = model.allreduce_cost(1024, 512, 512, world_size=4)
    assert set(cost) == {"reduce_scatter", "allgather", "total"}
    for half in ("reduce_scatter", "allgather"):
        assert len(cost[half].tile_costs) == 24
        assert cost[half].sequential_us == pytest.approx(24 * one.sequential_us)
        assert cost[half].pipelined_us == pytest.approx(one.sequential_us + 23 * one.overlapped_us)
    total = cost["total"]
    assert len(total.tile_costs) == 48
    assert total.sequential_us == pytest.approx(48 * one.sequential_us)
    assert total.pipelined_us == pytest.approx(2 * (one.sequential_us + 23 * one.overlapped_us))
    assert total.overlap_ratio == pytest.approx(1.0 - total.pipelined_us / total.sequential_us)
    assert total.bottleneck == cost["reduce_scatter"].bottleneck
