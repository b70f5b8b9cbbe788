"""GEMM-output AllGather (Gate 1) in the S0 / S1 / S2 variants against the CPU oracle.

Placement and copied bytes must be bit-exact against the GEMM output; the GEMM itself is
held to the fp32-matmul tolerance.  The full-size benchmark configurations are covered through
size-independent properties (both slices end identical, idempotence, counters)."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu

VARIANTS = ["s0", "s1", "s2"]
# 128: one launch whose workgroups split into a GEMM role and a communication role.
# 256: large-tile launch; pushes leave from the GEMM epilogue, S2 pulls run inside the K loop.
MACRO = [128, 256]


def make(world, M, N, dtype=torch.float16, heap_bytes=256 << 20, **kw):
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(heap_bytes, world)
    ops = [FusedGemmAllGather(h, M, N, dtype, **kw) for h in heaps]
    return heaps, ops


def fill_peer_blocks(ops, M, N, dtype, seed=2):
    """Each peer's own row block is a seeded N(0,1) tensor resident in its slice."""
    blocks = {}
    for p, op in enumerate(ops):
        if p == 0:
            continue
        blocks[p] = seeded((M, N), seed + p, dtype)
        op.out.zero_()
        op.out[p * M:(p + 1) * M].copy_(blocks[p])
    return blocks


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("directions", ["both", "push", "pull"])
@pytest.mark.parametrize("macro", MACRO)
def test_small_two_ranks_against_oracle(lib, variant, directions, macro):
    M, N, K = 512, 512, 256
    heaps, ops = make(2, M, N, directions=directions, macro_tile=macro)
    try:
        op = ops[0]
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        blocks = fill_peer_blocks(ops, M, N, torch.float16)
        op.out.zero_()
        op.mark_peers_ready()
        op(A, B, variant)
        op.check_faults()
        # oracle on identical bits: slices as CPU tensors
        outs = [torch.zeros(2 * M, N, dtype=torch.float16) for _ in range(2)]
        outs[1][M:] = blocks[1]
        oracle.gemm_allgather(A_cpu, B_cpu, outs, 0, push=directions != "pull", pull=directions != "push")
        mine = op.out[:M].clone()
        assert_gemm_close(mine, A_cpu.float() @ B_cpu.float(), tight=0.004)
        assert (mine.cpu().float() - outs[0][:M].float()).abs().max().item() <= 0.004
        # everything that was *moved* is bit-exact
        if directions != "pull":
            assert torch.equal(bits(op.peer_out(1)[:M]), bits(mine))
        else:
            assert torch.count_nonzero(op.peer_out(1)[:M]).item() == 0  # nothing pushed
        if directions != "push":
            assert torch.equal(bits(op.out[M:]).cpu(), bits(blocks[1]))
        else:
            assert torch.count_nonzero(op.out[M:]).item() == 0  # nothing pulled
        assert torch.equal(bits(op.peer_out(1)[M:]).cpu(), bits(blocks[1]))  # the peer's own block is untouched
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("macro", MACRO)
def test_ragged_shape_four_ranks_many_groups(lib, variant, macro):
    """M not a multiple of the tile, several groups per rank, fan-out to three peers."""
    M, N, K = 1000, 264, 72
    heaps, ops = make(4, M, N, dtype=torch.bfloat16, tau_min_bytes=1, group_m=2, macro_tile=macro,
                      transport=__import__("tileccl_amd.v2", fromlist=["x"]).build_p2p_transport_plan(
                          comm_mode="push", copy_elems=1024))
    try:
        op = ops[0]
        assert op.plan.n_groups == 4 and op.plan.row_ends()[-1] == M
        A_cpu, B_cpu = seeded((M, K), 0, torch.bfloat16), seeded((K, N), 1, torch.bfloat16, scale=K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        blocks = fill_peer_blocks(ops, M, N, torch.bfloat16)
        op.out.zero_()
        op.mark_peers_ready()
        op(A, B, variant)
        op.check_faults()
        mine = op.out[:M].clone()
        assert_gemm_close(mine, A_cpu.float() @ B_cpu.float(), tight=0.032)
        for p in (1, 2, 3):
            assert torch.equal(bits(op.peer_out(p)[:M]), bits(mine)), f"push to {p}"
            assert torch.equal(bits(op.out[p * M:(p + 1) * M]).cpu(), bits(blocks[p])), f"pull from {p}"
        if variant == "s2":
            assert op.signals.counter.tolist() == oracle.expected_counters(op.plan.tile_counts())
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("local_M,block_m", [(4096, 128), (8192, 128), (8192, 256)])
def test_baseline_configs_1_and_2_properties(lib, local_M, block_m):
    """Configs 1 and 2 at full size: all variants give the same bytes, both slices end up
    identical, the gathered output equals [GEMM rows | peer rows], counters hit tile counts."""
    M, N, K = local_M, 4096, 1024
    heaps, ops = make(2, M, N, heap_bytes=1 << 30, block_m=block_m)
    try:
        op = ops[0]
        n_groups = M // (8 * block_m)
        assert op.plan.n_groups == n_groups and op.plan.tile_counts() == [256] * n_groups
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=K**-0.5))
        peer = seeded((M, N), 2)
        results = {}
        for variant in VARIANTS:
            op.out.zero_()
            ops[1].out.zero_()
            ops[1].out[M:].copy_(peer)
            op.mark_peers_ready()
            op(A, B, variant)
            op.check_faults()
            assert torch.equal(bits(op.out), bits(op.peer_out(1))), variant  # checksum of checksums: whole slices agree
            assert torch.equal(bits(op.out[M:]).cpu(), bits(peer)), variant
            results[variant] = op.out[:M].clone()
            # idempotence: a second launch changes nothing
            op.mark_peers_ready()
            op(A, B, variant)
            op.check_faults()
            assert torch.equal(bits(op.out[:M]), bits(results[variant]))
        assert torch.equal(bits(results["s0"]), bits(results["s1"])) and torch.equal(bits(results["s0"]), bits(results["s2"]))
        assert op.signals.counter.tolist() == oracle.expected_counters(op.plan.tile_counts(), op.words.epoch)
        # GEMM numerics on a slab (the CPU matmul of the whole thing is the slow part)
        rows = slice(M - 256, M)
        assert_gemm_close(results["s2"][rows], A[rows].float().cpu() @ B.float().cpu(), tight=0.004)
        # linearity property of the GEMM part: alpha = 2 doubles every normal-range output exactly
        # (scaling by a power of two commutes with rounding except among fp16 subnormals)
        op(A, B, "s2", alpha=2.0)
        op.check_faults()
        doubled, base = op.out[:M].float(), results["s2"].float()
        normal = base.abs() >= 2.0**-13
        assert torch.equal(doubled[normal], 2 * base[normal])
        assert (doubled - 2 * base).abs().max().item() <= 2.0**-23
    finally:
        for h in heaps:
            h.cleanup()


def test_pull_with_padded_rows_and_short_k(lib):
    """Large-tile S2 with fewer K steps than pieces per wavefront (the rest of the pull runs
    after the last tile) and a gathered buffer whose rows are not contiguous."""
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    M, N, K = 768, 520, 64
    heaps = SymmetricHeap.create_all(64 << 20, 3)
    try:
        ops = [FusedGemmAllGather(h, M, N, torch.float16, directions="both", macro_tile=256, tau_min_bytes=1, group_m=1)
               for h in heaps]
        op = ops[0]
        assert op.plan.n_groups > 1
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        blocks = fill_peer_blocks(ops, M, N, torch.float16)
        for variant in VARIANTS:
            op.out.zero_()
            op.mark_peers_ready()
            op(A, B, variant)
            op.check_faults()
            mine = op.out[:M].clone()
            assert_gemm_close(mine, A_cpu.float() @ B_cpu.float(), tight=0.004)
            for p in (1, 2):
                assert torch.equal(bits(op.peer_out(p)[:M]), bits(mine)), (variant, p)
                assert torch.equal(bits(op.out[p * M:(p + 1) * M]).cpu(), bits(blocks[p])), (variant, p)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("macro", MACRO)
def test_device_trace_of_a_tilegroup_launch(lib, macro):
    """A traced S2 launch leaves, per TileGroup, start <= ready <= done clocks; the recorder
    turns them into one produce and one transfer span per group."""
    from tileccl_amd.v2.runtime import TimelineRecorder

    M, N, K = 1024, 512, 256
    heaps, ops = make(2, M, N, macro_tile=macro, trace=True, tau_min_bytes=1, group_m=2)
    try:
        op = ops[0]
        assert op.plan.n_groups == 4
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=K**-0.5))
        fill_peer_blocks(ops, M, N, torch.float16)
        op.mark_peers_ready()
        op.signals.trace_start_clock.zero_()
        op.signals.trace_ready_clock.zero_()
        op.signals.trace_done_clock.zero_()
        op(A, B, "s2")
        op.check_faults()
        t0 = int(op.signals.trace_start_clock.cpu()[0])
        ready, done = op.signals.trace_ready_clock.cpu().tolist(), op.signals.trace_done_clock.cpu().tolist()
        assert t0 > 0
        for g in range(4):
            assert t0 <= ready[g] <= done[g], (g, t0, ready, done)
        rec = TimelineRecorder(benchmark="gemm_allgather", path_name=f"s2 macro {macro}")
        made = rec.record_signal_state(op.signals, op.plan, rank=0)
        assert len(made) == 8 and rec.to_payload()["lane_order"] == [f"group {g}" for g in range(4)]
        assert all(e.end_ms < 50.0 for e in made)  # milliseconds: a sub-millisecond launch
    finally:
        for h in heaps:
            h.cleanup()


def test_single_rank_is_a_plain_gemm(lib):
    heaps, ops = make(1, 256, 256)
    try:
        A, B = into_heap(heaps[0], seeded((256, 64), 0)), into_heap(heaps[0], seeded((64, 256), 1, scale=1 / 8))
        for variant in VARIANTS:
            ops[0].out.zero_()
            ops[0](A, B, variant)
            ops[0].check_faults()
            assert_gemm_close(ops[0].out, A.float().cpu() @ B.float().cpu(), tight=0.004)
    finally:
        heaps[0].cleanup()


def test_argument_errors(lib):
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(16 << 20, 2)
    try:
        op = FusedGemmAllGather(heaps[0], 256, 256)
        A, B = into_heap(heaps[0], seeded((256, 64), 0)), into_heap(heaps[0], seeded((64, 256), 1))
        with pytest.raises(ValueError, match="unknown variant 's9'"):
            op(A, B, "s9")
        with pytest.raises(ValueError, match=r"C shape mismatch"):
            op(A[:128], B, "s0")
        with pytest.raises(ValueError, match="unknown directions='sideways'"):
            FusedGemmAllGather(heaps[0], 256, 256, directions="sideways")
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("block_m", [128, 256])
def test_baseline_config_2_with_the_group_size_chosen_by_the_cost_model(lib, block_m):
    """Config 2 as it is worded: the TileGroup size comes from the cost model, fitted to
    transfers and a GEMM measured on this machine (calibrate -> choose_target_group_tiles ->
    build_tile_group_plan).  Whatever size comes out, S2 must move the bytes of the bulk
    variant, match the oracle on a slab and leave every group's counter at its tile count."""
    from tileccl_amd.v2 import SymmetricHeap
    from tileccl_amd.v2.calibrate import calibrate

    M, N, K = 8192, 4096, 1024
    cal_heaps = SymmetricHeap.create_all(256 << 20, 2)
    try:
        cal = calibrate(cal_heaps[0], gemm_shape=(M, N, K))
    finally:
        for h in cal_heaps:
            h.cleanup()
    chosen = cal.target_group_tiles(M, N, K, block_m=block_m)
    wave = 8 * (N // 128)
    assert chosen % wave == 0 and wave <= chosen <= (M // block_m) * (N // 128)  # whole swizzle waves
    assert cal.tau_min_bytes > 0 and cal.profile.beta_us_per_byte > 0
    heaps, ops = make(2, M, N, heap_bytes=1 << 30, block_m=block_m, target_group_tiles=chosen)
    try:
        op = ops[0]
        assert op.plan.target_group_tiles == chosen
        assert all(n >= chosen for n in op.plan.tile_counts()[:-1]) and sum(op.plan.tile_counts()) == (M // block_m) * (N // 128)
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        peer = seeded((M, N), 2)
        results = {}
        for variant in ("s0", "s2"):
            op.out.zero_()
            ops[1].out.zero_()
            ops[1].out[M:].copy_(peer)
            op.mark_peers_ready()
            op(A, B, variant)
            op.check_faults()
            assert torch.equal(bits(op.out), bits(op.peer_out(1))), variant
            assert torch.equal(bits(op.out[M:]).cpu(), bits(peer)), variant
            results[variant] = op.out[:M].clone()
        assert torch.equal(bits(results["s0"]), bits(results["s2"]))
        rows = slice(4000, 4128)
        want = oracle.gemm(A_cpu[rows], B_cpu, torch.float16)
        assert (results["s2"][rows].float().cpu() - want.float()).abs().max().item() <= 0.004
        assert op.signals.counter.tolist() == oracle.expected_counters(op.plan.tile_counts(), op.words.epoch)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("macro", MACRO)
def test_fused_launches_give_the_bulk_variant_bits_for_every_k_loop_length(lib, macro):
    """S0 runs the GEMM alone (on the 128 tile: five LDS stages), S1 / S2 the fused tile loop (three stages, pushes
    from the epilogue): the sums are formed in the same order, so the gathered bytes are the same, for every length
    of the K loop."""
    M, N = 256, 384
    for K in (8, 40, 64, 96, 136, 160, 200, 224, 296, 320):
        heaps, ops = make(2, M, N, macro_tile=macro, heap_bytes=64 << 20)
        try:
            op = ops[0]
            A, B = into_heap(heaps[0], seeded((M, K), 20 + K)), into_heap(heaps[0], seeded((K, N), 21 + K, scale=K**-0.5))
            blocks = fill_peer_blocks(ops, M, N, torch.float16)
            got = {}
            for variant in VARIANTS:
                op.out[:M].zero_()
                op.peer_out(1)[:M].zero_()
                op.mark_peers_ready()
                op(A, B, variant)
                op.check_faults()
                got[variant] = (bits(op.out).clone(), bits(op.peer_out(1)).clone())
            for variant in ("s1", "s2"):
                assert torch.equal(got[variant][0], got["s0"][0]), (K, variant)
                assert torch.equal(got[variant][1], got["s0"][1]), (K, variant)
            assert torch.equal(got["s0"][0][M:].cpu(), bits(blocks[1]))
        finally:
            for h in heaps:
                h.cleanup()
