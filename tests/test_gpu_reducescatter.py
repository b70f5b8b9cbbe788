"""GEMM to ReduceScatter (Gate 2) in the S0 / S1 / S2 variants against the CPU oracle.

The reduction is an fp32 sum of per-rank partials rounded once; with two ranks the sum of
two fp32 numbers does not depend on order, so the result is bit-exact against the oracle
run on the partial the GPU produced."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu

VARIANTS = ["s0", "s1", "s2"]


def make(world, M, N, heap_bytes=256 << 20, **kw):
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    heaps = SymmetricHeap.create_all(heap_bytes, world)
    return heaps, [FusedGemmReduceScatter(h, M, N, **kw) for h in heaps]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("partial_dtype,out_dtype", [(torch.float32, torch.float16), (torch.bfloat16, torch.bfloat16),
                                                    (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("macro", [128, 256])
def test_small_two_ranks_bit_exact(lib, variant, partial_dtype, out_dtype, macro):
    M, N, K = 512, 512, 256
    in_dtype = torch.bfloat16 if partial_dtype == torch.bfloat16 else torch.float16
    heaps, ops = make(2, M, N, partial_dtype=partial_dtype, out_dtype=out_dtype, macro_tile=macro)
    try:
        op = ops[0]
        assert op.plan.groups == [(0, 256, 8), (256, 512, 8)]  # one wave, cut at the owner border
        A_cpu, B_cpu = seeded((M, K), 0, in_dtype), seeded((K, N), 1, in_dtype, scale=K**-0.5)
        A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
        peer = seeded((M, N), 2, partial_dtype)
        ops[1].partial.copy_(peer)
        for o in ops:
            o.out.zero_()
        op.mark_peers_ready()
        op(A, B, variant)
        op.check_faults()
        assert_gemm_close(op.partial, A_cpu.float() @ B_cpu.float(), tight=1e-4 if partial_dtype == torch.float32 else 0.032)
        partials = [op.partial.cpu(), peer]
        for owner in (0, 1):
            want = oracle.reduce_rows(partials, owner, out_dtype)
            assert torch.equal(bits(ops[owner].out).cpu(), bits(want)), f"owner {owner}"
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("macro", [128, 256])
def test_without_peer_emulation_only_the_own_shard_is_written(lib, variant, macro):
    M, N, K = 512, 256, 64
    heaps, ops = make(2, M, N, emulate_peer=False, macro_tile=macro)
    try:
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=1 / 8))
        peer = seeded((M, N), 2, torch.float32)
        ops[1].partial.copy_(peer)
        for o in ops:
            o.out.fill_(7.0)
        ops[0].mark_peers_ready()
        ops[0](A, B, variant)
        ops[0].check_faults()
        want = oracle.reduce_rows([ops[0].partial.cpu(), peer], 0, torch.float16)
        assert torch.equal(bits(ops[0].out).cpu(), bits(want))
        assert torch.all(ops[1].out == 7.0)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("macro,M", [(128, 768), (256, 768), (256, 384)])
def test_three_ranks_sum_order_owner_first(lib, variant, macro, M):
    """With three addends the fp32 sum depends on order: owner first, then ascending ranks.
    M = 768 gives shards of whole 256-row tiles (the large-tile kernel reduces tile by tile);
    M = 384 gives 128-row shards (it reduces after its last tile instead)."""
    N, K = 264, 64
    heaps, ops = make(3, M, N, tau_min_bytes=1, group_m=1, macro_tile=macro)
    try:
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=1 / 8))
        peers = {p: seeded((M, N), 10 + p, torch.float32) * 1000.0 for p in (1, 2)}  # large magnitudes: order matters
        for p in (1, 2):
            ops[p].partial.copy_(peers[p])
        for o in ops:
            o.out.zero_()
        ops[0].mark_peers_ready()
        ops[0](A, B, variant)
        ops[0].check_faults()
        partials = [ops[0].partial.cpu(), peers[1], peers[2]]
        for owner in range(3):
            assert torch.equal(bits(ops[owner].out).cpu(), bits(oracle.reduce_rows(partials, owner, torch.float16))), owner
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("world,M,partial_dtype,out_dtype", [
    (2, 512, torch.float32, torch.float16),
    (2, 1024, torch.bfloat16, torch.bfloat16),
    (3, 768, torch.float32, torch.bfloat16),
])
def test_own_rows_kept_in_registers_give_the_same_bytes(lib, variant, world, M, partial_dtype, out_dtype):
    """Large-tile kernel with the owned rows' partial kept in the accumulators: every output
    equals the oracle's reduction of the stored partials of a plain run bit for bit (three
    ranks: order-sensitive magnitudes), the owned rows of `partial` are never written, the
    other rows are."""
    N, K = 264, 64
    in_dtype = torch.bfloat16 if partial_dtype == torch.bfloat16 else torch.float16
    A_cpu, B_cpu = seeded((M, K), 0, in_dtype), seeded((K, N), 1, in_dtype, scale=1 / 8)
    peers_cpu = {p: seeded((M, N), 10 + p, partial_dtype) * (1000.0 if world == 3 else 1.0) for p in range(1, world)}

    def run(flag):
        heaps, ops = make(world, M, N, partial_dtype=partial_dtype, out_dtype=out_dtype, macro_tile=256,
                          tau_min_bytes=1, group_m=1, own_rows_in_registers=flag)
        try:
            A, B = into_heap(heaps[0], A_cpu), into_heap(heaps[0], B_cpu)
            for p in range(1, world):
                ops[p].partial.copy_(peers_cpu[p])
            for o in ops:
                o.out.zero_()
            ops[0].partial.fill_(-3.0)
            ops[0].mark_peers_ready()
            ops[0](A, B, variant)
            ops[0].check_faults()
            return ops[0].partial.cpu(), [o.out.cpu() for o in ops]
        finally:
            for h in heaps:
                h.cleanup()

    plain_partial, plain_outs = run(False)
    kept_partial, kept_outs = run(True)
    shard = M // world
    partials = [plain_partial] + [peers_cpu[p] for p in range(1, world)]
    for owner in range(world):
        want = oracle.reduce_rows(partials, owner, out_dtype)
        assert torch.equal(bits(plain_outs[owner]), bits(want)), owner
        assert torch.equal(bits(kept_outs[owner]), bits(want)), owner
    assert torch.all(kept_partial[:shard] == -3.0)  # never stored
    assert torch.equal(bits(kept_partial[shard:]), bits(plain_partial[shard:]))


def check_full_size_config(heaps, ops, kept_ops, A, B, shard, out_dtype, gemm_ref, peer_cpu, **scales):
    """Shared body of the full-size reduce-scatter configurations.  `ops` store every partial;
    `kept_ops` (or None) are the same operation with the owned rows' partial kept in the
    accumulators, which is the mode the benchmark times.  `peer_cpu` is the peer's partial as the
    configuration states it (seeded on the CPU); both owners' whole shards are compared with the
    oracle's reduction of the CPU bits."""
    op = ops[0]
    ops[1].partial.copy_(peer_cpu)
    outs = {}
    for variant in VARIANTS:
        for o in ops:
            o.out.zero_()
        op.mark_peers_ready()
        op(A, B, variant, **scales)
        op.check_faults()
        outs[variant] = (ops[0].out.clone(), ops[1].out.clone())
    for v in ("s1", "s2"):
        assert torch.equal(bits(outs[v][0]), bits(outs["s0"][0])) and torch.equal(bits(outs[v][1]), bits(outs["s0"][1]))
    partials_cpu = [op.partial.cpu(), peer_cpu]  # rank 0's partial as its GEMM stored it, the peer's as seeded
    for owner in (0, 1):
        want = oracle.reduce_rows(partials_cpu, owner, out_dtype)
        assert torch.equal(bits(outs["s2"][owner].cpu()), bits(want)), owner
    gemm_ref(op.partial)
    assert op.signals.counter.tolist() == oracle.expected_counters(op.plan.tile_counts(), op.words.epoch)
    if kept_ops is None:
        return
    kept = kept_ops[0]
    kept_ops[1].partial.copy_(ops[1].partial)
    for variant in ("s1", "s2"):
        for o in kept_ops:
            o.out.zero_()
        kept.partial.fill_(-3.0)
        kept.mark_peers_ready()
        kept(A, B, variant, **scales)
        kept.check_faults()
        for owner in (0, 1):  # the bytes of the bulk variant on stored partials
            assert torch.equal(bits(kept_ops[owner].out), bits(outs["s0"][owner])), (variant, owner)
        assert torch.all(kept.partial[:shard] == -3.0), variant  # the owned rows' partial is never stored
        assert torch.equal(bits(kept.partial[shard:]), bits(op.partial[shard:])), variant
    assert kept.signals.counter.tolist() == oracle.expected_counters(kept.plan.tile_counts(), kept.words.epoch)


@pytest.mark.parametrize("own_rows", [False, True])
def test_baseline_config_3_properties(lib, own_rows):
    """8192x2048 @ 2048x4096 fp16, peer partial fp32 N(0,1): variants agree byte for byte,
    the result equals the oracle on a slab, counters match the plan; with the owned rows kept
    in registers (what the benchmark runs) the outputs are the same bytes."""
    from tileccl_amd.v2 import FusedGemmReduceScatter

    M, N, K = 8192, 4096, 2048
    heaps, ops = make(2, M, N, heap_bytes=1 << 30)
    try:
        op = ops[0]
        assert op.plan.n_groups == 8 and op.shard_rows == 4096
        kept_ops = [FusedGemmReduceScatter(h, M, N, own_rows_in_registers=True) for h in heaps] if own_rows else None
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=K**-0.5))
        peer_cpu = seeded((M, N), 2, torch.float32)  # the peer's partial: fp32 N(0, 1), seeded on the CPU

        def gemm_ref(partial):
            rows = slice(4000, 4128)
            assert_gemm_close(partial[rows], A[rows].float().cpu() @ B.float().cpu(), tight=1e-3)

        check_full_size_config(heaps, ops, kept_ops, A, B, 4096, torch.float16, gemm_ref, peer_cpu)
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
def test_tile_by_tile_reduce_gives_up_when_the_peer_never_publishes(lib, variant):
    """Large-tile kernel, own rows, a peer whose words stay at zero: the bounded wait expires,
    the launch ends normally with the partial complete, and the host raises."""
    M, N, K = 512, 256, 64
    heaps, ops = make(2, M, N, emulate_peer=False, macro_tile=256, spin_limit_ns=200_000)
    try:
        A, B = into_heap(heaps[0], seeded((M, K), 0)), into_heap(heaps[0], seeded((K, N), 1, scale=1 / 8))
        ops[0](A, B, variant)
        with pytest.raises(RuntimeError, match="gave up waiting"):
            ops[0].check_faults()
        assert_gemm_close(ops[0].partial, A.float().cpu() @ B.float().cpu(), tight=1e-3)
        ops[0].mark_peers_ready()
        ops[0](A, B, variant)
        ops[0].check_faults()
    finally:
        for h in heaps:
            h.cleanup()


def test_argument_errors(lib):
    from tileccl_amd.v2 import FusedGemmReduceScatter, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 3)
    try:
        with pytest.raises(ValueError, match=r"M=512 must be divisible by world_size=3"):
            FusedGemmReduceScatter(heaps[0], 512, 256)
        op = FusedGemmReduceScatter(heaps[0], 384, 256)  # shards of 128 rows: whole tiles
        A, B = into_heap(heaps[0], seeded((384, 64), 0)), into_heap(heaps[0], seeded((64, 256), 1))
        op.mark_peers_ready()
        op(A, B, "s0")
        bad = FusedGemmReduceScatter(heaps[0], 192, 256)  # shards of 64 rows cut a 128-row tile
        with pytest.raises(ValueError, match="shards of whole 128-row plan tiles"):
            bad(A[:192], B, "s2")
    finally:
        for h in heaps:
            h.cleanup()
