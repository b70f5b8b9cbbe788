"""tileccl.ops.gemm_allscatter on the GPU for the three patterns, against the CPU oracle.

Mirrors the reference's only numeric test (tests/test_gemm_allscatter_smoke.py) and adds the
two-rank benchmark configuration 0 (512x512x256), the sharded contracts and byte-exact placement checks."""

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import assert_gemm_close, bits, seeded

pytestmark = pytest.mark.gpu

PATTERNS = ["bulk_sync", "wg_specialized", "tile_group"]


def test_gemm_allscatter_single_gpu_smoke(lib):
    """The reference's smoke test, verbatim in structure: world_size 1, plain device tensors."""
    import tileccl_amd as tileccl
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    heaps = SymmetricHeap.create_all(size=64 * 1024 * 1024, world_size=1)
    try:
        ctx = tileccl.init(backend="hip", rank=0, world_size=1, heap=heaps[0], force_backend=True)
        a = torch.randn(128, 64, device=ctx.device, dtype=torch.float16)
        b = torch.randn(64, 128, device=ctx.device, dtype=torch.float16)
        c = torch.zeros(128, 128, device=ctx.device, dtype=torch.float16)
        tileccl.ops.gemm_allscatter(a, b, c, ctx=ctx, pattern="bulk_sync")
        torch.cuda.synchronize()
        ref = torch.matmul(a.float(), b.float()).half()
        assert torch.allclose(c, ref, rtol=1e-2, atol=1e-1)
        for pattern in ("auto", "wg_spec", "fused_seq", "pc", "s2"):
            c.zero_()
            tileccl.ops.gemm_allscatter(a, b, c, ctx=ctx, pattern=pattern)
            torch.cuda.synchronize()
            assert torch.allclose(c, ref, rtol=1e-2, atol=1e-1), pattern
    finally:
        for heap in heaps:
            heap.cleanup()


def test_operand_views_the_reference_kernels_accept(lib):
    """`tileccl.ops.gemm_allscatter` with a transposed A and a strided B (the reference's GEMM takes any strides,
    /root/reference/tileccl/kernels/gemm.py:63-66): the bits of the call on contiguous copies."""
    import tileccl_amd as tileccl
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    heaps = SymmetricHeap.create_all(size=64 * 1024 * 1024, world_size=1)
    try:
        ctx = tileccl.init(backend="hip", rank=0, world_size=1, heap=heaps[0], force_backend=True)
        a_t = seeded((72, 200), 3).cuda()  # (K, M): A is its transposed view
        wide_b = torch.zeros(72, 2 * 136, device=ctx.device, dtype=torch.float16)
        wide_b[:, ::2] = seeded((72, 136), 4, scale=72**-0.5).cuda()
        for pattern in PATTERNS:
            got = torch.zeros(200, 136, device=ctx.device, dtype=torch.float16)
            want = torch.zeros_like(got)
            tileccl.ops.gemm_allscatter(a_t.t(), wide_b[:, ::2], got, ctx=ctx, pattern=pattern)
            tileccl.ops.gemm_allscatter(a_t.t().contiguous(), wide_b[:, ::2].contiguous(), want, ctx=ctx, pattern=pattern)
            torch.cuda.synchronize()
            assert torch.equal(bits(got), bits(want)), pattern
            assert_gemm_close(got, a_t.t().float().cpu() @ wide_b[:, ::2].float().cpu())
    finally:
        for heap in heaps:
            heap.cleanup()


def _two_rank_case(pattern, M, K, N, dtype=torch.float16, world=2, inspect=None, **pattern_kw):
    import tileccl_amd as tileccl
    from tileccl_amd import ops

    ctxs = tileccl.init_local(world_size=world, heap_size=256 << 20)
    try:
        A_cpu = seeded((M, K), 0, dtype)
        B_cpu = seeded((K, N), 0 + 1, dtype, scale=K**-0.5)
        As = [c.as_symmetric(A_cpu.cuda()) for c in ctxs]
        Bs = [c.as_symmetric(B_cpu.cuda()) for c in ctxs]
        Cs = [c.zeros(M, N, dtype=dtype) for c in ctxs]
        plans = []
        for r, c in enumerate(ctxs):
            cls = ops._PATTERN_ALIASES[pattern]
            plan = ops.build_gemm_allscatter_plan(As[r], Bs[r], Cs[r], ctx=c, pattern=cls(c, **pattern_kw))
            plan.execute(As[r], Bs[r], Cs[r])
            plan.pattern_impl.check_faults()
            plans.append(plan)
        torch.cuda.synchronize()
        # oracle on the same bits
        want = [torch.zeros(M, N, dtype=dtype) for _ in range(world)]
        specs = [
            dict(src_col_offset=p.execution.scatter_src_col_offset, cols=p.execution.scatter_cols,
                 dst_ld=p.execution.scatter_dst_leading_dim, dst_col_offset=p.execution.scatter_dst_col_offset)
            for p in plans
        ]
        oracle.gemm_allscatter([A_cpu] * world, [B_cpu] * world, want, specs)
        ref32 = A_cpu.float() @ B_cpu.float()
        for r in range(world):
            assert_gemm_close(Cs[r], ref32, tight=0.004 if dtype == torch.float16 else 0.032)
            assert (Cs[r].cpu().float() - want[r].float()).abs().max().item() <= 0.032
        # placement is byte-exact: the column block rank p holds from rank r is rank r's GEMM output.
        # Same inputs on every rank -> every rank's local GEMM is bit-identical, so all C agree bit for bit.
        for r in range(1, world):
            assert torch.equal(bits(Cs[0]), bits(Cs[r]))
        if inspect is not None:
            inspect(plans)  # while the heaps (and the signal words in them) are still alive
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("pattern", PATTERNS)
def test_benchmark_configuration_0(lib, pattern):
    """512x256 @ 256x512 fp16, seed 0, world 2, tiles 128x128: each slice ends with the full C."""
    def inspect(plans):
        if pattern == "tile_group":
            plan = plans[0].pattern_impl.last_plan
            assert plan.groups == [(0, 512, 16)] and plan.group_table.tolist() == [0] * 16

    _two_rank_case(pattern, 512, 256, 512, inspect=inspect)


@pytest.mark.parametrize("pattern", PATTERNS)
def test_ragged_rows_three_ranks_bf16(lib, pattern):
    _two_rank_case(pattern, 200, 72, 384, dtype=torch.bfloat16, world=3)


@pytest.mark.parametrize("seed", [31, 32])
def test_random_shapes_every_pattern(lib, seed):
    """Seeded random shapes, worlds and TileGroup sizes through the full / full contract of every pattern."""
    import random

    rng = random.Random(seed)
    for _ in range(40):
        pattern = rng.choice(PATTERNS)
        world = rng.choice([1, 2, 3, 4])
        M, K = rng.randint(1, 1100), 8 * rng.randint(1, 48)
        N = 8 * world * rng.randint(1, 40)  # the full / full contract splits N over the ranks
        dtype = rng.choice([torch.float16, torch.bfloat16])
        kw = {}
        if pattern == "tile_group":
            kw = dict(tau_min_bytes=rng.choice([1, 1 << 16, 1 << 18]), GROUP_M=rng.choice([1, 2, 8]))
        try:
            _two_rank_case(pattern, M, K, N, dtype=dtype, world=world, **kw)
        except AssertionError as e:
            raise AssertionError(f"{pattern} world {world} M {M} K {K} N {N} {dtype} {kw}: {e}") from e


def test_tile_group_counters_and_many_groups(lib):
    def inspect(plans):
        impl = plans[0].pattern_impl
        plan, words = impl.last_plan, impl._last_sync
        assert plan.n_groups == 8 and plan.tile_counts() == [4] * 8
        assert words.counter.tolist() == oracle.expected_counters(plan.tile_counts(), words.epoch)
        # the column blocks leave from the GEMM's epilogue: no communication task is left to count
        # (a traced launch keeps the pushes as tasks of the communication workgroups, two per group here)
        assert words.barrier.tolist() == [0] * 8

    _two_rank_case("tile_group", 2048, 64, 256, tau_min_bytes=1, GROUP_M=2, inspect=inspect)


def test_repeated_launches_reuse_unreset_counters(lib):
    import tileccl_amd as tileccl
    from tileccl_amd.patterns import TileGroupPattern

    ctxs = tileccl.init_local(world_size=2, heap_size=64 << 20)
    try:
        A = ctxs[0].as_symmetric(seeded((512, 128), 0).cuda())
        B = ctxs[0].as_symmetric(seeded((128, 512), 1, scale=128**-0.5).cuda())
        Cd = ctxs[0].zeros(512, 512, dtype=torch.float16)
        ctxs[1].zeros(512 * 2, 512, dtype=torch.float16)  # keep the peer's slice offsets in step
        pat = TileGroupPattern(ctxs[0])
        for i in range(1, 6):
            tileccl.ops.gemm_allscatter(A, B, Cd, ctx=ctxs[0], pattern=pat)
            pat.check_faults()
            assert pat._last_sync.epoch == i
            assert pat._last_sync.counter.tolist() == [16 * i]
        pat._last_sync.reset()
        assert pat._last_sync.counter.tolist() == [0] and pat._last_sync.epoch == 0
    finally:
        for c in ctxs:
            c.heap.cleanup()


@pytest.mark.parametrize("pattern", ["auto", "bulk_sync", "wg_specialized", "tile_group", "s2"])
def test_patterns_named_by_string_take_heap_memory_once(lib, pattern):
    """A pattern given by name is instantiated on every call; its signal words are cut from the heap, which
    never gives memory back, so they must be found again instead of allocated again."""
    import tileccl_amd as tileccl

    ctxs = tileccl.init_local(world_size=2, heap_size=64 << 20)
    try:
        c = ctxs[0]
        A = c.as_symmetric(seeded((256, 64), 0).cuda())
        B = c.as_symmetric(seeded((64, 256), 1, scale=1 / 8).cuda())
        out = c.zeros(256, 256, dtype=torch.float16)
        ctxs[1].zeros(256 * 3, 256, dtype=torch.float16)  # the peer's slice is written at the same offsets
        tileccl.ops.gemm_allscatter(A, B, out, ctx=c, pattern=pattern)
        used = c.heap.bytes_allocated
        first = out.clone()
        for _ in range(20):
            tileccl.ops.gemm_allscatter(A, B, out, ctx=c, pattern=pattern)
        torch.cuda.synchronize()
        assert c.heap.bytes_allocated == used
        assert torch.equal(bits(out), bits(first))
    finally:
        for x in ctxs:
            x.heap.cleanup()


def test_sharded_and_mixed_contracts(lib):
    import tileccl_amd as tileccl
    from tileccl_amd import ops

    ctxs = tileccl.init_local(world_size=2, heap_size=64 << 20)
    try:
        M, K, N = 256, 64, 512
        A_cpu, B_cpu = seeded((M, K), 2), seeded((K, N), 3, scale=K**-0.5)
        ref32 = A_cpu.float() @ B_cpu.float()
        # full B, shard C: the host wrapper materialises the full output in a workspace
        for r, c in enumerate(ctxs):
            A, B = c.as_symmetric(A_cpu.cuda()), c.as_symmetric(B_cpu.cuda())
            Cs = c.zeros(M, N // 2, dtype=torch.float16)
            plan = ops.build_gemm_allscatter_plan(A, B, Cs, ctx=c, b_layout="full", c_layout="shard", pattern="s2")
            assert isinstance(plan, ops.GemmAllScatterMixedLayoutPlan) and plan.to_dict()["materialization"] == "full_to_shard"
            plan.execute(A, B, Cs)
            torch.cuda.synchronize()
            assert_gemm_close(Cs, ref32[:, r * 256:(r + 1) * 256], tight=0.004)
        # shard/shard expert contract: rank r multiplies its column shard and pushes it over the peers' shard
        shards = []
        for r, c in enumerate(ctxs):
            A = c.as_symmetric(A_cpu.cuda())
            Bs = c.as_symmetric(B_cpu[:, r * 256:(r + 1) * 256].contiguous().cuda())
            shards.append((A, Bs, c.zeros(M, 256, dtype=torch.float16)))
        for r, c in enumerate(ctxs):
            ops.gemm_allscatter_sharded(*shards[r], full_N=N, ctx=c, pattern="s1")
        torch.cuda.synchronize()
        # sequential single-process launches: the last rank's shard ends up everywhere
        for r in range(2):
            assert_gemm_close(shards[r][2], ref32[:, 256:512], tight=0.004)
        with pytest.raises(ValueError, match="only implemented for b_layout='full'"):
            ops.build_gemm_allscatter_plan(shards[0][0], shards[0][1], ctxs[0].zeros(M, N, dtype=torch.float16),
                                           ctx=ctxs[0], b_layout="shard", c_layout="full")
        with pytest.raises(ValueError, match="C must live in the symmetric heap"):
            A, B = ctxs[0].as_symmetric(A_cpu.cuda()), ctxs[0].as_symmetric(B_cpu.cuda())
            ops.gemm_allscatter(A, B, torch.zeros(M, N, dtype=torch.float16, device="cuda"), ctx=ctxs[0], pattern="s0")
    finally:
        for c in ctxs:
            c.heap.cleanup()


def test_benchmark_all_patterns_table(lib):
    """The comparison table of the reference (patterns/auto_select.py:194-308): every pattern runs,
    rows come sorted by mean latency, and the output still holds the product."""
    import tileccl_amd as tileccl
    from tileccl_amd.patterns.auto_select import benchmark_all_patterns

    ctxs = tileccl.init_local(world_size=2, heap_size=128 << 20)
    try:
        M, K, N = 512, 128, 512
        A_cpu, B_cpu = seeded((M, K), 0), seeded((K, N), 1, scale=K**-0.5)
        As = [c.as_symmetric(A_cpu.cuda()) for c in ctxs]  # every rank allocates alike: offsets must match
        Bs = [c.as_symmetric(B_cpu.cuda()) for c in ctxs]
        A, B = As[0], Bs[0]
        Cs = [c.zeros(M, N, dtype=torch.float16) for c in ctxs]
        table = benchmark_all_patterns(A, B, Cs[0], ctxs[0], warmup=1, iters=3)
        names = [r["pattern"] for r in table["results"]]
        assert sorted(names) == ["bulk_sync", "fused_sequential", "producer_consumer", "tile_group", "wg_specialized"]
        assert all("error" not in r and r["iters"] == 3 for r in table["results"])
        means = [r["mean_ms"] for r in table["results"]]
        assert means == sorted(means) and table["best"] == names[0]
        assert (table["M"], table["N"], table["K"], table["world_size"]) == (M, N, K, 2)
        torch.cuda.synchronize()
        assert_gemm_close(Cs[0], A_cpu.float() @ B_cpu.float(), tight=0.004)
        half = N // 2  # full/full: rank 0 sends its column block [0, N/2) to the peer and nothing else
        assert torch.equal(bits(Cs[1][:, :half]), bits(Cs[0][:, :half])) and torch.all(Cs[1][:, half:] == 0)
    finally:
        for c in ctxs:
            c.heap.cleanup()
