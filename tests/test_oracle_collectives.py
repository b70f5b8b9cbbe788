"""Pins for the collective half of the oracle: the vectorised placement against an
element-by-element loop with the reference's mask, exactness of the reduce, the gather
layout, and the GEMM restatement against hand-computable cases."""

import pytest
import torch

from oracle import collectives as oc
from tileccl_amd.patterns.contracts import resolve_pattern_execution


def test_gemm_restatement_on_hand_computable_inputs():
    A = torch.tensor([[1.0, 2.0], [3.0, 4.0]], dtype=torch.float16)
    B = torch.tensor([[5.0, 6.0], [7.0, 8.0]], dtype=torch.float16)
    assert oc.gemm(A, B, torch.float16).tolist() == [[19.0, 22.0], [43.0, 50.0]]
    assert oc.gemm(A, B, torch.float32, alpha=0.5).tolist() == [[9.5, 11.0], [21.5, 25.0]]
    # fp32 accumulation, one rounding: 2049 = 2048 + 1 is not an fp16 number and rounds to even (2048)
    ones = torch.ones(1, 2049, dtype=torch.float16)
    assert oc.gemm(ones, ones.t().contiguous(), torch.float16).item() == 2048.0
    assert oc.gemm(ones, ones.t().contiguous(), torch.float32).item() == 2049.0
    # identity
    g = torch.Generator().manual_seed(0)
    X = torch.randn(16, 16, generator=g).half()
    assert torch.equal(oc.gemm(X, torch.eye(16, dtype=torch.float16), torch.float16), X)


@pytest.mark.parametrize("M,N,world,rank", [(200, 264, 3, 1), (256, 256, 2, 0), (130, 48, 2, 1), (128, 512, 4, 3)])
def test_vectorised_placement_equals_the_masked_tile_loop(M, N, world, rank):
    g = torch.Generator().manual_seed(M + N)
    local = torch.randn(M, N, generator=g).half()
    spec = resolve_pattern_execution(torch.empty(M, 8), torch.empty(8, N), local, rank=rank, world_size=world,
                                     b_layout="full", c_layout="full")
    args = (spec.scatter_src_col_offset, spec.scatter_cols, spec.scatter_dst_leading_dim, spec.scatter_dst_col_offset)
    fast, slow = torch.zeros(M, N, dtype=torch.float16), torch.zeros(M, N, dtype=torch.float16)
    oc.scatter_into_peer(fast, local, *args)
    oc.scatter_into_peer_by_tiles(slow, local, *args, block_m=64, block_n=64)
    assert torch.equal(fast, slow)
    shard = N // world
    assert torch.equal(fast[:, rank * shard:(rank + 1) * shard], local[:, rank * shard:(rank + 1) * shard])
    mask = torch.ones(N, dtype=torch.bool)
    mask[rank * shard:(rank + 1) * shard] = False
    assert torch.count_nonzero(fast[:, mask]).item() == 0  # nothing outside the rank's block is touched


def test_shard_layout_placement_uses_its_own_leading_dimension():
    local = torch.arange(12, dtype=torch.float16).reshape(3, 4)
    dest = torch.zeros(3, 4, dtype=torch.float16)
    oc.scatter_into_peer(dest, local, 0, 4, 4, 0)
    assert torch.equal(dest, local)
    wide = torch.zeros(3, 8, dtype=torch.float16)
    oc.scatter_into_peer(wide, local, 1, 2, 8, 5)  # columns 1..2 land at columns 5..6 of an 8-wide peer
    assert wide[:, 5:7].tolist() == local[:, 1:3].tolist() and wide.sum() == local[:, 1:3].sum()


def test_full_full_allscatter_gives_every_rank_the_full_product():
    world, M, K, N = 2, 64, 32, 128
    g = torch.Generator().manual_seed(0)
    A, B = torch.randn(M, K, generator=g).half(), (torch.randn(K, N, generator=g) / K**0.5).half()
    Cs = [torch.zeros(M, N, dtype=torch.float16) for _ in range(world)]
    specs = []
    for r in range(world):
        s = resolve_pattern_execution(A, B, Cs[r], rank=r, world_size=world, b_layout="full", c_layout="full")
        specs.append(dict(src_col_offset=s.scatter_src_col_offset, cols=s.scatter_cols,
                          dst_ld=s.scatter_dst_leading_dim, dst_col_offset=s.scatter_dst_col_offset))
    oc.gemm_allscatter([A] * world, [B] * world, Cs, specs)
    want = (A.float() @ B.float()).half()
    assert torch.equal(Cs[0], want) and torch.equal(Cs[1], want)


def test_allgather_layout_and_directions():
    M, N = 4, 3
    outs = [torch.zeros(3 * M, N) for _ in range(3)]
    for r in range(3):
        outs[r][r * M:(r + 1) * M] = r + 1  # each rank's own block is resident
    oc.allgather_exchange(outs, rank=1, M=M, push=True, pull=False)
    assert all(torch.all(outs[p][M:2 * M] == 2) for p in range(3))  # rank 1's block is everywhere
    assert torch.all(outs[1][:M] == 0) and torch.all(outs[1][2 * M:] == 0)  # nothing came in
    oc.allgather_exchange(outs, rank=1, M=M, push=False, pull=True)
    assert outs[1][:, 0].tolist() == [1.0] * M + [2.0] * M + [3.0] * M  # [block_rank0 | block_rank1 | block_rank2]


def test_reduce_is_exact_fp32_then_one_rounding_owner_first():
    big, small = 2.0**24, 1.0
    # fp32: (big + small) + small == big, but (small + small) + big == big + 2: order is observable
    partials = [torch.tensor([[big], [small]]), torch.tensor([[small], [big]]), torch.tensor([[small], [small]])]
    partials = [p.repeat(1, 1) for p in partials]  # rows: shard 0 = row 0 (owner 0); world 3 needs 3 rows
    partials = [torch.cat([p, torch.zeros(1, 1)]) for p in partials]
    out0 = oc.reduce_rows(partials, 0, torch.float32)  # big first: big + 1 + 1 -> big (each +1 is lost)
    assert out0.item() == big
    out1 = oc.reduce_rows(partials, 1, torch.float32)  # owner 1 first: big, then rank 0: +1 lost, rank 2: +1 lost
    assert out1.item() == big
    swapped = [partials[2], partials[1], partials[0]]
    assert oc.reduce_rows(swapped, 0, torch.float32).item() == big + 2  # small + small first, then big: exact
    # rounding happens once, after the fp32 sum
    a = torch.tensor([[1.0 + 2.0**-11]], dtype=torch.float32)
    b = torch.tensor([[2.0**-11]], dtype=torch.float32)
    assert oc.reduce_rows([a, b][:1] + [b][:0], 0, torch.float16).item() == 1.0  # single addend: tie rounds to even
    two = oc.reduce_rows([torch.cat([a, a]), torch.cat([b, b])], 0, torch.float16)
    assert two.item() == float(torch.tensor(1.0 + 2.0**-10).half())  # the sum is representable: no double rounding
    assert oc.expected_counters([256, 128], epoch=3) == [768, 384]


def test_chained_gather_is_the_block_matrix_identity():
    """gather_cols(shards) @ W must equal sum_p shard_p @ W[p*Ks:(p+1)*Ks] (block product):
    a wrong column-block order or width breaks it.  Integer-valued inputs keep fp32 exact."""
    g = torch.Generator().manual_seed(5)
    world, M, ks, N = 3, 7, 4, 5
    shards = [torch.randint(-3, 4, (M, ks), generator=g).half() for _ in range(world)]
    W = torch.randint(-3, 4, (world * ks, N), generator=g).half()
    outs = [torch.zeros(M, N, dtype=torch.float16) for _ in range(world)]
    gathered = oc.chained_ag_gemm_rs(shards, W, outs, rank=1)
    assert gathered.shape == (M, world * ks)
    assert torch.equal(gathered[:, ks:2 * ks], shards[1]) and torch.equal(gathered[:, 2 * ks:], shards[2])
    want = sum(shards[p].float() @ W[p * ks:(p + 1) * ks].float() for p in range(world))
    for o in outs:  # every rank receives the same full product
        assert torch.equal(o.float(), want)


def test_standalone_collectives_against_element_loops():
    """allgather / broadcast / scatter / reduce_scatter / allreduce on tiny inputs, each against a
    plain Python loop over elements and against a value a wrong index would change."""
    world, block = 3, 8
    # rank p, element i holds 100*p + i: every element names where it came from
    tens = [torch.arange(world * block, dtype=torch.float32) + 100 * p for p in range(world)]
    blocks = [t[:block].clone() for t in tens]
    ag = oc.allgather(blocks)
    for out in ag:
        assert out.tolist() == [100 * (i // block) + i % block for i in range(world * block)]
    bc = oc.broadcast(blocks, root=2)
    assert all(t.tolist() == [200 + i for i in range(block)] for t in bc)
    sc = oc.scatter(tens[1], world)
    for r, out in enumerate(sc):
        assert out.tolist() == [100 + r * block + i for i in range(block)]
    halves = [t.half() for t in tens]
    rs = oc.reduce_scatter(halves, torch.float16)
    for r, out in enumerate(rs):
        # sum over p of (100p + r*block + i) = 300 + 3*(r*block + i): exact in fp16
        assert out.tolist() == [300 + 3 * (r * block + i) for i in range(block)]
    ar = oc.allreduce(halves)
    assert all(t.tolist() == [300 + 3 * i for i in range(world * block)] for t in ar)
    # the reference's own host restatement adds the ranks in ascending order in the tensor dtype
    # (primitives/collectives.py:2536-2545); on values exact in fp16 both orders agree
    plain = halves[0] + halves[1] + halves[2]
    assert torch.equal(ar[0], plain)


def test_staged_allreduce_restatement_is_pinned_without_its_own_formula():
    """Ascending-rank fp32 sum, one rounding: exact integer sums; equal to the reduce-scatter based
    all-reduce for two ranks (two addends commute); and a three-rank case where rounding after
    every addition in fp16 (what a dropped fp32 accumulator would do) gives a different answer."""
    g = torch.Generator().manual_seed(3)
    ints = [torch.randint(-100, 100, (64,), generator=g).half() for _ in range(4)]
    assert oc.allreduce_staged(ints)[2].tolist() == [float(sum(int(t[i]) for t in ints)) for i in range(64)]
    two = [torch.randn(256, generator=g).half() for _ in range(2)]
    assert torch.equal(oc.allreduce_staged(two)[1], oc.allreduce(two)[0])
    # 2048 + 1 + 1: fp16 spacing at 2048 is 2, so adding one at a time in fp16 stays at 2048,
    # while the fp32 sum 2050 is representable
    three = [torch.tensor([2048.0]).half(), torch.tensor([1.0]).half(), torch.tensor([1.0]).half()]
    got = oc.allreduce_staged(three)
    assert all(t.item() == 2050.0 for t in got)
    assert ((three[0] + three[1]) + three[2]).item() == 2048.0


def test_the_references_staged_order_known_answers():
    """fp16 values whose sums round differently depending on the order: spacing is 2 from 2048 on, ties go to the
    even mantissa.  Ranks hold [1, 2048, 1, 1].  The reference's order (own value first, then the others ascending,
    every addition rounded to fp16) leaves rank 0 with ((1 + 2048 -> 2048) + 1 -> 2048) + 1 -> 2048 and rank 2 with
    ((1 + 1) + 2048 = 2050) + 1 = 2051 -> 2052; this build's order (fp32, one rounding) gives 2051 -> 2052 everywhere."""
    ranks = [torch.tensor([v], dtype=torch.float16) for v in (1.0, 2048.0, 1.0, 1.0)]
    ref = oc.allreduce_staged_reference_order(ranks)
    assert [t.item() for t in ref] == [2048.0, 2048.0, 2052.0, 2052.0]
    ours = oc.allreduce_staged(ranks)
    assert [t.item() for t in ours] == [2052.0] * 4
    bound = oc.rounding_bound(ranks, 3)
    for r in range(4):
        assert (ours[r].float() - ref[r].float()).abs().item() <= bound.item()
    # a dropped addend is far outside the bound
    assert abs(2052.0 - 2048.0 - 1.0 - 1.0) <= bound.item() < 1.0 + 2048.0


def test_the_two_staged_orders_coincide_for_two_ranks_and_for_exact_sums():
    for dtype in (torch.float16, torch.bfloat16, torch.float32):
        pair = [torch.randn(4096, generator=torch.Generator().manual_seed(3 + r)).to(dtype) for r in range(2)]
        ref, ours = oc.allreduce_staged_reference_order(pair), oc.allreduce_staged(pair)
        for r in range(2):
            assert torch.equal(ref[r], ours[r])
    g = torch.Generator().manual_seed(5)
    exact = [torch.randint(-8, 9, (4096,), generator=g).to(torch.float16) for _ in range(5)]
    ref, ours = oc.allreduce_staged_reference_order(exact), oc.allreduce_staged(exact)
    for r in range(5):
        assert torch.equal(ref[r], ours[r])
