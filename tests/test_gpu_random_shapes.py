"""Seeded random shapes through the fused all-gather and reduce-scatter against the oracle:
worlds of 2 to 4 ranks, ragged M / N / K, both GEMM kernels, the three variants, both B layouts,
several TileGroup sizes; a second sweep draws larger shapes (K loops of up to 32 steps, several rounds
of large tiles).  Moved bytes and two-rank sums are bit-exact; the GEMM and the sums of
three or more ranks (whose fp32 order is pinned elsewhere) are held to the stated tolerances.
Which combinations the library refuses is decided here, from the case's parameters (a reduce-scatter whose shards
are not whole plan tiles): exactly those must be refused, with that message, and every other draw must run.
Any other ValueError fails the case."""

import ctypes as C
import random

import pytest
import torch

from oracle import collectives as oracle
from tests.gpu_util import bits, into_heap, seeded

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 120


def draw_large(rng):
    """Shapes with K loops of 2 to 32 steps, several rounds of large tiles and blocks of many pieces."""
    case = draw(rng)
    case.update(K=8 * rng.randint(16, 256), N=8 * rng.randint(32, 320))
    if case["kind"] == "ag":
        case.update(M=rng.randint(500, 5000))
    else:
        shard = rng.choice([512, 768, 1024, 2048]) if rng.random() < 0.8 else rng.randint(300, 1200)
        case.update(M=shard * case["world"])
    case["heap"] = 400 << 20
    return case


def draw(rng):
    case = dict(
        kind=rng.choice(["ag", "rs"]), world=rng.choice([2, 2, 3, 4]), macro=rng.choice([0, 128, 256]),
        variant=rng.choice(["s0", "s1", "s2"]), dtype=rng.choice([torch.float16, torch.bfloat16]),
        K=8 * rng.randint(1, 64), N=8 * rng.randint(1, 160), kmajor=rng.random() < 0.3,
        tau=rng.choice([1, 1 << 16, 1 << 18]), group_m=rng.choice([1, 2, 8]), block_m=rng.choice([128, 128, 256]),
    )
    if case["kind"] == "ag":
        case.update(M=rng.randint(1, 1500), directions=rng.choice(["both", "push", "pull"]))
    else:
        shard = rng.choice([128, 256, 384, 512]) if rng.random() < 0.7 else rng.randint(1, 400)
        case.update(M=shard * case["world"], own=rng.random() < 0.5, emul=rng.random() < 0.7)
        case["pdt"] = rng.choice([torch.float32, case["dtype"]])
    return case


def expected_refusal(case):
    """The message (a regular expression) the library must refuse this case with, or None if it must run."""
    if case["kind"] == "rs" and (case["M"] // case["world"]) % case["block_m"]:
        return r"must split into world_size=\d+ shards of whole \d+-row plan tiles"
    return None


def run_case(case, seed):
    """True: checked; None: refused by the library exactly as expected_refusal() says it must be."""
    refusal = expected_refusal(case)
    if refusal is None:
        return run_supported_case(case, seed)
    with pytest.raises(ValueError, match=refusal):
        run_supported_case(case, seed)
    return None


def run_supported_case(case, seed):
    from tileccl_amd import _launch, _lib
    from tileccl_amd.v2 import FusedGemmAllGather, FusedGemmReduceScatter, SymmetricHeap

    world, M, N, K, dtype = case["world"], case["M"], case["N"], case["K"], case["dtype"]
    heaps = SymmetricHeap.create_all(case.get("heap", 96 << 20), world)
    try:
        A_cpu, B_cpu = seeded((M, K), seed, dtype), seeded((K, N), seed + 1, dtype, scale=K**-0.5)
        common = dict(macro_tile=case["macro"], tau_min_bytes=case["tau"], group_m=case["group_m"], block_m=case["block_m"])
        if case["kind"] == "ag":
            ops = [FusedGemmAllGather(h, M, N, dtype, directions=case["directions"], **common) for h in heaps]
        else:
            ops = [FusedGemmReduceScatter(h, M, N, partial_dtype=case["pdt"], out_dtype=dtype,
                                          own_rows_in_registers=case["own"], emulate_peer=case["emul"], **common) for h in heaps]
        A = into_heap(heaps[0], A_cpu)
        if case["kmajor"]:
            B = heaps[0].allocate_tensor((N, K), dtype).t()
            B.copy_(B_cpu)
        else:
            B = into_heap(heaps[0], B_cpu)
        ref32 = A_cpu.float() @ B_cpu.float()
        tol = (0.004 if dtype == torch.float16 else 0.032) * max(1.0, ref32.abs().max().item() / 4)
        op = ops[0]
        if case["kind"] == "ag":
            blocks = {p: seeded((M, N), 100 + p, dtype) for p in range(1, world)}
            for p, o in enumerate(ops):
                o.out.zero_()
                if p:
                    o.out[p * M:(p + 1) * M].copy_(blocks[p])
            op.mark_peers_ready()
            op(A, B, case["variant"])
            op.check_faults()
            torch.cuda.synchronize()
            mine = op.out[:M].clone()
            assert (mine.float().cpu() - ref32).abs().max().item() <= tol
            for p in range(1, world):
                if case["directions"] != "pull":
                    assert torch.equal(bits(op.peer_out(p)[:M]), bits(mine)), f"push to {p}"
                if case["directions"] != "push":
                    assert torch.equal(bits(op.out[p * M:(p + 1) * M]).cpu(), bits(blocks[p])), f"pull from {p}"
            return True
        pdt = case["pdt"]
        peers = {p: seeded((M, N), 100 + p, pdt) for p in range(1, world)}
        for p in range(1, world):
            ops[p].partial.copy_(peers[p])
        for o in ops:
            o.out.zero_()
        op.mark_peers_ready()
        op(A, B, case["variant"])
        op.check_faults()
        torch.cuda.synchronize()
        # The partial as a plain GEMM launch stores it (the in-register mode never writes the owned
        # rows): the same kernel and k order, so the same bits.
        full = torch.empty(M, N, dtype=pdt, device="cuda")
        d = _launch.gemm_desc(A, B, full, macro_tile=case["macro"], block_m=case["block_m"], group_m=case["group_m"])
        _lib.check(_lib.load().tccl_gemm(C.byref(d), _launch.stream_ptr()), "tccl_gemm")
        torch.cuda.synchronize()
        assert (full.float().cpu() - ref32).abs().max().item() <= (tol if pdt != torch.float32 else 1e-3 * max(1.0, ref32.abs().max().item() / 4))
        partials = [full.cpu()] + [peers[p] for p in range(1, world)]
        for owner in (range(world) if case["emul"] else [0]):
            want = oracle.reduce_rows(partials, owner, dtype)
            if world == 2:
                assert torch.equal(bits(ops[owner].out).cpu(), bits(want)), f"owner {owner}"
            else:
                assert (ops[owner].out.cpu().float() - want.float()).abs().max().item() <= 2 * tol, f"owner {owner}"
        return True
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes(lib, seed):
    rng = random.Random(seed)
    checked = 0
    for i in range(CASES_PER_SEED):
        case = draw(rng)
        try:
            checked += 1 if run_case(case, 1000 * seed + i) else 0
        except (AssertionError, ValueError, pytest.fail.Exception) as e:
            raise AssertionError(f"case {i} of seed {seed}: {case}: {e}") from e
    assert checked >= CASES_PER_SEED // 2  # most draws are supported combinations


@pytest.mark.parametrize("seed", [21, 22])
def test_random_large_shapes(lib, seed):
    rng = random.Random(seed)
    checked = 0
    for i in range(40):
        case = draw_large(rng)
        try:
            checked += 1 if run_case(case, 1000 * seed + i) else 0
        except (AssertionError, ValueError, pytest.fail.Exception) as e:
            raise AssertionError(f"case {i} of seed {seed}: {case}: {e}") from e
    assert checked >= 20

