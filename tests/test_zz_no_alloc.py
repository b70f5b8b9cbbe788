"""``tccl_gemm_allgather_static``: the all-gather launch whose signal words and plan tables live
in the library's own file-scope device array, for callers that cannot allocate.

It is checked against ``tccl_gemm_allgather`` (words brought in by a ``tccl_sync_desc``), both
called through the C ABI with the same inputs: rank 1 pushes (which publishes its words),
then rank 0 pulls (which has to find rank 1's words in the shared array).  Two exchanges in
a row, the second with a smaller input: the array keeps the first call's contents, and the
second call must not be misled by them.  Bytes must be equal.

Collected last on purpose (the file name): a failure here must not hide the other tests."""

import ctypes as C

import pytest
import torch

from tests.gpu_util import assert_gemm_close, bits, into_heap, seeded

pytestmark = pytest.mark.gpu


def static_plan(plan):
    from tileccl_amd import _lib

    p = _lib.StaticPlan()
    p.n_groups = plan.n_groups
    for g, (lo, hi, n) in enumerate(zip(plan.row_starts(), plan.row_ends(), plan.tile_counts())):
        p.row_starts[g], p.row_ends[g], p.tile_counts[g] = lo, hi, n
    return p


@pytest.fixture(autouse=True)
def fresh_launch_numbers(lib):
    """Every test starts from call 1 on cleared words, whatever an earlier (or failed) test left behind."""
    from tileccl_amd import _launch, _lib

    _lib.check(lib.tccl_static_reset(_launch.stream_ptr()), "tccl_static_reset")
    torch.cuda.synchronize()
    yield


def launch_static(lib, op, A, B, variant, spin_limit_ns=2_000_000_000):
    """`op` supplies geometry, output and heap view; none of its signal words are passed."""
    from tileccl_amd import _launch, _lib

    gemm = _launch.gemm_desc(A, B, op.local_block, block_m=op.block_m, block_n=op.block_n, group_m=op.group_m,
                             macro_tile=op.macro_tile)
    view = _launch.heap_view(op.heap.get_heap_bases(), op.rank, op.world_size)
    transport = _launch.transport_desc(op.directions, op.transport.copy_elems, None, 0)
    plan = static_plan(op.plan)
    rc = lib.tccl_gemm_allgather_static(
        C.byref(gemm), _launch.ptr(op.out), int(op.out.stride(0)), C.byref(view), C.byref(plan), C.byref(transport),
        _launch.VARIANTS[variant], _launch.ptr(op.words.fault), spin_limit_ns, _launch.stream_ptr(),
    )
    _lib.check(rc, "tccl_gemm_allgather_static")


def exchange(lib, M, N, K, variant, macro, static, seed):
    """Rank 1 pushes its block, rank 0 pulls it; returns rank 0's and rank 1's gathered outputs."""
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        kw = dict(macro_tile=macro, tau_min_bytes=1, group_m=2)  # several TileGroups even at small sizes
        puller = FusedGemmAllGather(heaps[0], M, N, torch.float16, directions="pull", **kw)
        pusher = FusedGemmAllGather(heaps[1], M, N, torch.float16, directions="push", **kw)
        assert puller.plan.n_groups > 1
        A0, B0 = into_heap(heaps[0], seeded((M, K), seed)), into_heap(heaps[0], seeded((K, N), seed + 1, scale=K**-0.5))
        A1, B1 = into_heap(heaps[1], seeded((M, K), seed + 2)), into_heap(heaps[1], seeded((K, N), seed + 3, scale=K**-0.5))
        for o in (puller, pusher):
            o.out.zero_()
        run = (lambda op, A, B: launch_static(lib, op, A, B, variant)) if static else (lambda op, A, B: op(A, B, variant))
        run(pusher, A1, B1)
        pusher.check_faults()
        assert torch.equal(bits(puller.out[M:]), bits(pusher.out[M:]))  # delivered by the push ...
        puller.out[M:].zero_()  # ... and wiped, so that what is there afterwards came by the pull
        run(puller, A0, B0)
        puller.check_faults()
        assert_gemm_close(puller.out[:M], A0.float().cpu() @ B0.float().cpu(), tight=0.004)
        return puller.out.cpu(), pusher.out.cpu()
    finally:
        for h in heaps:
            h.cleanup()


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro", [128, 256])
def test_static_words_give_the_bytes_of_caller_supplied_words(lib, variant, macro):
    for M, N, K, seed in [(1024, 768, 256, 10), (512, 264, 128, 20)]:  # the second call is smaller
        want = exchange(lib, M, N, K, variant, macro, False, seed)
        got = exchange(lib, M, N, K, variant, macro, True, seed)
        for rank in (0, 1):
            assert torch.equal(bits(got[rank]), bits(want[rank])), (M, rank)
        assert torch.count_nonzero(got[0][M:]).item() > 0  # the pulled block is really there


@pytest.mark.parametrize("variant", ["s1", "s2"])
@pytest.mark.parametrize("macro", [128, 256])
def test_a_puller_ahead_of_its_peer_waits_and_gives_up(lib, variant, macro):
    """Call 1 in order (push, then pull).  In call 2 the puller is issued BEFORE the pusher: the peer's words
    still hold the values of call 1, which must not satisfy call 2; the puller's bounded wait expires, it raises its
    fault word and leaves the peer's rows of its output alone.  Nothing hangs: the wait is the kernel's own.
    Once the pusher has caught up (and made the call the puller gave up on), the next call works again."""
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    M, N, K = 512, 384, 128
    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        kw = dict(macro_tile=macro, tau_min_bytes=1, group_m=2)
        puller = FusedGemmAllGather(heaps[0], M, N, torch.float16, directions="pull", **kw)
        pusher = FusedGemmAllGather(heaps[1], M, N, torch.float16, directions="push", **kw)
        A0, B0 = into_heap(heaps[0], seeded((M, K), 1)), into_heap(heaps[0], seeded((K, N), 2, scale=K**-0.5))
        A1, B1 = into_heap(heaps[1], seeded((M, K), 3)), into_heap(heaps[1], seeded((K, N), 4, scale=K**-0.5))
        for o in (puller, pusher):
            o.out.zero_()
        launch_static(lib, pusher, A1, B1, variant)  # call 1
        launch_static(lib, puller, A0, B0, variant)
        puller.check_faults()
        pusher.check_faults()
        first = pusher.out[M:].clone()
        assert torch.equal(bits(puller.out[M:]), bits(first)) and torch.count_nonzero(first).item() > 0

        A1.copy_(seeded((M, K), 5))  # call 2: new inputs on the pushing rank ...
        puller.out[M:].fill_(-3.0)  # ... and a marker where its block would land
        launch_static(lib, puller, A0, B0, variant, spin_limit_ns=200_000)  # ahead of its peer
        torch.cuda.synchronize()
        assert int(puller.words.fault.item()) != 0, "the words of call 1 satisfied call 2"
        with pytest.raises(RuntimeError):
            puller.check_faults()
        assert torch.all(puller.out[M:] == -3.0), "rows were pulled although the peer had not produced them"
        assert_gemm_close(puller.out[:M], A0.float().cpu() @ B0.float().cpu(), tight=0.004)  # its own block is there
        puller.words.fault.zero_()

        launch_static(lib, pusher, A1, B1, variant)  # the peer's call 2 (nobody waits for it any more)
        launch_static(lib, pusher, A1, B1, variant)  # call 3, in order again
        launch_static(lib, puller, A0, B0, variant)
        puller.check_faults()
        pusher.check_faults()
        assert torch.equal(bits(puller.out[M:]), bits(pusher.out[M:]))
        assert not torch.equal(bits(pusher.out[M:]), bits(first))  # call 3 moved the new bytes
    finally:
        for h in heaps:
            h.cleanup()


def test_static_words_reject_what_does_not_fit(lib):
    from tileccl_amd import _launch, _lib
    from tileccl_amd.v2 import FusedGemmAllGather, SymmetricHeap

    heaps = SymmetricHeap.create_all(64 << 20, 2)
    try:
        op = FusedGemmAllGather(heaps[0], 512, 256, torch.float16, directions="push")
        A, B = into_heap(heaps[0], seeded((512, 64), 0)), into_heap(heaps[0], seeded((64, 256), 1))
        with pytest.raises(ValueError, match="keeps no signal words"):
            launch_static(lib, op, A, B, "s0")
        gemm = _launch.gemm_desc(A, B, op.local_block)
        view = _launch.heap_view(op.heap.get_heap_bases(), 0, 2)
        transport = _launch.transport_desc(_lib.DIR_PUSH, 16384, None, 0)
        plan = static_plan(op.plan)
        plan.n_groups = _lib.STATIC_MAX_GROUPS + 1
        rc = lib.tccl_gemm_allgather_static(C.byref(gemm), _launch.ptr(op.out), 256, C.byref(view), C.byref(plan),
                                            C.byref(transport), _lib.S2_TILEGROUP, None, 0, None)
        with pytest.raises(ValueError, match=r"n_groups=65 outside \[1, 64\]"):
            _lib.check(rc, "tccl_gemm_allgather_static")
        plan = static_plan(op.plan)
        plan.row_ends[0] = 4096  # beyond M
        rc = lib.tccl_gemm_allgather_static(C.byref(gemm), _launch.ptr(op.out), 256, C.byref(view), C.byref(plan),
                                            C.byref(transport), _lib.S2_TILEGROUP, None, 0, None)
        with pytest.raises(ValueError, match="not an ascending cover"):
            _lib.check(rc, "tccl_gemm_allgather_static")
    finally:
        for h in heaps:
            h.cleanup()


def test_static_words_reject_more_tiles_than_the_array_holds(lib):
    """16385 plan tiles of 128 x 128: refused before anything is launched (no GPU work needed,
    but the library looks the device up, so this runs with the GPU tests)."""
    from tileccl_amd import _lib

    gemm = _lib.GemmDesc()
    gemm.A = gemm.B = gemm.C = 256  # never dereferenced: the size check comes first
    gemm.M, gemm.N, gemm.K = 128 * 16385, 128, 64
    gemm.lda, gemm.ldb, gemm.ldc = 64, 128, 128
    gemm.in_dtype = gemm.out_dtype = _lib.F16
    gemm.alpha = 1.0
    gemm.block_m = gemm.block_n = 128
    gemm.group_m = 8
    view = _lib.HeapView()
    view.heap_bases, view.rank, view.world_size = 256, 0, 2
    plan = _lib.StaticPlan()
    plan.n_groups = 1
    plan.row_starts[0], plan.row_ends[0], plan.tile_counts[0] = 0, gemm.M, 16385
    rc = lib.tccl_gemm_allgather_static(C.byref(gemm), 256, 128, C.byref(view), C.byref(plan), None, _lib.S2_TILEGROUP,
                                        None, 0, None)
    with pytest.raises(ValueError, match="16385 plan tiles exceed the static scratch"):
        _lib.check(rc, "tccl_gemm_allgather_static")
