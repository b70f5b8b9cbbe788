"""Context and symmetric heap on the GPU (mirrors reference tests/test_context_smoke.py and
the heap surface of tileccl/memory/symmetric_heap.py, tileccl_v2/heap.py)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_init_single_gpu_context_smoke(lib):
    import tileccl_amd as tileccl

    ctx = tileccl.init(backend="hip", rank=0, world_size=1, heap_size=8 * 1024 * 1024, force_backend=True)
    try:
        assert ctx.has_heap and ctx.heap is not None and ctx.backend_name == "hip"
        zeros = ctx.zeros(8, 8, dtype=torch.float16)
        randn = ctx.randn(8, 8, dtype=torch.float16)
        empty = ctx.empty(8, dtype=torch.float32)
        assert zeros.shape == (8, 8) and randn.shape == (8, 8) and empty.shape == (8,)
        assert zeros.device.type == "cuda" and str(zeros.device) == ctx.device
        assert torch.count_nonzero(zeros).item() == 0
        assert randn.float().abs().sum().item() > 0
        ctx.barrier()
        assert tileccl.current_context() is ctx and tileccl.get_rank() == 0 and tileccl.get_world_size() == 1
        ws = ctx.workspace("scratch", 4, 4, dtype=torch.float32, zero=True)
        assert ctx.workspace("scratch", 4, 4, dtype=torch.float32) is ws
        assert ctx.heap_bases.tolist() == [ctx.heap.local_base]
        props = ctx.backend.get_device_properties()
        assert props.compute_units > 0 and props.wavefront_size == 64
    finally:
        ctx.heap.cleanup()
        ctx.heap.cleanup()  # idempotent


def test_v1_heap_slices_and_translation(lib):
    from tileccl_amd.memory.symmetric_heap import SymmetricHeap

    heaps = SymmetricHeap.create_all(size=1 << 20, world_size=3)
    try:
        h0, h1, h2 = heaps
        assert [h.rank for h in heaps] == [0, 1, 2] and all(h.world_size == 3 for h in heaps)
        assert h0.mode == "single_process" and h0.transport_strategy == "peer_access"
        bases = h0.get_heap_bases().tolist()
        assert bases == [h.local_base for h in heaps] and len(set(bases)) == 3
        a = h0.allocate_tensor((3, 5), torch.float16)  # 30 bytes
        b = h0.allocate_tensor((7,), torch.int32)
        assert a.data_ptr() == h0.local_base and b.data_ptr() == h0.local_base + 256  # start aligned to 256
        assert h0.bytes_allocated == 256 + 28 and h0.bytes_free == (1 << 20) - 284
        assert h0.owns_tensor(a) and not h1.owns_tensor(a) and h0.is_symmetric(b)
        assert not h0.owns_tensor(torch.zeros(4, device="cuda"))
        assert h0.get_offset(b.data_ptr()) == 256
        assert h0.translate(b.data_ptr(), 2) == bases[2] + 256
        with pytest.raises(ValueError, match="outside the heap"):
            h0.get_offset(h1.local_base)
        with pytest.raises(ValueError, match="to_rank=3 out of range"):
            h0.translate(a.data_ptr(), 3)
        # what rank 1 holds at the same offset is a different piece of HBM
        a1 = h1.allocate_tensor((3, 5), torch.float16)
        a.fill_(1.0)
        a1.fill_(2.0)
        assert h0.peer_view(a, 1).sum().item() == 30.0 and h0.get_peer_buffer(1).data_ptr() == bases[1]
        ext = h0.import_external_tensor(torch.arange(6, device="cuda", dtype=torch.float32).reshape(2, 3))
        assert h0.owns_tensor(ext) and ext.tolist() == [[0, 1, 2], [3, 4, 5]]
        with pytest.raises(ValueError, match="requires a contiguous tensor"):
            h0.as_symmetric(torch.zeros(4, 4, device="cuda").t()[1:])
        with pytest.raises(RuntimeError, match="Symmetric heap exhausted via allocator torch_bump"):
            h0.allocate_tensor((1 << 20,), torch.float32)
        h0.barrier()
        assert h0.metadata()["world_size"] == 3
    finally:
        for h in heaps:
            h.cleanup()
    with pytest.raises(RuntimeError, match="has been cleaned up"):
        heaps[0].allocate_tensor((1,), torch.float16)


def test_v2_heap(lib):
    from tileccl_amd.v2 import SymmetricHeap, allocate_tile_group_signals

    with pytest.raises(ValueError, match="Heap size must be positive"):
        SymmetricHeap(0, 0, 1)
    with pytest.raises(ValueError, match="rank=2 out of range for world_size=2"):
        SymmetricHeap(1024, 2, 2)
    with pytest.raises(RuntimeError, match="needs a second process"):
        SymmetricHeap(1024, 0, 2)
    heaps = SymmetricHeap.create_all(1 << 20, 2)
    try:
        h = heaps[0]
        assert h.device == torch.device("cuda:0") and heaps[1].device == torch.device("cuda:0")
        t = h.allocate_tensor((10,))  # fp16 default, size rounded up to 256
        assert t.dtype == torch.float16 and h.bytes_used == 256 and h.bytes_free == (1 << 20) - 256
        assert t.data_ptr() == h.local_ptr
        with pytest.raises(ValueError, match="shape must be non-empty"):
            h.allocate_tensor(())
        with pytest.raises(ValueError, match="All shape dimensions must be positive integers"):
            h.allocate_tensor((4, 0))
        with pytest.raises(RuntimeError, match=r"SymmetricHeap OOM: need 4194304 bytes but only 1048320 remaining"):
            h.allocate_tensor((1 << 20,), torch.float32)
        sig = h.allocate_signal_buffer(100)
        assert sig.dtype == torch.int32 and sig.sum().item() == 0
        state = allocate_tile_group_signals(heap=h, n_groups=4, device="cuda:0", extra_counters=("arrived",))
        assert h.owns_tensor(state.counter) and h.owns_tensor(state.barrier) and h.owns_tensor(state.extra("arrived"))
        assert not h.owns_tensor(state.trace_ready_clock) and state.trace_start_clock.shape == (1,)
        state.counter.fill_(5)
        state.reset()
        assert state.counter.sum().item() == 0 and state.trace_done_clock.sum().item() == 0
        with pytest.raises(KeyError, match="unknown TileGroup signal counter: nope"):
            state.extra("nope")
        with pytest.raises(ValueError, match="n_groups must be positive"):
            allocate_tile_group_signals(heap=h, n_groups=0, device="cuda:0")
        h.reset_allocator()
        assert h.bytes_used == 0
        with SymmetricHeap(1 << 16, 0, 1) as solo:
            assert solo.get_heap_bases().tolist() == [solo.local_ptr] and solo.mode == "single_process"
    finally:
        for h in heaps:
            h.cleanup()


def test_cost_model_calibration_on_the_device(lib):
    """Transfers of growing size through the C ABI, fitted by CostModelCalibrator: the fitted
    line must explain the large transfers and give a sane bandwidth for copies inside one HBM."""
    from tileccl_amd.v2 import SymmetricHeap
    from tileccl_amd.v2.calibrate import calibrate

    heaps = SymmetricHeap.create_all(512 << 20, 2)
    try:
        cal = calibrate(heaps[0], gemm_shape=(2048, 2048, 512))
        sizes = [p.nbytes for p in cal.points]
        assert sizes == sorted(sizes) and sizes[0] == 8192 and sizes[-1] == 32 << 20
        times = [p.measured_comm_us for p in cal.points]
        assert all(t > 0 for t in times) and times[-1] > times[0]
        prof = cal.profile
        assert 200.0 < prof.bandwidth_gb_s < 8000.0  # push = read + write of the payload through one HBM
        assert 0.5 < prof.min_comm_us < 50.0  # launch latency floor, microseconds
        big = cal.points[-1]
        predicted = max(prof.min_comm_us, prof.alpha_us + big.nbytes * prof.beta_us_per_byte)
        assert abs(predicted - big.measured_comm_us) / big.measured_comm_us < 0.25
        assert 50.0 < cal.gemm_tflops < 2500.0 and 0.0 < prof.gemm_efficiency <= 1.0
        tiles = cal.target_group_tiles(4096, 4096, 1024)
        assert tiles % (8 * 32) == 0 and 256 <= tiles <= 1024  # whole swizzle waves of the 4096 x 4096 plan
    finally:
        for h in heaps:
            h.cleanup()


def test_tensors_outlive_the_heap_objects(lib):
    """Heap objects cleaned up, dropped and garbage collected while a tensor allocated from
    them is still held: the arena's device memory must stay until that tensor is gone."""
    import gc
    import weakref

    from tileccl_amd.v2 import SymmetricHeap

    heaps = SymmetricHeap.create_all(1 << 20, 2)
    arena = weakref.ref(heaps[0]._arena)
    kept = heaps[1].allocate_tensor((64, 8), torch.float32)
    kept.fill_(3.5)
    for h in heaps:
        h.cleanup()
    del heaps, h
    gc.collect()
    assert arena() is not None and arena().live  # held by `kept` through its storage
    assert torch.all(kept == 3.5).item()
    with pytest.raises(RuntimeError, match="cleaned up"):
        arena().slice(0)
    del kept
    gc.collect()
    assert arena() is None  # collected, which is when the device memory is returned
