"""PatternExecutionSpec placement and the public gemm_allscatter contract: closed forms and
error messages (reference tileccl/patterns/contracts.py, tileccl/ops.py:1306-1404)."""

from types import SimpleNamespace

import pytest
import torch

from tileccl_amd.patterns.contracts import resolve_pattern_execution
from tileccl_amd.patterns.runtime import resolve_dual_role_scheduler


def T(rows, cols):
    return torch.empty(rows, cols, dtype=torch.float16)


def test_full_full_two_ranks_is_baseline_config_0():
    for rank in (0, 1):
        s = resolve_pattern_execution(T(512, 256), T(256, 512), T(512, 512), rank=rank, world_size=2,
                                      b_layout="full", c_layout="full")
        assert (s.M, s.K, s.full_N, s.local_N) == (512, 256, 512, 512)
        assert s.scatter_cols == 256
        assert s.scatter_src_col_offset == s.scatter_dst_col_offset == rank * 256
        assert s.scatter_dst_leading_dim == 512
        assert s.rhs_layout == s.output_layout == "full"
        assert s.rhs.full_shape == (256, 512) and s.output.local_shape == (512, 512)
        d = s.to_dict()
        assert d["scatter"] == {"src_col_offset": rank * 256, "cols": 256, "dst_leading_dim": 512, "dst_col_offset": rank * 256}
        assert d["rhs"]["layout_kind"] == "full" and d["output"]["full_shape"] == [512, 512]


def test_single_rank_scatters_everything_nowhere():
    s = resolve_pattern_execution(T(128, 64), T(64, 128), T(128, 128), rank=0, world_size=1)
    assert (s.scatter_cols, s.scatter_src_col_offset, s.scatter_dst_col_offset, s.scatter_dst_leading_dim) == (128, 0, 0, 128)
    assert s.output_layout == "full"


def test_shard_shard():
    s = resolve_pattern_execution(T(64, 32), T(32, 100), T(64, 100), rank=3, world_size=4, full_N=400,
                                  b_layout="shard", c_layout="shard")
    assert (s.full_N, s.local_N, s.scatter_cols, s.scatter_src_col_offset, s.scatter_dst_col_offset,
            s.scatter_dst_leading_dim) == (400, 100, 100, 0, 0, 100)
    assert s.output.cols == 100 and s.rhs.layout_kind == "shard"
    # full_N implied by the hints
    s2 = resolve_pattern_execution(T(64, 32), T(32, 100), T(64, 100), rank=0, world_size=4,
                                   b_layout="shard", c_layout="shard")
    assert s2.full_N == 400


def test_layout_inference_without_hints():
    # mixed widths (hi == lo*world) pin full_N, but mixed layouts are then rejected
    with pytest.raises(ValueError, match="Mixed multi-rank layouts are not implemented yet"):
        resolve_pattern_execution(T(8, 8), T(8, 64), T(8, 32), rank=0, world_size=2)
    with pytest.raises(ValueError, match="Ambiguous multi-rank pattern contract"):
        resolve_pattern_execution(T(8, 8), T(8, 64), T(8, 64), rank=0, world_size=2)
    s = resolve_pattern_execution(T(8, 8), T(8, 64), T(8, 64), rank=1, world_size=2, full_N=64)
    assert s.output_layout == "full" and s.scatter_src_col_offset == 32
    s = resolve_pattern_execution(T(8, 8), T(8, 64), T(8, 64), rank=1, world_size=2, full_N=128)
    assert s.output_layout == "shard"


@pytest.mark.parametrize(
    "args,kw,msg",
    [
        ((torch.empty(2, 2, 2), T(2, 2), T(2, 2)), dict(rank=0, world_size=1), "Pattern tensors must all be 2-D: got A.ndim=3"),
        ((T(2, 2), T(2, 2), T(2, 2)), dict(rank=0, world_size=0), "world_size must be >= 1, got 0"),
        ((T(2, 2), T(2, 2), T(2, 2)), dict(rank=2, world_size=2), "rank=2 out of range for world_size=2"),
        ((T(2, 3), T(2, 2), T(2, 2)), dict(rank=0, world_size=1), r"B.shape\[0\] must equal A.shape\[1\]: got 2 vs 3"),
        ((T(2, 2), T(2, 2), T(3, 2)), dict(rank=0, world_size=1), r"C.shape\[0\] must equal A.shape\[0\]: got 3 vs 2"),
        ((T(2, 2), T(2, 2), T(2, 2)), dict(rank=0, world_size=1, b_layout="diag"), r"b_layout must be one of \['full', 'shard'\], got 'diag'"),
        ((T(2, 2), T(2, 8), T(2, 8)), dict(rank=0, world_size=2, full_N=9, b_layout="full", c_layout="full"),
         r"full_N must be divisible by world_size: 9 % 2 != 0"),
        ((T(2, 2), T(2, 8), T(2, 8)), dict(rank=0, world_size=2, full_N=0), "full_N must be positive, got 0"),
        ((T(2, 2), T(2, 8), T(2, 4)), dict(rank=0, world_size=2, b_layout="full", c_layout="full"),
         r"Provided layout hints disagree on full_N: resolved candidates=\[4, 8\]"),
        ((T(2, 2), T(2, 6), T(2, 6)), dict(rank=0, world_size=2, full_N=8, b_layout="full", c_layout="full"),
         "B layout='full' expects 8 columns, got 6"),
        ((T(2, 2), T(2, 6), T(2, 6)), dict(rank=0, world_size=2, full_N=8), "Cannot infer B layout from cols=6, full_N=8, shard_N=4"),
        ((T(2, 2), T(2, 6), T(2, 6)), dict(rank=0, world_size=1, full_N=8), "B expects 8 columns, got 6"),
    ],
)
def test_contract_errors(args, kw, msg):
    with pytest.raises(ValueError, match=msg):
        resolve_pattern_execution(*args, **kw)


def test_dual_role_scheduler():
    s = resolve_dual_role_scheduler(256)
    assert (s.compute_sms, s.comm_sms, s.policy) == (205, 51, "fractional_split")
    s = resolve_dual_role_scheduler(132)
    assert (s.compute_sms, s.comm_sms) == (106, 26)
    s = resolve_dual_role_scheduler(2, comm_sm_fraction=0.99)
    assert (s.compute_sms, s.comm_sms) == (1, 1)
    s = resolve_dual_role_scheduler(256, compute_sms=200, comm_sms=40)
    assert (s.compute_sms, s.comm_sms, s.policy) == (200, 40, "explicit")
    assert s.to_dict() == {"total_sms": 256, "compute_sms": 200, "comm_sms": 40, "policy": "explicit"}
    assert resolve_dual_role_scheduler(3, comm_sm_fraction=0.0).comm_sms == 1  # never fewer than one mover
    with pytest.raises(ValueError, match="requires both compute_sms and comm_sms to be > 0"):
        resolve_dual_role_scheduler(256, comm_sms=8)
    with pytest.raises(ValueError, match="requires at least 2 compute units"):
        resolve_dual_role_scheduler(1)
    with pytest.raises(ValueError, match="requires both compute_sms and comm_sms to be > 0"):
        resolve_dual_role_scheduler(256, compute_sms=10)
    with pytest.raises(ValueError, match=r"cannot exceed the device SM count: 200 \+ 100 > 256"):
        resolve_dual_role_scheduler(256, compute_sms=200, comm_sms=100)


# ---- public op contract, exercised with a stand-in context on CPU tensors ---------------------------------
def fake_ctx(rank=0, world_size=2):
    return SimpleNamespace(rank=rank, world_size=world_size, device="cpu", backend_name="hip",
                           require_heap=lambda: object())


def test_public_layout_defaults_and_contract():
    from tileccl_amd import ops

    assert ops._resolve_public_layout_contract(b_layout=None, c_layout=None) == ("full", "full")
    with pytest.raises(ValueError, match="b_layout and c_layout must be specified together"):
        ops._resolve_public_layout_contract(b_layout="full", c_layout=None)
    k = ops._resolve_gemm_allscatter_contract(T(512, 256), T(256, 512), T(512, 512), ctx=fake_ctx(1), full_N=None,
                                              b_layout="full", c_layout="full", storage_kind="symmetric")
    assert k.to_dict() == dict(M=512, K=256, full_N=512, rhs_cols=512, output_cols=512, rank=1, world_size=2,
                               rhs_layout="full", output_layout="full", storage_kind="symmetric")
    k = ops._resolve_gemm_allscatter_contract(T(8, 8), T(8, 64), T(8, 32), ctx=fake_ctx(), full_N=None,
                                              b_layout="full", c_layout="shard", storage_kind="symmetric")
    assert (k.full_N, k.rhs_cols, k.output_cols) == (64, 64, 32)
    with pytest.raises(ValueError, match="gemm_allscatter tensors must all reside on the context device cuda:0"):
        bad = fake_ctx()
        bad.device = "cuda:0"
        ops._resolve_gemm_allscatter_contract(T(8, 8), T(8, 8), T(8, 8), ctx=bad, full_N=None, b_layout="full",
                                              c_layout="full", storage_kind="symmetric")
    with pytest.raises(ValueError, match="C layout='full' expects 64 columns, got 32"):
        ops._resolve_gemm_allscatter_contract(T(8, 8), T(8, 64), T(8, 32), ctx=fake_ctx(), full_N=64,
                                              b_layout="full", c_layout="full", storage_kind="symmetric")


def test_pattern_resolution_by_name_class_instance():
    from tileccl_amd import ops
    from tileccl_amd.patterns import BulkSyncPattern, TileGroupPattern, WGSpecializedPattern

    ctx = fake_ctx()
    spec = resolve_pattern_execution(T(8, 8), T(8, 8), T(8, 8), rank=0, world_size=2, b_layout="full", c_layout="full")
    pick = lambda p: ops._resolve_pattern_impl(pattern=p, ctx=ctx, execution=spec, hw_info=None)  # noqa: E731
    assert isinstance(pick("bulk_sync"), BulkSyncPattern) and isinstance(pick("wg_spec"), WGSpecializedPattern)
    assert isinstance(pick("s2"), TileGroupPattern) and isinstance(pick("auto"), TileGroupPattern)
    assert isinstance(pick(BulkSyncPattern), BulkSyncPattern)
    inst = WGSpecializedPattern(ctx)
    assert pick(inst) is inst
    with pytest.raises(ValueError, match="Unknown pattern 'warp_drive'"):
        pick("warp_drive")
    with pytest.raises(TypeError, match="pattern must be a pattern name"):
        pick(3.5)
    with pytest.raises(ValueError, match="Pattern instance rank does not match the provided context: 1 != 0"):
        pick(WGSpecializedPattern(fake_ctx(rank=1)))
    with pytest.raises(ValueError, match="BLOCK_K=32"):
        BulkSyncPattern(ctx, BLOCK_K=32)


def test_auto_select_reference_tree_and_measured_policy():
    """Each branch of the reference's decision tree (auto_select.py:128-188), by hand, at its
    default hardware (132 units, 300 GB/s -> bw_scale 1), and the policy used on MI355X."""
    import importlib

    sel = importlib.import_module("tileccl_amd.patterns.auto_select")  # the package re-exports the function of that name
    from tileccl_amd.patterns.hip_patterns import BulkSyncPattern, TileGroupPattern, WGSpecializedPattern

    ref = lambda M, N, K, ws: sel.reference_choice(M, N, K, ws, 132, 300.0)  # noqa: E731
    assert ref(128, 8192, 32768, 8) == "bulk_sync"                 # M < 256
    assert ref(4096, 4096, 16384, 8) == "fused_sequential"          # N/ws = 512 < 1024, K > 12288
    assert ref(4096, 8192, 8192, 8) == "producer_consumer"          # N/ws = 1024 < 2048, K > 6144
    assert ref(4096, 32768, 8192, 8) == "wg_specialized"            # 32 x 32 tiles >= 132, K > 4096
    assert ref(256, 16384, 16384, 2) == "wg_specialized"            # 2 x 64 = 128 tiles < 132; N > 4096, K > 8192
    assert ref(4096, 8192, 1024, 2) == "fused_sequential"           # intensity 2K = 2048 > 256, tiles > 16
    assert ref(256, 512, 64, 2) == "bulk_sync"                      # nothing applies
    # doubling the link bandwidth doubles the K thresholds: the producer_consumer case falls through
    assert sel.reference_choice(4096, 8192, 8192, 8, 132, 600.0) == "fused_sequential"
    assert sel.auto_select("gemm_allscatter", 4096, 8192, 1024, 2) is TileGroupPattern
    assert sel.auto_select("gemm_allscatter", 4096, 8192, 1024, 1) is BulkSyncPattern
    assert sel.auto_select("gemm_allgather", 64, 8192, 1024, 2) is TileGroupPattern
    assert sel.auto_select("gemm_allscatter", 4096, 32768, 8192, 8, policy="reference") is WGSpecializedPattern
    with pytest.raises(ValueError, match="Unsupported operation 'gemm'"):
        sel.auto_select("gemm", 1, 1, 1, 1)
    with pytest.raises(ValueError, match="unknown policy"):
        sel.auto_select("gemm_allscatter", 1, 1, 1, 1, policy="x")


def test_support_matrix_shape():
    """Sections and keys of the reference's matrix (support.py:67-88) on a stand-in context."""
    import tileccl_amd

    ctx = fake_ctx()
    ctx.backend_name, ctx.device, ctx.heap = "hip", "cuda:0", None
    m = tileccl_amd.describe_runtime_support(ctx).to_dict()
    assert list(m) == ["context", "runtime_surface", "ops", "contracts", "execution_paths", "collectives", "memory"]
    assert m["context"] == {"backend": "hip", "device": "cuda:0", "rank": 0, "world_size": 2, "has_heap": False,
                            "heap_mode": None, "transport_strategy": None}
    assert m["ops"]["gemm_allscatter"]["state"] == "partial"  # two ranks but no heap attached
    assert sorted(m["collectives"]) == ["allgather", "allreduce", "broadcast", "reduce_scatter", "scatter"]
    assert m["collectives"]["allreduce"]["state"] == "partial"  # needs a heap, like the ops
    assert m["execution_paths"]["tile_group"] == {"state": "supported", "detail": "one launch, per-TileGroup counters"}


def test_staged_allreduce_execution_policy():
    """Chunk and slot choice of the staged all-reduce: host arithmetic only."""
    from tileccl_amd.primitives.collectives import resolve_staged_execution as resolve

    # 1 MiB fp16 on two ranks: 64 chunks of 16 KiB, a slot each
    assert resolve(1 << 19, 2, 2) == (8192, 64, 64)
    # 16 MiB: the slots (256) no longer outnumber 16 KiB chunks -> 64 KiB chunks, every slot used once
    assert resolve(1 << 23, 2, 2) == (32768, 256, 256)
    # eight ranks: 128 slots each stay resident
    assert resolve(1 << 26, 2, 8) == (32768, 2048, 128)
    # a tensor smaller than a chunk: one chunk of its own size, rounded up to whole units
    assert resolve(24, 2, 2) == (24, 1, 1)
    assert resolve(8, 4, 3) == (8, 1, 1)
    # explicit values are kept; slots never exceed the chunks
    assert resolve(10000, 2, 2, chunk_elems=4096, pipeline_slots=8) == (4096, 3, 3)
    import pytest
    with pytest.raises(ValueError, match="multiple of 8"):
        resolve(4096, 2, 2, chunk_elems=100)
    with pytest.raises(ValueError, match="at least 1"):
        resolve(4096, 2, 2, pipeline_slots=0)


def test_b_operand_layouts():
    """Row-major B, or the transposed view of a row-major tensor (k-major), with rows on 16-byte boundaries, is
    read in place; every other layout is one the launch helper packs first (None)."""
    import pytest
    import torch

    from tileccl_amd import _launch, _lib

    B = torch.zeros(64, 128, dtype=torch.float16)
    assert _launch._b_layout(B) == (128, 0)
    assert _launch._b_layout(torch.zeros(64, 256, dtype=torch.float16)[:, :128]) == (256, 0)
    W = torch.zeros(128, 64, dtype=torch.float16)  # (N, K)
    assert _launch._b_layout(W.t()) == (64, _lib.GEMM_B_KMAJOR)
    assert _launch._b_layout(torch.zeros(128, 72, dtype=torch.float16)[:, :64].t()) == (72, _lib.GEMM_B_KMAJOR)
    assert _launch._b_layout(torch.zeros(8, 1, dtype=torch.float16).t()) == (8, 0)  # (1, 8): one row, contiguous
    assert _launch._b_layout(torch.zeros(64, 256, dtype=torch.float16)[:, ::2]) is None  # strided columns
    assert _launch._b_layout(torch.zeros(64, 132, dtype=torch.float16)[:, 4:]) is None  # rows off the 16-byte grid
    assert _launch._b_layout(torch.zeros(64, 132, dtype=torch.float16)[:, :128]) is None  # pitch no whole vector
    assert _launch._b_layout(torch.zeros(128, 128, dtype=torch.float16)[::2, ::2].t()) is None  # strided both ways
    with pytest.raises(ValueError, match="2-D"):
        _launch.gemm_operands(torch.zeros(4, 4, dtype=torch.float16), torch.zeros(4, 4, 4, dtype=torch.float16))
    # operands the kernels read in place pass through untouched, on any device
    A = torch.zeros(32, 64, dtype=torch.float16)
    a, b, k, lda, ldb, flags = _launch.gemm_operands(A, W.t())
    assert a is A and b.data_ptr() == W.data_ptr() and (k, lda, ldb, flags) == (64, 64, 64, _lib.GEMM_B_KMAJOR)


def test_context_and_pattern_helper_methods():
    """TileCCLContext.auto_select_pattern / support_matrix (reference __init__.py:180-206) and
    Pattern.require_device_remote_access_runtime (reference patterns/__init__.py:171-185)."""
    import tileccl_amd
    from tileccl_amd.patterns import Pattern
    from tileccl_amd.patterns.hip_patterns import BulkSyncPattern, TileGroupPattern

    ctx = tileccl_amd.TileCCLContext(rank=0, world_size=2, device="cuda:0", backend_name="hip", backend=None)
    chosen = ctx.auto_select_pattern("gemm_allscatter", 4096, 8192, 1024)
    assert type(chosen) is TileGroupPattern and chosen.ctx is ctx
    one = tileccl_amd.TileCCLContext(rank=0, world_size=1, device="cuda:0", backend_name="hip", backend=None)
    assert type(one.auto_select_pattern("gemm_allscatter", 4096, 8192, 1024)) is BulkSyncPattern
    m = ctx.support_matrix().to_dict()
    assert m["context"]["world_size"] == 2 and m["context"]["has_heap"] is False
    with pytest.raises(RuntimeError):  # no heap attached: the guard needs one, as every pattern does
        Pattern.require_device_remote_access_runtime(chosen, operation="gemm_allscatter")


def test_import_smoke_as_the_reference_has_it():
    """The reference's tests/test_import_smoke.py:10-18 on this package, plus its ``__all__``
    (tileccl/__init__.py:539-552): every public name resolves."""
    import importlib

    tileccl = importlib.import_module("tileccl_amd")
    assert isinstance(tileccl.__version__, str)
    assert callable(tileccl.init) and callable(tileccl.init_local)
    assert importlib.import_module("tileccl_amd.ops") is not None
    reference_all = ["__version__", "init", "init_local", "get_rank", "get_world_size", "current_context",
                     "describe_runtime_support", "TileCCLContext", "Tile", "SymmetricHeap", "patterns", "ops"]
    for name in reference_all:
        assert name in tileccl.__all__ and getattr(tileccl, name) is not None, name
    assert tileccl.Tile is tileccl.SymmetricHeap  # the reference's placeholder alias (tileccl/__init__.py:514-522)


def test_spill_check_reads_an_assembly_listing():
    """tileccl_amd.csrc.check_spills counts scratch-memory instructions between a kernel's first and last MFMA."""
    from tileccl_amd.csrc.check_spills import kernels

    name = "_ZN4tccl15fused256_kernelIDF16_DF16_Lb0ELb0ELb0EEEvNS_12Fused256ArgsE"
    asm = "\n".join([
        f"{name}:                         ; @{name}",
        "\tscratch_store_dword off, v2, off offset:8 ; 4-byte Folded Spill",
        "\tv_mfma_f32_16x16x32_f16 v[0:3], v[4:7], v[8:11], v[0:3]",
        "\tscratch_load_dword v178, off, off ; 4-byte Folded Reload",
        "\tds_read_b128 v[4:7], v9",
        "\tv_mfma_f32_16x16x32_f16 v[0:3], v[4:7], v[8:11], v[0:3]",
        "\tscratch_load_dword v2, off, off offset:8 ; 4-byte Folded Reload",
        "\ts_endpgm",
        ".Lfunc_end0:",
        "  - .name:           " + name,
        "    .sgpr_count:     104",
        "    .vgpr_count:     256",
    ]) + "\n"
    assert list(kernels(asm)) == [(name, 256, 1, 3)]


def test_spill_check_tells_reduce_scatter_kernels_apart():
    """Scratch accesses outside the K loops matter in the reduce-scatter kernels: the check marks them there."""
    from tileccl_amd.csrc.check_spills import is_reduce

    assert is_reduce("_ZN4tccl15fused256_kernelIDF16_fLb1ELb0ELb0ELb1EEEvNS_12Fused256ArgsE")
    assert is_reduce("_ZN4tccl15fused256_kernelINS_7fp8e4m3EDF16bLb1ELb0ELb1ELb1EEEvNS_12Fused256ArgsE")
    assert not is_reduce("_ZN4tccl15fused256_kernelIDF16_DF16_Lb0ELb1ELb0ELb1EEEvNS_12Fused256ArgsE")
    assert not is_reduce("_ZN4tccl14gemm256_kernelIDF16_fLb1EEEvNS_8GemmArgsENS_5MacroE")
