"""ctypes binding of ``libtileccl_hip.so`` (declarations: ``include/tileccl_hip.h``).

The reference reaches native code the same way -- ``ctypes`` into ``libamdhip64``
(``/root/reference/tileccl/backends/hip.py:67-197``) -- and turns non-zero return codes
into ``RuntimeError``; ``check`` below keeps that idiom.  The library is built in-tree by
``tileccl_amd/csrc/build.py`` (or ``__graft_entry__.build``); if it is missing, loading
fails loudly: there is no fallback path.
"""

from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

LIB_NAME = "libtileccl_hip.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

# enums (include/tileccl_hip.h)
F16, BF16, F32, F8E4M3 = 0, 1, 2, 3
S0_BULK, S1_TILE, S2_TILEGROUP = 0, 1, 2
DIR_PUSH, DIR_PULL = 1, 2
ERR_INVALID, ERR_UNSUPPORTED, ERR_NO_DEVICE, ERR_TIMEOUT = -1, -2, -3, -4
MAX_WORLD = 8
RS_EMULATE_PEERS, RS_PEERS_RESIDENT = 1, 2


class DeviceInfo(C.Structure):
    _fields_ = [
        ("compute_units", C.c_int32),
        ("clock_khz", C.c_int32),
        ("lds_bytes", C.c_int32),
        ("wavefront", C.c_int32),
        ("xcds", C.c_int32),
        ("reserved", C.c_int32 * 3),
        ("arch", C.c_char * 64),
    ]


class GemmDesc(C.Structure):
    _fields_ = [
        ("A", C.c_void_p),
        ("B", C.c_void_p),
        ("C", C.c_void_p),
        ("M", C.c_int32),
        ("N", C.c_int32),
        ("K", C.c_int32),
        ("lda", C.c_int64),
        ("ldb", C.c_int64),
        ("ldc", C.c_int64),
        ("in_dtype", C.c_int32),
        ("out_dtype", C.c_int32),
        ("alpha", C.c_float),
        ("block_m", C.c_int32),
        ("block_n", C.c_int32),
        ("group_m", C.c_int32),
        ("num_wgs", C.c_int32),
        ("macro_tile", C.c_int32),
        ("flags", C.c_int32),
        ("column_shards", C.c_int32),
    ]


GEMM_OWN_ROWS_IN_REGISTERS = 1  # TCCL_GEMM_OWN_ROWS_IN_REGISTERS
GEMM_B_KMAJOR = 2  # TCCL_GEMM_B_KMAJOR
STAGED_ALLREDUCE, STAGED_ALLGATHER, STAGED_REDUCE_SCATTER, STAGED_BROADCAST, STAGED_SCATTER = range(5)  # TCCL_STAGED_*


class SyncDesc(C.Structure):
    _fields_ = [
        ("locks", C.c_void_p),
        ("group_table", C.c_void_p),
        ("counter", C.c_void_p),
        ("barrier", C.c_void_p),
        ("n_groups", C.c_int32),
        ("epoch", C.c_int32),
        ("row_starts", C.c_void_p),
        ("row_ends", C.c_void_p),
        ("tile_counts", C.c_void_p),
        ("trace_comm_counter", C.c_void_p),
        ("trace_start_clock", C.c_void_p),
        ("trace_ready_clock", C.c_void_p),
        ("trace_done_clock", C.c_void_p),
        ("fault", C.c_void_p),
        ("spin_limit_ns", C.c_int64),
    ]


class HeapView(C.Structure):
    _fields_ = [("heap_bases", C.c_void_p), ("rank", C.c_int32), ("world_size", C.c_int32)]


class ScatterDesc(C.Structure):
    _fields_ = [
        ("src_col_offset", C.c_int32),
        ("cols", C.c_int32),
        ("dst_ld", C.c_int32),
        ("dst_col_offset", C.c_int32),
    ]


class TransportDesc(C.Structure):
    _fields_ = [
        ("directions", C.c_int32),
        ("copy_elems", C.c_int32),
        ("reduce_elems", C.c_int32),
        ("num_comm_wgs", C.c_int32),
    ]


STATIC_MAX_TILES, STATIC_MAX_GROUPS = 16384, 64


class StaticPlan(C.Structure):
    """Host-side plan rows of ``tccl_gemm_allgather_static`` (``tccl_static_plan``)."""

    _fields_ = [
        ("n_groups", C.c_int32),
        ("row_starts", C.c_int32 * STATIC_MAX_GROUPS),
        ("row_ends", C.c_int32 * STATIC_MAX_GROUPS),
        ("tile_counts", C.c_int32 * STATIC_MAX_GROUPS),
    ]


_P = C.POINTER
_i32, _i64, _vp = C.c_int32, C.c_int64, C.c_void_p

# name -> (restype, argtypes); every symbol include/tileccl_hip.h declares.
SIGNATURES = {
    "tccl_abi_version": (C.c_int, []),
    "tccl_last_error_string": (C.c_char_p, []),
    "tccl_device_query": (C.c_int, [C.c_int, _P(DeviceInfo)]),
    "tccl_tile_coords": (C.c_int, [_i32, _i32, _i32, _i32, _P(_i32), _P(_i32)]),
    "tccl_tile_for_slot": (C.c_int, [_i32, _i32, _i32, _i32, _P(_i32)]),
    "tccl_heap_create": (C.c_int, [C.c_size_t, C.c_int, _P(_vp), _P(_i64)]),
    "tccl_heap_destroy": (C.c_int, [_vp]),
    "tccl_fill_i32": (C.c_int, [_vp, _i64, _i32, _vp]),
    "tccl_pack_matrix": (C.c_int, [_vp, _i64, _i64, _i32, _i32, _vp, _i64, _i32, _i32, _i32, _vp]),
    "tccl_prim_signal": (C.c_int, [_vp, _i32, _vp]),
    "tccl_prim_signal_add": (C.c_int, [_vp, _i32, _i32, _vp, _vp]),
    "tccl_prim_try_wait": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp]),
    "tccl_prim_wait_ge": (C.c_int, [_vp, _i32, _i32, _i64, _vp, _vp]),
    "tccl_gemm": (C.c_int, [_P(GemmDesc), _vp]),
    "tccl_scatter_cols": (C.c_int, [_vp, _i32, _i64, _i32, _P(ScatterDesc), _P(HeapView), _vp]),
    "tccl_exchange_rows": (C.c_int, [_vp, _i32, _i32, _i64, _i32, _P(HeapView), _P(TransportDesc), _vp]),
    "tccl_reduce_rows": (
        C.c_int,
        [_vp, _i32, _i64, _vp, _i32, _i64, _i32, _i32, _P(HeapView), _P(TransportDesc), _i32, _vp],
    ),
    "tccl_collective_staged": (
        C.c_int,
        [_i32, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _i32, _i32, _i32, C.c_uint32, _i32, _P(HeapView), _vp, _i64, _vp],
    ),
    "tccl_allreduce_staged": (
        C.c_int,
        [_vp, _i32, _i64, _vp, _vp, _vp, _i32, _i32, _i32, C.c_uint32, _P(HeapView), _vp, _i64, _vp],
    ),
    "tccl_gemm_allscatter": (
        C.c_int,
        [_P(GemmDesc), _P(ScatterDesc), _P(HeapView), _P(SyncDesc), _P(TransportDesc), _i32, _vp],
    ),
    "tccl_copy_block": (C.c_int, [_vp, C.c_uint32, _vp, _i32, _i32, _i64, _i64, _i64, _P(HeapView), _vp]),
    "tccl_gather_cols": (C.c_int, [_vp, _i64, _vp, _i64, _i32, _i32, _i32, _P(HeapView), _P(TransportDesc), _vp]),
    "tccl_chained_ag_gemm_rs": (
        C.c_int,
        [_P(GemmDesc), _vp, _i64, _i32, _P(HeapView), _P(SyncDesc), _P(TransportDesc), _i32, _vp],
    ),
    "tccl_gemm_allgather": (
        C.c_int,
        [_P(GemmDesc), _vp, _i64, _P(HeapView), _P(SyncDesc), _P(TransportDesc), _i32, _vp],
    ),
    "tccl_gemm_allgather_static": (
        C.c_int,
        [_P(GemmDesc), _vp, _i64, _P(HeapView), _P(StaticPlan), _P(TransportDesc), _i32, _vp, _i64, _vp],
    ),
    "tccl_static_call_words": (C.c_int, [C.c_uint32, _i32, _P(_i32), _P(_i32), _P(_i32)]),
    "tccl_word_reached": (C.c_int, [_i32, _i32]),
    "tccl_static_reset": (C.c_int, [_vp]),
    "tccl_mfma_rate_probe": (C.c_int, [_i32, _vp, _i64, _vp, _i64, _vp, _i32, _i32, _vp]),
    "tccl_gemm_reducescatter": (
        C.c_int,
        [_P(GemmDesc), _vp, _i32, _i64, _P(HeapView), _P(SyncDesc), _P(TransportDesc), _i32, _i32, _vp],
    ),
}

_lib: C.CDLL | None = None


def load() -> C.CDLL:
    """Load the in-tree library once and type every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    path = Path(os.environ.get("TILECCL_HIP_LIB", LIB_PATH))
    if not path.exists():
        raise RuntimeError(
            f"{path} is missing: the HIP extension has not been built. "
            "Run `python -m tileccl_amd.csrc.build` (or __graft_entry__.build()) first; "
            "there is no non-HIP fallback."
        )
    lib = C.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the build and the header disagree
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.tccl_abi_version() != 1:
        raise RuntimeError(f"{path}: ABI version {lib.tccl_abi_version()} != 1")
    _lib = lib
    return lib


def last_error() -> str:
    return (load().tccl_last_error_string() or b"").decode("utf-8", "replace")


def check(code: int, what: str) -> None:
    """Map a return code to the exception the reference would raise for it.

    Contract violations are ``ValueError`` (reference ``ops.py:1341-1391``); everything the
    runtime refuses or fails at is ``RuntimeError`` (``backends/hip.py:194-197``).
    """
    if code == 0:
        return
    detail = last_error()
    if code in (ERR_INVALID, ERR_UNSUPPORTED):
        raise ValueError(f"{what}: {detail}")
    if code > 0:
        raise RuntimeError(f"HIP error in {what}: error code {code} ({detail})")
    raise RuntimeError(f"{what}: {detail} (code {code})")
