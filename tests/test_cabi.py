"""The C-ABI library without a GPU: it loads, exports every symbol the header declares,
rejects bad descriptors before touching a device, and its host-side index helpers (the very
functions the kernels inline) agree with the loop-form oracle."""

import ctypes as C
import re
from pathlib import Path

import pytest

from oracle import planning as ref

HEADER = Path(__file__).resolve().parent.parent / "include" / "tileccl_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(tccl_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_typed(lib):
    from tileccl_amd import _lib

    names = declared_functions()
    assert len(names) >= 22 and "tccl_copy_block" in names and "tccl_gemm_allgather" in names and "tccl_chained_ag_gemm_rs" in names
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names  # the ctypes table covers the header exactly
    assert lib.tccl_abi_version() == 1


def test_struct_layouts_match_the_header():
    from tileccl_amd import _lib

    # sizes follow from the header's field lists under the natural C alignment rules
    assert C.sizeof(_lib.GemmDesc) == 3 * 8 + 3 * 4 + 4 + 3 * 8 + 2 * 4 + 4 + 3 * 4 + 4 + 3 * 4
    assert C.sizeof(_lib.HeapView) == 16 and C.sizeof(_lib.ScatterDesc) == 16 and C.sizeof(_lib.TransportDesc) == 16
    assert C.sizeof(_lib.SyncDesc) == 4 * 8 + 2 * 4 + 8 * 8 + 8
    assert C.sizeof(_lib.DeviceInfo) == 8 * 4 + 64
    assert _lib.GemmDesc.lda.offset == 40 and _lib.SyncDesc.row_starts.offset == 40


def test_bad_descriptors_are_rejected_on_the_host(lib):
    from tileccl_amd import _lib

    assert lib.tccl_gemm(None, None) == _lib.ERR_INVALID
    assert b"NULL" in lib.tccl_last_error_string()
    d = _lib.GemmDesc()
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_INVALID
    d.A = d.B = d.C = 0x1000
    d.M, d.N, d.K = 128, 128, 0
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_INVALID
    assert b"M, N, K must be positive" in lib.tccl_last_error_string()
    d.K = 64
    d.lda, d.ldb, d.ldc = 64, 128, 128
    d.block_m, d.block_n, d.group_m = 96, 128, 8
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_UNSUPPORTED
    d.block_m = 128
    d.in_dtype = _lib.F32
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_UNSUPPORTED
    d.in_dtype = _lib.F16
    d.A = 0x1008  # not 16-byte aligned
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_UNSUPPORTED
    with pytest.raises(ValueError, match="16-byte boundaries"):
        _lib.check(_lib.ERR_UNSUPPORTED, "tccl_gemm")
    with pytest.raises(RuntimeError, match="HIP error in x: error code 2"):
        _lib.check(2, "x")
    d.A = 0x1000
    d.K, d.lda, d.ldb = 1 << 16, 1 << 16, 1 << 16  # B would span 8 GiB: 32-bit offsets cannot reach it
    d.N = d.ldc = 1 << 16
    assert lib.tccl_gemm(C.byref(d), None) == _lib.ERR_UNSUPPORTED
    assert b"spans more than 4 GiB" in lib.tccl_last_error_string()
    d.K, d.lda, d.ldb, d.N, d.ldc = 64, 64, 128, 128, 128
    h = _lib.HeapView(0x1000, 3, 2)
    assert lib.tccl_exchange_rows(0x1000, 8, 8, 8, 2, C.byref(h), None, None) == _lib.ERR_INVALID
    assert b"rank=3 out of range for world_size=2" in lib.tccl_last_error_string()
    # gather-columns and the chained operation: host-side checks come before any device call
    h2 = _lib.HeapView(0x1000, 0, 2)
    assert lib.tccl_gather_cols(0x2000, 128, 0x1000, 64, 16, 64, 2, None, None, None) == _lib.ERR_INVALID
    assert lib.tccl_gather_cols(0x2000, 100, 0x1000, 64, 16, 64, 2, C.byref(h2), None, None) == _lib.ERR_INVALID
    assert b"gathered rows hold 100 elements, need 128" in lib.tccl_last_error_string()
    assert lib.tccl_gather_cols(0x2000, 128, 0x1000, 64, 16, 60, 2, C.byref(h2), None, None) == _lib.ERR_UNSUPPORTED
    d.A = 0x1000
    d.K, d.lda = 192, 192
    assert lib.tccl_chained_ag_gemm_rs(C.byref(d), 0x3000, 64, 64, C.byref(h2), None, None, _lib.S0_BULK, None) == _lib.ERR_INVALID
    assert b"input_shard columns (64) * world_size (2) != W rows (192)" in lib.tccl_last_error_string()
    # block copy: argument checks come before any device call
    assert lib.tccl_copy_block(0x2000, 0b11, 0x1000, 2, 1, 64, 64, 64, C.byref(h2), None) == _lib.ERR_INVALID
    assert b"src_rank=2 out of range" in lib.tccl_last_error_string()
    assert lib.tccl_copy_block(0x2000, 0b100, 0x1000, 0, 1, 64, 64, 64, C.byref(h2), None) == _lib.ERR_INVALID
    assert b"names ranks beyond world_size=2" in lib.tccl_last_error_string()
    assert lib.tccl_copy_block(0x2000, 0b11, 0x1000, 0, 1, 40, 64, 64, C.byref(h2), None) == _lib.ERR_UNSUPPORTED
    assert lib.tccl_copy_block(0x2000, 0, 0x1000, 0, 1, 64, 64, 64, C.byref(h2), None) == 0  # nobody to write to
    # a block whose rows reach beyond 32-bit offsets is refused before any launch
    assert lib.tccl_exchange_rows(0x1000, 1 << 20, 4096, 4096, 2, C.byref(h2), None, None) == _lib.ERR_UNSUPPORTED
    assert b"spans more than 4 GiB" in lib.tccl_last_error_string()
    assert lib.tccl_heap_create(0, 2, None, None) == _lib.ERR_INVALID
    assert lib.tccl_heap_destroy(None) == 0
    assert lib.tccl_fill_i32(None, 0, 0, None) == 0


@pytest.mark.parametrize("tile_rows,tile_cols,group_m", [(32, 32, 8), (12, 2, 8), (7, 5, 3), (1, 9, 8), (64, 32, 8), (5, 1, 1)])
def test_device_tile_order_equals_the_reference_swizzle(lib, tile_rows, tile_cols, group_m):
    tm, tn = C.c_int32(), C.c_int32()
    seen = set()
    for t in range(tile_rows * tile_cols):
        assert lib.tccl_tile_coords(t, tile_rows, tile_cols, group_m, C.byref(tm), C.byref(tn)) == 0
        assert (tm.value, tn.value) == ref.swizzle(t, tile_rows, tile_cols, group_m)
        seen.add((tm.value, tn.value))
    assert len(seen) == tile_rows * tile_cols  # a bijection onto the tile grid
    assert lib.tccl_tile_coords(tile_rows * tile_cols, tile_rows, tile_cols, group_m, C.byref(tm), C.byref(tn)) != 0


@pytest.mark.parametrize("total,xcds,span", [(1024, 8, 32), (1000, 8, 32), (16, 8, 8), (2048, 8, 32), (513, 8, 4), (64, 1, 1), (4096, 8, 64),
                                             (1024, 8, 64), (256, 8, 32), (576, 8, 64), (100, 8, 12), (7, 8, 1)])
def test_xcd_remap_is_a_bijection_and_keeps_blocks(lib, total, xcds, span):
    out = C.c_int32()
    ids = []
    for slot in range(total):
        assert lib.tccl_tile_for_slot(slot, total, xcds, span, C.byref(out)) == 0
        ids.append(out.value)
    assert sorted(ids) == list(range(total))
    block = xcds * span
    for slot, tile in enumerate(ids):
        assert slot // block == tile // block  # a slot never leaves its block of xcds*span ids
        if xcds > 1 and (slot // block + 1) * block <= total:
            # XCD slot % xcds takes the span ids [x*span, (x+1)*span) of the block, in order
            assert (tile % block) // span == slot % xcds and (tile % block) % span == (slot % block) // xcds
        else:
            assert tile == slot


def test_signal_words_compare_as_sequence_numbers(lib):
    """word_reached: `word >= need` for values that have not wrapped, and across a wrap of either."""
    reached = lib.tccl_word_reached
    assert reached(5, 5) and reached(6, 5) and not reached(4, 5)
    assert reached(0, 0) and not reached(0, 1)
    top = 2**31 - 1
    assert reached(top, top - 10) and not reached(top - 10, top)
    assert reached(-(2**31), top)  # one past the largest int32: the word has wrapped, the threshold has not
    assert not reached(top, -(2**31))
    assert reached(-5, -9) and not reached(-9, -5)


def test_static_entry_launch_numbers(lib):
    """The bookkeeping of tccl_gemm_allgather_static: call n stores n into its locks and takes each TileGroup
    counter from `start` to `ready` = start + tile_count; a peer in call n waits for `ready`, and nothing that an
    earlier call left behind (with any tile count) satisfies it, nor anything call n itself writes before the
    group is complete -- also where the 32-bit values wrap."""
    from tileccl_amd import _lib

    def words(call, tiles):
        epoch, start, ready = C.c_int32(), C.c_int32(), C.c_int32()
        assert lib.tccl_static_call_words(call, tiles, C.byref(epoch), C.byref(start), C.byref(ready)) == 0
        return epoch.value, start.value, ready.value

    reached = lib.tccl_word_reached
    unit = 2 * _lib.STATIC_MAX_TILES
    assert words(1, 7) == (1, unit - 7, unit)
    assert words(2, 16384) == (2, 2 * unit - 16384, 2 * unit)
    wrap = 2**32 // unit  # the call at which counter values wrap modulo 2^32
    for call in (1, 2, 3, 1000, 65535, 65536, 65537, wrap - 1, wrap, wrap + 1, 2**31 - 2, 2**31 - 1, 2**31, 2**31 + 1, 2**32 - 1):
        for tiles in (1, 256, 16384):
            epoch, start, ready = words(call, tiles)
            assert 1 <= epoch <= 2**31 - 1
            assert (ready - start) % 2**32 == tiles
            assert reached(ready, ready) and not reached(start, ready)
            assert not reached((ready - 1 + 2**31) % 2**32 - 2**31, ready)  # one tile short
            if call > 1:
                for old_tiles in (1, 16384):
                    old_epoch, _, old_ready = words(call - 1, old_tiles)
                    assert not reached(old_ready, ready), (call, tiles)
                    if old_epoch < epoch:  # (the lock value restarts at 1 after 2^31 - 1 calls)
                        assert not reached(old_epoch, epoch)
    for bad in ((0, 1), (1, -1), (1, 16385)):
        assert lib.tccl_static_call_words(bad[0], bad[1], None, None, None) != 0
