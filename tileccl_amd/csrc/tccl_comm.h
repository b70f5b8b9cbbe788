// Communication role: the workgroups that move (or reduce) finished output while the
// MFMA workgroups keep producing.
//
// Everything that is moved lives in the symmetric heap, so a location is a pair
// (rank, byte offset inside that rank's slice); its address is heap_bases[rank] + offset
// (reference translate_ptr: tileccl/memory/translation.py:39-99).  A transfer is a
// rectangle of rows, cut into 16-byte units (copy) or 8-element units (reduce), and a
// task is a contiguous range of units of one rectangle.  Each lane moves 16 bytes per
// access (global_load_dwordx4 / global_store_dwordx4), a wavefront covers 1 KiB of a row
// per instruction, and every thread keeps several loads in flight before its stores.
//
// Four operations share the machinery (reference call sites in brackets):
//   all-scatter     column block of C -> every peer's C   [patterns/_helpers.py:86-199]
//   all-gather      row block of `out` <-> peers' `out`   [primitives/collectives.py:613-663]
//   reduce-scatter  out = cast(sum over ranks of partial) [primitives/collectives.py:730-783]
//   gather-columns  rank p's input shard -> column block p of this rank's gathered input
//                   [gather worker of patterns/chained_ag_gemm_rs.py:262-340]
// and three granularities: bulk (no waiting; the second kernel of S0), per plan tile
// (S1: locks[tile] >= epoch) and per TileGroup (S2: tile_wait_ge on counter[group]).
#pragma once

#include "tccl_device.h"

namespace tccl {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

enum OpKind { kOpNone = 0, kOpAllScatter = 1, kOpAllGather = 2, kOpReduceScatter = 3, kOpGatherCols = 4, kOpCopyBlock = 5 };
enum Granularity { kBulk = 0, kPerTile = 1, kPerGroup = 2 };
enum { kDirPush = 1, kDirPull = 2 };
enum { kF16 = 0, kBF16 = 1, kF32 = 2 };  // the codes of include/tileccl_hip.h

struct CommArgs {
  int op, granularity, directions;
  const int64_t* heap_bases;
  int rank, world;
  // GEMM output (C) of this rank: base, pitch, shape, element size, plan-tile geometry.
  char* C;
  int64_t ldc_bytes;
  int M, N, esize;
  int block_m, block_n, group_m, tile_rows, tile_cols, xcds, span;
  // all-scatter placement (elements)
  int src_col_off, cols, dst_ld, dst_col_off;
  // all-gather: gathered output of this rank; rank r's block starts at row r*M.
  // gather-columns: C is this rank's input shard (M x N), out the gathered input whose
  // column block r (N columns wide) comes from rank r's shard.
  // copy-block: the rectangle at C (M rows of N bytes, esize 1) is read in slice `copy_src_rank`
  // and written at out in every slice of the mask `copy_dst_ranks`.
  char* out;
  int64_t ld_out_bytes;
  int copy_src_rank;
  uint32_t copy_dst_ranks;
  // reduce-scatter: C is the partial; rs_out the owner's shard
  char* rs_out;
  int64_t ld_rs_out_bytes;
  int partial_dtype, out_dtype, emulate_peer;
  int peers_resident;  // reduce-scatter: the peers' partials are complete in memory, their words are not waited for
  // synchronisation words and TileGroups
  int32_t* locks;
  int32_t* counter;
  int32_t* barrier;
  const int32_t* row_starts;
  const int32_t* row_ends;
  const int32_t* tile_counts;
  int n_groups, epoch;
  int32_t* trace_comm_counter;
  int64_t* trace_ready_clock;
  int64_t* trace_done_clock;
  int64_t* fault;
  int64_t spin_ticks;
  int copy_units, reduce_units;  // units per task
  // Where a peer's signal words are.  0: in the peer's heap slice, at the offset of this
  // rank's.  Otherwise the ranks' words are consecutive blocks of this many bytes outside the
  // heap, rank r's block starting (r - rank) * word_stride bytes from this rank's.
  int64_t word_stride;
};

// Rank `rank`'s copy of the signal words `own` of rank a.rank.
template <typename T>
TCCL_D T* peer_words(const CommArgs& a, T* own, int rank) {
  if (a.word_stride) return (T*)((char*)own + (int64_t)(rank - a.rank) * a.word_stride);
  return translate_ptr(own, a.rank, rank, a.heap_bases);
}

// A rectangle to move.  Offsets are relative to a slice base.
struct Xfer {
  int reduce;          // 0: copy 16-byte units; 1: reduce 8-element units
  uint32_t src_ranks;  // bit mask of slices read (copy: exactly one)
  uint32_t dst_ranks;  // bit mask of slices written
  int first_rank;      // reduce: the addend taken first (the owner)
  int64_t src_off, dst_off;
  int64_t src_pitch, dst_pitch;
  int rows, upr;  // units per row
};

// A window onto a slice region for 16-byte buffer accesses with an explicit cache policy.
// Byte offsets are 32-bit: every rectangle moved here is far smaller than 4 GiB.
TCCL_D __amdgpu_buffer_rsrc_t window(int64_t address) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)(uintptr_t)address, 0, 0xffffffffu, 0x00020000);
}
template <int kPolicy>
TCCL_D u32x4 ld16(__amdgpu_buffer_rsrc_t w, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b128(w, off, 0, kPolicy); }
template <int kPolicy>
TCCL_D void st16(__amdgpu_buffer_rsrc_t w, uint32_t off, u32x4 v) { __builtin_amdgcn_raw_buffer_store_b128(v, w, off, 0, kPolicy); }

constexpr int kThreadsComm = 256;  // threads of a stand-alone communication workgroup
// Cache policy of the stand-alone bulk kernels (the second kernel of S0), measured on the
// 128 MiB exchange that follows the 4096 x 4096 x 1024 GEMM and on the reductions of the
// reduce-scatter configurations: plain (write-back) accesses for copies, 25.5 us against
// 29.8 us with nt; nt for reductions (8192 x 4096 fp32 partials: 66.4 us against 69.8 plain).
constexpr int kBulkCopyPolicy = 0;
constexpr int kBulkReducePolicy = kStreaming;

// ---- copy: units [u_lo, u_hi) of the rectangle, one source slice, any number of targets ----
// kPolicy is the cache policy of both sides: kCoherent inside fused launches (the source
// was just written by other workgroups, the target will be read by a peer), kStreaming
// for the stand-alone bulk kernel.
constexpr int kCopyHalf = 4;  // 16-byte accesses per thread in one of the two register sets

template <int kPolicy, int kThreads>
struct CopyBatch {
  const CommArgs& a;
  const Xfer& x;
  __amdgpu_buffer_rsrc_t src;
  bool flat;
  uint32_t sp, dp;
  int tid, u_hi;

  TCCL_D void load(int u0, u32x4 (&v)[kCopyHalf], uint32_t (&doff)[kCopyHalf]) const {
#pragma unroll
    for (int k = 0; k < kCopyHalf; ++k) {
      const int u = u0 + tid + k * kThreads;
      uint32_t soff;
      if (flat) {
        soff = (uint32_t)u * 16u;
        doff[k] = soff;
      } else {
        const uint32_t r = (uint32_t)u / (uint32_t)x.upr, c = (uint32_t)u - r * (uint32_t)x.upr;
        soff = r * sp + c * 16u;
        doff[k] = r * dp + c * 16u;
      }
      if (u >= u_hi) soff = 0;  // idle lane: harmless re-read of the first unit, nothing stored
      v[k] = ld16<kPolicy>(src, soff);
    }
  }
  TCCL_D void store(int u0, const u32x4 (&v)[kCopyHalf], const uint32_t (&doff)[kCopyHalf]) const {
    for (int q = 0; q < a.world; ++q) {
      if (!((x.dst_ranks >> q) & 1u)) continue;
      const __amdgpu_buffer_rsrc_t dst = window(a.heap_bases[q] + x.dst_off);
#pragma unroll
      for (int k = 0; k < kCopyHalf; ++k)
        if (u0 + tid + k * kThreads < u_hi) st16<kPolicy>(dst, doff[k], v[k]);
    }
  }
};

// Two register sets per thread, one being stored while the other is being loaded: from the second batch
// on a wavefront always has loads and stores in flight together, so the memory system sees reads and writes
// mixed instead of a read phase and a write phase (all workgroups of a launch start together and would
// otherwise alternate in step).
template <int kPolicy, int kThreads>
TCCL_D void run_copy(const CommArgs& a, const Xfer& x, int u_lo, int u_hi) {
  const int src_rank = __builtin_ctz(x.src_ranks);
  const CopyBatch<kPolicy, kThreads> b{a, x, window(a.heap_bases[src_rank] + x.src_off),
                                       (x.src_pitch == (int64_t)x.upr * 16) && (x.dst_pitch == x.src_pitch),
                                       (uint32_t)x.src_pitch, (uint32_t)x.dst_pitch, (int)threadIdx.x, u_hi};
  constexpr int kBatch = kThreads * kCopyHalf;
  u32x4 v0[kCopyHalf], v1[kCopyHalf];
  uint32_t d0[kCopyHalf], d1[kCopyHalf];
  int u0 = u_lo;
  if (u0 >= u_hi) return;
  b.load(u0, v0, d0);
  for (;;) {
    const int u1 = u0 + kBatch;
    if (u1 < u_hi) b.load(u1, v1, d1);
    b.store(u0, v0, d0);
    if (u1 >= u_hi) break;
    const int u2 = u1 + kBatch;
    if (u2 < u_hi) b.load(u2, v0, d0);
    b.store(u1, v1, d1);
    if (u2 >= u_hi) break;
    u0 = u2;
  }
}

// ---- reduce: 8 elements per unit, fp32 accumulation, one rounding to the output type --------
template <typename PT, int kPolicy>
struct Load8;
template <int kPolicy>
struct Load8<float, kPolicy> {
  static TCCL_D void run(__amdgpu_buffer_rsrc_t w, uint32_t off, float (&f)[8]) {
    const f32x4v a = __builtin_bit_cast(f32x4v, ld16<kPolicy>(w, off));
    const f32x4v b = __builtin_bit_cast(f32x4v, ld16<kPolicy>(w, off + 16));
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[e] = a[e];
      f[4 + e] = b[e];
    }
  }
};
template <int kPolicy>
struct Load8<_Float16, kPolicy> {
  static TCCL_D void run(__amdgpu_buffer_rsrc_t w, uint32_t off, float (&f)[8]) {
    const f16x8v h = __builtin_bit_cast(f16x8v, ld16<kPolicy>(w, off));
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (float)h[e];
  }
};
template <int kPolicy>
struct Load8<__bf16, kPolicy> {
  static TCCL_D void run(__amdgpu_buffer_rsrc_t w, uint32_t off, float (&f)[8]) {
    const bf16x8v h = __builtin_bit_cast(bf16x8v, ld16<kPolicy>(w, off));
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (float)h[e];
  }
};

template <typename OT>
TCCL_D u32x4 pack8(const float (&f)[8]);
template <>
TCCL_D u32x4 pack8<_Float16>(const float (&f)[8]) {
  f16x8v h;
#pragma unroll
  for (int e = 0; e < 8; ++e) h[e] = (_Float16)f[e];
  return __builtin_bit_cast(u32x4, h);
}
template <>
TCCL_D u32x4 pack8<__bf16>(const float (&f)[8]) {
  bf16x8v h;
#pragma unroll
  for (int e = 0; e < 8; ++e) h[e] = (__bf16)f[e];
  return __builtin_bit_cast(u32x4, h);
}


// One reduced unit (8 elements) to the output: 16 bytes of fp16 / bf16, 32 bytes of fp32.
template <typename OT, int kPolicy>
TCCL_D void store8(__amdgpu_buffer_rsrc_t w, uint32_t off, const float (&f)[8]) {
  if constexpr (sizeof(OT) == 4) {
    f32x4v lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = f[e];
      hi[e] = f[4 + e];
    }
    st16<kPolicy>(w, off, __builtin_bit_cast(u32x4, lo));
    st16<kPolicy>(w, off + 16, __builtin_bit_cast(u32x4, hi));
  } else {
    st16<kPolicy>(w, off, pack8<OT>(f));
  }
}

// Sum order: the owner's addend first, then the other ranks in ascending order
// (tile_reduce_scatter: local chunk, then peers ascending; collectives.py:766-781).
template <typename PT, typename OT, int kPolicy, int kThreads>
TCCL_D void run_reduce_t(const CommArgs& a, const Xfer& x, int u_lo, int u_hi) {
  constexpr uint32_t kSrcUnit = 8 * sizeof(PT);
  // Units a thread keeps in flight.  Measured on the bulk reductions of 8192 x 4096 fp32 and
  // 16384 x 4096 bf16 partials with 4 workgroups of 256 threads per CU: 2 units 68.0 / 126.0 us,
  // 4 units 66.4 / 114.3 us, 8 units 84.4 / 140.8 us (the registers of the widest path set the
  // occupancy of the whole kernel).
  constexpr int kReduceUnroll = 4;
  const int tid = threadIdx.x;
  const int dst_rank = __builtin_ctz(x.dst_ranks);
  const __amdgpu_buffer_rsrc_t dst = window(a.heap_bases[dst_rank] + x.dst_off);
  const __amdgpu_buffer_rsrc_t first = window(a.heap_bases[x.first_rank] + x.src_off);
  const uint32_t sp = (uint32_t)x.src_pitch, dp = (uint32_t)x.dst_pitch;
  for (int u0 = u_lo; u0 < u_hi; u0 += kThreads * kReduceUnroll) {
    float acc[kReduceUnroll][8];
    uint32_t soff[kReduceUnroll], doff[kReduceUnroll];
#pragma unroll
    for (int k = 0; k < kReduceUnroll; ++k) {
      const int u = u0 + tid + k * kThreads;
      const uint32_t r = (uint32_t)u / (uint32_t)x.upr, c = (uint32_t)u - r * (uint32_t)x.upr;
      soff[k] = r * sp + c * kSrcUnit;
      doff[k] = r * dp + c * (8u * (uint32_t)sizeof(OT));
      if (u >= u_hi) soff[k] = 0;  // idle lane: harmless re-read, nothing stored
      Load8<PT, kPolicy>::run(first, soff[k], acc[k]);
    }
    for (int p = 0; p < a.world; ++p) {
      if (p == x.first_rank || !((x.src_ranks >> p) & 1u)) continue;
      const __amdgpu_buffer_rsrc_t other = window(a.heap_bases[p] + x.src_off);
#pragma unroll
      for (int k = 0; k < kReduceUnroll; ++k) {
        float in[8];
        Load8<PT, kPolicy>::run(other, soff[k], in);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[k][e] += in[e];
      }
    }
#pragma unroll
    for (int k = 0; k < kReduceUnroll; ++k)
      if (u0 + tid + k * kThreads < u_hi) store8<OT, kPolicy>(dst, doff[k], acc[k]);
  }
}

template <int kPolicy, int kThreads>
TCCL_D void run_reduce(const CommArgs& a, const Xfer& x, int u_lo, int u_hi) {
  const int key = a.partial_dtype * 4 + a.out_dtype;
  switch (key) {
    case kF32 * 4 + kF16: run_reduce_t<float, _Float16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kF32 * 4 + kBF16: run_reduce_t<float, __bf16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kF16 * 4 + kF16: run_reduce_t<_Float16, _Float16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kBF16 * 4 + kBF16: run_reduce_t<__bf16, __bf16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kBF16 * 4 + kF16: run_reduce_t<__bf16, _Float16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kF16 * 4 + kBF16: run_reduce_t<_Float16, __bf16, kPolicy, kThreads>(a, x, u_lo, u_hi); break;
    case kF32 * 4 + kF32:  // the stand-alone reduction only: the fused launches write 16-bit shards
      if constexpr (kPolicy != kCoherent) run_reduce_t<float, float, kPolicy, kThreads>(a, x, u_lo, u_hi);
      break;
    default: break;
  }
}

// kOnly names what a stand-alone bulk kernel is compiled for (kAllRoles: everything, fused launches included).
enum BulkOnly { kAllRoles = 0, kBulkCopy = 1, kBulkReduce = 2 };

template <int kThreads, int kOnly = kAllRoles>
TCCL_D void run_xfer(const CommArgs& a, const Xfer& x, int u_lo, int u_hi) {
  if constexpr (kOnly == kBulkCopy) {
    run_copy<kBulkCopyPolicy, kThreads>(a, x, u_lo, u_hi);
    return;
  }
  if constexpr (kOnly == kBulkReduce) {
    if (x.reduce) run_reduce<kBulkReducePolicy, kThreads>(a, x, u_lo, u_hi);
    return;
  }
  const bool fused = a.granularity != kBulk;
  if (x.reduce) {
    if (fused)
      run_reduce<kCoherent, kThreads>(a, x, u_lo, u_hi);
    else
      run_reduce<kBulkReducePolicy, kThreads>(a, x, u_lo, u_hi);
  } else {
    if (fused)
      run_copy<kCoherent, kThreads>(a, x, u_lo, u_hi);
    else
      run_copy<kBulkCopyPolicy, kThreads>(a, x, u_lo, u_hi);
  }
}

// ---- rectangles of the three operations ----------------------------------------------------------
// `peer` is the other party of a pull (the slice read); pushes fan out to all peers.
// Rows [r0, r1) and columns [c0, c1) are relative to this rank's GEMM output C.
TCCL_D uint32_t all_ranks(int world) { return world >= 32 ? 0xffffffffu : ((1u << world) - 1u); }

TCCL_D int64_t slice_offset(const CommArgs& a, const char* p) { return (int64_t)(uintptr_t)p - a.heap_bases[a.rank]; }

// Returns false when the rectangle is empty.
TCCL_D bool make_xfer(const CommArgs& a, bool pull, int peer, int r0, int r1, int c0, int c1, Xfer& x) {
  if (r1 > a.M) r1 = a.M;
  if (c1 > a.N) c1 = a.N;
  x.reduce = 0;
  x.first_rank = a.rank;
  if (a.op == kOpAllScatter) {
    // Only columns inside [src_col_off, src_col_off + cols) travel (_helpers.py:148-151).
    const int lo = c0 > a.src_col_off ? c0 : a.src_col_off;
    const int hi = c1 < a.src_col_off + a.cols ? c1 : a.src_col_off + a.cols;
    if (lo >= hi || r0 >= r1) return false;
    const int64_t c_off = slice_offset(a, a.C);
    x.src_ranks = 1u << a.rank;
    x.dst_ranks = all_ranks(a.world) & ~(1u << a.rank);
    x.src_pitch = a.ldc_bytes;
    x.dst_pitch = (int64_t)a.dst_ld * a.esize;
    x.src_off = c_off + r0 * x.src_pitch + (int64_t)lo * a.esize;
    x.dst_off = c_off + r0 * x.dst_pitch + (int64_t)(a.dst_col_off + lo - a.src_col_off) * a.esize;
    x.rows = r1 - r0;
    x.upr = (hi - lo) * a.esize / 16;
    return x.dst_ranks != 0;
  }
  if (r0 >= r1 || c0 >= c1) return false;
  if (a.op == kOpAllGather) {
    // Block of rank b sits at rows [b*M, (b+1)*M) of every rank's `out` (collectives.py:628-630).
    const int owner = pull ? peer : a.rank;
    const int64_t off = slice_offset(a, a.out) + ((int64_t)owner * a.M + r0) * a.ld_out_bytes + (int64_t)c0 * a.esize;
    x.src_ranks = 1u << owner;
    x.dst_ranks = pull ? (1u << a.rank) : (all_ranks(a.world) & ~(1u << a.rank));
    x.src_off = x.dst_off = off;
    x.src_pitch = x.dst_pitch = a.ld_out_bytes;
    x.rows = r1 - r0;
    x.upr = (c1 - c0) * a.esize / 16;
    return x.dst_ranks != 0;
  }
  if (a.op == kOpCopyBlock) {
    // tile_put / tile_get (primitives/communication.py:133-225) on a whole rectangle: both
    // addresses are the calling rank's own, translated into the slices named.
    x.src_ranks = 1u << a.copy_src_rank;
    x.dst_ranks = a.copy_dst_ranks;
    x.src_pitch = a.ldc_bytes;
    x.dst_pitch = a.ld_out_bytes;
    x.src_off = slice_offset(a, a.C) + r0 * x.src_pitch + (int64_t)c0 * a.esize;
    x.dst_off = slice_offset(a, a.out) + r0 * x.dst_pitch + (int64_t)c0 * a.esize;
    x.rows = r1 - r0;
    x.upr = (c1 - c0) * a.esize / 16;
    return x.dst_ranks != 0;
  }
  if (a.op == kOpGatherCols) {
    // Column block `owner` of this rank's gathered input is rank `owner`'s shard
    // (chained_ag_gemm_rs.py:270-337); the "push" direction is the copy of the own shard.
    const int owner = pull ? peer : a.rank;
    x.src_ranks = 1u << owner;
    x.dst_ranks = 1u << a.rank;
    x.src_pitch = a.ldc_bytes;
    x.dst_pitch = a.ld_out_bytes;
    x.src_off = slice_offset(a, a.C) + r0 * x.src_pitch + (int64_t)c0 * a.esize;
    x.dst_off = slice_offset(a, a.out) + r0 * x.dst_pitch + ((int64_t)owner * a.N + c0) * a.esize;
    x.rows = r1 - r0;
    x.upr = (c1 - c0) * a.esize / 16;
    return true;
  }
  // Reduce-scatter: rows belong to owner = row / (M / world); the owner's shard is rs_out.
  const int shard = a.M / a.world;
  const int owner = r0 / shard;
  if (owner != a.rank && !a.emulate_peer) return false;
  const int out_esize = a.out_dtype == kF32 ? 4 : 2;
  x.reduce = 1;
  x.first_rank = owner;
  x.src_ranks = all_ranks(a.world);
  x.dst_ranks = 1u << owner;
  x.src_pitch = a.ldc_bytes;
  x.dst_pitch = a.ld_rs_out_bytes;
  x.src_off = slice_offset(a, a.C) + r0 * x.src_pitch + (int64_t)c0 * a.esize;
  x.dst_off = slice_offset(a, a.rs_out) + (int64_t)(r0 - owner * shard) * x.dst_pitch + (int64_t)c0 * out_esize;
  x.rows = r1 - r0;
  x.upr = (c1 - c0) / 8;
  return true;
}

// ---- waiting -------------------------------------------------------------------------------------
// One lane spins; the verdict is shared through one LDS word.  Returns false on timeout,
// after raising *fault, so that every workgroup still runs to its end.
struct Waiter {
  const CommArgs& a;
  volatile int* verdict;
  int64_t deadline;

  TCCL_D bool finish(bool ok) const {
    if (threadIdx.x == 0) {
      if (!ok && a.fault) *a.fault = 1;
      *verdict = ok ? 1 : 0;
    }
    __syncthreads();
    const bool all_ok = *verdict != 0;
    __syncthreads();
    return all_ok;  // the data itself is read with device-coherent loads: no cache invalidate
  }

  // S1: locks[tile] of `rank`'s slice has reached this launch's epoch (tile_publish).  The
  // word is only observed, whoever owns it: several parties may depend on the same tile.
  TCCL_D bool tile(int tile_id, int rank) const {
    if (rank != a.rank && a.peers_resident) return true;
    bool ok = true;
    if (threadIdx.x == 0) {
      const int32_t* w = peer_words(a, a.locks, rank);
      ok = tile_wait_ge<true>(w, tile_id, a.epoch, deadline);
    }
    return finish(ok);
  }

  // S2: counter[g] of every slice in `ranks` has reached epoch * tile_counts[g].
  TCCL_D bool group(int g, uint32_t ranks) const {
    bool ok = true;
    if (a.peers_resident) ranks &= 1u << a.rank;
    if (threadIdx.x == 0) {
      const int32_t need = (int32_t)((uint32_t)a.epoch * (uint32_t)a.tile_counts[g]);
      for (int r = 0; r < a.world && ok; ++r)
        if ((ranks >> r) & 1u) ok = tile_wait_ge<true>(peer_words(a, a.counter, r), g, need, deadline);
      if (ok && a.trace_ready_clock) {
        unsigned long long* slot = (unsigned long long*)&a.trace_ready_clock[g];
        atomicCAS(slot, 0ull, (unsigned long long)now_ticks());
      }
    }
    return finish(ok);
  }
};

// A finished task of group g: count it; the task that completes the group stamps the clock.
TCCL_D void task_done(const CommArgs& a, int g, int tasks_of_group) {
  wait_vmem();  // this wave's write-through stores have landed
  __syncthreads();
  if (threadIdx.x == 0) {
    if (a.trace_comm_counter) atomicAdd(&a.trace_comm_counter[g], 1);
    if (a.barrier) {
      const int32_t prev = tile_signal_add<true>(a.barrier, g, 1);
      if (prev + 1 == a.epoch * tasks_of_group && a.trace_done_clock) a.trace_done_clock[g] = now_ticks();
    }
  }
}

TCCL_D int cdiv(int x, int y) { return (x + y - 1) / y; }

// Without a plan (row_starts == nullptr) the whole output is one group; for a
// reduce-scatter it is one group per owner shard, so no task straddles two owners.
TCCL_D int group_lo(const CommArgs& a, int g) {
  if (a.row_starts) return a.row_starts[g];
  return a.op == kOpReduceScatter ? g * (a.M / a.world) : 0;
}
TCCL_D int group_hi(const CommArgs& a, int g) {
  if (a.row_ends) return a.row_ends[g];
  return a.op == kOpReduceScatter ? (g + 1) * (a.M / a.world) : a.M;
}
// Reduce-scatter rows this rank neither owns nor reduces on the owner's behalf.
TCCL_D bool rs_not_mine(const CommArgs& a, int row) {
  return a.op == kOpReduceScatter && !a.emulate_peer && row / (a.M / a.world) != a.rank;
}

// ---- the role ---------------------------------------------------------------------------------------
// Tasks are numbered so that whatever can start earliest comes first: pulls (their
// sources are ready or soon will be, independent of this rank's GEMM), then pushes /
// reductions in production order.  Workgroup w takes tasks w, w + n, w + 2n, ...; no
// GEMM workgroup ever waits on a communication workgroup, so the order is deadlock-free.
template <int kThreads = kThreadsComm, int kOnly = kAllRoles>
TCCL_D void comm_role(const CommArgs& a, int wg, int num_wgs, int* lds_word) {
  if (a.op == kOpNone || num_wgs <= 0) return;
  Waiter wait{a, lds_word, now_ticks() + a.spin_ticks};
  const int peers = a.world - 1;
  const bool is_rs = a.op == kOpReduceScatter;
  const bool do_pull = (a.op == kOpAllGather || a.op == kOpGatherCols) && (a.directions & kDirPull) && peers > 0;
  const bool do_push = is_rs || (a.directions & kDirPush);
  const int unit_elems = is_rs ? 8 : 16 / a.esize;
  const int units_per_task = is_rs ? a.reduce_units : a.copy_units;

  if (kOnly == kAllRoles && a.granularity == kPerTile) {
    const int total = a.tile_rows * a.tile_cols;
    const int n_pull = do_pull ? peers * total : 0;
    const int n_all = n_pull + (do_push ? total : 0);
    for (int t = wg; t < n_all; t += num_wgs) {
      const bool pull = t < n_pull;
      const int local = pull ? t % total : t - n_pull;
      int peer = a.rank;
      if (pull) {
        peer = t / total;
        if (peer >= a.rank) ++peer;
      }
      const int tile_id = tile_for_slot(local, total, a.xcds, a.span);
      const TileCoord tc = tile_coords(tile_id, a.tile_rows, a.tile_cols, a.group_m);
      bool ok;
      if (pull) {
        ok = wait.tile(tile_id, peer);
      } else {
        ok = wait.tile(tile_id, a.rank);
        if (is_rs)  // the peers' partial tiles must be there as well
          for (int p = 0; p < a.world && ok; ++p)
            if (p != a.rank) ok = wait.tile(tile_id, p);
      }
      Xfer x;
      const int r0 = tc.m * a.block_m, c0 = tc.n * a.block_n;
      if (ok && make_xfer(a, pull, peer, r0, r0 + a.block_m, c0, c0 + a.block_n, x)) run_xfer<kThreads>(a, x, 0, x.rows * x.upr);
    }
    return;
  }

  // Bulk and per-group: tasks are ranges of units_per_task units of a group's rectangle
  // (bulk treats the plan's groups as plain work partitions and never waits).
  const int row_units = is_rs ? a.N / 8 : (a.op == kOpAllScatter ? a.cols : a.N) / unit_elems;
  int total = 0;
  for (int g = 0; g < a.n_groups; ++g) total += cdiv((group_hi(a, g) - group_lo(a, g)) * row_units, units_per_task);
  const int n_pull = do_pull ? peers * total : 0;
  const int n_all = n_pull + (do_push ? total : 0);
  const int tasks_factor = (do_pull ? peers : 0) + (do_push ? 1 : 0);
  for (int t = wg; t < n_all; t += num_wgs) {
    const bool pull = t < n_pull;
    int local = pull ? t % total : t - n_pull;
    int peer = a.rank;
    if (pull) {
      peer = t / total;
      if (peer >= a.rank) ++peer;
    }
    int g = 0, tasks_g = 0;
    for (; g < a.n_groups; ++g) {
      tasks_g = cdiv((group_hi(a, g) - group_lo(a, g)) * row_units, units_per_task);
      if (local < tasks_g) break;
      local -= tasks_g;
    }
    if (g >= a.n_groups) break;
    if (rs_not_mine(a, group_lo(a, g))) continue;
    bool ok = true;
    if (kOnly == kAllRoles && a.granularity == kPerGroup) {
      uint32_t ranks = pull ? (1u << peer) : (is_rs ? all_ranks(a.world) : (1u << a.rank));
      ok = wait.group(g, ranks);
    }
    Xfer x;
    if (ok && make_xfer(a, pull, peer, group_lo(a, g), group_hi(a, g), 0, a.N, x)) {
      const int units = x.rows * x.upr;
      const int lo = local * units_per_task;
      const int hi = lo + units_per_task < units ? lo + units_per_task : units;
      if (lo < hi) run_xfer<kThreads, kOnly>(a, x, lo, hi);
    }
    if (kOnly == kAllRoles && a.granularity == kPerGroup) task_done(a, g, tasks_g * tasks_factor);
  }
}

}  // namespace tccl
