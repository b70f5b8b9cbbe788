// Persistent MFMA GEMM role for gfx950 (CDNA4), 16-bit inputs.
//
// One workgroup = 256 threads = 4 wavefronts (2 x 2), producing 128 x 128 output
// sub-tiles with K consumed 64 at a time.  A plan tile (block_m x block_n, multiples of
// 128) is a small loop of such sub-tiles; when the whole plan tile is in memory the
// workgroup publishes it (per-tile lock or per-TileGroup counter).
//
// Data path of one K step
//   global --16B/lane--> registers --> LDS --ds_read_b128--> MFMA operands
//   LDS holds both operands "k-chunked": [k/8][row][8 values], so one 16-byte read gives
//   a lane the 8 consecutive k it feeds to v_mfma_f32_32x32x16_{f16,bf16}.
//   A (M x K, k-contiguous) lands in that layout directly.  B (K x N, n-contiguous) is
//   transposed in registers on the way in: a thread owns a 4(k) x 8(n) patch, repacks it
//   to 8 x (4 consecutive k) and writes eight 8-byte words.
//   A k-major B (GemmArgs::b_kmajor: element (k, n) at B[n * ldb + k]) takes A's route: loaded
//   by rows of n, it is already in the k-chunked layout.
//   LDS is single-buffered; the next K step's global loads are issued before the MFMAs
//   of the current one, so two workgroups per CU keep the matrix cores fed.
//
// MFMA orientation: the B patch is passed as the instruction's first operand and the A
// patch as its second, i.e. the instruction computes the transposed 32 x 32 block.  Each
// lane then owns 4 *consecutive output columns* of one output row, which makes the
// register->LDS->global epilogue 8/16-byte wide instead of 2-byte wide.
//
// Reference semantics reproduced: C = A @ B with fp32 accumulation and one rounding to
// the output type (tileccl/kernels/gemm.py:139-167); rows/columns past M/N are not
// written (gemm.py:163-167); the K tail is zero-filled (gemm.py:153-160).
#pragma once

#include "tccl_device.h"

namespace tccl {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kTile = 128;        // sub-tile edge
constexpr int kBK = 64;           // K per step
constexpr int kThreads = 256;     // threads per workgroup
constexpr int kPlane = 130 * 16;  // bytes of one k-chunk plane: 128 rows x 16 B + 2 pad rows
constexpr int kOperandBytes = (kBK / 8) * kPlane;  // one operand, one K step
constexpr int kLdsBytes = 2 * kOperandBytes;       // A then B

enum SignalMode { kSignalNone = 0, kSignalTile = 1, kSignalGroup = 2 };

struct GemmArgs {
  const void* A;
  const void* B;
  void* C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  float alpha;
  int block_m, block_n, group_m;  // plan tile and swizzle band
  int tile_rows, tile_cols;       // plan tiles
  int xcds, span;                 // slot -> tile remap
  // Column shards stacked as row blocks (0: plain GEMM): C row block q of wrap_rows rows is
  // A (wrap_rows x K) times columns [q * N, (q + 1) * N) of B; tiles never straddle two blocks.
  int wrap_rows;
  // B is k-major: element (k, n) at B[n * ldb + k] (the `.t()` view of an (N, K) tensor).
  int b_kmajor;
};

// Where a tile whose first output row is row0 and first output column col0 reads its operands.
struct OperandOrigin {
  int a_row, a_rows;  // first row of A, rows A has
  int b_col, b_cols;  // first column of B, columns B has
};
TCCL_HD OperandOrigin operand_origin(const GemmArgs& g, int row0, int col0) {
  OperandOrigin o;
  if (g.wrap_rows > 0) {
    int wrap_rows = g.wrap_rows;
#if defined(__HIP_DEVICE_COMPILE__)
    // Hidden from the optimiser: it would otherwise prepare this division (a reciprocal and its
    // corrections) at the kernel's start for every launch, column shards or not.
    asm volatile("" : "+s"(wrap_rows));
#endif
    const int q = row0 / wrap_rows;
    o.a_row = row0 - q * wrap_rows;
    o.a_rows = wrap_rows;
    o.b_col = col0 + q * g.N;
    o.b_cols = (g.M / wrap_rows) * g.N;
  } else {
    o.a_row = row0;
    o.a_rows = g.M;
    o.b_col = col0;
    o.b_cols = g.N;
  }
  return o;
}

struct SignalArgs {
  int mode;
  int32_t* locks;
  const int32_t* group_table;
  int32_t* counter;
  const int32_t* tile_counts;
  int epoch;  // launch number: locks[tile] = epoch (tile mode); a group is complete at epoch * tile_counts[g]
  // optional device trace: the producer that completes a group stamps its clock
  int64_t* trace_ready_clock;
};

template <typename T>
struct Mfma;
template <>
struct Mfma<_Float16> {
  typedef f16x8 Vec;
  static TCCL_D f32x16 run(Vec a, Vec b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  // 16 x 16 x 32: lane l holds 8 consecutive k (group l / 16) of row / column l % 16 and gets
  // D[4 * (l / 16) + e][l % 16], e = 0..3.
  static TCCL_D f32x4 run16(Vec a, Vec b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <>
struct Mfma<__bf16> {
  typedef bf16x8 Vec;
  static TCCL_D f32x16 run(Vec a, Vec b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static TCCL_D f32x4 run16(Vec a, Vec b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

// fp32 -> output element, round to nearest even (what a cast of the accumulator does in
// the reference, gemm.py:167 / bulk_sync.py:238).
template <typename OutT>
TCCL_D OutT to_out(float v);
template <>
TCCL_D _Float16 to_out<_Float16>(float v) { return (_Float16)v; }
template <>
TCCL_D __bf16 to_out<__bf16>(float v) { return (__bf16)v; }
template <>
TCCL_D float to_out<float>(float v) { return v; }

// 16-byte slot of row `n` inside a k-chunk plane of the B operand.  The XOR keeps both
// the transposing writes (lanes 8 rows apart) and the MFMA reads (32 consecutive rows)
// spread over all LDS banks.
TCCL_D int b_slot(int n) { return n ^ (n >> 4); }

template <typename InT, typename OutT>
struct GemmRole {
  typedef typename Mfma<InT>::Vec Vec;

  const GemmArgs& g;
  char* lds;
  const int tid, lane, wave, wm, wn;

  TCCL_D GemmRole(const GemmArgs& args, char* smem)
      : g(args), lds(smem), tid(threadIdx.x), lane(threadIdx.x & 63), wave(threadIdx.x >> 6),
        wm((threadIdx.x >> 6) >> 1), wn((threadIdx.x >> 6) & 1) {}

  // ---- global -> registers ------------------------------------------------------------
  // Loads go through buffer resources: an access past num_records returns zero, which
  // pads rows >= M of A and rows >= K of B without branches or clamped addresses.
  //   A: chunk c = tid + 256*i covers row (c >> 3), k-chunk (c & 7).
  //   B: thread owns k rows 4*(tid >> 4) .. +3 and columns 8*(tid & 15) .. +7.
  // Columns >= N of B read whatever follows in memory (still inside the buffer); they
  // only feed output columns that are never stored.
  struct Source {
    __amdgpu_buffer_rsrc_t a, b;
    uint32_t off_a[4], off_b[4];  // byte offsets of this thread's 16-byte loads, K step 0
    uint32_t step_a, step_b;      // byte advance per K step
  };

  static TCCL_D uint32_t clamp_u32(int64_t v) { return v > 0xffffffffll ? 0xffffffffu : (v < 0 ? 0u : (uint32_t)v); }

  TCCL_D Source make_source(int row0, int col0) const {
    constexpr int kEsz = sizeof(InT);
    Source s;
    const OperandOrigin o = operand_origin(g, row0, col0);
    const InT* A = (const InT*)g.A + (int64_t)o.a_row * g.lda;
    const InT* B = (const InT*)g.B + (g.b_kmajor ? (int64_t)o.b_col * g.ldb : (int64_t)o.b_col);
    s.a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, clamp_u32(((int64_t)(o.a_rows - 1 - o.a_row) * g.lda + g.K) * kEsz), 0x00020000);
    const int64_t b_elems = g.b_kmajor ? (int64_t)(o.b_cols - 1 - o.b_col) * g.ldb + g.K : (int64_t)(g.K - 1) * g.ldb + (o.b_cols - o.b_col);
    s.b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, clamp_u32(b_elems * kEsz), 0x00020000);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s.off_a[i] = (uint32_t)(((tid >> 3) + 32 * i) * g.lda * kEsz + (tid & 7) * 16);
      s.off_b[i] = g.b_kmajor ? (uint32_t)(((tid >> 3) + 32 * i) * g.ldb * kEsz + (tid & 7) * 16)
                              : (uint32_t)(((tid >> 4) * 4 + i) * g.ldb * kEsz + (tid & 15) * 16);
    }
    s.step_a = kBK * kEsz;
    s.step_b = g.b_kmajor ? (uint32_t)(kBK * kEsz) : (uint32_t)(kBK * g.ldb * kEsz);
    return s;
  }

  // `tail`: this K step reaches past K, so A chunks at k >= K must read as zero too
  // (B rows >= K already do, being past the end of the buffer).
  TCCL_D void load_global(const Source& s, int kt, bool tail, u32x4 (&ra)[4], u32x4 (&rb)[4]) const {
    const uint32_t adv_a = kt * s.step_a, adv_b = kt * s.step_b;
    const bool dead = tail && (kt * kBK + (tid & 7) * 8 >= g.K);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t off = dead ? 0xfffffff0u : s.off_a[i] + adv_a;
      ra[i] = __builtin_amdgcn_raw_buffer_load_b128(s.a, off, 0, 0);
    }
    const bool dead_b = dead && g.b_kmajor;  // row-major B: rows >= K lie past the end of the buffer
#pragma unroll
    for (int i = 0; i < 4; ++i) rb[i] = __builtin_amdgcn_raw_buffer_load_b128(s.b, dead_b ? 0xfffffff0u : s.off_b[i] + adv_b, 0, 0);
  }

  // ---- registers -> LDS ---------------------------------------------------------------
  TCCL_D void store_lds(const u32x4 (&ra)[4], const u32x4 (&rb)[4]) const {
    char* la = lds + (tid & 7) * kPlane;
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4*)(la + ((tid >> 3) + 32 * i) * 16) = ra[i];

    if (g.b_kmajor) {  // rb[i]: the 8 consecutive k of column (tid >> 3) + 32 * i, as the reads want them
      char* lb = lds + kOperandBytes + (tid & 7) * kPlane;
#pragma unroll
      for (int i = 0; i < 4; ++i) *(u32x4*)(lb + b_slot((tid >> 3) + 32 * i) * 16) = rb[i];
      return;
    }
    // rb[i] holds columns n0..n0+7 of k row i as 4 dwords (two columns each).  Column
    // n0+j needs its four k values side by side: two dwords (k0|k1) and (k2|k3).
    const int kg = tid >> 4;
    char* lb = lds + kOperandBytes + (kg >> 1) * kPlane + (kg & 1) * 8;
    const int n0 = (tid & 15) * 8;
    const u32x4 r0 = rb[0], r1 = rb[1], r2 = rb[2], r3 = rb[3];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint2 even, odd;
      even.x = (r0[d] & 0xffffu) | (r1[d] << 16);
      even.y = (r2[d] & 0xffffu) | (r3[d] << 16);
      odd.x = (r0[d] >> 16) | (r1[d] & 0xffff0000u);
      odd.y = (r2[d] >> 16) | (r3[d] & 0xffff0000u);
      *(uint2*)(lb + b_slot(n0 + 2 * d) * 16) = even;
      *(uint2*)(lb + b_slot(n0 + 2 * d + 1) * 16) = odd;
    }
  }

  // ---- LDS -> MFMA, one K step -----------------------------------------------------------
  TCCL_D void compute(f32x16 (&acc)[2][2]) const {
    const int half = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      const char* pa = lds + (2 * kk + half) * kPlane;
      const char* pb = lds + kOperandBytes + (2 * kk + half) * kPlane;
      Vec fa[2], fb[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        fa[b] = *(const Vec*)(pa + (wm * 64 + b * 32 + l32) * 16);
        fb[b] = *(const Vec*)(pb + b_slot(wn * 64 + b * 32 + l32) * 16);
      }
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) acc[bi][bj] = Mfma<InT>::run(fb[bj], fa[bi], acc[bi][bj]);
    }
  }

  // ---- accumulators -> LDS -> global -------------------------------------------------------
  // Each wave stages its own 32-row slab (one bi at a time) in a private LDS window, then
  // writes it out with 16-byte stores that are contiguous along the row.
  template <int kPolicy>
  TCCL_D void epilogue(int row0, int col0, const f32x16 (&acc)[2][2]) const {
    constexpr int kEsz = sizeof(OutT);
    constexpr int kRowBytes = 64 * kEsz;       // one wave row: 64 columns
    constexpr int kChunks = kRowBytes / 16;    // 16-byte chunks per row (8 or 16)
    constexpr int kPerChunk = 16 / kEsz;       // elements per chunk
    char* win = lds + wave * (32 * 64 * 4);    // 8 KiB window per wave (fp32 worst case)
    // The lane id is taken afresh: what the epilogue derives from it is invariant across tiles
    // and would otherwise be hoisted out of the tile loop and held in registers through the K loop.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int half = ln >> 5, l32 = ln & 31;
    // Stores go through a buffer resource rooted at the sub-tile so that the cache policy
    // can be chosen: plain write-back when nobody waits for the tile, device-coherent
    // write-through when a communication workgroup will read it right after the signal.
    OutT* C = (OutT*)g.C + (int64_t)row0 * g.ldc + col0;
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void*)C, 0, 0xffffffffu, 0x00020000);

#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
      __syncthreads();  // window free: K loop reads / previous slab's reads are done
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n_local = bj * 32 + 8 * q + 4 * half;  // first of 4 consecutive columns
          OutT v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = to_out<OutT>(acc[bi][bj][4 * q + e] * g.alpha);
          const int byte = n_local * kEsz;
          const int chunk = (byte >> 4) ^ (l32 & 7);
          char* p = win + l32 * kRowBytes + chunk * 16 + (byte & 15);
          if constexpr (kEsz == 2) {
            uint2 u;
            __builtin_memcpy(&u, v, 8);
            *(uint2*)p = u;
          } else {
            uint4 u;
            __builtin_memcpy(&u, v, 16);
            *(uint4*)p = u;
          }
        }
      __syncthreads();
#pragma unroll
      for (int r = 0; r < (32 * kChunks) / 64; ++r) {
        const int idx = ln + 64 * r;
        const int row = idx / kChunks, chunk = idx % kChunks;
        const u32x4 v = *(const u32x4*)(win + row * kRowBytes + ((chunk ^ (row & 7)) * 16));
        const int lrow = wm * 64 + bi * 32 + row, lcol = wn * 64 + chunk * kPerChunk;
        if (row0 + lrow < g.M && col0 + lcol < g.N)
          __builtin_amdgcn_raw_buffer_store_b128(v, rc, (uint32_t)((lrow * g.ldc + lcol) * kEsz), 0, kPolicy);
      }
    }
  }

  // ---- one 128 x 128 sub-tile -------------------------------------------------------------------
  template <int kPolicy>
  TCCL_D void subtile(int row0, int col0) const {
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    u32x4 ra[4], rb[4];
    const Source src = make_source(row0, col0);
    const int ksteps = (g.K + kBK - 1) / kBK;
    const bool ragged = (g.K % kBK) != 0;
    load_global(src, 0, ragged && ksteps == 1, ra, rb);
    for (int kt = 0; kt < ksteps; ++kt) {
      __syncthreads();  // everyone is done reading the previous contents of LDS
      store_lds(ra, rb);
      __syncthreads();
      if (kt + 1 < ksteps) load_global(src, kt + 1, ragged && kt + 2 == ksteps, ra, rb);
      compute(acc);
    }
    epilogue<kPolicy>(row0, col0, acc);
  }

  // ---- persistent loop over plan tiles ----------------------------------------------------------
  TCCL_D void run(const SignalArgs& s, int wg, int num_wgs) const {
    const int total = g.tile_rows * g.tile_cols;
    for (int slot = wg; slot < total; slot += num_wgs) {
      const int tile_id = tile_for_slot(slot, total, g.xcds, g.span);
      const TileCoord tc = tile_coords(tile_id, g.tile_rows, g.tile_cols, g.group_m);
      for (int sm = 0; sm < g.block_m; sm += kTile)
        for (int sn = 0; sn < g.block_n; sn += kTile) {
          const int row0 = tc.m * g.block_m + sm, col0 = tc.n * g.block_n + sn;
          if (row0 >= g.M || col0 >= g.N) continue;
          if (s.mode == kSignalNone)
            subtile<0>(row0, col0);
          else
            subtile<kCoherent>(row0, col0);
        }
      if (s.mode != kSignalNone) {
        // The tile was stored write-through; once every wave's stores have completed the
        // data is visible device-wide and one lane may publish the signal.
        wait_vmem();
        __syncthreads();
        if (tid == 0) {
          if (s.mode == kSignalTile)
            tile_publish(s.locks, tile_id, s.epoch);
          else
            tile_signal_add<true>(s.counter, s.group_table[tile_id], 1);
        }
      }
    }
  }
};

}  // namespace tccl
