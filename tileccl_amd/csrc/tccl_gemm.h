// Persistent MFMA GEMM role for gfx950 (CDNA4), 16-bit inputs, 128 x 128 tiles.
//
// One workgroup = 256 threads = 4 wavefronts (2 x 2, wave tile 64 x 64), producing 128 x 128
// output sub-tiles with K consumed 32 at a time through three (or five) LDS stages of 16 KiB.  A plan tile
// (block_m x block_n, multiples of 128) is a small loop of such sub-tiles; when the whole plan
// tile is in memory the workgroup publishes it (per-tile lock or per-TileGroup counter).
// 48 KiB of LDS and <= 168 registers per lane let three workgroups share a CU (two that multiply
// and one that moves data, in the fused launches), each with one wavefront per SIMD and barriers
// of its own, so that one workgroup's waits are covered by the others' MFMAs.  The GEMM alone runs
// a five-stage form (80 KiB, two workgroups per CU).
//
// Data path of one K step
//   global --buffer_load_dwordx4 ... lds--> LDS stage --ds_read--> operands of v_mfma_f32_16x16x32
//   A stage: 128 rows x 64 B (32 k); 16-byte chunk kc of row r sits in slot kc ^ ((r >> 1) & 3).  (Measured
//            with the LDS saturated by eight wavefronts: a ds_read_b128 of rows l % 16, chunk l / 16 takes
//            1.78 times as long with ((r >> 2) & 3) or with no swizzle at all, and no longer than a
//            conflict-free read with this term.)
//   B stage: 32 k rows x 256 B (128 columns); chunk c of row k in slot c ^ 4 (k & 3) ^ 2 ((k >> 3) & 1);
//            operands come out through ds_read_b64_tr_b16 (the transposing read: within 16 lanes,
//            lane i supplies 4 columns of k row i / 4, lane j receives 4 k of column j), two per operand.
//   The hardware writes lane l's 16 bytes at base + 16 l, so the swizzles are applied on the global
//   side, by the choice of the chunk a lane fetches.  Rows >= M, columns >= N and k >= K read as
//   zero through the buffer bounds (A chunks at k >= K are redirected past the buffer's end).
//   A k-major B (GemmArgs::b_kmajor: element (k, n) at B[n * ldb + k]) takes A's route and layout.
//
// Pipeline (S stages: 3 in the fused launches, 5 in the GEMM-only kernel): step t computes from stage
// t % S and issues the loads of K step t + S - 1 into stage (t - 1) % S, which every wavefront finished
// reading before the barrier of step t - 1; one load per item, four items per step (one 16-row block of A
// against the four 16-column blocks of B).  The step's one barrier sits before its last item and waits
// with vmcnt(4 (S - 2) - 1): the loads of the last S - 2 steps may stay in flight, those of K step t + 1
// have landed.  Behind it the last item already fetches the next step's first operands, and reloads each
// B operand in place once its MFMA is issued.
// What bounds the tile shape: per K step a CU's address unit takes in 16 KiB (256 clocks at 64 B/clk) and
// its LDS 16 KiB of writes and 32 KiB of reads, against 256 clocks of MFMAs: all three are level, where
// the 256 x 256 tile has half the traffic per FLOP.  Measured at 4096 x 4096 x 1024: 41 us as it is,
// 29 us without the global loads, 36 us without the LDS reads, 24 us with neither (and no barrier).
//
// MFMA orientation: the B operand is passed first, i.e. the instruction computes the transposed
// 16 x 16 block.  Each lane then owns 4 consecutive output columns of one output row, and the
// register -> LDS -> global epilogue moves 8 / 16 bytes per access.
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

constexpr int kTile = 128;                        // sub-tile edge
constexpr int kBK = 32;                           // K per step
constexpr int kThreads = 256;                     // threads per workgroup
constexpr int kARow128 = kBK * 2;                 // bytes of an A row in a stage
constexpr int kAStage128 = kTile * kARow128;      // 8 192
constexpr int kBPitch128 = kTile * 2;             // bytes of a k row of B in a stage
constexpr int kBStage128 = kBK * kBPitch128;      // 8 192 (k-major B: 128 rows of 64 B, the same)
constexpr int kStage128 = kAStage128 + kBStage128;  // A then B: 16 384; three such stages per workgroup

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

// all-scatter / all-gather folded into the GEMM: the tile goes out from the staging LDS it
// already sits in, instead of being written, signalled, re-read and copied by a second party
// (reference: the per-tile scatter of patterns/_helpers.py:86-199, tile_allgather of
// primitives/collectives.py:613-663).
struct PushArgs {
  int world;           // ranks; every rank but `rank` is a target.  0: the epilogue writes C only
  int rank;
  int col_lo, col_hi;  // columns of C that travel
  int col_shift;       // target column = C column + col_shift
  int64_t ld;          // target pitch in elements
  const int64_t* heap_bases;  // C's address inside target q is C + heap_bases[q] - heap_bases[rank]
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

#if defined(__HIP_DEVICE_COMPILE__)
template <typename InT, typename OutT, int kStages = 3>
struct GemmRole {
  static_assert(kStages == 3 || kStages == 5, "three stages (48 KiB: three workgroups per CU) or five (80 KiB: two)");
  typedef typename Mfma<InT>::Vec Vec;
  static_assert(sizeof(InT) == 2, "16-bit inputs");
  typedef __attribute__((address_space(3))) void LdsVoid;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 LdsQuad;

  const GemmArgs& g;
  const PushArgs& push;  // world == 0: nothing leaves from the epilogue
  char* st0;
  char* st1;
  char* st2;
  char* st3;  // (five-stage form only)
  char* st4;
  const int tid, lane, wave, wm, wn;

  // The wavefront's number lives in a scalar register: the LDS addresses its loads land at derive from it.
  TCCL_D GemmRole(const GemmArgs& args, const PushArgs& push_args, char* s0, char* s1, char* s2, char* s3 = nullptr,
                  char* s4 = nullptr)
      : g(args), push(push_args), st0(s0), st1(s1), st2(s2), st3(s3), st4(s4), tid(threadIdx.x), lane(threadIdx.x & 63),
        wave(__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))), wm(wave >> 1), wn(wave & 1) {}

  static TCCL_D int fresh(int v) {
    asm volatile("" : "+v"(v));
    return v;
  }
  static TCCL_D uint32_t clamp_u32(int64_t v) { return v > 0xffffffffll ? 0xffffffffu : (v < 0 ? 0u : (uint32_t)v); }

  // ---- global -> LDS ------------------------------------------------------------------------
  // Per K step a wavefront fetches two 1 KiB pieces of each operand:
  //   A piece i: rows 16 (2 wave + i) .. + 15      (lane l: row + l / 4, slot l % 4)
  //   B piece j: k rows 4 (2 wave + j) .. + 3      (lane l: k row + l / 16, slot l % 16)
  //   k-major B piece j: columns 16 (2 wave + j) .. + 15, as A.
  struct Source {
    __amdgpu_buffer_rsrc_t a, b;
    uint32_t off_a[2], off_b[2];  // byte offsets of this lane's 16-byte loads, K step 0
    uint32_t step_a, step_b;      // byte advance per K step
    int k_lane;                   // first k of this lane's chunk of an A row (of a k-major B row) within a step
  };

  template <bool kBKMajor>
  TCCL_D Source make_source(int row0, int col0) const {
    Source s;
    const int ln = fresh(lane);
    const OperandOrigin o = operand_origin(g, row0, col0);
    const InT* A = (const InT*)g.A + (int64_t)o.a_row * g.lda;
    const InT* B = (const InT*)g.B + (kBKMajor ? (int64_t)o.b_col * g.ldb : (int64_t)o.b_col);
    s.a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, clamp_u32(((int64_t)(o.a_rows - 1 - o.a_row) * g.lda + g.K) * 2), 0x00020000);
    const int64_t b_elems = kBKMajor ? (int64_t)(o.b_cols - 1 - o.b_col) * g.ldb + g.K : (int64_t)(g.K - 1) * g.ldb + (o.b_cols - o.b_col);
    s.b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, clamp_u32(b_elems * 2), 0x00020000);
    // Bits 1 and 2 of a row's number come from the lane alone (a piece starts on a multiple of 16).
    const int kc = (ln & 3) ^ ((ln >> 3) & 3);
    s.k_lane = kc * 8;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 16 * (2 * wave + i) + (ln >> 2);
      s.off_a[i] = (uint32_t)(row * g.lda * 2 + kc * 16);
      if constexpr (kBKMajor) {
        s.off_b[i] = (uint32_t)(row * g.ldb * 2 + kc * 16);
      } else {
        const int k = 4 * (2 * wave + i) + (ln >> 4);
        const int c = (ln & 15) ^ (4 * (k & 3)) ^ (2 * ((k >> 3) & 1));
        s.off_b[i] = (uint32_t)(k * g.ldb * 2 + c * 16);
      }
    }
    s.step_a = kBK * 2;
    s.step_b = kBKMajor ? (uint32_t)(kBK * 2) : (uint32_t)(kBK * g.ldb * 2);
    return s;
  }

  // Piece i of K step kt, straight into `stage`.
  TCCL_D void issue_a(char* stage, const Source& s, int kt, int i) const {
    const bool dead = kt * kBK + s.k_lane >= g.K;
    const uint32_t oa = dead ? 0xfffffff0u : s.off_a[i] + kt * s.step_a;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(s.a, (LdsVoid*)(stage + (2 * wave + i) * 1024), 16, oa, 0, 0, 0);
  }
  template <bool kBKMajor>
  TCCL_D void issue_b(char* stage, const Source& s, int kt, int i) const {
    uint32_t ob = s.off_b[i] + kt * s.step_b;  // row-major B: rows >= K lie past the end of the buffer
    if constexpr (kBKMajor) ob = (kt * kBK + s.k_lane >= g.K) ? 0xfffffff0u : ob;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(s.b, (LdsVoid*)(stage + kAStage128 + (2 * wave + i) * 1024), 16, ob, 0, 0, 0);
  }
  template <bool kBKMajor>
  TCCL_D void issue_piece(char* stage, const Source& s, int kt, int i) const {
    issue_a(stage, s, kt, i);
    issue_b<kBKMajor>(stage, s, kt, i);
  }

  // ---- LDS -> MFMA operands -------------------------------------------------------------------
  // 16 x 16 x 32 operands: lane l holds the 8 consecutive k of group l / 16 for row (column) l % 16.
  struct Reader {
    uint32_t a_base;   // this lane's row of A row block 0, slot applied
    uint32_t b_base0;  // this lane's address for column block 0
  };
  template <bool kBKMajor>
  TCCL_D Reader make_reader() const {
    const int i16 = lane & 15, kg = lane >> 4;
    Reader r;
    r.a_base = (uint32_t)((wm * 64 + i16) * kARow128 + ((kg ^ ((i16 >> 1) & 3)) << 4));
    if constexpr (kBKMajor) {
      r.b_base0 = (uint32_t)(kAStage128 + (wn * 64 + i16) * kARow128 + ((kg ^ ((i16 >> 1) & 3)) << 4));
    } else {
      // Lane group kg covers k rows 8 kg .. + 7 in two transposing reads (k + 0, k + 4).
      const int t = i16 >> 2, cq = i16 & 3;
      const int chunk = (wn * 8 + (cq >> 1)) ^ (4 * t) ^ (2 * (kg & 1));
      r.b_base0 = (uint32_t)(kAStage128 + (8 * kg + t) * kBPitch128 + chunk * 16 + (cq & 1) * 8);
    }
    return r;
  }
  TCCL_D Vec load_a(const char* stage, const Reader& r, int rb) const { return *(const Vec*)(stage + r.a_base + rb * 16 * kARow128); }
  template <bool kBKMajor>
  TCCL_D Vec load_b(const char* stage, const Reader& r, int cb) const {
    if constexpr (kBKMajor) return *(const Vec*)(stage + r.b_base0 + cb * 16 * kARow128);
    // column block cb: two chunks further on (the XOR commutes with the swizzle terms)
    const char* pb = stage + (r.b_base0 ^ (uint32_t)(32 * cb));
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsQuad*)pb);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsQuad*)(pb + 4 * kBPitch128));
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(Vec, both);
  }

  struct Frags {
    Vec fa[4], fb[4];
  };

  // One K step: four items (A row block rb against the four B column blocks).  On entry fa[0], fa[1] and
  // fb[0..3] hold this step's operands; items 0 and 1 fetch fa[2] and fa[3]; the last item, behind the
  // barrier, fetches the next step's fa[0], fa[1] from `nxt` and reloads each fb in place.  The four loads of
  // K step kt_load into `far` (the stage read during the step before) go out one per item: a wavefront issues
  // nothing else while the address unit accepts its load, and the four wavefronts reach an item together.
  // The fourth goes out behind the barrier, so at the barrier the loads that may still be in flight are
  // those of the kStages - 2 steps before, less that one.
  static constexpr int kInFlight = 4 * (kStages - 2) - 1;
  template <bool kBKMajor>
  TCCL_D void k_step(const char* cur, const char* nxt, char* far, const Source& src, const Reader& rd, int kt_load,
                     f32x4 (&acc)[4][4], Frags& f) const {
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      if (rb == 3) {
        // The loads of K step t + 1 (into `nxt`) have landed; this wavefront's reads of `cur` are done.
        // The barrier is the bare instruction (__syncthreads() carries a release fence); the empty asm
        // keeps LDS accesses from moving across it.
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kInFlight) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        f.fa[0] = load_a(nxt, rd, 0);
        f.fa[1] = load_a(nxt, rd, 1);
      } else if (rb < 2) {
        f.fa[rb + 2] = load_a(cur, rd, rb + 2);
      }
      if (rb & 1)
        issue_b<kBKMajor>(far, src, kt_load, rb >> 1);
      else
        issue_a(far, src, kt_load, rb >> 1);
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        acc[rb][cb] = Mfma<InT>::run16(f.fb[cb], f.fa[rb], acc[rb][cb]);
        if (rb == 3) {
          __builtin_amdgcn_sched_barrier(0);
          f.fb[cb] = load_b<kBKMajor>(nxt, rd, cb);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- accumulators -> LDS -> global -------------------------------------------------------
  // Block (rb, cb) of the wave tile: the lane holds row 16 rb + l % 16, columns 16 cb + 4 (l / 16) .. + 3.
  // Each wavefront stages a 32-row slab (two row blocks) in its own 8 KiB window and writes it out
  // with 16-byte stores that are contiguous along the row; a wavefront's LDS operations execute in
  // the order issued, so nothing inside the loop waits for another wavefront.
  template <int kPolicy>
  TCCL_D void epilogue(int row0, int col0, const f32x4 (&acc)[4][4]) const {
    constexpr int kEsz = sizeof(OutT);
    constexpr int kRowBytes = 64 * kEsz;       // one wave row: 64 columns
    constexpr int kChunks = kRowBytes / 16;    // 16-byte chunks per row (8 or 16)
    constexpr int kPerChunk = 16 / kEsz;       // elements per chunk
    char* win = (wave < 2 ? st0 : st1) + (wave & 1) * 8192;  // 8 KiB per wavefront (fp32 worst case)
    // The lane id is taken afresh: what the epilogue derives from it is invariant across tiles
    // and would otherwise be hoisted out of the tile loop and held in registers through the K loop.
    const int ln = fresh(lane);
    const int i16 = ln & 15, kg = ln >> 4;
    // Stores go through a buffer resource rooted at the sub-tile so that the cache policy
    // can be chosen: plain write-back when nobody waits for the tile, device-coherent
    // write-through when a communication workgroup will read it right after the signal.
    OutT* C = (OutT*)g.C + (int64_t)row0 * g.ldc + col0;
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void*)C, 0, 0xffffffffu, 0x00020000);
    __syncthreads();  // every wavefront has left the K loop's stages
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
          const int row = 16 * r + i16;
          OutT v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = to_out<OutT>(acc[2 * bi + r][cb][e] * g.alpha);
          const int byte = (16 * cb + 4 * kg) * kEsz;
          const int chunk = (byte >> 4) ^ (row & 7);
          char* p = win + row * kRowBytes + chunk * 16 + (byte & 15);
          if constexpr (kEsz == 2) {
            uint2 u;
            __builtin_memcpy(&u, v, 8);
            *(uint2*)p = u;
          } else {
            u32x4 u;
            __builtin_memcpy(&u, v, 16);
            *(u32x4*)p = u;
          }
        }
      asm volatile("" ::: "memory");  // staged by this wavefront itself: LDS keeps the order
      constexpr int kRounds = (32 * kChunks) / 64;
      u32x4 v[kRounds];
      int lrow[kRounds], lcol[kRounds];
      bool live[kRounds];
#pragma unroll
      for (int r = 0; r < kRounds; ++r) {
        const int idx = ln + 64 * r;
        const int row = idx / kChunks, chunk = idx % kChunks;
        v[r] = *(const u32x4*)(win + row * kRowBytes + ((chunk ^ (row & 7)) * 16));
        lrow[r] = wm * 64 + bi * 32 + row;
        lcol[r] = wn * 64 + chunk * kPerChunk;
        live[r] = row0 + lrow[r] < g.M && col0 + lcol[r] < g.N;
        if (live[r]) __builtin_amdgcn_raw_buffer_store_b128(v[r], rc, (uint32_t)((lrow[r] * g.ldc + lcol[r]) * kEsz), 0, kPolicy);
      }
      // Fused push: the same chunks go to every peer's slice from the registers they sit in; the tile is
      // never read back.  The signal that follows the tile's last store covers these stores as well.
      for (int t = 0; t < push.world; ++t) {
        if (t == push.rank) continue;
        const int64_t push_ld = push.ld;
        const int col_lo = push.col_lo, col_hi = push.col_hi;
        typedef const __attribute__((address_space(4))) int64_t* Bases;
        const int64_t delta = ((Bases)push.heap_bases)[t] - ((Bases)push.heap_bases)[push.rank];
        char* base = (char*)g.C + delta + ((int64_t)row0 * push_ld + col0 + push.col_shift) * kEsz;
        const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xffffffffu, 0x00020000);
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
          const int col = col0 + lcol[r];
          if (live[r] && col >= col_lo && col < col_hi)
            __builtin_amdgcn_raw_buffer_store_b128(v[r], rt, (uint32_t)((lrow[r] * push_ld + lcol[r]) * kEsz), 0, kCoherent);
        }
      }
      asm volatile("" ::: "memory");
    }
  }

  // ---- one 128 x 128 sub-tile -------------------------------------------------------------------
  template <int kPolicy, bool kBKMajor>
  TCCL_D void subtile(int row0, int col0) const {
    f32x4 acc[4][4];  // cleared two registers per instruction
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
        f64x2 z;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          double d;
          asm volatile("v_mov_b64 %0, 0" : "=v"(d));
          z[e] = d;
        }
        acc[i][j] = __builtin_bit_cast(f32x4, z);
      }

    const Source src = make_source<kBKMajor>(row0, col0);
    const Reader rd = make_reader<kBKMajor>();
    const int ksteps = (g.K + kBK - 1) / kBK;
    __syncthreads();  // the previous sub-tile's epilogue has left LDS
    // K steps 0 .. kStages - 2 go out up front (past K: zeros, never consumed); the order within a step is
    // the one k_step() issues in (A 0, B 0, A 1, B 1).
    issue_piece<kBKMajor>(st0, src, 0, 0);
    issue_piece<kBKMajor>(st0, src, 0, 1);
    issue_piece<kBKMajor>(st1, src, 1, 0);
    issue_piece<kBKMajor>(st1, src, 1, 1);
    if constexpr (kStages == 5) {
      issue_piece<kBKMajor>(st2, src, 2, 0);
      issue_piece<kBKMajor>(st2, src, 2, 1);
      issue_piece<kBKMajor>(st3, src, 3, 0);
      issue_piece<kBKMajor>(st3, src, 3, 1);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * (kStages - 2)) : "memory");  // stage 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    Frags f;
    f.fa[0] = load_a(st0, rd, 0);
    f.fa[1] = load_a(st0, rd, 1);
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) f.fb[cb] = load_b<kBKMajor>(st0, rd, cb);
    // Step t computes from stage t % kStages, fetches its last operands from the next one and loads K step
    // t + kStages - 1 into the one before.  Stages are named statically (the compiler tracks loads into LDS
    // per array), so the loop comes in rounds of kStages steps with an exit after every step.
    if constexpr (kStages == 3) {
      for (int kt = 0;; kt += 3) {
        k_step<kBKMajor>(st0, st1, st2, src, rd, kt + 2, acc, f);
        if (kt + 1 >= ksteps) break;
        k_step<kBKMajor>(st1, st2, st0, src, rd, kt + 3, acc, f);
        if (kt + 2 >= ksteps) break;
        k_step<kBKMajor>(st2, st0, st1, src, rd, kt + 4, acc, f);
        if (kt + 3 >= ksteps) break;
      }
    } else {
      for (int kt = 0;; kt += 5) {
        k_step<kBKMajor>(st0, st1, st4, src, rd, kt + 4, acc, f);
        if (kt + 1 >= ksteps) break;
        k_step<kBKMajor>(st1, st2, st0, src, rd, kt + 5, acc, f);
        if (kt + 2 >= ksteps) break;
        k_step<kBKMajor>(st2, st3, st1, src, rd, kt + 6, acc, f);
        if (kt + 3 >= ksteps) break;
        k_step<kBKMajor>(st3, st4, st2, src, rd, kt + 7, acc, f);
        if (kt + 4 >= ksteps) break;
        k_step<kBKMajor>(st4, st0, st3, src, rd, kt + 8, acc, f);
        if (kt + 5 >= ksteps) break;
      }
    }
    wait_vmem();  // the look-ahead loads must not land on the epilogue's staging
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
          if (s.mode == kSignalNone) {
            if (g.b_kmajor)
              subtile<0, true>(row0, col0);
            else
              subtile<0, false>(row0, col0);
          } else {
            if (g.b_kmajor)
              subtile<kCoherent, true>(row0, col0);
            else
              subtile<kCoherent, false>(row0, col0);
          }
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
#endif  // __HIP_DEVICE_COMPILE__

}  // namespace tccl
