// Large-tile MFMA GEMM for gfx950: one workgroup of 512 threads (8 wavefronts, 2 x 4)
// produces a 256 x 256 macro tile, K consumed 64 at a time.
//
// Why a second GEMM: measured on MI355X, a CU's LDS takes ~78 B/clk of writes and 256 B/clk
// of reads.  A 128 x 128 tile needs 32 KB of operands written per 512 MFMA cycles (64 B/clk,
// most of what the LDS accepts); at 256 x 256 the same bytes feed four times the math.  A
// wave owns 128 x 64 outputs (128 fp32 accumulators per lane), which also cuts the LDS
// reads per MFMA.
//
// Global -> LDS: `buffer_load_dwordx4 ... lds` copies 16 bytes per lane straight into LDS (no
// staging registers, no ds_write).  The hardware places lane l's bytes at base + 16*l, so the
// LDS layout is fixed to "lanes in order" and the swizzle that keeps the MFMA reads free of
// bank conflicts is applied on the global side, by choosing which 16-byte chunk a lane
// fetches:
//   A stage: row-major, 128 B per row (64 k of a 16-bit type, 128 k of fp8); chunk kc of row r
//            lives in slot kc ^ ((r >> 1) & 7).
//   B stage: natural [k][n]; 16-bit: 512 B per k row, chunk c of row k in slot
//            c ^ (4 * (k & 3)) ^ (2 * ((k >> 3) & 1)); fp8: 256 B per k row, chunk c of row k in slot
//            c ^ (2 * (k & 7)) ^ ((k >> 4) & 1).
// fp8: the 32 k that lane group kg (lane / 16) holds of a 128-k step are k 16 kg .. 16 kg + 15 and
// 64 + 16 kg .. 64 + 16 kg + 15, for A and B alike (a sum over k does not care about the order).  A ds_read_b128
// serves lanes of all four groups in one pass: the groups' chunks kg and kg + 4 fall on different banks,
// the chunks 2 kg and 2 kg + 1 of 32 consecutive k per group did not (every read took twice as long).
// A operands are read with ds_read_b128.  B operands are read with the transposing LDS reads
// of gfx950 (semantics measured on the device, 16 lanes at a time):
//   ds_read_b64_tr_b16: lane i supplies 4 consecutive n of k row i/4 at column block i%4; lane j
//                       receives 4 consecutive k of column j (two reads = the 8 k a lane holds of
//                       a 16x16x32 operand);
//   ds_read_b64_tr_b8:  lane i supplies 8 consecutive n of k row i/2 at column block i%2; lane j
//                       receives 8 consecutive k of column j (four reads = the 32 k a lane holds of a
//                       16x16x128 operand).
//
// MFMA shape.  16-bit inputs use v_mfma_f32_16x16x32, not 32x32x16: with operands held in registers
// and nothing else running, the matrix pipes of the whole part sustain 1.49 PFLOP/s of 32x32x16 on
// N(0,1) fp16 data (2.3 PFLOP/s on zeros: the rate depends on the data, i.e. on power), 1.86 PFLOP/s of
// 16x16x32.  The K loop of this kernel ran at the 32x32x16 figure; on 16x16x32 the GEMM alone is 7-11 %
// faster.  fp8 inputs use v_mfma_scale_f32_16x16x128_f8f6f4 for the same reason (3.5 against 4.0 PFLOP/s
// sustained on N(0,1) e4m3 values; the fp8 GEMM, further from that bound, gained 2 %).
//
// Pipeline: LDS holds two stages.  The loads of step kt+1 are issued, woven between the
// first MFMAs of step kt, into the stage step kt-1 has left.  The step's one barrier
// (`s_waitcnt vmcnt(0) lgkmcnt(0)` + `s_barrier`) sits two items before the step's end: the
// stage being read is finished with, the next one has landed, and the last items already fetch
// the next step's first operands (see k_step16 / k_step8).
//
// The swapped-operand MFMA and the slab-wise epilogue are those of tccl_gemm.h.
//
// A macro tile covers (256/block_m) x (256/block_n) plan tiles; when it is stored, each of
// them is published under its swizzled tile id, so locks / group_table keep the
// reference's numbering (tileccl/kernels/gemm.py:118-123, tileccl_v2/tile_group.py:229-234).
#pragma once

#include "tccl_comm.h"
#include "tccl_gemm.h"

namespace tccl {

// OCP fp8 e4m3 ("e4m3fn"), the 8-bit input type of gfx950's v_mfma_f32_32x32x64_f8f6f4.
struct fp8e4m3 {
  uint8_t bits;
};
typedef int i32x8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
template <>
struct Mfma<fp8e4m3> {
  typedef i32x8 Vec;  // 32 consecutive k of one row / column
  // cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands select the unscaled form.
  static TCCL_D f32x16 run(Vec a, Vec b, f32x16 c) { return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0); }
  // 16 x 16 x 128: lane l holds 32 consecutive k (group l / 16) of row / column l % 16 and gets
  // D[4 * (l / 16) + e][l % 16], e = 0..3.
  static TCCL_D f32x4 run16(Vec a, Vec b, f32x4 c) { return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0); }
};
#endif

constexpr int kMacro = 256;
constexpr int kThreads256 = 512;
constexpr int kARow256 = 128;                              // A: bytes per row of one stage (64 k)
constexpr int kAStage256 = kMacro * kARow256;              // 32 768 B
constexpr int kBStage256 = 32768;                          // B: (128 / element size) k rows of 256 columns
constexpr int kStage256 = kAStage256 + kBStage256;         // A then B
constexpr int kLds256 = 2 * kStage256;                     // two stages: 131 072 B (two arrays)

struct Macro {
  int rows, cols;        // macro tile grid
  int rows_per_band;     // macro rows that form one swizzle band of the plan
  int xcds, span;        // slot -> macro id remap
  int row_shift;         // macro rows are visited starting at this one (wrapping around)
};

// Where the epilogue sends a finished tile besides C: the same rows of every listed target,
// columns [col_lo, col_hi) of C landing at column + col_shift.  This is the push half of an
// Reduce-scatter carried out tile by tile.  Once a macro tile's partial is stored and
// published, the workgroup waits for the other ranks' partials of the same tile, streams the
// tile back, adds in fp32 -- the owner's addend
// first, then ascending ranks; one rounding: tile_reduce_scatter, primitives/collectives.py:766-781
// -- and writes the owner's output shard.  The accumulators are dead by then, so the stream
// runs with many loads in flight.  Tiles are visited starting with the rows the other ranks
// own; a rank's own rows come last, and only tiles of own rows wait on a peer (reducing on a
// peer's behalf happens in single-GPU emulation, against resident partials).  A rank therefore
// only ever waits for tiles its peers produce early and without waiting: no cycle.
struct ReduceArgs {
  int active;
  int rank, world, emulate_peer;
  int peers_resident;             // the peers' partials are complete in memory: never wait for their words
  int shard_rows;                 // rows per owner; a multiple of the 256-row tile
  int out_bf16;                   // output element: 0 fp16, 1 bf16
  int own_in_registers;           // own rows: sum the peers' partials onto the accumulators, store no partial
  const int64_t* heap_bases;
  const char* out;                // the output shard in this rank's slice (the partial is the GEMM's C)
  int64_t ld_out;                 // output pitch in elements
  const int32_t* locks;           // this rank's words; a peer's sit at the same slice offset
  const int32_t* counter;
  const int32_t* tile_counts;
  int epoch;
  int64_t* fault;
  int64_t spin_ticks;
};

// Background transfer: the pull half of an all-gather, carried out in the shadow of the K
// loop (TileGroup variant): out[block of peer] <- the peer's copy of that block.
// A peer's block is cut into pieces of kPieceUnits units of 16 bytes; pulling wavefront w of
// the launch (the kPullWaves older wavefronts of every workgroup, see below) owns pieces w,
// w + W, w + 2W, ... (W = pulling wavefronts in the grid), so at any moment the grid sweeps a
// contiguous stretch.  In every K step, behind the step's operand loads, such a wavefront
// requests its next piece into registers; the step's barrier waits for this wave's loads
// anyway, and mid-way through the following step the piece is stored.  A
// piece is fetched only once
// the TileGroups covering its rows are complete on the peer (counter[g] >= epoch *
// tile_counts[g], the readiness rule of tileccl_v2/signal.py:43-66); that is found out by
// counter fetches which are themselves left in flight for one K step.  What the K loops did
// not get to is finished after the last tile, with bounded waits.  Groups must cover the rows
// in ascending order (build_tile_group_plan emits them so: tileccl_v2/tile_group.py:244-301).
enum BackgroundMode { kBgNone = 0, kBgGather = 1, kBgGatherCols = 2 };
struct PullArgs {
  int mode;
  int slots;                   // blocks to process: the peers
  int rank, world;
  const int64_t* heap_bases;
  const char* src0;            // block 0 of the gathered output in this rank's slice
  int64_t block_bytes;         // distance between consecutive blocks (rows * pitch)
  int block_rows;              // rows per block
  uint32_t pitch;              // bytes per row
  uint32_t upr;                // 16-byte units per row
  uint32_t units;              // units per block (rows * upr)
  int pieces;                  // pieces per block: ceil(units / kPieceUnits)
  // synchronisation
  const int32_t* counter;      // this rank's TileGroup counters; a peer's sit at the same slice offset
  const int32_t* row_ends;
  const int32_t* tile_counts;
  int n_groups, epoch;
  int32_t* barrier;            // every barrier[g] grows by the grid size once all shares are stored
  int64_t* trace_done_clock;
  int64_t* fault;
  int64_t spin_ticks;
  int64_t word_stride;         // as in CommArgs: 0 = a peer's counters sit in its heap slice
  uint32_t src_pitch;          // kBgGatherCols: bytes per row of a shard (`pitch` is the workspace's)
  // Addressing of a unit u of a block: row = u / row_units, byte offset = row * row_pitch + (u - row * row_units) * 16
  // (source: src_row_pitch).  The division is a multiplication: row = row_magic ? mulhi(u, row_magic) >> row_shift
  // : u >> row_shift (set_row_divider() in tccl_api.hip; exact for u < 2^31).  A block whose rows follow each
  // other without gaps is described as one row of `units` units.
  uint32_t row_units, row_magic, row_shift, row_pitch, src_row_pitch;
  // Tile-by-tile readiness (S1): `counter` points at the locks, a "group" is a pair of plan-tile
  // rows, complete once every lock of both rows has reached `epoch`; n_groups = ceil(tile_rows / 2).
  int tile_mode;
  int group_m_shift;           // log2 of the swizzle band height (tile mode needs a power of two)
};
// Gathered input read in place (the gather stage of ChainedAGGemmRSPattern folded into the
// GEMM, patterns/chained_ag_gemm_rs.py:262-391): the GEMM's A operand is the concatenation
// along K of every rank's (M x k_shard) shard, and shard p sits at the same offset of slice
// p.  The K loop fetches its A stages straight from the shard that holds the K range, so it
// does not depend on the gathered workspace; that workspace (GemmArgs::A) is still filled, by
// the background transfer (mode kBgGatherCols: every rank's shard, the own one included, is
// copied into its column block while the K loops run).  k_shard is a multiple of the K step.
struct GatherArgs {
  int active;
  int rank, world;
  const int64_t* heap_bases;
  const void* shard;   // this rank's shard; a peer's sits at the same slice offset
  int64_t ld_shard;    // elements
  int k_shard;         // columns per shard
};
constexpr int kBgWordBytes = 8 * 256;                   // a fetched counter word per wavefront (64 lanes x 4 B)
// Of a SIMD's two wavefronts the older one (wavefronts 0..3 of the workgroup) wins the matrix
// pipe and reaches each K step's barrier early, while the younger one runs alone for the rest of
// the step; scalar work of the younger one therefore delays the step, that of the older one is
// covered by the younger one's MFMAs.  The background pull is carried by the older wavefronts
// alone, two 16-byte units per lane and step, so that its bookkeeping runs once per 2 KiB and
// only where it is covered.
constexpr int kPullWaves = 4;                           // wavefronts of a workgroup that pull
constexpr int kPullLoads = 2;                           // 16-byte units per lane and piece
constexpr int kPieceUnits = 64 * kPullLoads;            // units per piece

TCCL_HD TileCoord macro_coords(int id, const Macro& m) {
  const int per_band = m.rows_per_band * m.cols;
  const int band = id / per_band;
  const int first = band * m.rows_per_band;
  const int height = (m.rows - first) < m.rows_per_band ? (m.rows - first) : m.rows_per_band;
  const int within = id - band * per_band;
  TileCoord c;
  c.m = first + within % height;
  c.n = within / height;
  return c;
}

// Device pass only: the host pass needs the launch signature, not the body.
#if defined(__HIP_DEVICE_COMPILE__)
// A by-value kernel argument read where it is used instead of at kernel entry: arguments
// that only the epilogue or the communication role need would otherwise sit in scalar
// registers (and spill into vector registers) all through the K loop.  The empty asm hides
// the address from the optimiser until control reaches this point.
template <typename T>
TCCL_D const __attribute__((address_space(4))) T* late_kernarg_ptr(int offset) {
  typedef const __attribute__((address_space(4))) char* KernargPtr;
  KernargPtr p = (KernargPtr)__builtin_amdgcn_kernarg_segment_ptr() + offset;
  asm volatile("" : "+s"(p));
  return (const __attribute__((address_space(4))) T*)p;
}
template <typename T>
TCCL_D T late_kernarg(int offset) {
  T v;
  __builtin_memcpy(&v, late_kernarg_ptr<T>(offset), sizeof(T));
  return v;
}

// Request every 64-byte line of the kernel arguments at once.  The compiler reads arguments
// where it first needs them, each group of reads followed by its own wait, so a kernel's
// start used to be a chain of a dozen dependent trips to memory before the first operand load
// could go out; after this the later reads hit in the scalar cache.
template <int kBytes>
TCCL_D void warm_kernargs() {
  typedef const __attribute__((address_space(4))) uint32_t* Words;
  Words p = (Words)__builtin_amdgcn_kernarg_segment_ptr();
  uint32_t any = 0;
#pragma unroll
  for (int o = 0; o < kBytes; o += 64) any |= p[o / 4];
  asm volatile("" ::"s"(any));
}

// kBKMajor: B is given with k contiguous (element (k, n) at B[n * ldb + k], what a `.t()` view of
// an (N, K) weight is: the reference's kernels take any strides, kernels/gemm.py:139-151).  The B
// stage then has the A stage's layout (256 n rows of 128 bytes, same swizzle) and is read with
// ds_read_b128 like A: no transposing reads.
template <typename InT, typename OutT, bool kWithReduce = false, bool kGatherA = false, bool kBKMajor = false>
struct Gemm256 {
  typedef typename Mfma<InT>::Vec Vec;
  static constexpr int kEszIn = sizeof(InT);
  static constexpr int kStepK = kARow256 / kEszIn;     // K per step: 64 (16-bit), 128 (fp8)
  static constexpr int kChunkK = 16 / kEszIn;          // elements per 16-byte chunk
  static constexpr int kBPitch = kMacro * kEszIn;      // bytes per k row of the B stage
  static constexpr int kBRowsPerPiece = 1024 / kBPitch;  // k rows one 1 KiB load covers: 2 or 4
  static constexpr bool kFp8 = kEszIn == 1;

  const GemmArgs& g;
  // Byte offset of a PullArgs in the kernel arguments (< 0: no background transfer).  Like the
  // push and reduce arguments it is read where it is used: taken as a kernel argument struct its
  // thirty-odd fields were loaded at the kernel's start and held in scalar registers (or the
  // lanes they spill to) through every K loop.
  const int pull_offset;
  const int push_offset;    // byte offset of a PushArgs in the kernel arguments; < 0: no push
  const int reduce_offset;  // byte offset of a ReduceArgs in the kernel arguments; < 0: none
  const int gather_offset;  // byte offset of a GatherArgs in the kernel arguments (kGatherA only)
  // The two pipeline stages are two separate __shared__ arrays: loads that write LDS directly
  // are tracked per LDS variable, so a read of one stage need not wait for a load into the other.
  char* lds;   // stage 0 (also the epilogue's staging area)
  char* lds1;  // stage 1
  char* bgw;   // landing words of the background transfer's counter fetches
  const int tid, lane, wave, wm, wn;
  // A per-lane value the optimiser must treat as new at this point (blocks hoisting of what is derived from it).
  static TCCL_D int fresh(int v) {
    asm volatile("" : "+v"(v));
    return v;
  }
  // The lane's number, counted afresh (two instructions): what the per-step code of the background
  // transfer derives from it is then formed where it is used instead of sitting in registers through
  // the K loop.
  // A wavefront-uniform sum the optimiser must take as a whole: split up, its loop-invariant part is added
  // to the per-lane offsets ahead of the K loop, one register per combination.
  static TCCL_D uint32_t whole(uint32_t v) {
    asm("" : "+s"(v));
    return v;
  }
  static TCCL_D int lane_now() { return fresh((int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }


  TCCL_D Gemm256(const GemmArgs& args, int pull_args_offset, int push_args_offset, int reduce_args_offset, char* stage0,
                 char* stage1, char* landing_words, int gather_args_offset = -1)
      : g(args), pull_offset(pull_args_offset), push_offset(push_args_offset), reduce_offset(reduce_args_offset), gather_offset(gather_args_offset), lds(stage0), lds1(stage1), bgw(landing_words), tid(threadIdx.x), lane(threadIdx.x & 63),
        // the wavefront's number is the same in all its lanes: held in a scalar register, and with it the LDS
        // addresses its loads land at (kept per lane they cost eight registers and a readfirstlane per load)
        wave(__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)), wm(__builtin_amdgcn_readfirstlane(threadIdx.x >> 8)),
        wn(__builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3)) {}

  typedef __attribute__((address_space(3))) void LdsVoid;
  typedef const __attribute__((address_space(4))) PullArgs* PullPtr;
  TCCL_D PullPtr pa() const { return late_kernarg_ptr<PullArgs>(pull_offset < 0 ? 0 : pull_offset); }
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 LdsQuad;

  // Where this lane's four A pieces and four B pieces of a K step come from (byte offsets
  // into the buffer resources at K step 0).  Piece i of wave w fills
  //   A rows 8*(4w+i) .. +7      (lane l: row + l/8, slot l%8)
  //   B k rows 2*(4w+i), +1      (lane l: k row + l/32, slot l%32)            16-bit inputs
  //   B k rows 4*(4w+i) .. +3    (lane l: k row + l/16, slot l%16)            fp8 inputs
  struct Source {
    __amdgpu_buffer_rsrc_t a, b;
    // Pieces 0 and 1 per lane; pieces 2 and 3 lie a fixed distance behind them (pair_a, pair_b), which is
    // added where a load is issued: half the registers through the K loop.
    uint32_t off_a[2], off_b[2];
    uint32_t pair_a, pair_b;
    uint32_t step_a, step_b;
    // kGatherA: `a` is the window onto the shard that holds K steps [kt_base, kt_switch)
    int kt_base, kt_switch, row0;
  };
  typedef const __attribute__((address_space(4))) GatherArgs* GatherPtr;

  // Point `s.a` at the shard that holds K step kt (kGatherA).  Steps past K stay on the last
  // shard: their chunks are redirected past the end of the window by issue_a and read as zero.
  TCCL_D void select_shard(Source& s, int kt) const {
    const GatherPtr ga = late_kernarg_ptr<GatherArgs>(gather_offset);
    const int per_shard = ga->k_shard / kStepK;
    int p = kt / per_shard;
    if (p >= ga->world) p = ga->world - 1;
    const int64_t base = (int64_t)(uintptr_t)ga->shard + (table(ga->heap_bases, p) - table(ga->heap_bases, ga->rank)) +
                         (int64_t)s.row0 * ga->ld_shard * kEszIn;
    s.a = __builtin_amdgcn_make_buffer_rsrc((void*)(uintptr_t)base, 0,
                                            clamp_u32(((int64_t)(g.M - 1 - s.row0) * ga->ld_shard + ga->k_shard) * kEszIn), 0x00020000);
    s.kt_base = p * per_shard;
    s.kt_switch = p + 1 < ga->world ? (p + 1) * per_shard : 0x7fffffff;
  }
  // Before the loads of K step kt are issued.
  TCCL_D void follow_shards(Source& s, int kt) const {
    if constexpr (kGatherA)
      if (kt >= s.kt_switch) select_shard(s, kt);
  }

  static TCCL_D uint32_t clamp_u32(int64_t v) { return v > 0xffffffffll ? 0xffffffffu : (v < 0 ? 0u : (uint32_t)v); }

  TCCL_D Source make_source(int row0, int col0) const {
    constexpr int kEsz = sizeof(InT);
    Source s;
    // The lane's number is taken afresh: derived from the member, the offsets below are the same for every
    // tile, get computed once at the kernel's start and, in the kernels that sit at the register limit, are
    // parked in scratch memory through the K loops; reloading them between a tile's first operand requests
    // made each reload wait for the requests ahead of it (three trips to memory in a row, 2 us per tile).
    const int lane = lane_now();
    const OperandOrigin o = operand_origin(g, row0, col0);
    const InT* A = (const InT*)g.A + (int64_t)o.a_row * g.lda;
    const InT* B = (const InT*)g.B + (kBKMajor ? (int64_t)o.b_col * g.ldb : (int64_t)o.b_col);
    s.a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, clamp_u32(((int64_t)(o.a_rows - 1 - o.a_row) * g.lda + g.K) * kEsz), 0x00020000);
    if constexpr (kBKMajor)
      s.b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, clamp_u32(((int64_t)(o.b_cols - 1 - o.b_col) * g.ldb + g.K) * kEsz), 0x00020000);
    else
      s.b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, clamp_u32(((int64_t)(g.K - 1) * g.ldb + (o.b_cols - o.b_col)) * kEsz), 0x00020000);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 8 * (4 * wave + i) + (lane >> 3);
      const int kc = (lane & 7) ^ ((row >> 1) & 7);
      int64_t lda = g.lda;
      if constexpr (kGatherA) lda = late_kernarg_ptr<GatherArgs>(gather_offset)->ld_shard;
      s.off_a[i] = (uint32_t)(row * lda * kEsz + kc * 16);
      if constexpr (kBKMajor) {
        s.off_b[i] = (uint32_t)(row * g.ldb * kEsz + kc * 16);
      } else if constexpr (kFp8) {
        const int k = 4 * (4 * wave + i) + (lane >> 4);
        const int c = (lane & 15) ^ (2 * (k & 7)) ^ ((k >> 4) & 1);
        s.off_b[i] = (uint32_t)(k * g.ldb * kEsz + c * 16);
      } else {
        const int k = 2 * (4 * wave + i) + (lane >> 5);
        const int c = (lane & 31) ^ (4 * (k & 3)) ^ (2 * ((k >> 3) & 1));
        s.off_b[i] = (uint32_t)(k * g.ldb * kEsz + c * 16);
      }
    }
    // Piece i + 2 covers rows (k rows) 16 (2 * kBRowsPerPiece) further on; the swizzle terms repeat with
    // that period (rows: (row >> 1) & 7; k rows: k & 3 resp. k & 7), and bit 3 of k (16-bit B) only
    // depends on the wave.
    {
      int64_t lda = g.lda;
      if constexpr (kGatherA) lda = late_kernarg_ptr<GatherArgs>(gather_offset)->ld_shard;
      s.pair_a = (uint32_t)(16 * lda * kEsz);
      s.pair_b = kBKMajor ? (uint32_t)(16 * g.ldb * kEsz) : (uint32_t)(2 * kBRowsPerPiece * g.ldb * kEsz);
    }
    s.step_a = kStepK * kEsz;
    s.step_b = kBKMajor ? (uint32_t)(kStepK * kEsz) : (uint32_t)(kStepK * g.ldb * kEsz);
    s.kt_base = 0;
    s.kt_switch = 0x7fffffff;
    s.row0 = row0;
    if constexpr (kGatherA) select_shard(s, 0);
    return s;
  }

  // Piece i of K step kt, straight into `stage`.  A chunks at k >= K are redirected past the
  // end of the buffer so that they read as zero (B rows >= K already lie past it).
  TCCL_D void issue_a(char* stage, const Source& s, int kt, int i) const {
    const int kc = (lane & 7) ^ ((4 * (i & 1) + (lane >> 4)) & 7);  // as in make_source
    const bool dead = kt * kStepK + kc * kChunkK >= g.K;
    const uint32_t oa = dead ? 0xfffffff0u : s.off_a[i & 1] + ((kGatherA ? kt - s.kt_base : kt) * s.step_a + (i >> 1) * s.pair_a);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(s.a, (LdsVoid*)(stage + 8 * (4 * wave + i) * kARow256), 16, oa, 0, 0, 0);
  }
  TCCL_D void issue_b(char* stage, const Source& s, int kt, int i) const {
    if constexpr (kBKMajor) {
      const int kc = (lane & 7) ^ ((4 * (i & 1) + (lane >> 4)) & 7);
      const bool dead = kt * kStepK + kc * kChunkK >= g.K;
      const uint32_t ob = dead ? 0xfffffff0u : s.off_b[i & 1] + whole(kt * s.step_b + (i >> 1) * s.pair_b);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s.b, (LdsVoid*)(stage + kAStage256 + 8 * (4 * wave + i) * kARow256), 16, ob, 0, 0, 0);
      return;
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(s.b, (LdsVoid*)(stage + kAStage256 + (4 * wave + i) * 1024), 16,
                                             s.off_b[i & 1] + whole(kt * s.step_b + (i >> 1) * s.pair_b), 0, 0, 0);
  }
  TCCL_D void issue_piece(char* stage, const Source& s, int kt, int i) const {
    issue_a(stage, s, kt, i);
    issue_b(stage, s, kt, i);
  }

  // Per-lane LDS read addresses that do not depend on the k-chunk.
  struct Reader {
    uint32_t a_base;   // row of this lane in the A stage
    uint32_t a_swz;    // XOR term of the A slot
    uint32_t b_base0;  // B address for the first column block, first k block (the others: load_b8 / load_b16)
  };

  TCCL_D Reader make_reader() const {
    const int i16 = lane & 15;
    Reader r;
    if constexpr (!kFp8) {
      // 16 x 16 x 32 operands: lane l reads row (column) l % 16 of a 16-row block, k group l / 16.
      const int kg = lane >> 4, t = i16 >> 2, cq = i16 & 3;
      r.a_base = (uint32_t)((wm * 128 + i16) * kARow256);
      r.a_swz = (uint32_t)((i16 >> 1) & 7);
      if constexpr (kBKMajor) {
        r.b_base0 = (uint32_t)(kAStage256 + (wn * 64 + i16) * kARow256);  // this lane's row of column block 0
      } else {
        // ds_read_b64_tr_b16: within 16 lanes, lane i supplies 4 consecutive columns (4 * (i % 4) ..) of
        // k row i / 4 and lane j receives those 4 k of column j.  Lane group kg covers k rows 8 * kg ..
        // + 7 in two reads (k + 0, k + 4).
        const int chunk = (wn * 8 + (cq >> 1)) ^ (4 * t) ^ (2 * (kg & 1));
        r.b_base0 = (uint32_t)(kAStage256 + (8 * kg + t) * kBPitch + chunk * 16 + (cq & 1) * 8);
      }
    } else {
      // 16 x 16 x 128 operands: lane l reads row (column) l % 16 of a 16-row block, k group l / 16 (32 k).
      const int kg = lane >> 4;
      r.a_base = (uint32_t)((wm * 128 + i16) * kARow256);
      r.a_swz = (uint32_t)((i16 >> 1) & 7);
      if constexpr (kBKMajor) {
        r.b_base0 = (uint32_t)(kAStage256 + (wn * 64 + i16) * kARow256);  // this lane's row of column block 0
      } else {
        // ds_read_b64_tr_b8: within 16 lanes, lane i supplies 8 consecutive columns (8 * (i % 2) ..) of k
        // row i / 2 and lane j receives those 8 k of column j.  Lane group kg covers k rows 16 * kg .. + 15 and
        // 64 + 16 * kg .. + 15 in four reads (k + 0, 8, 64, 72), the k that load_a8() gives the group.
        const int krow = i16 >> 1;
        const int chunk = (wn * 4) ^ (2 * krow) ^ (kg & 1);
        r.b_base0 = (uint32_t)(kAStage256 + (16 * kg + krow) * kBPitch + chunk * 16 + (i16 & 1) * 8);
      }
    }
    return r;
  }

  typedef int i32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) i32x2 LdsPair;

  // fp8 operands of a K step (128 k, one MFMA deep): the A rows of the 16-row block rb, the B columns of
  // the 16-column block cb.
  TCCL_D Vec load_a8(const char* stage, const Reader& r, int rb) const {
    const int kg = lane >> 4;
    // The two 16-byte chunks of a lane are chunks kg and kg + 4 of the row (chunk and chunk ^ 4 under the swizzle).
    // Both addresses are formed by adding to `stage`: flipping a bit of the pointer itself
    // would hide that it points into LDS, and the load would become a flat load, which
    // waits for every outstanding global load.
    const uint32_t chunk = ((uint32_t)kg) ^ r.a_swz;
    const char* row = stage + r.a_base + rb * 16 * kARow256;
    const u32x4 lo = *(const u32x4*)(row + (chunk << 4));
    const u32x4 hi = *(const u32x4*)(row + ((chunk ^ 4u) << 4));
    typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
    const u32x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(Vec, both);
  }
  TCCL_D Vec load_b8(const char* stage, const Reader& r, int cb) const {
    if constexpr (kBKMajor) {
      const int kg = lane >> 4;
      const uint32_t chunk = ((uint32_t)kg) ^ r.a_swz;
      const char* row = stage + r.b_base0 + cb * 16 * kARow256;
      const u32x4 lo = *(const u32x4*)(row + (chunk << 4));
      const u32x4 hi = *(const u32x4*)(row + ((chunk ^ 4u) << 4));
      typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
      const u32x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(Vec, both);
    }
    // column block cb: one chunk further on per block (the XOR commutes with the swizzle terms)
    const char* p = stage + (r.b_base0 ^ (uint32_t)(16 * cb));
    i32x2 q[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) q[t] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsPair*)(p + (8 * (t & 1) + 64 * (t >> 1)) * kBPitch));
    i32x8 v;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v[2 * t] = q[t][0];
      v[2 * t + 1] = q[t][1];
    }
    return __builtin_bit_cast(Vec, v);
  }

  // 16-bit operands of k-block kh (32 k): the A rows of the 16-row block rb; the B columns of the
  // wave's four 16-column blocks.
  TCCL_D Vec load_a16(const char* stage, const Reader& r, int kh, int rb) const {
    const int kg = lane >> 4;
    return *(const Vec*)(stage + r.a_base + ((((uint32_t)(4 * kh + kg)) ^ r.a_swz) << 4) + rb * 16 * kARow256);
  }
  TCCL_D Vec load_b16(const char* stage, const Reader& r, int kh, int cb) const {
    if constexpr (kBKMajor) {
      const int kg = lane >> 4;
      return *(const Vec*)(stage + r.b_base0 + ((((uint32_t)(4 * kh + kg)) ^ r.a_swz) << 4) + cb * 16 * kARow256);
    }
    // column block cb: two chunks further on per block; the XOR commutes with the swizzle terms (they touch
    // the chunk index only through XOR as well)
    const char* pb = stage + (r.b_base0 ^ (uint32_t)(32 * cb)) + 32 * kh * kBPitch;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsQuad*)pb);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsQuad*)(pb + 4 * kBPitch));
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(Vec, both);
  }

  // ---- background transfer -----------------------------------------------------------------------
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  struct PullState {
    int next_slot, next_lp;  // next piece of this wavefront: block slot, piece inside the block
    int stride;              // wavefronts in the grid
    int slot;                // slot that the bases and the readiness cache describe (-1: none)
    int gidx;                // first TileGroup of that block not yet known complete
    int row0;                // first row of that block in the plan's row numbering
    uint32_t ready_units;    // units [0, ready_units) of that block may be fetched
    int64_t src_base, dst_base;  // addresses of the block in the peer's slice and in this one
    int64_t counter_base;        // the peer's counter words
    int probe_group;         // group whose counters were fetched during the previous step (-1: none)
    int32_t need;            // epoch * tile_counts[gidx]: what the counters of group gidx must reach
    uint32_t group_units;    // ready_units once group gidx is complete
    int backoff;             // K steps to let pass before the counters are fetched again
    int pend_lp;             // piece of the selected block that was requested and is not yet stored (-1: none)
    // The piece itself.  One set of registers: a piece is stored (pull_retire) before the next one is
    // requested, in every path; a second set costs the fused kernels registers they do not have.
    u32x4 piece[1][kPullLoads];
    int probe_off;           // this wavefront's counter landing words
    // The counter word, read out of the landing words right behind a K step's barrier: read
    // there, it is older than every operand fetch that follows, so using it never waits for those.
    int32_t probe_val;
    // What the per-step code needs from PullArgs, kept in registers (reading a field through
    // the argument block is a scalar load plus a wait that also drains the operand fetches).
    bool active;
    uint32_t units;
    int pieces, slots, n_groups;
    uint32_t row_units, row_magic, row_shift, row_pitch;
  };

  // Values that are the same in every lane but that the compiler cannot prove so (loaded
  // through a pointer, derived from threadIdx) are moved to scalar registers explicitly;
  // otherwise each buffer descriptor built from them costs a per-lane loop.
  static TCCL_D int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
  // Read-only tables (plan rows, tile counts, slice bases) through the scalar path.
  template <typename T>
  static TCCL_D T table(const T* p, int i) {
    return ((const __attribute__((address_space(4))) T*)p)[i];
  }

  TCCL_D PullState pull_begin(PullPtr a, int wg, int num_wgs) const {
    PullState st;
    const int w = uniform(wave);
    st.probe_off = w * 256;
    st.stride = num_wgs * kPullWaves;
    st.next_slot = 0;
    st.next_lp = wg * kPullWaves + w;
    st.slot = -1;
    st.gidx = 0;
    st.row0 = 0;
    st.ready_units = 0;
    st.src_base = st.dst_base = st.counter_base = 0;
    st.probe_group = -1;
    st.need = 0;
    st.group_units = 0;
    st.backoff = 0;
    st.pend_lp = -1;
    st.probe_val = 0;
#pragma unroll
    for (int j = 0; j < kPullLoads; ++j) st.piece[0][j] = u32x4{0, 0, 0, 0};
    st.active = pull_offset >= 0 && a->mode != kBgNone && w < kPullWaves;
    st.units = 0;
    st.pieces = st.slots = st.n_groups = 0;
    st.row_units = 1;
    st.row_magic = st.row_shift = st.row_pitch = 0;
    if (st.active) {
      st.units = a->units;
      st.pieces = a->pieces;
      st.slots = a->slots;
      st.n_groups = a->n_groups;
      st.row_units = a->row_units;
      st.row_magic = a->row_magic;
      st.row_shift = a->row_shift;
      st.row_pitch = a->row_pitch;
      pull_normalise(st, a);
    }
    return st;
  }

  // Where this lane's unit j of piece lp lies inside a block: byte offsets on the destination and the source
  // side (kNoUnit / the block's first unit for lanes beyond the block's end: their stores fall outside the
  // buffer window and are dropped, their loads touch a unit that exists).  A handful of vector instructions
  // from three scalars, formed where a piece is requested and again where it is stored: whatever a pulling
  // lane carries from K step to K step besides the piece itself costs registers that the fused kernels do
  // not have (kept in LDS instead, its reads and their waits made the per-step code several times as long).
  static constexpr uint32_t kNoUnit = 0xffffffffu;
  TCCL_D void pull_where(const PullState& st, PullPtr a, int lp, int j, int ln, uint32_t& to, uint32_t& from) const {
    const uint32_t u = (uint32_t)lp * (uint32_t)kPieceUnits + (uint32_t)(64 * j + ln);
    const bool valid = u < st.units;
    const uint32_t uu = valid ? u : 0u;
    const uint32_t row = st.row_magic ? (__umulhi(uu, st.row_magic) >> st.row_shift) : (uu >> st.row_shift);
    const uint32_t col = uu - row * st.row_units;
    const uint32_t off = row * st.row_pitch + col * 16u;
    to = valid ? off : kNoUnit;
    from = off;
    if constexpr (kGatherA) from = row * a->src_row_pitch + col * 16u;
  }

  // Fetch the first counters in the first tile's prologue, so that the first K step can
  // already fetch a piece.
  TCCL_D void pull_prime(PullState& st, PullPtr a, char* landing) const {
    if constexpr (kWithReduce) return;  // that instantiation never pulls: its launch clears PullArgs
    if (!st.active || st.next_slot >= a->slots) return;
    pull_select(st, a, st.next_slot);
    pull_probe(st, a, landing);
  }

  // Every lane fetches the same word; it is read back from LDS one K step later.
  TCCL_D void pull_probe(PullState& st, PullPtr a, char* landing) const {
    if (st.gidx >= st.n_groups) return;
    if (st.backoff > 0) {
      --st.backoff;
      return;
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(window(st.counter_base), (LdsVoid*)(bgw + st.probe_off), 4, probe_offset(a, st.gidx), 0, 0,
                                             kCoherent);
    st.probe_group = st.gidx;
  }

  TCCL_D void pull_normalise(PullState& st, PullPtr a) const {
    while (st.next_lp >= a->pieces && st.next_slot < a->slots) {
      st.next_lp -= a->pieces;
      ++st.next_slot;
    }
  }

  TCCL_D uint32_t pull_last_unit(PullPtr a, int lp) const {
    const uint32_t last = (uint32_t)lp * (uint32_t)kPieceUnits + (uint32_t)(kPieceUnits - 1);
    return last < a->units ? last : a->units - 1u;
  }

  TCCL_D void pull_select(PullState& st, PullPtr a, int slot) const {
    if (slot == st.slot) return;
    st.slot = slot;
    st.ready_units = 0;
    st.probe_group = -1;
    st.backoff = 0;
    if constexpr (kGatherA) {
      // Block `slot` = rank `slot`'s shard (resident input: nothing to wait for) into column
      // block `slot` of the gathered workspace.
      const GatherPtr ga = late_kernarg_ptr<GatherArgs>(gather_offset);
      st.src_base = (int64_t)(uintptr_t)ga->shard + (table(ga->heap_bases, slot) - table(ga->heap_bases, ga->rank));
      st.dst_base = (int64_t)(uintptr_t)g.A + (int64_t)slot * ga->k_shard * kEszIn;
      st.ready_units = a->units;
      st.gidx = a->n_groups;
      return;
    }
    const int64_t mine = table(a->heap_bases, a->rank);
    const int peer = slot < a->rank ? slot : slot + 1;
    const int64_t theirs = table(a->heap_bases, peer);
    const int64_t rel = ((int64_t)(uintptr_t)a->src0 - mine) + (int64_t)peer * a->block_bytes;
    st.src_base = theirs + rel;
    st.dst_base = mine + rel;
    const int64_t stride = a->word_stride;
    st.counter_base = (int64_t)(uintptr_t)a->counter + (stride ? (int64_t)(peer - a->rank) * stride : theirs - mine);
    st.row0 = 0;  // the plan numbers the rows of one block
    st.gidx = 0;
    pull_group_facts(st, a);
  }

  static TCCL_D void unpack(u32x4 v, float (&f)[8], int& n) {
    if constexpr (sizeof(OutT) == 4) {
      const f32x4v x = __builtin_bit_cast(f32x4v, v);
      n = 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f[e] = x[e];
        f[4 + e] = 0.f;
      }
    } else if constexpr (__is_same(OutT, __bf16)) {
      const bf16x8v x = __builtin_bit_cast(bf16x8v, v);
      n = 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (float)x[e];
    } else {
      const f16x8v x = __builtin_bit_cast(f16x8v, v);
      n = 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (float)x[e];
    }
  }

  // Store the piece that is pending, if any.  Returns whether a store was issued.  The piece belongs
  // to the selected block: pull_issue() stores what is pending before it selects another one.
  TCCL_D bool pull_retire(PullState& st, PullPtr a, const char* landing, int) const {
    if constexpr (kWithReduce) return false;
    if (st.pend_lp < 0) return false;
    const __amdgpu_buffer_rsrc_t dst = window(st.dst_base);
    const int ln = lane_now();
#pragma unroll
    for (int j = 0; j < kPullLoads; ++j) {
      uint32_t to, from;
      pull_where(st, a, st.pend_lp, j, ln, to, from);
      st16<kStreaming>(dst, to, st.piece[0][j]);
    }
    st.pend_lp = -1;
    return true;
  }

  // The two facts about group gidx that the per-step code needs, fetched when gidx changes.
  TCCL_D void pull_group_facts(PullState& st, PullPtr a) const {
    if (st.gidx >= a->n_groups) return;
    if (a->tile_mode) {
      const int rows = (2 * st.gidx + 2) * g.block_m;
      st.need = a->epoch;
      st.group_units = (uint32_t)(rows < a->block_rows ? rows : a->block_rows) * a->upr;
      return;
    }
    st.need = (int32_t)((uint32_t)a->epoch * (uint32_t)table(a->tile_counts, st.gidx));
    st.group_units = (uint32_t)(table(a->row_ends, st.gidx) - st.row0) * a->upr;
  }
  // Byte offset, inside the peer's words, of the word this lane looks at to learn whether group
  // `gidx` is complete: the group's counter, or (tile mode) the lock of one plan tile of the
  // group's two tile rows: lanes 0..31 take the columns of row 2 gidx, lanes 32..63 those of row
  // 2 gidx + 1; lanes beyond the grid look at a tile that exists (a duplicate).
  TCCL_D uint32_t probe_offset(PullPtr a, int gidx) const {
    if (!a->tile_mode) return (uint32_t)gidx * 4u;
    const int ln = lane_now();
    int tm = 2 * gidx + (ln >> 5);
    if (tm >= g.tile_rows) tm = g.tile_rows - 1;
    int tn = ln & 31;
    if (tn >= g.tile_cols) tn = 0;
    const int sh = a->group_m_shift;
    const int first_m = (tm >> sh) << sh;
    const int height = g.tile_rows - first_m < (1 << sh) ? g.tile_rows - first_m : (1 << sh);
    return (uint32_t)(first_m * g.tile_cols + tn * height + (tm - first_m)) * 4u;
  }
  // Every lane's word has reached the threshold (one and the same word outside tile mode).
  static TCCL_D bool all_reached(int32_t word, int32_t need) { return __builtin_amdgcn_ballot_w64(!word_reached(word, need)) == 0ull; }
  TCCL_D void pull_group_done(PullState& st, PullPtr a) const {
    st.ready_units = st.group_units;
    ++st.gidx;
    pull_group_facts(st, a);
  }

  // Right behind a K step's barrier (this wave's loads, the counter fetch among them, have
  // landed): take the counter word out of the landing words.
  TCCL_D void pull_collect(PullState& st, PullPtr a, const char* landing, int slot) const {
    if constexpr (kWithReduce) return;
    if (!st.active) return;
    st.probe_val = *(const int32_t*)(bgw + st.probe_off + 4 * lane_now());  // lane l's word landed at 4 l
  }
  // Once per K step: learn about readiness, request the next piece into slot `slot` (its
  // previous piece was stored during the step before).  All control flow here is
  // wavefront-uniform.  Returns whether a piece was requested.
  TCCL_D bool pull_issue(PullState& st, PullPtr a, char* landing, int) const {
    if constexpr (kWithReduce) return false;
    if (!st.active) return false;
    if (st.probe_group >= 0) {
      const int g = st.probe_group;
      st.probe_group = -1;
      if (g == st.gidx) {
        if (all_reached(st.probe_val, st.need))
          pull_group_done(st, a);
        else
          st.backoff = 3;  // not there yet: fetching the counters every step only costs issue slots
      }
    }
    if (st.next_slot >= st.slots) return false;
    if (st.next_slot != st.slot) {
      pull_retire(st, a, landing, 0);  // a piece still pending belongs to the block being left
      pull_select(st, a, st.next_slot);
      pull_probe(st, a, landing);
      return false;
    }
    pull_probe(st, a, landing);  // look ahead: the next group's counters (issued before the piece, which stays the youngest load)
    const uint32_t first = (uint32_t)st.next_lp * (uint32_t)kPieceUnits;
    const uint32_t last = first + (uint32_t)(kPieceUnits - 1);
    if ((last < st.units ? last : st.units - 1u) < st.ready_units) {
      const __amdgpu_buffer_rsrc_t src = window(st.src_base);
      const int ln = lane_now();
#pragma unroll
      for (int j = 0; j < kPullLoads; ++j) {
        uint32_t to, from;
        pull_where(st, a, st.next_lp, j, ln, to, from);
        st.piece[0][j] = ld16<kCoherent>(src, from);
      }
      st.pend_lp = st.next_lp;
      st.next_lp += st.stride;
      if (st.next_lp >= st.pieces) pull_normalise(st, a);  // block finished: rare
      return true;
    }
    return false;
  }

  // Wait (bounded) until units [0, last] of the selected block may be fetched.
  TCCL_D bool pull_wait_ready(PullState& st, PullPtr a, uint32_t last, int64_t deadline) const {
    while (last >= st.ready_units) {
      if (st.gidx >= a->n_groups) return false;
      const int32_t need = st.need;
      const __amdgpu_buffer_rsrc_t words = window(st.counter_base);
      const uint32_t where = probe_offset(a, st.gidx);
      for (;;) {
        const int32_t seen = (int32_t)__builtin_amdgcn_raw_buffer_load_b32(words, where, 0, kCoherent);
        if (all_reached(seen, need)) break;
        if (now_ticks() > deadline) return false;
        __builtin_amdgcn_s_sleep(8);
      }
      pull_group_done(st, a);
    }
    return true;
  }

  // After the last tile: finish what is in flight, move the remaining pieces, report.
  TCCL_D void pull_finish(PullState& st, PullPtr a, const char* landing, int num_wgs) const {
    if constexpr (kWithReduce) return;
    if (pull_offset < 0 || a->mode == kBgNone) return;  // the same for every wavefront: a barrier follows
    bool ok = true;
    if (st.active) ok = pull_drain(st, a, landing);
    if (!ok && lane == 0 && a->fault) *a->fault = 1;
    wait_vmem();
    __syncthreads();
    // Only a traced launch counts arrivals: one per workgroup on barrier[0], and the last one
    // to arrive brings the other groups' words up to the same count and stamps the clocks.
    // Nobody waits on these words (a pull completes on the pulling rank, whose kernel ends;
    // pushes are announced by counter[g]), and 256 adds to one word cost ~7 ns each here,
    // ~1 us at the very end of every launch.
    if (tid == 0 && a->barrier && a->trace_done_clock) {
      const int32_t prev = tile_signal_add<true>(a->barrier, 0, 1);
      if (prev + 1 == a->epoch * num_wgs) {
        for (int g = 0; g < a->n_groups; ++g) {
          if (g > 0) tile_signal_add<true>(a->barrier, g, num_wgs);
          a->trace_done_clock[g] = now_ticks();
        }
      }
    }
  }

  // The pulling wavefronts' part of pull_finish; false if a bounded wait expired.
  TCCL_D bool pull_drain(PullState& st, PullPtr a, const char* landing) const {
    wait_vmem();
    pull_retire(st, a, landing, 0);
    st.probe_group = -1;
    const int64_t deadline = now_ticks() + a->spin_ticks;
    bool ok = true;
    constexpr int kBatch = 8;  // pieces in flight per pulling wavefront: the CU has no other work left
    while (ok && st.next_slot < a->slots) {
      pull_select(st, a, st.next_slot);
      u32x4 v[kBatch][kPullLoads];
      uint32_t off[kBatch][kPullLoads];
      bool loaded[kBatch];
      int n = 0;
      const __amdgpu_buffer_rsrc_t src = window(st.src_base);
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        loaded[k] = false;
        const int lp = st.next_lp + k * st.stride;
        if (ok && lp < a->pieces) {
          ok = pull_wait_ready(st, a, pull_last_unit(a, lp), deadline);
          if (ok) {
#pragma unroll
            for (int j = 0; j < kPullLoads; ++j) {
              uint32_t from;
              pull_where(st, a, lp, j, lane, off[k][j], from);
              v[k][j] = ld16<kCoherent>(src, from);
            }
            loaded[k] = true;
            n = k + 1;
          }
        }
      }
      const __amdgpu_buffer_rsrc_t dst = window(st.dst_base);
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        if (!loaded[k]) continue;
#pragma unroll
        for (int j = 0; j < kPullLoads; ++j)
          if (off[k][j] != kNoUnit) st16<kStreaming>(dst, off[k][j], v[k][j]);
      }
      st.next_lp += n * st.stride;
      if (n < kBatch) {  // the block is finished (or a wait gave up)
        st.next_lp -= a->pieces;
        if (st.next_lp < 0) st.next_lp = 0;  // only after a failed wait
        ++st.next_slot;
        pull_normalise(st, a);
      }
    }
    return ok;
  }

  // 16-bit operand registers; they live across K steps.
  struct Frags {
    Vec ring[4], fb[4];
  };

  // fp8 operand registers; they live across K steps.
  struct Frags8 {
    Vec ring[2], fb[4];
  };

  // One K step of the fp8 path (v_mfma_scale_f32_16x16x128_f8f6f4, 128 k per step): eight items of four
  // MFMAs, item d = the 16-row block d of the wave tile against its four 16-column blocks, read from
  // `cur` while the next step's operands stream into `nxt` (one pair of loads per item, items 0..3).
  // An fp8 operand is 8 registers: the A operand is fetched one item ahead (two register sets), the four
  // B operands have one set and are reloaded in place during the last item, each as soon as its MFMA is
  // issued.  As in the 16-bit path the step's one barrier sits inside the step, before item 7: the reads
  // of `cur` are done, the loads into `nxt` have landed, and item 7 fetches the next step's first
  // operands from `nxt` behind it.
  TCCL_D void k_step8(const char* cur, char* nxt, const Source& src, const Reader& rd, int kt_load, f32x16 (&acc)[4][2],
                      Frags8& f, PullState& pull, int parity) const {
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      if (d == 7) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        pull_collect(pull, pa(), bgw, parity);
      }
      const char* from = d + 1 < 8 ? cur : nxt;
      f.ring[(d + 1) & 1] = load_a8(from, rd, (d + 1) & 7);
      if (d < 4) issue_piece(nxt, src, kt_load, d);
      // The background transfer's one place in the step, as in the 16-bit path: behind the step's last
      // operand loads, the piece of the step before stored first, the next one requested into its registers.
      if constexpr (!kWithReduce) {
        if (d == 3 && pull.active) {
          pull_retire(pull, pa(), bgw, parity ^ 1);
          pull_issue(pull, pa(), bgw, parity);
        }
      }
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        f32x16& patch = acc[d >> 1][cb >> 1];
        const int q = 2 * (d & 1) + (cb & 1);
        f32x4 blk = {patch[4 * q], patch[4 * q + 1], patch[4 * q + 2], patch[4 * q + 3]};
        blk = Mfma<InT>::run16(f.fb[cb], f.ring[d & 1], blk);
#pragma unroll
        for (int e = 0; e < 4; ++e) patch[4 * q + e] = blk[e];
        if (d == 7) {
          __builtin_amdgcn_sched_barrier(0);
          f.fb[cb] = load_b8(nxt, rd, cb);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // One K step of the 16-bit path (v_mfma_f32_16x16x32): eight items of eight MFMAs each, read from `cur`
  // while the next step's operands stream into `nxt`.  Item d covers k block kh = d / 4 (32 k) and the
  // 16-row blocks 2 * (d % 4), + 1 of the wave tile, against all four 16-column blocks.
  //
  // A operands (two per item) are fetched one item ahead through four register sets.  B operands
  // (four per k block) have ONE register set: the last item of a k block runs column block by
  // column block, and as soon as a column block's two MFMAs are issued its registers take the next k
  // block's operand, which is first needed six MFMAs later (the first item of a k block runs in the
  // same order).  A second set would cost 16 registers, which the fused kernels do not have.
  // The scheduling barriers pin this order (left alone, the compiler hoists every read of the step and
  // spills).
  //
  // The step's one barrier sits before the last item, not at the end.  There this wave has issued
  // (and, after the lgkmcnt wait, finished) its last read of `cur`, and its loads into `nxt`,
  // issued during items 0..3, have landed; behind the barrier the last item already fetches
  // the next step's first operands from `nxt`, so the matrix pipe does not drain while the
  // first LDS reads of a step are in flight.
  //
  // Issuing a global load holds the wave for as long as the address unit takes to accept it (about 16
  // clocks per KiB instruction, four times that when the four SIMDs' waves issue in the same item),
  // and nothing else of the wave issues meanwhile; they go out two per item over items 0..3.
  TCCL_D void k_step16(const char* cur, char* nxt, const Source& src, const Reader& rd, int kt_load, f32x16 (&acc)[4][2],
                       Frags& f, PullState& pull, int parity) const {
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      const int rp = d & 3;
      if (d == 7) {
        // This wave's loads (and background fetch) have landed, its reads of `cur` are done.
        // The barrier is the bare instruction: __syncthreads() carries a workgroup-scope
        // release fence.  The empty asm keeps the compiler from moving LDS accesses across it.
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        pull_collect(pull, pa(), bgw, parity);
      }
      const int dn = (d + 1) & 7;
      const char* from = d + 1 < 8 ? cur : nxt;
      f.ring[2 * (dn & 1)] = load_a16(from, rd, dn >> 2, 2 * (dn & 3));
      f.ring[2 * (dn & 1) + 1] = load_a16(from, rd, dn >> 2, 2 * (dn & 3) + 1);
      if (d < 4) {
        issue_a(nxt, src, kt_load, d);
        issue_b(nxt, src, kt_load, d);
      }
      // The background transfer has one place in the step, behind the step's last operand loads (loads
      // complete in issue order: a request that goes out to the peer's memory ahead of them would hold
      // all of them back): the piece requested during the step before (it arrived before that step's
      // barrier) is stored, then the next one is requested into the same registers.  One place, under one
      // test: every call site splits the step into basic blocks, and where they join the compiler waits
      // for more than the code needs.  Spread over three items (state read an item ahead of its use) the
      // same work cost a launch of 4096 x 4096 x 1024 1.3 us more.
      if constexpr (!kWithReduce) {
        if (d == 3 && pull.active) {
          pull_retire(pull, pa(), bgw, parity ^ 1);
          pull_issue(pull, pa(), bgw, parity);
        }
      }
      // acc[rb / 2][cb / 2] holds a 32 x 32 patch as four 16 x 16 blocks: registers 4 * q .. 4 * q + 3 are
      // block q = 2 * (rb % 2) + cb % 2 (acc_spot() is the lane's place in it).
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int rb = 2 * rp + r;
          f32x16& patch = acc[rb >> 1][cb >> 1];
          const int q = 2 * (rb & 1) + (cb & 1);
          f32x4 blk = {patch[4 * q], patch[4 * q + 1], patch[4 * q + 2], patch[4 * q + 3]};
          blk = Mfma<InT>::run16(f.fb[cb], f.ring[2 * (d & 1) + r], blk);
#pragma unroll
          for (int e = 0; e < 4; ++e) patch[4 * q + e] = blk[e];
        }
        if (rp == 3) {
          __builtin_amdgcn_sched_barrier(0);
          f.fb[cb] = load_b16(from, rd, dn >> 2, cb);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // A finished macro tile whose signal is still owed.  What the signal needs from memory (the TileGroup of
  // each plan tile under the macro tile) is fetched when the tile is finished, through the scalar path and
  // ahead of the wait for the tile's stores: looked up behind that wait, by the publishing lane and one plan
  // tile after the other, the table reads were a chain of trips to memory (1.7 us at 4096 x 4096 x 1024)
  // between the moment the last store had landed and the moment the signal went out.
  struct Owed {
    int where;        // (macro row << 16) | macro column; < 0: nothing owed
    int32_t tile[4];  // plan tile ids under the macro tile (-1: outside the grid)
    int32_t gid[4];   // their TileGroups (group mode)
  };
  static TCCL_D Owed nothing_owed() {
    Owed o;
    o.where = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) o.tile[i] = o.gid[i] = -1;
    return o;
  }
  // Where registers 4 * q .. 4 * q + 3 of acc[bi][bj] sit in the 32-row slab bi of the wave tile: row inside
  // the slab, first of four consecutive columns inside the wave's 64.  The MFMAs in use (16 x 16 x 32 for
  // 16-bit inputs, 16 x 16 x 128 for fp8) leave block q of the 32 x 32 patch there: row l % 16 of the block,
  // columns 4 * (l / 16) .. .
  struct Spot {
    int row, col;
  };
  static TCCL_D Spot acc_spot(int ln, int bj, int q) {
    return Spot{16 * (q >> 1) + (ln & 15), bj * 32 + 16 * (q & 1) + 4 * (ln >> 4)};
  }

  // Stores the tile and, when a push is asked for, sends it to the peers from the same LDS staging.
  template <int kPolicy>
  TCCL_D void epilogue(int row0, int col0, const f32x16 (&acc)[4][2]) const {
    constexpr int kEsz = sizeof(OutT);
    constexpr int kRowBytes = 64 * kEsz;
    constexpr int kChunks = kRowBytes / 16;
    constexpr int kPerChunk = 16 / kEsz;
    char* win = lds + wave * (32 * 64 * 4);  // 8 KiB per wave, 64 KiB in all: inside stage 0
    // The lane id is taken afresh: derived from the member, every store offset below is
    // invariant across tiles, gets hoisted out of the tile loop and occupies registers all
    // through the K loop.
    const int ln = fresh(lane);
    OutT* C = (OutT*)g.C + (int64_t)row0 * g.ldc + col0;
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc((void*)C, 0, 0xffffffffu, 0x00020000);
    // Fields are read through the argument block itself: a local copy would sit in scalar
    // registers all through the K loop.
    const auto* push = late_kernarg_ptr<PushArgs>(push_offset < 0 ? 0 : push_offset);
    const int push_world = push_offset >= 0 ? push->world : 0;
    // Each wavefront stages through its own 8 KiB window, and a wavefront's LDS operations
    // execute in the order issued: inside the loop nothing has to wait for another wavefront,
    // nor (as a __syncthreads() with its release fence would) for the previous slab's global
    // stores to land.  One barrier up front: every wavefront has left the K loop's stages.
    __syncthreads();
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const Spot at = acc_spot(ln, bj, q);
          OutT v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = to_out<OutT>(acc[bi][bj][4 * q + e] * g.alpha);
          const int byte = at.col * kEsz;
          const int chunk = (byte >> 4) ^ (at.row & 7);
          char* p = win + at.row * kRowBytes + chunk * 16 + (byte & 15);
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
        lrow[r] = wm * 128 + bi * 32 + row;
        lcol[r] = wn * 64 + chunk * kPerChunk;
        live[r] = row0 + lrow[r] < g.M && col0 + lcol[r] < g.N;
        if (live[r]) __builtin_amdgcn_raw_buffer_store_b128(v[r], rc, (uint32_t)((lrow[r] * g.ldc + lcol[r]) * kEsz), 0, kPolicy);
      }
      for (int t = 0; t < push_world; ++t) {
        if (t == push->rank) continue;
        const int64_t push_ld = push->ld;
        const int col_lo = push->col_lo, col_hi = push->col_hi;
        const int64_t delta = table(push->heap_bases, t) - table(push->heap_bases, push->rank);
        char* base = (char*)g.C + delta + ((int64_t)row0 * push_ld + col0 + push->col_shift) * kEsz;
        const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xffffffffu, 0x00020000);
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
          const int col = col0 + lcol[r];
          if (live[r] && col >= col_lo && col < col_hi)
            __builtin_amdgcn_raw_buffer_store_b128(v[r], rt, (uint32_t)((lrow[r] * push_ld + lcol[r]) * kEsz), 0, kCoherent);
        }
      }
    }
  }

  typedef const __attribute__((address_space(4))) ReduceArgs* ReducePtr;

  // Epilogue of a tile whose rows this rank owns, reduce-scatter with the partial kept in
  // registers: each 32-row slab is rounded to the partial type and staged through LDS exactly
  // as epilogue() does, but instead of being stored it takes the peers' partials of the same
  // 16-byte chunks (ascending rank: the owner's addend, this one, comes first) in fp32, is
  // rounded once to the output type and lands in the output shard.  The bytes equal those of
  // storing the partial and reducing it afterwards; 64 MiB less is written and read at c3.
  //
  // `owner` is the rank whose shard the rows belong to.  For owner != rank (two ranks, the
  // peer's reduction carried out on its behalf under single-GPU emulation) the partial is
  // stored as well, as that peer would read it, and the sum lands in the owner's slice; with
  // two addends the order of the sum does not matter.
  TCCL_D void epilogue_reduce(ReducePtr ra, int row0, int col0, const f32x16 (&acc)[4][2], int owner, bool store_partial) const {
    constexpr int kEsz = sizeof(OutT);
    constexpr int kRowBytes = 64 * kEsz;
    constexpr int kChunks = kRowBytes / 16;
    constexpr int kPerChunk = 16 / kEsz;
    constexpr int kRounds = (32 * kChunks) / 64;
    char* win = lds + wave * (32 * 64 * 4);
    const int ln = fresh(lane);  // as in epilogue(): keeps the offsets below out of the K loop's registers
    const int world = ra->world, rank = ra->rank;
    const int64_t my_base = ra->heap_bases[rank];
    const int64_t tile_off = ((int64_t)row0 * g.ldc + col0) * kEsz;
    const uint32_t ld_out = (uint32_t)ra->ld_out;
    const __amdgpu_buffer_rsrc_t r_out = window((int64_t)(uintptr_t)ra->out + (ra->heap_bases[owner] - my_base) +
                                                ((int64_t)(row0 - owner * ra->shard_rows) * ra->ld_out + col0) * 2);
    const __amdgpu_buffer_rsrc_t r_mine = window((int64_t)(uintptr_t)g.C + tile_off);
    const bool bf = ra->out_bf16 != 0;
    // Each wavefront stages through its own 8 KiB window, and a wavefront's LDS operations
    // execute in the order issued: inside the loop nothing has to wait for another wavefront,
    // nor (as a __syncthreads() with its release fence would) for the previous slab's global
    // stores to land.  One barrier up front: every wavefront has left the K loop's stages.
    __syncthreads();
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const Spot at = acc_spot(ln, bj, q);
          OutT v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = to_out<OutT>(acc[bi][bj][4 * q + e] * g.alpha);
          const int byte = at.col * kEsz;
          const int chunk = (byte >> 4) ^ (at.row & 7);
          char* p = win + at.row * kRowBytes + chunk * 16 + (byte & 15);
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
      // kBatch chunks per lane at a time: the accumulators of the later slabs are still live.
      constexpr int kBatch = kRounds > 4 ? 4 : kRounds;
#pragma unroll
      for (int r0 = 0; r0 < kRounds; r0 += kBatch) {
        uint32_t src[kBatch], dst[kBatch];
        bool live[kBatch];
        float sum[kBatch][8];
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
          const int idx = ln + 64 * (r0 + r);
          const int row = idx / kChunks, chunk = idx % kChunks;
          const u32x4 v = *(const u32x4*)(win + row * kRowBytes + ((chunk ^ (row & 7)) * 16));
          const int lrow = wm * 128 + bi * 32 + row, lcol = wn * 64 + chunk * kPerChunk;
          live[r] = row0 + lrow < g.M && col0 + lcol < g.N;
          // idle lanes re-read the tile's first chunk and store nothing
          src[r] = live[r] ? (uint32_t)((lrow * g.ldc + lcol) * kEsz) : 0u;
          dst[r] = (uint32_t)((lrow * ld_out + lcol) * 2);
          if (store_partial && live[r]) __builtin_amdgcn_raw_buffer_store_b128(v, r_mine, src[r], 0, kCoherent);
          int n;
          unpack(v, sum[r], n);
        }
        for (int p = 0; p < world; ++p) {
          if (p == rank) continue;
          const __amdgpu_buffer_rsrc_t r_peer = window((int64_t)(uintptr_t)g.C + (ra->heap_bases[p] - my_base) + tile_off);
          u32x4 addend[kBatch];
#pragma unroll
          for (int r = 0; r < kBatch; ++r) addend[r] = ld16<kCoherent>(r_peer, src[r]);
#pragma unroll
          for (int r = 0; r < kBatch; ++r) {
            float f[8];
            int n;
            unpack(addend[r], f, n);
#pragma unroll
            for (int e = 0; e < kPerChunk; ++e) sum[r][e] += f[e];
          }
        }
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
          if constexpr (kPerChunk == 4) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            u32x2 o;
            if (bf) {
              const __bf16 h[4] = {(__bf16)sum[r][0], (__bf16)sum[r][1], (__bf16)sum[r][2], (__bf16)sum[r][3]};
              __builtin_memcpy(&o, h, 8);
            } else {
              const _Float16 h[4] = {(_Float16)sum[r][0], (_Float16)sum[r][1], (_Float16)sum[r][2], (_Float16)sum[r][3]};
              __builtin_memcpy(&o, h, 8);
            }
            if (live[r]) __builtin_amdgcn_raw_buffer_store_b64(o, r_out, dst[r], 0, kStreaming);
          } else {
            const u32x4 o = bf ? pack8<__bf16>(sum[r]) : pack8<_Float16>(sum[r]);
            if (live[r]) st16<kStreaming>(r_out, dst[r], o);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_sched_barrier(0);  // one slab's addends at a time: the accumulators are still live
    }
  }

  template <int kPolicy>
  // `unpublished` carries a finished tile whose signal is still owed (-1: none): instead of
  // waiting for its stores to land right after its epilogue, the next tile's prologue, which
  // has to wait for its first operands anyway, publishes it.
  // `ahead`: `src` describes this tile and its first operands are already requested (a workgroup's first tile: run()).
  TCCL_D void macro_tile(const SignalArgs& s, int mm, int mn, PullState& pull, Owed& unpublished, Source& src, bool ahead) const {
    const int row0 = mm * kMacro, col0 = mn * kMacro;
    if (!ahead) {
      src = make_source(row0, col0);
      __syncthreads();  // the previous tile's epilogue has left LDS
#pragma unroll
      for (int i = 0; i < 4; ++i) issue_piece(lds, src, 0, i);
    }
    // K steps are taken in pairs so that each call names its two stages statically and the
    // accumulators flow through one straight loop body.  An odd step count is rounded up: the
    // extra step (like the final look-ahead load) lies wholly past K and reads zeros.
    const int ksteps = ((g.K + kStepK - 1) / kStepK + 1) & ~1;
    // The accumulators are cleared two registers per instruction (64-bit moves): 128 single moves per
    // wavefront, two wavefronts per SIMD, were half a microsecond of a tile's start.
    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        typedef double f64x8 __attribute__((ext_vector_type(8)));
        f64x8 z;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          double d;
          asm volatile("v_mov_b64 %0, 0" : "=v"(d));
          z[e] = d;
        }
        acc[i][j] = __builtin_bit_cast(f32x16, z);
      }
    const Reader rd = make_reader();
    wait_vmem();  // the first operands are there, and so is everything the previous tile stored
    __syncthreads();
    publish_owed(s, unpublished);
    pull_collect(pull, pa(), bgw, 0);  // the counters fetched before this tile (no piece is pending here)
    if constexpr (kFp8) {
      Frags8 f;
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) f.fb[cb] = load_b8(lds, rd, cb);
      f.ring[0] = load_a8(lds, rd, 0);
      for (int kt = 0; kt < ksteps; kt += 2) {
        follow_shards(src, kt + 1);
        k_step8(lds, lds1, src, rd, kt + 1, acc, f, pull, 0);
        follow_shards(src, kt + 2);
        k_step8(lds1, lds, src, rd, kt + 2, acc, f, pull, 1);
      }
    } else {
      Frags f;
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) f.fb[cb] = load_b16(lds, rd, 0, cb);
      f.ring[0] = load_a16(lds, rd, 0, 0);
      f.ring[1] = load_a16(lds, rd, 0, 1);
      for (int kt = 0; kt < ksteps; kt += 2) {
        follow_shards(src, kt + 1);
        k_step16(lds, lds1, src, rd, kt + 1, acc, f, pull, 0);
        follow_shards(src, kt + 2);
        k_step16(lds1, lds, src, rd, kt + 2, acc, f, pull, 1);
      }
      pull_retire(pull, pa(), bgw, 1);  // the last step's piece: nothing is carried through the epilogue
    }
    if constexpr (kWithReduce) {
      // Rows this rank owns, partial kept in registers: the peers' partials are added in the
      // epilogue and the tile's partial is never stored (it is still published: the counters
      // keep one meaning).  If the wait for the peers expires the partial is stored as usual.
      const ReducePtr ra = late_kernarg_ptr<ReduceArgs>(reduce_offset);
      if (ra->active && ra->own_in_registers) {
        const int owner = row0 / ra->shard_rows;
        // The other owner's rows, reduced on its behalf (emulation, two ranks): the partial is
        // stored as that owner would read it, and the same registers enter its sum (the staged,
        // rounded values: the bits of a sum that read the stored partial back).
        // (The fp8 kernels once read the partial back instead: this path cost them registers they kept in
        // scratch memory inside the K loops, +4 % at 16384x4096x2048; with the wavefront number and the LDS
        // addresses in scalar registers they have the room, and the saved read-back is worth 6 %.)
        const bool for_peer = owner != ra->rank && ra->emulate_peer && ra->world == 2;
        if ((owner == ra->rank || for_peer) && reduce_wait(ra, s, mm, mn)) {
          epilogue_reduce(ra, row0, col0, acc, owner, for_peer);
          unpublished = publish_lookup(s, mm, mn);
          return;
        }
      }
    }
    epilogue<kPolicy>(row0, col0, acc);
    if constexpr (kPolicy != 0) {
      unpublished = publish_lookup(s, mm, mn);
      if constexpr (!kWithReduce) return;
      wait_vmem();  // the tile's write-through stores have landed
      __syncthreads();
      publish_owed(s, unpublished);
      if constexpr (kWithReduce) {
        const ReducePtr ra = late_kernarg_ptr<ReduceArgs>(reduce_offset);
        if (ra->active) {
          const int owner = row0 / ra->shard_rows;
          if ((owner == ra->rank || ra->emulate_peer) && reduce_wait(ra, s, mm, mn)) reduce_tile(ra, row0, col0, owner);
        }
      }
    }
  }

  TCCL_D Owed publish_lookup(const SignalArgs& s, int mm, int mn) const {
    Owed o = nothing_owed();
    o.where = (mm << 16) | mn;
    if (s.mode == kSignalNone) return o;
    const int per_m = g.block_m == kMacro ? 1 : 2, per_n = g.block_n == kMacro ? 1 : 2;  // plan tiles are 128 or 256 on a side here
    const int tm0 = mm * per_m, tn0 = mn * per_n;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dm = i >> 1, dn = i & 1;
      const int tm = tm0 + dm, tn = tn0 + dn;
      if (dm < per_m && dn < per_n && tm < g.tile_rows && tn < g.tile_cols) o.tile[i] = tile_id_of(tm, tn, g.tile_rows, g.tile_cols, g.group_m);
    }
    if (s.mode != kSignalTile) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o.tile[i] >= 0) o.gid[i] = table(s.group_table, o.tile[i]);
    }
    return o;
  }

  // Call behind a wait for this wavefront's stores and a barrier: every store of the owed tile has landed.
  // Plan tiles of one TileGroup are summed up and the group gets one add (concurrent adds to one word serialise).
  TCCL_D void publish_owed(const SignalArgs& s, Owed& o) const {
    if (o.where < 0) return;
    if (tid == 0 && s.mode != kSignalNone) {
      if (s.mode == kSignalTile) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (o.tile[i] >= 0) tile_publish(s.locks, o.tile[i], s.epoch);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (o.tile[i] < 0) continue;
          bool counted = false;  // an earlier plan tile of the same group has taken this one along
          int count = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (o.tile[j] < 0 || o.gid[j] != o.gid[i]) continue;
            if (j < i) counted = true;
            ++count;
          }
          if (!counted) add_to_group(s, o.gid[i], count);
        }
      }
    }
    o.where = -1;
  }

  // Are the peers' partials of the plan tiles under macro tile (mm, mn) published?  One lane
  // waits (bounded); the verdict travels through an LDS word of the idle stage.
  TCCL_D bool reduce_wait(ReducePtr ra, const SignalArgs& s, int mm, int mn) const {
    if (ra->peers_resident) return true;  // the same for every wavefront
    volatile int* verdict = (volatile int*)lds1;
    if (tid == 0) {
      bool ok = true;
      const int64_t deadline = now_ticks() + ra->spin_ticks;
      const int64_t mine = ra->heap_bases[ra->rank];
      const int tm0 = mm * (kMacro / g.block_m), tn0 = mn * (kMacro / g.block_n);
      for (int p = 0; p < ra->world && ok; ++p) {
        if (p == ra->rank) continue;
        const int64_t delta = ra->heap_bases[p] - mine;
        int waited_group = -1;
        for (int dm = 0; dm < kMacro / g.block_m && ok; ++dm)
          for (int dn = 0; dn < kMacro / g.block_n && ok; ++dn) {
            const int tm = tm0 + dm, tn = tn0 + dn;
            if (tm >= g.tile_rows || tn >= g.tile_cols) continue;
            const int tile_id = tile_id_of(tm, tn, g.tile_rows, g.tile_cols, g.group_m);
            if (s.mode == kSignalTile) {
              ok = tile_wait_ge<true>((const int32_t*)((const char*)ra->locks + delta), tile_id, ra->epoch, deadline);
            } else {
              const int gi = s.group_table[tile_id];
              if (gi == waited_group) continue;
              waited_group = gi;
              ok = tile_wait_ge<true>((const int32_t*)((const char*)ra->counter + delta), gi, (int32_t)((uint32_t)ra->epoch * (uint32_t)ra->tile_counts[gi]), deadline);
            }
          }
      }
      if (!ok && ra->fault) *ra->fault = 1;
      *verdict = ok ? 1 : 0;
    }
    __syncthreads();
    const bool all_ok = *verdict != 0;
    __syncthreads();
    return all_ok;
  }

  // out_owner[tile] = cast(sum over ranks of partial_rank[tile]); the whole workgroup streams
  // the tile in 16-byte units, kUnroll units per thread in flight.
  TCCL_D void reduce_tile(ReducePtr ra, int row0, int col0, int owner) const {
    constexpr int kEsz = sizeof(OutT);
    constexpr int kE = 16 / kEsz;
    constexpr int kUnroll = 4;
    const int rows = g.M - row0 < kMacro ? g.M - row0 : kMacro;
    const int cols = g.N - col0 < kMacro ? g.N - col0 : kMacro;
    const int upr = cols / kE;  // N is a multiple of 8, so a row holds whole units
    const int total = rows * upr;
    const int world = ra->world, rank = ra->rank;
    const int64_t my_base = ra->heap_bases[rank];
    const int64_t tile_off = ((int64_t)row0 * g.ldc + col0) * kEsz;
    const int64_t ld_out = ra->ld_out;
    const __amdgpu_buffer_rsrc_t r_mine = window((int64_t)(uintptr_t)g.C + tile_off);
    const __amdgpu_buffer_rsrc_t r_out = window((int64_t)(uintptr_t)ra->out + (ra->heap_bases[owner] - my_base) +
                                                ((int64_t)(row0 - owner * ra->shard_rows) * ld_out + col0) * 2);
    const bool bf = ra->out_bf16 != 0;
    for (int u0 = fresh(tid); u0 < total; u0 += kThreads256 * kUnroll) {
      u32x4 mine[kUnroll];
      uint32_t src[kUnroll], dst[kUnroll];
      bool live[kUnroll];
      float sum[kUnroll][8];
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int u = u0 + k * kThreads256;
        live[k] = u < total;
        const uint32_t uu = live[k] ? (uint32_t)u : 0u;  // idle lanes re-read the first unit and store nothing
        const uint32_t r = uu / (uint32_t)upr, c = uu - r * (uint32_t)upr;
        src[k] = (uint32_t)((r * g.ldc + c * kE) * kEsz);
        dst[k] = (uint32_t)((r * ld_out + c * kE) * 2);
        mine[k] = ld16<0>(r_mine, src[k]);  // written by this workgroup itself: a plain load sees it
      }
      for (int step = 0; step < world; ++step) {
        // owner first, then the other ranks in ascending order
        const int p = step == 0 ? owner : (step - 1 < owner ? step - 1 : step);
        u32x4 addend[kUnroll];
        if (p == rank) {
#pragma unroll
          for (int k = 0; k < kUnroll; ++k) addend[k] = mine[k];
        } else {
          const __amdgpu_buffer_rsrc_t r_peer = window((int64_t)(uintptr_t)g.C + (ra->heap_bases[p] - my_base) + tile_off);
#pragma unroll
          for (int k = 0; k < kUnroll; ++k) addend[k] = ld16<kCoherent>(r_peer, src[k]);
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
          float f[8];
          int n;
          unpack(addend[k], f, n);
#pragma unroll
          for (int e = 0; e < 8; ++e) sum[k][e] = step == 0 ? f[e] : sum[k][e] + f[e];
        }
      }
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        if constexpr (kE == 4) {
          typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
          u32x2 o;
          if (bf) {
            const __bf16 h[4] = {(__bf16)sum[k][0], (__bf16)sum[k][1], (__bf16)sum[k][2], (__bf16)sum[k][3]};
            __builtin_memcpy(&o, h, 8);
          } else {
            const _Float16 h[4] = {(_Float16)sum[k][0], (_Float16)sum[k][1], (_Float16)sum[k][2], (_Float16)sum[k][3]};
            __builtin_memcpy(&o, h, 8);
          }
          if (live[k]) __builtin_amdgcn_raw_buffer_store_b64(o, r_out, dst[k], 0, kStreaming);
        } else {
          const u32x4 o = bf ? pack8<__bf16>(sum[k]) : pack8<_Float16>(sum[k]);
          if (live[k]) st16<kStreaming>(r_out, dst[k], o);
        }
      }
    }
  }

  TCCL_D void add_to_group(const SignalArgs& s, int group, int count) const {
    // The previous value is only needed for the trace stamp.  Without it the add is issued and
    // forgotten: waiting for the old value costs a round trip that grows with the number of
    // workgroups adding to the same word at the same moment (all of them, at c1).
    if (s.trace_ready_clock) {
      const int32_t prev = tile_signal_add<true>(s.counter, group, count);
      if (prev + count == s.epoch * s.tile_counts[group]) s.trace_ready_clock[group] = now_ticks();
    } else {
      (void)tile_signal_add<true>(s.counter, group, count);
    }
  }

  // n / d for n >= 0, d > 0.  The divisors of the slot -> tile map are powers of two for most shapes (a
  // shift), and an unsigned division is half the instructions of a signed one: the map runs at the very
  // start of a kernel, where one wavefront per SIMD executes a few hundred scalar instructions with
  // nothing to overlap them, ahead of the first operand request.
  static TCCL_D uint32_t quotient(uint32_t n, uint32_t d) {
    if ((d & (d - 1)) == 0) return n >> (31 - __builtin_clz(d));
    // The divisor is hidden from the optimiser here: it would otherwise form the reciprocals of every
    // divisor once, ahead of the tile loop (i.e. at the kernel's start), whether this path is taken or not.
    asm volatile("" : "+s"(d));
    return n / d;
  }
  // tile_for_slot() followed by macro_coords() and the row shift, in that arithmetic.
  static TCCL_D TileCoord tile_of_slot(int slot, int total, const Macro& m) {
    const uint32_t block = (uint32_t)(m.xcds * m.span);
    uint32_t id = (uint32_t)slot;
    const uint32_t base = quotient(id, block) * block;
    if (m.xcds > 1 && base + block <= (uint32_t)total) {
      const uint32_t r = id - base, q = quotient(r, (uint32_t)m.xcds);
      id = base + (r - q * (uint32_t)m.xcds) * (uint32_t)m.span + q;
    }
    const uint32_t per_band = (uint32_t)(m.rows_per_band * m.cols);
    const uint32_t band = quotient(id, per_band);
    const uint32_t first = band * (uint32_t)m.rows_per_band;
    const uint32_t left = (uint32_t)m.rows - first;
    const uint32_t height = left < (uint32_t)m.rows_per_band ? left : (uint32_t)m.rows_per_band;
    const uint32_t within = id - band * per_band;
    const uint32_t col = quotient(within, height);
    TileCoord c;
    c.m = (int)(first + (within - col * height)) + m.row_shift;
    c.n = (int)col;
    if (c.m >= m.rows) c.m -= m.rows;
    return c;
  }

  TCCL_D void run(const SignalArgs& s, const Macro& m, int wg, int num_wgs) const {
    const int total = m.rows * m.cols;
    // A workgroup's first operand requests go out before anything else it sets up: a kernel's start is
    // a few hundred scalar and address instructions of one wavefront per SIMD with nothing to overlap
    // them, followed by a trip to memory, and only what those requests themselves need should come
    // ahead of that trip.  The rest (the background transfer's state and its first counter fetch, which
    // is a chain of dependent scalar loads; whatever the optimiser computes once for all tiles) runs
    // while the operands are in flight.  LDS is free at this point: no barrier.
    // (A workgroup beyond the last tile requests some tile's operands and never uses them.)
    const TileCoord c0 = tile_of_slot(wg < total ? wg : total - 1, total, m);
    Source src = make_source(c0.m * kMacro, c0.n * kMacro);
#pragma unroll
    for (int i = 0; i < 4; ++i) issue_piece(lds, src, 0, i);
    __builtin_amdgcn_sched_barrier(0);
    PullState pull = pull_begin(pa(), wg, num_wgs);
    pull_prime(pull, pa(), bgw);
    Owed unpublished = nothing_owed();
    // A launch with at most one tile per workgroup does not enter the tile loop: what the compiler computes
    // once for all tiles of a loop it computes ahead of the loop, i.e. between a workgroup's first operand
    // requests and its first barrier, where a fused kernel already has more to do than the requests take to
    // land (4096 x 4096 x 1024: 0.35 us per launch).  With several tiles per workgroup the loop form is the
    // faster one (the same values would be computed between the first tile and the second).
    if ((push_offset >= 0 || pull_offset >= 0 || reduce_offset >= 0) && total <= num_wgs) {  // (the plain GEMM has next to nothing to hoist)
      if (wg < total) {
        if (s.mode == kSignalNone && push_offset < 0)
          macro_tile<0>(s, c0.m, c0.n, pull, unpublished, src, true);
        else
          macro_tile<kCoherent>(s, c0.m, c0.n, pull, unpublished, src, true);
      }
    } else {
      for (int slot = wg; slot < total; slot += num_wgs) {
        const TileCoord c = tile_of_slot(slot, total, m);
        if (s.mode == kSignalNone && push_offset < 0)
          macro_tile<0>(s, c.m, c.n, pull, unpublished, src, slot == wg);
        else
          macro_tile<kCoherent>(s, c.m, c.n, pull, unpublished, src, slot == wg);
      }
    }
    if (unpublished.where >= 0) {  // the last tile: nothing follows that would wait for its stores
      wait_vmem();
      __syncthreads();
      publish_owed(s, unpublished);
    }
    pull_finish(pull, pa(), bgw, num_wgs);
  }
};
#endif  // __HIP_DEVICE_COMPILE__

}  // namespace tccl
