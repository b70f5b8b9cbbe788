/*
 * tileccl_hip.h -- C ABI of libtileccl_hip.so (gfx950 / MI355X).
 *
 * The reference is pure Python + Triton: its host code reaches the GPU through Triton
 * launches (`kernel[grid](...)`) and, for the runtime, through ctypes into libamdhip64
 * (/root/reference/tileccl/backends/hip.py:67-186).  Each entry point below replaces
 * one of those launch sites with a hand-written HIP kernel; the comment on each names
 * the reference launch it stands in for.
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t, or a negative
 *     tccl_status; tccl_last_error_string() describes the last failure on the calling
 *     thread.  Nothing throws, nothing touches Python.
 *   - all pointers inside descriptors are DEVICE pointers valid for the duration of the
 *     call's stream work; the library never owns tensor memory.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Launches
 *     are asynchronous; no entry point synchronises the device.
 *   - matrices are row-major; leading dimensions are in elements.
 *   - not re-entrant across host threads for one device (same as the reference, which
 *     keeps process-global context state: tileccl/__init__.py:228).
 */
#ifndef TILECCL_HIP_H
#define TILECCL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TCCL_ABI_VERSION 1
#define TCCL_MAX_WORLD 8

typedef enum tccl_status {
  TCCL_OK = 0,
  TCCL_ERR_INVALID = -1,     /* bad argument / descriptor */
  TCCL_ERR_UNSUPPORTED = -2, /* layout, dtype or shape this build has no kernel for */
  TCCL_ERR_NO_DEVICE = -3,
  TCCL_ERR_TIMEOUT = -4      /* a bounded device-side wait expired (see tccl_read_fault) */
} tccl_status;

typedef enum tccl_dtype {
  TCCL_F16 = 0,
  TCCL_BF16 = 1,
  TCCL_F32 = 2,
  TCCL_F8E4M3 = 3 /* OCP e4m3fn, max 448: the fp8 format of gfx950 MFMA */
} tccl_dtype;

/* S0 bulk / S1 tile-by-tile / S2 TileGroup (reference README.md:66-84). */
typedef enum tccl_variant {
  TCCL_S0_BULK = 0,
  TCCL_S1_TILE = 1,
  TCCL_S2_TILEGROUP = 2
} tccl_variant;

/* Transfer directions carried out by one launch (bit mask).  PUSH: this rank's rows go
 * to the peers (reference tileccl_v2/transport.py:18 CommMode.PUSH).  PULL: the peers'
 * rows are read into this rank's slice (CommMode.PULL).  On one GPU, PUSH|PULL runs both
 * halves of a two-rank exchange through the same HBM. */
#define TCCL_DIR_PUSH 1
#define TCCL_DIR_PULL 2

typedef struct tccl_device_info {
  int32_t compute_units;   /* CUs (256 on MI355X) */
  int32_t clock_khz;       /* engine clock */
  int32_t lds_bytes;       /* LDS per workgroup limit */
  int32_t wavefront;       /* 64 */
  int32_t xcds;            /* accelerator dies sharing one L2 each (8 on MI355X) */
  int32_t reserved[3];
  char arch[64];           /* "gfx950..." */
} tccl_device_info;

/* ---- one GEMM: C[M,N] = alpha * A[M,K] @ B[K,N], fp32 accumulate ------------------
 * Stands in for gemm_kernel (tileccl/kernels/gemm.py:53-167) and the GEMM bodies of the
 * patterns (patterns/bulk_sync.py:162-238, wg_specialized.py:263-310).
 * A must be k-contiguous (lda = row stride), B n-contiguous (ldb = row stride).
 * Plan tiles are block_m x block_n; tile ids follow the group_m swizzle of the
 * reference GEMM (kernels/gemm.py:118-123) so that they index group_table / locks. */
typedef struct tccl_gemm_desc {
  const void* A;
  const void* B;
  void* C;
  int32_t M, N, K;
  int64_t lda, ldb, ldc;
  int32_t in_dtype;  /* tccl_dtype of A and B: F16, BF16 or F8E4M3 */
  int32_t out_dtype; /* tccl_dtype of C: F16, BF16 or F32 */
  float alpha;       /* applied to the fp32 accumulator (fp8: scale_a * scale_b) */
  int32_t block_m, block_n, group_m; /* plan tile and swizzle band: 128/128/8 or 256/128/8 */
  int32_t num_wgs;   /* GEMM workgroups; 0 = library default for the device */
  int32_t macro_tile; /* output tile one workgroup computes: 0 = choose by shape, 128, or 256 */
  int32_t flags;      /* TCCL_GEMM_* bits */
  /* Column shards stacked as row blocks (the rank_major_column_shards layout of
   * tileccl.ops.gemm_reducescatter, ops.py:315,646).  0 or 1: plain GEMM.  w > 1: A has M/w
   * rows and B has w*N columns; row block q of C (rows [q*M/w, (q+1)*M/w)) is
   * A @ B[:, q*N:(q+1)*N].  M/w must be a multiple of the plan tile's rows. */
  int32_t column_shards;
} tccl_gemm_desc;

/* tccl_gemm_reducescatter, variants S1 / S2 on the 256 x 256 tile with shards of whole tiles:
 * the partial of the rows this rank owns stays in the accumulators, takes the peers' partials
 * in the GEMM epilogue and is never stored to gemm->C (those rows of C keep their old
 * contents); the output is bit-identical to storing and reducing.  Ignored elsewhere.
 * (The reference's fused proof kernels have no counterpart in its tree; tile_reduce_scatter,
 * primitives/collectives.py:730-783, always reads a stored partial.) */
#define TCCL_GEMM_OWN_ROWS_IN_REGISTERS 1
/* B is k-major: element (k, n) is at B[n * ldb + k], i.e. B is the `.t()` view of an (N, K)
 * tensor (the layout of a linear layer's weight); ldb is then the pitch between columns and must
 * be >= K.  The reference's GEMM takes arbitrary strides (kernels/gemm.py:139-151); this and the
 * row-major form are the two it meets in practice.  With column_shards = w, B has w * N columns. */
#define TCCL_GEMM_B_KMAJOR 2

#define TCCL_RS_EMULATE_PEERS 1
#define TCCL_RS_PEERS_RESIDENT 2

/* ---- per-launch synchronisation words ------------------------------------------------
 * Stands in for the lock tensor of WGSpecializedPattern (wg_specialized.py:104-124) and
 * for TileGroupSignalState (tileccl_v2/signal.py:14-40).
 *   locks      int32[total_tiles]   S1: launch number `epoch` is stored per finished tile; a tile is ready
 *                                   once its word has reached `epoch` (stands in for tile_signal /
 *                                   tile_wait, sync/primitives.py:357-414, without consuming the flag)
 *   group_table int32[total_tiles]  S2: swizzled tile id -> group id (tile_group.py:214-241)
 *   counter    int32[n_groups]      S2: tile_signal_add / tile_wait_ge (tileccl_v2/ipc.py:231-254)
 *   barrier    int32[n_groups]      S2: finished communication tasks (or workgroups, see below) per group
 *   trace_*    optional device-clock stamps (signal.py:18-24); NULL to skip
 * locks, counter and barrier live in the symmetric heap, so a peer's copy sits at the
 * same offset in the peer's slice.  The host zeroes them once
 * (TileGroupSignalState.reset, signal.py:32-40; wg_specialized.py:122-123 zeroes its locks per
 * call); `epoch` lets repeated launches reuse them without a reset: a tile is ready when
 * locks[t] >= epoch, a group when counter[g] >= epoch * tile_counts[g].  S1 and S2 launches
 * on the same words number their launches separately (each counts the launches that wrote
 * its words), and ranks that wait on each other must pass the same number. */
typedef struct tccl_sync_desc {
  int32_t* locks;
  const int32_t* group_table;
  int32_t* counter;
  int32_t* barrier;
  int32_t n_groups;
  int32_t epoch; /* >= 1: the number of this launch among those of its variant on these words */
  const int32_t* row_starts; /* int32[n_groups], rows relative to the GEMM's C */
  const int32_t* row_ends;   /* clamped to M */
  const int32_t* tile_counts;
  int32_t* trace_comm_counter;  /* int32[n_groups] or NULL */
  int64_t* trace_start_clock;   /* int64[1] or NULL */
  int64_t* trace_ready_clock;   /* int64[n_groups] or NULL */
  int64_t* trace_done_clock;    /* int64[n_groups] or NULL */
  int64_t* fault;               /* int64[1] or NULL: set non-zero if a bounded wait expired */
  int64_t spin_limit_ns;        /* bound of every device-side wait; 0 = library default (2 s) */
} tccl_sync_desc;

/* ---- symmetric heap view -------------------------------------------------------------
 * heap_bases is the int64[world_size] device array of slice base addresses
 * (tileccl_v2/heap.py:143-145, memory/symmetric_heap.py:929-938); rank / world_size as
 * in the reference context.  translate(ptr, to) = heap_bases[to] + (ptr - heap_bases[rank])
 * (memory/translation.py:39-99). */
typedef struct tccl_heap_view {
  const int64_t* heap_bases;
  int32_t rank;
  int32_t world_size;
} tccl_heap_view;

/* ---- all-scatter placement (tileccl.ops.gemm_allscatter) ------------------------------
 * The four integers of PatternExecutionSpec (patterns/contracts.py:206-215) consumed by
 * scatter_tile_to_peer (patterns/_helpers.py:145-157): columns
 * [src_col_offset, src_col_offset+cols) of the local C go to every peer's C at
 * row*dst_ld + dst_col_offset + (col - src_col_offset). */
typedef struct tccl_scatter_desc {
  int32_t src_col_offset;
  int32_t cols;
  int32_t dst_ld;
  int32_t dst_col_offset;
} tccl_scatter_desc;

/* ---- transport knobs (tileccl_v2/transport.py:23-53, wg.py:10-51) --------------------- */
typedef struct tccl_transport_desc {
  int32_t directions;   /* TCCL_DIR_* mask */
  int32_t copy_elems;   /* elements per copy task */
  int32_t reduce_elems; /* elements per reduce task (0: use copy_elems) */
  int32_t num_comm_wgs; /* communication workgroups of a fused launch; 0 = default */
} tccl_transport_desc;

/* ---- runtime -------------------------------------------------------------------------*/
int tccl_abi_version(void);
const char* tccl_last_error_string(void);
/* backends/hip.py:458-490 get_device_properties (compute_units et al.). */
int tccl_device_query(int device, tccl_device_info* out);
/* Pure host helper: swizzled tile id -> (tile_m, tile_n); same code the kernels run
 * (kernels/gemm.py:118-123).  Exposed so CPU tests can pin the device-side index math. */
int tccl_tile_coords(int32_t tile_id, int32_t tile_rows, int32_t tile_cols, int32_t group_m,
                     int32_t* tile_m, int32_t* tile_n);
/* Pure host helper: launch slot -> swizzled tile id after the XCD-aware remap (each XCD
 * takes `span` consecutive ids out of every block of xcds*span). */
int tccl_tile_for_slot(int32_t slot, int32_t total_tiles, int32_t xcds, int32_t span, int32_t* tile_id);

/* ---- symmetric heap: one hipMalloc arena cut into world_size slices -------------------
 * Replaces one torch.empty per rank + IPC/peer mapping (tileccl_v2/heap.py:137,225-264;
 * memory/symmetric_heap.py:239-343).  bases_out: host int64[world_size]. */
int tccl_heap_create(size_t slice_bytes, int world_size, void** arena_out, int64_t* bases_out);
int tccl_heap_destroy(void* arena);

/* ---- small device utilities ---------------------------------------------------------- */
/* Fill kernel (never hipMemsetAsync): signal reset, signal.py:32-40. */
int tccl_fill_i32(int32_t* words, int64_t n, int32_t value, void* stream);
/* Strided 2-D matrix (strides in elements, >= 0) -> dense rows of pitch ld_dst, zero-filled from
 * (rows, cols) up to (dst_rows, dst_cols).  The reference's GEMM addresses its operands with any
 * stride_am / stride_ak / stride_bk / stride_bn (kernels/gemm.py:63-66,139-151); the MFMA kernels here
 * read 16-byte row vectors, so a host binding packs an operand of any other layout (a transposed
 * A, a column slice, a K that is no multiple of the vector) with this launch first.  elem_bytes 1, 2, 4. */
int tccl_pack_matrix(const void* src, int64_t stride_row, int64_t stride_col, int32_t rows, int32_t cols,
                     void* dst, int64_t ld_dst, int32_t dst_rows, int32_t dst_cols, int32_t elem_bytes,
                     void* stream);
/* Single-word primitives, one launch each, for tests of the device semantics
 * (sync/primitives.py:357-500, tileccl_v2/ipc.py:137-254).  result: device int32[1]. */
int tccl_prim_signal(int32_t* locks, int32_t index, void* stream);
int tccl_prim_signal_add(int32_t* words, int32_t index, int32_t value, int32_t* result, void* stream);
int tccl_prim_try_wait(int32_t* locks, int32_t index, int32_t max_spins, int32_t consume,
                       int32_t* result, void* stream);
int tccl_prim_wait_ge(int32_t* words, int32_t index, int32_t threshold, int64_t spin_limit_ns,
                      int32_t* result, void* stream);

/* ---- GEMM alone ------------------------------------------------------------------------ */
int tccl_gemm(const tccl_gemm_desc* gemm, void* stream);

/* ---- communication phases alone (the second kernel of S0) ------------------------------
 * tccl_scatter_cols: BulkSyncPattern._scatter_kernel (patterns/bulk_sync.py:242-299).
 * elem_bytes: size of one element of C. */
int tccl_scatter_cols(const void* C, int32_t M, int64_t ldc, int32_t elem_bytes,
                      const tccl_scatter_desc* scatter, const tccl_heap_view* heap, void* stream);
/* tccl_exchange_rows: the row-block exchange of GEMM-output AllGather
 * (tile_allgather layout [block_rank0 | block_rank1 | ...], primitives/collectives.py:613-663).
 * `out` is this rank's gathered output (world*rows_per_rank x N, leading dim ld) in its
 * slice; rank r's block occupies rows [r*rows_per_rank, (r+1)*rows_per_rank). */
int tccl_exchange_rows(void* out, int32_t rows_per_rank, int32_t N, int64_t ld, int32_t elem_bytes,
                       const tccl_heap_view* heap, const tccl_transport_desc* transport, void* stream);
/* tccl_copy_block: tile_put / tile_get (primitives/communication.py:133-225) for a whole
 * rectangle, and the copy kernels of the stand-alone collectives (_allgather_kernel,
 * _broadcast_kernel, _scatter_kernel: primitives/collectives.py:1074-1094, 1369-1389,
 * 1595-1621).  `src` and `dst` are addresses inside the calling rank's slice; the rectangle
 * (rows x row_bytes, pitches in bytes) is read at `src` translated into slice `src_rank`
 * and written at `dst` translated into every slice whose bit is set in `dst_ranks`.
 * Rows, pitches and both addresses must be multiples of 16 bytes. */
int tccl_copy_block(void* dst, uint32_t dst_ranks, const void* src, int32_t src_rank, int32_t rows,
                    int64_t row_bytes, int64_t src_pitch_bytes, int64_t dst_pitch_bytes,
                    const tccl_heap_view* heap, void* stream);
/* tccl_gather_cols: the gather worker of ChainedAGGemmRSPattern
 * (patterns/chained_ag_gemm_rs.py:262-340).  Every rank holds an M x cols `shard` at the same
 * heap offset; column block p of this rank's `gathered` (M x world*cols, leading dim
 * ld_gathered, in its slice) receives rank p's shard: the own one by a local copy, the
 * others by remote loads. */
int tccl_gather_cols(void* gathered, int64_t ld_gathered, const void* shard, int64_t ld_shard, int32_t M,
                     int32_t cols, int32_t elem_bytes, const tccl_heap_view* heap,
                     const tccl_transport_desc* transport, void* stream);
/* tccl_reduce_rows: pull-reduce of tile_reduce_scatter (collectives.py:730-783) over row
 * shards with fp32 accumulation: out[r - row_lo] = cast(sum_p partial_p[r]) for
 * r in [row_lo, row_hi), where partial_p is `partial` translated into slice p, summed
 * local first, then peers in ascending rank.  If `emulate_peer` is non-zero the same
 * reduction is also carried out for every other rank's shard into that rank's `out`.
 * `out` is fp16 or bf16, or fp32 when the partials are fp32. */
int tccl_reduce_rows(const void* partial, int32_t partial_dtype, int64_t ld_partial, void* out,
                     int32_t out_dtype, int64_t ld_out, int32_t M, int32_t N,
                     const tccl_heap_view* heap, const tccl_transport_desc* transport,
                     int32_t emulate_peer, void* stream);

/* tccl_collective_staged: the staged peer-read collectives of the public launchers
 * (_allreduce_staged_kernel, primitives/collectives.py:840-962, and the two-rank kernels
 * _allreduce_ / _allgather_ / _reduce_scatter_ / _broadcast_ / _scatter_staged_kernel_ws2,
 * :966-1592; launchers :1882-2478, workspace :2813-2838), for any world size.  Buffers are given
 * by rank `heap->rank`'s addresses and sit at the same offset of every rank's slice.
 *   op              src                      dst                       a block is
 *   ALLREDUCE       unused (NULL)            the tensor, in place      the tensor
 *   ALLGATHER       the rank's block         world blocks              src
 *   REDUCE_SCATTER  world blocks             one block                 dst
 *   BROADCAST       unused (NULL)            the tensor, in place      the tensor
 *   SCATTER         world blocks (root's)    one block                 dst
 * block_elems elements of `dtype` (whole 16-byte units); reductions take F16 / BF16 / F32 and
 * accumulate in fp32 with one rounding (all-reduce: ranks ascending, the same bits on every rank;
 * reduce-scatter: the owner's block first, then ranks ascending; the reference adds in the
 * tensor's type), copies move bytes of any listed dtype.  Per chunk of chunk_elems a publisher
 * (every rank; BROADCAST / SCATTER: `root`) snapshots what its peers need into its `staging` slot
 * and stores epoch base_epoch + chunk in `published[slot]`; a consumer waits for that epoch, reads
 * the slot, writes its own output and adds 1 to the publisher's `consumed[slot]`; the publisher
 * leaves the slot at world - 1.  staging holds slots x segments x chunk_elems elements (segments
 * = world for REDUCE_SCATTER and SCATTER, else 1); published and consumed are int32[slots], zero
 * before the first call; all three live in the heap.  The caller advances base_epoch by the chunk
 * count per call.  `ranks` is the bit mask of the ranks whose roles this launch carries: one
 * process per GPU passes 1 << rank; on one GPU, where the ranks are slices of one arena, all of
 * them run as workgroups of one launch (slots workgroups per rank, all resident).  `fault` /
 * `spin_limit_ns` as in tccl_sync_desc: a wait that expires raises *fault and ends its role. */
#define TCCL_STAGED_ALLREDUCE 0
#define TCCL_STAGED_ALLGATHER 1
#define TCCL_STAGED_REDUCE_SCATTER 2
#define TCCL_STAGED_BROADCAST 3
#define TCCL_STAGED_SCATTER 4
int tccl_collective_staged(int32_t op, const void* src, void* dst, int32_t dtype, int64_t block_elems, void* staging,
                           int32_t* published, int32_t* consumed, int32_t chunk_elems, int32_t slots,
                           int32_t base_epoch, uint32_t ranks, int32_t root, const tccl_heap_view* heap,
                           int64_t* fault, int64_t spin_limit_ns, void* stream);

/* tccl_allreduce_staged: tccl_collective_staged(TCCL_STAGED_ALLREDUCE, NULL, tensor, ...), the
 * kernel behind the reference's public allreduce (primitives/collectives.py:1905-1946). */
int tccl_allreduce_staged(void* tensor, int32_t dtype, int64_t numel, void* staging, int32_t* published,
                          int32_t* consumed, int32_t chunk_elems, int32_t slots, int32_t base_epoch,
                          uint32_t ranks, const tccl_heap_view* heap, int64_t* fault, int64_t spin_limit_ns,
                          void* stream);

/* ---- fused operations --------------------------------------------------------------------
 * variant S0: GEMM kernel, then the communication kernel, stream-ordered.
 * variant S1: one launch; GEMM workgroups signal locks[tile]; communication workgroups
 *             wait per tile (WGSpecializedPattern, wg_specialized.py:212-352).
 * variant S2: one launch; GEMM workgroups add to counter[group_table[tile]];
 *             communication workgroups wait per TileGroup and move copy_elems-sized
 *             tasks (reference README.md:66-84; contract in the tileccl_v2 modules).
 * In S1 and S2 the pushes of an all-scatter / all-gather leave from the GEMM's epilogue (the tile goes to
 * the peers' slices from the registers it is stored from, ahead of its signal); the communication
 * workgroups carry the pulls and the reductions, and barrier[g] counts those tasks only.  A launch with
 * trace pointers keeps the pushes as tasks of the communication workgroups.
 * With the 256 x 256 GEMM tile (gemm->macro_tile) S1 and S2 are still one launch, but a
 * workgroup fills its CU, so the communication is done by the GEMM workgroups themselves:
 * pushes leave from the epilogue, all-gather pulls run inside the K loops (gated on the
 * TileGroup counters in S2, on the per-tile locks in S1; what the K loops did not cover follows
 * the workgroup's last tile), reduce-scatter tiles are reduced right after they are
 * published.  barrier[g] then advances by the grid size per launch, not by the task count.
 * Every device-side wait is bounded by sync->spin_limit_ns; an expired wait sets *sync->fault
 * and the kernel still runs to its end. */

/* tileccl.ops.gemm_allscatter (ops.py:810-888): C = A@B locally, then the rank's column
 * block is stored into every peer's C. */
int tccl_gemm_allscatter(const tccl_gemm_desc* gemm, const tccl_scatter_desc* scatter,
                         const tccl_heap_view* heap, const tccl_sync_desc* sync,
                         const tccl_transport_desc* transport, int32_t variant, void* stream);

/* ChainedAGGemmRSPattern.execute (patterns/chained_ag_gemm_rs.py:120-200): gather the ranks'
 * column shards of the input into gemm->A (M x K, K = world * k_shard, in this rank's slice),
 * output = gathered @ W (gemm->B), and store every output tile into every peer's output at
 * the same offset (scatter worker, :393-425).  `variant` selects how the three stages overlap.
 * S0: a gather launch, the GEMM kernel, then a copy kernel.  S1 / S2: one launch as
 * tccl_gemm_allscatter, in which (256 x 256 tile, output of the input type, row-major B) the K
 * loops read every rank's shard where it lies while gemm->A is filled in their background;
 * otherwise the gather is a bulk launch of its own ahead of that launch. */
int tccl_chained_ag_gemm_rs(const tccl_gemm_desc* gemm, const void* shard, int64_t ld_shard, int32_t k_shard,
                            const tccl_heap_view* heap, const tccl_sync_desc* sync,
                            const tccl_transport_desc* transport, int32_t variant, void* stream);

/* GEMM-output AllGather (Gate 1).  gemm->C must point at row rank*M of `out`. */
int tccl_gemm_allgather(const tccl_gemm_desc* gemm, void* out, int64_t ld_out,
                        const tccl_heap_view* heap, const tccl_sync_desc* sync,
                        const tccl_transport_desc* transport, int32_t variant, void* stream);

/* GEMM to ReduceScatter (Gate 2).  gemm->C is the rank's partial (M x N, dtype
 * gemm->out_dtype) in its slice; `out` receives the rank's M/world_size row shard.
 * emulate_peer is a bit mask: TCCL_RS_EMULATE_PEERS also carries out the other owners'
 * reductions into their slices (the whole operation on one GPU); TCCL_RS_PEERS_RESIDENT
 * declares the peers' partials complete in memory, so that no launch waits for their signal
 * words (ranks emulated one after another in one process, where a peer cannot be running). */
int tccl_gemm_reducescatter(const tccl_gemm_desc* gemm, void* out, int32_t out_dtype, int64_t ld_out,
                            const tccl_heap_view* heap, const tccl_sync_desc* sync,
                            const tccl_transport_desc* transport, int32_t emulate_peer,
                            int32_t variant, void* stream);

/* ---- one entry point that allocates nothing ------------------------------------------------
 * No counterpart in the reference (its lock / signal tensors are torch allocations made by
 * the caller's process: wg_specialized.py:104-124, tileccl_v2/signal.py:43-66).  It is for
 * callers that cannot allocate device memory for the signal words: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.
 *
 * tccl_gemm_allgather (S1 or S2) with the signal words and plan tables -- locks, counter,
 * barrier, group_table, row_starts, row_ends, tile_counts -- kept in a file-scope device array
 * of the library (about 581 KiB on every GPU the process uses, for the life of the process)
 * instead of being brought in by a tccl_sync_desc.  The caller still passes the operands, the
 * gathered output and the heap view; `plan` is HOST memory and travels in the kernel
 * arguments of a small set-up kernel that also prepares the calling rank's words for this
 * call.  group_table is derived on the device from the plan's rows by the rule of
 * build_group_table (tileccl_v2/tile_group.py:214-241).
 *
 * Launch numbers.  The library counts the calls per device and rank (host memory).  Call n of
 * a rank stores n into its locks and brings every TileGroup counter to n * 2 *
 * TCCL_STATIC_MAX_TILES (the set-up kernel starts the counter the group's tile count short of
 * that), and waits for its peers' words to reach the same values: what a peer's call n - 1
 * left behind, with the same plan or another one, never satisfies call n.  Ranks that wait on
 * each other must therefore have made the same number of calls on their devices, as with
 * tccl_gemm_allgather's `epoch`; a rank whose peer is a call behind waits (bounded by
 * `spin_limit_ns`) and raises `fault`.  Words are compared as sequence numbers
 * (tccl_word_reached), so the count may wrap.  A call recorded into a HIP graph replays with
 * the number it was recorded with: replays of two ranks' graphs must keep the producer ahead
 * of the consumer on the stream, as a replay cannot be told from the one before it.
 * tccl_static_call_words returns the values call number `call` works with.
 *
 * Limits: at most TCCL_STATIC_MAX_TILES plan tiles and TCCL_STATIC_MAX_GROUPS TileGroups
 * (larger inputs are rejected with TCCL_ERR_UNSUPPORTED), groups ascending and disjoint.
 * The ranks emulated on one GPU share the array, each with its own block of words.  Calls
 * that overlap in time on one GPU race on the shared plan tables (and on their own words when
 * they are calls of the same rank): order them on one stream.  The first call on a device
 * looks up the array's address (no allocation); make it before a capture begins.
 * `fault` (device int64[1] or NULL) and `spin_limit_ns` as in tccl_sync_desc.  Calls
 * no hipMalloc / hipFree and no allocating library routine. */
#define TCCL_STATIC_MAX_TILES 16384
#define TCCL_STATIC_MAX_GROUPS 64
typedef struct tccl_static_plan {
  int32_t n_groups; /* 1 .. TCCL_STATIC_MAX_GROUPS */
  int32_t row_starts[TCCL_STATIC_MAX_GROUPS]; /* rows relative to the GEMM's C */
  int32_t row_ends[TCCL_STATIC_MAX_GROUPS];   /* clamped to M */
  int32_t tile_counts[TCCL_STATIC_MAX_GROUPS];
} tccl_static_plan;
int tccl_gemm_allgather_static(const tccl_gemm_desc* gemm, void* out, int64_t ld_out,
                               const tccl_heap_view* heap, const tccl_static_plan* plan,
                               const tccl_transport_desc* transport, int32_t variant,
                               int64_t* fault, int64_t spin_limit_ns, void* stream);
/* The launch number call `call` (1, 2, ...) of tccl_gemm_allgather_static stores into its locks,
 * where it starts a TileGroup counter of `tile_count` tiles and what that counter reads once the
 * group is complete (what a peer in its own call `call` waits for).  Host arithmetic only. */
int tccl_static_call_words(uint32_t call, int32_t tile_count, int32_t* epoch, int32_t* counter_start,
                           int32_t* counter_ready);
/* Start the launch numbers of tccl_gemm_allgather_static over on the current device: every rank's
 * next call is call 1 again, and every rank's words in the library's array are cleared by a fill
 * kernel on `stream` (no allocation, no memset).  For ranks whose call counts have come apart (a
 * call that gave up on its wait, a rank that was restarted): all ranks that wait on each other
 * must reset together, with none of their calls in flight. */
int tccl_static_reset(void* stream);
/* The comparison every wait on a signal word uses: 1 if `word` has reached `need`, as sequence
 * numbers (the difference modulo 2^32 is non-negative); words and thresholds may wrap. */
int tccl_word_reached(int32_t word, int32_t need);

/* ---- measurement aid: what the matrix pipes sustain by themselves ------------------------------
 * No counterpart in the reference.  A launch shaped like the large-tile GEMM (`workgroups` x 512
 * threads, 128 accumulator registers per lane) whose lanes load 96 operand registers once --
 * row operands from `a_like`, column operands from `b_like`, each lane its own 16- or 32-byte
 * units, wrapping around the buffers -- and then issue nothing but MFMAs: `steps` times the
 * MFMAs of one K step of a 256 x 256 tile, i.e. 2 * 256 * 256 * 64 FLOP per workgroup and step
 * for the 16-bit kinds and 2 * 256 * 256 * 128 for the fp8 kinds.  No LDS and no memory access
 * inside the loop, so (time(steps2) - time(steps1)) / (steps2 - steps1) is the matrix pipes'
 * own time per step on that operand data.  `sink` takes one float per thread. */
#define TCCL_PROBE_F16_32X32X16 0
#define TCCL_PROBE_F16_16X16X32 1
#define TCCL_PROBE_BF16_16X16X32 2
#define TCCL_PROBE_F8_16X16X128 3
#define TCCL_PROBE_F8_32X32X64 4
int tccl_mfma_rate_probe(int32_t kind, const void* a_like, int64_t a_bytes, const void* b_like,
                         int64_t b_bytes, float* sink, int32_t steps, int32_t workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TILECCL_HIP_H */
