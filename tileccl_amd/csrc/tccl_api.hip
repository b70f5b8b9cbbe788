// Host side of libtileccl_hip.so: argument checks, launch geometry, and the extern "C"
// entry points declared in include/tileccl_hip.h.  No Python, no torch types.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <type_traits>

// The library is built with -fvisibility=hidden: only what the public header declares is exported.
#pragma GCC visibility push(default)
#include "../../include/tileccl_hip.h"
#pragma GCC visibility pop
#include "tccl_comm.h"
#include "tccl_gemm.h"
#include "tccl_gemm256.h"
#include "tccl_kernels256.h"
#include "tccl_probe.h"
#include "tccl_staged.h"

namespace {

using tccl::Fused256Args;

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail((int)e, "HIP error in %s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

#define TCCL_HIP(call)                                  \
  do {                                                  \
    hipError_t e_ = (call);                             \
    if (e_ != hipSuccess) return hip_fail(e_, #call);   \
  } while (0)

struct DeviceCache {
  bool valid = false;
  int device = -1;
  tccl_device_info info;
};
thread_local DeviceCache g_dev;  // per host thread: no lock, no sharing

int query_device(int device, tccl_device_info* out) {
  if (device < 0) TCCL_HIP(hipGetDevice(&device));
  if (!g_dev.valid || g_dev.device != device) {
    hipDeviceProp_t p;
    TCCL_HIP(hipGetDeviceProperties(&p, device));
    tccl_device_info i;
    memset(&i, 0, sizeof i);
    i.compute_units = p.multiProcessorCount;
    i.clock_khz = p.clockRate;
    i.lds_bytes = (int)p.sharedMemPerBlock;
    i.wavefront = p.warpSize;
    strncpy(i.arch, p.gcnArchName, sizeof(i.arch) - 1);
    // MI300/MI350 class parts expose 8 accelerator dies; each owns compute_units / 8 CUs
    // and one L2.  Smaller parts are treated as one die.
    i.xcds = (i.compute_units >= 64 && i.compute_units % 8 == 0) ? 8 : 1;
    g_dev.info = i;
    g_dev.device = device;
    g_dev.valid = true;
  }
  *out = g_dev.info;
  return 0;
}

size_t dtype_size(int dt) {
  switch (dt) {
    case TCCL_F16:
    case TCCL_BF16: return 2;
    case TCCL_F32: return 4;
    case TCCL_F8E4M3: return 1;
    default: return 0;
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// ------------------------------------------------------------------------------------------
// Kernels
// ------------------------------------------------------------------------------------------
// One launch holds both roles: workgroups [0, num_compute) run the GEMM, the rest move
// data.  Three waves per SIMD (two GEMM workgroups plus one communication workgroup per
// CU) bounds the register budget.
template <typename InT, typename OutT>
__global__ __launch_bounds__(256, 3) void fused_kernel(tccl::GemmArgs g, tccl::SignalArgs s, tccl::CommArgs c, tccl::PushArgs push,
                                                       int num_compute, int64_t* trace_start) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(1024))) char stage0[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage1[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage2[tccl::kStage128];
  if ((int)blockIdx.x < num_compute) {
    if (trace_start && blockIdx.x == 0 && threadIdx.x == 0) *trace_start = tccl::now_ticks();
    tccl::GemmRole<InT, OutT>(g, push, stage0, stage1, stage2).run(s, (int)blockIdx.x, num_compute);
  } else {
    tccl::comm_role(c, (int)blockIdx.x - num_compute, (int)gridDim.x - num_compute, (int*)stage0);
  }
#endif
}

// The GEMM alone on 128 x 128 tiles: no communication workgroup has to fit beside it, so it takes five
// stages (80 KiB, two workgroups per CU): a load then has three steps and a half to arrive instead of
// one and a half.
template <typename InT, typename OutT>
__global__ __launch_bounds__(256, 2) void gemm128_kernel(tccl::GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(1024))) char stage0[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage1[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage2[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage3[tccl::kStage128];
  __shared__ __attribute__((aligned(1024))) char stage4[tccl::kStage128];
  tccl::SignalArgs s;
  s.mode = tccl::kSignalNone;
  tccl::PushArgs push;
  push.world = 0;
  tccl::GemmRole<InT, OutT, 5>(g, push, stage0, stage1, stage2, stage3, stage4).run(s, (int)blockIdx.x, (int)gridDim.x);
#endif
}

// The stand-alone bulk kernels (S0's second kernel, the scatter / gather / block copies, the stand-alone
// reduction): the communication role with everything else compiled out.  The full role (per-tile and
// per-group waits, every reduction type) is a large kernel, and a launch of it took 1.2 us longer to move
// the same bytes (the 128 MiB exchange of the 4096 x 4096 x 1024 all-gather: 21.5 against 20.3 us).
__global__ __launch_bounds__(256) void copy_kernel(tccl::CommArgs c) {
  __shared__ int word[4];
  tccl::comm_role<tccl::kThreadsComm, tccl::kBulkCopy>(c, (int)blockIdx.x, (int)gridDim.x, word);
}
__global__ __launch_bounds__(256) void reduce_kernel(tccl::CommArgs c) {
  __shared__ int word[4];
  tccl::comm_role<tccl::kThreadsComm, tccl::kBulkReduce>(c, (int)blockIdx.x, (int)gridDim.x, word);
}

// Staged collectives: workgroup w carries slot w % slots of the (w / slots)-th rank named in a.ranks.
__global__ __launch_bounds__(256) void staged_kernel(tccl::StagedArgs a) {
  __shared__ int word;
  int which = (int)blockIdx.x / a.slots, r = 0;
  for (; r < a.world; ++r)
    if (((a.ranks >> r) & 1u) && which-- == 0) break;
  if (r >= a.world) return;
  const int slot = (int)blockIdx.x % a.slots;
  if (a.dtype == tccl::kF16)
    tccl::staged_role<_Float16>(a, r, slot, &word);
  else if (a.dtype == tccl::kBF16)
    tccl::staged_role<__bf16>(a, r, slot, &word);
  else
    tccl::staged_role<float>(a, r, slot, &word);
}

__global__ void fill_kernel(int32_t* w, int64_t n, int32_t v) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) w[i] = v;
}

// Strided matrix -> dense rows, one 64 x 64 patch per workgroup through LDS: the patch is read along
// whichever source index is closer in memory and written along the destination's rows, so both sides
// move whole lines whatever the source's strides are.  Elements outside the source are written as zero.
template <typename T>
__global__ __launch_bounds__(256) void pack_kernel(const T* src, int64_t stride_row, int64_t stride_col, int rows, int cols,
                                                   T* dst, int64_t ld_dst, int dst_rows, int dst_cols) {
  __shared__ T patch[64][65];
  const int r0 = (int)blockIdx.y * 64, c0 = (int)blockIdx.x * 64;
  const int fast = (int)threadIdx.x & 63, slow = (int)threadIdx.x >> 6;
  const bool along_cols = stride_col <= stride_row;
  for (int i = slow; i < 64; i += 4) {
    const int r = along_cols ? i : fast, c = along_cols ? fast : i;
    T v = 0;
    if (r0 + r < rows && c0 + c < cols) v = src[(int64_t)(r0 + r) * stride_row + (int64_t)(c0 + c) * stride_col];
    patch[r][c] = v;
  }
  __syncthreads();
  for (int i = slow; i < 64; i += 4)
    if (r0 + i < dst_rows && c0 + fast < dst_cols) dst[(int64_t)(r0 + i) * ld_dst + c0 + fast] = patch[i][fast];
}

__global__ void prim_signal_kernel(int32_t* locks, int i) { tccl::tile_signal(locks, i); }
__global__ void prim_signal_add_kernel(int32_t* w, int i, int v, int32_t* res) { *res = tccl::tile_signal_add(w, i, v); }
__global__ void prim_try_wait_kernel(int32_t* locks, int i, int spins, int consume, int32_t* res) {
  *res = tccl::tile_try_wait(locks, i, spins, consume != 0) ? 1 : 0;
}
__global__ void prim_wait_ge_kernel(int32_t* w, int i, int thr, int64_t ticks, int32_t* res) {
  *res = tccl::tile_wait_ge(w, i, thr, tccl::now_ticks() + ticks) ? 1 : 0;
}

// ------------------------------------------------------------------------------------------
// Argument translation
// ------------------------------------------------------------------------------------------
constexpr int64_t kDefaultSpinNs = 2000000000ll;

bool plan_tile_fits_macro(const tccl_gemm_desc* d) {
  return (d->block_m == 128 || d->block_m == 256) && (d->block_n == 128 || d->block_n == 256);
}

int check_gemm(const tccl_gemm_desc* d) {
  if (!d) return fail(TCCL_ERR_INVALID, "gemm descriptor is NULL");
  if (!d->A || !d->B || !d->C) return fail(TCCL_ERR_INVALID, "gemm: A, B and C must be non-NULL");
  if (d->M <= 0 || d->N <= 0 || d->K <= 0) return fail(TCCL_ERR_INVALID, "gemm: M, N, K must be positive (got %d, %d, %d)", d->M, d->N, d->K);
  if (d->block_m <= 0 || d->block_n <= 0 || d->group_m <= 0) return fail(TCCL_ERR_INVALID, "gemm: block_m, block_n, group_m must be positive");
  if (d->block_m % tccl::kTile || d->block_n % tccl::kTile)
    return fail(TCCL_ERR_UNSUPPORTED, "gemm: plan tile %dx%d must be a multiple of 128x128", d->block_m, d->block_n);
  if (d->macro_tile != 0 && d->macro_tile != 128 && d->macro_tile != 256)
    return fail(TCCL_ERR_INVALID, "gemm: macro_tile=%d must be 0, 128 or 256", d->macro_tile);
  const size_t isz = dtype_size(d->in_dtype), osz = dtype_size(d->out_dtype);
  if (!isz || !osz) return fail(TCCL_ERR_INVALID, "gemm: unknown dtype");
  if (d->in_dtype == TCCL_F32) return fail(TCCL_ERR_UNSUPPORTED, "gemm: fp32 inputs have no MFMA kernel here");
  if (d->in_dtype == TCCL_F8E4M3 && (d->macro_tile == 128 || !plan_tile_fits_macro(d)))
    return fail(TCCL_ERR_UNSUPPORTED, "gemm: fp8 inputs need the 256x256 kernel (macro_tile 0 or 256, plan tile edges 128 or 256)");
  if (d->out_dtype == TCCL_F8E4M3) return fail(TCCL_ERR_UNSUPPORTED, "gemm: fp8 output is not supported");
  const int shards = d->column_shards > 1 ? d->column_shards : 1;
  if (d->column_shards < 0 || d->M % shards || (shards > 1 && (d->M / shards) % d->block_m))
    return fail(TCCL_ERR_INVALID, "gemm: column_shards=%d must split M=%d into blocks of whole %d-row plan tiles", d->column_shards, d->M, d->block_m);
  if (d->in_dtype == TCCL_F8E4M3 && shards > 1 && (d->M / shards) % 256)
    return fail(TCCL_ERR_UNSUPPORTED, "gemm: fp8 inputs with column_shards need row blocks of whole 256-row tiles");
  const int in_vec = (int)(16 / isz), out_vec = (int)(16 / osz);
  if (d->K % in_vec) return fail(TCCL_ERR_UNSUPPORTED, "gemm: K=%d must be a multiple of %d", d->K, in_vec);
  if (d->N % 8) return fail(TCCL_ERR_UNSUPPORTED, "gemm: N=%d must be a multiple of 8", d->N);
  const bool b_kmajor = (d->flags & TCCL_GEMM_B_KMAJOR) != 0;
  if (d->lda < d->K || d->ldb < (b_kmajor ? (int64_t)d->K : (int64_t)d->N * shards) || d->ldc < d->N)
    return fail(TCCL_ERR_INVALID, "gemm: leading dimension smaller than the row length");
  if (d->lda % in_vec || d->ldb % in_vec || d->ldc % out_vec || !aligned16(d->A) || !aligned16(d->B) || !aligned16(d->C))
    return fail(TCCL_ERR_UNSUPPORTED, "gemm: A, B, C rows must start on 16-byte boundaries");
  // The kernels address an operand with 32-bit byte offsets from a per-tile base: B from its
  // first row down to row K-1 (k-major B: over the 256 columns of a tile), A and C over the 256 rows of a tile.
  const int64_t limit = 0xffffffffll;
  const int64_t b_span = (b_kmajor ? 255 * d->ldb + d->K : (int64_t)(d->K - 1) * d->ldb + (int64_t)d->N * shards) * (int64_t)isz;
  const int64_t a_span = (255 * d->lda + d->K) * (int64_t)isz;
  const int64_t c_span = (255 * d->ldc + d->N) * (int64_t)osz;
  if (b_span > limit || a_span > limit || c_span > limit)
    return fail(TCCL_ERR_UNSUPPORTED, "gemm: an operand spans more than 4 GiB from a tile's base (B %lld, A %lld, C %lld bytes)",
                (long long)b_span, (long long)a_span, (long long)c_span);
  return 0;
}

int gemm_span(int in_flight, int group_m, int xcds) {
  // Tile ids an XCD takes from each block of xcds * span ids: its share of the tiles in flight, in whole
  // columns of a band (ids run down the group_m rows of a band column, then to the next column), so that
  // the tiles resident on an XCD at one time form a compact patch and share their operand panels in its
  // L2.  What an XCD's L2 misses comes over the fabric, which is what bounds the 128 x 128-tile kernel:
  // with 32 tiles in flight per XCD a patch of 8 x 4 tiles reads 12 panels, one of 8 x 2 twice over 20.
  if (xcds <= 1) return 1;
  int span = in_flight / xcds;
  if (span >= group_m) span = span / group_m * group_m;
  return span > 0 ? span : 1;
}

int build_gemm_args(const tccl_gemm_desc* d, const tccl_device_info& dev, tccl::GemmArgs* g) {
  g->A = d->A;
  g->B = d->B;
  g->C = d->C;
  g->M = d->M;
  g->N = d->N;
  g->K = d->K;
  g->lda = d->lda;
  g->ldb = d->ldb;
  g->ldc = d->ldc;
  g->alpha = d->alpha;
  g->block_m = d->block_m;
  g->block_n = d->block_n;
  g->group_m = d->group_m;
  g->tile_rows = (d->M + d->block_m - 1) / d->block_m;
  g->tile_cols = (d->N + d->block_n - 1) / d->block_n;
  g->xcds = dev.xcds;
  {
    const int total = g->tile_rows * g->tile_cols;
    int wgs = d->num_wgs > 0 ? d->num_wgs : 2 * dev.compute_units;  // default_gemm_wgs()
    g->span = gemm_span(wgs < total ? wgs : total, d->group_m, dev.xcds);
  }
  g->wrap_rows = d->column_shards > 1 ? d->M / d->column_shards : 0;
  g->b_kmajor = (d->flags & TCCL_GEMM_B_KMAJOR) ? 1 : 0;
  return 0;
}

int default_gemm_wgs(const tccl_gemm_desc* d, const tccl_device_info& dev, int total_tiles) {
  int n = d->num_wgs > 0 ? d->num_wgs : 2 * dev.compute_units;
  if (n > total_tiles) n = total_tiles;
  return n < 1 ? 1 : n;
}

void fill_comm_common(tccl::CommArgs* c, const tccl::GemmArgs& g, int esize, const tccl_heap_view* heap,
                      const tccl_sync_desc* sync, const tccl_transport_desc* tr) {
  memset(c, 0, sizeof *c);
  c->heap_bases = heap->heap_bases;
  c->rank = heap->rank;
  c->world = heap->world_size;
  c->C = (char*)g.C;
  c->ldc_bytes = g.ldc * esize;
  c->M = g.M;
  c->N = g.N;
  c->esize = esize;
  c->block_m = g.block_m;
  c->block_n = g.block_n;
  c->group_m = g.group_m;
  c->tile_rows = g.tile_rows;
  c->tile_cols = g.tile_cols;
  c->xcds = g.xcds;
  c->span = g.span;
  c->directions = tr ? tr->directions : TCCL_DIR_PUSH;
  c->n_groups = 1;
  c->epoch = 1;
  c->spin_ticks = kDefaultSpinNs / 10;
  if (sync) {
    c->locks = sync->locks;
    c->counter = sync->counter;
    c->barrier = sync->barrier;
    c->row_starts = sync->row_starts;
    c->row_ends = sync->row_ends;
    c->tile_counts = sync->tile_counts;
    if (sync->row_starts && sync->n_groups > 0) c->n_groups = sync->n_groups;
    c->epoch = sync->epoch > 0 ? sync->epoch : 1;
    c->trace_comm_counter = sync->trace_comm_counter;
    c->trace_ready_clock = sync->trace_ready_clock;
    c->trace_done_clock = sync->trace_done_clock;
    c->fault = sync->fault;
    if (sync->spin_limit_ns > 0) c->spin_ticks = sync->spin_limit_ns / 10 + 1;
  }
}

int check_heap(const tccl_heap_view* h) {
  if (!h || !h->heap_bases) return fail(TCCL_ERR_INVALID, "heap view / heap_bases is NULL");
  if (h->world_size < 1 || h->world_size > TCCL_MAX_WORLD) return fail(TCCL_ERR_INVALID, "world_size=%d outside [1, %d]", h->world_size, TCCL_MAX_WORLD);
  if (h->rank < 0 || h->rank >= h->world_size) return fail(TCCL_ERR_INVALID, "rank=%d out of range for world_size=%d", h->rank, h->world_size);
  return 0;
}

int set_task_units(tccl::CommArgs* c, const tccl_transport_desc* tr, bool reduce) {
  const int unit_elems = reduce ? 8 : 16 / c->esize;
  int elems = tr ? (reduce && tr->reduce_elems > 0 ? tr->reduce_elems : tr->copy_elems) : 0;
  if (elems <= 0) elems = 16384;
  if (elems % unit_elems) return fail(TCCL_ERR_UNSUPPORTED, "task size %d elements is not a multiple of %d", elems, unit_elems);
  c->copy_units = c->reduce_units = elems / unit_elems;
  return 0;
}

int check_sync(const tccl_sync_desc* s, int variant) {
  if (variant == TCCL_S0_BULK) return 0;
  if (!s) return fail(TCCL_ERR_INVALID, "variant S%d needs a sync descriptor", variant);
  if (variant == TCCL_S1_TILE && !s->locks) return fail(TCCL_ERR_INVALID, "S1 needs locks");
  if (s->epoch < 1) return fail(TCCL_ERR_INVALID, "S%d epoch must be >= 1", variant);
  if (variant == TCCL_S2_TILEGROUP) {
    if (!s->counter || !s->group_table || !s->row_starts || !s->row_ends || !s->tile_counts || s->n_groups <= 0)
      return fail(TCCL_ERR_INVALID, "S2 needs counter, group_table, row_starts, row_ends, tile_counts and n_groups > 0");
  }
  return 0;
}

// ------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------
template <typename InT, typename OutT>
int launch_fused_t(const tccl::GemmArgs& g, const tccl::SignalArgs& s, const tccl::CommArgs& c, const tccl::PushArgs& push,
                   int compute, int comm, int64_t* trace_start, hipStream_t stream) {
  if (comm == 0 && s.mode == tccl::kSignalNone && !trace_start)
    hipLaunchKernelGGL((gemm128_kernel<InT, OutT>), dim3(compute), dim3(tccl::kThreads), 0, stream, g);
  else
    hipLaunchKernelGGL((fused_kernel<InT, OutT>), dim3(compute + comm), dim3(tccl::kThreads), 0, stream, g, s, c, push, compute,
                       trace_start);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int launch_fused(int in_dtype, int out_dtype, const tccl::GemmArgs& g, const tccl::SignalArgs& s, const tccl::CommArgs& c,
                 int compute, int comm, int64_t* trace_start, hipStream_t stream, const tccl::PushArgs* push_args = nullptr) {
  tccl::PushArgs push;
  memset(&push, 0, sizeof push);
  if (push_args) push = *push_args;
  if (in_dtype == TCCL_F16 && out_dtype == TCCL_F16) return launch_fused_t<_Float16, _Float16>(g, s, c, push, compute, comm, trace_start, stream);
  if (in_dtype == TCCL_F16 && out_dtype == TCCL_F32) return launch_fused_t<_Float16, float>(g, s, c, push, compute, comm, trace_start, stream);
  if (in_dtype == TCCL_BF16 && out_dtype == TCCL_BF16) return launch_fused_t<__bf16, __bf16>(g, s, c, push, compute, comm, trace_start, stream);
  if (in_dtype == TCCL_BF16 && out_dtype == TCCL_F32) return launch_fused_t<__bf16, float>(g, s, c, push, compute, comm, trace_start, stream);
  return fail(TCCL_ERR_UNSUPPORTED, "gemm: no kernel for in_dtype=%d, out_dtype=%d", in_dtype, out_dtype);
}

// ---- large-tile path ----------------------------------------------------------------------------

// 256 x 256 tiles pay off once there are enough of them to occupy most CUs; below that
// the 128 x 128 kernel spreads the work over more workgroups.  With large tiles on exactly half of the CUs
// the GEMM alone is 5-6 % faster on small tiles (2048 x 4096 x 1024: 22.3 against 23.3 us; 4096 x 2048 x 2048:
// 38.1 against 40.6; 96 large tiles: 63.3 against 73.8), from 144 large tiles on it is slower (3072^3: 76.6
// against 58.5 us); the fused launches keep the large tiles there (their transfers ride on the K loops).
bool use_macro(const tccl_gemm_desc* d, const tccl_device_info& dev, bool fused = true) {
  if (d->in_dtype == TCCL_F8E4M3) return true;  // fp8 exists only as the large-tile kernel (check_gemm vets the plan tile)
  if (!plan_tile_fits_macro(d)) return false;
  if (d->column_shards > 1 && (d->M / d->column_shards) % 256) return false;  // a tile must not straddle two row blocks
  if (d->macro_tile == 128) return false;
  if (d->macro_tile == 256) return true;
  const int64_t tiles = (int64_t)((d->M + 255) / 256) * ((d->N + 255) / 256);
  return fused ? tiles * 2 >= dev.compute_units : tiles * 2 > dev.compute_units;
}

tccl::Macro build_macro(const tccl_gemm_desc* d, const tccl_device_info& dev, int num_wgs) {
  tccl::Macro m;
  m.rows = (d->M + 255) / 256;
  m.cols = (d->N + 255) / 256;
  const int band_rows = d->group_m * d->block_m / 256;
  m.rows_per_band = band_rows > 0 ? band_rows : 1;
  m.xcds = dev.xcds;
  // Ids an XCD takes from each block: its share of the tiles in flight, in whole band columns.
  const int total = m.rows * m.cols;
  const int in_flight = total < num_wgs ? total : num_wgs;
  int span = in_flight / (dev.xcds > 0 ? dev.xcds : 1);
  span = span / m.rows_per_band * m.rows_per_band;
  m.span = span > 0 ? span : 1;
  m.row_shift = 0;
  return m;
}

int default_macro_wgs(const tccl_gemm_desc* d, const tccl_device_info& dev) {
  const int total = ((d->M + 255) / 256) * ((d->N + 255) / 256);
  int n = d->num_wgs > 0 ? d->num_wgs : dev.compute_units;
  // One workgroup fills a CU, and workgroups of a fused launch wait on each other's tiles
  // after their own: every workgroup must be resident, so the grid never exceeds the CUs.
  if (n > dev.compute_units) n = dev.compute_units;
  if (n > total) n = total;
  return n < 1 ? 1 : n;
}

// Large-tile kernels: B row-major ones are instantiated here, the k-major ones in tccl_kmajor.hip.
int launch_status(int rc, int in_dtype, int out_dtype) {
  if (rc == 0) return 0;
  if (rc == tccl::kNoKernel) return fail(TCCL_ERR_UNSUPPORTED, "gemm: no kernel for in_dtype=%d, out_dtype=%d", in_dtype, out_dtype);
  if (rc == tccl::kGatherTypes) return fail(TCCL_ERR_UNSUPPORTED, "gathered input read in place: output type must equal the input type, B row-major");
  return hip_fail((hipError_t)rc, "large-tile kernel launch");
}

int launch_gemm256(int in_dtype, int out_dtype, const tccl::GemmArgs& g, const tccl::Macro& m, int wgs, hipStream_t stream) {
  const int rc = g.b_kmajor ? tccl::launch_gemm256_kmajor(in_dtype, out_dtype, g, m, wgs, stream)
                            : tccl::launch_gemm256_table<false>(in_dtype, out_dtype, g, m, wgs, stream);
  return launch_status(rc, in_dtype, out_dtype);
}

int launch_fused256(int in_dtype, int out_dtype, const Fused256Args& f, int wgs, hipStream_t stream) {
  const int rc = f.g.b_kmajor ? tccl::launch_fused256_kmajor(in_dtype, out_dtype, f, wgs, stream)
                              : tccl::launch_fused256_table<false>(in_dtype, out_dtype, f, wgs, stream);
  return launch_status(rc, in_dtype, out_dtype);
}

// How the background transfer addresses the 16-byte units of a block (PullArgs::row_units and what follows):
// rows of `upr` units, `pitch` bytes apart on the destination side and `src_pitch` on the source side.  Rows that
// follow each other without gaps on both sides are one long row.  The kernel divides by multiplying:
// u / d = mulhi(u, magic) >> shift with shift = floor(log2 d), magic = ceil(2^(32 + shift) / d), which fits 32
// bits for every d that is not a power of two and is exact for u < 2^31 (the error term u * (magic * d -
// 2^(32 + shift)) stays below 2^(32 + shift)); a power of two is magic = 0 and a plain shift.
void set_row_divider(tccl::PullArgs* p, uint32_t upr, uint32_t pitch, uint32_t src_pitch) {
  const bool flat = pitch == upr * 16u && src_pitch == upr * 16u;
  const uint32_t d = flat ? (p->units > 0 ? p->units : 1u) : upr;
  p->row_units = d;
  p->row_pitch = pitch;
  p->src_row_pitch = src_pitch;
  uint32_t shift = 0;
  while ((2ull << shift) <= d) ++shift;  // floor(log2 d)
  p->row_shift = shift;
  p->row_magic = (d & (d - 1)) == 0 ? 0u : (uint32_t)((((uint64_t)1 << (32 + shift)) + d - 1) / d);
}

// The pull half of a TileGroup all-gather, as the large-tile K loop performs it in the
// background.  Returns false when there is nothing of the kind to do (the communication role
// after the last tile then does it).
bool build_background(const tccl::CommArgs& c, tccl::PullArgs* p) {
  memset(p, 0, sizeof *p);
  if (c.op != tccl::kOpAllGather || c.granularity == tccl::kBulk || !(c.directions & tccl::kDirPull) || c.world <= 1) return false;
  const bool by_tile = c.granularity == tccl::kPerTile;
  int band_shift = 0;
  if (by_tile) {
    // One probe looks at the locks of two plan-tile rows, 32 lanes each; the lock index needs
    // the swizzle band as a shift.
    while ((1 << band_shift) < c.group_m) ++band_shift;
    if (!c.locks || c.tile_cols > 32 || (1 << band_shift) != c.group_m) return false;
  } else if (!c.row_ends || !c.tile_counts || !c.counter) {
    return false;
  }
  const int64_t row_bytes = (int64_t)c.N * c.esize;
  const int64_t block_bytes = (int64_t)c.M * c.ld_out_bytes;
  if (row_bytes % 16 || c.ld_out_bytes % 16 || block_bytes >= (int64_t)1 << 32) return false;
  p->mode = tccl::kBgGather;
  p->slots = c.world - 1;
  p->rank = c.rank;
  p->world = c.world;
  p->heap_bases = c.heap_bases;
  p->src0 = c.out;
  p->block_bytes = block_bytes;
  p->block_rows = c.M;
  p->pitch = (uint32_t)c.ld_out_bytes;
  p->upr = (uint32_t)(row_bytes / 16);
  p->units = (uint32_t)p->block_rows * p->upr;
  p->pieces = (int)((p->units + tccl::kPieceUnits - 1) / tccl::kPieceUnits);
  set_row_divider(p, p->upr, p->pitch, p->pitch);
  p->counter = by_tile ? c.locks : c.counter;
  p->row_ends = c.row_ends;
  p->tile_counts = c.tile_counts;
  p->n_groups = by_tile ? (c.tile_rows + 1) / 2 : c.n_groups;
  p->tile_mode = by_tile ? 1 : 0;
  p->group_m_shift = band_shift;
  p->epoch = c.epoch;
  p->barrier = c.barrier;
  p->trace_done_clock = c.trace_done_clock;
  p->fault = c.fault;
  p->spin_ticks = c.spin_ticks;
  p->word_stride = c.word_stride;
  return true;
}

// A reduce-scatter whose reduction the large-tile kernel can perform tile by tile.
bool build_reduce(const tccl::CommArgs& c, const tccl_sync_desc* sync, int flags, tccl::ReduceArgs* r, tccl::Macro* m) {
  memset(r, 0, sizeof *r);
  if (c.op != tccl::kOpReduceScatter || c.world <= 1 || c.M % c.world) return false;
  const int shard = c.M / c.world;
  if (shard % tccl::kMacro) return false;  // a tile must not straddle two owners
  if (c.out_dtype != tccl::kF16 && c.out_dtype != tccl::kBF16) return false;
  if (c.ld_rs_out_bytes % 8) return false;
  r->active = 1;
  r->rank = c.rank;
  r->world = c.world;
  r->emulate_peer = c.emulate_peer;
  r->peers_resident = c.peers_resident;
  r->shard_rows = shard;
  r->out_bf16 = c.out_dtype == tccl::kBF16;
  r->own_in_registers = (flags & TCCL_GEMM_OWN_ROWS_IN_REGISTERS) != 0;
  r->heap_bases = c.heap_bases;
  r->out = c.rs_out;
  r->ld_out = c.ld_rs_out_bytes / 2;
  r->locks = sync->locks;
  r->counter = sync->counter;
  r->tile_counts = sync->tile_counts;
  r->epoch = c.epoch;
  r->fault = c.fault;
  r->spin_ticks = c.spin_ticks;
  m->row_shift = ((c.rank + 1) % c.world) * (shard / tccl::kMacro);  // this rank's own rows come last
  return true;
}

// The push half of an all-scatter / all-gather, as the large-tile epilogue performs it.
// Returns false when the operation has no push to fold (reduce-scatter, push not asked for).
bool build_push(const tccl::CommArgs& c, const tccl::GemmArgs& g, tccl::PushArgs* p) {
  memset(p, 0, sizeof *p);
  if (!(c.directions & tccl::kDirPush) || c.world <= 1) return false;
  if (c.op != tccl::kOpAllScatter && c.op != tccl::kOpAllGather) return false;
  p->world = c.world;
  p->rank = c.rank;
  p->heap_bases = c.heap_bases;  // device memory: only the kernel reads it
  if (c.op == tccl::kOpAllScatter) {
    p->col_lo = c.src_col_off;
    p->col_hi = c.src_col_off + c.cols;
    p->col_shift = c.dst_col_off - c.src_col_off;
    p->ld = c.dst_ld;
  } else {
    p->col_lo = 0;
    p->col_hi = g.N;
    p->col_shift = 0;
    p->ld = g.ldc;
  }
  return true;
}

// The communication code addresses a rectangle (at most all M rows of one block) with 32-bit
// byte offsets from the rectangle's base.
int check_rows_span(int64_t rows, int64_t pitch_bytes) {
  if (rows * pitch_bytes > 0xffffffffll)
    return fail(TCCL_ERR_UNSUPPORTED, "a block of %lld rows of %lld bytes spans more than 4 GiB", (long long)rows,
                (long long)pitch_bytes);
  return 0;
}

int check_comm_span(const tccl::CommArgs& c) {
  int64_t pitch = c.ldc_bytes;
  if (c.ld_out_bytes > pitch) pitch = c.ld_out_bytes;
  if (c.ld_rs_out_bytes > pitch) pitch = c.ld_rs_out_bytes;
  if ((int64_t)c.dst_ld * c.esize > pitch) pitch = (int64_t)c.dst_ld * c.esize;
  return check_rows_span(c.M, pitch);
}

int launch_comm(const tccl::CommArgs& c, int wgs, hipStream_t stream) {
  const int span = check_comm_span(c);
  if (span) return span;
  if (wgs < 1) wgs = 1;
  if (c.granularity != tccl::kBulk) return fail(TCCL_ERR_INVALID, "a stand-alone communication launch is a bulk one");
  if (c.op == tccl::kOpReduceScatter)
    hipLaunchKernelGGL(reduce_kernel, dim3(wgs), dim3(tccl::kThreadsComm), 0, stream, c);
  else
    hipLaunchKernelGGL(copy_kernel, dim3(wgs), dim3(tccl::kThreadsComm), 0, stream, c);
  TCCL_HIP(hipGetLastError());
  return 0;
}

// Workgroups of a stand-alone bulk kernel, per CU: 8 for copies, 4 for reductions.  Swept on the 128 MiB
// exchange of the 4096 x 4096 x 1024 all-gather (2 / 4 / 8 per CU: 20.7 / 20.3 / 19.7 us; tasks of 128 KiB
// instead of 32 KiB: 21.7 us) and on the reductions of the reduce-scatter configurations (4 per CU ahead
// of 8 by 3-4 %).
#ifndef TCCL_BULK_COPY_WGS
#define TCCL_BULK_COPY_WGS 8
#endif
int bulk_comm_wgs(const tccl_device_info& dev, const tccl::CommArgs& c) {
  return dev.compute_units * (c.op == tccl::kOpReduceScatter ? 4 : TCCL_BULK_COPY_WGS);
}

// The second kernel of S0 waits for nothing, so a plan's TileGroups mean nothing to it: it
// sweeps the whole block (a reduce-scatter: each owner's shard) as one run of tasks.  Cut
// along the plan's groups, its tasks came out ragged at every group border (8192 x 4096
// all-gather: 123 us with eight groups against 117 us with one).
void make_bulk(tccl::CommArgs* c) {
  c->granularity = tccl::kBulk;
  c->row_starts = c->row_ends = c->tile_counts = nullptr;
  c->n_groups = c->op == tccl::kOpReduceScatter ? c->world : 1;
}

// The shards that make up the GEMM's A operand, when the chained operation reads them in place.
struct GatherSpec {
  const void* shard;
  int64_t ld_shard;
  int k_shard;
};

// Can the one-launch variants of the chained operation read the gathered input in place?
// Large-tile kernel, 16-bit inputs and an output of the same type, shards of whole K steps.
bool gather_in_place(const tccl_gemm_desc* d, const tccl_device_info& dev, int k_shard, int variant);

// The background transfer that fills the gathered workspace (gemm->A) while the K loops run.
void build_gather_background(const tccl_gemm_desc* d, const GatherSpec& gs, const tccl_heap_view* heap, const tccl::CommArgs& c,
                             tccl::PullArgs* p, tccl::GatherArgs* ga) {
  const int esz = (int)dtype_size(d->in_dtype);
  memset(ga, 0, sizeof *ga);
  ga->active = 1;
  ga->rank = heap->rank;
  ga->world = heap->world_size;
  ga->heap_bases = heap->heap_bases;
  ga->shard = gs.shard;
  ga->ld_shard = gs.ld_shard;
  ga->k_shard = gs.k_shard;
  memset(p, 0, sizeof *p);
  p->mode = tccl::kBgGatherCols;
  p->slots = heap->world_size;  // every rank's shard, the own one included
  p->rank = heap->rank;
  p->world = heap->world_size;
  p->heap_bases = heap->heap_bases;
  p->block_rows = d->M;
  p->pitch = (uint32_t)(d->lda * esz);
  p->src_pitch = (uint32_t)(gs.ld_shard * esz);
  p->upr = (uint32_t)((int64_t)gs.k_shard * esz / 16);
  p->units = (uint32_t)d->M * p->upr;
  p->pieces = (int)((p->units + tccl::kPieceUnits - 1) / tccl::kPieceUnits);
  set_row_divider(p, p->upr, p->pitch, p->src_pitch);
  p->epoch = 1;
  p->fault = c.fault;
  p->spin_ticks = c.spin_ticks;
}

bool gather_in_place(const tccl_gemm_desc* d, const tccl_device_info& dev, int k_shard, int variant) {
  if (variant == TCCL_S0_BULK || !use_macro(d, dev)) return false;
  if (d->in_dtype != d->out_dtype || (d->in_dtype != TCCL_F16 && d->in_dtype != TCCL_BF16)) return false;
  return k_shard % 64 == 0 && d->column_shards <= 1 && !(d->flags & TCCL_GEMM_B_KMAJOR);
}

// GEMM (+ optional communication role) for one of the three operations.
int run_variant(const tccl_gemm_desc* d, tccl::CommArgs& c, const tccl_sync_desc* sync, const tccl_transport_desc* tr,
                int variant, const tccl_device_info& dev, const tccl::GemmArgs& g, hipStream_t stream,
                const GatherSpec* gather = nullptr, const tccl_heap_view* heap = nullptr) {
  const int span = c.op != tccl::kOpNone ? check_comm_span(c) : 0;
  if (span) return span;
  const int total_tiles = g.tile_rows * g.tile_cols;
  const int compute = default_gemm_wgs(d, dev, total_tiles);
  tccl::SignalArgs s;
  memset(&s, 0, sizeof s);
  int64_t* trace_start = sync ? sync->trace_start_clock : nullptr;
  if (use_macro(d, dev, variant != TCCL_S0_BULK)) {
    const int wgs = default_macro_wgs(d, dev);
    const tccl::Macro m = build_macro(d, dev, wgs);
    if (variant == TCCL_S0_BULK) {
      int rc = launch_gemm256(d->in_dtype, d->out_dtype, g, m, wgs, stream);
      if (rc) return rc;
      make_bulk(&c);
      if (c.world <= 1 && c.op != tccl::kOpReduceScatter) return 0;
      return launch_comm(c, bulk_comm_wgs(dev, c), stream);
    }
    Fused256Args f;
    f.g = g;
    f.m = m;
    f.trace_start = trace_start;
    s.epoch = sync->epoch > 0 ? sync->epoch : 1;
    if (variant == TCCL_S1_TILE) {
      s.mode = tccl::kSignalTile;
      s.locks = sync->locks;
      c.granularity = tccl::kPerTile;
    } else {
      s.mode = tccl::kSignalGroup;
      s.counter = sync->counter;
      s.group_table = sync->group_table;
      s.tile_counts = sync->tile_counts;
      s.trace_ready_clock = sync->trace_ready_clock;
      c.granularity = tccl::kPerGroup;
    }
    f.s = s;
    // Pushes leave from the epilogue; what remains for the communication role are the
    // pulls (and, for a reduce-scatter, the reductions).
    if (build_push(c, g, &f.push)) c.directions &= ~tccl::kDirPush;
    memset(&f.reduce, 0, sizeof f.reduce);
    memset(&f.gather, 0, sizeof f.gather);
    if (gather) {
      build_gather_background(d, *gather, heap, c, &f.pull, &f.gather);
    } else if (build_reduce(c, sync, d->flags, &f.reduce, &f.m)) {
      c.op = tccl::kOpNone;
      memset(&f.pull, 0, sizeof f.pull);
    } else if (build_background(c, &f.pull)) {
      c.directions &= ~tccl::kDirPull;
    }
    if (c.op != tccl::kOpReduceScatter && !(c.directions & (tccl::kDirPush | tccl::kDirPull))) c.op = tccl::kOpNone;
    f.comm = c;
    return launch_fused256(d->in_dtype, d->out_dtype, f, wgs, stream);
  }
  if (variant == TCCL_S0_BULK) {
    tccl::CommArgs none;
    memset(&none, 0, sizeof none);
    int rc = launch_fused(d->in_dtype, d->out_dtype, g, s, none, compute, 0, trace_start, stream);
    if (rc) return rc;
    make_bulk(&c);
    if (c.world <= 1 && c.op != tccl::kOpReduceScatter) return 0;
    return launch_comm(c, bulk_comm_wgs(dev, c), stream);
  }
  int comm = tr && tr->num_comm_wgs > 0 ? tr->num_comm_wgs : dev.compute_units;
  s.epoch = sync->epoch > 0 ? sync->epoch : 1;
  if (variant == TCCL_S1_TILE) {
    s.mode = tccl::kSignalTile;
    s.locks = sync->locks;
    c.granularity = tccl::kPerTile;
  } else {
    s.mode = tccl::kSignalGroup;
    s.counter = sync->counter;
    s.group_table = sync->group_table;
    c.granularity = tccl::kPerGroup;
  }
  // Pushes leave from the GEMM's epilogue (the tile goes to the peers from the registers it is stored from and
  // is never read back); what remains for the communication workgroups are pulls and reductions.  A traced
  // launch keeps the pushes in the communication role, whose tasks carry the per-group clock stamps.
  tccl::PushArgs push;
  memset(&push, 0, sizeof push);
  const bool traced = sync->trace_start_clock || sync->trace_ready_clock || sync->trace_done_clock;
  if (!traced && build_push(c, g, &push)) {
    c.directions &= ~tccl::kDirPush;
    if (c.op != tccl::kOpReduceScatter && !(c.directions & tccl::kDirPull)) comm = 0;
  }
  return launch_fused(d->in_dtype, d->out_dtype, g, s, c, compute, comm, trace_start, stream, &push);
}


// GEMM-output AllGather.  word_stride: 0 when the ranks' signal words live in the heap (a
// peer's at the same slice offset), else the distance between consecutive ranks' words.
int allgather_impl(const tccl_gemm_desc* d, void* out, int64_t ld_out, const tccl_heap_view* heap, const tccl_sync_desc* sync,
                   const tccl_transport_desc* tr, int32_t variant, int64_t word_stride, hipStream_t stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  if ((rc = check_heap(heap))) return rc;
  if (variant < TCCL_S0_BULK || variant > TCCL_S2_TILEGROUP) return fail(TCCL_ERR_INVALID, "unknown variant %d", variant);
  if ((rc = check_sync(sync, variant))) return rc;
  if (!out) return fail(TCCL_ERR_INVALID, "allgather: out is NULL");
  const int esize = (int)dtype_size(d->out_dtype);
  if (ld_out != d->ldc) return fail(TCCL_ERR_INVALID, "allgather: ld_out must equal the GEMM's ldc");
  const char* want = (const char*)out + (int64_t)heap->rank * d->M * ld_out * esize;
  if ((const char*)d->C != want) return fail(TCCL_ERR_INVALID, "allgather: gemm C must point at row rank*M of out");
  if ((d->N * esize) % 16 || (ld_out * esize) % 16) return fail(TCCL_ERR_UNSUPPORTED, "allgather: rows must be multiples of 16 bytes");
  if (tr && !(tr->directions & (TCCL_DIR_PUSH | TCCL_DIR_PULL))) return fail(TCCL_ERR_INVALID, "allgather: no transfer direction selected");
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  build_gemm_args(d, dev, &g);
  tccl::CommArgs c;
  fill_comm_common(&c, g, esize, heap, sync, tr);
  c.op = tccl::kOpAllGather;
  c.out = (char*)out;
  c.ld_out_bytes = ld_out * esize;
  c.word_stride = word_stride;
  if ((rc = set_task_units(&c, tr, false))) return rc;
  return run_variant(d, c, sync, tr, variant, dev, g, stream);
}

// ---- signal words that the library keeps itself (tccl_gemm_allgather_static) --------------------
// One rank's words, then the next rank's: a peer's words are a fixed distance away.
struct StaticWords {
  int32_t locks[TCCL_STATIC_MAX_TILES];
  int32_t counter[TCCL_STATIC_MAX_GROUPS];
  int32_t barrier[TCCL_STATIC_MAX_GROUPS];
};
struct StaticScratch {
  int32_t group_table[TCCL_STATIC_MAX_TILES];
  int32_t row_starts[TCCL_STATIC_MAX_GROUPS];
  int32_t row_ends[TCCL_STATIC_MAX_GROUPS];
  int32_t tile_counts[TCCL_STATIC_MAX_GROUPS];
  StaticWords words[TCCL_MAX_WORLD];
};
// Device memory that exists from the moment the library is loaded: about 581 KiB on every
// GPU the process uses.  In host code this name is only a handle for hipGetSymbolAddress; the
// address kernels and copies may use is the one static_scratch() returns.
static __device__ __align__(256) unsigned char scratch[sizeof(StaticScratch)];

constexpr int kMaxDevices = 64;
StaticScratch* g_scratch_ptr[kMaxDevices];  // per device, resolved on first use
// Calls of tccl_gemm_allgather_static so far, per device and rank (host memory: nothing is allocated).
// Call n of a rank stores n into its locks and brings each of its TileGroup counters to n * kStaticGroupUnit,
// so what call n - 1 left behind (or what a call with another plan left) never satisfies a peer that is in
// its own call n: the guarantee tccl_gemm_allgather gets from the caller's growing launch numbers.
uint32_t g_static_calls[kMaxDevices][TCCL_MAX_WORLD];
std::mutex g_scratch_mutex;
// What every TileGroup counter of the static words grows to per call, whatever the group's tile count (the
// set-up kernel starts the counter that many tiles short of the next multiple): more than any group can hold.
constexpr int32_t kStaticGroupUnit = 2 * TCCL_STATIC_MAX_TILES;

void static_call_words(uint32_t call, int32_t tile_count, int32_t* epoch, int32_t* counter_start, int32_t* counter_ready) {
  const uint32_t n = (call - 1u) % 0x7fffffffu + 1u;  // 1 .. 2^31 - 1, then 1 again: a lock value is a positive int32
  const uint32_t ready = n * (uint32_t)kStaticGroupUnit;  // modulo 2^32, compared as sequence numbers (word_reached)
  *epoch = (int32_t)n;
  *counter_ready = (int32_t)ready;
  *counter_start = (int32_t)(ready - (uint32_t)tile_count);
}

// The current device's copy of the scratch.  The first call on a device asks the runtime for
// the symbol's address on that device (no allocation); later calls read the cached pointer.
int static_scratch(StaticScratch** out) {
  int device = -1;
  TCCL_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(TCCL_ERR_NO_DEVICE, "device %d outside [0, %d)", device, kMaxDevices);
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    TCCL_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(TCCL_ERR_NO_DEVICE, "the static scratch has no address on device %d", device);
    g_scratch_ptr[device] = (StaticScratch*)p;
  }
  *out = g_scratch_ptr[device];
  return 0;
}

// Prepares rank `rank`'s words for its call number `call` and writes the plan tables: group_table by the
// rule of build_group_table (tileccl_v2/tile_group.py:214-241: the first group whose rows contain the
// tile's first row, 0 if none), under the tile numbering of tile_coords.  A counter starts its tile count
// short of call * kStaticGroupUnit, the table of tile counts that the kernels multiply the launch number
// with holds kStaticGroupUnit for every group, and locks keep what the call before stored (a smaller
// launch number).  The other ranks' words are left as their own last call left them.
__global__ void static_setup_kernel(StaticScratch* s, tccl_static_plan plan, int rank, uint32_t call, int tile_rows, int tile_cols,
                                    int block_m, int group_m) {
  const int total = tile_rows * tile_cols;
  StaticWords* mine = &s->words[rank];
  const int first = blockIdx.x * blockDim.x + threadIdx.x, stride = gridDim.x * blockDim.x;
  for (int t = first; t < total; t += stride) {
    const int row = tccl::tile_coords(t, tile_rows, tile_cols, group_m).m * block_m;
    int gid = 0;
    for (int g = plan.n_groups - 1; g >= 0; --g)
      if (plan.row_starts[g] <= row && row < plan.row_ends[g]) gid = g;
    s->group_table[t] = gid;
  }
  for (int g = first; g < plan.n_groups; g += stride) {
    s->row_starts[g] = plan.row_starts[g];
    s->row_ends[g] = plan.row_ends[g];
    s->tile_counts[g] = kStaticGroupUnit;
    const uint32_t n = (call - 1u) % 0x7fffffffu + 1u;
    mine->counter[g] = (int32_t)(n * (uint32_t)kStaticGroupUnit - (uint32_t)plan.tile_counts[g]);
    mine->barrier[g] = 0;
  }
}

}  // namespace

// ============================================================================================
// extern "C"
// ============================================================================================
extern "C" {

int tccl_abi_version(void) { return TCCL_ABI_VERSION; }

const char* tccl_last_error_string(void) { return g_error; }

int tccl_device_query(int device, tccl_device_info* out) {
  if (!out) return fail(TCCL_ERR_INVALID, "out is NULL");
  return query_device(device, out);
}

int tccl_tile_coords(int32_t tile_id, int32_t tile_rows, int32_t tile_cols, int32_t group_m, int32_t* tile_m, int32_t* tile_n) {
  if (tile_rows <= 0 || tile_cols <= 0 || group_m <= 0 || tile_id < 0 || tile_id >= tile_rows * tile_cols || !tile_m || !tile_n)
    return fail(TCCL_ERR_INVALID, "tile_coords: bad arguments");
  const tccl::TileCoord c = tccl::tile_coords(tile_id, tile_rows, tile_cols, group_m);
  *tile_m = c.m;
  *tile_n = c.n;
  return 0;
}

int tccl_tile_for_slot(int32_t slot, int32_t total_tiles, int32_t xcds, int32_t span, int32_t* tile_id) {
  if (slot < 0 || slot >= total_tiles || xcds <= 0 || span <= 0 || !tile_id) return fail(TCCL_ERR_INVALID, "tile_for_slot: bad arguments");
  *tile_id = tccl::tile_for_slot(slot, total_tiles, xcds, span);
  return 0;
}

int tccl_heap_create(size_t slice_bytes, int world_size, void** arena_out, int64_t* bases_out) {
  if (!arena_out || !bases_out) return fail(TCCL_ERR_INVALID, "heap_create: NULL output");
  if (slice_bytes == 0) return fail(TCCL_ERR_INVALID, "heap_create: slice size must be positive");
  if (world_size < 1 || world_size > TCCL_MAX_WORLD) return fail(TCCL_ERR_INVALID, "heap_create: world_size=%d outside [1, %d]", world_size, TCCL_MAX_WORLD);
  // Slices start on 2 MiB boundaries so that symmetric offsets keep page alignment.
  const size_t align = 2u << 20;
  const size_t stride = (slice_bytes + align - 1) / align * align;
  void* p = nullptr;
  TCCL_HIP(hipMalloc(&p, stride * (size_t)world_size));
  *arena_out = p;
  for (int r = 0; r < world_size; ++r) bases_out[r] = (int64_t)(uintptr_t)p + (int64_t)(stride * (size_t)r);
  return 0;
}

int tccl_heap_destroy(void* arena) {
  if (!arena) return 0;
  TCCL_HIP(hipFree(arena));
  return 0;
}

int tccl_fill_i32(int32_t* words, int64_t n, int32_t value, void* stream) {
  if (n <= 0) return 0;
  if (!words) return fail(TCCL_ERR_INVALID, "fill: NULL pointer");
  int blocks = (int)((n + 255) / 256);
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(fill_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, words, n, value);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_pack_matrix(const void* src, int64_t stride_row, int64_t stride_col, int32_t rows, int32_t cols, void* dst,
                     int64_t ld_dst, int32_t dst_rows, int32_t dst_cols, int32_t elem_bytes, void* stream) {
  if (dst_rows <= 0 || dst_cols <= 0) return 0;
  if (!src || !dst) return fail(TCCL_ERR_INVALID, "pack_matrix: NULL pointer");
  if (rows < 0 || cols < 0 || rows > dst_rows || cols > dst_cols || stride_row < 0 || stride_col < 0 || ld_dst < dst_cols)
    return fail(TCCL_ERR_INVALID, "pack_matrix: source %dx%d (strides %lld, %lld) does not fit a %dx%d destination of pitch %lld",
                rows, cols, (long long)stride_row, (long long)stride_col, dst_rows, dst_cols, (long long)ld_dst);
  const dim3 grid((unsigned)((dst_cols + 63) / 64), (unsigned)((dst_rows + 63) / 64));
  if (grid.y > 65535u) return fail(TCCL_ERR_UNSUPPORTED, "pack_matrix: more than 65535 x 64 rows");
  const hipStream_t st = (hipStream_t)stream;
  if (elem_bytes == 1)
    hipLaunchKernelGGL(pack_kernel<uint8_t>, grid, dim3(256), 0, st, (const uint8_t*)src, stride_row, stride_col, rows, cols,
                       (uint8_t*)dst, ld_dst, dst_rows, dst_cols);
  else if (elem_bytes == 2)
    hipLaunchKernelGGL(pack_kernel<uint16_t>, grid, dim3(256), 0, st, (const uint16_t*)src, stride_row, stride_col, rows, cols,
                       (uint16_t*)dst, ld_dst, dst_rows, dst_cols);
  else if (elem_bytes == 4)
    hipLaunchKernelGGL(pack_kernel<uint32_t>, grid, dim3(256), 0, st, (const uint32_t*)src, stride_row, stride_col, rows, cols,
                       (uint32_t*)dst, ld_dst, dst_rows, dst_cols);
  else
    return fail(TCCL_ERR_INVALID, "pack_matrix: elem_bytes=%d must be 1, 2 or 4", elem_bytes);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_prim_signal(int32_t* locks, int32_t index, void* stream) {
  if (!locks || index < 0) return fail(TCCL_ERR_INVALID, "prim_signal: bad arguments");
  hipLaunchKernelGGL(prim_signal_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, locks, index);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_prim_signal_add(int32_t* words, int32_t index, int32_t value, int32_t* result, void* stream) {
  if (!words || !result || index < 0) return fail(TCCL_ERR_INVALID, "prim_signal_add: bad arguments");
  hipLaunchKernelGGL(prim_signal_add_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, words, index, value, result);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_prim_try_wait(int32_t* locks, int32_t index, int32_t max_spins, int32_t consume, int32_t* result, void* stream) {
  if (!locks || !result || index < 0 || max_spins < 0) return fail(TCCL_ERR_INVALID, "prim_try_wait: bad arguments");
  hipLaunchKernelGGL(prim_try_wait_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, locks, index, max_spins, consume, result);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_prim_wait_ge(int32_t* words, int32_t index, int32_t threshold, int64_t spin_limit_ns, int32_t* result, void* stream) {
  if (!words || !result || index < 0) return fail(TCCL_ERR_INVALID, "prim_wait_ge: bad arguments");
  if (spin_limit_ns <= 0 || spin_limit_ns > kDefaultSpinNs) spin_limit_ns = kDefaultSpinNs;
  hipLaunchKernelGGL(prim_wait_ge_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, words, index, threshold, spin_limit_ns / 10 + 1, result);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_gemm(const tccl_gemm_desc* d, void* stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  build_gemm_args(d, dev, &g);
  tccl::SignalArgs s;
  memset(&s, 0, sizeof s);
  if (use_macro(d, dev, false)) {
    const int wgs = default_macro_wgs(d, dev);
    return launch_gemm256(d->in_dtype, d->out_dtype, g, build_macro(d, dev, wgs), wgs, (hipStream_t)stream);
  }
  tccl::CommArgs none;
  memset(&none, 0, sizeof none);
  return launch_fused(d->in_dtype, d->out_dtype, g, s, none, default_gemm_wgs(d, dev, g.tile_rows * g.tile_cols), 0, nullptr,
                      (hipStream_t)stream);
}

static int check_scatter(const tccl_scatter_desc* sc, int M, int N, int esize, int64_t ldc, const void* C) {
  if (!sc) return fail(TCCL_ERR_INVALID, "scatter descriptor is NULL");
  if (sc->cols <= 0 || sc->src_col_offset < 0 || sc->dst_col_offset < 0 || sc->dst_ld <= 0)
    return fail(TCCL_ERR_INVALID, "scatter: bad placement (src_col_offset=%d cols=%d dst_ld=%d dst_col_offset=%d)", sc->src_col_offset, sc->cols, sc->dst_ld, sc->dst_col_offset);
  if (sc->src_col_offset + sc->cols > N) return fail(TCCL_ERR_INVALID, "scatter: source columns [%d, %d) exceed N=%d", sc->src_col_offset, sc->src_col_offset + sc->cols, N);
  if (sc->dst_col_offset + sc->cols > sc->dst_ld) return fail(TCCL_ERR_INVALID, "scatter: destination columns exceed dst_ld");
  const int v = 16 / esize;
  if (sc->src_col_offset % v || sc->cols % v || sc->dst_col_offset % v || sc->dst_ld % v || ldc % v || !aligned16(C))
    return fail(TCCL_ERR_UNSUPPORTED, "scatter: column offsets, widths and leading dimensions must be multiples of %d elements", v);
  (void)M;
  return 0;
}

int tccl_scatter_cols(const void* C, int32_t M, int64_t ldc, int32_t elem_bytes, const tccl_scatter_desc* sc,
                      const tccl_heap_view* heap, void* stream) {
  int rc = check_heap(heap);
  if (rc) return rc;
  if (!C || M <= 0 || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4)) return fail(TCCL_ERR_INVALID, "scatter_cols: bad arguments");
  if (!sc) return fail(TCCL_ERR_INVALID, "scatter descriptor is NULL");
  const int N = sc->src_col_offset + sc->cols;
  if ((rc = check_scatter(sc, M, N, elem_bytes, ldc, C))) return rc;
  if (heap->world_size == 1) return 0;
  if ((rc = check_rows_span(M, (ldc > sc->dst_ld ? ldc : (int64_t)sc->dst_ld) * elem_bytes))) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  memset(&g, 0, sizeof g);
  g.C = (void*)C;
  g.M = M;
  g.N = N;
  g.ldc = ldc;
  g.block_m = g.block_n = 128;
  g.group_m = 8;
  g.tile_rows = (M + 127) / 128;
  g.tile_cols = (N + 127) / 128;
  g.xcds = 1;
  g.span = 1;
  tccl::CommArgs c;
  fill_comm_common(&c, g, elem_bytes, heap, nullptr, nullptr);
  c.op = tccl::kOpAllScatter;
  c.granularity = tccl::kBulk;
  c.src_col_off = sc->src_col_offset;
  c.cols = sc->cols;
  c.dst_ld = sc->dst_ld;
  c.dst_col_off = sc->dst_col_offset;
  if ((rc = set_task_units(&c, nullptr, false))) return rc;
  return launch_comm(c, bulk_comm_wgs(dev, c), (hipStream_t)stream);
}

int tccl_exchange_rows(void* out, int32_t rows_per_rank, int32_t N, int64_t ld, int32_t elem_bytes,
                       const tccl_heap_view* heap, const tccl_transport_desc* tr, void* stream) {
  int rc = check_heap(heap);
  if (rc) return rc;
  if (!out || rows_per_rank <= 0 || N <= 0 || ld < N || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4))
    return fail(TCCL_ERR_INVALID, "exchange_rows: bad arguments");
  const int v = 16 / elem_bytes;
  if (N % v || ld % v || !aligned16(out)) return fail(TCCL_ERR_UNSUPPORTED, "exchange_rows: rows must be multiples of 16 bytes");
  if (heap->world_size == 1) return 0;
  if ((rc = check_rows_span(rows_per_rank, ld * elem_bytes))) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  memset(&g, 0, sizeof g);
  g.C = (char*)out + (int64_t)heap->rank * rows_per_rank * ld * elem_bytes;
  g.M = rows_per_rank;
  g.N = N;
  g.ldc = ld;
  g.block_m = g.block_n = 128;
  g.group_m = 8;
  g.tile_rows = (rows_per_rank + 127) / 128;
  g.tile_cols = (N + 127) / 128;
  g.xcds = 1;
  g.span = 1;
  tccl::CommArgs c;
  fill_comm_common(&c, g, elem_bytes, heap, nullptr, tr);
  c.op = tccl::kOpAllGather;
  c.granularity = tccl::kBulk;
  c.out = (char*)out;
  c.ld_out_bytes = ld * elem_bytes;
  if ((rc = set_task_units(&c, tr, false))) return rc;
  return launch_comm(c, bulk_comm_wgs(dev, c), (hipStream_t)stream);
}

int tccl_copy_block(void* dst, uint32_t dst_ranks, const void* src, int32_t src_rank, int32_t rows, int64_t row_bytes,
                    int64_t src_pitch_bytes, int64_t dst_pitch_bytes, const tccl_heap_view* heap, void* stream) {
  int rc = check_heap(heap);
  if (rc) return rc;
  if (!dst || !src || rows <= 0 || row_bytes <= 0 || src_pitch_bytes < row_bytes || dst_pitch_bytes < row_bytes)
    return fail(TCCL_ERR_INVALID, "copy_block: bad arguments");
  if (src_rank < 0 || src_rank >= heap->world_size)
    return fail(TCCL_ERR_INVALID, "copy_block: src_rank=%d out of range for world_size=%d", src_rank, heap->world_size);
  if (heap->world_size < 32 && (dst_ranks >> heap->world_size))
    return fail(TCCL_ERR_INVALID, "copy_block: dst_ranks=0x%x names ranks beyond world_size=%d", dst_ranks, heap->world_size);
  if (row_bytes % 16 || src_pitch_bytes % 16 || dst_pitch_bytes % 16 || !aligned16(dst) || !aligned16(src))
    return fail(TCCL_ERR_UNSUPPORTED, "copy_block: rows must be multiples of 16 bytes and 16-byte aligned");
  if (row_bytes > 0x7fffffffll) return fail(TCCL_ERR_UNSUPPORTED, "copy_block: rows of %lld bytes (limit 2 GiB)", (long long)row_bytes);
  if ((rc = check_rows_span(rows, src_pitch_bytes > dst_pitch_bytes ? src_pitch_bytes : dst_pitch_bytes))) return rc;
  if (dst_ranks == 0) return 0;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  memset(&g, 0, sizeof g);
  g.C = (void*)src;
  g.M = rows;
  g.N = (int)row_bytes;
  g.ldc = src_pitch_bytes;
  g.block_m = g.block_n = 128;
  g.group_m = 8;
  g.tile_rows = (rows + 127) / 128;
  g.tile_cols = (int)((row_bytes + 127) / 128);
  g.xcds = 1;
  g.span = 1;
  tccl::CommArgs c;
  fill_comm_common(&c, g, 1, heap, nullptr, nullptr);
  c.op = tccl::kOpCopyBlock;
  c.granularity = tccl::kBulk;
  c.out = (char*)dst;
  c.ld_out_bytes = dst_pitch_bytes;
  c.copy_src_rank = src_rank;
  c.copy_dst_ranks = dst_ranks;
  // 32 KiB per task, whatever the element type of the caller's data
  c.copy_units = c.reduce_units = 2048;
  return launch_comm(c, bulk_comm_wgs(dev, c), (hipStream_t)stream);
}

int tccl_gather_cols(void* gathered, int64_t ld_gathered, const void* shard, int64_t ld_shard, int32_t M,
                     int32_t cols, int32_t elem_bytes, const tccl_heap_view* heap, const tccl_transport_desc* tr,
                     void* stream) {
  int rc = check_heap(heap);
  if (rc) return rc;
  if (!gathered || !shard || M <= 0 || cols <= 0 || ld_shard < cols || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4))
    return fail(TCCL_ERR_INVALID, "gather_cols: bad arguments");
  if (ld_gathered < (int64_t)cols * heap->world_size)
    return fail(TCCL_ERR_INVALID, "gather_cols: gathered rows hold %lld elements, need %lld", (long long)ld_gathered,
                (long long)cols * heap->world_size);
  const int v = 16 / elem_bytes;
  if (cols % v || ld_shard % v || ld_gathered % v || !aligned16(gathered) || !aligned16(shard))
    return fail(TCCL_ERR_UNSUPPORTED, "gather_cols: shard rows must be multiples of 16 bytes and 16-byte aligned");
  if ((rc = check_rows_span(M, (ld_gathered > ld_shard ? ld_gathered : ld_shard) * elem_bytes))) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  memset(&g, 0, sizeof g);
  g.C = (void*)shard;
  g.M = M;
  g.N = cols;
  g.ldc = ld_shard;
  g.block_m = g.block_n = 128;
  g.group_m = 8;
  g.tile_rows = (M + 127) / 128;
  g.tile_cols = (cols + 127) / 128;
  g.xcds = 1;
  g.span = 1;
  tccl::CommArgs c;
  fill_comm_common(&c, g, elem_bytes, heap, nullptr, tr);
  c.op = tccl::kOpGatherCols;
  c.granularity = tccl::kBulk;
  c.directions = TCCL_DIR_PUSH | TCCL_DIR_PULL;  // the own shard is copied, the peers' are pulled
  c.out = (char*)gathered;
  c.ld_out_bytes = ld_gathered * elem_bytes;
  if ((rc = set_task_units(&c, tr, false))) return rc;
  return launch_comm(c, bulk_comm_wgs(dev, c), (hipStream_t)stream);
}

static int fill_reduce(tccl::CommArgs* c, const void* partial, int partial_dtype, void* out, int out_dtype, int64_t ld_out,
                       int M, int N, int world, int emulate_peer, bool allow_f32_out = false) {
  if (partial_dtype != TCCL_F16 && partial_dtype != TCCL_BF16 && partial_dtype != TCCL_F32)
    return fail(TCCL_ERR_UNSUPPORTED, "reduce: partial dtype %d", partial_dtype);
  if (out_dtype == TCCL_F32 && !(allow_f32_out && partial_dtype == TCCL_F32))
    return fail(TCCL_ERR_UNSUPPORTED, "reduce: fp32 output only from fp32 partials in the stand-alone reduction");
  if (out_dtype != TCCL_F16 && out_dtype != TCCL_BF16 && out_dtype != TCCL_F32)
    return fail(TCCL_ERR_UNSUPPORTED, "reduce: output dtype must be fp16, bf16 or fp32");
  if (partial_dtype != TCCL_F32 && partial_dtype != out_dtype && !(partial_dtype == TCCL_BF16 || partial_dtype == TCCL_F16))
    return fail(TCCL_ERR_UNSUPPORTED, "reduce: dtype combination");
  if (M % world) return fail(TCCL_ERR_INVALID, "reduce: M=%d must be divisible by world_size=%d", M, world);
  if (N % 8 || ld_out % 8 || !aligned16(out) || !aligned16(partial)) return fail(TCCL_ERR_UNSUPPORTED, "reduce: rows must be multiples of 8 elements and 16-byte aligned");
  c->op = tccl::kOpReduceScatter;
  c->rs_out = (char*)out;
  c->ld_rs_out_bytes = ld_out * (out_dtype == TCCL_F32 ? 4 : 2);
  c->partial_dtype = partial_dtype;
  c->out_dtype = out_dtype;
  c->emulate_peer = (emulate_peer & TCCL_RS_EMULATE_PEERS) != 0;
  c->peers_resident = (emulate_peer & TCCL_RS_PEERS_RESIDENT) != 0;
  // Without a plan the kernel works shard by shard (one implicit group per owner).
  if (!c->row_starts) c->n_groups = world;
  return 0;
}

int tccl_reduce_rows(const void* partial, int32_t partial_dtype, int64_t ld_partial, void* out, int32_t out_dtype,
                     int64_t ld_out, int32_t M, int32_t N, const tccl_heap_view* heap, const tccl_transport_desc* tr,
                     int32_t emulate_peer, void* stream) {
  int rc = check_heap(heap);
  if (rc) return rc;
  if (!partial || !out || M <= 0 || N <= 0 || ld_partial < N || ld_out < N) return fail(TCCL_ERR_INVALID, "reduce_rows: bad arguments");
  const int esize = (int)dtype_size(partial_dtype);
  if (!esize || ld_partial % (16 / esize)) return fail(TCCL_ERR_UNSUPPORTED, "reduce_rows: partial rows must be 16-byte multiples");
  if ((rc = check_rows_span(M, ld_partial * esize)) || (rc = check_rows_span(M, ld_out * 4))) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  memset(&g, 0, sizeof g);
  g.C = (void*)partial;
  g.M = M;
  g.N = N;
  g.ldc = ld_partial;
  g.block_m = g.block_n = 128;
  g.group_m = 8;
  g.tile_rows = (M + 127) / 128;
  g.tile_cols = (N + 127) / 128;
  g.xcds = 1;
  g.span = 1;
  tccl::CommArgs c;
  fill_comm_common(&c, g, esize, heap, nullptr, tr);
  if ((rc = fill_reduce(&c, partial, partial_dtype, out, out_dtype, ld_out, M, N, heap->world_size, emulate_peer, true))) return rc;
  c.granularity = tccl::kBulk;
  if ((rc = set_task_units(&c, tr, true))) return rc;
  return launch_comm(c, bulk_comm_wgs(dev, c), (hipStream_t)stream);
}

static int allscatter_impl(const tccl_gemm_desc* d, const tccl_scatter_desc* sc, const tccl_heap_view* heap,
                           const tccl_sync_desc* sync, const tccl_transport_desc* tr, int32_t variant, const GatherSpec* gather,
                           hipStream_t stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  if ((rc = check_heap(heap))) return rc;
  if (variant < TCCL_S0_BULK || variant > TCCL_S2_TILEGROUP) return fail(TCCL_ERR_INVALID, "unknown variant %d", variant);
  if ((rc = check_sync(sync, variant))) return rc;
  const int esize = (int)dtype_size(d->out_dtype);
  if ((rc = check_scatter(sc, d->M, d->N, esize, d->ldc, d->C))) return rc;
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  build_gemm_args(d, dev, &g);
  tccl::CommArgs c;
  fill_comm_common(&c, g, esize, heap, sync, tr);
  c.op = tccl::kOpAllScatter;
  c.directions = TCCL_DIR_PUSH;
  c.src_col_off = sc->src_col_offset;
  c.cols = sc->cols;
  c.dst_ld = sc->dst_ld;
  c.dst_col_off = sc->dst_col_offset;
  if ((rc = set_task_units(&c, tr, false))) return rc;
  return run_variant(d, c, sync, tr, variant, dev, g, stream, gather, heap);
}

int tccl_collective_staged(int32_t op, const void* src, void* dst, int32_t dtype, int64_t block_elems, void* staging,
                           int32_t* published, int32_t* consumed, int32_t chunk_elems, int32_t slots, int32_t base_epoch,
                           uint32_t ranks, int32_t root, const tccl_heap_view* heap, int64_t* fault, int64_t spin_limit_ns,
                           void* stream) {
  static const char* const names[] = {"allreduce", "allgather", "reduce_scatter", "broadcast", "scatter"};
  int rc = check_heap(heap);
  if (rc) return rc;
  if (op < TCCL_STAGED_ALLREDUCE || op > TCCL_STAGED_SCATTER) return fail(TCCL_ERR_INVALID, "collective_staged: unknown op %d", op);
  const char* name = names[op];
  const bool reduces = op == TCCL_STAGED_ALLREDUCE || op == TCCL_STAGED_REDUCE_SCATTER;
  const bool in_place = op == TCCL_STAGED_ALLREDUCE || op == TCCL_STAGED_BROADCAST;
  const bool rooted = op == TCCL_STAGED_BROADCAST || op == TCCL_STAGED_SCATTER;
  const int esize = (int)dtype_size(dtype);
  if (!esize || (reduces && dtype != TCCL_F16 && dtype != TCCL_BF16 && dtype != TCCL_F32))
    return fail(TCCL_ERR_UNSUPPORTED, "%s_staged: dtype %d", name, dtype);
  if (!dst || (!in_place && !src) || !staging || !published || !consumed || block_elems <= 0 || chunk_elems <= 0 || slots <= 0 ||
      base_epoch < 1)
    return fail(TCCL_ERR_INVALID, "%s_staged: bad arguments", name);
  if (rooted && (root < 0 || root >= heap->world_size)) return fail(TCCL_ERR_INVALID, "%s_staged: root=%d out of range [0, %d)", name, root, heap->world_size);
  const int per_unit = 16 / esize;
  if (block_elems % per_unit || chunk_elems % per_unit || !aligned16(dst) || !aligned16(src) || !aligned16(staging))
    return fail(TCCL_ERR_UNSUPPORTED, "%s_staged: blocks and chunks must be whole 16-byte units (%d elements)", name, per_unit);
  if ((int64_t)chunk_elems * esize * heap->world_size > 0x7fffffffll) return fail(TCCL_ERR_UNSUPPORTED, "%s_staged: chunk too large", name);
  if (heap->world_size < 32 && (ranks >> heap->world_size))
    return fail(TCCL_ERR_INVALID, "%s_staged: ranks=0x%x names ranks beyond world_size=%d", name, ranks, heap->world_size);
  const int roles = __builtin_popcount(ranks);
  if (roles == 0) return 0;
  const int64_t chunks = (block_elems + chunk_elems - 1) / chunk_elems;
  if ((int64_t)base_epoch + chunks > 0x7fffffffll) return fail(TCCL_ERR_INVALID, "%s_staged: epoch range overflows int32", name);
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  // Every (rank, slot) workgroup waits on others of the same launch: all must be resident.
  if ((int64_t)roles * slots > (int64_t)dev.compute_units * 4)
    return fail(TCCL_ERR_UNSUPPORTED, "%s_staged: %d roles x %d slots exceed what the device keeps resident (%d workgroups)", name, roles,
                slots, dev.compute_units * 4);
  tccl::StagedArgs a;
  memset(&a, 0, sizeof a);
  a.heap_bases = heap->heap_bases;
  a.rank = heap->rank;
  a.world = heap->world_size;
  a.ranks = ranks;
  a.op = op;
  a.root = root;
  a.src = (char*)src;
  a.dst = (char*)dst;
  a.staging = (char*)staging;
  a.published = published;
  a.consumed = consumed;
  a.units = block_elems / per_unit;
  a.chunk_units = chunk_elems / per_unit;
  a.slots = slots;
  a.base_epoch = base_epoch;
  a.dtype = reduces ? dtype : TCCL_F16;  // copies move bytes
  a.fault = fault;
  a.spin_ticks = (spin_limit_ns > 0 ? spin_limit_ns : kDefaultSpinNs) / 10 + 1;
  hipLaunchKernelGGL(staged_kernel, dim3(roles * slots), dim3(256), 0, (hipStream_t)stream, a);
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_allreduce_staged(void* tensor, int32_t dtype, int64_t numel, void* staging, int32_t* published, int32_t* consumed,
                          int32_t chunk_elems, int32_t slots, int32_t base_epoch, uint32_t ranks, const tccl_heap_view* heap,
                          int64_t* fault, int64_t spin_limit_ns, void* stream) {
  return tccl_collective_staged(TCCL_STAGED_ALLREDUCE, nullptr, tensor, dtype, numel, staging, published, consumed, chunk_elems, slots,
                                base_epoch, ranks, 0, heap, fault, spin_limit_ns, stream);
}

int tccl_gemm_allscatter(const tccl_gemm_desc* d, const tccl_scatter_desc* sc, const tccl_heap_view* heap,
                         const tccl_sync_desc* sync, const tccl_transport_desc* tr, int32_t variant, void* stream) {
  return allscatter_impl(d, sc, heap, sync, tr, variant, nullptr, (hipStream_t)stream);
}

int tccl_chained_ag_gemm_rs(const tccl_gemm_desc* d, const void* shard, int64_t ld_shard, int32_t k_shard,
                            const tccl_heap_view* heap, const tccl_sync_desc* sync, const tccl_transport_desc* tr,
                            int32_t variant, void* stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  if ((rc = check_heap(heap))) return rc;
  if (k_shard <= 0 || (int64_t)k_shard * heap->world_size != d->K)
    return fail(TCCL_ERR_INVALID, "chained: input_shard columns (%d) * world_size (%d) != W rows (%d)", k_shard,
                heap->world_size, d->K);
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  // Stages 2 and 3: the GEMM, whose whole output goes to every peer's output.
  tccl_scatter_desc sc;
  sc.src_col_offset = 0;
  sc.cols = d->N;
  sc.dst_ld = (int32_t)d->ldc;
  sc.dst_col_offset = 0;
  const int esz = (int)dtype_size(d->in_dtype);
  const bool shard_ok = shard && ld_shard >= k_shard && (ld_shard * esz) % 16 == 0 && ((int64_t)k_shard * esz) % 16 == 0 &&
                        aligned16(shard) && (255 * ld_shard + k_shard) * (int64_t)esz <= 0xffffffffll;
  if (shard_ok && gather_in_place(d, dev, k_shard, variant)) {
    // One launch: the K loops read every rank's shard where it lies, and the gathered
    // workspace (gemm->A) is filled on the side while they run.
    if ((rc = check_rows_span(d->M, (d->lda > ld_shard ? d->lda : ld_shard) * esz))) return rc;
    const GatherSpec gs{shard, ld_shard, k_shard};
    return allscatter_impl(d, &sc, heap, sync, tr, variant, &gs, (hipStream_t)stream);
  }
  // Stage 1 as a launch of its own: the gathered input (gemm->A) is filled from every rank's shard.
  if ((rc = tccl_gather_cols((void*)d->A, d->lda, shard, ld_shard, d->M, k_shard, (int32_t)esz, heap, tr, stream)))
    return rc;
  return allscatter_impl(d, &sc, heap, sync, tr, variant, nullptr, (hipStream_t)stream);
}

int tccl_gemm_allgather(const tccl_gemm_desc* d, void* out, int64_t ld_out, const tccl_heap_view* heap,
                        const tccl_sync_desc* sync, const tccl_transport_desc* tr, int32_t variant, void* stream) {
  return allgather_impl(d, out, ld_out, heap, sync, tr, variant, 0, (hipStream_t)stream);
}

int tccl_gemm_allgather_static(const tccl_gemm_desc* d, void* out, int64_t ld_out, const tccl_heap_view* heap,
                               const tccl_static_plan* plan, const tccl_transport_desc* tr, int32_t variant,
                               int64_t* fault, int64_t spin_limit_ns, void* stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  if ((rc = check_heap(heap))) return rc;
  if (variant != TCCL_S1_TILE && variant != TCCL_S2_TILEGROUP)
    return fail(TCCL_ERR_INVALID, "allgather_static: variant %d keeps no signal words; use tccl_gemm_allgather with sync = NULL", variant);
  if (!plan) return fail(TCCL_ERR_INVALID, "allgather_static: plan is NULL");
  if (plan->n_groups < 1 || plan->n_groups > TCCL_STATIC_MAX_GROUPS)
    return fail(TCCL_ERR_INVALID, "allgather_static: n_groups=%d outside [1, %d]", plan->n_groups, TCCL_STATIC_MAX_GROUPS);
  const int tile_rows = (d->M + d->block_m - 1) / d->block_m, tile_cols = (d->N + d->block_n - 1) / d->block_n;
  const int64_t tiles = (int64_t)tile_rows * tile_cols;
  if (tiles > TCCL_STATIC_MAX_TILES)
    return fail(TCCL_ERR_UNSUPPORTED, "allgather_static: %lld plan tiles exceed the static scratch (%d tiles)", (long long)tiles, TCCL_STATIC_MAX_TILES);
  for (int g = 0; g < plan->n_groups; ++g)
    if (plan->row_starts[g] < 0 || plan->row_ends[g] <= plan->row_starts[g] || plan->row_ends[g] > d->M || plan->tile_counts[g] <= 0 ||
        (g > 0 && plan->row_starts[g] < plan->row_ends[g - 1]))
      return fail(TCCL_ERR_INVALID, "allgather_static: group %d = rows [%d, %d), %d tiles is not an ascending cover of M=%d", g,
                  plan->row_starts[g], plan->row_ends[g], plan->tile_counts[g], d->M);
  StaticScratch* sc = nullptr;
  if ((rc = static_scratch(&sc))) return rc;
  int device = -1;
  TCCL_HIP(hipGetDevice(&device));
  uint32_t call;
  {
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    call = ++g_static_calls[device][heap->rank];
  }
  int32_t epoch, start, ready;
  static_call_words(call, 0, &epoch, &start, &ready);
  // One small kernel prepares this rank's words for this call and (re)writes the plan tables; it is
  // ordered before the fused launch by the stream.  Nothing is allocated and nothing is memset.
  const int threads = 256;
  int blocks = (int)((tiles + threads - 1) / threads);
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(static_setup_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, sc, *plan, heap->rank, call, tile_rows,
                     tile_cols, d->block_m, d->group_m);
  TCCL_HIP(hipGetLastError());
  tccl_sync_desc sync;
  memset(&sync, 0, sizeof sync);
  StaticWords* mine = &sc->words[heap->rank];
  sync.locks = mine->locks;
  sync.counter = mine->counter;
  sync.barrier = mine->barrier;
  sync.group_table = sc->group_table;
  sync.row_starts = sc->row_starts;
  sync.row_ends = sc->row_ends;
  sync.tile_counts = sc->tile_counts;
  sync.n_groups = plan->n_groups;
  sync.epoch = epoch;
  sync.fault = fault;
  sync.spin_limit_ns = spin_limit_ns;
  return allgather_impl(d, out, ld_out, heap, &sync, tr, variant, (int64_t)sizeof(StaticWords), (hipStream_t)stream);
}

int tccl_static_call_words(uint32_t call, int32_t tile_count, int32_t* epoch, int32_t* counter_start, int32_t* counter_ready) {
  if (call == 0 || tile_count < 0 || tile_count > TCCL_STATIC_MAX_TILES || !epoch || !counter_start || !counter_ready)
    return fail(TCCL_ERR_INVALID, "static_call_words: call numbers start at 1, tile_count within [0, %d]", TCCL_STATIC_MAX_TILES);
  static_call_words(call, tile_count, epoch, counter_start, counter_ready);
  return 0;
}

int tccl_word_reached(int32_t word, int32_t need) { return tccl::word_reached(word, need) ? 1 : 0; }

int tccl_mfma_rate_probe(int32_t kind, const void* a_like, int64_t a_bytes, const void* b_like, int64_t b_bytes, float* sink,
                         int32_t steps, int32_t workgroups, void* stream) {
  if (!a_like || !b_like || !sink) return fail(TCCL_ERR_INVALID, "mfma_rate_probe: NULL buffer");
  if (a_bytes < 32 || b_bytes < 32 || a_bytes % 32 || b_bytes % 32 || a_bytes > 0x7fffffffll || b_bytes > 0x7fffffffll)
    return fail(TCCL_ERR_INVALID, "mfma_rate_probe: operand buffers must hold a multiple of 32 bytes, below 2 GiB (got %lld, %lld)",
                (long long)a_bytes, (long long)b_bytes);
  if (steps < 0 || workgroups < 1) return fail(TCCL_ERR_INVALID, "mfma_rate_probe: steps=%d, workgroups=%d", steps, workgroups);
  const dim3 grid(workgroups), block(tccl::kThreads256);
  const char* a = (const char*)a_like;
  const char* b = (const char*)b_like;
  const uint32_t an = (uint32_t)a_bytes, bn = (uint32_t)b_bytes;
  hipStream_t st = (hipStream_t)stream;
  switch (kind) {
    case TCCL_PROBE_F16_32X32X16: hipLaunchKernelGGL((tccl::mfma_rate_wide_kernel<_Float16>), grid, block, 0, st, a, an, b, bn, sink, steps); break;
    case TCCL_PROBE_F16_16X16X32: hipLaunchKernelGGL((tccl::mfma_rate_kernel<_Float16>), grid, block, 0, st, a, an, b, bn, sink, steps); break;
    case TCCL_PROBE_BF16_16X16X32: hipLaunchKernelGGL((tccl::mfma_rate_kernel<__bf16>), grid, block, 0, st, a, an, b, bn, sink, steps); break;
    case TCCL_PROBE_F8_16X16X128: hipLaunchKernelGGL((tccl::mfma_rate_kernel<tccl::fp8e4m3>), grid, block, 0, st, a, an, b, bn, sink, steps); break;
    case TCCL_PROBE_F8_32X32X64: hipLaunchKernelGGL((tccl::mfma_rate_wide_kernel<tccl::fp8e4m3>), grid, block, 0, st, a, an, b, bn, sink, steps); break;
    default: return fail(TCCL_ERR_INVALID, "mfma_rate_probe: unknown kind %d", kind);
  }
  TCCL_HIP(hipGetLastError());
  return 0;
}

int tccl_static_reset(void* stream) {
  StaticScratch* sc = nullptr;
  int rc = static_scratch(&sc);
  if (rc) return rc;
  int device = -1;
  TCCL_HIP(hipGetDevice(&device));
  {
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    for (int r = 0; r < TCCL_MAX_WORLD; ++r) g_static_calls[device][r] = 0;
  }
  return tccl_fill_i32((int32_t*)sc->words, (int64_t)(sizeof(sc->words) / sizeof(int32_t)), 0, stream);
}

int tccl_gemm_reducescatter(const tccl_gemm_desc* d, void* out, int32_t out_dtype, int64_t ld_out,
                            const tccl_heap_view* heap, const tccl_sync_desc* sync, const tccl_transport_desc* tr,
                            int32_t emulate_peer, int32_t variant, void* stream) {
  int rc = check_gemm(d);
  if (rc) return rc;
  if ((rc = check_heap(heap))) return rc;
  if (variant < TCCL_S0_BULK || variant > TCCL_S2_TILEGROUP) return fail(TCCL_ERR_INVALID, "unknown variant %d", variant);
  if ((rc = check_sync(sync, variant))) return rc;
  if (!out || ld_out < d->N) return fail(TCCL_ERR_INVALID, "reducescatter: bad output");
  const int esize = (int)dtype_size(d->out_dtype);
  const int shard = d->M / heap->world_size;
  if (d->M % heap->world_size || shard % d->block_m)
    return fail(TCCL_ERR_INVALID, "reducescatter: M=%d must split into world_size=%d shards of whole %d-row plan tiles", d->M, heap->world_size, d->block_m);
  tccl_device_info dev;
  if ((rc = query_device(-1, &dev))) return rc;
  tccl::GemmArgs g;
  build_gemm_args(d, dev, &g);
  tccl::CommArgs c;
  fill_comm_common(&c, g, esize, heap, sync, tr);
  if ((rc = fill_reduce(&c, d->C, d->out_dtype, out, out_dtype, ld_out, d->M, d->N, heap->world_size, emulate_peer))) return rc;
  if ((rc = set_task_units(&c, tr, true))) return rc;
  return run_variant(d, c, sync, tr, variant, dev, g, (hipStream_t)stream);
}

}  // extern "C"
