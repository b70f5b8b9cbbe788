/* A plain C program on the library's C ABI: no Python, no torch.
 *
 * Two ranks as slices of one arena.  Each computes C_r = A_r @ B (256 x 128 @ 128 x 256, fp16
 * operands holding small integers, so every output value is an integer that fp16 holds exactly)
 * and gathers the blocks with the TileGroup variant of tccl_gemm_allgather_static, the entry
 * point that needs no signal words from the caller.  Both ranks' gathered outputs are compared
 * with an integer matrix product computed here on the host, value for value.
 *
 * Exit status 0 and a last line "ok" on success; a message and status 1 otherwise. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tileccl_hip.h"

enum { WORLD = 2, M = 256, N = 256, K = 128 };
enum { OFF_A = 0, OFF_B = 64 << 10, OFF_OUT = 128 << 10, OFF_FAULT = 384 << 10, SLICE = 1 << 20 };

static int failures = 0;

#define HIP_OK(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      printf("%s failed: %s\n", #call, hipGetErrorString(e_));                              \
      return 1;                                                                             \
    }                                                                                       \
  } while (0)
#define TCCL_OK(call)                                                                       \
  do {                                                                                      \
    int rc_ = (call);                                                                       \
    if (rc_ != 0) {                                                                         \
      printf("%s returned %d: %s\n", #call, rc_, tccl_last_error_string());                 \
      return 1;                                                                             \
    }                                                                                       \
  } while (0)

/* fp16 bits of an integer of magnitude <= 2048 (exact) */
static uint16_t half_of_int(int v) {
  unsigned a = (unsigned)(v < 0 ? -v : v), e = 0;
  if (a == 0) return 0;
  while ((a >> (e + 1)) != 0) ++e;
  return (uint16_t)((v < 0 ? 0x8000u : 0u) | ((e + 15u) << 10) | ((e <= 10 ? a << (10 - e) : a >> (e - 10)) & 0x3ffu));
}

/* the integer an fp16 holds, or INT32_MIN if it is not one (subnormal, fraction, inf, nan) */
static int32_t int_of_half(uint16_t h) {
  const int exp = (h >> 10) & 31, mant = h & 0x3ff;
  int32_t a;
  if (exp == 0) return mant == 0 ? 0 : INT32_MIN;
  if (exp == 31 || exp < 15) return INT32_MIN;
  if (exp - 15 >= 10) {
    a = (int32_t)((1024 + mant) << (exp - 25));
  } else {
    if (mant & ((1 << (25 - exp)) - 1)) return INT32_MIN;
    a = (1024 + mant) >> (25 - exp);
  }
  return (h & 0x8000) ? -a : a;
}

static int a_value(int rank, int i, int k) { return (i + 2 * k + rank) % 5 - 2; }
static int b_value(int k, int j) { return (3 * k + j) % 7 - 3; }

int main(void) {
  tccl_device_info info;
  void* arena = NULL;
  int64_t bases[WORLD];
  int64_t* d_bases = NULL;
  static uint16_t a_bits[M * K], b_bits[K * N], got[WORLD * M * N];
  static int32_t want[WORLD][M * N];
  int rank, i, j, k;

  if (tccl_abi_version() != 1) {
    printf("unexpected ABI version %d\n", tccl_abi_version());
    return 1;
  }
  TCCL_OK(tccl_device_query(0, &info));
  printf("device %s, %d CUs\n", info.arch, info.compute_units);
  TCCL_OK(tccl_heap_create(SLICE, WORLD, &arena, bases));
  HIP_OK(hipMalloc((void**)&d_bases, sizeof bases));
  HIP_OK(hipMemcpy(d_bases, bases, sizeof bases, hipMemcpyHostToDevice));

  for (k = 0; k < K; ++k)
    for (j = 0; j < N; ++j) b_bits[k * N + j] = half_of_int(b_value(k, j));
  for (rank = 0; rank < WORLD; ++rank) {
    char* slice = (char*)(intptr_t)bases[rank];
    for (i = 0; i < M; ++i)
      for (k = 0; k < K; ++k) a_bits[i * K + k] = half_of_int(a_value(rank, i, k));
    for (i = 0; i < M; ++i)
      for (j = 0; j < N; ++j) {
        int32_t s = 0;
        for (k = 0; k < K; ++k) s += a_value(rank, i, k) * b_value(k, j);
        want[rank][i * N + j] = s;
      }
    HIP_OK(hipMemcpy(slice + OFF_A, a_bits, sizeof a_bits, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(slice + OFF_B, b_bits, sizeof b_bits, hipMemcpyHostToDevice));
    HIP_OK(hipMemset(slice + OFF_OUT, 0xff, sizeof got)); /* NaN patterns: every value must be overwritten */
    HIP_OK(hipMemset(slice + OFF_FAULT, 0, 8));
  }

  for (rank = 0; rank < WORLD; ++rank) {
    char* slice = (char*)(intptr_t)bases[rank];
    tccl_gemm_desc g;
    tccl_heap_view heap;
    tccl_transport_desc tr;
    tccl_static_plan plan;
    memset(&g, 0, sizeof g);
    memset(&plan, 0, sizeof plan);
    g.A = slice + OFF_A;
    g.B = slice + OFF_B;
    g.C = slice + OFF_OUT + (size_t)rank * M * N * 2; /* the rank's own block of its gathered output */
    g.M = M, g.N = N, g.K = K;
    g.lda = K, g.ldb = N, g.ldc = N;
    g.in_dtype = TCCL_F16, g.out_dtype = TCCL_F16;
    g.alpha = 1.0f;
    g.block_m = 128, g.block_n = 128, g.group_m = 8;
    heap.heap_bases = d_bases, heap.rank = rank, heap.world_size = WORLD;
    tr.directions = TCCL_DIR_PUSH, tr.copy_elems = 16384, tr.reduce_elems = 0, tr.num_comm_wgs = 0;
    plan.n_groups = 1; /* one TileGroup: all rows, (M / 128) * (N / 128) plan tiles */
    plan.row_starts[0] = 0, plan.row_ends[0] = M, plan.tile_counts[0] = (M / 128) * (N / 128);
    TCCL_OK(tccl_gemm_allgather_static(&g, slice + OFF_OUT, N, &heap, &plan, &tr, TCCL_S2_TILEGROUP,
                                       (int64_t*)(slice + OFF_FAULT), 0, NULL));
  }
  HIP_OK(hipDeviceSynchronize());

  for (rank = 0; rank < WORLD; ++rank) {
    char* slice = (char*)(intptr_t)bases[rank];
    int64_t fault = -1;
    int block;
    HIP_OK(hipMemcpy(got, slice + OFF_OUT, sizeof got, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(&fault, slice + OFF_FAULT, 8, hipMemcpyDeviceToHost));
    if (fault != 0) {
      printf("rank %d: a device-side wait expired (fault word %lld)\n", rank, (long long)fault);
      ++failures;
    }
    for (block = 0; block < WORLD; ++block)
      for (i = 0; i < M * N; ++i) {
        const int32_t v = int_of_half(got[block * M * N + i]);
        if (v != want[block][i] && failures++ < 10)
          printf("rank %d, block %d, element %d: got bits 0x%04x, want %d\n", rank, block, i, got[block * M * N + i],
                 want[block][i]);
      }
  }
  HIP_OK(hipFree(d_bases));
  TCCL_OK(tccl_heap_destroy(arena));
  if (failures) {
    printf("%d mismatches\n", failures);
    return 1;
  }
  printf("ok\n");
  return 0;
}
