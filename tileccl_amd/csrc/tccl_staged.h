// Staged peer-read all-reduce: the reference's public allreduce fast path
// (_allreduce_staged_kernel, tileccl/primitives/collectives.py:840-962; its two-rank
// specialisation :966-1044 is the same protocol with one peer).
//
// A rank's role is a set of pipeline slots.  The workgroup of (rank r, slot s) processes the
// chunks s, s + S, s + 2S, ... of r's tensor (S = slots); per chunk c, with epoch = base + c:
//   1. snapshot the chunk into r's staging slot s (device-coherent stores);
//   2. consumed[r][s] = 0, then published[r][s] = epoch;
//   3. for every peer p: wait until published[p][s] == epoch; then add the ranks' values in
//      ascending rank order, r's own from its tensor and a peer's from its staging slot s
//      (fp32 accumulation, one rounding, so every rank stores the same bits; the reference
//      starts from its own values and adds in the tensor's type), then consumed[p][s] += 1;
//   4. store the sum into r's tensor (a rank only ever writes its own tensor);
//   5. wait until consumed[r][s] == world - 1 (the reference only when the slot is used again
//      in the same call, which leaves a race with the next call to its caller).
// staging, published and consumed live in the symmetric heap (a peer's copy at the same slice
// offset).  Epochs only grow, so the words need no reset between calls.
//
// One GPU: the ranks are slices of one arena and cannot be separate processes, so one launch
// carries the roles of every rank named in `ranks`, (rank, slot) -> workgroup; all of them are
// resident at once (the host checks the grid against the device), which is what the waits
// need.  Every wait is bounded; an expired one raises *fault and the role stops.
#pragma once

#include "tccl_comm.h"

namespace tccl {

struct StagedArgs {
  const int64_t* heap_bases;
  int rank;            // the rank whose addresses tensor / staging / published / consumed are
  int world;
  uint32_t ranks;      // roles carried by this launch (bit per rank)
  char* tensor;
  char* staging;       // slots x chunk_units x 16 bytes
  int32_t* published;  // int32[slots]
  int32_t* consumed;   // int32[slots]
  int64_t units;       // 16-byte units in the tensor
  int chunk_units;     // units per chunk
  int slots;
  int base_epoch;      // >= 1
  int dtype;           // kF16 / kBF16 / kF32
  int64_t* fault;
  int64_t spin_ticks;
};

template <typename T>
TCCL_D void staged_accumulate(u32x4 v, float (&acc)[8], bool first) {
  constexpr int n = 16 / sizeof(T);
  T e[n];
  __builtin_memcpy(e, &v, 16);
#pragma unroll
  for (int i = 0; i < n; ++i) acc[i] = first ? (float)e[i] : acc[i] + (float)e[i];
}
template <typename T>
TCCL_D u32x4 staged_pack(const float (&acc)[8]) {
  constexpr int n = 16 / sizeof(T);
  T e[n];
#pragma unroll
  for (int i = 0; i < n; ++i) e[i] = (T)acc[i];
  u32x4 v;
  __builtin_memcpy(&v, e, 16);
  return v;
}

// One lane waits (bounded) until *word == value; the verdict is shared through `lds_word`.
TCCL_D bool staged_wait_eq(const int32_t* word, int32_t value, int64_t deadline, volatile int* lds_word) {
  if (threadIdx.x == 0) {
    bool ok = false;
    for (;;) {
      if (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == value) {
        ok = true;
        break;
      }
      if (now_ticks() > deadline) break;
      __builtin_amdgcn_s_sleep(4);
    }
    *lds_word = ok ? 1 : 0;
  }
  __syncthreads();
  const bool ok = *lds_word != 0;
  __syncthreads();
  return ok;
}

template <typename T>
TCCL_D void staged_role(const StagedArgs& a, int r, int slot, volatile int* lds_word) {
  const int64_t mine = a.heap_bases[a.rank];
  const int64_t delta_r = a.heap_bases[r] - mine;  // rank r's copy of an address of rank a.rank
  const int tid = threadIdx.x, threads = blockDim.x;
  const int64_t chunks = (a.units + a.chunk_units - 1) / a.chunk_units;
  const int64_t deadline = now_ticks() + a.spin_ticks;
  int32_t* pub_r = (int32_t*)((char*)a.published + delta_r) + slot;
  int32_t* con_r = (int32_t*)((char*)a.consumed + delta_r) + slot;
  const int64_t stage_off = (int64_t)slot * a.chunk_units * 16;
  for (int64_t c = slot; c < chunks; c += a.slots) {
    const int64_t u0 = c * a.chunk_units;
    const int n = (int)(a.units - u0 < a.chunk_units ? a.units - u0 : a.chunk_units);
    const int32_t epoch = a.base_epoch + (int32_t)c;
    const __amdgpu_buffer_rsrc_t tens = window((int64_t)(uintptr_t)a.tensor + delta_r + u0 * 16);
    const __amdgpu_buffer_rsrc_t stage = window((int64_t)(uintptr_t)a.staging + delta_r + stage_off);
    // 1. snapshot
    for (int u = tid; u < n; u += threads) st16<kCoherent>(stage, (uint32_t)u * 16u, ld16<0>(tens, (uint32_t)u * 16u));
    wait_vmem();
    __syncthreads();
    // 2. publish
    if (tid == 0) {
      __hip_atomic_store(con_r, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pub_r, epoch, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
    // 3. peers, ascending; own values first
    bool ok = true;
    for (int p = 0; p < a.world && ok; ++p) {
      if (p == r) continue;
      const int64_t delta_p = a.heap_bases[p] - mine;
      ok = staged_wait_eq((const int32_t*)((const char*)a.published + delta_p) + slot, epoch, deadline, lds_word);
    }
    if (!ok) {
      if (tid == 0 && a.fault) *a.fault = 1;
      return;  // uniform: every thread saw the same verdict
    }
    for (int u = tid; u < n; u += threads) {
      float acc[8];
      for (int p = 0; p < a.world; ++p) {  // ascending ranks, own values in their place: every rank rounds the same sum
        u32x4 v;
        if (p == r) {
          v = ld16<0>(tens, (uint32_t)u * 16u);
        } else {
          const __amdgpu_buffer_rsrc_t theirs = window((int64_t)(uintptr_t)a.staging + (a.heap_bases[p] - mine) + stage_off);
          v = ld16<kCoherent>(theirs, (uint32_t)u * 16u);
        }
        staged_accumulate<T>(v, acc, p == 0);
      }
      st16<0>(tens, (uint32_t)u * 16u, staged_pack<T>(acc));  // 4. own tensor only
    }
    wait_vmem();  // this wave's reads of the peers' staging have returned
    __syncthreads();
    if (tid == 0)
      for (int p = 0; p < a.world; ++p)
        if (p != r) __hip_atomic_fetch_add((int32_t*)((char*)a.consumed + (a.heap_bases[p] - mine)) + slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // 5. the slot is free again once every peer has read it (also after its last chunk: the
    //    next call may start on this rank while a peer still reads)
    if (!staged_wait_eq(con_r, a.world - 1, deadline, lds_word)) {
      if (tid == 0 && a.fault) *a.fault = 1;
      return;
    }
  }
}

}  // namespace tccl
