// Staged peer-read collectives: the slot protocol of the reference's public launchers
// (_allreduce_staged_kernel, tileccl/primitives/collectives.py:840-962, and its two-rank
// specialisations for all-reduce :966-1044, all-gather :1129-1215, reduce-scatter :1276-1366,
// broadcast :1391-1486 and scatter :1489-1592), written once for any world size.
//
// A rank's role is a set of pipeline slots.  The workgroup of (rank r, slot s) processes the
// chunks s, s + S, s + 2S, ... (S = slots) of a block of `units` 16-byte units; per chunk c, with
// epoch = base + c:
//   publishers (every rank; broadcast / scatter: the root) copy what their peers need into their
//   staging slot s, clear consumed[r][s] and store published[r][s] = epoch;
//   consumers (every rank; broadcast / scatter: every rank but the root) wait until
//   published[p][s] == epoch for each publisher p, read p's staging slot, produce their own
//   output, and add 1 to consumed[p][s];
//   a publisher leaves the slot once consumed[r][s] == world - 1.  (The reference's generic
//   all-reduce only waits when the slot is used again in the same call, which leaves a race
//   with the next call to its caller; its two-rank kernels acknowledge with the epoch instead of
//   a count.)
// What is staged and what a consumer does with it:
//   all-reduce      the rank's chunk of `dst` (in place).  Consumer: the ranks' values added in
//                   ascending rank order, its own taken from `dst`, fp32 accumulation and one
//                   rounding, so every rank stores the same bits (the reference starts from its
//                   own values and adds in the tensor's type).
//   all-gather      the rank's chunk of `src`, also stored into block r of its own `dst`.
//                   Consumer: p's chunk into block p of `dst`.
//   reduce-scatter  for every other rank q, the chunk of block q of `src`, in segment q of the
//                   slot.  Consumer r: block r of its own `src` first, then segment r of the
//                   peers' slots in ascending rank (tile_reduce_scatter's order, :766-781; fp32
//                   accumulation, one rounding) into `dst`.
//   broadcast       the root's chunk of `dst`.  Consumer: copy into `dst`.
//   scatter         for every other rank q, the root's chunk of block q of `src`, in segment q;
//                   the root copies block root into its own `dst`.  Consumer r: segment r into `dst`.
// staging (slots x segments x chunk; segments = world for reduce-scatter and scatter, else 1),
// published and consumed live in the symmetric heap (a peer's copy at the same slice offset).
// Epochs only grow, so the words need no reset between calls.
//
// One GPU: the ranks are slices of one arena and cannot be separate processes, so one launch
// carries the roles of every rank named in `ranks`, (rank, slot) -> workgroup; all of them are
// resident at once (the host checks the grid against the device), which is what the waits
// need.  Every wait is bounded; an expired one raises *fault and the role stops.
#pragma once

#include "tccl_comm.h"

namespace tccl {

enum StagedOp { kStagedAllReduce = 0, kStagedAllGather = 1, kStagedReduceScatter = 2, kStagedBroadcast = 3, kStagedScatter = 4 };

struct StagedArgs {
  const int64_t* heap_bases;
  int rank;            // the rank whose addresses src / dst / staging / published / consumed are
  int world;
  uint32_t ranks;      // roles carried by this launch (bit per rank)
  int op, root;
  char* src;           // all-gather: the block; reduce-scatter / scatter: world blocks; else unused
  char* dst;           // all-reduce / broadcast: the tensor; all-gather: world blocks; else one block
  char* staging;       // slots x segments x chunk_units x 16 bytes
  int32_t* published;  // int32[slots]
  int32_t* consumed;   // int32[slots]
  int64_t units;       // 16-byte units in a block
  int chunk_units;     // units per chunk
  int slots;
  int base_epoch;      // >= 1
  int dtype;           // kF16 / kBF16 / kF32 (the reductions; copies move bytes)
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
  const int op = a.op, world = a.world;
  const bool rooted = op == kStagedBroadcast || op == kStagedScatter;
  const bool publishes = !rooted || r == a.root, consumes = !rooted || r != a.root;
  const int segments = (op == kStagedReduceScatter || op == kStagedScatter) ? world : 1;
  const int64_t chunks = (a.units + a.chunk_units - 1) / a.chunk_units;
  const int64_t deadline = now_ticks() + a.spin_ticks;
  int32_t* pub_r = (int32_t*)((char*)a.published + delta_r) + slot;
  int32_t* con_r = (int32_t*)((char*)a.consumed + delta_r) + slot;
  const int64_t chunk_bytes = (int64_t)a.chunk_units * 16, block_bytes = a.units * 16;
  const int64_t slot_off = (int64_t)slot * segments * chunk_bytes;
  const int64_t src_r = (int64_t)(uintptr_t)a.src + delta_r, dst_r = (int64_t)(uintptr_t)a.dst + delta_r;
  const int64_t stage_r = (int64_t)(uintptr_t)a.staging + delta_r + slot_off;
  for (int64_t c = slot; c < chunks; c += a.slots) {
    const int64_t u0 = c * a.chunk_units, b0 = u0 * 16;
    const int n = (int)(a.units - u0 < a.chunk_units ? a.units - u0 : a.chunk_units);
    const int32_t epoch = a.base_epoch + (int32_t)c;
    if (publishes) {
      if (segments == 1) {
        const __amdgpu_buffer_rsrc_t from = window((op == kStagedAllGather ? src_r : dst_r) + b0);
        const __amdgpu_buffer_rsrc_t stage = window(stage_r);
        const __amdgpu_buffer_rsrc_t keep = window(dst_r + (int64_t)r * block_bytes + b0);  // all-gather: own block
        for (int u = tid; u < n; u += threads) {
          const u32x4 v = ld16<0>(from, (uint32_t)u * 16u);
          st16<kCoherent>(stage, (uint32_t)u * 16u, v);
          if (op == kStagedAllGather) st16<0>(keep, (uint32_t)u * 16u, v);
        }
      } else {
        for (int q = 0; q < world; ++q) {
          const __amdgpu_buffer_rsrc_t from = window(src_r + (int64_t)q * block_bytes + b0);
          if (q == r) {
            if (op == kStagedScatter) {  // the root's own block goes straight to its output
              const __amdgpu_buffer_rsrc_t keep = window(dst_r + b0);
              for (int u = tid; u < n; u += threads) st16<0>(keep, (uint32_t)u * 16u, ld16<0>(from, (uint32_t)u * 16u));
            }
            continue;
          }
          const __amdgpu_buffer_rsrc_t stage = window(stage_r + (int64_t)q * chunk_bytes);
          for (int u = tid; u < n; u += threads) st16<kCoherent>(stage, (uint32_t)u * 16u, ld16<0>(from, (uint32_t)u * 16u));
        }
      }
      wait_vmem();
      __syncthreads();
      if (tid == 0) {
        __hip_atomic_store(con_r, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(pub_r, epoch, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (consumes) {
      bool ok = true;
      for (int p = 0; p < world && ok; ++p) {
        if (p == r || (rooted && p != a.root)) continue;
        ok = staged_wait_eq((const int32_t*)((const char*)a.published + (a.heap_bases[p] - mine)) + slot, epoch, deadline, lds_word);
      }
      if (!ok) {
        if (tid == 0 && a.fault) *a.fault = 1;
        return;  // uniform: every thread saw the same verdict
      }
      // segment of a publisher's slot that is meant for this rank
      const int64_t seg_off = segments == 1 ? 0 : (int64_t)r * chunk_bytes;
      if (op == kStagedAllReduce || op == kStagedReduceScatter) {
        const bool owner_first = op == kStagedReduceScatter;
        const __amdgpu_buffer_rsrc_t own = window(op == kStagedAllReduce ? dst_r + b0 : src_r + (int64_t)r * block_bytes + b0);
        const __amdgpu_buffer_rsrc_t out = window(dst_r + b0);
        for (int u = tid; u < n; u += threads) {
          float acc[8];
          if (owner_first) staged_accumulate<T>(ld16<0>(own, (uint32_t)u * 16u), acc, true);
          for (int p = 0; p < world; ++p) {
            u32x4 v;
            if (p == r) {
              if (owner_first) continue;
              v = ld16<0>(own, (uint32_t)u * 16u);
            } else {
              const __amdgpu_buffer_rsrc_t theirs = window((int64_t)(uintptr_t)a.staging + (a.heap_bases[p] - mine) + slot_off + seg_off);
              v = ld16<kCoherent>(theirs, (uint32_t)u * 16u);
            }
            staged_accumulate<T>(v, acc, !owner_first && p == 0);
          }
          st16<0>(out, (uint32_t)u * 16u, staged_pack<T>(acc));
        }
      } else {
        for (int p = 0; p < world; ++p) {
          if (p == r || (rooted && p != a.root)) continue;
          const __amdgpu_buffer_rsrc_t theirs = window((int64_t)(uintptr_t)a.staging + (a.heap_bases[p] - mine) + slot_off + seg_off);
          const __amdgpu_buffer_rsrc_t out = window(dst_r + (op == kStagedAllGather ? (int64_t)p * block_bytes : 0) + b0);
          for (int u = tid; u < n; u += threads) st16<0>(out, (uint32_t)u * 16u, ld16<kCoherent>(theirs, (uint32_t)u * 16u));
        }
      }
      wait_vmem();  // this wave's reads of the publishers' staging have returned
      __syncthreads();
      if (tid == 0)
        for (int p = 0; p < world; ++p)
          if (p != r && !(rooted && p != a.root))
            __hip_atomic_fetch_add((int32_t*)((char*)a.consumed + (a.heap_bases[p] - mine)) + slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // the slot is free again once every consumer has read it (also after its last chunk: the
    // next call may start on this rank while a peer still reads)
    if (publishes && !staged_wait_eq(con_r, world - 1, deadline, lds_word)) {
      if (tid == 0 && a.fault) *a.fault = 1;
      return;
    }
  }
}

}  // namespace tccl
