// Device-side primitives shared by every kernel of libtileccl_hip: index math of the
// persistent GEMM's tile order, symmetric-heap pointer translation, and the
// signal / wait words.  Index helpers are __host__ __device__ so CPU tests can call the
// very code the kernels run.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TCCL_HD __host__ __device__ __forceinline__
#define TCCL_D __device__ __forceinline__

namespace tccl {

// ---------------------------------------------------------------------------------------
// Tile order.  Swizzled tile id -> (tile_m, tile_n): inside a band of group_m tile rows
// (fewer in the last band) ids walk down the rows first, then across the columns.
// Reference: tileccl/kernels/gemm.py:118-123, tileccl_v2/tile_group.py:229-234.
// ---------------------------------------------------------------------------------------
struct TileCoord {
  int m, n;
};

TCCL_HD TileCoord tile_coords(int tile_id, int tile_rows, int tile_cols, int group_m) {
  const int per_band = group_m * tile_cols;
  const int band = tile_id / per_band;
  const int first_m = band * group_m;
  const int height = (tile_rows - first_m) < group_m ? (tile_rows - first_m) : group_m;
  const int within = tile_id - band * per_band;
  TileCoord c;
  c.m = first_m + within % height;
  c.n = within / height;
  return c;
}

// Inverse of tile_coords.
TCCL_HD int tile_id_of(int tile_m, int tile_n, int tile_rows, int tile_cols, int group_m) {
  const int band = tile_m / group_m;
  const int first_m = band * group_m;
  const int height = (tile_rows - first_m) < group_m ? (tile_rows - first_m) : group_m;
  return band * group_m * tile_cols + tile_n * height + (tile_m - first_m);
}

// Launch slot -> tile id.  Workgroups are handed to the XCDs round-robin (slot % xcds),
// and each XCD has a private L2.  Inside every full block of xcds*span consecutive tile
// ids, XCD x takes the ids [x*span, (x+1)*span): with the row-fastest swizzle that is a
// compact patch of the output (span/group_m tile columns of one band), so the A rows and
// B columns it touches stay in that XCD's L2.  A trailing partial block keeps the
// identity order.  The map is a bijection on [0, total_tiles).
TCCL_HD int tile_for_slot(int slot, int total_tiles, int xcds, int span) {
  const int block = xcds * span;
  const int base = (slot / block) * block;
  if (xcds <= 1 || base + block > total_tiles) return slot;
  const int r = slot - base;
  return base + (r % xcds) * span + r / xcds;
}

#ifdef __HIPCC__
// ---------------------------------------------------------------------------------------
// Symmetric heap.  translate(ptr, from, to) = bases[to] + (ptr - bases[from]).
// Reference: tileccl/memory/translation.py:39-99, tileccl_v2/ipc.py:24-63.
// ---------------------------------------------------------------------------------------
template <typename T>
TCCL_D T* translate_ptr(T* ptr, int from_rank, int to_rank, const int64_t* heap_bases) {
  const int64_t off = (int64_t)(uintptr_t)ptr - heap_bases[from_rank];
  return (T*)(uintptr_t)(heap_bases[to_rank] + off);
}

// 100 MHz constant clock; one tick = 10 ns.
TCCL_D int64_t now_ticks() { return (int64_t)wall_clock64(); }

// ---------------------------------------------------------------------------------------
// Signal words (int32, in the heap).
//
// Two flavours of every primitive:
//  * the stand-alone form carries the ordering itself (release on signal, acquire on a
//    successful wait), like the reference's Triton atomics with sem="release"/"acquire"
//    (sync/primitives.py:357-500, tileccl_v2/ipc.py:137-254);
//  * the `Relaxed` form is for the fused kernels, whose *data path* is already coherent:
//    producers store finished output with device-coherent write-through stores
//    (kCoherent cache policy) and wait for them to complete before signalling, consumers
//    read with device-coherent loads.  An agent-scope release/acquire on gfx950 writes
//    back / invalidates the whole per-XCD L2; doing that once per tile from hundreds of
//    workgroups evicts the GEMM's operands over and over, so the fused path avoids it.
// One GPU: agent scope reaches every workgroup on every XCD; real peers would need system
// scope (the reference's v1 default is "gpu", v2 "sys").
// ---------------------------------------------------------------------------------------

// Cache policy bits of raw buffer loads/stores on gfx950: sc0 = 1, nt = 2, sc1 = 16.
constexpr int kCoherent = 17;  // sc0 sc1: write through to / read from memory, visible to every XCD
constexpr int kStreaming = 2;  // nt: data is touched once

// All of this wave's outstanding global loads and stores have completed.
TCCL_D void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <bool Relaxed = false>
TCCL_D void tile_signal(int32_t* locks, int i) {
  __hip_atomic_exchange(&locks[i], 1, Relaxed ? __ATOMIC_RELAXED : __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// One CAS probe: consuming (1 -> 0, tile_wait / tile_try_wait) or non-consuming
// (1 -> 1, tile_poll / tile_try_poll).  (sync/primitives.py:390-439, ipc.py:193-228)
template <bool Relaxed = false>
TCCL_D bool tile_probe(int32_t* locks, int i, bool consume) {
  int32_t expected = 1;
  return __hip_atomic_compare_exchange_strong(&locks[i], &expected, consume ? 0 : 1,
                                              Relaxed ? __ATOMIC_RELAXED : __ATOMIC_ACQUIRE, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
}

// tile_try_wait / tile_try_poll: at most max_spins probes; true when the flag was seen.
TCCL_D bool tile_try_wait(int32_t* locks, int i, int max_spins, bool consume) {
  for (int s = 0; s < max_spins; ++s)
    if (tile_probe(locks, i, consume)) return true;
  return false;
}

// tile_wait / tile_poll with a deadline: the reference spins forever
// (sync/primitives.py:390-414); here every wait gives up at `deadline` (now_ticks units)
// and reports false so the kernel can drain and the host can raise.  The spin reads the
// word with relaxed loads; the CAS runs once the flag has been seen.
template <bool Relaxed = false>
TCCL_D bool tile_wait(int32_t* locks, int i, bool consume, int64_t deadline) {
  for (;;) {
    for (int s = 0; s < 32; ++s) {
      if (__hip_atomic_load(&locks[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1) {
        if (tile_probe<Relaxed>(locks, i, consume)) return true;
      }
      __builtin_amdgcn_s_sleep(4);
    }
    if (now_ticks() > deadline) return false;
  }
}

// Epoch-valued tile flags of the fused tile-by-tile launches: launch e stores e into
// locks[tile], and a tile counts as ready for launch e once its word has reached e
// (tile_wait_ge).  Nothing is consumed, so the owner's communication role and any number of
// peers can watch the same word, and a flag left behind by launch e-1 is never taken for
// launch e's.  (The reference gets the second property by zeroing its lock tensor before
// every call: patterns/wg_specialized.py:122-123.)
TCCL_D void tile_publish(int32_t* locks, int i, int32_t epoch) {
  __hip_atomic_store(&locks[i], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// tile_signal_add: counter[i] += v; returns the previous value. (ipc.py:231-241)
template <bool Relaxed = false>
TCCL_D int32_t tile_signal_add(int32_t* words, int i, int32_t v) {
  return __hip_atomic_fetch_add(&words[i], v, Relaxed ? __ATOMIC_RELAXED : __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// Has a signal word reached the value a waiter needs?  Words only ever grow, and the comparison is the
// one of sequence numbers (the difference, taken modulo 2^32, is non-negative): a word and a threshold
// that have both wrapped around still compare correctly, as long as they are less than 2^31 apart.
TCCL_HD bool word_reached(int32_t word, int32_t need) { return (int32_t)((uint32_t)word - (uint32_t)need) >= 0; }

// tile_wait_ge: spin until counter[i] >= threshold (word_reached).  The reference reads the word with
// atomic_add(0, acquire) (ipc.py:244-254); relaxed loads followed by one acquire fence
// observe the same value without taking the line exclusive.  Bounded like tile_wait.
template <bool Relaxed = false>
TCCL_D bool tile_wait_ge(const int32_t* words, int i, int32_t threshold, int64_t deadline) {
  for (;;) {
    for (int s = 0; s < 32; ++s) {
      if (word_reached(__hip_atomic_load(&words[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), threshold)) {
        if (!Relaxed) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        return true;
      }
      __builtin_amdgcn_s_sleep(4);
    }
    if (now_ticks() > deadline) return false;
  }
}
#endif  // __HIPCC__

}  // namespace tccl
