// The large-tile kernels (__global__ wrappers around Gemm256) and their launch tables, shared by
// the library's two translation units: tccl_api.hip instantiates the kernels for row-major B,
// tccl_kmajor.hip those for k-major B, so that the two sets compile side by side.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <type_traits>

#include "tccl_comm.h"
#include "tccl_gemm256.h"

namespace tccl {

// Large-tile GEMM: 512 threads, one workgroup per CU, both LDS stages resident.
template <typename InT, typename OutT, bool kBKMajor>
__global__ __launch_bounds__(512, 2) void gemm256_kernel(GemmArgs g, Macro m) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char stage0[kStage256];
  __shared__ __attribute__((aligned(16))) char stage1[kStage256];
  warm_kernargs<(int)(sizeof(GemmArgs) + sizeof(Macro))>();
  SignalArgs s;
  s.mode = kSignalNone;
  Gemm256<InT, OutT, false, false, kBKMajor>(g, -1, -1, -1, stage0, stage1, nullptr).run(s, m, (int)blockIdx.x, (int)gridDim.x);
#endif
}

// Large-tile GEMM whose workgroups, once their tiles are stored (and pushed to the peers
// from the epilogue), turn into the communication role.  The tile fills a CU's LDS and
// registers, so no separate communication workgroup could share the CU with it; instead
// every workgroup produces first and moves data afterwards.  No workgroup waits before its
// own tiles are published and the grid never exceeds the CU count, so every wait is on a
// workgroup that is running.  `push` and `comm` are read from the argument block at their
// point of use (late_kernarg), never through the parameter itself.
struct Fused256Args {
  GemmArgs g;
  SignalArgs s;
  Macro m;
  int64_t* trace_start;
  PullArgs pull;
  PushArgs push;
  ReduceArgs reduce;
  GatherArgs gather;
  CommArgs comm;
};

// kPull = false: the launch has no background transfer (an all-gather that only pushes: what a rank of a
// real pair runs).  The transfer's arguments are then withheld from Gemm256 at compile time and its
// per-step code, which costs a launch 1.9 us at 4096 x 4096 x 1024 even when every call returns at
// once, is not generated at all.
template <typename InT, typename OutT, bool kWithReduce, bool kGatherA, bool kBKMajor, bool kPull = true>
__global__ __launch_bounds__(512, 2) void fused256_kernel(Fused256Args f) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char stage0[kStage256];
  __shared__ __attribute__((aligned(16))) char stage1[kStage256];
  __shared__ __attribute__((aligned(16))) char landing_words[kBgWordBytes];
  warm_kernargs<(int)sizeof(Fused256Args)>();
  if (f.trace_start && blockIdx.x == 0 && threadIdx.x == 0) *f.trace_start = now_ticks();
  Gemm256<InT, OutT, kWithReduce, kGatherA, kBKMajor>(f.g, kPull ? (int)offsetof(Fused256Args, pull) : -1, (int)offsetof(Fused256Args, push),
                                                      (int)offsetof(Fused256Args, reduce), stage0, stage1, landing_words,
                                                      (int)offsetof(Fused256Args, gather))
      .run(f.s, f.m, (int)blockIdx.x, (int)gridDim.x);
  __syncthreads();
  const CommArgs c = late_kernarg<CommArgs>((int)offsetof(Fused256Args, comm));
  comm_role<kThreads256>(c, (int)blockIdx.x, (int)gridDim.x, (int*)stage1);
#endif
}

// Launch tables.  Return 0, a hipError_t, or one of:
enum { kNoKernel = -1000, kGatherTypes = -1001 };
enum { kInF16 = 0, kInBF16 = 1, kInF32 = 2, kInF8 = 3 };  // the dtype codes of include/tileccl_hip.h

template <typename InT, typename OutT, bool kBKMajor>
int launch_gemm256_t(const GemmArgs& g, const Macro& m, int wgs, hipStream_t stream) {
  hipLaunchKernelGGL((gemm256_kernel<InT, OutT, kBKMajor>), dim3(wgs), dim3(kThreads256), 0, stream, g, m);
  return (int)hipGetLastError();
}

template <typename InT, typename OutT, bool kBKMajor>
int launch_fused256_t(const Fused256Args& f, int wgs, hipStream_t stream) {
  // The tile-by-tile reduce-scatter is a separate instantiation: its code would otherwise
  // raise the register pressure of every fused kernel.
  if (f.gather.active) {
    // Instantiated for outputs of the input type and row-major B only (gather_in_place() admits nothing else).
    if constexpr (std::is_same<InT, OutT>::value && !kBKMajor)
      hipLaunchKernelGGL((fused256_kernel<InT, OutT, false, true, false>), dim3(wgs), dim3(kThreads256), 0, stream, f);
    else
      return kGatherTypes;
  } else if (f.reduce.active)
    hipLaunchKernelGGL((fused256_kernel<InT, OutT, true, false, kBKMajor>), dim3(wgs), dim3(kThreads256), 0, stream, f);
  else if (f.pull.mode == kBgNone)
    hipLaunchKernelGGL((fused256_kernel<InT, OutT, false, false, kBKMajor, false>), dim3(wgs), dim3(kThreads256), 0, stream, f);
  else
    hipLaunchKernelGGL((fused256_kernel<InT, OutT, false, false, kBKMajor>), dim3(wgs), dim3(kThreads256), 0, stream, f);
  return (int)hipGetLastError();
}

template <bool kBKMajor>
int launch_gemm256_table(int in_dtype, int out_dtype, const GemmArgs& g, const Macro& m, int wgs, hipStream_t stream) {
  if (in_dtype == kInF16 && out_dtype == kInF16) return launch_gemm256_t<_Float16, _Float16, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInF16 && out_dtype == kInF32) return launch_gemm256_t<_Float16, float, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInBF16 && out_dtype == kInBF16) return launch_gemm256_t<__bf16, __bf16, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInBF16 && out_dtype == kInF32) return launch_gemm256_t<__bf16, float, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInBF16) return launch_gemm256_t<fp8e4m3, __bf16, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInF16) return launch_gemm256_t<fp8e4m3, _Float16, kBKMajor>(g, m, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInF32) return launch_gemm256_t<fp8e4m3, float, kBKMajor>(g, m, wgs, stream);
  return kNoKernel;
}

template <bool kBKMajor>
int launch_fused256_table(int in_dtype, int out_dtype, const Fused256Args& f, int wgs, hipStream_t stream) {
  if (in_dtype == kInF16 && out_dtype == kInF16) return launch_fused256_t<_Float16, _Float16, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInF16 && out_dtype == kInF32) return launch_fused256_t<_Float16, float, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInBF16 && out_dtype == kInBF16) return launch_fused256_t<__bf16, __bf16, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInBF16 && out_dtype == kInF32) return launch_fused256_t<__bf16, float, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInBF16) return launch_fused256_t<fp8e4m3, __bf16, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInF16) return launch_fused256_t<fp8e4m3, _Float16, kBKMajor>(f, wgs, stream);
  if (in_dtype == kInF8 && out_dtype == kInF32) return launch_fused256_t<fp8e4m3, float, kBKMajor>(f, wgs, stream);
  return kNoKernel;
}

// Defined in tccl_kmajor.hip.
int launch_gemm256_kmajor(int in_dtype, int out_dtype, const GemmArgs& g, const Macro& m, int wgs, hipStream_t stream);
int launch_fused256_kmajor(int in_dtype, int out_dtype, const Fused256Args& f, int wgs, hipStream_t stream);

}  // namespace tccl
