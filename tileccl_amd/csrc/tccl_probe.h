// What the matrix pipes sustain by themselves: a kernel with the large-tile GEMM's shape (512 threads =
// 8 wavefronts per workgroup, one workgroup per CU, 128 x 64 outputs per wavefront in 128 accumulator
// registers) that loads its operand registers once and then issues nothing but MFMAs: no LDS, no global
// memory, no barrier inside the loop.  One "step" is the MFMA work of one K step of a 256 x 256 tile
// (64 k for 16-bit inputs, 128 k for fp8), with as many distinct operand registers as the real K step
// feeds from LDS (96 per lane), so that the operand buses toggle as they do there.
//
// The rate this reaches depends on the instruction shape and on the operand DATA (all-zero operands run
// at the published peak, normally distributed ones well below it), which is why it is measured rather
// than assumed; bench.py reports it next to the published peak.
#pragma once

#include "tccl_gemm256.h"

namespace tccl {

enum ProbeKind { kProbeF16Wide = 0, kProbeF16 = 1, kProbeBF16 = 2, kProbeF8 = 3, kProbeF8Wide = 4 };

#if defined(__HIP_DEVICE_COMPILE__)
// Operand registers of one lane: kBlocks k-blocks of kA row operands and kB column operands.  Row operands are
// read from `a_like`, column operands from `b_like` (each lane its own 16-byte units, wrapping around the buffers).
template <typename Vec, int kBlocks, int kA, int kB>
struct ProbeOperands {
  Vec a[kBlocks][kA], b[kBlocks][kB];
  TCCL_D void load(const char* a_like, uint32_t a_bytes, const char* b_like, uint32_t b_bytes) {
    constexpr uint32_t kVec = sizeof(Vec);
    const uint32_t lane_id = blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
    for (int k = 0; k < kBlocks; ++k) {
#pragma unroll
      for (int i = 0; i < kA; ++i) a[k][i] = *(const Vec*)(a_like + ((lane_id * (uint32_t)(kBlocks * kA) + (uint32_t)(k * kA + i)) * kVec) % a_bytes);
#pragma unroll
      for (int j = 0; j < kB; ++j) b[k][j] = *(const Vec*)(b_like + ((lane_id * (uint32_t)(kBlocks * kB) + (uint32_t)(k * kB + j)) * kVec) % b_bytes);
    }
  }
};
#endif

// 16 x 16 x K MFMAs (the shapes the K loops use): 8 x 4 blocks per wavefront and k-block.
template <typename InT>
__global__ __launch_bounds__(512, 2) void mfma_rate_kernel(const char* a_like, uint32_t a_bytes, const char* b_like, uint32_t b_bytes,
                                                           float* sink, int steps) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Mfma<InT>::Vec Vec;
  constexpr int kBlocks = sizeof(InT) == 1 ? 1 : 2;  // k-blocks per step: 128 k of fp8 in one MFMA, 64 k of a 16-bit type in two
  ProbeOperands<Vec, kBlocks, 8, 4> op;
  op.load(a_like, a_bytes, b_like, b_bytes);
  f32x4 acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < steps; ++s) {
#pragma unroll
    for (int k = 0; k < kBlocks; ++k)
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Mfma<InT>::run16(op.b[k][j], op.a[k][i], acc[i][j]);
    __builtin_amdgcn_sched_barrier(0);
  }
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) t += acc[i][j][0] + acc[i][j][3];
  sink[blockIdx.x * blockDim.x + threadIdx.x] = t;
#endif
}

// 32 x 32 x K MFMAs: 4 x 2 patches per wavefront and k-block.
template <typename InT>
__global__ __launch_bounds__(512, 2) void mfma_rate_wide_kernel(const char* a_like, uint32_t a_bytes, const char* b_like, uint32_t b_bytes,
                                                                float* sink, int steps) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Mfma<InT>::Vec Vec;
  constexpr int kBlocks = sizeof(InT) == 1 ? 2 : 4;  // 64 k of fp8 resp. 16 k of a 16-bit type per MFMA
  ProbeOperands<Vec, kBlocks, 4, 2> op;
  op.load(a_like, a_bytes, b_like, b_bytes);
  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int s = 0; s < steps; ++s) {
#pragma unroll
    for (int k = 0; k < kBlocks; ++k)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<InT>::run(op.b[k][j], op.a[k][i], acc[i][j]);
    __builtin_amdgcn_sched_barrier(0);
  }
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) t += acc[i][j][0] + acc[i][j][15];
  sink[blockIdx.x * blockDim.x + threadIdx.x] = t;
#endif
}

}  // namespace tccl
