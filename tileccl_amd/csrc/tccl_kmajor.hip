// Second translation unit of libtileccl_hip.so: the large-tile kernels for k-major B (B given as
// the `.t()` view of an (N, K) tensor).  Kept apart from tccl_api.hip only so that the two sets
// of kernels compile in parallel.
#include "tccl_kernels256.h"

namespace tccl {

int launch_gemm256_kmajor(int in_dtype, int out_dtype, const GemmArgs& g, const Macro& m, int wgs,
                                                                hipStream_t stream) {
  return launch_gemm256_table<true>(in_dtype, out_dtype, g, m, wgs, stream);
}

int launch_fused256_kmajor(int in_dtype, int out_dtype, const Fused256Args& f, int wgs,
                                                                 hipStream_t stream) {
  return launch_fused256_table<true>(in_dtype, out_dtype, f, wgs, stream);
}

}  // namespace tccl
