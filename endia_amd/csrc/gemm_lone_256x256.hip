// The 256x256 tile of the one-wave-per-SIMD fp32 GEMM (gemm_lone.h): every transpose form and epilogue.
#include "gemm_lone.h"

namespace endia_gemm {
int32_t launch_lone_256x256(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s) {
  return launch_lone<4, 4, 1>(p, epi, transA, transB, grid, s);
}
}  // namespace endia_gemm
