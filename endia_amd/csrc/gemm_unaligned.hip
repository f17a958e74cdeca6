// The shared-CU tiles of the fp32 GEMM for operands that cannot be read 16 bytes at a time: a base address, a leading
// dimension or a contiguous extent that is not a multiple of four floats. The reference's matmul takes any shape and any
// view (endia/functional/binary_ops/matmul_op.mojo:93-199; its own test multiplies (30,40) by (40,50),
// tests/test_endia/test_functional/test_binary_ops/test_matmul_op.mojo:18-59). Same tile body, LDS layouts and MFMA
// loop as gemm.hip; only the global loads differ (four 32-bit buffer loads per piece, each bounds-tested).
#include "gemm_tile.h"

namespace endia_gemm {

template <bool A_VEC, bool B_VEC>
static void launch_tile(const GemmArgs& p, int epi, int tile, int transA, int transB, dim3 grid, hipStream_t s) {
  if (tile == 128) launch_mfma_epi<2, false, A_VEC, B_VEC>(p, epi, transA, transB, grid, s);
  else launch_mfma_epi<1, false, A_VEC, B_VEC>(p, epi, transA, transB, grid, s);
}

// a_vec / b_vec: that operand alone could be read 16 bytes at a time, and is (at least one of them cannot)
void launch_mfma_unaligned(const GemmArgs& p, int epi, int tile, bool a_vec, bool b_vec, int transA, int transB, dim3 grid, hipStream_t s) {
  if (a_vec) launch_tile<true, false>(p, epi, tile, transA, transB, grid, s);
  else if (b_vec) launch_tile<false, true>(p, epi, tile, transA, transB, grid, s);
  else launch_tile<false, false>(p, epi, tile, transA, transB, grid, s);
}

}  // namespace endia_gemm
