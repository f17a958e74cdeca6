// Several independent fp32 products in ONE launch of the 256 x 128 one-wave-per-SIMD tile (gemm_lone.h). A product of
// the size a second-order pass issues by the dozen (1024 x 2048 x 2048: 64 such tiles) cannot fill 256 CUs alone and
// runs at 72 % of the matrix peak on the smaller shared-CU tiles; four of them, or two of 2048 x 2048 x 1024, are one
// tile per CU and run at 87-91 %. Every work-group looks up which product its tile belongs to (a scalar walk over at
// most eight counts) and runs that product's loop: the forms differ only in their global -> LDS paths, so all of them
// live in the one kernel and a work-group executes exactly one. Members are ordered longest reduction first by the
// caller, so that the work-groups dispatched later, onto CUs that have finished a tile, are the short ones.
#include "gemm_lone.h"

namespace endia_gemm {

template <int FM, int FN>
__global__ __launch_bounds__(NTHREADS, 1) void sgemm_lone_grouped_kernel(GroupArgs g) {
  extern __shared__ __attribute__((aligned(16))) float smem_lone[];
  const int b = blockIdx.x;
  int i = 0;
  while (i + 1 < g.count && b >= g.first[i + 1]) ++i;
  const GemmArgs& p = g.p[i];
  const int blk = b - g.first[i], n = g.first[i + 1] - g.first[i];
  switch (g.kind[i]) {
    case 0: gemm_tile_lone<true, true, ENDIA_EPI_NONE, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 1: gemm_tile_lone<true, false, ENDIA_EPI_NONE, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 2: gemm_tile_lone<false, true, ENDIA_EPI_NONE, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 3: gemm_tile_lone<false, false, ENDIA_EPI_NONE, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 4: gemm_tile_lone<true, true, ENDIA_EPI_BIAS, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 5: gemm_tile_lone<true, false, ENDIA_EPI_BIAS, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    case 6: gemm_tile_lone<false, true, ENDIA_EPI_BIAS, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
    default: gemm_tile_lone<false, false, ENDIA_EPI_BIAS, FM, FN, 1>(p, blk, n, 0, smem_lone); break;
  }
}

int32_t launch_lone_grouped_256x128(const GroupArgs& g, hipStream_t s) {
  constexpr int FM = 4, FN = 2;
  // the largest stage pair of the four forms; at least 84 KiB so that no CU ever holds two of these work-groups
  constexpr size_t need = 2 * (size_t)(TileShape<false, 64 * FM>::FLOATS + TileShape<false, 64 * FN>::FLOATS) * sizeof(float);
  constexpr size_t need_k = 2 * (size_t)(TileShape<true, 64 * FM>::FLOATS + TileShape<true, 64 * FN>::FLOATS) * sizeof(float);
  constexpr size_t most = need > need_k ? need : need_k;
  constexpr size_t lds = most > 84 * 1024 ? most : 84 * 1024;
  static bool allowed = false;
  if (!allowed) {
    ENDIA_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sgemm_lone_grouped_kernel<FM, FN>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed = true;
  }
  hipLaunchKernelGGL((sgemm_lone_grouped_kernel<FM, FN>), dim3((unsigned)g.first[g.count]), dim3(NTHREADS), lds, s, g);
  return ENDIA_HIP_OK;
}

}  // namespace endia_gemm
