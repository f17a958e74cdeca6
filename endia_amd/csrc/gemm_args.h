// Kernel arguments and epilogue bodies shared by the fp32 GEMM kernels (gemm.hip and the one-wave-per-SIMD tiles of
// gemm_lone.h, which are compiled in translation units of their own).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/endia_hip.h"

namespace endia_gemm {

constexpr int NTHREADS = 256;  // four waves, 2 x 2

struct GemmArgs {
  const float* A;
  const float* B;
  float* C;
  const float* bias;
  const float* aux_in;
  float* aux_out;
  int64_t lda, ldb, ldc;
  int64_t sA, sB, sC;
  int M, N, K;
  int tiles_m, tiles_n;
  int k_split;    // > 0: grid.y indexes slices of K of this length instead of batch entries
  int splits;     // > 0: the slices' partial sums meet in `part` and the last group of a tile to arrive finishes it
  float* part;    // [splits][tiles][accumulator registers][256 lanes]
  unsigned* tickets;  // one arrival counter per tile, zero between launches
  int act;        // endia_hip_unary_op
  int from_out;   // activation gradient from stored output instead of pre-activation
  int accumulate;
  int colsum;     // also write sum_k B[k][n] to aux_out[n] (B MN-major; done by the work-groups of the first tile row)
};

__device__ __forceinline__ float act_fwd(int act, float z) {
  switch (act) {
    case ENDIA_OP_RELU: return z > 0.f ? z : 0.f;
    case ENDIA_OP_TANH: return tanhf(z);
    case ENDIA_OP_SIN: return sinf(z);
    default: return z;
  }
}

__device__ __forceinline__ float act_grad(int act, int from_out, float aux) {
  switch (act) {
    case ENDIA_OP_RELU: return aux > 0.f ? 1.f : 0.f;
    case ENDIA_OP_TANH: {
      float a = from_out ? aux : tanhf(aux);
      return 1.f - a * a;
    }
    case ENDIA_OP_SIN: return cosf(aux);
    default: return 1.f;
  }
}

// bias_v = bias[col] and aux_v = aux_in[row, col], fetched by the caller (early, where registers allow)
// old_v: what C holds at (row, col), fetched by the caller ahead of its stores when it accumulates (null: read here)
template <int EPI>
__device__ __forceinline__ void epilogue_apply(const GemmArgs& p, float* __restrict__ C, float* __restrict__ aux_out,
                                               int row, int col, float v, float bias_v, float aux_v, const float* old_v = nullptr) {
  int64_t off = (int64_t)row * p.ldc + col;
  if (EPI == ENDIA_EPI_BIAS) {
    v += bias_v;
  } else if (EPI == ENDIA_EPI_BIAS_ACT) {
    v += bias_v;
    if (aux_out) aux_out[off] = v;
    v = act_fwd(p.act, v);
  } else if (EPI == ENDIA_EPI_ACT_GRAD) {
    v *= act_grad(p.act, p.from_out, aux_v);
  }
  if (p.accumulate) v += old_v ? *old_v : C[off];
  C[off] = v;
}

template <int EPI>
__device__ __forceinline__ void epilogue_store(const GemmArgs& p, float* __restrict__ C,
                                               const float* __restrict__ aux_in,
                                               float* __restrict__ aux_out, int row, int col, float v) {
  const float bias_v = (EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) ? p.bias[col] : 0.f;
  const float aux_v = EPI == ENDIA_EPI_ACT_GRAD ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
  epilogue_apply<EPI>(p, C, aux_out, row, col, v, bias_v, aux_v);
}

// Several independent products in one launch of the 256 x 128 one-wave-per-SIMD tile (gemm_lone_grouped.hip): the
// work-groups [first[i], first[i + 1]) are the tiles of product i. kind = form (0: A and B K-major, 1: A only, 2: B
// only, 3: neither) + 4 for the bias epilogue; accumulation is the member's own flag.
constexpr int kMaxGroup = 8;
struct GroupArgs {
  int count;
  int first[kMaxGroup + 1];
  int kind[kMaxGroup];
  GemmArgs p[kMaxGroup];
};
int32_t launch_lone_grouped_256x128(const GroupArgs& g, hipStream_t s);

// Launcher of the shared-CU tiles (tile = 64 or 128) for operands read 4 bytes at a time (gemm_unaligned.hip).
void launch_mfma_unaligned(const GemmArgs& p, int epi, int tile, bool a_vec, bool b_vec, int transA, int transB, dim3 grid, hipStream_t s);

// Products with at most 16 output columns and a long reduction over a row-major A (gemm_narrow.hip): whether the kernel takes
// the product, and its launch.
bool narrow_ok(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch, const float* A, int64_t lda, const float* B,
               int64_t ldb, int colsum);
int32_t launch_narrow(const GemmArgs& p, int epi, int transB, hipStream_t s);

// Launchers of the one-wave-per-SIMD tiles, one translation unit per tile shape (gemm_lone_*.hip).
// The caller checks the launch with hipGetLastError.
int32_t launch_lone_256x256(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s);
int32_t launch_lone_256x128(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s);

}  // namespace endia_gemm
