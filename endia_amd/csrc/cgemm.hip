// complex64 GEMM: the complex branch of matmul_fwd (endia/functional/binary_ops/matmul_op.mojo:201-238).
//
// The reference de-interleaves 2*nelts floats per load and forms, per element,
//   re += ar*br - ai*bi ;  im += ar*bi + ai*br            (matmul_op.mojo:216-217)
// Here the interleaved operands are split once into planar fp32 matrices (one streaming pass,
// folding the optional conjugation into the sign of the imaginary plane) and the products run on
// the fp32 MFMA GEMM:
//   4M:  Cr = Ar Br + (-Ai) Bi ;  Ci = Ar Bi + Ai Br        -- the reference's four products
//   3M:  T1 = Ar Br, T2 = Ai Bi, T3 = (Ar+Ai)(Br+Bi) ;  Cr = T1 - T2 ;  Ci = T3 - T1 - T2
// 3M does 6 MNK flops instead of 8 MNK but its imaginary part is a difference of larger numbers,
// so its rounding error is larger than 4M's.
// 4M runs as ONE real GEMM of shape M x 2N x 2K on the real embedding of the right operand: an
// interleaved complex matrix IS a real matrix with twice the columns, and with
//   E(B)[2k  , 2n..2n+1] = ( Br[k,n], Bi[k,n])       (row k of B as stored)
//   E(B)[2k+1, 2n..2n+1] = (-Bi[k,n], Br[k,n])       (row k of i*B)
// the real product  A_real (M x 2K) . E(B) (2K x 2N)  is C as stored, interleaved: the same four
// products, the two sums of each output taken inside one K loop. So a non-transposed A is used in
// place, C is written (or accumulated) in place by the GEMM epilogue, and only B is rewritten. A
// transposed A is copied into stacked planes [Re ; Im] (2K x M) and E(B) orders its rows to match.
// One launch with twice the reduction length and twice the tiles also keeps the matrix pipe busier
// than four launches of M x N x K (2048^3: 0.50 ms against 0.56 ms).
#include "common.h"

namespace endia {
int32_t sgemm_impl(int transA, int transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                   const float* B, int64_t ldb, float* C, int64_t ldc, int64_t batch, int64_t sA,
                   int64_t sB, int64_t sC, int epi_flags, int act_flags, const float* bias,
                   const float* aux_in, float* aux_out);
}

namespace {

constexpr int TPB = 256;

// 3M operand split. src: rows x cols complex, row stride ld (complex). Planes are compact rows x cols:
// re = Re, im = sign*Im, sum = Re + sign*Im.
__global__ __launch_bounds__(TPB) void split_kernel(const float2* __restrict__ src, int64_t rows, int64_t cols,
                                                    int64_t ld, float sign, float* __restrict__ re,
                                                    float* __restrict__ im, float* __restrict__ sum) {
  int64_t n = rows * cols;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    int64_t r = j / cols, c = j - r * cols;
    float2 z = src[r * ld + c];
    float i = sign * z.y;
    re[j] = z.x;
    im[j] = i;
    sum[j] = z.x + i;
  }
}

// Left operand used through its transpose (src: K rows x M cols complex): out is 2K x M real, the Re plane
// followed by the Im plane, so that the real GEMM sees op(A) as M x 2K with k order (all Re, all Im).
__global__ __launch_bounds__(TPB) void stack_planes_kernel(const float2* __restrict__ src, int64_t rows, int64_t cols, int64_t ld,
                                                           float* __restrict__ out) {
  const int64_t n = rows * cols, stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    const int64_t r = j / cols, c = j - r * cols;
    const float2 z = src[r * ld + c];
    out[j] = z.x;
    out[n + j] = z.y;
  }
}

// Real embedding E(op(B)) of the right operand, in the orientation B is stored in.
//   src: rows x cols complex; bsign = -1 conjugates B; asign = -1 stands for a conjugated A (it negates the
//   rows that multiply Im A). `blocked`: k order (all Re, all Im) to match stack_planes_kernel, else (Re, Im) pairs.
//   not transposed (rows = K, cols = N): out is 2K x 2N, out[row(k,0)] = (Br, Bi) pairs, out[row(k,1)] = asign * (-Bi, Br)
//   transposed     (rows = N, cols = K): out is 2N x 2K (the transpose of the above):
//                  out[2n][col(k,0)] = Br, out[2n][col(k,1)] = -asign*Bi, out[2n+1][col(k,0)] = Bi, out[2n+1][col(k,1)] = asign*Br
__global__ __launch_bounds__(TPB) void embed_b_kernel(const float2* __restrict__ src, int64_t rows, int64_t cols, int64_t ld,
                                                      float bsign, float asign, int trans, int blocked, float* __restrict__ out) {
  const int64_t n = rows * cols, stride = (int64_t)gridDim.x * TPB;
  const int64_t ldo = 2 * cols;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    const int64_t r = j / cols, c = j - r * cols;
    const float2 z = src[r * ld + c];
    const float br = z.x, bi = bsign * z.y;
    if (!trans) {  // r = k, c = n
      const int64_t row0 = blocked ? r : 2 * r, row1 = blocked ? rows + r : 2 * r + 1;
      *reinterpret_cast<float2*>(out + row0 * ldo + 2 * c) = make_float2(br, bi);
      *reinterpret_cast<float2*>(out + row1 * ldo + 2 * c) = make_float2(-asign * bi, asign * br);
    } else {       // r = n, c = k
      const int64_t col0 = blocked ? c : 2 * c, col1 = blocked ? cols + c : 2 * c + 1;
      out[(2 * r) * ldo + col0] = br;
      out[(2 * r) * ldo + col1] = -asign * bi;
      out[(2 * r + 1) * ldo + col0] = bi;
      out[(2 * r + 1) * ldo + col1] = asign * br;
    }
  }
}

// 3M: C = (t1 - t2, t3 - t1 - t2)
__global__ __launch_bounds__(TPB) void join_kernel(float2* __restrict__ dst, int64_t rows, int64_t cols, int64_t ld,
                                                   const float* __restrict__ p0, const float* __restrict__ p1,
                                                   const float* __restrict__ p2, int accumulate) {
  int64_t n = rows * cols;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    int64_t r = j / cols, c = j - r * cols;
    float t1 = p0[j], t2 = p1[j], t3 = p2[j];
    float2 z = make_float2(t1 - t2, (t3 - t1) - t2);
    if (accumulate) {
      float2 o = dst[r * ld + c];
      z.x += o.x;
      z.y += o.y;
    }
    dst[r * ld + c] = z;
  }
}

inline int grid_for(int64_t n) {
  int64_t b = ceil_div64(n, TPB), cap = (int64_t)endia::ctx().cu_count * 8;
  if (b > cap) b = cap;
  return (int)(b < 1 ? 1 : b);
}

}  // namespace

using namespace endia;

extern "C" int32_t endia_hip_cgemm(int32_t transA, int32_t conjA, int32_t transB, int32_t conjB, int64_t M, int64_t N,
                                   int64_t K, const float* A, int64_t lda, const float* B, int64_t ldb, float* C,
                                   int64_t ldc, int64_t batch, int64_t strideA, int64_t strideB, int64_t strideC,
                                   int32_t algo, int32_t accumulate) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "cgemm: negative dimension");
  ENDIA_CHECK_ARG(algo == ENDIA_CGEMM_4M || algo == ENDIA_CGEMM_3M, "cgemm: unknown algorithm %d", algo);
  if (M == 0 || N == 0 || batch == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(C != nullptr, "cgemm: C is null");
  ENDIA_CHECK_ARG(K == 0 || (A && B), "cgemm: A or B is null");
  const int64_t a_rows = transA ? K : M, a_cols = transA ? M : K;
  const int64_t b_rows = transB ? N : K, b_cols = transB ? K : N;
  ENDIA_CHECK_ARG(lda >= a_cols && ldb >= b_cols && ldc >= N, "cgemm: leading dimension too small");
  ENDIA_CHECK_ARG(strideA >= 0 && strideB >= 0 && strideC >= 0, "cgemm: negative batch stride");
  hipStream_t s = ctx().stream;

  auto pad4 = [](int64_t n) { return (n + 3) / 4 * 4; };
  const int three_m = algo == ENDIA_CGEMM_3M;

  if (!three_m) {
    // one real GEMM: A as stored (or its stacked planes), the embedded B, C written in place
    const int64_t na = transA ? pad4(2 * M * K) : 0, nb = pad4(4 * K * N);
    void* ws = nullptr;
    int32_t rc = workspace((na + nb) * (int64_t)sizeof(float), &ws);
    if (rc) return rc;
    float* Ae = static_cast<float*>(ws);
    float* Be = Ae + na;
    for (int64_t b = 0; b < batch; ++b) {
      const float2* Ab = reinterpret_cast<const float2*>(A) + b * strideA;
      const float2* Bb = reinterpret_cast<const float2*>(B) + b * strideB;
      float* Cb = C + 2 * b * strideC;
      if (K > 0) {
        if (transA && (b == 0 || strideA != 0))  // operands that broadcast over the batch are prepared once
          hipLaunchKernelGGL(stack_planes_kernel, dim3(grid_for(M * K)), dim3(TPB), 0, s, Ab, a_rows, a_cols, lda, Ae);
        if (b == 0 || strideB != 0)
          hipLaunchKernelGGL(embed_b_kernel, dim3(grid_for(K * N)), dim3(TPB), 0, s, Bb, b_rows, b_cols, ldb,
                             conjB ? -1.f : 1.f, conjA ? -1.f : 1.f, transB ? 1 : 0, transA ? 1 : 0, Be);
        ENDIA_LAUNCH_CHECK();
      }
      const float* Ar = transA ? Ae : reinterpret_cast<const float*>(Ab);
      rc = sgemm_impl(transA, transB, M, 2 * N, 2 * K, Ar, transA ? M : 2 * lda, Be, 2 * b_cols, Cb, 2 * ldc, 1, 0, 0, 0,
                      ENDIA_EPI_NONE | (accumulate ? ENDIA_GEMM_ACCUMULATE : 0), ENDIA_OP_IDENTITY, nullptr, nullptr, nullptr);
      if (rc) return rc;
    }
    return ENDIA_HIP_OK;
  }

  // 3M: planes are padded to a multiple of 4 floats each so every plane starts 16-byte aligned
  const int64_t na = pad4(M * K), nb = pad4(K * N), nc = pad4(M * N);
  const int64_t floats = 3 * na + 3 * nb + 3 * nc;
  void* ws = nullptr;
  int32_t rc = workspace(floats * (int64_t)sizeof(float), &ws);
  if (rc) return rc;
  float* Ar = static_cast<float*>(ws);
  float* Ai = Ar + na;
  float* A3 = Ai + na;  // Ar + Ai
  float* Br = A3 + na;
  float* Bi = Br + nb;
  float* B3 = Bi + nb;  // Br + Bi
  float* P0 = B3 + nb;
  float* P1 = P0 + nc;
  float* P2 = P1 + nc;

  for (int64_t b = 0; b < batch; ++b) {
    const float2* Ab = reinterpret_cast<const float2*>(A) + b * strideA;
    const float2* Bb = reinterpret_cast<const float2*>(B) + b * strideB;
    float2* Cb = reinterpret_cast<float2*>(C) + b * strideC;
    if (K > 0) {
      if (b == 0 || strideA != 0)
        hipLaunchKernelGGL(split_kernel, dim3(grid_for(M * K)), dim3(TPB), 0, s, Ab, a_rows, a_cols, lda,
                           conjA ? -1.f : 1.f, Ar, Ai, A3);
      if (b == 0 || strideB != 0)
        hipLaunchKernelGGL(split_kernel, dim3(grid_for(K * N)), dim3(TPB), 0, s, Bb, b_rows, b_cols, ldb,
                           conjB ? -1.f : 1.f, Br, Bi, B3);
      ENDIA_LAUNCH_CHECK();
    }
    // the three products are independent: one batched launch (the planes are na / nb / nc floats apart)
    rc = sgemm_impl(transA, transB, M, N, K, Ar, a_cols, Br, b_cols, P0, N, 3, na, nb, nc, ENDIA_EPI_NONE, ENDIA_OP_IDENTITY,
                    nullptr, nullptr, nullptr);
    if (rc) return rc;
    hipLaunchKernelGGL(join_kernel, dim3(grid_for(M * N)), dim3(TPB), 0, s, Cb, M, N, ldc, P0, P1, P2, accumulate ? 1 : 0);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}
