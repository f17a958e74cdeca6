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
#include "common.h"

namespace endia {
int32_t sgemm_impl(int transA, int transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                   const float* B, int64_t ldb, float* C, int64_t ldc, int64_t batch, int64_t sA,
                   int64_t sB, int64_t sC, int epi_flags, int act_flags, const float* bias,
                   const float* aux_in, float* aux_out);
}

namespace {

constexpr int TPB = 256;

// src: rows x cols complex, row stride ld (complex). Planes are compact rows x cols.
// re = Re, im = sign*Im, third = (mode 0: -im plane i.e. -sign*Im ; mode 1: re + im ; mode 2: none)
__global__ __launch_bounds__(TPB) void split_kernel(const float2* __restrict__ src, int64_t rows, int64_t cols,
                                                    int64_t ld, float sign, float* __restrict__ re,
                                                    float* __restrict__ im, float* __restrict__ third, int mode) {
  int64_t n = rows * cols;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    int64_t r = j / cols, c = j - r * cols;
    float2 z = src[r * ld + c];
    float i = sign * z.y;
    re[j] = z.x;
    im[j] = i;
    if (mode == 0) third[j] = -i;
    else if (mode == 1) third[j] = z.x + i;
  }
}

// 4M: C = (cr, ci) ; 3M: C = (t1 - t2, t3 - t1 - t2)
__global__ __launch_bounds__(TPB) void join_kernel(float2* __restrict__ dst, int64_t rows, int64_t cols, int64_t ld,
                                                   const float* __restrict__ p0, const float* __restrict__ p1,
                                                   const float* __restrict__ p2, int three_m, int accumulate) {
  int64_t n = rows * cols;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) {
    int64_t r = j / cols, c = j - r * cols;
    float2 z;
    if (three_m) {
      float t1 = p0[j], t2 = p1[j], t3 = p2[j];
      z = make_float2(t1 - t2, (t3 - t1) - t2);
    } else {
      z = make_float2(p0[j], p1[j]);
    }
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

  // planes are padded to a multiple of 4 floats each so every plane starts 16-byte aligned
  auto pad4 = [](int64_t n) { return (n + 3) / 4 * 4; };
  const int64_t na = pad4(M * K), nb = pad4(K * N), nc = pad4(M * N);
  const int64_t floats = 3 * na + 3 * nb + 3 * nc;
  void* ws = nullptr;
  int32_t rc = workspace(floats * (int64_t)sizeof(float), &ws);
  if (rc) return rc;
  float* Ar = static_cast<float*>(ws);
  float* Ai = Ar + na;
  float* A3 = Ai + na;  // 4M: -Ai ; 3M: Ar + Ai
  float* Br = A3 + na;
  float* Bi = Br + nb;
  float* B3 = Bi + nb;  // 3M: Br + Bi
  float* P0 = B3 + nb;
  float* P1 = P0 + nc;
  float* P2 = P1 + nc;
  const int three_m = algo == ENDIA_CGEMM_3M;

  for (int64_t b = 0; b < batch; ++b) {
    const float2* Ab = reinterpret_cast<const float2*>(A) + b * strideA;
    const float2* Bb = reinterpret_cast<const float2*>(B) + b * strideB;
    float2* Cb = reinterpret_cast<float2*>(C) + b * strideC;
    if (K > 0) {
      // operands that broadcast over the batch are split once
      if (b == 0 || strideA != 0)
        hipLaunchKernelGGL(split_kernel, dim3(grid_for(M * K)), dim3(TPB), 0, s, Ab, a_rows, a_cols, lda,
                           conjA ? -1.f : 1.f, Ar, Ai, A3, three_m ? 1 : 0);
      if (b == 0 || strideB != 0)
        hipLaunchKernelGGL(split_kernel, dim3(grid_for(K * N)), dim3(TPB), 0, s, Bb, b_rows, b_cols, ldb,
                           conjB ? -1.f : 1.f, Br, Bi, B3, three_m ? 1 : 2);
      ENDIA_LAUNCH_CHECK();
    }
    auto mm = [&](const float* X, const float* Y, float* Z, int acc) {
      return sgemm_impl(transA, transB, M, N, K, X, a_cols, Y, b_cols, Z, N, 1, 0, 0, 0,
                        ENDIA_EPI_NONE | (acc ? ENDIA_GEMM_ACCUMULATE : 0), ENDIA_OP_IDENTITY, nullptr, nullptr, nullptr);
    };
    if (three_m) {
      if ((rc = mm(Ar, Br, P0, 0))) return rc;
      if ((rc = mm(Ai, Bi, P1, 0))) return rc;
      if ((rc = mm(A3, B3, P2, 0))) return rc;
    } else {
      if ((rc = mm(Ar, Br, P0, 0))) return rc;
      if ((rc = mm(A3, Bi, P0, 1))) return rc;
      if ((rc = mm(Ar, Bi, P1, 0))) return rc;
      if ((rc = mm(Ai, Br, P1, 1))) return rc;
    }
    hipLaunchKernelGGL(join_kernel, dim3(grid_for(M * N)), dim3(TPB), 0, s, Cb, M, N, ldc, P0, P1, P2, three_m,
                       accumulate ? 1 : 0);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}
