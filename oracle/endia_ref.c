/*
 * endia_ref.c -- TEST INFRASTRUCTURE, not product code.
 *
 * A single-threaded CPU restatement, in plain C, of the algorithms on Endia's dense-layer training
 * path, written from the text of the reference (Mojo 24.5, which cannot be built in this image).
 * It keeps the reference's loop structure, its fp32 storage of every intermediate and its
 * accumulation order ("ref order"), so that it serves both as the parity checker of the HIP
 * kernels and as the timed "Endia CPU path" stand-in. Only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may call it; nothing shipped links against it.
 *
 * Build: see oracle/Makefile (-O3, -ffp-contract=off so that no product-sum is fused).
 *
 * How each function is pinned (tests/test_oracle.py, no GPU needed):
 *   matmul (real, complex), binary ops + broadcast (incl. pow and the comparisons), the 21 unary ops
 *   and their VJPs, the complex unary bodies, reduce_add, mse, conv1d / conv2d / conv3d forward, max and
 *   average pooling forward, the strided gather and scatter behind slice / pad / as_strided and their
 *   gradients, SGD, Adam and the full MLP step are compared with PyTorch float64 -- the oracle
 *   the reference's own tests use (tests/test_endia/.../test_matmul_op.mojo:18-59 and siblings,
 *   metric endia/utils/array_conversions.mojo:63-135) -- with the doc known-answers
 *   (README.md:74-76,106-108; examples/custom_ops_examples/custom_mul.mojo:64-71) and with
 *   invariants (adjoint identities for the convolution and pooling gradients, which the reference does
 *   not have; torch autograd gives the same gradients).
 *   Parity unpinned by any reference test: complex matmul VJP without conjugation (pinned by
 *   reading matmul_op.mojo:278-283 only), the convolution gradients (absent from the reference,
 *   conv2d_op.mojo:198-200) and the pooling gradients (absent, max_pool2d_op.mojo:152-154).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* nelts = 2 * simdwidthof[float32] (endia/utils/aliases.mojo:20-21); 8-lane AVX2 host assumed */
#define NELTS 16

enum { OP_RELU, OP_TANH, OP_SIN, OP_COS, OP_NEG, OP_SQUARE, OP_SQRT, OP_ABS, OP_IDENTITY, OP_GREATER0, OP_EXP, OP_LOG,
       OP_SIGMOID, OP_SINH, OP_COSH, OP_TAN, OP_ASIN, OP_ACOS, OP_ATAN, OP_RECIPROCAL, OP_SIGN };
enum { BIN_ADD, BIN_SUB, BIN_MUL, BIN_DIV, BIN_GREATER, BIN_POW, BIN_GREATER_EQUAL, BIN_LESS, BIN_LESS_EQUAL, BIN_EQUAL,
       BIN_NOT_EQUAL };

/* Every op output is a freshly allocated, zero-filled buffer: functional/_utils.mojo:319-324 */
static float* fresh(int64_t n) { return (float*)calloc((size_t)(n > 0 ? n : 1), sizeof(float)); }

/* SIMD reduce_add: pairwise halving of the lane vector */
static float lanes_reduce(float* v, int n) {
  for (int w = n / 2; w >= 1; w /= 2)
    for (int i = 0; i < w; ++i) v[i] = v[i] + v[i + w];
  return v[0];
}

/* ---- execute_copy_raw / contiguous: functional/_utils.mojo:79-205 ----------------------------- */
void ref_strided_copy(int32_t ndim, const int64_t* shape, const int64_t* strides, int64_t offset,
                      const float* src, float* dst, int32_t is_complex) {
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  for (int64_t j = 0; j < n; ++j) {
    int64_t r = j, is = offset;
    for (int k = ndim - 1; k >= 0; --k) {
      is += (r % shape[k]) * strides[k];
      r /= shape[k];
    }
    if (is_complex) {
      dst[2 * j] = src[2 * is];
      dst[2 * j + 1] = src[2 * is + 1];
    } else {
      dst[j] = src[is];
    }
  }
}

/* ---- the store side of a view. Pad.__call__ (view_ops/pad_op.mojo:115-142) stores its argument element
 * by element through a slice view of the zero-filled result; AsStridedInv.__call__
 * (view_ops/as_strided_op.mojo:169-190) adds it, in row-major order of the view, so that overlapping
 * windows accumulate. dst must already hold the zero-filled target. */
void ref_strided_scatter(int32_t ndim, const int64_t* shape, const int64_t* strides, int64_t offset,
                         const float* src, float* dst, int32_t accumulate, int32_t is_complex) {
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  const int w = is_complex ? 2 : 1;
  for (int64_t j = 0; j < n; ++j) {
    int64_t r = j, id = offset;
    for (int k = ndim - 1; k >= 0; --k) {
      id += (r % shape[k]) * strides[k];
      r /= shape[k];
    }
    for (int c = 0; c < w; ++c) {
      if (accumulate) dst[w * id + c] = dst[w * id + c] + src[w * j + c];
      else dst[w * id + c] = src[w * j + c];
    }
  }
}

/* ---- matmul_fwd: binary_ops/matmul_op.mojo:93-254 ---------------------------------------------
 * A is addressed as A[b*a_bs + m*a_rs + k*a_cs], B as B[b*b_bs + k*b_rs + n*b_cs] (element strides, so
 * a .T() view is a_rs/a_cs swapped). Step 1: contiguous copy of the LHS (:107). Step 2: contiguous
 * TRANSPOSED copy of the RHS, [N][K] (:111-136; the square-matrix shortcut of :121-129 is not
 * reproduced -- the documented semantics are). Step 3: one dot product per output element with NELTS
 * partial sums, a horizontal add, then a scalar tail (:181-199). */
void ref_matmul(int64_t batch, int64_t M, int64_t N, int64_t K, const float* A, int64_t a_bs, int64_t a_rs,
                int64_t a_cs, const float* B, int64_t b_bs, int64_t b_rs, int64_t b_cs, float* C) {
  float* lhs = fresh(M * K);
  float* rhs = fresh(N * K);
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) lhs[m * K + k] = A[b * a_bs + m * a_rs + k * a_cs];
    for (int64_t n = 0; n < N; ++n)
      for (int64_t k = 0; k < K; ++k) rhs[n * K + k] = B[b * b_bs + k * b_rs + n * b_cs];
    int64_t k_end = K - (K % NELTS);
    float* Cb = C + b * M * N;
    for (int64_t m = 0; m < M; ++m) {
      const float* l = lhs + m * K;
      for (int64_t n = 0; n < N; ++n) {
        const float* r = rhs + n * K;
        float sum[NELTS];
        for (int i = 0; i < NELTS; ++i) sum[i] = 0.f;
        for (int64_t k = 0; k < k_end; k += NELTS)
          for (int i = 0; i < NELTS; ++i) sum[i] = sum[i] + l[k + i] * r[k + i];
        float s = lanes_reduce(sum, NELTS);
        for (int64_t k = k_end; k < K; ++k) s = s + l[k] * r[k];
        Cb[m * N + n] = s;
      }
    }
  }
  free(lhs);
  free(rhs);
}

/* complex branch: matmul_op.mojo:201-238. Interleaved operands, strides in complex elements. */
void ref_cmatmul(int64_t batch, int64_t M, int64_t N, int64_t K, const float* A, int64_t a_bs, int64_t a_rs,
                 int64_t a_cs, const float* B, int64_t b_bs, int64_t b_rs, int64_t b_cs, float* C) {
  float* lhs = fresh(2 * M * K);
  float* rhs = fresh(2 * N * K);
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) {
        int64_t s = b * a_bs + m * a_rs + k * a_cs;
        lhs[2 * (m * K + k)] = A[2 * s];
        lhs[2 * (m * K + k) + 1] = A[2 * s + 1];
      }
    for (int64_t n = 0; n < N; ++n)
      for (int64_t k = 0; k < K; ++k) {
        int64_t s = b * b_bs + k * b_rs + n * b_cs;
        rhs[2 * (n * K + k)] = B[2 * s];
        rhs[2 * (n * K + k) + 1] = B[2 * s + 1];
      }
    int64_t k_end = K - (K % NELTS);
    float* Cb = C + 2 * b * M * N;
    for (int64_t m = 0; m < M; ++m) {
      const float* l = lhs + 2 * m * K;
      for (int64_t n = 0; n < N; ++n) {
        const float* r = rhs + 2 * n * K;
        float sr[NELTS], si[NELTS];
        for (int i = 0; i < NELTS; ++i) sr[i] = si[i] = 0.f;
        for (int64_t k = 0; k < k_end; k += NELTS)
          for (int i = 0; i < NELTS; ++i) {
            float lr = l[2 * (k + i)], li = l[2 * (k + i) + 1], rr = r[2 * (k + i)], ri = r[2 * (k + i) + 1];
            sr[i] = sr[i] + (lr * rr - li * ri);
            si[i] = si[i] + (lr * ri + li * rr);
          }
        float re = lanes_reduce(sr, NELTS), im = lanes_reduce(si, NELTS);
        for (int64_t k = k_end; k < K; ++k) {
          float lr = l[2 * k], li = l[2 * k + 1], rr = r[2 * k], ri = r[2 * k + 1];
          re = re + (lr * rr - li * ri);
          im = im + (lr * ri + li * rr);
        }
        Cb[2 * (m * N + n)] = re;
        Cb[2 * (m * N + n) + 1] = im;
      }
    }
  }
  free(lhs);
  free(rhs);
}

/* ---- unary forward bodies (real path = complex SIMD body with imag = 0) ------------------------ */
static float unary_real(int op, float x) {
  switch (op) {
    case OP_RELU: return x > 0.f ? x : 0.f;                          /* relu_op.mojo:115-117 */
    case OP_TANH: return sinhf(2.f * x) / (coshf(2.f * x) + cosf(0.f)); /* tanh_op.mojo:112-115 */
    case OP_SIN: return sinf(x) * coshf(0.f);                        /* sin_op.mojo:112-114 */
    case OP_COS: return cosf(x) * coshf(0.f);                        /* cos_op.mojo:113-115 */
    case OP_NEG: return -x;                                          /* neg_op.mojo:111-113 */
    case OP_SQUARE: return x * x - 0.f * 0.f;                        /* square_op.mojo:117-119 */
    case OP_SQRT: {                                                  /* sqrt_op.mojo:111-114 */
      float r = sqrtf(x * x + 0.f);
      return sqrtf((r + x) / 2.f);
    }
    case OP_ABS: return sqrtf(x * x + 0.f);                          /* abs_op.mojo:114-115 */
    case OP_GREATER0: return x > 0.f ? 1.f : 0.f;                    /* greater_op.mojo:46-60 */
    case OP_EXP: return expf(x) * cosf(0.f);                         /* exp_op.mojo:113 */
    case OP_LOG: return logf(sqrtf(x * x + 0.f));                    /* log_op.mojo:111-113 */
    case OP_SIGMOID: return 1.f / (1.f + expf(-x));                  /* sigmoid_op.mojo:120 */
    case OP_SINH: return sinhf(x) * cosf(0.f);                       /* sinh_op.mojo:108 */
    case OP_COSH: return coshf(x) * cosf(0.f);                       /* cosh_op.mojo:109 */
    case OP_TAN: return tanf(x);                                     /* tan_op.mojo (real body) */
    case OP_ASIN: return asinf(x) * coshf(0.f);                      /* asin_op.mojo:103 */
    case OP_ACOS: return acosf(x);                                   /* acos_op.mojo:111 */
    case OP_ATAN: return atanf(x);                                   /* atan_op.mojo:105 */
    case OP_RECIPROCAL: return x / (x * x + 0.f);                    /* reciprocal_op.mojo:115-116 */
    case OP_SIGN: return x / sqrtf(x * x + 0.f);                     /* sign_op.mojo:78-79 */
    default: return x;
  }
}

/* execute_unary_op: unary_ops/_utils.mojo:77-134 */
void ref_unary(int32_t op, int64_t n, const float* x, float* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = unary_real(op, x[i]);
}

/* flat binary op on materialised operands: binary_ops/_utils.mojo:93-177 */
static void binary_flat(int op, int64_t n, const float* a, const float* b, float* o) {
  switch (op) {
    case BIN_ADD: for (int64_t i = 0; i < n; ++i) o[i] = a[i] + b[i]; break;
    case BIN_SUB: for (int64_t i = 0; i < n; ++i) o[i] = a[i] - b[i]; break;
    case BIN_MUL: for (int64_t i = 0; i < n; ++i) o[i] = a[i] * b[i]; break;
    case BIN_DIV: for (int64_t i = 0; i < n; ++i) o[i] = a[i] / b[i]; break;
    case BIN_POW: /* pow_op.mojo:139-146 with zero imaginary parts */
      for (int64_t i = 0; i < n; ++i) {
        float log_mag = logf(sqrtf(a[i] * a[i] + 0.f));
        float arg = atan2f(0.f, a[i]);
        float u = expf(log_mag * b[i] - arg * 0.f);
        float v = log_mag * 0.f + arg * b[i];
        o[i] = u * cosf(v);
      }
      break;
    case BIN_GREATER_EQUAL: for (int64_t i = 0; i < n; ++i) o[i] = a[i] >= b[i] ? 1.f : 0.f; break;
    case BIN_LESS: for (int64_t i = 0; i < n; ++i) o[i] = a[i] < b[i] ? 1.f : 0.f; break;
    case BIN_LESS_EQUAL: for (int64_t i = 0; i < n; ++i) o[i] = a[i] <= b[i] ? 1.f : 0.f; break;
    case BIN_EQUAL: for (int64_t i = 0; i < n; ++i) o[i] = a[i] == b[i] ? 1.f : 0.f; break;
    case BIN_NOT_EQUAL: for (int64_t i = 0; i < n; ++i) o[i] = a[i] != b[i] ? 1.f : 0.f; break;
    default: for (int64_t i = 0; i < n; ++i) o[i] = a[i] > b[i] ? 1.f : 0.f; break;
  }
}

static void binary_flat_complex(int op, int64_t n, const float* a, const float* b, float* o) {
  for (int64_t i = 0; i < n; ++i) {
    float ar = a[2 * i], ai = a[2 * i + 1], br = b[2 * i], bi = b[2 * i + 1];
    switch (op) {
      case BIN_ADD: o[2 * i] = ar + br; o[2 * i + 1] = ai + bi; break;      /* add_op.mojo:134 */
      case BIN_SUB: o[2 * i] = ar - br; o[2 * i + 1] = ai - bi; break;      /* sub_op.mojo:136 */
      case BIN_MUL: o[2 * i] = ar * br - ai * bi; o[2 * i + 1] = ar * bi + ai * br; break; /* mul_op.mojo:152-155 */
      case BIN_POW: {                                                       /* pow_op.mojo:139-146 */
        float log_mag = logf(sqrtf(ar * ar + ai * ai));
        float arg = atan2f(ai, ar);
        float u = expf(log_mag * br - arg * bi);
        float v = log_mag * bi + arg * br;
        o[2 * i] = u * cosf(v);
        o[2 * i + 1] = u * sinf(v);
        break;
      }
      default: {                                                            /* div_op.mojo:117-142 */
        float d = br * br + bi * bi;
        o[2 * i] = (ar * br + ai * bi) / d;
        o[2 * i + 1] = (ai * br - ar * bi) / d;
      }
    }
  }
}

/* binary_op_array + execute_binary_op: both operands are expanded to the broadcast shape (stride-0
 * views, binary_ops/_utils.mojo:83-86) and then made contiguous, i.e. materialised (:95-96). */
void ref_binary(int32_t op, int32_t ndim, const int64_t* shape, const int64_t* a_strides, const int64_t* b_strides,
                const float* a, const float* b, float* out, int32_t is_complex) {
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  int w = is_complex ? 2 : 1;
  float* am = fresh(n * w);
  float* bm = fresh(n * w);
  ref_strided_copy(ndim, shape, a_strides, 0, a, am, is_complex);
  ref_strided_copy(ndim, shape, b_strides, 0, b, bm, is_complex);
  if (is_complex) binary_flat_complex(op, n, am, bm, out);
  else binary_flat(op, n, am, bm, out);
  free(am);
  free(bm);
}

/* VJP rules, composed from the same ops the reference composes them from */
void ref_unary_vjp(int32_t op, int64_t n, const float* x, const float* g, float* dx) {
  float* t = fresh(n);
  float* u = fresh(n);
  switch (op) {
    case OP_RELU: /* greater(x, zeros) * g : relu_op.mojo:95 */
      for (int64_t i = 0; i < n; ++i) t[i] = x[i] > 0.f ? 1.f : 0.f;
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_TANH: /* (1 - square(tanh(x))) * g : tanh_op.mojo:92 */
      ref_unary(OP_TANH, n, x, t);
      ref_unary(OP_SQUARE, n, t, u);
      for (int64_t i = 0; i < n; ++i) t[i] = 1.f - u[i];
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_SIN: /* cos(x) * g : sin_op.mojo:92 */
      ref_unary(OP_COS, n, x, t);
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_COS: /* -sin(x) * g : cos_op.mojo:93 */
      ref_unary(OP_SIN, n, x, t);
      ref_unary(OP_NEG, n, t, u);
      binary_flat(BIN_MUL, n, u, g, dx);
      break;
    case OP_NEG: /* -g : neg_op.mojo:91 */
      ref_unary(OP_NEG, n, g, dx);
      break;
    case OP_SQUARE: /* 2 * x * g : square_op.mojo:96 */
      for (int64_t i = 0; i < n; ++i) t[i] = 2.f * x[i];
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_SQRT: /* g / (2 * sqrt(x)) : sqrt_op.mojo:91 */
      ref_unary(OP_SQRT, n, x, t);
      for (int64_t i = 0; i < n; ++i) u[i] = 2.f * t[i];
      binary_flat(BIN_DIV, n, g, u, dx);
      break;
    case OP_ABS: /* sign(x) * g, sign = x / |x| : abs_op.mojo:93, sign_op.mojo:78-81 (NaN at 0) */
      for (int64_t i = 0; i < n; ++i) t[i] = x[i] / sqrtf(x[i] * x[i] + 0.f);
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_EXP: /* exp(x) * g : exp_op.mojo:92 */
      ref_unary(OP_EXP, n, x, t);
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_LOG: /* g / x : log_op.mojo:91 */
      binary_flat(BIN_DIV, n, g, x, dx);
      break;
    case OP_SIGMOID: /* out * (1 - out) * g : sigmoid_op.mojo:98 */
      ref_unary(OP_SIGMOID, n, x, t);
      for (int64_t i = 0; i < n; ++i) u[i] = 1.f - t[i];
      binary_flat(BIN_MUL, n, t, u, u);
      binary_flat(BIN_MUL, n, u, g, dx);
      break;
    case OP_SINH: /* cosh(x) * g : sinh_op.mojo:88 */
      ref_unary(OP_COSH, n, x, t);
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_COSH: /* sinh(x) * g : cosh_op.mojo:89 */
      ref_unary(OP_SINH, n, x, t);
      binary_flat(BIN_MUL, n, t, g, dx);
      break;
    case OP_TAN: /* g * (1 + square(out)) : tan_op.mojo:81 */
      ref_unary(OP_TAN, n, x, t);
      ref_unary(OP_SQUARE, n, t, u);
      for (int64_t i = 0; i < n; ++i) t[i] = 1.f + u[i];
      binary_flat(BIN_MUL, n, g, t, dx);
      break;
    case OP_ASIN: /* g / sqrt(1 - x ** 2) : asin_op.mojo:83 */
    case OP_ACOS: /* -1 / sqrt(1 - x ** 2) * g : acos_op.mojo:91 */
      for (int64_t i = 0; i < n; ++i) u[i] = 2.f;
      binary_flat(BIN_POW, n, x, u, t);
      for (int64_t i = 0; i < n; ++i) u[i] = 1.f - t[i];
      ref_unary(OP_SQRT, n, u, t);
      if (op == OP_ASIN) {
        binary_flat(BIN_DIV, n, g, t, dx);
      } else {
        for (int64_t i = 0; i < n; ++i) u[i] = -1.f / t[i];
        binary_flat(BIN_MUL, n, u, g, dx);
      }
      break;
    case OP_ATAN: /* g / (1 + square(x)) : atan_op.mojo:85 */
      ref_unary(OP_SQUARE, n, x, t);
      for (int64_t i = 0; i < n; ++i) u[i] = 1.f + t[i];
      binary_flat(BIN_DIV, n, g, u, dx);
      break;
    case OP_RECIPROCAL: /* -g / square(x) : reciprocal_op.mojo:95 */
      ref_unary(OP_NEG, n, g, t);
      ref_unary(OP_SQUARE, n, x, u);
      binary_flat(BIN_DIV, n, t, u, dx);
      break;
    default: /* identity; sign hands the gradient on (default_vjp, sign_op.mojo:58, _array.mojo:43-47) */
      memcpy(dx, g, (size_t)n * sizeof(float));
  }
  free(t);
  free(u);
}

/* complex -> complex forward bodies, interleaved in and out */
void ref_unary_complex(int32_t op, int64_t n, const float* z, float* y) {
  for (int64_t i = 0; i < n; ++i) {
    float a = z[2 * i], b = z[2 * i + 1], re = a, im = b;
    switch (op) {
      case OP_NEG: re = -a; im = -b; break;                                             /* neg_op.mojo:111-113 */
      case OP_SQUARE: re = a * a - b * b; im = 2.f * a * b; break;                      /* square_op.mojo:117-119 */
      case OP_SIN: re = sinf(a) * coshf(b); im = cosf(a) * sinhf(b); break;             /* sin_op.mojo:112-113 */
      case OP_COS: re = cosf(a) * coshf(b); im = -sinf(a) * sinhf(b); break;            /* cos_op.mojo:113-114 */
      case OP_TANH: {                                                                   /* tanh_op.mojo:112-115 */
        float d = coshf(2.f * a) + cosf(2.f * b);
        re = sinhf(2.f * a) / d; im = sinf(2.f * b) / d;
        break;
      }
      case OP_EXP: re = expf(a) * cosf(b); im = expf(a) * sinf(b); break;               /* exp_op.mojo:113-114 */
      case OP_LOG: re = logf(sqrtf(a * a + b * b)); im = atan2f(b, a); break;           /* log_op.mojo:111-114 */
      case OP_SINH: re = sinhf(a) * cosf(b); im = coshf(a) * sinf(b); break;            /* sinh_op.mojo:108-109 */
      case OP_COSH: re = coshf(a) * cosf(b); im = sinhf(a) * sinf(b); break;            /* cosh_op.mojo:109-110 */
      case OP_SQRT: {                                                                   /* sqrt_op.mojo:111-113 */
        float r = sqrtf(a * a + b * b);
        re = sqrtf((r + a) / 2.f); im = copysignf(sqrtf((r - a) / 2.f), b);
        break;
      }
      case OP_RECIPROCAL: { float d = a * a + b * b; re = a / d; im = -b / d; break; }  /* reciprocal_op.mojo:115-117 */
      case OP_SIGN: { float r = sqrtf(a * a + b * b); re = a / r; im = b / r; break; }  /* sign_op.mojo:78-80 */
      default: break;
    }
    y[2 * i] = re;
    y[2 * i + 1] = im;
  }
}

/* complex |z| forward (n real outputs) and its VJP sign(z)*complex(g,0): abs_op.mojo:93,114-115,157;
 * sign_op.mojo:78-81; real_op.mojo:74-77 */
void ref_cabs(int64_t n, const float* z, float* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = sqrtf(z[2 * i] * z[2 * i] + z[2 * i + 1] * z[2 * i + 1]);
}
void ref_cabs_vjp(int64_t n, const float* z, const float* g, float* dz) {
  for (int64_t i = 0; i < n; ++i) {
    float norm = sqrtf(z[2 * i] * z[2 * i] + z[2 * i + 1] * z[2 * i + 1]);
    float sr = z[2 * i] / norm, si = z[2 * i + 1] / norm;
    dz[2 * i] = sr * g[i] - si * 0.f;
    dz[2 * i + 1] = sr * 0.f + si * g[i];
  }
}

/* ---- ReduceAdd.__call__: reduce_ops/reduce_add_op.mojo:65-210. Axes with mask bit set are summed and
 * kept as size 1. The output is zero-initialised and every input element is added to its target in
 * row-major input order (:112-159); the rank-1 full reduction adds one NELTS-wide horizontal sum
 * per step and then a scalar tail (:160-190). */
void ref_reduce_add(int32_t ndim, const int64_t* shape, uint32_t mask, const float* x, float* out, int32_t is_complex) {
  int64_t n = 1, nout = 1, tstride[8];
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  for (int i = ndim - 1; i >= 0; --i) {
    int red = (mask >> i) & 1;
    tstride[i] = red ? 0 : nout;
    if (!red) nout *= shape[i];
  }
  int w = is_complex ? 2 : 1;
  for (int64_t i = 0; i < nout * w; ++i) out[i] = 0.f;
  if (ndim == 1 && (mask & 1) && !is_complex) {
    int64_t end = n - n % NELTS;
    for (int64_t i = 0; i < end; i += NELTS) {
      float v[NELTS];
      for (int k = 0; k < NELTS; ++k) v[k] = x[i + k];
      out[0] = out[0] + lanes_reduce(v, NELTS);
    }
    for (int64_t i = end; i < n; ++i) out[0] = out[0] + x[i];
    return;
  }
  for (int64_t j = 0; j < n; ++j) {
    int64_t r = j, t = 0;
    for (int k = ndim - 1; k >= 0; --k) {
      t += (r % shape[k]) * tstride[k];
      r /= shape[k];
    }
    if (is_complex) {
      out[2 * t] = out[2 * t] + x[2 * j];
      out[2 * t + 1] = out[2 * t + 1] + x[2 * j + 1];
    } else {
      out[t] = out[t] + x[j];
    }
  }
}

/* ---- ReduceMax / ReduceMin / ReduceMul .__call__ (reduce_ops/reduce_max_op.mojo:66-190, reduce_min_op.mojo:66-190,
 * reduce_mul_op.mojo:65-210) and ReduceArgMax / ReduceArgMin .__call__ (reduce_argmax_op.mojo:66-163,
 * reduce_argmin_op.mojo:66-163). op: 0 max, 1 min, 2 product, 3 argmax, 4 argmin. The output starts at -inf / +inf /
 * 1 (the arg variants at -1 beside a running extreme of -inf / +inf) and every input element is folded into its
 * target in row-major input order; an arg variant records the element's position along the ONE reduced axis when
 * the element is strictly beyond the running extreme (reduce_argmax_op.mojo:136-142; for one reduced axis the
 * recorded quotient arg_max_idx // denom is that position). */
void ref_reduce_op(int32_t op, int32_t ndim, const int64_t* shape, uint32_t mask, const float* x, float* out) {
  int64_t n = 1, nout = 1, tstride[8], red_axis = -1;
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  for (int i = ndim - 1; i >= 0; --i) {
    int red = (mask >> i) & 1;
    tstride[i] = red ? 0 : nout;
    if (!red) nout *= shape[i];
    else red_axis = i;
  }
  const int arg = op >= 3, up = (op == 0 || op == 3);
  float* run = arg ? fresh(nout) : out;  /* the running extreme (tmp_max in the reference's arg variants) */
  for (int64_t i = 0; i < nout; ++i) {
    run[i] = op == 2 ? 1.f : (up ? -INFINITY : INFINITY);
    if (arg) out[i] = -1.f;
  }
  for (int64_t j = 0; j < n; ++j) {
    int64_t r = j, t = 0, pos = 0;
    for (int k = ndim - 1; k >= 0; --k) {
      int64_t idx = r % shape[k];
      t += idx * tstride[k];
      if (k == red_axis) pos = idx;
      r /= shape[k];
    }
    const float v = x[j];
    if (op == 2) {
      run[t] = run[t] * v;
    } else {
      const float next = up ? (run[t] > v ? run[t] : v) : (run[t] < v ? run[t] : v);
      if (arg && (up ? next > run[t] : next < run[t])) out[t] = (float)pos;
      run[t] = next;
    }
  }
  if (arg) free(run);
}

/* ---- mse: loss_ops/mse_op.mojo:17-20 = sum((p - t) * (p - t)) / n, and the gradient its VJP chain
 * yields: Div.vjp g/n (div_op.mojo:108-110), ReduceAdd.vjp expand (reduce_add_op.mojo:234), Mul.vjp
 * returns diff*g for both operands, which land on the same tensor and are added
 * (mul_op.mojo:125-128, autograd/functional.mojo:55-57), Sub.vjp passes g to pred (sub_op.mojo:109-112). */
void ref_mse(int64_t n, const float* pred, const float* target, float* loss, float* dpred) {
  float* diff = fresh(n);
  float* sq = fresh(n);
  binary_flat(BIN_SUB, n, pred, target, diff);
  binary_flat(BIN_MUL, n, diff, diff, sq);
  float s = 0.f;
  for (int64_t i = 0; i < n; ++i) s = s + sq[i];
  float nf = (float)n;
  if (loss) *loss = s / nf;
  if (dpred) {
    float g = 1.f / nf;
    for (int64_t i = 0; i < n; ++i) {
      float a = diff[i] * g;
      dpred[i] = a + a;
    }
  }
  free(diff);
  free(sq);
}

/* ---- Conv2d.__call__: spacial_ops/conv2d_op.mojo:88-196 (groups = 1) -------------------------- */
typedef struct {
  int64_t N, C, H, W, K, R, S;
  int64_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, groups;
} conv_desc;

static void conv_out(const conv_desc* d, int64_t* P, int64_t* Q) {
  *P = (d->H + 2 * d->pad_h - d->dil_h * (d->R - 1) - 1) / d->stride_h + 1; /* conv2d_op.mojo:65-84 */
  *Q = (d->W + 2 * d->pad_w - d->dil_w * (d->S - 1) - 1) / d->stride_w + 1;
}

void ref_conv2d_fwd(const conv_desc* d, const float* x, const float* w, const float* bias, float* y) {
  int64_t P, Q;
  conv_out(d, &P, &Q);
  for (int64_t n = 0; n < d->N; ++n)
    for (int64_t k = 0; k < d->K; ++k)
      for (int64_t p = 0; p < P; ++p) {
        int64_t h0 = p * d->stride_h - d->pad_h;
        for (int64_t q = 0; q < Q; ++q) {
          float value = 0.f;
          int64_t w0 = q * d->stride_w - d->pad_w;
          for (int64_t c = 0; c < d->C; ++c)
            for (int64_t r = 0; r < d->R; ++r) {
              int64_t h = h0 + r * d->dil_h;
              if (h < 0 || h >= d->H) continue;
              for (int64_t s = 0; s < d->S; ++s) {
                int64_t ww = w0 + s * d->dil_w;
                if (ww < 0 || ww >= d->W) continue;
                value = value + x[((n * d->C + c) * d->H + h) * d->W + ww] * w[((k * d->C + c) * d->R + r) * d->S + s];
              }
            }
          y[((n * d->K + k) * P + p) * Q + q] = value + (bias ? bias[k] : 0.f);
        }
      }
}

/* Adjoints of the loop above (not in the reference: Conv2d.vjp is default_vjp, conv2d_op.mojo:198-200).
 * Brute force: every (output element, tap) pair of the forward loop scatters its contribution. */
void ref_conv2d_bwd(const conv_desc* d, const float* x, const float* w, const float* dy, float* dx, float* dw, float* db) {
  int64_t P, Q;
  conv_out(d, &P, &Q);
  if (dx) memset(dx, 0, sizeof(float) * (size_t)(d->N * d->C * d->H * d->W));
  if (dw) memset(dw, 0, sizeof(float) * (size_t)(d->K * d->C * d->R * d->S));
  if (db) memset(db, 0, sizeof(float) * (size_t)d->K);
  for (int64_t n = 0; n < d->N; ++n)
    for (int64_t k = 0; k < d->K; ++k)
      for (int64_t p = 0; p < P; ++p)
        for (int64_t q = 0; q < Q; ++q) {
          float g = dy[((n * d->K + k) * P + p) * Q + q];
          if (db) db[k] = db[k] + g;
          int64_t h0 = p * d->stride_h - d->pad_h, w0 = q * d->stride_w - d->pad_w;
          for (int64_t c = 0; c < d->C; ++c)
            for (int64_t r = 0; r < d->R; ++r) {
              int64_t h = h0 + r * d->dil_h;
              if (h < 0 || h >= d->H) continue;
              for (int64_t s = 0; s < d->S; ++s) {
                int64_t ww = w0 + s * d->dil_w;
                if (ww < 0 || ww >= d->W) continue;
                int64_t xi = ((n * d->C + c) * d->H + h) * d->W + ww, wi = ((k * d->C + c) * d->R + r) * d->S + s;
                if (dx) dx[xi] = dx[xi] + g * w[wi];
                if (dw) dw[wi] = dw[wi] + g * x[xi];
              }
            }
        }
}

/* ---- pooling: MaxPool{1,2,3}d.__call__ / AvgPool{1,2,3}d.__call__ (spacial_ops/max_pool2d_op.mojo:88-150,
 * avg_pool2d_op.mojo:84-140 and their 1-D / 3-D siblings) over [N, C, D, H, W]; the 1-D and 2-D ops are the
 * cases D = 1 (and H = 1). mode 0 = max, 1 = average over the taps inside the array. ---------------- */
typedef struct {
  int64_t N, C, D, H, W;
  int64_t kernel[3], stride[3], padding[3], dilation[3];
} pool_desc;

static void pool_out(const pool_desc* d, int64_t* o) {
  const int64_t in[3] = {d->D, d->H, d->W};
  for (int i = 0; i < 3; ++i) /* max_pool2d_op.mojo:57-82 */
    o[i] = (in[i] + 2 * d->padding[i] - d->dilation[i] * (d->kernel[i] - 1) - 1) / d->stride[i] + 1;
}

void ref_pool_out_shape(const pool_desc* d, int64_t* o) { pool_out(d, o); }

void ref_pool_fwd(const pool_desc* d, int32_t mode, const float* x, float* y) {
  int64_t o[3];
  pool_out(d, o);
  for (int64_t nc = 0; nc < d->N * d->C; ++nc)
    for (int64_t oz = 0; oz < o[0]; ++oz)
      for (int64_t oy = 0; oy < o[1]; ++oy)
        for (int64_t ox = 0; ox < o[2]; ++ox) {
          int64_t z0 = oz * d->stride[0] - d->padding[0], y0 = oy * d->stride[1] - d->padding[1],
                  x0 = ox * d->stride[2] - d->padding[2];
          float max_val = -INFINITY, sum_val = 0.f;
          int64_t count = 0;
          for (int64_t kz = 0; kz < d->kernel[0]; ++kz) {
            int64_t z = z0 + kz * d->dilation[0];
            if (z < 0 || z >= d->D) continue;
            for (int64_t ky = 0; ky < d->kernel[1]; ++ky) {
              int64_t yy = y0 + ky * d->dilation[1];
              if (yy < 0 || yy >= d->H) continue;
              for (int64_t kx = 0; kx < d->kernel[2]; ++kx) {
                int64_t xx = x0 + kx * d->dilation[2];
                if (xx < 0 || xx >= d->W) continue;
                float val = x[((nc * d->D + z) * d->H + yy) * d->W + xx];
                max_val = max_val > val ? max_val : val; /* max(max_val, val): max_pool2d_op.mojo:137 */
                sum_val = sum_val + val;                 /* avg_pool2d_op.mojo:129-130 */
                ++count;
              }
            }
          }
          y[((nc * o[0] + oz) * o[1] + oy) * o[2] + ox] =
              mode == 0 ? max_val : (count > 0 ? sum_val / (float)count : 0.f); /* avg_pool2d_op.mojo:137-140 */
        }
}

/* Adjoint of the loop above (the reference has none: vjp = default_vjp, max_pool2d_op.mojo:152-154), in
 * scatter form: every output hands its gradient to the first tap that attains its maximum (max), or an
 * equal share to every tap inside the array (average). */
void ref_pool_bwd(const pool_desc* d, int32_t mode, const float* x, const float* dy, float* dx) {
  int64_t o[3];
  pool_out(d, o);
  memset(dx, 0, sizeof(float) * (size_t)(d->N * d->C * d->D * d->H * d->W));
  for (int64_t nc = 0; nc < d->N * d->C; ++nc)
    for (int64_t oz = 0; oz < o[0]; ++oz)
      for (int64_t oy = 0; oy < o[1]; ++oy)
        for (int64_t ox = 0; ox < o[2]; ++ox) {
          int64_t z0 = oz * d->stride[0] - d->padding[0], y0 = oy * d->stride[1] - d->padding[1],
                  x0 = ox * d->stride[2] - d->padding[2];
          float g = dy[((nc * o[0] + oz) * o[1] + oy) * o[2] + ox];
          int64_t count = 0, best = -1;
          for (int pass = 0; pass < 2; ++pass)
            for (int64_t kz = 0; kz < d->kernel[0]; ++kz) {
              int64_t z = z0 + kz * d->dilation[0];
              if (z < 0 || z >= d->D) continue;
              for (int64_t ky = 0; ky < d->kernel[1]; ++ky) {
                int64_t yy = y0 + ky * d->dilation[1];
                if (yy < 0 || yy >= d->H) continue;
                for (int64_t kx = 0; kx < d->kernel[2]; ++kx) {
                  int64_t xx = x0 + kx * d->dilation[2];
                  if (xx < 0 || xx >= d->W) continue;
                  int64_t at = ((nc * d->D + z) * d->H + yy) * d->W + xx;
                  if (pass == 0) {
                    ++count;
                    if (best < 0 || x[at] > x[best]) best = at;
                  } else if (mode == 1) {
                    dx[at] = dx[at] + g / (float)count;
                  }
                }
              }
            }
          if (mode == 0 && best >= 0) dx[best] = dx[best] + g;
        }
}

/* ---- Conv3d.__call__: spacial_ops/conv3d_op.mojo:104-259 (groups = 1); Conv1d is the case D = H = 1
 * (spacial_ops/conv1d_op.mojo). x [N,C,D,H,W], w [K,C,T,R,S], bias [K] or null. -------------------- */
typedef struct {
  int64_t N, C, D, H, W, K, T, R, S;
  int64_t stride[3], padding[3], dilation[3];
} conv3d_desc;

static void conv3d_out(const conv3d_desc* d, int64_t* o) {
  const int64_t in[3] = {d->D, d->H, d->W}, k[3] = {d->T, d->R, d->S};
  for (int i = 0; i < 3; ++i) o[i] = (in[i] + 2 * d->padding[i] - d->dilation[i] * (k[i] - 1) - 1) / d->stride[i] + 1;
}

void ref_conv3d_out_shape(const conv3d_desc* d, int64_t* o) { conv3d_out(d, o); }

/* forward when dx, dw, db are all null; otherwise the adjoints, every (output, tap) pair scattering its term */
void ref_conv3d(const conv3d_desc* d, const float* x, const float* w, const float* bias, float* y, const float* dy,
                float* dx, float* dw, float* db) {
  int64_t o[3];
  conv3d_out(d, o);
  int bwd = dx || dw || db;
  if (dx) memset(dx, 0, sizeof(float) * (size_t)(d->N * d->C * d->D * d->H * d->W));
  if (dw) memset(dw, 0, sizeof(float) * (size_t)(d->K * d->C * d->T * d->R * d->S));
  if (db) memset(db, 0, sizeof(float) * (size_t)d->K);
  for (int64_t n = 0; n < d->N; ++n)
    for (int64_t k = 0; k < d->K; ++k)
      for (int64_t oz = 0; oz < o[0]; ++oz)
        for (int64_t oy = 0; oy < o[1]; ++oy)
          for (int64_t ox = 0; ox < o[2]; ++ox) {
            int64_t oi = (((n * d->K + k) * o[0] + oz) * o[1] + oy) * o[2] + ox;
            float value = 0.f, g = bwd ? dy[oi] : 0.f;
            if (db) db[k] = db[k] + g;
            int64_t z0 = oz * d->stride[0] - d->padding[0], y0 = oy * d->stride[1] - d->padding[1],
                    x0 = ox * d->stride[2] - d->padding[2];
            for (int64_t c = 0; c < d->C; ++c)
              for (int64_t kz = 0; kz < d->T; ++kz) {
                int64_t z = z0 + kz * d->dilation[0];
                if (z < 0 || z >= d->D) continue;
                for (int64_t ky = 0; ky < d->R; ++ky) {
                  int64_t yy = y0 + ky * d->dilation[1];
                  if (yy < 0 || yy >= d->H) continue;
                  for (int64_t kx = 0; kx < d->S; ++kx) {
                    int64_t xx = x0 + kx * d->dilation[2];
                    if (xx < 0 || xx >= d->W) continue;
                    int64_t xi = (((n * d->C + c) * d->D + z) * d->H + yy) * d->W + xx;
                    int64_t wi = (((k * d->C + c) * d->T + kz) * d->R + ky) * d->S + kx;
                    if (!bwd) value = value + x[xi] * w[wi]; /* conv3d_op.mojo:196-236 */
                    if (dx) dx[xi] = dx[xi] + g * w[wi];
                    if (dw) dw[wi] = dw[wi] + g * x[xi];
                  }
                }
              }
            if (!bwd) y[oi] = value + (bias ? bias[k] : 0.f); /* conv3d_op.mojo:238-240 */
          }
}

/* ---- optimizers ------------------------------------------------------------------------------
 * SGD plain path: p -= lr * g (optim/sgd.mojo:61-62). Adam: optim/adam.mojo:47-65, one fp32 Array op
 * at a time. Scalars are fp32 (adam.mojo:19-23); t starts at 1 and is incremented by the caller. */
void ref_sgd(int64_t n, float* p, const float* g, float lr) {
  for (int64_t i = 0; i < n; ++i) {
    float u = lr * g[i];
    p[i] = p[i] - u;
  }
}

void ref_adam(int64_t n, float* p, const float* g, float* m, float* v, float lr, float b1, float b2, float eps, float t) {
  float omb1 = 1.f - b1, omb2 = 1.f - b2;
  float c1 = 1.f - powf(b1, t), c2 = 1.f - powf(b2, t);
  for (int64_t i = 0; i < n; ++i) {
    float a = b1 * m[i], b = omb1 * g[i];
    m[i] = a + b;
    float c = b2 * v[i], e = omb2 * g[i];
    e = e * g[i];
    v[i] = c + e;
    float mh = m[i] / c1, vh = v[i] / c2;
    float num = lr * mh;
    float den = unary_real(OP_SQRT, vh) + eps;
    float q = num / den;
    p[i] = p[i] - q;
  }
}

/* SGD with momentum / weight decay (optim/sgd.mojo:42-60), Adagrad (optim/adagrad.mojo:36-45), RMSprop
 * (optim/rmsprop.mojo:39-53), one fp32 Array op at a time. vel may be NULL when momentum == 0. */
void ref_sgd_momentum(int64_t n, float* p, const float* g, float* vel, float lr, float momentum, float wd) {
  for (int64_t i = 0; i < n; ++i) {
    float c = g[i];
    if (wd > 0.f) { float w = wd * p[i]; c = g[i] + w; }
    float d = lr * c;
    if (momentum > 0.f) {
      float m = momentum * vel[i];
      vel[i] = m - d;
      p[i] = p[i] + vel[i];
    } else {
      p[i] = p[i] - d;
    }
  }
}

void ref_adagrad(int64_t n, float* p, const float* g, float* cache, float lr, float eps) {
  for (int64_t i = 0; i < n; ++i) {
    float gg = g[i] * g[i];
    cache[i] = cache[i] + gg;
    float num = lr * g[i];
    float den = unary_real(OP_SQRT, cache[i]) + eps;
    float q = num / den;
    p[i] = p[i] - q;
  }
}

void ref_rmsprop(int64_t n, float* p, const float* g, float* cache, float lr, float alpha, float eps) {
  float oma = 1.f - alpha;
  for (int64_t i = 0; i < n; ++i) {
    float x = alpha * cache[i], y = oma * g[i];
    y = y * g[i];
    cache[i] = x + y;
    float num = lr * g[i];
    float den = unary_real(OP_SQRT, cache[i]) + eps;
    float q = num / den;
    p[i] = p[i] - q;
  }
}

/* ---- one imperative training step: benchmarks/mlp_benchmarks/mlp_imp.mojo:47-75 -----------------
 * forward (nn/modules/_mlp.mojo:47-53): pred = act(pred @ W_i + b_i), no activation after the last layer;
 * loss = mse(pred, y); backward in jacrev order (autograd/functional.mojo:40-65); optimizer step.
 * W_i is [widths[i], widths[i+1]], b_i [widths[i+1]]. opt: 0 = none, 1 = SGD, 2 = Adam.
 * Gradients are written to dW[i], db[i] (caller-allocated). Returns the loss. */
float ref_mlp_step(int32_t L, const int64_t* widths, int64_t batch, int32_t act, const float* x, const float* target,
                   float** W, float** b, float** dW, float** db, int32_t opt, float lr, float b1, float b2, float eps,
                   float t, float** mW, float** vW, float** mb, float** vb) {
  float** Z = (float**)calloc((size_t)L, sizeof(float*));
  float** A = (float**)calloc((size_t)L + 1, sizeof(float*));
  A[0] = (float*)x;
  for (int l = 0; l < L; ++l) {
    int64_t K = widths[l], N = widths[l + 1];
    float* mm = fresh(batch * N);
    ref_matmul(1, batch, N, K, A[l], 0, K, 1, W[l], 0, N, 1, mm);
    Z[l] = fresh(batch * N);
    int64_t shape[2] = {batch, N}, fs[2] = {N, 1}, bs[2] = {0, 1};
    ref_binary(BIN_ADD, 2, shape, fs, bs, mm, b[l], Z[l], 0);
    free(mm);
    if (l < L - 1) {
      A[l + 1] = fresh(batch * N);
      ref_unary(act, batch * N, Z[l], A[l + 1]);
    } else {
      A[l + 1] = Z[l];
    }
  }
  int64_t n_out = batch * widths[L];
  float loss = 0.f;
  float* delta = fresh(n_out);
  ref_mse(n_out, A[L], target, &loss, delta);
  for (int l = L - 1; l >= 0; --l) {
    int64_t K = widths[l], N = widths[l + 1];
    /* Expand.vjp: reduce_add over the broadcast axis (expand_op.mojo:121-126) -> db [1, N] */
    int64_t shape[2] = {batch, N};
    ref_reduce_add(2, shape, 1u, delta, db[l], 0);
    /* matmul_vjp (matmul_op.mojo:278-283): dW = A^T @ delta, dA = delta @ W^T (skipped for the input) */
    ref_matmul(1, K, N, batch, A[l], 0, 1, K, delta, 0, N, 1, dW[l]);
    if (l > 0) {
      float* dA = fresh(batch * K);
      ref_matmul(1, batch, K, N, delta, 0, N, 1, W[l], 0, 1, N, dA);
      float* nd = fresh(batch * K);
      ref_unary_vjp(act, batch * K, Z[l - 1], dA, nd);
      free(dA);
      free(delta);
      delta = nd;
    }
  }
  free(delta);
  for (int l = 0; l < L; ++l) {
    int64_t nW = widths[l] * widths[l + 1], nb = widths[l + 1];
    if (opt == 1) {
      ref_sgd(nW, W[l], dW[l], lr);
      ref_sgd(nb, b[l], db[l], lr);
    } else if (opt == 2) {
      ref_adam(nW, W[l], dW[l], mW[l], vW[l], lr, b1, b2, eps, t);
      ref_adam(nb, b[l], db[l], mb[l], vb[l], lr, b1, b2, eps, t);
    }
  }
  for (int l = 0; l < L; ++l) {
    free(Z[l]);
    if (l > 0 && l < L) free(A[l]);
  }
  free(Z);
  free(A);
  return loss;
}
