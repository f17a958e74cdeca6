// Device-side bodies of the elementwise ops: one definition shared by the single-op streaming
// kernels (where `op` is a template constant and the switch folds away) and by the fused
// elementwise program kernel (where `op` is wave-uniform and the switch is a scalar branch).
// The real forms are the reference's complex SIMD bodies evaluated at imag = 0
// (execute_unary_op, endia/functional/unary_ops/_utils.mojo:77-134).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/endia_hip.h"

namespace endia {

__device__ __forceinline__ float unary_real(int op, float x) {
  switch (op) {
    case ENDIA_OP_RELU: return x > 0.f ? x : 0.f;
    case ENDIA_OP_TANH: return tanhf(x);
    case ENDIA_OP_SIN: return sinf(x);
    case ENDIA_OP_COS: return cosf(x);
    case ENDIA_OP_NEG: return -x;
    case ENDIA_OP_SQUARE: return x * x;
    case ENDIA_OP_SQRT: return sqrtf((fabsf(x) + x) * 0.5f);  // 0 for negative x: sqrt_op.mojo:111-114
    case ENDIA_OP_ABS: return fabsf(x);
    case ENDIA_OP_GREATER0: return x > 0.f ? 1.f : 0.f;
    case ENDIA_OP_EXP: return expf(x);                      // exp_op.mojo:113
    case ENDIA_OP_LOG: return logf(fabsf(x));               // log of the modulus: log_op.mojo:111-113
    case ENDIA_OP_SIGMOID: return 1.f / (1.f + expf(-x));   // sigmoid_op.mojo:120
    case ENDIA_OP_SINH: return sinhf(x);                    // sinh_op.mojo:108
    case ENDIA_OP_COSH: return coshf(x);                    // cosh_op.mojo:109
    case ENDIA_OP_TAN: return tanf(x);                      // tan_op.mojo
    case ENDIA_OP_ASIN: return asinf(x);                    // asin_op.mojo:103
    case ENDIA_OP_ACOS: return acosf(x);                    // acos_op.mojo:111
    case ENDIA_OP_ATAN: return atanf(x);                    // atan_op.mojo:105
    case ENDIA_OP_RECIPROCAL: return x / (x * x);           // reciprocal_op.mojo:115-116
    case ENDIA_OP_SIGN: return x / fabsf(x);                // sign_op.mojo:78-79 (NaN at 0)
    default: return x;
  }
}

// g * d(op)/dx at x: the reference's VJP rule of each op collapsed into one expression
__device__ __forceinline__ float unary_vjp_real(int op, float x, float g) {
  switch (op) {
    case ENDIA_OP_RELU: return x > 0.f ? g : 0.f;
    case ENDIA_OP_TANH: { float t = tanhf(x); return (1.f - t * t) * g; }
    case ENDIA_OP_SIN: return cosf(x) * g;
    case ENDIA_OP_COS: return -sinf(x) * g;
    case ENDIA_OP_NEG: return -g;
    case ENDIA_OP_SQUARE: return 2.f * x * g;
    case ENDIA_OP_SQRT: return g / (2.f * sqrtf((fabsf(x) + x) * 0.5f));
    case ENDIA_OP_ABS: return (x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f)) * g;
    case ENDIA_OP_GREATER0: return 0.f;
    case ENDIA_OP_EXP: return expf(x) * g;                                   // exp_op.mojo:92
    case ENDIA_OP_LOG: return g / x;                                         // log_op.mojo:91
    case ENDIA_OP_SIGMOID: { float s = 1.f / (1.f + expf(-x)); return s * (1.f - s) * g; }  // sigmoid_op.mojo:98
    case ENDIA_OP_SINH: return coshf(x) * g;                                 // sinh_op.mojo:88
    case ENDIA_OP_COSH: return sinhf(x) * g;                                 // cosh_op.mojo:89
    case ENDIA_OP_TAN: { float t = tanf(x); return g * (1.f + t * t); }      // tan_op.mojo:81
    case ENDIA_OP_ASIN: return g / sqrtf(1.f - x * x);                       // asin_op.mojo:83
    case ENDIA_OP_ACOS: return -1.f / sqrtf(1.f - x * x) * g;                // acos_op.mojo:91
    case ENDIA_OP_ATAN: return g / (1.f + x * x);                            // atan_op.mojo:85
    case ENDIA_OP_RECIPROCAL: return -g / (x * x);                           // reciprocal_op.mojo:95
    default: return g;  // identity, and sign (default_vjp passes the gradient on: _array.mojo:43-47)
  }
}

// g * d(op)/dx from the op's OUTPUT y, for the ops whose derivative is a function of y
__host__ __device__ constexpr bool unary_has_output_rule(int op) {
  return op == ENDIA_OP_RELU || op == ENDIA_OP_TANH || op == ENDIA_OP_SQRT || op == ENDIA_OP_IDENTITY ||
         op == ENDIA_OP_EXP || op == ENDIA_OP_SIGMOID || op == ENDIA_OP_TAN;
}

__device__ __forceinline__ float unary_vjp_from_output(int op, float y, float g) {
  switch (op) {
    case ENDIA_OP_RELU: return y > 0.f ? g : 0.f;
    case ENDIA_OP_TANH: return (1.f - y * y) * g;
    case ENDIA_OP_SQRT: return g / (2.f * y);
    case ENDIA_OP_EXP: return y * g;
    case ENDIA_OP_SIGMOID: return y * (1.f - y) * g;
    case ENDIA_OP_TAN: return g * (1.f + y * y);
    default: return g;
  }
}

__device__ __forceinline__ float bin_real(int op, float a, float b) {
  switch (op) {
    case ENDIA_BIN_ADD: return a + b;
    case ENDIA_BIN_SUB: return a - b;
    case ENDIA_BIN_MUL: return a * b;
    case ENDIA_BIN_DIV: return a / b;
    case ENDIA_BIN_GREATER: return a > b ? 1.f : 0.f;
    case ENDIA_BIN_POW: {  // |a|^b * cos(arg(a) * b): pow_op.mojo:139-146 with zero imaginary parts
      float u = expf(logf(fabsf(a)) * b);
      return a < 0.f ? u * cosf(3.14159265358979323846f * b) : u;
    }
    case ENDIA_BIN_GREATER_EQUAL: return a >= b ? 1.f : 0.f;
    case ENDIA_BIN_LESS: return a < b ? 1.f : 0.f;
    case ENDIA_BIN_LESS_EQUAL: return a <= b ? 1.f : 0.f;
    case ENDIA_BIN_EQUAL: return a == b ? 1.f : 0.f;
    case ENDIA_BIN_NOT_EQUAL: return a != b ? 1.f : 0.f;
    default: return a;
  }
}

__host__ __device__ constexpr bool unary_has_complex_form(int op) {
  switch (op) {
    case ENDIA_OP_NEG: case ENDIA_OP_SQUARE: case ENDIA_OP_ABS: case ENDIA_OP_IDENTITY: case ENDIA_OP_SIN:
    case ENDIA_OP_COS: case ENDIA_OP_TANH: case ENDIA_OP_EXP: case ENDIA_OP_LOG: case ENDIA_OP_SINH:
    case ENDIA_OP_COSH: case ENDIA_OP_SQRT: case ENDIA_OP_RECIPROCAL: case ENDIA_OP_SIGN:
      return true;
    default: return false;
  }
}

// complex -> complex bodies (|z| is handled by its own kernel since it returns a real array)
__device__ __forceinline__ float2 unary_complex(int op, float2 z) {
  switch (op) {
    case ENDIA_OP_NEG: return make_float2(-z.x, -z.y);
    case ENDIA_OP_SQUARE: return make_float2(z.x * z.x - z.y * z.y, 2.f * z.x * z.y);
    case ENDIA_OP_SIN: return make_float2(sinf(z.x) * coshf(z.y), cosf(z.x) * sinhf(z.y));     // sin_op.mojo:112-113
    case ENDIA_OP_COS: return make_float2(cosf(z.x) * coshf(z.y), -sinf(z.x) * sinhf(z.y));    // cos_op.mojo:113-114
    case ENDIA_OP_TANH: {                                                                       // tanh_op.mojo:112-115
      float d = coshf(2.f * z.x) + cosf(2.f * z.y);
      return make_float2(sinhf(2.f * z.x) / d, sinf(2.f * z.y) / d);
    }
    case ENDIA_OP_EXP: { float e = expf(z.x); return make_float2(e * cosf(z.y), e * sinf(z.y)); }  // exp_op.mojo:113-114
    case ENDIA_OP_LOG: return make_float2(logf(sqrtf(z.x * z.x + z.y * z.y)), atan2f(z.y, z.x));   // log_op.mojo:111-114
    case ENDIA_OP_SINH: return make_float2(sinhf(z.x) * cosf(z.y), coshf(z.x) * sinf(z.y));        // sinh_op.mojo:108-109
    case ENDIA_OP_COSH: return make_float2(coshf(z.x) * cosf(z.y), sinhf(z.x) * sinf(z.y));        // cosh_op.mojo:109-110
    case ENDIA_OP_SQRT: {                                                                           // sqrt_op.mojo:111-113
      float r = sqrtf(z.x * z.x + z.y * z.y);
      return make_float2(sqrtf((r + z.x) * 0.5f), copysignf(sqrtf((r - z.x) * 0.5f), z.y));
    }
    case ENDIA_OP_RECIPROCAL: { float d = z.x * z.x + z.y * z.y; return make_float2(z.x / d, -z.y / d); }  // reciprocal_op.mojo:115-117
    case ENDIA_OP_SIGN: { float r = sqrtf(z.x * z.x + z.y * z.y); return make_float2(z.x / r, z.y / r); }  // sign_op.mojo:78-80
    default: return z;
  }
}

__host__ __device__ constexpr bool binary_has_complex_form(int op) { return op <= ENDIA_BIN_DIV || op == ENDIA_BIN_POW; }

__device__ __forceinline__ float2 bin_complex(int op, float2 a, float2 b) {
  switch (op) {
    case ENDIA_BIN_ADD: return make_float2(a.x + b.x, a.y + b.y);
    case ENDIA_BIN_SUB: return make_float2(a.x - b.x, a.y - b.y);
    case ENDIA_BIN_MUL: return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);  // mul_op.mojo:152-155
    case ENDIA_BIN_POW: {  // pow_op.mojo:139-146
      float log_mag = logf(sqrtf(a.x * a.x + a.y * a.y));
      float arg = atan2f(a.y, a.x);
      float u = expf(log_mag * b.x - arg * b.y);
      float v = log_mag * b.y + arg * b.x;
      return make_float2(u * cosf(v), u * sinf(v));
    }
    default: {  // div_op.mojo:117-142
      float d = b.x * b.x + b.y * b.y;
      return make_float2((a.x * b.x + a.y * b.y) / d, (a.y * b.x - a.x * b.y) / d);
    }
  }
}

}  // namespace endia
