// Streaming (HBM-bound) kernels: fills, unary forward / VJP, broadcasting binary ops, axpby and the
// strided gather copy. Each replaces a run of full-tensor passes in the reference
// (execute_unary_op, endia/functional/unary_ops/_utils.mojo:77-134; execute_binary_op,
// endia/functional/binary_ops/_utils.mojo:93-177; execute_copy_raw, endia/functional/_utils.mojo:79-163)
// with ONE coalesced pass: every lane moves 16 bytes per access, a wave covers 1 KiB of
// consecutive addresses, and the grid is a few work-groups per CU walking the tensor with a
// grid stride.
#include "common.h"
#include "ew_ops.h"

#include <utility>

namespace {

using endia::bin_complex;
using endia::bin_real;
using endia::unary_complex;
using endia::unary_real;
using endia::unary_vjp_real;

constexpr int TPB = 256;

inline int stream_grid(int64_t nvec) {
  int64_t blocks = ceil_div64(nvec, TPB);
  int64_t cap = (int64_t)endia::ctx().cu_count * 8;
  if (cap < 256) cap = 2048;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- fill -----------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void fill_kernel(float* __restrict__ p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  int64_t n4 = n >> 2;
  float4 v4 = make_float4(v, v, v, v);
  float4* p4 = reinterpret_cast<float4*>(p);
  for (int64_t j = i; j < n4; j += stride) p4[j] = v4;
  for (int64_t j = (n4 << 2) + i; j < n; j += stride) p[j] = v;
}

__global__ __launch_bounds__(TPB) void fill_scalar_kernel(float* __restrict__ p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += stride) p[j] = v;
}

// ---- unary ----------------------------------------------------------------------------------
template <int OP, bool VEC>
__global__ __launch_bounds__(TPB) void unary_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  if (VEC) {
    int64_t n4 = n >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    float4* y4 = reinterpret_cast<float4*>(y);
    for (int64_t j = i; j < n4; j += stride) {
      float4 a = x4[j];
      y4[j] = make_float4(unary_real(OP, a.x), unary_real(OP, a.y), unary_real(OP, a.z), unary_real(OP, a.w));
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) y[j] = unary_real(OP, x[j]);
  } else {
    for (int64_t j = i; j < n; j += stride) y[j] = unary_real(OP, x[j]);
  }
}

template <int OP, bool VEC>
__global__ __launch_bounds__(TPB) void unary_vjp_kernel(const float* __restrict__ x, const float* __restrict__ g,
                                                        float* __restrict__ dx, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  if (VEC) {
    int64_t n4 = n >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    float4* d4 = reinterpret_cast<float4*>(dx);
    for (int64_t j = i; j < n4; j += stride) {
      float4 a = x4[j], b = g4[j];
      d4[j] = make_float4(unary_vjp_real(OP, a.x, b.x), unary_vjp_real(OP, a.y, b.y),
                          unary_vjp_real(OP, a.z, b.z), unary_vjp_real(OP, a.w, b.w));
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) dx[j] = unary_vjp_real(OP, x[j], g[j]);
  } else {
    for (int64_t j = i; j < n; j += stride) dx[j] = unary_vjp_real(OP, x[j], g[j]);
  }
}

__global__ __launch_bounds__(TPB) void vjp_from_output_kernel(int op, const float* __restrict__ y,
                                                              const float* __restrict__ g, float* __restrict__ dx,
                                                              int64_t n) {
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride)
    dx[j] = endia::unary_vjp_from_output(op, y[j], g[j]);
}

// complex forward: one complex element (8 bytes) per lane access
__global__ __launch_bounds__(TPB) void unary_fwd_complex_kernel(int op, const float2* __restrict__ x,
                                                                float* __restrict__ y, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  float2* y2 = reinterpret_cast<float2*>(y);
  for (int64_t j = i; j < n; j += stride) {
    float2 z = x[j];
    if (op == ENDIA_OP_ABS) y[j] = sqrtf(z.x * z.x + z.y * z.y);
    else y2[j] = unary_complex(op, z);
  }
}

// complex VJPs under the reference's rules (no conjugation: mul_op.mojo:125-128)
__global__ __launch_bounds__(TPB) void unary_vjp_complex_kernel(int op, const float2* __restrict__ x,
                                                                const float* __restrict__ g,
                                                                float2* __restrict__ dx, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  const float2* g2 = reinterpret_cast<const float2*>(g);
  for (int64_t j = i; j < n; j += stride) {
    float2 z = x[j];
    switch (op) {
      case ENDIA_OP_NEG: { float2 c = g2[j]; dx[j] = make_float2(-c.x, -c.y); break; }
      case ENDIA_OP_SQUARE: {  // 2 * z * g, square_op.mojo:96
        float2 c = g2[j];
        dx[j] = make_float2(2.f * (z.x * c.x - z.y * c.y), 2.f * (z.x * c.y + z.y * c.x));
        break;
      }
      case ENDIA_OP_ABS: {  // sign(z) * g with real g: abs_op.mojo:93, sign_op.mojo:78-81, real_op.mojo:74-77
        float r = sqrtf(z.x * z.x + z.y * z.y);
        float c = g[j];
        dx[j] = make_float2(z.x / r * c, z.y / r * c);
        break;
      }
      default: dx[j] = g2[j]; break;
    }
  }
}

// ---- binary with broadcast -------------------------------------------------------------------
struct BinDesc {
  int ndim;
  int64_t shape[8];
  int64_t as[8];
  int64_t bs[8];
};

// Same-shape contiguous operands.
template <int OP>
__global__ __launch_bounds__(TPB) void bin_flat_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                       float* __restrict__ o, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  int64_t n4 = n >> 2;
  const float4* a4 = reinterpret_cast<const float4*>(a);
  const float4* b4 = reinterpret_cast<const float4*>(b);
  float4* o4 = reinterpret_cast<float4*>(o);
  for (int64_t j = i; j < n4; j += stride) {
    float4 x = a4[j], y = b4[j];
    o4[j] = make_float4(bin_real(OP, x.x, y.x), bin_real(OP, x.y, y.y), bin_real(OP, x.z, y.z), bin_real(OP, x.w, y.w));
  }
  for (int64_t j = (n4 << 2) + i; j < n; j += stride) o[j] = bin_real(OP, a[j], b[j]);
}

// [rows, cols] op with one operand a row vector [cols] (bias add and friends) or a scalar.
// amode/bmode: 0 = full, 1 = row vector (index = col), 2 = scalar (index 0).
template <int OP>
__global__ __launch_bounds__(TPB) void bin_rowvec_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         float* __restrict__ o, int64_t n, int64_t cols,
                                                         int amode, int bmode) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += stride) {
    int64_t c = j % cols;
    float x = a[amode == 0 ? j : (amode == 1 ? c : 0)];
    float y = b[bmode == 0 ? j : (bmode == 1 ? c : 0)];
    o[j] = bin_real(OP, x, y);
  }
}

template <int OP, bool CPLX>
__global__ __launch_bounds__(TPB) void bin_general_kernel(BinDesc d, const float* __restrict__ a,
                                                          const float* __restrict__ b, float* __restrict__ o,
                                                          int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += stride) {
    int64_t r = j, ia = 0, ib = 0;
    for (int k = d.ndim - 1; k >= 0; --k) {
      int64_t q = r / d.shape[k];
      int64_t c = r - q * d.shape[k];
      ia += c * d.as[k];
      ib += c * d.bs[k];
      r = q;
    }
    if (CPLX) {
      float2 x = reinterpret_cast<const float2*>(a)[ia];
      float2 y = reinterpret_cast<const float2*>(b)[ib];
      reinterpret_cast<float2*>(o)[j] = bin_complex(OP, x, y);
    } else {
      o[j] = bin_real(OP, a[ia], b[ib]);
    }
  }
}

// 2-D op where one operand is a transposed view (element strides (1, ld)) and the other is
// contiguous: the transposed operand goes through a 32 x 32 LDS tile so that its reads, the other
// operand's reads and the writes all run along contiguous memory. (This is the shape of x + y.T(),
// which a second backward pass produces whenever a weight is used through its transposed view.)
template <int OP>
__global__ __launch_bounds__(256) void bin_transposed_kernel(const float* __restrict__ full, const float* __restrict__ tr,
                                                            float* __restrict__ o, int64_t rows, int64_t cols,
                                                            int64_t ld_tr, int tr_is_lhs) {
  __shared__ float t[32][33];
  const int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int k = ty; k < 32; k += 8) {  // tr[(r, c)] lives at c * ld_tr + r: walk r fastest
    int64_t c = c0 + k, r = r0 + tx;
    t[k][tx] = (c < cols && r < rows) ? tr[c * ld_tr + r] : 0.f;
  }
  __syncthreads();
  for (int k = ty; k < 32; k += 8) {
    int64_t r = r0 + k, c = c0 + tx;
    if (r < rows && c < cols) {
      float x = full[r * cols + c], y = t[tx][k];
      o[r * cols + c] = tr_is_lhs ? bin_real(OP, y, x) : bin_real(OP, x, y);
    }
  }
}

__global__ __launch_bounds__(TPB) void axpby_kernel(int64_t n, float alpha, const float* __restrict__ a, float beta,
                                                    const float* __restrict__ b, float* __restrict__ o, int vec) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  if (vec) {
    int64_t n4 = n >> 2;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* b4 = reinterpret_cast<const float4*>(b);
    float4* o4 = reinterpret_cast<float4*>(o);
    for (int64_t j = i; j < n4; j += stride) {
      float4 x = a4[j];
      float4 r = make_float4(alpha * x.x, alpha * x.y, alpha * x.z, alpha * x.w);
      if (b) {
        float4 y = b4[j];
        r.x += beta * y.x; r.y += beta * y.y; r.z += beta * y.z; r.w += beta * y.w;
      }
      o4[j] = r;
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) o[j] = alpha * a[j] + (b ? beta * b[j] : 0.f);
  } else {
    for (int64_t j = i; j < n; j += stride) o[j] = alpha * a[j] + (b ? beta * b[j] : 0.f);
  }
}

__global__ __launch_bounds__(TPB) void complex_pack_kernel(int64_t n, const float* __restrict__ re,
                                                           const float* __restrict__ im, float2* __restrict__ out) {
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride)
    out[j] = make_float2(re[j], im ? im[j] : 0.f);
}

// ---- strided gather copy ---------------------------------------------------------------------
struct CopyDesc {
  int ndim;
  int64_t shape[8];
  int64_t st[8];
  int64_t offset;
};

template <bool CPLX>
__global__ __launch_bounds__(TPB) void strided_copy_kernel(CopyDesc d, const float* __restrict__ src,
                                                           float* __restrict__ dst, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += stride) {
    int64_t r = j, is = d.offset;
    for (int k = d.ndim - 1; k >= 0; --k) {
      int64_t q = r / d.shape[k];
      is += (r - q * d.shape[k]) * d.st[k];
      r = q;
    }
    if (CPLX) reinterpret_cast<float2*>(dst)[j] = reinterpret_cast<const float2*>(src)[is];
    else dst[j] = src[is];
  }
}

// The store side of a view: dst[offset + sum i_k * stride_k] (=, +=) src[j] for the row-major index j. With
// ACC the view's elements may alias (overlapping windows of an as_strided view), so the add is atomic.
template <bool CPLX, bool ACC>
__global__ __launch_bounds__(TPB) void strided_scatter_kernel(CopyDesc d, const float* __restrict__ src,
                                                              float* __restrict__ dst, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += stride) {
    int64_t r = j, id = d.offset;
    for (int k = d.ndim - 1; k >= 0; --k) {
      int64_t q = r / d.shape[k];
      id += (r - q * d.shape[k]) * d.st[k];
      r = q;
    }
    if (CPLX) {
      const float2 v = reinterpret_cast<const float2*>(src)[j];
      if (ACC) {
        atomicAdd(&dst[2 * id], v.x);
        atomicAdd(&dst[2 * id + 1], v.y);
      } else {
        reinterpret_cast<float2*>(dst)[id] = v;
      }
    } else {
      if (ACC) atomicAdd(&dst[id], src[j]);
      else dst[id] = src[j];
    }
  }
}

// 2-D transpose through LDS: dst[r][c] = src[c*ld + r]; both sides coalesced.
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                        int64_t rows, int64_t cols, int64_t ld, int64_t off) {
  __shared__ float t[32][33];
  int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
  int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int k = ty; k < 32; k += 8) {
    int64_t c = c0 + k, r = r0 + tx;  // read src row c (contiguous in r)
    t[k][tx] = (c < cols && r < rows) ? src[off + c * ld + r] : 0.f;
  }
  __syncthreads();
  for (int k = ty; k < 32; k += 8) {
    int64_t r = r0 + k, c = c0 + tx;
    if (r < rows && c < cols) dst[r * cols + c] = t[tx][k];
  }
}

template <int... I, typename F>
bool dispatch_seq(int op, std::integer_sequence<int, I...>, F&& f) {
  return ((op == I ? (f(std::integral_constant<int, I>()), true) : false) || ...);
}

template <typename F>
int32_t dispatch_unary(int op, F&& f) {
  return dispatch_seq(op, std::make_integer_sequence<int, ENDIA_OP_COUNT>(), f) ? 0 : -1;
}

template <typename F>
int32_t dispatch_binary(int op, F&& f) {
  return dispatch_seq(op, std::make_integer_sequence<int, ENDIA_BIN_COUNT>(), f) ? 0 : -1;
}

}  // namespace

using namespace endia;

extern "C" {

int32_t endia_hip_fill(float* p, int64_t n, float value) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_fill: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(p != nullptr, "endia_hip_fill: null pointer");
  if (al16(p))
    hipLaunchKernelGGL(fill_kernel, dim3(stream_grid((n + 3) / 4)), dim3(TPB), 0, ctx().stream, p, n, value);
  else
    hipLaunchKernelGGL(fill_scalar_kernel, dim3(stream_grid(n)), dim3(TPB), 0, ctx().stream, p, n, value);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

// A fill kernel rather than hipMemsetAsync, so that a caller may record it into a HIP graph.
int32_t endia_hip_memset0(void* p, int64_t bytes) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(bytes >= 0 && bytes % 4 == 0, "endia_hip_memset0: size %lld is not a multiple of 4", (long long)bytes);
  return endia_hip_fill(static_cast<float*>(p), bytes / 4, 0.f);
}

int32_t endia_hip_unary_fwd(int32_t op, int64_t n, const float* x, float* y, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_unary_fwd: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && y, "endia_hip_unary_fwd: null pointer");
  hipStream_t s = ctx().stream;
  if (is_complex) {
    ENDIA_CHECK_ARG(op >= 0 && op < ENDIA_OP_COUNT, "endia_hip_unary_fwd: unknown op %d", op);
    if (!endia::unary_has_complex_form(op))
      return fail(ENDIA_HIP_ERR_UNSUPPORTED, "endia_hip_unary_fwd: op %d has no complex form", op);
    hipLaunchKernelGGL(unary_fwd_complex_kernel, dim3(stream_grid(n)), dim3(TPB), 0, s, op,
                       reinterpret_cast<const float2*>(x), y, n);
  } else {
    bool vec = al16(x) && al16(y);
    int grid = stream_grid(vec ? (n + 3) / 4 : n);
    int rc = dispatch_unary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      if (vec) hipLaunchKernelGGL((unary_fwd_kernel<OP, true>), dim3(grid), dim3(TPB), 0, s, x, y, n);
      else hipLaunchKernelGGL((unary_fwd_kernel<OP, false>), dim3(grid), dim3(TPB), 0, s, x, y, n);
    });
    ENDIA_CHECK_ARG(rc == 0, "endia_hip_unary_fwd: unknown op %d", op);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_unary_vjp(int32_t op, int64_t n, const float* x, const float* g, float* dx, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_unary_vjp: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && g && dx, "endia_hip_unary_vjp: null pointer");
  hipStream_t s = ctx().stream;
  if (is_complex) {
    if (!(op == ENDIA_OP_NEG || op == ENDIA_OP_SQUARE || op == ENDIA_OP_ABS || op == ENDIA_OP_IDENTITY))
      return fail(ENDIA_HIP_ERR_UNSUPPORTED, "endia_hip_unary_vjp: op %d has no complex form here", op);
    hipLaunchKernelGGL(unary_vjp_complex_kernel, dim3(stream_grid(n)), dim3(TPB), 0, s, op,
                       reinterpret_cast<const float2*>(x), g, reinterpret_cast<float2*>(dx), n);
  } else {
    bool vec = al16(x) && al16(g) && al16(dx);
    int grid = stream_grid(vec ? (n + 3) / 4 : n);
    int rc = dispatch_unary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      if (vec) hipLaunchKernelGGL((unary_vjp_kernel<OP, true>), dim3(grid), dim3(TPB), 0, s, x, g, dx, n);
      else hipLaunchKernelGGL((unary_vjp_kernel<OP, false>), dim3(grid), dim3(TPB), 0, s, x, g, dx, n);
    });
    ENDIA_CHECK_ARG(rc == 0, "endia_hip_unary_vjp: unknown op %d", op);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_unary_vjp_from_output(int32_t op, int64_t n, const float* y, const float* g, float* dx) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_unary_vjp_from_output: negative n");
  ENDIA_CHECK_ARG(endia::unary_has_output_rule(op),
                  "endia_hip_unary_vjp_from_output: op %d cannot be differentiated from its output", op);
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(y && g && dx, "endia_hip_unary_vjp_from_output: null pointer");
  hipLaunchKernelGGL(vjp_from_output_kernel, dim3(stream_grid(n)), dim3(TPB), 0, ctx().stream, op, y, g, dx, n);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_binary(int32_t op, int32_t ndim, const int64_t* shape, const int64_t* a_strides,
                         const int64_t* b_strides, const float* a, const float* b, float* out, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(ndim >= 0 && ndim <= 8, "endia_hip_binary: ndim %d out of [0,8]", ndim);
  ENDIA_CHECK_ARG(ndim == 0 || (shape && a_strides && b_strides), "endia_hip_binary: null descriptor");
  ENDIA_CHECK_ARG(op >= 0 && op < ENDIA_BIN_COUNT, "endia_hip_binary: unknown op %d", op);
  ENDIA_CHECK_ARG(!(is_complex && !endia::binary_has_complex_form(op)), "endia_hip_binary: comparisons are real only (op %d)", op);
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    ENDIA_CHECK_ARG(shape[i] >= 0 && a_strides[i] >= 0 && b_strides[i] >= 0, "endia_hip_binary: negative extent or stride");
    n *= shape[i];
  }
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(a && b && out, "endia_hip_binary: null pointer");
  hipStream_t s = ctx().stream;

  // classify each operand: contiguous-full, row vector along the last axis, scalar, or general
  auto classify = [&](const int64_t* st) {
    bool full = true, rowvec = ndim >= 1, scalar = true;
    int64_t expect = 1;
    for (int i = ndim - 1; i >= 0; --i) {
      if (shape[i] != 1) {
        if (st[i] != expect) full = false;
        if (st[i] != 0) scalar = false;
        if (i == ndim - 1) { if (st[i] != 1) rowvec = false; }
        else if (st[i] != 0) rowvec = false;
      }
      expect *= shape[i];
    }
    return full ? 0 : (scalar ? 2 : (rowvec ? 1 : 3));
  };
  int am = classify(a_strides), bm = classify(b_strides);
  int rc = 0;
  // [R, C] with one operand contiguous and the other a transposed view
  auto transposed = [&](const int64_t* st) {
    return ndim == 2 && shape[0] > 1 && shape[1] > 1 && st[0] == 1 && st[1] >= shape[0];
  };
  if (!is_complex && ndim == 2 && ((am == 0 && transposed(b_strides)) || (bm == 0 && transposed(a_strides))) &&
      ceil_div64(shape[0], 32) <= 65535) {
    const bool tr_is_lhs = am != 0;
    const float* full = tr_is_lhs ? b : a;
    const float* tr = tr_is_lhs ? a : b;
    const int64_t ld = tr_is_lhs ? a_strides[1] : b_strides[1];
    dim3 grid((unsigned)ceil_div64(shape[1], 32), (unsigned)ceil_div64(shape[0], 32));
    rc = dispatch_binary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      hipLaunchKernelGGL((bin_transposed_kernel<OP>), grid, dim3(256), 0, s, full, tr, out, shape[0], shape[1], ld,
                         tr_is_lhs ? 1 : 0);
    });
  } else if (!is_complex && am == 0 && bm == 0 && al16(a) && al16(b) && al16(out)) {
    rc = dispatch_binary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      hipLaunchKernelGGL((bin_flat_kernel<OP>), dim3(stream_grid((n + 3) / 4)), dim3(TPB), 0, s, a, b, out, n);
    });
  } else if (!is_complex && am != 3 && bm != 3) {
    int64_t cols = ndim ? shape[ndim - 1] : 1;
    rc = dispatch_binary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      hipLaunchKernelGGL((bin_rowvec_kernel<OP>), dim3(stream_grid(n)), dim3(TPB), 0, s, a, b, out, n, cols, am, bm);
    });
  } else {
    BinDesc d;
    d.ndim = ndim;
    for (int i = 0; i < 8; ++i) {
      d.shape[i] = i < ndim ? shape[i] : 1;
      d.as[i] = i < ndim ? a_strides[i] : 0;
      d.bs[i] = i < ndim ? b_strides[i] : 0;
    }
    rc = dispatch_binary(op, [&](auto tag) {
      constexpr int OP = decltype(tag)::value;
      if (is_complex) {
        if constexpr (endia::binary_has_complex_form(OP))
          hipLaunchKernelGGL((bin_general_kernel<OP, true>), dim3(stream_grid(n)), dim3(TPB), 0, s, d, a, b, out, n);
      } else {
        hipLaunchKernelGGL((bin_general_kernel<OP, false>), dim3(stream_grid(n)), dim3(TPB), 0, s, d, a, b, out, n);
      }
    });
  }
  ENDIA_CHECK_ARG(rc == 0, "endia_hip_binary: unknown op %d", op);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_axpby(int64_t n, float alpha, const float* a, float beta, const float* b, float* out) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_axpby: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(a && out, "endia_hip_axpby: null pointer");
  int vec = al16(a) && al16(out) && (!b || al16(b));
  hipLaunchKernelGGL(axpby_kernel, dim3(stream_grid(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, ctx().stream, n, alpha, a,
                     beta, b, out, vec);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_complex_pack(int64_t n, const float* re, const float* im, float* out) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_complex_pack: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(re && out, "endia_hip_complex_pack: null pointer");
  hipLaunchKernelGGL(complex_pack_kernel, dim3(stream_grid(n)), dim3(TPB), 0, ctx().stream, n, re, im,
                     reinterpret_cast<float2*>(out));
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_strided_copy(int32_t ndim, const int64_t* shape, const int64_t* src_strides, int64_t src_offset,
                               const float* src, float* dst, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(ndim >= 0 && ndim <= 8, "endia_hip_strided_copy: ndim %d out of [0,8]", ndim);
  ENDIA_CHECK_ARG(ndim == 0 || (shape && src_strides), "endia_hip_strided_copy: null descriptor");
  ENDIA_CHECK_ARG(src_offset >= 0, "endia_hip_strided_copy: negative offset");
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    ENDIA_CHECK_ARG(shape[i] >= 0 && src_strides[i] >= 0, "endia_hip_strided_copy: negative extent or stride");
    n *= shape[i];
  }
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(src && dst, "endia_hip_strided_copy: null pointer");
  hipStream_t s = ctx().stream;
  // plain 2-D transpose (the .T() of a contiguous matrix) goes through LDS so both sides coalesce
  if (!is_complex && ndim == 2 && src_strides[0] == 1 && src_strides[1] >= shape[0] && shape[0] > 1 && shape[1] > 1) {
    dim3 grid((unsigned)ceil_div64(shape[1], 32), (unsigned)ceil_div64(shape[0], 32));
    if (grid.y <= 65535) {
      hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, s, src, dst, shape[0], shape[1], src_strides[1], src_offset);
      ENDIA_LAUNCH_CHECK();
      return ENDIA_HIP_OK;
    }
  }
  CopyDesc d;
  d.ndim = ndim;
  d.offset = src_offset;
  for (int i = 0; i < 8; ++i) {
    d.shape[i] = i < ndim ? shape[i] : 1;
    d.st[i] = i < ndim ? src_strides[i] : 0;
  }
  if (is_complex)
    hipLaunchKernelGGL((strided_copy_kernel<true>), dim3(stream_grid(n)), dim3(TPB), 0, s, d, src, dst, n);
  else
    hipLaunchKernelGGL((strided_copy_kernel<false>), dim3(stream_grid(n)), dim3(TPB), 0, s, d, src, dst, n);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_strided_scatter(int32_t ndim, const int64_t* shape, const int64_t* dst_strides, int64_t dst_offset,
                                  const float* src, float* dst, int32_t accumulate, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(ndim >= 0 && ndim <= 8, "endia_hip_strided_scatter: ndim %d out of [0,8]", ndim);
  ENDIA_CHECK_ARG(ndim == 0 || (shape && dst_strides), "endia_hip_strided_scatter: null descriptor");
  ENDIA_CHECK_ARG(dst_offset >= 0, "endia_hip_strided_scatter: negative offset");
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    ENDIA_CHECK_ARG(shape[i] >= 0 && dst_strides[i] >= 0, "endia_hip_strided_scatter: negative extent or stride");
    n *= shape[i];
  }
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(src && dst, "endia_hip_strided_scatter: null pointer");
  if (!accumulate) {
    // plain stores need a view whose elements are distinct: sorted by stride, every stride must step past
    // the whole extent of the axes below it
    int order[8], m = 0;
    for (int i = 0; i < ndim; ++i)
      if (shape[i] > 1) order[m++] = i;
    for (int a = 1; a < m; ++a)
      for (int b = a; b > 0 && dst_strides[order[b]] < dst_strides[order[b - 1]]; --b) {
        int t = order[b]; order[b] = order[b - 1]; order[b - 1] = t;
      }
    int64_t span = 0;  // largest offset reachable with the axes seen so far
    for (int a = 0; a < m; ++a) {
      ENDIA_CHECK_ARG(dst_strides[order[a]] > span, "endia_hip_strided_scatter: the view's elements overlap; pass accumulate = 1");
      span += (shape[order[a]] - 1) * dst_strides[order[a]];
    }
  }
  CopyDesc d;
  d.ndim = ndim;
  d.offset = dst_offset;
  for (int i = 0; i < 8; ++i) {
    d.shape[i] = i < ndim ? shape[i] : 1;
    d.st[i] = i < ndim ? dst_strides[i] : 0;
  }
  hipStream_t s = ctx().stream;
  const dim3 grid(stream_grid(n)), block(TPB);
  if (is_complex && accumulate) hipLaunchKernelGGL((strided_scatter_kernel<true, true>), grid, block, 0, s, d, src, dst, n);
  else if (is_complex) hipLaunchKernelGGL((strided_scatter_kernel<true, false>), grid, block, 0, s, d, src, dst, n);
  else if (accumulate) hipLaunchKernelGGL((strided_scatter_kernel<false, true>), grid, block, 0, s, d, src, dst, n);
  else hipLaunchKernelGGL((strided_scatter_kernel<false, false>), grid, block, 0, s, d, src, dst, n);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

}  // extern "C"
