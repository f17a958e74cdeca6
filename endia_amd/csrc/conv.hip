// conv2d (NCHW, cross-correlation, groups = 1): forward as in Conv2d.__call__
// (endia/functional/spacial_ops/conv2d_op.mojo:88-196; output shape rule conv2d_op.mojo:31-85) and the
// three adjoints of that loop. The reference registers no backward rule for conv2d
// (Conv2d.vjp = default_vjp, conv2d_op.mojo:198-200), so the gradients are defined here as
//   db[k]       = sum_{n,p,q} dy[n,k,p,q]
//   dw[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c, p*sh - ph + r*dh, q*sw - pw + s*dw]
//   dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * w[k,c,r,s]  over (p,q) with p*sh - ph + r*dh = h, q*sw - pw + s*dw = w
// with out-of-range taps contributing zero, exactly as the forward loop skips them.
#include "common.h"

namespace endia {
int32_t col_reduce(int64_t batch, int64_t R, int64_t C, const float* x, float* out, float scale);
int32_t row_reduce(int64_t R, int64_t C, const float* x, float* out, float scale);
}

namespace {

constexpr int TPB = 256;

struct ConvP {
  int N, C, H, W, K, R, S, P, Q;
  int sh, sw, ph, pw, dh, dw;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// one lane per output element; consecutive lanes walk q, so x reads and y writes coalesce
__global__ __launch_bounds__(TPB) void conv_fwd_direct_kernel(ConvP p, const float* __restrict__ x,
                                                              const float* __restrict__ w, const float* __restrict__ bias,
                                                              float* __restrict__ y, int relu) {
  int64_t total = (int64_t)p.N * p.K * p.P * p.Q;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t idx = (int64_t)blockIdx.x * TPB + threadIdx.x; idx < total; idx += stride) {
    int q = (int)(idx % p.Q);
    int64_t t = idx / p.Q;
    int pp = (int)(t % p.P);
    t /= p.P;
    int k = (int)(t % p.K);
    int n = (int)(t / p.K);
    float acc = 0.f;
    const int h0 = pp * p.sh - p.ph, w0 = q * p.sw - p.pw;
    for (int c = 0; c < p.C; ++c) {
      const float* xc = x + ((int64_t)n * p.C + c) * p.H * p.W;
      const float* wc = w + ((int64_t)k * p.C + c) * p.R * p.S;
      for (int r = 0; r < p.R; ++r) {
        int h = h0 + r * p.dh;
        if (h < 0 || h >= p.H) continue;
        for (int s = 0; s < p.S; ++s) {
          int ww = w0 + s * p.dw;
          if (ww < 0 || ww >= p.W) continue;
          acc = fmaf(xc[(int64_t)h * p.W + ww], wc[r * p.S + s], acc);
        }
      }
    }
    if (bias) acc += bias[k];
    if (relu) acc = acc > 0.f ? acc : 0.f;
    y[idx] = acc;
  }
}

// one lane per input element: gather form of the transposed convolution
__global__ __launch_bounds__(TPB) void conv_bwd_data_direct_kernel(ConvP p, const float* __restrict__ dy,
                                                                   const float* __restrict__ w, float* __restrict__ dx) {
  int64_t total = (int64_t)p.N * p.C * p.H * p.W;
  int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t idx = (int64_t)blockIdx.x * TPB + threadIdx.x; idx < total; idx += stride) {
    int ww = (int)(idx % p.W);
    int64_t t = idx / p.W;
    int h = (int)(t % p.H);
    t /= p.H;
    int c = (int)(t % p.C);
    int n = (int)(t / p.C);
    float acc = 0.f;
    for (int r = 0; r < p.R; ++r) {
      int hn = h + p.ph - r * p.dh;
      if (hn < 0 || hn % p.sh) continue;
      int pp = hn / p.sh;
      if (pp >= p.P) continue;
      for (int s = 0; s < p.S; ++s) {
        int wn = ww + p.pw - s * p.dw;
        if (wn < 0 || wn % p.sw) continue;
        int q = wn / p.sw;
        if (q >= p.Q) continue;
        const float* dyp = dy + ((int64_t)n * p.K * p.P + pp) * p.Q + q;
        const float* wp = w + ((int64_t)c * p.R + r) * p.S + s;
        for (int k = 0; k < p.K; ++k)
          acc = fmaf(dyp[(int64_t)k * p.P * p.Q], wp[(int64_t)k * p.C * p.R * p.S], acc);
      }
    }
    dx[idx] = acc;
  }
}

// one work-group per filter tap (k,c,r,s): lanes stride over (n,p,q)
__global__ __launch_bounds__(TPB) void conv_bwd_weight_direct_kernel(ConvP p, const float* __restrict__ x,
                                                                     const float* __restrict__ dy, float* __restrict__ dw) {
  __shared__ float red[4];
  int64_t tap = blockIdx.x;
  int s = (int)(tap % p.S);
  int64_t t = tap / p.S;
  int r = (int)(t % p.R);
  t /= p.R;
  int c = (int)(t % p.C);
  int k = (int)(t / p.C);
  const int64_t PQ = (int64_t)p.P * p.Q;
  const int64_t total = (int64_t)p.N * PQ;
  float acc = 0.f;
  for (int64_t j = threadIdx.x; j < total; j += TPB) {
    int n = (int)(j / PQ);
    int rem = (int)(j - (int64_t)n * PQ);
    int pp = rem / p.Q, q = rem - pp * p.Q;
    int h = pp * p.sh - p.ph + r * p.dh, ww = q * p.sw - p.pw + s * p.dw;
    if (h < 0 || h >= p.H || ww < 0 || ww >= p.W) continue;
    acc = fmaf(dy[((int64_t)n * p.K + k) * PQ + rem], x[(((int64_t)n * p.C + c) * p.H + h) * p.W + ww], acc);
  }
  acc = wave_sum(acc);
  int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (lane == 0) red[wv] = acc;
  __syncthreads();
  if (threadIdx.x == 0) dw[tap] = (red[0] + red[1]) + (red[2] + red[3]);
}

int32_t make_params(const endia_hip_conv2d_desc* d, ConvP& p) {
  if (!d) return endia::fail(ENDIA_HIP_ERR_INVALID, "conv2d: descriptor is null");
  if (d->N < 0 || d->C <= 0 || d->H <= 0 || d->W <= 0 || d->K <= 0 || d->R <= 0 || d->S <= 0)
    return endia::fail(ENDIA_HIP_ERR_INVALID, "conv2d: non-positive extent");
  if (d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0 || d->pad_h < 0 || d->pad_w < 0)
    return endia::fail(ENDIA_HIP_ERR_INVALID, "conv2d: bad stride, dilation or padding");
  if (d->groups != 1)
    return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "conv2d: groups = %lld; only groups = 1 is implemented", (long long)d->groups);
  int64_t P = (d->H + 2 * d->pad_h - d->dil_h * (d->R - 1) - 1) / d->stride_h + 1;
  int64_t Q = (d->W + 2 * d->pad_w - d->dil_w * (d->S - 1) - 1) / d->stride_w + 1;
  if (d->H + 2 * d->pad_h - d->dil_h * (d->R - 1) - 1 < 0 || d->W + 2 * d->pad_w - d->dil_w * (d->S - 1) - 1 < 0)
    return endia::fail(ENDIA_HIP_ERR_INVALID, "conv2d: kernel larger than padded input");
  const int64_t lim = 1ll << 31;
  if (d->N * d->C * d->H * d->W >= lim * 4 || d->N * d->K * P * Q >= lim * 4 || d->K * d->C * d->R * d->S >= lim)
    return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "conv2d: tensor too large");
  p.N = (int)d->N; p.C = (int)d->C; p.H = (int)d->H; p.W = (int)d->W; p.K = (int)d->K; p.R = (int)d->R; p.S = (int)d->S;
  p.P = (int)P; p.Q = (int)Q;
  p.sh = (int)d->stride_h; p.sw = (int)d->stride_w; p.ph = (int)d->pad_h; p.pw = (int)d->pad_w;
  p.dh = (int)d->dil_h; p.dw = (int)d->dil_w;
  return ENDIA_HIP_OK;
}

inline int grid_for(int64_t n) {
  int64_t b = ceil_div64(n, TPB), cap = (int64_t)endia::ctx().cu_count * 16;
  if (b > cap) b = cap;
  return (int)(b < 1 ? 1 : b);
}

}  // namespace

using namespace endia;

extern "C" {

int32_t endia_hip_conv2d_out_shape(const endia_hip_conv2d_desc* d, int64_t* P, int64_t* Q) {
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  ENDIA_CHECK_ARG(P && Q, "endia_hip_conv2d_out_shape: null output");
  *P = p.P;
  *Q = p.Q;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_conv2d_fwd(const endia_hip_conv2d_desc* d, const float* x, const float* w, const float* bias, float* y,
                             int32_t act) {
  ENDIA_REQUIRE_INIT();
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  ENDIA_CHECK_ARG(act == ENDIA_OP_IDENTITY || act == ENDIA_OP_RELU, "endia_hip_conv2d_fwd: activation must be identity or relu");
  int64_t total = (int64_t)p.N * p.K * p.P * p.Q;
  if (total == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && w && y, "endia_hip_conv2d_fwd: null pointer");
  hipLaunchKernelGGL(conv_fwd_direct_kernel, dim3(grid_for(total)), dim3(TPB), 0, ctx().stream, p, x, w, bias, y,
                     act == ENDIA_OP_RELU ? 1 : 0);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_conv2d_bwd_data(const endia_hip_conv2d_desc* d, const float* dy, const float* w, float* dx) {
  ENDIA_REQUIRE_INIT();
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  int64_t total = (int64_t)p.N * p.C * p.H * p.W;
  if (total == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(dy && w && dx, "endia_hip_conv2d_bwd_data: null pointer");
  hipLaunchKernelGGL(conv_bwd_data_direct_kernel, dim3(grid_for(total)), dim3(TPB), 0, ctx().stream, p, dy, w, dx);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_conv2d_bwd_weight(const endia_hip_conv2d_desc* d, const float* x, const float* dy, float* dw) {
  ENDIA_REQUIRE_INIT();
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  int64_t taps = (int64_t)p.K * p.C * p.R * p.S;
  ENDIA_CHECK_ARG(dw != nullptr, "endia_hip_conv2d_bwd_weight: dw is null");
  if ((int64_t)p.N * p.P * p.Q == 0) return endia_hip_fill(dw, taps, 0.f);
  ENDIA_CHECK_ARG(x && dy, "endia_hip_conv2d_bwd_weight: null pointer");
  hipLaunchKernelGGL(conv_bwd_weight_direct_kernel, dim3((unsigned)taps), dim3(TPB), 0, ctx().stream, p, x, dy, dw);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_conv2d_bwd_bias(const endia_hip_conv2d_desc* d, const float* dy, float* db) {
  ENDIA_REQUIRE_INIT();
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  ENDIA_CHECK_ARG(db != nullptr, "endia_hip_conv2d_bwd_bias: db is null");
  const int64_t PQ = (int64_t)p.P * p.Q, rows = (int64_t)p.N * p.K;
  if (rows * PQ == 0) return endia_hip_fill(db, p.K, 0.f);
  ENDIA_CHECK_ARG(dy != nullptr, "endia_hip_conv2d_bwd_bias: dy is null");
  ENDIA_CHECK_ARG(rows <= 65535, "endia_hip_conv2d_bwd_bias: N*K = %lld exceeds 65535", (long long)rows);
  // [N*K, P*Q] -> [N*K] with wave-shuffle row sums, then [N, K] -> [K]
  void* tmp = nullptr;
  rc = endia_hip_malloc(rows * (int64_t)sizeof(float), &tmp);
  if (rc) return rc;
  rc = row_reduce(rows, PQ, dy, static_cast<float*>(tmp), 1.f);
  if (!rc) rc = col_reduce(1, p.N, p.K, static_cast<float*>(tmp), db, 1.f);
  endia_hip_free(tmp);  // stream-ordered: later users of the buffer run after the kernels above
  return rc;
}

}  // extern "C"
