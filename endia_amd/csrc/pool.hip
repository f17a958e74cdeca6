// Max and average pooling over 1, 2 or 3 spatial axes of an [N, C, D, H, W] array (unused leading
// spatial axes have extent 1), forward and backward.
//
// Forward follows MaxPool{1,2,3}d.__call__ and AvgPool{1,2,3}d.__call__
// (endia/functional/spacial_ops/max_pool2d_op.mojo:88-150, avg_pool2d_op.mojo:84-140 and their 1-D / 3-D
// siblings; output extent (in + 2*pad - dil*(k-1) - 1) / stride + 1, max_pool2d_op.mojo:57-82):
//   window of output o = taps  o*stride - pad + k*dil,  taps outside the array are skipped;
//   max:  the largest tap (-inf when the window is empty);
//   avg:  sum of the taps / number of taps INSIDE the array (0 when the window is empty).
// The reference registers no backward rule for pooling (vjp = default_vjp, max_pool2d_op.mojo:152-154);
// the gradients here are the adjoints of those loops:
//   max:  dx[i] = sum of dy[o] over the outputs o whose window maximum sits at i (the first tap in scan
//         order that attains the maximum; its flat index within the (D,H,W) volume is written by the forward),
//   avg:  dx[i] = sum over the outputs o whose window holds i of dy[o] / count[o].
// Both directions are gathers (one lane per result element, no atomics), so results do not depend
// on scheduling. The kernels are HBM-bound: algorithmic traffic is the input once and the output once.
#include "common.h"
#include "mfma_tile.h"

namespace {

using mfma::FastDiv;
using mfma::fdiv;

constexpr int TPB = 256;

struct PoolP {
  int D, H, W, Do, Ho, Wo;
  int kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw;
  FastDiv d_wo, d_ho, d_do;  // decode a flat output index
  FastDiv d_w, d_h, d_d;     // decode a flat input index
  FastDiv d_sd, d_sh, d_sw;  // divide by the strides (backward)
  int64_t n_out, n_in;       // N*C*Do*Ho*Wo, N*C*D*H*W
};

inline int stream_grid(int64_t n) {
  int64_t blocks = ceil_div64(n, TPB);
  int64_t cap = (int64_t)endia::ctx().cu_count * 8;
  if (cap < 256) cap = 2048;
  return (int)(blocks > cap ? cap : (blocks < 1 ? 1 : blocks));
}

// flat index within [0, 2^32): split into (plane, z, y, x) with three magic-number divisions
__device__ __forceinline__ void decode(uint32_t j, const FastDiv& dx, const FastDiv& dy, const FastDiv& dz, int X, int Y, int Z,
                                       uint32_t& plane, int& z, int& y, int& x) {
  uint32_t q = fdiv(j, dx);
  x = (int)(j - q * (uint32_t)X);
  uint32_t q2 = fdiv(q, dy);
  y = (int)(q - q2 * (uint32_t)Y);
  plane = fdiv(q2, dz);
  z = (int)(q2 - plane * (uint32_t)Z);
}

template <bool MAX>
__global__ __launch_bounds__(TPB) void pool_fwd_kernel(PoolP p, const float* __restrict__ x, float* __restrict__ y,
                                                       int32_t* __restrict__ arg) {
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t vol = (int64_t)p.D * p.H * p.W;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < p.n_out; j += stride) {
    uint32_t plane;
    int oz, oy, ox;
    decode((uint32_t)j, p.d_wo, p.d_ho, p.d_do, p.Wo, p.Ho, p.Do, plane, oz, oy, ox);
    const float* src = x + plane * vol;
    const int z0 = oz * p.sd - p.pd, y0 = oy * p.sh - p.ph, x0 = ox * p.sw - p.pw;
    float best = -INFINITY, sum = 0.f;
    int best_at = -1, count = 0;
    for (int a = 0; a < p.kd; ++a) {
      const int z = z0 + a * p.dd;
      if ((unsigned)z >= (unsigned)p.D) continue;
      for (int b = 0; b < p.kh; ++b) {
        const int yy = y0 + b * p.dh;
        if ((unsigned)yy >= (unsigned)p.H) continue;
        const int row = (z * p.H + yy) * p.W;
        for (int c = 0; c < p.kw; ++c) {
          const int xx = x0 + c * p.dw;
          if ((unsigned)xx >= (unsigned)p.W) continue;
          const float v = src[row + xx];
          if (MAX) {
            if (best_at < 0 || v > best) { best = v; best_at = row + xx; }
          } else {
            sum += v;
            ++count;
          }
        }
      }
    }
    if (MAX) {
      y[j] = best;
      if (arg) arg[j] = best_at;
    } else {
      y[j] = count > 0 ? sum / (float)count : 0.f;
    }
  }
}

// Windows that tile the input (stride = kernel, no padding, unit dilation; the usual 2 x 2 / 2), W a multiple of 4:
// a lane reads its windows' rows 16 bytes at a time (four consecutive input elements are 4 / KW whole windows
// along the row) and writes 4 / KW outputs. Same visiting order as pool_fwd_kernel (depth, row, column), so the
// first maximum wins and the average adds up in the same order. KW = kernel width in {1, 2, 4}.
template <bool MAX, int KW>
__global__ __launch_bounds__(TPB) void pool_fwd_tiling_kernel(PoolP p, FastDiv d_w4, const float* __restrict__ x,
                                                              float* __restrict__ y, int32_t* __restrict__ arg) {
  constexpr int NWIN = 4 / KW;
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t vol = (int64_t)p.D * p.H * p.W, ovol = (int64_t)p.Do * p.Ho * p.Wo;
  const int W4 = p.W >> 2;
  const int64_t total = (p.n_out / p.Wo) * W4;  // (plane, oz, oy) rows times groups of four input columns
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < total; j += stride) {
    uint32_t plane;
    int oz, oy, x4;
    decode((uint32_t)j, d_w4, p.d_ho, p.d_do, W4, p.Ho, p.Do, plane, oz, oy, x4);
    const float* src = x + plane * vol;
    float best[NWIN], sum[NWIN];
    int at[NWIN];
#pragma unroll
    for (int w = 0; w < NWIN; ++w) { best[w] = 0.f; sum[w] = 0.f; at[w] = -1; }
    for (int a = 0; a < p.kd; ++a)
      for (int b = 0; b < p.kh; ++b) {
        const int row = ((oz * p.kd + a) * p.H + oy * p.kh + b) * p.W + x4 * 4;
        const float4 v4 = *reinterpret_cast<const float4*>(src + row);
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int w = e / KW;
          if (MAX) {
            if (at[w] < 0 || v[e] > best[w]) { best[w] = v[e]; at[w] = row + e; }
          } else {
            sum[w] += v[e];
          }
        }
      }
    const int64_t o = plane * ovol + ((int64_t)oz * p.Ho + oy) * p.Wo + x4 * NWIN;
#pragma unroll
    for (int w = 0; w < NWIN; ++w) {
      if (x4 * NWIN + w >= p.Wo) break;
      if (MAX) {
        y[o + w] = best[w];
        if (arg) arg[o + w] = at[w];
      } else {
        y[o + w] = sum[w] / (float)(p.kd * p.kh * KW);
      }
    }
  }
}

// number of taps of output coordinate o that fall inside [0, extent); without padding every tap does
__device__ __forceinline__ int taps_inside(int o, int k, int s, int pad, int dil, int extent) {
  if (pad == 0) return k;
  int n = 0;
  for (int a = 0; a < k; ++a) n += (unsigned)(o * s - pad + a * dil) < (unsigned)extent;
  return n;
}

// The outputs along one axis whose window holds input coordinate i, for dilation 1: a contiguous range
// lo..hi (empty when lo > hi), o*s - pad <= i <= o*s - pad + k - 1.
__device__ __forceinline__ void covering(int i, int k, int pad, int n_out, const FastDiv& ds, int& lo, int& hi) {
  const int top = i + pad, bottom = i + pad - (k - 1);
  hi = (int)fdiv((uint32_t)top, ds);
  if (hi > n_out - 1) hi = n_out - 1;
  lo = bottom <= 0 ? 0 : (int)fdiv((uint32_t)(bottom + (int)ds.d - 1), ds);
}

// UNIT: every dilation is 1, so the covering outputs are ranges; otherwise each tap is tried in turn.
template <bool MAX, bool UNIT>
__global__ __launch_bounds__(TPB) void pool_bwd_kernel(PoolP p, const float* __restrict__ dy, const int32_t* __restrict__ arg,
                                                       float* __restrict__ dx) {
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t ovol = (int64_t)p.Do * p.Ho * p.Wo;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < p.n_in; j += stride) {
    uint32_t plane;
    int z, yy, xx;
    decode((uint32_t)j, p.d_w, p.d_h, p.d_d, p.W, p.H, p.D, plane, z, yy, xx);
    const float* g = dy + plane * ovol;
    const int32_t* at = MAX ? arg + plane * ovol : nullptr;
    const int self = (z * p.H + yy) * p.W + xx;
    float acc = 0.f;
    if (UNIT) {
      int z_lo, z_hi, y_lo, y_hi, x_lo, x_hi;
      covering(z, p.kd, p.pd, p.Do, p.d_sd, z_lo, z_hi);
      covering(yy, p.kh, p.ph, p.Ho, p.d_sh, y_lo, y_hi);
      covering(xx, p.kw, p.pw, p.Wo, p.d_sw, x_lo, x_hi);
      for (int oz = z_lo; oz <= z_hi; ++oz) {
        const int cz = MAX ? 0 : taps_inside(oz, p.kd, p.sd, p.pd, 1, p.D);
        for (int oy = y_lo; oy <= y_hi; ++oy) {
          const int cy = MAX ? 0 : taps_inside(oy, p.kh, p.sh, p.ph, 1, p.H);
          for (int ox = x_lo; ox <= x_hi; ++ox) {
            const int o = (oz * p.Ho + oy) * p.Wo + ox;
            if (MAX) {
              if (at[o] == self) acc += g[o];
            } else {
              acc += g[o] / (float)(cz * cy * taps_inside(ox, p.kw, p.sw, p.pw, 1, p.W));
            }
          }
        }
      }
    } else {
      // outputs whose window holds this element: o*stride - pad + k*dil = coordinate, per axis
      for (int a = 0; a < p.kd; ++a) {
        const int tz = z + p.pd - a * p.dd;
        if (tz < 0) continue;
        const int oz = (int)fdiv((uint32_t)tz, p.d_sd);
        if (oz * p.sd != tz || oz >= p.Do) continue;
        const int cz = MAX ? 0 : taps_inside(oz, p.kd, p.sd, p.pd, p.dd, p.D);
        for (int b = 0; b < p.kh; ++b) {
          const int ty = yy + p.ph - b * p.dh;
          if (ty < 0) continue;
          const int oy = (int)fdiv((uint32_t)ty, p.d_sh);
          if (oy * p.sh != ty || oy >= p.Ho) continue;
          const int cy = MAX ? 0 : taps_inside(oy, p.kh, p.sh, p.ph, p.dh, p.H);
          for (int c = 0; c < p.kw; ++c) {
            const int tx = xx + p.pw - c * p.dw;
            if (tx < 0) continue;
            const int ox = (int)fdiv((uint32_t)tx, p.d_sw);
            if (ox * p.sw != tx || ox >= p.Wo) continue;
            const int o = (oz * p.Ho + oy) * p.Wo + ox;
            if (MAX) {
              if (at[o] == self) acc += g[o];
            } else {
              acc += g[o] / (float)(cz * cy * taps_inside(ox, p.kw, p.sw, p.pw, p.dw, p.W));
            }
          }
        }
      }
    }
    dx[j] = acc;
  }
}

// Unit dilation, W a multiple of 4: one lane produces 4 consecutive elements of a row, so the index
// decode and the depth / height ranges are shared by the four and the store is 16 bytes.
template <bool MAX>
__global__ __launch_bounds__(TPB) void pool_bwd_row4_kernel(PoolP p, FastDiv d_w4, const float* __restrict__ dy,
                                                            const int32_t* __restrict__ arg, float* __restrict__ dx) {
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t ovol = (int64_t)p.Do * p.Ho * p.Wo;
  const int W4 = p.W >> 2;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < (p.n_in >> 2); j += stride) {
    uint32_t plane;
    int z, yy, x4;
    decode((uint32_t)j, d_w4, p.d_h, p.d_d, W4, p.H, p.D, plane, z, yy, x4);
    const float* g = dy + plane * ovol;
    const int32_t* at = MAX ? arg + plane * ovol : nullptr;
    const int self0 = (z * p.H + yy) * p.W + x4 * 4;
    int z_lo, z_hi, y_lo, y_hi;
    covering(z, p.kd, p.pd, p.Do, p.d_sd, z_lo, z_hi);
    covering(yy, p.kh, p.ph, p.Ho, p.d_sh, y_lo, y_hi);
    int x_lo[4], x_hi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) covering(x4 * 4 + e, p.kw, p.pw, p.Wo, p.d_sw, x_lo[e], x_hi[e]);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int oz = z_lo; oz <= z_hi; ++oz) {
      const int cz = MAX ? 0 : taps_inside(oz, p.kd, p.sd, p.pd, 1, p.D);
      for (int oy = y_lo; oy <= y_hi; ++oy) {
        const int czy = MAX ? 0 : cz * taps_inside(oy, p.kh, p.sh, p.ph, 1, p.H);
        const int row = (oz * p.Ho + oy) * p.Wo;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          for (int ox = x_lo[e]; ox <= x_hi[e]; ++ox) {
            if (MAX) {
              if (at[row + ox] == self0 + e) acc[e] += g[row + ox];
            } else {
              acc[e] += g[row + ox] / (float)(czy * taps_inside(ox, p.kw, p.sw, p.pw, 1, p.W));
            }
          }
      }
    }
    reinterpret_cast<float4*>(dx)[j] = make_float4(acc[0], acc[1], acc[2], acc[3]);
  }
}

// Windows that tile the input (stride = kernel, no padding, unit dilation; the usual 2 x 2 / 2): an input
// element lies in at most one window, found with one division per axis, so the gradient is one select
// (or one scale) per element. KW = kernel width in {1, 2, 4}; a lane writes 4 consecutive elements.
template <bool MAX, int KW>
__global__ __launch_bounds__(TPB) void pool_bwd_tiling_kernel(PoolP p, FastDiv d_w4, const float* __restrict__ dy,
                                                              const int32_t* __restrict__ arg, float* __restrict__ dx, float taps) {
  constexpr int NWIN = 4 / KW;  // windows met by the lane's four elements
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t ovol = (int64_t)p.Do * p.Ho * p.Wo;
  const int W4 = p.W >> 2;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < (p.n_in >> 2); j += stride) {
    uint32_t plane;
    int z, yy, x4;
    decode((uint32_t)j, d_w4, p.d_h, p.d_d, W4, p.H, p.D, plane, z, yy, x4);
    const int oz = (int)fdiv((uint32_t)z, p.d_sd), oy = (int)fdiv((uint32_t)yy, p.d_sh), ox0 = x4 * NWIN;
    float out[4] = {0.f, 0.f, 0.f, 0.f};
    if (oz < p.Do && oy < p.Ho) {  // rows and slabs past the last whole window receive no gradient
      const int64_t row = plane * ovol + ((int64_t)oz * p.Ho + oy) * p.Wo;
      const int self0 = (z * p.H + yy) * p.W + x4 * 4;
#pragma unroll
      for (int w = 0; w < NWIN; ++w) {
        if (ox0 + w >= p.Wo) break;
        const float g = dy[row + ox0 + w];
        if (MAX) {
          const int at = arg[row + ox0 + w];
#pragma unroll
          for (int e = 0; e < KW; ++e) out[w * KW + e] = at == self0 + w * KW + e ? g : 0.f;
        } else {
#pragma unroll
          for (int e = 0; e < KW; ++e) out[w * KW + e] = g / taps;
        }
      }
    }
    reinterpret_cast<float4*>(dx)[j] = make_float4(out[0], out[1], out[2], out[3]);
  }
}

template <bool MAX>
void launch_tiling(const PoolP& p, FastDiv d_w4, int grid, hipStream_t s, const float* dy, const int32_t* arg, float* dx) {
  const float inv = (float)(p.kd * p.kh * p.kw);  // every tap of every window lies inside the array
  if (p.kw == 1) hipLaunchKernelGGL((pool_bwd_tiling_kernel<MAX, 1>), dim3(grid), dim3(TPB), 0, s, p, d_w4, dy, arg, dx, inv);
  else if (p.kw == 2) hipLaunchKernelGGL((pool_bwd_tiling_kernel<MAX, 2>), dim3(grid), dim3(TPB), 0, s, p, d_w4, dy, arg, dx, inv);
  else hipLaunchKernelGGL((pool_bwd_tiling_kernel<MAX, 4>), dim3(grid), dim3(TPB), 0, s, p, d_w4, dy, arg, dx, inv);
}

int32_t make_params(const endia_hip_pool_desc* d, PoolP& p, const char* who) {
  if (!d) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null descriptor", who);
  const int64_t in[3] = {d->D, d->H, d->W};
  int64_t out[3];
  if (d->N < 0 || d->C < 0) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: negative batch or channel count", who);
  for (int i = 0; i < 3; ++i) {
    if (in[i] < 1 || d->kernel[i] < 1 || d->stride[i] < 1 || d->padding[i] < 0 || d->dilation[i] < 1)
      return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: axis %d: extent %lld kernel %lld stride %lld padding %lld dilation %lld", who,
                         i, (long long)in[i], (long long)d->kernel[i], (long long)d->stride[i], (long long)d->padding[i],
                         (long long)d->dilation[i]);
    const int64_t span = in[i] + 2 * d->padding[i] - d->dilation[i] * (d->kernel[i] - 1) - 1;
    if (span < 0) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: axis %d: the window does not fit the padded input", who, i);
    out[i] = span / d->stride[i] + 1;
    if (in[i] >= (1ll << 30) || d->kernel[i] > 1024 || d->padding[i] > (1 << 20) || d->dilation[i] > (1 << 20) || d->stride[i] > (1 << 20))
      return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: axis %d: window parameters out of range", who, i);
  }
  p.n_in = d->N * d->C * in[0] * in[1] * in[2];
  p.n_out = d->N * d->C * out[0] * out[1] * out[2];
  if (p.n_in >= (1ll << 31) || p.n_out >= (1ll << 31))
    return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: more than 2^31 elements", who);
  p.D = (int)in[0]; p.H = (int)in[1]; p.W = (int)in[2];
  p.Do = (int)out[0]; p.Ho = (int)out[1]; p.Wo = (int)out[2];
  p.kd = (int)d->kernel[0]; p.kh = (int)d->kernel[1]; p.kw = (int)d->kernel[2];
  p.sd = (int)d->stride[0]; p.sh = (int)d->stride[1]; p.sw = (int)d->stride[2];
  p.pd = (int)d->padding[0]; p.ph = (int)d->padding[1]; p.pw = (int)d->padding[2];
  p.dd = (int)d->dilation[0]; p.dh = (int)d->dilation[1]; p.dw = (int)d->dilation[2];
  p.d_wo = make_fastdiv(p.Wo); p.d_ho = make_fastdiv(p.Ho); p.d_do = make_fastdiv(p.Do);
  p.d_w = make_fastdiv(p.W); p.d_h = make_fastdiv(p.H); p.d_d = make_fastdiv(p.D);
  p.d_sd = make_fastdiv(p.sd); p.d_sh = make_fastdiv(p.sh); p.d_sw = make_fastdiv(p.sw);
  return ENDIA_HIP_OK;
}

}  // namespace

using namespace endia;

extern "C" {

int32_t endia_hip_pool_out_shape(const endia_hip_pool_desc* desc, int64_t* out_dhw) {
  PoolP p;
  int32_t rc = make_params(desc, p, __func__);
  if (rc) return rc;
  ENDIA_CHECK_ARG(out_dhw, "endia_hip_pool_out_shape: null output");
  out_dhw[0] = p.Do; out_dhw[1] = p.Ho; out_dhw[2] = p.Wo;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_pool_fwd(const endia_hip_pool_desc* desc, int32_t mode, const float* x, float* y, int32_t* argmax) {
  ENDIA_REQUIRE_INIT();
  PoolP p;
  int32_t rc = make_params(desc, p, __func__);
  if (rc) return rc;
  ENDIA_CHECK_ARG(mode == ENDIA_POOL_MAX || mode == ENDIA_POOL_AVG, "endia_hip_pool_fwd: unknown mode %d", mode);
  if (p.n_out == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && y, "endia_hip_pool_fwd: null pointer");
  const int grid = stream_grid(p.n_out);
  const bool tiling = p.dd == 1 && p.dh == 1 && p.dw == 1 && p.sd == p.kd && p.sh == p.kh && p.sw == p.kw && p.pd == 0 &&
                      p.ph == 0 && p.pw == 0 && (p.kw == 1 || p.kw == 2 || p.kw == 4);
  if (tiling && p.W % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const FastDiv d_w4 = make_fastdiv(p.W / 4);
    const int g4 = stream_grid(p.n_out / p.Wo * (p.W / 4));
    hipStream_t s = ctx().stream;
    int32_t* none = nullptr;
#define ENDIA_POOL_FWD_TILING(KW)                                                                                         \
  do {                                                                                                                    \
    if (mode == ENDIA_POOL_MAX) hipLaunchKernelGGL((pool_fwd_tiling_kernel<true, KW>), dim3(g4), dim3(TPB), 0, s, p, d_w4, x, y, argmax); \
    else hipLaunchKernelGGL((pool_fwd_tiling_kernel<false, KW>), dim3(g4), dim3(TPB), 0, s, p, d_w4, x, y, none);             \
  } while (0)
    if (p.kw == 1) ENDIA_POOL_FWD_TILING(1);
    else if (p.kw == 2) ENDIA_POOL_FWD_TILING(2);
    else ENDIA_POOL_FWD_TILING(4);
#undef ENDIA_POOL_FWD_TILING
  } else if (mode == ENDIA_POOL_MAX) {
    hipLaunchKernelGGL((pool_fwd_kernel<true>), dim3(grid), dim3(TPB), 0, ctx().stream, p, x, y, argmax);
  } else {
    hipLaunchKernelGGL((pool_fwd_kernel<false>), dim3(grid), dim3(TPB), 0, ctx().stream, p, x, y, (int32_t*)nullptr);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_pool_bwd(const endia_hip_pool_desc* desc, int32_t mode, const float* dy, const int32_t* argmax, float* dx) {
  ENDIA_REQUIRE_INIT();
  PoolP p;
  int32_t rc = make_params(desc, p, __func__);
  if (rc) return rc;
  ENDIA_CHECK_ARG(mode == ENDIA_POOL_MAX || mode == ENDIA_POOL_AVG, "endia_hip_pool_bwd: unknown mode %d", mode);
  if (p.n_in == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(dy && dx, "endia_hip_pool_bwd: null pointer");
  ENDIA_CHECK_ARG(mode != ENDIA_POOL_MAX || argmax, "endia_hip_pool_bwd: max pooling needs the argmax array of the forward");
  const int grid = stream_grid(p.n_in);
  const bool unit = p.dd == 1 && p.dh == 1 && p.dw == 1;
  const bool tiling = unit && p.sd == p.kd && p.sh == p.kh && p.sw == p.kw && p.pd == 0 && p.ph == 0 && p.pw == 0 &&
                      (p.kw == 1 || p.kw == 2 || p.kw == 4);
  if (tiling && p.W % 4 == 0 && (reinterpret_cast<uintptr_t>(dx) & 15) == 0) {
    const FastDiv d_w4 = make_fastdiv(p.W / 4);
    const int g4 = stream_grid(p.n_in / 4);
    if (mode == ENDIA_POOL_MAX) launch_tiling<true>(p, d_w4, g4, ctx().stream, dy, argmax, dx);
    else launch_tiling<false>(p, d_w4, g4, ctx().stream, dy, argmax, dx);
  } else if (unit && p.W % 4 == 0 && (reinterpret_cast<uintptr_t>(dx) & 15) == 0) {
    const FastDiv d_w4 = make_fastdiv(p.W / 4);
    const int g4 = stream_grid(p.n_in / 4);
    if (mode == ENDIA_POOL_MAX) hipLaunchKernelGGL((pool_bwd_row4_kernel<true>), dim3(g4), dim3(TPB), 0, ctx().stream, p, d_w4, dy, argmax, dx);
    else hipLaunchKernelGGL((pool_bwd_row4_kernel<false>), dim3(g4), dim3(TPB), 0, ctx().stream, p, d_w4, dy, argmax, dx);
  } else if (mode == ENDIA_POOL_MAX) {
    if (unit) hipLaunchKernelGGL((pool_bwd_kernel<true, true>), dim3(grid), dim3(TPB), 0, ctx().stream, p, dy, argmax, dx);
    else hipLaunchKernelGGL((pool_bwd_kernel<true, false>), dim3(grid), dim3(TPB), 0, ctx().stream, p, dy, argmax, dx);
  } else {
    if (unit) hipLaunchKernelGGL((pool_bwd_kernel<false, true>), dim3(grid), dim3(TPB), 0, ctx().stream, p, dy, argmax, dx);
    else hipLaunchKernelGGL((pool_bwd_kernel<false, false>), dim3(grid), dim3(TPB), 0, ctx().stream, p, dy, argmax, dx);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

}  // extern "C"
