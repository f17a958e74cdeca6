// Sum reductions: ReduceAdd.__call__ (endia/functional/reduce_ops/reduce_add_op.mojo:65-210), which
// is also Expand.vjp, the bias gradient db = 1^T dZ (endia/functional/view_ops/expand_op.mojo:121-126),
// sum and mean (sum_op.mojo:35-62, mean_op.mojo:35-65), and the fused MSE loss + gradient
// (endia/functional/loss_ops/mse_op.mojo:17-20).
//
// The reference accumulates sequentially in fp32 into a zeroed output. Here every reduction is two
// stages with a fixed shape (so results are run-to-run identical): stage 1 spreads the input over
// enough work-groups to fill the chip, each wave reading 1 KiB of consecutive addresses per access
// and combining lanes with wave shuffles; stage 2 adds the per-group partials in index order.
#include "common.h"

namespace {

constexpr int TPB = 256;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// all 256 threads call; result valid in thread 0
__device__ __forceinline__ float block_sum(float v, float* red /* >= 4 floats */) {
  v = wave_sum(v);
  int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// ---- column reduction: x[batch][R][C] -> out[batch][C] (sum over R) --------------------------
// grid (ceil(C/256), S, batch). A wave reads 256 consecutive columns of one row per access (float4
// per lane); the four waves of a group take rows r, r+1, r+2, r+3 (mod 4) of the group's row range.
__global__ __launch_bounds__(TPB) void col_reduce_vec_kernel(const float* __restrict__ x, float* __restrict__ part,
                                                             int64_t R, int64_t C, int64_t rows_per_split) {
  __shared__ float4 red[4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t c = ((int64_t)blockIdx.x * 64 + lane) * 4;
  const int64_t b = blockIdx.z;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_split;
  int64_t r1 = r0 + rows_per_split;
  if (r1 > R) r1 = R;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (c < C) {
    const float* base = x + b * R * C + c;
#pragma unroll 8
    for (int64_t r = r0 + w; r < r1; r += 4) {
      float4 v = *reinterpret_cast<const float4*>(base + r * C);
      acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
  }
  red[w][lane] = acc;
  __syncthreads();
  if (w == 0 && c < C) {
    float4 a = red[0][lane], b1 = red[1][lane], c1 = red[2][lane], d = red[3][lane];
    float4 s = make_float4((a.x + b1.x) + (c1.x + d.x), (a.y + b1.y) + (c1.y + d.y),
                           (a.z + b1.z) + (c1.z + d.z), (a.w + b1.w) + (c1.w + d.w));
    *reinterpret_cast<float4*>(part + ((b * gridDim.y + blockIdx.y) * C + c)) = s;
  }
}

// A mid-size input (up to 2^22 elements, at most 2048 rows: the bias gradient of a layer a few thousand wide over a
// batch of about a thousand) in ONE launch: a group owns 16 columns, its 256 threads are 4 column quads x 64 row lanes,
// a thread adds rows lane, lane + 64, ... with sixteen 16-byte loads in flight, and the 64 partial rows meet in LDS in a
// fixed pairwise order. Two launches (first stage over the whole chip, then the partial sums) take 9.0 us at 1024 x 2048
// where this takes 7.4: one launch fewer per bias gradient for steps that are counted in launches.
__device__ __forceinline__ void col_reduce_mid_body(const float* __restrict__ x, float* __restrict__ out, int64_t R, int64_t C,
                                                    float scale, int64_t group) {
  __shared__ float4 red[64][4];
  const int cl = threadIdx.x & 3, rl = threadIdx.x >> 2;
  const int64_t c = (group * 4 + cl) * 4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (c < C) {
    const float* base = x + c;
#pragma unroll 16
    for (int64_t r = rl; r < R; r += 64) {
      const float4 v = *reinterpret_cast<const float4*>(base + r * C);
      acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
  }
  red[rl][cl] = acc;
  __syncthreads();
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) {
    if (rl < s) {
      const float4 a = red[rl][cl], b = red[rl + s][cl];
      red[rl][cl] = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
    }
    __syncthreads();
  }
  if (rl == 0 && c < C) {
    const float4 t = red[0][cl];
    *reinterpret_cast<float4*>(out + c) = make_float4(t.x * scale, t.y * scale, t.z * scale, t.w * scale);
  }
}

__global__ __launch_bounds__(TPB) void col_reduce_mid_kernel(const float* __restrict__ x, float* __restrict__ out, int64_t R, int64_t C,
                                                             float scale) {
  col_reduce_mid_body(x, out, R, C, scale, blockIdx.x);
}

// Several such sums in one launch (endia_hip_col_sum_multi): the work-groups [first[m], first[m + 1]) are the column groups
// of member m, each computed exactly as the single launch computes it.
constexpr int kMaxSums = 16;
struct ColSumMembers {
  int count;
  int first[kMaxSums + 1];
  const float* x[kMaxSums];
  float* out[kMaxSums];
  int64_t R[kMaxSums], C[kMaxSums];
  float scale[kMaxSums];
};

__global__ __launch_bounds__(TPB) void col_reduce_mid_multi_kernel(const ColSumMembers a) {
  int m = 0;
  while (m + 1 < a.count && (int)blockIdx.x >= a.first[m + 1]) ++m;
  col_reduce_mid_body(a.x[m], a.out[m], a.R[m], a.C[m], a.scale[m], (int64_t)blockIdx.x - a.first[m]);
}

// scalar variant for C not a multiple of 4 or unaligned: thread per column, 256 columns per group
__global__ __launch_bounds__(TPB) void col_reduce_scalar_kernel(const float* __restrict__ x, float* __restrict__ part,
                                                                int64_t R, int64_t C, int64_t rows_per_split) {
  const int64_t c = (int64_t)blockIdx.x * TPB + threadIdx.x;
  const int64_t b = blockIdx.z;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_split;
  int64_t r1 = r0 + rows_per_split;
  if (r1 > R) r1 = R;
  if (c >= C) return;
  float acc = 0.f;
  const float* base = x + b * R * C + c;
  for (int64_t r = r0; r < r1; ++r) acc += base[r * C];
  part[(b * gridDim.y + blockIdx.y) * C + c] = acc;
}

// stage 2: out[b][c] = scale * sum_s part[b][s][c]. 64 columns per group; the four waves take
// s = w, w+4, ... and are combined through LDS in wave order, so the result does not depend on timing.
// inner > 0: the columns are an [C / inner][inner] array and the sums are stored transposed, as [inner][C / inner] (the
// 3 x 3 weight gradient sums its partial products in [tap][k][c] order and stores them as the weights' [k][c][tap]).
__device__ __forceinline__ void col_reduce_final_body(const float* __restrict__ part, float* __restrict__ out, int64_t S, int64_t C,
                                                      float scale, int64_t inner, int64_t group, int64_t b) {
  __shared__ float red[4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t c = group * 64 + lane;
  float acc = 0.f;
  if (c < C) {
#pragma unroll 8
    for (int64_t s = w; s < S; s += 4) acc += part[(b * S + s) * C + c];
  }
  red[w][lane] = acc;
  __syncthreads();
  if (w == 0 && c < C) {
    int64_t at = c;
    if (inner > 0) {
      const int64_t o = c / inner;
      at = (c - o * inner) * (C / inner) + o;
    }
    out[b * C + at] = ((red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane])) * scale;
  }
}

__global__ __launch_bounds__(TPB) void col_reduce_final_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                               int64_t S, int64_t C, int64_t batch, float scale, int64_t inner) {
  col_reduce_final_body(part, out, S, C, scale, inner, blockIdx.x, blockIdx.y);
}

// The last stage of one reduction and, in the work-groups behind its own, a second small reduction that needs this stage
// only (a weight gradient's partial sums and its bias gradient's: one launch instead of two). Each as the kernel above
// computes it.
struct FinalJob {
  const float* part;
  float* out;
  int64_t S, C, inner;
  float scale;
};
__global__ __launch_bounds__(TPB) void col_reduce_final_pair_kernel(const FinalJob a, const FinalJob b, int groups_a) {
  if ((int)blockIdx.x < groups_a) col_reduce_final_body(a.part, a.out, a.S, a.C, a.scale, a.inner, blockIdx.x, 0);
  else col_reduce_final_body(b.part, b.out, b.S, b.C, b.scale, b.inner, (int)blockIdx.x - groups_a, 0);
}

// ---- row reduction: x[R][C] -> out[R] (sum over C) --------------------------------------------
// grid (S, R). Each group sums a contiguous chunk of one row; partials [R][S].
__global__ __launch_bounds__(TPB) void row_reduce_kernel(const float* __restrict__ x, float* __restrict__ part,
                                                         int64_t C, int64_t chunk, int vec, float scale) {
  __shared__ float red[4];
  const int64_t r = blockIdx.y;
  const int64_t c0 = (int64_t)blockIdx.x * chunk;
  int64_t c1 = c0 + chunk;
  if (c1 > C) c1 = C;
  const float* row = x + r * C;
  float acc = 0.f;
  if (vec) {  // chunk % 4 == 0, row base 16-byte aligned
    int64_t n4 = (c1 - c0) >> 2;
    const float4* p4 = reinterpret_cast<const float4*>(row + c0);
#pragma unroll 4
    for (int64_t j = threadIdx.x; j < n4; j += TPB) {
      float4 v = p4[j];
      acc += (v.x + v.y) + (v.z + v.w);
    }
    for (int64_t j = c0 + (n4 << 2) + threadIdx.x; j < c1; j += TPB) acc += row[j];
  } else {
    for (int64_t j = c0 + threadIdx.x; j < c1; j += TPB) acc += row[j];
  }
  float s = block_sum(acc, red);
  if (threadIdx.x == 0) part[r * gridDim.x + blockIdx.x] = s * scale;
}

// stage 2: out[r] = scale * sum_s part[r][s]; one wave per row
__global__ __launch_bounds__(TPB) void row_reduce_final_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                               int64_t R, int64_t S, float scale) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= R) return;
  // (eight loads in flight: a full reduction's 2048 partial sums are 32 rounds of one dependent load each otherwise)
  float acc = 0.f;
  int64_t s = lane;
  for (; s + 7 * 64 < S; s += 8 * 64) {
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) t[u] = part[r * S + s + 64 * u];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += t[u];
  }
  for (; s < S; s += 64) acc += part[r * S + s];
  acc = wave_sum(acc);
  if (lane == 0) out[r] = acc * scale;
}

// ---- any mask: one work-group per output element ----------------------------------------------
struct RedDesc {
  int nk, nr;            // number of kept / reduced axes
  int64_t kshape[8], kstride[8];
  int64_t rshape[8], rstride[8];
};

__global__ __launch_bounds__(TPB) void generic_reduce_kernel(RedDesc d, const float* __restrict__ x,
                                                             float* __restrict__ out, int64_t nred, float scale) {
  __shared__ float red[4];
  int64_t o = blockIdx.x, rem = o, base = 0;
  for (int k = d.nk - 1; k >= 0; --k) {
    int64_t q = rem / d.kshape[k];
    base += (rem - q * d.kshape[k]) * d.kstride[k];
    rem = q;
  }
  float acc = 0.f;
  for (int64_t j = threadIdx.x; j < nred; j += TPB) {
    int64_t r = j, off = base;
    for (int k = d.nr - 1; k >= 0; --k) {
      int64_t q = r / d.rshape[k];
      off += (r - q * d.rshape[k]) * d.rstride[k];
      r = q;
    }
    acc += x[off];
  }
  float s = block_sum(acc, red);
  if (threadIdx.x == 0) out[o] = s * scale;
}

// ---- max / min / product and the positions of the extrema: one work-group per output element ----
// Each thread walks its share of the reduced elements in ascending order, so "first" means the same in every
// thread; threads are then combined by value, ties going to the smaller position.
struct Extreme {
  float v;
  int64_t at;
};

template <int OP>
__device__ __forceinline__ bool better(float v, float best) {
  return (OP == ENDIA_REDUCE_MAX || OP == ENDIA_REDUCE_ARGMAX) ? v > best : v < best;
}

template <int OP>
__device__ __forceinline__ Extreme pick(Extreme a, Extreme b) {
  if (better<OP>(b.v, a.v)) return b;
  if (better<OP>(a.v, b.v)) return a;
  if (a.at < 0) return b;  // neither holds a value yet, or equal values: the smaller position
  if (b.at < 0) return a;
  return a.at <= b.at ? a : b;
}

template <int OP>
__global__ __launch_bounds__(TPB) void reduce_op_kernel(RedDesc d, const float* __restrict__ x, float* __restrict__ out,
                                                        int64_t nred) {
  constexpr bool ARG = OP == ENDIA_REDUCE_ARGMAX || OP == ENDIA_REDUCE_ARGMIN;
  constexpr bool MUL = OP == ENDIA_REDUCE_MUL;
  constexpr bool UP = OP == ENDIA_REDUCE_MAX || OP == ENDIA_REDUCE_ARGMAX;
  __shared__ float red_v[4];
  __shared__ long long red_at[4];
  int64_t o = blockIdx.x, rem = o, base = 0;
  for (int k = d.nk - 1; k >= 0; --k) {
    int64_t q = rem / d.kshape[k];
    base += (rem - q * d.kshape[k]) * d.kstride[k];
    rem = q;
  }
  Extreme e = {MUL ? 1.f : (UP ? -INFINITY : INFINITY), -1};
  for (int64_t j = threadIdx.x; j < nred; j += TPB) {
    int64_t r = j, off = base;
    for (int k = d.nr - 1; k >= 0; --k) {
      int64_t q = r / d.rshape[k];
      off += (r - q * d.rshape[k]) * d.rstride[k];
      r = q;
    }
    const float v = x[off];
    if (MUL) e.v *= v;
    else if (better<OP>(v, e.v)) { e.v = v; e.at = j; }
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) {
    Extreme other = {__shfl_down(e.v, s, 64), (int64_t)__shfl_down((long long)e.at, s, 64)};
    if (MUL) e.v *= other.v;
    else e = pick<OP>(e, other);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) { red_v[w] = e.v; red_at[w] = e.at; }
  __syncthreads();
  if (threadIdx.x == 0) {
    Extreme t = {red_v[0], (int64_t)red_at[0]};
    for (int i = 1; i < 4; ++i) {
      Extreme other = {red_v[i], (int64_t)red_at[i]};
      if (MUL) t.v *= other.v;
      else t = pick<OP>(t, other);
    }
    out[o] = ARG ? (float)t.at : t.v;
  }
}

// ---- MSE ------------------------------------------------------------------------------------
// One pass: dpred = 2 (p - t) / n and per-group partial sums of (p - t)^2.
__global__ __launch_bounds__(TPB) void mse_kernel(const float* __restrict__ p, const float* __restrict__ t,
                                                  float* __restrict__ dp, float* __restrict__ part, int64_t n,
                                                  float two_over_n, int vec, float part_scale) {
  __shared__ float red[4];
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  float acc = 0.f;
  if (vec) {
    int64_t n4 = n >> 2;
    const float4* p4 = reinterpret_cast<const float4*>(p);
    const float4* t4 = reinterpret_cast<const float4*>(t);
    float4* d4 = reinterpret_cast<float4*>(dp);
    for (int64_t j = i; j < n4; j += stride) {
      float4 a = p4[j], b = t4[j];
      float4 d = make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w);
      acc += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
      if (dp) d4[j] = make_float4(d.x * two_over_n, d.y * two_over_n, d.z * two_over_n, d.w * two_over_n);
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) {
      float d = p[j] - t[j];
      acc += d * d;
      if (dp) dp[j] = d * two_over_n;
    }
  } else {
    for (int64_t j = i; j < n; j += stride) {
      float d = p[j] - t[j];
      acc += d * d;
      if (dp) dp[j] = d * two_over_n;
    }
  }
  float s = block_sum(acc, red);
  if (part && threadIdx.x == 0) part[blockIdx.x] = s * part_scale;
}

__global__ __launch_bounds__(TPB) void sum_partials_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                           int64_t S, float scale) {
  __shared__ float red[4];
  float acc = 0.f;
  for (int64_t j = threadIdx.x; j < S; j += TPB) acc += part[j];
  float s = block_sum(acc, red);
  if (threadIdx.x == 0) out[0] = s * scale;
}

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

// Scratch of endia_hip_col_sum_static, the entry point for callers that cannot allocate: the first-stage partial sums
// live in this array instead of the library's growing workspace. Every device the library runs on holds its own copy
// (1 MiB) until the process ends. In host code the name `scratch` is only a handle for hipGetSymbolAddress, never an
// address a kernel could use: static_scratch_init() resolves it once per device and everything else uses that pointer.
constexpr int64_t kStaticScratchFloats = 1 << 18;
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices] = {};

namespace endia {

// Called by endia_hip_init with `device` current: the address of this device's copy of the static scratch array.
int32_t static_scratch_init(int device) {
  if (device < 0 || device >= kMaxDevices) return ENDIA_HIP_OK;  // endia_hip_col_sum_static reports it when called
  if (g_scratch_ptr[device]) return ENDIA_HIP_OK;
  float* ptr = nullptr;
  ENDIA_HIP_CALL(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
  g_scratch_ptr[device] = ptr;
  return ENDIA_HIP_OK;
}

// How the column reduction cuts its rows: S splits of rows_per_split rows each (S = 0: one launch, no first stage;
// S = -1: the columns do not fit `part_floats`, the room the caller has for first-stage partial sums, 0 = no limit).
// Pure arithmetic, no device: endia_hip_col_sum_plan exposes it so that the clamp can be tested on any host.
// vec: C is a multiple of 4 and x and out start on 16-byte boundaries (the one-launch kernel for mid-size inputs needs it).
static bool col_reduce_mid(int64_t batch, int64_t R, int64_t C, bool vec) {
  return vec && batch == 1 && R <= 2048 && R >= 64 && R * C <= (1 << 22);
}
static void col_reduce_plan(int64_t batch, int64_t R, int64_t C, int64_t cus, int64_t part_floats, bool vec, int64_t* S_out, int64_t* rows_out) {
  const int64_t col_tiles = ceil_div64(C, 256);
  if ((R <= 1024 && batch * R * C <= (1 << 20)) || col_reduce_mid(batch, R, C, vec)) {
    *S_out = 0;
    *rows_out = R;
    return;
  }
  // enough row splits for ~4 groups per CU, at least 16 rows each
  int64_t S = cus * 4 / (col_tiles * batch);
  const int64_t cap = col_tiles * batch * 64 < cus ? 256 : 64;  // a narrow input needs more row splits to fill the chip
  if (S > cap) S = cap;
  if (S < 1) S = 1;
  const int64_t max_s = ceil_div64(R, 16);
  if (S > max_s) S = max_s;
  if (S > 1024) S = 1024;
  if (part_floats > 0 && S * batch * C > part_floats) S = part_floats / (batch * C);
  if (S < 1) {
    *S_out = -1;
    *rows_out = 0;
    return;
  }
  const int64_t rows_per_split = ceil_div64(R, S);
  *S_out = ceil_div64(R, rows_per_split);
  *rows_out = rows_per_split;
}

// out[b][c] = scale * sum_r x[b][r][c]. The first-stage partial sums go to `part` (room for part_floats) when the
// caller brings it, else to the library's workspace; with too little room the rows are cut into fewer splits.
// rider: a second reduction out2[c] = sum_r x2[r][c] of at most 1024 rows and 2^20 elements (batch 1 only), whose one stage
// shares the launch of this reduction's last stage where there is one.
struct ColSumRider {
  int64_t R, C;
  const float* x;
  float* out;
};
static int32_t col_reduce_with(int64_t batch, int64_t R, int64_t C, const float* x, float* out, float scale, float* part,
                               int64_t part_floats, int64_t inner = 0, const ColSumRider* rider = nullptr) {
  hipStream_t s = ctx().stream;
  const bool ride = rider && batch == 1 && rider->R >= 1 && rider->R <= 1024 && rider->R * rider->C <= (1 << 20) && rider->C >= 1 &&
                    ceil_div64(C, 64) + ceil_div64(rider->C, 64) < (1ll << 31);
  // (the last stage, alone or with the rider in its launch)
  auto last_stage = [&](const float* from, int64_t rows) {
    if (ride) {
      const FinalJob a{from, out, rows, C, inner, scale}, b{rider->x, rider->out, rider->R, rider->C, 0, 1.f};
      const int groups_a = (int)ceil_div64(C, 64);
      hipLaunchKernelGGL(col_reduce_final_pair_kernel, dim3((unsigned)(groups_a + ceil_div64(rider->C, 64))), dim3(TPB), 0, s, a, b, groups_a);
    } else {
      hipLaunchKernelGGL(col_reduce_final_kernel, dim3((unsigned)ceil_div64(C, 64), (unsigned)batch), dim3(TPB), 0, s, from, out, rows,
                         C, batch, scale, inner);
    }
  };
  const bool vec = (C % 4 == 0) && al16(x);
  const int64_t col_tiles = ceil_div64(C, 256);
  if (col_tiles * 1 > 2147483647ll || batch > 65535)
    return fail(ENDIA_HIP_ERR_UNSUPPORTED, "col_reduce: extent too large");
  // A small input (the bias gradient of a narrow layer) is one launch: the second-stage kernel applied to the
  // input itself, 64 columns per group, the four waves taking alternate rows.
  int64_t S = 0, rows_per_split = 0;
  const bool vec_out = vec && al16(out) && inner == 0;  // (the one-launch kernel for mid-size inputs stores in place)
  col_reduce_plan(batch, R, C, ctx().cu_count, part ? part_floats : 0, vec_out, &S, &rows_per_split);
  if (S == 0 && !(R <= 1024 && batch * R * C <= (1 << 20))) {
    hipLaunchKernelGGL(col_reduce_mid_kernel, dim3((unsigned)ceil_div64(C, 16)), dim3(TPB), 0, s, x, out, R, C, scale);
    ENDIA_LAUNCH_CHECK();
    return rider ? col_reduce_with(1, rider->R, rider->C, rider->x, rider->out, 1.f, nullptr, 0) : ENDIA_HIP_OK;
  }
  if (S == 0) {
    last_stage(x, R);
    ENDIA_LAUNCH_CHECK();
    return rider && !ride ? col_reduce_with(1, rider->R, rider->C, rider->x, rider->out, 1.f, nullptr, 0) : ENDIA_HIP_OK;
  }
  if (S < 0) return fail(ENDIA_HIP_ERR_INVALID, "col_reduce: %lld columns do not fit the %lld floats of scratch", (long long)(batch * C), (long long)part_floats);
  if (!part) {
    void* ws = nullptr;
    int32_t rc = workspace(batch * S * C * (int64_t)sizeof(float), &ws);
    if (rc) return rc;
    part = static_cast<float*>(ws);
  }
  dim3 grid((unsigned)col_tiles, (unsigned)S, (unsigned)batch);
  if (vec) hipLaunchKernelGGL(col_reduce_vec_kernel, grid, dim3(TPB), 0, s, x, part, R, C, rows_per_split);
  else hipLaunchKernelGGL(col_reduce_scalar_kernel, grid, dim3(TPB), 0, s, x, part, R, C, rows_per_split);
  ENDIA_LAUNCH_CHECK();
  last_stage(part, S);
  ENDIA_LAUNCH_CHECK();
  return rider && !ride ? col_reduce_with(1, rider->R, rider->C, rider->x, rider->out, 1.f, nullptr, 0) : ENDIA_HIP_OK;
}

int32_t col_reduce(int64_t batch, int64_t R, int64_t C, const float* x, float* out, float scale) {
  return col_reduce_with(batch, R, C, x, out, scale, nullptr, 0);
}

// Whether col_reduce(1, R, C, x, out, ...) is the one launch of col_reduce_mid_kernel.
bool col_reduce_is_mid(int64_t R, int64_t C, const float* x, const float* out) {
  if (R < 1 || C < 1 || C >= (1ll << 31)) return false;
  const bool vec = (C % 4 == 0) && al16(x) && al16(out);
  int64_t S = 0, rows = 0;
  col_reduce_plan(1, R, C, ctx().cu_count, 0, vec, &S, &rows);
  return S == 0 && !(R <= 1024 && R * C <= (1 << 20));
}

// The same with the sums stored transposed: column c = o * inner + i goes to out[i * (C / inner) + o]. inner divides C.
int32_t col_reduce_transposed(int64_t R, int64_t C, int64_t inner, const float* x, float* out) {
  return col_reduce_with(1, R, C, x, out, 1.f, nullptr, 0, inner);
}

// col_reduce_transposed (inner > 0) or col_reduce (inner = 0) of x, and the plain column sums of x2 [R2][C2] into out2 as
// col_reduce(1, R2, C2, x2, out2, 1) gives them, in the same launch where x2 is small enough to need one stage only.
int32_t col_reduce_with_rider(int64_t R, int64_t C, int64_t inner, const float* x, float* out, int64_t R2, int64_t C2, const float* x2,
                              float* out2) {
  const ColSumRider rider{R2, C2, x2, out2};
  return col_reduce_with(1, R, C, x, out, 1.f, nullptr, 0, inner, &rider);
}

// out[r] = scale * sum_c x[r][c]
int32_t row_reduce(int64_t R, int64_t C, const float* x, float* out, float scale) {
  hipStream_t s = ctx().stream;
  if (R > 65535) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "row_reduce: more than 65535 rows");
  if (C <= 4096 && R * C <= (1 << 20)) {  // small input: one wave per row, one launch
    hipLaunchKernelGGL(row_reduce_final_kernel, dim3((unsigned)ceil_div64(R, 4)), dim3(TPB), 0, s, x, out, R, C, scale);
    ENDIA_LAUNCH_CHECK();
    return ENDIA_HIP_OK;
  }
  int64_t want = (int64_t)ctx().cu_count * 8;
  int64_t S = want / R;
  if (S < 1) S = 1;
  int64_t max_s = ceil_div64(C, 4096);
  if (S > max_s) S = max_s;
  int64_t chunk = ceil_div64(ceil_div64(C, S), 4) * 4;
  S = ceil_div64(C, chunk);
  const int vec = (C % 4 == 0) && al16(x);
  if (S == 1) {  // one group per row: its sum is the result, no second stage
    hipLaunchKernelGGL(row_reduce_kernel, dim3(1, (unsigned)R), dim3(TPB), 0, s, x, out, C, chunk, vec, scale);
    ENDIA_LAUNCH_CHECK();
    return ENDIA_HIP_OK;
  }
  void* ws = nullptr;
  int32_t rc = workspace(R * S * (int64_t)sizeof(float), &ws);
  if (rc) return rc;
  float* part = static_cast<float*>(ws);
  hipLaunchKernelGGL(row_reduce_kernel, dim3((unsigned)S, (unsigned)R), dim3(TPB), 0, s, x, part, C, chunk, vec, 1.f);
  ENDIA_LAUNCH_CHECK();
  hipLaunchKernelGGL(row_reduce_final_kernel, dim3((unsigned)ceil_div64(R, 4)), dim3(TPB), 0, s, part, out, R, S, scale);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

}  // namespace endia

using namespace endia;

extern "C" {

int32_t endia_hip_col_sum_plan(int64_t R, int64_t C, int64_t cu_count, int64_t scratch_floats, int32_t aligned16, int64_t* splits,
                               int64_t* rows_per_split) {
  ENDIA_CHECK_ARG(R >= 1 && C >= 1 && cu_count >= 1 && scratch_floats >= 0 && splits && rows_per_split,
                  "endia_hip_col_sum_plan: R, C, cu_count >= 1, scratch_floats >= 0 and non-null outputs");
  col_reduce_plan(1, R, C, cu_count, scratch_floats, aligned16 != 0 && C % 4 == 0, splits, rows_per_split);
  return ENDIA_HIP_OK;
}

int32_t endia_hip_reduce_add(int32_t ndim, const int64_t* shape, uint32_t reduce_mask, const float* x, float* out,
                             float scale, int32_t is_complex) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(ndim >= 0 && ndim <= 8, "endia_hip_reduce_add: ndim %d out of [0,8]", ndim);
  ENDIA_CHECK_ARG(ndim == 0 || shape, "endia_hip_reduce_add: null shape");
  ENDIA_CHECK_ARG(ndim == 8 ? true : (reduce_mask >> ndim) == 0, "endia_hip_reduce_add: mask 0x%x names an axis >= ndim", reduce_mask);
  ENDIA_CHECK_ARG(!(is_complex && ndim == 8), "endia_hip_reduce_add: complex needs ndim <= 7");
  // collapse neighbouring axes with the same status into groups; size-1 axes join either side
  int64_t gshape[9];
  int gred[9];
  int ng = 0;
  int64_t total = 1, nout = 1;
  for (int i = 0; i < ndim; ++i) {
    ENDIA_CHECK_ARG(shape[i] >= 0, "endia_hip_reduce_add: negative extent");
    total *= shape[i];
    int red = (reduce_mask >> i) & 1;
    if (!red) nout *= shape[i];
    if (shape[i] == 1) continue;
    if (ng && gred[ng - 1] == red) gshape[ng - 1] *= shape[i];
    else { gshape[ng] = shape[i]; gred[ng] = red; ++ng; }
  }
  if (is_complex) {  // trailing kept axis of the (re, im) pair
    if (ng && gred[ng - 1] == 0) gshape[ng - 1] *= 2;
    else { gshape[ng] = 2; gred[ng] = 0; ++ng; }
    nout *= 2;
  }
  if (nout == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(out != nullptr, "endia_hip_reduce_add: out is null");
  if (total == 0) return endia_hip_fill(out, nout, 0.f);  // empty sum
  ENDIA_CHECK_ARG(x != nullptr, "endia_hip_reduce_add: x is null");

  if (ng == 0) return endia_hip_axpby(1, scale, x, 0.f, nullptr, out);
  if (ng == 1 && !gred[0]) return endia_hip_axpby(gshape[0], scale, x, 0.f, nullptr, out);
  if (ng == 1 && gred[0]) return row_reduce(1, gshape[0], x, out, scale);
  if (ng == 2 && gred[0] && !gred[1]) return col_reduce(1, gshape[0], gshape[1], x, out, scale);
  if (ng == 2 && !gred[0] && gred[1] && gshape[0] <= 65535) return row_reduce(gshape[0], gshape[1], x, out, scale);
  if (ng == 3 && !gred[0] && gred[1] && !gred[2] && gshape[0] <= 65535)
    return col_reduce(gshape[0], gshape[1], gshape[2], x, out, scale);

  // everything else (e.g. N,C,H,W -> C): one work-group per output element
  RedDesc d;
  d.nk = d.nr = 0;
  int64_t st = 1, nred = 1;
  int64_t strides[9];
  for (int g = ng - 1; g >= 0; --g) { strides[g] = st; st *= gshape[g]; }
  for (int g = 0; g < ng; ++g) {
    if (gred[g]) { d.rshape[d.nr] = gshape[g]; d.rstride[d.nr] = strides[g]; ++d.nr; nred *= gshape[g]; }
    else { d.kshape[d.nk] = gshape[g]; d.kstride[d.nk] = strides[g]; ++d.nk; }
  }
  ENDIA_CHECK_ARG(nout <= 2147483647ll, "endia_hip_reduce_add: too many outputs for the general path");
  hipLaunchKernelGGL(generic_reduce_kernel, dim3((unsigned)nout), dim3(TPB), 0, ctx().stream, d, x, out, nred, scale);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_col_sum_multi(int32_t count, const endia_hip_col_sum_desc* members) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(count >= 0 && count <= 64 && (count == 0 || members), "endia_hip_col_sum_multi: count %d out of [0, 64] or null members", count);
  for (int i = 0; i < count; ++i) {
    const endia_hip_col_sum_desc& d = members[i];
    ENDIA_CHECK_ARG(d.R >= 0 && d.C >= 0, "endia_hip_col_sum_multi: member %d has a negative extent", i);
    ENDIA_CHECK_ARG(d.C == 0 || d.out, "endia_hip_col_sum_multi: member %d has no output", i);
    ENDIA_CHECK_ARG(d.R == 0 || d.C == 0 || d.x, "endia_hip_col_sum_multi: member %d has no input", i);
  }
  // members that the single call would run as its one-launch kernel share launches, up to kMaxSums at a time; the others
  // run as the single call runs them
  ColSumMembers a;
  a.count = 0;
  a.first[0] = 0;
  auto launch = [&]() -> int32_t {
    if (a.count == 0) return ENDIA_HIP_OK;
    if (a.count == 1) {
      hipLaunchKernelGGL(col_reduce_mid_kernel, dim3((unsigned)a.first[1]), dim3(TPB), 0, ctx().stream, a.x[0], a.out[0], a.R[0], a.C[0], a.scale[0]);
    } else {
      hipLaunchKernelGGL(col_reduce_mid_multi_kernel, dim3((unsigned)a.first[a.count]), dim3(TPB), 0, ctx().stream, a);
    }
    a.count = 0;
    ENDIA_LAUNCH_CHECK();
    return ENDIA_HIP_OK;
  };
  for (int i = 0; i < count; ++i) {
    const endia_hip_col_sum_desc& d = members[i];
    if (d.C == 0) continue;
    if (d.R == 0) {
      int32_t rc = endia_hip_fill(d.out, d.C, 0.f);
      if (rc) return rc;
      continue;
    }
    if (!col_reduce_is_mid(d.R, d.C, d.x, d.out)) {
      int32_t rc = col_reduce(1, d.R, d.C, d.x, d.out, d.scale);
      if (rc) return rc;
      continue;
    }
    const int64_t groups = ceil_div64(d.C, 16);
    if (a.count == kMaxSums || a.first[a.count] + groups > (1 << 30)) {
      int32_t rc = launch();
      if (rc) return rc;
    }
    const int m = a.count++;
    a.x[m] = d.x; a.out[m] = d.out; a.R[m] = d.R; a.C[m] = d.C; a.scale[m] = d.scale;
    a.first[m + 1] = a.first[m] + (int)groups;
  }
  return launch();
}

int32_t endia_hip_col_sum_static(int64_t R, int64_t C, const float* x, float* out, float scale) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(R >= 0 && C >= 0, "endia_hip_col_sum_static: negative extent (R=%lld C=%lld)", (long long)R, (long long)C);
  if (C == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(C <= kStaticScratchFloats, "endia_hip_col_sum_static: %lld columns exceed the maximum of %lld (the static scratch holds one row of partial sums per row split)",
                  (long long)C, (long long)kStaticScratchFloats);
  ENDIA_CHECK_ARG(out != nullptr, "endia_hip_col_sum_static: out is null");
  if (R == 0) return endia_hip_fill(out, C, 0.f);  // empty sum (a fill kernel: no allocation, safe to record)
  ENDIA_CHECK_ARG(x != nullptr, "endia_hip_col_sum_static: x is null");
  const int dev = ctx().device;
  float* part = (dev >= 0 && dev < kMaxDevices) ? g_scratch_ptr[dev] : nullptr;
  if (!part) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "endia_hip_col_sum_static: no static scratch was resolved for device %d", dev);
  return col_reduce_with(1, R, C, x, out, scale, part, kStaticScratchFloats);
}

int32_t endia_hip_reduce(int32_t op, int32_t ndim, const int64_t* shape, uint32_t reduce_mask, const float* x, float* out) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(op >= ENDIA_REDUCE_MAX && op <= ENDIA_REDUCE_ARGMIN, "endia_hip_reduce: unknown op %d", op);
  ENDIA_CHECK_ARG(ndim >= 0 && ndim <= 8, "endia_hip_reduce: ndim %d out of [0,8]", ndim);
  ENDIA_CHECK_ARG(ndim == 0 || shape, "endia_hip_reduce: null shape");
  ENDIA_CHECK_ARG(ndim == 8 ? true : (reduce_mask >> ndim) == 0, "endia_hip_reduce: mask 0x%x names an axis >= ndim", reduce_mask);
  const bool arg = op == ENDIA_REDUCE_ARGMAX || op == ENDIA_REDUCE_ARGMIN;
  ENDIA_CHECK_ARG(!arg || __builtin_popcount(reduce_mask) == 1, "endia_hip_reduce: argmax / argmin reduce exactly one axis");
  // neighbouring axes with the same status collapse into groups, as in endia_hip_reduce_add
  int64_t gshape[8];
  int gred[8];
  int ng = 0;
  int64_t total = 1, nout = 1;
  for (int i = 0; i < ndim; ++i) {
    ENDIA_CHECK_ARG(shape[i] >= 0, "endia_hip_reduce: negative extent");
    total *= shape[i];
    const int red = (reduce_mask >> i) & 1;
    if (!red) nout *= shape[i];
    if (shape[i] == 1) continue;
    if (ng && gred[ng - 1] == red) gshape[ng - 1] *= shape[i];
    else { gshape[ng] = shape[i]; gred[ng] = red; ++ng; }
  }
  if (nout == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(out != nullptr, "endia_hip_reduce: out is null");
  const float start = op == ENDIA_REDUCE_MUL ? 1.f : (arg ? -1.f : (op == ENDIA_REDUCE_MAX ? -INFINITY : INFINITY));
  if (total == 0) return endia_hip_fill(out, nout, start);
  ENDIA_CHECK_ARG(x != nullptr, "endia_hip_reduce: x is null");
  ENDIA_CHECK_ARG(nout <= 2147483647ll, "endia_hip_reduce: too many outputs");
  RedDesc d;
  d.nk = d.nr = 0;
  int64_t st = 1, nred = 1, strides[8];
  for (int g = ng - 1; g >= 0; --g) { strides[g] = st; st *= gshape[g]; }
  for (int g = 0; g < ng; ++g) {
    if (gred[g]) { d.rshape[d.nr] = gshape[g]; d.rstride[d.nr] = strides[g]; ++d.nr; nred *= gshape[g]; }
    else { d.kshape[d.nk] = gshape[g]; d.kstride[d.nk] = strides[g]; ++d.nk; }
  }
  const dim3 grid((unsigned)nout), block(TPB);
  hipStream_t s = ctx().stream;
  switch (op) {
    case ENDIA_REDUCE_MAX: hipLaunchKernelGGL((reduce_op_kernel<ENDIA_REDUCE_MAX>), grid, block, 0, s, d, x, out, nred); break;
    case ENDIA_REDUCE_MIN: hipLaunchKernelGGL((reduce_op_kernel<ENDIA_REDUCE_MIN>), grid, block, 0, s, d, x, out, nred); break;
    case ENDIA_REDUCE_MUL: hipLaunchKernelGGL((reduce_op_kernel<ENDIA_REDUCE_MUL>), grid, block, 0, s, d, x, out, nred); break;
    case ENDIA_REDUCE_ARGMAX: hipLaunchKernelGGL((reduce_op_kernel<ENDIA_REDUCE_ARGMAX>), grid, block, 0, s, d, x, out, nred); break;
    default: hipLaunchKernelGGL((reduce_op_kernel<ENDIA_REDUCE_ARGMIN>), grid, block, 0, s, d, x, out, nred); break;
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_mse_fwd_bwd(int64_t n, const float* pred, const float* target, float* loss, float* dpred) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n > 0, "endia_hip_mse_fwd_bwd: n must be positive (got %lld)", (long long)n);
  ENDIA_CHECK_ARG(pred && target, "endia_hip_mse_fwd_bwd: null input");
  ENDIA_CHECK_ARG(loss || dpred, "endia_hip_mse_fwd_bwd: nothing to compute");
  hipStream_t s = ctx().stream;
  const int vec = al16(pred) && al16(target) && (!dpred || al16(dpred));
  int64_t blocks = ceil_div64(vec ? (n + 3) / 4 : n, TPB);
  int64_t cap = (int64_t)ctx().cu_count * 8;
  if (blocks > cap) blocks = cap;
  float* part = nullptr;
  float part_scale = 1.f;
  const float inv_n = 1.0f / (float)n;
  if (loss && blocks == 1) {  // a single group: its sum is the loss, no second launch
    part = loss;
    part_scale = inv_n;
  } else if (loss) {
    void* ws = nullptr;
    int32_t rc = workspace(blocks * (int64_t)sizeof(float), &ws);
    if (rc) return rc;
    part = static_cast<float*>(ws);
  }
  hipLaunchKernelGGL(mse_kernel, dim3((unsigned)blocks), dim3(TPB), 0, s, pred, target, dpred, part, n, 2.0f * inv_n, vec, part_scale);
  ENDIA_LAUNCH_CHECK();
  if (loss && blocks > 1) {
    hipLaunchKernelGGL(sum_partials_kernel, dim3(1), dim3(TPB), 0, s, part, loss, blocks, inv_n);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}

}  // extern "C"
