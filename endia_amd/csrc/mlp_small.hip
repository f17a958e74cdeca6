// A whole small dense model per launch: nn.MLP.forward (endia/nn/modules/_mlp.mojo:47-53) and its backward pass.
//
// The reference's own benchmark model (benchmarks/mlp_benchmarks/mlp_imp.mojo:35-75: widths 1-32-64-128-128-128-64-32-1,
// batch 128) is eight products of a few hundred kilo-flops each. One kernel per layer makes a training step a chain of
// ~19 dependent launches whose cost is the launches. But every row of the batch is independent through all layers, in
// the forward pass and in the chain of cotangents alike, so for layers of at most 128 units a work-group owns a few
// rows of the batch and runs ALL layers back to back: activations stay in LDS, the weights (a few tens of KiB,
// resident in L2) go straight from memory into MFMA operands, the next layer's while the current layer computes.
//   mlp_fwd4_kernel / mlp_delta4_kernel   FOUR rows per work-group on v_mfma_f32_4x4x1_16b_f32, for batches of up to
//                     2048 rows (the reference's 128 rows are 32 work-groups); every weight request covers whole
//                     128-byte lines;
//   mlp_fwd_kernel / mlp_delta_kernel     sixteen rows per work-group on v_mfma_f32_16x16x4_f32, beyond;
//   mlp_wgrad_kernel  dW_l = h_{l-1}^T delta_l and db_l = 1^T delta_l for ALL layers in one launch, a work-group per
//                     32 x 32 tile of a gradient on v_mfma_f32_32x32x2_f32, a fixed order of summation (results
//                     repeat bit for bit).
// No work-group ever waits for another (the forward launch with the MSE loss on top meets at a ticket at its end).
//
// What the measurements behind these kernels say about this machine: a wave's request is delivered at 64 bytes a clock
// when its lanes cover whole 128-byte lines and at a quarter of that when they cover 64-byte pieces of many lines;
// a width test around a request or an MFMA makes the compiler wait for memory between requests, or copy accumulators
// around branches, so runs of requests and of MFMAs are kept straight.
//
// MFMA 16x16x4: A is 16 x 4 (lane: row = lane % 16, k = lane / 16), B is 4 x 16 (lane: column = lane % 16, k = lane / 16),
// the accumulator holds rows 4 * (lane / 16) + v, v = 0..3, of column lane % 16. A sum over k may be taken in any
// order: "super-step" t of a reduction uses k = 16 t + 4 g + i (g = lane / 16) in its MFMA i = 0..3, so that a lane's
// four A values are one 16-byte LDS read.
#include "common.h"
#include "mfma_tile.h"
#include "ticket.h"

namespace {

using mfma::buffer_load_f1;
using mfma::buffer_load_f4;
using mfma::make_rsrc;
using mfma::OOB_OFFSET;

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int ROWS = 16;        // rows of the batch per work-group of the sixteen-row kernels
constexpr int MAXW = ENDIA_MLP_MAX_WIDTH;
constexpr int LD = MAXW + 4;    // LDS row stride: 16 rows x 16-byte reads fall into distinct banks
constexpr int MAXT = MAXW / 16; // super-steps of a full-width reduction
constexpr int NW = 8;             // waves per work-group of the two row-block kernels (4 were measured slower: 22 -> 16 us for the chain of cotangents)
constexpr int SLOTS = MAXW / 16 / NW;  // 16-column blocks per wave

struct MlpArgs {
  int layers, act, batch;
  int width[ENDIA_MLP_MAX_LAYERS + 1];
  const float* W[ENDIA_MLP_MAX_LAYERS];
  const float* b[ENDIA_MLP_MAX_LAYERS];
  float* h[ENDIA_MLP_MAX_LAYERS];      // forward: outputs; backward: the stored activations
  float* delta[ENDIA_MLP_MAX_LAYERS];  // backward: cotangents of the pre-activations (delta[layers - 1] is the incoming one)
  float* dW[ENDIA_MLP_MAX_LAYERS];
  float* db[ENDIA_MLP_MAX_LAYERS];
  const float* x;
  float* dx;
  int tile0[ENDIA_MLP_MAX_LAYERS + 1];  // weight gradients: first 32 x 32 tile of every layer in the launch's grid
  // weight gradients of a large batch: the launch's grid.y slices of rows_per_slice rows leave their sums in wpart
  // ([slice][woff[layers]] floats; layer l: dW at woff[l], db behind it), which a second launch adds up in slice order
  float* wpart;
  int woff[ENDIA_MLP_MAX_LAYERS + 1];
  int rows_per_slice;
  // forward with the MSE loss on top (target != null): d loss / d output = 2 (out - target) / n goes to dpred, every
  // work-group leaves its sum of squared differences in loss_part and the last one to arrive adds them up, in row order
  const float* target;
  float* dpred;
  float* loss;
  float* loss_part;
  unsigned* ticket;
  float inv_n;
  int chain;  // forward with the MSE loss: also run the chain of cotangents from the loss gradient (delta, dx as in the backward pass)
};

__device__ __forceinline__ float act_apply(int act, float z) {
  return act == ENDIA_OP_RELU ? (z > 0.f ? z : 0.f) : (act == ENDIA_OP_TANH ? tanhf(z) : z);
}
// derivative from the stored OUTPUT h = act(z): relu' = [h > 0] (relu_op.mojo:95: z > 0 iff h > 0), tanh' = 1 - h^2 (tanh_op.mojo:92)
__device__ __forceinline__ float act_slope(int act, float h) {
  return act == ENDIA_OP_RELU ? (h > 0.f ? 1.f : 0.f) : (act == ENDIA_OP_TANH ? 1.f - h * h : 1.f);
}

// B operands of one layer for this wave: element [t][s][i] multiplies k = 16 t + 4 g + i into column 16 (wave + 4 s) + c.
// TRANSPOSED reads W^T: the reduction runs over W's columns and the output column is W's row.
struct WFrag {
  float v[MAXT][SLOTS][4];
};

// Loader of one layer's B operands. Every load is a buffer load whose offset is out of range where the element does
// not exist (it then reads as zero): no branch and no wait sits between two loads, so a layer's 16 to 64 requests per
// lane are all in flight together, and they are issued one super-step at a time between the MFMAs of the layer that is
// being computed. Per request the lane's offset costs at most one addition: the lane-dependent part is fixed per layer.
// The transposed form reads four consecutive floats of a row of W per request when rows are whole 16-byte pieces.
template <bool TRANSPOSED>
struct WLoader {
  __amdgpu_buffer_rsrc_t rs;
  uint32_t voff[SLOTS], voff_tail[SLOTS];
  int red, N, g4;
  bool vec, any;
  // plain: out = in[., K] W[K, N]: reduction index k < K, column n < N.  transposed: out = in[., N] W^T: reduction n < N, column k < K.
  __device__ __forceinline__ void init(const float* __restrict__ W, int K, int N_, int wave, int c, int g) {
    any = W != nullptr;
    N = N_;
    g4 = 4 * g;
    red = TRANSPOSED ? N : K;
    const int cols = TRANSPOSED ? K : N;
    rs = make_rsrc(W, any ? (int64_t)K * N * 4 : 0);
    vec = TRANSPOSED && (N & 3) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const int col = 16 * (wave + NW * s) + c;
      // rows of the plain form past K lie past the end of the buffer; the transposed form would run into the next
      // row of W instead, so its last, partial super-step has offsets of its own
      voff[s] = col < cols ? (uint32_t)((TRANSPOSED ? col * N + 4 * g : 4 * g * N + col) * 4) : OOB_OFFSET;
      voff_tail[s] = 4 * g < (N & 15) ? voff[s] : OOB_OFFSET;
    }
  }
  __device__ __forceinline__ void load_step(WFrag& f, int t) const {
    if (!any || 16 * t >= red) return;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      if (!TRANSPOSED) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f.v[t][s][i] = buffer_load_f1(rs, voff[s] + (uint32_t)((16 * t + i) * N * 4));
      } else if (vec) {
        const float4 w = buffer_load_f4(rs, (16 * t + 16 <= N ? voff[s] : voff_tail[s]) + (uint32_t)(64 * t));
        f.v[t][s][0] = w.x; f.v[t][s][1] = w.y; f.v[t][s][2] = w.z; f.v[t][s][3] = w.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // rows of W that are not whole 16-byte pieces: element by element, the tail tested per lane
          f.v[t][s][i] = buffer_load_f1(rs, 16 * t + i + g4 < N ? voff[s] + (uint32_t)((16 * t + i) * 4) : OOB_OFFSET);
        }
      }
    }
  }
};

// acc[s] = in[16 x red] (LDS) . cur, for the wave's column blocks; between the super-steps, the requests for `nxt`
template <bool TRANSPOSED>
__device__ __forceinline__ void layer_mfma(const float* __restrict__ in, const WFrag& cur, int red, int cols, int wave, int c, int g,
                                           floatx4 (&acc)[SLOTS], const WLoader<TRANSPOSED>& next, WFrag& nxt) {
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) acc[s] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < MAXT; ++t) {
    next.load_step(nxt, t);
    if (16 * t < red) {
      const float4 a = *reinterpret_cast<const float4*>(&in[c * LD + 16 * t + 4 * g]);
      const float av[4] = {a.x, a.y, a.z, a.w};
      // (four MFMAs in a row into the same accumulator: measured twice as fast as alternating between the column blocks)
#pragma unroll
      for (int s = 0; s < SLOTS; ++s)
        if (16 * (wave + NW * s) < cols) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[s] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], cur.v[t][s][i], acc[s], 0, 0, 0);
        }
    }
  }
}

// Stage 16 rows of a [batch, width] array into LDS, zero beyond the array's rows and up to the next multiple of 16
// columns (a reduction reads whole super-steps of 16; everything else in LDS is written before it is read).
__device__ __forceinline__ void stage_rows(float* __restrict__ dst, const float* __restrict__ src, int row0, int batch, int width, int tid) {
  const int padded = (width + 15) & ~15;
  for (int e = tid; e < ROWS * padded; e += 64 * NW) {
    const int r = e / padded, k = e - r * padded;
    dst[r * LD + k] = (row0 + r < batch && k < width) ? src[(int64_t)(row0 + r) * width + k] : 0.f;
  }
}

// Forward layers whose rows of W are whole 16-byte pieces read W sixteen bytes per lane: a wave owns 64 consecutive
// output columns as four MFMA blocks whose column c is output column 4 c + j (j = block), so that a lane's four B values
// of one reduction index are four neighbouring floats of a row of W, and a request of the wave covers whole rows (1 KiB)
// instead of sixteen floats of each of four rows. The NW waves share the two column groups of a layer and split its
// reduction: wave w takes group w % groups and the super-steps t = w / groups (mod NW / groups); the partial sums meet
// in LDS, where bias and activation are applied. (Other layers, e.g. a 1-wide last one, take the plan of WLoader.)
struct VFrag {
  float4 b[2][4];  // [u][i]: super-step t = q + parts * u, reduction index 16 t + 4 g + i
};
constexpr int PLD = MAXW + 4;  // row stride of the partial sums

struct VPlan {
  __amdgpu_buffer_rsrc_t rs;
  uint32_t voff;
  int K, N, G, q, parts;
  bool vec;
  __device__ __forceinline__ void init(const float* __restrict__ W, int K_, int N_, int wave, int c, int g) {
    K = K_;
    N = N_;
    vec = W != nullptr && (N & 3) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;
    const int groups = (N + 63) / 64;
    parts = NW / groups;
    G = wave % groups;
    q = wave / groups;
    rs = make_rsrc(W, vec ? (int64_t)K * N * 4 : 0);
    const int col = 64 * G + 4 * c;
    voff = col < N ? (uint32_t)((4 * g * N + col) * 4) : OOB_OFFSET;  // rows past K lie past the end of the buffer
  }
  __device__ __forceinline__ void request(VFrag& f) const {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int t = q + parts * u;
      if (16 * t < K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f.b[u][i] = buffer_load_f4(rs, voff + (uint32_t)((16 * t + i) * N * 4));
      }
    }
  }
};

__global__ __launch_bounds__(64 * NW, 1) void mlp_fwd_kernel(MlpArgs p) {
  static_assert(NW == 8 && SLOTS == 1 && MAXW == 128, "the reduction split below is written for eight waves and two column groups");
  __shared__ __attribute__((aligned(16))) float hs[2][ROWS * LD];
  __shared__ __attribute__((aligned(16))) float part[NW * ROWS * PLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, g = lane >> 4;
  const int row0 = blockIdx.x * ROWS;
  WFrag cur_s, nxt_s;
  VFrag cur_v, nxt_v;
  WLoader<false> loader;
  VPlan plan, plan_next;
  // what a thread adds when the partial sums meet: four neighbouring bias values (16-byte layers) or its block's one
  float4 bias4_cur, bias4_nxt;
  float bias1_cur, bias1_nxt;
  const int er = tid >> 5, en = (tid & 31) * 4;  // the four outputs a thread finishes in a 16-byte layer: row er, columns en .. en + 3
  auto request_layer = [&](int l, VPlan& pl, VFrag& fv, WFrag& fs, float4& b4, float& b1) {
    pl.init(p.W[l], p.width[l], p.width[l + 1], wave, c, g);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b[l], (int64_t)p.width[l + 1] * 4);
    if (pl.vec) {
      pl.request(fv);
      b4 = buffer_load_f4(rb, (uint32_t)(en * 4));  // (columns past the width read as zero and are never stored)
    } else {
      loader.init(p.W[l], p.width[l], p.width[l + 1], wave, c, g);
#pragma unroll
      for (int t = 0; t < MAXT; ++t) loader.load_step(fs, t);
      b1 = buffer_load_f1(rb, (uint32_t)((16 * wave + c) * 4));
    }
  };
  request_layer(0, plan, cur_v, cur_s, bias4_cur, bias1_cur);  // the first layer's weights travel while the input is staged
  stage_rows(hs[0], p.x, row0, p.batch, p.width[0], tid);
  __syncthreads();
  for (int l = 0; l < p.layers; ++l) {
    const int K = p.width[l], N = p.width[l + 1];
    const bool last = l + 1 == p.layers;
    if (!last) request_layer(l + 1, plan_next, nxt_v, nxt_s, bias4_nxt, bias1_nxt);  // travels while this layer computes
    const float* in = hs[l & 1];
    float* out = hs[(l & 1) ^ 1];
    if (plan.vec) {
      floatx4 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int t = plan.q + plan.parts * u;
        if (16 * t < K) {
          const float4 a = *reinterpret_cast<const float4*>(&in[c * LD + 16 * t + 4 * g]);
          const float av[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float bj = j == 0 ? cur_v.b[u][i].x : (j == 1 ? cur_v.b[u][i].y : (j == 2 ? cur_v.b[u][i].z : cur_v.b[u][i].w));
              acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bj, acc[j], 0, 0, 0);
            }
        }
      }
      if (64 * plan.G < N) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
          *reinterpret_cast<float4*>(&part[(plan.q * ROWS + 4 * g + v) * PLD + 64 * plan.G + 4 * c]) =
              make_float4(acc[0][v], acc[1][v], acc[2][v], acc[3][v]);
      }
      __syncthreads();
      const int npad = (N + 15) & ~15;
      if (en < npad) {
        float4 z = bias4_cur;
        for (int qq = 0; qq < plan.parts; ++qq) {  // partial sums in the order of their reduction ranges
          const float4 t4 = *reinterpret_cast<const float4*>(&part[(qq * ROWS + er) * PLD + en]);
          z.x += t4.x; z.y += t4.y; z.z += t4.z; z.w += t4.w;
        }
        if (!last) {
          z.x = act_apply(p.act, z.x); z.y = act_apply(p.act, z.y); z.z = act_apply(p.act, z.z); z.w = act_apply(p.act, z.w);
        }
        if (en >= N) z = make_float4(0.f, 0.f, 0.f, 0.f);  // columns past the width feed the next reduction as zeros
        *reinterpret_cast<float4*>(&out[er * LD + en]) = z;
        if (en < N && row0 + er < p.batch) *reinterpret_cast<float4*>(&p.h[l][(int64_t)(row0 + er) * N + en]) = z;
      }
    } else {
      floatx4 acc[SLOTS];
      WLoader<false> none;
      none.init(nullptr, 1, 1, wave, c, g);
      layer_mfma<false>(in, cur_s, K, N, wave, c, g, acc, none, nxt_s);
      const int col = 16 * wave + c;
      if (16 * wave < N) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int r = 4 * g + v;
          float z = acc[0][v] + bias1_cur;
          if (!last) z = act_apply(p.act, z);
          if (col >= N) z = 0.f;  // the block's columns past the layer's width feed the next reduction as zeros
          out[r * LD + col] = z;
          if (col < N && row0 + r < p.batch) p.h[l][(int64_t)(row0 + r) * N + col] = z;
        }
      }
    }
    __syncthreads();
    if (!last) {  // (the requests above have had the whole layer to arrive)
      plan = plan_next;
      cur_v = nxt_v;
      cur_s = nxt_s;
      bias4_cur = bias4_nxt;
      bias1_cur = bias1_nxt;
    }
  }
  if (p.target) {  // mse = sum((out - target)^2) / n (mse_op.mojo:17-20) and its gradient; the outputs of these rows are still in LDS
    __shared__ float red[NW];
    const int L = p.layers, N = p.width[L], npad = (N + 15) & ~15;
    const float* out = hs[L & 1];
    const float two_over_n = 2.0f * p.inv_n;
    float acc = 0.f;
    for (int e = tid; e < ROWS * npad; e += 64 * NW) {
      const int r = e / npad, col = e - r * npad;
      if (row0 + r < p.batch && col < N) {
        const int64_t at = (int64_t)(row0 + r) * N + col;
        const float d = out[r * LD + col] - p.target[at];
        acc += d * d;
        if (p.dpred) p.dpred[at] = d * two_over_n;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
    if (lane == 0) red[wave] = acc;
    __syncthreads();
    if (tid == 0) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) sum += red[w];
      endia::store_shared(&p.loss_part[blockIdx.x], sum);
    }
    if (endia::arrive_last(p.ticket, gridDim.x, reinterpret_cast<int*>(part)) && tid == 0) {
      float sum = 0.f;
      for (unsigned i = 0; i < gridDim.x; ++i) sum += endia::load_shared(&p.loss_part[i]);
      p.loss[0] = sum * p.inv_n;
    }
  }
}

// delta[layers - 1] holds the incoming cotangent (the last layer has no activation). For l = layers - 1 .. 1:
// delta[l - 1] = (delta[l] W_l^T) * act'(h[l - 1]); finally dx = delta[0] W_0^T when asked for.
__global__ __launch_bounds__(64 * NW, 1) void mlp_delta_kernel(MlpArgs p) {
  __shared__ __attribute__((aligned(16))) float ds[2][ROWS * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, g = lane >> 4;
  const int row0 = blockIdx.x * ROWS;
  const int L = p.layers;
  const int first = p.dx ? 0 : 1;  // lowest layer whose W^T is applied
  if (L - 1 < first) return;
  WFrag cur, nxt;
  WLoader<true> loader;
  loader.init(p.W[L - 1], p.width[L - 1], p.width[L], wave, c, g);
#pragma unroll
  for (int t = 0; t < MAXT; ++t) loader.load_step(cur, t);
  stage_rows(ds[0], p.delta[L - 1], row0, p.batch, p.width[L], tid);
  __syncthreads();
  int buf = 0;
  for (int l = L - 1; l >= first; --l) {
    const int K = p.width[l], N = p.width[l + 1];  // W_l is K x N; the product is [rows, N] . [N, K]
    const bool more = l - 1 >= first;
    loader.init(more ? p.W[l - 1] : nullptr, more ? p.width[l - 1] : 1, p.width[l], wave, c, g);
    // outputs of the activation that produced this layer's input (none below the first layer)
    float hprev[SLOTS][4];
    const __amdgpu_buffer_rsrc_t rh = make_rsrc(l > 0 ? p.h[l - 1] : p.x, l > 0 ? (int64_t)p.batch * K * 4 : 0);
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int col = 16 * (wave + NW * s) + c, r = row0 + 4 * g + v;
        hprev[s][v] = buffer_load_f1(rh, (l > 0 && col < K && r < p.batch) ? (uint32_t)((r * K + col) * 4) : OOB_OFFSET);
      }
    floatx4 acc[SLOTS];
    layer_mfma<true>(ds[buf], cur, N, K, wave, c, g, acc, loader, nxt);
    float* out = ds[buf ^ 1];
    float* dst = l > 0 ? p.delta[l - 1] : p.dx;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const int col = 16 * (wave + NW * s) + c;
      if (16 * (wave + NW * s) < K) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int r = 4 * g + v;
          float d = col < K ? acc[s][v] * (l > 0 ? act_slope(p.act, hprev[s][v]) : 1.f) : 0.f;
          out[r * LD + col] = d;
          if (col < K && row0 + r < p.batch) dst[(int64_t)(row0 + r) * K + col] = d;
        }
      }
    }
    __syncthreads();
    buf ^= 1;
    if (more) cur = nxt;
  }
}

// ---- row-block kernels on v_mfma_f32_4x4x1_16b_f32 ---------------------------------------------------------------
// The instruction computes sixteen independent 4 x 4 outer products: block B = lane / 4 takes its four A values from
// the lanes 4 B + i (rows) and its four B values from the lanes 4 B + j (columns) and adds A[i] * B[j] to register i of
// lane 4 B + j (checked against the hardware with distinct values in every lane). It runs at the rate of the 16 x 16 x 4
// form (256 multiply-adds in 8 cycles, measured) but its left operand is 4 rows, not 16, so a work-group can own FOUR
// rows of the batch without idle MFMA rows: the reference's model at batch 128 becomes 32 work-groups instead of 8,
// each with a quarter of the MFMA work per layer. What the sixteen blocks stand for differs between the two kernels:
// it is chosen so that a wave's weight requests cover whole 128-byte lines (see each kernel).
constexpr int LD4 = MAXW + 16;  // LDS row stride = 16 (mod 64): 16-byte reads of the rows i = 0..3 start 16 banks apart

// v + (v rotated right by N lanes within each row of 16 lanes)
template <int CTRL>
__device__ __forceinline__ float row_ror_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// the sum over four lanes 4 apart within a row of 16, left in all four of them
__device__ __forceinline__ float sum_slices(float v) { return row_ror_add<0x124>(row_ror_add<0x128>(v)); }

__device__ __forceinline__ float pick(const floatx4& a, int i) { return i == 0 ? a[0] : (i == 1 ? a[1] : (i == 2 ? a[2] : a[3])); }

template <int RQ>
__device__ __forceinline__ void stage_rows4(float* __restrict__ dst, const float* __restrict__ src, int row0, int batch, int width, int tid,
                                            int pad = 16) {
  const int padded = (width + pad - 1) & ~(pad - 1);  // zeros up to the reduction's step
  for (int e = tid; e < 4 * RQ * padded; e += 64 * NW) {
    const int r = e / padded, k = e - r * padded;
    dst[r * LD4 + k] = (row0 + r < batch && k < width) ? src[(int64_t)(row0 + r) * width + k] : 0.f;
  }
}

// Everything a layer consumes from memory is requested one layer ahead, and a layer's outputs are stored one layer
// later, from registers. Each layer begins by waiting for ALL outstanding memory operations: the compiler then knows
// that the operands at hand have arrived and places no wait of its own further down (left to count the requests that
// sit under the width tests, it waits for the NEXT layer's weights ahead of the current layer's MFMAs).
__device__ __forceinline__ void wait_vm_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0), other counters untouched

// delta[layers - 1] holds the incoming cotangent (the last layer has no activation). For l = layers - 1 .. 1:
// delta[l - 1] = (delta[l] W_l^T) * act'(h[l - 1]); finally dx = delta[0] W_0^T when asked for.
//
// Here the reduction runs along the rows of W, so a wave owns 16 output columns = 16 rows of W_l for the whole
// reduction, and a lane's B operands are 16-byte pieces of one row. For a request to cover whole 128-byte lines, eight
// lanes must sit side by side in a row of W: the sixteen blocks of an MFMA are 8 slices of the reduction (s) x 2 column
// quads (cq), MFMA (T, e) multiplies reduction index 32 T + 4 s + e, and the wave's sixteen columns take two passes of
// eight that share the left operand. A request then reads 128 consecutive bytes of each of eight rows. The eight
// slices are added with two row rotations and one swap of the wave's halves; afterwards lane (cq, s, j) finishes row
// s % 4 of column 16 wave + 8 (s / 4) + 4 cq + j.
struct FragD {
  float v[2][MAXW / 32][4];  // [pass][T][e]: W[16 wave + 8 pass + 4 cq + j][32 T + 4 s + e]
  float slope[4];            // the stored activations at the lane's outputs, per row quad
};

// the sum over the eight slices: lanes 4 and 8 apart within a row of 16, and the wave's other half
__device__ __forceinline__ float sum_slices8(float v) {
  v = sum_slices(v);
  typedef unsigned uint2v __attribute__((ext_vector_type(2)));
  const unsigned u = __float_as_uint(v);
  const uint2v r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // {[lo | lo], [hi | hi]} of the two halves
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int RQ, int NT>
__device__ __forceinline__ void rows_mfma(const float* __restrict__ in, const FragD& w, int s, int j, floatx4 (&out)[RQ][2]) {
  floatx4 acc[RQ][2];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) acc[rq][0] = acc[rq][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int T = 0; T < NT; ++T) {
    float av[RQ][4];
#pragma unroll
    for (int rq = 0; rq < RQ; ++rq) {
      const float4 a = *reinterpret_cast<const float4*>(&in[(4 * rq + j) * LD4 + 32 * T + 4 * s]);
      av[rq][0] = a.x; av[rq][1] = a.y; av[rq][2] = a.z; av[rq][3] = a.w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int pass = 0; pass < 2; ++pass)
#pragma unroll
        for (int rq = 0; rq < RQ; ++rq) acc[rq][pass] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[rq][e], w.v[pass][T][e], acc[rq][pass], 0, 0, 0);
  }
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq)
#pragma unroll
    for (int pass = 0; pass < 2; ++pass)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[rq][pass][i] = sum_slices8(acc[rq][pass][i]);
}

// The chain of cotangents for the four-row kernels. `ds`: two LDS row blocks; ds[0] receives delta[layers - 1] of
// this group's rows from stage() (zeros up to the next multiple of 32 columns), which runs after the first weights
// have been asked for. LDS_ACTS: the stored activations come from `acts` (acts[l] = the input of layer l, LDS row
// blocks left there by the forward pass of the same launch) instead of from memory.
template <int RQ, bool LDS_ACTS, class Stage>
__device__ __forceinline__ void delta_chain(const MlpArgs& p, float (*ds)[4 * RQ * LD4], const float (*acts)[4 * RQ * LD4], int row0, Stage stage) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 3, cq = (lane >> 4) & 1;
  const int s = ((lane >> 2) & 3) | ((lane >> 5) << 2);
  const int wrow = 4 * cq + j;                             // + 8 pass: the lane's rows of W within the wave's sixteen
  const int ocol = 16 * wave + 8 * (s >> 2) + wrow, orow = s & 3;  // the output this lane finishes, per row quad
  const int L = p.layers;
  const int first = p.dx ? 0 : 1;  // lowest layer whose W^T is applied
  if (L - 1 < first) {
    stage();
    return;
  }
  // (a wave is at work while its columns begin below the width rounded up to 32: the next reduction reads that far)
  auto active = [&](int K) { return 16 * wave < ((K + 31) & ~31); };
  auto request = [&](int l, FragD& f) {
    const int K = p.width[l], N = p.width[l + 1];
    if (!active(K)) return;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.W[l], (int64_t)K * N * 4);
    const bool vec = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(p.W[l]) & 15) == 0;
    // (no width test around a request: with one, the compiler can no longer tell which registers have a request
    // outstanding and waits for memory between any two of them; a request past the width costs next to nothing)
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int c = 16 * wave + 8 * pass + wrow;
      const uint32_t base = (uint32_t)((c * N + 4 * s) * 4);
#pragma unroll
      for (int T = 0; T < MAXW / 32; ++T) {
        if (32 * T >= N) continue;
        const int n0 = 32 * T + 4 * s;
        if (vec) {
          const float4 w = buffer_load_f4(rs, (c < K && n0 < N) ? base + (uint32_t)(128 * T) : OOB_OFFSET);
          f.v[pass][T][0] = w.x; f.v[pass][T][1] = w.y; f.v[pass][T][2] = w.z; f.v[pass][T][3] = w.w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) f.v[pass][T][e] = buffer_load_f1(rs, (c < K && n0 + e < N) ? base + (uint32_t)((32 * T + e) * 4) : OOB_OFFSET);
        }
      }
    }
    // the outputs of the activation that produced this layer's input (none below the first layer)
    if (LDS_ACTS) {
#pragma unroll
      for (int rq = 0; rq < RQ; ++rq) f.slope[rq] = l > 0 ? acts[l][(4 * rq + orow) * LD4 + ocol] : 1.f;
    } else {
      const __amdgpu_buffer_rsrc_t rh = make_rsrc(l > 0 ? p.h[l - 1] : p.x, l > 0 ? (int64_t)p.batch * K * 4 : 0);
#pragma unroll
      for (int rq = 0; rq < RQ; ++rq) {
        const int r = row0 + 4 * rq + orow;
        f.slope[rq] = buffer_load_f1(rh, (l > 0 && ocol < K && r < p.batch) ? (uint32_t)((r * K + ocol) * 4) : OOB_OFFSET);
      }
    }
  };
  float d[RQ];  // the outputs this lane finished in the last layer
  auto store = [&](int l) {  // outputs of layer l: delta[l - 1], or dx
    const int K = p.width[l];
    float* dst = l > 0 ? p.delta[l - 1] : p.dx;
    if (ocol < K) {
#pragma unroll
      for (int rq = 0; rq < RQ; ++rq) {
        const int r = row0 + 4 * rq + orow;
        if (r < p.batch) dst[(int64_t)r * K + ocol] = d[rq];
      }
    }
  };
  int buf = 0;
  auto layer = [&](int l, const FragD& cur, FragD& nxt) {
    const int K = p.width[l], N = p.width[l + 1];
    wait_vm_all();
    if (l - 1 >= first) request(l - 1, nxt);
    if (l < L - 1) store(l + 1);
    if (active(K)) {
      floatx4 acc[RQ][2];
      switch ((N + 31) >> 5) {
        case 1: rows_mfma<RQ, 1>(ds[buf], cur, s, j, acc); break;
        case 2: rows_mfma<RQ, 2>(ds[buf], cur, s, j, acc); break;
        case 3: rows_mfma<RQ, 3>(ds[buf], cur, s, j, acc); break;
        default: rows_mfma<RQ, 4>(ds[buf], cur, s, j, acc); break;
      }
      float* out = ds[buf ^ 1];
#pragma unroll
      for (int rq = 0; rq < RQ; ++rq) {
        const float v = s < 4 ? pick(acc[rq][0], orow) : pick(acc[rq][1], orow);
        d[rq] = ocol < K ? v * (l > 0 ? act_slope(p.act, cur.slope[rq]) : 1.f) : 0.f;  // columns past the width feed the next reduction as zeros
        out[(4 * rq + orow) * LD4 + ocol] = d[rq];
      }
    }
    __syncthreads();
    buf ^= 1;
  };
  FragD wa, wb;
  request(L - 1, wa);
  stage();
  __syncthreads();
  int l = L - 1;
  for (; l >= first; l -= 2) {
    layer(l, wa, wb);
    if (l - 1 >= first) layer(l - 1, wb, wa);
  }
  store(first);
}

__global__ __launch_bounds__(64 * NW, 1) void mlp_delta4_kernel(MlpArgs p) {
  constexpr int RQ = 1;  // row quads per work-group, as in the forward kernel
  __shared__ __attribute__((aligned(16))) float ds[2][4 * RQ * LD4];
  const int row0 = blockIdx.x * 4 * RQ;
  delta_chain<RQ, false>(p, ds, nullptr, row0, [&]() { stage_rows4<RQ>(ds[0], p.delta[p.layers - 1], row0, p.batch, p.width[p.layers], threadIdx.x, 32); });
}

// Forward pass. A request of a wave must cover whole 128-byte lines to be delivered at the CU's full rate (four times
// the rate of 64-byte pieces, measured), and rows of W run along the OUTPUT columns. So here a wave owns sixteen rows
// of W (reduction indices 16 wave .. 16 wave + 15) and all columns: the sixteen blocks of an MFMA are sixteen column
// quads (lane = column within a half of 64), the left operand is the same in all blocks, and a request reads 256
// consecutive bytes of one row. The eight waves' partial sums (4 RQ x 128 floats each) meet in LDS, where thread t
// finishes column t % 128 of row t / 128 (+ 4 per further row quad): bias, activation, LDS, and the global store one
// layer later.
struct FragF {
  float v[16][2];  // [kk][half]: W[16 wave + kk][64 half + lane]
  float bias;
};

// The MFMAs of one wave for one layer: its sixteen reduction indices times HALVES column halves, and the partial sums
// to LDS. Within an active wave all sixteen indices are in order: the input's columns are zero up to the next multiple
// of 16 and rows of W past the last read as zero.
template <int RQ, int HALVES>
__device__ __forceinline__ void slab_mfma(const float* __restrict__ in, const FragF& w, int wave, int lane, float (*part)[MAXW]) {
  const int j = lane & 3;
  floatx4 acc[RQ][HALVES];
  float a[RQ][16];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
#pragma unroll
    for (int h = 0; h < HALVES; ++h) acc[rq][h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 t = *reinterpret_cast<const float4*>(&in[(4 * rq + j) * LD4 + 16 * wave + 4 * q]);
      a[rq][4 * q] = t.x; a[rq][4 * q + 1] = t.y; a[rq][4 * q + 2] = t.z; a[rq][4 * q + 3] = t.w;
    }
  }
#pragma unroll
  for (int kk = 0; kk < 16; ++kk)
#pragma unroll
    for (int h = 0; h < HALVES; ++h)
#pragma unroll
      for (int rq = 0; rq < RQ; ++rq) acc[rq][h] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[rq][kk], w.v[kk][h], acc[rq][h], 0, 0, 0);
#pragma unroll
  for (int h = 0; h < HALVES; ++h)
#pragma unroll
    for (int rq = 0; rq < RQ; ++rq)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[4 * rq + i][64 * h + lane] = acc[rq][h][i];
}

__global__ __launch_bounds__(64 * NW, 1) void mlp_fwd4_kernel(MlpArgs p) {
  constexpr int RQ = 1;  // row quads per work-group (more were measured slower than the sixteen-row kernel at the batches where they would apply)
  static_assert(NW * 16 == MAXW && 64 * NW == 4 * MAXW, "one wave per 16 reduction indices; one thread per output of a row quad");
  constexpr int R = 4 * RQ;
  // every layer's input stays in LDS: the next layer reads it, and the chain of cotangents (when this launch runs it) takes the
  // activations' slopes from it
  __shared__ __attribute__((aligned(16))) float acts[ENDIA_MLP_MAX_LAYERS + 1][R * LD4];
  __shared__ __attribute__((aligned(16))) float ds[2][R * LD4];
  __shared__ float part[NW][R][MAXW];
  __shared__ int meet;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ocol = tid & (MAXW - 1), orow = tid >> 7;  // the outputs this thread finishes: column ocol of rows orow + 4 u
  const int row0 = blockIdx.x * R;
  auto request = [&](int l, FragF& f) {
    const int K = p.width[l], N = p.width[l + 1];
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b[l], (int64_t)N * 4);
    f.bias = buffer_load_f1(rb, ocol < N ? (uint32_t)(ocol * 4) : OOB_OFFSET);
    if (16 * wave >= K) return;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.W[l], (int64_t)K * N * 4);  // rows past K lie past the end of the buffer
#pragma unroll
    for (int half = 0; half < 2; ++half)
      if (64 * half < N) {
        const uint32_t base = 64 * half + lane < N ? (uint32_t)((16 * wave * N + 64 * half + lane) * 4) : OOB_OFFSET;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) f.v[kk][half] = buffer_load_f1(rs, base + (uint32_t)(kk * N * 4));
      }
  };
  float z[RQ];  // the outputs this thread finished in the last layer
  auto store = [&](int l) {
    const int N = p.width[l + 1];
    if (ocol < N) {
#pragma unroll
      for (int u = 0; u < RQ; ++u) {
        const int r = row0 + orow + 4 * u;
        if (r < p.batch) p.h[l][(int64_t)r * N + ocol] = z[u];
      }
    }
  };
  auto layer = [&](int l, const FragF& cur, FragF& nxt) {
    const int K = p.width[l], N = p.width[l + 1];
    const bool last = l + 1 == p.layers;
    wait_vm_all();
    if (!last) request(l + 1, nxt);
    if (l > 0) store(l - 1);
    const float* in = acts[l];
    float* out = acts[l + 1];
    if (16 * wave < K) {
      // (one straight run of MFMAs per case: a width test inside the run costs a branch and register copies per MFMA)
      if (N > 64) slab_mfma<RQ, 2>(in, cur, wave, lane, part[wave]);
      else slab_mfma<RQ, 1>(in, cur, wave, lane, part[wave]);
    }
    __syncthreads();
    const int npad = (N + 15) & ~15, slabs = (K + 15) >> 4;
    if (ocol < npad) {
#pragma unroll
      for (int u = 0; u < RQ; ++u) {
        float pw[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) pw[w] = part[w][orow + 4 * u][ocol];  // (all eight reads travel together; idle waves' slots hold leftovers)
        float v = cur.bias;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += w < slabs ? pw[w] : 0.f;  // partial sums in the order of their reduction ranges
        if (!last) v = act_apply(p.act, v);
        if (ocol >= N) v = 0.f;  // columns up to the next multiple of 16 feed the next reduction as zeros
        out[(orow + 4 * u) * LD4 + ocol] = v;
        z[u] = v;
      }
    }
    __syncthreads();
  };
  // the targets of this thread's outputs of the last layer, asked for now and needed at the very end
  const int NL = p.width[p.layers];
  const bool mine = p.target != nullptr && ocol < NL;
  float tgt[RQ];
#pragma unroll
  for (int u = 0; u < RQ; ++u) {
    const int r = row0 + orow + 4 * u;
    tgt[u] = (mine && r < p.batch) ? p.target[(int64_t)r * NL + ocol] : 0.f;
  }
  FragF wa, wb;
  request(0, wa);  // the first layer's weights travel while the input is staged
  stage_rows4<RQ>(acts[0], p.x, row0, p.batch, p.width[0], tid);
  __syncthreads();
  for (int l = 0; l < p.layers; l += 2) {  // (two layers per round: the operands change places without copies)
    layer(l, wa, wb);
    if (l + 1 < p.layers) layer(l + 1, wb, wa);
  }
  store(p.layers - 1);
  if (p.target) {  // mse = sum((out - target)^2) / n (mse_op.mojo:17-20) and its gradient, from the outputs still in registers
    __shared__ float red[NW];
    float acc = 0.f, dp[RQ];
#pragma unroll
    for (int u = 0; u < RQ; ++u) {
      const int r = row0 + orow + 4 * u;
      dp[u] = 0.f;
      if (mine && r < p.batch) {
        const float d = z[u] - tgt[u];
        acc += d * d;
        dp[u] = d * (2.0f * p.inv_n);
        if (p.dpred) p.dpred[(int64_t)r * NL + ocol] = dp[u];
      }
    }
    if (p.chain) {
      // the cotangents of all layers for these rows, from the loss gradient at hand: the backward pass is left with the
      // weight gradients (rows are independent through the whole chain; nobody waits for another group)
      delta_chain<RQ, true>(p, ds, acts, row0, [&]() {
        if (ocol < ((NL + 31) & ~31)) {
#pragma unroll
          for (int u = 0; u < RQ; ++u) ds[0][(orow + 4 * u) * LD4 + ocol] = dp[u];
        }
      });
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
    if (lane == 0) red[wave] = acc;
    __syncthreads();
    if (tid == 0) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) sum += red[w];
      endia::store_shared(&p.loss_part[blockIdx.x], sum);
    }
    if (endia::arrive_last(p.ticket, gridDim.x, &meet) && wave == 0) {
      // the groups' sums in a fixed order: lane i takes groups i, i + 64, .., then the lanes pairwise
      float sum = 0.f;
      for (unsigned i = lane; i < gridDim.x; i += 64) sum += endia::load_shared(&p.loss_part[i]);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sum += __shfl_down(sum, o);
      if (lane == 0) p.loss[0] = sum * p.inv_n;
    }
  }
}

// dW_l = h_{l-1}^T delta_l and db_l = 1^T delta_l for ALL layers in one launch: a work-group per 32 x 32 tile of a
// gradient, v_mfma_f32_32x32x2_f32 (left operand: lane = column of h, two rows of the batch per MFMA; a request reads
// 128 consecutive bytes of each of two rows, whole lines). The four waves take rows 32 w .. 32 w + 31 of every 128 of
// the batch; their partial tiles meet in LDS and are added in wave order, so results repeat bit for bit. The tiles
// with bk = 0 also sum delta's columns (db).
constexpr int WG_PITCH = 40;  // row pitch of a partial tile: the two half-waves of a store fall into different banks

__global__ __launch_bounds__(256) void mlp_wgrad_kernel(MlpArgs p) {
  __shared__ float part[4][32 * WG_PITCH];
  __shared__ float bsum[4][2][32];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 31, h = lane >> 5;
  int l = 0;
  while (l + 1 < p.layers && (int)blockIdx.x >= p.tile0[l + 1]) ++l;
  const int K = p.width[l], N = p.width[l + 1];
  const int tn = (N + 31) >> 5, t = (int)blockIdx.x - p.tile0[l];
  const int bk = t / tn, bn = t - bk * tn;
  const float* __restrict__ hp = l == 0 ? p.x : p.h[l - 1];  // [batch, K]
  const float* __restrict__ dl = p.delta[l];                 // [batch, N]
  const int m = 32 * bk + c, n = 32 * bn + c;
  // (rows past the batch lie past the end of both buffers and read as zero)
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(hp, (int64_t)p.batch * K * 4), rb = make_rsrc(dl, (int64_t)p.batch * N * 4);
  const uint32_t va = m < K ? (uint32_t)((h * K + m) * 4) : OOB_OFFSET, vb = n < N ? (uint32_t)((h * N + n) * 4) : OOB_OFFSET;
  mfma::floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  float colsum = 0.f;
  // two sets of operands: the next 32 rows travel while the MFMAs of the current ones run (requests past the batch
  // read zeros, so the last one needs no test)
  float a[2][16], b[2][16];
  auto request = [&](int r0, float (&av)[16], float (&bv)[16]) {
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      av[s] = buffer_load_f1(ra, va + (uint32_t)((r0 + 2 * s) * K * 4));
      bv[s] = buffer_load_f1(rb, vb + (uint32_t)((r0 + 2 * s) * N * 4));
    }
  };
  auto multiply = [&](const float (&av)[16], const float (&bv)[16]) {
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s], bv[s], acc, 0, 0, 0);
      colsum += bv[s];
    }
  };
  const int begin = (int)blockIdx.y * p.rows_per_slice;  // (a multiple of 128; one slice unless the batch is large)
  const int end = min(p.batch, begin + p.rows_per_slice);
  request(begin + 32 * wave, a[0], b[0]);
  for (int r0 = begin + 32 * wave; r0 < end; r0 += 256) {
    request(r0 + 128, a[1], b[1]);
    multiply(a[0], b[0]);
    if (r0 + 128 >= end) break;
    request(r0 + 256, a[0], b[0]);
    multiply(a[1], b[1]);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) part[wave][mfma::acc_row(v, h) * WG_PITCH + c] = acc[v];
  bsum[wave][h][c] = colsum;
  __syncthreads();
  const int ocol = tid & 31, nn = 32 * bn + ocol;
  if (nn >= N) return;
  // one slice: the gradients themselves; several: this slice's sums
  float* dWl = gridDim.y > 1 ? p.wpart + (int64_t)blockIdx.y * p.woff[p.layers] + p.woff[l] : p.dW[l];
  float* dbl = gridDim.y > 1 ? dWl + K * N : p.db[l];
  if (dWl) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int row = (tid >> 5) + 8 * u, k = 32 * bk + row;
      const float sum = ((part[0][row * WG_PITCH + ocol] + part[1][row * WG_PITCH + ocol]) + part[2][row * WG_PITCH + ocol]) + part[3][row * WG_PITCH + ocol];
      if (k < K) dWl[(int64_t)k * N + nn] = sum;
    }
  }
  if (bk == 0 && tid < 32 && dbl) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) sum += bsum[w][0][ocol] + bsum[w][1][ocol];
    dbl[nn] = sum;
  }
}

// The second launch of a large batch's weight gradients: every gradient element is the sum of its slices, in slice order.
__global__ __launch_bounds__(256) void mlp_wgrad_sum_kernel(MlpArgs p, int slices) {
  const int total = p.woff[p.layers];
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  int l = 0;
  while (l + 1 < p.layers && e >= p.woff[l + 1]) ++l;
  const int at = e - p.woff[l], kn = p.width[l] * p.width[l + 1];
  float* dst = at < kn ? (p.dW[l] ? p.dW[l] + at : nullptr) : (p.db[l] ? p.db[l] + (at - kn) : nullptr);
  if (!dst) return;
  float sum = 0.f;
  for (int s = 0; s < slices; ++s) sum += p.wpart[(int64_t)s * total + e];
  *dst = sum;
}

// The kernels read and write activations, cotangents, biases and gradients 16 bytes at a time wherever a layer's width is
// a multiple of four; only the weights have an element-by-element route. So every other array has to start on a
// 16-byte boundary (what every allocator hands out).
bool on_16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
#define ENDIA_MLP_ALIGNED(ptr, what, l) \
  ENDIA_CHECK_ARG(on_16(ptr), "%s: %s of layer %d is not 16-byte aligned (only the weight matrices may start anywhere)", who, what, l)

int32_t fill_args(MlpArgs& a, const endia_hip_mlp_desc* d, const char* who) {
  ENDIA_CHECK_ARG(d != nullptr, "%s: null descriptor", who);
  ENDIA_CHECK_ARG(d->layers >= 1 && d->layers <= ENDIA_MLP_MAX_LAYERS, "%s: %d layers, 1..%d supported", who, d->layers, ENDIA_MLP_MAX_LAYERS);
  ENDIA_CHECK_ARG(d->act == ENDIA_OP_RELU || d->act == ENDIA_OP_TANH || d->act == ENDIA_OP_IDENTITY,
                  "%s: activation %d is not relu, tanh or identity", who, d->act);
  ENDIA_CHECK_ARG(d->batch >= 0 && d->batch <= (1 << 20), "%s: batch %lld out of range", who, (long long)d->batch);
  for (int i = 0; i <= d->layers; ++i)
    ENDIA_CHECK_ARG(d->widths[i] >= 1 && d->widths[i] <= ENDIA_MLP_MAX_WIDTH, "%s: width %lld of layer boundary %d is not in 1..%d", who,
                    (long long)d->widths[i], i, ENDIA_MLP_MAX_WIDTH);
  a = MlpArgs{};
  a.layers = d->layers;
  a.act = d->act;
  a.batch = (int)d->batch;
  for (int i = 0; i <= d->layers; ++i) a.width[i] = (int)d->widths[i];
  return ENDIA_HIP_OK;
}

// Four rows per work-group up to 2048 rows (two groups per CU), sixteen rows on the 16 x 16 x 4 MFMA beyond: every group
// fetches every weight, so more groups cost more traffic. Measured, forward + backward of four 128-wide layers replayed as
// a graph: 2048 rows 72 us on the four-row kernels against 80 us, 4096 rows 102 against 98, 8192 rows 166 against 150.
constexpr int64_t kFourRowBatch = 2048;
int64_t fwd_groups(const MlpArgs& a) { return ceil_div64(a.batch, a.batch <= kFourRowBatch ? 4 : ROWS); }

void launch_fwd(const MlpArgs& a, hipStream_t s) {
  if (a.batch <= kFourRowBatch) hipLaunchKernelGGL(mlp_fwd4_kernel, dim3((unsigned)fwd_groups(a)), dim3(64 * NW), 0, s, a);
  else hipLaunchKernelGGL(mlp_fwd_kernel, dim3((unsigned)fwd_groups(a)), dim3(64 * NW), 0, s, a);
}
void launch_delta(const MlpArgs& a, hipStream_t s) {
  if (a.batch <= kFourRowBatch) hipLaunchKernelGGL(mlp_delta4_kernel, dim3((unsigned)fwd_groups(a)), dim3(64 * NW), 0, s, a);
  else hipLaunchKernelGGL(mlp_delta_kernel, dim3((unsigned)fwd_groups(a)), dim3(64 * NW), 0, s, a);
}

}  // namespace

using namespace endia;

extern "C" int32_t endia_hip_mlp_fwd(const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* b,
                                     float* const* h) {
  ENDIA_REQUIRE_INIT();
  MlpArgs a;
  int32_t rc = fill_args(a, desc, "endia_hip_mlp_fwd");
  if (rc) return rc;
  if (a.batch == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && W && b && h, "endia_hip_mlp_fwd: null argument");
  const char* who = "endia_hip_mlp_fwd";
  ENDIA_MLP_ALIGNED(x, "x", 0);
  for (int l = 0; l < a.layers; ++l) {
    ENDIA_CHECK_ARG(W[l] && b[l] && h[l], "endia_hip_mlp_fwd: null pointer for layer %d", l);
    ENDIA_MLP_ALIGNED(b[l], "b", l);
    ENDIA_MLP_ALIGNED(h[l], "h", l);
    a.W[l] = W[l];
    a.b[l] = b[l];
    a.h[l] = h[l];
  }
  a.x = x;
  launch_fwd(a, ctx().stream);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

namespace {

// The forward launch with the MSE loss on top; with `delta` also the chain of cotangents from the loss gradient.
int32_t fwd_mse(const char* who, const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* b,
                const float* target, float* const* h, float* dpred, float* loss, float* const* delta, float* dx) {
  ENDIA_REQUIRE_INIT();
  MlpArgs a;
  int32_t rc = fill_args(a, desc, who);
  if (rc) return rc;
  ENDIA_CHECK_ARG(loss != nullptr, "%s: loss is null", who);
  if (a.batch == 0) return endia_hip_fill(loss, 1, 0.f);
  ENDIA_CHECK_ARG(x && W && b && h && target, "%s: null argument", who);
  for (int l = 0; l < a.layers; ++l) {
    ENDIA_CHECK_ARG(W[l] && b[l] && h[l] && (!delta || delta[l]), "%s: null pointer for layer %d", who, l);
    ENDIA_MLP_ALIGNED(b[l], "b", l);
    ENDIA_MLP_ALIGNED(h[l], "h", l);
    if (delta) ENDIA_MLP_ALIGNED(delta[l], "delta", l);
    a.W[l] = W[l];
    a.b[l] = b[l];
    a.h[l] = h[l];
    if (delta) a.delta[l] = delta[l];
  }
  ENDIA_MLP_ALIGNED(x, "x", 0);
  ENDIA_MLP_ALIGNED(target, "target", a.layers - 1);
  ENDIA_MLP_ALIGNED(dpred, "dpred", a.layers - 1);
  ENDIA_MLP_ALIGNED(dx, "dx", 0);
  a.x = x;
  const int64_t groups = fwd_groups(a);
  struct Scratch {  // partial sums from the library's pool, handed back on scope exit (reuse is stream-ordered)
    void* p = nullptr;
    ~Scratch() { if (p) endia_hip_free(p); }
  } part;
  if ((rc = endia_hip_malloc(groups * 4, &part.p))) return rc;
  a.target = target;
  a.dpred = delta ? delta[a.layers - 1] : dpred;
  a.loss = loss;
  a.loss_part = static_cast<float*>(part.p);
  a.ticket = ctx().tickets + (kTicketCount - 1);
  a.inv_n = 1.0f / (float)((int64_t)a.batch * a.width[a.layers]);
  a.dx = delta ? dx : nullptr;
  // the four-row kernel runs the chain itself; beyond its batches the chain is the launch it always was
  a.chain = delta != nullptr && a.batch <= kFourRowBatch;
  launch_fwd(a, ctx().stream);
  ENDIA_LAUNCH_CHECK();
  if (delta && !a.chain && (a.layers > 1 || dx)) {
    launch_delta(a, ctx().stream);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}

}  // namespace

extern "C" int32_t endia_hip_mlp_fwd_mse(const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* b,
                                         const float* target, float* const* h, float* dpred, float* loss) {
  return fwd_mse("endia_hip_mlp_fwd_mse", desc, x, W, b, target, h, dpred, loss, nullptr, nullptr);
}

extern "C" int32_t endia_hip_mlp_fwd_mse_delta(const endia_hip_mlp_desc* desc, const float* x, const float* const* W,
                                               const float* const* b, const float* target, float* const* h, float* const* delta,
                                               float* loss, float* dx) {
  ENDIA_CHECK_ARG(delta != nullptr, "endia_hip_mlp_fwd_mse_delta: delta is null");
  return fwd_mse("endia_hip_mlp_fwd_mse_delta", desc, x, W, b, target, h, nullptr, loss, delta, dx);
}

namespace {

int32_t bwd(const char* who, const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* h,
            float* const* delta, float* const* dW, float* const* db, float* dx, bool chain) {
  ENDIA_REQUIRE_INIT();
  MlpArgs a;
  int32_t rc = fill_args(a, desc, who);
  if (rc) return rc;
  if (a.batch == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(x && (W || !chain) && h && delta && dW && db, "%s: null argument", who);
  int blocks = 0;
  for (int l = 0; l < a.layers; ++l) {
    ENDIA_CHECK_ARG((!chain || W[l]) && delta[l] && (l + 1 == a.layers || h[l]), "%s: null pointer for layer %d", who, l);
    ENDIA_MLP_ALIGNED(h[l], "h", l);
    ENDIA_MLP_ALIGNED(delta[l], "delta", l);
    ENDIA_MLP_ALIGNED(dW[l], "dW", l);
    ENDIA_MLP_ALIGNED(db[l], "db", l);
    a.W[l] = chain ? W[l] : nullptr;
    a.h[l] = const_cast<float*>(h[l]);
    a.delta[l] = delta[l];
    a.dW[l] = dW[l];
    a.db[l] = db[l];
    a.tile0[l] = blocks;
    blocks += ((a.width[l] + 31) / 32) * ((a.width[l + 1] + 31) / 32);
  }
  a.tile0[a.layers] = blocks;
  ENDIA_MLP_ALIGNED(x, "x", 0);
  ENDIA_MLP_ALIGNED(dx, "dx", 0);
  a.x = x;
  a.dx = dx;
  hipStream_t s = ctx().stream;
  if (chain && (a.layers > 1 || dx)) {
    launch_delta(a, s);
    ENDIA_LAUNCH_CHECK();
  }
  // A large batch is cut into slices of at least 1024 rows, enough of them for two work-groups per CU; their sums meet in
  // a second launch (pooled scratch, handed back on scope exit: reuse is stream-ordered).
  int total = 0;
  for (int l = 0; l < a.layers; ++l) {
    a.woff[l] = total;
    total += a.width[l] * a.width[l + 1] + a.width[l + 1];
  }
  a.woff[a.layers] = total;
  int64_t slices = std::min<int64_t>(std::max<int64_t>(1, 2 * ctx().cu_count / blocks), a.batch / 1024);
  if (slices < 1) slices = 1;
  a.rows_per_slice = (int)(ceil_div64(ceil_div64(a.batch, slices), 128) * 128);
  slices = ceil_div64(a.batch, a.rows_per_slice);
  struct Scratch {
    void* p = nullptr;
    ~Scratch() { if (p) endia_hip_free(p); }
  } part;
  if (slices > 1) {
    if ((rc = endia_hip_malloc(slices * total * 4, &part.p))) return rc;
    a.wpart = static_cast<float*>(part.p);
  }
  hipLaunchKernelGGL(mlp_wgrad_kernel, dim3((unsigned)blocks, (unsigned)slices), dim3(256), 0, s, a);
  ENDIA_LAUNCH_CHECK();
  if (slices > 1) {
    hipLaunchKernelGGL(mlp_wgrad_sum_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a, (int)slices);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}

}  // namespace

extern "C" int32_t endia_hip_mlp_bwd(const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* h,
                                     float* const* delta, float* const* dW, float* const* db, float* dx) {
  return bwd("endia_hip_mlp_bwd", desc, x, W, h, delta, dW, db, dx, true);
}

extern "C" int32_t endia_hip_mlp_wgrad(const endia_hip_mlp_desc* desc, const float* x, const float* const* h,
                                       const float* const* delta, float* const* dW, float* const* db) {
  return bwd("endia_hip_mlp_wgrad", desc, x, nullptr, h, const_cast<float* const*>(delta), dW, db, nullptr, false);
}
