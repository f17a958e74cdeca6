// conv1d / conv2d / conv3d (channels-first, cross-correlation, groups = 1) as implicit GEMMs on the fp32
// matrix cores. Everything below is written for [N, C, D, H, W] with a [K, C, T, R, S] kernel; the 2-D op is
// the case D = T = 1 (the extra index decodes cost nothing there) and the formulas in this header are
// written for it. Conv3d.__call__ is endia/functional/spacial_ops/conv3d_op.mojo:104-259.
//
// Forward follows Conv2d.__call__ (endia/functional/spacial_ops/conv2d_op.mojo:88-196; output shape rule
// conv2d_op.mojo:31-85):
//   y[n,k,p,q] = b[k] + sum_{c,r,s} x[n,c, p*sh - ph + r*dh, q*sw - pw + s*dw] * w[k,c,r,s]
// with out-of-range taps contributing zero. The reference registers no backward rule for conv2d
// (Conv2d.vjp = default_vjp, conv2d_op.mojo:198-200); the gradients here are the adjoints of that loop:
//   db[k]       = sum_{n,p,q} dy[n,k,p,q]
//   dw[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c, p*sh - ph + r*dh, q*sw - pw + s*dw]
//   dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * w[k,c,r,s]  over (p,q) with p*sh - ph + r*dh = h, q*sw - pw + s*dw = w
//
// GEMM views (no im2col matrix is ever written; the gather happens on the way into LDS):
//   forward   C[K, N*P*Q]   = Wp[K, C*R*S]    . col(x)[C*R*S, N*P*Q]
//   data grad C[C, N*H*W]   = WpT[C, K*R*S]   . col'(dy)[K*R*S, N*H*W]      (transposed convolution)
//   weight    C[K, C*R*S]   = dy[K, N*P*Q]    . col(x)[C*R*S, N*P*Q]^T      (split over N*P*Q, partials
//                                                                            summed in a fixed order)
// Wp / WpT are the weights repacked once per call into a row-padded matrix (a few hundred KiB).
// The 7-deep scalar loop of the reference becomes: K tile of 32, 128 x 128 (or 64 x 128) tile of C per
// work-group, v_mfma_f32_32x32x2_f32, the same LDS layouts as the dense GEMM.
#include "common.h"
#include "mfma_tile.h"

namespace endia {
int32_t col_reduce(int64_t batch, int64_t R, int64_t C, const float* x, float* out, float scale);
int32_t col_reduce_transposed(int64_t R, int64_t C, int64_t inner, const float* x, float* out);
int32_t col_reduce_with_rider(int64_t R, int64_t C, int64_t inner, const float* x, float* out, int64_t R2, int64_t C2, const float* x2,
                              float* out2);
int32_t row_reduce(int64_t R, int64_t C, const float* x, float* out, float scale);
}

namespace {

using namespace mfma;

constexpr int TPB = 256;
constexpr int FAR = -(1 << 28);  // coordinate that fails every bounds test
int g_forced_path = 0;  // endia_hip_conv_force_path

struct ConvP {
  int N, C, D, H, W, K, T, R, S, O, P, Q;  // O, P, Q: output depth, height, width
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
};

enum { MODE_FWD = 0, MODE_BWD_DATA = 1 };

// ---- forward and data gradient ------------------------------------------------------------------
struct IgemmArgs {
  const float* src;   // fwd: x [N,C,H,W]; data grad: dy [N,K,P,Q]
  const float* wp;    // packed weights [Mrows, Kd_pad]
  const float* bias;  // fwd: [K] or null
  float* out;         // fwd: y; data grad: dx
  int Mrows, Cred;    // output channels of this GEMM; channels reduced over
  int SD, SH, SW, OD, OH, OW; // source and output spatial extents
  int Kd, Kd_pad;     // Cred*T*R*S and its multiple-of-4 padding
  int Ncols;          // N*OD*OH*OW
  int T, R, S, sd, sh, sw, pd, ph, pw, dd, dh, dw;
  FastDiv d_trs, d_rs, d_s, d_ovol, d_ohw, d_ow, d_sd, d_sh, d_sw;
  int tiles_m, tiles_n, relu;
  int64_t src_bytes;
};

// B operand: rows = reduction index t = (ch, kz, r, s), columns = output pixels j = (n, oz, oy, ox).
// A lane owns 4 consecutive columns for the whole kernel (decoded once) and PASSES rows per K tile.
template <int MODE, int BN, int NT>
struct GatherColsLoader {
  static constexpr int F4_PER_ROW = BN / 4;
  static constexpr int ROWS_PER_PASS = NT / F4_PER_ROW;
  static constexpr int PASSES = BK / ROWS_PER_PASS;
  static constexpr int LD = TileShape<false, BN>::LD;
  int base[4], z0[4], y0[4], x0[4];
  int r, lds_off;
  float reg[PASSES][4];

  __device__ __forceinline__ void init(const IgemmArgs& a, int n0, int tid) {
    r = tid / F4_PER_ROW;
    const int c4 = (tid % F4_PER_ROW) * 4;
    lds_off = r * LD + c4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      int j = n0 + c4 + e;
      if (j < a.Ncols) {
        int n = (int)fdiv((uint32_t)j, a.d_ovol);
        int rem = j - n * a.OD * a.OH * a.OW;
        int oz = (int)fdiv((uint32_t)rem, a.d_ohw);
        rem -= oz * a.OH * a.OW;
        int oy = (int)fdiv((uint32_t)rem, a.d_ow);
        int ox = rem - oy * a.OW;
        base[e] = n * a.Cred * a.SD * a.SH * a.SW;
        z0[e] = MODE == MODE_FWD ? oz * a.sd - a.pd : oz + a.pd;
        y0[e] = MODE == MODE_FWD ? oy * a.sh - a.ph : oy + a.ph;
        x0[e] = MODE == MODE_FWD ? ox * a.sw - a.pw : ox + a.pw;
      } else {
        base[e] = 0;
        z0[e] = 0;
        y0[e] = FAR;
        x0[e] = 0;
      }
    }
  }
  __device__ __forceinline__ void load(const IgemmArgs& a, int k0) {
    __amdgpu_buffer_rsrc_t rs = make_rsrc(a.src, a.src_bytes);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      int t = k0 + r + i * ROWS_PER_PASS;
      int ch = (int)fdiv((uint32_t)t, a.d_trs);
      int rem = t - ch * a.T * a.R * a.S;
      int kz = (int)fdiv((uint32_t)rem, a.d_rs);
      rem -= kz * a.R * a.S;
      int rr = (int)fdiv((uint32_t)rem, a.d_s);
      int ss = rem - rr * a.S;
      int roff = ch * a.SD * a.SH * a.SW;
      int dzv = kz * a.dd;
      int dyv = t < a.Kd ? rr * a.dh : (MODE == MODE_FWD ? FAR : -FAR);
      int dxv = ss * a.dw;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int iz, iy, ix;
        bool ok;
        if (MODE == MODE_FWD) {
          iz = z0[e] + dzv;
          iy = y0[e] + dyv;
          ix = x0[e] + dxv;
          ok = (unsigned)iz < (unsigned)a.SD && (unsigned)iy < (unsigned)a.SH && (unsigned)ix < (unsigned)a.SW;
        } else {
          int tz = z0[e] - dzv, ty = y0[e] - dyv, tx = x0[e] - dxv;
          if (a.sd == 1 && a.sh == 1 && a.sw == 1) {
            iz = tz;
            iy = ty;
            ix = tx;
            ok = (unsigned)iz < (unsigned)a.SD && (unsigned)iy < (unsigned)a.SH && (unsigned)ix < (unsigned)a.SW;
          } else {
            ok = tz >= 0 && ty >= 0 && tx >= 0;
            iz = (int)fdiv((uint32_t)(ok ? tz : 0), a.d_sd);
            iy = (int)fdiv((uint32_t)(ok ? ty : 0), a.d_sh);
            ix = (int)fdiv((uint32_t)(ok ? tx : 0), a.d_sw);
            ok = ok && iz * a.sd == tz && iy * a.sh == ty && ix * a.sw == tx && iz < a.SD && iy < a.SH && ix < a.SW;
          }
        }
        uint32_t off = ok ? (uint32_t)(base[e] + roff + (iz * a.SH + iy) * a.SW + ix) * 4u : OOB_OFFSET;
        reg[i][e] = buffer_load_f1(rs, off);
      }
    }
  }
  __device__ __forceinline__ void store(float* lds) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LD]) = make_float4(reg[i][0], reg[i][1], reg[i][2], reg[i][3]);
  }
};

template <int MODE, int WGM, int WGN, int FM, int FN>
__global__ __launch_bounds__(WGM* WGN * 64, 3) void conv_igemm_kernel(IgemmArgs a) {
  constexpr int NT = WGM * WGN * 64, BM = WGM * FM * 32, BN = WGN * FN * 32;
  using LA = MatrixTileLoader<true, BM, NT>;
  using LB = GatherColsLoader<MODE, BN, NT>;
  __shared__ __attribute__((aligned(16))) float As[TileShape<true, BM>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<false, BN>::FLOATS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, h = lane >> 5;
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, a.tiles_m, a.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  LA la;
  LB lb;
  la.init(a.wp, a.Kd_pad, m0, a.Mrows, a.Kd_pad, tid);
  lb.init(a, n0, tid);

  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);

  la.load(a.Kd_pad);
  lb.load(a, 0);
  la.store(As);
  lb.store(Bs);
  __syncthreads();

  for (int k0 = 0; k0 < a.Kd_pad; k0 += BK) {
    const bool more = k0 + BK < a.Kd_pad;
    if (more) {
      la.advance();
      la.load(a.Kd_pad - k0 - BK);
      lb.load(a, k0 + BK);
    }
    compute_ktile<true, false, FM, FN, BM, BN>(As, Bs, wm * FM * 32 + l32, wn * FN * 32 + l32, h, acc);
    if (more) {
      __syncthreads();
      la.store(As);
      lb.store(Bs);
      __syncthreads();
    }
  }

  const int64_t ohw = (int64_t)a.OD * a.OH * a.OW;  // output positions per image
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    int j = n0 + wn * FN * 32 + fn * 32 + l32;
    if (j >= a.Ncols) continue;
    int n = (int)fdiv((uint32_t)j, a.d_ovol);
    int64_t col_off = (int64_t)n * a.Mrows * ohw + (j - (int64_t)n * ohw);
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int m = m0 + wm * FM * 32 + fm * 32 + acc_row(v, h);
        if (m < a.Mrows) {
          float val = acc[fm][fn][v];
          if (MODE == MODE_FWD) {
            if (a.bias) val += a.bias[m];
            if (a.relu) val = val > 0.f ? val : 0.f;
          }
          a.out[col_off + m * ohw] = val;
        }
      }
  }
}

// ---- weight gradient ------------------------------------------------------------------------------
struct WgradArgs {
  const float* x;
  const float* dy;
  float* part;  // [splits][K][Kd]
  int N, C, D, H, W, K, T, R, S, O, P, Q, sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int Kd;
  int total_j, chunk;  // N*O*P*Q and the slice of it one split reduces over (multiple of 32)
  FastDiv d_opq, d_pq, d_q, d_trs, d_rs, d_s;
  int tiles_m, tiles_n;
  int64_t x_bytes, dy_bytes;
};

// dy as the A operand: rows = output channel k, 32 consecutive j = (n, o, p, q) per tile.
template <int BM, int NT>
struct DyRowsLoader {
  static constexpr int ROWS_PER_PASS = NT / 8;
  static constexpr int PASSES = BM / ROWS_PER_PASS;
  int rowoff[PASSES];  // k * P*Q, or -1 for rows past K
  int c4, lds_off;
  float reg[PASSES][4];
  __device__ __forceinline__ void init(const WgradArgs& a, int m0, int tid) {
    const int r = tid / 8;
    c4 = (tid % 8) * 4;
    lds_off = r * LDK + c4;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      int m = m0 + r + i * ROWS_PER_PASS;
      rowoff[i] = m < a.K ? m * a.O * a.P * a.Q : -1;
    }
  }
  __device__ __forceinline__ void load(const WgradArgs& a, int jt, int j_end) {
    __amdgpu_buffer_rsrc_t rs = make_rsrc(a.dy, a.dy_bytes);
    const int pq_n = a.O * a.P * a.Q;
    int j = jt + c4;
    int n = (int)fdiv((uint32_t)j, a.d_opq);
    int pq = j - n * pq_n;
    int off[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      off[e] = (j + e < j_end) ? n * a.K * pq_n + pq : -1;
      if (++pq == pq_n) { pq = 0; ++n; }
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bool ok = rowoff[i] >= 0 && off[e] >= 0;
        reg[i][e] = buffer_load_f1(rs, ok ? (uint32_t)(off[e] + rowoff[i]) * 4u : OOB_OFFSET);
      }
  }
  __device__ __forceinline__ void store(float* lds) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LDK]) = make_float4(reg[i][0], reg[i][1], reg[i][2], reg[i][3]);
  }
};

// col(x) as the B operand: rows = filter tap t = (c, kz, r, s), 32 consecutive j per tile.
template <int BN, int NT>
struct TapRowsLoader {
  static constexpr int ROWS_PER_PASS = NT / 8;
  static constexpr int PASSES = BN / ROWS_PER_PASS;
  int roff[PASSES], dzv[PASSES], dyv[PASSES], dxv[PASSES];
  int c4, lds_off;
  float reg[PASSES][4];
  __device__ __forceinline__ void init(const WgradArgs& a, int n0, int tid) {
    const int r = tid / 8;
    c4 = (tid % 8) * 4;
    lds_off = r * LDK + c4;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      int t = n0 + r + i * ROWS_PER_PASS;
      int ch = (int)fdiv((uint32_t)t, a.d_trs);
      int rem = t - ch * a.T * a.R * a.S;
      int kz = (int)fdiv((uint32_t)rem, a.d_rs);
      rem -= kz * a.R * a.S;
      int rr = (int)fdiv((uint32_t)rem, a.d_s);
      int ss = rem - rr * a.S;
      roff[i] = ch * a.D * a.H * a.W;
      dzv[i] = kz * a.dd - a.pd;
      dyv[i] = t < a.Kd ? rr * a.dh - a.ph : FAR;
      dxv[i] = ss * a.dw - a.pw;
    }
  }
  __device__ __forceinline__ void load(const WgradArgs& a, int jt, int j_end) {
    __amdgpu_buffer_rsrc_t rs = make_rsrc(a.x, a.x_bytes);
    int j = jt + c4;
    int n = (int)fdiv((uint32_t)j, a.d_opq);
    int rem = j - n * a.O * a.P * a.Q;
    int o = (int)fdiv((uint32_t)rem, a.d_pq);
    rem -= o * a.P * a.Q;
    int p = (int)fdiv((uint32_t)rem, a.d_q);
    int q = rem - p * a.Q;
    int base[4], ze[4], ye[4], xe[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      base[e] = n * a.C * a.D * a.H * a.W;
      ze[e] = o * a.sd;
      ye[e] = (j + e < j_end) ? p * a.sh : FAR;
      xe[e] = q * a.sw;
      if (++q == a.Q) { q = 0; if (++p == a.P) { p = 0; if (++o == a.O) { o = 0; ++n; } } }
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int iz = ze[e] + dzv[i], iy = ye[e] + dyv[i], ix = xe[e] + dxv[i];
        bool ok = (unsigned)iz < (unsigned)a.D && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
        reg[i][e] = buffer_load_f1(rs, ok ? (uint32_t)(base[e] + roff[i] + (iz * a.H + iy) * a.W + ix) * 4u : OOB_OFFSET);
      }
  }
  __device__ __forceinline__ void store(float* lds) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LDK]) = make_float4(reg[i][0], reg[i][1], reg[i][2], reg[i][3]);
  }
};

template <int WGM, int WGN, int FM, int FN>
__global__ __launch_bounds__(WGM* WGN * 64, 2) void conv_wgrad_kernel(WgradArgs a) {
  constexpr int NT = WGM * WGN * 64, BM = WGM * FM * 32, BN = WGN * FN * 32;
  using LA = DyRowsLoader<BM, NT>;
  using LB = TapRowsLoader<BN, NT>;
  __shared__ __attribute__((aligned(16))) float As[TileShape<true, BM>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<true, BN>::FLOATS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, h = lane >> 5;
  const int tm = blockIdx.x / a.tiles_n, tn = blockIdx.x % a.tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;
  const int split = blockIdx.y;
  const int j_begin = split * a.chunk;
  const int j_end = j_begin + a.chunk < a.total_j ? j_begin + a.chunk : a.total_j;

  LA la;
  LB lb;
  la.init(a, m0, tid);
  lb.init(a, n0, tid);
  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);

  la.load(a, j_begin, j_end);
  lb.load(a, j_begin, j_end);
  la.store(As);
  lb.store(Bs);
  __syncthreads();
  for (int jt = j_begin; jt < j_end; jt += BK) {
    const bool more = jt + BK < j_end;
    if (more) {
      la.load(a, jt + BK, j_end);
      lb.load(a, jt + BK, j_end);
    }
    compute_ktile<true, true, FM, FN, BM, BN>(As, Bs, wm * FM * 32 + l32, wn * FN * 32 + l32, h, acc);
    if (more) {
      __syncthreads();
      la.store(As);
      lb.store(Bs);
      __syncthreads();
    }
  }

  float* out = a.part + (int64_t)split * a.K * a.Kd;
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    int t = n0 + wn * FN * 32 + fn * 32 + l32;
    if (t >= a.Kd) continue;
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int m = m0 + wm * FM * 32 + fm * 32 + acc_row(v, h);
        if (m < a.K) out[(int64_t)m * a.Kd + t] = acc[fm][fn][v];
      }
  }
}

// ---- fast path: unit stride along the row, output width a multiple of 4, padded source ------------
// The source tensor is first copied into a zero-padded tensor, so no tap is ever out of range, and a
// table gives every reduction index t its byte offset inside one padded image. A lane's four
// consecutive output pixels then read four consecutive source floats: ONE 16-byte buffer load at
// colbase(j) + table[t], and the whole gather is one integer add per load.
struct VecArgs {
  const float* src;   // padded source [N, Cred, Dp, Hp, Wp]
  const float* wp;    // packed weights [Mrows, Kd_pad]
  const int* table;   // [Kd_pad] byte offset of reduction index t inside an image; OOB_OFFSET for padding rows
  const float* bias;
  float* out;
  int Mrows, OD, OH, OW, Ncols, Kd_pad;
  int img_floats, Wp, sh, zstep;  // floats per padded image, padded row length, stride along rows, floats per output depth step
  FastDiv d_ovol, d_ohw, d_ow;
  int tiles_m, tiles_n, relu;
  int64_t src_bytes;
};

template <int WGM, int WGN, int FM, int FN, bool FWD>
__global__ __launch_bounds__(WGM* WGN * 64, 4) void conv_igemm_vec_kernel(VecArgs a) {
  constexpr int NT = WGM * WGN * 64, BM = WGM * FM * 32, BN = WGN * FN * 32;
  constexpr int F4_PER_ROW = BN / 4, ROWS_PER_PASS = NT / F4_PER_ROW, PASSES = BK / ROWS_PER_PASS;
  constexpr int LDB = TileShape<false, BN>::LD;
  using LA = MatrixTileLoader<true, BM, NT>;
  __shared__ __attribute__((aligned(16))) float As[TileShape<true, BM>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<false, BN>::FLOATS];
  extern __shared__ int tab[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, h = lane >> 5;
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, a.tiles_m, a.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  for (int i = tid; i < a.Kd_pad; i += NT) tab[i] = a.table[i];

  LA la;
  la.init(a.wp, a.Kd_pad, m0, a.Mrows, a.Kd_pad, tid);
  const int r = tid / F4_PER_ROW, c4 = (tid % F4_PER_ROW) * 4;
  const int lds_off = r * LDB + c4;
  uint32_t colbase = OOB_OFFSET;
  {
    int j = n0 + c4;
    if (j < a.Ncols) {
      int n = (int)fdiv((uint32_t)j, a.d_ovol);
      int rem = j - n * a.OD * a.OH * a.OW;
      int oz = (int)fdiv((uint32_t)rem, a.d_ohw);
      rem -= oz * a.OH * a.OW;
      int oy = (int)fdiv((uint32_t)rem, a.d_ow);
      int ox = rem - oy * a.OW;
      colbase = (uint32_t)(n * a.img_floats + oz * a.zstep + oy * a.sh * a.Wp + ox) * 4u;
    }
  }
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.src, a.src_bytes);
  float4 breg[PASSES];
  __syncthreads();  // table visible

  auto load_b = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) breg[i] = buffer_load_f4(rs, colbase + (uint32_t)tab[k0 + r + i * ROWS_PER_PASS]);
  };
  auto store_b = [&]() {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) *reinterpret_cast<float4*>(&Bs[lds_off + i * ROWS_PER_PASS * LDB]) = breg[i];
  };

  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);
  la.load(a.Kd_pad);
  load_b(0);
  la.store(As);
  store_b();
  __syncthreads();
  for (int k0 = 0; k0 < a.Kd_pad; k0 += BK) {
    const bool more = k0 + BK < a.Kd_pad;
    if (more) {
      la.advance();
      la.load(a.Kd_pad - k0 - BK);
      load_b(k0 + BK);
    }
    compute_ktile<true, false, FM, FN, BM, BN>(As, Bs, wm * FM * 32 + l32, wn * FN * 32 + l32, h, acc);
    if (more) {
      __syncthreads();
      la.store(As);
      store_b();
      __syncthreads();
    }
  }

  const int64_t ohw = (int64_t)a.OD * a.OH * a.OW;  // output positions per image
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    int j = n0 + wn * FN * 32 + fn * 32 + l32;
    if (j >= a.Ncols) continue;
    int n = (int)fdiv((uint32_t)j, a.d_ovol);
    int64_t col_off = (int64_t)n * a.Mrows * ohw + (j - (int64_t)n * ohw);
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int m = m0 + wm * FM * 32 + fm * 32 + acc_row(v, h);
        if (m < a.Mrows) {
          float val = acc[fm][fn][v];
          if (FWD) {
            if (a.bias) val += a.bias[m];
            if (a.relu) val = val > 0.f ? val : 0.f;
          }
          a.out[col_off + m * ohw] = val;
        }
      }
  }
}

struct WgradVecArgs {
  const float* xpad;  // [N, C, Dp, Hp, Wp]
  const float* dy;    // [N, K, O, P, Q], Q % 4 == 0 (GATE 1: one float, the same for every element)
  const float* gate;  // GATE > 0: the stored output y of relu(conv + bias), same shape; dy counts where y > 0
  const int* table;   // [tiles_n * BN] byte offset of tap t inside a padded image; OOB_OFFSET past Kd
  float* part;
  float* bias_part;   // may be null: [splits][K] sums of the (gated) dy over each split's columns
  int K, Kd, OPQ, PQ, Q, sh, Wp, img_floats, zstep;
  int total_j, chunk;
  FastDiv d_opq, d_pq, d_q;
  int tiles_m, tiles_n;
  int64_t x_bytes, dy_bytes;
};

// GATE 0: dy as it is. GATE 1 / 2: dy (1: a scalar, 2: a tensor) gated by [y > 0] as the A operand is loaded, so that
// the gradient of the ReLU is never written out. In every mode the work-groups of the first tile column can also sum
// the rows of what they load, which is the bias gradient.
template <int WGM, int WGN, int FM, int FN, int GATE>
__global__ __launch_bounds__(WGM* WGN * 64, FM* FN >= 6 ? 2 : 4) void conv_wgrad_vec_kernel(WgradVecArgs a) {
  constexpr int NT = WGM * WGN * 64, BM = WGM * FM * 32, BN = WGN * FN * 32;
  constexpr int ROWS_PER_PASS = NT / 8, PA = BM / ROWS_PER_PASS, PB = BN / ROWS_PER_PASS;
  __shared__ __attribute__((aligned(16))) float As[TileShape<true, BM>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<true, BN>::FLOATS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, h = lane >> 5;
  const int tm = blockIdx.x / a.tiles_n, tn = blockIdx.x % a.tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;
  const int split = blockIdx.y;
  const int j_begin = split * a.chunk;
  const int j_end = j_begin + a.chunk < a.total_j ? j_begin + a.chunk : a.total_j;

  const int r = tid / 8, c4 = (tid % 8) * 4;
  const int lds_off = r * LDK + c4;
  uint32_t rowa[PA], rowb[PB];
#pragma unroll
  for (int i = 0; i < PA; ++i) {
    int m = m0 + r + i * ROWS_PER_PASS;
    rowa[i] = m < a.K ? (uint32_t)(m * a.OPQ) * 4u : OOB_OFFSET;
  }
#pragma unroll
  for (int i = 0; i < PB; ++i) rowb[i] = (uint32_t)a.table[n0 + r + i * ROWS_PER_PASS];
  const __amdgpu_buffer_rsrc_t rs_dy = make_rsrc(GATE == 1 ? a.gate : a.dy, a.dy_bytes);
  const __amdgpu_buffer_rsrc_t rs_gate = make_rsrc(a.gate, a.dy_bytes);
  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(a.xpad, a.x_bytes);
  float4 ra[PA], rb[PB], rg[GATE == 2 ? PA : 1];
  const float dy_scalar = GATE == 1 ? a.dy[0] : 0.f;
  const bool sum_rows = a.bias_part != nullptr && tn == 0;
  float row_sum[PA];
#pragma unroll
  for (int i = 0; i < PA; ++i) row_sum[i] = 0.f;

  auto load = [&](int jt) {
    int j = jt + c4;
    uint32_t ca = OOB_OFFSET, cb = OOB_OFFSET;
    if (j < j_end) {
      int n = (int)fdiv((uint32_t)j, a.d_opq);
      int opq = j - n * a.OPQ;
      int o = (int)fdiv((uint32_t)opq, a.d_pq);
      int pq = opq - o * a.PQ;
      int p = (int)fdiv((uint32_t)pq, a.d_q);
      int q = pq - p * a.Q;
      ca = (uint32_t)(n * a.K * a.OPQ + opq) * 4u;
      cb = (uint32_t)(n * a.img_floats + o * a.zstep + p * a.sh * a.Wp + q) * 4u;
    }
#pragma unroll
    for (int i = 0; i < PA; ++i) ra[i] = buffer_load_f4(rs_dy, ca + rowa[i]);
    if (GATE == 2) {
#pragma unroll
      for (int i = 0; i < PA; ++i) rg[i] = buffer_load_f4(rs_gate, ca + rowa[i]);
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) rb[i] = buffer_load_f4(rs_x, cb + rowb[i]);
  };
  // applied to the staged pieces in registers ahead of the barrier that precedes the stores
  auto gate = [&]() {
    if (GATE > 0) {  // out-of-range pieces were loaded as zeros and stay zeros: 0 > 0 is false
#pragma unroll
      for (int i = 0; i < PA; ++i) {
        const float4 y = GATE == 1 ? ra[i] : rg[i];
        const float4 g = GATE == 1 ? make_float4(dy_scalar, dy_scalar, dy_scalar, dy_scalar) : ra[i];
        ra[i] = make_float4(y.x > 0.f ? g.x : 0.f, y.y > 0.f ? g.y : 0.f, y.z > 0.f ? g.z : 0.f, y.w > 0.f ? g.w : 0.f);
      }
    }
    if (sum_rows) {
#pragma unroll
      for (int i = 0; i < PA; ++i) row_sum[i] += (ra[i].x + ra[i].y) + (ra[i].z + ra[i].w);
    }
  };
  auto store = [&]() {
#pragma unroll
    for (int i = 0; i < PA; ++i) *reinterpret_cast<float4*>(&As[lds_off + i * ROWS_PER_PASS * LDK]) = ra[i];
#pragma unroll
    for (int i = 0; i < PB; ++i) *reinterpret_cast<float4*>(&Bs[lds_off + i * ROWS_PER_PASS * LDK]) = rb[i];
  };

  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);
  load(j_begin);
  gate();
  store();
  __syncthreads();
  for (int jt = j_begin; jt < j_end; jt += BK) {
    const bool more = jt + BK < j_end;
    if (more) load(jt + BK);
    compute_ktile<true, true, FM, FN, BM, BN>(As, Bs, wm * FM * 32 + l32, wn * FN * 32 + l32, h, acc);
    if (more) {
      gate();
      __syncthreads();
      store();
      __syncthreads();
    }
  }

  if (sum_rows) {  // the eight threads of a row are neighbours in a wave; fixed order of additions
#pragma unroll
    for (int i = 0; i < PA; ++i) {
      float v = row_sum[i];
      v += __shfl_xor(v, 1);
      v += __shfl_xor(v, 2);
      v += __shfl_xor(v, 4);
      const int m = m0 + r + i * ROWS_PER_PASS;
      if ((tid & 7) == 0 && m < a.K) a.bias_part[(int64_t)split * a.K + m] = v;
    }
  }

  float* out = a.part + (int64_t)split * a.K * a.Kd;
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    int t = n0 + wn * FN * 32 + fn * 32 + l32;
    if (t >= a.Kd) continue;
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int m = m0 + wm * FM * 32 + fm * 32 + acc_row(v, h);
        if (m < a.K) out[(int64_t)m * a.Kd + t] = acc[fm][fn][v];
      }
  }
}

// ---- 3 x 3 weight gradient, unit stride and dilation, padding 0 or 1: rows of x and dy cached in LDS ---------
// dW[k][c][r][s] = sum over n, p, q of dy[n][k][p][q] * x[n][c][p + r - ph][q + s - pw]: nine products with one left
// operand. The output channels k sit on the MFMA's rows, the input channels c on its columns and the PIXELS of an
// output row on its reduction axis (two per step, the half-wave picks one), so that one accumulator block per tap
// (r, s) reads its B fragment at (cached row p + r, column q + s) of the lane's channel: the shift is a constant of the
// LDS instruction, x is cached ONCE (no padded copy in memory, no gather that writes an element nine times) and
// nothing is tested in the loop (rows outside the image and the column on either side are zeros in the cache).
// A work-group (4 waves, 128 output channels x 32 input channels x 9 taps, 144 accumulator registers a lane) walks
// the output rows [p_begin, p_end) of ONE image: per row it brings in the row of dy (128 x Q) and ONE new row of x
// (the ring keeps the last three and the one arriving), both requested a row ahead into registers. Rows are 66 words
// apart in LDS (2 mod 64), so that the 32 lanes of a fragment (one channel each) and the two half-waves (neighbouring
// pixels) read 64 distinct banks. 252 MFMAs per wave between two barrier pairs; two work-groups per CU.
// Every work-group writes its partial gradient [tap][k][c] (the lanes of a store are 32 neighbouring c); the
// partials are added in split order by the column-reduction kernels and a last small kernel turns [tap][k][c] into
// the [k][c][tap] of the weights.
constexpr int W3_LD = 66;                 // floats between cached rows
constexpr int W3_BK = 128, W3_BC = 32;    // output / input channels per work-group
constexpr int W3_SLOT = W3_BC * W3_LD;    // one ring slot: one row of every input channel
constexpr int W3_PD = 7, W3_PX = 2;       // 16-byte pieces per thread: of a dy row (128 x 56 / 4 / 256), of an x row (32 x 64 / 4 / 256)

struct Wgrad3Args {
  const float* x;     // [N, C, H, W]
  const float* dy;    // [N, K, P, Q] (GATE 1: one float)
  const float* gate;  // GATE > 0: the stored output y, same shape as dy
  float* part;        // [splits][9][K][C]
  float* bias_part;   // [splits][K] or null
  int C, H, W, K, P, Q, ph, pw;
  int rows_per_wg, wgs_per_image, tiles_c;
  int64_t x_bytes, dy_bytes;
};

template <int GATE>
__global__ __launch_bounds__(256, 2) void conv_wgrad3x3_kernel(Wgrad3Args a) {
  __shared__ __attribute__((aligned(16))) float Xs[4 * W3_SLOT];
  __shared__ __attribute__((aligned(16))) float Ds[W3_BK * W3_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int tk = blockIdx.x / a.tiles_c, tc = blockIdx.x - tk * a.tiles_c;
  const int k0 = tk * W3_BK, c0 = tc * W3_BC;
  const int split = blockIdx.y, n = split / a.wgs_per_image;
  const int p_begin = (split - n * a.wgs_per_image) * a.rows_per_wg;
  const int p_end = p_begin + a.rows_per_wg < a.P ? p_begin + a.rows_per_wg : a.P;

  for (int i = tid; i < 4 * W3_SLOT; i += 256) Xs[i] = 0.f;
  for (int i = tid; i < W3_BK * W3_LD; i += 256) Ds[i] = 0.f;

  // the pieces this thread stages: byte offset of the piece in row 0 (of the image / of the output) and where it goes in LDS
  const int Q4 = a.Q >> 2, W4 = a.W >> 2;
  uint32_t dvoff[W3_PD], xvoff[W3_PX];
  int dl[W3_PD], xl[W3_PX];
#pragma unroll
  for (int j = 0; j < W3_PD; ++j) {
    const int u = tid + 256 * j, k = u / Q4, c4 = u - k * Q4;
    const bool in = u < W3_BK * Q4;
    dl[j] = in ? k * W3_LD + 4 * c4 : -1;
    dvoff[j] = in && k0 + k < a.K ? (uint32_t)(((n * a.K + k0 + k) * a.P * a.Q + 4 * c4) * 4) : OOB_OFFSET;
  }
#pragma unroll
  for (int j = 0; j < W3_PX; ++j) {
    const int u = tid + 256 * j, c = u / W4, c4 = u - c * W4;
    const bool in = u < W3_BC * W4;
    xl[j] = in ? c * W3_LD + 2 + 4 * c4 : -1;  // column xc of a row sits at word xc + 2: words 1 and W + 2 stay zero
    xvoff[j] = in && c0 + c < a.C ? (uint32_t)(((n * a.C + c0 + c) * a.H * a.W + 4 * c4) * 4) : OOB_OFFSET;
  }
  const __amdgpu_buffer_rsrc_t rs_dy = make_rsrc(GATE == 1 ? a.gate : a.dy, a.dy_bytes);
  const __amdgpu_buffer_rsrc_t rs_gate = make_rsrc(a.gate, a.dy_bytes);
  const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(a.x, a.x_bytes);
  const float dy_scalar = GATE == 1 ? a.dy[0] : 0.f;
  const bool sum_rows = a.bias_part != nullptr && tc == 0;

  float4 rd[W3_PD], rg[GATE == 2 ? W3_PD : 1], rx[W3_PX];
  float row_sum[W3_PD];
#pragma unroll
  for (int j = 0; j < W3_PD; ++j) row_sum[j] = 0.f;
  auto load_dy = [&](int p) {
    const int soff = p * a.Q * 4;
#pragma unroll
    for (int j = 0; j < W3_PD; ++j) {
      v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_dy, (int)dvoff[j], soff, 0);
      rd[j] = *reinterpret_cast<float4*>(&v);
    }
    if (GATE == 2) {
#pragma unroll
      for (int j = 0; j < W3_PD; ++j) {
        v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_gate, (int)dvoff[j], soff, 0);
        rg[j] = *reinterpret_cast<float4*>(&v);
      }
    }
  };
  auto load_x = [&](int xr) {  // image row xr, zeros where the image has no such row
    const bool row_in = (unsigned)xr < (unsigned)a.H;
    const int soff = row_in ? xr * a.W * 4 : 0;
#pragma unroll
    for (int j = 0; j < W3_PX; ++j) {
      v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_x, row_in ? (int)xvoff[j] : (int)OOB_OFFSET, soff, 0);
      rx[j] = *reinterpret_cast<float4*>(&v);
    }
  };
  auto gate_dy = [&]() {  // in registers, ahead of the barrier that precedes the stores
    if (GATE > 0) {
#pragma unroll
      for (int j = 0; j < W3_PD; ++j) {
        const float4 y = GATE == 1 ? rd[j] : rg[j];
        const float4 g = GATE == 1 ? make_float4(dy_scalar, dy_scalar, dy_scalar, dy_scalar) : rd[j];
        rd[j] = make_float4(y.x > 0.f ? g.x : 0.f, y.y > 0.f ? g.y : 0.f, y.z > 0.f ? g.z : 0.f, y.w > 0.f ? g.w : 0.f);
      }
    }
    if (sum_rows) {
#pragma unroll
      for (int j = 0; j < W3_PD; ++j) row_sum[j] += (rd[j].x + rd[j].y) + (rd[j].z + rd[j].w);
    }
  };
  // rows are 8-byte, not 16-byte, aligned in LDS (66 words): a piece goes as two 8-byte stores
  auto store_dy = [&]() {
#pragma unroll
    for (int j = 0; j < W3_PD; ++j)
      if (dl[j] >= 0) {
        *reinterpret_cast<float2*>(&Ds[dl[j]]) = make_float2(rd[j].x, rd[j].y);
        *reinterpret_cast<float2*>(&Ds[dl[j] + 2]) = make_float2(rd[j].z, rd[j].w);
      }
  };
  auto store_x = [&](int xr) {
    float* slot = Xs + ((xr + 4) & 3) * W3_SLOT;
#pragma unroll
    for (int j = 0; j < W3_PX; ++j)
      if (xl[j] >= 0) {
        *reinterpret_cast<float2*>(&slot[xl[j]]) = make_float2(rx[j].x, rx[j].y);
        *reinterpret_cast<float2*>(&slot[xl[j] + 2]) = make_float2(rx[j].z, rx[j].w);
      }
  };

  floatx16 acc[9];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  if (p_begin < p_end) {
    __syncthreads();  // the zeros are in place
    // the three rows of x under the first output row, and its row of dy
    for (int r = 0; r < 3; ++r) {
      load_x(p_begin - a.ph + r);
      store_x(p_begin - a.ph + r);
    }
    load_dy(p_begin);
    gate_dy();
    store_dy();
    __syncthreads();
    const int steps8 = (a.Q + 7) >> 3;  // groups of four MFMA steps = eight pixels (the cache is zero beyond Q)
    const float* a_at = Ds + (wave * 32 + l32) * W3_LD + h;
    const int b_lane = l32 * W3_LD + h + 2 - a.pw;
    for (int p = p_begin; p < p_end; ++p) {
      const bool more = p + 1 < p_end;
      if (more) {
        load_dy(p + 1);
        load_x(p + 3 - a.ph);
      }
      const float* b_at[3];
#pragma unroll
      for (int r = 0; r < 3; ++r) b_at[r] = Xs + ((p - a.ph + r + 4) & 3) * W3_SLOT + b_lane;
      // the four dy values of a group of steps are read one group ahead (the cache row is 66 words: the read past
      // the last group stays inside it)
      float a_cur[4], a_nxt[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a_cur[i] = a_at[2 * i];
      for (int g8 = 0; g8 < steps8; ++g8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) a_nxt[i] = a_at[8 * g8 + 8 + 2 * i];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int q = 8 * g8 + 2 * i;
#pragma unroll
          for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int sx = 0; sx < 3; ++sx)
              acc[3 * r + sx] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[i], b_at[r][q + sx], acc[3 * r + sx], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) a_cur[i] = a_nxt[i];
      }
      if (more) {
        gate_dy();
        __syncthreads();
        store_dy();
        store_x(p + 3 - a.ph);
        __syncthreads();
      }
    }
  }

  // partial gradient of this work-group, [tap][k][c]
  float* out = a.part + (int64_t)split * 9 * a.K * a.C;
  const int c = c0 + l32;
  if (c < a.C) {
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int k = k0 + wave * 32 + acc_row(v, h);
        if (k < a.K) out[((int64_t)t * a.K + k) * a.C + c] = acc[t][v];
      }
  }
  if (sum_rows) {  // the pieces of a row of dy belong to Q / 4 neighbouring threads: added per row in piece order
    __syncthreads();
#pragma unroll
    for (int j = 0; j < W3_PD; ++j) Xs[tid + 256 * j] = row_sum[j];
    __syncthreads();
    if (tid < W3_BK && k0 + tid < a.K) {
      float sum = 0.f;
      for (int i = 0; i < Q4; ++i) sum += Xs[tid * Q4 + i];
      a.bias_part[(int64_t)split * a.K + k0 + tid] = sum;
    }
  }
}

// [9][K][C] -> [K][C][9]
__global__ __launch_bounds__(TPB) void wgrad3x3_order_kernel(const float* __restrict__ src, float* __restrict__ dw, int K, int C) {
  const int64_t total = (int64_t)9 * K * C;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < total; i += (int64_t)gridDim.x * TPB) {
    const int t = (int)(i / ((int64_t)K * C));
    const int64_t kc = i - (int64_t)t * K * C;
    dw[kc * 9 + t] = src[i];
  }
}

// ---- 3 x 3, unit stride and dilation, padding 0 or 1: rows of the source cached in LDS --------------------
// The gathers above write every source element into LDS once per tap it serves (nine times for a 3 x 3 kernel).
// Here a work-group keeps, for eight input channels at a time, the three source rows under each output row of its
// 128-pixel tile in LDS, each row once, with a zero column on either side and zero rows where the image ends, so
// that nothing is padded in memory and no tap is ever tested: the B fragment of tap (r, s) for a lane's pixel is
// the word at (its row + r, its column + s), an LDS read whose offset is a constant of the instruction. The
// reduction over one chunk is 8 channels x 9 taps = 72 long; the MFMA takes it in pairs (half-wave h holds the
// second element), and the pair is made of the SAME tap in two neighbouring channels, so the half-waves differ by
// one cached channel, a constant folded into the lane's base address. Within a chunk, element (group j, row, h, i)
// of the packed weights belongs to step 4j + i = 9 * (channel pair) + 3r + s and to channel 2 * (channel pair) + h.
// The weights do not pass through LDS at all (see the tile function). 72 or 144 MFMAs per wave between two barriers
// (the dense kernel has 64 at its large tile), three or four work-groups per CU.
struct DirectArgs {
  const float* src;      // [N, Cred, SH, SW]
  const float* gscalar;  // GATE 1: src is the stored output y; the cotangent is *gscalar where y > 0, zero elsewhere
  const float* wp;    // [chunks][9 groups][tiles_m * BM][8], packed as described above
  const float* bias;
  float* out;         // [N, Mrows, OH, OW]
  int Mrows, Cred, chunks, OH, OW, SH, SW, Ncols, NOH;
  int py, px;         // zero rows / columns in front of the source (0 or 1)
  int MR, plane;      // output rows a pixel tile can touch; floats per cached channel = 3 * MR * PITCH + 32
  int tasks;          // 16-byte pieces of source rows per chunk: 8 * 3 * MR * SW / 4
  FastDiv d_ohw, d_ow, d_oh, d_f4row;
  FastDiv d_tiles_m;
  const int2* plan;               // staging plan of a 128-pixel tile (2048 entries) and of a 64-pixel tile (2048 more), see direct3x3_plan
  int tiles_m, relu;
  int full_blocks, full_tiles_n;  // tiles of 128 pixels: full_tiles_n per tile row
  int MR_half, tasks_half;        // the same for the 64-pixel tiles behind them
  int64_t src_bytes, wp_bytes, out_bytes;
};

// One tile: rows [tm * 64 * FM, ...) of the output channels, pixels [n0, n0 + 64 * FN). MR / tasks: the cache rows and
// staging pieces a tile of that many pixels needs.
template <int FM, int FN, int PITCH, bool FWD, int GATE>
__device__ __forceinline__ void direct3x3_tile(const DirectArgs& a, int tm, int n0, int MR, const int2* __restrict__ plan, float* smem) {
  constexpr int BM = 64 * FM, CC = 8, KC = 72, PB = 8;
  float* Bc = smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, h = lane >> 5;
  const int m0 = tm * BM;
  const int ohw = a.OH * a.OW;
  // global output row (image * OH + row) of the tile's first pixel
  const int img0 = (int)fdiv((uint32_t)n0, a.d_ohw);
  const int grow0 = img0 * a.OH + (int)fdiv((uint32_t)(n0 - img0 * ohw), a.d_ow);

  // What a wave does outside its MFMA loop is vector-ALU work that the MFMAs of the SIMD's other waves wait for, so the
  // set-up is kept short: which cached row and which 16-byte piece of it a thread stages (task u = tid + 256 p) is the
  // same for every tile and comes from a table made once per call (direct3x3_plan); what depends on the tile, the
  // source row under each cached row, is worked out by one lane per cached row and handed over through LDS.
  int2 te[PB];
#pragma unroll
  for (int p = 0; p < PB; ++p) te[p] = plan[tid + p * 256];
  int* rowbase = reinterpret_cast<int*>(smem + CC * a.plane);  // [3 * MR] byte offsets of the source rows, channel 0
  if (tid < 3 * MR) {
    // cached row 3g + r holds source row oy - py + r of the image that output row grow0 + g belongs to, or zeros when
    // that row does not exist
    const int g = (int)((uint32_t)tid * 43691u >> 17), r = tid - 3 * g, grow = grow0 + g;
    uint32_t off = OOB_OFFSET;
    if (grow < a.NOH) {
      const int img = (int)fdiv((uint32_t)grow, a.d_oh), y = grow - img * a.OH - a.py + r;
      if ((unsigned)y < (unsigned)a.SH) off = (uint32_t)((img * a.Cred * a.SH + y) * a.SW) * 4u;
    }
    rowbase[tid] = (int)off;
  }
  // the columns on either side of a cached row are never written again: zero them once (everything between them is
  // rewritten with every chunk, zeros included where a row lies outside its image)
  if (tid < 3 * MR) {
#pragma unroll
    for (int cc = 0; cc < CC; ++cc) {
      const int at = cc * a.plane + tid * PITCH;
      Bc[at + 3] = 0.f;
      Bc[at + 4 + a.SW] = 0.f;
    }
  }
  __syncthreads();
  uint32_t goff[PB];
  int loff[PB];
#pragma unroll
  for (int p = 0; p < PB; ++p) {
    const bool task = te[p].x >= 0;  // (entries past the last task are negative)
    const uint32_t rb = (uint32_t)rowbase[(te[p].x >> 16) & 63];
    goff[p] = (task && rb != OOB_OFFSET) ? rb + (uint32_t)te[p].y : OOB_OFFSET;
    loff[p] = task ? (te[p].x & 0xffff) : -1;
  }
  const __amdgpu_buffer_rsrc_t rs_src = make_rsrc(a.src, a.src_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(a.wp, a.wp_bytes);
  const uint32_t src_step = (uint32_t)(CC * a.SH * a.SW) * 4u, w_step = (uint32_t)(a.tiles_m * BM * KC) * 4u;
  const float gs = GATE == 1 ? a.gscalar[0] : 0.f;
  float4 rb[PB];
  auto load = [&](int chunk) {
#pragma unroll
    for (int p = 0; p < PB; ++p) {
      v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_src, (int)goff[p], (int)(chunk * src_step), 0);
      rb[p] = *reinterpret_cast<float4*>(&v);
    }
  };
  // GATE 1: what was staged is y; the cotangent is *gscalar where y > 0. Applied in registers ahead of the barrier that
  // precedes the stores (the work-group's other waves may still be in their MFMAs then; between the two barriers
  // nothing else runs). Rows outside the image were loaded as zeros and stay zeros.
  auto gate = [&]() {
    if (GATE == 1) {
#pragma unroll
      for (int p = 0; p < PB; ++p)
        rb[p] = make_float4(rb[p].x > 0.f ? gs : 0.f, rb[p].y > 0.f ? gs : 0.f, rb[p].z > 0.f ? gs : 0.f, rb[p].w > 0.f ? gs : 0.f);
    }
  };
  auto store = [&]() {
#pragma unroll
    for (int p = 0; p < PB; ++p)
      if (loff[p] >= 0) *reinterpret_cast<float4*>(&Bc[loff[p]]) = rb[p];
  };

  // this lane's pixels: cache position of tap (0, 0), with the half-wave's channel folded in
  int pix[FN];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    const int j = n0 + wn * 32 * FN + fn * 32 + l32;
    pix[fn] = h * a.plane;
    if (j < a.Ncols) {
      const int img = (int)fdiv((uint32_t)j, a.d_ohw), rem = j - img * ohw;
      const int oy = (int)fdiv((uint32_t)rem, a.d_ow), ox = rem - oy * a.OW;
      pix[fn] += 3 * (img * a.OH + oy - grow0) * PITCH + 4 + ox - a.px;
    }
  }
  const int a_row = wm * 32 * FM + l32;

  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);
  // The weights go from memory straight into the A fragments: every lane reads its own rows of the packed weights
  // (group jg of a chunk holds, for every row, the four steps of either half-wave: 32 bytes a row, 1 KiB a fragment
  // in one piece), three groups of four steps ahead of the MFMAs that use them. All work-groups read the same few
  // hundred KiB, which stay in L2; LDS holds the row cache alone.
  constexpr int AD = 3;  // groups in flight; 9 groups a chunk, so a group's slot is a constant of the unrolled loop
  uint32_t arow[FM];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) arow[fm] = (uint32_t)(((m0 + a_row + 32 * fm) * 8 + 4 * h) * 4);
  const uint32_t g_step = (uint32_t)(a.tiles_m * BM) * 32u;  // bytes between the groups of the packed weights
  float4 afn[AD][FM];
  auto fetch_a = [&](int chunk, int jg) {
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
      v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (int)arow[fm], (int)((chunk * (KC / 8) + jg) * g_step), 0);
      afn[jg % AD][fm] = *reinterpret_cast<float4*>(&v);
    }
  };
  load(0);
#pragma unroll
  for (int jg = 0; jg < AD; ++jg) fetch_a(0, jg);
  gate();
  __syncthreads();  // border columns zeroed before the first rows land in the cache
  store();
  __syncthreads();
  for (int chunk = 0; chunk < a.chunks; ++chunk) {
    const bool more = chunk + 1 < a.chunks;
    if (more) load(chunk + 1);
#pragma unroll
    for (int jg = 0; jg < KC / 8; ++jg) {  // nine groups of four steps
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int q = 4 * jg + i, ccp = q / 9, tap = q - 9 * ccp, r = tap / 3, sx = tap - 3 * r;
        float bf[FN];
#pragma unroll
        for (int fn = 0; fn < FN; ++fn) bf[fn] = Bc[pix[fn] + 2 * ccp * a.plane + r * PITCH + sx];
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          const float4& t = afn[jg % AD][fm];
          const float av = i == 0 ? t.x : (i == 1 ? t.y : (i == 2 ? t.z : t.w));
#pragma unroll
          for (int fn = 0; fn < FN; ++fn) acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bf[fn], acc[fm][fn], 0, 0, 0);
        }
      }
      // the group's slot is free once its MFMAs have been issued: the request for the group three further on goes
      // behind them, so that the fragments are used where they arrive and never copied
      if (jg + AD < KC / 8) fetch_a(chunk, jg + AD);
      else if (more) fetch_a(chunk + 1, jg + AD - KC / 8);
    }
    if (more) {
      gate();
      __syncthreads();
      store();
      __syncthreads();
    }
  }

  // the bias of this lane's rows, fetched before the stores (which the compiler must assume to alias it)
  float bias_v[FM][16];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm * 32 * FM + fm * 32 + acc_row(v, h);
      bias_v[fm][v] = (FWD && a.bias && m < a.Mrows) ? a.bias[m] : 0.f;
    }
  // A tile whose rows all exist, in an output of less than 2 GiB: buffer stores, one 32-bit offset per lane and pixel
  // column, the row's part of the address a scalar of the instruction, no test per element (a pixel past the end gets
  // an offset the descriptor rejects). What a wave does outside its MFMA loop is vector-ALU work that the SIMD's other
  // waves' MFMAs wait for, so the fewer instructions here the better.
  if (m0 + BM <= a.Mrows && a.out_bytes < (1ll << 31)) {
    const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(a.out, a.out_bytes);
    const uint32_t row_bytes = (uint32_t)ohw * 4u;
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
      const int j = n0 + wn * 32 * FN + fn * 32 + l32;
      const int img = (int)fdiv((uint32_t)j, a.d_ohw);
      const uint32_t at = j < a.Ncols ? (uint32_t)((img * a.Mrows + m0 + wm * 32 * FM + 4 * h) * ohw + (j - img * ohw)) * 4u : OOB_OFFSET;
#pragma unroll
      for (int fm = 0; fm < FM; ++fm)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float val = acc[fm][fn][v];
          if (FWD) {
            val += bias_v[fm][v];
            if (a.relu) val = val > 0.f ? val : 0.f;
          }
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(val), rs_out, (int)at, (int)((uint32_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * row_bytes), 0);
        }
    }
    return;
  }
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    const int j = n0 + wn * 32 * FN + fn * 32 + l32;
    if (j >= a.Ncols) continue;
    const int img = (int)fdiv((uint32_t)j, a.d_ohw);
    const int64_t col_off = (int64_t)img * a.Mrows * ohw + (j - (int64_t)img * ohw);
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 32 * FM + fm * 32 + acc_row(v, h);
        if (m < a.Mrows) {
          float val = acc[fm][fn][v];
          if (FWD) {
            val += bias_v[fm][v];
            if (a.relu) val = val > 0.f ? val : 0.f;
          }
          a.out[col_off + (int64_t)m * ohw] = val;
        }
      }
  }
}

// Whole tiles of 128 pixels first; what is left after the last full round over the CUs is cut into tiles of 64
// pixels, so that the CUs that get one more tile than the others get half a tile more (see run_direct3x3).
template <int FM, int PITCH, bool FWD, int GATE>
__global__ __launch_bounds__(256, 2) void conv_direct3x3_kernel(DirectArgs a) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int b = blockIdx.x;
  if (b < a.full_blocks) {
    int tm, tn;
    if (a.tiles_m <= 8) {  // tile_of_block for at most one band of tile rows, without its divisions by run-time values
      int lid = b;
      if ((a.full_blocks & 7) == 0) lid = (b & 7) * (a.full_blocks >> 3) + (b >> 3);
      tn = (int)fdiv((uint32_t)lid, a.d_tiles_m);
      tm = lid - tn * a.tiles_m;
    } else {
      tile_of_block(b, a.full_blocks, a.tiles_m, a.full_tiles_n, tm, tn);
    }
    direct3x3_tile<FM, 2, PITCH, FWD, GATE>(a, tm, tn * 128, a.MR, a.plan, smem);
  } else {
    const int hb = b - a.full_blocks, tn = (int)fdiv((uint32_t)hb, a.d_tiles_m), tm = hb - tn * a.tiles_m;
    direct3x3_tile<FM, 1, PITCH, FWD, GATE>(a, tm, a.full_tiles_n * 128 + tn * 64, a.MR_half, a.plan + 2048, smem);
  }
}

// The staging plan of conv_direct3x3_kernel: task u (a channel of the chunk, a cached row, a 16-byte piece of that row)
// as {LDS word of the piece | cached row << 16, byte offset of the piece from the start of its source row in channel 0
// of its image}; entries past the last task are negative. One table for 128-pixel tiles, one for 64-pixel tiles.
struct DirectPlanArgs {
  int2* plan;
  int MR, MR_half, f4row, plane, pitch, SH, SW;
};
constexpr int PLAN_BLOCKS = 4096 / TPB;
__device__ __forceinline__ void direct3x3_plan(const DirectPlanArgs& d, int u) {
  int2* __restrict__ plan = d.plan;
  const int MR = d.MR, MR_half = d.MR_half, f4row = d.f4row, plane = d.plane, pitch = d.pitch, SH = d.SH, SW = d.SW;
  const int mr = u < 2048 ? MR : MR_half, t = u & 2047;
  const int rowid = t / f4row, c4 = t - rowid * f4row;
  const int cc = rowid / (3 * mr), rr = rowid - cc * 3 * mr;
  int2 e = make_int2(-1, 0);
  if (t < 8 * 3 * mr * f4row) e = make_int2((cc * plane + rr * pitch + 4 + 4 * c4) | (rr << 16), (cc * SH * SW + 4 * c4) * 4);
  plan[u] = e;
}

// Weights in the order conv_direct3x3_kernel reads them. forward: rows m = output channel, reduced channel ch = input
// channel, tap (r, s); data gradient: rows m = input channel, reduced channel = output channel, tap (2 - r, 2 - s).
// (The last PLAN_BLOCKS work-groups of the launch write the staging plan instead: one launch for both.)
__global__ __launch_bounds__(TPB) void pack_direct3x3_kernel(const float* __restrict__ w, float* __restrict__ wp, int K, int C,
                                                             int rows_pad, int chunks, int flip, DirectPlanArgs plan) {
  const int packers = (int)gridDim.x - PLAN_BLOCKS;
  if ((int)blockIdx.x >= packers) {
    direct3x3_plan(plan, ((int)blockIdx.x - packers) * TPB + (int)threadIdx.x);
    return;
  }
  const int Mrows = flip ? C : K, Cred = flip ? K : C;
  const int64_t total = (int64_t)chunks * rows_pad * 72;
  for (int64_t idx = (int64_t)blockIdx.x * TPB + threadIdx.x; idx < total; idx += (int64_t)packers * TPB) {
    // [chunk][group j of four steps][row m][half-wave h][step i]: the 64 lanes of a fragment load (32 rows, both
    // half-waves) read 1 KiB in one piece
    const int e = (int)(idx & 7), h = e >> 2, i = e & 3;
    const int64_t rest = idx >> 3;
    const int m = (int)(rest % rows_pad), gj = (int)(rest / rows_pad), j = gj % 9, chunk = gj / 9;
    const int q = 4 * j + i, ccp = q / 9, tap = q - 9 * ccp, r = tap / 3, s = tap - 3 * r;
    const int ch = chunk * 8 + 2 * ccp + h;
    float v = 0.f;
    if (m < Mrows && ch < Cred)
      v = flip ? w[(((int64_t)ch * C + m) * 3 + (2 - r)) * 3 + (2 - s)] : w[(((int64_t)m * C + ch) * 3 + r) * 3 + s];
    wp[idx] = v;
  }
}

// ---- weight repacking -------------------------------------------------------------------------------
// fwd:  wp[k][t]          = w[k][t]                     t = (c, kz, r, s), rows padded to Kd_pad with zeros
// data: wp[c][(k,kz,r,s)] = w[k][c][kz][r][s]            (RS below is T*R*S)
__global__ __launch_bounds__(TPB) void pack_weights_kernel(const float* __restrict__ w, float* __restrict__ wp, int K, int C,
                                                           int RS, int Kd_pad, int transpose) {
  const int rows = transpose ? C : K;
  const int64_t total = (int64_t)rows * Kd_pad;
  const int kd = (transpose ? K : C) * RS;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < total; i += (int64_t)gridDim.x * TPB) {
    int m = (int)(i / Kd_pad), t = (int)(i - (int64_t)m * Kd_pad);
    float v = 0.f;
    if (t < kd) {
      if (!transpose) v = w[(int64_t)m * kd + t];
      else { int k = t / RS, rs = t - k * RS; v = w[((int64_t)k * C + m) * RS + rs]; }
    }
    wp[i] = v;
  }
}

// The set-up of a vectorised call in ONE launch: the first work-groups write the tap table, the next ones repack
// the weights (when there are any to repack), the rest make the zero-padded copy. The three are independent;
// as three launches they cost about ten microseconds of a call that lasts three hundred.
//   table[t], t = (ch, kz, r, s): byte offset ((ch*Dp + kz*dd)*Hp + r*dh)*Wp + s*dw inside a padded image; the data
//     gradient walks the taps in reverse (kz -> T-1-kz, r -> R-1-r, s -> S-1-s); entries past Kd get OOB_OFFSET.
//   padded copy: dst[pl][z][y][x] = src[pl][z - pz][y - py][x - px] where in range, else 0; padded rows are a whole
//     number of 16-byte pieces, one piece per thread (32-bit index arithmetic with precomputed divisions).
struct PrepArgs {
  const float* src; float* dst; int64_t rows_total; int D, H, W, Dp, Hp, Wp, pz, py, px;   // padded copy
  FastDiv d_w4, d_hp, d_dp;                                                                 // Wp / 4, Hp, Dp
  int* table; int tn, Kd, T, R, S, dd, dh, dw, flip;                                        // tap table
  const float* w; float* wp; int K, C, RS, Kd_pad, transpose;                               // weight repacking (w may be null)
  int table_blocks, pack_blocks;
};

__global__ __launch_bounds__(TPB) void conv_prep_kernel(PrepArgs a) {
  const int b = blockIdx.x;
  if (b < a.table_blocks) {
    int t = b * TPB + threadIdx.x;
    if (t >= a.tn) return;
    if (t >= a.Kd) { a.table[t] = (int)OOB_OFFSET; return; }
    int ch = t / (a.T * a.R * a.S), rem = t - ch * a.T * a.R * a.S, kz = rem / (a.R * a.S);
    rem -= kz * a.R * a.S;
    int r = rem / a.S, s = rem - r * a.S;
    if (a.flip) { kz = a.T - 1 - kz; r = a.R - 1 - r; s = a.S - 1 - s; }
    a.table[t] = (((ch * a.Dp + kz * a.dd) * a.Hp + r * a.dh) * a.Wp + s * a.dw) * 4;
  } else if (b < a.table_blocks + a.pack_blocks) {
    const int rows = a.transpose ? a.C : a.K;
    const int64_t total = (int64_t)rows * a.Kd_pad;
    const int kd = (a.transpose ? a.K : a.C) * a.RS;
    for (int64_t i = (int64_t)(b - a.table_blocks) * TPB + threadIdx.x; i < total; i += (int64_t)a.pack_blocks * TPB) {
      int m = (int)(i / a.Kd_pad), t = (int)(i - (int64_t)m * a.Kd_pad);
      float v = 0.f;
      if (t < kd) {
        if (!a.transpose) v = a.w[(int64_t)m * kd + t];
        else { int k = t / a.RS, rs = t - k * a.RS; v = a.w[((int64_t)k * a.C + m) * a.RS + rs]; }
      }
      a.wp[i] = v;
    }
  } else {
    // one 16-byte piece of a padded row per thread: interior pieces are one (unaligned) 16-byte load, pieces that touch
    // the zero columns load their elements one by one
    struct __attribute__((packed, aligned(4))) Quad { float x, y, z, w; };
    const int first = a.table_blocks + a.pack_blocks;
    const int W4 = a.Wp >> 2;
    const uint32_t total = (uint32_t)a.rows_total * (uint32_t)W4, stride = (uint32_t)(gridDim.x - first) * TPB;
    for (uint32_t idx = (uint32_t)(b - first) * TPB + threadIdx.x; idx < total; idx += stride) {
      const uint32_t row = fdiv(idx, a.d_w4), c4 = idx - row * (uint32_t)W4;
      const uint32_t slab = fdiv(row, a.d_hp);  // (plane, padded depth)
      const int sy = (int)(row - slab * (uint32_t)a.Hp) - a.py;
      const uint32_t pl = fdiv(slab, a.d_dp);
      const int sz = (int)(slab - pl * (uint32_t)a.Dp) - a.pz;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if ((unsigned)sy < (unsigned)a.H && (unsigned)sz < (unsigned)a.D) {
        const float* s = a.src + (((int64_t)pl * a.D + sz) * a.H + sy) * a.W;
        const int x0 = (int)(c4 * 4) - a.px;
        if (x0 >= 0 && x0 + 3 < a.W) {
          const Quad q = *reinterpret_cast<const Quad*>(s + x0);
          v = make_float4(q.x, q.y, q.z, q.w);
        } else {
          if ((unsigned)x0 < (unsigned)a.W) v.x = s[x0];
          if ((unsigned)(x0 + 1) < (unsigned)a.W) v.y = s[x0 + 1];
          if ((unsigned)(x0 + 2) < (unsigned)a.W) v.z = s[x0 + 2];
          if ((unsigned)(x0 + 3) < (unsigned)a.W) v.w = s[x0 + 3];
        }
      }
      reinterpret_cast<float4*>(a.dst)[idx] = v;
    }
  }
}

struct ConvIn {  // the descriptor fields of either entry-point family, depth first
  int64_t N, C, K, in[3], k[3], stride[3], pad[3], dil[3], groups;
};

int32_t make_params(const char* op, const ConvIn& d, ConvP& p) {
  if (d.N < 0 || d.C <= 0 || d.K <= 0) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: non-positive extent", op);
  if (d.groups != 1)
    return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: groups = %lld; only groups = 1 is implemented", op, (long long)d.groups);
  int64_t out[3];
  for (int i = 0; i < 3; ++i) {
    if (d.in[i] <= 0 || d.k[i] <= 0) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: non-positive extent", op);
    if (d.stride[i] <= 0 || d.dil[i] <= 0 || d.pad[i] < 0)
      return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: bad stride, dilation or padding", op);
    int64_t e = d.in[i] + 2 * d.pad[i] - d.dil[i] * (d.k[i] - 1) - 1;  // conv2d_op.mojo:65-84, conv3d_op.mojo:71-101
    if (e < 0) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: kernel larger than padded input", op);
    out[i] = e / d.stride[i] + 1;
    if (d.pad[i] >= (1 << 20) || d.dil[i] * d.k[i] >= (1 << 20) || d.stride[i] >= (1 << 20))
      return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: stride, padding or dilated kernel extent of 2^20 or more", op);
  }
  // element offsets are 32-bit with 4-byte scaling inside the gathers: every tensor must stay below 2^29 elements
  const int64_t lim = 1ll << 29;
  if (d.N * d.C * d.in[0] * d.in[1] * d.in[2] >= lim || d.N * d.K * out[0] * out[1] * out[2] >= lim ||
      d.K * d.C * d.k[0] * d.k[1] * d.k[2] >= lim)
    return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: tensor has 2^29 elements or more", op);
  p.N = (int)d.N; p.C = (int)d.C; p.K = (int)d.K;
  p.D = (int)d.in[0]; p.H = (int)d.in[1]; p.W = (int)d.in[2];
  p.T = (int)d.k[0]; p.R = (int)d.k[1]; p.S = (int)d.k[2];
  p.O = (int)out[0]; p.P = (int)out[1]; p.Q = (int)out[2];
  p.sd = (int)d.stride[0]; p.sh = (int)d.stride[1]; p.sw = (int)d.stride[2];
  p.pd = (int)d.pad[0]; p.ph = (int)d.pad[1]; p.pw = (int)d.pad[2];
  p.dd = (int)d.dil[0]; p.dh = (int)d.dil[1]; p.dw = (int)d.dil[2];
  return ENDIA_HIP_OK;
}

int32_t make_params(const endia_hip_conv2d_desc* d, ConvP& p) {
  if (!d) return endia::fail(ENDIA_HIP_ERR_INVALID, "conv2d: descriptor is null");
  ConvIn in = {d->N, d->C, d->K, {1, d->H, d->W}, {1, d->R, d->S}, {1, d->stride_h, d->stride_w},
               {0, d->pad_h, d->pad_w}, {1, d->dil_h, d->dil_w}, d->groups};
  return make_params("conv2d", in, p);
}

int32_t make_params(const endia_hip_conv3d_desc* d, ConvP& p) {
  if (!d) return endia::fail(ENDIA_HIP_ERR_INVALID, "conv3d: descriptor is null");
  ConvIn in = {d->N, d->C, d->K, {d->D, d->H, d->W}, {d->T, d->R, d->S},
               {d->stride[0], d->stride[1], d->stride[2]}, {d->padding[0], d->padding[1], d->padding[2]},
               {d->dilation[0], d->dilation[1], d->dilation[2]}, d->groups};
  return make_params("conv3d", in, p);
}

// Row length of a zero-padded copy: the padding on both sides, rounded up to whole 16-byte pieces so that the copy
// writes aligned float4s (the extra columns are zeros that no tap reaches).
inline int padded_row(int W, int px) { return (W + 2 * px + 3) & ~3; }

struct PoolBuf {  // scratch from the library's pool, returned on scope exit (stream-ordered reuse)
  void* p = nullptr;
  ~PoolBuf() { if (p) endia_hip_free(p); }
};

inline int grid_for(int64_t n) {
  int64_t b = (n + TPB - 1) / TPB, cap = (int64_t)endia::ctx().cu_count * 16;
  if (b > cap) b = cap;
  return (int)(b < 1 ? 1 : b);
}

int32_t pack_weights(const ConvP& p, const float* w, int transpose, int Kd_pad, PoolBuf& buf) {
  const int rows = transpose ? p.C : p.K;
  int32_t rc = endia_hip_malloc((int64_t)rows * Kd_pad * 4, &buf.p);
  if (rc) return rc;
  int64_t total = (int64_t)rows * Kd_pad;
  int blocks = (int)((total + TPB - 1) / TPB);
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(pack_weights_kernel, dim3(blocks), dim3(TPB), 0, endia::ctx().stream, w, static_cast<float*>(buf.p),
                     p.K, p.C, p.T * p.R * p.S, Kd_pad, transpose);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

// Padded copy of src (spad stays empty when the source needs none), tap table of n entries and (when w is given)
// repacked weights, from one launch.
int32_t prep_vec(const ConvP& p, const float* src, int64_t planes, int SD, int SH, int SW, int pz, int py, int px, int n_table,
                 int Kd, int flip, const float* w, int transpose, int Kd_pad, PoolBuf& spad, PoolBuf& table, PoolBuf& wp) {
  const int Dp = SD + 2 * pz, Hp = SH + 2 * py, Wp = padded_row(SW, px);
  // nothing to pad (a 1 x 1 kernel, an unpadded convolution over rows of whole 16-byte pieces): the source serves as it is
  const bool copy = pz || py || px || Wp != SW || (reinterpret_cast<uintptr_t>(src) & 15);
  int32_t rc = ENDIA_HIP_OK;
  if (copy && (rc = endia_hip_malloc(planes * Dp * Hp * Wp * 4, &spad.p))) return rc;
  if ((rc = endia_hip_malloc((int64_t)n_table * 4, &table.p))) return rc;
  PrepArgs a = {};
  a.src = src; a.dst = static_cast<float*>(spad.p); a.rows_total = copy ? planes * Dp * Hp : 0;
  a.D = SD; a.H = SH; a.W = SW; a.Dp = Dp; a.Hp = Hp; a.Wp = Wp; a.pz = pz; a.py = py; a.px = px;
  a.d_w4 = make_fastdiv(Wp / 4); a.d_hp = make_fastdiv(Hp); a.d_dp = make_fastdiv(Dp);
  a.table = static_cast<int*>(table.p); a.tn = n_table; a.Kd = Kd; a.T = p.T; a.R = p.R; a.S = p.S;
  a.dd = p.dd; a.dh = p.dh; a.dw = p.dw; a.flip = flip;
  a.table_blocks = (n_table + TPB - 1) / TPB;
  a.pack_blocks = 0;
  if (w) {
    const int rows = transpose ? p.C : p.K;
    if ((rc = endia_hip_malloc((int64_t)rows * Kd_pad * 4, &wp.p))) return rc;
    a.w = w; a.wp = static_cast<float*>(wp.p); a.K = p.K; a.C = p.C; a.RS = p.T * p.R * p.S; a.Kd_pad = Kd_pad; a.transpose = transpose;
    int64_t pb = ((int64_t)rows * Kd_pad + TPB - 1) / TPB;
    a.pack_blocks = (int)(pb > 2048 ? 2048 : pb);
  }
  int64_t pad_blocks = (a.rows_total * (Wp / 4) + TPB - 1) / TPB, cap = (int64_t)endia::ctx().cu_count * 16;
  if (pad_blocks > cap) pad_blocks = cap;
  if (pad_blocks < 1 && copy) pad_blocks = 1;
  hipLaunchKernelGGL(conv_prep_kernel, dim3((unsigned)(a.table_blocks + a.pack_blocks + pad_blocks)), dim3(TPB), 0,
                     endia::ctx().stream, a);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

// Fast path of forward / data gradient (see VecArgs). Returns 1 when the shape does not qualify.
int32_t run_igemm_vec(int mode, const ConvP& p, const float* src, const float* w, const float* bias, float* out, int relu) {
  const bool fwd = mode == MODE_FWD;
  const int OW = fwd ? p.Q : p.W, OH = fwd ? p.P : p.H, OD = fwd ? p.O : p.D;
  const int SD = fwd ? p.D : p.O, SH = fwd ? p.H : p.P, SW = fwd ? p.W : p.Q;
  const int Cred = fwd ? p.C : p.K, Mrows = fwd ? p.K : p.C;
  int pz, py, px, row_stride, depth_stride;
  if (fwd) {
    if (p.sw != 1 || OW % 4) return 1;
    pz = p.pd; py = p.ph; px = p.pw; row_stride = p.sh; depth_stride = p.sd;
  } else {  // transposed convolution with unit strides: pad by (R-1)*d - p
    if (p.sd != 1 || p.sh != 1 || p.sw != 1 || OW % 4) return 1;
    pz = (p.T - 1) * p.dd - p.pd; py = (p.R - 1) * p.dh - p.ph; px = (p.S - 1) * p.dw - p.pw;
    row_stride = 1; depth_stride = 1;
    if (pz < 0 || py < 0 || px < 0) return 1;
  }
  const int Dp = SD + 2 * pz, Hp = SH + 2 * py, Wp = padded_row(SW, px);
  const int Kd = Cred * p.T * p.R * p.S, Kd_pad = (Kd + 31) / 32 * 32;
  if ((int64_t)p.N * Cred * Dp * Hp * Wp >= (1ll << 29) || Kd_pad > 8192) return 1;
  // the last reads of a row group must stay inside the padded image rows: ox + 3 + (S-1)*dw <= Wp - 1 holds because
  // OW - 1 + (S-1)*dw <= Wp - 1 by the output-size rule; nothing else to check.
  PoolBuf spad, wp, table;
  int32_t rc = prep_vec(p, src, (int64_t)p.N * Cred, SD, SH, SW, pz, py, px, Kd_pad, Kd, fwd ? 0 : 1, w, fwd ? 0 : 1, Kd_pad,
                        spad, table, wp);
  if (rc) return rc;
  VecArgs a;
  a.src = spad.p ? static_cast<const float*>(spad.p) : src; a.wp = static_cast<const float*>(wp.p);
  a.table = static_cast<const int*>(table.p); a.bias = bias; a.out = out; a.relu = relu;
  a.Mrows = Mrows; a.OD = OD; a.OH = OH; a.OW = OW; a.Ncols = p.N * OD * OH * OW; a.Kd_pad = Kd_pad;
  a.img_floats = Cred * Dp * Hp * Wp; a.Wp = Wp; a.sh = row_stride; a.zstep = depth_stride * Hp * Wp;
  a.d_ovol = make_fastdiv(OD * OH * OW); a.d_ohw = make_fastdiv(OH * OW); a.d_ow = make_fastdiv(OW);
  a.src_bytes = (int64_t)p.N * Cred * Dp * Hp * Wp * 4;
  a.tiles_n = (a.Ncols + 127) / 128;
  hipStream_t s = endia::ctx().stream;
  const size_t dyn = (size_t)Kd_pad * 4;
  // 128-row tiles, or 64-row tiles when they waste fewer MFMA rows or spread more evenly over the CUs
  // (the busiest CU sets the time: ceil(tiles / CUs) against tiles / CUs)
  const double cus = (double)endia::ctx().cu_count;
  auto cost = [&](int bm) {
    double tm = (double)((Mrows + bm - 1) / bm), t = tm * a.tiles_n;
    double rounds = t >= cus ? ((int64_t)((t + cus - 1) / cus)) / (t / cus) : 1.0;
    return rounds * (tm * bm) / (double)Mrows;
  };
  if (Mrows <= 32) {  // a 32-row tile wastes no MFMA rows on a thin output
    a.tiles_m = 1;
    dim3 grid((unsigned)a.tiles_n);
    if (fwd) hipLaunchKernelGGL((conv_igemm_vec_kernel<1, 4, 1, 1, true>), grid, dim3(256), dyn, s, a);
    else hipLaunchKernelGGL((conv_igemm_vec_kernel<1, 4, 1, 1, false>), grid, dim3(256), dyn, s, a);
  } else if (cost(128) <= cost(64) * 0.97) {
    a.tiles_m = (Mrows + 127) / 128;
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n));
    if (fwd) hipLaunchKernelGGL((conv_igemm_vec_kernel<2, 2, 2, 2, true>), grid, dim3(256), dyn, s, a);
    else hipLaunchKernelGGL((conv_igemm_vec_kernel<2, 2, 2, 2, false>), grid, dim3(256), dyn, s, a);
  } else {
    a.tiles_m = (Mrows + 63) / 64;
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n));
    if (fwd) hipLaunchKernelGGL((conv_igemm_vec_kernel<1, 4, 2, 1, true>), grid, dim3(256), dyn, s, a);
    else hipLaunchKernelGGL((conv_igemm_vec_kernel<1, 4, 2, 1, false>), grid, dim3(256), dyn, s, a);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

// 3 x 3 kernels with unit stride and dilation and at most one zero row / column around the source
// (conv_direct3x3_kernel). Returns 1 when the shape does not qualify.
// gate_mode 1 (data gradient only): src is the stored output y of relu(conv + bias) and stands for a cotangent that
// is *gscalar where y > 0 and zero elsewhere. (A tensor cotangent gated in the staging loads was measured slower than
// writing the gated cotangent out first: twice the loads and 151 registers, three work-groups per CU instead of four.)
int32_t run_direct3x3(int mode, const ConvP& p, const float* src, const float* w, const float* bias, float* out, int relu,
                      int gate_mode = 0, const float* gscalar = nullptr) {
  const bool fwd = mode == MODE_FWD;
  if (p.T != 1 || p.D != 1 || p.R != 3 || p.S != 3 || p.dh != 1 || p.dw != 1 || p.sh != 1 || p.sw != 1 || p.sd != 1) return 1;
  const int OH = fwd ? p.P : p.H, OW = fwd ? p.Q : p.W, SH = fwd ? p.H : p.P, SW = fwd ? p.W : p.Q;
  const int Cred = fwd ? p.C : p.K, Mrows = fwd ? p.K : p.C;
  const int py = fwd ? p.ph : 2 - p.ph, px = fwd ? p.pw : 2 - p.pw;
  if (py < 0 || py > 1 || px < 0 || px > 1 || Cred % 8 || SW % 4 || (reinterpret_cast<uintptr_t>(src) & 15)) return 1;
  const int pitch = SW + 5 <= 64 ? 64 : (SW + 5 <= 128 ? 128 : 0);
  if (!pitch) return 1;
  const int MR = (127 + OW - 1) / OW + 1;
  const int tasks = 8 * 3 * MR * (SW / 4);
  // 64 output channels per work-group up to 128 channels in all (twice the tiles to spread over the CUs, four work-groups
  // per CU instead of three; measured the same speed as 128 at 128 channels), 128 beyond
  const int fm = Mrows > 128 ? 2 : 1, BM = 64 * fm;
  // a cached channel is 3 * MR rows plus half a row of banks, so that the two half-waves of a fragment read (one
  // channel apart) fall into opposite halves of the 64 LDS banks
  const int plane = 3 * MR * pitch + 32;
  const size_t lds = (size_t)8 * plane * 4 + 64 * 4;  // the row cache and one source-row offset per cached row
  if (tasks > 2048 || 3 * MR > 64 || lds > 64 * 1024 || (int64_t)p.N * Cred * SH * SW >= (1ll << 29)) return 1;
  DirectArgs a;
  a.tiles_m = (Mrows + BM - 1) / BM;
  a.chunks = Cred / 8;
  const int rows_pad = a.tiles_m * BM;
  PoolBuf wp, plan;
  int32_t rc = endia_hip_malloc((int64_t)a.chunks * rows_pad * 72 * 4, &wp.p);
  if (rc) return rc;
  if ((rc = endia_hip_malloc(4096 * sizeof(int2), &plan.p))) return rc;
  hipStream_t s = endia::ctx().stream;
  const DirectPlanArgs plan_args{static_cast<int2*>(plan.p), MR, (63 + OW - 1) / OW + 1, SW / 4, plane, pitch, SH, SW};
  hipLaunchKernelGGL(pack_direct3x3_kernel, dim3(grid_for((int64_t)a.chunks * rows_pad * 72) + PLAN_BLOCKS), dim3(TPB), 0, s, w,
                     static_cast<float*>(wp.p), p.K, p.C, rows_pad, a.chunks, fwd ? 0 : 1, plan_args);
  ENDIA_LAUNCH_CHECK();
  a.src = src; a.wp = static_cast<const float*>(wp.p); a.bias = bias; a.out = out; a.relu = relu;
  a.gscalar = gscalar;
  a.Mrows = Mrows; a.Cred = Cred; a.OH = OH; a.OW = OW; a.SH = SH; a.SW = SW; a.Ncols = p.N * OH * OW; a.NOH = p.N * OH;
  a.py = py; a.px = px; a.MR = MR; a.plane = plane; a.tasks = tasks;
  a.d_ohw = make_fastdiv(OH * OW); a.d_ow = make_fastdiv(OW); a.d_oh = make_fastdiv(OH); a.d_f4row = make_fastdiv(SW / 4);
  a.src_bytes = (int64_t)p.N * Cred * SH * SW * 4;
  a.wp_bytes = (int64_t)a.chunks * rows_pad * 72 * 4;
  a.out_bytes = (int64_t)p.N * Mrows * OH * OW * 4;
  // The busiest CU sets the time, and with t tiles on c CUs it works on ceil(t / c) of them. When the tiles beyond the
  // last full round are few (at most one for every other CU), they are cut into 64-pixel tiles: twice as many CUs get
  // half as much extra work. 200704 pixels, 64 channels per tile row: 1568 tiles = 6 rounds + 32 -> 6 rounds + 64 halves.
  const int tiles_n = (a.Ncols + 127) / 128, cus = endia::ctx().cu_count;
  const int total = a.tiles_m * tiles_n, beyond = total % cus;
  a.full_tiles_n = tiles_n;
  if (total > cus && beyond > 0 && beyond <= cus / 2 && cus % a.tiles_m == 0) a.full_tiles_n = (total - beyond) / a.tiles_m;
  a.full_blocks = a.tiles_m * a.full_tiles_n;
  const int left = a.Ncols - a.full_tiles_n * 128;  // pixels for the 64-pixel tiles
  const int half_tiles_n = left > 0 ? (left + 63) / 64 : 0;
  a.MR_half = (63 + OW - 1) / OW + 1;
  a.tasks_half = 8 * 3 * a.MR_half * (SW / 4);
  a.d_tiles_m = make_fastdiv(a.tiles_m);
  a.plan = static_cast<const int2*>(plan.p);
  const dim3 grid((unsigned)(a.full_blocks + a.tiles_m * half_tiles_n));
#define ENDIA_LAUNCH_DIRECT(FM, PITCH)                                                                                       \
  do {                                                                                                                       \
    if (fwd) hipLaunchKernelGGL((conv_direct3x3_kernel<FM, PITCH, true, 0>), grid, dim3(256), lds, s, a);                      \
    else if (gate_mode == 0) hipLaunchKernelGGL((conv_direct3x3_kernel<FM, PITCH, false, 0>), grid, dim3(256), lds, s, a);     \
    else hipLaunchKernelGGL((conv_direct3x3_kernel<FM, PITCH, false, 1>), grid, dim3(256), lds, s, a);                         \
  } while (0)
  if (fm == 2 && pitch == 64) ENDIA_LAUNCH_DIRECT(2, 64);
  else if (fm == 2) ENDIA_LAUNCH_DIRECT(2, 128);
  else if (pitch == 64) ENDIA_LAUNCH_DIRECT(1, 64);
  else ENDIA_LAUNCH_DIRECT(1, 128);
#undef ENDIA_LAUNCH_DIRECT
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t run_igemm(int mode, const ConvP& p, const float* src, const float* w, const float* bias, float* out, int relu) {
  {
    int32_t rc = run_direct3x3(mode, p, src, w, bias, out, relu);
    if (rc != 1) return rc;
    rc = run_igemm_vec(mode, p, src, w, bias, out, relu);
    if (rc != 1) return rc;
  }
  hipStream_t s = endia::ctx().stream;
  IgemmArgs a;
  const bool fwd = mode == MODE_FWD;
  a.src = src; a.bias = bias; a.out = out; a.relu = relu;
  a.Mrows = fwd ? p.K : p.C;
  a.Cred = fwd ? p.C : p.K;
  a.SD = fwd ? p.D : p.O; a.SH = fwd ? p.H : p.P; a.SW = fwd ? p.W : p.Q;
  a.OD = fwd ? p.O : p.D; a.OH = fwd ? p.P : p.H; a.OW = fwd ? p.Q : p.W;
  a.Kd = a.Cred * p.T * p.R * p.S;
  a.Kd_pad = (a.Kd + 3) / 4 * 4;
  a.Ncols = p.N * a.OD * a.OH * a.OW;
  a.T = p.T; a.R = p.R; a.S = p.S; a.sd = p.sd; a.sh = p.sh; a.sw = p.sw; a.pd = p.pd; a.ph = p.ph; a.pw = p.pw;
  a.dd = p.dd; a.dh = p.dh; a.dw = p.dw;
  a.d_trs = make_fastdiv(p.T * p.R * p.S); a.d_rs = make_fastdiv(p.R * p.S); a.d_s = make_fastdiv(p.S);
  a.d_ovol = make_fastdiv(a.OD * a.OH * a.OW); a.d_ohw = make_fastdiv(a.OH * a.OW); a.d_ow = make_fastdiv(a.OW);
  a.d_sd = make_fastdiv(p.sd); a.d_sh = make_fastdiv(p.sh); a.d_sw = make_fastdiv(p.sw);
  a.src_bytes = (int64_t)p.N * a.Cred * a.SD * a.SH * a.SW * 4;

  PoolBuf wp;
  int32_t rc = pack_weights(p, w, fwd ? 0 : 1, a.Kd_pad, wp);
  if (rc) return rc;
  a.wp = static_cast<const float*>(wp.p);
  a.tiles_n = (a.Ncols + 127) / 128;
  if (a.Mrows <= 32) {
    a.tiles_m = 1;
    dim3 grid((unsigned)a.tiles_n);
    if (fwd) hipLaunchKernelGGL((conv_igemm_kernel<MODE_FWD, 1, 4, 1, 1>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_igemm_kernel<MODE_BWD_DATA, 1, 4, 1, 1>), grid, dim3(256), 0, s, a);
  } else if (a.Mrows > 64) {
    a.tiles_m = (a.Mrows + 127) / 128;
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n));
    if (fwd) hipLaunchKernelGGL((conv_igemm_kernel<MODE_FWD, 2, 2, 2, 2>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_igemm_kernel<MODE_BWD_DATA, 2, 2, 2, 2>), grid, dim3(256), 0, s, a);
  } else {  // up to 64 output channels: a 64 x 128 tile wastes no MFMA rows
    a.tiles_m = 1;
    dim3 grid((unsigned)a.tiles_n);
    if (fwd) hipLaunchKernelGGL((conv_igemm_kernel<MODE_FWD, 1, 4, 2, 1>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_igemm_kernel<MODE_BWD_DATA, 1, 4, 2, 1>), grid, dim3(256), 0, s, a);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t conv_fwd(const char* who, const ConvP& p, const float* x, const float* w, const float* bias, float* y, int32_t act) {
  if (!(act == ENDIA_OP_IDENTITY || act == ENDIA_OP_RELU))
    return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: activation must be identity or relu", who);
  if ((int64_t)p.N * p.K * p.O * p.P * p.Q == 0) return ENDIA_HIP_OK;
  if (!(x && w && y)) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  return run_igemm(MODE_FWD, p, x, w, bias, y, act == ENDIA_OP_RELU ? 1 : 0);
}

int32_t conv_bwd_data(const char* who, const ConvP& p, const float* dy, const float* w, float* dx) {
  int64_t total = (int64_t)p.N * p.C * p.D * p.H * p.W;
  if (total == 0) return ENDIA_HIP_OK;
  if (!dx) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: dx is null", who);
  if ((int64_t)p.O * p.P * p.Q == 0) return endia_hip_fill(dx, total, 0.f);
  if (!(dy && w)) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  return run_igemm(MODE_BWD_DATA, p, dy, w, nullptr, dx, 0);
}

// The vectorised weight-gradient kernel serves unit stride along the row, output rows that are whole 16-byte pieces
// and 32-bit offsets into the padded copy. `rows` is the tensor its A operand is loaded from.
bool wgrad_vec_ok(const ConvP& p, const float* rows) {
  const int Dp = p.D + 2 * p.pd, Hp = p.H + 2 * p.ph, Wp = padded_row(p.W, p.pw);
  return p.sw == 1 && p.Q % 4 == 0 && (int64_t)p.N * p.C * Dp * Hp * Wp < (1ll << 29) &&
         (reinterpret_cast<uintptr_t>(rows) & 15) == 0;
}

// The row-cache weight gradient (conv_wgrad3x3_kernel) where it applies: 1 if it does not. Same gate modes and bias
// sums as conv_bwd_weight below.
int32_t run_wgrad3x3(const ConvP& p, const float* x, const float* dy, float* dw, int gate_mode, const float* gate, float* db) {
  if (g_forced_path == 1) return 1;
  if (p.T != 1 || p.D != 1 || p.R != 3 || p.S != 3 || p.dh != 1 || p.dw != 1 || p.sh != 1 || p.sw != 1 || p.sd != 1) return 1;
  if (p.ph < 0 || p.ph > 1 || p.pw < 0 || p.pw > 1 || p.W % 4 || p.Q % 4 || p.Q < 8 || p.Q > 56) return 1;
  const float* rows = gate_mode == 1 ? gate : dy;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(rows) | (gate_mode == 2 ? reinterpret_cast<uintptr_t>(gate) : 0)) & 15) return 1;
  const int64_t x_bytes = (int64_t)p.N * p.C * p.H * p.W * 4, dy_bytes = (int64_t)p.N * p.K * p.P * p.Q * 4;
  if (x_bytes >= (1ll << 31) || dy_bytes >= (1ll << 31)) return 1;
  Wgrad3Args a;
  const int tiles_k = (p.K + W3_BK - 1) / W3_BK;
  a.tiles_c = (p.C + W3_BC - 1) / W3_BC;
  // few channels would leave most of the 128 x 32 tile's MFMA rows or columns multiplying zeros: the gather kernels have smaller tiles
  if ((double)tiles_k * W3_BK * a.tiles_c * W3_BC > 1.5 * (double)p.K * p.C && g_forced_path != 2) return 1;
  const int64_t tiles = (int64_t)tiles_k * a.tiles_c;
  // about two work-groups per CU in all (what a CU holds), each on a run of output rows of one image
  int64_t per_image = (2 * (int64_t)endia::ctx().cu_count + tiles * p.N - 1) / (tiles * p.N);
  if (per_image < 1) per_image = 1;
  if (per_image > p.P) per_image = p.P;
  a.rows_per_wg = (int)((p.P + per_image - 1) / per_image);
  a.wgs_per_image = (p.P + a.rows_per_wg - 1) / a.rows_per_wg;
  const int64_t splits = (int64_t)p.N * a.wgs_per_image;
  if (splits > 65535 || tiles > (1ll << 30)) return 1;
  const int64_t taps = (int64_t)9 * p.K * p.C;
  PoolBuf part, bias_part;
  int32_t rc;
  if ((rc = endia_hip_malloc(splits * taps * 4, &part.p))) return rc;
  float* db_part = db;
  if (db && splits > 1) {
    if ((rc = endia_hip_malloc(splits * p.K * 4, &bias_part.p))) return rc;
    db_part = static_cast<float*>(bias_part.p);
  }
  a.x = x; a.dy = dy; a.gate = gate; a.part = static_cast<float*>(part.p); a.bias_part = db_part;
  a.C = p.C; a.H = p.H; a.W = p.W; a.K = p.K; a.P = p.P; a.Q = p.Q; a.ph = p.ph; a.pw = p.pw;
  a.x_bytes = x_bytes; a.dy_bytes = dy_bytes;
  hipStream_t s = endia::ctx().stream;
  const dim3 grid((unsigned)tiles, (unsigned)splits);
  if (gate_mode == 0) hipLaunchKernelGGL((conv_wgrad3x3_kernel<0>), grid, dim3(256), 0, s, a);
  else if (gate_mode == 1) hipLaunchKernelGGL((conv_wgrad3x3_kernel<1>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((conv_wgrad3x3_kernel<2>), grid, dim3(256), 0, s, a);
  ENDIA_LAUNCH_CHECK();
  if (splits > 1) {  // partials added in split order; the last stage of the sum stores [tap][k][c] as the weights' [k][c][tap]
    // (the bias gradient's partial sums ride in the launch of the weight gradient's last stage)
    if (db) return endia::col_reduce_with_rider(splits, taps, (int64_t)p.K * p.C, a.part, dw, splits, p.K, db_part, db);
    return endia::col_reduce_transposed(splits, taps, (int64_t)p.K * p.C, a.part, dw);
  }
  hipLaunchKernelGGL(wgrad3x3_order_kernel, dim3(grid_for(taps)), dim3(TPB), 0, s, a.part, dw, p.K, p.C);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

// gate_mode 0: the plain weight gradient. 1 / 2 (only where wgrad_vec_ok): dy (1: one float, 2: a tensor) counts
// where gate > 0. db (may be null, only where wgrad_vec_ok) receives the sums of the (gated) dy over n, o, p, q.
int32_t conv_bwd_weight(const char* who, const ConvP& p, const float* x, const float* dy, float* dw, int gate_mode = 0,
                        const float* gate = nullptr, float* db = nullptr) {
  const int Kd = p.C * p.T * p.R * p.S;
  const int64_t taps = (int64_t)p.K * Kd;
  if (!dw) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: dw is null", who);
  const int64_t total_j = (int64_t)p.N * p.O * p.P * p.Q;
  if (total_j == 0) return endia_hip_fill(dw, taps, 0.f);
  if (!(x && dy)) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  {
    int32_t rc3 = run_wgrad3x3(p, x, dy, dw, gate_mode, gate, db);
    if (rc3 != 1) return rc3;
  }
  hipStream_t s = endia::ctx().stream;

  WgradArgs a;
  a.x = x; a.dy = dy;
  a.N = p.N; a.C = p.C; a.D = p.D; a.H = p.H; a.W = p.W; a.K = p.K; a.T = p.T; a.R = p.R; a.S = p.S;
  a.O = p.O; a.P = p.P; a.Q = p.Q;
  a.sd = p.sd; a.sh = p.sh; a.sw = p.sw; a.pd = p.pd; a.ph = p.ph; a.pw = p.pw; a.dd = p.dd; a.dh = p.dh; a.dw = p.dw;
  a.Kd = Kd;
  a.total_j = (int)total_j;
  a.d_opq = make_fastdiv(p.O * p.P * p.Q); a.d_pq = make_fastdiv(p.P * p.Q); a.d_q = make_fastdiv(p.Q);
  a.d_trs = make_fastdiv(p.T * p.R * p.S); a.d_rs = make_fastdiv(p.R * p.S); a.d_s = make_fastdiv(p.S);
  a.x_bytes = (int64_t)p.N * p.C * p.D * p.H * p.W * 4;
  a.dy_bytes = (int64_t)p.N * p.K * p.O * p.P * p.Q * 4;
  const int Dp = p.D + 2 * p.pd, Hp = p.H + 2 * p.ph, Wp = padded_row(p.W, p.pw);
  const bool vec = wgrad_vec_ok(p, gate_mode == 1 ? gate : dy) && (gate_mode != 2 || (reinterpret_cast<uintptr_t>(gate) & 15) == 0);
  if ((gate_mode || db) && !vec) return endia::fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: gated weight gradient outside the vectorised kernel", who);
  // 64-wide tiles over the taps when the last 128-wide tile would be at most half full
  int bn = (vec && Kd % 128 != 0 && Kd % 128 <= 64) ? 64 : 128;
  // likewise 64-high tiles over the output channels
  const int bm = (vec && p.K % 128 != 0 && p.K % 128 <= 64) ? 64 : 128;
  // 192-wide tiles (six accumulator blocks a wave) where they cover the taps with no more padding than the above
  if (vec && bm == 128 && Kd >= 192 && (Kd + 191) / 192 * 192 <= (Kd + bn - 1) / bn * bn) bn = 192;
  a.tiles_m = (p.K + bm - 1) / bm;
  a.tiles_n = (Kd + bn - 1) / bn;
  // split the N*O*P*Q reduction so that as many work-groups exist as the CUs hold at once (4 each, 2 of the 192-wide
  // tile); every split reduces >= 256 columns
  int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  int64_t splits = ((int64_t)endia::ctx().cu_count * (bn == 192 ? 2 : 4) + tiles - 1) / tiles;
  int64_t max_splits = (total_j + 255) / 256;
  if (splits > max_splits) splits = max_splits;
  if (splits > 1024) splits = 1024;
  if (splits < 1) splits = 1;
  int64_t chunk = ((total_j + splits - 1) / splits + 31) / 32 * 32;
  splits = (total_j + chunk - 1) / chunk;
  a.chunk = (int)chunk;

  PoolBuf part, bias_part;
  int32_t rc;
  float* db_part = db;
  if (splits > 1) {
    rc = endia_hip_malloc(splits * taps * 4, &part.p);
    if (rc) return rc;
    a.part = static_cast<float*>(part.p);
    if (db) {
      if ((rc = endia_hip_malloc(splits * p.K * 4, &bias_part.p))) return rc;
      db_part = static_cast<float*>(bias_part.p);
    }
  } else {
    a.part = dw;
  }
  dim3 grid((unsigned)tiles, (unsigned)splits);
  if (vec) {
    PoolBuf xpad, table, none;
    if ((rc = prep_vec(p, x, (int64_t)p.N * p.C, p.D, p.H, p.W, p.pd, p.ph, p.pw, a.tiles_n * bn, Kd, 0, nullptr, 0, 0, xpad, table,
                       none)))
      return rc;
    WgradVecArgs v;
    v.xpad = xpad.p ? static_cast<const float*>(xpad.p) : x; v.dy = dy; v.table = static_cast<const int*>(table.p); v.part = a.part;
    v.gate = gate; v.bias_part = db_part;
    v.K = p.K; v.Kd = Kd; v.OPQ = p.O * p.P * p.Q; v.PQ = p.P * p.Q; v.Q = p.Q; v.sh = p.sh; v.Wp = Wp;
    v.img_floats = p.C * Dp * Hp * Wp; v.zstep = p.sd * Hp * Wp;
    v.total_j = a.total_j; v.chunk = a.chunk; v.d_opq = a.d_opq; v.d_pq = a.d_pq; v.d_q = a.d_q;
    v.tiles_m = a.tiles_m; v.tiles_n = a.tiles_n;
    v.x_bytes = (int64_t)p.N * p.C * Dp * Hp * Wp * 4; v.dy_bytes = a.dy_bytes;
#define ENDIA_WGRAD_VEC(FM_, FN_)                                                                                     \
  do {                                                                                                                \
    if (gate_mode == 0) hipLaunchKernelGGL((conv_wgrad_vec_kernel<2, 2, FM_, FN_, 0>), grid, dim3(256), 0, s, v);      \
    else if (gate_mode == 1) hipLaunchKernelGGL((conv_wgrad_vec_kernel<2, 2, FM_, FN_, 1>), grid, dim3(256), 0, s, v); \
    else hipLaunchKernelGGL((conv_wgrad_vec_kernel<2, 2, FM_, FN_, 2>), grid, dim3(256), 0, s, v);                     \
  } while (0)
    if (bn == 192) ENDIA_WGRAD_VEC(2, 3);
    else if (bm == 128 && bn == 128) ENDIA_WGRAD_VEC(2, 2);
    else if (bm == 128) ENDIA_WGRAD_VEC(2, 1);
    else if (bn == 128) ENDIA_WGRAD_VEC(1, 2);
    else ENDIA_WGRAD_VEC(1, 1);
#undef ENDIA_WGRAD_VEC
  } else {
    hipLaunchKernelGGL((conv_wgrad_kernel<2, 2, 2, 2>), grid, dim3(256), 0, s, a);
  }
  ENDIA_LAUNCH_CHECK();
  if (splits > 1) {  // partials added in split order
    if (db) return endia::col_reduce_with_rider(splits, taps, 0, a.part, dw, splits, p.K, db_part, db);
    if ((rc = endia::col_reduce(1, splits, taps, a.part, dw, 1.f))) return rc;
  }
  return ENDIA_HIP_OK;
}

int32_t conv_bwd_bias(const char* who, const ConvP& p, const float* dy, float* db) {
  if (!db) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: db is null", who);
  const int64_t PQ = (int64_t)p.O * p.P * p.Q, rows = (int64_t)p.N * p.K;
  if (rows * PQ == 0) return endia_hip_fill(db, p.K, 0.f);
  if (!dy) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: dy is null", who);
  if (rows > 65535) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: N*K = %lld exceeds 65535", who, (long long)rows);
  // [N*K, O*P*Q] -> [N*K] with wave-shuffle row sums, then [N, K] -> [K]
  PoolBuf tmp;
  int32_t rc = endia_hip_malloc(rows * (int64_t)sizeof(float), &tmp.p);
  if (rc) return rc;
  rc = endia::row_reduce(rows, PQ, dy, static_cast<float*>(tmp.p), 1.f);
  if (!rc) rc = endia::col_reduce(1, p.N, p.K, static_cast<float*>(tmp.p), db, 1.f);
  return rc;
}

__global__ __launch_bounds__(TPB) void relu_gate_kernel(const float* __restrict__ y, const float* __restrict__ dy, int dy_is_scalar,
                                                        float* __restrict__ g, int64_t n, int vec) {
  const float sv = dy_is_scalar ? dy[0] : 0.f;
  const int64_t i0 = (int64_t)blockIdx.x * TPB + threadIdx.x, stride = (int64_t)gridDim.x * TPB;
  const int64_t n4 = vec ? n >> 2 : 0;
  for (int64_t i = i0; i < n4; i += stride) {  // 16 bytes per lane and stream
    const float4 a = reinterpret_cast<const float4*>(y)[i];
    const float4 d = dy_is_scalar ? make_float4(sv, sv, sv, sv) : reinterpret_cast<const float4*>(dy)[i];
    reinterpret_cast<float4*>(g)[i] = make_float4(a.x > 0.f ? d.x : 0.f, a.y > 0.f ? d.y : 0.f, a.z > 0.f ? d.z : 0.f, a.w > 0.f ? d.w : 0.f);
  }
  for (int64_t i = (n4 << 2) + i0; i < n; i += stride) g[i] = y[i] > 0.f ? (dy_is_scalar ? sv : dy[i]) : 0.f;
}

// Every gradient of y = relu(conv(x, w) + bias) from the stored y. dy * [y > 0] is formed inside the kernels as they
// load their operands where that is the faster way (see the policy below) and written out once, by one streaming
// kernel, where it is not; either way the bias gradient comes out of the weight-gradient launch where that is the
// vectorised kernel.
int32_t conv_bwd_relu(const char* who, const ConvP& p, const float* x, const float* w, const float* y, const float* dy,
                      int dy_is_scalar, float* dx, float* dw, float* db) {
  const int64_t out_total = (int64_t)p.N * p.K * p.O * p.P * p.Q;
  const int64_t x_total = (int64_t)p.N * p.C * p.D * p.H * p.W;
  int32_t rc;
  if (out_total == 0) {
    if (dw && (rc = endia_hip_fill(dw, (int64_t)p.K * p.C * p.T * p.R * p.S, 0.f))) return rc;
    if (db && (rc = endia_hip_fill(db, p.K, 0.f))) return rc;
    if (dx && x_total && (rc = endia_hip_fill(dx, x_total, 0.f))) return rc;
    return ENDIA_HIP_OK;
  }
  if (!(y && dy)) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  if ((dw && !x) || (dx && !w)) return endia::fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  PoolBuf gbuf;
  auto gated = [&](const float** g) -> int32_t {  // dy * [y > 0] in memory, made at most once
    if (!gbuf.p) {
      int32_t r = endia_hip_malloc(out_total * 4, &gbuf.p);
      if (r) return r;
      const int vec = ((reinterpret_cast<uintptr_t>(y) | (dy_is_scalar ? 0 : reinterpret_cast<uintptr_t>(dy))) & 15) == 0;
      hipLaunchKernelGGL(relu_gate_kernel, dim3(grid_for((out_total + 3) / 4)), dim3(TPB), 0, endia::ctx().stream, y, dy, dy_is_scalar,
                         static_cast<float*>(gbuf.p), out_total, vec);
      ENDIA_LAUNCH_CHECK();
    }
    *g = static_cast<const float*>(gbuf.p);
    return ENDIA_HIP_OK;
  };
  const float* g = nullptr;
  // A scalar cotangent is gated inside both kernels (they read y instead of a cotangent tensor). A tensor cotangent
  // is gated inside the weight-gradient kernel when only dw / db are wanted; with dx as well, writing the gated
  // cotangent out once (36 us at the 56 x 56 benchmark shape) and running the plain kernels on it is the faster way.
  const bool want_dx = dx && x_total;
  bool dx_done = false;
  if (want_dx && dy_is_scalar) {
    rc = run_direct3x3(MODE_BWD_DATA, p, y, w, nullptr, dx, 0, 1, dy);
    if (rc != 0 && rc != 1) return rc;
    dx_done = rc == 0;
  }
  if (want_dx && !dx_done) {
    if ((rc = gated(&g))) return rc;
    if ((rc = conv_bwd_data(who, p, g, w, dx))) return rc;
  }
  if (dw && g) {  // the gated cotangent exists: the plain kernel on it, which also sums db where it is the vectorised one
    const bool vec = wgrad_vec_ok(p, g);
    if ((rc = conv_bwd_weight(who, p, x, g, dw, 0, nullptr, vec ? db : nullptr))) return rc;
    if (db && !vec && (rc = conv_bwd_bias(who, p, g, db))) return rc;
  } else if (dw && wgrad_vec_ok(p, dy_is_scalar ? y : dy) && (dy_is_scalar || (reinterpret_cast<uintptr_t>(y) & 15) == 0)) {
    if ((rc = conv_bwd_weight(who, p, x, dy, dw, dy_is_scalar ? 1 : 2, y, db))) return rc;
  } else if (dw || db) {
    if ((rc = gated(&g))) return rc;
    if (dw && (rc = conv_bwd_weight(who, p, x, g, dw))) return rc;
    if (db && (rc = conv_bwd_bias(who, p, g, db))) return rc;
  }
  return ENDIA_HIP_OK;
}

}  // namespace

using namespace endia;

#define ENDIA_CONV_PARAMS(d)       \
  ENDIA_REQUIRE_INIT();            \
  ConvP p;                         \
  {                                \
    int32_t rc_ = make_params(d, p); \
    if (rc_) return rc_;           \
  }

extern "C" {

int32_t endia_hip_conv_force_path(int32_t path) {
  ENDIA_CHECK_ARG(path >= 0 && path <= 2, "endia_hip_conv_force_path: path %d is not one of 0, 1, 2", path);
  g_forced_path = path;
  return ENDIA_HIP_OK;
}

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
  ENDIA_CONV_PARAMS(d);
  return conv_fwd(__func__, p, x, w, bias, y, act);
}

int32_t endia_hip_conv2d_bwd_data(const endia_hip_conv2d_desc* d, const float* dy, const float* w, float* dx) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_data(__func__, p, dy, w, dx);
}

int32_t endia_hip_conv2d_bwd_weight(const endia_hip_conv2d_desc* d, const float* x, const float* dy, float* dw) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_weight(__func__, p, x, dy, dw);
}

int32_t endia_hip_conv2d_bwd_relu(const endia_hip_conv2d_desc* d, const float* x, const float* w, const float* y,
                                  const float* dy, int32_t dy_is_scalar, float* dx, float* dw, float* db) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_relu("conv2d_bwd_relu", p, x, w, y, dy, dy_is_scalar, dx, dw, db);
}

int32_t endia_hip_conv2d_bwd_bias(const endia_hip_conv2d_desc* d, const float* dy, float* db) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_bias(__func__, p, dy, db);
}

int32_t endia_hip_conv3d_out_shape(const endia_hip_conv3d_desc* d, int64_t* out_dhw) {
  ConvP p;
  int32_t rc = make_params(d, p);
  if (rc) return rc;
  ENDIA_CHECK_ARG(out_dhw, "endia_hip_conv3d_out_shape: null output");
  out_dhw[0] = p.O;
  out_dhw[1] = p.P;
  out_dhw[2] = p.Q;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_conv3d_fwd(const endia_hip_conv3d_desc* d, const float* x, const float* w, const float* bias, float* y,
                             int32_t act) {
  ENDIA_CONV_PARAMS(d);
  return conv_fwd(__func__, p, x, w, bias, y, act);
}

int32_t endia_hip_conv3d_bwd_data(const endia_hip_conv3d_desc* d, const float* dy, const float* w, float* dx) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_data(__func__, p, dy, w, dx);
}

int32_t endia_hip_conv3d_bwd_weight(const endia_hip_conv3d_desc* d, const float* x, const float* dy, float* dw) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_weight(__func__, p, x, dy, dw);
}

int32_t endia_hip_conv3d_bwd_bias(const endia_hip_conv3d_desc* d, const float* dy, float* db) {
  ENDIA_CONV_PARAMS(d);
  return conv_bwd_bias(__func__, p, dy, db);
}

}  // extern "C"
