// Building blocks shared by the fp32 MFMA kernels (dense GEMM and the implicit-GEMM convolutions):
// the LDS tile layouts, the per-K-tile MFMA loop, buffer-resource helpers and the work-group -> tile map.
//
// A work-group of WGM x WGN waves owns a (WGM*FM*32) x (WGN*FN*32) tile of C; each wave owns FM x FN
// blocks of v_mfma_f32_32x32x2_f32 (16 accumulator registers per block and lane). K advances 32 per
// tile. An operand tile is stored in LDS in one of two layouts:
//   K-major  [row][32 + 4] : fetched with one 128-bit read per four MFMA steps;
//   MN-major [k][width + 8]: fetched with 32-bit reads.
// The MFMA takes K in pairs (lanes 0-31 hold one k, lanes 32-63 the next). A sum over k may be taken in
// any order, so step s = 4j + i of a tile uses k = 8j + 4h + i for half-wave h; that permutation is
// what lets a K-major operand feed four steps from one 128-bit read. Both operands use it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mfma {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int BK = 32;
constexpr int LDK = BK + 4;  // row stride (floats) of a K-major tile
constexpr uint32_t OOB_OFFSET = 0x80000000u;  // byte offset beyond every descriptor built below

template <bool KMAJOR, int BMN>
struct TileShape {
  static constexpr int LD = KMAJOR ? LDK : BMN + 8;
  static constexpr int FLOATS = KMAJOR ? BMN * LDK : BK * (BMN + 8);
};

// Buffer resource over `bytes` bytes starting at base: loads at offsets >= bytes return zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float* base, int64_t bytes) {
  if (bytes < 0) bytes = 0;
  if (bytes > 0x7FFFFFF0ll) bytes = 0x7FFFFFF0ll;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float4 buffer_load_f4(__amdgpu_buffer_rsrc_t rs, uint32_t byte_off) {
  v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)byte_off, 0, 0);
  return *reinterpret_cast<float4*>(&v);
}

__device__ __forceinline__ float buffer_load_f1(__amdgpu_buffer_rsrc_t rs, uint32_t byte_off) {
  int v = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)byte_off, 0, 0);
  return __int_as_float(v);
}

// All MFMAs of one K tile. a_row / b_col: this lane's row of the A tile / column of the B tile for
// block 0 (blocks are 32 apart); h = lane / 32.
template <bool AK, bool BKM, int FM, int FN, int BM, int BN>
__device__ __forceinline__ void load_fragments(const float* __restrict__ As, const float* __restrict__ Bs, int a_row, int b_col,
                                               int h, int j, float (&af)[FM][4], float (&bf)[FN][4]) {
  constexpr int LDA = TileShape<AK, BM>::LD, LDB = TileShape<BKM, BN>::LD;
#pragma unroll
  for (int f = 0; f < FM; ++f) {
    if (AK) {
      float4 t = *reinterpret_cast<const float4*>(&As[(a_row + 32 * f) * LDA + 8 * j + 4 * h]);
      af[f][0] = t.x; af[f][1] = t.y; af[f][2] = t.z; af[f][3] = t.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) af[f][i] = As[(8 * j + 4 * h + i) * LDA + a_row + 32 * f];
    }
  }
#pragma unroll
  for (int f = 0; f < FN; ++f) {
    if (BKM) {
      float4 t = *reinterpret_cast<const float4*>(&Bs[(b_col + 32 * f) * LDB + 8 * j + 4 * h]);
      bf[f][0] = t.x; bf[f][1] = t.y; bf[f][2] = t.z; bf[f][3] = t.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) bf[f][i] = Bs[(8 * j + 4 * h + i) * LDB + b_col + 32 * f];
    }
  }
}

// The fragment of ONE 32-row block for step group j (the four steps 4j .. 4j + 3); row: this lane's row of the tile.
template <bool KMAJOR, int BMN>
__device__ __forceinline__ void load_fragment_block(const float* __restrict__ S, int row, int h, int j, float (&f)[4]) {
  constexpr int LD = TileShape<KMAJOR, BMN>::LD;
  if (KMAJOR) {
    float4 t = *reinterpret_cast<const float4*>(&S[row * LD + 8 * j + 4 * h]);
    f[0] = t.x; f[1] = t.y; f[2] = t.z; f[3] = t.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = S[(8 * j + 4 * h + i) * LD + row];
  }
}

// The same with the lane's part of the address already in `at` (its row and half-wave, in floats from `S`), so that
// block f and step group j only add constants that fit the instruction's offset field.
template <bool KMAJOR, int BMN>
__device__ __forceinline__ int fragment_lane_offset(int row, int h) {
  constexpr int LD = TileShape<KMAJOR, BMN>::LD;
  return KMAJOR ? row * LD + 4 * h : 4 * h * LD + row;
}
template <bool KMAJOR, int BMN>
__device__ __forceinline__ void load_fragment_at(const float* __restrict__ S, int at, int f, int j, float (&out)[4]) {
  constexpr int LD = TileShape<KMAJOR, BMN>::LD;
  if (KMAJOR) {
    float4 t = *reinterpret_cast<const float4*>(&S[at + 32 * f * LD + 8 * j]);
    out[0] = t.x; out[1] = t.y; out[2] = t.z; out[3] = t.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = S[at + (8 * j + i) * LD + 32 * f];
  }
}

template <bool AK, bool BKM, int FM, int FN, int BM, int BN>
__device__ __forceinline__ void compute_ktile(const float* __restrict__ As, const float* __restrict__ Bs, int a_row,
                                              int b_col, int h, floatx16 (&acc)[FM][FN]) {
  if constexpr (FM * FN == 1) {
    // One MFMA block per wave leaves registers to spare: the fragments of all four step groups are
    // fetched up front, so the LDS latency is paid once per K tile instead of once per group.
    float af[4][FM][4], bf[4][FN][4];
#pragma unroll
    for (int j = 0; j < BK / 8; ++j) load_fragments<AK, BKM, FM, FN, BM, BN>(As, Bs, a_row, b_col, h, j, af[j], bf[j]);
#pragma unroll
    for (int j = 0; j < BK / 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[j][0][i], bf[j][0][i], acc[0][0], 0, 0, 0);
  } else {
#pragma unroll
    for (int j = 0; j < BK / 8; ++j) {
      float af[FM][4], bf[FN][4];
      load_fragments<AK, BKM, FM, FN, BM, BN>(As, Bs, a_row, b_col, h, j, af, bf);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int fm = 0; fm < FM; ++fm)
#pragma unroll
          for (int fn = 0; fn < FN; ++fn)
            acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[fm][i], bf[fn][i], acc[fm][fn], 0, 0, 0);
    }
  }
}

template <int FM, int FN>
__device__ __forceinline__ void zero_acc(floatx16 (&acc)[FM][FN]) {
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// Row of the 32 x 32 block that accumulator register v of this lane holds (the column is lane % 32).
__device__ __forceinline__ int acc_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

// Loader of one K tile of a plain row-major matrix operand: global -> registers -> LDS.
// KMAJOR: tile rows are the M (or N) index and hold 32 consecutive k; otherwise tile rows are k and hold
// BMN consecutive m (or n). Buffer loads carry the bounds check in their descriptor: an offset past
// `records` returns zero, which pads the M/N edge of K-major operands and the K tail of MN-major
// operands. The other edge (K tail of a K-major operand, M/N edge of an MN-major operand) is folded
// into the offset, which becomes OOB_OFFSET. One 32-bit offset per pass is the only per-lane address
// state. VEC requires 4-float alignment of the base, the leading dimension and the contiguous extent. Without it
// (any view of any matrix: the reference's matmul has no alignment rule, matmul_op.mojo:93-199) a thread reads the same
// four elements with four 32-bit loads, each with its own bounds test, and the LDS side is unchanged.
template <bool KMAJOR, int BMN, int NTHREADS, bool VEC = true>
struct MatrixTileLoader {
  static constexpr int F4_PER_ROW = KMAJOR ? BK / 4 : BMN / 4;
  static constexpr int ROWS_PER_PASS = NTHREADS / F4_PER_ROW;
  static constexpr int PASSES = (KMAJOR ? BMN : BK) / ROWS_PER_PASS;
  static constexpr int LD = TileShape<KMAJOR, BMN>::LD;
  static_assert(PASSES >= 1 && PASSES * ROWS_PER_PASS == (KMAJOR ? BMN : BK), "tile does not divide among the threads");
  uint32_t voff[PASSES];
  const float* base;
  int64_t records, step;
  int c, lds_off;
  int nvalid;  // !VEC, MN-major: how many of this thread's four columns lie inside the operand
  float4 reg[PASSES];

  // X: the operand; mn0: first row (K-major) or column (MN-major) of the tile; MN, K: operand extents
  __device__ __forceinline__ void init(const float* X, int64_t ld, int mn0, int MN, int K, int tid) {
    const int r = tid / F4_PER_ROW;
    c = (tid % F4_PER_ROW) * 4;
    const int valid = MN - mn0 < BMN ? MN - mn0 : BMN;
    if (KMAJOR) {
      base = X + (int64_t)mn0 * ld;
      records = (((int64_t)valid - 1) * ld + K) * 4;
      step = BK * 4;
#pragma unroll
      for (int i = 0; i < PASSES; ++i) voff[i] = (uint32_t)(((int64_t)(r + i * ROWS_PER_PASS) * ld + c) * 4);
    } else {
      base = X + mn0;
      records = (((int64_t)K - 1) * ld + valid) * 4;
      step = (int64_t)BK * ld * 4;
#pragma unroll
      for (int i = 0; i < PASSES; ++i)
        voff[i] = (c < valid) ? (uint32_t)(((int64_t)(r + i * ROWS_PER_PASS) * ld + c) * 4) : OOB_OFFSET;
    }
    nvalid = valid - c;
    lds_off = r * LD + c;
  }
  // one piece of four consecutive elements; k_left as in load()
  __device__ __forceinline__ float4 load_piece(__amdgpu_buffer_rsrc_t rs, uint32_t o, int k_left) const {
    if constexpr (VEC) {
      if (KMAJOR) o = (c < k_left) ? o : OOB_OFFSET;
      return buffer_load_f4(rs, o);
    } else {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool in = KMAJOR ? (c + e < k_left) : (e < nvalid);
        v[e] = buffer_load_f1(rs, in ? o + 4u * e : OOB_OFFSET);
      }
      return make_float4(v[0], v[1], v[2], v[3]);
    }
  }
  // k_left = K - (first k of the tile being loaded); base/records already point at that tile
  __device__ __forceinline__ void load(int k_left) {
    __amdgpu_buffer_rsrc_t rs = make_rsrc(base, records);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) reg[i] = load_piece(rs, voff[i], k_left);
  }
  // The same two steps with the staging registers held by the caller (several tiles in flight at once).
  __device__ __forceinline__ void load_into(float4 (&dst)[PASSES], int k_left) {
    __amdgpu_buffer_rsrc_t rs = make_rsrc(base, records);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) dst[i] = load_piece(rs, voff[i], k_left);
  }
  __device__ __forceinline__ void store_from(float* lds, const float4 (&src)[PASSES]) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LD]) = src[i];
  }
  // One pass at a time, for loops that spread a tile's loads and LDS stores between their MFMAs.
  // No address arithmetic per pass: the caller has run mask_tail for a tile that reaches past the end of K.
  __device__ __forceinline__ void load_pass(int i, __amdgpu_buffer_rsrc_t rs) {
    static_assert(VEC, "the hand-scheduled loops read 16 bytes per request");
    reg[i] = buffer_load_f4(rs, voff[i]);
  }
  // A K-major tile that holds fewer than BK reduction elements: the pieces beyond them read as zeros from here on
  // (every later tile lies further out). The descriptor bounds do the same for an MN-major tile.
  __device__ __forceinline__ void mask_tail(int k_left) {
    if (KMAJOR) {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) voff[i] = (c < k_left) ? voff[i] : OOB_OFFSET;
    }
  }
  __device__ __forceinline__ void store_pass(float* lds, int i) {
    *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LD]) = reg[i];
  }
  __device__ __forceinline__ void store_pass_at(float* lds, int at, int i) {  // at: lds_off plus the tile's place in LDS
    *reinterpret_cast<float4*>(&lds[at + i * ROWS_PER_PASS * LD]) = reg[i];
  }
  __device__ __forceinline__ void advance() {
    base = reinterpret_cast<const float*>(reinterpret_cast<const char*>(base) + step);
    records -= step;
  }
  __device__ __forceinline__ void store(float* lds) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) *reinterpret_cast<float4*>(&lds[lds_off + i * ROWS_PER_PASS * LD]) = reg[i];
  }
};

// Map the linear work-group id to a tile. Work-groups are dealt round-robin to the 8 XCDs, each with
// a private L2, so first give every XCD a contiguous range of tile ids, then walk that range in
// column-major order inside bands of 8 tile-rows so that concurrently resident tiles share A rows
// and B columns.
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n, int& tm, int& tn) {
  int lid = bid;
  if ((nblocks & 7) == 0) {
    int per = nblocks >> 3;
    lid = (bid & 7) * per + (bid >> 3);
  }
  const int GM = 8;
  int band = GM * tiles_n;
  int g = lid / band;
  int first_m = g * GM;
  int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
  int r = lid - g * band;
  tm = first_m + r % gsz;
  tn = r / gsz;
}

// Unsigned division by a divisor fixed for the whole launch (n < 2^31): q = mulhi(n, mul) >> shift.
struct FastDiv {
  uint32_t mul, shift, d;
};

__device__ __forceinline__ uint32_t fdiv(uint32_t n, FastDiv f) {
  return f.d == 1 ? n : (__umulhi(n, f.mul) >> f.shift);
}

}  // namespace mfma

// host side
inline mfma::FastDiv make_fastdiv(uint32_t d) {
  mfma::FastDiv f;
  f.d = d;
  if (d <= 1) {
    f.mul = 0;
    f.shift = 0;
    return f;
  }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;  // l = ceil(log2 d) >= 1
  f.mul = (uint32_t)(((1ull << (31 + l)) + d - 1) / d);
  f.shift = l - 1;
  return f;
}
