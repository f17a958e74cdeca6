// fp32 GEMM on the CDNA4 matrix cores: matmul_fwd and both products of matmul_vjp
// (endia/functional/binary_ops/matmul_op.mojo:93-254, 278-283) as ONE kernel family.
//
// The reference makes the left operand contiguous, materialises a transposed copy of the right
// operand and then runs one dot product per output element (matmul_op.mojo:107-199). Here a
// transposed operand is only a different global->LDS path, selected by transA/transB, and the
// products run on v_mfma_f32_32x32x2_f32.
//
// Tiling: a 256-thread work-group (four 64-lane waves, 2 x 2) owns a 128 x 128 tile of C; each
// wave owns 64 x 64 as 2 x 2 MFMA blocks of 32 x 32 (64 accumulator registers per lane). Products
// too small to give every CU work at that size use 64 x 64 tiles (one MFMA block per wave). The K
// loop advances 32 at a time: the next tile's global loads (buffer loads, bounds-checked by their
// descriptor) are issued into registers before the MFMAs of the current tile and written to LDS
// after them. 128 registers per lane and 36 KiB of LDS per group give 4 groups per CU.
//
// LDS layouts. An operand whose K index is contiguous in memory ("K-major": A when transA = 0,
// B when transB = 1) is stored [row][32 + 4] and fetched with one 128-bit read per four MFMA
// steps; an operand whose M (or N) index is contiguous ("MN-major") is stored [k][128 + 8] and
// fetched with 32-bit reads. The MFMA takes K in pairs (lanes 0-31 hold k, lanes 32-63 hold
// k + 1); because a sum over k may be taken in any order, step s = 4j + i of a tile uses
// k = 8j + 4h + i for half-wave h, which is what makes the 128-bit fetch possible. Both
// operands use the same mapping.
#include "common.h"
#include "gemm_args.h"
#include "gemm_tile.h"

#include <stdlib.h>

#include <algorithm>
#include <functional>
#include <map>
#include <queue>
#include <type_traits>
#include <vector>

namespace {

using namespace mfma;

using namespace endia_gemm;  // GemmArgs, epilogue bodies, launchers of the one-wave-per-SIMD tiles (gemm_args.h)

// Backward of a small dense layer in ONE launch: the first nx work-groups compute the tiles of
// dx = (g W^T) * act'(aux) (both operands K-major, activation-gradient or plain epilogue), the others the tiles of
// dW = x^T g (both MN-major) and, in their first tile row, db = column sums of g. Both reductions are at most four
// K tiles long. For models of this size a step costs what its launches cost, and this halves the backward's.
template <int EPI_X>
__global__ __launch_bounds__(NTHREADS, 4) void linear_bwd_small_kernel(GemmArgs px, GemmArgs pw, int nx) {
  static_assert(TileShape<true, 64>::FLOATS == TileShape<false, 64>::FLOATS, "one LDS pair serves both layouts");
  __shared__ __attribute__((aligned(16))) float As[TileShape<true, 64>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<true, 64>::FLOATS];
  if ((int)blockIdx.x < nx) gemm_tile<true, true, EPI_X, 1, true>(px, blockIdx.x, nx, 0, As, Bs);
  else gemm_tile<false, false, ENDIA_EPI_NONE, 1, true>(pw, blockIdx.x - nx, gridDim.x - nx, 0, As, Bs);
}

// Fallback for operands the vector path cannot take (leading dimensions, sizes or pointers that are
// not multiples of 4 floats, e.g. the 1-wide first and last layers of the reference's sine-fit
// MLP, benchmarks/mlp_benchmarks/mlp_imp.mojo:35-37). 64 x 64 tile, 16 x 16 threads, 4 x 4 each.
template <int EPI>
__global__ __launch_bounds__(256) void sgemm_generic_kernel(GemmArgs p, int transA, int transB) {
  constexpr int T = 64, TK = 16;
  __shared__ float As[TK][T + 1];
  __shared__ float Bs[TK][T + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
  const int64_t bz = blockIdx.z;
  const float* __restrict__ A = p.A + bz * p.sA;
  const float* __restrict__ B = p.B + bz * p.sB;
  const int64_t cz = p.splits ? 0 : bz;  // every slice of a split reduction belongs to the one C
  float* __restrict__ C = p.C + cz * p.sC;
  const float* __restrict__ aux_in = p.aux_in ? p.aux_in + cz * p.sC : nullptr;
  float* __restrict__ aux_out = p.aux_out ? p.aux_out + cz * p.sC : nullptr;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += TK) {
    for (int e = tid; e < T * TK; e += 256) {
      int kk, mm;
      if (transA) { kk = e / T; mm = e % T; } else { mm = e / TK; kk = e % TK; }
      int m = m0 + mm, k = k0 + kk;
      float v = 0.f;
      if (m < p.M && k < p.K) v = transA ? A[(int64_t)k * p.lda + m] : A[(int64_t)m * p.lda + k];
      As[kk][mm] = v;
      int nn;
      if (transB) { nn = e / TK; kk = e % TK; } else { kk = e / T; nn = e % T; }
      int n = n0 + nn;
      k = k0 + kk;
      v = 0.f;
      if (n < p.N && k < p.K) v = transB ? B[(int64_t)n * p.ldb + k] : B[(int64_t)k * p.ldb + n];
      Bs[kk][nn] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty + 16 * i]; b[i] = Bs[kk][tx + 16 * i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int row = m0 + ty + 16 * i, col = n0 + tx + 16 * j;
      if (row < p.M && col < p.N) epilogue_store<EPI>(p, C, aux_in, aux_out, row, col, acc[i][j]);
    }
}

// A product with very few outputs and a long reduction (the weight gradient of a 1-wide layer over a
// batch: 32 outputs, K = 128) is bound by memory latency in any tiled kernel, whose K loop is a chain
// of dependent load -> LDS -> barrier rounds. Here one 128-thread group owns one output element: every
// thread issues all its loads at once, and the partial sums meet in a wave shuffle and an LDS add.
__global__ __launch_bounds__(128) void sgemm_skinny_kernel(GemmArgs p, int transA, int transB) {
  __shared__ float red[2];
  const int out = blockIdx.x;
  const bool colsum = out >= p.M * p.N;  // the groups past the last output element sum the columns of B
  const int m = colsum ? 0 : out / p.N, n = colsum ? out - p.M * p.N : out - m * p.N;
  const int64_t bz = blockIdx.y;
  const float* __restrict__ A = p.A + bz * p.sA;
  const float* __restrict__ B = p.B + bz * p.sB;
  float acc = 0.f;
  for (int k = threadIdx.x; k < p.K; k += 128) {
    const float a = colsum ? 1.f : (transA ? A[(int64_t)k * p.lda + m] : A[(int64_t)m * p.lda + k]);
    const float b = transB ? B[(int64_t)n * p.ldb + k] : B[(int64_t)k * p.ldb + n];
    acc = fmaf(a, b, acc);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float v = red[0] + red[1];
    if (colsum) {
      p.aux_out[n] = v;
    } else {
      float* c = p.C + bz * p.sC + (int64_t)m * p.ldc + n;
      float r = p.bias ? v + p.bias[n] : v;          // bias: the BIAS and BIAS_ACT epilogues
      if (p.bias && p.aux_out && !p.colsum) p.aux_out[bz * p.sC + (int64_t)m * p.ldc + n] = r;
      r = act_fwd(p.act, r);                         // identity unless BIAS_ACT
      *c = p.accumulate ? *c + r : r;
    }
  }
}

// A reduction of one to four terms (the 1-wide first layer of the reference's sine-fit MLP and the data gradient
// of its 1-wide last layer are outer products): one thread per output element, every epilogue.
template <int EPI>
__global__ __launch_bounds__(256) void sgemm_thin_k_kernel(GemmArgs p, int transA, int transB) {
  const int64_t bz = blockIdx.y;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)p.M * p.N) return;
  const int m = (int)(i / p.N), n = (int)(i - (int64_t)m * p.N);
  const float* __restrict__ A = p.A + bz * p.sA;
  const float* __restrict__ B = p.B + bz * p.sB;
  float acc = 0.f;
  for (int k = 0; k < p.K; ++k) {
    const float a = transA ? A[(int64_t)k * p.lda + m] : A[(int64_t)m * p.lda + k];
    const float b = transB ? B[(int64_t)n * p.ldb + k] : B[(int64_t)k * p.ldb + n];
    acc = fmaf(a, b, acc);
  }
  epilogue_store<EPI>(p, p.C + bz * p.sC, p.aux_in ? p.aux_in + bz * p.sC : nullptr, p.aux_out ? p.aux_out + bz * p.sC : nullptr, m, n, acc);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

namespace endia {
int32_t col_reduce(int64_t batch, int64_t R, int64_t C, const float* x, float* out, float scale);
}

namespace {
struct PoolBuf {  // scratch from the library's pool, handed back on scope exit (reuse is stream-ordered)
  void* p = nullptr;
  ~PoolBuf() { if (p) endia_hip_free(p); }
};

// per-launch event pairs for endia_hip_gemm_timing_*
struct GemmTiming {
  bool on = false;
  std::vector<hipEvent_t> start, stop;
  size_t used = 0;
  double flops = 0.0;
};
GemmTiming g_timing;
int g_forced_tile = 0;  // endia_hip_gemm_force_tile
}  // namespace

namespace endia {

// Shared by endia_hip_sgemm and the complex and convolution front ends.
int32_t sgemm_impl(int transA, int transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                   const float* B, int64_t ldb, float* C, int64_t ldc, int64_t batch, int64_t sA,
                   int64_t sB, int64_t sC, int epi_flags, int act_flags, const float* bias,
                   const float* aux_in, float* aux_out) {
  const int epi = epi_flags & 0xff;
  const int accumulate = (epi_flags & ENDIA_GEMM_ACCUMULATE) ? 1 : 0;
  const int colsum = (epi_flags & ENDIA_GEMM_COLSUM_B) ? 1 : 0;
  const int act = act_flags & 0xff;
  const int from_out = (act_flags & ENDIA_ACT_FROM_OUTPUT) ? 1 : 0;
  ENDIA_CHECK_ARG(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "sgemm: negative dimension (M=%lld N=%lld K=%lld batch=%lld)",
                  (long long)M, (long long)N, (long long)K, (long long)batch);
  ENDIA_CHECK_ARG(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && batch <= 65535,
                  "sgemm: dimension too large");
  ENDIA_CHECK_ARG(epi >= ENDIA_EPI_NONE && epi <= ENDIA_EPI_ACT_GRAD, "sgemm: unknown epilogue %d", epi);
  ENDIA_CHECK_ARG((epi_flags & ~(0xff | ENDIA_GEMM_ACCUMULATE | ENDIA_GEMM_COLSUM_B)) == 0, "sgemm: unknown epilogue flag bits 0x%x", epi_flags);
  ENDIA_CHECK_ARG(!colsum || (epi == ENDIA_EPI_NONE && !transB && batch == 1 && ldb == N && aux_out != nullptr),
                  "sgemm: COLSUM_B needs the plain epilogue, transB = 0, batch = 1, ldb = N and aux_out");
  ENDIA_CHECK_ARG(act == ENDIA_OP_RELU || act == ENDIA_OP_TANH || act == ENDIA_OP_SIN || act == ENDIA_OP_IDENTITY,
                  "sgemm: activation %d is not one of relu/tanh/sin/identity", act);
  ENDIA_CHECK_ARG(!(from_out && act == ENDIA_OP_SIN), "sgemm: sin gradient needs the pre-activation, not the output");
  if (N == 0 || batch == 0) return ENDIA_HIP_OK;
  if (M == 0) return colsum ? col_reduce(1, K, N, B, aux_out, 1.f) : ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(C != nullptr, "sgemm: C is null");
  ENDIA_CHECK_ARG(K == 0 || (A != nullptr && B != nullptr), "sgemm: A or B is null");
  ENDIA_CHECK_ARG(lda >= (transA ? M : K) && ldb >= (transB ? K : N) && ldc >= N,
                  "sgemm: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)", (long long)lda,
                  (long long)ldb, (long long)ldc);
  ENDIA_CHECK_ARG(sA >= 0 && sB >= 0 && sC >= 0, "sgemm: negative batch stride");
  ENDIA_CHECK_ARG(batch == 1 || sC >= (M - 1) * ldc + N, "sgemm: batch stride of C overlaps");
  if (epi == ENDIA_EPI_BIAS || epi == ENDIA_EPI_BIAS_ACT) ENDIA_CHECK_ARG(bias != nullptr, "sgemm: epilogue needs bias");
  if (epi == ENDIA_EPI_ACT_GRAD) ENDIA_CHECK_ARG(aux_in != nullptr, "sgemm: ACT_GRAD epilogue needs aux_in");

  GemmArgs p{};
  p.A = A; p.B = B; p.C = C; p.bias = bias; p.aux_in = aux_in;
  p.aux_out = (epi == ENDIA_EPI_BIAS_ACT) ? aux_out : nullptr;
  p.colsum = 0;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc; p.sA = sA; p.sB = sB; p.sC = sC;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.act = act; p.from_out = from_out; p.accumulate = accumulate;
  hipStream_t s = ctx().stream;

  // A classifier head: a handful of output columns, a long reduction. One pass over A at memory speed (gemm_narrow.hip).
  if (g_forced_tile == 0 && narrow_ok(transA, transB, M, N, K, batch, A, lda, B, ldb, colsum)) {
    const int32_t rc = launch_narrow(p, epi, transB, s);
    if (rc) return rc;
    ENDIA_LAUNCH_CHECK();
    return ENDIA_HIP_OK;
  }

  // The vector path loads 4 floats at a time along the contiguous index of each operand.
  const bool a_ok = aligned16(A) && lda % 4 == 0 && sA % 4 == 0 && (transA ? M % 4 == 0 : K % 4 == 0);
  const bool b_ok = aligned16(B) && ldb % 4 == 0 && sB % 4 == 0 && (transB ? K % 4 == 0 : N % 4 == 0);
  const bool big = M * N >= 64 * 64 && K >= 8 && lda < (1ll << 22) && ldb < (1ll << 22);  // 32-bit tile offsets
  const bool vec = a_ok && b_ok;  // otherwise the same tiles with 4-byte loads (gemm_unaligned.hip)
  if (big) {
    // 128 x 128 or 64 x 64 tiles. The large tile is the faster one per flop, but only when the chip holds
    // enough of them (two or more per CU) and the tile count divides evenly over the CUs: every CU works
    // on ceil(tiles / CUs) tiles while the average is tiles / CUs. Relative speeds measured on 2048..4096
    // products: large tile 1.00 at >= 3 per CU, 0.95 at 2, 0.80 below; small tile 0.92.
    const int64_t cus = ctx().cu_count;
    const int64_t t128 = ceil_div64(M, 128) * ceil_div64(N, 128) * batch;
    const int64_t t64 = ceil_div64(M, 64) * ceil_div64(N, 64) * batch;
    const bool fits128 = (double)(ceil_div64(M, 128) * 128) * (double)(ceil_div64(N, 128) * 128) <= 1.25 * (double)M * (double)N;
    auto balance = [&](int64_t tiles) { return ((double)tiles / (double)cus) / (double)ceil_div64(tiles, cus); };
    const double per_cu = (double)t128 / (double)cus;
    const double score128 = balance(t128) * (per_cu >= 3.0 ? 1.0 : (per_cu >= 2.0 ? 0.95 : 0.80));
    const double score64 = balance(t64) * 0.92;
    int F = (fits128 && score128 >= score64) ? 2 : 1;
    // One-wave-per-SIMD tiles (gemm_lone.h), one work-group per CU at a time: 256 x 256 or 256 x 128, the larger one
    // whose tiles fill every round over the CUs (4096^2 outputs are 256 tiles of 256 x 256, 2048 x 4096 outputs 256 of
    // 256 x 128). Smaller tiles written the same way (128 x 128, 128 x 64) were measured and bring nothing over the
    // shared-CU kernels below: their K tile is so short that the LDS traffic per MFMA stalls a lone wave's issue.
    // (The descriptors count bytes in 32 bits; the column sums of a small B ride in the launch of the other kernels.)
    const bool lone_ok = vec && !(colsum && K * N <= (1ll << 20)) && (transA ? K : M) * lda < (1ll << 29) && (transB ? N : K) * ldb < (1ll << 29);
    static const int lone_bm[2] = {256, 256}, lone_bn[2] = {256, 128};
    int lone = -1;  // index into the tables above
    if (lone_ok && g_forced_tile == 0 && K >= 256) {
      for (int i = 0; i < 2 && lone < 0; ++i) {
        const int64_t tm_ = ceil_div64(M, lone_bm[i]), tn_ = ceil_div64(N, lone_bn[i]), t = tm_ * tn_ * batch;
        const bool fits = (double)(tm_ * lone_bm[i]) * (double)(tn_ * lone_bn[i]) <= 1.1 * (double)M * (double)N;
        if (fits && t >= cus && balance(t) >= 0.9) lone = i;
      }
    } else if (lone_ok) {
      lone = g_forced_tile == 256 ? 0 : g_forced_tile == 256128 ? 1 : -1;
    }
    if (g_forced_tile == 64) F = 1;
    else if (g_forced_tile == 128) F = 2;
    const int BM_ = lone >= 0 ? lone_bm[lone] : 64 * F, BN_ = lone >= 0 ? lone_bn[lone] : 64 * F;
    if (lone >= 0) F = 0;  // none of the shared-CU tiles
    p.tiles_m = (int)ceil_div64(M, BM_);
    p.tiles_n = (int)ceil_div64(N, BN_);
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    ENDIA_CHECK_ARG(tiles < (1ll << 31), "sgemm: too many output tiles");
    // A product with fewer than about three tiles per CU is split along K so that more groups are in flight (a lone group
    // per CU spends most of its time waiting for loads). Up to 16 slices of at least 128: the slices of a tile are
    // added, in slice order, by whichever of its groups finishes last, inside the one launch, with any epilogue.
    // A long reduction with very few tiles (dW of a narrow layer over a large batch) wants more slices than one
    // group should add up: its partial products are added, also in slice order, by a second, chip-wide launch.
    int64_t splits = 1;
    bool meet_in_kernel = false;
    if (F == 1 && batch == 1 && K >= 256) {  // (the 128 x 128 tile is only chosen where there are enough tiles)
      int64_t want = (5 * cus + tiles / 2) / tiles;  // about five groups per CU in all (measured optimum 4-6)
      if (want > K / 128) want = K / 128;
      if (want > 16 && epi == ENDIA_EPI_NONE && !accumulate && ldc == N && K >= 2048) {
        splits = (4 * cus + tiles - 1) / tiles;
        if (splits > K / 256) splits = K / 256;
        if (splits > 1024) splits = 1024;
      } else if (want >= 2 && tiles <= kTicketCount) {
        splits = want < 16 ? want : 16;
        meet_in_kernel = true;
      }
    }
    PoolBuf part;
    float* const C_final = C;
    p.k_split = 0;
    // Small B: the launch below produces the column sums as well (a launch saved where launches are what a step
    // costs). For a large B the first tile row's groups would finish last and hold up the whole launch, and the
    // separate streaming reduction is cheaper.
    if (colsum && splits == 1 && K * N <= (1ll << 20)) {
      p.colsum = 1;
      p.aux_out = aux_out;
    }
    int64_t chunk = K;
    if (splits > 1) {
      chunk = ceil_div64(ceil_div64(K, splits), BK) * BK;
      splits = ceil_div64(K, chunk);
    }
    if (splits > 1) {
      const int64_t part_floats = meet_in_kernel ? splits * tiles * (64 * F) * (64 * F) : splits * M * N;
      int32_t rc = endia_hip_malloc(part_floats * 4, &part.p);
      if (rc) return rc;
      p.k_split = (int)chunk;
      p.sA = chunk * (transA ? lda : 1);
      p.sB = chunk * (transB ? 1 : ldb);
      if (meet_in_kernel) {
        p.splits = (int)splits;
        p.part = static_cast<float*>(part.p);
        p.tickets = ctx().tickets;
      } else {
        p.C = static_cast<float*>(part.p);
        p.ldc = N;
        p.sC = M * N;
      }
    }
    dim3 grid((unsigned)tiles, (unsigned)(splits > 1 ? splits : batch));
    const bool timed = g_timing.on && !ctx().capturing;
    if (timed) {
      if (g_timing.used == g_timing.start.size()) {
        hipEvent_t a, b;
        ENDIA_HIP_CALL(hipEventCreate(&a));
        ENDIA_HIP_CALL(hipEventCreate(&b));
        g_timing.start.push_back(a);
        g_timing.stop.push_back(b);
      }
      ENDIA_HIP_CALL(hipEventRecord(g_timing.start[g_timing.used], s));
    }
    if (lone >= 0) {
      int32_t rc = lone == 0 ? launch_lone_256x256(p, epi, transA, transB, grid, s) : launch_lone_256x128(p, epi, transA, transB, grid, s);
      if (rc) return rc;
    } else if (!vec) launch_mfma_unaligned(p, epi, 64 * F, a_ok, b_ok, transA, transB, grid, s);
    else if (F == 2) launch_mfma_epi<2>(p, epi, transA, transB, grid, s);
    else if (K <= 4 * BK && splits == 1) launch_mfma_epi<1, true>(p, epi, transA, transB, grid, s);
    else launch_mfma_epi<1>(p, epi, transA, transB, grid, s);
    if (timed) {
      ENDIA_HIP_CALL(hipEventRecord(g_timing.stop[g_timing.used], s));
      g_timing.used++;
      g_timing.flops += 2.0 * (double)M * (double)N * (double)K * (double)batch;
    }
    if (splits > 1 && !meet_in_kernel) {
      ENDIA_LAUNCH_CHECK();
      int32_t rc = col_reduce(1, splits, M * N, p.C, C_final, 1.f);  // partials added in slice order
      if (rc || !colsum) return rc;
    }
  } else if (K >= 1 && K <= 4 && M * N < (1ll << 31) * 256) {
    p.k_split = 0;
    dim3 grid((unsigned)ceil_div64(M * N, 256), (unsigned)batch);
    switch (epi) {
      case ENDIA_EPI_NONE: hipLaunchKernelGGL((sgemm_thin_k_kernel<ENDIA_EPI_NONE>), grid, dim3(256), 0, s, p, transA, transB); break;
      case ENDIA_EPI_BIAS: hipLaunchKernelGGL((sgemm_thin_k_kernel<ENDIA_EPI_BIAS>), grid, dim3(256), 0, s, p, transA, transB); break;
      case ENDIA_EPI_BIAS_ACT: hipLaunchKernelGGL((sgemm_thin_k_kernel<ENDIA_EPI_BIAS_ACT>), grid, dim3(256), 0, s, p, transA, transB); break;
      default: hipLaunchKernelGGL((sgemm_thin_k_kernel<ENDIA_EPI_ACT_GRAD>), grid, dim3(256), 0, s, p, transA, transB); break;
    }
  } else if (epi != ENDIA_EPI_ACT_GRAD && M * N <= 2048 && K >= (epi == ENDIA_EPI_NONE ? 64 : 16)) {
    p.k_split = 0;
    if (epi == ENDIA_EPI_NONE) p.bias = nullptr;
    if (epi != ENDIA_EPI_BIAS_ACT) p.act = ENDIA_OP_IDENTITY;
    if (colsum) {  // N more groups produce the column sums of B in the same launch
      p.colsum = 1;
      p.aux_out = aux_out;
    }
    hipLaunchKernelGGL(sgemm_skinny_kernel, dim3((unsigned)(M * N + (colsum ? N : 0)), (unsigned)batch), dim3(128), 0, s, p, transA, transB);
  } else {
    p.k_split = 0;
    p.tiles_m = (int)ceil_div64(M, 64);
    p.tiles_n = (int)ceil_div64(N, 64);
    ENDIA_CHECK_ARG(p.tiles_m <= 65535, "sgemm: M too large for the unaligned path");
    dim3 grid((unsigned)p.tiles_n, (unsigned)p.tiles_m, (unsigned)batch);
    switch (epi) {
      case ENDIA_EPI_NONE: hipLaunchKernelGGL((sgemm_generic_kernel<ENDIA_EPI_NONE>), grid, dim3(256), 0, s, p, transA, transB); break;
      case ENDIA_EPI_BIAS: hipLaunchKernelGGL((sgemm_generic_kernel<ENDIA_EPI_BIAS>), grid, dim3(256), 0, s, p, transA, transB); break;
      case ENDIA_EPI_BIAS_ACT: hipLaunchKernelGGL((sgemm_generic_kernel<ENDIA_EPI_BIAS_ACT>), grid, dim3(256), 0, s, p, transA, transB); break;
      default: hipLaunchKernelGGL((sgemm_generic_kernel<ENDIA_EPI_ACT_GRAD>), grid, dim3(256), 0, s, p, transA, transB); break;
    }
  }
  ENDIA_LAUNCH_CHECK();
  if (colsum && !p.colsum) return col_reduce(1, K, N, B, aux_out, 1.f);  // paths that do not fuse it
  return ENDIA_HIP_OK;
}

// dx = (g W^T) * act'(aux), dW = x^T g, db = column sums of g; see endia_hip_linear_bwd.
int32_t linear_bwd_impl(int64_t B, int64_t K, int64_t N, const float* x, const float* W, const float* g, int act_flags,
                        const float* aux, float* dx, float* dW, float* db) {
  ENDIA_CHECK_ARG(B >= 0 && K >= 0 && N >= 0, "linear_bwd: negative dimension");
  ENDIA_CHECK_ARG(g != nullptr || B * N == 0, "linear_bwd: g is null");
  ENDIA_CHECK_ARG(!dx || W, "linear_bwd: dx needs W");
  ENDIA_CHECK_ARG(!dW || x, "linear_bwd: dW needs x");
  const int epi_x = aux ? ENDIA_EPI_ACT_GRAD : ENDIA_EPI_NONE;
  const int act = act_flags & 0xff;
  // One launch for all three when every operand takes the vector path and both reductions fit four K tiles.
  const bool small = dx && dW && db && B > 0 && K > 0 && N > 0 && N <= 4 * BK && B <= 4 * BK && K % 4 == 0 && N % 4 == 0 &&
                     N >= 8 && B >= 8 && aligned16(x) && aligned16(W) && aligned16(g) &&
                     (act == ENDIA_OP_RELU || act == ENDIA_OP_TANH || act == ENDIA_OP_SIN || act == ENDIA_OP_IDENTITY) &&
                     !((act_flags & ENDIA_ACT_FROM_OUTPUT) && act == ENDIA_OP_SIN);
  if (small) {
    GemmArgs px{}, pw{};
    px.A = g; px.B = W; px.C = dx; px.aux_in = aux; px.lda = N; px.ldb = N; px.ldc = K;
    px.M = (int)B; px.N = (int)K; px.K = (int)N;
    px.tiles_m = (int)ceil_div64(B, 64); px.tiles_n = (int)ceil_div64(K, 64);
    px.act = act; px.from_out = (act_flags & ENDIA_ACT_FROM_OUTPUT) ? 1 : 0;
    pw.A = x; pw.B = g; pw.C = dW; pw.aux_out = db; pw.lda = K; pw.ldb = N; pw.ldc = N;
    pw.M = (int)K; pw.N = (int)N; pw.K = (int)B;
    pw.tiles_m = (int)ceil_div64(K, 64); pw.tiles_n = (int)ceil_div64(N, 64);
    pw.act = ENDIA_OP_IDENTITY; pw.colsum = 1;
    const int nx = px.tiles_m * px.tiles_n, nw = pw.tiles_m * pw.tiles_n;
    hipStream_t s = ctx().stream;
    if (aux) hipLaunchKernelGGL((linear_bwd_small_kernel<ENDIA_EPI_ACT_GRAD>), dim3((unsigned)(nx + nw)), dim3(NTHREADS), 0, s, px, pw, nx);
    else hipLaunchKernelGGL((linear_bwd_small_kernel<ENDIA_EPI_NONE>), dim3((unsigned)(nx + nw)), dim3(NTHREADS), 0, s, px, pw, nx);
    ENDIA_LAUNCH_CHECK();
    return ENDIA_HIP_OK;
  }
  // dx first: the weight gradient is then the last thing written, and an optimizer update issued right behind this call
  // (optim.Adam(fused_backward=True)) finds it in the last-level cache
  if (dx) {
    int32_t rc = sgemm_impl(0, 1, B, K, N, g, N, W, N, dx, K, 1, 0, 0, 0, epi_x, aux ? act_flags : ENDIA_OP_IDENTITY, nullptr, aux, nullptr);
    if (rc) return rc;
  }
  if (dW) {
    return sgemm_impl(1, 0, K, N, B, x, K, g, N, dW, N, 1, 0, 0, 0, ENDIA_EPI_NONE | (db ? ENDIA_GEMM_COLSUM_B : 0),
                      ENDIA_OP_IDENTITY, nullptr, nullptr, db);
  } else if (db && N > 0) {
    return col_reduce(1, B, N, g, db, 1.f);
  }
  return ENDIA_HIP_OK;
}

}  // namespace endia

extern "C" int32_t endia_hip_linear_bwd(int64_t B, int64_t K, int64_t N, const float* x, const float* W, const float* g,
                                        int32_t act, const float* aux, float* dx, float* dW, float* db) {
  ENDIA_REQUIRE_INIT();
  return endia::linear_bwd_impl(B, K, N, x, W, g, act, aux, dx, dW, db);
}

extern "C" int32_t endia_hip_sgemm(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K,
                                   const float* A, int64_t lda, const float* B, int64_t ldb, float* C,
                                   int64_t ldc, int64_t batch, int64_t strideA, int64_t strideB,
                                   int64_t strideC, int32_t epilogue, int32_t act, const float* bias,
                                   const float* aux_in, float* aux_out) {
  ENDIA_REQUIRE_INIT();
  return endia::sgemm_impl(transA, transB, M, N, K, A, lda, B, ldb, C, ldc, batch, strideA, strideB,
                           strideC, epilogue, act, bias, aux_in, aux_out);
}

namespace endia {

// endia_hip_sgemm_grouped: which members share a launch. A member that can run on the 256 x 128 one-wave-per-SIMD tile
// is a number of equal tiles, each a number of K tiles long; a launch puts one work-group on every CU, in block order,
// and a CU takes the next block when it is done (longest first: the caller's blocks are sorted that way). A set of
// members is worth one launch when that schedule keeps the CUs busy: its length, priced at what a K tile of this
// kernel takes, has to beat the members launched one by one at the rate the shared-CU tiles reach on such products.
namespace {
struct Member {
  int index;        // in the caller's array
  int64_t tiles;    // 256 x 128 tiles
  int64_t ktiles;   // K tiles of 32 per tile
  double alone_us;  // estimate for endia_hip_sgemm on it alone
};

// length, in K tiles, of the schedule of `set` (sorted by ktiles, descending) on `cus` CUs
int64_t schedule_length(const std::vector<Member>& set, int64_t cus) {
  std::priority_queue<int64_t, std::vector<int64_t>, std::greater<int64_t>> busy;  // when each CU is free again
  for (int64_t c = 0; c < cus; ++c) busy.push(0);
  int64_t longest = 0;
  for (const Member& m : set)
    for (int64_t t = 0; t < m.tiles; ++t) {
      const int64_t end = busy.top() + m.ktiles;
      busy.pop();
      busy.push(end);
      if (end > longest) longest = end;
    }
  return longest;
}
constexpr double kGroupFixedUs = 11.4, kGroupKtileUs = 3.57;  // measured: 2 x (2048 x 2048 x 1024) 125.7 us, 4 x (1024 x 2048 x 2048) 240.4 us
constexpr double kAloneTflops = 113.0;                        // what such a product reaches alone (64 x 64 tiles, K split in the launch)
}  // namespace

// The members of `pool` (indices into `can`, none of them used) that should share a launch with can[seed]: grown one
// member at a time by whichever keeps the CUs busiest, then cut back to the size that saves most over launching the
// members one by one. Empty when no shared launch beats that.
static std::vector<size_t> pick_group_uncached(const std::vector<Member>& can, size_t seed, const std::vector<bool>& used, int64_t cus);

// A training loop offers the same shapes in the same order step after step: the choice is looked up by them.
static std::vector<size_t> pick_group(const std::vector<Member>& can, size_t seed, const std::vector<bool>& used, int64_t cus) {
  static std::map<std::vector<int64_t>, std::vector<size_t>> known;
  std::vector<int64_t> key{(int64_t)seed, cus};
  for (size_t j = 0; j < can.size(); ++j) {
    key.push_back(used[j] ? -1 : can[j].tiles);
    key.push_back(can[j].ktiles);
  }
  auto it = known.find(key);
  if (it != known.end()) return it->second;
  if (known.size() > 4096) known.clear();
  return known[key] = pick_group_uncached(can, seed, used, cus);
}

static std::vector<size_t> pick_group_uncached(const std::vector<Member>& can, size_t seed, const std::vector<bool>& used, int64_t cus) {
  auto by_length = [](const Member& a, const Member& b) { return a.ktiles > b.ktiles; };
  std::vector<size_t> chosen{seed};
  std::vector<Member> set{can[seed]};
  auto work = [](const std::vector<Member>& v) {
    double w = 0.0;
    for (const Member& m : v) w += (double)m.tiles * (double)m.ktiles;
    return w;
  };
  auto gain = [&](const std::vector<Member>& v) {
    double sum = 0.0;
    for (const Member& m : v) sum += m.alone_us;
    return sum - (kGroupFixedUs + kGroupKtileUs * (double)schedule_length(v, cus));
  };
  double eff = work(set) / ((double)cus * (double)schedule_length(set, cus));
  double best_gain = 0.0;
  size_t best_size = 0;  // how many of `chosen` to keep
  while ((int)set.size() < kMaxGroup) {
    size_t pick = can.size();
    double pick_eff = eff;
    for (size_t j = 0; j < can.size(); ++j) {
      if (used[j] || std::find(chosen.begin(), chosen.end(), j) != chosen.end()) continue;
      std::vector<Member> trial = set;
      trial.push_back(can[j]);
      std::stable_sort(trial.begin(), trial.end(), by_length);
      const double e = work(trial) / ((double)cus * (double)schedule_length(trial, cus));
      if (e > pick_eff + 1e-9) { pick = j; pick_eff = e; }
    }
    if (pick == can.size()) break;
    chosen.push_back(pick);
    set.push_back(can[pick]);
    std::stable_sort(set.begin(), set.end(), by_length);
    eff = pick_eff;
    const double g = gain(set);
    if (g > best_gain + 1.0) { best_gain = g; best_size = chosen.size(); }
  }
  chosen.resize(best_size);
  return chosen;
}

int32_t sgemm_grouped_impl(int32_t count, const endia_hip_sgemm_desc* d, int32_t need, int32_t* launched) {
  ENDIA_CHECK_ARG(count >= 0 && count <= 64, "sgemm_grouped: count %d out of [0, 64]", count);
  ENDIA_CHECK_ARG(count == 0 || d != nullptr, "sgemm_grouped: null descriptors");
  ENDIA_CHECK_ARG(need >= -1 && need < count, "sgemm_grouped: need = %d with %d members", need, count);
  ENDIA_CHECK_ARG(need < 0 || launched != nullptr, "sgemm_grouped: need >= 0 reports what it launched: launched is null");
  const int64_t cus = ctx().cu_count;
  std::vector<Member> can;
  std::vector<int> alone;
  for (int i = 0; i < count; ++i) {
    if (launched) launched[i] = 0;
    const endia_hip_sgemm_desc& m = d[i];
    const int epi = m.epilogue & 0xff;
    ENDIA_CHECK_ARG((epi == ENDIA_EPI_NONE || epi == ENDIA_EPI_BIAS) && (m.epilogue & ~(0xff | ENDIA_GEMM_ACCUMULATE)) == 0,
                    "sgemm_grouped: member %d: epilogue 0x%x is not NONE or BIAS, optionally with ACCUMULATE", i, m.epilogue);
    ENDIA_CHECK_ARG(m.M >= 0 && m.N >= 0 && m.K >= 0 && m.M < (1ll << 31) && m.N < (1ll << 31) && m.K < (1ll << 31),
                    "sgemm_grouped: member %d: bad dimensions", i);
    const bool a_ok = aligned16(m.A) && m.lda % 4 == 0 && (m.transA ? m.M % 4 == 0 : m.K % 4 == 0);
    const bool b_ok = aligned16(m.B) && m.ldb % 4 == 0 && (m.transB ? m.K % 4 == 0 : m.N % 4 == 0);
    const int64_t tiles = ceil_div64(m.M, 256) * ceil_div64(m.N, 128);
    const bool fits = (double)(ceil_div64(m.M, 256) * 256) * (double)(ceil_div64(m.N, 128) * 128) <= 1.1 * (double)m.M * (double)m.N;
    const bool lone_ok = a_ok && b_ok && m.A && m.B && m.C && (epi != ENDIA_EPI_BIAS || m.bias) && m.K >= 256 && fits && tiles < cus &&
                         m.lda >= (m.transA ? m.M : m.K) && m.ldb >= (m.transB ? m.K : m.N) && m.ldc >= m.N &&
                         m.lda < (1ll << 22) && m.ldb < (1ll << 22) && (m.transA ? m.K : m.M) * m.lda < (1ll << 29) &&
                         (m.transB ? m.N : m.K) * m.ldb < (1ll << 29) && g_forced_tile == 0;
    if (lone_ok) can.push_back({i, tiles, ceil_div64(m.K, BK), 2.0 * (double)m.M * (double)m.N * (double)m.K / (kAloneTflops * 1e6)});
    else if (need < 0 || i == need) alone.push_back(i);
  }
  std::vector<std::vector<Member>> groups;
  std::vector<bool> used(can.size(), false);
  for (size_t i = 0; i < can.size(); ++i) {
    if (used[i] || (need >= 0 && can[i].index != need)) continue;
    std::vector<size_t> chosen = pick_group(can, i, used, cus);
    if (chosen.size() >= 2) {
      std::vector<Member> set;
      for (size_t c : chosen) {
        set.push_back(can[c]);
        used[c] = true;
      }
      std::stable_sort(set.begin(), set.end(), [](const Member& a, const Member& b) { return a.ktiles > b.ktiles; });
      groups.push_back(set);
    } else {
      used[i] = true;
      alone.push_back(can[i].index);
    }
  }
  hipStream_t s = ctx().stream;
  for (const std::vector<Member>& set : groups) {
    GroupArgs g{};
    g.count = (int)set.size();
    double flops = 0.0;
    for (size_t k = 0; k < set.size(); ++k) {
      const endia_hip_sgemm_desc& m = d[set[k].index];
      if (launched) launched[set[k].index] = 1;
      GemmArgs& p = g.p[k];
      p.A = m.A; p.B = m.B; p.C = m.C; p.bias = m.bias;
      p.lda = m.lda; p.ldb = m.ldb; p.ldc = m.ldc;
      p.M = (int)m.M; p.N = (int)m.N; p.K = (int)m.K;
      p.tiles_m = (int)ceil_div64(m.M, 256); p.tiles_n = (int)ceil_div64(m.N, 128);
      p.act = ENDIA_OP_IDENTITY;
      p.accumulate = (m.epilogue & ENDIA_GEMM_ACCUMULATE) ? 1 : 0;
      g.first[k + 1] = g.first[k] + (int)set[k].tiles;
      g.kind[k] = (m.transA ? 2 : 0) + (m.transB ? 0 : 1) + ((m.epilogue & 0xff) == ENDIA_EPI_BIAS ? 4 : 0);
      flops += 2.0 * (double)m.M * (double)m.N * (double)m.K;
    }
    const bool timed = g_timing.on && !ctx().capturing;
    if (timed) {
      if (g_timing.used == g_timing.start.size()) {
        hipEvent_t a, b;
        ENDIA_HIP_CALL(hipEventCreate(&a));
        ENDIA_HIP_CALL(hipEventCreate(&b));
        g_timing.start.push_back(a);
        g_timing.stop.push_back(b);
      }
      ENDIA_HIP_CALL(hipEventRecord(g_timing.start[g_timing.used], s));
    }
    int32_t rc = launch_lone_grouped_256x128(g, s);
    if (rc) return rc;
    if (timed) {
      ENDIA_HIP_CALL(hipEventRecord(g_timing.stop[g_timing.used], s));
      g_timing.used++;
      g_timing.flops += flops;
    }
    ENDIA_LAUNCH_CHECK();
  }
  std::sort(alone.begin(), alone.end());
  for (int i : alone) {
    const endia_hip_sgemm_desc& m = d[i];
    if (launched) launched[i] = 1;
    int32_t rc = sgemm_impl(m.transA, m.transB, m.M, m.N, m.K, m.A, m.lda, m.B, m.ldb, m.C, m.ldc, 1, 0, 0, 0, m.epilogue,
                            ENDIA_OP_IDENTITY, m.bias, nullptr, nullptr);
    if (rc) return rc;
  }
  return ENDIA_HIP_OK;
}

}  // namespace endia

extern "C" int32_t endia_hip_sgemm_grouped(int32_t count, const endia_hip_sgemm_desc* members, int32_t need, int32_t* launched) {
  ENDIA_REQUIRE_INIT();
  return endia::sgemm_grouped_impl(count, members, need, launched);
}

extern "C" int32_t endia_hip_gemm_force_tile(int32_t tile) {
  ENDIA_CHECK_ARG(tile == 0 || tile == 64 || tile == 128 || tile == 256 || tile == 256128,
                  "endia_hip_gemm_force_tile: tile %d is not one of 0, 64, 128, 256, 256128", tile);
  g_forced_tile = tile;
  return ENDIA_HIP_OK;
}

extern "C" int32_t endia_hip_gemm_timing_begin(void) {
  ENDIA_REQUIRE_INIT();
  g_timing.on = true;
  g_timing.used = 0;
  g_timing.flops = 0.0;
  return ENDIA_HIP_OK;
}

extern "C" int32_t endia_hip_gemm_timing_end(int64_t* launches, double* total_ms, double* total_flops) {
  ENDIA_REQUIRE_INIT();
  g_timing.on = false;
  ENDIA_HIP_CALL(hipStreamSynchronize(endia::ctx().stream));
  double ms = 0.0;
  for (size_t i = 0; i < g_timing.used; ++i) {
    float t = 0.f;
    ENDIA_HIP_CALL(hipEventElapsedTime(&t, g_timing.start[i], g_timing.stop[i]));
    ms += t;
  }
  if (launches) *launches = (int64_t)g_timing.used;
  if (total_ms) *total_ms = ms;
  if (total_flops) *total_flops = g_timing.flops;
  return ENDIA_HIP_OK;
}

