// C[M, N] = A[M, K] . B with at most 16 output columns: the forward product of a classifier head (matmul_fwd,
// endia/functional/binary_ops/matmul_op.mojo:93-199, with a [K, 10] weight). The product is a stream over A: every byte of A
// is used once, against a B that fits in L2, so the kernel is built to keep HBM busy rather than the matrix cores.
//
// A work-group owns 16 rows of A and all of K; its 16 waves take turns along K, 64 k at a time (wave w multiplies
// k in [64 w + 1024 t, 64 w + 1024 t + 64) for t = 0, 1, ...), on v_mfma_f32_16x16x4_f32 (rows = the 16 rows of A, columns =
// output columns padded to 16): the four lanes that share a row fetch 64 consecutive bytes of it per load, and the loads of
// four turns (16 per lane) go out before anything is multiplied, B's two turns ahead of their use. Which k lands in which
// reduction slot of which step is a fixed permutation applied to A and B alike (a sum over k does not care). B stored
// [N, K] (the transposed form) is fetched like A. B stored [K, N] goes through a per-wave LDS staging area, one row per k
// with a pitch that lets a fragment read touch every bank once; without padding between its rows (ldb = N) the 64 rows of a
// piece are fetched as one run of 16-byte pieces, otherwise a lane fetches a row. Every load takes its bounds from a buffer
// descriptor, so that the loads are straight-line code, complete in the order they were issued, and the products of a turn
// wait for that turn's loads only. The 16 partial tiles of a work-group meet in LDS and are added in wave order, so results
// repeat bit for bit; then the epilogue. (Spans of K in separate, smaller work-groups meeting at a ticket were measured and
// are slower: 22.1 against 20.4 us at 4096 x 10 x 4096 with B stored [N, K], before the loads were made straight-line.)
#include "common.h"
#include "gemm_args.h"
#include "mfma_tile.h"

namespace endia_gemm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int NW = 16;          // waves per work-group
constexpr int SUB = 64;         // k per turn of a wave
constexpr int TURNS = 4;        // turns whose loads are in flight together
constexpr int BPITCH = 20;      // words per row of a staged B piece: 4 rows apart is a quarter of the banks apart, so a fragment read meets every bank once
constexpr int BAREA = 65 * BPITCH;  // a staged piece: 64 rows of k, and one that takes what lies past the piece

// B_FORM: 0 = B stored [K, N] with any leading dimension, 1 = stored [N, K], 2 = stored [K, N] without padding (ldb = N) and
// 16-byte aligned, so that the 64 rows of a piece are one run of memory.
template <int B_FORM, int EPI>
__global__ __launch_bounds__(NW * 64) void sgemm_narrow_kernel(const GemmArgs p) {
  constexpr bool B_KMAJOR = B_FORM == 1;
  extern __shared__ float stage[];  // B pieces, one area of BAREA words per wave (form [K, N] only); afterwards the waves' partial tiles
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, g = lane >> 4;
  const int row = blockIdx.x * 16 + i;
  const bool row_ok = row < p.M;
  // Every load goes through a buffer descriptor and takes its bounds from it (an offset past the end reads as zero), so the
  // loads are straight-line code and the products of a turn wait for that turn's loads only: behind a branch per load the
  // compiler waits for ALL outstanding loads before the first product, and nothing of the arithmetic overlaps the stream.
  const int rows_here = p.M - (int)blockIdx.x * 16 < 16 ? p.M - (int)blockIdx.x * 16 : 16;
  const __amdgpu_buffer_rsrc_t ra = mfma::make_rsrc(p.A + (int64_t)blockIdx.x * 16 * p.lda, ((int64_t)(rows_here - 1) * p.lda + p.K) * 4);
  const __amdgpu_buffer_rsrc_t rb =
      mfma::make_rsrc(p.B, B_KMAJOR ? ((int64_t)(p.N - 1) * p.ldb + p.K) * 4 : ((int64_t)(p.K - 1) * p.ldb + p.N) * 4);
  // (a condition becomes the top bit of the offset by arithmetic: written as a select it is compiled into a branch around the load)
  auto past = [](int have, int want) { return (uint32_t)(have - 1 - want) & mfma::OOB_OFFSET; };  // want >= have: out of bounds
  const uint32_t aoff = (((uint32_t)(row_ok ? i : 0) * (uint32_t)p.lda + 4u * g) * 4u) | past(p.M, row);  // bytes
  const int k_first = wave * SUB, k_end = p.K;
  float* mine = stage + wave * BAREA;
  v4f acc = {0.f, 0.f, 0.f, 0.f};

  auto load4 = [&](__amdgpu_buffer_rsrc_t rs, uint32_t off) {
    const float4 t = mfma::buffer_load_f4(rs, off);
    return v4f{t.x, t.y, t.z, t.w};
  };
  // this lane's 16 values of A for the 64 k from k0: load j covers k0 + 16 j + 4 g .. + 3 (K is a multiple of 4)
  auto load_a = [&](int k0, v4f (&a)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + 16 * j + 4 * g;
      a[j] = load4(ra, (aoff + (uint32_t)(k0 + 16 * j) * 4u) | past(k_end, k));
    }
  };
  // B stored [N, K]: column i of the output is row i of B, fetched the same way
  auto load_bt = [&](int k0, v4f (&b)[4]) {
    const uint32_t boff = (((uint32_t)(i < p.N ? i : 0) * (uint32_t)p.ldb + 4u * g) * 4u) | past(p.N, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + 16 * j + 4 * g;
      b[j] = load4(rb, (boff + (uint32_t)(k0 + 16 * j) * 4u) | past(k_end, k));
    }
  };
  // B stored [K, N]: the 64 x N piece from k0, lane l holding row k0 + l, into registers ...
  auto load_b = [&](int k0, float (&b)[16]) {
    const int k = k0 + lane;
    const uint32_t brow = ((uint32_t)(k < k_end ? k : 0) * (uint32_t)p.ldb * 4u) | past(k_end, k);
#pragma unroll
    for (int n = 0; n < 16; ++n) b[n] = mfma::buffer_load_f1(rb, (brow + 4u * n) | past(p.N, n));
  };
  // The same piece without padding between the rows is 64 N consecutive floats: every lane fetches the 16-byte pieces
  // lane, lane + 64, ... of it (whole lines per request, where a lane per row touches a line per lane and element) ...
  auto load_b_flat = [&](int k0, float (&b)[16]) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int f = 4 * (lane + 64 * m);
      const float4 t = mfma::buffer_load_f4(rb, ((uint32_t)(k0 * p.N + f) * 4u) | past(64 * p.N, f));
      b[4 * m] = t.x; b[4 * m + 1] = t.y; b[4 * m + 2] = t.z; b[4 * m + 3] = t.w;
    }
  };
  // ... and element f of the piece is row f / N, column f % N (a multiplication: f < 1024, N <= 16). Elements past the piece
  // go to a word of the area's padding.
  const uint32_t inv_n = (65536u + (uint32_t)p.N - 1u) / (uint32_t)p.N;
  auto stage_b_flat = [&](const float (&b)[16]) {
    int l = lane;
    asm volatile("" : "+v"(l));  // (the sixteen positions are worked out again per turn: kept across turns they cost sixteen registers, and spills)
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int f = 4 * (l + 64 * m) + e;
        const int kr = (int)(((uint32_t)f * inv_n) >> 16), n = f - kr * p.N;
        mine[f < 64 * p.N ? kr * BPITCH + n : 64 * BPITCH + (l & 15)] = b[4 * m + e];
      }
  };
  // ... and from there into this wave's staging area, row k of the piece at k * BPITCH
  auto stage_b = [&](const float (&b)[16]) {
    float* dst = mine + lane * BPITCH;
#pragma unroll
    for (int n = 0; n < 16; n += 4) *reinterpret_cast<v4f*>(dst + n) = v4f{b[n], b[n + 1], b[n + 2], b[n + 3]};
  };

  for (int k0 = k_first; k0 < k_end; k0 += TURNS * NW * SUB) {
    v4f a[TURNS][4];
    if constexpr (B_KMAJOR) {
      v4f b[2][4];
      // (loads complete in the order they are issued: B's first two turns go out in front of the A loads they meet, so that
      // the products of a turn can start when that turn's piece of A is there and not when all of A is)
      load_a(k0, a[0]);
      load_bt(k0, b[0]);
      load_a(k0 + NW * SUB, a[1]);
      load_bt(k0 + NW * SUB, b[1]);
#pragma unroll
      for (int t = 2; t < TURNS; ++t) load_a(k0 + t * NW * SUB, a[t]);
      __builtin_amdgcn_sched_barrier(0);  // (left alone, the scheduler sinks each load to its use to save registers)
#pragma unroll
      for (int t = 0; t < TURNS; ++t) {
#pragma unroll
        for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][s >> 2][s & 3], b[t & 1][s >> 2][s & 3], acc, 0, 0, 0);
        if (t + 2 < TURNS) load_bt(k0 + (t + 2) * NW * SUB, b[t & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      float b[2][16];
      auto fetch_b = [&](int kk, float (&bb)[16]) {
        if constexpr (B_FORM == 2) load_b_flat(kk, bb);
        else load_b(kk, bb);
      };
      load_a(k0, a[0]);
      fetch_b(k0, b[0]);
      load_a(k0 + NW * SUB, a[1]);
      fetch_b(k0 + NW * SUB, b[1]);
#pragma unroll
      for (int t = 2; t < TURNS; ++t) load_a(k0 + t * NW * SUB, a[t]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TURNS; ++t) {
        // the wave's own area: no barrier, a wave's LDS accesses stay in order
        if constexpr (B_FORM == 2) stage_b_flat(b[t & 1]);
        else stage_b(b[t & 1]);
        if (t + 2 < TURNS) fetch_b(k0 + (t + 2) * NW * SUB, b[t & 1]);
#pragma unroll
        for (int s = 0; s < 16; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][s >> 2][s & 3], mine[(16 * (s >> 2) + 4 * g + (s & 3)) * BPITCH + i], acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // the waves' partial tiles meet: lane holds rows 4 g + r, column i
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) stage[wave * 256 + (4 * g + r) * 16 + i] = acc[r];
  __syncthreads();
  if (threadIdx.x < 256) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += stage[w * 256 + threadIdx.x];
    const int r = blockIdx.x * 16 + (threadIdx.x >> 4), c = threadIdx.x & 15;
    if (r < p.M && c < p.N) epilogue_store<EPI>(p, p.C, p.aux_in, p.aux_out, r, c, v);
  }
}

}  // namespace

// Whether the narrow-output kernel takes this product. A is read 16 bytes at a time along K.
bool narrow_ok(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch, const float* A, int64_t lda, const float* B,
               int64_t ldb, int colsum) {
  // (the loads address 16 rows of A, and all of B, with 32-bit byte offsets)
  if (transA || batch != 1 || colsum || N > 16 || M < 256 || K < 512 || K % 4 || lda % 4 || lda >= (1ll << 24) || (reinterpret_cast<uintptr_t>(A) & 15)) return false;
  if (transB && (ldb % 4 || ldb >= (1ll << 24) || (reinterpret_cast<uintptr_t>(B) & 15))) return false;
  if (!transB && K * ldb >= (1ll << 29)) return false;
  return M < (1ll << 31) - 16 && K < (1ll << 24);
}

int32_t launch_narrow(const GemmArgs& p, int epi, int transB, hipStream_t s) {
  const dim3 grid((unsigned)((p.M + 15) / 16)), block(NW * 64);
  const size_t lds = (transB ? NW * 256 : NW * BAREA) * sizeof(float);  // 16 KB / 81 KB
#define ENDIA_NARROW(FORM_, EPI_)                                                                                            \
  do {                                                                                                                       \
    static bool big_lds = false;                                                                                             \
    if (!big_lds && lds > 64 * 1024) {                                                                                       \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_narrow_kernel<FORM_, EPI_>),                               \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)                           \
        return endia::fail(ENDIA_HIP_ERR_RUNTIME, "sgemm: cannot reserve %d bytes of LDS", (int)lds);                          \
      big_lds = true;                                                                                                        \
    }                                                                                                                        \
    hipLaunchKernelGGL((sgemm_narrow_kernel<FORM_, EPI_>), grid, block, lds, s, p);                                          \
  } while (0)
#define ENDIA_NARROW_EPI(FORM_)                                                        \
  switch (epi) {                                                                       \
    case ENDIA_EPI_NONE: ENDIA_NARROW(FORM_, ENDIA_EPI_NONE); break;                   \
    case ENDIA_EPI_BIAS: ENDIA_NARROW(FORM_, ENDIA_EPI_BIAS); break;                   \
    case ENDIA_EPI_BIAS_ACT: ENDIA_NARROW(FORM_, ENDIA_EPI_BIAS_ACT); break;           \
    default: ENDIA_NARROW(FORM_, ENDIA_EPI_ACT_GRAD); break;                           \
  }
  const bool flat = !transB && p.ldb == p.N && (reinterpret_cast<uintptr_t>(p.B) & 15) == 0;
  if (transB) { ENDIA_NARROW_EPI(1) } else if (flat) { ENDIA_NARROW_EPI(2) } else { ENDIA_NARROW_EPI(0) }
#undef ENDIA_NARROW_EPI
#undef ENDIA_NARROW
  return ENDIA_HIP_OK;
}

}  // namespace endia_gemm
