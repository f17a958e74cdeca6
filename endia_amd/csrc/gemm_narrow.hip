// C[M, N] = A[M, K] . B with at most 16 output columns: the forward product of a classifier head (matmul_fwd,
// endia/functional/binary_ops/matmul_op.mojo:93-199, with a [K, 10] weight). The product is a stream over A: every byte of A
// is used once, against a B that fits in L2, so the kernel is built to keep HBM busy rather than the matrix cores.
//
// A work-group owns 16 rows of A and all of K; its 16 waves take turns along K, 64 k at a time (wave w multiplies
// k in [64 w + 1024 t, 64 w + 1024 t + 64) for t = 0, 1, ...), on v_mfma_f32_16x16x4_f32 (rows = the 16 rows of A, columns =
// output columns padded to 16): the four lanes that share a row fetch 64 consecutive bytes of it per load, and the loads of
// four turns (16 per lane) go out before anything is multiplied, B's two turns ahead of their use. Which k lands in which
// reduction slot of which step is a fixed permutation applied to A and B alike (a sum over k does not care). B, stored
// [K, N], goes through a per-wave LDS staging area laid out by (slot, step) so that a fragment read touches every bank once;
// stored [N, K] (the transposed form) it is fetched like A. The 16 partial tiles of a work-group meet in LDS and are added
// in wave order, so results repeat bit for bit; then the epilogue. (Spans of K in separate, smaller work-groups meeting at a
// ticket were measured and are slower: 22.1 against 20.4 us at 4096 x 10 x 4096 with B stored [N, K].)
#include "common.h"
#include "gemm_args.h"

namespace endia_gemm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int NW = 16;          // waves per work-group
constexpr int SUB = 64;         // k per turn of a wave
constexpr int TURNS = 4;        // turns whose loads are in flight together
constexpr int BSLOT = 16 * 16 + 16;  // words per reduction slot of a staged B piece: [step][column] + a quarter of the banks

template <bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(NW * 64) void sgemm_narrow_kernel(const GemmArgs p) {
  extern __shared__ float stage[];  // B pieces, one area of 4 * BSLOT words per wave (form [K, N] only); afterwards the waves' partial tiles
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, g = lane >> 4;
  const int row = blockIdx.x * 16 + i;
  const bool row_ok = row < p.M;
  const float* abase = p.A + (int64_t)blockIdx.x * 16 * p.lda;  // uniform; the lane's part is a 32-bit offset
  const unsigned aoff = (unsigned)(row_ok ? i : 0) * (unsigned)p.lda + 4u * g;
  const int k_first = wave * SUB, k_end = p.K;
  float* mine = stage + wave * 4 * BSLOT;
  v4f acc = {0.f, 0.f, 0.f, 0.f};

  // this lane's 16 values of A for the 64 k from k0: load j covers k0 + 16 j + 4 g .. + 3 (K is a multiple of 4)
  auto load_a = [&](int k0, v4f (&a)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + 16 * j + 4 * g;
      a[j] = (row_ok && k < k_end) ? *reinterpret_cast<const v4f*>(abase + (k0 + 16 * j) + aoff) : v4f{0.f, 0.f, 0.f, 0.f};
    }
  };
  // B stored [N, K]: column i of the output is row i of B, fetched the same way
  auto load_bt = [&](int k0, v4f (&b)[4]) {
    const unsigned boff = (unsigned)(i < p.N ? i : 0) * (unsigned)p.ldb + 4u * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + 16 * j + 4 * g;
      b[j] = (i < p.N && k < k_end) ? *reinterpret_cast<const v4f*>(p.B + (k0 + 16 * j) + boff) : v4f{0.f, 0.f, 0.f, 0.f};
    }
  };
  // B stored [K, N]: the 64 x N piece from k0, lane l holding row k0 + l, into registers ...
  auto load_b = [&](int k0, float (&b)[16]) {
    const int k = k0 + lane;
    const float* brow = p.B + (int64_t)(k < k_end ? k : 0) * p.ldb;
#pragma unroll
    for (int n = 0; n < 16; ++n) b[n] = (n < p.N && k < k_end) ? brow[n] : 0.f;
  };
  // ... and from there into this wave's staging area: k = 16 j + 4 slot + e sits at [slot][4 j + e][column]
  auto stage_b = [&](const float (&b)[16]) {
    const int j = lane >> 4, slot = (lane >> 2) & 3, e = lane & 3;
    float* dst = mine + slot * BSLOT + (4 * j + e) * 16;
#pragma unroll
    for (int n = 0; n < 16; n += 4) *reinterpret_cast<v4f*>(dst + n) = v4f{b[n], b[n + 1], b[n + 2], b[n + 3]};
  };

  for (int k0 = k_first; k0 < k_end; k0 += TURNS * NW * SUB) {
    v4f a[TURNS][4];
    if constexpr (B_KMAJOR) {
      v4f b[2][4];
#pragma unroll
      for (int t = 0; t < TURNS; ++t) load_a(k0 + t * NW * SUB, a[t]);
      load_bt(k0, b[0]);
      load_bt(k0 + NW * SUB, b[1]);
#pragma unroll
      for (int t = 0; t < TURNS; ++t) {
#pragma unroll
        for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][s >> 2][s & 3], b[t & 1][s >> 2][s & 3], acc, 0, 0, 0);
        if (t + 2 < TURNS) load_bt(k0 + (t + 2) * NW * SUB, b[t & 1]);
      }
    } else {
      float b[2][16];
#pragma unroll
      for (int t = 0; t < TURNS; ++t) load_a(k0 + t * NW * SUB, a[t]);
      load_b(k0, b[0]);
      load_b(k0 + NW * SUB, b[1]);
#pragma unroll
      for (int t = 0; t < TURNS; ++t) {
        stage_b(b[t & 1]);  // the wave's own area: no barrier, a wave's LDS accesses stay in order
        if (t + 2 < TURNS) load_b(k0 + (t + 2) * NW * SUB, b[t & 1]);
#pragma unroll
        for (int s = 0; s < 16; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][s >> 2][s & 3], mine[g * BSLOT + s * 16 + i], acc, 0, 0, 0);
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
  if (transA || batch != 1 || colsum || N > 16 || M < 256 || K < 512 || K % 4 || lda % 4 || lda >= (1ll << 27) || (reinterpret_cast<uintptr_t>(A) & 15)) return false;
  if (transB && (ldb % 4 || ldb >= (1ll << 27) || (reinterpret_cast<uintptr_t>(B) & 15))) return false;
  return M < (1ll << 31) - 16 && K < (1ll << 30);
}

int32_t launch_narrow(const GemmArgs& p, int epi, int transB, hipStream_t s) {
  const dim3 grid((unsigned)((p.M + 15) / 16)), block(NW * 64);
  const size_t lds = (transB ? NW * 256 : NW * 4 * BSLOT) * sizeof(float);  // 16 KB / 68 KB
#define ENDIA_NARROW(BK_, EPI_)                                                                                              \
  do {                                                                                                                       \
    static bool big_lds = false;                                                                                             \
    if (!big_lds && lds > 64 * 1024) {                                                                                       \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_narrow_kernel<BK_, EPI_>),                                 \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)                           \
        return endia::fail(ENDIA_HIP_ERR_RUNTIME, "sgemm: cannot reserve %d bytes of LDS", (int)lds);                          \
      big_lds = true;                                                                                                        \
    }                                                                                                                        \
    hipLaunchKernelGGL((sgemm_narrow_kernel<BK_, EPI_>), grid, block, lds, s, p);                                            \
  } while (0)
  if (transB) {
    switch (epi) {
      case ENDIA_EPI_NONE: ENDIA_NARROW(true, ENDIA_EPI_NONE); break;
      case ENDIA_EPI_BIAS: ENDIA_NARROW(true, ENDIA_EPI_BIAS); break;
      case ENDIA_EPI_BIAS_ACT: ENDIA_NARROW(true, ENDIA_EPI_BIAS_ACT); break;
      default: ENDIA_NARROW(true, ENDIA_EPI_ACT_GRAD); break;
    }
  } else {
    switch (epi) {
      case ENDIA_EPI_NONE: ENDIA_NARROW(false, ENDIA_EPI_NONE); break;
      case ENDIA_EPI_BIAS: ENDIA_NARROW(false, ENDIA_EPI_BIAS); break;
      case ENDIA_EPI_BIAS_ACT: ENDIA_NARROW(false, ENDIA_EPI_BIAS_ACT); break;
      default: ENDIA_NARROW(false, ENDIA_EPI_ACT_GRAD); break;
    }
  }
#undef ENDIA_NARROW
  return ENDIA_HIP_OK;
}

}  // namespace endia_gemm
