// The shared-CU tiles of the fp32 GEMM (64 x 64 and 128 x 128 per work-group, four work-groups per CU): the tile body
// and its kernels, included by the translation units that instantiate them (gemm.hip: operands that can be read 16
// bytes at a time; gemm_unaligned.hip: any base address, leading dimension and extent, read 4 bytes at a time).
#pragma once
#include "common.h"
#include "gemm_args.h"
#include "mfma_tile.h"
#include "ticket.h"

namespace endia_gemm {

using namespace mfma;

// F = MFMA blocks per wave in each direction: F = 2 gives the 128 x 128 tile, F = 1 the 64 x 64 tile
// used when the larger one would leave CUs without work.
// SHORTK (64 x 64 tile only): the reduction is at most four K tiles long, which is the case of every product
// of a small model (the reference's sine-fit MLP has K <= 128 throughout). Such launches are a handful of
// work-groups whose time is a chain of global-load latencies, one per K tile; here the loads of all four tiles
// are issued before anything else, so that latency is paid once.
// One work-group's tile of one product: group `block` of `nblocks`, batch entry (or K slice) bz, LDS handed in.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int F, bool SHORTK, bool A_VEC = true, bool B_VEC = true>
__device__ __forceinline__ void gemm_tile(const GemmArgs& p, int block, int nblocks, int64_t bz, float* __restrict__ As,
                                          float* __restrict__ Bs) {
  static_assert(!SHORTK || F == 1, "the short-reduction variant exists for the 64 x 64 tile");
  constexpr int BM = 64 * F, BN = 64 * F;
  using LA = MatrixTileLoader<A_KMAJOR, BM, NTHREADS, A_VEC>;
  using LB = MatrixTileLoader<B_KMAJOR, BN, NTHREADS, B_VEC>;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, h = lane >> 5;

  int tm, tn;
  tile_of_block(block, nblocks, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int64_t cz = p.splits ? 0 : bz;  // every slice of a split reduction belongs to the one C
  float* __restrict__ C = p.C + cz * p.sC;
  const float* __restrict__ aux_in = p.aux_in ? p.aux_in + cz * p.sC : nullptr;
  float* __restrict__ aux_out = p.aux_out ? p.aux_out + cz * p.sC : nullptr;

  // split-K: this group reduces k in [bz * k_split, bz * k_split + K) and writes slice bz of the partials
  const int K = p.k_split ? (p.K - (int)bz * p.k_split < p.k_split ? p.K - (int)bz * p.k_split : p.k_split) : p.K;
  LA la;
  LB lb;
  la.init(p.A + bz * p.sA, p.lda, m0, p.M, K, tid);
  lb.init(p.B + bz * p.sB, p.ldb, n0, p.N, K, tid);

  floatx16 acc[F][F];
  zero_acc<F, F>(acc);

  // Column sums of B (the bias gradient when C = A^T dY): the first tile row's groups add up their B tiles as
  // they pass through LDS, one column per thread, k ascending.
  float colsum = 0.f;
  const bool do_colsum = !B_KMAJOR && EPI == ENDIA_EPI_NONE && p.colsum && tm == 0 && tid < BN;
  auto add_colsum = [&]() {
    if (do_colsum) {
#pragma unroll 8
      for (int k = 0; k < BK; ++k) colsum += Bs[k * TileShape<B_KMAJOR, BN>::LD + tid];
    }
  };

  // The small tile has registers to spare: what the epilogue reads (a bias element, 16 elements of the activation
  // operand) is requested here, behind the tile loads, instead of after the last MFMA, where it would be one more
  // memory round trip on the critical path of a launch that is a few such round trips long.
  constexpr bool PRE = F == 1 && EPI != ENDIA_EPI_NONE;
  float bias_pre = 0.f, aux_pre[PRE ? 16 : 1];
  auto prefetch_epilogue = [&]() {
    if constexpr (PRE) {
      const int col = n0 + wn * 32 + l32;
      if (EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) bias_pre = col < p.N ? p.bias[col] : 0.f;
      if (EPI == ENDIA_EPI_ACT_GRAD) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = m0 + wm * 32 + acc_row(v, h);
          aux_pre[v] = (row < p.M && col < p.N) ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
        }
      }
    }
  };

  if constexpr (SHORTK) {
    constexpr int DEPTH = 4;
    float4 ra[DEPTH][LA::PASSES], rb[DEPTH][LB::PASSES];
#pragma unroll
    for (int t = 0; t < DEPTH; ++t) {  // tiles past the end of K load as zeros without touching memory
      la.load_into(ra[t], K - t * BK);
      lb.load_into(rb[t], K - t * BK);
      la.advance();
      lb.advance();
    }
    prefetch_epilogue();
#pragma unroll
    for (int t = 0; t < DEPTH; ++t) {
      if (t * BK >= K) break;
      if (t) __syncthreads();
      la.store_from(As, ra[t]);
      lb.store_from(Bs, rb[t]);
      __syncthreads();
      add_colsum();
      compute_ktile<A_KMAJOR, B_KMAJOR, F, F, BM, BN>(As, Bs, wm * 32 * F + l32, wn * 32 * F + l32, h, acc);
    }
  } else {
  la.load(K);
  lb.load(K);
  prefetch_epilogue();
  la.store(As);
  lb.store(Bs);
  __syncthreads();

  for (int k0 = 0; k0 < K; k0 += BK) {
    const bool more = k0 + BK < K;
    if (more) {  // next tile: global -> registers, in flight during this tile's MFMAs
      la.advance();
      lb.advance();
      la.load(K - k0 - BK);
      lb.load(K - k0 - BK);
    }
    add_colsum();
    compute_ktile<A_KMAJOR, B_KMAJOR, F, F, BM, BN>(As, Bs, wm * 32 * F + l32, wn * 32 * F + l32, h, acc);
    if (more) {
      __syncthreads();
      la.store(As);
      lb.store(Bs);
      __syncthreads();
    }
  }
  }

  if (do_colsum && n0 + tid < p.N) p.aux_out[n0 + tid] = colsum;

  // K split over gridDim.y groups per tile: every group leaves its accumulators in memory (register order, so the
  // stores and loads are contiguous per wave) and takes a ticket; the group that draws the last ticket adds the
  // slices in slice order, whichever group it is, so the sum does not depend on timing, and runs the epilogue.
  if (p.splits) {
    constexpr int64_t SLICE = (int64_t)F * F * 16 * NTHREADS;
    float* mine = p.part + (bz * nblocks + block) * SLICE + tid;
#pragma unroll
    for (int f = 0; f < F * F; ++f)
#pragma unroll
      for (int v = 0; v < 16; ++v) endia::store_shared(mine + (f * 16 + v) * NTHREADS, acc[f / F][f % F][v]);
    if (!endia::arrive_last(&p.tickets[block], (unsigned)p.splits, reinterpret_cast<int*>(As))) return;
    zero_acc<F, F>(acc);
    for (int s = 0; s < p.splits; ++s) {
      const float* theirs = p.part + ((int64_t)s * nblocks + block) * SLICE + tid;
#pragma unroll
      for (int f = 0; f < F * F; ++f) {
        float t[16];  // sixteen loads in flight, then sixteen additions
#pragma unroll
        for (int v = 0; v < 16; ++v) t[v] = endia::load_shared(theirs + (f * 16 + v) * NTHREADS);
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[f / F][f % F][v] += t[v];
      }
    }
  }

  // The 128 x 128 tile inside the matrix, no accumulation, relu or tanh: a body with everything uniform decided once.
  // The general loop below tests bounds, accumulation and the kind of activation per element with the bodies of tanh
  // and sin inlined 64 times, and fetching those instructions costs more than running them.
  if constexpr (F == 2 && EPI != ENDIA_EPI_NONE) {
    const bool relu = p.act == ENDIA_OP_RELU, tanh_ok = p.act == ENDIA_OP_TANH && (EPI != ENDIA_EPI_ACT_GRAD || p.from_out);
    const bool plain_store = !p.accumulate && !p.splits && !(EPI == ENDIA_EPI_BIAS_ACT && aux_out);
    if (m0 + BM <= p.M && n0 + BN <= p.N && plain_store && (EPI == ENDIA_EPI_BIAS || relu || tanh_ok)) {
      const int64_t at = (int64_t)(m0 + wm * 64 + 4 * h) * p.ldc + (n0 + wn * 64 + l32);
      float* __restrict__ Ct = C + at;
      float bias2[F];
#pragma unroll
      for (int fn = 0; fn < F; ++fn) bias2[fn] = (EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) ? p.bias[n0 + wn * 64 + fn * 32 + l32] : 0.f;
#pragma unroll
      for (int fm = 0; fm < F; ++fm)
#pragma unroll
        for (int fn = 0; fn < F; ++fn) {
          float aux[16] = {};
          if constexpr (EPI == ENDIA_EPI_ACT_GRAD) {
#pragma unroll
            for (int v = 0; v < 16; ++v) aux[v] = aux_in[at + (int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32];
          }
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float r = acc[fm][fn][v] + bias2[fn];
            if constexpr (EPI == ENDIA_EPI_BIAS_ACT) r = relu ? (r > 0.f ? r : 0.f) : tanhf(r);
            if constexpr (EPI == ENDIA_EPI_ACT_GRAD) r *= relu ? (aux[v] > 0.f ? 1.f : 0.f) : 1.f - aux[v] * aux[v];
            Ct[(int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32] = r;
          }
        }
      return;
    }
  }

#pragma unroll
  for (int fm = 0; fm < F; ++fm)
#pragma unroll
    for (int fn = 0; fn < F; ++fn) {
      int col = n0 + wn * 32 * F + fn * 32 + l32;
      if (col >= p.N) continue;
      // accumulation: the block's sixteen old values are requested together, ahead of the stores (the compiler must
      // assume that a store changes what a later load reads, and would wait for each in turn)
      float old[16];
      if (p.accumulate) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = m0 + wm * 32 * F + fm * 32 + acc_row(v, h);
          old[v] = row < p.M ? C[(int64_t)row * p.ldc + col] : 0.f;
        }
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int row = m0 + wm * 32 * F + fm * 32 + acc_row(v, h);
        if (row >= p.M) continue;
        if constexpr (PRE) epilogue_apply<EPI>(p, C, aux_out, row, col, acc[fm][fn][v], bias_pre, aux_pre[v], &old[v]);
        else {
          const float bias_v = (EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) ? p.bias[col] : 0.f;
          const float aux_v = EPI == ENDIA_EPI_ACT_GRAD ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
          epilogue_apply<EPI>(p, C, aux_out, row, col, acc[fm][fn][v], bias_v, aux_v, &old[v]);
        }
      }
    }
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int F, bool SHORTK = false, bool A_VEC = true, bool B_VEC = true>
__global__ __launch_bounds__(NTHREADS, 4) void sgemm_mfma_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) float As[TileShape<A_KMAJOR, 64 * F>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<B_KMAJOR, 64 * F>::FLOATS];
  gemm_tile<A_KMAJOR, B_KMAJOR, EPI, F, SHORTK, A_VEC, B_VEC>(p, blockIdx.x, gridDim.x, blockIdx.y, As, Bs);
}

template <int EPI, int F, bool SHORTK, bool A_VEC = true, bool B_VEC = true>
void launch_mfma(const GemmArgs& p, int transA, int transB, dim3 grid, hipStream_t s) {
  const bool ak = !transA, bk = transB != 0;
  if (ak && bk) hipLaunchKernelGGL((sgemm_mfma_kernel<true, true, EPI, F, SHORTK, A_VEC, B_VEC>), grid, dim3(NTHREADS), 0, s, p);
  else if (ak && !bk) hipLaunchKernelGGL((sgemm_mfma_kernel<true, false, EPI, F, SHORTK, A_VEC, B_VEC>), grid, dim3(NTHREADS), 0, s, p);
  else if (!ak && bk) hipLaunchKernelGGL((sgemm_mfma_kernel<false, true, EPI, F, SHORTK, A_VEC, B_VEC>), grid, dim3(NTHREADS), 0, s, p);
  else hipLaunchKernelGGL((sgemm_mfma_kernel<false, false, EPI, F, SHORTK, A_VEC, B_VEC>), grid, dim3(NTHREADS), 0, s, p);
}

template <int F, bool SHORTK = false, bool A_VEC = true, bool B_VEC = true>
void launch_mfma_epi(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s) {
  switch (epi) {
    case ENDIA_EPI_NONE: launch_mfma<ENDIA_EPI_NONE, F, SHORTK, A_VEC, B_VEC>(p, transA, transB, grid, s); break;
    case ENDIA_EPI_BIAS: launch_mfma<ENDIA_EPI_BIAS, F, SHORTK, A_VEC, B_VEC>(p, transA, transB, grid, s); break;
    case ENDIA_EPI_BIAS_ACT: launch_mfma<ENDIA_EPI_BIAS_ACT, F, SHORTK, A_VEC, B_VEC>(p, transA, transB, grid, s); break;
    default: launch_mfma<ENDIA_EPI_ACT_GRAD, F, SHORTK, A_VEC, B_VEC>(p, transA, transB, grid, s); break;
  }
}

}  // namespace endia_gemm
