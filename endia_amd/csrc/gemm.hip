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
#include "mfma_tile.h"
#include "ticket.h"

#include <stdlib.h>

#include <type_traits>
#include <vector>

namespace {

using namespace mfma;

constexpr int NTHREADS = 256;  // four waves, 2 x 2

struct GemmArgs {
  const float* A;
  const float* B;
  float* C;
  const float* bias;
  const float* aux_in;
  float* aux_out;
  int64_t lda, ldb, ldc;
  int64_t sA, sB, sC;
  int M, N, K;
  int tiles_m, tiles_n;
  int k_split;    // > 0: grid.y indexes slices of K of this length instead of batch entries
  int splits;     // > 0: the slices' partial sums meet in `part` and the last group of a tile to arrive finishes it
  float* part;    // [splits][tiles][accumulator registers][256 lanes]
  unsigned* tickets;  // one arrival counter per tile, zero between launches
  int act;        // endia_hip_unary_op
  int from_out;   // activation gradient from stored output instead of pre-activation
  int accumulate;
  int colsum;     // also write sum_k B[k][n] to aux_out[n] (B MN-major; done by the work-groups of the first tile row)
};

__device__ __forceinline__ float act_fwd(int act, float z) {
  switch (act) {
    case ENDIA_OP_RELU: return z > 0.f ? z : 0.f;
    case ENDIA_OP_TANH: return tanhf(z);
    case ENDIA_OP_SIN: return sinf(z);
    default: return z;
  }
}

__device__ __forceinline__ float act_grad(int act, int from_out, float aux) {
  switch (act) {
    case ENDIA_OP_RELU: return aux > 0.f ? 1.f : 0.f;
    case ENDIA_OP_TANH: {
      float a = from_out ? aux : tanhf(aux);
      return 1.f - a * a;
    }
    case ENDIA_OP_SIN: return cosf(aux);
    default: return 1.f;
  }
}

// bias_v = bias[col] and aux_v = aux_in[row, col], fetched by the caller (early, where registers allow)
template <int EPI>
__device__ __forceinline__ void epilogue_apply(const GemmArgs& p, float* __restrict__ C, float* __restrict__ aux_out,
                                               int row, int col, float v, float bias_v, float aux_v) {
  int64_t off = (int64_t)row * p.ldc + col;
  if (EPI == ENDIA_EPI_BIAS) {
    v += bias_v;
  } else if (EPI == ENDIA_EPI_BIAS_ACT) {
    v += bias_v;
    if (aux_out) aux_out[off] = v;
    v = act_fwd(p.act, v);
  } else if (EPI == ENDIA_EPI_ACT_GRAD) {
    v *= act_grad(p.act, p.from_out, aux_v);
  }
  if (p.accumulate) v += C[off];
  C[off] = v;
}

template <int EPI>
__device__ __forceinline__ void epilogue_store(const GemmArgs& p, float* __restrict__ C,
                                               const float* __restrict__ aux_in,
                                               float* __restrict__ aux_out, int row, int col, float v) {
  const float bias_v = (EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) ? p.bias[col] : 0.f;
  const float aux_v = EPI == ENDIA_EPI_ACT_GRAD ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
  epilogue_apply<EPI>(p, C, aux_out, row, col, v, bias_v, aux_v);
}

// F = MFMA blocks per wave in each direction: F = 2 gives the 128 x 128 tile, F = 1 the 64 x 64 tile
// used when the larger one would leave CUs without work.
// SHORTK (64 x 64 tile only): the reduction is at most four K tiles long, which is the case of every product
// of a small model (the reference's sine-fit MLP has K <= 128 throughout). Such launches are a handful of
// work-groups whose time is a chain of global-load latencies, one per K tile; here the loads of all four tiles
// are issued before anything else, so that latency is paid once.
// One work-group's tile of one product: group `block` of `nblocks`, batch entry (or K slice) bz, LDS handed in.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int F, bool SHORTK>
__device__ __forceinline__ void gemm_tile(const GemmArgs& p, int block, int nblocks, int64_t bz, float* __restrict__ As,
                                          float* __restrict__ Bs) {
  static_assert(!SHORTK || F == 1, "the short-reduction variant exists for the 64 x 64 tile");
  constexpr int BM = 64 * F, BN = 64 * F;
  using LA = MatrixTileLoader<A_KMAJOR, BM, NTHREADS>;
  using LB = MatrixTileLoader<B_KMAJOR, BN, NTHREADS>;

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
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int row = m0 + wm * 32 * F + fm * 32 + acc_row(v, h);
        if (row >= p.M) continue;
        if constexpr (PRE) epilogue_apply<EPI>(p, C, aux_out, row, col, acc[fm][fn][v], bias_pre, aux_pre[v]);
        else epilogue_store<EPI>(p, C, aux_in, aux_out, row, col, acc[fm][fn][v]);
      }
    }
}

// The 256 x 256 tile: one work-group per CU, one wave per SIMD, each wave 128 x 128 = 4 x 4 MFMA blocks (256 accumulator
// registers per lane). With nobody else on the SIMD to fill a wave's stalls, the order of instructions is the
// schedule, and whatever is not an MFMA is hidden only if it sits BETWEEN two MFMAs (the matrix pipe is busy for 64
// cycles per instruction; what follows in program order issues meanwhile). So a K tile is 16 steps of 16 MFMAs, cut
// into quads, and in front of every quad goes one small piece of the other work, fenced by scheduling barriers so the
// compiler keeps it there:
//   * LDS holds two stages; steps 0-11 read, block by block, the fragments of the next group of four steps from the
//     current stage (one group ahead of their use), steps 12-15 the first fragments of the next tile from the other
//     stage, behind the tile's only barrier (at step 12 everybody has written its share of that stage and has read
//     the last of this one);
//   * steps 0-11 also move the next tile, one 16-byte piece per lane at a time, from registers to the other stage and
//     request the same piece of the tile after it from memory, which then has a whole K tile (~7 us) to arrive.
// Tiles past the end of K load as zeros (descriptor bounds) into a stage nobody reads.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI>
__device__ __forceinline__ void gemm_tile256(const GemmArgs& p, int block, int nblocks, int64_t bz, float* __restrict__ smem) {
  constexpr int F = 4, BM = 256, BN = 256;
  using LA = MatrixTileLoader<A_KMAJOR, BM, NTHREADS>;
  using LB = MatrixTileLoader<B_KMAJOR, BN, NTHREADS>;
  constexpr int SA = TileShape<A_KMAJOR, BM>::FLOATS, STAGE = SA + TileShape<B_KMAJOR, BN>::FLOATS;
  static_assert(BK == 32 && LA::PASSES == 8 && LB::PASSES == 8, "the step plan below is written for these");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, h = lane >> 5;
  int tm, tn;
  tile_of_block(block, nblocks, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  float* __restrict__ C = p.C + bz * p.sC;
  const float* __restrict__ aux_in = p.aux_in ? p.aux_in + bz * p.sC : nullptr;
  float* __restrict__ aux_out = p.aux_out ? p.aux_out + bz * p.sC : nullptr;
  const int K = p.K;
  LA la;
  LB lb;
  la.init(p.A + bz * p.sA, p.lda, m0, p.M, K, tid);
  lb.init(p.B + bz * p.sB, p.ldb, n0, p.N, K, tid);

  floatx16 acc[F][F];
  zero_acc<F, F>(acc);
  const int a_row = wm * 128 + l32, b_col = wn * 128 + l32;

  la.load(K);
  lb.load(K);
  la.store(smem);
  lb.store(smem + SA);
  la.advance();
  lb.advance();
  la.load(K - BK);
  lb.load(K - BK);
  __syncthreads();
  float af[2][F][4], bf[2][F][4];
#pragma unroll
  for (int f = 0; f < F; ++f) {
    load_fragment_block<A_KMAJOR, BM>(smem, a_row + 32 * f, h, 0, af[0][f]);
    load_fragment_block<B_KMAJOR, BN>(smem + SA, b_col + 32 * f, h, 0, bf[0][f]);
  }
  // Loop state that changes from tile to tile lives in scalar registers: operand base pointers and the bytes left in
  // their descriptors (32-bit: the host takes this tile only for operands below 2 GiB). A vector ALU instruction
  // between two MFMAs of a lone wave is not hidden the way an LDS or memory instruction is (a select per load cost
  // 4 % of the kernel), so there is none: LDS addresses are loop constants because the loop body is written out for
  // both stages, and the K tail is handled once, when it comes, by rewriting the lanes' offsets.
  const char* base_a = reinterpret_cast<const char*>(la.base);
  const char* base_b = reinterpret_cast<const char*>(lb.base);
  int rec_a = (int)(la.records < 0 ? 0 : (la.records > 0x7FFFFFF0ll ? 0x7FFFFFF0ll : la.records));
  int rec_b = (int)(lb.records < 0 ? 0 : (lb.records > 0x7FFFFFF0ll ? 0x7FFFFFF0ll : lb.records));
  const int step_a = (int)la.step, step_b = (int)lb.step;
  int k_left = K - BK;  // reduction elements from the tile the loaders point at to the end
  // Per stage and operand, the lane's LDS position for fragment reads and for staging stores, each in a register of
  // its own (the empty asm keeps the compiler from deriving one from another with an addition inside the loop);
  // everything else in an LDS address is a constant within reach of the instruction's 64 KiB offset field.
  int fa_at[2], fb_at[2], sa_at[2], sb_at[2];
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    fa_at[st] = st * STAGE + fragment_lane_offset<A_KMAJOR, BM>(a_row, h);
    fb_at[st] = st * STAGE + SA + fragment_lane_offset<B_KMAJOR, BN>(b_col, h);
    sa_at[st] = st * STAGE + la.lds_off;
    sb_at[st] = st * STAGE + SA + lb.lds_off;
    asm volatile("" : "+v"(fa_at[st]), "+v"(fb_at[st]), "+v"(sa_at[st]), "+v"(sb_at[st]));
  }
  auto tile_body = [&](auto stage) {
    constexpr int ST = decltype(stage)::value;
    base_a += step_a;  // the tile after the next one
    base_b += step_b;
    rec_a = rec_a > step_a ? rec_a - step_a : 0;
    rec_b = rec_b > step_b ? rec_b - step_b : 0;
    k_left -= BK;
    if (k_left < BK) {
      la.mask_tail(k_left);
      lb.mask_tail(k_left);
    }
    const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_a), 0, rec_a, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_b), 0, rec_b, 0x00020000);
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      const int j = s >> 2, i = s & 3, cur = j & 1, nxt = cur ^ 1;
      if (s == 12) __syncthreads();
      const int fs = s < 12 ? ST : ST ^ 1;  // stage the fragments are read from
      const int jn = s < 12 ? j + 1 : 0;
      auto quad = [&](int fm) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int fn = 0; fn < F; ++fn)
          acc[fm][fn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][fm][i], bf[cur][fn][i], acc[fm][fn], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      };
      load_fragment_at<A_KMAJOR, BM>(smem, fa_at[fs], i, jn, af[nxt][i]);
      quad(0);
      load_fragment_at<B_KMAJOR, BN>(smem, fb_at[fs], i, jn, bf[nxt][i]);
      quad(1);
      if (s < 8) {
        la.store_pass_at(smem, sa_at[ST ^ 1], s);
        la.load_pass(s, rsa);
      } else if (s < 12) {
        lb.store_pass_at(smem, sb_at[ST ^ 1], s - 4);
        lb.load_pass(s - 4, rsb);
      }
      quad(2);
      if (s < 4) {
        lb.store_pass_at(smem, sb_at[ST ^ 1], s);
        lb.load_pass(s, rsb);
      }
      quad(3);
    }
  };
  // two K tiles per trip, one per LDS stage; an odd tile count runs one more tile of zeros
  const int T = (K + BK - 1) / BK;
  for (int t = 0; t < T; t += 2) {
    tile_body(std::integral_constant<int, 0>());
    tile_body(std::integral_constant<int, 1>());
  }

  // Epilogue. Nothing overlaps it (the CU's only tile ends here), so what it reads is requested ahead of the stores,
  // which the compiler must assume to alias it: the bias of the lane's four columns up front, and the activation
  // operand of the next 32 x 32 block before the current block is stored.
  // The general form below tests bounds, accumulation and the kind of activation per element; written out for 256
  // elements per lane with the bodies of tanh and sin inlined that is 60-70 thousand instructions, and fetching them
  // costs more than executing them (60-90 us per launch at 4096^3). The usual cases (a tile inside the matrix, no
  // accumulation, relu or tanh) therefore have a body of their own with everything uniform decided once.
  float bias_v[F];
#pragma unroll
  for (int fn = 0; fn < F; ++fn) {
    const int col = n0 + wn * 128 + fn * 32 + l32;
    bias_v[fn] = ((EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) && col < p.N) ? p.bias[col] : 0.f;
  }
  auto fetch_aux = [&](int blk, float (&aux)[16]) {
    if constexpr (EPI == ENDIA_EPI_ACT_GRAD) {
      const int fm = blk >> 2, fn = blk & 3;
      const int col = n0 + wn * 128 + fn * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 128 + fm * 32 + acc_row(v, h);
        aux[v] = (row < p.M && col < p.N) ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
      }
    }
  };
  // ACT: ENDIA_OP_TANH or ENDIA_OP_RELU (ignored by the plain and bias epilogues); the tile lies inside C, C = result
  auto store_inside = [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    float* __restrict__ Ct = C + (int64_t)(m0 + wm * 128 + 4 * h) * p.ldc + (n0 + wn * 128 + l32);
    const float* __restrict__ Xt = EPI == ENDIA_EPI_ACT_GRAD ? aux_in + (int64_t)(m0 + wm * 128 + 4 * h) * p.ldc + (n0 + wn * 128 + l32) : nullptr;
    float cur[16] = {}, nxt[16] = {};
    auto fetch = [&](int blk, float (&aux)[16]) {
      if constexpr (EPI == ENDIA_EPI_ACT_GRAD) {
        const int fm = blk >> 2, fn = blk & 3;
#pragma unroll
        for (int v = 0; v < 16; ++v) aux[v] = Xt[(int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32];
      }
    };
    fetch(0, cur);
#pragma unroll
    for (int blk = 0; blk < F * F; ++blk) {
      const int fm = blk >> 2, fn = blk & 3;
      if (blk + 1 < F * F) fetch(blk + 1, nxt);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float r = acc[fm][fn][v];
        if constexpr (EPI == ENDIA_EPI_BIAS) r += bias_v[fn];
        if constexpr (EPI == ENDIA_EPI_BIAS_ACT) {
          r += bias_v[fn];
          r = ACT == ENDIA_OP_TANH ? tanhf(r) : (r > 0.f ? r : 0.f);
        }
        if constexpr (EPI == ENDIA_EPI_ACT_GRAD) r *= ACT == ENDIA_OP_TANH ? 1.f - cur[v] * cur[v] : (cur[v] > 0.f ? 1.f : 0.f);
        Ct[(int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32] = r;
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) cur[v] = nxt[v];
    }
  };
  if (m0 + BM <= p.M && n0 + BN <= p.N && !p.accumulate) {
    if constexpr (EPI == ENDIA_EPI_NONE || EPI == ENDIA_EPI_BIAS) {
      store_inside(std::integral_constant<int, ENDIA_OP_RELU>());
      return;
    } else if constexpr (EPI == ENDIA_EPI_BIAS_ACT) {
      if (!aux_out && p.act == ENDIA_OP_TANH) { store_inside(std::integral_constant<int, ENDIA_OP_TANH>()); return; }
      if (!aux_out && p.act == ENDIA_OP_RELU) { store_inside(std::integral_constant<int, ENDIA_OP_RELU>()); return; }
    } else {
      if (p.act == ENDIA_OP_TANH && p.from_out) { store_inside(std::integral_constant<int, ENDIA_OP_TANH>()); return; }
      if (p.act == ENDIA_OP_RELU) { store_inside(std::integral_constant<int, ENDIA_OP_RELU>()); return; }
    }
  }
  float aux_cur[16] = {}, aux_nxt[16] = {};
  fetch_aux(0, aux_cur);
#pragma unroll
  for (int blk = 0; blk < F * F; ++blk) {
    const int fm = blk >> 2, fn = blk & 3;
    if (blk + 1 < F * F) fetch_aux(blk + 1, aux_nxt);
    const int col = n0 + wn * 128 + fn * 32 + l32;
    if (col < p.N) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 128 + fm * 32 + acc_row(v, h);
        if (row < p.M) epilogue_apply<EPI>(p, C, aux_out, row, col, acc[fm][fn][v], bias_v[fn], aux_cur[v]);
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) aux_cur[v] = aux_nxt[v];
  }
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(NTHREADS, 1) void sgemm_mfma256_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) float smem256[];
  gemm_tile256<A_KMAJOR, B_KMAJOR, EPI>(p, blockIdx.x, gridDim.x, blockIdx.y, smem256);
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int F, bool SHORTK = false>
__global__ __launch_bounds__(NTHREADS, 4) void sgemm_mfma_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) float As[TileShape<A_KMAJOR, 64 * F>::FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[TileShape<B_KMAJOR, 64 * F>::FLOATS];
  gemm_tile<A_KMAJOR, B_KMAJOR, EPI, F, SHORTK>(p, blockIdx.x, gridDim.x, blockIdx.y, As, Bs);
}

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

template <int EPI, int F, bool SHORTK>
void launch_mfma(const GemmArgs& p, int transA, int transB, dim3 grid, hipStream_t s) {
  const bool ak = !transA, bk = transB != 0;
  if (ak && bk) hipLaunchKernelGGL((sgemm_mfma_kernel<true, true, EPI, F, SHORTK>), grid, dim3(NTHREADS), 0, s, p);
  else if (ak && !bk) hipLaunchKernelGGL((sgemm_mfma_kernel<true, false, EPI, F, SHORTK>), grid, dim3(NTHREADS), 0, s, p);
  else if (!ak && bk) hipLaunchKernelGGL((sgemm_mfma_kernel<false, true, EPI, F, SHORTK>), grid, dim3(NTHREADS), 0, s, p);
  else hipLaunchKernelGGL((sgemm_mfma_kernel<false, false, EPI, F, SHORTK>), grid, dim3(NTHREADS), 0, s, p);
}

template <bool AK, bool BKM, int EPI>
int32_t launch_one256(const GemmArgs& p, dim3 grid, hipStream_t s) {
  constexpr size_t lds = 2 * (size_t)(TileShape<AK, 256>::FLOATS + TileShape<BKM, 256>::FLOATS) * sizeof(float);
  static bool allowed = false;  // more than 64 KiB of LDS has to be asked for, once per kernel
  if (!allowed) {
    ENDIA_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sgemm_mfma256_kernel<AK, BKM, EPI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed = true;
  }
  hipLaunchKernelGGL((sgemm_mfma256_kernel<AK, BKM, EPI>), grid, dim3(NTHREADS), lds, s, p);
  return ENDIA_HIP_OK;
}

template <int EPI>
int32_t launch_mfma256(const GemmArgs& p, int transA, int transB, dim3 grid, hipStream_t s) {
  const bool ak = !transA, bk = transB != 0;
  if (ak && bk) return launch_one256<true, true, EPI>(p, grid, s);
  if (ak && !bk) return launch_one256<true, false, EPI>(p, grid, s);
  if (!ak && bk) return launch_one256<false, true, EPI>(p, grid, s);
  return launch_one256<false, false, EPI>(p, grid, s);
}

int32_t launch_mfma256_epi(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s) {
  switch (epi) {
    case ENDIA_EPI_NONE: return launch_mfma256<ENDIA_EPI_NONE>(p, transA, transB, grid, s);
    case ENDIA_EPI_BIAS: return launch_mfma256<ENDIA_EPI_BIAS>(p, transA, transB, grid, s);
    case ENDIA_EPI_BIAS_ACT: return launch_mfma256<ENDIA_EPI_BIAS_ACT>(p, transA, transB, grid, s);
    default: return launch_mfma256<ENDIA_EPI_ACT_GRAD>(p, transA, transB, grid, s);
  }
}

template <int F, bool SHORTK = false>
void launch_mfma_epi(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s) {
  switch (epi) {
    case ENDIA_EPI_NONE: launch_mfma<ENDIA_EPI_NONE, F, SHORTK>(p, transA, transB, grid, s); break;
    case ENDIA_EPI_BIAS: launch_mfma<ENDIA_EPI_BIAS, F, SHORTK>(p, transA, transB, grid, s); break;
    case ENDIA_EPI_BIAS_ACT: launch_mfma<ENDIA_EPI_BIAS_ACT, F, SHORTK>(p, transA, transB, grid, s); break;
    default: launch_mfma<ENDIA_EPI_ACT_GRAD, F, SHORTK>(p, transA, transB, grid, s); break;
  }
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

  // The vector path loads 4 floats at a time along the contiguous index of each operand.
  const bool a_ok = aligned16(A) && lda % 4 == 0 && sA % 4 == 0 && (transA ? M % 4 == 0 : K % 4 == 0);
  const bool b_ok = aligned16(B) && ldb % 4 == 0 && sB % 4 == 0 && (transB ? K % 4 == 0 : N % 4 == 0);
  const bool big = M * N >= 64 * 64 && K >= 8 && lda < (1ll << 22) && ldb < (1ll << 22);  // 32-bit tile offsets
  if (a_ok && b_ok && big) {
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
    // 256 x 256 tiles, one per CU at a time: when they fill every round over the CUs (4096^2 outputs are 256 of them)
    const int64_t t256 = ceil_div64(M, 256) * ceil_div64(N, 256) * batch;
    const bool fits256 = (double)(ceil_div64(M, 256) * 256) * (double)(ceil_div64(N, 256) * 256) <= 1.1 * (double)M * (double)N;
    // (its descriptors count bytes in 32 bits; the column sums of a small B ride in the launch of the other kernels)
    const bool has256 = !(colsum && K * N <= (1ll << 20)) && (transA ? K : M) * lda < (1ll << 29) && (transB ? N : K) * ldb < (1ll << 29);
    if (g_forced_tile == 64) F = 1;
    else if (g_forced_tile == 128) F = 2;
    if (has256 && (g_forced_tile == 256 || (g_forced_tile == 0 && fits256 && t256 >= cus && balance(t256) >= 0.9 && K >= 256))) F = 4;
    p.tiles_m = (int)ceil_div64(M, 64 * F);
    p.tiles_n = (int)ceil_div64(N, 64 * F);
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
    if (F == 4) {
      int32_t rc = launch_mfma256_epi(p, epi, transA, transB, grid, s);
      if (rc) return rc;
    } else if (F == 2) launch_mfma_epi<2>(p, epi, transA, transB, grid, s);
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
  if (dW) {
    int32_t rc = sgemm_impl(1, 0, K, N, B, x, K, g, N, dW, N, 1, 0, 0, 0, ENDIA_EPI_NONE | (db ? ENDIA_GEMM_COLSUM_B : 0),
                            ENDIA_OP_IDENTITY, nullptr, nullptr, db);
    if (rc) return rc;
  } else if (db && N > 0) {
    int32_t rc = col_reduce(1, B, N, g, db, 1.f);
    if (rc) return rc;
  }
  if (dx) return sgemm_impl(0, 1, B, K, N, g, N, W, N, dx, K, 1, 0, 0, 0, epi_x, aux ? act_flags : ENDIA_OP_IDENTITY, nullptr, aux, nullptr);
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

extern "C" int32_t endia_hip_gemm_force_tile(int32_t tile) {
  ENDIA_CHECK_ARG(tile == 0 || tile == 64 || tile == 128 || tile == 256, "endia_hip_gemm_force_tile: tile %d is not one of 0, 64, 128, 256", tile);
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
