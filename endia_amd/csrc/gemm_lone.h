// fp32 GEMM tiles that run ONE work-group per CU and one wave per SIMD: matmul_fwd and both products of matmul_vjp
// (endia/functional/binary_ops/matmul_op.mojo:162-199, 278-283) for products whose tiles fill the chip about once.
//
// A work-group of four waves (2 x 2) owns a (64 FM) x (64 FN) tile of C; each wave owns FM x FN blocks of
// v_mfma_f32_32x32x2_f32. With nobody else on the SIMD to fill a wave's stalls, the order of instructions is the
// schedule, and whatever is not an MFMA is hidden only if it sits BETWEEN two MFMAs (the matrix pipe is busy for 64
// cycles per instruction; what follows in program order issues meanwhile) and is not a vector ALU instruction. So a K
// tile (32) is 16 steps of FM x FN MFMAs, cut into up to four groups, and in front of every group goes one small piece
// of the other work, fenced by scheduling barriers so that the compiler keeps it there:
//   * LDS holds two stages; steps 0-11 read, block by block, the fragments of the next group of four steps from the
//     current stage (one group ahead of their use), steps 12-15 the first fragments of the next tile from the other
//     stage, behind the tile's only barrier (at step 12 everybody has written its share of that stage and has read
//     the last of this one);
//   * steps 0-11 also move the next tile, one 16-byte piece per lane at a time, from registers to the other stage and
//     request the same piece of a later tile from memory: the tile after the next one (DEPTH 1, a whole K tile of
//     time to arrive) or the one after that (DEPTH 2, two register sets; measured on 128 x 64 tiles, whose K tile
//     takes under a microsecond: no gain, the loads are not what such a tile waits for, so every tile here uses 1).
// Tiles past the end of K load as zeros (descriptor bounds) into a stage nobody reads.
// The loop holds no vector ALU instruction: what changes per tile (operand base pointers, bytes left in the
// descriptors, 32-bit) lives in scalar registers; every LDS address is a per-lane register fixed before the loop plus a
// constant within the instruction's offset field, which takes the loop body written out once per stage.
#pragma once
#include <type_traits>

#include "common.h"
#include "gemm_args.h"
#include "mfma_tile.h"

namespace endia_gemm {

using namespace mfma;

template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int FM, int FN, int DEPTH>
__device__ __forceinline__ void gemm_tile_lone(const GemmArgs& p, int block, int nblocks, int64_t bz, float* __restrict__ smem) {
  constexpr int BM = 64 * FM, BN = 64 * FN;
  using LA = MatrixTileLoader<A_KMAJOR, BM, NTHREADS>;
  using LB = MatrixTileLoader<B_KMAJOR, BN, NTHREADS>;
  constexpr int PA = LA::PASSES, PB = LB::PASSES, P = PA + PB;  // 16-byte pieces per lane and K tile
  constexpr int SA = TileShape<A_KMAJOR, BM>::FLOATS, STAGE = SA + TileShape<B_KMAJOR, BN>::FLOATS;
  constexpr int NMFMA = FM * FN;                  // per step
  constexpr int GROUP = NMFMA >= 4 ? NMFMA / 4 : 1;  // MFMAs between two pieces of other work
  constexpr int NGROUPS = NMFMA / GROUP;
  constexpr int NBLK = FM + FN;                   // fragment blocks per group of four steps
  static_assert(BK == 32 && P <= 16 && (DEPTH == 1 || DEPTH == 2), "the step plan below is written for these");
  static_assert(NGROUPS * GROUP == NMFMA, "MFMAs of a step do not divide into groups");

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

  floatx16 acc[FM][FN];
  zero_acc<FM, FN>(acc);
  const int a_row = wm * 32 * FM + l32, b_col = wn * 32 * FN + l32;

  // staging registers: tile u of the reduction waits in set u % DEPTH
  float4 ra[DEPTH][PA], rb[DEPTH][PB];
  auto request = [&](int set, __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb) {
#pragma unroll
    for (int i = 0; i < PA; ++i) ra[set][i] = buffer_load_f4(rsa, la.voff[i]);
#pragma unroll
    for (int i = 0; i < PB; ++i) rb[set][i] = buffer_load_f4(rsb, lb.voff[i]);
  };
  // prologue: tiles 0 .. DEPTH requested, tile 0 in stage 0
#pragma unroll
  for (int u = 0; u <= DEPTH; ++u) {
    if (u) {
      la.advance();
      lb.advance();
    }
    la.mask_tail(K - u * BK);
    lb.mask_tail(K - u * BK);
    if (u == DEPTH) {  // tile 0 leaves its registers for the tile requested now
#pragma unroll
      for (int i = 0; i < PA; ++i) *reinterpret_cast<float4*>(&smem[la.lds_off + i * LA::ROWS_PER_PASS * LA::LD]) = ra[0][i];
#pragma unroll
      for (int i = 0; i < PB; ++i) *reinterpret_cast<float4*>(&smem[SA + lb.lds_off + i * LB::ROWS_PER_PASS * LB::LD]) = rb[0][i];
    }
    request(u % DEPTH, make_rsrc(la.base, la.records), make_rsrc(lb.base, lb.records));
  }
  __syncthreads();
  float af[2][FM][4], bf[2][FN][4];
#pragma unroll
  for (int f = 0; f < FM; ++f) load_fragment_block<A_KMAJOR, BM>(smem, a_row + 32 * f, h, 0, af[0][f]);
#pragma unroll
  for (int f = 0; f < FN; ++f) load_fragment_block<B_KMAJOR, BN>(smem + SA, b_col + 32 * f, h, 0, bf[0][f]);

  const char* base_a = reinterpret_cast<const char*>(la.base);
  const char* base_b = reinterpret_cast<const char*>(lb.base);
  int rec_a = (int)(la.records < 0 ? 0 : (la.records > 0x7FFFFFF0ll ? 0x7FFFFFF0ll : la.records));
  int rec_b = (int)(lb.records < 0 ? 0 : (lb.records > 0x7FFFFFF0ll ? 0x7FFFFFF0ll : lb.records));
  const int step_a = (int)la.step, step_b = (int)lb.step;
  int k_left = K - DEPTH * BK;  // reduction elements from the tile the loaders point at to the end
  // Per stage and operand, the lane's LDS position for fragment reads and for staging stores, each in a register of
  // its own (the empty asm keeps the compiler from deriving one from another with an addition inside the loop).
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
    constexpr int SET = DEPTH == 2 ? (ST ^ 1) : 0;  // registers of the tile that moves to LDS during this body
    base_a += step_a;  // the tile requested during this body
    base_b += step_b;
    rec_a = rec_a > step_a ? rec_a - step_a : 0;
    rec_b = rec_b > step_b ? rec_b - step_b : 0;
    k_left -= BK;
    if (k_left < BK) {
      // Only the last tiles of the reduction come here. The empty asm keeps this a real (scalar) branch: turned into
      // per-lane selects, as the compiler otherwise does, it would put a dozen vector ALU instructions into every tile.
      asm volatile("" ::: "memory");
      la.mask_tail(k_left);
      lb.mask_tail(k_left);
    }
    const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_a), 0, rec_a, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_b), 0, rec_b, 0x00020000);
    // piece q of the next tile: registers -> other stage, then the request for the same piece of a later tile
    auto move_piece = [&](int q) {
      if (q < PA) {
        *reinterpret_cast<float4*>(&smem[sa_at[ST ^ 1] + q * LA::ROWS_PER_PASS * LA::LD]) = ra[SET][q];
        ra[SET][q] = buffer_load_f4(rsa, la.voff[q]);
      } else {
        const int b = (q - PA + (P > 12 ? PB / 2 : 0)) % PB;
        *reinterpret_cast<float4*>(&smem[sb_at[ST ^ 1] + b * LB::ROWS_PER_PASS * LB::LD]) = rb[SET][b];
        rb[SET][b] = buffer_load_f4(rsb, lb.voff[b]);
      }
    };
    // fragment block r of the next group of four steps, A and B blocks alternating while both last
    auto read_block = [&](int r, int fs, int jn, int nxt) {
      constexpr int PAIRS = FM < FN ? FM : FN;
      const bool is_a = r < 2 * PAIRS ? (r & 1) == 0 : FM > FN;
      const int f = r < 2 * PAIRS ? r >> 1 : r - PAIRS;
      if (is_a) load_fragment_at<A_KMAJOR, BM>(smem, fa_at[fs], f, jn, af[nxt][f]);
      else load_fragment_at<B_KMAJOR, BN>(smem, fb_at[fs], f, jn, bf[nxt][f]);
    };
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      const int j = s >> 2, i = s & 3, cur = j & 1, nxt = cur ^ 1;
      if (s == 12) __syncthreads();
      const int fs = s < 12 ? ST : ST ^ 1;  // stage the fragments are read from
      const int jn = s < 12 ? j + 1 : 0;
      // This step's other work, in the order it is issued (at most four pieces): fragment blocks r with
      // floor(4 r / NBLK) = i, then the pieces of the next tile that fall to step s. Piece number c of the step goes in
      // front of MFMA group c.
      const int first_r = (i * NBLK + 3) / 4, n_frag = ((i + 1) * NBLK + 3) / 4 - first_r;
#pragma unroll
      for (int g = 0; g < NGROUPS; ++g) {
#pragma unroll
        for (int r = 0; r < NBLK; ++r) {
          const int c = r - first_r;
          if (c >= 0 && c < n_frag && (c < NGROUPS ? c : NGROUPS - 1) == g) read_block(r, fs, jn, nxt);
        }
        if (s < 12) {
#pragma unroll
          for (int q = 0; q < P; ++q) {
            const bool mine = P > 12 ? (q == s || q == 12 + s) : (q * 12 / P == s);
            const int c = n_frag + (q >= 12 ? 1 : 0);
            if (mine && (c < NGROUPS ? c : NGROUPS - 1) == g) move_piece(q);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = g * GROUP; m < (g + 1) * GROUP; ++m)
          acc[m / FN][m % FN] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][m / FN][i], bf[cur][m % FN][i], acc[m / FN][m % FN], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // two K tiles per trip, one per LDS stage; an odd tile count runs one more tile of zeros
  const int T = (K + BK - 1) / BK;
  for (int t = 0; t < T; t += 2) {
    tile_body(std::integral_constant<int, 0>());
    tile_body(std::integral_constant<int, 1>());
  }

  // Epilogue. Nothing overlaps it (the CU's only tile ends here), so what it reads is requested ahead of the stores,
  // which the compiler must assume to alias it: the bias of the lane's columns up front, and the activation operand
  // of the next 32 x 32 block before the current block is stored.
  // The general form below tests bounds, accumulation and the kind of activation per element; written out for up to
  // 256 elements per lane with the bodies of tanh and sin inlined that is tens of thousands of instructions, and
  // fetching them costs more than executing them. The usual cases (a tile inside the matrix, no accumulation, relu or
  // tanh) therefore have a body of their own with everything uniform decided once.
  float bias_v[FN];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    const int col = n0 + wn * 32 * FN + fn * 32 + l32;
    bias_v[fn] = ((EPI == ENDIA_EPI_BIAS || EPI == ENDIA_EPI_BIAS_ACT) && col < p.N) ? p.bias[col] : 0.f;
  }
  auto fetch_aux = [&](int blk, float (&aux)[16]) {
    if constexpr (EPI == ENDIA_EPI_ACT_GRAD) {
      const int fm = blk / FN, fn = blk % FN;
      const int col = n0 + wn * 32 * FN + fn * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 32 * FM + fm * 32 + acc_row(v, h);
        aux[v] = (row < p.M && col < p.N) ? aux_in[(int64_t)row * p.ldc + col] : 0.f;
      }
    }
  };
  // ACT: ENDIA_OP_TANH, ENDIA_OP_RELU or ENDIA_OP_SIN (ignored by the plain and bias epilogues); the tile lies inside
  // C, C = result. SIN as a gradient takes the pre-activation (cos), the others the stored output.
  // ACCUM (plain and bias epilogues): C += result, with the old values of the next block requested before the current
  // block is stored (read where they are used, every element is a load, an addition and a store that wait for each
  // other: 57 us for the 128 elements of a lane against 6).
  auto store_inside = [&](auto act_c, auto keep_z, auto accum_c) {
    constexpr int ACT = decltype(act_c)::value;
    constexpr bool KEEP_Z = decltype(keep_z)::value;  // BIAS_ACT: also store the pre-activation to aux_out
    constexpr bool ACCUM = decltype(accum_c)::value;
    const int64_t at = (int64_t)(m0 + wm * 32 * FM + 4 * h) * p.ldc + (n0 + wn * 32 * FN + l32);
    float* __restrict__ Ct = C + at;
    float* __restrict__ Zt = KEEP_Z ? aux_out + at : nullptr;
    const float* __restrict__ Xt = EPI == ENDIA_EPI_ACT_GRAD ? aux_in + at : nullptr;
    float cur[16] = {}, nxt[16] = {};
    auto fetch = [&](int blk, float (&aux)[16]) {
      if constexpr (EPI == ENDIA_EPI_ACT_GRAD || ACCUM) {
        const float* from = ACCUM ? Ct : Xt;  // (based on Ct: no second restrict name for C)
        const int fm = blk / FN, fn = blk % FN;
#pragma unroll
        for (int v = 0; v < 16; ++v) aux[v] = from[(int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32];
      }
    };
    fetch(0, cur);
#pragma unroll
    for (int blk = 0; blk < FM * FN; ++blk) {
      const int fm = blk / FN, fn = blk % FN;
      if (blk + 1 < FM * FN) fetch(blk + 1, nxt);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t o = (int64_t)(fm * 32 + 8 * (v >> 2) + (v & 3)) * p.ldc + fn * 32;
        float r = acc[fm][fn][v];
        if constexpr (EPI == ENDIA_EPI_BIAS) r += bias_v[fn];
        if constexpr (EPI == ENDIA_EPI_BIAS_ACT) {
          r += bias_v[fn];
          if constexpr (KEEP_Z) Zt[o] = r;
          r = ACT == ENDIA_OP_TANH ? tanhf(r) : (ACT == ENDIA_OP_SIN ? sinf(r) : (r > 0.f ? r : 0.f));
        }
        if constexpr (ACCUM) r += cur[v];
        else if constexpr (EPI == ENDIA_EPI_ACT_GRAD)
          r *= ACT == ENDIA_OP_TANH ? 1.f - cur[v] * cur[v] : (ACT == ENDIA_OP_SIN ? cosf(cur[v]) : (cur[v] > 0.f ? 1.f : 0.f));
        Ct[o] = r;
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) cur[v] = nxt[v];
    }
  };
  using Relu = std::integral_constant<int, ENDIA_OP_RELU>;
  using Tanh = std::integral_constant<int, ENDIA_OP_TANH>;
  using Sin = std::integral_constant<int, ENDIA_OP_SIN>;
  // (sin and cos bring their argument reduction, a few hundred instructions and a scratch array per use: the largest
  // tile, which no sin model of the benchmarks reaches, leaves them to the general form below)
  constexpr bool SIN_BODY = FM * FN < 16;
  if constexpr (EPI == ENDIA_EPI_NONE || EPI == ENDIA_EPI_BIAS) {
    if (m0 + BM <= p.M && n0 + BN <= p.N && p.accumulate) {
      store_inside(Relu(), std::false_type(), std::true_type());
      return;
    }
  }
  if (m0 + BM <= p.M && n0 + BN <= p.N && !p.accumulate) {
    if constexpr (EPI == ENDIA_EPI_NONE || EPI == ENDIA_EPI_BIAS) {
      store_inside(Relu(), std::false_type(), std::false_type());
      return;
    } else if constexpr (EPI == ENDIA_EPI_BIAS_ACT) {
      if (!aux_out && p.act == ENDIA_OP_TANH) { store_inside(Tanh(), std::false_type(), std::false_type()); return; }
      if (!aux_out && p.act == ENDIA_OP_RELU) { store_inside(Relu(), std::false_type(), std::false_type()); return; }
      if constexpr (SIN_BODY) {
        if (aux_out && p.act == ENDIA_OP_SIN) { store_inside(Sin(), std::true_type(), std::false_type()); return; }
      }
    } else {
      if (p.act == ENDIA_OP_TANH && p.from_out) { store_inside(Tanh(), std::false_type(), std::false_type()); return; }
      if (p.act == ENDIA_OP_RELU) { store_inside(Relu(), std::false_type(), std::false_type()); return; }
      if constexpr (SIN_BODY) {
        if (p.act == ENDIA_OP_SIN && !p.from_out) { store_inside(Sin(), std::false_type(), std::false_type()); return; }
      }
    }
  }
  float aux_cur[16] = {}, aux_nxt[16] = {};
  fetch_aux(0, aux_cur);
#pragma unroll
  for (int blk = 0; blk < FM * FN; ++blk) {
    const int fm = blk / FN, fn = blk % FN;
    if (blk + 1 < FM * FN) fetch_aux(blk + 1, aux_nxt);
    const int col = n0 + wn * 32 * FN + fn * 32 + l32;
    if (col < p.N) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 32 * FM + fm * 32 + acc_row(v, h);
        if (row < p.M) epilogue_apply<EPI>(p, C, aux_out, row, col, acc[fm][fn][v], bias_v[fn], aux_cur[v]);
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) aux_cur[v] = aux_nxt[v];
  }
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int FM, int FN, int DEPTH>
__global__ __launch_bounds__(NTHREADS, 1) void sgemm_lone_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) float smem_lone[];
  gemm_tile_lone<A_KMAJOR, B_KMAJOR, EPI, FM, FN, DEPTH>(p, blockIdx.x, gridDim.x, blockIdx.y, smem_lone);
}

template <bool AK, bool BKM, int EPI, int FM, int FN, int DEPTH>
int32_t launch_lone_one(const GemmArgs& p, dim3 grid, hipStream_t s) {
  // At least 84 KiB of the CU's 160, so that no CU ever holds two of these work-groups: the dispatcher does not spread a
  // grid of one group per CU evenly when two would fit, and a CU with two groups finishes last by a factor.
  constexpr size_t need = 2 * (size_t)(TileShape<AK, 64 * FM>::FLOATS + TileShape<BKM, 64 * FN>::FLOATS) * sizeof(float);
  constexpr size_t lds = need > 84 * 1024 ? need : 84 * 1024;
  static bool allowed = false;  // more than 64 KiB of LDS has to be asked for, once per kernel
  if (!allowed && lds > 65536) {
    ENDIA_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sgemm_lone_kernel<AK, BKM, EPI, FM, FN, DEPTH>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed = true;
  }
  hipLaunchKernelGGL((sgemm_lone_kernel<AK, BKM, EPI, FM, FN, DEPTH>), grid, dim3(NTHREADS), lds, s, p);
  return ENDIA_HIP_OK;
}

template <int EPI, int FM, int FN, int DEPTH>
int32_t launch_lone_form(const GemmArgs& p, int transA, int transB, dim3 grid, hipStream_t s) {
  const bool ak = !transA, bk = transB != 0;
  if (ak && bk) return launch_lone_one<true, true, EPI, FM, FN, DEPTH>(p, grid, s);
  if (ak && !bk) return launch_lone_one<true, false, EPI, FM, FN, DEPTH>(p, grid, s);
  if (!ak && bk) return launch_lone_one<false, true, EPI, FM, FN, DEPTH>(p, grid, s);
  return launch_lone_one<false, false, EPI, FM, FN, DEPTH>(p, grid, s);
}

template <int FM, int FN, int DEPTH>
int32_t launch_lone(const GemmArgs& p, int epi, int transA, int transB, dim3 grid, hipStream_t s) {
  switch (epi) {
    case ENDIA_EPI_NONE: return launch_lone_form<ENDIA_EPI_NONE, FM, FN, DEPTH>(p, transA, transB, grid, s);
    case ENDIA_EPI_BIAS: return launch_lone_form<ENDIA_EPI_BIAS, FM, FN, DEPTH>(p, transA, transB, grid, s);
    case ENDIA_EPI_BIAS_ACT: return launch_lone_form<ENDIA_EPI_BIAS_ACT, FM, FN, DEPTH>(p, transA, transB, grid, s);
    default: return launch_lone_form<ENDIA_EPI_ACT_GRAD, FM, FN, DEPTH>(p, transA, transB, grid, s);
  }
}

}  // namespace endia_gemm
