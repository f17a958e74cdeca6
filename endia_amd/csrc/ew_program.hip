// Fused elementwise programs: a run of unary / binary elementwise ops evaluated in ONE pass over
// memory. The reference fuses runs of unary ops on one array into a single SIMD loop
// (simd_op_list + execute_fwds, endia/_array/_array.mojo:90-101,756-782) and hands larger
// elementwise subgraphs to its JIT (FxSubgraph, endia/compile/fx.mojo:105-159). Here the run is a
// short program for an accumulator machine that every lane interprets on its own 4 elements:
//
//   acc            the running value
//   slot[0..3]     saved intermediate values (for subexpressions that are used more than once or
//                  that are the left operand of a non-leaf right operand)
//   inputs         up to 8 arrays: full [rows*cols], a row vector [cols] broadcast over rows, or a
//                  one-element array broadcast everywhere
//   outputs        up to 4 full arrays
//
// The program is wave-uniform (it lives in the kernel arguments), so interpreting it costs scalar
// branches only; the per-element work is the ops themselves and the kernel stays HBM-bound:
// algorithmic traffic 4 bytes per element per full input and per output.
#include "common.h"
#include "ew_ops.h"

#include <string.h>

namespace {

constexpr int TPB = 256;

struct EwArgs {
  const float* in[ENDIA_EW_MAX_INPUTS];
  float* out[ENDIA_EW_MAX_OUTPUTS];
  int32_t mode[ENDIA_EW_MAX_INPUTS];
  int32_t n_steps;
  int32_t need_col;
  int64_t begin;  // first element this launch handles
  int64_t n;      // one past the last
  int64_t cols;
  uint2 steps[ENDIA_EW_MAX_STEPS];  // x = kind | op << 8 | src_kind << 16 | src_index << 24, y = bits of imm
};

// The values one lane holds for one register of the machine: C chunks of W consecutive elements.
// Tiled kernel: C = 4, W = 4 (chunk c of a lane starts 256 elements after chunk c-1, so that the
// 64 lanes of a wave read 1 KiB of consecutive addresses per chunk). Tail kernel: C = W = 1.
template <int C, int W>
struct Reg {
  float v[C * W];
};

template <int C, int W>
__device__ __forceinline__ Reg<C, W> splat(float s) {
  Reg<C, W> r;
#pragma unroll
  for (int e = 0; e < C * W; ++e) r.v[e] = s;
  return r;
}

// p points at this lane's first element of chunk 0
template <int C, int W>
__device__ __forceinline__ Reg<C, W> load_full(const float* p) {
  Reg<C, W> r;
  if constexpr (W == 4) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
      float4 t = *reinterpret_cast<const float4*>(p + c * 256);
      r.v[4 * c] = t.x; r.v[4 * c + 1] = t.y; r.v[4 * c + 2] = t.z; r.v[4 * c + 3] = t.w;
    }
  } else {
    r.v[0] = *p;
  }
  return r;
}

template <int C, int W>
__device__ __forceinline__ Reg<C, W> load_row(const float* p, const int (&col)[C]) {
  Reg<C, W> r;
  if constexpr (W == 4) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
      float4 t = *reinterpret_cast<const float4*>(p + col[c]);
      r.v[4 * c] = t.x; r.v[4 * c + 1] = t.y; r.v[4 * c + 2] = t.z; r.v[4 * c + 3] = t.w;
    }
  } else {
    r.v[0] = p[col[0]];
  }
  return r;
}

template <int C, int W>
__device__ __forceinline__ void store_full(float* p, const Reg<C, W>& r) {
  if constexpr (W == 4) {
#pragma unroll
    for (int c = 0; c < C; ++c)
      *reinterpret_cast<float4*>(p + c * 256) = make_float4(r.v[4 * c], r.v[4 * c + 1], r.v[4 * c + 2], r.v[4 * c + 3]);
  } else {
    *p = r.v[0];
  }
}

#define ENDIA_EW_UNARY_CASE(OP)                                                                    \
  case OP:                                                                                         \
    _Pragma("unroll") for (int e = 0; e < C * W; ++e) acc.v[e] = endia::unary_real(OP, acc.v[e]);  \
    break;
#define ENDIA_EW_BINARY_CASE(OP)                                                                       \
  case OP:                                                                                             \
    if (kind == ENDIA_EW_BINARY) {                                                                     \
      _Pragma("unroll") for (int e = 0; e < C * W; ++e) acc.v[e] = endia::bin_real(OP, acc.v[e], x.v[e]); \
    } else {                                                                                           \
      _Pragma("unroll") for (int e = 0; e < C * W; ++e) acc.v[e] = endia::bin_real(OP, x.v[e], acc.v[e]); \
    }                                                                                                  \
    break;

// Interpret the program for the elements of one lane: `base` is the lane's first element of chunk 0,
// col[c] the column of the first element of chunk c (used by row-vector inputs only). The step
// decode and dispatch are scalar work shared by the C * W elements of the lane, which is what the
// wide tile is for: with 4 elements per lane the dispatch alone costs more than the memory time.
// Only the accumulator is carried from step to step in registers; the four save slots live in LDS
// (`slots`, indexed [slot][chunk][thread]). Carrying them in registers as well makes the compiler
// shuffle the whole 80-register state at every step, which costs more than the op itself.
template <int C, int W, typename SlotT>
__device__ __forceinline__ void run_program(const EwArgs& a, int64_t base, const int (&col)[C],
                                            SlotT (*slots)[C][TPB]) {
  Reg<C, W> acc = splat<C, W>(0.f);
  const int tid = threadIdx.x;
  uint2 next = a.steps[0];
  for (int t = 0; t < a.n_steps; ++t) {
    const uint2 st = next;
    if (t + 1 < a.n_steps) next = a.steps[t + 1];  // the next step's scalar load overlaps this step's work
    const int kind = st.x & 0xff, op = (st.x >> 8) & 0xff, src_kind = (st.x >> 16) & 0xff, src_index = st.x >> 24;
    Reg<C, W> x;
    if (kind == ENDIA_EW_LOAD || kind == ENDIA_EW_BINARY || kind == ENDIA_EW_RBINARY) {
      if (src_kind == ENDIA_EW_SRC_INPUT) {
        const float* p = a.in[src_index];
        const int m = a.mode[src_index];
        if (m == ENDIA_EW_FULL) x = load_full<C, W>(p + base);
        else if (m == ENDIA_EW_ROW_VECTOR) x = load_row<C, W>(p, col);
        else x = splat<C, W>(*p);
      } else if (src_kind == ENDIA_EW_SRC_SLOT) {
#pragma unroll
        for (int c = 0; c < C; ++c) {
          const SlotT v = slots[src_index][c][tid];
          if constexpr (W == 4) { x.v[4 * c] = v.x; x.v[4 * c + 1] = v.y; x.v[4 * c + 2] = v.z; x.v[4 * c + 3] = v.w; }
          else x.v[c] = v;
        }
      } else {
        x = splat<C, W>(__uint_as_float(st.y));
      }
    }
    if (kind == ENDIA_EW_LOAD) {
      acc = x;
    } else if (kind == ENDIA_EW_UNARY) {
      switch (op) {
        ENDIA_EW_UNARY_CASE(ENDIA_OP_RELU) ENDIA_EW_UNARY_CASE(ENDIA_OP_TANH) ENDIA_EW_UNARY_CASE(ENDIA_OP_SIN)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_COS) ENDIA_EW_UNARY_CASE(ENDIA_OP_NEG) ENDIA_EW_UNARY_CASE(ENDIA_OP_SQUARE)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_SQRT) ENDIA_EW_UNARY_CASE(ENDIA_OP_ABS) ENDIA_EW_UNARY_CASE(ENDIA_OP_GREATER0)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_EXP) ENDIA_EW_UNARY_CASE(ENDIA_OP_LOG) ENDIA_EW_UNARY_CASE(ENDIA_OP_SIGMOID)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_SINH) ENDIA_EW_UNARY_CASE(ENDIA_OP_COSH) ENDIA_EW_UNARY_CASE(ENDIA_OP_TAN)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_ASIN) ENDIA_EW_UNARY_CASE(ENDIA_OP_ACOS) ENDIA_EW_UNARY_CASE(ENDIA_OP_ATAN)
        ENDIA_EW_UNARY_CASE(ENDIA_OP_RECIPROCAL) ENDIA_EW_UNARY_CASE(ENDIA_OP_SIGN)
        default: break;  // identity
      }
    } else if (kind == ENDIA_EW_BINARY || kind == ENDIA_EW_RBINARY) {
      switch (op) {
        ENDIA_EW_BINARY_CASE(ENDIA_BIN_ADD) ENDIA_EW_BINARY_CASE(ENDIA_BIN_SUB) ENDIA_EW_BINARY_CASE(ENDIA_BIN_MUL)
        ENDIA_EW_BINARY_CASE(ENDIA_BIN_DIV) ENDIA_EW_BINARY_CASE(ENDIA_BIN_GREATER) ENDIA_EW_BINARY_CASE(ENDIA_BIN_POW)
        ENDIA_EW_BINARY_CASE(ENDIA_BIN_GREATER_EQUAL) ENDIA_EW_BINARY_CASE(ENDIA_BIN_LESS)
        ENDIA_EW_BINARY_CASE(ENDIA_BIN_LESS_EQUAL) ENDIA_EW_BINARY_CASE(ENDIA_BIN_EQUAL)
        ENDIA_EW_BINARY_CASE(ENDIA_BIN_NOT_EQUAL)
        default: break;
      }
    } else if (kind == ENDIA_EW_SAVE) {
#pragma unroll
      for (int c = 0; c < C; ++c) {
        if constexpr (W == 4) slots[src_index][c][tid] = make_float4(acc.v[4 * c], acc.v[4 * c + 1], acc.v[4 * c + 2], acc.v[4 * c + 3]);
        else slots[src_index][c][tid] = acc.v[c];
      }
    } else {  // ENDIA_EW_STORE
      store_full<C, W>(a.out[src_index] + base, acc);
    }
  }
}

// One wave per tile of 256 * C elements, waves striding over the tiles of [begin, n). n - begin is a multiple of the
// tile. C = 4 shares a step's decode among sixteen elements of a lane, which is what an array that fills the chip
// many times over wants; an array of a few million elements has fewer such tiles than the chip has wave slots and is
// bound by the latency of one wave's chain of loads, so it takes C = 2 or 1 and spreads over four times the waves.
template <int C>
__global__ __launch_bounds__(TPB) void ew_program_tiled_kernel(const EwArgs a) {
  // 4 * C KiB per save slot that the program uses (dynamic, so a program without saved values does not
  // pay for them in occupancy)
  extern __shared__ float4 slot_mem[];
  float4 (*slots)[C][TPB] = reinterpret_cast<float4 (*)[C][TPB]>(slot_mem);
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
  const int64_t waves = (int64_t)gridDim.x * (TPB / 64);
  const int64_t tiles = (a.n - a.begin) / (256 * C);
  for (int64_t t = wave; t < tiles; t += waves) {
    const int64_t base = a.begin + t * (256 * C) + lane * 4;
    int col[C];
#pragma unroll
    for (int c = 0; c < C; ++c) col[c] = 0;
    if (a.need_col) {
      const int cols = (int)a.cols;  // the host takes this path only for cols < 2^31
      int c0 = (int)(base % a.cols);
#pragma unroll
      for (int c = 0; c < C; ++c) col[c] = (int)(((unsigned)c0 + 256u * c) % (unsigned)cols);
    }
    run_program<C, 4, float4>(a, base, col, slots);
  }
}

template <int C>
int resident_tiled_groups(size_t lds) {
  int r = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, ew_program_tiled_kernel<C>, TPB, lds) != hipSuccess || r < 1) r = 2;
  return r;
}

// One element per lane over [begin, n): unaligned operands, odd row lengths and the tail of the tiled kernel.
__global__ __launch_bounds__(TPB) void ew_program_scalar_kernel(const EwArgs a) {
  __shared__ float slots[ENDIA_EW_MAX_SLOTS][1][TPB];
  const int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = a.begin + (int64_t)blockIdx.x * TPB + threadIdx.x; j < a.n; j += stride) {
    int col[1] = {0};
    if (a.need_col) col[0] = (int)(j % a.cols);
    run_program<1, 1, float>(a, j, col, slots);
  }
}

}  // namespace

using namespace endia;

extern "C" int32_t endia_hip_ew_program(int64_t rows, int64_t cols, int32_t n_inputs, const float* const* inputs,
                                        const int32_t* input_modes, int32_t n_outputs, float* const* outputs,
                                        int32_t n_steps, const endia_hip_ew_step* steps) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(rows >= 0 && cols >= 0, "endia_hip_ew_program: negative extent");
  ENDIA_CHECK_ARG(n_inputs >= 0 && n_inputs <= ENDIA_EW_MAX_INPUTS, "endia_hip_ew_program: %d inputs, at most %d",
                  n_inputs, ENDIA_EW_MAX_INPUTS);
  ENDIA_CHECK_ARG(n_outputs >= 1 && n_outputs <= ENDIA_EW_MAX_OUTPUTS, "endia_hip_ew_program: %d outputs, need 1..%d",
                  n_outputs, ENDIA_EW_MAX_OUTPUTS);
  ENDIA_CHECK_ARG(n_steps >= 1 && n_steps <= ENDIA_EW_MAX_STEPS, "endia_hip_ew_program: %d steps, need 1..%d", n_steps,
                  ENDIA_EW_MAX_STEPS);
  ENDIA_CHECK_ARG(steps && outputs && (n_inputs == 0 || (inputs && input_modes)), "endia_hip_ew_program: null table");
  EwArgs a = {};
  a.n = rows * cols;
  a.cols = cols;
  a.n_steps = n_steps;
  bool vec = cols % 4 == 0;
  for (int i = 0; i < n_inputs; ++i) {
    ENDIA_CHECK_ARG(input_modes[i] >= ENDIA_EW_FULL && input_modes[i] <= ENDIA_EW_SCALAR,
                    "endia_hip_ew_program: input %d has unknown mode %d", i, input_modes[i]);
    ENDIA_CHECK_ARG(inputs[i] != nullptr || a.n == 0, "endia_hip_ew_program: input %d is null", i);
    a.in[i] = inputs[i];
    a.mode[i] = input_modes[i];
    if (input_modes[i] == ENDIA_EW_ROW_VECTOR) {
      a.need_col = 1;
      if (cols >= (1ll << 31))
        return fail(ENDIA_HIP_ERR_UNSUPPORTED, "endia_hip_ew_program: a row-vector input with 2^31 columns or more");
    }
    if (input_modes[i] != ENDIA_EW_SCALAR && (reinterpret_cast<uintptr_t>(inputs[i]) & 15)) vec = false;
  }
  for (int i = 0; i < n_outputs; ++i) {
    ENDIA_CHECK_ARG(outputs[i] != nullptr || a.n == 0, "endia_hip_ew_program: output %d is null", i);
    a.out[i] = outputs[i];
    if (reinterpret_cast<uintptr_t>(outputs[i]) & 15) vec = false;
  }
  uint32_t stored = 0, saved = 0;
  int n_slots = 0;
  for (int t = 0; t < n_steps; ++t) {
    const endia_hip_ew_step& st = steps[t];
    ENDIA_CHECK_ARG(st.kind >= ENDIA_EW_LOAD && st.kind <= ENDIA_EW_STORE, "endia_hip_ew_program: step %d has unknown kind %d",
                    t, st.kind);
    if (st.kind == ENDIA_EW_UNARY)
      ENDIA_CHECK_ARG(st.op >= 0 && st.op < ENDIA_OP_COUNT, "endia_hip_ew_program: step %d has unknown unary op %d", t, st.op);
    if (st.kind == ENDIA_EW_BINARY || st.kind == ENDIA_EW_RBINARY)
      ENDIA_CHECK_ARG(st.op >= 0 && st.op < ENDIA_BIN_COUNT, "endia_hip_ew_program: step %d has unknown binary op %d", t, st.op);
    if (st.kind == ENDIA_EW_LOAD || st.kind == ENDIA_EW_BINARY || st.kind == ENDIA_EW_RBINARY) {
      ENDIA_CHECK_ARG(st.src_kind >= ENDIA_EW_SRC_INPUT && st.src_kind <= ENDIA_EW_SRC_IMM,
                      "endia_hip_ew_program: step %d has unknown operand kind %d", t, st.src_kind);
      if (st.src_kind == ENDIA_EW_SRC_INPUT)
        ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < n_inputs, "endia_hip_ew_program: step %d reads input %d of %d", t,
                        st.src_index, n_inputs);
      if (st.src_kind == ENDIA_EW_SRC_SLOT)
        ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < ENDIA_EW_MAX_SLOTS && (saved >> st.src_index & 1),
                        "endia_hip_ew_program: step %d reads slot %d, which no earlier step saved", t, st.src_index);
    }
    if (st.kind == ENDIA_EW_SAVE)
      ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < ENDIA_EW_MAX_SLOTS, "endia_hip_ew_program: step %d writes slot %d", t,
                      st.src_index);
    if (st.kind == ENDIA_EW_SAVE) {
      saved |= 1u << st.src_index;
      if (st.src_index + 1 > n_slots) n_slots = st.src_index + 1;
    }
    if (st.kind == ENDIA_EW_STORE) {
      ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < n_outputs, "endia_hip_ew_program: step %d writes output %d of %d", t,
                      st.src_index, n_outputs);
      stored |= 1u << st.src_index;
    }
    uint32_t imm_bits;
    memcpy(&imm_bits, &st.imm, 4);
    a.steps[t] = make_uint2((uint32_t)st.kind | ((uint32_t)st.op << 8) | ((uint32_t)st.src_kind << 16) |
                                ((uint32_t)(st.src_index & 0xff) << 24), imm_bits);
  }
  ENDIA_CHECK_ARG(stored == (1u << n_outputs) - 1, "endia_hip_ew_program: not every output is stored");
  if (a.n == 0) return ENDIA_HIP_OK;
  // A grid-stride kernel wants exactly as many work-groups as fit on the chip at once: one more and
  // the extra groups run as a second round after the first has finished.
  static int resident_scalar = 0, resident_tiled[3][ENDIA_EW_MAX_SLOTS + 1] = {{0}};
  if (resident_scalar == 0) {
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident_scalar, ew_program_scalar_kernel, TPB, 0) != hipSuccess ||
        resident_scalar < 1)
      resident_scalar = 4;
  }
  const int64_t cus = ctx().cu_count > 0 ? ctx().cu_count : 256;
  const int64_t total = a.n;
  vec = vec && cols < (1ll << 31) - 1024;
  // chunks per lane: the most (4, 2, 1) that still gives every wave slot of the chip a tile
  int ci = 2;  // index into {1, 2, 4}
  if (vec) {
    for (; ci > 0; --ci) {
      const size_t lds_c = (size_t)n_slots * (1 << ci) * TPB * sizeof(float4);
      if (resident_tiled[ci][n_slots] == 0)
        resident_tiled[ci][n_slots] = ci == 2 ? resident_tiled_groups<4>(lds_c) : resident_tiled_groups<2>(lds_c);
      if (2 * (total / (256 << ci)) >= cus * resident_tiled[ci][n_slots] * (TPB / 64)) break;
    }
    if (ci == 0 && resident_tiled[0][n_slots] == 0)
      resident_tiled[0][n_slots] = resident_tiled_groups<1>((size_t)n_slots * TPB * sizeof(float4));
  }
  const int chunks = 1 << ci;
  const int64_t tile = 256 * chunks;
  const size_t lds = (size_t)n_slots * chunks * TPB * sizeof(float4);
  const int resident[2] = {resident_scalar, vec ? resident_tiled[ci][n_slots] : 0};
  const int64_t tiled_n = vec ? total / tile * tile : 0;
  if (tiled_n > 0) {
    a.begin = 0;
    a.n = tiled_n;
    int64_t blocks = ceil_div64(tiled_n / tile, TPB / 64);
    if (blocks > cus * resident[1]) blocks = cus * resident[1];
    if (chunks == 4) hipLaunchKernelGGL(ew_program_tiled_kernel<4>, dim3((unsigned)blocks), dim3(TPB), lds, ctx().stream, a);
    else if (chunks == 2) hipLaunchKernelGGL(ew_program_tiled_kernel<2>, dim3((unsigned)blocks), dim3(TPB), lds, ctx().stream, a);
    else hipLaunchKernelGGL(ew_program_tiled_kernel<1>, dim3((unsigned)blocks), dim3(TPB), lds, ctx().stream, a);
  }
  if (tiled_n < total) {
    a.begin = tiled_n;
    a.n = total;
    int64_t blocks = ceil_div64(total - tiled_n, TPB);
    if (blocks > cus * resident[0]) blocks = cus * resident[0];
    hipLaunchKernelGGL(ew_program_scalar_kernel, dim3((unsigned)blocks), dim3(TPB), 0, ctx().stream, a);
  }
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}
