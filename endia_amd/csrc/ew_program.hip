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

namespace {

constexpr int TPB = 256;

struct EwArgs {
  const float* in[ENDIA_EW_MAX_INPUTS];
  float* out[ENDIA_EW_MAX_OUTPUTS];
  int32_t mode[ENDIA_EW_MAX_INPUTS];
  int32_t n_steps;
  int32_t need_col;
  int64_t n;
  int64_t cols;
  endia_hip_ew_step steps[ENDIA_EW_MAX_STEPS];
};

template <int V>
struct Vec {
  float v[V];
};

template <int V>
__device__ __forceinline__ Vec<V> load_vec(const float* p) {
  Vec<V> r;
  if constexpr (V == 4) {
    float4 t = *reinterpret_cast<const float4*>(p);
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
  } else {
    r.v[0] = *p;
  }
  return r;
}

template <int V>
__device__ __forceinline__ void store_vec(float* p, const Vec<V>& r) {
  if constexpr (V == 4) *reinterpret_cast<float4*>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
  else *p = r.v[0];
}

// Evaluate the program for the V consecutive elements starting at `base` (column `col` of their row).
template <int V>
__device__ __forceinline__ void run_program(const EwArgs& a, int64_t base, int64_t col) {
  Vec<V> acc, s0, s1, s2, s3;
#pragma unroll
  for (int e = 0; e < V; ++e) acc.v[e] = s0.v[e] = s1.v[e] = s2.v[e] = s3.v[e] = 0.f;
  for (int t = 0; t < a.n_steps; ++t) {
    const endia_hip_ew_step st = a.steps[t];
    Vec<V> x;
    if (st.kind != ENDIA_EW_UNARY && st.kind != ENDIA_EW_SAVE && st.kind != ENDIA_EW_STORE) {
      if (st.src_kind == ENDIA_EW_SRC_INPUT) {
        const float* p = a.in[st.src_index];
        const int m = a.mode[st.src_index];
        if (m == ENDIA_EW_FULL) x = load_vec<V>(p + base);
        else if (m == ENDIA_EW_ROW_VECTOR) x = load_vec<V>(p + col);
        else {
          float s = *p;
#pragma unroll
          for (int e = 0; e < V; ++e) x.v[e] = s;
        }
      } else if (st.src_kind == ENDIA_EW_SRC_SLOT) {
        x = st.src_index == 0 ? s0 : (st.src_index == 1 ? s1 : (st.src_index == 2 ? s2 : s3));
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) x.v[e] = st.imm;
      }
    }
    switch (st.kind) {
      case ENDIA_EW_LOAD: acc = x; break;
      case ENDIA_EW_UNARY:
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] = endia::unary_real(st.op, acc.v[e]);
        break;
      case ENDIA_EW_BINARY:
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] = endia::bin_real(st.op, acc.v[e], x.v[e]);
        break;
      case ENDIA_EW_RBINARY:
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] = endia::bin_real(st.op, x.v[e], acc.v[e]);
        break;
      case ENDIA_EW_SAVE:
        if (st.src_index == 0) s0 = acc;
        else if (st.src_index == 1) s1 = acc;
        else if (st.src_index == 2) s2 = acc;
        else s3 = acc;
        break;
      default:  // ENDIA_EW_STORE
        store_vec<V>(a.out[st.src_index] + base, acc);
        break;
    }
  }
}

template <int V>
__global__ __launch_bounds__(TPB) void ew_program_kernel(const EwArgs a) {
  const int64_t stride = (int64_t)gridDim.x * TPB;
  const int64_t nvec = a.n / V;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < nvec; j += stride) {
    const int64_t base = j * V;
    run_program<V>(a, base, a.need_col ? base % a.cols : 0);
  }
  if (V > 1) {  // the last n % V elements, one lane each
    const int64_t j = nvec * V + (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (j < a.n) run_program<1>(a, j, a.need_col ? j % a.cols : 0);
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
    if (input_modes[i] == ENDIA_EW_ROW_VECTOR) a.need_col = 1;
    if (input_modes[i] != ENDIA_EW_SCALAR && (reinterpret_cast<uintptr_t>(inputs[i]) & 15)) vec = false;
  }
  for (int i = 0; i < n_outputs; ++i) {
    ENDIA_CHECK_ARG(outputs[i] != nullptr || a.n == 0, "endia_hip_ew_program: output %d is null", i);
    a.out[i] = outputs[i];
    if (reinterpret_cast<uintptr_t>(outputs[i]) & 15) vec = false;
  }
  uint32_t stored = 0;
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
        ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < ENDIA_EW_MAX_SLOTS, "endia_hip_ew_program: step %d reads slot %d", t,
                        st.src_index);
    }
    if (st.kind == ENDIA_EW_SAVE)
      ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < ENDIA_EW_MAX_SLOTS, "endia_hip_ew_program: step %d writes slot %d", t,
                      st.src_index);
    if (st.kind == ENDIA_EW_STORE) {
      ENDIA_CHECK_ARG(st.src_index >= 0 && st.src_index < n_outputs, "endia_hip_ew_program: step %d writes output %d of %d", t,
                      st.src_index, n_outputs);
      stored |= 1u << st.src_index;
    }
    a.steps[t] = st;
  }
  ENDIA_CHECK_ARG(stored == (1u << n_outputs) - 1, "endia_hip_ew_program: not every output is stored");
  if (a.n == 0) return ENDIA_HIP_OK;
  const int64_t work = vec ? (a.n + 3) / 4 : a.n;
  int64_t blocks = ceil_div64(work, TPB);
  int64_t cap = (int64_t)ctx().cu_count * 8;
  if (cap < 256) cap = 2048;
  if (blocks > cap) blocks = cap;
  if (vec) hipLaunchKernelGGL((ew_program_kernel<4>), dim3((unsigned)blocks), dim3(TPB), 0, ctx().stream, a);
  else hipLaunchKernelGGL((ew_program_kernel<1>), dim3((unsigned)blocks), dim3(TPB), 0, ctx().stream, a);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}
