// Fused optimizer steps. The reference builds each update from ~3 (SGD, endia/optim/sgd.mojo:61-62)
// or ~14 (Adam, endia/optim/adam.mojo:47-65) separate full-tensor Array ops with temporaries and a raw
// copy back into the parameter (endia/_array/_array.mojo:998-1006). Here each is ONE pass: SGD moves
// 12 bytes per parameter (read p, g; write p), Adam 28 (read p, g, m, v; write p, m, v).
//
// Every intermediate of the reference is an fp32 Array, so each arithmetic step rounds to fp32. The
// kernels keep that: floating-point contraction is switched off for this file, so no product-sum
// pair is fused into an fma and the results equal the reference's op-by-op arithmetic bit for bit.
#include "common.h"

#include <math.h>

#pragma clang fp contract(off)

namespace {

constexpr int TPB = 256;

struct AdamK {
  float lr, b1, b2, eps, omb1, omb2, c1, c2;  // c1 = 1 - b1^t, c2 = 1 - b2^t
};

// Plain operators, not the __f*_rn helpers: those are inline functions of a header compiled with
// contraction allowed, and would carry that permission into this file after inlining.
__device__ __forceinline__ void adam_one(float& p, float g, float& m, float& v, const AdamK& k) {
  float a = k.b1 * m, b = k.omb1 * g;
  m = a + b;
  float c = k.b2 * v, e = k.omb2 * g;
  e = e * g;
  v = c + e;
  float mh = m / k.c1;
  float vh = v / k.c2;
  // the reference's real sqrt is sqrt((|x|+x)/2) (sqrt_op.mojo:111-114): equal to sqrt(x) for x >= 0
  float r = (fabsf(vh) + vh) * 0.5f;
  float den = __builtin_sqrtf(r) + k.eps;
  float num = k.lr * mh;
  p = p - num / den;
}

__device__ __forceinline__ float sgd_one(float p, float g, float lr) {
  float u = lr * g;
  return p - u;
}

__global__ __launch_bounds__(TPB) void adam_kernel(int64_t n, float* __restrict__ p, const float* __restrict__ g,
                                                   float* __restrict__ m, float* __restrict__ v, AdamK k, int vec) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  if (vec) {
    int64_t n4 = n >> 2;
    float4* p4 = reinterpret_cast<float4*>(p);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    float4* m4 = reinterpret_cast<float4*>(m);
    float4* v4 = reinterpret_cast<float4*>(v);
    for (int64_t j = i; j < n4; j += stride) {
      float4 P = p4[j], G = g4[j], M = m4[j], V = v4[j];
      adam_one(P.x, G.x, M.x, V.x, k);
      adam_one(P.y, G.y, M.y, V.y, k);
      adam_one(P.z, G.z, M.z, V.z, k);
      adam_one(P.w, G.w, M.w, V.w, k);
      p4[j] = P; m4[j] = M; v4[j] = V;
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) adam_one(p[j], g[j], m[j], v[j], k);
  } else {
    for (int64_t j = i; j < n; j += stride) adam_one(p[j], g[j], m[j], v[j], k);
  }
}

__global__ __launch_bounds__(TPB) void sgd_kernel(int64_t n, float* __restrict__ p, const float* __restrict__ g, float lr,
                                                  int vec) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  if (vec) {
    int64_t n4 = n >> 2;
    float4* p4 = reinterpret_cast<float4*>(p);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    for (int64_t j = i; j < n4; j += stride) {
      float4 P = p4[j], G = g4[j];
      P.x = sgd_one(P.x, G.x, lr);
      P.y = sgd_one(P.y, G.y, lr);
      P.z = sgd_one(P.z, G.z, lr);
      P.w = sgd_one(P.w, G.w, lr);
      p4[j] = P;
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) p[j] = sgd_one(p[j], g[j], lr);
  } else {
    for (int64_t j = i; j < n; j += stride) p[j] = sgd_one(p[j], g[j], lr);
  }
}

// Plain SGD over several parameter tensors in one launch (blockIdx.y picks the tensor). A model of many
// small tensors is bound by launch latency, not bandwidth: the reference's sine-fit MLP has 16 of them.
constexpr int MULTI_MAX = 32;
struct SgdMulti {
  float* p[MULTI_MAX];
  const float* g[MULTI_MAX];
  int64_t n[MULTI_MAX];
};

__global__ __launch_bounds__(TPB) void sgd_multi_kernel(SgdMulti t, float lr) {
  const int k = blockIdx.y;
  float* __restrict__ p = t.p[k];
  const float* __restrict__ g = t.g[k];
  const int64_t n = t.n[k];
  const int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) p[j] = sgd_one(p[j], g[j], lr);
}

// Adam over several tensors with the step counter in device memory: nothing that changes from step to step is a
// kernel argument, so the launch can be recorded into a HIP graph and replayed. Every group computes the two bias
// corrections from *t itself (two powf per group).
struct AdamMulti {
  float* p[MULTI_MAX];
  const float* g[MULTI_MAX];
  float* m[MULTI_MAX];
  float* v[MULTI_MAX];
  int64_t n[MULTI_MAX];
};

__global__ __launch_bounds__(TPB) void adam_multi_kernel(AdamMulti t, AdamK k, const float* __restrict__ step) {
  const int i = blockIdx.y;
  const float ts = step[0];
  k.c1 = 1.0f - powf(k.b1, ts);
  k.c2 = 1.0f - powf(k.b2, ts);
  float* __restrict__ p = t.p[i];
  const float* __restrict__ g = t.g[i];
  float* __restrict__ m = t.m[i];
  float* __restrict__ v = t.v[i];
  const int64_t n = t.n[i];
  const int64_t stride = (int64_t)gridDim.x * TPB;
  for (int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x; j < n; j += stride) adam_one(p[j], g[j], m[j], v[j], k);
}

__global__ void counter_add_kernel(float* __restrict__ c, float delta) {
  if (threadIdx.x == 0 && blockIdx.x == 0) c[0] = c[0] + delta;
}

// kind: 0 = SGD with momentum / weight decay, 1 = Adagrad, 2 = RMSprop. `s` is the state tensor (velocity or cache).
struct OptK {
  int kind;
  float lr, a, b, eps;  // SGD: a = momentum, b = weight decay; RMSprop: a = alpha, b = 1 - alpha
};

__device__ __forceinline__ void opt_one(float& p, float g, float& s, const OptK& k, bool has_state) {
  if (k.kind == 0) {
    float c = g;
    if (k.b > 0.f) { float w = k.b * p; c = g + w; }
    float d = k.lr * c;
    if (k.a > 0.f && has_state) {
      float m = k.a * s;
      s = m - d;
      p = p + s;
    } else {
      p = p - d;
    }
  } else {
    float gg;
    if (k.kind == 1) {
      gg = g * g;
      s = s + gg;
    } else {
      float x = k.a * s, y = k.b * g;
      y = y * g;
      s = x + y;
    }
    float r = (fabsf(s) + s) * 0.5f;  // the reference's real sqrt, sqrt_op.mojo:111-114
    float den = __builtin_sqrtf(r) + k.eps;
    float num = k.lr * g;
    p = p - num / den;
  }
}

__global__ __launch_bounds__(TPB) void opt_kernel(int64_t n, float* __restrict__ p, const float* __restrict__ g,
                                                  float* __restrict__ s, OptK k, int vec) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * TPB;
  const bool hs = s != nullptr;
  if (vec) {
    int64_t n4 = n >> 2;
    float4* p4 = reinterpret_cast<float4*>(p);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    float4* s4 = reinterpret_cast<float4*>(s);
    for (int64_t j = i; j < n4; j += stride) {
      float4 P = p4[j], G = g4[j], S = hs ? s4[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      opt_one(P.x, G.x, S.x, k, hs);
      opt_one(P.y, G.y, S.y, k, hs);
      opt_one(P.z, G.z, S.z, k, hs);
      opt_one(P.w, G.w, S.w, k, hs);
      p4[j] = P;
      if (hs) s4[j] = S;
    }
    for (int64_t j = (n4 << 2) + i; j < n; j += stride) {
      float S = hs ? s[j] : 0.f;
      opt_one(p[j], g[j], S, k, hs);
      if (hs) s[j] = S;
    }
  } else {
    for (int64_t j = i; j < n; j += stride) {
      float S = hs ? s[j] : 0.f;
      opt_one(p[j], g[j], S, k, hs);
      if (hs) s[j] = S;
    }
  }
}

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

inline int stream_grid(int64_t nvec) {
  int64_t blocks = ceil_div64(nvec, TPB);
  int64_t cap = (int64_t)endia::ctx().cu_count * 8;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

}  // namespace

using namespace endia;

extern "C" {

int32_t endia_hip_sgd_step(int64_t n, float* p, const float* g, float lr) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_sgd_step: negative n");
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(p && g, "endia_hip_sgd_step: null pointer");
  int vec = al16(p) && al16(g);
  hipLaunchKernelGGL(sgd_kernel, dim3(stream_grid(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, ctx().stream, n, p, g, lr, vec);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_sgd_step_multi(int32_t count, const int64_t* n, float* const* p, const float* const* g, float lr) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(count >= 0, "endia_hip_sgd_step_multi: negative count");
  if (count == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(n && p && g, "endia_hip_sgd_step_multi: null table");
  for (int32_t first = 0; first < count; first += MULTI_MAX) {
    const int32_t m = count - first < MULTI_MAX ? count - first : MULTI_MAX;
    SgdMulti t = {};
    int64_t largest = 0;
    for (int32_t i = 0; i < m; ++i) {
      ENDIA_CHECK_ARG(n[first + i] >= 0, "endia_hip_sgd_step_multi: tensor %d has a negative size", first + i);
      ENDIA_CHECK_ARG(n[first + i] == 0 || (p[first + i] && g[first + i]), "endia_hip_sgd_step_multi: tensor %d has a null pointer",
                      first + i);
      t.p[i] = p[first + i];
      t.g[i] = g[first + i];
      t.n[i] = n[first + i];
      if (t.n[i] > largest) largest = t.n[i];
    }
    if (largest == 0) continue;
    hipLaunchKernelGGL(sgd_multi_kernel, dim3((unsigned)stream_grid(largest), (unsigned)m), dim3(TPB), 0, ctx().stream, t, lr);
    ENDIA_LAUNCH_CHECK();
  }
  return ENDIA_HIP_OK;
}

int32_t endia_hip_adam_step_multi(int32_t count, const int64_t* n, float* const* p, const float* const* g, float* const* m,
                                  float* const* v, float lr, float beta1, float beta2, float eps, float* step) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(count >= 0, "endia_hip_adam_step_multi: negative count");
  ENDIA_CHECK_ARG(step != nullptr, "endia_hip_adam_step_multi: the step counter is null");
  if (count == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(n && p && g && m && v, "endia_hip_adam_step_multi: null table");
  AdamK k;
  k.lr = lr; k.b1 = beta1; k.b2 = beta2; k.eps = eps;
  k.omb1 = 1.0f - beta1;
  k.omb2 = 1.0f - beta2;
  k.c1 = k.c2 = 1.f;  // set on the device from the counter
  for (int32_t first = 0; first < count; first += MULTI_MAX) {
    const int32_t cnt = count - first < MULTI_MAX ? count - first : MULTI_MAX;
    AdamMulti t = {};
    int64_t largest = 0;
    for (int32_t i = 0; i < cnt; ++i) {
      const int32_t j = first + i;
      ENDIA_CHECK_ARG(n[j] >= 0, "endia_hip_adam_step_multi: tensor %d has a negative size", j);
      ENDIA_CHECK_ARG(n[j] == 0 || (p[j] && g[j] && m[j] && v[j]), "endia_hip_adam_step_multi: tensor %d has a null pointer", j);
      t.p[i] = p[j]; t.g[i] = g[j]; t.m[i] = m[j]; t.v[i] = v[j]; t.n[i] = n[j];
      if (t.n[i] > largest) largest = t.n[i];
    }
    if (largest == 0) continue;
    hipLaunchKernelGGL(adam_multi_kernel, dim3((unsigned)stream_grid(largest), (unsigned)cnt), dim3(TPB), 0, ctx().stream, t, k, step);
    ENDIA_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(counter_add_kernel, dim3(1), dim3(64), 0, ctx().stream, step, 1.0f);  // t + 1 after all parameters (adam.mojo:65)
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

static int32_t launch_opt(const char* who, int64_t n, float* p, const float* g, float* s, const OptK& k, bool need_state) {
  ENDIA_REQUIRE_INIT();
  if (n < 0) return fail(ENDIA_HIP_ERR_INVALID, "%s: negative n", who);
  if (n == 0) return ENDIA_HIP_OK;
  if (!p || !g || (need_state && !s)) return fail(ENDIA_HIP_ERR_INVALID, "%s: null pointer", who);
  int vec = al16(p) && al16(g) && (!s || al16(s));
  hipLaunchKernelGGL(opt_kernel, dim3(stream_grid(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, ctx().stream, n, p, g, s, k, vec);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_sgd_momentum_step(int64_t n, float* p, const float* g, float* vel, float lr, float momentum,
                                    float weight_decay) {
  ENDIA_CHECK_ARG(momentum >= 0.f && weight_decay >= 0.f, "endia_hip_sgd_momentum_step: negative momentum or weight decay");
  OptK k;
  k.kind = 0; k.lr = lr; k.a = momentum; k.b = weight_decay; k.eps = 0.f;
  return launch_opt("endia_hip_sgd_momentum_step", n, p, g, momentum > 0.f ? vel : nullptr, k, momentum > 0.f);
}

int32_t endia_hip_adagrad_step(int64_t n, float* p, const float* g, float* cache, float lr, float eps) {
  OptK k;
  k.kind = 1; k.lr = lr; k.a = 0.f; k.b = 0.f; k.eps = eps;
  return launch_opt("endia_hip_adagrad_step", n, p, g, cache, k, true);
}

int32_t endia_hip_rmsprop_step(int64_t n, float* p, const float* g, float* cache, float lr, float alpha, float eps) {
  OptK k;
  k.kind = 2; k.lr = lr; k.a = alpha; k.b = 1.0f - alpha; k.eps = eps;
  return launch_opt("endia_hip_rmsprop_step", n, p, g, cache, k, true);
}

int32_t endia_hip_adam_step(int64_t n, float* p, const float* g, float* m, float* v, float lr, float beta1, float beta2,
                            float eps, float t) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(n >= 0, "endia_hip_adam_step: negative n");
  ENDIA_CHECK_ARG(t >= 1.0f, "endia_hip_adam_step: step counter t = %g must start at 1", (double)t);
  if (n == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(p && g && m && v, "endia_hip_adam_step: null pointer");
  AdamK k;
  k.lr = lr; k.b1 = beta1; k.b2 = beta2; k.eps = eps;
  k.omb1 = 1.0f - beta1;
  k.omb2 = 1.0f - beta2;
  k.c1 = 1.0f - powf(beta1, t);
  k.c2 = 1.0f - powf(beta2, t);
  int vec = al16(p) && al16(g) && al16(m) && al16(v);
  hipLaunchKernelGGL(adam_kernel, dim3(stream_grid(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, ctx().stream, n, p, g, m, v, k,
                     vec);
  ENDIA_LAUNCH_CHECK();
  return ENDIA_HIP_OK;
}

}  // extern "C"
