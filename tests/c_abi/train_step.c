/* A client of libendia_hip.so written in plain C: one training step of a two-layer tanh MLP
 * (forward with fused epilogues, fused MSE, backward with the activation-gradient epilogue, bias
 * gradients, multi-tensor SGD) driven through include/endia_hip.h only, checked against the same
 * step computed here in double precision. It shows that the header is a C header and that the
 * boundary needs nothing but pointers and sizes. Exit status 0 = every tensor within 1e-4 relative. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "endia_hip.h"

#define B 64
#define D0 16
#define D1 32
#define D2 8

#define CHECK(call)                                                              \
  do {                                                                           \
    int32_t rc_ = (call);                                                        \
    if (rc_ != ENDIA_HIP_OK) {                                                   \
      fprintf(stderr, "%s -> %d: %s\n", #call, (int)rc_, endia_hip_last_error()); \
      return 2;                                                                  \
    }                                                                            \
  } while (0)

static unsigned long long lcg = 88172645463325252ULL;
static float rnd(void) { /* uniform in (-1, 1) */
  lcg = lcg * 6364136223846793005ULL + 1442695040888963407ULL;
  return (float)((double)(lcg >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

static float* upload(const float* h, size_t n) {
  void* d = NULL;
  if (endia_hip_malloc((int64_t)(n * sizeof(float)), &d) != ENDIA_HIP_OK) return NULL;
  if (endia_hip_memcpy_h2d(d, h, (int64_t)(n * sizeof(float))) != ENDIA_HIP_OK) return NULL;
  return (float*)d;
}

static float* device(size_t n) {
  void* d = NULL;
  return endia_hip_malloc((int64_t)(n * sizeof(float)), &d) == ENDIA_HIP_OK ? (float*)d : NULL;
}

static double rel_err(const float* got, const double* want, size_t n) {
  double num = 0.0, den = 0.0;
  size_t i;
  for (i = 0; i < n; ++i) {
    num += ((double)got[i] - want[i]) * ((double)got[i] - want[i]);
    den += want[i] * want[i];
  }
  return sqrt(num / (den > 0.0 ? den : 1.0));
}

int main(void) {
  static float x[B * D0], W1[D0 * D1], b1[D1], W2[D1 * D2], b2[D2], y[B * D2];
  static double a1[B * D1], dp[B * D2], dz1[B * D1], gW1[D0 * D1], gb1[D1], gW2[D1 * D2], gb2[D2];
  static double nW1[D0 * D1], nb1[D1], nW2[D1 * D2], nb2[D2];
  static float out[D0 * D1 + D1 * D2];
  const float lr = 0.05f;
  double loss = 0.0, worst = 0.0, e;
  float loss_gpu = 0.f;
  int i, j, k;

  for (i = 0; i < B * D0; ++i) x[i] = rnd();
  for (i = 0; i < D0 * D1; ++i) W1[i] = 0.4f * rnd();
  for (i = 0; i < D1; ++i) b1[i] = 0.1f * rnd();
  for (i = 0; i < D1 * D2; ++i) W2[i] = 0.3f * rnd();
  for (i = 0; i < D2; ++i) b2[i] = 0.1f * rnd();
  for (i = 0; i < B * D2; ++i) y[i] = rnd();

  /* ---- the step in double precision ---- */
  for (i = 0; i < B; ++i)
    for (j = 0; j < D1; ++j) {
      double z = b1[j];
      for (k = 0; k < D0; ++k) z += (double)x[i * D0 + k] * W1[k * D1 + j];
      a1[i * D1 + j] = tanh(z);
    }
  for (i = 0; i < B; ++i)
    for (j = 0; j < D2; ++j) {
      double z = b2[j];
      for (k = 0; k < D1; ++k) z += a1[i * D1 + k] * W2[k * D2 + j];
      loss += (z - y[i * D2 + j]) * (z - y[i * D2 + j]);
      dp[i * D2 + j] = 2.0 * (z - y[i * D2 + j]) / (B * D2);
    }
  loss /= B * D2;
  memset(gW2, 0, sizeof gW2); memset(gb2, 0, sizeof gb2); memset(gW1, 0, sizeof gW1); memset(gb1, 0, sizeof gb1);
  for (i = 0; i < B; ++i)
    for (j = 0; j < D2; ++j) {
      gb2[j] += dp[i * D2 + j];
      for (k = 0; k < D1; ++k) gW2[k * D2 + j] += a1[i * D1 + k] * dp[i * D2 + j];
    }
  for (i = 0; i < B; ++i)
    for (k = 0; k < D1; ++k) {
      double g = 0.0;
      for (j = 0; j < D2; ++j) g += dp[i * D2 + j] * W2[k * D2 + j];
      dz1[i * D1 + k] = g * (1.0 - a1[i * D1 + k] * a1[i * D1 + k]);
      gb1[k] += dz1[i * D1 + k];
    }
  for (i = 0; i < B; ++i)
    for (k = 0; k < D0; ++k)
      for (j = 0; j < D1; ++j) gW1[k * D1 + j] += (double)x[i * D0 + k] * dz1[i * D1 + j];
  for (i = 0; i < D0 * D1; ++i) nW1[i] = W1[i] - lr * gW1[i];
  for (i = 0; i < D1; ++i) nb1[i] = b1[i] - lr * gb1[i];
  for (i = 0; i < D1 * D2; ++i) nW2[i] = W2[i] - lr * gW2[i];
  for (i = 0; i < D2; ++i) nb2[i] = b2[i] - lr * gb2[i];

  /* ---- the same step through the C ABI ---- */
  CHECK(endia_hip_init(0));
  {
    float *dx = upload(x, B * D0), *dW1 = upload(W1, D0 * D1), *db1 = upload(b1, D1), *dW2 = upload(W2, D1 * D2),
          *db2 = upload(b2, D2), *dy = upload(y, B * D2);
    float *da1 = device(B * D1), *dpred = device(B * D2), *dloss = device(1), *ddp = device(B * D2), *ddz1 = device(B * D1);
    float *dgW1 = device(D0 * D1), *dgb1 = device(D1), *dgW2 = device(D1 * D2), *dgb2 = device(D2);
    int64_t shape1[2] = {B, D1}, shape2[2] = {B, D2};
    int64_t sizes[4] = {D0 * D1, D1, D1 * D2, D2};
    float* params[4];
    const float* grads[4];
    if (!dx || !dW1 || !db1 || !dW2 || !db2 || !dy || !da1 || !dpred || !dloss || !ddp || !ddz1 || !dgW1 || !dgb1 || !dgW2 || !dgb2) {
      fprintf(stderr, "allocation failed: %s\n", endia_hip_last_error());
      return 2;
    }
    /* a1 = tanh(x W1 + b1); pred = a1 W2 + b2 */
    CHECK(endia_hip_sgemm(0, 0, B, D1, D0, dx, D0, dW1, D1, da1, D1, 1, 0, 0, 0, ENDIA_EPI_BIAS_ACT, ENDIA_OP_TANH, db1, NULL, NULL));
    CHECK(endia_hip_sgemm(0, 0, B, D2, D1, da1, D1, dW2, D2, dpred, D2, 1, 0, 0, 0, ENDIA_EPI_BIAS, ENDIA_OP_IDENTITY, db2, NULL, NULL));
    CHECK(endia_hip_mse_fwd_bwd(B * D2, dpred, dy, dloss, ddp));
    /* dW2 = a1^T dp; db2 = column sums of dp; dz1 = (dp W2^T) * tanh'(from the stored output a1) */
    CHECK(endia_hip_sgemm(1, 0, D1, D2, B, da1, D1, ddp, D2, dgW2, D2, 1, 0, 0, 0, ENDIA_EPI_NONE, ENDIA_OP_IDENTITY, NULL, NULL, NULL));
    CHECK(endia_hip_reduce_add(2, shape2, 1u, ddp, dgb2, 1.0f, 0));
    CHECK(endia_hip_sgemm(0, 1, B, D1, D2, ddp, D2, dW2, D2, ddz1, D1, 1, 0, 0, 0, ENDIA_EPI_ACT_GRAD,
                          ENDIA_OP_TANH | ENDIA_ACT_FROM_OUTPUT, NULL, da1, NULL));
    CHECK(endia_hip_sgemm(1, 0, D0, D1, B, dx, D0, ddz1, D1, dgW1, D1, 1, 0, 0, 0, ENDIA_EPI_NONE, ENDIA_OP_IDENTITY, NULL, NULL, NULL));
    CHECK(endia_hip_reduce_add(2, shape1, 1u, ddz1, dgb1, 1.0f, 0));
    params[0] = dW1; params[1] = db1; params[2] = dW2; params[3] = db2;
    grads[0] = dgW1; grads[1] = dgb1; grads[2] = dgW2; grads[3] = dgb2;
    CHECK(endia_hip_sgd_step_multi(4, sizes, params, grads, lr));

    CHECK(endia_hip_memcpy_d2h(&loss_gpu, dloss, sizeof(float)));
    e = fabs((double)loss_gpu - loss) / loss; if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, dgW1, sizeof(float) * D0 * D1)); e = rel_err(out, gW1, D0 * D1); if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, dgW2, sizeof(float) * D1 * D2)); e = rel_err(out, gW2, D1 * D2); if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, dW1, sizeof(float) * D0 * D1)); e = rel_err(out, nW1, D0 * D1); if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, db1, sizeof(float) * D1)); e = rel_err(out, nb1, D1); if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, dW2, sizeof(float) * D1 * D2)); e = rel_err(out, nW2, D1 * D2); if (e > worst) worst = e;
    CHECK(endia_hip_memcpy_d2h(out, db2, sizeof(float) * D2)); e = rel_err(out, nb2, D2); if (e > worst) worst = e;
  }
  CHECK(endia_hip_shutdown());
  printf("c client: loss %.6f (double precision %.6f), worst relative error %.2e\n", loss_gpu, loss, worst);
  return worst <= 1e-4 ? 0 : 1;
}
