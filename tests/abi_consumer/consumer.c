/* A C99 caller of the library, with nothing between it and the C ABI: what a cgo, JNI or Rust FFI
 * binding does, written out by hand.  It runs one layer of the reference's forward and backward
 * pass on small operands - gemm (src/ops2/gemm/cpu_stack.rs:16-46), add_row (src/ops2/row_op/cpu.rs),
 * relu (src/matrix.rs:169-190), softmax (src/ops2/softmax/cpu.rs:11-16), Tgemm for the weight gradient
 * (src/ops2/gemm/grad/cpu_stack.rs:24-41), sum_rows for the bias gradient (src/ops2/sum/cpu.rs:66-76),
 * transpose (src/ops2/transpose/cpu.rs:10-25) - and compares every result with plain loops in this
 * file.  Exit status 0 and a last line "PASS" when everything agrees; 2 when the library reports that
 * it has no device to run on (the message of slhip_last_error_string is printed); 1 on a mismatch. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "sliced_hip.h"

#define M 200
#define K 96
#define N 24

static float frand(unsigned* s) {
  *s = *s * 1664525u + 1013904223u;
  return (float)((*s >> 8) & 0xffff) / 65536.0f - 0.5f;
}

#define CHECK(call)                                                                              \
  do {                                                                                           \
    int32_t rc_ = (call);                                                                        \
    if (rc_ != SLHIP_OK) {                                                                       \
      fprintf(stderr, "%s failed (%d): %s\n", #call, (int)rc_, slhip_last_error_string());       \
      return 1;                                                                                  \
    }                                                                                            \
  } while (0)

static int close_enough(const char* what, const float* got, const double* want, size_t n, double tol) {
  size_t i;
  for (i = 0; i < n; ++i) {
    if (fabs((double)got[i] - want[i]) > tol * (1.0 + fabs(want[i]))) {
      fprintf(stderr, "%s: element %lu is %.9g, expected %.9g\n", what, (unsigned long)i, (double)got[i], want[i]);
      return 0;
    }
  }
  printf("%-12s ok (%lu values)\n", what, (unsigned long)n);
  return 1;
}

int main(void) {
  static float x[M * K], w[K * N], b[N], h[M * N], p[M * N], xt[K * M], dw[K * N], db[N];
  static double h_ref[M * N], p_ref[M * N], xt_ref[K * M], dw_ref[K * N], db_ref[N];
  slhip_ctx* ctx = NULL;
  void *dx = NULL, *dwt = NULL, *dbias = NULL, *dh = NULL, *dp = NULL, *dxt = NULL, *ddw = NULL, *ddb = NULL;
  char name[64];
  unsigned seed = 12345u;
  size_t i, j, k;
  int ok = 1;

  if (slhip_init(0, &ctx) != SLHIP_OK) {
    fprintf(stderr, "slhip_init: %s\n", slhip_last_error_string());
    return 2;
  }
  CHECK(slhip_device_name(ctx, name, sizeof name));
  printf("device: %s\n", name);

  for (i = 0; i < M * K; ++i) x[i] = frand(&seed);
  for (i = 0; i < K * N; ++i) w[i] = frand(&seed);
  for (i = 0; i < N; ++i) b[i] = frand(&seed);

  /* the same arithmetic in plain loops, in double */
  for (i = 0; i < M; ++i)
    for (j = 0; j < N; ++j) {
      double s = 0.0;
      for (k = 0; k < K; ++k) s += (double)x[i * K + k] * (double)w[k * N + j];
      s += (double)b[j];
      h_ref[i * N + j] = s >= 0.0 ? s : 0.0;
    }
  for (i = 0; i < M; ++i) {
    double mx = h_ref[i * N], sum = 0.0;
    for (j = 1; j < N; ++j) mx = h_ref[i * N + j] > mx ? h_ref[i * N + j] : mx;
    for (j = 0; j < N; ++j) sum += exp(h_ref[i * N + j] - mx);
    for (j = 0; j < N; ++j) p_ref[i * N + j] = exp(h_ref[i * N + j] - mx) / sum;
  }
  for (i = 0; i < M; ++i)
    for (k = 0; k < K; ++k) xt_ref[k * M + i] = (double)x[i * K + k];
  for (k = 0; k < K; ++k)
    for (j = 0; j < N; ++j) {
      double s = 0.0;
      for (i = 0; i < M; ++i) s += (double)x[i * K + k] * p_ref[i * N + j];
      dw_ref[k * N + j] = s;
    }
  for (j = 0; j < N; ++j) {
    double s = 0.0;
    for (i = 0; i < M; ++i) s += p_ref[i * N + j];
    db_ref[j] = s;
  }

  CHECK(slhip_malloc(ctx, sizeof x, &dx));
  CHECK(slhip_malloc(ctx, sizeof w, &dwt));
  CHECK(slhip_malloc(ctx, sizeof b, &dbias));
  CHECK(slhip_malloc(ctx, sizeof h, &dh));
  CHECK(slhip_malloc(ctx, sizeof p, &dp));
  CHECK(slhip_malloc(ctx, sizeof xt, &dxt));
  CHECK(slhip_malloc(ctx, sizeof dw, &ddw));
  CHECK(slhip_malloc(ctx, sizeof db, &ddb));
  CHECK(slhip_memcpy_h2d(ctx, dx, x, sizeof x));
  CHECK(slhip_memcpy_h2d(ctx, dwt, w, sizeof w));
  CHECK(slhip_memcpy_h2d(ctx, dbias, b, sizeof b));

  /* forward: h = relu(x w + b), p = softmax(h) */
  CHECK(slhip_sgemm(ctx, 0, 0, M, N, K, (const float*)dx, (const float*)dwt, (float*)dh, 0.0f));
  CHECK(slhip_add_row(ctx, M, N, (const float*)dh, (const float*)dbias, (float*)dh));
  CHECK(slhip_ew_unary(ctx, SLHIP_RELU, 0.0f, 0.0f, (size_t)M * N, (const float*)dh, (float*)dh));
  CHECK(slhip_softmax(ctx, M, N, (const float*)dh, (float*)dp));
  /* backward pieces with p standing in for the upstream gradient: dw = x^T p, db = column sums of p */
  CHECK(slhip_sgemm(ctx, 1, 0, K, N, M, (const float*)dx, (const float*)dp, (float*)ddw, 0.0f));
  CHECK(slhip_sum_rows(ctx, M, N, (const float*)dp, (float*)ddb));
  CHECK(slhip_transpose(ctx, M, K, (const float*)dx, (float*)dxt, 0.0f));

  CHECK(slhip_memcpy_d2h(ctx, h, dh, sizeof h));
  CHECK(slhip_memcpy_d2h(ctx, p, dp, sizeof p));
  CHECK(slhip_memcpy_d2h(ctx, dw, ddw, sizeof dw));
  CHECK(slhip_memcpy_d2h(ctx, db, ddb, sizeof db));
  CHECK(slhip_memcpy_d2h(ctx, xt, dxt, sizeof xt));

  ok &= close_enough("linear+relu", h, h_ref, M * N, 2e-5);
  ok &= close_enough("softmax", p, p_ref, M * N, 2e-5);
  ok &= close_enough("Tgemm", dw, dw_ref, K * N, 2e-5);
  ok &= close_enough("sum_rows", db, db_ref, N, 2e-5);
  ok &= close_enough("transpose", xt, xt_ref, K * M, 0.0);

  /* an error is reported, not swallowed: a null operand */
  if (slhip_sgemm(ctx, 0, 0, M, N, K, NULL, (const float*)dwt, (float*)dh, 0.0f) == SLHIP_OK) {
    fprintf(stderr, "a null operand was accepted\n");
    ok = 0;
  } else {
    printf("%-12s ok (%s)\n", "null operand", slhip_last_error_string());
  }

  CHECK(slhip_free(ctx, dx)); CHECK(slhip_free(ctx, dwt)); CHECK(slhip_free(ctx, dbias)); CHECK(slhip_free(ctx, dh));
  CHECK(slhip_free(ctx, dp)); CHECK(slhip_free(ctx, dxt)); CHECK(slhip_free(ctx, ddw)); CHECK(slhip_free(ctx, ddb));
  CHECK(slhip_destroy(ctx));
  puts(ok ? "PASS" : "FAIL");
  return ok ? 0 : 1;
}
