/* A plain C host of libggufhip.so: no Python, no torch, only include/ggufhip.h. It runs y = x W^T, the two backward
 * products, the product-plus-matrix and sum-of-products calls and one AdamW step on small matrices, checks them against straightforward loops, and prints "ok".
 * Built and run by tests/test_gpu_abi_c.py:  gcc abi_host.c -I include -L <pkg> -lggufhip */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include "ggufhip.h"

#define CHECK(call) do { if ((call) != 0) { fprintf(stderr, "%s failed: %s\n", #call, gt_last_error(ctx)); return 1; } } while (0)

static float frand(unsigned *s) { *s = *s * 1664525u + 1013904223u; return (float)((*s >> 8) & 0xFFFF) / 65536.0f - 0.5f; }

int main(void) {
  gt_ctx *ctx = NULL;
  if (gt_ctx_create(0, &ctx) != 0) { fprintf(stderr, "gt_ctx_create: %s\n", gt_last_error(NULL)); return 2; }
  enum { T = 70, IN = 83, OUT = 75 };
  static float x[T * IN], w[OUT * IN], dy[T * OUT], y[T * OUT], dx[T * IN], dw[OUT * IN];
  unsigned seed = 1;
  for (int i = 0; i < T * IN; i++) x[i] = frand(&seed);
  for (int i = 0; i < OUT * IN; i++) w[i] = frand(&seed);
  for (int i = 0; i < T * OUT; i++) dy[i] = frand(&seed);
  gt_buf bx, bw, bdy, by, bdx, bdw, bm, bv;
  CHECK(gt_alloc(ctx, sizeof x, 0, &bx)); CHECK(gt_alloc(ctx, sizeof w, 0, &bw)); CHECK(gt_alloc(ctx, sizeof dy, 0, &bdy));
  CHECK(gt_alloc(ctx, sizeof y, 0, &by)); CHECK(gt_alloc(ctx, sizeof dx, 0, &bdx)); CHECK(gt_alloc(ctx, sizeof dw, 0, &bdw));
  CHECK(gt_alloc(ctx, sizeof w, 1, &bm)); CHECK(gt_alloc(ctx, sizeof w, 1, &bv));
  CHECK(gt_h2d(ctx, bx, x, sizeof x)); CHECK(gt_h2d(ctx, bw, w, sizeof w)); CHECK(gt_h2d(ctx, bdy, dy, sizeof dy));
  CHECK(gt_gemm(ctx, GT_NT, 0, T, OUT, IN, bx, bw, by));        /* y  = x W^T  */
  CHECK(gt_gemm(ctx, GT_NN, 0, T, IN, OUT, bdy, bw, bdx));      /* dX = dY W   */
  CHECK(gt_gemm(ctx, GT_TN, 0, OUT, IN, T, bdy, bx, bdw));      /* dW = dY^T X */
  CHECK(gt_d2h(ctx, y, by, sizeof y)); CHECK(gt_d2h(ctx, dx, bdx, sizeof dx)); CHECK(gt_d2h(ctx, dw, bdw, sizeof dw));
  double worst = 0;
  for (int t = 0; t < T; t++)
    for (int o = 0; o < OUT; o++) {
      double s = 0;
      for (int k = 0; k < IN; k++) s += (double)x[t * IN + k] * w[o * IN + k];
      worst = fmax(worst, fabs(s - y[t * OUT + o]));
    }
  for (int t = 0; t < T; t++)
    for (int k = 0; k < IN; k++) {
      double s = 0;
      for (int o = 0; o < OUT; o++) s += (double)dy[t * OUT + o] * w[o * IN + k];
      worst = fmax(worst, fabs(s - dx[t * IN + k]));
    }
  for (int o = 0; o < OUT; o++)
    for (int k = 0; k < IN; k++) {
      double s = 0;
      for (int t = 0; t < T; t++) s += (double)dy[t * OUT + o] * x[t * IN + k];
      worst = fmax(worst, fabs(s - dw[o * IN + k]));
    }
  if (worst > 2e-5) { fprintf(stderr, "GEMM mismatch %g\n", worst); return 1; }

  /* product plus matrix, and a sum of two products, each in one call: y + x W^T = 2y and dY W + dY W = 2 dX */
  {
    static float y2[T * OUT], dx2[T * IN];
    const int ks[2] = {OUT, OUT};
    const gt_buf as[2] = {bdy, bdy}, bs[2] = {bw, bw};
    CHECK(gt_gemm_add(ctx, GT_NT, T, OUT, IN, bx, bw, by, by));
    CHECK(gt_gemm_sum(ctx, GT_NN, 0, T, IN, 2, ks, as, bs, bdx));
    CHECK(gt_d2h(ctx, y2, by, sizeof y2)); CHECK(gt_d2h(ctx, dx2, bdx, sizeof dx2));
    for (int i = 0; i < T * OUT; i++) worst = fmax(worst, fabs(2.0 * y[i] - y2[i]));
    for (int i = 0; i < T * IN; i++) worst = fmax(worst, fabs(2.0 * dx[i] - dx2[i]));
    if (worst > 4e-5) { fprintf(stderr, "gemm_add / gemm_sum mismatch %g\n", worst); return 1; }
  }

  /* one AdamW step on w with gradient dw, no clipping, against adam.ts:46-82 in double */
  gt_adamw *opt = NULL;
  int64_t size = OUT * IN;
  const double lr = 1e-2, b1 = 0.9, b2 = 0.95, eps = 1e-8, wd = 0.1;
  CHECK(gt_adamw_create(ctx, 1, &bw, &bdw, &bm, &bv, &size, b1, b2, eps, wd, 0.0, &opt));
  CHECK(gt_adamw_step(ctx, opt, lr, 1 - b1, 1 - b2));
  static float w1[OUT * IN];
  CHECK(gt_d2h(ctx, w1, bw, sizeof w1));
  worst = 0;
  for (int i = 0; i < OUT * IN; i++) {
    double g = dw[i], m = (1 - b1) * g, v = (1 - b2) * g * g;
    double upd = (m / (1 - b1)) / (sqrt(v / (1 - b2)) + eps) + wd * w[i];
    worst = fmax(worst, fabs((w[i] - lr * upd) - w1[i]));
  }
  if (worst > 1e-6) { fprintf(stderr, "AdamW mismatch %g\n", worst); return 1; }
  /* a contract violation is refused with a message, not a crash */
  if (gt_gemm(ctx, 7, 0, T, OUT, IN, bx, bw, by) == 0 || !gt_last_error(ctx)[0]) { fprintf(stderr, "bad kind accepted\n"); return 1; }
  CHECK(gt_adamw_destroy(ctx, opt));
  CHECK(gt_free(ctx, bx)); CHECK(gt_free(ctx, bw)); CHECK(gt_free(ctx, bdy)); CHECK(gt_free(ctx, by));
  CHECK(gt_free(ctx, bdx)); CHECK(gt_free(ctx, bdw)); CHECK(gt_free(ctx, bm)); CHECK(gt_free(ctx, bv));
  printf("ok on %s\n", gt_device_name(ctx));
  return gt_ctx_destroy(ctx);
}
