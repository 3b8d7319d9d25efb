/*
 * CPU oracle for the training hot path of felladrin/gguf-trainer.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing shipped may import, link or call this
 * file: it is the checker the HIP kernels are compared with, and the timed
 * "cpu_baseline" leg of the benchmark. It restates, loop for loop, the
 * reference's single-threaded CPU ops (src/model/autograd.ts), its AdamW
 * (src/train/adam.ts) and its Muon / Newton-Schulz (src/train/muon.ts).
 *
 * Arithmetic type. The reference is JavaScript: every scalar local is an IEEE
 * double, every tensor is a Float32Array, so each store into a tensor rounds to
 * f32 and each read widens to double. Every function below keeps exactly that
 * discipline: `double` locals, `float` arrays, and `x[i] = (float)(...)` at the
 * same places the reference assigns into a Float32Array (including the
 * element-by-element `+=` into gradient arrays, which rounds once per add).
 * What can still differ from V8 is libm (exp, log, tanh, pow, cos, sin) in the
 * last ulp of a double, which vanishes in the f32 store except in rare ties.
 *
 * Parity pinning (what each function is checked against, in tests/):
 *   or_ce_*            closed-form rows of tests/gradcheck.ts:321-335 and
 *                      tests/gpu-parity.ts:776-784, all-ignored == 0, torch f64
 *   or_linear/add/mul/silu/gelu/scale/rmsnorm/rmsnorm_heads/embedding/rope/
 *   attention          central finite differences with the reference's recipe
 *                      (tests/gradcheck.ts:100-168) and torch float64 autograd
 *   or_fused_ce_*      equals dense CE of or_linear (tests/gradcheck.ts:854-877)
 *   or_soft_ce_*       finite differences; reduces to hard CE for one-hot q;
 *                      k = 3 float64 closed form sum_j q_j (lse - z[id_j]) with a
 *                      duplicated id, a zero-probability slot, mass < 1
 *   or_linear_bwd_dots or_linear_bwd and a float64 product, ragged shapes,
 *                      non-zero starting gradients, frozen weight
 *   or_adamw_step      torch.optim.AdamW in float64 (same closed form)
 *   or_newton_schulz   SVD closed form (the quintic acts on singular values),
 *                      flip invariance
 *   or_mulberry32      integer recurrence, known first outputs
 *
 * `OR_PAR` marks loops that may run under OpenMP when the library is built
 * with -fopenmp and or_set_threads(n>1) is called (cpu_baseline only). Each
 * such loop writes disjoint outputs per iteration, so results do not depend on
 * the thread count. Gradient loops whose iterations share an accumulator stay
 * serial, as in the reference.
 */
#define _GNU_SOURCE
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
static int g_threads = 1;
void or_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int or_get_threads(void) { return g_threads; }
int or_max_threads(void) { return omp_get_num_procs(); }
#define OR_PAR _Pragma("omp parallel for schedule(static) num_threads(g_threads)")
#else
void or_set_threads(int n) { (void)n; }
int or_get_threads(void) { return 1; }
int or_max_threads(void) { return 1; }
#define OR_PAR
#endif

#define D(x) ((double)(x))

/* ---- seeded inputs: src/model/autograd.ts:61-78 --------------------------- */

/* mulberry32 (autograd.ts:69-78). State is a uint32; returns a double in [0,1). */
double or_mulberry32_next(uint32_t *state) {
  uint32_t a = *state;
  a = a + 0x6d2b79f5u;
  *state = a;
  uint32_t t = (a ^ (a >> 15)) * (1u | a);              /* Math.imul */
  t = (t + ((t ^ (t >> 7)) * (61u | t))) ^ t;
  return (double)((t ^ (t >> 14))) / 4294967296.0;
}

/* Box-Muller (autograd.ts:61-66). */
double or_randn(uint32_t *state) {
  double u = 0, v = 0;
  while (u == 0) u = or_mulberry32_next(state);
  while (v == 0) v = or_mulberry32_next(state);
  return sqrt(-2.0 * log(u)) * cos(2.0 * M_PI * v);
}

/* param()/randTensor(): out[i] = randn * std (autograd.ts:54-58). */
void or_fill_randn(float *out, int64_t n, double std, uint32_t *state) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(or_randn(state) * std);
}

void or_fill_uniform(float *out, int64_t n, double lo, double hi, uint32_t *state) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(lo + (hi - lo) * or_mulberry32_next(state));
}

/* ---- linear: autograd.ts:321-379 ------------------------------------------ */

void or_linear_fwd(const float *x, const float *w, float *out, int T, int in, int outd) {
  OR_PAR
  for (int t = 0; t < T; t++) {
    for (int o = 0; o < outd; o++) {
      double acc = 0;
      const float *xr = x + (size_t)t * in, *wr = w + (size_t)o * in;
      for (int i = 0; i < in; i++) acc += D(xr[i]) * D(wr[i]);
      out[(size_t)t * outd + o] = (float)acc;
    }
  }
}

/* gw may be NULL (frozen weight: autograd.ts:359,372-374). Serial: gw is shared
 * across t, gx across o, and the reference's rounding order is (t, o, i). */
void or_linear_bwd(const float *x, const float *w, const float *gout, float *gx, float *gw,
                   int T, int in, int outd) {
  for (int t = 0; t < T; t++) {
    for (int o = 0; o < outd; o++) {
      double g = gout[(size_t)t * outd + o];
      if (g == 0) continue;
      size_t xb = (size_t)t * in, wb = (size_t)o * in;
      if (gw) {
        for (int i = 0; i < in; i++) {
          gx[xb + i] = (float)(D(gx[xb + i]) + g * D(w[wb + i]));
          gw[wb + i] = (float)(D(gw[wb + i]) + g * D(x[xb + i]));
        }
      } else {
        for (int i = 0; i < in; i++) gx[xb + i] = (float)(D(gx[xb + i]) + g * D(w[wb + i]));
      }
    }
  }
}

/* Same gradients with the per-output f64 dot product the forward uses: one f32
 * rounding per element instead of one per term, every output element owned by
 * one iteration (OpenMP-safe). It is the checker of the whole-model GPU
 * comparisons at real head geometry, where the serial form would take minutes,
 * and the linear backward of the timed CPU baseline. Pinned against
 * or_linear_bwd and a float64 product (tests/test_oracle_torch64.py). */
void or_linear_bwd_dots(const float *x, const float *w, const float *gout, float *gx, float *gw,
                        int T, int in, int outd) {
  /* Each output element sums its terms in ascending o (gx) or ascending t (gw) in
   * a double; the loops are interchanged so that memory is walked along rows. */
  enum { CH = 512 };
  OR_PAR
  for (int t = 0; t < T; t++) {
    const float *gr = gout + (size_t)t * outd;
    for (int i0 = 0; i0 < in; i0 += CH) {
      int n = in - i0 < CH ? in - i0 : CH;
      double acc[CH];
      for (int i = 0; i < n; i++) acc[i] = 0;
      for (int o = 0; o < outd; o++) {
        double g = gr[o];
        const float *wr = w + (size_t)o * in + i0;
        for (int i = 0; i < n; i++) acc[i] += g * D(wr[i]);
      }
      float *gxr = gx + (size_t)t * in + i0;
      for (int i = 0; i < n; i++) gxr[i] = (float)(D(gxr[i]) + acc[i]);
    }
  }
  if (!gw) return;
  OR_PAR
  for (int o = 0; o < outd; o++) {
    for (int i0 = 0; i0 < in; i0 += CH) {
      int n = in - i0 < CH ? in - i0 : CH;
      double acc[CH];
      for (int i = 0; i < n; i++) acc[i] = 0;
      for (int t = 0; t < T; t++) {
        double g = gout[(size_t)t * outd + o];
        const float *xr = x + (size_t)t * in + i0;
        for (int i = 0; i < n; i++) acc[i] += g * D(xr[i]);
      }
      float *gwr = gw + (size_t)o * in + i0;
      for (int i = 0; i < n; i++) gwr[i] = (float)(D(gwr[i]) + acc[i]);
    }
  }
}

/* ---- elementwise: autograd.ts:382-469 ------------------------------------- */

void or_add_fwd(const float *a, const float *b, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(D(a[i]) + D(b[i]));
}
/* ga and gb may alias (add(t,t)): sequential adds, like the reference. */
void or_add_bwd(const float *gout, float *ga, float *gb, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    ga[i] = (float)(D(ga[i]) + D(gout[i]));
    gb[i] = (float)(D(gb[i]) + D(gout[i]));
  }
}
void or_mul_fwd(const float *a, const float *b, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(D(a[i]) * D(b[i]));
}
void or_mul_bwd(const float *a, const float *b, const float *gout, float *ga, float *gb, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    ga[i] = (float)(D(ga[i]) + D(gout[i]) * D(b[i]));
    gb[i] = (float)(D(gb[i]) + D(gout[i]) * D(a[i]));
  }
}
/* silu keeps the sigmoid as an f32 array (autograd.ts:415-419). */
void or_silu_fwd(const float *x, float *out, float *sig, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double s = 1.0 / (1.0 + exp(-D(x[i])));
    sig[i] = (float)s;
    out[i] = (float)(D(x[i]) * s);
  }
}
void or_silu_bwd(const float *x, const float *sig, const float *gout, float *gx, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double s = sig[i];
    gx[i] = (float)(D(gx[i]) + D(gout[i]) * (s + D(x[i]) * s * (1 - s)));
  }
}
#define GELU_K 0.7978845608028654
#define GELU_A 0.044715
void or_gelu_fwd(const float *x, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double v = x[i];
    out[i] = (float)(0.5 * v * (1 + tanh(GELU_K * (v + GELU_A * v * v * v))));
  }
}
void or_gelu_bwd(const float *x, const float *gout, float *gx, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double v = x[i], v2 = v * v;
    double u = GELU_K * (v + GELU_A * v * v2);
    double th = tanh(u);
    double dudx = GELU_K * (1 + 3 * GELU_A * v2);
    double g = 0.5 * (1 + th) + 0.5 * v * (1 - th * th) * dudx;
    gx[i] = (float)(D(gx[i]) + D(gout[i]) * g);
  }
}
void or_scale_fwd(const float *x, float *out, double c, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(D(x[i]) * c);
}
void or_scale_bwd(const float *gout, float *gx, double c, int64_t n) {
  for (int64_t i = 0; i < n; i++) gx[i] = (float)(D(gx[i]) + D(gout[i]) * c);
}

/* ---- rmsNorm / rmsNormHeads: autograd.ts:472-545 --------------------------
 * rmsNormHeads is the same arithmetic with rows = T*H and d = hd, so one pair
 * of functions serves both (the reference's two loops differ only in indexing). */

void or_rmsnorm_fwd(const float *x, const float *w, float *out, float *rinv, int rows, int d, double eps) {
  OR_PAR
  for (int t = 0; t < rows; t++) {
    size_t b = (size_t)t * d;
    double ms = 0;
    for (int j = 0; j < d; j++) ms += D(x[b + j]) * D(x[b + j]);
    ms /= d;
    double r = 1.0 / sqrt(ms + eps);
    rinv[t] = (float)r;
    for (int j = 0; j < d; j++) out[b + j] = (float)(D(x[b + j]) * r * D(w[j]));
  }
}
void or_rmsnorm_bwd(const float *x, const float *w, const float *rinv, const float *gout,
                    float *gx, float *gw, int rows, int d) {
  for (int t = 0; t < rows; t++) {
    size_t b = (size_t)t * d;
    double r = rinv[t];
    double S = 0;
    for (int j = 0; j < d; j++) S += D(gout[b + j]) * D(w[j]) * D(x[b + j]);
    for (int j = 0; j < d; j++) {
      double g = gout[b + j];
      gx[b + j] = (float)(D(gx[b + j]) + (D(w[j]) * r * g - (D(x[b + j]) / d) * r * r * r * S));
      if (gw) gw[j] = (float)(D(gw[j]) + g * D(x[b + j]) * r);
    }
  }
}

/* ---- embedding: autograd.ts:548-573 --------------------------------------- */

void or_embedding_fwd(const float *w, const int32_t *ids, float *out, int T, int d) {
  for (int t = 0; t < T; t++) memcpy(out + (size_t)t * d, w + (size_t)ids[t] * d, sizeof(float) * d);
}
void or_embedding_bwd(const int32_t *ids, const float *gout, float *gw, int T, int d) {
  if (!gw) return;
  for (int t = 0; t < T; t++) {
    size_t src = (size_t)ids[t] * d, dst = (size_t)t * d;
    for (int j = 0; j < d; j++) gw[src + j] = (float)(D(gw[src + j]) + D(gout[dst + j]));
  }
}

/* ---- rope: autograd.ts:579-632 (NeoX pairing j, j+hd/2) -------------------- */

static void rope_tables(float *cs, float *sn, int T, int hd, double base, int pos_offset) {
  int half = hd / 2;
  for (int t = 0; t < T; t++) {
    double pos = t + pos_offset;
    for (int j = 0; j < half; j++) {
      double freq = pow(base, (-2.0 * j) / hd);
      double ang = pos * freq;
      cs[t * half + j] = (float)cos(ang);
      sn[t * half + j] = (float)sin(ang);
    }
  }
}
void or_rope_fwd(const float *x, float *out, int T, int H, int hd, double base, int pos_offset) {
  int half = hd / 2;
  float *cs = malloc(sizeof(float) * T * half), *sn = malloc(sizeof(float) * T * half);
  rope_tables(cs, sn, T, hd, base, pos_offset);
  for (int t = 0; t < T; t++)
    for (int h = 0; h < H; h++) {
      size_t b = (size_t)t * H * hd + (size_t)h * hd;
      for (int j = 0; j < half; j++) {
        double c = cs[t * half + j], s = sn[t * half + j];
        double x0 = x[b + j], x1 = x[b + j + half];
        out[b + j] = (float)(x0 * c - x1 * s);
        out[b + j + half] = (float)(x0 * s + x1 * c);
      }
    }
  free(cs); free(sn);
}
void or_rope_bwd(const float *gout, float *gx, int T, int H, int hd, double base, int pos_offset) {
  int half = hd / 2;
  float *cs = malloc(sizeof(float) * T * half), *sn = malloc(sizeof(float) * T * half);
  rope_tables(cs, sn, T, hd, base, pos_offset);
  for (int t = 0; t < T; t++)
    for (int h = 0; h < H; h++) {
      size_t b = (size_t)t * H * hd + (size_t)h * hd;
      for (int j = 0; j < half; j++) {
        double c = cs[t * half + j], s = sn[t * half + j];
        double g0 = gout[b + j], g1 = gout[b + j + half];
        gx[b + j] = (float)(D(gx[b + j]) + (c * g0 + s * g1));
        gx[b + j + half] = (float)(D(gx[b + j + half]) + (-s * g0 + c * g1));
      }
    }
  free(cs); free(sn);
}

/* ---- attention: autograd.ts:640-729 ----------------------------------------
 * probs is the reference's probs[h][t] ragged table flattened to [Hq][T][T];
 * entries outside [winStart(t), t] are left untouched (callers zero it). */

static inline int win_start(int t, int window) { return (window > 0 && t + 1 > window) ? t + 1 - window : 0; }

void or_attention_fwd(const float *q, const float *k, const float *v, float *out, float *probs,
                      int T, int Hq, int Hkv, int hd, int window) {
  int group = Hq / Hkv;
  double scale = 1.0 / sqrt((double)hd);
  size_t qs = (size_t)Hq * hd, kvs = (size_t)Hkv * hd;
  memset(out, 0, sizeof(float) * T * qs);
  OR_PAR
  for (int h = 0; h < Hq; h++) {
    int kv = h / group;
    for (int t = 0; t < T; t++) {
      int s0 = win_start(t, window);
      float *sc = probs + ((size_t)h * T + t) * T;
      double maxS = -INFINITY;
      size_t qb = (size_t)t * qs + (size_t)h * hd;
      for (int s = s0; s <= t; s++) {
        size_t kb = (size_t)s * kvs + (size_t)kv * hd;
        double dot = 0;
        for (int d = 0; d < hd; d++) dot += D(q[qb + d]) * D(k[kb + d]);
        dot *= scale;
        sc[s] = (float)dot;
        if (dot > maxS) maxS = dot;
      }
      double sum = 0;
      for (int s = s0; s <= t; s++) {
        double e = exp(D(sc[s]) - maxS);
        sc[s] = (float)e;
        sum += e;
      }
      for (int s = s0; s <= t; s++) sc[s] = (float)(D(sc[s]) / sum);
      size_t ob = qb;
      for (int s = s0; s <= t; s++) {
        double p = sc[s];
        size_t vb = (size_t)s * kvs + (size_t)kv * hd;
        for (int d = 0; d < hd; d++) out[ob + d] = (float)(D(out[ob + d]) + p * D(v[vb + d]));
      }
    }
  }
}

/* Serial over h: query heads of one group share gk/gv rows, and the reference's
 * rounding order is (h, t, s, d). */
void or_attention_bwd(const float *q, const float *k, const float *v, const float *probs,
                      const float *gout, float *gq, float *gk, float *gv,
                      int T, int Hq, int Hkv, int hd, int window) {
  int group = Hq / Hkv;
  double scale = 1.0 / sqrt((double)hd);
  size_t qs = (size_t)Hq * hd, kvs = (size_t)Hkv * hd;
  float *dP = malloc(sizeof(float) * T);
  for (int h = 0; h < Hq; h++) {
    int kv = h / group;
    for (int t = 0; t < T; t++) {
      int s0 = win_start(t, window);
      const float *p = probs + ((size_t)h * T + t) * T;
      size_t ob = (size_t)t * qs + (size_t)h * hd, qb = ob;
      for (int s = s0; s <= t; s++) {
        size_t vb = (size_t)s * kvs + (size_t)kv * hd;
        double acc = 0;
        for (int d = 0; d < hd; d++) {
          acc += D(gout[ob + d]) * D(v[vb + d]);
          gv[vb + d] = (float)(D(gv[vb + d]) + D(p[s]) * D(gout[ob + d]));
        }
        dP[s] = (float)acc;
      }
      double dot = 0;
      for (int s = s0; s <= t; s++) dot += D(p[s]) * D(dP[s]);
      for (int s = s0; s <= t; s++) {
        double dscore = D(p[s]) * (D(dP[s]) - dot) * scale;
        size_t kb = (size_t)s * kvs + (size_t)kv * hd;
        for (int d = 0; d < hd; d++) {
          gq[qb + d] = (float)(D(gq[qb + d]) + dscore * D(k[kb + d]));
          gk[kb + d] = (float)(D(gk[kb + d]) + dscore * D(q[qb + d]));
        }
      }
    }
  }
  free(dP);
}

/* Parallel-safe attention backward: the same per-(h,t) arithmetic as or_attention_bwd,
 * with dK/dV accumulated per kv-head in f64 scratch and rounded once (so it differs from
 * the serial form by f32 rounding of the running dK/dV sums only). It is the checker of the
 * GPU comparisons at T = 2048 and of the real-width layer test, where the serial form takes
 * minutes, and the attention backward of the timed CPU baseline. Pinned against float64
 * autograd directly (window 0 and > 0, GQA group 3) and against the serial form. */
void or_attention_bwd_par(const float *q, const float *k, const float *v, const float *probs,
                          const float *gout, float *gq, float *gk, float *gv,
                          int T, int Hq, int Hkv, int hd, int window) {
  int group = Hq / Hkv;
  double scale = 1.0 / sqrt((double)hd);
  size_t qs = (size_t)Hq * hd, kvs = (size_t)Hkv * hd;
  OR_PAR
  for (int kv = 0; kv < Hkv; kv++) {
    double *ak = calloc((size_t)T * hd, sizeof(double)), *av = calloc((size_t)T * hd, sizeof(double));
    double *dP = malloc(sizeof(double) * T);
    for (int h = kv * group; h < (kv + 1) * group; h++) {
      for (int t = 0; t < T; t++) {
        int s0 = win_start(t, window);
        const float *p = probs + ((size_t)h * T + t) * T;
        size_t ob = (size_t)t * qs + (size_t)h * hd, qb = ob;
        for (int s = s0; s <= t; s++) {
          size_t vb = (size_t)s * kvs + (size_t)kv * hd;
          double acc = 0;
          for (int d = 0; d < hd; d++) {
            acc += D(gout[ob + d]) * D(v[vb + d]);
            av[(size_t)s * hd + d] += D(p[s]) * D(gout[ob + d]);
          }
          dP[s] = (float)acc;
        }
        double dot = 0;
        for (int s = s0; s <= t; s++) dot += D(p[s]) * dP[s];
        for (int s = s0; s <= t; s++) {
          double dscore = D(p[s]) * (dP[s] - dot) * scale;
          size_t kb = (size_t)s * kvs + (size_t)kv * hd;
          for (int d = 0; d < hd; d++) {
            gq[qb + d] = (float)(D(gq[qb + d]) + dscore * D(k[kb + d]));
            ak[(size_t)s * hd + d] += dscore * D(q[qb + d]);
          }
        }
      }
    }
    for (int s = 0; s < T; s++)
      for (int d = 0; d < hd; d++) {
        size_t kb = (size_t)s * kvs + (size_t)kv * hd + d;
        gk[kb] = (float)(D(gk[kb]) + ak[(size_t)s * hd + d]);
        gv[kb] = (float)(D(gv[kb]) + av[(size_t)s * hd + d]);
      }
    free(ak); free(av); free(dP);
  }
}

/* ---- crossEntropy: autograd.ts:897-952 ------------------------------------ */

/* kept is the count of targets >= 0 (keptRowsInVocab, autograd.ts:875-894). */
double or_ce_fwd(const float *logits, const int32_t *targets, float *probs, int T, int V, int kept) {
  double total = 0;
  double *rowloss = calloc(T, sizeof(double));
  OR_PAR
  for (int t = 0; t < T; t++) {
    size_t b = (size_t)t * V;
    double maxL = -INFINITY;
    for (int v = 0; v < V; v++) if (D(logits[b + v]) > maxL) maxL = logits[b + v];
    double sum = 0;
    for (int v = 0; v < V; v++) {
      double e = exp(D(logits[b + v]) - maxL);
      probs[b + v] = (float)e;
      sum += e;
    }
    for (int v = 0; v < V; v++) probs[b + v] = (float)(D(probs[b + v]) / sum);
    if (targets[t] >= 0) rowloss[t] = log(sum) + maxL - D(logits[b + targets[t]]);
  }
  for (int t = 0; t < T; t++) if (targets[t] >= 0) total += rowloss[t];
  free(rowloss);
  double denom = kept > 0 ? kept : 1;
  return (double)(float)(total / denom);       /* loss.data[0] is a Float32Array slot */
}
/* seed is loss.grad[0] (an f32). */
void or_ce_bwd(const float *probs, const int32_t *targets, float seed, float *glogits, int T, int V, int kept) {
  double denom = kept > 0 ? kept : 1;
  double scale = D(seed) / denom;
  OR_PAR
  for (int t = 0; t < T; t++) {
    if (targets[t] < 0) continue;
    size_t b = (size_t)t * V;
    for (int v = 0; v < V; v++)
      glogits[b + v] = (float)(D(glogits[b + v]) + scale * (D(probs[b + v]) - (v == targets[t] ? 1 : 0)));
  }
}

/* ---- fusedCrossEntropy: autograd.ts:968-1055 ------------------------------- */

static inline double dotrow(const float *a, const float *b, int n) {
  double acc = 0;
  for (int i = 0; i < n; i++) acc += D(a[i]) * D(b[i]);
  return acc;
}
/* row_max/row_sum are the f32 state arrays the backward reads. */
double or_fused_ce_fwd(const float *hidden, const float *w, const int32_t *targets, int chunk,
                       float *row_max, float *row_sum, int T, int H, int V, int kept) {
  float *tgt = calloc(T, sizeof(float));
  for (int t = 0; t < T; t++) { row_max[t] = -INFINITY; row_sum[t] = 0; }
  for (int v0 = 0; v0 < V; v0 += chunk) {
    int v1 = v0 + chunk < V ? v0 + chunk : V;
    OR_PAR
    for (int t = 0; t < T; t++) {
      const float *hr = hidden + (size_t)t * H;
      double cmax = -INFINITY;
      for (int v = v0; v < v1; v++) { double z = dotrow(hr, w + (size_t)v * H, H); if (z > cmax) cmax = z; }
      double mNew = D(row_max[t]) > cmax ? D(row_max[t]) : cmax;
      double sum = 0;
      for (int v = v0; v < v1; v++) sum += exp(dotrow(hr, w + (size_t)v * H, H) - mNew);
      row_sum[t] = (float)(D(row_sum[t]) * exp(D(row_max[t]) - mNew) + sum);
      row_max[t] = (float)mNew;
      int g = targets[t];
      if (g >= v0 && g < v1) tgt[t] = (float)dotrow(hr, w + (size_t)g * H, H);
    }
  }
  double total = 0;
  for (int t = 0; t < T; t++) {
    if (targets[t] < 0) continue;
    total += log(D(row_sum[t])) + D(row_max[t]) - D(tgt[t]);
  }
  free(tgt);
  double denom = kept > 0 ? kept : 1;
  return (double)(float)(total / denom);
}
void or_fused_ce_bwd(const float *hidden, const float *w, const int32_t *targets, int chunk,
                     const float *row_max, const float *row_sum, float seed,
                     float *ghidden, float *gw, int T, int H, int V, int kept) {
  double denom = kept > 0 ? kept : 1;
  double scale = D(seed) / denom;
  for (int v0 = 0; v0 < V; v0 += chunk) {
    int v1 = v0 + chunk < V ? v0 + chunk : V;
    for (int t = 0; t < T; t++) {
      if (targets[t] < 0) continue;
      const float *hr = hidden + (size_t)t * H;
      for (int v = v0; v < v1; v++) {
        double p = exp(dotrow(hr, w + (size_t)v * H, H) - D(row_max[t])) / D(row_sum[t]);
        double d = scale * (p - (v == targets[t] ? 1 : 0));
        for (int i = 0; i < H; i++) {
          ghidden[(size_t)t * H + i] = (float)(D(ghidden[(size_t)t * H + i]) + d * D(w[(size_t)v * H + i]));
          if (gw) gw[(size_t)v * H + i] = (float)(D(gw[(size_t)v * H + i]) + d * D(hr[i]));
        }
      }
    }
  }
}

/* ---- softCrossEntropy: autograd.ts:1076-1138 -------------------------------
 * teacher_probs is f64 here because the reference takes a number[] (doubles). */
double or_soft_ce_fwd(const float *logits, const int32_t *tids, const double *tprobs, int k,
                      float *probs, float *row_mass, int T, int V, int kept) {
  double total = 0;
  for (int t = 0; t < T; t++) {
    size_t b = (size_t)t * V;
    row_mass[t] = 0;
    double maxL = -INFINITY;
    for (int v = 0; v < V; v++) if (D(logits[b + v]) > maxL) maxL = logits[b + v];
    double sum = 0;
    for (int v = 0; v < V; v++) {
      double e = exp(D(logits[b + v]) - maxL);
      probs[b + v] = (float)e;
      sum += e;
    }
    for (int v = 0; v < V; v++) probs[b + v] = (float)(D(probs[b + v]) / sum);
    if (tids[(size_t)t * k] < 0) continue;
    for (int j = 0; j < k; j++) {
      int id = tids[(size_t)t * k + j];
      double q = tprobs[(size_t)t * k + j];
      if (q == 0) continue;
      total += q * (log(sum) + maxL - D(logits[b + id]));
      row_mass[t] = (float)(D(row_mass[t]) + q);
    }
  }
  double denom = kept > 0 ? kept : 1;
  return (double)(float)(total / denom);
}
void or_soft_ce_bwd(const float *probs, const float *row_mass, const int32_t *tids, const double *tprobs,
                    int k, float seed, float *glogits, int T, int V, int kept) {
  double denom = kept > 0 ? kept : 1;
  double scale = D(seed) / denom;
  for (int t = 0; t < T; t++) {
    if (tids[(size_t)t * k] < 0) continue;
    size_t b = (size_t)t * V;
    for (int v = 0; v < V; v++)
      glogits[b + v] = (float)(D(glogits[b + v]) + scale * D(row_mass[t]) * D(probs[b + v]));
    for (int j = 0; j < k; j++) {
      size_t i = b + tids[(size_t)t * k + j];
      glogits[i] = (float)(D(glogits[i]) - scale * tprobs[(size_t)t * k + j]);
    }
  }
}

/* ---- AdamW: src/train/adam.ts:46-82 ----------------------------------------
 * One call = one step() over the whole parameter list (the clip norm is global).
 * t is the step count AFTER the increment (1 on the first call). Gradients are
 * scaled in place when the clip triggers, as in the reference. */
void or_adamw_step(int n_params, float **p, float **g, float **m, float **v, const int64_t *sizes,
                   double lr, double beta1, double beta2, double eps, double wd, double clip, int t) {
  if (clip > 0) {
    double sq = 0;
    for (int pi = 0; pi < n_params; pi++)
      for (int64_t i = 0; i < sizes[pi]; i++) sq += D(g[pi][i]) * D(g[pi][i]);
    double norm = sqrt(sq);
    if (norm > clip) {
      double sc = clip / (norm + 1e-12);
      for (int pi = 0; pi < n_params; pi++)
        for (int64_t i = 0; i < sizes[pi]; i++) g[pi][i] = (float)(D(g[pi][i]) * sc);
    }
  }
  double bc1 = 1 - pow(beta1, t), bc2 = 1 - pow(beta2, t);
  for (int pi = 0; pi < n_params; pi++) {
    float *pp = p[pi], *gg = g[pi], *mm = m[pi], *vv = v[pi];
    int64_t n = sizes[pi];
    OR_PAR
    for (int64_t i = 0; i < n; i++) {
      double gi = gg[i];
      mm[i] = (float)(beta1 * D(mm[i]) + (1 - beta1) * gi);
      vv[i] = (float)(beta2 * D(vv[i]) + (1 - beta2) * gi * gi);
      double mHat = D(mm[i]) / bc1, vHat = D(vv[i]) / bc2;
      double update = mHat / (sqrt(vHat) + eps);
      if (wd > 0) update += wd * D(pp[i]);
      pp[i] = (float)(D(pp[i]) - lr * update);
    }
  }
}

/* ---- Muon / Newton-Schulz: src/train/muon.ts:69-158 ------------------------ */

static float *ns_transpose(const float *A, int r, int c) {
  float *out = malloc(sizeof(float) * r * c);
  for (int i = 0; i < r; i++) for (int j = 0; j < c; j++) out[(size_t)j * r + i] = A[(size_t)i * c + j];
  return out;
}
/* muon.ts:113-130: C += a*B row-wise, each += rounding to f32. */
static float *ns_matmul(const float *A, int ra, int ca, const float *B, int cb) {
  float *C = calloc((size_t)ra * cb, sizeof(float));
  OR_PAR
  for (int i = 0; i < ra; i++)
    for (int k = 0; k < ca; k++) {
      double a = A[(size_t)i * ca + k];
      if (a == 0) continue;
      const float *br = B + (size_t)k * cb;
      float *cr = C + (size_t)i * cb;
      for (int j = 0; j < cb; j++) cr[j] = (float)(D(cr[j]) + a * D(br[j]));
    }
  return C;
}
#define NS_A 3.4445
#define NS_B (-4.7750)
#define NS_C 2.0315
/* out[m*n] = newtonSchulz(G[m,n]) (muon.ts:137-158). */
void or_newton_schulz(const float *G, float *out, int m, int n, int steps) {
  int flip = m > n;
  int r = flip ? n : m, c = flip ? m : n;
  float *X = flip ? ns_transpose(G, m, n) : memcpy(malloc(sizeof(float) * m * n), G, sizeof(float) * m * n);
  size_t len = (size_t)m * n;
  double s = 0;
  for (size_t i = 0; i < len; i++) s += D(X[i]) * D(X[i]);
  double norm = sqrt(s) + 1e-7;
  for (size_t i = 0; i < len; i++) X[i] = (float)(D(X[i]) / norm);
  for (int it = 0; it < steps; it++) {
    float *Xt = ns_transpose(X, r, c);
    float *A = ns_matmul(X, r, c, Xt, r);
    float *AA = ns_matmul(A, r, r, A, r);
    float *B = malloc(sizeof(float) * r * r);
    for (size_t i = 0; i < (size_t)r * r; i++) B[i] = (float)(NS_B * D(A[i]) + NS_C * D(AA[i]));
    float *BX = ns_matmul(B, r, r, X, c);
    for (size_t i = 0; i < len; i++) X[i] = (float)(NS_A * D(X[i]) + D(BX[i]));
    free(Xt); free(A); free(AA); free(B); free(BX);
  }
  if (flip) { float *R = ns_transpose(X, r, c); memcpy(out, R, sizeof(float) * len); free(R); }
  else memcpy(out, X, sizeof(float) * len);
  free(X);
}
/* One Muon matrix update (muon.ts:69-95): momentum, optional Nesterov, NS, scaled descent. */
void or_muon_update(float *p, const float *g, float *buf, int rows, int cols,
                    double lr, double momentum, int nesterov, int ns_steps) {
  size_t len = (size_t)rows * cols;
  float *update = malloc(sizeof(float) * len), *ortho = malloc(sizeof(float) * len);
  for (size_t k = 0; k < len; k++) buf[k] = (float)(momentum * D(buf[k]) + D(g[k]));
  if (nesterov) for (size_t k = 0; k < len; k++) update[k] = (float)(D(g[k]) + momentum * D(buf[k]));
  else memcpy(update, buf, sizeof(float) * len);
  or_newton_schulz(update, ortho, rows, cols, ns_steps);
  double r = (double)rows / cols;
  double scale = sqrt(r > 1 ? r : 1);
  for (size_t k = 0; k < len; k++) p[k] = (float)(D(p[k]) - lr * D(ortho[k]) * scale);
  free(update); free(ortho);
}
