// Elementwise forward/backward bodies (src/backend/webgpu.ts:905-1078 over srcElementwise,
// src/backend/wgsl.ts:199-209) and the fused gated-activation pair. All are streaming kernels:
// float4 per lane, grid-stride, one owner per output element.
#include <algorithm>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));

#define GELU_K 0.7978845608028654f
#define GELU_A 0.044715f

// full-accuracy expf/tanhf: these kernels wait on HBM, not on the ALU
__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float tanhf_(float u) { return tanhf(u); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoidf_(x); }
__device__ __forceinline__ float silu_d(float x) { float s = sigmoidf_(x); return s + x * s * (1.f - s); }
__device__ __forceinline__ float gelu_f(float v) { return 0.5f * v * (1.f + tanhf_(GELU_K * (v + GELU_A * v * v * v))); }
__device__ __forceinline__ float gelu_d(float v) {
  float v2 = v * v, th = tanhf_(GELU_K * (v + GELU_A * v * v2));
  return 0.5f * (1.f + th) + 0.5f * v * (1.f - th * th) * (GELU_K * (1.f + 3.f * GELU_A * v2));
}

enum { OP_ADD, OP_MUL, OP_SILU, OP_GELU, OP_SCALE, OP_GLU_SILU, OP_GLU_GELU };

// out = f(a, b, c)
template <int OP> __device__ __forceinline__ float fwd1(float a, float b, float c) {
  switch (OP) {
    case OP_ADD: return a + b;
    case OP_MUL: return a * b;
    case OP_SILU: return silu_f(a);
    case OP_GELU: return gelu_f(a);
    case OP_SCALE: return a * c;
    case OP_GLU_SILU: return silu_f(a) * b;
    default: return gelu_f(a) * b;
  }
}
template <int OP, bool HASB>
__global__ __launch_bounds__(256) void ew_fwd(int64_t n, const float *__restrict__ a, const float *__restrict__ b, float c,
                                              float *__restrict__ out) {
  int64_t n4 = n / 4, stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    v4f x = reinterpret_cast<const v4f *>(a)[i], y = {0, 0, 0, 0}, o;
    if (HASB) y = reinterpret_cast<const v4f *>(b)[i];
#pragma unroll
    for (int j = 0; j < 4; j++) o[j] = fwd1<OP>(x[j], y[j], c);
    reinterpret_cast<v4f *>(out)[i] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x < n % 4) {
    int64_t i = n4 * 4 + threadIdx.x;
    out[i] = fwd1<OP>(a[i], HASB ? b[i] : 0.f, c);
  }
}

// Backward: contributions (ga, gb) of one element given upstream g and saved inputs a, b.
template <int OP> __device__ __forceinline__ void bwd1(float g, float a, float b, float c, float &ga, float &gb) {
  switch (OP) {
    case OP_ADD: ga = g; gb = g; break;
    case OP_MUL: ga = g * b; gb = g * a; break;
    case OP_SILU: ga = g * silu_d(a); gb = 0; break;
    case OP_GELU: ga = g * gelu_d(a); gb = 0; break;
    case OP_SCALE: ga = g * c; gb = 0; break;
    case OP_GLU_SILU: ga = g * b * silu_d(a); gb = g * silu_f(a); break;
    default: ga = g * b * gelu_d(a); gb = g * gelu_f(a); break;
  }
}
// NEEDA/NEEDB: the op reads saved inputs a / b. da, db may be null (skipped). When da == db the
// host passes same = 1 and the single destination receives ga + gb.
template <int OP, bool NEEDA, bool NEEDB>
__global__ __launch_bounds__(256) void ew_bwd(int64_t n, const float *__restrict__ g, const float *__restrict__ a,
                                              const float *__restrict__ b, float c, float *da, int acc_a, float *db,
                                              int acc_b, int same) {
  int64_t n4 = n / 4, stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    v4f gg = reinterpret_cast<const v4f *>(g)[i], x = {0, 0, 0, 0}, y = {0, 0, 0, 0}, ra, rb;
    if (NEEDA) x = reinterpret_cast<const v4f *>(a)[i];
    if (NEEDB) y = reinterpret_cast<const v4f *>(b)[i];
#pragma unroll
    for (int j = 0; j < 4; j++) { float ta, tb; bwd1<OP>(gg[j], x[j], y[j], c, ta, tb); ra[j] = ta; rb[j] = tb; }
    if (same) {
      v4f s = ra + rb;
      if (acc_a) s += reinterpret_cast<v4f *>(da)[i];
      reinterpret_cast<v4f *>(da)[i] = s;
    } else {
      if (da) { if (acc_a) ra += reinterpret_cast<v4f *>(da)[i]; reinterpret_cast<v4f *>(da)[i] = ra; }
      if (db) { if (acc_b) rb += reinterpret_cast<v4f *>(db)[i]; reinterpret_cast<v4f *>(db)[i] = rb; }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < n % 4) {
    int64_t i = n4 * 4 + threadIdx.x;
    float ra, rb;
    bwd1<OP>(g[i], NEEDA ? a[i] : 0.f, NEEDB ? b[i] : 0.f, c, ra, rb);
    if (same) da[i] = (acc_a ? da[i] : 0.f) + ra + rb;
    else {
      if (da) da[i] = (acc_a ? da[i] : 0.f) + ra;
      if (db) db[i] = (acc_b ? db[i] : 0.f) + rb;
    }
  }
}

static inline unsigned ew_grid(gt_ctx *ctx, int64_t n) {
  int64_t b = cdiv(cdiv(n, 4), 256);
  int64_t cap = (int64_t)ctx->num_cu * 16;
  return (unsigned)std::max<int64_t>(1, std::min(b, cap));
}

template <int OP, bool HASB>
static int run_fwd(gt_ctx *ctx, const char *label, int64_t n, gt_buf a, gt_buf b, float c, gt_buf out) {
  const double bytes = 4.0 * n * (HASB ? 3 : 2);
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && a && out && (!HASB || b), "%s: null operand", label);
  GT_REQUIRE(ctx, (a | b | out) % 16 == 0, "%s: buffers must be 16-byte aligned", label);
  if (n == 0) return 0;
  ProfScope ps(ctx, label, bytes);
  hipLaunchKernelGGL((ew_fwd<OP, HASB>), dim3(ew_grid(ctx, n)), dim3(256), 0, ctx->stream, n, P<const float>(a),
                     P<const float>(b), c, P<float>(out));
  GT_LAUNCHED(ctx);
  return 0;
}
template <int OP, bool NEEDA, bool NEEDB>
static int run_bwd(gt_ctx *ctx, const char *label, int64_t n, gt_buf g, gt_buf a, gt_buf b, float c, gt_buf da, int acc_a,
                   gt_buf db, int acc_b) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && g && (!NEEDA || a) && (!NEEDB || b), "%s: null operand", label);
  GT_REQUIRE(ctx, (g | a | b | da | db) % 16 == 0, "%s: buffers must be 16-byte aligned", label);
  if (n == 0 || (!da && !db)) return 0;
  int same = (da && da == db) ? 1 : 0;
  // algorithmic bytes: g and the saved inputs read once, each destination written once
  const double bytes = 4.0 * n * (1 + (NEEDA ? 1 : 0) + (NEEDB ? 1 : 0) + (da ? 1 : 0) + ((db && !same) ? 1 : 0));
  ProfScope ps(ctx, label, bytes);
  hipLaunchKernelGGL((ew_bwd<OP, NEEDA, NEEDB>), dim3(ew_grid(ctx, n)), dim3(256), 0, ctx->stream, n, P<const float>(g),
                     P<const float>(a), P<const float>(b), c, P<float>(da), acc_a, P<float>(db), acc_b, same);
  GT_LAUNCHED(ctx);
  return 0;
}

extern "C" {
int gt_add_fwd(gt_ctx *ctx, int64_t n, gt_buf a, gt_buf b, gt_buf out) { return run_fwd<OP_ADD, true>(ctx, "add", n, a, b, 0, out); }
int gt_mul_fwd(gt_ctx *ctx, int64_t n, gt_buf a, gt_buf b, gt_buf out) { return run_fwd<OP_MUL, true>(ctx, "mul", n, a, b, 0, out); }
int gt_silu_fwd(gt_ctx *ctx, int64_t n, gt_buf x, gt_buf out) { return run_fwd<OP_SILU, false>(ctx, "silu", n, x, 0, 0, out); }
int gt_gelu_fwd(gt_ctx *ctx, int64_t n, gt_buf x, gt_buf out) { return run_fwd<OP_GELU, false>(ctx, "gelu", n, x, 0, 0, out); }
int gt_scale_fwd(gt_ctx *ctx, int64_t n, gt_buf x, float c, gt_buf out) { return run_fwd<OP_SCALE, false>(ctx, "scale", n, x, 0, c, out); }
int gt_glu_fwd(gt_ctx *ctx, int act, int64_t n, gt_buf gate, gt_buf up, gt_buf out) {
  return act == 0 ? run_fwd<OP_GLU_SILU, true>(ctx, "glu", n, gate, up, 0, out) : run_fwd<OP_GLU_GELU, true>(ctx, "glu", n, gate, up, 0, out);
}
int gt_add_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf da, int acc_a, gt_buf db, int acc_b) {
  return run_bwd<OP_ADD, false, false>(ctx, "add.bwd", n, g, 0, 0, 0, da, acc_a, db, acc_b);
}
int gt_mul_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf a, gt_buf b, gt_buf da, int acc_a, gt_buf db, int acc_b) {
  return run_bwd<OP_MUL, true, true>(ctx, "mul.bwd", n, g, a, b, 0, da, acc_a, db, acc_b);
}
int gt_silu_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf x, gt_buf dx, int acc) {
  return run_bwd<OP_SILU, true, false>(ctx, "silu.bwd", n, g, x, 0, 0, dx, acc, 0, 0);
}
int gt_gelu_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf x, gt_buf dx, int acc) {
  return run_bwd<OP_GELU, true, false>(ctx, "gelu.bwd", n, g, x, 0, 0, dx, acc, 0, 0);
}
int gt_scale_bwd(gt_ctx *ctx, int64_t n, gt_buf g, float c, gt_buf dx, int acc) {
  return run_bwd<OP_SCALE, false, false>(ctx, "scale.bwd", n, g, 0, 0, c, dx, acc, 0, 0);
}
int gt_glu_bwd(gt_ctx *ctx, int act, int64_t n, gt_buf g, gt_buf gate, gt_buf up, gt_buf dgate, int acc_gate, gt_buf dup,
               int acc_up) {
  return act == 0 ? run_bwd<OP_GLU_SILU, true, true>(ctx, "glu.bwd", n, g, gate, up, 0, dgate, acc_gate, dup, acc_up)
                  : run_bwd<OP_GLU_GELU, true, true>(ctx, "glu.bwd", n, g, gate, up, 0, dgate, acc_gate, dup, acc_up);
}
}
