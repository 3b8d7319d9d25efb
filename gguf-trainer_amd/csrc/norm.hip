// RMSNorm forward and backward (srcRmsNormFwd / BwdX / BwdW, src/backend/wgsl.ts:217-303), also
// serving per-head QK-norm as rows = T*H, d = hd (src/backend/webgpu.ts:1085-1088).
//
// A row is handled by LPR lanes of one wavefront (LPR = 16, 32 or 64, the smallest that keeps
// float4 per lane useful), so hd = 64 packs four rows per wavefront instead of idling 48 lanes.
// Backward makes ONE pass over x and g: the row sum S and dx for the row, and per-lane column
// partials of dw = sum_rows g*x*r kept in registers across the rows a workgroup owns. The
// partials are reduced across the workgroup in LDS, written as one row per workgroup and summed
// in workgroup order by a second small kernel: the reference's one-thread-per-column scan
// (wgsl.ts:286-303) without its strided re-reads, and still deterministic.
#include <algorithm>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));

template <int LPR> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

// NJ = float4 chunks per lane: d <= LPR*4*NJ. d % 4 == 0.
template <int LPR, int NJ>
__global__ __launch_bounds__(256) void rmsnorm_fwd_k(int rows, int d, float eps, const float *__restrict__ x,
                                                     const float *__restrict__ w, float *__restrict__ y,
                                                     float *__restrict__ rinv) {
  constexpr int RPW = WAVE / LPR;                // rows per wavefront
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int sub = lane / LPR, li = lane % LPR;
  const int d4 = d / 4;
  v4f wv[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    int c = li + j * LPR;
    wv[j] = c < d4 ? reinterpret_cast<const v4f *>(w)[c] : v4f{0, 0, 0, 0};
  }
  for (int64_t row = ((int64_t)blockIdx.x * 4 + wave) * RPW + sub; row < rows; row += (int64_t)gridDim.x * 4 * RPW) {
    const v4f *xr = reinterpret_cast<const v4f *>(x + row * d);
    v4f xv[NJ];
    float ss = 0;
#pragma unroll
    for (int j = 0; j < NJ; j++) xv[j] = xr[min(li + j * LPR, d4 - 1)];      // all loads first, none conditional
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      if (li + j * LPR >= d4) xv[j] = v4f{0, 0, 0, 0};
      ss += xv[j][0] * xv[j][0] + xv[j][1] * xv[j][1] + xv[j][2] * xv[j][2] + xv[j][3] * xv[j][3];
    }
    ss = group_sum<LPR>(ss);
    float r = 1.0f / sqrtf(ss / (float)d + eps);
    if (li == 0) rinv[row] = r;
    v4f *yr = reinterpret_cast<v4f *>(y + row * d);
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      int c = li + j * LPR;
      if (c < d4) yr[c] = xv[j] * r * wv[j];
    }
  }
}

template <int LPR, int NJ>
__global__ __launch_bounds__(256) void rmsnorm_bwd_k(int rows, int d, const float *__restrict__ x,
                                                     const float *__restrict__ w, const float *__restrict__ g,
                                                     const float *__restrict__ rinv, float *dx, int acc_dx,
                                                     const float *dx_old, float *__restrict__ dw_part) {
  constexpr int RPW = WAVE / LPR;
  constexpr int NG = 4 * RPW;                    // row groups per workgroup
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int sub = lane / LPR, li = lane % LPR;
  const int d4 = d / 4;
  const float invd = 1.0f / (float)d;
  v4f wv[NJ], dwv[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    int c = li + j * LPR;
    wv[j] = c < d4 ? reinterpret_cast<const v4f *>(w)[c] : v4f{0, 0, 0, 0};
    dwv[j] = v4f{0, 0, 0, 0};
  }
  // Two rows of this lane group in flight, and every load of an iteration (x, g and, when accumulating, the old
  // dx) issued before the first use, unconditionally: a chunk past the row end re-reads the row's last chunk and a
  // row past the end re-reads row 0. Their products vanish where it matters (w is zero there, nothing is stored).
  const int64_t rstep = (int64_t)gridDim.x * 4 * RPW;
  int cc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) cc[j] = min(li + j * LPR, d4 - 1);
  for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW + sub; row0 < rows; row0 += 2 * rstep) {
    v4f xv[2][NJ], gv[2][NJ], ov[2][NJ];
    float rr[2];
    float S[2] = {0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int64_t row = row0 + u * rstep;
      const int64_t rl = row < rows ? row : 0;
      const v4f *xr = reinterpret_cast<const v4f *>(x + rl * d);
      const v4f *gr = reinterpret_cast<const v4f *>(g + rl * d);
      const v4f *dr = reinterpret_cast<const v4f *>(dx_old + rl * d);     // what dx is added to (dx itself, or another buffer)
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        xv[u][j] = xr[cc[j]];
        gv[u][j] = gr[cc[j]];
        if (acc_dx) ov[u][j] = dr[cc[j]];
      }
      rr[u] = rinv[rl];
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        v4f t = gv[u][j] * wv[j] * xv[u][j];
        S[u] += t[0] + t[1] + t[2] + t[3];
      }
      S[u] = group_sum<LPR>(S[u]);
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int64_t row = row0 + u * rstep;
      if (row >= rows) continue;
      const float r = rr[u];
      const float k2 = r * r * r * S[u] * invd;
      v4f *dxr = reinterpret_cast<v4f *>(dx + row * d);
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        int c = li + j * LPR;
        v4f o = wv[j] * gv[u][j] * r - xv[u][j] * k2;
        if (acc_dx) o += ov[u][j];
        if (c < d4) dxr[c] = o;
        dwv[j] += gv[u][j] * xv[u][j] * r;
      }
    }
  }
  if (!dw_part) return;
  // workgroup reduction of the NG row groups' column partials, fixed order
  extern __shared__ float sm[];                  // [NG][d]
  const int grp = wave * RPW + sub;
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    int c = li + j * LPR;
    if (c < d4) reinterpret_cast<v4f *>(sm + (size_t)grp * d)[c] = dwv[j];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < d; c += 256) {
    float s = 0;
#pragma unroll
    for (int q = 0; q < NG; q++) s += sm[(size_t)q * d + c];
    dw_part[(size_t)blockIdx.x * d + c] = s;
  }
}

// dw[c] (+)= sum over the nparts partial rows, in a fixed order: 16 columns per workgroup (one 64-byte line per
// load), sixteen lane groups each summing every sixteenth partial row with eight independent loads in flight, then
// the group sums added in group order. Narrow workgroups because the launch is latency-bound: d = 576 gives 36 of them.
#define CS_COLS 16
#define CS_GRPS 16
__device__ __forceinline__ void colsum_body(const float *__restrict__ part, int nparts, int d, float *dw, int acc, int blk) {
  __shared__ float sm[CS_GRPS][CS_COLS];
  const int cl = threadIdx.x % CS_COLS, grp = threadIdx.x / CS_COLS;
  const int c = blk * CS_COLS + cl;
  const int cr = min(c, d - 1);
  float s = 0;
  int p = grp;
  for (; p + 7 * CS_GRPS < nparts; p += 8 * CS_GRPS) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = part[(size_t)(p + CS_GRPS * u) * d + cr];
#pragma unroll
    for (int u = 0; u < 8; u++) s += v[u];
  }
  for (; p < nparts; p += CS_GRPS) s += part[(size_t)p * d + cr];
  sm[grp][cl] = s;
  __syncthreads();
  if (grp == 0 && c < d) {
    float t = sm[0][cl];
#pragma unroll
    for (int q = 1; q < CS_GRPS; q++) t += sm[q][cl];
    dw[c] = acc ? dw[c] + t : t;
  }
}
__global__ __launch_bounds__(256) void colsum_reduce(const float *__restrict__ part, int nparts, int d, float *dw, int acc) {
  colsum_body(part, nparts, d, dw, acc, blockIdx.x);
}
// The column sums of several normalisations' partials in one launch (the dw of every norm a backward pass went through,
// summed when somebody is about to read them instead of once per norm): workgroup -> (entry, 16-column block) through the
// table in the kernel arguments, then colsum_reduce's arithmetic, so each dw has the bits its own launch would give it.
#define CSG_MAX 96
struct CsEntry { const float *part; float *dw; int nparts, d, acc, blk0; };
struct CsGroup { CsEntry e[CSG_MAX]; int n; };
__global__ __launch_bounds__(256) void colsum_group_k(CsGroup G) {
  int i = 0;
  for (int q = 1; q < G.n; q++) if ((int)blockIdx.x >= G.e[q].blk0) i = q;
  const CsEntry &e = G.e[i];
  colsum_body(e.part, e.nparts, e.d, e.dw, e.acc, (int)blockIdx.x - e.blk0);
}

// scalar fallback for d % 4 != 0 or very wide rows: one wavefront per row
__global__ __launch_bounds__(256) void rmsnorm_fwd_gen(int rows, int d, float eps, const float *__restrict__ x,
                                                       const float *__restrict__ w, float *__restrict__ y,
                                                       float *__restrict__ rinv) {
  const int lane = threadIdx.x % WAVE;
  int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (row >= rows) return;
  const float *xr = x + row * d;
  float ss = 0;
  for (int j = lane; j < d; j += WAVE) ss += xr[j] * xr[j];
  ss = wave_sum(ss);
  float r = 1.0f / sqrtf(ss / (float)d + eps);
  if (lane == 0) rinv[row] = r;
  for (int j = lane; j < d; j += WAVE) y[row * d + j] = xr[j] * r * w[j];
}
__global__ __launch_bounds__(256) void rmsnorm_bwd_gen(int rows, int d, const float *__restrict__ x,
                                                       const float *__restrict__ w, const float *__restrict__ g,
                                                       const float *__restrict__ rinv, float *dx, int acc_dx,
                                                       const float *dx_old) {
  const int lane = threadIdx.x % WAVE;
  int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (row >= rows) return;
  const float *xr = x + row * d, *gr = g + row * d;
  float S = 0;
  for (int j = lane; j < d; j += WAVE) S += gr[j] * w[j] * xr[j];
  S = wave_sum(S);
  float r = rinv[row], k2 = r * r * r * S / (float)d;
  for (int j = lane; j < d; j += WAVE) {
    float o = w[j] * r * gr[j] - xr[j] * k2;
    dx[row * d + j] = acc_dx ? dx_old[row * d + j] + o : o;
  }
}
// dw for the fallback: one thread per column over a slab of rows, partials per slab
__global__ __launch_bounds__(256) void rmsnorm_dw_gen(int rows, int d, int slab, const float *__restrict__ x,
                                                      const float *__restrict__ g, const float *__restrict__ rinv,
                                                      float *__restrict__ part) {
  int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= d) return;
  int64_t r0 = (int64_t)blockIdx.y * slab, r1 = std::min<int64_t>(rows, r0 + slab);
  float s = 0;
  for (int64_t r = r0; r < r1; r++) s += g[r * d + c] * x[r * d + c] * rinv[r];
  part[(size_t)blockIdx.y * d + c] = s;
}

// Scratch of gt_rmsnorm_bwd_static, the entry point that allocates nothing: the per-workgroup dw partial rows, at most
// two workgroups per CU of up to RMS_STATIC_MAX_D columns. Every GPU the library runs on holds its own copy until the
// process ends. In host code the name is only a handle for hipGetSymbolAddress; kernels get the address it returns.
#define RMS_STATIC_MAX_D 2048
#define RMS_STATIC_FLOATS (512 * RMS_STATIC_MAX_D)          // 4 MiB
static __device__ __align__(256) float scratch[RMS_STATIC_FLOATS];

// The array is one per device and every context on the device shares it. The last context that queued a static call on
// each device is remembered: a call from another context while that one's stream has not been waited for since would race
// on the partials and is refused.
#define RMS_STATIC_MAX_DEV 64
static gt_ctx *g_static_last[RMS_STATIC_MAX_DEV];

void rmsnorm_static_forget(gt_ctx *ctx) {
  if (ctx->device >= 0 && ctx->device < RMS_STATIC_MAX_DEV && g_static_last[ctx->device] == ctx) g_static_last[ctx->device] = nullptr;
}

int rmsnorm_static_init(gt_ctx *ctx) {
  void *ptr = nullptr;
  GT_HIP(ctx, hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));      // this device's copy: the context's device is current
  GT_REQUIRE(ctx, ptr != nullptr, "hipGetSymbolAddress gave a null address for the static scratch array");
  ctx->rms_static = static_cast<float *>(ptr);
  return 0;
}

template <int LPR, int NJ>
static int launch_fast(gt_ctx *ctx, bool bwd, int rows, int d, float eps, gt_buf x, gt_buf w, gt_buf y_or_g, gt_buf rinv,
                       gt_buf dx, int acc_dx, gt_buf dx_old, gt_buf dw, int acc_dw, float *static_part = nullptr, bool defer = false) {
  constexpr int RPB = 4 * (WAVE / LPR);
  int64_t nb = std::min<int64_t>(cdiv(rows, RPB), (int64_t)ctx->num_cu * 2);
  if (!bwd) {
    hipLaunchKernelGGL((rmsnorm_fwd_k<LPR, NJ>), dim3((unsigned)nb), dim3(256), 0, ctx->stream, rows, d, eps,
                       P<const float>(x), P<const float>(w), P<float>(y_or_g), P<float>(rinv));
    GT_LAUNCHED(ctx);
    return 0;
  }
  float *part = nullptr;
  if (defer) part = static_part;                 // the caller's buffer of nb x d floats; it sums the columns later
  else if (dw && static_part) {
    GT_REQUIRE(ctx, (size_t)nb * d <= RMS_STATIC_FLOATS, "rmsnorm backward: %lld partial rows of %d columns exceed the static scratch",
               (long long)nb, d);
    part = static_part;
  } else if (dw) {
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)nb * d * sizeof(float), &ws)) return 1;
    part = static_cast<float *>(ws);
  }
  size_t smem = dw ? (size_t)RPB * d * sizeof(float) : 0;
  hipLaunchKernelGGL((rmsnorm_bwd_k<LPR, NJ>), dim3((unsigned)nb), dim3(256), smem, ctx->stream, rows, d,
                     P<const float>(x), P<const float>(w), P<const float>(y_or_g), P<const float>(rinv), P<float>(dx),
                     acc_dx, P<const float>(dx_old), part);
  GT_LAUNCHED(ctx);
  if (dw && !defer) {
    hipLaunchKernelGGL(colsum_reduce, dim3((unsigned)cdiv(d, CS_COLS)), dim3(256), 0, ctx->stream, part, (int)nb, d,
                       P<float>(dw), acc_dw);
    GT_LAUNCHED(ctx);
  }
  return 0;
}
// partial rows the fast backward kernel writes for (rows, d): one per workgroup
static int fast_parts_rows(gt_ctx *ctx, int rows, int d) {
  const int d4 = d / 4;
  const int lpr = d4 <= 16 ? 16 : d4 <= 32 ? 32 : 64;
  return (int)std::min<int64_t>(cdiv(rows, 4 * (WAVE / lpr)), (int64_t)ctx->num_cu * 2);
}

static int dispatch(gt_ctx *ctx, bool bwd, int rows, int d, float eps, gt_buf x, gt_buf w, gt_buf y_or_g, gt_buf rinv,
                    gt_buf dx, int acc_dx, gt_buf dx_old, gt_buf dw, int acc_dw, float *static_part = nullptr, bool defer = false) {
  bool aligned = (x | w | y_or_g | dx | dx_old) % 16 == 0;
  int d4 = d / 4;
#define FAST(LPR, NJ) return launch_fast<LPR, NJ>(ctx, bwd, rows, d, eps, x, w, y_or_g, rinv, dx, acc_dx, dx_old, dw, acc_dw, static_part, defer)
  if (d % 4 == 0 && aligned && d <= RMS_STATIC_MAX_D) {
    if (d4 <= 16) FAST(16, 1);
    if (d4 <= 32) FAST(32, 1);
    if (d4 <= 64) FAST(64, 1);
    if (d4 <= 128) FAST(64, 2);
    if (d4 <= 192) FAST(64, 3);
    if (d4 <= 256) FAST(64, 4);
    FAST(64, 8);
  }
#undef FAST
  GT_REQUIRE(ctx, !static_part, "%s: d = %d must be a multiple of 4, at most %d, and every operand 16-byte aligned",
             defer ? "gt_rmsnorm_bwd_parts" : "gt_rmsnorm_bwd_static", d, RMS_STATIC_MAX_D);
  unsigned nb = (unsigned)cdiv(rows, 4);
  if (!bwd) {
    hipLaunchKernelGGL(rmsnorm_fwd_gen, dim3(nb), dim3(256), 0, ctx->stream, rows, d, eps, P<const float>(x),
                       P<const float>(w), P<float>(y_or_g), P<float>(rinv));
    GT_LAUNCHED(ctx);
    return 0;
  }
  hipLaunchKernelGGL(rmsnorm_bwd_gen, dim3(nb), dim3(256), 0, ctx->stream, rows, d, P<const float>(x), P<const float>(w),
                     P<const float>(y_or_g), P<const float>(rinv), P<float>(dx), acc_dx, P<const float>(dx_old));
  GT_LAUNCHED(ctx);
  if (dw) {
    int slab = 256, ns = (int)cdiv(rows, slab);
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)ns * d * sizeof(float), &ws)) return 1;
    hipLaunchKernelGGL(rmsnorm_dw_gen, dim3((unsigned)cdiv(d, 256), ns), dim3(256), 0, ctx->stream, rows, d, slab,
                       P<const float>(x), P<const float>(y_or_g), P<const float>(rinv), static_cast<float *>(ws));
    GT_LAUNCHED(ctx);
    hipLaunchKernelGGL(colsum_reduce, dim3((unsigned)cdiv(d, CS_COLS)), dim3(256), 0, ctx->stream, static_cast<float *>(ws), ns,
                       d, P<float>(dw), acc_dw);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

extern "C" {
int gt_rmsnorm_fwd(gt_ctx *ctx, int rows, int d, float eps, gt_buf x, gt_buf w, gt_buf y, gt_buf rinv) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && x && w && y && rinv, "gt_rmsnorm_fwd: bad arguments (rows %d, d %d)", rows, d);
  if (rows == 0) return 0;
  ProfScope ps(ctx, "rmsnorm", 8.0 * rows * d);
  return dispatch(ctx, false, rows, d, eps, x, w, y, rinv, 0, 0, 0, 0, 0);
}
int gt_rmsnorm_bwd(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx, int acc_dx,
                   gt_buf dw, int acc_dw) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && x && w && g && rinv && dx, "gt_rmsnorm_bwd: bad arguments (rows %d, d %d)", rows, d);
  if (rows == 0) {
    if (dw && !acc_dw) GT_HIP(ctx, hipMemsetAsync(P<void>(dw), 0, (size_t)d * 4, ctx->stream));
    return 0;
  }
  ProfScope ps(ctx, "rmsnorm.bwd", 12.0 * rows * d);   // read x, g; write dx
  return dispatch(ctx, true, rows, d, 0.f, x, w, g, rinv, dx, acc_dx, dx, dw, acc_dw);
}
__global__ __launch_bounds__(256) void fill_zero_k(int n, float *p) {
  int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}
// gt_rmsnorm_bwd for callers that cannot allocate: the same kernels with the dw partials in the static array above.
// No hipMalloc, no workspace growth, no profiling events, no memset node (a fill kernel clears dw for rows = 0).
int gt_rmsnorm_bwd_static(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx, int acc_dx,
                          gt_buf dw, int acc_dw) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && x && w && g && rinv && dx, "gt_rmsnorm_bwd_static: bad arguments (rows %d, d %d)", rows, d);
  GT_REQUIRE(ctx, d <= RMS_STATIC_MAX_D, "gt_rmsnorm_bwd_static: d = %d is more than the static scratch is sized for (%d)", d, RMS_STATIC_MAX_D);
  GT_REQUIRE(ctx, ctx->rms_static, "gt_rmsnorm_bwd_static: the static scratch array has no device address");
  GT_REQUIRE(ctx, ctx->device < RMS_STATIC_MAX_DEV, "gt_rmsnorm_bwd_static: device %d is beyond the %d this entry point keeps track of", ctx->device, RMS_STATIC_MAX_DEV);
  gt_ctx *last = g_static_last[ctx->device];
  GT_REQUIRE(ctx, !dw || !last || last == ctx || !last->rms_static_pending,
             "gt_rmsnorm_bwd_static: another context's call on this device is still queued and shares the scratch array; gt_sync that context first");
  if (rows == 0) {
    if (dw && !acc_dw) {
      hipLaunchKernelGGL(fill_zero_k, dim3((unsigned)cdiv(d, 256)), dim3(256), 0, ctx->stream, d, P<float>(dw));
      GT_LAUNCHED(ctx);
    }
    return 0;
  }
  if (dw) { g_static_last[ctx->device] = ctx; ctx->rms_static_pending = true; }      // without dw the array is not touched
  return dispatch(ctx, true, rows, d, 0.f, x, w, g, rinv, dx, acc_dx, dx, dw, acc_dw, ctx->rms_static);
}
int gt_rmsnorm_parts_rows(gt_ctx *ctx, int rows, int d, int *nparts) {
  if (!ctx || !nparts) return 1;
  *nparts = (rows >= 1 && d >= 4 && d % 4 == 0 && d <= RMS_STATIC_MAX_D) ? fast_parts_rows(ctx, rows, d) : 0;
  return 0;
}
int gt_rmsnorm_bwd_parts(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx_old, gt_buf dx, int acc_dx,
                         gt_buf parts) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && d >= 4 && d % 4 == 0 && d <= RMS_STATIC_MAX_D && x && w && g && rinv && dx && dx_old && parts && parts % 16 == 0,
             "gt_rmsnorm_bwd_parts: bad arguments (rows %d, d %d: rows >= 1, d a multiple of 4 up to %d)", rows, d, RMS_STATIC_MAX_D);
  ProfScope ps(ctx, "rmsnorm.bwd", 12.0 * rows * d);
  return dispatch(ctx, true, rows, d, 0.f, x, w, g, rinv, dx, acc_dx, dx_old, parts, 0, P<float>(parts), true);
}
int gt_colsum_group(gt_ctx *ctx, int n, const gt_buf *parts, const int *nparts, const int *d, const gt_buf *dw, const int *acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && (n == 0 || (parts && nparts && d && dw && acc)), "gt_colsum_group: %d entries or a null table", n);
  for (int i0 = 0; i0 < n; i0 += CSG_MAX) {
    CsGroup G;
    memset(&G, 0, sizeof G);
    G.n = std::min(CSG_MAX, n - i0);
    int blocks = 0;
    for (int q = 0; q < G.n; q++) {
      const int i = i0 + q;
      GT_REQUIRE(ctx, parts[i] && dw[i] && nparts[i] >= 1 && d[i] >= 1, "gt_colsum_group: entry %d is malformed", i);
      for (int j = i0; j < i; j++) GT_REQUIRE(ctx, dw[j] != dw[i], "gt_colsum_group: entries %d and %d write the same sums", j, i);
      G.e[q] = {P<const float>(parts[i]), P<float>(dw[i]), nparts[i], d[i], acc[i], blocks};
      blocks += (int)cdiv(d[i], CS_COLS);
    }
    ProfScope ps(ctx, "rmsnorm.colsum");
    hipLaunchKernelGGL(colsum_group_k, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, G);
    GT_LAUNCHED(ctx);
  }
  return 0;
}
int gt_rmsnorm_bwd_from(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx_old, gt_buf dx,
                        gt_buf dw, int acc_dw) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && x && w && g && rinv && dx && dx_old, "gt_rmsnorm_bwd_from: bad arguments (rows %d, d %d)", rows, d);
  if (rows == 0) {
    if (dw && !acc_dw) GT_HIP(ctx, hipMemsetAsync(P<void>(dw), 0, (size_t)d * 4, ctx->stream));
    return 0;
  }
  ProfScope ps(ctx, "rmsnorm.bwd", 12.0 * rows * d);
  return dispatch(ctx, true, rows, d, 0.f, x, w, g, rinv, dx, 1, dx_old, dw, acc_dw);
}
}
