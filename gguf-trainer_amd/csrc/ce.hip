// Softmax cross-entropy, forward and backward, dense and vocab-chunked, plus the sparse-teacher
// soft variant (srcCeFwd / CeReduce / CeBwd / CeChunkStats / CeLossFromStats / CeChunkGrad /
// SoftCe*, src/backend/wgsl.ts:936-1247; dispatch src/backend/webgpu.ts:1214-1378).
//
// The reference's forward writes the unnormalised exponentials of the whole [T,V] matrix and the
// backward reads them back: 24 B per logit in all. Here the forward keeps only the per-row
// log-sum-exp (one online max/sum pass over the row) and the backward recomputes
// softmax = exp(z - lse) while it writes the gradient: read z once, write dz once, 8 B per logit.
// The loss is log(sum exp(z-m)) + m - z_target, never -log(p_target) (autograd.ts:928-935).
#include <algorithm>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));
#define IGN (-1)

__device__ __forceinline__ void online(float &m, float &l, float z) {
  float mn = fmaxf(m, z);
  l = l * __expf(m - mn) + __expf(z - mn);
  m = mn;
}
__device__ __forceinline__ void merge(float &m, float &l, float m2, float l2) {
  float mn = fmaxf(m, m2);
  float a = (m == -INFINITY) ? 0.f : l * __expf(m - mn);
  float b = (m2 == -INFINITY) ? 0.f : l2 * __expf(m2 - mn);
  m = mn; l = a + b;
}
// (max, sum exp(z-max)) of one row of n values by a workgroup of 256; every thread gets the result
__device__ __forceinline__ void row_stats(const float *__restrict__ zr, int n, float &M, float &L, float *sm) {
  float m = -INFINITY, l = 0;
  const bool vec = ((reinterpret_cast<uintptr_t>(zr) & 15) == 0);
  if (vec) {
    int n4 = n / 4;
    const v4f *z4 = reinterpret_cast<const v4f *>(zr);
    for (int i0 = threadIdx.x; i0 < n4; i0 += 1024) {
      v4f zz[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        int i = i0 + u * 256;
        zz[u] = i < n4 ? __builtin_nontemporal_load(z4 + i) : v4f{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      }
      float mx = m;
#pragma unroll
      for (int u = 0; u < 4; u++) mx = fmaxf(mx, fmaxf(fmaxf(zz[u][0], zz[u][1]), fmaxf(zz[u][2], zz[u][3])));
      float acc = l * __expf(m - mx);
#pragma unroll
      for (int u = 0; u < 4; u++) acc += __expf(zz[u][0] - mx) + __expf(zz[u][1] - mx) + __expf(zz[u][2] - mx) + __expf(zz[u][3] - mx);
      l = (mx == -INFINITY) ? 0.f : acc;
      m = mx;
    }
    for (int i = n4 * 4 + threadIdx.x; i < n; i += 256) online(m, l, zr[i]);
  } else {
    for (int i = threadIdx.x; i < n; i += 256) online(m, l, zr[i]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float m2 = __shfl_xor(m, o, WAVE), l2 = __shfl_xor(l, o, WAVE);
    merge(m, l, m2, l2);
  }
  int w = threadIdx.x / WAVE;
  __syncthreads();
  if (threadIdx.x % WAVE == 0) { sm[w] = m; sm[4 + w] = l; }
  __syncthreads();
  M = sm[0]; L = sm[4];
#pragma unroll
  for (int i = 1; i < 4; i++) merge(M, L, sm[i], sm[4 + i]);
}

// one workgroup per row: lse[row] = M + log(L); nll[row] = lse - z_target (0 when ignored)
__global__ __launch_bounds__(256) void ce_fwd_rows(int V, const float *__restrict__ z, const int *__restrict__ tgt,
                                                   float *__restrict__ lse, float *__restrict__ nll, int *bad) {
  __shared__ float sm[8];
  int64_t row = blockIdx.x;
  const float *zr = z + row * V;
  float M, L;
  row_stats(zr, V, M, L, sm);
  if (threadIdx.x == 0) {
    float ls = M + logf(L);
    lse[row] = ls;
    int g = tgt[row];
    if (g < IGN || g >= V) {                    // no such logit: the row counts as ignored here and the host hears of it
      note_bad_id(bad, GT_BAD_TARGET, row, g, V);
      g = IGN;
    }
    nll[row] = g == IGN ? 0.f : (logf(L) + M - zr[g]);
  }
}
// loss[s] = inv_denom[s] * sum of nll over the T rows of sequence s, fixed-order tree
__global__ __launch_bounds__(256) void ce_seq_loss(int T, const float *__restrict__ nll, const float *__restrict__ inv_denom,
                                                   float *__restrict__ loss) {
  __shared__ float sm[4];
  int s = blockIdx.x;
  float a = 0;
  for (int t = threadIdx.x; t < T; t += 256) a += nll[(size_t)s * T + t];
  a = block_sum<4>(a, sm);
  if (threadIdx.x == 0) loss[s] = a * inv_denom[s];
}

// dz[row, :] (+)= seed*inv_denom[seq] * (exp(z - lse) - onehot). One workgroup per contiguous span of CE_SPAN logits
// of a row, spans of a row numbered fastest: workgroups that run at the same time then work on neighbouring memory,
// which the DRAM pages like much better than 2048 rows streamed side by side. Each thread has four float4 loads in
// flight; z and dz are touched exactly once, so both use streaming (non-temporal) accesses.
// SOFT: the dense half of the sparse-teacher loss, dz (+)= seed*inv_denom * mass[row] * exp(z - lse): no one-hot term (the
// teacher terms are subtracted by soft_ce_bwd_q afterwards), the row's scale carries its teacher mass, tgt holds k ids per
// row and a row is ignored when its first id is -1, inv_denom is one number.
#define CE_SPAN 4096
template <bool SOFT>
__global__ __launch_bounds__(256) void ce_bwd_k(int V, int T, int spans, const float *__restrict__ z,
                                                const int *__restrict__ tgt, const float *__restrict__ inv_denom,
                                                const float *__restrict__ lse, float seed, float *dz, int acc,
                                                const float *__restrict__ mass, int k) {
  const int64_t row = blockIdx.x / spans;
  const int span = blockIdx.x % spans;
  int g = SOFT ? (tgt[row * k] == IGN ? IGN : -2) : tgt[row];     // -2: no column matches
  if (!SOFT && (g < IGN || g >= V)) g = IGN;           // no such logit: ignored, as the forward counted it (and reported it)
  if (g == IGN && acc) return;                         // untouched, as the reference leaves it
  const float sc = SOFT ? seed * mass[row] : seed * inv_denom[row / T];
  const float ls = lse[row];
  const float *zr = z + row * V;
  float *dr = dz + row * V;
  const bool vec = (V % 4 == 0) && (((reinterpret_cast<uintptr_t>(zr) | reinterpret_cast<uintptr_t>(dr)) & 15) == 0);
  if (vec) {
    const int n4 = V / 4;
    const v4f *z4 = reinterpret_cast<const v4f *>(zr);
    v4f *d4 = reinterpret_cast<v4f *>(dr);
    const int i0 = span * (CE_SPAN / 4) + threadIdx.x;
    v4f zz[4], dd[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      int i = i0 + u * 256;
      if (g != IGN && i < n4) zz[u] = __builtin_nontemporal_load(z4 + i);
      if (acc && i < n4) dd[u] = d4[i];
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      int i = i0 + u * 256;
      if (i >= n4) continue;
      v4f o = {0, 0, 0, 0};
      if (g != IGN) {
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = sc * (__expf(zz[u][j] - ls) - ((i * 4 + j) == g ? 1.f : 0.f));
      }
      if (acc) o += dd[u];
      __builtin_nontemporal_store(o, d4 + i);
    }
  } else {
    const int end = min(V, (span + 1) * CE_SPAN);
    for (int i = span * CE_SPAN + threadIdx.x; i < end; i += 256) {
      float o = g == IGN ? 0.f : sc * (__expf(zr[i] - ls) - (i == g ? 1.f : 0.f));
      dr[i] = acc ? dr[i] + o : o;
    }
  }
}

// ---- chunked: per-row running (max, sum, target logit) across vocab spans ------------------------
__global__ __launch_bounds__(256) void ce_chunk_stats_k(int V, int vc, int v0, int first, const float *__restrict__ chunk,
                                                        const int *__restrict__ tgt, float *row_max, float *row_sum,
                                                        float *tgt_logit, int *bad) {
  __shared__ float sm[8];
  int64_t row = blockIdx.x;
  const float *zr = chunk + row * vc;
  float M, L;
  row_stats(zr, vc, M, L, sm);
  if (threadIdx.x == 0) {
    float m0 = first ? -INFINITY : row_max[row], l0 = first ? 0.f : row_sum[row];
    merge(m0, l0, M, L);
    row_max[row] = m0;
    row_sum[row] = l0;
    int g = tgt[row];
    if (first) {
      tgt_logit[row] = 0.f;
      if (g < IGN || g >= V) note_bad_id(bad, GT_BAD_TARGET, row, g, V);    // once per row; every kernel below ignores the row
    }
    if (g >= v0 && g < v0 + vc && g < V) tgt_logit[row] = zr[g - v0];
  }
}
__global__ __launch_bounds__(256) void ce_loss_from_stats_k(int V, int T, const int *__restrict__ tgt, const float *__restrict__ inv_denom,
                                                            const float *__restrict__ row_max, const float *__restrict__ row_sum,
                                                            const float *__restrict__ tgt_logit, float *__restrict__ loss) {
  __shared__ float sm[4];
  int s = blockIdx.x;
  float a = 0;
  for (int t = threadIdx.x; t < T; t += 256) {
    size_t r = (size_t)s * T + t;
    const int g = tgt[r];
    if (g >= 0 && g < V) a += logf(row_sum[r]) + row_max[r] - tgt_logit[r];
  }
  a = block_sum<4>(a, sm);
  if (threadIdx.x == 0) loss[s] = a * inv_denom[s];
}
// in place: chunk logits -> chunk dlogits; ignored rows zeroed (wgsl.ts:1242)
__global__ __launch_bounds__(256) void ce_chunk_grad_k(int V, int vc, int v0, int T, int spans, float *chunk,
                                                       const int *__restrict__ tgt, const float *__restrict__ inv_denom,
                                                       const float *__restrict__ row_max, const float *__restrict__ row_sum,
                                                       float seed) {
  const int64_t row = blockIdx.x / spans;        // spans of a row are numbered fastest, as in ce_bwd_k
  const int span = blockIdx.x % spans;
  int g = tgt[row];
  if (g < IGN || g >= V) g = IGN;
  const float sc = seed * inv_denom[row / T];
  const float m = row_max[row], il = 1.0f / row_sum[row];
  float *zr = chunk + row * vc;
  const int end = min(vc, (span + 1) * CE_SPAN);
  for (int i = span * CE_SPAN + threadIdx.x; i < end; i += 256)
    zr[i] = g == IGN ? 0.f : sc * (__expf(zr[i] - m) * il - ((i + v0) == g ? 1.f : 0.f));
}

// ---- sparse-teacher soft CE (autograd.ts:1076-1138) -------------------------------------------------
__global__ __launch_bounds__(256) void soft_ce_fwd_rows(int V, int k, const float *__restrict__ z, const int *__restrict__ tid,
                                                        const float *__restrict__ tq, float *__restrict__ lse,
                                                        float *__restrict__ mass, float *__restrict__ nll, int *bad) {
  __shared__ float sm[8];
  int64_t row = blockIdx.x;
  const float *zr = z + row * V;
  float M, L;
  row_stats(zr, V, M, L, sm);
  if (threadIdx.x == 0) {
    float ls = M + logf(L);
    lse[row] = ls;
    float tot = 0, ms = 0;
    if (tid[row * k] != IGN) {
      for (int j = 0; j < k; j++) {
        float qv = tq[row * k + j];
        if (qv == 0.f) continue;
        const int id = tid[row * k + j];
        if (id < 0 || id >= V) { note_bad_id(bad, GT_BAD_TEACHER_ID, row, id, V); continue; }
        tot += qv * (logf(L) + M - zr[id]);
        ms += qv;
      }
    }
    mass[row] = ms;
    nll[row] = tot;
  }
}
__global__ __launch_bounds__(256) void sum_scale_k(int n, const float *__restrict__ x, float sc, float *__restrict__ out) {
  __shared__ float sm[4];
  float a = 0;
  for (int i = threadIdx.x; i < n; i += 256) a += x[i];
  a = block_sum<4>(a, sm);
  if (threadIdx.x == 0) out[0] = a * sc;
}
// sparse half of the soft loss, one thread per row after the dense half (ce_bwd_k<true>): duplicate ids in a row are
// applied one after another by that thread, so they cannot race (wgsl.ts:1086-1090)
__global__ __launch_bounds__(64) void soft_ce_bwd_q(int rows, int V, int k, const int *__restrict__ tid,
                                                    const float *__restrict__ tq, float sc, float *dz, int *bad) {
  int64_t row = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (row >= rows || tid[row * k] == IGN) return;
  for (int j = 0; j < k; j++) {
    const int id = tid[row * k + j];
    if (id < 0 || id >= V) { note_bad_id(bad, GT_BAD_TEACHER_ID, row, id, V); continue; }
    dz[row * V + id] -= sc * tq[row * k + j];
  }
}

extern "C" {
int gt_ce_fwd(gt_ctx *ctx, int rows, int V, int T, gt_buf logits, gt_buf targets, gt_buf inv_denom, gt_buf loss, gt_buf lse) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && V >= 1 && T >= 1 && rows % T == 0, "gt_ce_fwd: rows %d must be a positive multiple of T %d", rows, T);
  GT_REQUIRE(ctx, logits && targets && inv_denom && loss && lse, "gt_ce_fwd: null operand");
  ProfScope ps(ctx, "ce", 4.0 * rows * V);
  void *ws;
  if (gt_ws_reserve(ctx, (size_t)rows * sizeof(float), &ws)) return 1;
  hipLaunchKernelGGL(ce_fwd_rows, dim3(rows), dim3(256), 0, ctx->stream, V, P<const float>(logits), P<const int>(targets),
                     P<float>(lse), static_cast<float *>(ws), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  hipLaunchKernelGGL(ce_seq_loss, dim3(rows / T), dim3(256), 0, ctx->stream, T, static_cast<const float *>(ws),
                     P<const float>(inv_denom), P<float>(loss));
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_ce_bwd(gt_ctx *ctx, int rows, int V, int T, gt_buf logits, gt_buf targets, gt_buf inv_denom, gt_buf lse, float seed,
              gt_buf dlogits, int acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && V >= 1 && T >= 1 && rows % T == 0, "gt_ce_bwd: rows %d must be a positive multiple of T %d", rows, T);
  GT_REQUIRE(ctx, logits && targets && inv_denom && lse && dlogits, "gt_ce_bwd: null operand");
  ProfScope ps(ctx, "ce.bwd", 8.0 * rows * V);          // read z, write dz
  const int spans = (int)cdiv(V, CE_SPAN);
  GT_REQUIRE(ctx, (int64_t)rows * spans < (int64_t)1 << 31, "gt_ce_bwd: %d rows x %d logits is more than one launch covers", rows, V);
  hipLaunchKernelGGL(ce_bwd_k<false>, dim3((unsigned)((int64_t)rows * spans)), dim3(256), 0, ctx->stream, V, T, spans, P<const float>(logits),
                     P<const int>(targets), P<const float>(inv_denom), P<const float>(lse), seed, P<float>(dlogits), acc,
                     (const float *)nullptr, 1);
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_ce_chunk_stats(gt_ctx *ctx, int rows, int V, int vc, int v0, int first, gt_buf chunk, gt_buf targets, gt_buf row_max,
                      gt_buf row_sum, gt_buf tgt_logit) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && vc >= 1 && v0 >= 0 && (int64_t)v0 + vc <= V && chunk && targets && row_max && row_sum && tgt_logit,
             "gt_ce_chunk_stats: bad arguments (span [%d, %d) of %d logits)", v0, v0 + vc, V);
  ProfScope ps(ctx, "ce.chunk");
  hipLaunchKernelGGL(ce_chunk_stats_k, dim3(rows), dim3(256), 0, ctx->stream, V, vc, v0, first, P<const float>(chunk),
                     P<const int>(targets), P<float>(row_max), P<float>(row_sum), P<float>(tgt_logit), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_ce_loss_from_stats(gt_ctx *ctx, int rows, int V, int T, gt_buf targets, gt_buf inv_denom, gt_buf row_max, gt_buf row_sum,
                          gt_buf tgt_logit, gt_buf loss) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && V >= 1 && T >= 1 && rows % T == 0 && targets && inv_denom && row_max && row_sum && tgt_logit && loss,
             "gt_ce_loss_from_stats: bad arguments");
  ProfScope ps(ctx, "ce.chunk");
  hipLaunchKernelGGL(ce_loss_from_stats_k, dim3(rows / T), dim3(256), 0, ctx->stream, V, T, P<const int>(targets),
                     P<const float>(inv_denom), P<const float>(row_max), P<const float>(row_sum), P<const float>(tgt_logit),
                     P<float>(loss));
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_ce_chunk_grad(gt_ctx *ctx, int rows, int V, int vc, int v0, int T, gt_buf chunk, gt_buf targets, gt_buf inv_denom,
                     gt_buf row_max, gt_buf row_sum, float seed) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && vc >= 1 && v0 >= 0 && (int64_t)v0 + vc <= V && T >= 1 && rows % T == 0 && chunk && targets && inv_denom && row_max && row_sum,
             "gt_ce_chunk_grad: bad arguments");
  ProfScope ps(ctx, "ce.chunk.bwd");
  const int spans = (int)cdiv(vc, CE_SPAN);
  GT_REQUIRE(ctx, (int64_t)rows * spans < (int64_t)1 << 31, "gt_ce_chunk_grad: %d rows x %d logits is more than one launch covers", rows, vc);
  hipLaunchKernelGGL(ce_chunk_grad_k, dim3((unsigned)((int64_t)rows * spans)), dim3(256), 0, ctx->stream, V, vc, v0, T, spans,
                     P<float>(chunk), P<const int>(targets), P<const float>(inv_denom), P<const float>(row_max),
                     P<const float>(row_sum), seed);
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_soft_ce_fwd(gt_ctx *ctx, int rows, int V, int k, gt_buf logits, gt_buf teacher_ids, gt_buf teacher_probs,
                   float inv_denom, gt_buf loss, gt_buf lse, gt_buf row_mass) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && V >= 1 && k >= 1 && logits && teacher_ids && teacher_probs && loss && lse && row_mass,
             "gt_soft_ce_fwd: bad arguments");
  ProfScope ps(ctx, "softce", 4.0 * rows * V);
  void *ws;
  if (gt_ws_reserve(ctx, (size_t)rows * sizeof(float), &ws)) return 1;
  hipLaunchKernelGGL(soft_ce_fwd_rows, dim3(rows), dim3(256), 0, ctx->stream, V, k, P<const float>(logits),
                     P<const int>(teacher_ids), P<const float>(teacher_probs), P<float>(lse), P<float>(row_mass),
                     static_cast<float *>(ws), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  hipLaunchKernelGGL(sum_scale_k, dim3(1), dim3(256), 0, ctx->stream, rows, static_cast<const float *>(ws), inv_denom, P<float>(loss));
  GT_LAUNCHED(ctx);
  return 0;
}
int gt_soft_ce_bwd(gt_ctx *ctx, int rows, int V, int k, gt_buf logits, gt_buf teacher_ids, gt_buf teacher_probs,
                   float inv_denom, gt_buf lse, gt_buf row_mass, float seed, gt_buf dlogits, int acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && V >= 1 && k >= 1 && logits && teacher_ids && teacher_probs && lse && row_mass && dlogits,
             "gt_soft_ce_bwd: bad arguments");
  ProfScope ps(ctx, "softce.bwd", 8.0 * rows * V);
  float sc = seed * inv_denom;
  const int spans = (int)cdiv(V, CE_SPAN);
  GT_REQUIRE(ctx, (int64_t)rows * spans < (int64_t)1 << 31, "gt_soft_ce_bwd: %d rows x %d logits is more than one launch covers", rows, V);
  hipLaunchKernelGGL(ce_bwd_k<true>, dim3((unsigned)((int64_t)rows * spans)), dim3(256), 0, ctx->stream, V, rows, spans, P<const float>(logits),
                     P<const int>(teacher_ids), (const float *)nullptr, P<const float>(lse), sc, P<float>(dlogits), acc,
                     P<const float>(row_mass), k);
  GT_LAUNCHED(ctx);
  hipLaunchKernelGGL(soft_ce_bwd_q, dim3((unsigned)cdiv(rows, 64)), dim3(64), 0, ctx->stream, rows, V, k,
                     P<const int>(teacher_ids), P<const float>(teacher_probs), sc, P<float>(dlogits), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  return 0;
}
}
