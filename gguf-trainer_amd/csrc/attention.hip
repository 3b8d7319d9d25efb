// Causal / sliding-window GQA attention, forward and backward, softmax recomputed in backward
// from a saved per-row log-sum-exp (srcAttnFwd / BwdD / BwdDq / BwdDkv, src/backend/wgsl.ts:657-918;
// dispatch src/backend/webgpu.ts:1142-1174). Layout: q,out [B*T, Hq*hd], k,v [B*T, Hkv*hd], row-major,
// head-major inside a row; query head h reads kv head h / (Hq/Hkv); query t attends keys
// [max(0, t-window+1), t], window 0 = full causal (src/model/autograd.ts:651-661).
//
// The saved statistic is lse2 = m*c + log2(sum exp2(s*c - m*c)) with c = log2(e)/sqrt(hd): scores
// live in the log2 domain so p = exp2(s*c - lse2) is one v_exp_f32, as in wgsl.ts:460-464.
//
// This file holds the shape-generic kernels (any hd, any T): one wavefront per query row (forward,
// dQ) or per key row (dK/dV). A 64-key (or 64-query) tile is scored with lanes across keys, the
// probabilities go through LDS, and the value/key accumulation runs with lanes across head dims,
// so global reads of K/V/Q/dO rows in that phase are contiguous. dK/dV sums over the query heads
// of the group and over queries in a fixed order; nothing is atomic.
// The MFMA kernels for hd = 64 and 128 live in attention_mfma.hip and take over when they apply.
#include <algorithm>
#include "common.h"

#define MAXD 4          // head dims per lane in the lanes-across-dims phase: hd <= 64*MAXD

struct AttnP {
  int B, T, Hq, Hkv, hd, window;
  float c2;              // log2(e)/sqrt(hd)
  float scale;           // 1/sqrt(hd)
  int splits;            // MFMA kernels: workgroups per tile (1 unless the launch is small)
};

__device__ __forceinline__ int win_lo(int t, int window) { return (window > 0 && t + 1 > window) ? t + 1 - window : 0; }

// dot of q-row (in LDS, broadcast reads) with a key row in global memory
__device__ __forceinline__ float dot_row(const float *__restrict__ qs, const float *__restrict__ kr, int hd) {
  float s = 0;
  if ((hd & 3) == 0) {
    for (int d = 0; d < hd; d += 4) {
      float4 kv = *reinterpret_cast<const float4 *>(kr + d);
      s += qs[d] * kv.x + qs[d + 1] * kv.y + qs[d + 2] * kv.z + qs[d + 3] * kv.w;
    }
  } else {
    for (int d = 0; d < hd; d++) s += qs[d] * kr[d];
  }
  return s;
}

// ---- forward ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_fwd_gen(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                    const float *__restrict__ v, float *__restrict__ out,
                                                    float *__restrict__ lse) {
  extern __shared__ float sm[];                       // per wave: q[hd] + p[64]
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  float *qs = sm + wave * (p.hd + WAVE), *ps = qs + p.hd;
  int64_t rid = (int64_t)blockIdx.x * 4 + wave;       // (b, h, t), t fastest
  if (rid >= (int64_t)p.B * p.Hq * p.T) return;
  const int t = (int)(rid % p.T), h = (int)((rid / p.T) % p.Hq), b = (int)(rid / ((int64_t)p.T * p.Hq));
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * p.hd, kstr = (size_t)p.Hkv * p.hd;
  const float *qr = q + ((size_t)b * p.T + t) * qstr + (size_t)h * p.hd;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * p.hd;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * p.hd;
  for (int d = lane; d < p.hd; d += WAVE) qs[d] = qr[d] * p.c2;
  __builtin_amdgcn_wave_barrier();
  const int s0 = win_lo(t, p.window);
  // pass 1: row max and sum in the log2 domain, lane-local online then combined
  float m = -INFINITY, l = 0;
  for (int s = s0 + lane; s <= t; s += WAVE) {
    float sc = dot_row(qs, kb + (size_t)s * kstr, p.hd);
    float mn = fmaxf(m, sc);
    l = l * exp2f(m - mn) + exp2f(sc - mn);
    m = mn;
  }
  float M = wave_max(m);
  l = wave_sum(l * exp2f(m - M));                     // lanes with no key: l = 0, exp2(-inf) = 0
  const float L2 = M + log2f(l);
  if (lane == 0) lse[rid] = L2;
  // pass 2: probabilities through LDS, output with lanes across head dims
  float acc[MAXD] = {0, 0, 0, 0};
  for (int base = s0; base <= t; base += WAVE) {
    int s = base + lane;
    float pr = 0;
    if (s <= t) pr = exp2f(dot_row(qs, kb + (size_t)s * kstr, p.hd) - L2);
    __builtin_amdgcn_wave_barrier();
    ps[lane] = pr;
    __builtin_amdgcn_wave_barrier();
    int cnt = min(WAVE, t - base + 1);
    for (int j = 0; j < cnt; j++) {
      float pj = ps[j];
      const float *vr = vb + (size_t)(base + j) * kstr;
#pragma unroll
      for (int i = 0; i < MAXD; i++) { int d = lane + i * WAVE; if (d < p.hd) acc[i] += pj * vr[d]; }
    }
  }
  float *orow = out + ((size_t)b * p.T + t) * qstr + (size_t)h * p.hd;
#pragma unroll
  for (int i = 0; i < MAXD; i++) { int d = lane + i * WAVE; if (d < p.hd) orow[d] = acc[i]; }
}

// D[b,h,t] = sum_d dO*O  (srcAttnBwdD, wgsl.ts:711-730)
__global__ __launch_bounds__(256) void attn_bwd_d(AttnP p, const float *__restrict__ o, const float *__restrict__ go,
                                                  float *__restrict__ Dr) {
  const int lane = threadIdx.x % WAVE;
  int64_t rid = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (rid >= (int64_t)p.B * p.Hq * p.T) return;
  const int t = (int)(rid % p.T), h = (int)((rid / p.T) % p.Hq), b = (int)(rid / ((int64_t)p.T * p.Hq));
  size_t off = ((size_t)b * p.T + t) * p.Hq * p.hd + (size_t)h * p.hd;
  float s = 0;
  for (int d = lane; d < p.hd; d += WAVE) s += o[off + d] * go[off + d];
  s = wave_sum(s);
  if (lane == 0) Dr[rid] = s;
}

// The same sums for head dims that are 4 x a power of two (16 .. 256): G = hd/4 lanes take one (row, head) with one
// float4 each, so a wavefront streams 1 KB of O and of dO per load in memory order [row][head][hd]; the G partial sums
// are folded by a fixed butterfly. Eight items per lane group per workgroup pass keep enough loads in flight.
template <int G>
__global__ __launch_bounds__(256) void attn_bwd_d_vec(AttnP p, const float *__restrict__ o, const float *__restrict__ go,
                                                      float *__restrict__ Dr) {
  constexpr int PER = 8;                                   // items per lane group
  typedef float f4 __attribute__((ext_vector_type(4)));
  const unsigned items = (unsigned)p.B * p.T * p.Hq;       // numbered in memory order: (b*T + t)*Hq + h
  const int sub = threadIdx.x % G;
  const unsigned grp = blockIdx.x * (256 / G) + threadIdx.x / G;
  const unsigned stride = gridDim.x * (256 / G);
  f4 a[PER], g[PER];
  // every load is issued before the first use; a group past the end re-reads the last item and drops the result
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const unsigned m = min(grp + i * stride, items - 1);
    a[i] = *(reinterpret_cast<const f4 *>(o + (size_t)m * p.hd) + sub);
    g[i] = *(reinterpret_cast<const f4 *>(go + (size_t)m * p.hd) + sub);
  }
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const unsigned m = grp + i * stride;
    float s = (a[i].x * g[i].x + a[i].y * g[i].y) + (a[i].z * g[i].z + a[i].w * g[i].w);
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
    if (sub == 0 && m < items) {
      const unsigned bt = m / (unsigned)p.Hq, h = m - bt * (unsigned)p.Hq, b = bt / (unsigned)p.T, t = bt - b * (unsigned)p.T;
      Dr[((size_t)b * p.Hq + h) * p.T + t] = s;
    }
  }
}

// ---- dQ: one wavefront per query row (srcAttnBwdDq, wgsl.ts:741-784) -----------------------------
__global__ __launch_bounds__(256) void attn_bwd_dq_gen(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                       const float *__restrict__ v, const float *__restrict__ go,
                                                       const float *__restrict__ lse, const float *__restrict__ Dr,
                                                       float *dq, int acc_q) {
  extern __shared__ float sm[];                       // per wave: q[hd] + dO[hd] + ds[64]
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  float *qs = sm + wave * (2 * p.hd + WAVE), *gs = qs + p.hd, *ds = gs + p.hd;
  int64_t rid = (int64_t)blockIdx.x * 4 + wave;
  if (rid >= (int64_t)p.B * p.Hq * p.T) return;
  const int t = (int)(rid % p.T), h = (int)((rid / p.T) % p.Hq), b = (int)(rid / ((int64_t)p.T * p.Hq));
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * p.hd, kstr = (size_t)p.Hkv * p.hd;
  const size_t qoff = ((size_t)b * p.T + t) * qstr + (size_t)h * p.hd;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * p.hd;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * p.hd;
  for (int d = lane; d < p.hd; d += WAVE) { qs[d] = q[qoff + d] * p.c2; gs[d] = go[qoff + d]; }
  __builtin_amdgcn_wave_barrier();
  const float L2 = lse[rid], Dt = Dr[rid];
  const int s0 = win_lo(t, p.window);
  float acc[MAXD] = {0, 0, 0, 0};
  for (int base = s0; base <= t; base += WAVE) {
    int s = base + lane;
    float dsv = 0;
    if (s <= t) {
      float pr = exp2f(dot_row(qs, kb + (size_t)s * kstr, p.hd) - L2);
      float dp = dot_row(gs, vb + (size_t)s * kstr, p.hd);
      dsv = pr * (dp - Dt) * p.scale;
    }
    __builtin_amdgcn_wave_barrier();
    ds[lane] = dsv;
    __builtin_amdgcn_wave_barrier();
    int cnt = min(WAVE, t - base + 1);
    for (int j = 0; j < cnt; j++) {
      float dj = ds[j];
      const float *kr = kb + (size_t)(base + j) * kstr;
#pragma unroll
      for (int i = 0; i < MAXD; i++) { int d = lane + i * WAVE; if (d < p.hd) acc[i] += dj * kr[d]; }
    }
  }
#pragma unroll
  for (int i = 0; i < MAXD; i++) {
    int d = lane + i * WAVE;
    if (d < p.hd) dq[qoff + d] = acc_q ? dq[qoff + d] + acc[i] : acc[i];
  }
}

// ---- dK, dV: one wavefront per key row, summed over the group's query heads
// (srcAttnBwdDkv, wgsl.ts:804-918) ---------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_bwd_dkv_gen(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                        const float *__restrict__ v, const float *__restrict__ go,
                                                        const float *__restrict__ lse, const float *__restrict__ Dr,
                                                        float *dk, int acc_k, float *dv, int acc_v) {
  extern __shared__ float sm[];                       // per wave: k[hd] + v[hd] + p[64] + ds[64]
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  float *ks = sm + wave * (2 * p.hd + 2 * WAVE), *vs = ks + p.hd, *ps = vs + p.hd, *ds = ps + WAVE;
  int64_t rid = (int64_t)blockIdx.x * 4 + wave;       // (b, kvh, s), s fastest
  if (rid >= (int64_t)p.B * p.Hkv * p.T) return;
  const int s = (int)(rid % p.T), kvh = (int)((rid / p.T) % p.Hkv), b = (int)(rid / ((int64_t)p.T * p.Hkv));
  const int group = p.Hq / p.Hkv;
  const size_t qstr = (size_t)p.Hq * p.hd, kstr = (size_t)p.Hkv * p.hd;
  const size_t koff = ((size_t)b * p.T + s) * kstr + (size_t)kvh * p.hd;
  for (int d = lane; d < p.hd; d += WAVE) { ks[d] = k[koff + d] * p.c2; vs[d] = v[koff + d]; }
  __builtin_amdgcn_wave_barrier();
  // queries that see key s: t in [s, min(T-1, s+window-1)]
  const int t1 = p.window > 0 ? min(p.T - 1, s + p.window - 1) : p.T - 1;
  float ak[MAXD] = {0, 0, 0, 0}, av[MAXD] = {0, 0, 0, 0};
  for (int hh = 0; hh < group; hh++) {
    const int h = kvh * group + hh;
    const float *qb = q + (size_t)b * p.T * qstr + (size_t)h * p.hd;
    const float *gb = go + (size_t)b * p.T * qstr + (size_t)h * p.hd;
    const float *lb = lse + ((size_t)b * p.Hq + h) * p.T, *db = Dr + ((size_t)b * p.Hq + h) * p.T;
    for (int base = s; base <= t1; base += WAVE) {
      int t = base + lane;
      float pr = 0, dsv = 0;
      if (t <= t1) {
        pr = exp2f(dot_row(ks, qb + (size_t)t * qstr, p.hd) - lb[t]);
        float dp = dot_row(vs, gb + (size_t)t * qstr, p.hd);
        dsv = pr * (dp - db[t]) * p.scale;
      }
      __builtin_amdgcn_wave_barrier();
      ps[lane] = pr;
      ds[lane] = dsv;
      __builtin_amdgcn_wave_barrier();
      int cnt = min(WAVE, t1 - base + 1);
      for (int j = 0; j < cnt; j++) {
        float pj = ps[j], dj = ds[j];
        const float *gr = gb + (size_t)(base + j) * qstr, *qr = qb + (size_t)(base + j) * qstr;
#pragma unroll
        for (int i = 0; i < MAXD; i++) {
          int d = lane + i * WAVE;
          if (d < p.hd) { av[i] += pj * gr[d]; ak[i] += dj * qr[d]; }
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MAXD; i++) {
    int d = lane + i * WAVE;
    if (d < p.hd) {
      dk[koff + d] = acc_k ? dk[koff + d] + ak[i] : ak[i];
      dv[koff + d] = acc_v ? dv[koff + d] + av[i] : av[i];
    }
  }
}

// attention_mfma.hip, compiled once per head dim
int attn_fwd_mfma32(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, float *fpart, float *sco);
int attn_bwd_mfma32(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr, float *part,
                    float *dqpart, float *dsb, const float *sco, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v,
                    const float *rot_q, const float *rot_k, float *bandp, int band_splits);
int attn_fwd_mfma64(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, float *fpart, float *sco);
int attn_fwd_mfma128(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, float *fpart, float *sco);
int attn_bwd_mfma64(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr, float *part,
                    float *dqpart, float *dsb, const float *sco, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v,
                    const float *rot_q, const float *rot_k, float *bandp, int band_splits);
int attn_bwd_mfma128(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr, float *part,
                     float *dqpart, float *dsb, const float *sco, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v,
                     const float *rot_q, const float *rot_k, float *bandp, int band_splits);
static int attn_mfma_supported(int hd) { return hd == 32 || hd == 64 || hd == 128; }

// A launch with fewer 128-row tiles than three per CU is cut further (measured at T = 2048, 9 heads: 1 sequence runs
// 2.3x faster with 6 workgroups per tile, 2 sequences 1.5x with 3, 4 sequences 1.13x with 2, 8 gain nothing): every tile's loop range goes to `splits`
// workgroups (at most 8, at most one per 64-key stage of the longest tile) whose partial results are folded afterwards.
static int attn_splits(gt_ctx *ctx, int B, int T, int Hq) {
  const int64_t tiles = cdiv(T, 128) * Hq * B;
  int s = 1;
  if (tiles < 3 * (int64_t)ctx->num_cu) s = (int)std::min<int64_t>(8, cdiv(3 * (int64_t)ctx->num_cu, tiles));
  if (ctx->opt_attn_splits >= 1) s = std::min(ctx->opt_attn_splits, 8);
  return (int)std::max<int64_t>(1, std::min<int64_t>(s, cdiv(T, 64)));
}

// out = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), lse2 = m + log2(that sum), m = max_s m_s: the online-softmax
// merge of the splits' partial results, in split order. One thread per float4 of the output.
__global__ __launch_bounds__(256) void attn_fwd_combine(AttnP p, const float *__restrict__ fpart, float *__restrict__ out,
                                                        float *__restrict__ lse) {
  const int hd4 = p.hd / 4;
  const int64_t n = (int64_t)p.B * p.T * p.Hq * hd4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int d4 = (int)(i % hd4), h = (int)((i / hd4) % p.Hq);
  const int64_t row = i / ((int64_t)hd4 * p.Hq);            // b*T + t
  const int64_t b = row / p.T, t = row % p.T;
  const size_t slice = (size_t)p.B * p.T * p.Hq * p.hd, rows = (size_t)p.B * p.Hq * p.T;
  const size_t sidx = ((size_t)b * p.Hq + h) * p.T + t;
  const float *mp = fpart + (size_t)p.splits * slice, *lp = mp + (size_t)p.splits * rows;
  float m = -1.0e30f;
  for (int s = 0; s < p.splits; s++) m = fmaxf(m, mp[s * rows + sidx]);
  float L = 0.f;
  float4 o = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < p.splits; s++) {
    const float wgt = __builtin_amdgcn_exp2f(mp[s * rows + sidx] - m);
    L += lp[s * rows + sidx] * wgt;
    const float4 x = reinterpret_cast<const float4 *>(fpart + s * slice)[i];
    o.x += x.x * wgt; o.y += x.y * wgt; o.z += x.z * wgt; o.w += x.w * wgt;
  }
  const float inv = 1.0f / L;
  reinterpret_cast<float4 *>(out)[i] = float4{o.x * inv, o.y * inv, o.z * inv, o.w * inv};
  if (d4 == 0) lse[sidx] = m + log2f(L);
}
// dst (+)= sum of `ns` slices of n4 float4 each, in slice order
__global__ __launch_bounds__(256) void attn_slice_sum(const float *__restrict__ part, int ns, size_t n4, float *dst, int acc) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const float4 *pp = reinterpret_cast<const float4 *>(part);
  float4 a = pp[i];
  for (int s = 1; s < ns; s++) { float4 x = pp[(size_t)s * n4 + i]; a.x += x.x; a.y += x.y; a.z += x.z; a.w += x.w; }
  float4 *o = reinterpret_cast<float4 *>(dst) + i;
  if (acc) { float4 y = *o; a.x += y.x; a.y += y.y; a.z += y.z; a.w += y.w; }
  *o = a;
}

static int attn_fwd_mfma(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, gt_buf scores) {
  float *sco = P<float>(scores);
  float *fpart = nullptr;
  if (p.splits > 1) {
    const size_t slice = (size_t)p.B * p.T * p.Hq * p.hd, rows = (size_t)p.B * p.Hq * p.T;
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)p.splits * (slice + 2 * rows) * sizeof(float), &ws)) return 1;
    fpart = static_cast<float *>(ws);
  }
  if (p.hd == 32 ? attn_fwd_mfma32(ctx, p, q, k, v, out, lse, fpart, sco)
      : p.hd == 64 ? attn_fwd_mfma64(ctx, p, q, k, v, out, lse, fpart, sco) : attn_fwd_mfma128(ctx, p, q, k, v, out, lse, fpart, sco)) return 1;
  if (p.splits > 1) {
    const int64_t n = (int64_t)p.B * p.T * p.Hq * (p.hd / 4);
    hipLaunchKernelGGL(attn_fwd_combine, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, ctx->stream, p, fpart, P<float>(out), P<float>(lse));
    GT_LAUNCHED(ctx);
  }
  return 0;
}
static int attn_bwd_mfma(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr,
                         float *part, float *dqpart, float *dsb, const float *sco, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv,
                         int acc_v, const float *rot_q, const float *rot_k, float *bandp, int band_splits) {
  if (p.hd == 32 ? attn_bwd_mfma32(ctx, p, q, k, v, dout, lse, Dr, part, dqpart, dsb, sco, dq, acc_q, dk, acc_k, dv, acc_v, rot_q, rot_k, bandp, band_splits)
      : p.hd == 64 ? attn_bwd_mfma64(ctx, p, q, k, v, dout, lse, Dr, part, dqpart, dsb, sco, dq, acc_q, dk, acc_k, dv, acc_v, rot_q, rot_k, bandp, band_splits)
                   : attn_bwd_mfma128(ctx, p, q, k, v, dout, lse, Dr, part, dqpart, dsb, sco, dq, acc_q, dk, acc_k, dv, acc_v, rot_q, rot_k, bandp, band_splits))
    return 1;
  if (p.splits > 1 && !dsb) {
    const size_t n4 = (size_t)p.B * p.T * p.Hq * p.hd / 4;
    hipLaunchKernelGGL(attn_slice_sum, dim3((unsigned)cdiv((int64_t)n4, 256)), dim3(256), 0, ctx->stream, dqpart, p.splits, n4,
                       P<float>(dq), acc_q);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

static int check(gt_ctx *ctx, const char *who, int B, int T, int Hq, int Hkv, int hd, int window) {
  GT_REQUIRE(ctx, B >= 1 && T >= 1 && Hq >= 1 && Hkv >= 1 && hd >= 1 && window >= 0, "%s: bad shape", who);
  GT_REQUIRE(ctx, Hq % Hkv == 0, "%s: %d query heads do not group over %d kv heads", who, Hq, Hkv);
  GT_REQUIRE(ctx, hd <= WAVE * MAXD, "%s: head dim %d exceeds %d", who, hd, WAVE * MAXD);
  return 0;
}

// (query, key) pairs a causal / windowed sequence of T scores
static double attn_pairs(int T, int window) {
  double p = 0;
  for (int t = 0; t < T; t++) p += (window > 0 && t + 1 > window) ? window : t + 1;
  return p;
}

// kept scores: the MFMA kernels on whole 128-row tiles only (the blocks are addressed per 32 x 32 sub-tile)
static bool scores_supported(gt_ctx *ctx, int T, int hd) {
  return !ctx->opt_attn_generic && attn_mfma_supported(hd) && hd >= 64 && T % 128 == 0;
}

static int attn_fwd_impl(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                         gt_buf lse, gt_buf scores) {
  GT_ENTER(ctx);
  if (check(ctx, "gt_attn_fwd", B, T, Hq, Hkv, hd, window)) return 1;
  GT_REQUIRE(ctx, q && k && v && out && lse, "gt_attn_fwd: null operand");
  GT_REQUIRE(ctx, !scores || (scores_supported(ctx, T, hd) && scores % 16 == 0),
             "gt_attn_fwd_scores: scores are kept for T a multiple of 128 and head dim 64 or 128 only (T %d, hd %d)", T, hd);
  AttnP p{B, T, Hq, Hkv, hd, window, 1.4426950408889634f / sqrtf((float)hd), 1.0f / sqrtf((float)hd), 1};
  if (!ctx->opt_attn_generic && attn_mfma_supported(hd)) p.splits = attn_splits(ctx, B, T, Hq);
  ProfScope ps(ctx, "attention", 2.0 * 2 * hd * attn_pairs(T, window) * Hq * B);   // QK^T and PV
  if (!ctx->opt_attn_generic && attn_mfma_supported(hd)) return attn_fwd_mfma(ctx, p, q, k, v, out, lse, scores);
  int64_t rows = (int64_t)B * Hq * T;
  size_t smem = 4 * (size_t)(hd + WAVE) * sizeof(float);
  hipLaunchKernelGGL(attn_fwd_gen, dim3((unsigned)cdiv(rows, 4)), dim3(256), smem, ctx->stream, p, P<const float>(q),
                     P<const float>(k), P<const float>(v), P<float>(out), P<float>(lse));
  GT_LAUNCHED(ctx);
  return 0;
}

// rope: with rot_q / rot_k set, q / k are rows that went through the rotation (base, pos) and dq / dk receive the gradients
// with respect to the rows BEFORE it (MFMA kernels only: the caller has checked that)
struct RopeBack { double base = 0; int pos = 0, rot_q = 0, rot_k = 0; };
static int attn_bwd_impl(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                         gt_buf dout, gt_buf lse, gt_buf scores, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v,
                         const RopeBack &rope = RopeBack()) {
  GT_ENTER(ctx);
  if (check(ctx, "gt_attn_bwd", B, T, Hq, Hkv, hd, window)) return 1;
  GT_REQUIRE(ctx, q && k && v && out && dout && lse && dq && dk && dv, "gt_attn_bwd: null operand");
  GT_REQUIRE(ctx, !scores || (scores_supported(ctx, T, hd) && scores % 16 == 0),
             "gt_attn_bwd_scores: scores are kept for T a multiple of 128 and head dim 64 or 128 only (T %d, hd %d)", T, hd);
  AttnP p{B, T, Hq, Hkv, hd, window, 1.4426950408889634f / sqrtf((float)hd), 1.0f / sqrtf((float)hd), 1};
  int64_t rows = (int64_t)B * Hq * T, krows = (int64_t)B * Hkv * T;
  ProfScope whole(ctx, "attention.bwd", 5.0 * 2 * hd * attn_pairs(T, window) * Hq * B);   // S, dP, dV, dK, dQ
  // workspace: D per (sequence, head, row); then (MFMA path) one dK and one dV slice per (split, query head of the kv
  // group) when there is more than one, and one dQ partial per split when the launch is split
  const bool mfma = !ctx->opt_attn_generic && attn_mfma_supported(hd);
  const int group = Hq / Hkv;
  if (mfma) p.splits = attn_splits(ctx, B, T, Hq);
  const size_t d_floats = ((size_t)rows + 63) / 64 * 64;
  const size_t part_floats = (mfma && p.splits * group > 1) ? (size_t)2 * p.splits * group * krows * hd : 0;
  // dS kept for the dQ product (one [T][T] matrix per sequence and head) when the tiles are whole and the matrices fit
  // the limit; otherwise dQ recomputes the scores in its own kernel (with one partial per split when the launch is split)
  size_t ds_floats = (mfma && ctx->opt_attn_keep_ds && T % 128 == 0 && hd >= 64) ? (size_t)rows * T : 0;
  if (ds_floats * sizeof(float) > ((size_t)ctx->opt_attn_ds_limit_mb << 20)) ds_floats = 0;
  const size_t dq_floats = (mfma && p.splits > 1 && !ds_floats) ? (size_t)p.splits * rows * hd : 0;
  // a small launch of the banded dQ product cuts its K ranges into parts, one plane of dQ's size each (gemm_band_dq_splits)
  const int band_splits = ds_floats ? gemm_band_dq_splits(ctx, B, T, Hq, window) : 1;
  const size_t band_floats = band_splits > 1 ? (size_t)band_splits * rows * hd : 0;
  void *ws;
  if (gt_ws_reserve(ctx, (d_floats + part_floats + dq_floats + ds_floats + band_floats) * sizeof(float), &ws)) return 1;
  float *Dr = static_cast<float *>(ws);
  float *part = part_floats ? Dr + d_floats : nullptr;
  float *dqpart = dq_floats ? Dr + d_floats + part_floats : nullptr;
  float *dsb = ds_floats ? Dr + d_floats + part_floats + dq_floats : nullptr;
  float *bandp = band_floats ? Dr + d_floats + part_floats + dq_floats + ds_floats : nullptr;
  {
    ProfScope ps(ctx, "attention.bwd.D");
    const int G = p.hd / 4;
    const bool vec = p.hd % 4 == 0 && G >= 4 && G <= 64 && (G & (G - 1)) == 0 && (out | dout) % 16 == 0 && rows < ((int64_t)1 << 31);
    if (vec) {
      const unsigned nb = (unsigned)cdiv(rows, (int64_t)(256 / G) * 8);
#define GO_D(GG) hipLaunchKernelGGL((attn_bwd_d_vec<GG>), dim3(nb), dim3(256), 0, ctx->stream, p, P<const float>(out), P<const float>(dout), Dr)
      switch (G) {
        case 4: GO_D(4); break;
        case 8: GO_D(8); break;
        case 16: GO_D(16); break;
        case 32: GO_D(32); break;
        default: GO_D(64); break;
      }
#undef GO_D
    } else {
      hipLaunchKernelGGL(attn_bwd_d, dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, ctx->stream, p, P<const float>(out),
                         P<const float>(dout), Dr);
    }
    GT_LAUNCHED(ctx);
  }
  float *rot = nullptr;
  if (rope.rot_q || rope.rot_k) {
    GT_REQUIRE(ctx, mfma, "gt_attn_bwd_scores_rope: the rotation's backward rides the matrix-core kernels only");
    if (rope_table_get(ctx, T, hd, rope.base, rope.pos, &rot)) return 1;
  }
  if (mfma) return attn_bwd_mfma(ctx, p, q, k, v, dout, lse, Dr, part, dqpart, dsb, P<const float>(scores), dq, acc_q, dk, acc_k, dv, acc_v,
                                 rope.rot_q ? rot : nullptr, rope.rot_k ? rot : nullptr, bandp, band_splits);
  {
    ProfScope ps(ctx, "attention.bwd.dq");
    size_t smem = 4 * (size_t)(2 * hd + WAVE) * sizeof(float);
    hipLaunchKernelGGL(attn_bwd_dq_gen, dim3((unsigned)cdiv(rows, 4)), dim3(256), smem, ctx->stream, p, P<const float>(q),
                       P<const float>(k), P<const float>(v), P<const float>(dout), P<const float>(lse), Dr, P<float>(dq), acc_q);
    GT_LAUNCHED(ctx);
  }
  {
    ProfScope ps(ctx, "attention.bwd.dkv");
    size_t smem = 4 * (size_t)(2 * hd + 2 * WAVE) * sizeof(float);
    hipLaunchKernelGGL(attn_bwd_dkv_gen, dim3((unsigned)cdiv(krows, 4)), dim3(256), smem, ctx->stream, p, P<const float>(q),
                       P<const float>(k), P<const float>(v), P<const float>(dout), P<const float>(lse), Dr, P<float>(dk), acc_k,
                       P<float>(dv), acc_v);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

extern "C" {
int gt_attn_fwd(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                gt_buf lse) {
  return attn_fwd_impl(ctx, B, T, Hq, Hkv, hd, window, q, k, v, out, lse, 0);
}
int gt_attn_bwd(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                gt_buf dout, gt_buf lse, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v) {
  return attn_bwd_impl(ctx, B, T, Hq, Hkv, hd, window, q, k, v, out, dout, lse, 0, dq, acc_q, dk, acc_k, dv, acc_v);
}
int gt_attn_scores_bytes(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, uint64_t *bytes) {
  GT_ENTER(ctx);
  if (check(ctx, "gt_attn_scores_bytes", B, T, Hq, Hkv, hd, window)) return 1;
  GT_REQUIRE(ctx, bytes, "gt_attn_scores_bytes: null result");
  *bytes = scores_supported(ctx, T, hd) ? (uint64_t)B * Hq * T * T * sizeof(float) : 0;
  return 0;
}
int gt_attn_fwd_scores(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                       gt_buf lse, gt_buf scores) {
  if (ctx && !scores) GT_FAIL(ctx, "gt_attn_fwd_scores: null scores buffer");
  return attn_fwd_impl(ctx, B, T, Hq, Hkv, hd, window, q, k, v, out, lse, scores);
}
int gt_attn_bwd_scores(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                       gt_buf dout, gt_buf lse, gt_buf scores, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v) {
  if (ctx && !scores) GT_FAIL(ctx, "gt_attn_bwd_scores: null scores buffer");
  return attn_bwd_impl(ctx, B, T, Hq, Hkv, hd, window, q, k, v, out, dout, lse, scores, dq, acc_q, dk, acc_k, dv, acc_v);
}
int gt_attn_bwd_scores_rope(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, gt_buf q, gt_buf k, gt_buf v, gt_buf out,
                            gt_buf dout, gt_buf lse, gt_buf scores, double rope_base, int rope_pos, int rot_q, int rot_k,
                            gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v) {
  if (ctx && !scores) GT_FAIL(ctx, "gt_attn_bwd_scores_rope: null scores buffer");
  if (ctx && hd % 8 != 0) GT_FAIL(ctx, "gt_attn_bwd_scores_rope: head dim %d is not a multiple of 8", hd);
  RopeBack r;
  r.base = rope_base; r.pos = rope_pos; r.rot_q = rot_q != 0; r.rot_k = rot_k != 0;
  return attn_bwd_impl(ctx, B, T, Hq, Hkv, hd, window, q, k, v, out, dout, lse, scores, dq, acc_q, dk, acc_k, dv, acc_v, r);
}
}
