// Attention forward / backward on the FP32 matrix cores (v_mfma_f32_32x32x2_f32) for head dims that
// are multiples of 32 (64 and 128 are the shapes of every config). Same math and saved statistic as
// the generic kernels in attention.hip: causal / sliding window, GQA, scores in the log2 domain,
// softmax recomputed in backward from lse2.
//
// How the tiles map onto a 64-lane wavefront. A wavefront owns 32 queries (forward, dQ) or 32 keys
// (dK/dV); a workgroup is four of them. Scores are computed TRANSPOSED, S^T[key][query] = K.Q^T
// (forward, dQ), so that an accumulator lane holds ONE query (column lane%32) and 16 keys: the
// softmax row statistics are per-lane scalars and the row reduction is in-register plus one
// cross-half shuffle. In dK/dV it is S[query][key] = Q.K^T, one key per lane. Either way the 16
// accumulator registers of a lane sit at rows 8*(r/4) + 4*(lane/32) + r%4, which is exactly the K
// index order an MFMA step sequence consumes when step i takes row 8*(i/4) + 4*(lane/32) + i%4 from
// its half: the probability / dS tile feeds the second contraction (P.V, dS.K, P^T.dO, dS^T.Q)
// straight from the accumulators, with no transpose through LDS.
//
// Operand staging. The 32-row tile that changes per iteration (K,V in forward and dQ; Q,dO in dK/dV)
// is staged in LDS as [row][hd+4]. The first contraction reads it with ds_read_b128 (a lane's MFMA
// inputs for four steps; row stride hd+4 words keeps every 8-lane group on distinct banks), the
// second reads columns of the same tile with ds_read_b32 (consecutive lanes, consecutive banks).
// The operand that stays fixed for the whole loop (this lane's query / key row) lives in registers.
// Global loads of the next tile are issued into registers before the MFMAs of the current one.
//
// dK/dV loops over the query heads of the kv group inside the workgroup and over query tiles in
// increasing order, so the GQA sum has a fixed order and needs no atomics.
#include <algorithm>
#include "common.h"

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct AttnP {
  int B, T, Hq, Hkv, hd, window;
  float c2;
  float scale;
};

#define NEG_BIG (-1.0e30f)

__device__ __forceinline__ int win_lo_m(int t, int window) { return (window > 0 && t + 1 > window) ? t + 1 - window : 0; }
// row of accumulator register r (== K index of MFMA step r) for lane half g
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }

template <int HD> struct TileIO {
  static constexpr int LD = HD + 4;
  static constexpr int PER = (32 * HD / 4) / 256;            // float4 units per thread
  static_assert((32 * HD / 4) % 256 == 0, "head dim must be a multiple of 32");
  // rows [row0, row0+32) of a row-major matrix with `stride` floats per row, columns [0,HD) at src
  __device__ static __forceinline__ void load(v4f (&reg)[PER], const float *__restrict__ src, size_t stride, int row0, int rmax, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * 256, row = u / (HD / 4), c4 = u % (HD / 4);
      v4f v = {0.f, 0.f, 0.f, 0.f};
      if (row0 + row < rmax) v = *reinterpret_cast<const v4f *>(src + (size_t)(row0 + row) * stride + c4 * 4);
      reg[i] = v;
    }
  }
  __device__ static __forceinline__ void store(const v4f (&reg)[PER], float *lds, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * 256, row = u / (HD / 4), c4 = u % (HD / 4);
      *reinterpret_cast<v4f *>(lds + row * LD + c4 * 4) = reg[i];
    }
  }
};

// this lane's row as MFMA B-operand registers: reg[4j+s] = x[8j + 4g + s] * mul
template <int HD>
__device__ __forceinline__ void load_row_regs(float (&reg)[HD / 2], const float *__restrict__ row, bool valid, int g, float mul) {
#pragma unroll
  for (int j = 0; j < HD / 8; j++) {
    v4f v = {0.f, 0.f, 0.f, 0.f};
    if (valid) v = *reinterpret_cast<const v4f *>(row + 8 * j + 4 * g);
#pragma unroll
    for (int s = 0; s < 4; s++) reg[4 * j + s] = v[s] * mul;
  }
}

// acc = Tile(rows) . reg^T : A from LDS rows (b128), B from this lane's registers
template <int HD>
__device__ __forceinline__ v16f tile_dot_regs(const float *lds, const float (&reg)[HD / 2], int l32, int g) {
  constexpr int LD = HD + 4;
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
  for (int j = 0; j < HD / 8; j++) {
    v4f a = *reinterpret_cast<const v4f *>(lds + l32 * LD + 8 * j + 4 * g);
#pragma unroll
    for (int s = 0; s < 4; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], reg[4 * j + s], acc, 0, 0, 0);
  }
  return acc;
}

// out[dt] += Tile^T(cols of dt) . w : A = columns of the LDS tile (b32), B = the 16 accumulator-ordered weights
template <int HD>
__device__ __forceinline__ void tile_t_dot_acc(v16f (&out)[HD / 32], const float *lds, const float (&w)[16], int l32, int g) {
  constexpr int LD = HD + 4;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const float *rowp = lds + acc_row(i, g) * LD + l32;
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++) out[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(rowp[dt * 32], w[i], out[dt], 0, 0, 0);
  }
}

// write this lane's 32x(HD) transposed accumulator column (one row t of a [rows][stride] matrix)
template <int HD>
__device__ __forceinline__ void store_row(float *row, const v16f (&acc)[HD / 32], int g, float mul, int add) {
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      v4f o = {acc[dt][4 * a] * mul, acc[dt][4 * a + 1] * mul, acc[dt][4 * a + 2] * mul, acc[dt][4 * a + 3] * mul};
      v4f *dst = reinterpret_cast<v4f *>(row + dt * 32 + 8 * a + 4 * g);
      if (add) o += *dst;
      *dst = o;
    }
}

// ---- forward --------------------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_fwd_mfma_k(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                       const float *__restrict__ v, float *__restrict__ out,
                                                       float *__restrict__ lse) {
  using IO = TileIO<HD>;
  constexpr int LD = HD + 4;
  __shared__ __attribute__((aligned(16))) float sK[32 * LD];
  __shared__ __attribute__((aligned(16))) float sV[32 * LD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, g = lane / 32, l32 = lane % 32;
  const int qtile = gridDim.x - 1 - blockIdx.x;          // longest rows first
  const int h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int tq0 = qtile * 128 + wave * 32, t = tq0 + l32;
  const int tq1 = min(tq0 + 31, p.T - 1);
  const bool tv = t < p.T;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  float qreg[HD / 2];
  load_row_regs<HD>(qreg, q + ((size_t)b * p.T + (tv ? t : 0)) * qstr + (size_t)h * HD, tv, g, p.c2);
  const int lo_t = win_lo_m(t, p.window);
  const int kt_lo = win_lo_m(qtile * 128, p.window) / 32;
  const int kt_hi = min(p.T - 1, qtile * 128 + 127) / 32;
  const int wave_lo = win_lo_m(tq0, p.window);

  v16f oacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  float m = NEG_BIG, l = 0.f;

  v4f pk[IO::PER], pv[IO::PER];
  IO::load(pk, kb, kstr, kt_lo * 32, p.T, tid);
  IO::load(pv, vb, kstr, kt_lo * 32, p.T, tid);
  for (int kt = kt_lo; kt <= kt_hi; kt++) {
    __syncthreads();
    IO::store(pk, sK, tid);
    IO::store(pv, sV, tid);
    __syncthreads();
    if (kt < kt_hi) {
      IO::load(pk, kb, kstr, (kt + 1) * 32, p.T, tid);
      IO::load(pv, vb, kstr, (kt + 1) * 32, p.T, tid);
    }
    const int k0 = kt * 32;
    if (k0 > tq1 || k0 + 31 < wave_lo || tq0 >= p.T) continue;      // wave-uniform: nothing of this tile is visible
    v16f s = tile_dot_regs<HD>(sK, qreg, l32, g);
    float pr[16];
    float mx = NEG_BIG;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int key = k0 + acc_row(r, g);
      bool ok = tv && key <= t && key >= lo_t;
      pr[r] = ok ? s[r] : NEG_BIG;
      mx = fmaxf(mx, pr[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float alpha = exp2f(m - mn);
    float ls = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      pr[r] = pr[r] > -1.0e29f ? exp2f(pr[r] - mn) : 0.f;
      ls += pr[r];
    }
    l = l * alpha + ls;
    m = mn;
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
    tile_t_dot_acc<HD>(oacc, sV, pr, l32, g);
  }
  const float lt = l + __shfl_xor(l, 32, 64);
  if (tv) {
    store_row<HD>(out + ((size_t)b * p.T + t) * qstr + (size_t)h * HD, oacc, g, 1.0f / lt, 0);
    if (g == 0) lse[((size_t)b * p.Hq + h) * p.T + t] = m + log2f(lt);
  }
}

// ---- dQ -----------------------------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_bwd_dq_mfma_k(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v, const float *__restrict__ go,
                                                          const float *__restrict__ lse, const float *__restrict__ Dr,
                                                          float *dq, int acc_q) {
  using IO = TileIO<HD>;
  constexpr int LD = HD + 4;
  __shared__ __attribute__((aligned(16))) float sK[32 * LD];
  __shared__ __attribute__((aligned(16))) float sV[32 * LD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, g = lane / 32, l32 = lane % 32;
  const int qtile = gridDim.x - 1 - blockIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int tq0 = qtile * 128 + wave * 32, t = tq0 + l32;
  const int tq1 = min(tq0 + 31, p.T - 1);
  const bool tv = t < p.T;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const size_t qoff = ((size_t)b * p.T + (tv ? t : 0)) * qstr + (size_t)h * HD;
  float qreg[HD / 2], greg[HD / 2];
  load_row_regs<HD>(qreg, q + qoff, tv, g, p.c2);
  load_row_regs<HD>(greg, go + qoff, tv, g, 1.0f);
  const size_t sidx = ((size_t)b * p.Hq + h) * p.T + (tv ? t : 0);
  const float L2 = tv ? lse[sidx] : 0.f, Dt = tv ? Dr[sidx] : 0.f;
  const int lo_t = win_lo_m(t, p.window);
  const int kt_lo = win_lo_m(qtile * 128, p.window) / 32;
  const int kt_hi = min(p.T - 1, qtile * 128 + 127) / 32;
  const int wave_lo = win_lo_m(tq0, p.window);

  v16f dacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dacc[dt][r] = 0.f;

  v4f pk[IO::PER], pv[IO::PER];
  IO::load(pk, kb, kstr, kt_lo * 32, p.T, tid);
  IO::load(pv, vb, kstr, kt_lo * 32, p.T, tid);
  for (int kt = kt_lo; kt <= kt_hi; kt++) {
    __syncthreads();
    IO::store(pk, sK, tid);
    IO::store(pv, sV, tid);
    __syncthreads();
    if (kt < kt_hi) {
      IO::load(pk, kb, kstr, (kt + 1) * 32, p.T, tid);
      IO::load(pv, vb, kstr, (kt + 1) * 32, p.T, tid);
    }
    const int k0 = kt * 32;
    if (k0 > tq1 || k0 + 31 < wave_lo || tq0 >= p.T) continue;
    v16f s = tile_dot_regs<HD>(sK, qreg, l32, g);
    v16f dp = tile_dot_regs<HD>(sV, greg, l32, g);
    float ds[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int key = k0 + acc_row(r, g);
      bool ok = tv && key <= t && key >= lo_t;
      float pr = ok ? exp2f(s[r] - L2) : 0.f;
      ds[r] = pr * (dp[r] - Dt) * p.scale;
    }
    tile_t_dot_acc<HD>(dacc, sK, ds, l32, g);
  }
  if (tv) store_row<HD>(dq + qoff, dacc, g, 1.0f, acc_q);
}

// ---- dK, dV ---------------------------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_bwd_dkv_mfma_k(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                           const float *__restrict__ v, const float *__restrict__ go,
                                                           const float *__restrict__ lse, const float *__restrict__ Dr,
                                                           float *dk, int acc_k, float *dv, int acc_v) {
  using IO = TileIO<HD>;
  constexpr int LD = HD + 4;
  __shared__ __attribute__((aligned(16))) float sQ[32 * LD];
  __shared__ __attribute__((aligned(16))) float sG[32 * LD];
  __shared__ float sL[32], sD[32];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, g = lane / 32, l32 = lane % 32;
  const int ktile = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int group = p.Hq / p.Hkv;
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int sk0 = ktile * 128 + wave * 32, s = sk0 + l32;
  const bool sv = s < p.T;
  const size_t koff = ((size_t)b * p.T + (sv ? s : 0)) * kstr + (size_t)kvh * HD;
  float kreg[HD / 2], vreg[HD / 2];
  load_row_regs<HD>(kreg, k + koff, sv, g, p.c2);
  load_row_regs<HD>(vreg, v + koff, sv, g, 1.0f);
  // queries that can see a key of this workgroup: t in [ktile*128, last key + window - 1]
  const int qt_lo = ktile * 4;
  const int t_last = p.window > 0 ? min(p.T - 1, ktile * 128 + 127 + p.window - 1) : p.T - 1;
  const int qt_hi = t_last / 32;
  const int nqt = qt_hi - qt_lo + 1;
  const int wave_t_hi = p.window > 0 ? sk0 + 31 + p.window - 1 : p.T - 1;   // last query that sees a key of this wave

  v16f kacc[HD / 32], vacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) { kacc[dt][r] = 0.f; vacc[dt][r] = 0.f; }

  const int niter = group * nqt;
  v4f pq[IO::PER], pg[IO::PER];
  float pstat = 0.f;
  auto prefetch = [&](int it) {
    int hh = it / nqt, qt = qt_lo + it % nqt;
    int h = kvh * group + hh;
    const float *qb = q + (size_t)b * p.T * qstr + (size_t)h * HD;
    const float *gb = go + (size_t)b * p.T * qstr + (size_t)h * HD;
    IO::load(pq, qb, qstr, qt * 32, p.T, tid);
    IO::load(pg, gb, qstr, qt * 32, p.T, tid);
    if (tid < 64) {
      int tt = qt * 32 + (tid % 32);
      size_t si = ((size_t)b * p.Hq + h) * p.T + tt;
      pstat = tt < p.T ? (tid < 32 ? lse[si] : Dr[si]) : 0.f;
    }
  };
  prefetch(0);
  for (int it = 0; it < niter; it++) {
    __syncthreads();
    IO::store(pq, sQ, tid);
    IO::store(pg, sG, tid);
    if (tid < 32) sL[tid] = pstat;
    else if (tid < 64) sD[tid - 32] = pstat;
    __syncthreads();
    if (it + 1 < niter) prefetch(it + 1);
    const int t0 = (qt_lo + it % nqt) * 32;
    if (t0 + 31 < sk0 || t0 > wave_t_hi || sk0 >= p.T) continue;      // wave-uniform: no (query, key) pair of this tile is live
    v16f sc = tile_dot_regs<HD>(sQ, kreg, l32, g);
    v16f dp = tile_dot_regs<HD>(sG, vreg, l32, g);
    float pr[16], ds[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int ql = acc_row(r, g), tq = t0 + ql;
      bool ok = sv && tq < p.T && s <= tq && (p.window == 0 || s + p.window > tq);
      pr[r] = ok ? exp2f(sc[r] - sL[ql]) : 0.f;
      ds[r] = pr[r] * (dp[r] - sD[ql]) * p.scale;
    }
    tile_t_dot_acc<HD>(vacc, sG, pr, l32, g);
    tile_t_dot_acc<HD>(kacc, sQ, ds, l32, g);
  }
  if (sv) {
    store_row<HD>(dk + koff, kacc, g, 1.0f, acc_k);
    store_row<HD>(dv + koff, vacc, g, 1.0f, acc_v);
  }
}

int attn_mfma_supported(int hd) { return hd == 64; }

int attn_fwd_mfma(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse) {
  GT_REQUIRE(ctx, (q | k | v | out) % 16 == 0, "attention: buffers must be 16-byte aligned");
  dim3 grid((unsigned)cdiv(p.T, 128), p.Hq, p.B);
  hipLaunchKernelGGL((attn_fwd_mfma_k<64>), grid, dim3(256), 0, ctx->stream, p, P<const float>(q), P<const float>(k),
                     P<const float>(v), P<float>(out), P<float>(lse));
  GT_LAUNCHED(ctx);
  return 0;
}

int attn_bwd_mfma(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr, gt_buf dq,
                  int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v) {
  GT_REQUIRE(ctx, (q | k | v | dout | dq | dk | dv) % 16 == 0, "attention: buffers must be 16-byte aligned");
  {
    ProfScope ps(ctx, "attention.bwd.dq");
    dim3 grid((unsigned)cdiv(p.T, 128), p.Hq, p.B);
    hipLaunchKernelGGL((attn_bwd_dq_mfma_k<64>), grid, dim3(256), 0, ctx->stream, p, P<const float>(q), P<const float>(k),
                       P<const float>(v), P<const float>(dout), P<const float>(lse), Dr, P<float>(dq), acc_q);
    GT_LAUNCHED(ctx);
  }
  {
    ProfScope ps(ctx, "attention.bwd.dkv");
    dim3 grid((unsigned)cdiv(p.T, 128), p.Hkv, p.B);
    hipLaunchKernelGGL((attn_bwd_dkv_mfma_k<64>), grid, dim3(256), 0, ctx->stream, p, P<const float>(q), P<const float>(k),
                       P<const float>(v), P<const float>(dout), P<const float>(lse), Dr, P<float>(dk), acc_k, P<float>(dv), acc_v);
    GT_LAUNCHED(ctx);
  }
  return 0;
}
