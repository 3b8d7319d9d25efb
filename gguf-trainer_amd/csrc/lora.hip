// Rank-r products of the LoRA linear (autograd.ts:311-319 composes them from three `linear` calls): with r = 16 they
// are one pass over a [rows, K] activation or gradient and almost no arithmetic, so they are written as streaming
// kernels around v_mfma_f32_16x16x4_f32, whose 16-wide tile IS the rank, instead of going through the 32x32 GEMM
// tiles with three quarters of every tile empty.
//
//   gt_rank_down:  h[rows, r]  = alpha * x[rows, K] . s^T     (h = x.A^T with s = A [r, K]; dh = g.B with s = B [K, r])
//   gt_rank_grad:  p (+)= h^T . y  as [r, K]                   (dA = dh^T.x)
//                  p (+)= y^T . h  as [K, r]                   (dB = g^T.h)
//
// Operand mapping. A 16x16x4 step takes A[i = lane%16][k = lane/16] and B[k = lane/16][j = lane%16]. The order in which
// the contraction index is consumed is free as long as both operands agree, so lane group kq = lane/16 takes
// k = 4*kq + s at step s of a run of four: its four values are contiguous in a k-contiguous operand and come from one
// 16-byte load. Accumulator register q of a lane is D[4*(lane/16) + q][lane%16].
//
// Both kernels read every element of the large operand exactly once, straight from global memory into MFMA operand
// registers (no LDS staging), several loads ahead. Sums over wavefronts and over row slices have a fixed order.
#include <algorithm>
#include <cstring>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));

#define RD_WAVES 8          // wavefronts of a rank_down workgroup: each takes every 8th run of 16 k
#define RG_WAVES 4          // wavefronts of a rank_grad workgroup: each takes every 4th block of 16 rows
#define RG_COLS 64          // columns of y per rank_grad workgroup (four interleaved 16-wide tiles)

// h[row0 .. row0+16) = alpha * x . s^T. NR = number of 16-wide rank tiles (r <= 16*NR). SK: s is [K, r] (else [r, K]).
template <int NR, bool SK>
__global__ __launch_bounds__(RD_WAVES * 64) void rank_down_k(int rows, int K, int r, const float *__restrict__ x,
                                                             const float *__restrict__ s, float alpha, float *__restrict__ h) {
  __shared__ float red[RD_WAVES][NR][4][64];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l16 = lane % 16, kq = lane / 16;
  const int row0 = blockIdx.x * 16;
  const float *xr = x + (size_t)min(row0 + l16, rows - 1) * K + 4 * kq;     // a row past the end re-reads the last one
  v4f acc[NR];
#pragma unroll
  for (int t = 0; t < NR; t++) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};
  const int nrun = K / 16;
  constexpr int U = 4;                                                        // runs in flight per wavefront
  for (int run0 = wave; run0 < nrun; run0 += RD_WAVES * U) {
    v4f xv[U], sv[U][NR];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int run = min(run0 + u * RD_WAVES, nrun - 1);
      const int k = run * 16;
      xv[u] = *reinterpret_cast<const v4f *>(xr + k);
#pragma unroll
      for (int t = 0; t < NR; t++) {
        const int j = min(16 * t + l16, r - 1);
        if (!SK) sv[u][t] = *reinterpret_cast<const v4f *>(s + (size_t)j * K + k + 4 * kq);
        else {
          const float *sp = s + (size_t)(k + 4 * kq) * r + j;
          sv[u][t] = v4f{sp[0], sp[r], sp[2 * r], sp[3 * r]};
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (run0 + u * RD_WAVES >= nrun) continue;                              // wave-uniform
#pragma unroll
      for (int t = 0; t < NR; t++)
#pragma unroll
        for (int q = 0; q < 4; q++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u][q], sv[u][t][q], acc[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < NR; t++)
#pragma unroll
    for (int q = 0; q < 4; q++) red[wave][t][q][lane] = acc[t][q];
  __syncthreads();
  // element (t, q, lane) of the tile: row 4*(lane/16) + q, rank column 16*t + lane%16; summed over wavefronts in order
  for (int e = threadIdx.x; e < NR * 256; e += RD_WAVES * 64) {
    const int t = e / 256, q = (e / 64) % 4, ln = e % 64;
    float sum = red[0][t][q][ln];
#pragma unroll
    for (int w = 1; w < RD_WAVES; w++) sum += red[w][t][q][ln];
    const int row = row0 + 4 * (ln / 16) + q, j = 16 * t + ln % 16;
    if (row < rows && j < r) h[(size_t)row * r + j] = alpha * sum;
  }
}

// Partial of p over the row range of blockIdx.y, for the RG_COLS columns of blockIdx.x: out[j][col] = sum_rows h[row][j] * y[row][col].
// TR: store as [K, r] instead of [r, K]. part != nullptr: write the partial of this row slice to part[slice][...] (same
// layout as p); else store / accumulate into p directly (one slice).
template <int NR, bool TR>
__global__ __launch_bounds__(RG_WAVES * 64) void rank_grad_k(int rows, int K, int r, int rows_per_slice, const float *__restrict__ hm,
                                                             const float *__restrict__ y, float *p, int accp, float *__restrict__ part) {
  __shared__ float red[RG_WAVES][NR][4][4][64];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, l16 = lane % 16, kq = lane / 16;
  const int c0 = blockIdx.x * RG_COLS;
  const int rbeg = blockIdx.y * rows_per_slice, rend = min(rows, rbeg + rows_per_slice);
  v4f acc[NR][4];
#pragma unroll
  for (int t = 0; t < NR; t++)
#pragma unroll
    for (int n = 0; n < 4; n++) acc[t][n] = v4f{0.f, 0.f, 0.f, 0.f};
  int jc[NR];
#pragma unroll
  for (int t = 0; t < NR; t++) jc[t] = min(16 * t + l16, r - 1);
  constexpr int U = 2;                                        // 16-row blocks in flight per wavefront
  for (int rb0 = rbeg + 16 * wave; rb0 < rend; rb0 += 16 * RG_WAVES * U) {
    v4f yv[U][4];
    float hv[U][NR][4];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int rb = rb0 + u * 16 * RG_WAVES;
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int row = min(rb + 4 * kq + q, rows - 1);        // clamped: its h value is zeroed below when out of range
        yv[u][q] = *reinterpret_cast<const v4f *>(y + (size_t)row * K + c0 + 4 * l16);
#pragma unroll
        for (int t = 0; t < NR; t++) hv[u][t][q] = hm[(size_t)row * r + jc[t]];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int rb = rb0 + u * 16 * RG_WAVES;
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const bool live = rb + 4 * kq + q < rend;
#pragma unroll
        for (int t = 0; t < NR; t++) {
          const float a = live ? hv[u][t][q] : 0.f;
#pragma unroll
          for (int n = 0; n < 4; n++) acc[t][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, yv[u][q][n], acc[t][n], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < NR; t++)
#pragma unroll
    for (int n = 0; n < 4; n++)
#pragma unroll
      for (int q = 0; q < 4; q++) red[wave][t][n][q][lane] = acc[t][n][q];
  __syncthreads();
  // element (t, n, q, lane): rank row j = 16*t + 4*(lane/16) + q, column c0 + 4*(lane%16) + n
  float *dst = part ? part + (size_t)blockIdx.y * r * K : p;
  const bool add = part ? false : accp != 0;
  for (int e = threadIdx.x; e < NR * 1024; e += RG_WAVES * 64) {
    const int t = e / 1024, n = (e / 256) % 4, q = (e / 64) % 4, ln = e % 64;
    float sum = red[0][t][n][q][ln];
#pragma unroll
    for (int w = 1; w < RG_WAVES; w++) sum += red[w][t][n][q][ln];
    const int j = 16 * t + 4 * (ln / 16) + q, col = c0 + 4 * (ln % 16) + n;
    if (j < r) {
      float *o = dst + (TR ? (size_t)col * r + j : (size_t)j * K + col);
      *o = add ? *o + sum : sum;
    }
  }
}

// p (+)= sum over slices, in slice order
__global__ __launch_bounds__(256) void rank_slices_sum(const float *__restrict__ part, int slices, int n, float *p, int accp) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = part[i];
  for (int z = 1; z < slices; z++) s += part[(size_t)z * n + i];
  p[i] = accp ? p[i] + s : s;
}

// The slice sums of several rank gradients as one launch (the adapter gradients of a whole backward pass are not read
// before the optimizer, so their sums can wait and go out together): workgroup -> (entry, block of 256 elements) through
// the table in the kernel arguments, then rank_slices_sum's arithmetic, so every gradient has the bits its own launch gives.
#define RSG_MAX 96
struct RsEntry { const float *part; float *p; int slices, n, acc, blk0; };
struct RsGroup { RsEntry e[RSG_MAX]; int n; };
__global__ __launch_bounds__(256) void rank_slices_group_k(RsGroup G) {
  int i = 0;
  for (int q = 1; q < G.n; q++) if ((int)blockIdx.x >= G.e[q].blk0) i = q;
  const RsEntry &e = G.e[i];
  const int k = ((int)blockIdx.x - e.blk0) * 256 + threadIdx.x;
  if (k >= e.n) return;
  float s = e.part[k];
  for (int z = 1; z < e.slices; z++) s += e.part[(size_t)z * e.n + k];
  e.p[k] = e.acc ? e.p[k] + s : s;
}

// how the streaming rank-gradient kernel cuts `rows`: slices of rows_per_slice rows (a whole number of workgroup passes)
static int rank_grad_cut(gt_ctx *ctx, int rows, int K, int *rows_per_slice) {
  const int colblocks = K / RG_COLS;
  const int pass = 16 * RG_WAVES * 2;
  int slices = (int)std::max<int64_t>(1, std::min<int64_t>(cdiv(3 * ctx->num_cu, colblocks), cdiv(rows, pass)));
  *rows_per_slice = (int)(cdiv(cdiv(rows, slices), pass) * pass);
  return (int)cdiv(rows, *rows_per_slice);
}
static bool rank_grad_streams(int K, int r, gt_buf y) { return !(r > 32 || K % RG_COLS != 0 || y % 16 != 0); }

extern "C" {

int gt_rank_down(gt_ctx *ctx, int rows, int K, int r, gt_buf x, gt_buf s, int s_kmajor, float alpha, gt_buf h) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && K >= 1 && r >= 1 && x && s && h, "gt_rank_down: bad arguments (rows %d, K %d, r %d)", rows, K, r);
  if (r > 32 || K % 16 != 0 || (x | s) % 16 != 0) {
    // any other shape: the general GEMM, then the scale
    if (gt_gemm(ctx, s_kmajor ? GT_NN : GT_NT, 0, rows, r, K, x, s, h)) return 1;
    return alpha == 1.0f ? 0 : gt_scale_fwd(ctx, (int64_t)rows * r, h, alpha, h);
  }
  ProfScope ps(ctx, "rank.down", 4.0 * ((double)rows * K + (double)rows * r));
  dim3 grid((unsigned)cdiv(rows, 16)), block(RD_WAVES * 64);
#define GO(NR, SK) hipLaunchKernelGGL((rank_down_k<NR, SK>), grid, block, 0, ctx->stream, rows, K, r, P<const float>(x), P<const float>(s), alpha, P<float>(h))
  if (r <= 16) { if (s_kmajor) GO(1, true); else GO(1, false); }
  else { if (s_kmajor) GO(2, true); else GO(2, false); }
#undef GO
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_rank_grad(gt_ctx *ctx, int rows, int K, int r, gt_buf h, gt_buf y, int transpose_out, int acc, gt_buf p) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && K >= 1 && r >= 1 && h && y && p, "gt_rank_grad: bad arguments (rows %d, K %d, r %d)", rows, K, r);
  if (!rank_grad_streams(K, r, y)) {
    return transpose_out ? gt_gemm(ctx, GT_TN, acc, K, r, rows, y, h, p) : gt_gemm(ctx, GT_TN, acc, r, K, rows, h, y, p);
  }
  ProfScope ps(ctx, "rank.grad", 4.0 * ((double)rows * K + (double)rows * r));
  // enough row slices to give every CU a few workgroups; a slice is a whole number of passes of the workgroup
  const int colblocks = K / RG_COLS;
  int rows_per_slice;
  const int slices = rank_grad_cut(ctx, rows, K, &rows_per_slice);
  float *part = nullptr;
  if (slices > 1) {
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)slices * r * K * sizeof(float), &ws)) return 1;
    part = static_cast<float *>(ws);
  }
  dim3 grid((unsigned)colblocks, (unsigned)slices), block(RG_WAVES * 64);
#define GO(NR, TR) hipLaunchKernelGGL((rank_grad_k<NR, TR>), grid, block, 0, ctx->stream, rows, K, r, rows_per_slice, P<const float>(h), P<const float>(y), P<float>(p), acc, part)
  if (r <= 16) { if (transpose_out) GO(1, true); else GO(1, false); }
  else { if (transpose_out) GO(2, true); else GO(2, false); }
#undef GO
  GT_LAUNCHED(ctx);
  if (part) {
    const int n = r * K;
    hipLaunchKernelGGL(rank_slices_sum, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, ctx->stream, part, slices, n, P<float>(p), acc);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

int gt_rank_grad_slices(gt_ctx *ctx, int rows, int K, int r, gt_buf y, int *slices) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && K >= 1 && r >= 1 && slices, "gt_rank_grad_slices: bad arguments (rows %d, K %d, r %d)", rows, K, r);
  int rps;
  const int n = rank_grad_streams(K, r, y) ? rank_grad_cut(ctx, rows, K, &rps) : 0;
  *slices = n > 1 ? n : 0;          // one slice is written straight to its destination: nothing to hold back
  return 0;
}

int gt_rank_grad_parts(gt_ctx *ctx, int rows, int K, int r, gt_buf h, gt_buf y, int transpose_out, gt_buf parts) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 1 && K >= 1 && r >= 1 && h && y && parts, "gt_rank_grad_parts: bad arguments (rows %d, K %d, r %d)", rows, K, r);
  GT_REQUIRE(ctx, rank_grad_streams(K, r, y), "gt_rank_grad_parts: this shape does not take the streaming kernel (ask gt_rank_grad_slices first)");
  int rows_per_slice;
  const int slices = rank_grad_cut(ctx, rows, K, &rows_per_slice);
  GT_REQUIRE(ctx, slices > 1, "gt_rank_grad_parts: a single slice has no partial sums (ask gt_rank_grad_slices first)");
  ProfScope ps(ctx, "rank.grad", 4.0 * ((double)rows * K + (double)rows * r));
  dim3 grid((unsigned)(K / RG_COLS), (unsigned)slices), block(RG_WAVES * 64);
#define GO(NR, TR) hipLaunchKernelGGL((rank_grad_k<NR, TR>), grid, block, 0, ctx->stream, rows, K, r, rows_per_slice, P<const float>(h), P<const float>(y), (float *)nullptr, 0, P<float>(parts))
  if (r <= 16) { if (transpose_out) GO(1, true); else GO(1, false); }
  else { if (transpose_out) GO(2, true); else GO(2, false); }
#undef GO
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_rank_slices_group(gt_ctx *ctx, int n, const gt_buf *parts, const int *slices, const int *len, const gt_buf *p, const int *acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && (n == 0 || (parts && slices && len && p && acc)), "gt_rank_slices_group: %d entries or a null table", n);
  for (int i0 = 0; i0 < n; i0 += RSG_MAX) {
    RsGroup G;
    memset(&G, 0, sizeof G);
    G.n = std::min(RSG_MAX, n - i0);
    int blocks = 0;
    for (int q = 0; q < G.n; q++) {
      const int i = i0 + q;
      GT_REQUIRE(ctx, parts[i] && p[i] && slices[i] >= 1 && len[i] >= 1, "gt_rank_slices_group: entry %d is malformed", i);
      for (int j = i0; j < i; j++) GT_REQUIRE(ctx, p[j] != p[i], "gt_rank_slices_group: entries %d and %d write the same gradient", j, i);
      G.e[q] = {P<const float>(parts[i]), P<float>(p[i]), slices[i], len[i], acc[i], blocks};
      blocks += (int)cdiv(len[i], 256);
    }
    ProfScope ps(ctx, "rank.slices");
    hipLaunchKernelGGL(rank_slices_group_k, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, G);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

}  // extern "C"
