// FP32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32), the contraction behind
// linear forward (NT), dX = dY.W (NN) and dW = dY^T.X (TN), the chunked-CE readout and the
// Newton-Schulz products. Replaces srcGemm (src/backend/wgsl.ts:87-196).
//
// Two kernels share the tile shapes and the epilogue. gemm_direct (aligned shapes: K a multiple of 32, whole 16-byte
// chunks along every operand's contiguous index) brings operand tiles from global memory straight into LDS, double
// buffered, one barrier per K step; it is described where it is defined. gemm_kernel, described here, stages them
// through registers and takes every shape (two-segment products with a long or odd second segment included).
//
// Shape of the kernel. A workgroup of WM x WN wavefronts owns a BM x BN tile of C and walks K in
// steps of 16 or 32. Each wavefront owns a (BM/WM) x (BN/WN) sub-tile as TM x TN MFMA tiles of 32x32,
// 16 accumulator VGPRs each. Global loads for step i+1 are issued into registers before the
// MFMAs of step i and stored to LDS after them, so HBM/L2 latency hides under 32+ MFMAs.
//
// LDS layout. Every operand tile is kept as [row][BK+4] so that a lane fetches its MFMA inputs for
// four consecutive steps with one ds_read_b128. An operand whose K index is contiguous in memory
// (A of NT/NN, B of NT) is copied float4 for float4; one whose row index is contiguous (A of TN,
// B of NN/TN) is transposed on the way in (see Tile). Because an MFMA step consumes K pairs
// (lane/32 selects which), the order in which K is consumed is free as long as A and B agree:
// inside every run of 8, lane group g takes k = 4g + i at step i, which is what lets the b128
// fetch feed four steps.
//
// dW has a small output and a long K (rows of the batch), so it is split along K over blockIdx.z
// into per-split partial tiles in the workspace, summed in split order by a second kernel: no
// atomics, bit-identical from run to run.
#include <algorithm>
#include "common.h"

#include "gemm_tile.h"

// C_i (+)= sum over splits of the group's partials, in split order; one thread per output element of the whole group
__global__ __launch_bounds__(256) void group_reduce(GroupArgs g, const float *__restrict__ Pp, int64_t total, int splits) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  int i = 0;
#pragma unroll
  for (int q = 1; q < GT_GROUP_MAX; q++) if (q < g.n && e >= g.p[q].e0) i = q;
  const GroupProb &p = g.p[i];
  const int64_t n = (int64_t)p.M * p.N, l = e - p.e0;
  const float *pp = Pp + (size_t)splits * p.e0 + l;
  float s = pp[0];
  for (int z = 1; z < splits; z++) s += pp[(size_t)z * n];
  p.C[l] = p.acc ? p.C[l] + s : s;
}

template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2>
static int launch_direct_kind(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {       // once per context (device): more LDS than a kernel gets by default
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, SEG2>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, SEG2>), dim3(a.nbm * a.nbn, 1, zdim), dim3(WM * WN * 64), smem, ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}
// slot: index of the tile shape (0..5); the bit of (shape, kind, one or two segments) in gemm_direct_set follows from it
template <int BM, int BN, int WM, int WN, int BK, int NSTG>
static int launch_direct(gt_ctx *ctx, int kind, GemmArgs &a, int zdim, int slot) {
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  const int b1 = slot < 5 ? 3 * slot : 45 + 3 * (slot - 5), b2 = slot < 5 ? 15 + 2 * slot : 54 + 2 * (slot - 5);
  if (a.K2 > 0) {                // two K segments: NT / NN only
    if (kind == GT_NT) return launch_direct_kind<BM, BN, WM, WN, GT_NT, BK, NSTG, true>(ctx, a, zdim, b2);
    return launch_direct_kind<BM, BN, WM, WN, GT_NN, BK, NSTG, true>(ctx, a, zdim, b2 + 1);
  }
  if (kind == GT_NT) return launch_direct_kind<BM, BN, WM, WN, GT_NT, BK, NSTG, false>(ctx, a, zdim, b1);
  if (kind == GT_NN) return launch_direct_kind<BM, BN, WM, WN, GT_NN, BK, NSTG, false>(ctx, a, zdim, b1 + 1);
  return launch_direct_kind<BM, BN, WM, WN, GT_TN, BK, NSTG, false>(ctx, a, zdim, b1 + 2);
}

// C (+)= sum over splits, in split order
__global__ __launch_bounds__(256) void splitk_reduce(const float *__restrict__ Pp, float *__restrict__ C, int64_t n,
                                                     int splits, int acc, const float *__restrict__ D, int scaled, float dscale,
                                                     float pscale) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = Pp[i];
  for (int z = 1; z < splits; z++) s += Pp[(size_t)z * n + i];
  C[i] = D ? (scaled ? dscale * D[i] + pscale * s : D[i] + s) : acc ? C[i] + s : s;
}

template <int BM, int BN, int WM, int WN, int BKT>
static int launch_cfg(gt_ctx *ctx, int kind, bool vec, GemmArgs &a, int zdim) {
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  dim3 grid(a.nbm * a.nbn, 1, zdim), block(WM * WN * 64);
#define GO(KIND, VEC) hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, BKT, KIND, VEC>), grid, block, 0, ctx->stream, a)
#define GO2(KIND) hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, BKT, KIND, true, true>), grid, block, 0, ctx->stream, a)
  if (a.K2 > 0) {                // two K segments: aligned NT / NN only (gemm_impl sends everything else as two launches)
    if (kind == GT_NT) GO2(GT_NT); else GO2(GT_NN);
  }
  else if (kind == GT_NT) { if (vec) GO(GT_NT, true); else GO(GT_NT, false); }
  else if (kind == GT_NN) { if (vec) GO(GT_NN, true); else GO(GT_NN, false); }
  else { if (vec) GO(GT_TN, true); else GO(GT_TN, false); }
#undef GO2
#undef GO
  GT_LAUNCHED(ctx);
  return 0;
}

static int reduce_splits(gt_ctx *ctx, const GemmArgs &a, int M, int N, int splits, int acc) {
  if (splits > 1) {
    int64_t n = (int64_t)M * N;
    hipLaunchKernelGGL(splitk_reduce, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, ctx->stream, a.Pp, a.C, n, splits, acc, a.D, a.scaled, a.dscale, a.pscale);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

struct TileCfg { int bm, bn, bk; };
static const TileCfg kTiles[] = {{64, 64, 16}, {128, 64, 16}, {128, 128, 16}, {128, 192, 16}, {128, 96, 16}, {256, 128, 16},
                                 {128, 128, 32}, {128, 192, 32}, {128, 96, 32}, {256, 128, 32}, {64, 192, 16}, {128, 64, 32}, {64, 192, 32}, {128, 160, 32}};
#define NCFG ((int)(sizeof(kTiles) / sizeof(kTiles[0])))

// Tile and split-K choice by a small cost model over the tile shapes that measured best on MI355X:
// time ~ flops / (tile efficiency x edge utilisation x wave quantisation) + the cost of the split-K reduction pass,
// for one product (batched `count` times) or a group of `np` products with a common K launched together.
struct Cand { int cfg; double eff; };
static void pick_tile(gt_ctx *ctx, int kind, bool direct_ok, int np, const int *Ms, const int *Ns, int K, int count, bool two_seg,
                      int *cfg_out, int *splits_out, int fixed_splits = 0, int only_cfg = -1) {
  // relative tile efficiencies as measured (asymptotic rate of each tile over the best one's)
  static const Cand cand_nn[] = {{7, 1.00}, {6, 0.98}, {8, 0.98}, {10, 0.95}, {11, 0.82}, {0, 0.78}};
  static const Cand cand_tn[] = {{8, 1.00}, {11, 0.99}, {10, 0.92}, {6, 0.90}, {7, 0.78}, {0, 0.72}};
  static const Cand cand_nn_direct[] = {{7, 1.00}, {8, 1.00}, {13, 1.00}, {6, 0.98}, {12, 0.97}, {11, 0.92}, {10, 0.85}, {0, 0.72}};
  static const Cand cand_tn_direct[] = {{8, 1.00}, {12, 1.00}, {13, 0.99}, {7, 0.98}, {11, 0.96}, {6, 0.88}, {10, 0.85}, {0, 0.68}};
  const Cand *cand = direct_ok ? (kind == GT_TN ? cand_tn_direct : cand_nn_direct) : (kind == GT_TN ? cand_tn : cand_nn);
  const int ncand = direct_ok ? 8 : 6;
  int cfg = 0, splits = 1;
  double elems = 0;
  for (int i = 0; i < np; i++) elems += (double)Ms[i] * Ns[i];
  const double flops = 2.0 * elems * K * count;
  const double t0 = flops / (direct_ok ? 132e12 : 125e12);   // seconds at the best tile's asymptotic rate
  double best = 1e30;
  for (int ci = 0; ci < ncand; ci++) {
    const Cand &c = cand[ci];
    const TileCfg &tc = kTiles[c.cfg];
    if (only_cfg >= 0 && c.cfg != only_cfg) continue;
    if (np > 1 && !(c.cfg == 6 || c.cfg == 7 || c.cfg == 8 || c.cfg == 11 || c.cfg == 12 || c.cfg == 13)) continue;   // group launches: direct tiles only
    int64_t tiles = 0;
    for (int i = 0; i < np; i++) tiles += cdiv(Ms[i], tc.bm) * cdiv(Ns[i], tc.bn);
    const double util = elems / ((double)tiles * tc.bm * tc.bn);
    // any split count, not only powers of two: 72 output tiles x 14 splits is 3.94 workgroups per CU, x 16 is 4.5,
    // and with workgroups of equal length the CUs that get the fifth one set the time
    for (int sp = fixed_splits > 0 ? fixed_splits : 1; sp <= (fixed_splits > 0 ? fixed_splits : 64); sp++) {
      // split only when the output tiles alone cannot give every CU a workgroup (a group's split count is given)
      if (!fixed_splits && sp > 1 && (count > 1 || two_seg || tiles >= ctx->num_cu || K / sp < 8 * tc.bk)) break;
      const double waves = (double)tiles * sp * count / ctx->num_cu;
      const double quant = waves / ceil(waves);
      // a CU with few workgroups over the whole launch overlaps their fills and write-backs less (fitted on the
      // dW shapes: 1 workgroup per CU runs 15 % and 2 run 6 % below the rate reached from 4 per CU on)
      const double conc = std::min(1.0, 1.0625 * waves / (waves + 0.25));
      // short K per workgroup pays the prologue/epilogue more: ~2 K-steps of overhead
      const double ksteps = (double)K / sp / tc.bk;
      const double depth = ksteps / (ksteps + 2.0);
      double t = t0 / (c.eff * util * quant * depth * conc);
      if (sp > 1) t += ((double)(sp + 2) * elems * 4.0) / 3.5e12 + 4e-6;
      if (t < best) { best = t; cfg = c.cfg; splits = sp; }
    }
  }
  *cfg_out = cfg;
  *splits_out = splits;
}

static int gemm_impl(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, int64_t sA, gt_buf B, int64_t sB,
                     gt_buf C, int64_t sC, int count, int K2 = 0, gt_buf A2 = 0, gt_buf B2 = 0, gt_buf D = 0, int64_t sD = 0,
                     int scaled = 0, float dscale = 1.f, float pscale = 1.f) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2, "gt_gemm: kind %d is not NT(0)/NN(1)/TN(2)", kind);
  GT_REQUIRE(ctx, M >= 1 && N >= 1 && K >= 1 && count >= 1, "gt_gemm: M,N,K,count must be >= 1 (got %d,%d,%d,%d)", M, N, K, count);
  GT_REQUIRE(ctx, A && B && C, "gt_gemm: null operand");
  GemmArgs a;
  a.A = P<const float>(A); a.B = P<const float>(B); a.C = P<float>(C);
  a.M = M; a.N = N; a.K = K;
  a.lda = (kind == GT_TN) ? M : K;
  a.ldb = (kind == GT_NT) ? K : N;
  a.ldc = N;
  a.acc = acc; a.kchunk = K; a.splits = 1; a.Pp = nullptr;
  a.sA = sA; a.sB = sB; a.sC = sC;
  a.zdiv = a.zgroup = 1; a.window = 0; a.sB2 = a.sC2 = 0; a.nx = 0; a.D = P<const float>(D);
  a.sD = sD; a.scaled = scaled; a.dscale = dscale; a.pscale = pscale; a.rope = nullptr;
  GT_REQUIRE(ctx, !D || K2 == 0, "gt_gemm_add: single-segment products only");
  GT_REQUIRE(ctx, !scaled || D, "scaled write-back needs the matrix it combines the product with");
  bool vec = (a.lda % 4 == 0) && (a.ldb % 4 == 0) && (A % 16 == 0) && (B % 16 == 0) &&
             (sA % 4 == 0) && (sB % 4 == 0);
  a.K2 = K2; a.A2 = P<const float>(A2); a.B2 = P<const float>(B2);
  a.lda2 = (kind == GT_TN) ? M : K2;
  a.ldb2 = (kind == GT_NT) ? K2 : N;
  if (K2 > 0) vec = vec && (a.lda2 % 4 == 0) && (a.ldb2 % 4 == 0) && (A2 % 16 == 0) && (B2 % 16 == 0);

  // Tile and split-K choice: pick_tile. N = 576 (SmolLM2) is 3x192 = 6x96; dW has a 1536x576 output and
  // K = 16384 rows, which only fills 256 CUs when K is split.
  // Tiles with a K step of 32 have a variant that loads operands straight into LDS (gemm_direct); it wants whole K
  // steps and whole 16-byte chunks along the contiguous index of every operand. Where it applies it is 2-8 % faster
  // than the register-staged kernel of the same tile and changes which tile is best, hence two tables.
  // a lane's byte offset inside a tile (up to 192 rows of ld floats) must fit the 32 bits the direct kernels keep it in
  const bool direct_ok = vec && K % 32 == 0 && (kind != GT_TN || (M % 4 == 0 && M >= 4)) && (kind == GT_NT || (N % 4 == 0 && N >= 4)) &&
                         std::max(std::max(a.lda, a.ldb), K2 > 0 ? std::max(a.lda2, a.ldb2) : 0) <= GT_DIRECT_LD_MAX &&
                         (K2 == 0 || (kind != GT_TN && K2 % 8 == 0 && K2 <= 32));   // a short second segment rides in one more stage
  int cfg = 0, splits = 1;
  // "gemm.split_bf16": every product the direct kernels take runs on the bf16 MFMA instead, on 128 x 192 or 128 x 128 tiles
  const bool split = direct_ok && ctx->opt_gemm_split && (K2 == 0 || K2 == 16 || K2 == 32) && !ctx->opt_gemm_staged;
  const bool wide = N % 192 == 0;
  pick_tile(ctx, kind, direct_ok, 1, &M, &N, K, count, K2 > 0, &cfg, &splits, 0, split ? (wide ? 7 : 6) : -1);
  if (!split && ctx->opt_gemm_tile >= 0 && ctx->opt_gemm_tile < NCFG) cfg = ctx->opt_gemm_tile;
  const int bm = kTiles[cfg].bm, bn = kTiles[cfg].bn, bk = kTiles[cfg].bk;
  if (count == 1 && K2 == 0 && ctx->opt_gemm_splitk >= 1) splits = ctx->opt_gemm_splitk;
  if (splits > 1) {
    int64_t kc = cdiv(cdiv(K, splits), bk) * bk;
    splits = (int)cdiv(K, kc);
    a.kchunk = (int)kc;
  }
  if (splits > 1) {
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)splits * M * N * sizeof(float), &ws)) return 1;
    a.splits = splits; a.Pp = static_cast<float *>(ws);
  }
  int zdim = splits > 1 ? splits : count;
  char label[32];
  snprintf(label, sizeof label, "gemm.%s.%dx%dx%d%s%s", kind == GT_NT ? "nt" : kind == GT_NN ? "nn" : "tn", bm, bn, split ? 32 : bk,
           split ? ".bf16x6" : "", splits > 1 ? ".splitk" : "");
  ProfScope ps(ctx, label, 2.0 * M * N * ((double)K + K2) * count);
  int rc;
  if (split) return gemm_split_launch(ctx, kind, wide, false, a, zdim) || reduce_splits(ctx, a, M, N, splits, acc);
  if (direct_ok && !ctx->opt_gemm_staged) {
    switch (cfg) {
      case 6: return launch_direct<128, 128, 2, 2, 32, 2>(ctx, kind, a, zdim, 0) || reduce_splits(ctx, a, M, N, splits, acc);
      case 7: return launch_direct<128, 192, 2, 2, 32, 2>(ctx, kind, a, zdim, 1) || reduce_splits(ctx, a, M, N, splits, acc);
      case 8: return launch_direct<128, 96, 4, 1, 32, 2>(ctx, kind, a, zdim, 2) || reduce_splits(ctx, a, M, N, splits, acc);
      case 11: return launch_direct<128, 64, 2, 2, 32, 2>(ctx, kind, a, zdim, 3) || reduce_splits(ctx, a, M, N, splits, acc);
      case 12: return launch_direct<64, 192, 2, 2, 32, 2>(ctx, kind, a, zdim, 4) || reduce_splits(ctx, a, M, N, splits, acc);
      case 13: return launch_direct<128, 160, 4, 1, 32, 2>(ctx, kind, a, zdim, 5) || reduce_splits(ctx, a, M, N, splits, acc);
      default: break;
    }
  }
  switch (cfg) {
    case 0: rc = launch_cfg<64, 64, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 1: rc = launch_cfg<128, 64, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 2: rc = launch_cfg<128, 128, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 3: rc = launch_cfg<128, 192, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 4: rc = launch_cfg<128, 96, 4, 1, 16>(ctx, kind, vec, a, zdim); break;
    case 5: rc = launch_cfg<256, 128, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 6: rc = launch_cfg<128, 128, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 7: rc = launch_cfg<128, 192, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 8: rc = launch_cfg<128, 96, 4, 1, 32>(ctx, kind, vec, a, zdim); break;
    case 9: rc = launch_cfg<256, 128, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 10: rc = launch_cfg<64, 192, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 11: rc = launch_cfg<128, 64, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 13: rc = launch_cfg<128, 160, 4, 1, 32>(ctx, kind, vec, a, zdim); break;
    default: rc = launch_cfg<64, 192, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
  }
  if (rc) return rc;
  return reduce_splits(ctx, a, M, N, splits, acc);
}

// dQ[b][t][h*hd + :] (+)= sum over the keys s visible from t of dS[b*Hq + h][t][s] * K[b][s][(h/group)*hd + :] for every
// (sequence, head): one banded NN product per pair, all in one launch. dS holds B*Hq [T][T] matrices in blocks
// [row tile of 128][key step of 32][128 rows][32 keys] (what one pipeline stage loads is one contiguous 16 KB block)
// whose blocks inside each row tile's band are all written (zeros where a pair is masked); T is a multiple of 128.
// Head dim 128 runs two pipeline stages, not three: 98 KB of LDS left one workgroup per CU, 68 KB lets two stay (341 -> 318 us
// per launch at 4 x 2048 tokens of 16 heads).
template <int BN, int NSTG = 3>
static int launch_band(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int BM = 128, BK = 32, WM = 2, WN = 2;
  constexpr int smem = band_lds_bytes<BM, BN, BK, NSTG>();
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, GT_NN, BK, NSTG, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, GT_NN, BK, NSTG, false, true>), dim3(zdim, a.splits, a.nbm * a.nbn), dim3(WM * WN * 64), smem,
                     ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}

// dQ (+)= sum of the band product's split partials, in split order, rotated back where the rows are wanted before their
// rotation ((lo, hi) -> (c lo + s hi, -s lo + c hi) per pair (j, j + hd/2), the reference's srcRope backward, wgsl.ts:346-384):
// one thread per float4 of a row's low half and its partner in the high half. rows = B*T rows of Hq heads.
__global__ __launch_bounds__(256) void band_dq_reduce(const float *__restrict__ Pp, int splits, int64_t plane, float *dq, int acc,
                                                      const float *__restrict__ rot, int64_t rows, int T, int Hq, int hd) {
  const int upr = hd / 8;                                  // float4 units in the low half of a head's row
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= rows * Hq * upr) return;
  const int c4 = (int)(u % upr);
  const int64_t rh = u / upr, row = rh / Hq;
  const size_t lo = (size_t)rh * hd + 4 * c4, hi = lo + hd / 2;
  v4f a = *reinterpret_cast<const v4f *>(Pp + lo), b = *reinterpret_cast<const v4f *>(Pp + hi);
  for (int z = 1; z < splits; z++) {
    a += *reinterpret_cast<const v4f *>(Pp + (size_t)z * plane + lo);
    b += *reinterpret_cast<const v4f *>(Pp + (size_t)z * plane + hi);
  }
  if (rot) {
    const float *cs = rot + ((size_t)(row % T) * (hd / 2) + 4 * c4) * 2;
    const v4f c0 = *reinterpret_cast<const v4f *>(cs), c1 = *reinterpret_cast<const v4f *>(cs + 4);
    const v4f c = {c0[0], c0[2], c1[0], c1[2]}, sn = {c0[1], c0[3], c1[1], c1[3]};
    const v4f r0 = c * a + sn * b, r1 = -sn * a + c * b;
    a = r0;
    b = r1;
  }
  if (acc) {
    a += *reinterpret_cast<const v4f *>(dq + lo);
    b += *reinterpret_cast<const v4f *>(dq + hi);
  }
  *reinterpret_cast<v4f *>(dq + lo) = a;
  *reinterpret_cast<v4f *>(dq + hi) = b;
}

// how many parts a small launch of the banded product cuts every row tile's K range into (1: none), so that a single
// sequence's 16 row tiles per head, whose longest has 16 times the K range of the shortest, become enough workgroups of
// bounded length to fill the chip; the caller provides that many planes of B*T*Hq*hd floats
int gemm_band_dq_splits(gt_ctx *ctx, int B, int T, int Hq, int window) {
  const int64_t tiles = (int64_t)B * Hq * (T / 128);
  if (ctx->opt_attn_band_splits >= 1) return (int)std::min<int64_t>(std::min(ctx->opt_attn_band_splits, 8), std::max(1, T / 128));
  // the longest K range of a row tile: the whole sequence, or a window's band (there the tiles are short and alike: no cut)
  const int kmax = window > 0 ? std::min(T, ((window + 126) & ~127) + 128) : T;
  if (tiles >= 2 * ctx->num_cu || kmax < 1024) return 1;
  return (int)std::min<int64_t>(std::min<int64_t>(8, kmax / 256), cdiv(2 * ctx->num_cu, tiles));
}

int gemm_band_dq(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, const float *dS, const float *K, float *dQ, int acc,
                 const float *rot, float *parts, int splits) {
  GT_REQUIRE(ctx, T % 128 == 0 && (hd == 64 || hd == 128), "banded dQ product: T %d must be a multiple of 128 and hd %d 64 or 128", T, hd);
  GT_REQUIRE(ctx, ((reinterpret_cast<uintptr_t>(dS) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(dQ)) & 15) == 0,
             "banded dQ product: operands must be 16-byte aligned");
  GemmArgs a;
  a.A = dS; a.B = K; a.C = dQ;
  a.M = T; a.N = hd; a.K = T;
  a.lda = T; a.ldb = Hkv * hd; a.ldc = Hq * hd;
  GT_REQUIRE(ctx, splits >= 1 && (splits == 1 || parts), "banded dQ product: %d splits without a workspace", splits);
  a.acc = acc; a.kchunk = T; a.splits = splits; a.Pp = parts; a.sP = (int64_t)B * T * Hq * hd;
  a.sA = (int64_t)T * T; a.sB = (int64_t)T * Hkv * hd; a.sC = (int64_t)T * Hq * hd;
  a.zdiv = Hq; a.zgroup = Hq / Hkv; a.window = window; a.sB2 = hd; a.sC2 = hd;
  a.A2 = a.B2 = nullptr; a.K2 = 0; a.lda2 = a.ldb2 = 0; a.nx = 0; a.D = nullptr; a.sD = 0; a.scaled = 0; a.dscale = a.pscale = 1.f;
  a.rope = rot;
  GT_REQUIRE(ctx, !rot || (Hq * hd) % 4 == 0, "banded dQ product: rotated rows need 16-byte aligned output rows");
  GT_REQUIRE(ctx, T / 128 <= 65535, "banded dQ product: %d row tiles exceed the grid", T / 128);
  if (ctx->opt_attn_pieces) {          // "attn.split_bf16": the product on the bf16 matrix instruction
    if (gemm_split_launch_band(ctx, a, B * Hq)) return 1;
  } else if (hd == 64 ? launch_band<64>(ctx, a, B * Hq, 25) : launch_band<128, 2>(ctx, a, B * Hq, 26)) return 1;
  if (splits > 1) {
    const int64_t rows = (int64_t)B * T, units = rows * Hq * (hd / 8);
    hipLaunchKernelGGL(band_dq_reduce, dim3((unsigned)cdiv(units, 256)), dim3(256), 0, ctx->stream, parts, splits, a.sP, dQ, acc, rot, rows, T, Hq, hd);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

// C (+)= sum over i of A_i.B_i with the K segments chained in one loop (NT / NN, every K_i a multiple of 32)
template <int BM, int BN, int WM, int WN, int KIND>
static int launch_multi(gt_ctx *ctx, GemmArgs &a, int slot) {
  constexpr int BK = 32, NSTG = 2, smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, false, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, false, false, true>), dim3(a.nbm * a.nbn, 1, 1), dim3(WM * WN * 64), smem,
                     ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}

template <int BM, int BN, int WM, int WN>
static int launch_group(gt_ctx *ctx, GemmArgs &a, GroupArgs &g, int slot) {
  constexpr int BK = 32, NSTG = 2, smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_group_tn<BM, BN, WM, WN, BK, NSTG>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  int tiles = 0;
  for (int i = 0; i < g.n; i++) {
    g.p[i].tile0 = tiles;
    g.p[i].nbn = (int)cdiv(g.p[i].N, BN);
    tiles += (int)cdiv(g.p[i].M, BM) * g.p[i].nbn;
  }
  g.ntiles = tiles;
  hipLaunchKernelGGL((gemm_group_tn<BM, BN, WM, WN, BK, NSTG>), dim3((unsigned)tiles * a.splits), dim3(WM * WN * 64), smem, ctx->stream, a, g);
  GT_LAUNCHED(ctx);
  return 0;
}

extern "C" {
int gt_gemm_group(gt_ctx *ctx, int kind, int count, const int *M, const int *N, int K, const gt_buf *A, const gt_buf *B,
                  const gt_buf *C, const int *acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2 && count >= 1 && M && N && A && B && C && acc && K >= 1,
             "gt_gemm_group: kind %d, %d products, K %d, or a null table", kind, count, K);
  // What a product's result is, bit for bit, must not depend on which other products it shares a launch with (the host
  // groups what happens to be pending: with and without recomputed regions those are different sets). The tile shape
  // does not enter the arithmetic of an output element (every direct tile walks K in the same order); the K split does.
  // So the split is a function of K alone: ranges of max(512, K/8) rows, at most eight partials per output. A product
  // that fills the chip on its own (at least one 128 x 96 tile per CU) is not split and goes as its own launch.
  const int64_t big = (int64_t)ctx->num_cu * 128 * 96;
  int idx[GT_GROUP_MAX], ng = 0;
  bool eligible = kind == GT_TN && K % 32 == 0 && !ctx->opt_gemm_staged && ctx->opt_gemm_group;      // (TN: ld = M, N, below GT_DIRECT_LD_MAX for any grouped size)
  for (int i = 0; i < count; i++) {
    GT_REQUIRE(ctx, M[i] >= 1 && N[i] >= 1 && A[i] && B[i] && C[i], "gt_gemm_group: product %d has M %d, N %d or a null operand", i, M[i], N[i]);
    for (int j = 0; j < i; j++)
      GT_REQUIRE(ctx, C[i] + (uint64_t)M[i] * N[i] * 4 <= C[j] || C[j] + (uint64_t)M[j] * N[j] * 4 <= C[i],
                 "gt_gemm_group: the outputs of products %d and %d overlap", j, i);
  }
  const int pin = ctx->opt_gemm_tile;
  GT_REQUIRE(ctx, !(eligible && pin >= 0 && pin != 6 && pin != 7 && pin != 8 && pin != 11 && pin != 12 && pin != 13),
             "gt_gemm_group: \"gemm.tile\" pins tile %d, which the grouped launch does not have (6, 7, 8, 11, 12 or 13; -1 = choose)", pin);
  if (count > GT_GROUP_MAX) {
    for (int i = 0; i < count; i += GT_GROUP_MAX)
      if (gt_gemm_group(ctx, kind, std::min(GT_GROUP_MAX, count - i), M + i, N + i, K, A + i, B + i, C + i, acc + i)) return 1;
    return 0;
  }
  for (int i = 0; i < count; i++) {
    const bool fits = eligible && M[i] % 4 == 0 && N[i] % 4 == 0 && (A[i] | B[i] | C[i]) % 16 == 0 && (int64_t)M[i] * N[i] < big &&
                      M[i] <= GT_DIRECT_LD_MAX && N[i] <= GT_DIRECT_LD_MAX;
    if (fits) idx[ng++] = i;
    else if (gemm_impl(ctx, kind, acc[i], M[i], N[i], K, A[i], 0, B[i], 0, C[i], 0, 1)) return 1;
  }
  if (ng == 0) return 0;
  GemmArgs a;
  memset(&a, 0, sizeof a);
  a.K = K; a.kchunk = K; a.splits = 1; a.zdiv = a.zgroup = 1;
  GroupArgs g;
  memset(&g, 0, sizeof g);
  g.n = ng;
  int64_t elems = 0;
  int gm[GT_GROUP_MAX], gn[GT_GROUP_MAX];
  for (int q = 0; q < ng; q++) {
    const int i = idx[q];
    g.p[q].A = P<const float>(A[i]); g.p[q].B = P<const float>(B[i]); g.p[q].C = P<float>(C[i]);
    g.p[q].M = gm[q] = M[i]; g.p[q].N = gn[q] = N[i]; g.p[q].acc = acc[i]; g.p[q].e0 = elems;
    elems += (int64_t)M[i] * N[i];
  }
  int64_t kc = std::max<int64_t>(512, cdiv(cdiv(K, 8), 32) * 32);
  if (ctx->opt_gemm_splitk >= 1) kc = cdiv(cdiv(K, ctx->opt_gemm_splitk), 32) * 32;
  int splits = (int)cdiv(K, kc), cfg = 0, unused = 0;
  pick_tile(ctx, GT_TN, true, ng, gm, gn, K, 1, false, &cfg, &unused, splits);
  if (pin == 6 || pin == 7 || pin == 8 || pin == 11 || pin == 12 || pin == 13) cfg = pin;
  if (splits > 1) {
    a.kchunk = (int)kc;
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)splits * elems * sizeof(float), &ws)) return 1;
    a.splits = splits; a.Pp = static_cast<float *>(ws);
  }
  char label[32];
  bool wide = true;
  for (int q = 0; q < ng; q++) wide = wide && gn[q] % 192 == 0;
  if (ctx->opt_gemm_split) snprintf(label, sizeof label, "gemm.tn.group.128x%d.bf16x6%s", wide ? 192 : 128, splits > 1 ? ".splitk" : "");
  else snprintf(label, sizeof label, "gemm.tn.group.%dx%d%s", kTiles[cfg].bm, kTiles[cfg].bn, splits > 1 ? ".splitk" : "");
  ProfScope ps(ctx, label, 2.0 * elems * K);
  int rc;
  if (ctx->opt_gemm_split) rc = gemm_split_launch_group(ctx, wide, a, g);
  else switch (cfg) {
    case 6: rc = launch_group<128, 128, 2, 2>(ctx, a, g, 40); break;
    case 7: rc = launch_group<128, 192, 2, 2>(ctx, a, g, 41); break;
    case 8: rc = launch_group<128, 96, 4, 1>(ctx, a, g, 42); break;
    case 11: rc = launch_group<128, 64, 2, 2>(ctx, a, g, 43); break;
    case 13: rc = launch_group<128, 160, 4, 1>(ctx, a, g, 58); break;
    default: rc = launch_group<64, 192, 2, 2>(ctx, a, g, 44); break;
  }
  if (rc) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(group_reduce, dim3((unsigned)cdiv(elems, 256)), dim3(256), 0, ctx->stream, g, a.Pp, elems, splits);
    GT_LAUNCHED(ctx);
  }
  return 0;
}
}

// C_i = dscale * D_i + pscale * A_i.B_i for a batch of `count` products (strides in elements; D laid out as C)
int gemm_scaled_batched(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, int64_t sA, gt_buf B, int64_t sB, gt_buf D, int64_t sD,
                        float dscale, float pscale, gt_buf C, int64_t sC, int count) {
  return gemm_impl(ctx, kind, 0, M, N, K, A, sA, B, sB, C, sC, count, 0, 0, 0, D, sD, 1, dscale, pscale);
}

extern "C" {
int gt_gemm_sum(gt_ctx *ctx, int kind, int acc, int M, int N, int count, const int *K, const gt_buf *A, const gt_buf *B, gt_buf C) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, count >= 1 && count <= 3 && K && A && B && C, "gt_gemm_sum: 1 to 3 products with their sizes and operands (got %d)", count);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2 && M >= 1 && N >= 1, "gt_gemm_sum: kind %d, M %d, N %d", kind, M, N);
  bool fused = count > 1 && kind != GT_TN && !ctx->opt_gemm_staged && C % 16 == 0 && N % 4 == 0 && (kind == GT_NT || N >= 4);
  for (int i = 0; i < count; i++) {
    GT_REQUIRE(ctx, K[i] >= 1 && A[i] && B[i], "gt_gemm_sum: product %d has K %d or a null operand", i, K[i]);
    fused = fused && K[i] % 32 == 0 && A[i] % 16 == 0 && B[i] % 16 == 0 && K[i] <= GT_DIRECT_LD_MAX;
  }
  fused = fused && N <= GT_DIRECT_LD_MAX;
  // the chained loop has one tile shape and no K split: below one workgroup per CU the single products, which pick
  // smaller tiles and split K, fill the chip better
  // Tile of the chained loop: 128 x 96, 128 x 160 or 128 x 128, whichever leaves the least idle in edge tiles and in the
  // last round of workgroups (two are resident per CU). 576 = 6 x 96; 640 = 4 x 160: a 16384-row output is 512 tiles, one
  // full round, where 128 x 128 makes 640 tiles for 512 slots and a quarter-full second round.
  int bn_sum = 128;
  {
    double best = 0;
    const int cands[3] = {128, 160, 96};
    for (int ci = 0; ci < 3; ci++) {
      const int bn = cands[ci];
      if (bn != 128 && N % bn != 0) continue;
      const double tiles = (double)cdiv(M, 128) * cdiv(N, bn), rounds = tiles / (2.0 * ctx->num_cu);
      const double score = ((double)M * N) / (tiles * 128.0 * bn) * (rounds / ceil(rounds));
      if (score > best * 1.02) { best = score; bn_sum = bn; }
    }
  }
  const bool t96 = bn_sum == 96, t160 = bn_sum == 160;
  if (fused && cdiv(M, 128) * cdiv(N, bn_sum) < (ctx->opt_gemm_sum_min_tiles >= 0 ? ctx->opt_gemm_sum_min_tiles : ctx->num_cu)) fused = false;
  if (!fused) {        // one launch per product, each adding to the one before
    for (int i = 0; i < count; i++)
      if (gemm_impl(ctx, kind, i ? 1 : acc, M, N, K[i], A[i], 0, B[i], 0, C, 0, 1)) return 1;
    return 0;
  }
  GemmArgs a;
  a.A = P<const float>(A[0]); a.B = P<const float>(B[0]); a.C = P<float>(C);
  a.M = M; a.N = N; a.K = K[0];
  a.lda = K[0]; a.ldb = kind == GT_NT ? K[0] : N; a.ldc = N;
  a.acc = acc; a.kchunk = K[0]; a.splits = 1; a.Pp = nullptr;
  a.sA = a.sB = a.sC = 0;
  a.zdiv = a.zgroup = 1; a.window = 0; a.sB2 = a.sC2 = 0;
  a.A2 = a.B2 = nullptr; a.K2 = 0; a.lda2 = a.ldb2 = 0;
  a.nx = count - 1; a.D = nullptr; a.sD = 0; a.scaled = 0; a.dscale = a.pscale = 1.f; a.rope = nullptr;
  double ksum = K[0];
  for (int i = 1; i < count; i++) {
    a.xA[i - 1] = P<const float>(A[i]); a.xB[i - 1] = P<const float>(B[i]);
    a.xK[i - 1] = K[i]; a.xlda[i - 1] = K[i]; a.xldb[i - 1] = kind == GT_NT ? K[i] : N;
    ksum += K[i];
  }
  char label[32];
  if (ctx->opt_gemm_split) {
    snprintf(label, sizeof label, "gemm.%s.128x%dx%d.bf16x6", kind == GT_NT ? "nt" : "nn", N % 192 == 0 ? 192 : 128, 32);
    ProfScope ps(ctx, label, 2.0 * M * N * ksum);
    return gemm_split_launch(ctx, kind, N % 192 == 0, true, a, 1);
  }
  snprintf(label, sizeof label, "gemm.%s.128x%dx32", kind == GT_NT ? "nt" : "nn", bn_sum);
  ProfScope ps(ctx, label, 2.0 * M * N * ksum);
  if (kind == GT_NN)
    return t96 ? launch_multi<128, 96, 4, 1, GT_NN>(ctx, a, 30) : t160 ? launch_multi<128, 160, 4, 1, GT_NN>(ctx, a, 34)
                                                                       : launch_multi<128, 128, 2, 2, GT_NN>(ctx, a, 31);
  return t96 ? launch_multi<128, 96, 4, 1, GT_NT>(ctx, a, 32) : t160 ? launch_multi<128, 160, 4, 1, GT_NT>(ctx, a, 35)
                                                                     : launch_multi<128, 128, 2, 2, GT_NT>(ctx, a, 33);
}
int gt_gemm(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, gt_buf B, gt_buf C) {
  return gemm_impl(ctx, kind, acc, M, N, K, A, 0, B, 0, C, 0, 1);
}
int gt_gemm_add(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, gt_buf B, gt_buf D, gt_buf C) {
  if (ctx && !D) GT_FAIL(ctx, "gt_gemm_add: null addend");
  return gemm_impl(ctx, kind, 0, M, N, K, A, 0, B, 0, C, 0, 1, 0, 0, 0, D);
}
int gt_gemm_pair(gt_ctx *ctx, int kind, int acc, int M, int N, int K1, gt_buf A1, gt_buf B1, int K2, gt_buf A2, gt_buf B2,
                 gt_buf C) {
  if (ctx && (K2 < 1 || !A2 || !B2)) GT_FAIL(ctx, "gt_gemm_pair: the second product needs K2 >= 1 and both operands (got K2 = %d)", K2);
  // one K loop over both products for 16-byte aligned NT / NN operands; otherwise two launches, the second adding
  const int lda1 = kind == GT_TN ? M : K1, ldb1 = kind == GT_NT ? K1 : N, lda2 = kind == GT_TN ? M : K2, ldb2 = kind == GT_NT ? K2 : N;
  const bool fused = kind != GT_TN && K1 >= 1 && (lda1 % 4 == 0) && (ldb1 % 4 == 0) && (lda2 % 4 == 0) && (ldb2 % 4 == 0) &&
                     ((A1 | B1 | A2 | B2) % 16 == 0);
  if (fused) return gemm_impl(ctx, kind, acc, M, N, K1, A1, 0, B1, 0, C, 0, 1, K2, A2, B2);
  if (gemm_impl(ctx, kind, acc, M, N, K1, A1, 0, B1, 0, C, 0, 1)) return 1;
  return gemm_impl(ctx, kind, 1, M, N, K2, A2, 0, B2, 0, C, 0, 1);
}
int gt_gemm_batched(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, int64_t strideA, gt_buf B,
                    int64_t strideB, gt_buf C, int64_t strideC, int count) {
  return gemm_impl(ctx, kind, acc, M, N, K, A, strideA, B, strideB, C, strideC, count);
}
}
