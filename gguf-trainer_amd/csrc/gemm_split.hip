// The FP32 products of gemm.hip on the bf16 matrix instruction: every operand element is cut into three bf16 pieces as
// it is read from LDS and a pair of 32 x 32 x 16 blocks takes six MFMAs (gemm_tile.h, SplitFrag). Selected per context by
// the option "gemm.split_bf16"; tiles, ring, K splits, batches, summed segments and write-back are the direct kernels'.
#include "gemm_tile.h"

#define GT_SPLIT_BK 32
#define GT_SPLIT_NSTG 2
template <int BM, int BN, int WM, int WN, int KIND, bool MSEG, bool SEG2 = false>
static int launch_split_kind(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int smem = GT_SPLIT_NSTG * (BM + BN) * GT_SPLIT_BK * 4;
  if (!(ctx->gemm_split_set & (1ull << slot))) {       // once per context (device): more LDS than a kernel gets by default
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, KIND, GT_SPLIT_BK, GT_SPLIT_NSTG, SEG2, false, MSEG, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_split_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, KIND, GT_SPLIT_BK, GT_SPLIT_NSTG, SEG2, false, MSEG, true>), dim3(a.nbm * a.nbn, 1, zdim),
                     dim3(WM * WN * 64), smem, ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}
template <bool MSEG>
static int launch_split(gt_ctx *ctx, int kind, bool wide, GemmArgs &a, int zdim) {
  const int s = (MSEG ? 6 : 0) + (wide ? 3 : 0) + kind;
  if (wide) {
    if (kind == GT_NT) return launch_split_kind<128, 192, 2, 2, GT_NT, MSEG>(ctx, a, zdim, s);
    if (kind == GT_NN) return launch_split_kind<128, 192, 2, 2, GT_NN, MSEG>(ctx, a, zdim, s);
    if (!MSEG) return launch_split_kind<128, 192, 2, 2, GT_TN, false>(ctx, a, zdim, s);
  }
  if (kind == GT_NT) return launch_split_kind<128, 128, 2, 2, GT_NT, MSEG>(ctx, a, zdim, s);
  if (kind == GT_NN) return launch_split_kind<128, 128, 2, 2, GT_NN, MSEG>(ctx, a, zdim, s);
  if (!MSEG) return launch_split_kind<128, 128, 2, 2, GT_TN, false>(ctx, a, zdim, s);
  GT_FAIL(ctx, "summed products are NT or NN");
}
// two K segments (the second 16 or 32 long, riding in one more stage): NT / NN
static int launch_split_seg2(gt_ctx *ctx, int kind, bool wide, GemmArgs &a, int zdim) {
  const int s = 14 + (wide ? 2 : 0) + kind;
  if (wide) return kind == GT_NT ? launch_split_kind<128, 192, 2, 2, GT_NT, false, true>(ctx, a, zdim, s)
                                 : launch_split_kind<128, 192, 2, 2, GT_NN, false, true>(ctx, a, zdim, s);
  return kind == GT_NT ? launch_split_kind<128, 128, 2, 2, GT_NT, false, true>(ctx, a, zdim, s)
                       : launch_split_kind<128, 128, 2, 2, GT_NN, false, true>(ctx, a, zdim, s);
}
int gemm_split_launch(gt_ctx *ctx, int kind, bool wide, bool summed, GemmArgs &a, int zdim) {
  if (a.K2 > 0) return launch_split_seg2(ctx, kind, wide, a, zdim);
  return summed ? launch_split<true>(ctx, kind, wide, a, zdim) : launch_split<false>(ctx, kind, wide, a, zdim);
}

template <int BM, int BN, int WM, int WN>
static int launch_group_split(gt_ctx *ctx, GemmArgs &a, GroupArgs &g, int slot) {
  constexpr int smem = GT_SPLIT_NSTG * (BM + BN) * GT_SPLIT_BK * 4;
  if (!(ctx->gemm_split_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_group_tn<BM, BN, WM, WN, GT_SPLIT_BK, GT_SPLIT_NSTG, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_split_set |= 1ull << slot;
  }
  int tiles = 0;
  for (int i = 0; i < g.n; i++) {
    g.p[i].tile0 = tiles;
    g.p[i].nbn = (int)cdiv(g.p[i].N, BN);
    tiles += (int)cdiv(g.p[i].M, BM) * g.p[i].nbn;
  }
  g.ntiles = tiles;
  hipLaunchKernelGGL((gemm_group_tn<BM, BN, WM, WN, GT_SPLIT_BK, GT_SPLIT_NSTG, true>), dim3((unsigned)tiles * a.splits), dim3(WM * WN * 64), smem,
                     ctx->stream, a, g);
  GT_LAUNCHED(ctx);
  return 0;
}
int gemm_split_launch_group(gt_ctx *ctx, bool wide, GemmArgs &a, GroupArgs &g) {
  return wide ? launch_group_split<128, 192, 2, 2>(ctx, a, g, 12) : launch_group_split<128, 128, 2, 2>(ctx, a, g, 13);
}

template <int HD>
static int launch_split_band(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int BM = 128, BN = HD, WM = 2, WN = HD / 64;
  constexpr int smem = band_lds_bytes<BM, BN, GT_SPLIT_BK, GT_SPLIT_NSTG>();
  if (!(ctx->gemm_split_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, GT_NN, GT_SPLIT_BK, GT_SPLIT_NSTG, false, true, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_split_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, GT_NN, GT_SPLIT_BK, GT_SPLIT_NSTG, false, true, false, true>), dim3(zdim, a.splits, a.nbm * a.nbn),
                     dim3(WM * WN * 64), smem, ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}

int gemm_split_launch_band(gt_ctx *ctx, GemmArgs &a, int zdim) {
  return a.N == 64 ? launch_split_band<64>(ctx, a, zdim, 18) : launch_split_band<128>(ctx, a, zdim, 19);
}
