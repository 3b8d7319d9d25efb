// MFMA attention kernels (hd = 64 / 128). Placeholder: reports no supported head dim until the
// kernels land, so every shape takes the generic wavefront-per-row path in attention.hip.
#include "common.h"
struct AttnP;
int attn_mfma_supported(int hd) { (void)hd; return 0; }
int attn_fwd_mfma(gt_ctx *ctx, const AttnP &, gt_buf, gt_buf, gt_buf, gt_buf, gt_buf) { GT_FAIL(ctx, "attn_fwd_mfma: not built"); }
int attn_bwd_mfma(gt_ctx *ctx, const AttnP &, gt_buf, gt_buf, gt_buf, gt_buf, gt_buf, const float *, gt_buf, int, gt_buf, int,
                  gt_buf, int) { GT_FAIL(ctx, "attn_bwd_mfma: not built"); }
