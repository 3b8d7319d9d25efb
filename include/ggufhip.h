/*
 * libggufhip: C ABI of the MI355X (gfx950) device backend for gguf-trainer's training hot path:
 * backward pass, fused gradient kernels, optimizer step, and the forward producers the backward
 * reads. A host binds these symbols (Deno.dlopen, ctypes) and keeps its own tape; the library owns
 * one HIP stream per context and every call below only enqueues work on it, except gt_sync,
 * gt_d2h and gt_prof_end, which wait.
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on error; gt_last_error() gives the message.
 *     Asynchronous HIP errors are sticky: the next call (or gt_sync) reports them.
 *   - gt_buf is a device address (64-bit). Offsets into a buffer are plain additions, which is how
 *     a vocab span of the readout matrix or one sequence of a batch is addressed.
 *   - tensors are f32, row-major; ids / targets are int32 with -1 as the ignore marker. They are device buffers,
 *     so their range cannot be checked before a launch: it is a precondition of each entry point that takes them, and
 *     a kernel that meets a value outside it skips that row instead of indexing with it; gt_sync, gt_d2h and
 *     gt_prof_end then return an error once ("... is outside [0, V): that row was skipped").
 *   - "acc" arguments: 0 = the kernel stores its result (the destination need not be cleared),
 *     1 = it adds to what the destination holds. The reference zeroes every gradient buffer and
 *     always adds (src/backend/webgpu.ts:21-26, 1397-1429); a host that knows a gradient's first
 *     writer can skip both the clear and the read. No kernel uses floating-point atomics: one
 *     thread owns one output element and every float reduction has a fixed order, so results
 *     are run-to-run identical (the one integer atomicAdd, in the embedding id ranking, is exact
 *     in any order).
 *   - rows-batched extension: where the reference runs one sequence of T rows per call, these take
 *     `rows` (= B*T, sequences stacked) plus what per-sequence structure the op needs (T for
 *     positions, B for attention, one denominator per sequence for the loss). B = 1 is the
 *     reference call.
 *
 * Reference interface replaced: OpsBackend (src/model/autograd.ts:103-151), RegionBackend
 * (:160-164), WebGPUBackend's buffer surface (src/backend/webgpu.ts:1446-1537), AdamWGpu
 * (src/backend/adamw-gpu.ts:131-251) and MuonGpu (src/backend/muon-gpu.ts:351-470).
 */
#ifndef GGUFHIP_H
#define GGUFHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gt_ctx gt_ctx;
typedef struct gt_adamw gt_adamw;
typedef struct gt_muon gt_muon;
typedef uint64_t gt_buf;

/* ---- context, memory, transfers ------------------------------------------------------------
 * Replaces initWebGPU / GpuDevice+queue (webgpu.ts:129-141, 1823), createStateBuffer (:1465),
 * writeStateBuffer (:1482), readStateBuffer (:1492), clearBuffer (:1421-1427),
 * copyBufferToBuffer in seedGradFrom (:742-761), sync (:419-576), residentBytes (:774). */
int gt_ctx_create(int device, gt_ctx **out);
int gt_ctx_destroy(gt_ctx *ctx);
const char *gt_last_error(gt_ctx *ctx);            /* ctx may be NULL: error of a failed create */
const char *gt_device_name(gt_ctx *ctx);
int gt_alloc(gt_ctx *ctx, size_t bytes, int zero, gt_buf *out);
int gt_free(gt_ctx *ctx, gt_buf buf);
int gt_memset0(gt_ctx *ctx, gt_buf buf, size_t bytes);
int gt_h2d(gt_ctx *ctx, gt_buf dst, const void *src, size_t bytes);   /* enqueued; src is copied before return */
int gt_d2h(gt_ctx *ctx, void *dst, gt_buf src, size_t bytes);         /* waits for the stream */
int gt_d2d(gt_ctx *ctx, gt_buf dst, gt_buf src, size_t bytes);
int gt_sync(gt_ctx *ctx);
/* Ordering between the streams of two contexts on one device without the host waiting (no reference counterpart: a
 * WebGPU device has one queue, webgpu.ts:129-141; a host that records independent micro-batches on several contexts needs
 * it where they meet: weights written by an optimizer step on one stream and read by forward passes on the others).
 * gt_stream_mark(a) notes the point a's stream has reached; gt_stream_wait(b, a) makes everything queued on b afterwards
 * start only when a's work up to its latest mark has finished. Neither call blocks the host or allocates. */
int gt_stream_mark(gt_ctx *ctx);
int gt_stream_wait(gt_ctx *ctx, gt_ctx *marked);
int gt_resident_bytes(gt_ctx *ctx, uint64_t *bytes);                  /* live gt_alloc bytes + workspace */
/* Kernel-selection switches for tests and tuning (no reference counterpart; WebGPUBackend exposes
 * attnFlashMinT as a public field for the same purpose, webgpu.ts:305):
 *   "attn.generic" 1 = always take the shape-generic attention kernels, 0 = MFMA kernels where they apply
 *   "gemm.tile"    -1 = heuristic, 0..13 = pin the GEMM tile configuration (tests and tuning)
 *   "gemm.splitk"  -1 = heuristic, n >= 1 = pin the split-K factor
 *   "gemm.group"   1 (default) = gt_gemm_group runs its TN products as one launch; 0 = one launch per product
 *   "gemm.staged"  1 = always stage GEMM operands through registers (0: aligned shapes load straight into LDS)
 *   "gemm.split_bf16" 1 = every product the LDS-direct kernels take (K a multiple of 32, whole 16-byte chunks along each operand's
 *                  contiguous index; a second segment of 16 or 32) runs on the bf16 matrix instruction: each FP32 element as three
 *                  exact bf16 pieces, six of the nine piece products, FP32 accumulation. As close to float64 as the FP32 MFMA kernels,
 *                  about 1.3 x their rate; not bit-identical to them; inf / NaN operands give NaN, and operands below 2^-110 in
 *                  magnitude lose their lower pieces (they would be bf16 denormals). 0 (default) = FP32 MFMA
 *   "gemm.sum_min_tiles" gt_gemm_sum chains its products in one loop from this many 128-row output tiles on
 *                  (-1 = one per CU, the default; 0 = always, for tests of the chained kernel on small shapes)
 *   "attn.splits"  -1 = heuristic, n >= 1 = pin the workgroups per attention tile (MFMA kernels, at most 8)
 *   "attn.keep_ds" 1 (default) = attention backward keeps the score gradients dS in the workspace and computes dQ as one
 *                  banded product over them (T a multiple of 128, hd 64 or 128); 0 = dQ always
 *                  recomputes the scores in its own kernel
 *   "attn.ds_limit_mb" largest dS workspace taken for that, in MiB (default 8192; B*Hq*T*T*4 bytes are needed)
 *   "attn.split_bf16" 1 = the attention forward and the banded dQ product (head dims 64 and 128), and at head dim 64 the dK/dV kernel (where
 *                  the forward kept its scores), run their contractions the same way (rows, tiles, probabilities and score gradients
 *                  as bf16 pieces); everything else in attention stays on FP32 MFMA. 0 (default) = FP32 MFMA
 *   "attn.band_splits" -1 = heuristic, n >= 1 = pin the parts that banded product cuts each row tile's key range into (at most
 *                  8; launches with fewer row tiles than two per CU are cut so that a single sequence fills the chip)
 *   "prof.sample"  n >= 1: gt_prof_begin/end time about 1 in n launches of a label (default 1 = all) */
int gt_set_option(gt_ctx *ctx, const char *key, int value);

/* ---- GEMM: srcGemm (src/backend/wgsl.ts:87-196), WebGPUBackend.gemm (webgpu.ts:1654) ---------
 * kind 0 "NT": C[M,N] = A[M,K] . B[N,K]^T      forward y = x W^T           (webgpu.ts:892)
 * kind 1 "NN": C[M,N] = A[M,K] . B[K,N]        dX = dY W                   (webgpu.ts:896)
 * kind 2 "TN": C[M,N] = A[K,M]^T . B[K,N]      dW = dY^T X                 (webgpu.ts:900)
 * FP32 MFMA, f32 accumulate. Any M, N, K >= 1. */
enum { GT_NT = 0, GT_NN = 1, GT_TN = 2 };
int gt_gemm(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, gt_buf B, gt_buf C);
/* C (+)= A1.B1 + A2.B2: two products of the same kind, M and N summed in one K loop (K1 then K2). It is the LoRA
 * linear of src/model/autograd.ts:760-781 without the [rows, out] add: y = x W^T + (s h) B^T with A2 = s h
 * [rows, r], and in the backward dX = dY W + dH A. Bits differ from two gt_gemm calls with acc = 1 only by the order
 * of the final additions. */
int gt_gemm_pair(gt_ctx *ctx, int kind, int acc, int M, int N, int K1, gt_buf A1, gt_buf B1, int K2, gt_buf A2, gt_buf B2,
                 gt_buf C);
/* The rank-r products of the LoRA linear (src/model/autograd.ts:311-319 makes them `linear` calls; src/train/lora.ts:69-82
 * sizes them), each one streaming pass over the [rows, K] operand:
 *   gt_rank_down: h[rows, r] = alpha * x[rows, K] . s^T, s = [r, K] (s_kmajor = 0: h = x A^T) or [K, r] (s_kmajor = 1:
 *                 dh = g B). alpha is the adapter scale, applied here instead of on a [rows, out] product.
 *   gt_rank_grad: p (+)= h^T . y as [r, K] (transpose_out = 0: dA = dh^T x) or y^T . h as [K, r] (transpose_out = 1:
 *                 dB = g^T h); h [rows, r], y [rows, K].
 * Any r, K >= 1: r <= 32 with K a multiple of 16 (down) / 64 (grad) and 16-byte aligned operands take the streaming
 * kernels, everything else the general GEMM. */
int gt_rank_down(gt_ctx *ctx, int rows, int K, int r, gt_buf x, gt_buf s, int s_kmajor, float alpha, gt_buf h);
int gt_rank_grad(gt_ctx *ctx, int rows, int K, int r, gt_buf h, gt_buf y, int transpose_out, int acc, gt_buf p);
/* gt_rank_grad in two parts, for a host that holds the sums back: an adapter's gradient is not read before the optimizer
 * (src/backend/adamw-gpu.ts:131-251), so the partial sums of a whole backward pass can be added up by ONE launch instead
 * of one small launch per adapter matrix (the reference has no counterpart: its rank-r products are ordinary GEMMs).
 *   gt_rank_grad_slices:  how many row slices gt_rank_grad would cut this product into; 0 when it would not go through
 *                         partial sums at all (one slice, or a shape that takes the general GEMM): call gt_rank_grad then.
 *   gt_rank_grad_parts:   the slices' partial products into parts[slices][r * K] (laid out as p), nothing summed.
 *   gt_rank_slices_group: p_i (+)= parts_i[0] + parts_i[1] + ... for n gradients at once (host arrays of n entries, len_i =
 *                         r * K elements each; distinct p_i), in slice order: the bits gt_rank_grad gives. */
int gt_rank_grad_slices(gt_ctx *ctx, int rows, int K, int r, gt_buf y, int *slices);
int gt_rank_grad_parts(gt_ctx *ctx, int rows, int K, int r, gt_buf h, gt_buf y, int transpose_out, gt_buf parts);
int gt_rank_slices_group(gt_ctx *ctx, int n, const gt_buf *parts, const int *slices, const int *len, const gt_buf *p,
                         const int *acc);
/* C = D + A.B with D a matrix laid out as C (it may be C itself): a linear whose output is at once added to the residual
 * stream, add(h, linear(x, W)) in the reference's layer bodies (src/arch/llama.ts:131-222), as one launch
 * with no [rows, out] round trip for the product. */
int gt_gemm_add(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, gt_buf B, gt_buf D, gt_buf C);
/* C (+)= A_0.B_0 + A_1.B_1 (+ A_2.B_2): up to three products with the same M, N and kind summed in one launch, e.g. the
 * input gradient of sibling projections of one activation, dX = dQ.Wq + dK.Wk + dV.Wv (the reference issues one
 * accumulating GEMM per projection, webgpu.ts:893-901). K, A, B are host arrays of `count` entries; operand i is laid out
 * as for gt_gemm with K = K[i]. NT / NN with every K[i] a multiple of 32, 16-byte aligned operands and at least one
 * 128-row output tile per CU chain the K segments in one loop; anything else is one gt_gemm per product, each adding to
 * the one before. */
int gt_gemm_sum(gt_ctx *ctx, int kind, int acc, int M, int N, int count, const int *K, const gt_buf *A, const gt_buf *B,
                gt_buf C);
/* `count` independent products of one kind with a common K, each with its own M, N, operands, output and acc flag
 * (host arrays of `count` entries; operand i is laid out as for gt_gemm with M[i], N[i], K): the weight gradients
 * dW_i = dY_i^T . X_i of consecutive linears over the same rows (webgpu.ts:900 issues one GEMM per linear), whose outputs
 * are too small to fill the chip one at a time. TN products with K a multiple of 32, M and N multiples of 4 and 16-byte
 * aligned operands run as ONE launch over the tiles of all of them (groups of up to 8) with one ordered reduction for the
 * group; anything else, and a product large enough to fill the chip alone, is one gt_gemm per product. K is split into
 * ranges of max(512, K/8) rows whatever the group holds, and no tile shape changes the order in which an output element
 * sums over K, so a product's result does not depend, bit for bit, on what it shares the launch with. Outputs must be
 * distinct buffers. */
int gt_gemm_group(gt_ctx *ctx, int kind, int count, const int *M, const int *N, int K, const gt_buf *A, const gt_buf *B,
                  const gt_buf *C, const int *acc);
/* batch of `count` independent products with element strides between consecutive problems
 * (Newton-Schulz over same-shaped matrices; no counterpart call in the reference, which loops). */
int gt_gemm_batched(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, int64_t strideA,
                    gt_buf B, int64_t strideB, gt_buf C, int64_t strideC, int count);

/* ---- elementwise: srcElementwise (wgsl.ts:199-209) with the bodies of webgpu.ts:905-1078 ------ */
int gt_add_fwd(gt_ctx *ctx, int64_t n, gt_buf a, gt_buf b, gt_buf out);
int gt_mul_fwd(gt_ctx *ctx, int64_t n, gt_buf a, gt_buf b, gt_buf out);
int gt_silu_fwd(gt_ctx *ctx, int64_t n, gt_buf x, gt_buf out);
int gt_gelu_fwd(gt_ctx *ctx, int64_t n, gt_buf x, gt_buf out);       /* tanh form, K=0.7978845608028654, A=0.044715 */
int gt_scale_fwd(gt_ctx *ctx, int64_t n, gt_buf x, float c, gt_buf out);
/* a destination of 0 is skipped; da == db (add(t,t), mul(t,t)) is allowed and receives both terms */
int gt_add_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf da, int acc_a, gt_buf db, int acc_b);
int gt_mul_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf a, gt_buf b, gt_buf da, int acc_a, gt_buf db, int acc_b);
int gt_silu_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf x, gt_buf dx, int acc);
int gt_gelu_bwd(gt_ctx *ctx, int64_t n, gt_buf g, gt_buf x, gt_buf dx, int acc);
int gt_scale_bwd(gt_ctx *ctx, int64_t n, gt_buf g, float c, gt_buf dx, int acc);
/* out = act(gate) * up and its backward in one pass each (act 0 = silu, 1 = gelu-tanh): the
 * mul(silu(gate), up) / mul(gelu(gate), up) pair of src/arch/llama.ts:207-209, gemma3.ts:205-207
 * fused; backward reads g, gate, up and writes dgate, dup (20 B per element). */
int gt_glu_fwd(gt_ctx *ctx, int act, int64_t n, gt_buf gate, gt_buf up, gt_buf out);
int gt_glu_bwd(gt_ctx *ctx, int act, int64_t n, gt_buf g, gt_buf gate, gt_buf up,
               gt_buf dgate, int acc_gate, gt_buf dup, int acc_up);

/* ---- RMSNorm: srcRmsNormFwd / BwdX / BwdW (wgsl.ts:217-303), rmsNormRows (webgpu.ts:1680-1699) -
 * Serves rmsNorm (rows = T, d = hidden) and rmsNormHeads (rows = T*H, d = hd; webgpu.ts:1085-1088).
 * Backward computes dx and the per-column dw sums in one pass over x and g; dw == 0 skips it. */
int gt_rmsnorm_fwd(gt_ctx *ctx, int rows, int d, float eps, gt_buf x, gt_buf w, gt_buf y, gt_buf rinv);
int gt_rmsnorm_bwd(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv,
                   gt_buf dx, int acc_dx, gt_buf dw, int acc_dw);
/* The same with the gradient's old contents in another buffer: dx = dx_old + (the normalisation's input gradient). For a
 * gradient whose only contribution so far is a copy of an upstream gradient (the add of a residual stream,
 * webgpu.ts:921-937): the copy is skipped and the upstream buffer is read here instead. */
int gt_rmsnorm_bwd_from(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx_old, gt_buf dx,
                        gt_buf dw, int acc_dw);
/* The weight gradient's column sums put off. srcRmsNormBwdW (wgsl.ts:286-303) runs once per normalisation; here the backward
 * kernel already leaves one partial row per workgroup, and a host that knows nobody reads dw before the end of the backward
 * pass can keep those rows and sum the columns of every normalisation in ONE launch at that point:
 *   gt_rmsnorm_parts_rows: how many partial rows of d floats gt_rmsnorm_bwd_parts writes for (rows, d); 0 = this shape is
 *                          not served (d not a multiple of 4 or above 2048: use gt_rmsnorm_bwd)
 *   gt_rmsnorm_bwd_parts:  dx = (acc_dx ? dx_old : 0) + the normalisation's input gradient (dx_old may be dx itself), and the
 *                          partial rows into `parts` (the caller's buffer, 16-byte aligned); no dw is written
 *   gt_colsum_group:       dw_i (+)= the column sums of parts_i, for n entries in one launch (host arrays of n entries);
 *                          bit for bit what gt_rmsnorm_bwd would have written. Entries must have distinct dw. */
int gt_rmsnorm_parts_rows(gt_ctx *ctx, int rows, int d, int *nparts);
int gt_rmsnorm_bwd_parts(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv, gt_buf dx_old, gt_buf dx,
                         int acc_dx, gt_buf parts);
int gt_colsum_group(gt_ctx *ctx, int n, const gt_buf *parts, const int *nparts, const int *d, const gt_buf *dw, const int *acc);

/* gt_rmsnorm_bwd for callers that cannot allocate device memory: code under HIP graph capture, tight loops of a serving
 * process, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments and bit-identical
 * results; the per-workgroup dw partials go to a 4 MiB array that is part of the library's code object (one copy per GPU,
 * held until the process ends) instead of the context's grow-only workspace, and the call makes no hipMalloc / hipFree,
 * creates no events (it is not seen by gt_prof_begin / gt_prof_end) and records no memset node. Limits: d a multiple of
 * 4 and at most 2048, every operand 16-byte aligned; anything else is refused with an error. All calls on one GPU share
 * that GPU's array: two calls that overlap in time on one GPU (two contexts, i.e. two streams) race on it; calls on one
 * context are ordered by its stream. */
int gt_rmsnorm_bwd_static(gt_ctx *ctx, int rows, int d, gt_buf x, gt_buf w, gt_buf g, gt_buf rinv,
                          gt_buf dx, int acc_dx, gt_buf dw, int acc_dw);

/* ---- embedding: srcEmbeddingFwd / Bwd (wgsl.ts:305-344) -------------------------------------
 * Precondition: every id is in [0, V) (the reference checks this above the dispatch, autograd.ts:324-346; ids live on
 * the device here, so the library cannot look before it launches). A kernel that meets an id outside the range does not
 * touch memory for it: the forward writes a zero row, the backward adds nothing, and the next gt_sync / gt_d2h /
 * gt_prof_end fails once, naming the row and the id. */
int gt_embedding_fwd(gt_ctx *ctx, int rows, int d, int V, gt_buf ids, gt_buf W, gt_buf out);
int gt_embedding_bwd(gt_ctx *ctx, int rows, int d, int V, gt_buf ids, gt_buf g, gt_buf dW, int acc);

/* ---- RoPE: srcRope (wgsl.ts:346-384), NeoX pairing (j, j+hd/2); position of row r is
 * (r mod T) + pos. backward = 1 applies the transposed rotation. */
int gt_rope(gt_ctx *ctx, int rows, int T, int H, int hd, double base, int pos, int backward,
            gt_buf in, gt_buf out, int acc);
/* The same rotation over two tensors that share rows, T, hd, base and pos (the q and k of a layer: two srcRope dispatches,
 * webgpu.ts:1110-1121) as one launch; H1 and H2 heads per row. Results are those of two gt_rope calls. */
int gt_rope_pair(gt_ctx *ctx, int rows, int T, int hd, double base, int pos, int backward, int H1, gt_buf in1, gt_buf out1, int acc1,
                 int H2, gt_buf in2, gt_buf out2, int acc2);

/* ---- attention: srcAttnFwd / BwdD / BwdDq / BwdDkv (wgsl.ts:657-918), webgpu.ts:1142-1189 -----
 * q[B*T, Hq*hd], k,v[B*T, Hkv*hd], causal, window > 0 keeps keys [t-window+1, t]; GQA head h reads
 * kv head h / (Hq/Hkv). lse[B*Hq*T] is the saved softmax statistic (log2 domain). */
int gt_attn_fwd(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window,
                gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse);
int gt_attn_bwd(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window,
                gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf dout, gt_buf lse,
                gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v);
/* The same pair with the scores kept from the forward to the backward, as the reference's small-T path keeps its
 * probabilities and score gradients ([Hq,T,T] transients of srcAttnProbs / srcAttnDScore, wgsl.ts:492-583, webgpu.ts:1176-1189): the backward then reads S instead of recomputing
 * Q.K^T for dK/dV. gt_attn_scores_bytes gives the size of the scores buffer for a shape (B*Hq*T*T*4), or 0 where scores
 * are not kept (T not a multiple of 128, head dims other than 64 and 128, "attn.generic"); the buffer belongs to the
 * caller, must live until the backward call and holds the library's own layout (32 x 32 blocks, masked pairs marked). Results equal gt_attn_fwd / gt_attn_bwd up to rounding. */
int gt_attn_scores_bytes(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, uint64_t *bytes);
int gt_attn_fwd_scores(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window,
                       gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, gt_buf scores);
int gt_attn_bwd_scores(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window,
                       gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf dout, gt_buf lse, gt_buf scores,
                       gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v);
/* gt_attn_bwd_scores for q and / or k that are the outputs of a rope (src/arch/llama.ts:196-199 rotates both before attention):
 * with rot_q (rot_k) set, dq (dk) receives the gradient with respect to the rows BEFORE the rotation (base rope_base,
 * offset rope_pos, as gt_rope takes them), i.e. what gt_rope(backward = 1) would make of the gradient this call computes, applied
 * in the write-backs of the dQ product and of dK. The reference runs srcRope's backward as a dispatch of its own per tensor
 * (webgpu.ts:1117-1121). Same conditions as gt_attn_bwd_scores; the results differ from the two-call form by rounding only. */
int gt_attn_bwd_scores_rope(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window,
                            gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf dout, gt_buf lse, gt_buf scores,
                            double rope_base, int rope_pos, int rot_q, int rot_k,
                            gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv, int acc_v);

/* ---- cross-entropy: srcCeFwd / CeReduce / CeBwd (wgsl.ts:936-1133), webgpu.ts:1281-1327 ------
 * rows = n_seq * T. Sequence s owns rows [s*T, (s+1)*T) and its own denominator
 * max(kept_s, 1) (autograd.ts:938), passed as inv_denom[s] = 1/denominator (f32, device).
 * fwd writes loss[s] = inv_denom[s] * sum over kept rows of (logsumexp - z_target) and lse[rows].
 * bwd: dlogits[r,:] (+)= seed * inv_denom[s] * (softmax - onehot); ignored rows get 0 (acc = 0)
 * or are left alone (acc = 1).
 * Precondition: every target is -1 or in [0, V) (checked above the dispatch in the reference, autograd.ts:875-894).
 * A target outside that range is never used as an index: every kernel, forward and backward, dense and chunked, treats
 * the row as ignored; gt_ce_fwd (dense) and the first gt_ce_chunk_stats of a pass (chunked) note it and the next gt_sync /
 * gt_d2h / gt_prof_end fails once, naming the row. */
int gt_ce_fwd(gt_ctx *ctx, int rows, int V, int T, gt_buf logits, gt_buf targets, gt_buf inv_denom,
              gt_buf loss, gt_buf lse);
int gt_ce_bwd(gt_ctx *ctx, int rows, int V, int T, gt_buf logits, gt_buf targets, gt_buf inv_denom,
              gt_buf lse, float seed, gt_buf dlogits, int acc);
/* chunked path: srcCeChunkStats / CeLossFromStats / CeChunkGrad (wgsl.ts:1153-1247),
 * fusedCrossEntropy (webgpu.ts:1214-1278). `chunk` holds logits of vocab span [v0, v0+vc) of the V-wide vocabulary. */
int gt_ce_chunk_stats(gt_ctx *ctx, int rows, int V, int vc, int v0, int first, gt_buf chunk, gt_buf targets,
                      gt_buf row_max, gt_buf row_sum, gt_buf tgt_logit);
int gt_ce_loss_from_stats(gt_ctx *ctx, int rows, int V, int T, gt_buf targets, gt_buf inv_denom,
                          gt_buf row_max, gt_buf row_sum, gt_buf tgt_logit, gt_buf loss);
int gt_ce_chunk_grad(gt_ctx *ctx, int rows, int V, int vc, int v0, int T, gt_buf chunk, gt_buf targets,
                     gt_buf inv_denom, gt_buf row_max, gt_buf row_sum, float seed);
/* sparse-teacher soft CE: srcSoftCeFwd / BwdP / BwdQ (wgsl.ts:1004-1110), webgpu.ts:1331-1378. teacher_ids[rows*k]:
 * a row whose first id is -1 is ignored; every other id must be in [0, V) (autograd.ts:974-998 checks it above the
 * dispatch). An id outside the range is skipped by both kernels and reported by the next gt_sync / gt_d2h / gt_prof_end. */
int gt_soft_ce_fwd(gt_ctx *ctx, int rows, int V, int k, gt_buf logits, gt_buf teacher_ids, gt_buf teacher_probs,
                   float inv_denom, gt_buf loss, gt_buf lse, gt_buf row_mass);
int gt_soft_ce_bwd(gt_ctx *ctx, int rows, int V, int k, gt_buf logits, gt_buf teacher_ids, gt_buf teacher_probs,
                   float inv_denom, gt_buf lse, gt_buf row_mass, float seed, gt_buf dlogits, int acc);

/* ---- AdamW: AdamWGpu (adamw-gpu.ts:131-251), spec src/train/adam.ts:46-82 --------------------
 * One object per parameter group; step() = global grad-norm clip over the whole group (when
 * clip > 0) followed by the fused element update, two launches for any number of tensors.
 * bc1 = 1 - beta1^t and bc2 = 1 - beta2^t come from the host, as in adamw-gpu.ts:211-218.
 * Hyperparameters are doubles (JS numbers): 1 - beta and 1/bc are formed in f64 and rounded once,
 * since 1.0f - 0.999f is already 1.3e-5 off. */
int gt_adamw_create(gt_ctx *ctx, int n, const gt_buf *w, const gt_buf *g, const gt_buf *m, const gt_buf *v,
                    const int64_t *sizes, double beta1, double beta2, double eps, double weight_decay, double clip,
                    gt_adamw **out);
int gt_adamw_step(gt_ctx *ctx, gt_adamw *opt, double lr, double bc1, double bc2);
int gt_adamw_grad_norm(gt_ctx *ctx, gt_adamw *opt, float *norm);   /* last step's global norm; waits */
int gt_adamw_destroy(gt_ctx *ctx, gt_adamw *opt);

/* dst[i] (+)= src[i*nsrc + 0] + src[i*nsrc + 1] + ... (a source of 0 is skipped), i < n, sizes[i] elements each, one
 * launch for the whole list: parameter-gradient accumulators that micro-batches recorded on different streams kept
 * apart, summed in a fixed order into the one the optimizer reads. dst_acc[i] = 0 stores, 1 adds to dst's contents.
 * nsrc <= 7. The reference keeps one accumulator per parameter and one queue (webgpu.ts:21-26); no counterpart there. */
int gt_grad_fold(gt_ctx *ctx, int n, const gt_buf *dst, const int *dst_acc, int nsrc, const gt_buf *src, const int64_t *sizes);

/* ---- Muon: MuonGpu (muon-gpu.ts:351-470), buildNewtonSchulz (:224-252), spec src/train/muon.ts -
 * Matrices w[i] are [rows[i], cols[i]]; buf[i] is the momentum. step(): buf = mu*buf + g;
 * U = nesterov ? g + mu*buf : buf; X = NS(U); w -= lr*sqrt(max(1, rows/cols))*X. */
int gt_muon_create(gt_ctx *ctx, int n, const gt_buf *w, const gt_buf *g, const gt_buf *buf,
                   const int *rows, const int *cols, double momentum, int nesterov, int ns_steps, gt_muon **out);
int gt_muon_step(gt_ctx *ctx, gt_muon *opt, double lr);
int gt_muon_destroy(gt_ctx *ctx, gt_muon *opt);
/* newtonSchulzGpu (muon-gpu.ts:259-283): out[m,n] = NS(G[m,n]) */
int gt_newton_schulz(gt_ctx *ctx, int m, int n, int steps, gt_buf G, gt_buf out);

/* ---- profiling: startProfile / stopProfile (webgpu.ts:830-880) --------------------------------
 * Between begin and end every launch whose label starts with `prefix` (NULL or "" = all) is
 * bracketed by HIP events on the context's stream and summed per label, together with the
 * algorithmic work the call states for itself (FLOP for the contractions, bytes for the streaming
 * kernels). GEMM labels carry the kernel's tile shape ("gemm.nn.128x192"). gt_prof_end waits, then
 * fills up to `cap` records. An event pair delays the stream by a few microseconds; with the option
 * "prof.sample" = n about 1 in n launches of a label is bracketed (a fixed pseudo-random choice over
 * the label's launch numbers); `count` and `work` still cover every launch and `ms` is the timed
 * launches' time scaled by all work / timed work. */
typedef struct gt_prof_rec { char label[32]; double ms; int64_t count; double work; } gt_prof_rec;
int gt_prof_begin(gt_ctx *ctx, const char *prefix);
int gt_prof_end(gt_ctx *ctx, gt_prof_rec *out, int cap, int *n);
/* One event pair around everything queued between the two calls (the same startProfile / stopProfile surface, for a
 * run of back-to-back launches as the device sees it, without a pair per launch). gt_timer_stop waits for the stream
 * and gives the elapsed milliseconds. */
int gt_timer_start(gt_ctx *ctx);
int gt_timer_stop(gt_ctx *ctx, double *ms);

#ifdef __cplusplus
}
#endif
#endif
