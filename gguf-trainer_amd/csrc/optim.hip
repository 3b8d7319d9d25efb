// Device-resident AdamW and Muon (src/backend/adamw-gpu.ts, src/backend/muon-gpu.ts; the CPU
// specs are src/train/adam.ts:46-82 and src/train/muon.ts:69-158).
//
// AdamW. The reference issues two reduction dispatches and one update dispatch per tensor (816
// launches for a 272-tensor model). Here the group is described once by a chunk table on the
// device (tensor index, offset, length per 2048-element chunk) and a step is three launches for any
// number of tensors: per-chunk sum of squares, a single-workgroup fold of the chunk sums into the
// clip scale, and the fused element update. The fold runs in chunk order, so the norm and
// everything downstream is identical from run to run.
//
// Muon. Per matrix: momentum + Nesterov + sum of squares, normalise, five quintic Newton-Schulz
// iterations of three MFMA GEMMs each, then the scaled descent. The reference transposes a tall matrix
// so that the Gram matrix is the small one (muon.ts:137-158); here a tall matrix stays as it lies and
// its iteration is written on the other side (A = X^T X, X <- a X + X B), which is the same
// arithmetic without the two transposing passes. The two combines of an iteration, b A + c A.A and
// a X + B.X, are the write-backs of the products that feed them (C = dscale*D + pscale*A.B), so an
// iteration is three launches and no elementwise pass. Matrices of equal shape are stepped together
// as one batch (see below).
#include <algorithm>
#include <vector>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));

#define CHUNK 2048

struct Chunk { int tensor; int len; int64_t off; };
struct TensorPtrs { float *w, *g, *m, *v; };

struct gt_adamw {
  int n = 0, nchunks = 0;
  double total_elems = 0;
  double beta1, beta2, eps, wd, clip;
  Chunk *chunks = nullptr;
  TensorPtrs *ptrs = nullptr;
  float *partial = nullptr;     // [nchunks]
  float *scale = nullptr;       // [2]: clip scale, grad norm
};

__global__ __launch_bounds__(256) void adamw_ssq_k(const Chunk *__restrict__ chunks, const TensorPtrs *__restrict__ ptrs,
                                                   float *__restrict__ partial) {
  __shared__ float sm[4];
  Chunk c = chunks[blockIdx.x];
  const float *g = ptrs[c.tensor].g + c.off;
  float s = 0;
  if ((reinterpret_cast<uintptr_t>(g) & 15) == 0) {
    // read once: streaming loads, four float4 in flight per thread
    int n4 = c.len / 4;
    float s4[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i0 = threadIdx.x; i0 < n4; i0 += 1024) {
      v4f x[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        int i = i0 + u * 256;
        x[u] = i < n4 ? __builtin_nontemporal_load(reinterpret_cast<const v4f *>(g) + i) : v4f{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < 4; u++) s4[u] += x[u][0] * x[u][0] + x[u][1] * x[u][1] + x[u][2] * x[u][2] + x[u][3] * x[u][3];
    }
    s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    for (int i = n4 * 4 + threadIdx.x; i < c.len; i += 256) s += g[i] * g[i];
  } else {
    for (int i = threadIdx.x; i < c.len; i += 256) s += g[i] * g[i];
  }
  s = block_sum<4>(s, sm);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
// scale = norm > clip ? clip/(norm + 1e-12) : 1   (adam.ts:56-62, adamw-gpu.ts:84-95)
__global__ __launch_bounds__(1024) void adamw_scale_k(int nchunks, const float *__restrict__ partial, float clip,
                                                      float *__restrict__ scale) {
  __shared__ float sm[16];
  // eight independent loads per thread and round, so the fold is not a chain of dependent memory latencies; the
  // order of the sum is fixed by the thread count, not by timing
  float s8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int i0 = threadIdx.x; i0 < nchunks; i0 += 8 * 1024) {
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; u++) x[u] = partial[min(i0 + u * 1024, nchunks - 1)];       // unconditional: all in flight together
#pragma unroll
    for (int u = 0; u < 8; u++) s8[u] += i0 + u * 1024 < nchunks ? x[u] : 0.f;
  }
  float s = ((s8[0] + s8[1]) + (s8[2] + s8[3])) + ((s8[4] + s8[5]) + (s8[6] + s8[7]));
  s = block_sum<16>(s, sm);
  if (threadIdx.x == 0) {
    float norm = sqrtf(s);
    scale[0] = norm > clip ? clip / (norm + 1e-12f) : 1.0f;
    scale[1] = norm;
  }
}
struct AdamH { float b1, b2, omb1, omb2, eps, wd, lr, ibc1, ibc2; };
__device__ __forceinline__ void adam1(float g, float &m, float &v, float &w, const AdamH &h) {
  const float b1 = h.b1, b2 = h.b2, eps = h.eps, wd = h.wd, lr = h.lr, ibc1 = h.ibc1, ibc2 = h.ibc2;
  m = b1 * m + h.omb1 * g;
  v = b2 * v + h.omb2 * g * g;
  float upd = (m * ibc1) / (sqrtf(v * ibc2) + eps);
  if (wd > 0.f) upd += wd * w;
  w -= lr * upd;
}
__global__ __launch_bounds__(256) void adamw_update_k(const Chunk *__restrict__ chunks, const TensorPtrs *__restrict__ ptrs,
                                                      const float *__restrict__ scale, AdamH h) {
  Chunk c = chunks[blockIdx.x];
  TensorPtrs p = ptrs[c.tensor];
  const float sc = scale[0];
  float *w = p.w + c.off, *m = p.m + c.off, *v = p.v + c.off;
  const float *g = p.g + c.off;
  bool vec = ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(m) | reinterpret_cast<uintptr_t>(v) |
               reinterpret_cast<uintptr_t>(g)) & 15) == 0;
  int n4 = vec ? c.len / 4 : 0;
  // every array is touched once per step: streaming accesses (the weights too: 4 bytes per parameter of them do not
  // stay cached until the next forward reads them), UF float4 per array in flight
  constexpr int UF = 2;
  for (int i0 = threadIdx.x; i0 < n4; i0 += 256 * UF) {
    v4f gg[UF], mm[UF], vv[UF], ww[UF];
#pragma unroll
    for (int u = 0; u < UF; u++) {
      int i = i0 + u * 256;
      if (i < n4) {
        gg[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(g) + i) * sc;
        mm[u] = __builtin_nontemporal_load(reinterpret_cast<v4f *>(m) + i);
        vv[u] = __builtin_nontemporal_load(reinterpret_cast<v4f *>(v) + i);
        ww[u] = __builtin_nontemporal_load(reinterpret_cast<v4f *>(w) + i);
      }
    }
#pragma unroll
    for (int u = 0; u < UF; u++) {
      int i = i0 + u * 256;
      if (i >= n4) continue;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float tm = mm[u][j], tv = vv[u][j], tw = ww[u][j];
        adam1(gg[u][j], tm, tv, tw, h);
        mm[u][j] = tm; vv[u][j] = tv; ww[u][j] = tw;
      }
      __builtin_nontemporal_store(mm[u], reinterpret_cast<v4f *>(m) + i);
      __builtin_nontemporal_store(vv[u], reinterpret_cast<v4f *>(v) + i);
      __builtin_nontemporal_store(ww[u], reinterpret_cast<v4f *>(w) + i);
    }
  }
  for (int i = n4 * 4 + threadIdx.x; i < c.len; i += 256) adam1(g[i] * sc, m[i], v[i], w[i], h);
}


// ---- gradient fold ------------------------------------------------------------------------------------
// dst_i (+)= src_i0 + src_i1 + ... for a list of tensors in one launch: the accumulators that micro-batches recorded on
// different streams kept apart, summed in stream order into the accumulator the optimizer reads.
#define FOLD_CHUNK 8192
#define FOLD_MAX_SRC 7
struct FoldPtrs { float *dst; const float *src[FOLD_MAX_SRC]; int acc, nsrc; };
__global__ __launch_bounds__(256) void grad_fold_k(const Chunk *__restrict__ chunks, const FoldPtrs *__restrict__ ptrs) {
  const Chunk c = chunks[blockIdx.x];
  const FoldPtrs p = ptrs[c.tensor];
  float *dst = p.dst + c.off;
  bool vec = (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
  for (int s = 0; s < p.nsrc; s++) vec = vec && (reinterpret_cast<uintptr_t>(p.src[s] + c.off) & 15) == 0;
  const int n4 = vec ? c.len / 4 : 0;
  for (int i = threadIdx.x; i < n4; i += 256) {
    v4f x[FOLD_MAX_SRC + 1];
    if (p.acc) x[0] = reinterpret_cast<const v4f *>(dst)[i];
#pragma unroll
    for (int s = 0; s < FOLD_MAX_SRC; s++)
      if (s < p.nsrc) x[s + 1] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p.src[s] + c.off) + i);
    v4f sum = p.acc ? x[0] + x[1] : x[1];
#pragma unroll
    for (int s = 1; s < FOLD_MAX_SRC; s++)
      if (s < p.nsrc) sum += x[s + 1];
    reinterpret_cast<v4f *>(dst)[i] = sum;
  }
  for (int i = n4 * 4 + threadIdx.x; i < c.len; i += 256) {
    float sum = p.acc ? dst[i] + p.src[0][c.off + i] : p.src[0][c.off + i];
    for (int s = 1; s < p.nsrc; s++) sum += p.src[s][c.off + i];
    dst[i] = sum;
  }
}

// ---- Muon -------------------------------------------------------------------------------------------
// Matrices of equal shape form a group that is stepped as one batch: every elementwise stage runs over the
// group's concatenated work buffers (blockIdx.y = matrix), and each Newton-Schulz product is one batched GEMM
// launch. A 12-layer model with four distinct projection shapes takes 4 x 29 launches per step instead of
// 84 x 29.

struct MuonGroup {
  int rows, cols, count;
  float **w = nullptr, **g = nullptr, **buf = nullptr;          // device tables of per-matrix pointers
  float *U = nullptr, *X = nullptr, *A = nullptr, *AA = nullptr, *BX = nullptr, *part = nullptr;
  size_t bytes = 0;
};
struct gt_muon {
  std::vector<MuonGroup> groups;
  float momentum; int nesterov, ns_steps;
};

#define NS_A 3.4445f
#define NS_B (-4.7750f)
#define NS_C 2.0315f
#define RED_BLOCKS 256

// buf = mu*buf + g; U = nesterov ? g + mu*buf : buf; per-workgroup sum of U^2 (muon-gpu.ts:51-92).
// With null tables (Newton-Schulz on a caller's matrix) U is only read.
__global__ __launch_bounds__(256) void muon_momentum_k(int64_t n, float *const *__restrict__ gt, float *const *__restrict__ bt,
                                                       float *__restrict__ Uall, float mu, int nesterov, float *__restrict__ part) {
  __shared__ float sm[4];
  const int mi = blockIdx.y;
  float *U = Uall + (size_t)mi * n;
  const float *g = gt ? gt[mi] : nullptr;
  float *buf = bt ? bt[mi] : nullptr;
  float s = 0;
  const bool vec = (n % 4 == 0) && (((reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(buf)) & 15) == 0);
  if (vec) {
    // every array is touched once: float4 per lane, the partial sum of a workgroup taken in a fixed order
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n / 4; i += (int64_t)gridDim.x * 256) {
      v4f u;
      if (buf) {
        const v4f gi = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(g) + i);
        const v4f b = reinterpret_cast<const v4f *>(buf)[i] * mu + gi;
        reinterpret_cast<v4f *>(buf)[i] = b;
        u = nesterov ? gi + b * mu : b;
        reinterpret_cast<v4f *>(U)[i] = u;
      } else u = reinterpret_cast<const v4f *>(U)[i];
      s += (u[0] * u[0] + u[1] * u[1]) + (u[2] * u[2] + u[3] * u[3]);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
      float u;
      if (buf) {
        float gi = g[i];
        float b = mu * buf[i] + gi;
        buf[i] = b;
        u = nesterov ? gi + mu * b : b;
        U[i] = u;
      } else u = U[i];
      s += u * u;
    }
  }
  s = block_sum<4>(s, sm);
  if (threadIdx.x == 0) part[(size_t)mi * gridDim.x + blockIdx.x] = s;
}
// X = U / (sqrt(sum part) + 1e-7), one matrix of `total` elements per blockIdx.y (muon.ts:137-144 without the transpose)
__global__ __launch_bounds__(256) void muon_normalize_k(int64_t total, const float *__restrict__ Uall,
                                                        const float *__restrict__ part, int nparts, float *__restrict__ Xall) {
  __shared__ float sm[4];
  const int mi = blockIdx.y;
  const float *U = Uall + (size_t)mi * total;
  float *X = Xall + (size_t)mi * total;
  float s = 0;
  for (int i = threadIdx.x; i < nparts; i += 256) s += part[(size_t)mi * nparts + i];
  s = block_sum<4>(s, sm);
  const float inv = 1.0f / (sqrtf(s) + 1e-7f);
  const bool vec = (total % 4 == 0) && (((reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(X)) & 15) == 0);
  if (vec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total / 4; i += (int64_t)gridDim.x * 256)
      reinterpret_cast<v4f *>(X)[i] = reinterpret_cast<const v4f *>(U)[i] * inv;
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) X[i] = U[i] * inv;
  }
}
// W -= f * X, one matrix per blockIdx.y
__global__ __launch_bounds__(256) void muon_apply_k(int64_t total, float *const *__restrict__ wt, float *Wone,
                                                    const float *__restrict__ Xall, float f) {
  const int mi = blockIdx.y;
  float *W = wt ? wt[mi] : Wone;
  const float *X = Xall + (size_t)mi * total;
  const bool vec = (total % 4 == 0) && (((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(X)) & 15) == 0);
  if (vec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total / 4; i += (int64_t)gridDim.x * 256)
      reinterpret_cast<v4f *>(W)[i] -= reinterpret_cast<const v4f *>(X)[i] * f;
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) W[i] -= f * X[i];
  }
}

static inline unsigned sgrid(gt_ctx *ctx, int64_t n) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>(cdiv(n, 256), (int64_t)ctx->num_cu * 8)); }

// Leaves NS(U), laid out as U ([count][m,n]), in *result (G.X or G.BX); U holds the inputs, part their per-workgroup
// sums of squares. Per iteration (muon.ts:146-156 with A the r x r Gram matrix, r = min(m, n)):
//   wide (m <= n):  A = X X^T          B = b A + c A.A      X <- a X + B.X
//   tall (m >  n):  A = X^T X          B = b A + c A.A      X <- a X + X.B
static int newton_schulz_run(gt_ctx *ctx, const MuonGroup &G, int steps, int nparts, float **result) {
  const int m = G.rows, n = G.cols, cnt = G.count;
  const bool tall = m > n;
  const int r = tall ? n : m;
  const int64_t size = (int64_t)m * n, rr = (int64_t)r * r;
  hipLaunchKernelGGL(muon_normalize_k, dim3(sgrid(ctx, size / 4 + 1), cnt), dim3(256), 0, ctx->stream, size, G.U, G.part, nparts, G.X);
  GT_LAUNCHED(ctx);
  gt_buf bX = reinterpret_cast<gt_buf>(G.X), bY = reinterpret_cast<gt_buf>(G.BX), bA = reinterpret_cast<gt_buf>(G.A), bB = reinterpret_cast<gt_buf>(G.AA);
  for (int s = 0; s < steps; s++) {
    if (tall) { if (gt_gemm_batched(ctx, GT_TN, 0, r, r, m, bX, size, bX, size, bA, rr, cnt)) return 1; }       // A = X^T X
    else if (gt_gemm_batched(ctx, GT_NT, 0, r, r, n, bX, size, bX, size, bA, rr, cnt)) return 1;               // A = X X^T
    if (gemm_scaled_batched(ctx, GT_NN, r, r, r, bA, rr, bA, rr, bA, rr, NS_B, NS_C, bB, rr, cnt)) return 1;   // B = b A + c A.A
    if (tall) { if (gemm_scaled_batched(ctx, GT_NN, m, n, n, bX, size, bB, rr, bX, size, NS_A, 1.f, bY, size, cnt)) return 1; }   // a X + X.B
    else if (gemm_scaled_batched(ctx, GT_NN, m, n, m, bB, rr, bX, size, bX, size, NS_A, 1.f, bY, size, cnt)) return 1;          // a X + B.X
    std::swap(bX, bY);
  }
  *result = reinterpret_cast<float *>(bX);
  return 0;
}

static void group_release(gt_ctx *ctx, MuonGroup &G) {
  (void)hipStreamSynchronize(ctx->stream);
  float *bufs[] = {G.U, G.X, G.BX, G.A, G.AA, G.part};
  for (float *b : bufs) if (b) (void)hipFree(b);
  G.U = G.X = G.BX = G.A = G.AA = G.part = nullptr;
  if (G.w) (void)hipFree(G.w);
  if (G.g) (void)hipFree(G.g);
  if (G.buf) (void)hipFree(G.buf);
  G.w = G.g = G.buf = nullptr;
  ctx->live_bytes -= G.bytes;
  G.bytes = 0;
}
// all of a group's work buffers, or none (what one failed allocation leaves behind is freed)
static int group_alloc(gt_ctx *ctx, MuonGroup &G) {
  const size_t elems = (size_t)G.rows * G.cols * G.count, r = std::min(G.rows, G.cols);
  float **dst[] = {&G.U, &G.X, &G.BX, &G.A, &G.AA, &G.part};
  const size_t bytes[] = {elems * 4, elems * 4, elems * 4, r * r * G.count * 4, r * r * G.count * 4, (size_t)RED_BLOCKS * G.count * 4};
  for (int i = 0; i < 6; i++) {
    hipError_t e = hipMalloc((void **)dst[i], bytes[i]);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      group_release(ctx, G);
      GT_FAIL(ctx, "Muon work buffers: hipMalloc of %zu bytes failed: %s", bytes[i], hipGetErrorString(e));
    }
  }
  G.bytes = elems * 12 + r * r * G.count * 8 + (size_t)RED_BLOCKS * G.count * 4;
  ctx->live_bytes += G.bytes;
  return 0;
}

static void adamw_release(gt_adamw *o) {
  if (o->chunks) (void)hipFree(o->chunks);
  if (o->ptrs) (void)hipFree(o->ptrs);
  if (o->partial) (void)hipFree(o->partial);
  if (o->scale) (void)hipFree(o->scale);
  delete o;
}
static void muon_release(gt_ctx *ctx, gt_muon *o) {
  for (auto &G : o->groups) group_release(ctx, G);
  delete o;
}
// optimizers a caller never destroyed go with their context
void optim_release_all(gt_ctx *ctx) {
  for (void *o : ctx->adamws) adamw_release(static_cast<gt_adamw *>(o));
  for (void *o : ctx->muons) muon_release(ctx, static_cast<gt_muon *>(o));
  ctx->adamws.clear();
  ctx->muons.clear();
}

extern "C" {

int gt_adamw_create(gt_ctx *ctx, int n, const gt_buf *w, const gt_buf *g, const gt_buf *m, const gt_buf *v,
                    const int64_t *sizes, double beta1, double beta2, double eps, double weight_decay, double clip, gt_adamw **out) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && out && (n == 0 || (w && g && m && v && sizes)), "gt_adamw_create: bad arguments");
  gt_adamw *o = new gt_adamw();
  o->n = n; o->beta1 = beta1; o->beta2 = beta2; o->eps = eps; o->wd = weight_decay; o->clip = clip;
  std::vector<Chunk> ch;
  std::vector<TensorPtrs> tp(n);
  for (int i = 0; i < n; i++) {
    if (!(w[i] && g[i] && m[i] && v[i] && sizes[i] >= 0)) { delete o; GT_FAIL(ctx, "gt_adamw_create: tensor %d has a null buffer", i); }
    tp[i] = {P<float>(w[i]), P<float>(g[i]), P<float>(m[i]), P<float>(v[i])};
    o->total_elems += (double)sizes[i];
    for (int64_t off = 0; off < sizes[i]; off += CHUNK) ch.push_back({i, (int)std::min<int64_t>(CHUNK, sizes[i] - off), off});
  }
  o->nchunks = (int)ch.size();
  size_t cb = std::max<size_t>(1, ch.size()) * sizeof(Chunk), pb = std::max<size_t>(1, tp.size()) * sizeof(TensorPtrs);
  float one[2] = {1.0f, 0.0f};
  hipError_t e;
  if ((e = hipMalloc((void **)&o->chunks, cb)) != hipSuccess || (e = hipMalloc((void **)&o->ptrs, pb)) != hipSuccess ||
      (e = hipMalloc((void **)&o->partial, std::max<size_t>(1, ch.size()) * 4)) != hipSuccess ||
      (e = hipMalloc((void **)&o->scale, 8)) != hipSuccess ||
      (!ch.empty() && (e = hipMemcpy(o->chunks, ch.data(), ch.size() * sizeof(Chunk), hipMemcpyHostToDevice)) != hipSuccess) ||
      (!tp.empty() && (e = hipMemcpy(o->ptrs, tp.data(), tp.size() * sizeof(TensorPtrs), hipMemcpyHostToDevice)) != hipSuccess) ||
      (e = hipMemcpy(o->scale, one, 8, hipMemcpyHostToDevice)) != hipSuccess) {
    (void)hipGetLastError();
    adamw_release(o);
    GT_FAIL(ctx, "gt_adamw_create: setting up the chunk tables failed: %s", hipGetErrorString(e));
  }
  ctx->adamws.insert(o);
  *out = o;
  return 0;
}

int gt_grad_fold(gt_ctx *ctx, int n, const gt_buf *dst, const int *dst_acc, int nsrc, const gt_buf *src, const int64_t *sizes) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && nsrc >= 1 && nsrc <= FOLD_MAX_SRC && (n == 0 || (dst && dst_acc && src && sizes)),
             "gt_grad_fold: %d tensors with %d sources each (at most %d), or a null table", n, nsrc, FOLD_MAX_SRC);
  std::vector<Chunk> ch;
  std::vector<FoldPtrs> tp;
  double bytes = 0;
  for (int i = 0; i < n; i++) {
    FoldPtrs p;
    memset(&p, 0, sizeof p);
    p.dst = P<float>(dst[i]); p.acc = dst_acc[i];
    for (int s = 0; s < nsrc; s++)
      if (src[(size_t)i * nsrc + s]) p.src[p.nsrc++] = P<const float>(src[(size_t)i * nsrc + s]);     // absent ones are skipped
    GT_REQUIRE(ctx, dst[i] && sizes[i] >= 0, "gt_grad_fold: tensor %d has a null destination or a negative size", i);
    if (p.nsrc == 0 || sizes[i] == 0) continue;
    bytes += 4.0 * sizes[i] * (p.nsrc + 1 + (p.acc ? 1 : 0));
    const int t = (int)tp.size();
    tp.push_back(p);
    for (int64_t off = 0; off < sizes[i]; off += FOLD_CHUNK) ch.push_back({t, (int)std::min<int64_t>(FOLD_CHUNK, sizes[i] - off), off});
  }
  if (ch.empty()) return 0;
  // the tables ride in the context's workspace: the copies and the kernel are ordered on the stream with whatever used it
  // before and uses it next (the source vectors are pageable, so the copy has staged them when it returns)
  const size_t cb = (ch.size() * sizeof(Chunk) + 255) & ~(size_t)255, pb = tp.size() * sizeof(FoldPtrs);
  void *ws;
  if (gt_ws_reserve(ctx, cb + pb, &ws)) return 1;
  Chunk *dch = static_cast<Chunk *>(ws);
  FoldPtrs *dtp = reinterpret_cast<FoldPtrs *>(static_cast<char *>(ws) + cb);
  GT_HIP(ctx, hipMemcpyAsync(dch, ch.data(), ch.size() * sizeof(Chunk), hipMemcpyHostToDevice, ctx->stream));
  GT_HIP(ctx, hipMemcpyAsync(dtp, tp.data(), pb, hipMemcpyHostToDevice, ctx->stream));
  ProfScope ps(ctx, "grad.fold", bytes);
  hipLaunchKernelGGL(grad_fold_k, dim3((unsigned)ch.size()), dim3(256), 0, ctx->stream, dch, dtp);
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_adamw_step(gt_ctx *ctx, gt_adamw *o, double lr, double bc1, double bc2) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, o, "gt_adamw_step: null optimizer");
  GT_REQUIRE(ctx, bc1 > 0 && bc2 > 0, "gt_adamw_step: bias corrections must be positive");
  if (o->nchunks == 0) return 0;
  int64_t total = 0;
  ProfScope ps(ctx, "adamw", o->total_elems * (o->clip > 0 ? 32.0 : 28.0));   // g,m,v,w read; m,v,w written; +g for the norm
  (void)total;
  if (o->clip > 0) {
    hipLaunchKernelGGL(adamw_ssq_k, dim3(o->nchunks), dim3(256), 0, ctx->stream, o->chunks, o->ptrs, o->partial);
    GT_LAUNCHED(ctx);
    hipLaunchKernelGGL(adamw_scale_k, dim3(1), dim3(1024), 0, ctx->stream, o->nchunks, o->partial, (float)o->clip, o->scale);
    GT_LAUNCHED(ctx);
  }
  // every constant is formed in f64 and rounded to f32 once
  AdamH h{(float)o->beta1, (float)o->beta2, (float)(1.0 - o->beta1), (float)(1.0 - o->beta2), (float)o->eps, (float)o->wd,
          (float)lr, (float)(1.0 / bc1), (float)(1.0 / bc2)};
  hipLaunchKernelGGL(adamw_update_k, dim3(o->nchunks), dim3(256), 0, ctx->stream, o->chunks, o->ptrs, o->scale, h);
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_adamw_grad_norm(gt_ctx *ctx, gt_adamw *o, float *norm) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, o && norm, "gt_adamw_grad_norm: null argument");
  float s[2];
  GT_HIP(ctx, hipMemcpyAsync(s, o->scale, 8, hipMemcpyDeviceToHost, ctx->stream));
  GT_HIP(ctx, hipStreamSynchronize(ctx->stream));
  *norm = s[1];
  return 0;
}

int gt_adamw_destroy(gt_ctx *ctx, gt_adamw *o) {
  GT_ENTER(ctx);
  if (!o) return 0;
  GT_REQUIRE(ctx, ctx->adamws.erase(o) == 1, "gt_adamw_destroy: not an optimizer of this context");
  (void)hipStreamSynchronize(ctx->stream);
  adamw_release(o);
  return 0;
}

int gt_muon_create(gt_ctx *ctx, int n, const gt_buf *w, const gt_buf *g, const gt_buf *buf, const int *rows, const int *cols,
                   double momentum, int nesterov, int ns_steps, gt_muon **out) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, n >= 0 && out && ns_steps >= 0 && (n == 0 || (w && g && buf && rows && cols)), "gt_muon_create: bad arguments");
  for (int i = 0; i < n; i++)
    GT_REQUIRE(ctx, w[i] && g[i] && buf[i] && rows[i] >= 1 && cols[i] >= 1, "gt_muon_create: matrix %d is malformed", i);
  gt_muon *o = new gt_muon();
  o->momentum = (float)momentum; o->nesterov = nesterov; o->ns_steps = ns_steps;
  std::vector<char> placed(n, 0);
  for (int i = 0; i < n; i++) {
    if (placed[i]) continue;
    MuonGroup G;
    G.rows = rows[i]; G.cols = cols[i];
    std::vector<float *> pw, pg, pb;
    for (int j = i; j < n; j++)
      if (!placed[j] && rows[j] == G.rows && cols[j] == G.cols) {
        placed[j] = 1;
        pw.push_back(P<float>(w[j])); pg.push_back(P<float>(g[j])); pb.push_back(P<float>(buf[j]));
      }
    G.count = (int)pw.size();
    size_t tb = pw.size() * sizeof(float *);
    if (hipMalloc((void **)&G.w, tb) != hipSuccess || hipMalloc((void **)&G.g, tb) != hipSuccess ||
        hipMalloc((void **)&G.buf, tb) != hipSuccess || group_alloc(ctx, G) ||
        hipMemcpy(G.w, pw.data(), tb, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(G.g, pg.data(), tb, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(G.buf, pb.data(), tb, hipMemcpyHostToDevice) != hipSuccess) {
      (void)hipGetLastError();
      group_release(ctx, G);              // frees whichever of this group's buffers exist
      muon_release(ctx, o);
      GT_FAIL(ctx, "gt_muon_create: setting up the %dx%d group failed (out of device memory?)", G.rows, G.cols);
    }
    o->groups.push_back(G);
  }
  ctx->muons.insert(o);
  *out = o;
  return 0;
}

int gt_muon_step(gt_ctx *ctx, gt_muon *o, double lr) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, o, "gt_muon_step: null optimizer");
  ProfScope ps(ctx, "muon");
  for (auto &G : o->groups) {
    const int64_t size = (int64_t)G.rows * G.cols;
    const unsigned nb = (unsigned)std::min<int64_t>(RED_BLOCKS, cdiv(size, 1024));
    hipLaunchKernelGGL(muon_momentum_k, dim3(nb, G.count), dim3(256), 0, ctx->stream, size, G.g, G.buf, G.U, o->momentum, o->nesterov, G.part);
    GT_LAUNCHED(ctx);
    float *X = nullptr;
    if (newton_schulz_run(ctx, G, o->ns_steps, (int)nb, &X)) return 1;
    const float f = (float)(lr * sqrt(std::max(1.0, (double)G.rows / (double)G.cols)));
    hipLaunchKernelGGL(muon_apply_k, dim3(sgrid(ctx, size / 4 + 1), G.count), dim3(256), 0, ctx->stream, size, G.w, (float *)nullptr, X, f);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

int gt_muon_destroy(gt_ctx *ctx, gt_muon *o) {
  GT_ENTER(ctx);
  if (!o) return 0;
  GT_REQUIRE(ctx, ctx->muons.erase(o) == 1, "gt_muon_destroy: not an optimizer of this context");
  muon_release(ctx, o);
  return 0;
}

int gt_newton_schulz(gt_ctx *ctx, int m, int n, int steps, gt_buf G, gt_buf out) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, m >= 1 && n >= 1 && steps >= 0 && G && out, "gt_newton_schulz: bad arguments");
  ProfScope ps(ctx, "muon");
  MuonGroup T;
  T.rows = m; T.cols = n; T.count = 1;
  if (group_alloc(ctx, T)) return 1;
  const size_t size = (size_t)m * n;
  hipError_t ce = hipMemcpyAsync(T.U, P<void>(G), size * 4, hipMemcpyDeviceToDevice, ctx->stream);
  if (ce != hipSuccess) {
    group_release(ctx, T);
    GT_FAIL(ctx, "gt_newton_schulz: copying the matrix failed: %s", hipGetErrorString(ce));
  }
  const unsigned nb = (unsigned)std::min<int64_t>(RED_BLOCKS, cdiv((int64_t)size, 1024));
  // sums of squares of U only (no momentum buffer, no gradient)
  hipLaunchKernelGGL(muon_momentum_k, dim3(nb, 1), dim3(256), 0, ctx->stream, (int64_t)size, (float *const *)nullptr,
                     (float *const *)nullptr, T.U, 0.f, 0, T.part);
  int rc = hipGetLastError() != hipSuccess;
  float *X = nullptr;
  if (!rc) rc = newton_schulz_run(ctx, T, steps, (int)nb, &X);
  if (!rc) rc = hipMemcpyAsync(P<void>(out), X, size * 4, hipMemcpyDeviceToDevice, ctx->stream) != hipSuccess;
  group_release(ctx, T);
  return rc;
}
}
