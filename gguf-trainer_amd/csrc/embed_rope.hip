// Embedding gather / scatter-add (srcEmbeddingFwd / Bwd, src/backend/wgsl.ts:305-344) and RoPE
// (srcRope, wgsl.ts:346-384).
//
// Embedding backward. The reference gives one thread to every (vocab row, column) and scans all T
// ids: V*d*T work. Here the ids are ranked on the device (a stable counting rank, O(T^2) integer
// compares over LDS-staged tiles), which yields the tokens grouped by id in position order; one
// workgroup per distinct id then sums that id's gradient rows in that fixed order and adds the
// sum to its dW row. No atomics, no dependence on launch timing, repeated ids (Zipf) included.
//
// RoPE. cos/sin per (position, pair) are computed once per (T, hd, base, pos) in f64 and kept as
// an f32 table in the context, like the reference CPU op's precomputed Float32Array tables
// (src/model/autograd.ts:590-601); evaluating pow/cos/sin in f32 per element, as the WGSL does,
// loses ~1e-4 at position 2047.
#include <algorithm>
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void embedding_fwd_k(int rows, int d, int V, const int *__restrict__ ids,
                                                       const float *__restrict__ W, float *__restrict__ out, int *bad) {
  // one wavefront per row, float4 when d % 4 == 0
  const int lane = threadIdx.x % WAVE;
  int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (row >= rows) return;
  const int id = ids[row];
  float *dst = out + row * d;
  if (id < 0 || id >= V) {                      // no such table row: the output row is zero and the host hears of it
    if (lane == 0) note_bad_id(bad, GT_BAD_EMBED_ID, row, id, V);
    for (int j = lane; j < d; j += WAVE) dst[j] = 0.f;
    return;
  }
  const float *src = W + (size_t)id * d;
  if (d % 4 == 0) {
    for (int j = lane; j < d / 4; j += WAVE) reinterpret_cast<v4f *>(dst)[j] = reinterpret_cast<const v4f *>(src)[j];
  } else {
    for (int j = lane; j < d; j += WAVE) dst[j] = src[j];
  }
}

// pos[t] = #{t' : id[t'] < id[t]} + #{t' < t : id[t'] == id[t]}: the stable sorted position. The T x T compare is
// split over blockIdx.y segments of the t' range; the per-segment counts are integers, so adding them into pos[]
// with atomicAdd is exact and order-independent (the float sums further down never use atomics).
__global__ __launch_bounds__(256) void rank_ids_k(int n, int seg, const int *__restrict__ ids, int *__restrict__ pos) {
  __shared__ int tile[256];
  int t = blockIdx.x * 256 + threadIdx.x;
  int mine = t < n ? ids[t] : 0x7fffffff;
  int cnt = 0;
  int b0 = blockIdx.y * seg, b1 = min(n, b0 + seg);
  for (int base = b0; base < b1; base += 256) {
    int j = base + threadIdx.x;
    __syncthreads();
    tile[threadIdx.x] = j < b1 ? ids[j] : 0x7fffffff;
    __syncthreads();
    int lim = min(256, b1 - base);
    for (int q = 0; q < lim; q++) {
      int o = tile[q];
      cnt += (o < mine) || (o == mine && base + q < t);
    }
  }
  if (t < n && cnt) atomicAdd(pos + t, cnt);
}
__global__ __launch_bounds__(256) void scatter_ids_k(int n, const int *__restrict__ ids, const int *__restrict__ pos,
                                                     int *__restrict__ order, int *__restrict__ sorted) {
  int t = blockIdx.x * 256 + threadIdx.x;
  if (t < n) { order[pos[t]] = t; sorted[pos[t]] = ids[t]; }
}

// one workgroup per sorted slot; only the first slot of each id does work: it sums that id's gradient rows in
// position order (eight row loads in flight per thread) and adds the sum to the id's dW row
__global__ __launch_bounds__(256) void embedding_bwd_k(int n, int d, int V, const int *__restrict__ order,
                                                       const int *__restrict__ sorted, const float *__restrict__ g,
                                                       float *dW, int *bad) {
  int p = blockIdx.x;
  int id = sorted[p];
  if (p > 0 && sorted[p - 1] == id) return;
  if (id < 0 || id >= V) {                      // no such dW row: nothing is added
    if (threadIdx.x == 0) note_bad_id(bad, GT_BAD_EMBED_ID, order[p], id, V);
    return;
  }
  int e = p + 1;
  while (e < n && sorted[e] == id) e++;
  float *dst = dW + (size_t)id * d;
  if (d % 4 == 0) {
    for (int c = threadIdx.x; c < d / 4; c += 256) {
      v4f s = {0, 0, 0, 0};
      int q = p;
      for (; q + 8 <= e; q += 8) {
        v4f r[8];
#pragma unroll
        for (int u = 0; u < 8; u++) r[u] = reinterpret_cast<const v4f *>(g + (size_t)order[q + u] * d)[c];
#pragma unroll
        for (int u = 0; u < 8; u++) s += r[u];
      }
      for (; q < e; q++) s += reinterpret_cast<const v4f *>(g + (size_t)order[q] * d)[c];
      reinterpret_cast<v4f *>(dst)[c] += s;
    }
  } else {
    for (int c = threadIdx.x; c < d; c += 256) {
      float s = 0;
      for (int q = p; q < e; q++) s += g[(size_t)order[q] * d + c];
      dst[c] += s;
    }
  }
}

// ---- RoPE ------------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void rope_table_k(int T, int hd, double base, int pos, float *__restrict__ tab) {
  int half = hd / 2;
  int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= T * half) return;
  int t = i / half, j = i % half;
  double freq = pow(base, (-2.0 * j) / hd);
  double ang = (double)(t + pos) * freq;
  tab[2 * i] = (float)cos(ang);
  tab[2 * i + 1] = (float)sin(ang);
}

template <bool BWD>
__global__ __launch_bounds__(256) void rope_k(int64_t npairs, int T, int H, int hd, const float2 *__restrict__ tab,
                                              const float *__restrict__ in, float *out, int acc) {
  int half = hd / 2;
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < npairs; i += stride) {
    int j = (int)(i % half);
    int64_t rh = i / half;                        // row*H + h
    int64_t row = rh / H;
    int t = (int)(row % T);
    float2 cs = tab[(size_t)t * half + j];
    int64_t b = rh * hd + j;
    float a0 = in[b], a1 = in[b + half], o0, o1;
    if (!BWD) { o0 = a0 * cs.x - a1 * cs.y; o1 = a0 * cs.y + a1 * cs.x; }
    else { o0 = cs.x * a0 + cs.y * a1; o1 = -cs.y * a0 + cs.x * a1; }
    if (acc) { o0 += out[b]; o1 += out[b + half]; }
    out[b] = o0;
    out[b + half] = o1;
  }
}

// The same rotation four pairs at a time for hd % 8 == 0: a thread takes four consecutive j of one (row, head), i.e.
// one float4 of each half of the head and two float4 of the table, with 32-bit index arithmetic (the scalar kernel's
// 64-bit divisions cost more than its memory traffic). Two units per thread and pass, all loads before the first use.
template <bool BWD>
__global__ __launch_bounds__(256) void rope_vec_k(unsigned nunits, int T, int H, int hd, const float *__restrict__ tab,
                                                  const float *__restrict__ in, float *out, int acc) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const unsigned q = (unsigned)hd / 8;                    // float4 units per half head
  const unsigned stride = gridDim.x * 256;
  for (unsigned i0 = blockIdx.x * 256 + threadIdx.x; i0 < nunits; i0 += 2 * stride) {
    f4 a0[2], a1[2], c0[2], c1[2], o0[2], o1[2];
    size_t off[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const unsigned i = min(i0 + u * stride, nunits - 1);
      const unsigned rh = i / q, j4 = i - rh * q;           // rh = row*H + h
      const unsigned row = rh / (unsigned)H, t = row % (unsigned)T;
      off[u] = (size_t)rh * hd + 4 * j4;
      const f4 *tp = reinterpret_cast<const f4 *>(tab + ((size_t)t * (hd / 2) + 4 * j4) * 2);
      a0[u] = *reinterpret_cast<const f4 *>(in + off[u]);
      a1[u] = *reinterpret_cast<const f4 *>(in + off[u] + hd / 2);
      c0[u] = tp[0];                                        // cos, sin of pairs j, j+1
      c1[u] = tp[1];                                        // and of pairs j+2, j+3
      if (acc) {
        o0[u] = *reinterpret_cast<const f4 *>(out + off[u]);
        o1[u] = *reinterpret_cast<const f4 *>(out + off[u] + hd / 2);
      }
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      if (i0 + u * stride >= nunits) continue;
      const f4 cs = {c0[u][0], c0[u][2], c1[u][0], c1[u][2]}, sn = {c0[u][1], c0[u][3], c1[u][1], c1[u][3]};
      f4 r0, r1;
      if (!BWD) { r0 = a0[u] * cs - a1[u] * sn; r1 = a0[u] * sn + a1[u] * cs; }
      else { r0 = cs * a0[u] + sn * a1[u]; r1 = -sn * a0[u] + cs * a1[u]; }
      if (acc) { r0 += o0[u]; r1 += o1[u]; }
      *reinterpret_cast<f4 *>(out + off[u]) = r0;
      *reinterpret_cast<f4 *>(out + off[u] + hd / 2) = r1;
    }
  }
}

// The same rotation over two tensors that share rows, T, hd and the table (q and k of a layer) in one launch: units
// [0, n1) belong to the first, [n1, n1 + n2) to the second. Per element the arithmetic is rope_vec_k's.
struct RopeT { const float *in; float *out; int H, acc; };
template <bool BWD>
__global__ __launch_bounds__(256) void rope_vec2_k(unsigned n1, unsigned n2, int T, int hd, const float *__restrict__ tab, RopeT A, RopeT B) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const unsigned q = (unsigned)hd / 8;                    // float4 units per half head
  const unsigned stride = gridDim.x * 256, nunits = n1 + n2;
  for (unsigned i0 = blockIdx.x * 256 + threadIdx.x; i0 < nunits; i0 += 2 * stride) {
    f4 a0[2], a1[2], c0[2], c1[2], o0[2], o1[2];
    float *op[2];
    bool ac[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const unsigned ig = min(i0 + u * stride, nunits - 1);
      const bool second = ig >= n1;
      const unsigned i = second ? ig - n1 : ig;
      const unsigned H = (unsigned)(second ? B.H : A.H);
      const float *in = second ? B.in : A.in;
      ac[u] = (second ? B.acc : A.acc) != 0;
      const unsigned rh = i / q, j4 = i - rh * q;           // rh = row*H + h
      const unsigned row = rh / H, t = row % (unsigned)T;
      const size_t off = (size_t)rh * hd + 4 * j4;
      op[u] = (second ? B.out : A.out) + off;
      const f4 *tp = reinterpret_cast<const f4 *>(tab + ((size_t)t * (hd / 2) + 4 * j4) * 2);
      a0[u] = *reinterpret_cast<const f4 *>(in + off);
      a1[u] = *reinterpret_cast<const f4 *>(in + off + hd / 2);
      c0[u] = tp[0];                                        // cos, sin of pairs j, j+1
      c1[u] = tp[1];                                        // and of pairs j+2, j+3
      if (ac[u]) {
        o0[u] = *reinterpret_cast<const f4 *>(op[u]);
        o1[u] = *reinterpret_cast<const f4 *>(op[u] + hd / 2);
      }
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      if (i0 + u * stride >= nunits) continue;
      const f4 cs = {c0[u][0], c0[u][2], c1[u][0], c1[u][2]}, sn = {c0[u][1], c0[u][3], c1[u][1], c1[u][3]};
      f4 r0, r1;
      if (!BWD) { r0 = a0[u] * cs - a1[u] * sn; r1 = a0[u] * sn + a1[u] * cs; }
      else { r0 = cs * a0[u] + sn * a1[u]; r1 = -sn * a0[u] + cs * a1[u]; }
      if (ac[u]) { r0 += o0[u]; r1 += o1[u]; }
      *reinterpret_cast<f4 *>(op[u]) = r0;
      *reinterpret_cast<f4 *>(op[u] + hd / 2) = r1;
    }
  }
}

extern "C" {
int gt_embedding_fwd(gt_ctx *ctx, int rows, int d, int V, gt_buf ids, gt_buf W, gt_buf out) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && V >= 1 && ids && W && out, "gt_embedding_fwd: bad arguments");
  if (rows == 0) return 0;
  ProfScope ps(ctx, "embedding");
  hipLaunchKernelGGL(embedding_fwd_k, dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, ctx->stream, rows, d, V, P<const int>(ids),
                     P<const float>(W), P<float>(out), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_embedding_bwd(gt_ctx *ctx, int rows, int d, int V, gt_buf ids, gt_buf g, gt_buf dW, int acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && d >= 1 && V >= 1 && ids && g && dW, "gt_embedding_bwd: bad arguments");
  ProfScope ps(ctx, "embedding.bwd", 8.0 * rows * d);
  if (!acc) GT_HIP(ctx, hipMemsetAsync(P<void>(dW), 0, (size_t)V * d * sizeof(float), ctx->stream));
  if (rows == 0) return 0;
  GT_REQUIRE(ctx, (g | dW) % 16 == 0, "gt_embedding_bwd: buffers must be 16-byte aligned");
  void *ws;
  if (gt_ws_reserve(ctx, (size_t)rows * 3 * sizeof(int), &ws)) return 1;
  int *order = static_cast<int *>(ws), *sorted = order + rows, *pos = sorted + rows;
  GT_HIP(ctx, hipMemsetAsync(pos, 0, (size_t)rows * sizeof(int), ctx->stream));
  const int nseg = (int)std::max<int64_t>(1, std::min<int64_t>(32, cdiv(rows, 1024)));
  const int seg = (int)(cdiv(cdiv(rows, nseg), 256) * 256);
  hipLaunchKernelGGL(rank_ids_k, dim3((unsigned)cdiv(rows, 256), (unsigned)cdiv(rows, seg)), dim3(256), 0, ctx->stream, rows, seg,
                     P<const int>(ids), pos);
  GT_LAUNCHED(ctx);
  hipLaunchKernelGGL(scatter_ids_k, dim3((unsigned)cdiv(rows, 256)), dim3(256), 0, ctx->stream, rows, P<const int>(ids), pos, order, sorted);
  GT_LAUNCHED(ctx);
  hipLaunchKernelGGL(embedding_bwd_k, dim3((unsigned)rows), dim3(256), 0, ctx->stream, rows, d, V, order, sorted,
                     P<const float>(g), P<float>(dW), ctx->bad_dev);
  GT_LAUNCHED(ctx);
  return 0;
}

static int rope_table(gt_ctx *ctx, int T, int hd, double base, int pos, float **out) {
  gt_ctx::RopeKey key{T, hd, pos, base};
  auto it = ctx->rope_tables.find(key);
  if (it != ctx->rope_tables.end()) { *out = it->second; return 0; }
  float *tab;
  int n = T * (hd / 2);
  GT_HIP(ctx, hipMalloc(reinterpret_cast<void **>(&tab), (size_t)n * 2 * sizeof(float)));
  hipLaunchKernelGGL(rope_table_k, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, ctx->stream, T, hd, base, pos, tab);
  GT_LAUNCHED(ctx);
  ctx->rope_tables[key] = tab;
  *out = tab;
  return 0;
}

}
int rope_table_get(gt_ctx *ctx, int T, int hd, double base, int pos, float **out) { return rope_table(ctx, T, hd, base, pos, out); }
extern "C" {

int gt_rope(gt_ctx *ctx, int rows, int T, int H, int hd, double base, int pos, int backward, gt_buf in, gt_buf out, int acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && T >= 1 && H >= 1 && hd >= 2 && hd % 2 == 0 && in && out, "gt_rope: bad arguments (hd %d)", hd);
  GT_REQUIRE(ctx, rows % T == 0, "gt_rope: rows %d is not a whole number of sequences of %d", rows, T);
  if (rows == 0) return 0;
  ProfScope ps(ctx, backward ? "rope.bwd" : "rope", 8.0 * rows * H * hd);
  float *tab;
  if (rope_table(ctx, T, hd, base, pos, &tab)) return 1;
  int64_t npairs = (int64_t)rows * H * (hd / 2);
  if (hd % 8 == 0 && npairs / 4 < ((int64_t)1 << 31) && (in | out) % 16 == 0) {
    const unsigned nunits = (unsigned)(npairs / 4);
    const unsigned nbv = (unsigned)std::min<int64_t>(cdiv(nunits, 512), (int64_t)ctx->num_cu * 16);
    if (backward)
      hipLaunchKernelGGL((rope_vec_k<true>), dim3(nbv), dim3(256), 0, ctx->stream, nunits, T, H, hd, tab, P<const float>(in), P<float>(out), acc);
    else
      hipLaunchKernelGGL((rope_vec_k<false>), dim3(nbv), dim3(256), 0, ctx->stream, nunits, T, H, hd, tab, P<const float>(in), P<float>(out), acc);
    GT_LAUNCHED(ctx);
    return 0;
  }
  unsigned nb = (unsigned)std::min<int64_t>(cdiv(npairs, 256), (int64_t)ctx->num_cu * 16);
  if (backward)
    hipLaunchKernelGGL((rope_k<true>), dim3(nb), dim3(256), 0, ctx->stream, npairs, T, H, hd, reinterpret_cast<const float2 *>(tab),
                       P<const float>(in), P<float>(out), acc);
  else
    hipLaunchKernelGGL((rope_k<false>), dim3(nb), dim3(256), 0, ctx->stream, npairs, T, H, hd, reinterpret_cast<const float2 *>(tab),
                       P<const float>(in), P<float>(out), acc);
  GT_LAUNCHED(ctx);
  return 0;
}

int gt_rope_pair(gt_ctx *ctx, int rows, int T, int hd, double base, int pos, int backward, int H1, gt_buf in1, gt_buf out1, int acc1, int H2,
                 gt_buf in2, gt_buf out2, int acc2) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, rows >= 0 && T >= 1 && H1 >= 1 && H2 >= 1 && hd >= 2 && hd % 2 == 0 && in1 && out1 && in2 && out2,
             "gt_rope_pair: bad arguments (hd %d)", hd);
  GT_REQUIRE(ctx, rows % T == 0, "gt_rope_pair: rows %d is not a whole number of sequences of %d", rows, T);
  if (rows == 0) return 0;
  const int64_t u1 = (int64_t)rows * H1 * (hd / 2) / 4, u2 = (int64_t)rows * H2 * (hd / 2) / 4;
  if (!(hd % 8 == 0 && u1 + u2 < ((int64_t)1 << 31) && (in1 | out1 | in2 | out2) % 16 == 0)) {     // the shapes the one-tensor kernels take
    if (gt_rope(ctx, rows, T, H1, hd, base, pos, backward, in1, out1, acc1)) return 1;
    return gt_rope(ctx, rows, T, H2, hd, base, pos, backward, in2, out2, acc2);
  }
  ProfScope ps(ctx, backward ? "rope.bwd" : "rope", 8.0 * rows * (H1 + H2) * hd);
  float *tab;
  if (rope_table(ctx, T, hd, base, pos, &tab)) return 1;
  const unsigned nbv = (unsigned)std::min<int64_t>(cdiv(u1 + u2, 512), (int64_t)ctx->num_cu * 16);
  RopeT A{P<const float>(in1), P<float>(out1), H1, acc1}, B{P<const float>(in2), P<float>(out2), H2, acc2};
  if (backward) hipLaunchKernelGGL((rope_vec2_k<true>), dim3(nbv), dim3(256), 0, ctx->stream, (unsigned)u1, (unsigned)u2, T, hd, tab, A, B);
  else hipLaunchKernelGGL((rope_vec2_k<false>), dim3(nbv), dim3(256), 0, ctx->stream, (unsigned)u1, (unsigned)u2, T, hd, tab, A, B);
  GT_LAUNCHED(ctx);
  return 0;
}
}
