// Shared by every translation unit of libggufhip: the context, error plumbing, launch helpers
// and wavefront (64-lane) reductions. gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "../../include/ggufhip.h"

#define WAVE 64

struct ProfEvent { std::string label; hipEvent_t a, b; double work; };

struct gt_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  char err[512] = {0};
  char name[256] = {0};
  int num_cu = 256;
  uint64_t live_bytes = 0;
  std::map<uint64_t, size_t> allocs;
  std::set<void *> adamws, muons;              // live optimizer objects: gt_ctx_destroy releases what the caller did not
  // grow-only scratch for kernels that need more than inputs and outputs (split-K partials,
  // per-block dw partials, embedding sort keys). One stream => one user at a time.
  void *ws = nullptr; size_t ws_bytes = 0;
  // RoPE cos/sin tables keyed by (T, hd, base, pos): computed once in f64, kept as f32.
  struct RopeKey { int T, hd, pos; double base; bool operator<(const RopeKey &o) const {
    if (T != o.T) return T < o.T; if (hd != o.hd) return hd < o.hd; if (pos != o.pos) return pos < o.pos; return base < o.base; } };
  std::map<RopeKey, float *> rope_tables;
  int opt_attn_generic = 0, opt_gemm_tile = -1, opt_gemm_splitk = -1, opt_attn_splits = -1, opt_gemm_staged = 0;
  int opt_gemm_group = 1;                       // 0: gt_gemm_group launches its products one by one
  int opt_attn_pieces = 0;                      // 1: attention forward and the banded dQ product (head dims 64, 128) and dK/dV (64) on the bf16 matrix instruction too
  int opt_gemm_split = 0;                       // 1: aligned FP32 products run as six bf16 MFMA products of three-piece operands
  int opt_attn_keep_ds = 1, opt_attn_ds_limit_mb = 8192, opt_gemm_sum_min_tiles = -1;
  int opt_attn_band_splits = -1;       // parts the banded dQ product cuts its K ranges into (-1: chosen from the launch's size)
  bool prof_on = false;
  std::string prof_prefix;
  std::vector<ProfEvent> prof;
  unsigned attn_smem_set = 0;                   // head dims whose attention kernels have their LDS size attribute set: bits 32 | 64 | 128 dK/dV, the same << 8 forward
  uint64_t gemm_direct_set = 0;                 // direct-to-LDS GEMM variants whose LDS size attribute is set
  uint64_t gemm_split_set = 0;                  // the same for the bf16-piece variants
  int opt_prof_sample = 1;                      // events around every n-th launch of a label
  // Pinned host words a kernel writes when it meets an id / target outside its range (it skips that row):
  // [0] = which check (GT_BAD_*), [1] = row, [2] = the value, [3] = the bound. Read after the stream has drained.
  int *bad_host = nullptr, *bad_dev = nullptr;
  float *rms_static = nullptr;                  // this device's address of norm.hip's static scratch array
  bool rms_static_pending = false;              // a gt_rmsnorm_bwd_static call is queued on this stream and the stream has not been waited for since
  hipEvent_t timer_a = nullptr, timer_b = nullptr;   // gt_timer_start / gt_timer_stop
  hipEvent_t mark = nullptr;                    // gt_stream_mark records it, another context's gt_stream_wait waits for it
  struct ProfSeen { int64_t n = 0; double work = 0; };
  std::map<std::string, ProfSeen> prof_seen;    // launches and their work per label since gt_prof_begin, timed or not
};

extern thread_local char g_create_err[512];

#define GT_FAIL(ctx, ...) do { snprintf((ctx)->err, sizeof((ctx)->err), __VA_ARGS__); return 1; } while (0)
#define GT_HIP(ctx, call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { \
  snprintf((ctx)->err, sizeof((ctx)->err), "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
  return 1; } } while (0)
// after a launch: a bad configuration shows here, a fault inside the kernel at the next sync
#define GT_LAUNCHED(ctx) GT_HIP(ctx, hipGetLastError())
#define GT_ENTER(ctx) do { if (!(ctx)) return 1; GT_HIP(ctx, hipSetDevice((ctx)->device)); } while (0)
#define GT_REQUIRE(ctx, cond, ...) do { if (!(cond)) GT_FAIL(ctx, __VA_ARGS__); } while (0)

int gt_ws_reserve(gt_ctx *ctx, size_t bytes, void **out);
// ids, targets and teacher ids live on the device, so the host cannot look at them before a launch: a kernel that meets
// one outside its range skips the row and notes it here; gt_sync / gt_d2h / gt_prof_end then fail once with that note.
enum { GT_BAD_EMBED_ID = 1, GT_BAD_TARGET = 2, GT_BAD_TEACHER_ID = 3 };
__device__ __forceinline__ void note_bad_id(int *bad, int what, int64_t row, int value, int bound) {
  bad[1] = (int)row; bad[2] = value; bad[3] = bound; bad[0] = what;
}
int gt_report_bad_id(gt_ctx *ctx);
void optim_release_all(gt_ctx *ctx);            // optim.hip
int rmsnorm_static_init(gt_ctx *ctx);           // norm.hip: looks up the static scratch array's address on ctx's device
void rmsnorm_static_forget(gt_ctx *ctx);        // norm.hip: ctx is going away and must not be remembered as the array's last user
// gemm.hip: C_i = dscale * D_i + pscale * A_i.B_i, a batch of `count` products of one kind (strides in elements)
int gemm_scaled_batched(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, int64_t sA, gt_buf B, int64_t sB, gt_buf D, int64_t sD,
                        float dscale, float pscale, gt_buf C, int64_t sC, int count);
// gemm.hip: dQ (+)= dS.K per (sequence, head) over each row tile's band of visible keys
// rot: the rotation table of the rope the query rows went through ([T][hd/2] (cos, sin) pairs), when dQ is wanted with respect
// to the rows before that rotation (the write-back then applies the rotation's backward), else null
int gemm_band_dq_splits(gt_ctx *ctx, int B, int T, int Hq, int window);
int gemm_band_dq(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, const float *dS, const float *K, float *dQ, int acc,
                 const float *rot = nullptr, float *parts = nullptr, int splits = 1);
// embed_rope.hip: the (cos, sin) table of a rotation, built once per (T, hd, base, pos) and kept with the context
int rope_table_get(gt_ctx *ctx, int T, int hd, double base, int pos, float **out);

// Brackets the launches made during its lifetime with a pair of events when profiling is on.
struct ProfScope {
  gt_ctx *c; bool on; size_t idx = 0;
  ProfScope(gt_ctx *ctx, const char *label, double work = 0) : c(ctx), on(ctx->prof_on) {
    if (on && !ctx->prof_prefix.empty() && strncmp(label, ctx->prof_prefix.c_str(), ctx->prof_prefix.size()) != 0) on = false;
    if (!on) return;
    // an event pair costs the stream about as much as a small kernel: with sampling only about 1 in n launches of a
    // label is timed and gt_prof_end scales the timed sum up to the work of all of them. Which launches: a fixed
    // pseudo-random choice over the label's launch numbers, so that a label whose launches cycle through a few
    // shapes is not sampled in step with the cycle.
    auto &seen = ctx->prof_seen[label];
    const uint32_t nth = (uint32_t)(seen.n++);
    seen.work += work;
    if (ctx->opt_prof_sample > 1 && ((nth * 2654435761u) >> 15) % (uint32_t)ctx->opt_prof_sample != 0) { on = false; return; }
    ProfEvent e; e.label = label; e.work = work;
    (void)hipEventCreate(&e.a); (void)hipEventCreate(&e.b);
    (void)hipEventRecord(e.a, c->stream);
    c->prof.push_back(e);
    idx = c->prof.size() - 1;
  }
  ~ProfScope() { if (on) (void)hipEventRecord(c->prof[idx].b, c->stream); }
};

template <typename T> static inline T *P(gt_buf b) { return reinterpret_cast<T *>(b); }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}
// Sum over a block of NW wavefronts; every thread gets the result. `sm` holds NW floats.
template <int NW> __device__ __forceinline__ float block_sum(float v, float *sm) {
  v = wave_sum(v);
  int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) sm[w] = v;
  __syncthreads();
  float r = 0;
#pragma unroll
  for (int i = 0; i < NW; i++) r += sm[i];
  return r;
}
template <int NW> __device__ __forceinline__ float block_max(float v, float *sm) {
  v = wave_max(v);
  int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) sm[w] = v;
  __syncthreads();
  float r = sm[0];
#pragma unroll
  for (int i = 1; i < NW; i++) r = fmaxf(r, sm[i]);
  return r;
}
