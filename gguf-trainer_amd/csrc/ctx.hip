// Context, device memory, transfers, profiling records.
#include "common.h"

thread_local char g_create_err[512] = {0};

extern "C" {

static void ctx_release(gt_ctx *c) {
  if (c->ws) hipFree(c->ws);
  if (c->bad_host) hipHostFree(c->bad_host);
  if (c->mark) hipEventDestroy(c->mark);
  if (c->timer_a) hipEventDestroy(c->timer_a);
  if (c->timer_b) hipEventDestroy(c->timer_b);
  if (c->stream) hipStreamDestroy(c->stream);
  delete c;
}

int gt_ctx_create(int device, gt_ctx **out) {
  if (!out) return 1;
  *out = nullptr;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    snprintf(g_create_err, sizeof g_create_err, "no HIP device available (%s)", hipGetErrorString(e));
    return 1;
  }
  if (device < 0 || device >= n) {
    snprintf(g_create_err, sizeof g_create_err, "device %d out of range (%d visible)", device, n);
    return 1;
  }
  gt_ctx *c = new gt_ctx();
  c->device = device;
  hipDeviceProp_t p;
  if ((e = hipSetDevice(device)) != hipSuccess || (e = hipGetDeviceProperties(&p, device)) != hipSuccess) {
    snprintf(g_create_err, sizeof g_create_err, "context setup failed: %s", hipGetErrorString(e));
    ctx_release(c);
    return 1;
  }
  snprintf(c->name, sizeof c->name, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
  c->num_cu = p.multiProcessorCount;
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    snprintf(g_create_err, sizeof g_create_err, "libggufhip is built for gfx950 only; device is %s", p.gcnArchName);
    ctx_release(c);
    return 1;
  }
  // the stream, and the pinned words kernels note an out-of-range id in
  if ((e = hipStreamCreate(&c->stream)) != hipSuccess ||
      (e = hipEventCreateWithFlags(&c->mark, hipEventDisableTiming)) != hipSuccess ||
      (e = hipHostMalloc(reinterpret_cast<void **>(&c->bad_host), 4 * sizeof(int), hipHostMallocMapped)) != hipSuccess ||
      (e = hipHostGetDevicePointer(reinterpret_cast<void **>(&c->bad_dev), c->bad_host, 0)) != hipSuccess) {
    snprintf(g_create_err, sizeof g_create_err, "context setup failed: %s", hipGetErrorString(e));
    ctx_release(c);
    return 1;
  }
  memset(c->bad_host, 0, 4 * sizeof(int));
  if (rmsnorm_static_init(c)) {
    snprintf(g_create_err, sizeof g_create_err, "context setup failed: %s", c->err);
    ctx_release(c);
    return 1;
  }
  *out = c;
  return 0;
}

int gt_ctx_destroy(gt_ctx *ctx) {
  if (!ctx) return 0;
  hipSetDevice(ctx->device);
  hipStreamSynchronize(ctx->stream);
  rmsnorm_static_forget(ctx);
  optim_release_all(ctx);
  for (auto &kv : ctx->allocs) hipFree(reinterpret_cast<void *>(kv.first));
  for (auto &kv : ctx->rope_tables) hipFree(kv.second);
  for (auto &e : ctx->prof) { hipEventDestroy(e.a); hipEventDestroy(e.b); }
  ctx_release(ctx);
  return 0;
}

const char *gt_last_error(gt_ctx *ctx) { return ctx ? ctx->err : g_create_err; }
const char *gt_device_name(gt_ctx *ctx) { return ctx ? ctx->name : ""; }

int gt_alloc(gt_ctx *ctx, size_t bytes, int zero, gt_buf *out) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, out, "gt_alloc: out is NULL");
  void *p = nullptr;
  size_t sz = bytes ? bytes : 4;
  hipError_t e = hipMalloc(&p, sz);
  if (e != hipSuccess) {
    (void)hipGetLastError();       // a caller may free memory and ask again: the next launch check must not report this failure
    GT_FAIL(ctx, "gt_alloc: hipMalloc of %zu bytes failed: %s", sz, hipGetErrorString(e));
  }
  if (zero) GT_HIP(ctx, hipMemsetAsync(p, 0, sz, ctx->stream));
  ctx->allocs[reinterpret_cast<uint64_t>(p)] = sz;
  ctx->live_bytes += sz;
  *out = reinterpret_cast<uint64_t>(p);
  return 0;
}

int gt_free(gt_ctx *ctx, gt_buf buf) {
  GT_ENTER(ctx);
  auto it = ctx->allocs.find(buf);
  GT_REQUIRE(ctx, it != ctx->allocs.end(), "gt_free: %llx was not returned by gt_alloc", (unsigned long long)buf);
  GT_HIP(ctx, hipStreamSynchronize(ctx->stream));      // nothing queued may still touch it
  GT_HIP(ctx, hipFree(reinterpret_cast<void *>(buf)));
  ctx->live_bytes -= it->second;
  ctx->allocs.erase(it);
  return 0;
}

int gt_memset0(gt_ctx *ctx, gt_buf buf, size_t bytes) {
  GT_ENTER(ctx);
  ProfScope ps(ctx, "clear");
  if (bytes) GT_HIP(ctx, hipMemsetAsync(P<void>(buf), 0, bytes, ctx->stream));
  return 0;
}

int gt_h2d(gt_ctx *ctx, gt_buf dst, const void *src, size_t bytes) {
  GT_ENTER(ctx);
  // pageable source: the runtime stages it before returning, so the caller may reuse src at once
  if (bytes) GT_HIP(ctx, hipMemcpyAsync(P<void>(dst), src, bytes, hipMemcpyHostToDevice, ctx->stream));
  return 0;
}

int gt_d2h(gt_ctx *ctx, void *dst, gt_buf src, size_t bytes) {
  GT_ENTER(ctx);
  if (bytes) GT_HIP(ctx, hipMemcpyAsync(dst, P<void>(src), bytes, hipMemcpyDeviceToHost, ctx->stream));
  GT_HIP(ctx, hipStreamSynchronize(ctx->stream));
  ctx->rms_static_pending = false;
  return gt_report_bad_id(ctx);
}

int gt_d2d(gt_ctx *ctx, gt_buf dst, gt_buf src, size_t bytes) {
  GT_ENTER(ctx);
  ProfScope ps(ctx, "copy");
  if (bytes) GT_HIP(ctx, hipMemcpyAsync(P<void>(dst), P<void>(src), bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return 0;
}

int gt_sync(gt_ctx *ctx) {
  GT_ENTER(ctx);
  GT_HIP(ctx, hipStreamSynchronize(ctx->stream));
  ctx->rms_static_pending = false;
  return gt_report_bad_id(ctx);
}

// Ordering between two contexts' streams without the host waiting: everything queued on `ctx` so far ...
int gt_stream_mark(gt_ctx *ctx) {
  GT_ENTER(ctx);
  GT_HIP(ctx, hipEventRecord(ctx->mark, ctx->stream));
  return 0;
}
// ... is finished before anything queued on `ctx` after this call starts, where `other` is the context that was marked.
int gt_stream_wait(gt_ctx *ctx, gt_ctx *other) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, other && other->device == ctx->device, "gt_stream_wait: the other context is null or on another device");
  if (other == ctx) return 0;
  GT_HIP(ctx, hipStreamWaitEvent(ctx->stream, other->mark, 0));
  return 0;
}

// One pair of events around whatever the caller queues between the two calls: the time of a run of launches as the
// device sees it, without a pair per launch.
int gt_timer_start(gt_ctx *ctx) {
  GT_ENTER(ctx);
  if (!ctx->timer_a) {
    GT_HIP(ctx, hipEventCreate(&ctx->timer_a));
    GT_HIP(ctx, hipEventCreate(&ctx->timer_b));
  }
  GT_HIP(ctx, hipEventRecord(ctx->timer_a, ctx->stream));
  return 0;
}
int gt_timer_stop(gt_ctx *ctx, double *ms) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, ms && ctx->timer_a, "gt_timer_stop: no result pointer, or gt_timer_start was not called");
  GT_HIP(ctx, hipEventRecord(ctx->timer_b, ctx->stream));
  GT_HIP(ctx, hipEventSynchronize(ctx->timer_b));
  float t = 0;
  GT_HIP(ctx, hipEventElapsedTime(&t, ctx->timer_a, ctx->timer_b));
  *ms = t;
  return 0;
}

int gt_resident_bytes(gt_ctx *ctx, uint64_t *bytes) {
  if (!ctx || !bytes) return 1;
  *bytes = ctx->live_bytes + ctx->ws_bytes;
  return 0;
}

int gt_set_option(gt_ctx *ctx, const char *key, int value) {
  if (!ctx || !key) return 1;
  if (!strcmp(key, "attn.generic")) ctx->opt_attn_generic = value;
  else if (!strcmp(key, "attn.keep_ds")) ctx->opt_attn_keep_ds = value;
  else if (!strcmp(key, "attn.ds_limit_mb")) ctx->opt_attn_ds_limit_mb = value < 0 ? 0 : value;
  else if (!strcmp(key, "attn.splits")) ctx->opt_attn_splits = value;
  else if (!strcmp(key, "attn.band_splits")) ctx->opt_attn_band_splits = value;
  else if (!strcmp(key, "prof.sample")) ctx->opt_prof_sample = value >= 1 ? value : 1;
  else if (!strcmp(key, "gemm.tile")) ctx->opt_gemm_tile = value;
  else if (!strcmp(key, "gemm.splitk")) ctx->opt_gemm_splitk = value;
  else if (!strcmp(key, "gemm.staged")) ctx->opt_gemm_staged = value;
  else if (!strcmp(key, "gemm.group")) ctx->opt_gemm_group = value;
  else if (!strcmp(key, "gemm.split_bf16")) ctx->opt_gemm_split = value;
  else if (!strcmp(key, "attn.split_bf16")) ctx->opt_attn_pieces = value;
  else if (!strcmp(key, "gemm.sum_min_tiles")) ctx->opt_gemm_sum_min_tiles = value;
  else GT_FAIL(ctx, "gt_set_option: unknown key '%s'", key);
  return 0;
}

int gt_prof_begin(gt_ctx *ctx, const char *prefix) {
  GT_ENTER(ctx);
  ctx->prof_prefix = prefix ? prefix : "";
  for (auto &e : ctx->prof) { hipEventDestroy(e.a); hipEventDestroy(e.b); }
  ctx->prof.clear();
  ctx->prof_seen.clear();
  ctx->prof_on = true;
  return 0;
}

int gt_prof_end(gt_ctx *ctx, gt_prof_rec *out, int cap, int *n) {
  GT_ENTER(ctx);
  ctx->prof_on = false;
  GT_HIP(ctx, hipStreamSynchronize(ctx->stream));
  struct Acc { double ms = 0, work = 0; int64_t n = 0; };
  std::map<std::string, Acc> sum;
  std::vector<std::string> order;
  for (auto &e : ctx->prof) {
    float ms = 0;
    GT_HIP(ctx, hipEventElapsedTime(&ms, e.a, e.b));
    if (!sum.count(e.label)) order.push_back(e.label);
    sum[e.label].ms += ms;
    sum[e.label].n += 1;
    sum[e.label].work += e.work;
    hipEventDestroy(e.a); hipEventDestroy(e.b);
  }
  ctx->prof.clear();
  int k = 0;
  for (auto &l : order) {
    if (k >= cap) break;
    snprintf(out[k].label, sizeof out[k].label, "%s", l.c_str());
    // count and work = every launch of the label; time = the timed launches' time scaled by all work / timed work
    // (by all launches / timed launches for a label that states no work)
    const auto &seen = ctx->prof_seen[l];
    const double scale = sum[l].work > 0 ? seen.work / sum[l].work : (double)seen.n / (double)sum[l].n;
    out[k].ms = sum[l].ms * scale;
    out[k].count = seen.n;
    out[k].work = seen.work;
    k++;
  }
  if (n) *n = k;
  return gt_report_bad_id(ctx);
}

}  // extern "C"

// Call with the stream drained. Reports an out-of-range id once and re-arms the note.
int gt_report_bad_id(gt_ctx *ctx) {
  volatile int *b = ctx->bad_host;
  const int what = b[0];
  if (!what) return 0;
  const int row = b[1], value = b[2], bound = b[3];
  b[0] = 0;
  const char *name = what == GT_BAD_EMBED_ID ? "embedding id" : what == GT_BAD_TARGET ? "cross-entropy target" : "teacher id";
  GT_FAIL(ctx, "%s %d at row %d is outside [%d, %d): that row was skipped", name, value, row, what == GT_BAD_TARGET ? -1 : 0, bound);
}

int gt_ws_reserve(gt_ctx *ctx, size_t bytes, void **out) {
  if (bytes > ctx->ws_bytes) {
    // queued kernels may still read the old block
    GT_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->ws) GT_HIP(ctx, hipFree(ctx->ws));
    ctx->ws = nullptr; ctx->ws_bytes = 0;
    size_t sz = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    GT_HIP(ctx, hipMalloc(&ctx->ws, sz));
    ctx->ws_bytes = sz;
  }
  *out = ctx->ws;
  return 0;
}
