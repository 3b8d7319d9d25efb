// src/backend/hip.ts: the MI355X (gfx950) device backend of gguf-trainer, bound over Deno.dlopen to libggufhip.so
// (C ABI: include/ggufhip.h). It takes the place of WebGPUBackend (src/backend/webgpu.ts:290-1888) behind the same
// interfaces: OpsBackend and RegionBackend (src/model/autograd.ts:103-164), the buffer surface the optimizers and the
// trainer use (webgpu.ts:393-862, 1432-1510), and the two device-resident optimizers (src/backend/adamw-gpu.ts:131-251,
// src/backend/muon-gpu.ts:351-470). Nothing in src/train, src/model, src/arch or src/gguf changes:
//
//   const gpu = await requireHip("training");            // instead of requireGPU(...)
//   const opt = new MuonHip(gpu, muon, aux, opts);       // instead of new MuonGpu(...)
//   await trainLMGpuResident(model, gpu, { optimizer: opt, ... });
//
// deno run --allow-ffi --allow-env ...   GGUFHIP_LIB=/path/to/libggufhip.so (default: ./libggufhip.so)
//
// What this host does, and what it leaves to a later pass. Every op is one or two gt_* calls recorded on the library's
// stream, in tape order. Gradient buffers are not cleared and then added to (webgpu.ts:21-26, 1397-1429): every backward
// entry point takes an `acc` flag, and this host knows the first writer of each gradient in an accumulation window, so an
// intermediate's gradient costs one write instead of clear + read + write, and gradient buffers of intermediates are only
// allocated when a backward reaches them. silu / gelu outputs are lazy, so mul(silu(g), u) runs the fused gated-activation
// kernels. Attention keeps its scores from the forward to the backward where memory allows (as the reference's small-T
// path keeps its probabilities, webgpu.ts:1176-1189). Host arrays of intermediates are allocated only when somebody reads
// them. The launch scheduling of the Python mirror (held-back and grouped GEMM launches, residual adds in the products'
// write-backs, micro-batches dealt to several streams) is not repeated here: each of those is an optional entry point of
// the same library (gt_gemm_sum, gt_gemm_group, gt_gemm_add, gt_rope_pair, gt_grad_fold, gt_stream_mark / gt_stream_wait).
import { setOpsBackend, Tensor } from "../model/autograd.ts";
import type { OpsBackend, RegionBackend } from "../model/autograd.ts";
import type { AdamOpts } from "../train/adam.ts";

// ---- the C ABI --------------------------------------------------------------------------------------------------------
// One row per entry point of include/ggufhip.h. Opaque handles passed by value (gt_ctx *,
// gt_adamw *, gt_muon *) are "pointer"; everything the library reads from or writes to host memory (out-parameters,
// id / pointer / size tables, NUL-terminated option keys and label prefixes, gt_prof_rec arrays) is a TypedArray
// ("buffer"); device addresses (gt_buf) are "u64" and travel as bigint.
const u64 = "u64", i32 = "i32", i64 = "i64", f32 = "f32", f64 = "f64", ptr = "pointer", buf = "buffer", usize = "usize";
const SYMBOLS = {
  gt_ctx_create:         { parameters: [i32, buf], result: i32 },
  gt_ctx_destroy:        { parameters: [ptr], result: i32 },
  gt_last_error:         { parameters: [ptr], result: ptr },
  gt_device_name:        { parameters: [ptr], result: ptr },
  gt_alloc:              { parameters: [ptr, usize, i32, buf], result: i32 },
  gt_free:               { parameters: [ptr, u64], result: i32 },
  gt_memset0:            { parameters: [ptr, u64, usize], result: i32 },
  gt_h2d:                { parameters: [ptr, u64, buf, usize], result: i32 },
  gt_d2h:                { parameters: [ptr, buf, u64, usize], result: i32 },
  gt_d2d:                { parameters: [ptr, u64, u64, usize], result: i32 },
  gt_sync:               { parameters: [ptr], result: i32 },
  gt_stream_mark:        { parameters: [ptr], result: i32 },
  gt_stream_wait:        { parameters: [ptr, ptr], result: i32 },
  gt_resident_bytes:     { parameters: [ptr, buf], result: i32 },
  gt_set_option:         { parameters: [ptr, buf, i32], result: i32 },
  gt_gemm:               { parameters: [ptr, i32, i32, i32, i32, i32, u64, u64, u64], result: i32 },
  gt_gemm_pair:          { parameters: [ptr, i32, i32, i32, i32, i32, u64, u64, i32, u64, u64, u64], result: i32 },
  gt_rank_down:          { parameters: [ptr, i32, i32, i32, u64, u64, i32, f32, u64], result: i32 },
  gt_rank_grad:          { parameters: [ptr, i32, i32, i32, u64, u64, i32, i32, u64], result: i32 },
  gt_rank_grad_slices:   { parameters: [ptr, i32, i32, i32, u64, buf], result: i32 },
  gt_rank_grad_parts:    { parameters: [ptr, i32, i32, i32, u64, u64, i32, u64], result: i32 },
  gt_rank_slices_group:  { parameters: [ptr, i32, buf, buf, buf, buf, buf], result: i32 },
  gt_gemm_add:           { parameters: [ptr, i32, i32, i32, i32, u64, u64, u64, u64], result: i32 },
  gt_gemm_sum:           { parameters: [ptr, i32, i32, i32, i32, i32, buf, buf, buf, u64], result: i32 },
  gt_gemm_group:         { parameters: [ptr, i32, i32, buf, buf, i32, buf, buf, buf, buf], result: i32 },
  gt_gemm_batched:       { parameters: [ptr, i32, i32, i32, i32, i32, u64, i64, u64, i64, u64, i64, i32], result: i32 },
  gt_add_fwd:            { parameters: [ptr, i64, u64, u64, u64], result: i32 },
  gt_mul_fwd:            { parameters: [ptr, i64, u64, u64, u64], result: i32 },
  gt_silu_fwd:           { parameters: [ptr, i64, u64, u64], result: i32 },
  gt_gelu_fwd:           { parameters: [ptr, i64, u64, u64], result: i32 },
  gt_scale_fwd:          { parameters: [ptr, i64, u64, f32, u64], result: i32 },
  gt_add_bwd:            { parameters: [ptr, i64, u64, u64, i32, u64, i32], result: i32 },
  gt_mul_bwd:            { parameters: [ptr, i64, u64, u64, u64, u64, i32, u64, i32], result: i32 },
  gt_silu_bwd:           { parameters: [ptr, i64, u64, u64, u64, i32], result: i32 },
  gt_gelu_bwd:           { parameters: [ptr, i64, u64, u64, u64, i32], result: i32 },
  gt_scale_bwd:          { parameters: [ptr, i64, u64, f32, u64, i32], result: i32 },
  gt_glu_fwd:            { parameters: [ptr, i32, i64, u64, u64, u64], result: i32 },
  gt_glu_bwd:            { parameters: [ptr, i32, i64, u64, u64, u64, u64, i32, u64, i32], result: i32 },
  gt_rmsnorm_fwd:        { parameters: [ptr, i32, i32, f32, u64, u64, u64, u64], result: i32 },
  gt_rmsnorm_bwd:        { parameters: [ptr, i32, i32, u64, u64, u64, u64, u64, i32, u64, i32], result: i32 },
  gt_rmsnorm_bwd_static: { parameters: [ptr, i32, i32, u64, u64, u64, u64, u64, i32, u64, i32], result: i32 },
  gt_rmsnorm_bwd_from:   { parameters: [ptr, i32, i32, u64, u64, u64, u64, u64, u64, u64, i32], result: i32 },
  gt_rmsnorm_parts_rows: { parameters: [ptr, i32, i32, buf], result: i32 },
  gt_rmsnorm_bwd_parts:  { parameters: [ptr, i32, i32, u64, u64, u64, u64, u64, u64, i32, u64], result: i32 },
  gt_colsum_group:       { parameters: [ptr, i32, buf, buf, buf, buf, buf], result: i32 },
  gt_embedding_fwd:      { parameters: [ptr, i32, i32, i32, u64, u64, u64], result: i32 },
  gt_embedding_bwd:      { parameters: [ptr, i32, i32, i32, u64, u64, u64, i32], result: i32 },
  gt_rope:               { parameters: [ptr, i32, i32, i32, i32, f64, i32, i32, u64, u64, i32], result: i32 },
  gt_rope_pair:          { parameters: [ptr, i32, i32, i32, f64, i32, i32, i32, u64, u64, i32, i32, u64, u64, i32], result: i32 },
  gt_attn_fwd:           { parameters: [ptr, i32, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64], result: i32 },
  gt_attn_bwd:           { parameters: [ptr, i32, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64, u64, u64, i32, u64, i32, u64, i32], result: i32 },
  gt_attn_scores_bytes:  { parameters: [ptr, i32, i32, i32, i32, i32, i32, buf], result: i32 },
  gt_attn_fwd_scores:    { parameters: [ptr, i32, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64, u64], result: i32 },
  gt_attn_bwd_scores:    { parameters: [ptr, i32, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64, u64, u64, u64, i32, u64, i32, u64, i32], result: i32 },
  gt_attn_bwd_scores_rope: { parameters: [ptr, i32, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64, u64, u64, f64, i32, i32, i32, u64, i32, u64, i32, u64, i32], result: i32 },
  gt_ce_fwd:             { parameters: [ptr, i32, i32, i32, u64, u64, u64, u64, u64], result: i32 },
  gt_ce_bwd:             { parameters: [ptr, i32, i32, i32, u64, u64, u64, u64, f32, u64, i32], result: i32 },
  gt_ce_chunk_stats:     { parameters: [ptr, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64], result: i32 },
  gt_ce_loss_from_stats: { parameters: [ptr, i32, i32, i32, u64, u64, u64, u64, u64, u64], result: i32 },
  gt_ce_chunk_grad:      { parameters: [ptr, i32, i32, i32, i32, i32, u64, u64, u64, u64, u64, f32], result: i32 },
  gt_soft_ce_fwd:        { parameters: [ptr, i32, i32, i32, u64, u64, u64, f32, u64, u64, u64], result: i32 },
  gt_soft_ce_bwd:        { parameters: [ptr, i32, i32, i32, u64, u64, u64, f32, u64, u64, f32, u64, i32], result: i32 },
  gt_grad_fold:          { parameters: [ptr, i32, buf, buf, i32, buf, buf], result: i32 },
  gt_adamw_create:       { parameters: [ptr, i32, buf, buf, buf, buf, buf, f64, f64, f64, f64, f64, buf], result: i32 },
  gt_adamw_step:         { parameters: [ptr, ptr, f64, f64, f64], result: i32 },
  gt_adamw_grad_norm:    { parameters: [ptr, ptr, buf], result: i32 },
  gt_adamw_destroy:      { parameters: [ptr, ptr], result: i32 },
  gt_muon_create:        { parameters: [ptr, i32, buf, buf, buf, buf, buf, f64, i32, i32, buf], result: i32 },
  gt_muon_step:          { parameters: [ptr, ptr, f64], result: i32 },
  gt_muon_destroy:       { parameters: [ptr, ptr], result: i32 },
  gt_newton_schulz:      { parameters: [ptr, i32, i32, i32, u64, u64], result: i32 },
  gt_prof_begin:         { parameters: [ptr, buf], result: i32 },
  gt_prof_end:           { parameters: [ptr, buf, i32, buf], result: i32 },
  gt_timer_start:        { parameters: [ptr], result: i32 },
  gt_timer_stop:         { parameters: [ptr, buf], result: i32 },
} as const;

type Lib = Deno.DynamicLibrary<typeof SYMBOLS>;
type Sym = Lib["symbols"];
/** A device address (gt_buf). */
export type DevBuf = bigint;

const NT = 0, NN = 1, TN = 2;
const ALIGN = 256;
const enc = new TextEncoder();
const cstr = (s: string) => enc.encode(s + "\0");
const prod = (shape: number[]) => shape.reduce((a, b) => a * b, 1);
const EMPTY = new Float32Array(0);

export interface KernelTime {
  label: string;
  ms: number;
  count: number;
  /** algorithmic work the calls stated for themselves: FLOP for the contractions, bytes for the streaming kernels */
  work: number;
}

interface Entry {
  data: DevBuf;
  grad: DevBuf;
  bytes: number;
  external: boolean;
  /** some kernel has written this gradient in the current accumulation window: the next writer adds */
  gradInit: boolean;
  /** (pre-activation, 0 = silu | 1 = gelu) while a silu / gelu output has not been computed */
  lazyAct: { x: Tensor; act: number } | null;
  consumers: number;
  fusedUses: number;
  keepGrad: boolean;
  /** a saved buffer that lives and dies with this output (attention scores) */
  extra: { buf: DevBuf; bytes: number } | null;
  /** an intermediate below a trainable tensor: a backward through it may be asked for */
  needsGrad: boolean;
}

/** An op output whose host arrays are allocated only when somebody reads them (the reference's makeOut allocates two
 * zero-filled Float32Arrays per intermediate, webgpu.ts:1575-1593; at [2048, 49152] logits that is 0.8 GB of host
 * memory per micro-batch that nothing ever looks at). The constructor still runs, so `seq` keeps its order. */
function lazyTensor(shape: number[], prev: Tensor[]): Tensor {
  const t = new Tensor(EMPTY, [0]);
  t.shape = shape;
  t._prev = prev;
  const n = prod(shape);
  for (const key of ["data", "grad"] as const) {
    let arr: Float32Array | null = null;
    Object.defineProperty(t, key, {
      configurable: true,
      enumerable: true,
      get: () => (arr ??= new Float32Array(n)),
      set: (v: Float32Array) => {
        arr = v;
      },
    });
  }
  return t;
}

export class HipBackend implements OpsBackend, RegionBackend {
  readonly adapterName: string;
  /** kept for interface parity (webgpu.ts:305); one kernel family serves every T here */
  attnFlashMinT = 2048;
  lastSyncReadbackBytes = 0;
  /** stays at the number of trainable parameters: only a never-written accumulator is ever cleared */
  gradClearsIssued = 0;
  fuseGlu = true;
  attnKeepScores = true;
  attnScoresMaxBytes = 4 * 2 ** 30;
  attnScoresBudgetBytes = 96 * 2 ** 30;
  /** set by a caller around a checkpointed block's first forward, whose interior is never differentiated */
  forwardOnlyRegion = false;

  private sym: Sym;
  private lib: Lib;
  private ctx: Deno.PointerValue;
  private pool = new Map<number, DevBuf[]>();
  private poolBytes = 0;
  private stateBytes = 0;
  private entries = new WeakMap<Tensor, Entry>();
  private touched: Tensor[] = [];
  private touchedSet = new Set<Tensor>();
  private transients: { t: Tensor; e: Entry }[] = [];
  private scratch: { buf: DevBuf; bytes: number }[] = [];
  private regionsOpened = 0;
  private scoresTaken = 0;
  private destroyed = false;

  constructor(libPath: string, device = 0) {
    this.lib = Deno.dlopen(libPath, SYMBOLS);
    this.sym = this.lib.symbols;
    const out = new BigUint64Array(1);
    if (this.sym.gt_ctx_create(device, out) !== 0) {
      const msg = new Deno.UnsafePointerView(this.sym.gt_last_error(null)!).getCString();
      this.lib.close();
      throw new Error("gt_ctx_create: " + msg);
    }
    this.ctx = Deno.UnsafePointer.create(out[0]);
    this.adapterName = new Deno.UnsafePointerView(this.sym.gt_device_name(this.ctx)!).getCString();
  }

  /** The library context, for the optimizers and for raw calls in tests. */
  get context(): Deno.PointerValue {
    return this.ctx;
  }
  get symbols(): Sym {
    return this.sym;
  }

  check(rc: number, what: string) {
    if (rc !== 0) {
      const p = this.sym.gt_last_error(this.ctx);
      throw new Error(`${what}: ${p ? new Deno.UnsafePointerView(p).getCString() : "unknown error"}`);
    }
  }

  // ---- install (webgpu.ts:393-399) --------------------------------------------------------------------------------
  install() {
    setOpsBackend(this);
  }
  uninstall() {
    setOpsBackend(null);
  }

  // ---- raw memory ----------------------------------------------------------------------------------------------------
  private sizeClass(bytes: number): number {
    return Math.max(ALIGN, Math.ceil(bytes / ALIGN) * ALIGN);
  }
  private acquire(bytes: number): DevBuf {
    const size = this.sizeClass(bytes);
    const free = this.pool.get(size);
    if (free && free.length) return free.pop()!;
    const out = new BigUint64Array(1);
    if (this.sym.gt_alloc(this.ctx, BigInt(size), 0, out) !== 0) {
      // device memory may be full of free buffers of other size classes: give them back and ask once more
      if (!this.trimPool()) this.check(1, "gt_alloc");
      this.check(this.sym.gt_alloc(this.ctx, BigInt(size), 0, out), "gt_alloc");
    }
    this.poolBytes += size;
    return out[0];
  }
  private recycle(b: DevBuf, bytes: number) {
    const size = this.sizeClass(bytes);
    let free = this.pool.get(size);
    if (!free) this.pool.set(size, free = []);
    free.push(b);
  }
  /** Return every free pool buffer to the device. Gives the bytes freed. */
  trimPool(): number {
    this.check(this.sym.gt_sync(this.ctx), "gt_sync"); // queued kernels may still use a recycled buffer
    let freed = 0;
    for (const [size, free] of this.pool) {
      for (const b of free) {
        this.check(this.sym.gt_free(this.ctx, b), "gt_free");
        freed += size;
      }
      free.length = 0;
    }
    this.poolBytes -= freed;
    return freed;
  }
  private scratchBuf(bytes: number): DevBuf {
    const b = this.acquire(bytes);
    this.scratch.push({ buf: b, bytes });
    return b;
  }
  private upload(arr: Int32Array | Float32Array): DevBuf {
    const b = this.scratchBuf(arr.byteLength);
    this.check(this.sym.gt_h2d(this.ctx, b, arr, BigInt(arr.byteLength)), "gt_h2d");
    return b;
  }

  // ---- entries (webgpu.ts:1539-1593) ------------------------------------------------------------------------------
  private newEntry(bytes: number, external: boolean): Entry {
    return {
      data: 0n, grad: 0n, bytes, external, gradInit: false, lazyAct: null, consumers: 0, fusedUses: 0,
      keepGrad: false, extra: null, needsGrad: false,
    };
  }
  /** Device buffers of an existing tensor; a tensor never seen before is external (a parameter or a test input): it
   * gets a persistent data buffer, uploaded once. A frozen external never gets a gradient buffer. */
  private entryFor(t: Tensor): Entry {
    let e = this.entries.get(t);
    if (!e) {
      if (t._prev.length) {
        throw new Error("backward over a graph built before a sync(): that sync recycled the graph's buffers");
      }
      e = this.newEntry(prod(t.shape) * 4, true);
      e.data = this.acquire(e.bytes);
      this.check(this.sym.gt_h2d(this.ctx, e.data, t.data, BigInt(e.bytes)), "gt_h2d");
      this.entries.set(t, e);
    }
    if (e.external && t.requiresGrad && !this.touchedSet.has(t)) {
      this.touchedSet.add(t);
      this.touched.push(t);
    }
    return e;
  }
  private makeOut(shape: number[], prev: Tensor[], alloc = true): { t: Tensor; e: Entry } {
    const t = lazyTensor(shape, prev);
    const e = this.newEntry(prod(shape) * 4, false);
    if (alloc) e.data = this.acquire(e.bytes);
    for (const p of prev) {
      const pe = this.entries.get(p);
      if (p.requiresGrad || (pe && pe.needsGrad)) {
        e.needsGrad = true;
        break;
      }
    }
    this.entries.set(t, e);
    this.transients.push({ t, e });
    return { t, e };
  }
  /** Device address of t's values, as an op input. */
  private dataOf(t: Tensor): DevBuf {
    const e = this.entryFor(t);
    e.consumers += 1;
    if (e.lazyAct) this.materialise(t, e);
    return e.data;
  }
  private materialise(t: Tensor, e: Entry) {
    const { x, act } = e.lazyAct!;
    e.lazyAct = null;
    e.data = this.acquire(e.bytes);
    const xe = this.entryFor(x);
    const fn = act === 0 ? this.sym.gt_silu_fwd : this.sym.gt_gelu_fwd;
    this.check(fn(this.ctx, BigInt(prod(t.shape)), xe.data, e.data), "act.fwd");
  }
  /** [gradient buffer, acc] for a backward kernel about to contribute to t's gradient; [0n, 0] when t takes none. */
  private gradDst(t: Tensor): [DevBuf, number] {
    const e = this.entryFor(t);
    if (e.external && !t.requiresGrad) return [0n, 0];
    if (e.grad === 0n) e.grad = this.acquire(e.bytes);
    const acc = e.gradInit ? 1 : 0;
    e.gradInit = true;
    return [e.grad, acc];
  }
  /** Gradient buffer of an op output inside its backward closure. */
  private gradOf(t: Tensor): DevBuf {
    const e = this.entries.get(t);
    if (!e) {
      throw new Error(
        "backward over a graph built before a sync(): that sync recycled the graph's gradient buffers, " +
          "so this backward would read pool garbage",
      );
    }
    if (e.grad === 0n || !e.gradInit) {
      // nothing downstream wrote it (an output the loss does not depend on): its gradient is zero
      if (e.grad === 0n) e.grad = this.acquire(e.bytes);
      this.check(this.sym.gt_memset0(this.ctx, e.grad, BigInt(e.bytes)), "gt_memset0");
      this.gradClearsIssued++;
      e.gradInit = true;
    }
    return e.grad;
  }

  // ---- public buffer surface (webgpu.ts:406, 1432-1510) -------------------------------------------------------------
  uploadParams(tensors: Tensor[]) {
    for (const t of tensors) {
      const e = this.entryFor(t);
      this.check(this.sym.gt_h2d(this.ctx, e.data, t.data, BigInt(e.bytes)), "gt_h2d");
    }
  }
  buffersFor(t: Tensor): { data: DevBuf; grad: DevBuf } {
    const e = this.entryFor(t);
    if (t.requiresGrad && e.grad === 0n) {
      e.grad = this.acquire(e.bytes);
      this.check(this.sym.gt_memset0(this.ctx, e.grad, BigInt(e.bytes)), "gt_memset0");
      this.gradClearsIssued++;
    }
    return { data: e.data, grad: e.grad };
  }
  keepGradOnDevice(t: Tensor) {
    this.entryFor(t).keepGrad = true;
  }
  /** The optimizer has read these accumulators: the next backward write stores instead of adding (the reference's
   * deferred per-step clear, muon-gpu.ts:8-16). */
  gradsConsumed(tensors: Tensor[]) {
    for (const t of tensors) {
      const e = this.entries.get(t);
      if (e) e.gradInit = false;
    }
  }
  /** An accumulator no kernel wrote since it was last consumed holds zero, as a cleared one would. */
  ensureGradsDefined(tensors: Tensor[]) {
    for (const t of tensors) {
      const e = this.entryFor(t);
      if (e.grad === 0n) e.grad = this.acquire(e.bytes);
      if (!e.gradInit) {
        this.check(this.sym.gt_memset0(this.ctx, e.grad, BigInt(e.bytes)), "gt_memset0");
        this.gradClearsIssued++;
        e.gradInit = true;
      }
    }
  }
  seedGradFromHost(t: Tensor) {
    const e = this.entries.get(t);
    if (!e) throw new Error("seedGradFromHost: tensor has no device buffers");
    if (e.grad === 0n) e.grad = this.acquire(e.bytes);
    this.check(this.sym.gt_h2d(this.ctx, e.grad, t.grad, BigInt(e.bytes)), "gt_h2d");
    e.gradInit = true;
  }
  /** A zero-initialised buffer outside the pool (optimizer state). */
  createStateBuffer(bytes: number): DevBuf {
    const out = new BigUint64Array(1);
    const size = Math.max(4, bytes);
    this.check(this.sym.gt_alloc(this.ctx, BigInt(size), 1, out), "gt_alloc");
    this.stateBytes += size;
    return out[0];
  }
  freeStateBuffer(b: DevBuf) {
    this.check(this.sym.gt_free(this.ctx, b), "gt_free");
  }
  writeStateBuffer(b: DevBuf, values: Float32Array) {
    this.check(this.sym.gt_h2d(this.ctx, b, values, BigInt(values.byteLength)), "gt_h2d");
  }
  // deno-lint-ignore require-await
  async readStateBuffer(b: DevBuf, elems: number): Promise<Float32Array> {
    const out = new Float32Array(elems);
    this.check(this.sym.gt_d2h(this.ctx, out, b, BigInt(out.byteLength)), "gt_d2h");
    return out;
  }
  setOption(key: string, value: number) {
    this.check(this.sym.gt_set_option(this.ctx, cstr(key), value), "gt_set_option");
  }
  residentBytes(): { pool: number; state: number; total: number } {
    const v = new BigUint64Array(1);
    this.sym.gt_resident_bytes(this.ctx, v);
    return { pool: this.poolBytes, state: this.stateBytes, total: Number(v[0]) };
  }
  regionCount(): number {
    return this.regionsOpened;
  }

  // ---- sync / reclaim (webgpu.ts:419-636) --------------------------------------------------------------------------
  private releaseTransients(keep: Tensor[] = []) {
    const keepSet = new Set(keep);
    const kept: { t: Tensor; e: Entry }[] = [];
    for (const it of this.transients) {
      if (keepSet.has(it.t)) {
        kept.push(it);
        continue;
      }
      this.releaseEntry(it.t, it.e);
    }
    this.transients = kept;
    for (const s of this.scratch) this.recycle(s.buf, s.bytes);
    this.scratch = [];
  }
  private releaseEntry(t: Tensor, e: Entry) {
    if (e.data !== 0n) this.recycle(e.data, e.bytes);
    if (e.grad !== 0n) this.recycle(e.grad, e.bytes);
    if (e.extra) {
      this.recycle(e.extra.buf, e.extra.bytes);
      this.scoresTaken -= e.extra.bytes;
      e.extra = null;
    }
    e.data = e.grad = 0n;
    this.entries.delete(t);
  }
  /** Wait for the stream; read back `reads` (values) and the accumulated gradients of every trainable external tensor
   * touched since the last sync that is not kept on the device; recycle all intermediates. The graph is unusable for
   * backward afterwards. */
  // deno-lint-ignore require-await
  async sync(reads: Tensor[] = []): Promise<void> {
    let nbytes = 0;
    for (const t of reads) {
      const e = this.entries.get(t);
      if (!e) throw new Error("sync: tensor has no device buffers");
      if (e.lazyAct) this.materialise(t, e);
      this.check(this.sym.gt_d2h(this.ctx, t.data, e.data, BigInt(e.bytes)), "gt_d2h");
      nbytes += e.bytes;
    }
    for (const t of this.touched) {
      const e = this.entries.get(t);
      if (!e || e.keepGrad) continue;
      if (t.requiresGrad) {
        if (e.grad !== 0n && e.gradInit) {
          this.check(this.sym.gt_d2h(this.ctx, t.grad, e.grad, BigInt(e.bytes)), "gt_d2h");
          nbytes += e.bytes;
        } else {
          t.grad.fill(0);
        }
      }
      // the window ends here: the next one starts this accumulator from zero (also for a parameter frozen after its
      // backward and thawed later, gpu-parity.ts:1980-2028)
      e.gradInit = false;
    }
    this.touched = [];
    this.touchedSet.clear();
    this.check(this.sym.gt_sync(this.ctx), "gt_sync");
    this.lastSyncReadbackBytes = nbytes;
    this.releaseTransients();
    this.scoresTaken = 0;
  }
  /** Free a finished micro-batch's intermediates mid-step; parameter gradients keep accumulating. */
  // deno-lint-ignore require-await
  async reclaimStepTransients(keep: Tensor[] = []): Promise<void> {
    this.check(this.sym.gt_sync(this.ctx), "gt_sync");
    this.releaseTransients(keep);
  }
  destroy() {
    if (!this.destroyed) {
      this.destroyed = true;
      this.sym.gt_ctx_destroy(this.ctx); // frees every buffer and every optimizer of the context
      this.lib.close();
    }
  }
  get isDestroyed(): boolean {
    return this.destroyed;
  }

  // ---- profiling (webgpu.ts:830-880) ---------------------------------------------------------------------------------
  startProfile(prefix = "") {
    this.check(this.sym.gt_prof_begin(this.ctx, cstr(prefix)), "gt_prof_begin");
  }
  stopProfile(): { kernels: KernelTime[]; overflow: boolean } {
    // gt_prof_rec { char label[32]; double ms; int64_t count; double work; } = 56 bytes
    const cap = 128, rec = 56;
    const raw = new Uint8Array(cap * rec);
    const n = new Int32Array(1);
    this.check(this.sym.gt_prof_end(this.ctx, raw, cap, n), "gt_prof_end");
    const view = new DataView(raw.buffer);
    const dec = new TextDecoder();
    const kernels: KernelTime[] = [];
    for (let i = 0; i < n[0]; i++) {
      const o = i * rec;
      let len = 0;
      while (len < 32 && raw[o + len] !== 0) len++;
      kernels.push({
        label: dec.decode(raw.subarray(o, o + len)),
        ms: view.getFloat64(o + 32, true),
        count: Number(view.getBigInt64(o + 40, true)),
        work: view.getFloat64(o + 48, true),
      });
    }
    return { kernels, overflow: n[0] === cap };
  }

  // ---- RegionBackend (webgpu.ts:639-761) ---------------------------------------------------------------------------
  beginRegion(): number {
    this.regionsOpened++;
    return this.transients.length;
  }
  endRegion(mark: number, keep: Tensor[]): void {
    const keepSet = new Set(keep);
    const tail = this.transients.splice(mark);
    for (const it of tail) {
      if (keepSet.has(it.t)) this.transients.push(it);
      else this.releaseEntry(it.t, it.e);
    }
  }
  seedGradFrom(dst: Tensor, src: Tensor): void {
    const n = prod(dst.shape);
    if (n !== prod(src.shape)) throw new Error(`seedGradFrom: size mismatch ${n} vs ${prod(src.shape)}`);
    const g = this.gradOf(src);
    const [d] = this.gradDst(dst);
    this.check(this.sym.gt_d2d(this.ctx, d, g, BigInt(n * 4)), "gt_d2d");
  }

  // ---- ops (webgpu.ts:884-1378) ----------------------------------------------------------------------------------------
  linear(x: Tensor, w: Tensor): Tensor {
    const [T, inDim] = x.shape, outDim = w.shape[0];
    const xd = this.dataOf(x), wd = this.dataOf(w);
    const { t: out, e } = this.makeOut([T, outDim], [x, w]);
    this.check(this.sym.gt_gemm(this.ctx, NT, 0, T, outDim, inDim, xd, wd, e.data), "linear");
    const wantsDW = w.requiresGrad;
    out._backward = () => {
      const g = this.gradOf(out);
      const [dx, acc] = this.gradDst(x);
      if (dx !== 0n) this.check(this.sym.gt_gemm(this.ctx, NN, acc, T, inDim, outDim, g, wd, dx), "linear.dx");
      if (wantsDW) {
        const [dw, accw] = this.gradDst(w);
        if (dw !== 0n) this.check(this.sym.gt_gemm(this.ctx, TN, accw, outDim, inDim, T, g, xd, dw), "linear.dw");
      }
    };
    return out;
  }

  add(a: Tensor, b: Tensor): Tensor {
    const n = prod(a.shape);
    const ad = this.dataOf(a), bd = this.dataOf(b);
    const { t: out, e } = this.makeOut(a.shape, [a, b]);
    this.check(this.sym.gt_add_fwd(this.ctx, BigInt(n), ad, bd, e.data), "add");
    out._backward = () => {
      const g = this.gradOf(out);
      if (a === b) {
        const [da, acc] = this.gradDst(a);
        if (da !== 0n) this.check(this.sym.gt_add_bwd(this.ctx, BigInt(n), g, da, acc, da, acc), "add.bwd");
        return;
      }
      const [da, acca] = this.gradDst(a);
      const [db, accb] = this.gradDst(b);
      this.check(this.sym.gt_add_bwd(this.ctx, BigInt(n), g, da, acca, db, accb), "add.bwd");
    };
    return out;
  }

  mul(a: Tensor, b: Tensor): Tensor {
    const n = prod(a.shape);
    const ea = this.entryFor(a), eb = this.entryFor(b);
    if (this.fuseGlu && a !== b) {
      // gate * up with a lazy activation on one side: the fused kernels work on the pre-activation
      const lazy = ea.lazyAct ? a : eb.lazyAct ? b : null;
      const other = lazy === a ? b : a;
      if (lazy && !this.entries.get(other)!.lazyAct) {
        const le = this.entries.get(lazy)!;
        const { x: gate, act } = le.lazyAct!;
        le.consumers += 1;
        le.fusedUses += 1;
        const gd = this.dataOf(gate), ud = this.dataOf(other);
        const { t: out, e } = this.makeOut(a.shape, [a, b]);
        this.check(this.sym.gt_glu_fwd(this.ctx, act, BigInt(n), gd, ud, e.data), "glu");
        out._backward = () => {
          const g = this.gradOf(out);
          const [dg, accg] = this.gradDst(gate);
          const [du, accu] = this.gradDst(other);
          this.check(this.sym.gt_glu_bwd(this.ctx, act, BigInt(n), g, gd, ud, dg, accg, du, accu), "glu.bwd");
        };
        return out;
      }
    }
    const ad = this.dataOf(a), bd = this.dataOf(b);
    const { t: out, e } = this.makeOut(a.shape, [a, b]);
    this.check(this.sym.gt_mul_fwd(this.ctx, BigInt(n), ad, bd, e.data), "mul");
    out._backward = () => {
      const g = this.gradOf(out);
      if (a === b) {
        const [da, acc] = this.gradDst(a);
        if (da !== 0n) this.check(this.sym.gt_mul_bwd(this.ctx, BigInt(n), g, ad, ad, da, acc, da, acc), "mul.bwd");
        return;
      }
      const [da, acca] = this.gradDst(a);
      const [db, accb] = this.gradDst(b);
      this.check(this.sym.gt_mul_bwd(this.ctx, BigInt(n), g, ad, bd, da, acca, db, accb), "mul.bwd");
    };
    return out;
  }

  private activation(x: Tensor, act: number): Tensor {
    const n = prod(x.shape);
    const xe = this.entryFor(x);
    xe.consumers += 1;
    if (xe.lazyAct) this.materialise(x, xe);
    const xd = xe.data;
    const { t: out, e } = this.makeOut(x.shape, [x], !this.fuseGlu);
    if (this.fuseGlu) {
      e.lazyAct = { x, act };
    } else {
      const fn = act === 0 ? this.sym.gt_silu_fwd : this.sym.gt_gelu_fwd;
      this.check(fn(this.ctx, BigInt(n), xd, e.data), "act");
    }
    out._backward = () => {
      const oe = this.entries.get(out);
      if (!oe) throw new Error("backward over a graph built before a sync()");
      if (oe.fusedUses && oe.fusedUses === oe.consumers) return; // every use was a fused gate*up, which wrote x's gradient
      if (oe.grad === 0n && oe.fusedUses) return; // its other consumers contributed nothing
      const g = this.gradOf(out);
      const [dx, acc] = this.gradDst(x);
      if (dx === 0n) return;
      const fn = act === 0 ? this.sym.gt_silu_bwd : this.sym.gt_gelu_bwd;
      this.check(fn(this.ctx, BigInt(n), g, xd, dx, acc), "act.bwd");
    };
    return out;
  }
  silu(x: Tensor): Tensor {
    return this.activation(x, 0);
  }
  gelu(x: Tensor): Tensor {
    return this.activation(x, 1);
  }

  scale(x: Tensor, c: number): Tensor {
    const n = prod(x.shape);
    const xd = this.dataOf(x);
    const { t: out, e } = this.makeOut(x.shape, [x]);
    this.check(this.sym.gt_scale_fwd(this.ctx, BigInt(n), xd, c, e.data), "scale");
    out._backward = () => {
      const g = this.gradOf(out);
      const [dx, acc] = this.gradDst(x);
      if (dx !== 0n) this.check(this.sym.gt_scale_bwd(this.ctx, BigInt(n), g, c, dx, acc), "scale.bwd");
    };
    return out;
  }

  private rmsRows(x: Tensor, weight: Tensor, rows: number, d: number, eps: number, shape: number[]): Tensor {
    const xd = this.dataOf(x), wd = this.dataOf(weight);
    const { t: out, e } = this.makeOut(shape, [x, weight]);
    const rinv = this.scratchBuf(rows * 4);
    this.check(this.sym.gt_rmsnorm_fwd(this.ctx, rows, d, eps, xd, wd, e.data, rinv), "rmsnorm");
    const wantsDW = weight.requiresGrad;
    out._backward = () => {
      const g = this.gradOf(out);
      const [dx, acc] = this.gradDst(x);
      const [dw, accw] = wantsDW ? this.gradDst(weight) : [0n, 0] as [DevBuf, number];
      if (dx === 0n) {
        // a frozen input (a test's leaf): the kernel still needs a destination for dx
        const tmp = this.scratchBuf(rows * d * 4);
        this.check(this.sym.gt_rmsnorm_bwd(this.ctx, rows, d, xd, wd, g, rinv, tmp, 0, dw, accw), "rmsnorm.bwd");
        return;
      }
      this.check(this.sym.gt_rmsnorm_bwd(this.ctx, rows, d, xd, wd, g, rinv, dx, acc, dw, accw), "rmsnorm.bwd");
    };
    return out;
  }
  rmsNorm(x: Tensor, weight: Tensor, eps: number): Tensor {
    const [T, d] = x.shape;
    return this.rmsRows(x, weight, T, d, eps, [T, d]);
  }
  rmsNormHeads(x: Tensor, weight: Tensor, T: number, H: number, hd: number, eps: number): Tensor {
    return this.rmsRows(x, weight, T * H, hd, eps, [T, H * hd]);
  }

  embedding(weight: Tensor, ids: number[]): Tensor {
    const [V, d] = weight.shape;
    const T = ids.length;
    const wd = this.dataOf(weight);
    const idb = this.upload(Int32Array.from(ids));
    const { t: out, e } = this.makeOut([T, d], [weight]);
    this.check(this.sym.gt_embedding_fwd(this.ctx, T, d, V, idb, wd, e.data), "embedding");
    const wantsDW = weight.requiresGrad;
    out._backward = () => {
      if (!wantsDW) return;
      const g = this.gradOf(out);
      const [dw, acc] = this.gradDst(weight);
      this.check(this.sym.gt_embedding_bwd(this.ctx, T, d, V, idb, g, dw, acc), "embedding.bwd");
    };
    return out;
  }

  rope(x: Tensor, T: number, H: number, hd: number, base: number, posOffset: number): Tensor {
    const rows = x.shape[0];
    const xd = this.dataOf(x);
    const { t: out, e } = this.makeOut([rows, H * hd], [x]);
    this.check(this.sym.gt_rope(this.ctx, rows, T, H, hd, base, posOffset, 0, xd, e.data, 0), "rope");
    out._backward = () => {
      const g = this.gradOf(out);
      const [dx, acc] = this.gradDst(x);
      if (dx !== 0n) this.check(this.sym.gt_rope(this.ctx, rows, T, H, hd, base, posOffset, 1, g, dx, acc), "rope.bwd");
    };
    return out;
  }

  attention(q: Tensor, k: Tensor, v: Tensor, T: number, Hq: number, Hkv: number, hd: number, window: number): Tensor {
    const rows = q.shape[0];
    if (rows % T) throw new Error(`attention: ${rows} rows are not a whole number of sequences of ${T}`);
    const B = rows / T;
    const qd = this.dataOf(q), kd = this.dataOf(k), vd = this.dataOf(v);
    const { t: out, e } = this.makeOut([rows, Hq * hd], [q, k, v]);
    const lse = this.scratchBuf(B * Hq * T * 4);
    let scores = 0n;
    if (this.attnKeepScores && !this.forwardOnlyRegion && e.needsGrad) {
      const need = new BigUint64Array(1);
      this.check(this.sym.gt_attn_scores_bytes(this.ctx, B, T, Hq, Hkv, hd, window, need), "attention");
      const nb = Number(need[0]);
      if (nb > 0 && nb <= this.attnScoresMaxBytes && this.scoresTaken + nb <= this.attnScoresBudgetBytes) {
        scores = this.acquire(nb);
        e.extra = { buf: scores, bytes: nb };
        this.scoresTaken += nb;
      }
    }
    if (scores !== 0n) {
      this.check(
        this.sym.gt_attn_fwd_scores(this.ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, e.data, lse, scores),
        "attention",
      );
    } else {
      this.check(this.sym.gt_attn_fwd(this.ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, e.data, lse), "attention");
    }
    const od = e.data;
    out._backward = () => {
      const g = this.gradOf(out);
      // frozen q / k / v (a test's leaves) still need destinations: the kernels write all three
      const dst = (t: Tensor): [DevBuf, number] => {
        const [d, a] = this.gradDst(t);
        return d !== 0n ? [d, a] : [this.scratchBuf(prod(t.shape) * 4), 0];
      };
      const [dq, aq] = dst(q), [dk, ak] = dst(k), [dv, av] = dst(v);
      if (scores !== 0n) {
        this.check(
          this.sym.gt_attn_bwd_scores(this.ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, od, g, lse, scores, dq, aq, dk, ak, dv, av),
          "attention.bwd",
        );
      } else {
        this.check(
          this.sym.gt_attn_bwd(this.ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, od, g, lse, dq, aq, dk, ak, dv, av),
          "attention.bwd",
        );
      }
    };
    return out;
  }

  crossEntropy(logits: Tensor, targets: number[], kept: number): Tensor {
    const [rows, V] = logits.shape;
    const zd = this.dataOf(logits);
    const tg = this.upload(Int32Array.from(targets));
    const inv = this.upload(Float32Array.of(1 / Math.max(kept, 1)));
    const lse = this.scratchBuf(rows * 4);
    const { t: loss, e } = this.makeOut([1], [logits]);
    this.check(this.sym.gt_ce_fwd(this.ctx, rows, V, rows, zd, tg, inv, e.data, lse), "crossEntropy");
    loss._backward = () => {
      if (!this.entries.get(loss)) throw new Error("backward over a graph built before a sync()");
      const seed = loss.grad[0];
      const [dz, acc] = this.gradDst(logits);
      if (dz !== 0n) this.check(this.sym.gt_ce_bwd(this.ctx, rows, V, rows, zd, tg, inv, lse, seed, dz, acc), "crossEntropy.bwd");
    };
    return loss;
  }

  fusedCrossEntropy(hidden: Tensor, w: Tensor, targets: number[], chunk: number, kept: number): Tensor {
    const [rows, H] = hidden.shape;
    const V = w.shape[0];
    const hd = this.dataOf(hidden), wd = this.dataOf(w);
    const tg = this.upload(Int32Array.from(targets));
    const inv = this.upload(Float32Array.of(1 / Math.max(kept, 1)));
    const rmax = this.scratchBuf(rows * 4), rsum = this.scratchBuf(rows * 4), tl = this.scratchBuf(rows * 4);
    const width = Math.min(chunk, V);
    const cb = this.scratchBuf(rows * width * 4);
    const spans: [number, number][] = [];
    for (let v0 = 0; v0 < V; v0 += chunk) spans.push([v0, Math.min(v0 + chunk, V) - v0]);
    const wAt = (v0: number) => wd + BigInt(v0) * BigInt(H * 4);
    spans.forEach(([v0, vc], i) => {
      this.check(this.sym.gt_gemm(this.ctx, NT, 0, rows, vc, H, hd, wAt(v0), cb), "fusedCE.logits");
      this.check(this.sym.gt_ce_chunk_stats(this.ctx, rows, V, vc, v0, i === 0 ? 1 : 0, cb, tg, rmax, rsum, tl), "fusedCE.stats");
    });
    const { t: loss, e } = this.makeOut([1], [hidden, w]);
    this.check(this.sym.gt_ce_loss_from_stats(this.ctx, rows, V, rows, tg, inv, rmax, rsum, tl, e.data), "fusedCE.loss");
    const wantsDW = w.requiresGrad;
    loss._backward = () => {
      if (!this.entries.get(loss)) throw new Error("backward over a graph built before a sync()");
      const seed = loss.grad[0];
      let [dh, acch] = this.gradDst(hidden);
      const [dw, accw] = wantsDW ? this.gradDst(w) : [0n, 0] as [DevBuf, number];
      for (const [v0, vc] of spans) {
        this.check(this.sym.gt_gemm(this.ctx, NT, 0, rows, vc, H, hd, wAt(v0), cb), "fusedCE.logits");
        this.check(this.sym.gt_ce_chunk_grad(this.ctx, rows, V, vc, v0, rows, cb, tg, inv, rmax, rsum, seed), "fusedCE.grad");
        if (dh !== 0n) {
          this.check(this.sym.gt_gemm(this.ctx, NN, acch, rows, H, vc, cb, wAt(v0), dh), "fusedCE.dh");
          acch = 1;
        }
        // rows [v0, v0+vc) of dW are written by this span only
        if (dw !== 0n) this.check(this.sym.gt_gemm(this.ctx, TN, accw, vc, H, rows, cb, hd, dw + BigInt(v0) * BigInt(H * 4)), "fusedCE.dw");
      }
    };
    return loss;
  }

  softCrossEntropy(logits: Tensor, teacherIds: number[], teacherProbs: number[], k: number, kept: number): Tensor {
    const [rows, V] = logits.shape;
    const inv = 1 / Math.max(kept, 1);
    const zd = this.dataOf(logits);
    const ti = this.upload(Int32Array.from(teacherIds));
    const tp = this.upload(Float32Array.from(teacherProbs));
    const lse = this.scratchBuf(rows * 4), mass = this.scratchBuf(rows * 4);
    const { t: loss, e } = this.makeOut([1], [logits]);
    this.check(this.sym.gt_soft_ce_fwd(this.ctx, rows, V, k, zd, ti, tp, inv, e.data, lse, mass), "softCE");
    loss._backward = () => {
      if (!this.entries.get(loss)) throw new Error("backward over a graph built before a sync()");
      const seed = loss.grad[0];
      const [dz, acc] = this.gradDst(logits);
      if (dz !== 0n) this.check(this.sym.gt_soft_ce_bwd(this.ctx, rows, V, k, zd, ti, tp, inv, lse, mass, seed, dz, acc), "softCE.bwd");
    };
    return loss;
  }

  /** Raw GEMM for tests and benches (webgpu.ts:1654). */
  gemm(kind: number, acc: number, M: number, N: number, K: number, a: DevBuf, b: DevBuf, c: DevBuf) {
    this.check(this.sym.gt_gemm(this.ctx, kind, acc, M, N, K, a, b, c), "gemm");
  }
}

// ---- optimizers ---------------------------------------------------------------------------------------------------------
const u64s = (v: DevBuf[]) => BigUint64Array.from(v.length ? v : [0n]);

/** AdamWGpu (adamw-gpu.ts:131-251) over gt_adamw_*: weights, gradients and moments stay on the device; a step is three
 * launches for any number of tensors (sum of squares, clip scale, fused update). */
export class AdamWHip {
  readonly params: Tensor[];
  private gpu: HipBackend;
  private opts: Required<AdamOpts>;
  private baseLr: number;
  private lrScale = 1;
  private t = 0;
  private handle: Deno.PointerValue = null;
  private mBufs: DevBuf[] = [];
  private vBufs: DevBuf[] = [];

  constructor(gpu: HipBackend, params: Tensor[], opts: AdamOpts) {
    this.gpu = gpu;
    this.params = params;
    this.opts = { beta1: 0.9, beta2: 0.999, eps: 1e-8, weightDecay: 0.0, clip: 1.0, ...opts };
    this.baseLr = opts.lr;
    const w: DevBuf[] = [], g: DevBuf[] = [];
    for (const p of params) {
      const b = gpu.buffersFor(p); // uploads host weights once; accumulator on the device
      gpu.keepGradOnDevice(p);
      w.push(b.data);
      g.push(b.grad);
      this.mBufs.push(gpu.createStateBuffer(p.size * 4));
      this.vBufs.push(gpu.createStateBuffer(p.size * 4));
    }
    const sizes = BigInt64Array.from(params.length ? params.map((p) => BigInt(p.size)) : [0n]);
    const out = new BigUint64Array(1);
    const o = this.opts;
    gpu.check(
      gpu.symbols.gt_adamw_create(gpu.context, params.length, u64s(w), u64s(g), u64s(this.mBufs), u64s(this.vBufs), sizes,
        o.beta1, o.beta2, o.eps, o.weightDecay, o.clip, out),
      "gt_adamw_create",
    );
    this.handle = Deno.UnsafePointer.create(out[0]);
  }
  setLrScale(scale: number) {
    this.lrScale = scale;
  }
  /** No-op: accumulators live on the device and are re-armed when a step has consumed them. */
  zeroGrad() {}
  recordStep() {
    this.t += 1;
    const o = this.opts;
    const bc1 = 1 - Math.pow(o.beta1, this.t), bc2 = 1 - Math.pow(o.beta2, this.t);
    this.gpu.ensureGradsDefined(this.params);
    this.gpu.check(this.gpu.symbols.gt_adamw_step(this.gpu.context, this.handle, this.baseLr * this.lrScale, bc1, bc2), "gt_adamw_step");
    this.gpu.gradsConsumed(this.params);
  }
  /** ||g|| of the last step (what the clip compared with its threshold). */
  gradNorm(): number {
    const v = new Float32Array(1);
    this.gpu.check(this.gpu.symbols.gt_adamw_grad_norm(this.gpu.context, this.handle, v), "gt_adamw_grad_norm");
    return v[0];
  }
  async syncWeightsToHost(): Promise<void> {
    await this.gpu.sync(this.params);
  }
  async exportState(): Promise<{ m: Float32Array[]; v: Float32Array[]; t: number }> {
    const m: Float32Array[] = [], v: Float32Array[] = [];
    for (let i = 0; i < this.params.length; i++) {
      m.push(await this.gpu.readStateBuffer(this.mBufs[i], this.params[i].size));
      v.push(await this.gpu.readStateBuffer(this.vBufs[i], this.params[i].size));
    }
    return { m, v, t: this.t };
  }
  importState(s: { m: Float32Array[]; v: Float32Array[]; t: number }): void {
    if (s.m.length !== this.params.length || s.v.length !== this.params.length) {
      throw new Error(`adam state count mismatch: ${s.m.length}/${s.v.length} vs ${this.params.length}`);
    }
    for (let i = 0; i < this.params.length; i++) {
      this.gpu.writeStateBuffer(this.mBufs[i], s.m[i]);
      this.gpu.writeStateBuffer(this.vBufs[i], s.v[i]);
    }
    this.t = s.t;
  }
  destroy() {
    if (this.gpu.isDestroyed) { // the context took the tables and the buffers with it
      this.handle = null;
      this.mBufs = this.vBufs = [];
      return;
    }
    if (this.handle) {
      this.gpu.check(this.gpu.symbols.gt_adamw_destroy(this.gpu.context, this.handle), "gt_adamw_destroy");
      this.handle = null;
    }
    for (const b of [...this.mBufs, ...this.vBufs]) this.gpu.freeStateBuffer(b);
    this.mBufs = this.vBufs = [];
  }
}

export interface MuonHipOpts {
  lr: number;
  momentum?: number; // default 0.95
  nesterov?: boolean; // default true
  nsSteps?: number; // Newton-Schulz iterations, default 5
  aux: AdamOpts; // AdamW settings for the non-Muon group
}

/** MuonGpu (muon-gpu.ts:351-470) over gt_muon_*: matrices of equal shape are stepped as one batch. */
export class MuonHip {
  readonly auxParams: Tensor[];
  private gpu: HipBackend;
  private muonParams: Tensor[];
  private aux: AdamWHip;
  private baseLr: number;
  private lr: number;
  private handle: Deno.PointerValue = null;
  private momentumBufs: DevBuf[] = [];

  constructor(gpu: HipBackend, muonParams: Tensor[], auxParams: Tensor[], opts: MuonHipOpts) {
    this.gpu = gpu;
    this.muonParams = muonParams;
    this.auxParams = auxParams;
    this.aux = new AdamWHip(gpu, auxParams, opts.aux);
    this.baseLr = this.lr = opts.lr;
    const w: DevBuf[] = [], g: DevBuf[] = [], rows: number[] = [], cols: number[] = [];
    for (const p of muonParams) {
      if (p.shape.length !== 2) throw new Error("Muon param must be 2-D");
      const b = gpu.buffersFor(p);
      gpu.keepGradOnDevice(p);
      w.push(b.data);
      g.push(b.grad);
      rows.push(p.shape[0]);
      cols.push(p.shape[1]);
      this.momentumBufs.push(gpu.createStateBuffer(p.size * 4)); // zero at start
    }
    const out = new BigUint64Array(1);
    gpu.check(
      gpu.symbols.gt_muon_create(gpu.context, muonParams.length, u64s(w), u64s(g), u64s(this.momentumBufs),
        Int32Array.from(rows.length ? rows : [0]), Int32Array.from(cols.length ? cols : [0]),
        opts.momentum ?? 0.95, (opts.nesterov ?? true) ? 1 : 0, opts.nsSteps ?? 5, out),
      "gt_muon_create",
    );
    this.handle = Deno.UnsafePointer.create(out[0]);
  }
  setLrScale(scale: number) {
    this.lr = this.baseLr * scale;
    this.aux.setLrScale(scale);
  }
  zeroGrad() {
    this.aux.zeroGrad();
  }
  recordStep() {
    if (this.muonParams.length) {
      this.gpu.ensureGradsDefined(this.muonParams);
      this.gpu.check(this.gpu.symbols.gt_muon_step(this.gpu.context, this.handle, this.lr), "gt_muon_step");
      this.gpu.gradsConsumed(this.muonParams);
    }
    this.aux.recordStep();
  }
  async syncWeightsToHost(): Promise<void> {
    await this.gpu.sync([...this.muonParams, ...this.auxParams]);
  }
  async exportState(): Promise<{ muonMomentum: Float32Array[]; adamM: Float32Array[]; adamV: Float32Array[]; adamT: number }> {
    const muonMomentum: Float32Array[] = [];
    for (let i = 0; i < this.momentumBufs.length; i++) {
      muonMomentum.push(await this.gpu.readStateBuffer(this.momentumBufs[i], this.muonParams[i].size));
    }
    const adam = await this.aux.exportState();
    return { muonMomentum, adamM: adam.m, adamV: adam.v, adamT: adam.t };
  }
  importState(s: { muonMomentum: Float32Array[]; adamM: Float32Array[]; adamV: Float32Array[]; adamT: number }): void {
    if (s.muonMomentum.length !== this.momentumBufs.length) {
      throw new Error(`muon momentum count mismatch: ${s.muonMomentum.length} vs ${this.momentumBufs.length}`);
    }
    for (let i = 0; i < this.momentumBufs.length; i++) this.gpu.writeStateBuffer(this.momentumBufs[i], s.muonMomentum[i]);
    this.aux.importState({ m: s.adamM, v: s.adamV, t: s.adamT });
  }
  destroy() {
    if (!this.gpu.isDestroyed) {
      if (this.handle) this.gpu.check(this.gpu.symbols.gt_muon_destroy(this.gpu.context, this.handle), "gt_muon_destroy");
      for (const b of this.momentumBufs) this.gpu.freeStateBuffer(b);
    }
    this.handle = null;
    this.momentumBufs = [];
    this.aux.destroy();
  }
}

/** newtonSchulzGpu (muon-gpu.ts:259-283): the raw orthogonalisation of one matrix. */
export async function newtonSchulzHip(gpu: HipBackend, g: Float32Array, m: number, n: number, steps: number): Promise<Float32Array> {
  const src = gpu.createStateBuffer(m * n * 4), out = gpu.createStateBuffer(m * n * 4);
  try {
    gpu.writeStateBuffer(src, g);
    gpu.check(gpu.symbols.gt_newton_schulz(gpu.context, m, n, steps, src, out), "gt_newton_schulz");
    return await gpu.readStateBuffer(out, m * n);
  } finally {
    gpu.freeStateBuffer(src);
    gpu.freeStateBuffer(out);
  }
}

// ---- factories (webgpu.ts:1812-1888) -------------------------------------------------------------------------------------
function libPath(): string {
  return Deno.env.get("GGUFHIP_LIB") ?? "./libggufhip.so";
}
/** initWebGPU analogue: a backend, or null when the library or an MI355X is not there. */
// deno-lint-ignore require-await
export async function initHip(device = 0): Promise<HipBackend | null> {
  try {
    return new HipBackend(libPath(), device);
  } catch {
    return null;
  }
}
/** requireGPU analogue: there is no CPU path behind this backend. */
// deno-lint-ignore require-await
// bf16Pieces: the FP32 products and the attention kernels that have such a form on the bf16 matrix instruction (each FP32 element as three
// exact bf16 pieces, FP32 accumulation): as close to float64 as the FP32 MFMA kernels, about 1.3 x faster steps, not bit-identical to them.
export async function requireHip(purpose: string, device = 0, bf16Pieces = false): Promise<HipBackend> {
  try {
    const hip = new HipBackend(libPath(), device);
    if (bf16Pieces) {
      hip.setOption("gemm.split_bf16", 1);
      hip.setOption("attn.split_bf16", 1);
    }
    return hip;
  } catch (e) {
    throw new Error(`${purpose} needs an MI355X and libggufhip.so (GGUFHIP_LIB): ${(e as Error).message}`);
  }
}
