"""HipBackend: the device backend behind the autograd op set, on one MI355X.

Mirrors the public surface of WebGPUBackend (src/backend/webgpu.ts:290-1888): it implements
OpsBackend (every op records device work, installs `out._backward`, returns at once) and
RegionBackend (begin_region / end_region / seed_grad_from for `checkpoint`), plus the buffer
surface the device optimizers and the trainer use (buffers_for, keep_grad_on_device,
create/write/read_state_buffer, upload_params, sync, reclaim_step_transients, resident_bytes,
region_count, start/stop_profile). All work goes to the one HIP stream the library context owns.

What differs from the reference, on purpose:
  * Gradient buffers are not cleared and then added to. Each backward kernel is told whether it is
    the first writer of its destination in this accumulation window (store) or a later one (add),
    so an intermediate's gradient costs one write instead of clear + read + write, and
    `grad_clears_issued` stays near zero. Parameter accumulators follow the same rule across the
    micro-batches of a step and are re-armed when the optimizer has consumed them.
  * Intermediate gradient buffers are allocated at their first write in backward, not at forward.
  * silu/gelu outputs are lazy: when their only use is the gate of `mul`, forward and backward run
    the fused gated-activation kernels on the pre-activation and the activation tensor never
    exists in memory. Any other consumer materialises it and the unfused kernels run.
  * Host arrays of intermediates are never allocated unless sync() is asked to read them.
  * Launches are held back where the next op can ride them. A linear's forward waits one op: a second linear of the
    same shape over the same input joins it as a batch of two (k and v, gate and up), an add of its output is written
    by the product's own write-back (the residual add). A linear's input gradient waits until that gradient is next
    touched: sibling projections then leave as one summed product. A linear's weight gradient waits for up to seven more:
    consecutive ones leave as one grouped launch. add's backward launches nothing where it is the
    first writer: the operand's gradient points at the upstream buffer until somebody adds to it.
  * attention keeps its scores from the forward to the backward where a backward can come and a byte budget allows,
    as the reference's small-T path keeps its probabilities (webgpu.ts:1176-1189).
  * Consecutive micro-batches are recorded on different streams (see __init__), each with its own pool of transient
    buffers and its own parameter-gradient accumulators, summed in stream order before anything reads them.
  Each of these has a switch (batch_linears, fuse_residual_add, fuse_sibling_dx, group_dw, alias_add_grads, attn_keep_scores) and
  gives the same gradients as the one-launch-per-op form: bit for bit, or to rounding where a sum changes its order.
"""
from __future__ import annotations

import ctypes as C
import gc
import math
import weakref

import numpy as np

from . import autograd as ag
from .autograd import Tensor
from .lib import NN, NT, TN, HipError, ProfRec, buf as c_buf, check, lib

_ALIGN = 256


class _EntryMap:
    """Tensor -> device record, the WeakMap<Tensor, Entry> of webgpu.ts:322. The record sits in the tensor's own `_dev` slot
    (a plain attribute read where a WeakKeyDictionary costs a weak reference and a hash per look-up, tens of thousands per
    step); it dies with the tensor. A tensor already claimed by another live backend falls back to a weak dictionary."""
    __slots__ = ("_key", "_spill")

    def __init__(self):
        self._key = object()
        self._spill = weakref.WeakKeyDictionary()

    def get(self, t, default=None):
        d = t._dev
        if d is not None and d[0] is self._key:
            return d[1]
        if self._spill:
            return self._spill.get(t, default)
        return default

    def __getitem__(self, t):
        e = self.get(t)
        if e is None:
            raise KeyError(t)
        return e

    def __setitem__(self, t, e):
        d = t._dev
        if d is None or d[0] is self._key:
            t._dev = (self._key, e)
        else:
            self._spill[t] = e

    def pop(self, t, default=None):
        d = t._dev
        if d is not None and d[0] is self._key:
            t._dev = None
            return d[1]
        return self._spill.pop(t, default)


class _Entry:
    __slots__ = ("data", "grad", "nbytes", "external", "grad_init", "lazy_act", "consumers", "fused_uses",
                 "region", "keep_grad", "extra", "needs_grad", "lazy_lin", "grad_src", "stream", "sgrad", "rope_of", "rope_fused")

    def __init__(self, nbytes, external):
        self.data = 0
        self.grad = 0
        self.nbytes = nbytes
        self.external = external
        self.grad_init = False
        self.lazy_act = None        # (x tensor, act id) while a silu/gelu output has not been computed
        self.consumers = 0
        self.fused_uses = 0
        self.region = 0
        self.keep_grad = False
        self.extra = None           # (buf, nbytes) of a saved buffer that lives and dies with this output (attention scores)
        self.needs_grad = False     # an intermediate below a trainable tensor: a backward through it may be asked for
        self.lazy_lin = None        # (rows, out, in, x data, w data) while a linear's output lives only inside a fused add
        self.grad_src = 0           # another tensor's gradient buffer that holds this gradient's value so far (add's backward)
        self.stream = 0             # the stream whose launches produce and consume this tensor (its buffers come from that stream's pool)
        self.sgrad = None           # parameters: {stream: [accumulator, written?]} of the streams other than the first
        self.rope_of = None         # a rotation's output: (input tensor, (T, hd, base, pos))
        self.rope_fused = False     # an attention backward wrote the rotation's input gradient itself: the rotation's closure has nothing to do


class HipBackend:
    def __init__(self, device: int = 0, streams: int = 4):
        """streams: how many HIP streams (library contexts on the one device) consecutive micro-batches are dealt to.
        The reference's trainer records one sequence's forward and backward at a time (src/backend/train-gpu.ts:200-219);
        a 2048-row graph cannot fill 256 CUs launch by launch, but micro-batches are independent until their parameter
        gradients meet, so each goes to the next stream, keeps its own parameter-gradient accumulators there, and the
        accumulators are summed in stream order (gt_grad_fold) before anything reads them. 1 = everything on one stream."""
        self._nstreams = max(1, min(int(streams), 8))
        self._ctxs = []
        for _ in range(self._nstreams):
            c = C.c_void_p()
            if lib.gt_ctx_create(device, C.byref(c)) != 0:
                msg = (lib.gt_last_error(None) or b"").decode()
                for made in self._ctxs:
                    lib.gt_ctx_destroy(made)
                raise HipError("gt_ctx_create: " + msg)
            self._ctxs.append(c)
        self._cur = 0                     # stream of the micro-batch being recorded
        self._used = set()                # streams other than the first with work queued since the last join
        self._bw_seen = False             # a backward closure has run since the last switch: the next graph root starts a micro-batch
        self.backward_depth = 0           # raised by autograd while closures are walked: a checkpoint's replay is not a new graph
        # the first stream holds work (uploads, an optimizer step, a fold) another stream must not overtake: the point is
        # marked on the first stream when that work is queued, and a stream that starts a micro-batch afterwards waits for
        # the mark on the device (the host does not wait, and the first stream's own micro-batch is not waited for)
        self._s0_barrier = False
        self._s0_waited: set = set()
        self._sfold: list = []            # (tensor, entry) of parameters with a written accumulator on another stream
        self._limbo: list = []            # entries of parameters that were released or collected: their buffers return to the pools at the next sync
        self.adapter_name = lib.gt_device_name(self._ctx).decode()
        self.attn_flash_min_t = 2048      # kept for interface parity; one kernel family serves every T here
        self.last_sync_readback_bytes = 0
        self.grad_clears_issued = 0
        self.fuse_glu = True
        self._pools = [dict() for _ in range(self._nstreams)]     # per stream: size class -> free buffers
        self._pool_bytes = 0
        self._state_bytes = 0
        self._entries = _EntryMap()
        self._externals: "weakref.WeakSet[Tensor]" = weakref.WeakSet()
        self._touched: list = []
        self._touched_ids: set = set()
        self._transients: list = []       # (tensor weakref-free strong ref, entry) in creation order
        self._scratch: list = []          # (buf, nbytes) raw transients: id uploads, saved statistics
        self._regions_opened = 0
        self._pend = None                 # (x, T, out, in, x data, w data, out data) of a held-back linear launch
        self._pend_rope = None            # ((rows, T, hd, base, pos, backward), H, source, destination, accumulate) of a held-back rotation
        self.pair_ropes = True
        # input gradients of linears held back in the backward, by input tensor: id(x) -> (x, rows, in, [(dY, W, out), ...]).
        # Sibling projections of one activation (q/k/v, gate/up) then leave as ONE product dX = sum of dY_i.W_i; whoever
        # touches x's gradient next, and every point where buffers can change hands, sends what is held first.
        self._pend_dx: dict = {}
        self.fuse_sibling_dx = True
        # weight gradients of linears held back in the backward: [(rows, dY, x data, dW, acc, out, in)]. Up to eight
        # consecutive ones over the same number of rows leave as ONE grouped launch (gt_gemm_group): the dW of a layer's
        # seven projections are each too small an output to fill the chip, together they are not. Sent when the group is
        # full, when a weight in it is touched again (its gradient read or written: tied matrices, a weight used twice),
        # and at every point where buffers can change hands.
        self._pend_dw: list = []
        self._pend_dw_ids: set = set()
        self.group_dw = True
        # weight gradients of normalisations held back in the backward: the kernel leaves one partial row per workgroup and
        # the column sums of every pending one leave as ONE launch (gt_colsum_group) when anything is about to read or write
        # one of those gradients, and wherever buffers can change hands: [(parts, rows of parts, d, dw, acc)]
        self._pend_cs: list = []
        self._pend_cs_ids: set = set()
        self.defer_norm_dw = True
        self._pend_rs: list = []          # held-back slice sums of adapter gradients: (parts, slices, len, destination, acc)
        self._pend_rs_ids: set = set()
        self.defer_rank_sums = True
        # attention's backward applies the backward of the rotations its q and k came through in the write-backs of dQ and
        # dK (gt_attn_bwd_scores_rope) where q / k are rotation outputs nobody else has read: no rope.bwd launch is left
        self.fuse_rope_bwd = True
        self.fuse_residual_add = True
        # add's backward hands its upstream gradient on instead of copying it: an operand whose gradient has no writer yet
        # points at the upstream buffer (grad_src). A reader takes that buffer as it is; the first later writer adds to its
        # contents (rmsNorm's backward reads them from there, any other op has them copied first); aliases are settled
        # before any buffer they point at can be recycled.
        self.alias_add_grads = True
        self._aliased: list = []
        self.batch_linears = True
        # attention keeps its scores from the forward to the backward (one [T, T] matrix per sequence and head) when a
        # gradient will be asked for, one call's matrices fit attn_scores_max_bytes and the live ones together stay
        # within attn_scores_budget_bytes: memory spent to take one of four contractions out of dK/dV
        self.attn_keep_scores = True
        self.attn_scores_max_bytes = 4 << 30
        self.attn_scores_budget_bytes = 96 << 30
        self._scores_taken = 0
        self.forward_only_region = False  # set by checkpoint() around a block's first forward, whose interior is never differentiated
        self._profiling = False
        self._destroyed = False
        self._explicit_micro_batches = False     # set by next_micro_batch(): boundaries are told, not inferred
        self.manage_gc = True
        self._gc_managed = False
        self._gc_was_enabled = True

    # ---- streams ------------------------------------------------------------------------------------------------
    @property
    def _ctx(self):
        return self._ctxs[self._cur]

    def _op_begin(self, *inputs):
        """Called first thing by every forward op. After a backward has run, an op whose inputs are all parameters or
        host data is the root of the next micro-batch's graph: it goes to the next stream."""
        if not self._bw_seen or self._nstreams == 1 or self.backward_depth or self._explicit_micro_batches:
            return                  # (a forward op inside a backward is a checkpoint replaying its block: same micro-batch)
        for t in inputs:
            e = self._entries.get(t)
            if e is not None and not e.external:
                return
        self._advance_stream()

    def next_micro_batch(self):
        """The trainer says where a micro-batch's graph begins: call it at the top of the loop body that builds one
        sequence's forward and backward (train-gpu.ts:200-219). From the first call on the backend stops inferring the
        boundary from the ops' inputs (see _op_begin: that inference holds for graphs whose first op takes only parameters
        and host data, like the three in arch.py, and for nothing else). A call before any backward has run since the last
        boundary changes nothing, so the first micro-batch of a step stays on the first stream."""
        self._explicit_micro_batches = True
        if self._bw_seen and self._nstreams > 1 and not self.backward_depth:
            self._advance_stream()

    def _advance_stream(self):
        self._flush()
        self._flush_dx()
        self._cur = (self._cur + 1) % self._nstreams
        if self._cur:
            self._used.add(self._cur)
            if self._s0_barrier and self._cur not in self._s0_waited:
                check(self._ctx, lib.gt_stream_wait(self._ctx, self._ctxs[0]), "gt_stream_wait")
                self._s0_waited.add(self._cur)
        self._bw_seen = False

    def _barrier0(self):
        """Work that the other streams must not overtake has just been queued on the first stream."""
        check(self._ctxs[0], lib.gt_stream_mark(self._ctxs[0]), "gt_stream_mark")
        self._s0_barrier = True
        self._s0_waited = set()

    def _join(self):
        """Everything recorded on the other streams has finished and their parameter-gradient accumulators are summed, in
        stream order, into the first stream's; recording continues on the first stream."""
        self._flush()
        self._flush_dx()
        self._bw_seen = False
        if self._cur == 0 and not self._used and not self._sfold:
            return
        for s in sorted(self._used):
            check(self._ctxs[s], lib.gt_sync(self._ctxs[s]), "gt_sync")
        self._used = set()
        self._cur = 0
        self._bw_seen = False
        if self._sfold:
            seen, items = set(), []
            for t, e in self._sfold:
                if id(e) not in seen:
                    seen.add(id(e))
                    items.append((t, e))
            self._sfold = []
            n, ns = len(items), self._nstreams - 1
            dst, acc, src, sizes = (c_buf * n)(), (C.c_int * n)(), (c_buf * (n * ns))(), (C.c_int64 * n)()
            for i, (t, e) in enumerate(items):
                if e.grad == 0:
                    e.grad = self._acquire(e.nbytes, 0)
                dst[i], acc[i], sizes[i] = e.grad, 1 if e.grad_init else 0, e.nbytes // 4
                for s_ in range(1, self._nstreams):
                    slot = e.sgrad.get(s_)
                    if slot is not None and slot[1]:
                        src[i * ns + s_ - 1] = slot[0]
                        slot[1] = False
                e.grad_init = True
            check(self._ctxs[0], lib.gt_grad_fold(self._ctxs[0], n, dst, acc, ns, src, sizes), "gt_grad_fold")
            self._barrier0()

    # ---- install (webgpu.ts:393-399) ---------------------------------------------------------------
    # ---- a linear's forward launch is held back by one op: two consecutive linears over the same input with the same
    # shape (k and v, gate and up) then go out as ONE batched launch, which fills the chip better than two small ones
    def _flush(self):
        p = self._pend
        if p is not None:
            self._pend = None
            check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, p[1], p[2], p[3], p[4], p[5], p[6]), "linear")
        r = self._pend_rope
        if r is not None:
            self._pend_rope = None
            self._launch_rope(r)

    # ---- a forward rotation is held back by one op as well: the q and k of a layer (same rows, T, head dim, base and
    # offset) then leave as ONE launch. Anything that reads or writes a buffer goes through _flush first.
    def _launch_rope(self, r, other=None):
        (rows, T, hd, base, pos, bwd), H, src, dst, acc = r
        if other is None:
            check(self._ctx, lib.gt_rope(self._ctx, rows, T, H, hd, base, pos, bwd, src, dst, acc), "rope.bwd" if bwd else "rope")
        else:
            _, H2, src2, dst2, acc2 = other
            check(self._ctx, lib.gt_rope_pair(self._ctx, rows, T, hd, base, pos, bwd, H, src, dst, acc, H2, src2, dst2, acc2),
                  "rope.bwd" if bwd else "rope")

    def _rope(self, r):
        """Launch r with the held-back rotation if they match, else launch that one and hold r. The caller has already
        taken self._pend_rope (as `held`, passed inside r's call) so that its own buffer lookups did not flush it."""
        held, r = r
        if not self.pair_ropes:
            if held is not None:
                self._launch_rope(held)
            self._launch_rope(r)
        elif held is not None and held[0] == r[0]:
            self._launch_rope(held, r)
        else:
            if held is not None:
                self._launch_rope(held)
            self._pend_rope = r

    def _flush_dw(self):
        """Launch the held-back weight-gradient products as one group."""
        pend = self._pend_dw
        if not pend:
            return
        self._pend_dw = []
        self._pend_dw_ids = set()
        n = len(pend)           # a single one goes the same way: its K split must not depend on the company it has
        ms = (C.c_int * n)(*[p[5] for p in pend])
        ns = (C.c_int * n)(*[p[6] for p in pend])
        gs = (c_buf * n)(*[p[1] for p in pend])
        xs = (c_buf * n)(*[p[2] for p in pend])
        ds = (c_buf * n)(*[p[3] for p in pend])
        accs = (C.c_int * n)(*[p[4] for p in pend])
        check(self._ctx, lib.gt_gemm_group(self._ctx, TN, n, ms, ns, pend[0][0], gs, xs, ds, accs), "linear.dw")

    def _hold_dw(self, w: Tensor, rows, g, xd, dw, accw, outd, ind):
        if self._pend_dw and self._pend_dw[0][0] != rows:
            self._flush_dw()
        self._pend_dw.append((rows, g, xd, dw, accw, outd, ind))
        self._pend_dw_ids.add(id(w))
        if len(self._pend_dw) == 8:
            self._flush_dw()

    def _flush_cs(self):
        """The column sums of every held-back normalisation weight gradient, one launch."""
        pend = self._pend_cs
        if not pend:
            return
        self._pend_cs = []
        self._pend_cs_ids = set()
        n = len(pend)
        check(self._ctx, lib.gt_colsum_group(self._ctx, n, (c_buf * n)(*[p[0] for p in pend]), (C.c_int * n)(*[p[1] for p in pend]),
                                             (C.c_int * n)(*[p[2] for p in pend]), (c_buf * n)(*[p[3] for p in pend]),
                                             (C.c_int * n)(*[p[4] for p in pend])), "rmsnorm.dw")

    def _flush_rs(self):
        """The slice sums of every held-back adapter gradient, one launch."""
        pend = self._pend_rs
        if not pend:
            return
        self._pend_rs = []
        self._pend_rs_ids = set()
        n = len(pend)
        check(self._ctx, lib.gt_rank_slices_group(self._ctx, n, (c_buf * n)(*[p[0] for p in pend]), (C.c_int * n)(*[p[1] for p in pend]),
                                                  (C.c_int * n)(*[p[2] for p in pend]), (c_buf * n)(*[p[3] for p in pend]),
                                                  (C.c_int * n)(*[p[4] for p in pend])), "lora.slices")

    def _rank_grad(self, param, rows, K, r, h, y, transpose_out, acc, dst, label):
        """dst (+)= the rank-r gradient product; its slice sums are held back for one grouped launch when the library
        would go through partial sums and nobody can be reading the gradient before the backward ends."""
        if self.defer_rank_sums:
            ns = C.c_int(0)
            check(self._ctx, lib.gt_rank_grad_slices(self._ctx, rows, K, r, y, C.byref(ns)), label)
            if ns.value > 0:
                parts = self._scratch_buf(ns.value * r * K * 4)
                check(self._ctx, lib.gt_rank_grad_parts(self._ctx, rows, K, r, h, y, transpose_out, parts), label)
                self._pend_rs.append((parts, ns.value, r * K, dst, acc))
                self._pend_rs_ids.add(id(param))
                return
        check(self._ctx, lib.gt_rank_grad(self._ctx, rows, K, r, h, y, transpose_out, acc, dst), label)

    def _flush_dx(self, t: Tensor = None):
        """Launch the held-back input-gradient products: those into t's gradient, or all of them (then the held-back
        weight-gradient products and column sums go too)."""
        if t is None and self._pend_dw:
            self._flush_dw()
        if t is None and self._pend_cs:
            self._flush_cs()
        if t is None and self._pend_rs:
            self._flush_rs()
        if not self._pend_dx:
            return
        if t is None:
            items = list(self._pend_dx.values())
            self._pend_dx.clear()
        else:
            it = self._pend_dx.pop(id(t), None)
            if it is None:
                return
            items = [it]
        for x, rows, ind, parts in items:
            dx, acc = self._gdst(x)
            if not dx:
                continue
            if len(parts) == 1:
                g, wd, outd = parts[0]
                check(self._ctx, lib.gt_gemm(self._ctx, NN, acc, rows, ind, outd, g, wd, dx), "linear.dx")
            else:
                n = len(parts)
                ks = (C.c_int * n)(*[p[2] for p in parts])
                gs = (c_buf * n)(*[p[0] for p in parts])
                ws = (c_buf * n)(*[p[1] for p in parts])
                check(self._ctx, lib.gt_gemm_sum(self._ctx, NN, acc, rows, ind, n, ks, gs, ws, dx), "linear.dx")

    def install(self):
        """Becomes the ops backend (webgpu.ts:393-399). While installed, and unless manage_gc is off, the interpreter's cyclic
        garbage collector runs only inside sync(): a step's graph is tens of thousands of tensors and closures that refer to
        each other, and collections triggered in the middle of recording cost 50 ms of host time per step of eight 2048-row
        graphs (one in four steps 50 ms more, a full collection), during which the device runs out of queued work. What exists
        at install time (modules, the model) is frozen out of the collector's sight so that the collection in sync() only
        walks what a step made."""
        ag.set_ops_backend(self)
        if self.manage_gc and not self._gc_managed:
            self._gc_managed = True
            self._gc_was_enabled = gc.isenabled()
            gc.freeze()
            gc.disable()

    def uninstall(self):
        ag.set_ops_backend(None)
        if self._gc_managed:
            self._gc_managed = False
            gc.unfreeze()
            if self._gc_was_enabled:
                gc.enable()

    # ---- raw memory ------------------------------------------------------------------------------------
    def _acquire(self, nbytes: int, stream: int = None) -> int:
        """A buffer from the pool of `stream` (default: the one being recorded on). A buffer only ever returns to the pool
        it came from, so it is only ever reused by launches ordered after its last use."""
        s_ = self._cur if stream is None else stream
        size = max(_ALIGN, (nbytes + _ALIGN - 1) // _ALIGN * _ALIGN)
        free = self._pools[s_].get(size)
        if free:
            return free.pop()
        out = c_buf()
        ctx = self._ctxs[s_]
        if lib.gt_alloc(ctx, size, 0, C.byref(out)) != 0:
            # device memory is full of free buffers of other size classes (another model shape ran before): give them
            # back and ask again; only then is it an error
            if not self.trim_pool():
                check(ctx, 1, "gt_alloc")
            check(ctx, lib.gt_alloc(ctx, size, 0, C.byref(out)), "gt_alloc")
        self._pool_bytes += size
        return out.value

    def trim_pool(self) -> int:
        """Return every free buffer of the pool to the device (buffers in use stay). Gives the bytes freed."""
        freed = 0
        for ctx, pool in zip(self._ctxs, self._pools):
            check(ctx, lib.gt_sync(ctx), "gt_sync")      # queued kernels may still use a buffer recycled at a region's end
            for size, free in pool.items():
                for b in free:
                    check(ctx, lib.gt_free(ctx, b), "gt_free")
                    freed += size
                free.clear()
        self._pool_bytes -= freed
        return freed

    def _recycle(self, b: int, nbytes: int, stream: int = None):
        size = max(_ALIGN, (nbytes + _ALIGN - 1) // _ALIGN * _ALIGN)
        self._pools[self._cur if stream is None else stream].setdefault(size, []).append(b)

    def _scratch_buf(self, nbytes: int) -> int:
        b = self._acquire(nbytes)
        self._scratch.append((b, nbytes, self._cur))
        return b

    def _upload(self, arr: np.ndarray) -> int:
        arr = np.ascontiguousarray(arr)
        b = self._scratch_buf(arr.nbytes)
        check(self._ctx, lib.gt_h2d(self._ctx, b, arr.ctypes.data_as(C.c_void_p), arr.nbytes), "gt_h2d")
        return b

    # ---- entries (webgpu.ts:1539-1593) -----------------------------------------------------------------
    def _entry_for(self, t: Tensor) -> _Entry:
        """Device buffers of an existing tensor; a tensor never seen before is external (a parameter):
        it gets a persistent data buffer, uploaded once."""
        e = self._entries.get(t)
        if e is None:
            if t._prev:
                raise RuntimeError("backward over a graph built before a sync(): that sync recycled the graph's buffers")
            e = _Entry(t.size * 4, True)
            e.data = self._acquire(e.nbytes, 0)
            c0 = self._ctxs[0]
            check(c0, lib.gt_h2d(c0, e.data, t.data.ctypes.data_as(C.c_void_p), e.nbytes), "gt_h2d")
            if self._cur:
                check(c0, lib.gt_sync(c0), "gt_sync")       # uploaded on the first stream, read by this one
            else:
                self._barrier0()
            self._entries[t] = e
            self._externals.add(t)
            # when the tensor is collected its device buffers go back to the pools (at the next sync: queued work may still read them)
            weakref.finalize(t, self._limbo.append, e)
        if e.external and t.requires_grad and id(t) not in self._touched_ids:
            self._touched_ids.add(id(t))
            self._touched.append(t)
        return e

    def _make_out(self, shape, prev, alloc=True) -> tuple:
        out = Tensor(None, shape)
        out._prev = list(prev)
        e = _Entry(out.size * 4, False)
        e.stream = self._cur
        if alloc:
            e.data = self._acquire(e.nbytes)
        e.region = self._regions_opened
        for p in prev:
            pe = self._entries.get(p)
            if p.requires_grad or (pe is not None and pe.needs_grad):
                e.needs_grad = True
                break
        self._entries[out] = e
        self._transients.append((out, e))
        return out, e

    def _data(self, t: Tensor, launch_held: bool = True) -> int:
        """Device address of t's values, as an op input. launch_held = False is for an op that only records the
        address for later (a lazy activation): a held-back linear launch may then stay held."""
        if launch_held:
            self._flush()
        e = self._entry_for(t)
        if e.stream != self._cur and not e.external:
            # an intermediate of another micro-batch: that stream's work must be done before this one reads it
            check(self._ctxs[e.stream], lib.gt_sync(self._ctxs[e.stream]), "gt_sync")
        e.consumers += 1
        if e.lazy_act is not None:
            self._materialise(t, e)
        if e.lazy_lin is not None:
            self._materialise_lin(e)
        return e.data

    def _materialise(self, t: Tensor, e: _Entry):
        self._flush()
        x, act = e.lazy_act
        e.lazy_act = None
        e.data = self._acquire(e.nbytes, e.stream)
        xe = self._entry_for(x)
        fn = lib.gt_silu_fwd if act == 0 else lib.gt_gelu_fwd
        check(self._ctx, fn(self._ctx, t.size, xe.data, e.data), "act.fwd")

    def _materialise_lin(self, e: _Entry):
        """A linear output that went straight into a residual add is wanted on its own after all: compute it now."""
        rows, outd, ind, xd, wd = e.lazy_lin
        e.lazy_lin = None
        e.data = self._acquire(e.nbytes, e.stream)
        check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, rows, outd, ind, xd, wd, e.data), "linear")

    def _same_stream(self, e: _Entry):
        """An intermediate made by another micro-batch's stream is about to have its gradient read or written here
        (a closure walked after the recording moved on): that stream's queued work goes first."""
        if e.stream != self._cur and not e.external:
            check(self._ctxs[e.stream], lib.gt_sync(self._ctxs[e.stream]), "gt_sync")

    def _gdst(self, t: Tensor) -> tuple:
        """(gradient buffer, acc) for a backward kernel about to contribute to t's gradient;
        (0, 0) when t takes no gradient (a frozen parameter)."""
        self._flush()
        if self._pend_dx:
            self._flush_dx(t)       # products held back for this gradient go first: the order of its writers is kept
        if self._pend_dw and id(t) in self._pend_dw_ids:
            self._flush_dw()
        if self._pend_cs and id(t) in self._pend_cs_ids:
            self._flush_cs()
        if self._pend_rs and id(t) in self._pend_rs_ids:
            self._flush_rs()
        e = self._entries.get(t)
        if e is None:
            e = self._entry_for(t)
        self._bw_seen = True
        self._same_stream(e)
        if e.external and not t.requires_grad:
            return 0, 0
        if e.external and self._cur:
            # a parameter's gradient from a micro-batch on another stream than the first: that stream's own accumulator
            if e.sgrad is None:
                e.sgrad = {}
            slot = e.sgrad.get(self._cur)
            if slot is None:
                slot = e.sgrad[self._cur] = [self._acquire(e.nbytes), False]
            acc = 1 if slot[1] else 0
            if not slot[1]:
                slot[1] = True
                self._sfold.append((t, e))
            return slot[0], acc
        if e.grad == 0:
            e.grad = self._acquire(e.nbytes, e.stream)
        if e.grad_src:
            check(self._ctx, lib.gt_d2d(self._ctx, e.grad, e.grad_src, e.nbytes), "gt_d2d")
            e.grad_src = 0
        acc = 1 if e.grad_init else 0
        e.grad_init = True
        return e.grad, acc

    def _gdst_from(self, t: Tensor) -> tuple:
        """(gradient buffer, acc, buffer holding its contents so far) for a kernel that can read the old contents from
        another buffer than the one it writes: a handed-on upstream gradient is then never copied."""
        e = self._entries.get(t)
        if e is not None and e.grad_src:
            self._flush()
            if self._pend_dx:
                self._flush_dx(t)
        if e is not None and e.grad_src:
            src = e.grad_src
            e.grad_src = 0
            if e.grad == 0:
                e.grad = self._acquire(e.nbytes, e.stream)
            return e.grad, 1, src
        dst, acc = self._gdst(t)
        return dst, acc, dst

    def _settle_aliases(self, released_ids):
        """Before buffers are recycled: a handed-on gradient of a tensor that lives on gets its own copy, one of a tensor
        that is being released is dropped."""
        if not self._aliased:
            return
        for t in self._aliased:
            e = self._entries.get(t)
            if e is None or not e.grad_src:
                continue
            if id(t) in released_ids:
                e.grad_src = 0
                e.grad_init = False
            else:
                if e.grad == 0:
                    e.grad = self._acquire(e.nbytes, e.stream)
                check(self._ctx, lib.gt_d2d(self._ctx, e.grad, e.grad_src, e.nbytes), "gt_d2d")
                e.grad_src = 0
        self._aliased = []

    def _gsrc(self, t: Tensor) -> int:
        """Gradient buffer of an op output inside its backward closure."""
        self._flush()
        if self._pend_dx:
            self._flush_dx(t)
        if self._pend_dw and id(t) in self._pend_dw_ids:
            self._flush_dw()
        if self._pend_cs and id(t) in self._pend_cs_ids:
            self._flush_cs()
        if self._pend_rs and id(t) in self._pend_rs_ids:
            self._flush_rs()
        e = self._entries.get(t)
        if e is None:
            raise RuntimeError("backward over a graph built before a sync(): that sync recycled the graph's "
                               "gradient buffers, so this backward would read pool garbage")
        self._bw_seen = True
        self._same_stream(e)
        if e.grad_src:
            return e.grad_src       # handed on by an add's backward and not written since: read it where it is
        if e.grad == 0 or not e.grad_init:
            # nothing downstream wrote it (an output the loss does not depend on): its gradient is zero
            if e.grad == 0:
                e.grad = self._acquire(e.nbytes, e.stream)
            check(self._ctx, lib.gt_memset0(self._ctx, e.grad, e.nbytes), "gt_memset0")
            self.grad_clears_issued += 1
            e.grad_init = True
        return e.grad

    # ---- public buffer surface (webgpu.ts:1432-1537) ----------------------------------------------------
    def upload_params(self, tensors):
        self._join()
        for t in tensors:
            e = self._entry_for(t)
            check(self._ctx, lib.gt_h2d(self._ctx, e.data, t.data.ctypes.data_as(C.c_void_p), e.nbytes), "gt_h2d")
        self._barrier0()

    def buffers_for(self, t: Tensor) -> dict:
        self._join()
        e = self._entry_for(t)
        if t.requires_grad and e.grad == 0:
            e.grad = self._acquire(e.nbytes, e.stream)
            check(self._ctx, lib.gt_memset0(self._ctx, e.grad, e.nbytes), "gt_memset0")
            self.grad_clears_issued += 1
        return {"data": e.data, "grad": e.grad}

    def release(self, tensors):
        """Give back the device buffers of parameters that are no longer needed (a model being dropped): values, gradient
        accumulators on every stream. They return to the pools at the next sync(); a tensor used again after that is
        uploaded afresh."""
        self._join()
        for t in tensors:
            e = self._entries.get(t)
            if e is not None and e.external:
                self._entries.pop(t, None)
                self._externals.discard(t)
                self._limbo.append(e)

    def _drain_limbo(self):
        """Called with every stream idle."""
        seen = set()
        while self._limbo:
            e = self._limbo.pop()
            if id(e) in seen:
                continue
            seen.add(id(e))
            if e.data:
                self._recycle(e.data, e.nbytes, 0)
            if e.grad:
                self._recycle(e.grad, e.nbytes, 0)
            for s_, slot in (e.sgrad or {}).items():
                self._recycle(slot[0], e.nbytes, s_)
            e.data = e.grad = 0
            e.sgrad = None
        self._sfold = [(t, e) for t, e in self._sfold if e.data]

    def free_state_buffer(self, b: int):
        """Free a buffer made by create_state_buffer (waits for the first stream)."""
        c0 = self._ctxs[0]
        check(c0, lib.gt_free(c0, b), "gt_free")

    def keep_grad_on_device(self, t: Tensor):
        self._entry_for(t).keep_grad = True

    def grads_consumed(self, tensors):
        """The optimizer has read these accumulators: the next backward write stores instead of adding
        (the reference's deferred per-step clear, src/backend/muon-gpu.ts:8-16)."""
        self._join()
        self._barrier0()             # the optimizer's launches are on the first stream: no other stream may read weights before them
        for t in tensors:
            e = self._entries.get(t)
            if e is not None:
                e.grad_init = False

    def ensure_grads_defined(self, tensors):
        """An accumulator no kernel wrote since it was last consumed holds zero, as a cleared one would."""
        self._join()
        for t in tensors:
            e = self._entry_for(t)
            if e.grad == 0:
                e.grad = self._acquire(e.nbytes, e.stream)
            if not e.grad_init:
                check(self._ctx, lib.gt_memset0(self._ctx, e.grad, e.nbytes), "gt_memset0")
                self.grad_clears_issued += 1
                e.grad_init = True

    def seed_grad_from_host(self, t: Tensor):
        self._flush()
        self._flush_dx()
        e = self._entries.get(t)
        if e is None:
            raise RuntimeError("seed_grad_from_host: tensor has no device buffers")
        if e.grad == 0:
            e.grad = self._acquire(e.nbytes, e.stream)
        check(self._ctx, lib.gt_h2d(self._ctx, e.grad, t.grad.ctypes.data_as(C.c_void_p), e.nbytes), "gt_h2d")
        e.grad_init = True
        e.grad_src = 0

    def create_state_buffer(self, nbytes: int) -> int:
        out = c_buf()
        c0 = self._ctxs[0]
        check(c0, lib.gt_alloc(c0, max(4, nbytes), 1, C.byref(out)), "gt_alloc")
        self._barrier0()
        self._state_bytes += max(4, nbytes)
        return out.value

    def write_state_buffer(self, b: int, arr: np.ndarray):
        self._join()
        arr = np.ascontiguousarray(arr)
        check(self._ctx, lib.gt_h2d(self._ctx, b, arr.ctypes.data_as(C.c_void_p), arr.nbytes), "gt_h2d")
        self._barrier0()

    def read_state_buffer(self, b: int, n: int, dtype=np.float32) -> np.ndarray:
        self._join()
        out = np.empty(n, dtype=dtype)
        check(self._ctx, lib.gt_d2h(self._ctx, out.ctypes.data_as(C.c_void_p), b, out.nbytes), "gt_d2h")
        return out

    def set_option(self, key: str, value: int):
        """Kernel-selection switches for tests and tuning: "attn.generic", "attn.splits", "gemm.tile", "gemm.splitk", "gemm.staged",
        and "prof.sample" (time every n-th launch of a label)."""
        if key == "attn.generic" and self._transients:
            # an attention forward already recorded has chosen its kernel family (and may hold kept scores in that
            # family's layout); its backward must run in the same one
            raise RuntimeError("set_option: attn.generic cannot change while a graph is live; sync() first")
        for c in self._ctxs:
            check(c, lib.gt_set_option(c, key.encode(), int(value)), "gt_set_option")

    def resident_bytes(self) -> int:
        total = 0
        for c in self._ctxs:
            v = C.c_uint64()
            lib.gt_resident_bytes(c, C.byref(v))
            total += int(v.value)
        return total

    def region_count(self) -> int:
        return self._regions_opened

    @property
    def ctx(self):
        """The first stream's library context: state buffers, optimizers and raw calls of tests live there."""
        return self._ctxs[0]

    # ---- sync / reclaim (webgpu.ts:419-636) -------------------------------------------------------------
    def _release_transients(self, keep=()):
        keep_ids = {id(t) for t in keep}
        self._settle_aliases({id(t) for t, _ in self._transients if id(t) not in keep_ids})
        kept = []
        for t, e in self._transients:
            if id(t) in keep_ids:
                kept.append((t, e))
                continue
            if e.data:
                self._recycle(e.data, e.nbytes, e.stream)
            if e.grad:
                self._recycle(e.grad, e.nbytes, e.stream)
            if e.extra:
                self._recycle(e.extra[0], e.extra[1], e.stream)
                self._scores_taken -= e.extra[1]
                e.extra = None
            e.data = e.grad = 0
            self._entries.pop(t, None)
        self._transients = kept
        for b, n, s_ in self._scratch:
            self._recycle(b, n, s_)
        self._scratch = []

    def sync(self, reads=()):
        """Wait for the stream; read back `reads` (values) and the accumulated gradients of every
        trainable external tensor touched since the last sync that is not kept on the device; recycle
        all intermediates. The graph is unusable for backward afterwards."""
        if self._gc_managed:
            self._flush()
            self._flush_dx()
            gc.collect()                # the last step's graph, while the device still has this step's launches to run
        self._join()
        nbytes = 0
        for t in reads:
            e = self._entries.get(t)
            if e is None:
                raise RuntimeError("sync: tensor has no device buffers")
            if e.lazy_act is not None:
                self._materialise(t, e)
            if e.lazy_lin is not None:
                self._materialise_lin(e)
            check(self._ctx, lib.gt_d2h(self._ctx, t.data.ctypes.data_as(C.c_void_p), e.data, e.nbytes), "gt_d2h")
            nbytes += e.nbytes
        for t in self._touched:
            e = self._entries.get(t)
            if e is None or e.keep_grad:
                continue
            if t.requires_grad:
                if e.grad and e.grad_init:
                    check(self._ctx, lib.gt_d2h(self._ctx, t.grad.ctypes.data_as(C.c_void_p), e.grad, e.nbytes), "gt_d2h")
                    nbytes += e.nbytes
                else:
                    t.grad.fill(0)
            # The window ends here: the next one starts this accumulator from zero. Keyed on the accumulator, not on
            # the flag as it reads now: a parameter frozen after its backward and thawed later would otherwise have the
            # next window add on top of this one's gradients (gpu-parity.ts:1980-2028).
            e.grad_init = False
        self._touched = []
        self._touched_ids = set()
        check(self._ctx, lib.gt_sync(self._ctx), "gt_sync")
        self._s0_barrier = False
        self.last_sync_readback_bytes = nbytes
        self._release_transients()
        self._scores_taken = 0
        if self._limbo:
            self._drain_limbo()

    def reclaim_step_transients(self, keep=()):
        """Free a finished micro-batch's intermediates mid-step; parameter gradients keep accumulating. Every stream is
        waited for, but the micro-batches keep their streams and accumulators: which stream the next one goes to, and
        the order in which gradients are summed, are the same with and without this call, so it changes no bit."""
        self._flush()
        self._flush_dx()
        for c in self._ctxs:
            check(c, lib.gt_sync(c), "gt_sync")
        self._s0_barrier = False
        self._release_transients(keep)

    def destroy(self):
        self._pend = None
        self._pend_rope = None
        self._pend_dx = {}
        self._pend_dw = []
        self._pend_cs = []
        self._pend_rs = []
        if self._gc_managed:             # destroyed while installed: hand the collector back
            self._gc_managed = False
            gc.unfreeze()
            if self._gc_was_enabled:
                gc.enable()
        if not self._destroyed:
            self._destroyed = True
            for c in self._ctxs:
                lib.gt_ctx_destroy(c)

    # ---- profiling (webgpu.ts:830-880) -----------------------------------------------------------------------
    def start_profile(self, prefix: str = ""):
        """Time every launch whose label starts with `prefix` ("" = all) with HIP events on the stream."""
        self._join()
        for c in self._ctxs:
            check(c, lib.gt_prof_begin(c, prefix.encode()), "gt_prof_begin")

    def stop_profile(self) -> dict:
        """label -> (total ms, launches, algorithmic work: FLOP or bytes)."""
        self._join()
        out = {}
        for c in self._ctxs:
            recs = (ProfRec * 128)()
            n = C.c_int()
            check(c, lib.gt_prof_end(c, recs, 128, C.byref(n)), "gt_prof_end")
            for i in range(n.value):
                k = recs[i].label.decode()
                ms, cnt, work = out.get(k, (0.0, 0, 0.0))
                out[k] = (ms + recs[i].ms, cnt + recs[i].count, work + recs[i].work)
        return out

    # ---- RegionBackend (webgpu.ts:639-761) ------------------------------------------------------------------------
    def begin_region(self) -> int:
        self._regions_opened += 1
        return len(self._transients)

    def end_region(self, mark: int, keep):
        self._flush()
        self._flush_dx()
        keep_ids = {id(t) for t in keep}
        tail = self._transients[mark:]
        self._settle_aliases({id(t) for t, _ in tail if id(t) not in keep_ids})
        del self._transients[mark:]
        for t, e in tail:
            if id(t) in keep_ids:
                self._transients.append((t, e))
                continue
            if e.data:
                self._recycle(e.data, e.nbytes, e.stream)
            if e.grad:
                self._recycle(e.grad, e.nbytes, e.stream)
            if e.extra:
                self._recycle(e.extra[0], e.extra[1], e.stream)
                self._scores_taken -= e.extra[1]
                e.extra = None
            e.data = e.grad = 0
            self._entries.pop(t, None)

    def seed_grad_from(self, dst: Tensor, src: Tensor):
        if dst.size != src.size:
            raise ValueError(f"seed_grad_from: size mismatch {dst.size} vs {src.size}")
        g = self._gsrc(src)
        d, _ = self._gdst(dst)
        check(self._ctx, lib.gt_d2d(self._ctx, d, g, dst.size * 4), "gt_d2d")

    # ---- ops --------------------------------------------------------------------------------------------------------
    def linear(self, x: Tensor, w: Tensor) -> Tensor:
        self._op_begin(x, w)
        T, ind = x.shape
        outd = w.shape[0]
        p = self._pend
        pair = self.batch_linears and p is not None and p[0] is x and p[1:4] == (T, outd, ind)
        if pair:
            self._pend = None               # taken: _data below must not launch it on its own
        xd, wd = self._data(x), self._data(w)
        out, e = self._make_out([T, outd], [x, w])
        if pair and (wd - p[5]) % 16 == 0 and (e.data - p[6]) % 16 == 0:
            # the held-back linear and this one as one batch of two: same input, weights and outputs a stride apart
            check(self._ctx, lib.gt_gemm_batched(self._ctx, NT, 0, T, outd, ind, xd, 0, p[5], (wd - p[5]) // 4,
                                                 p[6], (e.data - p[6]) // 4, 2), "linear x2")
        else:
            if pair:
                check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, p[1], p[2], p[3], p[4], p[5], p[6]), "linear")
            if self.batch_linears:
                self._pend = (x, T, outd, ind, xd, wd, e.data)      # launched by the next op, or paired with it
            else:
                check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, T, outd, ind, xd, wd, e.data), "linear")
        wants_dw = w.requires_grad

        def bw():
            g = self._gsrc(out)
            if self.fuse_sibling_dx:
                held = self._pend_dx.get(id(x))
                if held is None:
                    self._pend_dx[id(x)] = (x, T, ind, [(g, wd, outd)])
                else:
                    held[3].append((g, wd, outd))
                    if len(held[3]) == 3:
                        self._flush_dx(x)
            else:
                dx, acc = self._gdst(x)
                if dx:
                    check(self._ctx, lib.gt_gemm(self._ctx, NN, acc, T, ind, outd, g, wd, dx), "linear.dx")
            if wants_dw:
                dw, accw = self._gdst(w)
                if dw:
                    if self.group_dw:
                        self._hold_dw(w, T, g, xd, dw, accw, outd, ind)
                    else:
                        check(self._ctx, lib.gt_gemm(self._ctx, TN, accw, outd, ind, T, g, xd, dw), "linear.dw")

        out._backward = bw
        return out

    def lora_linear(self, x: Tensor, w: Tensor, a: Tensor, b: Tensor, sc: float) -> Tensor:
        """linear(x, w) + sc * linear(linear(x, a), b) (autograd.ts:760-781) as one recorded op. The scale is applied to
        the rank-r activation h = x.a^T (inside the streaming rank kernels) instead of the [rows, out] product, the adapter product is
        accumulated into the base output by the GEMM itself, and the backward reads the upstream gradient directly:
        no [rows, out] elementwise pass in either direction."""
        self._op_begin(x, w, a, b)
        T, ind = x.shape
        outd, r = w.shape[0], a.shape[0]
        xd, wd, ad, bd = self._data(x), self._data(w), self._data(a), self._data(b)
        out, e = self._make_out([T, outd], [x, w, a, b])
        hs = self._scratch_buf(T * r * 4)
        check(self._ctx, lib.gt_rank_down(self._ctx, T, ind, r, xd, ad, 0, sc, hs), "lora.h")
        check(self._ctx, lib.gt_gemm_pair(self._ctx, NT, 0, T, outd, ind, xd, wd, r, hs, bd, e.data), "lora.y")
        wants_dw, wants_da, wants_db = w.requires_grad, a.requires_grad, b.requires_grad

        def bw():
            g = self._gsrc(out)
            dx, acc = self._gdst(x)
            if wants_dw:
                dw, accw = self._gdst(w)
                if dw:
                    check(self._ctx, lib.gt_gemm(self._ctx, TN, accw, outd, ind, T, g, xd, dw), "linear.dw")
            if wants_db:
                db, accb = self._gdst(b)
                if db:
                    self._rank_grad(b, T, outd, r, hs, g, 1, accb, db, "lora.db")
            if dx or wants_da:
                dh = self._scratch_buf(T * r * 4)
                check(self._ctx, lib.gt_rank_down(self._ctx, T, outd, r, g, bd, 1, sc, dh), "lora.dh")
                if wants_da:
                    da, acca = self._gdst(a)
                    if da:
                        self._rank_grad(a, T, ind, r, dh, xd, 0, acca, da, "lora.da")
                if dx:      # dX (+)= dY.W + dH.A in one K loop
                    check(self._ctx, lib.gt_gemm_pair(self._ctx, NN, acc, T, ind, outd, g, wd, r, dh, ad, dx), "lora.dx")

        out._backward = bw
        return out

    def add(self, a: Tensor, b: Tensor) -> Tensor:
        self._op_begin(a, b)
        p = self._pend
        lin = None
        if self.fuse_residual_add and p is not None and a is not b:
            # the linear whose launch is still held back is one of the operands and nothing else has read it: the residual
            # add of a layer, h + linear(x, W). One launch writes h + x.W^T; the product never exists on its own.
            for cand in (b, a):
                ce = self._entries.get(cand)
                if ce is not None and ce.data == p[6] and ce.consumers == 0 and not ce.external:
                    lin = cand
                    break
        if lin is not None:
            other = a if lin is b else b
            le = self._entries[lin]
            self._pend = None
            od = self._data(other)
            out, e = self._make_out(a.shape, [a, b])
            check(self._ctx, lib.gt_gemm_add(self._ctx, NT, p[1], p[2], p[3], p[4], p[5], od, e.data), "linear+add")
            le.consumers += 1
            le.lazy_lin = (p[1], p[2], p[3], p[4], p[5])
            self._recycle(le.data, le.nbytes, le.stream)
            le.data = 0
        else:
            ad, bd = self._data(a), self._data(b)
            out, e = self._make_out(a.shape, [a, b])
            check(self._ctx, lib.gt_add_fwd(self._ctx, out.size, ad, bd, e.data), "add")

        def bw():
            g = self._gsrc(out)
            if a is b:
                da, acc = self._gdst(a)
                check(self._ctx, lib.gt_add_bwd(self._ctx, out.size, g, da, acc, da, acc), "add.bwd")
                return
            todo = []
            for t in (a, b):
                te = self._entries.get(t)
                if (self.alias_add_grads and te is not None and not te.external and not te.keep_grad and not te.grad_init
                        and not te.grad_src and id(t) not in self._pend_dx):
                    te.grad_src = g             # first writer: the gradient IS the upstream one so far, nothing to launch
                    te.grad_init = True
                    self._aliased.append(t)
                else:
                    todo.append(t)
            if len(todo) == 2:
                da, acca = self._gdst(a)
                db, accb = self._gdst(b)
                check(self._ctx, lib.gt_add_bwd(self._ctx, out.size, g, da, acca, db, accb), "add.bwd")
            elif todo:
                d1, acc1 = self._gdst(todo[0])
                if d1:
                    check(self._ctx, lib.gt_scale_bwd(self._ctx, out.size, g, 1.0, d1, acc1), "add.bwd")

        out._backward = bw
        return out

    def mul(self, a: Tensor, b: Tensor) -> Tensor:
        self._op_begin(a, b)
        ea, eb = self._entry_for(a), self._entry_for(b)
        if self.fuse_glu and a is not b:
            # gate * up with a lazy activation on one side: run the fused kernels on the pre-activation
            lazy, other = (a, b) if ea.lazy_act is not None else ((b, a) if eb.lazy_act is not None else (None, None))
            if lazy is not None and self._entries[other].lazy_act is None:
                le = self._entries[lazy]
                gate, act = le.lazy_act
                le.consumers += 1
                le.fused_uses += 1
                gd, ud = self._data(gate), self._data(other)
                out, e = self._make_out(a.shape, [a, b])
                check(self._ctx, lib.gt_glu_fwd(self._ctx, act, out.size, gd, ud, e.data), "glu")

                def bw_fused():
                    g = self._gsrc(out)
                    dg, accg = self._gdst(gate)
                    du, accu = self._gdst(other)
                    check(self._ctx, lib.gt_glu_bwd(self._ctx, act, out.size, g, gd, ud, dg, accg, du, accu), "glu.bwd")

                out._backward = bw_fused
                return out
        ad, bd = self._data(a), self._data(b)
        out, e = self._make_out(a.shape, [a, b])
        check(self._ctx, lib.gt_mul_fwd(self._ctx, out.size, ad, bd, e.data), "mul")

        def bw():
            g = self._gsrc(out)
            if a is b:
                da, acc = self._gdst(a)
                check(self._ctx, lib.gt_mul_bwd(self._ctx, out.size, g, ad, ad, da, acc, da, acc), "mul.bwd")
                return
            da, acca = self._gdst(a)
            db, accb = self._gdst(b)
            check(self._ctx, lib.gt_mul_bwd(self._ctx, out.size, g, ad, bd, da, acca, db, accb), "mul.bwd")

        out._backward = bw
        return out

    def _activation(self, x: Tensor, act: int) -> Tensor:
        self._op_begin(x)
        xd = self._data(x, launch_held=not self.fuse_glu)
        out, e = self._make_out(x.shape, [x], alloc=not self.fuse_glu)
        if self.fuse_glu:
            e.lazy_act = (x, act)
        else:
            fn = lib.gt_silu_fwd if act == 0 else lib.gt_gelu_fwd
            check(self._ctx, fn(self._ctx, out.size, xd, e.data), "act")

        def bw():
            oe = self._entries.get(out)
            if oe is None:
                raise RuntimeError("backward over a graph built before a sync()")
            if oe.fused_uses and oe.fused_uses == oe.consumers:
                return                       # every use was a fused gate*up, which already wrote x's gradient
            if oe.grad == 0 and not oe.grad_src and oe.fused_uses:
                return                       # its other consumers contributed nothing
            g = self._gsrc(out)
            dx, acc = self._gdst(x)
            fn = lib.gt_silu_bwd if act == 0 else lib.gt_gelu_bwd
            check(self._ctx, fn(self._ctx, out.size, g, xd, dx, acc), "act.bwd")

        out._backward = bw
        return out

    def silu(self, x: Tensor) -> Tensor:
        return self._activation(x, 0)

    def gelu(self, x: Tensor) -> Tensor:
        return self._activation(x, 1)

    def scale(self, x: Tensor, c: float) -> Tensor:
        self._op_begin(x)
        xd = self._data(x)
        out, e = self._make_out(x.shape, [x])
        check(self._ctx, lib.gt_scale_fwd(self._ctx, out.size, xd, c, e.data), "scale")

        def bw():
            g = self._gsrc(out)
            dx, acc = self._gdst(x)
            if dx:
                check(self._ctx, lib.gt_scale_bwd(self._ctx, out.size, g, c, dx, acc), "scale.bwd")

        out._backward = bw
        return out

    def _rms_rows(self, x, weight, rows, d, eps, shape):
        self._op_begin(x, weight)
        xd, wd = self._data(x), self._data(weight)
        out, e = self._make_out(shape, [x, weight])
        rinv = self._scratch_buf(rows * 4)
        check(self._ctx, lib.gt_rmsnorm_fwd(self._ctx, rows, d, eps, xd, wd, e.data, rinv), "rmsnorm")
        wants_dw = weight.requires_grad

        def bw():
            g = self._gsrc(out)
            dx, acc, old = self._gdst_from(x)
            dw, accw = self._gdst(weight) if wants_dw else (0, 0)
            if dw and self.defer_norm_dw:
                nparts = C.c_int(0)
                check(self._ctx, lib.gt_rmsnorm_parts_rows(self._ctx, rows, d, C.byref(nparts)), "rmsnorm.bwd")
                if nparts.value > 0 and (xd | wd | g | dx | old) % 16 == 0:
                    parts = self._scratch_buf(nparts.value * d * 4)
                    check(self._ctx, lib.gt_rmsnorm_bwd_parts(self._ctx, rows, d, xd, wd, g, rinv, old, dx, 1 if old != dx else acc, parts),
                          "rmsnorm.bwd")
                    self._pend_cs.append((parts, nparts.value, d, dw, accw))
                    self._pend_cs_ids.add(id(weight))
                    return
            if old != dx:
                check(self._ctx, lib.gt_rmsnorm_bwd_from(self._ctx, rows, d, xd, wd, g, rinv, old, dx, dw, accw), "rmsnorm.bwd")
            else:
                check(self._ctx, lib.gt_rmsnorm_bwd(self._ctx, rows, d, xd, wd, g, rinv, dx, acc, dw, accw), "rmsnorm.bwd")

        out._backward = bw
        return out

    def rms_norm(self, x, weight, eps):
        T, d = x.shape
        return self._rms_rows(x, weight, T, d, eps, [T, d])

    def rms_norm_heads(self, x, weight, T, H, hd, eps):
        return self._rms_rows(x, weight, T * H, hd, eps, [T, H * hd])

    def embedding(self, weight: Tensor, ids) -> Tensor:
        self._op_begin(weight)
        V, d = weight.shape
        ids32 = np.ascontiguousarray(ids, dtype=np.int32)
        T = ids32.size
        wd = self._data(weight)
        idb = self._upload(ids32)
        out, e = self._make_out([T, d], [weight])
        check(self._ctx, lib.gt_embedding_fwd(self._ctx, T, d, V, idb, wd, e.data), "embedding")
        wants_dw = weight.requires_grad

        def bw():
            if not wants_dw:
                return
            g = self._gsrc(out)
            dw, acc = self._gdst(weight)
            check(self._ctx, lib.gt_embedding_bwd(self._ctx, T, d, V, idb, g, dw, acc), "embedding.bwd")

        out._backward = bw
        return out

    def rope(self, x, T, H, hd, base, pos_offset=0):
        self._op_begin(x)
        rows = x.shape[0]
        held, self._pend_rope = self._pend_rope, None
        xd = self._data(x)
        out, e = self._make_out([rows, H * hd], [x])
        e.rope_of = (x, (T, hd, float(base), int(pos_offset)))
        self._rope((held, ((rows, T, hd, float(base), pos_offset, 0), H, xd, e.data, 0)))

        def bw():           # the two backward rotations are never neighbours in the tape's order (k's linear sits between them)
            oe = self._entries.get(out)
            if oe is not None and oe.rope_fused:
                return      # the attention that consumed this rotation wrote x's gradient in its own write-back
            g = self._gsrc(out)
            dx, acc = self._gdst(x)
            if dx:
                check(self._ctx, lib.gt_rope(self._ctx, rows, T, H, hd, base, pos_offset, 1, g, dx, acc), "rope.bwd")

        out._backward = bw
        return out

    def attention(self, q, k, v, T, Hq, Hkv, hd, window=0):
        self._op_begin(q, k, v)
        rows = q.shape[0]
        if rows % T:
            raise ValueError(f"attention: {rows} rows are not a whole number of sequences of {T}")
        B = rows // T
        qd, kd, vd = self._data(q), self._data(k), self._data(v)
        out, e = self._make_out([rows, Hq * hd], [q, k, v])
        lse = self._scratch_buf(B * Hq * T * 4)
        scores = 0
        if self.attn_keep_scores and not self.forward_only_region and e.needs_grad:
            need = C.c_uint64(0)
            check(self._ctx, lib.gt_attn_scores_bytes(self._ctx, B, T, Hq, Hkv, hd, window, C.byref(need)), "attention")
            if 0 < need.value <= self.attn_scores_max_bytes and self._scores_taken + need.value <= self.attn_scores_budget_bytes:
                scores = self._acquire(need.value)
                e.extra = (scores, need.value)
                self._scores_taken += need.value
        if scores:
            check(self._ctx, lib.gt_attn_fwd_scores(self._ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, e.data, lse, scores), "attention")
        else:
            check(self._ctx, lib.gt_attn_fwd(self._ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, e.data, lse), "attention")
        od = e.data

        def rope_source(t):
            """t's rotation (input tensor, parameters) when its backward can ride this attention's write-backs: t is a
            rotation's output that only this attention has read and whose gradient nobody has touched."""
            te = self._entries.get(t)
            if (not self.fuse_rope_bwd or not scores or te is None or te.rope_of is None or te.consumers != 1 or te.grad_init
                    or te.grad_src or te.keep_grad or te.grad or hd % 8 or id(t) in self._pend_dx):
                return None
            src, par = te.rope_of
            if par[0] != T or par[1] != hd:
                return None
            se = self._entries.get(src)
            if se is None or (se.external and not src.requires_grad):
                return None
            return src, par

        def bw():
            g = self._gsrc(out)
            rq, rk = rope_source(q), (rope_source(k) if k is not q else None)
            if rq and rk and rq[1] != rk[1]:
                rk = None                           # two different rotations: one table per call
            if rq or rk:
                par = (rq or rk)[1]
                dq, aq = self._gdst(rq[0] if rq else q)
                dk, ak = self._gdst(rk[0] if rk else k)
                dv, av = self._gdst(v)
                if rq:
                    self._entries[q].rope_fused = True
                if rk:
                    self._entries[k].rope_fused = True
                check(self._ctx, lib.gt_attn_bwd_scores_rope(self._ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, od, g, lse, scores,
                                                             par[2], par[3], 1 if rq else 0, 1 if rk else 0,
                                                             dq, aq, dk, ak, dv, av), "attention.bwd")
                return
            dq, aq = self._gdst(q)
            dk, ak = self._gdst(k)
            dv, av = self._gdst(v)
            if scores:
                check(self._ctx, lib.gt_attn_bwd_scores(self._ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, od, g, lse, scores,
                                                        dq, aq, dk, ak, dv, av), "attention.bwd")
            else:
                check(self._ctx, lib.gt_attn_bwd(self._ctx, B, T, Hq, Hkv, hd, window, qd, kd, vd, od, g, lse,
                                                 dq, aq, dk, ak, dv, av), "attention.bwd")

        out._backward = bw
        return out

    @staticmethod
    def _inv_denoms(kept):
        kept = np.atleast_1d(np.asarray(kept, dtype=np.int64))
        return (1.0 / np.maximum(kept, 1)).astype(np.float32)

    def cross_entropy(self, logits, targets, kept) -> Tensor:
        self._op_begin(logits)
        rows, V = logits.shape
        inv = self._inv_denoms(kept)
        nseq = inv.size
        T = rows // nseq
        zd = self._data(logits)
        tg = self._upload(np.ascontiguousarray(targets, dtype=np.int32))
        invb = self._upload(inv)
        lse = self._scratch_buf(rows * 4)
        loss, e = self._make_out([nseq], [logits])
        check(self._ctx, lib.gt_ce_fwd(self._ctx, rows, V, T, zd, tg, invb, e.data, lse), "crossEntropy")

        def bw():
            if self._entries.get(loss) is None:
                raise RuntimeError("backward over a graph built before a sync()")
            seed = float(loss.grad[0])
            dz, acc = self._gdst(logits)
            check(self._ctx, lib.gt_ce_bwd(self._ctx, rows, V, T, zd, tg, invb, lse, seed, dz, acc), "crossEntropy.bwd")

        loss._backward = bw
        return loss

    def fused_cross_entropy(self, hidden, w, targets, chunk, kept) -> Tensor:
        self._op_begin(hidden, w)
        rows, H = hidden.shape
        V = w.shape[0]
        inv = self._inv_denoms(kept)
        nseq = inv.size
        T = rows // nseq
        hd_, wd = self._data(hidden), self._data(w)
        tg = self._upload(np.ascontiguousarray(targets, dtype=np.int32))
        invb = self._upload(inv)
        rmax, rsum, tl = (self._scratch_buf(rows * 4) for _ in range(3))
        width = min(chunk, V)
        cb = self._scratch_buf(rows * width * 4)
        spans = [(v0, min(v0 + chunk, V) - v0) for v0 in range(0, V, chunk)]
        for i, (v0, vc) in enumerate(spans):
            check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, rows, vc, H, hd_, wd + v0 * H * 4, cb), "fusedCE.logits")
            check(self._ctx, lib.gt_ce_chunk_stats(self._ctx, rows, V, vc, v0, 1 if i == 0 else 0, cb, tg, rmax, rsum, tl), "fusedCE.stats")
        loss, e = self._make_out([nseq], [hidden, w])
        check(self._ctx, lib.gt_ce_loss_from_stats(self._ctx, rows, V, T, tg, invb, rmax, rsum, tl, e.data), "fusedCE.loss")
        wants_dw = w.requires_grad

        def bw():
            if self._entries.get(loss) is None:
                raise RuntimeError("backward over a graph built before a sync()")
            seed = float(loss.grad[0])
            dh, acch = self._gdst(hidden)
            dw, accw = self._gdst(w) if wants_dw else (0, 0)
            for v0, vc in spans:
                check(self._ctx, lib.gt_gemm(self._ctx, NT, 0, rows, vc, H, hd_, wd + v0 * H * 4, cb), "fusedCE.logits")
                check(self._ctx, lib.gt_ce_chunk_grad(self._ctx, rows, V, vc, v0, T, cb, tg, invb, rmax, rsum, seed), "fusedCE.grad")
                check(self._ctx, lib.gt_gemm(self._ctx, NN, acch, rows, H, vc, cb, wd + v0 * H * 4, dh), "fusedCE.dh")
                acch = 1
                if dw:
                    # rows [v0, v0+vc) of dW are written by this span only
                    check(self._ctx, lib.gt_gemm(self._ctx, TN, accw, vc, H, rows, cb, hd_, dw + v0 * H * 4), "fusedCE.dw")

        loss._backward = bw
        return loss

    def soft_cross_entropy(self, logits, teacher_ids, teacher_probs, k, kept) -> Tensor:
        self._op_begin(logits)
        rows, V = logits.shape
        inv = 1.0 / max(int(kept), 1)
        zd = self._data(logits)
        ti = self._upload(np.ascontiguousarray(teacher_ids, dtype=np.int32))
        tp = self._upload(np.ascontiguousarray(teacher_probs, dtype=np.float32))
        lse, mass = self._scratch_buf(rows * 4), self._scratch_buf(rows * 4)
        loss, e = self._make_out([1], [logits])
        check(self._ctx, lib.gt_soft_ce_fwd(self._ctx, rows, V, k, zd, ti, tp, inv, e.data, lse, mass), "softCE")

        def bw():
            if self._entries.get(loss) is None:
                raise RuntimeError("backward over a graph built before a sync()")
            seed = float(loss.grad[0])
            dz, acc = self._gdst(logits)
            check(self._ctx, lib.gt_soft_ce_bwd(self._ctx, rows, V, k, zd, ti, tp, inv, lse, mass, seed, dz, acc), "softCE.bwd")

        loss._backward = bw
        return loss

    # ---- raw GEMM for tests and benches (webgpu.ts:1654) --------------------------------------------------------------
    def gemm(self, kind: int, acc: int, M: int, N: int, K: int, a: int, b: int, c: int):
        self._join()
        check(self._ctx, lib.gt_gemm(self._ctx, kind, acc, M, N, K, a, b, c), "gemm")


def init_hip(device: int = 0, streams: int = 4):
    """initWebGPU analogue (webgpu.ts:1823): a backend, or None when no MI355X is visible."""
    try:
        return HipBackend(device, streams)
    except HipError:
        return None


def require_gpu(purpose: str, device: int = 0, streams: int = 4, bf16_pieces: bool = False) -> HipBackend:
    """requireGPU analogue (webgpu.ts:1812). bf16_pieces: run the FP32 products and the attention kernels that have such a form on
    the bf16 matrix instruction (library options "gemm.split_bf16" and "attn.split_bf16": each FP32 element as three exact bf16
    pieces, FP32 accumulation; as close to float64 as the FP32 MFMA kernels, about 1.3 x faster steps, not bit-identical to them)."""
    try:
        gpu = HipBackend(device, streams)
        if bf16_pieces:
            gpu.set_option("gemm.split_bf16", 1)
            gpu.set_option("attn.split_bf16", 1)
        return gpu
    except HipError as e:
        raise RuntimeError(f"{purpose} needs an MI355X: {e}") from e
