"""Device-resident optimizers: AdamWHip and MuonHip, mirrors of AdamWGpu
(src/backend/adamw-gpu.ts:131-251) and MuonGpu (src/backend/muon-gpu.ts:351-470).

Weights, gradients, moments and momentum stay on the device; record_step() only enqueues work.
The .optstate sidecar layout of muon-gpu.ts:293-349 is kept: "OPT1" magic, adamT, three length
lists, then f32 blobs in the order muonMomentum, adamM, adamV.
"""
from __future__ import annotations

import ctypes as C
import struct

import numpy as np

from .lib import buf as c_buf, check, lib


def _bufs(vals):
    return (c_buf * len(vals))(*vals)


class AdamWHip:
    def __init__(self, gpu, params, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, clip=1.0):
        self.gpu = gpu
        self.params = list(params)
        self.base_lr = lr
        self.lr_scale = 1.0
        self.beta1, self.beta2, self.eps, self.weight_decay, self.clip = beta1, beta2, eps, weight_decay, clip
        self.t = 0
        self._m, self._v = [], []
        w, g = [], []
        for p in self.params:
            b = gpu.buffers_for(p)          # uploads host weights once; accumulator on the device
            gpu.keep_grad_on_device(p)
            w.append(b["data"])
            g.append(b["grad"])
            self._m.append(gpu.create_state_buffer(p.size * 4))
            self._v.append(gpu.create_state_buffer(p.size * 4))
        self._h = C.c_void_p()
        n = len(self.params)
        sizes = (C.c_int64 * max(1, n))(*[p.size for p in self.params])
        check(gpu.ctx, lib.gt_adamw_create(gpu.ctx, n, _bufs(w), _bufs(g), _bufs(self._m), _bufs(self._v), sizes,
                                           beta1, beta2, eps, weight_decay, clip, C.byref(self._h)), "gt_adamw_create")

    def set_lr_scale(self, s: float):
        self.lr_scale = s

    def destroy(self):
        """Release the device-side tables; the moment buffers go back with the backend's state buffers."""
        if self.gpu._destroyed:             # the library context is gone and took the tables and the buffers with it
            self._h, self._m, self._v = C.c_void_p(), [], []
            return
        if self._h:
            check(self.gpu.ctx, lib.gt_adamw_destroy(self.gpu.ctx, self._h), "gt_adamw_destroy")
            self._h = C.c_void_p()
        for b in self._m + self._v:
            self.gpu.free_state_buffer(b)
        self._m, self._v = [], []

    def zero_grad(self):
        """No-op: accumulators live on the device and are re-armed when a step has consumed them."""

    def record_step(self):
        self.t += 1
        bc1 = 1 - self.beta1 ** self.t
        bc2 = 1 - self.beta2 ** self.t
        self.gpu.ensure_grads_defined(self.params)
        check(self.gpu.ctx, lib.gt_adamw_step(self.gpu.ctx, self._h, self.base_lr * self.lr_scale, bc1, bc2), "gt_adamw_step")
        self.gpu.grads_consumed(self.params)

    def grad_norm(self) -> float:
        v = C.c_float()
        check(self.gpu.ctx, lib.gt_adamw_grad_norm(self.gpu.ctx, self._h, C.byref(v)), "gt_adamw_grad_norm")
        return float(v.value)

    def sync_weights_to_host(self):
        for p in self.params:
            p.data[:] = self.gpu.read_state_buffer(self.gpu.buffers_for(p)["data"], p.size)

    def export_state(self):
        return {"m": [self.gpu.read_state_buffer(b, p.size) for b, p in zip(self._m, self.params)],
                "v": [self.gpu.read_state_buffer(b, p.size) for b, p in zip(self._v, self.params)], "t": self.t}

    def import_state(self, s):
        if len(s["m"]) != len(self.params) or len(s["v"]) != len(self.params):
            raise ValueError(f"adam state count mismatch: {len(s['m'])}/{len(s['v'])} vs {len(self.params)}")
        for b, a in zip(self._m, s["m"]):
            self.gpu.write_state_buffer(b, np.asarray(a, dtype=np.float32))
        for b, a in zip(self._v, s["v"]):
            self.gpu.write_state_buffer(b, np.asarray(a, dtype=np.float32))
        self.t = int(s["t"])


class MuonHip:
    def __init__(self, gpu, muon_params, aux_params, lr, momentum=0.95, nesterov=True, ns_steps=5, aux=None):
        self.gpu = gpu
        self.muon_params = list(muon_params)
        self.aux_params = list(aux_params)
        self.aux = AdamWHip(gpu, self.aux_params, **(aux or {"lr": lr}))
        self.base_lr = lr
        self.lr = lr
        self._bufs = []
        w, g, rows, cols = [], [], [], []
        for p in self.muon_params:
            if len(p.shape) != 2:
                raise ValueError("Muon param must be 2-D")
            b = gpu.buffers_for(p)
            gpu.keep_grad_on_device(p)
            w.append(b["data"])
            g.append(b["grad"])
            rows.append(p.shape[0])
            cols.append(p.shape[1])
            self._bufs.append(gpu.create_state_buffer(p.size * 4))
        n = len(self.muon_params)
        self._h = C.c_void_p()
        check(gpu.ctx, lib.gt_muon_create(gpu.ctx, n, _bufs(w), _bufs(g), _bufs(self._bufs),
                                          (C.c_int * max(1, n))(*rows), (C.c_int * max(1, n))(*cols),
                                          momentum, 1 if nesterov else 0, ns_steps, C.byref(self._h)), "gt_muon_create")

    def set_lr_scale(self, s: float):
        self.lr = self.base_lr * s
        self.aux.set_lr_scale(s)

    def destroy(self):
        """Release the per-shape work buffers and pointer tables, the momentum buffers and the auxiliary AdamW."""
        if self.gpu._destroyed:
            self._h, self._bufs = C.c_void_p(), []
            self.aux.destroy()
            return
        if self._h:
            check(self.gpu.ctx, lib.gt_muon_destroy(self.gpu.ctx, self._h), "gt_muon_destroy")
            self._h = C.c_void_p()
        for b in self._bufs:
            self.gpu.free_state_buffer(b)
        self._bufs = []
        self.aux.destroy()

    def zero_grad(self):
        self.aux.zero_grad()

    def record_step(self):
        if self.muon_params:
            self.gpu.ensure_grads_defined(self.muon_params)
            check(self.gpu.ctx, lib.gt_muon_step(self.gpu.ctx, self._h, self.lr), "gt_muon_step")
            self.gpu.grads_consumed(self.muon_params)
        self.aux.record_step()

    def sync_weights_to_host(self):
        for p in self.muon_params:
            p.data[:] = self.gpu.read_state_buffer(self.gpu.buffers_for(p)["data"], p.size)
        self.aux.sync_weights_to_host()

    def export_state(self):
        a = self.aux.export_state()
        return {"muonMomentum": [self.gpu.read_state_buffer(b, p.size) for b, p in zip(self._bufs, self.muon_params)],
                "adamM": a["m"], "adamV": a["v"], "adamT": a["t"]}

    def import_state(self, s):
        if len(s["muonMomentum"]) != len(self._bufs):
            raise ValueError(f"muon momentum count mismatch: {len(s['muonMomentum'])} vs {len(self._bufs)}")
        for b, a in zip(self._bufs, s["muonMomentum"]):
            self.gpu.write_state_buffer(b, np.asarray(a, dtype=np.float32))
        self.aux.import_state({"m": s["adamM"], "v": s["adamV"], "t": s["adamT"]})


OPT_MAGIC = 0x4F505431  # "OPT1"


def serialize_opt_state(s) -> bytes:
    """muon-gpu.ts:297-323: u32 magic, u32 adamT, then per group (muonMomentum, adamM, adamV) a u32 count
    followed by that many u32 lengths, then every f32 blob in the same order. Little-endian."""
    groups = [s["muonMomentum"], s["adamM"], s["adamV"]]
    head = struct.pack("<II", OPT_MAGIC, int(s["adamT"]))
    for g in groups:
        head += struct.pack("<I", len(g)) + b"".join(struct.pack("<I", int(np.asarray(a).size)) for a in g)
    blobs = b"".join(np.ascontiguousarray(a, dtype="<f4").tobytes() for g in groups for a in g)
    return head + blobs


def deserialize_opt_state(raw: bytes):
    """muon-gpu.ts:326-349."""
    magic, t = struct.unpack_from("<II", raw, 0)
    if magic != OPT_MAGIC:
        raise ValueError("bad optstate magic")
    off = 8
    all_lens = []
    for _ in range(3):
        (count,) = struct.unpack_from("<I", raw, off)
        off += 4
        all_lens.append(list(struct.unpack_from(f"<{count}I", raw, off)))
        off += 4 * count
    out = []
    for lens in all_lens:
        g = []
        for n in lens:
            g.append(np.frombuffer(raw, dtype="<f4", count=n, offset=off).copy())
            off += 4 * n
        out.append(g)
    return {"muonMomentum": out[0], "adamM": out[1], "adamV": out[2], "adamT": t}
