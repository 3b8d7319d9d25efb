"""CPU oracle, Python side: the reference's tape, op wrappers, model graphs, optimizers
and CPU training loop, restated over the C loops in oracle.c.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, always as the checker and never as a computation the
product ships. The product package never imports this module.

Reference files followed (path:line in felladrin/gguf-trainer):
  src/model/autograd.ts:20-93     Tensor, backward (topological walk, seed)
  src/model/autograd.ts:234-273   checkpoint (replay in backward)
  src/model/autograd.ts:311-319   LoRA-aware linear
  src/model/autograd.ts:382-1138  op set (the loops themselves are in oracle.c)
  src/arch/llama.ts:183-221, src/arch/qwen3.ts:153-195, src/arch/gemma3.ts:173-223  graphs
  src/train/adam.ts:46-82, src/train/muon.ts:69-158, src/train/trainer.ts:51-87
  src/train/schedule.ts, src/train/qk-clip.ts, src/train/lora.ts:46-108
"""
from __future__ import annotations

import ctypes as C
import math
import os
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def _load():
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(f"{_LIB_PATH} is not built: run `make -C oracle` (or __graft_entry__.build())")
    return C.CDLL(_LIB_PATH)


_lib = _load()
_F = C.POINTER(C.c_float)
_I = C.POINTER(C.c_int32)
_Dp = C.POINTER(C.c_double)


def _f(a):
    return None if a is None else a.ctypes.data_as(_F)


def _i(a):
    return a.ctypes.data_as(_I)


_lib.or_mulberry32_next.restype = C.c_double
_lib.or_randn.restype = C.c_double
_lib.or_ce_fwd.restype = C.c_double
_lib.or_fused_ce_fwd.restype = C.c_double
_lib.or_soft_ce_fwd.restype = C.c_double


# Timed CPU baseline only: route linear / attention backward through the OpenMP-safe variants in oracle.c
# (per-output f64 dot products, rounded once). Parity tests leave this False and use the literal loops.
PARALLEL_BWD = False


def set_threads(n: int) -> None:
    _lib.or_set_threads(int(n))


def max_threads() -> int:
    return int(_lib.or_max_threads())


# ---- seeded inputs (autograd.ts:54-78) ---------------------------------------------

class Mulberry32:
    """mulberry32(seed); call it for the next uniform in [0,1)."""

    def __init__(self, seed: int):
        self.state = C.c_uint32(seed & 0xFFFFFFFF)

    def __call__(self) -> float:
        return _lib.or_mulberry32_next(C.byref(self.state))

    def randn(self) -> float:
        return _lib.or_randn(C.byref(self.state))

    def fill_randn(self, shape, std=1.0) -> np.ndarray:
        out = np.empty(shape, dtype=np.float32)
        _lib.or_fill_randn(_f(out), C.c_int64(out.size), C.c_double(std), C.byref(self.state))
        return out

    def fill_uniform(self, shape, lo=-1.0, hi=1.0) -> np.ndarray:
        out = np.empty(shape, dtype=np.float32)
        _lib.or_fill_uniform(_f(out), C.c_int64(out.size), C.c_double(lo), C.c_double(hi), C.byref(self.state))
        return out


# ---- Tensor and tape (autograd.ts:20-93) -------------------------------------------

_created = 0


class Tensor:
    def __init__(self, data: np.ndarray, shape=None, requires_grad=False):
        global _created
        data = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        self.shape = list(shape if shape is not None else data.shape)
        if data.size != int(np.prod(self.shape)):
            raise ValueError(f"data length {data.size} != shape {self.shape}")
        self.data = data
        self.grad = np.zeros_like(data)
        self.requires_grad = requires_grad
        self._backward = lambda: None
        self._prev: list[Tensor] = []
        self.seq = _created
        _created += 1

    @staticmethod
    def zeros(shape, requires_grad=False):
        return Tensor(np.zeros(int(np.prod(shape)), dtype=np.float32), shape, requires_grad)

    def zero_grad(self):
        self.grad.fill(0)

    @property
    def size(self):
        return self.data.size


def param(shape, std, rng: Mulberry32) -> Tensor:
    return Tensor(rng.fill_randn(shape, std), shape, True)


def ones(shape) -> Tensor:
    return Tensor(np.ones(int(np.prod(shape)), dtype=np.float32), shape, True)


def _topo(root: Tensor, seen: set):
    """Post-order DFS, iterative (the reference recurses; same order)."""
    topo = []
    stack = [(root, 0)]
    if id(root) in seen:
        return topo
    seen.add(id(root))
    while stack:
        t, i = stack.pop()
        if i < len(t._prev):
            stack.append((t, i + 1))
            p = t._prev[i]
            if id(p) not in seen:
                seen.add(id(p))
                stack.append((p, 0))
        else:
            topo.append(t)
    return topo


def backward(loss: Tensor, seed=1.0):
    topo = _topo(loss, set())
    loss.grad[0] = seed
    for t in reversed(topo):
        t._backward()


def backward_from(out: Tensor, grad_out: np.ndarray):
    """tests/gradcheck.ts:61-73: seed a full gradient on a non-scalar output."""
    topo = _topo(out, set())
    out.grad[:] = np.asarray(grad_out, dtype=np.float32).reshape(-1)
    for t in reversed(topo):
        t._backward()


_checkpointing = False


def set_checkpointing(on: bool):
    global _checkpointing
    _checkpointing = on


def _assert_self_contained(out, inputs, born):
    """src/model/autograd.ts:198-215: the block may read its declared inputs and leaves (parameters); a computed tensor
    built before the block began would have its backward run once per block."""
    seen = {id(t) for t in inputs}
    if id(out) in seen:
        raise ValueError("checkpoint: fn returned one of its inputs; there is nothing to recompute")
    stack = [out]
    while stack:
        t = stack.pop()
        if id(t) in seen:
            continue
        seen.add(id(t))
        if t._prev and t.seq < born:
            raise ValueError("checkpoint: the block reads a computed tensor it did not create. "
                             "Pass it in `inputs`, or move its computation inside the block.")
        stack.extend(t._prev)


def checkpoint(inputs, fn):
    """src/model/autograd.ts:234-273."""
    if not _checkpointing:
        return fn()
    born = _created
    out = fn()
    _assert_self_contained(out, inputs, born)
    out._prev = list(inputs)

    def bw():
        replay = fn()
        replay.grad[:] = out.grad
        topo = _topo(replay, {id(t) for t in inputs})
        for t in reversed(topo):
            t._backward()

    out._backward = bw
    return out


# ---- LoRA-aware linear (autograd.ts:290-319) ------------------------------------------

_lora: dict[int, tuple] = {}


def set_lora_adapters(m: dict):
    """m maps id(weight tensor) -> (a, b, scale); None or {} removes every adapter."""
    global _lora
    _lora = m or {}


def linear(x: Tensor, w: Tensor) -> Tensor:
    if _lora:
        ad = _lora.get(id(w))
        if ad is not None:
            a, b, sc = ad
            return add(linear_raw(x, w), scale(linear_raw(linear_raw(x, a), b), sc))
    return linear_raw(x, w)


def linear_raw(x: Tensor, w: Tensor) -> Tensor:
    T, ind = x.shape
    outd, ind2 = w.shape
    if ind != ind2:
        raise ValueError(f"linear dim mismatch: x is {x.shape} and w is {w.shape}")
    out = Tensor.zeros([T, outd])
    _lib.or_linear_fwd(_f(x.data), _f(w.data), _f(out.data), T, ind, outd)
    out._prev = [x, w]
    wants_dw = w.requires_grad

    def bw():
        fn = _lib.or_linear_bwd_dots if PARALLEL_BWD else _lib.or_linear_bwd
        fn(_f(x.data), _f(w.data), _f(out.grad), _f(x.grad), _f(w.grad) if wants_dw else None, T, ind, outd)

    out._backward = bw
    return out


def add(a: Tensor, b: Tensor) -> Tensor:
    out = Tensor.zeros(a.shape)
    _lib.or_add_fwd(_f(a.data), _f(b.data), _f(out.data), C.c_int64(out.size))
    out._prev = [a, b]
    out._backward = lambda: _lib.or_add_bwd(_f(out.grad), _f(a.grad), _f(b.grad), C.c_int64(out.size))
    return out


def mul(a: Tensor, b: Tensor) -> Tensor:
    out = Tensor.zeros(a.shape)
    _lib.or_mul_fwd(_f(a.data), _f(b.data), _f(out.data), C.c_int64(out.size))
    out._prev = [a, b]
    out._backward = lambda: _lib.or_mul_bwd(_f(a.data), _f(b.data), _f(out.grad), _f(a.grad), _f(b.grad),
                                            C.c_int64(out.size))
    return out


def silu(x: Tensor) -> Tensor:
    out = Tensor.zeros(x.shape)
    sig = np.empty_like(x.data)
    _lib.or_silu_fwd(_f(x.data), _f(out.data), _f(sig), C.c_int64(x.size))
    out._prev = [x]
    out._backward = lambda: _lib.or_silu_bwd(_f(x.data), _f(sig), _f(out.grad), _f(x.grad), C.c_int64(x.size))
    return out


def gelu(x: Tensor) -> Tensor:
    out = Tensor.zeros(x.shape)
    _lib.or_gelu_fwd(_f(x.data), _f(out.data), C.c_int64(x.size))
    out._prev = [x]
    out._backward = lambda: _lib.or_gelu_bwd(_f(x.data), _f(out.grad), _f(x.grad), C.c_int64(x.size))
    return out


def scale(x: Tensor, c: float) -> Tensor:
    out = Tensor.zeros(x.shape)
    _lib.or_scale_fwd(_f(x.data), _f(out.data), C.c_double(c), C.c_int64(x.size))
    out._prev = [x]
    out._backward = lambda: _lib.or_scale_bwd(_f(out.grad), _f(x.grad), C.c_double(c), C.c_int64(x.size))
    return out


def _rms(x: Tensor, weight: Tensor, rows: int, d: int, eps: float, shape) -> Tensor:
    out = Tensor.zeros(shape)
    rinv = np.empty(rows, dtype=np.float32)
    _lib.or_rmsnorm_fwd(_f(x.data), _f(weight.data), _f(out.data), _f(rinv), rows, d, C.c_double(eps))
    out._prev = [x, weight]
    wants_dw = weight.requires_grad
    out.rinv = rinv

    def bw():
        _lib.or_rmsnorm_bwd(_f(x.data), _f(weight.data), _f(rinv), _f(out.grad), _f(x.grad),
                            _f(weight.grad) if wants_dw else None, rows, d)

    out._backward = bw
    return out


def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    T, d = x.shape
    return _rms(x, weight, T, d, eps, [T, d])


def rms_norm_heads(x: Tensor, weight: Tensor, T: int, H: int, hd: int, eps: float) -> Tensor:
    return _rms(x, weight, T * H, hd, eps, [T, H * hd])


def embedding(weight: Tensor, ids) -> Tensor:
    V, d = weight.shape
    ids32 = np.ascontiguousarray(ids, dtype=np.int32)
    if ids32.size and (ids32.min() < 0 or ids32.max() >= V):
        raise ValueError("embedding: id out of range")
    T = ids32.size
    out = Tensor.zeros([T, d])
    _lib.or_embedding_fwd(_f(weight.data), _i(ids32), _f(out.data), T, d)
    out._prev = [weight]
    wants_dw = weight.requires_grad
    out._backward = lambda: _lib.or_embedding_bwd(_i(ids32), _f(out.grad), _f(weight.grad) if wants_dw else None, T, d)
    return out


def rope(x: Tensor, T: int, H: int, hd: int, base: float, pos_offset: int = 0) -> Tensor:
    out = Tensor.zeros([T, H * hd])
    _lib.or_rope_fwd(_f(x.data), _f(out.data), T, H, hd, C.c_double(base), pos_offset)
    out._prev = [x]
    out._backward = lambda: _lib.or_rope_bwd(_f(out.grad), _f(x.grad), T, H, hd, C.c_double(base), pos_offset)
    return out


def attention(q: Tensor, k: Tensor, v: Tensor, T: int, Hq: int, Hkv: int, hd: int, window: int = 0,
              parallel_bwd: bool = False) -> Tensor:
    out = Tensor.zeros([T, Hq * hd])
    probs = np.zeros((Hq, T, T), dtype=np.float32)
    _lib.or_attention_fwd(_f(q.data), _f(k.data), _f(v.data), _f(out.data), _f(probs), T, Hq, Hkv, hd, window)
    out._prev = [q, k, v]
    out.probs = probs
    def bw():
        fn = _lib.or_attention_bwd_par if (parallel_bwd or PARALLEL_BWD) else _lib.or_attention_bwd
        fn(_f(q.data), _f(k.data), _f(v.data), _f(probs), _f(out.grad), _f(q.grad), _f(k.grad), _f(v.grad),
           T, Hq, Hkv, hd, window)

    out._backward = bw
    return out


def kept_rows_in_vocab(targets, T: int, V: int, where: str) -> int:
    """autograd.ts:875-894."""
    if len(targets) != T:
        raise ValueError(f"{where}: {len(targets)} targets for {T} logit rows")
    kept = 0
    for t, g in enumerate(targets):
        if int(g) != g or g < -1 or g >= V:
            raise ValueError(f"{where}: target {g} at position {t} is not -1 (ignore) or an integer in [0,{V})")
        if g >= 0:
            kept += 1
    return kept


def cross_entropy(logits: Tensor, targets) -> Tensor:
    T, V = logits.shape
    kept = kept_rows_in_vocab(targets, T, V, "crossEntropy")
    tg = np.ascontiguousarray(targets, dtype=np.int32)
    loss = Tensor.zeros([1])
    probs = np.empty(T * V, dtype=np.float32)
    loss.data[0] = _lib.or_ce_fwd(_f(logits.data), _i(tg), _f(probs), T, V, kept)
    loss._prev = [logits]
    loss._backward = lambda: _lib.or_ce_bwd(_f(probs), _i(tg), C.c_float(loss.grad[0]), _f(logits.grad), T, V, kept)
    return loss


def fused_cross_entropy(hidden: Tensor, w: Tensor, targets, chunk: int) -> Tensor:
    T, H = hidden.shape
    V, H2 = w.shape
    if H != H2:
        raise ValueError(f"fusedCrossEntropy dim mismatch {H} vs {H2}")
    if chunk <= 0:
        raise ValueError(f"fusedCrossEntropy chunk must be positive, got {chunk}")
    if id(w) in _lora:
        raise ValueError("fusedCrossEntropy: the readout weight carries a LoRA adapter")
    kept = kept_rows_in_vocab(targets, T, V, "fusedCrossEntropy")
    tg = np.ascontiguousarray(targets, dtype=np.int32)
    loss = Tensor.zeros([1])
    rmax = np.empty(T, dtype=np.float32)
    rsum = np.empty(T, dtype=np.float32)
    loss.data[0] = _lib.or_fused_ce_fwd(_f(hidden.data), _f(w.data), _i(tg), chunk, _f(rmax), _f(rsum), T, H, V, kept)
    loss._prev = [hidden, w]
    wants_dw = w.requires_grad
    loss._backward = lambda: _lib.or_fused_ce_bwd(
        _f(hidden.data), _f(w.data), _i(tg), chunk, _f(rmax), _f(rsum), C.c_float(loss.grad[0]),
        _f(hidden.grad), _f(w.grad) if wants_dw else None, T, H, V, kept)
    return loss


def kept_teacher_rows(tids, tprobs, T, k, V) -> int:
    """autograd.ts:760-791."""
    if k < 1:
        raise ValueError(f"softCrossEntropy: k must be >= 1, got {k}")
    if len(tids) != T * k or len(tprobs) != T * k:
        raise ValueError(f"softCrossEntropy: teacher arrays must be [T*k]={T * k}")
    kept = 0
    for t in range(T):
        if tids[t * k] == -1:
            continue
        for j in range(k):
            i = tids[t * k + j]
            if int(i) != i or i < 0 or i >= V:
                raise ValueError(f"softCrossEntropy: teacher id {i} at slot {j} of row {t} is not an integer in [0,{V})")
        kept += 1
    return kept


def soft_cross_entropy(logits: Tensor, teacher_ids, teacher_probs, k: int) -> Tensor:
    T, V = logits.shape
    kept = kept_teacher_rows(teacher_ids, teacher_probs, T, k, V)
    ti = np.ascontiguousarray(teacher_ids, dtype=np.int32)
    tp = np.ascontiguousarray(teacher_probs, dtype=np.float64)
    loss = Tensor.zeros([1])
    probs = np.empty(T * V, dtype=np.float32)
    mass = np.zeros(T, dtype=np.float32)
    loss.data[0] = _lib.or_soft_ce_fwd(_f(logits.data), _i(ti), tp.ctypes.data_as(_Dp), k, _f(probs), _f(mass), T, V, kept)
    loss._prev = [logits]
    loss._backward = lambda: _lib.or_soft_ce_bwd(_f(probs), _f(mass), _i(ti), tp.ctypes.data_as(_Dp), k,
                                                 C.c_float(loss.grad[0]), _f(logits.grad), T, V, kept)
    return loss


# ---- model graphs (arch/llama.ts, qwen3.ts, gemma3.ts) ----------------------------------

@dataclass
class ModelConfig:
    arch: str                 # "llama" | "qwen3" | "gemma3"
    vocab: int
    hidden: int
    layers: int
    heads: int
    kv_heads: int
    head_dim: int
    ffn: int
    rope_base: float = 10000.0
    rms_eps: float = 1e-5
    tie: bool = True
    # gemma3 only
    sliding_window: int = 0
    swa_pattern: int = 0
    rope_base_local: float = 10000.0


LAYER_KEYS = {
    "llama": ["attnNorm", "qProj", "kProj", "vProj", "oProj", "ffnNorm", "gate", "up", "down"],
    "qwen3": ["attnNorm", "qProj", "kProj", "vProj", "oProj", "qNorm", "kNorm", "ffnNorm", "gate", "up", "down"],
    "gemma3": ["attnNorm", "qProj", "kProj", "vProj", "oProj", "qNorm", "kNorm", "postAttnNorm", "ffnNorm",
               "gate", "up", "down", "postFfnNorm"],
}
MATRIX_KEYS = ("qProj", "kProj", "vProj", "oProj", "gate", "up", "down")


def layer_shapes(c: ModelConfig) -> dict:
    h, qd, kvd = c.hidden, c.heads * c.head_dim, c.kv_heads * c.head_dim
    s = {"attnNorm": [h], "qProj": [qd, h], "kProj": [kvd, h], "vProj": [kvd, h], "oProj": [h, qd],
         "qNorm": [c.head_dim], "kNorm": [c.head_dim], "postAttnNorm": [h], "ffnNorm": [h],
         "gate": [c.ffn, h], "up": [c.ffn, h], "down": [h, c.ffn], "postFfnNorm": [h]}
    return {k: s[k] for k in LAYER_KEYS[c.arch]}


def is_global_layer(c: ModelConfig, il: int) -> bool:
    return c.swa_pattern > 0 and il % c.swa_pattern == c.swa_pattern - 1


class Model:
    """Parameter order and graph of the reference's LlamaModel / Qwen3Model / Gemma3Model.

    `weights`, when given, is a dict name -> np.float32 array (names: tokenEmbd, outputNorm,
    output, L{i}.{key}); otherwise matrices draw N(0, std) from rng in the constructor's order and
    norm gains are ones.
    """

    def __init__(self, cfg: ModelConfig, rng: Mulberry32 | None = None, std: float | None = None, weights=None):
        self.cfg = c = cfg

        def mk(name, shape, default_std):
            if weights is not None:
                return Tensor(np.array(weights[name], dtype=np.float32), shape, True)
            if len(shape) == 1:
                return ones(shape)
            return param(shape, default_std if std is None else std, rng)

        self.tokenEmbd = mk("tokenEmbd", [c.vocab, c.hidden], 0.02)
        self.outputNorm = mk("outputNorm", [c.hidden], 0)
        self.output = None if c.tie else mk("output", [c.vocab, c.hidden], 0.02)
        self.layers = []
        for l in range(c.layers):
            L = {}
            for k, shp in layer_shapes(c).items():
                L[k] = mk(f"L{l}.{k}", shp, 1 / math.sqrt(shp[-1]) if len(shp) == 2 else 0)
            self.layers.append(L)

    def named_params(self):
        out = [("tokenEmbd", self.tokenEmbd), ("outputNorm", self.outputNorm)]
        if self.output is not None:
            out.append(("output", self.output))
        for l, L in enumerate(self.layers):
            out += [(f"L{l}.{k}", L[k]) for k in LAYER_KEYS[self.cfg.arch]]
        return out

    def params(self):
        return [p for _, p in self.named_params()]

    def param_groups(self):
        muon, aux = [], [self.tokenEmbd, self.outputNorm]
        if self.output is not None:
            aux.append(self.output)
        for L in self.layers:
            muon += [L[k] for k in MATRIX_KEYS]
            aux += [L[k] for k in LAYER_KEYS[self.cfg.arch] if k not in MATRIX_KEYS]
        return muon, aux

    def qk_norms(self):
        return [(L["qNorm"], L["kNorm"]) for L in self.layers if "qNorm" in L]

    def forward_to_readout(self, ids):
        c = self.cfg
        T = len(ids)
        h = embedding(self.tokenEmbd, ids)
        if c.arch == "gemma3":
            h = scale(h, math.sqrt(c.hidden))
        for il, L in enumerate(self.layers):
            h = checkpoint([h], self._block(h, L, il, T))
        return rms_norm(h, self.outputNorm, c.rms_eps), (self.output if self.output is not None else self.tokenEmbd)

    def _block(self, h_in, L, il, T):
        c = self.cfg

        def fn():
            h = h_in
            window, rope_b = 0, c.rope_base
            if c.arch == "gemma3":
                glob = is_global_layer(c, il)
                window = 0 if glob else c.sliding_window
                rope_b = c.rope_base if glob else c.rope_base_local
            n1 = rms_norm(h, L["attnNorm"], c.rms_eps)
            q = linear(n1, L["qProj"])
            k = linear(n1, L["kProj"])
            v = linear(n1, L["vProj"])
            if c.arch in ("qwen3", "gemma3"):
                q = rms_norm_heads(q, L["qNorm"], T, c.heads, c.head_dim, c.rms_eps)
                k = rms_norm_heads(k, L["kNorm"], T, c.kv_heads, c.head_dim, c.rms_eps)
            q = rope(q, T, c.heads, c.head_dim, rope_b)
            k = rope(k, T, c.kv_heads, c.head_dim, rope_b)
            a = attention(q, k, v, T, c.heads, c.kv_heads, c.head_dim, window)
            attn_out = linear(a, L["oProj"])
            if c.arch == "gemma3":
                attn_out = rms_norm(attn_out, L["postAttnNorm"], c.rms_eps)
            h = add(h, attn_out)
            n2 = rms_norm(h, L["ffnNorm"], c.rms_eps)
            g = (gelu if c.arch == "gemma3" else silu)(linear(n2, L["gate"]))
            u = linear(n2, L["up"])
            down = linear(mul(g, u), L["down"])
            if c.arch == "gemma3":
                down = rms_norm(down, L["postFfnNorm"], c.rms_eps)
            return add(h, down)

        return fn

    def forward(self, ids):
        hidden, readout = self.forward_to_readout(ids)
        return linear(hidden, readout)


def sequence_loss(model: Model, input_ids, target_ids, loss_chunk=0) -> Tensor:
    """src/train/loss.ts:104-115."""
    if loss_chunk > 0:
        hidden, readout = model.forward_to_readout(input_ids)
        return fused_cross_entropy(hidden, readout, target_ids, loss_chunk)
    return cross_entropy(model.forward(input_ids), target_ids)


# ---- optimizers (train/adam.ts, train/muon.ts) ---------------------------------------------

def _ptr_array(arrs):
    return (_F * len(arrs))(*[a.ctypes.data_as(_F) for a in arrs])


class AdamW:
    def __init__(self, params, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, clip=1.0):
        self.params = list(params)
        self.base_lr = self.lr = lr
        self.beta1, self.beta2, self.eps, self.wd, self.clip = beta1, beta2, eps, weight_decay, clip
        self.m = [np.zeros(p.size, dtype=np.float32) for p in self.params]
        self.v = [np.zeros(p.size, dtype=np.float32) for p in self.params]
        self.t = 0

    def zero_grad(self):
        for p in self.params:
            p.grad.fill(0)

    def set_lr_scale(self, s):
        self.lr = self.base_lr * s

    def step(self):
        self.t += 1
        n = len(self.params)
        if n == 0:
            return
        sizes = (C.c_int64 * n)(*[p.size for p in self.params])
        _lib.or_adamw_step(n, _ptr_array([p.data for p in self.params]), _ptr_array([p.grad for p in self.params]),
                           _ptr_array(self.m), _ptr_array(self.v), sizes,
                           C.c_double(self.lr), C.c_double(self.beta1), C.c_double(self.beta2),
                           C.c_double(self.eps), C.c_double(self.wd), C.c_double(self.clip), self.t)


def newton_schulz(G: np.ndarray, m: int, n: int, steps: int) -> np.ndarray:
    G = np.ascontiguousarray(G, dtype=np.float32).reshape(-1)
    out = np.empty_like(G)
    _lib.or_newton_schulz(_f(G), _f(out), m, n, steps)
    return out


class Muon:
    def __init__(self, muon_params, aux_params, lr, momentum=0.95, nesterov=True, ns_steps=5, aux=None):
        self.muon_params = list(muon_params)
        self.base_lr = self.lr = lr
        self.momentum, self.nesterov, self.ns_steps = momentum, nesterov, ns_steps
        self.bufs = [np.zeros(p.size, dtype=np.float32) for p in self.muon_params]
        self.aux = AdamW(aux_params, **(aux or {"lr": lr}))

    def zero_grad(self):
        for p in self.muon_params:
            p.grad.fill(0)
        self.aux.zero_grad()

    def set_lr_scale(self, s):
        self.lr = self.base_lr * s
        self.aux.set_lr_scale(s)

    def step(self):
        for p, buf in zip(self.muon_params, self.bufs):
            if len(p.shape) != 2:
                raise ValueError("Muon param must be 2-D")
            rows, cols = p.shape
            _lib.or_muon_update(_f(p.data), _f(p.grad), _f(buf), rows, cols, C.c_double(self.lr),
                                C.c_double(self.momentum), int(self.nesterov), self.ns_steps)
        self.aux.step()


def wsd_schedule(warmup_steps, stable_steps, cooldown_steps, min_scale=0.0):
    """src/train/schedule.ts:20-36: step -> lr multiplier."""
    warmup = max(0, math.floor(warmup_steps))
    stable = max(0, math.floor(stable_steps))
    cooldown = max(0, math.floor(cooldown_steps))
    cooldown_start = warmup + stable
    total = cooldown_start + cooldown

    def f(step):
        if warmup > 0 and step < warmup:
            return (step + 1) / warmup
        if step < cooldown_start:
            return 1.0
        if cooldown > 0 and step < total:
            frac = (step - cooldown_start + 1) / cooldown
            return 1 - (1 - min_scale) * frac
        return 1.0 if step < total else min_scale

    return f


def attach_lora(model: Model, rank: int, alpha: float, rng: Mulberry32, a_std: float | None = None):
    """src/train/lora.ts:46-108: freeze every parameter, adapt the seven projections per layer with
    A ~ N(0, a_std) [rank,in] and B = 0 [out,rank]; returns (adapter dict for set_lora_adapters, adapter params)."""
    for p in model.params():
        p.requires_grad = False
    m, params = {}, []
    for L in model.layers:
        for k in MATRIX_KEYS:
            w = L[k]
            outd, ind = w.shape
            a = param([rank, ind], a_std if a_std is not None else 1 / math.sqrt(ind), rng)
            b = Tensor.zeros([outd, rank], True)
            m[id(w)] = (a, b, alpha / rank)
            params += [a, b]
    return m, params


def qk_logit_scale(q_norm, k_norm, head_dim: int) -> float:
    """src/train/qk-clip.ts:32-39: sqrt(sum_d (qNorm[d]*kNorm[d])^2) / sqrt(headDim), doubles over f32 gains."""
    s = 0.0
    for d in range(head_dim):
        p = float(q_norm[d]) * float(k_norm[d])
        s += p * p
    return math.sqrt(s) / math.sqrt(head_dim)


def apply_qk_clip(model: Model, tau: float) -> int:
    """src/train/qk-clip.ts:46-66: a layer whose proxy s exceeds tau has qNorm and kNorm multiplied by
    sqrt(tau/s) element by element (f32 stores), so the proxy lands on tau; returns the layers clipped."""
    if not tau > 0:
        raise ValueError("qk-clip tau must be > 0")
    pairs = model.qk_norms()
    if not pairs:
        return 0
    hd = model.cfg.head_dim
    clipped = 0
    for qn, kn in pairs:
        s = qk_logit_scale(qn.data, kn.data, hd)
        if s > tau:
            f = math.sqrt(tau / s)
            for d in range(hd):
                qn.data[d] = np.float32(float(qn.data[d]) * f)
                kn.data[d] = np.float32(float(kn.data[d]) * f)
            clipped += 1
    return clipped


def draw_windows(tokens, seq_len: int, rng, count: int, supervised=None):
    """The windows src/train/trainer.ts:56-70 draws: start = floor(rng() * (len - seq_len - 1)), inputs
    tokens[start:start+T], targets tokens[start+1:start+1+T] with unsupervised positions set to -1
    (maskWindow, trainer.ts:45-49). `rng` is a callable returning the next uniform."""
    max_start = len(tokens) - seq_len - 1
    if max_start <= 0:
        raise ValueError("Not enough tokens for one training window")
    out = []
    for _ in range(count):
        start = int(math.floor(rng() * max_start))
        ids = [int(t) for t in tokens[start:start + seq_len]]
        tg = [int(t) for t in tokens[start + 1:start + 1 + seq_len]]
        if supervised is not None:
            m = supervised[start + 1:start + 1 + seq_len]
            tg = [t if m[k] else -1 for k, t in enumerate(tg)]
        out.append((ids, tg))
    return out


def train_lm(model: Model, optimizer, windows, batch_per_step: int, steps: int, loss_chunk=0, schedule=None,
             qk_clip_tau: float = 0.0):
    """src/train/trainer.ts:51-87 with the window sampling hoisted: `windows` yields
    (input_ids, target_ids) in the order the reference's rng would have drawn them."""
    hist = []
    it = iter(windows)
    for step in range(steps):
        if schedule:
            optimizer.set_lr_scale(schedule(step))
        optimizer.zero_grad()
        loss_sum = 0.0
        for _ in range(batch_per_step):
            ids, tg = next(it)
            loss = sequence_loss(model, ids, tg, loss_chunk)
            backward(loss, 1 / batch_per_step)
            loss_sum += float(loss.data[0])
        optimizer.step()
        if qk_clip_tau:
            apply_qk_clip(model, qk_clip_tau)
        hist.append(loss_sum / batch_per_step)
    return hist
