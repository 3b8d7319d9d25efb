"""llama / qwen3 / gemma3 forward graphs as compositions of the autograd ops, in the op order of
src/arch/llama.ts:183-221, src/arch/qwen3.ts:153-195 and src/arch/gemma3.ts:173-223. They exist
here because they define the graph the backward pass runs over; config parsing, GGUF naming and
CLI flags of src/arch/ are not reproduced.

`ids` may hold B sequences of `seq_len` tokens stacked (rows = B*seq_len); seq_len defaults to
len(ids), the reference's one-sequence call.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

from . import autograd as ag
from .autograd import Tensor


@dataclass
class ModelConfig:
    arch: str                  # "llama" | "qwen3" | "gemma3"
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
    sliding_window: int = 0    # gemma3
    swa_pattern: int = 0       # gemma3: every swa_pattern-th layer is global
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
    """gemma3.ts:75-77."""
    return c.swa_pattern > 0 and il % c.swa_pattern == c.swa_pattern - 1


def param_names(c: ModelConfig):
    names = ["tokenEmbd", "outputNorm"] + ([] if c.tie else ["output"])
    for l in range(c.layers):
        names += [f"L{l}.{k}" for k in LAYER_KEYS[c.arch]]
    return names


def param_shape(c: ModelConfig, name: str):
    if name in ("tokenEmbd", "output"):
        return [c.vocab, c.hidden]
    if name == "outputNorm":
        return [c.hidden]
    return layer_shapes(c)[name.split(".", 1)[1]]


class Model:
    """weights: dict name -> float32 array, names as in param_names()."""

    def __init__(self, cfg: ModelConfig, weights: dict):
        self.cfg = cfg
        self.p = {n: Tensor(np.asarray(weights[n], dtype=np.float32), param_shape(cfg, n), True) for n in param_names(cfg)}
        self.tokenEmbd = self.p["tokenEmbd"]
        self.outputNorm = self.p["outputNorm"]
        self.output = self.p.get("output")
        self.layers = [{k: self.p[f"L{l}.{k}"] for k in LAYER_KEYS[cfg.arch]} for l in range(cfg.layers)]

    def named_params(self):
        return list(self.p.items())

    def params(self):
        return list(self.p.values())

    def param_groups(self):
        """(muon, aux) as in llama.ts:170-181 / qwen3.ts:131-142 / gemma3.ts:151-162."""
        muon, aux = [], [self.tokenEmbd, self.outputNorm] + ([self.output] if self.output is not None else [])
        for L in self.layers:
            muon += [L[k] for k in MATRIX_KEYS]
            aux += [L[k] for k in LAYER_KEYS[self.cfg.arch] if k not in MATRIX_KEYS]
        return muon, aux

    def qk_norms(self):
        return [(L["qNorm"], L["kNorm"]) for L in self.layers if "qNorm" in L]

    def forward_to_readout(self, ids, seq_len=None):
        c = self.cfg
        rows = len(ids)
        T = rows if seq_len is None else int(seq_len)
        h = ag.embedding(self.tokenEmbd, ids)
        if c.arch == "gemma3":
            h = ag.scale(h, math.sqrt(c.hidden))
        for il, L in enumerate(self.layers):
            h = ag.checkpoint([h], self._block(h, L, il, rows, T))
        return ag.rms_norm(h, self.outputNorm, c.rms_eps), (self.output if self.output is not None else self.tokenEmbd)

    def _block(self, h_in, L, il, rows, T):
        c = self.cfg

        def fn():
            h = h_in
            window, rope_b = 0, c.rope_base
            if c.arch == "gemma3":
                glob = is_global_layer(c, il)
                window = 0 if glob else c.sliding_window
                rope_b = c.rope_base if glob else c.rope_base_local
            n1 = ag.rms_norm(h, L["attnNorm"], c.rms_eps)
            q = ag.linear(n1, L["qProj"])
            k = ag.linear(n1, L["kProj"])
            v = ag.linear(n1, L["vProj"])
            if c.arch in ("qwen3", "gemma3"):
                q = ag.rms_norm_heads(q, L["qNorm"], rows, c.heads, c.head_dim, c.rms_eps)
                k = ag.rms_norm_heads(k, L["kNorm"], rows, c.kv_heads, c.head_dim, c.rms_eps)
            q = ag.rope(q, T, c.heads, c.head_dim, rope_b)
            k = ag.rope(k, T, c.kv_heads, c.head_dim, rope_b)
            a = ag.attention(q, k, v, T, c.heads, c.kv_heads, c.head_dim, window)
            attn_out = ag.linear(a, L["oProj"])
            if c.arch == "gemma3":
                attn_out = ag.rms_norm(attn_out, L["postAttnNorm"], c.rms_eps)
            h = ag.add(h, attn_out)
            n2 = ag.rms_norm(h, L["ffnNorm"], c.rms_eps)
            g = (ag.gelu if c.arch == "gemma3" else ag.silu)(ag.linear(n2, L["gate"]))
            u = ag.linear(n2, L["up"])
            down = ag.linear(ag.mul(g, u), L["down"])
            if c.arch == "gemma3":
                down = ag.rms_norm(down, L["postFfnNorm"], c.rms_eps)
            return ag.add(h, down)

        return fn

    def forward(self, ids, seq_len=None):
        hidden, readout = self.forward_to_readout(ids, seq_len)
        return ag.linear(hidden, readout)


def sequence_loss(model: Model, input_ids, target_ids, loss_chunk: int = 0, seq_len=None) -> Tensor:
    """src/train/loss.ts:104-115."""
    if loss_chunk > 0:
        hidden, readout = model.forward_to_readout(input_ids, seq_len)
        return ag.fused_cross_entropy(hidden, readout, target_ids, loss_chunk, seq_len)
    return ag.cross_entropy(model.forward(input_ids, seq_len), target_ids, seq_len)


def apply_lora(model: Model, rank: int, alpha: float, adapters: dict):
    """src/train/lora.ts:46-82: freeze every existing parameter and route the seven projections of each layer
    through A [rank,in], B [out,rank]. `adapters` maps parameter name -> (A array, B array). Returns the
    trainable adapter tensors (the aux group) and installs them in `linear`."""
    if rank <= 0:
        raise ValueError(f"applyLora: rank must be positive, got {rank}")
    if alpha <= 0:
        raise ValueError(f"applyLora: alpha must be positive, got {alpha}")
    for t in model.params():
        t.requires_grad = False
    m, aux = {}, []
    for l, L in enumerate(model.layers):
        for k in MATRIX_KEYS:
            w = L[k]
            a_arr, b_arr = adapters[f"L{l}.{k}"]
            a = Tensor(a_arr, [rank, w.shape[1]], True)
            b = Tensor(b_arr, [w.shape[0], rank], True)
            m[id(w)] = (a, b, alpha / rank)
            aux += [a, b]
    ag.set_lora_adapters(m)
    return aux


def clear_lora(model: Model | None = None):
    """lora.ts:114-120."""
    ag.set_lora_adapters({})
    if model is not None:
        for t in model.params():
            t.requires_grad = True
