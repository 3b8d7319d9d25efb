"""The device-resident step loop, order of operations of trainLMGpuResident
(src/backend/train-gpu.ts:162-258): per step set the lr scale, run the micro-batches
(sequence_loss then backward with seed 1/batch), sync once to read the loss scalars, record the
optimizer step, sync again (reading the QK-norm gains back when the logit clip is on), clip and
re-upload them, then the checkpoint triggers; one weight readback at the end.

Windows come either from an iterator of (input_ids, target_ids) pairs or from a WindowSampler, which draws
them from a token array with the reference's rng call order (injection and supervision masks included).

stacked=True runs the B sequences of a step as one graph over B*T rows (one backward pass, one
loss per sequence, each over its own kept count and seeded 1/B): the same gradients with B times
fewer, B times larger launches. stacked=False is the reference's sequential accumulation.
"""
from __future__ import annotations

import math
import time

import numpy as np

from . import autograd as ag
from .arch import Model, sequence_loss


class WindowSampler:
    """Training windows drawn as the reference's loops draw them (src/backend/train-gpu.ts:170-209,
    src/train/trainer.ts:56-70): start = floor(rng() * (len - seq_len - 1)), inputs = tokens[start : start+T],
    targets = tokens[start+1 : start+1+T]; positions whose `supervised` mask is 0 become -1
    (maskWindow, trainer.ts:45-49). From step `inject_from_step` on a micro-batch is drawn from `inject` instead
    with probability `inject_frac`; that decision costs one extra rng() call and is made ONLY while injection is
    active, so the stream of an uninjected run is untouched. Injected windows are never masked."""

    def __init__(self, tokens, seq_len: int, rng, supervised=None, inject=None, inject_frac: float = 0.0,
                 inject_from_step: int = 0):
        self.tokens = np.asarray(tokens)
        self.seq_len = int(seq_len)
        self.rng = rng
        self.supervised = None if supervised is None else np.asarray(supervised)
        self.inject = None if inject is None else np.asarray(inject)
        self.inject_frac = float(inject_frac)
        self.inject_from_step = int(inject_from_step)
        self.max_start = len(self.tokens) - self.seq_len - 1
        if self.max_start <= 0:
            raise ValueError("Not enough tokens for one training window")
        self.inject_max_start = len(self.inject) - self.seq_len - 1 if self.inject is not None else 0

    def draw(self, step: int):
        T = self.seq_len
        use_inject = (self.inject is not None and step >= self.inject_from_step and self.inject_frac > 0
                      and self.inject_max_start > 0 and self.rng() < self.inject_frac)
        src = self.inject if use_inject else self.tokens
        start = int(math.floor(self.rng() * (self.inject_max_start if use_inject else self.max_start)))
        ids = np.array(src[start:start + T], dtype=np.int64)
        tg = np.array(src[start + 1:start + 1 + T], dtype=np.int64)
        if self.supervised is not None and not use_inject:
            tg[self.supervised[start + 1:start + 1 + T] == 0] = -1
        return ids, tg


def qk_logit_scale(q_norm: np.ndarray, k_norm: np.ndarray, head_dim: int) -> float:
    """src/train/qk-clip.ts:32-39: std of a QK-normed attention logit, sqrt(sum (q_d k_d)^2) / sqrt(hd).
    Products and the sum are doubles over f32 gains, as there."""
    p = q_norm[:head_dim].astype(np.float64) * k_norm[:head_dim].astype(np.float64)
    s = 0.0
    for v in p:
        s += v * v
    return math.sqrt(s) / math.sqrt(head_dim)


def apply_qk_clip(model: Model, tau: float) -> int:
    """src/train/qk-clip.ts:46-66: every layer whose proxy exceeds tau gets qNorm and kNorm scaled by
    sqrt(tau / s) in place (each product rounded to f32, as a Float32Array store does). Returns the number of
    layers clipped; a model without QK-norm has nothing to clip."""
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
            qn.data[:hd] = (qn.data[:hd].astype(np.float64) * f).astype(np.float32)
            kn.data[:hd] = (kn.data[:hd].astype(np.float64) * f).astype(np.float32)
            clipped += 1
    return clipped


def train_lm_hip_resident(model: Model, gpu, optimizer, batches, steps: int, batch_per_step: int, seq_len: int,
                          loss_chunk: int = 0, schedule=None, stacked: bool = True, reclaim: bool = False,
                          on_step_time=None, qk_clip_tau: float = 0.0, checkpoint_every: int = 0,
                          checkpoint_every_ms: float = 0.0, on_checkpoint=None, log_every: int = 1, on_log=None,
                          history=None):
    """batches: a WindowSampler, or an iterator of (input_ids, target_ids), one sequence each.
    Returns the mean loss of every step; `history`, when given a list, receives the reference's log records
    {step, loss} (every `log_every` steps and the last one)."""
    draw = batches.draw if hasattr(batches, "draw") else None
    it = None if draw else iter(batches)
    hist = []
    # the clip rewrites the QK-norm gains on the host; they live on the device, so they ride along in the
    # optimizer-flush sync (a few KB), are clipped, and go back up before the next forward
    norm_tensors = [t for pair in model.qk_norms() for t in pair] if qk_clip_tau else []
    last_checkpoint_at = time.perf_counter()
    gpu.install()
    try:
        for step in range(steps):
            t0 = time.perf_counter()
            if schedule:
                optimizer.set_lr_scale(schedule(step))
            optimizer.zero_grad()
            seqs = [draw(step) if draw else next(it) for _ in range(batch_per_step)]
            losses = []
            if stacked:
                ids = np.concatenate([np.asarray(s[0]) for s in seqs])
                tg = np.concatenate([np.asarray(s[1]) for s in seqs])
                loss = sequence_loss(model, ids, tg, loss_chunk, seq_len)
                ag.backward(loss, 1.0 / batch_per_step)
                losses.append(loss)
            else:
                for b, (ids, tg) in enumerate(seqs):
                    loss = sequence_loss(model, ids, tg, loss_chunk)
                    ag.backward(loss, 1.0 / batch_per_step)
                    losses.append(loss)
                    if reclaim and b < batch_per_step - 1:
                        gpu.reclaim_step_transients(losses)
            gpu.sync(losses)
            readback = gpu.last_sync_readback_bytes
            t1 = time.perf_counter()
            optimizer.record_step()
            gpu.sync(norm_tensors)
            if qk_clip_tau:
                apply_qk_clip(model, qk_clip_tau)
                gpu.upload_params(norm_tensors)
            if on_step_time:
                on_step_time(t1 - t0, time.perf_counter() - t1, readback)
            avg = float(sum(float(l.data.astype(np.float64).sum()) for l in losses) / batch_per_step)
            hist.append(avg)
            if step % log_every == 0 or step == steps - 1:
                if history is not None:
                    history.append({"step": step, "loss": avg})
                if on_log:
                    on_log(step, avg)
            due_by_step = bool(checkpoint_every) and step % checkpoint_every == 0
            due_by_time = bool(checkpoint_every_ms) and (time.perf_counter() - last_checkpoint_at) * 1e3 >= checkpoint_every_ms
            if on_checkpoint and step > 0 and (due_by_step or due_by_time):
                optimizer.sync_weights_to_host()          # device-resident weights come down before an export
                on_checkpoint(step)
                last_checkpoint_at = time.perf_counter()
    finally:
        gpu.uninstall()
    optimizer.sync_weights_to_host()      # host arrays are authoritative again for sampling and export
    return hist
