"""The device-resident step loop, order of operations of trainLMGpuResident
(src/backend/train-gpu.ts:162-258): per step set the lr scale, run the micro-batches
(sequence_loss then backward with seed 1/batch), sync once to read the loss scalars, record the
optimizer step, sync again. Window sampling, injection, supervision masks and checkpoint cadence
are the caller's: `batches` yields what the reference's rng would have drawn.

stacked=True runs the B sequences of a step as one graph over B*T rows (one backward pass, one
loss per sequence, each over its own kept count and seeded 1/B): the same gradients with B times
fewer, B times larger launches. stacked=False is the reference's sequential accumulation.
"""
from __future__ import annotations

import time

import numpy as np

from . import autograd as ag
from .arch import Model, sequence_loss


def train_lm_hip_resident(model: Model, gpu, optimizer, batches, steps: int, batch_per_step: int, seq_len: int,
                          loss_chunk: int = 0, schedule=None, stacked: bool = True, reclaim: bool = False,
                          on_step_time=None):
    """batches: iterator of (input_ids, target_ids), one sequence each. Returns the mean loss per step."""
    it = iter(batches)
    hist = []
    gpu.install()
    try:
        for step in range(steps):
            t0 = time.perf_counter()
            if schedule:
                optimizer.set_lr_scale(schedule(step))
            optimizer.zero_grad()
            seqs = [next(it) for _ in range(batch_per_step)]
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
            t1 = time.perf_counter()
            optimizer.record_step()
            gpu.sync([])
            if on_step_time:
                on_step_time(t1 - t0, time.perf_counter() - t1, gpu.last_sync_readback_bytes)
            hist.append(float(sum(float(l.data.astype(np.float64).sum()) for l in losses) / batch_per_step))
    finally:
        gpu.uninstall()
    return hist
