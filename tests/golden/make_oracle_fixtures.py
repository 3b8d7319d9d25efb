"""Writes the committed fixtures of this folder from the CPU oracle (run from the repository root:
`python tests/golden/make_oracle_fixtures.py`). Nothing of the reference is imported or executed: the inputs are seeded
arrays, the expected outputs are the oracle's, and the oracle itself is pinned elsewhere (finite differences, float64
autograd, the literal vectors in reference_vectors.json).

  step_<arch>.npz    one training step's loss and gradients of a two-layer llama / qwen3 / gemma3 model, two
                     micro-batches of 19 tokens accumulated with seed 1/2, masked targets (the procedure of
                     tests/gpu-parity.ts:333-428 in the reference)
  adamw_3step.npz    the three-step AdamW case of tests/gpu-parity.ts:1044-1093 (clip triggers, then relaxes)
  newton_schulz.npz  five Newton-Schulz steps on the four shapes of tests/gpu-parity.ts:974-987

The GPU parity tests compare the device path with these files as well as with the live oracle, and a CPU test checks that
the oracle still reproduces them bit for bit."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

STEP_MODELS = {
    "llama": dict(arch="llama", vocab=61, hidden=48, layers=2, heads=6, kv_heads=2, head_dim=8, ffn=80, rope_base=1e5),
    "qwen3": dict(arch="qwen3", vocab=61, hidden=48, layers=2, heads=4, kv_heads=2, head_dim=16, ffn=80, rope_base=1e6, rms_eps=1e-6),
    "gemma3": dict(arch="gemma3", vocab=61, hidden=48, layers=3, heads=4, kv_heads=1, head_dim=16, ffn=80, rope_base=1e6,
                   rope_base_local=1e4, sliding_window=7, swa_pattern=3, rms_eps=1e-6),
}
STEP_T, STEP_B, STEP_MASK_EVERY = 19, 2, 5
NS_SHAPES = [(5, 9), (24, 17), (33, 33), (16, 64)]


def step_inputs(ref, name):
    """Seeded weights (gains jittered off 1) and token windows of one step case."""
    kw = STEP_MODELS[name]
    rmodel = ref.Model(ref.ModelConfig(**kw), ref.Mulberry32(1), std=0.1)
    rng = ref.Mulberry32(101)
    for p in rmodel.params():
        if len(p.shape) == 1:
            p.data[:] = 1 + 0.2 * rng.fill_randn([p.size])
    rng = ref.Mulberry32(5)
    seqs = []
    for _ in range(STEP_B):
        ids = [int(rng() * kw["vocab"]) for _ in range(STEP_T + 1)]
        tg = [-1 if i % STEP_MASK_EVERY == 2 else g for i, g in enumerate(ids[1:])]
        seqs.append((ids[:-1], tg))
    return rmodel, seqs


def step_case(ref, name):
    rmodel, seqs = step_inputs(ref, name)
    out = {"ids": np.int32([s[0] for s in seqs]), "targets": np.int32([s[1] for s in seqs])}
    for n, p in rmodel.named_params():
        out["w:" + n] = p.data.reshape(p.shape).copy()
        p.zero_grad()
    losses = []
    for ids, tg in seqs:
        loss = ref.sequence_loss(rmodel, ids, tg, 0)
        ref.backward(loss, 1.0 / STEP_B)
        losses.append(loss.data[0])
    out["loss"] = np.float32(losses)
    for n, p in rmodel.named_params():
        out["g:" + n] = p.grad.reshape(p.shape).copy()
    return out


def adamw_case(ref):
    rng = ref.Mulberry32(42)
    shapes = [[12, 8], [5]]
    init = [rng.fill_randn(s, 0.5) for s in shapes]
    ps = [ref.Tensor(a, s, True) for a, s in zip(init, shapes)]
    opt = ref.AdamW(ps, lr=5e-3, weight_decay=0.01, clip=1.0)
    out = {f"w0:{i}": a.copy() for i, a in enumerate(init)}
    for step, gs in enumerate((0.5, 0.05, 0.01)):
        for i, (p, s) in enumerate(zip(ps, shapes)):
            g = rng.fill_randn(s, gs)
            p.grad[:] = g.reshape(-1)
            out[f"g{step}:{i}"] = g.copy()
        opt.step()
        for i, p in enumerate(ps):
            out[f"w{step + 1}:{i}"] = p.data.reshape(p.shape).copy()
    for i in range(len(ps)):
        out[f"m:{i}"] = np.asarray(opt.m[i], dtype=np.float32).copy()
        out[f"v:{i}"] = np.asarray(opt.v[i], dtype=np.float32).copy()
    return out


def ns_case(ref):
    out = {}
    for m, n in NS_SHAPES:
        G = ref.Mulberry32(m * 100 + n).fill_randn([m, n])
        out[f"in:{m}x{n}"] = G.copy()
        out[f"out:{m}x{n}"] = np.asarray(ref.newton_schulz(G, m, n, 5), dtype=np.float32).reshape(m, n).copy()
    return out


def build_all(ref):
    files = {f"step_{name}.npz": step_case(ref, name) for name in STEP_MODELS}
    files["adamw_3step.npz"] = adamw_case(ref)
    files["newton_schulz.npz"] = ns_case(ref)
    return files


if __name__ == "__main__":
    from oracle import ref
    for fn, arrays in build_all(ref).items():
        np.savez_compressed(os.path.join(HERE, fn), **arrays)
        print(fn, sum(a.nbytes for a in arrays.values()), "bytes of arrays")
