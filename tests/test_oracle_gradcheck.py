"""Central finite differences over the oracle with the reference's own recipe
(tests/gradcheck.ts:53-55, 100-168): eps 1e-2, divide by the f32-rounded step actually applied,
rtol 1.5e-2 / atol 2e-3, upstream gradient r ~ U(-1,1) from mulberry32(0xbeef), the op cases of
tests/gradcheck.ts:174-247 (same shapes, same spreads) and its negative control (:994-1013)."""
import math

import numpy as np
import pytest

EPS, RTOL, ATOL = 1e-2, 1.5e-2, 2e-3


def fd_check(ref, inputs, fwd, sample=None, rtol=RTOL, atol=ATOL):
    """Returns the number of elements outside atol + rtol*max(|fd|,|g|)."""
    rng_r = ref.Mulberry32(0xBEEF)
    out0 = fwd()
    n = out0.size
    r = np.array([1.0 if n == 1 else rng_r() * 2 - 1 for _ in range(n)], dtype=np.float32)
    for x in inputs:
        x.zero_grad()
    ref.backward_from(out0, r)
    analytic = [x.grad.copy() for x in inputs]
    r64 = r.astype(np.float64)
    wl = lambda o: float((o.data.astype(np.float64) * r64).sum())
    pick = ref.Mulberry32(0xCAFE)
    bad = 0
    for k, x in enumerate(inputs):
        if sample is not None and x.size > sample:
            s = set()
            while len(s) < sample:
                s.add(int(pick() * x.size))
            idxs = list(s)
        else:
            idxs = range(x.size)
        for i in idxs:
            orig = x.data[i]
            xp, xm = np.float32(np.float64(orig) + EPS), np.float32(np.float64(orig) - EPS)
            x.data[i] = xp
            lp = wl(fwd())
            x.data[i] = xm
            lm = wl(fwd())
            x.data[i] = orig
            fd = (lp - lm) / (float(xp) - float(xm))
            g = float(analytic[k][i])
            if abs(fd - g) > atol + rtol * max(abs(fd), abs(g)):
                bad += 1
    return bad


def rand_tensor(ref, shape, rng, scale=0.8):
    return ref.Tensor(rng.fill_randn(shape, scale), shape, True)


def gain(ref, n, rng):
    return ref.Tensor(np.array([1 + 0.3 * rng.randn() for _ in range(n)], dtype=np.float32), [n], True)


def test_fd_elementwise_linear_norms(ref):
    rng = ref.Mulberry32(1234)
    a, b = rand_tensor(ref, [4, 6], rng), rand_tensor(ref, [4, 6], rng)
    assert fd_check(ref, [a, b], lambda: ref.add(a, b)) == 0
    a, b = rand_tensor(ref, [4, 6], rng), rand_tensor(ref, [4, 6], rng)
    assert fd_check(ref, [a, b], lambda: ref.mul(a, b)) == 0
    x = rand_tensor(ref, [5, 7], rng, 1.5)
    assert fd_check(ref, [x], lambda: ref.silu(x)) == 0
    x = rand_tensor(ref, [5, 7], rng, 1.5)
    assert fd_check(ref, [x], lambda: ref.gelu(x)) == 0
    x = rand_tensor(ref, [4, 6], rng)
    assert fd_check(ref, [x], lambda: ref.scale(x, 2.5)) == 0
    x, w = rand_tensor(ref, [3, 5], rng), rand_tensor(ref, [4, 5], rng)
    assert fd_check(ref, [x, w], lambda: ref.linear(x, w)) == 0
    x, w = rand_tensor(ref, [4, 6], rng), gain(ref, 6, rng)
    assert fd_check(ref, [x, w], lambda: ref.rms_norm(x, w, 1e-6)) == 0
    T, H, hd = 3, 2, 4
    x, w = rand_tensor(ref, [T, H * hd], rng), gain(ref, hd, rng)
    assert fd_check(ref, [x, w], lambda: ref.rms_norm_heads(x, w, T, H, hd, 1e-6)) == 0


def test_fd_embedding_rope_attention_ce(ref):
    rng = ref.Mulberry32(1234)
    w = rand_tensor(ref, [7, 4], rng)
    assert fd_check(ref, [w], lambda: ref.embedding(w, [0, 3, 3, 6, 1, 3])) == 0
    T, H, hd = 4, 2, 6
    x = rand_tensor(ref, [T, H * hd], rng)
    assert fd_check(ref, [x], lambda: ref.rope(x, T, H, hd, 10000)) == 0
    assert fd_check(ref, [x], lambda: ref.rope(x, T, H, hd, 10000, 5)) == 0
    T, Hq, Hkv, hd = 5, 4, 2, 6
    q, k, v = (rand_tensor(ref, [T, n * hd], rng) for n in (Hq, Hkv, Hkv))
    assert fd_check(ref, [q, k, v], lambda: ref.attention(q, k, v, T, Hq, Hkv, hd)) == 0
    T, W = 6, 3
    q, k, v = (rand_tensor(ref, [T, n * hd], rng) for n in (Hq, Hkv, Hkv))
    assert fd_check(ref, [q, k, v], lambda: ref.attention(q, k, v, T, Hq, Hkv, hd, W)) == 0
    z = rand_tensor(ref, [4, 9], rng)
    assert fd_check(ref, [z], lambda: ref.cross_entropy(z, [2, 7, 2, 0])) == 0
    z = rand_tensor(ref, [5, 9], rng)
    assert fd_check(ref, [z], lambda: ref.cross_entropy(z, [2, -1, 2, 0, -1])) == 0


def test_fd_lora_fused_soft(ref):
    rng = ref.Mulberry32(77)
    T, ind, outd, rank = 4, 5, 6, 2
    x, w = rand_tensor(ref, [T, ind], rng), rand_tensor(ref, [outd, ind], rng)
    a, b = rand_tensor(ref, [rank, ind], rng), rand_tensor(ref, [outd, rank], rng)
    ref.set_lora_adapters({id(w): (a, b, 2.0)})
    try:
        assert fd_check(ref, [x, a, b], lambda: ref.linear(x, w)) == 0
    finally:
        ref.set_lora_adapters({})
    h, w = rand_tensor(ref, [5, 6], rng), rand_tensor(ref, [11, 6], rng)
    assert fd_check(ref, [h, w], lambda: ref.fused_cross_entropy(h, w, [3, -1, 10, 0, 5], 4)) == 0
    z = rand_tensor(ref, [4, 9], rng)
    tids = [2, 5, -1, 0, 7, 1, 3, 3]
    tp = [0.5, 0.2, 0.0, 0.0, 0.7, 0.0, 0.3, 0.3]
    assert fd_check(ref, [z], lambda: ref.soft_cross_entropy(z, tids, tp, 2)) == 0


def test_fd_negative_control(ref):
    """tests/gradcheck.ts:994-1013: a silu whose backward drops the x*s*(1-s) term must be flagged."""
    rng = ref.Mulberry32(1234)
    x = rand_tensor(ref, [5, 7], rng, 1.5)

    def broken():
        out = ref.silu(x)
        sig = 1 / (1 + np.exp(-x.data.astype(np.float64)))

        def bw():
            x.grad[:] = (x.grad + out.grad * sig).astype(np.float32)

        out._backward = bw
        return out

    assert fd_check(ref, [x], broken) > 0


CFGS = {
    "llama": dict(arch="llama", vocab=19, hidden=8, layers=2, heads=2, kv_heads=1, head_dim=4, ffn=12),
    "qwen3": dict(arch="qwen3", vocab=19, hidden=8, layers=2, heads=4, kv_heads=2, head_dim=4, ffn=12, rms_eps=1e-6),
    "gemma3": dict(arch="gemma3", vocab=19, hidden=8, layers=3, heads=2, kv_heads=1, head_dim=4, ffn=12,
                   sliding_window=3, swa_pattern=3, rope_base=1e6, rope_base_local=1e4, rms_eps=1e-6),
}


@pytest.mark.parametrize("arch", ["llama", "qwen3", "gemma3"])
def test_fd_whole_model(ref, arch):
    """tests/gradcheck.ts:919-943: whole-model loss at O(1) parameter scale (matrices 0.5*randn, gains
    1+0.2*randn from mulberry32(4321)), 6 sampled elements per parameter, rtol 2e-2 / atol 3e-3."""
    cfg = ref.ModelConfig(**CFGS[arch])
    model = ref.Model(cfg, ref.Mulberry32(99))
    rng = ref.Mulberry32(4321)
    for p in model.params():
        is_norm = len(p.shape) == 1
        p.data[:] = np.array([1 + 0.2 * rng.randn() if is_norm else 0.5 * rng.randn() for _ in range(p.size)],
                             dtype=np.float32)
    ids, tg = [1, 5, 2, 9, 5], [5, 2, 9, 5, 12]
    assert fd_check(ref, model.params(), lambda: ref.sequence_loss(model, ids, tg), sample=6,
                    rtol=2e-2, atol=3e-3) == 0


@pytest.mark.parametrize("arch", ["llama", "qwen3", "gemma3"])
def test_directional_derivative_at_real_init(ref, arch):
    """tests/gradcheck.ts:945-991: 4 random unit directions over all parameters, eps 2e-3,
    fail when rel > 5e-2 and abs > 1e-3."""
    cfg = ref.ModelConfig(**CFGS[arch])
    model = ref.Model(cfg, ref.Mulberry32(99))
    ids, tg = [1, 5, 2, 9, 5], [5, 2, 9, 5, 12]
    params = model.params()
    ref.backward(ref.sequence_loss(model, ids, tg), 1)
    rng = ref.Mulberry32(777)
    for _ in range(4):
        dirs = [np.array([rng.randn() for _ in range(p.size)]) for p in params]
        norm = math.sqrt(sum(float((d * d).sum()) for d in dirs))
        dirs = [d / norm for d in dirs]
        dot = sum(float((p.grad.astype(np.float64) * d).sum()) for p, d in zip(params, dirs))
        saved = [p.data.copy() for p in params]

        def at(sign):
            for p, s0, d in zip(params, saved, dirs):
                p.data[:] = (s0 + sign * 2e-3 * d).astype(np.float32)
            return float(ref.sequence_loss(model, ids, tg).data[0])

        lp, lm = at(1), at(-1)
        for p, s0 in zip(params, saved):
            p.data[:] = s0
        fd = (lp - lm) / 4e-3
        assert not (abs(fd - dot) / max(abs(fd), abs(dot), 1e-12) > 5e-2 and abs(fd - dot) > 1e-3)


@pytest.mark.parametrize("arch", ["llama", "gemma3"])
def test_checkpoint_bit_identical(ref, arch):
    """tests/gradcheck.ts:770-831: --recompute on/off gives bit-identical loss and gradients."""
    cfg = ref.ModelConfig(**CFGS[arch])
    ids, tg = [1, 5, 5, 18, 0, 7], [5, 5, 18, -1, 7, 2]
    res = []
    for on in (False, True):
        model = ref.Model(cfg, ref.Mulberry32(3))
        ref.set_checkpointing(on)
        try:
            loss = ref.sequence_loss(model, ids, tg)
            ref.backward(loss, 0.5)
        finally:
            ref.set_checkpointing(False)
        res.append((loss.data.copy(), [p.grad.copy() for p in model.params()]))
    assert res[0][0].tobytes() == res[1][0].tobytes()
    for g0, g1 in zip(res[0][1], res[1][1]):
        assert g0.tobytes() == g1.tobytes()
    assert any(np.any(g) for g in res[0][1])


def test_checkpoint_input_guard(ref):
    """gradcheck.ts:808-829: a checkpointed block that reads a computed tensor built outside it, or that returns one
    of its inputs, is refused; the same tensor declared as an input is allowed."""
    r = ref.Mulberry32(12)
    x = ref.Tensor(r.fill_randn([5, 6], 0.8), [5, 6], True)
    w1 = ref.Tensor(r.fill_randn([6, 6], 0.8), [6, 6], True)
    ref.set_checkpointing(True)
    try:
        shared = ref.linear(x, w1)
        with pytest.raises(ValueError, match="did not create"):
            ref.checkpoint([x], lambda: ref.add(ref.silu(ref.linear(x, w1)), shared))
        with pytest.raises(ValueError, match="one of its inputs"):
            ref.checkpoint([x], lambda: x)
        out = ref.checkpoint([x, shared], lambda: ref.add(ref.silu(ref.linear(x, w1)), shared))
        assert out.shape == [5, 6]
    finally:
        ref.set_checkpointing(False)
