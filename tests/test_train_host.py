"""Host side of the step loop: window sampling in the reference's rng order, supervision masks, injection,
and the QK-logit clip (src/train/qk-clip.ts) — the oracle against the reference's own literal checks
(tests/gradcheck.ts:1054-1103) and the package's restatement against the oracle."""
import importlib
import math

import numpy as np
import pytest

from test_oracle_golden import js_mulberry32

QK_CFG = dict(arch="gemma3", vocab=13, hidden=8, layers=2, heads=2, kv_heads=1, head_dim=4, ffn=16, rope_base=1e6,
              rope_base_local=1e4, rms_eps=1e-6, sliding_window=16, swa_pattern=2)


def mod(name):
    return importlib.import_module(f"gguf-trainer_amd.{name}")


def models(ref):
    rmodel = ref.Model(ref.ModelConfig(**QK_CFG), ref.Mulberry32(99))
    arch = mod("arch")
    model = arch.Model(arch.ModelConfig(**QK_CFG), {n: p.data.copy() for n, p in rmodel.named_params()})
    return rmodel, model


def test_qk_clip_reference_case(ref):
    """gradcheck.ts:1054-1103: proxy 1 at init, 6 for gains 3 and 2, the clip lands exactly on tau, scales q and k
    by the same sqrt(tau/s), counts both layers, and clipping again changes nothing."""
    train = mod("train")
    rmodel, model = models(ref)
    for m, clip, scale in ((rmodel, ref.apply_qk_clip, ref.qk_logit_scale), (model, train.apply_qk_clip, train.qk_logit_scale)):
        q0, k0 = m.qk_norms()[0]
        assert abs(scale(q0.data, k0.data, 4) - 1) <= 1e-6
        q0.data[:4] = 3
        k0.data[:4] = 2
        before = scale(q0.data, k0.data, 4)
        assert abs(before - 6) <= 1e-6
        qb, kb = q0.data.copy(), k0.data.copy()
        assert clip(m, 0.5) == 2                      # layer 1 sits at proxy 1 > 0.5 too
        assert abs(scale(q0.data, k0.data, 4) - 0.5) <= 1e-6
        f = math.sqrt(0.5 / before)
        assert np.all(np.abs(q0.data[:4] - qb[:4] * f) <= 1e-6) and np.all(np.abs(k0.data[:4] - kb[:4] * f) <= 1e-6)
        clip(m, 0.5)
        assert scale(q0.data, k0.data, 4) <= 0.5 + 1e-6
        with pytest.raises(ValueError):
            clip(m, 0.0)
    # the two restatements agree to the bit, also on uneven gains and with one layer under tau
    rmodel, model = models(ref)
    r = ref.Mulberry32(3)
    for (rq, rk), (q, k) in zip(rmodel.qk_norms(), model.qk_norms()):
        rq.data[:] = 1 + 0.5 * r.fill_randn([4])
        rk.data[:] = 1 + 0.5 * r.fill_randn([4])
        q.data[:] = rq.data
        k.data[:] = rk.data
    rmodel.qk_norms()[1][0].data[:] *= 0.1
    model.qk_norms()[1][0].data[:] *= 0.1
    assert ref.apply_qk_clip(rmodel, 0.7) == train.apply_qk_clip(model, 0.7) == 1
    for (rq, rk), (q, k) in zip(rmodel.qk_norms(), model.qk_norms()):
        assert np.array_equal(rq.data, q.data) and np.array_equal(rk.data, k.data)


def test_qk_clip_without_qk_norm_is_a_no_op(ref):
    kw = dict(arch="llama", vocab=13, hidden=8, layers=1, heads=2, kv_heads=1, head_dim=4, ffn=16)
    rmodel = ref.Model(ref.ModelConfig(**kw), ref.Mulberry32(1))
    before = [p.data.copy() for p in rmodel.params()]
    assert ref.apply_qk_clip(rmodel, 0.5) == 0
    assert all(np.array_equal(a, p.data) for a, p in zip(before, rmodel.params()))


def test_window_sampler_follows_the_reference_rng_order(ref):
    """trainer.ts:66-70 / train-gpu.ts:200-209: one rng() per window, start = floor(rng * (len - T - 1))."""
    train, ag = mod("train"), mod("autograd")
    tok_rng = js_mulberry32(0x70CC)
    tokens = [int(math.floor(tok_rng() * 50)) for _ in range(160)]
    T = 8
    want_rng = js_mulberry32(7)
    want = []
    for _ in range(8):
        s = int(math.floor(want_rng() * (160 - T - 1)))
        want.append((tokens[s:s + T], tokens[s + 1:s + 1 + T]))
    oracle = ref.draw_windows(tokens, T, ref.Mulberry32(7), 8)
    smp = train.WindowSampler(tokens, T, ag.mulberry32(7))
    got = [smp.draw(i // 2) for i in range(8)]
    for (wi, wt), (oi, ot), (gi, gt) in zip(want, oracle, got):
        assert wi == oi == gi.tolist() and wt == ot == gt.tolist()
    with pytest.raises(ValueError):
        train.WindowSampler(tokens[:9], T, ag.mulberry32(7))


def test_window_sampler_supervision_mask(ref):
    """maskWindow (trainer.ts:45-49): target k is kept iff supervised[start + 1 + k] is set."""
    train, ag = mod("train"), mod("autograd")
    tokens = [(i * 7 + 3) % 50 for i in range(100)]
    sup = [1 if (i // 5) % 2 else 0 for i in range(100)]
    smp = train.WindowSampler(tokens, 12, ag.mulberry32(11), supervised=sup)
    oracle = ref.draw_windows(tokens, 12, ref.Mulberry32(11), 5, supervised=sup)
    chk = js_mulberry32(11)
    for i in range(5):
        ids, tg = smp.draw(i)
        s = int(math.floor(chk() * (100 - 12 - 1)))
        assert ids.tolist() == tokens[s:s + 12] == oracle[i][0]
        assert tg.tolist() == [t if sup[s + 1 + k] else -1 for k, t in enumerate(tokens[s + 1:s + 13])] == oracle[i][1]
        assert -1 in tg.tolist()


def test_window_sampler_injection(ref):
    """train-gpu.ts:200-209: the inject decision draws an extra rng() only from inject_from_step on; before that the
    stream is the uninjected one; injected windows come from the other source and are never masked."""
    train, ag = mod("train"), mod("autograd")
    tokens = [(i * 7 + 3) % 50 for i in range(100)]
    inject = [50 + (i % 9) for i in range(40)]
    sup = [0] * 100
    T = 6
    plain = train.WindowSampler(tokens, T, ag.mulberry32(5))
    inj = train.WindowSampler(tokens, T, ag.mulberry32(5), supervised=sup, inject=inject, inject_frac=0.5, inject_from_step=2)
    for step in (0, 1):                              # not yet active: same starts, one rng() each
        a, b = plain.draw(step), inj.draw(step)
        assert a[0].tolist() == b[0].tolist() and set(b[1].tolist()) == {-1}
    chk = js_mulberry32(5)
    chk(), chk()
    seen = set()
    for step in range(2, 14):
        ids, tg = inj.draw(step)
        use = chk() < 0.5
        s = int(math.floor(chk() * ((40 - T - 1) if use else (100 - T - 1))))
        src = inject if use else tokens
        assert ids.tolist() == src[s:s + T]
        assert tg.tolist() == (src[s + 1:s + 1 + T] if use else [-1] * T)
        seen.add(use)
    assert seen == {True, False}
    # a zero fraction or a source too short for one window never draws the extra number
    off = train.WindowSampler(tokens, T, ag.mulberry32(5), inject=inject, inject_frac=0.0)
    short = train.WindowSampler(tokens, T, ag.mulberry32(5), inject=inject[:T + 1], inject_frac=0.9)
    plain = train.WindowSampler(tokens, T, ag.mulberry32(5))
    for step in range(4):
        want = plain.draw(step)[0].tolist()
        assert off.draw(step)[0].tolist() == want and short.draw(step)[0].tolist() == want


def test_device_records_ride_on_the_tensor():
    """HipBackend's tensor -> device record map (webgpu.ts:322's WeakMap): the record sits in the tensor's own slot; two
    maps (two backends) that meet on one tensor do not see each other's record; pop clears; a record dies with its tensor."""
    import gc
    import weakref
    hb, ag = mod("hip_backend"), mod("autograd")
    a, b = hb._EntryMap(), hb._EntryMap()
    t, u = ag.Tensor(None, [2, 3]), ag.Tensor(None, [4])
    assert a.get(t) is None and a.get(t, 7) == 7
    with pytest.raises(KeyError):
        a[t]
    ea, eb = hb._Entry(24, False), hb._Entry(24, True)
    a[t] = ea
    assert a[t] is ea and a.get(t) is ea and b.get(t) is None and a.get(u) is None
    b[t] = eb                                     # claimed by a: b keeps its record aside
    assert b[t] is eb and a[t] is ea
    e2 = hb._Entry(24, False)
    a[t] = e2                                     # the owner may replace its record
    assert a[t] is e2 and b[t] is eb
    assert a.pop(t) is e2 and a.get(t) is None and a.pop(t, 5) == 5 and b[t] is eb
    assert b.pop(t) is eb and b.get(t) is None
    class Rec:                                    # (a stand-in that can be weakly referenced)
        pass
    rec = Rec()
    b[u] = rec
    wr = weakref.ref(rec)
    del rec, u
    gc.collect()
    assert wr() is None
