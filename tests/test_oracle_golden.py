"""The oracle against every literal vector the reference's own tests hold for this path, and
against closed forms / invariants those tests state (tests/gradcheck.ts, tests/gpu-parity.ts)."""
import math

import numpy as np
import pytest


def js_mulberry32(seed):
    """Independent restatement of autograd.ts:69-78 with Python big ints and explicit ToInt32 /
    ToUint32 / Math.imul, so a wrap-around mistake in the C version cannot hide."""
    def to_i32(x):
        x &= 0xFFFFFFFF
        return x - (1 << 32) if x & 0x80000000 else x

    def imul(a, b):
        return to_i32((a & 0xFFFFFFFF) * (b & 0xFFFFFFFF))

    a = seed & 0xFFFFFFFF
    def nxt():
        nonlocal a
        a = to_i32(a)
        a = to_i32(a + 0x6D2B79F5)
        t = imul(a ^ ((a & 0xFFFFFFFF) >> 15), 1 | a)
        t = to_i32(t + imul(t ^ ((t & 0xFFFFFFFF) >> 7), 61 | t)) ^ t
        return ((t ^ ((t & 0xFFFFFFFF) >> 14)) & 0xFFFFFFFF) / 4294967296
    return nxt


@pytest.mark.parametrize("seed", [0, 1234, 0xBEEF, 0xCAFE, 0xFFFFFFFF])
def test_mulberry32_matches_js_semantics(ref, seed):
    a, b = ref.Mulberry32(seed), js_mulberry32(seed)
    for _ in range(2000):
        assert a() == b()


def test_mulberry32_known_first_output(ref):
    # mulberry32(0)() as published with the generator
    assert ref.Mulberry32(0)() == 0.26642920868471265


def test_randn_and_fills_match_box_muller_over_the_js_generator(ref):
    """autograd.ts:54-66: randn = sqrt(-2 ln u) cos(2 pi v) with u, v the next two non-zero uniforms; param() /
    randTensor() store randn * std as f32; the uniform fill is lo + (hi - lo) * u. Replayed on the big-int generator
    with math.sqrt/log/cos. libm and Python's math share the platform's log/cos, so the f64 values agree to the last
    bit or one ulp; the f32 stores are compared exactly except where an f64 ulp straddles an f32 rounding tie."""
    for seed in (0, 7, 0xBEEF):
        js = js_mulberry32(seed)
        def js_randn():
            u = v = 0.0
            while u == 0.0:
                u = js()
            while v == 0.0:
                v = js()
            return math.sqrt(-2.0 * math.log(u)) * math.cos(2.0 * math.pi * v)
        a = ref.Mulberry32(seed)
        for _ in range(500):
            got, want = a.randn(), js_randn()
            assert abs(got - want) <= 4e-16 * max(1.0, abs(want))
        # the generator state stays in step (two uniforms per normal): the fills continue the same stream
        got = ref.Mulberry32(seed).fill_randn([1000], 0.02)
        js = js_mulberry32(seed)
        want = np.array([js_randn() * 0.02 for _ in range(1000)])
        assert np.count_nonzero(got != want.astype(np.float32)) <= 1
        assert np.all(np.abs(got.astype(np.float64) - want) <= 2.0 ** -24 * np.abs(want) + 1e-45)
        # sample moments of N(0, 0.02^2): a dropped factor 2 or a sine for the cosine would still pass these,
        # the replay above would not; a wrong std or a uniform in place of a normal fails here
        big = ref.Mulberry32(seed).fill_randn([200000], 0.02).astype(np.float64)
        assert abs(big.mean()) < 2e-4 and abs(big.std() - 0.02) < 2e-4
        assert abs(np.mean(big ** 4) / big.var() ** 2 - 3.0) < 0.05
        gotu = ref.Mulberry32(seed).fill_uniform([1000], -1.0, 1.0)
        js = js_mulberry32(seed)
        wantu = np.array([-1.0 + 2.0 * js() for _ in range(1000)]).astype(np.float32)
        assert np.array_equal(gotu, wantu)
        gotu = ref.Mulberry32(seed).fill_uniform([64], 0.25, 3.0)
        js = js_mulberry32(seed)
        assert np.array_equal(gotu, np.array([0.25 + 2.75 * js() for _ in range(64)]).astype(np.float32))


def test_ce_closed_form_big_gaps(ref):
    """tests/gradcheck.ts:321-335: rows [gap,0,0,-3], target 3, tolerance 1e-4, hard and soft (q=0.6)."""
    for gap in [1, 10, 30, 60, 90]:
        row = np.array([gap, 0, 0, -3], dtype=np.float32)
        exact = math.log(math.exp(gap) + 2 + math.exp(-3)) + 3
        got = ref.cross_entropy(ref.Tensor(row, [1, 4], True), [3]).data[0]
        assert abs(got - exact) < 1e-4
        soft = ref.soft_cross_entropy(ref.Tensor(row, [1, 4], True), [3], [0.6], 1).data[0]
        assert abs(soft - 0.6 * exact) < 1e-4


def test_ce_device_case_rows(ref):
    """tests/gpu-parity.ts:776-784: logits [[90,0,0,-3],[60,1,0,0]], targets [3,2]."""
    z = np.array([[90, 0, 0, -3], [60, 1, 0, 0]], dtype=np.float32)
    exact = (math.log(math.exp(90) + 2 + math.exp(-3)) + 3 + math.log(math.exp(60) + math.e + 2) - 0) / 2
    got = ref.cross_entropy(ref.Tensor(z, [2, 4], True), [3, 2]).data[0]
    assert abs(got - exact) < 1e-4


def test_ce_all_ignored_is_exactly_zero(ref):
    """tests/gradcheck.ts:676, tests/gpu-parity.ts:2419-2502: zero loss and zero gradient, not NaN."""
    rng = ref.Mulberry32(7)
    z = ref.Tensor(rng.fill_randn([5, 11]), [5, 11], True)
    loss = ref.cross_entropy(z, [-1] * 5)
    ref.backward(loss)
    assert loss.data[0] == 0.0 and not np.any(z.grad)
    h = ref.Tensor(rng.fill_randn([5, 6]), [5, 6], True)
    w = ref.Tensor(rng.fill_randn([11, 6]), [11, 6], True)
    loss = ref.fused_cross_entropy(h, w, [-1] * 5, 4)
    ref.backward(loss)
    assert loss.data[0] == 0.0 and not np.any(h.grad) and not np.any(w.grad)


def test_ce_mean_times_kept_is_summed_nll(ref):
    """tests/gradcheck.ts:692-723: targets [-1,-1,-1,4,9,2,17]."""
    rng = ref.Mulberry32(99)
    T, V = 7, 20
    tg = [-1, -1, -1, 4, 9, 2, 17]
    z = rng.fill_randn([T, V], 0.8)
    loss = ref.cross_entropy(ref.Tensor(z, [T, V], True), tg).data[0]
    z64 = z.astype(np.float64)
    nll = 0.0
    for t, g in enumerate(tg):
        if g >= 0:
            nll += math.log(np.exp(z64[t] - z64[t].max()).sum()) + z64[t].max() - z64[t, g]
    assert abs(loss * 4 - nll) < 1e-5


def test_fused_ce_equals_dense(ref):
    """tests/gradcheck.ts:854-877: fused == crossEntropy(linear(h,w)) to 1e-5, loss and gradients,
    for chunk widths that do and do not divide V."""
    rng = ref.Mulberry32(4321)
    T, H, V = 6, 8, 23
    hd, wd = rng.fill_randn([T, H], 0.8), rng.fill_randn([V, H], 0.8)
    tg = [3, -1, 22, 0, 7, -1]
    h0, w0 = ref.Tensor(hd, [T, H], True), ref.Tensor(wd, [V, H], True)
    dense = ref.cross_entropy(ref.linear(h0, w0), tg)
    ref.backward(dense)
    for chunk in [1, 5, 8, 23, 64]:
        h1, w1 = ref.Tensor(hd, [T, H], True), ref.Tensor(wd, [V, H], True)
        fused = ref.fused_cross_entropy(h1, w1, tg, chunk)
        ref.backward(fused)
        assert abs(fused.data[0] - dense.data[0]) < 1e-5
        assert np.abs(h1.grad - h0.grad).max() < 1e-5
        assert np.abs(w1.grad - w0.grad).max() < 1e-5


def test_soft_ce_one_hot_teacher_is_hard_ce(ref):
    rng = ref.Mulberry32(5)
    T, V = 5, 13
    z = rng.fill_randn([T, V])
    tg = [1, -1, 12, 0, 6]
    a, b = ref.Tensor(z, [T, V], True), ref.Tensor(z, [T, V], True)
    hard = ref.cross_entropy(a, tg)
    soft = ref.soft_cross_entropy(b, [g for g in tg], [1.0] * T, 1)
    ref.backward(hard)
    ref.backward(soft)
    assert abs(hard.data[0] - soft.data[0]) < 1e-6
    assert np.abs(a.grad - b.grad).max() < 1e-6


def test_wsd_literal_vector(ref):
    """tests/gradcheck.ts:1037-1052."""
    s = ref.wsd_schedule(4, 3, 4, 0.1)
    want = [0.25, 0.5, 0.75, 1, 1, 1, 1, 0.775, 0.55, 0.325, 0.1, 0.1]
    assert all(abs(s(i) - w) < 1e-6 for i, w in enumerate(want))
    assert ref.wsd_schedule(0, 2, 2)(0) == 1
    nc = ref.wsd_schedule(0, 2, 0, 0)
    assert nc(1) == 1 and nc(2) == 0


def test_seed_linearity(ref):
    """tests/gradcheck.ts:1015-1032: backward(loss, s) scales every gradient by s."""
    rng = ref.Mulberry32(11)
    x = rng.fill_randn([4, 6])
    w = rng.fill_randn([9, 6])
    grads = []
    for seed in (1.0, 0.25):
        xt, wt = ref.Tensor(x, [4, 6], True), ref.Tensor(w, [9, 6], True)
        ref.backward(ref.cross_entropy(ref.linear(ref.silu(xt), wt), [1, 2, -1, 8]), seed)
        grads.append((xt.grad.copy(), wt.grad.copy()))
    for g1, g2 in zip(*grads):
        assert np.allclose(g1 * 0.25, g2, rtol=1e-6, atol=1e-9)


def test_lora_freeze_and_merge(ref):
    """tests/gradcheck.ts:248-301: frozen base gets exactly zero, adapters get gradient, merged == adapted."""
    rng = ref.Mulberry32(1234)
    T, ind, outd, rank, alpha = 4, 5, 6, 2, 4
    x = ref.Tensor(rng.fill_randn([T, ind], 0.8), [T, ind], True)
    w = ref.Tensor(rng.fill_randn([outd, ind], 0.8), [outd, ind], False)
    a = ref.Tensor(rng.fill_randn([rank, ind], 0.8), [rank, ind], True)
    b = ref.Tensor(rng.fill_randn([outd, rank], 0.8), [outd, rank], True)
    sc = alpha / rank
    ref.set_lora_adapters({id(w): (a, b, sc)})
    try:
        out = ref.linear(x, w)
        ref.backward_from(out, np.ones(out.size, dtype=np.float32))
    finally:
        ref.set_lora_adapters({})
    assert not np.any(w.grad)
    assert np.abs(a.grad).max() > 0 and np.abs(b.grad).max() > 0
    merged = w.data.reshape(outd, ind).astype(np.float64) + sc * (
        b.data.reshape(outd, rank).astype(np.float64) @ a.data.reshape(rank, ind).astype(np.float64))
    plain = ref.linear(x, ref.Tensor(merged.astype(np.float32), [outd, ind], True))
    assert np.abs(out.data - plain.data).max() < 1e-5
