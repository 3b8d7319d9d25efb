"""The oracle against independent derivations: torch float64 autograd on the same graphs
(library attention / cross_entropy / gelu / silu / rms_norm, not the oracle's formulas),
torch.optim.AdamW for the AdamW step, and the SVD closed form of the quintic Newton-Schulz."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

torch.set_num_threads(2)


def t64(a, shape, grad=True):
    return torch.tensor(np.asarray(a, dtype=np.float64).reshape(shape), dtype=torch.float64, requires_grad=grad)


def relerr(a, b, floor=1e-6):
    a, b = np.asarray(a, dtype=np.float64).ravel(), np.asarray(b, dtype=np.float64).ravel()
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), floor)


def torch_rope(x, T, H, hd, base, pos=0):
    half = hd // 2
    inv = base ** (-2.0 * torch.arange(half, dtype=torch.float64) / hd)
    ang = (torch.arange(T, dtype=torch.float64) + pos)[:, None] * inv[None, :]
    z = torch.view_as_complex(torch.stack([x.view(T, H, hd)[..., :half], x.view(T, H, hd)[..., half:]], -1).contiguous())
    z = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    return torch.cat([z.real, z.imag], -1).reshape(T, H * hd)


def torch_attention(q, k, v, T, Hq, Hkv, hd, window):
    g = Hq // Hkv
    qh = q.view(T, Hq, hd).transpose(0, 1)
    kh = k.view(T, Hkv, hd).transpose(0, 1).repeat_interleave(g, 0)
    vh = v.view(T, Hkv, hd).transpose(0, 1).repeat_interleave(g, 0)
    i = torch.arange(T)
    mask = i[None, :] <= i[:, None]
    if window > 0:
        mask &= i[None, :] > i[:, None] - window
    o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask)
    return o.transpose(0, 1).reshape(T, Hq * hd)


def torch_rms(x, w, eps):
    return F.rms_norm(x, (x.shape[-1],), w, eps)


def check(ref, build_ref, build_torch, arrays, tol=2e-6, floor=1e-6):
    """arrays: list of (np.float32 array, shape). Same seeded upstream gradient on both sides."""
    rts = [ref.Tensor(a, s, True) for a, s in arrays]
    tts = [t64(a, s) for a, s in arrays]
    out_r = build_ref(*rts)
    out_t = build_torch(*tts)
    assert relerr(out_r.data, out_t.detach().numpy()) < tol
    up = ref.Mulberry32(0xBEEF).fill_uniform([out_r.size])
    ref.backward_from(out_r, up)
    out_t.backward(torch.tensor(up.astype(np.float64)).reshape(out_t.shape))
    for r, t in zip(rts, tts):
        assert relerr(r.grad, t.grad.numpy(), floor) < tol


def test_ops_vs_torch64(ref):
    rng = ref.Mulberry32(2024)
    R = lambda *s, sc=0.8: (rng.fill_randn(list(s), sc), list(s))
    check(ref, ref.linear, lambda x, w: x @ w.T, [R(7, 12), R(9, 12)])
    check(ref, ref.silu, F.silu, [R(6, 10, sc=1.5)])
    check(ref, ref.gelu, lambda x: F.gelu(x, approximate="tanh"), [R(6, 10, sc=1.5)])
    check(ref, lambda x: ref.scale(x, 2.5), lambda x: x * 2.5, [R(6, 10)])
    check(ref, ref.mul, lambda a, b: a * b, [R(6, 10), R(6, 10)])
    check(ref, ref.add, lambda a, b: a + b, [R(6, 10), R(6, 10)])
    check(ref, lambda x: ref.add(x, x), lambda x: x + x, [R(6, 10)])
    check(ref, lambda x: ref.mul(x, x), lambda x: x * x, [R(6, 10)])
    g = (1 + 0.3 * rng.fill_randn([16]), [16])
    check(ref, lambda x, w: ref.rms_norm(x, w, 1e-5), lambda x, w: torch_rms(x, w, 1e-5), [R(9, 16), g])
    g = (1 + 0.3 * rng.fill_randn([8]), [8])
    check(ref, lambda x, w: ref.rms_norm_heads(x, w, 5, 3, 8, 1e-6),
          lambda x, w: torch_rms(x.view(5, 3, 8), w, 1e-6).reshape(5, 24), [R(5, 24), g])
    ids = [0, 3, 3, 6, 1, 3, 0]
    check(ref, lambda w: ref.embedding(w, ids), lambda w: w[torch.tensor(ids)], [R(7, 5)])
    for pos in (0, 5):
        check(ref, lambda x: ref.rope(x, 9, 3, 8, 10000.0, pos), lambda x: torch_rope(x, 9, 3, 8, 10000.0, pos), [R(9, 24)])


@pytest.mark.parametrize("T,Hq,Hkv,hd,window", [(17, 4, 2, 8, 0), (33, 6, 2, 16, 0), (40, 4, 1, 8, 7), (12, 2, 2, 4, 1),
                                                (64, 9, 3, 64, 0), (50, 4, 2, 32, 16)])
def test_attention_vs_torch64(ref, T, Hq, Hkv, hd, window):
    rng = ref.Mulberry32(T * 131 + hd)
    arrs = [(rng.fill_randn([T, n * hd], 0.8), [T, n * hd]) for n in (Hq, Hkv, Hkv)]
    check(ref, lambda q, k, v: ref.attention(q, k, v, T, Hq, Hkv, hd, window),
          lambda q, k, v: torch_attention(q, k, v, T, Hq, Hkv, hd, window), arrs,
          # window 1: dq, dk are exactly 0; the reference's f32-rounded scores leave ~1e-8 there
          floor=1.0 if window == 1 else 1e-6)


@pytest.mark.parametrize("T,Hq,Hkv,hd,window", [(40, 6, 2, 16, 9), (33, 6, 2, 16, 0), (64, 9, 3, 64, 0), (50, 9, 3, 8, 16),
                                                (21, 4, 4, 8, 5)])
def test_attention_parallel_bwd_variant_matches(ref, T, Hq, Hkv, hd, window):
    """or_attention_bwd_par (dK/dV summed per kv head in f64 and rounded once) is the checker of the GPU attention
    comparisons at T = 2048 and the attention backward of the timed CPU baseline: pinned against torch float64
    autograd directly, with and without a window and with a GQA group of 3, and against the serial form."""
    rng = ref.Mulberry32(9 + T)
    arrs = [rng.fill_randn([T, n * hd], 0.8) for n in (Hq, Hkv, Hkv)]
    up = ref.Mulberry32(1).fill_uniform([T * Hq * hd])
    res = []
    for par in (False, True):
        q, k, v = (ref.Tensor(a, list(a.shape), True) for a in arrs)
        o = ref.attention(q, k, v, T, Hq, Hkv, hd, window, parallel_bwd=par)
        ref.backward_from(o, up)
        res.append([q.grad, k.grad, v.grad])
    for a, b in zip(*res):
        assert relerr(a, b) < 1e-6
    tq, tk, tv = (t64(a, list(a.shape)) for a in arrs)
    torch_attention(tq, tk, tv, T, Hq, Hkv, hd, window).backward(torch.tensor(up.astype(np.float64)).reshape(T, Hq * hd))
    for a, t in zip(res[1], (tq, tk, tv)):
        assert relerr(a, t.grad.numpy()) < 2e-6


@pytest.mark.parametrize("T,ind,outd,frozen", [(7, 12, 9, False), (33, 17, 5, False), (1, 3, 40, False), (19, 31, 23, True)])
def test_linear_dots_bwd_variant_matches_serial_and_float64(ref, T, ind, outd, frozen):
    """or_linear_bwd_dots (the OpenMP-safe backward the whole-model GPU comparisons at tuned shapes and the timed CPU
    baseline run through) against the reference-ordered or_linear_bwd and against a float64 matrix product, from non-zero
    starting gradients, on ragged shapes, with a frozen weight (no dW) as one case, and with zeros in the upstream
    gradient (the serial form skips those terms)."""
    rng = ref.Mulberry32(T * 1009 + ind * 31 + outd)
    x, w = rng.fill_randn([T, ind], 0.8), rng.fill_randn([outd, ind], 0.8)
    gx0, gw0 = rng.fill_randn([T, ind], 0.5), rng.fill_randn([outd, ind], 0.5)
    up = rng.fill_uniform([T * outd]).reshape(T, outd)
    up[::3, ::2] = 0.0
    res = []
    for par in (False, True):
        ref.PARALLEL_BWD = par
        try:
            xt, wt = ref.Tensor(x, [T, ind], True), ref.Tensor(w, [outd, ind], not frozen)
            xt.grad[:] = gx0.ravel()
            wt.grad[:] = gw0.ravel()
            out = ref.linear(xt, wt)
            out.grad[:] = up.ravel()
            out._backward()
        finally:
            ref.PARALLEL_BWD = False
        res.append((xt.grad.copy(), wt.grad.copy()))
    x64, w64, up64 = x.astype(np.float64).reshape(T, ind), w.astype(np.float64).reshape(outd, ind), up.astype(np.float64)
    want_gx = gx0.astype(np.float64).reshape(T, ind) + up64 @ w64
    want_gw = gw0.astype(np.float64).reshape(outd, ind) + (0 if frozen else up64.T @ x64)
    for gx, gw in res:
        assert relerr(gx, want_gx) < 2e-7
        assert relerr(gw, want_gw) < 2e-7
    assert relerr(res[1][0], res[0][0]) < 2e-7 and relerr(res[1][1], res[0][1]) < 2e-7
    if frozen:
        assert np.array_equal(res[0][1], gw0.ravel()) and np.array_equal(res[1][1], gw0.ravel())


def test_soft_ce_k3_vs_float64_closed_form(ref):
    """softCrossEntropy with k = 3 teachers per row (autograd.ts:1076-1138) against its closed form written with library
    routines in float64: loss = (1/kept) sum_rows sum_j q_j (logsumexp(z) - z[id_j]), gradient by torch autograd. The rows
    hold a duplicated id (its two probabilities both count), a zero-probability pad slot, a teacher mass below 1, and an
    ignored row (first id -1); a forward that mis-weights teachers j >= 1 fails the loss, a backward that drops the
    duplicate's second term fails the gradient."""
    rng = ref.Mulberry32(77)
    T, V, k = 6, 29, 3
    z = rng.fill_randn([T, V], 2.0)
    ids = [[4, 17, 9], [5, 5, 2], [28, 0, 3], [-1, 0, 0], [11, 12, 12], [7, 1, 20]]
    q = [[0.5, 0.3, 0.2], [0.4, 0.35, 0.1], [0.7, 0.0, 0.25], [0.0, 0.0, 0.0], [0.2, 0.3, 0.1], [0.05, 0.9, 0.05]]
    flat_ids = [i for r in ids for i in r]
    flat_q = [p for r in q for p in r]
    zt = ref.Tensor(z, [T, V], True)
    loss = ref.soft_cross_entropy(zt, flat_ids, flat_q, k)
    ref.backward(loss, 0.75)

    z64 = t64(z, [T, V])
    lse = torch.logsumexp(z64, dim=1)
    total = torch.zeros((), dtype=torch.float64)
    kept = 0
    for t in range(T):
        if ids[t][0] < 0:
            continue
        kept += 1
        for j in range(k):
            total = total + q[t][j] * (lse[t] - z64[t, ids[t][j]])
    want = total / kept
    want.backward(torch.tensor(0.75, dtype=torch.float64))
    want = float(want.detach())
    assert kept == 5
    assert abs(float(loss.data[0]) - want) <= 2e-7 * abs(want)
    assert relerr(zt.grad, z64.grad.numpy()) < 2e-7
    assert np.all(zt.grad.reshape(T, V)[3] == 0)


def test_ce_vs_torch64(ref):
    rng = ref.Mulberry32(31)
    T, V = 9, 37
    tg = [3, -1, 36, 0, 7, -1, 7, 20, 1]
    z = (rng.fill_randn([T, V], 2.0), [T, V])
    check(ref, lambda x: ref.cross_entropy(x, tg),
          lambda x: F.cross_entropy(x, torch.tensor(tg), ignore_index=-1).reshape(1), [z])
    h, w = (rng.fill_randn([T, 10], 0.8), [T, 10]), (rng.fill_randn([V, 10], 0.8), [V, 10])
    check(ref, lambda a, b: ref.fused_cross_entropy(a, b, tg, 8),
          lambda a, b: F.cross_entropy(a @ b.T, torch.tensor(tg), ignore_index=-1).reshape(1), [h, w])


def torch_model_loss(ref, model, P, ids, tg):
    c = model.cfg
    T = len(ids)
    h = P["tokenEmbd"][torch.tensor(ids)]
    if c.arch == "gemma3":
        h = h * math.sqrt(c.hidden)
    for il in range(c.layers):
        L = lambda k: P[f"L{il}.{k}"]
        window, rb = 0, c.rope_base
        if c.arch == "gemma3":
            glob = ref.is_global_layer(c, il)
            window, rb = (0, c.rope_base) if glob else (c.sliding_window, c.rope_base_local)
        n1 = torch_rms(h, L("attnNorm"), c.rms_eps)
        q, k, v = n1 @ L("qProj").T, n1 @ L("kProj").T, n1 @ L("vProj").T
        if c.arch != "llama":
            q = torch_rms(q.view(T, c.heads, c.head_dim), L("qNorm"), c.rms_eps).reshape(T, -1)
            k = torch_rms(k.view(T, c.kv_heads, c.head_dim), L("kNorm"), c.rms_eps).reshape(T, -1)
        q, k = torch_rope(q, T, c.heads, c.head_dim, rb), torch_rope(k, T, c.kv_heads, c.head_dim, rb)
        a = torch_attention(q, k, v, T, c.heads, c.kv_heads, c.head_dim, window) @ L("oProj").T
        if c.arch == "gemma3":
            a = torch_rms(a, L("postAttnNorm"), c.rms_eps)
        h = h + a
        n2 = torch_rms(h, L("ffnNorm"), c.rms_eps)
        act = (lambda x: F.gelu(x, approximate="tanh")) if c.arch == "gemma3" else F.silu
        d = (act(n2 @ L("gate").T) * (n2 @ L("up").T)) @ L("down").T
        if c.arch == "gemma3":
            d = torch_rms(d, L("postFfnNorm"), c.rms_eps)
        h = h + d
    hid = torch_rms(h, P["outputNorm"], c.rms_eps)
    return F.cross_entropy(hid @ P["tokenEmbd"].T, torch.tensor(tg), ignore_index=-1)


@pytest.mark.parametrize("arch", ["llama", "qwen3", "gemma3"])
def test_whole_model_vs_torch64(ref, arch):
    """Tied embeddings, GQA, QK-norm, sliding window on 2 of 3 layers, masked targets; two micro-batches
    accumulated with seed 1/2 (tests/gpu-parity.ts:395-428)."""
    kw = dict(arch=arch, vocab=53, hidden=24, layers=3, heads=4, kv_heads=2, head_dim=8, ffn=40, rms_eps=1e-5,
              rope_base=1e5)
    if arch == "gemma3":
        kw.update(sliding_window=5, swa_pattern=3, rope_base_local=1e4)
    cfg = ref.ModelConfig(**kw)
    model = ref.Model(cfg, ref.Mulberry32(0), std=0.3)
    rng = ref.Mulberry32(17)
    for p in model.params():
        if len(p.shape) == 1:
            p.data[:] = 1 + 0.2 * rng.fill_randn([p.size])
    P = {n: t64(p.data, p.shape) for n, p in model.named_params()}
    batches = []
    for _ in range(2):
        ids = [int(rng() * cfg.vocab) for _ in range(14)]
        tg = ids[1:] + [int(rng() * cfg.vocab)]
        tg[3] = tg[9] = -1
        batches.append((ids, tg))
    total_t = 0
    for ids, tg in batches:
        loss = ref.sequence_loss(model, ids, tg)
        ref.backward(loss, 0.5)
        lt = torch_model_loss(ref, model, P, ids, tg)
        assert abs(loss.data[0] - lt.item()) / abs(lt.item()) < 1e-6
        total_t = total_t + 0.5 * lt
    total_t.backward()
    for n, p in model.named_params():
        assert relerr(p.grad, P[n].grad.numpy()) < 5e-6, n


def test_adamw_three_steps_vs_torch(ref):
    """tests/gpu-parity.ts:1044-1093: shapes [12,8] and [5], lr 5e-3, wd 0.01, clip 1, gradient scales
    0.5 / 0.05 / 0.01 so the clip triggers on step 1 and relaxes after. The update is checked with
    torch.optim.AdamW in float64, whose decoupled decay p*(1-lr*wd) - lr*mhat/(sqrt(vhat)+eps) is the
    same closed form as src/train/adam.ts:72-78; only the global-norm clip (eps 1e-12, applied when
    norm > clip) is computed by hand, since torch's clip uses a different epsilon."""
    rng = ref.Mulberry32(42)
    shapes = [[12, 8], [5]]
    ps = [ref.Tensor(rng.fill_randn(s, 0.5), s, True) for s in shapes]
    tp = [t64(p.data, p.shape) for p in ps]
    opt_r = ref.AdamW(ps, lr=5e-3, weight_decay=0.01, clip=1.0)
    opt_t = torch.optim.AdamW(tp, lr=5e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    clipped = []
    for gs in (0.5, 0.05, 0.01):
        gr = [rng.fill_randn(s, gs) for s in shapes]
        norm = math.sqrt(sum(float((g.astype(np.float64) ** 2).sum()) for g in gr))
        clipped.append(norm > 1.0)
        sc = 1.0 / (norm + 1e-12) if norm > 1.0 else 1.0
        for p, t, g in zip(ps, tp, gr):
            p.grad[:] = g.reshape(-1)
            t.grad = torch.tensor(g.astype(np.float64) * sc).reshape(t.shape)
        opt_r.step()
        opt_t.step()
        for p, t in zip(ps, tp):
            assert relerr(p.data, t.detach().numpy()) < 3e-7
    assert clipped == [True, False, False]


def test_adamw_config1_hyperparameters_vs_torch(ref):
    rng = ref.Mulberry32(3)
    p = ref.Tensor(rng.fill_randn([40, 6], 0.02), [40, 6], True)
    t = t64(p.data, p.shape)
    o_r = ref.AdamW([p], lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=0.0)
    o_t = torch.optim.AdamW([t], lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for _ in range(5):
        g = rng.fill_randn([40, 6], 0.1)
        p.grad[:] = g.reshape(-1)
        t.grad = torch.tensor(g.astype(np.float64))
        o_r.step()
        o_t.step()
    assert relerr(p.data, t.detach().numpy()) < 3e-7


def ns_closed_form(G, steps):
    """The quintic X <- aX + (bA + cA^2)X with A = XX^T acts on each singular value as
    s <- a s + b s^3 + c s^5 and leaves the singular vectors alone."""
    G = G.astype(np.float64)
    U, s, Vt = np.linalg.svd(G / (np.linalg.norm(G) + 1e-7), full_matrices=False)
    for _ in range(steps):
        s = 3.4445 * s - 4.7750 * s ** 3 + 2.0315 * s ** 5
    return (U * s) @ Vt


@pytest.mark.parametrize("m,n", [(5, 9), (24, 17), (33, 33), (16, 64)])
def test_newton_schulz_vs_svd_closed_form(ref, m, n):
    """Shapes of tests/gpu-parity.ts:974-987 (m<n, m>n, m=n), 5 steps."""
    rng = ref.Mulberry32(m * 100 + n)
    G = rng.fill_randn([m, n])
    got = ref.newton_schulz(G, m, n, 5).reshape(m, n)
    want = ns_closed_form(G, 5)
    assert relerr(got, want) < 2e-5
    sv = np.linalg.svd(got.astype(np.float64), compute_uv=False)
    assert sv.max() < 1.25 and sv.min() > 0.3
    flipped = ref.newton_schulz(np.ascontiguousarray(G.T), n, m, 5).reshape(n, m)
    assert relerr(flipped.T, got) < 1e-5


def test_muon_step_vs_closed_form(ref):
    """Two steps so the momentum buffer carries over (tests/gpu-parity.ts:996-1032)."""
    rng = ref.Mulberry32(8)
    m, n = 24, 10
    p = ref.Tensor(rng.fill_randn([m, n], 0.5), [m, n], True)
    w = p.data.astype(np.float64).reshape(m, n)
    buf = np.zeros((m, n))
    opt = ref.Muon([p], [], lr=0.02)
    for _ in range(2):
        g = rng.fill_randn([m, n], 0.1)
        p.grad[:] = g.reshape(-1)
        opt.step()
        buf = 0.95 * buf + g
        w = w - 0.02 * math.sqrt(max(1, m / n)) * ns_closed_form(g + 0.95 * buf, 5)
        assert relerr(p.data, w) < 2e-5
