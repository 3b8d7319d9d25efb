"""benchmark config 2 at full size (X [16384x576], W [576x1536], dY [16384x1536]; logits [16384x49152]; RMSNorm
[16384x576]): too large for the scalar oracle end to end, so parity is through sampled entries computed in
float64 on the host, the oracle on sampled rows, and size-independent properties."""
import numpy as np
import pytest

from gpu_common import assert_close, mod

pytestmark = pytest.mark.gpu

ROWS, H, F, V = 16384, 576, 1536, 49152


def dev(gpu, arr):
    b = gpu.create_state_buffer(arr.nbytes)
    gpu.write_state_buffer(b, arr)
    return b


def test_mlp_backward_gemms_full_size(gpu):
    """dX = dY.W (NN) and dW = dY^T.X (TN), the up-projection of the SmolLM2 MLP: sampled outputs against float64 dot
    products; accumulate mode adds exactly once; linearity in dY."""
    lib = mod("lib")
    rs = np.random.RandomState(0)
    X = rs.standard_normal((ROWS, H)).astype(np.float32)
    W = rs.standard_normal((F, H)).astype(np.float32)
    dY = rs.standard_normal((ROWS, F)).astype(np.float32)
    bX, bW, bdY = dev(gpu, X), dev(gpu, W), dev(gpu, dY)
    bdX, bdW = gpu.create_state_buffer(X.nbytes), gpu.create_state_buffer(W.nbytes)
    gpu.gemm(lib.NN, 0, ROWS, H, F, bdY, bW, bdX)
    gpu.gemm(lib.TN, 0, F, H, ROWS, bdY, bX, bdW)
    dX = gpu.read_state_buffer(bdX, X.size).reshape(ROWS, H)
    dW = gpu.read_state_buffer(bdW, W.size).reshape(F, H)
    W64, X64, dY64 = W.astype(np.float64), X.astype(np.float64), dY.astype(np.float64)
    rr = rs.randint(0, ROWS, 64)
    assert_close(dX[rr], dY64[rr] @ W64, "dX sampled rows")
    rw = rs.randint(0, F, 48)
    assert_close(dW[rw], dY64[:, rw].T @ X64, "dW sampled rows")
    # accumulate: a second product on top doubles the value exactly (x + x is exact in f32)
    gpu.gemm(lib.NN, 1, ROWS, H, F, bdY, bW, bdX)
    gpu.gemm(lib.TN, 1, F, H, ROWS, bdY, bX, bdW)
    assert np.array_equal(gpu.read_state_buffer(bdX, X.size).reshape(ROWS, H), 2 * dX)
    assert np.array_equal(gpu.read_state_buffer(bdW, W.size).reshape(F, H), 2 * dW)
    # forward NT on the same operands
    bY = gpu.create_state_buffer(dY.nbytes)
    gpu.gemm(lib.NT, 0, ROWS, F, H, bX, bW, bY)
    Y = gpu.read_state_buffer(bY, dY.size).reshape(ROWS, F)
    assert_close(Y[rr], X64[rr] @ W64.T, "Y sampled rows")


def test_ce_backward_full_size(gpu, ref):
    """logits [16384 x 49152] ~ N(0,2), uniform targets, 10% masked: every kept row of dz sums to zero and ignored
    rows are zero (softmax - onehot), sampled rows equal the oracle's, the loss equals a float64 logsumexp."""
    ag = mod("autograd")
    rs = np.random.RandomState(1)
    z = (2.0 * rs.standard_normal((ROWS, V))).astype(np.float32)
    tg = rs.randint(0, V, ROWS)
    tg[rs.rand(ROWS) < 0.1] = -1
    hz = ag.Tensor(z, [ROWS, V], True)
    gpu.install()
    try:
        loss = ag.cross_entropy(hz, tg)
        ag.backward(loss, 1.0)
        gpu.sync([loss])
    finally:
        gpu.uninstall()
    dz = hz.grad.reshape(ROWS, V)
    kept = tg >= 0
    z64 = z[:512].astype(np.float64)
    m = z64.max(axis=1)
    lse = np.log(np.exp(z64 - m[:, None]).sum(axis=1)) + m
    assert not np.any(dz[~kept])
    rowsum = dz.astype(np.float64).sum(axis=1)
    scale = 1.0 / kept.sum()
    assert np.abs(rowsum[kept]).max() < 1e-4 * scale
    sample = np.concatenate([np.arange(8), rs.randint(0, ROWS, 8)])
    rz = ref.Tensor(z[sample], [len(sample), V], True)
    rl = ref.cross_entropy(rz, [int(t) for t in tg[sample]])
    ref.backward(rl, 1.0)
    ks = max(int((tg[sample] >= 0).sum()), 1)
    assert_close(dz[sample] * (kept.sum() / ks), rz.grad.reshape(len(sample), V), "CE dz sampled rows")
    # loss over all kept rows, float64 on the host
    zt = z[np.arange(ROWS), np.maximum(tg, 0)].astype(np.float64)
    tot = 0.0
    for r0 in range(0, ROWS, 1024):
        blk = z[r0:r0 + 1024].astype(np.float64)
        mm = blk.max(axis=1)
        l = np.log(np.exp(blk - mm[:, None]).sum(axis=1)) + mm
        k = kept[r0:r0 + 1024]
        tot += (l[k] - zt[r0:r0 + 1024][k]).sum()
    want = tot / kept.sum()
    assert abs(loss.data[0] - want) <= 1e-5 * want


def test_rmsnorm_backward_full_size(gpu, ref):
    """RMSNorm backward on [16384 x 576] against the oracle directly (9.4 M elements)."""
    ag = mod("autograd")
    rs = np.random.RandomState(2)
    x = rs.standard_normal((ROWS, H)).astype(np.float32)
    w = (1 + 0.3 * rs.standard_normal(H)).astype(np.float32)
    g = rs.standard_normal((ROWS, H)).astype(np.float32)
    hx, hw = ag.Tensor(x, [ROWS, H], True), ag.Tensor(w, [H], True)
    from gpu_common import backward_from
    gpu.install()
    try:
        out = ag.rms_norm(hx, hw, 1e-5)
        backward_from(gpu, ag, out, g)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    rx, rw = ref.Tensor(x, [ROWS, H], True), ref.Tensor(w, [H], True)
    ro = ref.rms_norm(rx, rw, 1e-5)
    ref.backward_from(ro, g)
    assert_close(out.data, ro.data, "rmsNorm full y")
    assert_close(hx.grad, rx.grad, "rmsNorm full dx")
    assert_close(hw.grad, rw.grad, "rmsNorm full dw")


def test_glu_backward_full_size(gpu, ref):
    """SwiGLU backward on [16384 x 1536] against the oracle (25 M elements)."""
    ag = mod("autograd")
    from gpu_common import backward_from
    rs = np.random.RandomState(3)
    a, b, g = (rs.standard_normal((ROWS, F)).astype(np.float32) for _ in range(3))
    ha, hb2 = ag.Tensor(a, [ROWS, F], True), ag.Tensor(b, [ROWS, F], True)
    gpu.install()
    try:
        out = ag.mul(ag.silu(ha), hb2)
        backward_from(gpu, ag, out, g)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    ra, rb = ref.Tensor(a, [ROWS, F], True), ref.Tensor(b, [ROWS, F], True)
    ro = ref.mul(ref.silu(ra), rb)
    ref.backward_from(ro, g)
    assert_close(out.data, ro.data, "SwiGLU full out")
    assert_close(ha.grad, ra.grad, "SwiGLU full dgate")
    assert_close(hb2.grad, rb.grad, "SwiGLU full dup")


FULL = {
    # benchmark configs 4, 3 and 5 at their real shapes
    "smollm2": dict(model=dict(arch="llama", vocab=49152, hidden=576, layers=30, heads=9, kv_heads=3, head_dim=64, ffn=1536,
                               rope_base=1e5, rms_eps=1e-5), batch=8),
    "gemma3": dict(model=dict(arch="gemma3", vocab=32768, hidden=640, layers=12, heads=10, kv_heads=2, head_dim=64, ffn=2048,
                              rope_base=1e6, rope_base_local=1e4, sliding_window=512, swa_pattern=6, rms_eps=1e-6), batch=8),
    "qwen3_lora": dict(model=dict(arch="qwen3", vocab=151936, hidden=1024, layers=28, heads=16, kv_heads=8, head_dim=128, ffn=3072,
                                  rope_base=1e6, rms_eps=1e-6), batch=4, lora=16),
}


@pytest.mark.parametrize("which", ["smollm2", "gemma3", "qwen3_lora"])
def test_full_size_step_properties(gpu, which):
    """benchmark configs 4 (SmolLM2-135M shape), 3 (gemma-style, sliding window 512 on 5 of 6 layers, QK-norm) and 5
    (Qwen3-0.6B shape, head dim 128, vocabulary 151936, frozen base with rank-16 LoRA) at their real sizes, sequences
    of 2048 tokens, forward + backward. Far beyond the scalar oracle, so: the loss of a near-zero random init is ln(V)
    per sequence; the stacked graph (one launch set over B*2048 rows) and the reference's sequential accumulation (B
    graphs of 2048 rows: other GEMM tiles, split-K counts and attention splits) give the same gradients; --recompute
    changes no bit; two runs are bit-identical; half the seed gives exactly half of every gradient (a power-of-two
    factor commutes with every f32 rounding on the way); a frozen base never gets a gradient buffer."""
    from test_gpu_model import hip_step
    arch, ag = mod("arch"), mod("autograd")
    spec = FULL[which]
    cfg = arch.ModelConfig(**spec["model"])
    rs = np.random.RandomState(0)
    weights = {}
    for n in arch.param_names(cfg):
        shp = arch.param_shape(cfg, n)
        weights[n] = (1 + 0.1 * rs.standard_normal(shp)).astype(np.float32) if len(shp) == 1 else (0.02 * rs.standard_normal(shp)).astype(np.float32)
    model = arch.Model(cfg, weights)
    base = list(model.params())
    if spec.get("lora"):
        r = spec["lora"]
        adapters = {}
        for l in range(cfg.layers):
            for k in arch.MATRIX_KEYS:
                outd, ind = arch.layer_shapes(cfg)[k]
                adapters[f"L{l}.{k}"] = ((0.02 * rs.standard_normal((r, ind))).astype(np.float32),
                                         (0.02 * rs.standard_normal((outd, r))).astype(np.float32))
        trainable = arch.apply_lora(model, r, 16.0, adapters)
    else:
        trainable = base
    B, T = spec["batch"], 2048
    toks = rs.randint(0, cfg.vocab, (B, T + 1))
    seqs = []
    for b in range(B):
        tg = toks[b, 1:].copy()
        tg[rs.rand(T) < 0.1] = -1
        seqs.append((toks[b, :-1].copy(), tg))

    def grads():
        return [p.grad.copy() for p in trainable]

    try:
        l_st, _ = hip_step(gpu, model, seqs, True, T)
        g_st = grads()
        assert l_st.shape == (B,) and np.all(np.abs(l_st - np.log(cfg.vocab)) < 0.05 * np.log(cfg.vocab)), l_st
        assert all(np.isfinite(g).all() and np.abs(g).max() > 0 for g in g_st)
        l2, _ = hip_step(gpu, model, seqs, True, T)
        assert l2.tobytes() == l_st.tobytes()
        assert all(a.tobytes() == p.grad.tobytes() for a, p in zip(g_st, trainable)), "run-to-run"
        l2, _ = hip_step(gpu, model, seqs, True, T, recompute=True)
        assert l2.tobytes() == l_st.tobytes()
        assert all(a.tobytes() == p.grad.tobytes() for a, p in zip(g_st, trainable)), "recompute"
        l2, _ = hip_step(gpu, model, seqs, False, T)
        assert np.all(np.abs(l2 - l_st) <= 1e-5 * np.abs(l_st)), (l2, l_st)
        for i, (a, p) in enumerate(zip(g_st, trainable)):
            # two f32 device results with different summation orders, each held to 1e-5 of the exact value
            # elsewhere: 2e-5 between them
            assert_close(p.grad, a, f"{which}: sequential vs stacked, trainable tensor {i} {p.shape}", rel_l2=2e-5)
        gpu.install()
        try:
            loss = arch.sequence_loss(model, np.concatenate([s[0] for s in seqs]), np.concatenate([s[1] for s in seqs]), 0, T)
            ag.backward(loss, 0.5 / B)
            gpu.sync([loss])
        finally:
            gpu.uninstall()
        assert all(np.array_equal(p.grad * 2, a) for a, p in zip(g_st, trainable)), "seed linearity"
        if spec.get("lora"):
            assert all(gpu._entries[p].grad == 0 for p in base), "a frozen base parameter got a gradient buffer"
    finally:
        ag.set_lora_adapters(None)


def test_adamw_full_size_tensor_list(gpu):
    """benchmark config 4's optimizer step at its real size: the 272 tensors of the SmolLM2-135M shape (134.5 M
    parameters), two steps with the global clip active in the first and inactive in the second. Every tensor against
    the closed form of src/train/adam.ts:46-82 evaluated in float64 (vectorised; the scalar oracle covers the small
    cases), and the clip scale against a float64 norm over all gradients."""
    ag, arch, optim = mod("autograd"), mod("arch"), mod("optim")
    cfg = arch.ModelConfig(**FULL["smollm2"]["model"])
    rs = np.random.RandomState(3)
    names = arch.param_names(cfg)
    params = []
    for n in names:
        shp = arch.param_shape(cfg, n)
        params.append(ag.Tensor((0.05 * rs.standard_normal(shp)).astype(np.float32), list(shp), True))
    assert len(params) == 272 and sum(p.size for p in params) == 134515008
    lr, b1, b2, eps, wd, clip = 1e-3, 0.9, 0.95, 1e-8, 0.1, 1.0
    opt = optim.AdamWHip(gpu, params, lr=lr, beta1=b1, beta2=b2, eps=eps, weight_decay=wd, clip=clip)
    w = [p.data.astype(np.float64) for p in params]
    m = [np.zeros(p.size) for p in params]
    v = [np.zeros(p.size) for p in params]
    for t, gscale in ((1, 3e-4), (2, 2e-5)):
        grads = [(gscale * rs.standard_normal(p.size)).astype(np.float32) for p in params]
        for p, g in zip(params, grads):
            gpu.write_state_buffer(gpu.buffers_for(p)["grad"], g)
            gpu._entries[p].grad_init = True
        opt.record_step()
        norm = np.sqrt(sum(float(np.dot(g.astype(np.float64), g.astype(np.float64))) for g in grads))
        assert (norm > clip) == (t == 1)                         # the clip triggers in step 1 only
        assert abs(opt.grad_norm() - norm) <= 1e-5 * norm
        sc = clip / (norm + 1e-12) if norm > clip else 1.0
        bc1, bc2 = 1 - b1 ** t, 1 - b2 ** t
        for i, g in enumerate(grads):
            g64 = g.astype(np.float64) * sc
            m[i] = b1 * m[i] + (1 - b1) * g64
            v[i] = b2 * v[i] + (1 - b2) * g64 * g64
            w[i] -= lr * ((m[i] / bc1) / (np.sqrt(v[i] / bc2) + eps) + wd * w[i])
    opt.sync_weights_to_host()
    st = opt.export_state()
    for i, p in enumerate(params):
        assert_close(p.data, w[i], f"AdamW weights of {names[i]}")
        assert_close(st["m"][i], m[i], f"AdamW first moment of {names[i]}")
        assert_close(st["v"][i], v[i], f"AdamW second moment of {names[i]}")


def test_muon_full_size_matrices(gpu):
    """benchmark config 3's Muon step on its real matrix shapes (640x640, 128x640, 2048x640, 640x2048; one layer's
    seven matrices twice over so the per-shape batches hold several matrices): momentum, Nesterov, five Newton-Schulz
    iterations and the scaled apply against a float64 evaluation of src/train/muon.ts:69-158, and the property the
    quintic is built for: the singular values of the orthogonalised update land in about [0.7, 1.2]."""
    ag, optim, L = mod("autograd"), mod("optim"), mod("lib")
    rs = np.random.RandomState(4)
    shapes = [(640, 640), (128, 640), (128, 640), (640, 640), (2048, 640), (2048, 640), (640, 2048)] * 2
    params = [ag.Tensor((0.02 * rs.standard_normal(s)).astype(np.float32), list(s), True) for s in shapes]
    aux = ag.Tensor(np.ones(640, np.float32), [640], True)
    lr, mu = 0.01, 0.95
    opt = optim.MuonHip(gpu, params, [aux], lr=lr, momentum=mu, nesterov=True, ns_steps=5, aux={"lr": 3e-3})
    w = [p.data.astype(np.float64).reshape(s) for p, s in zip(params, shapes)]
    buf = [np.zeros(s) for s in shapes]

    def ns64(G):
        tr = G.shape[0] > G.shape[1]
        X = (G.T if tr else G) / (np.linalg.norm(G) + 1e-7)
        for _ in range(5):
            A = X @ X.T
            X = 3.4445 * X + (-4.7750 * A + 2.0315 * (A @ A)) @ X
        return X.T if tr else X

    for step in range(2):
        grads = [(0.01 * rs.standard_normal(s)).astype(np.float32) for s in shapes]
        for p, g in zip(params + [aux], grads + [np.zeros(640, np.float32)]):
            gpu.write_state_buffer(gpu.buffers_for(p)["grad"], g)
            gpu._entries[p].grad_init = True
        opt.record_step()
        for i, (g, s) in enumerate(zip(grads, shapes)):
            g64 = g.astype(np.float64)
            buf[i] = mu * buf[i] + g64
            O = ns64(g64 + mu * buf[i])
            if step == 0 and i in (0, 1, 4, 6):
                # (a square Gaussian matrix has singular values down to zero, which five steps cannot lift: there the
                # bound holds for the bulk; a rectangular one is well conditioned and every value lands in the band)
                sv = np.linalg.svd(O, compute_uv=False)
                assert sv.max() < 1.25, (s, sv.max())
                if s[0] != s[1]:
                    assert sv.min() > 0.65, (s, sv.min())
                else:
                    assert np.mean((sv > 0.65) & (sv < 1.25)) > 0.85, (s, np.mean(sv > 0.65))
            w[i] -= lr * np.sqrt(max(1.0, s[0] / s[1])) * O
    opt.sync_weights_to_host()
    st = opt.export_state()
    for i, (p, s) in enumerate(zip(params, shapes)):
        # the update is lr * O(1) on weights of 0.02: 2e-5 of the Newton-Schulz output is far inside 1e-5 of the weight
        assert_close(p.data, w[i], f"Muon weights {s} #{i}")
        assert_close(st["muonMomentum"][i], buf[i], f"Muon momentum {s} #{i}")
    # the device Newton-Schulz alone on the widest shape
    G = (0.01 * rs.standard_normal((2048, 640))).astype(np.float32)
    bi, bo = gpu.create_state_buffer(G.nbytes), gpu.create_state_buffer(G.nbytes)
    gpu.write_state_buffer(bi, G)
    L.check(gpu.ctx, L.lib.gt_newton_schulz(gpu.ctx, 2048, 640, 5, bi, bo), "gt_newton_schulz")
    assert_close(gpu.read_state_buffer(bo, G.size), ns64(G.astype(np.float64)), "Newton-Schulz 2048x640", rel_l2=2e-5)
