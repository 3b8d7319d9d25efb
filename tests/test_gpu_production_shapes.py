"""Parity at the sizes the benchmark configurations run at, against the CPU oracle where it finishes in seconds and
against float64 closed forms where it does not: attention at T = 2048 on the three head layouts of the benchmark
models through both backward paths, one SmolLM2-width layer with the real vocabulary over a Zipf-distributed sequence,
the embedding backward over 16384 Zipf tokens, the sparse-teacher and the vocab-chunked cross-entropy at vocabularies of
49152 and 151936, and the device-side range guard of ids that arrive as device buffers."""
import ctypes as C

import numpy as np
import pytest

from gpu_common import LOSS_REL, assert_close, backward_from, mod

pytestmark = pytest.mark.gpu


def zipf_tokens(vocab, n, seed, s=1.1):
    """Zipf(1.1) over the vocabulary by inverse CDF on a fixed permutation of the ids (the benchmark's token stream)."""
    rs = np.random.RandomState(seed)
    p = 1.0 / np.arange(1, vocab + 1, dtype=np.float64) ** s
    cdf = np.cumsum(p / p.sum())
    perm = np.random.RandomState(12345).permutation(vocab)
    return perm[np.minimum(np.searchsorted(cdf, rs.rand(n)), vocab - 1)].astype(np.int64)


def dev(gpu, arr):
    b = gpu.create_state_buffer(arr.nbytes)
    gpu.write_state_buffer(b, arr)
    return b


# (B, T, Hq, Hkv, hd, window): one sequence as the reference calls the backend (webgpu.ts:1142-1174, train-gpu.ts:200-219)
# and two stacked ones with one workgroup per tile, which is how a stacked batch of eight runs
LAYOUTS = [(1, 2048, 9, 3, 64, 0), (2, 2048, 9, 3, 64, 0),            # SmolLM2-135M
           (1, 2048, 10, 2, 64, 512), (2, 2048, 10, 2, 64, 512),      # the gemma-style model's sliding-window layers
           (1, 2048, 10, 2, 64, 0),                                   # and its global layers
           (1, 2048, 16, 8, 128, 0), (2, 2048, 16, 8, 128, 0)]        # Qwen3-0.6B


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", LAYOUTS)
@pytest.mark.parametrize("path", ["kept-scores", "recompute"])
def test_attention_full_length_vs_oracle(gpu, ref, B, T, Hq, Hkv, hd, window, path):
    """tests/gpu-parity.ts:872-930 at the benchmark shapes. "kept-scores": gt_attn_fwd_scores keeps S, dK/dV reads it
    and stores dS, dQ is the banded product over dS (the path a training step takes). "recompute": gt_attn_fwd /
    gt_attn_bwd with the score gradients not kept, every kernel recomputing S. out, dq, dk, dv of every sequence
    against the oracle: 1e-5 relative L2, 1e-4 max error over max magnitude."""
    lib = mod("lib")
    rs = np.random.RandomState(T + Hq + hd + window)
    arrs = {n: (0.8 * rs.standard_normal((B * T, h * hd))).astype(np.float32) for n, h in (("q", Hq), ("k", Hkv), ("v", Hkv), ("up", Hq))}
    bufs = {n: dev(gpu, a) for n, a in arrs.items()}
    out, dq = (gpu.create_state_buffer(arrs["q"].nbytes) for _ in range(2))
    dk, dv = (gpu.create_state_buffer(arrs["k"].nbytes) for _ in range(2))
    lse = gpu.create_state_buffer(B * Hq * T * 4)
    if B > 1:
        gpu.set_option("attn.splits", 1)
    try:
        if path == "kept-scores":
            need = C.c_uint64(0)
            lib.check(gpu.ctx, lib.lib.gt_attn_scores_bytes(gpu.ctx, B, T, Hq, Hkv, hd, window, C.byref(need)), "bytes")
            assert need.value == B * Hq * T * T * 4
            sco = gpu.create_state_buffer(need.value)
            gpu.set_option("attn.keep_ds", 1)
            lib.check(gpu.ctx, lib.lib.gt_attn_fwd_scores(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out, lse, sco), "fwd")
            lib.check(gpu.ctx, lib.lib.gt_attn_bwd_scores(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out,
                                                          bufs["up"], lse, sco, dq, 0, dk, 0, dv, 0), "bwd")
        else:
            gpu.set_option("attn.keep_ds", 0)
            lib.check(gpu.ctx, lib.lib.gt_attn_fwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out, lse), "fwd")
            lib.check(gpu.ctx, lib.lib.gt_attn_bwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out,
                                                   bufs["up"], lse, dq, 0, dk, 0, dv, 0), "bwd")
        got = {n: gpu.read_state_buffer(b, a.size).reshape(B, -1) for n, b, a in (("out", out, arrs["q"]), ("dq", dq, arrs["q"]),
                                                                                 ("dk", dk, arrs["k"]), ("dv", dv, arrs["k"]))}
    finally:
        gpu.set_option("attn.splits", -1)
        gpu.set_option("attn.keep_ds", 1)
    ref.set_threads(min(16, ref.max_threads()))
    try:
        for b in range(B):
            s = slice(b * T, (b + 1) * T)
            rq, rk, rv = (ref.Tensor(arrs[n][s], [T, arrs[n].shape[1]], True) for n in ("q", "k", "v"))
            o = ref.attention(rq, rk, rv, T, Hq, Hkv, hd, window, parallel_bwd=True)
            ref.backward_from(o, arrs["up"][s].reshape(-1))
            assert_close(got["out"][b], o.data, f"{path} out[{b}]")
            for nm, rr in (("dq", rq), ("dk", rk), ("dv", rv)):
                assert_close(got[nm][b], rr.grad, f"{path} {nm}[{b}]")
    finally:
        ref.set_threads(1)


def test_one_layer_at_real_widths_full_length_vs_oracle(gpu, ref):
    """One SmolLM2-135M layer at its real widths (hidden 576, 9/3 heads of 64, SwiGLU 1536, tied readout over the real
    vocabulary of 49152) on one sequence of 2048 Zipf(1.1) tokens with masked targets: loss and every gradient tensor
    against the oracle. The embedding backward sees 2048 tokens over the real table, the tied matrix takes the readout's
    and the embedding's gradients, attention runs the kept-scores path at T = 2048, CE at V = 49152."""
    from test_gpu_model import build_pair, compare, hip_step, ref_step
    kw = dict(arch="llama", vocab=49152, hidden=576, layers=1, heads=9, kv_heads=3, head_dim=64, ffn=1536, rope_base=1e5, rms_eps=1e-5)
    rmodel, model = build_pair(ref, kw, seed=21, std=0.02)
    T = 2048
    toks = zipf_tokens(kw["vocab"], T + 1, 7)
    tg = toks[1:].copy()
    tg[np.random.RandomState(8).rand(T) < 0.1] = -1
    seqs = [([int(t) for t in toks[:-1]], [int(t) for t in tg])]
    assert len(set(seqs[0][0])) < T // 2            # Zipf: the embedding backward sums many rows per id
    lh, gh = hip_step(gpu, model, seqs, False, T)
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        lr, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    compare(lh, gh, lr, gr, "SmolLM2 layer, T 2048, V 49152")


def test_embedding_backward_zipf_batch_vs_oracle(gpu, ref):
    """The embedding backward of the headline step: 16384 Zipf(1.1) tokens over a [49152, 576] table, against the oracle's
    scatter-add (autograd.ts:545-560), once storing and once adding on top of a used accumulator."""
    ag = mod("autograd")
    V, d, n = 49152, 576, 16384
    ids = zipf_tokens(V, n, 100)
    rs = np.random.RandomState(4)
    w = (0.02 * rs.standard_normal((V, d))).astype(np.float32)
    g = rs.standard_normal((n, d)).astype(np.float32)
    hw = ag.Tensor(w, [V, d], True)
    gpu.install()
    try:
        for _ in range(2):                          # the second micro-batch adds to the first one's accumulator
            out = ag.embedding(hw, ids)
            backward_from(gpu, ag, out, g)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    rw = ref.Tensor(w, [V, d], True)
    for _ in range(2):
        ro = ref.embedding(rw, [int(i) for i in ids])
        ref.backward_from(ro, g.reshape(-1))
    assert np.array_equal(out.data, ro.data)
    assert_close(hw.grad, rw.grad, "embedding dW, 16384 Zipf tokens twice")
    untouched = np.ones(V, bool)
    untouched[ids] = False
    assert not np.any(hw.grad.reshape(V, d)[untouched])


@pytest.mark.parametrize("V,k", [(49152, 4), (151936, 8)])
def test_soft_cross_entropy_production_vocab(gpu, ref, V, k):
    """softCrossEntropy (webgpu.ts:1331-1378) over [2048, V] logits with k sparse teachers per row: the loss against
    the float64 closed form sum_j q_j (logsumexp(z) - z[id_j]) / kept over all rows, every kept row of dz summing to
    scale * (S - sum q) = 0, ignored rows exactly zero, and 24 sampled rows of dz against the oracle. Rows carry a
    duplicated id, a zero-probability slot and a teacher mass below one."""
    ag = mod("autograd")
    rows = 2048
    rs = np.random.RandomState(V % 1000 + k)
    z = (2.0 * rs.standard_normal((rows, V))).astype(np.float32)
    ids = rs.randint(0, V, (rows, k))
    q = rs.rand(rows, k)
    q = (0.9 * q / q.sum(axis=1, keepdims=True)).round(4)
    ids[::5, 1] = ids[::5, 0]                       # duplicate id
    q[::7, k - 1] = 0.0                             # zero-probability pad slot
    ids[::11, 0] = -1                               # ignored rows
    flat_ids = [int(i) for i in ids.ravel()]
    flat_q = [float(p) for p in q.ravel()]
    hz = ag.Tensor(z, [rows, V], True)
    gpu.install()
    try:
        loss = ag.soft_cross_entropy(hz, flat_ids, flat_q, k)
        ag.backward(loss, 0.5)
        gpu.sync([loss])
    finally:
        gpu.uninstall()
    kept = ids[:, 0] >= 0
    nk = int(kept.sum())
    lse = np.empty(rows)
    for r0 in range(0, rows, 256):
        blk = z[r0:r0 + 256].astype(np.float64)
        m = blk.max(axis=1)
        lse[r0:r0 + 256] = np.log(np.exp(blk - m[:, None]).sum(axis=1)) + m
    zt = z[np.arange(rows)[:, None], np.maximum(ids, 0)].astype(np.float64)
    want = ((q * (lse[:, None] - zt)).sum(axis=1)[kept]).sum() / nk
    assert abs(float(loss.data[0]) - want) <= LOSS_REL * abs(want)
    dz = hz.grad.reshape(rows, V)
    assert not np.any(dz[~kept])
    rowsum = dz.astype(np.float64).sum(axis=1)
    assert np.abs(rowsum[kept]).max() < 1e-4 * 0.5 / nk
    sample = np.concatenate([np.arange(12), rs.randint(0, rows, 12)])
    rz = ref.Tensor(z[sample], [len(sample), V], True)
    rl = ref.soft_cross_entropy(rz, [int(i) for i in ids[sample].ravel()], [float(p) for p in q[sample].ravel()], k)
    ref.backward(rl, 0.5)
    ks = max(int(kept[sample].sum()), 1)
    assert_close(dz[sample] * (nk / ks), rz.grad.reshape(len(sample), V), "softCE dz sampled rows")


@pytest.mark.parametrize("frozen", [False, True])
def test_fused_cross_entropy_wide_spans_vs_oracle(gpu, ref, frozen):
    """fusedCrossEntropy (webgpu.ts:1214-1278) with chunk 8192 over a vocabulary of three whole spans and a ragged
    fourth (each chunk wider than one workgroup's share), masked rows, two stacked sequences, a trainable and a frozen
    readout: loss, dH and dW against the oracle's chunked form."""
    from gpu_common import op_case
    V, H, T, chunk = 3 * 8192 + 100, 32, 40, 8192
    rs = np.random.RandomState(31 + frozen)
    h = rs.standard_normal((T, H)).astype(np.float32)
    w = (0.5 * rs.standard_normal((V, H))).astype(np.float32)
    tg = [int(t) for t in rs.randint(0, V, T)]
    tg[3] = -1
    tg[17] = V - 1                                  # in the ragged last span
    tg[18] = 8192                                   # first column of the second span
    op_case(gpu, ref, [h, w], lambda ag, a, b: ag.fused_cross_entropy(a, b, tg, chunk),
            lambda rf, a, b: rf.fused_cross_entropy(a, b, tg, chunk), f"fusedCE chunk 8192, frozen={frozen}",
            frozen=(1,) if frozen else ())


def test_loss_chunk_at_the_qwen3_readout_equals_dense(gpu, ref):
    """--loss-chunk 8192 at the Qwen3-0.6B readout (V = 151936, H = 1024: 18 whole spans and one of 4480 columns) on one
    sequence of 2048 rows with a 60 % loss mask: loss, dH and dW equal the dense path's (cross_entropy over linear) to
    the parity bound, as tests/gradcheck.ts:854-877 asks of the two forms."""
    ag = mod("autograd")
    rows, H, V, chunk = 2048, 1024, 151936, 8192
    rs = np.random.RandomState(9)
    h = rs.standard_normal((rows, H)).astype(np.float32)
    w = (0.02 * rs.standard_normal((V, H))).astype(np.float32)
    tg = rs.randint(0, V, rows)
    tg[rs.rand(rows) >= 0.6] = -1
    res = []
    for fused in (False, True):
        hh, hw = ag.Tensor(h, [rows, H], True), ag.Tensor(w, [V, H], True)
        gpu.install()
        try:
            loss = ag.fused_cross_entropy(hh, hw, tg, chunk) if fused else ag.cross_entropy(ag.linear(hh, hw), tg)
            ag.backward(loss, 1.0)
            gpu.sync([loss])
        finally:
            gpu.uninstall()
        res.append((float(loss.data[0]), hh.grad.copy(), hw.grad.copy()))
    (ld, dhd, dwd), (lf, dhf, dwf) = res
    assert abs(lf - ld) <= LOSS_REL * abs(ld)
    assert_close(dhf, dhd, "loss-chunk dH vs dense")
    assert_close(dwf, dwd, "loss-chunk dW vs dense")
    # the dense form itself against float64 on sampled entries: loss rows, and rows of dW = dz^T h
    kept = tg >= 0
    sample = np.flatnonzero(kept)[:64]
    z = h[sample].astype(np.float64) @ w.astype(np.float64).T
    m = z.max(axis=1)
    nll = np.log(np.exp(z - m[:, None]).sum(axis=1)) + m - z[np.arange(len(sample)), tg[sample]]
    hs = ag.Tensor(h[sample], [len(sample), H], False)
    hw = ag.Tensor(w, [V, H], False)
    gpu.install()
    try:
        ls = ag.fused_cross_entropy(hs, hw, tg[sample], chunk)
        gpu.sync([ls])
    finally:
        gpu.uninstall()
    assert abs(float(ls.data[0]) - nll.mean()) <= LOSS_REL * nll.mean()


def test_out_of_range_ids_are_skipped_and_reported(gpu):
    """Ids, targets and teacher ids reach the library as device buffers, so the range check the reference makes above the
    dispatch (autograd.ts:324-346, 875-894, 974-998) cannot be made before the launch. One bad value among good ones:
    the call itself succeeds, the kernel does not index with the value, the next gt_sync returns an error that names it,
    and the sync after that is clean again."""
    lib = mod("lib")
    L = lib.lib

    def sync_error():
        rc = L.gt_sync(gpu.ctx)
        return L.gt_last_error(gpu.ctx).decode() if rc else ""

    assert sync_error() == ""
    V, d, n = 50, 8, 6
    rs = np.random.RandomState(0)
    W = rs.standard_normal((V, d)).astype(np.float32)
    g = rs.standard_normal((n, d)).astype(np.float32)
    ids = np.array([3, 7, 50, 7, 0, 49], np.int32)               # 50 == V is one past the table
    bW, bg, bids = dev(gpu, W), dev(gpu, g), dev(gpu, ids)
    bout, bdW = gpu.create_state_buffer(g.nbytes), gpu.create_state_buffer(W.nbytes)
    lib.check(gpu.ctx, L.gt_embedding_fwd(gpu.ctx, n, d, V, bids, bW, bout), "embedding")
    msg = sync_error()
    assert "embedding id 50 at row 2 is outside [0, 50)" in msg, msg
    assert sync_error() == ""
    out = gpu.read_state_buffer(bout, n * d).reshape(n, d)
    good = ids < V
    assert np.array_equal(out[good], W[ids[good]]) and not np.any(out[2])
    lib.check(gpu.ctx, L.gt_embedding_bwd(gpu.ctx, n, d, V, bids, bg, bdW, 0), "embedding.bwd")
    assert "embedding id 50 at row 2" in sync_error()
    want = np.zeros((V, d), np.float64)
    for t in np.flatnonzero(good):
        want[ids[t]] += g[t]
    assert_close(gpu.read_state_buffer(bdW, V * d), want, "embedding dW without the bad row")
    bneg = dev(gpu, np.array([3, -1, 2, 7, 0, 49], np.int32))
    lib.check(gpu.ctx, L.gt_embedding_fwd(gpu.ctx, n, d, V, bneg, bW, bout), "embedding")
    assert "embedding id -1 at row 1" in sync_error()

    rows, Vc = 4, 12
    z = rs.standard_normal((rows, Vc)).astype(np.float32)
    tg = np.array([5, -1, 12, 0], np.int32)                      # 12 == V
    bz, btg = dev(gpu, z), dev(gpu, tg)
    binv = dev(gpu, np.array([0.5], np.float32))
    bloss, blse, bdz = (gpu.create_state_buffer(s * 4) for s in (1, rows, rows * Vc))
    lib.check(gpu.ctx, L.gt_ce_fwd(gpu.ctx, rows, Vc, rows, bz, btg, binv, bloss, blse), "ce")
    assert "cross-entropy target 12 at row 2 is outside [-1, 12)" in sync_error()
    z64 = z.astype(np.float64)
    lse = np.log(np.exp(z64).sum(axis=1))
    want = 0.5 * ((lse[0] - z64[0, 5]) + (lse[3] - z64[3, 0]))
    assert abs(gpu.read_state_buffer(bloss, 1)[0] - want) <= 1e-5 * abs(want)
    lib.check(gpu.ctx, L.gt_ce_bwd(gpu.ctx, rows, Vc, rows, bz, btg, binv, blse, 1.0, bdz, 0), "ce.bwd")
    assert sync_error() == ""                                    # reported once, by the forward
    dzb = gpu.read_state_buffer(bdz, rows * Vc).reshape(rows, Vc)
    pz = np.exp(z64 - lse[:, None])
    wantb = 0.5 * pz
    wantb[0, 5] -= 0.5
    wantb[3, 0] -= 0.5
    wantb[1] = 0
    wantb[2] = 0                                                 # the bad row is ignored in the backward as in the forward
    assert_close(dzb, wantb, "dense CE backward with an out-of-range target")
    # the chunked path (two spans of 6): the first statistics pass notes the row, loss and gradient ignore it
    brm, brs, btl = (gpu.create_state_buffer(rows * 4) for _ in range(3))
    bl2 = gpu.create_state_buffer(4)
    chunks = [np.ascontiguousarray(z[:, v0:v0 + 6]) for v0 in (0, 6)]
    bch = [dev(gpu, c) for c in chunks]
    for i, v0 in enumerate((0, 6)):
        lib.check(gpu.ctx, L.gt_ce_chunk_stats(gpu.ctx, rows, Vc, 6, v0, 1 if i == 0 else 0, bch[i], btg, brm, brs, btl), "stats")
    lib.check(gpu.ctx, L.gt_ce_loss_from_stats(gpu.ctx, rows, Vc, rows, btg, binv, brm, brs, btl, bl2), "loss")
    assert "cross-entropy target 12 at row 2 is outside [-1, 12)" in sync_error()
    assert abs(gpu.read_state_buffer(bl2, 1)[0] - want) <= 1e-5 * abs(want)
    for i, v0 in enumerate((0, 6)):
        lib.check(gpu.ctx, L.gt_ce_chunk_grad(gpu.ctx, rows, Vc, 6, v0, rows, bch[i], btg, binv, brm, brs, 1.0), "grad")
        assert_close(gpu.read_state_buffer(bch[i], rows * 6).reshape(rows, 6), wantb[:, v0:v0 + 6], f"chunked CE gradient, span {i}")
    assert sync_error() == ""
    rc = L.gt_ce_chunk_stats(gpu.ctx, rows, Vc, 8, 6, 0, bch[1], btg, brm, brs, btl)      # span [6, 14) of 12 logits
    assert rc != 0 and "span [6, 14) of 12" in L.gt_last_error(gpu.ctx).decode()

    k = 2
    tid = np.array([1, 2, -1, 0, 3, 40, 4, 4], np.int32)         # row 2: second teacher id 40 >= V
    tq = np.array([0.5, 0.5, 0, 0, 0.6, 0.4, 0.3, 0.3], np.float32)
    btid, btq = dev(gpu, tid), dev(gpu, tq)
    bmass = gpu.create_state_buffer(rows * 4)
    lib.check(gpu.ctx, L.gt_soft_ce_fwd(gpu.ctx, rows, Vc, k, bz, btid, btq, 1.0 / 3, bloss, blse, bmass), "softce")
    assert "teacher id 40 at row 2 is outside [0, 12)" in sync_error()
    lib.check(gpu.ctx, L.gt_soft_ce_bwd(gpu.ctx, rows, Vc, k, bz, btid, btq, 1.0 / 3, blse, bmass, 1.0, bdz, 0), "softce.bwd")
    assert "teacher id 40 at row 2" in sync_error()
    dz = gpu.read_state_buffer(bdz, rows * Vc).reshape(rows, Vc)
    p = np.exp(z64 - lse[:, None])
    want2 = (0.6 * p[2]) / 3                                     # the bad slot's mass and term are dropped
    want2[3] -= 0.6 / 3
    assert_close(dz[2], want2, "softCE row with a skipped teacher")
    assert sync_error() == ""
