"""Central finite differences ON THE DEVICE path, independent of the CPU oracle: the recipe of
tests/gpu-parity.ts:241-300 (which applies it to `linear` only) and tests/gradcheck.ts:100-168: loss = sum(out * r)
with r ~ U(-1,1) from mulberry32(0xbeef), step 1e-2 with the difference divided by the f32-rounded step actually
taken, sampled elements from mulberry32(0xcafe), |fd - g| <= 2e-3 + 1.5e-2 max(|fd|, |g|). Every op of the backend
interface goes through it, so a kernel and the oracle sharing a wrong formula would still be caught here."""
import math

import numpy as np
import pytest

from gpu_common import backward_from, mod

pytestmark = pytest.mark.gpu

EPS = 1e-2
PICKS = 6


def fd_case(gpu, ref, arrays, fwd, what, skip=(), picks=PICKS):
    ag = mod("autograd")
    ts = [ag.Tensor(a, list(a.shape), True) for a in arrays]
    gpu.install()
    try:
        out0 = fwd(ag, *ts)
        r = ref.Mulberry32(0xBEEF).fill_uniform([out0.size])
        backward_from(gpu, ag, out0, r)
        gpu.sync([out0])
        analytic = [t.grad.copy() for t in ts]

        def loss():
            out = fwd(ag, *ts)
            gpu.sync([out])
            return float(np.dot(out.data.astype(np.float64), r.astype(np.float64)))

        pick = ref.Mulberry32(0xCAFE)
        bad = []
        for k, t in enumerate(ts):
            if k in skip:
                continue
            for _ in range(picks):
                i = int(math.floor(pick() * t.size))
                orig = t.data[i]
                xp, xm = np.float32(orig + np.float32(EPS)), np.float32(orig - np.float32(EPS))
                t.data[i] = xp
                gpu.upload_params([t])
                lp = loss()
                t.data[i] = xm
                gpu.upload_params([t])
                lm = loss()
                t.data[i] = orig
                gpu.upload_params([t])
                fd = (lp - lm) / (float(xp) - float(xm))
                g = float(analytic[k][i])
                if abs(fd - g) > 2e-3 + 1.5e-2 * max(abs(fd), abs(g)):
                    bad.append((k, i, g, fd))
        assert not bad, f"{what}: analytic vs finite difference {bad}"
    finally:
        gpu.uninstall()
        gpu.sync([])


def R(ref, seed):
    r = ref.Mulberry32(seed)
    return lambda *s, scale=0.8: r.fill_randn(list(s), scale)


def test_fd_linear_reference_case(gpu, ref):
    """gpu-parity.ts:241-300: x [5,7], w [6,7] from mulberry32(31337), 6 sampled elements per tensor."""
    g = R(ref, 31337)
    fd_case(gpu, ref, [g(5, 7), g(6, 7)], lambda ag, x, w: ag.linear(x, w), "linear 5x7 . 6x7^T")


def test_fd_linear_tiled_and_split_k(gpu, ref):
    g = R(ref, 1)
    fd_case(gpu, ref, [g(70, 83), g(75, 83)], lambda ag, x, w: ag.linear(x, w), "linear 70x83 . 75x83^T")
    fd_case(gpu, ref, [g(700, 24, scale=0.3), g(16, 24)], lambda ag, x, w: ag.linear(x, w), "linear, long-K dW")


def test_fd_elementwise(gpu, ref):
    g = R(ref, 2)
    fd_case(gpu, ref, [g(9, 13), g(9, 13)], lambda ag, a, b: ag.add(a, b), "add")
    fd_case(gpu, ref, [g(9, 13), g(9, 13)], lambda ag, a, b: ag.mul(a, b), "mul")
    fd_case(gpu, ref, [g(9, 13)], lambda ag, x: ag.silu(x), "silu")
    fd_case(gpu, ref, [g(9, 13)], lambda ag, x: ag.gelu(x), "gelu")
    fd_case(gpu, ref, [g(9, 13)], lambda ag, x: ag.scale(x, 2.5), "scale")
    fd_case(gpu, ref, [g(9, 13), g(9, 13)], lambda ag, a, b: ag.mul(ag.silu(a), b), "SwiGLU (fused backward)")
    fd_case(gpu, ref, [g(9, 13), g(9, 13)], lambda ag, a, b: ag.mul(ag.gelu(a), b), "GeGLU (fused backward)")
    fd_case(gpu, ref, [g(9, 13)], lambda ag, x: ag.mul(x, x), "mul(t, t)")


def test_fd_norms(gpu, ref):
    g = R(ref, 3)
    fd_case(gpu, ref, [g(11, 24), 1 + 0.3 * g(24)], lambda ag, x, w: ag.rms_norm(x, w, 1e-6), "rmsNorm")
    fd_case(gpu, ref, [g(7, 3 * 16), 1 + 0.3 * g(16)], lambda ag, x, w: ag.rms_norm_heads(x, w, 7, 3, 16, 1e-6), "rmsNormHeads")
    fd_case(gpu, ref, [g(5, 4 * 64), 1 + 0.3 * g(64)], lambda ag, x, w: ag.rms_norm_heads(x, w, 5, 4, 64, 1e-6), "rmsNormHeads hd 64")


def test_fd_embedding_and_rope(gpu, ref):
    g = R(ref, 4)
    fd_case(gpu, ref, [g(10, 12)], lambda ag, w: ag.embedding(w, [3, 1, 3, 9, 0, 3]), "embedding (repeated ids)", picks=12)
    fd_case(gpu, ref, [g(9, 2 * 16)], lambda ag, x: ag.rope(x, 9, 2, 16, 10000.0), "rope")
    fd_case(gpu, ref, [g(9, 2 * 16)], lambda ag, x: ag.rope(x, 9, 2, 16, 1e6, 5), "rope (posOffset 5)")


@pytest.mark.parametrize("T,Hq,Hkv,hd,window", [(19, 4, 2, 8, 0), (19, 4, 2, 8, 5), (70, 2, 1, 64, 0), (70, 2, 1, 64, 33),
                                                  (40, 2, 2, 128, 0), (150, 3, 1, 64, 0), (90, 4, 2, 32, 0), (90, 4, 2, 32, 40)])
def test_fd_attention(gpu, ref, T, Hq, Hkv, hd, window):
    """Generic kernels (hd 8) and the matrix-core kernels (hd 32 / 64 / 128), GQA, full causal and windowed."""
    g = R(ref, 5 + T + hd)
    fd_case(gpu, ref, [g(T, Hq * hd, scale=0.6), g(T, Hkv * hd, scale=0.6), g(T, Hkv * hd)],
            lambda ag, q, k, v: ag.attention(q, k, v, T, Hq, Hkv, hd, window), f"attention T={T} {Hq}/{Hkv}x{hd} w={window}")


def test_fd_attention_split_tiles(gpu, ref):
    """The same check with every attention tile cut into three workgroups (partials folded by a second kernel)."""
    g = R(ref, 77)
    T, Hq, Hkv, hd = 200, 2, 1, 64
    gpu.set_option("attn.splits", 3)
    try:
        fd_case(gpu, ref, [g(T, Hq * hd, scale=0.6), g(T, Hkv * hd, scale=0.6), g(T, Hkv * hd)],
                lambda ag, q, k, v: ag.attention(q, k, v, T, Hq, Hkv, hd, 0), "attention, 3 splits")
    finally:
        gpu.set_option("attn.splits", -1)


def test_fd_losses(gpu, ref):
    g = R(ref, 6)
    tg = [3, -1, 0, 299, 7, -1, 12]
    fd_case(gpu, ref, [g(7, 300, scale=2.0)], lambda ag, z: ag.cross_entropy(z, tg), "crossEntropy (ignore-index, V > 256)")
    fd_case(gpu, ref, [g(7, 24), g(300, 24, scale=0.3)], lambda ag, h, w: ag.fused_cross_entropy(h, w, tg, 128), "fusedCrossEntropy, 3 chunks")
    fd_case(gpu, ref, [g(7, 24), g(300, 24, scale=0.3)], lambda ag, h, w: ag.cross_entropy(ag.linear(h, w), tg), "CE(linear)")
    K = 3
    ids = [(5 * i + j * 17) % 300 for i in range(7) for j in range(K)]
    pr = ref.Mulberry32(9).fill_uniform([7 * K], 0.05, 1.0).reshape(7, K)
    pr[2] = 0                                            # an all-pad row
    pr[4, 1] = 0                                         # a zero-weight pad inside a row
    s = pr.sum(1, keepdims=True)
    pr = np.where(s > 0, pr / np.where(s > 0, s, 1), 0).astype(np.float32)
    fd_case(gpu, ref, [g(7, 300, scale=2.0)], lambda ag, z: ag.soft_cross_entropy(z, ids, pr.ravel().tolist(), K), "softCrossEntropy")


def test_fd_lora_linear(gpu, ref):
    """autograd.ts:311-319 as the backend records it (one op, two-segment GEMMs): x, A and B by finite differences;
    the frozen base takes no gradient."""
    ag = mod("autograd")
    g = R(ref, 8)
    w = ag.Tensor(g(20, 24), [20, 24], False)
    arrays = [g(9, 24), g(4, 24, scale=0.3), g(20, 4, scale=0.3)]

    def fwd(ag_, x, a, b):
        ag_.set_lora_adapters({id(w): (a, b, 2.0)})
        try:
            return ag_.linear(x, w)
        finally:
            ag_.set_lora_adapters(None)
    fd_case(gpu, ref, arrays, fwd, "LoRA linear")
