"""Whole-graph parity: the three architectures, micro-batch accumulation, --recompute, LoRA, stacked
sequences and benchmark config 1, HIP backend (through the C ABI) against the CPU oracle."""
import math

import numpy as np
import pytest

from gpu_common import LOSS_REL, assert_close, backward_from, mod

pytestmark = pytest.mark.gpu

SMALL = {
    "llama": dict(arch="llama", vocab=61, hidden=48, layers=2, heads=6, kv_heads=2, head_dim=8, ffn=80, rope_base=1e5),
    "qwen3": dict(arch="qwen3", vocab=61, hidden=48, layers=2, heads=4, kv_heads=2, head_dim=16, ffn=80, rope_base=1e6, rms_eps=1e-6),
    "gemma3": dict(arch="gemma3", vocab=61, hidden=48, layers=3, heads=4, kv_heads=1, head_dim=16, ffn=80, rope_base=1e6,
                   rope_base_local=1e4, sliding_window=7, swa_pattern=3, rms_eps=1e-6),
}
# benchmark config 1
TINY = dict(arch="llama", vocab=512, hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=352, rope_base=1e4, rms_eps=1e-5)


def build_pair(ref, kw, seed=0, std=0.02, jitter_gains=True):
    arch = mod("arch")
    rmodel = ref.Model(ref.ModelConfig(**kw), ref.Mulberry32(seed), std=std)
    if jitter_gains:
        rng = ref.Mulberry32(seed + 100)
        for p in rmodel.params():
            if len(p.shape) == 1:
                p.data[:] = 1 + 0.2 * rng.fill_randn([p.size])
    weights = {n: p.data.copy() for n, p in rmodel.named_params()}
    return rmodel, arch.Model(arch.ModelConfig(**kw), weights)


def batches(ref, vocab, T, n, seed, mask_every=0):
    rng = ref.Mulberry32(seed)
    out = []
    for _ in range(n):
        ids = [int(rng() * vocab) for _ in range(T + 1)]
        tg = ids[1:]
        if mask_every:
            tg = [-1 if i % mask_every == 2 else g for i, g in enumerate(tg)]
        out.append((ids[:-1], tg))
    return out


def hip_step(gpu, model, seqs, stacked, seq_len, loss_chunk=0, recompute=False):
    ag, arch = mod("autograd"), mod("arch")
    B = len(seqs)
    gpu.install()
    ag.set_checkpointing(recompute)
    try:
        losses = []
        if stacked:
            ids = np.concatenate([s[0] for s in seqs])
            tg = np.concatenate([s[1] for s in seqs])
            loss = arch.sequence_loss(model, ids, tg, loss_chunk, seq_len)
            ag.backward(loss, 1.0 / B)
            losses = [loss]
        else:
            for ids, tg in seqs:
                loss = arch.sequence_loss(model, ids, tg, loss_chunk)
                ag.backward(loss, 1.0 / B)
                losses.append(loss)
        gpu.sync(losses)
    finally:
        ag.set_checkpointing(False)
        gpu.uninstall()
    lv = np.concatenate([l.data for l in losses])
    return lv, {n: p.grad.copy() for n, p in model.named_params()}


def ref_step(ref, rmodel, seqs, loss_chunk=0):
    B = len(seqs)
    for p in rmodel.params():
        p.zero_grad()
    lv = []
    for ids, tg in seqs:
        l = ref.sequence_loss(rmodel, ids, tg, loss_chunk)
        ref.backward(l, 1.0 / B)
        lv.append(float(l.data[0]))
    return np.array(lv), {n: p.grad.copy() for n, p in rmodel.named_params()}


def compare(lh, gh, lr, gr, what):
    assert np.all(np.abs(lh - lr) <= LOSS_REL * np.abs(lr)), f"{what}: loss {lh} vs {lr}"
    for n in gr:
        assert_close(gh[n], gr[n], f"{what} grad {n}")


@pytest.mark.parametrize("arch_name", ["llama", "qwen3", "gemma3"])
@pytest.mark.parametrize("stacked", [False, True])
def test_whole_model_two_micro_batches(gpu, ref, arch_name, stacked):
    """gpu-parity.ts:333-428: loss and every gradient tensor; two micro-batches accumulated with seed 1/2, masked
    targets; the same step as one stacked graph over 2*T rows."""
    kw = SMALL[arch_name]
    rmodel, model = build_pair(ref, kw, seed=1, std=0.1)
    seqs = batches(ref, kw["vocab"], 19, 2, seed=5, mask_every=5)
    lh, gh = hip_step(gpu, model, seqs, stacked, 19)
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(lh, gh, lr, gr, f"{arch_name} stacked={stacked}")


REAL = {
    # SmolLM2-135M layer geometry (9/3 heads x 64, hidden 576, SwiGLU 1536), two layers, reduced vocabulary
    "smollm2": dict(arch="llama", vocab=4096, hidden=576, layers=2, heads=9, kv_heads=3, head_dim=64, ffn=1536,
                    rope_base=1e5, rms_eps=1e-5),
    # Qwen3 head layout: head dim 128 with QK-norm, GQA 4/2
    "qwen3-hd128": dict(arch="qwen3", vocab=2048, hidden=256, layers=2, heads=4, kv_heads=2, head_dim=128, ffn=512,
                        rope_base=1e6, rms_eps=1e-6),
    # tests/qwen3-wide-heads.ts:30-43: the attention block wider than the model (16 heads of 128 over a width of 544)
    "qwen3-wide": dict(arch="qwen3", vocab=1024, hidden=544, layers=1, heads=16, kv_heads=8, head_dim=128, ffn=2560,
                       rope_base=1e6, rms_eps=1e-6),
    # Gemma3: GeGLU, sliding window that cuts the 128-row attention tiles, one global layer in three
    "gemma3-window": dict(arch="gemma3", vocab=2048, hidden=320, layers=3, heads=5, kv_heads=1, head_dim=64, ffn=768,
                          rope_base=1e6, rope_base_local=1e4, sliding_window=96, swa_pattern=3, rms_eps=1e-6),
}


@pytest.mark.parametrize("name", sorted(REAL))
@pytest.mark.parametrize("stacked", [False, True])
def test_whole_model_real_head_geometry(gpu, ref, name, stacked):
    """The shapes the tuned kernels are built for, inside whole graphs: matrix-core attention (head dims 64 and 128, GQA,
    windows), the large GEMM tiles with split-K dW, row lengths of 576 / 1536 in the normalisation and gated-activation
    kernels. Two sequences of 200 tokens (ragged against every tile size), masked targets, loss and every gradient."""
    kw = REAL[name]
    rmodel, model = build_pair(ref, kw, seed=11, std=0.05)
    seqs = batches(ref, kw["vocab"], 200, 2, seed=12, mask_every=7)
    lh, gh = hip_step(gpu, model, seqs, stacked, 200)
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        lr, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    compare(lh, gh, lr, gr, f"{name} stacked={stacked}")


@pytest.mark.parametrize("arch_name", ["llama", "qwen3", "gemma3"])
def test_recompute_is_bit_identical_and_matches(gpu, ref, arch_name):
    """gpu-parity.ts:536-564, 1299-1338: --recompute on/off gives bit-identical loss and gradients."""
    kw = SMALL[arch_name]
    seqs = batches(ref, kw["vocab"], 23, 2, seed=6, mask_every=4)
    res = []
    for rc in (False, True):
        rmodel, model = build_pair(ref, kw, seed=2, std=0.1)
        regions0 = gpu.region_count()
        res.append(hip_step(gpu, model, seqs, False, 23, recompute=rc))
        if rc:
            assert gpu.region_count() > regions0
    assert res[0][0].tobytes() == res[1][0].tobytes()
    for n in res[0][1]:
        assert res[0][1][n].tobytes() == res[1][1][n].tobytes(), n
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(res[1][0], res[1][1], lr, gr, f"{arch_name} recompute")


def test_run_to_run_determinism(gpu, ref):
    kw = SMALL["llama"]
    seqs = batches(ref, kw["vocab"], 40, 3, seed=9)
    a = hip_step(gpu, build_pair(ref, kw, seed=3, std=0.1)[1], seqs, True, 40)
    b = hip_step(gpu, build_pair(ref, kw, seed=3, std=0.1)[1], seqs, True, 40)
    assert a[0].tobytes() == b[0].tobytes()
    for n in a[1]:
        assert a[1][n].tobytes() == b[1][n].tobytes(), n


@pytest.mark.parametrize("chunk", [16, 61])
def test_loss_chunk_path(gpu, ref, chunk):
    """gpu-parity.ts:438-565: --loss-chunk gives the dense loss and gradients."""
    kw = SMALL["qwen3"]
    rmodel, model = build_pair(ref, kw, seed=4, std=0.1)
    seqs = batches(ref, kw["vocab"], 17, 2, seed=7, mask_every=6)
    lh, gh = hip_step(gpu, model, seqs, False, 17, loss_chunk=chunk)
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(lh, gh, lr, gr, f"loss-chunk {chunk}")


@pytest.mark.parametrize("recompute", [False, True])
def test_lora(gpu, ref, recompute):
    """gpu-parity.ts:2037-2138: base frozen (no gradient buffers), adapters trained; with --recompute too."""
    ag, arch = mod("autograd"), mod("arch")
    kw = SMALL["qwen3"]
    rmodel, model = build_pair(ref, kw, seed=5, std=0.1)
    rank, alpha = 4, 8.0
    rmap, rparams = ref.attach_lora(rmodel, rank, alpha, ref.Mulberry32(11), a_std=0.1)
    rng = ref.Mulberry32(12)
    for a, b, _ in rmap.values():
        b.data[:] = rng.fill_randn([b.size], 0.1)          # B != 0 so that dA is non-trivial
    adapters = {}
    for l, L in enumerate(rmodel.layers):
        for k in ref.MATRIX_KEYS:
            a, b, _ = rmap[id(L[k])]
            adapters[f"L{l}.{k}"] = (a.data.copy(), b.data.copy())
    aux = arch.apply_lora(model, rank, alpha, adapters)
    ref.set_lora_adapters(rmap)
    seqs = batches(ref, kw["vocab"], 15, 2, seed=8, mask_every=3)
    try:
        lh, _ = hip_step(gpu, model, seqs, False, 15, recompute=recompute)
        lr, _ = ref_step(ref, rmodel, seqs)
    finally:
        ref.set_lora_adapters({})
        arch.clear_lora(model)
    assert np.all(np.abs(lh - lr) <= LOSS_REL * np.abs(lr))
    for i, (h, r) in enumerate(zip(aux, rparams)):
        assert_close(h.grad, r.grad, f"lora adapter {i}")
    for p in model.params():                                 # frozen base: no accumulator was ever created
        assert gpu._entries[p].grad == 0


def test_lora_adapter_gradient_sums_held_back(gpu, ref):
    """Sequences long enough for the rank-r gradient products to go through row slices (300 tokens): the host holds the
    slice sums of a backward pass back and adds them up in grouped launches. Same bits as summing each at once, parity
    with the oracle, stacked and one sequence at a time (where the sums go out before the stream changes)."""
    ag, arch = mod("autograd"), mod("arch")
    kw = SMALL["qwen3"]
    rank, alpha = 4, 8.0

    def build():
        rmodel, model = build_pair(ref, kw, seed=5, std=0.1)
        rmap, rparams = ref.attach_lora(rmodel, rank, alpha, ref.Mulberry32(11), a_std=0.1)
        rng = ref.Mulberry32(12)
        for a, b, _ in rmap.values():
            b.data[:] = rng.fill_randn([b.size], 0.1)
        adapters = {}
        for l, L in enumerate(rmodel.layers):
            for k in ref.MATRIX_KEYS:
                a, b, _ = rmap[id(L[k])]
                adapters[f"L{l}.{k}"] = (a.data.copy(), b.data.copy())
        return rmodel, model, rmap, rparams, arch.apply_lora(model, rank, alpha, adapters)

    seqs = batches(ref, kw["vocab"], 300, 3, seed=9, mask_every=4)
    rmodel, model, rmap, rparams, aux = build()
    ref.set_lora_adapters(rmap)
    try:
        lr, _ = ref_step(ref, rmodel, seqs)
    finally:
        ref.set_lora_adapters({})
    want = [r.grad.copy() for r in rparams]
    held = []
    flush = gpu._flush_rs

    def counting_flush():
        if gpu._pend_rs:
            held.append(len(gpu._pend_rs))
        flush()

    gpu._flush_rs = counting_flush
    got = {}
    try:
        for stacked in (True, False):
            for defer in (True, False):
                _, model, _, _, aux = build()
                gpu.defer_rank_sums = defer
                held.clear()
                try:
                    lh, _ = hip_step(gpu, model, seqs, stacked, 300)
                finally:
                    arch.clear_lora(model)
                assert (len(held) > 0) == defer, (stacked, defer, held)
                if defer:
                    assert sum(held) >= 2 * (1 if stacked else len(seqs)), held      # (the products whose K the streaming kernel takes)
                got[(stacked, defer)] = [h.grad.copy() for h in aux]
                if not stacked:
                    assert np.all(np.abs(lh - lr) <= LOSS_REL * np.abs(lr))
                for i, (h, w) in enumerate(zip(aux, want)):
                    assert_close(h.grad, w, f"lora adapter {i}, stacked {stacked}, held back {defer}")
    finally:
        gpu.defer_rank_sums = True
        gpu._flush_rs = flush
    for stacked in (True, False):
        for a, b in zip(got[(stacked, True)], got[(stacked, False)]):
            assert a.tobytes() == b.tobytes(), f"held-back sums change bits (stacked {stacked})"


def test_config1_tiny_llama_step(gpu, ref):
    """benchmark config 1: vocab 512, hidden 128, 2 layers, 4/2 heads x 32, SwiGLU 352, tied, weights N(0,0.02) seed 0,
    4 sequences of 128 tokens, targets shifted by one; forward + backward + AdamW(lr 1e-3, betas 0.9/0.95, wd 0.1)."""
    optim = mod("optim")
    clears0 = gpu.grad_clears_issued
    rmodel, model = build_pair(ref, TINY, seed=0, std=0.02, jitter_gains=False)
    seqs = batches(ref, TINY["vocab"], 128, 4, seed=0)
    ref.set_threads(min(8, ref.max_threads()))
    try:
        lr_, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.set_threads(1)
    opt = optim.AdamWHip(gpu, model.params(), lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0)
    ag, arch = mod("autograd"), mod("arch")
    gpu.install()
    try:
        ids = np.concatenate([s[0] for s in seqs])
        tg = np.concatenate([s[1] for s in seqs])
        loss = arch.sequence_loss(model, ids, tg, 0, 128)
        ag.backward(loss, 0.25)
        gpu.sync([loss])
        gh = {n: gpu.read_state_buffer(gpu.buffers_for(p)["grad"], p.size) for n, p in model.named_params()}
        opt.record_step()
        gpu.sync([])
        opt.sync_weights_to_host()
    finally:
        gpu.uninstall()
    compare(loss.data.copy(), gh, lr_, gr, "config 1")
    ropt = ref.AdamW(rmodel.params(), lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0)
    ropt.step()
    # The first Adam step is g/(|g|+eps): where |g| is near eps = 1e-8 the update turns rounding noise in g (1e-9
    # absolute, far inside the gradient tolerance) into O(lr) differences in w. Gradients are held to 1e-5 above;
    # the weights to 1e-4 relative L2 / 5e-3 max-rel. Identical gradients give 1e-5 (test_gpu_optim.py).
    for n, p in rmodel.named_params():
        assert_close(model.p[n].data, p.data, f"config 1 weight after AdamW {n}", rel_l2=1e-4, max_rel=5e-3)
    # first-writer stores: one clear per parameter accumulator when the optimizer allocates it, none per tape node
    assert gpu.grad_clears_issued - clears0 <= len(model.params())


def test_device_behaviour_gates(gpu, ref):
    """gpu-parity.ts:1363-2028: after warm-up a device-resident step reads back the loss scalars only, issues no
    gradient clears, stops allocating (the pool plateaus), and a stacked step uses B times fewer launches' worth of
    regions than the sequential one when recomputing."""
    optim, train = mod("optim"), mod("train")
    kw = SMALL["llama"]
    _, model = build_pair(ref, kw, seed=7, std=0.1)
    seqs = batches(ref, kw["vocab"], 32, 12, seed=11)
    opt = optim.AdamWHip(gpu, model.params(), lr=1e-3)
    times, flush = [], []

    def on_step_time(fwd_bwd, opt_time, readback):
        times.append(readback)
        flush.append(gpu.last_sync_readback_bytes)
    train.train_lm_hip_resident(model, gpu, opt, seqs[:4], 2, 2, 32, stacked=True, on_step_time=on_step_time)
    clears0, res0 = gpu.grad_clears_issued, gpu.resident_bytes()
    pool0 = gpu._pool_bytes
    train.train_lm_hip_resident(model, gpu, opt, seqs[4:], 4, 2, 32, stacked=True, on_step_time=on_step_time)
    assert gpu.grad_clears_issued == clears0            # first-writer stores: nothing to clear per step
    assert gpu._pool_bytes == pool0 and gpu.resident_bytes() == res0   # no allocation after warm-up
    assert all(rb == 8 for rb in times)                 # the step's sync reads back one f32 loss per sequence, no gradient
    assert all(rb == 0 for rb in flush)                 # the optimizer-flush sync reads nothing back
    # the loss sync itself: one f32 per sequence
    ag, arch = mod("autograd"), mod("arch")
    gpu.install()
    try:
        ids = np.concatenate([s[0] for s in seqs[:2]])
        tg = np.concatenate([s[1] for s in seqs[:2]])
        loss = arch.sequence_loss(model, ids, tg, 0, 32)
        ag.backward(loss, 0.5)
        gpu.sync([loss])
        assert gpu.last_sync_readback_bytes == 8
    finally:
        gpu.uninstall()
        gpu.sync([])


def test_single_row_and_single_token_edges(gpu, ref):
    """T = 1 (one query sees one key), one-row GEMMs, a one-token vocabulary span: the ragged-edge guards."""
    from gpu_common import op_case
    r = ref.Mulberry32(5)
    R = lambda *s: r.fill_randn(list(s), 0.8)
    op_case(gpu, ref, [R(1, 64), R(1, 64), R(1, 64)], lambda ag, q, k, v: ag.attention(q, k, v, 1, 1, 1, 64, 0),
            lambda rf, q, k, v: rf.attention(q, k, v, 1, 1, 1, 64, 0), "attention T=1", floor=1.0)
    op_case(gpu, ref, [R(1, 7), R(1, 7)], lambda ag, x, w: ag.linear(x, w), lambda rf, x, w: rf.linear(x, w), "linear 1x7x1")
    op_case(gpu, ref, [R(1, 5)], lambda ag, z: ag.cross_entropy(z, [4]), lambda rf, z: rf.cross_entropy(z, [4]), "CE one row")
    op_case(gpu, ref, [R(3, 1)], lambda ag, z: ag.cross_entropy(z, [0, -1, 0]), lambda rf, z: rf.cross_entropy(z, [0, -1, 0]),
            "CE one-logit vocabulary", floor=1.0)
    w = 1 + 0.3 * R(4)
    op_case(gpu, ref, [R(1, 4), w], lambda ag, x, g: ag.rms_norm(x, g, 1e-6), lambda rf, x, g: rf.rms_norm(x, g, 1e-6), "rmsNorm one row")
    op_case(gpu, ref, [R(5, 3)], lambda ag, e: ag.embedding(e, [4]), lambda rf, e: rf.embedding(e, [4]), "embedding one id")


@pytest.mark.parametrize("loss_chunk", [0, 64])
def test_forward_only_scoring_reads_back_the_loss_alone(gpu, ref, loss_chunk):
    """gpu-parity.ts:1430-1495 (eval freeze gate), for this backend's protocol: a scoring pass (forward, sync, no
    backward) stages back the loss scalar and nothing else whether or not the parameters are frozen, allocates no
    gradient accumulator in either arm (they are created by the first backward write), and freezing moves no bit of
    the score."""
    ag, arch = mod("autograd"), mod("arch")
    kw = dict(arch="gemma3", vocab=64, hidden=64, layers=4, heads=4, kv_heads=2, head_dim=16, ffn=256, rope_base=1e6,
              rope_base_local=1e4, sliding_window=16, swa_pattern=2, rms_eps=1e-6)
    ids = np.array([(i * 11 + 5) % 64 for i in range(65)])
    out = {}
    for freeze in (False, True):
        _, model = build_pair(ref, kw, seed=5, std=0.05)
        if freeze:
            for p in model.params():
                p.requires_grad = False
        gpu.install()
        try:
            gpu.upload_params(model.params())
            clears = gpu.grad_clears_issued
            loss = arch.sequence_loss(model, ids[:-1], ids[1:], loss_chunk)
            gpu.sync([loss])
            assert gpu.grad_clears_issued == clears        # a forward-only window zeroes nothing (gpu-parity.ts:1825-1950)
            out[freeze] = (gpu.last_sync_readback_bytes, float(loss.data[0]),
                           sum(1 for p in model.params() if gpu._entries[p].grad != 0))
        finally:
            gpu.uninstall()
            gpu.sync([])
    assert out[False][0] == 4 and out[True][0] == 4, out
    assert out[False][2] == 0 and out[True][2] == 0, out
    assert out[False][1] == out[True][1] and np.isfinite(out[True][1])


@pytest.mark.parametrize("recompute", [False, True])
def test_kept_attention_scores_policy(gpu, ref, recompute):
    """The host keeps attention's scores from the forward to the backward only where a backward can come: a trainable
    model takes one scores buffer per layer (recomputed layers: one at a time, and none in the discarded first pass), a
    model frozen for scoring takes none; with and without them the step gives the same loss bits and gradients to the
    parity bound, and both agree with the oracle."""
    kw = dict(arch="qwen3", vocab=97, hidden=128, layers=3, heads=2, kv_heads=1, head_dim=64, ffn=192, rope_base=1e6, rms_eps=1e-6)
    T, B = 128, 2
    per_call = B * kw["heads"] * T * T * 4
    rmodel, model = build_pair(ref, kw, seed=21, std=0.05)
    seqs = batches(ref, kw["vocab"], T, B, seed=22, mask_every=6)
    taken = []
    acquire = gpu._acquire

    def spy(nbytes, *stream):
        taken.append(nbytes)
        return acquire(nbytes, *stream)

    gpu._acquire = spy
    res = {}
    try:
        for keep in (True, False):
            gpu.attn_keep_scores = keep
            taken.clear()
            res[keep] = hip_step(gpu, model, seqs, True, T, recompute=recompute)
            assert taken.count(per_call) == (kw["layers"] if keep else 0), (keep, taken.count(per_call))
            assert gpu._scores_taken == 0
        gpu.attn_keep_scores = True
        for p in model.params():
            p.requires_grad = False
        taken.clear()
        gpu.install()
        try:
            loss = mod("arch").sequence_loss(model, np.concatenate([s[0] for s in seqs]), np.concatenate([s[1] for s in seqs]), 0, T)
            gpu.sync([loss])
        finally:
            gpu.uninstall()
        assert taken.count(per_call) == 0
        assert np.array_equal(loss.data, res[True][0])
    finally:
        gpu._acquire = acquire
        gpu.attn_keep_scores = True
        for p in model.params():
            p.requires_grad = True
    assert np.array_equal(res[True][0], res[False][0])
    for n in res[True][1]:
        assert_close(res[True][1][n], res[False][1][n], f"kept scores vs recomputed, grad {n}")
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(res[True][0], res[True][1], lr, gr, f"kept scores recompute={recompute}")


def test_sibling_input_gradients_leave_as_one_product(gpu, ref):
    """The dX of linears that share their input is held back and sent as one summed product (q/k/v, gate/up). Same
    gradients as one accumulating product per linear to the parity bound, against the oracle too, and fewer NN launches:
    per layer q+k+v -> 1 and gate+up -> 1."""
    kw = dict(arch="llama", vocab=64, hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=256, rope_base=1e4, rms_eps=1e-5)
    rmodel, model = build_pair(ref, kw, seed=31, std=0.05)
    seqs = batches(ref, kw["vocab"], 64, 2, seed=32, mask_every=5)
    res, launches = {}, {}
    gpu.set_option("gemm.sum_min_tiles", 0)        # 128 rows: below the size from which the library chains the products
    try:
        for fuse in (True, False):
            gpu.fuse_sibling_dx = fuse
            gpu.start_profile("gemm.nn")
            res[fuse] = hip_step(gpu, model, seqs, True, 64)
            launches[fuse] = sum(v[1] for v in gpu.stop_profile().values())
    finally:
        gpu.fuse_sibling_dx = True
        gpu.set_option("gemm.sum_min_tiles", -1)
    assert launches[False] - launches[True] == kw["layers"] * 3, launches      # (3 - 1) + (2 - 1) per layer
    assert np.array_equal(res[True][0], res[False][0])
    for n in res[True][1]:
        assert_close(res[True][1][n], res[False][1][n], f"fused vs separate dX, grad {n}")
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(res[True][0], res[True][1], lr, gr, "fused sibling dX")


def test_held_back_input_gradient_keeps_the_order_of_writers(gpu, ref):
    """x feeds two linears, an elementwise op and a third linear further on: whoever writes or reads dx while products
    into it are held back sends them first. Against the oracle, with the elementwise consumer before, between and after."""
    ag = mod("autograd")
    r = ref.Mulberry32(77)
    T, d = 70, 64
    xa = r.fill_randn([T, d], 0.8)
    ws = [r.fill_randn([d, d], 0.3) for _ in range(3)]
    up = r.fill_uniform([T * d])

    def graph(m, x, w1, w2, w3, order):
        parts = {"a": lambda: m.linear(x, w1), "b": lambda: m.linear(x, w2), "e": lambda: m.mul(x, x)}
        t = [parts[k]() for k in order]
        y = m.add(m.add(t[0], t[1]), t[2])
        return m.add(m.linear(m.silu(y), w3), x)

    for order in ("abe", "aeb", "eab"):
        hx, rx = ag.Tensor(xa, [T, d], True), ref.Tensor(xa, [T, d], True)
        hw = [ag.Tensor(w, [d, d], True) for w in ws]
        rw = [ref.Tensor(w, [d, d], True) for w in ws]
        gpu.install()
        try:
            out = graph(ag, hx, *hw, order)
            from gpu_common import backward_from
            backward_from(gpu, ag, out, up)
            gpu.sync([out])
        finally:
            gpu.uninstall()
        rout = graph(ref, rx, *rw, order)
        ref.backward_from(rout, up)
        assert_close(out.data, rout.data, f"{order} forward")
        assert_close(hx.grad, rx.grad, f"{order} dx")
        for i, (h, rr) in enumerate(zip(hw, rw)):
            assert_close(h.grad, rr.grad, f"{order} dw{i}")


def test_residual_add_rides_the_linear_launch(gpu, ref):
    """h + linear(x, W) leaves as one launch (the product is added to h in the GEMM's write-back): every bit of the loss
    and of every gradient is what the linear and the add as two launches give, with two add launches fewer per layer."""
    kw = dict(arch="llama", vocab=64, hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=256, rope_base=1e4, rms_eps=1e-5)
    _, model = build_pair(ref, kw, seed=41, std=0.05)
    seqs = batches(ref, kw["vocab"], 50, 2, seed=42, mask_every=5)
    res, adds = {}, {}
    try:
        for fuse in (True, False):
            gpu.fuse_residual_add = fuse
            gpu.start_profile("add")
            res[fuse] = hip_step(gpu, model, seqs, True, 50)
            adds[fuse] = sum(v[1] for k, v in gpu.stop_profile().items() if k == "add")
    finally:
        gpu.fuse_residual_add = True
    assert adds[False] - adds[True] == 2 * kw["layers"], adds
    assert np.array_equal(res[True][0], res[False][0])
    for n in res[True][1]:
        assert np.array_equal(res[True][1][n], res[False][1][n]), n


@pytest.mark.parametrize("arch_name", ["llama", "gemma3"])
@pytest.mark.parametrize("recompute", [False, True])
def test_q_and_k_rotations_leave_as_one_launch(gpu, ref, arch_name, recompute):
    """rope(q), rope(k) of a layer go out as one forward launch: every bit of the loss and of every gradient is what one
    launch per rotation gives, with half the forward rotation launches; stacked and one sequence at a time (four streams),
    with and without recomputed layers."""
    kw = dict(arch="llama", vocab=64, hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=256, rope_base=1e4, rms_eps=1e-5)
    if arch_name == "gemma3":
        kw = dict(REAL["gemma3-window"], layers=3, vocab=256)
    _, model = build_pair(ref, kw, seed=51, std=0.05)
    seqs = batches(ref, kw["vocab"], 48, 3, seed=52, mask_every=5)
    for stacked in (True, False):
        res, n = {}, {}
        try:
            for pair in (True, False):
                gpu.pair_ropes = pair
                gpu.start_profile("rope")
                res[pair] = hip_step(gpu, model, seqs, stacked, 48, recompute=recompute)
                n[pair] = {k: v[1] for k, v in gpu.stop_profile().items()}
        finally:
            gpu.pair_ropes = True
        assert n[False]["rope"] == 2 * n[True]["rope"] > 0 and n[False]["rope.bwd"] == n[True]["rope.bwd"], n
        assert np.array_equal(res[True][0], res[False][0])
        for name in res[True][1]:
            assert np.array_equal(res[True][1][name], res[False][1][name]), name


def test_linear_output_used_again_after_its_fused_add(gpu, ref):
    """The product that went straight into an add is computed after all when something else wants it: a later op, a
    readback. Against the oracle."""
    ag = mod("autograd")
    r = ref.Mulberry32(91)
    T, d = 70, 64
    ha, xa, wa = r.fill_randn([T, d], 0.8), r.fill_randn([T, d], 0.8), r.fill_randn([d, d], 0.3)
    up = r.fill_uniform([T * d])

    def graph(m, h, x, w):
        y = m.linear(x, w)
        z = m.add(h, y)
        return m.mul(z, y), y

    hs = [ag.Tensor(a, list(a.shape), True) for a in (ha, xa, wa)]
    rs = [ref.Tensor(a, list(a.shape), True) for a in (ha, xa, wa)]
    gpu.install()
    try:
        out, y = graph(ag, *hs)
        from gpu_common import backward_from
        backward_from(gpu, ag, out, up)
        gpu.sync([out, y])
    finally:
        gpu.uninstall()
    rout, ry = graph(ref, *rs)
    ref.backward_from(rout, up)
    assert_close(out.data, rout.data, "forward")
    assert_close(y.data, ry.data, "the product read back")
    for h, rr, nm in zip(hs, rs, ("dh", "dx", "dw")):
        assert_close(h.grad, rr.grad, nm)
    # read back only: the product has no other consumer than the fused add
    hs = [ag.Tensor(a, list(a.shape), False) for a in (ha, xa, wa)]
    gpu.install()
    try:
        y = ag.linear(hs[1], hs[2])
        z = ag.add(hs[0], y)
        gpu.sync([z, y])
    finally:
        gpu.uninstall()
    assert_close(y.data, ry.data, "the product read back, no other consumer")
    assert_close(z.data, (ha + ry.data.reshape(T, d)).reshape(-1), "sum")


@pytest.mark.parametrize("arch_name", ["llama", "gemma3"])
@pytest.mark.parametrize("recompute", [False, True])
def test_add_backward_hands_its_gradient_on(gpu, ref, arch_name, recompute):
    """add's backward launches nothing where it is the first writer of an intermediate's gradient: the operand points at
    the upstream buffer, a reader takes it there, rmsNorm's backward adds to it from there, anything else gets a copy
    first, and aliases are settled before a region's buffers are recycled. Every bit of the step is what the copying
    backward gives, with fewer add.bwd launches; also against the oracle."""
    kw = SMALL[arch_name]
    rmodel, model = build_pair(ref, kw, seed=51, std=0.1)
    seqs = batches(ref, kw["vocab"], 23, 2, seed=52, mask_every=5)
    res, n = {}, {}
    try:
        for alias in (True, False):
            gpu.alias_add_grads = alias
            gpu.start_profile("")
            res[alias] = hip_step(gpu, model, seqs, True, 23, recompute=recompute)
            prof = gpu.stop_profile()
            n[alias] = sum(v[1] for k, v in prof.items() if k == "add.bwd")
    finally:
        gpu.alias_add_grads = True
    assert n[True] < n[False], n
    assert np.array_equal(res[True][0], res[False][0])
    for name in res[True][1]:
        assert np.array_equal(res[True][1][name], res[False][1][name]), name
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(res[True][0], res[True][1], lr, gr, f"{arch_name} handed-on add gradients recompute={recompute}")


def test_handed_on_gradient_with_other_readers_and_writers(gpu, ref):
    """An intermediate whose gradient was handed on by an add and is then written by a product, an elementwise op and
    another add, or only read. Against the oracle."""
    ag = mod("autograd")
    r = ref.Mulberry32(61)
    T, d = 40, 64
    xa, wa, ga = r.fill_randn([T, d], 0.8), r.fill_randn([d, d], 0.3), 1 + 0.2 * r.fill_randn([d])
    up = r.fill_uniform([T * d])

    def graph(m, x, w, gain):
        t = m.scale(x, 0.5)                                  # an intermediate with four consumers
        u = m.add(t, m.silu(t))                              # handed on to t first (add runs its backward first)
        v = m.add(u, m.linear(t, w))                         # a product into t's gradient
        return m.add(m.mul(v, t), m.rms_norm(m.add(t, u), gain, 1e-5))

    hs = [ag.Tensor(a, list(a.shape), True) for a in (xa, wa, ga)]
    rs = [ref.Tensor(a, list(a.shape), True) for a in (xa, wa, ga)]
    gpu.install()
    try:
        out = graph(ag, *hs)
        from gpu_common import backward_from
        backward_from(gpu, ag, out, up)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    rout = graph(ref, *rs)
    ref.backward_from(rout, up)
    assert_close(out.data, rout.data, "forward")
    for h, rr, nm in zip(hs, rs, ("dx", "dw", "dgain")):
        assert_close(h.grad, rr.grad, nm)


def test_trim_pool_returns_free_buffers_and_work_goes_on(gpu, ref):
    """Free buffers of the size-class pool go back to the device on request (and on their own when an allocation fails);
    buffers in use stay, and the next step allocates afresh and gives the same bits."""
    kw = SMALL["llama"]
    _, model = build_pair(ref, kw, seed=3, std=0.1)
    seqs = batches(ref, kw["vocab"], 19, 2, seed=4)
    l0, g0 = hip_step(gpu, model, seqs, True, 19)
    before = gpu.resident_bytes()
    freed = gpu.trim_pool()
    assert freed > 0 and gpu.resident_bytes() == before - freed
    assert all(not free for pool in gpu._pools for free in pool.values())
    l1, g1 = hip_step(gpu, model, seqs, True, 19)
    assert np.array_equal(l0, l1) and all(np.array_equal(g0[n], g1[n]) for n in g0)


def test_gradient_rearm_survives_a_mid_window_freeze(gpu, ref):
    """gpu-parity.ts:1980-2028: parameters frozen between a window's backward and its sync, thawed afterwards. The
    accumulators still hold that window's gradients, so the window after the thaw must start them afresh: same inputs
    and weights give the first window's gradients, not twice them."""
    ag, arch = mod("autograd"), mod("arch")
    kw = dict(arch="gemma3", vocab=64, hidden=64, layers=4, heads=4, kv_heads=2, head_dim=16, ffn=256, rope_base=1e6,
              rope_base_local=1e4, sliding_window=16, swa_pattern=2, rms_eps=1e-6)
    ids = np.array([(i * 11 + 5) % 64 for i in range(33)])
    _, model = build_pair(ref, kw, seed=5, std=0.05)
    gpu.install()
    try:
        gpu.upload_params(model.params())

        def window(freeze_before_sync=False):
            loss = arch.sequence_loss(model, ids[:-1], ids[1:], 0)
            ag.backward(loss, 1.0)
            if freeze_before_sync:
                for p in model.params():
                    p.requires_grad = False
            gpu.sync([loss])
            return [p.grad.copy() for p in model.params()]

        first = window()
        window(freeze_before_sync=True)
        for p in model.params():
            p.requires_grad = True
        third = window()
    finally:
        gpu.uninstall()
        gpu.sync([])
    worst, n = 0.0, 0
    for a, b in zip(first, third):
        keep = np.abs(a) >= 1e-6
        if keep.any():
            worst = max(worst, float(np.abs(b[keep] / a[keep] - 1).max()))
            n += int(keep.sum())
    assert n > 0 and worst < 1e-4, (worst, n)


def test_empty_sync_recycles_without_corrupting_queued_work(gpu, ref):
    """gpu-parity.ts:2338-2410: with gradients kept on the device a bare sync() stages nothing and hands every
    intermediate back to the pool; a second chain then reuses exactly those buffers (the pool does not grow) while the
    first chain's gradients, already queued, still come out right."""
    ag = mod("autograd")
    T, HID, OUT = 24, 64, 40
    r = ref.Mulberry32(0xFEED)
    xs, w1s, w2s = r.fill_randn([T, HID], 0.8), r.fill_randn([HID, HID], 0.8), r.fill_randn([OUT, HID], 0.8)
    targets = [(i * 7 + 3) % OUT for i in range(T)]
    rt = [ref.Tensor(a, list(a.shape), True) for a in (xs, w1s, w2s)]
    ref.backward(ref.cross_entropy(ref.linear(ref.gelu(ref.linear(rt[0], rt[1])), rt[2]), targets), 1.0)
    ht = [ag.Tensor(a, list(a.shape), True) for a in (xs, w1s, w2s)]
    for t in ht:
        gpu.keep_grad_on_device(t)
    gpu.install()
    try:
        ag.backward(ag.cross_entropy(ag.linear(ag.gelu(ag.linear(ht[0], ht[1])), ht[2]), targets), 1.0)
        gpu.sync([])                         # stages nothing, recycles everything
        assert gpu.last_sync_readback_bytes == 0
        pool_before = gpu._pool_bytes
        ag.gelu(ag.linear(ht[0], ht[1]))     # reuses the buffers the first chain released
        assert gpu._pool_bytes == pool_before
        gpu.sync([])
        for t, rr, nm in zip(ht, rt, ("x", "w1", "w2")):
            got = gpu.read_state_buffer(gpu.buffers_for(t)["grad"], t.size)
            assert_close(got, rr.grad, f"recycle reuse d{nm}")
    finally:
        gpu.uninstall()
        gpu.sync([])


def test_recompute_memory_gate(ref):
    """gpu-parity.ts:1363-1420: the buffer pool (a high-water mark) is flat in the number of steps (sync drains the
    regions' buffers), flat in the number of micro-batches when transients are reclaimed between them, and clearly
    smaller with recompute than without. A fresh backend per arm, sequential micro-batches of 128 tokens, on one stream
    (the reference's one queue) and on four (bounded by four micro-batches in flight)."""
    ag, optim, train, hb = mod("autograd"), mod("optim"), mod("train"), mod("hip_backend")
    kw = dict(arch="gemma3", vocab=64, hidden=64, layers=4, heads=4, kv_heads=2, head_dim=16, ffn=256, rope_base=1e6,
              rope_base_local=1e4, sliding_window=16, swa_pattern=2, rms_eps=1e-6)
    tokens = [(i * 7 + 3) % 64 for i in range(8192)]

    def pool_for(recompute, reclaim, steps, batch, streams=1):
        g = hb.HipBackend(0, streams=streams)
        _, model = build_pair(ref, kw, seed=5, std=0.05)
        hm, ha = model.param_groups()
        ag.set_checkpointing(recompute)
        try:
            train.train_lm_hip_resident(model, g, optim.MuonHip(g, hm, ha, lr=0.01, momentum=0.95, aux={"lr": 3e-3, "weight_decay": 0.0, "clip": 1.0}),
                                        train.WindowSampler(tokens, 128, ag.mulberry32(7)), steps, batch, 128, stacked=False,
                                        reclaim=reclaim, log_every=100)
            return g._pool_bytes
        finally:
            ag.set_checkpointing(False)
            g.destroy()

    s2, s6 = pool_for(True, False, 2, 2), pool_for(True, False, 6, 2)
    assert s6 <= s2 * 1.01, (s2, s6)
    b2, b4 = pool_for(True, True, 3, 2), pool_for(True, True, 3, 4)
    assert b4 <= b2 * 1.05, (b2, b4)
    dense = pool_for(False, True, 3, 2)
    assert b2 < 0.9 * dense, (b2, dense)
    # micro-batches dealt to four streams: every stream has its own pool, so the mark is that of four micro-batches in
    # flight, and flat from there on
    m4, m8 = pool_for(True, True, 3, 4, streams=4), pool_for(True, True, 3, 8, streams=4)
    assert m8 <= m4 * 1.05, (m4, m8)
    assert m4 <= 4 * b2 * 1.05, (b2, m4)


def test_resident_step_then_sample_readback(gpu, ref):
    """gpu-parity.ts:1671-1735: a device-resident step stages back its loss scalars only, and a forward pass after it
    (sampling) stages back its logits only: the optimizer's parameters keep their gradients on the device."""
    ag, arch, optim, train = mod("autograd"), mod("arch"), mod("optim"), mod("train")
    kw = dict(arch="gemma3", vocab=64, hidden=64, layers=4, heads=4, kv_heads=2, head_dim=16, ffn=256, rope_base=1e6,
              rope_base_local=1e4, sliding_window=16, swa_pattern=2, rms_eps=1e-6)
    tokens = [(i * 7 + 3) % 64 for i in range(2048)]
    _, model = build_pair(ref, kw, seed=5, std=0.05)
    hm, ha = model.param_groups()
    seen = []
    train.train_lm_hip_resident(model, gpu, optim.MuonHip(gpu, hm, ha, lr=0.01, momentum=0.95, aux={"lr": 3e-3}),
                                train.WindowSampler(tokens, 64, ag.mulberry32(7)), 1, 1, 64, stacked=False, reclaim=True,
                                on_step_time=lambda a, b, rb: seen.append(rb))
    assert seen == [4]                                   # one micro-batch: one f32 loss
    prompt = np.array([3, 11, 29, 5, 17])
    gpu.install()
    try:
        logits = model.forward(prompt)
        gpu.sync([logits])
        assert gpu.last_sync_readback_bytes == len(prompt) * kw["vocab"] * 4
        assert np.isfinite(logits.data).all()
    finally:
        gpu.uninstall()
        gpu.sync([])


def test_checkpoint_input_guard_on_device(gpu, ref):
    """gradcheck.ts:808-829 through the device backend: the guard runs above the dispatch, and a refused block leaves
    the backend usable (its region is closed by the next sync)."""
    ag = mod("autograd")
    r = ref.Mulberry32(12)
    x = ag.Tensor(r.fill_randn([5, 6], 0.8), [5, 6], True)
    w1 = ag.Tensor(r.fill_randn([6, 6], 0.8), [6, 6], True)
    gpu.install()
    ag.set_checkpointing(True)
    try:
        shared = ag.linear(x, w1)
        with pytest.raises(ValueError, match="did not create"):
            ag.checkpoint([x], lambda: ag.add(ag.silu(ag.linear(x, w1)), shared))
        with pytest.raises(ValueError, match="one of its inputs"):
            ag.checkpoint([x], lambda: x)
        out = ag.checkpoint([x, shared], lambda: ag.add(ag.silu(ag.linear(x, w1)), shared))
        gpu.sync([out])
        want = ref.add(ref.silu(ref.linear(ref.Tensor(x.data, [5, 6]), ref.Tensor(w1.data, [6, 6]))),
                       ref.linear(ref.Tensor(x.data, [5, 6]), ref.Tensor(w1.data, [6, 6])))
        assert_close(out.data, want.data, "checkpointed block with a declared shared input")
    finally:
        ag.set_checkpointing(False)
        gpu.uninstall()
        gpu.sync([])


def test_micro_batches_on_several_streams(gpu, ref):
    """Six sequential micro-batches (the reference's call pattern, train-gpu.ts:200-219) on the backend's four streams:
    micro-batch i runs on stream i mod 4 with that stream's own parameter-gradient accumulators, summed in stream order
    before the first reader. Losses equal, and every gradient within the parity bound of, the oracle's sequential
    accumulation; two runs are bit-identical; a one-stream backend gives the same losses bit for bit and the same
    gradients up to the order of six additions."""
    hb = mod("hip_backend")
    assert gpu._nstreams == 4
    kw = REAL["smollm2"]
    rmodel, model = build_pair(ref, kw, seed=31, std=0.05)
    seqs = batches(ref, kw["vocab"], 150, 6, seed=32, mask_every=9)
    l1, g1 = hip_step(gpu, model, seqs, False, 150)
    l2, g2 = hip_step(gpu, model, seqs, False, 150)
    assert l1.tobytes() == l2.tobytes() and all(g1[n].tobytes() == g2[n].tobytes() for n in g1), "run-to-run"
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        lr, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    compare(l1, g1, lr, gr, "six micro-batches on four streams")
    one = hb.HipBackend(0, streams=1)
    try:
        _, model1 = build_pair(ref, kw, seed=31, std=0.05)
        ls, gs = hip_step(one, model1, seqs, False, 150)
    finally:
        one.destroy()
    assert ls.tobytes() == l1.tobytes()
    for n in gs:
        assert_close(g1[n], gs[n], f"four streams vs one, {n}", rel_l2=2e-6, max_rel=2e-5)


def test_micro_batch_boundaries_told_by_the_trainer(ref):
    """next_micro_batch(): the trainer marks where a sequence's graph begins instead of the backend inferring it from the
    first op's inputs. On the llama graph (where the inference holds) both give the same streams and the same bits; a
    graph whose every forward op reads an intermediate made before the loop (which the inference takes for the
    continuation of the previous micro-batch) is dealt to the streams only when told. Gradients against one stream."""
    hb, ag = mod("hip_backend"), mod("autograd")
    kw = REAL["smollm2"]
    seqs = batches(ref, kw["vocab"], 150, 5, seed=41, mask_every=7)

    def run(explicit, streams=4):
        be = hb.HipBackend(0, streams=streams)
        arch = mod("arch")
        try:
            _, model = build_pair(ref, kw, seed=40, std=0.05)
            be.install()
            seen, losses = [], []
            for ids, tg in seqs:
                if explicit:
                    be.next_micro_batch()
                loss = arch.sequence_loss(model, ids, tg, 0)
                seen.append(be._cur)
                ag.backward(loss, 1.0 / len(seqs))
                losses.append(loss)
            be.sync(losses)
            be.uninstall()
            return seen, np.concatenate([l.data for l in losses]), {n: p.grad.copy() for n, p in model.named_params()}
        finally:
            be.destroy()

    s_inf, l_inf, g_inf = run(False)
    s_exp, l_exp, g_exp = run(True)
    assert s_inf == s_exp == [0, 1, 2, 3, 0]
    assert l_inf.tobytes() == l_exp.tobytes() and all(g_inf[n].tobytes() == g_exp[n].tobytes() for n in g_inf)

    # a graph the inference does not cut: every micro-batch starts from one shared, gradient-free feature h0 = x W0^T
    # computed once (W0 frozen), which the inference takes for the continuation of the graph before it
    r = ref.Mulberry32(43)
    xs = r.fill_randn([64, 32], 1.0)
    w0d, w1d = r.fill_randn([32, 32], 0.3), r.fill_randn([48, 32], 0.3)
    scales = [0.5, 1.5, -1.0, 2.0]

    def shared_root(explicit, streams):
        be = hb.HipBackend(0, streams=streams)
        try:
            x = ag.Tensor(xs, [64, 32])
            w0, w1 = ag.Tensor(w0d, [32, 32], False), ag.Tensor(w1d, [48, 32], True)
            be.install()
            h0 = ag.linear(x, w0)
            seen, outs = [], []
            for c in scales:
                if explicit:
                    be.next_micro_batch()
                y = ag.linear(ag.silu(ag.scale(h0, c)), w1)
                seen.append(be._cur)
                ag.backward(y, 0.25)          # seeds dy = 0.25 everywhere
                outs.append(y)
            be.sync(outs)
            be.uninstall()
            return seen, w1.grad.copy(), [o.data.copy() for o in outs]
        finally:
            be.destroy()

    s1, a1, ya = shared_root(False, 4)
    s2, b1, yb = shared_root(True, 4)
    s3, c1, yc = shared_root(True, 1)
    assert s1 == [0, 0, 0, 0], s1                      # inferred: all one micro-batch, one stream
    assert s2 == [0, 1, 2, 3] and s3 == [0, 0, 0, 0]
    assert all(u.tobytes() == v.tobytes() == w.tobytes() for u, v, w in zip(ya, yb, yc))
    assert a1.tobytes() == c1.tobytes()
    assert_close(b1, c1, "told boundaries on four streams vs one stream, dW1", rel_l2=2e-6, max_rel=2e-5)


def test_collector_runs_only_at_sync_while_installed(ref):
    """install() takes the interpreter's cyclic collector out of the recording (disabled, what already exists frozen) and
    hands it back on uninstall() or on destroy() while installed; sync() collects the previous step's graph; manage_gc =
    False leaves the collector alone."""
    import gc
    import weakref
    hb, ag, arch = mod("hip_backend"), mod("autograd"), mod("arch")
    assert gc.isenabled()
    kw = SMALL["llama"]
    _, model = build_pair(ref, kw, seed=3, std=0.05)
    seqs = batches(ref, kw["vocab"], 12, 2, seed=4)
    be = hb.HipBackend(0, streams=2)
    try:
        be.install()
        assert not gc.isenabled() and gc.get_freeze_count() > 0
        loss = arch.sequence_loss(model, seqs[0][0], seqs[0][1], 0)
        ag.backward(loss, 1.0)
        probe = weakref.ref(loss._prev[0])           # an intermediate of this step's graph (part of a reference cycle)
        be.sync([loss])
        assert probe() is not None                  # the graph is alive: the caller holds the loss
        del loss
        loss2 = arch.sequence_loss(model, seqs[1][0], seqs[1][1], 0)
        ag.backward(loss2, 1.0)
        be.sync([loss2])                            # collects the previous step's graph
        assert probe() is None
        be.uninstall()
        assert gc.isenabled() and gc.get_freeze_count() == 0
        be.install()
        assert not gc.isenabled()
    finally:
        be.destroy()                                # while installed
        ag.set_ops_backend(None)
    assert gc.isenabled() and gc.get_freeze_count() == 0
    be = hb.HipBackend(0, streams=1)
    be.manage_gc = False
    try:
        be.install()
        assert gc.isenabled() and gc.get_freeze_count() == 0
        be.uninstall()
    finally:
        be.destroy()


def test_grad_fold_sums_in_source_order(gpu):
    """gt_grad_fold: dst (+)= src0 + src1 + ... per tensor in one launch, bit for bit the f32 sums taken in that order;
    absent sources skipped, store and accumulate, sizes that are no multiple of four and an unaligned tensor."""
    import ctypes as C
    lib = mod("lib")
    rs = np.random.RandomState(3)
    sizes = [8192 * 3 + 5, 7, 4096, 100000]
    ns = 3
    dst0 = [rs.standard_normal(n).astype(np.float32) for n in sizes]
    srcs = [[rs.standard_normal(n).astype(np.float32) for _ in range(ns)] for n in sizes]
    present = [[1, 1, 1], [1, 0, 1], [0, 0, 1], [1, 1, 0]]
    accs = [1, 0, 1, 0]
    big = gpu.create_state_buffer(4 * (sizes[1] + 1))               # tensor 1's destination starts 4 bytes into a buffer
    db = [gpu.create_state_buffer(4 * n) for n in sizes]
    db[1] = big + 4
    for b, a in zip(db, dst0):
        lib.check(gpu.ctx, lib.lib.gt_h2d(gpu.ctx, b, a.ctypes.data_as(C.c_void_p), a.nbytes), "h2d")
    sb = []
    for i, n in enumerate(sizes):
        for s_ in range(ns):
            if present[i][s_]:
                b = gpu.create_state_buffer(4 * n)
                gpu.write_state_buffer(b, srcs[i][s_])
                sb.append(b)
            else:
                sb.append(0)
    n = len(sizes)
    lib.check(gpu.ctx, lib.lib.gt_grad_fold(gpu.ctx, n, (C.c_uint64 * n)(*db), (C.c_int * n)(*accs), ns, (C.c_uint64 * (n * ns))(*sb),
                                            (C.c_int64 * n)(*sizes)), "gt_grad_fold")
    for i in range(n):
        want = dst0[i].copy() if accs[i] else None
        for s_ in range(ns):
            if present[i][s_]:
                want = srcs[i][s_].copy() if want is None else (want + srcs[i][s_]).astype(np.float32)
        got = gpu.read_state_buffer(db[i], sizes[i])
        assert np.array_equal(got, want), f"tensor {i}"


def test_parameter_buffers_return_when_released_or_collected(gpu, ref):
    """Device buffers of parameters (values, gradient accumulators, the per-stream ones too) go back to the pool when the
    host releases the tensors or drops its last reference to them: the next model of the same shape reuses them and the
    pool does not grow. Optimizers release their tables and moments with destroy()."""
    import gc
    ag, optim = mod("autograd"), mod("optim")
    kw = SMALL["llama"]
    seqs = batches(ref, kw["vocab"], 19, 3, seed=5)

    def one_model(explicit):
        _, model = build_pair(ref, kw, seed=3, std=0.1)
        opt = optim.AdamWHip(gpu, model.params(), lr=1e-3)
        hip_step(gpu, model, seqs, False, 19)
        gpu.install()
        try:
            opt.record_step()
            gpu.sync([])
        finally:
            gpu.uninstall()
        opt.destroy()
        if explicit:
            gpu.release(model.params())
        del model, opt
        gc.collect()
        gpu.sync([])

    one_model(True)
    pool0, res0 = gpu._pool_bytes, gpu.resident_bytes()
    one_model(True)
    assert (gpu._pool_bytes, gpu.resident_bytes()) == (pool0, res0), "explicit release"
    one_model(False)
    assert (gpu._pool_bytes, gpu.resident_bytes()) == (pool0, res0), "collected tensors"


def test_kernel_family_cannot_change_under_a_live_graph(gpu, ref):
    ag = mod("autograd")
    r = ref.Mulberry32(4)
    q, k, v = (ag.Tensor(r.fill_randn([128, 2 * 64], 0.5), [128, 128], True) for _ in range(3))
    gpu.install()
    try:
        out = ag.attention(q, k, v, 128, 2, 2, 64, 0)
        with pytest.raises(RuntimeError, match="attn.generic cannot change"):
            gpu.set_option("attn.generic", 1)
        gpu.sync([out])
        gpu.set_option("attn.generic", 1)
        gpu.set_option("attn.generic", 0)
    finally:
        gpu.uninstall()


def test_checkpoint_over_leaf_inputs_after_an_earlier_backward(gpu, ref):
    """A checkpointed block whose declared inputs are parameters (the gradcheck-style use, gradcheck.ts:770-806), differentiated
    after another graph's backward has already run: the block's replay records forward ops in the middle of a backward,
    all of whose inputs are leaves. That replay belongs to the graph being differentiated: it must not start a micro-batch
    on another stream (the replayed output's gradient, the seed copy and the rest of the tape would then run on two
    streams with nothing ordering them). Gradients against the oracle and against a one-stream backend, bit for bit."""
    hb, ag = mod("hip_backend"), mod("autograd")
    assert gpu._nstreams == 4
    r = ref.Mulberry32(77)
    T, d = 96, 64
    xs, w1s, w2s, w0s = r.fill_randn([T, d], 0.8), r.fill_randn([d, d], 0.3), r.fill_randn([d, d], 0.3), r.fill_randn([d, d], 0.3)
    up = ref.Mulberry32(5).fill_uniform([T * d])

    def run(be):
        x, w1, w2, w0 = (ag.Tensor(a, list(a.shape), True) for a in (xs, w1s, w2s, w0s))
        be.install()
        ag.set_checkpointing(True)
        try:
            first = ag.linear(x, w0)                             # an earlier graph and its backward
            backward_from(be, ag, first, up)
            streams_seen = []
            def block():
                o = ag.linear(ag.silu(ag.linear(x, w1)), w2)
                streams_seen.append(be._cur)                     # the stream the block's ops were recorded on
                return o
            out = ag.checkpoint([x, w1, w2], block)              # every declared input is a leaf
            y = ag.add(out, ag.linear(x, w0))
            cur = be._cur
            backward_from(be, ag, y, up)
            assert be._cur == cur, "the replay inside the backward moved the recording to another stream"
            assert streams_seen == [cur, cur]
            be.sync([y])
        finally:
            ag.set_checkpointing(False)
            be.uninstall()
        return y.data.copy(), [t.grad.copy() for t in (x, w1, w2, w0)]

    y4, g4 = run(gpu)
    one = hb.HipBackend(0, streams=1)
    try:
        y1, g1 = run(one)
    finally:
        one.destroy()
    assert y4.tobytes() == y1.tobytes()
    for a, b, n in zip(g4, g1, "x w1 w2 w0".split()):
        assert_close(a, b, f"four streams vs one, d{n}", rel_l2=2e-6, max_rel=2e-5)
    rx, rw1, rw2, rw0 = (ref.Tensor(a, list(a.shape), True) for a in (xs, w1s, w2s, w0s))
    ref.backward_from(ref.linear(rx, rw0), up)
    ry = ref.add(ref.linear(ref.silu(ref.linear(rx, rw1)), rw2), ref.linear(rx, rw0))
    ref.backward_from(ry, up)
    assert_close(y4, ry.data, "checkpointed block over leaf inputs, forward")
    for a, t, n in zip(g4, (rx, rw1, rw2, rw0), "x w1 w2 w0".split()):
        assert_close(a, t.grad, f"checkpointed block over leaf inputs, d{n}")


def test_optimizer_destroy_after_the_backend_is_gone(ref):
    """gt_ctx_destroy releases every live optimizer of the context; an optimizer object destroyed after its backend must
    not hand the freed handles back to the library."""
    hb, optim, ag = mod("hip_backend"), mod("optim"), mod("autograd")
    be = hb.HipBackend(0, streams=2)
    r = ref.Mulberry32(3)
    ps = [ag.Tensor(r.fill_randn([8, 8], 0.1), [8, 8], True), ag.Tensor(r.fill_randn([8], 0.1), [8], True)]
    mu = optim.MuonHip(be, ps[:1], ps[1:], lr=0.01)
    ad = optim.AdamWHip(be, ps, lr=1e-3)
    be.destroy()
    mu.destroy()
    ad.destroy()
    assert not ad._h and not mu._h and ad._m == [] and mu._bufs == []


@pytest.mark.parametrize("name", ["smollm2", "gemma3-window", "qwen3-hd128"])
@pytest.mark.parametrize("recompute", [False, True])
def test_rotation_backward_rides_the_attention_write_backs(gpu, ref, name, recompute):
    """With kept scores (T a multiple of 128) the backward of rope(q) and rope(k) is applied where attention's backward
    writes dQ and dK: no rope.bwd launch is left, the loss is bit-identical and every gradient equals the unfused path's to
    rounding and the oracle's to the parity bound. llama (rotation straight after the projections), gemma-style and qwen3
    (after the per-head norms), GQA, a window, with and without recomputed layers."""
    kw = dict(REAL[name], layers=2)
    rmodel, model = build_pair(ref, kw, seed=61, std=0.05)
    T = 128
    seqs = batches(ref, kw["vocab"], T, 2, seed=62, mask_every=7)
    res, n = {}, {}
    try:
        for fuse in (True, False):
            gpu.fuse_rope_bwd = fuse
            gpu.start_profile("rope")
            res[fuse] = hip_step(gpu, model, seqs, True, T, recompute=recompute)
            n[fuse] = {k: v[1] for k, v in gpu.stop_profile().items()}
    finally:
        gpu.fuse_rope_bwd = True
    assert n[True].get("rope.bwd", 0) == 0 and n[False]["rope.bwd"] == 2 * kw["layers"], n
    assert np.array_equal(res[True][0], res[False][0])
    for pname in res[True][1]:
        assert_close(res[True][1][pname], res[False][1][pname], f"fused vs separate rotations, {pname}", rel_l2=2e-6, max_rel=2e-5)
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        lr, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    compare(res[True][0], res[True][1], lr, gr, f"{name}, rotations' backward in the attention write-backs")
