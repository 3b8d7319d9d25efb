"""Optimizer-step parity: AdamWHip and MuonHip (through the C ABI) against the CPU oracle, and multi-step
trajectories against the oracle's CPU training loop."""
import math

import numpy as np
import pytest

from gpu_common import assert_close, mod
from test_gpu_model import SMALL, batches, build_pair

pytestmark = pytest.mark.gpu


def test_adamw_three_steps_clip_triggers_then_relaxes(gpu, ref):
    """gpu-parity.ts:1044-1093: shapes [12,8] and [5], lr 5e-3, wd 0.01, clip 1, gradient scales 0.5 / 0.05 / 0.01."""
    ag, optim = mod("autograd"), mod("optim")
    rng = ref.Mulberry32(42)
    shapes = [[12, 8], [5]]
    init = [rng.fill_randn(s, 0.5) for s in shapes]
    rp = [ref.Tensor(a, s, True) for a, s in zip(init, shapes)]
    hp = [ag.Tensor(a, s, True) for a, s in zip(init, shapes)]
    ropt = ref.AdamW(rp, lr=5e-3, weight_decay=0.01, clip=1.0)
    hopt = optim.AdamWHip(gpu, hp, lr=5e-3, weight_decay=0.01, clip=1.0)
    norms = []
    for gs in (0.5, 0.05, 0.01):
        grads = [rng.fill_randn(s, gs) for s in shapes]
        for r, h, g in zip(rp, hp, grads):
            r.grad[:] = g.reshape(-1)
            gpu.write_state_buffer(gpu.buffers_for(h)["grad"], g)
            gpu._entries[h].grad_init = True
        ropt.step()
        hopt.record_step()
        norms.append(hopt.grad_norm())
        hopt.sync_weights_to_host()
        for r, h in zip(rp, hp):
            assert_close(h.data, r.data, f"AdamW weights, grad scale {gs}")
    assert norms[0] > 1.0 and norms[1] < 1.0 and norms[2] < 1.0
    st = hopt.export_state()
    assert st["t"] == 3
    for m, r in zip(st["m"], ropt.m):
        assert_close(m, r, "AdamW first moment")
    for v, r in zip(st["v"], ropt.v):
        assert_close(v, r, "AdamW second moment")


def test_adamw_many_tensors_one_launch_group(gpu, ref):
    """A group larger than one chunk per tensor and with odd sizes: the chunk table covers every element once."""
    ag, optim = mod("autograd"), mod("optim")
    rng = ref.Mulberry32(7)
    shapes = [[70001], [3], [257, 129], [1], [65536], [65537]]
    init = [rng.fill_randn(s, 0.3) for s in shapes]
    rp = [ref.Tensor(a, s, True) for a, s in zip(init, shapes)]
    hp = [ag.Tensor(a, s, True) for a, s in zip(init, shapes)]
    ropt = ref.AdamW(rp, lr=1e-3, beta2=0.95, weight_decay=0.1, clip=1.0)
    hopt = optim.AdamWHip(gpu, hp, lr=1e-3, beta2=0.95, weight_decay=0.1, clip=1.0)
    ref.set_threads(min(8, ref.max_threads()))
    try:
        for _ in range(2):
            for r, h, s in zip(rp, hp, shapes):
                g = rng.fill_randn(s, 0.01)
                r.grad[:] = g.reshape(-1)
                gpu.write_state_buffer(gpu.buffers_for(h)["grad"], g)
                gpu._entries[h].grad_init = True
            ropt.step()
            hopt.record_step()
    finally:
        ref.set_threads(1)
    hopt.sync_weights_to_host()
    for r, h in zip(rp, hp):
        assert_close(h.data, r.data, "AdamW group")


@pytest.mark.parametrize("m,n", [(5, 9), (24, 17), (33, 33), (16, 64), (128, 640), (200, 72)])
def test_newton_schulz(gpu, ref, m, n):
    """gpu-parity.ts:974-987: m<n, m>n, m=n, 5 steps. f32 GEMM accumulation order differs from the oracle's, and five
    quintic iterations amplify that: 2e-5 relative L2 (the per-gradient bound is 1e-5)."""
    G = ref.Mulberry32(m * 100 + n).fill_randn([m, n])
    want = ref.newton_schulz(G, m, n, 5)
    b_in = gpu.create_state_buffer(G.nbytes)
    b_out = gpu.create_state_buffer(G.nbytes)
    gpu.write_state_buffer(b_in, G)
    lib = mod("lib")
    lib.check(gpu.ctx, lib.lib.gt_newton_schulz(gpu.ctx, m, n, 5, b_in, b_out), "gt_newton_schulz")
    got = gpu.read_state_buffer(b_out, m * n)
    assert_close(got, want, f"NS {m}x{n}", rel_l2=2e-5, max_rel=1e-4)


def test_muon_two_steps_momentum_carries(gpu, ref):
    """gpu-parity.ts:996-1032."""
    ag, optim = mod("autograd"), mod("optim")
    rng = ref.Mulberry32(8)
    shapes = [[24, 10], [12, 40], [16, 16]]
    init = [rng.fill_randn(s, 0.5) for s in shapes]
    rp = [ref.Tensor(a, s, True) for a, s in zip(init, shapes)]
    hp = [ag.Tensor(a, s, True) for a, s in zip(init, shapes)]
    raux = ref.Tensor(init[0][:3].copy(), [3, 10], True)
    haux = ag.Tensor(init[0][:3].copy(), [3, 10], True)
    ropt = ref.Muon(rp, [raux], lr=0.02, aux={"lr": 3e-3})
    hopt = optim.MuonHip(gpu, hp, [haux], lr=0.02, aux={"lr": 3e-3})
    for _ in range(2):
        for r, h, s in zip(rp + [raux], hp + [haux], shapes + [[3, 10]]):
            g = rng.fill_randn(s, 0.1)
            r.grad[:] = g.reshape(-1)
            gpu.write_state_buffer(gpu.buffers_for(h)["grad"], g)
            gpu._entries[h].grad_init = True
        ropt.step()
        hopt.record_step()
    hopt.sync_weights_to_host()
    for r, h in zip(rp + [raux], hp + [haux]):
        assert_close(h.data, r.data, "Muon weights", rel_l2=2e-5)
    st = hopt.export_state()
    for b, r in zip(st["muonMomentum"], ropt.bufs):
        assert_close(b, r, "Muon momentum")
    raw = optim.serialize_opt_state(st)
    back = optim.deserialize_opt_state(raw)
    assert back["adamT"] == 2 and all(np.array_equal(a, b) for a, b in zip(back["muonMomentum"], st["muonMomentum"]))


@pytest.mark.parametrize("which", ["adamw", "muon_wsd"])
def test_four_step_trajectory_vs_cpu_trainer(gpu, ref, which):
    """gpu-parity.ts:1104-1289: four optimizer steps of the device-resident loop against the CPU loop, same batches."""
    optim, train = mod("optim"), mod("train")
    kw = SMALL["gemma3" if which == "muon_wsd" else "llama"]
    rmodel, model = build_pair(ref, kw, seed=6, std=0.1)
    seqs = batches(ref, kw["vocab"], 21, 8, seed=10, mask_every=7)
    sched = ref.wsd_schedule(1, 1, 2, 0.1) if which == "muon_wsd" else None
    if which == "adamw":
        ropt = ref.AdamW(rmodel.params(), lr=1e-3, beta2=0.95, weight_decay=0.1)
        hopt = optim.AdamWHip(gpu, model.params(), lr=1e-3, beta2=0.95, weight_decay=0.1)
    else:
        rm, ra = rmodel.param_groups()
        hm, ha = model.param_groups()
        ropt = ref.Muon(rm, ra, lr=0.01, aux={"lr": 3e-3})
        hopt = optim.MuonHip(gpu, hm, ha, lr=0.01, aux={"lr": 3e-3})
    rh = ref.train_lm(rmodel, ropt, seqs, 2, 4, schedule=sched)
    hh = train.train_lm_hip_resident(model, gpu, hopt, seqs, 4, 2, 21, schedule=sched, stacked=(which == "adamw"))
    for a, b in zip(hh, rh):
        assert abs(a - b) <= 1e-3 * abs(b), (hh, rh)
    hopt.sync_weights_to_host()
    for n, p in rmodel.named_params():
        # Adam's g/(|g|+eps) and Newton-Schulz both amplify rounding-level gradient differences: weights after
        # four steps are held to 1e-3 relative L2, the loss curve above to the north-star 1e-3
        assert_close(model.p[n].data, p.data, f"{which} trajectory weight {n}", rel_l2=1e-3, max_rel=2e-2)


def test_fifty_step_loss_curve(gpu, ref):
    """north-star gate: 50-step loss curves within 1e-3 relative (AdamW, stacked micro-batches on the device,
    sequential on the CPU)."""
    optim, train = mod("optim"), mod("train")
    kw = dict(arch="llama", vocab=64, hidden=32, layers=2, heads=4, kv_heads=2, head_dim=8, ffn=64, rope_base=1e4)
    rmodel, model = build_pair(ref, kw, seed=0, std=0.02, jitter_gains=False)
    rng = ref.Mulberry32(3)
    seqs = []
    for _ in range(100):                      # a learnable stream: the next token is a fixed function of the current
        t = int(rng() * 64)
        ids = []
        for _ in range(17):
            ids.append(t)
            t = (t * 5 + 3) % 64
        seqs.append((ids[:-1], ids[1:]))
    ropt = ref.AdamW(rmodel.params(), lr=3e-3, beta2=0.95, weight_decay=0.1)
    hopt = optim.AdamWHip(gpu, model.params(), lr=3e-3, beta2=0.95, weight_decay=0.1)
    rh = ref.train_lm(rmodel, ropt, seqs, 2, 50)
    hh = train.train_lm_hip_resident(model, gpu, hopt, seqs, 50, 2, 16, stacked=True)
    worst = max(abs(a - b) / abs(b) for a, b in zip(hh, rh))
    assert worst <= 1e-3, worst
    assert rh[-1] < rh[0]


@pytest.mark.parametrize("which", ["llama_adamw", "gemma3_muon"])
def test_resume_through_gguf_and_optstate_is_bit_identical(gpu, ref, which):
    """A run checkpointed after two steps as an F32 GGUF (llama: Q/K rows permuted out and back) plus the .optstate
    sidecar bytes, rebuilt from those bytes alone and continued for two more steps, ends on the same losses and the same
    weights, bit for bit, as the uninterrupted four-step run. rms_eps is a power of two: the file stores it as f32."""
    optim, train, arch, gguf = mod("optim"), mod("train"), mod("arch"), mod("gguf")
    kw = dict(SMALL["gemma3" if which == "gemma3_muon" else "llama"], rms_eps=2.0 ** -20)
    seqs = batches(ref, kw["vocab"], 21, 8, seed=21, mask_every=6)
    sched = ref.wsd_schedule(1, 1, 2, 0.1)
    tok = dict(tokens=[f"t{i}" for i in range(kw["vocab"])], merges=[], bosId=0, eosId=1)

    def make_opt(model):
        if which == "llama_adamw":
            return optim.AdamWHip(gpu, model.params(), lr=1e-3, beta2=0.95, weight_decay=0.1)
        hm, ha = model.param_groups()
        return optim.MuonHip(gpu, hm, ha, lr=0.01, aux={"lr": 3e-3})

    def state_bytes(opt):
        st = opt.export_state()
        if which == "llama_adamw":
            st = {"muonMomentum": [], "adamM": st["m"], "adamV": st["v"], "adamT": st["t"]}
        return optim.serialize_opt_state(st)

    def restore(opt, raw):
        st = optim.deserialize_opt_state(raw)
        opt.import_state({"m": st["adamM"], "v": st["adamV"], "t": st["adamT"]} if which == "llama_adamw" else st)

    _, full = build_pair(ref, kw, seed=8, std=0.1)
    fopt = make_opt(full)
    hist_full = train.train_lm_hip_resident(full, gpu, fopt, seqs, 4, 2, 21, schedule=sched, stacked=True)
    fopt.sync_weights_to_host()

    _, first = build_pair(ref, kw, seed=8, std=0.1)
    opt1 = make_opt(first)
    hist_a = train.train_lm_hip_resident(first, gpu, opt1, seqs[:4], 2, 2, 21, schedule=sched, stacked=True)
    opt1.sync_weights_to_host()
    blob, side = gguf.export_gguf(first, tok, "f32", max_seq=64), state_bytes(opt1)
    del first, opt1

    second, cfg, max_seq, _ = gguf.load_model_from_gguf(blob)
    assert gguf.config_matches(arch.ModelConfig(**kw), cfg, 64, max_seq) is None
    opt2 = make_opt(second)
    restore(opt2, side)
    hist_b = train.train_lm_hip_resident(second, gpu, opt2, seqs[4:], 2, 2, 21, schedule=lambda s: sched(s + 2), stacked=True)
    opt2.sync_weights_to_host()
    assert hist_a + hist_b == hist_full
    for n, p in full.named_params():
        assert second.p[n].data.tobytes() == p.data.tobytes(), n


# microConfig() of gpu-parity.ts:307-325
MICRO = dict(arch="gemma3", vocab=50, hidden=32, layers=2, heads=4, kv_heads=2, head_dim=8, ffn=64, rope_base=1e6,
             rope_base_local=1e4, rms_eps=1e-6, sliding_window=32, swa_pattern=2)
MUON_HYPER = dict(lr=0.02, momentum=0.95, aux={"lr": 3e-3, "weight_decay": 0.0, "clip": 1.0})


def micro_tokens(ref, seed):
    r = ref.Mulberry32(seed)
    return [int(math.floor(r() * MICRO["vocab"])) for _ in range(160)]


@pytest.mark.parametrize("stacked", [False, True])
def test_qk_clip_trajectory(gpu, ref, stacked):
    """gpu-parity.ts:1233-1289: the logit clip is host math on the QK-norm gains between optimizer steps; tau = 0.5
    triggers from initialisation (gains of one give proxy 1), so every step clips on both paths, windows are drawn
    from the same token array by the same generator, and the trained model's proxies end at or under tau."""
    ag, optim, train = mod("autograd"), mod("optim"), mod("train")
    tokens = micro_tokens(ref, 0x70CC)
    rmodel, model = build_pair(ref, MICRO, seed=5, jitter_gains=False)
    rm, ra = rmodel.param_groups()
    hm, ha = model.param_groups()
    ropt = ref.Muon(rm, ra, **MUON_HYPER)
    hopt = optim.MuonHip(gpu, hm, ha, **MUON_HYPER)
    rh = ref.train_lm(rmodel, ropt, ref.draw_windows(tokens, 8, ref.Mulberry32(7), 8), 2, 4, qk_clip_tau=0.5)
    log = []
    hh = train.train_lm_hip_resident(model, gpu, hopt, train.WindowSampler(tokens, 8, ag.mulberry32(7)), 4, 2, 8,
                                     stacked=stacked, qk_clip_tau=0.5, history=log)
    assert [r["step"] for r in log] == [0, 1, 2, 3] and [r["loss"] for r in log] == hh
    for a, b in zip(hh, rh):
        assert abs(a - b) <= 1e-3 + 1e-3 * abs(b), (hh, rh)
    for n, p in rmodel.named_params():
        assert_close(model.p[n].data, p.data, f"qk-clip trajectory weight {n}", rel_l2=1e-3, max_rel=2e-2)
    for q, k in model.qk_norms():
        assert train.qk_logit_scale(q.data, k.data, MICRO["head_dim"]) <= 0.5 + 1e-4
    # and without the clip the gains would have stayed near one: the clip is what moved them
    assert max(float(np.abs(q.data).max()) for q, _ in model.qk_norms()) < 0.9


def test_checkpoint_cadence(gpu, ref):
    """gpu-parity.ts:2512-2563: the step trigger and the wall-clock trigger are ORed, never fire at step 0, and
    the weights are on the host when the callback runs."""
    ag, optim, train = mod("autograd"), mod("optim"), mod("train")
    tokens = micro_tokens(ref, 0x5EC2)

    def fired_at(**cadence):
        _, model = build_pair(ref, MICRO, seed=5, jitter_gains=False)
        hm, ha = model.param_groups()
        hit, moved = [], []
        w0 = model.p["tokenEmbd"].data.copy() if "tokenEmbd" in model.p else None

        def on_checkpoint(step):
            hit.append(step)
            if w0 is not None:
                moved.append(not np.array_equal(model.p["tokenEmbd"].data, w0))
        train.train_lm_hip_resident(model, gpu, optim.MuonHip(gpu, hm, ha, **MUON_HYPER),
                                    train.WindowSampler(tokens, 8, ag.mulberry32(7)), 6, 1, 8, log_every=100,
                                    on_checkpoint=on_checkpoint, **cadence)
        assert all(moved)               # trained weights, not the initial host copy
        return hit

    # a step takes milliseconds, so 1e-3 ms is due at every step and 1e9 ms at none
    assert fired_at(checkpoint_every=2) == [2, 4]
    assert fired_at(checkpoint_every_ms=1e-3) == [1, 2, 3, 4, 5]
    assert fired_at(checkpoint_every=2, checkpoint_every_ms=1e9) == [2, 4]
    assert fired_at(checkpoint_every=10 ** 9, checkpoint_every_ms=1e-3) == [1, 2, 3, 4, 5]
    assert fired_at() == []
    assert fired_at(checkpoint_every_ms=1e9) == []


def test_reclaim_transients_changes_no_bit(gpu, ref):
    """gpu-parity.ts:438-565: freeing each micro-batch's intermediates mid-step only recycles pool buffers earlier.
    Three micro-batches per step (two reclaim boundaries), Muon + AdamW, four steps: the dense loss, the chunked loss
    (chunk 16 over a vocabulary of 50: four spans with a ragged tail, tied readout accumulating into the embedding
    gradient) and the recomputed graph each give the same losses and weights with reclaim on and off, to the bit; the
    recomputed losses equal the dense ones to the bit, the chunked ones to 1e-3."""
    ag, optim, train = mod("autograd"), mod("optim"), mod("train")
    tokens = micro_tokens(ref, 0x5EC1)

    def run(reclaim, loss_chunk=0, recompute=False):
        _, model = build_pair(ref, MICRO, seed=5, jitter_gains=False)
        hm, ha = model.param_groups()
        ag.set_checkpointing(recompute)
        try:
            hist = train.train_lm_hip_resident(model, gpu, optim.MuonHip(gpu, hm, ha, **MUON_HYPER),
                                               train.WindowSampler(tokens, 8, ag.mulberry32(7)), 4, 3, 8, loss_chunk=loss_chunk,
                                               stacked=False, reclaim=reclaim)
        finally:
            ag.set_checkpointing(False)
        return hist, [p.data.copy() for p in model.params()]

    dense_off, dense_on = run(False), run(True)
    assert dense_on[0] == dense_off[0]
    assert all(np.array_equal(a, b) for a, b in zip(dense_on[1], dense_off[1]))
    chunk_off, chunk_on = run(False, 16), run(True, 16)
    assert chunk_on[0] == chunk_off[0]
    assert all(np.array_equal(a, b) for a, b in zip(chunk_on[1], chunk_off[1]))
    for a, b in zip(chunk_off[0], dense_off[0]):
        assert abs(a - b) <= 1e-3 + 1e-3 * abs(b), (chunk_off[0], dense_off[0])
    rc_off, rc_on = run(False, 0, True), run(True, 0, True)
    assert rc_off[0] == dense_off[0] and rc_on[0] == dense_off[0]
    assert all(np.array_equal(a, b) for a, b in zip(rc_on[1], dense_off[1]))
