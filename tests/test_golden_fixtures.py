"""The committed fixtures of tests/golden/.

reference_vectors.json holds the literal vectors of the reference's own tests for this path; the oracle (and the host
code that has a counterpart there) must meet each of them. The .npz files hold seeded inputs with the oracle's outputs
(written by tests/golden/make_oracle_fixtures.py): on the CPU the oracle must still reproduce them to the bit, on the GPU
the device path is compared with the files themselves, at the same tolerances as against the live oracle."""
import importlib.util
import json
import math
import os

import numpy as np
import pytest

from gpu_common import LOSS_REL, assert_close, mod

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
VEC = json.load(open(os.path.join(GOLDEN, "reference_vectors.json")))


def _generator():
    spec = importlib.util.spec_from_file_location("make_oracle_fixtures", os.path.join(GOLDEN, "make_oracle_fixtures.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def _load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


# ---------------------------------------------------------------- reference literals (CPU)

def test_reference_ce_vectors(ref):
    c = VEC["ce_closed_form"]
    for gap in c["gaps"]:
        row = np.float32([gap if v == "gap" else v for v in c["row"]])
        exact = math.log(math.exp(gap) + 2 + math.exp(-3)) + 3
        assert abs(ref.cross_entropy(ref.Tensor(row, [1, 4], True), [c["target"]]).data[0] - exact) < c["tolerance"]
        q = c["soft_teacher_prob"]
        soft = ref.soft_cross_entropy(ref.Tensor(row, [1, 4], True), [c["target"]], [q], 1).data[0]
        assert abs(soft - q * exact) < c["tolerance"]
    d = VEC["ce_device_case"]
    z = np.float32(d["logits"])
    exact = (math.log(math.exp(90) + 2 + math.exp(-3)) + 3 + math.log(math.exp(60) + math.e + 2)) / 2
    assert abs(ref.cross_entropy(ref.Tensor(z, [2, 4], True), d["targets"]).data[0] - exact) < d["tolerance"]
    k = VEC["ce_mean_times_kept"]
    assert sum(1 for t in k["targets"] if t >= 0) == k["kept"]
    rng = ref.Mulberry32(3)
    zz = rng.fill_randn([len(k["targets"]), 20], 0.8)
    mean = ref.cross_entropy(ref.Tensor(zz, list(zz.shape), True), k["targets"]).data[0]
    z64 = zz.astype(np.float64)
    nll = sum(math.log(np.exp(z64[t] - z64[t].max()).sum()) + z64[t].max() - z64[t, g] for t, g in enumerate(k["targets"]) if g >= 0)
    assert abs(mean * k["kept"] - nll) < 1e-5


def test_reference_schedule_clip_and_f16_vectors(ref):
    w = VEC["wsd"]
    s = ref.wsd_schedule(w["warmup"], w["stable"], w["decay"], w["floor"])
    assert all(abs(s(i) - e) < w["tolerance"] for i, e in enumerate(w["expected"]))
    q = VEC["qk_clip"]
    train = mod("train")
    hd = q["head_dim"]
    for scale in (ref.qk_logit_scale, train.qk_logit_scale):
        assert abs(scale(np.ones(hd, np.float32), np.ones(hd, np.float32), hd) - q["proxy_at_unit_gains"]) <= q["tolerance"]
        assert abs(scale(np.full(hd, q["q_gain"], np.float32), np.full(hd, q["k_gain"], np.float32), hd) - q["proxy_inflated"]) <= q["tolerance"]
    G = mod("gguf")
    f = VEC["f16_bits"]
    for v, bits in f["exact"]:
        assert int(G.f32_to_f16_bits(np.float32([v]))[0]) == bits
        assert float(G.f16_bits_to_f32(np.uint16([bits]))[0]) == v
    assert int(G.f32_to_f16_bits(np.float32([f["overflow"][0]]))[0]) == f["overflow"][1]
    assert float(G.f16_bits_to_f32(G.f32_to_f16_bits(np.float32([f["max_normal"]])))[0]) == f["max_normal"]


def test_case_tables_match_the_generator():
    gen = _generator()
    assert [list(s) for s in gen.NS_SHAPES] == VEC["newton_schulz_case"]["shapes"]
    assert VEC["adamw_case"]["grad_scales"] == [0.5, 0.05, 0.01]


def test_oracle_reproduces_the_committed_fixtures(ref):
    """Bit for bit: the oracle is single-threaded here and its arithmetic order is fixed."""
    files = _generator().build_all(ref)
    assert sorted(files) == sorted(f for f in os.listdir(GOLDEN) if f.endswith(".npz"))
    for fn, arrays in files.items():
        have = _load(fn)
        assert sorted(have) == sorted(arrays), fn
        for k, a in arrays.items():
            assert have[k].dtype == np.asarray(a).dtype and np.array_equal(have[k], a), f"{fn}:{k}"


# ---------------------------------------------------------------- device against the files (GPU)

@pytest.mark.gpu
@pytest.mark.parametrize("name", ["llama", "qwen3", "gemma3"])
@pytest.mark.parametrize("stacked", [False, True])
def test_device_step_against_committed_fixture(gpu, name, stacked):
    gen = _generator()
    fx = _load(f"step_{name}.npz")
    ag, arch = mod("autograd"), mod("arch")
    model = arch.Model(arch.ModelConfig(**gen.STEP_MODELS[name]), {k[2:]: v for k, v in fx.items() if k.startswith("w:")})
    ids, tg = fx["ids"], fx["targets"]
    B, T = ids.shape
    gpu.install()
    try:
        if stacked:
            losses = [arch.sequence_loss(model, ids.reshape(-1), tg.reshape(-1), 0, T)]
            ag.backward(losses[0], 1.0 / B)
        else:
            losses = []
            for b in range(B):
                losses.append(arch.sequence_loss(model, ids[b], tg[b], 0))
                ag.backward(losses[-1], 1.0 / B)
        gpu.sync(losses)
    finally:
        gpu.uninstall()
    lv = np.concatenate([l.data for l in losses])
    assert np.all(np.abs(lv - fx["loss"]) <= LOSS_REL * np.abs(fx["loss"])), (lv, fx["loss"])
    for n, p in model.named_params():
        assert_close(p.grad, fx["g:" + n], f"{name} stacked={stacked} grad {n}")


@pytest.mark.gpu
def test_device_adamw_against_committed_fixture(gpu):
    ag, optim = mod("autograd"), mod("optim")
    fx = _load("adamw_3step.npz")
    c = VEC["adamw_case"]
    ps = [ag.Tensor(fx[f"w0:{i}"], s, True) for i, s in enumerate(c["shapes"])]
    opt = optim.AdamWHip(gpu, ps, lr=c["lr"], weight_decay=c["weight_decay"], clip=c["clip"])
    for step in range(3):
        for i, p in enumerate(ps):
            gpu.write_state_buffer(gpu.buffers_for(p)["grad"], fx[f"g{step}:{i}"])
            gpu._entries[p].grad_init = True
        opt.record_step()
        opt.sync_weights_to_host()
        for i, p in enumerate(ps):
            assert_close(p.data, fx[f"w{step + 1}:{i}"], f"AdamW step {step + 1} tensor {i}")
    st = opt.export_state()
    for i in range(len(ps)):
        assert_close(st["m"][i], fx[f"m:{i}"], "first moment")
        assert_close(st["v"][i], fx[f"v:{i}"], "second moment")


@pytest.mark.gpu
def test_device_newton_schulz_against_committed_fixture(gpu):
    lib = mod("lib")
    fx = _load("newton_schulz.npz")
    for m, n in VEC["newton_schulz_case"]["shapes"]:
        G = fx[f"in:{m}x{n}"]
        b_in, b_out = gpu.create_state_buffer(G.nbytes), gpu.create_state_buffer(G.nbytes)
        gpu.write_state_buffer(b_in, G)
        lib.check(gpu.ctx, lib.lib.gt_newton_schulz(gpu.ctx, m, n, VEC["newton_schulz_case"]["steps"], b_in, b_out), "gt_newton_schulz")
        # five quintic iterations amplify the f32 accumulation-order difference: 2e-5 relative L2
        assert_close(gpu.read_state_buffer(b_out, m * n), fx[f"out:{m}x{n}"], f"NS {m}x{n}", rel_l2=2e-5, max_rel=1e-4)
