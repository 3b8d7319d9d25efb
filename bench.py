#!/usr/bin/env python3
"""Headline benchmark: train tokens/s of one full training step (forward + backward + AdamW, loss read
back every step) at the SmolLM2-135M shape, seq 2048 x batch 8, fp32, on one MI355X, plus the roofline of the
dominant kernel (the backward GEMMs, against the FP32 MFMA peak) and a CPU baseline beside it.

    python bench.py [--gpus 1] [--steps 20] [--warmup 3]

One JSON line on stdout. `value` is tokens/s with every input already resident in HBM at the start of the timed
region (weights, optimizer state and the token batches' ids are uploaded by the step itself: 128 KiB per step).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG = "gguf-trainer_amd"

PEAK_FP32_MFMA = 157.3e12      # MI355X dense FP32 matrix peak, FLOP/s
PEAK_HBM = 8.0e12              # B/s
PEAK_BF16_MFMA = 2500e12       # MI355X dense bf16 matrix peak, FLOP/s (what the bf16-piece leg executes on)
PROF_SAMPLE = 4                # the timed region brackets about 1 in 4 launches of a GEMM label with HIP events
# L2-miss traffic per launch (bytes) of the backward GEMM labels that lead the step, from two rocprofv3 --pmc passes over
# this file made separately (FETCH_SIZE x 2.00 + WRITE_SIZE x 1.00, the factors read off a plain streaming kernel of known
# size; see profiles/bench_smollm2_135m_pmc_fetch_write.txt). Averages over the shapes each label serves in the step: the NN
# label is 30 summed q+k+v products, 30 summed gate+up products, the 30 dX of the o projection and the readout's; the grouped
# TN labels include their reduction pass.
MEASURED_TRAFFIC = {"gemm.nn.128x96x32": (30 * (2 * 50010.9 + 36864.5) + 30 * (2 * 174988.0 + 36864.5) + 30 * (2 * 29882.9 + 36865.5) +
                                          (2 * 3508313.8 + 36865.5)) / 91 * 1024,
                    "gemm.tn.group.128x96.splitk": ((24 * 1200.5 + 18 * 943.5) / 42 + 151.9) * 1048576,
                    "gemm.tn.group.64x192.splitk": ((21 * 959.7 + 12 * 1193.4) / 33 + 151.9) * 1048576}

SMOLLM2 = dict(arch="llama", vocab=49152, hidden=576, layers=30, heads=9, kv_heads=3, head_dim=64, ffn=1536,
               rope_base=100000.0, rms_eps=1e-5, tie=True)
SEQ, BATCH = 2048, 8
# The other model-sized benchmark configs, runnable with --config (the default line is configs[3]).
GEMMA3_95M = dict(arch="gemma3", vocab=32768, hidden=640, layers=12, heads=10, kv_heads=2, head_dim=64, ffn=2048,
                  rope_base=1e6, rope_base_local=1e4, sliding_window=512, swa_pattern=6, rms_eps=1e-6, tie=True)
QWEN3_06B = dict(arch="qwen3", vocab=151936, hidden=1024, layers=28, heads=16, kv_heads=8, head_dim=128, ffn=3072,
                 rope_base=1e6, rms_eps=1e-6, tie=True)
WORKLOADS = {
    3: dict(name="configs[3]: SmolLM2-135M llama shape, fwd+bwd+AdamW, seq 2048 x batch 8, fp32", model=SMOLLM2, batch=8),
    2: dict(name="configs[2]: Gemma3-style 95M, --recompute, Muon (5 NS steps) + AdamW, seq 2048 x batch 8, fp32",
            model=GEMMA3_95M, batch=8, muon=True, recompute=True),
    4: dict(name="configs[4]: Qwen3-0.6B shape, base frozen, LoRA rank 16 on q/k/v/o/gate/up/down + AdamW, 60% loss mask, "
                 "seq 2048 x batch 4, fp32", model=QWEN3_06B, batch=4, lora=16, mask=0.6),
}


def synth_weights(arch, cfg, seed=0):
    """Random-init weights of the named architecture: matrices N(0, 0.02), norm gains 1."""
    rs = np.random.RandomState(seed)
    w = {}
    for n in arch.param_names(cfg):
        shp = arch.param_shape(cfg, n)
        w[n] = np.ones(shp, np.float32) if len(shp) == 1 else (0.02 * rs.standard_normal(shp)).astype(np.float32)
    return w


def zipf_tokens(vocab, n, seed, s=1.1):
    """Zipf(1.1) over the vocabulary by inverse CDF, on a fixed permutation of the ids."""
    rs = np.random.RandomState(seed)
    p = 1.0 / np.arange(1, vocab + 1, dtype=np.float64) ** s
    cdf = np.cumsum(p / p.sum())
    perm = np.random.RandomState(12345).permutation(vocab)
    return perm[np.minimum(np.searchsorted(cdf, rs.rand(n)), vocab - 1)].astype(np.int64)


def cpu_baseline():
    """The CPU oracle (a C restatement of the reference's CPU ops, kind "port") on the host cores, on bounded samples of
    the same workloads, each measured directly and labelled with what was sampled:
      * one SmolLM2 layer forward + backward on a whole sequence of T = 2048 (attention at its real length), the tied
        readout + cross-entropy on 512 of the sequence's 2048 rows (that part is linear in rows), AdamW over one layer's
        and the table's parameters: `value` is tokens/s of the whole step, 30 x layer + readout + optimizer;
      * benchmark configs[1]'s three isolated backward kernels on 1024 of their 16384 rows (dX and dW of the MLP
        up-projection, softmax-CE backward over 49152 logits, RMSNorm backward);
      * benchmark configs[0] (the tiny llama model the reference itself can run on a CPU): one full step, 4 x 128 tokens.
    OpenMP over the host cores where loop iterations write disjoint outputs (the reference's CPU path is
    single-threaded: `single_thread` divides by the ratio measured on one layer at T = 256). Reported, never a target."""
    from oracle import ref
    cores = max(1, min(ref.max_threads(), len(os.sched_getaffinity(0))))
    rs = np.random.RandomState(0)
    cfg = ref.ModelConfig(**dict(SMOLLM2, layers=1))
    T = SEQ

    def weights_for(c):
        w = {}
        for n, shp in [("tokenEmbd", [c.vocab, c.hidden]), ("outputNorm", [c.hidden])] + \
                      [(f"L{l}.{k}", s_) for l in range(c.layers) for k, s_ in ref.layer_shapes(c).items()]:
            w[n] = np.ones(shp, np.float32) if len(shp) == 1 else (0.02 * rs.standard_normal(shp)).astype(np.float32)
        return w

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    model = ref.Model(cfg, weights=weights_for(cfg))
    ids = zipf_tokens(cfg.vocab, T + 1, 1)
    ref.set_threads(cores)
    ref.PARALLEL_BWD = True
    REPS = 3

    def stats(fn):
        """one untimed warm-up, then REPS timed runs: (min, median, all)"""
        fn()
        ts = sorted(timed(fn) for _ in range(REPS))
        return ts[0], ts[len(ts) // 2], ts
    try:
        # (1) one layer, whole sequence
        h0 = ref.Tensor((0.5 * rs.standard_normal((T, cfg.hidden))).astype(np.float32), [T, cfg.hidden], True)
        up = rs.standard_normal(T * cfg.hidden).astype(np.float32)

        def layer():
            o = model._block(h0, model.layers[0], 0, T)()
            ref.backward_from(o, up)
        layer_min, layer_med, layer_all = stats(layer)
        # (2) readout + loss on a quarter of the rows
        RS = 512
        hs = ref.Tensor((0.5 * rs.standard_normal((RS, cfg.hidden))).astype(np.float32), [RS, cfg.hidden], True)

        def head():
            loss = ref.cross_entropy(ref.linear(ref.rms_norm(hs, model.outputNorm, cfg.rms_eps), model.tokenEmbd), ids[1:RS + 1].tolist())
            ref.backward(loss, 1.0)
        head_min, head_med, head_all = stats(head)
        # (3) AdamW over the layer + table + final norm
        opt = ref.AdamW(model.params(), lr=1e-3, beta2=0.95, weight_decay=0.1)
        opt_min, opt_med, opt_all = stats(opt.step)
        n_layer = sum(p.size for p in model.layers[0].values())
        n_head = model.tokenEmbd.size + model.outputNorm.size
        opt_scale = (n_head + 30 * n_layer) / (n_head + n_layer)

        def per_token_of(tl, th, to):
            return (30 * tl + th * (T / RS)) / T + to * opt_scale / (BATCH * SEQ)
        per_token = per_token_of(layer_med, head_med, opt_med)          # `value`: the median run
        per_token_best = per_token_of(layer_min, head_min, opt_min)
        t_layer, t_head, t_opt = layer_med, head_med * (T / RS), opt_med
        # (4) configs[1]: isolated backward kernels on 1024 of 16384 rows
        R1, H, F, V = 1024, 576, 1536, 49152
        x = ref.Tensor(rs.standard_normal((R1, H)).astype(np.float32), [R1, H], True)
        w = ref.Tensor(rs.standard_normal((F, H)).astype(np.float32), [F, H], True)
        y = ref.linear(x, w)
        y.grad[:] = rs.standard_normal(R1 * F).astype(np.float32)
        t_lin = timed(y._backward)
        z = ref.Tensor((2.0 * rs.standard_normal((R1, V))).astype(np.float32), [R1, V], True)
        tg = rs.randint(0, V, R1)
        tg[rs.rand(R1) < 0.1] = -1
        ce = ref.cross_entropy(z, tg.tolist())
        ce.grad[:] = 1.0
        t_ce = timed(ce._backward)
        xn = ref.Tensor(rs.standard_normal((R1, H)).astype(np.float32), [R1, H], True)
        wn = ref.Tensor((1 + 0.3 * rs.standard_normal(H)).astype(np.float32), [H], True)
        yn = ref.rms_norm(xn, wn, 1e-5)
        yn.grad[:] = rs.standard_normal(R1 * H).astype(np.float32)
        t_rms = timed(yn._backward)
        # (5) ratio of the literal serial loops on one thread to the OpenMP form, one layer at T = 256
        T1 = 256
        h1 = ref.Tensor(h0.data[:T1 * cfg.hidden].copy(), [T1, cfg.hidden], True)

        def layer_small():
            o = model._block(h1, model.layers[0], 0, T1)()
            ref.backward_from(o, up[:T1 * cfg.hidden])
        t_small_mt = timed(layer_small)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    t_small_1t = timed(layer_small)
    # (6) configs[0]: the tiny llama model, one full step on one thread, as the reference runs it
    tiny = ref.ModelConfig(arch="llama", vocab=512, hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=352, rope_base=1e4, rms_eps=1e-5)
    tmodel = ref.Model(tiny, ref.Mulberry32(0), std=0.02)
    topt = ref.AdamW(tmodel.params(), lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0)
    tt = rs.randint(0, 512, (4, 129))

    def tiny_step():
        for b in range(4):
            ref.backward(ref.sequence_loss(tmodel, tt[b, :-1].tolist(), tt[b, 1:].tolist()), 0.25)
        topt.step()
    t_tiny = timed(tiny_step)
    slowdown = t_small_1t / max(t_small_mt, 1e-9)
    return {"value": round(1.0 / per_token, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "runs": {"warmup": 1, "timed": REPS, "median_tokens_per_s": round(1.0 / per_token, 2), "best_tokens_per_s": round(1.0 / per_token_best, 2),
                     "layer_s": [round(t, 3) for t in layer_all], "readout_s": [round(t, 3) for t in head_all],
                     "adamw_s": [round(t, 4) for t in opt_all]},
            "sample": f"oracle (C restatement of the reference's CPU ops) under OpenMP, each part run once untimed and then {REPS} times "
                      f"(value = from the medians): one SmolLM2 layer fwd+bwd on a whole "
                      f"{T}-token sequence {t_layer:.2f} s (x30), tied readout + cross-entropy fwd+bwd on {RS} of {T} rows "
                      f"{t_head * RS / T:.2f} s (x{T // RS}), AdamW over one layer + table {t_opt:.2f} s (scaled to 134.5 M parameters, once per "
                      f"{BATCH * SEQ} tokens)",
            "single_thread": {"value": round(1.0 / per_token / slowdown, 2), "unit": "tokens/s", "cores": 1,
                              "sample": f"one layer fwd+bwd at T={T1}: the reference's literal serial loops on 1 thread {t_small_1t:.2f} s, the "
                                        f"OpenMP form on {cores} threads {t_small_mt:.2f} s; the {cores}-thread figure divided by that ratio"},
            "configs1_kernels": {"sample": f"{R1} of 16384 rows each, {cores} threads, seconds for the full 16384 rows by linear scaling",
                                 "dX+dW [16384x576x1536] s": round(t_lin * 16384 / R1, 2),
                                 "softmax-CE backward [16384x49152] s": round(t_ce * 16384 / R1, 2),
                                 "RMSNorm backward [16384x576] s": round(t_rms * 16384 / R1, 3)},
            "configs0_step": {"sample": "tiny llama (vocab 512, hidden 128, 2 layers), 4 x 128 tokens, fwd+bwd+AdamW, 1 thread",
                              "seconds": round(t_tiny, 3), "tokens/s": round(512 / t_tiny, 1)}}


def micro_kernels(gpu, L, reps=10, sustained=30):
    """benchmark configs[1]: the isolated backward kernels at the SmolLM2 MLP shape, timed with HIP events on the
    library's stream. fp32 dX = dY.W and dW = dY^T.X with X [16384x576], W [1536x576], dY [16384x1536]; softmax-CE
    backward over logits [16384x49152] with 10% of the targets masked; RMSNorm backward on [16384x576]; SwiGLU
    backward on [16384x1536]. Rates are algorithmic work (FLOP, or bytes each tensor is touched once) over time.
    Two figures per GEMM: `frac` is a single launch between other kernels (each round puts the 6.4 GB cross-entropy
    pass and four streaming kernels between two launches of the same product: cold caches, clocks and power ramping up
    from memory-bound work), `sustained_frac` is `sustained` launches back to back inside one pair of events once the
    clocks have settled on matrix work (see sustained_rate)."""
    import ctypes as C
    rs = np.random.RandomState(7)
    R, H, F, V = 16384, 576, 1536, 49152

    def dev(shape, scale=1.0, dtype=np.float32, data=None):
        a = data if data is not None else (scale * rs.standard_normal(shape)).astype(dtype)
        b = gpu.create_state_buffer(a.nbytes)
        gpu.write_state_buffer(b, a)
        return b

    def zeros(n):
        return gpu.create_state_buffer(4 * n)

    X, W, dY = dev((R, H)), dev((F, H)), dev((R, F))
    dX, dW = zeros(R * H), zeros(F * H)
    gate, up, dgate, dup = dev((R, F)), dev((R, F)), zeros(R * F), zeros(R * F)
    g_n, w_n, rinv, y_n, dx_n, dw_n = dev((R, H)), dev((H,)), zeros(R), zeros(R * H), zeros(R * H), zeros(H)
    blk = (2.0 * rs.standard_normal(1 << 24)).astype(np.float32)
    z = gpu.create_state_buffer(4 * R * V)
    for off in range(0, 4 * R * V, blk.nbytes):
        n = min(blk.nbytes, 4 * R * V - off)
        L.check(gpu.ctx, L.lib.gt_h2d(gpu.ctx, z + off, blk.ctypes.data_as(C.c_void_p), n), "h2d")
    dz = zeros(R * V)
    tg = rs.randint(0, V, R).astype(np.int32)
    tg[rs.rand(R) < 0.1] = -1
    tgb = dev(None, data=tg)
    inv = dev(None, data=np.array([1.0 / max(int((tg >= 0).sum()), 1)], np.float32))
    loss, lse = zeros(1), zeros(R)
    c, lib = gpu.ctx, L.lib
    L.check(c, lib.gt_rmsnorm_fwd(c, R, H, 1e-5, X, w_n, y_n, rinv), "rmsnorm")
    L.check(c, lib.gt_ce_fwd(c, R, V, R, z, tgb, inv, loss, lse), "ce")

    def run():
        L.check(c, lib.gt_gemm(c, L.NN, 0, R, H, F, dY, W, dX), "dX")
        L.check(c, lib.gt_gemm(c, L.TN, 0, F, H, R, dY, X, dW), "dW")
        L.check(c, lib.gt_ce_fwd(c, R, V, R, z, tgb, inv, loss, lse), "ce")
        L.check(c, lib.gt_ce_bwd(c, R, V, R, z, tgb, inv, lse, 1.0, dz, 0), "ce.bwd")
        L.check(c, lib.gt_rmsnorm_bwd(c, R, H, X, w_n, g_n, rinv, dx_n, 0, dw_n, 0), "rmsnorm.bwd")
        L.check(c, lib.gt_glu_bwd(c, 0, R * F, dY, gate, up, dgate, 0, dup, 0), "glu.bwd")
        # a plain streaming kernel of known size (read 100.7 MB, write 100.7 MB): the yardstick the FETCH_SIZE /
        # WRITE_SIZE counters are scaled by
        L.check(c, lib.gt_scale_fwd(c, R * F, gate, 1.0, dgate), "scale")
        # and the same copy over as many bytes as RMSNorm backward moves (113 MB in all): the floor for a launch that small
        L.check(c, lib.gt_add_fwd(c, R * H, X, g_n, dx_n), "add")

    run()
    gpu.start_profile("")
    for _ in range(reps):
        run()
    prof = gpu.stop_profile()

    SETTLE = 150

    def sustained_rate(fn, flop):
        """`sustained` launches of one product back to back inside one event pair, after SETTLE untimed ones: coming from
        memory-bound kernels the chip's clocks take about 25 ms of matrix work to settle (this product: 112-114 TFLOP/s over
        its first ten launches, 130 from the 110th on, by event pairs around consecutive groups of ten)"""
        for _ in range(SETTLE):
            fn()
        ms = C.c_double()
        L.check(c, lib.gt_timer_start(c), "gt_timer_start")
        for _ in range(sustained):
            fn()
        L.check(c, lib.gt_timer_stop(c, C.byref(ms)), "gt_timer_stop")
        return ms.value / sustained, flop * sustained / (ms.value * 1e-3)
    # RMSNorm backward is a 113 MB launch here, 25 us: its ramp and tail weigh as much as for the plain add of the same size
    # above. The same kernel over eight times the rows (906 MB) shows its rate without them.
    R8 = 8 * R
    x8, g8, dx8, rinv8 = zeros(R8 * H), zeros(R8 * H), zeros(R8 * H), zeros(R8)
    for off in range(0, 4 * R8 * H, blk.nbytes):
        nb_ = min(blk.nbytes, 4 * R8 * H - off)
        L.check(c, lib.gt_h2d(c, x8 + off, blk.ctypes.data_as(C.c_void_p), nb_), "h2d")
        L.check(c, lib.gt_h2d(c, g8 + off, blk.ctypes.data_as(C.c_void_p), nb_), "h2d")
    L.check(c, lib.gt_rmsnorm_fwd(c, R8, H, 1e-5, x8, w_n, dx8, rinv8), "rmsnorm")
    big = {}
    for name, fn in (("rmsnorm.bwd", lambda: L.check(c, lib.gt_rmsnorm_bwd(c, R8, H, x8, w_n, g8, rinv8, dx8, 0, dw_n, 0), "rmsnorm.bwd")),
                     ("add", lambda: L.check(c, lib.gt_add_fwd(c, R8 * H, x8, g8, dx8), "add"))):
        for _ in range(3):
            fn()
        ms8 = C.c_double()
        L.check(c, lib.gt_timer_start(c), "gt_timer_start")
        for _ in range(10):
            fn()
        L.check(c, lib.gt_timer_stop(c, C.byref(ms8)), "gt_timer_stop")
        big[name] = ms8.value / 10
    for b8 in (x8, g8, dx8, rinv8):
        L.check(c, lib.gt_free(c, b8), "gt_free")
    flop = 2.0 * R * H * F
    sus = {"gemm.nn": sustained_rate(lambda: L.check(c, lib.gt_gemm(c, L.NN, 0, R, H, F, dY, W, dX), "dX"), flop),
           "gemm.tn": sustained_rate(lambda: L.check(c, lib.gt_gemm(c, L.TN, 0, F, H, R, dY, X, dW), "dW"), flop)}
    # the same two products on the bf16-piece kernels ("gemm.split_bf16"), sustained, for the line's bf16_pieces figures
    gpu.set_option("gemm.split_bf16", 1)
    try:
        sus_p = {"gemm.nn": sustained_rate(lambda: L.check(c, lib.gt_gemm(c, L.NN, 0, R, H, F, dY, W, dX), "dX"), flop),
                 "gemm.tn": sustained_rate(lambda: L.check(c, lib.gt_gemm(c, L.TN, 0, F, H, R, dY, X, dW), "dW"), flop)}
    finally:
        gpu.set_option("gemm.split_bf16", 0)
    out = {}
    names = {"gemm.nn": ("dX = dY.W  [16384x576x1536]", "mfma"), "gemm.tn": ("dW = dY^T.X [1536x576x16384]", "mfma"),
             "ce.bwd": ("softmax-CE backward [16384x49152]", "hbm"), "ce": ("CE forward statistics [16384x49152]", "hbm"),
             "rmsnorm.bwd": ("RMSNorm backward [16384x576]", "hbm"), "glu.bwd": ("SwiGLU backward [16384x1536]", "hbm"),
             "scale": ("copy-like yardstick: out = 1.0*x [16384x1536]", "hbm"),
             "add": ("yardstick at the RMSNorm size: out = a + b [16384x576], 113 MB like RMSNorm backward", "hbm")}
    for label, (ms, cnt, work) in prof.items():
        key = next((k for k in sorted(names, key=len, reverse=True) if label == k or label.startswith(k + ".")), None)
        if key is None or cnt == 0:
            continue
        desc, bound = names[key]
        rate = work / (ms * 1e-3)
        peak = PEAK_FP32_MFMA if bound == "mfma" else PEAK_HBM
        out[desc] = {"kernel": label, "bound": bound, "us_per_launch": round(1e3 * ms / cnt, 1),
                     "achieved": round(rate / 1e12, 3), "unit": "TFLOP/s" if bound == "mfma" else "TB/s",
                     "frac": round(rate / peak, 4)}
        if key in sus:
            out[desc]["launch"] = "single launches, each between a 6.4 GB cross-entropy pass and four streaming kernels (cold)"
            out[desc]["sustained_us_per_launch"] = round(1e3 * sus[key][0], 1)
            out[desc]["sustained_achieved"] = round(sus[key][1] / 1e12, 3)
            out[desc]["sustained_frac"] = round(sus[key][1] / PEAK_FP32_MFMA, 4)
            out[desc]["sustained"] = (f"{sustained} launches back to back inside one event pair, after {SETTLE} untimed ones that let the clocks settle "
                                      f"(the reduction pass of a split-K product included)")
            out[desc]["bf16_pieces_sustained"] = {"us_per_launch": round(1e3 * sus_p[key][0], 1), "achieved": round(sus_p[key][1] / 1e12, 3),
                                                  "frac_of_fp32_mfma_peak": round(sus_p[key][1] / PEAK_FP32_MFMA, 4),
                                                  "executed_frac_of_bf16_mfma_peak": round(6 * sus_p[key][1] / PEAK_BF16_MFMA, 4)}
    for key, desc in (("rmsnorm.bwd", "RMSNorm backward [131072x576] (8x the rows, 10 launches back to back)"),
                      ("add", "yardstick out = a + b [131072x576] (8x the rows, 10 launches back to back)")):
        rate = 12.0 * R8 * H / (big[key] * 1e-3)
        out[desc] = {"kernel": key, "bound": "hbm", "us_per_launch": round(1e3 * big[key], 1), "achieved": round(rate / 1e12, 3), "unit": "TB/s",
                     "frac": round(rate / PEAK_HBM, 4)}
    for b in (X, W, dY, dX, dW, gate, up, dgate, dup, g_n, w_n, rinv, y_n, dx_n, dw_n, z, dz, tgb, inv, loss, lse):
        L.check(c, lib.gt_free(c, b), "gt_free")
    return out


def muon_flop(model):
    """Newton-Schulz work of one Muon step: 5 iterations of A = X X^T (2 r^2 c), A^2 (2 r^3) and (bA + cA^2) X (2 r^2 c)
    per matrix, r = min(rows, cols), c = max(rows, cols)."""
    mu, _ = model.param_groups()
    tot = 0.0
    for p in mu:
        r, c = min(p.shape), max(p.shape)
        tot += 5.0 * (4.0 * r * r * c + 2.0 * r * r * r)
    return tot


def run_workload(mods, config, steps, warmup, a, headline):
    """One training workload on its own backend: `warmup` untimed steps, `steps` timed ones (wall clock around them with the
    device idle on both sides, HIP events on the library's streams around a sample of the GEMM launches), then short legs
    outside the timed region. Returns the pieces of the JSON line."""
    import torch
    ag, hb, arch, optim = mods
    wl = WORKLOADS[config]
    batch = wl["batch"]
    cfg = arch.ModelConfig(**wl["model"])
    model = arch.Model(cfg, synth_weights(arch, cfg))
    n_params = sum(p.size for p in model.params())
    gpu = hb.require_gpu("bench.py", streams=a.streams)
    gpu.batch_linears = not a.no_pair
    gpu.attn_keep_scores = not a.no_keep_scores
    gpu.fuse_sibling_dx = "sibling_dx" not in a.no_fuse
    gpu.fuse_residual_add = "residual_add" not in a.no_fuse
    gpu.alias_add_grads = "add_grads" not in a.no_fuse
    for kv in a.set:
        key, _, val = kv.partition("=")
        gpu.set_option(key, int(val))
    if wl.get("lora"):
        rs = np.random.RandomState(3)
        rank = wl["lora"]
        adapters = {}
        for l in range(cfg.layers):
            for k in arch.MATRIX_KEYS:
                outd, ind = arch.layer_shapes(cfg)[k]
                adapters[f"L{l}.{k}"] = ((0.02 * rs.standard_normal((rank, ind))).astype(np.float32), np.zeros((outd, rank), np.float32))
        trainable = arch.apply_lora(model, rank, 16.0, adapters)
        opt = optim.AdamWHip(gpu, trainable, lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.0, clip=1.0)
    elif wl.get("muon"):
        mu, aux = model.param_groups()
        opt = optim.MuonHip(gpu, mu, aux, lr=0.01, momentum=0.95, nesterov=True, ns_steps=5, aux={"lr": 3e-3})
    else:
        opt = optim.AdamWHip(gpu, model.params(), lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0)
    ag.set_checkpointing(bool(wl.get("recompute")))
    total = steps + warmup
    if config == 3:
        toks = [zipf_tokens(cfg.vocab, batch * (SEQ + 1), 100 + i).reshape(batch, SEQ + 1) for i in range(total)]
    else:
        toks = [np.random.RandomState(100 + i).randint(0, cfg.vocab, (batch, SEQ + 1)).astype(np.int64) for i in range(total)]
    masks = [np.random.RandomState(500 + i).rand(batch, SEQ) < wl["mask"] for i in range(total)] if wl.get("mask") else None

    def step(i, sequential=a.sequential):
        t = toks[i]
        tgt = t[:, 1:].copy()
        if masks is not None:
            tgt[~masks[i]] = -1                 # loss mask: only the kept positions carry a target
        if sequential:
            losses = []
            for b in range(batch):
                loss = arch.sequence_loss(model, t[b, :-1], tgt[b], 0)
                ag.backward(loss, 1.0 / batch)
                losses.append(loss)
        else:
            loss = arch.sequence_loss(model, t[:, :-1].reshape(-1), tgt.reshape(-1), 0, SEQ)
            ag.backward(loss, 1.0 / batch)
            losses = [loss]
        gpu.sync(losses)                     # loss scalars back to the host, as train-gpu.ts:221
        opt.record_step()
        gpu.sync([])
        return float(np.mean(np.concatenate([l.data for l in losses])))

    def timed_leg(n, sequential, first=0):
        gpu.sync([])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(n):
            step((first + i) % total, sequential)
        gpu.sync([])
        torch.cuda.synchronize()
        return time.perf_counter() - t1

    res = {"wl": wl, "batch": batch, "n_params": n_params, "device": gpu.adapter_name}
    gpu.install()
    try:
        losses = [step(i) for i in range(warmup)]
        gpu.sync([])
        torch.cuda.synchronize()
        # HIP events on the library's stream around the GEMM launches of the timed region. A pair of events delays the
        # stream by about 3.5 us (measured: 4.4 ms per step with all 632 GEMM launches bracketed), so about 1 in 4
        # launches of each label is timed (a fixed pseudo-random choice); launch counts and work cover every launch and
        # a label's time is its timed launches' time scaled by all work / timed work
        gpu.set_option("prof.sample", 1 if a.profile_all else PROF_SAMPLE)
        gpu.start_profile("" if a.profile_all else "gemm.")
        t0 = time.perf_counter()
        for i in range(warmup, total):
            losses.append(step(i))
        gpu.sync([])
        torch.cuda.synchronize()
        res["wall"] = time.perf_counter() - t0
        res["prof"] = gpu.stop_profile()
        res["losses"] = losses
        gpu.set_option("prof.sample", 1)
        # the optimizer kernels alone, outside the timed region
        gpu.start_profile("muon" if wl.get("muon") else "adamw")
        step(total - 1)
        op = gpu.stop_profile()
        res["opt_prof"] = op.get("adamw")
        res["opt_sustained"] = None
        if headline and not wl.get("muon") and not wl.get("lora"):
            # ten AdamW steps back to back inside one event pair (gradients as the last backward left them): the kernel's rate
            # without the clock and cache state a whole training step leaves behind
            import ctypes as C
            Lm = importlib.import_module(f"{PKG}.lib")
            gpu.ensure_grads_defined(opt.params)
            ms = C.c_double()
            for _ in range(2):
                Lm.check(gpu.ctx, Lm.lib.gt_adamw_step(gpu.ctx, opt._h, 0.0, 0.5, 0.5), "gt_adamw_step")      # lr 0: the weights stay put
            Lm.check(gpu.ctx, Lm.lib.gt_timer_start(gpu.ctx), "gt_timer_start")
            for _ in range(10):
                Lm.check(gpu.ctx, Lm.lib.gt_adamw_step(gpu.ctx, opt._h, 0.0, 0.5, 0.5), "gt_adamw_step")
            Lm.check(gpu.ctx, Lm.lib.gt_timer_stop(gpu.ctx, C.byref(ms)), "gt_timer_stop")
            res["opt_sustained"] = ms.value / 10
        if wl.get("muon") and op.get("muon"):
            ms, cnt, _ = op["muon"]
            fl = muon_flop(model)
            res["muon"] = {"ms_per_step": round(ms / cnt, 3), "newton_schulz_TFLOP_per_step": round(fl / 1e12, 4),
                           "achieved": round(fl / (ms / cnt * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                           "frac": round(fl / (ms / cnt * 1e-3) / PEAK_FP32_MFMA, 4),
                           "note": "whole gt_muon_step (momentum, normalise, 5 Newton-Schulz iterations, apply) against the "
                                   "Newton-Schulz FLOP 5*(4 r^2 c + 2 r^3) per matrix"}
        # The same step the way the reference's trainer calls a backend (src/backend/train-gpu.ts:200-219): one sequence's
        # forward and backward at a time, B graphs of 2048 rows per step, gradients accumulated, then the optimizer. A short
        # leg outside the headline's timed region; the backend deals the micro-batches to its streams.
        res["call_pattern"] = None
        if headline and not a.sequential and not a.no_call_pattern:
            nseq = max(2, min(6, steps))
            for i in range(2):
                step(i % total, True)
            w1 = timed_leg(nseq, True, 2)
            res["call_pattern"] = {"graph": f"{batch} graphs of {SEQ} rows per step, one sequence at a time, as src/backend/train-gpu.ts:200-219 calls the backend",
                                   "streams": a.streams, "steps": nseq, "value": round(nseq * batch * SEQ / w1, 1), "unit": "tokens/s",
                                   "ms_per_step": round(1e3 * w1 / nseq, 2)}
        # The same stacked step with the library's FP32 products on the bf16 matrix instruction ("gemm.split_bf16": three exact
        # bf16 pieces per operand element, six of the nine piece products, FP32 accumulation; as close to float64 as the FP32
        # MFMA kernels, tests/test_gpu_gemm_bf16_pieces.py). Outside the headline's timed region; the headline stays on FP32 MFMA.
        res["bf16_pieces"] = None
        if not a.sequential and not a.no_bf16_pieces and not any(kv.startswith("gemm.split_bf16") for kv in a.set):
            nb = max(2, min(6, steps))
            gpu.set_option("gemm.split_bf16", 1)
            gpu.set_option("attn.split_bf16", 1)       # and the attention forward and banded dQ product (head dims 64, 128) and dK/dV (64)
            try:
                for i in range(2):
                    step(i % total, False)
                gpu.sync([])
                gpu.set_option("prof.sample", PROF_SAMPLE)
                gpu.start_profile("gemm.")
                w2 = timed_leg(nb, False, 2)
                p2 = gpu.stop_profile()
                # and in the reference's call pattern (one sequence per graph), as the leg above
                w3 = None
                if headline and not a.no_call_pattern:
                    step(0, True)
                    w3 = timed_leg(nb, True, 1)
            finally:
                gpu.set_option("prof.sample", 1)
                gpu.set_option("gemm.split_bf16", 0)
                gpu.set_option("attn.split_bf16", 0)
            _, allb2, per2 = gemm_summary(p2, nb)
            if allb2:
                allb2["executed_frac_of_bf16_mfma_peak"] = round(6 * allb2["achieved"] * 1e12 / PEAK_BF16_MFMA, 4)
            res["bf16_pieces"] = {"what": "the same step with gt_set_option(\"gemm.split_bf16\", 1) and (\"attn.split_bf16\", 1): every aligned FP32 product, "
                                          "and the attention forward and banded dQ product (head dims 64, 128) and dK/dV (64), as six bf16 MFMA products of three-piece operands, FP32 accumulate; "
                                          "same entry points, same parity tolerances",
                                  "steps": nb, "value": round(nb * batch * SEQ / w2, 1), "unit": "tokens/s", "ms_per_step": round(1e3 * w2 / nb, 2),
                                  "all_bwd_gemms": allb2, "per_kernel": per2,
                                  "reference_call_pattern": None if w3 is None else {"steps": nb, "value": round(nb * batch * SEQ / w3, 1), "unit": "tokens/s",
                                                                                     "ms_per_step": round(1e3 * w3 / nb, 2)},
                                  "note": "achieved = algorithmic 2MNK FLOP per second; frac is against the FP32 MFMA peak (157.3 TFLOP/s) and can "
                                          "exceed 1; the kernels execute 6 x that on the bf16 pipes (peak 2500 TFLOP/s)"}
    finally:
        gpu.uninstall()
        ag.set_checkpointing(False)
        if wl.get("lora"):
            arch.clear_lora(model)
    res["gpu"] = gpu
    res["model"] = model
    res["step"] = step
    res["timed_leg"] = timed_leg
    res["total"] = total
    return res


def naive_host_leg(mods, a, nsteps=3, streams=1):
    """What a literal shim over the C ABI gets: the reference's call pattern (one sequence per graph) on ONE stream with
    every host-side hold-back and fusion of HipBackend switched off, so that each autograd op issues its own gt_* call
    in tape order (separate k/v and gate/up products, one dX and one dW launch per linear, unfused residual adds and
    gated activations, separate q and k rotations, add's backward as a launch). Attention still keeps its scores:
    that is a choice inside the attention entry points, not a host fusion. streams > 1: the same literal calls with the
    micro-batches dealt to that many library contexts (the one piece of the host scheduler that needs no knowledge of the graph)."""
    import torch
    ag, hb, arch, optim = mods
    wl = WORKLOADS[3]
    batch = wl["batch"]
    cfg = arch.ModelConfig(**wl["model"])
    model = arch.Model(cfg, synth_weights(arch, cfg))
    gpu = hb.require_gpu("bench.py", streams=streams)
    gpu.batch_linears = gpu.fuse_sibling_dx = gpu.fuse_residual_add = gpu.alias_add_grads = False
    gpu.group_dw = gpu.pair_ropes = gpu.fuse_glu = False
    opt = optim.AdamWHip(gpu, model.params(), lr=1e-3, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0)
    toks = [zipf_tokens(cfg.vocab, batch * (SEQ + 1), 900 + i).reshape(batch, SEQ + 1) for i in range(nsteps + 1)]

    def step(i):
        t = toks[i]
        losses = []
        for b in range(batch):
            loss = arch.sequence_loss(model, t[b, :-1], t[b, 1:], 0)
            ag.backward(loss, 1.0 / batch)
            losses.append(loss)
        gpu.sync(losses)
        opt.record_step()
        gpu.sync([])
    gpu.install()
    try:
        step(0)
        gpu.sync([])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(nsteps):
            step(1 + i)
        gpu.sync([])
        torch.cuda.synchronize()
        w = time.perf_counter() - t0
    finally:
        gpu.uninstall()
        gpu.destroy()
    return {"graph": f"{batch} graphs of {SEQ} rows per step, {'one stream' if streams == 1 else f'{streams} streams'}, one gt_* call per autograd op (no held-back, batched, grouped or fused launches)",
            "steps": nsteps, "value": round(nsteps * batch * SEQ / w, 1), "unit": "tokens/s", "ms_per_step": round(1e3 * w / nsteps, 2)}


def gemm_summary(prof, steps):
    """Backward GEMM labels of a profiled region: the label with the most time, and all of them together."""
    bwd = {k: v for k, v in prof.items() if k.startswith("gemm.nn") or k.startswith("gemm.tn")}
    if not bwd:
        return None, None, None
    dom = max(bwd, key=lambda k: bwd[k][0])
    all_ms = sum(v[0] for v in bwd.values())
    all_work = sum(v[2] for v in bwd.values())
    per = {k: {"TFLOP/s": round(v[2] / (v[0] * 1e-3) / 1e12, 2), "ms_per_step": round(v[0] / steps, 2),
               "launches_per_step": v[1] // steps} for k, v in sorted(prof.items()) if v[0] > 0}
    allb = {"achieved": round(all_work / (all_ms * 1e-3) / 1e12, 3), "ms_per_step": round(all_ms / steps, 2),
            "frac": round(all_work / (all_ms * 1e-3) / PEAK_FP32_MFMA, 4)}
    return dom, allb, per


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--sequential", action="store_true", help="one sequence per graph, as the reference accumulates")
    ap.add_argument("--streams", type=int, default=4,
                    help="HIP streams the backend deals consecutive micro-batches to (matters for --sequential; 1 = one stream)")
    ap.add_argument("--no-call-pattern", action="store_true",
                    help="skip the short extra leg that runs the step the way the reference's trainer calls the backend")
    ap.add_argument("--no-micro", action="store_true", help="skip the isolated-kernel leg (benchmark configs[1] shapes)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short legs over benchmark configs[2] (gemma3-style, Muon) and configs[4] (Qwen3-0.6B, LoRA)")
    ap.add_argument("--no-bf16-pieces", action="store_true",
                    help="skip the short extra leg that reruns the step with the FP32 products on the bf16 matrix instruction")
    ap.add_argument("--naive-host", action="store_true",
                    help="add a leg that runs the reference's call pattern on one stream with every host-side hold-back and fusion off")
    ap.add_argument("--no-pair", action="store_true", help="launch every linear on its own (no batched k/v and gate/up pairs)")
    ap.add_argument("--no-keep-scores", action="store_true",
                    help="attention recomputes Q.K^T in the backward instead of keeping the forward's scores (saves B*Hq*T*T*4 bytes per layer)")
    ap.add_argument("--no-fuse", action="append", default=[], choices=["sibling_dx", "residual_add", "add_grads"],
                    help="switch one of the host-side launch fusions off for an A/B run (repeatable)")
    ap.add_argument("--set", action="append", default=[], metavar="KEY=VALUE",
                    help="library option for an A/B run, e.g. attn.keep_ds=0 (dQ recomputes the scores) or gemm.staged=1")
    ap.add_argument("--profile-all", action="store_true",
                    help="time every kernel label (not only the GEMMs) over the timed region and print the table to stderr")
    ap.add_argument("--config", type=int, default=3, choices=sorted(WORKLOADS),
                    help="index into BASELINE.json configs (default 3, the headline SmolLM2 shape)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(no collectives are part of it: the path would shard over sequences with one gradient sum per step)", file=sys.stderr)
        sys.exit(2)

    import torch  # device plumbing only: make sure a GPU is there before touching the library
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    mods = tuple(importlib.import_module(f"{PKG}.{m}") for m in ("autograd", "hip_backend", "arch", "optim"))
    Lmod = importlib.import_module(f"{PKG}.lib")

    r = run_workload(mods, a.config, a.steps, a.warmup, a, headline=True)
    wl, BATCH, prof, gpu, losses, wall = r["wl"], r["batch"], r["prof"], r["gpu"], r["losses"], r["wall"]
    kernels = None if a.no_micro else micro_kernels(gpu, Lmod)
    if kernels is not None and r["opt_prof"] and a.config == 3:
        ms, cnt, work = r["opt_prof"]
        kernels[f"AdamW step, {r['n_params']} params, clip on"] = {
            "kernel": "adamw", "bound": "hbm", "us_per_launch": round(1e3 * ms / cnt, 1),
            "achieved": round(work / (ms * 1e-3) / 1e12, 3), "unit": "TB/s", "frac": round(work / (ms * 1e-3) / PEAK_HBM, 4),
            "launch": "the one step after a training step (three launches: sum of squares, clip scale, update)"}
        if r.get("opt_sustained"):
            rate = work / cnt / (r["opt_sustained"] * 1e-3)
            kernels[f"AdamW step, {r['n_params']} params, clip on"].update(
                {"sustained_us_per_launch": round(1e3 * r["opt_sustained"], 1), "sustained_achieved": round(rate / 1e12, 3),
                 "sustained_frac": round(rate / PEAK_HBM, 4), "sustained": "10 steps back to back inside one event pair"})
    gpu.destroy()

    if a.profile_all:
        print(f"{'label':30s} {'ms/step':>9s} {'launches/step':>14s} {'T(FLOP|B)/s':>12s}", file=sys.stderr)
        for k, v in sorted(prof.items(), key=lambda kv: -kv[1][0]):
            print(f"{k:30s} {v[0] / a.steps:9.2f} {v[1] / a.steps:14.1f} {v[2] / (v[0] * 1e-3) / 1e12 if v[0] else 0:12.2f}", file=sys.stderr)
    tokens = a.steps * BATCH * SEQ
    # dominant kernel: the backward GEMMs (NN = dX, TN = dW); the one tile shape with the most time stands for it
    dom, allb, per = gemm_summary(prof, a.steps)
    roof = None
    if dom:
        ms, cnt, work = prof[dom]
        ach = work / (ms * 1e-3)
        roof = {"bound": "mfma", "kernel": dom, "achieved": round(ach / 1e12, 3), "peak": PEAK_FP32_MFMA / 1e12,
                "unit": "TFLOP/s", "frac": round(ach / PEAK_FP32_MFMA, 4),
                "traffic": MEASURED_TRAFFIC.get(dom) if a.config == 3 else None,
                "traffic_source": "profiles/bench_smollm2_135m_pmc_fetch_write.txt: two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over "
                                  "this file, made separately; not measured by this run" if a.config == 3 and MEASURED_TRAFFIC.get(dom) else None,
                "launches": int(cnt), "avg_launch_ms": round(ms / cnt, 4),
                "timed_launches": "all" if a.profile_all else f"1 in {PROF_SAMPLE} of each label",
                "all_bwd_gemms": allb, "per_kernel": per}

    # The other model-sized benchmark configs, three timed steps each on a backend of their own, outside the headline's
    # timed region: tokens/s, the backward GEMM label with the most time, and for configs[2] the Muon step.
    other = None
    if a.config == 3 and not a.no_other_configs:
        other = {}
        for ci in (2, 4):
            o = run_workload(mods, ci, 3, 2, a, headline=False)
            o["gpu"].destroy()
            d2, all2, per2 = gemm_summary(o["prof"], 3)
            ent = {"workload": o["wl"]["name"], "steps": 3, "warmup": 2, "value": round(3 * o["batch"] * SEQ / o["wall"], 1), "unit": "tokens/s",
                   "ms_per_step": round(1e3 * o["wall"] / 3, 2), "loss_first": round(o["losses"][0], 4), "loss_last": round(o["losses"][-1], 4)}
            if d2:
                ms2, cnt2, work2 = o["prof"][d2]
                ent["dominant_bwd_gemm"] = {"kernel": d2, "achieved": round(work2 / (ms2 * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                                            "frac": round(work2 / (ms2 * 1e-3) / PEAK_FP32_MFMA, 4), "ms_per_step": round(ms2 / 3, 2),
                                            "launches_per_step": int(cnt2) // 3}
                ent["all_bwd_gemms"] = all2
                ent["per_kernel"] = per2
            if o.get("muon"):
                ent["muon_step"] = o["muon"]
            if o.get("bf16_pieces"):        # the same workload with "gemm.split_bf16" on (Muon's Newton-Schulz products included)
                ent["bf16_pieces"] = {k: o["bf16_pieces"][k] for k in ("steps", "value", "unit", "ms_per_step", "all_bwd_gemms")}
            other[f"configs[{ci}]"] = ent
    naive = naive_host_leg(mods, a) if a.naive_host or (a.config == 3 and not a.no_call_pattern and not a.sequential) else None
    if naive is not None:          # the same literal calls, micro-batches dealt to the backend's streams
        n4 = naive_host_leg(mods, a, streams=a.streams)
        naive["with_streams"] = {"streams": a.streams, "value": n4["value"], "unit": "tokens/s", "ms_per_step": n4["ms_per_step"]}
    out = {
        "metric": "train tokens/s (SmolLM2-135M shape, 2048x8); bwd GEMM % FP32 MFMA peak" if a.config == 3 else
                  "train tokens/s (" + wl["name"].split(":")[0] + ")",
        "value": round(tokens / wall, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(1e3 * wall / a.steps, 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (weights N(0,0.02) random init, tokens Zipf(1.1) over the vocab)",
        "config": {"workload": wl["name"],
                   "params": r["n_params"], "global_batch": BATCH, "seq_len": SEQ,
                   "graph": f"sequential micro-batches on {a.streams} stream(s)" if a.sequential else f"{BATCH} sequences stacked into one {BATCH * SEQ}-row graph",
                   "device": r["device"]},
        "loss_first": round(losses[0], 4), "loss_last": round(losses[-1], 4),
        "reference_call_pattern": r["call_pattern"],
        "naive_host": naive,
        "bf16_pieces": r.get("bf16_pieces"),
        "roofline": roof,
        "muon_step": r.get("muon"),
        "kernels": kernels,
        "other_configs": other,
        "cpu_baseline": None if a.no_cpu else cpu_baseline(),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
