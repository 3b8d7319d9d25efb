"""The option "gemm.split_bf16": the FP32 products of the path on the bf16 matrix instruction, every operand element cut
into three bf16 pieces (exact) and six of the nine piece products kept. Same entry points, same tolerances as the FP32
MFMA kernels: every product kind against float64, the fused forms against their one-by-one counterparts, whole models
against the oracle (loss 1e-5, gradients 1e-5 relative L2 / 1e-4 max), and its error against float64 next to the
FP32 kernels' error."""
import ctypes as C

import numpy as np
import pytest

from gpu_common import assert_close, mod
from test_gpu_model import REAL, SMALL, batches, build_pair, compare, hip_step, ref_step

pytestmark = pytest.mark.gpu


@pytest.fixture()
def pieces(gpu):
    gpu.set_option("gemm.split_bf16", 1)
    yield gpu
    gpu.set_option("gemm.split_bf16", 0)
    gpu.set_option("gemm.splitk", -1)
    gpu.set_option("gemm.sum_min_tiles", -1)


def labels_of(gpu, run):
    gpu.start_profile("gemm.")
    run()
    return set(gpu.stop_profile())


def bufs(gpu, *arrays):
    out = []
    for a in arrays:
        b = gpu.create_state_buffer(a.nbytes)
        gpu.write_state_buffer(b, a)
        out.append(b)
    return out


@pytest.mark.parametrize("M,N,K", [(200, 152, 96), (132, 100, 64), (260, 196, 128), (300, 576, 576), (257, 192, 1536), (128, 384, 32),
                                   (4, 4, 32), (1000, 1536, 64)])
def test_every_kind_store_accumulate_and_k_split_against_float64(pieces, M, N, K):
    """NT / NN / TN on both tile shapes (N a multiple of 192 or not), partial tiles on both edges, one stage only (K = 32),
    store and accumulate, dW cut along K; the profile label says which kernel ran."""
    gpu = pieces
    rs = np.random.RandomState(M + N + K)
    a = rs.standard_normal((M, K)).astype(np.float32)
    b = rs.standard_normal((N, K)).astype(np.float32)
    c0 = rs.standard_normal((M, N)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    da, db, dc = bufs(gpu, a, b, c0)
    for kind, (A, B) in enumerate([(a, b), (a, np.ascontiguousarray(b.T)), (np.ascontiguousarray(a.T), np.ascontiguousarray(b.T))]):
        gpu.write_state_buffer(da, A)
        gpu.write_state_buffer(db, B)
        for splitk in ((-1, 1, 3) if kind == 2 else (-1,)):
            for acc in (0, 1):
                gpu.set_option("gemm.splitk", splitk)
                gpu.write_state_buffer(dc, c0)
                seen = labels_of(gpu, lambda: gpu.gemm(kind, acc, M, N, K, da, db, dc))
                # the direct kernels' condition: whole 16-byte chunks along every operand's contiguous index
                takes = (kind != 2 or M % 4 == 0) and (kind == 0 or N % 4 == 0)
                assert any(".bf16x6" in s for s in seen) == takes, seen
                got = gpu.read_state_buffer(dc, M * N).reshape(M, N)
                assert_close(got, (want + c0 if acc else want).astype(np.float32), f"kind {kind} splitk {splitk} acc {acc} {M}x{N}x{K}")
    for h in (da, db, dc):
        gpu.free_state_buffer(h)


@pytest.mark.parametrize("kind,M,N,K", [(0, 70, 83, 75), (1, 64, 64, 100), (2, 96, 66, 64), (0, 1, 5, 3)])
def test_shapes_the_direct_kernels_do_not_take_stay_on_the_fp32_kernels(pieces, kind, M, N, K):
    """K not a multiple of 32, or an operand whose contiguous index is not whole 16-byte chunks: the register-staged FP32
    kernels as before, with the option on."""
    gpu = pieces
    rs = np.random.RandomState(K)
    a = rs.standard_normal((K, M) if kind == 2 else (M, K)).astype(np.float32)
    b = rs.standard_normal((N, K) if kind == 0 else (K, N)).astype(np.float32)
    want = (a.T if kind == 2 else a).astype(np.float64) @ (b.T if kind == 0 else b).astype(np.float64)
    da, db, dc = bufs(gpu, a, b, np.zeros((M, N), np.float32))
    seen = labels_of(gpu, lambda: gpu.gemm(kind, 0, M, N, K, da, db, dc))
    assert seen and not any(".bf16x6" in s for s in seen), seen
    assert_close(gpu.read_state_buffer(dc, M * N).reshape(M, N), want.astype(np.float32), f"fallback kind {kind}")
    for h in (da, db, dc):
        gpu.free_state_buffer(h)


def test_error_against_float64_next_to_the_fp32_kernels(gpu):
    """Not reduced precision: over the layer's product shapes the rms error of the piece products against float64 stays
    within 1.25 x the FP32 MFMA kernels' own (measured 0.61 - 1.16 x, the same from seed to seed: both accumulate in FP32, in a different order)."""
    rs = np.random.RandomState(7)
    for kind, M, N, K in [(0, 512, 576, 1536), (1, 512, 1536, 576), (2, 576, 576, 16384), (0, 384, 1536, 576)]:
        a = rs.standard_normal((K, M) if kind == 2 else (M, K)).astype(np.float32)
        b = (0.02 * rs.standard_normal((N, K) if kind == 0 else (K, N))).astype(np.float32)
        want = (a.T if kind == 2 else a).astype(np.float64) @ (b.T if kind == 0 else b).astype(np.float64)
        da, db, dc = bufs(gpu, a, b, np.zeros((M, N), np.float32))
        err = []
        try:
            for on in (0, 1):
                gpu.set_option("gemm.split_bf16", on)
                gpu.gemm(kind, 0, M, N, K, da, db, dc)
                got = gpu.read_state_buffer(dc, M * N).reshape(M, N).astype(np.float64)
                err.append(np.sqrt(np.mean((got - want) ** 2)))
        finally:
            gpu.set_option("gemm.split_bf16", 0)
        assert err[1] <= 1.25 * err[0], (kind, M, N, K, err)
        for h in (da, db, dc):
            gpu.free_state_buffer(h)


@pytest.mark.parametrize("scale_a,scale_b", [(1e-12, 1e-9), (1e12, 1e3), (1e-20, 1e15), (0.0, 1.0)])
def test_magnitudes_far_from_one(pieces, scale_a, scale_b):
    """The pieces keep FP32's exponent range: no scaling of the operands is involved. Very small and very large operands give
    the same relative accuracy; a zero operand gives exact zeros."""
    gpu = pieces
    M, N, K = 256, 192, 256
    rs = np.random.RandomState(3)
    a = (scale_a * rs.standard_normal((M, K))).astype(np.float32)
    b = (scale_b * rs.standard_normal((N, K))).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    da, db, dc = bufs(gpu, a, b, np.ones((M, N), np.float32))
    gpu.gemm(0, 0, M, N, K, da, db, dc)
    got = gpu.read_state_buffer(dc, M * N).reshape(M, N)
    if scale_a == 0.0:
        assert not got.any()
    else:
        assert_close(got, want.astype(np.float32), f"scales {scale_a} x {scale_b}")
    for h in (da, db, dc):
        gpu.free_state_buffer(h)


@pytest.mark.parametrize("kind,M,N,K", [(0, 300, 576, 576), (0, 257, 576, 1536), (1, 130, 96, 64), (2, 96, 64, 2048)])
@pytest.mark.parametrize("in_place", [False, True])
def test_product_plus_addend(pieces, kind, M, N, K, in_place):
    """gt_gemm_add through the piece kernels: bit for bit the product into a buffer plus an elementwise add."""
    gpu, lib = pieces, mod("lib")
    rs = np.random.RandomState(M + K)
    a_ = rs.standard_normal((K, M) if kind == 2 else (M, K)).astype(np.float32)
    b_ = rs.standard_normal((N, K) if kind == 0 else (K, N)).astype(np.float32)
    d_ = rs.standard_normal((M, N)).astype(np.float32)
    da, db, dd, dc, dy = bufs(gpu, a_, b_, d_, d_ if in_place else np.zeros_like(d_), d_)
    lib.check(gpu.ctx, lib.lib.gt_gemm_add(gpu.ctx, kind, M, N, K, da, db, dc if in_place else dd, dc), "gt_gemm_add")
    got = gpu.read_state_buffer(dc, M * N).copy()
    lib.check(gpu.ctx, lib.lib.gt_gemm(gpu.ctx, kind, 0, M, N, K, da, db, dy), "gt_gemm")
    y = gpu.read_state_buffer(dy, M * N).copy()
    assert np.array_equal(got, (d_.reshape(-1) + y).astype(np.float32))
    for h in (da, db, dd, dc, dy):
        gpu.free_state_buffer(h)


def test_batch_of_two_and_scaled_write_back(pieces):
    """gt_gemm_batched (the gate and up projections as one launch) against float64 per member."""
    gpu, lib = pieces, mod("lib")
    M, N, K = 300, 192, 576
    rs = np.random.RandomState(9)
    a = rs.standard_normal((M, K)).astype(np.float32)
    b = rs.standard_normal((2, N, K)).astype(np.float32)
    da, db, dc = bufs(gpu, a, b, np.zeros((2, M, N), np.float32))
    lib.check(gpu.ctx, lib.lib.gt_gemm_batched(gpu.ctx, 0, 0, M, N, K, da, 0, db, N * K, dc, M * N, 2), "gt_gemm_batched")
    got = gpu.read_state_buffer(dc, 2 * M * N).reshape(2, M, N)
    for i in range(2):
        assert_close(got[i], (a.astype(np.float64) @ b[i].astype(np.float64).T).astype(np.float32), f"batch member {i}")
    for h in (da, db, dc):
        gpu.free_state_buffer(h)


@pytest.mark.parametrize("kind,M,N,Ks", [(1, 300, 576, (576, 192, 192)), (1, 257, 576, (1536, 1536)), (1, 128, 640, (640, 128, 128)),
                                         (0, 200, 192, (64, 96)), (1, 5600, 576, (576, 192, 192))])
@pytest.mark.parametrize("acc", [0, 1])
def test_summed_products_in_one_chained_loop(pieces, kind, M, N, Ks, acc):
    """gt_gemm_sum: the input gradient of sibling projections as one K loop over all their segments."""
    gpu, lib = pieces, mod("lib")
    rs = np.random.RandomState(M + sum(Ks))
    As = [rs.standard_normal((M, K)).astype(np.float32) for K in Ks]
    Bs = [rs.standard_normal((N, K) if kind == 0 else (K, N)).astype(np.float32) for K in Ks]
    c0 = rs.standard_normal((M, N)).astype(np.float32)
    ha, hb = bufs(gpu, *As), bufs(gpu, *Bs)
    (c,) = bufs(gpu, c0)
    n = len(Ks)
    gpu.set_option("gemm.sum_min_tiles", 0)
    seen = labels_of(gpu, lambda: lib.check(gpu.ctx, lib.lib.gt_gemm_sum(gpu.ctx, kind, acc, M, N, n, (C.c_int * n)(*Ks), (C.c_uint64 * n)(*ha),
                                                                        (C.c_uint64 * n)(*hb), c), "gt_gemm_sum"))
    assert len(seen) == 1 and ".bf16x6" in next(iter(seen)), seen
    want = c0.astype(np.float64) * acc
    for a_, b_ in zip(As, Bs):
        want = want + a_.astype(np.float64) @ (b_.T if kind == 0 else b_).astype(np.float64)
    assert_close(gpu.read_state_buffer(c, M * N).reshape(M, N), want.astype(np.float32), f"sum of {n}")
    for h in ha + hb + [c]:
        gpu.free_state_buffer(h)


@pytest.mark.parametrize("K,shapes", [(16384, [(576, 1536), (1536, 576), (576, 576), (192, 576)]),
                                      (2048, [(576, 1536), (1536, 576), (1536, 576), (576, 576), (576, 576), (192, 576), (192, 576), (576, 1536)]),
                                      (256, [(64, 64), (8, 12)]), (96, [(200, 152), (4, 4), (132, 100)])])
def test_grouped_weight_gradients(pieces, K, shapes):
    """gt_gemm_group: the layer's dW products as one launch over all their tiles, K cut into ranges, store and accumulate
    mixed; each member alone through the same entry point gives the same bits."""
    gpu, lib = pieces, mod("lib")
    rs = np.random.RandomState(K + len(shapes))
    n = len(shapes)
    As = [rs.standard_normal((K, M)).astype(np.float32) for M, N in shapes]
    Bs = [rs.standard_normal((K, N)).astype(np.float32) for M, N in shapes]
    C0 = [rs.standard_normal((M, N)).astype(np.float32) for M, N in shapes]
    accs = [i % 2 for i in range(n)]
    da, db, dc = bufs(gpu, *As), bufs(gpu, *Bs), bufs(gpu, *C0)
    Ms, Ns = (C.c_int * n)(*[m for m, _ in shapes]), (C.c_int * n)(*[n_ for _, n_ in shapes])
    seen = labels_of(gpu, lambda: lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, (C.c_uint64 * n)(*da), (C.c_uint64 * n)(*db),
                                                                          (C.c_uint64 * n)(*dc), (C.c_int * n)(*accs)), "gt_gemm_group"))
    assert any(".bf16x6" in s for s in seen), seen
    got = [gpu.read_state_buffer(b_, c_.size).copy() for b_, c_ in zip(dc, C0)]
    for i in range(n):
        want = As[i].astype(np.float64).T @ Bs[i].astype(np.float64) + (C0[i] if accs[i] else 0)
        assert_close(got[i], want.astype(np.float32), f"group member {i} {shapes[i]}")
        gpu.write_state_buffer(dc[i], C0[i])
        lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, 1, (C.c_int * 1)(shapes[i][0]), (C.c_int * 1)(shapes[i][1]), K, (C.c_uint64 * 1)(da[i]),
                                                 (C.c_uint64 * 1)(db[i]), (C.c_uint64 * 1)(dc[i]), (C.c_int * 1)(accs[i])), "gt_gemm_group")
        assert np.array_equal(gpu.read_state_buffer(dc[i], C0[i].size), got[i]), f"member {i} alone vs in the group"
    for h in da + db + dc:
        gpu.free_state_buffer(h)


@pytest.mark.parametrize("arch_name", ["llama", "qwen3", "gemma3"])
def test_small_models_against_the_oracle(pieces, ref, arch_name):
    kw = SMALL[arch_name]
    rmodel, model = build_pair(ref, kw, seed=1, std=0.1)
    seqs = batches(ref, kw["vocab"], 19, 2, seed=5, mask_every=5)
    lh, gh = hip_step(pieces, model, seqs, True, 19)
    lr, gr = ref_step(ref, rmodel, seqs)
    compare(lh, gh, lr, gr, f"{arch_name} with bf16 pieces")


@pytest.mark.parametrize("name", ["smollm2", "gemma3-window", "qwen3-hd128"])
@pytest.mark.parametrize("stacked", [False, True])
def test_real_head_geometry_against_the_oracle(pieces, ref, name, stacked):
    """Whole graphs at the widths the piece kernels are selected for (576 / 1536 / 640-class rows, 200-token sequences ragged
    against every tile): loss and every gradient tensor at the tolerances of the FP32 kernels."""
    kw = REAL[name]
    rmodel, model = build_pair(ref, kw, seed=11, std=0.05)
    seqs = batches(ref, kw["vocab"], 200, 2, seed=12, mask_every=7)
    seen = set()
    pieces.start_profile("gemm.")
    lh, gh = hip_step(pieces, model, seqs, stacked, 200)
    seen = set(pieces.stop_profile())
    assert any(".bf16x6" in s for s in seen), seen
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        lr, gr = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
    compare(lh, gh, lr, gr, f"{name} stacked={stacked} with bf16 pieces")


@pytest.mark.parametrize("M,N,K1,K2", [(200, 152, 96, 16), (300, 576, 576, 16), (257, 192, 1536, 32), (132, 100, 64, 32), (64, 64, 32, 16),
                                       (260, 196, 128, 8), (300, 576, 192, 24)])
def test_two_segment_products(pieces, M, N, K1, K2):
    """gt_gemm_pair (the LoRA linear and its dX): C (+)= A1.B1 + A2.B2 in one K loop. A second segment of 16 or 32 rides in one
    more stage of the piece kernels (16: the stage's other half is multiplied by zero pieces); 8 and 24 stay on the FP32
    kernels."""
    gpu, L = pieces, mod("lib")
    rs = np.random.RandomState(M + K2)
    a1, b1 = rs.standard_normal((M, K1)).astype(np.float32), rs.standard_normal((N, K1)).astype(np.float32)
    a2, b2 = rs.standard_normal((M, K2)).astype(np.float32), rs.standard_normal((N, K2)).astype(np.float32)
    c0 = rs.standard_normal((M, N)).astype(np.float32)
    want = a1.astype(np.float64) @ b1.astype(np.float64).T + a2.astype(np.float64) @ b2.astype(np.float64).T
    h = bufs(gpu, a1, b1, a2, b2, c0)
    T = lambda x: np.ascontiguousarray(x.T)
    for kind, ops in enumerate([(a1, b1, a2, b2), (a1, T(b1), a2, T(b2))]):
        for buf, arr in zip(h, ops):
            gpu.write_state_buffer(buf, arr)
        for acc in (0, 1):
            gpu.write_state_buffer(h[4], c0)
            seen = labels_of(gpu, lambda: L.check(gpu.ctx, L.lib.gt_gemm_pair(gpu.ctx, kind, acc, M, N, K1, h[0], h[1], K2, h[2], h[3], h[4]), "gt_gemm_pair"))
            assert any(".bf16x6" in s for s in seen) == (K2 in (16, 32)), seen
            got = gpu.read_state_buffer(h[4], M * N).reshape(M, N)
            assert_close(got, (want + c0 if acc else want).astype(np.float32), f"pair kind {kind} acc {acc} {M}x{N}x({K1}+{K2})")
    for b in h:
        gpu.free_state_buffer(b)


@pytest.mark.parametrize("recompute", [False, True])
def test_lora_against_the_oracle(pieces, ref, recompute):
    """Rank-16 adapters on a model of real widths (the two-segment forward and dX, the rank products on their own kernels)."""
    ag, arch = mod("autograd"), mod("arch")
    kw = REAL["smollm2"]
    rmodel, model = build_pair(ref, kw, seed=5, std=0.05)
    rank, alpha = 16, 16.0
    rmap, rparams = ref.attach_lora(rmodel, rank, alpha, ref.Mulberry32(11), a_std=0.05)
    rng = ref.Mulberry32(12)
    for a, b, _ in rmap.values():
        b.data[:] = rng.fill_randn([b.size], 0.05)
    adapters = {}
    for l, Lr in enumerate(rmodel.layers):
        for k in ref.MATRIX_KEYS:
            a, b, _ = rmap[id(Lr[k])]
            adapters[f"L{l}.{k}"] = (a.data.copy(), b.data.copy())
    aux = arch.apply_lora(model, rank, alpha, adapters)
    ref.set_lora_adapters(rmap)
    seqs = batches(ref, kw["vocab"], 200, 2, seed=8, mask_every=3)
    ref.PARALLEL_BWD = True
    ref.set_threads(min(16, ref.max_threads()))
    try:
        pieces.start_profile("gemm.")
        lh, _ = hip_step(pieces, model, seqs, True, 200, recompute=recompute)
        seen = set(pieces.stop_profile())
        lr, _ = ref_step(ref, rmodel, seqs)
    finally:
        ref.PARALLEL_BWD = False
        ref.set_threads(1)
        ref.set_lora_adapters({})
        arch.clear_lora(model)
    assert any(".bf16x6" in s for s in seen), seen
    assert np.all(np.abs(lh - lr) <= 1e-5 * np.abs(lr))
    for i, (h, r) in enumerate(zip(aux, rparams)):
        assert_close(h.grad, r.grad, f"lora adapter {i} with bf16 pieces")


@pytest.mark.parametrize("m,n", [(128, 640), (640, 128), (200, 72), (640, 640), (64, 2048)])
def test_newton_schulz_on_the_piece_kernels(pieces, ref, m, n):
    """Muon's Newton-Schulz products (batched, with the scaled write-back b A + c A.A and a X + B.X) at the gemma widths."""
    import test_gpu_optim
    test_gpu_optim.test_newton_schulz(pieces, ref, m, n)


def test_muon_trajectory_on_the_piece_kernels(pieces, ref):
    import test_gpu_optim
    test_gpu_optim.test_four_step_trajectory_vs_cpu_trainer(pieces, ref, "muon_wsd")


def test_fifty_step_loss_curve_on_the_piece_kernels(pieces, ref):
    """The 50-step loss curve gate (1e-3 relative) with every aligned product of the tiny model on the piece kernels."""
    import test_gpu_optim
    test_gpu_optim.test_fifty_step_loss_curve(pieces, ref)


def test_recompute_on_and_off_stay_bit_identical(pieces, ref):
    """The grouped dW products' K split follows K alone on the piece kernels too: with and without recomputed regions the
    host groups different sets of products, and the gradients may not differ by a bit."""
    import test_gpu_model
    test_gpu_model.test_recompute_is_bit_identical_and_matches(pieces, ref, "llama")


def test_two_runs_give_the_same_bits(pieces):
    gpu = pieces
    rs = np.random.RandomState(1)
    M, N, K = 640, 576, 4096
    a, b = rs.standard_normal((K, M)).astype(np.float32), rs.standard_normal((K, N)).astype(np.float32)
    da, db, dc = bufs(gpu, a, b, np.zeros((M, N), np.float32))
    runs = []
    for _ in range(2):
        gpu.gemm(2, 0, M, N, K, da, db, dc)          # dW with a K split: partials summed in split order
        runs.append(gpu.read_state_buffer(dc, M * N).copy())
    assert np.array_equal(runs[0], runs[1])
    for h in (da, db, dc):
        gpu.free_state_buffer(h)


# ---- "attn.split_bf16": the attention forward (head dims 64 and 128), dK/dV (64) and the banded dQ product on the same instruction ----

@pytest.fixture()
def attn_pieces(gpu):
    gpu.set_option("attn.split_bf16", 1)
    yield gpu
    gpu.set_option("attn.split_bf16", 0)
    gpu.set_option("attn.splits", -1)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 700, 4, 2, 64, 0), (2, 333, 6, 2, 64, 300), (1, 1024, 9, 3, 64, 0), (3, 129, 2, 1, 64, 33),
                                                  (1, 512, 3, 3, 64, 512), (1, 300, 4, 2, 128, 0), (2, 200, 8, 8, 128, 77), (1, 640, 16, 8, 128, 0)])
@pytest.mark.parametrize("splits", [-1, 1, 5])
def test_attention_forward_pieces_ragged_windows_gqa_splits(attn_pieces, ref, B, T, Hq, Hkv, hd, window, splits):
    """The head-dim-64 cases of the matrix-core attention tests with the forward on bf16 pieces: ragged T, windows that cut tiles, GQA,
    stacked sequences, split launches; output and all three gradients (the backward reads the forward's output and statistic)
    against the oracle at the FP32 kernels' tolerances."""
    import test_gpu_ops
    test_gpu_ops.test_attention_mfma_shapes(attn_pieces, ref, B, T, Hq, Hkv, hd, window, splits)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 1, 2, 1, 64, 0), (2, 31, 4, 2, 64, 0), (1, 65, 2, 1, 64, 0), (1, 97, 3, 1, 64, 40),
                                                  (1, 128, 2, 1, 64, 1), (2, 160, 4, 4, 64, 1000), (1, 127, 2, 2, 128, 0), (1, 129, 2, 1, 128, 128)])
def test_attention_forward_pieces_tile_edges(attn_pieces, ref, B, T, Hq, Hkv, hd, window):
    import test_gpu_ops
    test_gpu_ops.test_attention_mfma_tile_edges(attn_pieces, ref, B, T, Hq, Hkv, hd, window)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 256, 4, 2, 64, 0), (2, 384, 6, 2, 64, 100), (1, 640, 2, 2, 64, 129), (1, 1024, 9, 3, 64, 0),
                                                  (2, 256, 4, 2, 128, 0), (1, 384, 2, 1, 128, 130)])
@pytest.mark.parametrize("splits,keep_ds", [(1, 1), (3, 1), (1, 0)])
def test_attention_forward_pieces_kept_scores(attn_pieces, ref, B, T, Hq, Hkv, hd, window, splits, keep_ds):
    """The kept scores the piece forward writes feed the piece dK/dV kernel; without them dK/dV is the FP32 kernel that recomputes.
    Same output and statistic bit for bit with and without keeping them, gradients to the parity bound, the first sequence against
    the oracle. (Not window 1, where dq and dk are exactly zero and the comparison is between two kernels' rounding residues.)"""
    import test_gpu_ops
    test_gpu_ops.test_attention_kept_scores_equals_recomputed(attn_pieces, ref, B, T, Hq, Hkv, hd, window, splits, keep_ds)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 256, 4, 2, 64, 0), (2, 384, 6, 2, 64, 100), (1, 512, 2, 1, 64, 127), (1, 768, 2, 1, 64, 300),
                                                  (2, 256, 4, 2, 128, 0), (1, 384, 2, 1, 128, 130)])
@pytest.mark.parametrize("acc,splits", [(0, 1), (1, 1), (0, 5), (1, 3)])
def test_attention_pieces_kept_score_gradients(attn_pieces, ref, B, T, Hq, Hkv, hd, window, acc, splits):
    """dK/dV on pieces writes the score gradients the banded dQ product reads: against the pair that recomputes them and the oracle.
    (Window 1, where dq is exactly zero and the two pairs are compared on their rounding residue alone, is left to the FP32 kernels'
    test: the dQ kernel that recomputes stays on FP32 MFMA, so the residues differ.)"""
    import test_gpu_ops
    test_gpu_ops.test_attention_backward_kept_ds_equals_recomputed(attn_pieces, ref, B, T, Hq, Hkv, hd, window, acc, splits)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window,keep_ds", [(1, 256, 4, 2, 64, 0, 1), (2, 128, 3, 3, 64, 0, 1), (2, 256, 6, 2, 64, 70, 0), (8, 256, 9, 3, 64, 0, 1),
                                                          (1, 256, 4, 2, 128, 0, 1), (2, 256, 2, 1, 128, 70, 1)])
@pytest.mark.parametrize("acc", [0, 1])
def test_attention_pieces_rotations_in_the_write_backs(attn_pieces, B, T, Hq, Hkv, hd, window, keep_ds, acc):
    import test_gpu_ops
    test_gpu_ops.test_attention_backward_with_the_rotations_backward_in_its_write_backs(attn_pieces, B, T, Hq, Hkv, hd, window, keep_ds, acc)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 2048, 9, 3, 64, 0), (2, 1024, 6, 2, 64, 0), (1, 2048, 10, 2, 64, 1500), (1, 1024, 4, 2, 128, 0)])
def test_attention_pieces_banded_dq_cut_into_parts(attn_pieces, B, T, Hq, Hkv, hd, window):
    """The banded dQ product on pieces (128 x hd tiles, wavefronts of 64 x 64), its key ranges cut into parts for small launches."""
    import test_gpu_ops
    try:
        test_gpu_ops.test_banded_dq_product_cut_into_parts(attn_pieces, B, T, Hq, Hkv, hd, window)
    finally:
        attn_pieces.set_option("attn.band_splits", -1)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window,path", [(2, 2048, 9, 3, 64, 0, "kept-scores"), (1, 2048, 10, 2, 64, 512, "kept-scores"),
                                                       (1, 2048, 9, 3, 64, 0, "recompute"), (1, 2048, 16, 8, 128, 0, "kept-scores")])
def test_attention_forward_pieces_full_length(attn_pieces, ref, B, T, Hq, Hkv, hd, window, path):
    import test_gpu_production_shapes
    test_gpu_production_shapes.test_attention_full_length_vs_oracle(attn_pieces, ref, B, T, Hq, Hkv, hd, window, path)


@pytest.mark.parametrize("name", ["smollm2", "gemma3-window", "qwen3-hd128"])
def test_whole_models_with_both_options(pieces, attn_pieces, ref, name):
    test_real_head_geometry_against_the_oracle(pieces, ref, name, True)


def test_backend_factory_switch(ref):
    """require_gpu(..., bf16_pieces=True): both options set on every context of the backend; a step on it matches the oracle."""
    hb = mod("hip_backend")
    g = hb.require_gpu("the bf16-piece factory test", streams=2, bf16_pieces=True)
    try:
        kw = REAL["smollm2"]
        rmodel, model = build_pair(ref, kw, seed=3, std=0.05)
        seqs = batches(ref, kw["vocab"], 200, 2, seed=4, mask_every=7)
        g.start_profile("")
        lh, gh = hip_step(g, model, seqs, False, 200)          # one sequence per graph: both streams
        seen = set(g.stop_profile())
        assert any(".bf16x6" in s for s in seen), seen
        ref.PARALLEL_BWD = True
        ref.set_threads(min(16, ref.max_threads()))
        try:
            lr, gr = ref_step(ref, rmodel, seqs)
        finally:
            ref.PARALLEL_BWD = False
            ref.set_threads(1)
        compare(lh, gh, lr, gr, "factory switch")
    finally:
        g.destroy()
