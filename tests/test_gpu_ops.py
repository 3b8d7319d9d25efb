"""Per-op parity, HIP backend (through the C ABI) against the CPU oracle on identical seeded inputs:
the op cases of tests/gpu-parity.ts:654-930 and the edge cases it names."""
import ctypes as C
import math

import numpy as np
import pytest

from gpu_common import assert_close, backward_from, mod, op_case

pytestmark = pytest.mark.gpu


def R(ref, seed):
    rng = ref.Mulberry32(seed)
    return lambda *s, sc=0.8: rng.fill_randn(list(s), sc)


@pytest.mark.parametrize("T,ind,outd", [(70, 83, 75), (64, 64, 64), (1, 5, 3), (257, 128, 192), (128, 576, 1536),
                                        (130, 1536, 576), (33, 16, 200), (512, 40, 16), (300, 1000, 7)])
def test_linear(gpu, ref, T, ind, outd):
    """GEMM NT forward, NN dX, TN dW; 70x83 . (75x83)^T is the ragged case of gpu-parity.ts:654-672."""
    r = R(ref, T * 7 + ind)
    op_case(gpu, ref, [r(T, ind), r(outd, ind)], lambda ag, x, w: ag.linear(x, w), lambda rf, x, w: rf.linear(x, w),
            f"linear {T}x{ind}x{outd}")


def test_linear_frozen_weight_and_split_k(gpu, ref):
    """dW with a long K (rows) and a small output takes the split-K path; a frozen weight gets no dW."""
    r = R(ref, 5)
    op_case(gpu, ref, [r(4096, 48), r(40, 48)], lambda ag, x, w: ag.linear(x, w), lambda rf, x, w: rf.linear(x, w), "linear split-K")
    op_case(gpu, ref, [r(96, 48), r(40, 48)], lambda ag, x, w: ag.linear(x, w), lambda rf, x, w: rf.linear(x, w),
            "linear frozen", frozen=(1,))


@pytest.mark.parametrize("M,N,K", [(200, 152, 200), (130, 100, 72), (70, 83, 75), (257, 193, 101), (200, 152, 96), (132, 100, 64),
                                   (260, 196, 128)])
def test_gemm_every_tile_shape_and_kind(gpu, M, N, K):
    """Every tile configuration of the GEMM, NT / NN / TN, store and accumulate, split-K 1 and 3, on shapes that leave
    partial tiles on both edges and a K tail (aligned leading dimensions take the vectorised loaders with the
    steady-state loop, odd ones the tested loaders), against a float64 product."""
    rs = np.random.RandomState(M + N + K)
    a = rs.standard_normal((M, K)).astype(np.float32)
    b = rs.standard_normal((N, K)).astype(np.float32)
    c0 = rs.standard_normal((M, N)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    da, db, dc = (gpu.create_state_buffer(x.nbytes) for x in (a, b, c0))
    try:
        for kind, (A, B) in enumerate([(a, b), (a, np.ascontiguousarray(b.T)), (np.ascontiguousarray(a.T), np.ascontiguousarray(b.T))]):
            gpu.write_state_buffer(da, A)
            gpu.write_state_buffer(db, B)
            for tile in range(14):
                for splitk in ((1, 3) if kind == 2 else (1,)):
                    for acc in (0, 1):
                        # staged = 1 pins the register-staged kernels; 0 lets the aligned shapes (K a multiple of 32, whole
                        # 16-byte chunks) take the kernels that load operands straight into LDS where the tile has one
                        for staged in ((0, 1) if K % 32 == 0 else (0,)):
                            gpu.set_option("gemm.tile", tile)
                            gpu.set_option("gemm.splitk", splitk)
                            gpu.set_option("gemm.staged", staged)
                            gpu.write_state_buffer(dc, c0)
                            gpu.gemm(kind, acc, M, N, K, da, db, dc)
                            got = gpu.read_state_buffer(dc, M * N).reshape(M, N)
                            assert_close(got, (want + c0 if acc else want).astype(np.float32),
                                         f"gemm kind {kind} tile {tile} splitk {splitk} acc {acc} staged {staged} {M}x{N}x{K}")
    finally:
        gpu.set_option("gemm.tile", -1)
        gpu.set_option("gemm.splitk", -1)
        gpu.set_option("gemm.staged", 0)


@pytest.mark.parametrize("K,shapes", [(16384, [(576, 1536), (1536, 576), (1536, 576), (576, 576), (576, 576), (192, 576), (192, 576)]),
                                      (2048, [(576, 1536), (1536, 576), (1536, 576), (576, 576), (576, 576), (192, 576), (192, 576), (576, 1536)]),
                                      (256, [(64, 64), (8, 12)]), (96, [(200, 152), (4, 4), (132, 100)]),
                                      (100, [(64, 64), (32, 96)]), (64, [(30, 64), (64, 64)]),
                                      (128, [(64, 96)] * 11)])
@pytest.mark.parametrize("splitk", [-1, 1, 3])
def test_gemm_group_equals_the_products_one_by_one(gpu, K, shapes, splitk):
    """gt_gemm_group: the weight gradients of consecutive linears as one launch, against one gt_gemm per product (same
    tile arithmetic per output element when the K split is the same: compared at 1e-5 / 1e-4 since the split of a
    grouped product follows K alone and a single gt_gemm's follows its shape), against each product alone through the
    same entry point (bit for bit: what a product shares its launch with does not enter its result) and against float64. The seven dW shapes of a SmolLM2 layer at 16384 and at
    2048 rows (a full group of eight), tiny and ragged outputs next to large ones, and the cases that go product by
    product: K not a multiple of 32, M not a multiple of 4, more than eight products. Store and accumulate mixed in one
    group; every tile shape a group can take."""
    lib = mod("lib")
    rs = np.random.RandomState(K + len(shapes))
    n = len(shapes)
    As = [rs.standard_normal((K, M)).astype(np.float32) for M, N in shapes]
    Bs = [rs.standard_normal((K, N)).astype(np.float32) for M, N in shapes]
    C0 = [rs.standard_normal((M, N)).astype(np.float32) for M, N in shapes]
    accs = [i % 2 for i in range(n)]
    da = [gpu.create_state_buffer(a_.nbytes) for a_ in As]
    db = [gpu.create_state_buffer(b_.nbytes) for b_ in Bs]
    dc = [gpu.create_state_buffer(c_.nbytes) for c_ in C0]
    for b_, a_ in zip(da + db, As + Bs):
        gpu.write_state_buffer(b_, a_)
    want = [a_.astype(np.float64).T @ b_.astype(np.float64) + (c_ if acc else 0) for a_, b_, c_, acc in zip(As, Bs, C0, accs)]
    Ms, Ns = (C.c_int * n)(*[m for m, _ in shapes]), (C.c_int * n)(*[n_ for _, n_ in shapes])
    aa, bb, cc, ac = (C.c_uint64 * n)(*da), (C.c_uint64 * n)(*db), (C.c_uint64 * n)(*dc), (C.c_int * n)(*accs)
    gpu.set_option("gemm.splitk", splitk)
    try:
        for tile in ((-1, 6, 7, 8, 11, 12, 13) if K == 256 or K == 96 else (-1,)):
            gpu.set_option("gemm.tile", tile)
            for b_, c_ in zip(dc, C0):
                gpu.write_state_buffer(b_, c_)
            lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, aa, bb, cc, ac), "gt_gemm_group")
            got = [gpu.read_state_buffer(b_, c_.size).copy() for b_, c_ in zip(dc, C0)]
            for i in range(n):
                assert_close(got[i], want[i], f"group member {i} {shapes[i]} tile {tile} vs float64")
        gpu.set_option("gemm.tile", -1)
        # a product's bits do not depend on the company it has in the launch: each one alone, through the same entry point
        for i in range(n):
            gpu.write_state_buffer(dc[i], C0[i])
            lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, 1, (C.c_int * 1)(shapes[i][0]), (C.c_int * 1)(shapes[i][1]), K,
                                                     (C.c_uint64 * 1)(da[i]), (C.c_uint64 * 1)(db[i]), (C.c_uint64 * 1)(dc[i]),
                                                     (C.c_int * 1)(accs[i])), "gt_gemm_group")
            assert np.array_equal(gpu.read_state_buffer(dc[i], C0[i].size), got[i]), f"member {i} alone vs in the group"
        gpu.set_option("gemm.group", 0)
        for b_, c_ in zip(dc, C0):
            gpu.write_state_buffer(b_, c_)
        lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, aa, bb, cc, ac), "gt_gemm_group")
        single = [gpu.read_state_buffer(b_, c_.size).copy() for b_, c_ in zip(dc, C0)]
        for i in range(n):
            assert_close(got[i], single[i], f"group member {i} vs its own launch")
        if splitk == 1:          # no K split on either side: the same arithmetic per output element
            assert all(np.array_equal(g_, s_) for g_, s_ in zip(got, single))
    finally:
        gpu.set_option("gemm.group", 1)
        gpu.set_option("gemm.tile", -1)
        gpu.set_option("gemm.splitk", -1)
    with pytest.raises(lib.HipError, match="overlap"):
        cc2 = (C.c_uint64 * n)(*([dc[0]] * n))
        lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, aa, bb, cc2, ac), "gt_gemm_group")
    if n >= 2 and shapes[0][0] * shapes[0][1] > 4:
        with pytest.raises(lib.HipError, match="overlap"):      # the second output starts inside the first
            cc3 = (C.c_uint64 * n)(*([dc[0], dc[0] + 16] + dc[2:]))
            lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, aa, bb, cc3, ac), "gt_gemm_group")
    if K % 32 == 0:
        gpu.set_option("gemm.tile", 3)                           # a register-staged tile: the grouped launch has none such
        try:
            with pytest.raises(lib.HipError, match="pins tile 3"):
                lib.check(gpu.ctx, lib.lib.gt_gemm_group(gpu.ctx, 2, n, Ms, Ns, K, aa, bb, cc, ac), "gt_gemm_group")
        finally:
            gpu.set_option("gemm.tile", -1)


@pytest.mark.parametrize("rows,K,r", [(16, 64, 16), (100, 192, 16), (257, 1024, 16), (333, 128, 8), (64, 64, 3), (129, 256, 32),
                                      (200, 320, 20), (70, 48, 16), (50, 64, 40), (90, 100, 16), (2100, 576, 16)])
def test_rank_products(gpu, rows, K, r):
    """The rank-r products of the LoRA linear against float64: h = alpha x s^T for both layouts of s, p (+)= h^T y in both
    output orientations, store and accumulate; rows and ranks that leave partial 16-blocks, K that does and does not
    take the streaming kernels (48, 100: the GEMM fallback; r = 40: too wide), several row slices (2100 rows)."""
    L = mod("lib")
    rs = np.random.RandomState(rows + K + r)
    x = rs.standard_normal((rows, K)).astype(np.float32)
    s = rs.standard_normal((r, K)).astype(np.float32)
    hh = rs.standard_normal((rows, r)).astype(np.float32)
    p0 = rs.standard_normal((r, K)).astype(np.float32)
    bx, bs, bh, bp = (gpu.create_state_buffer(a.nbytes) for a in (x, s, hh, p0))
    bo = gpu.create_state_buffer(rows * r * 4)
    gpu.write_state_buffer(bx, x)
    gpu.write_state_buffer(bh, hh)
    want_h = 0.37 * (x.astype(np.float64) @ s.astype(np.float64).T)
    for kmajor, arr in ((0, s), (1, np.ascontiguousarray(s.T))):
        gpu.write_state_buffer(bs, arr)
        gpu.write_state_buffer(bo, np.full((rows, r), 7.0, np.float32))
        L.check(gpu.ctx, L.lib.gt_rank_down(gpu.ctx, rows, K, r, bx, bs, kmajor, 0.37, bo), "gt_rank_down")
        assert_close(gpu.read_state_buffer(bo, rows * r).reshape(rows, r), want_h.astype(np.float32), f"rank_down kmajor {kmajor} {rows}x{K}x{r}")
    want_p = hh.astype(np.float64).T @ x.astype(np.float64)
    for tr in (0, 1):
        for acc in (0, 1):
            base = p0 if not tr else np.ascontiguousarray(p0.T)
            gpu.write_state_buffer(bp, base)
            L.check(gpu.ctx, L.lib.gt_rank_grad(gpu.ctx, rows, K, r, bh, bx, tr, acc, bp), "gt_rank_grad")
            got = gpu.read_state_buffer(bp, r * K).reshape((K, r) if tr else (r, K))
            want = (want_p.T if tr else want_p) + (base if acc else 0)
            assert_close(got, want.astype(np.float32), f"rank_grad transpose {tr} acc {acc} {rows}x{K}x{r}")
    rc = L.lib.gt_rank_down(gpu.ctx, 0, K, r, bx, bs, 0, 1.0, bo)
    assert rc != 0 and b"gt_rank_down" in L.lib.gt_last_error(gpu.ctx)


def test_held_back_rank_gradient_sums_equal_the_direct_ones(gpu):
    """gt_rank_grad_slices / gt_rank_grad_parts / gt_rank_slices_group: the partial products of several adapter gradients
    summed by one launch give, bit for bit, what gt_rank_grad gives each of them (both orientations, store and accumulate,
    different shapes in one group); shapes that do not go through partial sums report zero slices; malformed groups fail."""
    import ctypes as C
    L = mod("lib")
    lib, c = L.lib, gpu.ctx
    rs = np.random.RandomState(5)
    cases = [(2100, 576, 16, 0, 0), (2100, 576, 16, 1, 1), (4096, 1024, 16, 1, 0), (3000, 192, 8, 0, 1), (2500, 320, 20, 0, 0)]
    parts, nsl, lens, dsts, accs, wants = [], [], [], [], [], []
    for rows, K, r, tr, acc in cases:
        h = rs.standard_normal((rows, r)).astype(np.float32)
        y = rs.standard_normal((rows, K)).astype(np.float32)
        p0 = rs.standard_normal(r * K).astype(np.float32)
        bh, by, bd, bw = (gpu.create_state_buffer(a.nbytes) for a in (h, y, p0, p0))
        gpu.write_state_buffer(bh, h)
        gpu.write_state_buffer(by, y)
        gpu.write_state_buffer(bd, p0)
        gpu.write_state_buffer(bw, p0)
        L.check(c, lib.gt_rank_grad(c, rows, K, r, bh, by, tr, acc, bw), "gt_rank_grad")
        wants.append(gpu.read_state_buffer(bw, r * K))
        ns = C.c_int(-1)
        L.check(c, lib.gt_rank_grad_slices(c, rows, K, r, by, C.byref(ns)), "gt_rank_grad_slices")
        assert ns.value >= 2, (rows, K, r, ns.value)
        bp = gpu.create_state_buffer(ns.value * r * K * 4)
        L.check(c, lib.gt_rank_grad_parts(c, rows, K, r, bh, by, tr, bp), "gt_rank_grad_parts")
        parts.append(bp); nsl.append(ns.value); lens.append(r * K); dsts.append(bd); accs.append(acc)
    n = len(cases)
    L.check(c, lib.gt_rank_slices_group(c, n, (L.buf * n)(*parts), (C.c_int * n)(*nsl), (C.c_int * n)(*lens), (L.buf * n)(*dsts),
                                        (C.c_int * n)(*accs)), "gt_rank_slices_group")
    for i, (rows, K, r, tr, acc) in enumerate(cases):
        got = gpu.read_state_buffer(dsts[i], r * K)
        assert got.tobytes() == wants[i].tobytes(), f"held-back sums differ from gt_rank_grad: {cases[i]}"
    # nothing to hold back: one slice (few rows), or a shape that takes the general GEMM
    for rows, K, r in ((64, 576, 16), (2100, 100, 16), (2100, 576, 40)):
        ns = C.c_int(-1)
        L.check(c, lib.gt_rank_grad_slices(c, rows, K, r, parts[0], C.byref(ns)), "gt_rank_grad_slices")
        assert ns.value == 0, (rows, K, r, ns.value)
    assert lib.gt_rank_grad_parts(c, 64, 576, 16, parts[0], parts[0], 0, parts[0]) != 0
    assert b"single slice" in lib.gt_last_error(c)
    two = (L.buf * 2)(dsts[0], dsts[0])
    assert lib.gt_rank_slices_group(c, 2, (L.buf * 2)(parts[0], parts[1]), (C.c_int * 2)(nsl[0], nsl[1]), (C.c_int * 2)(lens[0], lens[1]),
                                    two, (C.c_int * 2)(0, 0)) != 0
    assert b"write the same gradient" in lib.gt_last_error(c)
    L.check(c, lib.gt_rank_slices_group(c, 0, None, None, None, None, None), "empty group")


@pytest.mark.parametrize("M,N,K1,K2", [(200, 152, 96, 16), (130, 100, 72, 5), (257, 193, 101, 33), (64, 64, 16, 16), (260, 196, 128, 8),
                                       (132, 100, 64, 32), (300, 576, 192, 24), (200, 152, 96, 40)])
def test_gemm_pair(gpu, M, N, K1, K2):
    """C (+)= A1.B1 + A2.B2 in one K loop (the LoRA linear and its dX): every kind, store and accumulate, several tile
    shapes, against a float64 sum of the two products. K1 a multiple of 32 with K2 = 8 ... 32 takes the kernels that
    load operands straight into LDS (the second segment fills one more stage partly); the rest the staged ones."""
    rs = np.random.RandomState(M + K2)
    a1, b1 = rs.standard_normal((M, K1)).astype(np.float32), rs.standard_normal((N, K1)).astype(np.float32)
    a2, b2 = rs.standard_normal((M, K2)).astype(np.float32), rs.standard_normal((N, K2)).astype(np.float32)
    c0 = rs.standard_normal((M, N)).astype(np.float32)
    want = a1.astype(np.float64) @ b1.astype(np.float64).T + a2.astype(np.float64) @ b2.astype(np.float64).T
    bufs = [gpu.create_state_buffer(x.nbytes) for x in (a1, b1, a2, b2, c0)]
    L = mod("lib")
    T = lambda x: np.ascontiguousarray(x.T)
    try:
        for kind, ops in enumerate([(a1, b1, a2, b2), (a1, T(b1), a2, T(b2)), (T(a1), T(b1), T(a2), T(b2))]):
            for buf, arr in zip(bufs, ops):
                gpu.write_state_buffer(buf, arr)
            for tile in (-1, 0, 6, 7, 8, 10, 11, 12, 13):
                for acc in (0, 1):
                    gpu.set_option("gemm.tile", tile)
                    gpu.write_state_buffer(bufs[4], c0)
                    L.check(gpu.ctx, L.lib.gt_gemm_pair(gpu.ctx, kind, acc, M, N, K1, bufs[0], bufs[1], K2, bufs[2], bufs[3],
                                                        bufs[4]), "gt_gemm_pair")
                    got = gpu.read_state_buffer(bufs[4], M * N).reshape(M, N)
                    assert_close(got, (want + c0 if acc else want).astype(np.float32),
                                 f"gemm pair kind {kind} tile {tile} acc {acc} {M}x{N}x({K1}+{K2})")
        rc = L.lib.gt_gemm_pair(gpu.ctx, 0, 0, M, N, K1, bufs[0], bufs[1], 0, bufs[2], bufs[3], bufs[4])
        assert rc != 0 and b"K2" in L.lib.gt_last_error(gpu.ctx)
    finally:
        gpu.set_option("gemm.tile", -1)


def test_elementwise(gpu, ref):
    r = R(ref, 11)
    for n in [(4, 6), (5, 7), (129, 33), (64, 1024)]:
        op_case(gpu, ref, [r(*n), r(*n)], lambda ag, a, b: ag.add(a, b), lambda rf, a, b: rf.add(a, b), f"add {n}")
        op_case(gpu, ref, [r(*n), r(*n)], lambda ag, a, b: ag.mul(a, b), lambda rf, a, b: rf.mul(a, b), f"mul {n}")
        op_case(gpu, ref, [r(*n, sc=1.5)], lambda ag, x: ag.silu(x), lambda rf, x: rf.silu(x), f"silu {n}")
        op_case(gpu, ref, [r(*n, sc=1.5)], lambda ag, x: ag.gelu(x), lambda rf, x: rf.gelu(x), f"gelu {n}")
        op_case(gpu, ref, [r(*n)], lambda ag, x: ag.scale(x, 2.5), lambda rf, x: rf.scale(x, 2.5), f"scale {n}")


def test_aliasing_add_mul_same_tensor(gpu, ref):
    """gpu-parity.ts:2166-2173: add(t,t) and mul(t,t) accumulate both contributions into one gradient."""
    r = R(ref, 12)
    op_case(gpu, ref, [r(9, 13)], lambda ag, t: ag.add(t, t), lambda rf, t: rf.add(t, t), "add(t,t)")
    op_case(gpu, ref, [r(9, 13)], lambda ag, t: ag.mul(t, t), lambda rf, t: rf.mul(t, t), "mul(t,t)")


@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_gated_activation_fused_and_unfused(gpu, ref, act, fuse):
    """mul(act(gate), up): the fused kernels and the unfused pair give the oracle's result; with a second
    consumer of the activation the fused path must still propagate that consumer's gradient."""
    r = R(ref, 13)
    old = gpu.fuse_glu
    gpu.fuse_glu = fuse
    try:
        op_case(gpu, ref, [r(37, 52, sc=1.5), r(37, 52)],
                lambda ag, g, u: ag.mul(getattr(ag, act)(g), u), lambda rf, g, u: rf.mul(getattr(rf, act)(g), u), f"glu {act}")
        op_case(gpu, ref, [r(37, 52, sc=1.5), r(37, 52)],
                lambda ag, g, u: ag.mul(u, getattr(ag, act)(g)), lambda rf, g, u: rf.mul(u, getattr(rf, act)(g)), f"glu swapped {act}")

        def two_uses(m, g, u):
            a = getattr(m, act)(g)
            return m.add(m.mul(a, u), a)
        op_case(gpu, ref, [r(21, 40, sc=1.5), r(21, 40)], lambda ag, g, u: two_uses(ag, g, u),
                lambda rf, g, u: two_uses(rf, g, u), f"glu + second consumer {act}")
    finally:
        gpu.fuse_glu = old


@pytest.mark.parametrize("rows,d", [(4, 6), (9, 64), (33, 128), (70, 576), (16, 640), (5, 1024), (3, 2048), (7, 2500), (12, 30)])
def test_rms_norm(gpu, ref, rows, d):
    r = R(ref, rows + d)
    w = 1 + 0.3 * r(d)
    op_case(gpu, ref, [r(rows, d), w], lambda ag, x, g: ag.rms_norm(x, g, 1e-5), lambda rf, x, g: rf.rms_norm(x, g, 1e-5), f"rmsNorm {rows}x{d}")
    op_case(gpu, ref, [r(rows, d), w], lambda ag, x, g: ag.rms_norm(x, g, 1e-5), lambda rf, x, g: rf.rms_norm(x, g, 1e-5),
            f"rmsNorm frozen gain {rows}x{d}", frozen=(1,))


@pytest.mark.parametrize("T,H,hd", [(3, 2, 4), (17, 9, 64), (20, 16, 128), (11, 3, 32), (5, 2, 6), (8200, 8, 4)])
def test_rms_norm_heads(gpu, ref, T, H, hd):
    r = R(ref, T + hd)
    w = 1 + 0.3 * r(hd)
    # (8200, 8, 4): 65600 rows, the count past one grid dimension's 65535 that gpu-parity.ts:690-702 folds into two
    op_case(gpu, ref, [r(T, H * hd), w], lambda ag, x, g: ag.rms_norm_heads(x, g, T, H, hd, 1e-6),
            lambda rf, x, g: rf.rms_norm_heads(x, g, T, H, hd, 1e-6), f"rmsNormHeads {T},{H},{hd}")


def test_embedding_repeated_ids(gpu, ref):
    r = R(ref, 3)
    ids = [0, 3, 3, 6, 1, 3]
    op_case(gpu, ref, [r(7, 4)], lambda ag, w: ag.embedding(w, ids), lambda rf, w: rf.embedding(w, ids), "embedding")
    rng = ref.Mulberry32(8)
    ids = [min(511, int(512 * rng() ** 3)) for _ in range(700)]       # skewed: many repeats of small ids
    op_case(gpu, ref, [r(512, 96)], lambda ag, w: ag.embedding(w, ids), lambda rf, w: rf.embedding(w, ids), "embedding skewed")
    ids = [5] * 300
    op_case(gpu, ref, [r(9, 33)], lambda ag, w: ag.embedding(w, ids), lambda rf, w: rf.embedding(w, ids), "embedding one id")


@pytest.mark.parametrize("T,H,hd,base,pos", [(4, 2, 6, 1e4, 0), (4, 2, 6, 1e4, 5), (130, 9, 64, 1e5, 0), (64, 3, 128, 1e6, 17)])
def test_rope(gpu, ref, T, H, hd, base, pos):
    r = R(ref, T + hd)
    op_case(gpu, ref, [r(T, H * hd)], lambda ag, x: ag.rope(x, T, H, hd, base, pos), lambda rf, x: rf.rope(x, T, H, hd, base, pos), "rope")


def test_rope_far_positions(gpu, ref):
    """Position 2047 at pair 0 is where per-element f32 angles lose ~1e-4; the f64-built table must not."""
    r = R(ref, 99)
    T, H, hd = 2048, 1, 64
    op_case(gpu, ref, [r(T, H * hd)], lambda ag, x: ag.rope(x, T, H, hd, 1e5, 0), lambda rf, x: rf.rope(x, T, H, hd, 1e5, 0), "rope T=2048")


@pytest.mark.parametrize("T,B,H1,H2,hd,pos", [(64, 2, 9, 3, 64, 0), (33, 1, 4, 4, 128, 5), (7, 3, 5, 1, 32, 0), (16, 1, 2, 3, 6, 2), (2048, 1, 9, 3, 64, 0)])
@pytest.mark.parametrize("backward", [0, 1])
def test_rope_pair_equals_two_single_launches(gpu, ref, T, B, H1, H2, hd, pos, backward):
    """gt_rope_pair: the q and k of a layer in one launch give, bit for bit, what two gt_rope calls give: storing and
    accumulating, the vector kernel's shapes and one it does not take (hd 6: the call falls back to two launches)."""
    lib = mod("lib")
    r = R(ref, T + H1 + hd)
    rows = T * B
    a1, a2 = r(rows, H1 * hd), r(rows, H2 * hd)
    o1, o2 = r(rows, H1 * hd), r(rows, H2 * hd)            # old contents of the outputs, for the accumulating calls
    bufs = [gpu.create_state_buffer(x.nbytes) for x in (a1, a2, o1, o2, o1, o2)]
    i1, i2, p1, p2, s1, s2 = bufs
    gpu.write_state_buffer(i1, a1)
    gpu.write_state_buffer(i2, a2)
    try:
        for acc1, acc2 in ((0, 0), (1, 0), (1, 1)):
            for b, o in ((p1, o1), (p2, o2), (s1, o1), (s2, o2)):
                gpu.write_state_buffer(b, o)
            lib.check(gpu.ctx, lib.lib.gt_rope_pair(gpu.ctx, rows, T, hd, 10000.0, pos, backward, H1, i1, p1, acc1, H2, i2, p2, acc2), "pair")
            lib.check(gpu.ctx, lib.lib.gt_rope(gpu.ctx, rows, T, H1, hd, 10000.0, pos, backward, i1, s1, acc1), "single")
            lib.check(gpu.ctx, lib.lib.gt_rope(gpu.ctx, rows, T, H2, hd, 10000.0, pos, backward, i2, s2, acc2), "single")
            for pb, sb, n in ((p1, s1, a1.size), (p2, s2, a2.size)):
                got, want = gpu.read_state_buffer(pb, n), gpu.read_state_buffer(sb, n)
                assert np.array_equal(got, want), (acc1, acc2)
    finally:
        for b in bufs:
            gpu.free_state_buffer(b)


@pytest.mark.parametrize("kind,M,N,K", [(0, 300, 576, 576), (0, 257, 576, 1536), (0, 70, 83, 75), (0, 64, 64, 4096), (1, 130, 96, 64),
                                        (2, 96, 64, 2048), (0, 1, 5, 3)])
@pytest.mark.parametrize("in_place", [False, True])
def test_gemm_add_is_the_product_plus_the_addend(gpu, ref, kind, M, N, K, in_place):
    """gt_gemm_add: C = D + A.B in one call, bit for bit what gt_gemm into a buffer and an elementwise add give (the same
    f32 sum of the same two numbers), for aligned and ragged shapes, the register-staged fallback, K splits (the reduce
    kernel adds D) and D = C."""
    lib = mod("lib")
    r = R(ref, M + N + K)
    a_ = r(K, M) if kind == 2 else r(M, K)
    b_ = r(N, K) if kind == 0 else r(K, N)
    d_ = r(M, N)
    da, db, dd, dc, dy = (gpu.create_state_buffer(x.nbytes) for x in (a_, b_, d_, d_, d_))
    gpu.write_state_buffer(da, a_)
    gpu.write_state_buffer(db, b_)
    gpu.write_state_buffer(dd, d_)
    gpu.write_state_buffer(dc, d_ if in_place else np.zeros_like(d_))
    lib.check(gpu.ctx, lib.lib.gt_gemm_add(gpu.ctx, kind, M, N, K, da, db, dc if in_place else dd, dc), "gt_gemm_add")
    got = gpu.read_state_buffer(dc, M * N).copy()
    lib.check(gpu.ctx, lib.lib.gt_gemm(gpu.ctx, kind, 0, M, N, K, da, db, dy), "gt_gemm")
    y = gpu.read_state_buffer(dy, M * N).copy()
    assert np.array_equal(got, (d_.reshape(-1) + y).astype(np.float32))
    with pytest.raises(lib.HipError, match="null addend"):
        lib.check(gpu.ctx, lib.lib.gt_gemm_add(gpu.ctx, kind, M, N, K, da, db, 0, dc), "gt_gemm_add")


@pytest.mark.parametrize("kind,M,N,Ks", [(1, 300, 576, (576, 192, 192)), (1, 257, 576, (1536, 1536)), (1, 128, 640, (640, 128, 128)),
                                         (0, 200, 192, (64, 96)), (0, 130, 96, (32, 32, 32)), (1, 64, 576, (576,)),
                                         (1, 100, 576, (576, 190)), (1, 100, 574, (64, 64)), (2, 96, 64, (128, 160)),
                                         (1, 5600, 576, (576, 192, 192)), (0, 260, 640, (64, 96)), (1, 300, 320, (2048, 2048))])
@pytest.mark.parametrize("acc", [0, 1])
def test_gemm_sum_equals_the_products_one_by_one(gpu, ref, kind, M, N, Ks, acc):
    """gt_gemm_sum: up to three products summed in one launch (the K segments chained in one loop for aligned NT / NN
    operands) against one accumulating gt_gemm per product, and against float64. Cases: the q/k/v and gate/up input
    gradients at the SmolLM2 widths with ragged row counts, gemma's 640 width, NT, one product only, and the shapes that
    fall back to single launches (a K that is no multiple of 32, an N that is no multiple of 4, TN)."""
    lib = mod("lib")
    r = R(ref, M + N + sum(Ks))
    As, Bs = [], []
    for K in Ks:
        As.append(r(K, M) if kind == 2 else r(M, K))
        Bs.append(r(N, K) if kind == 0 else r(K, N))
    c0 = r(M, N)
    ab = [(gpu.create_state_buffer(a_.nbytes), gpu.create_state_buffer(b_.nbytes)) for a_, b_ in zip(As, Bs)]
    for (da, db), a_, b_ in zip(ab, As, Bs):
        gpu.write_state_buffer(da, a_)
        gpu.write_state_buffer(db, b_)
    c = gpu.create_state_buffer(c0.nbytes)
    n = len(Ks)
    karr, aarr, barr = (C.c_int * n)(*Ks), (C.c_uint64 * n)(*[x[0] for x in ab]), (C.c_uint64 * n)(*[x[1] for x in ab])
    gpu.write_state_buffer(c, c0)
    gpu.set_option("gemm.sum_min_tiles", 0)          # the chained loop also below one tile per CU
    try:
        lib.check(gpu.ctx, lib.lib.gt_gemm_sum(gpu.ctx, kind, acc, M, N, n, karr, aarr, barr, c), "gt_gemm_sum")
    finally:
        gpu.set_option("gemm.sum_min_tiles", -1)
    got = gpu.read_state_buffer(c, M * N).copy()
    if M * N < 256 * 128 * 96:                        # default threshold: a small output goes product by product, bit for bit
        gpu.write_state_buffer(c, c0)
        lib.check(gpu.ctx, lib.lib.gt_gemm_sum(gpu.ctx, kind, acc, M, N, n, karr, aarr, barr, c), "gt_gemm_sum")
        small = gpu.read_state_buffer(c, M * N).copy()
    gpu.write_state_buffer(c, c0)
    for i, K in enumerate(Ks):
        lib.check(gpu.ctx, lib.lib.gt_gemm(gpu.ctx, kind, acc if i == 0 else 1, M, N, K, ab[i][0], ab[i][1], c), "gt_gemm")
    one_by_one = gpu.read_state_buffer(c, M * N).copy()
    want = c0.astype(np.float64) * acc
    for a_, b_ in zip(As, Bs):
        a64, b64 = a_.astype(np.float64), b_.astype(np.float64)
        want = want + (a64.T @ b64 if kind == 2 else a64 @ (b64.T if kind == 0 else b64))
    assert_close(got, want, "gemm_sum vs float64")
    assert_close(got, one_by_one, "gemm_sum vs one by one")
    if M * N < 256 * 128 * 96:
        assert np.array_equal(small, one_by_one)


ATTN = [(5, 4, 2, 6, 0), (67, 4, 2, 16, 0), (130, 6, 2, 32, 0), (193, 9, 3, 64, 0), (64, 2, 2, 64, 0), (256, 4, 1, 64, 0),
        (96, 16, 8, 128, 0), (6, 4, 2, 6, 3), (130, 4, 2, 16, 17), (200, 10, 2, 64, 64), (150, 2, 1, 64, 1)]


@pytest.mark.parametrize("T,Hq,Hkv,hd,window", ATTN)
def test_attention(gpu, ref, T, Hq, Hkv, hd, window):
    """gpu-parity.ts:872-930: GQA, head dims 6..128, full causal and sliding windows (1, smaller and larger than a tile)."""
    r = R(ref, T * 3 + hd + window)
    op_case(gpu, ref, [r(T, Hq * hd), r(T, Hkv * hd), r(T, Hkv * hd)],
            lambda ag, q, k, v: ag.attention(q, k, v, T, Hq, Hkv, hd, window),
            lambda rf, q, k, v: rf.attention(q, k, v, T, Hq, Hkv, hd, window), f"attention {T},{Hq},{Hkv},{hd},w{window}",
            # window 1: one key per query, dq and dk are exactly zero; both sides leave ~1e-8 of rounding there
            floor=1.0 if window == 1 else 0.0)


def test_attention_stacked_sequences(gpu, ref):
    """rows = B*T: each sequence attends only to itself, positions restart per sequence."""
    ag = mod("autograd")
    B, T, Hq, Hkv, hd = 3, 40, 4, 2, 16
    r = R(ref, 77)
    q, k, v = r(B * T, Hq * hd), r(B * T, Hkv * hd), r(B * T, Hkv * hd)
    up = ref.Mulberry32(1).fill_uniform([B * T * Hq * hd])
    hq, hk, hv = (ag.Tensor(a, list(a.shape), True) for a in (q, k, v))
    gpu.install()
    try:
        out = ag.attention(ag.rope(hq, T, Hq, hd, 1e4), ag.rope(hk, T, Hkv, hd, 1e4), hv, T, Hq, Hkv, hd, 0)
        backward_from(gpu, ag, out, up)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    for b in range(B):
        s = slice(b * T, (b + 1) * T)
        rq, rk, rv = (ref.Tensor(a[s], [T, a.shape[1]], True) for a in (q, k, v))
        o = ref.attention(ref.rope(rq, T, Hq, hd, 1e4), ref.rope(rk, T, Hkv, hd, 1e4), rv, T, Hq, Hkv, hd, 0)
        ref.backward_from(o, up.reshape(B, -1)[b])
        assert_close(out.data.reshape(B, -1)[b], o.data, f"stacked attention out[{b}]")
        for h, rr, nm in ((hq, rq, "q"), (hk, rk, "k"), (hv, rv, "v")):
            assert_close(h.grad.reshape(B, -1)[b], rr.grad, f"stacked attention d{nm}[{b}]")


def test_cross_entropy_cases(gpu, ref):
    """gpu-parity.ts:762-829: ignore-index rows, V > 256, a target far behind the maximum, closed-form rows."""
    r = R(ref, 21)
    tg = [2, 7, -1, 0, 8, -1, 3]
    op_case(gpu, ref, [r(7, 9)], lambda ag, z: ag.cross_entropy(z, tg), lambda rf, z: rf.cross_entropy(z, tg), "CE ignore")
    rng = ref.Mulberry32(4)
    tg = [int(rng() * 1000) for _ in range(33)]
    tg[5] = tg[20] = -1
    op_case(gpu, ref, [r(33, 1000, sc=2.0)], lambda ag, z: ag.cross_entropy(z, tg), lambda rf, z: rf.cross_entropy(z, tg), "CE V=1000")
    tg = [int(rng() * 1003) for _ in range(10)]
    op_case(gpu, ref, [r(10, 1003, sc=2.0)], lambda ag, z: ag.cross_entropy(z, tg), lambda rf, z: rf.cross_entropy(z, tg), "CE V=1003 (unaligned rows)")
    z = np.array([[90, 0, 0, -3], [60, 1, 0, 0]], dtype=np.float32)
    out_h, _ = op_case(gpu, ref, [z], lambda ag, x: ag.cross_entropy(x, [3, 2]), lambda rf, x: rf.cross_entropy(x, [3, 2]), "CE far-behind target")
    exact = (math.log(math.exp(90) + 2 + math.exp(-3)) + 3 + math.log(math.exp(60) + math.e + 2)) / 2
    assert abs(out_h.data[0] - exact) < 1e-4
    for gap in [1, 10, 30, 60, 90]:
        row = np.array([[gap, 0, 0, -3]], dtype=np.float32)
        out_h, _ = op_case(gpu, ref, [row], lambda ag, x: ag.cross_entropy(x, [3]), lambda rf, x: rf.cross_entropy(x, [3]), f"CE gap {gap}")
        assert abs(out_h.data[0] - (math.log(math.exp(gap) + 2 + math.exp(-3)) + 3)) < 1e-4


def test_cross_entropy_all_ignored_is_exactly_zero(gpu, ref):
    """gpu-parity.ts:2419-2502."""
    ag = mod("autograd")
    z = ag.Tensor(ref.Mulberry32(2).fill_randn([6, 50]), [6, 50], True)
    h = ag.Tensor(ref.Mulberry32(3).fill_randn([6, 8]), [6, 8], True)
    w = ag.Tensor(ref.Mulberry32(4).fill_randn([50, 8]), [50, 8], True)
    gpu.install()
    try:
        l1 = ag.cross_entropy(z, [-1] * 6)
        ag.backward(l1, 1.0)
        l2 = ag.fused_cross_entropy(h, w, [-1] * 6, 16)
        ag.backward(l2, 1.0)
        gpu.sync([l1, l2])
    finally:
        gpu.uninstall()
    assert l1.data[0] == 0.0 and l2.data[0] == 0.0
    assert not np.any(z.grad) and not np.any(h.grad) and not np.any(w.grad)


def test_cross_entropy_per_sequence_denominators(gpu, ref):
    """Stacked sequences: one loss per sequence over its own kept count, equal to separate calls."""
    ag = mod("autograd")
    B, T, V = 3, 11, 40
    z = ref.Mulberry32(6).fill_randn([B * T, V], 2.0)
    rng = ref.Mulberry32(7)
    tg = [int(rng() * V) if rng() > 0.4 else -1 for _ in range(B * T)]
    hz = ag.Tensor(z, [B * T, V], True)
    gpu.install()
    try:
        loss = ag.cross_entropy(hz, tg, seq_len=T)
        ag.backward(loss, 1.0 / B)
        gpu.sync([loss])
    finally:
        gpu.uninstall()
    for b in range(B):
        rz = ref.Tensor(z[b * T:(b + 1) * T], [T, V], True)
        rl = ref.cross_entropy(rz, tg[b * T:(b + 1) * T])
        ref.backward(rl, 1.0 / B)
        assert abs(loss.data[b] - rl.data[0]) <= 1e-5 * abs(rl.data[0])
        assert_close(hz.grad.reshape(B, -1)[b], rz.grad, f"stacked CE dz[{b}]")


@pytest.mark.parametrize("chunk", [1, 7, 16, 64, 100])
def test_fused_cross_entropy_equals_dense(gpu, ref, chunk):
    """gpu-parity.ts:166-208 / gradcheck.ts:854-877."""
    r = R(ref, 31)
    tg = [3, -1, 36, 0, 7, -1, 7, 20, 1]
    op_case(gpu, ref, [r(9, 24), r(37, 24)], lambda ag, h, w: ag.fused_cross_entropy(h, w, tg, chunk),
            lambda rf, h, w: rf.cross_entropy(rf.linear(h, w), tg), f"fusedCE chunk {chunk}")
    op_case(gpu, ref, [r(9, 24), r(37, 24)], lambda ag, h, w: ag.fused_cross_entropy(h, w, tg, chunk),
            lambda rf, h, w: rf.fused_cross_entropy(h, w, tg, chunk), f"fusedCE frozen readout {chunk}", frozen=(1,))


def test_soft_cross_entropy(gpu, ref):
    r = R(ref, 41)
    T, V, k = 6, 50, 3
    rng = ref.Mulberry32(9)
    tids, tp = [], []
    for t in range(T):
        row = [int(rng() * V) for _ in range(k)]
        pr = [0.5, 0.3, 0.0] if t % 2 else [0.4, 0.25, 0.1]
        if t == 2:
            row[0] = -1
        if t == 4:
            row[1] = row[0]           # duplicate id inside a row
        tids += row
        tp += pr
    op_case(gpu, ref, [r(T, V, sc=2.0)], lambda ag, z: ag.soft_cross_entropy(z, tids, tp, k),
            lambda rf, z: rf.soft_cross_entropy(z, tids, tp, k), "softCE")


def test_validators_refuse_above_the_dispatch(gpu, ref):
    """gpu-parity.ts:2203-2290: malformed inputs raise before any device work."""
    ag = mod("autograd")
    gpu.install()
    try:
        x = ag.Tensor(np.zeros((3, 5), np.float32), [3, 5], True)
        w = ag.Tensor(np.zeros((4, 6), np.float32), [4, 6], True)
        with pytest.raises(ValueError, match="linear dim mismatch"):
            ag.linear(x, w)
        e = ag.Tensor(np.zeros((4, 3), np.float32), [4, 3], True)
        with pytest.raises(ValueError, match="not an integer in"):
            ag.embedding(e, [0, 6])
        z = ag.Tensor(np.zeros((3, 6), np.float32), [3, 6], True)
        with pytest.raises(ValueError, match="not -1"):
            ag.cross_entropy(z, [0, 6, 1])
        with pytest.raises(ValueError, match="not -1"):
            ag.cross_entropy(z, [0, -2, 1])
        with pytest.raises(ValueError, match="targets for"):
            ag.cross_entropy(z, [0, 1])
        with pytest.raises(ValueError, match="chunk must be positive"):
            ag.fused_cross_entropy(x, ag.Tensor(np.zeros((7, 5), np.float32), [7, 5], True), [0, 1, 2], 0)
        with pytest.raises(ValueError, match="teacher id"):
            ag.soft_cross_entropy(z, [0, 9, 1], [1.0, 1.0, 1.0], 1)
    finally:
        gpu.uninstall()


def test_late_backward_after_sync_is_refused(gpu, ref):
    """webgpu.ts:1412-1418 (test gpu-parity.ts:1842-1850): a backward over a graph whose buffers a sync recycled throws."""
    ag = mod("autograd")
    x = ag.Tensor(np.ones((4, 8), np.float32), [4, 8], True)
    w = ag.Tensor(np.ones((8, 8), np.float32), [8, 8], True)
    gpu.install()
    try:
        loss = ag.cross_entropy(ag.linear(x, w), [1, 2, 3, 4])
        gpu.sync([loss])
        with pytest.raises(RuntimeError, match="before a sync"):
            ag.backward(loss, 1.0)
    finally:
        gpu.uninstall()
        gpu.sync([])


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 700, 4, 2, 64, 0), (2, 333, 6, 2, 64, 300), (1, 1024, 9, 3, 64, 0),
                                                  (3, 129, 2, 1, 64, 33), (1, 512, 3, 3, 64, 512),
                                                  (1, 300, 4, 2, 128, 0), (2, 200, 8, 8, 128, 77), (1, 640, 16, 8, 128, 0),
                                                  (4, 128, 4, 2, 32, 0), (1, 450, 6, 3, 32, 100), (2, 261, 2, 2, 32, 0)])
@pytest.mark.parametrize("splits", [-1, 1, 5])
def test_attention_mfma_shapes(gpu, ref, B, T, Hq, Hkv, hd, window, splits):
    """The matrix-core kernels (hd = 32, 64 and 128): tiles of 128 queries x 32 keys with ragged T, windows that cut tiles,
    GQA group sums, stacked sequences; 1024 x 9/3 x 64 is one SmolLM2 layer at half the sequence length, 16/8 x 128
    the Qwen3-0.6B head layout, 4 x 128 x 4/2 x 32 the attention of benchmark config 1. Each shape with one workgroup per tile, with the launch-size heuristic, and with five
    workgroups per tile (partial softmax / dQ / dK,dV folded afterwards, some of them over empty ranges)."""
    ag = mod("autograd")
    gpu.set_option("attn.splits", splits)
    r = R(ref, T + Hq + window)
    q, k, v = r(B * T, Hq * hd), r(B * T, Hkv * hd), r(B * T, Hkv * hd)
    up = ref.Mulberry32(1).fill_uniform([B * T * Hq * hd])
    hq, hk, hv = (ag.Tensor(a, list(a.shape), True) for a in (q, k, v))
    gpu.install()
    try:
        out = ag.attention(hq, hk, hv, T, Hq, Hkv, hd, window)
        backward_from(gpu, ag, out, up)
        gpu.sync([out])
    finally:
        gpu.uninstall()
        gpu.set_option("attn.splits", -1)
    ref.set_threads(min(8, ref.max_threads()))
    try:
        for b in range(B):
            s = slice(b * T, (b + 1) * T)
            rq, rk, rv = (ref.Tensor(a[s], [T, a.shape[1]], True) for a in (q, k, v))
            o = ref.attention(rq, rk, rv, T, Hq, Hkv, hd, window, parallel_bwd=True)
            ref.backward_from(o, up.reshape(B, -1)[b])
            assert_close(out.data.reshape(B, -1)[b], o.data, f"mfma attention out[{b}]")
            for h, rr, nm in ((hq, rq, "q"), (hk, rk, "k"), (hv, rv, "v")):
                assert_close(h.grad.reshape(B, -1)[b], rr.grad, f"mfma attention d{nm}[{b}]")
    finally:
        ref.set_threads(1)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 1, 2, 1, 64, 0), (2, 31, 4, 2, 64, 0), (1, 33, 2, 2, 32, 0), (1, 65, 2, 1, 64, 0),
                                                  (1, 97, 3, 1, 64, 40), (1, 127, 2, 2, 128, 0), (1, 128, 2, 1, 64, 1),
                                                  (1, 129, 2, 1, 128, 128), (2, 160, 4, 4, 64, 1000), (3, 95, 2, 1, 32, 7)])
def test_attention_mfma_tile_edges(gpu, ref, B, T, Hq, Hkv, hd, window):
    """Sequences that end one row before, on and one row after a tile or a 32- / 64-key stage, a single row, windows of
    one key, of exactly a tile and longer than the sequence: the last stage's rows past the end are read from the last
    row and must leave no trace. Against the oracle, every sequence of the stack."""
    ag = mod("autograd")
    r = R(ref, 7 * T + Hq + window + hd)
    q, k, v = r(B * T, Hq * hd), r(B * T, Hkv * hd), r(B * T, Hkv * hd)
    up = ref.Mulberry32(2).fill_uniform([B * T * Hq * hd])
    hq, hk, hv = (ag.Tensor(a, list(a.shape), True) for a in (q, k, v))
    gpu.install()
    try:
        out = ag.attention(hq, hk, hv, T, Hq, Hkv, hd, window)
        backward_from(gpu, ag, out, up)
        gpu.sync([out])
    finally:
        gpu.uninstall()
    for b in range(B):
        s = slice(b * T, (b + 1) * T)
        rq, rk, rv = (ref.Tensor(a[s], [T, a.shape[1]], True) for a in (q, k, v))
        o = ref.attention(rq, rk, rv, T, Hq, Hkv, hd, window)
        ref.backward_from(o, up.reshape(B, -1)[b])
        floor = 1.0 if window == 1 else 0.0          # one key per query: dq and dk are exactly zero up to rounding
        assert_close(out.data.reshape(B, -1)[b], o.data, f"out[{b}]")
        for h, rr, nm in ((hq, rq, "q"), (hk, rk, "k"), (hv, rv, "v")):
            assert_close(h.grad.reshape(B, -1)[b], rr.grad, f"d{nm}[{b}]", floor=floor)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 256, 4, 2, 64, 0), (2, 384, 6, 2, 64, 100), (1, 512, 2, 1, 64, 128),
                                                  (1, 512, 2, 1, 64, 127), (1, 640, 2, 2, 64, 129), (1, 256, 3, 1, 64, 1),
                                                  (3, 128, 2, 2, 64, 0), (1, 768, 2, 1, 64, 300), (2, 256, 4, 2, 128, 0),
                                                  (1, 384, 2, 1, 128, 130), (1, 1024, 9, 3, 64, 0)])
@pytest.mark.parametrize("acc,splits", [(0, 1), (1, 1), (0, 5), (1, 3)])
def test_attention_backward_kept_ds_equals_recomputed(gpu, ref, B, T, Hq, Hkv, hd, window, acc, splits):
    """Whole 128-row tiles, one or several workgroups per tile: dK/dV writes the score gradients and dQ is one banded product over them. Against
    the kernel pair that recomputes the scores for dQ (itself held to the oracle above) and, for the first sequence,
    against the oracle; windows that end on, before and after a tile edge, window 1, accumulation into a used dq
    (acc = 1: the gradient buffers start from the same random contents on both paths)."""
    lib = mod("lib")
    floor = 1.0 if window == 1 and not acc else 0.0        # window 1: dq and dk are zero up to rounding, compared absolutely
    r = R(ref, 3 * T + Hq + window)
    q, k, v = r(B * T, Hq * hd), r(B * T, Hkv * hd), r(B * T, Hkv * hd)
    up = r(B * T, Hq * hd)
    init = [r(B * T, Hq * hd), r(B * T, Hkv * hd), r(B * T, Hkv * hd)]
    bufs = {n: gpu.create_state_buffer(a.nbytes) for n, a in (("q", q), ("k", k), ("v", v), ("up", up), ("out", q), ("dq", q), ("dk", k), ("dv", k))}
    lse = gpu.create_state_buffer(B * Hq * T * 4)
    for n, a in (("q", q), ("k", k), ("v", v), ("up", up)):
        gpu.write_state_buffer(bufs[n], a)
    gpu.set_option("attn.splits", splits)
    res = []
    try:
        lib.check(gpu.ctx, lib.lib.gt_attn_fwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], bufs["out"], lse), "fwd")
        for keep in (0, 1):
            gpu.set_option("attn.keep_ds", keep)
            for n, a in zip(("dq", "dk", "dv"), init):
                gpu.write_state_buffer(bufs[n], a)
            lib.check(gpu.ctx, lib.lib.gt_attn_bwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], bufs["out"],
                                                   bufs["up"], lse, bufs["dq"], acc, bufs["dk"], acc, bufs["dv"], acc), "bwd")
            res.append([gpu.read_state_buffer(bufs[n], a.size).copy() for n, a in zip(("dq", "dk", "dv"), init)])
    finally:
        gpu.set_option("attn.keep_ds", 1)
        gpu.set_option("attn.splits", -1)
    for a, b, nm in zip(res[1], res[0], ("dq", "dk", "dv")):
        assert_close(a, b, f"kept dS vs recomputed {nm}", floor=floor)
    if splits == 1 or window == 0:      # dK, dV: the same arithmetic (a split windowed launch cuts its longer loop elsewhere)
        assert np.array_equal(res[1][1], res[0][1]) and np.array_equal(res[1][2], res[0][2])
    ref.set_threads(min(8, ref.max_threads()))
    try:
        s = slice(0, T)
        rq, rk, rv = (ref.Tensor(a[s], [T, a.shape[1]], True) for a in (q, k, v))
        o = ref.attention(rq, rk, rv, T, Hq, Hkv, hd, window, parallel_bwd=True)
        ref.backward_from(o, up[s].reshape(-1))
        want = rq.grad.reshape(T, -1) + (init[0][s] if acc else 0)
        if floor:       # exact result zero; f32 rounding of dP - D (two 64-term dot products of O(1) values) leaves ~1e-6 per element
            assert np.abs(res[1][0].reshape(B * T, -1)[s] - want).max() < 1e-5
        else:
            assert_close(res[1][0].reshape(B * T, -1)[s], want, "kept dS dq vs oracle")
    finally:
        ref.set_threads(1)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 256, 4, 2, 64, 0), (2, 384, 6, 2, 64, 100), (1, 512, 2, 1, 64, 128),
                                                  (1, 640, 2, 2, 64, 129), (1, 256, 3, 1, 64, 1), (3, 128, 2, 2, 64, 0),
                                                  (2, 256, 4, 2, 128, 0), (1, 384, 2, 1, 128, 130), (1, 1024, 9, 3, 64, 0)])
@pytest.mark.parametrize("splits,keep_ds", [(1, 1), (3, 1), (1, 0)])
def test_attention_kept_scores_equals_recomputed(gpu, ref, B, T, Hq, Hkv, hd, window, splits, keep_ds):
    """gt_attn_fwd_scores / gt_attn_bwd_scores (the forward keeps S, dK/dV reads it back) against gt_attn_fwd / gt_attn_bwd
    (dK/dV recomputes S): the same output and statistic bit for bit, the three gradients to the parity bound, and dq of
    the first sequence against the oracle. Split and unsplit launches, with and without the kept dS."""
    lib = mod("lib")
    floor = 1.0 if window == 1 else 0.0
    r = R(ref, 5 * T + Hq + window)
    arrs = dict(q=r(B * T, Hq * hd), k=r(B * T, Hkv * hd), v=r(B * T, Hkv * hd), up=r(B * T, Hq * hd))
    bufs = {n: gpu.create_state_buffer(a.nbytes) for n, a in arrs.items()}
    for n, a in arrs.items():
        gpu.write_state_buffer(bufs[n], a)
    out, dq = (gpu.create_state_buffer(arrs["q"].nbytes) for _ in range(2))
    dk, dv = (gpu.create_state_buffer(arrs["k"].nbytes) for _ in range(2))
    lse = gpu.create_state_buffer(B * Hq * T * 4)
    need = C.c_uint64(0)
    lib.check(gpu.ctx, lib.lib.gt_attn_scores_bytes(gpu.ctx, B, T, Hq, Hkv, hd, window, C.byref(need)), "bytes")
    assert need.value == B * Hq * T * T * 4
    sco = gpu.create_state_buffer(need.value)
    gpu.set_option("attn.splits", splits)
    gpu.set_option("attn.keep_ds", keep_ds)
    res = []
    try:
        for kept in (0, 1):
            if kept:
                lib.check(gpu.ctx, lib.lib.gt_attn_fwd_scores(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out, lse, sco), "fwd")
                lib.check(gpu.ctx, lib.lib.gt_attn_bwd_scores(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out,
                                                              bufs["up"], lse, sco, dq, 0, dk, 0, dv, 0), "bwd")
            else:
                lib.check(gpu.ctx, lib.lib.gt_attn_fwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out, lse), "fwd")
                lib.check(gpu.ctx, lib.lib.gt_attn_bwd(gpu.ctx, B, T, Hq, Hkv, hd, window, bufs["q"], bufs["k"], bufs["v"], out,
                                                       bufs["up"], lse, dq, 0, dk, 0, dv, 0), "bwd")
            res.append([gpu.read_state_buffer(b_, n_).copy() for b_, n_ in ((out, arrs["q"].size), (lse, B * Hq * T), (dq, arrs["q"].size),
                                                                            (dk, arrs["k"].size), (dv, arrs["k"].size))])
    finally:
        gpu.set_option("attn.splits", -1)
        gpu.set_option("attn.keep_ds", 1)
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    for a, b, nm in zip(res[1][2:], res[0][2:], ("dq", "dk", "dv")):
        assert_close(a, b, f"kept scores vs recomputed {nm}", floor=floor)
    ref.set_threads(min(8, ref.max_threads()))
    try:
        rq, rk, rv = (ref.Tensor(arrs[n][:T], [T, arrs[n].shape[1]], True) for n in ("q", "k", "v"))
        o = ref.attention(rq, rk, rv, T, Hq, Hkv, hd, window, parallel_bwd=True)
        ref.backward_from(o, arrs["up"][:T].reshape(-1))
        for got, want, nm in ((res[1][2], rq.grad, "dq"), (res[1][3], rk.grad, "dk"), (res[1][4], rv.grad, "dv")):
            got = got.reshape(B, -1)[0]
            if floor and nm != "dv":
                assert np.abs(got - want).max() < 1e-5
            else:
                assert_close(got, want, f"kept scores {nm} vs oracle")
    finally:
        ref.set_threads(1)


def test_attention_scores_are_refused_where_not_kept(gpu):
    lib = mod("lib")
    need = C.c_uint64(7)
    for B, T, Hq, Hkv, hd in ((1, 200, 4, 2, 64), (1, 256, 4, 2, 32), (1, 256, 4, 2, 16)):
        lib.check(gpu.ctx, lib.lib.gt_attn_scores_bytes(gpu.ctx, B, T, Hq, Hkv, hd, 0, C.byref(need)), "bytes")
        assert need.value == 0
    b = gpu.create_state_buffer(1 << 20)
    with pytest.raises(lib.HipError, match="scores are kept for T a multiple of 128"):
        lib.check(gpu.ctx, lib.lib.gt_attn_fwd_scores(gpu.ctx, 1, 200, 4, 2, 64, 0, b, b, b, b, b, b), "fwd")
    with pytest.raises(lib.HipError, match="null scores buffer"):
        lib.check(gpu.ctx, lib.lib.gt_attn_fwd_scores(gpu.ctx, 1, 256, 4, 2, 64, 0, b, b, b, b, b, 0), "fwd")


def test_attention_ds_workspace_limit_falls_back_to_recompute(gpu, ref):
    """A dS workspace above "attn.ds_limit_mb" is not taken: the backward is then the recomputing kernel pair, bit for bit."""
    lib = mod("lib")
    B, T, Hq, Hkv, hd = 2, 256, 4, 2, 64              # dS would be 2 MiB
    r = R(ref, 77)
    arrs = dict(q=r(B * T, Hq * hd), k=r(B * T, Hkv * hd), v=r(B * T, Hkv * hd), up=r(B * T, Hq * hd))
    bufs = {n: gpu.create_state_buffer(a.nbytes) for n, a in arrs.items()}
    for n, a in arrs.items():
        gpu.write_state_buffer(bufs[n], a)
    out, dq = (gpu.create_state_buffer(arrs["q"].nbytes) for _ in range(2))
    dk, dv = (gpu.create_state_buffer(arrs["k"].nbytes) for _ in range(2))
    lse = gpu.create_state_buffer(B * Hq * T * 4)
    lib.check(gpu.ctx, lib.lib.gt_attn_fwd(gpu.ctx, B, T, Hq, Hkv, hd, 0, bufs["q"], bufs["k"], bufs["v"], out, lse), "fwd")
    res = {}
    try:
        for name, opts in (("recompute", {"attn.keep_ds": 0}), ("limited", {"attn.ds_limit_mb": 1}), ("kept", {"attn.ds_limit_mb": 2})):
            for k_, v_ in {"attn.keep_ds": 1, "attn.ds_limit_mb": 8192, **opts}.items():
                gpu.set_option(k_, v_)
            lib.check(gpu.ctx, lib.lib.gt_attn_bwd(gpu.ctx, B, T, Hq, Hkv, hd, 0, bufs["q"], bufs["k"], bufs["v"], out, bufs["up"], lse,
                                                   dq, 0, dk, 0, dv, 0), "bwd")
            res[name] = gpu.read_state_buffer(dq, arrs["q"].size).copy()
    finally:
        gpu.set_option("attn.keep_ds", 1)
        gpu.set_option("attn.ds_limit_mb", 8192)
    assert np.array_equal(res["limited"], res["recompute"])
    assert not np.array_equal(res["kept"], res["recompute"])          # another summation order, so not the same bits
    assert_close(res["kept"], res["recompute"], "kept vs recomputed dq")


def test_attention_mfma_equals_generic_at_full_length(gpu, ref):
    """T = 2048, 9/3 heads x 64 (the SmolLM2 layer), two stacked sequences: both kernel families against each other."""
    ag = mod("autograd")
    B, T, Hq, Hkv, hd = 2, 2048, 9, 3, 64
    rs = np.random.RandomState(5)
    q, k, v = (rs.standard_normal((B * T, n * hd)).astype(np.float32) for n in (Hq, Hkv, Hkv))
    up = rs.standard_normal(B * T * Hq * hd).astype(np.float32)
    res = []
    for generic in (1, 0):
        gpu.set_option("attn.generic", generic)
        hq, hk, hv = (ag.Tensor(a, list(a.shape), True) for a in (q, k, v))
        gpu.install()
        try:
            out = ag.attention(hq, hk, hv, T, Hq, Hkv, hd, 0)
            backward_from(gpu, ag, out, up)
            gpu.sync([out])
        finally:
            gpu.uninstall()
            gpu.set_option("attn.generic", 0)
        res.append((out.data.copy(), hq.grad.copy(), hk.grad.copy(), hv.grad.copy()))
    for a, b, nm in zip(res[1], res[0], ("out", "dq", "dk", "dv")):
        assert_close(a, b, f"mfma vs generic {nm}")


def test_flat_elementwise_past_65535_workgroups(gpu, ref):
    """gpu-parity.ts:217-239: add over n = 65535*256 + 777 elements, every element exact."""
    ag = mod("autograd")
    n = 65535 * 256 + 777
    a = ag.Tensor(np.full(n, 1.0, np.float32), [n], False)
    b = ag.Tensor(np.full(n, 2.0, np.float32), [n], False)
    gpu.install()
    try:
        y = ag.add(a, b)
        gpu.sync([y])
        assert int(np.count_nonzero(y.data != 3.0)) == 0
    finally:
        gpu.uninstall()
        gpu.sync([])


@pytest.mark.parametrize("sample", [1, 3])
def test_profiler_labels_times_and_sampling(gpu, ref, sample):
    """gpu-parity.ts:134-156: profile silu(linear(x, w)) with the default prefix: both kernels are reported with
    non-negative times and positive counts. With sampling, counts and stated work still cover every launch."""
    ag = mod("autograd")
    r = R(ref, 5)
    x, w = ag.Tensor(r(40, 48), [40, 48], True), ag.Tensor(r(40, 48), [40, 48], True)
    gpu.install()
    try:
        gpu.set_option("prof.sample", sample)
        gpu.start_profile()
        for _ in range(7):
            y = ag.silu(ag.linear(x, w))
            gpu.sync([y])
        prof = gpu.stop_profile()
    finally:
        gpu.set_option("prof.sample", 1)
        gpu.uninstall()
        gpu.sync([])
    gemm = [k for k in prof if k.startswith("gemm.nt.")]
    assert len(gemm) == 1 and "silu" in prof, prof
    for label in (gemm[0], "silu"):
        ms, count, work = prof[label]
        assert ms >= 0 and count == 7
    assert prof[gemm[0]][2] == 7 * 2 * 40 * 40 * 48


def test_unknown_option_is_an_error(gpu):
    """gt_set_option refuses a key it does not know and says which; known keys round-trip."""
    L = mod("lib")
    rc = L.lib.gt_set_option(gpu.ctx, b"gemm.no_such_switch", 1)
    assert rc != 0 and b"gemm.no_such_switch" in L.lib.gt_last_error(gpu.ctx)
    with pytest.raises(RuntimeError, match="no_such_switch"):
        gpu.set_option("attn.no_such_switch", 0)
    for key, default in (("gemm.tile", -1), ("gemm.splitk", -1), ("gemm.staged", 0), ("gemm.group", 1), ("attn.generic", 0), ("attn.splits", -1),
                         ("prof.sample", 1)):
        gpu.set_option(key, default)


def test_paired_linear_launches(gpu, ref):
    """Two consecutive linears over the same input with the same shape (k and v, gate and up) go out as one batched
    launch; results and gradients are those of two launches, also when a lazy activation sits between them, when the
    first output is consumed by something else first, and when the second linear has another shape."""
    ag = mod("autograd")
    r = R(ref, 21)
    x, w1, w2, w3 = r(70, 48), r(40, 48), r(40, 48), r(24, 48)

    def pair(m, x_, a_, b_):
        return m.add(m.linear(x_, a_), m.linear(x_, b_))

    def gated(m, x_, a_, b_):                    # silu(linear) recorded between the two linears, then the fused product
        g = m.silu(m.linear(x_, a_))
        return m.mul(g, m.linear(x_, b_))

    def act_then_add(m, x_, a_, b_):             # the activation is consumed by add, not by a gate*up product
        g = m.silu(m.linear(x_, a_))
        return m.add(g, m.linear(x_, b_))

    def used_between(m, x_, a_, b_):             # the first output feeds another op before the second linear
        y1 = m.linear(x_, a_)
        s = m.scale(y1, 0.5)
        return m.add(s, m.linear(x_, b_))

    for name, fn in (("pair", pair), ("gated", gated), ("activation then add", act_then_add), ("used between", used_between)):
        op_case(gpu, ref, [x, w1, w2], lambda m, *t, fn=fn: fn(m, *t), lambda m, *t, fn=fn: fn(m, *t), f"paired linears: {name}")
    # a differently shaped second linear does not pair: q [40] then k [24] over the same input, summed over columns
    def mixed(m, x_, a_, b_):
        y1, y2 = m.linear(x_, a_), m.linear(x_, b_)
        return m.add(m.linear(y1, m_ones(m, 24, 40)), y2)
    ones = np.ones((24, 40), np.float32)

    def m_ones(m, o, i):
        return m.Tensor(ones, [o, i], False)
    op_case(gpu, ref, [x, w1, w3], mixed, mixed, "paired linears: other shape second")
    # the pair is one GEMM launch, the unpaired form two
    counts = {}
    for batch in (True, False):
        gpu.batch_linears = batch
        try:
            hx, ha, hb = (ag.Tensor(a, list(a.shape), False) for a in (x, w1, w2))
            gpu.install()
            gpu.start_profile("gemm.")
            y = pair(ag, hx, ha, hb)
            gpu.sync([y])
            counts[batch] = sum(v[1] for v in gpu.stop_profile().values())
        finally:
            gpu.uninstall()
            gpu.batch_linears = True
    assert counts == {True: 1, False: 2}, counts


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window", [(1, 2048, 9, 3, 64, 0), (1, 1024, 4, 2, 128, 0), (2, 1024, 6, 2, 64, 0), (1, 2048, 10, 2, 64, 1500)])
def test_banded_dq_product_cut_into_parts(gpu, B, T, Hq, Hkv, hd, window):
    """The banded dQ product of a small launch cuts every row tile's key range into parts (option "attn.band_splits": pinned
    1, 2, 4, 8 and the library's own choice) whose partial sums one kernel adds up, rotates back and accumulates: the same dq
    up to the order of the sums, storing and accumulating, with and without the rotation's backward; dk and dv do not change."""
    lib = mod("lib")
    L = lib.lib
    rs = np.random.RandomState(T + hd + window + B)
    rows = B * T
    mk = lambda n: rs.standard_normal((rows, n)).astype(np.float32)
    q, k, v, go, dq0 = mk(Hq * hd), mk(Hkv * hd), mk(Hkv * hd), mk(Hq * hd), mk(Hq * hd)
    c = gpu.ctx

    def dev(a):
        b = gpu.create_state_buffer(a.nbytes)
        gpu.write_state_buffer(b, a)
        return b
    bq, bk, bv, bgo = dev(q), dev(k), dev(v), dev(go)
    bout, blse = gpu.create_state_buffer(q.nbytes), gpu.create_state_buffer(B * Hq * T * 4)
    bdk, bdv = gpu.create_state_buffer(k.nbytes), gpu.create_state_buffer(v.nbytes)
    need = C.c_uint64()
    lib.check(c, L.gt_attn_scores_bytes(c, B, T, Hq, Hkv, hd, window, C.byref(need)), "bytes")
    bsc = gpu.create_state_buffer(need.value)
    lib.check(c, L.gt_attn_fwd_scores(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, blse, bsc), "fwd")
    try:
        for rot in (0, 1):
            for acc in (0, 1):
                ref_out = None
                for sp in (1, 2, 4, 8, -1):
                    gpu.set_option("attn.band_splits", sp)
                    bdq = dev(dq0)
                    lib.check(c, L.gt_attn_bwd_scores_rope(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, bgo, blse, bsc, 10000.0, 5, rot, 0,
                                                           bdq, acc, bdk, 0, bdv, 0), "bwd")
                    got = [gpu.read_state_buffer(b, n).copy() for b, n in ((bdq, q.size), (bdk, k.size), (bdv, v.size))]
                    gpu.free_state_buffer(bdq)
                    if ref_out is None:
                        ref_out = got
                        continue
                    assert_close(got[0], ref_out[0], f"dq in {sp} parts, rotation {rot}, acc {acc}", rel_l2=2e-6, max_rel=2e-5)
                    assert np.array_equal(got[1], ref_out[1]) and np.array_equal(got[2], ref_out[2])
    finally:
        gpu.set_option("attn.band_splits", -1)


@pytest.mark.parametrize("B,T,Hq,Hkv,hd,window,keep_ds", [(1, 256, 4, 2, 64, 0, 1), (2, 128, 3, 3, 64, 0, 1), (1, 384, 4, 1, 128, 100, 1),
                                                        (2, 256, 6, 2, 64, 70, 0), (1, 128, 2, 2, 128, 0, 0), (8, 256, 9, 3, 64, 0, 1)])
@pytest.mark.parametrize("acc", [0, 1])
def test_attention_backward_with_the_rotations_backward_in_its_write_backs(gpu, B, T, Hq, Hkv, hd, window, keep_ds, acc):
    """gt_attn_bwd_scores_rope against gt_attn_bwd_scores followed by gt_rope(backward = 1) on dq and dk: the gradients with
    respect to q and k before their rotation, by the banded dQ product's write-back (keep_ds = 1) and by the dQ kernel's
    (keep_ds = 0), dK direct (one head per kv head) and through the per-head slices (GQA, and the split launches of a small
    batch), head dims 64 and 128, with a window, storing and accumulating; and each of the two rotations alone."""
    lib = mod("lib")
    L = lib.lib
    rs = np.random.RandomState(T + hd + window)
    rows = B * T
    mk = lambda n: rs.standard_normal((rows, n)).astype(np.float32)
    q, k, v, go = mk(Hq * hd), mk(Hkv * hd), mk(Hkv * hd), mk(Hq * hd)
    dq0, dk0, dv0 = mk(Hq * hd), mk(Hkv * hd), mk(Hkv * hd)
    c = gpu.ctx

    def dev(a):
        b = gpu.create_state_buffer(a.nbytes)
        gpu.write_state_buffer(b, a)
        return b
    bq, bk, bv, bgo = dev(q), dev(k), dev(v), dev(go)
    bout, blse = gpu.create_state_buffer(q.nbytes), gpu.create_state_buffer(B * Hq * T * 4)
    need = C.c_uint64()
    lib.check(c, L.gt_attn_scores_bytes(c, B, T, Hq, Hkv, hd, window, C.byref(need)), "bytes")
    assert need.value > 0
    bsc = gpu.create_state_buffer(need.value)
    base, pos = 10000.0, 3
    gpu.set_option("attn.keep_ds", keep_ds)
    try:
        lib.check(c, L.gt_attn_fwd_scores(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, blse, bsc), "fwd")
        # the two-call form: gradients with respect to the rotated rows, then the rotation's backward
        tq, tk = gpu.create_state_buffer(q.nbytes), gpu.create_state_buffer(k.nbytes)
        rq, rk, rv = dev(dq0), dev(dk0), dev(dv0)
        lib.check(c, L.gt_attn_bwd_scores(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, bgo, blse, bsc, tq, 0, tk, 0, rv, acc), "bwd")
        lib.check(c, L.gt_rope(c, rows, T, Hq, hd, base, pos, 1, tq, rq, acc), "rope.bwd")
        lib.check(c, L.gt_rope(c, rows, T, Hkv, hd, base, pos, 1, tk, rk, acc), "rope.bwd")
        want = [gpu.read_state_buffer(b, n).copy() for b, n in ((rq, q.size), (rk, k.size), (rv, v.size))]
        plain = [gpu.read_state_buffer(b, n).copy() for b, n in ((tq, q.size), (tk, k.size))]
        for rot_q, rot_k in ((1, 1), (1, 0), (0, 1)):
            fq, fk, fv = dev(dq0), dev(dk0), dev(dv0)
            lib.check(c, L.gt_attn_bwd_scores_rope(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, bgo, blse, bsc, base, pos, rot_q, rot_k,
                                                   fq, acc, fk, acc, fv, acc), "bwd.rope")
            got = [gpu.read_state_buffer(b, n).copy() for b, n in ((fq, q.size), (fk, k.size), (fv, v.size))]
            wq = want[0] if rot_q else plain[0] + (dq0.ravel() if acc else 0)
            wk = want[1] if rot_k else plain[1] + (dk0.ravel() if acc else 0)
            assert_close(got[0], wq, f"dq, rotations ({rot_q}, {rot_k})", rel_l2=2e-6, max_rel=2e-5)
            assert_close(got[1], wk, f"dk, rotations ({rot_q}, {rot_k})", rel_l2=2e-6, max_rel=2e-5)
            assert np.array_equal(got[2], want[2]), "dv does not depend on the rotations"
            for b in (fq, fk, fv):
                gpu.free_state_buffer(b)
        rc = L.gt_attn_bwd_scores_rope(c, B, T, Hq, Hkv, hd, window, bq, bk, bv, bout, bgo, blse, 0, base, pos, 1, 1, tq, 0, tk, 0, rv, 0)
        assert rc != 0 and "null scores buffer" in L.gt_last_error(c).decode()
    finally:
        gpu.set_option("attn.keep_ds", 1)
        gpu.sync([])


def test_deferred_rmsnorm_weight_gradient_sums_equal_the_direct_ones(gpu):
    """gt_rmsnorm_bwd_parts + gt_colsum_group against gt_rmsnorm_bwd, bit for bit: dx (stored, added to its own contents, added
    to another buffer's) and dw (stored and accumulated) for several normalisations summed in ONE launch, per-row and per-head
    shapes, more entries than one launch's table holds (chunked), and the refusals: a shape the fast kernel does not serve
    reports 0 partial rows, two entries with one destination are an error."""
    lib = mod("lib")
    L, c = lib.lib, gpu.ctx
    rs = np.random.RandomState(5)
    shapes = [(2048, 576), (4096, 64), (300, 128), (16384, 576), (77, 2048), (1, 4)] + [(64 + i, 32) for i in range(100)]

    def dev(a):
        b = gpu.create_state_buffer(a.nbytes)
        gpu.write_state_buffer(b, a)
        return b
    want, pend, keep = [], [], []
    for i, (rows, d) in enumerate(shapes):
        x, g = rs.standard_normal((rows, d)).astype(np.float32), rs.standard_normal((rows, d)).astype(np.float32)
        w = (1 + 0.3 * rs.standard_normal(d)).astype(np.float32)
        dx0, dw0 = rs.standard_normal((rows, d)).astype(np.float32), rs.standard_normal(d).astype(np.float32)
        mode = i % 3                              # 0: dx stored, 1: dx += , 2: dx = other + ...
        accw = (i // 3) % 2
        bx, bg, bw = dev(x), dev(g), dev(w)
        by, br = gpu.create_state_buffer(x.nbytes), gpu.create_state_buffer(rows * 4)
        lib.check(c, L.gt_rmsnorm_fwd(c, rows, d, 1e-5, bx, bw, by, br), "fwd")
        # direct
        bdx, bdw, bold = dev(dx0), dev(dw0), dev(dx0)
        if mode == 2:
            lib.check(c, L.gt_rmsnorm_bwd_from(c, rows, d, bx, bw, bg, br, bold, bdx, bdw, accw), "bwd")
        else:
            lib.check(c, L.gt_rmsnorm_bwd(c, rows, d, bx, bw, bg, br, bdx, mode, bdw, accw), "bwd")
        want.append((gpu.read_state_buffer(bdx, rows * d).copy(), gpu.read_state_buffer(bdw, d).copy()))
        # deferred
        n = C.c_int(-1)
        lib.check(c, L.gt_rmsnorm_parts_rows(c, rows, d, C.byref(n)), "rows")
        assert n.value >= 1
        fdx, fdw = dev(dx0), dev(dw0)
        parts = gpu.create_state_buffer(n.value * d * 4)
        lib.check(c, L.gt_rmsnorm_bwd_parts(c, rows, d, bx, bw, bg, br, bold if mode == 2 else fdx, fdx, 1 if mode else 0, parts), "parts")
        pend.append((parts, n.value, d, fdw, accw))
        keep.append((fdx, fdw, rows, d))
    n = len(pend)
    lib.check(c, L.gt_colsum_group(c, n, (C.c_uint64 * n)(*[p[0] for p in pend]), (C.c_int * n)(*[p[1] for p in pend]),
                                   (C.c_int * n)(*[p[2] for p in pend]), (C.c_uint64 * n)(*[p[3] for p in pend]),
                                   (C.c_int * n)(*[p[4] for p in pend])), "colsum")
    for (fdx, fdw, rows, d), (wdx, wdw) in zip(keep, want):
        assert np.array_equal(gpu.read_state_buffer(fdx, rows * d), wdx), f"dx [{rows}, {d}]"
        assert np.array_equal(gpu.read_state_buffer(fdw, d), wdw), f"dw [{rows}, {d}]"
    for rows, d in ((10, 30), (10, 4096), (0, 64)):
        nn = C.c_int(-1)
        lib.check(c, L.gt_rmsnorm_parts_rows(c, rows, d, C.byref(nn)), "rows")
        assert nn.value == 0
    two = pend[:2]
    rc = L.gt_colsum_group(c, 2, (C.c_uint64 * 2)(two[0][0], two[1][0]), (C.c_int * 2)(two[0][1], two[1][1]), (C.c_int * 2)(two[0][2], two[0][2]),
                           (C.c_uint64 * 2)(two[0][3], two[0][3]), (C.c_int * 2)(0, 0))
    assert rc != 0 and "write the same sums" in L.gt_last_error(c).decode()
    gpu.sync([])


def test_stream_mark_and_wait_order_two_contexts(gpu):
    """gt_stream_mark / gt_stream_wait: work queued on a second context after the wait sees what the first context had queued
    before its mark, with no host wait in between; and gt_timer_start / gt_timer_stop bracket queued work."""
    lib, hb = mod("lib"), mod("hip_backend")
    L = lib.lib
    other = hb.HipBackend(0, streams=1)
    try:
        a, b = gpu.ctx, other.ctx
        n = 1 << 24
        x = gpu.create_state_buffer(n * 4)
        y = other.create_state_buffer(n * 4)
        gpu.write_state_buffer(x, np.full(n, 1.0, np.float32))
        lib.check(a, L.gt_sync(a), "sync")
        ms = C.c_double(-1)
        lib.check(a, L.gt_timer_start(a), "timer")
        for _ in range(200):                      # a long chain on the first stream: x *= 1.01, 200 times
            lib.check(a, L.gt_scale_fwd(a, n, x, 1.01, x), "scale")
        lib.check(a, L.gt_stream_mark(a), "mark")
        lib.check(b, L.gt_stream_wait(b, a), "wait")
        lib.check(b, L.gt_scale_fwd(b, n, x, 1.0, y), "copy")          # reads x on the second stream: must see all 200 updates
        got = other.read_state_buffer(y, n)
        lib.check(a, L.gt_timer_stop(a, C.byref(ms)), "timer")
        want = np.float32(1.0)
        for _ in range(200):
            want = np.float32(want * np.float32(1.01))
        assert np.all(got == want), (got[:4], want)
        assert ms.value > 0.5                                          # 200 passes over 64 MB took measurable time
        rc = L.gt_stream_wait(b, None)
        assert rc != 0 and "other context" in L.gt_last_error(b).decode()
        rc = L.gt_timer_stop(b, C.byref(ms))
        assert rc != 0 and "gt_timer_start" in L.gt_last_error(b).decode()
    finally:
        other.destroy()
    gpu.sync([])
