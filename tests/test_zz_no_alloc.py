"""gt_rmsnorm_bwd_static, the entry point that allocates nothing (its dw partials live in a static device array),
against gt_rmsnorm_bwd through the C ABI: bit-identical dx and dw on two calls in a row, the second with a smaller input,
and the stated limits refused with an error."""
import numpy as np
import pytest

from gpu_common import mod

pytestmark = pytest.mark.gpu


def dev(gpu, arr):
    b = gpu.create_state_buffer(arr.nbytes)
    gpu.write_state_buffer(b, arr)
    return b


def run_pair(gpu, rows, d, acc, seed):
    lib = mod("lib")
    L = lib.lib
    rs = np.random.RandomState(seed)
    x = rs.standard_normal((rows, d)).astype(np.float32)
    g = rs.standard_normal((rows, d)).astype(np.float32)
    w = (1 + 0.3 * rs.standard_normal(d)).astype(np.float32)
    dx0 = rs.standard_normal((rows, d)).astype(np.float32)
    dw0 = rs.standard_normal(d).astype(np.float32)
    bx, bg, bw = dev(gpu, x), dev(gpu, g), dev(gpu, w)
    by, brinv = gpu.create_state_buffer(x.nbytes), gpu.create_state_buffer(rows * 4)
    lib.check(gpu.ctx, L.gt_rmsnorm_fwd(gpu.ctx, rows, d, 1e-5, bx, bw, by, brinv), "fwd")
    res = []
    for fn in (L.gt_rmsnorm_bwd, L.gt_rmsnorm_bwd_static):
        bdx, bdw = dev(gpu, dx0), dev(gpu, dw0)
        lib.check(gpu.ctx, fn(gpu.ctx, rows, d, bx, bw, bg, brinv, bdx, acc, bdw, acc), "bwd")
        res.append((gpu.read_state_buffer(bdx, rows * d).copy(), gpu.read_state_buffer(bdw, d).copy()))
    (dx_a, dw_a), (dx_b, dw_b) = res
    assert np.array_equal(dx_a, dx_b), f"dx differs (rows {rows}, d {d}, acc {acc})"
    assert np.array_equal(dw_a, dw_b), f"dw differs (rows {rows}, d {d}, acc {acc})"
    # and the pair is not trivially equal: dw against float64
    r = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1) + 1e-5)
    want = (g.astype(np.float64) * x * r[:, None]).sum(axis=0) + (dw0 if acc else 0)
    assert np.abs(dw_b - want).max() <= 1e-4 * np.abs(want).max()


def test_static_scratch_rmsnorm_backward_equals_the_allocating_one(gpu):
    run_pair(gpu, 16384, 576, 0, 1)       # 512 partial rows of 576 columns in the static array
    run_pair(gpu, 100, 64, 1, 2)          # smaller, right after: stale partials of the first call must not be read
    run_pair(gpu, 4097, 2048, 0, 3)       # the widest row the array is sized for
    run_pair(gpu, 3, 128, 1, 4)


def test_static_scratch_rmsnorm_backward_refuses_what_it_cannot_hold(gpu):
    lib = mod("lib")
    L = lib.lib
    b = gpu.create_state_buffer(8 * 4096 * 4)
    with pytest.raises(lib.HipError, match="more than the static scratch"):
        lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, 8, 4096, b, b, b, b, b, 0, b, 0), "bwd")
    with pytest.raises(lib.HipError, match="multiple of 4"):
        lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, 8, 30, b, b, b, b, b, 0, b, 0), "bwd")
    with pytest.raises(lib.HipError, match="16-byte aligned"):
        lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, 8, 64, b + 4, b, b, b, b, 0, b, 0), "bwd")
    # rows = 0 with a store: dw is cleared by a kernel, nothing else happens
    dw = dev(gpu, np.ones(64, np.float32))
    lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, 0, 64, b, b, b, b, b, 0, dw, 0), "bwd")
    assert not np.any(gpu.read_state_buffer(dw, 64))


def test_static_scratch_is_not_shared_by_two_contexts_at_once(gpu):
    """The scratch array is one per device. A second context's call while the first one's is still queued would race on
    it: refused until the first context has been waited for."""
    lib, hb = mod("lib"), mod("hip_backend")
    L = lib.lib
    other = hb.HipBackend(0, streams=1)
    try:
        rows, d = 4096, 256
        rs = np.random.RandomState(9)
        x = rs.standard_normal((rows, d)).astype(np.float32)
        w = np.ones(d, np.float32)

        def bufs(be):
            bx, bw = dev(be, x), dev(be, w)
            br, bdx, bdw = be.create_state_buffer(rows * 4), be.create_state_buffer(x.nbytes), be.create_state_buffer(d * 4)
            lib.check(be.ctx, L.gt_rmsnorm_fwd(be.ctx, rows, d, 1e-5, bx, bw, bdx, br), "fwd")
            return bx, bw, br, bdx, bdw
        a, b = bufs(gpu), bufs(other)
        lib.check(gpu.ctx, L.gt_sync(gpu.ctx), "sync")
        lib.check(other.ctx, L.gt_sync(other.ctx), "sync")
        lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, rows, d, a[0], a[1], a[0], a[2], a[3], 0, a[4], 0), "bwd")
        rc = L.gt_rmsnorm_bwd_static(other.ctx, rows, d, b[0], b[1], b[0], b[2], b[3], 0, b[4], 0)
        assert rc != 0 and "gt_sync that context first" in L.gt_last_error(other.ctx).decode()
        # without dw the array is not touched: allowed
        lib.check(other.ctx, L.gt_rmsnorm_bwd_static(other.ctx, rows, d, b[0], b[1], b[0], b[2], b[3], 0, 0, 0), "bwd")
        lib.check(gpu.ctx, L.gt_sync(gpu.ctx), "sync")
        lib.check(other.ctx, L.gt_rmsnorm_bwd_static(other.ctx, rows, d, b[0], b[1], b[0], b[2], b[3], 0, b[4], 0), "bwd")
        got_a, got_b = gpu.read_state_buffer(a[4], d), other.read_state_buffer(b[4], d)
        assert np.array_equal(got_a, got_b)
    finally:
        other.destroy()
    # the context that last used the array is gone: the next caller is not held up by it
    lib.check(gpu.ctx, L.gt_rmsnorm_bwd_static(gpu.ctx, rows, d, a[0], a[1], a[0], a[2], a[3], 0, a[4], 0), "bwd")
    lib.check(gpu.ctx, L.gt_sync(gpu.ctx), "sync")
