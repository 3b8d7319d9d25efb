"""Shared helpers of the GPU parity tests: load the product package, run the same graph on the HIP
backend and on the CPU oracle from the same seeded arrays, compare with the stated tolerances.

Tolerances (relative to the oracle): loss <= 1e-5 relative; every gradient tensor <= 1e-5 relative
L2 and <= 1e-4 max error over max magnitude.
"""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG = "gguf-trainer_amd"
REL_L2 = 1e-5
MAX_REL = 1e-4
LOSS_REL = 1e-5


def mod(name):
    return importlib.import_module(f"{PKG}.{name}")


def errs(got, want, floor=0.0):
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), "non-finite values from the device"
    nrm = np.linalg.norm(want)
    mx = np.abs(want).max() if want.size else 0.0
    if floor > 0:                    # an exactly-zero gradient (attention window 1) compares absolutely
        nrm, mx = max(nrm, floor), max(mx, floor)
    l2 = np.linalg.norm(got - want) / nrm if nrm > 0 else np.linalg.norm(got - want)
    mr = np.abs(got - want).max() / mx if mx > 0 else (np.abs(got - want).max() if want.size else 0.0)
    return l2, mr


def assert_close(got, want, what="", rel_l2=REL_L2, max_rel=MAX_REL, floor=0.0):
    l2, mr = errs(got, want, floor)
    assert l2 <= rel_l2 and mr <= max_rel, f"{what}: rel L2 {l2:.3e} (<= {rel_l2:g}), max-rel {mr:.3e} (<= {max_rel:g})"
    return l2, mr


def backward_from(gpu, ag, out, grad_out):
    """tests/gradcheck.ts:61-73 on the device: seed a full upstream gradient on a non-scalar output."""
    topo = ag._topo(out, set())
    out.grad[:] = np.asarray(grad_out, dtype=np.float32).reshape(-1)
    gpu.seed_grad_from_host(out)
    for t in reversed(topo):
        t._backward()


def op_case(gpu, ref, arrays, fwd_hip, fwd_ref, what, frozen=(), rel_l2=REL_L2, max_rel=MAX_REL, seed=0xBEEF, floor=0.0):
    """tests/gpu-parity.ts:90-126: the same forward on both sides from the same arrays, the same seeded
    upstream gradient, compare the output and every input gradient."""
    ag = mod("autograd")
    hts = [ag.Tensor(a, list(a.shape), i not in frozen) for i, a in enumerate(arrays)]
    rts = [ref.Tensor(a, list(a.shape), i not in frozen) for i, a in enumerate(arrays)]
    gpu.install()
    try:
        out_h = fwd_hip(ag, *hts)
        out_r = fwd_ref(ref, *rts)
        up = ref.Mulberry32(seed).fill_uniform([out_r.size])
        backward_from(gpu, ag, out_h, up)
        gpu.sync([out_h])
    finally:
        gpu.uninstall()
    ref.backward_from(out_r, up)
    assert_close(out_h.data, out_r.data, f"{what} forward", rel_l2, max_rel)
    for i, (h, r) in enumerate(zip(hts, rts)):
        if i in frozen:
            continue
        assert_close(h.grad, r.grad, f"{what} grad[{i}]", rel_l2, max_rel, floor)
    return out_h, out_r
