"""Host tape above the device backend: Tensor, backward, checkpoint, the LoRA-aware `linear`
and the input validators, i.e. everything of src/model/autograd.ts that sits ABOVE the
OpsBackend dispatch (autograd.ts:20-93, 160-379 and the guards of :548-554, 760-894, 968-998).

There are no CPU ops here. Every op forwards to the installed backend (set_ops_backend); with
none installed the call raises, it does not compute.

Batched extension: the reference runs one sequence of T rows per call. Ops here accept rows = B*T
(sequences stacked); `rope` and `attention` take the per-sequence length T and derive B from the
row count, and the losses take `seq_len` (default: all rows are one sequence) and return one loss
per sequence, each over its own kept-row count as the reference's per-sequence calls would.
"""
from __future__ import annotations

import math

import numpy as np

_created = 0


def _prod(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


class Tensor:
    """autograd.ts:20-51. Host arrays are allocated on first touch: an intermediate that lives on
    the device only never pays for a host copy. They are authoritative only after backend.sync()."""

    __slots__ = ("shape", "requires_grad", "_backward", "_prev", "seq", "_data", "_grad", "_dev", "__weakref__")

    def __init__(self, data, shape, requires_grad=False):
        global _created
        self.shape = [int(s) for s in shape]
        if data is not None:
            data = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
            if data.size != _prod(self.shape):
                raise ValueError(f"data length {data.size} != shape {self.shape}")
        self._data = data
        self._grad = None
        self._dev = None                # a device backend's record for this tensor: (owner key, record)
        self.requires_grad = requires_grad
        self._backward = _noop
        self._prev = []
        self.seq = _created
        _created += 1

    @staticmethod
    def zeros(shape, requires_grad=False):
        return Tensor(None, shape, requires_grad)

    @property
    def data(self) -> np.ndarray:
        if self._data is None:
            self._data = np.zeros(self.size, dtype=np.float32)
        return self._data

    @data.setter
    def data(self, v):
        self._data = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)

    @property
    def grad(self) -> np.ndarray:
        if self._grad is None:
            self._grad = np.zeros(self.size, dtype=np.float32)
        return self._grad

    def zero_grad(self):
        if self._grad is not None:
            self._grad.fill(0)

    @property
    def size(self) -> int:
        return _prod(self.shape)


def _noop():
    return None


def mulberry32(seed: int):
    """autograd.ts:69-78."""
    a = seed & 0xFFFFFFFF

    def nxt():
        nonlocal a
        a = (a + 0x6D2B79F5) & 0xFFFFFFFF
        t = ((a ^ (a >> 15)) * (1 | a)) & 0xFFFFFFFF
        t = ((t + (((t ^ (t >> 7)) * (61 | t)) & 0xFFFFFFFF)) & 0xFFFFFFFF) ^ t
        return ((t ^ (t >> 14)) & 0xFFFFFFFF) / 4294967296

    return nxt


def randn(rng) -> float:
    """Box-Muller, autograd.ts:61-66."""
    u = v = 0.0
    while u == 0:
        u = rng()
    while v == 0:
        v = rng()
    return math.sqrt(-2 * math.log(u)) * math.cos(2 * math.pi * v)


def param(shape, std, rng) -> Tensor:
    n = _prod(shape)
    return Tensor(np.array([randn(rng) * std for _ in range(n)], dtype=np.float32), shape, True)


def _topo(root, seen):
    topo = []
    if id(root) in seen:
        return topo
    seen.add(id(root))
    stack = [(root, 0)]
    while stack:
        t, i = stack.pop()
        if i < len(t._prev):
            stack.append((t, i + 1))
            p = t._prev[i]
            if id(p) not in seen:
                seen.add(id(p))
                stack.append((p, 0))
        else:
            topo.append(t)
    return topo


class _backward_scope:
    """Tells a backend that keeps a `backward_depth` counter that closures are being walked: forward ops recorded
    meanwhile (a checkpoint's replay) belong to the graph being differentiated, not to a new one."""

    def __enter__(self):
        self.be = _backend if _backend is not None and hasattr(_backend, "backward_depth") else None
        if self.be is not None:
            self.be.backward_depth += 1

    def __exit__(self, *exc):
        if self.be is not None:
            self.be.backward_depth -= 1
        return False


def backward(loss: Tensor, seed: float = 1.0):
    """autograd.ts:81-93. A per-sequence loss vector gets the same seed in every slot."""
    topo = _topo(loss, set())
    loss.grad[:] = seed
    with _backward_scope():
        for t in reversed(topo):
            t._backward()


# ---- backend dispatch (autograd.ts:95-169, 275-279) -----------------------------------------------

_backend = None


def set_ops_backend(b):
    global _backend
    _backend = b


def _be():
    if _backend is None:
        raise RuntimeError("no device backend installed: call HipBackend.install() first (this package has no CPU ops)")
    return _backend


def _region_backend():
    b = _backend
    return b if b is not None and callable(getattr(b, "begin_region", None)) else None


_checkpointing = False


def set_checkpointing(on: bool):
    global _checkpointing
    _checkpointing = bool(on)


def _assert_self_contained(out, inputs, born):
    """autograd.ts:198-215."""
    seen = {id(t) for t in inputs}
    if id(out) in seen:
        raise ValueError("checkpoint: fn returned one of its inputs; there is nothing to recompute")
    stack = [out]
    while stack:
        t = stack.pop()
        if id(t) in seen:
            continue
        seen.add(id(t))
        if t._prev and t.seq < born:
            raise ValueError("checkpoint: the block reads a computed tensor it did not create. "
                             "Pass it in `inputs`, or move its computation inside the block.")
        stack.extend(t._prev)


def checkpoint(inputs, fn):
    """autograd.ts:234-273: keep the block's output, recompute its interior in backward."""
    if not _checkpointing:
        return fn()
    rb = _region_backend()
    born = _created
    mark = rb.begin_region() if rb else 0
    if rb is not None and hasattr(rb, "forward_only_region"):
        rb.forward_only_region = True          # this pass's interior is thrown away: nothing worth saving for a backward
        try:
            out = fn()
        finally:
            rb.forward_only_region = False
    else:
        out = fn()
    _assert_self_contained(out, inputs, born)
    if rb:
        rb.end_region(mark, [out])
    inputs = list(inputs)
    out._prev = inputs

    def bw():
        with _backward_scope():         # also when the closure is walked by hand (a test seeding a non-scalar output)
            mark2 = rb.begin_region() if rb else 0
            replay = fn()
            if rb:
                rb.seed_grad_from(replay, out)
            else:
                replay.grad[:] = out.grad
            topo = _topo(replay, {id(t) for t in inputs})
            for t in reversed(topo):
                t._backward()
            if rb:
                rb.end_region(mark2, [])

    out._backward = bw
    return out


# ---- LoRA-aware linear (autograd.ts:290-379) ----------------------------------------------------------

_lora: dict = {}


def set_lora_adapters(m: dict):
    """m: id(weight) -> (a [rank,in], b [out,rank], scale); None or {} removes every adapter."""
    global _lora
    _lora = m or {}


def linear(x: Tensor, w: Tensor) -> Tensor:
    if _lora:
        ad = _lora.get(id(w))
        if ad is not None:
            a, b, sc = ad
            be = _be()
            if hasattr(be, "lora_linear"):
                # the same composition as below, recorded as one op: the backend applies the scale to the rank-r
                # activation instead of the [rows, out] product and accumulates into the base output in place
                _check_linear_dims(x, w)
                _check_linear_dims(x, a)
                if b.shape[1] != a.shape[0]:
                    raise ValueError(f"linear dim mismatch: x is [{x.shape[0]}, {a.shape[0]}] and w is "
                                     f"[{', '.join(map(str, b.shape))}], so the contracted dimension is {a.shape[0]} on "
                                     f"one side and {b.shape[1]} on the other. A projection wired to the wrong config "
                                     "field is the usual cause.")
                return be.lora_linear(x, w, a, b, sc)
            return add(_linear_raw(x, w), scale(_linear_raw(_linear_raw(x, a), b), sc))
    return _linear_raw(x, w)


def _check_linear_dims(x, w):
    if x.shape[1] != w.shape[1]:
        raise ValueError(
            f"linear dim mismatch: x is [{', '.join(map(str, x.shape))}] and w is [{', '.join(map(str, w.shape))}], "
            f"so the contracted dimension is {x.shape[1]} on one side and {w.shape[1]} on the other. "
            "A projection wired to the wrong config field is the usual cause.")


def _linear_raw(x, w):
    _check_linear_dims(x, w)
    return _be().linear(x, w)


def add(a, b):
    return _be().add(a, b)


def mul(a, b):
    return _be().mul(a, b)


def silu(x):
    return _be().silu(x)


def gelu(x):
    return _be().gelu(x)


def scale(x, c: float):
    return _be().scale(x, c)


def rms_norm(x, weight, eps: float):
    return _be().rms_norm(x, weight, eps)


def rms_norm_heads(x, weight, T: int, H: int, hd: int, eps: float):
    return _be().rms_norm_heads(x, weight, T, H, hd, eps)


def assert_rank(t, rank, name, where):
    if len(t.shape) != rank:
        raise ValueError(f"{where}: {name} must be {rank}-D, got [{', '.join(map(str, t.shape))}]")


def assert_matrix(t, name, where):
    assert_rank(t, 2, name, where)


def _as_int_array(values, where, what):
    arr = np.asarray(values)
    if arr.dtype.kind == "f":
        if not np.all(arr == np.floor(arr)):
            bad = int(np.argmax(arr != np.floor(arr)))
            raise ValueError(f"{where}: {what} {arr[bad]} at position {bad} is not an integer")
        arr = arr.astype(np.int64)
    elif arr.dtype.kind not in "iu":
        raise ValueError(f"{where}: {what}s must be integers")
    return arr.astype(np.int64, copy=False).reshape(-1)


def assert_ids_in_table(ids, V, where):
    """autograd.ts:813-823."""
    arr = _as_int_array(ids, where, "id")
    bad = np.nonzero((arr < 0) | (arr >= V))[0]
    if bad.size:
        t = int(bad[0])
        raise ValueError(f"{where}: id {int(arr[t])} at position {t} is not an integer in [0,{V}). "
                         "A corpus tokenized with a different vocab than the checkpoint is the usual cause.")
    return arr


def embedding(weight, ids):
    assert_matrix(weight, "weight", "embedding")
    arr = assert_ids_in_table(ids, weight.shape[0], "embedding")
    return _be().embedding(weight, arr)


def rope(x, T: int, H: int, hd: int, base: float, pos_offset: int = 0):
    return _be().rope(x, T, H, hd, base, pos_offset)


def attention(q, k, v, T: int, Hq: int, Hkv: int, hd: int, window: int = 0):
    return _be().attention(q, k, v, T, Hq, Hkv, hd, window)


def kept_rows_in_vocab(targets, T, V, where, seq_len=None):
    """autograd.ts:875-894. Returns (int64 targets, kept count per sequence)."""
    n = len(targets)
    if n != T:
        raise ValueError(f"{where}: {n} targets for {T} logit rows. The loss sums T rows and means over the targets "
                         "it counts, so a mismatch reports a plausible wrong loss.")
    arr = _as_int_array(targets, where, "target")
    bad = np.nonzero((arr < -1) | (arr >= V))[0]
    if bad.size:
        t = int(bad[0])
        raise ValueError(f"{where}: target {int(arr[t])} at position {t} is not -1 (ignore) or an integer in [0,{V}). "
                         "A corpus tokenized with a different vocab than the checkpoint is the usual cause.")
    L = T if seq_len is None else int(seq_len)
    if L <= 0 or T % L != 0:
        raise ValueError(f"{where}: {T} rows are not a whole number of sequences of {L}")
    kept = (arr.reshape(-1, L) >= 0).sum(axis=1)
    return arr, kept


def cross_entropy(logits, targets, seq_len=None):
    assert_matrix(logits, "logits", "crossEntropy")
    T, V = logits.shape
    arr, kept = kept_rows_in_vocab(targets, T, V, "crossEntropy", seq_len)
    return _be().cross_entropy(logits, arr, kept)


def fused_cross_entropy(hidden, w, targets, chunk: int, seq_len=None):
    assert_matrix(hidden, "hidden", "fusedCrossEntropy")
    assert_matrix(w, "w", "fusedCrossEntropy")
    T, H = hidden.shape
    V, H2 = w.shape
    if H != H2:
        raise ValueError(f"fusedCrossEntropy dim mismatch {H} vs {H2}")
    if chunk <= 0:
        raise ValueError(f"fusedCrossEntropy chunk must be positive, got {chunk}")
    if id(w) in _lora:
        raise ValueError("fusedCrossEntropy: the readout weight carries a LoRA adapter, which this path cannot apply. "
                         "Put the readout in the aux param group, or use --loss-chunk 0.")
    arr, kept = kept_rows_in_vocab(targets, T, V, "fusedCrossEntropy", seq_len)
    return _be().fused_cross_entropy(hidden, w, arr, int(chunk), kept)


def kept_teacher_rows(teacher_ids, teacher_probs, T, k, V):
    """autograd.ts:760-791."""
    if k < 1:
        raise ValueError(f"softCrossEntropy: k must be >= 1, got {k}")
    if len(teacher_ids) != T * k or len(teacher_probs) != T * k:
        raise ValueError(f"softCrossEntropy: teacher arrays must be [T*k]={T * k}, got {len(teacher_ids)}/{len(teacher_probs)}")
    ids = _as_int_array(teacher_ids, "softCrossEntropy", "teacher id").reshape(T, k)
    live = ids[:, 0] != -1
    chk = ids[live]
    bad = np.argwhere((chk < 0) | (chk >= V))
    if bad.size:
        r, j = bad[0]
        row = int(np.nonzero(live)[0][r])
        raise ValueError(f"softCrossEntropy: teacher id {int(chk[r, j])} at slot {int(j)} of row {row} is not an integer "
                         f"in [0,{V}). Only -1 in the first slot marks an ignored row.")
    return ids.reshape(-1), int(live.sum())


def soft_cross_entropy(logits, teacher_ids, teacher_probs, k: int):
    assert_matrix(logits, "logits", "softCrossEntropy")
    T, V = logits.shape
    ids, kept = kept_teacher_rows(teacher_ids, teacher_probs, T, k, V)
    return _be().soft_cross_entropy(logits, ids, np.asarray(teacher_probs, dtype=np.float32).reshape(-1), k, kept)
