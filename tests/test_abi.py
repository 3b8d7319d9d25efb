"""No-GPU checks of the boundary: the shared library loads, exports every symbol include/ggufhip.h declares, the
ctypes table covers exactly that set, and a context cannot be created without a device (no compute calls here)."""
import ctypes
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    src = open(os.path.join(ROOT, "include", "ggufhip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(gt_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    lib = importlib.import_module("gguf-trainer_amd.lib")
    names = header_symbols()
    assert len(names) >= 45
    dll = ctypes.CDLL(lib.LIB_PATH)
    for n in names:
        assert hasattr(dll, n), f"{n} is declared in include/ggufhip.h but not exported"
    assert sorted(lib.EXPORTS) == names


def test_no_context_without_a_device_and_no_cpu_path():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    hb = importlib.import_module("gguf-trainer_amd.hip_backend")
    assert hb.init_hip() is None
    with pytest.raises(RuntimeError, match="needs an MI355X"):
        hb.require_gpu("this test")
    ag = importlib.import_module("gguf-trainer_amd.autograd")
    ag.set_ops_backend(None)
    import numpy as np
    x = ag.Tensor(np.zeros((2, 2), np.float32), [2, 2], True)
    with pytest.raises(RuntimeError, match="no device backend installed"):
        ag.add(x, x)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "gguf-trainer_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("checked against the CPU oracle", ""), f"{f} mentions the oracle"


def test_host_validators_and_optstate_roundtrip():
    import numpy as np
    ag = importlib.import_module("gguf-trainer_amd.autograd")
    optim = importlib.import_module("gguf-trainer_amd.optim")
    arr, kept = ag.kept_rows_in_vocab([1, -1, 3, 0, -1, -1], 6, 5, "t", seq_len=3)
    assert list(kept) == [2, 1]
    with pytest.raises(ValueError):
        ag.kept_rows_in_vocab([1, 5], 2, 5, "t")
    with pytest.raises(ValueError):
        ag.kept_rows_in_vocab([1.5, 0], 2, 5, "t")
    ids, k = ag.kept_teacher_rows([1, 2, -1, 9, 0, 0], [0.5, 0.5, 0, 0, 1, 0], 3, 2, 5)
    assert k == 2
    st = {"muonMomentum": [np.arange(6, dtype=np.float32)], "adamM": [np.ones(3, np.float32), np.zeros(2, np.float32)],
          "adamV": [np.full(3, 2, np.float32), np.full(2, 3, np.float32)], "adamT": 17}
    raw = optim.serialize_opt_state(st)
    assert raw[:4] == b"1TPO" and len(raw) == 4 * (2 + 2 + 3 + 3) + 4 * 16
    back = optim.deserialize_opt_state(raw)
    assert back["adamT"] == 17 and np.array_equal(back["adamV"][1], st["adamV"][1])
    r = ag.mulberry32(0)
    assert r() == 0.26642920868471265
