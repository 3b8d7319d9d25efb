import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ref():
    """The CPU oracle (oracle/ref.py over oracle/liboracle.so); built on demand."""
    lib = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(lib):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    from oracle import ref as r
    return r


@pytest.fixture(scope="session")
def gpu():
    """One HipBackend (one HIP context and stream) for the whole GPU test session."""
    import importlib
    hb = importlib.import_module("gguf-trainer_amd.hip_backend")
    g = hb.require_gpu("the GPU parity tests")
    print(f"[gpu] {g.adapter_name}", flush=True)
    yield g
    g.destroy()


@pytest.fixture(autouse=True)
def _name_the_case(request):
    # a GPU fault can take the box down before pytest reports: say which case is starting
    if request.node.get_closest_marker("gpu"):
        print(f"\n[case] {request.node.nodeid}", flush=True)
    yield
