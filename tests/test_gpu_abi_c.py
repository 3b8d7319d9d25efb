"""The C ABI from a plain C host: include/ggufhip.h compiled with gcc and linked against libggufhip.so, no Python or
torch in the process that makes the calls."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "gguf-trainer_amd")


def test_c_host_links_and_runs(tmp_path):
    exe = str(tmp_path / "abi_host")
    cc = subprocess.run(["gcc", "-O1", "-Wall", "-Werror", os.path.join(ROOT, "tests", "abi_host.c"), "-I", os.path.join(ROOT, "include"),
                         "-L", PKG, "-lggufhip", "-lm", f"-Wl,-rpath,{PKG}", "-o", exe], capture_output=True, text=True)
    assert cc.returncode == 0, cc.stderr
    print("running the C host", flush=True)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.startswith("ok on "), (run.returncode, run.stdout, run.stderr)
