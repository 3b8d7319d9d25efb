"""Resource limits of every kernel in the built library, read from the code object's own metadata (no GPU).

After tests/kernel-limits.ts: that file sums the workgroup arrays each emitted shader declares and holds them to the
device's portable floor, independently of the formulas the host sizes tiles with. Here the compiler's per-kernel
metadata plays that part: fixed LDS against the 64 KiB a launch may use without opting in, scratch (register spills)
against zero, and the register budget of a wavefront. A kernel that starts
spilling or grows its LDS past the limit fails here, before any GPU run."""
import os
import re
import shutil
import struct
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "..", "gguf-trainer_amd", "libggufhip.so")
READELF = shutil.which("llvm-readelf") or "/opt/rocm/llvm/bin/llvm-readelf"

LDS_STATIC_LIMIT = 64 * 1024          # beyond this a kernel must take dynamic LDS and raise its attribute
REGS_PER_LANE = 512                   # unified VGPR + AGPR file of a gfx950 wavefront at one wave per SIMD
# kernel name fragment -> bytes of scratch it may use: none does (a scratch access waits for every load in flight, a kernel's prefetches included)
SPILL_ALLOWED = {}


def code_objects(blob):
    """gfx950 code objects inside the clang offload bundles of a host library."""
    out = []
    for m in re.finditer(b"__CLANG_OFFLOAD_BUNDLE__", blob):
        p = m.start() + 24
        n, = struct.unpack_from("<Q", blob, p)
        p += 8
        for _ in range(n):
            off, size, tl = struct.unpack_from("<QQQ", blob, p)
            p += 24
            triple = blob[p:p + tl].decode()
            p += tl
            if "gfx950" in triple and size:
                out.append(blob[m.start() + off:m.start() + off + size])
    return out


def kernels_of(co):
    with tempfile.NamedTemporaryFile(suffix=".co", delete=False) as f:
        f.write(co)
    try:
        text = subprocess.run([READELF, "--notes", f.name], capture_output=True, text=True, check=True).stdout
    finally:
        os.unlink(f.name)
    for k in re.split(r"\n\s+- \.agpr_count", "\n" + text)[1:]:
        def num(key):
            return int(re.search(r"\.%s:\s+(\d+)" % key, k).group(1))
        yield dict(name=re.search(r"\.name:\s+(\S+)", k).group(1), lds=num("group_segment_fixed_size"),
                   scratch=num("private_segment_fixed_size"), vgpr=num("vgpr_count"), sgpr=num("sgpr_count"),
                   wg=num("max_flat_workgroup_size"), wave=num("wavefront_size"))


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(LIB):
        pytest.skip("library not built")
    if not os.path.exists(READELF):
        pytest.skip("llvm-readelf not found")
    ks = [k for co in code_objects(open(LIB, "rb").read()) for k in kernels_of(co)]
    assert len(ks) > 150, len(ks)
    return ks


def test_every_kernel_family_is_in_the_library(kernels):
    names = " ".join(k["name"] for k in kernels)
    for family in ("gemm_kernel", "gemm_direct", "splitk_reduce", "rank_down_k", "rank_grad_k", "attn_fwd_mfma_k32",
                   "attn_fwd_mfma_k64", "attn_fwd_mfma_k128", "attn_bwd_dq_mfma", "attn_bwd_dkv_mfma", "attn_bwd_d_vec",
                   "rmsnorm", "rope_vec_k", "adamw", "colsum"):
        assert family in names, family
    # the kept-scores variant of dK/dV (template argument true) and the banded dQ product (last template argument true)
    assert any("attn_bwd_dkv_mfma_k64ILb1ELb1E" in k["name"] for k in kernels)
    assert any("gemm_direct" in k["name"] and k["name"].endswith("Lb0ELb1EEv8GemmArgs") for k in kernels)


def test_wavefronts_are_64_wide(kernels):
    assert {k["wave"] for k in kernels} == {64}


def test_fixed_lds_fits_without_opt_in(kernels):
    over = [(k["name"], k["lds"]) for k in kernels if k["lds"] > LDS_STATIC_LIMIT]
    assert not over, over


def test_no_kernel_spills(kernels):
    bad = []
    for k in kernels:
        allowed = max([v for n, v in SPILL_ALLOWED.items() if n in k["name"]], default=0)
        if k["scratch"] > allowed:
            bad.append((k["name"], k["scratch"]))
    assert not bad, bad


def test_register_budget(kernels):
    # metadata's vgpr_count is the unified count (arch + accumulation registers) on gfx90a and later
    over = [(k["name"], k["vgpr"]) for k in kernels if k["vgpr"] > REGS_PER_LANE or k["sgpr"] > 108]
    assert not over, over
    # a kernel launched with 256 threads needs one wave per SIMD to fit at all: 512 registers per lane at most
    assert all(k["wg"] <= 1024 for k in kernels)
