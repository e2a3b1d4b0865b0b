"""Drop-in check of the header API: the reference's own sample kernels compile unchanged for gfx950
against rocwmma_amd/include.  Needs the reference tree and hipcc; skipped where either is absent
(the GPU box has no /root/reference)."""
import os
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/samples"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SAMPLES = ["simple_hgemm", "perf_hgemm", "simple_sgemv", "simple_dlrm", "simple_sgemm", "perf_sgemm", "simple_dgemm",
           "perf_dgemm", "simple_dgemv"]


@pytest.mark.skipif(not os.path.isdir(REF) or not os.path.exists(HIPCC), reason="needs the reference tree and hipcc")
@pytest.mark.parametrize("sample", SAMPLES)
def test_reference_sample_compiles_unchanged(sample):
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, sample + ".s")
        r = subprocess.run(
            [HIPCC, "--offload-arch=gfx950", "-std=c++17", "-O3", "-DNDEBUG", "--cuda-device-only", "-S",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "-I" + os.path.join(ROOT, "rocwmma_amd", "include"), "-I" + REF, os.path.join(REF, sample + ".cpp"), "-o", out],
            capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        asm = open(out).read()
        assert "v_mfma_" in asm  # the fragment API lowered to matrix instructions
        assert "scratch_" not in asm  # fragments stay in registers
