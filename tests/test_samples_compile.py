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


# Device headers of the reference's own test suites that stay inside the fragment API surface.
TEST_DEVICE_HEADERS = [
    "unit/load_store_matrix_sync_test/device/load_store_matrix_sync.hpp",
    "unit/load_store_matrix_coop_sync_test/device/load_store_matrix_coop_sync.hpp",
    "unit/fill_fragment_test/device/fill_fragment.hpp",
    "unit/contamination_test/device/load_contamination.hpp",
    "unit/contamination_test/device/store_contamination.hpp",
    "unit/map_util_test/device/map_block_to_matrix.hpp",
    "unit/map_util_test/device/map_block_to_matrix_override.hpp",
    "unit/map_util_test/device/map_matrix_to_data.hpp",
    "unit/map_util_test/device/map_matrix_to_data_override.hpp",
    "unit/map_util_test/device/map_thread_to_matrix.hpp",
    "unit/map_util_test/device/map_wave_to_matrix.hpp",
    "dlrm/device/dlrm_dot_fwd.hpp",
    "dlrm/device/dlrm_dot_bwd.hpp",
    "gemm/gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp",
    "gemm/gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp",
    "gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp",
    "dlrm/device/dlrm_dot_fwd_lds.hpp",
    "dlrm/device/dlrm_dot_bwd_lds.hpp",
]
REF_TEST = "/root/reference/test"


@pytest.mark.skipif(not os.path.isdir(REF_TEST) or not os.path.exists(HIPCC), reason="needs the reference tree and hipcc")
@pytest.mark.parametrize("header", TEST_DEVICE_HEADERS)
def test_reference_test_device_header_compiles_unchanged(header):
    """The kernels in these headers are templates; the translation unit here only has to parse and
    semantically check them against this library's headers (the run-time check of the DLRM ones is
    tests/test_ref_samples_run.py)."""
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "tu.hip")
        with open(src, "w") as f:
            f.write('#include <iostream>\n#include <hip/hip_runtime.h>\n#include <rocwmma/rocwmma.hpp>\n#include <rocwmma/rocwmma_coop.hpp>\n'
                    '#include <rocwmma/rocwmma_transforms.hpp>\n#include "%s"\n' % header)
        r = subprocess.run(
            [HIPCC, "--offload-arch=gfx950", "-std=c++17", "-O1", "-c", "--cuda-device-only", "-w",
             "-I" + os.path.join(ROOT, "rocwmma_amd", "include"), "-I" + REF_TEST, "-I" + os.path.join(REF_TEST, "unit"),
             "-I" + os.path.join(REF_TEST, "dlrm"), "-I" + os.path.join(REF_TEST, "gemm"), src, "-o",
             os.path.join(tmp, "tu.o")],
            capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]


def test_version_header_reports_the_api_version():
    """rocwmma/rocwmma-version.hpp: the three macros and rocwmma_get_version() the reference configures at build time
    (library/include/rocwmma/internal/rocwmma-version.hpp.in), host-only."""
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("needs g++")
    with tempfile.TemporaryDirectory() as tmp:
        src, exe = os.path.join(tmp, "v.cpp"), os.path.join(tmp, "v")
        with open(src, "w") as f:
            f.write('#include <rocwmma/rocwmma-version.hpp>\n#include <cstdio>\n'
                    'int main() { std::printf("%s %d", rocwmma_get_version().c_str(), ROCWMMA_VERSION_MAJOR * 10000 + '
                    'ROCWMMA_VERSION_MINOR * 100 + ROCWMMA_VERSION_PATCH); }\n')
        subprocess.check_call([gxx, "-std=c++17", "-I" + os.path.join(ROOT, "rocwmma_amd", "include"), src, "-o", exe])
        assert subprocess.check_output([exe], text=True) == "1.6.0 10600"
