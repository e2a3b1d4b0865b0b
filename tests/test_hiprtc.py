"""The header library under hipRTC (run-time compilation has no host headers): kernel strings that
include <rocwmma/rocwmma.hpp> compile with hiprtcCompileProgram for gfx950 (no GPU needed for that),
and the reference's samples/hipRTC_gemm.cpp, built as the program it is, compiles its kernel string
against these headers at run time on the GPU and passes its own validation."""
import ctypes
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "rocwmma_amd", "include")
REF_SAMPLE = "/root/reference/samples/hipRTC_gemm.cpp"
RTC_BINARY = os.path.join(ROOT, "tests", "kernels", "_ref", "hiprtc_gemm")


def _hiprtc():
    for name in ("libhiprtc.so", "/opt/rocm/lib/libhiprtc.so"):
        try:
            return ctypes.CDLL(name)
        except OSError:
            continue
    return None


def _compile(source, options):
    """hiprtcCompileProgram(source); returns (result code, log)."""
    lib = _hiprtc()
    prog = ctypes.c_void_p()
    assert lib.hiprtcCreateProgram(ctypes.byref(prog), source.encode(), b"kernel.cu", 0, None, None) == 0
    opts = (ctypes.c_char_p * len(options))(*[o.encode() for o in options])
    rc = lib.hiprtcCompileProgram(prog, len(options), opts)
    n = ctypes.c_size_t(0)
    lib.hiprtcGetProgramLogSize(prog, ctypes.byref(n))
    log = ctypes.create_string_buffer(n.value + 1)
    if n.value:
        lib.hiprtcGetProgramLog(prog, log)
    size = ctypes.c_size_t(0)
    if rc == 0:
        lib.hiprtcGetCodeSize(prog, ctypes.byref(size))
    lib.hiprtcDestroyProgram(ctypes.byref(prog))
    return rc, log.value.decode(errors="replace"), size.value


OPTIONS = ["--offload-arch=gfx950", "-D__HIP_PLATFORM_AMD__", "--std=c++17", "-I" + INCLUDE]

OWN_KERNELS = r"""
#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>
using namespace rocwmma;

template <typename InT, typename AccT, uint32_t BM, uint32_t BN, uint32_t BK>
__device__ void tile(const InT* a, const InT* b, AccT* d, uint32_t lda, uint32_t ldb, uint32_t ldd)
{
    fragment<matrix_a, BM, BN, BK, InT, row_major> fa;
    fragment<matrix_b, BM, BN, BK, InT, col_major> fb;
    fragment<accumulator, BM, BN, BK, AccT>        fc;
    fill_fragment(fc, AccT(0));
    load_matrix_sync(fa, a, lda);
    load_matrix_sync(fb, b, ldb);
    mma_sync(fc, fa, fb, fc);
    store_matrix_sync(d, fc, ldd, mem_row_major);
}
extern "C" __global__ void k_f16(const float16_t* a, const float16_t* b, float32_t* d, uint32_t l) { tile<float16_t, float32_t, 32, 32, 16>(a, b, d, l, l, l); }
extern "C" __global__ void k_bf16(const bfloat16_t* a, const bfloat16_t* b, float32_t* d, uint32_t l) { tile<bfloat16_t, float32_t, 16, 16, 32>(a, b, d, l, l, l); }
extern "C" __global__ void k_i8(const int8_t* a, const int8_t* b, int32_t* d, uint32_t l) { tile<int8_t, int32_t, 16, 16, 64>(a, b, d, l, l, l); }
extern "C" __global__ void k_f8(const float8_t* a, const float8_t* b, float32_t* d, uint32_t l) { tile<float8_t, float32_t, 32, 32, 16>(a, b, d, l, l, l); }
extern "C" __global__ void k_f64(const float64_t* a, const float64_t* b, float64_t* d, uint32_t l) { tile<float64_t, float64_t, 16, 16, 4>(a, b, d, l, l, l); }
extern "C" __global__ void k_coop(const float16_t* a, float16_t* lds, uint32_t l)
{
    using Big = fragment<matrix_a, 128, 32, 16, float16_t, col_major>;
    Big f;
    const uint32_t w = threadIdx.x / 64;
    load_matrix_coop_sync<4>(f, a, l, w);
    store_matrix_coop_sync<4>(lds, f, 128, w);
    auto t = applyTranspose(f);
    (void)t;
    synchronize_workgroup();
}
"""


@pytest.mark.skipif(_hiprtc() is None, reason="needs libhiprtc")
def test_headers_compile_under_hiprtc():
    rc, log, size = _compile(OWN_KERNELS, OPTIONS)
    assert rc == 0, log[-3000:]
    assert size > 0


@pytest.mark.skipif(_hiprtc() is None or not os.path.exists(REF_SAMPLE), reason="needs libhiprtc and the reference tree")
def test_reference_hiprtc_sample_kernel_string_compiles():
    # the raw string literal the sample hands to hiprtcCreateProgram (samples/hipRTC_gemm.cpp:73-183),
    # with the sample's own options (:206) plus the target
    text = open(REF_SAMPLE).read()
    m = re.search(r'std::string source = R"\((.*?)\)";', text, re.S)
    assert m, "kernel string not found in the sample"
    rc, log, size = _compile(m.group(1), OPTIONS)
    assert rc == 0, log[-3000:]
    assert size > 0


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(RTC_BINARY), reason="reference hipRTC sample not built (needs the reference tree at build time)")
def test_reference_hiprtc_sample_runs_and_validates():
    # The sample looks for the headers under $ROCM_PATH/include (samples/hipRTC_gemm.cpp:185-187):
    # give it a root whose include/rocwmma is this library.
    with tempfile.TemporaryDirectory() as tmp:
        os.makedirs(os.path.join(tmp, "include"))
        os.symlink(os.path.join(INCLUDE, "rocwmma"), os.path.join(tmp, "include", "rocwmma"))
        env = dict(os.environ, ROCM_PATH=tmp)
        r = subprocess.run([RTC_BINARY], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout + r.stderr)[-2000:]
    assert "PASSED!" in r.stdout, r.stdout[-2000:]
