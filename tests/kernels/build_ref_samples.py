"""Builds the reference's own sample kernels against this library's headers into shared objects the
GPU tests can call: the sample sources are compiled where they lie (REFERENCE_ROOT, default
/root/reference) -- nothing of them is copied -- and the outputs go to tests/kernels/_ref/, which is
kept out of version control.  Without the reference tree this is a no-op and the tests skip."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.environ.get("REFERENCE_ROOT", "/root/reference")
OUT = os.path.join(HERE, "_ref")
WRAPPERS = ["simple_hgemm", "perf_hgemm", "simple_dlrm", "simple_sgemv", "simple_sgemm", "simple_dgemm", "perf_sgemm",
            "perf_dgemm", "test_dlrm", "test_io_traits", "test_gemm_simple", "test_gemm_multi", "test_gemm_coop", "test_gemm_coop_typed",
            "test_unit"]


def _compile(name, samples):
    out = os.path.join(OUT, "libref_%s.so" % name)
    subprocess.check_call([
        os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-std=c++17", "-O3", "-fPIC", "-shared",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-w",
        "-I" + os.path.join(ROOT, "rocwmma_amd", "include"), "-I" + samples, "-I" + os.path.join(REF, "test", "dlrm"),
        "-I" + os.path.join(REF, "test"), "-I" + os.path.join(REF, "test", "unit"), "-I" + os.path.join(REF, "test", "gemm"),
        "-I" + REF,
        os.path.join(HERE, "ref_samples", "wrap_%s.hip" % name), "-o", out])
    return out


def _compile_hiprtc_sample(samples):
    """samples/hipRTC_gemm.cpp as the program it is: its host side compiles the kernel string at run
    time with hipRTC, against whatever <ROCM_PATH>/include/rocwmma holds (samples/hipRTC_gemm.cpp:185-206),
    runs it and validates against its own CPU GEMM (:359-381)."""
    out = os.path.join(OUT, "hiprtc_gemm")
    subprocess.check_call([
        os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-std=c++17", "-O2", "-w",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
        "-I" + os.path.join(ROOT, "rocwmma_amd", "include"), "-I" + samples,
        os.path.join(samples, "hipRTC_gemm.cpp"), "-o", out, "-lhiprtc"])
    return out


def build():
    samples = os.path.join(REF, "samples")
    if not os.path.isdir(samples):
        return []
    os.makedirs(OUT, exist_ok=True)
    from concurrent.futures import ThreadPoolExecutor

    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        rtc = pool.submit(_compile_hiprtc_sample, samples)
        return list(pool.map(lambda n: _compile(n, samples), WRAPPERS)) + [rtc.result()]


if __name__ == "__main__":
    print("\n".join(build()) or "reference tree not found at %s: nothing built" % REF, file=sys.stderr)
