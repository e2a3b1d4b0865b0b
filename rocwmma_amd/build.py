"""Builds the gfx950 shared library (csrc/*.hip, csrc/api.cpp -> lib/librocwmma_amd.so) with hipcc.

Usage: python -m rocwmma_amd.build [--force] [--timeline]
Objects are rebuilt when their source (or any header) is newer; translation units compile in parallel.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INC = os.path.join(HERE, "include")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "librocwmma_amd.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# (source, object stem, extra flags); gemm_tiled.hip is compiled once per kernel family so that the four
# parts build in parallel
SOURCES = [("api.cpp", "api", []), ("gemm_simple.hip", "gemm_simple", []),
           ("gemm_tiled.hip", "gemm_tiled_p0", ["-DR355_TILED_PART=0"]), ("gemm_tiled.hip", "gemm_tiled_p1", ["-DR355_TILED_PART=1"]),
           ("gemm_tiled.hip", "gemm_tiled_p2", ["-DR355_TILED_PART=2"]), ("gemm_tiled.hip", "gemm_tiled_p3", ["-DR355_TILED_PART=3"]),
           ("dlrm.hip", "dlrm", []), ("dlrm_general.hip", "dlrm_general", []), ("sparse.hip", "sparse", []), ("gemv.hip", "gemv", [])]

# packed-fp32 instructions are disabled on purpose (device pass only; the host pass warns that it
# does not know the feature, which is harmless)
FLAGS = [
    "--offload-arch=gfx950", "-std=c++17", "-O3", "-fPIC", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-I" + INC,
]


def _headers():
    hs = []
    for root in (CSRC, INC, os.path.join(os.path.dirname(HERE), "include")):
        for d, _, files in os.walk(root):
            hs += [os.path.join(d, f) for f in files if f.endswith((".hpp", ".h"))]
    return hs


def _compile(item, force):
    src, stem, extra = item
    obj = os.path.join(OBJDIR, stem + ".o")
    path = os.path.join(CSRC, src)
    newest = max(os.path.getmtime(p) for p in [path] + _headers())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj, False
    r = subprocess.run([HIPCC] + FLAGS + extra + ["-c", path, "-o", obj], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
    return obj, True


def build(force=False, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        results = list(ex.map(lambda s: _compile(s, force), SOURCES))
    objs = [o for o, _ in results]
    if force or any(c for _, c in results) or not os.path.exists(LIB):
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs,
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


TIMELINE_LIB = os.path.join(LIBDIR, "librocwmma_amd_timeline.so")


def build_timeline(verbose=True):
    """The profiling twin of the library (lib/librocwmma_amd_timeline.so, read by rocwmma_amd.timeline): the macro-tile
    kernels compiled with -DR355_TIMELINE, everything else from the ordinary objects.  Never loaded by the package itself."""
    build(verbose=False)
    tiled = [s for s in SOURCES if s[0] == "gemm_tiled.hip"]
    with ThreadPoolExecutor(max_workers=min(4, os.cpu_count() or 1)) as ex:
        tl = list(ex.map(lambda s: _compile((s[0], "tl_" + s[1], s[2] + ["-DR355_TIMELINE"]), False), tiled))
    objs = [os.path.join(OBJDIR, stem + ".o") for src, stem, _ in SOURCES if src != "gemm_tiled.hip"] + [o for o, _ in tl]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", TIMELINE_LIB] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", TIMELINE_LIB)
    return TIMELINE_LIB


def build_host_bench(verbose=True):
    """C++ host bench (csrc/host_bench.cpp -> lib/host_bench), linked against the C-ABI library."""
    exe = os.path.join(LIBDIR, "host_bench")
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-std=c++17", "-O2", "-x", "hip",
                        "-Wno-unused-command-line-argument", os.path.join(CSRC, "host_bench.cpp"), "-o", exe,
                        "-L" + LIBDIR, "-lrocwmma_amd", "-Wl,-rpath,$ORIGIN"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host_bench build failed:\n" + r.stderr)
    if verbose:
        print("built", exe)
    return exe


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    build_host_bench()
    if "--timeline" in sys.argv:
        build_timeline()
