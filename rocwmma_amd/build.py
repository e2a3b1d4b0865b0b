"""Builds the gfx950 shared library (csrc/*.hip, csrc/api.cpp -> lib/librocwmma_amd.so) with hipcc.

Usage: python -m rocwmma_amd.build [--force] [--timeline] [--variant <name> -D<macro> ...]
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


def _build_twin(prefix, defines, sources, out, verbose):
    """A second library beside the shipped one: the objects of `sources` (names of csrc files) recompiled with `defines`,
    everything else from the ordinary objects.  Never loaded by the package itself."""
    build(verbose=False)
    again = [s for s in SOURCES if s[0] in sources]
    with ThreadPoolExecutor(max_workers=min(4, os.cpu_count() or 1)) as ex:
        twin = list(ex.map(lambda s: _compile((s[0], prefix + s[1], s[2] + defines), False), again))
    objs = [os.path.join(OBJDIR, stem + ".o") for src, stem, _ in SOURCES if src not in sources] + [o for o, _ in twin]
    os.makedirs(os.path.dirname(out), exist_ok=True)
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", out)
    return out


def build_timeline(verbose=True):
    """The profiling twin of the library (lib/librocwmma_amd_timeline.so, read by rocwmma_amd.timeline): the macro-tile
    kernels compiled with -DR355_TIMELINE."""
    return _build_twin("tl_", ["-DR355_TIMELINE"], ["gemm_tiled.hip"], TIMELINE_LIB, verbose)


def build_variant(name, defines, verbose=True):
    """A measurement build (lib/variant_<name>/librocwmma_amd.so): the kernel sources that know measurement macros
    recompiled with `defines` (e.g. ["-DR355_ABLATE_MFMA"]).  `LD_LIBRARY_PATH=rocwmma_amd/lib/variant_<name>
    rocwmma_amd/lib/host_bench ...` then runs host_bench on it."""
    return _build_twin("var_%s_" % name, list(defines), ["sparse.hip", "dlrm.hip", "dlrm_general.hip"], os.path.join(LIBDIR, "variant_" + name, "librocwmma_amd.so"), verbose)


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
    if "--variant" in sys.argv:  # --variant <name> -D<macro> [-D<macro> ...]
        build_variant(sys.argv[sys.argv.index("--variant") + 1], [a for a in sys.argv if a.startswith("-D")])
