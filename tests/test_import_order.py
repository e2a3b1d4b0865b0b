"""The library loaded before torch is imported (a Python caller is free to do that): both must end up on one HIP runtime.
PyTorch wheels ship their own libamdhip64 and load it by path; with the system's runtime already in the process for this
library, torch's copy owned the device and every launch of this library failed with "no ROCm-capable device is detected".
Run in a child process, because the order of loading is the point."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
sys.path.insert(0, sys.argv[1])
import numpy as np
import rocwmma_amd as R
assert "torch" not in sys.modules
R.compress_24(np.zeros((16, 128), np.int8))      # loads the library: no torch in the process yet
import torch
a = torch.randint(-5, 5, (256 * 256,), dtype=torch.int8, device="cuda")
b = torch.randint(-5, 5, (256 * 256,), dtype=torch.int8, device="cuda")
d = torch.empty(256 * 256, dtype=torch.int32, device="cuda")
R.gemm(R.I8, R.I32, 256, 256, 256, a, b, None, d, 1.0, 0.0, R.ROW_MAJOR, R.COL_MAJOR, R.ROW_MAJOR, R.ROW_MAJOR)
torch.cuda.synchronize()
want = a.view(256, 256).to(torch.float64) @ b.view(256, 256).to(torch.float64).t()
assert torch.equal(d.view(256, 256).to(torch.float64), want)
runtimes = {l.split()[-1] for l in open("/proc/self/maps") if "libamdhip64" in l}
assert len(runtimes) == 1, runtimes
print("one runtime, result exact")
"""


def test_library_loaded_before_torch():
    r = subprocess.run([sys.executable, "-c", CHILD, ROOT], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "one runtime, result exact" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_stale_hip_error_of_another_caller_is_neither_reported_nor_consumed():
    """hipGetLastError is per thread and sticky: an earlier call of anybody that failed harmlessly (here a hipFree of a
    pointer nobody allocated, refused on the host) must not come back as this library's launch failure - and it must
    still be there for its owner afterwards: the entry points only peek at the pending error, as a plain kernel launch of
    the reference leaves it alone."""
    import ctypes

    import torch

    import rocwmma_amd as R

    a = torch.randint(-5, 5, (64 * 64,), dtype=torch.int8, device="cuda")
    d = torch.empty(64 * 64, dtype=torch.int32, device="cuda")
    y, ones_a, ones_x = torch.empty(64, device="cuda"), torch.ones(64 * 64, device="cuda"), torch.ones(64, device="cuda")
    loaded = sorted({l.split()[-1] for l in open("/proc/self/maps") if "libamdhip64" in l})
    assert len(loaded) == 1, loaded
    hip = ctypes.CDLL(loaded[0])  # the file is already mapped: this is a handle to the runtime in use, not another copy
    hip.hipFree.argtypes, hip.hipFree.restype = [ctypes.c_void_p], ctypes.c_int
    hip.hipGetLastError.argtypes, hip.hipGetLastError.restype = [], ctypes.c_int
    torch.cuda.synchronize()
    assert hip.hipGetLastError() == 0
    refused = hip.hipFree(ctypes.c_void_p(0x10))
    assert refused != 0
    R.gemm(R.I8, R.I32, 64, 64, 64, a, a, None, d, 1.0, 0.0, R.ROW_MAJOR, R.COL_MAJOR, R.ROW_MAJOR, R.ROW_MAJOR)  # no R355Error
    assert hip.hipGetLastError() == refused  # still pending for whoever caused it (fetched here, before torch trips over it)
    assert hip.hipGetLastError() == 0
    assert hip.hipFree(ctypes.c_void_p(0x10)) == refused
    R.gemv(R.ROW_MAJOR, 64, 64, ones_a, ones_x, None, y)
    assert hip.hipGetLastError() == refused and hip.hipGetLastError() == 0
    torch.cuda.synchronize()
    assert torch.equal(y, torch.full((64,), 64.0, device="cuda"))
    assert torch.equal(d.view(64, 64).double(), a.view(64, 64).double() @ a.view(64, 64).double().t())
