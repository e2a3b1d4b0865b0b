"""Helpers for the GPU parity tests: device buffers from numpy storage arrays, test-kernel library."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
API_LIB = os.path.join(_HERE, "kernels", "libapi_kernels.so")

_TORCH_VIEW = {1: "uint8", 2: "int16", 4: "int32", 8: "int64"}


def to_device(arr):
    """numpy array (any dtype) -> torch device tensor holding the same bytes."""
    import torch

    arr = np.ascontiguousarray(arr)
    raw = arr.view(getattr(np, _TORCH_VIEW[arr.dtype.itemsize])).reshape(-1)
    return torch.from_numpy(raw.copy()).cuda()


def device_filled(nbytes_elems, np_dtype, fill_byte=0xFF):
    """Device buffer of `nbytes_elems` elements of np_dtype, every byte = fill_byte (0xFF bytes are
    NaN for f16/bf16/f32/e4m3, so untouched outputs are caught)."""
    import torch

    itemsize = np.dtype(np_dtype).itemsize
    t = torch.full((nbytes_elems * itemsize,), fill_byte, dtype=torch.uint8, device="cuda")
    return t


def to_host(t, np_dtype, count=None):
    import torch

    torch.cuda.synchronize()
    a = t.cpu().numpy().view(np.uint8).reshape(-1)
    out = a.view(np_dtype)
    return out if count is None else out[:count]


def build_api_lib():
    src = os.path.join(_HERE, "kernels", "api_kernels.hip")
    inc = os.path.join(os.path.dirname(_HERE), "rocwmma_amd", "include")
    subprocess.check_call([
        os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-std=c++17", "-O3", "-fPIC", "-shared",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
        "-I" + inc, src, "-o", API_LIB])
    return API_LIB


_api = None


def api_lib():
    global _api
    if _api is None:
        if not os.path.exists(API_LIB):
            build_api_lib()
        _api = ctypes.CDLL(API_LIB)
    return _api
