"""rocwmma_amd: MI355X (gfx950) matrix-fragment hot path -- GEMM, DLRM dot interaction, GEMV.

The device code lives in csrc/ (hand-written HIP) and include/rocwmma/ (the header-only
fragment API, same names as the reference's rocwmma.hpp).  This module is the thin host
side: it loads lib/librocwmma_amd.so and calls its C ABI (include/r355_wmma.h) with device
pointers.  There is no CPU fallback: if the library is missing, every call raises.

Argument order follows the reference kernel signature (test/gemm/gemm_kernel_base.hpp:101-114):
(m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librocwmma_amd.so")

# r355_dtype
F16, BF16, E4M3, I8, F32, I32, F64, E5M2 = range(8)
# r355_layout
ROW_MAJOR, COL_MAJOR = 0, 1
# r355_gemm_kernel
KERNEL_AUTO, KERNEL_SIMPLE, KERNEL_TILED, KERNEL_TILED_128, KERNEL_TILED_128_SPLITK, KERNEL_TILED_DEEP = 0, 1, 2, 3, 4, 5

DTYPE_BYTES = {F16: 2, BF16: 2, E4M3: 1, I8: 1, F32: 4, I32: 4, F64: 8, E5M2: 1}

EXPORTS = [
    "r355_gemm", "r355_gemm_noalloc", "r355_gemm_query", "r355_gemm_timed", "r355_dlrm_fwd", "r355_dlrm_fwd_timed",
    "r355_dlrm_bwd", "r355_gemv", "r355_gemv_timed", "r355_dgemv", "r355_gemv_workspace_bytes", "r355_gemv_ws", "r355_dgemv_ws", "r355_compress_24", "r355_decompress_24", "r355_compress_24_16", "r355_decompress_24_16",
    "r355_get_device_info", "r355_last_error", "r355_version",
]


class R355Error(RuntimeError):
    def __init__(self, code, message):
        super().__init__("r355 status %d: %s" % (code, message))
        self.code = code


class GemmArgs(ctypes.Structure):
    _fields_ = [
        ("in_type", ctypes.c_int32), ("out_type", ctypes.c_int32),
        ("layout_a", ctypes.c_int32), ("layout_b", ctypes.c_int32),
        ("layout_c", ctypes.c_int32), ("layout_d", ctypes.c_int32),
        ("m", ctypes.c_uint32), ("n", ctypes.c_uint32), ("k", ctypes.c_uint32),
        ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("c", ctypes.c_void_p), ("d", ctypes.c_void_p),
        ("lda", ctypes.c_uint32), ("ldb", ctypes.c_uint32), ("ldc", ctypes.c_uint32), ("ldd", ctypes.c_uint32),
        ("alpha", ctypes.c_double), ("beta", ctypes.c_double),
        ("sparse24", ctypes.c_int32), ("a_meta", ctypes.c_void_p),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_uint64),
    ]


class GemmPlan(ctypes.Structure):
    _fields_ = [
        ("kernel", ctypes.c_int32),
        ("macro_tile_m", ctypes.c_uint32), ("macro_tile_n", ctypes.c_uint32), ("macro_tile_k", ctypes.c_uint32),
        ("grid_x", ctypes.c_uint32), ("grid_y", ctypes.c_uint32),
        ("block_x", ctypes.c_uint32), ("block_y", ctypes.c_uint32),
        ("lds_bytes", ctypes.c_uint32),
        ("split_k", ctypes.c_uint32), ("workspace_bytes", ctypes.c_uint64),
    ]


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("arch", ctypes.c_char * 64), ("compute_units", ctypes.c_int32), ("wave_size", ctypes.c_int32),
        ("clock_mhz", ctypes.c_int32), ("memory_clock_mhz", ctypes.c_int32),
        ("lds_bytes_per_block", ctypes.c_int32), ("hbm_bytes", ctypes.c_uint64),
    ]


_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (python -m rocwmma_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "rocwmma_amd: %s is missing -- build it with `python -m rocwmma_amd.build`; "
                "there is no CPU fallback" % LIB_PATH)
        _share_torch_hip_runtime()
        L = ctypes.CDLL(LIB_PATH)
        vp, u32, i32, f32 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int32, ctypes.c_float
        fp = ctypes.POINTER(ctypes.c_float)
        L.r355_gemm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.r355_gemm_noalloc.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.r355_gemm_query.argtypes = [ctypes.POINTER(GemmArgs), ctypes.POINTER(GemmPlan)]
        L.r355_gemm_timed.argtypes = [ctypes.POINTER(GemmArgs), vp, ctypes.c_int, ctypes.c_int, fp]
        L.r355_dlrm_fwd.argtypes = [i32, vp, vp, u32, u32, u32, vp]
        L.r355_dlrm_fwd_timed.argtypes = [i32, vp, vp, u32, u32, u32, vp, ctypes.c_int, ctypes.c_int, fp]
        L.r355_dlrm_bwd.argtypes = [i32, vp, vp, vp, vp, u32, u32, u32, vp]
        L.r355_gemv.argtypes = [i32, u32, u32, vp, u32, vp, vp, vp, f32, f32, vp]
        L.r355_gemv_timed.argtypes = [i32, u32, u32, vp, u32, vp, vp, vp, f32, f32, vp, ctypes.c_int, ctypes.c_int, fp]
        L.r355_dgemv.argtypes = [i32, u32, u32, vp, u32, vp, vp, vp, ctypes.c_double, ctypes.c_double, vp]
        L.r355_gemv_workspace_bytes.argtypes, L.r355_gemv_workspace_bytes.restype = [i32, u32, u32, u32], ctypes.c_size_t
        L.r355_gemv_ws.argtypes = [i32, u32, u32, vp, u32, vp, vp, vp, f32, f32, vp, ctypes.c_size_t, vp]
        L.r355_dgemv_ws.argtypes = [i32, u32, u32, vp, u32, vp, vp, vp, ctypes.c_double, ctypes.c_double, vp, ctypes.c_size_t, vp]
        L.r355_compress_24.argtypes = [vp, u32, u32, vp, vp]
        L.r355_decompress_24.argtypes = [vp, vp, u32, u32, vp]
        L.r355_compress_24_16.argtypes = [vp, u32, u32, vp, vp]
        L.r355_decompress_24_16.argtypes = [vp, vp, u32, u32, vp]
        L.r355_get_device_info.argtypes = [ctypes.POINTER(DeviceInfo)]
        L.r355_last_error.argtypes = []
        L.r355_version.argtypes = []
        L.r355_last_error.restype = ctypes.c_char_p
        L.r355_version.restype = ctypes.c_char_p
        for name in EXPORTS:
            if name not in ("r355_last_error", "r355_version"):
                getattr(L, name).restype = ctypes.c_int
        _lib = L
    return _lib


def _share_torch_hip_runtime():
    """One HIP runtime per process.  A PyTorch wheel ships its own libamdhip64 and loads it by path; this library asks the
    loader for the system's.  With torch imported first the loader hands this library torch's copy (same SONAME) and all
    is well; the other way round the process ends up with two runtimes, torch's owns the device and every launch of this
    library fails with "no ROCm-capable device is detected".  So when a torch installation is present its runtime is
    loaded first - without importing torch."""
    import importlib.util
    import sys

    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return
    if spec is None or not spec.submodule_search_locations:
        return
    path = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if os.path.exists(path):
        try:
            ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        except OSError:
            pass  # (the system's runtime then; only a later `import torch` in this process would be a problem)


def _check(rc):
    if rc != 0:
        raise R355Error(rc, lib().r355_last_error().decode())


def _ptr(t):
    """Device (or host) address of a torch tensor / numpy array / raw int / None."""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data


def _stream_handle(stream):
    if stream is None:
        return None
    return getattr(stream, "cuda_stream", stream)


def default_ld(rows, cols, layout):
    return cols if layout == ROW_MAJOR else rows


def gemm_args(in_type, out_type, m, n, k, a, b, c, d, alpha, beta, layout_a, layout_b, layout_c, layout_d,
              lda=None, ldb=None, ldc=None, ldd=None, kernel=KERNEL_AUTO, a_meta=None, workspace=None, workspace_bytes=None):
    sparse = a_meta is not None
    g = GemmArgs()
    g.in_type, g.out_type = in_type, out_type
    g.layout_a, g.layout_b, g.layout_c, g.layout_d = layout_a, layout_b, layout_c, layout_d
    g.m, g.n, g.k = m, n, k
    g.a, g.b, g.c, g.d = _ptr(a), _ptr(b), _ptr(c), _ptr(d)
    g.lda = lda if lda is not None else default_ld(m, k // 2 if sparse else k, layout_a)
    g.ldb = ldb if ldb is not None else default_ld(k, n, layout_b)
    g.ldc = ldc if ldc is not None else default_ld(m, n, layout_c)
    g.ldd = ldd if ldd is not None else default_ld(m, n, layout_d)
    g.alpha, g.beta = alpha, beta
    g.sparse24, g.a_meta = int(sparse), _ptr(a_meta)
    g.kernel = kernel
    g.workspace = _ptr(workspace)
    if workspace_bytes is None:
        workspace_bytes = workspace.numel() * workspace.element_size() if hasattr(workspace, "numel") else 0
    g.workspace_bytes = workspace_bytes
    return g


def gemm(in_type, out_type, m, n, k, a, b, c, d, alpha=1.0, beta=0.0, layout_a=ROW_MAJOR, layout_b=COL_MAJOR,
         layout_c=ROW_MAJOR, layout_d=ROW_MAJOR, lda=None, ldb=None, ldc=None, ldd=None, kernel=KERNEL_AUTO,
         a_meta=None, stream=None, workspace=None):
    """D = alpha * A * B + beta * C on device buffers; asynchronous on `stream`."""
    g = gemm_args(in_type, out_type, m, n, k, a, b, c, d, alpha, beta, layout_a, layout_b, layout_c, layout_d,
                  lda, ldb, ldc, ldd, kernel, a_meta, workspace)
    _check(lib().r355_gemm(ctypes.byref(g), _stream_handle(stream)))


def gemm_noalloc(g, stream=None):
    """r355_gemm_noalloc on prepared GemmArgs: split-K partial results go to the library's static device buffer."""
    _check(lib().r355_gemm_noalloc(ctypes.byref(g), _stream_handle(stream)))


def gemm_query(g):
    plan = GemmPlan()
    _check(lib().r355_gemm_query(ctypes.byref(g), ctypes.byref(plan)))
    return plan


def gemm_timed(g, warmup, iters, stream=None):
    """Average milliseconds per launch (hipEvents on the launch stream, reference protocol)."""
    ms = ctypes.c_float(0.0)
    _check(lib().r355_gemm_timed(ctypes.byref(g), _stream_handle(stream), warmup, iters, ctypes.byref(ms)))
    return ms.value


def dlrm_fwd(dtype, x, out, m, k, batch, stream=None):
    _check(lib().r355_dlrm_fwd(dtype, _ptr(x), _ptr(out), m, k, batch, _stream_handle(stream)))


def dlrm_fwd_timed(dtype, x, out, m, k, batch, warmup, iters, stream=None):
    ms = ctypes.c_float(0.0)
    _check(lib().r355_dlrm_fwd_timed(dtype, _ptr(x), _ptr(out), m, k, batch, _stream_handle(stream), warmup, iters,
                                     ctypes.byref(ms)))
    return ms.value


def dlrm_bwd(dtype, x, upstream, mlp_grad, in_grad, m, k, batch, stream=None):
    _check(lib().r355_dlrm_bwd(dtype, _ptr(x), _ptr(upstream), _ptr(mlp_grad), _ptr(in_grad), m, k, batch,
                               _stream_handle(stream)))


def gemv_workspace_bytes(layout_a, m, k, elem_bytes=4):
    """Bytes of workspace the split-K form of the GEMV wants for a shape (0: the plain kernels serve it)."""
    return int(lib().r355_gemv_workspace_bytes(layout_a, m, k, elem_bytes))


def gemv(layout_a, m, k, a, x, y_in, y_out, alpha=1.0, beta=0.0, lda=None, stream=None, workspace=None, workspace_bytes=None):
    """workspace (device memory; workspace_bytes defaults to its size): r355_gemv_ws, which splits K where that pays."""
    lda = lda if lda is not None else default_ld(m, k, layout_a)
    if workspace is None:
        _check(lib().r355_gemv(layout_a, m, k, _ptr(a), lda, _ptr(x), _ptr(y_in), _ptr(y_out), alpha, beta,
                               _stream_handle(stream)))
    else:
        nbytes = workspace_bytes if workspace_bytes is not None else workspace.numel() * workspace.element_size()
        _check(lib().r355_gemv_ws(layout_a, m, k, _ptr(a), lda, _ptr(x), _ptr(y_in), _ptr(y_out), alpha, beta,
                                  _ptr(workspace), nbytes, _stream_handle(stream)))


def dgemv(layout_a, m, k, a, x, y_in, y_out, alpha=1.0, beta=0.0, lda=None, stream=None, workspace=None, workspace_bytes=None):
    """f64 GEMV (the reference's simple_dgemv sample); workspace as for gemv."""
    lda = lda if lda is not None else default_ld(m, k, layout_a)
    if workspace is None:
        _check(lib().r355_dgemv(layout_a, m, k, _ptr(a), lda, _ptr(x), _ptr(y_in), _ptr(y_out), alpha, beta,
                                _stream_handle(stream)))
    else:
        nbytes = workspace_bytes if workspace_bytes is not None else workspace.numel() * workspace.element_size()
        _check(lib().r355_dgemv_ws(layout_a, m, k, _ptr(a), lda, _ptr(x), _ptr(y_in), _ptr(y_out), alpha, beta,
                                   _ptr(workspace), nbytes, _stream_handle(stream)))


def gemv_timed(layout_a, m, k, a, x, y_in, y_out, alpha, beta, warmup, iters, lda=None, stream=None):
    lda = lda if lda is not None else default_ld(m, k, layout_a)
    ms = ctypes.c_float(0.0)
    _check(lib().r355_gemv_timed(layout_a, m, k, _ptr(a), lda, _ptr(x), _ptr(y_in), _ptr(y_out), alpha, beta,
                                 _stream_handle(stream), warmup, iters, ctypes.byref(ms)))
    return ms.value


def compress_24(dense):
    """Host-side 2:4 compression of a (m, k) numpy array of 1-byte (uint8 / int8) or 2-byte (uint16: f16 / bf16
    bit patterns, or float16) elements -> (values, meta) in the library's K-blocked storage (include/r355_wmma.h):
    values [stages][m / 16][4][16][16 / es] elements, meta [stages][m / 16][4][16][4 / es] bytes, a stage being
    128 / es dense elements of k.  m % 16 == 0, k % (128 / es) == 0."""
    import numpy as np

    dense = np.ascontiguousarray(dense)
    m, k = dense.shape
    es = dense.dtype.itemsize
    stages = k * es // 128
    values = np.zeros(m * k // 2, dtype=dense.dtype)
    meta = np.zeros(m * k // 8, dtype=np.uint8)
    fn = {1: lib().r355_compress_24, 2: lib().r355_compress_24_16}[es]
    _check(fn(_ptr(dense), m, k, _ptr(values), _ptr(meta)))
    return values.reshape(stages, m // 16, 4, 16, 16 // es), meta.reshape(stages, m // 16, 4, 16, 4 // es)


def decompress_24(values, meta):
    import numpy as np

    values, meta = np.ascontiguousarray(values), np.ascontiguousarray(meta)
    es = values.dtype.itemsize
    m, k = values.shape[1] * 16, values.shape[0] * 128 // es
    dense = np.zeros((m, k), dtype=values.dtype)
    fn = {1: lib().r355_decompress_24, 2: lib().r355_decompress_24_16}[es]
    _check(fn(_ptr(values), _ptr(meta), m, k, _ptr(dense)))
    return dense


def device_info():
    info = DeviceInfo()
    _check(lib().r355_get_device_info(ctypes.byref(info)))
    return info


def version():
    return lib().r355_version().decode()
