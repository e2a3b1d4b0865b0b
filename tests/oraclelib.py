"""ctypes binding of the CPU oracle (oracle/liboracle.so) plus seeded input generators.

Test infrastructure only: imported by tests/, the smoke check and the benchmark's
cpu_baseline leg, never by the product package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")

F16, BF16, E4M3, I8, F32, I32, F64, E5M2 = range(8)
ROW, COL = 0, 1  # row_major ("T" in BLAS letters), col_major ("N")

NP_STORAGE = {F16: np.uint16, BF16: np.uint16, E4M3: np.uint8, I8: np.int8, F32: np.float32, I32: np.int32,
              F64: np.float64, E5M2: np.uint8}

_lib = None


def lib():
    global _lib
    if _lib is None:
        so = os.path.join(_ORACLE_DIR, "liboracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", _ORACLE_DIR, "-s"])
        L = ctypes.CDLL(so)
        vp, u32, i, f = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_float
        L.orc_gemm.argtypes = [i, i, i, i, i, i, u32, u32, u32, vp, vp, vp, vp, ctypes.c_double, ctypes.c_double]
        L.orc_gemm.restype = i
        L.orc_gemm_rows.argtypes = [i, i, i, i, u32, u32, u32, vp, vp, vp, u32, vp, ctypes.c_double]
        L.orc_gemm_rows.restype = i
        L.orc_dlrm_fwd.argtypes = [i, vp, vp, u32, u32, u32]
        L.orc_dlrm_fwd.restype = i
        L.orc_dlrm_bwd.argtypes = [i, vp, vp, vp, vp, u32, u32, u32]
        L.orc_dlrm_bwd.restype = i
        L.orc_compare.argtypes = [i, vp, vp, ctypes.c_size_t, ctypes.c_double, ctypes.POINTER(ctypes.c_double)]
        L.orc_compare.restype = i
        L.orc_fill_ref.argtypes = [i, vp, u32, u32, i]
        L.orc_fill_ref.restype = i
        L.orc_compress24.argtypes = [vp, u32, u32, vp, vp]
        L.orc_compress24.restype = i
        L.orc_decompress24.argtypes = [vp, vp, u32, u32, vp]
        L.orc_decompress24.restype = i
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = f
        L.orc_f32_to_f16.argtypes = [f]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = f
        L.orc_f32_to_bf16.argtypes = [f]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.orc_e4m3_to_f32.restype = f
        L.orc_f32_to_e4m3.argtypes = [f]
        L.orc_f32_to_e4m3.restype = ctypes.c_uint8
        L.orc_num_threads.restype = i
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def gemm(in_type, out_type, la, lb, lc, ld, m, n, k, a, b, c, alpha, beta):
    """Oracle GEMM on flat numpy storage arrays; returns flat D (layout ld)."""
    d = np.zeros(m * n, dtype=NP_STORAGE[out_type])
    if c is None:
        c = np.zeros(m * n, dtype=NP_STORAGE[out_type])
    a, b, c = np.ascontiguousarray(a), np.ascontiguousarray(b), np.ascontiguousarray(c)
    rc = lib().orc_gemm(in_type, out_type, la, lb, lc, ld, m, n, k, _p(a), _p(b), _p(c), _p(d), alpha, beta)
    if rc != 0:
        raise ValueError("oracle: unsupported type combination")
    return d


def gemm_rows(in_type, out_type, la, lb, m, n, k, a, b, rows, alpha=1.0):
    rows = np.ascontiguousarray(rows, dtype=np.uint32)
    d = np.zeros(len(rows) * n, dtype=NP_STORAGE[out_type])
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    rc = lib().orc_gemm_rows(in_type, out_type, la, lb, m, n, k, _p(a), _p(b), _p(rows), len(rows), _p(d), alpha)
    if rc != 0:
        raise ValueError("oracle: bad row index")
    return d.reshape(len(rows), n)


def dlrm_fwd(dtype, x, m, k, batch):
    x = np.ascontiguousarray(x)
    out = np.zeros(batch * (m * (m - 1) // 2 + k), dtype=NP_STORAGE[dtype])
    rc = lib().orc_dlrm_fwd(dtype, _p(x), _p(out), m, k, batch)
    assert rc == 0
    return out.reshape(batch, -1)


def dlrm_bwd(dtype, x, up, m, k, batch):
    x, up = np.ascontiguousarray(x), np.ascontiguousarray(up)
    mlp = np.zeros(batch * k, dtype=NP_STORAGE[dtype])
    out = np.zeros(batch * m * k, dtype=NP_STORAGE[dtype])
    rc = lib().orc_dlrm_bwd(dtype, _p(x), _p(up), _p(mlp), _p(out), m, k, batch)
    assert rc == 0
    return mlp.reshape(batch, k), out.reshape(batch, m, k)


def compare(dtype, x, y, tolerance=10.0):
    """Reference metric max |a-b|/(|a|+|b|+1); returns (passed, max_rel)."""
    x, y = np.ascontiguousarray(x).ravel(), np.ascontiguousarray(y).ravel()
    assert x.size == y.size and x.dtype == y.dtype
    mx = ctypes.c_double(0.0)
    rc = lib().orc_compare(dtype, _p(x), _p(y), x.size, tolerance, ctypes.byref(mx))
    assert rc >= 0
    return bool(rc), mx.value


def fill_ref(dtype, m, n, layout):
    mat = np.zeros(m * n, dtype=NP_STORAGE[dtype])
    assert lib().orc_fill_ref(dtype, _p(mat), m, n, layout) == 0
    return mat


def compress24(dense_u8, m, k):
    """K-blocked 2:4 storage of a (m, k) matrix of 1-byte elements: values [k / 128][m / 16][4][16][16] and
    meta [k / 128][m / 16][4][16][4] (see orc_compress24)."""
    dense_u8 = np.ascontiguousarray(dense_u8).view(np.uint8)
    vals = np.zeros(m * k // 2, dtype=np.uint8)
    meta = np.zeros(m * k // 8, dtype=np.uint8)
    rc = lib().orc_compress24(_p(dense_u8), m, k, _p(vals), _p(meta))
    if rc != 0:
        raise ValueError("not a 2:4 matrix (or m % 16, k % 128)")
    return vals.reshape(k // 128, m // 16, 4, 16, 16), meta.reshape(k // 128, m // 16, 4, 16, 4)


def decompress24(vals, meta, m, k):
    vals, meta = np.ascontiguousarray(vals), np.ascontiguousarray(meta)
    dense = np.zeros(m * k, dtype=np.uint8)
    assert lib().orc_decompress24(_p(vals), _p(meta), m, k, _p(dense)) == 0
    return dense.reshape(m, k)


def plain_to_kblocked(plain, m, k, es=1):
    """Independent statement of the K-blocked order with array axes instead of offsets: `plain` is (m, bytes per row)
    with the row's bytes in k order (kept values: k / 2 * es bytes, metadata: k / 8 bytes); a stage is 128 dense bytes
    of k and splits a row's bytes into 4 equal lane-group pieces."""
    plain = np.ascontiguousarray(plain).view(np.uint8).reshape(m, -1)
    stages = k * es // 128
    piece = plain.shape[1] // stages // 4
    return plain.reshape(m // 16, 16, stages, 4, piece).transpose(2, 0, 3, 1, 4).copy()


# ----------------------------------------------------------------- conversions (vectorised)

def f32_to_storage(x, dtype):
    """Round a float32 numpy array to the storage bits of dtype (RNE)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == F16:
        return x.astype(np.float16).view(np.uint16)
    if dtype == BF16:
        u = x.view(np.uint32).astype(np.uint64)
        u = u + 0x7FFF + ((u >> 16) & 1)
        return (u >> 16).astype(np.uint16)
    if dtype == E4M3:
        return e4m3_encode(x)
    if dtype == I8:
        return x.astype(np.int8)
    if dtype == F32:
        return x
    if dtype == I32:
        return x.astype(np.int32)
    if dtype == F64:
        return x.astype(np.float64)
    raise ValueError(dtype)


def storage_to_f32(s, dtype):
    s = np.asarray(s)
    if dtype == F16:
        return s.view(np.float16).astype(np.float32)
    if dtype == BF16:
        return (s.astype(np.uint32) << 16).view(np.float32)
    if dtype == E4M3:
        return E4M3_TABLE[s.view(np.uint8)]
    if dtype == E5M2:  # the high byte of the binary16 with the same value
        return (s.view(np.uint8).astype(np.uint16) << 8).view(np.float16).astype(np.float32)
    return s.astype(np.float32)


def _e4m3_table():
    t = np.zeros(256, dtype=np.float32)
    for v in range(256):
        s, e, m = v >> 7, (v >> 3) & 0xF, v & 7
        if e == 15 and m == 7:
            r = float("nan")
        elif e == 0:
            r = m * 2.0 ** -9
        else:
            r = (8 + m) * 2.0 ** (e - 10)
        t[v] = -r if s else r
    return t


E4M3_TABLE = _e4m3_table()


def e4m3_encode(x):
    """Vectorised OCP e4m3 encode, RNE, saturate-to-finite (independent of the C oracle:
    nearest-code search over the sorted table of finite positive codes)."""
    x = np.asarray(x, dtype=np.float32)
    pos = E4M3_TABLE[:0x7F].astype(np.float64)  # codes 0..0x7E ascending
    a = np.abs(x.astype(np.float64))
    a = np.minimum(a, 448.0)
    hi = np.searchsorted(pos, a, side="left").clip(0, 0x7E)
    lo = (hi - 1).clip(0, 0x7E)
    dlo, dhi = np.abs(a - pos[lo]), np.abs(pos[hi] - a)
    pick = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    code = pick.astype(np.uint8) | (np.signbit(x).astype(np.uint8) << 7)
    code = np.where(np.isnan(x), np.uint8(0x7F), code)
    return code.astype(np.uint8)


# ----------------------------------------------------------------- seeded inputs

def _splitmix64(seed, n):
    """Counter-based generator: element i depends only on (seed, i)."""
    with np.errstate(over="ignore"):
        z = (np.arange(n, dtype=np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15) + np.uint64(seed) * np.uint64(0xD1B54A32D192ED03)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform_pm1(seed, n):
    """float32 uniform in [-1, 1)."""
    u = (_splitmix64(seed, n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (2.0 * u - 1.0).astype(np.float32)


def uniform_int8(seed, n):
    return ((_splitmix64(seed, n) >> np.uint64(32)) & np.uint64(0xFF)).astype(np.uint8).view(np.int8)


def normal(seed, n):
    """float32 N(0,1) by Box-Muller on two counter streams."""
    u1 = ((_splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
    u2 = (_splitmix64(seed + 7919, n) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    return (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def sparse24_mask(seed, m, k):
    """Boolean m x k mask with exactly two True per aligned group of four along k."""
    r = (_splitmix64(seed, m * (k // 4)) >> np.uint64(20)) % np.uint64(6)
    pairs = np.array([[0, 1], [0, 2], [0, 3], [1, 2], [1, 3], [2, 3]], dtype=np.int64)
    sel = pairs[r.astype(np.int64)]
    mask = np.zeros((m * (k // 4), 4), dtype=bool)
    rows = np.arange(mask.shape[0])
    mask[rows, sel[:, 0]] = True
    mask[rows, sel[:, 1]] = True
    return mask.reshape(m, k)


def as_matrix(flat, rows, cols, layout):
    """View flat storage as a logical rows x cols array."""
    return flat.reshape(rows, cols) if layout == ROW else flat.reshape(cols, rows).T


def to_flat(mat, layout):
    return np.ascontiguousarray(mat if layout == ROW else mat.T).ravel()
