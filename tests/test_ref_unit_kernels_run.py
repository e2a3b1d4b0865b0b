"""The reference's unit-test device kernels (test/unit/**/device/*.hpp: load/store round trip, cooperative
load/store, fill, load and store contamination, for matrix_a / matrix_b / accumulator fragments, and the
MappingUtil kernels of test/unit/map_util_test), compiled
UNCHANGED against this library's headers by tests/kernels/build_ref_samples.py where the reference tree is
available, checked with the reference suite's own pass criteria on MI355X.  The shared object is a build
output (tests/kernels/_ref/); when it is absent the tests skip."""
import ctypes
import os

import numpy as np
import pytest

from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernels", "_ref", "libref_test_unit.so")
N_CASES = 22
ROLES = {0: "A", 1: "B", 2: "Acc"}
_lib_cache = []


def _lib():
    if not os.path.exists(_SO):
        pytest.skip("libref_test_unit.so not built (needs the reference tree at build time)")
    if not _lib_cache:
        L = ctypes.CDLL(_SO)
        L.ref_unit_run.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                   ctypes.c_void_p, ctypes.c_uint32, ctypes.c_double, ctypes.c_double]
        _lib_cache.append(L)
    return _lib_cache[0]


def _info(cid):
    bm, bn, eb, rm = (ctypes.c_uint32() for _ in range(4))
    assert _lib().ref_unit_case_info(cid, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(eb), ctypes.byref(rm)) == 0
    return bm.value, bn.value, eb.value, bool(rm.value)


_DT = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}


def _matrix(rows, cols, eb, seed):
    """Distinct-ish finite bit patterns (small positive numbers in every float format)."""
    limit = {1: 0x70, 2: 0x3C00, 4: 0x3F800000, 8: 0x3FF0000000000000}[eb]
    v = (np.arange(rows * cols, dtype=np.uint64) * 2654435761 + seed) % limit
    return v.astype(_DT[eb]).reshape(rows, cols)


def _flat(mat, row_major):
    return np.ascontiguousarray(mat if row_major else mat.T).ravel()


def _unflat(flat, rows, cols, row_major):
    return flat.reshape(rows, cols) if row_major else flat.reshape(cols, rows).T


def _run(kind, cid, m, n, d_in, d_out, ld, p1=0.0, p2=0.0):
    rc = _lib().ref_unit_run(kind, cid, m, n, ctypes.c_void_p(d_in.data_ptr() if d_in is not None else 0),
                             ctypes.c_void_p(d_out.data_ptr()), ld, p1, p2)
    assert rc == 0


@pytest.mark.parametrize("role", [0, 1, 2])
@pytest.mark.parametrize("cid", range(N_CASES))
def test_load_store_matrix_sync(cid, role):
    # pass criterion of the suite: output == input (test/unit/load_store_matrix_sync_test)
    bm, bn, eb, rm = _info(cid)
    m, n = 4 * bm, 4 * bn
    mat = _matrix(m, n, eb, cid)
    d_in, d_out = to_device(_flat(mat, rm)), device_filled(m * n, _DT[eb], 0xEE)
    _run(role, cid, m, n, d_in, d_out, n if rm else m)
    assert np.array_equal(_unflat(to_host(d_out, _DT[eb]), m, n, rm), mat)


@pytest.mark.parametrize("share", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("role", [0, 1, 2])
@pytest.mark.parametrize("cid", range(0, N_CASES, 2))
def test_load_store_matrix_coop_sync(cid, role, share):
    # param1: waves of one workgroup row (0) or column (1) cooperate; param2: which row / column.  The
    # cooperating waves copy every block the workgroup covers: output == input
    # (test/unit/load_store_matrix_coop_sync_test)
    bm, bn, eb, rm = _info(cid)
    m, n = 4 * bm, 4 * bn
    mat = _matrix(m, n, eb, 100 + cid)
    d_in, d_out = to_device(_flat(mat, rm)), device_filled(m * n, _DT[eb], 0xEE)
    _run(3 + role, cid, m, n, d_in, d_out, n if rm else m, float(share[0]), float(share[1]))
    assert np.array_equal(_unflat(to_host(d_out, _DT[eb]), m, n, rm), mat)


@pytest.mark.parametrize("role", [0, 1, 2])
@pytest.mark.parametrize("cid", range(N_CASES))
def test_fill_fragment(cid, role):
    # pass criterion: every element == param1 (test/unit/fill_fragment_test)
    bm, bn, eb, rm = _info(cid)
    m, n = 2 * bm, 2 * bn
    d_out = device_filled(m * n, _DT[eb], 0xEE)
    _run(6 + role, cid, m, n, None, d_out, n if rm else m, 5.0)
    out = to_host(d_out, _DT[eb])
    assert np.all(out == out[0]) and out[0] != np.frombuffer(bytes([0xEE] * eb), dtype=_DT[eb])[0]


@pytest.mark.parametrize("role", [0, 1, 2])
@pytest.mark.parametrize("cid", range(0, N_CASES, 2))
def test_load_and_store_contamination(cid, role):
    # the matrix sits inside a frame of param1 rows / param2 columns on every side; loads must not read
    # the frame into the result and stores must not write into it (test/unit/contamination_test)
    bm, bn, eb, rm = _info(cid)
    m, n = 2 * bm, 2 * bn
    pr = pc = 16 // eb * 2  # keeps every block origin 16-byte aligned
    canary = np.frombuffer(bytes([0xEE] * eb), dtype=_DT[eb])[0]
    mat = _matrix(m, n, eb, 200 + cid)
    framed = np.full((m + 2 * pr, n + 2 * pc), canary, dtype=_DT[eb])
    framed[pr:pr + m, pc:pc + n] = mat
    ld = n if rm else m
    # load contamination: framed input -> plain output
    d_in, d_out = to_device(_flat(framed, rm)), device_filled(m * n, _DT[eb], 0xAA)
    _run(9 + role, cid, m, n, d_in, d_out, ld, float(pr), float(pc))
    assert np.array_equal(_unflat(to_host(d_out, _DT[eb]), m, n, rm), mat)
    # store contamination: plain input -> framed output; the frame keeps its fill
    d_in, d_out = to_device(_flat(mat, rm)), device_filled(framed.size, _DT[eb], 0xEE)
    _run(12 + role, cid, m, n, d_in, d_out, ld, float(pr), float(pc))
    got = _unflat(to_host(d_out, _DT[eb]), m + 2 * pr, n + 2 * pc, rm)
    assert np.array_equal(got[pr:pr + m, pc:pc + n], mat)
    got[pr:pr + m, pc:pc + n] = canary
    assert np.all(got == canary)


# MappingUtil (test/unit/map_util_test): every wave copies the block its coordinates name; 2 x 2 workgroups of
# 2 x 2 waves cover a 4 x 4 grid of blocks
@pytest.mark.parametrize("kind", [15, 18, 21, 22])
@pytest.mark.parametrize("cid", range(N_CASES))
def test_map_util_identity_copies(cid, kind):
    # MapBlockToMatrix, MapMatrixToData, MapThreadToMatrix, MapWaveToMatrix: pass criterion output == input
    # (test/unit/map_util_test/detail/map_block_to_matrix.hpp:65-79)
    bm, bn, eb, rm = _info(cid)
    m, n = 4 * bm, 4 * bn
    mat = _matrix(m, n, eb, 300 + cid)
    d_in, d_out = to_device(_flat(mat, rm)), device_filled(m * n, _DT[eb], 0xEE)
    _run(kind, cid, m, n, d_in, d_out, n if rm else m)
    assert np.array_equal(_unflat(to_host(d_out, _DT[eb]), m, n, rm), mat)


@pytest.mark.parametrize("override", [0, 1, 3])
@pytest.mark.parametrize("kind", [16, 17, 19, 20])
@pytest.mark.parametrize("cid", range(0, N_CASES, 2))
def test_map_util_block_overrides(cid, kind, override):
    # ...OverrideM / ...OverrideN: every block is read from block row (column) param1 - MapMatrixToData...: from matrix
    # row (column) param1 - instead of its own, and written to its own place
    # (test/unit/map_util_test/detail/map_block_to_matrix_override.hpp:118-150, map_matrix_to_data_override.hpp:130-150)
    bm, bn, eb, rm = _info(cid)
    m, n = 4 * bm, 4 * bn
    along_m = kind in (16, 19)
    blk = bm if along_m else bn
    if kind in (16, 17):
        param, first = override, override * blk
    else:  # a matrix coordinate; kept on 16-element steps so that the fragments' vector accesses stay aligned
        param = first = min(16 * override * override, 3 * blk) // 16 * 16
    mat = _matrix(m, n, eb, 400 + cid)
    d_in, d_out = to_device(_flat(mat, rm)), device_filled(m * n, _DT[eb], 0xEE)
    _run(kind, cid, m, n, d_in, d_out, n if rm else m, float(param))
    want = mat.copy()
    for b in range(4):
        if along_m:
            want[b * bm:(b + 1) * bm, :] = mat[first:first + bm, :]
        else:
            want[:, b * bn:(b + 1) * bn] = mat[:, first:first + bn]
    assert np.array_equal(_unflat(to_host(d_out, _DT[eb]), m, n, rm), want)
