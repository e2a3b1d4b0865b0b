"""GPU checks of the header-only fragment API (rocwmma_amd/include/rocwmma) through small device
kernels (tests/kernels/api_kernels.hip).  The invariants are the reference's unit-test invariants:
load -> store returns the block and nothing else (test/unit/load_store_matrix_sync_test,
contamination_test), fill stores a constant (fill_fragment_test), cooperative load/store over
1..8 waves reproduces the block (load_store_matrix_coop_sync_test), MappingUtil arithmetic
(map_util_test), and mma_sync on one tile equals the CPU oracle's gemm."""
import ctypes

import numpy as np
import pytest

import oraclelib as O
from gpuutil import api_lib, device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

CASES = list(range(94))


def _info(cid):
    r, c, eb, rm, ne = (ctypes.c_uint32() for _ in range(5))
    assert api_lib().api_case_info(cid, ctypes.byref(r), ctypes.byref(c), ctypes.byref(eb), ctypes.byref(rm), ctypes.byref(ne)) == 0
    return r.value, c.value, eb.value, bool(rm.value), ne.value


def _np_dtype(eb):
    return {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[eb]


def _padded(rows, cols, eb, row_major, pad, seed):
    """A (rows+2pad) x (cols+2pad) matrix of distinct-ish bytes; returns storage, ld, block offset."""
    R_, C_ = rows + 2 * pad, cols + 2 * pad
    dt = _np_dtype(eb)
    vals = (np.arange(R_ * C_, dtype=np.uint64) * 2654435761 + seed) % (1 << (8 * eb) - 1)
    if eb == 4:
        vals = vals % (1 << 22)  # keep f32 patterns finite
    if eb == 8:
        vals = vals % (1 << 52)
    mat = vals.astype(dt).reshape(R_, C_)
    ld = C_ if row_major else R_
    off = pad * ld + pad
    flat = mat.ravel() if row_major else np.ascontiguousarray(mat.T).ravel()
    return mat, flat, ld, off


@pytest.mark.parametrize("cid", CASES)
def test_load_store_round_trip_leaves_padding_untouched(cid):
    rows, cols, eb, rm, _ = _info(cid)
    # alignment: vector accesses need the block origin aligned to 16 bytes along the contiguous dim
    pad = 16 // eb
    mat, flat, ld, off = _padded(rows, cols, eb, rm, pad, cid)
    d_in = to_device(flat)
    d_out = device_filled(flat.size, flat.dtype, 0xEE)
    rc = api_lib().api_round_trip(cid, ctypes.c_void_p(d_in.data_ptr() + off * eb), ctypes.c_void_p(d_out.data_ptr() + off * eb), ld, ld)
    assert rc == 0
    out = to_host(d_out, flat.dtype)
    out2d = out.reshape(mat.shape) if rm else out.reshape(mat.shape[::-1]).T
    assert np.array_equal(out2d[pad:pad + rows, pad:pad + cols], mat[pad:pad + rows, pad:pad + cols])
    canary = np.frombuffer(bytes([0xEE] * eb), dtype=flat.dtype)[0]
    mask = np.ones(mat.shape, dtype=bool)
    mask[pad:pad + rows, pad:pad + cols] = False
    assert np.all(out2d[mask] == canary)


@pytest.mark.parametrize("cid", [0, 3, 8, 9, 10, 11, 12, 22, 30, 41, 52, 57, 66, 75, 78, 81, 83, 88])
def test_runtime_layout_overloads(cid):
    rows, cols, eb, rm, _ = _info(cid)
    mat, flat, ld, _ = _padded(rows, cols, eb, rm, 0, 77 + cid)
    d_in, d_out = to_device(flat), device_filled(flat.size, flat.dtype, 0xEE)
    assert api_lib().api_round_trip_runtime(cid, ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), ld) == 0
    assert np.array_equal(to_host(d_out, flat.dtype), flat)


# element type of each case, for the expected fill pattern (mirrors FRAG_CASES in api_kernels.hip)
def _case_types():
    import os, re
    src = open(os.path.join(os.path.dirname(__file__), "kernels", "api_kernels.hip")).read()
    return {int(m.group(1)): m.group(2) for m in re.finditer(r"X\((\d+), \w+, \d+, \d+, \d+, (\w+), \w+\)", src)}


CASE_TYPE = _case_types()


@pytest.mark.parametrize("cid", [0, 5, 6, 8, 11, 13, 15, 17, 20, 22, 25] + list(range(26, 90, 3)))
def test_fill_fragment(cid):
    rows, cols, eb, rm, ne = _info(cid)
    assert ne == rows * cols // 64
    ld = cols if rm else rows
    d_out = device_filled(rows * cols, _np_dtype(eb), 0xEE)
    assert api_lib().api_fill(cid, ctypes.c_void_p(d_out.data_ptr()), ld, ctypes.c_float(-3.0)) == 0
    out = to_host(d_out, _np_dtype(eb))
    t = CASE_TYPE[cid]
    want = {"int8_t": lambda: np.int8(-3).view(np.uint8),
            "int32_t": lambda: np.int32(-3).view(np.uint32),
            "float8_t": lambda: O.f32_to_storage(np.float32([-3.0]), O.E4M3)[0],
            "bfloat16_t": lambda: O.f32_to_storage(np.float32([-3.0]), O.BF16)[0],
            "float16_t": lambda: np.float16(-3.0).view(np.uint16),
            "float32_t": lambda: np.float32(-3.0).view(np.uint32)}[t]()
    assert np.all(out == want)


@pytest.mark.parametrize("cid", [4, 7, 10, 17, 18, 19, 20, 21, 25, 32, 36, 48, 51, 61, 64, 72, 73, 79, 80, 85, 89])
# (3, 1), (3, 2) and (3, 4): wave counts that are not powers of two -- the largest power of two below them shares
# the work and the surplus waves return (the reference idles its surplus waves too, coop_load.hpp:101-131)
@pytest.mark.parametrize("waves", [(1, 1), (2, 1), (2, 2), (4, 2), (3, 1), (3, 2), (3, 4)])
@pytest.mark.parametrize("use_lds", [0, 1])
def test_cooperative_round_trip(cid, waves, use_lds):
    rows, cols, eb, rm, _ = _info(cid)
    mat, flat, ld, _ = _padded(rows, cols, eb, rm, 0, 5 * cid + 1)
    d_in, d_out = to_device(flat), device_filled(flat.size, flat.dtype, 0xEE)
    rc = api_lib().api_coop_round_trip(cid, ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), ld, waves[0], waves[1], use_lds)
    assert rc == 0
    assert np.array_equal(to_host(d_out, flat.dtype), flat)


@pytest.mark.parametrize("cid", [17, 18])
def test_cooperative_static_wave_count(cid):
    rows, cols, eb, rm, _ = _info(cid)
    mat, flat, ld, _ = _padded(rows, cols, eb, rm, 0, 31)
    d_in, d_out = to_device(flat), device_filled(flat.size, flat.dtype, 0xEE)
    assert api_lib().api_coop_round_trip_static4(cid, ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), ld) == 0
    assert np.array_equal(to_host(d_out, flat.dtype), flat)


def test_transpose_and_data_layout_relabels():
    # matrix_b 16(k) x 64(n) row-major viewed as matrix_a 64 x 16 col-major: same memory image
    k, n = 16, 64
    src = (np.arange(k * n) % 1000).astype(np.uint16)
    d_in, d_out = to_device(src), device_filled(src.size, np.uint16, 0xEE)
    assert api_lib().api_transpose_store(ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), n) == 0
    assert np.array_equal(to_host(d_out, np.uint16), src)
    # matrix_a 32 x 16 loaded row-major, stored through the col-major relabel: memory holds the transpose
    m, kk = 32, 16
    a = (np.arange(m * kk) * 7 % 1000).astype(np.uint16).reshape(m, kk)
    d_in, d_out = to_device(a.ravel()), device_filled(a.size, np.uint16, 0xEE)
    assert api_lib().api_relayout_store(ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), kk, m) == 0
    assert np.array_equal(to_host(d_out, np.uint16).reshape(kk, m), a.T)


def test_mapping_util_coordinates():
    gx, gy, wx, wy, ld = 3, 2, 2, 4, 640
    waves = gx * gy * wx * wy
    d_out = device_filled(waves * 8, np.uint32, 0xEE)
    assert api_lib().api_mapping_probe(ctypes.c_void_p(d_out.data_ptr()), ld, gx, gy, wx, wy) == 0
    out = to_host(d_out, np.uint32).reshape(waves, 8)
    for by in range(gy):
        for bx in range(gx):
            for w0 in range(wx):
                for w1 in range(wy):
                    w = (by * gx + bx) * wx * wy + w0 * wy + w1
                    blk = (bx * wx + w0, by * wy + w1)
                    mat = (blk[0] * 32, blk[1] * 16)
                    assert tuple(out[w, :6]) == (w0, w1, blk[0], blk[1], mat[0], mat[1])
                    assert out[w, 6] == mat[0] * ld + mat[1] and out[w, 7] == out[w, 6]


# 8: bf16 accumulator fragments; 9, 10: __half (hfloat16_t) operands, the reference's h16 tuples
# (test/gemm/gemm_common_test_params.hpp:50-130) - same bits as float16_t, so the same oracle types
TYPES = {0: (O.F16, O.F32), 1: (O.BF16, O.F32), 2: (O.E4M3, O.F32), 3: (O.I8, O.I32), 4: (O.F32, O.F32), 5: (O.F16, O.F16),
         6: (O.F64, O.F64), 8: (O.BF16, O.BF16), 9: (O.F16, O.F32), 10: (O.F16, O.F16)}
SHAPES = {0: [(16, 16), (16, 32), (32, 8), (32, 16)], 1: [(16, 16), (16, 32), (32, 8), (32, 16)],
          2: [(16, 32), (16, 64), (32, 16), (32, 32)], 3: [(16, 32), (16, 64), (32, 16), (32, 32)],
          4: [(16, 4), (16, 16), (32, 2), (32, 8)], 5: [(16, 16), (32, 16)], 6: [(16, 4), (16, 8), (16, 16), (16, 32)],
          8: [(16, 16), (16, 32), (32, 8), (32, 16)], 9: [(16, 16), (16, 32), (32, 8), (32, 16)], 10: [(16, 16), (32, 16)]}


@pytest.mark.parametrize("a_row,b_row,c_row", [(1, 0, 1), (0, 1, 0), (1, 1, 1), (0, 0, 0)])
def test_mma_sync_e5m2_single_tile(a_row, b_row, c_row):
    """bfloat8_t (OCP e5m2) fragments: an e5m2 code is the high byte of the f16 with the same value, so the
    operands decode exactly through numpy's float16 and the oracle runs its f32 GEMM on the decoded values
    (the reference lists the type in its test tuples, test/gemm/gemm_common_test_params.hpp:73-87, but has no
    matrix instruction for it on any gfx9, mfma_impl.hpp:1113-1170: parity is pinned by the decode alone)."""
    rng = np.random.default_rng(7)
    for blk, bk in [(16, 32), (16, 64), (32, 16), (32, 32)]:
        m = n = blk
        # finite codes only (exponent field 31 is inf / NaN): sign | exponent 0..30 | 2 mantissa bits
        a = (rng.integers(0, 0x7C, m * bk) | (rng.integers(0, 2, m * bk) << 7)).astype(np.uint8)
        b = (rng.integers(0, 0x7C, bk * n) | (rng.integers(0, 2, bk * n) << 7)).astype(np.uint8)
        a = np.where((a & 0x7F) > 0x47, a & 0xC7 | 0x40, a).astype(np.uint8)  # keep |x| <= 7 so that sums stay small
        b = np.where((b & 0x7F) > 0x47, b & 0xC7 | 0x40, b).astype(np.uint8)
        dec = lambda x: (x.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
        c = O.uniform_pm1(3, m * n)
        la, lb, lc = (O.ROW if a_row else O.COL), (O.ROW if b_row else O.COL), (O.ROW if c_row else O.COL)
        want = O.gemm(O.F32, O.F32, la, lb, lc, lc, m, n, bk, dec(a), dec(b), c, 1.0, 1.0)
        da, db, dc = to_device(a), to_device(b), to_device(c)
        dd = device_filled(m * n, np.float32, 0xFF)
        rc = api_lib().api_mma_tile(7, blk, bk, a_row, b_row, c_row, ctypes.c_void_p(da.data_ptr()),
                                    ctypes.c_void_p(db.data_ptr()), ctypes.c_void_p(dc.data_ptr()),
                                    ctypes.c_void_p(dd.data_ptr()), bk if a_row else m, n if b_row else bk, n if c_row else m)
        assert rc == 0, (blk, bk)
        g, w = to_host(dd, np.float32).astype(np.float64), want.astype(np.float64)
        assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= 1e-2, (blk, bk)


@pytest.mark.parametrize("type_id", sorted(TYPES))
@pytest.mark.parametrize("a_row,b_row,c_row", [(1, 0, 1), (0, 1, 0), (1, 1, 1), (0, 0, 0)])
def test_mma_sync_single_tile_matches_oracle(type_id, a_row, b_row, c_row):
    in_t, out_t = TYPES[type_id]
    for blk, bk in SHAPES[type_id]:
        m = n = blk
        if in_t == O.I8:
            a, b = O.uniform_int8(1, m * bk), O.uniform_int8(2, bk * n)
            c = (O.uniform_int8(3, m * n).astype(np.int32) * 100)
        else:
            src = O.normal if in_t == O.E4M3 else O.uniform_pm1
            a = O.f32_to_storage(src(1, m * bk), in_t)
            b = O.f32_to_storage(src(2, bk * n), in_t)
            c = O.f32_to_storage(O.uniform_pm1(3, m * n), out_t)
        la, lb, lc = (O.ROW if a_row else O.COL), (O.ROW if b_row else O.COL), (O.ROW if c_row else O.COL)
        want = O.gemm(in_t, out_t, la, lb, lc, lc, m, n, bk, a, b, c, 1.0, 1.0)
        da, db, dc = to_device(a), to_device(b), to_device(c)
        dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
        lda = bk if a_row else m
        ldb = n if b_row else bk
        rc = api_lib().api_mma_tile(type_id, blk, bk, a_row, b_row, c_row, ctypes.c_void_p(da.data_ptr()),
                                    ctypes.c_void_p(db.data_ptr()), ctypes.c_void_p(dc.data_ptr()),
                                    ctypes.c_void_p(dd.data_ptr()), lda, ldb, n if c_row else m)
        assert rc == 0, (blk, bk)
        got = to_host(dd, O.NP_STORAGE[out_t])
        if in_t == O.I8:
            assert np.array_equal(got, want), (blk, bk)
        else:
            # same products, different summation order than the sequential oracle: 10 eps of the
            # output type on the reference's metric (100 eps for the 16-bit accumulate type).
            # The fp8 matrix core does not keep full f32 precision inside one instruction
            # (observed 1e-4): it gets the stated fp8 bar of 1e-2.
            if in_t == O.E4M3:
                g, w = got.astype(np.float64), want.astype(np.float64)
                assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= 1e-2, (blk, bk)
            else:
                ok, mx = O.compare(out_t, got, want, 100.0 if out_t in (O.F16, O.BF16) else 10.0)
                assert ok, (blk, bk, mx)


# ------------------------------------------------------------------ 2:4 sparse fragments (rocwmma_sparse.hpp)
SPARSE_TYPES = {0: (O.F16, 2), 1: (O.BF16, 2), 2: (O.E4M3, 1), 3: (O.I8, 1), 7: (O.E5M2, 1)}


def _sparse_tile(type_id, blk, stages, b_row, c_row, dense, b, c):
    """dense: (blk, k) storage array with a 2:4 pattern; returns D = A B + C of one tile through the sparse fragment API."""
    import rocwmma_amd as R

    vals, meta = R.compress_24(dense)
    assert np.array_equal(R.decompress_24(vals, meta), dense)
    k = dense.shape[1]
    acc_dt = np.int32 if type_id == 3 else np.float32
    dv, dm, db, dc = to_device(vals), to_device(meta), to_device(b), to_device(c)
    dd = device_filled(blk * blk, acc_dt, 0xFF)
    rc = api_lib().api_sparse_mma_tile(type_id, blk, stages, b_row, c_row, ctypes.c_void_p(dv.data_ptr()), ctypes.c_void_p(dm.data_ptr()),
                                       ctypes.c_void_p(db.data_ptr()), ctypes.c_void_p(dc.data_ptr()), ctypes.c_void_p(dd.data_ptr()),
                                       blk if b_row else k, blk)
    assert rc == 0, (type_id, blk, stages)
    return to_host(dd, acc_dt)


@pytest.mark.parametrize("type_id", sorted(SPARSE_TYPES))
@pytest.mark.parametrize("blk,stages", [(16, 1), (16, 2), (32, 1), (32, 2)])
@pytest.mark.parametrize("b_row,c_row", [(0, 1), (1, 0)])
def test_sparse_mma_sync_single_tile_matches_dense_oracle(type_id, blk, stages, b_row, c_row):
    """Random 2:4 operands: the sparse tile equals the oracle's dense GEMM on the decompressed A (int8 bit-exact, fp8
    1e-2, 16-bit 1e-3 on the reference's metric: same products, another summation order)."""
    in_t, es = SPARSE_TYPES[type_id]
    k = stages * 128 // es
    m = n = blk
    mask = O.sparse24_mask(20 + type_id, m, k)
    if in_t == O.I8:
        a, b = O.uniform_int8(21, m * k).reshape(m, k), O.uniform_int8(22, k * n)
        c = O.uniform_int8(23, m * n).astype(np.int32) * 100
        dense = np.where(mask, a, np.int8(0)).astype(np.int8)
        dec = lambda x: x
        o_in, o_out = O.I8, O.I32
    else:
        if in_t == O.E5M2:  # finite codes with |x| <= 7; decoded exactly through float16
            rng = np.random.default_rng(5)
            mk = lambda nel: np.where((rng.integers(0, 0x48, nel) == 0), 1, rng.integers(0, 0x48, nel) | (rng.integers(0, 2, nel) << 7)).astype(np.uint8)
            a, b = mk(m * k).reshape(m, k), mk(k * n)
            dec = lambda x: (x.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
            o_in = O.F32
        else:
            src = O.normal if in_t == O.E4M3 else O.uniform_pm1
            a = O.f32_to_storage(src(21, m * k), in_t).reshape(m, k)
            b = O.f32_to_storage(src(22, k * n), in_t)
            dec = lambda x: x
            o_in = in_t
        c = O.uniform_pm1(23, m * n)
        dense = np.where(mask, a, a.dtype.type(0)).astype(a.dtype)
        o_out = O.F32
    lb, lc = (O.ROW if b_row else O.COL), (O.ROW if c_row else O.COL)
    want = O.gemm(o_in, o_out, O.ROW, lb, lc, lc, m, n, k, dec(dense).ravel(), dec(b), c, 1.0, 1.0)
    got = _sparse_tile(type_id, blk, stages, b_row, c_row, dense, b, c)
    if in_t == O.I8:
        assert np.array_equal(got, want)
    else:
        g, w = got.astype(np.float64), want.astype(np.float64)
        tol = 1e-2 if es == 1 else 1e-3
        assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= tol


@pytest.mark.parametrize("type_id,blk", [(3, 16), (3, 32), (0, 16), (0, 32)])
def test_sparse_mma_sync_one_hot_sweep(type_id, blk):
    """Every dense position of A in turn holds the only non-zero (row r has it at column (kk + r) % k): D must be the
    matching rows of B - exact, and wrong for any other pairing of lane groups, index bits or storage offsets."""
    in_t, es = SPARSE_TYPES[type_id]
    stages = 2
    k, m, n = stages * 128 // es, blk, blk
    if in_t == O.I8:
        b = ((np.arange(k * n) * 7 + 3) % 251 - 125).astype(np.int8)
        bf = b.astype(np.int32).reshape(n, k)  # col-major B: bf[col, kk]
        one, zero_c = np.int8(1), np.zeros(m * n, dtype=np.int32)
    else:
        b = O.f32_to_storage(((np.arange(k * n) % 2039) - 1000).astype(np.float32), O.F16)
        bf = b.view(np.float16).astype(np.float32).reshape(n, k)
        one, zero_c = np.float16(1.0).view(np.uint16), np.zeros(m * n, dtype=np.float32)
    for kk in range(k):
        dense = np.zeros((m, k), dtype=np.int8 if in_t == O.I8 else np.uint16)
        cols = (kk + np.arange(m)) % k
        dense[np.arange(m), cols] = one
        got = _sparse_tile(type_id, blk, stages, 0, 1, dense, b, zero_c).reshape(m, n)
        assert np.array_equal(got, bf[:, cols].T), kk
