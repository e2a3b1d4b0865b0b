"""GPU parity of the 2:4 structured-sparse GEMM (v_smfmac) against the oracle's dense GEMM on the
decompressed A.  The reference has no sparse path: parity is pinned by the oracle plus the format
invariants checked in test_oracle.py / test_cabi.py."""
import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from test_gemm import _embed
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

MACRO_TILES = (R.KERNEL_TILED, R.KERNEL_TILED_128)  # 256 x 256 and 128 x 128


def _close(got, want, in_t):
    """The bar of the element type: bit-exact for int8, 1e-2 (e4m3) / 1e-3 (16-bit) on the relative metric."""
    if in_t == O.I8:
        return np.array_equal(got, want)
    g, w = got.astype(np.float64), want.astype(np.float64)
    return bool(np.all(np.isfinite(g))) and np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= (1e-2 if in_t == O.E4M3 else 1e-3)


def _auto_kernels(m, n):
    """What AUTO may pick: a macro tile (which of the two depends on how many CUs the large tiles would fill) from
    128 x 128 on, the block-per-wave kernel below that."""
    return MACRO_TILES if (m >= 128 and n >= 128) else (R.KERNEL_SIMPLE,)


def _sparse_inputs(in_t, m, n, k, seed):
    mask = O.sparse24_mask(seed, m, k)
    if in_t == O.I8:
        vals = O.uniform_int8(seed + 1, m * k).reshape(m, k)
        b = O.uniform_int8(seed + 2, k * n)
    else:
        vals = O.f32_to_storage(O.normal(seed + 1, m * k), O.E4M3).view(np.int8).reshape(m, k)
        b = O.f32_to_storage(O.normal(seed + 2, k * n), O.E4M3)
    dense = np.where(mask, vals, np.int8(0)).astype(np.int8)
    return dense, b


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32)])
@pytest.mark.parametrize("m,n,k", [(32, 32, 128), (16, 48, 128), (96, 64, 256), (256, 128, 1024), (256, 256, 128), (256, 256, 640),
                                   (512, 768, 384), (256, 512, 896), (272, 400, 256), (144, 368, 384), (528, 128, 128)])
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_sparse_gemm_vs_dense_oracle(in_t, out_t, m, n, k, ldl):
    dense, b = _sparse_inputs(in_t, m, n, k, 40)
    vals, meta = R.compress_24(dense)
    assert np.array_equal(R.decompress_24(vals, meta), dense)
    storage = dense.view(np.uint8) if in_t == O.E4M3 else dense
    c = (O.uniform_int8(50, m * n).astype(np.int32) * 11) if in_t == O.I8 else O.uniform_pm1(50, m * n)
    want = O.gemm(in_t, out_t, O.ROW, O.COL, ldl, ldl, m, n, k, storage.ravel(), b, c, 1.0, 1.0)
    dv, dm, db, dc = to_device(vals), to_device(meta), to_device(b), to_device(c)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    R.gemm(in_t, out_t, m, n, k, dv, db, dc, dd, 1.0, 1.0, O.ROW, O.COL, ldl, ldl, a_meta=dm)
    got = to_host(dd, O.NP_STORAGE[out_t])
    plan = R.gemm_query(R.gemm_args(in_t, out_t, m, n, k, dv, db, dc, dd, 1.0, 1.0, O.ROW, O.COL, ldl, ldl, a_meta=dm))
    # the macro tiles take every K that fills whole 128-wide stages (1 .. 8 stages above: every remainder of the
    # six-stage loop trip) and, from 128 x 128 on, any m and n (edge tiles)
    assert plan.kernel in _auto_kernels(m, n)
    assert _close(got, want, in_t)
    for tile in MACRO_TILES:  # each tile size forced (any m, n)
        dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
        R.gemm(in_t, out_t, m, n, k, dv, db, dc, dd, 1.0, 1.0, O.ROW, O.COL, ldl, ldl, a_meta=dm, kernel=tile)
        assert _close(to_host(dd, O.NP_STORAGE[out_t]), want, in_t), tile


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32)])
def test_sparse_config4_sampled_rows(in_t, out_t):
    # benchmark configuration 4: M = N = 4096, dense-equivalent K = 8192, int8 and fp8 e4m3
    m, n, k = 4096, 4096, 8192
    dense, b = _sparse_inputs(in_t, m, n, k, 60)
    vals, meta = R.compress_24(dense)
    dv, dm, db = to_device(vals), to_device(meta), to_device(b)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    R.gemm(in_t, out_t, m, n, k, dv, db, None, dd, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, a_meta=dm)
    got = to_host(dd, O.NP_STORAGE[out_t]).reshape(m, n)
    # the same problem with B stored row-major (k x n, n contiguous): the same products in the same order
    dbt = to_device(np.ascontiguousarray(b.reshape(n, k).T))
    ddt = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    R.gemm(in_t, out_t, m, n, k, dv, dbt, None, ddt, 1.0, 0.0, O.ROW, O.ROW, O.ROW, O.ROW, a_meta=dm)
    assert np.array_equal(to_host(ddt, O.NP_STORAGE[out_t]).reshape(m, n).view(np.uint8), got.view(np.uint8))
    # ... and on the other macro tile (AUTO takes the 256 x 256 one here): every element of D sums the same stages in order
    assert R.gemm_query(R.gemm_args(in_t, out_t, m, n, k, dv, db, None, dd, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, a_meta=dm)).kernel == R.KERNEL_TILED
    for bb, lb in ((db, O.COL), (dbt, O.ROW)):
        R.gemm(in_t, out_t, m, n, k, dv, bb, None, ddt, 1.0, 0.0, O.ROW, lb, O.ROW, O.ROW, a_meta=dm, kernel=R.KERNEL_TILED_128)
        assert np.array_equal(to_host(ddt, O.NP_STORAGE[out_t]).reshape(m, n).view(np.uint8), got.view(np.uint8))
    rows = np.array([0, 31, 32, 2047, 4095, 1234], dtype=np.uint32)
    storage = dense.view(np.uint8) if in_t == O.E4M3 else dense
    want = O.gemm_rows(in_t, out_t, O.ROW, O.COL, m, n, k, storage.ravel(), b, rows)
    if in_t == O.I8:
        assert np.array_equal(got[rows], want)
        B = b.reshape(n, k).astype(np.int64)
        assert int(got.astype(np.int64).sum()) == int(dense.astype(np.int64).sum(axis=0) @ B.sum(axis=0))
    else:
        g, w = got[rows].astype(np.float64), want.astype(np.float64)
        assert np.all(np.isfinite(got))
        assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= 1e-2
        # column sums of D against (column sums of A) . B in float64: every element of D takes part
        A64 = O.storage_to_f32(storage, O.E4M3).astype(np.float64).reshape(m, k)
        B64 = O.storage_to_f32(b, O.E4M3).astype(np.float64).reshape(n, k)
        ref = A64.sum(axis=0) @ B64.T
        scale = np.abs(A64).sum(axis=0) @ np.abs(B64).T
        assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - ref) / scale) <= 1e-3


@pytest.mark.parametrize("in_t", [O.F16, O.BF16])
@pytest.mark.parametrize("m,n,k", [(32, 32, 64), (16, 48, 64), (96, 64, 192), (256, 128, 1024), (64, 32, 4096), (256, 256, 448),
                                   (272, 144, 320), (512, 256, 64)])
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_sparse_gemm_16bit_vs_dense_oracle(in_t, m, n, k, ldl):
    """f16 / bf16 operands on v_smfmac_f32_32x32x32 / 16x16x64_{f16,bf16} (block-per-wave kernel on the sparse fragment
    API, and the macro-tile kernel from 128 x 128 on), f32 out.  Same products as the
    oracle's dense GEMM on the decompressed A, summed in another order: the 16-bit bar of 1e-3 on the relative metric."""
    mask = O.sparse24_mask(70, m, k)
    a = O.f32_to_storage(O.uniform_pm1(71, m * k), in_t).reshape(m, k)
    dense = np.where(mask, a, np.uint16(0)).astype(np.uint16)
    b = O.f32_to_storage(O.uniform_pm1(72, k * n), in_t)
    vals, meta = R.compress_24(dense)
    assert vals.dtype == np.uint16 and np.array_equal(R.decompress_24(vals, meta), dense)
    c = O.uniform_pm1(73, m * n)
    want = O.gemm(in_t, O.F32, O.ROW, O.COL, ldl, ldl, m, n, k, dense.ravel(), b, c, 2.0, 2.0)
    dv, dm, db, dc = to_device(vals), to_device(meta), to_device(b), to_device(c)
    dd = device_filled(m * n, np.float32, 0xFF)
    R.gemm(in_t, O.F32, m, n, k, dv, db, dc, dd, 2.0, 2.0, O.ROW, O.COL, ldl, ldl, a_meta=dm)
    got = to_host(dd, np.float32)
    plan = R.gemm_query(R.gemm_args(in_t, O.F32, m, n, k, dv, db, dc, dd, 2.0, 2.0, O.ROW, O.COL, ldl, ldl, a_meta=dm))
    assert plan.kernel in _auto_kernels(m, n) and plan.macro_tile_k == 64
    assert _close(got, want, in_t)
    for tile in MACRO_TILES:
        dd = device_filled(m * n, np.float32, 0xFF)
        R.gemm(in_t, O.F32, m, n, k, dv, db, dc, dd, 2.0, 2.0, O.ROW, O.COL, ldl, ldl, a_meta=dm, kernel=tile)
        assert _close(to_host(dd, np.float32), want, in_t), tile


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32), (O.F16, O.F32), (O.BF16, O.F32)])
@pytest.mark.parametrize("m,n,k", [(32, 32, 128), (16, 48, 256), (272, 144, 384), (256, 256, 128), (512, 384, 896), (144, 400, 640)])
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_sparse_gemm_row_major_b(in_t, out_t, m, n, k, ldl):
    """B (k x n) with n contiguous: both kernels take either orientation of B (the macro tile stages k-rows of B and
    reads them back with transposing LDS reads), against the oracle's dense GEMM with the same orientation.  Sizes: below a
    tile, edge tiles in m and n, one to seven stages (every remainder of the six-stage loop trip)."""
    mask = O.sparse24_mask(80, m, k)
    if in_t == O.I8:
        dense = np.where(mask, O.uniform_int8(81, m * k).reshape(m, k), np.int8(0)).astype(np.int8)
        b = O.uniform_int8(82, k * n)
        storage = dense
    elif in_t == O.E4M3:
        dense = np.where(mask, O.f32_to_storage(O.normal(81, m * k), O.E4M3).view(np.int8).reshape(m, k), np.int8(0)).astype(np.int8)
        b = O.f32_to_storage(O.normal(82, k * n), O.E4M3)
        storage = dense.view(np.uint8)
    else:
        dense = np.where(mask, O.f32_to_storage(O.uniform_pm1(81, m * k), in_t).reshape(m, k), np.uint16(0)).astype(np.uint16)
        b = O.f32_to_storage(O.uniform_pm1(82, k * n), in_t)
        storage = dense
    vals, meta = R.compress_24(dense)
    c = (O.uniform_int8(83, m * n).astype(np.int32) * 7) if in_t == O.I8 else O.uniform_pm1(83, m * n)
    want = O.gemm(in_t, out_t, O.ROW, O.ROW, ldl, ldl, m, n, k, storage.ravel(), b, c, 1.0, 1.0)
    dv, dm, db, dc = to_device(vals), to_device(meta), to_device(b), to_device(c)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    args = R.gemm_args(in_t, out_t, m, n, k, dv, db, dc, dd, 1.0, 1.0, O.ROW, O.ROW, ldl, ldl, a_meta=dm)
    assert R.gemm_query(args).kernel in _auto_kernels(m, n)
    R.gemm(in_t, out_t, m, n, k, dv, db, dc, dd, 1.0, 1.0, O.ROW, O.ROW, ldl, ldl, a_meta=dm)
    assert _close(to_host(dd, O.NP_STORAGE[out_t]), want, in_t)
    # the macro tiles forced (any m, n: rows and columns beyond the matrix are clamped or load as zeros)
    for tile in MACRO_TILES:
        dd2 = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
        R.gemm(in_t, out_t, m, n, k, dv, db, dc, dd2, 1.0, 1.0, O.ROW, O.ROW, ldl, ldl, a_meta=dm, kernel=tile)
        assert _close(to_host(dd2, O.NP_STORAGE[out_t]), want, in_t), tile


@pytest.mark.parametrize("case", range(40))
def test_sparse_random_sweep(case):
    """Seeded random draw of element type, sizes (both kernels, edge tiles, every stage-count remainder), orientation of B
    and of C / D, scalars and kernel selector, against the oracle's dense GEMM on the decompressed A."""
    rng = np.random.default_rng(5000 + case)
    in_t, out_t = [(O.I8, O.I32), (O.E4M3, O.F32), (O.F16, O.F32), (O.BF16, O.F32)][case % 4]
    es = 2 if in_t in (O.F16, O.BF16) else 1
    big = bool(rng.integers(0, 2))
    m = 16 * int(rng.integers(8, 40) if big else rng.integers(1, 12))
    n = 16 * int(rng.integers(8, 40) if big else rng.integers(1, 12))
    k = (128 // es) * int(rng.integers(1, 14))
    lb = [O.COL, O.COL, O.ROW][int(rng.integers(0, 3))]
    ldl = [O.ROW, O.COL][int(rng.integers(0, 2))]
    alpha, beta = (float(rng.integers(-2, 3)), float(rng.integers(-1, 2))) if in_t == O.I8 else (float(rng.choice([1.0, 2.0, -0.5])), float(rng.choice([0.0, 1.0])))
    mask = O.sparse24_mask(case + 1, m, k)
    if in_t == O.I8:
        dense = np.where(mask, O.uniform_int8(case + 2, m * k).reshape(m, k), np.int8(0)).astype(np.int8)
        b, storage = O.uniform_int8(case + 3, k * n), dense
        c = O.uniform_int8(case + 4, m * n).astype(np.int32) * 5
    elif in_t == O.E4M3:
        dense = np.where(mask, O.f32_to_storage(O.normal(case + 2, m * k), O.E4M3).view(np.int8).reshape(m, k), np.int8(0)).astype(np.int8)
        b, storage = O.f32_to_storage(O.normal(case + 3, k * n), O.E4M3), dense.view(np.uint8)
        c = O.uniform_pm1(case + 4, m * n)
    else:
        dense = np.where(mask, O.f32_to_storage(O.uniform_pm1(case + 2, m * k), in_t).reshape(m, k), np.uint16(0)).astype(np.uint16)
        b, storage = O.f32_to_storage(O.uniform_pm1(case + 3, k * n), in_t), dense
        c = O.uniform_pm1(case + 4, m * n)
    vals, meta = R.compress_24(dense)
    assert np.array_equal(R.decompress_24(vals, meta), dense)
    want = O.gemm(in_t, out_t, O.ROW, lb, ldl, ldl, m, n, k, storage.ravel(), b, c, alpha, beta)
    dv, dm, db, dc = to_device(vals), to_device(meta), to_device(b), to_device(c)
    dd = device_filled(m * n + 4, O.NP_STORAGE[out_t], 0xEE)
    kernel = [R.KERNEL_AUTO, R.KERNEL_TILED, R.KERNEL_SIMPLE, R.KERNEL_TILED_128][int(rng.integers(0, 4))]
    # padded leading dimensions of B, C and D (drawn last, so the cases above keep their other draws)
    pad_b = (16 // es) * int(rng.integers(0, 3))
    pad_c, pad_d = 4 * int(rng.integers(0, 3)), 4 * int(rng.integers(0, 3))
    ldb = (n if lb == O.ROW else k) + pad_b
    ldc, ldd = (n if ldl == O.ROW else m) + pad_c, (n if ldl == O.ROW else m) + pad_d
    major, minor = (m, n) if ldl == O.ROW else (n, m)
    canary = np.array([0xEE] * 4, dtype=np.uint8).view(c.dtype)[0]
    db, dc = to_device(_embed(b, k, n, lb, ldb, 1)), to_device(_embed(c, m, n, ldl, ldc, canary))
    dd = device_filled(major * ldd + 4, O.NP_STORAGE[out_t], 0xEE)
    R.gemm(in_t, out_t, m, n, k, dv, db, dc if beta != 0.0 else None, dd, alpha, beta, O.ROW, lb, ldl, ldl, a_meta=dm, kernel=kernel,
           ldb=ldb, ldc=ldc, ldd=ldd)
    full = to_host(dd, O.NP_STORAGE[out_t])
    assert np.all(full[major * ldd:].view(np.uint8) == 0xEE)
    rows = full[:major * ldd].reshape(major, ldd)
    assert np.all(rows[:, minor:].view(np.uint8) == 0xEE), "bytes outside D were written"
    got = np.ascontiguousarray(rows[:, :minor]).ravel()
    assert _close(got, want, in_t), (m, n, k, lb, ldl, kernel)


def test_sparse_16bit_one_hot_positions():
    """Every (row, kept position) of A in turn is the only non-zero: D must be that row of B scaled - exact, and it
    fails for any wrong pairing of lane groups or index bits."""
    m, n, k = 32, 32, 128
    b = O.f32_to_storage(((np.arange(k * n) % 2039) - 1000).astype(np.float32), O.F16)  # distinct small integers
    bf = b.view(np.float16).astype(np.float32).reshape(n, k)  # col-major B: bf[col, kk]
    db = to_device(b)
    for kk in range(k):
        dense = np.zeros((m, k), dtype=np.uint16)
        cols = (kk + np.arange(m)) % k  # row r has its 1 at column (kk + r) % k
        dense[np.arange(m), cols] = np.float16(1.0).view(np.uint16)
        vals, meta = R.compress_24(dense)
        dv, dm = to_device(vals), to_device(meta)
        dd = device_filled(m * n, np.float32, 0xFF)
        R.gemm(O.F16, O.F32, m, n, k, dv, db, None, dd, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, a_meta=dm)
        got = to_host(dd, np.float32).reshape(m, n)
        assert np.array_equal(got, bf[:, cols].T), kk


def test_sparse_size_and_selector_errors():
    """Sizes off the storage grid and selectors without a kernel come back as errors, not as silent fallbacks."""
    g = lambda m, n, k, kernel=R.KERNEL_AUTO, lda=None: R.gemm_args(R.I8, R.I32, m, n, k, 0x1000, 0x2000, None, 0x3000, 1.0, 0.0,
                                                                  R.ROW_MAJOR, R.COL_MAJOR, R.ROW_MAJOR, R.ROW_MAJOR, a_meta=0x4000,
                                                                  kernel=kernel, lda=lda)
    for args, code in ((g(256, 256, 192), -3), (g(24, 256, 128), -3), (g(256, 256, 256, R.KERNEL_TILED_128_SPLITK), -2),
                       (g(256, 256, 256, lda=136), -1)):
        with pytest.raises(R.R355Error) as e:
            R.gemm_query(args)
        assert e.value.code == code
    assert R.gemm_query(g(256, 256, 128, R.KERNEL_TILED)).macro_tile_k == 128  # k % 128, as the header says
    assert R.gemm_query(g(48, 64, 128, R.KERNEL_TILED)).kernel == R.KERNEL_TILED  # forced: any m, n multiple of 16
    assert R.gemm_query(g(48, 64, 128)).kernel == R.KERNEL_SIMPLE
    small = R.gemm_query(g(48, 64, 128, R.KERNEL_TILED_128))
    assert (small.kernel, small.macro_tile_m, small.macro_tile_n, small.lds_bytes) == (R.KERNEL_TILED_128, 128, 128, 3 * 26 * 1024)
    large = R.gemm_query(g(48, 64, 128, R.KERNEL_TILED))
    assert (large.macro_tile_m, large.macro_tile_n, large.lds_bytes) == (256, 256, 3 * 52 * 1024)
    # AUTO: the small tile where the large tiles would leave most CUs idle, the large one where they fill the chip
    assert R.gemm_query(g(1024, 1024, 8192)).kernel == R.KERNEL_TILED_128
    assert R.gemm_query(g(4096, 4096, 8192)).kernel == R.KERNEL_TILED


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.F16, O.F32)])
def test_sparse_macro_tile_forced_on_small_and_ragged_shapes(in_t, out_t):
    """Both macro tiles on shapes far below a tile and off the tile grid: rows of A and B beyond the matrix load as zeros
    and nothing outside D is written (the output sits between two guard regions)."""
    for m, n, k, tile in [(m, n, k, t) for (m, n, k) in ((16, 16, 256), (48, 272, 128), (304, 80, 384), (144, 208, 896)) for t in MACRO_TILES]:
        es = 1 if in_t == O.I8 else 2
        k = k // es
        mask = O.sparse24_mask(80, m, k)
        if in_t == O.I8:
            a, b = O.uniform_int8(81, m * k).reshape(m, k), O.uniform_int8(82, k * n)
            dense = np.where(mask, a, np.int8(0)).astype(np.int8)
        else:
            a = O.f32_to_storage(O.uniform_pm1(81, m * k), in_t).reshape(m, k)
            b = O.f32_to_storage(O.uniform_pm1(82, k * n), in_t)
            dense = np.where(mask, a, np.uint16(0)).astype(np.uint16)
        vals, meta = R.compress_24(dense)
        want = O.gemm(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, dense.ravel(), b, None, 1.0, 0.0)
        dv, dm, db = to_device(vals), to_device(meta), to_device(b)
        guard = 4096
        dd = device_filled(m * n + 2 * guard, O.NP_STORAGE[out_t], 0xEE)
        # (device_filled hands back a byte tensor: the slice offset is in bytes)
        R.gemm(in_t, out_t, m, n, k, dv, db, None, dd[guard * 4:], 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, a_meta=dm, kernel=tile)
        full = to_host(dd, O.NP_STORAGE[out_t])
        assert np.all(full[:guard].view(np.uint32) == np.uint32(0xEEEEEEEE)) and np.all(full[guard + m * n:].view(np.uint32) == np.uint32(0xEEEEEEEE))
        assert _close(full[guard:guard + m * n], want, in_t), (m, n, k, tile)


@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_sparse_output_beyond_2_to_the_32_elements(ldl):
    # D (int32, 17 GB) has 65792 x 65536 elements: offsets into it pass 32 bits.  Lines of D on both sides of the boundary
    # against the dense oracle on the decompressed A.
    import torch

    m, n, k = (65536 + 256, 65536, 128) if ldl == O.ROW else (65536, 65536 + 256, 128)
    dense, b = _sparse_inputs(O.I8, m, n, k, 70)
    vals, meta = R.compress_24(dense)
    dv, dm, db = to_device(vals), to_device(meta), to_device(b)
    dd = device_filled(m * n, np.int32, 0xFF)
    R.gemm(O.I8, O.I32, m, n, k, dv, db, None, dd, 1.0, 0.0, O.ROW, O.COL, ldl, ldl, a_meta=dm, kernel=R.KERNEL_TILED)
    torch.cuda.synchronize()
    if ldl == O.ROW:
        lines = np.array([0, 1, 65535, 65536, 65537, m - 1], dtype=np.uint32)
        want = O.gemm_rows(O.I8, O.I32, O.ROW, O.COL, m, n, k, dense.ravel(), b, lines)
        length = n
    else:
        # columns of a col-major D are rows of D^T = B^T A^T (B col-major k x n is B^T row-major n x k)
        lines = np.array([0, 1, 65535, 65536, 65537, n - 1], dtype=np.uint32)
        want = O.gemm_rows(O.I8, O.I32, O.ROW, O.COL, n, m, k, b, dense.ravel(), lines)
        length = m
    for i, line in enumerate(lines):
        got = dd[int(line) * length * 4:(int(line) + 1) * length * 4].cpu().numpy().view(np.int32)
        assert np.array_equal(got, want[i]), line
    del dv, dm, db, dd
    torch.cuda.empty_cache()
