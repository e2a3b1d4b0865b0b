"""The reference's own sample kernels (samples/simple_hgemm.cpp, perf_hgemm.cpp, simple_dlrm.cpp,
simple_sgemv.cpp), compiled UNCHANGED against this library's headers by tests/kernels/build_ref_samples.py
where the reference tree is available, must produce the oracle's results on MI355X: run-time evidence for
"drop-in for the samples".  The shared objects are build outputs (tests/kernels/_ref/); when they are absent
the tests skip."""
import ctypes
import os

import numpy as np
import pytest

import oraclelib as O
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

_REF = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernels", "_ref")


def _lib(name):
    path = os.path.join(_REF, "libref_%s.so" % name)
    if not os.path.exists(path):
        pytest.skip("%s not built (needs the reference tree at build time)" % os.path.basename(path))
    return ctypes.CDLL(path)


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (256, 128, 192)])
def test_simple_hgemm_sample_kernel(m, n, k):
    # samples/simple_hgemm.cpp:66-79: A row-major, B col-major, C / D row-major f16, f32 accumulate
    L = _lib("simple_hgemm")
    a = O.f32_to_storage(O.uniform_pm1(1, m * k), O.F16)
    b = O.f32_to_storage(O.uniform_pm1(2, k * n), O.F16)
    c = O.f32_to_storage(O.uniform_pm1(3, m * n), O.F16)
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, np.uint16, 0xFF)
    rc = L.ref_simple_hgemm(m, n, k, _p(da), _p(db), _p(dc), _p(dd), k, k, n, n, ctypes.c_float(2.0), ctypes.c_float(2.0))
    assert rc == 0
    want = O.gemm(O.F16, O.F16, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    # the sample accumulates in f32 and rounds once: the reference's 10 eps(f16) bar plus one rounding
    ok, mx = O.compare(O.F16, to_host(dd, np.uint16), want, 10.0)
    assert ok, mx


@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (256, 384, 512)])
def test_perf_hgemm_sample_kernel(m, n, k):
    # samples/perf_hgemm.cpp:264-271: A col-major, B row-major, C / D row-major f16; cooperative loads,
    # LDS staging through applyDataLayout / applyTranspose, 2 x 2 blocks of 32 x 32 per wave
    L = _lib("perf_hgemm")
    a = O.f32_to_storage(O.uniform_pm1(4, m * k), O.F16)
    b = O.f32_to_storage(O.uniform_pm1(5, k * n), O.F16)
    c = O.f32_to_storage(O.uniform_pm1(6, m * n), O.F16)
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, np.uint16, 0xFF)
    rc = L.ref_perf_hgemm(m, n, k, _p(da), _p(db), _p(dc), _p(dd), m, n, n, n, ctypes.c_float(2.0), ctypes.c_float(2.0))
    assert rc == 0
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    ok, mx = O.compare(O.F16, to_host(dd, np.uint16), want, 10.0)
    assert ok, mx


def test_simple_dlrm_sample_forward_kernel():
    # samples/simple_dlrm.cpp:184-284: m and k multiples of the 16 x 16 tile, k a multiple of the 128-thread
    # block (the bottom-MLP copy loop, :205-217), f32 scratch acc[b][m][m]
    L = _lib("simple_dlrm")
    m, k, batch = 32, 128, 6
    x = O.f32_to_storage(O.normal(7, batch * m * k) * 0.5, O.F16)
    stride = k + m * (m - 1) // 2
    dx, dout = to_device(x), device_filled(batch * stride, np.uint16, 0xFF)
    dacc = device_filled(batch * m * m, np.float32, 0x00)
    rc = L.ref_simple_dlrm_fwd(_p(dx), _p(dout), _p(dacc), m, k, batch)
    assert rc == 0
    want = O.dlrm_fwd(O.F16, x, m, k, batch).ravel()
    ok, mx = O.compare(O.F16, to_host(dout, np.uint16), want, 10.0)
    assert ok, mx


def test_simple_sgemv_sample_kernel():
    # samples/simple_sgemv.cpp:88-101: y = alpha A x + beta y, A col-major m x k, f32; n = 1
    L = _lib("simple_sgemv")
    m, k = 512, 256
    a, x, y = O.uniform_pm1(8, m * k), O.uniform_pm1(9, k), O.uniform_pm1(10, m)
    # the sample's fragments are 16 columns wide: it reads 16 columns of "B" and reads / writes 16 columns
    # of "C" (column stride k and m), so the vector buffers here are 16 columns deep; only column 0 is data
    xb, yb = np.zeros(16 * k, np.float32), np.zeros(16 * m, np.float32)
    xb[:k], yb[:m] = x, y
    da, dx, dy = to_device(a), to_device(xb), to_device(yb)
    rc = L.ref_simple_sgemv(m, 1, k, _p(da), _p(dx), _p(dy), m, k, m, m, ctypes.c_float(2.0), ctypes.c_float(-1.0))
    assert rc == 0
    A = a.reshape(k, m).T.astype(np.float64)
    want = 2.0 * (A @ x.astype(np.float64)) - y.astype(np.float64)
    got = to_host(dy, np.float32)[:m].astype(np.float64)
    assert np.max(np.abs(got - want) / (np.abs(got) + np.abs(want) + 1.0)) <= k * 1e-7


@pytest.mark.parametrize("sample,dtype,la,lb,mnk", [
    ("simple_sgemm", O.F32, O.ROW, O.COL, (128, 64, 96)),
    ("simple_dgemm", O.F64, O.ROW, O.COL, (128, 64, 96)),
    ("perf_sgemm", O.F32, O.COL, O.ROW, (256, 128, 64)),
    ("perf_dgemm", O.F64, O.COL, O.ROW, (128, 192, 64)),
])
def test_f32_f64_gemm_sample_kernels(sample, dtype, la, lb, mnk):
    # simple_*gemm: A row-major, B col-major (samples/simple_sgemm.cpp:66-79); perf_*gemm: A col-major,
    # B row-major, LDS staging (samples/perf_sgemm.cpp:200-207); C / D row-major, alpha = beta = 2
    L = _lib(sample)
    m, n, k = mnk
    a = O.f32_to_storage(O.uniform_pm1(11, m * k), dtype)
    b = O.f32_to_storage(O.uniform_pm1(12, k * n), dtype)
    c = O.f32_to_storage(O.uniform_pm1(13, m * n), dtype)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    dd = device_filled(m * n, O.NP_STORAGE[dtype], 0xFF)
    lda = k if la == O.ROW else m
    ldb = n if lb == O.ROW else k
    fn = getattr(L, "ref_" + sample)
    rc = fn(m, n, k, _p(da), _p(db), _p(dc), _p(dd), lda, ldb, n, n, ctypes.c_double(2.0), ctypes.c_double(2.0))
    assert rc == 0
    want = O.gemm(dtype, dtype, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    # random data: the matrix core's summation order differs from the oracle's sequential one; two orders of a
    # k-term sum in the compute type differ by up to ~k eps / 2 on the reference's metric (10 eps is the
    # reference's bar for its integer-valued inputs, checked exactly below)
    ok, mx = O.compare(dtype, to_host(dd, O.NP_STORAGE[dtype]), want, max(10.0, k / 2.0))
    assert ok, mx
    a, b, c = O.fill_ref(dtype, m, k, la), O.fill_ref(dtype, k, n, lb), O.fill_ref(dtype, m, n, O.ROW)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    dd = device_filled(m * n, O.NP_STORAGE[dtype], 0xFF)
    assert fn(m, n, k, _p(da), _p(db), _p(dc), _p(dd), lda, ldb, n, n, ctypes.c_double(2.0), ctypes.c_double(2.0)) == 0
    want = O.gemm(dtype, dtype, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    assert np.array_equal(to_host(dd, O.NP_STORAGE[dtype]), want)


@pytest.mark.parametrize("dtype,tile", [(O.F16, 16), (O.F16, 32), (O.F32, 16), (O.F32, 32)])
def test_reference_dlrm_test_kernels_forward_and_backward(dtype, tile):
    # test/dlrm/device/dlrm_dot_fwd.hpp:37-138 and dlrm_dot_bwd.hpp:35-176 (trilReconstruct + dlrmDotBwd)
    L = _lib("test_dlrm")
    m, k, batch = 32, 128, 5
    stride = k + m * (m - 1) // 2
    st = O.NP_STORAGE[dtype]
    x = O.f32_to_storage(O.normal(14, batch * m * k) * 0.5, dtype)
    up = O.f32_to_storage(O.normal(15, batch * stride) * 0.5, dtype)
    dx, dup = to_device(x), to_device(up)
    dout = device_filled(batch * stride, st, 0xFF)
    dacc = device_filled(batch * m * m, np.float32, 0x00)
    assert L.ref_test_dlrm_fwd(dtype, tile, _p(dx), _p(dout), _p(dacc), m, k, batch) == 0
    want = O.dlrm_fwd(dtype, x, m, k, batch).ravel()
    tol = 10.0 if dtype == O.F16 else 40.0  # f32: two summation orders of 128 terms (see tests/test_dlrm.py)
    ok, mx = O.compare(dtype, to_host(dout, st), want, tol)
    assert ok, mx
    dgrad, dmlp = device_filled(batch * m * k, st, 0xFF), device_filled(batch * k, st, 0xFF)
    dacc2 = device_filled(batch * m * m, st, 0x00)
    assert L.ref_test_dlrm_bwd(dtype, tile, _p(dx), _p(dup), _p(dgrad), _p(dmlp), _p(dacc2), m, k, batch) == 0
    if dtype == O.F16:
        want_mlp, want_grad = O.dlrm_bwd(dtype, x, up, m, k, batch)
        assert np.array_equal(to_host(dmlp, st), want_mlp.ravel())
        ok, mx = O.compare(dtype, to_host(dgrad, st), want_grad.ravel(), 10.0)
        assert ok, mx
    else:
        want_mlp, want_grad = O.dlrm_bwd(dtype, x, up, m, k, batch)
        assert np.array_equal(to_host(dmlp, st), want_mlp.ravel())
        ok, mx = O.compare(dtype, to_host(dgrad, st), want_grad.ravel(), 40.0)
        assert ok, mx


def test_reference_io_traits_unit_kernel():
    # test/unit/io_traits_test/device/io_traits.hpp:34-101: PackTraits and IOTraits identities checked on the
    # device; 0 = SUCCESS_VALUE
    L = _lib("test_io_traits")
    n = L.ref_test_io_traits_cases()
    assert n >= 20
    assert [L.ref_test_io_traits(i) for i in range(n)] == [0] * n


@pytest.mark.parametrize("tile", [16, 32])
def test_reference_dlrm_lds_test_kernels(tile):
    # test/dlrm/device/dlrm_dot_fwd_lds.hpp / dlrm_dot_bwd_lds.hpp with the register-file LDS mapping
    # (test/dlrm/lds_mapping_util.hpp:63-367): fragments parked in LDS and re-read between K steps
    L = _lib("test_dlrm")
    m, k, batch = 32, 128, 5
    stride = k + m * (m - 1) // 2
    x = O.f32_to_storage(O.normal(16, batch * m * k) * 0.5, O.F16)
    up = O.f32_to_storage(O.normal(17, batch * stride) * 0.5, O.F16)
    dx, dup = to_device(x), to_device(up)
    dout = device_filled(batch * stride, np.uint16, 0xFF)
    dacc = device_filled(batch * m * m, np.float32, 0x00)
    assert L.ref_test_dlrm_fwd_lds(tile, _p(dx), _p(dout), _p(dacc), m, k, batch) == 0
    ok, mx = O.compare(O.F16, to_host(dout, np.uint16), O.dlrm_fwd(O.F16, x, m, k, batch).ravel(), 10.0)
    assert ok, mx
    dgrad, dmlp = device_filled(batch * m * k, np.uint16, 0xFF), device_filled(batch * k, np.uint16, 0xFF)
    dacc2 = device_filled(batch * m * m, np.uint16, 0x00)
    assert L.ref_test_dlrm_bwd_lds(tile, _p(dx), _p(dup), _p(dgrad), _p(dmlp), _p(dacc2), m, k, batch) == 0
    want_mlp, want_grad = O.dlrm_bwd(O.F16, x, up, m, k, batch)
    assert np.array_equal(to_host(dmlp, np.uint16), want_mlp.ravel())
    ok, mx = O.compare(O.F16, to_host(dgrad, np.uint16), want_grad.ravel(), 10.0)
    assert ok, mx


def _gemm_args(m, n, k, da, db, dc, dd, lda, ldb, alpha, beta):
    return (m, n, k, _p(da), _p(db), _p(dc), _p(dd), lda, ldb, n, n, ctypes.c_float(alpha), ctypes.c_float(beta))


@pytest.mark.parametrize("cid,in_t,out_t,la,lb", [(0, O.F16, O.F32, O.ROW, O.COL), (1, O.F16, O.F16, O.COL, O.ROW),
                                                  (2, O.I8, O.I32, O.ROW, O.COL)])
def test_reference_gemm_test_kernel_block_per_wave(cid, in_t, out_t, la, lb):
    # test/gemm/gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp:50-175
    L = _lib("test_gemm_simple")
    m, n, k = 128, 192, 96
    if in_t == O.I8:
        a, b = O.uniform_int8(21, m * k), O.uniform_int8(22, k * n)
        c = O.uniform_int8(23, m * n).astype(np.int32) * 11
    else:
        a = O.f32_to_storage(O.uniform_pm1(21, m * k), in_t)
        b = O.f32_to_storage(O.uniform_pm1(22, k * n), in_t)
        c = O.f32_to_storage(O.uniform_pm1(23, m * n), out_t)
    st = O.NP_STORAGE[out_t]
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, st, 0xFF)
    lda, ldb = (k if la == O.ROW else m), (n if lb == O.ROW else k)
    assert L.ref_test_gemm_simple(cid, *_gemm_args(m, n, k, da, db, dc, dd, lda, ldb, 2.0, 2.0)) == 0
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    got = to_host(dd, st)
    if in_t == O.I8:
        assert np.array_equal(got, want)
    else:
        ok, mx = O.compare(out_t, got, want, 10.0 if out_t == O.F16 else k / 2.0)
        assert ok, mx


@pytest.mark.parametrize("cid,in_t,out_t,la,lb", [(0, O.F16, O.F32, O.ROW, O.COL), (1, O.BF16, O.BF16, O.COL, O.ROW),
                                                  (2, O.I8, O.I32, O.ROW, O.COL), (3, O.F16, O.F16, O.ROW, O.ROW)])
def test_reference_gemm_test_kernel_multi_block(cid, in_t, out_t, la, lb):
    # test/gemm/gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp: BlocksX x BlocksY blocks per wave
    # (2 x 2, 4 x 2, 2 x 4, 8 x 8), no LDS, no cooperation
    L = _lib("test_gemm_multi")
    m, n, k = 256, 256, 96
    if in_t == O.I8:
        a, b = O.uniform_int8(24, m * k), O.uniform_int8(25, k * n)
        c = O.uniform_int8(26, m * n).astype(np.int32) * 11
    else:
        a = O.f32_to_storage(O.uniform_pm1(24, m * k), in_t)
        b = O.f32_to_storage(O.uniform_pm1(25, k * n), in_t)
        c = O.f32_to_storage(O.uniform_pm1(26, m * n), out_t)
    st = O.NP_STORAGE[out_t]
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, st, 0xFF)
    lda, ldb = (k if la == O.ROW else m), (n if lb == O.ROW else k)
    assert L.ref_test_gemm_multi(cid, *_gemm_args(m, n, k, da, db, dc, dd, lda, ldb, 2.0, 2.0)) == 0
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    got = to_host(dd, st)
    if in_t == O.I8:
        assert np.array_equal(got, want)
    else:
        ok, mx = O.compare(out_t, got, want, 10.0 if out_t in (O.F16, O.BF16) else k / 2.0)
        assert ok, mx


@pytest.mark.parametrize("lds_col_major", [0, 1])
@pytest.mark.parametrize("cid", range(6))
def test_reference_gemm_test_kernel_cooperative(cid, lds_col_major):
    # test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp:52-283 with the six CooperativeGemm
    # configurations of test/gemm/gemm_config.hpp:64-431 (workgroup / block / wave level cooperation, LDS
    # holding NT, TN or register-file images), both LDS data layouts
    L = _lib("test_gemm_coop")
    m, n, k = 256, 384, 128
    a = O.f32_to_storage(O.uniform_pm1(31, m * k), O.F16)
    b = O.f32_to_storage(O.uniform_pm1(32, k * n), O.F16)
    c = O.f32_to_storage(O.uniform_pm1(33, m * n), O.F16)
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, np.uint16, 0xFF)
    assert L.ref_test_gemm_coop(cid, lds_col_major, *_gemm_args(m, n, k, da, db, dc, dd, m, n, 2.0, 2.0)) == 0
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    ok, mx = O.compare(O.F16, to_host(dd, np.uint16), want, 10.0)
    assert ok, mx


_COOP_TYPED = {0: (O.I8, O.I32, O.ROW, O.COL), 1: (O.BF16, O.F32, O.ROW, O.ROW), 2: (O.F32, O.F32, O.COL, O.COL),
               3: (O.F64, O.F64, O.ROW, O.COL), 4: (O.E4M3, O.F32, O.COL, O.ROW)}


@pytest.mark.parametrize("cfg", range(3))
@pytest.mark.parametrize("variant", sorted(_COOP_TYPED))
def test_reference_gemm_test_kernel_cooperative_other_types(variant, cfg):
    # the same kernel with int8, bf16, f32, f64 and e4m3 operands in the other operand orientations (TN, TT, NN):
    # the type tuples of test/gemm/gemm_common_test_params.hpp:50-130, three of the CooperativeGemm configurations
    L = _lib("test_gemm_coop_typed")
    in_t, out_t, la, lb = _COOP_TYPED[variant]
    m, n, k = 256, 384, 128
    if in_t == O.I8:
        a, b = O.uniform_int8(41, m * k), O.uniform_int8(42, k * n)
        c = O.uniform_int8(43, m * n).astype(np.int32) * 11
    else:
        src = O.normal if in_t == O.E4M3 else O.uniform_pm1
        a = O.f32_to_storage(src(41, m * k), in_t)
        b = O.f32_to_storage(src(42, k * n), in_t)
        c = O.f32_to_storage(O.uniform_pm1(43, m * n), out_t)
    st = O.NP_STORAGE[out_t]
    da, db, dc, dd = to_device(a), to_device(b), to_device(c), device_filled(m * n, st, 0xFF)
    lda, ldb = (k if la == O.ROW else m), (n if lb == O.ROW else k)
    assert L.ref_test_gemm_coop_typed(variant, cfg, *_gemm_args(m, n, k, da, db, dc, dd, lda, ldb, 2.0, 2.0)) == 0
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    got = to_host(dd, st)
    if in_t == O.I8:
        assert np.array_equal(got, want)
    elif in_t == O.E4M3:
        g, w = got.astype(np.float64), want.astype(np.float64)
        assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= 1e-2
    else:
        ok, mx = O.compare(out_t, got, want, k / 2.0)
        assert ok, mx
