"""Pins the CPU oracle (oracle/oracle.c) against things that are not the oracle:
numpy library routines on inputs where the arithmetic is exact, closed forms,
brute force on tiny shapes, and the fixtures the reference's DLRM tests hold."""
import itertools
import os

import numpy as np
import pytest

import oraclelib as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LAYOUTS = [O.ROW, O.COL]


# ------------------------------------------------------------------ scalar conversions

def test_f16_decode_all_codes():
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = np.array([O.lib().orc_f16_to_f32(int(c)) for c in codes], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(got))  # NaN payloads may be quieted in transit
    assert np.array_equal(want.view(np.uint32)[~nan], got.view(np.uint32)[~nan])


def test_f16_encode_rne():
    # every representable value, every midpoint between neighbours, and just off the midpoints
    codes = np.arange(0, 0x7C00, dtype=np.uint16)
    v = codes.view(np.float16).astype(np.float64)
    mids = (v[:-1] + v[1:]) / 2
    pts = np.concatenate([v, mids, np.nextafter(mids.astype(np.float32), np.float32(0)).astype(np.float64),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)).astype(np.float64),
                          [65504.0, 65519.9, 65520.0, 65536.0, 1e9, 1e-9, 2.0 ** -25, 2.0 ** -24 * 1.5]])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    want = pts.astype(np.float16).view(np.uint16)
    got = np.array([O.lib().orc_f32_to_f16(float(p)) for p in pts], dtype=np.uint16)
    assert np.array_equal(want, got)


def test_bf16_roundtrip_and_rne():
    codes = np.arange(0, 0x7F80, 3, dtype=np.uint32)
    for c in codes[:: 97]:
        f = O.lib().orc_bf16_to_f32(int(c))
        assert np.float32(f).view(np.uint32) == (int(c) << 16)
        assert O.lib().orc_f32_to_bf16(f) == int(c)
    # midpoint ties go to even, just-above goes up
    for c in (0x3F80, 0x3F81, 0x4000, 0x0001, 0x7F00):
        lo = np.uint32(c << 16)
        tie = np.uint32(lo + 0x8000).view(np.float32)
        above = np.uint32(lo + 0x8001).view(np.float32)
        below = np.uint32(lo + 0x7FFF).view(np.float32)
        assert O.lib().orc_f32_to_bf16(float(tie)) == (c if c % 2 == 0 else c + 1)
        assert O.lib().orc_f32_to_bf16(float(above)) == c + 1
        assert O.lib().orc_f32_to_bf16(float(below)) == c


def test_e4m3_decode_closed_form():
    # OCP E4M3: (-1)^s * 2^(e-7) * (1 + m/8), subnormals m * 2^-9, NaN only at S.1111.111
    for v in range(256):
        got = O.lib().orc_e4m3_to_f32(v)
        if (v & 0x7F) == 0x7F:
            assert np.isnan(got)
        else:
            assert got == O.E4M3_TABLE[v]
    assert O.lib().orc_e4m3_to_f32(0x7E) == 448.0
    assert O.lib().orc_e4m3_to_f32(0x08) == 2.0 ** -6
    assert O.lib().orc_e4m3_to_f32(0x01) == 2.0 ** -9
    assert O.lib().orc_e4m3_to_f32(0x20) == 0.125  # numeric_limits epsilon (float8.hpp:549-580)


def test_e4m3_encode_midpoints_and_saturation():
    pos = O.E4M3_TABLE[:0x7F].astype(np.float64)
    mids = (pos[:-1] + pos[1:]) / 2
    pts = np.concatenate([pos, mids, mids * (1 + 1e-6), mids * (1 - 1e-6), [448.0, 449.0, 464.0, 480.0, 1e6, 3e38]])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    want = O.e4m3_encode(pts)
    got = np.array([O.lib().orc_f32_to_e4m3(float(p)) for p in pts], dtype=np.uint8)
    assert np.array_equal(want, got)
    # ties go to the even code; everything above max saturates to +-448 (no inf in the format)
    assert O.lib().orc_f32_to_e4m3(float(mids[8])) % 2 == 0
    assert O.lib().orc_f32_to_e4m3(1e30) == 0x7E and O.lib().orc_f32_to_e4m3(-1e30) == 0xFE
    assert O.lib().orc_f32_to_e4m3(float("nan")) & 0x7F == 0x7F


# ------------------------------------------------------------------ GEMM

@pytest.mark.parametrize("la,lb,lc,ld", list(itertools.product(LAYOUTS, repeat=4)))
def test_gemm_int8_all_layouts_vs_numpy(la, lb, lc, ld):
    m, n, k = 19, 23, 40
    A = O.uniform_int8(11, m * k).reshape(m, k)
    B = O.uniform_int8(12, k * n).reshape(k, n)
    C = (O.uniform_int8(13, m * n).astype(np.int32) * 1000).reshape(m, n)
    want = 3 * (A.astype(np.int64) @ B.astype(np.int64)) + (-2) * C.astype(np.int64)
    d = O.gemm(O.I8, O.I32, la, lb, lc, ld, m, n, k, O.to_flat(A, la), O.to_flat(B, lb), O.to_flat(C, lc), 3.0, -2.0)
    assert np.array_equal(O.as_matrix(d, m, n, ld).astype(np.int64), want)


@pytest.mark.parametrize("la,lb,lc,ld", [(O.ROW, O.COL, O.ROW, O.ROW), (O.COL, O.ROW, O.COL, O.ROW), (O.ROW, O.ROW, O.COL, O.COL)])
def test_gemm_int8_to_int8_is_the_low_byte_of_the_int32_result(la, lb, lc, ld):
    # (int8, int8, int32) of the reference's extended type list: int32 arithmetic, static_cast<int8_t> at the end,
    # pinned here by exact int64 arithmetic reduced modulo 256 (sums well beyond the int8 range)
    m, n, k = 17, 21, 48
    A = O.uniform_int8(21, m * k).reshape(m, k)
    B = O.uniform_int8(22, k * n).reshape(k, n)
    C = O.uniform_int8(23, m * n).reshape(m, n)
    full = 3 * (A.astype(np.int64) @ B.astype(np.int64)) + (-2) * C.astype(np.int64)
    want = (full & 0xFF).astype(np.uint8).view(np.int8)
    assert np.abs(full).max() > 1000
    d = O.gemm(O.I8, O.I8, la, lb, lc, ld, m, n, k, O.to_flat(A, la), O.to_flat(B, lb), O.to_flat(C, lc), 3.0, -2.0)
    assert d.dtype == np.int8 and np.array_equal(O.as_matrix(d, m, n, ld), want)


def test_gemm_int8_max_magnitude_k8192():
    # |sum| reaches 8192 * 128 * 128 = 2^27 exactly: no overflow, closed form
    m, n, k = 2, 3, 8192
    A = np.full((m, k), -128, dtype=np.int8)
    B = np.full((k, n), -128, dtype=np.int8)
    d = O.gemm(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, O.to_flat(A, O.ROW), O.to_flat(B, O.COL), None, 1.0, 0.0)
    assert np.all(d == 8192 * 128 * 128)


@pytest.mark.parametrize("in_type", [O.F16, O.BF16, O.E4M3, O.F32])
@pytest.mark.parametrize("la,lb", list(itertools.product(LAYOUTS, repeat=2)))
def test_gemm_float_reference_pattern_exact(in_type, la, lb):
    # The reference's own test inputs (small integers): every product and partial sum is an
    # exactly representable integer, so float64 matmul is the exact answer in any order.
    m, n, k = 48, 32, 80
    a = O.fill_ref(in_type, m, k, la)
    b = O.fill_ref(in_type, k, n, lb)
    c = O.fill_ref(O.F32, m, n, O.ROW)
    A = O.as_matrix(O.storage_to_f32(a, in_type), m, k, la).astype(np.float64)
    B = O.as_matrix(O.storage_to_f32(b, in_type), k, n, lb).astype(np.float64)
    C = O.as_matrix(c, m, n, O.ROW).astype(np.float64)
    # independent statement of the fill pattern (test/device/common.hpp:203-220)
    r, cc = np.meshgrid(np.arange(m), np.arange(k), indexing="ij")
    assert np.array_equal(A, -((r * k + cc) % 3).astype(np.float64))
    want = 2.0 * (A @ B) + 2.0 * C
    d = O.gemm(in_type, O.F32, la, lb, O.ROW, O.COL, m, n, k, a, b, c, 2.0, 2.0)
    assert np.array_equal(O.as_matrix(d, m, n, O.COL).astype(np.float64), want)


@pytest.mark.parametrize("in_type", [O.F16, O.BF16, O.E4M3])
def test_gemm_sequential_f32_sum_order(in_type):
    # products of two <=11-bit significands are exact in f32, so the only rounding is the
    # running sum; np.add.accumulate is sequential and pins the h = 0..k-1 order bit for bit.
    m, n, k = 5, 7, 300
    src = O.uniform_pm1 if in_type != O.E4M3 else O.normal
    a = O.f32_to_storage(src(21, m * k), in_type)
    b = O.f32_to_storage(src(22, k * n), in_type)
    A = O.storage_to_f32(a, in_type).reshape(m, k)
    B = O.storage_to_f32(b, in_type).reshape(n, k)  # col-major B: K contiguous
    want = np.zeros((m, n), dtype=np.float32)
    for i in range(m):
        for j in range(n):
            prod = (A[i].astype(np.float32) * B[j].astype(np.float32)).astype(np.float32)
            want[i, j] = np.add.accumulate(prod, dtype=np.float32)[-1]
    d = O.gemm(in_type, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0).reshape(m, n)
    assert np.array_equal(d.view(np.uint32), want.view(np.uint32))
    # a reversed summation order must NOT reproduce it (the check has teeth)
    rev = np.array([[np.add.accumulate((A[i] * B[j])[::-1], dtype=np.float32)[-1] for j in range(n)] for i in range(m)])
    if in_type != O.E4M3:  # e4m3 products carry so few bits that any order is exact
        assert not np.array_equal(rev.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("out_type", [O.F32, O.F16, O.BF16])
def test_gemm_epilogue_rounds_once(out_type):
    m, n, k = 9, 6, 64
    a = O.f32_to_storage(O.uniform_pm1(31, m * k), O.F16)
    b = O.f32_to_storage(O.uniform_pm1(32, k * n), O.F16)
    c = O.f32_to_storage(O.uniform_pm1(33, m * n), out_type)
    A = O.storage_to_f32(a, O.F16).reshape(m, k)
    B = O.storage_to_f32(b, O.F16).reshape(k, n)
    C = O.storage_to_f32(c, out_type).reshape(m, n)
    acc = np.zeros((m, n), dtype=np.float32)
    for h in range(k):
        acc = (acc + np.outer(A[:, h], B[h]).astype(np.float32)).astype(np.float32)
    for alpha, beta in ((2.0, 2.0), (1.0, 0.0), (0.5, -4.0)):
        # power-of-two scalars: both products exact, one f32 add, one cast to the output type
        want = O.f32_to_storage((np.float32(alpha) * acc + np.float32(beta) * C).astype(np.float32), out_type)
        d = O.gemm(O.F16, out_type, O.ROW, O.ROW, O.ROW, O.ROW, m, n, k, a, b, c, alpha, beta)
        assert np.array_equal(d.reshape(m, n), want)


def test_gemm_one_hot_indexing_brute_force():
    # a single 1 in A and in B: D has a single 1 at (i, j) iff the k indices meet
    m, n, k = 3, 5, 4
    for la, lb, ld in itertools.product(LAYOUTS, repeat=3):
        for i, h, j in itertools.product(range(m), range(k), range(n)):
            A = np.zeros((m, k), dtype=np.float32); A[i, h] = 1
            B = np.zeros((k, n), dtype=np.float32); B[h, j] = 1
            a = O.f32_to_storage(O.to_flat(A, la), O.F16)
            b = O.f32_to_storage(O.to_flat(B, lb), O.F16)
            d = O.as_matrix(O.gemm(O.F16, O.F32, la, lb, O.ROW, ld, m, n, k, a, b, None, 1.0, 0.0), m, n, ld)
            want = np.zeros((m, n), dtype=np.float32); want[i, j] = 1
            assert np.array_equal(d, want)


def test_gemm_rows_equals_full():
    m, n, k = 40, 24, 96
    for in_type, out_type in ((O.F16, O.F16), (O.BF16, O.BF16), (O.I8, O.I32), (O.E4M3, O.F32)):
        if in_type == O.I8:
            a, b = O.uniform_int8(1, m * k), O.uniform_int8(2, k * n)
        else:
            a = O.f32_to_storage(O.uniform_pm1(1, m * k), in_type)
            b = O.f32_to_storage(O.uniform_pm1(2, k * n), in_type)
        full = O.gemm(in_type, out_type, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0).reshape(m, n)
        rows = np.array([0, 7, 39, 13], dtype=np.uint32)
        part = O.gemm_rows(in_type, out_type, O.COL, O.ROW, m, n, k, a, b, rows)
        assert np.array_equal(part, full[rows])


# ------------------------------------------------------------------ DLRM (reference-held fixtures)

def _load(name, dtype):
    return np.fromfile(os.path.join(GOLD, "dlrm", name), dtype=dtype)


def test_dlrm_fwd_fixture_fp32():
    x = _load("input_fp32", np.float32)
    want = _load("output_fp32", np.float32).reshape(64, 479)
    got = O.dlrm_fwd(O.F32, x, 27, 128, 64)
    assert np.array_equal(got[:, :128], want[:, :128])
    ok, mx = O.compare(O.F32, got, want, 100.0)
    assert np.max(np.abs(got - want)) < 2e-5 and ok, mx


def test_dlrm_fwd_fixture_fp16():
    x = _load("input_fp16", np.uint16)
    want = _load("output_fp16", np.uint16).reshape(64, 479)
    got = O.dlrm_fwd(O.F16, x, 27, 128, 64)
    assert np.array_equal(got[:, :128], want[:, :128])
    ok, mx = O.compare(O.F16, got, want, 10.0)  # the reference's DLRM tolerance
    assert ok, mx
    # at most one fp16 ulp anywhere (the fixture was produced with a different summation order)
    g, w = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    assert np.all(np.abs(g - w) <= np.spacing(np.abs(w).astype(np.float16)).astype(np.float64))
    assert np.mean(got == want) > 0.9


def test_dlrm_fwd_layout_closed_form():
    # out[k + i(i-1)/2 + j] = <x_i, x_j> for j < i, on integer data (exact)
    m, k, batch = 6, 16, 3
    X = (O.uniform_int8(5, batch * m * k).astype(np.float32) % 5).reshape(batch, m, k)
    got = O.dlrm_fwd(O.F32, X.ravel(), m, k, batch)
    for b in range(batch):
        G = X[b].astype(np.float64) @ X[b].astype(np.float64).T
        assert np.array_equal(got[b, :k], X[b, 0])
        for i in range(m):
            for j in range(i):
                assert got[b, k + i * (i - 1) // 2 + j] == G[i, j]


@pytest.mark.parametrize("suffix,dtype,np_t,tol", [("fp32", O.F32, np.float32, 100.0), ("fp16", O.F16, np.uint16, 10.0)])
def test_dlrm_bwd_fixture(suffix, dtype, np_t, tol):
    x = _load("input_" + suffix, np_t)
    up = _load("input_grad_" + suffix, np_t)
    want = _load("output_input_grad_" + suffix, np_t).reshape(64, 27, 128)
    want_mlp = _load("output_mlp_input_grad_" + suffix, np_t).reshape(64, 128)
    mlp, got = O.dlrm_bwd(dtype, x, up, 27, 128, 64)
    assert np.array_equal(mlp, want_mlp)
    ok, mx = O.compare(dtype, got, want, tol)
    assert ok, mx


# ------------------------------------------------------------------ comparator

def test_compare_closed_forms():
    x = np.array([1.0, 2.0, -3.0], dtype=np.float32)
    assert O.compare(O.F32, x, x.copy()) == (True, 0.0)
    y = x.copy(); y[1] = 2.5
    ok, mx = O.compare(O.F32, x, y)
    assert not ok and mx == pytest.approx(0.5 / 5.5)
    y = x.copy(); y[2] = np.nextafter(np.float32(-3.0), np.float32(0))
    ok, mx = O.compare(O.F32, x, y)  # one ulp at 3.0: 2.4e-7/7 < 10 eps
    assert ok and 0 < mx < 1e-7
    y = x.copy(); y[0] = np.inf
    ok, mx = O.compare(O.F32, x, y)
    assert not ok and np.isinf(mx)
    y = x.copy(); y[0] = np.nan
    ok, mx = O.compare(O.F32, x, y)
    assert not ok and np.isnan(mx)
    # f16: eps = 2^-10, tolerance 10 -> threshold 0.009765625
    a = np.array([1.0], dtype=np.float16).view(np.uint16)
    b = np.array([1.03], dtype=np.float16).view(np.uint16)
    ok, mx = O.compare(O.F16, a, b)
    assert not ok and mx == pytest.approx((float(np.float16(1.03)) - 1.0) / (float(np.float16(1.03)) + 2.0))
    # integers: eps = 0, so only exact equality passes
    i1 = np.array([5, -7], dtype=np.int32)
    assert O.compare(O.I32, i1, i1.copy())[0]
    assert not O.compare(O.I32, i1, np.array([5, -6], dtype=np.int32))[0]


# ------------------------------------------------------------------ 2:4 format

def test_sparse24_format_invariants():
    m, k = 32, 256
    mask = O.sparse24_mask(3, m, k)
    assert np.all(mask.reshape(m, k // 4, 4).sum(axis=2) == 2)
    vals_dense = O.uniform_int8(4, m * k).reshape(m, k)
    vals_dense = np.where(vals_dense == 0, np.int8(1), vals_dense)
    dense = np.where(mask, vals_dense, np.int8(0)).astype(np.int8)
    vals, meta = O.compress24(dense.view(np.uint8), m, k)
    assert vals.shape == (k // 128, m // 16, 4, 16, 16) and meta.shape == (k // 128, m // 16, 4, 16, 4)
    # The expected storage from plain numpy: per row, the kept pair of each group in position order and a nibble
    # idx0 | idx1 << 2 per group (even group in the low nibble), then the K-blocked order by reshaping / transposing
    grp = dense.view(np.uint8).reshape(m, k // 4, 4)
    pos = np.argsort(~mask.reshape(m, k // 4, 4), axis=2, kind="stable")[:, :, :2]  # the two kept positions, increasing
    assert np.all(pos[:, :, 0] < pos[:, :, 1])
    plain_vals = np.take_along_axis(grp, pos, axis=2).reshape(m, k // 2)
    nib = (pos[:, :, 0] | (pos[:, :, 1] << 2)).astype(np.uint8)
    plain_meta = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    assert np.array_equal(vals, O.plain_to_kblocked(plain_vals, m, k))
    assert np.array_equal(meta, O.plain_to_kblocked(plain_meta, m, k))
    # spot check of one element against the description in words: row 21, dense k 200..203 = stage 1, lane group 2,
    # its group 2 of 8 -> kept bytes 4, 5 of the lane's 16; the nibble is the low half of index byte 1
    st, rb, lg, rr = 1, 1, 2, 5
    assert list(vals[st, rb, lg, rr, 4:6]) == list(plain_vals[21, 100:102])
    assert (meta[st, rb, lg, rr, 1] & 0xF) == nib[21, 50]
    assert np.array_equal(O.decompress24(vals, meta, m, k), dense.view(np.uint8))
    # a group with three non-zeros is rejected, and so are sizes off the 16 x 128 grid
    bad = dense.copy(); bad[0, :4] = 1
    with pytest.raises(ValueError):
        O.compress24(bad.view(np.uint8), m, k)
    with pytest.raises(ValueError):
        O.compress24(dense.view(np.uint8)[:, :64].copy(), m, 64)
    # groups with fewer than two non-zeros still round-trip
    few = dense.copy(); few[1, :8] = 0; few[2, 0:4] = [0, 0, 0, 9]
    v2, m2 = O.compress24(few.view(np.uint8), m, k)
    assert np.array_equal(O.decompress24(v2, m2, m, k), few.view(np.uint8))


def test_e4m3_matches_torch_float8_e4m3fn():
    """An independent implementation of the same OCP format: torch's float8_e4m3fn cast (round to
    nearest even; values beyond +-448 clamped first, as the saturating conversion does)."""
    torch = pytest.importorskip("torch")
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    x = np.concatenate([O.normal(11, 1 << 18), O.normal(12, 1 << 16) * 200.0, O.uniform_pm1(13, 1 << 16) * 2.0 ** -7,
                        np.float32([0.0, -0.0, 448.0, -448.0, 1e9, -1e9, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -11])])
    t = torch.from_numpy(x.copy()).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    got = O.f32_to_storage(x, O.E4M3)
    want = t.view(torch.uint8).numpy()
    # -0.0 and +0.0 encode to 0x80 / 0x00 in both; compare bytes
    assert np.array_equal(got, want)
    assert np.array_equal(O.storage_to_f32(got, O.E4M3), t.to(torch.float32).numpy())


def test_e5m2_decode_closed_form_and_torch():
    """OCP e5m2 (the reference's bfloat8_t): sign, 5 exponent bits (bias 15), 2 mantissa bits -- binary16 cut after
    two mantissa bits.  Every finite code against the closed form, against torch's float8_e5m2 where present, and
    through the oracle's GEMM (a 1 x 1 x 1 product with 1.0)."""
    codes = np.arange(256, dtype=np.uint8)
    dec = O.storage_to_f32(codes, O.E5M2)
    for v in range(256):
        s, e, m = v >> 7, (v >> 2) & 0x1F, v & 3
        if e == 31:
            assert not np.isfinite(dec[v])
            continue
        mag = (m / 4.0) * 2.0 ** -14 if e == 0 else (1.0 + m / 4.0) * 2.0 ** (e - 15)
        assert dec[v] == np.float32(-mag if s else mag), v
    finite = codes[((codes >> 2) & 0x1F) != 31]
    one = np.array([0x3C], dtype=np.uint8)  # 1.0
    for v in finite[::7]:
        d = O.gemm(O.E5M2, O.F32, O.ROW, O.COL, O.ROW, O.ROW, 1, 1, 1, np.array([v], np.uint8), one, None, 1.0, 0.0)
        assert d[0] == dec[v]
    torch = pytest.importorskip("torch")
    if hasattr(torch, "float8_e5m2"):
        t = torch.from_numpy(finite.copy()).view(torch.float8_e5m2).to(torch.float32).numpy()
        assert np.array_equal(t, dec[finite])


def test_gemm_f64_against_numpy():
    """f64 path (the reference's dgemm instantiation): exact on the reference's integer pattern in every
    layout combination; on random data equal to numpy's sequential float64 accumulation bit for bit."""
    m, n, k = 24, 40, 56
    for la in (O.ROW, O.COL):
        for lb in (O.ROW, O.COL):
            for ld in (O.ROW, O.COL):
                a, b, c = O.fill_ref(O.F64, m, k, la), O.fill_ref(O.F64, k, n, lb), O.fill_ref(O.F64, m, n, ld)
                A, B, C = O.as_matrix(a, m, k, la), O.as_matrix(b, k, n, lb), O.as_matrix(c, m, n, ld)
                got = O.as_matrix(O.gemm(O.F64, O.F64, la, lb, ld, ld, m, n, k, a, b, c, 2.0, -3.0), m, n, ld)
                assert np.array_equal(got, 2.0 * (A @ B) - 3.0 * C)
    a = O.normal(21, m * k).astype(np.float64) * 1.2345678901234
    b = O.normal(22, k * n).astype(np.float64) / 3.0
    A, B = a.reshape(m, k), b.reshape(k, n)
    got = O.gemm(O.F64, O.F64, O.ROW, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0).reshape(m, n)
    prod = A[:, :, None] * B[None, :, :]  # (m, k, n): products in k order
    seq = np.add.accumulate(prod, axis=1)[:, -1, :]  # sequential left-to-right sums
    assert np.array_equal(got, seq)
