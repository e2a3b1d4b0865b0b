"""GPU parity of the GEMM kernels (through the C ABI) against the CPU oracle.

Bars, on the reference's metric |a-b| / (|a|+|b|+1) (test/device/common.hpp:111-124):
  int8 -> int32            bit-exact
  f16, bf16 inputs         <= 1e-3 against the oracle's f32 result (f32 accumulation on both
                           sides, different summation order)
  fp8 e4m3 inputs          <= 1e-2
  16-bit outputs           the bound above plus half an ulp of the output type (2^-11 for f16,
                           2^-9 for bf16) against the oracle's f32 result, and never more than
                           one ulp away from the oracle's own 16-bit result
plus exact equality on the reference's integer-valued test inputs (test/device/common.hpp:203-220),
where every partial sum is exact in any order."""
import itertools

import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

REL_TOL = {O.F16: 1e-3, O.BF16: 1e-3, O.E4M3: 1e-2}


def _inputs(in_t, out_t, m, n, k, seed=1, pattern="random"):
    if pattern == "reference":
        return None
    if in_t == O.I8:
        a, b = O.uniform_int8(seed, m * k), O.uniform_int8(seed + 1, k * n)
        c = O.uniform_int8(seed + 2, m * n).astype(np.int32) * 37
    else:
        src = O.normal if in_t == O.E4M3 else O.uniform_pm1
        a = O.f32_to_storage(src(seed, m * k), in_t)
        b = O.f32_to_storage(src(seed + 1, k * n), in_t)
        c = O.f32_to_storage(O.uniform_pm1(seed + 2, m * n), out_t)
    return a, b, c


def _run(in_t, out_t, la, lb, lc, ld, m, n, k, a, b, c, alpha, beta, kernel):
    da, db = to_device(a), to_device(b)
    dc = to_device(c) if c is not None else None
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    R.gemm(in_t, out_t, m, n, k, da, db, dc, dd, alpha, beta, la, lb, lc, ld, kernel=kernel)
    return to_host(dd, O.NP_STORAGE[out_t])


def _max_rel(out_t, got, want):
    g = O.storage_to_f32(got, out_t).astype(np.float64)
    w = O.storage_to_f32(want, out_t).astype(np.float64)
    assert np.all(np.isfinite(g))
    return float(np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)))


HALF_ULP = {O.F16: 2.0 ** -11, O.BF16: 2.0 ** -9, O.F32: 0.0}


def _check(in_t, out_t, got, want, want_f32=None):
    """got / want in out_t storage; want_f32 = the oracle's f32-output result when out_t is 16-bit."""
    if in_t == O.I8:
        assert np.array_equal(got, want)
        return
    if out_t == O.F64:
        ok, mx = O.compare(O.F64, got, want, 10.0)  # the reference's 10 eps(f64), test/gemm/gemm_kernel_base_impl.hpp:906-918
        assert ok, mx
        return
    tol = REL_TOL.get(in_t, 1e-5)
    if out_t == O.F32:
        assert _max_rel(out_t, got, want) <= tol
        return
    g = O.storage_to_f32(got, out_t).astype(np.float64)
    assert np.all(np.isfinite(g))
    if want_f32 is not None:
        w = want_f32.astype(np.float64)
        assert np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= tol + HALF_ULP[out_t]
    # at most one ulp of the output type from the oracle's rounded result
    w16 = O.storage_to_f32(want, out_t).astype(np.float64)
    ulp = np.maximum(np.abs(w16), 2.0 ** -14) * (4 * HALF_ULP[out_t])
    assert np.all(np.abs(g - w16) <= ulp + tol * (np.abs(w16) + 1.0))


def test_config1_256_cubed_f16_tn_alpha_beta_2():
    # benchmark configuration 1: A row-major (T), B col-major (N), C/D f32 row-major, alpha = beta = 2
    m = n = k = 256
    a, b, c = _inputs(O.F16, O.F32, m, n, k, seed=1)
    want = O.gemm(O.F16, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    for kernel in (R.KERNEL_SIMPLE, R.KERNEL_TILED):
        got = _run(O.F16, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0, kernel)
        assert _max_rel(O.F32, got, want) <= 1e-3
    # the reference's own pass criterion (10 eps of f32) applies to its integer-valued inputs,
    # where GPU and CPU agree exactly
    a, b, c = O.fill_ref(O.F16, m, k, O.ROW), O.fill_ref(O.F16, k, n, O.COL), O.fill_ref(O.F32, m, n, O.ROW)
    want = O.gemm(O.F16, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    for kernel in (R.KERNEL_SIMPLE, R.KERNEL_TILED):
        got = _run(O.F16, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0, kernel)
        ok, mx = O.compare(O.F32, got, want, 10.0)
        assert ok and mx == 0.0, mx


TYPE_PAIRS = [(O.F16, O.F32), (O.F16, O.F16), (O.BF16, O.F32), (O.BF16, O.BF16), (O.E4M3, O.F32), (O.I8, O.I32), (O.F32, O.F32),
              (O.F64, O.F64)]


@pytest.mark.parametrize("in_t,out_t", TYPE_PAIRS)
@pytest.mark.parametrize("la,lb", list(itertools.product([O.ROW, O.COL], repeat=2)))
def test_simple_kernel_all_layouts_reference_inputs_exact(in_t, out_t, la, lb):
    # the reference's integer-valued inputs (test/device/common.hpp:203-220): GPU == CPU exactly
    m, n, k = 64, 96, 128
    a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
    for lc, ld in ((O.ROW, O.COL), (O.COL, O.ROW)):
        c = O.fill_ref(out_t, m, n, lc)
        want = O.gemm(in_t, out_t, la, lb, lc, ld, m, n, k, a, b, c, 2.0, 2.0)
        got = _run(in_t, out_t, la, lb, lc, ld, m, n, k, a, b, c, 2.0, 2.0, R.KERNEL_SIMPLE)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("in_t,out_t", TYPE_PAIRS)
def test_simple_kernel_random_inputs_and_block16(in_t, out_t):
    # 48 x 80: only the 16 x 16 block fits; non-square, ragged against the workgroup tile
    m, n, k = 48, 80, 96
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=5)
    want = O.gemm(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, -1.0)
    got = _run(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, -1.0, R.KERNEL_SIMPLE)
    w32 = None
    if out_t in (O.F16, O.BF16):
        c32 = O.storage_to_f32(c, out_t)
        w32 = O.gemm(in_t, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c32, 2.0, -1.0)
    _check(in_t, out_t, got, want, w32)


TILED_LAYOUTS_16 = list(itertools.product([O.ROW, O.COL], repeat=2))
TILE_SELECTORS = {"tiled": R.KERNEL_TILED, "tiled_128": R.KERNEL_TILED_128}  # 256 x 256 and 128 x 128 macro tiles


@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.BF16, O.F32)])
@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_tiled_kernel_16bit_layouts(in_t, out_t, la, lb, ldl):
    m, n, k = 512, 256, 384
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=11)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, 2.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, 2.0, R.KERNEL_TILED)
    w32 = None
    if out_t != O.F32:
        w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), 2.0, 2.0)
    _check(in_t, out_t, got, want, w32)
    # reference-pattern inputs: exact
    a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_TILED)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.BF16, O.F32)])
@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_small_tile_kernel_16bit_layouts(in_t, out_t, la, lb, ldl):
    # the 128 x 128 macro tile (wave tile 4 x 4 blocks): 3 x 2 tiles
    m, n, k = 384, 256, 384
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=12)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, 2.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, 2.0, R.KERNEL_TILED_128)
    w32 = None
    if out_t != O.F32:
        w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), 2.0, 2.0)
    _check(in_t, out_t, got, want, w32)
    a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_TILED_128)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("kernel", ["tiled", "tiled_128"])
def test_tiled_kernel_16bit_one_hot_operands(la, lb, kernel):
    # one non-zero in A and one in B: exactly one element of D, for both tile sizes and every orientation
    m, n, k = 256, 256, 128
    rng = np.random.default_rng(6)
    sel = TILE_SELECTORS[kernel]
    for _ in range(6):
        i, j, h = int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(k))
        a = np.zeros(m * k, np.float16)
        b = np.zeros(k * n, np.float16)
        a[i * k + h if la == O.ROW else h * m + i] = 3
        b[h * n + j if lb == O.ROW else j * k + h] = 5
        got = _run(O.F16, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a.view(np.uint16), b.view(np.uint16), None, 1.0, 0.0, sel)
        want = np.zeros((m, n), np.float32)
        want[i, j] = 15
        assert np.array_equal(got.reshape(m, n), want), (i, j, h)


@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.BF16, O.F32)])
@pytest.mark.parametrize("la,lb", [(O.COL, O.ROW), (O.ROW, O.COL)])
@pytest.mark.parametrize("m,n,k", [(272, 304, 256), (16, 528, 128), (1008, 16, 384), (144, 112, 640)])
def test_small_tile_kernel_edge_tiles_and_stage_counts(in_t, out_t, la, lb, m, n, k):
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=75 + m)
    for alpha, beta in ((1.0, 0.0), (2.0, 2.0)):
        cc = None if beta == 0.0 else c
        want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, cc, alpha, beta)
        got = _run(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, cc, alpha, beta, R.KERNEL_TILED_128)
        w32 = None
        if out_t != O.F32:
            c32 = None if cc is None else O.storage_to_f32(cc, out_t)
            w32 = O.gemm(in_t, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, c32, alpha, beta)
        _check(in_t, out_t, got, want, w32)


def test_auto_takes_the_small_tile_for_few_tile_problems():
    # 1024 x 768 has 12 tiles of 256 x 256 on 256 CUs: AUTO must resolve to the 128 x 128 tile and agree with the oracle
    m, n, k = 1024, 768, 512
    a, b, _ = _inputs(O.F16, O.F16, m, n, k, seed=77)
    g = R.gemm_args(R.F16, R.F16, m, n, k, 0x1000, 0x2000, None, 0x3000, 1.0, 0.0, O.COL, O.ROW, O.ROW, O.ROW)
    assert R.gemm_query(g).macro_tile_m == 128
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_AUTO)
    w32 = O.gemm(O.F16, O.F32, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    _check(O.F16, O.F16, got, want, w32)


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.F16, O.F16), (O.E4M3, O.F32), (O.BF16, O.F32)])
@pytest.mark.parametrize("m,n,kbytes,la,lb,ldl", [(4352, 4352, 1280, O.COL, O.ROW, O.ROW),   # 289 tiles: 256 + 33
                                                  (4368, 4112, 1168, O.ROW, O.COL, O.ROW),   # partial edge tiles: 18 x 17
                                                  (768, 22016, 1216, O.ROW, O.ROW, O.COL),   # 3 x 86 = 258: 2 left over
                                                  (5120, 4880, 1200, O.COL, O.COL, O.COL)])  # 20 x 20 = 400: 144 left, one launch
def test_auto_mixed_tiling_covers_every_tile_once(in_t, out_t, m, n, kbytes, la, lb, ldl):
    """AUTO on a problem whose last round of 256 x 256 tiles would fill at most half of the CUs: whole rounds on the
    large tile, the rest on 128 x 128 tiles in a second launch.  (K is more than 8 stages of 128 bytes: below that AUTO
    weighs the two tilings by their fixed costs and may take the small tile throughout.)  D starts as 0xFF bytes; four
    complete rows of every row of tiles are held against the oracle, and a tile nobody wrote shows as NaN, or in the
    checksum of checksums for int8."""
    k = kbytes // O.NP_STORAGE[in_t]().itemsize
    cus = R.device_info().compute_units
    total = -(-m // 256) * -(-n // 256)
    rest = total % cus
    mixed = total > cus and 0 < rest <= cus // 2
    a, b, _ = _inputs(in_t, out_t, m, n, k, seed=88)
    g = R.gemm_args(in_t, out_t, m, n, k, 0x1000, 0x2000, None, 0x4000, 1.0, 0.0, la, lb, ldl, ldl)
    plan = R.gemm_query(g)
    assert plan.macro_tile_m == 256 and plan.grid_x == (total - (rest if mixed else 0) + 7) // 8 * 8
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_AUTO)
    got = got.reshape(m, n) if ldl == O.ROW else got.reshape(n, m).T
    rows = sorted({min(m - 1, 256 * t + o) for t in range(-(-m // 256)) for o in (0, 127, 128, 255)})
    want = O.gemm_rows(in_t, out_t, la, lb, m, n, k, a, b, rows)
    if in_t == O.I8:
        assert np.array_equal(got[rows], want)
        A, B = O.as_matrix(a, m, k, la).astype(np.int64), O.as_matrix(b, k, n, lb).astype(np.int64)
        assert int(got.astype(np.int64).sum()) == int(A.sum(axis=0) @ B.sum(axis=1))
    else:
        w32 = O.gemm_rows(in_t, O.F32, la, lb, m, n, k, a, b, rows) if out_t != O.F32 else None
        _check(in_t, out_t, np.ascontiguousarray(got[rows]).ravel(), want.ravel(), None if w32 is None else w32.ravel())
        full = got if out_t == O.F32 else O.storage_to_f32(np.ascontiguousarray(got).ravel(), out_t)
        assert np.all(np.isfinite(full))


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32)])
@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_8bit_layouts(in_t, out_t, la, lb, ldl, kernel):
    # K-contiguous operands are read whole, M/N-contiguous ones through the transposing LDS read
    m, n, k = 256, 512, 768
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=21)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 1.0, 1.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 1.0, 1.0, TILE_SELECTORS[kernel])
    _check(in_t, out_t, got, want)
    # reference-pattern inputs: exact
    a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, TILE_SELECTORS[kernel])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_8bit_one_hot_operands(la, lb, kernel):
    # A single non-zero in A and in B lands in exactly one element of D only if every (row, k) and
    # (k, column) of the operand tiles reaches the matrix instruction it belongs to: probes the
    # global -> LDS placement and the (transposing) LDS reads of both orientations.
    m, n, k = 256, 256, 256
    rng = np.random.default_rng(5)
    for _ in range(6):
        i, j, h = int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(k))
        a = np.zeros(m * k, np.int8)
        b = np.zeros(k * n, np.int8)
        a[i * k + h if la == O.ROW else h * m + i] = 3
        b[h * n + j if lb == O.ROW else j * k + h] = 5
        got = _run(O.I8, O.I32, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, TILE_SELECTORS[kernel]).reshape(m, n)
        want = np.zeros((m, n), np.int32)
        want[i, j] = 15
        assert np.array_equal(got, want), (i, j, h)


# the sizes the reference's GEMM suites validate (test/gemm/gemm_common_test_params.hpp:336-348) with its
# alpha = beta = 2 (:363-373)
REFERENCE_VALIDATED_SIZES = [(64, 64, 1024), (32, 64, 1024), (64, 32, 1024), (256, 256, 1024), (2048, 64, 1024),
                             (64, 2048, 1024), (512, 512, 512)]


@pytest.mark.parametrize("m,n,k", REFERENCE_VALIDATED_SIZES)
@pytest.mark.parametrize("kernel", ["auto", "tiled"])
def test_reference_validated_problem_sizes(m, n, k, kernel):
    sel = R.KERNEL_AUTO if kernel == "auto" else R.KERNEL_TILED
    for in_t, out_t in ((O.F16, O.F32), (O.I8, O.I32)):
        a, b, c = _inputs(in_t, out_t, m, n, k, seed=5)
        want = O.gemm(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
        got = _run(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0, sel)
        _check(in_t, out_t, got, want)


RAGGED_SHAPES = [(272, 304, 256), (16, 528, 128), (1008, 16, 384), (496, 752, 128)]


@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.BF16, O.F32)])
@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("m,n,k", RAGGED_SHAPES)
def test_tiled_kernel_16bit_edge_tiles(in_t, out_t, la, lb, m, n, k):
    # m and n multiples of 16 that do not fill 256 x 256 tiles: edge tiles read clamped rows / chunks
    # and store only what lies inside D; beta != 0 exercises the guarded C loads as well
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=70 + m)
    for alpha, beta in ((1.0, 0.0), (2.0, 2.0)):
        cc = None if beta == 0.0 else c
        want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, cc, alpha, beta)
        got = _run(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, cc, alpha, beta, R.KERNEL_TILED)
        w32 = None
        if out_t != O.F32:
            c32 = None if cc is None else O.storage_to_f32(cc, out_t)
            w32 = O.gemm(in_t, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, c32, alpha, beta)
        _check(in_t, out_t, got, want, w32)


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32)])
@pytest.mark.parametrize("la,lb,ldl", [(O.ROW, O.COL, O.ROW), (O.ROW, O.COL, O.COL), (O.COL, O.ROW, O.ROW),
                                       (O.COL, O.COL, O.COL), (O.ROW, O.ROW, O.ROW)])
@pytest.mark.parametrize("m,n,k", RAGGED_SHAPES)
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_8bit_edge_tiles(in_t, out_t, la, lb, ldl, m, n, k, kernel):
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=80 + n)
    for alpha, beta in ((1.0, 0.0), (1.0, 1.0)):
        cc = None if beta == 0.0 else c
        want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta)
        got = _run(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta, TILE_SELECTORS[kernel])
        _check(in_t, out_t, got, want)


def test_edge_tiles_leave_neighbouring_memory_untouched():
    # D with a padded leading dimension: the columns between n and ldd must keep their prefill
    m, n, k, ldd = 272, 304, 128, 320
    a, b, _ = _inputs(O.F16, O.F32, m, n, k, seed=91)
    da, db = to_device(a), to_device(b)
    dd = device_filled(m * ldd, np.float32, 0xFF)
    R.gemm(R.F16, R.F32, m, n, k, da, db, None, dd, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, ldd=ldd, kernel=R.KERNEL_TILED)
    got = to_host(dd, np.float32).reshape(m, ldd)
    want = O.gemm(O.F16, O.F32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0).reshape(m, n)
    _check(O.F16, O.F32, np.ascontiguousarray(got[:, :n]).ravel(), want.ravel())
    assert np.all(np.ascontiguousarray(got[:, n:]).view(np.uint32) == 0xFFFFFFFF)


@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F32), (O.BF16, O.BF16)])
@pytest.mark.parametrize("la,lb", [(O.COL, O.ROW), (O.ROW, O.COL)])
@pytest.mark.parametrize("k", [128, 256, 640])
def test_tiled_kernel_16bit_stage_counts(in_t, out_t, la, lb, k):
    # the 16-bit kernel runs K stages of 64 in pairs and clamps its refills past the last stage:
    # the smallest K (one pair), two pairs and an odd number of pairs
    m, n = 256, 256
    a, b, _ = _inputs(in_t, out_t, m, n, k, seed=60 + k)
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_TILED)
    w32 = None
    if out_t != O.F32:
        w32 = O.gemm(in_t, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    _check(in_t, out_t, got, want, w32)


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.E4M3, O.F32)])
@pytest.mark.parametrize("la,lb", [(O.ROW, O.COL), (O.COL, O.ROW)])
@pytest.mark.parametrize("stages", [1, 2, 3, 4, 5, 6, 7, 11, 13])
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_8bit_stage_counts(in_t, out_t, la, lb, stages, kernel):
    # The 8-bit kernel rotates five LDS buffers with period six; cover every remainder of the K
    # stage count, including a single stage and counts beyond one period.
    m, n, k = 256, 256, 128 * stages
    a, b, _ = _inputs(in_t, out_t, m, n, k, seed=40 + stages)
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, TILE_SELECTORS[kernel])
    _check(in_t, out_t, got, want)


@pytest.mark.parametrize("in_t,out_t,ks", [(O.F16, O.F32, (8, 72, 136, 328)), (O.BF16, O.BF16, (24, 200)),
                                           (O.I8, O.I32, (16, 144, 400, 784)), (O.E4M3, O.F32, (48, 272))])
@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_k_tails(in_t, out_t, ks, la, lb, kernel):
    # K that does not fill the last 128-byte stage (16-bit: the last pair of stages): the loads complete it
    # with zeros, for K-contiguous operands per lane, for M/N-contiguous ones through the buffer's end.
    # The operands sit in the middle of a larger allocation filled with a value that would show up in D.
    m, n = 272, 144
    for k in ks:
        a, b, c = _inputs(in_t, out_t, m, n, k, seed=300 + k)
        want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 1.0, 1.0)
        poison = np.full(4096, 0x40 if a.dtype.itemsize == 1 else 0x4000, dtype=a.dtype)  # 2.0 in e4m3 / f16 / bf16, 64 as int8
        da = to_device(np.concatenate([poison, a, poison]))
        db = to_device(np.concatenate([poison, b, poison]))
        dc = to_device(c)
        dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
        R.gemm(in_t, out_t, m, n, k, da[4096:], db[4096:], dc, dd, 1.0, 1.0, la, lb, O.ROW, O.ROW, kernel=TILE_SELECTORS[kernel])
        got = to_host(dd, O.NP_STORAGE[out_t])
        w32 = None
        if out_t not in (O.F32, O.I32):
            w32 = O.gemm(in_t, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, O.storage_to_f32(c, out_t), 1.0, 1.0)
        _check(in_t, out_t, got, want, w32)


@pytest.mark.parametrize("kernel", ["simple", "tiled", "tiled_128"])
@pytest.mark.parametrize("la,lb,ldl", [(O.ROW, O.COL, O.ROW), (O.COL, O.ROW, O.COL), (O.ROW, O.ROW, O.ROW)])
def test_int8_to_int8_output(kernel, la, lb, ldl):
    # the reference's (int8, int8, int32) type tuple (test/gemm/gemm_common_test_params.hpp:52): int8 C and D,
    # int32 arithmetic, the result narrowed to its low byte; bit-exact, edge tiles and a K tail included
    sel = {"simple": R.KERNEL_SIMPLE, **TILE_SELECTORS}[kernel]
    for m, n, k in ((256, 384, 512), (272, 144, 160)):
        a, b = O.uniform_int8(91, m * k), O.uniform_int8(92, k * n)
        c = O.uniform_int8(93, m * n)
        for alpha, beta in ((1.0, 0.0), (3.0, -2.0)):
            cc = None if beta == 0.0 else c
            want = O.gemm(O.I8, O.I8, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta)
            got = _run(O.I8, O.I8, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta, sel)
            assert np.array_equal(got, want), (m, n, k, alpha, beta)


@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_f32_layouts_edges_and_k_tails(la, lb, ldl, kernel):
    # f32 on v_mfma_f32_16x16x4_f32 through the five-buffer body: K-contiguous operands arrive as 128-bit LDS reads,
    # M/N-contiguous ones element by element (there is no 32-bit transposing read); full tiles, edge tiles, K tails
    for m, n, k in ((256, 512, 160), (272, 144, 36), (16, 400, 260)):
        a, b, c = _inputs(O.F32, O.F32, m, n, k, seed=500 + k)
        want = O.gemm(O.F32, O.F32, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, -1.0)
        got = _run(O.F32, O.F32, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, -1.0, TILE_SELECTORS[kernel])
        _check(O.F32, O.F32, got, want)
        # integer-valued inputs: every partial sum is exact, so the result is bit-identical to the oracle's
        a, b = O.fill_ref(O.F32, m, k, la), O.fill_ref(O.F32, k, n, lb)
        want = O.gemm(O.F32, O.F32, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
        got = _run(O.F32, O.F32, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, TILE_SELECTORS[kernel])
        assert np.array_equal(got, want), (m, n, k)


@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_tiled_kernel_f64_layouts_edges_and_k_tails(la, lb, ldl):
    # f64 on v_mfma_f64_16x16x4_f64, 128 x 128 macro tile only (an accumulator block is 8 registers); the
    # accumulator elements of a lane are 4 columns apart, unlike every other type
    for m, n, k in ((256, 384, 48), (272, 144, 18), (16, 400, 130)):
        a, b, c = _inputs(O.F64, O.F64, m, n, k, seed=600 + k)
        if k <= 48:  # random operands: the reference's 10 eps(f64) holds for short sums in any order
            want = O.gemm(O.F64, O.F64, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, -1.0)
            got = _run(O.F64, O.F64, la, lb, ldl, ldl, m, n, k, a, b, c, 2.0, -1.0, R.KERNEL_AUTO)
            _check(O.F64, O.F64, got, want)
        a, b = O.fill_ref(O.F64, m, k, la), O.fill_ref(O.F64, k, n, lb)
        ci = np.round(c * 8.0)
        for alpha, beta in ((1.0, 0.0), (2.0, -1.0)):
            cc = None if beta == 0.0 else ci
            want = O.gemm(O.F64, O.F64, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta)
            got = _run(O.F64, O.F64, la, lb, ldl, ldl, m, n, k, a, b, cc, alpha, beta, R.KERNEL_TILED_128)
            assert np.array_equal(got, want), (m, n, k, alpha, beta)
    g = R.gemm_args(R.F64, R.F64, 256, 256, 64, 0x1000, 0x2000, None, 0x3000, 1.0, 0.0, la, lb, ldl, ldl)
    plan = R.gemm_query(g)
    assert plan.kernel == R.KERNEL_TILED and plan.macro_tile_m == 128 and plan.macro_tile_k == 16
    with pytest.raises(R.R355Error) as e:
        _run(O.F64, O.F64, la, lb, ldl, ldl, 256, 256, 64, a[:256 * 64], b[:64 * 256], None, 1.0, 0.0, R.KERNEL_TILED)
    assert e.value.code == -2


@pytest.mark.parametrize("kernel", ["simple", "tiled_128"])
def test_f64_scalars_keep_double_precision(kernel):
    # the reference passes ComputeT alpha, beta (test/gemm/gemm_kernel_base.hpp:112-113): double for f64.  1/3 and -1/7
    # are not representable in f32; rounding them on the way would move the result by ~1e-8 relative, far above the
    # reference's 10 eps(f64) (the negative control below shows the bar sees that)
    sel = {"simple": R.KERNEL_SIMPLE, **TILE_SELECTORS}[kernel]
    m, n, k = 144, 272, 48
    alpha, beta = 1.0 / 3.0, -1.0 / 7.0
    a, b, c = _inputs(O.F64, O.F64, m, n, k, seed=77)
    want = O.gemm(O.F64, O.F64, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, alpha, beta)
    got = _run(O.F64, O.F64, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, alpha, beta, sel)
    ok, mx = O.compare(O.F64, got, want, 10.0)
    assert ok, mx
    rounded = O.gemm(O.F64, O.F64, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, float(np.float32(alpha)), float(np.float32(beta)))
    assert not O.compare(O.F64, rounded, want, 10.0)[0]


@pytest.mark.parametrize("kernel", ["simple", "tiled", "tiled_128"])
def test_int8_scalars_beyond_f32_integers(kernel):
    # int32 alpha / beta (ComputeT = int32 for int8 inputs) above 2^24 are not f32 integers; int32 arithmetic wraps
    sel = {"simple": R.KERNEL_SIMPLE, **TILE_SELECTORS}[kernel]
    m, n, k = 272, 144, 160
    alpha, beta = float(2 ** 25 + 1), float(-(2 ** 24 + 3))
    a, b, c = _inputs(O.I8, O.I32, m, n, k, seed=78)
    want = O.gemm(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, alpha, beta)
    got = _run(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, alpha, beta, sel)
    assert np.array_equal(got, want)
    # closed form on the host, independent of the oracle: wrap-around int32 arithmetic
    acc = a.reshape(m, k).astype(np.int64) @ b.reshape(n, k).T.astype(np.int64)
    ref = ((2 ** 25 + 1) * acc - (2 ** 24 + 3) * c.reshape(m, n).astype(np.int64)) & 0xFFFFFFFF
    assert np.array_equal(got.view(np.uint32).reshape(m, n), ref.astype(np.uint32))


@pytest.mark.parametrize("la,lb", [(O.ROW, O.COL), (O.COL, O.ROW)])
def test_f64_random_operands_long_k(la, lb):
    # Random f64 operands over a long K: the matrix instructions sum in another order than the oracle's sequential loop,
    # so the two are compared with the exact product (80-bit accumulation on the host) under the forward error bound that
    # holds for any summation order, |fl(sum) - sum| <= gamma_k * sum |a_i b_i|, gamma_k = k u / (1 - k u), u = 2^-53.
    m, n, k = 144, 128, 2064
    a, b, _ = _inputs(O.F64, O.F64, m, n, k, seed=79)
    got = _run(O.F64, O.F64, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_AUTO).reshape(m, n)
    A = a.reshape(m, k) if la == O.ROW else a.reshape(k, m).T
    B = b.reshape(k, n) if lb == O.ROW else b.reshape(n, k).T
    exact = A.astype(np.longdouble) @ B.astype(np.longdouble)
    bound = (k * 2.0 ** -53 / (1 - k * 2.0 ** -53)) * (np.abs(A) @ np.abs(B))
    assert np.all(np.abs(got.astype(np.longdouble) - exact) <= bound)
    want = O.gemm(O.F64, O.F64, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0).reshape(m, n)
    assert np.all(np.abs(want.astype(np.longdouble) - exact) <= bound)
    # and the bound has teeth: the typical distance is far below it, an index error is far above
    assert np.max(np.abs(got - want)) < 1e-12 < np.max(np.abs(np.roll(got, 1, axis=1) - want))


@pytest.mark.parametrize("la,lb", TILED_LAYOUTS_16)
@pytest.mark.parametrize("kernel", list(TILE_SELECTORS))
def test_tiled_kernel_f32_one_hot_operands(la, lb, kernel):
    m, n, k = 256, 256, 64
    rng = np.random.default_rng(8)
    for _ in range(6):
        i, j, h = int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(k))
        a = np.zeros(m * k, np.float32)
        b = np.zeros(k * n, np.float32)
        a[i * k + h if la == O.ROW else h * m + i] = 3
        b[h * n + j if lb == O.ROW else j * k + h] = 5
        got = _run(O.F32, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, TILE_SELECTORS[kernel]).reshape(m, n)
        want = np.zeros((m, n), np.float32)
        want[i, j] = 15
        assert np.array_equal(got, want), (i, j, h)


def _e5m2_operand(seed, n):
    """n finite e5m2 codes of magnitude 2^-4 .. 2 (random sign, exponent 11 .. 15, mantissa)."""
    rng = np.random.default_rng(seed)
    return ((rng.integers(0, 2, n) << 7) | (rng.integers(11, 16, n) << 2) | rng.integers(0, 4, n)).astype(np.uint8)


@pytest.mark.parametrize("kernel", ["simple", "tiled", "tiled_128"])
@pytest.mark.parametrize("la,lb,ldl", [(O.ROW, O.COL, O.ROW), (O.COL, O.ROW, O.COL), (O.ROW, O.ROW, O.ROW), (O.COL, O.COL, O.ROW)])
def test_e5m2_gemm(kernel, la, lb, ldl):
    # OCP e5m2 operands (the reference's bfloat8_t tuple, test/gemm/gemm_common_test_params.hpp:73-87), f32 result:
    # v_mfma_f32_16x16x128_f8f6f4 with both format fields set to e5m2 in the macro-tile kernels,
    # v_mfma_f32_*_bf8_bf8 behind the fragment API in the block-per-wave one
    sel = {"simple": R.KERNEL_SIMPLE, **TILE_SELECTORS}[kernel]
    for m, n, k in ((256, 384, 512), (272, 144, 160)):
        a, b = _e5m2_operand(31, m * k), _e5m2_operand(32, k * n)
        c = O.uniform_pm1(33, m * n)
        want = O.gemm(O.E5M2, O.F32, la, lb, ldl, ldl, m, n, k, a, b, c, 1.0, 1.0)
        got = _run(O.E5M2, O.F32, la, lb, ldl, ldl, m, n, k, a, b, c, 1.0, 1.0, sel)
        assert _max_rel(O.F32, got, want) <= 1e-2, (m, n, k)
    # powers of two only: every product and every partial sum is exact, the result must match bit for bit
    m, n, k = 256, 256, 256
    rng = np.random.default_rng(34)
    a = ((rng.integers(0, 2, m * k) << 7) | (rng.integers(13, 17, m * k) << 2)).astype(np.uint8)
    b = ((rng.integers(0, 2, k * n) << 7) | (rng.integers(13, 17, k * n) << 2)).astype(np.uint8)
    want = O.gemm(O.E5M2, O.F32, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(O.E5M2, O.F32, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0, sel)
    assert np.array_equal(got, want)


def test_tiled_kernel_many_tiles_xcd_mapping():
    # 5 x 3 tiles: a tile count that is not a multiple of 8 and a partial row group
    m, n, k = 1280, 768, 256
    a, b, _ = _inputs(O.I8, O.I32, m, n, k, seed=31)
    want = O.gemm(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_TILED)
    assert np.array_equal(got, want)


def test_auto_falls_back_and_bad_sizes_error():
    m, n, k = 96, 64, 64
    a, b, _ = _inputs(O.F16, O.F16, m, n, k)
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got = _run(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0, R.KERNEL_AUTO)
    _check(O.F16, O.F16, got, want)
    with pytest.raises(R.R355Error) as e:
        _run(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, 100, 64, 64, a, b, None, 1.0, 0.0, R.KERNEL_AUTO)
    assert e.value.code == -3


@pytest.mark.parametrize("in_t,out_t,la,lb", [(O.F16, O.F16, O.COL, O.ROW), (O.BF16, O.BF16, O.COL, O.ROW),
                                               (O.I8, O.I32, O.ROW, O.COL), (O.E4M3, O.F32, O.ROW, O.COL),
                                               (O.I8, O.I32, O.COL, O.ROW)])
def test_full_size_8192_sampled_rows(in_t, out_t, la, lb):
    # benchmark configurations 2 and 3 at full size.  Each element of the oracle depends only on its own row
    # of A and column of B, so complete rows computed by the oracle are exactly its values.
    import torch

    m = n = k = 8192
    if in_t == O.I8:
        a, b = O.uniform_int8(1, m * k), O.uniform_int8(2, k * n)
    else:
        src = O.normal if in_t == O.E4M3 else O.uniform_pm1
        a, b = O.f32_to_storage(src(1, m * k), in_t), O.f32_to_storage(src(2, k * n), in_t)
    da, db = to_device(a), to_device(b)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    R.gemm(in_t, out_t, m, n, k, da, db, None, dd, 1.0, 0.0, la, lb, O.ROW, O.ROW, kernel=R.KERNEL_TILED)
    got = to_host(dd, O.NP_STORAGE[out_t]).reshape(m, n)
    rows = np.array([0, 1, 255, 256, 4095, 5000, 8191, 7777], dtype=np.uint32)
    want = O.gemm_rows(in_t, out_t, la, lb, m, n, k, a, b, rows)
    if in_t == O.I8:
        assert np.array_equal(got[rows], want)
        # checksum of checksums over the whole matrix: sum(D) = (1^T A)(B 1), exact in int64
        A = O.as_matrix(a, m, k, la).astype(np.int64)
        B = O.as_matrix(b, k, n, lb).astype(np.int64)
        assert int(got.astype(np.int64).sum()) == int(A.sum(axis=0) @ B.sum(axis=1))
    else:
        w32 = O.gemm_rows(in_t, O.F32, la, lb, m, n, k, a, b, rows) if out_t != O.F32 else None
        _check(in_t, out_t, got[rows].ravel(), want.ravel(), None if w32 is None else w32.ravel())
        # size-independent property on the full matrix: column sums against a float64 matvec
        A = O.storage_to_f32(O.as_matrix(a, m, k, la), in_t).astype(np.float64)
        B = O.storage_to_f32(O.as_matrix(b, k, n, lb), in_t).astype(np.float64)
        colsum = A.sum(axis=0) @ B
        gs = O.storage_to_f32(got, out_t).astype(np.float64).sum(axis=0)
        scale = np.abs(A).sum(axis=0) @ np.abs(B)
        assert np.max(np.abs(gs - colsum) / scale) < (2e-3 if in_t != O.E4M3 else 1e-3)
    del da, db, dd
    torch.cuda.empty_cache()


@pytest.mark.parametrize("in_t,out_t,la,lb,ldl,kernel", [(O.F16, O.F16, O.COL, O.ROW, O.ROW, "tiled"), (O.I8, O.I32, O.ROW, O.COL, O.ROW, "tiled"),
                                                          (O.F16, O.F16, O.ROW, O.COL, O.COL, "tiled"), (O.F16, O.F32, O.ROW, O.COL, O.ROW, "simple")])
def test_output_beyond_2_to_the_32_elements(in_t, out_t, la, lb, ldl, kernel):
    # D has 65792 x 65536 = 2^32 + 2^24 elements (8.6 to 17 GB): element offsets into D do not fit 32 bits.  Complete rows
    # (columns of a col-major D) on both sides of the 2^32 boundary against the oracle's rows.
    import torch

    m, n, k = 65536 + 256, 65536, 64
    if ldl == O.COL:
        m, n = n, m  # the long dimension is the one D's lines run along
    if in_t == O.I8:
        a, b = O.uniform_int8(5, m * k), O.uniform_int8(6, k * n)
    else:
        a, b = O.f32_to_storage(O.uniform_pm1(5, m * k), in_t), O.f32_to_storage(O.uniform_pm1(6, k * n), in_t)
    da, db = to_device(a), to_device(b)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    sel = {"tiled": R.KERNEL_TILED, "simple": R.KERNEL_SIMPLE}[kernel]
    R.gemm(in_t, out_t, m, n, k, da, db, None, dd, 1.0, 0.0, la, lb, ldl, ldl, kernel=sel)
    torch.cuda.synchronize()
    es = np.dtype(O.NP_STORAGE[out_t]).itemsize
    if ldl == O.ROW:
        lines = np.array([0, 1, 32767, 65535, 65536, 65537, m - 1], dtype=np.uint32)  # rows of D; 65536 starts at element 2^32
        want = O.gemm_rows(in_t, out_t, la, lb, m, n, k, a, b, lines)
        length = n
    else:
        # columns of a col-major D are rows of D^T = B^T A^T: the oracle's rows with the operands exchanged
        lines = np.array([0, 1, 32767, 65535, 65536, 65537, n - 1], dtype=np.uint32)
        other = {O.ROW: O.COL, O.COL: O.ROW}
        want = O.gemm_rows(in_t, out_t, other[lb], other[la], n, m, k, b, a, lines)
        length = m
    for i, line in enumerate(lines):
        got = dd[int(line) * length * es:(int(line) + 1) * length * es].cpu().numpy().view(O.NP_STORAGE[out_t])
        if in_t == O.I8:
            assert np.array_equal(got, want[i]), line
        else:
            _check(in_t, out_t, got, want[i].ravel())
    del da, db, dd
    torch.cuda.empty_cache()


def _embed(flat, rows, cols, layout, ld, fill):
    """Packed rows x cols matrix (layout) -> storage with leading dimension ld, padding = fill."""
    major, minor = (rows, cols) if layout == O.ROW else (cols, rows)
    out = np.full(major * ld, fill, dtype=flat.dtype)
    out.reshape(major, ld)[:, :minor] = flat.reshape(major, minor)
    return out


@pytest.mark.parametrize("kernel", ["tiled", "simple"])
@pytest.mark.parametrize("in_t,out_t,la,lb,ldl", [(O.F16, O.F16, O.COL, O.ROW, O.ROW), (O.F16, O.F32, O.ROW, O.COL, O.COL),
                                                  (O.BF16, O.BF16, O.ROW, O.ROW, O.ROW), (O.I8, O.I32, O.ROW, O.COL, O.ROW),
                                                  (O.E4M3, O.F32, O.ROW, O.COL, O.COL), (O.I8, O.I32, O.COL, O.ROW, O.ROW),
                                                  (O.E4M3, O.F32, O.COL, O.COL, O.ROW)])
def test_padded_leading_dimensions(kernel, in_t, out_t, la, lb, ldl):
    """Operands and result embedded in wider buffers (ld > extent): the reference kernels take lda..ldd
    (test/gemm/gemm_kernel_base.hpp:101-114); bytes outside the m x n block of D must stay untouched."""
    m, n, k = (256, 512, 512) if kernel == "tiled" else (96, 64, 128)
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=41)
    alpha, beta = (1.0, 1.0) if in_t in (O.I8, O.E4M3) else (2.0, -1.0)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, alpha, beta)
    es_in, es_out = a.dtype.itemsize, c.dtype.itemsize
    pad_in, pad_out = 48 // es_in * 2, 32 // es_out * 2  # keeps 16-byte alignment of every row / column
    lda = (k if la == O.ROW else m) + pad_in
    ldb = (n if lb == O.ROW else k) + pad_in
    ldc = (n if ldl == O.ROW else m) + pad_out
    ldd = ldc + pad_out
    canary = np.array([0xEE] * es_out, dtype=np.uint8).view(c.dtype)[0]
    ea, eb = _embed(a, m, k, la, lda, 1), _embed(b, k, n, lb, ldb, 1)
    ec = _embed(c, m, n, ldl, ldc, canary)
    da, db, dc = to_device(ea), to_device(eb), to_device(ec)
    major = m if ldl == O.ROW else n
    dd = device_filled(major * ldd, O.NP_STORAGE[out_t], 0xEE)
    R.gemm(in_t, out_t, m, n, k, da, db, dc, dd, alpha, beta, la, lb, ldl, ldl, lda=lda, ldb=ldb, ldc=ldc, ldd=ldd,
           kernel=R.KERNEL_TILED if kernel == "tiled" else R.KERNEL_SIMPLE)
    full = to_host(dd, O.NP_STORAGE[out_t]).reshape(major, ldd)
    minor = n if ldl == O.ROW else m
    assert np.all(full[:, minor:] == canary)
    got = np.ascontiguousarray(full[:, :minor]).ravel()
    w32 = None
    if out_t in (O.F16, O.BF16):
        w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), alpha, beta)
    _check(in_t, out_t, got, want, w32)


@pytest.mark.parametrize("kernel", ["tiled", "auto", "simple"])
@pytest.mark.parametrize("la", [O.ROW, O.COL])
@pytest.mark.parametrize("in_t", [O.I8, O.F16])
def test_operand_beyond_4_gib(in_t, la, kernel):
    """A is 4.6 GB, so byte offsets into it pass 2^32: for int8, rows past row 65536 of a row-major A (lda = k = 65536) or
    K rows past 32704 of a col-major one (lda = m = 131328); for f16 (values -3 .. 3, every sum exact in f32) half as many
    columns.  Complete rows of D from both sides of the boundary, and rows whose dot product runs across it, against the
    oracle on the same rows of A; the checksum of checksums covers the rest."""
    import torch

    es = 1 if in_t == O.I8 else 2
    if la == O.ROW:
        m, n, k = 70000, 64, 65536 // es
        rows = [0, 1, 65535, 65536, 65537, 69999]
    else:
        m, n, k = 131072 + 256, 64, 34816 // es
        rows = [0, 255, 256, 70001, 131071, 131327]
    g = torch.Generator(device="cuda").manual_seed(21)
    if in_t == O.I8:
        out_t, tdt = O.I32, torch.int32
        da = torch.randint(-128, 128, (m * k,), dtype=torch.int8, device="cuda", generator=g)
        db = torch.randint(-128, 128, (k * n,), dtype=torch.int8, device="cuda", generator=g)  # col-major: n columns of k
    else:
        out_t, tdt = O.F32, torch.float32
        da = torch.randint(-3, 4, (m * k,), dtype=torch.int8, device="cuda", generator=g).to(torch.float16)
        db = torch.randint(-3, 4, (k * n,), dtype=torch.int8, device="cuda", generator=g).to(torch.float16)
    dd = device_filled(m * n, np.int32, 0xEE)
    sel = {"tiled": R.KERNEL_TILED, "auto": R.KERNEL_AUTO, "simple": R.KERNEL_SIMPLE}[kernel]
    R.gemm(in_t, out_t, m, n, k, da, db, None, dd, 1.0, 0.0, la, O.COL, O.ROW, O.ROW, kernel=sel)
    torch.cuda.synchronize()
    A = da.view(m, k) if la == O.ROW else da.view(k, m).t()
    host = (lambda t: t.cpu().numpy()) if in_t == O.I8 else (lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16))
    a_rows = host(A[torch.tensor(rows, device="cuda")].contiguous())  # (len(rows), k), row-major
    want = O.gemm(in_t, out_t, O.ROW, O.COL, O.ROW, O.ROW, len(rows), n, k, a_rows.ravel(), host(db), None, 1.0, 0.0)
    got = dd.view(tdt).view(m, n)
    assert np.array_equal(got[torch.tensor(rows, device="cuda")].cpu().numpy(), want.reshape(len(rows), n))
    # sum(D) = (1^T A)(B 1), exact in int64
    col_sums = torch.zeros(k, dtype=torch.int64, device="cuda")
    step = 8192 if la == O.ROW else k
    for r0 in range(0, m if la == O.ROW else k, step):  # in slices: a widened copy of all of A would not fit beside it
        if la == O.ROW:
            col_sums += da.view(m, k)[r0:r0 + step].to(torch.int32).sum(dim=0, dtype=torch.int64)
        else:
            col_sums = da.view(k, m).to(torch.float32).sum(dim=1).to(torch.int64) if in_t == O.F16 else da.view(k, m).sum(dim=1, dtype=torch.int64)
    row_sums = db.view(n, k).to(torch.float32).sum(dim=0).to(torch.int64)
    assert int(got.to(torch.float64).sum().item()) == int((col_sums * row_sums).sum().item())
    del da, db, dd, A, got
    torch.cuda.empty_cache()


@pytest.mark.parametrize("kernel", ["tiled", "auto", "simple"])
@pytest.mark.parametrize("lb", [O.COL, O.ROW])
def test_b_operand_beyond_4_gib(lb, kernel):
    """The same for B: 4.6 GB of int8, columns past 65536 of a col-major B (ldb = k = 65536) or K rows past 32704 of a
    row-major one (ldb = n = 131328); complete columns of D against the oracle on the same columns of B."""
    import torch

    if lb == O.COL:
        m, n, k = 64, 70000, 65536
        cols = [0, 1, 65535, 65536, 65537, 69999]
    else:
        m, n, k = 64, 131072 + 256, 34816
        cols = [0, 255, 256, 70001, 131071, 131327]
    g = torch.Generator(device="cuda").manual_seed(22)
    da = torch.randint(-128, 128, (m * k,), dtype=torch.int8, device="cuda", generator=g)  # row-major: m rows of k
    db = torch.randint(-128, 128, (k * n,), dtype=torch.int8, device="cuda", generator=g)
    dd = device_filled(m * n, np.int32, 0xEE)
    sel = {"tiled": R.KERNEL_TILED, "auto": R.KERNEL_AUTO, "simple": R.KERNEL_SIMPLE}[kernel]
    R.gemm(O.I8, O.I32, m, n, k, da, db, None, dd, 1.0, 0.0, O.ROW, lb, O.ROW, O.ROW, kernel=sel)
    torch.cuda.synchronize()
    Bt = db.view(n, k) if lb == O.COL else db.view(k, n).t()  # (n, k): row j is column j of B
    b_cols = Bt[torch.tensor(cols, device="cuda")].contiguous().cpu().numpy()  # as a col-major k x len(cols) matrix
    want = O.gemm(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, len(cols), k, da.cpu().numpy(), b_cols.ravel(), None, 1.0, 0.0)
    got = dd.view(torch.int32).view(m, n)
    assert np.array_equal(got[:, torch.tensor(cols, device="cuda")].cpu().numpy(), want.reshape(m, len(cols)))
    col_sums = da.view(m, k).to(torch.int64).sum(dim=0)
    row_sums = Bt.to(torch.int32).sum(dim=0, dtype=torch.int64) if lb == O.COL else db.view(k, n).to(torch.int32).sum(dim=1, dtype=torch.int64)
    assert int(got.to(torch.int64).sum().item()) == int((col_sums * row_sums).sum().item())
    del da, db, dd, Bt, got
    torch.cuda.empty_cache()


@pytest.mark.parametrize("la,lb", [(O.COL, O.ROW), (O.ROW, O.COL), (O.ROW, O.ROW), (O.COL, O.COL)])
@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.BF16, O.F32)])
def test_deep_pipeline_16_bit(in_t, out_t, la, lb):
    """R355_KERNEL_TILED_DEEP: the 256 x 256 tile of the 16-bit types on the five-buffer K loop (what AUTO takes for operands
    beyond the memory-side cache, forced here at a size the oracle finishes quickly): partial edge tiles in both
    directions, a K tail, six stages and a remainder, padded leading dimensions, C read."""
    m, n, k = 16 * 37, 16 * 41, 64 * 7 + 24
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=71)
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, -1.0)
    lda, ldb = (k if la == O.ROW else m) + 8, (n if lb == O.ROW else k) + 16
    da, db, dc = to_device(_embed(a, m, k, la, lda, 1)), to_device(_embed(b, k, n, lb, ldb, 1)), to_device(c)
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xEE)
    args = R.gemm_args(in_t, out_t, m, n, k, da, db, dc, dd, 2.0, -1.0, la, lb, O.ROW, O.ROW, lda=lda, ldb=ldb, kernel=R.KERNEL_TILED_DEEP)
    plan = R.gemm_query(args)
    assert plan.kernel == R.KERNEL_TILED and plan.macro_tile_m == 256 and plan.lds_bytes == 5 * 32768
    R.gemm(in_t, out_t, m, n, k, da, db, dc, dd, 2.0, -1.0, la, lb, O.ROW, O.ROW, lda=lda, ldb=ldb, kernel=R.KERNEL_TILED_DEEP)
    got = to_host(dd, O.NP_STORAGE[out_t])
    w32 = None
    if out_t in (O.F16, O.BF16):
        w32 = O.gemm(in_t, O.F32, la, lb, O.ROW, O.ROW, m, n, k, a, b, O.storage_to_f32(c, out_t), 2.0, -1.0)
    _check(in_t, out_t, got, want, w32)
