"""GPU parity of split-K GEMM (128 x 128 tiles, several workgroups per tile along K, reduction kernel) against the
CPU oracle, through the C ABI.  The reference has no split-K; the results must meet the same bars as the single-pass
kernels (tests/test_gemm.py): int8 bit-exact, floating point within the per-type tolerance, exact on the reference's
integer-valued inputs (test/device/common.hpp:203-220), where every partial sum is exact in any order."""
import itertools

import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host
from test_gemm import _check, _inputs

pytestmark = pytest.mark.gpu

ACC_BYTES = {O.F64: 8}


def _plan(in_t, out_t, m, n, k, la, lb, ldl, workspace_bytes, kernel, beta=0.0):
    g = R.gemm_args(in_t, out_t, m, n, k, 0x1000, 0x2000, 0x3000 if beta else None, 0x4000, 1.0, beta, la, lb, ldl, ldl,
                    kernel=kernel, workspace=None, workspace_bytes=workspace_bytes)  # sizing needs no pointer
    return R.gemm_query(g)


def _run_split(in_t, out_t, la, lb, ldl, m, n, k, a, b, c, alpha, beta, kernel=R.KERNEL_TILED_128_SPLITK, slack=4096, fill=0xFF):
    """Runs with a workspace of exactly the bytes the plan asks for, followed by `slack` guard bytes; returns D and the plan."""
    plan = _plan(in_t, out_t, m, n, k, la, lb, ldl, 2 ** 62, kernel, beta)
    assert plan.split_k >= 2, plan.split_k
    assert plan.workspace_bytes == plan.split_k * m * n * ACC_BYTES.get(in_t, 4)
    assert plan.grid_y == plan.split_k and plan.macro_tile_m == 128
    need = int(plan.workspace_bytes)
    ws = device_filled(need + slack, np.uint8, fill)
    da, db = to_device(a), to_device(b)
    dc = to_device(c) if c is not None else None
    dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
    g = R.gemm_args(in_t, out_t, m, n, k, da, db, dc, dd, alpha, beta, la, lb, ldl, ldl, kernel=kernel, workspace=ws,
                    workspace_bytes=need)
    R._check(R.lib().r355_gemm(R.ctypes.byref(g), None))
    got = to_host(dd, O.NP_STORAGE[out_t])
    guard = to_host(ws, np.uint8)[need:]
    assert np.all(guard == fill), "split-K wrote beyond the workspace bytes the plan reports"
    return got, plan


def _k_for(in_t, stages, tail_chunks):
    """k (elements) spanning `stages` full stages of 128 bytes plus `tail_chunks` 16-byte chunks."""
    es = np.dtype(O.NP_STORAGE[in_t]).itemsize
    return (stages * 128 + tail_chunks * 16) // es


def _matrix(x, rows, cols, layout):
    return x.reshape(rows, cols) if layout == O.ROW else x.reshape(cols, rows).T


def _check_against_exact(in_t, m, n, k, la, lb, ldl, a, b, c, alpha, beta, got):
    u = 2.0 ** -24 if in_t == O.F32 else 2.0 ** -53
    A, B = _matrix(a, m, k, la).astype(np.longdouble), _matrix(b, k, n, lb).astype(np.longdouble)
    C, G = _matrix(c, m, n, ldl).astype(np.longdouble), _matrix(got, m, n, ldl).astype(np.longdouble)
    exact = alpha * (A @ B) + beta * C
    bound = (k + 4) * u * (abs(alpha) * (np.abs(A) @ np.abs(B)) + abs(beta) * np.abs(C))
    assert np.all(np.abs(G - exact) <= bound)
    # the bound sees an index error
    assert not np.all(np.abs(np.roll(G, 1, axis=1) - exact) <= bound)


TYPE_PAIRS = [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.BF16, O.F32), (O.E4M3, O.F32), (O.I8, O.I32), (O.I8, O.I8),
              (O.F32, O.F32), (O.F64, O.F64)]
LAYOUTS = list(itertools.product([O.ROW, O.COL], repeat=2))


@pytest.mark.parametrize("in_t,out_t", TYPE_PAIRS)
@pytest.mark.parametrize("la,lb", LAYOUTS)
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_split_k_types_layouts_edge_tiles_and_k_tail(in_t, out_t, la, lb, ldl):
    # 2 x 3 tiles of 128 x 128 with partial edge tiles; 37 stages and a tail of 3 chunks: 4 shares of 10, 10, 10, 8 stages
    m, n = 144, 272
    k = _k_for(in_t, 37, 3)
    if in_t == O.I8 and out_t == O.I8:
        a, b, c = O.uniform_int8(91, m * k), O.uniform_int8(92, k * n), O.uniform_int8(93, m * n)
    else:
        a, b, c = _inputs(in_t, out_t, m, n, k, seed=31)
    alpha, beta = (3.0, -2.0) if in_t == O.I8 else (2.0, 2.0)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, alpha, beta)
    got, plan = _run_split(in_t, out_t, la, lb, ldl, m, n, k, a, b, c, alpha, beta)
    assert plan.split_k == 4
    w32 = None
    if out_t in (O.F16, O.BF16):
        w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), alpha, beta)
    if in_t in (O.F32, O.F64):
        # long sums in the operand type itself: the kernel and the oracle's sequential loop both lie within the forward error
        # bound of any summation order around the exact result, (k + 4) u (|alpha| |A| |B| + |beta| |C|)
        _check_against_exact(in_t, m, n, k, la, lb, ldl, a, b, c, alpha, beta, got)
        _check_against_exact(in_t, m, n, k, la, lb, ldl, a, b, c, alpha, beta, want)
    else:
        _check(in_t, out_t, got, want, w32)
    if in_t != O.I8:
        # reference-pattern inputs: every partial sum exact, so equality (beta = 0: no C)
        a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
        want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, None, 1.0, 0.0)
        got, _ = _run_split(in_t, out_t, la, lb, ldl, m, n, k, a, b, None, 1.0, 0.0)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("in_t,out_t", [(O.I8, O.I32), (O.F16, O.F32), (O.E4M3, O.F32)])
@pytest.mark.parametrize("la,lb", [(O.ROW, O.COL), (O.COL, O.ROW)])
@pytest.mark.parametrize("stages,tail", [(16, 0), (16, 1), (17, 0), (23, 7), (31, 0), (33, 2), (63, 5), (100, 0)])
def test_split_k_share_boundaries(in_t, out_t, la, lb, stages, tail):
    # every K stage belongs to exactly one share, whatever the remainder: a one tile problem, operands that make a dropped or
    # doubled stage visible (int8: exact; floating point: the reference's integer pattern, exact as well)
    m, n = 128, 128
    k = _k_for(in_t, stages, tail)
    if in_t == O.I8:
        a, b, _ = _inputs(in_t, out_t, m, n, k, seed=stages)
    else:
        a, b = O.fill_ref(in_t, m, k, la), O.fill_ref(in_t, k, n, lb)
    want = O.gemm(in_t, out_t, la, lb, O.ROW, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    got, plan = _run_split(in_t, out_t, la, lb, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
    total = stages + (1 if tail else 0)
    share = -(-total // plan.split_k)
    assert (plan.split_k - 1) * share < total <= plan.split_k * share  # no empty share
    assert np.array_equal(got, want)


@pytest.mark.parametrize("la,lb", LAYOUTS)
def test_split_k_one_hot_operands(la, lb):
    # a single non-zero product a[i, h] * b[h, j]: lands in D[i, j] whichever share owns K index h
    m, n, k = 128, 256, 4096 + 48
    rng = np.random.default_rng(5)
    hs = [0, 127, 128, k - 1, k - 48] + [int(x) for x in rng.integers(k, size=5)]
    for h in hs:
        i, j = int(rng.integers(m)), int(rng.integers(n))
        a = np.zeros(m * k, np.int8)
        b = np.zeros(k * n, np.int8)
        a[i * k + h if la == O.ROW else h * m + i] = 3
        b[h * n + j if lb == O.ROW else j * k + h] = 5
        got, _ = _run_split(O.I8, O.I32, la, lb, O.ROW, m, n, k, a, b, None, 1.0, 0.0)
        want = np.zeros((m, n), np.int32)
        want[i, j] = 15
        assert np.array_equal(got.reshape(m, n), want), (i, j, h)


def test_split_k_is_deterministic_and_ignores_workspace_contents():
    m, n, k = 64, 512, 8192
    a, b, c = _inputs(O.F16, O.F16, m, n, k, seed=41)
    first, plan = _run_split(O.F16, O.F16, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 0.5, 1.5, fill=0xFF)
    again, _ = _run_split(O.F16, O.F16, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 0.5, 1.5, fill=0x3C)
    assert plan.split_k >= 8
    assert np.array_equal(first, again)
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, c, 0.5, 1.5)
    w32 = O.gemm(O.F16, O.F32, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, O.storage_to_f32(c, O.F16), 0.5, 1.5)
    _check(O.F16, O.F16, first, want, w32)


def test_split_k_f64_scalars_and_int8_wraparound():
    m, n = 144, 128
    k = _k_for(O.F64, 40, 0)
    alpha, beta = 1.0 / 3.0, -1.0 / 7.0
    a, b, c = _inputs(O.F64, O.F64, m, n, k, seed=77)
    got, _ = _run_split(O.F64, O.F64, O.ROW, O.COL, O.ROW, m, n, k, a, b, c, alpha, beta)
    A, B = a.reshape(m, k).astype(np.longdouble), b.reshape(n, k).T.astype(np.longdouble)
    exact = np.longdouble(alpha) * (A @ B) + np.longdouble(beta) * c.reshape(m, n).astype(np.longdouble)
    bound = ((k + 4) * 2.0 ** -53) * (abs(alpha) * (np.abs(A) @ np.abs(B)) + abs(beta) * np.abs(c.reshape(m, n)))
    assert np.all(np.abs(got.reshape(m, n).astype(np.longdouble) - exact) <= bound)
    # scalars rounded to f32 would be far outside that bound
    rounded = np.longdouble(np.float32(alpha)) * (A @ B) + np.longdouble(np.float32(beta)) * c.reshape(m, n).astype(np.longdouble)
    assert not np.all(np.abs(rounded - exact) <= bound)

    k = 4096
    alpha, beta = float(2 ** 25 + 1), float(-(2 ** 24 + 3))
    a, b, c = _inputs(O.I8, O.I32, m, n, k, seed=78)
    got, _ = _run_split(O.I8, O.I32, O.ROW, O.COL, O.ROW, m, n, k, a, b, c, alpha, beta)
    acc = a.reshape(m, k).astype(np.int64) @ b.reshape(n, k).T.astype(np.int64)
    ref = ((2 ** 25 + 1) * acc - (2 ** 24 + 3) * c.reshape(m, n).astype(np.int64)) & 0xFFFFFFFF
    assert np.array_equal(got.view(np.uint32).reshape(m, n), ref.astype(np.uint32))


def test_auto_splits_only_with_a_workspace_and_only_skinny_problems():
    cus = R.device_info().compute_units
    skinny = (O.F16, O.F16, 64, 1024, 8192, O.COL, O.ROW, O.ROW)
    assert _plan(*skinny, 0, R.KERNEL_AUTO).split_k == 1
    assert _plan(*skinny, 0, R.KERNEL_AUTO).workspace_bytes == 0
    p = _plan(*skinny, 2 ** 62, R.KERNEL_AUTO)
    tiles = 1 * 8
    assert p.split_k == min(cus // tiles, 128 // 8, 32) and p.macro_tile_m == 128
    assert p.workspace_bytes == p.split_k * 64 * 1024 * 4
    # a workspace one byte short: AUTO falls back to one workgroup per tile, the forced selector refuses
    assert _plan(*skinny, p.workspace_bytes - 1, R.KERNEL_AUTO).split_k == 1
    with pytest.raises(R.R355Error) as e:
        _plan(*skinny, p.workspace_bytes - 1, R.KERNEL_TILED_128_SPLITK)
    assert e.value.code == -3
    with pytest.raises(R.R355Error):
        _plan(*skinny, 0, R.KERNEL_TILED_128_SPLITK)
    # a launch needs the pointer: without it the forced selector is an error and AUTO does not split (the same D either way)
    in_t, out_t, m, n, k, la, lb, ldl = skinny
    g = R.gemm_args(in_t, out_t, m, n, k, 0x1000, 0x2000, None, 0x4000, 1.0, 0.0, la, lb, ldl, ldl, kernel=R.KERNEL_TILED_128_SPLITK,
                    workspace=None, workspace_bytes=2 ** 62)
    assert R.lib().r355_gemm(R.ctypes.byref(g), None) == -3
    g.workspace = 0x5008  # not 16-byte aligned
    assert R.lib().r355_gemm(R.ctypes.byref(g), None) == -3
    # problems that fill the chip or have a short K do not split
    assert _plan(O.F16, O.F16, 8192, 8192, 8192, O.COL, O.ROW, O.ROW, 2 ** 62, R.KERNEL_AUTO).split_k == 1
    assert _plan(O.F16, O.F16, 2048, 2048, 8192, O.COL, O.ROW, O.ROW, 2 ** 62, R.KERNEL_AUTO).split_k == 1
    assert _plan(O.F16, O.F16, 64, 1024, 512, O.COL, O.ROW, O.ROW, 2 ** 62, R.KERNEL_AUTO).split_k == 1
    # the other selectors never split
    for sel in (R.KERNEL_SIMPLE, R.KERNEL_TILED, R.KERNEL_TILED_128):
        assert _plan(*skinny, 2 ** 62, sel).split_k <= 1

    # AUTO with the workspace runs the split and agrees with the oracle
    in_t, out_t, m, n, k, la, lb, ldl = skinny
    a, b, c = _inputs(in_t, out_t, m, n, k, seed=55)
    got, _ = _run_split(in_t, out_t, la, lb, ldl, m, n, k, a, b, c, 1.0, 1.0, kernel=R.KERNEL_AUTO)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, 1.0, 1.0)
    w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), 1.0, 1.0)
    _check(in_t, out_t, got, want, w32)
