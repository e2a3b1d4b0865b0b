"""Seeded random sweep of the f32 and f64 GEMV kernels: orientation, sizes off every group edge (rows per wave, loads in
flight, both run widths of the col-major kernel), padded leading dimensions and scalars drawn together.  Operands are small
integers, so every product and partial sum is exact and the result must equal the oracle's (a GEMM with n = 1, as
samples/simple_sgemv.cpp validates) bit for bit in any summation order; the elements behind y keep their canary."""
import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host
from test_gemm import _embed

pytestmark = pytest.mark.gpu

CASES = 80


def _draw(case):
    rng = np.random.default_rng(11000 + case)
    f64 = bool(case % 2)
    v = 2 if f64 else 4  # elements of a 16-byte piece
    shape = int(rng.integers(0, 4))
    if shape == 0:  # tall
        m, k = v * int(rng.integers(2000, 12000)), v * int(rng.integers(1, 40))
    elif shape == 1:  # wide
        m, k = v * int(rng.integers(1, 40)), v * int(rng.integers(200, 1300))
    else:
        m, k = v * int(rng.integers(1, 700)), v * int(rng.integers(1, 700))
    layout = [O.ROW, O.COL][int(rng.integers(0, 2))]
    pad = v * int(rng.integers(0, 3))
    alpha, beta = float(rng.integers(-2, 3)), float(rng.integers(-1, 2))
    return f64, m, k, layout, pad, alpha, beta


@pytest.mark.parametrize("case", range(CASES))
def test_random_gemv_exact(case):
    f64, m, k, layout, pad, alpha, beta = _draw(case)
    t, dt = (O.F64, np.float64) if f64 else (O.F32, np.float32)
    a = np.round(O.uniform_pm1(case + 1, m * k) * 3.0).astype(dt)
    x = np.round(O.uniform_pm1(case + 2, k) * 3.0).astype(dt)
    y = np.round(O.uniform_pm1(case + 3, m) * 50.0).astype(dt)
    want = O.gemm(t, t, layout, O.COL, O.COL, O.COL, m, 1, k, a, x, y, alpha, beta)
    lda = (k if layout == O.ROW else m) + pad
    da, dx, dy = to_device(_embed(a, m, k, layout, lda, dt(7))), to_device(x), to_device(y)
    dout = device_filled(m + 4, dt, 0xEE)
    (R.dgemv if f64 else R.gemv)(layout, m, k, da, dx, dy if beta != 0.0 else None, dout, alpha, beta, lda=lda)
    full = to_host(dout, dt)
    assert np.all(full[m:].view(np.uint8) == 0xEE), "wrote behind y"
    assert np.array_equal(full[:m], want.ravel()), (f64, m, k, layout, pad, alpha, beta)


def _draw_split(case):
    """Shapes the split-K form is made for: a col-major A with few blocks of rows or a row count just above a multiple of
    what fills 256 CUs and a K of several pieces, a row-major A with few long rows."""
    rng = np.random.default_rng(12000 + case)
    f64 = bool(case % 2)
    v = 2 if f64 else 4
    kind = int(rng.integers(0, 3))
    if kind == 0:  # few rows, long K
        layout, m, k = O.COL, v * int(rng.integers(1, 300)), 4 * int(rng.integers(600, 2400))
    elif kind == 1:  # just above a whole round of workgroups (32 rows of f32, 16 of f64 each)
        layout, m, k = O.COL, 256 * 8 * v + v * int(rng.integers(1, 60)), 4 * int(rng.integers(520, 700))
    else:  # few rows of 256 KiB and more
        layout, m, k = O.ROW, v * int(rng.integers(1, 8)), (262144 // (16 // v)) + v * int(rng.integers(0, 9000))
    pad = v * int(rng.integers(0, 3))
    alpha, beta = float(rng.integers(-2, 3)), float(rng.integers(-1, 2))
    return f64, m, k, layout, pad, alpha, beta


@pytest.mark.parametrize("case", range(36))
def test_random_gemv_split_exact(case):
    """r355_gemv_ws / r355_dgemv_ws with the workspace the query asks for, on integer-valued operands: bit for bit the
    oracle's result; nothing behind y or behind the workspace is written."""
    f64, m, k, layout, pad, alpha, beta = _draw_split(case)
    t, dt = (O.F64, np.float64) if f64 else (O.F32, np.float32)
    a = np.round(O.uniform_pm1(case + 1, m * k) * 3.0).astype(dt)
    x = np.round(O.uniform_pm1(case + 2, k) * 3.0).astype(dt)
    y = np.round(O.uniform_pm1(case + 3, m) * 50.0).astype(dt)
    want = O.gemm(t, t, layout, O.COL, O.COL, O.COL, m, 1, k, a, x, y, alpha, beta)
    lda = (k if layout == O.ROW else m) + pad
    need = R.gemv_workspace_bytes(layout, m, k, 8 if f64 else 4)
    assert need > 0, (f64, m, k, layout)
    da, dx, dy = to_device(_embed(a, m, k, layout, lda, dt(7))), to_device(x), to_device(y)
    dout = device_filled(m + 4, dt, 0xEE)
    ws = device_filled(need + 64, np.uint8, 0xEE)
    (R.dgemv if f64 else R.gemv)(layout, m, k, da, dx, dy if beta != 0.0 else None, dout, alpha, beta, lda=lda, workspace=ws, workspace_bytes=need)
    full = to_host(dout, dt)
    assert np.all(full[m:].view(np.uint8) == 0xEE), "wrote behind y"
    assert np.all(to_host(ws, np.uint8)[need:] == 0xEE), "wrote behind the workspace"
    assert np.array_equal(full[:m], want.ravel()), (f64, m, k, layout, pad, alpha, beta)
