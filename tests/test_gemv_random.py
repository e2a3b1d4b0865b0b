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
