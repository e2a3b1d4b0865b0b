"""Seeded random sweep of the DLRM forward and backward kernels: element type, feature count m (2 .. 32, both sides of the
28-row LDS image), k, and ragged batches drawn together.  The inputs are small integers, so every product and every
partial sum is exact in f32 and the result must equal the oracle's bit for bit whatever the summation order; the bytes
behind every output must keep their canary."""
import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu

CASES = 60


def _draw(case):
    rng = np.random.default_rng(7000 + case)
    dtype = [O.F16, O.BF16, O.F32][case % 3]
    m = int(rng.integers(2, 33))
    k = int(rng.choice([32, 64, 128] if dtype == O.F32 else [32, 64, 128, 256]))
    batch = int(rng.integers(1, 100)) if rng.integers(0, 4) else int(rng.integers(100, 700))
    return dtype, m, k, batch


def _ints(seed, n, dtype):
    v = np.round(O.uniform_pm1(seed, n) * 3.0).astype(np.float32)  # -3 .. 3
    return v if dtype == O.F32 else O.f32_to_storage(v, dtype)


@pytest.mark.parametrize("case", range(CASES))
def test_random_dlrm_fwd_bwd_exact(case):
    dtype, m, k, batch = _draw(case)
    store = O.NP_STORAGE[dtype]
    stride = k + m * (m - 1) // 2
    x, up = _ints(case + 1, batch * m * k, dtype), _ints(case + 2, batch * stride, dtype)
    dx, dup = to_device(x), to_device(up)

    want = O.dlrm_fwd(dtype, x, m, k, batch)
    dout = device_filled(batch * stride + 8, store, 0xEE)
    R.dlrm_fwd(dtype, dx, dout, m, k, batch)
    out = to_host(dout, store)
    assert np.all(out[batch * stride:].view(np.uint8) == 0xEE), "forward wrote behind its output"
    assert np.array_equal(out[:batch * stride].view(np.uint8), want.ravel().view(np.uint8)), (dtype, m, k, batch)

    want_mlp, want_grad = O.dlrm_bwd(dtype, x, up, m, k, batch)
    dmlp, dgrad = device_filled(batch * k + 8, store, 0xEE), device_filled(batch * m * k + 8, store, 0xEE)
    R.dlrm_bwd(dtype, dx, dup, dmlp, dgrad, m, k, batch)
    mlp, grad = to_host(dmlp, store), to_host(dgrad, store)
    assert np.all(mlp[batch * k:].view(np.uint8) == 0xEE) and np.all(grad[batch * m * k:].view(np.uint8) == 0xEE)
    assert np.array_equal(mlp[:batch * k].view(np.uint8), want_mlp.ravel().view(np.uint8)), (dtype, m, k, batch)
    # -0.0 and +0.0 are the same gradient: compare values, not bits, where both are zero
    g, w = grad[:batch * m * k], want_grad.ravel()
    gf = g if dtype == O.F32 else O.storage_to_f32(g, dtype)
    wf = w if dtype == O.F32 else O.storage_to_f32(w, dtype)
    assert np.array_equal(gf, wf), (dtype, m, k, batch)
