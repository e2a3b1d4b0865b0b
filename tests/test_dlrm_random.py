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


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
def test_bwd_odd_upstream_run_of_the_last_group_repeated(dtype):
    """batch = 55, m = 31: the last workgroup's 7 upstream rows of 721 elements are an odd number of 16-bit elements, so
    the run ends in the middle of a 32-bit word: that last element is fetched on its own and must land in LDS after the
    16-byte piece around it, whichever wave writes that piece.  Forty launches, every one bit-exact."""
    m, k, batch = 31, 256, 55
    store = O.NP_STORAGE[dtype]
    stride = k + m * (m - 1) // 2
    assert ((batch % 8) * stride) % 2 == 1
    x, up = _ints(11, batch * m * k, dtype), _ints(12, batch * stride, dtype)
    up[-1] = O.f32_to_storage(np.array([3.0], np.float32), dtype)[0]  # the element in question is not zero
    dx, dup = to_device(x), to_device(up)
    want_mlp, want_grad = O.dlrm_bwd(dtype, x, up, m, k, batch)
    wf = O.storage_to_f32(want_grad.ravel(), dtype)
    for launch in range(40):
        dmlp, dgrad = device_filled(batch * k, store, 0xEE), device_filled(batch * m * k, store, 0xEE)
        R.dlrm_bwd(dtype, dx, dup, dmlp, dgrad, m, k, batch)
        assert np.array_equal(to_host(dmlp, store).view(np.uint8), want_mlp.ravel().view(np.uint8)), launch
        assert np.array_equal(O.storage_to_f32(to_host(dgrad, store), dtype), wf), launch
