"""GPU parity of the DLRM dot-interaction kernels against the reference-held fixtures
(test/dlrm/data, copied to tests/golden/dlrm) and the CPU oracle."""
import os

import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dlrm")


def _fwd(dtype, x, m, k, batch):
    dx = to_device(x)
    out_elems = batch * (k + m * (m - 1) // 2)
    dout = device_filled(out_elems + 8, np.uint16, 0xFF)
    R.dlrm_fwd(dtype, dx, dout, m, k, batch)
    full = to_host(dout, np.uint16)
    assert np.all(full[out_elems:] == 0xFFFF)  # nothing written past the end
    return full[:out_elems].reshape(batch, -1)


def test_fwd_reference_fixture_fp16():
    x = np.fromfile(os.path.join(GOLD, "input_fp16"), dtype=np.uint16)
    want = np.fromfile(os.path.join(GOLD, "output_fp16"), dtype=np.uint16).reshape(64, 479)
    got = _fwd(R.F16, x, 27, 128, 64)
    assert np.array_equal(got[:, :128], want[:, :128])
    ok, mx = O.compare(O.F16, got, want, 10.0)  # the reference's DLRM tolerance
    assert ok, mx
    # and against the oracle: f32 accumulation in a different order, then one f16 rounding
    oracle = O.dlrm_fwd(O.F16, x, 27, 128, 64)
    ok, mx = O.compare(O.F16, got, oracle, 10.0)
    assert ok, mx
    assert np.mean(got == oracle) > 0.95


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
@pytest.mark.parametrize("m,k,batch", [(32, 32, 64), (32, 128, 64), (27, 128, 13), (2, 64, 5), (17, 256, 9), (27, 128, 1)])
def test_fwd_shapes_vs_oracle(dtype, m, k, batch):
    x = O.f32_to_storage(O.normal(3, batch * m * k), dtype)
    want = O.dlrm_fwd(dtype, x, m, k, batch)
    got = _fwd(dtype, x, m, k, batch)
    assert np.array_equal(got[:, :k], want[:, :k])
    ok, mx = O.compare(dtype, got, want, 10.0)
    assert ok, mx


def test_fwd_integer_inputs_exact():
    # small integers: every partial sum exact, so the GPU must equal the oracle bit for bit
    m, k, batch = 27, 128, 40
    x = O.f32_to_storage((O.uniform_int8(8, batch * m * k).astype(np.float32) % 4) - 1, O.F16)
    assert np.array_equal(_fwd(O.F16, x, m, k, batch), O.dlrm_fwd(O.F16, x, m, k, batch))


def test_fwd_full_batch_65536_properties():
    # BASELINE config 5 at full size: oracle on a sample of the batch + symmetric-product identity
    m, k, batch = 27, 128, 65536
    x = O.f32_to_storage(O.normal(5, batch * m * k), O.F16)
    got = _fwd(O.F16, x, m, k, batch)
    sel = np.array([0, 1, 7, 8, 4095, 32768, 65535, 12345])
    xs = x.reshape(batch, m * k)[sel]
    want = O.dlrm_fwd(O.F16, xs.ravel(), m, k, len(sel))
    ok, mx = O.compare(O.F16, got[sel], want, 10.0)
    assert ok, mx
    # first 128 outputs of every sample are the first input row
    assert np.array_equal(got[:, :k], x.reshape(batch, m, k)[:, 0, :])
    # sum of the triangle = (|sum_i x_i|^2 - sum_i |x_i|^2) / 2 per sample, in float64
    X = x.view(np.float16).reshape(batch, m, k)[::257].astype(np.float64)
    tri = got.view(np.float16)[::257, k:].astype(np.float64).sum(axis=1)
    ident = ((X.sum(axis=1) ** 2).sum(axis=1) - (X ** 2).sum(axis=(1, 2))) / 2
    assert np.max(np.abs(tri - ident)) < 0.5  # 351 f16 roundings of values up to ~40


@pytest.mark.parametrize("suffix", ["fp16"])
def test_bwd_reference_fixture(suffix):
    x = np.fromfile(os.path.join(GOLD, "input_fp16"), dtype=np.uint16)
    up = np.fromfile(os.path.join(GOLD, "input_grad_fp16"), dtype=np.uint16)
    want = np.fromfile(os.path.join(GOLD, "output_input_grad_fp16"), dtype=np.uint16)
    want_mlp = np.fromfile(os.path.join(GOLD, "output_mlp_input_grad_fp16"), dtype=np.uint16)
    dx, dup = to_device(x), to_device(up)
    dmlp, dgrad = device_filled(64 * 128, np.uint16), device_filled(64 * 27 * 128, np.uint16)
    R.dlrm_bwd(R.F16, dx, dup, dmlp, dgrad, 27, 128, 64)
    assert np.array_equal(to_host(dmlp, np.uint16), want_mlp)
    got = to_host(dgrad, np.uint16)
    ok, mx = O.compare(O.F16, got, want, 10.0)
    assert ok, mx
    omlp, ograd = O.dlrm_bwd(O.F16, x, up, 27, 128, 64)
    ok, mx = O.compare(O.F16, got, ograd.ravel(), 10.0)
    assert ok, mx
