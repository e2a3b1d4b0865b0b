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


def _exact_fwd_f32(x, m, k, batch):
    """float64 evaluation of the interaction terms (inputs are exact in float64)."""
    X = x.reshape(batch, m, k).astype(np.float64)
    T = np.einsum("bik,bjk->bij", X, X)
    ii, jj = np.tril_indices(m, -1)
    return T[:, ii, jj]


def _rel(a, b):
    a, b = a.astype(np.float64), b.astype(np.float64)
    return float(np.max(np.abs(a - b) / (np.abs(a) + np.abs(b) + 1.0)))


# f32 bar.  Any two f32 summation orders of a k = 128 dot product differ by more than the
# reference's 10 eps (the reference-held output_fp32 fixture itself sits 12 eps from a sequential
# f32 sum and 13 eps from the exact value), so the f32 checks are: within 40 eps(f32) of the oracle
# and of the fixture in the reference's relative-error metric, and no further from the float64-exact
# value than 1.5 x the sequential-f32 oracle's own distance from it.
F32_TOL_EPS = 40.0
# Unit-normal inputs (the shape tests below) put the terms of a dot product an order of magnitude above the reference's fixture
# data: over 10^4 results the largest difference between two orders of summation reaches 41 - 46 eps in that metric for either
# f32 kernel (16 x 128 x 64, 25 x 128 x 64).  Their bar against the oracle is 80 eps; the sharp one is the distance from the exact value.
F32_NORMAL_TOL_EPS = 80.0


def _check_f32(got, want_oracle, x, m, k, batch, tol_eps=F32_TOL_EPS):
    assert np.array_equal(got[:, :k], want_oracle[:, :k])
    ok, mx = O.compare(O.F32, got, want_oracle, tol_eps)
    assert ok, mx
    exact = _exact_fwd_f32(x, m, k, batch)
    assert _rel(got[:, k:], exact) <= 1.5 * _rel(want_oracle[:, k:], exact) + 1e-9


def test_fwd_reference_fixture_fp32():
    x = np.fromfile(os.path.join(GOLD, "input_fp32"), dtype=np.float32)
    want = np.fromfile(os.path.join(GOLD, "output_fp32"), dtype=np.float32).reshape(64, 479)
    dx = to_device(x)
    dout = device_filled(64 * 479 + 4, np.float32, 0xFF)
    R.dlrm_fwd(R.F32, dx, dout, 27, 128, 64)
    full = to_host(dout, np.float32)
    assert np.all(np.isnan(full[64 * 479:]))
    got = full[:64 * 479].reshape(64, 479)
    assert np.array_equal(got[:, :128], want[:, :128])
    ok, mx = O.compare(O.F32, got, want, F32_TOL_EPS)
    assert ok, mx
    _check_f32(got, O.dlrm_fwd(O.F32, x, 27, 128, 64), x, 27, 128, 64)


@pytest.mark.parametrize("m,k,batch", [(32, 32, 64), (27, 128, 13), (2, 64, 5), (32, 128, 3), (17, 128, 70),
                                       # the kernel that feeds the matrix instructions from the loads: every instance (k, one or two
                                       # blocks of rows), the last shapes it takes (21 x 64, 24 x 128) and the first it leaves (22, 25)
                                       (32, 32, 700), (17, 32, 33), (20, 64, 70), (17, 128, 64), (17, 128, 515),
                                       # eight samples per workgroup, one run of output rows: both k, both images, batches that end
                                       # inside a workgroup, the shapes either side of the launcher's choices
                                       (21, 64, 70), (26, 64, 9), (27, 64, 70), (18, 128, 64), (25, 128, 61), (32, 128, 70), (29, 128, 1), (28, 128, 515),
                                       (22, 64, 1001),
                                       (16, 128, 64), (16, 128, 1000), (16, 32, 9), (8, 128, 517), (13, 64, 2049), (2, 32, 3), (5, 128, 1)])
def test_fwd_f32_shapes_vs_oracle(m, k, batch):
    x = O.normal(3, batch * m * k)
    want = O.dlrm_fwd(O.F32, x, m, k, batch)
    dx = to_device(x)
    dout = device_filled(want.size + 16, np.float32, 0xEE)
    R.dlrm_fwd(R.F32, dx, dout, m, k, batch)
    out = to_host(dout, np.float32)
    assert np.all(out[want.size:].view(np.uint8) == 0xEE)
    got = out[:want.size].reshape(batch, -1)
    if batch <= 100:
        _check_f32(got, want, x, m, k, batch, F32_NORMAL_TOL_EPS)
    else:
        # The largest of 10^5 differences between two orders of summation passes no fixed number of eps, and the largest distance
        # from the exact value is one element's luck (16 x 128 x 1000: 9.4e-6 against the oracle's 5.2e-6 in the reference's
        # metric, while the root mean square error is 1.66e-6 against 2.35e-6): the mean error is held against the oracle's,
        # the largest loosely
        assert np.array_equal(got[:, :k], want[:, :k])
        exact = _exact_fwd_f32(x, m, k, batch)
        rms = lambda a: float(np.sqrt(np.mean((a.astype(np.float64) - exact) ** 2)))
        assert rms(got[:, k:]) <= 1.05 * rms(want[:, k:]) + 1e-12
        assert _rel(got[:, k:], exact) <= 2.5 * _rel(want[:, k:], exact) + 1e-9
    # small integers: exact in any order of summation
    xi = np.round(O.uniform_pm1(5, batch * m * k) * 3.0).astype(np.float32)
    R.dlrm_fwd(R.F32, to_device(xi), dout, m, k, batch)
    assert np.array_equal(to_host(dout, np.float32)[:want.size].view(np.uint32), O.dlrm_fwd(O.F32, xi, m, k, batch).ravel().view(np.uint32))


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
    # benchmark configuration 5 at full size: oracle on a sample of the batch + symmetric-product identity
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


@pytest.mark.parametrize("dtype,m,k", [(O.F16, 8, 64), (O.BF16, 16, 128), (O.F32, 8, 128), (O.F16, 3, 32)])
def test_few_features_full_batch(dtype, m, k):
    """The benchmark's batch with few features (several samples per block of rows; f32 forward: the kernel fed from the loads),
    ending inside a block: integer-valued inputs, samples from the first, a middle and the last blocks bit for bit against the oracle."""
    batch = 65536 + 3
    stride = k + m * (m - 1) // 2
    store = O.NP_STORAGE[dtype]
    rt = {O.F16: R.F16, O.BF16: R.BF16, O.F32: R.F32}[dtype]
    pack = (lambda v: v.astype(np.float32)) if dtype == O.F32 else (lambda v: O.f32_to_storage(v.astype(np.float32), dtype))
    x, up = pack(np.round(O.uniform_pm1(31, batch * m * k) * 2.0)), pack(np.round(O.uniform_pm1(32, batch * stride) * 2.0))
    dx, dup = to_device(x), to_device(up)
    dout = device_filled(batch * stride + 8, store, 0xEE)
    dmlp, dgrad = device_filled(batch * k + 8, store, 0xEE), device_filled(batch * m * k + 8, store, 0xEE)
    R.dlrm_fwd(rt, dx, dout, m, k, batch)
    R.dlrm_bwd(rt, dx, dup, dmlp, dgrad, m, k, batch)
    out, mlp, grad = to_host(dout, store), to_host(dmlp, store), to_host(dgrad, store)
    assert np.all(out[batch * stride:].view(np.uint8) == 0xEE) and np.all(mlp[batch * k:].view(np.uint8) == 0xEE)
    assert np.all(grad[batch * m * k:].view(np.uint8) == 0xEE)
    sel = np.array(list(range(0, 40)) + list(range(32760, 32800)) + list(range(batch - 40, batch)))
    xs, ups = x.reshape(batch, m * k)[sel].ravel(), up.reshape(batch, stride)[sel].ravel()
    want = O.dlrm_fwd(dtype, xs, m, k, len(sel))
    assert np.array_equal(out[:batch * stride].reshape(batch, stride)[sel].view(np.uint8), want.reshape(len(sel), stride).view(np.uint8))
    wmlp, wgrad = O.dlrm_bwd(dtype, xs, ups, m, k, len(sel))
    assert np.array_equal(mlp[:batch * k].reshape(batch, k)[sel].view(np.uint8), wmlp.reshape(len(sel), k).view(np.uint8))
    g, w = grad[:batch * m * k].reshape(batch, m * k)[sel], wgrad.reshape(len(sel), m * k)
    gf, wf = (g, w) if dtype == O.F32 else (O.storage_to_f32(g.ravel(), dtype), O.storage_to_f32(w.ravel(), dtype))
    assert np.array_equal(gf, wf)  # (values: -0.0 and +0.0 are the same gradient)
    # every sample's first output values are its first input row, and the bottom-MLP gradient the head of its upstream row
    assert np.array_equal(out[:batch * stride].reshape(batch, stride)[:, :k].view(np.uint8), x.reshape(batch, m, k)[:, 0, :].view(np.uint8))
    assert np.array_equal(mlp[:batch * k].reshape(batch, k).view(np.uint8), up.reshape(batch, stride)[:, :k].view(np.uint8))


def test_fwd_and_bwd_batch_beyond_4_gib_of_input():
    # 700 000 samples of 27 x 128 f16 are 4.8 GB: byte offsets of samples from 621 379 on do not fit 32 bits.  Samples on
    # both sides of that boundary against the oracle (every sample is independent of the others).
    import torch

    m, k, batch = 27, 128, 700000
    tri = m * (m - 1) // 2
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(batch * m * k, device="cuda", generator=g).to(torch.float16)
    up = torch.randn(batch * (k + tri), device="cuda", generator=g).to(torch.float16)
    out = device_filled(batch * (k + tri), np.uint16)
    R.dlrm_fwd(R.F16, x, out, m, k, batch)
    mlp, grad = device_filled(batch * k, np.uint16), device_filled(batch * m * k, np.uint16)
    R.dlrm_bwd(R.F16, x, up, mlp, grad, m, k, batch)
    torch.cuda.synchronize()
    sel = [0, 1, 310000, 621377, 621378, 621379, 621380, batch - 1]
    take = lambda t, width: np.stack([t.view(torch.int16)[i * width:(i + 1) * width].cpu().numpy().view(np.uint16) for i in sel])
    xs, ups = take(x, m * k), take(up, k + tri)
    want = O.dlrm_fwd(O.F16, xs.ravel(), m, k, len(sel))
    ok, mx = O.compare(O.F16, take(out, k + tri), want, 10.0)
    assert ok, mx
    wmlp, wgrad = O.dlrm_bwd(O.F16, xs.ravel(), ups.ravel(), m, k, len(sel))
    assert np.array_equal(take(mlp, k), wmlp)
    ok, mx = O.compare(O.F16, take(grad, m * k).ravel(), wgrad.ravel(), 10.0)
    assert ok, mx
    del x, up, out, mlp, grad
    torch.cuda.empty_cache()


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


def _exact_bwd_f32(x, up, m, k, batch):
    """float64 gradient of the f32 inputs: S X with S = T + T^T from the upstream triangle."""
    X = x.reshape(batch, m, k).astype(np.float64)
    U = up.reshape(batch, k + m * (m - 1) // 2).astype(np.float64)
    S = np.zeros((batch, m, m))
    ii, jj = np.tril_indices(m, -1)
    S[:, ii, jj] = U[:, k:]
    S = S + S.transpose(0, 2, 1)
    return S @ X


def _check_bwd_f32(got, want_oracle, x, up, m, k, batch):
    # same bar as the f32 forward: within F32_TOL_EPS of the oracle, and no further from the float64
    # value than 1.5 x the sequential-f32 oracle's own distance from it
    ok, mx = O.compare(O.F32, got, want_oracle, F32_TOL_EPS)
    assert ok, mx
    exact = _exact_bwd_f32(x, up, m, k, batch).ravel()
    err_gpu = np.max(np.abs(got.astype(np.float64) - exact) / (np.abs(exact) + 1.0))
    err_orc = np.max(np.abs(want_oracle.astype(np.float64) - exact) / (np.abs(exact) + 1.0))
    assert err_gpu <= 1.5 * err_orc + 1e-7, (err_gpu, err_orc)


def test_bwd_f32_reference_fixture():
    x = np.fromfile(os.path.join(GOLD, "input_fp32"), dtype=np.float32)
    up = np.fromfile(os.path.join(GOLD, "input_grad_fp32"), dtype=np.float32)
    want = np.fromfile(os.path.join(GOLD, "output_input_grad_fp32"), dtype=np.float32)
    want_mlp = np.fromfile(os.path.join(GOLD, "output_mlp_input_grad_fp32"), dtype=np.float32)
    dx, dup = to_device(x), to_device(up)
    dmlp, dgrad = device_filled(64 * 128, np.float32), device_filled(64 * 27 * 128, np.float32)
    R.dlrm_bwd(R.F32, dx, dup, dmlp, dgrad, 27, 128, 64)
    assert np.array_equal(to_host(dmlp, np.float32), want_mlp)
    got = to_host(dgrad, np.float32)
    ok, mx = O.compare(O.F32, got, want, F32_TOL_EPS)
    assert ok, mx
    _, ograd = O.dlrm_bwd(O.F32, x, up, 27, 128, 64)
    _check_bwd_f32(got, ograd.ravel(), x, up, 27, 128, 64)


@pytest.mark.parametrize("m,k,batch", [(27, 128, 13), (32, 128, 40), (32, 32, 64), (2, 64, 5), (17, 128, 9), (28, 128, 1),
                                       (29, 64, 33)])
def test_bwd_f32_shapes_vs_oracle(m, k, batch):
    stride = k + m * (m - 1) // 2
    x = (O.normal(5, batch * m * k) * 0.5).astype(np.float32)
    up = (O.normal(6, batch * stride) * 0.5).astype(np.float32)
    want_mlp, want = O.dlrm_bwd(O.F32, x, up, m, k, batch)
    dx, dup = to_device(x), to_device(up)
    dmlp = device_filled(batch * k + 8, np.float32, 0xEE)
    dgrad = device_filled(batch * m * k + 8, np.float32, 0xEE)
    R.dlrm_bwd(R.F32, dx, dup, dmlp, dgrad, m, k, batch)
    mlp, grad = to_host(dmlp, np.float32), to_host(dgrad, np.float32)
    assert np.all(mlp[batch * k:].view(np.uint32) == 0xEEEEEEEE) and np.all(grad[batch * m * k:].view(np.uint32) == 0xEEEEEEEE)
    assert np.array_equal(mlp[:batch * k], want_mlp.ravel())
    _check_bwd_f32(grad[:batch * m * k], want.ravel(), x, up, m, k, batch)


def test_bwd_f32_integer_inputs_exact():
    m, k, batch = 27, 128, 24
    stride = k + m * (m - 1) // 2
    x = np.round(O.uniform_pm1(7, batch * m * k) * 3.0).astype(np.float32)
    up = np.round(O.uniform_pm1(8, batch * stride) * 3.0).astype(np.float32)
    want_mlp, want = O.dlrm_bwd(O.F32, x, up, m, k, batch)
    dx, dup = to_device(x), to_device(up)
    dmlp, dgrad = device_filled(batch * k, np.float32), device_filled(batch * m * k, np.float32)
    R.dlrm_bwd(R.F32, dx, dup, dmlp, dgrad, m, k, batch)
    assert np.array_equal(to_host(dmlp, np.float32), want_mlp.ravel())
    assert np.array_equal(to_host(dgrad, np.float32), want.ravel())


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
@pytest.mark.parametrize("m,k,batch", [(27, 128, 13), (32, 128, 8), (32, 32, 64), (2, 64, 5), (17, 256, 9), (28, 128, 1),
                                       (29, 64, 17)])
def test_bwd_shapes_vs_oracle(dtype, m, k, batch):
    """Ragged batches (not a multiple of the 8 samples a workgroup owns), both row bounds (m <= 28, m > 28),
    every supported k; padding bytes after both outputs must stay untouched."""
    stride = k + m * (m - 1) // 2
    x = O.f32_to_storage(O.normal(5, batch * m * k) * 0.5, dtype)
    up = O.f32_to_storage(O.normal(6, batch * stride) * 0.5, dtype)
    want_mlp, want = O.dlrm_bwd(dtype, x, up, m, k, batch)
    dx, dup = to_device(x), to_device(up)
    dmlp = device_filled(batch * k + 8, np.uint16, 0xEE)
    dgrad = device_filled(batch * m * k + 8, np.uint16, 0xEE)
    R.dlrm_bwd(R.F16 if dtype == O.F16 else R.BF16, dx, dup, dmlp, dgrad, m, k, batch)
    mlp, grad = to_host(dmlp, np.uint16), to_host(dgrad, np.uint16)
    assert np.all(mlp[batch * k:] == 0xEEEE) and np.all(grad[batch * m * k:] == 0xEEEE)
    assert np.array_equal(mlp[:batch * k], want_mlp.ravel())
    ok, mx = O.compare(dtype, grad[:batch * m * k], want.ravel(), 10.0)  # the reference's DLRM tolerance
    assert ok, mx


# Up to 16 features the 16-bit kernels take several consecutive samples as one block of rows (the products across samples
# are computed and dropped): every number of samples per block the launcher's rule yields (2 ... 16, both LDS-image
# instances), batches that end inside a block and inside a workgroup's 8 blocks, single samples
FEW_FEATURE_SHAPES = [(8, 128, 1), (8, 128, 2), (8, 128, 3), (8, 128, 25), (8, 128, 193), (16, 128, 9), (16, 32, 33), (15, 64, 17),
                      (5, 64, 77), (2, 256, 100), (2, 32, 131), (3, 32, 1000), (4, 64, 65), (9, 128, 50), (10, 128, 37), (12, 256, 19),
                      (14, 128, 15), (7, 32, 57), (6, 64, 200)]


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.F32])
@pytest.mark.parametrize("m,k,batch", FEW_FEATURE_SHAPES)
def test_few_features_share_a_block_fwd_and_bwd(dtype, m, k, batch):
    """(f32: the backward kernel shares blocks the same way; the forward kernel for these shapes is the one fed from the loads.)"""
    if dtype == O.F32 and k == 256:
        pytest.skip("k = 256 in f32 goes to the general kernels")
    stride = k + m * (m - 1) // 2
    store = O.NP_STORAGE[dtype]
    rt = {O.F16: R.F16, O.BF16: R.BF16, O.F32: R.F32}[dtype]
    tol = F32_NORMAL_TOL_EPS if dtype == O.F32 else 10.0
    pack = (lambda v: v.astype(np.float32)) if dtype == O.F32 else (lambda v: O.f32_to_storage(v.astype(np.float32), dtype))
    for exact in (False, True):
        if exact:  # small integers: every product and partial sum is exact, so any summation order gives the oracle's bits
            x, up = pack(np.round(O.uniform_pm1(17, batch * m * k) * 2.0)), pack(np.round(O.uniform_pm1(18, batch * stride) * 2.0))
        else:
            x, up = pack(O.normal(15, batch * m * k) * 0.5), pack(O.normal(16, batch * stride) * 0.5)
        dx, dup = to_device(x), to_device(up)
        dout = device_filled(batch * stride + 8, store, 0xEE)
        R.dlrm_fwd(rt, dx, dout, m, k, batch)
        out = to_host(dout, store)
        assert np.all(out[batch * stride:].view(np.uint8) == 0xEE)
        want = O.dlrm_fwd(dtype, x, m, k, batch).ravel()
        dmlp, dgrad = device_filled(batch * k + 8, store, 0xEE), device_filled(batch * m * k + 8, store, 0xEE)
        R.dlrm_bwd(rt, dx, dup, dmlp, dgrad, m, k, batch)
        mlp, grad = to_host(dmlp, store), to_host(dgrad, store)
        assert np.all(mlp[batch * k:].view(np.uint8) == 0xEE) and np.all(grad[batch * m * k:].view(np.uint8) == 0xEE)
        want_mlp, want_grad = O.dlrm_bwd(dtype, x, up, m, k, batch)
        assert np.array_equal(mlp[:batch * k].view(np.uint8), want_mlp.ravel().view(np.uint8))
        if exact:
            assert np.array_equal(out[:batch * stride].view(np.uint8), want.view(np.uint8))
            assert np.array_equal(grad[:batch * m * k].view(np.uint8), want_grad.ravel().view(np.uint8))
        else:
            ok, mx = O.compare(dtype, out[:batch * stride], want, tol)
            assert ok, mx
            ok, mx = O.compare(dtype, grad[:batch * m * k], want_grad.ravel(), tol)
            assert ok, mx


def test_bwd_integer_inputs_exact():
    """Small integers: every product and partial sum is exact, so any summation order gives the oracle's bits."""
    m, k, batch = 27, 128, 24
    stride = k + m * (m - 1) // 2
    x = O.f32_to_storage(np.round(O.uniform_pm1(7, batch * m * k) * 3.0), O.F16)
    up = O.f32_to_storage(np.round(O.uniform_pm1(8, batch * stride) * 3.0), O.F16)
    want_mlp, want = O.dlrm_bwd(O.F16, x, up, m, k, batch)
    dx, dup = to_device(x), to_device(up)
    dmlp, dgrad = device_filled(batch * k, np.uint16), device_filled(batch * m * k, np.uint16)
    R.dlrm_bwd(R.F16, dx, dup, dmlp, dgrad, m, k, batch)
    assert np.array_equal(to_host(dmlp, np.uint16), want_mlp.ravel())
    assert np.array_equal(to_host(dgrad, np.uint16), want.ravel())


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.F32])
@pytest.mark.parametrize("m,k,batch", [(128, 128, 64),   # the reference's own test sizes: test/dlrm/test/dlrm_test_params.hpp:57
                                       (1024, 1024, 2),  # (its fourth size with a smaller batch: the oracle's time)
                                       (48, 80, 9),      # 3 x 5 blocks of 16: neither a power of two
                                       (256, 256, 64),   # the register-blocked kernels (they need a launch of 2 / 8 waves per CU), whole super-blocks
                                       (80, 96, 700),    # 5 x 6 blocks: the forward kernel's 4 x 4 super-blocks and the backward kernel's 2 x 4 with partial edges
                                       (112, 48, 600),   # 7 x 3 blocks; k not a multiple of 32 (16-bit: the 16-deep K step)
                                       (32, 512, 5),     # few features, an embedding width the specialised kernels have no instance for
                                       (16, 256, 7)])    # (f32: k = 256 is beyond the specialised f32 kernels)
def test_general_shapes_fwd_and_bwd(dtype, m, k, batch):
    """More than 32 features, or an embedding width other than 32 / 64 / 128 / 256: the block-per-wave and the register-blocked
    kernels on the fragment API.  Forward and backward against the oracle on the reference's metric (10 eps of the type); integer-valued inputs
    must come out exactly."""
    if dtype != O.F32 and (m, k) == (16, 256):
        pytest.skip("the specialised 16-bit kernels take this shape")
    store = O.NP_STORAGE[dtype]
    stride = k + m * (m - 1) // 2
    scale = 1.0 / np.sqrt(k)  # keeps the dot products of k terms near 1
    xf, uf = O.normal(91, batch * m * k) * scale, O.normal(92, batch * stride)
    x = xf.astype(np.float32) if dtype == O.F32 else O.f32_to_storage(xf.astype(np.float32), dtype)
    up = uf.astype(np.float32) if dtype == O.F32 else O.f32_to_storage(uf.astype(np.float32), dtype)
    dx, dup = to_device(x), to_device(up)
    dout = device_filled(batch * stride + 8, store, 0xEE)
    R.dlrm_fwd(dtype, dx, dout, m, k, batch)
    out = to_host(dout, store)
    assert np.all(out[batch * stride:].view(np.uint8) == 0xEE)
    want = O.dlrm_fwd(dtype, x, m, k, batch)
    tol = 40.0 if dtype == O.F32 else 10.0  # (f32: the bar of the specialised f32 kernels, a different summation order than the oracle's)
    ok, mx = O.compare(dtype, out[:batch * stride], want.ravel(), tol)
    assert ok, mx
    dmlp, dgrad = device_filled(batch * k + 8, store, 0xEE), device_filled(batch * m * k + 8, store, 0xEE)
    R.dlrm_bwd(dtype, dx, dup, dmlp, dgrad, m, k, batch)
    mlp, grad = to_host(dmlp, store), to_host(dgrad, store)
    assert np.all(mlp[batch * k:].view(np.uint8) == 0xEE) and np.all(grad[batch * m * k:].view(np.uint8) == 0xEE)
    wmlp, wgrad = O.dlrm_bwd(dtype, x, up, m, k, batch)
    assert np.array_equal(mlp[:batch * k].view(np.uint8), wmlp.ravel().view(np.uint8))
    ok, mx = O.compare(dtype, grad[:batch * m * k], wgrad.ravel(), tol)
    assert ok, mx
    # small integers: exact in any order
    xi = np.round(O.uniform_pm1(93, batch * m * k) * 2.0).astype(np.float32)
    ui = np.round(O.uniform_pm1(94, batch * stride) * 2.0).astype(np.float32)
    if m * 4 * 2 > 2048 and dtype != O.F32:
        return  # sums of m products of up to 4 leave the integers a 16-bit gradient holds exactly
    xi_s, ui_s = (xi, ui) if dtype == O.F32 else (O.f32_to_storage(xi, dtype), O.f32_to_storage(ui, dtype))
    R.dlrm_fwd(dtype, to_device(xi_s), dout, m, k, batch)
    assert np.array_equal(to_host(dout, store)[:batch * stride].view(np.uint8), O.dlrm_fwd(dtype, xi_s, m, k, batch).ravel().view(np.uint8))
    R.dlrm_bwd(dtype, to_device(xi_s), to_device(ui_s), dmlp, dgrad, m, k, batch)
    g = to_host(dgrad, store)[:batch * m * k]
    w = O.dlrm_bwd(dtype, xi_s, ui_s, m, k, batch)[1].ravel()
    gf, wf = (g, w) if dtype == O.F32 else (O.storage_to_f32(g, dtype), O.storage_to_f32(w, dtype))
    assert np.array_equal(gf, wf)


def test_general_shapes_take_a_batch_beyond_one_grid_dimension():
    """The general kernels put the batch into a grid dimension (at most 65535); a larger batch goes out in several
    launches, as the specialised kernels take any batch.  Samples either side of the launch boundary against the oracle."""
    m, k, batch = 48, 16, 65536 + 40
    stride = k + m * (m - 1) // 2
    x = O.f32_to_storage(np.round(O.uniform_pm1(95, batch * m * k) * 2.0), O.F16)
    up = O.f32_to_storage(np.round(O.uniform_pm1(96, batch * stride) * 2.0), O.F16)
    dx, dup = to_device(x), to_device(up)
    dout = device_filled(batch * stride + 8, np.uint16, 0xEE)
    dmlp, dgrad = device_filled(batch * k + 8, np.uint16, 0xEE), device_filled(batch * m * k + 8, np.uint16, 0xEE)
    R.dlrm_fwd(R.F16, dx, dout, m, k, batch)
    R.dlrm_bwd(R.F16, dx, dup, dmlp, dgrad, m, k, batch)
    out, mlp, grad = to_host(dout, np.uint16), to_host(dmlp, np.uint16), to_host(dgrad, np.uint16)
    assert np.all(out[batch * stride:] == 0xEEEE) and np.all(mlp[batch * k:] == 0xEEEE) and np.all(grad[batch * m * k:] == 0xEEEE)
    for first, count in ((0, 8), (65535 - 20, 40), (batch - 8, 8)):
        xs, us = x[first * m * k:(first + count) * m * k], up[first * stride:(first + count) * stride]
        assert np.array_equal(out[first * stride:(first + count) * stride], O.dlrm_fwd(O.F16, xs, m, k, count).ravel())
        wmlp, wgrad = O.dlrm_bwd(O.F16, xs, us, m, k, count)
        assert np.array_equal(mlp[first * k:(first + count) * k], wmlp.ravel())
        assert np.array_equal(grad[first * m * k:(first + count) * m * k], wgrad.ravel())
