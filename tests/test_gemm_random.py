"""Seeded random sweep of r355_gemm against the CPU oracle: type pair, the four operand
orientations, C/D orientation, sizes off every tile edge, K tails, padded leading dimensions, scalars, the kernel selector and
an optional split-K workspace are drawn together, so that combinations no hand-written case lists are exercised too.  Bars as in
test_gemm.py (bit-exact for int8; the reference's relative metric for the rest); bytes of D outside the m x n block must
keep their canary."""
import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host
from test_gemm import _check, _e5m2_operand, _embed, _inputs

pytestmark = pytest.mark.gpu

PAIRS = [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.BF16, O.F32), (O.I8, O.I32), (O.I8, O.I8), (O.E4M3, O.F32),
         (O.E5M2, O.F32), (O.F32, O.F32), (O.F64, O.F64)]
CASES = 100


def _draw(case):
    rng = np.random.default_rng(9000 + case)
    in_t, out_t = PAIRS[case % len(PAIRS)]
    es_in, es_out = O.NP_STORAGE[in_t]().itemsize, O.NP_STORAGE[out_t]().itemsize
    shape = rng.integers(0, 5)
    if shape == 4:  # enough tiles for the 256 x 256 macro tile (and its mixed last round) under AUTO
        m, n, k = 16 * int(rng.integers(150, 300)), 16 * int(rng.integers(150, 300)), 16 * int(rng.integers(1, 10))
    elif shape == 0:  # skinny with a long K: split-K territory when a workspace is offered
        m, n, k = 16 * int(rng.integers(1, 5)), 16 * int(rng.integers(1, 40)), 16 * int(rng.integers(128, 400))
    elif shape == 1:  # around the 256 x 256 tile edges
        m, n, k = 16 * int(rng.integers(14, 36)), 16 * int(rng.integers(14, 36)), 16 * int(rng.integers(1, 40))
    else:  # anything small
        m, n, k = 16 * int(rng.integers(1, 24)), 16 * int(rng.integers(1, 24)), 16 * int(rng.integers(1, 70))
    if rng.integers(0, 2):  # a K tail: the smallest step the tiled kernels take is one 16-byte chunk
        k += (16 // es_in) * int(rng.integers(1, max(2, es_in * 16 // 16 + 7)))
    if in_t in (O.F32, O.F64):
        k = min(k, 1024)  # keeps the f32 bar of 1e-5 meaningful
    la, lb, ldl = (int(rng.integers(0, 2)) for _ in range(3))
    pad_in = (16 // es_in) * int(rng.integers(0, 4))
    pad_out = (16 // es_out) * int(rng.integers(0, 4))
    if in_t == O.I8:
        alpha, beta = float(rng.integers(-3, 4)), float(rng.integers(-2, 3))
    elif in_t in (O.E4M3, O.E5M2):
        alpha, beta = 1.0, float(rng.integers(0, 2))
    else:
        alpha, beta = float(rng.choice([1.0, 2.0, -0.5, 0.75])), float(rng.choice([0.0, 1.0, -1.0, 0.5]))
    workspace = bool(rng.integers(0, 2))
    kernel = [R.KERNEL_AUTO, R.KERNEL_AUTO, R.KERNEL_TILED, R.KERNEL_TILED_128, R.KERNEL_SIMPLE][int(rng.integers(0, 5))]
    if shape == 4 and kernel == R.KERNEL_SIMPLE:
        kernel = R.KERNEL_AUTO
    if kernel == R.KERNEL_TILED and case % 2:
        kernel = R.KERNEL_TILED_DEEP  # the five-buffer K loop also for 16-bit operands (for the others it is the same kernel)
    return in_t, out_t, m, n, k, la, lb, ldl, pad_in, pad_out, alpha, beta, workspace, kernel


# 167, 477: e5m2 -> f32 on the 128 x 128 tile over some 4000 wave tiles.  A 128-bit store whose data registers the next
# instruction rewrote put that new value into D a few times per thousand wave tiles; only launches this large showed it.
@pytest.mark.parametrize("case", list(range(CASES)) + [167, 477])
def test_random_gemm_vs_oracle(case):
    in_t, out_t, m, n, k, la, lb, ldl, pad_in, pad_out, alpha, beta, workspace, kernel = _draw(case)
    layouts = [O.ROW, O.COL]
    la, lb, ldl = layouts[la], layouts[lb], layouts[ldl]
    if in_t in (O.F32, O.F64):
        a = O.uniform_pm1(case + 1, m * k).astype(O.NP_STORAGE[in_t])
        b = O.uniform_pm1(case + 2, k * n).astype(O.NP_STORAGE[in_t])
        c = O.uniform_pm1(case + 3, m * n).astype(O.NP_STORAGE[out_t])
    elif in_t == O.E5M2:
        a, b = _e5m2_operand(case + 1, m * k), _e5m2_operand(case + 2, k * n)
        c = O.uniform_pm1(case + 3, m * n)
    else:
        a, b, c = _inputs(in_t, out_t, m, n, k, seed=case + 1)
    if in_t == O.I8 and out_t == O.I8:
        c = O.uniform_int8(case + 3, m * n)
    want = O.gemm(in_t, out_t, la, lb, ldl, ldl, m, n, k, a, b, c, alpha, beta)
    lda = (k if la == O.ROW else m) + pad_in
    ldb = (n if lb == O.ROW else k) + pad_in
    ldc = (n if ldl == O.ROW else m) + pad_out
    ldd = ldc + pad_out
    es_out = c.dtype.itemsize
    canary = np.array([0xEE] * es_out, dtype=np.uint8).view(c.dtype)[0]
    da, db = to_device(_embed(a, m, k, la, lda, 1)), to_device(_embed(b, k, n, lb, ldb, 1))
    dc = to_device(_embed(c, m, n, ldl, ldc, canary))
    major, minor = (m, n) if ldl == O.ROW else (n, m)
    dd = device_filled(major * ldd, O.NP_STORAGE[out_t], 0xEE)
    ws = device_filled(8 << 20, np.uint8, 0xA5) if workspace else None
    args = dict(lda=lda, ldb=ldb, ldc=ldc, ldd=ldd, workspace=ws)
    try:  # a forced selector that has no kernel for this problem is an error, not a fallback: then AUTO decides
        R.gemm_query(R.gemm_args(in_t, out_t, m, n, k, da, db, dc if beta != 0.0 else None, dd, alpha, beta, la, lb, ldl, ldl,
                                 kernel=kernel, **args))
    except R.R355Error:
        kernel = R.KERNEL_AUTO
    R.gemm(in_t, out_t, m, n, k, da, db, dc if beta != 0.0 else None, dd, alpha, beta, la, lb, ldl, ldl, kernel=kernel, **args)
    full = to_host(dd, O.NP_STORAGE[out_t]).reshape(major, ldd)
    assert np.all(full[:, minor:] == canary), "bytes outside D were written"
    got = np.ascontiguousarray(full[:, :minor]).ravel()
    w32 = None
    if out_t in (O.F16, O.BF16):
        w32 = O.gemm(in_t, O.F32, la, lb, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), alpha, beta)
    if in_t == O.E5M2:
        g, w = got.astype(np.float64), want.astype(np.float64)
        assert np.all(np.isfinite(g)) and np.max(np.abs(g - w) / (np.abs(g) + np.abs(w) + 1.0)) <= 1e-2
    elif in_t == O.F32:
        # both sides accumulate in f32, in different orders: compare each with the exact product
        A = a.astype(np.float64).reshape((m, k) if la == O.ROW else (k, m))
        B = b.astype(np.float64).reshape((k, n) if lb == O.ROW else (n, k))
        A = A if la == O.ROW else A.T
        B = B if lb == O.ROW else B.T
        C = c.astype(np.float64).reshape((m, n) if ldl == O.ROW else (n, m))
        C = C if ldl == O.ROW else C.T
        exact = alpha * (A @ B) + beta * C
        bound = (k + 4) * 2.0 ** -24 * (abs(alpha) * (np.abs(A) @ np.abs(B)) + abs(beta) * np.abs(C)) + 1e-30
        G = got.astype(np.float64).reshape((m, n) if ldl == O.ROW else (n, m))
        G = G if ldl == O.ROW else G.T
        assert np.all(np.abs(G - exact) <= bound)
    else:
        _check(in_t, out_t, got, want, w32)


@pytest.mark.parametrize("kernel", ["auto_large", "tiled_128", "simple", "split_k"])
@pytest.mark.parametrize("in_t,out_t", [(O.F16, O.F16), (O.F16, O.F32), (O.BF16, O.BF16), (O.I8, O.I32), (O.I8, O.I8), (O.E4M3, O.F32),
                                        (O.F32, O.F32), (O.F64, O.F64)])
@pytest.mark.parametrize("ldl", [O.ROW, O.COL])
def test_c_may_alias_d(kernel, in_t, out_t, ldl):
    """D = alpha A B + beta D in place (C and D the same pointer, leading dimension and orientation): every kernel reads
    an element's C before it writes that element's D, and tiles, waves and passes own disjoint elements."""
    if kernel == "auto_large":
        m, n, k = 16 * 70, 16 * 66, 16 * 10  # several 256 x 256 tiles plus partial ones
    elif kernel == "split_k":
        m, n, k = 64, 192, 16 * 300
        if in_t in (O.F32, O.F64):
            pytest.skip("split-K is offered for the 16-bit and 8-bit kernels")
    else:
        m, n, k = 16 * 13, 16 * 11, 16 * 8
    if in_t in (O.F32, O.F64):
        a = O.uniform_pm1(31, m * k).astype(O.NP_STORAGE[in_t])
        b = O.uniform_pm1(32, k * n).astype(O.NP_STORAGE[in_t])
        c = O.uniform_pm1(33, m * n).astype(O.NP_STORAGE[out_t])
    else:
        a, b, c = _inputs(in_t, out_t, m, n, k, seed=31)
    if in_t == O.I8 and out_t == O.I8:
        c = O.uniform_int8(33, m * n)
    alpha, beta = (2.0, -1.0) if in_t == O.I8 else (1.0, 1.0) if in_t == O.E4M3 else (0.5, 2.0)
    want = O.gemm(in_t, out_t, O.ROW, O.COL, ldl, ldl, m, n, k, a, b, c, alpha, beta)
    da, db, dcd = to_device(a), to_device(b), to_device(c)
    sel = {"auto_large": R.KERNEL_AUTO, "tiled_128": R.KERNEL_TILED_128, "simple": R.KERNEL_SIMPLE, "split_k": R.KERNEL_AUTO}[kernel]
    ws = device_filled(8 << 20, np.uint8, 0xA5) if kernel == "split_k" else None
    if kernel == "split_k":
        q = R.gemm_query(R.gemm_args(in_t, out_t, m, n, k, da, db, dcd, dcd, alpha, beta, O.ROW, O.COL, ldl, ldl, workspace=ws))
        assert q.split_k > 1
    R.gemm(in_t, out_t, m, n, k, da, db, dcd, dcd, alpha, beta, O.ROW, O.COL, ldl, ldl, kernel=sel, workspace=ws)
    got = to_host(dcd, O.NP_STORAGE[out_t])
    w32 = None
    if out_t in (O.F16, O.BF16):
        w32 = O.gemm(in_t, O.F32, O.ROW, O.COL, ldl, ldl, m, n, k, a, b, O.storage_to_f32(c, out_t), alpha, beta)
    if in_t == O.F32:
        assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) <= 1e-4
    else:
        _check(in_t, out_t, got, want, w32)
