"""r355_gemm_noalloc (split-K partial results in the library's static device buffer, no allocation) against r355_gemm
with a caller-provided workspace: the same kernels in the same order, so the results must be bit-identical; the
workspace path itself is held against the CPU oracle in tests/test_gemm_splitk.py, and once more here."""
import ctypes

import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host
from test_gemm import _check, _inputs

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 16 << 20


def _both(in_t, out_t, la, lb, m, n, k, seed, alpha, beta):
    """D of r355_gemm_noalloc and of r355_gemm with a workspace, same operands; also the plan and the operands."""
    import torch

    a, b, c = _inputs(in_t, out_t, m, n, k, seed=seed)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    probe = R.gemm_args(in_t, out_t, m, n, k, da, db, dc, 0x1000, alpha, beta, la, lb, O.ROW, O.ROW, workspace=0x2000,
                        workspace_bytes=2 ** 62)
    plan = R.gemm_query(probe)
    outs = []
    for which in ("noalloc", "workspace"):
        dd = device_filled(m * n, O.NP_STORAGE[out_t], 0xFF)
        if which == "noalloc":
            before = torch.cuda.memory_allocated()
            g = R.gemm_args(in_t, out_t, m, n, k, da, db, dc, dd, alpha, beta, la, lb, O.ROW, O.ROW)
            R.gemm_noalloc(g)
            assert torch.cuda.memory_allocated() == before
        else:
            ws = device_filled(max(int(plan.workspace_bytes), 16), np.uint8, 0xFF)
            g = R.gemm_args(in_t, out_t, m, n, k, da, db, dc, dd, alpha, beta, la, lb, O.ROW, O.ROW, workspace=ws)
            R._check(R.lib().r355_gemm(ctypes.byref(g), None))
        outs.append(to_host(dd, O.NP_STORAGE[out_t]).copy())
    return outs[0], outs[1], plan, (a, b, c)


def test_noalloc_matches_workspace_split_k_on_consecutive_calls():
    # first call: 16 tiles x 16 shares of f32 partial results = exactly the 16 MiB the static buffer holds
    m, n, k = 512, 512, 8192
    got, ref, plan, (a, b, c) = _both(O.F16, O.F16, O.COL, O.ROW, m, n, k, 61, 2.0, 2.0)
    assert plan.split_k == 16 and plan.workspace_bytes == SCRATCH_BYTES
    assert np.array_equal(got, ref)
    want = O.gemm(O.F16, O.F16, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, c, 2.0, 2.0)
    w32 = O.gemm(O.F16, O.F32, O.COL, O.ROW, O.ROW, O.ROW, m, n, k, a, b, O.storage_to_f32(c, O.F16), 2.0, 2.0)
    _check(O.F16, O.F16, got, want, w32)

    # second call, smaller, other type and other data: what the first call left in the buffer must not show
    m, n, k = 144, 272, 4096 + 48
    got, ref, plan, (a, b, c) = _both(O.I8, O.I32, O.ROW, O.COL, m, n, k, 62, 3.0, -2.0)
    assert plan.split_k >= 2 and plan.workspace_bytes < SCRATCH_BYTES
    assert np.array_equal(got, ref)
    assert np.array_equal(got, O.gemm(O.I8, O.I32, O.ROW, O.COL, O.ROW, O.ROW, m, n, k, a, b, c, 3.0, -2.0))

    # third: a problem that does not split runs as r355_gemm does
    m, n, k = 1024, 768, 256
    got, ref, plan, _ = _both(O.BF16, O.F32, O.ROW, O.COL, m, n, k, 63, 1.0, 1.0)
    assert plan.split_k == 1 and plan.workspace_bytes == 0
    assert np.array_equal(got, ref)


def test_noalloc_refuses_what_the_static_buffer_cannot_hold():
    # f64: 128 tiles x 2 shares x 8 bytes = 32 MiB
    m, n, k = 1024, 2048, 512
    g = R.gemm_args(O.F64, O.F64, m, n, k, 0x1000, 0x2000, None, 0x3000, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, workspace=0x4000,
                    workspace_bytes=2 ** 62)
    assert R.gemm_query(g).workspace_bytes == 32 << 20
    with pytest.raises(R.R355Error) as e:
        R.gemm_noalloc(g)
    assert e.value.code == -3 and "16777216" in str(e.value)
    # invalid arguments are reported as by r355_gemm
    bad = R.gemm_args(O.F16, O.F16, 100, 256, 256, 0x1000, 0x2000, None, 0x3000, 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW)
    with pytest.raises(R.R355Error) as e:
        R.gemm_noalloc(bad)
    assert e.value.code == -3
