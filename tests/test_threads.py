"""Several host threads calling the entry points at once, each on its own stream and buffers (ctypes drops the GIL during a
call, so the calls really overlap): results must equal the single-threaded ones bit for bit and every call must succeed.
The library keeps no state between calls apart from the thread-local error text, the cached CU count and the
no-allocation buffer's address table."""
import threading

import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import to_device

pytestmark = pytest.mark.gpu

THREADS, ROUNDS = 4, 40


def test_concurrent_callers_on_their_own_streams():
    import torch

    m, n, k = 16 * 23, 16 * 19, 16 * 37
    f, kd, batch = 27, 128, 61
    stride = kd + f * (f - 1) // 2
    work = []
    for t in range(THREADS):
        a, b = O.uniform_int8(100 + t, m * k), O.uniform_int8(200 + t, k * n)
        x = O.f32_to_storage(O.uniform_pm1(300 + t, batch * f * kd), O.F16)
        work.append(dict(a=to_device(a), b=to_device(b), x=to_device(x),
                         d=torch.empty(m * n, dtype=torch.int32, device="cuda"),
                         out=torch.empty(batch * stride, dtype=torch.int16, device="cuda"),
                         stream=torch.cuda.Stream()))
    # single-threaded results first
    want = []
    for w in work:
        R.gemm(O.I8, O.I32, m, n, k, w["a"], w["b"], None, w["d"], 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW)
        R.dlrm_fwd(O.F16, w["x"], w["out"], f, kd, batch)
        torch.cuda.synchronize()
        want.append((w["d"].clone(), w["out"].clone()))
    errors = []

    def run(t):
        w = work[t]
        try:
            for _ in range(ROUNDS):
                w["d"].fill_(-1)
                w["out"].fill_(-1)
                w["stream"].wait_stream(torch.cuda.current_stream())
                R.gemm(O.I8, O.I32, m, n, k, w["a"], w["b"], None, w["d"], 1.0, 0.0, O.ROW, O.COL, O.ROW, O.ROW, stream=w["stream"])
                R.dlrm_fwd(O.F16, w["x"], w["out"], f, kd, batch, stream=w["stream"])
                w["stream"].synchronize()
                if not (torch.equal(w["d"], want[t][0]) and torch.equal(w["out"], want[t][1])):
                    errors.append((t, "mismatch"))
                    return
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=run, args=(t,)) for t in range(THREADS)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
