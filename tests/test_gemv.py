"""GPU parity of the f32 GEMV kernel against the oracle's GEMM with n = 1 (the reference validates
its GEMV sample the same way: samples/simple_sgemv.cpp runs gemm_cpu_h with n = 1)."""
import numpy as np
import pytest

import oraclelib as O
import rocwmma_amd as R
from gpuutil import device_filled, to_device, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", [O.ROW, O.COL])
@pytest.mark.parametrize("m,k", [(256, 256), (1024, 512), (8192, 8192), (4100, 260), (65536 + 256, 64),
                                 # whole groups of loads plus a remainder, partial last workgroups, both run widths of the
                                 # col-major kernel (128- and 256-byte runs: the wide one from 16384 rows on)
                                 (96, 2500), (272, 1300), (16384 + 68, 1100), (20, 4096 + 4)])
def test_gemv_vs_oracle(layout, m, k):
    a, x, y = O.uniform_pm1(1, m * k), O.uniform_pm1(2, k), O.uniform_pm1(3, m)
    want = O.gemm(O.F32, O.F32, layout, O.COL, O.COL, O.COL, m, 1, k, a, x, y, 2.0, 2.0)
    da, dx, dy = to_device(a), to_device(x), to_device(y)
    dout = device_filled(m, np.float32, 0xFF)
    R.gemv(layout, m, k, da, dx, dy, dout, 2.0, 2.0)
    got = to_host(dout, np.float32)
    # f32 sums of k products in a different order: k * eps relative to sum |a||x|
    A = O.as_matrix(a, m, k, layout).astype(np.float64)
    bound = (np.abs(A) @ np.abs(x.astype(np.float64))) * 2.0 * k * 6e-8 + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= bound)
    # and close to the exact (float64) result on the reference's metric: k f32 roundings
    exact = 2.0 * (A @ x.astype(np.float64)) + 2.0 * y.astype(np.float64)
    g = got.astype(np.float64)
    assert np.max(np.abs(g - exact) / (np.abs(g) + np.abs(exact) + 1.0)) <= 1e-7 * k


@pytest.mark.parametrize("layout", [O.ROW, O.COL])
@pytest.mark.parametrize("m,k", [(256, 256), (4098, 262), (32768 + 128, 64), (66, 2310), (8192 + 6, 1030)])
def test_dgemv_vs_oracle(layout, m, k):
    """The f64 twin (samples/simple_dgemv.cpp): against the oracle's f64 GEMM with n = 1 and the exact integer case."""
    a = O.uniform_pm1(4, m * k).astype(np.float64) + O.uniform_pm1(5, m * k).astype(np.float64) * 2.0 ** -30
    x = O.uniform_pm1(6, k).astype(np.float64)
    y = O.uniform_pm1(7, m).astype(np.float64)
    want = O.gemm(O.F64, O.F64, layout, O.COL, O.COL, O.COL, m, 1, k, a, x, y, 2.0, 2.0)
    da, dx, dy = to_device(a), to_device(x), to_device(y)
    dout = device_filled(m, np.float64, 0xFF)
    R.dgemv(layout, m, k, da, dx, dy, dout, 2.0, 2.0)
    got = to_host(dout, np.float64)
    A = O.as_matrix(a, m, k, layout)
    bound = (np.abs(A) @ np.abs(x)) * 2.0 * k * 1.2e-16 + 1e-15
    assert np.all(np.abs(got - want) <= bound)
    # integer-valued operands: exact in any summation order
    ai, xi = np.round(a * 8.0), np.round(x * 8.0)
    want = O.gemm(O.F64, O.F64, layout, O.COL, O.COL, O.COL, m, 1, k, ai, xi, None, 1.0, 0.0)
    R.dgemv(layout, m, k, to_device(ai), to_device(xi), None, dout, 1.0, 0.0)
    assert np.array_equal(to_host(dout, np.float64), want)


@pytest.mark.parametrize("layout", [O.ROW, O.COL])
def test_gemv_matrix_beyond_4_gib(layout):
    # A is 36864 x 32768 f32 = 4.8 GB: byte (and, for a 2^32-element matrix, element) offsets past 32 bits.  Sampled
    # elements of y on both sides of the boundary against a float64 dot product of the same row of A.
    import torch

    m, k = 36864, 32768
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.rand(m * k, device="cuda", generator=g) * 2 - 1
    x = torch.rand(k, device="cuda", generator=g) * 2 - 1
    y = torch.empty(m, device="cuda")
    R.gemv(layout, m, k, a, x, None, y, 1.0, 0.0)
    torch.cuda.synchronize()
    A = a.view(m, k) if layout == O.ROW else a.view(k, m).t()
    rows = torch.tensor([0, 1, 16383, 32767, 32768, 32769, m - 1], device="cuda")  # row 32768 starts at byte 2^32 (row-major)
    exact = (A[rows].double() @ x.double()).cpu().numpy()
    bound = (A[rows].abs().double() @ x.abs().double()).cpu().numpy() * k * 6e-8
    got = y[rows].double().cpu().numpy()
    assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
    # the bound sees a wrong row
    assert not np.all(np.abs(np.roll(got, 1) - exact) <= bound)


@pytest.mark.parametrize("dtype,m,k,pad", [("f32", 10920, 6148, 4),   # rows of 24 KiB: three slices and a bit
                                           ("f32", 4100, 16392, 8),   # rows of 64 KiB and a bit: eight waves per row
                                           ("f32", 2052, 32772, 0),   # rows beyond 128 KiB: sixteen waves per row
                                           ("f64", 4098, 8200, 2),    # f64, eight waves; the last workgroup holds two rows
                                           ("f64", 2050, 16386, 0)])  # f64, sixteen waves
def test_row_major_rows_shared_by_a_workgroup(dtype, m, k, pad):
    _shared_rows_case(dtype, m, k, pad)


def _random_shared_rows_case(seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = "f32" if seed % 2 == 0 else "f64"
    size, v = (4, 4) if dtype == "f32" else (8, 2)
    k = int(rng.integers((16 << 10) // size, (300 << 10) // size)) // v * v
    pad = int(rng.integers(0, 17)) * v
    m = ((256 << 20) // ((k + pad) * size) + 1 + int(rng.integers(1, 60)) + v - 1) // v * v
    return dtype, max(m, 2048 + v), k, pad


@pytest.mark.parametrize("seed", range(10))
def test_row_major_shared_rows_random_shapes(seed):
    _shared_rows_case(*_random_shared_rows_case(seed))


@pytest.mark.parametrize("dtype,m,k,pad", [("f32", 300, 32772, 4), ("f32", 512, 40000, 0), ("f32", 4, 65536, 0),
                                           ("f32", 700, 131076, 0), ("f64", 66, 16386, 2), ("f64", 2, 20000, 0)])
def test_row_major_few_long_rows(dtype, m, k, pad):
    """Up to 512 rows of 128 KiB and more (768 of 512 KiB and more): a workgroup per row, whatever the size of the matrix."""
    _shared_rows_case(dtype, m, k, pad, streamed=False)


@pytest.mark.parametrize("dtype,m,k,pad", [("f32", 1028, 65540, 4),    # 257 groups of four rows or 514 of two: uneven rounds, so a wave per row (split: four rows)
                                           ("f32", 512, 131076, 0),    # 256 groups of two rows
                                           ("f32", 772, 90000, 8),     # 193 groups of four rows
                                           ("f64", 386, 131074, 2),    # f64, 193 groups of two rows
                                           ("f64", 768, 49154, 2)])    # f64, 192 groups of four rows
@pytest.mark.parametrize("workspace", [False, True])
def test_row_major_long_rows_of_a_streamed_matrix(dtype, m, k, pad, workspace):
    """384 ... 2047 rows of 256 KiB and more, A beyond 256 MiB: without a workspace the batched shared-row kernel (two or four
    rows per workgroup share the loads of x), with one the split form (four rows per workgroup, pieces of 128 KiB)."""
    _shared_rows_case(dtype, m, k, pad, workspace=workspace)


def _shared_rows_case(dtype, m, k, pad, streamed=True, workspace=False):
    """Row-major A beyond 256 MiB with rows of 16 KiB and more takes the kernel whose workgroups share each row; the
    shapes leave a partly filled last slice of k, a partly filled last group of rows and a padded leading dimension.
    Every row against a float64 (f64: exact integer) evaluation on the device."""
    import torch

    tdt = torch.float32 if dtype == "f32" else torch.float64
    fn = R.gemv if dtype == "f32" else R.dgemv
    lda = k + pad
    assert not streamed or m * lda * (4 if dtype == "f32" else 8) > (256 << 20)
    g = torch.Generator(device="cuda").manual_seed(11)
    a = (torch.rand(m * lda, device="cuda", generator=g, dtype=tdt) * 2 - 1)
    x = (torch.rand(k, device="cuda", generator=g, dtype=tdt) * 2 - 1)
    yin = (torch.rand(m, device="cuda", generator=g, dtype=tdt) * 2 - 1)
    A = a.view(m, lda)
    A[:, k:] = float("nan")  # the padding is never read
    y = torch.full((m,), float("nan"), device="cuda", dtype=tdt)
    ws = None
    if workspace:
        need = R.gemv_workspace_bytes(O.ROW, m, k, a.element_size())
        assert need > 0
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
    fn(O.ROW, m, k, a, x, yin, y, 2.0, 2.0, lda=lda, workspace=ws)
    torch.cuda.synchronize()
    Ad, xd = A[:, :k].double(), x.double()
    exact = 2.0 * (Ad @ xd) + 2.0 * yin.double()
    eps = 6e-8 if dtype == "f32" else 1.2e-16
    bound = (Ad.abs() @ xd.abs()) * 2.0 * k * eps + 4.0 * eps
    err = (y.double() - exact).abs()
    assert bool((err <= bound).all()), float((err / bound).max())
    # the bound sees a wrong row
    assert not bool(((torch.roll(y, 1).double() - exact).abs() <= bound).all())
    if dtype == "f64":
        # integer-valued operands: exact in any summation order
        ai, xi = torch.round(a * 8.0), torch.round(x * 8.0)
        ai.view(m, lda)[:, k:] = float("nan")
        fn(O.ROW, m, k, ai, xi, None, y, 1.0, 0.0, lda=lda, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(y, ai.view(m, lda)[:, :k] @ xi)


# ---- K split over several workgroups per block of rows (r355_gemv_ws / r355_dgemv_ws)

SPLIT_SHAPES = [  # layout, m, k: each one a shape the query wants a workspace for
    (O.COL, 256, 32768 + 260),   # few rows: 8 blocks of rows, 32 splits, the last one short and off the unrolled trip
    (O.COL, 8256, 2048 + 8),     # 258 blocks: a row count just above what fills the CUs; 2 splits
    (O.COL, 4, 16384),           # a single partial block of rows
    (O.COL, 16384 + 576, 2052),  # the 256-byte-run kernel (64 rows per workgroup), 265 blocks
    (O.ROW, 128, 65536 + 4100),  # few long rows: a workgroup per (row, split), the last split short
    (O.ROW, 20, 262144),
]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("layout,m,k", SPLIT_SHAPES)
def test_gemv_split_k_vs_oracle(dtype, layout, m, k):
    """The split form against the oracle's GEMM with n = 1 (same bound as the plain kernels), with padded leading
    dimension, alpha and beta, a workspace full of NaN bit patterns before the call and guard bytes behind it; twice
    in a row: bit-identical (the partial sums are added in split order)."""
    import torch

    f64 = dtype == "f64"
    if f64 and layout == O.ROW:
        k = k // 2 + 2  # (rows of the same byte length)
    nt, ot, es = (np.float64, O.F64, 8) if f64 else (np.float32, O.F32, 4)
    need = R.gemv_workspace_bytes(layout, m, k, es)
    assert need > 0 and need % (m * es) == 0
    pad = 4
    lda = (k if layout == O.ROW else m) + pad
    a = O.uniform_pm1(21, m * k).astype(nt)
    x, y = O.uniform_pm1(22, k).astype(nt), O.uniform_pm1(23, m).astype(nt)
    want = O.gemm(ot, ot, layout, O.COL, O.COL, O.COL, m, 1, k, a, x, y, 2.0, -1.0)
    A = O.as_matrix(a, m, k, layout)
    padded = np.full((m, lda) if layout == O.ROW else (k, lda), 7.0, dtype=nt)
    if layout == O.ROW:
        padded[:, :k] = A
    else:
        padded[:, :m] = A.T
    da, dx, dy = to_device(padded.ravel()), to_device(x), to_device(y)
    guard = 4096
    ws = device_filled((need + guard) // 4, np.float32, 0xFF)
    call = R.dgemv if f64 else R.gemv
    outs = []
    for _ in range(2):
        dout = device_filled(m, nt, 0xFF)
        call(layout, m, k, da, dx, dy, dout, 2.0, -1.0, lda=lda, workspace=ws, workspace_bytes=need)
        outs.append(to_host(dout, nt))
    torch.cuda.synchronize()
    assert np.all(to_host(ws, np.float32).view(np.uint8)[need:] == 0xFF), "bytes behind the workspace were written"
    got = outs[0]
    assert np.array_equal(outs[0].view(np.uint8), outs[1].view(np.uint8))
    eps = 1.2e-16 if f64 else 6e-8
    bound = (np.abs(A.astype(np.float64)) @ np.abs(x.astype(np.float64))) * 2.0 * k * eps + np.abs(y) * 4 * eps + (1e-15 if f64 else 1e-6)
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= bound)
    exact = 2.0 * (A.astype(np.float64) @ x.astype(np.float64)) - y.astype(np.float64)
    g = got.astype(np.float64)
    assert np.max(np.abs(g - exact) / (np.abs(g) + np.abs(exact) + 1.0)) <= (2e-16 if f64 else 1e-7) * k
    # integer-valued operands: exact in any summation order, so the split form and the plain kernel agree bit for bit
    ai, xi = np.round(padded * 8.0), np.round(x * 8.0)
    dai, dxi = to_device(ai.ravel()), to_device(xi)
    plain, split = device_filled(m, nt, 0xFF), device_filled(m, nt, 0xFF)
    call(layout, m, k, dai, dxi, None, plain, 1.0, 0.0, lda=lda)
    call(layout, m, k, dai, dxi, None, split, 1.0, 0.0, lda=lda, workspace=ws, workspace_bytes=need)
    assert np.array_equal(to_host(plain, nt), to_host(split, nt))


def test_gemv_split_k_workspace_rules():
    """The query is 0 where the plain kernels serve the shape; a workspace that is null, too small or not wanted runs the
    plain kernel (same bits as r355_gemv); a misaligned one is an error."""
    assert R.gemv_workspace_bytes(O.COL, 8192, 8192, 4) == 0 and R.gemv_workspace_bytes(O.ROW, 8192, 8192, 4) == 0
    assert R.gemv_workspace_bytes(O.COL, 64, 64, 4) == 0  # too short to split
    m, k = 256, 16384
    need = R.gemv_workspace_bytes(O.COL, m, k, 4)
    assert need == 16 * m * 4  # 16 splits of 1024 columns
    a, x = O.uniform_pm1(31, m * k), O.uniform_pm1(32, k)
    da, dx = to_device(a), to_device(x)
    ws = device_filled(need // 4, np.float32, 0xFF)
    plain = device_filled(m, np.float32, 0xFF)
    R.gemv(O.COL, m, k, da, dx, None, plain)
    for nbytes in (0, need - 4):
        out = device_filled(m, np.float32, 0xFF)
        R.gemv(O.COL, m, k, da, dx, None, out, workspace=ws, workspace_bytes=nbytes)
        assert np.array_equal(to_host(out, np.float32), to_host(plain, np.float32))
        assert np.all(to_host(ws, np.float32).view(np.uint8) == 0xFF)  # untouched
    with pytest.raises(R.R355Error) as e:
        R.gemv(O.COL, m, k, da, dx, None, plain, workspace=ws[4:], workspace_bytes=need - 4)
    assert e.value.code == -4
    # a shape the plain kernels serve: the workspace is left alone
    out, ref = device_filled(8192, np.float32, 0xFF), device_filled(8192, np.float32, 0xFF)
    a2, x2 = to_device(O.uniform_pm1(33, 8192 * 256)), to_device(O.uniform_pm1(34, 256))
    R.gemv(O.COL, 8192, 256, a2, x2, None, ref)
    R.gemv(O.COL, 8192, 256, a2, x2, None, out, workspace=ws)
    assert np.array_equal(to_host(out, np.float32), to_host(ref, np.float32))
    assert np.all(to_host(ws, np.float32).view(np.uint8) == 0xFF)
