"""CPU-side checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and validates arguments before touching a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest

import rocwmma_amd as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "r355_wmma.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(r355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 12
    L = ctypes.CDLL(R.LIB_PATH)
    for name in names:
        assert hasattr(L, name), name
    assert sorted(R.EXPORTS) == names


def test_every_export_has_a_ctypes_prototype():
    """Without argtypes ctypes passes a Python int as a C int: a 64-bit stream handle or pointer would lose its upper half
    (a call with stream = None hides it).  Every parameter of every declaration must be covered."""
    text = open(os.path.join(ROOT, "include", "r355_wmma.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    L = R.lib()
    for name, params in re.findall(r"\b(r355_[a-z0-9_]+)\s*\(([^)]*)\)", text):
        want = 0 if params.strip() in ("", "void") else params.count(",") + 1
        fn = getattr(L, name)
        assert fn.argtypes is not None and len(fn.argtypes) == want, (name, want, fn.argtypes)


def test_version_and_error_channel():
    assert "gfx950" in R.version()
    g = R.gemm_args(R.F16, R.F16, 0, 256, 256, 1, 1, None, 1, 1.0, 0.0, R.ROW_MAJOR, R.COL_MAJOR, R.ROW_MAJOR, R.ROW_MAJOR)
    with pytest.raises(R.R355Error) as e:
        R.gemm_query(g)
    assert e.value.code == -1 and "non-zero" in str(e.value)


def _args(**kw):
    base = dict(in_type=R.F16, out_type=R.F16, m=256, n=256, k=256, a=0x1000, b=0x2000, c=None, d=0x3000, alpha=1.0,
                beta=0.0, layout_a=R.COL_MAJOR, layout_b=R.ROW_MAJOR, layout_c=R.ROW_MAJOR, layout_d=R.ROW_MAJOR)
    base.update(kw)
    return R.gemm_args(**base)


def test_query_selects_kernel_family_and_reports_launch_shape():
    plan = R.gemm_query(_args(m=8192, n=8192, k=8192))
    assert plan.kernel == R.KERNEL_TILED
    assert (plan.macro_tile_m, plan.macro_tile_n, plan.macro_tile_k) == (256, 256, 64)
    assert plan.grid_x == 1024 and plan.block_x == 256 and plan.lds_bytes == 131072
    # int8: 128 elements of K per stage
    plan = R.gemm_query(_args(in_type=R.I8, out_type=R.I32, m=512, n=256, k=1024, layout_a=R.ROW_MAJOR, layout_b=R.COL_MAJOR))
    assert plan.kernel == R.KERNEL_TILED and plan.macro_tile_k == 128 and plan.grid_x == 8
    # 16-bit problems whose 256 x 256 tiles would leave most of the 256 CUs idle take the 128 x 128 tile
    plan = R.gemm_query(_args(m=2048, n=2048, k=2048))
    assert plan.kernel == R.KERNEL_TILED and (plan.macro_tile_m, plan.macro_tile_n) == (128, 128)
    assert plan.grid_x == 256 and plan.lds_bytes == 81920
    plan = R.gemm_query(_args(m=4096, n=4096, k=4096))
    assert (plan.macro_tile_m, plan.grid_x) == (256, 256)
    plan = R.gemm_query(_args(m=2048, n=2048, k=2048, kernel=R.KERNEL_TILED))
    assert (plan.macro_tile_m, plan.grid_x) == (256, 64)
    plan = R.gemm_query(_args(m=8192, n=8192, k=256, kernel=R.KERNEL_TILED_128))
    assert (plan.macro_tile_m, plan.grid_x) == (128, 4096)
    plan = R.gemm_query(_args(in_type=R.E4M3, out_type=R.F32, m=1024, n=1024, k=1024))
    assert (plan.macro_tile_m, plan.macro_tile_k, plan.grid_x, plan.lds_bytes) == (128, 128, 64, 81920)
    # small problems take the 128 x 128 tile with clamped edge loads; what the macro-tile kernels do not
    # take (here f64 rows off 16-byte alignment) falls back to one block per wave
    plan = R.gemm_query(_args(m=64, n=48, k=80))
    assert plan.kernel == R.KERNEL_TILED and plan.macro_tile_m == 128 and plan.grid_x == 8
    plan = R.gemm_query(_args(m=64, n=48, k=80, in_type=R.F32, out_type=R.F32))
    assert plan.kernel == R.KERNEL_TILED and plan.macro_tile_k == 32 and plan.lds_bytes == 81920
    plan = R.gemm_query(_args(m=64, n=48, k=80, in_type=R.F64, out_type=R.F64, layout_a=R.ROW_MAJOR, layout_b=R.COL_MAJOR,
                              lda=81, ldb=81))
    assert plan.kernel == R.KERNEL_SIMPLE and plan.lds_bytes == 0 and plan.macro_tile_m == 32


def test_query_sizes_a_split_k_workspace_without_a_pointer():
    # (no device needed: 256 CUs are assumed when none answers)
    skinny = dict(m=64, n=1024, k=8192)
    plan = R.gemm_query(_args(**skinny))
    assert plan.split_k == 1 and plan.workspace_bytes == 0 and plan.grid_y == 1
    plan = R.gemm_query(_args(workspace=None, workspace_bytes=2 ** 64 - 1, **skinny))
    assert plan.split_k == 16 and plan.grid_y == 16 and plan.workspace_bytes == 16 * 64 * 1024 * 4
    assert (plan.macro_tile_m, plan.grid_x) == (128, 8)
    assert R.gemm_query(_args(workspace=None, workspace_bytes=plan.workspace_bytes - 1, **skinny)).split_k == 1
    f64 = dict(in_type=R.F64, out_type=R.F64, m=128, n=128, k=1024, layout_a=R.ROW_MAJOR, layout_b=R.COL_MAJOR)
    plan = R.gemm_query(_args(workspace=None, workspace_bytes=2 ** 64 - 1, **f64))
    assert plan.split_k == 8 and plan.workspace_bytes == 8 * 128 * 128 * 8  # 64 stages, at least 8 per share; f64 partial sums
    # problems that fill the chip, short K, other selectors: no split
    assert R.gemm_query(_args(m=8192, n=8192, k=8192, workspace_bytes=2 ** 64 - 1)).split_k == 1
    assert R.gemm_query(_args(m=64, n=1024, k=512, workspace_bytes=2 ** 64 - 1)).split_k == 1
    assert R.gemm_query(_args(kernel=R.KERNEL_TILED_128, workspace_bytes=2 ** 64 - 1, **skinny)).split_k == 1


def test_query_plans_cover_every_tile_and_every_k_stage():
    # seeded sweep over shapes and types: the launch shape the plan reports covers the problem, and a split-K plan gives
    # every share at least one whole stage, needs exactly split_k * m * n accumulator elements and never exceeds 32 shares
    import random
    rng = random.Random(7)
    types = [(R.F16, R.F16, 2), (R.BF16, R.F32, 2), (R.I8, R.I32, 1), (R.E4M3, R.F32, 1), (R.F32, R.F32, 4), (R.F64, R.F64, 8)]
    for _ in range(400):
        in_t, out_t, es = rng.choice(types)
        m, n = 16 * rng.randint(1, 300), 16 * rng.randint(1, 300)
        k = (16 // es) * rng.randint(1, 4000)
        la, lb = rng.choice([R.ROW_MAJOR, R.COL_MAJOR]), rng.choice([R.ROW_MAJOR, R.COL_MAJOR])
        plan = R.gemm_query(_args(in_type=in_t, out_type=out_t, m=m, n=n, k=k, layout_a=la, layout_b=lb, workspace_bytes=2 ** 64 - 1))
        assert plan.kernel == R.KERNEL_TILED
        tm, tn = plan.macro_tile_m, plan.macro_tile_n
        assert (tm, tn) in ((128, 128), (256, 256)) and plan.macro_tile_k * es == 128
        tiles = -(-m // tm) * -(-n // tn)
        stages = -(-k * es // 128)
        if plan.split_k > 1:
            assert tm == 128 and 2 * tiles <= 256 and stages >= 16 and plan.split_k <= 32 and plan.grid_y == plan.split_k
            share = -(-stages // plan.split_k)
            assert share >= 8 or plan.split_k * 8 > stages - 8  # at least 8 stages per share where K allows
            assert (plan.split_k - 1) * share < stages  # the last share is not empty
            assert plan.workspace_bytes == plan.split_k * m * n * (8 if in_t == R.F64 else 4)
            assert plan.grid_x >= tiles
        else:
            assert plan.workspace_bytes == 0 and plan.grid_y == 1
            # one launch covers every tile, or the rest (at most half a round of 256 x 256 tiles) runs in the second launch
            assert plan.grid_x >= tiles or (tm == 256 and tiles > 256 and 0 < tiles % 256 <= 128 and plan.grid_x >= tiles - tiles % 256)


@pytest.mark.parametrize("kw,code", [
    (dict(a=None), -1),
    (dict(beta=1.0, c=None), -1),
    (dict(layout_a=7), -1),
    (dict(in_type=R.F16, out_type=R.I32), -2),
    (dict(m=100, n=256), -3),
    (dict(k=20), -3),
    (dict(kernel=R.KERNEL_TILED, m=120), -3),
    (dict(kernel=R.KERNEL_TILED, k=100), -3),
    (dict(kernel=R.KERNEL_TILED_128, m=120), -3),
    (dict(kernel=6), -1),
    (dict(kernel=R.KERNEL_TILED_DEEP, in_type=R.F64, out_type=R.F64), -2),
    (dict(kernel=R.KERNEL_TILED_128_SPLITK), -3),  # no workspace
    (dict(kernel=R.KERNEL_TILED, in_type=R.I8, out_type=R.I32, layout_a=R.ROW_MAJOR, layout_b=R.COL_MAJOR, k=(1 << 23) + 16), -2),
    (dict(kernel=R.KERNEL_TILED, in_type=R.F64, out_type=R.F64), -2),
    (dict(a=0x1002, layout_a=R.ROW_MAJOR), -4),
    (dict(lda=8), -1),
])
def test_argument_validation(kw, code):
    with pytest.raises(R.R355Error) as e:
        R.gemm_query(_args(**kw))
    assert e.value.code == code, str(e.value)
    assert str(e.value)


def test_sparse_macro_tile_ignores_the_orientation_of_an_unread_c():
    # beta == 0: C is never read, so layout_c means nothing and must not push the call off the sparse macro tiles
    sp = dict(in_type=R.I8, out_type=R.I32, m=512, n=512, k=1024, lda=512, layout_a=R.ROW_MAJOR, layout_b=R.COL_MAJOR,
              a_meta=0x4000)
    assert R.gemm_query(_args(layout_c=R.COL_MAJOR, layout_d=R.ROW_MAJOR, **sp)).kernel in (R.KERNEL_TILED, R.KERNEL_TILED_128)
    for tile in (R.KERNEL_TILED, R.KERNEL_TILED_128):
        assert R.gemm_query(_args(layout_c=R.COL_MAJOR, layout_d=R.ROW_MAJOR, kernel=tile, **sp)).kernel == tile
    # beta != 0 with differing orientations: the block-per-wave kernel, and the forced macro tile is refused
    assert R.gemm_query(_args(layout_c=R.COL_MAJOR, layout_d=R.ROW_MAJOR, beta=1.0, c=0x5000, **sp)).kernel == R.KERNEL_SIMPLE
    with pytest.raises(R.R355Error) as e:
        R.gemm_query(_args(layout_c=R.COL_MAJOR, layout_d=R.ROW_MAJOR, beta=1.0, c=0x5000, kernel=R.KERNEL_TILED, **sp))
    assert e.value.code == -2


def test_dlrm_and_gemv_validation_without_gpu():
    with pytest.raises(R.R355Error) as e:
        R.dlrm_fwd(R.F16, 0x1000, 0x2000, 40, 128, 8)
    assert e.value.code == -3
    with pytest.raises(R.R355Error) as e:
        R.dlrm_fwd(R.F16, 0x1000, 0x2000, 27, 100, 8)
    assert e.value.code == -3
    with pytest.raises(R.R355Error) as e:
        R.dlrm_fwd(R.I8, 0x1000, 0x2000, 27, 128, 8)
    assert e.value.code == -2
    with pytest.raises(R.R355Error) as e:
        R.dlrm_fwd(R.F32, 0x1000, 0x2000, 27, 256, 8)
    assert e.value.code == -3
    with pytest.raises(R.R355Error) as e:
        R.gemv(R.COL_MAJOR, 10, 16, 0x1000, 0x2000, None, 0x3000)
    assert e.value.code == -3


def test_compress_24_host_roundtrip_and_rejection():
    import oraclelib as O

    m, k = 32, 256
    mask = O.sparse24_mask(9, m, k)
    dense = np.where(mask, np.maximum(O.uniform_int8(10, m * k).reshape(m, k), 1), 0).astype(np.int8)
    vals, meta = R.compress_24(dense)
    # same format as the oracle's compressor
    ov, om = O.compress24(dense.view(np.uint8), m, k)
    assert np.array_equal(vals.view(np.uint8), ov) and np.array_equal(meta, om)
    assert np.array_equal(R.decompress_24(vals, meta), dense)
    bad = dense.copy()
    bad[3, 4:8] = 1
    with pytest.raises(R.R355Error) as e:
        R.compress_24(bad)
    assert e.value.code == -6 and "row 3" in str(e.value)
    with pytest.raises(R.R355Error) as e:  # k must fill whole 128-byte stages, m whole 16-row blocks
        R.compress_24(dense[:, :64])
    assert e.value.code == -3
    with pytest.raises(R.R355Error) as e:
        R.compress_24(dense[:24])
    assert e.value.code == -3


def test_compress_24_16bit_elements_same_format():
    """2-byte elements: a stage is 64 dense elements (128 bytes), a lane group 16 of them: 8 kept elements (16 bytes)
    and 4 nibbles (2 bytes).  Checked against plain numpy indexing and the axis statement of the K-blocked order."""
    import oraclelib as O

    m, k = 16, 128
    mask = O.sparse24_mask(11, m, k)
    dense = np.where(mask, (np.arange(m * k).reshape(m, k) % 60000 + 1), 0).astype(np.uint16)
    dense[2, 8:12] = 0  # an all-zero group keeps positions 0 and 1
    dense[5, 16:20] = [0, 0x8000, 0, 0]  # -0.0 is a kept value: all-zero bits are what counts as zero
    vals, meta = R.compress_24(dense)
    assert vals.shape == (2, 1, 4, 16, 8) and meta.shape == (2, 1, 4, 16, 2)
    grp = dense.reshape(m, k // 4, 4)
    nz = grp != 0
    # kept positions: the non-zeros, completed with the lowest free positions
    order = np.argsort(~nz, axis=2, kind="stable")[:, :, :2]
    pos = np.sort(order, axis=2)
    assert np.all(pos[:, :, 0] < pos[:, :, 1])
    plain_vals = np.take_along_axis(grp, pos, axis=2).reshape(m, k // 2)
    nib = (pos[:, :, 0] | (pos[:, :, 1] << 2)).astype(np.uint8)
    plain_meta = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    assert np.array_equal(vals.view(np.uint8).reshape(2, 1, 4, 16, 16), O.plain_to_kblocked(plain_vals, m, k, es=2))
    assert np.array_equal(meta, O.plain_to_kblocked(plain_meta, m, k, es=2))
    assert np.array_equal(R.decompress_24(vals, meta), dense)
    bad = dense.copy()
    bad[3, 4:8] = 1
    with pytest.raises(R.R355Error) as e:
        R.compress_24(bad)
    assert e.value.code == -6


def test_deep_pipeline_is_chosen_by_operand_footprint():
    # A and B of 8192^3 f16 are 256 MiB together - the two-buffer kernel (128 KiB of LDS); a little more k, or a padded
    # leading dimension, and they no longer fit the memory-side cache: the five-buffer K loop (160 KiB)
    def q(k, pad, kern=R.KERNEL_AUTO, t=R.F16):
        return R.gemm_query(_args(in_type=t, out_type=t if t != R.I8 else R.I32, m=8192, n=8192, k=k, layout_a=R.ROW_MAJOR,
                                  layout_b=R.COL_MAJOR, lda=k + pad, ldb=k + pad, kernel=kern))
    assert q(8192, 0).lds_bytes == 131072 and q(8192, 0, R.KERNEL_TILED).lds_bytes == 131072
    assert q(8192, 64).lds_bytes == 163840 and q(8192 + 256, 0).lds_bytes == 163840
    assert q(16384, 0, R.KERNEL_TILED).lds_bytes == 163840 and q(8192, 0, R.KERNEL_TILED_DEEP).lds_bytes == 163840
    assert q(8192, 0, R.KERNEL_TILED_DEEP, R.I8).lds_bytes == q(8192, 0, R.KERNEL_TILED, R.I8).lds_bytes == 163840
    assert q(8192, 0, R.KERNEL_TILED_DEEP).kernel == R.KERNEL_TILED and q(8192, 0, R.KERNEL_TILED_DEEP).macro_tile_m == 256
