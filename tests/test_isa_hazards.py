"""Static check of the generated gfx950 code (no GPU needed): no buffer store of more than 64 bits may name a scalar
register in its offset field.  For that form the compiler inserts no wait state before the next write of the store's data
registers, and on MI355X such a store has been seen to write the new value of a data register.  The kernels add the
wave-uniform offset to the lane offset instead (gemm_tiled.hip, storeTileStaged); this keeps it that way."""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from rocwmma_amd import build as B

UNITS = [("gemm_tiled.hip", ["-DR355_TILED_PART=2"]), ("dlrm.hip", []), ("sparse.hip", [])]
WIDE_STORE_SCALAR_OFFSET = re.compile(r"buffer_store_dwordx[34]\s+v\[\d+:\d+\],\s*\S+,\s*s\[\d+:\d+\],\s*s\d+")


def _asm(unit):
    src, extra = unit
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "unit.s")
        subprocess.check_call([B.HIPCC] + B.FLAGS + extra + ["-S", "--cuda-device-only", os.path.join(B.CSRC, src), "-o", out],
                              stderr=subprocess.DEVNULL)
        return open(out).read()


@pytest.mark.skipif(not os.path.exists(B.HIPCC), reason="hipcc not installed")
def test_no_wide_buffer_store_with_scalar_register_offset():
    with ThreadPoolExecutor(max_workers=len(UNITS)) as pool:
        texts = list(pool.map(_asm, UNITS))
    wide = 0
    for (src, _), text in zip(UNITS, texts):
        bad = WIDE_STORE_SCALAR_OFFSET.findall(text)
        assert not bad, (src, bad[:3])
        wide += len(re.findall(r"buffer_store_dwordx[34]", text))
    assert wide > 1000  # the pattern above is looking at the right instructions
    # and it does recognise the form it is there to catch
    assert WIDE_STORE_SCALAR_OFFSET.search("\tbuffer_store_dwordx4 v[2:5], v69, s[0:3], s4 offen nt")
    assert not WIDE_STORE_SCALAR_OFFSET.search("\tbuffer_store_dwordx4 v[2:5], v69, s[0:3], 0 offen nt")
