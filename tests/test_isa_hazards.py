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


STORE = re.compile(r"^(buffer|global|flat|scratch)_store_dwordx[34]\s+(.*)$")


def _registers(token):
    m = re.match(r"v\[(\d+):(\d+)\]$", token)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", token)
    return {int(m.group(1))} if m else set()


def _early_overwrites(text):
    """Wide stores whose data registers a vector instruction writes again with fewer than two wait states between them (an
    instruction in between is one wait state, s_nop N is N + 1), within straight-line code."""
    found = []
    lines = [l.strip() for l in text.splitlines()]
    for i, line in enumerate(lines):
        m = STORE.match(line)
        if not m:
            continue
        ops = [o.strip() for o in m.group(2).split(",")]
        data = _registers(ops[0] if m.group(1) == "buffer" else ops[1])
        waits = 0
        for nxt in lines[i + 1:i + 8]:
            if not nxt or nxt.startswith((";", ".")) and not nxt.endswith(":"):
                continue  # comments and directives
            if nxt.endswith(":") or nxt.startswith(("s_endpgm", "s_branch", "s_cbranch", "s_setpc")) or waits >= 2:
                break  # another block, or far enough
            nop = re.match(r"s_nop\s+(\d+)", nxt)
            if nop:
                waits += int(nop.group(1)) + 1
                continue
            if nxt.startswith("v_") and not nxt.startswith("v_cmp"):
                if _registers(nxt.split(None, 1)[1].split(",")[0].strip()) & data:
                    found.append((line, nxt, waits))
            waits += 1
    return found


@pytest.mark.skipif(not os.path.exists(B.HIPCC), reason="hipcc not installed")
def test_no_wide_buffer_store_with_scalar_register_offset():
    with ThreadPoolExecutor(max_workers=len(UNITS)) as pool:
        texts = list(pool.map(_asm, UNITS))
    for (src, _), text in zip(UNITS, texts):  # the general form of the hazard, whatever the addressing
        assert not _early_overwrites(text), (src, _early_overwrites(text)[:3])
    sample = "\tbuffer_store_dwordx4 v[2:5], v69, s[0:3], s4 offen nt\n\tv_bitop3_b32 v3, v71, v0, 36 bitop3:0x36\n"
    assert _early_overwrites(sample) and not _early_overwrites(sample.replace("\tv_bitop3", "\ts_nop 1\n\tv_bitop3"))
    wide = 0
    for (src, _), text in zip(UNITS, texts):
        bad = WIDE_STORE_SCALAR_OFFSET.findall(text)
        assert not bad, (src, bad[:3])
        wide += len(re.findall(r"buffer_store_dwordx[34]", text))
    assert wide > 1000  # the pattern above is looking at the right instructions
    # and it does recognise the form it is there to catch
    assert WIDE_STORE_SCALAR_OFFSET.search("\tbuffer_store_dwordx4 v[2:5], v69, s[0:3], s4 offen nt")
    assert not WIDE_STORE_SCALAR_OFFSET.search("\tbuffer_store_dwordx4 v[2:5], v69, s[0:3], 0 offen nt")
