"""Static checks of the generated gfx950 code (no GPU needed).

1. No buffer store of more than 64 bits may name a scalar register in its offset field.  For that form the compiler
   inserts no wait state before the next write of the store's data registers, and on MI355X such a store has been seen to
   write the new value of a data register.  The kernels add the wave-uniform offset to the lane offset instead
   (gemm_tiled.hip, storeTileStaged); this keeps it that way.
2. The macro-tile kernels place their matrix instructions as inline assembly, which the compiler's hazard recogniser does
   not see.  A vector-ALU write of a register needs two wait states before a matrix instruction reads it (that is what the
   compiler itself leaves for the builtin forms: the same scan finds exactly two in gemm_simple.hip and dlrm.hip); met once
   as a stale index operand of v_smfmac behind a v_and.  No matrix instruction of any unit may read a register that a
   vector-ALU instruction wrote fewer than two wait states earlier."""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from rocwmma_amd import build as B

UNITS = [("gemm_tiled.hip", ["-DR355_TILED_PART=0"]), ("gemm_tiled.hip", ["-DR355_TILED_PART=1"]), ("gemm_tiled.hip", ["-DR355_TILED_PART=2"]),
         ("gemm_tiled.hip", ["-DR355_TILED_PART=3"]), ("dlrm.hip", []), ("sparse.hip", []), ("gemm_simple.hip", []), ("dlrm_general.hip", [])]
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


def _stale_matrix_operands(text, need=2):
    """Matrix instructions (v_mfma_*, v_smfmac_*) that read a vector register fewer than `need` wait states after a
    vector-ALU instruction wrote it (an instruction in between is one wait state, s_nop N is N + 1).  Labels are ignored:
    a write at the end of one block followed by a read at the top of the next counts as well."""
    ins = [l.strip() for l in text.splitlines()]
    ins = [l for l in ins if l and not l.startswith((";", ".", "//")) and not l.endswith(":")]
    found = []
    for i, line in enumerate(ins):
        if not line.startswith(("v_mfma", "v_smfmac")):
            continue
        src = set()
        for op in line.split(None, 1)[1].split(",")[1:]:
            src |= _registers(op.strip().split()[0]) if op.strip() else set()
        waits = 0
        for prev in reversed(ins[max(0, i - need):i]):
            nop = re.match(r"s_nop\s+(\d+)", prev)
            if nop:
                waits += int(nop.group(1)) + 1
            else:
                if prev.startswith("v_") and not prev.startswith(("v_mfma", "v_smfmac", "v_cmp")) and waits < need \
                        and _registers(prev.split(None, 1)[1].split(",")[0].strip()) & src:
                    found.append((prev, line, waits))
                waits += 1
            if waits >= need:
                break
    return found


_TEXTS = {}


def _texts():
    if not _TEXTS:
        with ThreadPoolExecutor(max_workers=min(8, len(UNITS))) as pool:
            for unit, text in zip(UNITS, pool.map(_asm, UNITS)):
                _TEXTS[(unit[0], tuple(unit[1]))] = text
    return [_TEXTS[(u[0], tuple(u[1]))] for u in UNITS]


@pytest.mark.skipif(not os.path.exists(B.HIPCC), reason="hipcc not installed")
def test_no_matrix_instruction_reads_a_register_a_vector_instruction_has_just_written():
    texts = _texts()
    matrix = 0
    for (src, extra), text in zip(UNITS, texts):
        bad = _stale_matrix_operands(text)
        assert not bad, (src, extra, bad[:3])
        matrix += len(re.findall(r"^\s*v_s?mfmac?_", text, flags=re.M))
    assert matrix > 50000  # the scan is looking at the kernels' matrix instructions
    # and it recognises the sequence it is there to catch, with and without enough wait states in between
    bad = "\tv_and_b32_e32 v59, 0xffff, v59\n\tv_smfmac_f32_16x16x64_f16 a[60:63], v[8:11], v[0:7], v59\n"
    assert _stale_matrix_operands(bad) and _stale_matrix_operands(bad.replace("\tv_smfmac", "\ts_nop 0\n\tv_smfmac"))
    assert not _stale_matrix_operands(bad.replace("\tv_smfmac", "\ts_nop 1\n\tv_smfmac"))
    assert not _stale_matrix_operands(bad.replace("v59\n", "v58\n"))
    assert _stale_matrix_operands("\tv_mov_b32_e32 v9, v1\n\tds_read_b32 v100, v101\n\tv_mfma_i32_16x16x64_i8 a[0:3], v[8:11], v[0:3], a[0:3]\n")


@pytest.mark.skipif(not os.path.exists(B.HIPCC), reason="hipcc not installed")
def test_no_wide_buffer_store_with_scalar_register_offset():
    texts = _texts()
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
