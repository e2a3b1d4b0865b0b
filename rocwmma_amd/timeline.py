"""Where a macro tile's time goes: runs one 8192^3 GEMM on the profiling build of the library
(`python -m rocwmma_amd.build --timeline` -> lib/librocwmma_amd_timeline.so, whose 256 x 256 tile kernels record the
100 MHz counter at entry, when the first stage is in LDS, after the K loop and after the last store, plus their CU) and
prints, per phase, the mean / minimum / median / maximum over the workgroups, the gap between consecutive workgroups
on one CU and how far apart the K loops of a round end.

Usage: python -m rocwmma_amd.timeline [--type f16|bf16|i8|e4m3] [--layout nt|tn] [--size 8192] [--zero]
"""
import argparse
import ctypes
import os
import sys

import numpy as np


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--type", default="i8", choices=["f16", "bf16", "i8", "e4m3"])
    ap.add_argument("--layout", default=None, choices=["nt", "tn"])
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--zero", action="store_true", help="all-zero operands (no switching power)")
    args = ap.parse_args()

    import torch

    import rocwmma_amd as R
    from rocwmma_amd.build import TIMELINE_LIB

    if not os.path.exists(TIMELINE_LIB):
        sys.exit("build the profiling library first: python -m rocwmma_amd.build --timeline")
    R.LIB_PATH = TIMELINE_LIB
    in_t = {"f16": R.F16, "bf16": R.BF16, "i8": R.I8, "e4m3": R.E4M3}[args.type]
    out_t = {"f16": R.F16, "bf16": R.BF16, "i8": R.I32, "e4m3": R.F32}[args.type]
    part = {"f16": 0, "bf16": 1, "i8": 2, "e4m3": 2}[args.type]
    layout = args.layout or ("nt" if args.type in ("f16", "bf16") else "tn")
    la = R.ROW_MAJOR if layout[0] == "t" else R.COL_MAJOR
    lb = R.ROW_MAJOR if layout[1] == "t" else R.COL_MAJOR
    s = args.size
    if (s // 256) ** 2 > 8192 or s % 256:
        sys.exit("size: a multiple of 256, at most 8192 tiles")

    def operand(n):
        if args.zero:
            return torch.zeros(n * R.DTYPE_BYTES[in_t], dtype=torch.uint8, device="cuda")
        if in_t == R.I8:
            return torch.randint(-128, 128, (n,), dtype=torch.int16, device="cuda").to(torch.int8)
        if in_t == R.E4M3:
            return torch.randn(n, device="cuda").to(torch.float8_e4m3fn).view(torch.uint8)
        return (torch.rand(n, device="cuda") * 2 - 1).to(torch.float16 if in_t == R.F16 else torch.bfloat16)

    a, b = operand(s * s), operand(s * s)
    d = torch.empty(s * s * R.DTYPE_BYTES[out_t], dtype=torch.uint8, device="cuda")
    g = R.gemm_args(in_t, out_t, s, s, s, a, b, None, d, 1.0, 0.0, la, lb, R.ROW_MAJOR, R.ROW_MAJOR, kernel=R.KERNEL_TILED)
    ms = R.gemm_timed(g, 150, 20)  # settle the clocks, then time
    torch.cuda.synchronize()
    R._check(R.lib().r355_gemm(ctypes.byref(g), None))
    torch.cuda.synchronize()
    tiles = (s // 256) ** 2
    buf = np.zeros(8192 * 8, np.uint64)
    reader = getattr(R.lib(), "r355_timeline_read_p%d" % part)
    assert reader(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.nbytes)) == 0
    t = buf.reshape(8192, 8)[:tiles]
    us = (t[:, :4].astype(np.int64) - int(t[:, 0].min())) / 100.0
    cu = (t[:, 5] & 0xF).astype(np.int64) * 65536 + ((t[:, 4] >> 8) & 0xFF).astype(np.int64)
    cus = sorted(set(cu.tolist()))
    print("%s %s %d^3, %s operands: %.4f ms per launch by HIP events (%.1f T(FL)OP/s); stamped launch spans %.1f us on %d CUs" % (
        args.type, layout.upper(), s, "all-zero" if args.zero else "random", ms, 2.0 * s ** 3 / ms / 1e9, us[:, 3].max(), len(cus)))
    print("| phase | mean us | min | median | max |\n|---|---|---|---|---|")
    for name, v in (("prologue (entry -> first stage in LDS)", us[:, 1] - us[:, 0]), ("K loop", us[:, 2] - us[:, 1]),
                    ("epilogue (-> last store acknowledged)", us[:, 3] - us[:, 2])):
        print("| %s | %.2f | %.2f | %.2f | %.2f |" % (name, v.mean(), v.min(), np.median(v), v.max()))
    gaps = []
    for c in cus:
        idx = np.where(cu == c)[0]
        idx = idx[np.argsort(us[idx, 0])]
        gaps += [us[j, 0] - us[i, 3] for i, j in zip(idx[:-1], idx[1:])]
    if gaps:
        gaps = np.array(gaps)
        print("| gap to the CU's next workgroup | %.2f | %.2f | %.2f | %.2f |" % (gaps.mean(), gaps.min(), np.median(gaps), gaps.max()))
    # the XCDs (each with a clock of its own under the board's power management): mean K loop and when the last epilogue ends
    xcd = (t[:, 5] & 0xF).astype(np.int64)
    kloop = us[:, 2] - us[:, 1]
    print("per XCD (mean K loop us / last epilogue ends at us): " + ", ".join(
        "%d: %.1f / %.1f" % (x, kloop[xcd == x].mean(), us[xcd == x, 3].max()) for x in sorted(set(xcd.tolist()))))
    order = np.argsort(us[:, 2])
    per = len(cus)
    for r in range(-(-tiles // per)):
        sel = order[r * per:(r + 1) * per]
        print("round %d: K loops end %.1f .. %.1f us, epilogues end %.1f .. %.1f us" % (r, us[sel, 2].min(), us[sel, 2].max(), us[sel, 3].min(), us[sel, 3].max()))


if __name__ == "__main__":
    main()
