"""Shape survey of r355_gemm: for each problem the three macro-tile variants forced (256 x 256 two-buffer where the type has
it, 128 x 128, 256 x 256 five-buffer), what R355_KERNEL_AUTO picks and how far that is from the best of the three, and
optionally the vendor library (torch.matmul / torch._int_mm) on the same operands.  This is the measurement behind the
constants of the tile choice (gemm_tiled.hip: macroTile, deepPipeline).  Every figure is the best of `--reps` rounds of 40
launches by HIP events, each after a settling period of launches of the same kernel (short kernels report up to 15 % low
on cold clocks).

Usage: python -m rocwmma_amd.survey [--types f16,i8,e4m3,bf16] [--layouts tn,nt,nn] [--sizes 4096,6144,8192]
                                    [--ks 256,512,1024,2048,4096] [--shapes MxNxK,...] [--vendor] [--reps 3]
"""
import argparse
import ctypes
import time


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--types", default="f16,i8,e4m3")
    ap.add_argument("--layouts", default="tn")
    ap.add_argument("--sizes", default="4096,6144,8192", help="m = n for the size x k grid")
    ap.add_argument("--ks", default="256,512,1024,2048,4096")
    ap.add_argument("--shapes", default="", help="extra problems as MxNxK, comma-separated")
    ap.add_argument("--vendor", action="store_true", help="time torch.matmul / torch._int_mm beside (f16, bf16, i8)")
    ap.add_argument("--reps", type=int, default=3)
    args = ap.parse_args()

    import torch

    import rocwmma_amd as R

    def settle(fn, secs):
        t0 = time.time()
        while time.time() - t0 < secs:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()

    def timed(fn, launches=40):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / launches

    def operands(kind, m, n, k):
        if kind in ("f16", "bf16"):
            dt = torch.float16 if kind == "f16" else torch.bfloat16
            t = R.F16 if kind == "f16" else R.BF16
            return (torch.rand(m, k, device="cuda") * 2 - 1).to(dt), (torch.rand(k, n, device="cuda") * 2 - 1).to(dt), t, t
        if kind == "e4m3":
            f8 = lambda r, c: torch.randn(r, c, device="cuda").to(torch.float8_e4m3fn).view(torch.uint8)
            return f8(m, k), f8(k, n), R.E4M3, R.F32
        i8 = lambda r, c: torch.randint(-128, 128, (r, c), dtype=torch.int16, device="cuda").to(torch.int8)
        return i8(m, k), i8(k, n), R.I8, R.I32

    def one(kind, lay, m, n, k):
        A, B, it, ot = operands(kind, m, n, k)
        a_s = A.contiguous() if lay[0] == "t" else A.t().contiguous()  # "t": A row-major (K-contiguous)
        b_s = B.t().contiguous() if lay[1] == "n" else B.contiguous()  # "n": B col-major (K-contiguous)
        la = R.ROW_MAJOR if lay[0] == "t" else R.COL_MAJOR
        lb = R.COL_MAJOR if lay[1] == "n" else R.ROW_MAJOR
        d = torch.empty(m * n * R.DTYPE_BYTES[ot], dtype=torch.uint8, device="cuda")
        kernels = (("256", R.KERNEL_TILED), ("128", R.KERNEL_TILED_128), ("deep", R.KERNEL_TILED_DEEP), ("auto", R.KERNEL_AUTO))
        gs = [R.gemm_args(it, ot, m, n, k, a_s, b_s, None, d, 1.0, 0.0, la, lb, R.ROW_MAJOR, R.ROW_MAJOR, kernel=kern) for _, kern in kernels]
        fns = [(lambda g=g: R.lib().r355_gemm(ctypes.byref(g), None)) for g in gs]
        names = [nm for nm, _ in kernels]
        if args.vendor and kind != "e4m3":
            va = a_s if lay[0] == "t" else a_s.t()
            vb = b_s.t() if lay[1] == "n" else b_s
            fns.append((lambda: torch._int_mm(va, vb)) if kind == "i8" else (lambda: torch.matmul(va, vb)))
            names.append("vendor")
        settle(fns[0], 0.12)
        best = [float("inf")] * len(fns)
        for _ in range(args.reps):
            for i, fn in enumerate(fns):
                settle(fn, 0.03)
                best[i] = min(best[i], timed(fn))
        plan = R.gemm_query(gs[3])
        w = min(range(3), key=lambda i: best[i])
        tops = lambda ms: 2.0 * m * n * k / ms / 1e9
        cells = " | ".join("%.4f (%.0f)" % (ms, tops(ms)) for ms in best)
        deep = plan.macro_tile_m == 256 and plan.lds_bytes == 163840 and kind in ("f16", "bf16")
        print("| %s %s | %d x %d x %d | %s | %d%s | %s %+.1f %% |" % (kind, lay, m, n, k, cells, plan.macro_tile_m, " deep" if deep else "",
                                                                     names[w], (best[w] / best[3] - 1.0) * 100.0), flush=True)

    shapes = [(s, s, k) for s in map(int, args.sizes.split(",")) for k in map(int, args.ks.split(","))] if args.sizes else []
    shapes += [tuple(int(v) for v in sh.split("x")) for sh in args.shapes.split(",") if sh]
    head = ["case", "m x n x k", "256 x 256", "128 x 128", "256 x 256 five-buffer", "AUTO"] + (["vendor"] if args.vendor else [])
    print("| " + " | ".join(head) + " | AUTO's tile | best forced, AUTO against it |")
    print("|" + "---|" * (len(head) + 2))
    print("(cells: ms (TFLOP/s or TOP/s))")
    for kind in args.types.split(","):
        for lay in args.layouts.split(","):
            for m, n, k in shapes:
                if kind == "i8" and args.vendor and m <= 16:
                    continue  # torch._int_mm wants more than 16 rows
                one(kind, lay, m, n, k)


if __name__ == "__main__":
    main()
