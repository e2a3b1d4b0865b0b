#!/usr/bin/env python3
"""Headline benchmark: dense GEMM M = N = K = 8192, f16 inputs (A col-major, B row-major = "NT"),
f32 accumulation, f16 row-major output, alpha = 1, beta = 0 -- on one MI355X through the C ABI.

One "step" is one GEMM launch on device-resident operands.  Prints ONE JSON line:
  value        TFLOP/s over the timed region (2 m n k flop per step, wall clock between two
               torch.cuda.synchronize() calls)
  roofline     the same kernel timed with HIP events on its launch stream, against MI355X's
               published dense f16 MFMA peak (2.5 PFLOP/s)
  cpu_baseline the CPU oracle (port of the reference's OpenMP gemm_CPU) timed on a bounded sample
               of complete output rows of the same workload; the same rows validate the GPU result
  extra        the other benchmark configurations (bf16, int8, fp8, 2:4 sparse, DLRM) with their
               own roofline fractions (skipped with --quick)
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "e4m3": 5000.0, "i8": 5000.0, "f32": 157.3, "f64": 78.6}
HBM_PEAK_GBPS = 8000.0
# rocprofv3 --pmc results per benchmark case (MFMA busy, LDS bank conflicts, bytes across the L2 <-> fabric
# boundary), one table row per case.  Each row carries the SHA-256 (first 16 hex digits) of the kernel sources it
# was measured on; a row whose digest differs from the sources of this tree is reported as null, so a counter
# can never outlive the kernel it belongs to.
COUNTERS_FILE = os.path.join(ROOT, "profiles", "bench_counters.md")
KERNEL_SOURCES = {"gemm": ["gemm_tiled.hip", "tile_map.hpp", "lds_dma.hpp", "operand_tile.hpp"],
                  "sparse": ["sparse.hip", "tile_map.hpp", "lds_dma.hpp", "operand_tile.hpp"],
                  "dlrm": ["dlrm.hip"]}


# Matrix-core operations per CU and clock of gfx950, dense (the Multiplier of the reference's peak model,
# test/performance.hpp:435-442: peak = Multiplier x CUs x clock; 2:4 sparse doubles it): published peak / (256 CUs x 2.4 GHz)
MULTIPLIER = {"f16": 4096, "bf16": 4096, "e4m3": 8192, "i8": 8192, "f32": 256, "f64": 128}


class ClockSampler:
    """Engine clock (sclk) of the benchmarked GPU, read while a timed loop runs: rsmi_dev_gpu_clk_freq_get(RSMI_CLK_TYPE_SYS)
    of librocm_smi64 -- the call the reference's harness makes once before its runs (test/hip_device.cpp:99-146) -- from
    a helper thread of this process, every few milliseconds.  Without the library (or a matching device) every reading is
    None and the clock-relative figures are reported as null."""

    class _Freq(ctypes.Structure):
        _fields_ = [("has_deep_sleep", ctypes.c_bool), ("num_supported", ctypes.c_uint32), ("current", ctypes.c_uint32),
                    ("frequency", ctypes.c_uint64 * 33)]

    def __init__(self, torch):
        self.lib, self.index, self.samples, self._stop, self._thread = None, None, [], False, None
        try:
            lib = ctypes.CDLL("librocm_smi64.so")
        except OSError:
            try:
                lib = ctypes.CDLL("/opt/rocm/lib/librocm_smi64.so")
            except OSError:
                return
        try:
            if lib.rsmi_init(ctypes.c_uint64(0)) != 0:
                return
            count = ctypes.c_uint32(0)
            if lib.rsmi_num_monitor_devices(ctypes.byref(count)) != 0 or count.value == 0:
                return
            props = torch.cuda.get_device_properties(0)
            bus = getattr(props, "pci_bus_id", None)
            index = 0 if count.value == 1 else None
            for i in range(count.value):  # the device whose PCI bus number is HIP's (bits 8..15 of rocm_smi's id)
                pci = ctypes.c_uint64(0)
                if lib.rsmi_dev_pci_id_get(ctypes.c_uint32(i), ctypes.byref(pci)) == 0 and bus is not None \
                        and ((pci.value >> 8) & 0xFF) == (bus & 0xFF):
                    index = i
                    break
            if index is None:
                return
            self.lib, self.index = lib, index
            if self.read() is None:
                self.lib = None
        except Exception:
            self.lib = None

    def read(self):
        if self.lib is None:
            return None
        f = ClockSampler._Freq()
        if self.lib.rsmi_dev_gpu_clk_freq_get(ctypes.c_uint32(self.index), ctypes.c_int(0), ctypes.byref(f)) != 0 \
                or f.current >= 33:
            return None
        return f.frequency[f.current] / 1e6

    def measure(self, fn, lead_s=0.0):
        """fn() with the clock sampled meanwhile (readings of the first lead_s seconds dropped); returns (fn's result,
        median MHz or None, number of readings)."""
        import threading

        self.samples, self._stop = [], False
        t0 = time.perf_counter()

        def loop():
            while not self._stop:
                v = self.read()
                if v is not None and time.perf_counter() - t0 >= lead_s:
                    self.samples.append(v)
                time.sleep(0.002)

        th = None
        if self.lib is not None:
            th = threading.Thread(target=loop, daemon=True)
            th.start()
        try:
            res = fn()
        finally:
            self._stop = True
            if th is not None:
                th.join()
        if not self.samples:
            return res, None, 0
        vals = sorted(self.samples)
        return res, vals[len(vals) // 2], len(vals)


def clock_fields(kind, achieved, clock_mhz, cus, sparse=False):
    """The reference's efficiency figure (test/performance.hpp:435-442): achieved / (Multiplier x CUs x clock), at the clock
    measured while the kernel ran."""
    if clock_mhz is None:
        return {"clock_mhz_measured": None, "frac_at_measured_clock": None}
    peak = MULTIPLIER[kind] * (2 if sparse else 1) * cus * clock_mhz * 1e-6  # T(FL)OP/s
    return {"clock_mhz_measured": round(clock_mhz, 1), "peak_at_measured_clock": round(peak, 1),
            "frac_at_measured_clock": round(achieved / peak, 4)}


def source_digest(family):
    import hashlib

    h = hashlib.sha256()
    for f in KERNEL_SOURCES[family]:
        with open(os.path.join(ROOT, "rocwmma_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def load_counters():
    """{case: {"mfma_busy_pct", "lds_bank_conflicts", "fetch_bytes", "write_bytes"}} from the table rows
    `| case | family | digest | MFMA busy % | LDS bank conflicts | fetch bytes | write bytes |` whose digest matches."""
    out = {}
    if not os.path.exists(COUNTERS_FILE):
        return out
    digests = {}
    for line in open(COUNTERS_FILE):
        cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
        if len(cells) != 7 or cells[1] not in KERNEL_SOURCES:
            continue
        fam = cells[1]
        digests.setdefault(fam, source_digest(fam))
        if cells[2] != digests[fam]:
            continue
        num = lambda c: None if c in ("", "-") else float(c)
        out[cells[0]] = {"mfma_busy_pct": num(cells[3]), "lds_bank_conflicts": num(cells[4]), "fetch_bytes": num(cells[5]),
                         "write_bytes": num(cells[6]), "source": "profiles/bench_counters.md"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--size", type=int, default=8192, help="M = N = K (default: the headline size)")
    ap.add_argument("--cpu-rows", type=int, default=512, help="output rows the CPU baseline computes")
    ap.add_argument("--quick", action="store_true", help="skip the extra configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (got --gpus %d); every kernel here is a "
              "single-device kernel and nothing is sharded" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import oraclelib as O  # CPU oracle: used only for cpu_baseline and for validating the result
    import rocwmma_amd as R

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if not os.path.exists(R.LIB_PATH):
        from rocwmma_amd import build

        build.build()
    dev = R.device_info()
    m = n = k = args.size
    flop = 2.0 * m * n * k

    # ---- workload: seeded U[-1, 1) rounded to f16 (seeds 1, 2), generated on the host so that the
    # CPU baseline sees the same bits
    a = O.f32_to_storage(O.uniform_pm1(1, m * k), O.F16)  # col-major m x k
    b = O.f32_to_storage(O.uniform_pm1(2, k * n), O.F16)  # row-major k x n
    da = torch.from_numpy(a.view(np.int16)).cuda()
    db = torch.from_numpy(b.view(np.int16)).cuda()
    dd = torch.full((m * n,), -1, dtype=torch.int16, device="cuda")  # 0xFFFF = NaN prefill
    g = R.gemm_args(R.F16, R.F16, m, n, k, da, db, None, dd, 1.0, 0.0, R.COL_MAJOR, R.ROW_MAJOR, R.ROW_MAJOR,
                    R.ROW_MAJOR, kernel=R.KERNEL_AUTO)
    plan = R.gemm_query(g)

    launch = R.lib().r355_gemm
    gref = ctypes.byref(g)
    # untimed: bring the device to its sustained clocks first (a handful of 0.7 ms launches after the host-side
    # set-up above under-reports by up to 10 %), then the W warm-up steps the caller asked for
    settle(torch, lambda: launch(gref, None), 0.25)
    for _ in range(args.warmup):
        assert launch(gref, None) == 0, R.lib().r355_last_error()
    torch.cuda.synchronize()
    status = 0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        status |= launch(gref, None)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    assert status == 0, R.lib().r355_last_error()
    value = flop / wall_ms / 1e9

    # kernel duration by HIP events on the launch stream, the engine clock read meanwhile (the warm-up launches of the
    # event-timed run are the sampler's lead time)
    clocks = ClockSampler(torch)
    ev_ms, head_mhz, head_reads = clocks.measure(lambda: R.gemm_timed(g, args.warmup, max(args.steps, 100)),
                                                 lead_s=args.warmup * wall_ms * 1e-3)
    achieved = flop / ev_ms / 1e9

    # ---- CPU baseline on a bounded sample (complete rows of D), doubling as validation
    rows = np.linspace(0, m - 1, args.cpu_rows).astype(np.uint32)
    t0 = time.perf_counter()
    want = O.gemm_rows(O.F16, O.F16, O.COL, O.ROW, m, n, k, a, b, rows)
    cpu_s = time.perf_counter() - t0
    cpu_tflops = 2.0 * len(rows) * n * k / cpu_s / 1e12
    got = dd.cpu().numpy().view(np.uint16).reshape(m, n)[rows]
    gf, wf = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    max_rel = float(np.max(np.abs(gf - wf) / (np.abs(gf) + np.abs(wf) + 1.0)))
    validated = bool(np.all(np.isfinite(gf)) and max_rel <= 1e-3)

    counters = load_counters()
    extra = {}
    if not args.quick:
        extra = run_extras(R, O, np, torch, args, counters, clocks, dev.compute_units)
    head = counters.get("gemm_f16_nt_8192") if args.size == 8192 else None

    line = {
        "metric": "TFLOPS at 8192^3 f16 GEMM (f32 accumulate, NT, f16 out); int8 / bf16 / fp8 / sparse / DLRM in extra",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "dense GEMM M=N=K=%d, f16 A (col-major) x f16 B (row-major) -> f16 row-major, "
                               "f32 accumulate, alpha=1 beta=0 (headline configuration)" % m,
                   "kernel": {1: "block-per-wave", 2: "macro-tile"}[plan.kernel],
                   "macro_tile": [plan.macro_tile_m, plan.macro_tile_n, plan.macro_tile_k],
                   "lds_bytes": plan.lds_bytes, "grid": plan.grid_x, "block": plan.block_x,
                   "seeds": {"A": 1, "B": 2}},
        "frac_of_peak": round(value / PEAK_TFLOPS["f16"], 4),
        "validated": validated,
        "max_rel_error_vs_oracle": max_rel,
        # measured in this run: achieved, frac, kernel_ms (HIP events) and the clock figures (rocm_smi readings during the
        # event-timed launches); looked up, not measured in this run: traffic and the *_from_profile counters (rocprofv3 --pmc
        # runs of this very kernel source, profiles/bench_counters.md, keyed by a digest of the sources); computed:
        # algorithmic_gbps = algorithmic bytes / kernel time (not a counter)
        "roofline": dict({"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                          "frac": round(achieved / PEAK_TFLOPS["f16"], 4),
                          "traffic": int(head["fetch_bytes"] + head["write_bytes"]) if head and head["fetch_bytes"] and head["write_bytes"] else None,
                          "traffic_measured_in_this_run": False,
                          "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel source (profiles/bench_counters.md)" if head else None,
                          "mfma_busy_pct_from_profile": head["mfma_busy_pct"] if head else None,
                          "lds_bank_conflicts_from_profile": head["lds_bank_conflicts"] if head else None,
                          "algorithmic_gbps": round(((m * k + k * n) * 2 + m * n * 2) / ev_ms / 1e6, 1),
                          "kernel_ms": round(ev_ms, 4), "algorithmic_flop": flop,
                          "algorithmic_bytes": (m * k + k * n) * 2 + m * n * 2, "clock_readings": head_reads},
                         **clock_fields("f16", achieved, head_mhz, dev.compute_units)),
        "cpu_baseline": {"value": round(cpu_tflops, 6), "unit": "TFLOP/s", "cores": O.lib().orc_num_threads(),
                         "kind": "port",
                         "sample": "%d complete rows of D (all %d columns, full K=%d) of the same workload, %.1f s; "
                                   "extrapolated full problem %.0f s" % (len(rows), n, k, cpu_s, cpu_s * m / len(rows))},
        "device": {"arch": dev.arch.decode(), "cus": dev.compute_units, "clock_mhz_max": dev.clock_mhz},
        "extra": extra,
    }
    line["child_processes_at_end"] = end_child_processes()
    print(json.dumps(line))
    sys.stdout.flush()


def end_child_processes():
    """Names of the processes this one has started that are still alive (none are expected: the benchmark starts no
    helper programs itself, but a library it loads may), each ended by its process id so that nothing outlives the run."""
    try:
        import psutil
    except ImportError:
        return None
    left = []
    for child in psutil.Process().children(recursive=True):
        try:
            left.append(" ".join(child.cmdline()[:3]) or child.name())
            child.terminate()
        except psutil.Error:
            pass
    return left


def settle(torch, fn, seconds=0.1):
    """Untimed launches of fn for `seconds` of wall time before a short kernel is timed: after the host-side set-up
    between two cases the device needs some tens of milliseconds of load to return to its sustained
    clocks, more than a handful of 0.1 ms launches provide."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def run_extras(R, O, np, torch, args, counters, clocks, cus):
    """The remaining benchmark configurations, each timed with HIP events over args.steps launches; every result is
    checked for finite values and on sampled elements (GEMM), samples (DLRM) or rows (GEMV) against a float64 / int64 evaluation on the device
    (the oracle-based parity of the same configurations is in tests/)."""
    out = {}
    s = args.size

    def with_counters(name, rec):
        c = counters.get(name)
        if c:  # looked up (rocprofv3 --pmc runs of this kernel source), not measured in this run
            rec["counters_from_profile"] = {k: v for k, v in c.items() if v is not None}
        return rec

    def dlrm_ok(x, o, up, gmlp, gin, bsz, mm, kk, tol):
        """32 evenly spaced samples of the batch against a float64 evaluation on the device: the forward's row copy and
        interaction triangle when `o` is given, the backward's two gradients when `up` is."""
        pick = torch.arange(0, bsz, bsz // 32, device="cuda")
        ii, jj = torch.tril_indices(mm, mm, -1, device="cuda")
        xs = x.view(bsz, mm, kk)[pick].double()
        close = lambda got, want: bool(((got.double() - want).abs() <= tol * (want.abs() + 1.0)).all())
        if o is not None:
            os_ = o.view(bsz, -1)[pick]
            return close(os_[:, :kk], xs[:, 0]) and close(os_[:, kk:], (xs @ xs.transpose(1, 2))[:, ii, jj])
        us = up.view(bsz, -1)[pick].double()
        sm = torch.zeros(len(pick), mm, mm, dtype=torch.float64, device="cuda")
        sm[:, ii, jj] = us[:, kk:]
        sm = sm + sm.transpose(1, 2)
        return close(gmlp.view(bsz, kk)[pick], us[:, :kk]) and close(gin.view(bsz, mm, kk)[pick], sm @ xs)

    def sampled_ok(in_t, out_t, la, lb, mm, nn, kk, a, b, d, sparse_rows):
        """Dense cases: 64 sampled elements of D against a float64 dot product of the operands as stored.  2:4 sparse cases:
        `sparse_rows` = (row numbers, the oracle's dense GEMM of those complete rows on the uncompressed A): int8
        bit-exact, e4m3 within 1e-2 on the relative metric of the parity tests."""
        tdt = {R.F16: torch.float16, R.BF16: torch.bfloat16, R.I8: torch.int8, R.E4M3: torch.float8_e4m3fn, R.F32: torch.float32,
               R.F64: torch.float64, R.I32: torch.int32}
        dv = d.view(tdt[out_t]).view(mm, nn)
        if not bool(torch.isfinite(dv.to(torch.float64)).all()):
            return False
        if sparse_rows is not None:
            rows, want = sparse_rows
            got = dv[torch.from_numpy(rows.astype(np.int64)).cuda()].cpu().numpy()
            if in_t == R.I8:
                return bool(np.array_equal(got, want))
            gf, wf = got.astype(np.float64), want.astype(np.float64)
            return bool(np.max(np.abs(gf - wf) / (np.abs(gf) + np.abs(wf) + 1.0)) <= 1e-2)
        av = a.view(tdt[in_t]).view((mm, kk) if la == R.ROW_MAJOR else (kk, mm))
        bv = b.view(tdt[in_t]).view((kk, nn) if lb == R.ROW_MAJOR else (nn, kk))
        g = torch.Generator(device="cpu").manual_seed(5)
        ri, ci = torch.randint(0, mm, (64,), generator=g).cuda(), torch.randint(0, nn, (64,), generator=g).cuda()
        ar = (av[ri] if la == R.ROW_MAJOR else av[:, ri].t()).to(torch.float64)
        bc = (bv[:, ci].t() if lb == R.ROW_MAJOR else bv[ci]).to(torch.float64)
        want = (ar * bc).sum(1)
        got = dv[ri, ci].to(torch.float64)
        tol = {R.I8: 0.0, R.F64: 1e-10, R.F32: 1e-4}.get(in_t, 1e-2)
        return bool(((got - want).abs() <= tol * (want.abs() + got.abs() + 1.0) + (2e-3 * want.abs() if out_t in (R.F16, R.BF16) else 0)).all())

    def rnd16(nel, bf):
        t = (torch.rand(nel, device="cuda") * 2 - 1)
        return t.to(torch.bfloat16 if bf else torch.float16)

    KIND = {R.F16: "f16", R.BF16: "bf16", R.E4M3: "e4m3", R.I8: "i8", R.F32: "f32", R.F64: "f64"}

    def gemm_case(name, in_t, out_t, la, lb, a, b, peak, unit, sparse_meta=None, mm=s, nn=s, kk=s, peak_scale=1.0, workspace=None,
                  sparse_rows=None):
        d = torch.empty(mm * nn * R.DTYPE_BYTES[out_t], dtype=torch.uint8, device="cuda")
        g = R.gemm_args(in_t, out_t, mm, nn, kk, a, b, None, d, 1.0, 0.0, la, lb, R.ROW_MAJOR, R.ROW_MAJOR,
                        a_meta=sparse_meta, workspace=workspace)
        settle(torch, lambda: R.lib().r355_gemm(ctypes.byref(g), None))
        # event-timed launches with the engine clock read meanwhile; short kernels run more launches so that the
        # sampler sees at least ~60 ms of them
        probe = R.gemm_timed(g, 5, 5)
        steps = max(args.steps, int(60.0 / max(probe, 1e-3)))
        ms, mhz, _ = clocks.measure(lambda: R.gemm_timed(g, args.warmup, steps), lead_s=args.warmup * probe * 1e-3)
        tf = 2.0 * mm * nn * kk / ms / 1e9
        rec = {"ms": round(ms, 4), "value": round(tf, 2), "unit": unit, "peak": peak * peak_scale,
               "frac": round(tf / (peak * peak_scale), 4), "launches_timed": steps,
               "validated": sampled_ok(in_t, out_t, la, lb, mm, nn, kk, a, b, d, sparse_rows)}
        rec.update(clock_fields(KIND[in_t], tf, mhz, cus, sparse=sparse_meta is not None))
        out[name] = with_counters(name, rec)
        if workspace is not None:  # split-K: the same problem with one workgroup per tile beside it
            out[name]["split_k"] = R.gemm_query(g).split_k
            g1 = R.gemm_args(in_t, out_t, mm, nn, kk, a, b, None, d, 1.0, 0.0, la, lb, R.ROW_MAJOR, R.ROW_MAJOR)
            out[name]["ms_without_workspace"] = round(R.gemm_timed(g1, args.warmup, args.steps), 4)

    if s == 8192:  # a problem with too few 256 x 256 tiles for the 256 CUs: the 128 x 128 macro tile
        gemm_case("gemm_f16_nt_2048x2048x8192", R.F16, R.F16, R.COL_MAJOR, R.ROW_MAJOR, rnd16(2048 * s, False),
                  rnd16(s * 2048, False), PEAK_TFLOPS["f16"], "TFLOP/s", mm=2048, nn=2048, kk=s)
    if s == 8192:  # few tiles and a long K: split-K over a caller-provided workspace (16 tiles of 128 x 128 x 16 shares of K)
        gemm_case("gemm_f16_nt_splitk_512x512x32768", R.F16, R.F16, R.COL_MAJOR, R.ROW_MAJOR, rnd16(512 * 32768, False),
                  rnd16(32768 * 512, False), PEAK_TFLOPS["f16"], "TFLOP/s", mm=512, nn=512, kk=32768,
                  workspace=torch.empty(32 * 512 * 512 * 4, dtype=torch.uint8, device="cuda"))
    if s == 8192:  # the reference perf sample's default size (samples/perf_hgemm.cpp:945): 784 tiles of 256 x 256 = 3 rounds
        # on 256 CUs + 16 tiles, which run on 128 x 128 tiles in a second launch (mixed tiling)
        # (f32 output: a kernel instantiation of its own, so that a kernel trace of this run keeps the headline's rows apart)
        gemm_case("gemm_f16_nt_f32out_7168", R.F16, R.F32, R.COL_MAJOR, R.ROW_MAJOR, rnd16(7168 * 7168, False),
                  rnd16(7168 * 7168, False), PEAK_TFLOPS["f16"], "TFLOP/s", mm=7168, nn=7168, kk=7168)
    if s == 8192:  # operands beyond the 256 MiB memory-side cache (2 x 256 MiB): the 16-bit 256 x 256 tile on its five-buffer K loop
        gemm_case("gemm_f16_tn_8192x8192x16384", R.F16, R.F16, R.ROW_MAJOR, R.COL_MAJOR, rnd16(s * 16384, False),
                  rnd16(16384 * s, False), PEAK_TFLOPS["f16"], "TFLOP/s", mm=s, nn=s, kk=16384)
    # f32 and f64 (the reference's perf_sgemm / perf_dgemm samples), TN
    for nm, it, dt, key in (("gemm_f32_tn_%d" % s, R.F32, torch.float32, "f32"), ("gemm_f64_tn_%d" % s, R.F64, torch.float64, "f64")):
        gemm_case(nm, it, it, R.ROW_MAJOR, R.COL_MAJOR, torch.rand(s * s, device="cuda", dtype=dt) * 2 - 1,
                  torch.rand(s * s, device="cuda", dtype=dt) * 2 - 1, PEAK_TFLOPS[key], "TFLOP/s")
    abf, bbf = rnd16(s * s, True), rnd16(s * s, True)
    gemm_case("gemm_bf16_nt_8192", R.BF16, R.BF16, R.COL_MAJOR, R.ROW_MAJOR, abf, bbf, PEAK_TFLOPS["bf16"], "TFLOP/s")
    af16, bf16_ = rnd16(s * s, False), rnd16(s * s, False)
    gemm_case("gemm_f16_tn_8192", R.F16, R.F16, R.ROW_MAJOR, R.COL_MAJOR, af16, bf16_, PEAK_TFLOPS["f16"], "TFLOP/s")
    # the same operands with an f32 result (f16 -> fp32 as the benchmark's target is worded; D is 256 MiB instead of 128)
    gemm_case("gemm_f16_nt_f32out_8192", R.F16, R.F32, R.COL_MAJOR, R.ROW_MAJOR, af16, bf16_, PEAK_TFLOPS["f16"], "TFLOP/s")
    i8 = lambda nel: torch.randint(-128, 128, (nel,), dtype=torch.int16, device="cuda").to(torch.int8)
    ai8, bi8 = i8(s * s), i8(s * s)
    gemm_case("gemm_i8_tn_8192", R.I8, R.I32, R.ROW_MAJOR, R.COL_MAJOR, ai8, bi8, PEAK_TFLOPS["i8"], "TOP/s")
    gemm_case("gemm_i8_nt_8192", R.I8, R.I32, R.COL_MAJOR, R.ROW_MAJOR, ai8, bi8, PEAK_TFLOPS["i8"], "TOP/s")
    # e4m3: N(0, 1) draws rounded to nearest-even and saturated to the finite range (|x| <= 448;
    # scale 1.0, so saturation never triggers in practice)
    f8 = lambda nel: torch.randn(nel, device="cuda").clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    af8, bf8 = f8(s * s), f8(s * s)
    gemm_case("gemm_e4m3_tn_8192", R.E4M3, R.F32, R.ROW_MAJOR, R.COL_MAJOR, af8, bf8, PEAK_TFLOPS["e4m3"], "TFLOP/s")
    out["same_box_comparison"] = same_box_comparison(torch, args, s, af16, bf16_, abf, bbf, ai8, bi8, af8, bf8)
    # 2:4 sparse, benchmark configuration 4: M = N = 4096, dense-equivalent K = 8192, int8 and fp8 e4m3; dense-equivalent
    # ops against the sparse peak (2 x dense).  A is drawn dense on the host -- seeded values under a seeded mask that keeps 2 of
    # every group of 4 along k at random positions -- and compressed with the library's own r355_compress_24; sampled complete
    # rows of D are held against the oracle's dense GEMM on the uncompressed A (int8: bit for bit).
    # (third row: a quarter of the size, 64 tiles of 256 x 256 - the shape class the 128 x 128 sparse tile is for)
    sk = 8192
    for name, in_t, out_t, key, unit, sm in (("gemm_i8_sparse24_4096x4096x8192", R.I8, R.I32, "i8", "TOP/s (dense-equivalent)", 4096),
                                             ("gemm_e4m3_sparse24_4096x4096x8192", R.E4M3, R.F32, "e4m3", "TFLOP/s (dense-equivalent)", 4096),
                                             ("gemm_i8_sparse24_2048x2048x8192", R.I8, R.I32, "i8", "TOP/s (dense-equivalent)", 2048),
                                             # (beyond the benchmark's configurations: the 16-bit sparse instruction, U[-1, 1] operands)
                                             ("gemm_f16_sparse24_4096x4096x8192", R.F16, R.F32, "f16", "TFLOP/s (dense-equivalent)", 4096)):
        sn = sm
        mask = O.sparse24_mask(60, sm, sk)
        srows = np.array([0, 31, 32, 1234, 2047, sm // 2, sm - 32, sm - 1], dtype=np.uint32)
        if in_t == R.I8:
            av, bh = O.uniform_int8(61, sm * sk).reshape(sm, sk), O.uniform_int8(62, sk * sn)
        elif in_t == R.F16:
            av = O.f32_to_storage(O.uniform_pm1(61, sm * sk), O.F16).reshape(sm, sk)
            bh = O.f32_to_storage(O.uniform_pm1(62, sk * sn), O.F16)
        else:
            av = O.f32_to_storage(O.normal(61, sm * sk), O.E4M3).view(np.int8).reshape(sm, sk)
            bh = O.f32_to_storage(O.normal(62, sk * sn), O.E4M3)
        dense = np.where(mask, av, av.dtype.type(0)).astype(av.dtype)
        vals, meta = R.compress_24(dense)
        storage = dense.view(np.uint8) if in_t == R.E4M3 else dense
        want = O.gemm_rows(in_t, out_t, O.ROW, O.COL, sm, sn, sk, storage.ravel(), bh, srows)
        gemm_case(name, in_t, out_t, R.ROW_MAJOR, R.COL_MAJOR, torch.from_numpy(np.ascontiguousarray(vals).view(np.uint8)).cuda(),
                  torch.from_numpy(bh.view(np.uint8)).cuda(), PEAK_TFLOPS[key], unit,
                  sparse_meta=torch.from_numpy(meta).cuda(), mm=sm, nn=sn, kk=sk, peak_scale=2.0, sparse_rows=(srows, want))
        del av, bh, dense, vals, meta, storage, mask
    # DLRM dot interaction forward, benchmark configuration 5
    bsz, mm, kk = 65536, 27, 128
    x = torch.randn(bsz * mm * kk, device="cuda").to(torch.float16)
    o = torch.empty(bsz * (kk + mm * (mm - 1) // 2), dtype=torch.float16, device="cuda")
    settle(torch, lambda: R.dlrm_fwd(R.F16, x, o, mm, kk, bsz))
    ms = R.dlrm_fwd_timed(R.F16, x, o, mm, kk, bsz, args.warmup, args.steps)
    byts = bsz * (mm * kk + kk + mm * (mm - 1) // 2) * 2
    out["dlrm_fwd_b65536_f27_d128"] = with_counters("dlrm_fwd_b65536_f27_d128", {
        "ms": round(ms, 4), "value": round(byts / ms / 1e6, 1), "unit": "GB/s", "peak": HBM_PEAK_GBPS,
        "frac": round(byts / ms / 1e6 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": byts,
        "gflops_ref_convention": round(2.0 * mm * mm * kk * bsz / ms / 1e6, 1),
        "validated": bool(torch.isfinite(o.float()).all()) and dlrm_ok(x, o, None, None, None, bsz, mm, kk, 2e-3)})
    # DLRM backward on the same shape: reads X and the upstream gradient, writes both gradients
    up = torch.randn(bsz * (kk + mm * (mm - 1) // 2), device="cuda").to(torch.float16)
    gmlp = torch.empty(bsz * kk, dtype=torch.float16, device="cuda")
    gin = torch.empty(bsz * mm * kk, dtype=torch.float16, device="cuda")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    settle(torch, lambda: R.dlrm_bwd(R.F16, x, up, gmlp, gin, mm, kk, bsz))
    for it in range(args.warmup + args.steps):
        if it == args.warmup:
            e0.record()  # the C ABI launches on the null stream, which torch's default stream is
        R.dlrm_bwd(R.F16, x, up, gmlp, gin, mm, kk, bsz)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    byts = (2 * bsz * mm * kk + bsz * (kk + mm * (mm - 1) // 2) + bsz * kk) * 2
    out["dlrm_bwd_b65536_f27_d128"] = with_counters("dlrm_bwd_b65536_f27_d128", {
        "ms": round(ms, 4), "value": round(byts / ms / 1e6, 1), "unit": "GB/s", "peak": HBM_PEAK_GBPS,
        "frac": round(byts / ms / 1e6 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": byts,
        "validated": bool(torch.isfinite(gin.float()).all() and torch.isfinite(gmlp.float()).all())
        and dlrm_ok(x, None, up, gmlp, gin, bsz, mm, kk, 4e-3)})
    del up, gmlp, gin, x, o
    # the same DLRM configuration in f32 (the reference's second DLRM type: test/dlrm/test/dlrm_test_params.hpp:50-53)
    x32 = torch.randn(bsz * mm * kk, device="cuda")
    o32 = torch.empty(bsz * (kk + mm * (mm - 1) // 2), device="cuda")
    up32 = torch.randn(bsz * (kk + mm * (mm - 1) // 2), device="cuda")
    gmlp32, gin32 = torch.empty(bsz * kk, device="cuda"), torch.empty(bsz * mm * kk, device="cuda")

    def event_ms(fn):
        settle(torch, fn)
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for it in range(args.warmup + args.steps):
            if it == args.warmup:
                a0.record()
            fn()
        a1.record()
        torch.cuda.synchronize()
        return a0.elapsed_time(a1) / args.steps

    def hbm_case(name, ms, byts, ok, note=None):
        out[name] = {"ms": round(ms, 4), "value": round(byts / ms / 1e6, 1), "unit": "GB/s", "peak": HBM_PEAK_GBPS,
                     "frac": round(byts / ms / 1e6 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": byts, "validated": ok}
        if note:
            out[name]["note"] = note

    ms = event_ms(lambda: R.dlrm_fwd(R.F32, x32, o32, mm, kk, bsz))
    hbm_case("dlrm_fwd_f32_b65536_f27_d128", ms, bsz * (mm * kk + kk + mm * (mm - 1) // 2) * 4,
             bool(torch.isfinite(o32).all()) and dlrm_ok(x32, o32, None, None, None, bsz, mm, kk, 1e-5))
    ms = event_ms(lambda: R.dlrm_bwd(R.F32, x32, up32, gmlp32, gin32, mm, kk, bsz))
    hbm_case("dlrm_bwd_f32_b65536_f27_d128", ms, (2 * bsz * mm * kk + bsz * (kk + mm * (mm - 1) // 2) + bsz * kk) * 4,
             bool(torch.isfinite(gin32).all() and torch.isfinite(gmlp32).all()) and dlrm_ok(x32, None, up32, gmlp32, gin32, bsz, mm, kk, 1e-5))
    del x32, o32, up32, gmlp32, gin32
    # few features (8 x 64, f16): the kernels take four consecutive samples as one block of rows
    fm, fk = 8, 64
    fstride = fk + fm * (fm - 1) // 2
    x8 = torch.randn(bsz * fm * fk, device="cuda").to(torch.float16)
    o8 = torch.empty(bsz * fstride, dtype=torch.float16, device="cuda")
    up8 = torch.randn(bsz * fstride, device="cuda").to(torch.float16)
    gmlp8 = torch.empty(bsz * fk, dtype=torch.float16, device="cuda")
    gin8 = torch.empty(bsz * fm * fk, dtype=torch.float16, device="cuda")
    ms = event_ms(lambda: R.dlrm_fwd(R.F16, x8, o8, fm, fk, bsz))
    hbm_case("dlrm_fwd_b65536_f8_d64", ms, bsz * (fm * fk + fstride) * 2,
             bool(torch.isfinite(o8.float()).all()) and dlrm_ok(x8, o8, None, None, None, bsz, fm, fk, 2e-3))
    ms = event_ms(lambda: R.dlrm_bwd(R.F16, x8, up8, gmlp8, gin8, fm, fk, bsz))
    hbm_case("dlrm_bwd_b65536_f8_d64", ms, (2 * bsz * fm * fk + bsz * fstride + bsz * fk) * 2,
             bool(torch.isfinite(gin8.float()).all() and torch.isfinite(gmlp8.float()).all())
             and dlrm_ok(x8, None, up8, gmlp8, gin8, bsz, fm, fk, 4e-3))
    del x8, o8, up8, gmlp8, gin8
    # GEMV y = A x (the reference's simple_sgemv / simple_dgemv samples), A read once: bytes of A, x and y over the HBM peak;
    # checked against a float64 product on sampled rows
    # The HBM fraction of GEMV is the one of the 16384^2 cases (1 GiB of A, four times the 256 MiB memory-side cache, read with
    # nontemporal loads).  The 8192^2 f32 matrix is exactly the size of that cache and the f64 one twice it: launched again and
    # again as here, part of A is served from the cache, so those rows are labelled cache-assisted and are not HBM rates.
    cache_note = "cache-assisted: A (%d MiB) is within reach of the 256 MiB memory-side cache across the repeated launches; not an HBM rate"
    for name, dt, fn, gm, gk in (("gemv_f32_col_16384", torch.float32, R.gemv, 16384, 16384), ("gemv_f32_row_16384", torch.float32, R.gemv, 16384, 16384),
                                 ("gemv_f32_col_8192", torch.float32, R.gemv, 8192, 8192), ("gemv_f64_col_8192", torch.float64, R.dgemv, 8192, 8192)):
        lay = R.COL_MAJOR if "_col_" in name else R.ROW_MAJOR
        av = torch.rand(gm * gk, device="cuda", dtype=dt) * 2 - 1
        xv = torch.rand(gk, device="cuda", dtype=dt) * 2 - 1
        yv = torch.empty(gm, device="cuda", dtype=dt)
        ms = event_ms(lambda: fn(lay, gm, gk, av, xv, None, yv, 1.0, 0.0))
        rows = torch.arange(0, gm, gm // 64, device="cuda")
        amat = av.view(gm, gk) if lay == R.ROW_MAJOR else av.view(gk, gm).t()
        want = amat[rows].double() @ xv.double()
        ok = bool(((yv[rows].double() - want).abs() <= 1e-4 * (want.abs() + 1.0)).all())
        a_mib = gm * gk * av.element_size() >> 20
        hbm_case(name, ms, (gm * gk + gm + gk) * av.element_size(), ok, cache_note % a_mib if a_mib <= 512 else None)
        del av, xv, yv
    # K split over several workgroups per block of rows (r355_gemv_ws): a col-major A with few rows, whose plain launch has
    # eight workgroups, and a row count just above what fills the CUs (260 blocks of 64 rows)
    for name, gm, gk in (("gemv_f32_col_splitk_256x1048576", 256, 1048576), ("gemv_f32_col_splitk_16640x16384", 16640, 16384)):
        av = torch.rand(gm * gk, device="cuda") * 2 - 1
        xv = torch.rand(gk, device="cuda") * 2 - 1
        yv = torch.empty(gm, device="cuda")
        need = R.gemv_workspace_bytes(R.COL_MAJOR, gm, gk, 4)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        ms = event_ms(lambda: R.gemv(R.COL_MAJOR, gm, gk, av, xv, None, yv, 1.0, 0.0, workspace=ws))
        rows = torch.arange(0, gm, gm // 64, device="cuda")
        want = av.view(gk, gm).t()[rows].double() @ xv.double()
        ok = need > 0 and bool(((yv[rows].double() - want).abs() <= 1e-4 * (want.abs() + 1.0)).all())
        hbm_case(name, ms, (gm * gk + gm + gk) * 4, ok, "plain r355_gemv on this shape: %.4f ms" % event_ms(
            lambda: R.gemv(R.COL_MAJOR, gm, gk, av, xv, None, yv, 1.0, 0.0)))
        del av, xv, yv, ws
    return out


def same_box_comparison(torch, args, s, af16, bf16_, abf, bbf, ai8, bi8, af8, bf8):
    """Context only, never part of `value`: the vendor GEMM library as torch dispatches it, on the same
    operand bits and shapes as the cases above, and -- where its shared object was built -- the kernel of
    the reference's samples/perf_hgemm.cpp (macro tile 128 x 128 x 16, samples/perf_hgemm.cpp:224-237,
    515-711) compiled unchanged against this library's headers."""
    res, flop = {}, 2.0 * s * s * s

    def timed(fn):
        settle(torch, fn)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = args.steps
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    def case(name, fn, unit="TFLOP/s"):
        try:
            ms = timed(fn)
            res[name] = {"ms": round(ms, 4), "value": round(flop / ms / 1e9, 2), "unit": unit}
        except Exception as e:  # a library without this type pair is not an error of this benchmark
            res[name] = {"error": repr(e)[:160]}

    v = lambda t, dt=None: (t if dt is None else t.view(dt)).view(s, s)
    case("torch_matmul_f16_nt", lambda: torch.matmul(v(af16).t(), v(bf16_)))
    case("torch_matmul_f16_tn", lambda: torch.matmul(v(af16), v(bf16_).t()))
    case("torch_matmul_bf16_nt", lambda: torch.matmul(v(abf).t(), v(bbf)))
    case("torch_int_mm_i8_tn", lambda: torch._int_mm(v(ai8), v(bi8).t()), "TOP/s")
    one = torch.ones((), device="cuda")
    f8t = torch.float8_e4m3fn
    case("torch_scaled_mm_e4m3_tn_f32", lambda: torch._scaled_mm(v(af8, f8t), v(bf8, f8t).t(), scale_a=one, scale_b=one,
                                                                 out_dtype=torch.float32))
    lib = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "kernels", "_ref", "libref_perf_hgemm.so")
    if os.path.exists(lib):
        L = ctypes.CDLL(lib)
        d = torch.empty(s * s, dtype=torch.float16, device="cuda")
        P = lambda t: ctypes.c_void_p(t.data_ptr())

        def ref():  # the wrapper synchronises after each launch
            if L.ref_perf_hgemm(s, s, s, P(af16), P(bf16_), P(d), P(d), s, s, s, s, ctypes.c_float(1.0),
                                ctypes.c_float(0.0)) != 0:
                raise RuntimeError("reference sample kernel failed")

        case("reference_perf_hgemm_kernel_f16_nt", ref)
    return res


if __name__ == "__main__":
    main()
