#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Headline workload: D = A*B + C at M = N = K = 8192 with f16 and with
bf16 inputs, f32 C/D, all four A/B layout combinations.  One "step" is one pass over those
eight GEMMs; the reported value is total flops / total time in TFLOP/s (2*M*N*K per GEMM,
reference formula test/performance.hpp:424-433).  Inputs are synthetic, uniform[-1, 1], already
resident in HBM when the timed region starts.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline     : the dominant kernel (f16, A row-major, B col-major) against the 2.5 PFLOP/s dense
                 f16 MFMA peak, timed with events on the launch stream; next to the nominal peak,
                 what a loop of nothing but matrix instructions sustains on this box on the same
                 operand distribution and on all-zero operands (the part is power managed and the
                 sustained rate depends on the operand bits), and the same kernel on all-zero operands;
  cpu_baseline : the CPU oracle (a port of the reference's OpenMP gemm_CPU) timed on this box's
                 host cores on a bounded sample of the same workload; the rows it computes also
                 check the GPU result of the timed case (outside the timed region);
  extra        : the other configurations (quantised GEMMs, GEMV, DLRM) with their own rooflines.

--only NAME runs one case alone (for profiling): a headline case (f16_rc, bf16_cr, ...: dtype_{A}{B}
layouts) or one of the extra cases by its key in the JSON line (gemm_fp8_m4096, gemm_i8_m128,
gemv_8192x8192_n8, dlrm_bwd_b262144, ...).
"""
import argparse
import ctypes
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "fp8": 5000.0, "i8": 5000.0}  # dense MFMA, MI355X
PEAK_HBM_GBS = 8000.0
FP8_BLOCKED_SHAPE = "fp8_16x16x128"  # the matrix instruction of the blocked kernel's 256 x 256 fp8 configuration (A row / B col)
# Bytes moved through the L2s per launch come from rocprofv3 counter runs of this file (counters cannot
# be read from inside this process): profiles/traffic.json holds the figures of the committed counter
# summaries together with a digest of the kernel sources they were taken on, and a figure whose digest
# no longer matches is reported as null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
KERNEL_SOURCES = {
    "gemm_blocked": ["rocwmma_amd/csrc/gemm_blocked.hip", "rocwmma_amd/csrc/gemm_blocked_launch.hpp",
                     "rocwmma_amd/csrc/gemm_blocked_core.hpp", "include/rocwmma/rocwmma_lds.hpp"],
}


def sources_digest(family):
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES[family]:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(key, family):
    """Bytes per launch recorded for `key`, or None when nothing current is recorded."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f).get(key)
    except (OSError, ValueError):
        return None
    if not rec or rec.get("sources_digest") != sources_digest(family):
        return None
    return rec.get("bytes")


def record_traffic(spec):
    """--record-traffic KEY:FAMILY:FETCH_KIB:WRITE_KIB:COPY_FETCH_KIB:COPY_WRITE_KIB -- store what a pair of
    rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE: per-dispatch averages of the kernel, in the counters' own
    units) read for case KEY, scaled by what the same counters read for the 1 GiB copy of --calibrate-copy,
    together with the digest of the kernel sources it was measured on."""
    key, family, fetch, write, cfetch, cwrite = spec.split(":")
    gib_kib = float(1 << 20)
    f_factor, w_factor = gib_kib / float(cfetch), gib_kib / float(cwrite)
    byts = (float(fetch) * f_factor + float(write) * w_factor) * 1024.0
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    table[key] = {"bytes": round(byts), "fetch_size": float(fetch), "write_size": float(write),
                  "fetch_factor": round(f_factor, 3), "write_factor": round(w_factor, 3),
                  "sources_digest": sources_digest(family)}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({key: table[key]}))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--size", type=int, default=8192, help="M = N = K of the headline GEMM")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 1 GiB device copy (known traffic) for counter calibration")
    ap.add_argument("--shapes", action="store_true",
                    help="also time GEMM shapes below the headline size, one per kernel / tile configuration "
                         "(extra.shapes in the JSON line)")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the MFMA-only ceiling loops and the all-zero-operand run (counter runs)")
    ap.add_argument("--record-traffic", default=None, metavar="KEY:FAMILY:FETCH:WRITE:COPY_FETCH:COPY_WRITE",
                    help="no GPU work: rewrite the entry of profiles/traffic.json for one case from counter readings")
    ap.add_argument("--only", default=None,
                    help="run one case only: a headline case such as f16_rc (dtype_{r|c}{r|c} = A,B layout) or an "
                         "extra case by its JSON key (gemm_fp8_m4096, gemv_8192x8192_n8, ...): for profiling")
    return ap.parse_args()


def compute_units_of(rw):
    return rw.device_info()["compute_units"]


def event_ms(fn, iters, torch):
    """Average duration of fn() in ms over `iters` launches, events on the current stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def graph_ms(fn, iters, torch):
    """Average duration of fn() in ms with `iters` launches recorded into one HIP graph and the graph
    replayed: the kernels then run back to back without per-launch host work, which is what a
    microsecond-scale kernel's own duration needs (a Python loop issues a launch every 6-9 us).
    None when the capture is not possible."""
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            graph.replay()
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop) / iters
            best = ms if best is None or ms < best else best
        return best
    except Exception:  # capture refused: the event-timed figure stands alone
        try:
            torch.cuda.synchronize()
        except Exception:
            pass
        return None


def launch_stats(fn, iters, torch):
    """(median, min) duration in ms of single launches of fn(), one event pair per launch."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in pairs)
    return t[len(t) // 2], t[0]


class ClockSampler:
    """Samples the shader clock the driver reports (the starred line of pp_dpm_sclk in sysfs) every 2 ms from a
    thread while launches run.  The reference prices a kernel against Multiplier x CUs x *current* MHz read
    from rocm_smi (test/performance.hpp:435-442, test/hip_device.cpp:104-136); this is that clock.  mhz() is
    None where the file does not exist or cannot be read."""

    def __init__(self):
        import glob

        self.paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.samples = []

    def _read(self):
        try:
            with open(self.paths[0]) as f:
                for line in f:
                    if "*" in line:
                        return float(line.split(":")[1].lower().split("mhz")[0])
        except (OSError, ValueError, IndexError):
            pass
        return None

    def __enter__(self):
        import threading

        self.stop = threading.Event()

        def run():
            while not self.stop.is_set():
                v = self._read()
                if v is not None:
                    self.samples.append(v)
                time.sleep(0.002)

        self.thread = threading.Thread(target=run, daemon=True)
        if self.paths:
            self.thread.start()
        return self

    def __exit__(self, *exc):
        self.stop.set()
        if self.paths:
            self.thread.join()

    def mhz(self):
        if not self.samples:
            return None
        t = sorted(self.samples)
        return t[len(t) // 2]


HEADLINE_TAGS = [f"{d}_{a}{b}" for d in ("f16", "bf16") for a in "rc" for b in "rc"]


def main():
    args = parse_args()
    if args.record_traffic:
        record_traffic(args.record_traffic)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import rocwmma_amd as rw

    if not os.path.exists(rw.library_path()) or not os.path.exists(rw.aux_library_path()):
        import __graft_entry__ as g

        g.build()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    info = rw.device_info()
    assert info["is_gfx950"], info
    dev = torch.device("cuda:0")
    RM, CM = rw.ROW_MAJOR, rw.COL_MAJOR
    S = args.size
    gen = torch.Generator(device=dev).manual_seed(0x5EED0002)

    if args.calibrate_copy:
        # reads 1 GiB, writes 1 GiB: the reference point FETCH_SIZE / WRITE_SIZE are scaled by
        src = torch.ones(1 << 28, device=dev, dtype=torch.float32)
        dst = torch.empty_like(src)
        ms = event_ms(lambda: dst.copy_(src), 5, torch)
        print(json.dumps({"calibrate_copy_bytes_each_way": src.numel() * 4, "ms": round(ms, 4),
                          "gbs": round(2 * src.numel() * 4 / ms / 1e6, 1)}))
        return

    if args.only and args.only not in HEADLINE_TAGS:
        # one extra case alone (profiling): a few launches, nothing else on the device
        out = run_extras(rw, torch, dev, gen, only=args.only)
        assert out, f"no case matches --only {args.only}"
        print(json.dumps({"only": args.only, "device": info, "result": out}))
        return

    def rand(count, dtype):
        return (torch.rand(count, device=dev, generator=gen) * 2 - 1).to(dtype)

    # ------------------------------------------------------------------ headline: 8 GEMMs
    data = {
        "f16": (rw.F16, rand(S * S, torch.float16), rand(S * S, torch.float16)),
        "bf16": (rw.BF16, rand(S * S, torch.bfloat16), rand(S * S, torch.bfloat16)),
    }
    C = rand(S * S, torch.float32)
    D = torch.empty(S * S, device=dev, dtype=torch.float32)
    cases = []
    for name, (code, A, B) in data.items():
        for la in (RM, CM):
            for lb in (RM, CM):
                tag = f"{name}_{'rc'[la]}{'rc'[lb]}"
                if args.only and tag != args.only:
                    continue
                cases.append((tag, code, la, lb, A, B))
    assert cases, f"no case matches --only {args.only}"

    def run_case(case):
        _, code, la, lb, A, B = case
        rw.gemm(code, rw.F32, la, lb, RM, S, S, S, A, B, C, D, 1.0, 1.0)

    def step():
        for case in cases:
            run_case(case)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    flops_per_gemm = 2.0 * S * S * S
    value = flops_per_gemm * len(cases) / (ms_per_step * 1e-3) / 1e12

    # per-case kernel time (events on the launch stream)
    per_case = {}
    for case in cases:
        ms = event_ms(lambda: run_case(case), max(args.steps, 5), torch)
        med, best = launch_stats(lambda: run_case(case), 20, torch)
        per_case[case[0]] = {"ms": round(ms, 4), "tflops": round(flops_per_gemm / ms / 1e9, 1),
                             "ms_median": round(med, 4), "ms_min": round(best, 4)}
    dom = "f16_rc" if "f16_rc" in per_case else cases[0][0]
    dom_dtype = "bf16" if dom.startswith("bf16") else "f16"
    dom_peak = PEAK_TFLOPS[dom_dtype]
    roofline = {
        "bound": "mfma", "kernel": f"gemmBlockedKernel {dom} {S}^3",
        "achieved": per_case[dom]["tflops"], "peak": dom_peak, "unit": "TFLOP/s",
        "frac": round(per_case[dom]["tflops"] / dom_peak, 4),
        "traffic": measured_traffic(f"{dom}_{S}", "gemm_blocked"),
        "ms": per_case[dom]["ms"],
    }

    # The shader clock the driver reports while the dominant kernel runs back to back (about 50 launches),
    # next to the nominal clock the peak is quoted at, and the kernel against the peak at that clock: the
    # reference's own efficiency definition.
    dom_case_ = next(c for c in cases if c[0] == dom)
    with ClockSampler() as clk:
        event_ms(lambda: run_case(dom_case_), 50, torch)
    roofline["nominal_clock_mhz"] = info.get("clock_mhz")
    roofline["observed_clock_mhz"] = clk.mhz()
    if clk.mhz() and info.get("clock_mhz"):
        roofline["frac_of_peak_at_observed_clock"] = round(
            per_case[dom]["tflops"] / (dom_peak * clk.mhz() / info["clock_mhz"]), 4)

    # The matrix pipes' own ceiling on this box (no memory traffic at all) for the dominant kernel's
    # instruction, on this operand distribution and on all-zero operands, and the dominant kernel on
    # all-zero operands: the gap between the two operand patterns is the device's power management,
    # not the kernel's schedule.
    if (not args.only or args.only == dom) and not args.no_ceiling:
        ceiling = run_ceiling(rw, torch, dev, gen, [dom_dtype] if args.only else None)
        key = f"{dom_dtype}_16x16x32"
        dom_case = next(c for c in cases if c[0] == dom)
        zeros = torch.zeros(S * S, device=dev, dtype=dom_case[4].dtype)
        rw.gemm(dom_case[1], rw.F32, dom_case[2], dom_case[3], RM, S, S, S, zeros, zeros, C, D, 1.0, 1.0)
        ms_zero = event_ms(lambda: rw.gemm(dom_case[1], rw.F32, dom_case[2], dom_case[3], RM, S, S, S, zeros, zeros,
                                           C, D, 1.0, 1.0), max(args.steps, 5), torch)
        del zeros
        roofline["mfma_only_ceiling"] = ceiling
        roofline["frac_of_mfma_only_ceiling"] = round(per_case[dom]["tflops"] / ceiling[key]["data"], 4)
        # What the device sustains when the tile's matrix instructions run next to the byte streams a 256 x 256
        # tile of 16-bit operands needs (192 KiB of LDS reads and 64 KiB of L2 -> LDS copies per 64 of K per compute
        # unit) and nothing else -- no barrier, no tile bookkeeping, no epilogue: the ceiling of the tiling itself on
        # this power-managed part, on the benchmark's operands and on all-zero ones.
        if S == 8192 and dom_dtype == "f16":
            streams = run_streams_ceiling(rw, torch, dev, gen, dom_case[4], dom_case[5])
            roofline["mfma_with_operand_streams"] = streams
            roofline["frac_of_operand_streams_ceiling"] = round(per_case[dom]["tflops"] / streams["data"]["with_lds_reads_and_l2_copies"], 4)
            if not args.only:
                # the same for the instructions of the 8-bit kernels (same byte streams: 128 bytes of K per row and stage),
                # on the operand distributions of the quantised cases
                n8 = 8192 * 16384
                a8 = torch.randint(-128, 128, (n8,), device=dev, dtype=torch.int8, generator=gen)
                b8 = torch.randint(-128, 128, (n8,), device=dev, dtype=torch.int8, generator=gen)
                roofline["mfma_with_operand_streams_8bit"] = {"i8_16x16x64": run_streams_ceiling(rw, torch, dev, gen, a8, b8, rw.STREAMS_I8)}
                del a8, b8
                a8 = (torch.randn(n8, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
                b8 = (torch.randn(n8, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
                roofline["mfma_with_operand_streams_8bit"]["fp8_16x16x128"] = run_streams_ceiling(rw, torch, dev, gen, a8, b8, rw.STREAMS_FP8)
                del a8, b8
        roofline["zero_operands"] = {
            "ms": round(ms_zero, 4), "tflops": round(flops_per_gemm / ms_zero / 1e9, 1),
            "frac": round(flops_per_gemm / ms_zero / 1e9 / dom_peak, 4),
            "frac_of_mfma_only_ceiling": round(flops_per_gemm / ms_zero / 1e9 / ceiling[key]["zero"], 4),
        }

    # ------------------------------------------------------------------ CPU baseline (oracle port)
    cpu_baseline = None
    if not args.no_cpu_baseline and "f16_rc" in per_case:
        import oracle as orc

        rows_n = 1024 if S >= 4096 else S
        rows = np.arange(0, S, S // rows_n, dtype=np.uint32)[:rows_n]
        code, A, B = data["f16"]
        a_bits = A.view(torch.int16).cpu().numpy().view(np.uint16)
        b_bits = B.view(torch.int16).cpu().numpy().view(np.uint16)
        c_host = C.cpu().numpy()
        t0 = time.perf_counter()
        want = orc.gemm(orc.F16, orc.F32, 0, 1, 0, 0, S, S, S, a_bits, b_bits, c_host, 1.0, 1.0, rows=rows)
        dt = time.perf_counter() - t0
        # the same rows of the GPU result of the timed f16 A-row / B-col case, outside the timed region
        D.fill_(float("nan"))
        run_case(next(c for c in cases if c[0] == "f16_rc"))
        torch.cuda.synchronize()
        got = D.view(S, S)[torch.from_numpy(rows.astype(np.int64)).to(dev)].cpu().numpy().ravel()
        ref = want.reshape(S, S)[rows].ravel()
        err, inf, nan = orc.compare_equal(orc.F32, got, orc.F32, ref)
        assert not inf and not nan and err <= 1e-3, f"timed GEMM differs from the CPU oracle: {err} {inf} {nan}"
        assert not bool(torch.isnan(D).any()), "NaN left in D after the timed case"
        cpu_baseline = {
            "value": round(2.0 * rows.size * S * S / dt / 1e12, 5), "unit": "TFLOP/s",
            "cores": orc.num_threads(), "kind": "port",
            "sample": f"{rows.size} of {S} output rows (every column) of the f16 A-row/B-col {S}^3 case, "
                      f"{dt:.1f} s incl. operand decode",
            "gpu_result_checked": {"rows": int(rows.size), "max_rel_err": float(f"{err:.3e}"), "tolerance": 1e-3},
        }
        del a_bits, b_bits, c_host, want

    # ------------------------------------------------------------------ other configurations
    extra = {"device": info, "cases": per_case}
    if not args.no_extras and not args.only:
        extra.update(run_extras(rw, torch, dev, gen))
        # the MFMA-bound quantised case against the matrix pipes' own ceiling for its instruction
        for key, shape in (("gemm_i8_m4096", "i8_16x16x64"), ("gemm_fp8_m4096", FP8_BLOCKED_SHAPE),
                           ("gemm_i8_8192cubed", "i8_16x16x64"), ("gemm_fp8_8192cubed", FP8_BLOCKED_SHAPE)):
            if key in extra and shape in roofline.get("mfma_only_ceiling", {}):
                extra[key]["frac_of_mfma_only_ceiling"] = round(
                    extra[key]["tops"] / roofline["mfma_only_ceiling"][shape]["data"], 4)
            if key in extra and shape in roofline.get("mfma_with_operand_streams_8bit", {}):
                # (main loop only: these launches also write 224 MiB of D, a quarter of their time)
                extra[key]["frac_of_operand_streams_ceiling"] = round(
                    extra[key]["tops"] / roofline["mfma_with_operand_streams_8bit"][shape]["data"]["with_lds_reads_and_l2_copies"], 4)
    if args.shapes:
        extra["shapes"] = run_shapes(rw, torch, dev, gen)

    print(json.dumps({
        "metric": "gemm_tflops_8192cubed_f16_bf16_4layouts", "value": round(value, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16/bf16 in, f32 accumulate",
        "data": "synthetic uniform[-1,1], resident in HBM",
        "config": {"workload": f"D = A*B + C, M=N=K={S}, f16 and bf16 inputs, f32 C/D, A,B in row/col x row/col "
                               f"({len(cases)} GEMMs per step), alpha=beta=1"},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "extra": extra,
    }))


def run_streams_ceiling(rw, torch, dev, gen, A, B, kind=None):
    """T(FL)OP/s of the matrix-pipes-next-to-their-operand-streams probe (rocwmma_amd_bench_mfma_streams): matrix
    instructions only, with the LDS fragment reads, with those and the global -> LDS copies; on the operands of
    the timed GEMM (A, B: 128 MiB each, rows of 16 KiB) and on all-zero ones.  Ten launches of four tiles per compute
    unit after ten warm-up launches."""
    kind = rw.STREAMS_F16 if kind is None else kind
    bytes_a = A.view(torch.uint8)
    tables = {"data": (bytes_a[: 65536].contiguous(), A, B),
              "zero": (torch.zeros(65536, device=dev, dtype=torch.uint8), torch.zeros_like(A), None)}
    sink = torch.empty(rw.device_info()["compute_units"] * 512, device=dev)
    out = {}
    for label, (table, a_, b_) in tables.items():
        b_ = a_ if b_ is None else b_
        res = {}
        for name, streams in (("mfma_only", 0), ("with_lds_reads", 1), ("with_lds_reads_and_l2_copies", 3)):
            fn = lambda: rw.bench_mfma_streams(streams, 4, a_, b_, table, sink, kind)
            ops = fn()
            for _ in range(9):
                fn()
            ms = event_ms(fn, 10, torch)
            res[name] = round(ops / ms / 1e9, 1)
        out[label] = res
    return out


def run_ceiling(rw, torch, dev, gen, dtypes=None):
    """TFLOP/s (TOP/s) of a loop of nothing but matrix instructions, two waves per SIMD on every compute
    unit, operands in registers: per instruction shape, on the benchmark's operand distribution for
    that type ("data") and on all-zero operands ("zero").  Each figure is a launch of about 10 ms
    after a warm-up launch of the same length (shorter launches still see the clock ramp)."""
    n = 65536
    tables = {
        "f16": (torch.rand(n // 2, device=dev, generator=gen) * 2 - 1).to(torch.float16).view(torch.uint8),
        "bf16": (torch.rand(n // 2, device=dev, generator=gen) * 2 - 1).to(torch.bfloat16).view(torch.uint8),
        "i8": torch.randint(-128, 128, (n,), device=dev, dtype=torch.int8, generator=gen).view(torch.uint8),
        "fp8": (torch.randn(n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn).view(torch.uint8),
        "zero": torch.zeros(n, device=dev, dtype=torch.uint8),
    }
    shapes = [("f16_16x16x32", rw.MFMA_F16_16X16X32, "f16", 20000), ("f16_32x32x16", rw.MFMA_F16_32X32X16, "f16", 7000),
              ("bf16_16x16x32", rw.MFMA_BF16_16X16X32, "bf16", 20000), ("i8_16x16x64", rw.MFMA_I8_16X16X64, "i8", 20000),
              ("fp8_32x32x64", rw.MFMA_F8_32X32X64, "fp8", 5000), ("fp8_16x16x128", rw.MFMA_F8_16X16X128, "fp8", 10000),
              ("fp8_16x16x128_scaled", rw.MFMA_F8_16X16X128_SCALED, "fp8", 10000)]
    sink = torch.empty(info_lanes(rw), device=dev)
    out = {}
    for name, shape, kind, trips in shapes:
        if dtypes is not None and kind not in dtypes:
            continue
        res = {}
        for label, table in (("data", tables[kind]), ("zero", tables["zero"])):
            rw.bench_mfma_ceiling(shape, trips, 2, table, sink)
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            ops = rw.bench_mfma_ceiling(shape, trips, 2, table, sink)
            stop.record()
            stop.synchronize()
            res[label] = round(ops / start.elapsed_time(stop) / 1e9, 1)
        out[name] = res
    return out


def info_lanes(rw):
    return rw.device_info()["compute_units"] * 2 * 256


def run_shapes(rw, torch, dev, gen):
    """GEMM shapes off the headline size, through AUTO, one or two per kernel / rung of the tile
    ladder: microseconds per launch with the weights rotated over buffers of more than 256 MiB in
    total (so they come from HBM), A row-major / B col-major unless noted."""
    RM, CM = rw.ROW_MAJOR, rw.COL_MAJOR
    shapes = [
        # dtype, m, n, k, (layout a, layout b), what serves it on a 256-unit device
        ("f16", 16, 14336, 4096, (RM, CM), "weight-streaming, all of A in LDS"),
        ("f16", 32, 14336, 4096, (RM, CM), "K-sliced weight-streaming"),
        ("f16", 48, 14336, 4096, (RM, CM), "K-sliced weight-streaming"),
        ("f16", 64, 14336, 4096, (RM, CM), "blocked, 64 x 64 tiles"),
        ("f16", 192, 14336, 4096, (RM, CM), "blocked, 64 x 64 tiles"),
        ("f16", 128, 14336, 4096, (RM, CM), "blocked, 128 x 64 tiles"),
        ("f16", 256, 14336, 4096, (RM, CM), "blocked, 128 x 128 tiles"),
        ("f16", 512, 512, 4096, (RM, CM), "blocked, 64 x 64 tiles (small problem)"),
        ("f16", 512, 512, 4096, (RM, RM), "blocked, 64 x 128 tiles (B row-major)"),
        ("f16", 512, 512, 4096, (CM, RM), "blocked, 128 x 128 tiles (A col-major, B row-major)"),
        ("f16", 2048, 2048, 2048, (RM, CM), "blocked, 128 x 128 tiles"),
        ("f16", 3072, 3072, 3072, (RM, CM), "blocked, 256 x 256 tiles, 144 of them"),
        ("f16", 4096, 4096, 4096, (RM, CM), "blocked, 256 x 256 tiles"),
        ("i8", 48, 14336, 4096, (RM, CM), "K-sliced weight-streaming"),
        ("i8", 64, 14336, 4096, (RM, CM), "blocked, 64 x 64 tiles"),
        ("i8", 112, 14336, 4096, (RM, CM), "K-sliced weight-streaming"),
        ("i8", 256, 14336, 4096, (RM, CM), "blocked, 128 x 128 tiles"),
        ("i8", 8192, 8192, 8192, (RM, CM), "blocked, 256 x 256 tiles"),
        ("fp8", 256, 14336, 4096, (RM, CM), "blocked, 128 x 128 tiles"),
        ("fp8", 8192, 8192, 8192, (RM, CM), "blocked, 256 x 256 tiles"),
    ]
    out = []
    for tag, m, n, k, (la, lb), what in shapes:
        esize = 2 if tag == "f16" else 1
        copies = max(2, min(6, -(-(300 << 20) // (n * k * esize))))  # weights rotate over >= 300 MiB, at most 6 buffers
        if tag == "f16":
            A = (torch.rand(m * k, device=dev, generator=gen) * 2 - 1).to(torch.float16)
            Bs = [(torch.rand(k * n, device=dev, generator=gen) * 2 - 1).to(torch.float16) for _ in range(copies)]
            code, ocode, D = rw.F16, rw.F32, torch.empty(m * n, device=dev)
        elif tag == "i8":
            A = torch.randint(-128, 128, (m * k,), device=dev, dtype=torch.int8, generator=gen)
            Bs = [torch.randint(-128, 128, (k * n,), device=dev, dtype=torch.int8, generator=gen) for _ in range(copies)]
            code, ocode, D = rw.I8, rw.I32, torch.empty(m * n, device=dev, dtype=torch.int32)
        else:
            A = (torch.randn(m * k, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
            Bs = [(torch.randn(k * n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn) for _ in range(copies)]
            code, ocode, D = rw.E4M3, rw.F32, torch.empty(m * n, device=dev)
        state = {"i": 0}

        def fn():
            rw.gemm(code, ocode, la, lb, RM, m, n, k, A, Bs[state["i"] % copies], None, D, 1.0, 0.0)
            state["i"] += 1

        fn(), fn()
        ms = min(event_ms(fn, 20, torch) for _ in range(3))
        out.append({"dtype": tag, "m": m, "n": n, "k": k, "a": "row" if la == RM else "col",
                    "b": "col" if lb == CM else "row", "us": round(ms * 1e3, 1),
                    "tflops": round(2.0 * m * n * k / ms / 1e9, 1), "kernel": what})
        del A, Bs, D
    return out


def run_extras(rw, torch, dev, gen, only=None):
    """The small GEMM (config 1), quantised GEMMs (config 3), GEMV (config 4), DLRM (config 5): kernel
    time by events.  `only`: one case by its key (a few launches of that case and nothing else)."""
    RM, CM = rw.ROW_MAJOR, rw.COL_MAJOR
    out = {}
    iters = 20 if only is None else 5

    def wanted(key):
        return only is None or only == key

    # config 1: 256^3 f16 -> f32, A row / B col, alpha = beta = 2: launch latency, reported only
    m1 = 256
    if any(wanted(f"gemm_f16_256cubed_{t}") for t in ("wave_tile", "blocked")):
        A1 = (torch.rand(m1 * m1, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        B1 = (torch.rand(m1 * m1, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        C1 = torch.rand(m1 * m1, device=dev, generator=gen) * 2 - 1
        D1 = torch.empty(m1 * m1, device=dev)
        for tag, algo in (("wave_tile", rw.GEMM_WAVE_TILE), ("blocked", rw.GEMM_BLOCKED)):
            if not wanted(f"gemm_f16_256cubed_{tag}"):
                continue

            def fn1():
                rw.gemm(rw.F16, rw.F32, RM, CM, RM, m1, m1, m1, A1, B1, C1, D1, 2.0, 2.0, algo=algo)

            fn1()
            ms = event_ms(fn1, 100, torch)
            msg = graph_ms(fn1, 50, torch) if only is None else None
            out[f"gemm_f16_256cubed_{tag}"] = {"us": round(ms * 1e3, 2), "tflops": round(2.0 * m1 ** 3 / ms / 1e9, 2),
                                               "us_graph_replay": None if msg is None else round(msg * 1e3, 2),
                                               "note": "back-to-back launches, launch-latency bound"}

    # A GEMM written against the public fragment API only (the reference's perf_hgemm data flow: cooperative
    # global reads, LDS slabs, mma_sync), 8192^3 f16 -> f32.  A col-major / B row-major makes every global
    # and LDS access a dim-major fragment access; A row / B col are K-contiguous in global memory.
    for tag, la_, lb_ in (("cr", CM, RM), ("rc", RM, CM)):
        key = f"public_api_gemm_f16_{tag}_8192"
        if not wanted(key):
            continue
        sz = 8192
        Ap = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Bp = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Cp = torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1
        Dp = torch.empty(sz * sz, device=dev)

        def fnp():
            rw.selftest_coop_gemm(la_, lb_, sz, sz, sz, Ap, Bp, Cp, Dp, 1.0, 1.0)

        fnp()
        ms = event_ms(fnp, 3, torch)
        out[key] = {"ms": round(ms, 3), "tflops": round(2.0 * sz ** 3 / ms / 1e9, 1),
                    "note": "fragment API only (load/store_matrix_coop_sync, applyDataLayout, applyTranspose, mma_sync); "
                            "32x32x16 blocks, 128 x 128 macro tile, single LDS buffer"}
        del Ap, Bp, Cp, Dp

    # The same through the public fragment API only, laid out for this device instead of after perf_hgemm:
    # 256 x 256 macro tile, eight waves, 16 x 16 x 32 blocks, two padded LDS buffers, the next K stage prefetched.
    for tag, la_, lb_ in (("cr", CM, RM), ("rc", RM, CM)):
        key = f"public_api_tiled_gemm_f16_{tag}_8192"
        if not wanted(key):
            continue
        sz = 8192
        Ap = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Bp = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Cp = torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1
        Dp = torch.empty(sz * sz, device=dev)

        def fnt():
            rw.selftest_tiled_gemm(la_, lb_, sz, sz, sz, Ap, Bp, Cp, Dp, 1.0, 1.0)

        fnt()
        ms = event_ms(fnt, 5, torch)
        out[key] = {"ms": round(ms, 3), "tflops": round(2.0 * sz ** 3 / ms / 1e9, 1),
                    "note": "fragment API only (load/store_matrix_coop_sync, applyDataLayout, applyTranspose, mma_sync); "
                            "16x16x32 blocks, 256 x 256 macro tile, two LDS buffers of 64 + 8 halves per row"}
        del Ap, Bp, Cp, Dp

    # the headline f16 A-row / B-col GEMM with the fused epilogue (bias per column, GELU) against the same
    # GEMM without it: what the epilogue costs when it rides on the accumulators
    if wanted("gemm_f16_rc_8192_bias_gelu"):
        sz = 8192
        Af = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Bf_ = (torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        Cf = torch.rand(sz * sz, device=dev, generator=gen) * 2 - 1
        Df = torch.empty(sz * sz, device=dev)
        bias = torch.rand(sz, device=dev, generator=gen) * 2 - 1

        def fn_fused():
            rw.gemm_bias_act(rw.F16, rw.F32, RM, CM, RM, sz, sz, sz, Af, Bf_, Cf, Df, 1.0, 1.0, bias, rw.ACT_GELU)

        def fn_plain():
            rw.gemm(rw.F16, rw.F32, RM, CM, RM, sz, sz, sz, Af, Bf_, Cf, Df, 1.0, 1.0)

        # (the two are timed in alternation, five rounds of ten launches each, and the medians reported: timed one
        # after the other, whichever came first read several per cent slower, more than the epilogue costs)
        t_fused, t_plain = [], []
        fn_fused(), fn_plain()
        for _ in range(5):
            t_fused.append(event_ms(fn_fused, 10, torch))
            t_plain.append(event_ms(fn_plain, 10, torch))
        ms, ms_plain = sorted(t_fused)[2], sorted(t_plain)[2]
        out["gemm_f16_rc_8192_bias_gelu"] = {"ms": round(ms, 4), "tflops": round(2.0 * sz ** 3 / ms / 1e9, 1),
                                             "ms_without_epilogue": round(ms_plain, 4),
                                             "epilogue_us": round((ms - ms_plain) * 1e3, 1),
                                             "note": "D = gelu(A*B + C + bias[column]), f32 C/D; medians of five alternating "
                                                     "rounds of ten launches"}
        del Af, Bf_, Cf, Df, bias

    # config 3: N = 14336, K = 4096, M in {16, 128, 4096}; int8 and e4m3, A row / B col.  The weight
    # matrix (56 MiB) would stay in the 256 MiB Infinity Cache between launches, so the timed loop
    # rotates over 5 weight buffers (280 MiB); the cache-resident time is reported beside it.
    n, k = 14336, 4096
    wcopies = 5
    q_keys = [(tag, m) for m in (16, 128, 4096) for tag in ("i8", "fp8") if wanted(f"gemm_{tag}_m{m}")]
    if q_keys:
        Bq = Bf = None
        if any(t == "i8" for t, _ in q_keys):
            Bq = [torch.randint(-128, 128, (k * n,), device=dev, dtype=torch.int8, generator=gen) for _ in range(wcopies)]
        if any(t == "fp8" for t, _ in q_keys):
            Bf = [(torch.randn(k * n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn) for _ in range(wcopies)]
        for tag, m in q_keys:
            if tag == "i8":
                A = torch.randint(-128, 128, (m * k,), device=dev, dtype=torch.int8, generator=gen)
                Dx = torch.empty(m * n, device=dev, dtype=torch.int32)
                code, ocode, Bs = rw.I8, rw.I32, Bq
            else:
                A = (torch.randn(m * k, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
                Dx = torch.empty(m * n, device=dev, dtype=torch.float32)
                code, ocode, Bs = rw.E4M3, rw.F32, Bf
            flops = 2.0 * m * n * k
            state = {"i": 0}

            def fn():
                rw.gemm(code, ocode, RM, CM, RM, m, n, k, A, Bs[state["i"] % wcopies], None, Dx, 1.0, 0.0)
                state["i"] += 1

            def fn_resident():
                rw.gemm(code, ocode, RM, CM, RM, m, n, k, A, Bs[0], None, Dx, 1.0, 0.0)

            fn()
            ms = event_ms(fn, iters, torch)
            fn_resident()
            ms_res = event_ms(fn_resident, iters, torch)
            byts = m * k + n * k + 4.0 * m * n
            out[f"gemm_{tag}_m{m}"] = {
                "ms": round(ms, 4), "tops": round(flops / ms / 1e9, 1),
                "frac_mfma": round(flops / ms / 1e9 / PEAK_TFLOPS[tag], 4),
                "gbs": round(byts / ms / 1e6, 1), "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4),
                "ms_weights_cache_resident": round(ms_res, 4),
            }
            if m <= 128 and only is None:
                # launches of 10-20 us, as the plain streams they are priced against: replayed as one HIP graph as well
                msg = graph_ms(fn, iters, torch)
                if msg is not None:
                    out[f"gemm_{tag}_m{m}"].update({"ms_graph_replay": round(msg, 4), "gbs_graph_replay": round(byts / msg / 1e6, 1),
                                                    "frac_hbm_graph_replay": round(byts / msg / 1e6 / PEAK_HBM_GBS, 4)})
        del Bq, Bf

    # the headline size with the 8-bit types (A row / B col, alpha = 1, beta = 0; operands as in config 3):
    # the size the fp8 / int8 targets are quoted on next to the f16 / bf16 one
    for tag in ("i8", "fp8"):
        key = f"gemm_{tag}_8192cubed"
        if not wanted(key):
            continue
        sz = 8192
        if tag == "i8":
            A8 = torch.randint(-128, 128, (sz * sz,), device=dev, dtype=torch.int8, generator=gen)
            B8 = torch.randint(-128, 128, (sz * sz,), device=dev, dtype=torch.int8, generator=gen)
            D8 = torch.empty(sz * sz, device=dev, dtype=torch.int32)
            code, ocode = rw.I8, rw.I32
        else:
            A8 = (torch.randn(sz * sz, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
            B8 = (torch.randn(sz * sz, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
            D8 = torch.empty(sz * sz, device=dev, dtype=torch.float32)
            code, ocode = rw.E4M3, rw.F32

        def fn8():
            rw.gemm(code, ocode, RM, CM, RM, sz, sz, sz, A8, B8, None, D8, 1.0, 0.0)

        fn8()
        fn8()
        ms = event_ms(fn8, iters, torch)
        out[key] = {"ms": round(ms, 4), "tops": round(2.0 * sz ** 3 / ms / 1e9, 1),
                    "frac_mfma": round(2.0 * sz ** 3 / ms / 1e9 / PEAK_TFLOPS[tag], 4)}
        del A8, B8, D8

    # config 3's fp8 shape with block scales (one E8M0 byte per 32 elements of K): the same blocked kernel
    # on the scaled matrix instruction, plus the small kernels that re-order the scales
    if wanted("gemm_mxfp8_m4096"):
        m = 4096
        Am = (torch.randn(m * k, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
        Bm = (torch.randn(k * n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
        SAm = torch.randint(124, 131, (m * (k // 32),), device=dev, dtype=torch.uint8, generator=gen)
        SBm = torch.randint(124, 131, (n * (k // 32),), device=dev, dtype=torch.uint8, generator=gen)
        Dm = torch.empty(m * n, device=dev, dtype=torch.float32)
        ws = torch.empty(rw.gemm_mx_workspace_size(m, n, k), device=dev, dtype=torch.uint8)

        def fnm():
            rw.gemm_mx(rw.E4M3, RM, CM, RM, m, n, k, Am, SAm, Bm, SBm, None, Dm, 1.0, 0.0, workspace=ws)

        fnm()
        ms = event_ms(fnm, iters, torch)
        flops = 2.0 * m * n * k
        out["gemm_mxfp8_m4096"] = {"ms": round(ms, 4), "tops": round(flops / ms / 1e9, 1),
                                   "frac_mfma": round(flops / ms / 1e9 / PEAK_TFLOPS["fp8"], 4),
                                   "note": "E4M3 operands, E8M0 scales per 32 elements of K, scale re-ordering included"}
        del Am, Bm, SAm, SBm, Dm, ws

    # ... its 128-token shape (mid-size scaled tiles): scales re-ordered on every call against scales packed once
    if wanted("gemm_mxfp8_m128"):
        m = 128
        Am = (torch.randn(m * k, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
        Bm = (torch.randn(k * n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
        SAm = torch.randint(124, 131, (m * (k // 32),), device=dev, dtype=torch.uint8, generator=gen)
        SBm = torch.randint(124, 131, (n * (k // 32),), device=dev, dtype=torch.uint8, generator=gen)
        Dm = torch.empty(m * n, device=dev, dtype=torch.float32)
        ws = torch.empty(rw.gemm_mx_workspace_size(m, n, k), device=dev, dtype=torch.uint8)

        def fn_each():
            rw.gemm_mx(rw.E4M3, RM, CM, RM, m, n, k, Am, SAm, Bm, SBm, None, Dm, 1.0, 0.0, workspace=ws)

        def fn_packed():
            rw.gemm_mx_packed(rw.E4M3, RM, CM, RM, m, n, k, Am, Bm, None, Dm, 1.0, 0.0, ws)

        fn_each()
        ms_each = event_ms(fn_each, iters, torch)
        rw.gemm_mx_pack_scales(RM, CM, RM, m, n, k, SAm, SBm, ws)
        fn_packed()
        ms_packed = event_ms(fn_packed, iters, torch)
        out["gemm_mxfp8_m128"] = {"ms": round(ms_each, 4), "ms_scales_packed_once": round(ms_packed, 4),
                                  "note": "E4M3 operands, E8M0 scales per 32 elements of K; weights cache resident"}
        del Am, Bm, SAm, SBm, Dm, ws

    # ... and its 16-token shape (weight streaming): weights and their scales rotated over 5 buffers
    if wanted("gemm_mxfp8_m16"):
        m = 16
        Am = (torch.randn(m * k, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn)
        Bms = [(torch.randn(k * n, device=dev, generator=gen) * 0.1).to(torch.float8_e4m3fn) for _ in range(wcopies)]
        SAm = torch.randint(124, 131, (m * (k // 32),), device=dev, dtype=torch.uint8, generator=gen)
        SBms = [torch.randint(124, 131, (n * (k // 32),), device=dev, dtype=torch.uint8, generator=gen) for _ in range(wcopies)]
        Dm = torch.empty(m * n, device=dev, dtype=torch.float32)
        state = {"i": 0}

        def fnm16():
            j = state["i"] % wcopies
            rw.gemm_mx(rw.E4M3, RM, CM, RM, m, n, k, Am, SAm, Bms[j], SBms[j], None, Dm, 1.0, 0.0)
            state["i"] += 1

        fnm16()
        ms = event_ms(fnm16, iters, torch)
        byts = m * k + n * k + (m + n) * (k // 32) + 4.0 * m * n
        out["gemm_mxfp8_m16"] = {"ms": round(ms, 4), "gbs": round(byts / ms / 1e6, 1),
                                 "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4),
                                 "note": "E4M3 operands, E8M0 scales per 32 elements of K (scale bytes counted)"}
        del Am, Bms, SAm, SBms, Dm

    # config 4: GEMV, buffers rotated over > 512 MB so the 256 MB Infinity Cache cannot serve A
    for (m, kk) in ((8192, 8192), (14336, 4096)):
        cols = [nc for nc in (1, 4, 8) if wanted(f"gemv_{m}x{kk}_n{nc}")]
        if not cols:
            continue
        copies = 5
        As = [(torch.rand(m * kk, device=dev, generator=gen) * 2 - 1).to(torch.float16) for _ in range(copies)]
        for ncols in cols:
            x = (torch.rand(kk * ncols, device=dev, generator=gen) * 2 - 1).to(torch.float16)
            y = torch.zeros(m * ncols, device=dev)
            state = {"i": 0}

            def fn():
                rw.gemv(m, kk, ncols, As[state["i"] % copies], x, y, 1.0, 0.0)
                state["i"] += 1

            fn()
            ms = event_ms(fn, iters, torch)
            byts = 2.0 * m * kk + 2.0 * kk * ncols + 4.0 * m * ncols
            out[f"gemv_{m}x{kk}_n{ncols}"] = {"ms": round(ms, 5), "gbs": round(byts / ms / 1e6, 1),
                                             "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
            if only is None:
                msg = graph_ms(fn, iters, torch)
                if msg is not None:
                    out[f"gemv_{m}x{kk}_n{ncols}"].update({"ms_graph_replay": round(msg, 5), "gbs_graph_replay": round(byts / msg / 1e6, 1),
                                                           "frac_hbm_graph_replay": round(byts / msg / 1e6 / PEAK_HBM_GBS, 4)})
        del As

    # config 5: DLRM, batch 2048 (cache resident, latency bound) and a batch that streams from HBM
    mm, kd = 27, 128
    width = kd + mm * (mm - 1) // 2
    for batch, copies in ((2048, 1), (262144, 3)):
        if not (wanted(f"dlrm_fwd_b{batch}") or wanted(f"dlrm_bwd_b{batch}")):
            continue
        Fs = [(torch.rand(batch * mm * kd, device=dev, generator=gen) * 2 - 1).to(torch.float16) for _ in range(copies)]
        up = (torch.rand(batch * width, device=dev, generator=gen) * 2 - 1).to(torch.float16)
        o = torch.empty(batch * width, device=dev, dtype=torch.float16)
        gr = torch.empty(batch * mm * kd, device=dev, dtype=torch.float16)
        mg = torch.empty(batch * kd, device=dev, dtype=torch.float16)
        state = {"i": 0}

        def fwd():
            rw.dlrm_fwd(Fs[state["i"] % copies], o, mm, kd, batch)
            state["i"] += 1

        def bwd():
            rw.dlrm_bwd(Fs[state["i"] % copies], up, gr, mg, mm, kd, batch)
            state["i"] += 1

        bf = batch * (mm * kd * 2.0 + width * 2.0)
        bb = batch * (mm * kd * 2.0 + width * 2.0 + mm * kd * 2.0 + kd * 2.0)
        for tag, fnx, byts in (("fwd", fwd, bf), ("bwd", bwd, bb)):
            if not wanted(f"dlrm_{tag}_b{batch}"):
                continue
            fnx()
            ms = event_ms(fnx, iters, torch)
            out[f"dlrm_{tag}_b{batch}"] = {"ms": round(ms, 5), "gbs": round(byts / ms / 1e6, 1),
                                           "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
            if batch == 2048 and only is None:
                # the kernels take 4-10 us, less than a Python loop needs per launch: graph replay as well
                msg = graph_ms(fnx, iters, torch)
                if msg is not None:
                    out[f"dlrm_{tag}_b{batch}"].update({"ms_graph_replay": round(msg, 5),
                                                        "gbs_graph_replay": round(byts / msg / 1e6, 1),
                                                        "frac_hbm_graph_replay": round(byts / msg / 1e6 / PEAK_HBM_GBS, 4)})
        del Fs

    # The reference's largest DLRM test size, (m, k, batch) = (1024, 1024, 64) (test/dlrm/test/dlrm_test_params.hpp:51-68):
    # a sample is a 1024^3 matrix product of its own, so these are compute bound (tiles of 128 x 128 per workgroup, no
    # m x m scratch in global memory).  flops: forward m (m - 1) k (the strict lower triangle), backward 2 m^2 k.
    ml, kl, bl = 1024, 1024, 64
    wl = kl + ml * (ml - 1) // 2
    for tdt, code, tag in ((torch.float16, rw.F16, "f16"), (torch.float32, rw.F32, "f32")):
        if not (wanted(f"dlrm_fwd_{tag}_m1024_k1024_b64") or wanted(f"dlrm_bwd_{tag}_m1024_k1024_b64")):
            continue
        Fl = (torch.rand(bl * ml * kl, device=dev, generator=gen) * 2 - 1).to(tdt)
        upl = (torch.rand(bl * wl, device=dev, generator=gen) * 2 - 1).to(tdt)
        ol = torch.empty(bl * wl, device=dev, dtype=tdt)
        grl = torch.empty(bl * ml * kl, device=dev, dtype=tdt)
        mgl = torch.empty(bl * kl, device=dev, dtype=tdt)
        peak = PEAK_TFLOPS["f16"] if tag == "f16" else 157.3  # dense MFMA, MI355X: f16, float32
        for name, fnx, flops in ((f"dlrm_fwd_{tag}_m1024_k1024_b64", lambda: rw.dlrm_fwd(Fl, ol, ml, kl, bl, code), 1.0 * bl * ml * (ml - 1) * kl),
                                 (f"dlrm_bwd_{tag}_m1024_k1024_b64", lambda: rw.dlrm_bwd(Fl, upl, grl, mgl, ml, kl, bl, code), 2.0 * bl * ml * ml * kl)):
            if not wanted(name):
                continue
            fnx()
            ms = event_ms(fnx, iters, torch)
            out[name] = {"ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 1), "frac_mfma": round(flops / ms / 1e9 / peak, 4)}
        del Fl, upl, ol, grl, mgl

    # What plain streaming kernels reach on this device for the byte counts of the bandwidth-bound cases
    # (one read-only / copy kernel, windows rotated through 2 GiB so that every launch reads from HBM):
    # at tens of megabytes a launch is over before the memory system reaches the rate of a long stream.
    if only is None or only == "stream_ceiling":
        MiB = 1 << 20
        src = torch.ones(2048 * MiB // 4, device=dev, dtype=torch.int32)
        dst = torch.empty(2048 * MiB // 4, device=dev, dtype=torch.int32)
        ceil = {}
        for tag, mode, nbytes in (("read_56MiB", rw.STREAM_READ, 56 * MiB), ("read_128MiB", rw.STREAM_READ, 128 * MiB),
                                  ("read_1792MiB", rw.STREAM_READ, 1792 * MiB), ("copy_1792MiB", rw.STREAM_COPY, 1792 * MiB),
                                  # the DLRM backward pass's mix: 1.1 bytes read per byte written
                                  ("copy_896MiB_plus_tenth_reads", rw.STREAM_COPY_READ_MORE, 896 * MiB),
                                  # what a GEMM's result write can reach: the 256 MiB of an 8192^3 f32 result, to one
                                  # buffer over and over as the benchmark's GEMMs do (it fits the Infinity Cache) and
                                  # through 2 GiB (what the HBM itself takes)
                                  ("write_256MiB_same_buffer", rw.STREAM_WRITE, 256 * MiB),
                                  ("write_1792MiB", rw.STREAM_WRITE, 1792 * MiB)):
            windows = 1 if (tag.endswith("same_buffer") or mode == rw.STREAM_COPY_READ_MORE) else max(1, (2048 * MiB) // nbytes)
            state = {"i": 0}
            # (raw addresses and the stream handle prepared up front: a launch of 10 us must not wait for Python)
            srcs = [ctypes.c_void_p(src.data_ptr() + w * nbytes) for w in range(windows)]
            dsts = [ctypes.c_void_p(dst.data_ptr() + w * nbytes) for w in range(windows)]
            strm = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

            def fns():
                w = state["i"] % windows
                rw.bench_stream(mode, srcs[w], dsts[w], nbytes, strm)
                state["i"] += 1

            def fns_current_stream():
                w = state["i"] % windows
                rw.bench_stream(mode, srcs[w], dsts[w], nbytes)
                state["i"] += 1

            fns()
            ms = event_ms(fns, iters, torch)
            # launches of 10-20 us: replayed as one HIP graph as well, and the shorter of the two counts
            msg = graph_ms(fns_current_stream, iters, torch) if (nbytes <= 128 * MiB and only is None) else None
            best = ms if msg is None else min(ms, msg)
            moved = nbytes * {rw.STREAM_COPY: 2.0, rw.STREAM_COPY_READ_MORE: 2.1}.get(mode, 1.0)
            ceil[tag] = {"ms": round(ms, 5), "ms_graph_replay": None if msg is None else round(msg, 5),
                         "gbs": round(moved / best / 1e6, 1), "frac_hbm": round(moved / best / 1e6 / PEAK_HBM_GBS, 4)}
        # what the compute units can draw from their L2s: 16 MiB (one workgroup per compute unit re-reading its
        # own 64 KiB, 2 MiB per XCD) read 256 times in one launch; the operand streams of the tiled kernels
        # (L2 -> LDS copies of the GEMM, of the tiled DLRM kernels) are a fraction of this rate
        nres = 16 * MiB
        res_fn = lambda: rw.bench_stream(rw.STREAM_READ_RESIDENT, src, dst, nres)
        res_fn()
        ms = event_ms(res_fn, iters, torch)
        moved = float(nres) * rw.STREAM_RESIDENT_PASSES
        ceil["l2_resident_read_16MiB"] = {"ms": round(ms, 5), "gbs": round(moved / ms / 1e6, 1),
                                          "gbs_per_compute_unit": round(moved / ms / 1e6 / compute_units_of(rw), 1)}
        del src, dst
        out["stream_ceiling"] = ceil
        # the bandwidth-bound cases against the plain stream of the nearest size and kind
        for key, ref in (("gemm_i8_m16", "read_56MiB"), ("gemm_fp8_m16", "read_56MiB"), ("gemm_i8_m128", "read_56MiB"),
                         ("gemm_fp8_m128", "read_56MiB"), ("gemv_8192x8192_n1", "read_128MiB"),
                         ("gemv_8192x8192_n4", "read_128MiB"), ("gemv_8192x8192_n8", "read_128MiB"),
                         ("gemv_14336x4096_n1", "read_128MiB"), ("gemv_14336x4096_n4", "read_128MiB"),
                         ("gemv_14336x4096_n8", "read_128MiB"), ("dlrm_fwd_b262144", "read_1792MiB"),
                         ("dlrm_bwd_b262144", "copy_896MiB_plus_tenth_reads")):
            if key in out:
                # (the shorter of the two timings on both sides)
                best_gbs = max(out[key]["gbs"], out[key].get("gbs_graph_replay", 0.0))
                out[key]["frac_of_stream_ceiling"] = round(best_gbs / ceil[ref]["gbs"], 4)
    return out


if __name__ == "__main__":
    main()
