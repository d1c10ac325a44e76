#!/usr/bin/env python3
"""Benchmark of the legacy op-execution path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--families] [--no-cpu]

A step is one pass of the headline workload: execPairwiseTransformFloat Add, execPairwiseTransformFloat
Multiply and execBroadcastFloat Add of a row vector on fp32 [65536,1024] c-order operands that are already
resident in HBM (in two device copies used in turn, so that no pass finds its operands in the 256 MiB
last-level cache).  The line printed at the end is one JSON object:

  value      algorithmic GB/s of the whole step loop (host clock around K steps, device idle before and after)
  roofline   the dominant kernel (the 16-byte-vector elementwise kernel running pairwise Add): algorithmic
             bytes per launch / average launch duration from HIP events recorded on the launch stream inside
             the timed loop, against 8 TB/s
  cpu_baseline  the same step on the host cores (compiled reference loops when oracle/_ref is present, else
             this repository's CPU restatement), a bounded sample
  families   every case of the other configurations as {case: [ms per launch, fraction of 8 TB/s]}, each timed with
             HIP events over K back-to-back launches (--no-families leaves them out)

The printed line stays under 4 KB.  The full family rows (GB/s, elements/s, CPU time of the same case, measured HBM
traffic, vector-instruction figures, notes) go to stderr as a table and to the file named by --families-out.

Inputs are synthetic (seeded numpy generators); nothing is read from disk.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3  # dense fp32 on the matrix unit


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--families", action="store_true", help="(default) also time every op family of the other configurations")
    ap.add_argument("--no-families", action="store_true", help="headline step only")
    ap.add_argument("--families-cpu-seconds", type=float, default=25.0,
                    help="total budget of the CPU passes beside the family rows; cases left over when it is spent get no "
                         "CPU column")
    ap.add_argument("--families-out", default=os.path.join(ROOT, "gpurun_out", "bench_families.json"),
                    help="file that receives the full family rows (the printed line carries [ms, frac] per case only)")
    ap.add_argument("--only", default="", help="with --families: comma-separated workload builders to run "
                                               "(transform,pairwise,half,reductions,reduce3,stats,views,random,movement,whole)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU sample of the headline step")
    ap.add_argument("--counters", action="store_true",
                    help="for hardware-counter runs: launch the yardstick copy kernel (256 MiB) and each headline kernel "
                         "3 times and exit")
    ap.add_argument("--traffic", default=os.path.join(ROOT, "profiles", "all_families_hbm_traffic.txt"),
                    help="rocprofv3 counter summary holding the measured HBM bytes per launch of the dominant kernel")
    ap.add_argument("--instructions", default=os.path.join(ROOT, "profiles", "all_families_instruction_counters.txt"),
                    help="rocprofv3 counter summary holding the vector instructions per element of the benchmark cases")
    return ap.parse_args()


class EventTimer(object):
    """HIP events on the stream the library launches on."""

    def __init__(self, dev, count):
        self.dev = dev
        self.ev = [dev.ops.amd_timerCreate() for _ in range(count)]
        if not all(self.ev):
            raise RuntimeError("hipEventCreate failed")

    def record(self, i):
        if self.dev.ops.amd_timerRecord(self.ev[i], self.dev.stream) != 1:
            raise RuntimeError("hipEventRecord failed")

    def ms(self, i, j):
        return float(self.dev.ops.amd_timerElapsedMs(self.ev[i], self.ev[j]))

    def destroy(self):
        for e in self.ev:
            self.dev.ops.amd_timerDestroy(e)


def time_case(dev, case, steps, warmup):
    """Average device time of one launch of `case`, HIP events around `steps` back-to-back launches."""
    t = EventTimer(dev, 2)
    for k in range(warmup):
        case.gpu(k)
    dev.sync()
    t.record(0)
    for k in range(steps):
        case.gpu(warmup + k)
    t.record(1)
    dev.sync()
    ms = t.ms(0, 1) / steps
    t.destroy()
    return ms


def kernel_sources_digest():
    """Digest of the kernel and host sources the library is built from: a counter summary under profiles/ records the
    digest it was measured on, and its figures are only quoted while the sources still are what they were then."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "libnd4j_amd", "csrc")
    for name in sorted(os.listdir(src)):
        path = os.path.join(src, name)
        if os.path.isfile(path) and name.rsplit(".", 1)[-1] in ("hip", "cuh", "h", "cpp"):
            h.update(name.encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(path, key):
    """HBM bytes per launch (or per call) of the line that starts with `key` in a committed counter summary (FETCH_SIZE
    and WRITE_SIZE runs of `bench.py --counters`, scaled by a copy kernel of known size).  None when the summary is not
    there, has no such line, or was measured on other sources than the ones in this tree (its `sources:` line)."""
    if not path or not os.path.exists(path):
        return None
    with open(path) as f:
        lines = f.read().splitlines()
    for line in lines:
        if line.startswith("sources:") and line.split()[1] != kernel_sources_digest():
            return None
    for line in lines:
        if line.startswith(key):
            try:
                return int(line.split()[-1])
            except ValueError:
                return None
    return None


def family_builders(workloads):
    return [("transform", workloads.transform_tanh), ("pairwise", lambda d: workloads.pairwise_broadcast(d, copies=2)),
            ("half", lambda d: workloads.pairwise_broadcast(d, dtype="float16")),
            ("reductions", workloads.reductions), ("reduce3", workloads.reduce3_pairs),
            ("stats", workloads.stats_softmax), ("views", workloads.general_views), ("random", workloads.random_fills),
            ("movement", workloads.data_movement), ("whole", workloads.whole_array_transforms)]


def valu_per_element(path, case, field="VALU/element"):
    """VALU instructions per element of `case` from the committed instruction-counter summary (its line
    "<case> ... VALU/element <v>"; `field` names another figure of that line), or None: as measured_traffic, only while
    the sources are what they were."""
    if not path or not os.path.exists(path):
        return None
    with open(path) as f:
        lines = f.read().splitlines()
    for line in lines:
        if line.startswith("sources:") and line.split()[1] != kernel_sources_digest():
            return None
    for line in lines:
        if line.startswith(case + " ") and field in line:
            try:
                return float(line.split(field)[1].split()[0])
            except (ValueError, IndexError):
                return None
    return None


def load_cpu():
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import cpu_ref
    lib = cpu_ref.load_reference()
    if lib is None:
        lib = cpu_ref.load_oracle()
    return lib, ("reference" if lib.kind == "reference" else "port")


def cpu_time(fn, lib, budget_s, min_runs=3, max_runs=5000):
    fn(lib)  # warm-up (page faults of the output buffer, OpenMP pool start)
    times = []
    start = time.perf_counter()
    while len(times) < max_runs and (len(times) < min_runs or time.perf_counter() - start < budget_s):
        t0 = time.perf_counter()
        fn(lib)
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)


MAX_LINE_BYTES = 6000  # whoever runs this keeps only the last 8000 bytes of stdout: the result line must fit with room to spare


def result_line(out, family_rows):
    """The one line printed on stdout: the headline object plus, per family case, [ms per launch, fraction of the HBM
    peak].  Aims at under 4 KB - the per-kernel breakdown of the headline step goes first when the cases are many - and
    raises when it would not fit in MAX_LINE_BYTES."""
    line = dict(out)
    if family_rows is not None:
        line["families"] = {r["case"]: [r["ms"], round(r["frac"], 3)] for r in family_rows}
    text = json.dumps(line, separators=(",", ":"))
    if len(text) >= 4096 and "kernels" in line:
        del line["kernels"]  # (it is in the file of full rows and on stderr)
        text = json.dumps(line, separators=(",", ":"))
    if len(text) >= MAX_LINE_BYTES:
        raise RuntimeError("the result line has grown to %d bytes (limit %d)" % (len(text), MAX_LINE_BYTES))
    return text


def write_family_rows(path, out, family_rows):
    """The full rows, beside the headline they belong to; a directory that cannot be written is reported, not fatal."""
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump({"headline": out, "families": family_rows}, f, indent=1)
    except OSError as e:
        print("bench.py: could not write %s: %s" % (path, e), file=sys.stderr)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (one process, one device, no collectives); "
              "--gpus %d is not supported, run with --gpus 1" % args.gpus, file=sys.stderr)
        return 2
    from libnd4j_amd import harness, workloads

    dev = harness.Device()  # raises when the HIP library or the GPU is missing: there is no CPU fallback
    K, W = args.steps, args.warmup

    # ---- headline: configs[1] ---------------------------------------------------------------------
    w = workloads.pairwise_broadcast(dev)
    add, mul, bca = w.case("pairwise_add"), w.case("pairwise_multiply"), w.case("broadcast_add_row")
    step_cases = (add, mul, bca)
    step_bytes = sum(c.bytes for c in step_cases)
    step_elems = sum(c.elements for c in step_cases)
    if args.counters:
        # For a `rocprofv3 --pmc` run: the yardstick copy kernel (256 MiB read, 256 MiB written) 3 times, then every case
        # 3 times, each case behind a small copy whose size (4096 bytes times the case's number) marks it in the trace.
        src, dst = dev.empty(1 << 28), dev.empty(1 << 28)
        for _ in range(3):
            dev.ops.amd_copyKernel(dev.extra(), dst.ptr, src.ptr, 1 << 28)
        listed = []

        def run(cases):
            for c in cases:
                listed.append({"case": c.name, "bytes": c.bytes, "elements": c.elements, "marker_bytes": 4096 * (len(listed) + 1)})
                dev.ops.amd_copyKernel(dev.extra(), dst.ptr, src.ptr, listed[-1]["marker_bytes"])
                for k in range(3):
                    c.gpu(k)
                dev.sync()

        run(step_cases)
        w.free()
        only = [o for o in args.only.split(",") if o]
        stepped = set(c.name for c in step_cases)
        for key, build in family_builders(workloads):
            if only and key not in only:
                continue
            wl = build(dev)
            run([c for c in wl.cases if c.name not in stepped])  # (the headline step's cases have run above)
            wl.free()
        print(json.dumps({"counters_run": {"copy_bytes_read": 1 << 28, "copy_bytes_written": 1 << 28, "sources": kernel_sources_digest(),
                                           "cases": listed}}))
        return 0
    for k in range(W):
        for c in step_cases:
            c.gpu(k)
    dev.sync()
    ev = EventTimer(dev, 4 * K)
    t0 = time.perf_counter()
    for s in range(K):
        ev.record(4 * s)
        add.gpu(W + s)
        ev.record(4 * s + 1)
        mul.gpu(W + s)
        ev.record(4 * s + 2)
        bca.gpu(W + s)
        ev.record(4 * s + 3)
    dev.sync()
    wall = time.perf_counter() - t0
    per_kernel_ms = [sum(ev.ms(4 * s + k, 4 * s + k + 1) for s in range(K)) / K for k in range(3)]
    ev.destroy()
    ms_per_step = wall * 1e3 / K
    value = step_bytes / (wall / K) / 1e9

    traffic = measured_traffic(args.traffic, "pairwise_add ")
    achieved = add.bytes / (per_kernel_ms[0] * 1e-3) / 1e9
    out = {
        "metric": "achieved HBM GB/s (algorithmic bytes) of the legacy op path: pairwise add + pairwise multiply + broadcast add row",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: " + w.name + ", seed 7", "elements_per_step": step_elems,
                   "bytes_per_step": step_bytes},
        "elements_per_sec": round(step_elems / (wall / K), 1),
        "pct_of_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "kernels": {c.name: {"ms": round(ms, 4), "GB/s": round(c.bytes / ms / 1e6, 1),
                             "frac": round(c.bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
                    for c, ms in zip(step_cases, per_kernel_ms)},
        "roofline": {"bound": "hbm", "kernel": "ewVecKernel (pairwise Add, fp32, 16-byte vectors)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "bytes_per_launch": add.bytes, "avg_launch_ms": round(per_kernel_ms[0], 4)},
    }

    cpu_lib = None
    if not args.no_cpu:
        cpu_lib, kind = load_cpu()
        cores = cpu_lib.lib.nd4j_cpu_get_threads()

        def cpu_step(lib):
            for c in step_cases:
                c.cpu(lib)

        med, runs = cpu_time(cpu_step, cpu_lib, args.cpu_seconds)
        out["cpu_baseline"] = {"value": round(step_bytes / med / 1e9, 2), "unit": "GB/s", "cores": int(cores), "kind": kind,
                               "sample": "%d full passes of the same step (all 3 calls on the full [65536,1024] operands), "
                                         "median; %.1f ms per step, %.3g elements/s" % (runs, med * 1e3, step_elems / med),
                               "elements_per_sec": round(step_elems / med, 1)}
    else:
        out["cpu_baseline"] = None
    w.free()

    # ---- every other family ---------------------------------------------------------------------------
    if not args.no_families:
        fam = []
        cpu_left = args.families_cpu_seconds
        only = [o for o in args.only.split(",") if o]
        for key, build in family_builders(workloads):
            if only and key not in only:
                continue
            wl = build(dev)
            for c in wl.cases:
                fetched = dev.ops.amd_hostFetchCount()
                ms = time_case(dev, c, max(3, min(K, 20)), 2)
                fetched = dev.ops.amd_hostFetchCount() - fetched
                row = {"case": c.name, "family": c.family, "ms": round(ms, 4), "GB/s": round(c.bytes / ms / 1e6, 1),
                       "frac": round(c.bytes / ms / 1e6 / HBM_PEAK_GBS, 4), "elements_per_sec": float("%.4g" % (c.elements / ms * 1e3))}
                if fetched:  # shapeInfo / dimension read-backs (each one a stream synchronisation)
                    row["host_fetches"] = int(fetched)
                row["bound"] = getattr(c, "bound", "hbm")
                if row["bound"] == "mfma":  # against the chip's dense fp32 matrix peak
                    tflops = getattr(c, "flops", 0) / ms / 1e9
                    row["mfma"] = {"achieved": round(tflops, 1), "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                                   "frac": round(tflops / MFMA_FP32_PEAK_TFLOPS, 4)}
                v = valu_per_element(args.instructions, c.name)
                if v is not None:
                    # A SIMD is 16 lanes wide: a wave64 vector instruction holds it for 4 cycles (plain fp32 and integer
                    # instructions measure 2.9 to 4.7 on this chip; the data sheet's 157.3 TFLOP/s take the packed forms,
                    # two results per lane and cycle, which this build does not use).  At 4 cycles apiece the call's vector
                    # instructions need this long on the chip's 1024 SIMDs
                    issue_ms = v * c.elements / 64.0 * 4.0 / (1024 * 2.4e9) * 1e3
                    row["valu"] = {"instructions_per_element": v, "issue_ms": round(issue_ms, 4), "frac": round(issue_ms / ms, 4)}
                t = measured_traffic(args.traffic, c.name + " ")
                if t is not None:  # HBM bytes the call moved, by the chip's counters (profiles/): well above `bytes` = re-reads
                    row["traffic"] = t
                    row["traffic_over_algorithmic"] = round(t / float(c.bytes), 3)
                # one warm-up and up to three timed passes of the compiled reference, while the budget lasts; a case whose
                # single pass is known to take seconds (note "cpu once") is run once, cold
                if cpu_lib is not None and c.cpu is not None and not (c.name.endswith("float16")) and cpu_left > 0:
                    t_cpu = time.perf_counter()
                    if getattr(c, "cpu_once", False):
                        t0 = time.perf_counter()
                        c.cpu(cpu_lib)
                        med = time.perf_counter() - t0
                    else:
                        med, runs = cpu_time(c.cpu, cpu_lib, 0.3, min_runs=1, max_runs=3)
                    cpu_left -= time.perf_counter() - t_cpu
                    row["cpu_ms"] = round(med * 1e3, 3)
                    row["cpu_GB/s"] = round(c.bytes / med / 1e9, 2)
                    time.sleep(0.05)  # the OpenMP workers spin for a while after a parallel region: let them go to sleep
                                      # before the next case's host thread needs a core to itself
                if c.note:
                    row["note"] = c.note
                fam.append(row)
                print("%-22s %-12s %9.4f ms %8.1f GB/s %5.1f%%%s%s" % (
                    c.name, c.family, ms, row["GB/s"], 100 * row["frac"],
                    "   cpu %9.2f ms" % row["cpu_ms"] if "cpu_ms" in row else "",
                    "   (%d read-backs from the device)" % fetched if fetched else "") + ("   [%s]" % c.note if c.note else ""),
                    file=sys.stderr, flush=True)
            wl.free()
        write_family_rows(args.families_out, out, fam)
        print(result_line(out, fam), flush=True)
        return 0
    print(result_line(out, None), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
