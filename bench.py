#!/usr/bin/env python3
"""Benchmark driver: GFLOP/s of one tensor contraction on one MI355X, with its roofline fraction.

A "step" is one launch of the contraction through the per-expression C-ABI object, inputs resident
in HBM.  The headline workload is BASELINE config 2 (fp64, 4-D output, one contracted index, all
extents 72); the other BASELINE configs are timed the same way and listed under "all_configs".

  value          flops / wall-clock time of K back-to-back launches (flops = 2 * product of extents,
                 cogent/src/codes/kernels/tc_interface.py:289-305; cogent/data-tccg.py:49)
  roofline       algorithmic bytes sizeof(T) * (|A| + |B| + 2|C|) per launch / mean per-launch
                 duration from HIP events recorded between launches on the launch stream
  cpu_baseline   the reference's host nested-loop contraction (CPU oracle) timed on this box's cores
                 on the same seeded inputs, and used to verify the GPU result element by element

Output buffers are rotated through a pool larger than the 256 MB Infinity Cache so that no launch
finds its output tensor cached by the previous one.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cgo2019-ae_amd"))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f64": 78.6, "f32": 157.3}
TOL = {"f64": 1e-12, "f32": 1e-5}
HEADLINE = "cfg2_f64"


def read_traffic(name):
    """HBM bytes per launch from the rocprofv3 counter summary under profiles/ (FETCH_SIZE and WRITE_SIZE of the
    contraction kernel, each scaled by what the same counter reads for a plain copy of known size), or None."""
    path = os.path.join(ROOT, "profiles", "counters_%s.txt" % name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("hbm_bytes_per_launch:"):
            return float(line.split(":")[1])
    return None


def read_mfma_busy(name):
    """Fraction of the kernel's active cycles with the matrix cores busy, from the counter summary under profiles/, or None."""
    path = os.path.join(ROOT, "profiles", "counters_%s.txt" % name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("mfma_busy_fraction:"):
            return float(line.split(":")[1])
    return None


class Workload:
    def __init__(self, pkg, tools, entry, sizes):
        import numpy as np
        import torch
        self.name = entry["name"]
        self.plan_file = entry["file"]
        self.sizes = list(sizes)
        self.ex = pkg.Expression(self.name)
        self.plan = tools.plan(pkg.expression_text(self.name), entry["dtype"])
        self.dtype = self.ex.dtype
        np_dtype = np.float64 if self.dtype == "f64" else np.float32
        names = self.plan.info["out_idx"] + self.plan.info["sum_idx"]
        ext = dict(zip(names, self.sizes))
        count = lambda idx: int(np.prod([ext[i] for i in idx], dtype=np.int64))
        self.nC, self.nA, self.nB = count(self.plan.info["out_idx"]), count(self.plan.info["a_idx"]), count(self.plan.info["b_idx"])
        self.flops = self.plan.flops(self.sizes)
        self.bytes = self.plan.bytes(self.sizes)
        esize = 8 if self.dtype == "f64" else 4
        # seeds 1, 2, 3 for A, B, C; C starts at zero unless the config says it is seeded
        self.hA = tools.fill_uniform(np.empty(self.nA, np_dtype), 1)
        self.hB = tools.fill_uniform(np.empty(self.nB, np_dtype), 2)
        if entry.get("c_init") == "seeded":
            self.hC = tools.fill_uniform(np.empty(self.nC, np_dtype), 3)
        else:
            self.hC = np.zeros(self.nC, np_dtype)
        self.dA = torch.from_numpy(self.hA).cuda()
        self.dB = torch.from_numpy(self.hB).cuda()
        n_rot = max(2, min(8, int(1.2e9 // (self.nC * esize)) + 1))
        c0 = torch.from_numpy(self.hC).cuda()
        self.dC = [c0] + [c0.clone() for _ in range(n_rot - 1)]

    def c_ptrs(self):
        return [c.data_ptr() for c in self.dC]

    def launch(self, i):
        rc = self.ex.run(self.sizes, self.dC[i % len(self.dC)].data_ptr(), self.dA.data_ptr(), self.dB.data_ptr(), None, 0)
        if rc:
            raise RuntimeError("launch failed (%d): %s" % (rc, self.ex.last_error()))

    def reset_c(self):
        import torch
        src = torch.from_numpy(self.hC).cuda()
        for c in self.dC:
            c.copy_(src)
        torch.cuda.synchronize()


def roofline(w, mean_ms):
    sec = mean_ms * 1e-3
    gbs = w.bytes / sec / 1e9
    tfl = w.flops / sec / 1e12
    hbm = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)}
    mfma = {"bound": "mfma", "achieved": round(tfl, 3), "peak": MFMA_PEAK_TFLOPS[w.dtype], "unit": "TFLOP/s",
            "frac": round(tfl / MFMA_PEAK_TFLOPS[w.dtype], 4)}
    t_hbm = w.bytes / (HBM_PEAK_GBS * 1e9)
    t_mfma = w.flops / (MFMA_PEAK_TFLOPS[w.dtype] * 1e12)
    return (hbm, mfma) if t_hbm >= t_mfma else (mfma, hbm)


def time_workload(driver, w, warmup, iters, min_warm_ms=30.0):
    # After the allocations and copies of a new workload the first launches run up to 15 % slow (every output buffer
    # is touched for the first time, clocks ramp): warm every buffer, and for at least min_warm_ms of kernel time.
    warmup = max(warmup, len(w.dC))
    probe = driver.time(w.ex, w.sizes, w.c_ptrs(), w.dA.data_ptr(), w.dB.data_ptr(), warmup, 3)
    warmup = len(w.dC) + int(min(2000, max(0.0, min_warm_ms / max(probe["mean_ms"], 1e-3) - warmup)))
    st = driver.time(w.ex, w.sizes, w.c_ptrs(), w.dA.data_ptr(), w.dB.data_ptr(), warmup, iters)
    # the launch duration: `iters` launches back to back between two HIP events on the launch stream.  (The same launches
    # with an event between every two of them -- kernel_us_each_* below -- read 2-3 us longer each: the event's own cost.)
    mean_ms = st["batch_mean_ms"]
    primary, secondary = roofline(w, mean_ms)
    for r in (primary, secondary):
        if r["bound"] == "hbm":
            r["traffic"] = read_traffic(w.name)
        elif read_mfma_busy(w.name) is not None:
            r["mfma_busy_fraction_rocprof"] = read_mfma_busy(w.name)
    row = {"name": w.name, "sizes": w.sizes, "dtype": w.dtype, "flops": w.flops, "algorithmic_bytes": w.bytes,
           "kernel_us_mean": round(mean_ms * 1e3, 2),
           "kernel_us_each_mean": round(st["mean_ms"] * 1e3, 2), "kernel_us_median": round(st["median_ms"] * 1e3, 2),
           "kernel_us_min": round(st["min_ms"] * 1e3, 2),
           "gflops": round(w.flops / (mean_ms * 1e-3) / 1e9, 1),
           "roofline": primary, "roofline_other": secondary,
           "mapping": w.ex.info["spec"], "kernel": w.ex.last_kernel()}
    if primary["bound"] == "hbm" and 2 * w.nC * (8 if w.dtype == "f64" else 4) > 0.5 * w.bytes:
        # the same output tensor read, incremented and written back by a bare streaming kernel (non-temporal, 8 loads
        # in flight per lane) on the same rotated buffers: what the memory system gives the C traffic alone
        esize = 8 if w.dtype == "f64" else 4
        ms = driver.time_rmw(w.c_ptrs(), w.nC * esize, 1, 20, 50)
        row["c_rmw_stream_us"] = round(ms * 1e3, 2)
        row["c_rmw_stream_GBps"] = round(2 * w.nC * esize / ms / 1e6, 1)
        w.reset_c()
    return row


def cpu_baseline_and_verify(w, one_thread=False, repeat_s=1.0):
    """The CPU oracle (the reference's host nested-loop contraction, cogent/drivers/tccg/code_main_tccg_01.c:117-133)
    computes the WHOLE contraction on this box's cores: timed (median of a few runs when one takes under repeat_s
    seconds) and used to check EVERY element of one GPU launch from a fresh C.  one_thread: also one run on a single thread."""
    import numpy as np
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import helpers
    oracle = helpers.Oracle()
    expr = helpers.parse_expression(open(os.path.join(ROOT, "cgo2019-ae_amd", "expressions", w.plan_file)).read())
    threads = min(oracle.max_threads(), 16)
    want = w.hC.copy()
    runs = []
    while True:
        np.copyto(want, w.hC)
        t0 = time.perf_counter()
        oracle.contract(expr, w.sizes, want, w.hA, w.hB, threads=threads)
        runs.append(time.perf_counter() - t0)
        if sum(runs) >= repeat_s or len(runs) >= 9:
            break
    cpu_s = sorted(runs)[len(runs) // 2]
    base = {"value": round(w.flops / cpu_s / 1e9, 2), "unit": "GFLOP/s", "cores": threads, "kind": "port",
            "sample": "the whole contraction (%d flop), median of %d run(s), %.3f s each on %d threads" % (w.flops, len(runs), cpu_s, threads)}
    if one_thread:
        scratch = w.hC.copy()
        t0 = time.perf_counter()
        oracle.contract(expr, w.sizes, scratch, w.hA, w.hB, threads=1)
        t1 = time.perf_counter() - t0
        base["one_thread"] = {"value": round(w.flops / t1 / 1e9, 2), "unit": "GFLOP/s", "cores": 1, "seconds": round(t1, 3),
                              "identical_to_all_threads": bool(np.array_equal(scratch, want))}
    # one GPU launch from a fresh C, every element compared
    w.reset_c()
    w.launch(0)
    torch.cuda.synchronize()
    got = w.dC[0].cpu().numpy()
    err = helpers.rel_error(got, want)
    w.reset_c()
    verify = {"checked_elements": int(want.size), "of_elements": int(w.nC), "max_rel_err": err, "max_abs_err": float(np.max(np.abs(got.astype(np.float64) - want))),
              "tolerance": TOL[w.dtype], "definition": "|gpu-ref| / max(|ref|, rms(ref))", "pass": bool(err <= TOL[w.dtype])}
    return base, verify


ONE_THREAD = ("cfg1_", "cfg2_", "cfg4_16_", "cfg5_")      # the configs a single-thread CPU figure is reported for


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only-headline", action="store_true", help="skip the table of the other BASELINE configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / verification leg")
    ap.add_argument("--workload", default=HEADLINE, help="expression object to use as the headline workload")
    ap.add_argument("--suite", default="", help="'fused': time the fused groups of the manifest; 'tccg': time the 48 TCCG contractions at the sizes of the reference's "
                    "bench script (cogent/bench_tccg.sh:5-54) and print one JSON line with the table, instead of the headline run; "
                    "any other value: the manifest entries whose names start with it (comma-separated prefixes, e.g. 'smallk,ext4')")
    ap.add_argument("--ceilings", action="store_true",
                    help="only run the memory yardsticks: plain copy and bare read-modify-write streams (flat, and in the streaming "
                         "kernel's tiles of config 2's output) at the output sizes of the HBM-bound configs; one JSON line")
    ap.add_argument("--copy-only", type=int, default=0, metavar="BYTES",
                    help="only run the plain device-to-device copy kernel on BYTES bytes, --steps times "
                         "(the known-size yardstick the FETCH_SIZE / WRITE_SIZE counter readings are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (output tiles are independent, so "
              "the contraction would shard over the slowest output index without collectives, but no multi-GPU path is built)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import cogent_mi355 as pkg
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    tools = pkg.HostTools()
    driver = pkg.Driver()

    if args.copy_only:
        src = torch.ones(args.copy_only // 8, dtype=torch.float64, device="cuda")
        dst = torch.zeros(args.copy_only // 8, dtype=torch.float64, device="cuda")
        ms = driver.time_copy(src.data_ptr(), dst.data_ptr(), args.copy_only, args.warmup, args.steps)
        print(json.dumps({"copy_bytes": args.copy_only, "ms_per_copy": ms,
                          "GBps_read_plus_write": round(2 * args.copy_only / ms / 1e6, 1)}))
        return

    if args.ceilings:
        rows = []
        for label, nbytes in (("C4-16 output (fp32 16^6)", 4 * 16 ** 6), ("C5 output (fp64 16^6)", 8 * 16 ** 6),
                              ("C2 output (fp64 72^4)", 8 * 72 ** 4), ("C4-24 output (fp32 24^6)", 4 * 24 ** 6)):
            n_rot = max(2, min(8, int(1.2e9 // nbytes) + 1))
            bufs = [torch.zeros(nbytes // 8, dtype=torch.float64, device="cuda") for _ in range(n_rot)]
            ptrs = [b.data_ptr() for b in bufs]
            row = {"what": label, "bytes": nbytes, "buffers_rotated": n_rot}
            for mode, key in ((0, "rmw_flat"), (1, "rmw_flat_nontemporal")) + (((2, "rmw_stream_kernel_tiles"), (3, "rmw_stream_kernel_tiles_interleaved")) if nbytes == 8 * 72 ** 4 else ()):
                ms = min(driver.time_rmw(ptrs, nbytes, mode, 30, max(20, args.steps)) for _ in range(3))
                row[key] = {"us": round(ms * 1e3, 2), "GBps_read_plus_write": round(2 * nbytes / ms / 1e6, 1), "frac_of_8TBps": round(2 * nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
            ms = driver.time_copy(bufs[0].data_ptr(), bufs[1].data_ptr(), nbytes, 30, max(20, args.steps))
            row["copy"] = {"us": round(ms * 1e3, 2), "GBps_read_plus_write": round(2 * nbytes / ms / 1e6, 1)}
            rows.append(row)
            print("%-28s %s" % (label, {k: v["us"] for k, v in row.items() if isinstance(v, dict)}), file=sys.stderr, flush=True)
            del bufs
            torch.cuda.empty_cache()
        print(json.dumps({"ceilings": rows, "unit": "us per launch, mean over back-to-back launches on rotated buffers", "hbm_peak_GBps": HBM_PEAK_GBS}))
        return

    if args.suite == "fused":
        # fused groups: N contractions into one output in ONE kernel.  Algorithmic bytes: every input once,
        # the output read once and written once -- not once per term.
        import numpy as np
        rows = []
        for e in pkg.group_manifest():
            g = pkg.Group(e["name"])
            sizes = e["bench_sizes"]
            np_dtype = np.float64 if g.dtype == "f64" else np.float32
            esz = 8 if g.dtype == "f64" else 4
            ext = dict(zip(g.info["out_idx"] + g.info["sum_idx"], sizes))
            count = lambda names: int(np.prod([ext[n] for n in names], dtype=np.int64))
            nC = count(g.info["out_idx"])
            dev, in_elems = [], 0
            for k, term in enumerate(g.info["terms"]):
                m = term["mapping"]
                names = {"x": [n for n, _ in m["x"]] + [n for n, _ in m["k"]], "y": [n for n, _ in m["y"]] + [n for n, _ in m["k"]]}
                x_is_a = (m["x_operand"] == term["text"].split("*")[1].split("[")[0].strip())
                for which in ((0, 1) if x_is_a else (1, 0)):
                    n = count(names["x" if which == 0 else "y"])
                    in_elems += n
                    dev.append(torch.from_numpy(tools.fill_uniform(np.empty(n, np_dtype), 10 + len(dev))).cuda())
            n_rot = max(2, min(8, int(1.2e9 // (nC * esz)) + 1))
            cbufs = [torch.zeros(nC, dtype=torch.float64 if g.dtype == "f64" else torch.float32, device="cuda") for _ in range(n_rot)]
            st = driver.time_group(g, sizes, [c.data_ptr() for c in cbufs], [d.data_ptr() for d in dev], 3, max(5, min(args.steps, 50)))
            flops = 2 * int(np.prod(sizes, dtype=np.int64)) * g.n_terms
            nbytes = esz * (in_elems + 2 * nC)
            sec = st["batch_mean_ms"] * 1e-3            # launches back to back between two events (see time_workload)
            hbm = {"bound": "hbm", "achieved": round(nbytes / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                   "frac": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)}
            mfma = {"bound": "mfma", "achieved": round(flops / sec / 1e12, 3), "peak": MFMA_PEAK_TFLOPS[g.dtype],
                    "unit": "TFLOP/s", "frac": round(flops / sec / 1e12 / MFMA_PEAK_TFLOPS[g.dtype], 4)}
            # the bound is the pipe whose minimum time is longer: with the output moved once, the nine terms are MFMA work
            primary, secondary = (hbm, mfma) if nbytes / (HBM_PEAK_GBS * 1e9) >= flops / (MFMA_PEAK_TFLOPS[g.dtype] * 1e12) else (mfma, hbm)
            rows.append({"name": e["name"], "sizes": sizes, "dtype": g.dtype, "n_terms": g.n_terms, "flops": flops, "algorithmic_bytes": nbytes,
                         "bytes_if_run_term_by_term": esz * (in_elems + 2 * nC * g.n_terms),
                         "kernel_us_mean": round(sec * 1e6, 2), "kernel_us_each_mean": round(st["mean_ms"] * 1e3, 2), "kernel_us_min": round(st["min_ms"] * 1e3, 2),
                         "gflops": round(flops / sec / 1e9, 1),
                         "roofline": primary, "roofline_other": secondary,
                         "c_tile": g.info["c_tile"]})
            print("%-16s %s  %d terms  %8.1f us  %9.1f GFLOP/s" % (e["name"], sizes, g.n_terms, sec * 1e6, flops / sec / 1e9),
                  file=sys.stderr, flush=True)
        print(json.dumps({"suite": "fused", "unit": "GFLOP/s", "n_gpus": 1, "data": "synthetic", "rows": rows}))
        return

    if args.suite:
        rows = []
        for e in pkg.manifest():
            if not e["name"].startswith(tuple(args.suite.split(","))):
                continue
            wl = Workload(pkg, tools, e, e["bench_sizes"])
            r = time_workload(driver, wl, max(1, min(args.warmup, 3)), max(3, min(args.steps, 20)))
            rows.append(r)
            print("%-14s %-30s %10.1f us %9.1f GFLOP/s  %s %.3f" % (r["name"], r["sizes"], r["kernel_us_mean"], r["gflops"],
                                                              r["roofline"]["bound"], r["roofline"]["frac"]), file=sys.stderr, flush=True)
            del wl
            torch.cuda.empty_cache()
        print(json.dumps({"suite": args.suite, "unit": "GFLOP/s", "n_gpus": 1, "data": "synthetic", "rows": rows}))
        return

    entry = pkg.manifest_entry(args.workload)
    w = Workload(pkg, tools, entry, entry["bench_sizes"])

    cpu, verify = (None, None)
    if not args.no_cpu:
        cpu, verify = cpu_baseline_and_verify(w, one_thread=w.name.startswith(ONE_THREAD), repeat_s=5.0)

    # ---- the timed region: W warm-up steps, then exactly K steps between two synchronisations
    for i in range(args.warmup):
        w.launch(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        w.launch(i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # ---- per-launch kernel durations from HIP events on the launch stream
    head = time_workload(driver, w, args.warmup, args.steps)
    head["roofline"].setdefault("traffic", read_traffic(w.name))

    table = []
    if not args.only_headline:
        del w
        torch.cuda.empty_cache()
        for e in pkg.manifest():
            if not e["name"].startswith("cfg"):
                continue
            for sizes in [e["bench_sizes"]] + e.get("alt_sizes", []):
                wl = Workload(pkg, tools, e, sizes)
                row = time_workload(driver, wl, 10, 50)
                if not args.no_cpu:
                    row["cpu_baseline"], row["verify"] = cpu_baseline_and_verify(wl, one_thread=wl.name.startswith(ONE_THREAD))
                table.append(row)
                print("%-12s %-28s %8.1f us  %s %.3f  verify %s" % (row["name"], row["sizes"], row["kernel_us_mean"], row["roofline"]["bound"],
                      row["roofline"]["frac"], row.get("verify", {}).get("pass")), file=sys.stderr, flush=True)
                del wl
                torch.cuda.empty_cache()

    out = {
        "metric": "GFLOP/s per contraction (fp64/fp32) + % MFMA peak or % HBM GB/s, 1 GPU",
        "value": round(head["flops"] / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": "BASELINE config 2: fp64 C[a,b,c,d] += sum_e A[a,e,b]*B[d,e,c], all extents 72 "
                               "(column-major: %s)" % pkg.Expression(args.workload).expression.strip()
                   if args.workload == HEADLINE else args.workload,
                   "sizes": head["sizes"], "flops_per_step": head["flops"], "algorithmic_bytes_per_step": head["algorithmic_bytes"],
                   "mapping": head["mapping"], "c_buffers_rotated": True},
        "kernel_us_mean": head["kernel_us_mean"], "kernel_us_median": head["kernel_us_median"],
        "roofline": head["roofline"], "roofline_other": head["roofline_other"],
        "cpu_baseline": cpu, "verify": verify,
        "all_configs": table,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
