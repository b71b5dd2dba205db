#!/usr/bin/env python3
"""Benchmark of the MI355X Accelerate backend.

Headline (the JSON line's `value`, `roofline`, `cpu_baseline`): one step = one application of the
prepared program `runN (scanl1 (+))` to a device-resident Int64 vector of 2^28 elements (one
launch of the pipelined single-pass scan kernel), through the C ABI.  The same line carries, under
"configs", every benchmark configuration (dotp, both scans, foldSeg, histogram, Jacobi) and the
2^28 map / dotp the bandwidth target is stated for, each with its own roofline entry and the CPU
figures of the same workload on one core and on all host cores.  Every roofline figure, the
headline's and the configurations', is algorithmic bytes / the MEAN time of a step over the timed
region, between HIP events recorded on the library's stream; the median is reported next to it
("us_median").  "transfer" gives what acchip_poke / acchip_peek move per second for the headline's
2 GiB input (never part of `value`).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--no-cpu] [--only ID]

--only ID runs one workload and nothing else (the form profiles are taken in); --quick the
headline only.  HBM traffic per launch comes from profiles/traffic.json, which records what
rocprofv3 counted for the kernels with the cache keys named there; a figure recorded for other
code is reported as null.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published peak
LLC_BYTES = 256 << 20   # MI355X last-level (memory-side) cache
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


WARMUP_FLOOR_MS = 40.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(ctx, run, args, steps, warmup):
    """(wall ms per step over exactly `steps` applications, list of per-step ms between events of a
    second pass, mean ms per step between the two events around the first pass)"""
    res = None
    t0 = time.perf_counter()
    for _ in range(warmup):
        res = run.execute(*args)
    ctx.sync()
    # Short steps: W of them end before the device has settled (foldSeg, 0.12 ms a step: 0.54 of
    # the roofline after 10 warm-up steps, 0.60 after 200 and after 1000), so the untimed part
    # lasts WARMUP_FLOOR_MS at least.  The timed part is exactly `steps` steps either way.
    while warmup > 0 and (time.perf_counter() - t0) * 1e3 < WARMUP_FLOOR_MS:
        for _ in range(10):
            res = run.execute(*args)
        ctx.sync()
    # exactly `steps` steps between two events (and two synchronisations): the figure
    e0 = ctx.event()
    t0 = time.perf_counter()
    for _ in range(steps):
        res = run.execute(*args)
    e1 = ctx.event()
    ctx.sync()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    mean = e0.elapsed_ms(e1) / steps
    # and once more with an event after every step, for the median: an event between two launches
    # costs the stream 1 to 3 us, which a step of 20 to 100 us would carry in its mean
    ev = [ctx.event()]
    for _ in range(steps):
        res = run.execute(*args)
        ev.append(ctx.event())
    ctx.sync()
    per = [ev[k].elapsed_ms(ev[k + 1]) for k in range(steps)]
    del res
    return wall, per, mean


def cpu_time(fn, reps):
    fn()
    best = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best.append(time.perf_counter() - t0)
    return statistics.median(best)


def traffic_for(workload, keys):
    """HBM bytes per launch recorded for this workload's kernels, or None when the record was
    taken on kernels with other cache keys (stale) or is absent."""
    try:
        rec = json.load(open(TRAFFIC_FILE))["workloads"].get(workload)
    except (OSError, ValueError, KeyError):
        return None
    if not rec or sorted(rec.get("kernel_keys", [])) != sorted(keys):
        return None
    return int(rec["fetch_bytes"] + rec["write_bytes"])


class Workloads:
    """The configurations: program, seeded inputs, algorithmic bytes, CPU loops."""

    def __init__(self):
        from accelerate_amd import ir as A, programs as P, workloads as W
        self.A, self.P, self.W = A, P, W
        self._cache = {}

    def ids(self):
        return ["scan_i64", "scan_f32", "map_f32", "dotp_2p28", "dotp_2p24", "foldseg", "histogram", "jacobi"]

    def vec(self, kind, n, seed):
        key = (kind, n, seed)
        if key not in self._cache:
            W = self.W
            self._cache[key] = {"i64": lambda: W.uniform_int(n, seed), "f01": lambda: W.uniform_f32(n, seed, 0.0, 1.0),
                                "f11": lambda: W.uniform_f32(n, seed)}[kind]()
        return self._cache[key]

    def drop(self):
        self._cache.clear()

    def make(self, wid):
        """dict(name, program, arg types, host args, elements, bytes, kernel, cpu(seq, omp) closures)"""
        A, P, W = self.A, self.P, self.W
        from oracle import c as OC
        n28 = 1 << 28
        if wid == "scan_i64":
            x = self.vec("i64", n28, 20240601)
            return dict(name="scanl1 (+) Int64 n=2^28", prog=P.scanl1_sum(A.i64), tys=[A.tarray(1, A.i64)], args=[x],
                        n=n28, bytes=16 * n28, kernel="acc_scan_pipe", unit="Gelem/s",
                        seq=lambda: OC.scanl1_i64(x), omp=lambda: OC.omp_scanl1(x), sample="full workload")
        if wid == "scan_f32":
            x = self.vec("f01", n28, 11)
            return dict(name="scanl1 (+) Float32 n=2^28", prog=P.scanl1_sum(A.f32), tys=[A.tarray(1, A.f32)], args=[x],
                        n=n28, bytes=8 * n28, kernel="acc_scan_pipe", unit="Gelem/s",
                        seq=lambda: OC.scanl1_f32(x), omp=lambda: OC.omp_scanl1(x), sample="full workload")
        if wid == "map_f32":
            x = self.vec("f01", n28, 11)
            return dict(name="map (\\x -> 2*x+1) Float32 n=2^28", prog=P.map_affine(), tys=[A.tarray(1, A.f32)], args=[x],
                        n=n28, bytes=8 * n28, kernel="acc_map_stream", unit="Gelem/s",
                        seq=lambda: np.add(np.multiply(x, np.float32(2)), np.float32(1)), omp=None,
                        sample="full workload (numpy, one core)")
        if wid in ("dotp_2p28", "dotp_2p24"):
            n = n28 if wid == "dotp_2p28" else 1 << 24
            x, y = self.vec("f01", n28, 11)[:n], self.vec("f11", n28, 12)[:n]
            return dict(name="dotp Float32 n=2^%d" % (28 if n == n28 else 24), prog=P.dotp(),
                        tys=[A.tarray(1, A.f32)] * 2, args=[x, y], n=n, bytes=8 * n + 4,
                        kernel="acc_fold_main_stream" if n == n28 else "acc_fold_main", unit="Gelem/s",
                        seq=lambda: OC.dotp_f32(x, y), omp=lambda: OC.omp_dotp_f32(x, y), sample="full workload")
        if wid == "foldseg":
            nseg, total = 1 << 20, 1 << 27
            vals, lens = W.uniform_int(total, 13, dtype=np.int32), W.segment_lengths(nseg, total, 14)
            offs = OC.offsets_i32(lens)
            return dict(name="foldSeg (+) 0 Int32, 2^27 values / 2^20 segments (offsets scan included)",
                        prog=P.foldseg_sum(), tys=[A.tarray(1, A.i32), A.tarray(1, A.i32)], args=[vals, lens], n=total,
                        bytes=4 * total + 4 * (nseg + 1) + 4 * nseg + 8 * nseg + 4, kernel="acc_foldseg", unit="Gelem/s",
                        seq=lambda: OC.foldseg_i32(vals, lens), omp=lambda: OC.omp_foldseg_i32(vals, OC.offsets_i32(lens)),
                        sample="full workload", check=lambda got: np.array_equal(got, OC.seq_foldseg_offsets_i32(vals, offs)))
        if wid == "histogram":
            nk, nb = 1 << 26, 1 << 16
            keys = W.zipf_keys(nk, nb, 15)
            counts = np.bincount(keys, minlength=nb)
            return dict(hot=(int(counts.max()), float(counts.max()) / nk),
                        name="histogram: permute (+) of 2^26 Zipf(1.1) keys into 2^16 Int32 bins", prog=P.histogram(nb),
                        tys=[A.tarray(1, A.i32)], args=[keys], n=nk, bytes=4 * nk + 8 * nb, kernel="acc_permute_count",
                        unit="Gelem/s", seq=lambda: OC.histogram_i32(keys, nb), omp=lambda: OC.omp_histogram_i32(keys, nb),
                        sample="full workload", check=lambda got: np.array_equal(got, np.bincount(keys, minlength=nb)))
        if wid == "jacobi":
            side = 8192
            g = W.uniform_f32(side * side, 16, 0.0, 1.0).reshape(side, side)
            return dict(name="Jacobi 3x3 cross, clamp, 8192x8192 Float32, per sweep of 100", prog=P.jacobi_step(),
                        tys=[A.tarray(2, A.f32)], args=[g], n=side * side, bytes=8 * side * side, kernel="acc_stencil2d",
                        unit="Gcell/s", iterate=100,
                        resident=True,   # a sweep reads the 256 MiB the previous one wrote
                        seq=lambda: OC.jacobi_f32(g, 2), omp=lambda: OC.omp_jacobi_f32(g, 4),
                        seq_units=2, omp_units=4, sample="2 (one core) / 4 (all cores) sweeps of the 100")
        raise KeyError(wid)


def run_workload(ctx, wl, steps, warmup, with_cpu, cpu_reps=3):
    """Time one workload on the GPU (and the CPU); returns (entry, wall ms per step, mean event ms)."""
    from accelerate_amd import hip  # noqa: F401
    run = ctx.compile(wl["prog"])
    dev = [ctx.to_device(a, t) for a, t in zip(wl["args"], wl["tys"])]
    if wl.get("iterate"):
        # the stencil configuration: `iterate` sweeps, each fed with the previous one's result
        it = wl["iterate"]
        g = dev[0]
        tw = time.perf_counter()
        for _ in range(max(5, warmup)):
            g = run.execute(g)
        ctx.sync()
        while (time.perf_counter() - tw) * 1e3 < WARMUP_FLOOR_MS:   # as in time_steps
            for _ in range(10):
                g = run.execute(g)
            ctx.sync()
        per, total, rounds = [], 0.0, max(1, steps // 10)
        t0 = time.perf_counter()
        for _ in range(rounds):   # the figure: `it` sweeps between two events
            g = dev[0]
            e0 = ctx.event()
            for _ in range(it):
                g = run.execute(g)
            e1 = ctx.event()
            ctx.sync()
            total += e0.elapsed_ms(e1)
        wall = (time.perf_counter() - t0) * 1e3 / (rounds * it)
        mean = total / (rounds * it)
        for _ in range(rounds):   # the median: an event after every sweep (see time_steps)
            g = dev[0]
            ev = [ctx.event()]
            for _ in range(it):
                g = run.execute(g)
                ev.append(ctx.event())
            ctx.sync()
            per += [ev[k].elapsed_ms(ev[k + 1]) for k in range(it)]
        del g
    else:
        wall, per, mean = time_steps(ctx, run, dev, steps, warmup)
    if "check" in wl:
        assert wl["check"](run.execute(*dev).to_host()), "result of %s differs from the oracle" % wl["name"]
    med = statistics.median(per)
    gbs = wl["bytes"] / mean / 1e6
    ws = wl.get("working_set", wl["bytes"])
    entry = {"workload": wl["name"], "elements": wl["n"], "algorithmic_bytes": wl["bytes"], "us": round(mean * 1e3, 2),
             "us_median": round(med * 1e3, 2), "steps_timed": len(per), "value": round(wl["n"] / mean / 1e6, 2),
             "unit": wl["unit"],
             "roofline": {"bound": "hbm", "kernel": wl["kernel"], "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                          "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                          "traffic": traffic_for(wl["name"], run.kernel_keys)},
             # what a step touches against the 256 MiB last-level cache: a resident working set is
             # served by the cache from the second step on, and its figure says nothing about HBM
             "working_set_bytes": ws, "cache_resident": bool(ws <= LLC_BYTES or wl.get("resident")),
             "kernel_keys": run.kernel_keys}
    if "hot" in wl:
        keys_hot, share = wl["hot"]
        entry["hottest_bin"] = {"updates_per_launch": keys_hot, "share_of_keys": round(share, 4),
                                "updates_per_s": round(keys_hot / (mean * 1e-3), 1),
                                "note": "updates of the most popular bin's counters per second of the whole step"}
    del dev
    if with_cpu:
        from oracle import c as OC
        su, ou = wl.get("seq_units", 1), wl.get("omp_units", 1)
        dt = cpu_time(wl["seq"], cpu_reps)
        entry["cpu_seq"] = {"value": round(wl["n"] * su / dt / 1e9, 4), "unit": wl["unit"], "cores": 1, "kind": "port",
                            "sample": wl["sample"]}
        if wl["omp"] is not None:
            dt = cpu_time(wl["omp"], cpu_reps)
            entry["cpu_omp"] = {"value": round(wl["n"] * ou / dt / 1e9, 4), "unit": wl["unit"], "cores": OC.omp_threads(),
                                "kind": "port", "sample": wl["sample"]}
    return entry, wall, mean


def measure_transfer(ctx, x, aty):
    """Host <-> device rates of the boundary's copies (acchip_poke / acchip_peek through pinned
    staging buffers) for one array, from and to pageable numpy memory; the second of two rounds."""
    out = {}
    for _ in range(2):
        t0 = time.perf_counter()
        d = ctx.to_device(x, aty)
        ctx.sync()
        t1 = time.perf_counter()
        h = d.to_host()
        t2 = time.perf_counter()
        out = {"bytes": int(x.nbytes), "h2d_GBs": round(x.nbytes / (t1 - t0) / 1e9, 2), "d2h_GBs": round(x.nbytes / (t2 - t1) / 1e9, 2),
               "note": "acchip_poke / acchip_peek of the headline's input, pageable host memory; not part of `value`"}
        del d, h
    return out


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (the first half dozen launches after an idle period run 3-5 % slower than the rest: the
    # default warm-up covers them; a step takes under a millisecond)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--quick", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--only", default=None, help="run one workload (an id of Workloads.ids()) and print its entry")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this backend runs on one GPU per process and has no multi-GPU path; "
                 "run with --gpus 1 (the per-GPU figure is the whole-job figure)")

    from accelerate_amd import hip
    ctx = hip.Context(0)   # fails loudly without the HIP library or a GPU: there is no fallback
    wls = Workloads()

    if a.only:
        entry, _, _ = run_workload(ctx, wls.make(a.only), a.steps, a.warmup, not a.no_cpu)
        print(json.dumps(entry), flush=True)
        return

    # ---- headline: scanl1 (+) on Int64, n = 2^28 -------------------------------------------
    log("headline: scanl1 (+) Int64 n=2^28 ...")
    wl = wls.make("scan_i64")
    x = wl["args"][0]
    wl["check"] = lambda got: int(got[-1]) == int(x.sum())     # cheap integrity check of the timed path
    head, wall, mean = run_workload(ctx, wl, a.steps, a.warmup, not a.no_cpu)
    achieved = wl["bytes"] / mean / 1e6       # average launch duration over the timed region
    transfer = measure_transfer(ctx, x, wl["tys"][0])
    cpu = None
    if not a.no_cpu:
        cpu = dict(head["cpu_omp"])
        cpu["sample"] = ("full workload (2^28 Int64), median of 3 runs of oracle/configs_omp.c oracle_omp_scanl1_i64 on %d "
                         "threads (%s); one core, oracle/configs.c: %s Gelem/s" % (cpu["cores"], cpu_model(),
                                                                                 head["cpu_seq"]["value"]))
        cpu["seq_value"] = head["cpu_seq"]["value"]
    out = {
        "metric": "Gelem/s + HBM GB/s (% peak) per skeleton: fold, scan, foldSeg, permute, stencil",
        "value": round(wl["n"] / wall / 1e6, 3), "unit": "Gelem/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int64", "data": "synthetic",
        "config": {"workload": "scanl1 (+) on an Int64 vector, n=2^28, uniform integers in [-1000,1000]",
                   "program": "Scan LeftToRight (+) Nothing (Manifest (Avar a0))", "kernel": "acc_scan_pipe"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": head["roofline"]["traffic"]},
        "cpu_baseline": cpu,
        "transfer": transfer,
        "warmup_floor_ms": WARMUP_FLOOR_MS,
    }

    # ---- every configuration, with its own roofline and CPU figures -------------------------
    if not a.quick:
        entries = [head]
        for wid in wls.ids()[1:]:
            log(wid, "...")
            steps = 50 if wid == "dotp_2p24" else max(20, a.steps)
            e, _, _ = run_workload(ctx, wls.make(wid), steps, a.warmup, not a.no_cpu)
            entries.append(e)
            if wid in ("dotp_2p24",):
                wls.drop()
        out["configs"] = entries
        out["host"] = {"cpu": cpu_model(), "threads": os.cpu_count()}

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
