"""Turn rocprofv3 CSV output for the benchmark workloads into the summaries kept under profiles/.

Input: one directory per workload id (bench.py --only ID), holding

  entry.json            the line bench.py --only ID printed (workload name, kernel cache keys)
  kt/    rocprofv3 --kernel-trace --stats ...           -> *_kernel_stats.csv
  fetch/ rocprofv3 --pmc FETCH_SIZE --kernel-trace ...  -> *_counter_collection.csv
  write/ rocprofv3 --pmc WRITE_SIZE --kernel-trace ...
  sq1/, sq2/, ...  further --pmc passes (any counters)

  python -m accelerate_amd.rocprof_summary RUN_DIR --calibrate map_f32 --out profiles

writes profiles/<id>.md per workload and profiles/traffic.json.  FETCH_SIZE and WRITE_SIZE count
KiB per dispatch in units that are not bytes on every part; both are scaled by what they read for
the map kernel of the calibration workload, which moves exactly 4 bytes per element each way.
"""
from __future__ import annotations

import argparse
import csv
import glob
import json
import os
from collections import defaultdict


def _find(d, pattern):
    hits = glob.glob(os.path.join(d, "**", pattern), recursive=True)
    return hits[0] if hits else None


def kernel_stats(d):
    """[(kernel, calls, average ns, min ns, max ns)] from a --kernel-trace --stats run."""
    f = _find(d, "*kernel_stats.csv")
    if not f:
        return []
    out = []
    for r in csv.DictReader(open(f)):
        out.append((r["Name"], int(r["Calls"]), float(r["AverageNs"]), float(r["MinNs"]), float(r["MaxNs"])))
    return out


def kernel_trace(d):
    """{kernel: [duration ns of every dispatch, in start order]} from a --kernel-trace run."""
    f = _find(d, "*kernel_trace.csv")
    if not f:
        return {}
    per = defaultdict(list)
    for r in csv.DictReader(open(f)):
        per[r["Kernel_Name"]].append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]) - int(r["Start_Timestamp"])))
    return {k: [d for _, d in sorted(v)] for k, v in per.items()}


def counters(d):
    """{kernel: {counter: mean value per dispatch}} from a --pmc run."""
    f = _find(d, "*counter_collection.csv")
    if not f:
        return {}
    acc = defaultdict(lambda: defaultdict(list))
    per_dispatch = defaultdict(lambda: defaultdict(float))
    for r in csv.DictReader(open(f)):
        per_dispatch[(r["Kernel_Name"], r["Dispatch_Id"])][r["Counter_Name"]] += float(r["Counter_Value"])
    for (k, _), cs in per_dispatch.items():
        for c, v in cs.items():
            acc[k][c].append(v)
    return {k: {c: sum(v) / len(v) for c, v in cs.items()} for k, cs in acc.items()}


def derived(others, avg_ns, elements):
    """What the counters say about where a kernel's time goes, per kernel that runs for at least
    10 us: the share of their life the waves spend waiting (SQ_WAIT_ANY / SQ_WAVE_CYCLES) and
    waiting for LDS, vector instructions per element of the workload, the time the vector
    instructions alone would take on 1024 SIMDs at 4 cycles each and 2.4 GHz, and the share of
    LDS cycles lost to bank conflicts."""
    out = ["## Derived", "", "| kernel | waves waiting | waiting for LDS | VALU instr / element | VALU issue time | LDS cycles in conflict |",
           "|---|---|---|---|---|---|"]
    rows = 0
    for k in sorted(others):
        c = others[k]
        if avg_ns.get(k, 0.0) < 10e3 or not c.get("SQ_WAVE_CYCLES"):
            continue
        valu = c.get("SQ_INSTS_VALU", 0.0)
        issue_us = valu / 1024.0 * 4.0 / 2400.0
        conflict = c.get("SQ_LDS_BANK_CONFLICT", 0.0) / c["SQ_LDS_IDX_ACTIVE"] if c.get("SQ_LDS_IDX_ACTIVE") else 0.0
        out.append("| `%s` | %.0f %% | %.0f %% | %.1f | %.0f us of %.0f us | %.0f %% |"
                   % (k, 100.0 * c.get("SQ_WAIT_ANY", 0.0) / c["SQ_WAVE_CYCLES"],
                      100.0 * c.get("SQ_WAIT_INST_LDS", 0.0) / c["SQ_WAVE_CYCLES"], valu * 64.0 / elements, issue_us,
                      avg_ns[k] / 1e3, 100.0 * conflict))
        rows += 1
    return out + [""] if rows else []


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("run_dir")
    ap.add_argument("--calibrate", default="map_f32", help="workload id whose map kernel moves 4 B per element each way")
    ap.add_argument("--out", default="profiles")
    ap.add_argument("--commands", default=None, help="text file with the commands that produced RUN_DIR (quoted in the summaries)")
    a = ap.parse_args()
    ids = sorted(x for x in os.listdir(a.run_dir) if os.path.isdir(os.path.join(a.run_dir, x)))
    cal = os.path.join(a.run_dir, a.calibrate)
    entry = json.load(open(os.path.join(cal, "entry.json")))
    moved = entry["elements"] * 4
    fk = counters(os.path.join(cal, "fetch"))
    wk = counters(os.path.join(cal, "write"))
    mapk = [k for k in fk if k.startswith("acc_map")][0]
    f_fetch = moved / (fk[mapk]["FETCH_SIZE"] * 1024.0)
    f_write = moved / (wk[mapk]["WRITE_SIZE"] * 1024.0)
    commands = open(a.commands).read() if a.commands else ""
    traffic = {"calibration": {"workload": entry["workload"], "kernel": mapk, "bytes_each_way": moved,
                               "fetch_factor": round(f_fetch, 4), "write_factor": round(f_write, 4)},
               "workloads": {}}
    os.makedirs(a.out, exist_ok=True)
    for wid in ids:
        d = os.path.join(a.run_dir, wid)
        if not os.path.exists(os.path.join(d, "entry.json")):
            continue
        e = json.load(open(os.path.join(d, "entry.json")))
        ks = kernel_stats(os.path.join(d, "kt"))
        fc, wc = counters(os.path.join(d, "fetch")), counters(os.path.join(d, "write"))
        others = {}
        for sub in sorted(os.listdir(d)):
            if sub.startswith("sq") and os.path.isdir(os.path.join(d, sub)):
                for k, cs in counters(os.path.join(d, sub)).items():
                    others.setdefault(k, {}).update(cs)
        lines = ["# %s" % e["workload"], "",
                 "Workload id `%s` of bench.py; kernel cache keys: %s." % (wid, ", ".join("`%s`" % k[:16] for k in e["kernel_keys"])),
                 "bench.py's own figure in the profiled run: %.2f us per step (mean; median %.2f), %.1f GB/s of %d algorithmic bytes = %.4f of 8 TB/s."
                 % (e["us"], e.get("us_median", e["us"]), e["roofline"]["achieved"], e["algorithmic_bytes"], e["roofline"]["frac"]), ""]
        if wid == a.calibrate:
            lines += ["This workload is the calibration of FETCH_SIZE / WRITE_SIZE: its traffic below equals its algorithmic bytes by "
                      "construction and is not a measurement.", ""]
        # The profiled run launches every kernel a few times before the launches bench.py times
        # (warm-up), and those run slower; "later half" is the mean over the second half of a
        # kernel's dispatches in start order, which holds timed launches only, and is the figure
        # to hold against bench.py's.
        kt = kernel_trace(os.path.join(d, "kt"))
        lines += ["## Kernel trace (rocprofv3 --kernel-trace --stats)", "",
                  "| kernel | calls | average us (all) | median us | later half us | min us | max us |", "|---|---|---|---|---|---|---|"]
        for name, calls, avg, mn, mx in ks:
            ds = kt.get(name, [])
            later = ds[len(ds) // 2:]
            med = sorted(ds)[len(ds) // 2] / 1e3 if ds else float("nan")
            lh = sum(later) / len(later) / 1e3 if later else float("nan")
            lines.append("| `%s` | %d | %.2f | %.2f | %.2f | %.2f | %.2f |" % (name, calls, avg / 1e3, med, lh, mn / 1e3, mx / 1e3))
        lines += ["", "## HBM traffic per launch (FETCH_SIZE, WRITE_SIZE; factors %.4f / %.4f from `%s` over %d bytes each way)"
                  % (f_fetch, f_write, mapk, moved), "", "| kernel | read MiB | written MiB |", "|---|---|---|"]
        tot_f = tot_w = 0.0
        for k in sorted(set(fc) | set(wc)):
            rb = fc.get(k, {}).get("FETCH_SIZE", 0.0) * 1024.0 * f_fetch
            wb = wc.get(k, {}).get("WRITE_SIZE", 0.0) * 1024.0 * f_write
            tot_f += rb
            tot_w += wb
            lines.append("| `%s` | %.2f | %.2f |" % (k, rb / 2**20, wb / 2**20))
        lines += ["", "All launches of one step together: %.2f MiB read + %.2f MiB written = %.3f x the %.2f MiB the algorithm needs."
                  % (tot_f / 2**20, tot_w / 2**20, (tot_f + tot_w) / e["algorithmic_bytes"], e["algorithmic_bytes"] / 2**20), ""]
        if others:
            lines += ["## Other counters (mean per launch, summed over the device)", ""]
            for k in sorted(others):
                lines.append("`%s`: " % k + ", ".join("%s %d" % (c, round(v)) for c, v in sorted(others[k].items())))
                lines.append("")
            lines += derived(others, {name: avg for name, _, avg, _, _ in ks}, e["elements"])
        if commands:
            lines += ["## Commands", "", "```", commands.replace("$ID", wid).rstrip(), "```", ""]
        open(os.path.join(a.out, wid + ".md"), "w").write("\n".join(lines))
        traffic["workloads"][e["workload"]] = {"id": wid, "kernel_keys": e["kernel_keys"], "fetch_bytes": int(tot_f),
                                               "write_bytes": int(tot_w)}
    json.dump(traffic, open(os.path.join(a.out, "traffic.json"), "w"), indent=1, sort_keys=True)
    print("wrote", len(traffic["workloads"]), "summaries to", a.out)


if __name__ == "__main__":
    main()
