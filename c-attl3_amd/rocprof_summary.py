"""Turns rocprofv3 output of `bench.py` runs into the short summaries kept under profiles/.

    python -m c-attl3_amd.rocprof_summary kernels  <dir with *_results.db>
    python -m c-attl3_amd.rocprof_summary counters <dir with *counter_collection.csv> [...]
    python -m c-attl3_amd.rocprof_summary traffic  <FETCH_SIZE dir> <WRITE_SIZE dir> --dtype f32 --batch 256 [--write]

(The package directory is not an identifier: run it as `python c-attl3_amd/rocprof_summary.py ...`.)

`traffic` needs the two counter runs to have been made with `bench.py --copy-calibration`, which adds a plain copy kernel of
known size: each counter is scaled by what it reads for that copy. With --write it rewrites
profiles/conv_cfg4_hbm_traffic.json, which `bench.py` reads for `roofline.traffic`, together with a hash of the kernel
sources, so that figures measured on other sources are never reported.
"""
import argparse
import collections
import csv
import glob
import hashlib
import json
import os
import sqlite3
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNEL_SOURCES = ("c-attl3_amd/csrc/gemm_kernels.hip", "c-attl3_amd/csrc/common.hpp")      # as in bench.py
PASSES = ("gather_gemm_kernel (forward)", "wgrad_kernel (+ reduce, bias column sums)", "gather_gemm_kernel (input gradient)")


def short(name):
    return name.replace("void cattle_hip::(anonymous namespace)::", "").split("(")[0]


def kernel_sources_hash():
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def kernels(directory, limit=16):
    """The top_kernels view of a `rocprofv3 --kernel-trace --stats` run as a markdown table (microseconds)."""
    out = ["| kernel | calls | total us | average us | % |", "|---|---|---|---|---|"]
    for db in sorted(glob.glob(os.path.join(directory, "**", "*_results.db"), recursive=True)):
        con = sqlite3.connect(db)
        rows = con.execute("select name, total_calls, total_duration, average, percentage from top_kernels").fetchall()
        for name, calls, total, avg, pct in rows[:limit]:
            out.append("| `%s` | %d | %.1f | %.1f | %.2f |" % (short(name), calls, total, avg, pct))      # the view is in microseconds
    return "\n".join(out)


def read_counters(directory):
    """[(dispatch id, kernel, counter, value)] of a `rocprofv3 --pmc ... --output-format csv` run, in dispatch order."""
    rows = []
    for path in sorted(glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)):
        with open(path) as f:
            for r in csv.DictReader(f):
                rows.append((int(r["Dispatch_Id"]), short(r["Kernel_Name"]), r["Counter_Name"], float(r["Counter_Value"])))
    rows.sort(key=lambda r: r[0])
    return rows


def counters(directories):
    """Mean counter value per dispatch, per kernel, as a markdown table."""
    agg = collections.OrderedDict()
    names = []
    for d in directories:
        for _, kernel, counter, value in read_counters(d):
            agg.setdefault(kernel, collections.OrderedDict()).setdefault(counter, []).append(value)
            if counter not in names:
                names.append(counter)
    out = ["| kernel | dispatches | " + " | ".join(names) + " |", "|---|---|" + "---|" * len(names)]
    for kernel, per in agg.items():
        n = max(len(v) for v in per.values())
        cells = ["%.6g" % (sum(per[c]) / len(per[c])) if c in per else "" for c in names]
        out.append("| `%s` | %d | %s |" % (kernel, n, " | ".join(cells)))
    return "\n".join(out)


def per_pass(rows, copy_kernel_prefix="act_forward_kernel"):
    """Mean counter value per dispatch for the three GEMM passes (each with its reduce launch) and for the
    calibration copy. A gather launch that follows a weight-gradient launch is the input gradient, any other one the
    forward pass; reduce launches belong to the GEMM launch before them."""
    sums = collections.defaultdict(list)
    last = None
    current = None
    for _, kernel, _, value in rows:
        if kernel.startswith("gather_gemm_kernel"):
            current = PASSES[2] if last == "wgrad" else PASSES[0]
            last = "gather"
            sums[current + " | kernel"].append(value)
        elif kernel.startswith("wgrad_kernel"):
            current = PASSES[1]
            last = "wgrad"
            sums[current + " | kernel"].append(value)
        elif kernel.startswith("split_reduce_kernel") or kernel.startswith("reduce_partials"):
            if current is not None:
                sums[current + " | reduce"].append(value)
        elif kernel.startswith(copy_kernel_prefix):
            sums["copy"].append(value)
    return {k: sum(v) / len(v) for k, v in sums.items()}


def traffic(fetch_dir, write_dir, dtype, batch, write):
    es = 4 if dtype == "f32" else 8
    copy_bytes = batch * 56 * 56 * 64 * es             # the identity activation reads and writes one input-sized tensor
    fetch, wr = per_pass(read_counters(fetch_dir)), per_pass(read_counters(write_dir))
    if "copy" not in fetch or "copy" not in wr:
        sys.exit("no calibration copy in the counter runs: run bench.py with --copy-calibration")
    f_fac, w_fac = copy_bytes / (fetch["copy"] * 1024.0), copy_bytes / (wr["copy"] * 1024.0)
    entry = {}
    lines = ["| pass | read MB (kernel + reduce) | written MB (kernel + reduce) | total MB |", "|---|---|---|---|"]
    for p in PASSES:
        rk, rr = fetch.get(p + " | kernel", 0.0) * 1024 * f_fac, fetch.get(p + " | reduce", 0.0) * 1024 * f_fac
        wk, wrd = wr.get(p + " | kernel", 0.0) * 1024 * w_fac, wr.get(p + " | reduce", 0.0) * 1024 * w_fac
        entry[p] = round(rk + rr + wk + wrd)
        lines.append("| %s | %.1f + %.1f | %.1f + %.1f | %.1f |" % (p, rk / 1e6, rr / 1e6, wk / 1e6, wrd / 1e6, entry[p] / 1e6))
    print("calibration copy: %d bytes each way; FETCH_SIZE reads %.1f KiB (factor %.3f), WRITE_SIZE %.1f KiB (factor %.3f)"
          % (copy_bytes, fetch["copy"], f_fac, wr["copy"], w_fac))
    print("\n".join(lines))
    if write:
        path = os.path.join(ROOT, "profiles", "conv_cfg4_hbm_traffic.json")
        try:
            with open(path) as f:
                rec = json.load(f)
        except (OSError, ValueError):
            rec = {}
        h = kernel_sources_hash()
        if rec.get("kernel_sources_sha256_16") != h:
            rec = {"entries": {}}
        rec["kernel_sources_sha256_16"] = h
        rec["kernel_sources"] = list(KERNEL_SOURCES)
        rec["fetch_factor"], rec["write_factor"] = round(f_fac, 4), round(w_fac, 4)
        rec["unit"] = "bytes per launch, kernel and its reduce launch, read + written"
        rec["entries"]["%s:%d" % (dtype, batch)] = entry
        with open(path, "w") as f:
            json.dump(rec, f, indent=1, sort_keys=True)
            f.write("\n")
        print("wrote", path)


def main():
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="cmd", required=True)
    k = sub.add_parser("kernels")
    k.add_argument("directory")
    c = sub.add_parser("counters")
    c.add_argument("directories", nargs="+")
    t = sub.add_parser("traffic")
    t.add_argument("fetch_dir")
    t.add_argument("write_dir")
    t.add_argument("--dtype", default="f32")
    t.add_argument("--batch", type=int, default=256)
    t.add_argument("--write", action="store_true")
    a = ap.parse_args()
    if a.cmd == "kernels":
        print(kernels(a.directory))
    elif a.cmd == "counters":
        print(counters(a.directories))
    else:
        traffic(a.fetch_dir, a.write_dir, a.dtype, a.batch, a.write)


if __name__ == "__main__":
    main()
