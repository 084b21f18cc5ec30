"""Condenses rocprofv3 output into the short text summaries kept under profiles/.

    # counters (one rocprofv3 --pmc run per counter group; csv output):
    python sparse-ops_amd/bench/pmc_summary.py counters <counter_collection.csv> [...more csv] [--kernels REGEX]
    # kernel durations of a --kernel-trace run (csv output):
    python sparse-ops_amd/bench/pmc_summary.py trace <kernel_trace.csv> [--kernels REGEX] [--skip N]
    # the kernels of one forward pass of a layer chain, in launch order (averages over the passes found):
    python sparse-ops_amd/bench/pmc_summary.py layers <kernel_trace.csv> --last gap_kernel
    # HBM-side bytes per launch from a FETCH_SIZE run and a WRITE_SIZE run, scaled by the plain copy
    # kernel of known size that `bench.py --calibrate-copy` launches, written into the table bench.py
    # reads `roofline.traffic` from:
    python sparse-ops_amd/bench/pmc_summary.py traffic <fetch.csv> <write.csv> --update profiles/hbm_traffic.json

Every mode prints per-kernel averages per dispatch; template arguments are kept, argument lists cut.
"""
import argparse
import collections
import csv
import hashlib
import json
import os
import re
import statistics
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
COPY_KERNEL = "act_kernel<0,true>"     # the streaming instantiation of the plain copy, as short_name() writes it
COPY_KIB = 262144.0      # bench.py --calibrate-copy: 256 MiB read, 256 MiB written per launch (run it with
                         # --skip-extra stream_copy --skip-extra stream_copy_256MiB: the same kernel at other sizes)

# Source files whose text decides a kernel's memory traffic: the table stores their hash, and
# bench.py reports a kernel's traffic only while the hash still matches.
KERNEL_SOURCES = {
    "ellpack_matmul_tiled_kernel": ["sparse-ops_amd/csrc/matmul_tiled.hip", "sparse-ops_amd/csrc/dpp_steps.h",
                                    "sparse-ops_amd/csrc/lds_sync.h", "sparse-ops_amd/csrc/so_internal.h"],
    "ellpack_matmul_rbm_kernel": ["sparse-ops_amd/csrc/matmul_rbm.hip", "sparse-ops_amd/csrc/gen_matmul_rbm_steps.py",
                                  "sparse-ops_amd/csrc/so_internal.h"],
    "ellpack_matmul_kernel": ["sparse-ops_amd/csrc/matmul.hip", "sparse-ops_amd/csrc/so_internal.h"],
    "matvec_rows_kernel": ["sparse-ops_amd/csrc/matvec.hip"],
    "matvec_binned_kernel": ["sparse-ops_amd/csrc/matvec.hip"],
}


def short_name(name):
    """void ns::kernel<1, 2>(args...) [clone] -> kernel<1, 2>"""
    name = re.sub(r"\s*\[clone.*$", "", name.strip())
    name = name.replace("(anonymous namespace)::", "")
    depth, cut = 0, len(name)
    for i, ch in enumerate(name):
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            cut = i
            break
    return re.sub(r"^void\s+", "", name[:cut]).replace(", ", ",")


def source_hash(kernel):
    """sha1 over the kernel's source files (None for a kernel not in KERNEL_SOURCES)."""
    base = kernel.split("<")[0]
    files = KERNEL_SOURCES.get(base)
    if not files:
        return None
    h = hashlib.sha1()
    for f in files:
        with open(os.path.join(ROOT, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def read_counters(paths, pattern):
    vals = collections.defaultdict(lambda: collections.defaultdict(list))
    for path in paths:
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                k = short_name(r["Kernel_Name"])
                if pattern and not re.search(pattern, k):
                    continue
                vals[k][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return vals


def cmd_counters(a):
    vals = read_counters(a.csv, a.kernels)
    print("%-52s %-28s %10s %18s %16s %16s" % ("kernel", "counter", "dispatches", "avg per dispatch", "min", "max"))
    for k in sorted(vals):
        for c in sorted(vals[k]):
            v = vals[k][c]
            print("%-52s %-28s %10d %18.1f %16.1f %16.1f" % (k, c, len(v), sum(v) / len(v), min(v), max(v)))


def cmd_trace(a):
    dur = collections.defaultdict(list)
    with open(a.csv[0], newline="") as f:
        for r in csv.DictReader(f):
            k = short_name(r["Kernel_Name"])
            if a.kernels and not re.search(a.kernels, k):
                continue
            dur[k].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    total = sum(sum(v) for v in dur.values())
    print("%-52s %8s %12s %12s %12s %12s %8s" % ("kernel", "calls", "avg us", "median us", "min us", "max us", "% time"))
    for k, v in sorted(dur.items(), key=lambda kv: -sum(kv[1])):
        w = v[a.skip:] if len(v) > a.skip else v
        print("%-52s %8d %12.2f %12.2f %12.2f %12.2f %8.1f" % (k, len(v), sum(w) / len(w), statistics.median(w), min(w), max(w),
                                                               100.0 * sum(v) / total))
    if a.skip:
        print("(avg / median / min / max leave out each kernel's first %d calls)" % a.skip)


def cmd_layers(a):
    """A forward pass = the dispatches up to and including the one after each dispatch of the kernel
    named by --last (a chain's second-to-last layer) whose grid is the largest seen for that kernel
    (the largest batch); passes are as long as the most common distance between two such dispatches."""
    with open(a.csv[0], newline="") as f:
        rows = sorted(csv.DictReader(f), key=lambda r: int(r["Start_Timestamp"]))
    names = [short_name(r["Kernel_Name"]) for r in rows]
    grid = [int(r.get("Grid_Size") or r.get("Grid_Size_X") or 0) for r in rows]
    marks = [i for i, k in enumerate(names) if k.split("<")[0] == a.last]
    if not marks:
        sys.exit("no dispatch of %s in the trace" % a.last)
    big = max(grid[i] for i in marks)
    marks = [i for i in marks if grid[i] == big and i + 1 < len(rows)]
    gaps = collections.Counter(b - c for c, b in zip(marks, marks[1:]))
    if not gaps:
        sys.exit("fewer than two passes in the trace")
    count = gaps.most_common(1)[0][0]
    passes = [list(range(i + 2 - count, i + 2)) for i in marks if i + 2 - count >= 0]
    ref = [names[j] for j in passes[-1]]
    passes = [p for p in passes if [names[j] for j in p] == ref]
    print("%d kernels per pass, %d passes with this sequence (grid of %s: %d work-items)" % (count, len(passes), a.last, big))
    print("%3s %-44s %12s %10s %10s %10s" % ("#", "kernel", "grid", "avg us", "min us", "max us"))
    total = 0.0
    for pos in range(count):
        d = [(int(rows[p[pos]]["End_Timestamp"]) - int(rows[p[pos]]["Start_Timestamp"])) / 1e3 for p in passes]
        total += sum(d) / len(d)
        print("%3d %-44s %12d %10.1f %10.1f %10.1f" % (pos + 1, ref[pos], grid[passes[-1][pos]], sum(d) / len(d), min(d), max(d)))
    span = [(int(rows[p[-1]]["End_Timestamp"]) - int(rows[p[0]]["Start_Timestamp"])) / 1e3 for p in passes]
    print("sum of the kernels %.1f us; first start to last end of a pass: avg %.1f us, min %.1f us" % (total, sum(span) / len(span), min(span)))


def cmd_traffic(a):
    fetch = read_counters([a.csv[0]], None)
    write = read_counters([a.csv[1]], None)

    def avg(table, kernel, counter):
        v = table.get(kernel, {}).get(counter)
        return sum(v) / len(v) if v else None
    f_copy, w_copy = avg(fetch, COPY_KERNEL, "FETCH_SIZE"), avg(write, COPY_KERNEL, "WRITE_SIZE")
    if not f_copy or not w_copy:
        sys.exit("the runs hold no %s dispatches: run bench.py with --calibrate-copy" % COPY_KERNEL)
    f_scale, w_scale = COPY_KIB / f_copy, COPY_KIB / w_copy
    print("calibration: %s reads and writes %.0f KiB; FETCH_SIZE reads %.1f (x %.3f), WRITE_SIZE reads %.1f (x %.3f)"
          % (COPY_KERNEL, COPY_KIB, f_copy, f_scale, w_copy, w_scale))
    table = {}
    if a.update and os.path.exists(a.update):
        with open(a.update) as f:
            table = json.load(f)
    print("%-52s %14s %14s %16s" % ("kernel", "fetched KiB", "written KiB", "bytes per launch"))
    for k in sorted(fetch):
        if k == COPY_KERNEL or k.startswith("__amd") or (a.kernels and not re.search(a.kernels, k)):
            continue
        fk, wk = avg(fetch, k, "FETCH_SIZE"), avg(write, k, "WRITE_SIZE")
        if fk is None or wk is None:
            continue
        nbytes = int(round((fk * f_scale + wk * w_scale) * 1024))
        print("%-52s %14.1f %14.1f %16d" % (k, fk * f_scale, wk * w_scale, nbytes))
        sha = source_hash(k)
        if sha:
            entry = {"bytes_per_launch": nbytes, "fetched_kib": round(fk * f_scale, 1), "written_kib": round(wk * w_scale, 1),
                     "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4), "source_sha1": sha,
                     "dispatches": len(fetch[k]["FETCH_SIZE"])}
            if a.workload:
                entry["workload"] = a.workload
            table[k if not a.workload else k + " | " + a.workload] = entry
    if a.update:
        with open(a.update, "w") as f:
            json.dump(table, f, indent=1, sort_keys=True)
            f.write("\n")
        print("updated", a.update)


def lookup_traffic(table_path, kernel, workload=None):
    """bench.py's reader: bytes per launch of `kernel` (with its template arguments, or the bare name:
    then any instantiation measured on `workload` matches), or None when the table has no such entry
    or the kernel's sources have changed since it was measured."""
    try:
        with open(table_path) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    for key, e in table.items():
        name, _, wl = key.partition(" | ")
        if (name == kernel or name.split("<")[0] == kernel) and (workload is None or wl == workload):
            return e["bytes_per_launch"] if e.get("source_sha1") == source_hash(name) else None
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("mode", choices=["counters", "trace", "layers", "traffic"])
    ap.add_argument("csv", nargs="+")
    ap.add_argument("--kernels", default=None, help="regular expression on the short kernel name")
    ap.add_argument("--skip", type=int, default=0, help="trace: calls to leave out of the averages (warm-up)")
    ap.add_argument("--last", default="gap_kernel", help="layers: name of the chain's second-to-last kernel")
    ap.add_argument("--update", default=None, help="traffic: JSON table to update")
    ap.add_argument("--workload", default=None, help="traffic: key suffix when one kernel is measured on several workloads")
    a = ap.parse_args()
    {"counters": cmd_counters, "trace": cmd_trace, "layers": cmd_layers, "traffic": cmd_traffic}[a.mode](a)


if __name__ == "__main__":
    main()
