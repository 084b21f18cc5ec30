"""Runs bench/bench_vendor over the reference's published sweep (docs/performance.md: 512/1024/2048
square, C = 64, sparsity 0.9-0.5), the headline shape with and without a dense last row, the matvec
shape, and -- through --ellpack-file -- the benchmark configurations' own matrices (config 3: per-row
top-k; config 2b: Zipf row lengths), and prints one table.

    python sparse-ops_amd/bench/vendor_sweep.py [--runs 50] [--quick]
"""
import argparse
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "python"))
import datagen  # noqa: E402

BIN = os.path.join(HERE, "bench_vendor")
LINE = re.compile(r"^(.*?)\s*:\s+([0-9.]+) us\s+.*max rel diff(?: vs so_\w+)? ([0-9.e+-]+)\s*$")


def run(args):
    out = subprocess.run([BIN] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    if out.returncode != 0:
        sys.stdout.write(out.stdout)
        raise SystemExit("bench_vendor %s failed (%d)" % (" ".join(args), out.returncode))
    rows = {}
    for line in out.stdout.splitlines():
        m = LINE.match(line)
        if m:
            rows[m.group(1).strip()] = (float(m.group(2)), float(m.group(3)))
    return rows


def summarize(label, rows):
    ours = min((v[0], k) for k, v in rows.items() if k.startswith("Ellpack"))
    sparse = [(v[0], k) for k, v in rows.items() if k.startswith("rocSPARSE")]
    dense = [v[0] for k, v in rows.items() if k.startswith("rocBLAS")]
    worst = max(v[1] for v in rows.values())
    best_sparse = min(sparse) if sparse else (float("nan"), "-")
    print("| %-44s | %8.1f (%s) | %8.1f (%s) | %8.1f | %.1e |" % (
        label, ours[0], ours[1].split("(")[-1].rstrip(")"), best_sparse[0], best_sparse[1].split("(")[-1].rstrip(")"), dense[0] if dense else float("nan"), worst))
    sys.stdout.flush()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--runs", type=int, default=50)
    ap.add_argument("--quick", action="store_true", help="small shapes only")
    a = ap.parse_args()
    runs = ["--runs", str(a.runs)]
    print("| case | so_matmul / so_matvec us (fastest kernel) | rocSPARSE CSR us (best algorithm) | rocBLAS dense us | max rel diff |")
    print("|---|---|---|---|---|")
    sizes = [512] if a.quick else [512, 1024, 2048]
    for n in sizes:
        for sp in (0.9, 0.8, 0.7, 0.5):
            summarize("matmul %d^2 x 64 @ %.1f" % (n, sp),
                      run(["matmul", "--M", str(n), "--N", str(n), "--C", "64", "--sparsity", str(sp)] + runs))
    if not a.quick:
        for irr in (0, 1):
            summarize("matmul 4096^2 x 256 @ 0.9%s" % (", dense last row" if irr else ""),
                      run(["matmul", "--M", "4096", "--N", "4096", "--C", "256", "--sparsity", "0.9", "--irregular", str(irr)] + runs))
        for irr in (0, 1):
            summarize("matvec 16384^2 @ 0.95%s" % (", dense last row" if irr else ""),
                      run(["matvec", "--M", "16384", "--N", "16384", "--sparsity", "0.95", "--irregular", str(irr)] + runs))
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "m.ellpack")
        if a.quick:
            E, _, _ = datagen.config3(m=512, n=512, C=64)
            datagen.save_ellpack(path, E)
            summarize("matmul per-row top-10% 512^2 x 64 (file)", run(["matmul", "--ellpack-file", path, "--C", "64"] + runs))
        else:
            E, _, _ = datagen.config3()
            datagen.save_ellpack(path, E)
            summarize("config 3: matmul per-row top-10% 4096^2 x 256", run(["matmul", "--ellpack-file", path, "--C", "256"] + runs))
            E = datagen.config2b()[0]
            datagen.save_ellpack(path, E)
            summarize("config 2b: matvec Zipf rows 16384^2", run(["matvec", "--ellpack-file", path] + runs))


if __name__ == "__main__":
    main()
