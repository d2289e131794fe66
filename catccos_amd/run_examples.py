"""Runs every operator of this build over the reference's own shape lists, the way the reference's
examples/run_all_examples.sh walks its example directories: one driver run per operator (which walks the list like the
example's scripts/run.sh), the log checked for the reference's failure patterns (run_all_examples.sh:38-70:
"error num: <n>", "[ERROR]", ...), a summary at the end, exit status 1 if anything failed.

    python -m catccos_amd.run_examples                       # perf mode (constant inputs), shape lists of tests/golden/reference_shapes.json
    python -m catccos_amd.run_examples --reference /path/to/catccos   # shape lists read from <reference>/examples/<op>/scripts/test_shapes.csv
    python -m catccos_amd.run_examples --only a5moe,dgds --iters 50

The numerical checks live in tests/ (the driver with data directories, against the oracle); this is the harness that
shows every operator starts, runs every listed shape on the tiled kernels and reports its latency.
"""
import argparse
import csv
import json
import os
import re
import subprocess
import sys
import tempfile

PKG = os.path.dirname(os.path.abspath(__file__))
DRIVER = os.path.join(PKG, "catccos_run")

# example directory of the reference -> (driver's short kernel name, options its scripts/run.sh implies)
OPERATORS = [
    ("ascend950_mx_quant_allgather", "mxqtag", []),
    ("allgather_matmul_dequant", "agmmdq", []),
    ("ascend950_mxfp8_matmul_reduce_scatter", "a5mxfp8mmrs", ["--transB", "1"]),
    ("dispatch_gmm_dequant_swiglu", "dgds", ["--experts", "16"]),
    ("ascend950_fp4_mx_alltoallv_grouped_matmul", "a5fp4mxatavgmm", ["--experts", "8"]),
    ("ascend950_fp8_mx_alltoallv_grouped_matmul", "a5fp8mxatavgmm", ["--experts", "8"]),
    ("ascend950_fp8_mx_grouped_matmul_alltoallv", "a5fp8gmmata", ["--experts", "8"]),
    ("ascend950_fp4_mx_grouped_matmul_alltoallv", "a5fp4gmmata", ["--experts", "8"]),
    ("ascend950_dispatch_ffn_combine", "a5moe", ["--experts", "16", "--topk", "6"]),
]

FAILURE_PATTERNS = [r"error num: [1-9][0-9]*", r"cchError:-?[0-9]+", r"\[ERROR\]", r"(^|\s)ERROR(\s|$)", r"\[WARN\] catccos_hip: GEMM .* falls back"]


def shape_lists(reference):
    """{example directory: [[M, K, N], ...]}"""
    if reference:
        out = {}
        for op, _, _ in OPERATORS:
            path = os.path.join(reference, "examples", op, "scripts", "test_shapes.csv")
            with open(path) as f:
                rows = [r for r in csv.reader(f) if r and r[0].strip()]
            out[op] = [[int(v) for v in r[:3]] for r in rows[1:]]
        return out
    fixture = os.path.join(os.path.dirname(PKG), "tests", "golden", "reference_shapes.json")
    with open(fixture) as f:
        return json.load(f)


def run_one(op, kernel, options, shapes, iters, warmup, log_dir):
    csv_path = os.path.join(log_dir, op + "_shapes.csv")
    with open(csv_path, "w") as f:
        f.write("M,K,N\n" + "".join("%d,%d,%d\n" % tuple(s) for s in shapes))
    cmd = [DRIVER, kernel, "--shapes", csv_path, "-"] + options + ["--iters", str(iters), "--warmup", str(warmup)]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = p.stdout
    with open(os.path.join(log_dir, op + ".log"), "w") as f:
        f.write(" ".join(cmd) + "\n" + log)
    bad = [pat for pat in FAILURE_PATTERNS if re.search(pat, log, re.M)]
    lat = [float(x) for x in re.findall(r"\[PERF\] Avg latency: ([0-9.]+) us/iter", log)]
    ok = p.returncode == 0 and not bad and len(lat) == len(shapes) and ("%d shapes finished" % len(shapes)) in log
    return ok, lat, bad, p.returncode


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--reference", help="root of a reference checkout: read its examples/<op>/scripts/test_shapes.csv")
    ap.add_argument("--only", help="comma-separated short kernel names (see catccos_run --list)")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--logs", help="directory for the per-operator logs (default: a temporary one)")
    a = ap.parse_args()
    if not os.path.exists(DRIVER):
        print("[ERROR] %s is missing: build it with `python -m catccos_amd.build`" % DRIVER)
        return 1
    lists = shape_lists(a.reference)
    only = set(a.only.split(",")) if a.only else None
    log_dir = a.logs or tempfile.mkdtemp(prefix="catccos_examples_")
    os.makedirs(log_dir, exist_ok=True)
    failed, total = [], 0
    print("%-46s %-16s %-22s %s" % ("example", "kernel", "shape (M,K,N)", "us/iter"))
    for op, kernel, options in OPERATORS:
        if only and kernel not in only:
            continue
        shapes = lists.get(op)
        if not shapes:
            print("%-46s %-16s no shape list" % (op, kernel))
            failed.append(op)
            continue
        total += 1
        ok, lat, bad, rc = run_one(op, kernel, options, shapes, a.iters, a.warmup, log_dir)
        for i, s in enumerate(shapes):
            print("%-46s %-16s %-22s %s" % (op, kernel, "%d,%d,%d" % tuple(s), "%.1f" % lat[i] if i < len(lat) else "-"))
        if not ok:
            failed.append(op)
            print("  FAILED (exit status %d%s): see %s" % (rc, "; log matches " + ", ".join(bad) if bad else "", os.path.join(log_dir, op + ".log")))
    print("summary: %d of %d operators ran every shape of their lists; logs in %s" % (total - len(failed), total, log_dir))
    if failed:
        print("failed: " + ", ".join(failed))
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
