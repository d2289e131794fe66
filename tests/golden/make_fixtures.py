#!/usr/bin/env python3
"""Writes the fixtures of this directory from the data the reference's own tests hold.

Run in a container that has the reference tree (default /root/reference); the fixtures are
committed, so tests never need the tree.  Nothing of the reference is imported or executed: the
shape lists are CSV data files, the scheduler vector is a brace list of integers read as text.

    python tests/golden/make_fixtures.py [/path/to/reference]

reference_shapes.json   {operator directory: [[M, K, N], ...]} from examples/<op>/scripts/test_shapes.csv
scheduler_kat.json      the expected vector of the reference's only numeric known-answer test
                        (tests/comm_block_scheduler_alltoallv_gmm/test_comm_block_scheduler_alltoallv_gmm.cpp:96-98)
                        with the parameters it is computed for (:37-60 of the same file)
"""
import csv
import json
import os
import re
import sys

OPS = [
    "ascend950_mx_quant_allgather", "allgather_matmul_dequant", "ascend950_mxfp8_matmul_reduce_scatter",
    "dispatch_gmm_dequant_swiglu", "ascend950_fp4_mx_alltoallv_grouped_matmul", "ascend950_fp8_mx_alltoallv_grouped_matmul",
    "ascend950_fp8_mx_grouped_matmul_alltoallv", "ascend950_fp4_mx_grouped_matmul_alltoallv", "ascend950_dispatch_ffn_combine",
]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    shapes = {}
    for op in OPS:
        with open(os.path.join(ref, "examples", op, "scripts", "test_shapes.csv")) as f:
            rows = list(csv.reader(f))
        assert [c.strip() for c in rows[0][:3]] == ["M", "K", "N"], rows[0]
        shapes[op] = [[int(v) for v in r[:3]] for r in rows[1:] if r and r[0].strip()]
    with open(os.path.join(here, "reference_shapes.json"), "w") as f:
        json.dump(shapes, f, indent=1, sort_keys=True)
        f.write("\n")

    src = open(os.path.join(ref, "tests", "comm_block_scheduler_alltoallv_gmm", "test_comm_block_scheduler_alltoallv_gmm.cpp")).read()
    m = re.search(r"expected\s*=\s*\{([^}]*)\}", src)
    expected = [int(v) for v in m.group(1).replace("\n", " ").split(",") if v.strip()]
    kat = {
        "source": "tests/comm_block_scheduler_alltoallv_gmm/test_comm_block_scheduler_alltoallv_gmm.cpp:96-98",
        "rank": 2, "ep": 4, "expert_per_rank": 2, "token_data": "i + 1 for i in range(32)",
        "queries": [{"core": 1, "num": 3}, {"core": 4, "num": 6}, {"core": 0, "num": 3}],
        "expected": expected,
    }
    with open(os.path.join(here, "scheduler_kat.json"), "w") as f:
        json.dump(kat, f, indent=1)
        f.write("\n")
    print("wrote reference_shapes.json (%d operators), scheduler_kat.json (%d values)" % (len(shapes), len(expected)))


if __name__ == "__main__":
    main()
