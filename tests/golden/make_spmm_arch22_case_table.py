"""Writes tests/golden/spmm_arch22_cases.csv: the case table of the reference's arch22 SpMM test program
(kTestCases in test/spmm/arch22/spmm_test.cpp:446-), as data: M, K, N, nnz, alpha, beta, row distribution.

The reference file is read as text; nothing of it is run.

    python tests/golden/make_spmm_arch22_case_table.py /root/reference
"""
import csv
import os
import re
import sys

ROW = re.compile(r"\{\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*([-\d.]+)f\s*,\s*([-\d.]+)f\s*,\s*DIST_(UNIFORM|POWERLAW)\s*\}")


def main(ref_root):
    src = open(os.path.join(ref_root, "test/spmm/arch22/spmm_test.cpp"), encoding="utf-8").read()
    table = src[src.index("kTestCases[] = {"):]
    table = table[:table.index("};")]
    rows = [[m.group(1), m.group(2), m.group(3), m.group(4), m.group(5), m.group(6), m.group(7).lower()]
            for m in ROW.finditer(table)]
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "spmm_arch22_cases.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["m", "k", "n", "nnz", "alpha", "beta", "dist"])
        w.writerows(rows)
    print("%d cases" % len(rows))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
