"""Writes tests/golden/spmm_arch22_cases.csv: the case table of the reference's arch22 SpMM test program
(kTestCases in test/spmm/arch22/spmm_test.cpp:446-), as data: M, K, N, nnz, alpha, beta, row distribution.

The reference file is read as text; nothing of it is run.

The program draws every column index from one thread_local std::mt19937(42) that is never re-seeded
(random_col, :42-51), so the matrix of a case depends on how many engine outputs the cases before it used.
That number is the last column, `engine_outputs_before`: found here by running this repository's restatement
of the generators (oracle.spmm22_csr) over the table in order, without storing anything.  A test can then put
the engine where the reference's is at the start of any case (oracle.spmm22_seek).

    python tests/golden/make_spmm_arch22_case_table.py /root/reference
"""
import csv
import os
import re
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import oracle  # noqa: E402

ROW = re.compile(r"\{\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*([-\d.]+)f\s*,\s*([-\d.]+)f\s*,\s*DIST_(UNIFORM|POWERLAW)\s*\}")


def main(ref_root):
    src = open(os.path.join(ref_root, "test/spmm/arch22/spmm_test.cpp"), encoding="utf-8").read()
    table = src[src.index("kTestCases[] = {"):]
    table = table[:table.index("};")]
    rows = [[m.group(1), m.group(2), m.group(3), m.group(4), m.group(5), m.group(6), m.group(7).lower()]
            for m in ROW.finditer(table)]
    oracle.spmm22_seek(0)
    for r in rows:
        r.append(str(oracle.spmm22_outputs_used()))
        m, k, n, nnz = (int(v) for v in r[:4])
        if m and k and n and nnz:  # run_spmm_test skips a case with a zero size before it generates anything (:391-394)
            oracle.spmm22_csr(r[6], m, k, nnz, store=False)
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "spmm_arch22_cases.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["m", "k", "n", "nnz", "alpha", "beta", "dist", "engine_outputs_before"])
        w.writerows(rows)
    print("%d cases" % len(rows))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
