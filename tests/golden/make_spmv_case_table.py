"""Writes tests/golden/spmv_arch22_cases.csv: the named cases of the reference's SpMV test program
(test/spmv/arch22/spmv_test.cpp:593-777, the RunAndTrack<...>(M, N, sparsity, alpha, beta, transpose, ..., "tag")
calls of its main), as data: tag, compute / value / output type, shape, sparsity, alpha, beta, transpose.

The reference file is read as text; nothing of it is run.  The random-parameter loops of the same main
(RunRandomParams, seeded from the clock) have no fixed cases to list and are covered by the seeded random tests.

    python tests/golden/make_spmv_case_table.py /root/reference
"""
import csv
import os
import re
import sys

TYPE = {"float": "f32", "half": "f16", "bfloat16_t": "bf16", "int32_t": "i32"}
CALL = re.compile(r'RunAndTrack<([^>]+)>\(\s*(\d+)\s*,\s*(\d+)\s*,\s*([-\d.]+)f?\s*,\s*([-\d.]+)f?\s*,\s*([-\d.]+)f?\s*,'
                  r'\s*(true|false)\s*,\s*stats\s*,\s*stream\s*,\s*"([^"]+)"\)')


def main(ref_root):
    src = open(os.path.join(ref_root, "test/spmv/arch22/spmv_test.cpp"), encoding="utf-8").read()
    rows = []
    for m in CALL.finditer(src):
        types = [TYPE[t.strip()] for t in m.group(1).split(",")]
        comp = types[0]
        val = types[1] if len(types) > 1 else comp
        out = types[2] if len(types) > 2 else comp
        rows.append([m.group(8), comp, val, out, m.group(2), m.group(3), m.group(4), m.group(5), m.group(6),
                     int(m.group(7) == "true")])
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "spmv_arch22_cases.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["tag", "compute", "value", "output", "rows", "cols", "sparsity", "alpha", "beta", "transpose"])
        w.writerows(rows)
    print("%d cases" % len(rows))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
