"""Writes tests/golden/fill_generator.json: fingerprints of arrays produced by the
REFERENCE's own seeded generator (test/frame/fill.h, compiled into
oracle/_ref/libref_fill.so by oracle/Makefile).  Needs the reference tree, so it
runs where that tree is mounted; the JSON it writes is what travels.

    python tests/golden/make_fill_fixture.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402


def main():
    if oracle.ref_fill() is None:
        oracle.build()
    if oracle.ref_fill() is None:
        sys.exit("oracle/_ref/libref_fill.so could not be built (reference tree missing)")
    out = {"source": "SparseFillGenerator / makeDenseFloat of the reference's test/frame/fill.h via oracle/_ref",
           "csr": [], "dense": []}
    cases = [(42, 4096, 4096, 65536, -1.0, 1.0, 0.0),      # the reference-runnable SpMV configuration
             (7, 100, 50, 1000, -3.0, 3.0, 0.3),
             (1234, 333, 777, 333 * 9, -2.0, 2.0, 0.0),
             (5, 1, 1000, 999, -3.0, 3.0, 0.0)]
    # (nnz_hint <= 0: binomial row lengths at density 1 - sparsity, the path the SpMVOp case table takes)
    cases = [c + (0.9,) for c in cases] + [(42, 4, 4, -1, -5.0, 5.0, 0.0, 0.5), (61, 1024, 1024, -1, -5.0, 5.0, 0.0, 0.9),
                                           (77, 300, 5000, -1, -5.0, 5.0, 0.25, 0.99), (9, 2000, 64, -1, -5.0, 5.0, 0.1, 0.3)]
    for seed, rows, cols, hint, lo, hi, p, sparsity in cases:
        rowptr, colind, val = oracle.ref_fill_csr(seed, rows, cols, hint, sparsity=sparsity, empty_row_prob=p, lo=lo,
                                                  hi=hi)
        out["csr"].append({
            "seed": seed, "rows": rows, "cols": cols, "nnz_hint": hint, "sparsity": sparsity, "lo": lo, "hi": hi,
            "empty_row_prob": p,
            "nnz": int(colind.size), "rowptr_fnv1a": "%016x" % oracle.fnv1a(rowptr),
            "colind_fnv1a": "%016x" % oracle.fnv1a(colind), "values_fnv1a": "%016x" % oracle.fnv1a(val),
            "colind_head": colind[:4].tolist(), "values_head": [float(v) for v in val[:2]]})
    for seed, n, lo, hi in [(43, 4096, -1.0, 1.0), (44, 17, -3.0, 3.0)]:
        v = oracle.ref_fill_dense(seed, n, lo, hi)
        out["dense"].append({"seed": seed, "n": n, "lo": lo, "hi": hi, "fnv1a": "%016x" % oracle.fnv1a(v),
                             "head": [float(x) for x in v[:2]]})
    with open(os.path.join(HERE, "fill_generator.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote fill_generator.json")


if __name__ == "__main__":
    main()
