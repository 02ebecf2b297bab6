"""The case table of the reference's arch22 SpMM test program, row by row, through the three-step aclsparseSpMM API.

tests/golden/spmm_arch22_cases.csv holds kTestCases of test/spmm/arch22/spmm_test.cpp:446- (M, K, N, nnz, alpha,
beta, row distribution: 200 rows from 16 x 16 to 65 536 x 65 536 with 16.7 M entries, and the number of engine
outputs the program has used when it reaches the row).  Every case is built by that program's own generators
(:42-131, :376-383), restated in oracle/ with their seeded engine, so the inputs are the reference's: `uniform` gives
every row nnz / M entries (the first nnz % M one more), `powerlaw` shares nnz out by Zipf weights 1 / (row + 1),
capped at K; distinct random columns in the order drawn (not sorted); values 0.1 + 0.0001 * position;
B[i] = 0.5 + 0.0001 * (i % 1000), C[i] = 0.01 * (i % 100), both compact row-major.  Judged by that program's rule (verify_result, :149-170, called with 1e-3 / 1e-3: an element fails
when it is off by more than 1e-3 absolutely AND relatively) against its fp32 golden (spmm_csr_cpu, :132-147), and by
this build's bar, 1e-5 per element against the fp64-accumulated oracle, on the leading rows (all of them unless the
case is large: the oracle is a CPU loop).
"""
import csv
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import run_spmm

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spmm_arch22_cases.csv")) as f:
    CASES = list(csv.DictReader(f))


def _matrix(c):
    """The matrix the reference's program builds for this row of its table: its generators restated in oracle/
    (generate_random_csr / generate_powerlaw_csr over random_col's engine), the engine put where the program's is
    when it reaches the case — cases that run in table order continue it, any other order seeks."""
    before = int(c["engine_outputs_before"])
    if oracle.spmm22_outputs_used() != before:
        oracle.spmm22_seek(before)
    return oracle.spmm22_csr(c["dist"], int(c["m"]), int(c["k"]), int(c["nnz"]))


def _rows_within(rowptr, n, budget, from_end=False):
    """How many leading (trailing) rows hold at most `budget` multiply-adds, at least one."""
    work = rowptr.astype(np.int64) * n
    if from_end:
        return max(1, int(rowptr.size - 1 - np.searchsorted(work, work[-1] - budget, side="left")))
    return max(1, int(np.searchsorted(work, budget, side="right")) - 1)


@pytest.mark.parametrize("c", CASES, ids=["%s-%sx%sx%s-nnz%s-a%s-b%s" % (c["dist"], c["m"], c["k"], c["n"], c["nnz"],
                                                                          c["alpha"], c["beta"]) for c in CASES])
def test_reference_arch22_case(osa, gpu_ctx, c):
    m, k, n, nnz = int(c["m"]), int(c["k"]), int(c["n"]), int(c["nnz"])
    alpha, beta = float(c["alpha"]), float(c["beta"])
    dev = gpu_ctx[0]
    rowptr, colind, val = _matrix(c)
    lengths = np.diff(rowptr)
    assert all(np.unique(colind[rowptr[r]:rowptr[r + 1]]).size == lengths[r] for r in (0, m // 2, m - 1))
    B = (np.float32(0.5) + np.float32(0.0001) * (np.arange(k * n) % 1000).astype(np.float32)).astype(np.float32)
    C0 = (np.float32(0.01) * (np.arange(m * n) % 100).astype(np.float32)).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, alpha, beta).reshape(m, n)

    # The oracles are CPU loops: a large case is checked on its leading and its trailing rows (power law: the long
    # rows and the short ones), 2^28 multiply-adds each for the fp32 golden and 2^26 for the fp64 oracle.
    def check(lo, rows, f64):
        ptr = rowptr[lo: lo + rows + 1]
        sub = (rows, n, ptr - ptr[0], colind[ptr[0]: ptr[-1]], val[ptr[0]: ptr[-1]], B, n,
               C0.reshape(m, n)[lo: lo + rows], n, alpha, beta)
        mine = got[lo: lo + rows]
        if f64:
            assert oracle.max_rel_err(mine.ravel(), np.asarray(oracle.spmm_f64_rowmajor(*sub)).ravel()) <= 1e-5
            return
        g32 = np.asarray(oracle.spmm_f32_threads(*sub, oracle.host_threads())).reshape(rows, n)
        diff = np.abs(mine - g32)
        bad = (diff > 1e-3) & (diff / np.maximum(np.abs(g32), 1e-6) > 1e-3)
        assert not bad.any(), "%d elements fail the reference's rule" % int(bad.sum())

    for budget, f64 in ((1 << 28, False), (1 << 26, True)):
        lead = min(m, _rows_within(rowptr, n, budget))
        check(0, lead, f64)
        if lead < m:
            tail = min(m, _rows_within(rowptr, n, budget, from_end=True))
            check(m - tail, tail, f64)
