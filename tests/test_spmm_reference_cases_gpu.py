"""The case table of the reference's arch22 SpMM test program, row by row, through the three-step aclsparseSpMM API.

tests/golden/spmm_arch22_cases.csv holds kTestCases of test/spmm/arch22/spmm_test.cpp:446- (M, K, N, nnz, alpha,
beta, row distribution: 200 rows from 16 x 16 to 65 536 x 65 536 with 16.7 M entries).  Every case is built the way
that program builds it (:42-131, :376-383): `uniform` gives every row nnz / M entries (the first nnz % M one more),
`powerlaw` shares nnz out by Zipf weights 1 / (row + 1), capped at K; distinct random columns in the order drawn
(not sorted); values 0.1 + 0.0001 * position; B[i] = 0.5 + 0.0001 * (i % 1000), C[i] = 0.01 * (i % 100), both
compact row-major.  Judged by that program's rule (verify_result, :149-170, called with 1e-3 / 1e-3: an element fails
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


def _matrix(m, k, nnz, dist, dev, seed):
    """Row lengths by the reference's two recipes; distinct uniformly random columns per row in the order drawn.
    Drawn with torch on `dev` (the largest case has 16.7 M entries): every entry gets a random column, entries that
    repeat an earlier column of their row are drawn again until none is left; rows that fill more than a sixteenth
    of the columns take the head of a random permutation instead."""
    if dist == "uniform":
        lengths = np.full(m, nnz // m, np.int64)
        lengths[: nnz % m] += 1
    else:
        weight = 1.0 / np.arange(1, m + 1, dtype=np.float64)
        lengths = (nnz * weight / weight.sum()).astype(np.int64)
        lengths[: max(0, min(m, nnz - int(lengths.sum())))] += 1
    lengths = np.minimum(lengths, k)
    rowptr = np.concatenate([[0], np.cumsum(lengths)])
    total = int(rowptr[-1])
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    row_of = torch.repeat_interleave(torch.arange(m, device=dev), torch.from_numpy(lengths).to(dev))
    col = torch.randint(0, k, (total,), generator=gen, device=dev)
    crowded = 16 * lengths > k
    for r in np.nonzero(crowded)[0]:
        col[rowptr[r]:rowptr[r + 1]] = torch.randperm(k, generator=gen, device=dev)[: int(lengths[r])]
    redraw = ~torch.from_numpy(crowded).to(dev)[row_of]
    while True:
        keys, order = torch.sort(row_of * k + col, stable=True)
        later = torch.zeros(total, dtype=torch.bool, device=dev)
        later[1:] = keys[1:] == keys[:-1]
        again = order[later]
        again = again[redraw[again]]
        if again.numel() == 0:
            break
        col[again] = torch.randint(0, k, (again.numel(),), generator=gen, device=dev)
    colind = col.to(torch.int32).cpu().numpy()
    val = np.float32(0.1) + np.float32(0.0001) * np.arange(total, dtype=np.float32)
    return rowptr.astype(np.int32), colind, val


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
    rowptr, colind, val = _matrix(m, k, nnz, c["dist"], dev, m * 7 + k * 3 + n + nnz)
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
