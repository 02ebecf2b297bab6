"""Bit-wise repeatable results where the reference promises them: ACL_SPARSE_SPMV_CSR_ALG2
(reference include/cann_ops_sparse.h:162-164) and every aclsparseSpMVOp algorithm (the same file, :57-69), on the
matrices that get the blocked-gather layout.

The data is chosen so that the ORDER of a row's additions shows in the result: the products are exact in fp64
(x is +-1, the values are powers of two), their exponents span ninety binades and the large ones cancel in pairs, so
(big + small) - big and (big - big) + small differ in most rows.  The tests first show that (the same matrix with
every row's entries stored in another order gives other bits in thousands of rows), then that the library's order
is fixed: the same plan run again and again, and a second plan built into a second buffer, give the same bits.
A sum taken with atomics in the order the wavefronts arrive fails this within a few runs."""
import ctypes
import math

import numpy as np
import pytest
import torch

from helpers import to_dev

pytestmark = pytest.mark.gpu

ROWS, COLS = 300_000, 1_400_000
RUNS = 6


@pytest.fixture(autouse=True)
def _layout_for_small_matrices(monkeypatch):
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.setenv("OPS_SPARSE_ORDERED_LIVE_MIN_COLS", "0")   # (the ordered live layout: from 2.6 M columns)


def _cancelling(seed):
    """Short scattered rows and long ones with ascending columns (summed panel by panel by another kernel); in every
    row of 4 entries and more, pairs of +-2^k with k in 40 .. 60 among entries of 2^-30 .. 2^0."""
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, 24, ROWS)
    long_rows = {3: 1500, 4: 1100, 70_000: 5000, 70_001: 9000, 150_000: 40_000, ROWS - 1: 4500}
    for r, n in long_rows.items():
        lengths[r] = n
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    nnz = int(rowptr[-1])
    colind = rng.integers(0, COLS, nnz).astype(np.int32)
    for r in long_rows:
        a, b = rowptr[r], rowptr[r + 1]
        colind[a:b] = np.sort(rng.choice(COLS, b - a, replace=False)).astype(np.int32)
    val = np.ldexp(1.0, rng.integers(-30, 1, nnz)).astype(np.float32) * rng.choice([-1.0, 1.0], nnz).astype(np.float32)
    # the cancelling pairs: two random places of a row get +2^k and -2^k
    for r in np.nonzero(lengths >= 4)[0]:
        a, n = int(rowptr[r]), int(lengths[r])
        pairs = max(1, n // 6)
        at = rng.choice(n, 2 * pairs, replace=False)
        k = np.ldexp(1.0, rng.integers(40, 61, pairs)).astype(np.float32)
        val[a + at[:pairs]] = k
        val[a + at[pairs:]] = -k
    x = rng.choice([-1.0, 1.0], COLS).astype(np.float32)
    # x = 1 at the pairs' columns would need unique columns; instead give the pair the sign that cancels with x
    val *= x[colind]                                          # now every product is the value drawn above
    y0 = rng.uniform(-1, 1, ROWS).astype(np.float32)
    return rowptr, colind, val, x, y0


def _rows_stored_backwards(rowptr, colind, val):
    """The same matrix with every SHORT row's entries in reverse order (long rows keep their ascending columns)."""
    ci, va = colind.copy(), val.copy()
    for r in np.nonzero(np.diff(rowptr) < 1000)[0]:
        a, b = rowptr[r], rowptr[r + 1]
        ci[a:b] = colind[a:b][::-1]
        va[a:b] = val[a:b][::-1]
    return ci, va


def _check_some_rows(y, rowptr, colind, val, x, rows_to_check):
    """Against the exactly rounded sum (math.fsum): whatever the order, fp64 partial sums stay within
    n * 2^-53 * sum |terms| of it."""
    for r in rows_to_check:
        a, b = int(rowptr[r]), int(rowptr[r + 1])
        terms = val[a:b].astype(np.float64) * x[colind[a:b]].astype(np.float64)
        exact = math.fsum(terms)
        slack = (b - a + 2) * 2.0 ** -52 * float(np.abs(terms).sum()) + abs(exact) * 2.0 ** -23
        assert abs(float(y[r]) - exact) <= slack, (r, float(y[r]), exact)


CASES = ["spmv_alg2", "spmv_alg2_transposed", "spmv_default_repeatable", "spmv_default_transposed",
         "spmvop_default", "spmvop_alg1", "spmvop_alg2"]


@pytest.mark.parametrize("case", CASES)
def test_same_bits_from_every_run_and_every_plan(osa, gpu_ctx, case, monkeypatch):
    dev, stream, handle = gpu_ctx
    rowptr, colind, val, x, y0 = _cancelling(101)
    transposed = case.endswith("transposed")
    if transposed:
        # op(A) = A^T of the CSC view: the matrix handed over is the transpose, so that the product is the same
        import scipy.sparse as sp
        m = sp.csr_matrix((val, colind, rowptr), shape=(ROWS, COLS))
        m.sort_indices()                                      # (csc of the sorted matrix: rows ascending per column)
        t = m.tocsc()
        h_rp, h_ci, h_va = t.indptr.astype(np.int32), t.indices.astype(np.int32), t.data.astype(np.float32)
        a_rows, a_cols = COLS, ROWS
        rowptr_n, colind_n, val_n = m.indptr.astype(np.int32), m.indices.astype(np.int32), m.data.astype(np.float32)
    else:
        h_rp, h_ci, h_va = rowptr, colind, val
        a_rows, a_cols = ROWS, COLS
        rowptr_n, colind_n, val_n = rowptr, colind, val
    if case == "spmv_default_repeatable":
        monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")

    def product(h_colind, h_values, alpha, beta, runs):
        """`runs` results of one plan on fresh device copies of the arrays."""
        d = [to_dev(a, dev) for a in (h_rp, h_colind, h_values, x)]
        A = osa.Csr(a_rows, a_cols, d[0], d[1], d[2])
        d_y = to_dev(y0, dev)
        if case.startswith("spmvop"):
            alg = {"spmvop_default": osa.ACL_SPARSE_SPMVOP_ALG_DEFAULT, "spmvop_alg1": osa.ACL_SPARSE_SPMVOP_ALG1,
                   "spmvop_alg2": osa.ACL_SPARSE_SPMVOP_ALG2}[case]
            Y = osa.DnVec(d_y)
            op = osa.SpmvOpPlan(handle, A, osa.DnVec(d[3]), Y, Y, alg=alg)
            assert op.buffer_bytes > 0                        # a re-stored layout, not the row-wise kernels
        else:
            alg = osa.ACL_SPARSE_SPMV_CSR_ALG2 if "alg2" in case else osa.ACL_SPARSE_SPMV_ALG_DEFAULT
            op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y),
                            op=osa.ACL_SPARSE_OP_TRANSPOSE if transposed else osa.ACL_SPARSE_OP_NON_TRANSPOSE, alg=alg)
            assert op.buffer.numel() > osa.lib().opsparse_spmv_csr_workspace_bytes(a_rows, h_colind.size)
        out = []
        for _ in range(runs):
            d_y.copy_(torch.from_numpy(y0))
            op(alpha, beta)
            stream.synchronize()
            out.append(d_y.clone())
        return out

    first = product(h_ci, h_va, 1.0, 0.0, RUNS)
    for y in first[1:]:
        assert torch.equal(y, first[0])
    second = product(h_ci, h_va, 1.0, 0.0, 2)                # another buffer, another analysis
    assert torch.equal(second[0], first[0]) and torch.equal(second[1], first[0])
    y = first[0].cpu().numpy()
    check_rows = [3, 4, 5, 6, 70_000, 70_001, 150_000, ROWS - 1] + list(range(1000, 1040))
    _check_some_rows(y, rowptr_n, colind_n, val_n, x, check_rows)
    with_beta = product(h_ci, h_va, -1.5, 0.75, 3)
    assert torch.equal(with_beta[1], with_beta[0]) and torch.equal(with_beta[2], with_beta[0])
    if not transposed:
        # the order matters on this data: the rows stored backwards give other bits in many rows, within the bound
        ci_b, va_b = _rows_stored_backwards(h_rp, h_ci, h_va)
        other = product(ci_b, va_b, 1.0, 0.0, 2)
        assert torch.equal(other[0], other[1])
        differing = int((other[0] != first[0]).sum())
        assert differing > 1000, differing
