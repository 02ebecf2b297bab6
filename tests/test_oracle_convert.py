"""Pins the CPU oracles of the CSR producers (oracle.coo2csr / csr2coo / csrsort / cscsort / coosort / csr2csc):
against the reference's own goldens compiled in place (oracle/_ref/libref_convert.so,
skipped where that is not built), against numpy / scipy formulations of the same
definitions, and against hand-written small cases.  Everything is bit-exact."""
import ctypes

import numpy as np
import pytest
import scipy.sparse as sp

import oracle
from helpers import random_csr


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


CASES = [(1, 1, 1.0, 0), (4, 4, 0.5, 1), (37, 11, 0.3, 0), (200, 300, 0.05, 1), (64, 64, 0.0, 0), (500, 7, 0.9, 1),
         (1, 5000, 0.4, 0), (3000, 1, 0.5, 1)]


def _csr(m, n, density, seed, base, **kw):
    rowptr, colind, val = random_csr(m, n, density, seed, **kw)
    return rowptr + base, colind + base, val


def test_hand_cases():
    assert oracle.coo2csr([0, 0, 2, 2, 2, 3], 5).tolist() == [0, 2, 2, 5, 6, 6]
    assert oracle.coo2csr([1, 1, 3, 3, 3, 4], 5, base=1).tolist() == [1, 3, 3, 6, 7, 7]
    assert oracle.coo2csr([], 3, base=1).tolist() == [1, 1, 1, 1]
    assert oracle.coo2csr([7, -1, 1], 3).tolist() == [0, 0, 1, 1]          # rows outside [0, m) are not counted
    assert oracle.csr2coo([0, 2, 2, 5], 5).tolist() == [0, 0, 2, 2, 2]
    assert oracle.csr2coo([1, 3, 3, 6], 5, base=1).tolist() == [1, 1, 3, 3, 3]
    c, p = oracle.csrsort([0, 4, 4, 6], [3, 1, 3, 0, 9, 2], [10, 11, 12, 13, 14, 15])
    assert c.tolist() == [0, 1, 3, 3, 2, 9] and p.tolist() == [13, 11, 10, 12, 15, 14]   # equal keys keep their order
    colptr, rowind, val = oracle.csr2csc(3, 3, [0, 2, 3, 5], [0, 2, 2, 0, 1], np.array([1, 2, 3, 4, 5], np.float32))
    assert colptr.tolist() == [0, 2, 3, 5] and rowind.tolist() == [0, 2, 2, 0, 1] and val.tolist() == [1, 4, 5, 2, 3]


@pytest.mark.parametrize("m,n,density,base", CASES)
def test_against_numpy_and_scipy(m, n, density, base):
    rowptr, colind, val = _csr(m, n, density, m * 7 + n, base, empty_row_prob=0.2, unsorted=True)
    nnz = colind.size
    rows0 = np.repeat(np.arange(m, dtype=np.int32), np.diff(rowptr))
    assert np.array_equal(oracle.csr2coo(rowptr, nnz, base), rows0 + base)
    assert np.array_equal(oracle.coo2csr(rows0 + base, m, base), rowptr)
    # per-row stable sort == stable argsort of (row, col)
    perm0 = np.arange(nnz, dtype=np.int32)[::-1].copy()
    order = np.lexsort((colind, rows0))                      # lexsort is stable; primary key rows0
    c, p = oracle.csrsort(rowptr, colind, perm0, base)
    assert np.array_equal(c, colind[order]) and np.array_equal(p, perm0[order])
    # CSR -> CSC == stable sort by column; scipy agrees on the structure
    by_col = np.argsort(colind, kind="stable")
    colptr, rowind, cval = oracle.csr2csc(m, n, rowptr, colind, val, base)
    assert np.array_equal(rowind, rows0[by_col] + base) and np.array_equal(cval, val[by_col])
    assert np.array_equal(colptr, np.concatenate([[0], np.cumsum(np.bincount(colind - base, minlength=n))]) + base)
    if nnz:
        A = sp.csr_matrix((np.arange(1, nnz + 1, dtype=np.float64), colind - base, rowptr - base), shape=(m, n)).tocsc()
        assert np.array_equal(A.indptr + base, colptr)
    for dt in (np.int8, np.float16):                          # values move as raw bytes, any width
        v = (np.arange(nnz) % 100).astype(dt)
        assert np.array_equal(oracle.csr2csc(m, n, rowptr, colind, v, base)[2], v[by_col])
    assert oracle.csr2csc(m, n, rowptr, colind, None, base)[2] is None


@pytest.mark.parametrize("m,n,density,base", CASES)
def test_against_reference_goldens(m, n, density, base):
    R = oracle.ref_convert()
    if R is None:
        pytest.skip("oracle/_ref/libref_convert.so not built (needs the reference tree)")
    rowptr, colind, val = _csr(m, n, density, m * 13 + n, base, empty_row_prob=0.3, unsorted=True, duplicates=True)
    nnz = colind.size
    i32 = ctypes.c_int32
    rows = oracle.csr2coo(rowptr, nnz, base)
    got = np.zeros(nnz, np.int32)
    R.ref_csr2coo(_p(rowptr), ctypes.c_int64(m), ctypes.c_int64(nnz), i32(base), _p(got))
    assert np.array_equal(got, rows)
    got = np.zeros(m + 1, np.int32)
    R.ref_coo2csr(_p(rows), i32(nnz), i32(m), i32(base), _p(got))
    assert np.array_equal(got, oracle.coo2csr(rows, m, base)) and np.array_equal(got, rowptr)
    c, p = colind.copy(), np.arange(nnz, dtype=np.int32) * 3
    R.ref_csrsort(_p(rowptr), i32(m), i32(nnz), i32(base), _p(c), _p(p))
    oc, op = oracle.csrsort(rowptr, colind, np.arange(nnz, dtype=np.int32) * 3, base)
    assert np.array_equal(c, oc) and np.array_equal(p, op)
    colptr, rowind, cval = np.zeros(n + 1, np.int32), np.zeros(nnz, np.int32), np.zeros(nnz, np.float32)
    R.ref_csr2csc(i32(m), i32(n), i32(nnz), i32(base), _p(rowptr), _p(colind), _p(val), _p(colptr), _p(rowind), _p(cval))
    ocp, ori, ocv = oracle.csr2csc(m, n, rowptr, colind, val, base)
    assert np.array_equal(colptr, ocp) and np.array_equal(rowind, ori) and np.array_equal(cval.view(np.uint32),
                                                                                             ocv.view(np.uint32))


def test_round_trips():
    """csr2coo . coo2csr = identity; CSR -> CSC twice = sorted CSR."""
    m, n = 300, 200
    rowptr, colind, val = random_csr(m, n, 0.05, 3, unsorted=True)
    assert np.array_equal(oracle.coo2csr(oracle.csr2coo(rowptr, colind.size), m), rowptr)
    colptr, rowind, cval = oracle.csr2csc(m, n, rowptr, colind, val)
    rp2, ci2, v2 = oracle.csr2csc(n, m, colptr, rowind, cval)
    sc, sperm = oracle.csrsort(rowptr, colind, np.arange(colind.size, dtype=np.int32))
    assert np.array_equal(rp2, rowptr) and np.array_equal(ci2, sc) and np.array_equal(v2, val[sperm])


# ------------------------------------------------------- cscsort / coosort

def _coo(nnz, lo, hi, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi, nnz).astype(np.int32), rng.integers(lo, hi, nnz).astype(np.int32)


def test_sort_hand_cases():
    # ByRowBasic / ByColumnBasic of test/coosort/arch35/coosort_test.cpp:233-249
    rows, cols = [2, 0, 3, 0, 1, 2], [1, 3, 2, 1, 0, 3]
    r, c, p = oracle.coosort(rows, cols, np.arange(6), True)
    assert (r.tolist(), c.tolist(), p.tolist()) == ([0, 0, 1, 2, 2, 3], [1, 3, 0, 1, 3, 2], [3, 1, 4, 0, 5, 2])
    r, c, p = oracle.coosort(rows, cols, np.arange(6), False)
    assert (r.tolist(), c.tolist(), p.tolist()) == ([1, 0, 2, 3, 0, 2], [0, 1, 1, 2, 3, 3], [4, 3, 0, 2, 1, 5])
    # equal (row, col) pairs keep their input order; P travels whatever it holds; negative indices sort first
    r, c, p = oracle.coosort([1, -2, 1, 1, -2], [5, 0, 5, -7, 0], [50, 40, 30, 20, 10], True)
    assert (r.tolist(), c.tolist(), p.tolist()) == ([-2, -2, 1, 1, 1], [0, 0, -7, 5, 5], [40, 10, 20, 50, 30])
    # a CSC matrix with columns of 3, 0 and 2 entries, base 1
    r, p = oracle.cscsort([1, 4, 4, 6], [3, 1, 3, 9, 2], [10, 11, 12, 13, 14], base=1)
    assert (r.tolist(), p.tolist()) == ([1, 3, 3, 2, 9], [11, 10, 12, 14, 13])


@pytest.mark.parametrize("nnz,lo,hi", [(0, 0, 5), (1, 0, 5), (12, 0, 4), (388, 0, 50), (5000, -300, 300),
                                        (20000, 0, 7), (3000, -2 ** 31, 2 ** 31 - 1)])
@pytest.mark.parametrize("by_row", [True, False])
def test_coosort_against_numpy_and_the_reference_golden(nnz, lo, hi, by_row):
    rows, cols = _coo(nnz, lo, hi, nnz + 7)
    perm0 = np.arange(nnz, dtype=np.int32)
    r, c, p = oracle.coosort(rows, cols, perm0, by_row)
    # numpy: lexsort is stable and takes the LAST key as the primary one
    order = np.lexsort((cols, rows) if by_row else (rows, cols)).astype(np.int32)
    assert np.array_equal(p, order) and np.array_equal(r, rows[order]) and np.array_equal(c, cols[order])
    # P travels with its entry whatever it holds
    other = (perm0 * 7 - 3).astype(np.int32)
    assert np.array_equal(oracle.coosort(rows, cols, other, by_row)[2], other[order])
    R = oracle.ref_convert()
    if R is not None and hasattr(R, "ref_coosort"):
        gr, gc, gp = np.zeros(nnz, np.int32), np.zeros(nnz, np.int32), np.zeros(nnz, np.int32)
        R.ref_coosort(_p(rows), _p(cols), ctypes.c_int32(nnz), ctypes.c_int32(1 if by_row else 0), _p(gr), _p(gc),
                      _p(gp))
        assert np.array_equal(gr, r) and np.array_equal(gc, c) and np.array_equal(gp, p)


@pytest.mark.parametrize("m,n,density,base", CASES)
def test_cscsort_against_csrsort_of_the_transpose_and_the_reference_golden(m, n, density, base):
    # a CSC matrix of m x n is stored exactly like a CSR matrix of n x m
    colptr, rowind, _ = _csr(n, m, density, m * 7 + n, base, empty_row_prob=0.3, unsorted=True, duplicates=True)
    nnz = rowind.size
    perm0 = (np.arange(nnz, dtype=np.int32) * 5 + 1).astype(np.int32)
    r, p = oracle.cscsort(colptr, rowind, perm0, base)
    for j in range(n):                                       # every column by numpy's stable sort
        a, b = colptr[j] - base, colptr[j + 1] - base
        order = np.argsort(rowind[a:b], kind="stable")
        assert np.array_equal(r[a:b], rowind[a:b][order]) and np.array_equal(p[a:b], perm0[a:b][order])
    R = oracle.ref_convert()
    if R is not None and hasattr(R, "ref_cscsort"):
        gr, gp = rowind.copy(), perm0.copy()
        R.ref_cscsort(_p(colptr), ctypes.c_int32(n), ctypes.c_int32(nnz), ctypes.c_int32(base), _p(gr), _p(gp))
        assert np.array_equal(gr, r) and np.array_equal(gp, p)
