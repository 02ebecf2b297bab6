"""Seeded random differential tests: the aclsparse entry points against the oracle on shapes nobody chose by hand.

Every seed draws a matrix (rows and columns from a few magnitudes incl. 1; row lengths all short, all equal, medium,
power-law with one long row, a dense stretch among empty rows, or mostly empty; unsorted columns with repeats),
alpha / beta from a set that contains 0 and 1, and one of: SpMV (either op(A), prepared or not, fp32 or fp16
values), SpMVOp (any algorithm, 32- / 64-bit offsets, base 0 / 1, Z aliasing Y, scalars on the host or the device),
SpMM in any storage order / op(B) with padded leading dimensions and widths that are not whole vectors, SpMM
fp16 -> fp32 and int8 -> int32.  Bars as everywhere else: 1e-5 against the fp64 oracle, the reference's rule for
op(A) = A^T (fp32 atomics), bit-exact for int8.  An earlier, longer run of the same generator is how the
per-workgroup summation of op(A) = A^T onto few columns came about.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import run_spmm, run_spmv
from test_spmv_op_gpu import run_op

pytestmark = pytest.mark.gpu


def _matrix(rng):
    rows, cols = int(rng.choice([1, 7, 300, 2049, 5000, 40000])), int(rng.choice([1, 9, 513, 4097, 30000]))
    kind = int(rng.integers(0, 6))
    if kind == 0:
        lengths = rng.integers(0, 9, rows)
    elif kind == 1:
        lengths = np.full(rows, rng.integers(1, 50))
    elif kind == 2:
        lengths = rng.integers(40, 200, rows)
    elif kind == 3:
        lengths = np.minimum((rng.pareto(1.1, rows) * 3).astype(np.int64), 5000)
        lengths[rng.integers(0, rows)] = rng.integers(300, 6000)
    elif kind == 4:
        lengths = np.zeros(rows, np.int64)
        a = int(rng.integers(0, rows))
        lengths[a:a + max(1, rows // 7)] = rng.integers(1, 70)
    else:
        lengths = rng.integers(0, 3, rows) * rng.integers(0, 30, rows)
    lengths = np.minimum(np.asarray(lengths, np.int64), 6000)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    return rows, cols, rowptr, colind, val


def _half(a):
    return torch.from_numpy(a).to(torch.float16).float().numpy()


@pytest.mark.parametrize("seed", range(80))
def test_random_case(osa, gpu_ctx, seed):
    rng = np.random.default_rng(9_000 + seed)
    rows, cols, rowptr, colind, val = _matrix(rng)
    alpha, beta = float(rng.choice([1.0, -0.5, 2.25, 0.0])), float(rng.choice([0.0, 1.0, 0.5, -1.5]))
    what = seed % 5
    if what < 2:                                                     # SpMV
        trans, prep, half = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 4) == 0)
        nin, nout = (rows, cols) if trans else (cols, rows)
        x, y0 = rng.uniform(-1, 1, nin).astype(np.float32), rng.uniform(-1, 1, nout).astype(np.float32)
        if half:
            val, x = _half(val), _half(x)
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, alpha, beta, preprocess=prep,
                     op=osa.ACL_SPARSE_OP_TRANSPOSE if trans else osa.ACL_SPARSE_OP_NON_TRANSPOSE,
                     val_dtype=torch.float16 if half else None, out_dtype=torch.float32 if half else None)
        if trans:
            gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
            d = np.abs(y - gold)
            assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2
        else:
            assert oracle.max_rel_err(y, oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)) <= 1e-5
    elif what == 2:                                                  # SpMVOp
        x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
        z = run_op(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, alpha, beta,
                   mode="DEVICE" if rng.integers(0, 3) == 0 else "HOST", i64=bool(rng.integers(0, 2)),
                   alias=bool(rng.integers(0, 2)), alg=int(rng.integers(0, 3)), base=int(rng.integers(0, 2)))
        assert oracle.max_rel_err(z, oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)) <= 1e-5
    elif what == 3:                                                  # SpMM, any layout
        n = int(rng.choice([1, 3, 8, 17, 32, 64, 100]))
        if max(rows, cols) * n > 3_000_000:
            n = min(n, 8)
        b_rm, c_rm, trans_b = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 3) == 0)
        eff_col = (not b_rm) != trans_b                              # which index of B is contiguous
        ldb = max(cols if eff_col else n, n if b_rm else cols) + int(rng.integers(0, 5))
        ldc = (n + int(rng.integers(0, 9))) if c_rm else (rows + int(rng.integers(0, 5)))
        B = rng.uniform(-1, 1, (n if eff_col else cols) * ldb + 8).astype(np.float32)
        C0 = rng.uniform(-1, 1, (rows if c_rm else n) * ldc).astype(np.float32)
        got = run_spmm(osa, gpu_ctx, rows, cols, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta,
                       order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                       order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                       op_b=osa.ACL_SPARSE_OP_TRANSPOSE if trans_b else osa.ACL_SPARSE_OP_NON_TRANSPOSE)
        gold = oracle.spmm_f64(rows, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, b_row_major=b_rm,
                               trans_b=trans_b, c_row_major=c_rm)
        assert oracle.max_rel_err(got, gold) <= 1e-5
    else:                                                            # SpMM, other types
        n = int(rng.choice([1, 5, 8, 16, 24, 40, 64, 128]))
        if max(rows, cols) * n > 3_000_000:
            n = min(n, 8)
        ldb, ldc = n + int(rng.choice([0, 0, 3, 8])), n + int(rng.choice([0, 0, 5, 16]))
        if rng.integers(0, 2):
            v8 = rng.integers(-128, 128, colind.size).astype(np.int8)
            B = rng.integers(-128, 128, cols * ldb).astype(np.int8)
            C0 = rng.integers(-1000, 1000, rows * ldc).astype(np.int32)
            ai, bi = int(rng.choice([1, 3, -2, 70000])), int(rng.choice([0, 1, -2]))
            got = run_spmm(osa, gpu_ctx, rows, cols, n, rowptr, colind, v8, B, ldb, C0, ldc, ai, bi,
                           val_dtype=torch.int8, c_dtype=torch.int32, compute_type=osa.ACL_INT32)
            assert np.array_equal(got, oracle.spmm_i8(rows, n, rowptr, colind, v8, B, ldb, C0, ldc, ai, bi,
                                                      saturate=True))
        else:
            vh, B = _half(val), _half(rng.uniform(-1, 1, cols * ldb).astype(np.float32))
            C0 = rng.uniform(-1, 1, rows * ldc).astype(np.float32)
            got = run_spmm(osa, gpu_ctx, rows, cols, n, rowptr, colind, vh, B, ldb, C0, ldc, alpha, beta,
                           val_dtype=torch.float16, c_dtype=torch.float32)
            gold = oracle.spmm_f64(rows, n, rowptr, colind, vh, B, ldb, C0, ldc, alpha, beta, b_row_major=True,
                                   trans_b=False, c_row_major=True)
            assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("seed", range(60))
def test_random_few_columns_case(osa, gpu_ctx, seed):
    """SpMM with 1 - 16 columns of B on the same random matrices (those without a row beyond 200 entries take the
    kernel for narrow B, one or two column-major columns the SpMV kernels; the others the lane-group kernels): any
    storage order, padded leading dimensions, fp32 or fp16 values with fp32 C."""
    rng = np.random.default_rng(77_000 + seed)
    rows, cols, rowptr, colind, val = _matrix(rng)
    alpha, beta = float(rng.choice([1.0, -0.5, 2.25])), float(rng.choice([0.0, 1.0, -1.5]))
    n = int(rng.integers(1, 17))
    half = bool(rng.integers(0, 3) == 0)
    b_rm, c_rm = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    pad = int(rng.choice([0, 0, 1, 4]))
    ldb = (n if b_rm else cols) + pad
    ldc = (n if c_rm else rows) + pad
    B = rng.uniform(-1, 1, (cols if b_rm else n) * ldb).astype(np.float32)
    C0 = rng.uniform(-1, 1, (rows if c_rm else n) * ldc).astype(np.float32)
    if half:
        val, B = _half(val), _half(B)
    got = run_spmm(osa, gpu_ctx, rows, cols, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta,
                   order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                   order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                   val_dtype=torch.float16 if half else None, c_dtype=torch.float32 if half else None)
    gold = oracle.spmm_f64(rows, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, b_row_major=b_rm,
                           trans_b=False, c_row_major=c_rm)
    assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("seed", range(30))
def test_random_conversion_case(osa, gpu_ctx, seed):
    """The CSR producers on the same random matrices (columns unsorted, with repeats): csrsort, the same arrays read
    as a CSC matrix through cscsort, the COO triples in a shuffled order through coosort by row and by column, and
    csr2csc; every output bit for bit against the oracle."""
    from test_convert_gpu import run_coosort, run_cscsort, run_csr2csc, run_csrsort
    rng = np.random.default_rng(19_000 + seed)
    rows, cols, rowptr, colind, val = _matrix(rng)
    base = int(rng.integers(0, 2))
    perm = rng.integers(-10 ** 6, 10 ** 6, colind.size).astype(np.int32) if seed % 2 else None
    run_csrsort(osa, gpu_ctx, rows, cols, rowptr + base, colind + base, base=base, perm=perm)
    run_cscsort(osa, gpu_ctx, cols, rows, rowptr + base, colind + base, base=base, perm=perm)
    order = rng.permutation(colind.size)
    coo_rows = oracle.csr2coo(rowptr, colind.size)[order]
    run_coosort(osa, gpu_ctx, rows, cols, coo_rows, colind[order], bool(seed % 2), perm=perm)
    run_coosort(osa, gpu_ctx, rows, cols, coo_rows - 3, colind[order] - 40_000, not bool(seed % 2))
    run_csr2csc(osa, gpu_ctx, rows, cols, rowptr + base, colind + base, val, np.float32, True, base)
