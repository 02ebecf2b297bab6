"""GPU parity of the remaining aclsparseSpMV operand modes: element types, op(A) = A^T,
device pointer mode.

Tolerances: outputs in fp16 / bf16 are compared after rounding the oracle to the
output type, allowing one unit in the last place of that type (2^-10 / 2^-7
relative) — the reference's own bars are 2^-9 and 2^-6 (spmv_test.cpp:212-215);
int32 is exact; the transposed product adds in fp32 with hardware atomics in
unspecified order, like the reference, and is held to the reference's fp32 rule
(|d| <= 2^-16 + 2^-10 |g| on >= 99 %, max |d| <= 1e-2)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import random_csr, run_spmv, to_dev

pytestmark = pytest.mark.gpu


def _problem(rows, cols, density, seed, lo=-2.0, hi=2.0):
    rowptr, colind, val = random_csr(rows, cols, density, seed, lo=lo, hi=hi, empty_row_prob=0.05)
    rng = np.random.default_rng(seed + 1)
    return rowptr, colind, val, rng.uniform(lo, hi, cols).astype(np.float32), rng.uniform(lo, hi, rows).astype(
        np.float32)


def _round(a, dtype):
    return torch.from_numpy(a).to(dtype).float().numpy()


@pytest.mark.parametrize("val_dtype,out_dtype,ulp", [(torch.float16, torch.float32, None),
                                                     (torch.float16, torch.float16, 2.0 ** -10),
                                                     (torch.bfloat16, torch.float32, None),
                                                     (torch.bfloat16, torch.bfloat16, 2.0 ** -7)])
@pytest.mark.parametrize("shape", [(600, 400, 0.02), (50, 3000, 0.3), (5000, 5000, 0.001)])
def test_half_precision_inputs(osa, gpu_ctx, val_dtype, out_dtype, ulp, shape):
    rows, cols, density = shape
    rowptr, colind, val, x, y0 = _problem(rows, cols, density, 31)
    val, x = _round(val, val_dtype), _round(x, val_dtype)          # the values the device really sees
    y0 = _round(y0, out_dtype)
    for pre in (True, False):
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5, preprocess=pre,
                     val_dtype=val_dtype, out_dtype=out_dtype)
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5)
        if ulp is None:
            assert oracle.max_rel_err(y, gold) <= 1e-5            # fp32 output: same bar as the fp32 path
        else:
            want = _round(gold, out_dtype)
            assert np.all(np.abs(y - want) <= ulp * np.maximum(np.abs(want), 2.0 ** -14))


def test_int32_exact(osa, gpu_ctx):
    rows, cols = 700, 900
    rowptr, colind, _ = random_csr(rows, cols, 0.03, 5)
    rng = np.random.default_rng(6)
    val = rng.integers(-50000, 50000, colind.size).astype(np.int32)
    x = rng.integers(-50000, 50000, cols).astype(np.int32)
    y0 = rng.integers(-1000, 1000, rows).astype(np.int32)
    for pre in (True, False):
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 3, -2, preprocess=pre,
                     compute_type=osa.ACL_INT32)
        assert np.array_equal(y, oracle.spmv_i32(rows, rowptr, colind, val, x, y0, 3, -2))   # wrap-around included


def test_int32_values_float_output(osa, gpu_ctx):
    rows, cols = 300, 300
    rowptr, colind, _ = random_csr(rows, cols, 0.05, 8)
    rng = np.random.default_rng(9)
    val = rng.integers(-1000, 1000, colind.size).astype(np.int32)
    x = rng.integers(-1000, 1000, cols).astype(np.int32)
    y0 = rng.uniform(-1, 1, rows).astype(np.float32)
    y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 0.5, 1.0)
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val.astype(np.float32), x.astype(np.float32), y0, 0.5, 1.0)
    assert oracle.max_rel_err(y, gold) <= 1e-5


@pytest.mark.parametrize("rows,cols,density", [(500, 300, 0.05), (64, 5000, 0.1), (3000, 40, 0.3), (1, 1, 1.0)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (2.0, 0.5), (1.0, 1.0), (0.0, 3.0)])
def test_transpose(osa, gpu_ctx, rows, cols, density, alpha, beta):
    rowptr, colind, val = random_csr(rows, cols, density, rows + cols)
    rng = np.random.default_rng(4)
    x = rng.uniform(-2, 2, rows).astype(np.float32)
    y0 = rng.uniform(-2, 2, cols).astype(np.float32)
    y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, alpha, beta,
                 op=osa.ACL_SPARSE_OP_TRANSPOSE)
    gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
    d = np.abs(y - gold)
    assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2
    g32 = oracle.spmv_trans_f32(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
    assert np.abs(y - g32).max() <= 1e-2


@pytest.mark.parametrize("val_dtype", [None, torch.float16])
def test_transpose_skewed_rows_split_by_entries(osa, gpu_ctx, val_dtype):
    """op(A) = A^T on rows of very different lengths after Preprocess: the work is cut into tiles of 2048 entries
    (a row of 60 000 entries is shared by thirty workgroups), the rows of a tile found through their offsets in
    LDS; long runs of empty rows in between make one tile span more rows than LDS holds.  The reference's fp32
    rule for the transposed product (atomics in unspecified order)."""
    rng = np.random.default_rng(31)
    lengths = rng.integers(0, 6, 40_000)
    lengths[5_000:12_000] = 0                       # thousands of empty rows inside one tile
    lengths[[3, 20_000, 39_999]] = [60_000, 9_000, 25_000]
    rows, cols = lengths.size, 70_000
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = np.concatenate([np.sort(rng.choice(cols, int(l), replace=False)) for l in lengths]).astype(np.int32)
    rt = (lambda a: a) if val_dtype is None else (lambda a: torch.from_numpy(a).to(val_dtype).float().numpy())
    val = rt(rng.uniform(-1, 1, colind.size).astype(np.float32))
    x, y0 = rt(rng.uniform(-1, 1, rows).astype(np.float32)), rng.uniform(-1, 1, cols).astype(np.float32)
    y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5, op=osa.ACL_SPARSE_OP_TRANSPOSE,
                 val_dtype=val_dtype, out_dtype=torch.float32 if val_dtype is not None else None)
    gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5)
    d = np.abs(y - gold)
    assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2


def test_device_pointer_mode(osa, gpu_ctx):
    """alpha / beta read by the kernel from device memory; changing them needs no new Preprocess."""
    dev, stream, handle = gpu_ctx
    rows, cols = 2000, 1500
    rowptr, colind, val, x, y0 = _problem(rows, cols, 0.01, 77)
    d_rowptr, d_colind, d_val = to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev)
    d_x = to_dev(x, dev)
    A = osa.Csr(rows, cols, d_rowptr, d_colind, d_val)
    scal = torch.tensor([1.25, -0.75], dtype=torch.float32, device=dev)
    L = osa.lib()
    handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_DEVICE)
    try:
        for buffered in (True, False):
            d_y = to_dev(y0, dev)
            X, Y = osa.DnVec(d_x), osa.DnVec(d_y)
            op = osa.SpmvOp(handle, A, X, Y, preprocess=buffered)
            buf = ctypes.c_void_p(op.buffer.data_ptr()) if buffered else None
            for a, b in ((1.25, -0.75), (-2.0, 0.5)):
                scal.copy_(torch.tensor([a, b]))
                d_y.copy_(torch.from_numpy(y0))
                torch.cuda.synchronize()
                rc = L.aclsparseSpMV(handle.h, 0, ctypes.c_void_p(scal.data_ptr()), A.d, X.d,
                                     ctypes.c_void_p(scal.data_ptr() + 4), Y.d, osa.ACL_FLOAT, 0, buf)
                assert rc == 0
                stream.synchronize()
                gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, a, b)
                assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    finally:
        handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_HOST)


def test_preprocessed_buffer_reused_and_rebound(osa, gpu_ctx):
    """Same buffer for many calls and new values behind the same pattern; a foreign buffer is not trusted."""
    dev, stream, handle = gpu_ctx
    rows, cols = 4000, 4000
    rowptr, colind, val, x, y0 = _problem(rows, cols, 0.002, 90)
    d_val = to_dev(val, dev)
    A = osa.Csr(rows, cols, to_dev(rowptr, dev), to_dev(colind, dev), d_val)
    d_y = to_dev(y0, dev)
    X, Y = osa.DnVec(to_dev(x, dev)), osa.DnVec(d_y)
    op = osa.SpmvOp(handle, A, X, Y)
    for scale in (1.0, 3.0):
        d_val.copy_(torch.from_numpy(val * scale))             # aclsparseSpMatSetValues-style update in place
        d_y.copy_(torch.from_numpy(y0))
        torch.cuda.synchronize()
        op(1.0, 1.0)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, (val * scale).astype(np.float32), x, y0, 1.0, 1.0)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    other = torch.zeros(op.buffer.numel(), dtype=torch.uint8, device=dev)   # never preprocessed
    d_y.copy_(torch.from_numpy(y0))
    torch.cuda.synchronize()
    rc = osa.lib().aclsparseSpMV(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, 0,
                                 ctypes.c_void_p(other.data_ptr()))
    assert rc == 0
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, (val * 3.0).astype(np.float32), x, y0, 1.0, 0.0)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def _wide_problem(rows, cols, seed, long_rows=(), per_row=12):
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, per_row, rows)
    for r, l in long_rows:
        lengths[r] = l
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = np.concatenate([np.sort(rng.choice(cols, int(l), replace=False)) for l in lengths] +
                            [np.zeros(0, np.int64)]).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    return rowptr, colind, val, rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)


@pytest.mark.parametrize("cols,panels", [(3_000_000, 3), (1_048_577, 2), (9_000_000, 9), (1_000_000, 0), (17_000_000, 0)])
def test_column_panels_csr_alg2(osa, gpu_ctx, cols, panels, monkeypatch):
    """ACL_SPARSE_SPMV_CSR_ALG2 with the blocked-gather layout switched off: Preprocess re-stores the matrix as
    panels of 2^20 columns (x wider than an L2); matrices with fewer than 2 or more than 16 panels silently take
    the ordinary families.  Same 1e-5 bar, and bit-equal from run to run (partials are added in panel order)."""
    monkeypatch.setenv("OPS_SPARSE_SPMV_NO_BLOCKED", "1")
    dev, stream, handle = gpu_ctx
    rows = 60_000
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, cols % 1000, long_rows=((7, 90_000), (59_999, 30_000)))
    L = osa.lib()
    assert (L.opsparse_spmv_csr_panels_workspace_bytes(rows, cols, colind.size) > 0) == (panels > 0)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y), alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    assert op.buffer.numel() >= L.opsparse_spmv_csr_panels_workspace_bytes(rows, cols, colind.size)
    outs = []
    for alpha, beta in ((1.0, 0.0), (-2.0, 0.75), (-2.0, 0.75)):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        outs.append(d_y.cpu().numpy())
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
        assert oracle.max_rel_err(outs[-1], gold) <= 1e-5
    assert np.array_equal(outs[1], outs[2])
    assert np.array_equal(d[1].cpu().numpy(), colind) and np.array_equal(d[2].cpu().numpy(), val)


def test_column_panels_through_spmvop_alg2(osa, gpu_ctx, monkeypatch):
    """aclsparseSpMVOp ALG2 on a wide matrix (blocked gather switched off) uses the panel layout; Z separate from Y
    and aliased."""
    monkeypatch.setenv("OPS_SPARSE_SPMV_NO_BLOCKED", "1")
    dev, stream, handle = gpu_ctx
    rows, cols = 40_000, 2_500_000
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, 5, long_rows=((3, 50_000),))
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    for alias in (False, True):
        d_y = to_dev(y0, dev)
        d_z = d_y if alias else torch.zeros(rows, dtype=torch.float32, device=dev)
        Y = osa.DnVec(d_y)
        Z = Y if alias else osa.DnVec(d_z)
        op = osa.SpmvOpPlan(handle, A, osa.DnVec(d[3]), Y, Z, alg=osa.ACL_SPARSE_SPMVOP_ALG2)
        assert op.buffer_bytes == osa.lib().opsparse_spmv_csr_panels_workspace_bytes(rows, cols, colind.size) > 0
        op(1.25, -0.5)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.25, -0.5)
        assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5
        op.close()


@pytest.mark.parametrize("rows,cols,applies", [(60_000, 3_000_000, True), (60_000, 1_048_577, True),
                                               (60_000, 9_000_000, True), (60_000, 1_000_000, True), (60_000, 262_144, False),
                                               (20_000, 17_000_000, True),      # 519 panels: chunks of 24 entries
                                               (300_000, 2_000_000, True)])
def test_blocked_gather_csr_alg2(osa, gpu_ctx, rows, cols, applies):
    """ACL_SPARSE_SPMV_CSR_ALG2 on a matrix whose x is wider than an L2: Preprocess re-stores the entries by
    panels of 2^15 columns and row blocks, SpMV gathers x from LDS in one pass and sums row blocks in LDS in a
    second.  Products are exact in fp64 and rounded once: the 1e-5 bar of every other family.  Rows longer than a
    row block's entry window, empty rows and a last partial panel / row block are all in."""
    dev, stream, handle = gpu_ctx
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, cols % 1000 + rows, per_row=max(12, 4_800_000 // rows),
                                               long_rows=((7, 90_000), (rows // 2, 1), (rows - 1, 30_000)))
    assert colind.size > 2_000_000      # smaller matrices keep the ordinary kernels
    L = osa.lib()
    need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0)
    assert (need > 0) == applies
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y), alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    assert op.buffer.numel() >= need
    for alpha, beta in ((1.0, 0.0), (-2.0, 0.75), (0.5, 1.0)):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    assert np.array_equal(d[1].cpu().numpy(), colind) and np.array_equal(d[2].cpu().numpy(), val)


def test_blocked_gather_hot_rows_and_unaligned_x(osa, gpu_ctx):
    """Rows that put dozens of entries into one (panel, row block) chunk — the in-register run sums before the LDS
    atomics — next to one- and two-entry rows, and an x that is only 4-byte aligned."""
    dev, stream, handle = gpu_ctx
    rows, cols = 50_000, 1_500_000
    rng = np.random.default_rng(11)
    lengths = rng.integers(0, 3, rows)
    hot = rng.choice(rows, 90, replace=False)
    lengths[hot] = rng.integers(2_000, 60_000, hot.size)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = np.concatenate([np.sort(rng.choice(cols, int(l), replace=False)) for l in lengths]).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x = rng.uniform(-1, 1, cols).astype(np.float32)
    y0 = rng.uniform(-1, 1, rows).astype(np.float32)
    assert osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0) > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    xbuf = torch.zeros(cols + 1, dtype=torch.float32, device=dev)
    xbuf[1:].copy_(torch.from_numpy(x))
    d_x = xbuf[1:]
    assert d_x.data_ptr() % 16 == 4
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d_x), osa.DnVec(d_y),
                    alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    op(1.5, -0.25)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, -0.25)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def test_blocked_gather_giant_row_and_device_scalars(osa, gpu_ctx):
    """One row of a million entries — a row block with more 64-entry groups than its chunk table in LDS
    covers, and whole wavefronts of a single row — and alpha / beta read from device memory."""
    dev, stream, handle = gpu_ctx
    rows, cols = 20_000, 2_200_000
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, 3, per_row=120,
                                               long_rows=((11_111, 1_000_000), (11_112, 70_000)))
    assert osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0) > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A, X = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3])
    d_y = to_dev(y0, dev)
    Y = osa.DnVec(d_y)
    op = osa.SpmvOp(handle, A, X, Y, alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    op(1.0, 0.0)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.0)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    scal = torch.tensor([-0.5, 2.0], dtype=torch.float32, device=dev)
    d_y.copy_(torch.from_numpy(y0))
    torch.cuda.synchronize()
    handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_DEVICE)
    try:
        rc = osa.lib().aclsparseSpMV(handle.h, 0, ctypes.c_void_p(scal.data_ptr()), A.d, X.d,
                                     ctypes.c_void_p(scal.data_ptr() + 4), Y.d, osa.ACL_FLOAT,
                                     osa.ACL_SPARSE_SPMV_CSR_ALG2, ctypes.c_void_p(op.buffer.data_ptr()))
        assert rc == 0
        stream.synchronize()
    finally:
        handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_HOST)
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, -0.5, 2.0)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("rows,cols", [(1_400_000, 50_000), (2_000_000, 2_000_000), (1_200_000, 900_000), (1_100_000, 300)])
def test_blocked_gather_transposed(osa, gpu_ctx, rows, cols):
    """ACL_SPARSE_SPMV_CSR_ALG2 with op(A) = A^T and more than 2^18 rows: the layout is built over the rows of A
    (panels, x) and its columns (row blocks, y), and the product has no atomics on y: the 1e-5 bar of op(A) = A,
    not the reference's loose rule for its atomic transpose path.  A plan built for A^T does not serve A: the
    same descriptor and buffer then run op(A) = A through the ordinary kernels."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(rows % 1000 + cols)
    lengths = rng.integers(0, 6, rows)
    lengths[[5, rows // 3]] = [min(cols, 40_000), min(cols, 9_000)]
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)     # unsorted, repeated columns
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x = rng.uniform(-1, 1, rows).astype(np.float32)
    y0 = rng.uniform(-1, 1, cols).astype(np.float32)
    L = osa.lib()
    need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 1)
    assert need > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y), op=osa.ACL_SPARSE_OP_TRANSPOSE,
                    alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    assert op.buffer.numel() >= need
    for alpha, beta in ((1.0, 0.0), (-1.5, 0.5)):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    # the same buffer handed to an op(A) = A call: ignored, result still right
    xn = rng.uniform(-1, 1, cols).astype(np.float32)
    yn0 = rng.uniform(-1, 1, rows).astype(np.float32)
    d_xn, d_yn = to_dev(xn, dev), to_dev(yn0, dev)
    Xn, Yn = osa.DnVec(d_xn), osa.DnVec(d_yn)
    one, half = ctypes.c_float(1.0), ctypes.c_float(0.5)
    rc = L.aclsparseSpMV(handle.h, 0, ctypes.byref(one), A.d, Xn.d, ctypes.byref(half), Yn.d, osa.ACL_FLOAT,
                         osa.ACL_SPARSE_SPMV_CSR_ALG2, ctypes.c_void_p(op.buffer.data_ptr()))
    assert rc == 0
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, xn, yn0, 1.0, 0.5)
    assert oracle.max_rel_err(d_yn.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("transpose,narrow_y", [(False, False), (True, False), (False, True), (True, True)])
def test_blocked_gather_csr_alg2_half_precision_values(osa, gpu_ctx, dtype, transpose, narrow_y):
    """fp16 / bf16 values and x with an fp32 y under ACL_SPARSE_SPMV_CSR_ALG2: the same re-stored layout (it keeps
    the values in their own type and widens x as it loads a panel's slice), long rows included;
    against the fp64 oracle on the rounded inputs at the fp32 bar.  A launch with values of another type than the
    layout was built from is refused by the raw layer."""
    dev, stream, handle = gpu_ctx
    rows, cols = (1_300_000, 60_000) if transpose else (60_000, 3_000_000)
    rng = np.random.default_rng(rows % 977 + (1 if dtype == torch.float16 else 2))
    if transpose:
        lengths = rng.integers(0, 6, rows)
        lengths[[5, rows // 3]] = [40_000, 9_000]
        rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
        val = rng.uniform(-1, 1, colind.size).astype(np.float32)
        x, y0 = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, cols).astype(np.float32)
    else:
        rowptr, colind, val, x, y0 = _wide_problem(rows, cols, 5, per_row=80,
                                                   long_rows=((7, 90_000), (rows // 2, 1), (rows - 1, 30_000), (100, 1024)))
    rnd = lambda a: torch.from_numpy(a).to(dtype).float().numpy()
    val, x = rnd(val), rnd(x)
    L = osa.lib()
    need = L.opsparse_spmv_csr_blocked_workspace_bytes(
        rows, cols, colind.size, (osa.OPSPARSE_BLOCKED_TRANSPOSE if transpose else 0) |
        (osa.OPSPARSE_BLOCKED_VALUES_F16 if dtype == torch.float16 else osa.OPSPARSE_BLOCKED_VALUES_BF16))
    assert need > 0
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    if narrow_y:                                             # y of the values' type: the fp64 sum rounded once
        y0 = rnd(y0)
    d_val, d_x, d_y = to_dev(val, dev, dtype), to_dev(x, dev, dtype), to_dev(y0, dev, dtype if narrow_y else None)
    half_ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8

    def close(gold):
        got = d_y.float().cpu().numpy()
        if narrow_y:
            return bool(np.all(np.abs(got - gold) <= 1.001 * half_ulp * np.maximum(np.abs(gold), 2.0 ** -14)))
        return oracle.max_rel_err(got, gold) <= 1e-5

    A = osa.Csr(rows, cols, d_rp, d_ci, d_val)
    op = osa.SpmvOp(handle, A, osa.DnVec(d_x), osa.DnVec(d_y), alg=osa.ACL_SPARSE_SPMV_CSR_ALG2,
                    op=osa.ACL_SPARSE_OP_TRANSPOSE if transpose else osa.ACL_SPARSE_OP_NON_TRANSPOSE)
    assert op.buffer.numel() >= need                         # the layout, not the ordinary plan's few hundred KB
    golden = oracle.spmv_trans_f64 if transpose else oracle.spmv_f64
    for alpha, beta in ((1.0, 0.0), (-2.0, 0.75)):
        d_y.copy_(torch.from_numpy(y0).to(d_y.dtype))
        op(alpha, beta)
        stream.synchronize()
        assert close(golden(rows, cols, rowptr, colind, val, x, y0, alpha, beta))
    # raw layer: the plan remembers the type it was built from
    sp = ctypes.c_void_p(stream.cuda_stream)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    flag = (4 if dtype == torch.float16 else 8) | (1 if transpose else 0)
    assert L.opsparse_spmv_csr_blocked_analyse(d_rp.data_ptr(), d_ci.data_ptr(), d_val.data_ptr(), rows, cols, colind.size,
                                               flag, ws.data_ptr(), need, ctypes.byref(plan), sp) == 0
    want = osa.OPSPARSE_F16 if dtype == torch.float16 else osa.OPSPARSE_BF16
    assert plan.kernel == osa.OPSPARSE_SPMV_BLOCKED_GATHER and plan.valueType == want and plan.liveValues == 0
    one, zero = osa.OpsparseScalar(1.0, None, 0, 0), osa.OpsparseScalar(0.0, None, 0, 0)
    launch = lambda vt, v, xx: L.opsparse_spmv_csr_launch(ctypes.byref(plan), 1 if transpose else 0, d_rp.data_ptr(),
                                                          d_ci.data_ptr(), v.data_ptr(), xx.data_ptr(), d_y.data_ptr(), rows,
                                                          cols, colind.size, one, zero, vt,
                                                          want if narrow_y else osa.OPSPARSE_F32, 0,
                                                          ws.data_ptr(), need, sp)
    assert launch(want, d_val, d_x) == 0
    stream.synchronize()
    assert close(golden(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.0))
    f_val, f_x = to_dev(val, dev), to_dev(x, dev)
    assert launch(osa.OPSPARSE_F32, f_val, f_x) != 0         # fp32 operands with a plan built from 2-byte values


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_blocked_gather_random_shapes(osa, gpu_ctx, seed):
    """Seeded random shapes, both op(A): uniform short rows, power-law rows with a few of several hundred thousand
    entries, or dense stretches between long runs of empty rows; unsorted columns with repeats.  The products are
    exact in fp64 and rounded once, the same 1e-5 bar."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(seed)
    transpose = seed % 2 == 0
    big, small = int(rng.integers(1_050_000, 4_000_000)), int(rng.integers(3_000, 400_000))
    rows, cols = (big, small) if transpose else (small, big)
    kind = ("uniform", "power", "clustered")[seed % 3]
    if kind == "uniform":
        lengths = rng.integers(0, 8, rows)
    elif kind == "power":
        lengths = np.minimum((rng.pareto(1.1, rows) * 3).astype(np.int64), 300_000)
        lengths[rng.integers(0, rows, 3)] = rng.integers(50_000, 300_000, 3)
    else:
        lengths = np.zeros(rows, np.int64)
        for _ in range(12):
            a, w = int(rng.integers(0, rows)), int(rng.integers(1, max(2, rows // 40)))
            lengths[a:a + w] = rng.integers(1, 60, min(w, rows - a))
    lengths = np.minimum(lengths + max(0, (2_300_000 - int(lengths.sum())) // rows + 1), cols)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    nin, nout = (rows, cols) if transpose else (cols, rows)
    x, y0 = rng.uniform(-1, 1, nin).astype(np.float32), rng.uniform(-1, 1, nout).astype(np.float32)
    assert osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, int(transpose)) > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y),
                    op=osa.ACL_SPARSE_OP_TRANSPOSE if transpose else osa.ACL_SPARSE_OP_NON_TRANSPOSE,
                    alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    op(-1.25, 0.5)
    stream.synchronize()
    gold = (oracle.spmv_trans_f64 if transpose else oracle.spmv_f64)(rows, cols, rowptr, colind, val, x, y0, -1.25, 0.5)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def test_alg2_keeps_row_kernels_for_local_gathers(osa, workloads, gpu_ctx):
    """A mesh matrix wide enough for the re-stored layouts (1.2 M columns, 6 M entries): its gathers stay within
    1100 columns of the diagonal, x stays in cache under the row-wise kernels, and Preprocess with CSR_ALG2 keeps
    those (the sampled-locality probe says "not scattered"); the same shape with random columns is scattered."""
    dev, stream, handle = gpu_ctx
    A = workloads.laplacian_2d(1100, dev)
    rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
    L = osa.lib()
    assert L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, 0) > 0
    ws = torch.zeros(256, dtype=torch.uint8, device=dev)
    flag = ctypes.c_int32(-1)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    sp = ctypes.c_void_p(stream.cuda_stream)
    torch.cuda.synchronize()
    assert L.opsparse_spmv_csr_gathers_scattered(p(A["rowptr"]), p(A["colind"]), rows, cols, nnz, p(ws), 256,
                                                 ctypes.byref(flag), sp) == 0 and flag.value == 0
    shuffled = torch.randint(0, cols, (nnz,), dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    assert L.opsparse_spmv_csr_gathers_scattered(p(A["rowptr"]), p(shuffled), rows, cols, nnz, p(ws), 256,
                                                 ctypes.byref(flag), sp) == 0 and flag.value > 700   # in a thousand
    # one column in five sent anywhere: every fifth sampled gather, less the few that land near the diagonal by chance
    some = A["colind"].clone()
    some[::5] = shuffled[::5]
    torch.cuda.synchronize()
    assert L.opsparse_spmv_csr_gathers_scattered(p(A["rowptr"]), p(some), rows, cols, nnz, p(ws), 256,
                                                 ctypes.byref(flag), sp) == 0 and 120 <= flag.value <= 200
    rng = np.random.default_rng(3)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d_x, d_y = to_dev(x, dev), to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, A["rowptr"], A["colind"], A["values"]), osa.DnVec(d_x), osa.DnVec(d_y),
                    alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    op(1.0, 0.5)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy(),
                           A["values"].cpu().numpy(), x, y0, 1.0, 0.5)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    # the buffer holds an ordinary plan: changing the values needs no new Preprocess
    A["values"].mul_(2.0)
    d_y.copy_(torch.from_numpy(y0))
    op(1.0, 0.5)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy(),
                           A["values"].cpu().numpy(), x, y0, 1.0, 0.5)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("shape", ["mesh 700^2", "random 500 000^2", "narrow y"])
def test_alg2_transposed_below_2_20_outputs(osa, workloads, gpu_ctx, shape):
    """op(A) = A^T under CSR_ALG2 where y fits an L2: a mesh keeps the ordinary (atomic) kernels, whose updates stay
    in cache — the buffer then holds an ordinary plan and the values may change without a new Preprocess — while
    scattered columns, and a y of so few elements that many rows add to each, get the re-stored layout.  Which one
    ran shows in what a change of the values does: the layout holds a copy and does not follow it."""
    dev, stream, handle = gpu_ctx
    if shape.startswith("mesh"):
        A = workloads.laplacian_2d(700, dev)
        follows = True
    elif shape.startswith("random"):
        A = workloads.uniform_rows_csr(500_000, 500_000, 6, 3, dev)
        follows = False
    else:
        A = workloads.uniform_rows_csr(300_000, 16_000, 8, 3, dev)
        follows = False
    rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
    assert osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, 1) > 0
    rng = np.random.default_rng(4)
    x, y0 = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, cols).astype(np.float32)
    d_x, d_y = to_dev(x, dev), to_dev(y0, dev)
    vals = A["values"].clone()
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, A["rowptr"], A["colind"], vals), osa.DnVec(d_x), osa.DnVec(d_y),
                    op=osa.ACL_SPARSE_OP_TRANSPOSE, alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    rp, ci = A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy()

    def close(want):
        got = d_y.cpu().numpy()
        if follows:                                           # fp32 atomics: the reference's rule for that path
            return bool(np.all(np.abs(got - want) <= 2.0 ** -16 + 2.0 ** -10 * np.abs(want)))
        return oracle.max_rel_err(got, want) <= 1e-5

    op(1.0, 0.5)
    stream.synchronize()
    v0 = vals.cpu().numpy()
    gold = oracle.spmv_trans_f64(rows, cols, rp, ci, v0, x, y0, 1.0, 0.5)
    assert close(gold)
    vals.mul_(2.0)
    d_y.copy_(torch.from_numpy(y0))
    op(1.0, 0.5)
    stream.synchronize()
    gold2 = oracle.spmv_trans_f64(rows, cols, rp, ci, 2.0 * v0, x, y0, 1.0, 0.5)
    assert close(gold2 if follows else gold) and not close(gold if follows else gold2)


def test_blocked_gather_through_spmvop_alg2(osa, gpu_ctx):
    """aclsparseSpMVOp ALG2 on a wide matrix uses the blocked-gather layout; Z separate from Y and aliased."""
    dev, stream, handle = gpu_ctx
    rows, cols = 40_000, 2_500_000
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, 5, long_rows=((3, 50_000),), per_row=120)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    for alias in (False, True):
        d_y = to_dev(y0, dev)
        d_z = d_y if alias else torch.zeros(rows, dtype=torch.float32, device=dev)
        Y = osa.DnVec(d_y)
        Z = Y if alias else osa.DnVec(d_z)
        op = osa.SpmvOpPlan(handle, A, osa.DnVec(d[3]), Y, Z, alg=osa.ACL_SPARSE_SPMVOP_ALG2)
        assert op.buffer_bytes == osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0) > 0
        op(1.25, -0.5)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.25, -0.5)
        assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5
        op.close()


def test_blocked_gather_rejects_column_out_of_range(osa, gpu_ctx):
    """The analysis checks every column index against cols (the kernels index LDS with it) and returns
    OPSPARSE_E_INVALID; aclsparseSpMVPreprocess turns that into INVALID_VALUE."""
    dev, stream, handle = gpu_ctx
    rows, cols = 30_000, 1_200_000
    rowptr, colind, val, x, y0 = _wide_problem(rows, cols, 9, per_row=160)
    colind = colind.copy()
    colind[colind.size // 2] = cols + 5
    L = osa.lib()
    need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0)
    assert need > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    torch.cuda.synchronize()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = L.opsparse_spmv_csr_blocked_analyse(p(d[0]), p(d[1]), p(d[2]), rows, cols, colind.size, 0, p(ws), need,
                                             ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream))
    assert rc == osa.OPSPARSE_E_INVALID
    d_x, d_y = to_dev(x, dev), to_dev(y0, dev)
    A, X, Y = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d_x), osa.DnVec(d_y)
    asked = ctypes.c_size_t(0)
    assert L.aclsparseSpMVGetBufferSize(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT,
                                        osa.ACL_SPARSE_SPMV_CSR_ALG2, ctypes.byref(asked)) == 0
    assert asked.value == need
    st = L.aclsparseSpMVPreprocess(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT,
                                   osa.ACL_SPARSE_SPMV_CSR_ALG2, p(ws))
    assert st == osa.ACL_SPARSE_STATUS_INVALID_VALUE


@pytest.mark.parametrize("dtype,rel", [(torch.float16, 2.0 ** -10), (torch.bfloat16, 2.0 ** -7)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_transpose_half_precision_output(osa, gpu_ctx, dtype, rel, beta):
    """y = alpha * A^T x + beta * y with fp16 / bf16 A, x and y: sums formed in an fp32 staging vector (handle
    workspace), rounded once.  Bar: one rounding of the output type (+ the fp32 atomics' 1e-4 absolute slack)."""
    rows, cols = 3000, 900
    rowptr, colind, val = random_csr(rows, cols, 0.02, 21, lo=-1.0, hi=1.0)
    rng = np.random.default_rng(6)
    rt = lambda a: torch.from_numpy(a).to(dtype).float().numpy()          # values as the kernel sees them
    val, x, y0 = rt(val), rt(rng.uniform(-1, 1, rows).astype(np.float32)), rt(rng.uniform(-1, 1, cols).astype(np.float32))
    y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 1.5, beta, op=osa.ACL_SPARSE_OP_TRANSPOSE,
                 val_dtype=dtype, out_dtype=dtype)
    gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, beta)
    assert np.all(np.abs(y - gold) <= rel * np.abs(gold) + 1e-4)


def test_transpose_half_precision_output_longer_than_the_workspace(osa, gpu_ctx):
    """fp16 y of 1.5 M elements under op(A) = A^T: its fp32 staging vector (6 MB) does not fit the handle's 4 MiB
    workspace.  aclsparseSpMVGetBufferSize counts it in, and the call sums in the preprocessed buffer; without
    Preprocess the call reports INSUFFICIENT_RESOURCES (aclsparseSetWorkspace is the way then) and leaves y."""
    dev, stream, handle = gpu_ctx
    rows, cols, per_row = 4000, 1_500_000, 25
    rng = np.random.default_rng(77)
    rowptr = (np.arange(rows + 1) * per_row).astype(np.int32)
    colind = rng.integers(0, cols, rows * per_row).astype(np.int32)
    rt = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.float16).float().numpy()
    val, x, y0 = rt(rng.uniform(-1, 1, colind.size)), rt(rng.uniform(-1, 1, rows)), rt(rng.uniform(-1, 1, cols))
    gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5)
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val, d_x = to_dev(val, dev, torch.float16), to_dev(x, dev, torch.float16)
    A, X = osa.Csr(rows, cols, d_rp, d_ci, d_val), osa.DnVec(d_x)
    # unprepared: the default workspace is too small
    d_y = to_dev(y0, dev, torch.float16)
    bare = osa.SpmvOp(handle, A, X, osa.DnVec(d_y), op=osa.ACL_SPARSE_OP_TRANSPOSE, preprocess=False)
    with pytest.raises(osa.AclsparseError) as err:
        bare(1.5, 0.5)
    assert err.value.status == osa.ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES
    stream.synchronize()
    assert np.array_equal(d_y.cpu().float().numpy(), y0)
    # preprocessed: the buffer holds the staging vector behind the plan
    Y = osa.DnVec(d_y)
    n = ctypes.c_size_t(0)
    L = osa.lib()
    assert L.aclsparseSpMVGetBufferSize(handle.h, osa.ACL_SPARSE_OP_TRANSPOSE, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT,
                                        0, ctypes.byref(n)) == 0
    assert n.value >= cols * 4
    op = osa.SpmvOp(handle, A, X, Y, op=osa.ACL_SPARSE_OP_TRANSPOSE)
    for _ in range(2):                                                     # the buffer serves every call
        d_y.copy_(torch.from_numpy(y0).to(torch.float16))
        op(1.5, 0.5)
        stream.synchronize()
        y = d_y.cpu().float().numpy()
        assert np.all(np.abs(y - gold) <= 2.0 ** -10 * np.abs(gold) + 1e-4)
    # the same buffer still serves op(A) = A (its own part is in front of the staging vector)
    d_x2, d_y2 = to_dev(rt(rng.uniform(-1, 1, cols)), dev, torch.float16), torch.zeros(rows, dtype=torch.float16, device=dev)
    (ka, pa), (kb, pb) = osa._scalar_ref(1.0, osa.ACL_FLOAT), osa._scalar_ref(0.0, osa.ACL_FLOAT)
    X2, Y2 = osa.DnVec(d_x2), osa.DnVec(d_y2)
    st = L.aclsparseSpMV(handle.h, 0, pa, A.d, X2.d, pb, Y2.d, osa.ACL_FLOAT, 0, ctypes.c_void_p(op.buffer.data_ptr()))
    assert st == 0
    stream.synchronize()
    gold2 = oracle.spmv_f64(rows, cols, rowptr, colind, val, d_x2.cpu().float().numpy(), np.zeros(rows, np.float32), 1.0, 0.0)
    assert np.all(np.abs(d_y2.cpu().float().numpy() - gold2) <= 2.0 ** -10 * np.abs(gold2) + 1e-4)


@pytest.mark.parametrize("per_row,out_dtype", [(4, None), (20, None), (6, torch.float16), (40, None)])
def test_unprepared_calls_survive_row_offsets_changed_in_place(osa, gpu_ctx, per_row, out_dtype):
    """The first call without a preprocessed buffer takes the row statistics of the matrix, and later ones run the
    stream-rows kernel they select, whose LDS is sized for the longest row seen.  Nobody promised those calls
    that the row offsets stay: rewritten in place afterwards — same array, same entry count, one row now thousands
    of entries long, others empty, one row twice as long inside an unchanged tile — they must still give the
    right product (such tiles are summed from memory).  After Preprocess the structure is the caller's promise."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(per_row)
    rows, cols = 60_000, 50_000
    lengths = np.full(rows, per_row, np.int64)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    if out_dtype is not None:
        val, x = (torch.from_numpy(a).to(out_dtype).float().numpy() for a in (val, x))
    vt = out_dtype or torch.float32
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val, d_x = torch.from_numpy(val).to(vt).to(dev), torch.from_numpy(x).to(vt).to(dev)
    d_y = torch.from_numpy(y0).to(vt).to(dev)
    A = osa.Csr(rows, cols, d_rp, d_ci, d_val)
    op = osa.SpmvOp(handle, A, osa.DnVec(d_x), osa.DnVec(d_y), preprocess=False)
    y0r = d_y.float().cpu().numpy()

    def check_against(rp):
        d_y.copy_(torch.from_numpy(y0r).to(vt))
        op(1.5, 0.5)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rp, colind, val, x, y0r, 1.5, 0.5)
        got = d_y.float().cpu().numpy()
        if out_dtype is None:
            assert oracle.max_rel_err(got, gold) <= 1e-5
        else:                                          # y rounded once to fp16: within an ulp of the rounded oracle
            want = _round(gold, out_dtype)
            assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 2.0 ** -14))

    check_against(rowptr)
    moved = lengths.copy()
    moved[5] += 3000                                   # far beyond what a tile's LDS was sized for
    taken, r = 0, 30_000
    while taken < 3000:                                # taken from rows that become empty / shorter
        t = min(per_row, 3000 - taken)
        moved[r] -= t
        taken += t
        r += 1
    moved[50_001] += moved[50_000]                     # a row twice as long, its tile's entry count unchanged
    moved[50_000] = 0
    assert moved.sum() == lengths.sum()
    rowptr2 = np.concatenate([[0], np.cumsum(moved)]).astype(np.int32)
    d_rp.copy_(torch.from_numpy(rowptr2))
    check_against(rowptr2)
    d_rp.copy_(torch.from_numpy(rowptr))
    check_against(rowptr)


@pytest.mark.parametrize("rows,cols,per_row,half", [(40_000, 9, 120, True), (200_000, 300, 20, False),
                                                    (60_000, 8192, 40, False), (30_000, 8193, 40, False),
                                                    (40_000, 16384, 30, False), (40_000, 16385, 30, False)])
def test_transpose_few_columns_accumulates_per_workgroup(osa, gpu_ctx, rows, cols, per_row, half):
    """op(A) = A^T onto a short y: hundreds of thousands of contributions per element.  With one fp32 atomic each
    (the reference's scheme) the rounding errors add up past 1e-2 in absolute terms; summed per workgroup in fp64
    and added to y once per workgroup they stay at fp32 round-off of the result.  16385 columns are one too many
    for that kernel and take the atomic one, under the loose rule only."""
    rng = np.random.default_rng(rows + cols)
    rowptr = (np.arange(rows + 1, dtype=np.int64) * per_row).astype(np.int32)
    colind = rng.integers(0, cols, rows * per_row).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, cols).astype(np.float32)
    if half:
        val, x = _round(val, torch.float16), _round(x, torch.float16)
    for prep in (False, True):
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 2.25, 0.5, preprocess=prep,
                     op=osa.ACL_SPARSE_OP_TRANSPOSE, val_dtype=torch.float16 if half else None,
                     out_dtype=torch.float32 if half else None)
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 2.25, 0.5)
        d = np.abs(y - gold)
        assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2
        if cols <= 16384:
            assert d.max() <= 1e-4 * max(1.0, float(np.abs(gold).max()))


@pytest.mark.parametrize("prepared", [True, False])
def test_rows_through_hundreds_of_merge_workgroups(osa, gpu_ctx, prepared):
    """Rows of 1.2 M, 140 000 and 131 entries between short ones: the long ones pass through 590 and 69 merge
    workgroups, whose carries the fix-up adds with a whole wavefront; the third through one or two (one lane)."""
    rng = np.random.default_rng(77)
    rows, cols = 30_000, 2_000_000
    lengths = rng.integers(0, 7, rows)
    lengths[[0, 12_345, 29_999]] = [140_000, 1_200_000, 131]
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, -1.5, 0.25, preprocess=prepared)
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, -1.5, 0.25)
    assert oracle.max_rel_err(y, gold) <= 1e-5


def test_transpose_few_long_rows_split_by_entries(osa, gpu_ctx):
    """Fifty rows of thousands of entries onto 200 000 columns: too few rows for a lane group each, the entries are
    dealt out 2048 to a workgroup and the row of an entry is looked up in the offsets (some rows empty)."""
    rng = np.random.default_rng(5)
    rows, cols = 50, 200_000
    lengths = rng.integers(2_000, 9_000, rows)
    lengths[[0, 17, 49]] = 0
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, cols).astype(np.float32)
    for prep in (True, False):
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, 1.5, -0.5, preprocess=prep,
                     op=osa.ACL_SPARSE_OP_TRANSPOSE)
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, -0.5)
        d = np.abs(y - gold)
        assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2


@pytest.mark.parametrize("short,out_dtype,prepared", [(5, None, True), (5, None, False), (20, None, True),
                                                      (7, torch.float16, True), (40, None, False)])
def test_short_rows_with_a_few_long_ones_beside(osa, gpu_ctx, short, out_dtype, prepared):
    """A banded matrix of short rows with a handful of long ones (65 - 8192 entries, some next to each other, one
    the first row, one the last): the stream-rows tiles are sized for the short rows and skip the long ones,
    which a second kernel sums with a workgroup each.  Every row must be written exactly once — in place with
    beta != 0 a second write would show.  Rows of 49 - 64 entries are too long for the tiles' sizing but not
    skipped: their tiles are summed from memory."""
    rng = np.random.default_rng(short)
    rows = cols = 300_000
    lengths = rng.integers(max(1, short - 3), short + 1, rows)
    lengths[rng.choice(rows, 40, replace=False)] = 0
    long_rows = np.array([0, 1, 2, 77_000, 150_000, 150_001, 299_999])
    lengths[long_rows] = [65, 3000, 8192, 512, 513, 8_000, 700]
    lengths[[5_000, 5_001, 250_000]] = [49, 64, 60]
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    centre = np.repeat(np.arange(rows), lengths)
    colind = np.clip(centre + rng.integers(-3000, 3001, centre.size), 0, cols - 1).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    if out_dtype is not None:
        val, x, y0 = _round(val, out_dtype), _round(x, out_dtype), _round(y0, out_dtype)
    if prepared:
        plan = osa.OpsparseSpmvPlan()
        dev, stream, handle = gpu_ctx
        d_rp = to_dev(rowptr, dev)
        L = osa.lib()
        ws = torch.empty(max(L.opsparse_spmv_csr_workspace_bytes(rows, colind.size), 256), dtype=torch.uint8, device=dev)
        assert L.opsparse_spmv_csr_analyse(d_rp.data_ptr(), rows, cols, colind.size, ws.data_ptr(), ws.numel(),
                                           osa.OPSPARSE_SPMV_AUTO, ctypes.byref(plan),
                                           ctypes.c_void_p(stream.cuda_stream)) == 0
        assert plan.kernel == osa.OPSPARSE_SPMV_STREAM_ROWS and plan.longRowsBeside == 1
        assert plan.tileRowNnz == short and plan.maxRowNnz == 8192
    for alpha, beta in ((1.5, 0.5), (2.0, 0.0)):
        y = run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, alpha, beta, preprocess=prepared,
                     val_dtype=out_dtype, out_dtype=out_dtype)
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
        if out_dtype is None:
            assert oracle.max_rel_err(y, gold) <= 1e-5
        else:
            want = _round(gold, out_dtype)
            assert np.all(np.abs(y - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 2.0 ** -14))
