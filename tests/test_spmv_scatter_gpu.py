"""The layout of op(A) = A^T under the default algorithm where the last bit of a result may vary (plan kernel
OPSPARSE_SPMV_SCATTER_LIVE): products sorted by output panel through LDS, then summed in LDS; no atomics on y and no
transposed copy.  Against the fp64 oracle of the transposed product.

Bars: the products are exact and the sums fp64, rounded once, as in the layouts of op(A) = A: fp32 y within 1e-5 of
the oracle element by element, fp16 / bf16 y within one unit in the last place of the oracle rounded to that type."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import to_dev

pytestmark = pytest.mark.gpu

PIECE = {torch.float32: 16384, torch.float16: 32768, torch.bfloat16: 32768}   # 128 KiB of exact products
ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


@pytest.fixture(autouse=True)
def _small_matrices(monkeypatch):
    """The layout is taken from 128 output panels (2 M columns) and, by the default algorithm, from 7 M entries on;
    the matrices here have 19 panels and 3 M entries so that the oracle stays quick.  Both switches are read at every
    size query and analysis."""
    monkeypatch.setenv("OPS_SPARSE_SCATTER_MIN_PANELS", "8")
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.delenv("OPS_SPARSE_SPMV_REPEATABLE", raising=False)


def _matrix(rows, cols, seed, per_row=5, hot_column=0, empty_run=0):
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, per_row, rows)
    lengths[[11, rows // 2]] = [30_000, 9_000]               # long rows of A are nothing special here
    if empty_run:
        lengths[1000:1000 + empty_run] = 0
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    if hot_column:
        colind[rng.choice(colind.size, hot_column, replace=False)] = 77
    return rowptr, colind


def _seen(a, dtype):
    return torch.from_numpy(a.astype(np.float32)).to(dtype).float().numpy()


def _check(got, gold, out_dtype):
    if out_dtype == torch.float32:
        assert oracle.max_rel_err(got, gold) <= 1e-5
    else:
        want = _seen(gold, out_dtype)
        assert np.all(np.abs(got - want) <= ULP[out_dtype] * np.maximum(np.abs(want), 2.0 ** -14))


def _flag(osa, dtype):
    return {torch.float32: 0, torch.float16: osa.OPSPARSE_BLOCKED_VALUES_F16,
            torch.bfloat16: osa.OPSPARSE_BLOCKED_VALUES_BF16}[dtype]


def _code(osa, dtype):
    return {torch.float32: osa.OPSPARSE_F32, torch.float16: osa.OPSPARSE_F16, torch.bfloat16: osa.OPSPARSE_BF16}[dtype]


@pytest.mark.parametrize("dtype,narrow_y", [(torch.float32, False), (torch.float16, False), (torch.float16, True),
                                            (torch.bfloat16, False), (torch.bfloat16, True)])
def test_scatter_layout_through_the_launch_layer(osa, gpu_ctx, dtype, narrow_y):
    """Analysis and launch through the raw entry points, every type pair: the plan's shape (19 panels of 2^14 columns,
    pieces of 128 KiB of products), the products for two pairs of scalars, and again after the values changed in place (the
    layout holds none).  The split form of the analysis leaves the same plan."""
    dev, stream, _ = gpu_ctx
    L = osa.lib()
    rows, cols = 1_400_000, 300_000
    rowptr, colind = _matrix(rows, cols, 5)
    nnz = colind.size
    rng = np.random.default_rng(6)
    out_dtype = dtype if narrow_y else torch.float32
    val, x = _seen(rng.uniform(-1, 1, nnz), dtype), _seen(rng.uniform(-1, 1, rows), dtype)
    y0 = _seen(rng.uniform(-1, 1, cols), out_dtype)
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val, d_x = to_dev(val, dev, dtype), to_dev(x, dev, dtype)
    need = L.opsparse_spmv_csr_scatter_workspace_bytes(rows, cols, nnz, _flag(osa, dtype))
    keep = L.opsparse_spmv_csr_scatter_resident_bytes(rows, cols, nnz, _flag(osa, dtype))
    per_entry = 6 + (8 if dtype == torch.float32 else 4)            # slot and row, local column, the product
    assert 0 < keep < need and keep < (per_entry + 1) * nnz + (1 << 22)   # ... and the chunk tables
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    sp = ctypes.c_void_p(stream.cuda_stream)
    assert L.opsparse_spmv_csr_scatter_analyse(pv(d_rp), pv(d_ci), rows, cols, nnz, _flag(osa, dtype), pv(ws), need,
                                               ctypes.byref(plan), sp) == 0
    assert plan.kernel == osa.OPSPARSE_SPMV_SCATTER_LIVE and plan.transposed == 1 and plan.liveValues == 1
    assert plan.numPanels == -(-cols // 16384) == 19 and plan.numRowBlocks == -(-nnz // PIECE[dtype])

    def run(buffer, values, alpha, beta):
        d_y = to_dev(y0, dev, out_dtype)
        sa, sb = osa.OpsparseScalar(alpha, None, 0, 0), osa.OpsparseScalar(beta, None, 0, 0)
        rc = L.opsparse_spmv_csr_launch(ctypes.byref(plan), 1, pv(d_rp), pv(d_ci), pv(d_val), pv(d_x), pv(d_y), rows, cols,
                                        nnz, sa, sb, _code(osa, dtype), _code(osa, out_dtype), 0, pv(buffer),
                                        buffer.numel(), sp)
        assert rc == 0
        stream.synchronize()
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        _check(d_y.float().cpu().numpy(), gold, out_dtype)

    run(ws, val, 1.0, 0.0)
    run(ws, val, -1.5, 0.5)
    val2 = _seen(rng.uniform(-2, 2, nnz), dtype)
    d_val.copy_(to_dev(val2, dev, dtype))
    run(ws, val2, 2.0, 1.0)
    # what the launches keep and the analysis' scratch in two pieces
    kept = torch.empty(keep, dtype=torch.uint8, device=dev)
    scratch = torch.empty(need - keep, dtype=torch.uint8, device=dev)
    plan2 = osa.OpsparseSpmvPlan()
    assert L.opsparse_spmv_csr_scatter_analyse_split(pv(d_rp), pv(d_ci), rows, cols, nnz, _flag(osa, dtype), pv(kept),
                                                     keep, pv(scratch), need - keep, ctypes.byref(plan2), sp) == 0
    assert bytes(plan2) == bytes(plan)
    del scratch
    run(kept, val2, 1.0, 0.0)


def _preprocess(osa, gpu_ctx, rowptr, colind, cols, seed=1, alg=0, dtype=torch.float32):
    """GetBufferSize / Preprocess for op(A) = A^T into a buffer pre-filled with a pattern; returns what a test needs to
    call and to see which part of the buffer Preprocess wrote."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, nnz = rowptr.size - 1, colind.size
    rng = np.random.default_rng(seed)
    val, x = _seen(rng.uniform(-1, 1, nnz), dtype), _seen(rng.uniform(-1, 1, rows), dtype)
    y0 = rng.uniform(-1, 1, cols).astype(np.float32)
    d = dict(rp=to_dev(rowptr, dev), ci=to_dev(colind, dev), val=to_dev(val, dev, dtype), x=to_dev(x, dev, dtype),
             y=to_dev(y0, dev))
    A, X, Y = osa.Csr(rows, cols, d["rp"], d["ci"], d["val"]), osa.DnVec(d["x"]), osa.DnVec(d["y"])
    asked = ctypes.c_size_t(0)
    T = osa.ACL_SPARSE_OP_TRANSPOSE
    assert L.aclsparseSpMVGetBufferSize(handle.h, T, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, alg,
                                        ctypes.byref(asked)) == 0
    buf = torch.full((asked.value,), 0x5A, dtype=torch.uint8, device=dev)
    pbuf = ctypes.c_void_p(buf.data_ptr())
    st = L.aclsparseSpMVPreprocess(handle.h, T, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, alg, pbuf)

    def call(values, alpha, beta):
        d["y"].copy_(torch.from_numpy(y0))
        a, b = ctypes.c_float(alpha), ctypes.c_float(beta)
        assert L.aclsparseSpMV(handle.h, T, ctypes.byref(a), A.d, X.d, ctypes.byref(b), Y.d, osa.ACL_FLOAT, alg,
                               pbuf) == 0
        stream.synchronize()
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        assert oracle.max_rel_err(d["y"].cpu().numpy(), gold) <= 1e-5
        return d["y"].clone()

    return st, buf, d, val, call, (A, X, Y)


def _untouched_from(buf, offset):
    return bool((buf[offset:] == 0x5A).all())


def test_default_algorithm_takes_the_scatter_layout_for_the_transposed_product(osa, gpu_ctx):
    """aclsparseSpMV with ALG_DEFAULT, op(A) = A^T, scattered columns: the size query answers with the ordered layout
    over a transposed copy (the larger of the two), Preprocess builds the scatter layout inside that buffer - seen
    from the bytes it leaves untouched - and the calls follow values changed in place."""
    L = osa.lib()
    rows, cols = 1_400_000, 300_000
    rowptr, colind = _matrix(rows, cols, 21)
    nnz = colind.size
    st, buf, d, val, call, _ = _preprocess(osa, gpu_ctx, rowptr, colind, cols)
    assert st == 0
    ordered = L.opsparse_spmv_csr_blocked_workspace_bytes(
        rows, cols, nnz, osa.OPSPARSE_BLOCKED_TRANSPOSE | osa.OPSPARSE_BLOCKED_LIVE_VALUES)
    scatter = L.opsparse_spmv_csr_scatter_workspace_bytes(rows, cols, nnz, 0)
    assert 0 < scatter < ordered <= buf.numel()
    assert _untouched_from(buf, scatter) and not _untouched_from(buf, scatter // 2)
    call(val, 1.0, 0.0)
    call(val, 1.5, -0.5)
    val2 = (val * np.float32(-0.5) + np.float32(0.25)).astype(np.float32)
    d["val"].copy_(torch.from_numpy(val2))
    call(val2, 1.0, 1.0)


@pytest.mark.parametrize("why", ["repeatable", "hot column", "runs of empty rows", "switched off"])
def test_ordered_layout_where_the_scatter_layout_does_not_serve(osa, gpu_ctx, why, monkeypatch):
    """Where the caller asked for repeatable results (OPS_SPARSE_SPMV_REPEATABLE), a column has more than 8192 entries
    (its products would queue for one LDS address), or a piece of 16 384 entries spans more than 65 535 rows,
    Preprocess builds the ordered layout over the transposed copy as before (it writes beyond the scatter layout's
    bytes); the products are right either way, and the repeatable ones repeat."""
    L = osa.lib()
    rows, cols = 1_400_000, 600_000
    if why == "repeatable":
        monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")
    if why == "switched off":
        monkeypatch.setenv("OPS_SPARSE_SPMV_NO_SCATTER", "1")
    rowptr, colind = _matrix(rows, cols, 23, hot_column=9000 if why == "hot column" else 0,
                             empty_run=80_000 if why == "runs of empty rows" else 0)
    nnz = colind.size
    st, buf, d, val, call, _ = _preprocess(osa, gpu_ctx, rowptr, colind, cols)
    assert st == 0
    scatter = L.opsparse_spmv_csr_scatter_workspace_bytes(rows, cols, nnz, 0)
    assert 0 < scatter < buf.numel() and not _untouched_from(buf, scatter)
    first = call(val, 1.0, 0.5)
    second = call(val, 1.0, 0.5)
    assert torch.equal(first, second)                         # the ordered kernels: the same bits


def test_scatter_analysis_refusals(osa, gpu_ctx):
    """The raw analysis: OPSPARSE_E_INVALID for a column index out of range, OPSPARSE_E_UNSUPPORTED for a hot column,
    for a piece that spans too many rows, for int32 values and for a matrix with too few columns; OPSPARSE_E_WORKSPACE
    for a buffer too small."""
    dev, stream, _ = gpu_ctx
    L = osa.lib()
    rows, cols = 1_400_000, 300_000
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    sp = ctypes.c_void_p(stream.cuda_stream)
    plan = osa.OpsparseSpmvPlan()

    def analyse(rowptr, colind, flags=0, cols_=cols, shrink=0):
        d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
        need = L.opsparse_spmv_csr_scatter_workspace_bytes(rows, cols_, colind.size, flags)
        ws = torch.empty(max(need - shrink, 256), dtype=torch.uint8, device=dev)
        return L.opsparse_spmv_csr_scatter_analyse(pv(d_rp), pv(d_ci), rows, cols_, colind.size, flags, pv(ws),
                                                   ws.numel(), ctypes.byref(plan), sp)

    rowptr, colind = _matrix(rows, cols, 31)
    assert analyse(rowptr, colind) == 0
    assert analyse(rowptr, colind, shrink=4096) == osa.OPSPARSE_E_WORKSPACE
    assert analyse(rowptr, colind, flags=osa.OPSPARSE_BLOCKED_VALUES_I32) == osa.OPSPARSE_E_UNSUPPORTED
    assert L.opsparse_spmv_csr_scatter_workspace_bytes(rows, 100_000, colind.size, 0) == 0       # 7 panels
    bad = colind.copy()
    bad[bad.size // 3] = cols
    assert analyse(rowptr, bad) == osa.OPSPARSE_E_INVALID
    assert analyse(*_matrix(rows, cols, 32, hot_column=9000)) == osa.OPSPARSE_E_UNSUPPORTED
    assert analyse(*_matrix(rows, cols, 33, empty_run=80_000)) == osa.OPSPARSE_E_UNSUPPORTED
