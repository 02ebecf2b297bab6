"""The plan aclsparseSpMVPreprocess picks for ACL_SPARSE_SPMV_ALG_DEFAULT on a large matrix with scattered
columns: a blocked-gather layout with live values — the one whose row blocks add with atomics (plan kernel
BLOCKED_LIVE) for op(A) = A and floating-point values, the ordered one (BLOCKED_GATHER, the same bits from every
call) with OPS_SPARSE_SPMV_REPEATABLE in the environment, for op(A) = A^T, for int32 values and under
aclsparseSpMVOp.  The contract under test: a caller that follows the
reference's call pattern (GetBufferSize, Preprocess, SpMV with the default algorithm) may change the values in
place, or hand the descriptor a new values array, between calls, and always gets the product of the values as
they are at the call.  An explicit ACL_SPARSE_SPMV_CSR_ALG2 request holds a copy of the values: there
aclsparseSpMatSetValues drops the plan and later calls run on the new array with the ordinary kernels."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _layout_for_small_matrices(monkeypatch):
    """The default plan takes the layout from 7 M entries on; the matrices here have 2.5 - 4 M so that the fp64
    oracle stays quick.  The override is read at every GetBufferSize / Preprocess."""
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.setenv("OPS_SPARSE_ORDERED_LIVE_MIN_COLS", "0")   # (the ordered live layout: from 2.6 M columns)


def _default_bytes(osa, rows, cols, nnz, repeatable):
    """What GetBufferSize answers for the default algorithm, op(A) = A, fp values, scattered columns."""
    L = osa.lib()
    if repeatable:
        return L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
    return L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)


@pytest.fixture(params=[False, True], ids=["atomics", "repeatable"])
def repeatable(request, monkeypatch):
    if request.param:
        monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")
    else:
        monkeypatch.delenv("OPS_SPARSE_SPMV_REPEATABLE", raising=False)
    return request.param


def _scattered(rows, cols, seed, per_row=16):
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, per_row, rows)
    lengths[rows // 2] = 30_000
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)  # unsorted, repeats possible
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    return rowptr, colind, val, rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)


def test_default_plan_is_the_live_blocked_layout_and_follows_the_values(osa, gpu_ctx, repeatable):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 5)
    nnz = colind.size
    want = _default_bytes(osa, rows, cols, nnz, repeatable)
    assert want > L.opsparse_spmv_csr_workspace_bytes(rows, nnz) > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A, X = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, X, osa.DnVec(d_y))           # ALG_DEFAULT
    assert op.buffer.numel() == want                        # GetBufferSize asked for the layout: the probe said scattered

    def check(values, alpha, beta):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    check(val, 1.0, 0.0)
    # values changed in place, same pointer
    val2 = (val * np.float32(-0.5) + np.float32(0.25)).astype(np.float32)
    d[2].copy_(torch.from_numpy(val2))
    check(val2, 1.5, -0.5)
    # a new values array in the same descriptor
    val3 = np.random.default_rng(9).uniform(-3, 3, nnz).astype(np.float32)
    d_val3 = to_dev(val3, dev)
    assert L.aclsparseSpMatSetValues(A.d, ctypes.c_void_p(d_val3.data_ptr())) == 0
    check(val3, -1.0, 0.0)
    # the layout only: a launch accepts a buffer cut down to the resident size
    resident = (L.opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
                if repeatable else L.opsparse_spmv_csr_live_resident_bytes(rows, cols, nnz))
    assert 0 < resident < want


@pytest.mark.parametrize("alias", [False, True])
def test_spmvop_default_algorithm_takes_the_live_layout_when_given_the_buffer(osa, gpu_ctx, alias):
    """aclsparseSpMVOp with the default algorithm on the same kind of matrix: bufferSize asks for the layout's
    buffer, createDescr builds the layout in it, and the executions follow the values as they change in place (ALG1
    promises nothing else).  Without the buffer the same call runs the ordinary kernels."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 6)
    nnz = colind.size
    want = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    d_z = d_y if alias else torch.zeros(rows, dtype=torch.float32, device=dev)
    Y = osa.DnVec(d_y)
    Z = Y if alias else osa.DnVec(d_z)
    op = osa.SpmvOpPlan(handle, A, osa.DnVec(d[3]), Y, Z)    # ALG_DEFAULT
    assert op.buffer_bytes == want > 0 and op.buffer is not None

    def check(values, alpha, beta):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5
        if not alias:
            assert np.array_equal(d_y.cpu().numpy(), y0)

    check(val, 1.0, 0.0)
    val2 = (val * np.float32(0.5) - np.float32(0.125)).astype(np.float32)
    d[2].copy_(torch.from_numpy(val2))
    check(val2, -1.5, 0.75)
    op.close()
    # no buffer: the ordinary kernels, the same result
    descr, plan = ctypes.c_void_p(), ctypes.c_void_p()
    X = osa.DnVec(d[3])
    common = (0, A.d, X.d, Y.d, Z.d, osa.ACL_FLOAT, osa.ACL_SPARSE_SPMVOP_ALG_DEFAULT)
    assert L.aclsparseSpMVOp_createDescr(handle.h, ctypes.byref(descr), *common, None) == 0
    assert L.aclsparseSpMVOp_createPlan(handle.h, descr, ctypes.byref(plan), None, 0) == 0
    one, zero = ctypes.c_float(1.0), ctypes.c_float(0.0)
    d_y.copy_(torch.from_numpy(y0))
    assert L.aclsparseSpMVOp(handle.h, plan, ctypes.byref(one), ctypes.byref(zero), X.d, Y.d, Z.d) == 0
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val2, x, y0, 1.0, 0.0)
    assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5
    L.aclsparseSpMVOp_destroyPlan(plan)
    L.aclsparseSpMVOp_destroyDescr(descr)


def _with_long_rows(rows, cols, seed):
    """Short scattered rows and, among them, long ones: first row, last row, two neighbours, one with repeated
    columns (ascending all the same), one whose columns do not ascend, lengths either side of the threshold."""
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, 20, rows)
    long_rows = {0: 9000, 7: 4096, 8: 4095, 1000: 40_000, 1001: 20_000, 150_000: 120_000, 200_000: 6000,
                 rows - 1: 5000}
    for r, l in long_rows.items():
        lengths[r] = l
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    for r in long_rows:
        a, b = rowptr[r], rowptr[r + 1]
        if r == 200_000:
            continue                                         # stays unsorted: not a long row to the library
        seg = np.sort(rng.integers(0, cols, b - a)) if r == 1001 else np.sort(rng.choice(cols, b - a, replace=False))
        colind[a:b] = seg.astype(np.int32)                   # row 1001 keeps its repeated columns
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    return rowptr, colind, val, rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("narrow_y", [False, True])
def test_default_plan_with_half_precision_values(osa, gpu_ctx, dtype, narrow_y, repeatable):
    """fp16 / bf16 values and x with an fp32 y get the same default plan: the live layout reads the caller's 2-byte
    values at every call (a row block's linearly, beside the gathered x in the block's LDS window, the long rows'
    straight into the sums of their panel) and widens x as it loads a panel's slice.  Values changed in place are
    followed."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 300_000, 1_400_000
    rowptr, colind, val, x, y0 = _with_long_rows(rows, cols, 13)
    rnd = lambda a: torch.from_numpy(a).to(dtype).float().numpy()
    val, x = rnd(val), rnd(x)
    nnz = colind.size
    want = (L.opsparse_spmv_csr_blocked_workspace_bytes(
                rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES |
                (osa.OPSPARSE_BLOCKED_VALUES_F16 if dtype == torch.float16 else osa.OPSPARSE_BLOCKED_VALUES_BF16))
            if repeatable else L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz))
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    vbuf = torch.zeros(nnz + 1, dtype=dtype, device=dev)      # values at an address that is only 2-byte aligned
    d_val = vbuf[1:]
    d_val.copy_(torch.from_numpy(val).to(dtype))
    assert d_val.data_ptr() % 4 == 2
    if narrow_y:                                              # y of the values' type: the fp64 sum rounded once
        y0 = rnd(y0)
    d_x, d_y = to_dev(x, dev, dtype), to_dev(y0, dev, dtype if narrow_y else None)
    A = osa.Csr(rows, cols, d_rp, d_ci, d_val)
    op = osa.SpmvOp(handle, A, osa.DnVec(d_x), osa.DnVec(d_y))
    assert op.buffer.numel() == want
    half_ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8

    def check(values, alpha, beta):
        d_y.copy_(torch.from_numpy(y0).to(d_y.dtype))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        got = d_y.float().cpu().numpy()
        if narrow_y:
            assert np.all(np.abs(got - gold) <= 1.001 * half_ulp * np.maximum(np.abs(gold), 2.0 ** -14))
        else:
            assert oracle.max_rel_err(got, gold) <= 1e-5

    check(val, 1.0, 0.0)
    val2 = rnd((val * np.float32(-0.5) + np.float32(0.25)).astype(np.float32))
    d_val.copy_(torch.from_numpy(val2).to(dtype))
    check(val2, 1.5, -0.5)


def test_default_plan_sums_long_rows_from_the_callers_arrays(osa, gpu_ctx, repeatable):
    """Rows of 64 entries per column panel and more (4096 at least) with ascending columns are kept out of the
    re-stored layout: the workgroup that has a panel's x in LDS sums their entries of that panel straight from
    colInd / csrValues.  The analysis must find exactly those rows; the product must follow values changed in
    place, a new x, beta != 0 and y read and written in place."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 300_000, 1_400_000                          # 43 panels: the threshold is the 4096 entries
    rowptr, colind, val, x, y0 = _with_long_rows(rows, cols, 11)
    nnz = colind.size
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    # the analysis through the raw layer: which rows it took
    need = _default_bytes(osa, rows, cols, nnz, repeatable)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    analyse = L.opsparse_spmv_csr_blocked_analyse if repeatable else L.opsparse_spmv_csr_live_analyse
    assert analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES, pv(ws), need,
                   ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream)) == 0
    assert plan.kernel == (osa.OPSPARSE_SPMV_BLOCKED_GATHER if repeatable else osa.OPSPARSE_SPMV_BLOCKED_LIVE)
    assert plan.liveValues == (1 if repeatable else 2)       # (atomics: 16-bit positions, every block is short)
    assert plan.numLongRows == 6                              # 9000, 4096, 40 000, 20 000, 120 000, 5000
    del ws
    A, X = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, X, osa.DnVec(d_y))            # ALG_DEFAULT
    assert op.buffer.numel() == need

    def check(values, xv, alpha, beta):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, xv, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    check(val, x, 1.0, 0.0)
    check(val, x, -0.75, 2.0)
    val2 = (val * np.float32(3.0) - np.float32(0.125)).astype(np.float32)
    d[2].copy_(torch.from_numpy(val2))                       # in place: long and short rows alike follow
    check(val2, x, 1.0, 0.5)
    x2 = np.random.default_rng(12).uniform(-2, 2, cols).astype(np.float32)
    d[3].copy_(torch.from_numpy(x2))
    check(val2, x2, 2.0, 0.0)


@pytest.mark.parametrize("live", [True, False])
def test_many_long_rows_in_one_row_block_are_summed_by_their_own_kernel(osa, gpu_ctx, live, monkeypatch):
    """A row block's workgroup adds up the partial sums of at most 64 long rows; a block with more of them (here
    200 neighbouring rows of 4200 .. 5000 entries among short ones, and in a second matrix nothing but long rows)
    leaves them to a kernel with a wavefront a row.  That is the layout with frozen values (ALG2); with live values
    a long row ends its row block (the block's other entries are then one piece of the caller's arrays), so no block
    holds more than one.  beta != 0 with y read and written in place."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    flags = osa.OPSPARSE_BLOCKED_LIVE_VALUES if live else 0
    monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")   # the default algorithm on the ordered layout too

    def run(rows, cols, lengths, want_long, seed):
        rng = np.random.default_rng(seed)
        rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
        for r in np.nonzero(lengths >= 1024)[0]:
            colind[rowptr[r]:rowptr[r + 1]].sort()
        val = rng.uniform(-1, 1, colind.size).astype(np.float32)
        x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
        nnz = colind.size
        need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, flags)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        plan = osa.OpsparseSpmvPlan()
        assert L.opsparse_spmv_csr_blocked_analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz, flags, pv(ws), need,
                                                   ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream)) == 0
        assert plan.numLongRows == want_long and plan.numDeferredLongRows == (0 if live else want_long)
        del ws
        d_y = to_dev(y0, dev)
        op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y),
                        alg=0 if live else osa.ACL_SPARSE_SPMV_CSR_ALG2)
        for alpha, beta in ((1.0, 0.0), (-1.5, 0.75)):
            d_y.copy_(torch.from_numpy(y0))
            op(alpha, beta)
            stream.synchronize()
            gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
            assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    rows, cols = 300_000, 1_400_000                          # 43 panels: long from 4096 (live) / 1024 (frozen) entries
    rng = np.random.default_rng(41)
    lengths = rng.integers(0, 20, rows)
    lengths[5000:5200] = rng.integers(4200, 5000, 200)
    run(rows, cols, lengths, 200, 42)
    run(700, 1_300_000, np.full(700, 4500), 700, 43)         # long rows only: no entry in the row-block order


def test_a_row_too_long_for_a_row_block_keeps_the_ordinary_plan(osa, gpu_ctx, monkeypatch):
    """The place of an entry in its row block is kept in 16 bits.  A row of 70 000 entries whose columns do not
    ascend cannot go the long rows' way and does not fit a block: the analysis says so (unsupported), and
    Preprocess leaves the ordinary plan in the buffer instead; same product.  A row of 30 000 such entries fits
    (a block worked in several windows)."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")
    rows, cols = 300_000, 1_400_000
    for longest, want_rc in ((70_000, osa.OPSPARSE_E_UNSUPPORTED), (30_000, 0)):
        rng = np.random.default_rng(31)
        lengths = rng.integers(0, 20, rows)
        lengths[123_456] = longest
        rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)      # unsorted everywhere
        val = rng.uniform(-1, 1, colind.size).astype(np.float32)
        x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
        nnz = colind.size
        need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        plan = osa.OpsparseSpmvPlan()
        pv = lambda t: ctypes.c_void_p(t.data_ptr())
        assert L.opsparse_spmv_csr_blocked_analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz,
                                                   osa.OPSPARSE_BLOCKED_LIVE_VALUES, pv(ws), need, ctypes.byref(plan),
                                                   ctypes.c_void_p(stream.cuda_stream)) == want_rc
        if want_rc == 0:
            assert plan.liveValues == 1 and plan.numLongRows == 0
        del ws
        d_y = to_dev(y0, dev)
        op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y))
        for values, alpha, beta in ((val, 1.0, 0.0), ((val * np.float32(-2.0)).astype(np.float32), 0.5, 1.5)):
            d[2].copy_(torch.from_numpy(values))
            d_y.copy_(torch.from_numpy(y0))
            op(alpha, beta)
            stream.synchronize()
            gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
            assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def test_default_plan_leaves_small_matrices_to_the_merge_path(osa, gpu_ctx, monkeypatch):
    """Below 7 M entries GetBufferSize asks for the merge-path tables only, scattered gathers or not; from there on
    (and with the tuning override at any size) for the layout."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 5)
    nnz = colind.size
    assert 2_000_000 < nnz < 7_000_000
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A, X, Y = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(to_dev(y0, dev))
    layout = L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
    assert layout > 0
    monkeypatch.delenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ")
    assert osa.SpmvOp(handle, A, X, Y).buffer.numel() == L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", str(nnz))
    assert osa.SpmvOp(handle, A, X, Y).buffer.numel() == layout
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", str(nnz + 1))
    op = osa.SpmvOp(handle, A, X, Y)
    assert op.buffer.numel() == L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
    op(1.0, 0.0)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.0)
    assert oracle.max_rel_err(Y.t.cpu().numpy(), gold) <= 1e-5


def test_default_plan_of_a_banded_matrix_stays_row_wise(osa, gpu_ctx, workloads):
    """Gathers near the diagonal: the probe says local, GetBufferSize asks for the merge-path tables only."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    A = workloads.laplacian_2d(1200, dev)                   # 1.44 M columns, 7.2 M entries: the layout would apply
    rows, nnz = A["rows"], int(A["colind"].numel())
    assert L.opsparse_spmv_csr_live_workspace_bytes(rows, rows, nnz) > 0
    x = workloads.uniform(3, rows, -1.0, 1.0, dev)
    y = torch.zeros(rows, device=dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, rows, A["rowptr"], A["colind"], A["values"]), osa.DnVec(x), osa.DnVec(y))
    assert op.buffer.numel() == L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
    op(1.0, 0.0)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, rows, A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy(),
                           A["values"].cpu().numpy(), x.cpu().numpy(), None, 1.0, 0.0)
    assert oracle.max_rel_err(y.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("far,layout_default,layout_alg2", [(1, False, False), (2, False, True), (4, True, True)])
def test_a_band_with_some_random_columns_gets_the_layout_only_where_it_pays(osa, gpu_ctx, far, layout_default,
                                                                             layout_alg2):
    """Eight entries a row, `far` of them anywhere and the others within a few columns of the diagonal.  The row-wise
    kernels pay for the far gathers only, the layouts for every entry: the default plan re-stores from 31 % far
    gathers on, ALG2 (values frozen, a cheaper layout) from 19 %.  One in eight: neither; two: ALG2 only; four: both.
    Which plan ran shows in the buffer the default plan asks for and, for ALG2, in the kernel of the plan bound."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows = 1_300_000
    rng = np.random.default_rng(far)
    near = (np.arange(rows)[:, None] + rng.integers(-40, 41, (rows, 8 - far))).clip(0, rows - 1)
    cols = np.concatenate([near, rng.integers(0, rows, (rows, far))], axis=1)
    colind = np.sort(cols, axis=1).astype(np.int32).reshape(-1)
    rowptr = (np.arange(rows + 1) * 8).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    nnz = colind.size
    A, X = osa.Csr(rows, rows, d[0], d[1], d[2]), osa.DnVec(d[3])
    gold = oracle.spmv_f64(rows, rows, rowptr, colind, val, x, y0, 1.0, 0.5)
    live_bytes = L.opsparse_spmv_csr_live_workspace_bytes(rows, rows, nnz)
    assert live_bytes > 0
    for alg, want_layout in ((osa.ACL_SPARSE_SPMV_ALG_DEFAULT, layout_default), (osa.ACL_SPARSE_SPMV_CSR_ALG2, layout_alg2)):
        d_y = to_dev(y0, dev)
        op = osa.SpmvOp(handle, A, X, osa.DnVec(d_y), alg=alg)
        if alg == osa.ACL_SPARSE_SPMV_ALG_DEFAULT:
            assert (op.buffer.numel() == live_bytes) == want_layout
        op(1.0, 0.5)
        stream.synchronize()
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    # the analysis ALG2's Preprocess runs, through the raw layer: the probe's figure against its threshold
    ws = torch.zeros(256, dtype=torch.uint8, device=dev)
    flag = ctypes.c_int32(-1)
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    assert L.opsparse_spmv_csr_gathers_scattered(pv(d[0]), pv(d[1]), rows, rows, nnz, pv(ws), 256, ctypes.byref(flag),
                                                 ctypes.c_void_p(stream.cuda_stream)) == 0
    assert abs(flag.value - 125 * far * (1 - 262144 / rows)) <= 15       # (a random column is near by chance one time in five)
    assert (flag.value >= 190) == layout_alg2 and (flag.value >= 310) == layout_default


def test_alg2_plan_is_dropped_when_the_values_array_is_replaced(osa, gpu_ctx):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 6)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y), alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    op(1.0, 0.0)
    stream.synchronize()
    assert oracle.max_rel_err(d_y.cpu().numpy(),
                              oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.0)) <= 1e-5
    val2 = np.random.default_rng(10).uniform(-2, 2, colind.size).astype(np.float32)
    d_val2 = to_dev(val2, dev)
    assert L.aclsparseSpMatSetValues(A.d, ctypes.c_void_p(d_val2.data_ptr())) == 0
    d_y.copy_(torch.from_numpy(y0))
    op(2.0, 0.5)                                             # same buffer: the plan in it no longer counts
    stream.synchronize()
    assert oracle.max_rel_err(d_y.cpu().numpy(),
                              oracle.spmv_f64(rows, cols, rowptr, colind, val2, x, y0, 2.0, 0.5)) <= 1e-5


def test_alg2_layout_streams_long_rows_panel_by_panel(osa, gpu_ctx):
    """ACL_SPARSE_SPMV_CSR_ALG2 (values frozen at Preprocess): rows of 1024 entries and more with ascending
    columns leave the row-block order; a panel's workgroup streams their entries of that panel, stored a second
    time in one piece, into one fp64 accumulator a row in LDS.  Cases: the mixed matrix of the test above (rows
    either side of the threshold, first and last row, neighbours, repeated columns, an unsorted long row), and a
    matrix with more long rows than the 3072 accumulators of a tile, short rows between them."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())

    def run(rows, cols, rowptr, colind, val, x, y0, want_long):
        nnz = colind.size
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
        need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, 0)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        plan = osa.OpsparseSpmvPlan()
        assert L.opsparse_spmv_csr_blocked_analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz, 0, pv(ws), need,
                                                   ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream)) == 0
        assert plan.liveValues == 0 and plan.numLongRows == want_long
        del ws
        d_y = to_dev(y0, dev)
        op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y),
                        alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
        for alpha, beta, xv in ((1.0, 0.0, x), (-0.75, 2.0, x),
                                (2.0, 0.5, np.random.default_rng(5).uniform(-2, 2, cols).astype(np.float32))):
            d[3].copy_(torch.from_numpy(xv))
            d_y.copy_(torch.from_numpy(y0))
            op(alpha, beta)
            stream.synchronize()
            gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, xv, y0, alpha, beta)
            assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    rows, cols = 300_000, 1_400_000
    # 9000, 4096, 4095, 40 000, 20 000, 120 000, 5000 (the 6000 of row 200 000 do not ascend)
    run(rows, cols, *_with_long_rows(rows, cols, 11), want_long=7)

    rng = np.random.default_rng(21)
    rows, cols = 120_000, 1_200_000
    lengths = rng.integers(0, 12, rows)
    long_at = rng.choice(rows, 3500, replace=False)
    lengths[long_at] = rng.integers(1024, 1400, long_at.size)
    lengths[long_at[:40]] = 1023                             # one short of the threshold
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    for r in long_at:
        colind[rowptr[r]:rowptr[r + 1]].sort()
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    run(rows, cols, rowptr, colind, val, rng.uniform(-1, 1, cols).astype(np.float32),
        rng.uniform(-1, 1, rows).astype(np.float32), want_long=3460)


def test_a_layout_is_only_built_into_a_buffer_that_a_size_query_sized(osa, gpu_ctx):
    """A caller may size the buffer from any earlier answer it trusts (the reference's SpMVOp answers 0 for ALG1,
    spmv_op_host.cpp:152-160) or skip the query: Preprocess / createDescr then get a buffer with room for the
    ordinary plan only.  The library builds a re-stored layout only where a size query ON THESE ARRAYS answered
    that layout's bytes: without one, the ordinary plan goes into the buffer and nothing is written behind it."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 8)
    nnz = colind.size
    plain = L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
    assert 0 < plain < L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.5)
    guard = 1 << 16

    def fresh():
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]   # new arrays: no query has seen them
        buf = torch.full((plain + guard,), 0xA5, dtype=torch.uint8, device=dev)
        return d, osa.Csr(rows, cols, d[0], d[1], d[2]), buf

    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    for alg in (osa.ACL_SPARSE_SPMV_ALG_DEFAULT, osa.ACL_SPARSE_SPMV_CSR_ALG2):
        d, A, buf = fresh()
        X, d_y = osa.DnVec(d[3]), to_dev(y0, dev)
        Y = osa.DnVec(d_y)
        assert L.aclsparseSpMVPreprocess(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, alg, pv(buf)) == 0
        stream.synchronize()
        assert bool((buf[plain:] == 0xA5).all())
        one, half = ctypes.c_float(1.0), ctypes.c_float(0.5)
        assert L.aclsparseSpMV(handle.h, 0, ctypes.byref(one), A.d, X.d, ctypes.byref(half), Y.d, osa.ACL_FLOAT, alg,
                               pv(buf)) == 0
        stream.synchronize()
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
        # a query for ANOTHER algorithm's layout does not count either: the default query, then an ALG2 Preprocess
        if alg == osa.ACL_SPARSE_SPMV_CSR_ALG2:
            n = ctypes.c_size_t(0)
            assert L.aclsparseSpMVGetBufferSize(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT,
                                                osa.ACL_SPARSE_SPMV_ALG_DEFAULT, ctypes.byref(n)) == 0
            assert n.value == L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
            assert L.aclsparseSpMVPreprocess(handle.h, 0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, alg, pv(buf)) == 0
            stream.synchronize()
            assert bool((buf[plain:] == 0xA5).all())
    for alg in (osa.ACL_SPARSE_SPMVOP_ALG1, osa.ACL_SPARSE_SPMVOP_ALG2):
        d, A, buf = fresh()
        X, d_y = osa.DnVec(d[3]), to_dev(y0, dev)
        Y = osa.DnVec(d_y)
        descr, plan = ctypes.c_void_p(), ctypes.c_void_p()
        assert L.aclsparseSpMVOp_createDescr(handle.h, ctypes.byref(descr), 0, A.d, X.d, Y.d, Y.d, osa.ACL_FLOAT, alg,
                                             pv(buf)) == 0
        assert L.aclsparseSpMVOp_createPlan(handle.h, descr, ctypes.byref(plan), None, 0) == 0
        one, half = ctypes.c_float(1.0), ctypes.c_float(0.5)
        assert L.aclsparseSpMVOp(handle.h, plan, ctypes.byref(one), ctypes.byref(half), X.d, Y.d, Y.d) == 0
        stream.synchronize()
        assert bool((buf[plain:] == 0xA5).all())
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
        L.aclsparseSpMVOp_destroyPlan(plan)
        L.aclsparseSpMVOp_destroyDescr(descr)


def _value_flag(osa, dtype):
    return {torch.float32: 0, torch.float16: osa.OPSPARSE_BLOCKED_VALUES_F16,
            torch.bfloat16: osa.OPSPARSE_BLOCKED_VALUES_BF16, torch.int32: osa.OPSPARSE_BLOCKED_VALUES_I32}[dtype]


@pytest.mark.parametrize("dtype,narrow_y", [(torch.float32, False), (torch.float16, False), (torch.float16, True),
                                            (torch.bfloat16, True)])
def test_default_plan_for_the_transposed_product(osa, gpu_ctx, dtype, narrow_y):
    """y = alpha * A^T x + beta * y with the default algorithm on a matrix whose updates of y are scattered:
    Preprocess transposes A into the buffer, keeps for every entry of the copy where its value sits in csrValues,
    and every call refreshes the copy's values from the caller's array before it runs the ordered kernels (no atomics
    on y).  Values changed in place and a replaced values array are followed; the transposed plan does not serve
    op(A) = A (that call runs without it, same buffer)."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 1_400_000, 300_000                          # A^T: 300 000 rows, x of 1.4 M elements
    rng = np.random.default_rng(17)
    lengths = rng.integers(0, 5, rows)
    lengths[[11, rows // 2]] = [30_000, 9_000]               # long rows of A: columns of A^T that hit many rows
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    colind[:6000] = 77                                       # a column of A with 6000 entries: a long row of A^T
    nnz = colind.size
    rnd = lambda a: torch.from_numpy(a).to(dtype).float().numpy()
    val, x = rnd(rng.uniform(-1, 1, nnz).astype(np.float32)), rnd(rng.uniform(-1, 1, rows).astype(np.float32))
    y0 = rng.uniform(-1, 1, cols).astype(np.float32)
    if narrow_y:
        y0 = rnd(y0)
    want = L.opsparse_spmv_csr_blocked_workspace_bytes(
        rows, cols, nnz, osa.OPSPARSE_BLOCKED_TRANSPOSE | osa.OPSPARSE_BLOCKED_LIVE_VALUES | _value_flag(osa, dtype))
    assert want > 0
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val, d_x = to_dev(val, dev, dtype), to_dev(x, dev, dtype)
    d_y = to_dev(y0, dev, dtype if narrow_y else None)
    A = osa.Csr(rows, cols, d_rp, d_ci, d_val)
    op = osa.SpmvOp(handle, A, osa.DnVec(d_x), osa.DnVec(d_y), op=osa.ACL_SPARSE_OP_TRANSPOSE)
    staging = 0 if not narrow_y else cols * 4                # (the fp32 staging vector of the atomics path, unused here)
    assert want <= op.buffer.numel() <= want + 256 + staging
    half_ulp = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}.get(dtype)

    def check(values, alpha, beta):
        d_y.copy_(torch.from_numpy(y0).to(d_y.dtype))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        got = d_y.float().cpu().numpy()
        if narrow_y:
            assert np.all(np.abs(got - gold) <= 1.001 * half_ulp * np.maximum(np.abs(gold), 2.0 ** -14))
        else:
            assert oracle.max_rel_err(got, gold) <= 1e-5     # fp64 sums rounded once: the bar of op(A) = A

    check(val, 1.0, 0.0)
    first = d_y.clone()
    check(val, 1.0, 0.0)
    assert torch.equal(first, d_y)
    val2 = rnd((val * np.float32(-0.5) + np.float32(0.25)).astype(np.float32))
    d_val.copy_(torch.from_numpy(val2).to(dtype))
    check(val2, 1.5, -0.5)
    val3 = rnd(np.random.default_rng(3).uniform(-3, 3, nnz).astype(np.float32))
    d_val3 = to_dev(val3, dev, dtype)
    assert L.aclsparseSpMatSetValues(A.d, ctypes.c_void_p(d_val3.data_ptr())) == 0
    check(val3, -1.0, 0.0)
    # the other op(A) on the same descriptor and buffer
    d_xn, d_yn = to_dev(rnd(y0), dev, dtype), torch.zeros(rows, dtype=torch.float32, device=dev)
    opn = osa.SpmvOp(handle, A, osa.DnVec(d_xn), osa.DnVec(d_yn), preprocess=False)
    opn.buffer = op.buffer
    opn(1.0, 0.0)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val3, rnd(y0), None, 1.0, 0.0)
    assert oracle.max_rel_err(d_yn.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("int_compute", [True, False])
def test_default_plan_with_int32_values(osa, gpu_ctx, transpose, int_compute):
    """int32 values and x.  Under the integer compute type y is int32 and the sums wrap around (bit for bit the
    oracle's, whatever the order); under ACL_FLOAT y is fp32 and the sums are fp64 of the exactly converted operands.
    Both get the ordered layout with live values."""
    import scipy.sparse as sp
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = (1_400_000, 300_000) if transpose else (300_000, 1_400_000)
    rng = np.random.default_rng(23 + transpose)
    lengths = rng.integers(0, 5 if transpose else 20, rows)
    lengths[[5, rows // 3]] = [40_000, 5_000]
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    for r in (5, rows // 3):
        colind[rowptr[r]:rowptr[r + 1]].sort()
    nnz = colind.size
    big = 50_000 if int_compute else 2_000                   # products wrap in the integer sums
    val = rng.integers(-big, big, nnz).astype(np.int32)
    n_x, n_y = (rows, cols) if transpose else (cols, rows)
    x = rng.integers(-big, big, n_x).astype(np.int32)
    y0 = rng.integers(-1000, 1000, n_y).astype(np.int32) if int_compute else rng.uniform(-1, 1, n_y).astype(np.float32)
    want = L.opsparse_spmv_csr_blocked_workspace_bytes(
        rows, cols, nnz, (osa.OPSPARSE_BLOCKED_TRANSPOSE if transpose else 0) | osa.OPSPARSE_BLOCKED_LIVE_VALUES |
        osa.OPSPARSE_BLOCKED_VALUES_I32)
    assert want > 0
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    op = osa.SpmvOp(handle, A, osa.DnVec(d[3]), osa.DnVec(d_y),
                    op=osa.ACL_SPARSE_OP_TRANSPOSE if transpose else osa.ACL_SPARSE_OP_NON_TRANSPOSE,
                    compute_type=osa.ACL_INT32 if int_compute else osa.ACL_FLOAT)
    assert op.buffer.numel() == want

    def check(values, alpha, beta):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        if transpose:                                        # the oracle's op(A) = A on the transposed arrays
            t = sp.csr_matrix((values, colind, rowptr), shape=(rows, cols)).tocsc()
            rp, ci, va = t.indptr.astype(np.int32), t.indices.astype(np.int32), t.data.astype(np.int32)
        else:
            rp, ci, va = rowptr, colind, values
        if int_compute:
            assert np.array_equal(d_y.cpu().numpy(), oracle.spmv_i32(n_y, rp, ci, va, x, y0, alpha, beta))
        else:
            gold = oracle.spmv_f64(n_y, n_x, rp, ci, va.astype(np.float32), x.astype(np.float32), y0, alpha, beta)
            assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    check(val, *((3, -2) if int_compute else (0.5, 1.0)))
    val2 = rng.integers(-big, big, nnz).astype(np.int32)
    d[2].copy_(torch.from_numpy(val2))                       # in place: followed
    check(val2, *((-1, 0) if int_compute else (1.0, 0.0)))


@pytest.mark.parametrize("how", ["switch", "long_block"])
def test_atomics_layout_with_32_bit_positions(osa, gpu_ctx, how, monkeypatch):
    """The atomics layout keeps where every entry sits in its row block in 16 bits when every block is shorter than
    65 535 positions, else in 32: asked for by the switch, and forced by a row of 70 000 entries whose columns do not
    ascend (it cannot go the long rows' way and makes one block that long).  Same products either way."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 300_000, 1_400_000
    rng = np.random.default_rng(37)
    lengths = rng.integers(0, 20, rows)
    if how == "long_block":
        lengths[123_456] = 70_000
    else:
        monkeypatch.setenv("OPS_SPARSE_BLOCKED_NO_SHORT_POSITIONS", "1")
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    nnz = colind.size
    need = L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    assert L.opsparse_spmv_csr_live_analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz, 0, pv(ws), need,
                                            ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream)) == 0
    assert plan.kernel == osa.OPSPARSE_SPMV_BLOCKED_LIVE and plan.liveValues == 1
    del ws
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y))
    assert op.buffer.numel() == need
    for values, alpha, beta in ((val, 1.0, 0.0), ((val * np.float32(-2.0)).astype(np.float32), 0.5, 1.5)):
        d[2].copy_(torch.from_numpy(values))
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, values, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def test_ordered_live_layout_only_where_x_is_out_of_reach_of_the_caches(osa, gpu_ctx, monkeypatch):
    """The layout with live values and ordered sums (aclsparseSpMVOp DEFAULT / ALG1, and the default algorithm asked
    for repeatable sums) is slower than the one with atomics; against the row-wise kernels it pays from 2.6 M
    columns on.  Below that aclsparseSpMVOp_bufferSize answers 0 for these algorithms, as the reference does."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 5)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    A = osa.Csr(rows, cols, d[0], d[1], d[2])
    d_y = to_dev(y0, dev)
    Y = osa.DnVec(d_y)
    monkeypatch.delenv("OPS_SPARSE_ORDERED_LIVE_MIN_COLS")
    op = osa.SpmvOpPlan(handle, A, osa.DnVec(d[3]), Y, Y)
    assert op.buffer_bytes == 0
    op(1.0, 0.5)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.0, 0.5)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5
    monkeypatch.setenv("OPS_SPARSE_SPMV_REPEATABLE", "1")
    plain = L.opsparse_spmv_csr_workspace_bytes(rows, colind.size)
    assert osa.SpmvOp(handle, A, osa.DnVec(d[3]), Y).buffer.numel() == plain
    monkeypatch.setenv("OPS_SPARSE_ORDERED_LIVE_MIN_COLS", str(cols))
    assert osa.SpmvOp(handle, A, osa.DnVec(d[3]), Y).buffer.numel() > plain


@pytest.mark.parametrize("alg_name", ["default", "alg2", "spmvop_default"])
def test_buffer_holds_only_what_the_calls_keep_when_the_handle_lends_the_scratch(osa, gpu_ctx, alg_name):
    """Two thirds of what a layout's analysis needs is scratch.  A handle that was given a workspace with room for it
    (aclsparseSetWorkspace) lends it to Preprocess / createDescr, and the size query then only asks the caller for
    what the later calls keep; without such a workspace the query asks for everything, as before.  Same products;
    nothing is written behind the smaller buffer; a handle whose workspace went away between the query and
    Preprocess gets the ordinary plan."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = 320_000, 1_500_000
    rowptr, colind, val, x, y0 = _scattered(rows, cols, 15)
    nnz = colind.size
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, -0.5)
    if alg_name == "alg2":
        whole = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, 0)
        keep = L.opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz, 0)
    elif alg_name == "default":
        whole = L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
        keep = L.opsparse_spmv_csr_live_resident_bytes(rows, cols, nnz)
    else:
        whole = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
        keep = L.opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz, osa.OPSPARSE_BLOCKED_LIVE_VALUES)
    assert 0 < keep < whole
    lent = torch.empty(whole - keep, dtype=torch.uint8, device=dev)
    guard = 1 << 16

    def product(buffer_bytes, expect_layout):
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
        A = osa.Csr(rows, cols, d[0], d[1], d[2])
        d_y = to_dev(y0, dev)
        X, Y = osa.DnVec(d[3]), osa.DnVec(d_y)
        one, half = ctypes.c_float(1.5), ctypes.c_float(-0.5)
        n = ctypes.c_size_t(0)
        if alg_name == "spmvop_default":
            common = (0, A.d, X.d, Y.d, Y.d, osa.ACL_FLOAT, osa.ACL_SPARSE_SPMVOP_ALG_DEFAULT)
            assert L.aclsparseSpMVOp_bufferSize(handle.h, *common, ctypes.byref(n)) == 0
        else:
            alg = osa.ACL_SPARSE_SPMV_CSR_ALG2 if alg_name == "alg2" else osa.ACL_SPARSE_SPMV_ALG_DEFAULT
            common = (0, None, A.d, X.d, None, Y.d, osa.ACL_FLOAT, alg)
            assert L.aclsparseSpMVGetBufferSize(handle.h, *common, ctypes.byref(n)) == 0
        assert n.value == buffer_bytes
        buf = torch.full((n.value + guard,), 0x77, dtype=torch.uint8, device=dev)
        pbuf = ctypes.c_void_p(buf.data_ptr())
        return d, A, X, Y, d_y, one, half, common, buf, pbuf, n.value

    def run(state):
        d, A, X, Y, d_y, one, half, common, buf, pbuf, size = state
        if alg_name == "spmvop_default":
            descr, plan = ctypes.c_void_p(), ctypes.c_void_p()
            assert L.aclsparseSpMVOp_createDescr(handle.h, ctypes.byref(descr), *common, pbuf) == 0
            assert L.aclsparseSpMVOp_createPlan(handle.h, descr, ctypes.byref(plan), None, 0) == 0
            assert L.aclsparseSpMVOp(handle.h, plan, ctypes.byref(one), ctypes.byref(half), X.d, Y.d, Y.d) == 0
            stream.synchronize()
            L.aclsparseSpMVOp_destroyPlan(plan)
            L.aclsparseSpMVOp_destroyDescr(descr)
        else:
            assert L.aclsparseSpMVPreprocess(handle.h, *common, pbuf) == 0
            assert L.aclsparseSpMV(handle.h, 0, ctypes.byref(one), A.d, X.d, ctypes.byref(half), Y.d, osa.ACL_FLOAT,
                                   common[-1], pbuf) == 0
            stream.synchronize()
        assert bool((buf[size:] == 0x77).all())
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5

    try:
        run(product(whole, True))                              # no workspace of the user's: everything in the buffer
        assert L.aclsparseSetWorkspace(handle.h, ctypes.c_void_p(lent.data_ptr()), lent.numel()) == 0
        run(product(keep, True))                               # the scratch is lent: the buffer keeps the layout only
        state = product(keep, True)
        assert L.aclsparseSetWorkspace(handle.h, None, 0) == 0  # ... and taken away again before Preprocess
        run(state)                                             # the ordinary plan, inside the smaller buffer
    finally:
        L.aclsparseSetWorkspace(handle.h, None, 0)
