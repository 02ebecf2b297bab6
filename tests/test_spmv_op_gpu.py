"""GPU parity tests for the aclsparseSpMVOp_* API (descriptor + plan, Z = alpha*A*X + beta*Y).

The case table is the reference's own (test/spmv_op/arch35/spmv_op_test.csv, kept as
the data fixture tests/golden/spmv_op_cases.csv) and every row is run the way
test/spmv_op/arch35/spmv_op_test.cpp:50-142 runs it: matrix from the reference's
fill generator (values in [-5, 5]), X / Y from makeDenseFloat(-3, 3, seed + 1 / + 2),
fp64 golden, MERE / MARE thresholds from the row.  The matrix generator with a
sparsity (binomial row lengths) is only available through the compiled oracle/_ref
helper; where that is absent a numpy generator of the same distribution stands in
(same shapes and statistics, different entries).

Tolerance (fp32): per element |d| <= 1e-5 * |oracle| against the fp64-accumulated
oracle, plus the row's own MERE / MARE limits.
"""
import csv
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import csr_from_lengths, random_csr, to_dev

pytestmark = pytest.mark.gpu

RTOL = 1e-5
HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "spmv_op_cases.csv")) as f:
    CASES = list(csv.DictReader(f))


def build_csr(c):
    m, k, seed = int(c["m"]), int(c["k"]), int(c["seed"])
    if c["pattern"] == "diag":
        return np.arange(m + 1, dtype=np.int32), np.arange(m, dtype=np.int32), np.ones(m, np.float32)
    if c["pattern"] == "empty" or m <= 0 or k <= 0:
        return np.zeros(max(m, 0) + 1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32)
    sparsity, erp = float(c["sparsity"]), float(c["empty_row_prob"])
    got = oracle.ref_fill_csr(seed, m, k, -1, sparsity, erp, -5.0, 5.0)
    if got is None:
        got = random_csr(m, k, 1.0 - sparsity, seed, -5.0, 5.0, empty_row_prob=erp)
    rowptr, colind, val = got
    if int(c["unsorted"]):
        rng = np.random.default_rng(seed)
        colind, val = colind.copy(), val.copy()
        for r in range(m):
            lo, hi = rowptr[r], rowptr[r + 1]
            perm = rng.permutation(hi - lo)
            colind[lo:hi], val[lo:hi] = colind[lo:hi][perm], val[lo:hi][perm]
    return rowptr, colind, val


def run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, y, alpha, beta, mode="HOST", i64=False, alias=False,
           alg=0, base=0):
    """One createDescr / createPlan / execute / destroy cycle; returns Z (and checks Y is untouched)."""
    dev, stream, handle = gpu_ctx
    rp = (rowptr.astype(np.int64) if i64 else rowptr) + base
    d_rp, d_ci, d_val = to_dev(rp, dev), to_dev(colind + base, dev), to_dev(val, dev)
    d_x, d_y = to_dev(x, dev), to_dev(y, dev)
    d_z = d_y if alias else torch.full((m,), float("nan"), dtype=torch.float32, device=dev)
    A = osa.Csr(m, k, d_rp, d_ci, d_val, index_base=base)
    X, Y = osa.DnVec(d_x), osa.DnVec(d_y)
    Z = Y if alias else osa.DnVec(d_z)
    if mode == "DEVICE":
        handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_DEVICE)
    try:
        op = osa.SpmvOpPlan(handle, A, X, Y, Z, alg=alg)
        if mode == "DEVICE":
            scal = torch.tensor([alpha, beta], dtype=torch.float32, device=dev)
            torch.cuda.synchronize()
            op(scal[0:1], scal[1:2])
        else:
            op(alpha, beta)
        stream.synchronize()
        op.close()
    finally:
        handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_HOST)
    if not alias:
        assert np.array_equal(d_y.cpu().numpy(), y)
    assert np.array_equal(d_x.cpu().numpy(), x) and np.array_equal(d_val.cpu().numpy(), val)
    return d_z.cpu().numpy()


def check(z, m, k, rowptr, colind, val, x, y, alpha, beta, mere_t=1e-6, mare_mult=5.0):
    gold = oracle.spmv_f64(m, k, rowptr, colind, val, x, y, float(np.float32(alpha)), float(np.float32(beta)))
    assert z.shape == (m,)
    if m == 0:
        return
    err = oracle.max_rel_err(z, gold)
    assert err <= RTOL, "max rel err %.3e" % err
    mere, mare, mism, _ = oracle.mere_mare(z, gold)
    assert mism == 0 and mere < mere_t and mare < mere_t * mare_mult, (mere, mare)


@pytest.mark.parametrize("c", CASES, ids=[c["case_name"] for c in CASES])
def test_reference_case_table(osa, gpu_ctx, c):
    assert c["expect_result"] == "SUCCESS"
    m, k, seed = int(c["m"]), int(c["k"]), int(c["seed"])
    alpha, beta = float(c["alpha"]), float(c["beta"])
    rowptr, colind, val = build_csr(c)
    x = oracle.fill_dense(seed + 1, k, -3.0, 3.0) if k > 0 else np.zeros(0, np.float32)
    y = oracle.fill_dense(seed + 2, m, -3.0, 3.0) if m > 0 else np.zeros(0, np.float32)
    alg = {"DEFAULT": osa.ACL_SPARSE_SPMVOP_ALG_DEFAULT, "ALG1": osa.ACL_SPARSE_SPMVOP_ALG1,
           "ALG2": osa.ACL_SPARSE_SPMVOP_ALG2}[c["alg"]]
    z = run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, y, alpha, beta, mode=c["pointer_mode"],
               i64=(c["row_offset_type"] == "i64"), alias=bool(int(c["alias_z_y"])), alg=alg)
    check(z, m, k, rowptr, colind, val, x, y, alpha, beta, float(c["mere_threshold"]), float(c["mare_multiplier"]))


def _problem(m, k, density, seed, **kw):
    rowptr, colind, val = random_csr(m, k, density, seed, **kw)
    rng = np.random.default_rng(seed + 1)
    return rowptr, colind, val, rng.uniform(-3, 3, k).astype(np.float32), rng.uniform(-3, 3, m).astype(np.float32)


@pytest.mark.parametrize("i64", [False, True])
@pytest.mark.parametrize("alg", [1, 2])
@pytest.mark.parametrize("mode", ["HOST", "DEVICE"])
def test_index_base_one(osa, gpu_ctx, i64, alg, mode):
    """One-based row offsets and column indices (spmv_op_host.cpp:585-592; kernel: spmv_op_kernel.cpp:139-181)."""
    m, k = 3001, 2500
    rowptr, colind, val, x, y = _problem(m, k, 0.01, 17, empty_row_prob=0.2)
    z = run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, y, 1.5, -0.25, mode=mode, i64=i64, alg=alg, base=1)
    check(z, m, k, rowptr, colind, val, x, y, 1.5, -0.25)
    za = run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, y, 1.5, -0.25, mode=mode, i64=i64, alg=alg, base=1,
                alias=True)
    assert np.array_equal(z, za)


@pytest.mark.parametrize("alg", [1, 2])
@pytest.mark.parametrize("shape", ["short", "medium", "skewed"])
def test_every_kernel_family_with_separate_z(osa, gpu_ctx, alg, shape):
    """Row-length mixes that send the dispatcher to each kernel family, with Z != Y, Z == Y and beta == 0 over a
    NaN-filled Y (Y must not be read)."""
    m, k = 20000, 20000
    rng = np.random.default_rng(5)
    if shape == "short":
        lengths = rng.integers(0, 9, m)
    elif shape == "medium":
        lengths = rng.integers(40, 90, m)
    else:
        lengths = rng.integers(0, 6, m)
        lengths[rng.integers(0, m, 5)] = 15000
    from helpers import csr_from_lengths
    rowptr, colind, val = csr_from_lengths(lengths, k, 8, -5.0, 5.0)
    x = rng.uniform(-3, 3, k).astype(np.float32)
    y = rng.uniform(-3, 3, m).astype(np.float32)
    for alias in (False, True):
        z = run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, y, 2.0, 0.5, alg=alg, alias=alias)
        check(z, m, k, rowptr, colind, val, x, y, 2.0, 0.5)
    ynan = np.full(m, np.nan, np.float32)
    dev, stream, handle = gpu_ctx
    z = run_op(osa, gpu_ctx, m, k, rowptr, colind, val, x, ynan, 1.0, 0.0, alg=alg, alias=True)
    check(z, m, k, rowptr, colind, val, x, np.zeros(m, np.float32), 1.0, 0.0)


@pytest.mark.parametrize("alg", [1, 2])
def test_plan_reuse_new_values_and_vectors(osa, gpu_ctx, alg):
    """One descriptor / plan executed many times: new alpha / beta, new matrix values behind the same pattern
    (include/cann_ops_sparse.h:57-69 of the reference promises this), other vector descriptors; bitwise repeatable."""
    dev, stream, handle = gpu_ctx
    m, k = 6000, 5000
    rowptr, colind, val, x, y = _problem(m, k, 0.004, 23)
    d_rp, d_ci, d_val = to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev)
    d_x, d_y = to_dev(x, dev), to_dev(y, dev)
    d_z = torch.zeros(m, dtype=torch.float32, device=dev)
    A = osa.Csr(m, k, d_rp, d_ci, d_val)
    X, Y, Z = osa.DnVec(d_x), osa.DnVec(d_y), osa.DnVec(d_z)
    op = osa.SpmvOpPlan(handle, A, X, Y, Z, alg=alg)
    assert (op.buffer_bytes > 0) == (alg == 2)
    first = None
    for alpha, beta in ((1.0, 1.0), (-2.0, 0.5), (1.0, 1.0)):
        op(alpha, beta)
        stream.synchronize()
        z = d_z.cpu().numpy()
        check(z, m, k, rowptr, colind, val, x, y, alpha, beta)
        if (alpha, beta) == (1.0, 1.0):
            first = z if first is None else first
            assert np.array_equal(z, first)
    val2 = (val * 0.5 + 1.0).astype(np.float32)
    d_val.copy_(torch.from_numpy(val2))
    x2 = (x[::-1] * 1.25).astype(np.float32).copy()
    d_x2, d_z2 = to_dev(x2, dev), torch.zeros(m, dtype=torch.float32, device=dev)
    X2, Z2 = osa.DnVec(d_x2), osa.DnVec(d_z2)
    torch.cuda.synchronize()
    op(0.75, -1.0, x=X2, z=Z2)
    stream.synchronize()
    check(d_z2.cpu().numpy(), m, k, rowptr, colind, val2, x2, y, 0.75, -1.0)
    op.close()


def test_raw_indexed_launch_matches_plain(osa, gpu_ctx):
    """The index-variant kernel of the raw layer against the plain one on the same matrix: equal within 1e-6."""
    import ctypes
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    m, k = 5000, 7000
    rowptr, colind, val, x, y = _problem(m, k, 0.003, 31)
    nnz = colind.size
    d_ci1, d_val, d_x, d_y = to_dev(colind + 1, dev), to_dev(val, dev), to_dev(x, dev), to_dev(y, dev)
    d_rp64 = to_dev(rowptr.astype(np.int64) + 1, dev)
    d_z = torch.zeros(m, dtype=torch.float32, device=dev)
    sa, sb = osa.OpsparseScalar(1.5, None, 0, 0), osa.OpsparseScalar(0.5, None, 0, 0)
    sp = ctypes.c_void_p(stream.cuda_stream)
    torch.cuda.synchronize()
    rc = L.opsparse_spmv_csr_indexed_launch(d_rp64.data_ptr(), 1, 1, d_ci1.data_ptr(), d_val.data_ptr(),
                                            d_x.data_ptr(), d_y.data_ptr(), d_z.data_ptr(), m, k, nnz, sa, sb, sp)
    assert rc == 0
    stream.synchronize()
    check(d_z.cpu().numpy(), m, k, rowptr, colind, val, x, y, 1.5, 0.5)
    assert L.opsparse_spmv_csr_indexed_launch(d_rp64.data_ptr(), 1, 2, d_ci1.data_ptr(), d_val.data_ptr(),
                                              d_x.data_ptr(), d_y.data_ptr(), d_z.data_ptr(), m, k, nnz, sa, sb,
                                              sp) == -1


@pytest.mark.parametrize("shape", ["short_rows", "even_rows", "skewed_rows"])
def test_alg1_repeated_executions_and_value_updates(osa, gpu_ctx, shape):
    """ALG1 supports changing csrValues under a live descriptor (reference include/cann_ops_sparse.h:58-63).  The
    first execution looks at the row lengths and later ones run the kernel they select (short rows: stream rows,
    even long rows: vector rows, skewed: the merge path every time); every execution must match the oracle on the
    values of that moment, with other calls using the handle's workspace in between."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(17)
    m, k = 50_000, 60_000
    if shape == "short_rows":
        lengths = rng.integers(0, 9, m)
    elif shape == "even_rows":
        lengths = rng.integers(60, 90, m)
    else:
        lengths = np.minimum((rng.pareto(1.1, m) * 2).astype(np.int64), 20_000)
        lengths[7] = 20_000
    rowptr, colind, val = csr_from_lengths(lengths, k, 23)
    x, y = rng.uniform(-1, 1, k).astype(np.float32), rng.uniform(-1, 1, m).astype(np.float32)
    d_rp, d_ci, d_val, d_x, d_y = (to_dev(a, dev) for a in (rowptr, colind, val, x, y))
    d_z = torch.zeros(m, dtype=torch.float32, device=dev)
    A = osa.Csr(m, k, d_rp, d_ci, d_val)
    op = osa.SpmvOpPlan(handle, A, osa.DnVec(d_x), osa.DnVec(d_y), osa.DnVec(d_z), alg=osa.ACL_SPARSE_SPMVOP_ALG1)
    # another user of the handle's workspace between the executions
    o_rp, o_ci, o_val = csr_from_lengths(np.minimum((rng.pareto(1.0, 3000) * 3).astype(np.int64), 2500), 4000, 29)
    o_x = rng.uniform(-1, 1, 4000).astype(np.float32)
    d_o = [to_dev(a, dev) for a in (o_rp, o_ci, o_val, o_x)]
    d_oy = torch.zeros(3000, dtype=torch.float32, device=dev)
    other = osa.SpmvOp(handle, osa.Csr(3000, 4000, d_o[0], d_o[1], d_o[2]), osa.DnVec(d_o[3]), osa.DnVec(d_oy),
                       preprocess=False)
    for step in range(4):
        if step:
            val = (val * np.float32(-0.5) + np.float32(0.125 * step)).astype(np.float32)
            d_val.copy_(torch.from_numpy(val))
        d_z.zero_()
        op(1.5, -0.25)
        stream.synchronize()
        check(d_z.cpu().numpy(), m, k, rowptr, colind, val, x, y, 1.5, -0.25)
        other(1.0, 0.0)
        stream.synchronize()
        assert oracle.max_rel_err(d_oy.cpu().numpy(),
                                  oracle.spmv_f64(3000, 4000, o_rp, o_ci, o_val, o_x, np.zeros(3000, np.float32),
                                                  1.0, 0.0)) <= 1e-5
    op.close()


@pytest.mark.parametrize("alias", [False, True])
def test_alg1_short_rows_with_long_ones_beside(osa, gpu_ctx, alias):
    """ALG1 on short rows with a few long ones: after the first execution the stream-rows tiles run with the long
    rows summed beside them by a second kernel; Z separate from Y and Z aliasing Y must both see every row written
    exactly once (beta != 0)."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(31)
    m = k = 120_000
    lengths = rng.integers(2, 7, m)
    lengths[[0, 500, 60_000, 119_999]] = [2_000, 65, 7_000, 300]
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = np.clip(np.repeat(np.arange(m), lengths) + rng.integers(-900, 901, int(rowptr[-1])), 0, k - 1).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y = rng.uniform(-1, 1, k).astype(np.float32), rng.uniform(-1, 1, m).astype(np.float32)
    d_rp, d_ci, d_val, d_x, d_y = (to_dev(a, dev) for a in (rowptr, colind, val, x, y))
    d_z = d_y if alias else torch.zeros(m, dtype=torch.float32, device=dev)
    Y = osa.DnVec(d_y)
    Z = Y if alias else osa.DnVec(d_z)
    op = osa.SpmvOpPlan(handle, osa.Csr(m, k, d_rp, d_ci, d_val), osa.DnVec(d_x), Y, Z, alg=osa.ACL_SPARSE_SPMVOP_ALG1)
    for step in range(3):                       # the first execution takes the statistics, the others use them
        d_y.copy_(torch.from_numpy(y))
        op(1.25, -0.5)
        stream.synchronize()
        check(d_z.cpu().numpy(), m, k, rowptr, colind, val, x, y, 1.25, -0.5)
    op.close()


def test_index_variants_run_the_binned_kernels(osa, gpu_ctx, workloads):
    """64-bit row offsets and index base 1 on a power-law matrix (rows up to 20 000 entries): same result as the
    32-bit zero-based descriptor to 1e-5 against the oracle, and no load-imbalance penalty — the calls take about
    as long (a lane group per row, the kernel these variants used to get, is several times slower here)."""
    import torch
    dev, stream, handle = gpu_ctx
    m = 400_000
    A = workloads.power_law_csr(m, m, 2.0, 1, 20_000, 77, dev)
    nnz = int(A["colind"].numel())
    x = workloads.uniform(78, m, -1.0, 1.0, dev)
    y0 = workloads.uniform(79, m, -1.0, 1.0, dev)
    gold = oracle.spmv_f64(m, m, A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy(), A["values"].cpu().numpy(),
                           x.cpu().numpy(), y0.cpu().numpy(), 1.5, -0.5)
    X, Y = osa.DnVec(x), osa.DnVec(y0)
    times = {}
    for name, rowptr, colind, base in (
            ("i32", A["rowptr"], A["colind"], osa.ACL_SPARSE_INDEX_BASE_ZERO),
            ("i64", A["rowptr"].to(torch.int64), A["colind"], osa.ACL_SPARSE_INDEX_BASE_ZERO),
            ("i64 base 1", A["rowptr"].to(torch.int64) + 1, A["colind"] + 1, osa.ACL_SPARSE_INDEX_BASE_ONE)):
        z = torch.zeros(m, device=dev)
        op = osa.SpmvOpPlan(handle, osa.Csr(m, m, rowptr, colind, A["values"], index_base=base), X, Y, osa.DnVec(z))
        op(1.5, -0.5)
        stream.synchronize()
        assert oracle.max_rel_err(z.cpu().numpy(), gold) <= 1e-5, name
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(20):
            op(1.5, -0.5)
        e1.record(stream)
        stream.synchronize()
        times[name] = e0.elapsed_time(e1) / 20
        op.close()
    print("SpMVOp per call, ms:", {k: round(v, 4) for k, v in times.items()})
    assert times["i64"] <= 1.5 * times["i32"] and times["i64 base 1"] <= 1.5 * times["i32"], times
