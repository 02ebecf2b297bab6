"""GPU parity tests for aclsparseSpMM (GetBufferSize -> Preprocess -> SpMM through
the C ABI) against the CPU oracle.

Tolerances, written per test:
  fp32              per element |d| <= 1e-5 * max(|oracle|, 1e-30) against the
                    fp64-accumulated oracle (the library accumulates in fp64),
                    plus the reference's own MERE < 2^-13 / MARE < 10 * 2^-13 rule
                    against its fp32 golden (test/spmm/arch35/spmm_test.cpp:525-526)
  fp16 in, fp32 out per element 1e-3 relative against the oracle on the fp16-rounded inputs
  fp16 in and out   the reference's fp16 recipe (:604-622): fp32 golden on rounded
                    inputs, clamp, re-round; MERE < 2^-10, MARE < 10 * 2^-10
  int8              bit-exact
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import csr_from_lengths, random_csr, run_spmm, to_dev

pytestmark = pytest.mark.gpu


def reference_random_csr(m, k, nnz, seed):
    """The reference's GenerateRandomCsr after std::srand(seed) (spmm_test.cpp:91-123, seeds :964-975 and :995),
    restated in oracle/: the same matrix the reference's program multiplies."""
    return oracle.spmm35_random_csr(seed, m, k, nnz)


def reference_dense(count):
    """The fill of B (and of C when beta != 0) in that program: -5 + 10 * (i % 10001) / 10000 (:406-415)."""
    i = (np.arange(count) % 10001).astype(np.float32)
    return (np.float32(-5.0) + np.float32(10.0) * i / np.float32(10000.0)).astype(np.float32)


def check_fp32(got, m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, **layout):
    gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, **layout)
    crm = layout.get("c_row_major", True)
    idx = (np.arange(m)[:, None] * ldc + np.arange(n)[None, :]) if crm else \
        (np.arange(n)[None, :] * ldc + np.arange(m)[:, None])
    err = oracle.max_rel_err(got[idx], gold[idx])
    assert err <= 1e-5, "max rel err %.3e" % err
    # padding between rows / columns must be untouched
    mask = np.ones(got.size, bool)
    mask[idx.ravel()] = False
    assert np.array_equal(got[mask], np.asarray(C0, np.float32)[mask])
    g32 = oracle.spmm_f32(m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, **layout)
    # Against the reference's fp32 golden only the mean is asserted: on elements that
    # nearly cancel, that golden's own rounding error exceeds the 10 * 2^-13 cap.
    mere, _, mism, _ = oracle.mere_mare(got[idx], g32[idx], eps=1e-7)
    assert mism == 0 and mere < 2.0 ** -13


def test_readme_known_answer(osa, gpu_ctx):
    """A (4x3, nnz 5) * B (3x2) = [[3,2],[0,3],[4,0],[5,5]] (reference sparse/spmm/README.md:275-303, :404-412)."""
    rowptr = np.array([0, 2, 3, 4, 5], np.int32)
    colind = np.array([0, 2, 1, 0, 2], np.int32)
    val = np.array([1, 2, 3, 4, 5], np.float32)
    B = np.array([1, 0, 0, 1, 1, 1], np.float32)
    C = run_spmm(osa, gpu_ctx, 4, 3, 2, rowptr, colind, val, B, 2, np.zeros(8, np.float32), 2, 1.0, 0.0,
                 alg=osa.ACL_SPARSE_SPMM_CSR_ALG1)
    assert np.array_equal(C.reshape(4, 2), np.array([[3, 2], [0, 3], [4, 0], [5, 5]], np.float32))


# the reference's five fp32 layout cases (spmm_test.cpp:964-975)
REF_CASES = [
    ("baseline_row_N_beta0", 256, 256, 64, 0, 1.0, 0.0, False, True, True, 42),
    ("opB_transpose", 256, 256, 64, 0, 1.0, 0.0, True, True, True, 43),
    ("B_C_col_major", 256, 256, 64, 0, 1.0, 0.0, False, False, False, 44),
    ("beta_nonzero", 256, 256, 64, 0, 1.0, 0.5, False, True, True, 45),
    ("small_shape", 32, 32, 16, 80, 1.0, 0.0, False, True, True, 46),
]


@pytest.mark.parametrize("name,m,k,n,nnz,alpha,beta,trans_b,b_rm,c_rm,seed", REF_CASES)
def test_reference_fp32_cases(osa, gpu_ctx, name, m, k, n, nnz, alpha, beta, trans_b, b_rm, c_rm, seed):
    nnz = nnz if nnz > 0 else m * k // 10
    rowptr, colind, val = reference_random_csr(m, k, nnz, seed)
    ldb = n if b_rm else k
    ldc = n if c_rm else m
    # B has k * ldb elements and C m * ldc, as that program sizes them (:406, :410): with op(B) = B^T or
    # column-major storage that is more than the product touches
    B = reference_dense(k * ldb)
    C0 = reference_dense(m * ldc)
    if beta == 0.0:
        C0[:] = np.nan  # the program zero-fills C then; here: must not be read
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta,
                   order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                   order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                   op_b=osa.ACL_SPARSE_OP_TRANSPOSE if trans_b else osa.ACL_SPARSE_OP_NON_TRANSPOSE)
    C0z = np.zeros_like(C0) if beta == 0.0 else C0
    gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, ldb, C0z, ldc, alpha, beta, b_row_major=b_rm,
                           trans_b=trans_b, c_row_major=c_rm)
    used = (np.arange(m)[:, None] * ldc + np.arange(n)[None, :]) if c_rm else \
        (np.arange(n)[None, :] * ldc + np.arange(m)[:, None])
    assert oracle.max_rel_err(got[used], gold[used]) <= 1e-5
    rest = np.ones(got.size, bool)
    rest[used.ravel()] = False
    assert np.array_equal(got[rest].view(np.uint32), C0[rest].view(np.uint32))  # what lies beyond C stays as it was


@pytest.mark.parametrize("n", [1, 3, 8, 17, 32, 64, 100, 128, 256, 260, 516, 1000])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, -2.0)])
def test_column_counts_and_padding(osa, gpu_ctx, n, alpha, beta):
    """n not a multiple of the vector width, and ldb / ldc padding."""
    m, k = 300, 200
    rowptr, colind, val = random_csr(m, k, 0.05, seed=n, empty_row_prob=0.1)
    ldb, ldc = n + (4 if n % 2 else 0), n + (8 if n % 3 == 0 else 0)
    rng = np.random.default_rng(n)
    B = rng.uniform(-2, 2, k * ldb).astype(np.float32)
    C0 = rng.uniform(-2, 2, m * ldc).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta)
    check_fp32(got, m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta)


@pytest.mark.parametrize("b_rm,c_rm,trans_b", [(True, False, False), (False, True, False), (False, False, True),
                                               (True, True, True), (False, True, True)])
def test_layouts(osa, gpu_ctx, b_rm, c_rm, trans_b):
    m, k, n = 120, 120, 24      # square so that every (order, op) reading of B stays in bounds
    rowptr, colind, val = random_csr(m, k, 0.1, seed=5, unsorted=True)
    ldb, ldc = 130, 125
    rng = np.random.default_rng(1)
    B = rng.uniform(-2, 2, 130 * ldb).astype(np.float32)
    C0 = rng.uniform(-2, 2, 125 * ldc).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C0, ldc, 1.5, 0.25,
                   order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                   order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                   op_b=osa.ACL_SPARSE_OP_TRANSPOSE if trans_b else osa.ACL_SPARSE_OP_NON_TRANSPOSE)
    check_fp32(got, m, n, rowptr, colind, val, B, ldb, C0, ldc, 1.5, 0.25, b_row_major=b_rm, trans_b=trans_b,
               c_row_major=c_rm)


@pytest.mark.parametrize("n", [64, 128, 16, 300])
def test_long_rows_are_binned(osa, gpu_ctx, n):
    """Rows far above the long-row threshold next to short and empty ones."""
    rng = np.random.default_rng(n)
    m, k = 2000, 60000
    lengths = rng.integers(0, 40, m)
    lengths[[3, 700, 701, 1999]] = [50000, 513, 512, 12345]
    rowptr, colind, val = csr_from_lengths(lengths, k, seed=2)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 2.0, 1.0)
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, C0, n, 2.0, 1.0)
    assert oracle.max_rel_err(got, gold) <= 1e-5


def test_high_precision_alg_same_result(osa, gpu_ctx):
    m, k, n = 500, 500, 64
    rowptr, colind, val = random_csr(m, k, 0.1, seed=8)
    rng = np.random.default_rng(8)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = np.zeros(m * n, np.float32)
    a = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.0)
    b = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.0,
                 alg=osa.ACL_SPARSE_SPMM_CSR_FP32_HIGH_PRECISION_ALG)
    assert np.array_equal(a, b)


def _fp16_inputs(m, k, n, seed):
    rowptr, colind, val = reference_random_csr(m, k, m * k // 10, seed)
    rng = np.random.default_rng(seed)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    rt = lambda a: oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(a))
    return rowptr, colind, rt(val), rt(B), rt(C0)


def test_fp16_in_fp16_out_reference_recipe(osa, gpu_ctx):
    import torch
    m, k, n = 256, 256, 64
    rowptr, colind, val, B, C0 = _fp16_inputs(m, k, n, 47)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.5, val_dtype=torch.float16,
                   c_dtype=torch.float16)
    gold = oracle.spmm_f32(m, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.5)
    gold = oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(np.clip(gold, -65504.0, 65504.0)))
    mere, mare, mism, _ = oracle.mere_mare(got, gold, eps=1e-7)
    assert mism == 0 and mere < 2.0 ** -10 and mare < 10 * 2.0 ** -10


def test_fp16_out_clamps(osa, gpu_ctx):
    import torch
    rowptr = np.array([0, 2, 4], np.int32)
    colind = np.array([0, 1, 0, 1], np.int32)
    val = np.array([60000, 60000, -60000, -60000], np.float32)
    B = np.ones(2 * 8, np.float32)
    got = run_spmm(osa, gpu_ctx, 2, 2, 8, rowptr, colind, val, B, 8, np.zeros(16, np.float32), 8, 1.0, 0.0,
                   val_dtype=torch.float16, c_dtype=torch.float16)
    assert np.array_equal(got.reshape(2, 8), np.array([[65504.0] * 8, [-65504.0] * 8], np.float32))


def test_fp16_in_fp32_out(osa, gpu_ctx):
    """fp16 A and B, fp32 accumulate and C: 1e-3 relative against the oracle on the rounded inputs."""
    import torch
    m, k, n = 400, 300, 128
    rowptr, colind, val, B, C0 = _fp16_inputs(m, k, n, 48)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.0, val_dtype=torch.float16)
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, np.zeros_like(C0), n, 1.0, 0.0)
    assert oracle.max_rel_err(got, gold) <= 1e-3


@pytest.mark.parametrize("alpha,beta", [(1, 0), (3, -2), (20000, 1)])
def test_int8_exact(osa, gpu_ctx, alpha, beta):
    import torch
    m, k, n = 256, 256, 64
    rowptr, colind, _ = reference_random_csr(m, k, m * k // 10, 49)
    rng = np.random.default_rng(49)
    val = rng.integers(-128, 128, colind.size).astype(np.int8)
    B = rng.integers(-128, 128, k * n).astype(np.int8)
    C0 = rng.integers(-1000, 1000, m * n).astype(np.int32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, alpha, beta, val_dtype=torch.int8,
                   c_dtype=torch.int32, compute_type=osa.ACL_INT32)
    gold = oracle.spmm_i8(m, n, rowptr, colind, val, B, n, C0, n, alpha, beta, saturate=True)
    assert np.array_equal(got, gold)


@pytest.mark.parametrize("n,b_rm,c_rm", [(64, True, True), (128, True, True), (50, True, True), (48, False, True),
                                         (16, True, False)])
def test_int8_vector_kernels_long_rows_and_layouts(osa, gpu_ctx, n, b_rm, c_rm):
    """int8 x int8 -> int32 on the 16-bytes-per-lane kernels (16 columns a lane): long rows through the segment
    path, a width that is not whole vectors and column-major operands through the staged copies; bit-exact,
    saturating epilogue."""
    import torch
    rng = np.random.default_rng(n)
    m, k = 2500, 4000
    lengths = rng.integers(0, 25, m)
    lengths[[7, 1200]] = [3000, 600]
    rowptr, colind, _ = csr_from_lengths(lengths, k, seed=n)
    val = rng.integers(-128, 128, colind.size).astype(np.int8)
    ldb, ldc = (n if b_rm else k), (n if c_rm else m)
    B = rng.integers(-128, 128, (k if b_rm else n) * ldb).astype(np.int8)
    C0 = rng.integers(-1000, 1000, (m if c_rm else n) * ldc).astype(np.int32)
    for alpha, beta in ((1, 0), (3, -2), (70000, 1)):
        got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta,
                       order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                       order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                       val_dtype=torch.int8, c_dtype=torch.int32, compute_type=osa.ACL_INT32)
        Bl = B.reshape(k, n) if b_rm else B.reshape(n, k).T          # logical k x n
        gold = oracle.spmm_i8(m, n, rowptr, colind, val, np.ascontiguousarray(Bl).ravel(), n,
                              (C0.reshape(m, n) if c_rm else C0.reshape(n, m).T).ravel().copy(), n, alpha, beta,
                              saturate=True).reshape(m, n)
        assert np.array_equal(got.reshape(m, n) if c_rm else got.reshape(n, m).T, gold)


def test_spmm_column_equals_spmv(osa, gpu_ctx):
    """Column j of the SpMM result equals the oracle SpMV with B[:, j]."""
    m, k, n = 333, 222, 8
    rowptr, colind, val = random_csr(m, k, 0.07, seed=12)
    rng = np.random.default_rng(12)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B.ravel(), n, np.zeros(m * n, np.float32), n, 1.0, 0.0)
    for j in range(n):
        y = oracle.spmv_f64(m, k, rowptr, colind, val, np.ascontiguousarray(B[:, j]), None, 1.0, 0.0)
        assert oracle.max_rel_err(got.reshape(m, n)[:, j], y) <= 1e-6


def _lengths(shape, m, rng):
    if shape == "mostly_empty":                 # windows of more than 255 empty rows
        lengths = np.zeros(m, np.int64)
        lengths[rng.choice(m, m // 100, replace=False)] = rng.integers(1, 30, m // 100)
    elif shape == "threshold":                  # 2048 is still a short row, 2049 is a long one
        lengths = rng.integers(0, 12, m)
        lengths[rng.choice(m, 40, replace=False)] = rng.choice([255, 300, 2047, 2048, 2049, 2100], 40)
    elif shape == "cut_rows":                   # rows that lie across several lane groups' shares of a slab
        lengths = rng.choice([0, 1, 2, 3, 15, 16, 17, 40, 100, 700, 1500, 2048], m,
                             p=[.1, .2, .2, .2, .05, .05, .05, .05, .05, .02, .02, .01])
    elif shape == "dense_slabs":                # a slab holds more entries than one LDS piece takes
        lengths = rng.integers(150, 257, m)
    elif shape == "alternating":
        lengths = np.arange(m) % 2
    elif shape == "power_law":
        lengths = np.minimum((1.0 / rng.uniform(1e-4, 1.0, m)).astype(np.int64), 4000)
    elif shape in ("sorted_up", "sorted_down"):  # a graph ordered by degree: slabs are cut by work, not by rows
        lengths = np.sort(np.minimum((1.0 / rng.uniform(1e-4, 1.0, m)).astype(np.int64), 4000))
        lengths = lengths[::-1].copy() if shape == "sorted_down" else lengths
    else:
        raise ValueError(shape)
    return lengths


@pytest.mark.parametrize("shape", ["mostly_empty", "threshold", "cut_rows", "dense_slabs", "alternating", "power_law",
                                   "sorted_up", "sorted_down"])
@pytest.mark.parametrize("n,beta", [(8, 0.0), (24, 0.5), (64, -1.0), (256, 0.0), (260, 0.5), (1000, 0.0)])
def test_row_length_mixes(osa, gpu_ctx, shape, n, beta):
    """Preprocessed fast path (rows worked in LDS-staged slabs, long rows in segments) on row-length mixes that
    hit its corner cases; n = 24 leaves lanes of a lane group without a column; n = 260 and 1000 are more columns
    than a lane group spans: several workgroups a slab, one a tile of columns."""
    rng = np.random.default_rng(len(shape) * 1000 + n)
    m = 1 if shape == "single" else (700 if shape == "dense_slabs" else 6000)
    k = 5000
    rowptr, colind, val = csr_from_lengths(_lengths(shape, m, rng), k, seed=n)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    if beta == 0.0:
        C0[::7] = np.nan                         # C must not be read
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.25, beta)
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, np.nan_to_num(C0), n, 1.25, beta)
    assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("longest,entries", [(256, 2048), (64, 1024)])
def test_slab_table_cuts_by_work(osa, gpu_ctx, longest, entries):
    """The analysis leaves, for the slab kernel, the first row of every slab: slab s starts at the first row with
    s * share entries + rows in front of it, whatever the order of the rows (checked against numpy on rows sorted
    by length, where slabs of equal numbers of rows would differ in work a hundredfold).  About 2048 entries a
    slab; 1024 where no row exceeds 64 entries and B has at most 128 columns."""
    import torch
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(3)
    m = 300_000
    lengths = np.sort(np.minimum((1.0 / rng.uniform(1e-4, 1.0, m)).astype(np.int64), longest))[::-1].copy()
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    nnz = int(rowptr[-1])
    L = osa.lib()
    d_rp = to_dev(rowptr, dev)
    size = ctypes.c_size_t(0)
    sp = ctypes.c_void_p(stream.cuda_stream)
    assert L.opsparse_spmm_csr_workspace_bytes(d_rp.data_ptr(), m, nnz, 64, sp, ctypes.byref(size)) == 0
    ws = torch.zeros(size.value, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmmPlan()
    assert L.opsparse_spmm_csr_analyse(d_rp.data_ptr(), m, nnz, 64, ws.data_ptr(), size.value, 0, ctypes.byref(plan),
                                       sp) == 0
    stream.synchronize()
    assert plan.numSlabs > 0 and plan.slabStartOff >= 256 and plan.bytes <= size.value
    table = ws[plan.slabStartOff: plan.slabStartOff + 4 * (plan.numSlabs + 1)].view(torch.int32).cpu().numpy()
    work = rowptr[:-1].astype(np.int64) + np.arange(m)            # entries + rows in front of row r
    share = entries + min(max(entries * m // nnz, 16), 4096)     # that many entries and their rows a slab
    assert plan.numSlabs == -(-(m + nnz) // share)
    want = np.concatenate([np.searchsorted(work, np.arange(plan.numSlabs) * share, side="left"), [m]])
    assert np.array_equal(table, want)
    per_slab = np.diff(np.concatenate([work, [m + nnz]])[table])
    assert per_slab.max() <= share + longest + 1                   # a slab overshoots its share by at most a row


def test_buffer_sized_for_a_wide_b_serves_a_narrow_one(osa, gpu_ctx):
    """GetBufferSize for n = 256, then the same buffer and matrix with n = 64 (rows of at most 64 entries, whose
    slabs are shorter, and their table longer, for a narrow B): the size asked for the wide B covers it, and the
    bytes behind the buffer stay as they were."""
    import torch
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rng = np.random.default_rng(8)
    m, k = 200_000, 5000
    rowptr, colind, val = csr_from_lengths(rng.integers(20, 41, m), k, seed=4)
    d_rp = to_dev(rowptr, dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    wide, narrow = ctypes.c_size_t(0), ctypes.c_size_t(0)
    nnz = int(rowptr[-1])
    assert L.opsparse_spmm_csr_workspace_bytes(d_rp.data_ptr(), m, nnz, 256, sp, ctypes.byref(wide)) == 0
    assert L.opsparse_spmm_csr_workspace_bytes(d_rp.data_ptr(), m, nnz, 64, sp, ctypes.byref(narrow)) == 0
    assert wide.value >= narrow.value > 0
    guard = 4096
    ws = torch.full((wide.value + guard,), 0x5A, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmmPlan()
    assert L.opsparse_spmm_csr_analyse(d_rp.data_ptr(), m, nnz, 64, ws.data_ptr(), wide.value, 0, ctypes.byref(plan),
                                       sp) == 0
    stream.synchronize()
    assert plan.bytes <= wide.value and plan.slabStartOff + 4 * (plan.numSlabs + 1) <= wide.value
    assert bool((ws[wide.value:] == 0x5A).all())
    table = ws[plan.slabStartOff: plan.slabStartOff + 4 * (plan.numSlabs + 1)].view(torch.int32).cpu().numpy()
    assert table[0] == 0 and table[-1] == m and np.all(np.diff(table) >= 0)


@pytest.mark.parametrize("lengths,binned", [("even 300", False), ("even 2048", False), ("even 2049", True),
                                            ("300 among 10", False), ("2100 among 10", True)])
def test_only_rows_beyond_2048_entries_are_cut_into_segments(osa, gpu_ctx, lengths, binned):
    """Rows of up to 2048 entries stay with the slabs, whose lane groups share them out; longer ones are cut into
    segments so that a power-law matrix balances.  GetBufferSize and the analysis agree, and the product is the
    oracle's either way."""
    import torch
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(len(lengths))
    k, n = 50_000, 64
    if lengths.startswith("even"):
        base_len = int(lengths.split()[1])
        m = 3000 if base_len < 1000 else 500
        lens = rng.integers(base_len - 40, base_len + 1, m)
        lens[7] = base_len
    else:
        m = 3000
        lens = np.full(m, 10)
        lens[[5, 2000]] = int(lengths.split()[0])
    rowptr, colind, val = csr_from_lengths(lens, k, seed=9)
    L = osa.lib()
    d_rp = to_dev(rowptr, dev)
    size = ctypes.c_size_t(0)
    sp = ctypes.c_void_p(stream.cuda_stream)
    nnz = int(rowptr[-1])
    assert L.opsparse_spmm_csr_workspace_bytes(d_rp.data_ptr(), m, nnz, n, sp, ctypes.byref(size)) == 0
    ws = torch.zeros(size.value, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmmPlan()
    assert L.opsparse_spmm_csr_analyse(d_rp.data_ptr(), m, nnz, n, ws.data_ptr(), size.value, 0, ctypes.byref(plan),
                                       sp) == 0
    assert (plan.numLongRows > 0) == binned and plan.bytes <= size.value
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, -0.5, 2.0)
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, C0, n, -0.5, 2.0)
    assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("n", [128, 520])
@pytest.mark.parametrize("shape", ["threshold", "cut_rows", "power_law"])
def test_row_length_mixes_fp16(osa, gpu_ctx, shape, n):
    import torch
    rng = np.random.default_rng(77)
    m, k = 5000, 4000
    rowptr, colind, val = csr_from_lengths(_lengths(shape, m, rng), k, seed=5)
    val = val.astype(np.float16).astype(np.float32)
    B = rng.uniform(-1, 1, k * n).astype(np.float16).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.5, val_dtype=torch.float16)
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, C0, n, 1.0, 0.5)
    assert oracle.max_rel_err(got, gold) <= 1e-3


@pytest.mark.parametrize("n", [4, 64, 512])
def test_raw_launch_without_plan(osa, gpu_ctx, n):
    """opsparse_spmm_csr_launch with plan == NULL: one lane group per row of any length, no workspace."""
    import ctypes
    import torch
    from helpers import to_dev
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(n)
    m, k = 3000, 9000
    lengths = rng.integers(0, 20, m)
    lengths[[5, 2000]] = [7000, 300]
    rowptr, colind, val = csr_from_lengths(lengths, k, seed=9)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, B, C0)]
    s = lambda v: osa.OpsparseScalar(v, None, 0, 0)
    torch.cuda.synchronize()
    rc = osa.lib().opsparse_spmm_csr_launch(None, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                            d[4].data_ptr(), m, k, n, colind.size, n, n, 0, 0, 0, s(0.5), s(2.0),
                                            osa.OPSPARSE_F32, osa.OPSPARSE_F32, None, 0,
                                            ctypes.c_void_p(stream.cuda_stream))
    assert rc == 0
    stream.synchronize()
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B, n, C0, n, 0.5, 2.0)
    assert oracle.max_rel_err(d[4].cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("b_rm,c_rm,trans_b", [(False, True, False), (True, False, False), (False, False, False),
                                               (True, True, True), (False, False, True)])
@pytest.mark.parametrize("n,half", [(64, False), (10, False), (44, True)])
def test_layouts_through_the_staging_area(osa, gpu_ctx, b_rm, c_rm, trans_b, n, half):
    """Column-major / transposed operands at a size with many tiles, long rows (the binned path) and a width that
    is not whole 16-byte vectors: Preprocess reserves row-major copies behind the plan, the product runs on them
    and C comes back in its own layout, padding of ldb / ldc untouched.  beta = 0 must not read C (NaN)."""
    rng = np.random.default_rng(n + 7 * b_rm + 3 * c_rm + trans_b)
    m = k = 3000
    lengths = rng.integers(0, 30, m)
    lengths[[5, 1500]] = [2800, 700]
    rowptr, colind, val = csr_from_lengths(lengths, k, seed=9)
    eff_col = (not b_rm) != trans_b                 # op(B) = B^T flips which index of B is contiguous
    ldb = k + 3 if (eff_col or not b_rm) else n + 4  # a column-major descriptor needs ld >= rows in any case
    ldc = n + 8 if c_rm else m + 5
    B = rng.uniform(-1, 1, (n if eff_col else k) * ldb).astype(np.float32)
    C_len = (m * ldc) if c_rm else (n * ldc)
    vd, cd, tol = (torch.float16, torch.float32, 1e-5) if half else (None, None, 1e-5)
    if half:
        val, B = (torch.from_numpy(a).to(torch.float16).float().numpy() for a in (val, B))
    for alpha, beta in ((1.5, 0.25), (2.0, 0.0)):
        C0 = rng.uniform(-1, 1, C_len).astype(np.float32)
        C_in = C0.copy()
        if beta == 0.0:
            logical = np.zeros(C_len, bool)
            idx = (np.arange(m)[:, None] * ldc + np.arange(n)[None, :]) if c_rm else \
                  (np.arange(m)[:, None] + np.arange(n)[None, :] * ldc)
            logical[idx.ravel()] = True
            C_in[logical] = np.nan               # must not be read; the padding keeps its values
        got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C_in, ldc, alpha, beta,
                       order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                       order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL,
                       op_b=osa.ACL_SPARSE_OP_TRANSPOSE if trans_b else osa.ACL_SPARSE_OP_NON_TRANSPOSE,
                       val_dtype=vd, c_dtype=cd)
        gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, b_row_major=b_rm,
                               trans_b=trans_b, c_row_major=c_rm)
        assert oracle.max_rel_err(got, gold) <= tol


def _mesh7(side):
    """The 7-point stencil on side^3 points, no wrap-around: rows, columns, row offsets, ascending column indices."""
    m = side ** 3
    r = np.arange(m)
    z, y, x = r // (side * side), (r // side) % side, r % side
    cols, keep = [], []
    for d, coord in ((-side * side, z), (-side, y), (-1, x), (0, None), (1, x), (side, y), (side * side, z)):
        ok = np.ones(m, bool) if coord is None else ((coord > 0) if d < 0 else (coord < side - 1))
        cols.append(r + d)
        keep.append(ok)
    cols, keep = np.stack(cols, 1), np.stack(keep, 1)
    rowptr = np.concatenate([[0], np.cumsum(keep.sum(1))]).astype(np.int32)
    return m, m, rowptr, cols[keep].astype(np.int32)


@pytest.mark.parametrize("shape", ["mesh", "band", "random"])
@pytest.mark.parametrize("n", [12, 16, 32, 64, 128])
def test_kernel_choice_by_shape_and_width(osa, gpu_ctx, shape, n, monkeypatch):
    """Preprocess picks, for a matrix without long rows, between the slabs staged through LDS and a lane group a row
    straight from memory: by the width of B, the mean row length and - where those leave it open - by a sample of
    how far the columns lie from the diagonal (a mesh of 7 entries a row, a band of 40, 40 random columns a row:
    the rule's three kinds).  Either choice must give the product; so must the rule switched off."""
    rng = np.random.default_rng(n)
    if shape == "mesh":
        m, k, rowptr, colind = _mesh7(20)
    else:
        m = 6000
        k = 6000 if shape == "band" else 300_000      # (the sample counts columns further than 2^17 from the diagonal)
        per = 40
        rowptr = (np.arange(m + 1) * per).astype(np.int32)
        if shape == "band":
            base = np.clip(np.arange(m)[:, None] - per // 2 + np.arange(per)[None, :], 0, k - 1)
            colind = base.ravel().astype(np.int32)
        else:
            colind = rng.integers(0, k, m * per).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, n, C0, n, 1.5, -0.5)
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.5, -0.5)
    assert oracle.max_rel_err(got, gold) <= 1e-5
    monkeypatch.setenv("OPS_SPARSE_SPMM_NO_ROWS_RULE", "1")
    got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, n, C0, n, 1.5, -0.5)
    assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("b_rm,c_rm", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("half", [False, True])
def test_few_columns_on_a_mesh(osa, gpu_ctx, n, b_rm, c_rm, half):
    """One to eight columns of B under a 7-point mesh matrix (block Krylov methods, a few right-hand sides): the
    widths are padded to whole 16-byte rows in the staging area where they are not, and the product of one or two
    such pieces a row takes the kernel for narrow B.  Every layout, fp32 and fp16 values, beta zero (C holds NaN
    and must not be read) and not."""
    m, k, rowptr, colind = _mesh7(24)
    rng = np.random.default_rng(n + 10 * b_rm + 20 * c_rm)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    ldb = (n + 3) if b_rm else (k + 2)
    ldc = (n + 1) if c_rm else (m + 6)
    B = rng.uniform(-1, 1, (k if b_rm else n) * ldb).astype(np.float32)
    vd, cd = (torch.float16, torch.float32) if half else (None, None)
    if half:
        val, B = (torch.from_numpy(a).to(torch.float16).float().numpy() for a in (val, B))
    for alpha, beta in ((1.25, 0.0), (0.5, -1.5)):
        C0 = rng.uniform(-1, 1, (m if c_rm else n) * ldc).astype(np.float32)
        C_in = C0.copy()
        if beta == 0.0:
            idx = (np.arange(m)[:, None] * ldc + np.arange(n)[None, :]) if c_rm else \
                  (np.arange(m)[:, None] + np.arange(n)[None, :] * ldc)
            C_in[idx.ravel()] = np.nan
        got = run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B, ldb, C_in, ldc, alpha, beta,
                       order_b=osa.ACL_SPARSE_ORDER_ROW if b_rm else osa.ACL_SPARSE_ORDER_COL,
                       order_c=osa.ACL_SPARSE_ORDER_ROW if c_rm else osa.ACL_SPARSE_ORDER_COL, val_dtype=vd, c_dtype=cd)
        gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, ldb, C0, ldc, alpha, beta, b_row_major=b_rm,
                               trans_b=False, c_row_major=c_rm)
        assert oracle.max_rel_err(got, gold) <= 1e-5


@pytest.mark.parametrize("half", [False, True])
def test_one_column_with_unit_leading_dimensions_runs_as_a_vector(osa, gpu_ctx, half):
    """n = 1, row-major B and C with a leading dimension of 1: the column is a vector in memory and the product
    runs under an SpMV plan made at Preprocess, like one or two columns of column-major operands
    (test_few_columns_on_a_mesh).  Called twice with other scalars: the plan is reused."""
    m, k = 5000, 4000
    rng = np.random.default_rng(11)
    rowptr, colind, val = csr_from_lengths(rng.integers(0, 12, m), k, seed=2)
    B = rng.uniform(-1, 1, k).astype(np.float32)
    vd, cd = (torch.float16, torch.float32) if half else (None, None)
    if half:
        val, B = (torch.from_numpy(a).to(torch.float16).float().numpy() for a in (val, B))
    dev, stream, handle = gpu_ctx
    C0 = rng.uniform(-1, 1, m).astype(np.float32)
    d = [to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev, vd), to_dev(B, dev, vd), to_dev(C0, dev, cd)]
    A = osa.Csr(m, k, d[0], d[1], d[2])
    op = osa.SpmmOp(handle, A, osa.DnMat(k, 1, 1, d[3]), osa.DnMat(m, 1, 1, d[4]))
    op(1.5, 0.5)
    stream.synchronize()
    first = oracle.spmm_f64(m, 1, rowptr, colind, val, B, 1, C0, 1, 1.5, 0.5)
    assert oracle.max_rel_err(d[4].cpu().numpy(), first) <= 1e-5
    d[4].fill_(float("nan"))
    op(-2.0, 0.0)
    stream.synchronize()
    again = oracle.spmm_f64(m, 1, rowptr, colind, val, B, 1, C0, 1, -2.0, 0.0)
    assert oracle.max_rel_err(d[4].cpu().numpy(), again) <= 1e-5


def test_staging_needs_a_buffer_preprocessed_for_it(osa, gpu_ctx):
    """A buffer sized and preprocessed for row-major operands (256 bytes here) and then used with a column-major B:
    no staging area was promised, the product must run in place (slowly) and stay inside the buffer — the guard
    bytes behind it keep their pattern."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(3)
    m, k, n = 500, 400, 12
    rowptr, colind, val = random_csr(m, k, 0.05, seed=4)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    d_B, d_C = to_dev(B, dev), to_dev(C0, dev)
    A = osa.Csr(m, k, d[0], d[1], d[2])
    B_row, B_col = osa.DnMat(k, n, n, d_B), osa.DnMat(k, n, k, d_B, osa.ACL_SPARSE_ORDER_COL)
    Cd = osa.DnMat(m, n, n, d_C)
    L = osa.lib()
    size = ctypes.c_size_t(0)
    args = lambda Bd: (handle.h, 0, 0, None, A.d, Bd.d, None, Cd.d, osa.ACL_FLOAT, osa.ACL_SPARSE_SPMM_ALG_DEFAULT)
    assert L.aclsparseSpMMGetBufferSize(*args(B_row), ctypes.byref(size)) == 0
    small = int(size.value)
    assert L.aclsparseSpMMGetBufferSize(*args(B_col), ctypes.byref(size)) == 0 and int(size.value) >= small + k * n * 4
    buf = torch.full((small + 4096,), 0x5A, dtype=torch.uint8, device=dev)
    bp = ctypes.c_void_p(buf.data_ptr())
    assert L.aclsparseSpMMPreprocess(*args(B_row), bp) == 0
    one, half_ = ctypes.c_float(1.0), ctypes.c_float(0.5)
    assert L.aclsparseSpMM(handle.h, 0, 0, ctypes.byref(one), A.d, B_col.d, ctypes.byref(half_), Cd.d, osa.ACL_FLOAT,
                           osa.ACL_SPARSE_SPMM_ALG_DEFAULT, bp) == 0
    stream.synchronize()
    assert bool((buf[small:] == 0x5A).all())
    gold = oracle.spmm_f64(m, n, rowptr, colind, val, B, k, C0, n, 1.0, 0.5, b_row_major=False, trans_b=False,
                           c_row_major=True)
    assert oracle.max_rel_err(d_C.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_b_of_4_gib_through_a_padded_leading_dimension(osa, gpu_ctx, dtype):
    """B with 2^20 rows and a leading dimension of 4 KiB spans 4 GiB: a row's offset no longer fits 32 bits and the
    slab kernel takes its instantiation with 64-bit gather addresses.  Only the 64 columns in use are ever touched
    (the rest of the allocation stays as it was); the last row of B, at the highest offset, is gathered."""
    dev, stream, handle = gpu_ctx
    m, k, n = 20_000, 1 << 20, 64
    ldb = 4096 // (4 if dtype == torch.float32 else 2)
    rng = np.random.default_rng(77)
    lengths = rng.integers(0, 33, m)
    lengths[17] = 3000                                        # a row cut into segments, too
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, k, int(rowptr[-1])).astype(np.int32)
    colind[:4] = [k - 1, 0, k - 2, k // 2]
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    Bc = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    if dtype == torch.float16:
        val = torch.from_numpy(val).half().float().numpy()
        Bc = torch.from_numpy(Bc).half().float().numpy()
    C0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    d_B = torch.full((k * ldb,), 7.0, dtype=dtype, device=dev)   # 4 GiB
    assert d_B.numel() * d_B.element_size() == 1 << 32
    d_B.view(k, ldb)[:, :n] = torch.from_numpy(Bc).to(dev).to(dtype)
    d = [to_dev(a, dev) for a in (rowptr, colind)]
    d_val = to_dev(val, dev, dtype)
    d_C = to_dev(C0.ravel(), dev)
    A = osa.Csr(m, k, d[0], d[1], d_val)
    op = osa.SpmmOp(handle, A, osa.DnMat(k, n, ldb, d_B), osa.DnMat(m, n, n, d_C))
    op(1.5, -0.5)
    stream.synchronize()
    gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, Bc, n, C0, n, 1.5, -0.5)
    assert oracle.max_rel_err(d_C.cpu().numpy(), np.asarray(gold).ravel()) <= (1e-5 if dtype == torch.float32 else 1e-3)
    assert bool((d_B.view(k, ldb)[:, n:] == 7.0).all())
    del d_B
    torch.cuda.empty_cache()


def test_buffer_preprocessed_for_a_narrow_c_is_not_re_analysed_for_a_wider_one(osa, gpu_ctx):
    """Preprocess with n = 8 into a buffer of exactly the size GetBufferSize asked for, long rows in the matrix (their
    segment table grows with n); then aclsparseSpMM on the same matrix and buffer with n = 256.  The library must
    not lay a wider plan's tables into the buffer: the product runs without tables, the bytes behind the buffer
    stay as they were, and the result is right.  The narrow product still works afterwards."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    m, k = 3000, 6000
    rng = np.random.default_rng(21)
    lengths = rng.integers(0, 30, m)
    lengths[[3, 1500, 2999]] = [5000, 2500, 4000]
    rowptr, colind, val = csr_from_lengths(lengths, k, seed=9)
    d_rp, d_ci, d_val = to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev)
    A = osa.Csr(m, k, d_rp, d_ci, d_val)

    def operands(n):
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        C0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
        d_B, d_C = to_dev(B.ravel(), dev), to_dev(C0.ravel(), dev)
        return B, C0, d_B, d_C, osa.DnMat(k, n, n, d_B), osa.DnMat(m, n, n, d_C)

    B8, C8, dB8, dC8, mB8, mC8 = operands(8)
    size = ctypes.c_size_t(0)
    one, half = ctypes.c_float(1.0), ctypes.c_float(0.5)
    args8 = (handle.h, 0, 0, ctypes.byref(one), A.d, mB8.d, ctypes.byref(half), mC8.d, osa.ACL_FLOAT, 0)
    assert L.aclsparseSpMMGetBufferSize(*args8, ctypes.byref(size)) == 0
    guard = 1 << 20
    buf = torch.full((size.value + guard,), 0x3C, dtype=torch.uint8, device=dev)
    pbuf = ctypes.c_void_p(buf.data_ptr())
    assert L.aclsparseSpMMPreprocess(*args8, pbuf) == 0
    B256, C256, dB256, dC256, mB256, mC256 = operands(256)
    args256 = (handle.h, 0, 0, ctypes.byref(one), A.d, mB256.d, ctypes.byref(half), mC256.d, osa.ACL_FLOAT, 0)
    wide = ctypes.c_size_t(0)
    assert L.aclsparseSpMMGetBufferSize(*args256, ctypes.byref(wide)) == 0 and wide.value > size.value
    assert L.aclsparseSpMM(*args256, pbuf) == 0
    stream.synchronize()
    assert bool((buf[size.value:] == 0x3C).all())
    gold = oracle.spmm_f64_rowmajor(m, 256, rowptr, colind, val, B256, 256, C256, 256, 1.0, 0.5)
    assert oracle.max_rel_err(dC256.cpu().numpy(), np.asarray(gold).ravel()) <= 1e-5
    assert L.aclsparseSpMM(*args8, pbuf) == 0
    stream.synchronize()
    gold = oracle.spmm_f64_rowmajor(m, 8, rowptr, colind, val, B8, 8, C8, 8, 1.0, 0.5)
    assert oracle.max_rel_err(dC8.cpu().numpy(), np.asarray(gold).ravel()) <= 1e-5
    assert bool((buf[size.value:] == 0x3C).all())
