"""Pins the CPU oracle (oracle/oracle.c) without a GPU: known answers from the
reference's own files, closed forms, brute force against dense fp64 products and
invariants chosen so that a dropped term, a wrong index or a transposed operand
fails at least one of them."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import dense_from_csr, random_csr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------- SpMV

def _rand_problem(rows, cols, density, seed, **kw):
    rowptr, colind, val = random_csr(rows, cols, density, seed, **kw)
    rng = np.random.default_rng(seed + 1000)
    x = rng.uniform(-3, 3, cols).astype(np.float32)
    y = rng.uniform(-3, 3, rows).astype(np.float32)
    return rowptr, colind, val, x, y


@pytest.mark.parametrize("rows,cols,density,seed", [(4, 4, 0.5, 42), (8, 8, 0.5, 49), (32, 32, 0.1, 53),
                                                    (4, 16, 0.5, 58), (16, 4, 0.5, 59), (57, 91, 0.2, 7)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (2.0, 1.0), (0.5, -1.0), (0.0, 1.0), (-1.0, 1.0)])
def test_spmv_f64_brute_force(rows, cols, density, seed, alpha, beta):
    """Against a dense fp64 matrix-vector product (duplicates summed, unsorted rows)."""
    rowptr, colind, val, x, y = _rand_problem(rows, cols, density, seed, unsorted=True, duplicates=True)
    A = dense_from_csr(rows, cols, rowptr, colind, val)
    want = (np.float64(np.float32(alpha)) * (A @ x.astype(np.float64)) +
            np.float64(np.float32(beta)) * y.astype(np.float64)).astype(np.float32)
    got = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y, alpha, beta)
    # fp64 sums in a different order agree to ~1e-15 relative; after rounding to fp32 at most 1 ulp apart
    assert np.allclose(got, want, rtol=2e-7, atol=1e-12)


def test_spmv_closed_forms():
    n = 64
    rowptr = np.arange(n + 1, dtype=np.int32)
    colind = np.arange(n, dtype=np.int32)
    d = np.full(n, 3.0, np.float32)
    x = np.arange(n, dtype=np.float32)
    y = np.ones(n, np.float32)
    # diagonal matrix: y = alpha * d * x + beta * y (test/frame/fill.h:211-225, csv row L0_diag_8x8)
    assert np.array_equal(oracle.spmv_f64(n, n, rowptr, colind, d, x, y, 2.0, -1.0), 6.0 * x - 1.0)
    assert np.array_equal(oracle.spmv_f32(n, rowptr, colind, d, x, y, 2.0, -1.0), 6.0 * x - 1.0)
    # empty matrix: y = beta * y (csv rows L0_4x4_empty, L1_nnz0_large)
    z = np.zeros(n + 1, np.int32)
    e = np.zeros(0, np.int32)
    assert np.array_equal(oracle.spmv_f64(n, n, z, e, np.zeros(0, np.float32), x, y, 1.0, 0.5), 0.5 * y)
    # k == 0: beta * y (spmv_op_golden.h:39-46); m == 0: empty result
    assert np.array_equal(oracle.spmv_f64(n, 0, z, e, np.zeros(0, np.float32), np.zeros(0, np.float32), y, 1.0, 2.0),
                          2.0 * y)
    assert oracle.spmv_f64(0, 5, np.zeros(1, np.int32), e, np.zeros(0, np.float32), x[:5], None, 1.0, 0.0).size == 0
    # beta == 0 ignores y entirely
    ynan = np.full(n, np.nan, np.float32)
    assert np.array_equal(oracle.spmv_f64(n, n, rowptr, colind, d, x, ynan, 1.0, 0.0), 3.0 * x)


def test_spmv_unit_vectors_give_columns():
    """A * e_j = column j: catches a row/column mix-up."""
    rows, cols = 9, 13
    rowptr, colind, val, _, y = _rand_problem(rows, cols, 0.4, 3)
    A = dense_from_csr(rows, cols, rowptr, colind, val)
    for j in range(cols):
        e = np.zeros(cols, np.float32)
        e[j] = 1.0
        got = oracle.spmv_f64(rows, cols, rowptr, colind, val, e, y, 1.0, 0.0)
        assert np.array_equal(got, A[:, j].astype(np.float32))


def test_spmv_transpose_matches_dense():
    rows, cols = 23, 17
    rowptr, colind, val, _, _ = _rand_problem(rows, cols, 0.3, 11)
    rng = np.random.default_rng(5)
    x = rng.uniform(-2, 2, rows).astype(np.float32)
    y = rng.uniform(-2, 2, cols).astype(np.float32)
    A = dense_from_csr(rows, cols, rowptr, colind, val)
    want = (1.5 * (A.T @ x.astype(np.float64)) + np.float64(np.float32(-0.25)) * y).astype(np.float32)
    got64 = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y, 1.5, -0.25)
    got32 = oracle.spmv_trans_f32(rows, cols, rowptr, colind, val, x, y, 1.5, -0.25)
    assert np.allclose(got64, want, rtol=2e-7, atol=1e-12)
    assert np.allclose(got32, want, rtol=1e-5, atol=1e-5)


def test_spmv_f32_golden_close_to_f64_oracle():
    """The reference's fp32 golden agrees with the fp64 oracle inside the reference's own rule
    (|d| <= 2^-16 + 2^-10 |g| for >= 99 % of the elements, test/spmv/arch22/spmv_test.cpp:208-220)."""
    rows, cols = 2000, 2000
    rowptr, colind, val, x, y = _rand_problem(rows, cols, 0.01, 21)
    g32 = oracle.spmv_f32(rows, rowptr, colind, val, x, y, 1.0, 1.0)
    g64 = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y, 1.0, 1.0)
    ok = np.abs(g32 - g64) <= 2.0 ** -16 + 2.0 ** -10 * np.abs(g64)
    assert ok.mean() >= 0.99
    assert not np.array_equal(g32, g64)  # they are different computations


def test_threaded_goldens_equal_the_single_thread_loops():
    """The all-cores CPU baselines of the benchmark are the reference loops with rows shared out among threads:
    bit-identical to the single-thread loops, whatever the number of threads."""
    rows, cols, n = 3000, 700, 9
    rowptr, colind, val = random_csr(rows, cols, 0.02, 5, empty_row_prob=0.1)
    rng = np.random.default_rng(6)
    x, y = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    B = rng.uniform(-1, 1, (cols, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (rows, n)).astype(np.float32)
    one = oracle.spmv_f32(rows, rowptr, colind, val, x, y, 1.5, -0.5)
    mm = oracle.spmm_f32(rows, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 1.5, -0.5)
    for threads in (1, 3, 8):
        assert np.array_equal(oracle.spmv_f32_threads(rows, rowptr, colind, val, x, y, 1.5, -0.5, threads), one)
        assert np.array_equal(oracle.spmm_f32_threads(rows, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 1.5,
                                                      -0.5, threads), mm)
    assert oracle.host_threads() >= 1


def test_spmv_int32_wraps():
    rowptr = np.array([0, 2, 3], np.int32)
    colind = np.array([0, 1, 1], np.int32)
    val = np.array([2 ** 30, 2 ** 30, -7], np.int32)
    x = np.array([2, 2], np.int32)
    y = np.array([5, 1], np.int32)
    got = oracle.spmv_i32(2, rowptr, colind, val, x, y, 1, 3)
    assert got.tolist() == [15, -11]   # 2^32 wraps to 0, + 3 * 5;  -14 + 3


# ------------------------------------------------------------------- SpMM

def test_spmm_readme_known_answer():
    """reference sparse/spmm/README.md:275-303 and its printed output :404-412."""
    rowptr = np.array([0, 2, 3, 4, 5], np.int32)
    colind = np.array([0, 2, 1, 0, 2], np.int32)
    val = np.array([1, 2, 3, 4, 5], np.float32)
    B = np.array([1, 0, 0, 1, 1, 1], np.float32)
    want = np.array([[3, 2], [0, 3], [4, 0], [5, 5]], np.float32)
    for fn in (oracle.spmm_f32, oracle.spmm_f64):
        assert np.array_equal(fn(4, 2, rowptr, colind, val, B, 2, np.zeros(8, np.float32), 2, 1.0, 0.0).reshape(4, 2),
                              want)
    assert np.array_equal(oracle.spmm_f64_rowmajor(4, 2, rowptr, colind, val, B, 2, np.zeros(8, np.float32), 2, 1.0,
                                                   0.0).reshape(4, 2), want)


@pytest.mark.parametrize("b_rm", [True, False])
@pytest.mark.parametrize("c_rm", [True, False])
@pytest.mark.parametrize("trans_b", [False, True])
def test_spmm_layouts_against_dense(b_rm, c_rm, trans_b):
    """Every (order B, order C, op B) combination against numpy with explicitly built operands."""
    m, k, n = 7, 5, 3
    rowptr, colind, val = random_csr(m, k, 0.5, seed=2, unsorted=True)
    A = dense_from_csr(m, k, rowptr, colind, val)
    rng = np.random.default_rng(3)
    Bmat = rng.uniform(-2, 2, (k, n)).astype(np.float32)       # op(B), k x n
    Cmat = rng.uniform(-2, 2, (m, n)).astype(np.float32)
    ldb, ldc = 9, 11
    # storage of B: the matrix whose op() is Bmat, in the requested order with padding
    stored = Bmat.T if trans_b else Bmat                        # what sits in memory as a 2-D array
    r, c = stored.shape
    Bflat = np.zeros(ldb * 12, np.float32)
    for i in range(r):
        for j in range(c):
            Bflat[(i * ldb + j) if b_rm else (j * ldb + i)] = stored[i, j]
    Cflat = np.full(ldc * 12, 7.0, np.float32)
    for i in range(m):
        for j in range(n):
            Cflat[(i * ldc + j) if c_rm else (j * ldc + i)] = Cmat[i, j]
    want = (1.5 * (A @ Bmat.astype(np.float64)) + 0.5 * Cmat).astype(np.float32)
    for fn in (oracle.spmm_f64, oracle.spmm_f32):
        out = fn(m, n, rowptr, colind, val, Bflat, ldb, Cflat, ldc, 1.5, 0.5, b_row_major=b_rm, trans_b=trans_b,
                 c_row_major=c_rm)
        got = np.array([[out[(i * ldc + j) if c_rm else (j * ldc + i)] for j in range(n)] for i in range(m)])
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
        touched = np.zeros(out.size, bool)
        for i in range(m):
            for j in range(n):
                touched[(i * ldc + j) if c_rm else (j * ldc + i)] = True
        assert np.all(out[~touched] == 7.0)


def test_spmm_column_is_spmv_and_rowmajor_variant_identical():
    m, k, n = 40, 30, 6
    rowptr, colind, val = random_csr(m, k, 0.2, seed=4)
    rng = np.random.default_rng(4)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    full = oracle.spmm_f64(m, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 2.0, -1.0).reshape(m, n)
    fast = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 2.0, -1.0).reshape(m, n)
    assert np.array_equal(full, fast)
    for j in range(n):
        col = oracle.spmv_f64(m, k, rowptr, colind, val, np.ascontiguousarray(B[:, j]),
                              np.ascontiguousarray(C[:, j]), 2.0, -1.0)
        assert np.array_equal(full[:, j], col)


def test_spmm_beta_zero_ignores_c():
    m, k, n = 5, 5, 4
    rowptr, colind, val = random_csr(m, k, 0.5, seed=6)
    B = np.ones(k * n, np.float32)
    nanC = np.full(m * n, np.nan, np.float32)
    out = oracle.spmm_f64(m, n, rowptr, colind, val, B, n, nanC, n, 1.0, 0.0)
    assert not np.isnan(out).any()


def test_spmm_int8_saturates_and_matches_numpy():
    m, k, n = 6, 6, 4
    rowptr, colind, _ = random_csr(m, k, 0.6, seed=8)
    rng = np.random.default_rng(8)
    val = rng.integers(-128, 128, colind.size).astype(np.int8)
    B = rng.integers(-128, 128, (k, n)).astype(np.int8)
    C = rng.integers(-100, 100, (m, n)).astype(np.int32)
    A = np.zeros((m, k), np.int64)
    for r in range(m):
        for p in range(rowptr[r], rowptr[r + 1]):
            A[r, colind[p]] += int(val[p])
    want = 3 * (A @ B.astype(np.int64)) - 2 * C
    got = oracle.spmm_i8(m, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 3, -2).reshape(m, n)
    assert np.array_equal(got, want)
    sat = oracle.spmm_i8(m, n, rowptr, colind, val, B.ravel(), n, C.ravel(), n, 2 ** 30, 0).reshape(m, n)
    assert np.array_equal(sat, np.clip((2 ** 30) * (A @ B.astype(np.int64)), -2 ** 31, 2 ** 31 - 1))


# ------------------------------------------------------------------- fp16

def test_fp16_conversions_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(h)
    ref = h.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32), ref.view(np.uint32))          # every pattern, NaN payloads included
    back = oracle.f32_to_f16_bits(f)
    finite = ~np.isnan(ref)
    assert np.array_equal(back[finite], h[finite])
    assert np.all((back[~finite] & 0x7C00) == 0x7C00) and np.all((back[~finite] & 0x03FF) != 0)


def test_fp16_rounding_matches_ieee():
    rng = np.random.default_rng(0)
    r = (rng.standard_normal(200000) * 10.0 ** rng.integers(-9, 6, 200000)).astype(np.float32)
    special = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                        2.0 ** -25 * 1.0000001, 2.0 ** -14, 5.9604645e-8, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11],
                       np.float32)
    a = np.concatenate([r, special])
    with np.errstate(over="ignore"):
        want = a.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(a), want)


# --------------------------------------------------------------- verifier

def test_mere_mare_hand_computed():
    eps = 2.0 ** -14
    gold = np.array([1.0, 2.0, -4.0], np.float32)
    out = np.array([1.5, 2.0, -5.0], np.float32)        # middle element is bit-equal: skipped
    mere, mare, mism, counted = oracle.mere_mare(out, gold)
    r0, r2 = 0.5 / (1.0 + eps), 1.0 / (4.0 + eps)
    assert counted == 2 and mism == 0
    assert mere == pytest.approx((r0 + r2) / 2, rel=1e-12) and mare == pytest.approx(r0, rel=1e-12)
    # NaN on both sides is skipped, on one side only it is a mismatch (test/frame/verify.h:117-133)
    mere, mare, mism, counted = oracle.mere_mare(np.array([np.nan, np.nan, 1.0], np.float32),
                                                 np.array([np.nan, 1.0, np.inf], np.float32))
    assert (mism, counted) == (2, 0)


# ------------------------------------------------------------- generators

def _fixture():
    with open(os.path.join(GOLDEN, "fill_generator.json")) as f:
        return json.load(f)


def test_fill_generator_matches_committed_fixture():
    """The restated generator reproduces the arrays the reference's own generator produced
    (fingerprints written by tests/golden/make_fill_fixture.py from oracle/_ref)."""
    for case in _fixture()["csr"]:
        if case["nnz_hint"] <= 0:
            continue  # binomial row lengths: restated in C++ (tests/cpp/frame.h), checked by frame_selftest
        rowptr, colind, val = oracle.fill_csr(case["seed"], case["rows"], case["cols"], case["nnz_hint"], case["lo"],
                                              case["hi"], case["empty_row_prob"])
        assert colind.size == case["nnz"]
        assert oracle.fnv1a(rowptr) == int(case["rowptr_fnv1a"], 16)
        assert oracle.fnv1a(colind) == int(case["colind_fnv1a"], 16)
        assert oracle.fnv1a(val) == int(case["values_fnv1a"], 16)
        assert colind[:4].tolist() == case["colind_head"]
        assert val[:2].tolist() == pytest.approx(case["values_head"], rel=0, abs=0)
    for case in _fixture()["dense"]:
        v = oracle.fill_dense(case["seed"], case["n"], case["lo"], case["hi"])
        assert oracle.fnv1a(v) == int(case["fnv1a"], 16)
        assert v[:2].tolist() == case["head"]


def test_fill_generator_matches_reference_library():
    """Where oracle/_ref was built, compare with the reference generator directly on more shapes."""
    if oracle.ref_fill() is None:
        pytest.skip("oracle/_ref not built (no reference tree on this machine)")
    for seed, rows, cols, hint, p in [(42, 4096, 4096, 65536, 0.0), (1, 10, 7, 40, 0.0), (9, 300, 50, 3000, 0.25),
                                      (123, 64, 64, 64 * 64, 0.0), (5, 1, 1000, 999, 0.0)]:
        a = oracle.fill_csr(seed, rows, cols, hint, -3.0, 3.0, p)
        b = oracle.ref_fill_csr(seed, rows, cols, hint, empty_row_prob=p, lo=-3.0, hi=3.0)
        assert all(np.array_equal(u, v) for u, v in zip(a, b))
    assert np.array_equal(oracle.fill_dense(43, 1000, -1.0, 1.0), oracle.ref_fill_dense(43, 1000, -1.0, 1.0))


def test_c1_structure():
    """The reference-runnable configuration: 4096 x 4096, exactly 16 sorted distinct columns per row."""
    rowptr, colind, val = oracle.fill_csr(42, 4096, 4096, 65536, -1.0, 1.0)
    assert np.array_equal(np.diff(rowptr), np.full(4096, 16))
    c = colind.reshape(4096, 16)
    assert np.all(np.diff(c, axis=1) > 0) and c.min() >= 0 and c.max() < 4096
    assert np.all(np.abs(val) <= 1.0)


# ------------------------------------------- the SpMM test programs' seeded generators

def _lemire(raw, rng_range):
    """libstdc++'s uniform_int_distribution on a 32-bit engine, from an iterator of raw engine outputs."""
    while True:
        product = int(next(raw)) * rng_range
        low = product & 0xFFFFFFFF
        if low >= rng_range or low >= ((1 << 32) - rng_range) % rng_range:
            return product >> 32


def _python_spmm22(rows, cols, nnz, raw):
    """generate_random_csr of the arch22 SpMM test program, written again in Python over numpy's MT19937 stream
    (RandomState(42) seeds like std::mt19937(42)): an independent second statement for small cases."""
    offsets, indices = [0], []
    for i in range(rows):
        used = set()
        for _ in range(nnz // rows + (1 if i < nnz % rows else 0)):
            col = _lemire(raw, cols)
            while col in used:
                col = _lemire(raw, cols)
            used.add(col)
            indices.append(col)
        offsets.append(len(indices))
    return np.array(offsets, np.int32), np.array(indices, np.int32)


def test_spmm22_generator_against_a_second_statement_and_its_invariants():
    raw = iter(np.random.RandomState(42).randint(0, 2 ** 32, size=200000, dtype=np.uint64))
    oracle.spmm22_seek(0)
    for rows, cols, nnz in ((16, 16, 128), (7, 300, 100), (40, 40, 1000), (3, 5, 15)):  # one engine, never re-seeded
        want_ptr, want_col = _python_spmm22(rows, cols, nnz, raw)
        ptr, col, val = oracle.spmm22_csr("uniform", rows, cols, nnz)
        assert np.array_equal(ptr, want_ptr) and np.array_equal(col, want_col)
        assert np.array_equal(np.diff(ptr), [nnz // rows + (i < nnz % rows) for i in range(rows)])
        assert np.array_equal(val, np.float32(0.1) + np.float32(0.0001) * np.arange(nnz, dtype=np.float32))
    used = oracle.spmm22_outputs_used()
    # the engine position is what seek() reproduces: the same case again from that position gives the same matrix
    a = oracle.spmm22_csr("powerlaw", 50, 64, 900)
    oracle.spmm22_seek(used)
    b = oracle.spmm22_csr("powerlaw", 50, 64, 900)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    # store=False moves the engine exactly as far
    after = oracle.spmm22_outputs_used()
    oracle.spmm22_seek(used)
    assert oracle.spmm22_csr("powerlaw", 50, 64, 900, store=False) == a[1].size and oracle.spmm22_outputs_used() == after
    # Zipf shares: truncated nnz * (1 / (i + 1)) / H, the remainder one each to the top rows, capped at the columns
    ptr, col, _ = a
    w = 1.0 / np.arange(1, 51)
    share = (900 * w / w.sum()).astype(np.int64)
    share[: 900 - share.sum()] += 1
    assert np.array_equal(np.diff(ptr), np.minimum(share, 64))
    assert all(np.unique(col[ptr[r]:ptr[r + 1]]).size == ptr[r + 1] - ptr[r] for r in range(50))


def test_spmm22_case_table_positions_are_those_of_the_generators():
    """The engine_outputs_before column of the committed case table, recomputed for the leading cases."""
    import csv
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spmm_arch22_cases.csv")) as f:
        cases = list(csv.DictReader(f))
    assert len(cases) == 200 and cases[0]["engine_outputs_before"] == "0"
    oracle.spmm22_seek(0)
    for c in cases[:25]:
        assert oracle.spmm22_outputs_used() == int(c["engine_outputs_before"])
        oracle.spmm22_csr(c["dist"], int(c["m"]), int(c["k"]), int(c["nnz"]), store=False)


def test_glibc_rand_restated_against_this_hosts_libc():
    """std::rand() of the arch35 SpMM test program is glibc's: the restatement against the C library itself."""
    import ctypes
    libc = ctypes.CDLL("libc.so.6")
    for seed in (42, 43, 44, 45, 46, 1, 0, 2 ** 31 + 5):
        libc.srand(ctypes.c_uint(seed))
        assert [libc.rand() for _ in range(2000)] == list(oracle.glibc_rand_stream(seed, 2000))


def test_spmm35_generator_invariants():
    for seed, m, k, nnz in ((42, 256, 256, 6553), (46, 32, 32, 80), (7, 5, 3, 100)):
        ptr, col, val = oracle.spmm35_random_csr(seed, m, k, nnz)
        lengths = np.minimum([nnz // m + (i < nnz % m) for i in range(m)], k)
        assert np.array_equal(np.diff(ptr), lengths)
        assert all(np.all(np.diff(col[ptr[r]:ptr[r + 1]]) > 0) for r in range(m))     # a std::set: ascending, distinct
        assert col.min() >= 0 and col.max() < k
        want = np.float32(-5.0) + np.float32(10.0) * (np.arange(col.size) % 10001).astype(np.float32) / np.float32(1e4)
        assert np.array_equal(val, want)
    # first row of seed 42: the first distinct values of rand() % 256, sorted
    stream = oracle.glibc_rand_stream(42, 400) % 256
    first = []
    for c in stream:
        if c not in first:
            first.append(int(c))
        if len(first) == 6553 // 256 + 1:
            break
    ptr, col, _ = oracle.spmm35_random_csr(42, 256, 256, 6553)
    assert list(col[: ptr[1]]) == sorted(first)
