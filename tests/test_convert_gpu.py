"""GPU parity tests of the CSR producers (aclsparseXcoo2csr, aclsparseXcsr2coo, aclsparseXcsrsort,
aclsparseXcscsort, aclsparseXcoosortByRow / ByColumn, aclsparseCsr2cscEx2) through the C ABI.  Every output is compared bit for bit with the CPU oracle.

The coo2csr / csr2coo / csr2csc case tables are the reference's own
(test/<op>/arch35/<op>_test.csv, kept as data fixtures under tests/golden/); matrices come
from the reference's fill generator through oracle/_ref where that is built and from a
numpy generator of the same distribution otherwise.  The csrsort cases restate the inputs of
test/csrsort/arch35/csrsort_test.cpp:239-650 (that test has no table).
"""
import csv
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import random_csr, to_dev

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def load_cases(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return list(csv.DictReader(line for line in f if line.strip() and not line.startswith("#")))


def matrix(c, lo=-5.0, hi=5.0):
    """Zero-based CSR of a case row (test/frame/fill.h generator, or its numpy twin)."""
    m, n, seed = int(c["m"]), int(c["n"]), int(c["seed"])
    sparsity = float(c["sparsity"])
    if c["pattern"] == "diag":
        return np.arange(m + 1, dtype=np.int32), np.arange(m, dtype=np.int32), np.ones(m, np.float32)
    if m <= 0 or n <= 0 or sparsity >= 1.0:
        return np.zeros(max(m, 0) + 1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32)
    got = oracle.ref_fill_csr(seed, m, n, -1, sparsity, float(c["empty_row_prob"]), lo, hi)
    if got is None:
        got = random_csr(m, n, 1.0 - sparsity, seed, lo, hi, empty_row_prob=float(c["empty_row_prob"]))
    return got


def dev_i32(a, dev):
    return to_dev(np.ascontiguousarray(a, np.int32), dev)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else None


# ------------------------------------------------------------------ coo2csr

COO2CSR = load_cases("coo2csr_cases.csv")


@pytest.mark.parametrize("c", COO2CSR, ids=[c["case_name"] for c in COO2CSR])
def test_coo2csr_reference_table(osa, gpu_ctx, c):
    dev, stream, handle = gpu_ctx
    m, base = int(c["m"]), int(c["idx_base"])
    if c["pattern"] == "allsame":
        nnz = max(int(m * int(c["n"]) * (1.0 - float(c["sparsity"]))), 1)
        rows = np.zeros(nnz, np.int32)
    else:
        rowptr, colind, _ = matrix(c)
        rows = oracle.csr2coo(rowptr, colind.size)
    rows = rows + base
    d_rows = dev_i32(rows, dev)
    d_ptr = torch.full((m + 1,), -7, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    rc = osa.lib().aclsparseXcoo2csr(handle.h, ptr(d_rows), rows.size, m, ctypes.c_void_p(d_ptr.data_ptr()), base)
    assert rc == 0
    stream.synchronize()
    assert np.array_equal(d_ptr.cpu().numpy(), oracle.coo2csr(rows, m, base))
    assert np.array_equal(d_rows.cpu().numpy(), rows)


@pytest.mark.parametrize("m,nnz,base", [(1, 1, 0), (5_000_000, 3_000_000, 1), (1000, 4_000_000, 0), (2049, 0, 1),
                                        (4_194_304, 20_000_000, 0)])
def test_coo2csr_large_and_unsorted(osa, gpu_ctx, m, nnz, base):
    """Sizes around the scan tile and far above it; a second run on shuffled input must still equal the
    count-based golden (coo2csr_golden.h:57-66 counts, it does not search)."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(m + nnz)
    rows = np.sort(rng.integers(0, m, nnz)).astype(np.int32) + base
    for shuffled in (False, True):
        if shuffled:
            rng.shuffle(rows)
            rows[: min(5, nnz)] = m + base + 3          # out of range: not counted
        d_rows = dev_i32(rows, dev)
        d_ptr = torch.empty(m + 1, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        assert osa.lib().aclsparseXcoo2csr(handle.h, ptr(d_rows), nnz, m, ctypes.c_void_p(d_ptr.data_ptr()), base) == 0
        stream.synchronize()
        assert np.array_equal(d_ptr.cpu().numpy(), oracle.coo2csr(rows, m, base))


# ------------------------------------------------------------------ csr2coo

CSR2COO = load_cases("csr2coo_cases.csv")


@pytest.mark.parametrize("c", CSR2COO, ids=[c["case_name"] for c in CSR2COO])
def test_csr2coo_reference_table(osa, gpu_ctx, c):
    dev, stream, handle = gpu_ctx
    m, n, base = int(c["m"]), int(c["n"]), int(c["idx_base"])
    rowptr, colind, val = matrix(c) if c["pattern"] != "csc" else matrix(dict(c, pattern="random"))
    if c["pattern"] == "csc":                       # the column offsets of the same matrix, expanded to column indices
        rowptr, _, _ = oracle.csr2csc(m, n, rowptr, colind, val)
        m = n
    nnz = int(rowptr[-1])
    rowptr = rowptr + base
    d_ptr = dev_i32(rowptr, dev)
    d_rows = torch.full((nnz,), -7, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    assert osa.lib().aclsparseXcsr2coo(handle.h, ptr(d_ptr), nnz, m, ptr(d_rows), base) == 0
    stream.synchronize()
    assert np.array_equal(d_rows.cpu().numpy(), oracle.csr2coo(rowptr, nnz, base))


def test_csr2coo_row_length_mix(osa, gpu_ctx):
    """Rows on both sides of the 16-entry switch, very long rows, runs of empty rows, m not a multiple of 64."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(4)
    lengths = rng.integers(0, 40, 100_003)
    lengths[rng.integers(0, lengths.size, 2000)] = 0
    lengths[[7, 50_000, 100_002]] = [300_000, 17, 65_000]
    lengths[1000:3000] = 0
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    nnz = int(rowptr[-1])
    for base in (0, 1):
        d_ptr = dev_i32(rowptr + base, dev)
        d_rows = torch.full((nnz,), -7, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        assert osa.lib().aclsparseXcsr2coo(handle.h, ptr(d_ptr), nnz, lengths.size, ptr(d_rows), base) == 0
        stream.synchronize()
        assert np.array_equal(d_rows.cpu().numpy(), oracle.csr2coo(rowptr + base, nnz, base))


@pytest.mark.parametrize("name,rowptr,nnz,base,compare", [
    ("non_monotonic", [0, 3, 1, 4], 4, 0, False),          # rows 0 and 2 overlap: which one wins is not defined
    ("nnz_mismatch", [0, 1, 2, 3], 5, 0, True),
    ("idxbase_mismatch", [0, 1, 2, 3, 4], 4, 1, True),
    ("simd_row_exceeds_nnz", [0, 5], 3, 0, True),
    ("simd_non_monotonic", [0, 250, 100], 300, 0, True),
    ("simd_idxbase_mismatch", [0, 3], 3, 1, True)])
def test_csr2coo_malformed_offsets_are_skipped(osa, gpu_ctx, name, rowptr, nnz, base, compare):
    """The abnormal-input cases of the reference test (csr2coo_test.cpp, ABN_*): offsets that do not describe a
    range inside [0, nnz) are not an error; such rows are skipped and nothing outside cooRowInd[0, nnz) is written
    (csr2coo_golden.h:51-53).  The output starts as zeros, as in that test, with a guard element behind it."""
    dev, stream, handle = gpu_ctx
    rowptr = np.asarray(rowptr, np.int32)
    d_ptr = dev_i32(rowptr, dev)
    d_rows = torch.zeros(nnz + 1, dtype=torch.int32, device=dev)
    d_rows[nnz] = -99
    torch.cuda.synchronize()
    assert osa.lib().aclsparseXcsr2coo(handle.h, ptr(d_ptr), nnz, rowptr.size - 1, ptr(d_rows), base) == 0
    stream.synchronize()
    got = d_rows.cpu().numpy()
    assert got[nnz] == -99
    if compare:
        assert np.array_equal(got[:nnz], oracle.csr2coo(rowptr, nnz, base))


# ------------------------------------------------------------------ csrsort

def run_csrsort(osa, gpu_ctx, m, n, rowptr, colind, base=0, perm=None, misalign=0):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    nnz = int(colind.size)
    perm = np.arange(nnz, dtype=np.int32) if perm is None else perm
    d_ptr, d_col, d_perm = dev_i32(rowptr, dev), dev_i32(colind, dev), dev_i32(perm, dev)
    size = ctypes.c_size_t(0)
    assert L.aclsparseXcsrsort_bufferSizeExt(handle.h, m, n, nnz, ptr(d_ptr), ptr(d_col), ctypes.byref(size)) == 0
    buf = torch.empty(size.value + 64, dtype=torch.uint8, device=dev)
    descr = ctypes.c_void_p(None)
    assert L.aclsparseCreateMatDescr(ctypes.byref(descr)) == 0
    L.aclsparseSetMatIndexBase(descr, base)
    torch.cuda.synchronize()
    rc = L.aclsparseXcsrsort(handle.h, m, n, nnz, descr, ptr(d_ptr), ptr(d_col), ptr(d_perm),
                             ctypes.c_void_p(buf.data_ptr() + misalign) if nnz else None)
    assert rc == 0
    stream.synchronize()
    L.aclsparseDestroyMatDescr(descr)
    want_c, want_p = oracle.csrsort(rowptr, colind, perm, base)
    assert np.array_equal(d_ptr.cpu().numpy(), rowptr)
    assert np.array_equal(d_col.cpu().numpy(), want_c) and np.array_equal(d_perm.cpu().numpy(), want_p)


def _rows(lengths, colfn):
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    col = np.concatenate([np.asarray(colfn(r, int(l)), np.int64) for r, l in enumerate(lengths)] + [np.zeros(0, np.int64)])
    return rowptr, col.astype(np.int32)


def _skewed(row):
    return 10000 if row % 64 == 0 else 2048 if row % 8 == 0 else (row % 7 if row % 5 != 0 else 0)


SORT_CASES = {
    "Basic": lambda: (3, 3, np.array([0, 3, 6, 9], np.int32), np.array([2, 1, 0, 0, 2, 1, 1, 2, 0], np.int32)),
    "EmptyRows": lambda: (4, 5, np.array([0, 0, 2, 2, 4], np.int32), np.array([3, 1, 4, 2], np.int32)),
    "AlreadySorted": lambda: (3, 5, np.array([0, 2, 4, 6], np.int32), np.array([0, 1, 2, 3, 0, 4], np.int32)),
    "Reverse": lambda: (1, 64, np.array([0, 64], np.int32), np.arange(63, -1, -1, dtype=np.int32)),
    "DuplicateCols": lambda: (2, 4, np.array([0, 6, 9], np.int32), np.array([3, 1, 3, 1, 0, 3, 2, 2, 2], np.int32)),
    "EmptyMatrix": lambda: (5, 5, np.zeros(6, np.int32), np.zeros(0, np.int32)),
    "SingleElemRows": lambda: (4, 9, np.arange(5, dtype=np.int32), np.array([8, 0, 3, 3], np.int32)),
    "ManySmallRows": lambda: (200, 10) + _rows(np.random.default_rng(99).integers(0, 4, 200),
                                               lambda r, l: np.random.default_rng(r).integers(0, 10, l)),
    "MultiCoreSkewedRows": lambda: (257, 4096) + _rows([_skewed(r) for r in range(257)],
                                                        lambda r, l: (r * 131 + l - np.arange(l)) % 4096),
    "LongRow": lambda: (1, 1000, np.array([0, 1000], np.int32), np.random.default_rng(123).permutation(1000).astype(np.int32)),
    "LongRowMultiRun": lambda: (1, 4096, np.array([0, 32768], np.int32),
                                np.random.default_rng(2026).permutation(np.arange(32768) % 4096).astype(np.int32)),
    "SingleHugeRow": lambda: (1, 65536, np.array([0, 1 << 20], np.int32),
                              ((np.arange(1 << 20, dtype=np.uint64) * 65521 + 7919) % 4096).astype(np.int32)),
    "LargeNnzMultiCoreRows": lambda: (64, 4096) + _rows([16384] * 64, lambda r, l: (r * 131 + l - np.arange(l)) % 4096),
    "RunBoundaries": lambda: (12, 5000) + _rows([63, 64, 65, 127, 128, 129, 2047, 2048, 2049, 4095, 4096, 4097],
                                                lambda r, l: np.random.default_rng(r).integers(0, 5000, l)),
    "AlternatingTinyAndLarge": lambda: (400, 3000) + _rows([1 if r % 2 else 1500 for r in range(400)],
                                                            lambda r, l: (np.arange(l) * 7919 + r) % 3000),
}


def _mixed_stress(run):
    """MixedShortAndMultiRunStress of the reference test (csrsort_test.cpp:604-656) with `run` for its run size."""
    lengths = [[0, 1, 17, run, run + 1, run + 37, 63, min(run, 2047)][row % 8] for row in range(193)]
    return (193, 16384) + _rows(lengths, lambda r, l: (r * 131 + (l - np.arange(l)) * 29 + np.arange(l) % 11) % 16384)


def _run_boundaries(run):
    """RunSizeBoundaries (csrsort_test.cpp:501-519): rows of run - 1, run and run + 1 entries, columns descending."""
    nnz = 3 * run
    return 3, 4096, np.array([0, run - 1, 2 * run - 1, nnz], np.int32), ((nnz - np.arange(nnz)) % 4096).astype(np.int32)


# The reference sizes these cases by the run its on-chip buffer holds (CsrsortTiling::FindMaxRunSize); here they are
# sized by the row lengths at which this library changes kernels: 64 (registers), 2048 (LDS), 16 384 (1024 lanes).
SORT_CASES.update({
    "RandomMedium": lambda: (50, 50) + _rows(np.random.default_rng(77).binomial(50, 0.15, 50),
                                             lambda r, l: np.random.default_rng(77 + r).permutation(50)[:l]),
    "Non64ElementCounts": lambda: (5, 257) + _rows([7, 63, 64, 65, 127], lambda r, l: (r * 37 + l - np.arange(l)) % 257),
    "LargeAlignmentBoundaryMatrix": lambda: (640, 4096) + _rows(
        [[31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 513, 1025][r % 15] for r in range(640)],
        lambda r, l: (r * 193 + np.arange(l) * 61 + l - np.arange(l)) % 4096),
    "RunSizeBoundaries64": lambda: _run_boundaries(64),
    "RunSizeBoundaries2048": lambda: _run_boundaries(2048),
    "RunSizeBoundaries16384": lambda: _run_boundaries(16384),
    "MixedShortAndMultiRunStress64": lambda: _mixed_stress(64),
    "MixedShortAndMultiRunStress2048": lambda: _mixed_stress(2048),
    "MixedShortAndMultiRunStress16384": lambda: _mixed_stress(16384),
})


def test_csrsort_alternating_rows_with_custom_perm(osa, gpu_ctx):
    """AlternatingTinyAndLargeShortRows as the reference runs it (csrsort_test.cpp:544-572): rows of 7 and of 4093
    entries in turn, 257 distinct columns (long runs of equal keys) and P = row * 100000 + position."""
    lengths = [7 if r % 2 == 0 else 4093 for r in range(512)]
    rowptr, colind = _rows(lengths, lambda r, l: (r * 17 + l - np.arange(l)) % 257)
    perm = np.concatenate([r * 100000 + np.arange(l) for r, l in enumerate(lengths)]).astype(np.int32)
    run_csrsort(osa, gpu_ctx, 512, 8192, rowptr, colind, perm=perm)


@pytest.mark.parametrize("name", list(SORT_CASES))
def test_csrsort_reference_cases(osa, gpu_ctx, name):
    m, n, rowptr, colind = SORT_CASES[name]()
    run_csrsort(osa, gpu_ctx, m, n, rowptr, colind)


def test_csrsort_base1_custom_perm_unaligned_buffer(osa, gpu_ctx):
    """Base1 / NonIdentityP / NonAlignedBuffer of the reference test in one matrix."""
    rng = np.random.default_rng(8)
    m, n = 3000, 70000
    lengths = rng.integers(0, 100, m)
    lengths[[5, 2999]] = [5000, 20000]
    rowptr, colind = _rows(lengths, lambda r, l: rng.integers(0, n, l))
    perm = rng.integers(-1000, 1000, colind.size).astype(np.int32)
    run_csrsort(osa, gpu_ctx, m, n, rowptr + 1, colind + 1, base=1, perm=perm, misalign=4)


@pytest.mark.parametrize("mean", [3, 7, 14, 40])
@pytest.mark.parametrize("n,base", [(1000, 0), ((1 << 26) - 70, 1), ((1 << 29) + 5, 0), (2 ** 31 - 2, 1)])
def test_csrsort_short_rows_every_group_size_and_key_width(osa, gpu_ctx, mean, n, base):
    """Rows sorted in registers by groups of 8, 16, 32 or 64 lanes (chosen from the mean row length), the keys
    column-and-lane packed into 32 bits where the column range leaves room and 64-bit otherwise: few and many
    distinct columns, the largest column indices an int32 holds, both index bases, rows of every length up to the
    group size and a few beyond it."""
    rng = np.random.default_rng(mean * 1000 + n % 997)
    m = 5000
    lengths = rng.integers(0, 2 * mean + 1, m)
    lengths[rng.choice(m, 20, replace=False)] = rng.integers(2 * mean, 2 * mean + 70, 20)
    hi = min(n, 2 ** 31 - 1 - base)
    rowptr, colind = _rows(lengths, lambda r, l: np.concatenate([rng.integers(0, hi, l - l // 3),
                                                                 hi - 1 - rng.integers(0, min(hi, 50), l // 3)]))
    run_csrsort(osa, gpu_ctx, m, n, rowptr + base, colind + base, base=base)


def test_csrsort_many_rows(osa, gpu_ctx):
    """A million short rows (one wavefront each) with a power-law tail."""
    rng = np.random.default_rng(9)
    m, n = 1_000_000, 1_000_000
    lengths = np.minimum((1.0 / rng.uniform(2e-5, 1.0, m)).astype(np.int64), 50000)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, n, int(rowptr[-1])).astype(np.int32)
    run_csrsort(osa, gpu_ctx, m, n, rowptr, colind)


@pytest.mark.parametrize("n", [7, 3_000_000])
def test_csrsort_rows_either_side_of_the_wide_launch(osa, gpu_ctx, n):
    """Rows of 16 383 - 16 385 entries and a few far longer ones among 3000 short rows: the listed rows are sorted by
    two launches, 256 lanes a row up to 16 384 entries and 1024 beyond; few distinct columns (long runs of equal
    keys, whose order P shows) and many (all key bits in use)."""
    rng = np.random.default_rng(n)
    lengths = rng.integers(0, 40, 3000)
    lengths[[0, 17, 18, 1500, 2998, 2999]] = [16385, 16384, 16383, 131_073, 40_000, 16_400]
    rowptr, colind = _rows(lengths, lambda r, l: rng.integers(0, n, l))
    run_csrsort(osa, gpu_ctx, 3000, n, rowptr, colind)


@pytest.mark.parametrize("lengths,n,base", [([300_000], 2_000_000, 0), ([0, 40_000, 0, 9_000, 70_000, 1, 0], 50_000, 1),
                                            ([4096] * 33, 17, 0), ([5000, 4000, 3500], 1, 0)])
def test_csrsort_long_rows_on_average(osa, gpu_ctx, lengths, n, base):
    """Thousands of entries per row on average: the whole matrix is sorted by the device-wide radix passes (by
    column, then stably by row) instead of a workgroup per row.  Repeated columns keep their order (P tells), empty
    rows, one row only, one column only, index base 1, P not the identity."""
    rng = np.random.default_rng(len(lengths) + n)
    assert sum(lengths) // len(lengths) >= 4096
    rowptr, colind = _rows(lengths, lambda r, l: rng.integers(0, n, l))
    perm = rng.integers(-1000, 1000, colind.size).astype(np.int32) if base else None
    run_csrsort(osa, gpu_ctx, len(lengths), n, rowptr + base, colind + base, base=base, perm=perm, misalign=4 * base)


# ------------------------------------------------------------------ cscsort

def run_cscsort(osa, gpu_ctx, m, n, colptr, rowind, base=0, perm=None):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    nnz = int(rowind.size)
    perm = np.arange(nnz, dtype=np.int32) if perm is None else perm
    d_ptr, d_row, d_perm = dev_i32(colptr, dev), dev_i32(rowind, dev), dev_i32(perm, dev)
    size = ctypes.c_size_t(0)
    assert L.aclsparseXcscsort_bufferSizeExt(handle.h, m, n, nnz, ptr(d_ptr), ptr(d_row), ctypes.byref(size)) == 0
    buf = torch.empty(size.value + 256, dtype=torch.uint8, device=dev)
    aligned = (buf.data_ptr() + 127) // 128 * 128                    # the reference asks for 128-byte alignment
    descr = ctypes.c_void_p(None)
    assert L.aclsparseCreateMatDescr(ctypes.byref(descr)) == 0
    L.aclsparseSetMatIndexBase(descr, base)
    torch.cuda.synchronize()
    if nnz:
        assert L.aclsparseXcscsort(handle.h, m, n, nnz, descr, ptr(d_ptr), ptr(d_row), ptr(d_perm),
                                   ctypes.c_void_p(aligned + 4)) == osa.ACL_SPARSE_STATUS_INVALID_VALUE
    assert L.aclsparseXcscsort(handle.h, m, n, nnz, descr, ptr(d_ptr), ptr(d_row), ptr(d_perm),
                               ctypes.c_void_p(aligned) if nnz else None) == 0
    stream.synchronize()
    L.aclsparseDestroyMatDescr(descr)
    want_r, want_p = oracle.cscsort(colptr, rowind, perm, base)
    assert np.array_equal(d_ptr.cpu().numpy(), colptr)
    assert np.array_equal(d_row.cpu().numpy(), want_r) and np.array_equal(d_perm.cpu().numpy(), want_p)


@pytest.mark.parametrize("name", list(SORT_CASES))
def test_cscsort_reference_cases(osa, gpu_ctx, name):
    """test/cscsort/arch35/cscsort_test.cpp:245-530 builds the same shapes as the csrsort test with the roles of
    rows and columns exchanged (Basic, EmptyCols, Reverse, DuplicateRows, ManySmallCols, MultiCoreSkewedCols,
    LongCol, LongColMultiRun, RandomMedium, RunSizeBoundaries, LargeNnzMultiCore ...): the csrsort cases, read
    as CSC matrices of n x m."""
    cols_, rows_, colptr, rowind = SORT_CASES[name]()
    run_cscsort(osa, gpu_ctx, rows_, cols_, colptr, rowind)


def test_cscsort_base1_custom_perm_last_column_empty_single_row(osa, gpu_ctx):
    """Base1 / NonIdentityP / LastColEmpty / SingleRow of the reference test."""
    rng = np.random.default_rng(18)
    m, n = 70000, 3000
    lengths = rng.integers(0, 100, n)
    lengths[[5, 2998]] = [5000, 20000]
    lengths[-1] = 0
    colptr, rowind = _rows(lengths, lambda c, l: rng.integers(0, m, l))
    perm = rng.integers(-1000, 1000, rowind.size).astype(np.int32)
    run_cscsort(osa, gpu_ctx, m, n, colptr + 1, rowind + 1, base=1, perm=perm)
    # one row: every column holds the row 0 once or not at all, several times in one (a stable no-op)
    colptr = np.array([0, 1, 1, 4, 5], np.int32)
    run_cscsort(osa, gpu_ctx, 1, 4, colptr, np.zeros(5, np.int32), perm=np.array([9, 8, 7, 6, 5], np.int32))
    run_cscsort(osa, gpu_ctx, 6, 6, np.zeros(7, np.int32), np.zeros(0, np.int32))       # EmptyMatrix


# ------------------------------------------------------------------ coosort

def run_coosort(osa, gpu_ctx, m, n, rows, cols, by_row, perm=None):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    rows, cols = np.ascontiguousarray(rows, np.int32), np.ascontiguousarray(cols, np.int32)
    nnz = int(rows.size)
    perm = np.arange(nnz, dtype=np.int32) if perm is None else perm
    d_r, d_c, d_p = dev_i32(rows, dev), dev_i32(cols, dev), dev_i32(perm, dev)
    size = ctypes.c_size_t(0)
    assert L.aclsparseXcoosort_bufferSizeExt(handle.h, m, n, nnz, ptr(d_r), ptr(d_c), ctypes.byref(size)) == 0
    assert (size.value > 0) == (nnz > 0)
    buf = torch.empty(size.value + 64, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    fn = L.aclsparseXcoosortByRow if by_row else L.aclsparseXcoosortByColumn
    # (the reference asks for no alignment of the buffer: 4 bytes off the allocation)
    assert fn(handle.h, m, n, nnz, ptr(d_r), ptr(d_c), ptr(d_p), ctypes.c_void_p(buf.data_ptr() + 4) if nnz else None) == 0
    stream.synchronize()
    want = oracle.coosort(rows, cols, perm, by_row)
    for got, exp, what in zip((d_r, d_c, d_p), want, ("rows", "cols", "P")):
        assert np.array_equal(got.cpu().numpy(), exp), what


@pytest.mark.parametrize("by_row", [True, False])
def test_coosort_reference_small_cases(osa, gpu_ctx, by_row):
    """ByRowBasic, ByColumnBasic, ByRowStableDuplicateKey, NnzZero and one entry
    (test/coosort/arch35/coosort_test.cpp:233-262, :531-546)."""
    run_coosort(osa, gpu_ctx, 4, 4, [2, 0, 3, 0, 1, 2], [1, 3, 2, 1, 0, 3], by_row)
    run_coosort(osa, gpu_ctx, 3, 5, [0, 0, 0, 1, 1, 2], [4, 1, 3, 2, 0, 9], by_row)
    run_coosort(osa, gpu_ctx, 4, 4, [], [], by_row)
    run_coosort(osa, gpu_ctx, 4, 4, [3], [2], by_row, perm=np.array([77], np.int32))


@pytest.mark.parametrize("nnz,m,n", [(12, 8, 8), (49, 16, 16), (103, 32, 24), (215, 40, 64), (388, 64, 64),
                                     (3839, 100, 100), (3840, 100, 100), (3841, 100, 100), (20000, 300, 200),
                                     (100_000, 5000, 7000), (1_000_003, 65536, 65536), (3_000_000, 4, 3)])
@pytest.mark.parametrize("by_row", [True, False])
def test_coosort_random_matrices(osa, gpu_ctx, nnz, m, n, by_row):
    """ByRowRandom_seed42..46 / ByColumnRandom (nnz 12 .. 388, coosort_test.cpp:266-352) and the multi-core cases
    (:563-680, hundreds of thousands of entries), duplicates of whole (row, column) pairs included: with few
    distinct pairs (4 x 3 over three million entries) the order inside a pair is what P shows.  Sizes either
    side of the 3840-entry tile of a pass."""
    rng = np.random.default_rng(nnz + (1 if by_row else 0))
    run_coosort(osa, gpu_ctx, m, n, rng.integers(0, m, nnz), rng.integers(0, n, nnz), by_row)


@pytest.mark.parametrize("by_row", [True, False])
def test_coosort_signed_indices_custom_perm_and_sorted_input(osa, gpu_ctx, by_row):
    """Indices are compared as signed integers and need not lie inside the matrix
    (test/coosort/arch35/coosort_golden.h:29): negative ones, the whole int32 range, a range of one value; P not
    the identity travels with its entry; input already sorted, and sorted the other way."""
    rng = np.random.default_rng(5)
    nnz = 50_000
    run_coosort(osa, gpu_ctx, 10, 10, rng.integers(-700, 300, nnz), rng.integers(-5, 5, nnz), by_row,
                perm=rng.integers(-10 ** 9, 10 ** 9, nnz).astype(np.int32))
    run_coosort(osa, gpu_ctx, 10, 10, rng.integers(-2 ** 31, 2 ** 31 - 1, nnz), rng.integers(-2 ** 31, 2 ** 31 - 1, nnz),
                by_row)
    ends = np.array([-2 ** 31, 2 ** 31 - 1, 0, -1, 1, 2 ** 31 - 1, -2 ** 31], np.int64)
    run_coosort(osa, gpu_ctx, 10, 10, ends, ends[::-1], by_row)
    run_coosort(osa, gpu_ctx, 10, 10, np.full(nnz, 7), rng.integers(0, 1000, nnz), by_row)     # one row only
    run_coosort(osa, gpu_ctx, 10, 10, np.full(5000, -3), np.full(5000, 12), by_row)           # one entry repeated
    r, c = np.divmod(np.arange(nnz), 250)
    run_coosort(osa, gpu_ctx, 200, 250, r, c, by_row)                                          # sorted by row
    run_coosort(osa, gpu_ctx, 200, 250, r[::-1], c[::-1], by_row)                              # reversed


def test_coosort_then_coo2csr_is_csr2csc(osa, gpu_ctx):
    """Sorting a matrix's COO triples by column and compressing the column indices gives its CSC form: the same
    row indices, values (through P) and column offsets as aclsparseCsr2cscEx2's oracle."""
    m, n = 3000, 2000
    rowptr, colind, val = random_csr(m, n, 0.01, 4, unsorted=True)
    nnz = colind.size
    rows = oracle.csr2coo(rowptr, nnz)
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    d_r, d_c, d_p = dev_i32(rows, dev), dev_i32(colind, dev), dev_i32(np.arange(nnz), dev)
    size = ctypes.c_size_t(0)
    assert L.aclsparseXcoosort_bufferSizeExt(handle.h, m, n, nnz, ptr(d_r), ptr(d_c), ctypes.byref(size)) == 0
    buf = torch.empty(size.value, dtype=torch.uint8, device=dev)
    assert L.aclsparseXcoosortByColumn(handle.h, m, n, nnz, ptr(d_r), ptr(d_c), ptr(d_p), ptr(buf)) == 0
    d_ptr = torch.empty(n + 1, dtype=torch.int32, device=dev)
    assert L.aclsparseXcoo2csr(handle.h, ptr(d_c), nnz, n, ptr(d_ptr), 0) == 0
    stream.synchronize()
    colptr, rowind, cval = oracle.csr2csc(m, n, rowptr, colind, val)
    assert np.array_equal(d_ptr.cpu().numpy(), colptr) and np.array_equal(d_r.cpu().numpy(), rowind)
    assert np.array_equal(val[d_p.cpu().numpy()].view(np.uint32), cval.view(np.uint32))


# ------------------------------------------------------------------ csr2csc

CSR2CSC = load_cases("csr2csc_cases.csv")
NP_TYPE = {"FP32": np.float32, "FP16": np.float16, "BF16": np.uint16, "INT8": np.int8}


def run_csr2csc(osa, gpu_ctx, m, n, rowptr, colind, val, vt, numeric, base, use_buffer=True):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    nnz = int(colind.size)
    acl = {np.dtype(np.float32): osa.ACL_FLOAT, np.dtype(np.float16): osa.ACL_FLOAT16, np.dtype(np.uint16): osa.ACL_BF16,
           np.dtype(np.int8): osa.ACL_INT8}[np.dtype(vt)]
    d_ptr, d_col = dev_i32(rowptr, dev), dev_i32(colind, dev)
    d_val = to_dev(np.ascontiguousarray(val).view(np.int16 if np.dtype(vt).itemsize == 2 else vt), dev)
    sentinel = 0x55
    o_val = torch.full((max(nnz, 1) * np.dtype(vt).itemsize,), sentinel, dtype=torch.uint8, device=dev)
    o_ptr = torch.full((n + 1,), -7, dtype=torch.int32, device=dev)
    o_row = torch.full((max(nnz, 1),), -7, dtype=torch.int32, device=dev)
    action = osa.ACL_SPARSE_ACTION_NUMERIC if numeric else osa.ACL_SPARSE_ACTION_SYMBOLIC
    args = (handle.h, m, n, nnz, ptr(d_val), ptr(d_ptr), ptr(d_col), ctypes.c_void_p(o_val.data_ptr()),
            ctypes.c_void_p(o_ptr.data_ptr()), ctypes.c_void_p(o_row.data_ptr()), acl, action, base, 0)
    size = ctypes.c_size_t(0)
    assert L.aclsparseCsr2cscEx2_bufferSize(*args, ctypes.byref(size)) == 0
    buf = torch.empty(max(size.value, 16), dtype=torch.uint8, device=dev) if use_buffer else None
    torch.cuda.synchronize()
    rc = L.aclsparseCsr2cscEx2(*args, ptr(buf))
    if not use_buffer and size.value > 4 * 1024 * 1024:
        assert rc == osa.ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES   # the handle's 4 MiB workspace cannot hold it
        return
    assert rc == 0
    stream.synchronize()
    want_ptr, want_row, want_val = oracle.csr2csc(m, n, rowptr, colind, val if numeric else None, base)
    assert np.array_equal(o_ptr.cpu().numpy(), want_ptr)
    assert np.array_equal(o_row.cpu().numpy()[:nnz], want_row)
    got_val = o_val.cpu().numpy()[: nnz * np.dtype(vt).itemsize]
    if numeric:
        assert np.array_equal(got_val, np.ascontiguousarray(want_val).view(np.uint8))
    else:
        assert np.all(got_val == sentinel)                           # SYMBOLIC leaves cscVal alone
    assert np.array_equal(d_ptr.cpu().numpy(), rowptr) and np.array_equal(d_col.cpu().numpy(), colind)


def _typed(val, name):
    if name == "INT8":
        return np.clip(np.rint(val * 20), -128, 127).astype(np.int8)
    if name == "BF16":
        return (val.view(np.uint32) >> 16).astype(np.uint16)
    return val.astype(NP_TYPE[name])


@pytest.mark.parametrize("c", CSR2CSC, ids=[c["case_name"] for c in CSR2CSC])
def test_csr2csc_reference_table(osa, gpu_ctx, c):
    m, n, base = int(c["m"]), int(c["n"]), int(c["idx_base"])
    rowptr, colind, val = matrix(c)
    run_csr2csc(osa, gpu_ctx, m, n, rowptr + base, colind + base, _typed(val, c["val_type"]), NP_TYPE[c["val_type"]],
                c["copy_values"] == "NUMERIC", base)


@pytest.mark.parametrize("m,n,density", [(1, 1, 1.0), (3, 100_000, 0.001), (100_000, 3, 0.5), (20000, 20000, 0.002),
                                         (1000, 1 << 20, 0.00002), (300, 17, 0.0)])
def test_csr2csc_shapes_unsorted_duplicates(osa, gpu_ctx, m, n, density):
    rowptr, colind, val = random_csr(m, n, density, m + n, unsorted=True, duplicates=True, empty_row_prob=0.1)
    for base in (0, 1):
        run_csr2csc(osa, gpu_ctx, m, n, rowptr + base, colind + base, val, np.float32, True, base)
    run_csr2csc(osa, gpu_ctx, m, n, rowptr, colind, val, np.float32, True, 0, use_buffer=False)


@pytest.mark.parametrize("val_type,numeric", [("FP16", True), ("BF16", True), ("INT8", True), ("FP32", False)])
@pytest.mark.parametrize("m,n,nnz", [(700, 5000, 3840 * 6), (50, 3, 3840 * 2 + 17), (9000, 40_000_000, 61_003),
                                     (1, 70_000, 3839)])
def test_csr2csc_value_sizes_and_key_widths_over_whole_tiles(osa, gpu_ctx, m, n, nnz, val_type, numeric):
    """The sort passes work on tiles of 3 840 entries, whole tiles in a loop and the last, partial one apart; the
    value size is compiled into the first and last pass.  Every value size (and none: SYMBOLIC) on entry counts
    that are a multiple of the tile, a multiple plus a few, and just under one tile, over 2, 13, 17 and 26 column
    bits (two to four passes), unsorted columns with repeats, both index bases."""
    rng = np.random.default_rng(nnz + n)
    cuts = np.sort(rng.integers(0, nnz + 1, m - 1)) if m > 1 else np.zeros(0, np.int64)
    rowptr = np.concatenate([[0], cuts, [nnz]]).astype(np.int32)
    colind = rng.integers(0, n, nnz).astype(np.int32)
    val = rng.uniform(-1, 1, nnz).astype(np.float32)
    for base in (0, 1):
        run_csr2csc(osa, gpu_ctx, m, n, rowptr + base, colind + base, _typed(val, val_type), NP_TYPE[val_type], numeric,
                    base)


def test_csr2csc_twice_is_sorted_csr(osa, gpu_ctx):
    """Size-independent property at a large size: CSR -> CSC -> CSR equals the row-sorted matrix (checked against
    csrsort on the GPU and the oracle on the host)."""
    m, n = 400_000, 300_000
    rng = np.random.default_rng(12)
    lengths = rng.integers(0, 30, m)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, n, int(rowptr[-1])).astype(np.int32)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    run_csr2csc(osa, gpu_ctx, m, n, rowptr, colind, val, np.float32, True, 0)
    colptr, rowind, cval = oracle.csr2csc(m, n, rowptr, colind, val)
    run_csr2csc(osa, gpu_ctx, n, m, colptr, rowind, cval, np.float32, True, 0)
    run_csrsort(osa, gpu_ctx, m, n, rowptr, colind)
