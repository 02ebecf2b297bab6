"""TEST INFRASTRUCTURE ONLY: numpy front end of oracle/liboracle.so.

The C file oracle/oracle.c restates the reference's CPU goldens for CSR
SpMV / SpMM; this module loads it with ctypes and wraps each function for
numpy arrays.  Only tests/, the smoke test and the cpu_baseline leg of
bench.py may import it; the product never does.

`ref_fill()` additionally exposes oracle/_ref/libref_fill.so — the reference's
own generator compiled from its header — when that library has been built.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_fill.so")

_lib = None
_ref = None

c_i64 = ctypes.c_int64
c_f32 = ctypes.c_float
c_i32 = ctypes.c_int32
c_dbl = ctypes.c_double


def build(force=False):
    """Compile oracle.c (and oracle/_ref when the reference tree is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    if force or not os.path.exists(_REF_PATH):
        subprocess.run(["make", "-C", _HERE, "ref"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        path = os.environ.get("OPS_SPARSE_ORACLE_LIBRARY")  # (another build of the checker: build.py --asan)
        if not path:
            if not os.path.exists(_LIB_PATH):
                build()
            path = _LIB_PATH
        _lib = ctypes.CDLL(path)
        _lib.oracle_fill_csr.restype = c_i64
        _lib.oracle_fnv1a.restype = ctypes.c_uint64
        _lib.oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [c_f32]
        _lib.oracle_f16_to_f32.restype = c_f32
        _lib.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    return _lib


def ref_fill():
    """The reference generator library, or None when it was not built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        _ref = ctypes.CDLL(_REF_PATH)
        _ref.ref_fill_csr.restype = c_i64
    return _ref


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ------------------------------------------------------------------- SpMV

def spmv_f64(rows, cols, rowptr, colind, val, x, y, alpha, beta):
    """fp64-accumulated oracle, result rounded once to float32."""
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x = _c(val, np.float32), _c(x, np.float32)
    y = _c(y, np.float32) if y is not None else np.zeros(rows, np.float32)
    z = np.empty(rows, np.float32)
    lib().oracle_spmv_f64(c_i64(rows), c_i64(cols), _p(rowptr), _p(colind), _p(val), _p(x), _p(y), c_f32(alpha),
                          c_f32(beta), _p(z))
    return z


def spmv_f32(rows, rowptr, colind, val, x, y, alpha, beta):
    """The reference's float-accumulating CPU golden (SpmvCpu)."""
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x, y = _c(val, np.float32), _c(x, np.float32), _c(y, np.float32)
    z = np.empty(rows, np.float32)
    lib().oracle_spmv_f32(c_i64(rows), _p(rowptr), _p(colind), _p(val), _p(x), _p(y), c_f32(alpha), c_f32(beta),
                          _p(z))
    return z


def spmv_f32_threads(rows, rowptr, colind, val, x, y, alpha, beta, threads):
    """spmv_f32 with the rows shared out among `threads` OpenMP threads (identical results)."""
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x, y = _c(val, np.float32), _c(x, np.float32), _c(y, np.float32)
    z = np.empty(rows, np.float32)
    lib().oracle_spmv_f32_threads(c_i64(rows), _p(rowptr), _p(colind), _p(val), _p(x), _p(y), c_f32(alpha),
                                  c_f32(beta), _p(z), ctypes.c_int(threads))
    return z


def spmv_trans_f32(rows, cols, rowptr, colind, val, x, y, alpha, beta):
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x, y = _c(val, np.float32), _c(x, np.float32), _c(y, np.float32)
    z = np.empty(cols, np.float32)
    lib().oracle_spmv_trans_f32(c_i64(rows), c_i64(cols), _p(rowptr), _p(colind), _p(val), _p(x), _p(y),
                                c_f32(alpha), c_f32(beta), _p(z))
    return z


def spmv_trans_f64(rows, cols, rowptr, colind, val, x, y, alpha, beta):
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x = _c(val, np.float32), _c(x, np.float32)
    y = _c(y, np.float32) if y is not None else np.zeros(cols, np.float32)
    z = np.empty(cols, np.float32)
    acc = np.empty(max(cols, 1), np.float64)
    lib().oracle_spmv_trans_f64(c_i64(rows), c_i64(cols), _p(rowptr), _p(colind), _p(val), _p(x), _p(y),
                                c_f32(alpha), c_f32(beta), _p(z), _p(acc))
    return z


def spmv_i32(rows, rowptr, colind, val, x, y, alpha, beta):
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, x, y = _c(val, np.int32), _c(x, np.int32), _c(y, np.int32)
    z = np.empty(rows, np.int32)
    lib().oracle_spmv_i32(c_i64(rows), _p(rowptr), _p(colind), _p(val), _p(x), _p(y), c_i32(alpha), c_i32(beta),
                          _p(z))
    return z


# ------------------------------------------------------------------- SpMM

def _spmm(fn, m, n, rowptr, colind, val, B, ldb, b_row_major, trans_b, C, ldc, c_row_major, alpha, beta):
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    out = np.array(C, dtype=np.float32, copy=True, order="C")
    fn(c_i64(m), c_i64(n), _p(rowptr), _p(colind), _p(val), _p(B), c_i64(ldb), c_i32(int(b_row_major)),
       c_i32(int(trans_b)), _p(out), c_i64(ldc), c_i32(int(c_row_major)), c_f32(alpha), c_f32(beta))
    return out


def spmm_f32(m, n, rowptr, colind, val, B, ldb, C, ldc, alpha, beta, b_row_major=True, trans_b=False,
             c_row_major=True):
    """The reference's float-accumulating SpMM golden (SpmmCpuFp32).  B and C
    are flat buffers in their storage layout; a copy of C is returned."""
    return _spmm(lib().oracle_spmm_f32, m, n, rowptr, colind, val, B, ldb, b_row_major, trans_b, C, ldc,
                 c_row_major, alpha, beta)


def spmm_f32_threads(m, n, rowptr, colind, val, B, ldb, C, ldc, alpha, beta, threads, b_row_major=True,
                     trans_b=False, c_row_major=True):
    """spmm_f32 with the rows shared out among `threads` OpenMP threads (identical results)."""
    fn = lib().oracle_spmm_f32_threads
    return _spmm(lambda *a: fn(*a, ctypes.c_int(threads)), m, n, rowptr, colind, val, B, ldb, b_row_major, trans_b,
                 C, ldc, c_row_major, alpha, beta)


def host_threads():
    """Threads the all-cores CPU baseline uses: OMP_NUM_THREADS when set, else the CPUs this process may run on."""
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) > 0:
        return int(env)
    return len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)


def spmm_f64(m, n, rowptr, colind, val, B, ldb, C, ldc, alpha, beta, b_row_major=True, trans_b=False,
             c_row_major=True):
    """fp64-accumulated SpMM oracle, any layout."""
    return _spmm(lib().oracle_spmm_f64, m, n, rowptr, colind, val, B, ldb, b_row_major, trans_b, C, ldc,
                 c_row_major, alpha, beta)


def spmm_f64_rowmajor(m, n, rowptr, colind, val, B, ldb, C, ldc, alpha, beta):
    """Same arithmetic as spmm_f64 for row-major B / C, cache-friendly loop order."""
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, B = _c(val, np.float32), _c(B, np.float32)
    out = np.array(C, dtype=np.float32, copy=True, order="C")
    acc = np.empty(max(n, 1), np.float64)
    lib().oracle_spmm_f64_rowmajor(c_i64(m), c_i64(n), _p(rowptr), _p(colind), _p(val), _p(B), c_i64(ldb), _p(out),
                                   c_i64(ldc), c_f32(alpha), c_f32(beta), _p(acc))
    return out


def spmm_i8(m, n, rowptr, colind, val, B, ldb, C, ldc, alpha, beta, b_row_major=True, trans_b=False,
            c_row_major=True, saturate=True):
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    val, B = _c(val, np.int8), _c(B, np.int8)
    out = np.array(C, dtype=np.int32, copy=True, order="C")
    lib().oracle_spmm_i8(c_i64(m), c_i64(n), _p(rowptr), _p(colind), _p(val), _p(B), c_i64(ldb),
                         c_i32(int(b_row_major)), c_i32(int(trans_b)), _p(out), c_i64(ldc), c_i32(int(c_row_major)),
                         c_i32(alpha), c_i32(beta), c_i32(int(saturate)))
    return out


# ------------------------------------------------------------------- fp16

def f32_to_f16_bits(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_f16_array(_p(a), _p(out), c_i64(a.size))
    return out


def f16_bits_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().oracle_f16_to_f32_array(_p(a), _p(out), c_i64(a.size))
    return out


# --------------------------------------------------------------- verifier

def mere_mare(out, gold, eps=2.0 ** -14):
    """(MERE, MARE, mismatches, counted) with the reference's floored denominator."""
    out, gold = _c(out, np.float32).ravel(), _c(gold, np.float32).ravel()
    res = np.zeros(4, np.float64)
    lib().oracle_mere_mare(_p(out), _p(gold), c_i64(out.size), c_dbl(eps), _p(res))
    return float(res[0]), float(res[1]), int(res[2]), int(res[3])


def max_rel_err(out, gold, tiny=1e-30):
    """Strict per-element relative error max |d| / max(|gold|, tiny)."""
    out = np.asarray(out, np.float64).ravel()
    gold = np.asarray(gold, np.float64).ravel()
    if out.size == 0:
        return 0.0
    return float(np.max(np.abs(out - gold) / np.maximum(np.abs(gold), tiny)))


# ------------------------------------------------------------- generators

def fill_csr(seed, rows, cols, nnz_hint, lo=-2.0, hi=2.0, empty_row_prob=0.0):
    """Restatement of SparseFillGenerator(seed).generateCsr(rows, cols, nnz_hint), nnz_hint > 0."""
    per_row = min(nnz_hint // max(rows, 1), cols) if rows > 0 and cols > 0 and nnz_hint > 0 else 0
    cap = max(rows * per_row, 1)
    rowptr = np.zeros(rows + 1, np.int32)
    colind = np.zeros(cap, np.int32)
    val = np.zeros(cap, np.float32)
    nnz = lib().oracle_fill_csr(ctypes.c_uint32(seed), c_i64(rows), c_i64(cols), c_i64(nnz_hint),
                                c_dbl(empty_row_prob), c_dbl(lo), c_dbl(hi), _p(rowptr), _p(colind), _p(val))
    return rowptr, colind[:nnz].copy(), val[:nnz].copy()


def fill_dense(seed, n, lo=-2.0, hi=2.0):
    """Restatement of makeDenseFloat(n, lo, hi, seed)."""
    out = np.zeros(max(n, 0), np.float32)
    lib().oracle_fill_dense(ctypes.c_uint32(seed), c_i64(n), c_dbl(lo), c_dbl(hi), _p(out))
    return out


def ref_fill_csr(seed, rows, cols, nnz_hint=-1, sparsity=0.9, empty_row_prob=0.0, lo=-2.0, hi=2.0):
    """The reference's own generateCsr through oracle/_ref (None if not built)."""
    r = ref_fill()
    if r is None:
        return None
    cap = max(rows * cols, 1) if nnz_hint <= 0 else max(nnz_hint, 1)
    rowptr = np.zeros(rows + 1, np.int32)
    colind = np.zeros(cap, np.int32)
    val = np.zeros(cap, np.float32)
    nnz = r.ref_fill_csr(ctypes.c_uint32(seed), c_i64(rows), c_i64(cols), c_i64(nnz_hint), c_dbl(sparsity),
                         c_dbl(empty_row_prob), c_dbl(lo), c_dbl(hi), _p(rowptr), _p(colind), _p(val), c_i64(cap))
    assert nnz <= cap
    return rowptr, colind[:nnz].copy(), val[:nnz].copy()


def ref_fill_dense(seed, n, lo=-2.0, hi=2.0):
    r = ref_fill()
    if r is None:
        return None
    out = np.zeros(max(n, 0), np.float32)
    r.ref_fill_dense(ctypes.c_uint32(seed), c_i64(n), c_dbl(lo), c_dbl(hi), _p(out))
    return out


def fnv1a(a):
    a = np.ascontiguousarray(a)
    return int(lib().oracle_fnv1a(_p(a), c_i64(a.nbytes)))


# --------------------------------------------------------- CSR producers

def coo2csr(row_ind, m, base=0):
    row_ind = _c(row_ind, np.int32)
    out = np.empty(m + 1, np.int32)
    lib().oracle_coo2csr(_p(row_ind), c_i64(row_ind.size), c_i64(m), c_i32(base), _p(out))
    return out


def csr2coo(rowptr, nnz, base=0):
    rowptr = _c(rowptr, np.int32)
    out = np.empty(max(nnz, 0), np.int32)
    lib().oracle_csr2coo(_p(rowptr), c_i64(rowptr.size - 1), c_i64(nnz), c_i32(base), _p(out))
    return out


def csrsort(rowptr, colind, perm, base=0):
    rowptr = _c(rowptr, np.int32)
    c, p = _c(colind, np.int32).copy(), _c(perm, np.int32).copy()
    lib().oracle_csrsort(_p(rowptr), c_i64(rowptr.size - 1), c_i32(base), _p(c), _p(p))
    return c, p


def cscsort(colptr, rowind, perm, base=0):
    colptr = _c(colptr, np.int32)
    r, p = _c(rowind, np.int32).copy(), _c(perm, np.int32).copy()
    lib().oracle_cscsort(_p(colptr), c_i64(colptr.size - 1), c_i32(base), _p(r), _p(p))
    return r, p


def coosort(rows, cols, perm, by_row=True):
    """(rows, cols, perm) stably sorted by (row, col), or by (col, row) when by_row is false."""
    r, c, p = _c(rows, np.int32).copy(), _c(cols, np.int32).copy(), _c(perm, np.int32).copy()
    lib().oracle_coosort(c_i64(r.size), c_i32(1 if by_row else 0), _p(r), _p(c), _p(p))
    return r, c, p


def csr2csc(m, n, rowptr, colind, val=None, base=0):
    """(colptr, rowind, cscval); val of any 1 / 2 / 4-byte dtype or None (structure only)."""
    rowptr, colind = _c(rowptr, np.int32), _c(colind, np.int32)
    nnz = colind.size
    colptr, rowind = np.empty(n + 1, np.int32), np.empty(nnz, np.int32)
    if val is None:
        lib().oracle_csr2csc(c_i64(m), c_i64(n), c_i64(nnz), c_i32(base), _p(rowptr), _p(colind), None, c_i32(0),
                             _p(colptr), _p(rowind), None)
        return colptr, rowind, None
    val = np.ascontiguousarray(val)
    out = np.empty_like(val)
    lib().oracle_csr2csc(c_i64(m), c_i64(n), c_i64(nnz), c_i32(base), _p(rowptr), _p(colind), _p(val),
                         c_i32(val.dtype.itemsize), _p(colptr), _p(rowind), _p(out))
    return colptr, rowind, out


_ref_conv = None


def ref_convert():
    """The reference's own goldens of the CSR producers (oracle/_ref), or None when not built."""
    global _ref_conv
    path = os.path.join(_HERE, "_ref", "libref_convert.so")
    if _ref_conv is None and os.path.exists(path):
        _ref_conv = ctypes.CDLL(path)
    return _ref_conv


# ------------------------------------- the SpMM test programs' seeded generators

def spmm22_seek(outputs=0):
    """Put the arch22 test program's thread_local std::mt19937(42) where it is after `outputs` engine outputs."""
    lib().oracle_spmm22_seek(ctypes.c_uint64(int(outputs)))


def spmm22_outputs_used():
    lib().oracle_spmm22_outputs_used.restype = ctypes.c_uint64
    return int(lib().oracle_spmm22_outputs_used())


def spmm22_csr(dist, rows, cols, nnz, store=True):
    """generate_random_csr (dist 'uniform') / generate_powerlaw_csr ('powerlaw') of test/spmm/arch22/spmm_test.cpp,
    continuing the engine where the last call (or spmm22_seek) left it.  store=False only moves the engine on and
    returns the number of entries."""
    L = lib()
    L.oracle_spmm22_csr.restype = c_i64
    power = 1 if dist == "powerlaw" else 0
    if not store:
        return int(L.oracle_spmm22_csr(power, ctypes.c_uint64(rows), ctypes.c_uint64(cols), ctypes.c_uint64(nnz), None,
                                       None, None))
    cap = max(min(nnz, rows * cols) + rows, 1)  # the power-law recipe may hand out a few entries more than nnz
    rowptr = np.zeros(rows + 1, np.int32)
    colind = np.zeros(cap, np.int32)
    val = np.zeros(cap, np.float32)
    total = int(L.oracle_spmm22_csr(power, ctypes.c_uint64(rows), ctypes.c_uint64(cols), ctypes.c_uint64(nnz),
                                    _p(rowptr), _p(colind), _p(val)))
    if total < 0:
        raise MemoryError("oracle_spmm22_csr")
    return rowptr, colind[:total].copy(), val[:total].copy()


def glibc_rand_stream(seed, count):
    out = np.zeros(count, np.int32)
    lib().oracle_glibc_rand_stream(ctypes.c_uint32(seed), c_i64(count), _p(out))
    return out


def spmm35_random_csr(seed, m, k, nnz):
    """GenerateRandomCsr of test/spmm/arch35/spmm_test.cpp after std::srand(seed) (glibc's rand())."""
    L = lib()
    L.oracle_spmm35_random_csr.restype = c_i64
    cap = max(min(nnz, m * k), 1)
    rowptr = np.zeros(max(m, 0) + 1, np.int32)
    colind = np.zeros(cap, np.int32)
    val = np.zeros(cap, np.float32)
    total = int(L.oracle_spmm35_random_csr(ctypes.c_uint32(seed), c_i32(m), c_i32(k), c_i32(nnz), _p(rowptr), _p(colind),
                                           _p(val)))
    return rowptr, colind[:total].copy(), val[:total].copy()
