"""Host-only tests of the C ABI: every symbol the public headers declare is exported,
and every argument check returns the status the reference returns for it, before any
device work.  Device pointers are fake (never dereferenced on these paths)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = ctypes.c_void_p(0x1000)
NULL = ctypes.c_void_p(None)


@pytest.fixture(scope="module")
def L(osa):
    return osa.lib()


def declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(%s\w+)\s*\(" % prefix, text)))


def test_every_declared_symbol_is_exported(osa, L):
    acl = declared("cann_ops_sparse.h", "aclsparse")
    raw = declared("ops_sparse_hip.h", "opsparse_")
    assert len(acl) >= 40 and len(raw) >= 7
    for name in acl + raw:
        assert hasattr(L, name), name + " is declared but not exported"
    # and the binding's own lists name exactly the declared functions
    assert sorted(osa.ACLSPARSE_SYMBOLS) == acl
    assert sorted(osa.OPSPARSE_SYMBOLS) == raw


def test_enum_values_match_header(osa):
    text = open(os.path.join(ROOT, "include", "cann_ops_sparse.h")).read()
    m = re.search(r"typedef OPSPARSE_ABI_ENUM\(aclsparseStatus_t\) \{(.*?)\}", text, re.S)
    names = re.findall(r"ACL_SPARSE_STATUS_(\w+)", m.group(1))
    assert names == osa.STATUS_NAMES
    assert osa.ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR == 10 and osa.ACL_SPARSE_STATUS_NOT_SUPPORTED == 8


def st(osa, name):
    return getattr(osa, "ACL_SPARSE_STATUS_" + name)


# ------------------------------------------------------------------ handle

def test_handle_lifecycle(osa, L):
    assert L.aclsparseCreate(None) == st(osa, "HANDLE_IS_NULLPTR")
    h = ctypes.c_void_p(None)
    assert L.aclsparseCreate(ctypes.byref(h)) == 0 and h.value
    assert L.aclsparseCreate(ctypes.byref(h)) == st(osa, "INVALID_VALUE")      # would overwrite a live handle
    v = ctypes.c_int(0)
    assert L.aclsparseGetVersion(None, ctypes.byref(v)) == 0 and v.value == 10000
    assert L.aclsparseGetVersion(h, None) == st(osa, "INVALID_VALUE")
    s = ctypes.c_void_p(123)
    assert L.aclsparseGetStream(h, ctypes.byref(s)) == 0 and s.value is None
    assert L.aclsparseSetStream(h, ctypes.c_void_p(0x55)) == 0
    assert L.aclsparseGetStream(h, ctypes.byref(s)) == 0 and s.value == 0x55
    assert L.aclsparseGetStream(h, None) == st(osa, "INVALID_VALUE")
    assert L.aclsparseSetStream(None, s) == st(osa, "HANDLE_IS_NULLPTR")
    mode = ctypes.c_int(-1)
    assert L.aclsparseGetPointerMode(h, ctypes.byref(mode)) == 0 and mode.value == osa.ACL_SPARSE_POINTER_MODE_HOST
    assert L.aclsparseSetPointerMode(h, 1) == 0
    assert L.aclsparseGetPointerMode(h, ctypes.byref(mode)) == 0 and mode.value == 1
    assert L.aclsparseSetPointerMode(h, 7) == st(osa, "INVALID_VALUE")
    assert L.aclsparseSetPointerMode(None, 0) == st(osa, "HANDLE_IS_NULLPTR")
    # workspace: grow-only user workspace, NULL switches back
    assert L.aclsparseSetWorkspace(h, FAKE, 0) == st(osa, "INVALID_VALUE")
    assert L.aclsparseSetWorkspace(h, FAKE, 1024) == 0
    ws, n = ctypes.c_void_p(None), ctypes.c_size_t(0)
    assert L.aclsparseGetWorkspace(h, ctypes.byref(ws), ctypes.byref(n)) == 0 and (ws.value, n.value) == (0x1000, 1024)
    assert L.aclsparseSetWorkspace(h, ctypes.c_void_p(0x2000), 512) == 0        # not larger: ignored
    assert L.aclsparseGetWorkspace(h, ctypes.byref(ws), ctypes.byref(n)) == 0 and (ws.value, n.value) == (0x1000, 1024)
    assert L.aclsparseSetWorkspace(h, ctypes.c_void_p(0x2000), 4096) == 0
    assert L.aclsparseGetWorkspace(h, ctypes.byref(ws), ctypes.byref(n)) == 0 and (ws.value, n.value) == (0x2000, 4096)
    assert L.aclsparseGetWorkspace(h, None, ctypes.byref(n)) == st(osa, "INVALID_VALUE")
    assert L.aclsparseGetWorkspace(None, ctypes.byref(ws), ctypes.byref(n)) == st(osa, "HANDLE_IS_NULLPTR")
    # stream back to null before destroy: no device work was ever queued
    assert L.aclsparseSetStream(h, NULL) == 0
    assert L.aclsparseDestroy(h) == 0
    assert L.aclsparseDestroy(None) == st(osa, "HANDLE_IS_NULLPTR")


# -------------------------------------------------------------- descriptors

def make_csr(osa, L, rows=4, cols=4, nnz=5, ptr=0, idx=0, base=0, vt=None, rp=FAKE, ci=FAKE, va=FAKE):
    d = ctypes.c_void_p(None)
    rc = L.aclsparseCreateCsr(ctypes.byref(d), rows, cols, nnz, rp, ci, va, ptr, idx, base,
                              osa.ACL_FLOAT if vt is None else vt)
    return rc, d


def make_vec(osa, L, n=4, vt=None, p=FAKE):
    d = ctypes.c_void_p(None)
    return L.aclsparseCreateDnVec(ctypes.byref(d), n, p, osa.ACL_FLOAT if vt is None else vt), d


def make_mat(osa, L, rows=4, cols=2, ld=2, vt=None, order=0, p=FAKE):
    d = ctypes.c_void_p(None)
    return L.aclsparseCreateDnMat(ctypes.byref(d), rows, cols, ld, p, osa.ACL_FLOAT if vt is None else vt, order), d


def test_descriptor_creators(osa, L):
    INV, NS = st(osa, "INVALID_VALUE"), st(osa, "NOT_SUPPORTED")
    assert L.aclsparseCreateCsr(None, 1, 1, 1, FAKE, FAKE, FAKE, 0, 0, 0, 0) == INV
    assert make_csr(osa, L, rows=-1)[0] == INV and make_csr(osa, L, nnz=-1)[0] == INV
    assert make_csr(osa, L, ptr=5)[0] == NS and make_csr(osa, L, idx=9)[0] == NS
    for ptr, idx in [(0, 0), (1, 0), (0, 1), (1, 1)]:          # every I32 / I64 mix can be described
        rc, d = make_csr(osa, L, ptr=ptr, idx=idx)
        assert rc == 0
        assert L.aclsparseDestroySpMat(d) == 0
    assert L.aclsparseDestroySpMat(None) == 0
    rc, d = make_csr(osa, L, rows=3, cols=7, nnz=5)
    r, c, z = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    assert L.aclsparseSpMatGetSize(d, ctypes.byref(r), ctypes.byref(c), ctypes.byref(z)) == 0
    assert (r.value, c.value, z.value) == (3, 7, 5)
    f = ctypes.c_int(-1)
    assert L.aclsparseSpMatGetFormat(d, ctypes.byref(f)) == 0 and f.value == osa.ACL_SPARSE_FORMAT_CSR
    v = ctypes.c_void_p(None)
    assert L.aclsparseSpMatSetValues(d, ctypes.c_void_p(0x77)) == 0
    assert L.aclsparseSpMatGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x77
    assert L.aclsparseConstSpMatGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x77
    assert L.aclsparseCsrSetPointers(d, FAKE, NULL, FAKE) == INV            # nnz > 0 needs indices
    assert L.aclsparseCsrSetPointers(d, FAKE, FAKE, ctypes.c_void_p(0x88)) == 0
    assert L.aclsparseSpMatGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x88
    assert L.aclsparseSpMatGetSize(None, None, None, None) == INV
    L.aclsparseDestroySpMat(d)

    assert make_vec(osa, L, n=-1)[0] == INV and make_vec(osa, L, n=3, p=NULL)[0] == INV
    assert make_vec(osa, L, vt=12345)[0] == INV
    rc, d = make_vec(osa, L, n=0, p=NULL)
    assert rc == 0
    n, t = ctypes.c_int64(-1), ctypes.c_int(-1)
    assert L.aclsparseDnVecGet(d, ctypes.byref(n), ctypes.byref(v), ctypes.byref(t)) == 0 and n.value == 0
    assert L.aclsparseDnVecSetValues(d, ctypes.c_void_p(0x99)) == 0
    assert L.aclsparseDnVecGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x99
    assert L.aclsparseConstDnVecGetValues(d, ctypes.byref(v)) == 0
    assert L.aclsparseDnVecGetValues(d, None) == INV
    assert L.aclsparseDestroyDnVec(d) == 0
    assert L.aclsparseDestroyDnVec(None) == INV
    assert L.aclsparseDnVecGet(None, None, None, None) == INV

    for kw in (dict(rows=0), dict(cols=0), dict(ld=0), dict(p=NULL), dict(vt=999), dict(order=5),
               dict(cols=8, ld=7), dict(rows=9, ld=8, order=1)):
        assert make_mat(osa, L, **kw)[0] == INV, kw
    rc, d = make_mat(osa, L, rows=6, cols=3, ld=5)
    a, b, c2, o = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int(-1)
    assert L.aclsparseDnMatGet(d, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c2), ctypes.byref(v), ctypes.byref(t),
                               ctypes.byref(o)) == 0
    assert (a.value, b.value, c2.value, o.value, v.value) == (6, 3, 5, 0, 0x1000)
    assert L.aclsparseDnMatSetValues(d, ctypes.c_void_p(0x66)) == 0
    assert L.aclsparseDnMatGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x66
    assert L.aclsparseDestroyDnMat(d) == 0
    assert L.aclsparseDestroyDnMat(None) == INV


# --------------------------------------------------------------------- SpMV

@pytest.fixture()
def handle(osa, L):
    h = ctypes.c_void_p(None)
    assert L.aclsparseCreate(ctypes.byref(h)) == 0
    assert L.aclsparseSetStream(h, ctypes.c_void_p(0x55)) == 0     # fake stream: never used on failing paths
    yield h
    L.aclsparseSetStream(h, NULL)
    L.aclsparseDestroy(h)


def spmv(osa, L, h, A, x, y, op=0, ct=None, alg=0, buf=NULL):
    return L.aclsparseSpMV(h, op, None, A, x, None, y, osa.ACL_FLOAT if ct is None else ct, alg, buf)


def test_spmv_status_table(osa, L, handle):
    """reference sparse/spmv/arch22/spmv_host.cpp:132-274, in its order."""
    INV, NS = st(osa, "INVALID_VALUE"), st(osa, "NOT_SUPPORTED")
    _, A = make_csr(osa, L)
    _, x = make_vec(osa, L, 4)
    _, y = make_vec(osa, L, 4)
    assert spmv(osa, L, None, A, x, y) == st(osa, "HANDLE_IS_NULLPTR")
    assert spmv(osa, L, handle, None, x, y) == INV
    assert spmv(osa, L, handle, A, None, y) == INV
    assert spmv(osa, L, handle, A, x, None) == INV
    assert spmv(osa, L, handle, A, x, y, alg=osa.ACL_SPARSE_SPMV_CSR_ALG1) == NS
    assert spmv(osa, L, handle, A, x, y, ct=osa.ACL_FLOAT16) == NS
    assert spmv(osa, L, handle, A, x, y, op=osa.ACL_SPARSE_OP_CONJUGATE_TRANSPOSE) == NS
    for kw in (dict(base=1), dict(ptr=1, idx=1), dict(ptr=1), dict(idx=1)):
        _, bad = make_csr(osa, L, **kw)
        assert spmv(osa, L, handle, bad, x, y) == NS, kw
        L.aclsparseDestroySpMat(bad)
    # no stream set
    L.aclsparseSetStream(handle, NULL)
    assert spmv(osa, L, handle, A, x, y) == INV
    L.aclsparseSetStream(handle, ctypes.c_void_p(0x55))
    # null device arrays
    _, bad = make_csr(osa, L, va=NULL)
    assert spmv(osa, L, handle, bad, x, y) == INV
    L.aclsparseDestroySpMat(bad)
    # vectors too short (x needs cols, y needs rows; swapped for the transpose)
    _, xs = make_vec(osa, L, 3)
    assert spmv(osa, L, handle, A, xs, y) == INV and spmv(osa, L, handle, A, x, xs) == INV
    _, R = make_csr(osa, L, rows=3, cols=4, nnz=2)
    assert spmv(osa, L, handle, R, x, xs, op=1) == INV           # transpose: y needs cols = 4
    _, x2 = make_vec(osa, L, 2)
    assert spmv(osa, L, handle, R, x2, y, op=1) == INV           # transpose: x needs rows = 3
    L.aclsparseDestroyDnVec(x2)
    # x type must equal A type; INT32 compute needs all-int32
    _, xh = make_vec(osa, L, 4, vt=osa.ACL_FLOAT16)
    assert spmv(osa, L, handle, A, xh, y) == NS
    assert spmv(osa, L, handle, A, x, y, ct=osa.ACL_INT32) == NS
    # GetBufferSize / Preprocess share the checks
    n = ctypes.c_size_t(0)
    assert L.aclsparseSpMVGetBufferSize(handle, 0, None, A, x, None, y, osa.ACL_FLOAT, 0, None) == INV
    assert L.aclsparseSpMVGetBufferSize(None, 0, None, A, x, None, y, osa.ACL_FLOAT, 0, ctypes.byref(n)) == \
        st(osa, "HANDLE_IS_NULLPTR")
    assert L.aclsparseSpMVGetBufferSize(handle, 0, None, A, x, None, y, osa.ACL_FLOAT, 0, ctypes.byref(n)) == 0
    assert n.value >= 256 and n.value == L.opsparse_spmv_csr_workspace_bytes(4, 5)
    assert L.aclsparseSpMVPreprocess(handle, 0, None, A, x, None, y, osa.ACL_FLOAT, 0, None) == \
        st(osa, "INSUFFICIENT_RESOURCES")
    for d in (x, y, xs, xh):
        L.aclsparseDestroyDnVec(d)
    L.aclsparseDestroySpMat(A)
    L.aclsparseDestroySpMat(R)


# --------------------------------------------------------------------- SpMM

def spmm_args(osa, h, A, B, C, opa=0, opb=0, ct=None, alg=0):
    return (h, opa, opb, None, A, B, None, C, osa.ACL_FLOAT if ct is None else ct, alg)


def test_spmm_status_table(osa, L, handle):
    """reference sparse/spmm/arch35/spmm_host.cpp:152-191, :213-234, :335-362, :364-394."""
    INV, NS, HN = st(osa, "INVALID_VALUE"), st(osa, "NOT_SUPPORTED"), st(osa, "HANDLE_IS_NULLPTR")
    _, A = make_csr(osa, L, rows=4, cols=3, nnz=5)
    _, B = make_mat(osa, L, rows=3, cols=2, ld=2)
    _, C = make_mat(osa, L, rows=4, cols=2, ld=2)
    n = ctypes.c_size_t(0)
    run = lambda *a, **k: L.aclsparseSpMM(*spmm_args(osa, *a, **k), FAKE)
    assert L.aclsparseSpMMGetBufferSize(*spmm_args(osa, handle, A, B, C), None) == INV
    assert run(handle, None, B, C) == HN and run(handle, A, None, C) == HN and run(handle, A, B, None) == HN
    assert run(handle, A, B, C, opa=1) == NS and run(handle, A, B, C, opb=2) == NS
    assert run(handle, A, B, C, alg=7) == NS
    assert run(handle, A, B, C, ct=osa.ACL_INT32) == NS                     # no (f32, f32, f32, i32) kernel
    for kw in (dict(base=1), dict(ptr=1, idx=1), dict(idx=1)):
        _, bad = make_csr(osa, L, rows=4, cols=3, nnz=5, **kw)
        assert run(handle, bad, B, C) == NS, kw
        L.aclsparseDestroySpMat(bad)
    _, Bh = make_mat(osa, L, rows=3, cols=2, ld=2, vt=osa.ACL_FLOAT16)
    assert run(handle, A, Bh, C) == NS                                       # mixed types
    _, B4 = make_mat(osa, L, rows=4, cols=2, ld=2)
    _, C3 = make_mat(osa, L, rows=4, cols=3, ld=3)
    _, C5 = make_mat(osa, L, rows=5, cols=2, ld=2)
    assert run(handle, A, B4, C) == INV and run(handle, A, B, C3) == INV and run(handle, A, B, C5) == INV
    # buffer and handle are checked after the descriptors, in this order
    assert L.aclsparseSpMM(*spmm_args(osa, handle, A, B, C), None) == st(osa, "INSUFFICIENT_RESOURCES")
    assert L.aclsparseSpMM(*spmm_args(osa, None, A, B, C), None) == st(osa, "INSUFFICIENT_RESOURCES")
    assert L.aclsparseSpMM(*spmm_args(osa, None, A, B, C), FAKE) == HN
    assert L.aclsparseSpMMPreprocess(*spmm_args(osa, handle, A, B, C), None) == st(osa, "INSUFFICIENT_RESOURCES")
    # a matrix this small cannot have a long row: 256-byte header, no device access; n = 2 is not a whole 16-byte
    # vector of fp32, so the buffer also holds padded copies of B (3 x 4) and C (4 x 4), 256 bytes each
    assert L.aclsparseSpMMGetBufferSize(*spmm_args(osa, None, A, B, C), ctypes.byref(n)) == 0 and n.value == 768
    _, B4w = make_mat(osa, L, rows=3, cols=4, ld=4)
    _, C4w = make_mat(osa, L, rows=4, cols=4, ld=4)
    assert L.aclsparseSpMMGetBufferSize(*spmm_args(osa, None, A, B4w, C4w), ctypes.byref(n)) == 0 and n.value == 256
    L.aclsparseDestroyDnMat(B4w)
    L.aclsparseDestroyDnMat(C4w)
    # Preprocess of an empty matrix is refused (reference spmm_csr_mat.cpp:148-150)
    _, E = make_csr(osa, L, rows=0, cols=3, nnz=0)
    _, C0 = make_mat(osa, L, rows=1, cols=2, ld=2)
    assert L.aclsparseSpMMPreprocess(*spmm_args(osa, handle, E, B, C0), FAKE) == INV  # rows mismatch first
    for d in (B, C, Bh, B4, C3, C5, C0):
        L.aclsparseDestroyDnMat(d)
    L.aclsparseDestroySpMat(A)
    L.aclsparseDestroySpMat(E)


def test_raw_layer_argument_checks(osa, L):
    plan = osa.OpsparseSpmvPlan()
    assert L.opsparse_spmv_csr_analyse(FAKE, -1, 1, 1, FAKE, 1 << 20, 0, ctypes.byref(plan), None) == -1
    assert L.opsparse_spmv_csr_analyse(FAKE, 10, 10, 20, None, 0, 0, ctypes.byref(plan), None) == -3
    assert L.opsparse_spmv_csr_analyse(FAKE, 10, 10, 0, None, 0, 0, ctypes.byref(plan), None) == 0
    assert plan.kernel == osa.OPSPARSE_SPMV_SCALE_ONLY
    s = osa.OpsparseScalar(1.0, None, 0, 0)
    assert L.opsparse_spmv_csr_launch(None, 0, FAKE, FAKE, FAKE, FAKE, FAKE, 0, 5, 0, s, s, 0, 0, 0, None, 0, None) == 0
    assert L.opsparse_spmv_csr_launch(None, 0, FAKE, FAKE, FAKE, FAKE, None, 3, 5, 2, s, s, 0, 0, 0, None, 0, None) == -1
    assert L.opsparse_spmv_csr_workspace_bytes(-1, 0) == 0
    n = ctypes.c_size_t(0)
    assert L.opsparse_spmm_csr_workspace_bytes(FAKE, 10, 20, 4, None, None) == -1
    assert L.opsparse_spmm_csr_workspace_bytes(FAKE, 10, 20, 4, None, ctypes.byref(n)) == 0 and n.value == 256
    mp = osa.OpsparseSpmmPlan()
    assert L.opsparse_spmm_csr_analyse(FAKE, 10, 20, 4, None, 0, 0, ctypes.byref(mp), None) == -3
    assert L.opsparse_spmm_csr_launch(None, FAKE, FAKE, FAKE, FAKE, FAKE, 0, 3, 4, 0, 4, 4, 0, 0, 0, s, s, 0, 0, None,
                                      0, None) == 0
    assert L.opsparse_spmm_csr_launch(None, FAKE, FAKE, FAKE, FAKE, FAKE, 2, 3, 4, 5, 0, 4, 0, 0, 0, s, s, 0, 0, None,
                                      0, None) == -1
    assert L.opsparse_copy_launch(FAKE, FAKE, 17, None) == -1 and L.opsparse_copy_launch(FAKE, FAKE, 0, None) == 0


def test_restored_layout_applicability(osa, L, handle):
    """When ACL_SPARSE_SPMV_CSR_ALG2 gets a re-stored layout, decided on the host from the sizes alone: blocked
    gather needs an x of more than 2^18 and at most 2^25 elements and 32 entries per (panel, row block) chunk;
    (and two million entries in all); column panels (op(A) = A only) need 2 .. 16 panels of 2^20 columns.  GetBufferSize reports the larger of
    that layout and the ordinary buffer, and the ordinary one for anything else."""
    blocked, panels = L.opsparse_spmv_csr_blocked_workspace_bytes, L.opsparse_spmv_csr_panels_workspace_bytes
    m = 1 << 23
    assert blocked(m, m, 8 * m, 0) > 12 * 8 * m and blocked(m, m, 8 * m, 1) > 12 * 8 * m
    assert blocked(m, 1 << 18, 8 * m, 0) == 0 and blocked(m, (1 << 18) + 1, 8 * m, 0) > 0     # x must be wide enough
    assert blocked(m, (1 << 25) + 1, 64 * m, 0) == 0                                         # too many panels
    assert blocked(m, m, m // 64, 0) == 0                                                    # chunks too short
    assert blocked(50_000, m, 1_900_000, 0) == 0 and blocked(50_000, m, 2_100_000, 0) > 0     # too few entries
    assert blocked(1 << 18, m, 8 * m, 1) == 0 and blocked(m, 1000, 8 * m, 1) > 0             # op(A) = A^T: x has m rows
    assert blocked(0, m, 0, 0) == 0 and blocked(m, m, (1 << 31), 0) == 0
    assert panels(m, m, 8 * m) > 0 and panels(m, 1 << 20, 8 * m) == 0 and panels(m, (1 << 24) + 1, 8 * m) == 0
    n = ctypes.c_size_t(0)
    A, X, Y = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert L.aclsparseCreateCsr(ctypes.byref(A), m, m, 8 * m, FAKE, FAKE, FAKE, 0, 0, 0, osa.ACL_FLOAT) == 0
    assert L.aclsparseCreateDnVec(ctypes.byref(X), m, FAKE, osa.ACL_FLOAT) == 0
    assert L.aclsparseCreateDnVec(ctypes.byref(Y), m, FAKE, osa.ACL_FLOAT) == 0
    plain = L.opsparse_spmv_csr_workspace_bytes(m, 8 * m)
    cases = [(0, osa.ACL_SPARSE_SPMV_CSR_ALG2, blocked(m, m, 8 * m, 0)),
             (1, osa.ACL_SPARSE_SPMV_CSR_ALG2, blocked(m, m, 8 * m, 1))]
    import torch
    if not torch.cuda.is_available():
        # with a device the default algorithm samples the column indices to decide, and these arrays are not real;
        # without one the sample fails and the answer is the ordinary buffer
        cases.append((0, osa.ACL_SPARSE_SPMV_ALG_DEFAULT, plain))
    for op, alg, want in cases:
        assert L.aclsparseSpMVGetBufferSize(handle, op, None, A, X, None, Y, osa.ACL_FLOAT, alg, ctypes.byref(n)) == 0
        assert n.value == max(want, plain)
    os.environ["OPS_SPARSE_SPMV_NO_BLOCKED"] = "1"
    try:
        assert L.aclsparseSpMVGetBufferSize(handle, 0, None, A, X, None, Y, osa.ACL_FLOAT,
                                            osa.ACL_SPARSE_SPMV_CSR_ALG2, ctypes.byref(n)) == 0
        assert n.value == max(panels(m, m, 8 * m), plain)
    finally:
        del os.environ["OPS_SPARSE_SPMV_NO_BLOCKED"]
    for d in (X, Y):
        assert L.aclsparseDestroyDnVec(d) == 0
    assert L.aclsparseDestroySpMat(A) == 0


# ------------------------------------------------------------------- SpMVOp

def test_spmvop_status_table(osa, L, handle):
    """reference sparse/spmv_op/arch35/spmv_op_host.cpp:64-297 (checks), :496-541, :603-746 (entry points)."""
    INV, NS, HN = st(osa, "INVALID_VALUE"), st(osa, "NOT_SUPPORTED"), st(osa, "HANDLE_IS_NULLPTR")
    ALG1, ALG2 = osa.ACL_SPARSE_SPMVOP_ALG1, osa.ACL_SPARSE_SPMVOP_ALG2
    F = osa.ACL_FLOAT
    _, A = make_csr(osa, L)
    _, x = make_vec(osa, L, 4)
    _, y = make_vec(osa, L, 4)
    _, z = make_vec(osa, L, 4)
    n = ctypes.c_size_t(77)

    # bufferSize: handle, (opA, computeType), matrix, alg, output pointer, in this order
    size = lambda h, A_, op=0, ct=F, alg=0, out=ctypes.byref(n): L.aclsparseSpMVOp_bufferSize(h, op, A_, x, y, z, ct, alg, out)
    assert size(None, A) == HN
    assert size(handle, A, op=1) == NS and size(handle, A, ct=osa.ACL_FLOAT16) == NS
    assert size(handle, None) == INV
    assert size(handle, A, alg=3) == NS
    assert size(handle, A, out=None) == INV
    assert size(handle, None, op=1) == NS                       # opA is looked at before the matrix
    assert size(handle, A) == 0 and n.value == 0
    assert size(handle, A, alg=ALG1) == 0 and n.value == 0
    assert size(handle, A, alg=ALG2) == 0 and n.value == L.opsparse_spmv_csr_workspace_bytes(4, 5)
    _, big = make_csr(osa, L, rows=(1 << 31), cols=4, nnz=5)
    assert size(handle, big) == NS
    bad_mats = [dict(vt=osa.ACL_FLOAT16), dict(idx=1), dict(ptr=1, idx=1)]
    for kw in bad_mats:
        _, bad = make_csr(osa, L, **kw)
        assert size(handle, bad) == NS, kw
        L.aclsparseDestroySpMat(bad)
    for kw in (dict(ptr=1), dict(base=1), dict(ptr=1, base=1)):       # 64-bit row offsets and base 1 are supported
        _, ok = make_csr(osa, L, **kw)
        assert size(handle, ok) == 0, kw
        L.aclsparseDestroySpMat(ok)

    # createDescr: handle, output pointer, matrix, alg, ALG2 buffer, (opA, computeType), rows
    d = ctypes.c_void_p(None)
    mk = lambda h, A_, op=0, ct=F, alg=0, buf=None, out=ctypes.byref(d): \
        L.aclsparseSpMVOp_createDescr(h, out, op, A_, x, y, z, ct, alg, buf)
    assert mk(None, A) == HN
    assert mk(handle, A, out=None) == INV
    assert mk(handle, None) == INV
    assert mk(handle, A, alg=9) == NS
    assert mk(handle, A, alg=ALG2, buf=None) == INV
    assert mk(handle, A, alg=ALG2, buf=None, op=1) == INV        # the buffer check comes before opA
    assert mk(handle, A, op=1) == NS and mk(handle, A, ct=osa.ACL_INT32) == NS
    assert mk(handle, big) == NS
    for kw in bad_mats:
        _, bad = make_csr(osa, L, **kw)
        assert mk(handle, bad) == NS, kw
        L.aclsparseDestroySpMat(bad)
    assert d.value is None                                          # nothing was created on the failing paths
    assert mk(handle, A) == 0 and d.value

    # createPlan
    p = ctypes.c_void_p(None)
    assert L.aclsparseSpMVOp_createPlan(None, d, ctypes.byref(p), None, 0) == HN
    assert L.aclsparseSpMVOp_createPlan(handle, None, ctypes.byref(p), None, 0) == INV
    assert L.aclsparseSpMVOp_createPlan(handle, d, None, None, 0) == INV
    assert L.aclsparseSpMVOp_createPlan(handle, d, ctypes.byref(p), FAKE, 0) == NS
    assert L.aclsparseSpMVOp_createPlan(handle, d, ctypes.byref(p), None, 8) == NS
    assert p.value is None
    assert L.aclsparseSpMVOp_createPlan(handle, d, ctypes.byref(p), None, 0) == 0 and p.value

    # setGlobalUserData: accepted and ignored when consistent
    sg = L.aclsparseSpMVOp_setGlobalUserData
    assert sg(None, p, b"e", None, 0) == HN and sg(handle, None, b"e", None, 0) == INV
    assert sg(handle, p, b"e", FAKE, 0) == INV and sg(handle, p, b"e", None, 4) == INV
    assert sg(handle, p, b"e", None, 0) == 0 and sg(handle, p, None, FAKE, 4) == 0

    # execute: handle, plan, alpha, beta, vectors, types, sizes
    one, zero = ctypes.c_float(1.0), ctypes.c_float(0.0)
    pa, pb = ctypes.cast(ctypes.pointer(one), ctypes.c_void_p), ctypes.cast(ctypes.pointer(zero), ctypes.c_void_p)
    run = lambda h=handle, pl=p, a=pa, b=pb, X=x, Y=y, Z=z: L.aclsparseSpMVOp(h, pl, a, b, X, Y, Z)
    assert run(h=None) == HN
    assert run(pl=None) == INV and run(a=None) == INV and run(b=None) == INV
    assert run(X=None) == INV and run(Y=None) == INV and run(Z=None) == INV
    _, xh = make_vec(osa, L, 4, vt=osa.ACL_FLOAT16)
    assert run(X=xh) == NS and run(Y=xh) == NS and run(Z=xh) == NS
    _, v3 = make_vec(osa, L, 3)
    _, v5 = make_vec(osa, L, 5)
    for bad in (v3, v5):                                            # sizes must match exactly, longer is wrong too
        assert run(X=bad) == INV and run(Y=bad) == INV and run(Z=bad) == INV
    assert run(X=xh, Y=v3) == NS                                    # types are checked before sizes

    # a matrix without rows executes to SUCCESS without touching the device
    _, E = make_csr(osa, L, rows=0, cols=4, nnz=0, rp=NULL, ci=NULL, va=NULL)
    de, pe = ctypes.c_void_p(None), ctypes.c_void_p(None)
    _, v0 = make_vec(osa, L, 0, p=NULL)
    assert L.aclsparseSpMVOp_createDescr(handle, ctypes.byref(de), 0, E, x, v0, v0, F, ALG2, FAKE) == 0
    assert L.aclsparseSpMVOp_createPlan(handle, de, ctypes.byref(pe), None, 0) == 0
    assert run(pl=pe, Y=v0, Z=v0) == 0
    assert run(pl=pe, Y=y, Z=v0) == INV

    # destroy: plan before descriptor; NULL is accepted
    assert L.aclsparseSpMVOp_destroyPlan(pe) == 0 and L.aclsparseSpMVOp_destroyDescr(de) == 0
    assert L.aclsparseSpMVOp_destroyPlan(p) == 0 and L.aclsparseSpMVOp_destroyDescr(d) == 0
    assert L.aclsparseSpMVOp_destroyPlan(None) == 0 and L.aclsparseSpMVOp_destroyDescr(None) == 0
    for v in (x, y, z, xh, v3, v5, v0):
        L.aclsparseDestroyDnVec(v)
    for m in (A, big, E):
        L.aclsparseDestroySpMat(m)


# ------------------------------------------------------------ CSR producers

def test_matdescr(osa, L):
    """reference sparse/common/aclsparse_matdescr.cpp:25-110."""
    assert L.aclsparseCreateMatDescr(None) == st(osa, "INVALID_VALUE")
    d = ctypes.c_void_p(None)
    assert L.aclsparseCreateMatDescr(ctypes.byref(d)) == 0 and d.value
    assert (L.aclsparseGetMatType(d), L.aclsparseGetMatIndexBase(d), L.aclsparseGetMatDiagType(d),
            L.aclsparseGetMatFillMode(d)) == (0, 0, 0, 0)
    L.aclsparseSetMatType(d, 3)
    L.aclsparseSetMatIndexBase(d, 1)
    L.aclsparseSetMatDiagType(d, 1)
    L.aclsparseSetMatFillMode(d, 1)
    assert (L.aclsparseGetMatType(d), L.aclsparseGetMatIndexBase(d), L.aclsparseGetMatDiagType(d),
            L.aclsparseGetMatFillMode(d)) == (3, 1, 1, 1)
    L.aclsparseSetMatIndexBase(None, 1)                       # ignored
    assert L.aclsparseGetMatIndexBase(None) == 0
    assert L.aclsparseDestroyMatDescr(d) == 0 and L.aclsparseDestroyMatDescr(None) == 0


def test_conversion_status_table(osa, L, handle):
    """reference coo2csr_host.cpp:38-80, csr2coo_host.cpp:66-115, csrsort_host.cpp:53-74 / :146-221,
    csr2csc_ex2_host.cpp:109-232 / :535-618."""
    INV, NS, HN = st(osa, "INVALID_VALUE"), st(osa, "NOT_SUPPORTED"), st(osa, "HANDLE_IS_NULLPTR")
    IMAX = 2 ** 31 - 1
    # coo2csr
    c = L.aclsparseXcoo2csr
    assert c(None, FAKE, 4, 4, FAKE, 0) == HN
    assert c(handle, FAKE, -1, 4, FAKE, 0) == INV and c(handle, FAKE, IMAX, 4, FAKE, 1) == INV
    assert c(handle, FAKE, 4, -1, FAKE, 0) == INV and c(handle, FAKE, 4, 0, FAKE, 0) == INV
    assert c(handle, FAKE, 4, 4, FAKE, 2) == INV
    assert c(handle, None, 4, 4, FAKE, 0) == INV and c(handle, FAKE, 4, 4, None, 0) == INV
    # csr2coo: its null-handle code is NOT_INITIALIZED
    r = L.aclsparseXcsr2coo
    assert r(None, FAKE, 4, 4, FAKE, 0) == st(osa, "NOT_INITIALIZED")
    assert r(handle, FAKE, -1, 4, FAKE, 0) == INV and r(handle, FAKE, 4, -1, FAKE, 0) == INV
    assert r(handle, FAKE, 4, 0, FAKE, 0) == INV and r(handle, FAKE, 4, 4, FAKE, 7) == INV
    assert r(handle, None, 4, 4, FAKE, 0) == INV and r(handle, FAKE, 4, 4, None, 0) == INV
    assert r(handle, FAKE, 2 ** 31, 4, FAKE, 0) == INV and r(handle, FAKE, 4, 2 ** 31, FAKE, 0) == INV
    assert r(handle, FAKE, 0, 4, None, 0) == 0 and r(handle, None, 0, 0, None, 1) == 0
    # csrsort
    n = ctypes.c_size_t(99)
    bs = L.aclsparseXcsrsort_bufferSizeExt
    assert bs(None, 4, 4, 5, FAKE, FAKE, ctypes.byref(n)) == HN
    assert bs(handle, 4, 4, 5, FAKE, FAKE, None) == INV
    for bad in ((-1, 4, 5), (4, -1, 5), (4, 4, -1), (0, 4, 5), (4, 0, 5)):
        assert bs(handle, *bad, FAKE, FAKE, ctypes.byref(n)) == INV, bad
    assert bs(handle, 4, 4, 5, None, FAKE, ctypes.byref(n)) == INV
    assert bs(handle, 4, 4, 5, FAKE, None, ctypes.byref(n)) == INV
    assert bs(handle, 4, 4, 0, FAKE, None, ctypes.byref(n)) == 0 and n.value == 0
    assert bs(handle, 4, 4, 5, FAKE, FAKE, ctypes.byref(n)) == 0 and n.value == L.opsparse_csrsort_workspace_bytes(4, 5)
    assert n.value >= 2 * 5 * 4                                   # at least the reference's 2 * nnz ints
    d = ctypes.c_void_p(None)
    L.aclsparseCreateMatDescr(ctypes.byref(d))
    so = L.aclsparseXcsrsort
    assert so(None, 4, 4, 5, d, FAKE, FAKE, FAKE, FAKE) == HN
    assert so(handle, 4, 4, -5, d, FAKE, FAKE, FAKE, FAKE) == INV and so(handle, 0, 4, 5, d, FAKE, FAKE, FAKE, FAKE) == INV
    assert so(handle, 4, 4, 5, d, None, FAKE, FAKE, FAKE) == INV and so(handle, 4, 4, 5, d, FAKE, None, FAKE, FAKE) == INV
    assert so(handle, 4, 4, 5, None, FAKE, FAKE, FAKE, FAKE) == INV
    L.aclsparseSetMatIndexBase(d, 5)
    assert so(handle, 4, 4, 5, d, FAKE, FAKE, FAKE, FAKE) == INV
    L.aclsparseSetMatIndexBase(d, 1)
    assert so(handle, 4, 4, 0, d, FAKE, None, None, None) == 0       # nothing to sort
    assert so(handle, 4, 4, 5, d, FAKE, FAKE, None, FAKE) == INV and so(handle, 4, 4, 5, d, FAKE, FAKE, FAKE, None) == INV
    L.aclsparseDestroyMatDescr(d)
    # cscsort (sparse/cscsort/arch35/cscsort_host.cpp:52-216): csrsort's checks with the columns in the rows' part,
    # and a buffer that must be 128-byte aligned
    bs = L.aclsparseXcscsort_bufferSizeExt
    assert bs(None, 4, 4, 5, FAKE, FAKE, ctypes.byref(n)) == HN
    assert bs(handle, 4, 4, 5, FAKE, FAKE, None) == INV
    for bad in ((-1, 4, 5), (4, -1, 5), (4, 4, -1), (0, 4, 5), (4, 0, 5)):
        assert bs(handle, *bad, FAKE, FAKE, ctypes.byref(n)) == INV, bad
    assert bs(handle, 4, 4, 5, None, FAKE, ctypes.byref(n)) == INV
    assert bs(handle, 4, 4, 5, FAKE, None, ctypes.byref(n)) == INV
    assert bs(handle, 4, 0, 0, None, None, ctypes.byref(n)) == 0 and n.value == 0   # no column: no colPtr needed
    assert bs(handle, 4, 6, 5, FAKE, FAKE, ctypes.byref(n)) == 0 and n.value == L.opsparse_csrsort_workspace_bytes(6, 5)
    assert n.value >= 2 * 5 * 4
    d = ctypes.c_void_p(None)
    L.aclsparseCreateMatDescr(ctypes.byref(d))
    so = L.aclsparseXcscsort
    ALIGNED, ODD = ctypes.c_void_p(0x7f0000001000), ctypes.c_void_p(0x7f0000001040)
    assert so(None, 4, 4, 5, d, FAKE, FAKE, FAKE, ALIGNED) == HN
    assert so(handle, 4, 4, -5, d, FAKE, FAKE, FAKE, ALIGNED) == INV and so(handle, 4, 0, 5, d, FAKE, FAKE, FAKE, ALIGNED) == INV
    assert so(handle, 4, 4, 5, d, None, FAKE, FAKE, ALIGNED) == INV and so(handle, 4, 4, 5, d, FAKE, None, FAKE, ALIGNED) == INV
    assert so(handle, 4, 4, 5, None, FAKE, FAKE, FAKE, ALIGNED) == INV
    L.aclsparseSetMatIndexBase(d, 5)
    assert so(handle, 4, 4, 5, d, FAKE, FAKE, FAKE, ALIGNED) == INV
    L.aclsparseSetMatIndexBase(d, 1)
    assert so(handle, 4, 4, 0, d, FAKE, None, None, None) == 0       # nothing to sort
    assert so(handle, 4, 4, 5, d, FAKE, FAKE, None, ALIGNED) == INV and so(handle, 4, 4, 5, d, FAKE, FAKE, FAKE, None) == INV
    assert so(handle, 4, 4, 5, d, FAKE, FAKE, FAKE, ODD) == INV      # 64-byte aligned only
    L.aclsparseDestroyMatDescr(d)
    # coosort (sparse/coosort/arch35/coosort_host.cpp:48-78, :262-371): m and n must be positive, whatever nnz
    bs = L.aclsparseXcoosort_bufferSizeExt
    assert bs(None, 4, 4, 5, FAKE, FAKE, ctypes.byref(n)) == HN
    assert bs(handle, 4, 4, 5, FAKE, FAKE, None) == INV
    for bad in ((0, 4, 5), (4, 0, 5), (-1, 4, 5), (4, -3, 5), (4, 4, -1), (0, 4, 0)):
        assert bs(handle, *bad, FAKE, FAKE, ctypes.byref(n)) == INV, bad
    assert bs(handle, 4, 4, 5, None, FAKE, ctypes.byref(n)) == INV and bs(handle, 4, 4, 5, FAKE, None, ctypes.byref(n)) == INV
    assert bs(handle, 4, 4, 0, None, None, ctypes.byref(n)) == 0 and n.value == 0
    assert bs(handle, 4, 4, 5, FAKE, FAKE, ctypes.byref(n)) == 0 and n.value == L.opsparse_coosort_workspace_bytes(5)
    assert n.value >= 5 * 12                                         # at least the reference's 12 bytes an entry
    assert bs(handle, 1, 1, IMAX, FAKE, FAKE, ctypes.byref(n)) == 0 and n.value >= 24 * IMAX
    for so in (L.aclsparseXcoosortByRow, L.aclsparseXcoosortByColumn):
        assert so(None, 4, 4, 5, FAKE, FAKE, FAKE, FAKE) == HN
        assert so(handle, 0, 4, 5, FAKE, FAKE, FAKE, FAKE) == INV and so(handle, 4, 0, 5, FAKE, FAKE, FAKE, FAKE) == INV
        assert so(handle, 4, 4, -1, FAKE, FAKE, FAKE, FAKE) == INV
        assert so(handle, 4, 4, 5, None, FAKE, FAKE, FAKE) == INV and so(handle, 4, 4, 5, FAKE, None, FAKE, FAKE) == INV
        assert so(handle, 4, 4, 0, None, None, None, None) == 0      # nothing to sort: P and the buffer may be NULL
        assert so(handle, 4, 4, 5, FAKE, FAKE, None, FAKE) == INV and so(handle, 4, 4, 5, FAKE, FAKE, FAKE, None) == INV
    # csr2csc
    F, NUM, SYM = osa.ACL_FLOAT, osa.ACL_SPARSE_ACTION_NUMERIC, osa.ACL_SPARSE_ACTION_SYMBOLIC
    ptrs = (FAKE, FAKE, FAKE, FAKE, FAKE, FAKE)
    cb = lambda h=handle, m=4, n_=4, nnz=5, p=ptrs, vt=F, cv=NUM, base=0, alg=0, out=ctypes.byref(n): \
        L.aclsparseCsr2cscEx2_bufferSize(h, m, n_, nnz, *p, vt, cv, base, alg, out)
    assert cb(h=None) == HN
    assert cb(m=-1) == INV and cb(n_=-1) == INV and cb(n_=IMAX) == INV and cb(nnz=-1) == INV
    assert cb(vt=osa.ACL_DOUBLE) == NS and cb(vt=osa.ACL_INT32) == NS
    assert cb(cv=2) == INV and cb(base=2) == INV and cb(alg=2) == INV and cb(out=None) == INV
    assert cb(m=-1, vt=osa.ACL_DOUBLE) == INV                       # sizes are checked before the value type
    for vt in (F, osa.ACL_FLOAT16, osa.ACL_BF16, osa.ACL_INT8):
        assert cb(vt=vt) == 0 and n.value == L.opsparse_csr2csc_workspace_bytes(4, 4, 5)
    assert cb(nnz=0) == 0 and n.value == 0 and cb(m=0, nnz=0) == 0 and n.value == 0
    cc = lambda h=handle, m=4, n_=4, nnz=5, p=ptrs, vt=F, cv=NUM, base=0, alg=1, buf=FAKE: \
        L.aclsparseCsr2cscEx2(h, m, n_, nnz, *p, vt, cv, base, alg, buf)
    assert cc(h=None) == HN and cc(vt=osa.ACL_INT64) == NS and cc(alg=5) == INV
    for i in range(6):
        p = list(ptrs)
        p[i] = None
        assert cc(p=tuple(p)) == INV, i
    sym = (None, FAKE, FAKE, None, FAKE, FAKE)                      # SYMBOLIC needs no value arrays ...
    assert cc(p=sym, cv=NUM) == INV
    assert cc(m=0, nnz=5) == INV and cc(n_=0, nnz=5) == INV
    assert cc(nnz=IMAX, base=1) == INV
