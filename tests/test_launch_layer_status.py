"""Status codes of the raw launch layer (include/ops_sparse_hip.h) for arguments it must refuse.

Every case here is answered by host code before anything is enqueued, so the file needs no GPU: the pointers are
addresses of host buffers that the library never follows on these paths.  (The aclsparse entry points' statuses are in
test_abi_status.py; these are the checks underneath them, which a caller of the launch layer meets directly.)"""
import ctypes

import pytest

OK, E_INVALID, E_UNSUPPORTED, E_WORKSPACE = 0, -1, -2, -3


@pytest.fixture(scope="module")
def L(osa):
    assert (osa.OPSPARSE_OK, osa.OPSPARSE_E_INVALID, osa.OPSPARSE_E_UNSUPPORTED, osa.OPSPARSE_E_WORKSPACE) == \
        (OK, E_INVALID, E_UNSUPPORTED, E_WORKSPACE)
    return osa.lib()


@pytest.fixture(scope="module")
def ptr():
    """The address of a host buffer: stands for any non-NULL pointer."""
    buf = ctypes.create_string_buffer(4096)
    yield ctypes.addressof(buf)
    del buf


def _scalars(osa, is_int=0):
    return osa.OpsparseScalar(1.0, None, is_int, 0), osa.OpsparseScalar(0.0, None, is_int, 0)


def _spmv(osa, L, ptr, plan=None, transpose=0, rows=10, cols=10, nnz=20, val=None, out=None, is_int=0, y=True,
          ws=None, ws_bytes=0, col_ind=True):
    a, b = _scalars(osa, is_int)
    return L.opsparse_spmv_csr_launch(ctypes.byref(plan) if plan is not None else None, transpose, ptr,
                                      ptr if col_ind else None, ptr, ptr, ptr if y else None, rows, cols, nnz, a, b,
                                      osa.OPSPARSE_F32 if val is None else val,
                                      osa.OPSPARSE_F32 if out is None else out, is_int, ws, ws_bytes, None)


def _plan(osa, kernel, rows=10, nnz=20, **fields):
    p = osa.OpsparseSpmvPlan()
    p.kernel, p.rows, p.nnz = kernel, rows, nnz
    for k, v in fields.items():
        setattr(p, k, v)
    return p


def test_spmv_launch_refuses_bad_shapes_and_pointers(osa, L, ptr):
    assert _spmv(osa, L, ptr, rows=-1) == E_INVALID
    assert _spmv(osa, L, ptr, nnz=-1) == E_INVALID
    assert _spmv(osa, L, ptr, y=False) == E_INVALID
    assert _spmv(osa, L, ptr, col_ind=False) == E_INVALID
    assert _spmv(osa, L, ptr, rows=0) == OK                                       # nothing to write
    assert _spmv(osa, L, ptr, transpose=1, cols=0) == OK
    assert _spmv(osa, L, ptr, plan=_plan(osa, osa.OPSPARSE_SPMV_MERGE_PATH, rows=11)) == E_INVALID   # another matrix's
    assert _spmv(osa, L, ptr, plan=_plan(osa, osa.OPSPARSE_SPMV_MERGE_PATH, nnz=21)) == E_INVALID


def test_spmv_launch_refuses_type_combinations_it_has_no_kernel_for(osa, L, ptr):
    F32, F16, BF16, I32, I8 = (osa.OPSPARSE_F32, osa.OPSPARSE_F16, osa.OPSPARSE_BF16, osa.OPSPARSE_I32,
                               osa.OPSPARSE_I8)
    for val, out in ((F32, F16), (F32, BF16), (F32, I32), (F16, BF16), (F16, I32), (BF16, F16), (BF16, I32),
                     (I32, F16), (I32, I32), (I8, F32)):
        assert _spmv(osa, L, ptr, val=val, out=out) == E_UNSUPPORTED              # (int32 y: integer compute type)
    assert _spmv(osa, L, ptr, val=F32, out=F32, is_int=1) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, val=I32, out=F32, is_int=1) == E_UNSUPPORTED
    # op(A) = A^T
    assert _spmv(osa, L, ptr, transpose=1, val=F32, out=I32, is_int=1) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, transpose=1, val=I8, out=F32) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, transpose=1, val=F32, out=I32) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, transpose=1, val=F16, out=F16) == E_WORKSPACE       # the fp32 staging vector of a 16-bit y


def test_spmv_launch_refuses_plans_it_cannot_run(osa, L, ptr):
    S, V, M, P = (osa.OPSPARSE_SPMV_STREAM_ROWS, osa.OPSPARSE_SPMV_VECTOR_ROWS, osa.OPSPARSE_SPMV_MERGE_PATH,
                  osa.OPSPARSE_SPMV_COLUMN_PANELS)
    assert _spmv(osa, L, ptr, plan=_plan(osa, S, lanesPerRow=3, rowsPerBlock=8, maxRowNnz=4)) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, S, lanesPerRow=2, rowsPerBlock=0, maxRowNnz=4)) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, S, lanesPerRow=2, rowsPerBlock=768, maxRowNnz=4)) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, V, lanesPerRow=5)) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, M, bytes=1024)) == E_WORKSPACE      # no workspace for the partition
    assert _spmv(osa, L, ptr, plan=_plan(osa, M, bytes=1024), ws=ptr, ws_bytes=512) == E_WORKSPACE
    assert _spmv(osa, L, ptr, plan=_plan(osa, P), val=osa.OPSPARSE_F16) == E_UNSUPPORTED   # the panel copy is fp32
    assert _spmv(osa, L, ptr, plan=_plan(osa, 99)) == E_INVALID
    # the re-stored layouts serve the op(A) and the arithmetic they were built for, on a matrix they fit
    G, LIVE = osa.OPSPARSE_SPMV_BLOCKED_GATHER, osa.OPSPARSE_SPMV_BLOCKED_LIVE
    assert _spmv(osa, L, ptr, plan=_plan(osa, G, transposed=1)) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, G, transposed=0), transpose=1) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, LIVE), transpose=1) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, LIVE), val=osa.OPSPARSE_I32, out=osa.OPSPARSE_I32, is_int=1) == E_INVALID
    assert _spmv(osa, L, ptr, plan=_plan(osa, LIVE, valueType=osa.OPSPARSE_F16)) == E_INVALID        # other values
    assert _spmv(osa, L, ptr, plan=_plan(osa, LIVE), out=osa.OPSPARSE_F16) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, plan=_plan(osa, LIVE, liveValues=1)) == E_INVALID                      # 10 columns: no layout
    assert _spmv(osa, L, ptr, plan=_plan(osa, G), out=osa.OPSPARSE_F16) == E_UNSUPPORTED
    assert _spmv(osa, L, ptr, plan=_plan(osa, G), out=osa.OPSPARSE_I32) == E_UNSUPPORTED             # int32 y, fp sums
    assert _spmv(osa, L, ptr, plan=_plan(osa, G)) == E_INVALID                                       # 10 columns: no layout


def test_spmv_analysis_entry_points_refuse_bad_arguments(osa, L, ptr):
    plan = osa.OpsparseSpmvPlan()
    ref = ctypes.byref(plan)
    assert L.opsparse_spmv_csr_analyse(ptr, 10, 10, 20, ptr, 1 << 20, 0, None, None) == E_INVALID
    assert L.opsparse_spmv_csr_analyse(None, 10, 10, 20, ptr, 1 << 20, 0, ref, None) == E_INVALID
    assert L.opsparse_spmv_csr_analyse(ptr, -1, 10, 20, ptr, 1 << 20, 0, ref, None) == E_INVALID
    assert L.opsparse_spmv_csr_analyse(ptr, 10, 10, 20, None, 0, 0, ref, None) == E_WORKSPACE
    assert L.opsparse_spmv_csr_analyse(ptr, 10, 10, 20, ptr, 8, 0, ref, None) == E_WORKSPACE
    assert L.opsparse_spmv_csr_analyse(ptr, 10, 10, 0, None, 0, 0, ref, None) == OK
    assert plan.kernel == osa.OPSPARSE_SPMV_SCALE_ONLY and plan.rows == 10 and plan.nnz == 0

    scattered = ctypes.c_int32(7)
    assert L.opsparse_spmv_csr_gathers_scattered(ptr, ptr, 10, 10, 20, ptr, 4096, None, None) == E_INVALID
    assert L.opsparse_spmv_csr_gathers_scattered(None, ptr, 10, 10, 20, ptr, 4096, ctypes.byref(scattered), None) == \
        E_INVALID
    assert L.opsparse_spmv_csr_gathers_scattered(ptr, ptr, 0, 10, 0, None, 0, ctypes.byref(scattered), None) == OK
    assert scattered.value == 0
    assert L.opsparse_spmv_csr_gathers_scattered(ptr, ptr, 10, 10, 20, None, 0, ctypes.byref(scattered), None) == \
        E_WORKSPACE

    wide = (300_000, 1_400_000, 3_000_000)                                        # a shape the layouts apply to
    assert L.opsparse_spmv_csr_panels_analyse(ptr, ptr, ptr, *wide, ptr, 4096, None, None) == E_INVALID
    assert L.opsparse_spmv_csr_panels_analyse(ptr, ptr, ptr, 10, 10, 20, ptr, 4096, ref, None) == E_UNSUPPORTED
    assert L.opsparse_spmv_csr_panels_analyse(ptr, ptr, ptr, *wide, None, 0, ref, None) == E_WORKSPACE
    assert L.opsparse_spmv_csr_panels_analyse(ptr, ptr, ptr, *wide, ptr, 4096, ref, None) == E_WORKSPACE
    for analyse, flag_refused in ((L.opsparse_spmv_csr_blocked_analyse, None),
                                  (L.opsparse_spmv_csr_live_analyse, osa.OPSPARSE_BLOCKED_TRANSPOSE)):
        assert analyse(ptr, ptr, ptr, *wide, 0, ptr, 1 << 40, None, None) == E_INVALID   # (the size is only compared)
        assert analyse(None, ptr, ptr, *wide, 0, ptr, 1 << 40, ref, None) == E_INVALID
        assert analyse(ptr, ptr, ptr, 10, 10, 20, 0, ptr, 4096, ref, None) == E_UNSUPPORTED
        assert analyse(ptr, ptr, ptr, *wide, 0, None, 0, ref, None) == E_WORKSPACE
        assert analyse(ptr, ptr, ptr, *wide, 0, ptr, 4096, ref, None) == E_WORKSPACE
        if flag_refused is not None:
            assert analyse(ptr, ptr, ptr, *wide, flag_refused, ptr, 1 << 40, ref, None) == E_UNSUPPORTED
    assert L.opsparse_spmv_csr_live_analyse(ptr, ptr, ptr, *wide, osa.OPSPARSE_BLOCKED_VALUES_I32, ptr, 1 << 40, ref,
                                            None) == E_UNSUPPORTED
    # the split form: the resident part is large enough, the scratch is not
    keep = L.opsparse_spmv_csr_blocked_resident_bytes(*wide, 0)
    assert 0 < keep < L.opsparse_spmv_csr_blocked_workspace_bytes(*wide, 0)
    assert L.opsparse_spmv_csr_blocked_analyse_split(ptr, ptr, ptr, *wide, 0, ptr, keep, ptr, 4096, ref, None) == \
        E_WORKSPACE
    keep = L.opsparse_spmv_csr_live_resident_bytes(*wide)
    assert 0 < keep < L.opsparse_spmv_csr_live_workspace_bytes(*wide)
    assert L.opsparse_spmv_csr_live_analyse_split(ptr, ptr, ptr, *wide, 0, ptr, keep, ptr, 4096, ref, None) == \
        E_WORKSPACE


def test_other_spmv_entry_points_refuse_bad_arguments(osa, L, ptr):
    a, b = _scalars(osa)
    assert L.opsparse_spmv_csr_launch_noalloc(ptr, ptr, ptr, ptr, ptr, -1, 10, 20, a, b, 0, 0, 0, None) == E_INVALID
    beyond = 1 << 29                                                              # tables of 4 MiB do not hold this
    assert L.opsparse_spmv_csr_workspace_bytes(beyond, beyond) > L.opsparse_spmv_csr_noalloc_max_bytes()
    assert L.opsparse_spmv_csr_launch_noalloc(ptr, ptr, ptr, ptr, ptr, beyond, 10, beyond, a, b, 0, 0, 0, None) == \
        E_WORKSPACE
    assert L.opsparse_rebase_offsets_launch(ptr, 0, 2, 10, ptr, None) == E_INVALID
    assert L.opsparse_rebase_offsets_launch(ptr, 0, 0, -1, ptr, None) == E_INVALID
    assert L.opsparse_rebase_offsets_launch(None, 0, 0, 10, ptr, None) == E_INVALID
    assert L.opsparse_rebase_offsets_launch(None, 1, 1, 0, None, None) == OK
    idx = lambda **kw: L.opsparse_spmv_csr_indexed_launch(
        kw.get("offsets", ptr), 0, kw.get("base", 0), ptr, ptr, ptr, ptr, kw.get("z", ptr), kw.get("rows", 10), 10, 20,
        a, b, None)
    assert idx(rows=-1) == E_INVALID and idx(base=2) == E_INVALID and idx(z=None) == E_INVALID
    assert idx(offsets=None) == E_INVALID and idx(rows=0) == OK


def test_spmm_launch_layer_refuses_bad_arguments(osa, L, ptr):
    a, b = _scalars(osa)
    plan = osa.OpsparseSpmmPlan()
    size = ctypes.c_size_t(0)
    assert L.opsparse_spmm_csr_analyse(ptr, 10, 20, 8, ptr, 4096, 0, None, None) == E_INVALID
    assert L.opsparse_spmm_csr_analyse(None, 10, 20, 8, ptr, 4096, 0, ctypes.byref(plan), None) == E_INVALID
    assert L.opsparse_spmm_csr_analyse(ptr, 10, 20, 8, None, 0, 0, ctypes.byref(plan), None) == E_WORKSPACE
    assert L.opsparse_spmm_csr_analyse(ptr, 10, 20, 8, ptr, 255, 0, ctypes.byref(plan), None) == E_WORKSPACE
    assert L.opsparse_spmm_csr_analyse(ptr, 10, 20, 8, ptr, 256, 0, ctypes.byref(plan), None) == OK   # no row is long
    assert plan.kernel == osa.OPSPARSE_SPMM_ROW_SPLIT and plan.bytes == 256

    def launch(plan=None, rows=10, k=10, n=8, nnz=20, ldb=8, ldc=8, col_ind=True, c=True, val=None, ct=None, ws=None,
               ws_bytes=0):
        return L.opsparse_spmm_csr_launch(ctypes.byref(plan) if plan is not None else None, ptr,
                                          ptr if col_ind else None, ptr, ptr, ptr if c else None, rows, k, n, nnz, ldb,
                                          ldc, 0, 0, 0, a, b, osa.OPSPARSE_F32 if val is None else val,
                                          osa.OPSPARSE_F32 if ct is None else ct, ws, ws_bytes, None)

    assert launch(rows=-1) == E_INVALID and launch(ldb=0) == E_INVALID and launch(n=1 << 31) == E_INVALID
    assert launch(rows=0) == OK and launch(n=0) == OK
    assert launch(col_ind=False) == E_INVALID and launch(c=False) == E_INVALID
    plan.rows, plan.nnz, plan.n = 10, 20, 8
    assert launch(plan=plan, nnz=21) == E_INVALID
    plan.kernel, plan.bytes = osa.OPSPARSE_SPMM_BINNED, 4096
    assert launch(plan=plan, n=16, ldb=16, ldc=16) == E_INVALID                   # analysed for another width
    assert launch(plan=plan) == E_WORKSPACE
    assert launch(plan=plan, ws=ptr, ws_bytes=1024) == E_WORKSPACE
    for val, ct in ((osa.OPSPARSE_F32, osa.OPSPARSE_F16), (osa.OPSPARSE_BF16, osa.OPSPARSE_F32),
                    (osa.OPSPARSE_I8, osa.OPSPARSE_F32), (osa.OPSPARSE_I32, osa.OPSPARSE_I32)):
        assert launch(val=val, ct=ct) == E_UNSUPPORTED

    restage = lambda **kw: L.opsparse_dense_restage(
        kw.get("src", ptr), kw.get("dst", ptr), kw.get("rows", 8), 8, kw.get("cols_dst", 8), kw.get("ld_src", 8), 0,
        kw.get("ld_dst", 8), kw.get("dst_col_major", 0), kw.get("elem", 4), None)
    assert restage(rows=-1) == E_INVALID and restage(cols_dst=7) == E_INVALID and restage(ld_src=0) == E_INVALID
    assert restage(elem=3) == E_INVALID and restage(ld_dst=7) == E_INVALID
    assert restage(rows=9, dst_col_major=1) == E_INVALID                          # column-major rows do not fit ldDst
    assert restage(rows=0) == OK
    assert restage(src=None) == E_INVALID and restage(dst=None) == E_INVALID
    assert restage(rows=1 << 30, cols_dst=1 << 20, ld_dst=1 << 20) == E_UNSUPPORTED   # more tiles than a grid holds


def test_conversion_launchers_refuse_bad_arguments(osa, L, ptr):
    big = 1 << 31
    coo2csr = lambda ind=ptr, nnz=20, m=10, out=ptr, base=0, ws=ptr, ws_bytes=1 << 20: \
        L.opsparse_coo2csr_launch(ind, nnz, m, out, base, ws, ws_bytes, None)
    assert coo2csr(nnz=-1) == E_INVALID and coo2csr(nnz=big) == E_INVALID and coo2csr(base=2) == E_INVALID
    assert coo2csr(out=None) == E_INVALID and coo2csr(ind=None) == E_INVALID and coo2csr(m=0) == E_INVALID
    assert coo2csr(ws=None) == E_WORKSPACE and coo2csr(ws_bytes=4) == E_WORKSPACE

    csr2coo = lambda ptr_=ptr, nnz=20, m=10, out=ptr, base=0: L.opsparse_csr2coo_launch(ptr_, nnz, m, out, base, None)
    assert csr2coo(nnz=-1) == E_INVALID and csr2coo(base=-1) == E_INVALID and csr2coo(m=0) == E_INVALID
    assert csr2coo(ptr_=None) == E_INVALID and csr2coo(out=None) == E_INVALID
    assert csr2coo(nnz=0) == OK and csr2coo(nnz=0, m=0, ptr_=None, out=None) == OK

    csrsort = lambda m=10, n=10, nnz=20, base=0, rp=ptr, ci=ptr, perm=ptr, ws=ptr, ws_bytes=1 << 20: \
        L.opsparse_csrsort_launch(m, n, nnz, base, rp, ci, perm, ws, ws_bytes, None)
    assert csrsort(m=-1) == E_INVALID and csrsort(nnz=big) == E_INVALID and csrsort(base=3) == E_INVALID
    assert csrsort(n=0) == E_INVALID                                              # entries without columns
    assert csrsort(nnz=0, rp=None, ci=None, perm=None, ws=None) == OK
    assert csrsort(rp=None) == E_INVALID and csrsort(ci=None) == E_INVALID and csrsort(perm=None) == E_INVALID
    assert csrsort(ws=None) == E_WORKSPACE and csrsort(ws_bytes=16) == E_WORKSPACE

    csr2csc = lambda m=10, n=10, nnz=20, val=ptr, rp=ptr, ci=ptr, cval=ptr, cp=ptr, ri=ptr, vb=4, base=0, ws=ptr, \
        ws_bytes=1 << 20: L.opsparse_csr2csc_launch(m, n, nnz, val, rp, ci, cval, cp, ri, vb, base, ws, ws_bytes, None)
    assert csr2csc(m=-1) == E_INVALID and csr2csc(nnz=big) == E_INVALID and csr2csc(base=2) == E_INVALID
    assert csr2csc(m=0) == E_INVALID and csr2csc(cp=None) == E_INVALID and csr2csc(vb=3) == E_INVALID
    assert csr2csc(rp=None) == E_INVALID and csr2csc(ri=None) == E_INVALID and csr2csc(val=None) == E_INVALID
    assert csr2csc(cval=None) == E_INVALID
    assert csr2csc(ws=None) == E_WORKSPACE and csr2csc(ws_bytes=64) == E_WORKSPACE

    coosort = lambda nnz=20, rows=ptr, cols=ptr, perm=ptr, ws=ptr, ws_bytes=1 << 20: \
        L.opsparse_coosort_launch(nnz, 1, rows, cols, perm, ws, ws_bytes, None)
    assert coosort(nnz=-1) == E_INVALID and coosort(nnz=big) == E_INVALID
    assert coosort(nnz=0, rows=None, cols=None, perm=None, ws=None) == OK
    assert coosort(rows=None) == E_INVALID and coosort(cols=None) == E_INVALID and coosort(perm=None) == E_INVALID
    assert coosort(ws=None) == E_WORKSPACE and coosort(ws_bytes=16) == E_WORKSPACE


def test_measurement_launchers_refuse_bad_arguments(osa, L, ptr):
    assert L.opsparse_copy_launch(None, ptr, 16, None) == E_INVALID
    assert L.opsparse_copy_launch(ptr, None, 16, None) == E_INVALID
    assert L.opsparse_copy_launch(ptr, ptr, 10, None) == E_INVALID
    assert L.opsparse_copy_launch(ptr, ptr, 0, None) == OK
    assert L.opsparse_read_launch(None, 16, None, None) == E_INVALID
    assert L.opsparse_read_launch(ptr, 0, None, None) == OK
    assert L.opsparse_gather_launch(None, ptr, 4, None, None) == E_INVALID
    assert L.opsparse_gather_launch(ptr, None, 4, None, None) == E_INVALID
    assert L.opsparse_gather_launch(ptr, ptr, 0, None, None) == OK
