"""Helpers shared by the parity tests: small seeded CSR builders (numpy), upload
to the GPU, and runners that call the library through its C ABI."""
import ctypes

import numpy as np


def random_csr(rows, cols, density, seed, lo=-5.0, hi=5.0, empty_row_prob=0.0, unsorted=False, duplicates=False):
    """Random CSR in the shape of the reference's GenerateCsr
    (test/spmv/arch22/spmv_test.cpp:102-152): binomial row lengths, distinct
    sorted columns, values U(lo, hi).  `unsorted` shuffles each row, `duplicates`
    repeats some column indices inside a row (both are legal inputs)."""
    rng = np.random.default_rng(seed)
    lengths = rng.binomial(cols, density, size=rows) if cols > 0 else np.zeros(rows, np.int64)
    if empty_row_prob > 0:
        lengths[rng.random(rows) < empty_row_prob] = 0
    rowptr = np.zeros(rows + 1, np.int64)
    np.cumsum(lengths, out=rowptr[1:])
    colind = np.empty(int(rowptr[-1]), np.int32)
    for r in range(rows):
        k = int(lengths[r])
        if k == 0:
            continue
        c = rng.choice(cols, size=k, replace=False)
        c.sort()
        if duplicates and k >= 2:
            c[1::3] = c[0::3][: len(c[1::3])]
        if unsorted:
            rng.shuffle(c)
        colind[rowptr[r]:rowptr[r + 1]] = c
    val = rng.uniform(lo, hi, size=colind.size).astype(np.float32)
    return rowptr.astype(np.int32), colind, val


def csr_from_lengths(lengths, cols, seed, lo=-1.0, hi=1.0):
    """CSR with prescribed row lengths, distinct sorted uniform columns."""
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, np.int64)
    rowptr = np.zeros(lengths.size + 1, np.int64)
    np.cumsum(lengths, out=rowptr[1:])
    colind = np.empty(int(rowptr[-1]), np.int32)
    for r, k in enumerate(lengths):
        if k:
            c = rng.choice(cols, size=int(k), replace=False)
            c.sort()
            colind[rowptr[r]:rowptr[r + 1]] = c
    val = rng.uniform(lo, hi, size=colind.size).astype(np.float32)
    return rowptr.astype(np.int32), colind, val


def dense_from_csr(rows, cols, rowptr, colind, val):
    """Dense fp64 matrix with duplicates summed (for brute-force checks)."""
    A = np.zeros((rows, cols), np.float64)
    for r in range(rows):
        for p in range(rowptr[r], rowptr[r + 1]):
            A[r, colind[p]] += float(val[p])
    return A


def to_dev(a, dev, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(dev)


def run_spmv(osa, gpu_ctx, rows, cols, rowptr, colind, val, x, y0, alpha, beta, preprocess=True,
             op=None, val_dtype=None, out_dtype=None, compute_type=None, force_kernel=None):
    """y = alpha*op(A)*x + beta*y0 through aclsparseSpMV (or, with force_kernel,
    through the raw launch layer with that kernel family).  Returns y as numpy."""
    import torch
    dev, stream, handle = gpu_ctx
    op = osa.ACL_SPARSE_OP_NON_TRANSPOSE if op is None else op
    compute_type = osa.ACL_FLOAT if compute_type is None else compute_type
    d_rowptr, d_colind = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val = to_dev(val, dev, val_dtype)
    d_x = to_dev(x, dev, val_dtype)
    d_y = to_dev(y0, dev, out_dtype)
    if force_kernel is not None:
        L = osa.lib()
        nnz = int(colind.size)
        ws_bytes = L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        plan = osa.OpsparseSpmvPlan()
        sp = ctypes.c_void_p(stream.cuda_stream)
        rc = L.opsparse_spmv_csr_analyse(d_rowptr.data_ptr(), rows, cols, nnz, ws.data_ptr(), ws_bytes, force_kernel,
                                         ctypes.byref(plan), sp)
        assert rc == 0, "analyse rc=%d" % rc
        dt = {torch.float32: osa.OPSPARSE_F32, torch.float16: osa.OPSPARSE_F16, torch.bfloat16: osa.OPSPARSE_BF16,
              torch.int32: osa.OPSPARSE_I32}
        sa = osa.OpsparseScalar(float(alpha), None, int(compute_type == osa.ACL_INT32), 0)
        sb = osa.OpsparseScalar(float(beta), None, int(compute_type == osa.ACL_INT32), 0)
        rc = L.opsparse_spmv_csr_launch(ctypes.byref(plan), 0, d_rowptr.data_ptr(), d_colind.data_ptr() or None,
                                        d_val.data_ptr() or None, d_x.data_ptr() or None, d_y.data_ptr(), rows, cols,
                                        nnz, sa, sb, dt[d_val.dtype], dt[d_y.dtype],
                                        int(compute_type == osa.ACL_INT32), ws.data_ptr(), ws_bytes, sp)
        assert rc == 0, "launch rc=%d" % rc
        stream.synchronize()
        return d_y.cpu().float().numpy() if d_y.dtype != torch.int32 else d_y.cpu().numpy()
    A = osa.Csr(rows, cols, d_rowptr, d_colind, d_val)
    X, Y = osa.DnVec(d_x), osa.DnVec(d_y)
    spmv = osa.SpmvOp(handle, A, X, Y, op=op, compute_type=compute_type, preprocess=preprocess)
    spmv(alpha, beta)
    stream.synchronize()
    # inputs must come back untouched
    assert np.array_equal(d_rowptr.cpu().numpy(), rowptr) and np.array_equal(d_colind.cpu().numpy(), colind)
    out = d_y.cpu()
    return out.numpy() if out.dtype == torch.int32 else out.float().numpy()


def run_spmm(osa, gpu_ctx, m, k, n, rowptr, colind, val, B_flat, ldb, C_flat, ldc, alpha, beta, order_b=None,
             order_c=None, op_b=None, val_dtype=None, c_dtype=None, compute_type=None, alg=None):
    """C = alpha*A*op(B) + beta*C through GetBufferSize / Preprocess / SpMM.
    B_flat and C_flat are flat arrays in storage layout.  Returns C flat (numpy)."""
    import torch
    dev, stream, handle = gpu_ctx
    order_b = osa.ACL_SPARSE_ORDER_ROW if order_b is None else order_b
    order_c = osa.ACL_SPARSE_ORDER_ROW if order_c is None else order_c
    op_b = osa.ACL_SPARSE_OP_NON_TRANSPOSE if op_b is None else op_b
    compute_type = osa.ACL_FLOAT if compute_type is None else compute_type
    alg = osa.ACL_SPARSE_SPMM_ALG_DEFAULT if alg is None else alg
    d_rowptr, d_colind = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val = to_dev(val, dev, val_dtype)
    d_B = to_dev(B_flat, dev, val_dtype)
    d_C = to_dev(C_flat, dev, c_dtype)
    A = osa.Csr(m, k, d_rowptr, d_colind, d_val)
    Bd = osa.DnMat(k, n, ldb, d_B, order_b)
    Cd = osa.DnMat(m, n, ldc, d_C, order_c)
    spmm = osa.SpmmOp(handle, A, Bd, Cd, op_b=op_b, compute_type=compute_type, alg=alg)
    spmm(alpha, beta)
    stream.synchronize()
    assert np.array_equal(d_rowptr.cpu().numpy(), rowptr) and np.array_equal(d_colind.cpu().numpy(), colind)
    out = d_C.cpu()
    return out.numpy() if out.dtype == torch.int32 else out.float().numpy()
