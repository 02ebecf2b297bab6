"""opsparse_spmv_csr_launch_noalloc (the entry point that allocates nothing) against opsparse_spmv_csr_launch with a
caller's workspace: same kernels, so the results must be bit-equal; and against the fp64 oracle to 1e-5.  Two calls
in a row on the shared static array, the second on a smaller matrix, then the size limit."""
import ctypes

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _matrix(workloads, dev, rows, cols, seed):
    # power-law rows with one long row, so that rows are cut by merge tiles and carries / heads are in play
    A = workloads.power_law_csr(rows, cols, 2.0, 1, min(cols, 6000), seed, dev)
    x = workloads.uniform(seed + 7, cols, -1.0, 1.0, dev)
    y0 = workloads.uniform(seed + 8, rows, -1.0, 1.0, dev)
    return A, x, y0


def test_noalloc_matches_workspace_launch(osa, workloads, gpu_ctx):
    import torch
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    S = lambda v: osa.OpsparseScalar(float(v), None, 0, 0)
    assert L.opsparse_spmv_csr_noalloc_max_bytes() == 4 << 20
    for rows, cols, seed, alpha, beta in ((60000, 50000, 11, 1.25, -0.5), (7000, 9000, 12, -2.0, 0.0)):
        A, x, y0 = _matrix(workloads, dev, rows, cols, seed)
        nnz = int(A["colind"].numel())
        need = L.opsparse_spmv_csr_workspace_bytes(rows, nnz)
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        y_ref, y_new = y0.clone(), y0.clone()
        rc = L.opsparse_spmv_csr_launch(None, 0, P(A["rowptr"]), P(A["colind"]), P(A["values"]), P(x), P(y_ref), rows,
                                        cols, nnz, S(alpha), S(beta), osa.OPSPARSE_F32, osa.OPSPARSE_F32, 0, P(ws),
                                        need, sp)
        assert rc == osa.OPSPARSE_OK
        rc = L.opsparse_spmv_csr_launch_noalloc(P(A["rowptr"]), P(A["colind"]), P(A["values"]), P(x), P(y_new), rows,
                                                cols, nnz, S(alpha), S(beta), osa.OPSPARSE_F32, osa.OPSPARSE_F32, 0, sp)
        assert rc == osa.OPSPARSE_OK
        stream.synchronize()
        assert torch.equal(y_ref, y_new)
        gold = oracle.spmv_f64(rows, cols, A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy(),
                               A["values"].cpu().numpy(), x.cpu().numpy(), y0.cpu().numpy(), alpha, beta)
        assert oracle.max_rel_err(y_new.cpu().numpy(), gold) <= 1e-5
        # and the device's free memory does not move over further calls (hipMemGetInfo: what any allocation, the
        # library's or the runtime's on its behalf, would show in)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
        for _ in range(5):
            assert L.opsparse_spmv_csr_launch_noalloc(P(A["rowptr"]), P(A["colind"]), P(A["values"]), P(x), P(y_new),
                                                      rows, cols, nnz, S(alpha), S(beta), osa.OPSPARSE_F32,
                                                      osa.OPSPARSE_F32, 0, sp) == osa.OPSPARSE_OK
        stream.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before


def test_noalloc_rejects_sizes_beyond_its_array(osa, gpu_ctx):
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    S = lambda v: osa.OpsparseScalar(float(v), None, 0, 0)
    rows, nnz = 1 << 20, 1 << 29  # merge tables of 5 MiB
    assert L.opsparse_spmv_csr_workspace_bytes(rows, nnz) > L.opsparse_spmv_csr_noalloc_max_bytes()
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first and nothing is launched
    rc = L.opsparse_spmv_csr_launch_noalloc(one, one, one, one, one, rows, rows, nnz, S(1), S(0), osa.OPSPARSE_F32,
                                            osa.OPSPARSE_F32, 0, ctypes.c_void_p(stream.cuda_stream))
    assert rc == osa.OPSPARSE_E_WORKSPACE
