"""The compute calls under HIP graph capture.

aclsparseSpMV / aclsparseSpMM only enqueue kernels on the handle's stream once their buffers exist
(GetBufferSize / Preprocess allocate nothing but synchronise; the handle's default workspace is allocated by the
first compute call that needs it), so a serving loop can capture them into a graph and replay it.  Every test
replays its graph three times with eager work of its own between the replays — new contents of x / B, a
synchronisation — and checks every replay against the oracle: a replay must read the operands as they are at
that moment, and must not depend on anything the capture left behind.  alpha / beta in host pointer mode are
frozen into the graph; in device pointer mode the kernels read them at replay time.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import csr_from_lengths, to_dev

pytestmark = pytest.mark.gpu


def _capture(stream, launch):
    launch()  # eager once: first-use allocations (the handle's workspace) happen outside the capture
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        launch()
    return graph


def _power_law(rows, cols, seed, longest, at_least=1):
    rng = np.random.default_rng(seed)
    lengths = np.minimum((rng.pareto(1.2, rows) + at_least).astype(np.int64), longest)
    lengths[rng.integers(0, rows, 3)] = longest
    return csr_from_lengths(lengths, cols, seed + 1)


@pytest.mark.parametrize("kind", ["stream_rows", "stream_rows_lane_groups", "merge_path", "blocked_gather"])
def test_spmv_replays(osa, gpu_ctx, kind):
    dev, stream, handle = gpu_ctx
    alg = osa.ACL_SPARSE_SPMV_ALG_DEFAULT
    if kind == "stream_rows":
        rows = cols = 40_000
        rowptr, colind, val = csr_from_lengths(np.full(rows, 5), cols, 1)
    elif kind == "stream_rows_lane_groups":                 # rows of 100 entries: the persistent kernel, 16 lanes a row
        rows = cols = 20_000
        rowptr, colind, val = csr_from_lengths(np.random.default_rng(5).integers(90, 101, rows), cols, 1)
    elif kind == "merge_path":
        rows, cols = 30_000, 50_000
        rowptr, colind, val = _power_law(rows, cols, 2, 9_000)
    else:
        rows, cols = 30_000, 1_300_000
        rowptr, colind, val = _power_law(rows, cols, 3, 60_000, at_least=80)
        alg = osa.ACL_SPARSE_SPMV_CSR_ALG2
        assert osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0) > 0
    rng = np.random.default_rng(7)
    y0 = rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    d_x = torch.zeros(cols, dtype=torch.float32, device=dev)
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d_x), osa.DnVec(d_y), alg=alg)
    graph = _capture(stream, lambda: op(0.75, -0.5))
    for replay in range(3):
        x = rng.uniform(-1, 1, cols).astype(np.float32)
        d_x.copy_(torch.from_numpy(x))
        d_y.copy_(torch.from_numpy(y0))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 0.75, -0.5)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5, replay


def test_transposed_scatter_layout_replays(osa, gpu_ctx, monkeypatch):
    """op(A) = A^T under the default algorithm with the layout that sorts the products by output panel (its two
    kernels and nothing else between capture and replay): new x and new values of A before every replay."""
    dev, stream, handle = gpu_ctx
    monkeypatch.setenv("OPS_SPARSE_SCATTER_MIN_PANELS", "8")
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.delenv("OPS_SPARSE_SPMV_REPEATABLE", raising=False)
    rows, cols = 1_200_000, 600_000
    rng = np.random.default_rng(11)
    lengths = rng.integers(0, 5, rows)
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    nnz = colind.size
    assert osa.lib().opsparse_spmv_csr_scatter_workspace_bytes(rows, cols, nnz, 0) > 0
    y0 = rng.uniform(-1, 1, cols).astype(np.float32)
    d_rp, d_ci = to_dev(rowptr, dev), to_dev(colind, dev)
    d_val = torch.zeros(nnz, dtype=torch.float32, device=dev)
    d_x = torch.zeros(rows, dtype=torch.float32, device=dev)
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d_rp, d_ci, d_val), osa.DnVec(d_x), osa.DnVec(d_y),
                    op=osa.ACL_SPARSE_OP_TRANSPOSE)
    graph = _capture(stream, lambda: op(1.5, 0.5))
    for replay in range(3):
        x, val = rng.uniform(-1, 1, rows).astype(np.float32), rng.uniform(-1, 1, nnz).astype(np.float32)
        d_x.copy_(torch.from_numpy(x))
        d_val.copy_(torch.from_numpy(val))
        d_y.copy_(torch.from_numpy(y0))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5, replay


def test_spmv_replays_read_device_scalars(osa, gpu_ctx):
    """Device pointer mode: the graph holds the addresses of alpha / beta, every replay reads their values."""
    dev, stream, handle = gpu_ctx
    rows, cols = 20_000, 20_000
    rowptr, colind, val = _power_law(rows, cols, 5, 4_000)
    rng = np.random.default_rng(9)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    A, X, Y = osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y)
    op = osa.SpmvOp(handle, A, X, Y)
    scal = torch.tensor([1.0, 0.0], dtype=torch.float32, device=dev)
    buf = ctypes.c_void_p(op.buffer.data_ptr())

    def launch():
        rc = osa.lib().aclsparseSpMV(handle.h, 0, ctypes.c_void_p(scal.data_ptr()), A.d, X.d,
                                     ctypes.c_void_p(scal.data_ptr() + 4), Y.d, osa.ACL_FLOAT, 0, buf)
        assert rc == 0

    handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_DEVICE)
    try:
        graph = _capture(stream, launch)
    finally:
        handle.set_pointer_mode(osa.ACL_SPARSE_POINTER_MODE_HOST)
    for alpha, beta in ((2.0, 0.0), (-1.5, 0.25), (0.5, 1.0)):
        scal.copy_(torch.tensor([alpha, beta]))
        d_y.copy_(torch.from_numpy(y0))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, alpha, beta)
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5, (alpha, beta)


def test_spmm_replays(osa, gpu_ctx):
    """Slab kernel with long-row segments and their fix-up: three kernels per call, partial rows in the buffer."""
    dev, stream, handle = gpu_ctx
    m, k, n = 6_000, 9_000, 32
    rowptr, colind, val = _power_law(m, k, 11, 3_000)
    rng = np.random.default_rng(13)
    c0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    d_b = torch.zeros(k * n, dtype=torch.float32, device=dev)
    d_c = to_dev(c0.ravel(), dev)
    op = osa.SpmmOp(handle, osa.Csr(m, k, d[0], d[1], d[2]), osa.DnMat(k, n, n, d_b), osa.DnMat(m, n, n, d_c))
    graph = _capture(stream, lambda: op(1.25, 0.5))
    for replay in range(3):
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        d_b.copy_(torch.from_numpy(b.ravel()))
        d_c.copy_(torch.from_numpy(c0.ravel()))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        gold = oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, b, n, c0, n, 1.25, 0.5)
        assert oracle.max_rel_err(d_c.cpu().numpy(), np.asarray(gold).ravel()) <= 1e-5, replay


def test_first_unprepared_call_inside_a_capture(osa, gpu_ctx):
    """The first aclsparseSpMV on a matrix without a preprocessed buffer normally synchronises once to read the row
    statistics.  Inside a capture nothing may synchronise: the call must notice, take the merge path, leave the
    capture intact, and the statistics are then taken by the next eager call."""
    dev, stream, handle = gpu_ctx
    rng = np.random.default_rng(41)
    warm = csr_from_lengths(np.full(100, 3), 100, 1)                 # the handle's workspace exists after this
    d_w = [to_dev(a, dev) for a in warm]
    wx, wy = torch.ones(100, device=dev), torch.zeros(100, device=dev)
    osa.SpmvOp(handle, osa.Csr(100, 100, *d_w), osa.DnVec(wx), osa.DnVec(wy), preprocess=False)(1.0, 0.0)
    stream.synchronize()

    rows = cols = 30_000
    rowptr, colind, val = csr_from_lengths(np.full(rows, 6), cols, 43)  # short even rows: stream rows once seen
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y), preprocess=False)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        op(2.0, 0.5)                                                 # never ran eagerly before
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 2.0, 0.5)
    for replay in range(2):
        d_y.copy_(torch.from_numpy(y0))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5, replay
    d_y.copy_(torch.from_numpy(y0))
    op(2.0, 0.5)                                                     # eager: statistics now, row-wise kernel
    op(1.0, 0.0)
    stream.synchronize()
    gold2 = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, gold.astype(np.float32), 1.0, 0.0)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold2) <= 1e-5


def test_unprepared_spmm_inside_a_capture(osa, gpu_ctx):
    """aclsparseSpMM on a buffer that was never preprocessed for the matrix would analyse the rows first, which
    synchronises; inside a capture it runs without a plan instead and leaves the capture intact.  The same call made
    eagerly afterwards analyses and binds the buffer as usual."""
    import ctypes
    dev, stream, handle = gpu_ctx
    m, k, n = 5_000, 7_000, 64
    rowptr, colind, val = _power_law(m, k, 17, 2_500)               # rows long enough for the binned plan
    rng = np.random.default_rng(19)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    c0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    d_b, d_c = to_dev(b.ravel(), dev), to_dev(c0.ravel(), dev)
    A, B, C = osa.Csr(m, k, d[0], d[1], d[2]), osa.DnMat(k, n, n, d_b), osa.DnMat(m, n, n, d_c)
    L = osa.lib()
    size = ctypes.c_size_t(0)
    args = (handle.h, 0, 0, None, A.d, B.d, None, C.d, osa.ACL_FLOAT, osa.ACL_SPARSE_SPMM_ALG_DEFAULT)
    assert L.aclsparseSpMMGetBufferSize(*args, ctypes.byref(size)) == 0
    buf = torch.empty(max(size.value, 16), dtype=torch.uint8, device=dev)   # sized, but never preprocessed
    alpha, beta = ctypes.c_float(1.5), ctypes.c_float(-0.25)

    def call():
        rc = L.aclsparseSpMM(handle.h, 0, 0, ctypes.byref(alpha), A.d, B.d, ctypes.byref(beta), C.d, osa.ACL_FLOAT,
                             osa.ACL_SPARSE_SPMM_ALG_DEFAULT, ctypes.c_void_p(buf.data_ptr()))
        assert rc == 0

    graph = _capture(stream, call)
    gold = np.asarray(oracle.spmm_f64_rowmajor(m, n, rowptr, colind, val, b, n, c0, n, 1.5, -0.25)).ravel()
    for replay in range(2):
        d_c.copy_(torch.from_numpy(c0.ravel()))
        stream.synchronize()
        graph.replay()
        stream.synchronize()
        assert oracle.max_rel_err(d_c.cpu().numpy(), gold) <= 1e-5, replay
    d_c.copy_(torch.from_numpy(c0.ravel()))
    call()                                                          # eager: analyses, binds, runs the binned kernels
    stream.synchronize()
    assert oracle.max_rel_err(d_c.cpu().numpy(), gold) <= 1e-5
