"""CPU tests of the synthetic workload generators (ops-sparse_amd/workloads.py) at small
sizes: structure invariants, closed forms, determinism, and the byte models."""
import numpy as np
import torch

import oracle


def _np(csr):
    return csr["rowptr"].numpy(), csr["colind"].numpy(), csr["values"].float().numpy()


def test_laplacian_structure_and_closed_form(workloads):
    g = 16
    A = workloads.laplacian_2d(g, "cpu")
    rowptr, colind, val = _np(A)
    m = g * g
    assert A["rows"] == m and colind.size == 5 * m - 4 * g
    lengths = np.diff(rowptr)
    assert lengths.min() == 3 and lengths.max() == 5
    for r in range(m):
        c = colind[rowptr[r]:rowptr[r + 1]]
        assert np.all(np.diff(c) > 0) and r in c
    # A * 1 = number of missing neighbours: 0 inside, 1 on an edge, 2 in a corner
    y = oracle.spmv_f64(m, m, rowptr, colind, val, np.ones(m, np.float32), None, 1.0, 0.0).reshape(g, g)
    assert np.all(y[1:-1, 1:-1] == 0) and y[0, 0] == 2 and y[0, 5] == 1 and y[7, g - 1] == 1
    # no wrap-around between the end of one mesh row and the start of the next
    r = g - 1
    assert r + 1 not in colind[rowptr[r]:rowptr[r + 1]]


def test_stencil_generator(workloads):
    """The general mesh generator: its 5-point stencil in two dimensions is the Laplacian above array for array; a
    27-point stencil has 27 entries inside and 8 in a corner, ascending columns, and A * 1 counts the neighbours that
    a point at a face lacks."""
    import itertools
    cross = [o for o in itertools.product((-1, 0, 1), repeat=2) if sum(abs(v) for v in o) <= 1]
    A, L = workloads.stencil_csr((7, 7), cross, "cpu"), workloads.laplacian_2d(7, "cpu")
    assert all(torch.equal(A[k], L[k]) for k in ("rowptr", "colind", "values"))
    shape = (4, 5, 6)
    B = workloads.stencil_csr(shape, list(itertools.product((-1, 0, 1), repeat=3)), "cpu")
    rowptr, colind, val = _np(B)
    m = 4 * 5 * 6
    lengths = np.diff(rowptr).reshape(shape)
    assert B["rows"] == m and lengths[1, 2, 3] == 27 and lengths[0, 0, 0] == 8 and lengths[0, 2, 3] == 18
    for r in range(m):
        c = colind[rowptr[r]:rowptr[r + 1]]
        assert np.all(np.diff(c) > 0) and r in c
    y = oracle.spmv_f64(m, m, rowptr, colind, val, np.ones(m, np.float32), None, 1.0, 0.0).reshape(shape)
    assert np.array_equal(y, 27 - lengths)


def test_sorted_unique_uniform_columns(workloads):
    A = workloads.uniform_rows_csr(500, 300, 32, 3001, "cpu")
    rowptr, colind, val = _np(A)
    assert np.array_equal(np.diff(rowptr), np.full(500, 32))
    c = colind.reshape(500, 32)
    assert np.all(np.diff(c, axis=1) > 0) and c.min() >= 0 and c.max() < 300
    assert np.all(np.abs(val) <= 1.0) and val.std() > 0.4
    B = workloads.uniform_rows_csr(500, 300, 32, 3001, "cpu")
    assert all(torch.equal(A[k], B[k]) for k in ("rowptr", "colind", "values"))      # deterministic


def test_power_law_lengths(workloads):
    A = workloads.power_law_csr(20000, 20000, 2.0, 1, 5000, 2001, "cpu")
    rowptr, colind, _ = _np(A)
    lengths = np.diff(rowptr)
    assert lengths.min() >= 1 and lengths.max() == 5000 and lengths[10000] == 5000
    assert np.median(lengths) <= 2 and 3.0 < lengths.mean() < 12.0                     # heavy tail, small median
    for r in (0, 10000, 19999):
        c = colind[rowptr[r]:rowptr[r + 1]]
        assert np.all(np.diff(c) > 0)
    G = workloads.power_law_csr(20000, 20000, 2.1, 1, 5000, 4001, "cpu", target_mean=16.0)
    gl = np.diff(G["rowptr"].numpy())
    assert 12.0 < gl.mean() < 20.0


def test_row_normalised_fp16(workloads):
    A = workloads.row_normalise_fp16(workloads.power_law_csr(2000, 2000, 2.1, 1, 500, 7, "cpu", target_mean=16.0))
    rowptr = A["rowptr"].numpy()
    v = A["values"].float().numpy()
    assert A["values"].dtype == torch.float16 and v.min() > 0
    sums = np.add.reduceat(v, rowptr[:-1])
    assert np.allclose(sums, 1.0, atol=2e-2)


def test_hash_is_device_independent_arithmetic(workloads):
    idx = torch.arange(5, dtype=torch.int64)
    h = workloads.hash64(1001, idx).numpy().astype(np.uint64)

    def splitmix(seed, i):
        m = (1 << 64) - 1
        z = (i * 0x9E3779B97F4A7C15 + seed * 0x9E3779B97F4A7C15 + 0x632BE59BD9B4E019) & m
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        return z ^ (z >> 31)

    assert [int(x) for x in h] == [splitmix(1001, i) for i in range(5)]
    u = workloads.uniform01(5, 1000, "cpu").numpy()
    assert u.min() >= 0 and u.max() < 1 and abs(u.mean() - 0.5) < 0.05
    assert np.all(u * 2.0 ** 24 == np.round(u * 2.0 ** 24))


def test_byte_models(workloads):
    # figures quoted for the benchmark configurations
    assert workloads.spmv_bytes_alg(4096, 4096, 65536) == 573444
    assert workloads.spmv_bytes_alg(4194304, 4194304, 20963328, beta_nonzero=True) == 234815492
    assert workloads.spmm_bytes_alg(1048576, 1048576, 64, 33554432) == 809500676
    assert workloads.spmm_bytes_gather(1048576, 1048576, 64, 33554432) == 9130999812
