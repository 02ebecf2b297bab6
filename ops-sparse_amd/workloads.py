"""Seeded synthetic CSR workloads for the SpMV / SpMM benchmark and the full-size tests.

Everything is generated with torch integer arithmetic from a counter-based
generator (splitmix64 of seed + index), so the same seed gives bit-identical
arrays on the CPU and on the GPU and on any machine — no library RNG stream is
involved.  Uniform floats are (hash >> 40) * 2^-24, exactly representable.

Workloads (sizes are parameters; the defaults are the benchmark's):
  laplacian_2d      5-point stencil on a grid x grid mesh, diagonal 4, off-diagonals -1
  power_law_csr     row lengths ~ l^-alpha on [lmin, lmax] by inverse-CDF table,
                    columns uniform, unique and sorted per row
  uniform_rows_csr  the same column sampling with a fixed number of entries per row
and the algorithmic (compulsory) byte counts the roofline figures are computed from.
"""
import torch

_MASK64 = (1 << 64) - 1


def _s64(v):
    """Python int (mod 2^64) -> the int64 with the same bits."""
    v &= _MASK64
    return v - (1 << 64) if v >= (1 << 63) else v


_GOLDEN = _s64(0x9E3779B97F4A7C15)
_M1 = _s64(0xBF58476D1CE4E5B9)
_M2 = _s64(0x94D049BB133111EB)


def _lsr(z, s):
    """Logical right shift of int64 tensors."""
    return (z >> s) & ((1 << (64 - s)) - 1)


def hash64(seed, idx):
    """splitmix64 output for counter `idx` (int64 tensor) of stream `seed`; int64 bits."""
    z = idx * _GOLDEN + _s64(seed * 0x9E3779B97F4A7C15 + 0x632BE59BD9B4E019)
    z = (z ^ _lsr(z, 30)) * _M1
    z = (z ^ _lsr(z, 27)) * _M2
    return z ^ _lsr(z, 31)


def uniform01(seed, n, device, offset=0):
    """n floats in [0, 1), multiples of 2^-24."""
    idx = torch.arange(offset, offset + n, dtype=torch.int64, device=device)
    return _lsr(hash64(seed, idx), 40).to(torch.float32) * (2.0 ** -24)


def uniform(seed, n, lo, hi, device):
    return uniform01(seed, n, device) * (hi - lo) + lo


def approx_normal(seed, n, device):
    """Irwin-Hall(12) - 6: mean 0, variance 1, exact float arithmetic on every device."""
    acc = torch.zeros(n, dtype=torch.float32, device=device)
    for k in range(12):
        acc += uniform01(seed + 7919 * (k + 1), n, device)
    return acc - 6.0


# ------------------------------------------------------------------ matrices

def laplacian_2d(grid, device):
    """5-point Laplacian on a grid x grid mesh: row i = (r, c) has columns
    {i - grid, i - 1, i, i + 1, i + grid} that exist (no wrap-around at the ends
    of a mesh row), sorted; diagonal 4.0, off-diagonals -1.0."""
    m = grid * grid
    i = torch.arange(m, dtype=torch.int64, device=device)
    r, c = i // grid, i % grid
    offs = (-grid, -1, 0, 1, grid)
    valid = (r > 0, c > 0, torch.ones_like(r, dtype=torch.bool), c < grid - 1, r < grid - 1)
    mask = torch.stack(valid, dim=1)                                   # m x 5, already in column order
    cols = torch.stack([i + o for o in offs], dim=1)
    vals = torch.tensor([-1.0, -1.0, 4.0, -1.0, -1.0], dtype=torch.float32, device=device).expand(m, 5)
    rowptr = torch.zeros(m + 1, dtype=torch.int64, device=device)
    rowptr[1:] = torch.cumsum(mask.sum(dim=1), dim=0)
    return {
        "rows": m, "cols": m,
        "rowptr": rowptr.to(torch.int32),
        "colind": cols[mask].to(torch.int32),
        "values": vals[mask].contiguous(),
    }


def stencil_csr(shape, offsets, device):
    """A stencil on a mesh of `shape` points (2 or 3 extents, the last one fastest): row i couples the point i with
    the points at `offsets` (tuples of as many signed steps) that exist - no wrap-around at the faces - columns
    ascending; the centre carries the number of its neighbours in the stencil, every neighbour -1."""
    dims = len(shape)
    m = 1
    for n in shape:
        m *= n
    i = torch.arange(m, dtype=torch.int64, device=device)
    coords, rest = [], i
    for n in reversed(shape):
        coords.append(rest % n)
        rest = rest // n
    coords.reverse()
    strides = [1] * dims
    for d in range(dims - 2, -1, -1):
        strides[d] = strides[d + 1] * shape[d + 1]
    offsets = sorted(offsets, key=lambda o: sum(o[d] * strides[d] for d in range(dims)))
    masks, cols, vals = [], [], []
    for o in offsets:
        ok = torch.ones(m, dtype=torch.bool, device=device)
        for d in range(dims):
            ok &= (coords[d] + o[d] >= 0) & (coords[d] + o[d] < shape[d])
        masks.append(ok)
        cols.append(i + sum(o[d] * strides[d] for d in range(dims)))
        vals.append(float(len(offsets) - 1) if all(v == 0 for v in o) else -1.0)
    mask = torch.stack(masks, dim=1)
    rowptr = torch.zeros(m + 1, dtype=torch.int64, device=device)
    rowptr[1:] = torch.cumsum(mask.sum(dim=1), dim=0)
    values = torch.tensor(vals, dtype=torch.float32, device=device).expand(m, len(offsets))
    return {"rows": m, "cols": m, "rowptr": rowptr.to(torch.int32),
            "colind": torch.stack(cols, dim=1)[mask].to(torch.int32), "values": values[mask].contiguous()}


def power_law_lengths(m, alpha, lmin, lmax, seed, device, target_mean=None, force_max_row=True):
    """Row lengths with P(l) ~ l^-alpha on [lmin, lmax] (inverse-CDF table lookup).
    target_mean rescales the draw (then clips again); force_max_row pins one row
    (row m // 2) to exactly lmax so the tail is always exercised."""
    l = torch.arange(lmin, lmax + 1, dtype=torch.float64, device=device)
    w = l.pow(-alpha)
    cdf = torch.cumsum(w, dim=0)
    cdf = cdf / cdf[-1]
    u = uniform01(seed, m, device).to(torch.float64)
    lengths = torch.searchsorted(cdf, u, right=True).clamp_(max=lmax - lmin) + lmin
    if target_mean is not None:
        scale = target_mean / lengths.to(torch.float64).mean().item()
        lengths = torch.round(lengths.to(torch.float64) * scale).to(torch.int64).clamp_(lmin, lmax)
    if force_max_row and m > 0:
        lengths[m // 2] = lmax
    return lengths.to(torch.int64)


def sample_sorted_unique_columns(lengths, n, seed, device):
    """For every row r, lengths[r] distinct columns uniform in [0, n), ascending.
    Draw with replacement, sort (row, col) keys, redraw the duplicates, repeat."""
    m = lengths.numel()
    rowptr = torch.zeros(m + 1, dtype=torch.int64, device=device)
    rowptr[1:] = torch.cumsum(lengths, dim=0)
    nnz = int(rowptr[-1].item())
    assert int(lengths.max().item()) <= n if m > 0 else True
    row_of = torch.repeat_interleave(torch.arange(m, dtype=torch.int64, device=device), lengths)
    slot = torch.arange(nnz, dtype=torch.int64, device=device)
    cols = _lsr(hash64(seed, slot), 11) % n
    keys = row_of * n + cols
    rnd = 0
    while True:
        keys, _ = torch.sort(keys)
        dup = torch.zeros(nnz, dtype=torch.bool, device=device)
        dup[1:] = keys[1:] == keys[:-1]
        ndup = int(dup.sum().item())
        if ndup == 0:
            break
        rnd += 1
        where = torch.nonzero(dup).squeeze(1)
        fresh = _lsr(hash64(seed + 104729 * rnd, where), 11) % n
        keys[where] = (keys[where] // n) * n + fresh
    return rowptr, (keys % n)


def power_law_csr(m, n, alpha, lmin, lmax, seed, device, target_mean=None, force_max_row=True):
    lengths = power_law_lengths(m, alpha, lmin, min(lmax, n), seed, device, target_mean, force_max_row)
    rowptr, cols = sample_sorted_unique_columns(lengths, n, seed + 1, device)
    nnz = cols.numel()
    return {
        "rows": m, "cols": n,
        "rowptr": rowptr.to(torch.int32),
        "colind": cols.to(torch.int32),
        "values": uniform(seed + 2, nnz, -1.0, 1.0, device),
    }


def uniform_rows_csr(m, n, per_row, seed, device):
    lengths = torch.full((m,), per_row, dtype=torch.int64, device=device)
    rowptr, cols = sample_sorted_unique_columns(lengths, n, seed, device)
    return {
        "rows": m, "cols": n,
        "rowptr": rowptr.to(torch.int32),
        "colind": cols.to(torch.int32),
        "values": uniform(seed + 1, cols.numel(), -1.0, 1.0, device),
    }


def row_normalise_fp16(csr):
    """Values U(0,1), each row divided by its fp32 row sum, rounded to fp16."""
    device = csr["values"].device
    nnz = csr["colind"].numel()
    u = uniform01(977, nnz, device) * (1.0 - 2.0 ** -10) + 2.0 ** -10      # keep away from 0
    rowptr = csr["rowptr"].to(torch.int64)
    lengths = rowptr[1:] - rowptr[:-1]
    row_of = torch.repeat_interleave(torch.arange(csr["rows"], dtype=torch.int64, device=device), lengths)
    sums = torch.zeros(csr["rows"], dtype=torch.float32, device=device).index_add_(0, row_of, u)
    out = dict(csr)
    out["values"] = (u / sums[row_of]).to(torch.float16)
    return out


# -------------------------------------------------------- benchmark configs

def config_c2(device, grid=2048):
    """SpMV, 5-point Laplacian, alpha = 1, beta = 0.5, x and y0 ~ U(-1, 1)."""
    A = laplacian_2d(grid, device)
    return {"name": "c2_laplacian2d_%d" % grid, "A": A, "x": uniform(1001, A["cols"], -1.0, 1.0, device),
            "y0": uniform(1002, A["rows"], -1.0, 1.0, device), "alpha": 1.0, "beta": 0.5}


def config_c3(device, m=8388608, lmax=200000):
    """SpMV, power-law row lengths (alpha 2.0 on [1, lmax]), alpha = 1, beta = 0."""
    A = power_law_csr(m, m, 2.0, 1, lmax, 2001, device)
    A["values"] = uniform(2002, A["colind"].numel(), -1.0, 1.0, device)
    return {"name": "c3_powerlaw_%d" % m, "A": A, "x": uniform(2003, m, -1.0, 1.0, device),
            "y0": torch.zeros(m, dtype=torch.float32, device=device), "alpha": 1.0, "beta": 0.0}


def config_c4(device, m=1048576, per_row=32, n=64):
    """SpMM fp32, exactly per_row entries per row, B m x n row-major ~ U(-1, 1)."""
    A = uniform_rows_csr(m, m, per_row, 3001, device)
    return {"name": "c4_spmm_uniform%d_%dx%d" % (per_row, m, n), "A": A,
            "B": uniform(3002, m * n, -1.0, 1.0, device).view(m, n), "n": n, "alpha": 1.0, "beta": 0.0}


def config_c5(device, m=2097152, n=128, lmax=50000, mean=16.0):
    """SpMM fp16 in / fp32 out on a power-law graph (alpha 2.1, mean 16), row-normalised values."""
    A = power_law_csr(m, m, 2.1, 1, lmax, 4001, device, target_mean=mean)
    A = row_normalise_fp16(A)
    B = approx_normal(4002, m * n, device).to(torch.float16).view(m, n)
    return {"name": "c5_spmm_gnn_%dx%d" % (m, n), "A": A, "B": B, "n": n, "alpha": 1.0, "beta": 0.0}


# ------------------------------------------------------------- byte models

def spmv_bytes_alg(rows, cols, nnz, val_bytes=4, x_bytes=4, y_bytes=4, beta_nonzero=False):
    """Compulsory traffic of one SpMV: every array once (y twice when it is also read)."""
    return nnz * (val_bytes + 4) + (rows + 1) * 4 + cols * x_bytes + rows * y_bytes * (2 if beta_nonzero else 1)


def spmv_bytes_gather(rows, cols, nnz, val_bytes=4, x_bytes=4, y_bytes=4, beta_nonzero=False):
    """Same with x counted once per non-zero (the per-use convention)."""
    return nnz * (val_bytes + 4 + x_bytes) + (rows + 1) * 4 + rows * y_bytes * (2 if beta_nonzero else 1)


def spmm_bytes_alg(rows, k, n, nnz, val_bytes=4, b_bytes=4, c_bytes=4, beta_nonzero=False):
    return nnz * (val_bytes + 4) + (rows + 1) * 4 + k * n * b_bytes + rows * n * c_bytes * (2 if beta_nonzero else 1)


def spmm_bytes_gather(rows, k, n, nnz, val_bytes=4, b_bytes=4, c_bytes=4, beta_nonzero=False):
    return nnz * (val_bytes + 4 + n * b_bytes) + (rows + 1) * 4 + rows * n * c_bytes * (2 if beta_nonzero else 1)
