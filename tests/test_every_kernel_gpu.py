"""Every kernel instantiation and dispatch arm of the launch layer, reached on purpose.

The dispatchers of spmv_kernels.hip, spmv_blocked*.hip and spmm_kernels.hip pick a kernel template by element types,
lanes a row, issue depth, lane-group width and address width.  The API tests reach the combinations that ordinary
matrices ask for; the cases here go through the raw launch layer (include/ops_sparse_hip.h) and set the plan fields
or operand shapes that select each remaining one, on matrices small enough for the fp64 oracle.  Each case names the
instantiations it is there for.

Bars: fp32 outputs 1e-5 relative to the largest element of the fp64 oracle; fp16 / bf16 outputs one unit in the last
place of the oracle rounded to that type; integer outputs exact."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import csr_from_lengths, to_dev

pytestmark = pytest.mark.gpu

# name -> (dtype of values and x, dtype of y, integer compute type)
SPMV_TYPES = {
    "f32": (torch.float32, torch.float32, False),
    "f16_f32": (torch.float16, torch.float32, False),
    "f16_f16": (torch.float16, torch.float16, False),
    "bf16_f32": (torch.bfloat16, torch.float32, False),
    "bf16_bf16": (torch.bfloat16, torch.bfloat16, False),
    "i32_f32": (torch.int32, torch.float32, False),
    "i32_i32": (torch.int32, torch.int32, True),
}
ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def _type_code(osa, dtype):
    return {torch.float32: osa.OPSPARSE_F32, torch.float16: osa.OPSPARSE_F16, torch.bfloat16: osa.OPSPARSE_BF16,
            torch.int32: osa.OPSPARSE_I32, torch.int8: osa.OPSPARSE_I8}[dtype]


def _as_seen(a, dtype):
    """The values the device sees after conversion to `dtype`, as fp32 (int32 stays int32)."""
    if dtype == torch.int32:
        return a.astype(np.int32)
    return torch.from_numpy(a.astype(np.float32)).to(dtype).float().numpy()


def _operands(rng, nnz, n_x, n_y, val_dtype, out_dtype, small=False):
    if val_dtype == torch.int32:
        # products wrap in the integer sums; `small`: sums that fp32 holds exactly whatever their order
        big = 40_000 if out_dtype == torch.int32 else (4 if small else 1_000)
        val, x = rng.integers(-big, big, nnz), rng.integers(-big, big, n_x)
    else:
        val, x = rng.uniform(-2, 2, nnz), rng.uniform(-2, 2, n_x)
    y0 = rng.integers(-1000, 1000, n_y).astype(np.int32) if out_dtype == torch.int32 else \
        _as_seen(rng.uniform(-2, 2, n_y), out_dtype)
    return _as_seen(val, val_dtype), _as_seen(x, val_dtype), y0


def _check_spmv(y, rows, cols, rowptr, colind, val, x, y0, alpha, beta, out_dtype, transpose=False):
    if out_dtype == torch.int32:
        assert not transpose
        assert np.array_equal(y, oracle.spmv_i32(rows, rowptr, colind, val, x, y0, alpha, beta))
        return
    fn = oracle.spmv_trans_f64 if transpose else oracle.spmv_f64
    gold = fn(rows, cols, rowptr, colind, val.astype(np.float32), x.astype(np.float32), y0, alpha, beta)
    if out_dtype == torch.float32:
        if transpose:                         # fp32 atomics in unspecified order: the reference's rule for op(A) = A^T
            d = np.abs(y - gold)
            assert (d <= 2.0 ** -16 + 2.0 ** -10 * np.abs(gold)).mean() >= 0.99 and d.max() <= 1e-2
        else:
            assert oracle.max_rel_err(y, gold) <= 1e-5
    else:
        want = _as_seen(gold, out_dtype)
        bar = ULP[out_dtype] * np.maximum(np.abs(want), 2.0 ** -14)
        if transpose:                         # fp32 sums in unspecified order, rounded once more to the type of y
            bar = 2 * bar + 2.0 ** -12
        assert np.all(np.abs(y - want) <= bar)


class RawSpmv:
    """A matrix and its operands on the device, launched through opsparse_spmv_csr_launch with a plan of the test's
    making."""

    def __init__(self, osa, gpu_ctx, rowptr, colind, cols, types, seed, transpose=False):
        self.osa, (self.dev, self.stream, _) = osa, gpu_ctx
        self.L = osa.lib()
        self.val_dtype, self.out_dtype, self.is_int = SPMV_TYPES[types]
        self.rowptr, self.colind, self.rows, self.cols = rowptr, colind, rowptr.size - 1, cols
        self.nnz, self.transpose = int(colind.size), transpose
        rng = np.random.default_rng(seed)
        n_x, n_y = (self.rows, cols) if transpose else (cols, self.rows)
        self.val, self.x, self.y0 = _operands(rng, self.nnz, n_x, n_y, self.val_dtype, self.out_dtype,
                                              small=transpose)
        self.d_rp, self.d_ci = to_dev(rowptr, self.dev), to_dev(colind, self.dev)
        self.d_val, self.d_x = to_dev(self.val, self.dev, self.val_dtype), to_dev(self.x, self.dev, self.val_dtype)
        self.d_y = to_dev(self.y0, self.dev, self.out_dtype)
        self.sp = ctypes.c_void_p(self.stream.cuda_stream)
        ws_bytes = max(self.L.opsparse_spmv_csr_workspace_bytes(self.rows, self.nnz), 4 * n_y + 256)
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device=self.dev)

    def analyse(self, family):
        plan = self.osa.OpsparseSpmvPlan()
        rc = self.L.opsparse_spmv_csr_analyse(self.d_rp.data_ptr(), self.rows, self.cols, self.nnz,
                                              self.ws.data_ptr(), self.ws.numel(), family, ctypes.byref(plan), self.sp)
        assert rc == 0, "analyse rc=%d" % rc
        return plan

    def launch_and_check(self, plan, alpha, beta):
        osa = self.osa
        self.d_y.copy_(to_dev(self.y0, self.dev, self.out_dtype))
        sa = osa.OpsparseScalar(float(alpha), None, int(self.is_int), 0)
        sb = osa.OpsparseScalar(float(beta), None, int(self.is_int), 0)
        rc = self.L.opsparse_spmv_csr_launch(ctypes.byref(plan) if plan is not None else None, int(self.transpose),
                                             self.d_rp.data_ptr(), self.d_ci.data_ptr() or None,
                                             self.d_val.data_ptr() or None, self.d_x.data_ptr() or None,
                                             self.d_y.data_ptr(), self.rows, self.cols, self.nnz, sa, sb,
                                             _type_code(osa, self.val_dtype), _type_code(osa, self.out_dtype),
                                             int(self.is_int), self.ws.data_ptr(), self.ws.numel(), self.sp)
        assert rc == 0, "launch rc=%d" % rc
        self.stream.synchronize()
        y = self.d_y.cpu()
        y = y.numpy() if y.dtype == torch.int32 else y.float().numpy()
        _check_spmv(y, self.rows, self.cols, self.rowptr, self.colind, self.val, self.x, self.y0, alpha, beta,
                    self.out_dtype, self.transpose)


def _rows_up_to(longest, rows, seed):
    """Row lengths 0 .. longest with the longest present, a few empty rows, not a multiple of any tile."""
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, longest + 1, rows)
    lengths[[3, rows // 2, rows - 1]] = longest
    lengths[[0, 5, rows - 2]] = 0
    return lengths


# ---------------------------------------------------------------------------------------------- stream rows

# longest row -> lanes a row that the analysis picks for it
STREAM_LANES = [(12, 1), (24, 2), (48, 4), (96, 8), (192, 16), (384, 32), (512, 64)]


@pytest.mark.parametrize("types", list(SPMV_TYPES))
@pytest.mark.parametrize("longest,lanes", STREAM_LANES)
def test_stream_rows_every_lane_group_and_issue_depth(osa, gpu_ctx, types, longest, lanes):
    """SpmvStreamRowsKernel<ValT, OutT, AccT, G, U> for every type triple, G = 1 .. 64 lanes a row and U = 1, 2, 3
    rounds of loads a tile (tiles of up to 1024, 2048, 3072 products: the analysis sizes its tiles for two rounds,
    the tuning switch OPS_SPARSE_STREAM_ROWS and a caller's own plan reach the others); with one lane a row and fp32
    y also SpmvStreamQuadRowsKernel<ValT, AccT, U, guard> (rows a tile a multiple of four), tiles guarded and not."""
    rows, cols = 701, 900
    rowptr, colind, _ = csr_from_lengths(_rows_up_to(longest, rows, longest), cols, seed=longest)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=lanes)
    plan = m.analyse(osa.OPSPARSE_SPMV_STREAM_ROWS)
    assert plan.kernel == osa.OPSPARSE_SPMV_STREAM_ROWS and plan.lanesPerRow == lanes and plan.tileRowNnz == longest
    for depth in (1, 2, 3):
        per_tile = depth * 1024 // longest
        assert (depth - 1) * 1024 < per_tile * longest <= depth * 1024
        shapes = [(per_tile, 0)]
        if lanes == 1:
            # rows a tile not a multiple of four: the one-row-a-lane kernel; a multiple of four: four rows a lane
            shapes = [(per_tile - 1 + per_tile % 2, 0), (per_tile & ~3, 0), (per_tile & ~3, 1)]
        for rows_per_tile, guard in shapes:
            assert (depth - 1) * 1024 < rows_per_tile * longest <= depth * 1024
            plan.rowsPerBlock, plan.guardTiles = rows_per_tile, guard
            m.launch_and_check(plan, *((3, -2) if m.is_int else (1.25, 0.75)))


@pytest.mark.parametrize("types", list(SPMV_TYPES))
def test_vector_rows_every_lane_group(osa, gpu_ctx, types):
    """SpmvVectorRowsKernel<ValT, OutT, AccT, G>, G = 4 .. 64 lanes a row, for every type triple (the analysis picks
    G from the mean row length; any G is right for any matrix)."""
    rows, cols = 333, 2000
    rowptr, colind, _ = csr_from_lengths(_rows_up_to(300, rows, 7), cols, seed=8)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=9)
    plan = m.analyse(osa.OPSPARSE_SPMV_VECTOR_ROWS)
    assert plan.kernel == osa.OPSPARSE_SPMV_VECTOR_ROWS
    for lanes in (4, 8, 16, 32, 64):
        plan.lanesPerRow = lanes
        m.launch_and_check(plan, 3 if m.is_int else -0.5, -2 if m.is_int else 1.5)


@pytest.mark.parametrize("types", list(SPMV_TYPES))
def test_long_rows_beside_the_tiles_for_every_type(osa, gpu_ctx, types):
    """Short rows with a few long ones among them: the analysis sizes the stream-rows tiles for the short rows and
    leaves the long ones to SpmvLongRowsKernel<ValT, OutT, AccT>, a workgroup a row."""
    rows, cols = 5000, 9000
    lengths = _rows_up_to(10, rows, 3)
    lengths[[17, 4000]] = [700, 3000]
    rowptr, colind, _ = csr_from_lengths(lengths, cols, seed=4)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=5)
    plan = m.analyse(osa.OPSPARSE_SPMV_AUTO)
    assert plan.kernel == osa.OPSPARSE_SPMV_STREAM_ROWS and plan.longRowsBeside == 1 and plan.tileRowNnz == 10
    m.launch_and_check(plan, 2 if m.is_int else 1.5, 1 if m.is_int else 0.5)


@pytest.mark.parametrize("types", list(SPMV_TYPES))
def test_merge_path_and_scale_only_for_every_type(osa, gpu_ctx, types):
    """SpmvMergeKernel / SpmvMergeFixupKernel with the partition made by the analysis and, without a plan, by the
    launch; and a matrix without entries, which is y = beta y (SpmvScaleKernel<OutT, AccT>)."""
    rows, cols = 4000, 12_000
    lengths = np.random.default_rng(12).integers(0, 40, rows)
    lengths[77] = 9000
    rowptr, colind, _ = csr_from_lengths(lengths, cols, seed=13)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=14)
    plan = m.analyse(osa.OPSPARSE_SPMV_MERGE_PATH)
    assert plan.kernel == osa.OPSPARSE_SPMV_MERGE_PATH and plan.partitionReady == 1
    m.launch_and_check(plan, 1, 1)
    m.launch_and_check(None, 2, 0)
    empty = RawSpmv(osa, gpu_ctx, np.zeros(rows + 1, np.int32), np.zeros(0, np.int32), cols, types, seed=15)
    empty.launch_and_check(None, 1, 3 if empty.is_int else 0.5)


# ---------------------------------------------------------------------------------------------- op(A) = A^T

TRANSPOSE_TYPES = [t for t in SPMV_TYPES if t != "i32_i32"]


@pytest.mark.parametrize("types", TRANSPOSE_TYPES)
@pytest.mark.parametrize("mean,lanes", [(10, 4), (24, 8), (50, 16), (100, 32), (200, 64)])
def test_transposed_scatter_every_lane_group(osa, gpu_ctx, types, mean, lanes):
    """SpmvTransposeScatterKernel<ValT, AccT, G> (a lane group a row, G from the mean row length: 4 up to 16 entries,
    8 up to 32, ... 64 beyond 128) for every value type, y in fp32 or staged for a 16-bit y."""
    rows, cols = 8500, 40_000                # too many columns for y in LDS, too many rows for the split by entries
    rowptr, colind, _ = csr_from_lengths(np.full(rows, mean), cols, seed=mean)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=lanes, transpose=True)
    m.launch_and_check(None, 1.5, 0.5)


def test_transposed_scatter_every_lane_group_int32(osa, gpu_ctx):
    """op(A) = A^T in int32 arithmetic: SpmvTransposeScatterKernel<int32, int32, G, int32>, wrap-around sums."""
    L = osa.lib()
    dev, stream, _ = gpu_ctx
    for mean in (10, 24, 50, 100, 200):
        rows, cols = 600, 40_000
        rowptr, colind, _ = csr_from_lengths(np.full(rows, mean), cols, seed=mean)
        rng = np.random.default_rng(mean)
        val = rng.integers(-40_000, 40_000, colind.size).astype(np.int32)
        x = rng.integers(-40_000, 40_000, rows).astype(np.int32)
        y0 = rng.integers(-1000, 1000, cols).astype(np.int32)
        d = [to_dev(a, dev) for a in (rowptr, colind, val, x, y0)]
        sa, sb = osa.OpsparseScalar(3.0, None, 1, 0), osa.OpsparseScalar(-2.0, None, 1, 0)
        rc = L.opsparse_spmv_csr_launch(None, 1, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                        d[4].data_ptr(), rows, cols, colind.size, sa, sb, osa.OPSPARSE_I32,
                                        osa.OPSPARSE_I32, 1, None, 0, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0
        stream.synchronize()
        want = (y0.astype(np.int64) * -2)
        np.add.at(want, colind, 3 * val.astype(np.int64) * np.repeat(x, np.diff(rowptr)).astype(np.int64))
        assert np.array_equal(d[4].cpu().numpy(), want.astype(np.int32))   # (astype wraps like the device's sums)


@pytest.mark.parametrize("types", TRANSPOSE_TYPES)
def test_transposed_other_shapes_for_every_type(osa, gpu_ctx, types):
    """The other arms of the transposed product for every value type: few columns (y of a workgroup in LDS:
    SpmvTransposeNarrowKernel for up to 8192 and up to 16 384 columns), few long rows (SpmvTransposeFlatKernel: equal
    entries a workgroup), and rows far longer than the mean after an analysis (SpmvTransposeLongRowsKernel beside
    the lane groups)."""
    rng = np.random.default_rng(5)
    for rows, cols, per_row in ((9000, 5000, 8), (20_000, 12_000, 8)):      # nnz >= 8 cols and >= 32 768
        rowptr, colind, _ = csr_from_lengths(np.full(rows, per_row), cols, seed=cols)
        RawSpmv(osa, gpu_ctx, rowptr, colind, cols, types, seed=1, transpose=True).launch_and_check(None, 1.0, 0.5)
    rowptr, colind, _ = csr_from_lengths(rng.integers(1500, 2500, 12), 60_000, seed=6)   # 12 rows, 24 000 entries
    RawSpmv(osa, gpu_ctx, rowptr, colind, 60_000, types, seed=2, transpose=True).launch_and_check(None, -1.0, 0.0)
    lengths = rng.integers(0, 6, 20_000)
    lengths[[9, 10_000]] = [30_000, 700]
    rowptr, colind, _ = csr_from_lengths(lengths, 70_000, seed=7)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, 70_000, types, seed=3, transpose=True)
    plan = m.analyse(osa.OPSPARSE_SPMV_AUTO)
    assert plan.maxRowNnz == 30_000
    m.launch_and_check(plan, 0.5, 1.0)


# ---------------------------------------------------------------------------------------------- indexed rows

@pytest.mark.parametrize("wide_offsets", [False, True])
@pytest.mark.parametrize("mean", [10, 24, 50, 100, 200])
def test_indexed_rows_every_lane_group(osa, gpu_ctx, wide_offsets, mean):
    """SpmvIndexedRowsKernel<RowT, float, float, double, G>: 32- and 64-bit row offsets with index base 0 and 1, G
    from the mean row length (the kernel that aclsparseSpMVOp keeps for matrices beyond 2^31 - 1 entries; here on a
    small one through its own launch entry)."""
    L = osa.lib()
    dev, stream, _ = gpu_ctx
    rows, cols = 500, 3000
    lengths = np.random.default_rng(mean).integers(mean - 5, mean + 6, rows)
    lengths[[0, 250]] = 0
    lengths = lengths * mean * rows // lengths.sum()           # the mean row length decides the lane group
    lengths[1] += mean * rows - lengths.sum()
    rowptr, colind, val = csr_from_lengths(lengths, cols, seed=mean)
    assert rowptr[-1] // rows == mean
    rng = np.random.default_rng(mean + 1)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    for base in (0, 1):
        offs = (rowptr.astype(np.int64) if wide_offsets else rowptr) + base
        d = [to_dev(a, dev) for a in (offs, colind + base, val, x, y0)]
        d_z = torch.zeros(rows, dtype=torch.float32, device=dev)
        sa, sb = osa.OpsparseScalar(1.5, None, 0, 0), osa.OpsparseScalar(-0.5, None, 0, 0)
        rc = L.opsparse_spmv_csr_indexed_launch(d[0].data_ptr(), int(wide_offsets), base, d[1].data_ptr(),
                                                d[2].data_ptr(), d[3].data_ptr(), d[4].data_ptr(), d_z.data_ptr(),
                                                rows, cols, colind.size, sa, sb, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0
        stream.synchronize()
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, -0.5)
        assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5
        assert np.array_equal(d[4].cpu().numpy(), y0)          # y is read, z written


# ---------------------------------------------------------------------------------------------- SpMM

# name -> (dtype of values and B, dtype of C, elements of B a lane on the vector kernels)
SPMM_TYPES = {
    "f32": (torch.float32, torch.float32, 4),
    "f16_f16": (torch.float16, torch.float16, 8),
    "f16_f32": (torch.float16, torch.float32, 8),
    "i8_i32": (torch.int8, torch.int32, None),                 # 4 up to n = 32, 8 beyond
}


def _spmm_widths(types):
    """The widths of B that select each lane-group width L = 2 .. 64 of the vector kernels (n = L x elements a lane),
    and one that needs two column tiles."""
    v = SPMM_TYPES[types][2]
    if v is None:
        return [8, 16, 32, 64, 128, 256, 512, 1024]           # L = 2, 4, 8 at 4 bytes a lane; 8 .. 64 and two tiles at 8
    return [v * l for l in (2, 4, 8, 16, 32, 64, 128)]


class RawSpmm:
    def __init__(self, osa, gpu_ctx, types, m, k, n, lengths, seed, used_rows=None, ldb=None):
        """B has `k` rows; with `used_rows` only those rows of B are named by the matrix (and hold data): the oracle
        then works on the compact B of those rows."""
        self.osa, (self.dev, self.stream, _) = osa, gpu_ctx
        self.L = osa.lib()
        self.val_dtype, self.c_dtype, _ = SPMM_TYPES[types]
        self.is_int = self.val_dtype == torch.int8
        self.m, self.k, self.n = m, k, n
        rng = np.random.default_rng(seed)
        compact_k = k if used_rows is None else used_rows.size
        self.rowptr, self.colind, _ = csr_from_lengths(lengths, compact_k, seed=seed + 1)
        self.nnz = int(self.colind.size)
        if self.is_int:
            self.val = rng.integers(-128, 128, self.nnz).astype(np.int8)
            self.B = rng.integers(-128, 128, (compact_k, n)).astype(np.int8)
            self.C0 = rng.integers(-1000, 1000, (m, n)).astype(np.int32)
        else:
            self.val = _as_seen(rng.uniform(-1, 1, self.nnz), self.val_dtype)
            self.B = _as_seen(rng.uniform(-1, 1, (compact_k, n)), self.val_dtype)
            self.C0 = _as_seen(rng.uniform(-1, 1, (m, n)), self.c_dtype)
        self.ldb = n if ldb is None else ldb
        dev = self.dev
        self.d_rp = to_dev(self.rowptr, dev)
        device_cols = self.colind if used_rows is None else used_rows[self.colind].astype(np.int32)
        self.d_ci = to_dev(device_cols, dev)
        self.d_val = to_dev(self.val, dev, self.val_dtype)
        if used_rows is None and self.ldb == n:
            self.d_B = to_dev(self.B.ravel(), dev, self.val_dtype)
        else:
            self.d_B = torch.full((k * self.ldb,), 7, dtype=self.val_dtype, device=dev)
            where = slice(None) if used_rows is None else torch.from_numpy(used_rows).to(dev)
            self.d_B.view(k, self.ldb)[where, :n] = to_dev(self.B, dev, self.val_dtype)
        self.d_C = to_dev(self.C0.ravel(), dev, self.c_dtype)
        self.sp = ctypes.c_void_p(self.stream.cuda_stream)
        self.ws = None

    def analyse(self):
        size = ctypes.c_size_t(0)
        assert self.L.opsparse_spmm_csr_workspace_bytes(self.d_rp.data_ptr(), self.m, self.nnz, self.n, self.sp,
                                                        ctypes.byref(size)) == 0
        self.ws = torch.zeros(max(size.value, 256), dtype=torch.uint8, device=self.dev)
        plan = self.osa.OpsparseSpmmPlan()
        assert self.L.opsparse_spmm_csr_analyse(self.d_rp.data_ptr(), self.m, self.nnz, self.n, self.ws.data_ptr(),
                                                self.ws.numel(), 0, ctypes.byref(plan), self.sp) == 0
        self.stream.synchronize()
        return plan

    def launch_and_check(self, plan, alpha, beta, b_col_major=False, c_col_major=False):
        """Row-major operands as stored; with b_col_major / c_col_major the device copies are laid out that way."""
        osa, dev = self.osa, self.dev
        d_B, ldb, ldc = self.d_B, self.ldb, self.n
        if b_col_major:
            d_B, ldb = to_dev(np.ascontiguousarray(self.B.T).ravel(), dev, self.val_dtype), self.k
        C0 = self.C0.T if c_col_major else self.C0
        if c_col_major:
            ldc = self.m
        self.d_C = to_dev(np.ascontiguousarray(C0).ravel(), dev, self.c_dtype)
        sa = osa.OpsparseScalar(float(alpha), None, int(self.is_int), 0)
        sb = osa.OpsparseScalar(float(beta), None, int(self.is_int), 0)
        rc = self.L.opsparse_spmm_csr_launch(ctypes.byref(plan) if plan is not None else None, self.d_rp.data_ptr(),
                                             self.d_ci.data_ptr(), self.d_val.data_ptr(), d_B.data_ptr(),
                                             self.d_C.data_ptr(), self.m, self.k, self.n, self.nnz, ldb, ldc,
                                             int(b_col_major), int(c_col_major), 0, sa, sb,
                                             _type_code(osa, self.val_dtype), _type_code(osa, self.c_dtype),
                                             self.ws.data_ptr() if self.ws is not None else None,
                                             self.ws.numel() if self.ws is not None else 0, self.sp)
        assert rc == 0, "launch rc=%d" % rc
        self.stream.synchronize()
        got = self.d_C.cpu()
        got = got.numpy() if self.is_int else got.float().numpy()
        got = got.reshape(self.n, self.m).T if c_col_major else got.reshape(self.m, self.n)
        n, m = self.n, self.m
        if self.is_int:
            gold = oracle.spmm_i8(m, n, self.rowptr, self.colind, self.val, self.B.ravel(), n, self.C0.ravel(), n,
                                  int(alpha), int(beta), saturate=True).reshape(m, n)
            assert np.array_equal(got, gold)
            return
        gold = np.asarray(oracle.spmm_f64_rowmajor(m, n, self.rowptr, self.colind, self.val, self.B, n, self.C0, n,
                                                   alpha, beta)).reshape(m, n)
        if self.c_dtype == torch.float32:
            assert oracle.max_rel_err(got.ravel(), gold.ravel()) <= 1e-5
        else:
            want = _as_seen(gold, self.c_dtype)
            assert np.all(np.abs(got - want) <= ULP[self.c_dtype] * np.maximum(np.abs(want), 2.0 ** -14))


def _spmm_lengths(m, seed, long_rows=True):
    lengths = np.random.default_rng(seed).integers(0, 30, m)
    if long_rows:
        lengths[[7, m // 2]] = [3000, 2100]                   # beyond 2048 entries: cut into segments
    return lengths


@pytest.mark.parametrize("types", list(SPMM_TYPES))
def test_spmm_vector_kernels_every_lane_group_width(osa, gpu_ctx, types, monkeypatch):
    """For every type pair and every width L of lane group (n = L x elements a lane; the widest also with two column
    tiles): without a plan SpmmRowSplitKernel<ValT, CT, AccT, V, L>; with an analysed plan and rows beyond 2048
    entries SpmmSlabKernel<..., V, L, true> (slabs and segments in one launch) and SpmmLongFixupKernel<CT, AccT>;
    with the slab kernel switched off the same plan through SpmmRowSplitKernel and SpmmLongSegmentKernel<ValT, AccT,
    V, L>."""
    m, k = 1500, 5000
    for n in _spmm_widths(types):
        p = RawSpmm(osa, gpu_ctx, types, m, k, n, _spmm_lengths(m, n), seed=n)
        a, b = (3, -2) if p.is_int else (1.5, -0.5)
        p.launch_and_check(None, a, b)
        plan = p.analyse()
        assert plan.kernel == osa.OPSPARSE_SPMM_BINNED and plan.numLongRows == 2
        p.launch_and_check(plan, a, b)
        monkeypatch.setenv("OPS_SPARSE_SPMM_NO_SLAB", "1")
        p.launch_and_check(plan, a, b)
        monkeypatch.delenv("OPS_SPARSE_SPMM_NO_SLAB")
        short = RawSpmm(osa, gpu_ctx, types, m, k, n, _spmm_lengths(m, n, long_rows=False), seed=n + 1)
        plan = short.analyse()
        assert plan.numLongRows == 0
        short.launch_and_check(plan, a, 0)
        monkeypatch.setenv("OPS_SPARSE_SPMM_NO_SLAB_TABLE", "1")        # slabs of equal numbers of rows
        short.launch_and_check(plan, a, b)
        monkeypatch.delenv("OPS_SPARSE_SPMM_NO_SLAB_TABLE")


@pytest.mark.parametrize("types", list(SPMM_TYPES))
def test_spmm_general_kernel_every_lane_group_width(osa, gpu_ctx, types):
    """SpmmGeneralKernel<ValT, CT, AccT, L>, a lane a column of C, L = 4 .. 64 from n: what the launch layer runs for
    a width that is not whole vectors and for column-major operands (the aclsparse host re-stages those; a caller
    of the launch layer may pass them)."""
    m, k = 700, 900
    for n in (3, 7, 13, 27, 50):
        p = RawSpmm(osa, gpu_ctx, types, m, k, n, _spmm_lengths(m, n, long_rows=False), seed=n)
        a, b = (2, 1) if p.is_int else (0.5, 1.5)
        p.launch_and_check(None, a, b)
        p.launch_and_check(None, a, b, b_col_major=True)
        p.launch_and_check(None, a, b, c_col_major=True)
        p.launch_and_check(p.analyse(), a, b, b_col_major=True, c_col_major=True)


@pytest.mark.parametrize("types", list(SPMM_TYPES))
def test_spmm_slab_kernel_with_64_bit_gather_addresses_every_width(osa, gpu_ctx, types):
    """B spanning 4 GiB (2^20 rows, a leading dimension of 4 KiB) takes SpmmSlabKernel<..., V, L, false> for every
    L: the matrix names 4096 rows of B, the first and the last among them, and only those hold data."""
    m, k = 1200, 1 << 20
    elem = {torch.float32: 4, torch.float16: 2, torch.int8: 1}[SPMM_TYPES[types][0]]
    ldb = 4096 // elem
    rng = np.random.default_rng(3)
    used = np.unique(np.concatenate([[0, k - 1], rng.integers(0, k, 4094)])).astype(np.int64)
    for n in _spmm_widths(types):
        if n > ldb:
            continue
        p = RawSpmm(osa, gpu_ctx, types, m, k, n, _spmm_lengths(m, n), seed=n, used_rows=used, ldb=ldb)
        assert p.d_B.numel() * p.d_B.element_size() == 1 << 32
        plan = p.analyse()
        p.launch_and_check(plan, *((3, -2) if p.is_int else (1.5, -0.5)))
        del p
        torch.cuda.empty_cache()


NARROW_WIDTHS = {"f32": (4, 8), "f16_f16": (8, 16), "f16_f32": (8, 16)}      # one and two 16-byte pieces a row of B


@pytest.mark.parametrize("types", list(NARROW_WIDTHS))
@pytest.mark.parametrize("mean", [2, 6, 12, 25, 50, 100, 180])
def test_spmm_narrow_kernel_every_width_and_lane_group(osa, gpu_ctx, types, mean, monkeypatch):
    """SpmmNarrowKernel<ValT, CT, AccT, W, G> for a B of one or two 16-byte pieces a row under an analysed matrix of
    short rows.  Rows of exactly `mean` entries select the lanes of a group: with one fp32 piece 1, 2, 4, 8, 16, 32
    for means 2 .. 100; with two pieces the same from 6 .. 180; fp16 rows take twice the lanes, and 16 fp16
    columns 2 .. 32.  The number of entries is odd, so the last lanes of the last tile read their entries a few
    places early and move them; B and C have a padded leading dimension; beta is zero and not.  The same plan with
    the kernel switched off must agree as well (SpmmSlabKernel)."""
    m, k = 1201, 5000
    for n in NARROW_WIDTHS[types]:
        if n == 4 and mean == 180:
            continue                                                     # (a 32-lane group is at mean 100 there)
        lengths = np.full(m, mean)
        lengths[::7] = mean - 1 if mean > 2 else 0                       # some variety; the longest row stays `mean`
        if lengths.sum() % 4 == 0:
            lengths[1] -= 1
        p = RawSpmm(osa, gpu_ctx, types, m, k, n, lengths, seed=mean + n, ldb=n + 16)
        assert p.nnz % 4 != 0
        plan = p.analyse()
        assert plan.kernel != osa.OPSPARSE_SPMM_BINNED and plan.maxRowNnz == mean and plan.slabStartOff > 0
        p.launch_and_check(plan, 1.5, 0.0)
        p.launch_and_check(plan, 0.75, -0.5)
        monkeypatch.setenv("OPS_SPARSE_SPMM_NO_NARROW", "1")
        p.launch_and_check(plan, 0.75, -0.5)
        monkeypatch.delenv("OPS_SPARSE_SPMM_NO_NARROW")
        if types == "f32":
            # one column fewer, at leading dimensions that are not multiples of four: rows that are not whole
            # 16-byte pieces, read and written where they are (SpmmNarrowKernel<..., W, G, true>)
            r = RawSpmm(osa, gpu_ctx, types, m, k, n - 1, lengths, seed=mean + n + 1, ldb=n + 1)
            ragged = r.analyse()
            assert osa.lib().opsparse_spmm_csr_narrow_rows(ctypes.byref(ragged), r.ws.data_ptr(), n - 1, r.nnz,
                                                           _type_code(osa, r.val_dtype),
                                                           _type_code(osa, r.c_dtype)) == 1
            r.launch_and_check(ragged, 1.25, 0.0)
            r.launch_and_check(ragged, -0.5, 2.0)


def test_spmm_narrow_kernel_rows_of_no_or_one_entry(osa, gpu_ctx):
    """Rows of 0 or 1 entries: a tile holds two turns of the lanes (500 rows), and whole stretches of empty rows."""
    m, k = 20000, 3000
    rng = np.random.default_rng(5)
    lengths = rng.integers(0, 2, m)
    lengths[3000:6000] = 0
    lengths[9000:9600] = 1
    for types, n in (("f32", 4), ("f32", 8), ("f16_f32", 16)):
        p = RawSpmm(osa, gpu_ctx, types, m, k, n, lengths, seed=n)
        plan = p.analyse()
        assert plan.maxRowNnz == 1 and plan.slabStartOff > 0
        p.launch_and_check(plan, 2.0, 0.25)


def test_spmm_narrow_kernel_on_row_offsets_that_changed_since_the_analysis(osa, gpu_ctx):
    """The slab table is made for the row offsets Preprocess saw.  A caller of the launch layer who passes other
    offsets of the same rows and entries with that plan still gets the product: a tile that no longer fits the
    kernel's LDS is summed straight from memory."""
    m, k, n = 4000, 6000, 4
    even = np.full(m, 6)
    p = RawSpmm(osa, gpu_ctx, "f32", m, k, n, even, seed=3)
    plan = p.analyse()
    skew = even.copy()
    skew[:100] = 126                                                     # 100 x 120 more entries in front ...
    skew[100:2100] = 0                                                   # ... taken from the 2000 rows behind
    assert skew.sum() == even.sum()
    q = RawSpmm(osa, gpu_ctx, "f32", m, k, n, skew, seed=4)
    q.ws = p.ws
    q.launch_and_check(plan, 1.0, 0.5)


# ---------------------------------------------------------------------------------------------- blocked layouts

def _wide_matrix(rows, cols, seed, long_rows=(), per_row=20):
    rng = np.random.default_rng(seed)
    lengths = rng.integers(0, per_row, rows)
    for r, n in long_rows:
        lengths[r] = n
    rowptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    colind = rng.integers(0, cols, int(rowptr[-1])).astype(np.int32)
    for r, _ in long_rows:
        colind[rowptr[r]:rowptr[r + 1]].sort()                 # ascending columns: a long row
    return rowptr, colind


@pytest.mark.parametrize("int_compute", [True, False])
@pytest.mark.parametrize("streamed", [True, False])
def test_frozen_layout_with_int32_values(osa, gpu_ctx, int_compute, streamed, monkeypatch):
    """ACL_SPARSE_SPMV_CSR_ALG2 on int32 values and x over 1.4 M columns: the layout with the values frozen, streamed
    blocks (SpmvBlockStreamKernel<int32, OutT, AccT>, StreamScatterKernel<int32>) and windowed ones, long rows summed
    by phase 1 (SpmvBlockGatherKernel<true, int32, AccT>, SpmvLongRowSumKernel).  Integer compute type: int32 y,
    wrap-around sums, exact; ACL_FLOAT: fp32 y from fp64 sums of the exactly converted operands."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    if not streamed:
        monkeypatch.setenv("OPS_SPARSE_BLOCKED_NO_STREAM", "1")
    rows, cols = 300_000, 1_400_000
    rowptr, colind = _wide_matrix(rows, cols, 61, long_rows=[(5, 40_000), (100_000, 5_000), (100_001, 2_000)])
    nnz = colind.size
    rng = np.random.default_rng(62)
    big = 50_000 if int_compute else 2_000
    val = rng.integers(-big, big, nnz).astype(np.int32)
    x = rng.integers(-big, big, cols).astype(np.int32)
    y0 = rng.integers(-1000, 1000, rows).astype(np.int32) if int_compute else rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y),
                    compute_type=osa.ACL_INT32 if int_compute else osa.ACL_FLOAT, alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    assert op.buffer.numel() == L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz,
                                                                           osa.OPSPARSE_BLOCKED_VALUES_I32) > 0
    for alpha, beta in (((3, -2), (-1, 0)) if int_compute else ((0.5, 1.0), (1.0, 0.0))):
        d_y.copy_(torch.from_numpy(y0))
        op(alpha, beta)
        stream.synchronize()
        if int_compute:
            assert np.array_equal(d_y.cpu().numpy(), oracle.spmv_i32(rows, rowptr, colind, val, x, y0, alpha, beta))
        else:
            gold = oracle.spmv_f64(rows, cols, rowptr, colind, val.astype(np.float32), x.astype(np.float32), y0,
                                   alpha, beta)
            assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("narrow_y", [False, True])
def test_atomics_layout_with_32_bit_positions_and_16_bit_values(osa, gpu_ctx, dtype, narrow_y, monkeypatch):
    """The default plan's layout on fp16 / bf16 values with the positions of the entries kept in 32 bits
    (live_layout::SpmvBlockReduceKernel<true, false, ValT, OutT>; 16 bits are the rule, 32 what a row block of
    65 535 positions and more takes, asked for here by the switch)."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.setenv("OPS_SPARSE_BLOCKED_NO_SHORT_POSITIONS", "1")
    monkeypatch.delenv("OPS_SPARSE_SPMV_REPEATABLE", raising=False)
    rows, cols = 300_000, 1_400_000
    rowptr, colind = _wide_matrix(rows, cols, 71, long_rows=[(9, 30_000)])
    nnz = colind.size
    rng = np.random.default_rng(72)
    out_dtype = dtype if narrow_y else torch.float32
    val, x = _as_seen(rng.uniform(-1, 1, nnz), dtype), _as_seen(rng.uniform(-1, 1, cols), dtype)
    y0 = _as_seen(rng.uniform(-1, 1, rows), out_dtype)
    d = [to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev, dtype), to_dev(x, dev, dtype)]
    d_y = to_dev(y0, dev, out_dtype)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y))
    assert op.buffer.numel() == L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
    op(1.5, 0.5)
    stream.synchronize()
    _check_spmv(d_y.cpu().float().numpy(), rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5, out_dtype)


@pytest.mark.parametrize("dtype,narrow_y", [(torch.float32, False), (torch.float16, False), (torch.float16, True),
                                            (torch.bfloat16, False), (torch.bfloat16, True)])
def test_atomics_layout_with_many_long_rows_in_one_block(osa, gpu_ctx, dtype, narrow_y, monkeypatch):
    """200 neighbouring rows of 4200 .. 5000 ascending entries among short ones: more long rows than the workgroup
    of a row block adds up itself (64), so their partial sums are left to live_layout::SpmvLongRowSumKernel<OutT>,
    a wavefront a row."""
    dev, stream, handle = gpu_ctx
    L = osa.lib()
    monkeypatch.setenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ", "0")
    monkeypatch.delenv("OPS_SPARSE_SPMV_REPEATABLE", raising=False)
    rows, cols = 300_000, 1_400_000
    rng = np.random.default_rng(81)
    long_rows = [(5000 + i, int(n)) for i, n in enumerate(rng.integers(4200, 5000, 200))]
    rowptr, colind = _wide_matrix(rows, cols, 82, long_rows=long_rows)
    nnz = colind.size
    out_dtype = dtype if narrow_y else torch.float32
    val, x = _as_seen(rng.uniform(-1, 1, nnz), dtype), _as_seen(rng.uniform(-1, 1, cols), dtype)
    y0 = _as_seen(rng.uniform(-1, 1, rows), out_dtype)
    d = [to_dev(rowptr, dev), to_dev(colind, dev), to_dev(val, dev, dtype), to_dev(x, dev, dtype)]
    need = L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    plan = osa.OpsparseSpmvPlan()
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    flag = {torch.float32: 0, torch.float16: osa.OPSPARSE_BLOCKED_VALUES_F16,
            torch.bfloat16: osa.OPSPARSE_BLOCKED_VALUES_BF16}[dtype]
    assert L.opsparse_spmv_csr_live_analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, nnz, flag, pv(ws), need,
                                            ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream)) == 0
    assert plan.numLongRows == 200 and plan.numDeferredLongRows > 0
    del ws
    d_y = to_dev(y0, dev, out_dtype)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y))
    assert op.buffer.numel() == need
    op(-1.5, 0.75)
    stream.synchronize()
    _check_spmv(d_y.cpu().float().numpy(), rows, cols, rowptr, colind, val, x, y0, -1.5, 0.75, out_dtype)


@pytest.mark.parametrize("elem", [1, 2, 4])
def test_dense_restage_of_narrow_matrices_every_form(osa, gpu_ctx, elem):
    """opsparse_dense_restage to at most 32 columns: DenseRestageNarrowKernel<T, VecSrc, VecDst>, a lane a row.  A
    row-major side whose rows are whole aligned groups of four elements travels as vectors; the other forms are a
    column-major side, a leading dimension that is not a multiple of four, and a base that is not aligned.  Padding
    columns of the destination come out zero, what lies between its rows or columns stays."""
    dev, stream, _ = gpu_ctx
    L = osa.lib()
    sp = ctypes.c_void_p(stream.cuda_stream)
    np_t, t_t = {1: (np.uint8, torch.uint8), 2: (np.int16, torch.int16), 4: (np.int32, torch.int32)}[elem]
    rng = np.random.default_rng(elem)
    rows = 1000
    # (cols, colsDst, source: column-major / ld / offset in elements, destination: the same)
    forms = [(5, 8, (False, 8, 0), (False, 8, 0)),       # vectors on both sides
             (5, 8, (False, 8, 0), (True, rows + 3, 0)),  # vectors in, columns out
             (3, 4, (True, rows + 1, 0), (False, 4, 0)),  # columns in, vectors out
             (6, 7, (False, 9, 0), (False, 7, 0)),        # leading dimensions that are not multiples of four
             (4, 4, (False, 4, 1), (False, 4, 1)),        # bases one element off
             (1, 4, (True, rows, 0), (True, rows, 0)),    # columns on both sides
             (12, 12, (False, 12, 0), (True, rows, 0))]
    for cols, cols_dst, (s_cm, s_ld, s_off), (d_cm, d_ld, d_off) in forms:
        src = rng.integers(1, 100, s_off + (cols * s_ld if s_cm else rows * s_ld)).astype(np_t)
        dst0 = rng.integers(100, 120, d_off + (cols_dst * d_ld if d_cm else rows * d_ld)).astype(np_t)
        d_src, d_dst = to_dev(src, dev, t_t), to_dev(dst0, dev, t_t)
        rc = L.opsparse_dense_restage(d_src.data_ptr() + s_off * elem, d_dst.data_ptr() + d_off * elem, rows, cols,
                                      cols_dst, s_ld, int(s_cm), d_ld, int(d_cm), elem, sp)
        assert rc == 0
        stream.synchronize()
        r, c = np.meshgrid(np.arange(rows), np.arange(cols_dst), indexing="ij")
        logical = np.zeros((rows, cols_dst), np_t)
        logical[:, :cols] = src[s_off + (c[:, :cols] * s_ld + r[:, :cols] if s_cm else r[:, :cols] * s_ld + c[:, :cols])]
        want = dst0.copy()
        want[d_off + (c * d_ld + r if d_cm else r * d_ld + c)] = logical
        assert np.array_equal(d_dst.cpu().numpy(), want), (cols, cols_dst, s_cm, d_cm)


# ---------------------------------------------------------------------------------------------- yard-stick kernels

def test_measurement_kernels_copy_read_gather(osa, gpu_ctx):
    """The yard-stick kernels that the benchmark times beside the products (CopyKernel, ReadKernel, GatherKernel): the
    copy is exact, read and gather return without touching their inputs (a NULL sink is allowed), sizes that are not
    whole 16-byte pieces are refused."""
    L = osa.lib()
    dev, stream, _ = gpu_ctx
    sp = ctypes.c_void_p(stream.cuda_stream)
    n = (1 << 20) + 4                                             # not a multiple of the workgroup's share
    src = torch.arange(n, dtype=torch.int32, device=dev)
    dst = torch.zeros(n + 4, dtype=torch.int32, device=dev)
    assert L.opsparse_copy_launch(src.data_ptr(), dst.data_ptr(), 4 * n, sp) == 0
    assert L.opsparse_read_launch(src.data_ptr(), 4 * n, None, sp) == 0
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    x = torch.ones(1000, dtype=torch.float32, device=dev)
    idx = torch.from_numpy(np.random.default_rng(1).integers(-1, 1000, 100_000).astype(np.int32)).to(dev)
    assert L.opsparse_gather_launch(idx.data_ptr(), x.data_ptr(), idx.numel(), sink.data_ptr(), sp) == 0
    assert L.opsparse_gather_launch(idx.data_ptr(), x.data_ptr(), idx.numel(), None, sp) == 0
    stream.synchronize()
    assert bool((dst[:n] == src).all()) and bool((dst[n:] == 0).all())
    assert bool((src == torch.arange(n, dtype=torch.int32, device=dev)).all()) and bool((x == 1).all())
    assert L.opsparse_copy_launch(src.data_ptr(), dst.data_ptr(), 4 * n + 4, sp) != 0
    assert L.opsparse_read_launch(src.data_ptr(), 10, None, sp) != 0


# ---------------------------------------------------------------------------------------------- remaining host arms

def test_spmv_without_plan_or_workspace_runs_a_lane_group_a_row(osa, gpu_ctx):
    """No plan and no workspace: the merge path has nowhere to put its partition, so the launch takes
    SpmvVectorRowsKernel with the lane group that the mean row length asks for; a NULL yIn of the z / y entry point
    means y is read in place."""
    L = osa.lib()
    dev, stream, _ = gpu_ctx
    rows, cols = 3000, 5000
    rowptr, colind, val = csr_from_lengths(np.random.default_rng(2).integers(0, 60, rows), cols, seed=3)
    rng = np.random.default_rng(4)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x, y0)]
    sa, sb = osa.OpsparseScalar(2.0, None, 0, 0), osa.OpsparseScalar(0.5, None, 0, 0)
    rc = L.opsparse_spmv_csr_launch_zy(None, 0, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                       None, d[4].data_ptr(), rows, cols, colind.size, sa, sb, osa.OPSPARSE_F32,
                                       osa.OPSPARSE_F32, 0, None, 0, ctypes.c_void_p(stream.cuda_stream))
    assert rc == 0
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 2.0, 0.5)
    assert oracle.max_rel_err(d[4].cpu().numpy(), gold) <= 1e-5
    # the indexed entry point reads z in place when yIn is NULL
    d_z = to_dev(y0, dev)
    rc = L.opsparse_spmv_csr_indexed_launch(d[0].data_ptr(), 0, 0, d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                            None, d_z.data_ptr(), rows, cols, colind.size, sa, sb,
                                            ctypes.c_void_p(stream.cuda_stream))
    assert rc == 0
    stream.synchronize()
    assert oracle.max_rel_err(d_z.cpu().numpy(), gold) <= 1e-5


def test_stream_rows_tile_height_override(osa, gpu_ctx, monkeypatch):
    """OPS_SPARSE_STREAM_ROWS sets the rows of a stream-rows tile at the analysis (a tuning switch, read there); a
    value whose products would not fit the tile's 3072 slots is ignored."""
    lengths = np.random.default_rng(1).integers(26, 31, 5000)     # nearly even rows: the analysis' own choice
    lengths[[3, 77]] = [30, 0]
    rowptr, colind, _ = csr_from_lengths(lengths, 4000, seed=2)
    m = RawSpmv(osa, gpu_ctx, rowptr, colind, 4000, "f32", seed=3)
    ordinary = m.analyse(osa.OPSPARSE_SPMV_AUTO).rowsPerBlock
    assert ordinary == 2048 // 30 // 4 * 4
    monkeypatch.setenv("OPS_SPARSE_STREAM_ROWS", "50")
    plan = m.analyse(osa.OPSPARSE_SPMV_AUTO)
    assert plan.kernel == osa.OPSPARSE_SPMV_STREAM_ROWS and plan.rowsPerBlock == 50
    m.launch_and_check(plan, 1.0, 0.0)
    monkeypatch.setenv("OPS_SPARSE_STREAM_ROWS", "200")            # 200 x 30 > 3072
    assert m.analyse(osa.OPSPARSE_SPMV_AUTO).rowsPerBlock == ordinary


def test_frozen_windowed_layout_without_long_rows(osa, gpu_ctx, monkeypatch):
    """ACL_SPARSE_SPMV_CSR_ALG2 with the streamed blocks and the long rows' way both switched off: the windowed blocks
    on frozen values with every entry in the row-block order, the row offsets copied into the buffer (a plan with
    frozen values reads nothing of the caller's arrays at the launches)."""
    dev, stream, handle = gpu_ctx
    monkeypatch.setenv("OPS_SPARSE_BLOCKED_NO_STREAM", "1")
    monkeypatch.setenv("OPS_SPARSE_BLOCKED_NO_LONG_ROWS", "1")
    rows, cols = 300_000, 1_400_000
    rowptr, colind = _wide_matrix(rows, cols, 91, long_rows=[(7, 20_000)])
    rng = np.random.default_rng(92)
    val = rng.uniform(-1, 1, colind.size).astype(np.float32)
    x, y0 = rng.uniform(-1, 1, cols).astype(np.float32), rng.uniform(-1, 1, rows).astype(np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val, x)]
    d_y = to_dev(y0, dev)
    op = osa.SpmvOp(handle, osa.Csr(rows, cols, d[0], d[1], d[2]), osa.DnVec(d[3]), osa.DnVec(d_y),
                    alg=osa.ACL_SPARSE_SPMV_CSR_ALG2)
    assert op.buffer.numel() == osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, 0) > 0
    d[0].zero_()                                               # the plan must not look at the caller's offsets again
    op(1.5, 0.5)
    stream.synchronize()
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, 1.5, 0.5)
    assert oracle.max_rel_err(d_y.cpu().numpy(), gold) <= 1e-5


def test_spmm_analysis_switches_and_small_workspace(osa, gpu_ctx, monkeypatch):
    """The remaining arms of the SpMM analysis: OPS_SPARSE_SPMM_NO_BINNING (no row is cut into segments: rows beyond
    the slab kernel's staging area then go to a lane group a row), OPS_SPARSE_SPMM_SLAB_ENTRIES (slabs of another
    length), and a workspace of 256 bytes for a matrix without long rows (no slab table: slabs of equal numbers of
    rows)."""
    m, k, n = 1500, 5000, 64
    p = RawSpmm(osa, gpu_ctx, "f32", m, k, n, _spmm_lengths(m, 5), seed=5)
    monkeypatch.setenv("OPS_SPARSE_SPMM_NO_BINNING", "1")
    plan = p.analyse()
    assert plan.numLongRows == 0 and plan.maxRowNnz == 3000
    p.launch_and_check(plan, 1.5, -0.5)
    monkeypatch.delenv("OPS_SPARSE_SPMM_NO_BINNING")
    monkeypatch.setenv("OPS_SPARSE_SPMM_SLAB_ENTRIES", "512")
    p.launch_and_check(p.analyse(), 1.5, -0.5)
    monkeypatch.delenv("OPS_SPARSE_SPMM_SLAB_ENTRIES")
    short = RawSpmm(osa, gpu_ctx, "f32", 40_000, k, n, _spmm_lengths(40_000, 6, long_rows=False), seed=6)
    short.ws = torch.zeros(256, dtype=torch.uint8, device=short.dev)
    plan = osa.OpsparseSpmmPlan()
    assert short.L.opsparse_spmm_csr_analyse(short.d_rp.data_ptr(), short.m, short.nnz, n, short.ws.data_ptr(), 256, 0,
                                             ctypes.byref(plan), short.sp) == 0
    assert plan.numSlabs == 0 and plan.bytes == 256
    short.launch_and_check(plan, 1.0, 0.0)


@pytest.mark.parametrize("which", ["frozen_transposed", "live_transposed", "atomics"])
def test_layout_analyses_refuse_a_column_out_of_range(osa, gpu_ctx, which):
    """Every layout analysis checks the column indices against cols before it indexes anything with them: the
    transposed layouts before they transpose, the atomics layout with its panel keys."""
    dev, stream, _ = gpu_ctx
    L = osa.lib()
    transposed = which != "atomics"
    rows, cols = (1_400_000, 300_000) if transposed else (300_000, 1_400_000)
    rowptr, colind = _wide_matrix(rows, cols, 95, per_row=5 if transposed else 20)
    colind[colind.size // 3] = cols
    val = np.ones(colind.size, np.float32)
    d = [to_dev(a, dev) for a in (rowptr, colind, val)]
    pv = lambda t: ctypes.c_void_p(t.data_ptr())
    plan = osa.OpsparseSpmvPlan()
    if which == "atomics":
        need = L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, colind.size)
        analyse, flags = L.opsparse_spmv_csr_live_analyse, 0
    else:
        flags = osa.OPSPARSE_BLOCKED_TRANSPOSE | (osa.OPSPARSE_BLOCKED_LIVE_VALUES if which == "live_transposed" else 0)
        need = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, colind.size, flags)
        analyse = L.opsparse_spmv_csr_blocked_analyse
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    rc = analyse(pv(d[0]), pv(d[1]), pv(d[2]), rows, cols, colind.size, flags, pv(ws), need, ctypes.byref(plan),
                 ctypes.c_void_p(stream.cuda_stream))
    assert rc == osa.OPSPARSE_E_INVALID
