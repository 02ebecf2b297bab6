/*
 * Thin C-ABI launch layer between the aclsparse host code and the HIP kernels
 * for gfx950.  Plain pointers and sizes only: this is the seam a foreign-
 * language binding (ctypes, cgo, JNI) or another host library would call when
 * it has its own descriptor handling and just wants the kernels.
 *
 * It plays the role the reference gives to its `extern "C"` kernel launchers:
 *   spmv_kernel_do      [ref: sparse/spmv/arch22/spmv_host.cpp:29-34,
 *                             sparse/spmv/arch22/kernels/spmv_kernel.cpp:21-55]
 *   spmm_kernel_launch  [ref: sparse/spmm/arch35/spmm_host.cpp:29-33,
 *                             sparse/spmm/arch35/spmm_kernel.cpp:447-477]
 * i.e. raw device pointers + sizes + scalars + a workspace + a stream, no
 * descriptor objects, no validation beyond what keeps a launch in bounds.
 *
 * All functions return 0 on success or a negative OPSPARSE_E_* code; nothing
 * is printed.  `stream` is a hipStream_t passed as void*.  Unless stated
 * otherwise a function only enqueues work and does not synchronise.
 */
#ifndef OPS_SPARSE_HIP_H_
#define OPS_SPARSE_HIP_H_

#include <stddef.h>
#include <stdint.h>

/* The enums of this ABI are passed by value and checked by the callee: a caller may hand over any int.  C++ leaves a
 * value outside an enum's enumerators undefined unless the enum has a fixed underlying type, so under C++ they get
 * one (int, what they are in C anyway: neither size nor calling convention changes). */
#ifndef OPSPARSE_ABI_ENUM
#ifdef __cplusplus
#define OPSPARSE_ABI_ENUM(name) enum name : int
#else
#define OPSPARSE_ABI_ENUM(name) enum name
#endif
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define OPSPARSE_OK 0
#define OPSPARSE_E_INVALID (-1)     /* bad argument (null pointer, negative size, unknown enum) */
#define OPSPARSE_E_UNSUPPORTED (-2) /* type / layout combination without a kernel */
#define OPSPARSE_E_WORKSPACE (-3)   /* workspace missing or too small */
#define OPSPARSE_E_LAUNCH (-4)      /* the HIP runtime reported an error */

/* Element types of device arrays. */
typedef OPSPARSE_ABI_ENUM(OpsparseDtype) {
    OPSPARSE_F32 = 0,
    OPSPARSE_F16 = 1,
    OPSPARSE_BF16 = 2,
    OPSPARSE_I32 = 3,
    OPSPARSE_I8 = 4
} OpsparseDtype;

/* alpha or beta.  devicePtr == NULL: `value` is used.  Otherwise the kernel
 * reads a float (isInt == 0) or an int32 (isInt != 0) from devicePtr. */
typedef struct OpsparseScalar {
    double value;
    const void *devicePtr;
    int32_t isInt;
    int32_t reserved;
} OpsparseScalar;

/* ------------------------------------------------------------------ SpMV */

/* Kernel families of the row-length-binned SpMV dispatcher. */
typedef OPSPARSE_ABI_ENUM(OpsparseSpmvKernel) {
    OPSPARSE_SPMV_AUTO = 0,        /* let the library pick from the statistics */
    OPSPARSE_SPMV_SCALE_ONLY = 1,  /* nnz == 0: y = beta * y */
    OPSPARSE_SPMV_STREAM_ROWS = 2, /* short rows: fixed row blocks, products staged in LDS,
                                      one or a few lanes per row */
    OPSPARSE_SPMV_VECTOR_ROWS = 3, /* medium rows: a 4..64-lane group per row, shuffle reduction */
    OPSPARSE_SPMV_MERGE_PATH = 4,  /* skewed rows: equal (rows + nnz) per workgroup, carry-out fix-up */
    OPSPARSE_SPMV_COLUMN_PANELS = 5,/* x larger than an L2: the matrix re-stored as panels of 2^20 columns, each
                                      worked on one XCD so that its slice of x stays in that L2; fp32 only; holds a
                                      copy of the VALUES as they were at analysis time */
    OPSPARSE_SPMV_BLOCKED_GATHER = 6,/* x larger than an L2: two passes.  The entries' columns re-stored by panels of
                                      2^15 columns, x gathered from LDS into a linear stream; then row blocks whose
                                      gathered x is put back into row order in LDS and summed against the values,
                                      read in place, in an order that the layout fixes: the same bits at every
                                      call.  16 bytes of traffic per entry and no line-sized gathers; fp32 / fp16 /
                                      bf16 / int32, op(A) = A or (on a transposed copy) A^T */
    OPSPARSE_SPMV_BLOCKED_LIVE = 7, /* the same two passes with the second one built for speed: it collects a row
                                      block's values in LDS, streams the block's entries panel by panel against
                                      them and adds into one fp64 accumulator a row with LDS atomics, in the order
                                      the wavefronts get there: the last bit of a result may differ between two
                                      calls.  The plan of aclsparseSpMVPreprocess under ACL_SPARSE_SPMV_ALG_DEFAULT,
                                      whose results the reference lets vary; fp32 / fp16 / bf16, op(A) = A, values
                                      read where the caller has them at every call */
    OPSPARSE_SPMV_SCATTER_LIVE = 8  /* op(A) = A^T with y larger than an L2, the mirror image: pieces of the caller's
                                      arrays multiplied by x[row] and written out sorted by output panel (2^14
                                      columns) through LDS, then a workgroup a panel adds the products, kept exactly,
                                      into fp64 sums in LDS with atomics.  26 bytes of traffic per entry, none on y;
                                      fp32 / fp16 / bf16, values read where the caller has them; like the reference's
                                      transposed kernel the last bit of a result may differ between two calls */
} OpsparseSpmvKernel;

#define OPSPARSE_SPMV_MAX_PANELS 16

/* Result of analysing one CSR matrix; plain data, safe to copy. */
typedef struct OpsparseSpmvPlan {
    int32_t kernel;        /* OpsparseSpmvKernel actually chosen */
    int32_t lanesPerRow;   /* VECTOR_ROWS / STREAM_ROWS: lanes cooperating on one row */
    int32_t rowsPerBlock;  /* STREAM_ROWS: rows owned by one workgroup */
    int32_t mergeBlocks;   /* MERGE_PATH: number of workgroups == partition entries - 1 */
    int32_t maxRowNnz;     /* longest row */
    int32_t partitionReady;/* MERGE_PATH: partition table already in the workspace */
    int32_t numPanels;     /* COLUMN_PANELS / BLOCKED_GATHER: number of column panels */
    int32_t panelShift;    /* COLUMN_PANELS / BLOCKED_GATHER: log2 of the panel width */
    int32_t numRowBlocks;  /* BLOCKED_GATHER: number of row blocks */
    int32_t entryWindow;   /* BLOCKED_GATHER: a row block also ends where the entry count passes a multiple of this */
    int32_t transposed;    /* BLOCKED_GATHER: the layout was built for op(A) = A^T and serves only that */
    int32_t guardTiles;    /* STREAM_ROWS: the row offsets may have changed since the analysis: a tile with more
                              entries than its LDS was sized for is summed from memory instead (set by callers
                              that keep a plan without the user having asked for one; 0 after analyse) */
    int32_t tileRowNnz;    /* STREAM_ROWS: the row length the tiles are sized for (0: maxRowNnz) */
    int32_t longRowsBeside;/* STREAM_ROWS: a few rows are longer than that: the tiles skip rows of more than 64
                              entries and a second kernel sums those, a workgroup per row */
    int32_t liveValues;    /* BLOCKED_GATHER / BLOCKED_LIVE: the layout holds no values; every launch takes the caller's
                              csrValues as they are then: nothing goes stale when values change in place or the
                              values pointer is replaced (BLOCKED_LIVE: 1: 32-bit positions of the entries, 2: 16-bit
                              ones relative to their row block, where every block is shorter than 65535) */
    int32_t numLongRows;   /* BLOCKED_GATHER: rows kept out of the re-stored layout: phase 1 sums them from the caller's
                              colInd / csrValues, panel by panel, with the panel's x in LDS */
    int32_t numDeferredLongRows; /* BLOCKED_GATHER: those of them that sit more than 64 to a row block: a third kernel,
                              a wavefront a row, adds their partial sums up instead of the block's workgroup */
    int32_t valueType;     /* BLOCKED_GATHER: the OPSPARSE_F32 / F16 / BF16 / I32 the layout was built from; launches
                              must bring values and x of that type (y: fp32, or that type) */
    int32_t numEmptyRows;  /* BLOCKED_GATHER: rows without entries; a small kernel of their own writes beta * y there */
    int32_t streamedBlocks;/* BLOCKED_GATHER: 1: the layout keeps the values, in (block, panel) order, and a wavefront
                              streams a run of row blocks; 0: values read in row order through a window in LDS */
    int32_t reserved0;
    int64_t rows;
    int64_t nnz;
    int64_t partOff;       /* byte offsets into the workspace */
    int64_t carryOff;
    int64_t headOff;
    int64_t bytes;         /* workspace bytes this plan uses */
    int64_t panelStart[OPSPARSE_SPMV_MAX_PANELS + 1]; /* COLUMN_PANELS: first entry of every panel */
} OpsparseSpmvPlan;

/* Bytes opsparse_spmv_csr_analyse / _launch may touch in `workspace`. */
size_t opsparse_spmv_csr_workspace_bytes(int64_t rows, int64_t nnz);

/*
 * Row-length statistics -> kernel choice (+ merge-path partition written to
 * `workspace`).  Synchronises `stream` once to read the statistics back.
 * `forceKernel` != AUTO overrides the choice (tuning, tests).
 */
int opsparse_spmv_csr_analyse(const int32_t *rowOffsets, int64_t rows, int64_t cols, int64_t nnz,
                              void *workspace, size_t workspaceBytes, int32_t forceKernel,
                              OpsparseSpmvPlan *plan, void *stream);

/*
 * y = alpha * A * x + beta * y (transpose == 0) or y = alpha * A^T * x + beta * y.
 * valType is the element type of csrValues and x, outType of y.
 * plan == NULL: no prior analysis; the merge-path family is used with the
 * partition rebuilt into `workspace` by a small kernel, or, when `workspace`
 * is too small, a workspace-free VECTOR_ROWS launch sized from nnz / rows.
 */
int opsparse_spmv_csr_launch(const OpsparseSpmvPlan *plan, int32_t transpose, const int32_t *rowOffsets,
                             const int32_t *colInd, const void *csrValues, const void *x, void *y, int64_t rows,
                             int64_t cols, int64_t nnz, OpsparseScalar alpha, OpsparseScalar beta, int32_t valType,
                             int32_t outType, int32_t computeIsInt, void *workspace, size_t workspaceBytes,
                             void *stream);

/*
 * How scattered are the gathers of x?  Samples up to 65 536 rows (32 entries each); *scattered = how many sampled
 * columns in a thousand lie further than 2^17 columns from where their row sits on the diagonal.  A banded or
 * mesh-like matrix keeps x in cache under the row-wise kernels, which then cost about 1.2 us per million entries
 * plus 13 us per million gathers that miss; the re-stored layouts cost 3.6 us (values frozen) and 5.2 us (live
 * values) per million entries whatever the columns, and pay from 190 and 310 in a thousand on.  `workspace` needs
 * 256 bytes.  Synchronises `stream` once.
 * No counterpart in the reference, whose ALG2 preprocessing (sparse/spmv_op/arch35/spmv_op_host.cpp:543-573)
 * reorders every matrix alike; here it is one of the questions that preprocessing asks.
 */
int opsparse_spmv_csr_gathers_scattered(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols,
                                        int64_t nnz, void *workspace, size_t workspaceBytes, int32_t *scattered,
                                        void *stream);

/*
 * COLUMN_PANELS analysis (fp32, op(A) = A): bytes of the workspace, or 0 when the
 * family does not apply (it needs 2..16 panels of 2^20 columns, i.e. 1 M < cols <= 16 M).
 * The analysis re-stores the matrix — column indices AND values — in the
 * workspace, panel by panel; launches with the resulting plan read that copy and
 * ignore the rowOffsets / colInd / csrValues arguments, so the analysis must be
 * repeated after the values change.  Synchronises `stream` once.
 */
size_t opsparse_spmv_csr_panels_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz);
int opsparse_spmv_csr_panels_analyse(const int32_t *rowOffsets, const int32_t *colInd, const float *csrValues,
                                     int64_t rows, int64_t cols, int64_t nnz, void *workspace, size_t workspaceBytes,
                                     OpsparseSpmvPlan *plan, void *stream);

/*
 * BLOCKED_GATHER analysis: bytes of the workspace, or 0 when the family does not apply (x must have more than 2^18
 * and at most 2^25 elements, the matrix at least two million entries, and a (panel, row block) chunk at least 8
 * entries on average).  Values and x are fp32, fp16, bf16 or int32 (`flags`); at the launches y is fp32 or of the
 * values' own type, int32 under the integer compute type.
 * The layout holds where the entries' columns sit in 2^15-column panels, the place of every entry in its row block,
 * and small tables by which a block's kernel tells its rows apart.  Every row is summed in an order that the layout
 * fixes (fp64 for floating-point data, rounded once; 32-bit wrap-around for the integer compute type): two launches
 * on the same data give the same bits.
 * `flags`:
 *   OPSPARSE_BLOCKED_LIVE_VALUES  no value is kept: every launch reads csrValues (and, for long rows, colInd) where
 *       the caller has them; rowOffsets / colInd must be the arrays of the analysis, the values may change.  Without
 *       it (values frozen) the analysis keeps a copy of the values, launches ignore the rowOffsets / colInd /
 *       csrValues arguments, and the analysis must be repeated after the values change; rows of 1024 entries and more
 *       are then stored a second time panel by panel, which halves what they cost.  Frozen values are kept in the
 *       order the second kernel streams them (plan->streamedBlocks = 1: row blocks of 2^10 rows, a wavefront
 *       each) where a (panel, block) chunk then still holds 16 entries and a row at most 16 a panel on average;
 *       else, like live values, they are read in row order through a window in LDS by a workgroup a block of 2^12
 *       rows (which cannot hold a row of more than 65 534 entries: see OPSPARSE_E_UNSUPPORTED below).
 *   OPSPARSE_BLOCKED_TRANSPOSE (= 1, so that a plain 0 / 1 "transpose" still reads right)  the layout of
 *       y = alpha * A^T * x + beta * y: the analysis transposes the matrix into the workspace (the CSC arrays of A
 *       are the CSR arrays of A^T) and builds the layout of that copy; no atomics on y.  With live values it keeps
 *       the entry of A behind every entry of the copy, and a launch first refreshes the copy's values from
 *       csrValues.  A plan serves the op(A) it was built for.
 *   OPSPARSE_BLOCKED_VALUES_F16 / _BF16 / _I32  the type of csrValues and x (default fp32).
 * Rows with many entries in every column panel and ascending columns ("long rows", plan->numLongRows of them) are
 * summed by the first kernel instead of going through the row blocks.  Returns OPSPARSE_E_INVALID for a column
 * index outside [0, cols), OPSPARSE_E_UNSUPPORTED for a matrix with a row of more than 65 534 entries that cannot
 * go the long rows' way (its columns do not ascend) where the blocks are the windowed ones.  Synchronises `stream`
 * twice (three times for op(A) = A^T) and allocates nothing.  Launches touch only the first opsparse_spmv_csr_blocked_resident_bytes() of the workspace; the rest
 * serves the analysis and may be handed back afterwards.
 */
#define OPSPARSE_BLOCKED_TRANSPOSE 1
#define OPSPARSE_BLOCKED_LIVE_VALUES 2
#define OPSPARSE_BLOCKED_VALUES_F16 4
#define OPSPARSE_BLOCKED_VALUES_BF16 8
#define OPSPARSE_BLOCKED_VALUES_I32 16
size_t opsparse_spmv_csr_blocked_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags);
size_t opsparse_spmv_csr_blocked_resident_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags);
int opsparse_spmv_csr_blocked_analyse(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                      int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                      size_t workspaceBytes, OpsparseSpmvPlan *plan, void *stream);
/* The same with the two parts of the workspace apart: `workspace` (opsparse_spmv_csr_blocked_resident_bytes()) is
 * what the launches keep, `scratchSpace` (the rest of opsparse_spmv_csr_blocked_workspace_bytes()) serves the analysis
 * only and is free again when the call returns. */
int opsparse_spmv_csr_blocked_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                            int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                            size_t workspaceBytes, void *scratchSpace, size_t scratchBytes,
                                            OpsparseSpmvPlan *plan, void *stream);

/*
 * BLOCKED_LIVE analysis (fp32, fp16 or bf16 values and x, op(A) = A, values read in place at every launch): the
 * layout of the plan kernel OPSPARSE_SPMV_BLOCKED_LIVE, whose second kernel adds into LDS with atomics in the order
 * the wavefronts get there — the fastest plan for a matrix with scattered columns whose values change between
 * calls, for callers who do not need the last bit of a result to repeat.  Same applicability bounds as BLOCKED_GATHER
 * except that a chunk needs 8 entries on average; `flags`: OPSPARSE_BLOCKED_VALUES_F16 / _BF16 only.  Synchronises
 * `stream` twice.  No counterpart in the reference.
 */
size_t opsparse_spmv_csr_live_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz);
size_t opsparse_spmv_csr_live_resident_bytes(int64_t rows, int64_t cols, int64_t nnz);
int opsparse_spmv_csr_live_analyse(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                   int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                   size_t workspaceBytes, OpsparseSpmvPlan *plan, void *stream);
int opsparse_spmv_csr_live_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                         int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                         size_t workspaceBytes, void *scratchSpace, size_t scratchBytes,
                                         OpsparseSpmvPlan *plan, void *stream);

/*
 * SCATTER_LIVE analysis (op(A) = A^T; fp32, fp16 or bf16 values and x, values read in place at every launch): the
 * layout of the plan kernel OPSPARSE_SPMV_SCATTER_LIVE.  Takes the place of the atomics on y of the reference's
 * transposed kernel (sparse/spmv/arch22/kernels/spmv_kernel.cpp:21-55).  It looks at the structure only: no value is
 * read or kept.  Applies from 128 output panels of 2^14 columns on (more than 2 M columns) up to 2^25 columns;
 * OPSPARSE_E_UNSUPPORTED also for a column with more than 8192 entries (all its products would queue for one
 * address of LDS) and for a piece (16 384 consecutive entries of fp32 values, 32 768 of 16-bit ones) that spans more
 * than 65 535 rows: the ordered layout
 * over a transposed copy (opsparse_spmv_csr_blocked_analyse with OPSPARSE_BLOCKED_TRANSPOSE) serves those.
 * OPSPARSE_E_INVALID for a column index outside [0, cols).  `flags`: OPSPARSE_BLOCKED_VALUES_F16 / _BF16 only.
 * Synchronises `stream` twice.  The launch is opsparse_spmv_csr_launch with transpose != 0 and the workspace.
 */
size_t opsparse_spmv_csr_scatter_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags);
size_t opsparse_spmv_csr_scatter_resident_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags);
int opsparse_spmv_csr_scatter_analyse(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols,
                                      int64_t nnz, int32_t flags, void *workspace, size_t workspaceBytes,
                                      OpsparseSpmvPlan *plan, void *stream);
int opsparse_spmv_csr_scatter_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols,
                                            int64_t nnz, int32_t flags, void *workspace, size_t workspaceBytes,
                                            void *scratchSpace, size_t scratchBytes, OpsparseSpmvPlan *plan,
                                            void *stream);

/* Same as opsparse_spmv_csr_launch with separate input and output vectors:
 * z = alpha * op(A) * x + beta * yIn.  z may be yIn (in place); yIn is only read
 * when beta != 0 and may then be NULL otherwise. */
int opsparse_spmv_csr_launch_zy(const OpsparseSpmvPlan *plan, int32_t transpose, const int32_t *rowOffsets,
                                const int32_t *colInd, const void *csrValues, const void *x, const void *yIn, void *z,
                                int64_t rows, int64_t cols, int64_t nnz, OpsparseScalar alpha, OpsparseScalar beta,
                                int32_t valType, int32_t outType, int32_t computeIsInt, void *workspace,
                                size_t workspaceBytes, void *stream);

/*
 * opsparse_spmv_csr_launch with plan == NULL for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): y = alpha * A * x + beta * y by the merge-path
 * kernels, whose partition, carries and heads live in a 4 MiB array that is part of the library's device image
 * (one copy per GPU, held until the process ends) instead of a caller's workspace.  No counterpart in the
 * reference.  Calls no hipMalloc / hipFree and no allocating library routine; the first call on a device looks
 * the array's address up (hipGetSymbolAddress), so make that call outside a capture.
 * Limit: opsparse_spmv_csr_workspace_bytes(rows, nnz) <= opsparse_spmv_csr_noalloc_max_bytes() (4 MiB: rows + nnz
 * up to about 4.2e8); beyond it the call returns OPSPARSE_E_WORKSPACE and launches nothing.
 * All calls on one GPU share the array: calls that overlap there (two streams, two threads) race; calls on one
 * stream are ordered and safe.  Same types, scalars and result as opsparse_spmv_csr_launch.
 */
size_t opsparse_spmv_csr_noalloc_max_bytes(void);
int opsparse_spmv_csr_launch_noalloc(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                     const void *x, void *y, int64_t rows, int64_t cols, int64_t nnz,
                                     OpsparseScalar alpha, OpsparseScalar beta, int32_t valType, int32_t outType,
                                     int32_t computeIsInt, void *stream);

/* out[i] = offsets[i] - indexBase as int32, i < count: 64-bit and / or one-based row offsets turned into what the
 * kernels above take.  With one-based column indices left as they are, a caller then passes x - 1 for x and
 * cols + 1 for cols: x[col - 1] is (x - 1)[col], and the row-wise kernels only touch x at the indices present
 * [ref: the index variants of sparse/spmv_op/arch35/spmv_op_kernel.cpp:139-181]. */
int opsparse_rebase_offsets_launch(const void *offsets, int32_t offsetsAre64, int32_t indexBase, int64_t count,
                                   int32_t *out, void *stream);

/* fp32 z = alpha * A * x + beta * yIn for the index variants of the SpMVOp API:
 * int32 or int64 row offsets (rowOffsetsAre64), int32 column indices, index
 * base 0 or 1 [ref: sparse/spmv_op/arch35/spmv_op_kernel.cpp:139-181].  One lane
 * group per row, no workspace: the route for matrices of more than 2^31 - 1 entries, which the 32-bit kernels
 * cannot index (aclsparseSpMVOp rebases smaller ones and runs the binned kernels). */
int opsparse_spmv_csr_indexed_launch(const void *rowOffsets, int32_t rowOffsetsAre64, int32_t indexBase,
                                     const int32_t *colInd, const float *csrValues, const float *x,
                                     const float *yIn, float *z, int64_t rows, int64_t cols, int64_t nnz,
                                     OpsparseScalar alpha, OpsparseScalar beta, void *stream);

/* ------------------------------------------------------------------ SpMM */

typedef OPSPARSE_ABI_ENUM(OpsparseSpmmKernel) {
    OPSPARSE_SPMM_AUTO = 0,
    OPSPARSE_SPMM_ROW_SPLIT = 1, /* no row above the long-row threshold: every row whole by one lane group */
    OPSPARSE_SPMM_BINNED = 2     /* rows up to the long-row threshold as ROW_SPLIT, longer rows cut into
                                    fixed nnz segments over several waves + a fix-up pass */
} OpsparseSpmmKernel;

typedef struct OpsparseSpmmPlan {
    int32_t kernel;        /* OpsparseSpmmKernel */
    int32_t maxRowNnz;
    int32_t longRowNnz;    /* rows with more nnz than this are "long" */
    int32_t numLongRows;
    int32_t numSegments;   /* segments over all long rows */
    int32_t segmentNnz;    /* nnz per segment */
    int64_t rows;
    int64_t nnz;
    int64_t n;             /* columns of C the partial buffer was sized for */
    int64_t longRowsOff;   /* int32 row ids of long rows */
    int64_t segRowOff;     /* int32 [numSegments]: index into long rows */
    int64_t segStartOff;   /* int32 [numSegments]: first nnz of the segment */
    int64_t longFirstSegOff; /* int32 [numLongRows + 1]: first segment of each long row */
    int64_t partialOff;    /* double [numSegments * n] */
    int64_t slabStartOff;  /* int32 [numSlabs + 1]: first row of every slab of the slab kernel (0: no table) */
    int64_t numSlabs;
    int64_t bytes;
} OpsparseSpmmPlan;

/* Exact workspace size for this matrix and n.  256 bytes when no row is long;
 * otherwise a device reduction over the row offsets counts the long rows and
 * their segments (allocates and frees a 256-byte device scratch, synchronises
 * `stream`). */
int opsparse_spmm_csr_workspace_bytes(const int32_t *rowOffsets, int64_t rows, int64_t nnz, int64_t n, void *stream,
                                      size_t *bytes);

/* Row statistics and, for BINNED, the long-row / segment tables (built on the
 * device; 12 bytes of statistics and one counter travel to the host).  Synchronises `stream`. */
int opsparse_spmm_csr_analyse(const int32_t *rowOffsets, int64_t rows, int64_t nnz, int64_t n, void *workspace,
                              size_t workspaceBytes, int32_t forceKernel, OpsparseSpmmPlan *plan, void *stream);

/*
 * C[rows x n] = alpha * A * op(B) + beta * C.
 * bColMajor / cColMajor select the storage order, ldb / ldc the leading
 * dimensions in elements; transB != 0 reads B as its transpose, with the index
 * formulas of the reference kernel [ref: sparse/spmm/arch35/spmm_kernel.cpp:155-168, :215-219].
 * clampF16: when cType is F16, clamp to +-65504 before rounding [ref: :229-237].
 * With a plan and row-major operands the rows are worked in slabs of consecutive
 * rows staged through LDS (short rows share gather batches); plan == NULL runs
 * one lane group per row without a workspace.  A plan made for n <= 16 of a matrix
 * whose longest row has at most 200 entries cuts the slabs for the kernel that
 * gathers whole rows of a B of 16 or 32 bytes a row (fp32 n = 4, 8; fp16 n = 8, 16;
 * ldb and ldc below 2^32): pass the n the plan was analysed for.
 */
int opsparse_spmm_csr_launch(const OpsparseSpmmPlan *plan, const int32_t *rowOffsets, const int32_t *colInd,
                             const void *csrValues, const void *B, void *C, int64_t rows, int64_t k, int64_t n,
                             int64_t nnz, int64_t ldb, int64_t ldc, int32_t bColMajor, int32_t cColMajor,
                             int32_t transB, OpsparseScalar alpha, OpsparseScalar beta, int32_t valType,
                             int32_t cType, void *workspace, size_t workspaceBytes, void *stream);

/*
 * 1 when opsparse_spmm_csr_launch with this analysed plan and workspace takes row-major fp32 B and C of n <= 8
 * columns at any leading dimension and 4-byte alignment where they are, with the kernel for a B of few columns; 0
 * when operands that are not whole aligned 16-byte rows would run a lane a column in place and are better copied
 * to padded rows first (opsparse_dense_restage).  The plan may have been analysed for n rounded up to a multiple of
 * 4.  aclsparseSpMM asks before it uses its staging area.
 */
int opsparse_spmm_csr_narrow_rows(const OpsparseSpmmPlan *plan, const void *workspace, int64_t n, int64_t nnz,
                                  int32_t valType, int32_t cType);

/*
 * Dense rows x cols matrix copied from one storage order / leading dimension to another (elements of 1, 2 or
 * 4 bytes); columns cols .. colsDst-1 of the destination are written as zero.  aclsparseSpMM uses it to hand
 * column-major or transposed B / C to the row-major kernels through a staging area of the SpMM buffer: the
 * index formulas are the reference kernel's [ref: sparse/spmm/arch35/spmm_kernel.cpp:155-168, :215-219], which
 * reads such operands in place, one element per line.
 */
int opsparse_dense_restage(const void *src, void *dst, int64_t rows, int64_t cols, int64_t colsDst, int64_t ldSrc,
                           int32_t srcColMajor, int64_t ldDst, int32_t dstColMajor, int32_t elemBytes, void *stream);

/* --------------------------------------------------------- CSR producers
 * Raw launchers of the format conversions; they play the role of the reference's
 * coo2csr_*_kernel_do / csr2coo_kernel_do / csrsort_kernel_do / csr2csc_ex2_*_kernel_do
 * launchers [ref: sparse/coo2csr/arch35/coo2csr_kernel.h, sparse/csr2coo/arch35/csr2coo_kernel.h,
 * sparse/csrsort/arch35/csrsort_kernel.h, sparse/csr2csc_ex2/arch35/csr2csc_ex2_kernel.h].
 * indexBase is 0 or 1.  Workspaces need 4-byte alignment. */

/* Scratch of the int32 prefix sum over `count` elements (the tile sums). */
size_t opsparse_scan_workspace_bytes(int64_t count);

/* csrRowPtr[0..m] from row indices; workspace >= opsparse_scan_workspace_bytes(m + 1). */
int opsparse_coo2csr_launch(const int32_t *cooRowInd, int64_t nnz, int64_t m, int32_t *csrRowPtr, int32_t indexBase,
                            void *workspace, size_t workspaceBytes, void *stream);

/* cooRowInd[0..nnz) from csrRowPtr[0..m]. */
int opsparse_csr2coo_launch(const int32_t *csrRowPtr, int64_t nnz, int64_t m, int32_t *cooRowInd, int32_t indexBase,
                            void *stream);

/* Per-row stable sort of csrColInd with perm carried along. */
size_t opsparse_csrsort_workspace_bytes(int64_t m, int64_t nnz);
int opsparse_csrsort_launch(int64_t m, int64_t n, int64_t nnz, int32_t indexBase, const int32_t *csrRowPtr,
                            int32_t *csrColInd, int32_t *perm, void *workspace, size_t workspaceBytes, void *stream);

/* Stable sort of (cooRows, cooCols, perm) triples in place: byRow != 0 ascending in the row and, among equal rows,
 * in the column; byRow == 0 the other way round.  Signed indices of any value.  Synchronises `stream` once (the
 * range the indices span is read back and sets the number of passes). */
size_t opsparse_coosort_workspace_bytes(int64_t nnz);
int opsparse_coosort_launch(int64_t nnz, int32_t byRow, int32_t *cooRows, int32_t *cooCols, int32_t *perm,
                            void *workspace, size_t workspaceBytes, void *stream);

/* CSR -> CSC.  valueBytes: 0 (structure only), 1, 2 or 4. */
size_t opsparse_csr2csc_workspace_bytes(int64_t m, int64_t n, int64_t nnz);
int opsparse_csr2csc_launch(int64_t m, int64_t n, int64_t nnz, const void *csrVal, const int32_t *csrRowPtr,
                            const int32_t *csrColInd, void *cscVal, int32_t *cscColPtr, int32_t *cscRowInd,
                            int32_t valueBytes, int32_t indexBase, void *workspace, size_t workspaceBytes,
                            void *stream);

/* ----------------------------------------------------------- measurement */

/* Plain device-to-device copy kernel (dwordx4 per lane) used as the HBM
 * bandwidth yard-stick and as the calibration kernel for the FETCH_SIZE /
 * WRITE_SIZE counters.  bytes must be a multiple of 16. */
int opsparse_copy_launch(const void *src, void *dst, size_t bytes, void *stream);

/* Reads `bytes` (a multiple of 16) once with non-temporal dwordx4 loads and
 * writes nothing: the read-bandwidth ceiling of a streaming kernel.  `sink`
 * (4 bytes, may be NULL) only keeps the loads alive. */
int opsparse_read_launch(const void *src, size_t bytes, void *sink, void *stream);

/* One independent 4-byte gather x[indices[i]] per index (indices streamed,
 * results summed in registers): the rate at which this GPU serves random
 * gathers from a vector of a given size, which bounds SpMV on matrices with
 * scattered columns.  Indices must be valid positions in x or negative. */
int opsparse_gather_launch(const int32_t *indices, const float *x, size_t count, void *sink, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* OPS_SPARSE_HIP_H_ */
