/*
 * Public C ABI of libops_sparse.so on AMD MI355X (gfx950): the generic CSR
 * SpMV / SpMM path of the aclsparse API.
 *
 * This header is a drop-in for the subset of the reference's
 * include/cann_ops_sparse.h that the CSR SpMV / SpMM path touches: the same
 * type names, enumerators (same order, hence same values), function names and
 * argument lists, so a caller written against the reference compiles and links
 * unchanged.  Every declaration cites the reference declaration it replaces as
 * [ref: file:line], relative to the reference tree.
 *
 * Conventions shared by every entry point
 *   - returns aclsparseStatus_t, never throws, never aborts;
 *   - "DEVICE" pointers are HIP device pointers that the library borrows and
 *     never frees; "HOST" pointers are ordinary process memory;
 *   - compute calls enqueue work on the handle's stream and return; the caller
 *     synchronises the stream before reading results;
 *   - a handle and the descriptors used with it must not be used from two
 *     threads at once.
 */
#ifndef CANN_OPS_SPARSE_H_
#define CANN_OPS_SPARSE_H_

#include <stddef.h>
#include <stdint.h>
#include <acl/acl_base_rt.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ enums */

/* [ref: include/cann_ops_sparse.h:24-28] operation applied to an operand. */
typedef OPSPARSE_ABI_ENUM(aclsparseOperation_t) {
    ACL_SPARSE_OP_NON_TRANSPOSE = 0,
    ACL_SPARSE_OP_TRANSPOSE,
    ACL_SPARSE_OP_CONJUGATE_TRANSPOSE
} aclsparseOperation_t;

/* [ref: :50-53] storage order of a dense matrix (B and C of SpMM). */
typedef OPSPARSE_ABI_ENUM(aclsparseOrder_t) {
    ACL_SPARSE_ORDER_ROW = 0,
    ACL_SPARSE_ORDER_COL = 1
} aclsparseOrder_t;

/* [ref: :56-70] algorithm selector of the SpMVOp API. */
typedef OPSPARSE_ABI_ENUM(aclsparseSpMVOpAlg_t) {
    ACL_SPARSE_SPMVOP_ALG_DEFAULT = 0,
    ACL_SPARSE_SPMVOP_ALG1,
    ACL_SPARSE_SPMVOP_ALG2
} aclsparseSpMVOpAlg_t;

/* [ref: :81-96] SpMM algorithm selector.  DEFAULT and CSR_ALG1 are the same
 * kernels.  The reference's third value selects Kahan-compensated fp32
 * accumulation; here every floating-point SpMM kernel already accumulates in
 * fp64 and rounds once, so the three values give identical results. */
typedef OPSPARSE_ABI_ENUM(aclsparseSpMMAlg_t) {
    ACL_SPARSE_SPMM_ALG_DEFAULT = 0,
    ACL_SPARSE_SPMM_CSR_ALG1,
    ACL_SPARSE_SPMM_CSR_FP32_HIGH_PRECISION_ALG
} aclsparseSpMMAlg_t;

/* [ref: :98-148] status codes. */
typedef OPSPARSE_ABI_ENUM(aclsparseStatus_t) {
    ACL_SPARSE_STATUS_SUCCESS = 0,
    ACL_SPARSE_STATUS_NOT_INITIALIZED,
    ACL_SPARSE_STATUS_ALLOC_FAILED,
    ACL_SPARSE_STATUS_INVALID_VALUE,
    ACL_SPARSE_STATUS_ARCH_MISMATCH,
    ACL_SPARSE_STATUS_EXECUTION_FAILED,
    ACL_SPARSE_STATUS_INTERNAL_ERROR,
    ACL_SPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED,
    ACL_SPARSE_STATUS_NOT_SUPPORTED,
    ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES,
    ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR
} aclsparseStatus_t;

/* [ref: :150-168] SpMV algorithm selector; only ALG_DEFAULT is accepted by
 * aclsparseSpMV, as in the reference (sparse/spmv/arch22/spmv_host.cpp:144). */
typedef OPSPARSE_ABI_ENUM(aclsparseSpMVAlg_t) {
    ACL_SPARSE_SPMV_ALG_DEFAULT,
    ACL_SPARSE_SPMV_COO_ALG1,
    ACL_SPARSE_SPMV_COO_ALG2,
    ACL_SPARSE_SPMV_CSR_ALG1,
    ACL_SPARSE_SPMV_CSR_ALG2,
    ACL_SPARSE_SPMV_SELL_ALG1
} aclsparseSpMVAlg_t;

/* [ref: :213-222] width of row offsets / column indices. */
typedef OPSPARSE_ABI_ENUM(aclsparseIndexType_t) {
    ACL_SPARSE_INDEX_32I = 0,
    ACL_SPARSE_INDEX_64I
} aclsparseIndexType_t;

/* [ref: :229-232] */
typedef OPSPARSE_ABI_ENUM(aclsparseIndexBase_t) {
    ACL_SPARSE_INDEX_BASE_ZERO = 0,
    ACL_SPARSE_INDEX_BASE_ONE
} aclsparseIndexBase_t;

/* [ref: :235-248] sparse storage format tag; only CSR descriptors can be
 * created through this library, the other tags exist so that
 * aclsparseSpMatGetFormat has the reference's value space. */
typedef OPSPARSE_ABI_ENUM(aclsparseFormat_t) {
    ACL_SPARSE_FORMAT_COO = 0,
    ACL_SPARSE_FORMAT_CSR,
    ACL_SPARSE_FORMAT_CSC,
    ACL_SPARSE_FORMAT_BLOCKED_ELL,
    ACL_SPARSE_FORMAT_SLICED_ELL,
    ACL_SPARSE_FORMAT_BSR
} aclsparseFormat_t;

/* [ref: :898-901] where alpha / beta live. */
typedef OPSPARSE_ABI_ENUM(aclsparsePointerMode_t) {
    ACL_SPARSE_POINTER_MODE_HOST = 0,
    ACL_SPARSE_POINTER_MODE_DEVICE = 1
} aclsparsePointerMode_t;

/* [ref: :192-210] attributes of the legacy matrix descriptor. */
typedef OPSPARSE_ABI_ENUM(aclsparseMatrixType_t) {
    ACL_SPARSE_MATRIX_TYPE_GENERAL = 0,
    ACL_SPARSE_MATRIX_TYPE_SYMMETRIC,
    ACL_SPARSE_MATRIX_TYPE_HERMITIAN,
    ACL_SPARSE_MATRIX_TYPE_TRIANGULAR
} aclsparseMatrixType_t;

typedef OPSPARSE_ABI_ENUM(aclsparseDiagType_t) {
    ACL_SPARSE_DIAG_TYPE_NON_UNIT = 0,
    ACL_SPARSE_DIAG_TYPE_UNIT
} aclsparseDiagType_t;

typedef OPSPARSE_ABI_ENUM(aclsparseFillMode_t) {
    ACL_SPARSE_FILL_MODE_LOWER = 0,
    ACL_SPARSE_FILL_MODE_UPPER
} aclsparseFillMode_t;

/* [ref: :1369-1379] CSR -> CSC: structure only, or structure and values; algorithm tag. */
typedef OPSPARSE_ABI_ENUM(aclsparseAction_t) {
    ACL_SPARSE_ACTION_SYMBOLIC = 0,
    ACL_SPARSE_ACTION_NUMERIC
} aclsparseAction_t;

typedef OPSPARSE_ABI_ENUM(aclsparseCsr2CscAlg_t) {
    ACL_SPARSE_CSR2CSC_ALG_DEFAULT = 0,
    ACL_SPARSE_CSR2CSC_ALG1
} aclsparseCsr2CscAlg_t;

/* ---------------------------------------------------------- opaque types */

/* [ref: :30-47, :73-78] */
struct aclsparseContext;
struct aclsparseSpMatDescr;
struct aclsparseDnVecDescr;
struct aclsparseDnMatDescr;
struct aclsparseSpMVOpDescr;
struct aclsparseSpMVOpPlan;
struct aclsparseMatDescr; /* [ref: :189-190] legacy descriptor: type, index base, diag, fill */

typedef struct aclsparseMatDescr *aclsparseMatDescr_t;
typedef struct aclsparseContext *aclsparseHandle_t;
typedef struct aclsparseSpMatDescr *aclsparseSpMatDescr_t;
typedef struct aclsparseDnVecDescr *aclsparseDnVecDescr_t;
typedef struct aclsparseDnMatDescr *aclsparseDnMatDescr_t;
typedef struct aclsparseSpMatDescr const *aclsparseConstSpMatDescr_t;
typedef struct aclsparseDnVecDescr const *aclsparseConstDnVecDescr_t;
typedef struct aclsparseDnMatDescr const *aclsparseConstDnMatDescr_t;
typedef struct aclsparseSpMVOpDescr *aclsparseSpMVOpDescr_t;
typedef struct aclsparseSpMVOpDescr const *aclsparseConstSpMVOpDescr_t;
typedef struct aclsparseSpMVOpPlan *aclsparseSpMVOpPlan_t;

/* ----------------------------------------------------------------- handle */

/* [ref: :817] Allocates a handle and its 4 MiB default device workspace.
 * *handle must be NULL on entry (INVALID_VALUE otherwise); handle == NULL
 * gives HANDLE_IS_NULLPTR. */
aclsparseStatus_t aclsparseCreate(aclsparseHandle_t *handle);

/* [ref: :828] Synchronises the handle's stream, frees the default workspace
 * and the handle.  The stream and any user workspace stay with the caller. */
aclsparseStatus_t aclsparseDestroy(aclsparseHandle_t handle);

/* [ref: :837, :848] The stream all compute calls of this handle enqueue on. */
aclsparseStatus_t aclsparseSetStream(aclsparseHandle_t handle, aclrtStream stream);
aclsparseStatus_t aclsparseGetStream(aclsparseHandle_t handle, aclrtStream *stream);

/* [ref: :867, :882] Borrow a caller-owned device workspace (grow-only: a
 * request not larger than the current user workspace is ignored; NULL returns
 * to the default workspace). */
aclsparseStatus_t aclsparseSetWorkspace(aclsparseHandle_t handle, void *workspace, size_t workspaceSize);
aclsparseStatus_t aclsparseGetWorkspace(aclsparseHandle_t handle, void **workspace, size_t *workspaceSize);

/* [ref: :894] MAJOR*10000 + MINOR*100 + PATCH; handle may be NULL. */
aclsparseStatus_t aclsparseGetVersion(aclsparseHandle_t handle, int *version);

/* [ref: :903-904] HOST (default): alpha/beta are dereferenced on the host at
 * call time.  DEVICE: they are device addresses read by the kernel, so no
 * host synchronisation is needed to change them. */
aclsparseStatus_t aclsparseSetPointerMode(aclsparseHandle_t handle, aclsparsePointerMode_t mode);
aclsparseStatus_t aclsparseGetPointerMode(aclsparseHandle_t handle, aclsparsePointerMode_t *mode);

/* ----------------------------------------------------------- dense vector */

/* [ref: :259, :264, :273] size >= 0; values may be NULL only when size == 0. */
aclsparseStatus_t aclsparseCreateDnVec(aclsparseDnVecDescr_t *dnVecDescr, int64_t size, void *values,
                                       aclDataType valueType);
aclsparseStatus_t aclsparseCreateConstDnVec(aclsparseConstDnVecDescr_t *dnVecDescr, int64_t size,
                                            const void *values, aclDataType valueType);
aclsparseStatus_t aclsparseDestroyDnVec(aclsparseConstDnVecDescr_t dnVecDescr);

/* [ref: :335-373] accessors; NULL out-pointers of the Get* forms are skipped. */
aclsparseStatus_t aclsparseDnVecGet(aclsparseDnVecDescr_t dnVecDescr, int64_t *size, void **values,
                                    aclDataType *valueType);
aclsparseStatus_t aclsparseConstDnVecGet(aclsparseConstDnVecDescr_t dnVecDescr, int64_t *size,
                                         const void **values, aclDataType *valueType);
aclsparseStatus_t aclsparseDnVecGetValues(aclsparseDnVecDescr_t dnVecDescr, void **values);
aclsparseStatus_t aclsparseConstDnVecGetValues(aclsparseConstDnVecDescr_t dnVecDescr, const void **values);
aclsparseStatus_t aclsparseDnVecSetValues(aclsparseDnVecDescr_t dnVecDescr, void *values);

/* ---------------------------------------------------------- sparse matrix */

/* [ref: :399-408] CSR descriptor over caller-owned device arrays:
 * csrRowOffsets[rows+1], csrColInd[nnz], csrValues[nnz].  All four I32/I64
 * combinations are accepted here; SpMV / SpMM accept (I32, I32) only. */
aclsparseStatus_t aclsparseCreateCsr(aclsparseSpMatDescr_t *spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                     void *csrRowOffsets, void *csrColInd, void *csrValues,
                                     aclsparseIndexType_t csrRowOffsetsType, aclsparseIndexType_t csrColIndType,
                                     aclsparseIndexBase_t idxBase, aclDataType valueType);
aclsparseStatus_t aclsparseCreateConstCsr(aclsparseConstSpMatDescr_t *spMatDescr, int64_t rows, int64_t cols,
                                          int64_t nnz, const void *csrRowOffsets, const void *csrColInd,
                                          const void *csrValues, aclsparseIndexType_t csrRowOffsetsType,
                                          aclsparseIndexType_t csrColIndType, aclsparseIndexBase_t idxBase,
                                          aclDataType valueType);

/* [ref: :446] replace the three device arrays of a CSR descriptor; drops any
 * preprocessing bound to the descriptor. */
aclsparseStatus_t aclsparseCsrSetPointers(aclsparseSpMatDescr_t descr, void *rowOffsets, void *colIndices,
                                          void *values);

/* [ref: :459] NULL is accepted and returns SUCCESS. */
aclsparseStatus_t aclsparseDestroySpMat(aclsparseConstSpMatDescr_t spMatDescr);

/* [ref: :465-478] */
aclsparseStatus_t aclsparseSpMatGetFormat(aclsparseConstSpMatDescr_t spMatDescr, aclsparseFormat_t *format);
aclsparseStatus_t aclsparseSpMatGetValues(aclsparseSpMatDescr_t spMatDescr, void **values);
aclsparseStatus_t aclsparseConstSpMatGetValues(aclsparseConstSpMatDescr_t spMatDescr, const void **values);
aclsparseStatus_t aclsparseSpMatSetValues(aclsparseSpMatDescr_t spMatDescr, void *values);
aclsparseStatus_t aclsparseSpMatGetSize(aclsparseConstSpMatDescr_t spMatDescr, int64_t *rows, int64_t *cols,
                                        int64_t *nnz);

/* ----------------------------------------------------------- dense matrix */

/* [ref: :552-564] rows > 0, cols > 0, ld >= cols (row-major) or >= rows
 * (column-major), values non-NULL. */
aclsparseStatus_t aclsparseCreateDnMat(aclsparseDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols, int64_t ld,
                                       void *values, aclDataType valueType, aclsparseOrder_t order);
aclsparseStatus_t aclsparseCreateConstDnMat(aclsparseConstDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols,
                                            int64_t ld, const void *values, aclDataType valueType,
                                            aclsparseOrder_t order);
aclsparseStatus_t aclsparseDestroyDnMat(aclsparseConstDnMatDescr_t dnMatDescr);

/* [ref: :581-614] */
aclsparseStatus_t aclsparseDnMatGet(aclsparseDnMatDescr_t dnMatDescr, int64_t *rows, int64_t *cols, int64_t *ld,
                                    void **values, aclDataType *valueType, aclsparseOrder_t *order);
aclsparseStatus_t aclsparseConstDnMatGet(aclsparseConstDnMatDescr_t dnMatDescr, int64_t *rows, int64_t *cols,
                                         int64_t *ld, const void **values, aclDataType *valueType,
                                         aclsparseOrder_t *order);
aclsparseStatus_t aclsparseDnMatGetValues(aclsparseDnMatDescr_t dnMatDescr, void **values);
aclsparseStatus_t aclsparseConstDnMatGetValues(aclsparseConstDnMatDescr_t dnMatDescr, const void **values);
aclsparseStatus_t aclsparseDnMatSetValues(aclsparseDnMatDescr_t dnMatDescr, void *values);

/* ------------------------------------------------------------------- SpMV */

/*
 * y = alpha * op(A) * x + beta * y, A in CSR with int32 zero-based indices.
 *
 * Type triples (A and x, y, computeType): (f32, f32, f32), (f16, f16, f32),
 * (f16, f32, f32), (bf16, bf16, f32), (bf16, f32, f32), (i32, f32, f32),
 * (i32, i32, i32) [ref: sparse/spmv/arch22/spmv.h:67-103].  Floating-point
 * rows are accumulated in fp64 in stored order and rounded once to the type
 * of y; y is not read when beta == 0.
 *
 * aclsparseSpMV [ref: include/cann_ops_sparse.h:531-533, implementation
 * sparse/spmv/arch22/spmv_host.cpp:121-295] needs no buffer: with
 * externalBuffer == NULL (or a buffer that was not preprocessed for matA) it
 * uses a partition kept in the handle's workspace.  GetBufferSize /
 * Preprocess [ref: :490-514, declared by the reference without a definition]
 * analyse the row-length distribution once and store the kernel choice and the
 * merge-path partition in the caller's buffer; later aclsparseSpMV calls that
 * pass the same buffer skip that work.  For a large matrix with scattered
 * columns the answer of GetBufferSize is larger and Preprocess re-stores the
 * matrix in the buffer; it does so only where a GetBufferSize call on the same
 * descriptor and arrays, with the same opA / types / alg, answered that size
 * (a buffer sized any other way gets the ordinary plan, which fits every
 * answer).  For such a matrix (more than 2^18 columns, 7 M entries or more)
 * GetBufferSize itself looks at the column indices: it launches one short
 * kernel on the handle's stream, uses the handle's workspace (created on first
 * use) and synchronises the stream once; inside a stream capture it does none of
 * that and answers the ordinary plan's size.  Preprocess synchronises the stream
 * (once for the ordinary plan, up to four times for a re-stored layout) and
 * must not be captured; aclsparseSpMV itself only enqueues kernels.
 *
 * Repeatability [ref: include/cann_ops_sparse.h:151-164]: ACL_SPARSE_SPMV_CSR_ALG2
 * gives bit-wise the same y from every call on the same data, for either op(A)
 * (the reference promises it for op(A) = A only).  So do ALG_DEFAULT / CSR_ALG1
 * with op(A) = A wherever the plan is row-wise or merge-path (every unprepared
 * call, every matrix under 7 M entries or with local columns) and for int32.
 * The plans that add in the order their wavefronts arrive are the default
 * algorithm's re-stored layouts on floating-point data (op(A) = A: row blocks
 * summed with LDS atomics; op(A) = A^T over more than 2 M columns: products
 * sorted by output panel and summed with LDS atomics) and op(A) = A^T without
 * Preprocess (fp32 atomics on y): there the last bit of an element may differ
 * between two calls, as the reference says of CSR_ALG1.
 * OPS_SPARSE_SPMV_REPEATABLE=1 in the environment makes Preprocess choose
 * the ordered layouts there too.
 *
 * alpha / beta: typed by computeType; NULL means alpha = 1, beta = 0
 * [ref: spmv_host.cpp:183-199]; read according to the handle's pointer mode.
 */
aclsparseStatus_t aclsparseSpMVGetBufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA, const void *alpha,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX,
                                             const void *beta, aclsparseDnVecDescr_t vecY, aclDataType computeType,
                                             aclsparseSpMVAlg_t alg, size_t *bufferSize);
aclsparseStatus_t aclsparseSpMVPreprocess(aclsparseHandle_t handle, aclsparseOperation_t opA, const void *alpha,
                                          aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX,
                                          const void *beta, aclsparseDnVecDescr_t vecY, aclDataType computeType,
                                          aclsparseSpMVAlg_t alg, void *externalBuffer);
aclsparseStatus_t aclsparseSpMV(aclsparseHandle_t handle, aclsparseOperation_t opA, const void *alpha,
                                aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX, const void *beta,
                                aclsparseDnVecDescr_t vecY, aclDataType computeType, aclsparseSpMVAlg_t alg,
                                void *externalBuffer);

/* ------------------------------------------------------------------- SpMM */

/*
 * C = alpha * A * op(B) + beta * C, A in CSR (int32, zero-based), B and C
 * dense in either order with leading dimensions honoured.
 * [ref: include/cann_ops_sparse.h:682-704, implementation
 * sparse/spmm/arch35/spmm_host.cpp:213-234, :335-362, :364-394]
 *
 * Type quadruples (A, B, C, computeType): (f32, f32, f32, f32),
 * (f16, f16, f16, f32) with the result clamped to +-65504 before the fp16
 * rounding, (i8, i8, i32, i32) saturating [ref: spmm_host.cpp:103-120], and
 * the extension (f16, f16, f32, f32) which is the fp16 case without the final
 * clamp and rounding.  C is not read when beta == 0.
 *
 * The three calls keep the reference's protocol: GetBufferSize reports the
 * bytes Preprocess needs, Preprocess fills the buffer and binds it to matA,
 * SpMM with the same buffer reuses it; SpMM with a different non-NULL buffer
 * preprocesses into that buffer first.  buffer == NULL gives
 * INSUFFICIENT_RESOURCES.  alpha / beta follow the handle's pointer mode;
 * NULL is read as 0 [ref: spmm_host.cpp:62-74].
 */
aclsparseStatus_t aclsparseSpMMGetBufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                             aclsparseOperation_t opB, const void *alpha,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnMatDescr_t matB,
                                             const void *beta, aclsparseDnMatDescr_t matC, aclDataType computeType,
                                             aclsparseSpMMAlg_t alg, size_t *size);
aclsparseStatus_t aclsparseSpMMPreprocess(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                          aclsparseOperation_t opB, const void *alpha,
                                          aclsparseConstSpMatDescr_t matA, aclsparseConstDnMatDescr_t matB,
                                          const void *beta, aclsparseDnMatDescr_t matC, aclDataType computeType,
                                          aclsparseSpMMAlg_t alg, void *buffer);
aclsparseStatus_t aclsparseSpMM(aclsparseHandle_t handle, aclsparseOperation_t opA, aclsparseOperation_t opB,
                                const void *alpha, aclsparseConstSpMatDescr_t matA,
                                aclsparseConstDnMatDescr_t matB, const void *beta, aclsparseDnMatDescr_t matC,
                                aclDataType computeType, aclsparseSpMMAlg_t alg, void *buffer);

/* ------------------------------------------------------------------ SpMVOp
 * [ref: include/cann_ops_sparse.h:1564-1637; host: sparse/spmv_op/arch35/spmv_op_host.cpp]
 *
 * Z = alpha * A * X + beta * Y with a descriptor / plan pair, fp32 only:
 * opA = NON_TRANSPOSE, computeType ACL_FLOAT, CSR with fp32 values, 32-bit
 * column indices, 32- or 64-bit row offsets, index base 0 or 1.  Z may be Y.
 * Results are bit-wise repeatable for every algorithm value [ref:
 * include/cann_ops_sparse.h:57-69]: every row is summed in fp64 in an order that
 * depends on the matrix and the plan only, never on scheduling (no atomics on
 * any path of this API), and rounded once.
 *
 *   bufferSize    for ALG2 the bytes of what createDescr writes (the
 *                 nnz-balanced partition, or a re-stored copy of the matrix
 *                 where x does not fit a cache); for ALG_DEFAULT / ALG1 0,
 *                 except for a large matrix with scattered columns (fp32,
 *                 zero-based 32-bit offsets, 7 M entries or more), where it is
 *                 the size of a re-stored index layout that createDescr builds
 *                 IF it is given a buffer (NULL stays legal: the ordinary
 *                 kernels then).  A layout is only built into a buffer when
 *                 bufferSize was asked on the same descriptor and arrays.  For
 *                 such a matrix bufferSize launches one short kernel on the
 *                 handle's stream, uses the handle's workspace and synchronises
 *                 once (not inside a stream capture, where it answers as for a
 *                 small matrix).
 *   createDescr   snapshots matA's pointers and sizes (not its values: they may
 *                 change between executions, except under ALG2); ALG2 needs
 *                 `buffer`, which must stay valid until destroyDescr.
 *   createPlan    only the identity epilogue: a non-NULL LTO buffer or a
 *                 non-zero size gives NOT_SUPPORTED.
 *   destroy*      NULL is accepted and gives SUCCESS.
 *   setGlobalUserData   checked and otherwise ignored (identity epilogue).
 *   aclsparseSpMVOp     X, Y, Z must be fp32 vectors of exactly cols / rows /
 *                 rows elements; Y's data may be NULL when beta is 0 (host
 *                 pointer mode) or in device pointer mode.
 */
aclsparseStatus_t aclsparseSpMVOp_bufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX,
                                             aclsparseConstDnVecDescr_t vecY, aclsparseDnVecDescr_t vecZ,
                                             aclDataType computeType, aclsparseSpMVOpAlg_t alg, size_t *bufferSize);
aclsparseStatus_t aclsparseSpMVOp_createDescr(aclsparseHandle_t handle, aclsparseSpMVOpDescr_t *descr,
                                              aclsparseOperation_t opA, aclsparseConstSpMatDescr_t matA,
                                              aclsparseConstDnVecDescr_t vecX, aclsparseConstDnVecDescr_t vecY,
                                              aclsparseDnVecDescr_t vecZ, aclDataType computeType,
                                              aclsparseSpMVOpAlg_t alg, void *buffer);
aclsparseStatus_t aclsparseSpMVOp_destroyDescr(aclsparseSpMVOpDescr_t descr);
aclsparseStatus_t aclsparseSpMVOp_createPlan(aclsparseHandle_t handle, aclsparseSpMVOpDescr_t descr,
                                             aclsparseSpMVOpPlan_t *plan, const void *epilogueLTOBuffer,
                                             size_t epilogueLTOBufferSize);
aclsparseStatus_t aclsparseSpMVOp_destroyPlan(aclsparseSpMVOpPlan_t plan);
aclsparseStatus_t aclsparseSpMVOp_setGlobalUserData(aclsparseHandle_t handle, aclsparseSpMVOpPlan_t plan,
                                                    const char *epilogueDataName, void *epilogueData,
                                                    size_t epilogueDataSize);
aclsparseStatus_t aclsparseSpMVOp(aclsparseHandle_t handle, aclsparseSpMVOpPlan_t plan, const void *alpha,
                                  const void *beta, aclsparseConstDnVecDescr_t vecX, aclsparseConstDnVecDescr_t vecY,
                                  aclsparseDnVecDescr_t vecZ);

/* ---------------------------------------------------------- CSR producers
 * Integer / byte operations; every output is bit-exact against the reference's
 * CPU goldens.  All enqueue on the handle's stream and return.
 */

/* Legacy matrix descriptor [ref: :910-919; sparse/common/aclsparse_matdescr.cpp:25-110].
 * Create gives GENERAL / base 0 / NON_UNIT / LOWER; Destroy(NULL) is SUCCESS;
 * setters ignore a NULL descriptor, getters return the default for it. */
aclsparseStatus_t aclsparseCreateMatDescr(aclsparseMatDescr_t *descr);
aclsparseStatus_t aclsparseDestroyMatDescr(aclsparseMatDescr_t descr);
void aclsparseSetMatType(aclsparseMatDescr_t descr, aclsparseMatrixType_t type);
void aclsparseSetMatIndexBase(aclsparseMatDescr_t descr, aclsparseIndexBase_t base);
void aclsparseSetMatDiagType(aclsparseMatDescr_t descr, aclsparseDiagType_t diagType);
void aclsparseSetMatFillMode(aclsparseMatDescr_t descr, aclsparseFillMode_t fillMode);
aclsparseMatrixType_t aclsparseGetMatType(aclsparseMatDescr_t descr);
aclsparseIndexBase_t aclsparseGetMatIndexBase(aclsparseMatDescr_t descr);
aclsparseDiagType_t aclsparseGetMatDiagType(aclsparseMatDescr_t descr);
aclsparseFillMode_t aclsparseGetMatFillMode(aclsparseMatDescr_t descr);

/* [ref: :1816-1822; host sparse/coo2csr/arch35/coo2csr_host.cpp:38-80]
 * csrRowPtr[0..m] from COO row indices (non-decreasing): per-row counts + prefix
 * sum, + idxBase.  Row indices outside [0, m) are not counted.  Uses the
 * handle's workspace (4 bytes per 2048 rows). */
aclsparseStatus_t aclsparseXcoo2csr(aclsparseHandle_t handle, const int *cooRowInd, int nnz, int m, int *csrRowPtr,
                                    aclsparseIndexBase_t idxBase);

/* [ref: :1886-1891; host sparse/csr2coo/arch35/csr2coo_host.cpp:66-115]
 * cooRowInd[j] = i + idxBase for j in [csrRowPtr[i], csrRowPtr[i+1]) - idxBase.
 * A NULL handle gives NOT_INITIALIZED (this entry point's own code). */
aclsparseStatus_t aclsparseXcsr2coo(aclsparseHandle_t handle, const int32_t *csrRowPtr, int64_t nnz, int64_t m,
                                    int32_t *cooRowInd, aclsparseIndexBase_t idxBase);

/* [ref: :1679-1711; host sparse/csrsort/arch35/csrsort_host.cpp:146-221]
 * Stable ascending sort of the column indices inside every row, in place; P
 * (any initial content, usually 0..nnz-1) is permuted the same way.  The index
 * base comes from descrA.  pBuffer needs 4-byte alignment only. */
aclsparseStatus_t aclsparseXcsrsort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz,
                                                  const int *csrRowPtr, const int *csrColInd,
                                                  size_t *pBufferSizeInBytes);
aclsparseStatus_t aclsparseXcsrsort(aclsparseHandle_t handle, int m, int n, int nnz, const aclsparseMatDescr_t descrA,
                                    const int *csrRowPtr, int *csrColInd, int *P, void *pBuffer);

/* [ref: :1825-1864; host sparse/cscsort/arch35/cscsort_host.cpp:52-216; order test/cscsort/arch35/cscsort_golden.h:30-70]
 * The column-wise twin of aclsparseXcsrsort: stable ascending sort of the row indices inside every column, in
 * place; P is permuted the same way; cscColPtr is not modified.  The index base comes from descrA.  pBuffer must
 * be 128-byte aligned (INVALID_VALUE otherwise, as in the reference). */
aclsparseStatus_t aclsparseXcscsort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz,
                                                  const int *cscColPtr, const int *cscRowInd,
                                                  size_t *pBufferSizeInBytes);
aclsparseStatus_t aclsparseXcscsort(aclsparseHandle_t handle, int m, int n, int nnz, const aclsparseMatDescr_t descrA,
                                    const int *cscColPtr, int *cscRowInd, int *P, void *pBuffer);

/* [ref: :1516-1563; host sparse/coosort/arch35/coosort_host.cpp:48-78, :262-371; order
 * test/coosort/arch35/coosort_golden.h:52-85]
 * Stable sort of the COO triples (row, column, P) in place.  ByRow: ascending in the row and, among equal rows,
 * in the column; ByColumn: ascending in the column and, among equal columns, in the row; equal (row, column)
 * keep their input order.  Indices are compared as signed integers and need not lie inside [0, m) x [0, n): m
 * and n are only checked to be positive.  P (usually preset to 0..nnz-1) travels with its entry, so that
 * sortedVal[i] = origVal[P[i]].  The call synchronises the handle's stream once. */
aclsparseStatus_t aclsparseXcoosort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz, const int *cooRowsA,
                                                  const int *cooColsA, size_t *pBufferSizeInBytes);
aclsparseStatus_t aclsparseXcoosortByRow(aclsparseHandle_t handle, int m, int n, int nnz, int *cooRowsA, int *cooColsA,
                                         int *P, void *pBuffer);
aclsparseStatus_t aclsparseXcoosortByColumn(aclsparseHandle_t handle, int m, int n, int nnz, int *cooRowsA,
                                            int *cooColsA, int *P, void *pBuffer);

/* [ref: :1401-1440; host sparse/csr2csc_ex2/arch35/csr2csc_ex2_host.cpp:109-232, :535-618]
 * CSR (m x n) -> CSC: cscColPtr[0..n], cscRowInd and, for NUMERIC, cscVal; the
 * entries of a column keep their CSR order (ascending rows).  Values are moved
 * as raw 1 / 2 / 4-byte items (ACL_INT8, ACL_FLOAT16, ACL_BF16, ACL_FLOAT).
 * buffer == NULL uses the handle's workspace when that is large enough. */
aclsparseStatus_t aclsparseCsr2cscEx2_bufferSize(aclsparseHandle_t handle, int m, int n, int nnz, const void *csrVal,
                                                 const int *csrRowPtr, const int *csrColInd, void *cscVal,
                                                 int *cscColPtr, int *cscRowInd, aclDataType valType,
                                                 aclsparseAction_t copyValues, aclsparseIndexBase_t idxBase,
                                                 aclsparseCsr2CscAlg_t alg, size_t *bufferSize);
aclsparseStatus_t aclsparseCsr2cscEx2(aclsparseHandle_t handle, int m, int n, int nnz, const void *csrVal,
                                      const int *csrRowPtr, const int *csrColInd, void *cscVal, int *cscColPtr,
                                      int *cscRowInd, aclDataType valType, aclsparseAction_t copyValues,
                                      aclsparseIndexBase_t idxBase, aclsparseCsr2CscAlg_t alg, void *buffer);

#ifdef __cplusplus
}
#endif

#endif /* CANN_OPS_SPARSE_H_ */
