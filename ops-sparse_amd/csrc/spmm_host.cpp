// aclsparseSpMMGetBufferSize / aclsparseSpMMPreprocess / aclsparseSpMM.
//
// Validation order and status codes follow the reference's arch35 host code
// (sparse/spmm/arch35/spmm_host.cpp:152-191 for the shared checks, :213-234,
// :335-362, :364-394 for the three entry points).  Not carried over: the
// synchronous device<->host round trip of the tiling struct on every SpMM call
// (:281-308); alpha / beta travel as kernel arguments instead.
#include <climits>

#include <cstdint>
#include <cstdlib>

#include "internal.h"

namespace {

struct SpmmTypes {
    int32_t valType;
    int32_t cType;
};

// (A, B, C, compute) combinations with a kernel.  The first three rows are the
// reference's table (spmm_host.cpp:103-120); the fourth is the fp16-in /
// fp32-out case.
bool ResolveTypes(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B, const aclsparseDnMatDescr *C,
                  aclDataType computeType, SpmmTypes *t)
{
    const aclDataType a = A->valueType, b = B->valueType, c = C->valueType;
    if (a == ACL_FLOAT && b == ACL_FLOAT && c == ACL_FLOAT && computeType == ACL_FLOAT) {
        *t = {OPSPARSE_F32, OPSPARSE_F32};
        return true;
    }
    if (a == ACL_FLOAT16 && b == ACL_FLOAT16 && c == ACL_FLOAT16 && computeType == ACL_FLOAT) {
        *t = {OPSPARSE_F16, OPSPARSE_F16};
        return true;
    }
    if (a == ACL_INT8 && b == ACL_INT8 && c == ACL_INT32 && computeType == ACL_INT32) {
        *t = {OPSPARSE_I8, OPSPARSE_I32};
        return true;
    }
    if (a == ACL_FLOAT16 && b == ACL_FLOAT16 && c == ACL_FLOAT && computeType == ACL_FLOAT) {
        *t = {OPSPARSE_F16, OPSPARSE_F32};
        return true;
    }
    return false;
}

aclsparseStatus_t Validate(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B, const aclsparseDnMatDescr *C,
                           aclsparseOperation_t opA, aclsparseOperation_t opB, aclDataType computeType,
                           aclsparseSpMMAlg_t alg, SpmmTypes *types)
{
    if (A == nullptr || B == nullptr || C == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (opA != ACL_SPARSE_OP_NON_TRANSPOSE) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (opB != ACL_SPARSE_OP_NON_TRANSPOSE && opB != ACL_SPARSE_OP_TRANSPOSE) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (A->format != ACL_SPARSE_FORMAT_CSR) {
        return ACL_SPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED;
    }
    if (A->rowOffsetsType != ACL_SPARSE_INDEX_32I || A->colIndType != ACL_SPARSE_INDEX_32I) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (A->idxBase != ACL_SPARSE_INDEX_BASE_ZERO) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (!ResolveTypes(A, B, C, computeType, types)) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    // The reference compares the descriptors' own rows / cols, not those of
    // op(B) (spmm_host.cpp:122-131); kept, so the same descriptors are accepted.
    if (A->cols != B->rows || A->rows != C->rows || B->cols != C->cols) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (alg != ACL_SPARSE_SPMM_ALG_DEFAULT && alg != ACL_SPARSE_SPMM_CSR_ALG1 &&
        alg != ACL_SPARSE_SPMM_CSR_FP32_HIGH_PRECISION_ALG) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (A->rows > INT32_MAX || C->cols > INT32_MAX) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t FromLaunch(int rc)
{
    switch (rc) {
        case OPSPARSE_OK: return ACL_SPARSE_STATUS_SUCCESS;
        case OPSPARSE_E_INVALID: return ACL_SPARSE_STATUS_INVALID_VALUE;
        case OPSPARSE_E_UNSUPPORTED: return ACL_SPARSE_STATUS_NOT_SUPPORTED;
        case OPSPARSE_E_WORKSPACE: return ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES;
        default: return ACL_SPARSE_STATUS_EXECUTION_FAILED;
    }
}

int64_t ElementBytes(int32_t type)
{
    return type == OPSPARSE_F32 || type == OPSPARSE_I32 ? 4 : (type == OPSPARSE_I8 ? 1 : 2);
}

// Column-major or transposed B, column-major C: the reference kernel reads them in place through its index
// formulas (spmm_kernel.cpp:155-168, :215-219), which here would mean one cache line per element (32/row, n = 64,
// column-major B: 37.8 ms against 1.2 ms row-major).  Instead the SpMM buffer carries, behind the plan's tables,
// room for compact row-major copies of such operands: B is copied in, the row-major kernels run, C is copied
// in (unless beta is known to be 0) and out.  n is padded to whole 16-byte vectors in the copies, so row-major
// operands of a width or leading dimension the vector kernels do not take go the same way (n = 62: 3.2 ms in
// place, n = 64: 1.2 ms).
struct Staging {
    bool b = false, c = false;
    int64_t nPadded = 0, bOff = 0, cOff = 0;
    int64_t bytes = 0;  // beyond the plan's own bytes, 0: the operands are used where they are
};

Staging MakeStaging(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B, const aclsparseDnMatDescr *C,
                    aclsparseOperation_t opB, const SpmmTypes &t, int64_t planBytes)
{
    Staging g{};
    const bool bColMajor = (B->order == ACL_SPARSE_ORDER_COL) != (opB == ACL_SPARSE_OP_TRANSPOSE);
    const bool cColMajor = C->order == ACL_SPARSE_ORDER_COL;
    if (A->rows <= 0 || A->cols <= 0 || C->cols <= 0) {
        return g;
    }
    const int64_t vec = 16 / ElementBytes(t.valType);
    g.nPadded = (C->cols + vec - 1) / vec * vec;
    // a width that is not whole vectors needs both copies: the kernels then run on the padded width; a row-major
    // operand whose leading dimension is not whole vectors needs its own
    g.b = bColMajor || g.nPadded != C->cols || B->ld % vec != 0;
    g.c = cColMajor || g.nPadded != C->cols || C->ld % vec != 0;
    if (!g.b && !g.c) {
        return g;
    }
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    int64_t off = align(planBytes);
    g.bOff = off;
    off += g.b ? align(A->cols * g.nPadded * ElementBytes(t.valType)) : 0;
    g.cOff = off;
    off += g.c ? align(A->rows * g.nPadded * ElementBytes(t.cType)) : 0;
    g.bytes = off - planBytes;
    return g;
}

// The width the plan is made for: the padded one when the product runs on staged copies.
int64_t PlanWidth(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B, const aclsparseDnMatDescr *C,
                  aclsparseOperation_t opB, const SpmmTypes &t)
{
    const Staging g = MakeStaging(A, B, C, opB, t, 0);
    return g.bytes > 0 ? g.nPadded : C->cols;
}

// One or two columns that lie in memory as vectors (column-major operands; a single column with a leading dimension
// of 1): the product is then n SpMV calls, which read the matrix n times and still beat the SpMM kernels, whose
// rows of B would be padded to 16 bytes in the staging area (5-point mesh of 4 M rows, n = 1: 37 us against 98 us;
// n = 2: 75 against 103; from n = 3 on the padded product wins, and for n = 2 already under rows of 27 entries:
// 244 us against 206, so two columns go this way up to 16 entries a row on average).  fp32, and fp16 with fp32 C:
// the fp16 C of SpMM is clamped to the finite range before rounding, which the SpMV kernels do not do.
bool ColumnsAreVectors(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B, const aclsparseDnMatDescr *C,
                       aclsparseOperation_t opB, const SpmmTypes &t)
{
    const int64_t n = C->cols;
    if (n < 1 || n > 2 || opB != ACL_SPARSE_OP_NON_TRANSPOSE || A->rows <= 0 || A->cols <= 0 || A->nnz <= 0 ||
        A->nnz > INT32_MAX || t.cType != OPSPARSE_F32 || (t.valType != OPSPARSE_F32 && t.valType != OPSPARSE_F16)) {
        return false;
    }
    if (n == 2 && A->nnz > 16 * A->rows) {
        return false;
    }
    const bool bVectors = B->order == ACL_SPARSE_ORDER_COL ? B->ld >= A->cols : (n == 1 && B->ld == 1);
    const bool cVectors = C->order == ACL_SPARSE_ORDER_COL ? C->ld >= A->rows : (n == 1 && C->ld == 1);
    return bVectors && cVectors;
}

// Whether a matrix without long rows, under a B of n elements of elemBytes, is better served by the kernel that
// gives every row whole to one lane group straight from memory than by the slabs staged through LDS.  Measured on
// fp32 (us, slabs / rows; 1 - 2 M rows of meshes, bands, and uniformly random columns):
//   n = 16: 5-point mesh 224 / 104, 27-point 439 / 280, band of 50 245 / 153, 32 random columns a row 494 / 415
//   n = 32: 5-point 255 / 182, 27-point 558 / 263, band of 200 190 / 103, 8 random 191 / 181, 32 random 315 / 375
//   n = 64: 5-point 392 / 365, 7-point 521 / 425, 27-point 772 / 423, band of 50 340 / 193, 32 random 592 / 631
//   n = 128: 5-point 694 / 730, 7-point 905 / 888, 27-point 1135 / 748, band of 200 458 / 299, 32 random 1198 / 1215
// The slabs win where the gathers of B are what the product waits for (random columns, wide rows of B) and on
// the shortest rows under the widest B; rows of even length whose columns stay near the diagonal, and any narrow
// B, run faster row by row.  Uneven rows stay with the slabs, which share them out by work.
bool PrefersWholeRows(const aclsparseSpMatDescr *A, const OpsparseSpmmPlan &plan, int64_t n, int64_t elemBytes,
                      void *buffer, hipStream_t stream)
{
    if (std::getenv("OPS_SPARSE_SPMM_NO_ROWS_RULE") != nullptr || stream == nullptr || elemBytes < 2 ||
        plan.kernel == OPSPARSE_SPMM_BINNED || plan.numLongRows != 0 || plan.maxRowNnz <= 0 || A->rows <= 0 ||
        A->colInd == nullptr) {
        return false;
    }
    const int64_t rowBytes = n * elemBytes;
    const double mean = static_cast<double>(A->nnz) / static_cast<double>(A->rows);
    if ((rowBytes == 16 || rowBytes == 32) && plan.maxRowNnz <= 200) {
        return false;  // the kernel for a B of one or two 16-byte pieces a row takes these
    }
    if (rowBytes > 512 || static_cast<double>(plan.maxRowNnz) > 4.0 * mean + 8.0) {
        return false;
    }
    if (elemBytes == 2) {
        // fp16, whose slab kernel is the one tuned on c5, keeps the slabs except under local rows of 16 entries or
        // more (us, slabs / rows: 27-point mesh n = 32 361 / 245, n = 64 459 / 399, n = 256 1401 / 1207; but 5-point
        // n = 64 267 / 305, n = 128 508 / 614, 32 random columns a row n = 32 292 / 412)
        if (mean < 16.0) {
            return false;
        }
    } else {
        if (rowBytes <= 64 || (rowBytes <= 128 && mean < 24.0)) {
            return true;
        }
        if (rowBytes > 256 && mean < 6.0) {
            return false;
        }
    }
    // what is left depends on whether the rows of B a row needs lie near each other: the sample of the SpMV plans
    // (the first 256 bytes of the buffer are the analyses' scratch: no launch reads them)
    int32_t scattered = 1000;
    if (opsparse_spmv_csr_gathers_scattered(static_cast<const int32_t *>(A->rowOffsets),
                                            static_cast<const int32_t *>(A->colInd), A->rows, A->cols, A->nnz, buffer,
                                            256, &scattered, stream) != OPSPARSE_OK) {
        return false;
    }
    return scattered < 250;
}

// Row statistics and long-row tables for width n into `buffer`; binds the buffer to A.
aclsparseStatus_t BuildPlan(const aclsparseSpMatDescr *A, int64_t n, int64_t elemBytes, void *buffer,
                            hipStream_t stream)
{
    // An empty matrix has nothing to preprocess (spmm_csr_mat.cpp:148-150).
    if (A->rows <= 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (A->rowOffsets == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    OpsparseSpmmPlan plan{};
    // Nothing says how large the caller's buffer is: it was sized by GetBufferSize for this matrix and width, and the
    // analysis lays out exactly what GetBufferSize counted (one reduction over the row offsets, no allocation).
    const size_t bytes = static_cast<size_t>(INT64_MAX);
    const int rc = opsparse_spmm_csr_analyse(static_cast<const int32_t *>(A->rowOffsets), A->rows, A->nnz, n, buffer,
                                             bytes, OPSPARSE_SPMM_AUTO, &plan, stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMM: analysis failed (%d)", rc);
        return FromLaunch(rc);
    }
    if (PrefersWholeRows(A, plan, n, elemBytes, buffer, stream)) {
        // a plan without tables: the launch layer then takes a lane group a row
        const int again = opsparse_spmm_csr_analyse(static_cast<const int32_t *>(A->rowOffsets), A->rows, A->nnz, n,
                                                    buffer, bytes, OPSPARSE_SPMM_ROW_SPLIT, &plan, stream);
        if (again != OPSPARSE_OK) {
            return FromLaunch(again);
        }
    }
    A->spmm.widestN = (A->spmm.buffer == buffer && A->spmm.widestN > n) ? A->spmm.widestN : n;
    A->spmm.buffer = buffer;
    A->spmm.plan = plan;
    A->spmm.stagingBytes = 0;
    A->spmm.vectorOff = 0;
    A->spmm.vectorBytes = 0;
    return ACL_SPARSE_STATUS_SUCCESS;
}

int64_t Align256(int64_t v)
{
    return (v + 255) / 256 * 256;
}

bool ScalarIsZero(const void *host, aclDataType computeType)
{
    return computeType == ACL_INT32 ? *static_cast<const int32_t *>(host) == 0
                                    : *static_cast<const float *>(host) == 0.0f;
}

// The product through the staging area: B copied to compact row-major (padded width), the row-major kernels,
// C copied in (unless beta is 0 for certain) and out.  Kernels only, all on `stream`.
int RunStaged(const Staging &g, const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *B,
              const aclsparseDnMatDescr *C, aclsparseOperation_t opB, OpsparseScalar alpha, OpsparseScalar beta,
              const SpmmTypes &t, bool betaIsZero, void *buffer, hipStream_t stream)
{
    auto *base = static_cast<unsigned char *>(buffer);
    const int64_t k = A->cols, m = A->rows, n = C->cols;
    const bool bColMajor = (B->order == ACL_SPARSE_ORDER_COL) != (opB == ACL_SPARSE_OP_TRANSPOSE);
    const bool cColMajor = C->order == ACL_SPARSE_ORDER_COL;
    const void *bUse = B->values;
    void *cUse = C->values;
    int64_t ldb = B->ld, ldc = C->ld;
    int rc = OPSPARSE_OK;
    if (g.b) {
        rc = opsparse_dense_restage(B->values, base + g.bOff, k, n, g.nPadded, B->ld, bColMajor ? 1 : 0, g.nPadded, 0,
                                    static_cast<int32_t>(ElementBytes(t.valType)), stream);
        bUse = base + g.bOff;
        ldb = g.nPadded;
    }
    if (rc == OPSPARSE_OK && g.c) {
        cUse = base + g.cOff;
        ldc = g.nPadded;
        if (!betaIsZero) {
            rc = opsparse_dense_restage(C->values, cUse, m, n, g.nPadded, C->ld, cColMajor ? 1 : 0, g.nPadded, 0,
                                        static_cast<int32_t>(ElementBytes(t.cType)), stream);
        }
    }
    if (rc != OPSPARSE_OK) {
        return rc;
    }
    // both copies exist whenever the width was padded, so the kernels may take the padded width as theirs
    const int64_t nRun = A->spmm.plan.n;  // the padded width, which the plan was made for
    rc = opsparse_spmm_csr_launch(&A->spmm.plan, static_cast<const int32_t *>(A->rowOffsets),
                                  static_cast<const int32_t *>(A->colInd), A->values, bUse, cUse, m, k, nRun, A->nnz,
                                  ldb, ldc, 0, g.c ? 0 : (cColMajor ? 1 : 0), 0, alpha, beta, t.valType, t.cType,
                                  buffer, static_cast<size_t>(A->spmm.plan.bytes), stream);
    if (rc == OPSPARSE_OK && g.c) {
        rc = opsparse_dense_restage(cUse, C->values, m, n, n, g.nPadded, 0, C->ld, cColMajor ? 1 : 0,
                                    static_cast<int32_t>(ElementBytes(t.cType)), stream);
    }
    return rc;
}

}  // namespace

extern "C" {

aclsparseStatus_t aclsparseSpMMGetBufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                             aclsparseOperation_t opB, const void * /*alpha*/,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnMatDescr_t matB,
                                             const void * /*beta*/, aclsparseDnMatDescr_t matC,
                                             aclDataType computeType, aclsparseSpMMAlg_t alg, size_t *size)
{
    if (size == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    SpmmTypes t{};
    const aclsparseStatus_t st = Validate(matA, matB, matC, opA, opB, computeType, alg, &t);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    // Matrices in which no row can be long need the 256-byte header only (no
    // device access); otherwise the long rows are counted on the device.
    if (matA->rows > 0 && matA->rowOffsets == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const int rc = opsparse_spmm_csr_workspace_bytes(static_cast<const int32_t *>(matA->rowOffsets), matA->rows,
                                                     matA->nnz, PlanWidth(matA, matB, matC, opB, t),
                                                     handle != nullptr ? handle->stream : nullptr, size);
    if (rc == OPSPARSE_OK) {
        *size += static_cast<size_t>(MakeStaging(matA, matB, matC, opB, t, static_cast<int64_t>(*size)).bytes);
        if (ColumnsAreVectors(matA, matB, matC, opB, t)) {
            // behind everything else: the workspace of the SpMV plan the columns run under
            *size = static_cast<size_t>(Align256(static_cast<int64_t>(*size))) +
                    opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
        }
    }
    return FromLaunch(rc);
}

aclsparseStatus_t aclsparseSpMMPreprocess(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                          aclsparseOperation_t opB, const void * /*alpha*/,
                                          aclsparseConstSpMatDescr_t matA, aclsparseConstDnMatDescr_t matB,
                                          const void * /*beta*/, aclsparseDnMatDescr_t matC, aclDataType computeType,
                                          aclsparseSpMMAlg_t alg, void *buffer)
{
    SpmmTypes t{};
    const aclsparseStatus_t st = Validate(matA, matB, matC, opA, opB, computeType, alg, &t);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (buffer == nullptr) {
        return ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES;
    }
    // The reference ignores the handle here; its stream is used when there is one.
    const aclsparseStatus_t built = BuildPlan(matA, PlanWidth(matA, matB, matC, opB, t), ElementBytes(t.valType),
                                              buffer, handle != nullptr ? handle->stream : nullptr);
    if (built == ACL_SPARSE_STATUS_SUCCESS) {
        // the buffer was sized by GetBufferSize for these operands: their staging area exists
        matA->spmm.stagingBytes = MakeStaging(matA, matB, matC, opB, t, matA->spmm.plan.bytes).bytes;
        if (ColumnsAreVectors(matA, matB, matC, opB, t)) {
            // (GetBufferSize counted this region for these operands)
            const int64_t off = Align256(matA->spmm.plan.bytes + matA->spmm.stagingBytes);
            const size_t bytes = opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
            OpsparseSpmvPlan vectorPlan{};
            const int rc = opsparse_spmv_csr_analyse(static_cast<const int32_t *>(matA->rowOffsets), matA->rows,
                                                     matA->cols, matA->nnz, static_cast<unsigned char *>(buffer) + off,
                                                     bytes, OPSPARSE_SPMV_AUTO, &vectorPlan,
                                                     handle != nullptr ? handle->stream : nullptr);
            if (rc == OPSPARSE_OK) {
                matA->spmm.vectorPlan = vectorPlan;
                matA->spmm.vectorOff = off;
                matA->spmm.vectorBytes = static_cast<int64_t>(bytes);
            }
        }
    }
    return built;
}

aclsparseStatus_t aclsparseSpMM(aclsparseHandle_t handle, aclsparseOperation_t opA, aclsparseOperation_t opB,
                                const void *alpha, aclsparseConstSpMatDescr_t matA,
                                aclsparseConstDnMatDescr_t matB, const void *beta, aclsparseDnMatDescr_t matC,
                                aclDataType computeType, aclsparseSpMMAlg_t alg, void *buffer)
{
    SpmmTypes t{};
    aclsparseStatus_t st = Validate(matA, matB, matC, opA, opB, computeType, alg, &t);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (buffer == nullptr) {
        return ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES;
    }
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    // Staged copies of B / C only in a buffer that Preprocess was given for operands needing at least as much:
    // nothing else says how large the buffer is.  A buffer that is not the one bound to matA is preprocessed first
    // (spmm_host.cpp:310-321), without a staging area.
    const Staging g = MakeStaging(matA, matB, matC, opB, t, matA->spmm.plan.bytes);
    const bool bound = matA->spmm.buffer == buffer && matA->spmm.plan.rows == matA->rows &&
                       matA->spmm.plan.nnz == matA->nnz;
    bool staged = bound && g.bytes > 0 && g.bytes <= matA->spmm.stagingBytes && matA->spmm.plan.n == g.nPadded &&
                  matA->nnz > 0;
    const OpsparseSpmmPlan *plan = &matA->spmm.plan;
    // A few row-major fp32 columns under a plan cut for the kernel for narrow B: that kernel reads and writes rows of
    // any width up to 8, leading dimension and 4-byte alignment where they are, and the copies through the staging
    // area are saved.
    const bool direct = staged && opB == ACL_SPARSE_OP_NON_TRANSPOSE && matB->order == ACL_SPARSE_ORDER_ROW &&
                        matC->order == ACL_SPARSE_ORDER_ROW &&
                        opsparse_spmm_csr_narrow_rows(plan, buffer, matC->cols, matA->nnz, t.valType, t.cType) != 0;
    if (direct) {
        staged = false;
    }
    if (!direct && !staged && (!bound || matA->spmm.plan.n != matC->cols)) {
        // The analysis reads two numbers back and synchronises, which a stream under capture must not: such a call
        // runs without a plan (a lane group per row, no tables), like the raw launch layer with plan == NULL.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(handle->stream, &capturing) != hipSuccess ||
            capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            plan = nullptr;
        } else if (bound && matC->cols > matA->spmm.widestN) {
            // The bound buffer was sized for a narrower C: the tables of a wider one (8 bytes per long-row segment
            // and column) need not fit it, and nothing says how large it is.  Without tables, then.
            plan = nullptr;
        } else {
            st = BuildPlan(matA, matC->cols, ElementBytes(t.valType), buffer, handle->stream);
            if (st != ACL_SPARSE_STATUS_SUCCESS) {
                return st;
            }
        }
    }
    // NULL scalars read as 0 (spmm_host.cpp:62-74).
    const OpsparseScalar a = opsparse::MakeScalar(alpha, computeType, handle->pointerMode, 0.0);
    const OpsparseScalar b = opsparse::MakeScalar(beta, computeType, handle->pointerMode, 0.0);
    int rc;
    const OpsparseSpmmBinding &bind = matA->spmm;
    if (bound && bind.vectorOff > 0 && bind.vectorPlan.rows == matA->rows && bind.vectorPlan.nnz == matA->nnz &&
        ColumnsAreVectors(matA, matB, matC, opB, t)) {
        const int64_t bStep = matB->order == ACL_SPARSE_ORDER_COL ? matB->ld : 0;
        const int64_t cStep = matC->order == ACL_SPARSE_ORDER_COL ? matC->ld : 0;
        rc = OPSPARSE_OK;
        for (int64_t j = 0; j < matC->cols && rc == OPSPARSE_OK; ++j) {
            const auto *x = static_cast<const unsigned char *>(matB->values) + j * bStep * ElementBytes(t.valType);
            auto *y = static_cast<unsigned char *>(matC->values) + j * cStep * ElementBytes(t.cType);
            rc = opsparse_spmv_csr_launch_zy(&bind.vectorPlan, 0, static_cast<const int32_t *>(matA->rowOffsets),
                                             static_cast<const int32_t *>(matA->colInd), matA->values, x, y, y,
                                             matA->rows, matA->cols, matA->nnz, a, b, t.valType, t.cType, 0,
                                             static_cast<unsigned char *>(buffer) + bind.vectorOff,
                                             static_cast<size_t>(bind.vectorBytes), handle->stream);
        }
    } else if (staged) {
        rc = RunStaged(g, matA, matB, matC, opB, a, b, t, handle->pointerMode == ACL_SPARSE_POINTER_MODE_HOST &&
                                                              beta != nullptr && ScalarIsZero(beta, computeType),
                       buffer, handle->stream);
    } else {
        rc = opsparse_spmm_csr_launch(
            plan, static_cast<const int32_t *>(matA->rowOffsets),
            static_cast<const int32_t *>(matA->colInd), matA->values, matB->values, matC->values, matA->rows,
            matA->cols, matC->cols, matA->nnz, matB->ld, matC->ld, matB->order == ACL_SPARSE_ORDER_COL ? 1 : 0,
            matC->order == ACL_SPARSE_ORDER_COL ? 1 : 0, opB == ACL_SPARSE_OP_TRANSPOSE ? 1 : 0, a, b, t.valType,
            t.cType, buffer, plan != nullptr ? static_cast<size_t>(plan->bytes) : 0, handle->stream);
    }
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMM: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

}  // extern "C"
