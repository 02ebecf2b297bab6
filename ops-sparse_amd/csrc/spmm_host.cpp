// aclsparseSpMMGetBufferSize / aclsparseSpMMPreprocess / aclsparseSpMM.
//
// Validation order and status codes follow the reference's arch35 host code
// (sparse/spmm/arch35/spmm_host.cpp:152-191 for the shared checks, :213-234,
// :335-362, :364-394 for the three entry points).  Not carried over: the
// synchronous device<->host round trip of the tiling struct on every SpMM call
// (:281-308); alpha / beta travel as kernel arguments instead.
#include <climits>

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

// Row statistics and long-row tables into `buffer`; binds the buffer to A.
aclsparseStatus_t BuildPlan(const aclsparseSpMatDescr *A, const aclsparseDnMatDescr *C, void *buffer,
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
    size_t bytes = 0;
    int rc = opsparse_spmm_csr_workspace_bytes(static_cast<const int32_t *>(A->rowOffsets), A->rows, A->nnz, C->cols,
                                               stream, &bytes);
    if (rc != OPSPARSE_OK) {
        return FromLaunch(rc);
    }
    rc = opsparse_spmm_csr_analyse(static_cast<const int32_t *>(A->rowOffsets), A->rows, A->nnz, C->cols,
                                             buffer, bytes, OPSPARSE_SPMM_AUTO, &plan, stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMM: analysis failed (%d)", rc);
        return FromLaunch(rc);
    }
    A->spmm.buffer = buffer;
    A->spmm.plan = plan;
    return ACL_SPARSE_STATUS_SUCCESS;
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
                                                     matA->nnz, matC->cols,
                                                     handle != nullptr ? handle->stream : nullptr, size);
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
    return BuildPlan(matA, matC, buffer, handle != nullptr ? handle->stream : nullptr);
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
    // A buffer that is not the one bound to matA is preprocessed first
    // (spmm_host.cpp:310-321).
    if (matA->spmm.buffer != buffer || matA->spmm.plan.rows != matA->rows || matA->spmm.plan.nnz != matA->nnz ||
        matA->spmm.plan.n != matC->cols) {
        st = BuildPlan(matA, matC, buffer, handle->stream);
        if (st != ACL_SPARSE_STATUS_SUCCESS) {
            return st;
        }
    }
    // NULL scalars read as 0 (spmm_host.cpp:62-74).
    const OpsparseScalar a = opsparse::MakeScalar(alpha, computeType, handle->pointerMode, 0.0);
    const OpsparseScalar b = opsparse::MakeScalar(beta, computeType, handle->pointerMode, 0.0);
    const int rc = opsparse_spmm_csr_launch(
        &matA->spmm.plan, static_cast<const int32_t *>(matA->rowOffsets), static_cast<const int32_t *>(matA->colInd),
        matA->values, matB->values, matC->values, matA->rows, matA->cols, matC->cols, matA->nnz, matB->ld, matC->ld,
        matB->order == ACL_SPARSE_ORDER_COL ? 1 : 0, matC->order == ACL_SPARSE_ORDER_COL ? 1 : 0,
        opB == ACL_SPARSE_OP_TRANSPOSE ? 1 : 0, a, b, t.valType, t.cType, buffer,
        static_cast<size_t>(matA->spmm.plan.bytes), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMM: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

}  // extern "C"
