// CSR producers of the aclsparse API: aclsparseXcoo2csr, aclsparseXcsr2coo,
// aclsparseXcsrsort / Xcscsort (+_bufferSizeExt), aclsparseXcoosortByRow / ByColumn (+_bufferSizeExt),
// aclsparseCsr2cscEx2(+_bufferSize) and the
// legacy matrix descriptor that csrsort takes its index base from.
//
// Argument checks, their order and status codes follow the reference's host
// files (sparse/coo2csr/arch35/coo2csr_host.cpp:38-80,
// sparse/csr2coo/arch35/csr2coo_host.cpp:66-115,
// sparse/csrsort/arch35/csrsort_host.cpp:53-74, :146-221,
// sparse/csr2csc_ex2/arch35/csr2csc_ex2_host.cpp:109-232, :535-618,
// sparse/common/aclsparse_matdescr.cpp:25-110).  Buffer sizes are this
// library's own: the buffers' contents are opaque in both implementations.
#include <climits>
#include <new>

#include "internal.h"

// reference: sparse/common/aclsparse_descr_internal.h (legacy MatDescr)
struct aclsparseMatDescr {
    aclsparseMatrixType_t type = ACL_SPARSE_MATRIX_TYPE_GENERAL;
    aclsparseIndexBase_t indexBase = ACL_SPARSE_INDEX_BASE_ZERO;
    aclsparseDiagType_t diagType = ACL_SPARSE_DIAG_TYPE_NON_UNIT;
    aclsparseFillMode_t fillMode = ACL_SPARSE_FILL_MODE_LOWER;
};

namespace {

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

bool ValidBase(aclsparseIndexBase_t b)
{
    return b == ACL_SPARSE_INDEX_BASE_ZERO || b == ACL_SPARSE_INDEX_BASE_ONE;
}

int32_t ValueBytes(aclDataType t)
{
    switch (t) {
        case ACL_INT8: return 1;
        case ACL_FLOAT16:
        case ACL_BF16: return 2;
        case ACL_FLOAT: return 4;
        default: return 0;
    }
}

aclsparseStatus_t CsrsortCommon(int m, int n, int nnz, const int *csrRowPtr, const int *csrColInd)
{
    if (m < 0 || n < 0 || nnz < 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((m == 0 || n == 0) && nnz != 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((m > 0 && csrRowPtr == nullptr) || (nnz > 0 && csrColInd == nullptr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t Csr2cscCommon(aclsparseHandle_t handle, int m, int n, int nnz, aclDataType valType,
                                aclsparseAction_t copyValues, aclsparseIndexBase_t idxBase, aclsparseCsr2CscAlg_t alg)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (m < 0 || n < 0 || n > INT32_MAX - 1 || nnz < 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (ValueBytes(valType) == 0) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (copyValues != ACL_SPARSE_ACTION_SYMBOLIC && copyValues != ACL_SPARSE_ACTION_NUMERIC) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (!ValidBase(idxBase)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (alg != ACL_SPARSE_CSR2CSC_ALG_DEFAULT && alg != ACL_SPARSE_CSR2CSC_ALG1) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

// ------------------------------------------------------------ legacy MatDescr

aclsparseStatus_t aclsparseCreateMatDescr(aclsparseMatDescr_t *descr)
{
    if (descr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    auto *d = new (std::nothrow) aclsparseMatDescr();
    if (d == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    *descr = d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDestroyMatDescr(aclsparseMatDescr_t descr)
{
    delete descr;  // NULL gives SUCCESS
    return ACL_SPARSE_STATUS_SUCCESS;
}

void aclsparseSetMatType(aclsparseMatDescr_t descr, aclsparseMatrixType_t type)
{
    if (descr != nullptr) {
        descr->type = type;
    }
}
void aclsparseSetMatIndexBase(aclsparseMatDescr_t descr, aclsparseIndexBase_t base)
{
    if (descr != nullptr) {
        descr->indexBase = base;
    }
}
void aclsparseSetMatDiagType(aclsparseMatDescr_t descr, aclsparseDiagType_t diagType)
{
    if (descr != nullptr) {
        descr->diagType = diagType;
    }
}
void aclsparseSetMatFillMode(aclsparseMatDescr_t descr, aclsparseFillMode_t fillMode)
{
    if (descr != nullptr) {
        descr->fillMode = fillMode;
    }
}
aclsparseMatrixType_t aclsparseGetMatType(aclsparseMatDescr_t descr)
{
    return descr != nullptr ? descr->type : ACL_SPARSE_MATRIX_TYPE_GENERAL;
}
aclsparseIndexBase_t aclsparseGetMatIndexBase(aclsparseMatDescr_t descr)
{
    return descr != nullptr ? descr->indexBase : ACL_SPARSE_INDEX_BASE_ZERO;
}
aclsparseDiagType_t aclsparseGetMatDiagType(aclsparseMatDescr_t descr)
{
    return descr != nullptr ? descr->diagType : ACL_SPARSE_DIAG_TYPE_NON_UNIT;
}
aclsparseFillMode_t aclsparseGetMatFillMode(aclsparseMatDescr_t descr)
{
    return descr != nullptr ? descr->fillMode : ACL_SPARSE_FILL_MODE_LOWER;
}

// ------------------------------------------------------------------ coo2csr

aclsparseStatus_t aclsparseXcoo2csr(aclsparseHandle_t handle, const int *cooRowInd, int nnz, int m, int *csrRowPtr,
                                    aclsparseIndexBase_t idxBase)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (nnz < 0 || (nnz == INT32_MAX && idxBase == ACL_SPARSE_INDEX_BASE_ONE) || m < 0 || (nnz > 0 && m == 0) ||
        !ValidBase(idxBase) || (nnz > 0 && cooRowInd == nullptr) || csrRowPtr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseStatus_t st = opsparse::EnsureWorkspace(handle);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    const int rc = opsparse_coo2csr_launch(cooRowInd, nnz, m, csrRowPtr, static_cast<int32_t>(idxBase),
                                           handle->workspace(), handle->workspaceBytes(), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseXcoo2csr: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

// ------------------------------------------------------------------ csr2coo

aclsparseStatus_t aclsparseXcsr2coo(aclsparseHandle_t handle, const int32_t *csrRowPtr, int64_t nnz, int64_t m,
                                    int32_t *cooRowInd, aclsparseIndexBase_t idxBase)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_NOT_INITIALIZED;  // this entry point's own code for a null handle
    }
    if (nnz < 0 || m < 0 || (m == 0 && nnz != 0) || !ValidBase(idxBase) || (m > 0 && csrRowPtr == nullptr) ||
        (nnz > 0 && cooRowInd == nullptr) || nnz > INT32_MAX || m > INT32_MAX) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (nnz == 0) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    const int rc = opsparse_csr2coo_launch(csrRowPtr, nnz, m, cooRowInd, static_cast<int32_t>(idxBase), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseXcsr2coo: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

// ------------------------------------------------------------------ csrsort

aclsparseStatus_t aclsparseXcsrsort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz,
                                                  const int *csrRowPtr, const int *csrColInd,
                                                  size_t *pBufferSizeInBytes)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (pBufferSizeInBytes == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseStatus_t st = CsrsortCommon(m, n, nnz, csrRowPtr, csrColInd);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    *pBufferSizeInBytes = opsparse_csrsort_workspace_bytes(m, nnz);  // 0 when nnz == 0
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseXcsrsort(aclsparseHandle_t handle, int m, int n, int nnz, const aclsparseMatDescr_t descrA,
                                    const int *csrRowPtr, int *csrColInd, int *P, void *pBuffer)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    const aclsparseStatus_t st = CsrsortCommon(m, n, nnz, csrRowPtr, csrColInd);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (descrA == nullptr || !ValidBase(descrA->indexBase)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (nnz == 0) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    if (P == nullptr || pBuffer == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const int rc = opsparse_csrsort_launch(m, n, nnz, static_cast<int32_t>(descrA->indexBase), csrRowPtr, csrColInd, P,
                                           pBuffer, opsparse_csrsort_workspace_bytes(m, nnz), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseXcsrsort: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

// ------------------------------------------------------------------ cscsort

// reference: sparse/cscsort/arch35/cscsort_host.cpp:52-72
static aclsparseStatus_t CscsortCommon(int m, int n, int nnz, const int *cscColPtr, const int *cscRowInd)
{
    if (m < 0 || n < 0 || nnz < 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((m == 0 || n == 0) && nnz != 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((n > 0 && cscColPtr == nullptr) || (nnz > 0 && cscRowInd == nullptr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseXcscsort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz,
                                                  const int *cscColPtr, const int *cscRowInd,
                                                  size_t *pBufferSizeInBytes)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (pBufferSizeInBytes == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseStatus_t st = CscsortCommon(m, n, nnz, cscColPtr, cscRowInd);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    *pBufferSizeInBytes = opsparse_csrsort_workspace_bytes(n, nnz);  // the columns take the rows' part; 0 when nnz == 0
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseXcscsort(aclsparseHandle_t handle, int m, int n, int nnz, const aclsparseMatDescr_t descrA,
                                    const int *cscColPtr, int *cscRowInd, int *P, void *pBuffer)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    const aclsparseStatus_t st = CscsortCommon(m, n, nnz, cscColPtr, cscRowInd);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (descrA == nullptr || !ValidBase(descrA->indexBase)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (nnz == 0) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    if (P == nullptr || pBuffer == nullptr || reinterpret_cast<uintptr_t>(pBuffer) % 128U != 0U) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // a CSC matrix is the CSR form of its transpose: n "rows" whose "column" indices lie below m
    const int rc = opsparse_csrsort_launch(n, m, nnz, static_cast<int32_t>(descrA->indexBase), cscColPtr, cscRowInd, P,
                                           pBuffer, opsparse_csrsort_workspace_bytes(n, nnz), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseXcscsort: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

// ------------------------------------------------------------------ coosort

// reference: sparse/coosort/arch35/coosort_host.cpp:48-78
static aclsparseStatus_t CoosortCommon(int m, int n, int nnz, const int *cooRowsA, const int *cooColsA)
{
    if (m <= 0 || n <= 0 || nnz < 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (nnz > 0 && (cooRowsA == nullptr || cooColsA == nullptr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseXcoosort_bufferSizeExt(aclsparseHandle_t handle, int m, int n, int nnz, const int *cooRowsA,
                                                  const int *cooColsA, size_t *pBufferSizeInBytes)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (pBufferSizeInBytes == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseStatus_t st = CoosortCommon(m, n, nnz, cooRowsA, cooColsA);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    *pBufferSizeInBytes = opsparse_coosort_workspace_bytes(nnz);  // 0 when nnz == 0
    return ACL_SPARSE_STATUS_SUCCESS;
}

static aclsparseStatus_t Coosort(const char *api, aclsparseHandle_t handle, int m, int n, int nnz, int byRow,
                                 int *cooRowsA, int *cooColsA, int *P, void *pBuffer)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    const aclsparseStatus_t st = CoosortCommon(m, n, nnz, cooRowsA, cooColsA);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (nnz == 0) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    if (P == nullptr || pBuffer == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const int rc = opsparse_coosort_launch(nnz, byRow, cooRowsA, cooColsA, P, pBuffer,
                                           opsparse_coosort_workspace_bytes(nnz), handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("%s: launch failed (%d)", api, rc);
    }
    return FromLaunch(rc);
}

aclsparseStatus_t aclsparseXcoosortByRow(aclsparseHandle_t handle, int m, int n, int nnz, int *cooRowsA, int *cooColsA,
                                         int *P, void *pBuffer)
{
    return Coosort("aclsparseXcoosortByRow", handle, m, n, nnz, 1, cooRowsA, cooColsA, P, pBuffer);
}

aclsparseStatus_t aclsparseXcoosortByColumn(aclsparseHandle_t handle, int m, int n, int nnz, int *cooRowsA,
                                            int *cooColsA, int *P, void *pBuffer)
{
    return Coosort("aclsparseXcoosortByColumn", handle, m, n, nnz, 0, cooRowsA, cooColsA, P, pBuffer);
}

// ------------------------------------------------------------------ csr2csc

aclsparseStatus_t aclsparseCsr2cscEx2_bufferSize(aclsparseHandle_t handle, int m, int n, int nnz,
                                                 const void * /*csrVal*/, const int * /*csrRowPtr*/,
                                                 const int * /*csrColInd*/, void * /*cscVal*/, int * /*cscColPtr*/,
                                                 int * /*cscRowInd*/, aclDataType valType,
                                                 aclsparseAction_t copyValues, aclsparseIndexBase_t idxBase,
                                                 aclsparseCsr2CscAlg_t alg, size_t *bufferSize)
{
    const aclsparseStatus_t st = Csr2cscCommon(handle, m, n, nnz, valType, copyValues, idxBase, alg);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (bufferSize == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *bufferSize = opsparse_csr2csc_workspace_bytes(m, n, nnz);  // 0 when nothing is to be moved
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseCsr2cscEx2(aclsparseHandle_t handle, int m, int n, int nnz, const void *csrVal,
                                      const int *csrRowPtr, const int *csrColInd, void *cscVal, int *cscColPtr,
                                      int *cscRowInd, aclDataType valType, aclsparseAction_t copyValues,
                                      aclsparseIndexBase_t idxBase, aclsparseCsr2CscAlg_t alg, void *buffer)
{
    aclsparseStatus_t st = Csr2cscCommon(handle, m, n, nnz, valType, copyValues, idxBase, alg);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    const bool numeric = copyValues == ACL_SPARSE_ACTION_NUMERIC;
    if ((m > 0 && csrRowPtr == nullptr) || (nnz > 0 && csrColInd == nullptr) ||
        (nnz > 0 && numeric && csrVal == nullptr) || cscColPtr == nullptr || (nnz > 0 && cscRowInd == nullptr) ||
        (nnz > 0 && numeric && cscVal == nullptr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((m == 0 || n == 0) && nnz > 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (nnz > INT32_MAX - static_cast<int>(idxBase)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // buffer == NULL falls back to the handle's workspace when that is large enough.
    void *ws = buffer;
    size_t wsBytes = opsparse_csr2csc_workspace_bytes(m, n, nnz);
    if (nnz > 0 && ws == nullptr) {
        st = opsparse::EnsureWorkspace(handle);
        if (st != ACL_SPARSE_STATUS_SUCCESS) {
            return st;
        }
        if (handle->workspace() == nullptr || handle->workspaceBytes() < wsBytes) {
            return ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES;
        }
        ws = handle->workspace();
        wsBytes = handle->workspaceBytes();
    }
    const int rc = opsparse_csr2csc_launch(m, n, nnz, csrVal, csrRowPtr, csrColInd, cscVal, cscColPtr, cscRowInd,
                                           numeric ? ValueBytes(valType) : 0, static_cast<int32_t>(idxBase), ws,
                                           wsBytes, handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseCsr2cscEx2: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

}  // extern "C"
