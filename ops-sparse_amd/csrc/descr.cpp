// CSR, dense-vector and dense-matrix descriptors: plain host objects that
// borrow device pointers.  Argument checks and status codes follow
// sparse/common/aclsparse_descr.cpp of the reference (DnVec :96-147, :306-368;
// CSR :370-422, :473-586; DnMat :588-743).
#include <new>

#include "internal.h"

namespace {

// reference: sparse/common/aclsparse_descr.cpp:41-66
bool KnownValueType(aclDataType t)
{
    switch (t) {
        case ACL_FLOAT:
        case ACL_FLOAT16:
        case ACL_DOUBLE:
        case ACL_INT8:
        case ACL_INT16:
        case ACL_INT32:
        case ACL_INT64:
        case ACL_UINT8:
        case ACL_UINT16:
        case ACL_UINT32:
        case ACL_UINT64:
        case ACL_BF16:
        case ACL_FLOAT8_E4M3FN:
        case ACL_FLOAT8_E5M2:
        case ACL_FLOAT4_E2M1:
        case ACL_COMPLEX64:
        case ACL_COMPLEX128:
            return true;
        default:
            return false;
    }
}

bool KnownIndexType(aclsparseIndexType_t t) { return t == ACL_SPARSE_INDEX_32I || t == ACL_SPARSE_INDEX_64I; }

bool LiveDnVec(const aclsparseDnVecDescr *d) { return d != nullptr && d->signature == opsparse::kDnVecSignature; }

}  // namespace

extern "C" {

// ------------------------------------------------------------ dense vector

aclsparseStatus_t aclsparseCreateDnVec(aclsparseDnVecDescr_t *dnVecDescr, int64_t size, void *values,
                                       aclDataType valueType)
{
    if (dnVecDescr == nullptr || size < 0 || (size > 0 && values == nullptr) || !KnownValueType(valueType)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    auto *d = new (std::nothrow) aclsparseDnVecDescr();
    if (d == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    d->signature = opsparse::kDnVecSignature;
    d->size = size;
    d->values = values;
    d->valueType = valueType;
    *dnVecDescr = d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseCreateConstDnVec(aclsparseConstDnVecDescr_t *dnVecDescr, int64_t size,
                                            const void *values, aclDataType valueType)
{
    if (dnVecDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    aclsparseDnVecDescr_t d = nullptr;
    const aclsparseStatus_t st = aclsparseCreateDnVec(&d, size, const_cast<void *>(values), valueType);
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        *dnVecDescr = d;
    }
    return st;
}

aclsparseStatus_t aclsparseDestroyDnVec(aclsparseConstDnVecDescr_t dnVecDescr)
{
    if (dnVecDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    auto *d = const_cast<aclsparseDnVecDescr *>(dnVecDescr);
    d->signature = 0;  // a stale pointer no longer passes the accessors' check
    delete d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDnVecGet(aclsparseDnVecDescr_t dnVecDescr, int64_t *size, void **values,
                                    aclDataType *valueType)
{
    if (!LiveDnVec(dnVecDescr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (size != nullptr) {
        *size = dnVecDescr->size;
    }
    if (values != nullptr) {
        *values = dnVecDescr->values;
    }
    if (valueType != nullptr) {
        *valueType = dnVecDescr->valueType;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseConstDnVecGet(aclsparseConstDnVecDescr_t dnVecDescr, int64_t *size,
                                         const void **values, aclDataType *valueType)
{
    void *v = nullptr;
    const aclsparseStatus_t st =
        aclsparseDnVecGet(const_cast<aclsparseDnVecDescr *>(dnVecDescr), size, &v, valueType);
    if (st == ACL_SPARSE_STATUS_SUCCESS && values != nullptr) {
        *values = v;
    }
    return st;
}

aclsparseStatus_t aclsparseDnVecGetValues(aclsparseDnVecDescr_t dnVecDescr, void **values)
{
    if (!LiveDnVec(dnVecDescr) || values == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *values = dnVecDescr->values;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseConstDnVecGetValues(aclsparseConstDnVecDescr_t dnVecDescr, const void **values)
{
    if (!LiveDnVec(dnVecDescr) || values == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *values = dnVecDescr->values;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDnVecSetValues(aclsparseDnVecDescr_t dnVecDescr, void *values)
{
    if (!LiveDnVec(dnVecDescr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    dnVecDescr->values = values;
    return ACL_SPARSE_STATUS_SUCCESS;
}

// ----------------------------------------------------------- sparse matrix

aclsparseStatus_t aclsparseCreateCsr(aclsparseSpMatDescr_t *spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                     void *csrRowOffsets, void *csrColInd, void *csrValues,
                                     aclsparseIndexType_t csrRowOffsetsType, aclsparseIndexType_t csrColIndType,
                                     aclsparseIndexBase_t idxBase, aclDataType valueType)
{
    if (spMatDescr == nullptr || rows < 0 || cols < 0 || nnz < 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // Any I32 / I64 mix may be described; the compute entry points narrow it.
    if (!KnownIndexType(csrRowOffsetsType) || !KnownIndexType(csrColIndType)) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    auto *d = new (std::nothrow) aclsparseSpMatDescr();
    if (d == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    d->format = ACL_SPARSE_FORMAT_CSR;
    d->rows = rows;
    d->cols = cols;
    d->nnz = nnz;
    d->rowOffsets = csrRowOffsets;
    d->colInd = csrColInd;
    d->values = csrValues;
    d->rowOffsetsType = csrRowOffsetsType;
    d->colIndType = csrColIndType;
    d->idxBase = idxBase;
    d->valueType = valueType;
    *spMatDescr = d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseCreateConstCsr(aclsparseConstSpMatDescr_t *spMatDescr, int64_t rows, int64_t cols,
                                          int64_t nnz, const void *csrRowOffsets, const void *csrColInd,
                                          const void *csrValues, aclsparseIndexType_t csrRowOffsetsType,
                                          aclsparseIndexType_t csrColIndType, aclsparseIndexBase_t idxBase,
                                          aclDataType valueType)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    aclsparseSpMatDescr_t d = nullptr;
    const aclsparseStatus_t st =
        aclsparseCreateCsr(&d, rows, cols, nnz, const_cast<void *>(csrRowOffsets), const_cast<void *>(csrColInd),
                           const_cast<void *>(csrValues), csrRowOffsetsType, csrColIndType, idxBase, valueType);
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        *spMatDescr = d;
    }
    return st;
}

aclsparseStatus_t aclsparseCsrSetPointers(aclsparseSpMatDescr_t descr, void *rowOffsets, void *colIndices,
                                          void *values)
{
    if (descr == nullptr || descr->format != ACL_SPARSE_FORMAT_CSR ||
        (rowOffsets == nullptr && descr->rows > 0 && descr->cols > 0) ||
        (descr->nnz > 0 && (colIndices == nullptr || values == nullptr))) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    descr->rowOffsets = rowOffsets;
    descr->colInd = colIndices;
    descr->values = values;
    // A different sparsity pattern may sit behind the new pointers.
    descr->spmv = OpsparseSpmvBinding{};
    descr->spmm = OpsparseSpmmBinding{};
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDestroySpMat(aclsparseConstSpMatDescr_t spMatDescr)
{
    delete const_cast<aclsparseSpMatDescr *>(spMatDescr);  // NULL is fine
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMatGetFormat(aclsparseConstSpMatDescr_t spMatDescr, aclsparseFormat_t *format)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (format != nullptr) {
        *format = spMatDescr->format;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMatGetValues(aclsparseSpMatDescr_t spMatDescr, void **values)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (values != nullptr) {
        *values = spMatDescr->values;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseConstSpMatGetValues(aclsparseConstSpMatDescr_t spMatDescr, const void **values)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (values != nullptr) {
        *values = spMatDescr->values;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMatSetValues(aclsparseSpMatDescr_t spMatDescr, void *values)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (values != spMatDescr->values) {
        // Same pattern, new numbers: preprocessing that only looked at the pattern stays valid.  The re-stored SpMV
        // layouts hold a copy of the values as they were at Preprocess: such a binding is dropped, later calls run
        // the row-wise kernels on the new array (a layout with live values reads the values at every call and stays).
        const OpsparseSpmvPlan &plan = spMatDescr->spmv.plan;
        if (plan.kernel == OPSPARSE_SPMV_COLUMN_PANELS ||
            (plan.kernel == OPSPARSE_SPMV_BLOCKED_GATHER && plan.liveValues == 0)) {
            spMatDescr->spmv = OpsparseSpmvBinding{};
        }
    }
    spMatDescr->values = values;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMatGetSize(aclsparseConstSpMatDescr_t spMatDescr, int64_t *rows, int64_t *cols,
                                        int64_t *nnz)
{
    if (spMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (rows != nullptr) {
        *rows = spMatDescr->rows;
    }
    if (cols != nullptr) {
        *cols = spMatDescr->cols;
    }
    if (nnz != nullptr) {
        *nnz = spMatDescr->nnz;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

// ------------------------------------------------------------ dense matrix

aclsparseStatus_t aclsparseCreateDnMat(aclsparseDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols, int64_t ld,
                                       void *values, aclDataType valueType, aclsparseOrder_t order)
{
    if (dnMatDescr == nullptr || rows <= 0 || cols <= 0 || ld <= 0 || values == nullptr ||
        !KnownValueType(valueType)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (order != ACL_SPARSE_ORDER_ROW && order != ACL_SPARSE_ORDER_COL) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const int64_t minLd = (order == ACL_SPARSE_ORDER_ROW) ? cols : rows;
    if (ld < minLd) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    auto *d = new (std::nothrow) aclsparseDnMatDescr();
    if (d == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    d->rows = rows;
    d->cols = cols;
    d->ld = ld;
    d->order = order;
    d->values = values;
    d->valueType = valueType;
    *dnMatDescr = d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseCreateConstDnMat(aclsparseConstDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols,
                                            int64_t ld, const void *values, aclDataType valueType,
                                            aclsparseOrder_t order)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    aclsparseDnMatDescr_t d = nullptr;
    const aclsparseStatus_t st =
        aclsparseCreateDnMat(&d, rows, cols, ld, const_cast<void *>(values), valueType, order);
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        *dnMatDescr = d;
    }
    return st;
}

aclsparseStatus_t aclsparseDestroyDnMat(aclsparseConstDnMatDescr_t dnMatDescr)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    delete const_cast<aclsparseDnMatDescr *>(dnMatDescr);
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDnMatGet(aclsparseDnMatDescr_t dnMatDescr, int64_t *rows, int64_t *cols, int64_t *ld,
                                    void **values, aclDataType *valueType, aclsparseOrder_t *order)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (rows != nullptr) {
        *rows = dnMatDescr->rows;
    }
    if (cols != nullptr) {
        *cols = dnMatDescr->cols;
    }
    if (ld != nullptr) {
        *ld = dnMatDescr->ld;
    }
    if (values != nullptr) {
        *values = dnMatDescr->values;
    }
    if (valueType != nullptr) {
        *valueType = dnMatDescr->valueType;
    }
    if (order != nullptr) {
        *order = dnMatDescr->order;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseConstDnMatGet(aclsparseConstDnMatDescr_t dnMatDescr, int64_t *rows, int64_t *cols,
                                         int64_t *ld, const void **values, aclDataType *valueType,
                                         aclsparseOrder_t *order)
{
    void *v = nullptr;
    const aclsparseStatus_t st =
        aclsparseDnMatGet(const_cast<aclsparseDnMatDescr *>(dnMatDescr), rows, cols, ld, &v, valueType, order);
    if (st == ACL_SPARSE_STATUS_SUCCESS && values != nullptr) {
        *values = v;
    }
    return st;
}

aclsparseStatus_t aclsparseDnMatGetValues(aclsparseDnMatDescr_t dnMatDescr, void **values)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (values != nullptr) {
        *values = dnMatDescr->values;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseConstDnMatGetValues(aclsparseConstDnMatDescr_t dnMatDescr, const void **values)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (values != nullptr) {
        *values = dnMatDescr->values;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDnMatSetValues(aclsparseDnMatDescr_t dnMatDescr, void *values)
{
    if (dnMatDescr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    dnMatDescr->values = values;
    return ACL_SPARSE_STATUS_SUCCESS;
}

}  // extern "C"
