// The aclsparseSpMVOp_* API: Z = alpha * A * X + beta * Y through a descriptor
// and a plan object.
//
// Argument checks, their order and status codes follow the reference
// (sparse/spmv_op/arch35/spmv_op_host.cpp: validation :64-297, bufferSize
// :496-541, createDescr :603-647, createPlan :660-686, execute :726-746 with the
// m == 0 / nnz == 0 short cuts of :465-486).  What differs is underneath: the
// reference runs one thread per row with a compensated dot product and, for
// ALG2, a device-side sort of the rows; here every algorithm value runs the
// fp64-accumulating SpMV kernels, which are deterministic.  64-bit row offsets
// and index base 1 reach the same kernels: the descriptor owns a 32-bit
// zero-based copy of the row offsets (rewritten from the caller's at every
// ALG1 execution, once for ALG2), and one-based column indices are used as they
// are with x - 1 in place of x.  ALG2's buffer holds
// what its analysis leaves: the merge-path partition (the nnz-balanced split
// that ALG2 asks for) or, for a wide matrix with scattered columns, the
// re-stored blocked-gather / column-panel layout.  ALG1 has no buffer: its
// first execution reads the row lengths once and later ones run the row-wise
// kernel they select.
#include <climits>
#include <new>

#include "internal.h"

// reference: sparse/common/aclsparse_descr_internal.h:139-158
struct aclsparseSpMVOpDescr {
    int64_t rows = 0;
    int64_t cols = 0;
    int64_t nnz = 0;
    aclsparseIndexBase_t indexBase = ACL_SPARSE_INDEX_BASE_ZERO;
    aclsparseIndexType_t rowOffsetsType = ACL_SPARSE_INDEX_32I;
    void *rowOffsets = nullptr;  // borrowed, like the matrix descriptor's
    void *colInd = nullptr;
    void *values = nullptr;
    aclsparseSpMVOpAlg_t alg = ACL_SPARSE_SPMVOP_ALG1;
    void *userBuffer = nullptr;  // ALG2: caller's buffer holding the partition
    bool planned = false;        // plan is valid (ALG2: userBuffer was analysed; ALG1: a row-wise kernel, no buffer)
    OpsparseSpmvPlan plan{};
    int32_t *offsets32 = nullptr;  // owned: the row offsets as int32, zero-based (64-bit offsets or index base 1 only)
};

struct aclsparseSpMVOpPlan {
    aclsparseSpMVOpDescr *descr = nullptr;
    // ALG1 has no buffer, but the row-wise kernels keep nothing in one: the first execution looks at the row
    // lengths once (one short kernel and a synchronisation) and later ones run the kernel they select.
    bool rowsLooked = false;
    bool rowsPlanned = false;
    OpsparseSpmvPlan rowsPlan{};
};

namespace {

aclsparseStatus_t ValidateMatrix(aclsparseConstSpMatDescr_t matA)
{
    if (matA == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (matA->format != ACL_SPARSE_FORMAT_CSR || matA->valueType != ACL_FLOAT) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    // row offsets may be 32 or 64 bit, column indices must be 32 bit
    if (matA->colIndType != ACL_SPARSE_INDEX_32I) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (matA->rowOffsetsType != ACL_SPARSE_INDEX_32I && matA->rowOffsetsType != ACL_SPARSE_INDEX_64I) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t ValidateCommon(aclsparseOperation_t opA, aclDataType computeType)
{
    if (opA != ACL_SPARSE_OP_NON_TRANSPOSE || computeType != ACL_FLOAT) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t ValidateAlg(aclsparseSpMVOpAlg_t alg)
{
    if (alg != ACL_SPARSE_SPMVOP_ALG_DEFAULT && alg != ACL_SPARSE_SPMVOP_ALG1 && alg != ACL_SPARSE_SPMVOP_ALG2) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

// The optimised kernels take 32-bit zero-based offsets.
bool Plain(const aclsparseSpMVOpDescr *d)
{
    return d->rowOffsetsType == ACL_SPARSE_INDEX_32I && d->indexBase == ACL_SPARSE_INDEX_BASE_ZERO;
}

// What they are given: the caller's offsets, or the descriptor's rebased copy of them.
const int32_t *Offsets32(const aclsparseSpMVOpDescr *d)
{
    return d->offsets32 != nullptr ? d->offsets32 : static_cast<const int32_t *>(d->rowOffsets);
}

int Rebase(const aclsparseSpMVOpDescr *d, hipStream_t stream)
{
    return opsparse_rebase_offsets_launch(d->rowOffsets, d->rowOffsetsType == ACL_SPARSE_INDEX_64I ? 1 : 0,
                                          d->indexBase == ACL_SPARSE_INDEX_BASE_ONE ? 1 : 0, d->rows + 1, d->offsets32,
                                          stream);
}

// First execution of an unplanned descriptor (ALG1): the row statistics into the handle's workspace.  A plan for
// the stream-rows or vector-rows kernel is kept (the 2048 x 2048 Laplacian: 41 us a call against 71 us for the
// merge path); a merge-path plan would live in that workspace, which other calls overwrite, and is dropped.
// Not under stream capture: the analysis synchronises.
void LookAtRows(aclsparseHandle_t handle, aclsparseSpMVOpPlan *plan)
{
    const aclsparseSpMVOpDescr *d = plan->descr;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(handle->stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return;  // looked at again by the next execution outside a capture
    }
    plan->rowsLooked = true;
    if (handle->workspaceBytes() < opsparse_spmv_csr_workspace_bytes(d->rows, d->nnz)) {
        return;
    }
    OpsparseSpmvPlan p{};
    const int rc = opsparse_spmv_csr_analyse(Offsets32(d), d->rows, d->cols, d->nnz, handle->workspace(),
                                             handle->workspaceBytes(), OPSPARSE_SPMV_AUTO, &p, handle->stream);
    if (rc == OPSPARSE_OK && (p.kernel == OPSPARSE_SPMV_STREAM_ROWS || p.kernel == OPSPARSE_SPMV_VECTOR_ROWS)) {
        plan->rowsPlan = p;
        plan->rowsPlan.guardTiles = 1;
        plan->rowsPlanned = true;
    }
}

// ALG2's device-side reorder is, for a matrix whose x does not fit an L2, a re-stored layout (blocked gather,
// else column panels): the buffer then holds a copy of the matrix (indices and values), which is why csrValues
// must not change under an ALG2 descriptor (reference include/cann_ops_sparse.h:64-69 says the same of its
// own ALG2).
// ALG1 / DEFAULT on a plain fp32 matrix whose gathers are scattered: the blocked-gather layout with live values,
// as under aclsparseSpMVPreprocess with the default algorithm — if the caller brings the buffer that
// aclsparseSpMVOp_bufferSize then asks for.  csrValues may change between executions, as ALG1 allows.
opsparse::RestoredChoice LiveLayout(aclsparseHandle_t handle, aclsparseConstSpMatDescr_t matA)
{
    if (matA->rowOffsetsType != ACL_SPARSE_INDEX_32I || matA->idxBase != ACL_SPARSE_INDEX_BASE_ZERO ||
        matA->valueType != ACL_FLOAT || matA->values == nullptr) {
        return {0, 0, false};
    }
    return opsparse::PickLiveLayout(handle, static_cast<const int32_t *>(matA->rowOffsets),
                                    static_cast<const int32_t *>(matA->colInd), matA->rows, matA->cols, matA->nnz,
                                    false, OPSPARSE_F32, /*repeatable=*/true);
}

opsparse::RestoredChoice RestoredLayout(aclsparseConstSpMatDescr_t matA)
{
    if (matA->rowOffsetsType != ACL_SPARSE_INDEX_32I || matA->idxBase != ACL_SPARSE_INDEX_BASE_ZERO) {
        return {0, 0, false};
    }
    return opsparse::PickRestoredLayout(matA->rows, matA->cols, matA->nnz, false, OPSPARSE_F32);
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

}  // namespace

extern "C" {

aclsparseStatus_t aclsparseSpMVOp_bufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t /*vecX*/,
                                             aclsparseConstDnVecDescr_t /*vecY*/, aclsparseDnVecDescr_t /*vecZ*/,
                                             aclDataType computeType, aclsparseSpMVOpAlg_t alg, size_t *bufferSize)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    aclsparseStatus_t st = ValidateCommon(opA, computeType);
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        st = ValidateMatrix(matA);
    }
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        st = ValidateAlg(alg);
    }
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (bufferSize == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (matA->rows > INT32_MAX) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    // ALG1 / DEFAULT need no buffer, but use one for a matrix with scattered gathers; ALG2 keeps its partition, or
    // its copy of the matrix, in one.
    *bufferSize = 0;
    if (alg == ACL_SPARSE_SPMVOP_ALG2) {
        const size_t plain = opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
        opsparse::RestoredChoice restored = RestoredLayout(matA);
        opsparse::TrimToWorkspace(handle, &restored, matA->rows, matA->cols, matA->nnz, false, OPSPARSE_F32);
        opsparse::RememberSized(matA, restored, false, OPSPARSE_F32);
        *bufferSize = restored.keep > plain ? restored.keep : plain;
    } else {
        opsparse::RestoredChoice live = LiveLayout(handle, matA);
        opsparse::TrimToWorkspace(handle, &live, matA->rows, matA->cols, matA->nnz, false, OPSPARSE_F32);
        opsparse::RememberSized(matA, live, false, OPSPARSE_F32);
        *bufferSize = live.keep;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVOp_createDescr(aclsparseHandle_t handle, aclsparseSpMVOpDescr_t *descr,
                                              aclsparseOperation_t opA, aclsparseConstSpMatDescr_t matA,
                                              aclsparseConstDnVecDescr_t /*vecX*/, aclsparseConstDnVecDescr_t /*vecY*/,
                                              aclsparseDnVecDescr_t /*vecZ*/, aclDataType computeType,
                                              aclsparseSpMVOpAlg_t alg, void *buffer)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (descr == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    aclsparseStatus_t st = ValidateMatrix(matA);
    if (st == ACL_SPARSE_STATUS_SUCCESS) {
        st = ValidateAlg(alg);
    }
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (alg == ACL_SPARSE_SPMVOP_ALG2 && buffer == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    st = ValidateCommon(opA, computeType);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (matA->rows > INT32_MAX) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (matA->idxBase != ACL_SPARSE_INDEX_BASE_ZERO && matA->idxBase != ACL_SPARSE_INDEX_BASE_ONE) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    auto *d = new (std::nothrow) aclsparseSpMVOpDescr();
    if (d == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    d->rows = matA->rows;
    d->cols = matA->cols;
    d->nnz = matA->nnz;
    d->indexBase = matA->idxBase;
    d->rowOffsetsType = matA->rowOffsetsType;
    d->rowOffsets = matA->rowOffsets;
    d->colInd = matA->colInd;
    d->values = matA->values;
    d->alg = (alg == ACL_SPARSE_SPMVOP_ALG_DEFAULT) ? ACL_SPARSE_SPMVOP_ALG1 : alg;
    if (!Plain(d) && d->rows > 0 && d->nnz > 0 && d->nnz <= INT32_MAX && d->rowOffsets != nullptr) {
        // 64-bit offsets and / or index base 1: a 32-bit zero-based copy for the binned kernels
        if (hipMalloc(reinterpret_cast<void **>(&d->offsets32), sizeof(int32_t) * static_cast<size_t>(d->rows + 1)) !=
            hipSuccess) {
            (void)hipGetLastError();
            delete d;
            return ACL_SPARSE_STATUS_ALLOC_FAILED;
        }
        if (Rebase(d, handle->stream) != OPSPARSE_OK) {
            (void)hipFree(d->offsets32);
            delete d;
            return ACL_SPARSE_STATUS_EXECUTION_FAILED;
        }
    }
    if (d->alg == ACL_SPARSE_SPMVOP_ALG2) {
        d->userBuffer = buffer;
        // The nnz-balanced split of ALG2: analyse the rows into the caller's buffer.
        if ((Plain(d) || d->offsets32 != nullptr) && d->rows > 0 && d->nnz > 0 && d->rowOffsets != nullptr) {
            // (a re-stored layout only into a buffer that a size query on these arrays sized for it)
            opsparse::RestoredChoice restored = RestoredLayout(matA);
            opsparse::TrimToWorkspace(handle, &restored, matA->rows, matA->cols, matA->nnz, false, OPSPARSE_F32);
            if (!opsparse::SizedFor(matA, restored, false, OPSPARSE_F32)) {
                restored = opsparse::RestoredChoice{0, 0, false};
            }
            const int rc =
                restored.kernel != 0 && d->colInd != nullptr && d->values != nullptr
                    ? opsparse::AnalyseRestored(restored.kernel, static_cast<const int32_t *>(d->rowOffsets),
                                                static_cast<const int32_t *>(d->colInd), d->values, OPSPARSE_F32,
                                                d->rows, d->cols, d->nnz, false, false, buffer, restored.keep,
                                                restored.scratch > 0 ? handle->userWorkspace : nullptr,
                                                restored.scratch > 0 ? handle->userWorkspaceBytes : 0, &d->plan,
                                                handle->stream)
                    : opsparse_spmv_csr_analyse(Offsets32(d), d->rows, d->cols, d->nnz, buffer,
                                                opsparse_spmv_csr_workspace_bytes(d->rows, d->nnz), OPSPARSE_SPMV_AUTO,
                                                &d->plan, handle->stream);
            if (rc != OPSPARSE_OK) {
                (void)hipFree(d->offsets32);
                delete d;
                return FromLaunch(rc);
            }
            d->planned = true;
        }
    }
    if (d->alg != ACL_SPARSE_SPMVOP_ALG2 && buffer != nullptr && Plain(d) && d->rows > 0 && d->nnz > 0) {
        // the buffer aclsparseSpMVOp_bufferSize asked for (it asks the same question of the same arrays)
        opsparse::RestoredChoice live = LiveLayout(handle, matA);
        opsparse::TrimToWorkspace(handle, &live, matA->rows, matA->cols, matA->nnz, false, OPSPARSE_F32);
        if (live.kernel != 0 && opsparse::SizedFor(matA, live, false, OPSPARSE_F32)) {
            const int rc = opsparse::AnalyseRestored(live.kernel, static_cast<const int32_t *>(d->rowOffsets),
                                                     static_cast<const int32_t *>(d->colInd), d->values, OPSPARSE_F32,
                                                     d->rows, d->cols, d->nnz, false, true, buffer, live.keep,
                                                     live.scratch > 0 ? handle->userWorkspace : nullptr,
                                                     live.scratch > 0 ? handle->userWorkspaceBytes : 0, &d->plan,
                                                     handle->stream);
            if (rc != OPSPARSE_OK) {
                delete d;
                return FromLaunch(rc);
            }
            d->userBuffer = buffer;
            d->planned = true;
        }
    }
    *descr = d;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVOp_destroyDescr(aclsparseSpMVOpDescr_t descr)
{
    if (descr != nullptr && descr->offsets32 != nullptr) {
        (void)hipFree(descr->offsets32);  // waits for the work that still reads it
    }
    delete descr;  // NULL is fine
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVOp_createPlan(aclsparseHandle_t handle, aclsparseSpMVOpDescr_t descr,
                                             aclsparseSpMVOpPlan_t *plan, const void *epilogueLTOBuffer,
                                             size_t epilogueLTOBufferSize)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (descr == nullptr || plan == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // Only the identity epilogue exists: a link-time-optimised one is refused.
    if (epilogueLTOBuffer != nullptr || epilogueLTOBufferSize > 0) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    auto *p = new (std::nothrow) aclsparseSpMVOpPlan();
    if (p == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    p->descr = descr;
    *plan = p;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVOp_destroyPlan(aclsparseSpMVOpPlan_t plan)
{
    delete plan;  // NULL is fine
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVOp_setGlobalUserData(aclsparseHandle_t handle, aclsparseSpMVOpPlan_t plan,
                                                    const char * /*epilogueDataName*/, void *epilogueData,
                                                    size_t epilogueDataSize)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (plan == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if ((epilogueData == nullptr) != (epilogueDataSize == 0)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    return ACL_SPARSE_STATUS_SUCCESS;  // the identity epilogue uses no data
}

aclsparseStatus_t aclsparseSpMVOp(aclsparseHandle_t handle, aclsparseSpMVOpPlan_t plan, const void *alpha,
                                  const void *beta, aclsparseConstDnVecDescr_t vecX,
                                  aclsparseConstDnVecDescr_t vecY, aclsparseDnVecDescr_t vecZ)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (plan == nullptr || plan->descr == nullptr || alpha == nullptr || beta == nullptr || vecX == nullptr ||
        vecY == nullptr || vecZ == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseSpMVOpDescr *d = plan->descr;
    if (vecX->valueType != ACL_FLOAT || vecY->valueType != ACL_FLOAT || vecZ->valueType != ACL_FLOAT) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (d->cols > 0 && vecX->values == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // Y may be absent when beta is known to be 0 on the host; in DEVICE mode the
    // kernel's own beta == 0 short cut is trusted (spmv_op_host.cpp:256-268).
    bool yMayBeNull = handle->pointerMode == ACL_SPARSE_POINTER_MODE_DEVICE;
    if (handle->pointerMode == ACL_SPARSE_POINTER_MODE_HOST) {
        yMayBeNull = (*static_cast<const float *>(beta) == 0.0f);
    }
    if (!yMayBeNull && d->rows > 0 && vecY->values == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (d->rows > 0 && vecZ->values == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (vecX->size != d->cols || vecY->size != d->rows || vecZ->size != d->rows) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (d->rows == 0) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    const OpsparseScalar a = opsparse::MakeScalar(alpha, ACL_FLOAT, handle->pointerMode, 0.0);
    const OpsparseScalar b = opsparse::MakeScalar(beta, ACL_FLOAT, handle->pointerMode, 0.0);
    int rc;
    if (Plain(d) || d->nnz == 0 || d->offsets32 != nullptr) {
        // index base 1: the column indices stay one-based, x - 1 stands for x (only indices that occur are read)
        const int64_t shift = (d->nnz > 0 && d->indexBase == ACL_SPARSE_INDEX_BASE_ONE) ? 1 : 0;
        const float *x = static_cast<const float *>(vecX->values) - shift;
        if (d->offsets32 != nullptr && d->nnz > 0 && d->alg != ACL_SPARSE_SPMVOP_ALG2) {
            rc = Rebase(d, handle->stream);  // ALG1 promises nothing about the offsets between executions
            if (rc != OPSPARSE_OK) {
                return FromLaunch(rc);
            }
        }
        const OpsparseSpmvPlan *p = d->planned ? &d->plan : nullptr;
        void *ws = d->planned ? d->userBuffer : nullptr;
        size_t wsBytes = d->planned ? static_cast<size_t>(d->plan.bytes) : 0;
        if (p == nullptr && d->nnz > 0) {
            const aclsparseStatus_t st = opsparse::EnsureWorkspace(handle);
            if (st != ACL_SPARSE_STATUS_SUCCESS) {
                return st;
            }
            ws = handle->workspace();
            wsBytes = handle->workspaceBytes();
            if (!plan->rowsLooked) {
                LookAtRows(handle, plan);
            }
            if (plan->rowsPlanned) {
                p = &plan->rowsPlan;
            }
        }
        // nnz == 0 needs no offsets at all: Z = beta * Y whatever their width.
        rc = opsparse_spmv_csr_launch_zy(p, 0, d->nnz > 0 ? Offsets32(d) : nullptr,
                                         static_cast<const int32_t *>(d->colInd), d->values, x, vecY->values,
                                         vecZ->values, d->rows, d->cols + shift, d->nnz, a, b, OPSPARSE_F32,
                                         OPSPARSE_F32, 0, ws, wsBytes, handle->stream);
    } else {
        rc = opsparse_spmv_csr_indexed_launch(d->rowOffsets, d->rowOffsetsType == ACL_SPARSE_INDEX_64I ? 1 : 0,
                                              d->indexBase == ACL_SPARSE_INDEX_BASE_ONE ? 1 : 0,
                                              static_cast<const int32_t *>(d->colInd),
                                              static_cast<const float *>(d->values),
                                              static_cast<const float *>(vecX->values),
                                              static_cast<const float *>(vecY->values),
                                              static_cast<float *>(vecZ->values), d->rows, d->cols, d->nnz, a, b,
                                              handle->stream);
    }
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMVOp: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

}  // extern "C"
