// aclsparseSpMVGetBufferSize / aclsparseSpMVPreprocess / aclsparseSpMV.
//
// Argument checks, their order and their status codes follow the reference's
// aclsparseSpMV (sparse/spmv/arch22/spmv_host.cpp:121-295).  Two things the
// reference does on every call are deliberately absent: the device-to-host
// copy of the whole row-offset array with a stream synchronisation (:86-112)
// and the on-chip-buffer limit on the longest row (:244-252) — rows of any
// length are handled by the merge-path kernels.
#include <cstdlib>

#include "internal.h"

namespace {

struct SpmvCall {
    const aclsparseSpMatDescr *A;
    const aclsparseDnVecDescr *x;
    const aclsparseDnVecDescr *y;
    bool transpose;
    int32_t valType, outType, computeIsInt;
};

int32_t DtypeOf(aclDataType t)
{
    switch (t) {
        case ACL_FLOAT: return OPSPARSE_F32;
        case ACL_FLOAT16: return OPSPARSE_F16;
        case ACL_BF16: return OPSPARSE_BF16;
        case ACL_INT32: return OPSPARSE_I32;
        case ACL_INT8: return OPSPARSE_I8;
        default: return -1;
    }
}

// Checks shared by the three entry points, in the reference's order
// (spmv_host.cpp:132-179, :225-240, :266-274).
aclsparseStatus_t Validate(aclsparseHandle_t handle, aclsparseOperation_t opA, aclsparseConstSpMatDescr_t matA,
                           aclsparseConstDnVecDescr_t vecX, aclsparseConstDnVecDescr_t vecY, aclDataType computeType,
                           aclsparseSpMVAlg_t alg, SpmvCall *out)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (matA == nullptr || vecX == nullptr || vecY == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // ALG_DEFAULT is the only value the reference accepts (spmv_host.cpp:144-146).  CSR_ALG2 is accepted here
    // as well: it asks Preprocess for the column-panel layout, which copies the VALUES into the buffer.
    if (alg != ACL_SPARSE_SPMV_ALG_DEFAULT && alg != ACL_SPARSE_SPMV_CSR_ALG2) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (computeType != ACL_FLOAT && computeType != ACL_INT32) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (matA->format != ACL_SPARSE_FORMAT_CSR || matA->idxBase != ACL_SPARSE_INDEX_BASE_ZERO) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (matA->rowOffsetsType != ACL_SPARSE_INDEX_32I || matA->colIndType != ACL_SPARSE_INDEX_32I) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (opA != ACL_SPARSE_OP_NON_TRANSPOSE && opA != ACL_SPARSE_OP_TRANSPOSE) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    out->A = matA;
    out->x = vecX;
    out->y = vecY;
    out->transpose = (opA == ACL_SPARSE_OP_TRANSPOSE);
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t ValidateData(SpmvCall *c, aclDataType computeType)
{
    const aclsparseSpMatDescr *A = c->A;
    // The reference insists on all five device pointers (spmv_host.cpp:225-230);
    // arrays that hold no element (nnz == 0, an empty vector) may be NULL here.
    if (A->rowOffsets == nullptr || (A->nnz > 0 && (A->colInd == nullptr || A->values == nullptr))) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const int64_t needX = c->transpose ? A->rows : A->cols;
    const int64_t needY = c->transpose ? A->cols : A->rows;
    if ((needX > 0 && c->x->values == nullptr) || (needY > 0 && c->y->values == nullptr)) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (c->x->size < needX || c->y->size < needY) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    if (c->x->valueType != A->valueType) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    if (computeType == ACL_INT32 && (A->valueType != ACL_INT32 || c->y->valueType != ACL_INT32)) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    c->valType = DtypeOf(A->valueType);
    c->outType = DtypeOf(c->y->valueType);
    c->computeIsInt = (computeType == ACL_INT32) ? 1 : 0;
    if (c->valType < 0 || c->outType < 0) {
        return ACL_SPARSE_STATUS_NOT_SUPPORTED;
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

// The re-stored layouts, where they apply (fp32, x larger than an L2).
// CSR_ALG2 asks for one: the blocked-gather layout first, the column panels where that one does not fit the
// matrix; both hold a copy of the values as they were at Preprocess.
// ALG_DEFAULT / CSR_ALG1 get a layout with LIVE values (every call re-reads the caller's values, so nothing can go
// stale) when the gathers of x are scattered: 0.35 ms against 1.1 ms for the merge path on an 8 M x 8 M power-law
// matrix.  For op(A) = A and floating-point values that is the layout whose row blocks add with LDS atomics: these
// algorithm values promise no bit-wise repeatable result (reference include/cann_ops_sparse.h:57-60, only CSR_ALG2
// is "deterministic").  OPS_SPARSE_SPMV_REPEATABLE in the environment (read at every size query / Preprocess) asks
// for the ordered layout there too: same bits from every call, about 0.5 ms on that matrix.  op(A) = A^T and
// int32 values always get the ordered one.  GetBufferSize and Preprocess ask the same question of the same arrays
// (a sample of the column indices, one short kernel and a synchronisation), so they agree on the size.
using Restored = opsparse::RestoredChoice;

// The OPSPARSE_* type of values and x where a re-stored layout can hold them, else -1.
int32_t RestoredValueType(aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX)
{
    if (matA->valueType != vecX->valueType) {
        return -1;
    }
    switch (matA->valueType) {
        case ACL_FLOAT:
            return OPSPARSE_F32;
        case ACL_FLOAT16:
            return OPSPARSE_F16;
        case ACL_BF16:
            return OPSPARSE_BF16;
        case ACL_INT32:
            return OPSPARSE_I32;
        default:
            return -1;
    }
}

Restored RestoredLayout(aclsparseHandle_t handle, aclsparseOperation_t opA, aclsparseConstSpMatDescr_t matA,
                        aclsparseConstDnVecDescr_t vecX, aclsparseConstDnVecDescr_t vecY, aclDataType computeType,
                        aclsparseSpMVAlg_t alg)
{
    // fp32 throughout, fp16 / bf16 values and x with y fp32 or of the same 16-bit type, or int32 values and x with
    // y int32 under the integer compute type and fp32 under the floating-point one (the blocked-gather layout
    // only: it reads the values where they are, widens x where it loads it, and rounds y once)
    const int32_t valueType = RestoredValueType(matA, vecX);
    if (valueType < 0) {
        return {0, 0, false};
    }
    if (valueType == OPSPARSE_I32) {
        if (vecY->valueType != (computeType == ACL_INT32 ? ACL_INT32 : ACL_FLOAT)) {
            return {0, 0, false};
        }
    } else if (computeType != ACL_FLOAT || (vecY->valueType != ACL_FLOAT && vecY->valueType != matA->valueType)) {
        return {0, 0, false};
    }
    const bool transpose = opA != ACL_SPARSE_OP_NON_TRANSPOSE;
    if (alg == ACL_SPARSE_SPMV_CSR_ALG2) {
        return opsparse::PickRestoredLayout(matA->rows, matA->cols, matA->nnz, transpose, valueType);
    }
    return opsparse::PickLiveLayout(handle, static_cast<const int32_t *>(matA->rowOffsets),
                                    static_cast<const int32_t *>(matA->colInd), matA->rows, matA->cols, matA->nnz,
                                    transpose, valueType, std::getenv("OPS_SPARSE_SPMV_REPEATABLE") != nullptr);
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

// An unprepared call (no preprocessed buffer bound to matA): the row statistics of matA, taken once per set of row
// offsets into the handle's workspace (one short kernel and a stream synchronisation; the reference copies all
// row offsets to the host at every call, spmv_host.cpp:86-112).  Returns the plan to run with, or NULL for the
// merge path, whose partition is rebuilt by every call because the workspace is shared.  The row-wise kernels read
// no buffer and stay correct, only slower, on row offsets that changed in place since the statistics were taken.
// Not under stream capture, where nothing may synchronise: such a call takes the merge path.
const OpsparseSpmvPlan *RowsSeen(aclsparseHandle_t handle, aclsparseConstSpMatDescr_t matA, bool transpose)
{
    OpsparseSpmvRowsSeen &seen = matA->rowsSeen;
    if (seen.rowOffsets != matA->rowOffsets || seen.rows != matA->rows || seen.nnz != matA->nnz) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(handle->stream, &capturing) != hipSuccess ||
            capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return nullptr;
        }
        if (handle->workspaceBytes() < opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz)) {
            return nullptr;
        }
        OpsparseSpmvPlan plan{};
        if (opsparse_spmv_csr_analyse(static_cast<const int32_t *>(matA->rowOffsets), matA->rows, matA->cols,
                                      matA->nnz, handle->workspace(), handle->workspaceBytes(), OPSPARSE_SPMV_AUTO,
                                      &plan, handle->stream) != OPSPARSE_OK) {
            return nullptr;
        }
        seen.rowOffsets = matA->rowOffsets;
        seen.rows = matA->rows;
        seen.nnz = matA->nnz;
        seen.plan = plan;
        seen.plan.guardTiles = 1;  // nobody promised that these row offsets stay as they are
    }
    // op(A) = A^T only takes the longest row from the plan, whatever its kernel
    if (transpose || seen.plan.kernel == OPSPARSE_SPMV_STREAM_ROWS || seen.plan.kernel == OPSPARSE_SPMV_VECTOR_ROWS) {
        return &seen.plan;
    }
    return nullptr;
}

}  // namespace

namespace opsparse {

int32_t BlockedFlags(bool transpose, bool liveValues, int32_t valueType)
{
    return (transpose ? OPSPARSE_BLOCKED_TRANSPOSE : 0) | (liveValues ? OPSPARSE_BLOCKED_LIVE_VALUES : 0) |
           (valueType == OPSPARSE_F16    ? OPSPARSE_BLOCKED_VALUES_F16
            : valueType == OPSPARSE_BF16 ? OPSPARSE_BLOCKED_VALUES_BF16
            : valueType == OPSPARSE_I32  ? OPSPARSE_BLOCKED_VALUES_I32
                                         : 0);
}

void RememberSized(aclsparseConstSpMatDescr_t matA, const RestoredChoice &choice, bool transpose, int32_t valueType)
{
    OpsparseSpmvSized &z = matA->spmvSized;
    z.rowOffsets = matA->rowOffsets;
    z.colInd = matA->colInd;
    z.rows = matA->rows;
    z.cols = matA->cols;
    z.nnz = matA->nnz;
    z.kernel = choice.kernel;
    z.transpose = transpose;
    z.liveValues = choice.liveValues;
    z.valueType = valueType;
    z.bytes = choice.keep;
}

bool SizedFor(aclsparseConstSpMatDescr_t matA, const RestoredChoice &choice, bool transpose, int32_t valueType)
{
    const OpsparseSpmvSized &z = matA->spmvSized;
    return choice.kernel != 0 && z.kernel == choice.kernel && z.bytes >= choice.keep && z.rowOffsets == matA->rowOffsets &&
           z.colInd == matA->colInd && z.rows == matA->rows && z.cols == matA->cols && z.nnz == matA->nnz &&
           z.transpose == transpose && z.liveValues == choice.liveValues && z.valueType == valueType;
}

void TrimToWorkspace(aclsparseHandle_t handle, RestoredChoice *choice, int64_t rows, int64_t cols, int64_t nnz,
                     bool transpose, int32_t valueType)
{
    choice->keep = choice->bytes;
    choice->scratch = 0;
    size_t resident = 0;
    if (choice->kernel == OPSPARSE_SPMV_BLOCKED_LIVE) {
        resident = opsparse_spmv_csr_live_resident_bytes(rows, cols, nnz);
    } else if (choice->kernel == OPSPARSE_SPMV_BLOCKED_GATHER) {
        resident = opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz,
                                                            BlockedFlags(transpose, choice->liveValues, valueType));
    }
    if (resident == 0 || resident >= choice->bytes || handle == nullptr || !handle->useUserWorkspace ||
        handle->userWorkspace == nullptr || handle->userWorkspaceBytes < choice->bytes - resident) {
        return;
    }
    choice->keep = resident;
    choice->scratch = choice->bytes - resident;
}

RestoredChoice PickLiveLayout(aclsparseHandle_t handle, const int32_t *rowOffsets, const int32_t *colInd, int64_t rows,
                              int64_t cols, int64_t nnz, bool transpose, int32_t valueType, bool repeatable)
{
    // (read at every call, like the other switches of the selection: a process may set them between two matrices)
    const bool off = std::getenv("OPS_SPARSE_SPMV_NO_DEFAULT_BLOCKED") != nullptr ||
                     std::getenv("OPS_SPARSE_SPMV_NO_BLOCKED") != nullptr;
    if (off || rowOffsets == nullptr || colInd == nullptr) {
        return {0, 0, false};
    }
    // Below 7 M entries the merge path on the caller's own arrays is as fast or faster (1 M rows x 4 entries: 30 us
    // against 44 with the layout; 1.5 M x 4: 51 against 57; 2 M x 4: 87 against 71).  Tuning override, read at
    // every call: OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ.
    const char *minEnv = std::getenv("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ");
    if (nnz < (minEnv != nullptr ? std::atoll(minEnv) : 7000000LL)) {
        return {0, 0, false};
    }
    // Results that may differ in the last bit between calls (the reference's ALG_DEFAULT / CSR_ALG1 of aclsparseSpMV)
    // get the layout whose row blocks add with atomics, where there is one: op(A) = A, floating-point data.
    const bool atomics = !repeatable && !transpose && valueType != OPSPARSE_I32;
    const size_t bytes =
        atomics ? opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
                : opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, BlockedFlags(transpose, true, valueType));
    if (bytes == 0) {
        return {0, 0, false};
    }
    // The ordered layout reads the values through a window in LDS and is about half again as slow as the one with
    // atomics: against the row-wise kernels on the caller's arrays it only wins where x is out of reach of the
    // caches (x of 3 M elements: 363 us against 447 for 3 M rows of 12, 177 against 392 for 4000 rows of 8000; x of
    // 2.2 M: 112 against 87 for 2 M rows of 4; x of 1 M and less: slower throughout).  (op(A) = A^T replaces atomics
    // on y and keeps the bounds of AnalyseRestored.)
    const char *minColsEnv = std::getenv("OPS_SPARSE_ORDERED_LIVE_MIN_COLS");  // tuning override, read at every call
    if (!atomics && !transpose && cols < (minColsEnv != nullptr ? std::atoll(minColsEnv) : kMinColsOrderedLive)) {
        return {0, 0, false};
    }
    // scattered gathers (op(A) = A^T: scattered updates of y)?  Not under stream capture (nothing may synchronise there) and not without a workspace.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(handle->stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return {0, 0, false};
    }
    if (EnsureWorkspace(handle) != ACL_SPARSE_STATUS_SUCCESS) {
        return {0, 0, false};
    }
    int32_t scattered = 0;
    if (opsparse_spmv_csr_gathers_scattered(rowOffsets, colInd, rows, cols, nnz, handle->workspace(),
                                            handle->workspaceBytes(), &scattered, handle->stream) != OPSPARSE_OK ||
        scattered < kScatteredForLiveLayout) {
        return {0, 0, false};
    }
    return {atomics ? OPSPARSE_SPMV_BLOCKED_LIVE : OPSPARSE_SPMV_BLOCKED_GATHER, bytes, true};
}

RestoredChoice PickRestoredLayout(int64_t rows, int64_t cols, int64_t nnz, bool transpose, int32_t valueType)
{
    if (std::getenv("OPS_SPARSE_SPMV_NO_BLOCKED") == nullptr) {
        const size_t blocked =
            opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, BlockedFlags(transpose, false, valueType));
        if (blocked > 0) {
            return {OPSPARSE_SPMV_BLOCKED_GATHER, blocked, false};
        }
    }
    // (the column panels hold and read fp32 only)
    const size_t panels =
        transpose || valueType != OPSPARSE_F32 ? 0 : opsparse_spmv_csr_panels_workspace_bytes(rows, cols, nnz);
    if (panels > 0) {
        return {OPSPARSE_SPMV_COLUMN_PANELS, panels, false};
    }
    return {0, 0, false};
}

int AnalyseRestored(int32_t kernel, const int32_t *rowOffsets, const int32_t *colInd, const void *values,
                    int32_t valueType, int64_t rows, int64_t cols, int64_t nnz, bool transpose, bool liveValues,
                    void *buffer, size_t bytes, void *scratch, size_t scratchBytes, OpsparseSpmvPlan *plan,
                    void *stream, bool mayVary)
{
    // A matrix whose gathers stay near the diagonal (a mesh, a band) keeps x in cache under the row-wise kernels:
    // those are then faster than any re-stored layout (the 2048 x 2048 Laplacian: 41 us against 91 us).  With some
    // gathers far from the diagonal among them the row-wise kernels take about 1.2 us per million entries and 13 us
    // per million far gathers (4 M rows of a band and 1 .. 6 random columns each); the layouts take 3.6 us (values
    // frozen) and 5.2 us (live values) per million entries whatever the columns.
    // op(A) = A^T with a y beyond an L2 keeps the layout either way: it replaces fp32 atomics on y, which it beats
    // on the same Laplacian (86 us against 119 us) and whose result depends on the order of the updates.  Where y
    // fits an L2 the atomics of a mesh stay there and are as fast or faster (1000 x 1000 Laplacian: 38 us against
    // 42 us; 700 x 700: 22 against 26), while scattered ones are not (500 000 x 500 000 with 16 random columns a
    // row: 392 us against 42 us with the layout): the same question then.  (Not below 2^18 columns, where no column
    // is far from any diagonal and many rows add to every element of y: 300 000 x 16 000 with 8 a row 111 us with
    // atomics, 23 us with the layout.)
    int32_t scattered = 1000;
    const bool ask = transpose ? cols > (int64_t{1} << 18) && cols <= (int64_t{1} << 20) : true;
    if (!liveValues && ask) {  // (a live-values request has asked already)
        int rc = opsparse_spmv_csr_gathers_scattered(rowOffsets, colInd, rows, cols, nnz, buffer, bytes, &scattered,
                                                     stream);
        if (rc != OPSPARSE_OK) {
            return rc;
        }
    }
    if (scattered < kScatteredForFrozenLayout) {
        return opsparse_spmv_csr_analyse(rowOffsets, rows, cols, nnz, buffer, bytes, OPSPARSE_SPMV_AUTO, plan, stream);
    }
    if (kernel == OPSPARSE_SPMV_BLOCKED_LIVE) {
        const int32_t flags = BlockedFlags(false, true, valueType);
        return scratchBytes > 0 ? opsparse_spmv_csr_live_analyse_split(rowOffsets, colInd, values, rows, cols, nnz, flags,
                                                                       buffer, bytes, scratch, scratchBytes, plan, stream)
                                : opsparse_spmv_csr_live_analyse(rowOffsets, colInd, values, rows, cols, nnz, flags, buffer,
                                                                 bytes, plan, stream);
    }
    if (kernel == OPSPARSE_SPMV_BLOCKED_GATHER && transpose && liveValues && mayVary && valueType != OPSPARSE_I32 &&
        std::getenv("OPS_SPARSE_SPMV_NO_SCATTER") == nullptr) {
        // op(A) = A^T where the last bit may differ between calls, as it may under the reference's atomics on y:
        // the layout that sorts the products by output panel through LDS and needs no transposed copy (the 8 M x 8 M
        // power-law matrix: 0.3 ms a call against 1.4 ms), where the matrix is one for it.  Its buffer is smaller
        // than the ordered layout's, which the size query answered with; where it does not apply (a column with
        // thousands of entries, fewer than 2 M columns) the ordered layout over the transposed copy follows.
        const int32_t flags = BlockedFlags(false, true, valueType);
        const size_t need = opsparse_spmv_csr_scatter_workspace_bytes(rows, cols, nnz, flags);
        const size_t keep = opsparse_spmv_csr_scatter_resident_bytes(rows, cols, nnz, flags);
        int rc = OPSPARSE_E_UNSUPPORTED;
        if (need > 0 && scratchBytes > 0 && keep <= bytes && need - keep <= scratchBytes) {
            rc = opsparse_spmv_csr_scatter_analyse_split(rowOffsets, colInd, rows, cols, nnz, flags, buffer, bytes, scratch,
                                                         scratchBytes, plan, stream);
        } else if (need > 0 && scratchBytes == 0 && need <= bytes) {
            rc = opsparse_spmv_csr_scatter_analyse(rowOffsets, colInd, rows, cols, nnz, flags, buffer, bytes, plan, stream);
        }
        if (rc != OPSPARSE_E_UNSUPPORTED && rc != OPSPARSE_E_WORKSPACE) {
            return rc;
        }
    }
    if (kernel == OPSPARSE_SPMV_BLOCKED_GATHER) {
        const int32_t flags = BlockedFlags(transpose, liveValues, valueType);
        const int rc = scratchBytes > 0
                           ? opsparse_spmv_csr_blocked_analyse_split(rowOffsets, colInd, values, rows, cols, nnz, flags,
                                                                     buffer, bytes, scratch, scratchBytes, plan, stream)
                           : opsparse_spmv_csr_blocked_analyse(rowOffsets, colInd, values, rows, cols, nnz, flags, buffer,
                                                               bytes, plan, stream);
        if (rc == OPSPARSE_E_UNSUPPORTED) {
            // (a row too long for a row block that cannot go the long rows' way: the ordinary plan)
            return opsparse_spmv_csr_analyse(rowOffsets, rows, cols, nnz, buffer, bytes, OPSPARSE_SPMV_AUTO, plan, stream);
        }
        return rc;
    }
    if (valueType != OPSPARSE_F32) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    return opsparse_spmv_csr_panels_analyse(rowOffsets, colInd, static_cast<const float *>(values), rows, cols, nnz,
                                            buffer, bytes, plan, stream);
}

}  // namespace opsparse

namespace {

// op(A) = A^T with fp16 / bf16 y: the sums are formed in an fp32 vector of `cols` elements and rounded once.
bool StagedTranspose(const SpmvCall &c)
{
    const int32_t yType = DtypeOf(c.y->valueType);  // (outType is only filled in by ValidateData)
    return c.transpose && (yType == OPSPARSE_F16 || yType == OPSPARSE_BF16);
}
size_t StagingBytes(aclsparseConstSpMatDescr_t matA) { return static_cast<size_t>(matA->cols) * sizeof(float); }

}  // namespace

extern "C" {

aclsparseStatus_t aclsparseSpMVGetBufferSize(aclsparseHandle_t handle, aclsparseOperation_t opA, const void * /*alpha*/,
                                             aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX,
                                             const void * /*beta*/, aclsparseDnVecDescr_t vecY,
                                             aclDataType computeType, aclsparseSpMVAlg_t alg, size_t *bufferSize)
{
    SpmvCall c{};
    const aclsparseStatus_t st = Validate(handle, opA, matA, vecX, vecY, computeType, alg, &c);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (bufferSize == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const size_t plain = opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
    Restored restored = RestoredLayout(handle, opA, matA, vecX, vecY, computeType, alg);
    opsparse::TrimToWorkspace(handle, &restored, matA->rows, matA->cols, matA->nnz, c.transpose,
                              RestoredValueType(matA, vecX));
    opsparse::RememberSized(matA, restored, c.transpose, RestoredValueType(matA, vecX));
    const size_t own = restored.keep > plain ? restored.keep : plain;
    *bufferSize = StagedTranspose(c) ? opsparse::AlignUp(own, 256) + StagingBytes(matA) : own;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMVPreprocess(aclsparseHandle_t handle, aclsparseOperation_t opA, const void * /*alpha*/,
                                          aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX,
                                          const void * /*beta*/, aclsparseDnVecDescr_t vecY, aclDataType computeType,
                                          aclsparseSpMVAlg_t alg, void *externalBuffer)
{
    SpmvCall c{};
    aclsparseStatus_t st = Validate(handle, opA, matA, vecX, vecY, computeType, alg, &c);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (handle->stream == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    st = ValidateData(&c, computeType);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    if (externalBuffer == nullptr) {
        return ACL_SPARSE_STATUS_INSUFFICIENT_RESOURCES;
    }
    OpsparseSpmvPlan plan{};
    Restored restored = RestoredLayout(handle, opA, matA, vecX, vecY, computeType, alg);
    opsparse::TrimToWorkspace(handle, &restored, matA->rows, matA->cols, matA->nnz, c.transpose,
                              RestoredValueType(matA, vecX));
    if (!opsparse::SizedFor(matA, restored, c.transpose, RestoredValueType(matA, vecX))) {
        // no size query on these arrays asked for the layout's bytes: the buffer may be as small as every query
        // answers at least, and the ordinary plan fits that
        restored = Restored{0, 0, false};
    }
    int rc;
    if (restored.kernel != 0) {
        rc = opsparse::AnalyseRestored(restored.kernel, static_cast<const int32_t *>(matA->rowOffsets),
                                       static_cast<const int32_t *>(matA->colInd), matA->values,
                                       RestoredValueType(matA, vecX), matA->rows, matA->cols, matA->nnz,
                                       opA != ACL_SPARSE_OP_NON_TRANSPOSE, restored.liveValues, externalBuffer,
                                       restored.keep, restored.scratch > 0 ? handle->userWorkspace : nullptr,
                                       restored.scratch > 0 ? handle->userWorkspaceBytes : 0, &plan, handle->stream,
                                       alg != ACL_SPARSE_SPMV_CSR_ALG2 &&
                                           std::getenv("OPS_SPARSE_SPMV_REPEATABLE") == nullptr);
    } else {
        const size_t bytes = opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
        rc = opsparse_spmv_csr_analyse(static_cast<const int32_t *>(matA->rowOffsets), matA->rows, matA->cols,
                                       matA->nnz, externalBuffer, bytes, OPSPARSE_SPMV_AUTO, &plan, handle->stream);
    }
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMVPreprocess: analysis failed (%d)", rc);
        return FromLaunch(rc);
    }
    matA->spmv.buffer = externalBuffer;
    matA->spmv.plan = plan;
    matA->spmv.stagingOffset = 0;
    matA->spmv.stagingBytes = 0;
    if (StagedTranspose(c)) {
        // behind everything GetBufferSize counted for the plan (the same sum as there)
        const size_t plain = opsparse_spmv_csr_workspace_bytes(matA->rows, matA->nnz);
        const size_t own = restored.keep > plain ? restored.keep : plain;
        matA->spmv.stagingOffset = static_cast<int64_t>(opsparse::AlignUp(own, 256));
        matA->spmv.stagingBytes = static_cast<int64_t>(StagingBytes(matA));
    }
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSpMV(aclsparseHandle_t handle, aclsparseOperation_t opA, const void *alpha,
                                aclsparseConstSpMatDescr_t matA, aclsparseConstDnVecDescr_t vecX, const void *beta,
                                aclsparseDnVecDescr_t vecY, aclDataType computeType, aclsparseSpMVAlg_t alg,
                                void *externalBuffer)
{
    SpmvCall c{};
    aclsparseStatus_t st = Validate(handle, opA, matA, vecX, vecY, computeType, alg, &c);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    // The reference refuses to run on the null stream (spmv_host.cpp:202-205).
    if (handle->stream == nullptr) {
        opsparse::LogError("aclsparseSpMV: no stream set, call aclsparseSetStream first");
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    st = ValidateData(&c, computeType);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    const OpsparseScalar a = opsparse::MakeScalar(alpha, computeType, handle->pointerMode, 1.0);
    const OpsparseScalar b = opsparse::MakeScalar(beta, computeType, handle->pointerMode, 0.0);

    // A preprocessed buffer is only trusted when it is the one bound to matA.
    const OpsparseSpmvPlan *plan = nullptr;
    void *ws = nullptr;
    size_t wsBytes = 0;
    const bool bound = externalBuffer != nullptr && matA->spmv.buffer == externalBuffer &&
                       matA->spmv.plan.rows == matA->rows && matA->spmv.plan.nnz == matA->nnz;
    const bool blockedPlan = bound && (matA->spmv.plan.kernel == OPSPARSE_SPMV_BLOCKED_GATHER ||
                                       matA->spmv.plan.kernel == OPSPARSE_SPMV_BLOCKED_LIVE ||
                                       matA->spmv.plan.kernel == OPSPARSE_SPMV_SCATTER_LIVE);
    if (blockedPlan && (matA->spmv.plan.transposed != 0) != c.transpose) {
        // Preprocess built the re-stored layout for the other op(A): this call runs without it
        if (matA->nnz > 0 || (c.transpose && c.outType != OPSPARSE_F32)) {
            st = opsparse::EnsureWorkspace(handle);
            if (st != ACL_SPARSE_STATUS_SUCCESS) {
                return st;
            }
            ws = handle->workspace();
            wsBytes = handle->workspaceBytes();
        }
    } else if (bound && (!c.transpose || blockedPlan)) {
        plan = &matA->spmv.plan;
        ws = externalBuffer;
        wsBytes = static_cast<size_t>(plan->bytes);
    } else if (matA->nnz > 0 || (c.transpose && c.outType != OPSPARSE_F32)) {
        if (c.transpose && bound) {
            plan = &matA->spmv.plan;  // op(A) = A^T only takes the row-length statistics from it
        }
        // the merge-path partition of an unprepared call, or the fp32 staging vector of a transposed
        // product with fp16 / bf16 y (cols * 4 bytes: enlarge it with aclsparseSetWorkspace if need be)
        st = opsparse::EnsureWorkspace(handle);
        if (st != ACL_SPARSE_STATUS_SUCCESS) {
            return st;
        }
        ws = handle->workspace();
        wsBytes = handle->workspaceBytes();
        if (plan == nullptr && matA->nnz > 0 && matA->rows > 0) {
            plan = RowsSeen(handle, matA, c.transpose);
        }
        if (StagedTranspose(c) && bound && wsBytes < StagingBytes(matA) &&
            matA->spmv.stagingBytes >= static_cast<int64_t>(StagingBytes(matA))) {
            // y too long for the handle's workspace: the buffer was preprocessed for this kind of call and has
            // the room (a transposed product uses the workspace for nothing else)
            ws = static_cast<unsigned char *>(externalBuffer) + matA->spmv.stagingOffset;
            wsBytes = static_cast<size_t>(matA->spmv.stagingBytes);
        }
    }
    const int rc = opsparse_spmv_csr_launch(
        plan, c.transpose ? 1 : 0, static_cast<const int32_t *>(matA->rowOffsets),
        static_cast<const int32_t *>(matA->colInd), matA->values, vecX->values, vecY->values, matA->rows, matA->cols,
        matA->nnz, a, b, c.valType, c.outType, c.computeIsInt, ws, wsBytes, handle->stream);
    if (rc != OPSPARSE_OK) {
        opsparse::LogError("aclsparseSpMV: launch failed (%d)", rc);
    }
    return FromLaunch(rc);
}

}  // extern "C"
