// Internal object layouts of libops_sparse.so (handle, descriptors, SpMV / SpMM
// plans).  Nothing here is visible through the public header: callers only see
// opaque pointers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "cann_ops_sparse.h"
#include "ops_sparse_hip.h"

namespace opsparse {

constexpr int kVersionMajor = 1;
constexpr int kVersionMinor = 0;
constexpr int kVersionPatch = 0;

// Size of the device workspace every handle owns
// (reference: sparse/common/aclsparse_handle_internal.h:44).
constexpr size_t kDefaultWorkspaceBytes = 4u * 1024u * 1024u;

// Tag stored in live dense-vector descriptors and checked by the accessors
// (reference: sparse/common/aclsparse_descr.cpp:29).
constexpr uint32_t kDnVecSignature = 0xD0D2D4D6u;

inline size_t AlignUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace opsparse

// What aclsparseSpMVPreprocess leaves behind for a matrix: the kernel family
// picked from the row-length statistics and, for the merge-path family, where
// in the caller's buffer the partition lives.
struct OpsparseSpmvBinding {
    const void *buffer = nullptr;  // buffer this plan was written into
    OpsparseSpmvPlan plan{};
    // op(A) = A^T with fp16 / bf16 y sums into an fp32 vector of `cols` elements: room for it behind the plan's
    // own part of the buffer (0 bytes: the buffer was preprocessed for a call that needs none)
    int64_t stagingOffset = 0;
    int64_t stagingBytes = 0;
};

// What the first aclsparseSpMV call without a preprocessed buffer learns about the rows of a matrix: the row-wise
// kernels keep nothing in a buffer, so later calls on the same row offsets run the one these statistics select.
struct OpsparseSpmvRowsSeen {
    const void *rowOffsets = nullptr;  // the statistics are of these offsets, this many rows and entries
    int64_t rows = -1;
    int64_t nnz = -1;
    OpsparseSpmvPlan plan{};
};

// What the last buffer-size query on a matrix answered (aclsparseSpMVGetBufferSize, aclsparseSpMVOp_bufferSize).
// Preprocess / createDescr only know the caller's buffer by its address: they write a re-stored layout into it
// only when this record says that a query on the same arrays asked for that many bytes; anything else (no query,
// arrays replaced since, a query under stream capture that could not look at the columns) gets the plan that fits
// the small size every query answers at least.
struct OpsparseSpmvSized {
    const void *rowOffsets = nullptr, *colInd = nullptr;
    int64_t rows = -1, cols = -1, nnz = -1;
    int32_t kernel = 0;      // OPSPARSE_SPMV_BLOCKED_GATHER / BLOCKED_LIVE / COLUMN_PANELS, 0: none
    bool transpose = false;  // ... for this op(A)
    bool liveValues = false;
    int32_t valueType = -1;
    size_t bytes = 0;        // of the layout
};

struct OpsparseSpmmBinding {
    const void *buffer = nullptr;
    OpsparseSpmmPlan plan{};
    int64_t stagingBytes = 0;  // room behind the plan's tables for row-major copies of B / C (0: none)
    int64_t widestN = 0;       // the widest C the buffer has been analysed for: its tables fit that width and less
    // One or two columns of B and C that are vectors in memory run as SpMV calls: their plan, and where in the
    // buffer its workspace lies (0: the buffer was not preprocessed for such operands).
    OpsparseSpmvPlan vectorPlan{};
    int64_t vectorOff = 0;
    int64_t vectorBytes = 0;
};

// reference: sparse/common/aclsparse_handle_internal.h:56-72
struct aclsparseContext {
    hipStream_t stream = nullptr;
    aclsparsePointerMode_t pointerMode = ACL_SPARSE_POINTER_MODE_HOST;
    void *defaultWorkspace = nullptr;
    size_t defaultWorkspaceBytes = 0;
    void *userWorkspace = nullptr;
    size_t userWorkspaceBytes = 0;
    bool useUserWorkspace = false;

    void *workspace() const { return useUserWorkspace ? userWorkspace : defaultWorkspace; }
    size_t workspaceBytes() const { return useUserWorkspace ? userWorkspaceBytes : defaultWorkspaceBytes; }
};

// reference: sparse/common/aclsparse_descr_internal.h:32-56 (the CSR part)
struct aclsparseSpMatDescr {
    aclsparseFormat_t format = ACL_SPARSE_FORMAT_CSR;
    int64_t rows = 0;
    int64_t cols = 0;
    int64_t nnz = 0;
    void *rowOffsets = nullptr;
    void *colInd = nullptr;
    void *values = nullptr;
    aclsparseIndexType_t rowOffsetsType = ACL_SPARSE_INDEX_32I;
    aclsparseIndexType_t colIndType = ACL_SPARSE_INDEX_32I;
    aclsparseIndexBase_t idxBase = ACL_SPARSE_INDEX_BASE_ZERO;
    aclDataType valueType = ACL_FLOAT;
    // Preprocess results.  The public API hands the matrix in as a pointer to
    // const, like the reference, and the reference's Preprocess records its
    // active buffer in the descriptor all the same
    // (sparse/spmm/arch35/spmm_host.cpp:360); `mutable` makes that explicit.
    mutable OpsparseSpmvBinding spmv;
    mutable OpsparseSpmvRowsSeen rowsSeen;
    mutable OpsparseSpmvSized spmvSized;
    mutable OpsparseSpmmBinding spmm;
};

// reference: sparse/common/aclsparse_descr_internal.h:102-107
struct aclsparseDnVecDescr {
    uint32_t signature = 0;
    int64_t size = 0;
    void *values = nullptr;
    aclDataType valueType = ACL_FLOAT;
};

// reference: sparse/common/aclsparse_descr_internal.h:121-128
struct aclsparseDnMatDescr {
    int64_t rows = 0;
    int64_t cols = 0;
    int64_t ld = 0;
    aclsparseOrder_t order = ACL_SPARSE_ORDER_ROW;
    void *values = nullptr;
    aclDataType valueType = ACL_FLOAT;
};

namespace opsparse {

// Error text goes to stderr only when OPS_SPARSE_LOG is set in the
// environment; the success path never prints.
void LogError(const char *fmt, ...);

// Allocates the handle's default 4 MiB device workspace on first use (no-op when
// a user workspace is active or the default one already exists).
aclsparseStatus_t EnsureWorkspace(aclsparseContext *h);

// Reads one scalar of `computeType` (ACL_FLOAT or ACL_INT32) for the launch
// layer.  In HOST mode the value is dereferenced now (NULL gives `dflt`); in
// DEVICE mode the address is passed on and the kernel reads it.
OpsparseScalar MakeScalar(const void *p, aclDataType computeType, aclsparsePointerMode_t mode, double dflt);

// The re-stored SpMV layout an ALG2 request gets for a plain fp32 CSR matrix (AnalyseRestored falls back to
// the ordinary analysis in the same buffer when a sample of the columns shows the gathers are local): BLOCKED_GATHER where it
// applies, else (op(A) = A only) COLUMN_PANELS, else none (kernel 0, 0 bytes).  OPS_SPARSE_SPMV_NO_BLOCKED in the
// environment skips the first (tuning, tests of the panel path).
// Sampled gathers in a thousand that must land far from the diagonal (opsparse_spmv_csr_gathers_scattered) for a
// re-stored layout to pay: with the values frozen, and with live values.
constexpr int32_t kScatteredForFrozenLayout = 190;
constexpr int32_t kScatteredForLiveLayout = 310;
// Columns from which the ordered layout with live values (repeatable sums) is taken for op(A) = A.
constexpr int64_t kMinColsOrderedLive = int64_t{5} << 19;  // 2.6 M

struct RestoredChoice {
    int32_t kernel;
    size_t bytes;     // of the whole layout, analysis scratch included
    bool liveValues;  // BLOCKED_GATHER / BLOCKED_LIVE: the layout holds no values, every call takes the caller's
    size_t keep = 0;     // what the caller's buffer has to hold: `bytes`, or only what the launches keep ...
    size_t scratch = 0;  // ... when the analysis takes this much from the handle's workspace (TrimToWorkspace)
};
// Where the handle has a workspace of the user's (aclsparseSetWorkspace) with room for the scratch of the layout's
// analysis, the caller's buffer only needs what the launches keep (the 8 M-row power-law matrix: 0.79 GiB instead
// of 2.09): sets keep / scratch accordingly, else keep = bytes.
void TrimToWorkspace(aclsparseHandle_t handle, RestoredChoice *choice, int64_t rows, int64_t cols, int64_t nnz,
                     bool transpose, int32_t valueType);
// The layout a default-algorithm request gets where it pays: blocked gather with live values (7 M
// entries or more, an x the layout applies to, and a sample of the columns that says the gathers are scattered:
// one short kernel and a synchronisation of the handle's stream), else none.  `repeatable`: the caller promises
// the same bits from every execution (aclsparseSpMVOp): BLOCKED_GATHER; else BLOCKED_LIVE where it exists
// (op(A) = A, floating-point values).
RestoredChoice PickLiveLayout(aclsparseHandle_t handle, const int32_t *rowOffsets, const int32_t *colInd, int64_t rows,
                              int64_t cols, int64_t nnz, bool transpose, int32_t valueType, bool repeatable);
// The size-query record of a matrix (OpsparseSpmvSized): written by the queries, asked by Preprocess / createDescr.
void RememberSized(aclsparseConstSpMatDescr_t matA, const RestoredChoice &choice, bool transpose, int32_t valueType);
bool SizedFor(aclsparseConstSpMatDescr_t matA, const RestoredChoice &choice, bool transpose, int32_t valueType);
// valueType: the OPSPARSE_* type of the values and of x.
RestoredChoice PickRestoredLayout(int64_t rows, int64_t cols, int64_t nnz, bool transpose, int32_t valueType);
// `scratch` / `scratchBytes`: where the analysis works when the buffer only has room for what the launches keep
// (scratchBytes == 0: behind that, in the buffer itself).  `mayVary`: the caller's algorithm value lets the last bit
// of a result differ between calls (aclsparseSpMV with ALG_DEFAULT / CSR_ALG1): op(A) = A^T may then take the
// SCATTER_LIVE layout inside the same buffer.
int AnalyseRestored(int32_t kernel, const int32_t *rowOffsets, const int32_t *colInd, const void *values,
                    int32_t valueType, int64_t rows, int64_t cols, int64_t nnz, bool transpose, bool liveValues,
                    void *buffer, size_t bytes, void *scratch, size_t scratchBytes, OpsparseSpmvPlan *plan,
                    void *stream, bool mayVary = false);

}  // namespace opsparse
