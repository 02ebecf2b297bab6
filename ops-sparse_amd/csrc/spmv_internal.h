// Pieces of the SpMV launcher shared by its translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "ops_sparse_hip.h"

namespace opsparse {

struct SpmvArgs {
    const int32_t *rowOffsets;
    const int32_t *colInd;
    const void *vals;
    const void *x;
    void *y;
    const void *yIn;  // old y (may be y itself)
    int64_t rows, cols, nnz;
    OpsparseScalar alpha, beta;
    void *ws;
    size_t wsBytes;
    hipStream_t stream;
};

inline int CheckLaunch()
{
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

// BLOCKED_GATHER launch (spmv_blocked.hip): values and x of valType, y of outType (fp32 or valType).
int LaunchBlocked(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType,
                  int32_t computeIsInt);

// BLOCKED_LIVE launch (spmv_blocked_live.hip): values and x of valType (fp32 / fp16 / bf16), y fp32 or of valType.
namespace live_layout {
int LaunchBlocked(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType);
}

// SCATTER_LIVE launch (spmv_scatter.hip): op(A) = A^T; a.rows / a.cols are those of A.
namespace scatter_layout {
int Launch(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType);
}

}  // namespace opsparse
