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

// BLOCKED_GATHER launch, fp32 values / x / y (spmv_blocked.hip).
int LaunchBlocked(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType);

}  // namespace opsparse
