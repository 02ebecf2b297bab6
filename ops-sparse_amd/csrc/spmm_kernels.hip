// CSR SpMM kernels for gfx950 and their C-ABI launcher.
//
// C = alpha * A * op(B) + beta * C, A in CSR (int32), B and C dense.
// Replaces the device side of the reference's aclsparseSpMM
// (sparse/spmm/arch35/spmm_kernel.cpp:88-270, launched by :447-477).  The
// reference gives every SIMT thread one (row, 8-column chunk) and lets it walk
// the row alone, so A is re-read n/8 times and B is read 32 bytes at a time.
// Here a group of L lanes owns a row and spans the n output columns, each lane
// holding V consecutive columns (16 bytes of B): one gather instruction of a
// wavefront fetches 64/L whole rows of B, fully coalesced, and A is read once.
// The (colind, value) pairs of a row are loaded L at a time, one pair per
// lane, non-temporally, and handed round the group with cross-lane shuffles.
//
// Floating-point products are accumulated in fp64 in stored order and rounded
// once, int8 products in int32 with an int64 saturating epilogue
// (spmm_kernel.cpp:251-266).
#include <type_traits>

#include "device_utils.h"

namespace opsparse {

// Index of element (r, c) of a dense matrix with leading dimension ld.
__device__ __forceinline__ int64_t DenseIndex(int64_t r, int64_t c, int64_t ld, bool colMajor)
{
    return colMajor ? c * ld + r : r * ld + c;
}

template <typename CT, typename AccT>
struct Epilogue {
    // Floating point: alpha * acc (+ beta * old); fp16 output is clamped to the
    // finite fp16 range before rounding (spmm_kernel.cpp:229-237).
    static __device__ __forceinline__ CT Apply(AccT acc, AccT alpha, AccT beta, bool betaZero, const CT *oldPtr,
                                               bool clampF16)
    {
        AccT r = alpha * acc;
        if (!betaZero) {
            r += beta * ToAcc<AccT>(*oldPtr);
        }
        if (std::is_same<CT, Half>::value && clampF16) {
            r = r > AccT(65504.0) ? AccT(65504.0) : r;
            r = r < AccT(-65504.0) ? AccT(-65504.0) : r;
        }
        return FromAcc<CT>(r);
    }
};

template <>
struct Epilogue<int32_t, int32_t> {
    static __device__ __forceinline__ int32_t Apply(int32_t acc, int32_t alpha, int32_t beta, bool betaZero,
                                                    const int32_t *oldPtr, bool)
    {
        int64_t wide = static_cast<int64_t>(alpha) * static_cast<int64_t>(acc);
        if (!betaZero) {
            wide += static_cast<int64_t>(beta) * static_cast<int64_t>(*oldPtr);
        }
        wide = wide > 2147483647LL ? 2147483647LL : wide;
        wide = wide < -2147483648LL ? -2147483648LL : wide;
        return static_cast<int32_t>(wide);
    }
};

// ---------------------------------------------------------------- fast path
// B row-major, op(B) = B, C row-major, n and both leading dimensions multiples
// of V, B and C 16-byte aligned.

template <typename ValT, typename CT, typename AccT, int V, int L>
__global__ __launch_bounds__(kBlockThreads) void SpmmRowSplitKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, CT *__restrict__ C, int64_t rows, int32_t n, int64_t ldb, int64_t ldc,
    int32_t rowsPerGroup, OpsparseScalar alphaS, OpsparseScalar betaS, int32_t clampF16)
{
    typedef ValT BVec __attribute__((ext_vector_type(V)));
    typedef CT CVec __attribute__((ext_vector_type(V), aligned(16)));
    constexpr int kGroups = kBlockThreads / L;
    constexpr int U = L < 16 ? L : 16;

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));

    const int32_t lane = threadIdx.x % L;
    const int32_t group = threadIdx.x / L;
    const int64_t tile = XcdContiguousTile(blockIdx.x, gridDim.x);
    const int64_t rowBase = tile * (static_cast<int64_t>(kGroups) * rowsPerGroup);

    for (int32_t it = 0; it < rowsPerGroup; ++it) {
        const int64_t r = rowBase + static_cast<int64_t>(it) * kGroups + group;
        if (r >= rows) {
            break;
        }
        const int32_t s = rowOffsets[r];
        const int32_t e = rowOffsets[r + 1];
        for (int32_t c0 = 0; c0 < n; c0 += L * V) {
            const int32_t col = c0 + lane * V;
            const bool active = col < n;
            AccT acc[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                acc[i] = AccT(0);
            }
            for (int32_t p0 = s; p0 < e; p0 += L) {
                int32_t myCol = 0;
                float myVal = 0.0f;
                if (p0 + lane < e) {
                    myCol = LoadStream(colInd + p0 + lane);
                    myVal = static_cast<float>(ToAcc<AccT>(LoadStream(vals + p0 + lane)));
                }
                const int32_t cnt = (e - p0 < L) ? e - p0 : L;
                if (cnt == L) {
                    // Full chunk: U gathers are issued back to back before their
                    // products are consumed, U * 16 bytes in flight per lane.
#pragma unroll
                    for (int q0 = 0; q0 < L; q0 += U) {
                        BVec b[U];
                        float v[U];
#pragma unroll
                        for (int q = 0; q < U; ++q) {
                            const int32_t c = __shfl(myCol, q0 + q, L);
                            v[q] = __shfl(myVal, q0 + q, L);
                            if (active) {
                                b[q] = *reinterpret_cast<const BVec *>(B + static_cast<int64_t>(c) * ldb + col);
                            }
                        }
                        if (active) {
#pragma unroll
                            for (int q = 0; q < U; ++q) {
                                const AccT vq = static_cast<AccT>(v[q]);
#pragma unroll
                                for (int i = 0; i < V; ++i) {
                                    acc[i] += vq * ToAcc<AccT>(b[q][i]);
                                }
                            }
                        }
                    }
                } else {
                    for (int32_t q = 0; q < cnt; ++q) {
                        const int32_t c = __shfl(myCol, q, L);
                        const AccT vq = static_cast<AccT>(__shfl(myVal, q, L));
                        if (active) {
                            const BVec b = *reinterpret_cast<const BVec *>(B + static_cast<int64_t>(c) * ldb + col);
#pragma unroll
                            for (int i = 0; i < V; ++i) {
                                acc[i] += vq * ToAcc<AccT>(b[i]);
                            }
                        }
                    }
                }
            }
            if (active) {
                CT *out = C + r * ldc + col;
                CVec res;
                if (betaZero) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        res[i] = Epilogue<CT, AccT>::Apply(acc[i], alpha, beta, true, nullptr, clampF16 != 0);
                    }
                } else {
                    const CVec old = *reinterpret_cast<const CVec *>(out);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const CT o = old[i];
                        res[i] = Epilogue<CT, AccT>::Apply(acc[i], alpha, beta, false, &o, clampF16 != 0);
                    }
                }
                *reinterpret_cast<CVec *>(out) = res;
            }
        }
    }
}

// ------------------------------------------------------------- general path
// Any storage order of B and C, op(B) = B or B^T, any n / ld: lanes of a group
// stride over the output columns of one row, one column at a time.

template <typename ValT, typename CT, typename AccT, int L>
__global__ __launch_bounds__(kBlockThreads) void SpmmGeneralKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, CT *__restrict__ C, int64_t rows, int32_t n, int64_t ldb, int64_t ldc,
    int32_t bColMajor, int32_t cColMajor, int32_t transB, OpsparseScalar alphaS, OpsparseScalar betaS,
    int32_t clampF16)
{
    constexpr int kGroups = kBlockThreads / L;
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    // Element (c, j) of op(B): B stored (c, j) for op = N, (j, c) for op = T
    // (spmm_kernel.cpp:155-168), so a transposed B swaps the roles of the two
    // indices, i.e. flips the effective storage order.
    const bool bEffColMajor = (bColMajor != 0) != (transB != 0);

    const int32_t lane = threadIdx.x % L;
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kGroups + threadIdx.x / L;
    if (r >= rows) {
        return;
    }
    const int32_t s = rowOffsets[r];
    const int32_t e = rowOffsets[r + 1];
    for (int32_t j = lane; j < n; j += L) {
        AccT acc = AccT(0);
        for (int32_t p = s; p < e; ++p) {
            const int64_t c = colInd[p];
            acc += ToAcc<AccT>(vals[p]) * ToAcc<AccT>(B[DenseIndex(c, j, ldb, bEffColMajor)]);
        }
        CT *out = C + DenseIndex(r, j, ldc, cColMajor != 0);
        *out = Epilogue<CT, AccT>::Apply(acc, alpha, beta, betaZero, out, clampF16 != 0);
    }
}

// =============================================================== host side

namespace {

struct SpmmArgs {
    const int32_t *rowOffsets;
    const int32_t *colInd;
    const void *vals;
    const void *B;
    void *C;
    int64_t rows, k, n, nnz, ldb, ldc;
    int32_t bColMajor, cColMajor, transB, clampF16;
    OpsparseScalar alpha, beta;
    hipStream_t stream;
};

inline int CheckLaunch()
{
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

template <typename ValT, typename CT, typename AccT, int V, int L>
int LaunchRowSplit(const SpmmArgs &a)
{
    constexpr int kGroups = kBlockThreads / L;
    // Each lane group walks a few rows so that a workgroup lives long enough to
    // hide its start-up latency.
    const int32_t rowsPerGroup = 4;
    const int64_t rowsPerBlock = static_cast<int64_t>(kGroups) * rowsPerGroup;
    const uint32_t grid = static_cast<uint32_t>((a.rows + rowsPerBlock - 1) / rowsPerBlock);
    hipLaunchKernelGGL((SpmmRowSplitKernel<ValT, CT, AccT, V, L>), dim3(grid), dim3(kBlockThreads), 0, a.stream,
                       a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.B),
                       static_cast<CT *>(a.C), a.rows, static_cast<int32_t>(a.n), a.ldb, a.ldc, rowsPerGroup, a.alpha,
                       a.beta, a.clampF16);
    return CheckLaunch();
}

template <typename ValT, typename CT, typename AccT, int L>
int LaunchGeneral(const SpmmArgs &a)
{
    constexpr int kGroups = kBlockThreads / L;
    const uint32_t grid = static_cast<uint32_t>((a.rows + kGroups - 1) / kGroups);
    hipLaunchKernelGGL((SpmmGeneralKernel<ValT, CT, AccT, L>), dim3(grid), dim3(kBlockThreads), 0, a.stream,
                       a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.B),
                       static_cast<CT *>(a.C), a.rows, static_cast<int32_t>(a.n), a.ldb, a.ldc, a.bColMajor,
                       a.cColMajor, a.transB, a.alpha, a.beta, a.clampF16);
    return CheckLaunch();
}

template <typename ValT, typename CT, typename AccT>
int RunGeneral(const SpmmArgs &a)
{
    if (a.n <= 4) return LaunchGeneral<ValT, CT, AccT, 4>(a);
    if (a.n <= 8) return LaunchGeneral<ValT, CT, AccT, 8>(a);
    if (a.n <= 16) return LaunchGeneral<ValT, CT, AccT, 16>(a);
    if (a.n <= 32) return LaunchGeneral<ValT, CT, AccT, 32>(a);
    return LaunchGeneral<ValT, CT, AccT, 64>(a);
}

template <typename ValT, typename CT, typename AccT>
int RunTyped(const SpmmArgs &a)
{
    constexpr int V = 16 / static_cast<int>(sizeof(ValT));  // 16 bytes of B per lane
    const bool fast = !a.bColMajor && !a.cColMajor && !a.transB && a.n % V == 0 && a.ldb % V == 0 &&
                      a.ldc % V == 0 && reinterpret_cast<uintptr_t>(a.B) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(a.C) % 16 == 0;
    if (!fast) {
        return RunGeneral<ValT, CT, AccT>(a);
    }
    const int64_t lanesNeeded = a.n / V;
    if (lanesNeeded <= 2) return LaunchRowSplit<ValT, CT, AccT, V, 2>(a);
    if (lanesNeeded <= 4) return LaunchRowSplit<ValT, CT, AccT, V, 4>(a);
    if (lanesNeeded <= 8) return LaunchRowSplit<ValT, CT, AccT, V, 8>(a);
    if (lanesNeeded <= 16) return LaunchRowSplit<ValT, CT, AccT, V, 16>(a);
    if (lanesNeeded <= 32) return LaunchRowSplit<ValT, CT, AccT, V, 32>(a);
    return LaunchRowSplit<ValT, CT, AccT, V, 64>(a);
}

}  // namespace
}  // namespace opsparse

using namespace opsparse;

extern "C" {

size_t opsparse_spmm_csr_workspace_bytes(int64_t rows, int64_t nnz, int64_t n)
{
    (void)rows;
    (void)nnz;
    (void)n;
    return 256;  // header only: the row-split kernels need no tables
}

int opsparse_spmm_csr_analyse(const int32_t *rowOffsets, int64_t rows, int64_t nnz, int64_t n, void *workspace,
                              size_t workspaceBytes, int32_t forceKernel, OpsparseSpmmPlan *plan, void *stream)
{
    (void)rowOffsets;
    (void)stream;
    (void)forceKernel;
    if (plan == nullptr || rows < 0 || nnz < 0 || n < 0) {
        return OPSPARSE_E_INVALID;
    }
    if (workspace == nullptr || workspaceBytes < 256) {
        return OPSPARSE_E_WORKSPACE;
    }
    OpsparseSpmmPlan p{};
    p.kernel = OPSPARSE_SPMM_ROW_SPLIT;
    p.rows = rows;
    p.nnz = nnz;
    p.n = n;
    p.bytes = 256;
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmm_csr_launch(const OpsparseSpmmPlan *plan, const int32_t *rowOffsets, const int32_t *colInd,
                             const void *csrValues, const void *B, void *C, int64_t rows, int64_t k, int64_t n,
                             int64_t nnz, int64_t ldb, int64_t ldc, int32_t bColMajor, int32_t cColMajor,
                             int32_t transB, OpsparseScalar alpha, OpsparseScalar beta, int32_t valType,
                             int32_t cType, void *workspace, size_t workspaceBytes, void *stream)
{
    (void)plan;
    (void)workspace;
    (void)workspaceBytes;
    if (rows < 0 || k < 0 || n < 0 || nnz < 0 || ldb <= 0 || ldc <= 0 || n > INT32_MAX) {
        return OPSPARSE_E_INVALID;
    }
    if (rows == 0 || n == 0) {
        return OPSPARSE_OK;
    }
    if (rowOffsets == nullptr || C == nullptr || (nnz > 0 && (colInd == nullptr || csrValues == nullptr || B == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    SpmmArgs a{rowOffsets, colInd, csrValues, B,      C,    rows, k, n, nnz, ldb, ldc, bColMajor, cColMajor,
               transB,     0,      alpha,     beta,   static_cast<hipStream_t>(stream)};
    if (valType == OPSPARSE_F32 && cType == OPSPARSE_F32) {
        return RunTyped<float, float, double>(a);
    }
    if (valType == OPSPARSE_F16 && cType == OPSPARSE_F16) {
        a.clampF16 = 1;
        return RunTyped<Half, Half, double>(a);
    }
    if (valType == OPSPARSE_F16 && cType == OPSPARSE_F32) {
        return RunTyped<Half, float, double>(a);
    }
    if (valType == OPSPARSE_I8 && cType == OPSPARSE_I32) {
        return RunGeneral<int8_t, int32_t, int32_t>(a);
    }
    return OPSPARSE_E_UNSUPPORTED;
}

}  // extern "C"
