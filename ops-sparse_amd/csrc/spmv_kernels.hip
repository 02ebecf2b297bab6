// CSR SpMV kernels for gfx950 and their C-ABI launcher.
//
// y = alpha * A * x + beta * y with A in CSR (int32 offsets and indices).
// Replaces the device side of the reference's aclsparseSpMV
// (sparse/spmv/arch22/kernels/spmv_kernel.h:27-310 for op = N, :321-640 for
// op = T, dispatched by kernels/spmv_kernel.cpp:21-55).  The reference walks
// one row at a time per core; here the rows are binned by length:
//
//   STREAM_ROWS  rows of at most a few dozen non-zeros.  A workgroup owns a
//                fixed block of consecutive rows, loads their contiguous
//                (colind, value) range with full-width coalesced non-temporal
//                loads, gathers x, parks the products in LDS and then lets
//                1..8 lanes per row add them up in stored order.  A few long
//                rows among short ones are left out by the tiles and summed
//                beside them, a workgroup per row (SpmvLongRowsKernel).
//   VECTOR_ROWS  long rows of nearly equal length: a group of 4..64 lanes
//                strides along one row and reduces with cross-lane shuffles.
//                Needs no workspace.
//   MERGE_PATH   everything else (power-law rows, rows of varying length): the
//                merge of "row ends" and "non-zero indices" is cut into equal
//                pieces, so every workgroup gets the same rows + nnz whatever
//                the row lengths are.  Products are staged in LDS as above; a
//                row cut by a workgroup boundary leaves a carry-out, and a
//                small fix-up kernel adds the pieces in a fixed order, so the
//                result is deterministic.
//
// The family is chosen per matrix from row statistics (opsparse_spmv_csr_analyse,
// where the measurements behind the rule are quoted).  op(A) = A^T has its own
// kernels further down: fp32 atomics per entry like the reference, per-workgroup
// sums in LDS when y is short, whole workgroups for long rows, an entry-split
// kernel when the rows are few.
//
// Memory traffic per launch is the compulsory nnz*(sizeof(val)+4) +
// (rows+1)*4 + rows*sizeof(y)*(1 + [beta != 0]) plus x: the kernels are
// HBM-bound streaming kernels, there is no matrix-core work in them.
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "convert_internal.h"
#include "spmv_internal.h"
#include "device_utils.h"

namespace opsparse {

// ------------------------------------------------------------- epilogue

template <typename OutT, typename AccT>
__device__ __forceinline__ void StoreRow(OutT *y, const OutT *yIn, int64_t row, AccT sum, AccT alpha, AccT beta,
                                         bool betaZero)
{
    AccT r = alpha * sum;
    if (!betaZero) {
        r += beta * ToAcc<AccT>(yIn[row]);
    }
    if constexpr (std::is_same<OutT, double>::value) {
        // fp64 outputs are the column panels' partial vectors: written once, read once by the combine
        // kernel, and they must not push the panel's slice of x out of the L2
        __builtin_nontemporal_store(r, y + row);
    } else {
        y[row] = FromAcc<OutT>(r);
    }
}

// Loads 4 consecutive values and converts them to the accumulator type.
template <typename AccT, typename ValT>
__device__ __forceinline__ void LoadVals4(const ValT *p, AccT out[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[i] = ToAcc<AccT>(LoadStream(p + i));
    }
}
template <>
__device__ __forceinline__ void LoadVals4<double, float>(const float *p, double out[4])
{
    const Float4U v = __builtin_nontemporal_load(reinterpret_cast<const Float4U *>(p));
    out[0] = v.x;
    out[1] = v.y;
    out[2] = v.z;
    out[3] = v.w;
}

// ------------------------------------------------------------- y = beta * y

template <typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvScaleKernel(OutT *y, const OutT *yIn, int64_t len,
                                                                 OpsparseScalar betaS)
{
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < len; i += stride) {
        y[i] = betaZero ? FromAcc<OutT>(AccT(0)) : FromAcc<OutT>(beta * ToAcc<AccT>(yIn[i]));
    }
}

// dst = beta * src widened to fp32 (0 when beta == 0: src is not read), and the way back: the transposed
// product adds into an fp32 vector, which for fp16 / bf16 y is a staging vector in the workspace.
template <typename InT>
__global__ __launch_bounds__(kBlockThreads) void ScaleIntoFloatKernel(float *__restrict__ dst, const InT *src,
                                                                      int64_t len, OpsparseScalar betaS)
{
    const double beta = ReadScalar<double>(betaS);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < len; i += stride) {
        dst[i] = beta == 0.0 ? 0.0f : static_cast<float>(beta * ToAcc<double>(src[i]));
    }
}

template <typename OutT>
__global__ __launch_bounds__(kBlockThreads) void ConvertFromFloatKernel(OutT *__restrict__ dst,
                                                                        const float *__restrict__ src, int64_t len)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < len; i += stride) {
        dst[i] = FromAcc<OutT>(static_cast<double>(src[i]));
    }
}

// ------------------------------------------------------------- row statistics

constexpr int kStreamMaxRow = 512;  // the stream-rows tiles are sized for rows up to this long
constexpr int kShortMaxRow = 48;    // "short rows with a few long ones among them": what counts as short
constexpr int kBesideRow = 64;      // with SpmvLongRowsKernel beside them, the stream-rows kernels skip longer rows
constexpr int kBesideMaxRow = 8192; // ... which one workgroup sums: beyond this length the merge path is the better answer

// stats[0] = longest row, stats[1] = longest row of at most kShortMaxRow entries, stats[2] = number of longer
// rows, stats[3] = their entries.  stats must be zeroed before the launch.
__global__ __launch_bounds__(kBlockThreads) void RowStatsKernel(const int32_t *__restrict__ rowOffsets, int64_t rows,
                                                                int32_t *__restrict__ stats)
{
    int32_t best = 0, bestShort = 0, numLong = 0;
    uint32_t nnzLong = 0;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; r < rows; r += stride) {
        const int32_t len = rowOffsets[r + 1] - rowOffsets[r];
        best = len > best ? len : best;
        if (len <= kShortMaxRow) {
            bestShort = len > bestShort ? len : bestShort;
        } else {
            ++numLong;
            nnzLong += static_cast<uint32_t>(len);
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int32_t other = __shfl_xor(best, off, kWave);
        best = other > best ? other : best;
        const int32_t otherShort = __shfl_xor(bestShort, off, kWave);
        bestShort = otherShort > bestShort ? otherShort : bestShort;
        numLong += __shfl_xor(numLong, off, kWave);
        nnzLong += __shfl_xor(nnzLong, off, kWave);
    }
    // one set of atomics per workgroup: thousands of wavefronts updating the same four words take longer than
    // reading the offsets does
    constexpr int kWaves = kBlockThreads / kWave;
    __shared__ int32_t waveBest[kWaves], waveShort[kWaves], waveLong[kWaves];
    __shared__ uint32_t waveNnz[kWaves];
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
        waveBest[wave] = best;
        waveShort[wave] = bestShort;
        waveLong[wave] = numLong;
        waveNnz[wave] = nnzLong;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kWaves; ++w) {
            best = waveBest[w] > best ? waveBest[w] : best;
            bestShort = waveShort[w] > bestShort ? waveShort[w] : bestShort;
            numLong += waveLong[w];
            nnzLong += waveNnz[w];
        }
        if (best > 0) {
            atomicMax(stats, best);
            atomicMax(stats + 1, bestShort);
            if (numLong > 0) {
                atomicAdd(stats + 2, numLong);
                atomicAdd(reinterpret_cast<uint32_t *>(stats) + 3, nnzLong);
            }
        }
    }
}

// How local are the gathers of x?  Every `rowStride`-th row is sampled, up to 32 of its entries each:
// counts[0] = sampled entries, counts[1] = those whose column lies more than `band` away from where the
// row sits on the diagonal (row * cols / rows).  counts must be zeroed before the launch.
__global__ __launch_bounds__(kBlockThreads) void GatherLocalityKernel(const int32_t *__restrict__ rowOffsets,
                                                                      const int32_t *__restrict__ colInd, int64_t rows,
                                                                      int64_t cols, int64_t rowStride, int64_t band,
                                                                      int32_t *__restrict__ counts)
{
    int32_t seen = 0, far = 0;
    const int64_t sample = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    const int64_t r = sample * rowStride;
    if (r < rows) {
        const int64_t centre = static_cast<int64_t>(static_cast<double>(r) * static_cast<double>(cols) /
                                                    static_cast<double>(rows));
        const int32_t first = rowOffsets[r];
        int32_t last = rowOffsets[r + 1];
        last = last - first > 32 ? first + 32 : last;
        for (int32_t k = first; k < last; ++k) {
            const int64_t d = static_cast<int64_t>(colInd[k]) - centre;
            ++seen;
            far += (d > band || d < -band) ? 1 : 0;
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        seen += __shfl_xor(seen, off, kWave);
        far += __shfl_xor(far, off, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0 && seen > 0) {
        atomicAdd(counts, seen);
        atomicAdd(counts + 1, far);
    }
}

// ------------------------------------------------------------- STREAM_ROWS

constexpr int kStreamRowsMax = 767;  // rows of a stream-rows tile at most (their offsets pass through LDS)

// Four consecutive matrix entries of one lane, still in storage type.
template <typename ValT>
struct Quad {
    Int4U col;
    ValT val[4];
};

// Requests the block's entries [k, k + 4) for this lane's U quads.  Nothing is
// waited for here: the caller does other work while the loads are in flight.
template <typename ValT, int U>
__device__ __forceinline__ void IssueQuads(const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
                                           int32_t count, Quad<ValT> (&q)[U])
{
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int32_t k = (u * kBlockThreads + static_cast<int32_t>(threadIdx.x)) * 4;
        if (k + 4 <= count) {
            q[u].col = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(colInd + k));
            // The four values as one load, whatever their type (four 2-byte loads a quad cost the fp16 Laplacian
            // more than the bytes they save: 45.9 us against 41.3 us in fp32).
            static_assert(sizeof(ValT) == 4 || sizeof(ValT) == 2, "values of 2 or 4 bytes");
            if constexpr (sizeof(ValT) == 4) {
                const Int4U v = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(vals + k));
                __builtin_memcpy(q[u].val, &v, 16);
            } else {
                const Short4U v = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(vals + k));
                __builtin_memcpy(q[u].val, &v, 8);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // the ragged quad at the end of the range, and lanes past it
                if (k + i < count) {
                    q[u].col[i] = LoadStream(colInd + k + i);
                    q[u].val[i] = LoadStream(vals + k + i);
                }
            }
        }
    }
}

// Gathers x for the quads requested by IssueQuads and writes the products to LDS.
template <typename ValT, typename AccT, int U>
__device__ __forceinline__ void FinishQuads(const Quad<ValT> (&q)[U], const ValT *__restrict__ x, int32_t count,
                                            AccT *__restrict__ prod)
{
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int32_t k = (u * kBlockThreads + static_cast<int32_t>(threadIdx.x)) * 4;
        if (k + 4 <= count) {
            const AccT x0 = ToAcc<AccT>(x[q[u].col.x]);
            const AccT x1 = ToAcc<AccT>(x[q[u].col.y]);
            const AccT x2 = ToAcc<AccT>(x[q[u].col.z]);
            const AccT x3 = ToAcc<AccT>(x[q[u].col.w]);
            prod[k + 0] = ToAcc<AccT>(q[u].val[0]) * x0;
            prod[k + 1] = ToAcc<AccT>(q[u].val[1]) * x1;
            prod[k + 2] = ToAcc<AccT>(q[u].val[2]) * x2;
            prod[k + 3] = ToAcc<AccT>(q[u].val[3]) * x3;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (k + i < count) {
                    prod[k + i] = ToAcc<AccT>(q[u].val[i]) * ToAcc<AccT>(x[q[u].col[i]]);
                }
            }
        }
    }
}

// A workgroup walks over tiles of `rowsPerBlock` consecutive rows (at most
// 1024 * U non-zeros each).  Per tile: the tile's contiguous (colind, value)
// range arrives through IssueQuads, the products go to LDS, then G lanes per row
// add them up in stored order.  The loads of the NEXT tile are issued before the
// current tile is reduced, so the matrix stream never drains, and the row
// bounds / old y of a lane's first row are fetched a tile ahead as well.
// Workgroups of one XCD share one contiguous range of tiles and take them
// interleaved, so the x lines neighbouring tiles share are fetched into that
// XCD's L2 once.
template <typename ValT, typename OutT, typename AccT, int G, int U>
__global__ __launch_bounds__(kBlockThreads) void SpmvStreamRowsKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows, int32_t rowsPerBlock, int32_t capacity,
    int32_t skipLonger, OpsparseScalar alphaS, OpsparseScalar betaS)
{
    extern __shared__ __align__(16) unsigned char ldsRaw[];
    AccT *prod = reinterpret_cast<AccT *>(ldsRaw);

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));

    constexpr int kGroups = kBlockThreads / G;
    const int32_t lane = threadIdx.x % G;
    const int32_t group = threadIdx.x / G;

    // This XCD's tiles, and this workgroup's stride through them.
    const int64_t numTiles = (rows + rowsPerBlock - 1) / rowsPerBlock;
    const int64_t xcd = blockIdx.x % kNumXcd;
    const int64_t perXcd = numTiles / kNumXcd, rem = numTiles % kNumXcd;
    const int64_t xcdFirst = xcd * perXcd + (xcd < rem ? xcd : rem);
    const int64_t xcdTiles = perXcd + (xcd < rem ? 1 : 0);
    const int64_t stride = (gridDim.x - xcd + kNumXcd - 1) / kNumXcd;  // workgroups living on this XCD
    int64_t t = blockIdx.x / kNumXcd;
    if (t >= xcdTiles) {
        return;
    }

    int64_t r0 = (xcdFirst + t) * rowsPerBlock;
    int64_t r1 = (r0 + rowsPerBlock < rows) ? r0 + rowsPerBlock : rows;
    int32_t first = rowOffsets[r0];
    int32_t count = rowOffsets[r1] - first;
    // `capacity` products fit the LDS of this launch (rowsPerBlock times the longest row the statistics saw).  A
    // tile with more entries — the row offsets changed since — stages nothing and sums straight from memory.
    bool staged = count <= capacity;

    // The tile's row offsets and old y reach the lanes that sum the rows through LDS: they are asked for together
    // with the tile's entries, a tile ahead, and the loop that sums the rows then holds no load from memory at
    // all.  (Loads come back in the order they were issued: a row offset asked for inside that loop had to wait
    // for the next tile's entries, asked for just before it, and the tile ahead was no longer ahead - a 27-point
    // stencil on 128^3 points 163 us, 117 us with a workgroup a tile and nothing fetched ahead.)
    // (behind the products in the launch's LDS: rowsPerBlock old y, rowsPerBlock + 1 offsets)
    AccT *const yLds = prod + capacity;
    int32_t *const rowLds = reinterpret_cast<int32_t *>(yLds + rowsPerBlock);
    constexpr int kBoundRegs = (kStreamRowsMax + 1 + kBlockThreads - 1) / kBlockThreads;
    int32_t bnd[kBoundRegs];
    AccT yv[kBoundRegs];
    auto issueBounds = [&](int64_t rFirst, int64_t rEnd) {
#pragma unroll
        for (int k = 0; k < kBoundRegs; ++k) {
            const int64_t rr = rFirst + k * kBlockThreads + static_cast<int64_t>(threadIdx.x);
            bnd[k] = 0;
            yv[k] = AccT(0);
            if (rr <= rEnd) {
                bnd[k] = rowOffsets[rr];
                if (!betaZero && rr < rEnd) {
                    yv[k] = ToAcc<AccT>(yIn[rr]);
                }
            }
        }
    };
    Quad<ValT> q[U];
    IssueQuads<ValT, U>(colInd + first, vals + first, staged ? count : 0, q);
    issueBounds(r0, r1);

    while (true) {
        // Bounds of the next tile (needed after the barrier to ask for its entries).
        const int64_t tNext = t + stride;
        const bool more = tNext < xcdTiles;
        int64_t r0Next = 0, r1Next = 0;
        int32_t firstNext = 0, countNext = 0;
        if (more) {
            r0Next = (xcdFirst + tNext) * rowsPerBlock;
            r1Next = (r0Next + rowsPerBlock < rows) ? r0Next + rowsPerBlock : rows;
            firstNext = rowOffsets[r0Next];
            countNext = rowOffsets[r1Next] - firstNext;
        }
        const int32_t tileRows = static_cast<int32_t>(r1 - r0);
#pragma unroll
        for (int k = 0; k < kBoundRegs; ++k) {
            const int32_t rr = k * kBlockThreads + static_cast<int32_t>(threadIdx.x);
            if (rr <= tileRows) {
                rowLds[rr] = bnd[k];
                if (rr < tileRows) {
                    yLds[rr] = yv[k];
                }
            }
        }
        FinishQuads<ValT, AccT, U>(q, x, staged ? count : 0, prod);
        __syncthreads();
        const bool stagedNext = countNext <= capacity;
        if (more) {
            IssueQuads<ValT, U>(colInd + firstNext, vals + firstNext, stagedNext ? countNext : 0, q);
            issueBounds(r0Next, r1Next);
        }

        for (int32_t rr = group; rr < tileRows; rr += kGroups) {
            const int32_t s = rowLds[rr], e = rowLds[rr + 1];
            AccT sum = AccT(0);
            // skipLonger > 0: rows longer than that are SpmvLongRowsKernel's, which runs after this kernel
            const bool skip = skipLonger > 0 && e - s > skipLonger;
            if (skip) {
            } else if (staged) {
                for (int32_t k = s - first + lane; k < e - first; k += G) {
                    sum += prod[k];
                }
            } else {
                for (int64_t k = static_cast<int64_t>(s) + lane; k < e; k += G) {
                    sum += ToAcc<AccT>(vals[k]) * ToAcc<AccT>(x[colInd[k]]);
                }
            }
            sum = GroupSum<G>(sum);
            if (lane == 0 && !skip) {
                AccT res = alpha * sum;
                if (!betaZero) {
                    res += beta * yLds[rr];
                }
                y[r0 + rr] = FromAcc<OutT>(res);
            }
        }
        if (!more) {
            break;
        }
        __syncthreads();  // everyone is done with prod and the row tables before the next tile overwrites them
        t = tNext;
        r0 = r0Next;
        r1 = r1Next;
        first = firstNext;
        count = countNext;
        staged = stagedNext;
    }
}

// STREAM_ROWS for the shortest rows (one lane per row would do) with fp32 y:
// every lane owns FOUR consecutive rows, so the row offsets and y travel as
// 16-byte vectors (one dwordx4 per lane instead of four dword instructions per
// 64 rows; the memory pipeline of a CU handles far fewer instructions for the
// same bytes).  One tile per workgroup; rowsPerBlock is a multiple of 4 and at
// most 1024, rowOffsets and y are 16-byte aligned.
template <typename ValT, typename AccT, int U, bool GuardTiles>
__global__ __launch_bounds__(kBlockThreads) void SpmvStreamQuadRowsKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, float *y, const float *yIn, int64_t rows, int32_t rowsPerBlock, int32_t guard,
    OpsparseScalar alphaS, OpsparseScalar betaS)
{
    // guard (read by the GuardTiles instantiation only): the products the LDS of this launch holds in its low 16
    // bits, above them the row length beyond which rows are left to SpmvLongRowsKernel (0: none)
    const int32_t capacity = guard & 0xffff, skipLonger = guard >> 16;
    typedef int32_t Int4A __attribute__((ext_vector_type(4)));
    typedef float Float4A __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char ldsRaw[];
    AccT *prod = reinterpret_cast<AccT *>(ldsRaw);

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));

    const int64_t tile = XcdContiguousTile(blockIdx.x, gridDim.x);
    const int64_t r0 = tile * rowsPerBlock;
    const int64_t r1 = (r0 + rowsPerBlock < rows) ? r0 + rowsPerBlock : rows;
    const int32_t first = rowOffsets[r0];
    const int32_t count = rowOffsets[r1] - first;

    // Offsets of this lane's rows r .. r+3 (bound[i] .. bound[i+1]) and their old y.
    const int64_t r = r0 + 4 * static_cast<int64_t>(threadIdx.x);
    const int32_t mine = r >= r1 ? 0 : (r + 4 <= r1 ? 4 : static_cast<int32_t>(r1 - r));
    int32_t bound[5] = {0, 0, 0, 0, 0};
    float yOld[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (mine == 4) {
        const Int4A b = *reinterpret_cast<const Int4A *>(rowOffsets + r);
        bound[0] = b.x;
        bound[1] = b.y;
        bound[2] = b.z;
        bound[3] = b.w;
        bound[4] = rowOffsets[r + 4];
        if (!betaZero) {
            const Float4A o = *reinterpret_cast<const Float4A *>(yIn + r);
            yOld[0] = o.x;
            yOld[1] = o.y;
            yOld[2] = o.z;
            yOld[3] = o.w;
        }
    } else {
        for (int32_t i = 0; i < mine; ++i) {
            bound[i] = rowOffsets[r + i];
            bound[i + 1] = rowOffsets[r + i + 1];
            if (!betaZero) {
                yOld[i] = yIn[r + i];
            }
        }
    }

    if (GuardTiles && count > capacity) {
        // More entries than the LDS of this launch holds (rowsPerBlock times the longest row the statistics saw):
        // the row offsets changed since.  The tile is summed straight from memory.  (A flag of the instantiation:
        // the test alone costs the 2048 x 2048 Laplacian 0.5 us of 41.)
        for (int32_t i = 0; i < mine; ++i) {
            if (skipLonger > 0 && bound[i + 1] - bound[i] > skipLonger) {
                continue;  // SpmvLongRowsKernel's, which runs after this kernel
            }
            AccT sum = AccT(0);
            for (int32_t k = bound[i]; k < bound[i + 1]; ++k) {
                sum += ToAcc<AccT>(vals[k]) * ToAcc<AccT>(x[colInd[k]]);
            }
            AccT res = alpha * sum;
            if (!betaZero) {
                res += beta * static_cast<AccT>(yOld[i]);
            }
            y[r + i] = static_cast<float>(res);
        }
        return;
    }
    {
        Quad<ValT> q[U];
        IssueQuads<ValT, U>(colInd + first, vals + first, count, q);
        FinishQuads<ValT, AccT, U>(q, x, count, prod);
    }
    __syncthreads();

    float out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        AccT sum = AccT(0);
        if (i < mine) {
            for (int32_t k = bound[i] - first; k < bound[i + 1] - first; ++k) {
                sum += prod[k];
            }
        }
        AccT res = alpha * sum;
        if (!betaZero) {
            res += beta * static_cast<AccT>(yOld[i]);
        }
        out[i] = static_cast<float>(res);
        if (GuardTiles && skipLonger > 0 && i < mine && bound[i + 1] - bound[i] > skipLonger) {
            // a long row inside a tile that fitted: SpmvLongRowsKernel's; y keeps what it held (beta == 0: anything)
            out[i] = betaZero ? 0.0f : yOld[i];
        }
    }
    if (mine == 4) {
        Float4A o;
        o.x = out[0];
        o.y = out[1];
        o.z = out[2];
        o.w = out[3];
        *reinterpret_cast<Float4A *>(y + r) = o;
    } else {
        for (int32_t i = 0; i < mine; ++i) {
            y[r + i] = out[i];
        }
    }
}

// The rows the stream-rows kernels skipped (longer than minLen), for matrices of short rows with a few long ones
// among them — a mesh with some dense constraint rows, a graph with a few hubs: a workgroup looks at 256
// consecutive rows, lists the long ones in LDS and sums each of them with all its lanes, in fp64, in a fixed order.
constexpr int kLongScanRows = 16;   // rows a lane looks at in SpmvLongRowsKernel's first pass (at most 32: a bit each)

template <typename ValT, typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvLongRowsKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows, int32_t minLen, OpsparseScalar alphaS,
    OpsparseScalar betaS)
{
    constexpr int kWaves = kBlockThreads / kWave;
    constexpr int64_t kSpan = static_cast<int64_t>(kBlockThreads) * kLongScanRows;  // rows of one workgroup
    __shared__ int32_t listed[kBlockThreads];
    __shared__ int32_t numListed;
    __shared__ AccT waveSum[kWaves];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int64_t span0 = static_cast<int64_t>(blockIdx.x) * kSpan;
    // Coarse pass: is any of this workgroup's rows long?  Nearly always not, and the workgroup is done after
    // reading its offsets once.
    __shared__ uint32_t groupsWithLong;  // bit i: a long row among rows span0 + 256 i ... + 255
    if (threadIdx.x == 0) {
        groupsWithLong = 0;
    }
    __syncthreads();
    uint32_t mine = 0;  // bit i: row span0 + 256 i + threadIdx.x is long (neighbouring rows in neighbouring lanes)
#pragma unroll
    for (int i = 0; i < kLongScanRows; ++i) {
        const int64_t r = span0 + static_cast<int64_t>(i) * kBlockThreads + threadIdx.x;
        if (r < rows && rowOffsets[r + 1] - rowOffsets[r] > minLen) {
            mine |= 1u << i;
        }
    }
    if (mine != 0) {
        atomicOr(&groupsWithLong, mine);
    }
    __syncthreads();
    const AccT alpha = ReadScalar<AccT>(alphaS), beta = ReadScalar<AccT>(betaS);
    for (uint32_t todo = groupsWithLong; todo != 0; todo &= todo - 1) {
        const int g = __ffs(static_cast<int>(todo)) - 1;
        const int64_t base = span0 + static_cast<int64_t>(g) * kBlockThreads;
        const bool isLong = (mine >> g) & 1u;
        if (threadIdx.x == 0) {
            numListed = 0;
        }
        __syncthreads();
        // listed in row order (a ballot per wavefront, the wavefronts one after the other), so that nothing about
        // the result depends on the order in which lanes arrive
        const uint64_t votes = __ballot(isLong);
        for (int w = 0; w < kWaves; ++w) {
            if (w == wave && isLong) {
                listed[numListed + __popcll(votes & ((uint64_t{1} << lane) - 1))] = static_cast<int32_t>(threadIdx.x);
            }
            __syncthreads();
            if (w == wave && lane == 0) {
                numListed += __popcll(votes);
            }
            __syncthreads();
        }
        const int32_t count = numListed;
        for (int32_t i = 0; i < count; ++i) {
            const int64_t row = base + listed[i];
            const int64_t e = rowOffsets[row + 1];
            // four entries per lane and round, loaded unconditionally (past the end: the last entry again, counted
            // as zero), so that four gathers are in flight: one workgroup is alone with this row
            AccT part[4] = {AccT(0), AccT(0), AccT(0), AccT(0)};
            for (int64_t k = static_cast<int64_t>(rowOffsets[row]) + threadIdx.x; k < e; k += 4 * kBlockThreads) {
                int32_t c[4];
                AccT v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int64_t ku = k + static_cast<int64_t>(u) * kBlockThreads;
                    const int64_t at = ku < e ? ku : e - 1;
                    c[u] = LoadStream(colInd + at);
                    v[u] = ku < e ? ToAcc<AccT>(LoadStream(vals + at)) : AccT(0);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    part[u] += v[u] * ToAcc<AccT>(x[c[u]]);
                }
            }
            AccT sum = (part[0] + part[1]) + (part[2] + part[3]);
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) {
                sum += __shfl_xor(sum, off, kWave);
            }
            if (lane == 0) {
                waveSum[wave] = sum;
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                AccT total = waveSum[0];
#pragma unroll
                for (int w = 1; w < kWaves; ++w) {
                    total += waveSum[w];
                }
                StoreRow<OutT, AccT>(y, yIn, row, total, alpha, beta, beta == AccT(0));
            }
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------- VECTOR_ROWS

template <typename ValT, typename OutT, typename AccT, int G>
__global__ __launch_bounds__(kBlockThreads) void SpmvVectorRowsKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows, OpsparseScalar alphaS, OpsparseScalar betaS)
{
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));

    constexpr int kGroups = kBlockThreads / G;
    const int64_t tile = XcdContiguousTile(blockIdx.x, gridDim.x);
    const int64_t r = tile * kGroups + threadIdx.x / G;
    const int32_t lane = threadIdx.x % G;
    if (r >= rows) {
        return;  // whole groups leave together: G divides the wavefront
    }
    const int32_t s = rowOffsets[r];
    const int32_t e = rowOffsets[r + 1];
    AccT sum0 = AccT(0), sum1 = AccT(0);
    int64_t k = static_cast<int64_t>(s) + lane;  // 64 bits: k + 2 G may pass 2^31 when nnz is close to it
    for (; k + G < e; k += 2 * G) {  // two independent gathers in flight per lane
        const int32_t c0 = LoadStream(colInd + k);
        const int32_t c1 = LoadStream(colInd + k + G);
        const AccT v0 = ToAcc<AccT>(LoadStream(vals + k));
        const AccT v1 = ToAcc<AccT>(LoadStream(vals + k + G));
        sum0 += v0 * ToAcc<AccT>(x[c0]);
        sum1 += v1 * ToAcc<AccT>(x[c1]);
    }
    if (k < e) {
        sum0 += ToAcc<AccT>(LoadStream(vals + k)) * ToAcc<AccT>(x[LoadStream(colInd + k)]);
    }
    const AccT sum = GroupSum<G>(sum0 + sum1);
    if (lane == 0) {
        StoreRow<OutT, AccT>(y, yIn, r, sum, alpha, beta, betaZero);
    }
}

// The same lane-group-per-row scheme for the index variants the SpMVOp API
// admits and the kernels above do not: 64-bit row offsets and / or index base 1
// (reference sparse/spmv_op/arch35/spmv_op_kernel.cpp:139-181 handles them in its
// one thread-per-row kernel).
template <typename RowT, typename ValT, typename OutT, typename AccT, int G>
__global__ __launch_bounds__(kBlockThreads) void SpmvIndexedRowsKernel(
    const RowT *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows, int32_t indexBase, OpsparseScalar alphaS,
    OpsparseScalar betaS)
{
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    constexpr int kGroups = kBlockThreads / G;
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kGroups + threadIdx.x / G;
    const int32_t lane = threadIdx.x % G;
    if (r >= rows) {
        return;
    }
    const int64_t s = static_cast<int64_t>(rowOffsets[r]) - indexBase;
    const int64_t e = static_cast<int64_t>(rowOffsets[r + 1]) - indexBase;
    AccT sum = AccT(0);
    for (int64_t k = s + lane; k < e; k += G) {
        sum += ToAcc<AccT>(LoadStream(vals + k)) * ToAcc<AccT>(x[LoadStream(colInd + k) - indexBase]);
    }
    sum = GroupSum<G>(sum);
    if (lane == 0) {
        StoreRow<OutT, AccT>(y, yIn, r, sum, alpha, beta, betaZero);
    }
}

// ------------------------------------------------------------- MERGE_PATH

constexpr int kMergeItems = 2048;  // rows + non-zeros consumed by one workgroup

__device__ __forceinline__ int64_t MergeDiagonal(int64_t block, int64_t rows, int64_t nnz)
{
    const int64_t d = block * kMergeItems;
    return d < rows + nnz ? d : rows + nnz;
}

// out[i] = in[i] - base as int32: row offsets of either width and index base for the kernels below.
template <typename RowT>
__global__ __launch_bounds__(kBlockThreads) void RebaseOffsetsKernel(const RowT *__restrict__ in, int64_t count,
                                                                     int32_t base, int32_t *__restrict__ out)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
        out[i] = static_cast<int32_t>(static_cast<int64_t>(in[i]) - base);
    }
}

__device__ __forceinline__ int64_t ClampTo(int64_t v, int64_t lo, int64_t hi)
{
    return v < lo ? lo : (v > hi ? hi : v);
}

// part[b] = number of rows completed before diagonal b * kMergeItems of the
// merge of (row end offsets, non-zero indices): the smallest i with
// rowOffsets[i + 1] > d - i - 1.
__global__ __launch_bounds__(kBlockThreads) void MergePartitionKernel(const int32_t *__restrict__ rowOffsets,
                                                                      int64_t rows, int64_t nnz, int32_t numBlocks,
                                                                      int32_t *__restrict__ part)
{
    const int64_t b = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    if (b > numBlocks) {
        return;
    }
    const int64_t d = MergeDiagonal(b, rows, nnz);
    int64_t lo = d > nnz ? d - nnz : 0;
    int64_t hi = d < rows ? d : rows;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (static_cast<int64_t>(rowOffsets[mid + 1]) <= d - mid - 1) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    part[b] = static_cast<int32_t>(lo);
}

template <typename OutT, typename AccT>
__device__ __forceinline__ void MergeTileRows(int64_t b, int64_t i0, int64_t i1, int64_t j0, int32_t count,
                                              const int32_t *__restrict__ rowOffsets, OutT *y, const OutT *yIn,
                                              int64_t rows, AccT *__restrict__ carry, AccT *__restrict__ head,
                                              AccT alpha, AccT beta, bool betaZero, const AccT *prod);

// Workgroup b consumes non-zeros [j0, j1) and completes rows [i0, i1), where
// (i0, j0) and (i1, j1) are the merge-path coordinates of its two diagonals.
//   - a completed row that started before j0 ("spanning" row, only i0 can be
//     one) is not written here: its last piece goes to head[b];
//   - the non-zeros after the last completed row belong to row i1, which ends
//     in a later workgroup: their sum goes to carry[b];
//   - every other completed row gets its final y value here.
template <typename ValT, typename OutT, typename AccT>
__device__ __forceinline__ void MergeTile(int64_t b, const int32_t *__restrict__ rowOffsets,
                                          const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
                                          const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows,
                                          int64_t nnz, const int32_t *__restrict__ part, AccT *__restrict__ carry,
                                          AccT *__restrict__ head, AccT alpha, AccT beta, bool betaZero,
                                          AccT *prod /* [kMergeItems] in LDS */)
{
    // The partition comes from a buffer the caller owns: whatever it holds, rows stay inside [0, rows] and the
    // entries of a tile inside [0, nnz] and inside the tile's LDS (a stale buffer gives wrong numbers, never an
    // access out of range).
    const int64_t i0 = ClampTo(part[b], 0, rows);
    const int64_t i1 = ClampTo(part[b + 1], i0, rows);
    const int64_t j0 = ClampTo(MergeDiagonal(b, rows, nnz) - i0, 0, nnz);
    const int64_t j1 = ClampTo(MergeDiagonal(b + 1, rows, nnz) - i1, j0, j0 + kMergeItems < nnz ? j0 + kMergeItems : nnz);
    const int32_t count = static_cast<int32_t>(j1 - j0);

    {
        Quad<ValT> q[2];  // 2 x 1024 entries cover the whole workgroup share
        IssueQuads<ValT, 2>(colInd + j0, vals + j0, count, q);
        FinishQuads<ValT, AccT, 2>(q, x, count, prod);
    }
    __syncthreads();
    MergeTileRows<OutT, AccT>(b, i0, i1, j0, count, rowOffsets, y, yIn, rows, carry, head, alpha, beta, betaZero, prod);
}

// The row phase of a merge tile: prod[0..count) holds the products of non-zeros
// j0 .. j0+count-1.
template <typename OutT, typename AccT>
__device__ __forceinline__ void MergeTileRows(int64_t b, int64_t i0, int64_t i1, int64_t j0, int32_t count,
                                              const int32_t *__restrict__ rowOffsets, OutT *y, const OutT *yIn,
                                              int64_t rows, AccT *__restrict__ carry, AccT *__restrict__ head,
                                              AccT alpha, AccT beta, bool betaZero, const AccT *prod)
{
    // Rows i0 .. i1-1 complete here; row i1 (if it exists) collects the tail.
    const int32_t numRows = static_cast<int32_t>(i1 - i0) + (i1 < rows ? 1 : 0);
    if (numRows == 0) {
        return;
    }
    // Lanes per row from the average row length of this workgroup.
    int g = 1;
    while (g < kWave && count > 8 * g * numRows) {
        g <<= 1;
    }
    const int32_t groups = kBlockThreads / g;
    const int32_t lane = threadIdx.x & (g - 1);
    for (int32_t q = threadIdx.x / g; q < numRows; q += groups) {
        const int64_t row = i0 + q;
        const bool completes = row < i1;
        const int64_t begin = LoadStream(rowOffsets + row);
        const int32_t s = begin > j0 ? static_cast<int32_t>(begin - j0 < count ? begin - j0 : count) : 0;
        const int64_t rowEnd = completes ? static_cast<int64_t>(LoadStream(rowOffsets + row + 1)) - j0 : count;
        const int32_t e = static_cast<int32_t>(rowEnd < count ? rowEnd : count);  // inside the staged products
        AccT sum = AccT(0);
        for (int32_t k = s + lane; k < e; k += g) {
            sum += prod[k];
        }
        sum = GroupSumDyn(sum, g);
        if (lane == 0) {
            if (!completes) {
                carry[b] = sum;
            } else if (begin < j0) {
                head[b] = sum;
            } else {
                StoreRow<OutT, AccT>(y, yIn, row, sum, alpha, beta, betaZero);
            }
        }
    }
}

template <typename ValT, typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvMergeKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, OutT *y, const OutT *yIn, int64_t rows, int64_t nnz,
    const int32_t *__restrict__ part, AccT *__restrict__ carry, AccT *__restrict__ head, OpsparseScalar alphaS,
    OpsparseScalar betaS)
{
    __shared__ AccT prod[kMergeItems];
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    MergeTile<ValT, OutT, AccT>(XcdContiguousTile(blockIdx.x, gridDim.x), rowOffsets, colInd, vals, x, y, yIn, rows, nnz,
                                part, carry, head, alpha, beta, beta == AccT(0), prod);
}

// The workgroup in which row i0, which ends in workgroup b, starts: the largest p < b whose first entry is not
// after `begin` (the first entry of a workgroup grows with its number, so this is a bisection).
__device__ __forceinline__ int64_t MergeRowFirstBlock(int64_t b, int64_t begin, int64_t rows, int64_t nnz,
                                                      const int32_t *__restrict__ part)
{
    int64_t lo = 0, hi = b - 1;
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (MergeDiagonal(mid, rows, nnz) - part[mid] <= begin) {
            lo = mid;
        } else {
            hi = mid - 1;
        }
    }
    return lo;
}

// Workgroup b of a merge kernel: if it completed a spanning row, add the carries of the workgroups the row passed
// through (in ascending order) to its head piece and write the row's final value.
template <typename OutT, typename AccT>
__device__ __forceinline__ void MergeFixupTile(int64_t b, const int32_t *__restrict__ rowOffsets, OutT *y,
                                               const OutT *yIn, int64_t rows, int64_t nnz,
                                               const int32_t *__restrict__ part, const AccT *__restrict__ carry,
                                               const AccT *__restrict__ head, AccT alpha, AccT beta)
{
    const int64_t i0 = part[b];
    const int64_t i1 = part[b + 1];
    if (i1 <= i0) {
        return;  // no row ends in this workgroup
    }
    const int64_t begin = rowOffsets[i0];
    if (begin >= MergeDiagonal(b, rows, nnz) - i0) {
        return;  // first completed row also starts here
    }
    AccT sum = AccT(0);
    for (int64_t p = MergeRowFirstBlock(b, begin, rows, nnz, part); p < b; ++p) {
        sum += carry[p];
    }
    sum += head[b];
    StoreRow<OutT, AccT>(y, yIn, i0, sum, alpha, beta, beta == AccT(0));
}

// Lane b stands for workgroup b of the merge kernel: if that workgroup completed a spanning row, the carries of the
// workgroups the row passed through and its own head piece make the row's final value.  The workgroup in which the
// row starts is found by bisection (the first entry of a workgroup grows with its number), and a row that passed
// through more than 64 workgroups — a row of well over a hundred thousand entries — has its carries added by the
// whole wavefront, 64 at a time, instead of one lane walking them (one row of 20 M entries: 2.4 -> 0.4 ms).
template <typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvMergeFixupKernel(
    const int32_t *__restrict__ rowOffsets, OutT *y, const OutT *yIn, int64_t rows, int64_t nnz, int32_t numBlocks,
    const int32_t *__restrict__ part, const AccT *__restrict__ carry, const AccT *__restrict__ head,
    OpsparseScalar alphaS, OpsparseScalar betaS)
{
    const AccT alpha = ReadScalar<AccT>(alphaS), beta = ReadScalar<AccT>(betaS);
    const int64_t b = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    const int lane = threadIdx.x % kWave;
    int64_t i0 = 0, first = b;  // first: the workgroup in which the spanning row starts
    bool spanning = false;
    if (b < numBlocks) {
        i0 = ClampTo(part[b], 0, rows);
        const int64_t i1 = ClampTo(part[b + 1], i0, rows);
        if (i1 > i0) {  // a row ends in this workgroup
            const int64_t begin = rowOffsets[i0];
            if (begin < MergeDiagonal(b, rows, nnz) - i0) {  // and it started before it
                spanning = true;
                first = MergeRowFirstBlock(b, begin, rows, nnz, part);
            }
        }
    }
    AccT sum = AccT(0);
    const bool wide = spanning && b - first > kWave;
    if (spanning && !wide) {
        for (int64_t p = first; p < b; ++p) {
            sum += carry[p];
        }
    }
    // rows that passed through many workgroups, one after the other, all lanes of the wavefront adding
    for (uint64_t todo = __ballot(wide); todo != 0; todo &= todo - 1) {
        const int owner = __ffsll(static_cast<unsigned long long>(todo)) - 1;
        const int64_t from = __shfl(first, owner), to = __shfl(b, owner);
        AccT piece = AccT(0);
        for (int64_t p = from + lane; p < to; p += kWave) {
            piece += carry[p];
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            piece += __shfl_xor(piece, off);
        }
        if (lane == owner) {
            sum = piece;
        }
    }
    if (spanning) {
        sum += head[b];
        StoreRow<OutT, AccT>(y, yIn, i0, sum, alpha, beta, beta == AccT(0));
    }
}

// --------------------------------------------------------- COLUMN_PANELS
// For matrices whose x does not fit an L2 (4 MB per XCD): the matrix is split at
// Preprocess into panels of 2^20 columns, each a CSR matrix of its own over all
// rows, and panel p is worked only by workgroups whose id is p modulo 8 — the
// hardware deals workgroup ids round-robin to the 8 XCDs, so the 4 MiB slice of
// x a panel gathers from stays in that XCD's L2 (measured: 181 G gathers/s
// against 64 G/s for gathers over all of x).  Every panel is a merge-path SpMV
// into its own fp64 partial vector; a last kernel adds a row's partials in panel
// order and applies alpha / beta.  Deterministic, no atomics.

struct PanelTable {
    int64_t start[OPSPARSE_SPMV_MAX_PANELS + 1];  // first entry of every panel in the panel-ordered arrays
};

__device__ __forceinline__ int64_t PanelTiles(int64_t rows, int64_t nnzP)
{
    return (rows + nnzP + kMergeItems - 1) / kMergeItems;
}

// Workgroup b: panel panelBase + b % 8, merge tile b / 8 of that panel.  (A
// persistent variant that requested the next tile's entries ahead of the row
// phase measured slower than letting the hardware schedule one short workgroup
// per tile: 986 against 859 us on an 8 M x 8 M power-law matrix.)
template <typename ValT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvPanelMergeKernel(
    const int32_t *__restrict__ rowPtrP, const int32_t *__restrict__ colIndP, const ValT *__restrict__ valsP,
    const ValT *__restrict__ x, AccT *__restrict__ ypart, int64_t rows, PanelTable pt, int32_t panelBase,
    int32_t numPanels, const int32_t *__restrict__ partAll, AccT *__restrict__ carryAll, AccT *__restrict__ headAll,
    int64_t tileBound)
{
    __shared__ AccT prod[kMergeItems];
    const int32_t p = panelBase + static_cast<int32_t>(blockIdx.x % kNumXcd);
    const int64_t tile = blockIdx.x / kNumXcd;
    if (p >= numPanels) {
        return;
    }
    const int64_t nnzP = pt.start[p + 1] - pt.start[p];
    if (tile >= PanelTiles(rows, nnzP)) {
        return;
    }
    AccT *yp = ypart + static_cast<int64_t>(p) * rows;
    MergeTile<ValT, AccT, AccT>(tile, rowPtrP + static_cast<int64_t>(p) * (rows + 1), colIndP + pt.start[p],
                                valsP + pt.start[p], x, yp, yp, rows, nnzP, partAll + static_cast<int64_t>(p) * (tileBound + 1),
                                carryAll + static_cast<int64_t>(p) * tileBound, headAll + static_cast<int64_t>(p) * tileBound,
                                AccT(1), AccT(0), true, prod);
}

// blockIdx.y = panel.
template <typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvPanelFixupKernel(const int32_t *__restrict__ rowPtrP,
                                                                     AccT *__restrict__ ypart, int64_t rows,
                                                                     PanelTable pt,
                                                                     const int32_t *__restrict__ partAll,
                                                                     const AccT *__restrict__ carryAll,
                                                                     const AccT *__restrict__ headAll,
                                                                     int64_t tileBound)
{
    const int32_t p = blockIdx.y;
    const int64_t b = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    const int64_t nnzP = pt.start[p + 1] - pt.start[p];
    if (b >= PanelTiles(rows, nnzP)) {
        return;
    }
    AccT *yp = ypart + static_cast<int64_t>(p) * rows;
    MergeFixupTile<AccT, AccT>(b, rowPtrP + static_cast<int64_t>(p) * (rows + 1), yp, yp, rows, nnzP,
                               partAll + static_cast<int64_t>(p) * (tileBound + 1),
                               carryAll + static_cast<int64_t>(p) * tileBound,
                               headAll + static_cast<int64_t>(p) * tileBound, AccT(1), AccT(0));
}

// y[r] = alpha * (ypart[0][r] + ... + ypart[P-1][r]) + beta * yIn[r], partials added in panel order.
template <typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvPanelCombineKernel(const AccT *__restrict__ ypart,
                                                                       int32_t numPanels, int64_t rows, OutT *y,
                                                                       const OutT *yIn, OpsparseScalar alphaS,
                                                                       OpsparseScalar betaS)
{
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; r < rows; r += stride) {
        AccT sum = AccT(0);
        for (int32_t p = 0; p < numPanels; ++p) {
            sum += LoadStream(ypart + static_cast<int64_t>(p) * rows + r);
        }
        StoreRow<OutT, AccT>(y, yIn, r, sum, alpha, beta, betaZero);
    }
}

// ------------------------------------------------------------- op(A) = A^T

// y[col] += alpha * x[row] * val for every stored element; y was scaled by
// beta beforehand.  Hardware atomic add on fp32 y: the order of the additions
// is not fixed, as in the reference's transpose path
// (sparse/spmv/arch22/kernels/spmv_kernel.h:584-624).  On int32 y (int32
// compute type) the additions wrap around, so their order does not show.
template <typename ValT, typename AccT, int G, typename YT = float>
__global__ __launch_bounds__(kBlockThreads) void SpmvTransposeScatterKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, YT *__restrict__ y, int64_t rows, int32_t maxLen, OpsparseScalar alphaS)
{
    const AccT alpha = ReadScalar<AccT>(alphaS);
    constexpr int kGroups = kBlockThreads / G;
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kGroups + threadIdx.x / G;
    if (r >= rows) {
        return;
    }
    const AccT ax = alpha * ToAcc<AccT>(x[r]);
    if (ax == AccT(0)) {
        return;
    }
    const int32_t e = rowOffsets[r + 1];
    if (e - rowOffsets[r] > maxLen) {
        return;  // left to SpmvTransposeLongRowsKernel
    }
    for (int64_t k = static_cast<int64_t>(rowOffsets[r]) + threadIdx.x % G; k < e; k += G) {
        atomicAdd(y + LoadStream(colInd + k), static_cast<YT>(ax * ToAcc<AccT>(LoadStream(vals + k))));
    }
}

// The rows the scatter kernel skipped (longer than minLen): a workgroup looks at 256 consecutive rows, lists the
// long ones among them in LDS and walks each of them with all its lanes.  With it a lane group is never left alone
// with a row of thousands of entries, and nothing has to be searched for: a matrix of short rows with a few long
// ones costs one more pass over the row offsets.
template <typename ValT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvTransposeLongRowsKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, float *__restrict__ y, int64_t rows, int32_t minLen, OpsparseScalar alphaS)
{
    __shared__ int32_t listed[kBlockThreads];
    __shared__ int32_t numListed;
    if (threadIdx.x == 0) {
        numListed = 0;
    }
    __syncthreads();
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    if (r < rows && rowOffsets[r + 1] - rowOffsets[r] > minLen) {
        listed[atomicAdd(&numListed, 1)] = static_cast<int32_t>(threadIdx.x);
    }
    __syncthreads();
    const int32_t count = numListed;
    if (count == 0) {
        return;
    }
    const AccT alpha = ReadScalar<AccT>(alphaS);
    for (int32_t i = 0; i < count; ++i) {
        const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlockThreads + listed[i];
        const AccT ax = alpha * ToAcc<AccT>(x[row]);
        if (ax == AccT(0)) {
            continue;
        }
        const int64_t e = rowOffsets[row + 1];
        for (int64_t k = static_cast<int64_t>(rowOffsets[row]) + threadIdx.x; k < e; k += kBlockThreads) {
            atomicAdd(y + LoadStream(colInd + k), static_cast<float>(ax * ToAcc<AccT>(LoadStream(vals + k))));
        }
    }
}

// Row that holds entry k: the largest r in [lo, hi] with offsets[r] <= k.
__device__ __forceinline__ int64_t RowOfEntry(const int32_t *offsets, int64_t lo, int64_t hi, int32_t k)
{
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (offsets[mid] <= k) {
            lo = mid;
        } else {
            hi = mid - 1;
        }
    }
    return lo;
}

constexpr int kTransposeTile = 2048;      // entries per workgroup
constexpr int kTransposeFewRows = 8192;   // fewer rows than this: split by entries instead of by rows
constexpr int kTransposeLongRow = 512;    // a row longer than this is walked by a whole workgroup
constexpr int kTransposeRowSlots = 2304;  // row offsets of one tile staged in LDS

// The same product with equal numbers of ENTRIES per workgroup, whatever the row lengths: a tile of
// kTransposeTile consecutive entries, the offsets of the rows it touches staged in LDS, every lane finds the
// row of its entries there.  A row of 200 000 entries is spread over a hundred workgroups instead of being
// walked by one lane group.
template <typename ValT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvTransposeFlatKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, float *__restrict__ y, int64_t rows, int64_t nnz, OpsparseScalar alphaS)
{
    __shared__ int32_t slice[kTransposeRowSlots];
    __shared__ int64_t bounds[2];
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const int64_t k0 = static_cast<int64_t>(blockIdx.x) * kTransposeTile;
    const int64_t k1 = k0 + kTransposeTile < nnz ? k0 + kTransposeTile : nnz;
    if (threadIdx.x < 2) {
        const int32_t k = static_cast<int32_t>(threadIdx.x == 0 ? k0 : k1 - 1);
        bounds[threadIdx.x] = RowOfEntry(rowOffsets, 0, rows - 1, k);
    }
    __syncthreads();
    const int64_t rLo = bounds[0], rHi = bounds[1];
    const bool staged = rHi - rLo + 2 <= kTransposeRowSlots;
    if (staged) {
        for (int64_t i = threadIdx.x; i <= rHi - rLo + 1; i += kBlockThreads) {
            slice[i] = rowOffsets[rLo + i];
        }
    }
    __syncthreads();
    for (int64_t k = k0 + threadIdx.x; k < k1; k += kBlockThreads) {
        const int32_t kk = static_cast<int32_t>(k);
        const int64_t r = staged ? rLo + RowOfEntry(slice, 0, rHi - rLo, kk) : RowOfEntry(rowOffsets, rLo, rHi, kk);
        const AccT ax = alpha * ToAcc<AccT>(x[r]);
        if (ax != AccT(0)) {
            atomicAdd(y + LoadStream(colInd + k), static_cast<float>(ax * ToAcc<AccT>(LoadStream(vals + k))));
        }
    }
}

constexpr int kNarrowCols = 16384;       // y of op(A) = A^T kept per workgroup in LDS up to this many columns
constexpr int kNarrowMaxBlocks = 1024;

// op(A) = A^T with few columns: millions of atomic updates would fall on a handful of addresses (40 000 rows of 120
// entries over 9 columns: half a million fp32 adds per element of y, one after the other in the L2).  Every
// workgroup instead takes a contiguous run of entry tiles, adds its products up in an fp64 copy of y in LDS, and
// at the end adds each non-zero element of that copy to y once: at most kNarrowMaxBlocks fp32 updates per element.
template <typename ValT, typename AccT, int Capacity>
__global__ __launch_bounds__(kBlockThreads) void SpmvTransposeNarrowKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ x, float *__restrict__ y, int64_t rows, int64_t cols, int64_t nnz, int64_t tilesPerBlock,
    OpsparseScalar alphaS)
{
    __shared__ AccT sums[Capacity];  // 64 KiB (two workgroups per CU) or 128 KiB
    __shared__ int32_t slice[kTransposeRowSlots];
    __shared__ int64_t bounds[2];
    const AccT alpha = ReadScalar<AccT>(alphaS);
    for (int64_t c = threadIdx.x; c < cols; c += kBlockThreads) {
        sums[c] = AccT(0);
    }
    const int64_t numTiles = (nnz + kTransposeTile - 1) / kTransposeTile;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * tilesPerBlock;
    const int64_t t1 = t0 + tilesPerBlock < numTiles ? t0 + tilesPerBlock : numTiles;
    for (int64_t t = t0; t < t1; ++t) {
        const int64_t k0 = t * kTransposeTile;
        const int64_t k1 = k0 + kTransposeTile < nnz ? k0 + kTransposeTile : nnz;
        __syncthreads();  // the previous tile's slice is no longer read; the first time: sums are zero
        if (threadIdx.x < 2) {
            const int32_t k = static_cast<int32_t>(threadIdx.x == 0 ? k0 : k1 - 1);
            bounds[threadIdx.x] = RowOfEntry(rowOffsets, 0, rows - 1, k);
        }
        __syncthreads();
        const int64_t rLo = bounds[0], rHi = bounds[1];
        const bool staged = rHi - rLo + 2 <= kTransposeRowSlots;
        if (staged) {
            for (int64_t i = threadIdx.x; i <= rHi - rLo + 1; i += kBlockThreads) {
                slice[i] = rowOffsets[rLo + i];
            }
        }
        __syncthreads();
        for (int64_t k = k0 + threadIdx.x; k < k1; k += kBlockThreads) {
            const int32_t kk = static_cast<int32_t>(k);
            const int64_t r = staged ? rLo + RowOfEntry(slice, 0, rHi - rLo, kk) : RowOfEntry(rowOffsets, rLo, rHi, kk);
            const int32_t c = LoadStream(colInd + k);
            if (c >= 0 && c < cols) {  // an index outside y must not reach LDS
                atomicAdd(&sums[c], alpha * ToAcc<AccT>(x[r]) * ToAcc<AccT>(LoadStream(vals + k)));
            }
        }
    }
    __syncthreads();
    for (int64_t c = threadIdx.x; c < cols; c += kBlockThreads) {
        const AccT v = sums[c];
        if (v != AccT(0)) {
            atomicAdd(y + c, static_cast<float>(v));
        }
    }
}

// =============================================================== host side

namespace {

// Number of compute units of the current device (256 on MI355X), read once.
inline int ComputeUnits()
{
    static const int cus = [] {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess ||
            prop.multiProcessorCount <= 0) {
            (void)hipGetLastError();
            return 256;
        }
        return prop.multiProcessorCount;
    }();
    return cus;
}

// Workgroups per CU of the persistent STREAM_ROWS launch (tuning override:
// OPS_SPARSE_STREAM_BLOCKS_PER_CU).
inline int StreamBlocksPerCu()
{
    static const int n = [] {
        const char *env = std::getenv("OPS_SPARSE_STREAM_BLOCKS_PER_CU");
        const int v = env != nullptr ? std::atoi(env) : 0;
        return (v >= 1 && v <= 64) ? v : 8;
    }();
    return n;
}

inline uint32_t GridFor(int64_t items, int64_t perBlock)
{
    return static_cast<uint32_t>((items + perBlock - 1) / perBlock);
}

struct MergeLayout {
    int32_t blocks;
    int64_t partOff, carryOff, headOff, bytes;
};

// Workspace layout of the merge-path family: 256-byte header (row statistics),
// partition table, carries, heads.  Carries are sized for the widest
// accumulator (8 bytes).
MergeLayout MakeMergeLayout(int64_t rows, int64_t nnz)
{
    MergeLayout l{};
    l.blocks = static_cast<int32_t>((rows + nnz + kMergeItems - 1) / kMergeItems);
    l.partOff = 256;
    l.carryOff = l.partOff + static_cast<int64_t>((static_cast<size_t>(l.blocks) + 1) * 4 + 255) / 256 * 256;
    l.headOff = l.carryOff + static_cast<int64_t>((static_cast<size_t>(l.blocks)) * 8 + 255) / 256 * 256;
    l.bytes = l.headOff + static_cast<int64_t>((static_cast<size_t>(l.blocks)) * 8 + 255) / 256 * 256;
    return l;
}

template <typename ValT, typename OutT, typename AccT, int G, int U>
int LaunchStreamU(const SpmvArgs &a, int32_t rowsPerBlock, size_t products, int32_t skipLonger)
{
    // the products of a tile, and behind them its old y and row offsets
    const size_t lds = products * sizeof(AccT) + static_cast<size_t>(rowsPerBlock) * sizeof(AccT) +
                       (static_cast<size_t>(rowsPerBlock) + 1) * sizeof(int32_t);
    if (rowsPerBlock < 1 || rowsPerBlock > kStreamRowsMax) {
        return OPSPARSE_E_INVALID;
    }
    // Persistent launch: the workgroups that fit a CU at once (eight at most) walk over all tiles.  One more than
    // fit would start when the first is done and finish last (8 asked for where 7 fit: 163 us against 127 us).
    const uint32_t tiles = GridFor(a.rows, rowsPerBlock);
    // (asked of the runtime once per kernel and LDS size and thread)
    thread_local size_t fitLds = ~static_cast<size_t>(0);
    thread_local int fit = 1;
    if (fitLds != lds) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit, SpmvStreamRowsKernel<ValT, OutT, AccT, G, U>,
                                                         kBlockThreads, lds) != hipSuccess ||
            fit < 1) {
            (void)hipGetLastError();
            fit = 1;
        }
        fitLds = lds;
    }
    const int perCu = StreamBlocksPerCu() < fit ? StreamBlocksPerCu() : fit;
    const uint32_t resident = static_cast<uint32_t>(ComputeUnits() * perCu);
    const uint32_t grid = tiles < resident ? tiles : resident;
    hipLaunchKernelGGL((SpmvStreamRowsKernel<ValT, OutT, AccT, G, U>), dim3(grid), dim3(kBlockThreads), lds, a.stream,
                       a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                       static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.rows, rowsPerBlock,
                       static_cast<int32_t>(products), skipLonger, a.alpha, a.beta);
    return CheckLaunch();
}

template <typename ValT, typename OutT, typename AccT, int G>
int LaunchStreamTiles(const SpmvArgs &a, int32_t rowsPerBlock, int32_t tileRowNnz, bool guardTiles, int32_t skipLonger)
{
    // LDS for the worst case of this block shape; the issue depth U covers it in one round.
    const size_t products = static_cast<size_t>(rowsPerBlock) * static_cast<size_t>(tileRowNnz);
    const size_t lds = products * sizeof(AccT);
    if constexpr (G == 1 && std::is_same<OutT, float>::value) {
        // Four rows per lane with vector row offsets / y where the shapes allow it.
        const bool quadOff = std::getenv("OPS_SPARSE_STREAM_NO_QUAD_ROWS") != nullptr;
        if (!quadOff && rowsPerBlock % 4 == 0 && rowsPerBlock <= 4 * kBlockThreads &&
            reinterpret_cast<uintptr_t>(a.rowOffsets) % 16 == 0 && reinterpret_cast<uintptr_t>(a.y) % 16 == 0 &&
            reinterpret_cast<uintptr_t>(a.yIn) % 16 == 0) {
            const uint32_t grid = GridFor(a.rows, rowsPerBlock);
            auto launch = [&](auto tag) {
                constexpr int U = decltype(tag)::value;
                auto kernel = guardTiles ? SpmvStreamQuadRowsKernel<ValT, AccT, U, true>
                                         : SpmvStreamQuadRowsKernel<ValT, AccT, U, false>;
                hipLaunchKernelGGL(kernel, dim3(grid), dim3(kBlockThreads), lds, a.stream, a.rowOffsets, a.colInd,
                                   static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                                   static_cast<float *>(a.y), static_cast<const float *>(a.yIn), a.rows, rowsPerBlock,
                                   static_cast<int32_t>(products) | (skipLonger << 16), a.alpha, a.beta);
            };
            if (products <= kBlockThreads * 4) {
                launch(std::integral_constant<int, 1>{});
            } else if (products <= kBlockThreads * 8) {
                launch(std::integral_constant<int, 2>{});
            } else {
                launch(std::integral_constant<int, 3>{});
            }
            return CheckLaunch();
        }
    }
    if (products <= kBlockThreads * 4) return LaunchStreamU<ValT, OutT, AccT, G, 1>(a, rowsPerBlock, products, skipLonger);
    if (products <= kBlockThreads * 8) return LaunchStreamU<ValT, OutT, AccT, G, 2>(a, rowsPerBlock, products, skipLonger);
    return LaunchStreamU<ValT, OutT, AccT, G, 3>(a, rowsPerBlock, products, skipLonger);
}

// The stream-rows family for a plan: the tiles, and the long rows beside them where the plan says so.
template <typename ValT, typename OutT, typename AccT, int G>
int LaunchStream(const SpmvArgs &a, const OpsparseSpmvPlan &plan)
{
    const bool beside = plan.longRowsBeside != 0;
    const int32_t tileRowNnz = plan.tileRowNnz > 0 ? plan.tileRowNnz : plan.maxRowNnz;
    // with long rows beside, the tiles must be guarded: a tile that holds one does not fit its LDS
    int rc = LaunchStreamTiles<ValT, OutT, AccT, G>(a, plan.rowsPerBlock, tileRowNnz, plan.guardTiles != 0 || beside,
                                                    beside ? kBesideRow : 0);
    if (rc == OPSPARSE_OK && beside) {
        hipLaunchKernelGGL((SpmvLongRowsKernel<ValT, OutT, AccT>),
                           dim3(GridFor(a.rows, static_cast<int64_t>(kBlockThreads) * kLongScanRows)),
                           dim3(kBlockThreads), 0, a.stream, a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                           static_cast<const ValT *>(a.x), static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn),
                           a.rows, kBesideRow, a.alpha, a.beta);
        rc = CheckLaunch();
    }
    return rc;
}

template <typename ValT, typename OutT, typename AccT, int G>
int LaunchVector(const SpmvArgs &a)
{
    const uint32_t grid = GridFor(a.rows, kBlockThreads / G);
    hipLaunchKernelGGL((SpmvVectorRowsKernel<ValT, OutT, AccT, G>), dim3(grid), dim3(kBlockThreads), 0, a.stream,
                       a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                       static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.rows, a.alpha, a.beta);
    return CheckLaunch();
}

template <typename ValT, typename OutT, typename AccT>
int LaunchMerge(const SpmvArgs &a, const OpsparseSpmvPlan &plan)
{
    auto *base = static_cast<unsigned char *>(a.ws);
    auto *part = reinterpret_cast<int32_t *>(base + plan.partOff);
    auto *carry = reinterpret_cast<AccT *>(base + plan.carryOff);
    auto *head = reinterpret_cast<AccT *>(base + plan.headOff);
    const int32_t nb = plan.mergeBlocks;
    if (!plan.partitionReady) {
        hipLaunchKernelGGL(MergePartitionKernel, dim3(GridFor(nb + 1, kBlockThreads)), dim3(kBlockThreads), 0,
                           a.stream, a.rowOffsets, a.rows, a.nnz, nb, part);
    }
    hipLaunchKernelGGL((SpmvMergeKernel<ValT, OutT, AccT>), dim3(nb), dim3(kBlockThreads), 0, a.stream, a.rowOffsets,
                       a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                       static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.rows, a.nnz, part, carry, head, a.alpha, a.beta);
    hipLaunchKernelGGL((SpmvMergeFixupKernel<OutT, AccT>), dim3(GridFor(nb, kBlockThreads)), dim3(kBlockThreads), 0,
                       a.stream, a.rowOffsets, static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.rows, a.nnz, nb, part, carry, head,
                       a.alpha, a.beta);
    return CheckLaunch();
}

template <typename OutT, typename AccT>
int LaunchScale(OutT *y, const OutT *yIn, int64_t len, OpsparseScalar beta, hipStream_t stream)
{
    if (len <= 0) {
        return OPSPARSE_OK;
    }
    int64_t grid = (len + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 65536 ? 65536 : grid;
    hipLaunchKernelGGL((SpmvScaleKernel<OutT, AccT>), dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0,
                       stream, y, yIn, len, beta);
    return CheckLaunch();
}

template <typename OutT>
int LaunchPanels(const SpmvArgs &a, const OpsparseSpmvPlan &plan);

template <typename ValT, typename OutT, typename AccT>
int RunPlanned(const SpmvArgs &a, const OpsparseSpmvPlan &plan)
{
    switch (plan.kernel) {
        case OPSPARSE_SPMV_SCALE_ONLY:
            return LaunchScale<OutT, AccT>(static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.rows, a.beta,
                                           a.stream);
        case OPSPARSE_SPMV_STREAM_ROWS:
            switch (plan.lanesPerRow) {
                case 1: return LaunchStream<ValT, OutT, AccT, 1>(a, plan);
                case 2: return LaunchStream<ValT, OutT, AccT, 2>(a, plan);
                case 4: return LaunchStream<ValT, OutT, AccT, 4>(a, plan);
                case 8: return LaunchStream<ValT, OutT, AccT, 8>(a, plan);
                case 16: return LaunchStream<ValT, OutT, AccT, 16>(a, plan);
                case 32: return LaunchStream<ValT, OutT, AccT, 32>(a, plan);
                case 64: return LaunchStream<ValT, OutT, AccT, 64>(a, plan);
                default: return OPSPARSE_E_INVALID;
            }
        case OPSPARSE_SPMV_VECTOR_ROWS:
            switch (plan.lanesPerRow) {
                case 4: return LaunchVector<ValT, OutT, AccT, 4>(a);
                case 8: return LaunchVector<ValT, OutT, AccT, 8>(a);
                case 16: return LaunchVector<ValT, OutT, AccT, 16>(a);
                case 32: return LaunchVector<ValT, OutT, AccT, 32>(a);
                case 64: return LaunchVector<ValT, OutT, AccT, 64>(a);
                default: return OPSPARSE_E_INVALID;
            }
        case OPSPARSE_SPMV_MERGE_PATH:
            if (a.ws == nullptr || static_cast<int64_t>(a.wsBytes) < plan.bytes) {
                return OPSPARSE_E_WORKSPACE;
            }
            return LaunchMerge<ValT, OutT, AccT>(a, plan);
        case OPSPARSE_SPMV_COLUMN_PANELS:
            if constexpr (std::is_same<ValT, float>::value && std::is_same<AccT, double>::value) {
                return LaunchPanels<OutT>(a, plan);
            } else {
                return OPSPARSE_E_UNSUPPORTED;  // the panel copy holds fp32 values
            }
        case OPSPARSE_SPMV_BLOCKED_GATHER:
        case OPSPARSE_SPMV_BLOCKED_LIVE:
        case OPSPARSE_SPMV_SCATTER_LIVE:
            return OPSPARSE_E_INVALID;  // (launched before the types are dispatched: opsparse_spmv_csr_launch_zy)
        default:
            return OPSPARSE_E_INVALID;
    }
}

// ---- COLUMN_PANELS: workspace layout, preprocessing, launch

constexpr int32_t kPanelShift = 20;  // 2^20 columns = 4 MiB of fp32 x per panel: one XCD's L2

int32_t PanelCount(int64_t cols)
{
    return static_cast<int32_t>((cols + (int64_t{1} << kPanelShift) - 1) >> kPanelShift);
}

struct PanelLayout {
    int64_t tileBound;  // upper bound of the merge tiles of one panel
    int64_t rowPtrOff, colIndOff, valsOff, partOff, carryOff, headOff, ypartOff;   // used by every launch
    int64_t posOff, rowOfPosOff, rowSortedOff, tableOff, scratchOff;               // preprocessing only
    int64_t bytes;
};

PanelLayout MakePanelLayout(int64_t rows, int64_t nnz, int32_t numPanels)
{
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    PanelLayout l{};
    const int64_t P = numPanels;
    l.tileBound = (rows + nnz + kMergeItems - 1) / kMergeItems + 1;
    int64_t off = 256;
    l.rowPtrOff = off; off += align(4 * P * (rows + 1));
    l.colIndOff = off; off += align(4 * nnz);
    l.valsOff = off; off += align(4 * nnz);
    l.partOff = off; off += align(4 * P * (l.tileBound + 1));
    l.carryOff = off; off += align(8 * P * l.tileBound);
    l.headOff = off; off += align(8 * P * l.tileBound);
    l.ypartOff = off; off += align(8 * P * rows);
    l.posOff = off; off += align(4 * nnz);
    l.rowOfPosOff = off; off += align(4 * nnz);
    l.rowSortedOff = off; off += align(4 * nnz);
    l.tableOff = off; off += align(4 * RadixTableInts(nnz));
    const int64_t scanA = ScanScratchInts(RadixTableInts(nnz)), scanB = ScanScratchInts(rows + 1);
    l.scratchOff = off; off += align(4 * (scanA > scanB ? scanA : scanB));
    l.bytes = off;
    return l;
}

template <typename OutT>
int LaunchPanels(const SpmvArgs &a, const OpsparseSpmvPlan &plan)
{
    using AccT = double;
    const int32_t P = plan.numPanels;
    const PanelLayout l = MakePanelLayout(a.rows, a.nnz, P);
    if (a.ws == nullptr || static_cast<int64_t>(a.wsBytes) < l.bytes || plan.bytes != l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto *base = static_cast<unsigned char *>(a.ws);
    const auto *rowPtrP = reinterpret_cast<const int32_t *>(base + l.rowPtrOff);
    const auto *colIndP = reinterpret_cast<const int32_t *>(base + l.colIndOff);
    const auto *valsP = reinterpret_cast<const float *>(base + l.valsOff);
    const auto *part = reinterpret_cast<const int32_t *>(base + l.partOff);
    auto *carry = reinterpret_cast<AccT *>(base + l.carryOff);
    auto *head = reinterpret_cast<AccT *>(base + l.headOff);
    auto *ypart = reinterpret_cast<AccT *>(base + l.ypartOff);
    PanelTable pt{};
    int64_t maxTiles = 0;
    for (int32_t p = 0; p <= P; ++p) {
        pt.start[p] = plan.panelStart[p];
    }
    // Panels in groups of 8, one per XCD.
    for (int32_t panelBase = 0; panelBase < P; panelBase += kNumXcd) {
        int64_t tiles = 0;
        for (int32_t p = panelBase; p < P && p < panelBase + kNumXcd; ++p) {
            const int64_t t = (a.rows + (pt.start[p + 1] - pt.start[p]) + kMergeItems - 1) / kMergeItems;
            tiles = t > tiles ? t : tiles;
        }
        maxTiles = tiles > maxTiles ? tiles : maxTiles;
        hipLaunchKernelGGL((SpmvPanelMergeKernel<float, AccT>), dim3(static_cast<uint32_t>(tiles * kNumXcd)),
                           dim3(kBlockThreads), 0, a.stream, rowPtrP, colIndP, valsP, static_cast<const float *>(a.x),
                           ypart, a.rows, pt, panelBase, P, part, carry, head, l.tileBound);
    }
    hipLaunchKernelGGL((SpmvPanelFixupKernel<AccT>), dim3(GridFor(maxTiles, kBlockThreads), static_cast<uint32_t>(P)),
                       dim3(kBlockThreads), 0, a.stream, rowPtrP, ypart, a.rows, pt, part, carry, head, l.tileBound);
    int64_t grid = (a.rows + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 16384 ? 16384 : grid;
    hipLaunchKernelGGL((SpmvPanelCombineKernel<OutT, AccT>), dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0,
                       a.stream, ypart, P, a.rows, static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.alpha,
                       a.beta);
    return CheckLaunch();
}

int32_t VectorLanesFor(int64_t rows, int64_t nnz)
{
    const int64_t mean = rows > 0 ? nnz / rows : 0;
    int32_t g = 4;
    while (g < kWave && mean > 4 * g) {
        g <<= 1;
    }
    return g;
}

// No plan: merge-path with the partition rebuilt into the workspace, or the
// workspace-free vector kernel when the workspace is too small.
OpsparseSpmvPlan AdHocPlan(int64_t rows, int64_t nnz, size_t wsBytes, const void *ws)
{
    OpsparseSpmvPlan p{};
    p.rows = rows;
    p.nnz = nnz;
    if (nnz == 0) {
        p.kernel = OPSPARSE_SPMV_SCALE_ONLY;
        return p;
    }
    const MergeLayout l = MakeMergeLayout(rows, nnz);
    if (ws != nullptr && static_cast<int64_t>(wsBytes) >= l.bytes) {
        p.kernel = OPSPARSE_SPMV_MERGE_PATH;
        p.mergeBlocks = l.blocks;
        p.partOff = l.partOff;
        p.carryOff = l.carryOff;
        p.headOff = l.headOff;
        p.bytes = l.bytes;
        p.partitionReady = 0;
    } else {
        p.kernel = OPSPARSE_SPMV_VECTOR_ROWS;
        p.lanesPerRow = VectorLanesFor(rows, nnz);
    }
    return p;
}

template <typename ValT, typename AccT>
int RunTranspose(const SpmvArgs &a, int32_t outType, bool skewedRows)
{
    if (outType != OPSPARSE_F32 && outType != OPSPARSE_F16 && outType != OPSPARSE_BF16) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    // y has `cols` elements for the transposed product.  fp16 / bf16 y: the sums are formed in an fp32
    // staging vector in the workspace and rounded once at the end.
    const bool staged = outType != OPSPARSE_F32;
    float *acc = static_cast<float *>(a.y);
    int64_t grid = (a.cols + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 65536 ? 65536 : (grid < 1 ? 1 : grid);
    int rc = OPSPARSE_OK;
    if (!staged) {
        rc = LaunchScale<float, AccT>(acc, static_cast<const float *>(a.yIn), a.cols, a.beta, a.stream);
    } else if (a.cols > 0) {
        if (a.ws == nullptr || a.wsBytes < static_cast<size_t>(a.cols) * sizeof(float)) {
            return OPSPARSE_E_WORKSPACE;
        }
        acc = static_cast<float *>(a.ws);
        if (outType == OPSPARSE_F16) {
            hipLaunchKernelGGL(ScaleIntoFloatKernel<Half>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0,
                               a.stream, acc, static_cast<const Half *>(a.yIn), a.cols, a.beta);
        } else {
            hipLaunchKernelGGL(ScaleIntoFloatKernel<Bf16>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0,
                               a.stream, acc, static_cast<const Bf16 *>(a.yIn), a.cols, a.beta);
        }
        rc = CheckLaunch();
    }
    auto finish = [&]() {
        if (staged && a.cols > 0) {
            if (outType == OPSPARSE_F16) {
                hipLaunchKernelGGL(ConvertFromFloatKernel<Half>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads),
                                   0, a.stream, static_cast<Half *>(a.y), acc, a.cols);
            } else {
                hipLaunchKernelGGL(ConvertFromFloatKernel<Bf16>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads),
                                   0, a.stream, static_cast<Bf16 *>(a.y), acc, a.cols);
            }
        }
        return CheckLaunch();
    };
    if (rc != OPSPARSE_OK) {
        return rc;
    }
    if (a.nnz == 0 || a.rows == 0) {
        return finish();
    }
    if (a.cols <= kNarrowCols && a.nnz >= 16 * kTransposeTile && a.nnz >= 8 * a.cols) {
        // few columns: y per workgroup in LDS, one global update per workgroup and element
        const int64_t numTiles = (a.nnz + kTransposeTile - 1) / kTransposeTile;
        const int64_t tilesPerBlock = (numTiles + kNarrowMaxBlocks - 1) / kNarrowMaxBlocks;
        auto narrow = a.cols <= kNarrowCols / 2 ? SpmvTransposeNarrowKernel<ValT, AccT, kNarrowCols / 2>
                                                : SpmvTransposeNarrowKernel<ValT, AccT, kNarrowCols>;
        hipLaunchKernelGGL(narrow, dim3(GridFor(numTiles, tilesPerBlock)), dim3(kBlockThreads), 0, a.stream,
                           a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                           acc, a.rows, a.cols, a.nnz, tilesPerBlock, a.alpha);
        return finish();
    }
    if (a.rows < kTransposeFewRows && a.nnz >= 8 * kTransposeTile) {
        // too few rows to occupy the GPU with a lane group each (ten rows of 2 M entries: 17 ms that way, 0.3 ms
        // here): equal entries per workgroup, the row of an entry looked up in the few offsets there are
        hipLaunchKernelGGL((SpmvTransposeFlatKernel<ValT, AccT>), dim3(GridFor(a.nnz, kTransposeTile)),
                           dim3(kBlockThreads), 0, a.stream, a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                           static_cast<const ValT *>(a.x), acc, a.rows, a.nnz, a.alpha);
        return finish();
    }
    // Rows far longer than the mean: the lane groups take the rows up to kTransposeLongRow entries, whole
    // workgroups the others.
    const int32_t maxLen = skewedRows ? kTransposeLongRow : INT32_MAX;
    const int32_t g = VectorLanesFor(a.rows, a.nnz);
    auto launch = [&](auto tag) {
        constexpr int G = decltype(tag)::value;
        hipLaunchKernelGGL((SpmvTransposeScatterKernel<ValT, AccT, G>), dim3(GridFor(a.rows, kBlockThreads / G)),
                           dim3(kBlockThreads), 0, a.stream, a.rowOffsets, a.colInd,
                           static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x),
                           acc, a.rows, maxLen, a.alpha);
        if (skewedRows) {
            hipLaunchKernelGGL((SpmvTransposeLongRowsKernel<ValT, AccT>), dim3(GridFor(a.rows, kBlockThreads)),
                               dim3(kBlockThreads), 0, a.stream, a.rowOffsets, a.colInd,
                               static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x), acc, a.rows, maxLen,
                               a.alpha);
        }
    };
    switch (g) {
        case 4: launch(std::integral_constant<int, 4>{}); break;
        case 8: launch(std::integral_constant<int, 8>{}); break;
        case 16: launch(std::integral_constant<int, 16>{}); break;
        case 32: launch(std::integral_constant<int, 32>{}); break;
        default: launch(std::integral_constant<int, 64>{}); break;
    }
    return finish();
}

// op(A) = A^T in int32 arithmetic (the reference's SpmvKernelTrans<int32_t, int32_t, int32_t>,
// sparse/spmv/arch22/kernels/spmv_kernel.cpp:21-55): y = beta * y, then an integer atomic add per entry, a lane
// group per row.  Products and sums wrap around like the reference's int32 arithmetic, so the result does not
// depend on the order of the additions.
int RunTransposeInt(const SpmvArgs &a)
{
    int32_t *y = static_cast<int32_t *>(a.y);
    const int rc = LaunchScale<int32_t, int32_t>(y, static_cast<const int32_t *>(a.yIn), a.cols, a.beta, a.stream);
    if (rc != OPSPARSE_OK || a.nnz == 0 || a.rows == 0) {
        return rc;
    }
    auto launch = [&](auto tag) {
        constexpr int G = decltype(tag)::value;
        hipLaunchKernelGGL((SpmvTransposeScatterKernel<int32_t, int32_t, G, int32_t>),
                           dim3(GridFor(a.rows, kBlockThreads / G)), dim3(kBlockThreads), 0, a.stream, a.rowOffsets,
                           a.colInd, static_cast<const int32_t *>(a.vals), static_cast<const int32_t *>(a.x), y, a.rows,
                           INT32_MAX, a.alpha);
    };
    switch (VectorLanesFor(a.rows, a.nnz)) {
        case 4: launch(std::integral_constant<int, 4>{}); break;
        case 8: launch(std::integral_constant<int, 8>{}); break;
        case 16: launch(std::integral_constant<int, 16>{}); break;
        case 32: launch(std::integral_constant<int, 32>{}); break;
        default: launch(std::integral_constant<int, 64>{}); break;
    }
    return CheckLaunch();
}

template <typename ValT, typename OutT, typename AccT>
int RunTyped(const OpsparseSpmvPlan *plan, const SpmvArgs &a)
{
    if (plan != nullptr) {
        return RunPlanned<ValT, OutT, AccT>(a, *plan);
    }
    const OpsparseSpmvPlan adhoc = AdHocPlan(a.rows, a.nnz, a.wsBytes, a.ws);
    return RunPlanned<ValT, OutT, AccT>(a, adhoc);
}

}  // namespace
}  // namespace opsparse

// ================================================================== C ABI

using namespace opsparse;

// Scratch of opsparse_spmv_csr_launch_noalloc: the merge-path partition, carries and heads of one launch.  Every
// GPU the library runs on holds its own 4 MiB copy until the process ends.  In host code the array's name is only
// a stand-in for the symbol; the device address comes from hipGetSymbolAddress, once per device (StaticScratch).
#define OPSPARSE_NOALLOC_SCRATCH_BYTES (4u << 20)
static __device__ __align__(256) unsigned char scratch[OPSPARSE_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device, resolved on the first call there; nullptr on failure.
void *StaticScratch()
{
    static std::mutex lock;
    static void *ptrOf[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(lock);
    if (ptrOf[dev] == nullptr) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        ptrOf[dev] = ptr;
    }
    return ptrOf[dev];
}

}  // namespace

extern "C" {

size_t opsparse_spmv_csr_workspace_bytes(int64_t rows, int64_t nnz)
{
    if (rows < 0 || nnz < 0) {
        return 0;
    }
    return static_cast<size_t>(MakeMergeLayout(rows, nnz).bytes);
}

int opsparse_spmv_csr_analyse(const int32_t *rowOffsets, int64_t rows, int64_t cols, int64_t nnz, void *workspace,
                              size_t workspaceBytes, int32_t forceKernel, OpsparseSpmvPlan *plan, void *stream)
{
    (void)cols;
    if (plan == nullptr || rows < 0 || nnz < 0 || (rows > 0 && rowOffsets == nullptr)) {
        return OPSPARSE_E_INVALID;
    }
    auto s = static_cast<hipStream_t>(stream);
    OpsparseSpmvPlan p{};
    p.rows = rows;
    p.nnz = nnz;
    if (rows == 0 || nnz == 0) {
        p.kernel = OPSPARSE_SPMV_SCALE_ONLY;
        *plan = p;
        return OPSPARSE_OK;
    }
    const MergeLayout l = MakeMergeLayout(rows, nnz);
    if (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    // Longest row, reduced on the device into the workspace header.
    auto *stats = static_cast<int32_t *>(workspace);
    if (hipMemsetAsync(stats, 0, 256, s) != hipSuccess) {
        return OPSPARSE_E_LAUNCH;
    }
    int64_t grid = (rows + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 2048 ? 2048 : grid;
    hipLaunchKernelGGL(RowStatsKernel, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0, s, rowOffsets, rows,
                       stats);
    int32_t seen[4] = {0, 0, 0, 0};  // longest row, longest of the short rows, rows longer than those, their entries
    if (hipMemcpyAsync(seen, stats, sizeof(seen), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        return OPSPARSE_E_LAUNCH;
    }
    const int32_t maxRow = seen[0], maxShort = seen[1], numLong = seen[2];
    const int64_t nnzShort = nnz - static_cast<int64_t>(static_cast<uint32_t>(seen[3]));
    p.maxRowNnz = maxRow;

    int32_t kernel = forceKernel;
    if (kernel == OPSPARSE_SPMV_AUTO) {
        // Measured on 64 M entries, even rows and rows of 0.5 - 1.5 times the mean, banded and random columns:
        // stream rows sizes its tiles for the longest row and wins while they are mostly full or the rows very
        // short (mean 16 - 48 even: 160 - 173 us against 195 - 200 us for the merge path; varied: 217 - 222 us
        // against 194 - 199 us); a lane group per row only pays for long rows of nearly equal length (mean 128 -
        // 256: 180 us against 195 us; varied rows 250 - 350 us against 189 us); the merge path does not care.
        // Since the stream-rows tiles take rows of up to 512 entries (8 - 64 lanes a row), even rows of 49 - 512
        // entries are theirs as well: 40 M entries in a band, 60 - 512 a row, 65 - 75 us against 64 - 116 us with a
        // lane group a row or the merge path (100 a row: 117 -> 74 us), and random columns 167 - 186 us against
        // 165 - 250 us.  That leaves nothing for the lane-group-a-row kernel to be chosen for here: it serves
        // forced plans and calls that come without a workspace.
        if (maxRow <= kStreamMaxRow && (maxRow <= 12 || static_cast<double>(maxRow) * static_cast<double>(rows) <=
                                                            1.25 * static_cast<double>(nnz))) {
            kernel = OPSPARSE_SPMV_STREAM_ROWS;
        } else if (maxRow > kShortMaxRow && maxRow <= kBesideMaxRow && maxShort >= 1 && numLong <= 4096 &&
                   static_cast<int64_t>(numLong) * 1024 <= rows &&
                   (maxShort <= 12 || static_cast<double>(maxShort) * static_cast<double>(rows) <=
                                          1.25 * static_cast<double>(nnzShort))) {
            // Short rows with a few long ones among them (at most one row in a thousand, 4096 in all: a mesh with
            // dense constraint rows, a graph with a few hubs): the stream-rows tiles sized for the short rows, the
            // long rows summed beside them by a workgroup each (2048 x 2048 mesh with 11 rows of 3000 entries:
            // 47 us, against 91 us for the merge path the longest row would otherwise call for).
            kernel = OPSPARSE_SPMV_STREAM_ROWS;
            p.longRowsBeside = 1;
            p.tileRowNnz = maxShort;
        } else {
            kernel = OPSPARSE_SPMV_MERGE_PATH;
        }
    }
    p.kernel = kernel;
    switch (kernel) {
        case OPSPARSE_SPMV_STREAM_ROWS: {
            // the row length the tiles are sized for: the longest row, or the longest short one with the rest beside
            const int32_t tileRow = p.longRowsBeside ? p.tileRowNnz : maxRow;
            if (tileRow > kStreamMaxRow) {
                return OPSPARSE_E_UNSUPPORTED;  // products of a row block would not fit LDS
            }
            p.tileRowNnz = tileRow;
            const int32_t g = tileRow <= 12 ? 1 : (tileRow <= 24 ? 2 : (tileRow <= 48 ? 4 : (tileRow <= 96 ? 8 : (tileRow <= 192 ? 16 : (tileRow <= 384 ? 32 : 64)))));
            p.lanesPerRow = g;
            // As many rows as keep the tile's worst-case products within two full
            // rounds of the workgroup's loads (2 x 1024 entries, 16 KiB of LDS):
            // measured best when a tile nearly fills whole rounds.
            int32_t rpb = 2048 / tileRow;
            rpb = rpb > 512 ? 512 : rpb;
            rpb &= ~3;  // whole groups of four rows for the vectorised y path
            p.rowsPerBlock = rpb < 4 ? 4 : rpb;
            if (tileRow > 48) {
                // Few rows a tile: as many as the lane groups sum in whole turns (a band of 81 entries a row: 32
                // rows 68.7 us, 25 rows 73.2 us, 37 rows 75.5 us) within the 3072 slots.  (g lanes serve rows of up
                // to 12 g entries, so at least one turn of the 256 / g groups always fits.)
                const int32_t groups = kBlockThreads / g;
                p.rowsPerBlock = 3072 / tileRow / groups * groups;
            }
            if (const char *env = std::getenv("OPS_SPARSE_STREAM_ROWS")) {
                const int v = std::atoi(env);  // tuning override
                if (v >= 1 && v <= kStreamRowsMax && static_cast<int64_t>(v) * tileRow <= 3072) {
                    p.rowsPerBlock = v;
                }
            }
            break;
        }
        case OPSPARSE_SPMV_VECTOR_ROWS:
            p.lanesPerRow = VectorLanesFor(rows, nnz);
            break;
        case OPSPARSE_SPMV_MERGE_PATH: {
            p.mergeBlocks = l.blocks;
            p.partOff = l.partOff;
            p.carryOff = l.carryOff;
            p.headOff = l.headOff;
            p.bytes = l.bytes;
            auto *part = reinterpret_cast<int32_t *>(static_cast<unsigned char *>(workspace) + l.partOff);
            hipLaunchKernelGGL(MergePartitionKernel, dim3(GridFor(l.blocks + 1, kBlockThreads)), dim3(kBlockThreads),
                               0, s, rowOffsets, rows, nnz, l.blocks, part);
            if (CheckLaunch() != OPSPARSE_OK) {
                return OPSPARSE_E_LAUNCH;
            }
            p.partitionReady = 1;
            break;
        }
        default:
            return OPSPARSE_E_INVALID;
    }
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmv_csr_gathers_scattered(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols,
                                        int64_t nnz, void *workspace, size_t workspaceBytes, int32_t *scattered,
                                        void *stream)
{
    if (scattered == nullptr || rows < 0 || cols < 0 || nnz < 0 ||
        (rows > 0 && nnz > 0 && (rowOffsets == nullptr || colInd == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    *scattered = 0;
    if (rows == 0 || nnz == 0 || cols == 0) {
        return OPSPARSE_OK;
    }
    if (workspace == nullptr || workspaceBytes < 256) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto *counts = static_cast<int32_t *>(workspace) + 8;  // header words 8 and 9
    LaunchFillI32(counts, 2, 0, s);
    constexpr int64_t kSamples = 65536;
    constexpr int64_t kBand = 131072;  // 2 * band * 4 bytes = 1 MiB of x around the diagonal: a quarter of an L2
    const int64_t rowStride = (rows + kSamples - 1) / kSamples;
    const int64_t samples = (rows + rowStride - 1) / rowStride;
    hipLaunchKernelGGL(GatherLocalityKernel, dim3(static_cast<uint32_t>((samples + kBlockThreads - 1) / kBlockThreads)),
                       dim3(kBlockThreads), 0, s, rowOffsets, colInd, rows, cols, rowStride, kBand, counts);
    int32_t host[2] = {0, 0};
    if (hipMemcpyAsync(host, counts, sizeof(host), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    // how many sampled gathers in a thousand land outside the band
    *scattered = host[0] > 0 ? static_cast<int32_t>(static_cast<int64_t>(host[1]) * 1000 / host[0]) : 0;
    return OPSPARSE_OK;
}

size_t opsparse_spmv_csr_panels_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz)
{
    const int32_t P = PanelCount(cols);
    if (rows <= 0 || nnz <= 0 || nnz > INT32_MAX || rows >= INT32_MAX || P < 2 || P > OPSPARSE_SPMV_MAX_PANELS) {
        return 0;
    }
    return static_cast<size_t>(MakePanelLayout(rows, nnz, P).bytes);
}

int opsparse_spmv_csr_panels_analyse(const int32_t *rowOffsets, const int32_t *colInd, const float *csrValues,
                                     int64_t rows, int64_t cols, int64_t nnz, void *workspace, size_t workspaceBytes,
                                     OpsparseSpmvPlan *plan, void *stream)
{
    if (plan == nullptr || rowOffsets == nullptr || colInd == nullptr || csrValues == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    const size_t need = opsparse_spmv_csr_panels_workspace_bytes(rows, cols, nnz);
    if (need == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    if (workspace == nullptr || workspaceBytes < need) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    const int32_t P = PanelCount(cols);
    const PanelLayout l = MakePanelLayout(rows, nnz, P);
    auto *base = static_cast<unsigned char *>(workspace);
    auto at = [&](int64_t off) { return reinterpret_cast<int32_t *>(base + off); };
    int32_t *rowPtrP = at(l.rowPtrOff), *colIndP = at(l.colIndOff), *pos = at(l.posOff);
    int32_t *rowOfPos = at(l.rowOfPosOff), *rowSorted = at(l.rowSortedOff), *table = at(l.tableOff);
    int32_t *scratch = at(l.scratchOff), *part = at(l.partOff);
    auto *valsP = reinterpret_cast<uint32_t *>(base + l.valsOff);

    // Entries in (panel, original position) order: one stable radix pass on the panel number.
    LaunchExpandRows(rowOffsets, rows, nnz, 0, rowOfPos, s);
    LaunchRadixPass(colInd, nullptr, colIndP, pos, nnz, 0, kPanelShift, table, scratch, s);
    LaunchGatherByPosition(pos, rowOfPos, reinterpret_cast<const uint32_t *>(csrValues), nnz, rowSorted, valsP, s);
    // First entry of every panel = first output position of its digit.
    const int64_t radixTiles = RadixTiles(nnz);
    OpsparseSpmvPlan p{};
    int32_t starts[OPSPARSE_SPMV_MAX_PANELS];
    for (int32_t d = 0; d < P; ++d) {
        if (hipMemcpyAsync(&starts[d], table + static_cast<int64_t>(d) * radixTiles, sizeof(int32_t),
                           hipMemcpyDeviceToHost, s) != hipSuccess) {
            (void)hipGetLastError();
            return OPSPARSE_E_LAUNCH;
        }
    }
    if (hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    for (int32_t d = 0; d < P; ++d) {
        p.panelStart[d] = starts[d];
    }
    p.panelStart[P] = nnz;
    // Row offsets (relative to the panel's first entry) and merge partition of every panel.
    for (int32_t d = 0; d < P; ++d) {
        const int64_t nnzP = p.panelStart[d + 1] - p.panelStart[d];
        if (nnzP < 0) {
            return OPSPARSE_E_INVALID;  // a column index outside [0, cols)
        }
        int32_t *rp = rowPtrP + static_cast<int64_t>(d) * (rows + 1);
        LaunchIndicesToOffsets(rowSorted + p.panelStart[d], nnzP, rows, 0, rp, scratch, s);
        const int32_t tiles = static_cast<int32_t>((rows + nnzP + kMergeItems - 1) / kMergeItems);
        hipLaunchKernelGGL(MergePartitionKernel, dim3(GridFor(tiles + 1, kBlockThreads)), dim3(kBlockThreads), 0, s, rp,
                           rows, nnzP, tiles, part + static_cast<int64_t>(d) * (l.tileBound + 1));
    }
    if (CheckLaunch() != OPSPARSE_OK) {
        return OPSPARSE_E_LAUNCH;
    }
    p.kernel = OPSPARSE_SPMV_COLUMN_PANELS;
    p.numPanels = P;
    p.panelShift = kPanelShift;
    p.rows = rows;
    p.nnz = nnz;
    p.bytes = l.bytes;
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmv_csr_launch(const OpsparseSpmvPlan *plan, int32_t transpose, const int32_t *rowOffsets,
                             const int32_t *colInd, const void *csrValues, const void *x, void *y, int64_t rows,
                             int64_t cols, int64_t nnz, OpsparseScalar alpha, OpsparseScalar beta, int32_t valType,
                             int32_t outType, int32_t computeIsInt, void *workspace, size_t workspaceBytes,
                             void *stream)
{
    return opsparse_spmv_csr_launch_zy(plan, transpose, rowOffsets, colInd, csrValues, x, y, y, rows, cols, nnz, alpha,
                                       beta, valType, outType, computeIsInt, workspace, workspaceBytes, stream);
}

int opsparse_spmv_csr_launch_zy(const OpsparseSpmvPlan *plan, int32_t transpose, const int32_t *rowOffsets,
                                const int32_t *colInd, const void *csrValues, const void *x, const void *yIn, void *y,
                                int64_t rows, int64_t cols, int64_t nnz, OpsparseScalar alpha, OpsparseScalar beta,
                                int32_t valType, int32_t outType, int32_t computeIsInt, void *workspace,
                                size_t workspaceBytes, void *stream)
{
    if (rows < 0 || cols < 0 || nnz < 0) {
        return OPSPARSE_E_INVALID;
    }
    const int64_t outLen = transpose ? cols : rows;
    if (outLen == 0) {
        return OPSPARSE_OK;  // nothing to write
    }
    if (y == nullptr ||
        (nnz > 0 && (rowOffsets == nullptr || colInd == nullptr || csrValues == nullptr || x == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    if (plan != nullptr && (plan->rows != rows || plan->nnz != nnz)) {
        return OPSPARSE_E_INVALID;
    }
    if (yIn == nullptr) {
        yIn = y;  // only read when beta != 0
    }
    SpmvArgs a{rowOffsets, colInd, csrValues, x,         y,     yIn, rows, cols, nnz, alpha, beta,
               workspace,  workspaceBytes, static_cast<hipStream_t>(stream)};

    if (plan != nullptr && plan->kernel == OPSPARSE_SPMV_BLOCKED_GATHER && (plan->transposed != 0) != (transpose != 0)) {
        return OPSPARSE_E_INVALID;  // the re-stored layout serves the op(A) it was built for
    }
    if (plan != nullptr && plan->kernel == OPSPARSE_SPMV_SCATTER_LIVE && nnz > 0) {
        if (!transpose || computeIsInt) {
            return OPSPARSE_E_INVALID;  // (built for op(A) = A^T and floating-point sums)
        }
        return scatter_layout::Launch(a, *plan, valType, outType);
    }
    if (plan != nullptr && plan->kernel == OPSPARSE_SPMV_BLOCKED_LIVE && nnz > 0) {
        if (transpose || computeIsInt) {
            return OPSPARSE_E_INVALID;  // (built for op(A) = A and floating-point sums)
        }
        return live_layout::LaunchBlocked(a, *plan, valType, outType);
    }
    if (plan != nullptr && plan->kernel == OPSPARSE_SPMV_BLOCKED_GATHER && nnz > 0) {
        SpmvArgs t = a;
        if (transpose) {  // the columns of A are the outputs, its rows the inputs
            t.rows = cols;
            t.cols = rows;
        }
        return LaunchBlocked(t, *plan, valType, outType, computeIsInt);
    }
    if (transpose) {
        if (computeIsInt) {
            return valType == OPSPARSE_I32 && outType == OPSPARSE_I32 ? RunTransposeInt(a) : OPSPARSE_E_UNSUPPORTED;
        }
        // The analysis found a row far longer than the mean: the transposed product then splits the work by
        // entries rather than by rows.
        const bool skewedRows = plan != nullptr && rows > 0 &&
                                static_cast<int64_t>(plan->maxRowNnz) > 16 * (nnz / rows) + 64;
        switch (valType) {
            case OPSPARSE_F32: return RunTranspose<float, double>(a, outType, skewedRows);
            case OPSPARSE_F16: return RunTranspose<Half, double>(a, outType, skewedRows);
            case OPSPARSE_BF16: return RunTranspose<Bf16, double>(a, outType, skewedRows);
            case OPSPARSE_I32: return RunTranspose<int32_t, double>(a, outType, skewedRows);  // int32 values, fp32 y
            default: return OPSPARSE_E_UNSUPPORTED;
        }
    }
    if (rows > 0 && nnz == 0) {
        plan = nullptr;  // AdHocPlan turns this into the scale kernel
    }
    if (computeIsInt) {
        if (valType == OPSPARSE_I32 && outType == OPSPARSE_I32) {
            return RunTyped<int32_t, int32_t, int32_t>(plan, a);
        }
        return OPSPARSE_E_UNSUPPORTED;
    }
    switch (valType) {
        case OPSPARSE_F32:
            if (outType == OPSPARSE_F32) return RunTyped<float, float, double>(plan, a);
            break;
        case OPSPARSE_F16:
            if (outType == OPSPARSE_F32) return RunTyped<Half, float, double>(plan, a);
            if (outType == OPSPARSE_F16) return RunTyped<Half, Half, double>(plan, a);
            break;
        case OPSPARSE_BF16:
            if (outType == OPSPARSE_F32) return RunTyped<Bf16, float, double>(plan, a);
            if (outType == OPSPARSE_BF16) return RunTyped<Bf16, Bf16, double>(plan, a);
            break;
        case OPSPARSE_I32:
            if (outType == OPSPARSE_F32) return RunTyped<int32_t, float, double>(plan, a);
            break;
        default:
            break;
    }
    return OPSPARSE_E_UNSUPPORTED;
}

size_t opsparse_spmv_csr_noalloc_max_bytes(void)
{
    return OPSPARSE_NOALLOC_SCRATCH_BYTES;
}

int opsparse_spmv_csr_launch_noalloc(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                     const void *x, void *y, int64_t rows, int64_t cols, int64_t nnz,
                                     OpsparseScalar alpha, OpsparseScalar beta, int32_t valType, int32_t outType,
                                     int32_t computeIsInt, void *stream)
{
    if (rows < 0 || cols < 0 || nnz < 0) {
        return OPSPARSE_E_INVALID;
    }
    // The merge-path tables of this matrix must fit the static array: no other kernel family is substituted, so
    // that a caller learns at once that the matrix is beyond this entry point.
    if (opsparse_spmv_csr_workspace_bytes(rows, nnz) > OPSPARSE_NOALLOC_SCRATCH_BYTES) {
        return OPSPARSE_E_WORKSPACE;
    }
    void *ws = StaticScratch();
    if (ws == nullptr) {
        return OPSPARSE_E_LAUNCH;
    }
    // Nothing in the tables has to start at zero: the partition kernel writes every partition entry, and the
    // fix-up kernel reads only carries and heads that the merge kernel of the same launch has written.
    return opsparse_spmv_csr_launch_zy(nullptr, 0, rowOffsets, colInd, csrValues, x, y, y, rows, cols, nnz, alpha, beta,
                                       valType, outType, computeIsInt, ws, OPSPARSE_NOALLOC_SCRATCH_BYTES, stream);
}

int opsparse_rebase_offsets_launch(const void *offsets, int32_t offsetsAre64, int32_t indexBase, int64_t count,
                                   int32_t *out, void *stream)
{
    if (count < 0 || (indexBase != 0 && indexBase != 1) || (count > 0 && (offsets == nullptr || out == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    if (count == 0) {
        return OPSPARSE_OK;
    }
    int64_t grid = (count + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 4096 ? 4096 : grid;
    auto s = static_cast<hipStream_t>(stream);
    if (offsetsAre64) {
        hipLaunchKernelGGL(RebaseOffsetsKernel<int64_t>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0, s,
                           static_cast<const int64_t *>(offsets), count, indexBase, out);
    } else {
        hipLaunchKernelGGL(RebaseOffsetsKernel<int32_t>, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0, s,
                           static_cast<const int32_t *>(offsets), count, indexBase, out);
    }
    return CheckLaunch();
}

int opsparse_spmv_csr_indexed_launch(const void *rowOffsets, int32_t rowOffsetsAre64, int32_t indexBase,
                                     const int32_t *colInd, const float *csrValues, const float *x,
                                     const float *yIn, float *z, int64_t rows, int64_t cols, int64_t nnz,
                                     OpsparseScalar alpha, OpsparseScalar beta, void *stream)
{
    if (rows < 0 || cols < 0 || nnz < 0 || (indexBase != 0 && indexBase != 1)) {
        return OPSPARSE_E_INVALID;
    }
    if (rows == 0) {
        return OPSPARSE_OK;
    }
    if (z == nullptr || rowOffsets == nullptr || (nnz > 0 && (colInd == nullptr || csrValues == nullptr || x == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    if (yIn == nullptr) {
        yIn = z;
    }
    auto s = static_cast<hipStream_t>(stream);
    const int32_t g = VectorLanesFor(rows, nnz);
    auto launch = [&](auto rowTag, auto gTag) {
        using RowT = typename decltype(rowTag)::type;
        constexpr int G = decltype(gTag)::value;
        hipLaunchKernelGGL((SpmvIndexedRowsKernel<RowT, float, float, double, G>),
                           dim3(GridFor(rows, kBlockThreads / G)), dim3(kBlockThreads), 0, s,
                           static_cast<const RowT *>(rowOffsets), colInd, csrValues, x, z, yIn, rows, indexBase, alpha,
                           beta);
    };
    auto byLanes = [&](auto rowTag) {
        switch (g) {
            case 4: launch(rowTag, std::integral_constant<int, 4>{}); break;
            case 8: launch(rowTag, std::integral_constant<int, 8>{}); break;
            case 16: launch(rowTag, std::integral_constant<int, 16>{}); break;
            case 32: launch(rowTag, std::integral_constant<int, 32>{}); break;
            default: launch(rowTag, std::integral_constant<int, 64>{}); break;
        }
    };
    if (rowOffsetsAre64) {
        byLanes(std::enable_if<true, int64_t>{});
    } else {
        byLanes(std::enable_if<true, int32_t>{});
    }
    return CheckLaunch();
}

}  // extern "C"
