// BLOCKED_LIVE: CSR SpMV, op(A) = A, for a matrix whose x does not fit a cache, with the values read where the
// caller has them at every call and the row sums formed with LDS atomics.
//
// Takes the place of aclsparseSpMV's kernel (sparse/spmv/arch22/kernels/spmv_kernel.h:27-310) under
// ACL_SPARSE_SPMV_ALG_DEFAULT / CSR_ALG1 for a matrix with scattered columns, after aclsparseSpMVPreprocess.  A
// row-wise kernel gathers x[col] straight from memory, and with random columns every gather moves a whole 128-byte
// line for 4 useful bytes: the gather rate, not the matrix stream, sets the time.  Here x is gathered from LDS.
// This is the fast sibling of the ordered layout of spmv_blocked.hip, whose kernels sum every row in a fixed order:
// the reference lets these two algorithm values differ in the last bit between runs
// (include/cann_ops_sparse.h:57-60), and this file uses that.
//
//   phase 1  the entries' local columns are stored a second time sorted by column panel (2^15 columns = 128 KiB
//            of x).  A workgroup copies its panel's slice of x into LDS and writes xg[i] = x[col[i]] for the panel's
//            entries: 2 bytes of local column index read, 4 bytes written per entry, both as linear streams.
//   phase 2  rows are grouped into row blocks of at most 2^12 rows and about 20 000 entries.  A workgroup owns one
//            block: it first collects the block's values, which are one piece of the caller's array, at their
//            positions of the (block, panel) order in a 96 KiB window of LDS (the positions, 16 bits relative to
//            the block where every block is shorter than 65 535, are part of the layout), then streams local row
//            and gathered x in that order - a contiguous piece per (panel, block) chunk, chunks padded to
//            multiples of 8 positions - against the window and adds val * xg (exact in fp64) to the row's fp64
//            accumulator in LDS with an LDS atomic.  A row is rounded once when the block is written.  The blocks
//            are started heaviest first.
//
// The order of the fp64 additions into a row's accumulator depends on scheduling: two calls may differ in the last
// bit of an element.  No value is kept: csrValues may change between calls, the structure may not.
//
// Preprocessing (once per structure, all on the device): a stable radix sort of the entries on the panel number
// keeps rows, hence row blocks, ascending inside a panel, so it yields the (panel, block) order directly; the
// position of a chunk in (block, panel) order follows from the chunk sizes by a prefix sum.
//
// Long rows.  A row of 4096 entries and 64 per panel or more whose columns ascend is kept out of the (block, panel)
// order: its entries of a panel are a contiguous piece of the caller's own arrays, found by a search in the sorted
// columns, and the phase-1 workgroup of the panel, which has the panel's x in LDS anyway, sums val * x over the
// piece with a lane group of 16 and leaves the fp64 sum in a small table; the phase-2 workgroup that owns the row
// (or, where a block holds more than 64 such rows, a kernel with a wavefront a row) adds the row's sums up in
// panel order.  8 bytes an entry instead of 18, and the values read are the caller's as they are at the call.
// (The template and layout arms for frozen values and op(A) = A^T that this file grew out of are those of
// spmv_blocked.hip; here they are compile-time constants and dropped by the compiler.)
#include <climits>
#include <cstdlib>

#include "convert_internal.h"
#include "device_utils.h"
#include "spmv_internal.h"

namespace opsparse {
namespace live_layout {

constexpr int kBlkThreads = 1024;                 // one workgroup per CU: it owns 128 KiB of LDS and more
constexpr int kPanelLog = 15;                     // columns per panel: 128 KiB of fp32 x
constexpr int kPanelCols = 1 << kPanelLog;
constexpr int kRowBlockLog = 14;                  // rows per row block: 128 KiB of fp64 accumulators
constexpr int kRowBlockRows = 1 << kRowBlockLog;
// Live values: the workgroup of a row block also holds the block's values, as they are at the call, in LDS
constexpr int kLiveRowBlockLog = 12;              // 32 KiB of accumulators
constexpr int kLiveRowBlockRows = 1 << kLiveRowBlockLog;
constexpr int kRefreshSpan = 24576;               // block-order positions whose values it holds at a time: 96 KiB
constexpr int64_t kLiveWindow = 20000;            // entries of a row block that is to fit that, padding included
constexpr int kMaxPanels = 1024;                  // chunk tables of one row block in LDS: 8 KiB
constexpr int kMaxGroups = 11776;                 // chunk of every 64th position of a row block in LDS: 23 KiB
constexpr int kGatherBatch = 8;                   // groups of 4 entries in flight per lane, phase 1
constexpr int kLaneEntries = 8;                   // consecutive entries a lane takes per batch, phase 2
constexpr uint32_t kPadRow = 0x8000;              // local row of a padding position in block order
constexpr int64_t kMinEntryWindow = 16384;
constexpr int64_t kMinEntryBlocks = 512;          // entry windows a matrix is cut into at least (if it has the entries)
constexpr int64_t kMinEntries = 2000000;          // below this the ordinary kernels are as fast or faster
// x of more than 2^18 elements.  An x of 1 - 4 MB fits an L2, but gathers scattered over it still cost the row-wise
// kernels 5.5 us per million (the rate at which an L2 answers them) against 3.6 us per million entries for the
// layout with frozen values: 1 M x 1 M with 32 random columns a row 189 -> 108 us (live values 143 us), over 2^19
// columns 157 -> 106 us, a power-law matrix of 1 M rows 100 -> 46 us and its transpose 533 -> 48 us.  (The bound
// used to be 2^20.)  Whether the gathers are scattered is for the sample of the column indices to say.
constexpr int64_t kMinCols = int64_t{1} << 18;
constexpr int64_t kMinChunkEntries = 32;          // below this mean chunk size the layout does not pay
// Live values (the default plan, which competes with the merge path on the caller's arrays rather than with a
// re-stored matrix): the window of values in LDS makes the row blocks short and the chunks with them; it pays down
// to 8 entries a chunk (2 M rows x 16 over 30 M columns, 17 a chunk: 212 us against 603 for the merge path; 6 M
// rows x 2 over 20 M columns, 9.5 a chunk: 123 us against 230).
constexpr int64_t kMinChunkEntriesLive = 8;
constexpr int64_t kLongChunkMean = 64;            // a row is "long" with this many entries per panel on average
constexpr int64_t kLongMinRow = 4096;             // and at least this many in all
// (frozen values: the long entries are stored again, a panel's in one piece, and stream whatever the rows' lengths;
// c3 per call: 218.8 us without long rows, 200.5 with the thresholds above, 194.5 with these)
constexpr int64_t kLongChunkMeanFrozen = 4;
constexpr int64_t kLongMinRowFrozen = 1024;
constexpr int kLongLanes = 16;        // lanes that sum one (long row, panel) piece in phase 1
constexpr int32_t kInBlockLongRows = 64;          // long rows a row block's own workgroup adds up at most
// acc[] of a long row whose sum is left to SpmvLongRowSumKernel: a NaN that no arithmetic on fp32 inputs yields
constexpr long long kDeferredRowMark = 0x7ff8dead0000beefLL;
constexpr int kLongTile = 3072;                   // long rows whose piece bounds a phase-1 workgroup stages in LDS at a time

typedef float Float4 __attribute__((ext_vector_type(4)));
typedef unsigned short Ushort4 __attribute__((ext_vector_type(4)));

// Row block of a row: 2^14-row blocks, cut again wherever the row's first entry
// passes a multiple of the entry window.  Monotone in the row number.
__device__ __forceinline__ int32_t RowBlockOf(const int32_t *__restrict__ rowOffsets, int32_t row, int32_t rowLog, int32_t window,
                                              int32_t numBlocks)
{
    const int32_t b = (row >> rowLog) + rowOffsets[row] / window;
    return b < 0 ? 0 : (b < numBlocks ? b : numBlocks - 1);  // in range whatever rowOffsets holds
}

// longBefore[r] = number of long rows among rows 0 .. r (an inclusive prefix sum of the flags).
__device__ __forceinline__ bool IsLongRow(const int32_t *__restrict__ longBefore, int32_t row)
{
    return longBefore[row] != (row > 0 ? longBefore[row - 1] : 0);
}

// ------------------------------------------------------------ preprocessing

// For the entries in (panel, original position) order: local column index, chunk
// key panel * B + block, and the row.  A column outside [0, cols) sets *status.
__global__ __launch_bounds__(kBlockThreads) void BlockedChunkKeysKernel(
    const int32_t *__restrict__ colSorted, const int32_t *__restrict__ pos, const int32_t *__restrict__ rowOfPos,
    const int32_t *__restrict__ rowOffsets, int64_t nnz, int64_t cols, int32_t numBlocks, int32_t rowLog, int32_t window,
    const int32_t *__restrict__ longBefore, uint16_t *__restrict__ colLocal, int32_t *__restrict__ chunkKey,
    int32_t *__restrict__ rowOfSrc, int32_t *__restrict__ status)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t col = colSorted[i];
        const int32_t row = rowOfPos[pos[i]];
        rowOfSrc[i] = row;
        colLocal[i] = static_cast<uint16_t>(col & (kPanelCols - 1));
        if (longBefore != nullptr && IsLongRow(longBefore, row)) {
            chunkKey[i] = -1;  // an entry of a long row (sorted behind every panel): phase 1 takes it from the CSR arrays
        } else if (col < 0 || col >= cols) {
            atomicOr(status, 1);
            chunkKey[i] = -1;
        } else {
            chunkKey[i] = (col >> kPanelLog) * numBlocks + RowBlockOf(rowOffsets, row, rowLog, window, numBlocks);
        }
    }
}

// flags[r] = 1 for a row of at least `minLen` entries.
__global__ __launch_bounds__(kBlockThreads) void LongRowFlagsKernel(const int32_t *__restrict__ rowOffsets,
                                                                    int64_t rows, int32_t minLen,
                                                                    int32_t *__restrict__ flags)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r < rows) {
        flags[r] = (rowOffsets[r + 1] - rowOffsets[r] >= minLen) ? 1 : 0;
    }
}

// Clears the flag of a row with a column outside [0, cols) or columns that do not ascend: such a row takes the
// ordinary way (which reports the bad column).
__global__ __launch_bounds__(kBlockThreads) void LongRowCheckKernel(const int32_t *__restrict__ rowOffsets,
                                                                    const int32_t *__restrict__ colInd,
                                                                    const int32_t *__restrict__ rowOfPos, int64_t nnz,
                                                                    int64_t cols, int32_t *flags)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t row = rowOfPos[i];
        if (flags[row] == 0) {
            continue;
        }
        const int32_t c = colInd[i];
        bool bad = c < 0 || c >= cols;
        if (i + 1 < rowOffsets[row + 1] && colInd[i + 1] < c) {
            bad = true;
        }
        if (bad) {
            flags[row] = 0;
        }
    }
}

// From the prefix-summed flags: the list of long rows, their number (header[1]) and entries (header[2], zero
// before).
__global__ __launch_bounds__(kBlockThreads) void LongRowListKernel(const int32_t *__restrict__ rowOffsets,
                                                                   const int32_t *__restrict__ longBefore,
                                                                   int64_t rows, int32_t maxLong,
                                                                   int32_t *__restrict__ longRows,
                                                                   int32_t *__restrict__ header)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const int32_t row = static_cast<int32_t>(r);
    if (r == rows - 1) {
        header[1] = longBefore[row] < maxLong ? longBefore[row] : maxLong;
    }
    if (IsLongRow(longBefore, row) && longBefore[row] <= maxLong) {
        longRows[longBefore[row] - 1] = row;
        atomicAdd(header + 2, rowOffsets[row + 1] - rowOffsets[row]);
    }
}

// Row offsets with the entries of the long rows taken out, which is what the row blocks are cut by (a block is to
// hold a share of the entries that phase 2 streams).  First out[r + 1] = entries of row r if it is long (out[0] =
// 0), then, after an inclusive prefix sum, out[r] = rowOffsets[r] - out[r].
__global__ __launch_bounds__(kBlockThreads) void LongRowEntriesKernel(const int32_t *__restrict__ rowOffsets,
                                                                      const int32_t *__restrict__ longBefore,
                                                                      int64_t rows, int32_t *__restrict__ out)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r == 0) {
        out[0] = 0;
    }
    if (r < rows) {
        const int32_t row = static_cast<int32_t>(r);
        out[r + 1] = IsLongRow(longBefore, row) ? rowOffsets[row + 1] - rowOffsets[row] : 0;
    }
}

__global__ __launch_bounds__(kBlockThreads) void ShortOffsetsKernel(const int32_t *__restrict__ rowOffsets,
                                                                    int64_t rows, int32_t *__restrict__ inOut)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r <= rows) {
        inOut[r] = rowOffsets[r] - inOut[r];
    }
}

// Sort keys of the entries in CSR order: the column, or for an entry of a long row a column past the last panel,
// which sorts it behind every panel: `longKey` itself (live values: the entries are then read where the caller
// has them), or longKey + column (frozen values: behind the short entries the long ones follow panel by panel,
// in row order inside a panel, and are stored there a second time like the short ones).
__global__ __launch_bounds__(kBlockThreads) void LongRowKeysKernel(const int32_t *__restrict__ colInd,
                                                                   const int32_t *__restrict__ rowOfPos,
                                                                   const int32_t *__restrict__ longBefore, int64_t nnz,
                                                                   int32_t longKey, int32_t byPanel,
                                                                   int32_t *__restrict__ keys)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t col = colInd[i];
        keys[i] = IsLongRow(longBefore, rowOfPos[i]) ? longKey + (byPanel != 0 ? col : 0) : col;
    }
}

// longChunk[p * maxLong + l] = first entry of long row l with a column in panel p or later (p == P: the row's end).
// Panel-major: the workgroup of a panel reads the bounds of all rows as two linear pieces.
__global__ __launch_bounds__(kBlockThreads) void LongRowChunksKernel(const int32_t *__restrict__ rowOffsets,
                                                                     const int32_t *__restrict__ colInd,
                                                                     const int32_t *__restrict__ longRows,
                                                                     const int32_t *__restrict__ header, int32_t P,
                                                                     int32_t maxLong, int32_t *__restrict__ longChunk)
{
    const int64_t total = static_cast<int64_t>(header[1]) * (P + 1);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < total; j += stride) {
        const int32_t l = static_cast<int32_t>(j / (P + 1)), p = static_cast<int32_t>(j % (P + 1));
        const int32_t row = longRows[l];
        int32_t lo = rowOffsets[row], hi = rowOffsets[row + 1];
        if (p == P) {
            lo = hi;
        } else {
            const int32_t want = p << kPanelLog;
            while (lo < hi) {
                const int32_t mid = lo + ((hi - lo) >> 1);
                if (colInd[mid] < want) {
                    lo = mid + 1;
                } else {
                    hi = mid;
                }
            }
        }
        longChunk[static_cast<int64_t>(p) * maxLong + l] = lo;
    }
}

// From srcStart (first entry of chunk (panel, block) in panel order, P * B + 1 values):
// dstStart[1 + block * P + panel] = size of the chunk, rounded up to a multiple of kLaneEntries (prefix-summed
// afterwards: in block order every chunk starts on such a multiple, the gap behind it is padding), and
// srcStartT[block * P + panel] = srcStart[panel * B + block].
__global__ __launch_bounds__(kBlockThreads) void BlockedTablesKernel(const int32_t *__restrict__ srcStart, int32_t P,
                                                                     int32_t B, int32_t *__restrict__ dstStart,
                                                                     int32_t *__restrict__ srcStartT)
{
    const int64_t total = static_cast<int64_t>(P) * B;
    const int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (j == 0) {
        dstStart[0] = 0;
    }
    if (j < total) {
        const int64_t b = j / P, p = j % P;
        const int32_t s = srcStart[p * B + b];
        const int32_t count = srcStart[p * B + b + 1] - s;
        dstStart[1 + j] = (count + kLaneEntries - 1) / kLaneEntries * kLaneEntries;
        srcStartT[j] = s;
    }
}

// blockRow[b] = first row of row block b (blockRow pre-filled with `rows`).
__global__ __launch_bounds__(kBlockThreads) void BlockedRowBlocksKernel(const int32_t *__restrict__ rowOffsets,
                                                                        int32_t rows, int32_t rowLog, int32_t window,
                                                                        int32_t B, int32_t *__restrict__ blockRow)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const int32_t row = static_cast<int32_t>(r);
    const int32_t cur = RowBlockOf(rowOffsets, row, rowLog, window, B);
    const int32_t prev = row > 0 ? RowBlockOf(rowOffsets, row - 1, rowLog, window, B) : -1;
    for (int32_t b = prev + 1; b <= cur; ++b) {
        blockRow[b] = row;
    }
}

// longFirst[b] = number of long rows in front of row block b (b = B: of all rows): block b has the long rows
// longFirst[b] .. longFirst[b + 1] - 1.
__global__ __launch_bounds__(kBlockThreads) void BlockedLongFirstKernel(const int32_t *__restrict__ blockRow,
                                                                        const int32_t *__restrict__ longBefore, int32_t B,
                                                                        int32_t *__restrict__ longFirst)
{
    const int32_t b = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (b <= B) {
        const int32_t row = blockRow[b];
        longFirst[b] = row > 0 ? longBefore[row - 1] : 0;
    }
}

// longDeferred[l] = 1 for the long rows of a row block that holds more than kInBlockLongRows of them, else 0;
// header[4] (zero before) = their number.
__global__ __launch_bounds__(kBlockThreads) void BlockedLongDeferKernel(const int32_t *__restrict__ longFirst, int32_t B,
                                                                        int32_t *__restrict__ longDeferred,
                                                                        int32_t *__restrict__ header)
{
    const int32_t b = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (b >= B) {
        return;
    }
    const int32_t l0 = longFirst[b], l1 = longFirst[b + 1];
    const int32_t defer = l1 - l0 > kInBlockLongRows ? 1 : 0;
    for (int32_t l = l0; l < l1; ++l) {
        longDeferred[l] = defer;
    }
    if (defer != 0) {
        atomicAdd(header + 4, l1 - l0);
    }
}

// A value or an element of x as the layout keeps it: fp32 (exact for fp16 and bf16).
__device__ __forceinline__ float AsFloat(float v) { return v; }
__device__ __forceinline__ float AsFloat(Half v) { return static_cast<float>(v); }
__device__ __forceinline__ float AsFloat(Bf16 v) { return Bf16ToFloat(v); }

// Four consecutive values of the caller's array as fp32, in one load (fp32: at any 4-byte-aligned address; fp16 /
// bf16: at any 2-byte-aligned one).
template <typename ValT>
__device__ __forceinline__ Float4U LoadFourValues(const ValT *p)
{
    if constexpr (std::is_same<ValT, float>::value) {
        return __builtin_nontemporal_load(reinterpret_cast<const Float4U *>(p));
    } else {
        const Short4U raw = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(p));
        ValT four[4];
        __builtin_memcpy(four, &raw, 8);
        return Float4U{AsFloat(four[0]), AsFloat(four[1]), AsFloat(four[2]), AsFloat(four[3])};
    }
}

// Values and local row indices into (block, panel) order.
template <typename ValT>
__global__ __launch_bounds__(kBlockThreads) void BlockedScatterKernel(
    const int32_t *__restrict__ pos, const int32_t *__restrict__ rowOfSrc, const int32_t *__restrict__ chunkKey,
    const ValT *__restrict__ vals, const int32_t *__restrict__ srcStart,
    const int32_t *__restrict__ dstStart, const int32_t *__restrict__ blockRow, int64_t nnz, int32_t P, int32_t B,
    float *__restrict__ valD, uint16_t *__restrict__ rowLocal, int32_t *__restrict__ dstOfPos,
    float *__restrict__ longVals, uint16_t *__restrict__ longRowOf, const int32_t *__restrict__ longBefore)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t key = chunkKey[i];
        if (key < 0) {
            if (longVals != nullptr) {
                // an entry of a long row, frozen values: its value and the number of its row among the long rows
                // beside its local column, all three at its place in the sorted order
                longVals[i] = AsFloat(vals[pos[i]]);
                longRowOf[i] = static_cast<uint16_t>(longBefore[rowOfSrc[i]] - 1);
            }
            continue;
        }
        const int32_t p = key / B, b = key % B;
        const int64_t dst = i - srcStart[key] + dstStart[static_cast<int64_t>(b) * P + p];
        if (valD != nullptr) {
            valD[dst] = AsFloat(vals[pos[i]]);
        }
        if (dstOfPos != nullptr) {
            dstOfPos[pos[i]] = static_cast<int32_t>(dst);
        }
        rowLocal[dst] = static_cast<uint16_t>((rowOfSrc[i] - blockRow[b]) & (kRowBlockRows - 1));  // < kPadRow
    }
}

// ------------------------------------------------ values of the caller, now


// Live values.  blockEntry[b] = first entry, in the caller's arrays, of row block b (b = B: the entry count);
// longSpan[2 l], [2 l + 1] = first entry of long row l and of the row behind it.
__global__ __launch_bounds__(kBlockThreads) void BlockedLiveTablesKernel(const int32_t *__restrict__ rowOffsets,
                                                                         const int32_t *__restrict__ blockRow, int32_t B,
                                                                         const int32_t *__restrict__ longRows,
                                                                         const int32_t *__restrict__ header,
                                                                         int32_t *__restrict__ blockEntry,
                                                                         int32_t *__restrict__ longSpan)
{
    const int32_t i = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (i <= B) {
        blockEntry[i] = rowOffsets[blockRow[i]];
    }
    if (header != nullptr && i < header[1]) {
        longSpan[2 * i] = rowOffsets[longRows[i]];
        longSpan[2 * i + 1] = rowOffsets[longRows[i] + 1];
    }
}

// header[3] = positions of the longest row block (zero before).
__global__ __launch_bounds__(kBlockThreads) void BlockedMaxPositionsKernel(const int32_t *__restrict__ dstStart,
                                                                           int32_t P, int32_t B,
                                                                           int32_t *__restrict__ header)
{
    const int32_t b = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (b < B) {
        atomicMax(header + 3, dstStart[static_cast<int64_t>(b + 1) * P] - dstStart[static_cast<int64_t>(b) * P]);
    }
}

constexpr uint32_t kNoPosition16 = 0xffffu;  // short position of an entry that has none (a long row's)
constexpr int32_t kLiveShortPositions = 2;   // plan.liveValues of a layout whose positions were re-stored that way

// Live values, every row block shorter than 65535 positions.  The block-order position of entry i of block b is
// re-stored as 16 bits relative to the block's first position, at ((uint16_t *)(dstOfPos + e0))[i - e0] with e0 the
// block's first entry: the short positions of a block lie in the front half of the bytes its 32-bit ones had, so
// a workgroup a block can convert in place, a piece at a time, reading a piece before it writes it (what it writes
// lies below what it has not read yet).
__global__ __launch_bounds__(kBlkThreads) void BlockedShortPositionsKernel(const int32_t *__restrict__ blockEntry,
                                                                          const int32_t *__restrict__ dstStart,
                                                                          int32_t P, int32_t *dstOfPos)
{
    constexpr int kPer = 8;
    const int64_t b = blockIdx.x;
    const int32_t e0 = blockEntry[b], e1 = blockEntry[b + 1], dBeg = dstStart[b * P];
    auto *out = reinterpret_cast<uint16_t *>(dstOfPos + e0);
    for (int32_t c0 = e0; c0 < e1; c0 += kBlkThreads * kPer) {
        int32_t v[kPer];
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int32_t i = c0 + u * kBlkThreads + static_cast<int32_t>(threadIdx.x);
            v[u] = i < e1 ? dstOfPos[i] : -1;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int32_t i = c0 + u * kBlkThreads + static_cast<int32_t>(threadIdx.x);
            if (i < e1) {
                out[i - e0] = static_cast<uint16_t>(v[u] < 0 ? kNoPosition16 : static_cast<uint32_t>(v[u] - dBeg));
            }
        }
        __syncthreads();
    }
}

// Live values.  The entries of a row block are one contiguous piece of the caller's arrays and one contiguous
// piece of the block order.  The workgroup that owns the block reads the former (values and their block-order
// positions, both linear) and keeps what falls into the window [w0, w0 + span) of the latter in LDS:
// win[position - w0] = value as it is at this call.  Entries of long rows have no position (-1, or kNoPosition16).
// A block of more than kRefreshSpan positions reads its entries once per window.  [e0, e1) here is a piece of the
// block's entries between two long rows (whose own entries are skipped); Short: the positions are the 16-bit ones
// of BlockedShortPositionsKernel, blockE0 and dBeg the block's first entry and first position.
template <bool Short, typename ValT>
__device__ __forceinline__ void FillLiveWindow(const ValT *__restrict__ vals, const int32_t *__restrict__ dstOfPos,
                                               int32_t e0, int32_t e1, int32_t w0, uint32_t span, float *win, int tid,
                                               int32_t blockE0, int32_t dBeg)
{
    typedef unsigned short Ushort4U __attribute__((ext_vector_type(4), aligned(2)));
    const uint16_t *pos16 = reinterpret_cast<const uint16_t *>(dstOfPos + blockE0) - blockE0;  // indexed by entry
    const uint32_t shift = static_cast<uint32_t>(dBeg - w0);
    // window-relative position of entry i, or a value >= span
    auto place = [&](int32_t i) {
        if (Short) {
            const uint32_t d = pos16[i];
            return d == kNoPosition16 ? 0xffffffffu : d + shift;
        }
        return static_cast<uint32_t>(dstOfPos[i] - w0);
    };
    // aligned groups of four entries as 16-byte loads, the ragged ends one by one
    const int32_t g0 = (e0 + 3) & ~3, g1 = e1 & ~3;
    if (g0 >= g1) {
        for (int32_t i = e0 + tid; i < e1; i += kBlkThreads) {
            const uint32_t at = place(i);
            if (at < span) {
                win[at] = AsFloat(vals[i]);
            }
        }
        return;
    }
    if (tid < 8) {
        const int32_t i = tid < 4 ? e0 + tid : g1 + (tid - 4);
        if ((tid < 4 && i < g0) || (tid >= 4 && i < e1)) {
            const uint32_t at = place(i);
            if (at < span) {
                win[at] = AsFloat(vals[i]);
            }
        }
    }
    const bool vecVals = (reinterpret_cast<uintptr_t>(vals) & (4 * sizeof(ValT) - 1)) == 0;
    // kRefreshBatch groups in flight per lane: loads first (clamped to the last group), then the LDS writes
    constexpr int kRefreshBatch = 6;  // (a block of kLiveWindow entries in one turn)
    for (int32_t i0 = g0 + tid * 4; i0 < g1; i0 += kBlkThreads * 4 * kRefreshBatch) {
        Int4U d[kRefreshBatch];
        Ushort4U d16[kRefreshBatch];
        Float4U v[kRefreshBatch];
#pragma unroll
        for (int u = 0; u < kRefreshBatch; ++u) {
            int32_t i = i0 + u * kBlkThreads * 4;
            i = i < g1 ? i : g1 - 4;
            if (Short) {
                d16[u] = __builtin_nontemporal_load(reinterpret_cast<const Ushort4U *>(pos16 + i));
            } else {
                d[u] = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(dstOfPos + i));
            }
            if (vecVals) {
                v[u] = LoadFourValues(vals + i);
            } else {
                v[u] = Float4U{AsFloat(vals[i]), AsFloat(vals[i + 1]), AsFloat(vals[i + 2]), AsFloat(vals[i + 3])};
            }
        }
#pragma unroll
        for (int u = 0; u < kRefreshBatch; ++u) {
            // (a clamped group writes the same values to the same places again)
            uint32_t a0, a1, a2, a3;
            if (Short) {
                const uint32_t q[4] = {d16[u].x, d16[u].y, d16[u].z, d16[u].w};
                a0 = q[0] == kNoPosition16 ? 0xffffffffu : q[0] + shift;
                a1 = q[1] == kNoPosition16 ? 0xffffffffu : q[1] + shift;
                a2 = q[2] == kNoPosition16 ? 0xffffffffu : q[2] + shift;
                a3 = q[3] == kNoPosition16 ? 0xffffffffu : q[3] + shift;
            } else {
                a0 = static_cast<uint32_t>(d[u].x - w0);
                a1 = static_cast<uint32_t>(d[u].y - w0);
                a2 = static_cast<uint32_t>(d[u].z - w0);
                a3 = static_cast<uint32_t>(d[u].w - w0);
            }
            if (a0 < span) win[a0] = v[u].x;
            if (a1 < span) win[a1] = v[u].y;
            if (a2 < span) win[a2] = v[u].z;
            if (a3 < span) win[a3] = v[u].w;
        }
    }
}

// ------------------------------------------------------------------ phase 1

// xg[i] = x[panel * 2^15 + colLocal[i]] for the entries of one panel (a part of them when
// `splits` > 1), the panel's slice of x held in LDS.
//
// Long rows: `header[1]` of them; longPartial[l * P + p] receives the fp64 sum of val * x over the entries of long
// row l in panel p.  Live values: these are the entries longChunk[p * maxLong + l] .. longChunk[(p + 1) * maxLong +
// l] of the caller's colInd / vals, and groups of kLongLanes lanes take the rows in turn.  Frozen values
// (LongSorted): the panel's long entries follow each other, in row order, at the positions longChunk[p * (maxLong
// + 1)] .. longChunk[p * (maxLong + 1) + header[1]] of colLocal, of xg (which there holds their values) and of
// longRowOf (the number l of each one's row); the workgroup streams them like phase 2 streams a row block, with an
// fp64 accumulator a row in LDS, kLongTile rows at a time ([.. + l] is where row l starts).

template <typename XT>
__global__ __launch_bounds__(kBlkThreads) void SpmvBlockGatherKernel(const uint16_t *__restrict__ colLocal,
                                                                     const XT *__restrict__ x,
                                                                     float *__restrict__ xg,
                                                                     const int32_t *__restrict__ srcStart,
                                                                     int64_t cols, int32_t B, int32_t splits,
                                                                     const int32_t *__restrict__ header,
                                                                     const int32_t *__restrict__ longChunk,
                                                                     const int32_t *__restrict__ colInd,
                                                                     const XT *__restrict__ vals, int64_t nnz,
                                                                     int32_t P, int32_t maxLong,
                                                                     const uint16_t *__restrict__ longRowOf,
                                                                     double *__restrict__ longPartial)
{
    __shared__ float xs[kPanelCols];
    __shared__ __align__(16) int32_t tileBuf[2 * kLongTile];  // piece bounds (live) or fp64 accumulators (frozen)
    int32_t *pieceLo = tileBuf, *pieceHi = tileBuf + kLongTile;
    const int tid = threadIdx.x;
    // Neighbouring panels on one XCD: the pieces of a long row in panels p and p + 1 are neighbours in memory, and
    // the cache line they share is then fetched once, by the L2 both workgroups sit behind.
    const int64_t p = splits == 1 ? XcdContiguousTile(blockIdx.x, gridDim.x) : blockIdx.x / splits;
    const int64_t part = splits == 1 ? 0 : blockIdx.x % splits;
    const int64_t c0 = p << kPanelLog;
    const int64_t cn = cols - c0 < kPanelCols ? cols - c0 : kPanelCols;
    const int64_t a = srcStart[p * B], e = srcStart[(p + 1) * B];
    if constexpr (std::is_same<XT, float>::value) {
        const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
        for (int64_t i = tid * 4; i < cn; i += kBlkThreads * 4) {
            if (vec && i + 4 <= cn) {
                *reinterpret_cast<Float4 *>(xs + i) = *reinterpret_cast<const Float4 *>(x + c0 + i);
            } else {
                for (int64_t k = i; k < cn && k < i + 4; ++k) {
                    xs[k] = x[c0 + k];
                }
            }
        }
    } else {
        // fp16 / bf16 x: widened once, here; the panel's slice starts at a multiple of 2^15
        // elements, so 8-byte loads are aligned where x is
        const bool vec = (reinterpret_cast<uintptr_t>(x) & 7) == 0;
        for (int64_t i = tid * 4; i < cn; i += kBlkThreads * 4) {
            if (vec && i + 4 <= cn) {
                XT four[4];
                *reinterpret_cast<uint2 *>(four) = *reinterpret_cast<const uint2 *>(x + c0 + i);
                Float4 f;
                f.x = AsFloat(four[0]);
                f.y = AsFloat(four[1]);
                f.z = AsFloat(four[2]);
                f.w = AsFloat(four[3]);
                *reinterpret_cast<Float4 *>(xs + i) = f;
            } else {
                for (int64_t k = i; k < cn && k < i + 4; ++k) {
                    xs[k] = AsFloat(x[c0 + k]);
                }
            }
        }
    }
    __syncthreads();
    const int64_t len = e - a;
    const int64_t lo = a + len * part / splits, hi = a + len * (part + 1) / splits;
    // Whole aligned groups of 4 entries go as 8-byte loads and 16-byte stores; what is left at
    // either end of [lo, hi) is done one by one.
    const int64_t g0 = (lo + 3) >> 2, g1 = hi >> 2;
    if (lo < hi && g0 > g1) {
        if (tid < 4 && lo + tid < hi) {
            xg[lo + tid] = xs[colLocal[lo + tid]];
        }
    } else if (lo < hi) {
        if (tid < 4) {
            const int64_t i = lo + tid;
            if (i < g0 * 4) {
                xg[i] = xs[colLocal[i]];
            }
        } else if (tid < 8) {
            const int64_t i = g1 * 4 + (tid - 4);
            if (i < hi) {
                xg[i] = xs[colLocal[i]];
            }
        }
        for (int64_t g = g0; g < g1; g += kGatherBatch * kBlkThreads) {
            Ushort4 c[kGatherBatch];
            // Unconditional loads (clamped to the last group): the compiler keeps all of them in flight.
#pragma unroll
            for (int u = 0; u < kGatherBatch; ++u) {
                int64_t gg = g + u * kBlkThreads + tid;
                gg = gg < g1 ? gg : g1 - 1;
                c[u] = __builtin_nontemporal_load(reinterpret_cast<const Ushort4 *>(colLocal) + gg);
            }
#pragma unroll
            for (int u = 0; u < kGatherBatch; ++u) {
                const int64_t gg = g + u * kBlkThreads + tid;
                Float4 r;
                r.x = xs[c[u].x];
                r.y = xs[c[u].y];
                r.z = xs[c[u].z];
                r.w = xs[c[u].w];
                if (gg < g1) {
                    *(reinterpret_cast<Float4 *>(xg) + gg) = r;
                }
            }
        }
    }
    // ---- long rows: this panel's piece of each, summed from the caller's arrays
    const int32_t numLong = header != nullptr ? header[1] : 0;
    if (numLong == 0) {
        return;
    }
    constexpr int kGroups = kBlkThreads / kLongLanes;
    const int32_t gl = tid / kLongLanes, gt = tid % kLongLanes;
    const int32_t base = static_cast<int32_t>(c0);
    const int32_t *loTab = longChunk + p * maxLong, *hiTab = longChunk + (p + 1) * maxLong;
    for (int32_t t0 = 0; t0 < numLong; t0 += kLongTile) {
        const int32_t tn = numLong - t0 < kLongTile ? numLong - t0 : kLongTile;
        __syncthreads();  // (the tile before is done with)
        for (int32_t i = tid; i < tn; i += kBlkThreads) {
            pieceLo[i] = loTab[t0 + i];
            pieceHi[i] = hiTab[t0 + i];
        }
        __syncthreads();
        // Groups of kLongLanes lanes take the rows of the tile in turn (a part of them when a panel has several
        // workgroups), each lane 16 bytes of either array per request.  Most pieces are a request or two long, so
        // what a group waits for is the round trip of each piece: the first request of the group's next piece is
        // made before this piece is added up (for the last piece the same one again: no branch around the loads).
        const int32_t stride = static_cast<int32_t>(splits) * kGroups;
        int32_t k = static_cast<int32_t>(part) + static_cast<int32_t>(splits) * gl;
        if (k < tn) {
            // Group q of a piece [i0, i1) holds its entries 4 q .. 4 q + 3; the last group may be short.  A request
            // is always four whole entries: it starts at most at i1 - 4 (never below 0), so the last group reads a
            // few entries in front of its own, and a group past the end re-reads the last one; `add` takes only the
            // entries that are the group's own.  No entry is ever fetched one by one.
            auto request = [&](int32_t i0, int32_t i1, int32_t q, Int4U *c, Float4U *v) {
                int64_t at = i0 + 4 * static_cast<int64_t>(q);
                at = at + 4 <= i1 ? at : static_cast<int64_t>(i1) - 4;
                at = at < 0 ? 0 : at;
                *c = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(colInd + at));
                *v = LoadFourValues(vals + at);
            };
            auto add = [&](int32_t i0, int32_t i1, int32_t q, const Int4U &c, const Float4U &v, double *sum) {
                const int64_t own = i0 + 4 * static_cast<int64_t>(q);  // first entry of the group
                int64_t at = own + 4 <= i1 ? own : static_cast<int64_t>(i1) - 4;
                at = at < 0 ? 0 : at;
                const uint32_t mask = kPanelCols - 1;  // an entry of the group is in the panel by construction
                const int32_t cs[4] = {c.x, c.y, c.z, c.w};
                const float vs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const double t = static_cast<double>(vs[j]) *
                                     static_cast<double>(xs[static_cast<uint32_t>(cs[j] - base) & mask]);
                    *sum += (at + j >= own && at + j < i1) ? t : 0.0;
                }
            };
            int32_t i0 = pieceLo[k], i1 = pieceHi[k];
            Int4U cFirst;
            Float4U vFirst;
            request(i0, i1, gt, &cFirst, &vFirst);
            while (true) {
                const int32_t kn = k + stride;
                const int32_t kk = kn < tn ? kn : k;
                const int32_t j0 = pieceLo[kk], j1 = pieceHi[kk];
                Int4U cAhead;
                Float4U vAhead;
                request(j0, j1, gt, &cAhead, &vAhead);
                const int32_t n4 = (i1 - i0 + 3) >> 2;  // groups of the piece, the last one maybe short
                double sum = 0.0;
                Int4U c = cFirst;
                Float4U v = vFirst;
                for (int32_t q = gt; q < n4; q += kLongLanes) {
                    Int4U cNext;
                    Float4U vNext;
                    request(i0, i1, q + kLongLanes, &cNext, &vNext);
                    add(i0, i1, q, c, v, &sum);
                    c = cNext;
                    v = vNext;
                }
#pragma unroll
                for (int off = kLongLanes / 2; off > 0; off >>= 1) {
                    sum += __shfl_xor(sum, off, kLongLanes);
                }
                if (gt == 0) {
                    longPartial[static_cast<int64_t>(t0 + k) * P + p] = sum;
                }
                if (kn >= tn) {
                    break;
                }
                k = kn;
                i0 = j0;
                i1 = j1;
                cFirst = cAhead;
                vFirst = vAhead;
            }
        }
    }
}

// ------------------------------------------------------------------ phase 2

typedef float Float4U1 __attribute__((ext_vector_type(4), aligned(4)));   // dword-aligned 16-byte load
typedef uint32_t Uint4 __attribute__((ext_vector_type(4)));
typedef uint32_t Uint2 __attribute__((ext_vector_type(2)));

// Adds the per-lane sums of a wavefront to acc[key] (key < 0: nothing pending).
__device__ __forceinline__ void FlushPending(double *acc, int32_t key, double pending)
{
    if (key < 0) {
        return;
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        pending += __shfl_xor(pending, off);
    }
    if (threadIdx.x % kWave == 0) {
        atomicAdd(&acc[key], pending);
    }
}

// Chunk (panel) of block-order position `pos`: the largest p with tabD[p] <= pos.
__device__ __forceinline__ int ChunkOf(const int32_t *tabD, int32_t P, int32_t pos)
{
    int lo = 0, hi = P;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tabD[mid] <= pos) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    return lo;
}

// What a lane loads for one batch: kSubBatches runs of kSubEntries consecutive positions of the block, run s
// at start + s * (64 * kSubEntries) + lane * kSubEntries, so that every load instruction of a wavefront covers
// one contiguous kilobyte (values, gathered x) or half of one (local rows).
constexpr int kSubEntries = 4;
constexpr int kSubBatches = kLaneEntries / kSubEntries;
constexpr int kSubSpan = kWave * kSubEntries;  // positions one load instruction of a wavefront covers

struct LanePiece {
    Float4U1 a[kSubBatches], x[kSubBatches];
    Uint2 rows[kSubBatches];
    bool live[kSubBatches];  // false: a run past the end, which re-read the last run
};

// (Row blocks of 2^13 or 2^12 rows, so that two or three workgroups of 512 or 1024 threads share a CU, were no
// faster on c3 with frozen values: 193.7 .. 211 us a call against 191.4; the shorter chunks cost what the overlap
// gains.)
constexpr int kRedThreads = kBlkThreads, kRedWaves = kRedThreads / kWave;

// One workgroup per row block: y[row] = alpha * sum(val * xg) + beta * yIn[row].
//
// In block order every (panel, block) chunk starts on a multiple of kLaneEntries and is padded to one
// (padding carries the local row kPadRow and the value 0).  A lane takes runs of kSubEntries consecutive
// positions, which therefore lie in one chunk.  tabD[p] is the first block-order position of the block's chunk
// from panel p, tabDelta[p] the distance from there to the chunk in panel order, groupChunk[g] the chunk of
// position 64 * g of the piece being streamed.  Two batches are in flight: the next one's loads are issued,
// unconditionally, before this one is added up.  Entries of one row are neighbours: a lane adds its runs up in
// registers and touches the row's accumulator in LDS once per run; a row that fills whole wavefronts is summed
// per lane in `pending` and reaches LDS once.
//
// Frozen values (Live == false): the block's positions are streamed in one piece, values from valD.  Live: window
// by window of kRefreshSpan positions (partDesc[partStart[block]] ..: entries, positions); the values of a window
// are first collected in LDS from the caller's array, and the stream takes them from there.  Padding positions of
// a window hold whatever LDS held: their products are formed and dropped.
template <bool Live, bool Short, typename ValT, typename OutT>
__global__ __launch_bounds__(kRedThreads) void SpmvBlockReduceKernel(
    const float *__restrict__ valD, const float *__restrict__ xg, const uint16_t *__restrict__ rowLocal,
    const int32_t *__restrict__ dstStart, const int32_t *__restrict__ srcStartT, int32_t P,
    const int32_t *__restrict__ blockOrder, const int32_t *__restrict__ blockRow, OutT *__restrict__ y,
    const OutT *__restrict__ yIn, OpsparseScalar alphaS, OpsparseScalar betaS, const int32_t *__restrict__ longFirst,
    const int32_t *__restrict__ longRows, const double *__restrict__ longPartial, const ValT *__restrict__ vals,
    const int32_t *__restrict__ dstOfPos, const int32_t *__restrict__ blockEntry, const int32_t *__restrict__ longSpan)
{
    constexpr int kGroupSlots = Live ? kRefreshSpan / kWave : kMaxGroups;
    constexpr int kAccRows = Live ? kLiveRowBlockRows : kRowBlockRows;
    __shared__ __align__(16) double acc[kAccRows];
    __shared__ int32_t tabD[kMaxPanels + 1];
    __shared__ int32_t tabDelta[kMaxPanels];
    __shared__ uint16_t groupChunk[kGroupSlots];
    __shared__ __align__(16) float win[Live ? kRefreshSpan : 4];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    // What a workgroup waits for is a chain of round trips to memory, one workgroup a CU: everything that does not
    // depend on an earlier load is asked for at the start.  (Live values: the blocks are alike in size by
    // construction and are taken in row order; the frozen layout starts its heaviest blocks first.)
    const int64_t blk = Live ? static_cast<int64_t>(blockIdx.x) : blockOrder[blockIdx.x];
    const int32_t row0 = blockRow[blk], row1 = blockRow[blk + 1];
    const int32_t l0 = longFirst != nullptr ? longFirst[blk] : 0, l1 = longFirst != nullptr ? longFirst[blk + 1] : 0;
    const int32_t dBeg = dstStart[blk * P], dEnd = dstStart[blk * P + P];  // the block's piece of the block order
    const int32_t e0 = Live ? blockEntry[blk] : 0, e1 = Live ? blockEntry[blk + 1] : 0;
    typedef double Double2 __attribute__((ext_vector_type(2)));
    for (int i = tid * 2; i < kAccRows; i += kRedThreads * 2) {
        *reinterpret_cast<Double2 *>(acc + i) = Double2{0.0, 0.0};
    }
    LdsBarrier();
    if (row0 >= row1) {
        return;  // a block number no row maps to
    }
    // the chunk tables, into registers for now (P + 1 <= 1025 entries: one a thread, thread 0 the last as well)
    const int32_t tabMine = tid <= P ? dstStart[blk * P + tid] : 0;
    const int32_t tabSrc = tid < P ? srcStartT[blk * P + tid] : 0;
    const int32_t tabLast = (tid == 0 && P >= kRedThreads) ? dstStart[blk * P + kRedThreads] : 0;
    const int32_t spanMax = Live ? kRefreshSpan : INT32_MAX;
    auto fillWindow = [&](int32_t w0, int32_t w1) {
        // the block's entries without those of its long rows
        int32_t cur = e0;
        for (int32_t l = l0; l < l1; ++l) {
            FillLiveWindow<Short, ValT>(vals, dstOfPos, cur, longSpan[2 * l], w0, static_cast<uint32_t>(w1 - w0), win, tid, e0,
                                  dBeg);
            cur = longSpan[2 * l + 1];
        }
        FillLiveWindow<Short, ValT>(vals, dstOfPos, cur, e1, w0, static_cast<uint32_t>(w1 - w0), win, tid, e0, dBeg);
    };
    if (Live && dBeg < dEnd) {
        fillWindow(dBeg, dEnd - dBeg > spanMax ? dBeg + spanMax : dEnd);
    }
    if (tid <= P) {
        tabD[tid] = tabMine;
    }
    if (tid < P) {
        tabDelta[tid] = tabSrc - tabMine;
    }
    if (tid == 0 && P >= kRedThreads) {
        tabD[kRedThreads] = tabLast;
    }
    // Long rows of this block: phase 1 left the fp64 sum of each of their panels; a wavefront adds a row's up, lane
    // by lane in panel order and then across the lanes, the same way at every call.  A block with more than
    // kInBlockLongRows of them leaves that to SpmvLongRowSumKernel (a matrix of long rows only has few blocks) and
    // marks the rows, which nothing else touches, so that they are not written here.
    const bool deferLong = l1 - l0 > kInBlockLongRows;
    if (deferLong) {
        for (int32_t l = l0 + tid; l < l1; l += kRedThreads) {
            acc[longRows[l] - row0] = __longlong_as_double(kDeferredRowMark);
        }
    }
    for (int32_t l = l0 + wave; l < l1 && !deferLong; l += kRedWaves) {
        double sum = 0.0;
        const double *from = longPartial + static_cast<int64_t>(l) * P;
        for (int32_t p0 = 0; p0 < P; p0 += 4 * kWave) {
            double v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int32_t p = p0 + u * kWave + lane;
                v[u] = from[p < P ? p : P - 1];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                sum += p0 + u * kWave + lane < P ? v[u] : 0.0;
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            sum += __shfl_xor(sum, off);
        }
        if (lane == 0) {
            atomicAdd(&acc[longRows[l] - row0], sum);
        }
    }
    constexpr int kBatch = kWave * kLaneEntries;
    constexpr int kStride = kRedWaves * kBatch;
    double pending = 0.0;
    int32_t pendingKey = -1;
    // the piece [d0, d1) of the block order, both multiples of kLaneEntries: all of the block, or window by window
    for (int32_t d0 = dBeg, d1; d0 < dEnd; d0 = d1) {
        d1 = dEnd - d0 > spanMax ? d0 + spanMax : dEnd;
        if (Live && d0 > dBeg) {
            __syncthreads();  // the window before is done with
            fillWindow(d0, d1);
        }
        __syncthreads();
        int32_t groups = (d1 - d0 + kWave - 1) / kWave;
        groups = groups < kGroupSlots ? groups : kGroupSlots;
        for (int32_t p = tid; p < P; p += kRedThreads) {
            int32_t g = (tabD[p] - d0 + kWave - 1) / kWave;
            int32_t gEnd = (tabD[p + 1] - d0 + kWave - 1) / kWave;
            g = g > 0 ? g : 0;
            gEnd = gEnd < groups ? gEnd : groups;
            for (; g < gEnd; ++g) {
                groupChunk[g] = static_cast<uint16_t>(p);
            }
        }
        __syncthreads();

        auto fetch = [&](int32_t start) {
            LanePiece piece;
#pragma unroll
            for (int s = 0; s < kSubBatches; ++s) {
                const int32_t mine = start + s * kSubSpan + lane * kSubEntries;
                piece.live[s] = mine < d1;
                const int32_t i0 = piece.live[s] ? mine : d1 - kSubEntries;
                const int32_t g = (i0 - d0) / kWave;
                int p = g < groups ? static_cast<int>(groupChunk[g]) : ChunkOf(tabD, P, i0);
                p += (p + 1 < P && tabD[p + 1] <= i0) ? 1 : 0;
                p += (p + 1 < P && tabD[p + 1] <= i0) ? 1 : 0;
                if (__any(p + 1 < P && tabD[p + 1] <= i0)) {
                    p = ChunkOf(tabD, P, i0);
                }
                if (Live) {
                    piece.a[s] = *reinterpret_cast<const Float4U1 *>(win + (i0 - d0));
                } else {
                    piece.a[s] = __builtin_nontemporal_load(reinterpret_cast<const Float4U1 *>(valD + i0));
                }
                piece.rows[s] = __builtin_nontemporal_load(reinterpret_cast<const Uint2 *>(rowLocal + i0));
                piece.x[s] = *reinterpret_cast<const Float4U1 *>(xg + (i0 + tabDelta[p]));
            }
            return piece;
        };

        int32_t start = d0 + wave * kBatch;
        if (start < d1) {
            LanePiece cur = fetch(start);
            while (true) {
                const LanePiece next = fetch(start + kStride);  // past the end: every lane re-reads the last run
#pragma unroll
                for (int s = 0; s < kSubBatches; ++s) {
                    const float av[kSubEntries] = {cur.a[s].x, cur.a[s].y, cur.a[s].z, cur.a[s].w};
                    const float xv[kSubEntries] = {cur.x[s].x, cur.x[s].y, cur.x[s].z, cur.x[s].w};
                    const uint32_t rws[2] = {cur.rows[s].x, cur.rows[s].y};
                    int32_t key[kSubEntries];
                    double t[kSubEntries];
                    bool same = true;
#pragma unroll
                    for (int j = 0; j < kSubEntries; ++j) {
                        const uint32_t k = (j & 1) ? rws[j / 2] >> 16 : rws[j / 2] & 0xffffu;
                        // padding and runs past the end carry key -1 and add nothing
                        key[j] = (cur.live[s] && k < kPadRow) ? static_cast<int32_t>(k & (kRowBlockRows - 1)) : -1;
                        t[j] = static_cast<double>(av[j]) * static_cast<double>(xv[j]);
                        same = same && key[j] == key[0];
                    }
                    const int32_t first = __builtin_amdgcn_readfirstlane(key[0]);
                    if (first >= 0 && __all(same && key[0] == first)) {
                        // one row fills the wavefront's 256 positions
                        if (first != pendingKey) {
                            FlushPending(acc, pendingKey, pending);
                            pendingKey = first;
                            pending = 0.0;
                        }
                        pending += (t[0] + t[1]) + (t[2] + t[3]);
                    } else {
                        double run = t[0];
#pragma unroll
                        for (int j = 1; j < kSubEntries; ++j) {
                            if (key[j] != key[j - 1]) {
                                if (key[j - 1] >= 0) {
                                    atomicAdd(&acc[key[j - 1]], run);
                                }
                                run = 0.0;
                            }
                            run += t[j];
                        }
                        if (key[kSubEntries - 1] >= 0) {
                            atomicAdd(&acc[key[kSubEntries - 1]], run);
                        }
                    }
                }
                start += kStride;
                if (start >= d1) {
                    break;
                }
                cur = next;
            }
        }
    }
    FlushPending(acc, pendingKey, pending);
    __syncthreads();
    const double alpha = ReadScalar<double>(alphaS), beta = ReadScalar<double>(betaS);
    for (int i = tid; i < row1 - row0; i += kRedThreads) {
        const int64_t row = row0 + i;
        if (deferLong && __double_as_longlong(acc[i]) == kDeferredRowMark) {
            continue;  // SpmvLongRowSumKernel's
        }
        double o = alpha * acc[i];
        if (beta != 0.0) {
            o += beta * ToAcc<double>(yIn[row]);
        }
        y[row] = FromAcc<OutT>(o);
    }
}

// The long rows of the row blocks that hold more than kInBlockLongRows of them (longDeferred[l] != 0), a wavefront a
// row: y[row] = alpha * (the row's partial sums, added up as phase 2 does) + beta * yIn[row].
template <typename OutT>
__global__ __launch_bounds__(kBlockThreads) void SpmvLongRowSumKernel(
    const int32_t *__restrict__ header, const int32_t *__restrict__ longRows, const int32_t *__restrict__ longDeferred,
    const double *__restrict__ longPartial, int32_t P, OutT *__restrict__ y, const OutT *__restrict__ yIn,
    OpsparseScalar alphaS, OpsparseScalar betaS)
{
    const int lane = threadIdx.x % kWave;
    const int32_t l = static_cast<int32_t>(blockIdx.x) * (kBlockThreads / kWave) + threadIdx.x / kWave;
    if (l >= header[1] || longDeferred[l] == 0) {
        return;
    }
    double sum = 0.0;
    const double *from = longPartial + static_cast<int64_t>(l) * P;
    for (int32_t p0 = 0; p0 < P; p0 += 4 * kWave) {
        double v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int32_t p = p0 + u * kWave + lane;
            v[u] = from[p < P ? p : P - 1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            sum += p0 + u * kWave + lane < P ? v[u] : 0.0;
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        sum += __shfl_xor(sum, off);
    }
    if (lane == 0) {
        const int64_t row = longRows[l];
        const double alpha = ReadScalar<double>(alphaS), beta = ReadScalar<double>(betaS);
        double o = alpha * sum;
        if (beta != 0.0) {
            o += beta * ToAcc<double>(yIn[row]);
        }
        y[row] = FromAcc<OutT>(o);
    }
}

// ------------------------------------------------------------------- host

namespace {

struct BlockedLayout {
    int32_t P, B, window, passes;
    int32_t rowLog;  // a row block has at most 2^rowLog rows
    int64_t padded;  // upper bound of the positions in block order
    // used by every launch (the first `resident` bytes)
    int64_t colLocalOff, xgOff, valOff, rowLocalOff, srcStartOff, dstStartOff, srcStartTOff, orderOff, blockRowOff;
    int64_t dstOfPosOff;  // live values only: block-order position of every entry of the caller's arrays
    int64_t blockEntryOff;  // live values only: first entry of every row block in the caller's arrays
    int64_t longSpanOff;    // live values only: first and end entry of every long row
    // long rows (op(A) = A): row ids, first entry of every (long row, panel) piece, fp64 sum of every piece
    int32_t longMinRow;   // rows of at least this many entries are candidates (0: no long-row path)
    int32_t maxLong;      // room for this many
    int64_t longRowsOff, longChunkOff, longPartialOff, longFirstOff, longDeferredOff;
    int64_t resident;
    // preprocessing only
    int64_t keys0Off, keys1Off, pos0Off, pos1Off, rowOfPosOff, outPtrOff, longBeforeOff, shortOffsetsOff, longCsrOff, tableOff,
        scratchOff;
    int64_t bytes;
};

// Layout for a product with `rows` outputs and `cols` inputs (op(A) = A^T: the columns of A are the outputs).
// 0 panels: the layout does not apply.
BlockedLayout MakeBlockedLayout(int64_t rows, int64_t cols, int64_t nnz)
{
    // This file's layout is the one with live values for op(A) = A; the arms below that ask are those of the
    // ordered layout it grew out of (spmv_blocked.hip), which the compiler drops here.
    constexpr bool transposed = false, live = true;
    BlockedLayout l{};
    if (rows <= 0 || cols <= 0 || nnz <= 0 || nnz > INT32_MAX || rows >= INT32_MAX || cols > INT32_MAX) {
        return l;
    }
    const int64_t P = (cols + kPanelCols - 1) >> kPanelLog;
    // Entry window: blocks of short rows get about nnz / (full row blocks) entries; a matrix of few, long rows is
    // still cut into kMinEntryBlocks pieces, or phase 2 would run on a handful of workgroups.
    const int rowLog = live ? kLiveRowBlockLog : kRowBlockLog;
    const int64_t fullBlocks = rows >> rowLog;
    static const int64_t minBlocks = [] {  // tuning override: entry windows a matrix is cut into at least
        const char *env = std::getenv("OPS_SPARSE_BLOCKED_WINDOWS");
        const int64_t v = env != nullptr ? std::atoll(env) : 0;
        return v;
    }();
    // With live values a block should fit one window of kRefreshSpan positions, padding included, or its entries
    // in the caller's arrays are read once per window at every call: blocks of about kLiveWindow entries.
    const int64_t liveBlocks = nnz / kLiveWindow > 6 * kMinEntryBlocks ? nnz / kLiveWindow : 6 * kMinEntryBlocks;
    const int64_t wantBlocks = minBlocks > 0 ? minBlocks : (live ? liveBlocks : kMinEntryBlocks);
    int64_t window = nnz / (fullBlocks > wantBlocks ? fullBlocks : wantBlocks);
    window = window < kMinEntryWindow ? kMinEntryWindow : window;
    const int64_t B = ((rows + (int64_t{1} << rowLog) - 1) >> rowLog) + nnz / window + 1;
    // x must be wide enough for scattered gathers to be what the row-wise kernels wait for, and the chunks long
    // enough to stream.
    // Positions are 32-bit, and phase 2 looks two batches past a block's end before it clamps.
    static const int64_t minCols = [] {  // tuning override
        const char *env = std::getenv("OPS_SPARSE_BLOCKED_MIN_COLS");
        return env != nullptr ? std::atoll(env) : kMinCols;
    }();
    if (cols <= minCols || nnz < kMinEntries || P > kMaxPanels ||
        P * B + 1 > INT32_MAX || nnz + kLaneEntries * P * B > INT32_MAX - 65536 ||
        nnz / (P * B) < (live ? kMinChunkEntriesLive : kMinChunkEntries)) {
        return l;
    }
    l.P = static_cast<int32_t>(P);
    l.B = static_cast<int32_t>(B);
    l.rowLog = rowLog;
    l.window = static_cast<int32_t>(window);
    int bits = 0;
    while ((int64_t{1} << bits) < P) {
        ++bits;
    }
    l.passes = (bits + 3) / 4;
    const bool noLong = std::getenv("OPS_SPARSE_BLOCKED_NO_LONG_ROWS") != nullptr;
    if (!transposed && !noLong) {
        static const int64_t chunkMean = [] {  // tuning override: entries a long row has per panel at least, on average
            const char *env = std::getenv("OPS_SPARSE_BLOCKED_LONG_MEAN");
            const int64_t v = env != nullptr ? std::atoll(env) : 0;
            return v;
        }();
        // live values: the pieces are read where the caller has them, scattered over the arrays, and pay from 64
        // entries (256 bytes of either array); frozen: they are stored again panel by panel and stream
        const int64_t mean = chunkMean > 0 ? chunkMean : (live ? kLongChunkMean : kLongChunkMeanFrozen);
        const int64_t floor = live ? kLongMinRow : kLongMinRowFrozen;
        int64_t minRow = mean * P > floor ? mean * P : floor;
        if (!live && nnz / minRow > 65535) {
            minRow = nnz / 65535 + 1;  // frozen values keep a long row's number, below nnz / minRow, in 16 bits
        }
        if (minRow <= INT32_MAX && nnz / minRow > 0) {
            l.longMinRow = static_cast<int32_t>(minRow);
            l.maxLong = static_cast<int32_t>(nnz / minRow);
            bits = 0;  // their entries sort as one more panel behind the others, or (frozen values) as P more
            while ((int64_t{1} << bits) < (live ? P + 1 : 2 * P)) {
                ++bits;
            }
            l.passes = (bits + 3) / 4;
        }
    }
    if (transposed) {
        // CSR order is ascending in the input index but not in the output block: sort on the whole chunk key
        bits = 0;
        while ((int64_t{1} << bits) < P * B) {
            ++bits;
        }
        l.passes = (bits + 3) / 4;
    }
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    int64_t off = 256;  // header: status word of the analysis
    const int64_t padded = nnz + kLaneEntries * P * B;  // every chunk padded to a multiple of kLaneEntries
    l.padded = padded;
    l.colLocalOff = off; off += align(2 * nnz + 8);
    l.xgOff = off; off += align(4 * nnz) + 256;  // a lane's 16-byte loads of xg may run 7 entries past a chunk
    l.valOff = off; off += live ? 0 : align(4 * padded);  // (live values: none are kept)
    l.rowLocalOff = off; off += align(2 * padded);
    l.srcStartOff = off; off += align(4 * (P * B + 1));
    l.dstStartOff = off; off += align(4 * (P * B + 1));
    l.srcStartTOff = off; off += align(4 * P * B);
    l.orderOff = off; off += align(4 * B);
    l.blockRowOff = off; off += align(4 * (B + 1));
    l.dstOfPosOff = off; off += live ? align(4 * nnz) : 0;
    l.blockEntryOff = off; off += live ? align(4 * (B + 1)) : 0;
    l.longSpanOff = off; off += live ? align(8 * static_cast<int64_t>(l.maxLong)) : 0;
    l.longRowsOff = off; off += align(4 * static_cast<int64_t>(l.maxLong));
    // live: first entry of piece (p, l) in the CSR arrays at [p * maxLong + l], p = 0 .. P; frozen: in the sorted
    // order at [p * (maxLong + 1) + l], l = 0 .. L
    l.longChunkOff = off; off += align(4 * (static_cast<int64_t>(l.maxLong) + 1) * (P + 1));
    l.longPartialOff = off; off += align(8 * static_cast<int64_t>(l.maxLong) * P);
    l.longFirstOff = off; off += l.maxLong > 0 ? align(4 * (B + 1)) : 0;
    l.longDeferredOff = off; off += align(4 * static_cast<int64_t>(l.maxLong));
    l.resident = off;
    l.keys0Off = off; off += align(4 * nnz);
    l.keys1Off = off; off += align(4 * nnz);
    l.pos0Off = off; off += align(4 * nnz);
    l.pos1Off = off; off += align(4 * nnz);
    l.rowOfPosOff = off; off += align(4 * nnz);
    l.outPtrOff = off; off += transposed ? align(4 * (rows + 1)) : 0;  // entries per output (column of A), prefix-summed
    l.longBeforeOff = off; off += l.maxLong > 0 ? align(4 * rows) : 0;  // long rows among rows 0 .. r
    l.shortOffsetsOff = off; off += l.maxLong > 0 ? align(4 * (rows + 1)) : 0;  // row offsets without their entries
    l.longCsrOff = off; off += l.maxLong > 0 && !live ? align(4 * static_cast<int64_t>(l.maxLong) * (P + 1)) : 0;
    l.tableOff = off; off += align(4 * RadixTableInts(nnz));
    int64_t scan = ScanScratchInts(RadixTableInts(nnz));
    scan = ScanScratchInts(P * B + 1) > scan ? ScanScratchInts(P * B + 1) : scan;
    scan = transposed && ScanScratchInts(rows + 1) > scan ? ScanScratchInts(rows + 1) : scan;
    scan = l.maxLong > 0 && ScanScratchInts(rows + 1) > scan ? ScanScratchInts(rows + 1) : scan;
    l.scratchOff = off; off += align(4 * scan);
    l.bytes = off;
    return l;
}

// Frozen values: the number of its long row, for a long entry at position i of the sorted order, is kept at
// rowLocal[i + LongRowOfShift]: the block order, which that array serves, ends in front of it (it holds the short
// entries and at most 8 positions of padding for each of the P x B chunks).
int64_t LongRowOfShift(const BlockedLayout &l) { return static_cast<int64_t>(kLaneEntries) * l.P * l.B; }

uint32_t GridOf(int64_t items, int64_t perBlock, int64_t cap)
{
    int64_t g = (items + perBlock - 1) / perBlock;
    g = g < 1 ? 1 : g;
    return static_cast<uint32_t>(g > cap ? cap : g);
}

}  // namespace

// valType: the type of the caller's values and of x (OPSPARSE_F32 / F16 / BF16); y is fp32.  Frozen fp16 and bf16
// values sit in the layout as fp32, live ones are widened where they are read, and phase 1 widens x as it loads
// the slice.
int LaunchBlocked(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType)
{
    if (plan.valueType != valType) {
        return OPSPARSE_E_INVALID;  // the plan was made for values of another type
    }
    if (outType != OPSPARSE_F32 && outType != valType) {
        return OPSPARSE_E_UNSUPPORTED;  // y is fp32, or of the 16-bit type of the values
    }
    // a.rows outputs, a.cols inputs: the caller has exchanged them for op(A) = A^T
    const BlockedLayout l = MakeBlockedLayout(a.rows, a.cols, a.nnz);
    if (l.P == 0 || plan.numPanels != l.P || plan.numRowBlocks != l.B) {
        return OPSPARSE_E_INVALID;
    }
    // a launch touches the first `resident` bytes only: the tail served the analysis and may have been handed back
    if (a.ws == nullptr || static_cast<int64_t>(a.wsBytes) < l.resident || plan.bytes != l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto *base = static_cast<unsigned char *>(a.ws);
    auto ints = [&](int64_t off) { return reinterpret_cast<const int32_t *>(base + off); };
    const auto *colLocal = reinterpret_cast<const uint16_t *>(base + l.colLocalOff);
    const auto *rowLocal = reinterpret_cast<const uint16_t *>(base + l.rowLocalOff);
    auto *xg = reinterpret_cast<float *>(base + l.xgOff);
    if (plan.liveValues == 0 || plan.transposed != 0 || a.vals == nullptr) {
        return OPSPARSE_E_INVALID;  // (this layout is the one with live values, for op(A) = A)
    }
    // Few panels: several workgroups per panel, so that every CU has one.
    const int32_t splits = l.P >= 192 ? 1 : (256 + l.P - 1) / l.P;
    // long rows: summed from the caller's own arrays (header[1] of them, counted by the analysis)
    const bool longRows = plan.numLongRows > 0;
    if (longRows && plan.liveValues != 0 && (a.vals == nullptr || a.colInd == nullptr)) {
        return OPSPARSE_E_INVALID;
    }
    const int32_t *header = longRows ? ints(0) : nullptr;
    auto *longPartial = reinterpret_cast<double *>(base + l.longPartialOff);
    auto gather = [&](auto xTag) {
        using XT = decltype(xTag);
        hipLaunchKernelGGL(SpmvBlockGatherKernel<XT>, dim3(static_cast<uint32_t>(l.P) * splits), dim3(kBlkThreads), 0,
                           a.stream, colLocal, static_cast<const XT *>(a.x), xg, ints(l.srcStartOff), a.cols, l.B, splits,
                           header, ints(l.longChunkOff), a.colInd, static_cast<const XT *>(a.vals), a.nnz, l.P, l.maxLong,
                           static_cast<const uint16_t *>(nullptr), longPartial);
    };
    if (valType == OPSPARSE_F16) {
        gather(Half{});
    } else if (valType == OPSPARSE_BF16) {
        gather(Bf16{});
    } else {
        gather(float{});
    }
    // phase 2 (and the sums of deferred long rows) for the types of the values and of y
    auto reduce = [&](auto valTag, auto outTag) {
        using ValT = decltype(valTag);
        using OutT = decltype(outTag);
        auto live = [&](auto shortTag) {
            constexpr bool kShort = decltype(shortTag)::value;
            hipLaunchKernelGGL((SpmvBlockReduceKernel<true, kShort, ValT, OutT>), dim3(static_cast<uint32_t>(l.B)),
                               dim3(kRedThreads), 0, a.stream, static_cast<const float *>(nullptr), xg, rowLocal,
                               ints(l.dstStartOff), ints(l.srcStartTOff), l.P, ints(l.orderOff), ints(l.blockRowOff),
                               static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.alpha, a.beta,
                               longRows ? ints(l.longFirstOff) : nullptr, ints(l.longRowsOff), longPartial,
                               static_cast<const ValT *>(a.vals), ints(l.dstOfPosOff), ints(l.blockEntryOff),
                               ints(l.longSpanOff));
        };
        if (plan.liveValues == kLiveShortPositions) {
            live(std::true_type{});
        } else {
            live(std::false_type{});
        }
        if (longRows && plan.numDeferredLongRows > 0) {
            constexpr int kRowsPerBlock = kBlockThreads / kWave;
            hipLaunchKernelGGL(SpmvLongRowSumKernel<OutT>, dim3((plan.numLongRows + kRowsPerBlock - 1) / kRowsPerBlock),
                               dim3(kBlockThreads), 0, a.stream, header, ints(l.longRowsOff), ints(l.longDeferredOff),
                               longPartial, l.P, static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.alpha,
                               a.beta);
        }
    };
    if (valType == OPSPARSE_F16) {
        if (outType == OPSPARSE_F16) {
            reduce(Half{}, Half{});
        } else {
            reduce(Half{}, float{});
        }
    } else if (valType == OPSPARSE_BF16) {
        if (outType == OPSPARSE_BF16) {
            reduce(Bf16{}, Bf16{});
        } else {
            reduce(Bf16{}, float{});
        }
    } else {
        reduce(float{}, float{});
    }
    return CheckLaunch();
}

}  // namespace live_layout
}  // namespace opsparse

using namespace opsparse;
using namespace opsparse::live_layout;

extern "C" {

size_t opsparse_spmv_csr_live_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz)
{
    return static_cast<size_t>(MakeBlockedLayout(rows, cols, nnz).bytes);
}

size_t opsparse_spmv_csr_live_resident_bytes(int64_t rows, int64_t cols, int64_t nnz)
{
    return static_cast<size_t>(MakeBlockedLayout(rows, cols, nnz).resident);
}

int opsparse_spmv_csr_live_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                      int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                      size_t workspaceBytes, void *scratchSpace, size_t scratchBytes,
                                      OpsparseSpmvPlan *plan, void *stream)
{
    if (plan == nullptr || rowOffsets == nullptr || colInd == nullptr || csrValues == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    if ((flags & (OPSPARSE_BLOCKED_TRANSPOSE | OPSPARSE_BLOCKED_VALUES_I32)) != 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    constexpr bool transposed = false, live = true;
    const int32_t valueType = (flags & OPSPARSE_BLOCKED_VALUES_F16) != 0    ? OPSPARSE_F16
                              : (flags & OPSPARSE_BLOCKED_VALUES_BF16) != 0 ? OPSPARSE_BF16
                                                                            : OPSPARSE_F32;
    const int64_t outputs = transposed ? cols : rows;
    const BlockedLayout l = MakeBlockedLayout(rows, cols, nnz);
    if (l.P == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    // what the launches keep goes into `workspace`, what only the analysis needs into `scratchSpace`
    if (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < l.resident || scratchSpace == nullptr ||
        static_cast<int64_t>(scratchBytes) < l.bytes - l.resident) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto *residentBase = static_cast<unsigned char *>(workspace);
    auto *scratchBase = static_cast<unsigned char *>(scratchSpace);
    const int64_t residentEnd = l.resident;
    auto at = [&](int64_t off) { return off < residentEnd ? residentBase + off : scratchBase + (off - residentEnd); };
    auto ints = [&](int64_t off) { return reinterpret_cast<int32_t *>(at(off)); };
    int32_t *status = ints(0);
    int32_t *keys[2] = {ints(l.keys0Off), ints(l.keys1Off)};
    int32_t *poss[2] = {ints(l.pos0Off), ints(l.pos1Off)};
    int32_t *rowOfPos = ints(l.rowOfPosOff), *table = ints(l.tableOff), *scratch = ints(l.scratchOff);
    int32_t *srcStart = ints(l.srcStartOff), *dstStart = ints(l.dstStartOff), *srcStartT = ints(l.srcStartTOff);
    int32_t *blockRow = ints(l.blockRowOff);
    auto *colLocal = reinterpret_cast<uint16_t *>(at(l.colLocalOff));
    auto *rowLocal = reinterpret_cast<uint16_t *>(at(l.rowLocalOff));
    auto *valD = reinterpret_cast<float *>(at(l.valOff));

    // status, number of long rows, their entries, positions of the longest block, long rows summed on their own
    LaunchFillI32(status, 5, 0, s);
    LaunchExpandRows(rowOffsets, rows, nnz, 0, rowOfPos, s);
    const int32_t *pos = nullptr, *outOffsets = rowOffsets;
    int32_t *chunkKey = nullptr, *rowOfSrc = nullptr;
    int32_t *longBefore = nullptr;
    if (l.maxLong > 0) {
        // Long rows: candidates by length, checked for ascending columns inside [0, cols), numbered, listed.
        longBefore = ints(l.longBeforeOff);
        hipLaunchKernelGGL(LongRowFlagsKernel, dim3(GridOf(rows, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, rows, l.longMinRow, longBefore);
        hipLaunchKernelGGL(LongRowCheckKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                           rowOffsets, colInd, rowOfPos, nnz, cols, longBefore);
        LaunchInclusiveScanI32(longBefore, longBefore, rows, 0, scratch, s);
        hipLaunchKernelGGL(LongRowListKernel, dim3(GridOf(rows, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, longBefore, rows, l.maxLong, ints(l.longRowsOff), status);
        hipLaunchKernelGGL(LongRowChunksKernel, dim3(GridOf(static_cast<int64_t>(l.maxLong) * (l.P + 1), kBlockThreads, 4096)),
                           dim3(kBlockThreads), 0, s, rowOffsets, colInd, ints(l.longRowsOff), status, l.P, l.maxLong,
                           ints(live ? l.longChunkOff : l.longCsrOff));
        int32_t *shortOffsets = ints(l.shortOffsetsOff);
        hipLaunchKernelGGL(LongRowEntriesKernel, dim3(GridOf(rows, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, longBefore, rows, shortOffsets);
        LaunchInclusiveScanI32(shortOffsets, shortOffsets, rows + 1, 0, scratch, s);
        hipLaunchKernelGGL(ShortOffsetsKernel, dim3(GridOf(rows + 1, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, rows, shortOffsets);
        outOffsets = shortOffsets;  // the row blocks are cut by the entries that stay
    }
    {
        // Entries in (panel, original position) order: stable 4-bit radix passes over the panel number.
        const int32_t *firstKeys = colInd;
        if (longBefore != nullptr) {
            hipLaunchKernelGGL(LongRowKeysKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                               colInd, rowOfPos, longBefore, nnz, static_cast<int32_t>(l.P) << kPanelLog, live ? 0 : 1,
                               keys[1]);
            firstKeys = keys[1];
        }
        int cur = 0;
        for (int32_t pass = 0; pass < l.passes; ++pass) {
            const int32_t *keysIn = pass == 0 ? firstKeys : keys[cur];
            const int32_t *posIn = pass == 0 ? nullptr : poss[cur];
            const int out = pass == 0 ? 0 : 1 - cur;
            LaunchRadixPass(keysIn, posIn, keys[out], poss[out], nnz, 0, kPanelLog + 4 * pass, table, scratch, s);
            cur = out;
        }
        pos = poss[cur];
        chunkKey = keys[1 - cur];
        rowOfSrc = poss[1 - cur];
        hipLaunchKernelGGL(BlockedChunkKeysKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                           keys[cur], pos, rowOfPos, outOffsets, nnz, cols, l.B, l.rowLog, l.window, longBefore, colLocal, chunkKey,
                           rowOfSrc, status);
    }
    int32_t head[3] = {0, 0, 0};  // status, long rows, their entries
    if (hipMemcpyAsync(head, status, sizeof(head), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    const int32_t bad = head[0];
    if (bad != 0) {
        return OPSPARSE_E_INVALID;  // a column index outside [0, cols)
    }
    const int64_t chunks = static_cast<int64_t>(l.P) * l.B;
    LaunchIndicesToOffsets(chunkKey, nnz, chunks, 0, srcStart, scratch, s);
    hipLaunchKernelGGL(BlockedTablesKernel, dim3(GridOf(chunks, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                       srcStart, l.P, l.B, dstStart, srcStartT);
    LaunchInclusiveScanI32(dstStart + 1, dstStart + 1, chunks, 0, scratch, s);
    // padding positions: local row kPadRow, value 0
    LaunchFillI32(reinterpret_cast<int32_t *>(rowLocal), (l.padded + 1) / 2, static_cast<int32_t>(kPadRow * 0x10001u), s);
    if (!live) {
        LaunchFillI32(reinterpret_cast<int32_t *>(valD), l.padded, 0, s);
    } else {
        LaunchFillI32(ints(l.dstOfPosOff), nnz, -1, s);  // entries of long rows have no place in block order
    }
    LaunchFillI32(blockRow, l.B + 1, static_cast<int32_t>(outputs), s);
    hipLaunchKernelGGL(BlockedRowBlocksKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                       s, outOffsets, static_cast<int32_t>(outputs), l.rowLog, l.window, l.B, blockRow);
    if (longBefore != nullptr) {
        hipLaunchKernelGGL(BlockedLongFirstKernel, dim3(GridOf(l.B + 1, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                           s, blockRow, longBefore, l.B, ints(l.longFirstOff));
        hipLaunchKernelGGL(BlockedLongDeferKernel, dim3(GridOf(l.B, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           ints(l.longFirstOff), l.B, ints(l.longDeferredOff), status);
    }
    auto scatter = [&](auto tag) {
        using ValT = decltype(tag);
        hipLaunchKernelGGL(BlockedScatterKernel<ValT>, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                           pos, rowOfSrc, chunkKey, static_cast<const ValT *>(csrValues), srcStart, dstStart, blockRow, nnz,
                           l.P, l.B, live ? nullptr : valD, rowLocal, live ? ints(l.dstOfPosOff) : nullptr,
                           longBefore != nullptr && !live ? reinterpret_cast<float *>(at(l.xgOff)) : nullptr,
                           rowLocal + LongRowOfShift(l), longBefore);
    };
    if (valueType == OPSPARSE_F16) {
        scatter(Half{});
    } else if (valueType == OPSPARSE_BF16) {
        scatter(Bf16{});
    } else {
        scatter(float{});
    }
    // (the blocks are alike in size by construction and are taken in row order)
    if (live) {
        const int64_t items = l.B + 1 > l.maxLong ? l.B + 1 : l.maxLong;
        hipLaunchKernelGGL(BlockedLiveTablesKernel, dim3(GridOf(items, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                           s, rowOffsets, blockRow, l.B, ints(l.longRowsOff), longBefore != nullptr ? status : nullptr,
                           ints(l.blockEntryOff), ints(l.longSpanOff));
    }
    int32_t liveKind = live ? 1 : 0;
    int32_t tail[2] = {0, 0};  // positions of the longest row block, long rows that are summed on their own
    if (live) {
        hipLaunchKernelGGL(BlockedMaxPositionsKernel, dim3(GridOf(l.B, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                           s, dstStart, l.P, l.B, status);
    }
    if (live || longBefore != nullptr) {
        if (hipMemcpyAsync(tail, status + 3, sizeof(tail), hipMemcpyDeviceToHost, s) != hipSuccess ||
            hipStreamSynchronize(s) != hipSuccess) {
            (void)hipGetLastError();
            return OPSPARSE_E_LAUNCH;
        }
    }
    if (live) {
        // Row blocks of fewer than 65535 positions, all of them (the rule unless a row that cannot go the long rows'
        // way is longer than that): 16-bit positions relative to the block, 2 bytes an entry less at every call.
        const int32_t longest = tail[0];
        // (tuning / test switch, read at every analysis)
        const bool noShort = std::getenv("OPS_SPARSE_BLOCKED_NO_SHORT_POSITIONS") != nullptr;
        if (!noShort && longest < static_cast<int32_t>(kNoPosition16)) {
            hipLaunchKernelGGL(BlockedShortPositionsKernel, dim3(static_cast<uint32_t>(l.B)), dim3(kBlkThreads), 0, s,
                               ints(l.blockEntryOff), dstStart, l.P, ints(l.dstOfPosOff));
            liveKind = kLiveShortPositions;
        }
    }
    if (CheckLaunch() != OPSPARSE_OK) {
        return OPSPARSE_E_LAUNCH;
    }
    OpsparseSpmvPlan p{};
    p.kernel = OPSPARSE_SPMV_BLOCKED_LIVE;
    p.numPanels = l.P;
    p.panelShift = kPanelLog;
    p.numRowBlocks = l.B;
    p.entryWindow = l.window;
    p.transposed = transposed ? 1 : 0;
    p.liveValues = liveKind;
    p.valueType = valueType;
    p.numDeferredLongRows = tail[1];
    p.numLongRows = head[1];
    p.rows = rows;
    p.nnz = nnz;
    p.bytes = l.bytes;
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmv_csr_live_analyse(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                      int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                      size_t workspaceBytes, OpsparseSpmvPlan *plan, void *stream)
{
    // one piece: the analysis' scratch follows what the launches keep
    const size_t resident = opsparse_spmv_csr_live_resident_bytes(rows, cols, nnz);
    if (resident == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    if (workspace == nullptr || workspaceBytes < resident) {
        return OPSPARSE_E_WORKSPACE;
    }
    return opsparse_spmv_csr_live_analyse_split(rowOffsets, colInd, csrValues, rows, cols, nnz, flags, workspace, resident,
                                         static_cast<unsigned char *>(workspace) + resident, workspaceBytes - resident, plan, stream);
}

}  // extern "C"
