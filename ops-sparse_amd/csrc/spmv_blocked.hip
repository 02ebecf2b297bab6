// BLOCKED_GATHER: CSR SpMV for a matrix whose x does not fit a cache.
//
// Takes the place of the reference's aclsparseSpMVOp with ALG2 — a device-side
// preprocessing pass that re-orders the rows into the caller's buffer, then a
// thread-per-row kernel (sparse/spmv_op/arch35/spmv_op_host.cpp:543-573 and
// :423-457, spmv_op_kernel.cpp:413-535) — and of aclsparseSpMV's kernel
// (sparse/spmv/arch22/kernels/spmv_kernel.h:27-310) for that case.  A
// row-wise kernel gathers x[col] straight from memory, and with random columns
// every gather moves a whole 128-byte line for 4 useful bytes: the gather
// rate, not the matrix stream, sets the time.  Here x is gathered from LDS
// instead, in two kernels.
//
//   phase 1  the entries' local column indices are stored a second time sorted
//            by column panel (2^15 columns = 128 KiB of x).  A workgroup copies
//            its panel's slice of x into LDS and writes xg[i] = x[col[i]] for
//            the panel's entries: 2 bytes read, 4 bytes written per entry, both
//            as linear streams.
//   phase 2  rows are grouped into row blocks (at most 2^12 rows, cut also
//            wherever the entry count passes a multiple of the entry window).
//            The entries of a block are one contiguous piece of the values in
//            row order, and a workgroup owns one block: it streams the block's
//            xg — in (block, panel) order, one contiguous piece per (panel,
//            block) chunk — together with a 16-bit "slot" per entry, the
//            entry's position in the block's row order, and drops every xg at
//            its slot of a window in LDS.  Then it streams the block's values
//            linearly, multiplies them with the window, and sums the rows with
//            a segmented reduction whose shape depends on the positions of
//            the entries only.
//
// Every entry costs 16 bytes of traffic (2 + 4 in phase 1, 2 + 4 + 4 in phase
// 2) against 8 algorithmic bytes plus a 128-byte line per gather in the
// row-wise kernels.  No value is stored: every call reads the values where
// the caller (or the copy described below) has them.  val * x is exact in
// fp64; the additions of a row are made in an order that the layout fixes —
// inside a lane in stored order, across the lanes of a wavefront by a scan of
// fixed shape, across wavefronts and windows by one thread in ascending order
// — so two calls on the same data give the same bits, and a row is rounded
// once.  Integer data is summed with wrap-around in 32 bits.
//
// Long rows (many entries in every panel, ascending columns) are kept out of
// the row blocks: the phase-1 workgroup of a panel, which has the panel's x in
// LDS anyway, sums val * x over the row's entries of that panel and leaves the
// sum in a table; phase 2 adds a row's sums up in panel order.  8 bytes an
// entry instead of 16.  Read where the caller has them (a row's entries of a
// panel are a contiguous piece of the CSR arrays; rows of 64 entries a panel
// or more), or, when the caller has promised that the values stay as they are
// (frozen values), stored a second time panel by panel as (local column,
// value, number of the row) and streamed flat (rows of 1024 entries and 4 a
// panel or more); the frozen form also keeps a copy of the other values.
//
// op(A) = A^T: the matrix is transposed into the buffer once (the CSC arrays
// of A are the CSR arrays of A^T) and the same two kernels run on that copy;
// with live values a permutation is kept beside it and the values of the copy
// are refreshed from the caller's at every call.
//
// Preprocessing (once per matrix, all on the device): a stable radix sort of
// the entries on the panel number keeps rows, hence row blocks, ascending inside
// a panel, so it yields the (panel, block) order directly; the position of a
// chunk in (block, panel) order follows from the chunk sizes by a prefix sum.
#include <climits>
#include <cstdlib>
#include <type_traits>

#include "convert_internal.h"
#include "device_utils.h"
#include "spmv_internal.h"

namespace opsparse {

constexpr int kBlkThreads = 1024;                 // phase 1: one workgroup per CU, it owns 128 KiB of LDS and more
constexpr int kPanelLog = 15;                     // columns per panel: 128 KiB of 32-bit x
constexpr int kPanelCols = 1 << kPanelLog;
constexpr int kRowBlockLog = 12;                  // rows per row block at most: the rows of its keys sit in LDS, and
                                                  // a sum for each of them in half of a window's memory
constexpr int kRowBlockRows = 1 << kRowBlockLog;
constexpr int kMaxPanels = 1024;
constexpr int kGatherBatch = 8;                   // groups of 4 entries in flight per lane, phase 1
constexpr int kLaneEntries = 8;                   // in block order a chunk is padded to a multiple of this
constexpr uint32_t kPadSlot = 0xffffu;            // slot of a padding position in block order
// Streamed row blocks (values kept or refreshed in block order): a wavefront owns a block, its rows' sums in LDS.
constexpr int kStreamRowLog = 10;                 // rows per block at most: 8 KiB of 64-bit sums a wavefront
constexpr int kStreamRows = 1 << kStreamRowLog;
constexpr int32_t kStreamWindow = 65536;          // a block is also cut wherever the entry count passes a multiple of this
constexpr int32_t kStreamMinWindow = 4096;        // (of this, where the matrix has few rows: MakeBlockedLayout)
constexpr int64_t kStreamBlocksWanted = 8192;
constexpr int64_t kStreamMinChunkEntries = 16;
constexpr int64_t kStreamMaxRowPanelEntries = 16;
constexpr int kStreamThreads = 64;                // a wavefront a workgroup: nothing is shared, nothing waits
constexpr int kTurnThreads = 256;
constexpr uint32_t kStreamPadRow = 0x7ffu;        // row field of a padding position (rows take 10 of its 11 bits)
constexpr int kStreamRoundShift = 11;             // above the row: the turn of the entry among those of its row that
constexpr uint32_t kStreamMaxRound = 31;          // one LDS instruction would add together (31: "31st or later")
constexpr int32_t kMaxBlockEntries = 65534;       // a block's slots are 16 bits
// Phase 2 holds the gathered x of a row block in a window of LDS (kRowsWindow entries: two workgroups then share a
// compute unit).  The blocks are cut at three quarters of that (plus the row in which the cut falls), so that
// nearly all of them fit one window.
constexpr int64_t kMinEntries = 2000000;          // below this the ordinary kernels are as fast or faster
// x of more than 2^18 elements.  An x of 1 - 4 MB fits an L2, but gathers scattered over it still cost the row-wise
// kernels 5.5 us per million (the rate at which an L2 answers them).  Whether the gathers are scattered is for the
// sample of the column indices to say.
constexpr int64_t kMinCols = int64_t{1} << 18;
constexpr int64_t kMinChunkEntries = 8;           // below this mean chunk size the layout does not pay
constexpr int64_t kLongChunkMean = 64;            // a row is "long" with this many entries per panel on average
constexpr int64_t kLongMinRow = 4096;             // and at least this many in all
constexpr int64_t kLongMaxMinRow = 32768;         // (but any row of this many is, or a block's slots would not do)
// (frozen values: the long entries are stored again, a panel's in one piece, and stream whatever the rows' lengths)
constexpr int64_t kLongChunkMeanFrozen = 4;
constexpr int64_t kLongMinRowFrozen = 1024;
constexpr int kLongLanes = 16;        // lanes that sum one (long row, panel) piece in phase 1
constexpr int32_t kInBlockLongRows = 64;          // long rows a row block's own workgroup adds up at most
constexpr int kLongTile = 3072;                   // long rows a phase-1 workgroup has in LDS at a time

typedef float Float4 __attribute__((ext_vector_type(4)));
typedef unsigned short Ushort4 __attribute__((ext_vector_type(4)));
typedef uint32_t Uint4 __attribute__((ext_vector_type(4)));
typedef uint32_t Uint4U __attribute__((ext_vector_type(4), aligned(4)));  // a 16-byte load at any dword
typedef uint32_t Uint2 __attribute__((ext_vector_type(2)));

// ---- data as 32 raw bits -------------------------------------------------------------------------------------
// x, gathered x and stored values travel as 32 raw bits: an fp32 (fp16 and bf16 widened, which is exact) or an int32.

__device__ __forceinline__ uint32_t ToRaw(float v) { return __float_as_uint(v); }
__device__ __forceinline__ uint32_t ToRaw(Half v) { return __float_as_uint(static_cast<float>(v)); }
__device__ __forceinline__ uint32_t ToRaw(Bf16 v) { return static_cast<uint32_t>(v.bits) << 16; }
__device__ __forceinline__ uint32_t ToRaw(int32_t v) { return static_cast<uint32_t>(v); }

// The sums: fp64 for floating-point data and for integers under a floating-point compute type, uint32 (wrap-around)
// for integers under the integer compute type.
template <typename AccT, bool IntData>
__device__ __forceinline__ AccT RawToAcc(uint32_t r)
{
    if constexpr (IntData) {
        if constexpr (std::is_same<AccT, uint32_t>::value) {
            return r;
        } else {
            return static_cast<AccT>(static_cast<int32_t>(r));
        }
    } else {
        return static_cast<AccT>(__uint_as_float(r));
    }
}

__device__ __forceinline__ uint64_t AccToSlot(double v) { return static_cast<uint64_t>(__double_as_longlong(v)); }
__device__ __forceinline__ uint64_t AccToSlot(uint32_t v) { return v; }
template <typename AccT>
__device__ __forceinline__ AccT SlotToAcc(uint64_t s)
{
    if constexpr (std::is_same<AccT, uint32_t>::value) {
        return static_cast<uint32_t>(s);
    } else {
        return __longlong_as_double(static_cast<long long>(s));
    }
}

// Four consecutive values of the caller's array as raw bits, in one load (32-bit types: at any 4-byte-aligned
// address; fp16 / bf16: at any 2-byte-aligned one).
template <typename ValT>
__device__ __forceinline__ Uint4 LoadFourRaw(const ValT *p)
{
    if constexpr (sizeof(ValT) == 4) {
        const Uint4U raw = __builtin_nontemporal_load(reinterpret_cast<const Uint4U *>(p));
        return Uint4{raw.x, raw.y, raw.z, raw.w};
    } else {
        const Short4U raw = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(p));
        ValT four[4];
        __builtin_memcpy(four, &raw, 8);
        return Uint4{ToRaw(four[0]), ToRaw(four[1]), ToRaw(four[2]), ToRaw(four[3])};
    }
}

// y[row] = alpha * sum + beta * yIn[row].
template <typename OutT, typename AccT>
__device__ __forceinline__ void StoreOut(OutT *y, const OutT *yIn, int64_t row, AccT sum, AccT alpha, AccT beta)
{
    if constexpr (std::is_same<AccT, uint32_t>::value) {
        uint32_t o = alpha * sum;
        if (beta != 0u) {
            o += beta * static_cast<uint32_t>(yIn[row]);
        }
        y[row] = static_cast<OutT>(static_cast<int32_t>(o));
    } else {
        double o = alpha * sum;
        if (beta != 0.0) {
            o += beta * ToAcc<double>(yIn[row]);
        }
        y[row] = FromAcc<OutT>(o);
    }
}

template <typename AccT>
__device__ __forceinline__ AccT ReadAcc(const OpsparseScalar &s)
{
    if constexpr (std::is_same<AccT, uint32_t>::value) {
        return static_cast<uint32_t>(ReadScalar<int32_t>(s));
    } else {
        return ReadScalar<double>(s);
    }
}

// ---- sums of a key-sorted stream -------------------------------------------------------------------------------
// A wavefront walks a stream of products whose keys (rows) come in runs, 4 consecutive entries a lane and 256 a
// round, and leaves the sum of every run that ends inside its stretch with `store`.  What it holds of the run that
// is still open is the carry (key and sum, the same in every lane).  The additions of a run are made in an order
// that depends on where its entries sit in the rounds only: inside a lane in stream order, then across the lanes by
// a segmented scan of fixed shape, then the carry in front.
constexpr int kSegEntries = 4;
constexpr int kRound = kWave * kSegEntries;
constexpr int32_t kNoKey = INT32_MAX;  // an entry outside the stream; `store` is not called for it

// Lane-to-lane moves inside the vector ALU (data-parallel primitives): the lanes that the control word gives no
// source, and the rows that the row mask leaves out, receive `old`.
constexpr int kDppRowShr1 = 0x111, kDppRowShr2 = 0x112, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;
constexpr int kDppWaveShr1 = 0x138;    // every lane from the lane before it; lane 0 has no source
constexpr int kDppRowBcast15 = 0x142;  // lane 15 of every row of 16 lanes to all lanes of the next row
constexpr int kDppRowBcast31 = 0x143;  // lane 31 to all lanes of rows 2 and 3

template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t DppMove(uint32_t old, uint32_t src)
{
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(old), static_cast<int>(src), kCtrl,
                                                             kRowMask, 0xf, false));
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ double DppMove(double old, double src)
{
    const uint32_t lo = DppMove<kCtrl, kRowMask>(static_cast<uint32_t>(__double2loint(old)),
                                                 static_cast<uint32_t>(__double2loint(src)));
    const uint32_t hi = DppMove<kCtrl, kRowMask>(static_cast<uint32_t>(__double2hiint(old)),
                                                 static_cast<uint32_t>(__double2hiint(src)));
    return __hiloint2double(static_cast<int>(hi), static_cast<int>(lo));
}
__device__ __forceinline__ uint32_t ReadLane63(uint32_t v)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), kWave - 1));
}
__device__ __forceinline__ double ReadLane63(double v)
{
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), kWave - 1),
                            __builtin_amdgcn_readlane(__double2loint(v), kWave - 1));
}

// One step of the segmented scan: v and `fresh` of the lanes that the move reaches take the lane's at the given
// distance in front of them in.
template <int kCtrl, int kRowMask, typename AccT>
__device__ __forceinline__ void SegScanStep(AccT &v, uint32_t &fresh)
{
    const AccT vUp = DppMove<kCtrl, kRowMask>(AccT(0), v);
    const uint32_t fUp = DppMove<kCtrl, kRowMask>(0u, fresh);
    if (fresh == 0) {
        v += vUp;
    }
    fresh |= fUp;
}

// All 64 lanes of the wavefront must be active.
template <typename AccT, typename StoreFn>
__device__ __forceinline__ void SegRound(const int32_t (&k)[kSegEntries], const AccT (&t)[kSegEntries], int lane,
                                         int32_t &carryKey, AccT &carrySum, StoreFn &&store)
{
    AccT headSum = AccT(0), run = t[0];
    int boundaries = 0;
#pragma unroll
    for (int j = 1; j < kSegEntries; ++j) {
        if (k[j] != k[j - 1]) {
            if (boundaries == 0) {
                headSum = run;  // the lane's first run ends here
            } else if (k[j - 1] != kNoKey) {
                store(k[j - 1], run);  // a run that begins and ends inside the lane
            }
            ++boundaries;
            run = AccT(0);
        }
        run += t[j];
    }
    // `run` is the lane's last run; v becomes the sum of that run's row up to the end of this lane
    const int32_t prevKey = static_cast<int32_t>(DppMove<kDppWaveShr1, 0xf>(
        static_cast<uint32_t>(carryKey), static_cast<uint32_t>(k[kSegEntries - 1])));  // lane 0: the carry's
    uint32_t fresh = (boundaries > 0 || prevKey != k[0]) ? 1u : 0u;  // the last run does not go on from the lane before
    AccT v = run;
    if (lane == 0 && fresh == 0) {
        v += carrySum;
    }
    SegScanStep<kDppRowShr1, 0xf>(v, fresh);
    SegScanStep<kDppRowShr2, 0xf>(v, fresh);
    SegScanStep<kDppRowShr4, 0xf>(v, fresh);
    SegScanStep<kDppRowShr8, 0xf>(v, fresh);
    SegScanStep<kDppRowBcast15, 0xa>(v, fresh);
    SegScanStep<kDppRowBcast31, 0xc>(v, fresh);
    const AccT prevSum = DppMove<kDppWaveShr1, 0xf>(carrySum, v);
    if (prevKey != k[0] && prevKey != kNoKey) {
        store(prevKey, prevSum);  // the row of the lane before ended with that lane
    }
    if (boundaries > 0 && k[0] != kNoKey) {
        store(k[0], prevKey == k[0] ? prevSum + headSum : headSum);
    }
    carryKey = static_cast<int32_t>(ReadLane63(static_cast<uint32_t>(k[kSegEntries - 1])));
    carrySum = ReadLane63(v);
}

// What a wavefront leaves of its stretch for the one thread that joins the stretches: the sum of its first run
// (which may go on from the stretch before) and of the run still open at its end.  ends: [2 * wave] head,
// [2 * wave + 1] tail; a key of kNoKey: none.
struct SegEnds {
    int32_t key[2 * (kBlkThreads / kWave)];
    uint64_t sum[2 * (kBlkThreads / kWave)];
};

// The `store` of a wavefront whose first run has the key firstKey.
template <typename AccT, typename OutFn>
__device__ __forceinline__ void SegStore(SegEnds &ends, int wave, int32_t firstKey, int32_t key, AccT sum, OutFn &&out)
{
    if (key == firstKey) {
        ends.sum[2 * wave] = AccToSlot(sum);
    } else {
        out(key, sum);
    }
}

// After its last round, by one lane: headKey / tailKey name the wavefront's first run and the run still open at its
// end (kNoKey: none) to the thread that joins the stretches; `same`: they are one run.
template <typename AccT>
__device__ __forceinline__ void SegLeave(SegEnds &ends, int wave, int32_t headKey, int32_t tailKey, bool same,
                                         AccT carrySum)
{
    ends.key[2 * wave] = headKey;
    if (same) {
        if (headKey != kNoKey) {
            ends.sum[2 * wave] = AccToSlot(carrySum);  // one row all along
        }
        ends.key[2 * wave + 1] = kNoKey;
    } else {
        ends.key[2 * wave + 1] = tailKey;
        ends.sum[2 * wave + 1] = AccToSlot(carrySum);
    }
}

// By one thread, after a barrier: the stretches joined in ascending order.  (pendKey, pendSum) is the run that is
// still open, also across calls; `out` receives the runs that ended.
template <typename AccT, typename OutFn>
__device__ __forceinline__ void SegJoin(const SegEnds &ends, int waves, int32_t &pendKey, AccT &pendSum, OutFn &&out)
{
    for (int w = 0; w < waves; ++w) {
        const int32_t hk = ends.key[2 * w], tk = ends.key[2 * w + 1];
        if (hk != kNoKey) {
            const AccT hs = SlotToAcc<AccT>(ends.sum[2 * w]);
            if (pendKey == hk) {
                pendSum += hs;
            } else {
                if (pendKey != kNoKey) {
                    out(pendKey, pendSum);
                }
                pendKey = hk;
                pendSum = hs;
            }
        }
        if (tk != kNoKey) {
            if (pendKey != kNoKey) {
                out(pendKey, pendSum);
            }
            pendKey = tk;
            pendSum = SlotToAcc<AccT>(ends.sum[2 * w + 1]);
        }
    }
}

// SegJoin by the lanes of one wavefront: lane w fetches what wavefront w left, the joining itself runs on values
// passed from lane to lane in turn (the same order, the same sums); lane 0 writes.  All 64 lanes call it.
template <typename AccT, typename OutFn>
__device__ __forceinline__ void SegJoinWave(const SegEnds &ends, int waves, int lane, int32_t &pendKey, AccT &pendSum,
                                            OutFn &&out)
{
    const int w = lane < waves ? lane : 0;
    const int32_t hkMine = ends.key[2 * w], tkMine = ends.key[2 * w + 1];
    const uint64_t hsMine = ends.sum[2 * w], tsMine = ends.sum[2 * w + 1];
    for (int i = 0; i < waves; ++i) {
        const int32_t hk = __shfl(hkMine, i), tk = __shfl(tkMine, i);
        const uint64_t hs = __shfl(static_cast<unsigned long long>(hsMine), i);
        const uint64_t ts = __shfl(static_cast<unsigned long long>(tsMine), i);
        if (hk != kNoKey) {
            if (pendKey == hk) {
                pendSum += SlotToAcc<AccT>(hs);
            } else {
                if (pendKey != kNoKey && lane == 0) {
                    out(pendKey, pendSum);
                }
                pendKey = hk;
                pendSum = SlotToAcc<AccT>(hs);
            }
        }
        if (tk != kNoKey) {
            if (pendKey != kNoKey && lane == 0) {
                out(pendKey, pendSum);
            }
            pendKey = tk;
            pendSum = SlotToAcc<AccT>(ts);
        }
    }
}

// ---- row blocks ------------------------------------------------------------------------------------------------

constexpr int kRowsWindow = 14336;  // entries of a row block whose gathered x a phase-2 workgroup holds in LDS at a time

// What the workgroup of a row block needs to know before anything else, in one piece.
struct BlockMeta {
    int32_t row0, nRows;   // the block's rows
    int32_t dBeg, dEnd;    // its piece of the block order
    int32_t base;          // first of its entries in the values array
    int32_t short0;        // first of its entries in the offsets
    int32_t l0, l1;        // its long rows
    int32_t bitsOff;       // first word of its row-start bits (and of their prefix counts)
    int32_t ordOff;        // its table of the rows of the keys
    int32_t nEntries;      // its entries (without those of long rows)
    int32_t pad;
};

// Where the tables of row block b start: its row-start bits take (entries + 1) bits, in whole words; the rows of its
// keys at most (rows + 2) entries.  Blocks partition the rows and the entries, so these are disjoint.
__host__ __device__ __forceinline__ int32_t BlockBitsOff(int32_t short0, int32_t b) { return ((short0 >> 5) & ~3) + 8 * b; }
__host__ __device__ __forceinline__ int32_t BlockOrdOff(int32_t row0, int32_t b) { return ((row0 + 7) & ~7) + 16 * b; }

// Row block of a row: blocks of 2^rowLog rows, cut again wherever the row's first entry passes a multiple of the entry
// window (`offsets`: the row offsets without the entries of long rows), and, with `longBefore` (the number of long
// rows among rows 0 .. r), behind every long row.  Monotone in the row number.
__device__ __forceinline__ int32_t RowBlockOf(const int32_t *__restrict__ offsets, int32_t row, int32_t window,
                                              int32_t numBlocks, const int32_t *__restrict__ longBefore, int32_t rowLog)
{
    int32_t b = (row >> rowLog) + offsets[row] / window;
    if (longBefore != nullptr && row > 0) {
        b += longBefore[row - 1];
    }
    return b < 0 ? 0 : (b < numBlocks ? b : numBlocks - 1);  // in range whatever the arrays hold
}

// longBefore[r] = number of long rows among rows 0 .. r (an inclusive prefix sum of the flags).
__device__ __forceinline__ bool IsLongRow(const int32_t *__restrict__ longBefore, int32_t row)
{
    return longBefore[row] != (row > 0 ? longBefore[row - 1] : 0);
}

// ------------------------------------------------------------ preprocessing

// status[0] |= 1 for a column index outside [0, cols).
__global__ __launch_bounds__(kBlockThreads) void CheckColumnsKernel(const int32_t *__restrict__ colInd, int64_t nnz,
                                                                    int64_t cols, int32_t *__restrict__ status)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    bool bad = false;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t c = colInd[i];
        bad = bad || c < 0 || c >= cols;
    }
    if (bad) {
        atomicOr(status, 1);
    }
}

__global__ __launch_bounds__(kBlockThreads) void IotaKernel(int32_t *__restrict__ out, int64_t n)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        out[i] = static_cast<int32_t>(i);
    }
}

// For the entries in (panel, original position) order: local column index, chunk
// key panel * B + block, and the row.  A column outside [0, cols) sets *status.
__global__ __launch_bounds__(kBlockThreads) void BlockedChunkKeysKernel(
    const int32_t *__restrict__ colSorted, const int32_t *__restrict__ pos, const int32_t *__restrict__ rowOfPos,
    const int32_t *__restrict__ offsets, int64_t nnz, int64_t cols, int32_t numBlocks, int32_t window,
    const int32_t *__restrict__ longBefore, int32_t cutBehindLong, int32_t rowLog, uint16_t *__restrict__ colLocal,
    int32_t *__restrict__ chunkKey, int32_t *__restrict__ rowOfSrc, int32_t *__restrict__ status)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t col = colSorted[i];
        const int32_t row = rowOfPos[pos[i]];
        rowOfSrc[i] = row;
        colLocal[i] = static_cast<uint16_t>(col & (kPanelCols - 1));
        if (longBefore != nullptr && IsLongRow(longBefore, row)) {
            chunkKey[i] = -1;  // an entry of a long row (sorted behind every panel): phase 1 sums it
        } else if (col < 0 || col >= cols) {
            atomicOr(status, 1);
            chunkKey[i] = -1;
        } else {
            chunkKey[i] = (col >> kPanelLog) * numBlocks +
                          RowBlockOf(offsets, row, window, numBlocks, cutBehindLong != 0 ? longBefore : nullptr, rowLog);
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

// Row offsets with the entries of the long rows taken out, which is what the row blocks are cut by and what phase
// 2 finds a row's entries by.  First out[r + 1] = entries of row r if it is long (out[0] = 0), then, after an
// inclusive prefix sum, out[r] = rowOffsets[r] - out[r].
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

// Frozen values.  pieceStart[p * (maxLong + 1) + l] = position, in the sorted order, of the first entry of long
// row l in panel p; the entry after the last row of a panel ends it.  First the panels' parts of the sorted order
// (l = 0): a panel's starts where the keys reach longKey + (p << 15), a search by one thread a panel.
__global__ __launch_bounds__(kBlockThreads) void LongRowPanelsKernel(const int32_t *__restrict__ sortedKeys, int64_t nnz,
                                                                     int32_t P, int32_t maxLong, int32_t longKey,
                                                                     int32_t *__restrict__ pieceStart)
{
    const int32_t p = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (p >= P) {
        return;
    }
    // (the order is by the panel field of the keys only: inside a panel the entries keep their CSR order)
    const int32_t want = (longKey >> kPanelLog) + p;
    int64_t lo = 0, hi = nnz;
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if ((sortedKeys[mid] >> kPanelLog) < want) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    pieceStart[static_cast<int64_t>(p) * (maxLong + 1)] = static_cast<int32_t>(lo);
}

// Then the rows l = 1 .. header[1] of every panel, a thread each.  Inside a panel's part the entries keep their CSR
// order, so their positions in the caller's arrays (`pos`) ascend there, and row l starts where they reach the
// row's first entry of this panel or a later one in the caller's arrays (csrChunk, panel-major).
__global__ __launch_bounds__(kBlockThreads) void LongRowPiecesKernel(const int32_t *__restrict__ pos, int64_t nnz,
                                                                     const int32_t *__restrict__ csrChunk,
                                                                     const int32_t *__restrict__ header, int32_t P,
                                                                     int32_t maxLong, int32_t *pieceStart)
{
    const int32_t numLong = header[1];
    const int64_t total = static_cast<int64_t>(numLong) * P;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < total; j += stride) {
        const int64_t p = j / numLong;
        const int32_t l = static_cast<int32_t>(j % numLong) + 1;
        int32_t lo = pieceStart[p * (maxLong + 1)];
        int32_t hi = p + 1 < P ? pieceStart[(p + 1) * (maxLong + 1)] : static_cast<int32_t>(nnz);
        if (l < numLong) {
            const int32_t want = csrChunk[p * maxLong + l];
            while (lo < hi) {
                const int32_t mid = lo + ((hi - lo) >> 1);
                if (pos[mid] < want) {
                    lo = mid + 1;
                } else {
                    hi = mid;
                }
            }
        }
        pieceStart[p * (maxLong + 1) + l] = hi;
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
// afterwards: in block order every chunk starts on such a multiple, the gap behind it is padding).
__global__ __launch_bounds__(kBlockThreads) void BlockedTablesKernel(const int32_t *__restrict__ srcStart, int32_t P,
                                                                     int32_t B, int32_t *__restrict__ dstStart)
{
    const int64_t total = static_cast<int64_t>(P) * B;
    const int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (j == 0) {
        dstStart[0] = 0;
    }
    if (j < total) {
        const int64_t b = j / P, p = j % P;
        const int32_t count = srcStart[p * B + b + 1] - srcStart[p * B + b];
        dstStart[1 + j] = (count + kLaneEntries - 1) / kLaneEntries * kLaneEntries;
    }
}

// blockRow[b] = first row of row block b (blockRow pre-filled with `rows`).
__global__ __launch_bounds__(kBlockThreads) void BlockedRowBlocksKernel(const int32_t *__restrict__ offsets,
                                                                        int32_t rows, int32_t window, int32_t B,
                                                                        const int32_t *__restrict__ longBefore,
                                                                        int32_t rowLog, int32_t *__restrict__ blockRow)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const int32_t row = static_cast<int32_t>(r);
    const int32_t cur = RowBlockOf(offsets, row, window, B, longBefore, rowLog);
    const int32_t prev = row > 0 ? RowBlockOf(offsets, row - 1, window, B, longBefore, rowLog) : -1;
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

// longDeferred[l] = 1 for the long rows of a row block that holds more than kInBlockLongRows of them (`always`: of
// every block: streamed blocks leave all long rows to SpmvLongRowSumKernel), else 0;
// header[4] (zero before) = their number.
__global__ __launch_bounds__(kBlockThreads) void BlockedLongDeferKernel(const int32_t *__restrict__ longFirst, int32_t B,
                                                                        int32_t always, int32_t *__restrict__ longDeferred,
                                                                        int32_t *__restrict__ header)
{
    const int32_t b = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (b >= B) {
        return;
    }
    const int32_t l0 = longFirst[b], l1 = longFirst[b + 1];
    const int32_t defer = (always != 0 || l1 - l0 > kInBlockLongRows) ? 1 : 0;
    for (int32_t l = l0; l < l1; ++l) {
        longDeferred[l] = defer;
    }
    if (defer != 0) {
        atomicAdd(header + 4, l1 - l0);
    }
}

// What phase 2 reads of row block b first (BlockMeta): its rows, its piece of the block order, its long rows, the
// first of its entries among the entries that phase 2 sums (offsets), and where its values start in the array that
// phase 2 reads them from: the caller's (valueOffsets = its row offsets; a block then holds no long row except as
// its last row, so that its other entries are one piece) or the compact copy (valueOffsets = offsets).
// blockShort[b] = the former, for the scatter kernel.  panelStart[p] = first entry of panel p in panel order
// (p = P: the number of entries there).  header[3] (zero before) = entries of the largest block.
__global__ __launch_bounds__(kBlockThreads) void BlockedBlockTablesKernel(
    const int32_t *__restrict__ offsets, const int32_t *__restrict__ valueOffsets, const int32_t *__restrict__ blockRow,
    const int32_t *__restrict__ dstStart, const int32_t *__restrict__ srcStart, const int32_t *__restrict__ longFirst,
    int32_t P, int32_t B, int32_t *__restrict__ blockShort, BlockMeta *__restrict__ meta,
    int32_t *__restrict__ panelStart, int32_t *__restrict__ header)
{
    const int32_t b = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (b <= B) {
        blockShort[b] = offsets[blockRow[b]];
    }
    if (b <= P) {
        panelStart[b] = srcStart[static_cast<int64_t>(b) * B];
    }
    if (b < B) {
        BlockMeta m;
        m.row0 = blockRow[b];
        m.nRows = blockRow[b + 1] - blockRow[b];
        m.dBeg = dstStart[static_cast<int64_t>(b) * P];
        m.dEnd = dstStart[static_cast<int64_t>(b + 1) * P];
        m.base = valueOffsets[blockRow[b]];
        m.short0 = offsets[blockRow[b]];
        m.l0 = longFirst != nullptr ? longFirst[b] : 0;
        m.l1 = longFirst != nullptr ? longFirst[b + 1] : 0;
        m.bitsOff = BlockBitsOff(m.short0, b);
        m.ordOff = BlockOrdOff(m.row0, b);
        m.nEntries = offsets[blockRow[b + 1]] - offsets[blockRow[b]];
        m.pad = 0;
        meta[b] = m;
        atomicMax(header + 3, offsets[blockRow[b + 1]] - offsets[blockRow[b]]);
    }
}

constexpr uint16_t kNoRow = 0xffffu;  // the row of the key of the entries behind a block's last: none

// Where entry e of a row block sits in the LDS window of phase 2 (plus the window's first entry): a lane takes 16
// consecutive entries there, and with the 1024 entries of a wavefront's round stored entry-of-the-lane-major, lane
// minor, the 64 lanes read 64 neighbouring words at a time.  The slots are stored like this.
__host__ __device__ __forceinline__ uint32_t WindowPlace(uint32_t e)
{
    return (e & ~1023u) | ((e & 15u) << 6) | ((e >> 4) & 63u);
}

// The tables by which phase 2 tells the rows of a block's entries apart, a workgroup a block.  The block's entries,
// in row order, are numbered from 0; bit e of the block's words is set where entry e is the first of its row, and
// bit (number of entries) as well, for what a lane reads behind the block's last entry; prefix[w] = bits in the
// words in front of word w.  The number of bits up to and including an entry's own is the entry's key: ordRow[key]
// = the row, counted from the block's first; the last key stands for no row.
constexpr int kTableThreads = 512;
constexpr int kTableWords = (kMaxBlockEntries + 1 + 31) / 32 + 1;

__global__ __launch_bounds__(kTableThreads) void BlockedRowTablesKernel(const BlockMeta *__restrict__ meta,
                                                                        const int32_t *__restrict__ offsets,
                                                                        uint32_t *__restrict__ rowBitsG,
                                                                        uint16_t *__restrict__ bitPrefixG,
                                                                        uint16_t *__restrict__ ordRowG)
{
    __shared__ uint32_t bits[kTableWords];
    __shared__ uint16_t prefix[kTableWords];
    __shared__ uint32_t waveTotal[kTableThreads / kWave];
    const int tid = threadIdx.x;
    const BlockMeta m = meta[blockIdx.x];
    if (m.nRows <= 0) {
        return;
    }
    const int32_t nRows = m.nRows < kRowBlockRows ? m.nRows : kRowBlockRows;
    int32_t nB = offsets[m.row0 + nRows] - m.short0;
    nB = nB < 0 ? 0 : (nB < kMaxBlockEntries ? nB : kMaxBlockEntries);
    const int32_t words = (nB + 32) / 32;  // bits 0 .. nB
    for (int32_t w = tid; w < words; w += kTableThreads) {
        bits[w] = 0;
    }
    __syncthreads();
    for (int32_t i = tid; i < nRows; i += kTableThreads) {
        const int32_t o = offsets[m.row0 + i] - m.short0, oNext = offsets[m.row0 + i + 1] - m.short0;
        if (oNext > o && o >= 0 && o < nB) {
            atomicOr(&bits[o >> 5], 1u << (o & 31));
        }
    }
    if (tid == 0) {
        atomicOr(&bits[nB >> 5], 1u << (nB & 31));
    }
    __syncthreads();
    // bits in front of every word: a thread's words one after the other, the threads by a scan in two steps
    const int32_t per = (words + kTableThreads - 1) / kTableThreads;
    uint32_t mine = 0;
    for (int32_t u = 0; u < per; ++u) {
        const int32_t w = tid * per + u;
        mine += w < words ? __popc(bits[w]) : 0;
    }
    uint32_t incl = mine, none = 0;
    SegScanStep<kDppRowShr1, 0xf>(incl, none);
    SegScanStep<kDppRowShr2, 0xf>(incl, none);
    SegScanStep<kDppRowShr4, 0xf>(incl, none);
    SegScanStep<kDppRowShr8, 0xf>(incl, none);
    SegScanStep<kDppRowBcast15, 0xa>(incl, none);
    SegScanStep<kDppRowBcast31, 0xc>(incl, none);
    if (tid % kWave == kWave - 1) {
        waveTotal[tid / kWave] = incl;
    }
    __syncthreads();
    uint32_t front = incl - mine;
    for (int w = 0; w < tid / kWave; ++w) {
        front += waveTotal[w];
    }
    for (int32_t u = 0; u < per; ++u) {
        const int32_t w = tid * per + u;
        if (w < words) {
            prefix[w] = static_cast<uint16_t>(front);
            front += __popc(bits[w]);
        }
    }
    __syncthreads();
    for (int32_t w = tid; w < words; w += kTableThreads) {
        rowBitsG[m.bitsOff + w] = bits[w];
        bitPrefixG[m.bitsOff + w] = prefix[w];
    }
    uint16_t *ord = ordRowG + m.ordOff;
    for (int32_t i = tid; i < nRows; i += kTableThreads) {
        const int32_t o = offsets[m.row0 + i] - m.short0, oNext = offsets[m.row0 + i + 1] - m.short0;
        if (oNext > o && o >= 0 && o < nB) {
            const uint32_t key = prefix[o >> 5] + __popc(bits[o >> 5] & (0xffffffffu >> (31 - (o & 31))));
            if (key <= static_cast<uint32_t>(nRows)) {
                ord[key] = static_cast<uint16_t>(i);
            }
        }
    }
    if (tid == 0) {
        const uint32_t last = prefix[nB >> 5] + __popc(bits[nB >> 5] & (0xffffffffu >> (31 - (nB & 31))));
        ord[0] = kNoRow;
        if (last <= static_cast<uint32_t>(nRows) + 1) {
            ord[last] = kNoRow;  // the key of bit nB
        }
    }
}

// flags[r] = 1 for a row without entries that is not a long row (phase 2 sees neither: y = beta * y is theirs).
__global__ __launch_bounds__(kBlockThreads) void EmptyRowFlagsKernel(const int32_t *__restrict__ rowOffsets,
                                                                     int64_t rows, int32_t *__restrict__ flags)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r < rows) {
        flags[r] = rowOffsets[r + 1] == rowOffsets[r] ? 1 : 0;  // (a long row is never empty)
    }
}

// From the prefix-summed flags: the list of those rows; header[5] = their number.
__global__ __launch_bounds__(kBlockThreads) void EmptyRowListKernel(const int32_t *__restrict__ emptyBefore, int64_t rows,
                                                                    int32_t *__restrict__ emptyRows,
                                                                    int32_t *__restrict__ header)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const int32_t upTo = emptyBefore[r], before = r > 0 ? emptyBefore[r - 1] : 0;
    if (upTo != before) {
        emptyRows[before] = static_cast<int32_t>(r);
    }
    if (r == rows - 1) {
        header[5] = upTo;
    }
}

// y[row] = beta * yIn[row] for the rows without entries.
template <typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvEmptyRowsKernel(const int32_t *__restrict__ emptyRows, int32_t count,
                                                                     int64_t rows, OutT *__restrict__ y,
                                                                     const OutT *__restrict__ yIn,
                                                                     OpsparseScalar alphaS, OpsparseScalar betaS)
{
    const int32_t i = static_cast<int32_t>(blockIdx.x * blockDim.x + threadIdx.x);
    if (i < count) {
        const int64_t row = emptyRows[i];
        if (row >= 0 && row < rows) {
            StoreOut<OutT, AccT>(y, yIn, row, AccT(0), ReadAcc<AccT>(alphaS), ReadAcc<AccT>(betaS));
        }
    }
}

// Slots into (block, panel) order, and for every eight positions there (a chunk starts on such a multiple, so they
// belong to one chunk) where they sit in panel order; with frozen values also the compact copy of the values that
// phase 2 reads, and the values and row numbers of the long entries beside their local columns.
template <typename ValT>
__global__ __launch_bounds__(kBlockThreads) void BlockedScatterKernel(
    const int32_t *__restrict__ pos, const int32_t *__restrict__ rowOfSrc, const int32_t *__restrict__ chunkKey,
    const ValT *__restrict__ vals, const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ srcStart, const int32_t *__restrict__ dstStart, const int32_t *__restrict__ blockShort,
    int64_t nnz, int32_t P, int32_t B, uint16_t *__restrict__ slot16, int32_t *__restrict__ src8,
    ValT *__restrict__ valS, uint32_t *__restrict__ longVals, uint16_t *__restrict__ longRowOf,
    const int32_t *__restrict__ longBefore)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t key = chunkKey[i];
        if (key < 0) {
            if (longVals != nullptr) {
                // an entry of a long row, frozen values: its value and the number of its row among the long rows
                // beside its local column, all three at its place in the sorted order
                longVals[i] = ToRaw(vals[pos[i]]);
                longRowOf[i] = static_cast<uint16_t>(longBefore[rowOfSrc[i]] - 1);
            }
            continue;
        }
        const int32_t p = key / B, b = key % B;
        const int64_t dst = i - srcStart[key] + dstStart[static_cast<int64_t>(b) * P + p];
        const int32_t row = rowOfSrc[i];
        const int32_t at = offsets[row] + (pos[i] - rowOffsets[row]);  // among the entries that phase 2 sums
        if (valS != nullptr) {
            valS[at] = vals[pos[i]];
        }
        int32_t slot = at - blockShort[b];
        slot = slot < 0 ? 0 : (slot < kMaxBlockEntries ? slot : kMaxBlockEntries - 1);
        slot16[dst] = static_cast<uint16_t>(WindowPlace(static_cast<uint32_t>(slot)));
        if ((dst & (kLaneEntries - 1)) == 0) {
            src8[dst / kLaneEntries] = static_cast<int32_t>(i);  // where these eight positions sit in panel order
        }
    }
}

// Streamed row blocks: what the scatter above does for the windowed ones.  Per position of the (block, panel) order
// the entry's row, counted from its block's first (the turn bits are added by StreamTurnsKernel), its value
// (`valD`: values frozen) or where its value sits in the value array (`posD`: values read at every call), and per
// eight positions where they sit in panel order.  Long entries as above.
template <typename ValT>
__global__ __launch_bounds__(kBlockThreads) void StreamScatterKernel(
    const int32_t *__restrict__ pos, const int32_t *__restrict__ rowOfSrc, const int32_t *__restrict__ chunkKey,
    const ValT *__restrict__ vals, const int32_t *__restrict__ srcStart, const int32_t *__restrict__ dstStart,
    const int32_t *__restrict__ blockRow, int64_t nnz, int32_t P, int32_t B, uint16_t *__restrict__ field,
    int32_t *__restrict__ src8, ValT *__restrict__ valD, int32_t *__restrict__ posD, uint32_t *__restrict__ longVals,
    uint16_t *__restrict__ longRowOf, const int32_t *__restrict__ longBefore)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int32_t key = chunkKey[i];
        if (key < 0) {
            if (longVals != nullptr) {
                longVals[i] = ToRaw(vals[pos[i]]);
                longRowOf[i] = static_cast<uint16_t>(longBefore[rowOfSrc[i]] - 1);
            }
            continue;
        }
        const int32_t p = key / B, b = key % B;
        const int64_t dst = i - srcStart[key] + dstStart[static_cast<int64_t>(b) * P + p];
        int32_t local = rowOfSrc[i] - blockRow[b];
        local = local < 0 ? 0 : (local < kStreamRows ? local : kStreamRows - 1);
        field[dst] = static_cast<uint16_t>(local);
        if (valD != nullptr) {
            valD[dst] = vals[pos[i]];
        }
        if (posD != nullptr) {
            posD[dst] = pos[i];
        }
        if ((dst & (kLaneEntries - 1)) == 0) {
            src8[dst / kLaneEntries] = static_cast<int32_t>(i);
        }
    }
}

// The turns.  SpmvBlockStreamKernel's wavefront takes 256 positions of its block at a time, lane l the four
// positions 4 l .. 4 l + 3 of them, and adds entry j of every lane to the rows' sums with one LDS instruction.  Two
// lanes of such an instruction that hold the same row must not add at once (the order of the two additions would be
// the hardware's choice): an entry's turn is the number of lower lanes of its instruction with the same row, and the
// kernel adds turn by turn.  A workgroup a block, a wavefront 256 positions at a time; turns of 31 and more are
// stored as 31 (the kernel takes those lanes one at a time, in lane order).
__global__ __launch_bounds__(kTurnThreads) void StreamTurnsKernel(const BlockMeta *__restrict__ meta,
                                                                    uint16_t *__restrict__ field)
{
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const BlockMeta m = meta[blockIdx.x];
    constexpr int kStep = kWave * 4;
    for (int32_t w = m.dBeg + wave * kStep; w < m.dEnd; w += (kTurnThreads / kWave) * kStep) {
        const int32_t at = w + lane * 4;  // (dBeg and dEnd are multiples of 8: the four positions are inside or outside)
        const bool inside = at < m.dEnd;
        Uint2 f = Uint2{kStreamPadRow * 0x10001u, kStreamPadRow * 0x10001u};
        if (inside) {
            f = *reinterpret_cast<const Uint2 *>(field + at);
        }
        const uint32_t row[4] = {f.x & 0x7ffu, (f.x >> 16) & 0x7ffu, f.y & 0x7ffu, (f.y >> 16) & 0x7ffu};
        uint32_t turn[4] = {0, 0, 0, 0};
        for (int other = 0; other < kWave - 1; ++other) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t theirs = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(row[j]), other));
                turn[j] += (other < lane && theirs == row[j]) ? 1u : 0u;
            }
        }
        if (inside) {
            uint32_t out[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t t = turn[j] < kStreamMaxRound ? turn[j] : kStreamMaxRound;
                out[j] = row[j] == kStreamPadRow ? kStreamPadRow : (row[j] | (t << kStreamRoundShift));
            }
            *reinterpret_cast<Uint2 *>(field + at) = Uint2{out[0] | (out[1] << 16), out[2] | (out[3] << 16)};
        }
    }
}

// dst[j] = src[perm[j]]: the values of the transposed copy, refreshed from the caller's.
template <typename ValT>
__global__ __launch_bounds__(kBlockThreads) void PermuteValuesKernel(const ValT *__restrict__ src,
                                                                     const int32_t *__restrict__ perm, int64_t nnz,
                                                                     ValT *__restrict__ dst)
{
    constexpr int kPer = 4;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * kPer;
    for (int64_t i0 = (static_cast<int64_t>(blockIdx.x) * blockDim.x * kPer) + threadIdx.x; i0 < nnz; i0 += stride) {
        int32_t at[kPer];
        ValT v[kPer];
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int64_t i = i0 + static_cast<int64_t>(u) * blockDim.x;
            at[u] = i < nnz ? __builtin_nontemporal_load(perm + i) : 0;
        }
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const uint32_t a = static_cast<uint32_t>(at[u]);
            v[u] = src[a < static_cast<uint64_t>(nnz) ? a : 0];
        }
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int64_t i = i0 + static_cast<int64_t>(u) * blockDim.x;
            if (i < nnz) {
                dst[i] = v[u];
            }
        }
    }
}

// ------------------------------------------------------------------ phase 1

// xg[i] = x[panel * 2^15 + colLocal[i]] for the entries of one panel (a part of them when
// `splits` > 1), the panel's slice of x held in LDS.
//
// Long rows: `header[1]` of them; longPartial[l * P + p] receives the sum of val * x over the entries of long row l
// in panel p.  Live values: these are the entries longChunk[p * maxLong + l] .. longChunk[(p + 1) * maxLong + l] of
// the caller's colInd / vals, and groups of kLongLanes lanes take the rows in turn.  Frozen values (LongSorted):
// the panel's long entries follow each other, in row order, at the positions longChunk[p * (maxLong + 1)] ..
// longChunk[p * (maxLong + 1) + header[1]] of colLocal, of xg (which there holds their values) and of longRowOf
// (the number l of each one's row); the workgroup streams them flat, every wavefront a stretch of its own, and sums
// the rows as SegRound does, kLongTile rows at a time ([.. + l] is where row l starts).
template <bool LongSorted, typename XT, typename AccT>
__global__ __launch_bounds__(kBlkThreads) void SpmvBlockGatherKernel(const uint16_t *__restrict__ colLocal,
                                                                     const XT *__restrict__ x,
                                                                     uint32_t *__restrict__ xg,
                                                                     const int32_t *__restrict__ panelStart,
                                                                     int64_t cols, int32_t splits,
                                                                     const int32_t *__restrict__ header,
                                                                     const int32_t *__restrict__ longChunk,
                                                                     const int32_t *__restrict__ colInd,
                                                                     const XT *__restrict__ vals, int64_t nnz,
                                                                     int32_t P, int32_t maxLong,
                                                                     const uint16_t *__restrict__ longRowOf,
                                                                     uint64_t *__restrict__ longPartial)
{
    constexpr bool kIntData = std::is_same<XT, int32_t>::value;
    __shared__ __align__(16) uint32_t xs[kPanelCols];
    __shared__ __align__(16) int32_t tileBuf[2 * kLongTile];  // piece bounds (live) or the sums of the rows (frozen)
    __shared__ SegEnds ends;
    int32_t *pieceLo = tileBuf, *pieceHi = tileBuf + kLongTile;
    const int tid = threadIdx.x;
    // Neighbouring panels on one XCD: the pieces of a long row in panels p and p + 1 are neighbours in memory, and
    // the cache line they share is then fetched once, by the L2 both workgroups sit behind.
    const int64_t p = splits == 1 ? XcdContiguousTile(blockIdx.x, gridDim.x) : blockIdx.x / splits;
    const int64_t part = splits == 1 ? 0 : blockIdx.x % splits;
    const int64_t c0 = p << kPanelLog;
    const int64_t cn = cols - c0 < kPanelCols ? cols - c0 : kPanelCols;
    const int64_t a = panelStart[p], e = panelStart[p + 1];
    if constexpr (sizeof(XT) == 4) {
        const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
        for (int64_t i = tid * 4; i < cn; i += kBlkThreads * 4) {
            if (vec && i + 4 <= cn) {
                *reinterpret_cast<Uint4 *>(xs + i) = *reinterpret_cast<const Uint4 *>(x + c0 + i);
            } else {
                for (int64_t k = i; k < cn && k < i + 4; ++k) {
                    xs[k] = ToRaw(x[c0 + k]);
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
                *reinterpret_cast<Uint4 *>(xs + i) = Uint4{ToRaw(four[0]), ToRaw(four[1]), ToRaw(four[2]), ToRaw(four[3])};
            } else {
                for (int64_t k = i; k < cn && k < i + 4; ++k) {
                    xs[k] = ToRaw(x[c0 + k]);
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
            xg[lo + tid] = xs[colLocal[lo + tid] & (kPanelCols - 1)];
        }
    } else if (lo < hi) {
        if (tid < 4) {
            const int64_t i = lo + tid;
            if (i < g0 * 4) {
                xg[i] = xs[colLocal[i] & (kPanelCols - 1)];
            }
        } else if (tid < 8) {
            const int64_t i = g1 * 4 + (tid - 4);
            if (i < hi) {
                xg[i] = xs[colLocal[i] & (kPanelCols - 1)];
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
                Uint4 r;
                r.x = xs[c[u].x & (kPanelCols - 1)];
                r.y = xs[c[u].y & (kPanelCols - 1)];
                r.z = xs[c[u].z & (kPanelCols - 1)];
                r.w = xs[c[u].w & (kPanelCols - 1)];
                if (gg < g1) {
                    *(reinterpret_cast<Uint4 *>(xg) + gg) = r;
                }
            }
        }
    }
    // ---- long rows: this panel's piece of each
    const int32_t numLong = header != nullptr ? header[1] : 0;
    if (numLong == 0) {
        return;
    }
    const int lane = tid % kWave, wave = tid / kWave;
    if constexpr (LongSorted) {
        // Tiles of long rows, shared out among the panel's workgroups where it has several (a partial sum has one
        // writer); as many tiles as workgroups at least.
        constexpr int kWaves = kBlkThreads / kWave;
        uint64_t *accL = reinterpret_cast<uint64_t *>(tileBuf);
        const int32_t *tab = longChunk + p * (maxLong + 1);
        int32_t tile = (numLong + static_cast<int32_t>(splits) - 1) / static_cast<int32_t>(splits);
        tile = (tile + kWave - 1) / kWave * kWave;
        tile = tile < kLongTile ? tile : kLongTile;
        for (int32_t t0 = static_cast<int32_t>(part) * tile; t0 < numLong; t0 += static_cast<int32_t>(splits) * tile) {
            const int32_t tn = numLong - t0 < tile ? numLong - t0 : tile;
            const int64_t from = tab[t0], to = tab[t0 + tn];
            __syncthreads();  // (the tile before is written out)
            for (int32_t i = tid; i < tn; i += kBlkThreads) {
                accL[i] = AccToSlot(AccT(0));
            }
            __syncthreads();
            // the stream [from, to) in rounds of 256 entries that start at multiples of 4, every wavefront a
            // stretch of consecutive rounds
            const int64_t first = from & ~int64_t{3};
            const int64_t rounds = to > from ? (to - first + kRound - 1) / kRound : 0;
            const int64_t perWave = (rounds + kWaves - 1) / kWaves;
            const int64_t rBeg = wave * perWave;
            const int64_t rEnd = rBeg + perWave < rounds ? rBeg + perWave : rounds;
            const int64_t lastGroup = to > from ? ((to - 1) & ~int64_t{3}) : first;
            int32_t carryKey = kNoKey, firstKey = kNoKey;
            AccT carrySum = AccT(0);
            struct Piece {
                Ushort4 c, r;
                Uint4 v;
            };
            auto fetch = [&](int64_t round) {
                int64_t i = first + round * kRound + lane * kSegEntries;
                i = i < lastGroup ? i : lastGroup;
                Piece pc;
                pc.c = __builtin_nontemporal_load(reinterpret_cast<const Ushort4 *>(colLocal + i));
                pc.r = __builtin_nontemporal_load(reinterpret_cast<const Ushort4 *>(longRowOf + i));
                const Uint4U v = __builtin_nontemporal_load(reinterpret_cast<const Uint4U *>(xg + i));
                pc.v = Uint4{v.x, v.y, v.z, v.w};
                return pc;
            };
            auto out = [&](int32_t key, AccT sum) { accL[key] = AccToSlot(sum); };
            if (rBeg < rEnd) {
                Piece cur = fetch(rBeg);
                for (int64_t round = rBeg; round < rEnd; ++round) {
                    const Piece next = fetch(round + 1 < rEnd ? round + 1 : round);
                    const int64_t i = first + round * kRound + lane * kSegEntries;
                    const uint32_t cs[4] = {cur.c.x, cur.c.y, cur.c.z, cur.c.w};
                    const uint32_t rw[4] = {cur.r.x, cur.r.y, cur.r.z, cur.r.w};
                    const uint32_t vs[4] = {cur.v.x, cur.v.y, cur.v.z, cur.v.w};
                    int32_t k[kSegEntries];
                    AccT t[kSegEntries];
#pragma unroll
                    for (int j = 0; j < kSegEntries; ++j) {
                        const int64_t en = i + j;
                        const uint32_t key = rw[j] - static_cast<uint32_t>(t0);
                        const bool in = en >= from && en < to && key < static_cast<uint32_t>(tn);
                        k[j] = in ? static_cast<int32_t>(key) : kNoKey;
                        const AccT prod = RawToAcc<AccT, kIntData>(vs[j]) *
                                          RawToAcc<AccT, kIntData>(xs[cs[j] & (kPanelCols - 1)]);
                        t[j] = in ? prod : AccT(0);
                    }
                    if (round == rBeg) {
                        firstKey = __shfl(k[0], 0);
                    }
                    SegRound<AccT>(k, t, lane, carryKey, carrySum,
                                   [&](int32_t key, AccT sum) { SegStore<AccT>(ends, wave, firstKey, key, sum, out); });
                    cur = next;
                }
            }
            if (lane == 0) {
                SegLeave<AccT>(ends, wave, firstKey, carryKey, firstKey == carryKey, carrySum);
            }
            __syncthreads();
            if (tid == 0) {
                int32_t pendKey = kNoKey;
                AccT pendSum = AccT(0);
                SegJoin<AccT>(ends, kWaves, pendKey, pendSum, out);
                if (pendKey != kNoKey) {
                    out(pendKey, pendSum);
                }
            }
            __syncthreads();
            for (int32_t i = tid; i < tn; i += kBlkThreads) {
                longPartial[static_cast<int64_t>(t0 + i) * P + p] = accL[i];
            }
        }
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
            auto request = [&](int32_t i0, int32_t i1, int32_t q, Int4U *c, Uint4 *v) {
                int64_t at = i0 + 4 * static_cast<int64_t>(q);
                at = at + 4 <= i1 ? at : static_cast<int64_t>(i1) - 4;
                at = at < 0 ? 0 : at;
                *c = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(colInd + at));
                *v = LoadFourRaw(vals + at);
            };
            auto add = [&](int32_t i0, int32_t i1, int32_t q, const Int4U &c, const Uint4 &v, AccT *sum) {
                const int64_t own = i0 + 4 * static_cast<int64_t>(q);  // first entry of the group
                int64_t at = own + 4 <= i1 ? own : static_cast<int64_t>(i1) - 4;
                at = at < 0 ? 0 : at;
                const uint32_t mask = kPanelCols - 1;  // an entry of the group is in the panel by construction
                const int32_t cs[4] = {c.x, c.y, c.z, c.w};
                const uint32_t vs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const AccT t = RawToAcc<AccT, kIntData>(vs[j]) *
                                   RawToAcc<AccT, kIntData>(xs[static_cast<uint32_t>(cs[j] - base) & mask]);
                    *sum += (at + j >= own && at + j < i1) ? t : AccT(0);
                }
            };
            int32_t i0 = pieceLo[k], i1 = pieceHi[k];
            Int4U cFirst;
            Uint4 vFirst;
            request(i0, i1, gt, &cFirst, &vFirst);
            while (true) {
                const int32_t kn = k + stride;
                const int32_t kk = kn < tn ? kn : k;
                const int32_t j0 = pieceLo[kk], j1 = pieceHi[kk];
                Int4U cAhead;
                Uint4 vAhead;
                request(j0, j1, gt, &cAhead, &vAhead);
                const int32_t n4 = (i1 - i0 + 3) >> 2;  // groups of the piece, the last one maybe short
                AccT sum = AccT(0);
                Int4U c = cFirst;
                Uint4 v = vFirst;
                for (int32_t q = gt; q < n4; q += kLongLanes) {
                    Int4U cNext;
                    Uint4 vNext;
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
                    longPartial[static_cast<int64_t>(t0 + k) * P + p] = AccToSlot(sum);
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

// The sum of a long row's partial sums, lane by lane in panel order and then across the lanes, the same way at
// every call; every lane returns it.
template <typename AccT>
__device__ __forceinline__ AccT LongRowTotal(const uint64_t *__restrict__ from, int32_t P, int lane)
{
    AccT sum = AccT(0);
    for (int32_t p0 = 0; p0 < P; p0 += 4 * kWave) {
        uint64_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int32_t p = p0 + u * kWave + lane;
            v[u] = from[p < P ? p : P - 1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            sum += p0 + u * kWave + lane < P ? SlotToAcc<AccT>(v[u]) : AccT(0);
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        sum += __shfl_xor(sum, off);
    }
    return sum;
}

constexpr int kRowsThreads = 512;  // threads of a phase-2 workgroup; two workgroups share a compute unit
constexpr int kLaneRun = 16;        // consecutive entries a lane sums in one round of phase 2
constexpr int kBigRound = kWave * kLaneRun;
constexpr int kStagePasses = 3;     // passes over a block's positions whose loads a wavefront has in flight at a time
constexpr uint64_t kJoinMark = 0x7ff8dead0000beefull;  // rowSum of a row that the joining thread writes

template <typename ValT, typename OutT>
struct BlockRowsArgs {
    const uint32_t *xg;
    const uint16_t *slot16;
    const int32_t *src8;
    const BlockMeta *meta;
    const uint32_t *rowBits;
    const uint16_t *bitPrefix, *ordRow;
    const ValT *vals;
    OutT *y;
    const OutT *yIn;
    OpsparseScalar alpha, beta;
    const int32_t *longRows;
    const uint64_t *longPartial;
    int32_t P;
    int32_t xgEntries;  // entries of xg (a position's place there is checked against it)
    int64_t valEntries; // entries of `vals`
};

// One workgroup per row block: y[row] = alpha * sum(val * x) + beta * yIn[row] for the rows of the block that have
// entries in it (rows without entries are SpmvEmptyRowsKernel's).
//
// In block order every (panel, block) chunk starts on a multiple of kLaneEntries and is padded to one (padding
// carries the slot kPadSlot); src8[d / 8] is where the eight positions from d on sit in panel order, i.e. in xg.
// The block's entries are entries meta.base .. of `vals` in row order.  The tables of BlockedRowTablesKernel tell
// their rows apart: the key of an entry is two reads and a population count.  A block of more than kRowsWindow
// entries is worked a window at a time: its positions are read once per window.
//
// A window, step by step.  (1) The gathered x of the block's positions is dropped at its slot of xwin.  (2) Every
// lane takes kLaneRun consecutive entries of the window into registers; behind a barrier the window's memory serves
// as rowSum[key - first key of the window].  (3) A lane adds its entries up run by run, in stored order; a run that
// begins and ends inside the lane is a row's sum and goes to rowSum.  The runs at the lanes' edges are joined by a
// segmented scan over the wavefront, the ones at the wavefronts' edges by one thread (SegJoin), which writes those
// rows itself.  (4) rowSum goes out, a key a lane.
template <int kThreads, typename ValT, typename OutT, typename AccT>
__global__ __launch_bounds__(kThreads, 2 * kThreads / kWave / 4) void SpmvBlockRowsKernel(
    const BlockRowsArgs<ValT, OutT> a)
{
    constexpr bool kIntData = std::is_same<ValT, int32_t>::value;
    constexpr int kW = kRowsWindow;
    constexpr int kWaves = kThreads / kWave;
    constexpr int kMaxRounds = (kW / kBigRound + kWaves - 1) / kWaves;
    constexpr int kWords = kW / 32 + 1;              // of a window's bits, the bit behind its last entry included
    constexpr int kPassSpan = kWave * kLaneEntries;  // positions a wavefront takes per pass: eight a lane
    constexpr int kOrdPer = (kRowBlockRows + 8 + 8 * kThreads - 1) / (8 * kThreads);  // 16-byte pieces of ordRow a thread
    static_assert(kW % kBigRound == 0 && kWords <= kThreads, "a window is whole rounds; a word of its bits a thread");
    static_assert(kW / 2 >= kRowBlockRows + 2, "a sum for every row of a block, and two more keys");
    static_assert(kLaneEntries == 8 && kLaneRun == 16, "the unpacking below");
    __shared__ __align__(16) uint32_t xwin[kW];
    __shared__ __align__(16) uint16_t ordRow[kRowBlockRows + 16];
    __shared__ uint32_t rowBits[kWords];
    __shared__ uint16_t bitPrefix[kWords];
    __shared__ SegEnds ends;
    uint64_t *rowSum = reinterpret_cast<uint64_t *>(xwin);  // (once every lane has its entries of the window)
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    // Neighbouring blocks on one XCD, at about the same time: the chunks (p, b) and (p, b + 1) are neighbours in
    // xg, and the line they share is fetched once by the L2 both workgroups sit behind.
    const int64_t blk = XcdContiguousTile(blockIdx.x, gridDim.x);
    const BlockMeta m = a.meta[blk];
    if (m.nRows <= 0) {
        return;  // a block number no row maps to
    }
    const int32_t row0 = m.row0, dBeg = m.dBeg, dEnd = m.dEnd, P = a.P;
    const int32_t nRows = m.nRows < kRowBlockRows ? m.nRows : kRowBlockRows;
    // ---- asked for at once: the rows of the keys, and the number of the block's entries (the last prefix count
    // belongs to the word of the bit behind the last entry; the words are found through it)
    Uint4 ordPiece[kOrdPer];
#pragma unroll
    for (int u = 0; u < kOrdPer; ++u) {
        const int32_t i = 8 * (tid + u * kThreads);
        ordPiece[u] = __builtin_nontemporal_load(
            reinterpret_cast<const Uint4 *>(a.ordRow + m.ordOff + (i <= nRows + 1 ? i : 0)));
    }
    const AccT alpha = ReadAcc<AccT>(a.alpha), beta = ReadAcc<AccT>(a.beta);
    auto out = [&](int32_t row, AccT sum) { StoreOut<OutT, AccT>(a.y, a.yIn, row0 + row, sum, alpha, beta); };
    // Long rows of this block: phase 1 left the sum of each of their panels.  A block with more than
    // kInBlockLongRows of them leaves them to SpmvLongRowSumKernel (a matrix of long rows only has few blocks).
    if (m.l1 - m.l0 <= kInBlockLongRows) {
        for (int32_t l = m.l0 + wave; l < m.l1; l += kWaves) {
            const AccT sum = LongRowTotal<AccT>(a.longPartial + static_cast<int64_t>(l) * P, P, lane);
            const uint32_t r = static_cast<uint32_t>(a.longRows[l] - row0);
            if (lane == 0 && r < static_cast<uint32_t>(nRows)) {
                out(static_cast<int32_t>(r), sum);
            }
        }
    }
    const int32_t nB = m.nEntries;  // entries of the block
    int32_t pendKey = kNoKey;  // (wavefront 0: the row that is still open across the wavefronts and windows)
    AccT pendSum = AccT(0);
    // (whatever the tables hold, a row outside the block is never written)
    auto outKey = [&](int32_t key, AccT sum) {
        const uint16_t row = ordRow[static_cast<uint32_t>(key) < static_cast<uint32_t>(kRowBlockRows + 8) ? key : 0];
        if (static_cast<int32_t>(row) < nRows) {
            out(row, sum);
        }
    };
    for (int32_t w0 = 0; w0 < nB; w0 += kW) {
        const int32_t nEnd = nB - w0 < kW ? nB : w0 + kW;  // the window holds the entries [w0, nEnd)
        const int32_t rounds = (nEnd - w0 + kBigRound - 1) / kBigRound;
        const int32_t perWave = (rounds + kWaves - 1) / kWaves;
        const int32_t rBeg = wave * perWave;
        const int32_t rEnd = rBeg + perWave < rounds ? rBeg + perWave : rounds;
        // ---- asked for in this order: the window's bits and their counts and where the block's positions sit in xg
        // (little); then, as soon as that is known, the gathered x, and behind it the values of the wavefront's
        // rounds: what waits for the gathered x does not wait for the values
        const int32_t wordsHere = (nEnd - w0) / 32 + 1;
        const int32_t wordAt = m.bitsOff + w0 / 32 + (tid < wordsHere ? tid : 0);
        const uint32_t myBits = __builtin_nontemporal_load(a.rowBits + wordAt);
        const uint16_t myPrefix = __builtin_nontemporal_load(a.bitPrefix + wordAt);
        Uint4 slots[kStagePasses];
        int32_t src[kStagePasses];
        Uint4 xa[kStagePasses], xb[kStagePasses];
        auto askPlaces = [&](int32_t start) {
#pragma unroll
            for (int u = 0; u < kStagePasses; ++u) {
                int32_t mine = start + u * kWaves * kPassSpan + lane * kLaneEntries;
                mine = mine < dEnd ? mine : dBeg;  // (a lane without positions reads the first ones again)
                slots[u] = __builtin_nontemporal_load(reinterpret_cast<const Uint4 *>(a.slot16 + mine));
                src[u] = __builtin_nontemporal_load(a.src8 + (mine >> 3));
            }
        };
        auto askGathered = [&]() {
#pragma unroll
            for (int u = 0; u < kStagePasses; ++u) {
                uint32_t at = static_cast<uint32_t>(src[u]);
                at = at < static_cast<uint32_t>(a.xgEntries) ? at : 0u;  // (in range whatever the table holds)
                const Uint4U v0 = *reinterpret_cast<const Uint4U *>(a.xg + at);
                const Uint4U v1 = *reinterpret_cast<const Uint4U *>(a.xg + at + 4);
                xa[u] = Uint4{v0.x, v0.y, v0.z, v0.w};
                xb[u] = Uint4{v1.x, v1.y, v1.z, v1.w};
            }
        };
        auto drop = [&](int32_t start) {
#pragma unroll
            for (int u = 0; u < kStagePasses; ++u) {
                const int32_t mine = start + u * kWaves * kPassSpan + lane * kLaneEntries;
                const uint32_t sl[8] = {slots[u].x & 0xffffu, slots[u].x >> 16, slots[u].y & 0xffffu, slots[u].y >> 16,
                                        slots[u].z & 0xffffu, slots[u].z >> 16, slots[u].w & 0xffffu, slots[u].w >> 16};
                const uint32_t xv[8] = {xa[u].x, xa[u].y, xa[u].z, xa[u].w, xb[u].x, xb[u].y, xb[u].z, xb[u].w};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t rel = sl[j] - static_cast<uint32_t>(w0);  // (a window is whole rounds: the
                                                                             // slots' order inside a round stays)
                    if (mine < dEnd && sl[j] != kPadSlot && rel < static_cast<uint32_t>(kW)) {
                        xwin[rel] = xv[j];
                    }
                }
            }
        };
        const int32_t start0 = dBeg + wave * kPassSpan;
        askPlaces(start0);
        askGathered();
        if (w0 == 0) {
            // (the rows of the keys have arrived with the places: nothing reads them before the next barrier)
#pragma unroll
            for (int u = 0; u < kOrdPer; ++u) {
                const int32_t i = 8 * (tid + u * kThreads);
                if (i <= nRows + 1) {
                    *reinterpret_cast<Uint4 *>(ordRow + i) = ordPiece[u];
                }
            }
        }
        // the values: four at a time at any entry of the block that is at least four in front of the array's end
        // (a lane behind the block's last entry reads its first ones; what it reads is not used)
        Uint4 vraw[kMaxRounds][kLaneRun / 4];
        const bool atArrayEnd = static_cast<int64_t>(m.base) + nB + 4 > a.valEntries;
#pragma unroll
        for (int u = 0; u < kMaxRounds; ++u) {
            const int32_t q = w0 + (rBeg + u) * kBigRound + lane * kLaneRun;
            const ValT *from = a.vals + m.base;
#pragma unroll
            for (int f = 0; f < kLaneRun / 4; ++f) {
                const int32_t qf = q + 4 * f;
                if (!atArrayEnd) {
                    vraw[u][f] = LoadFourRaw(from + (qf < nEnd ? qf : 0));
                } else {
                    vraw[u][f] = Uint4{0, 0, 0, 0};
                    if (qf + 4 <= nEnd) {
                        vraw[u][f] = LoadFourRaw(from + qf);
                    } else if (qf < nEnd) {
                        vraw[u][f].x = ToRaw(from[qf]);
                        vraw[u][f].y = qf + 1 < nEnd ? ToRaw(from[qf + 1]) : 0u;
                        vraw[u][f].z = qf + 2 < nEnd ? ToRaw(from[qf + 2]) : 0u;
                    }
                }
            }
        }
        if (w0 > 0) {
            LdsBarrier();  // (the window before is done with)
        }
        if (tid < wordsHere) {
            rowBits[tid] = myBits;
            bitPrefix[tid] = myPrefix;
        }
        // ---- the gathered x of the block's positions into the window, kStagePasses passes at a time
        drop(start0);
        for (int32_t start = start0 + kStagePasses * kWaves * kPassSpan; start < dEnd;
             start += kStagePasses * kWaves * kPassSpan) {
            askPlaces(start);
            askGathered();
            drop(start);
        }
        LdsBarrier();
        // ---- the window's entries into registers
        uint32_t xraw[kMaxRounds][kLaneRun];
        uint32_t bits[kMaxRounds];
        int32_t before[kMaxRounds];
        const int32_t keyWin = bitPrefix[0];  // the key of the entry in front of the window
        // the words behind the window's last (a lane whose entries all lie behind the block's last reads there): no
        // bits, and every bit of the window in front of them
        const int32_t keyAll = bitPrefix[wordsHere - 1] + __popc(rowBits[wordsHere - 1]);
#pragma unroll
        for (int u = 0; u < kMaxRounds; ++u) {
            const int32_t rel = (rBeg + u < rEnd ? rBeg + u : 0) * kBigRound + lane * kLaneRun;
#pragma unroll
            for (int j = 0; j < kLaneRun; ++j) {
                xraw[u][j] = xwin[(rel & ~1023) + j * kWave + lane];  // (WindowPlace of entry rel + j)
            }
            const bool inWords = (rel >> 5) < wordsHere;
            const uint32_t word = inWords ? rowBits[rel >> 5] : 0u;
            const uint32_t shift = rel & 16;  // (a lane's entries are one half of a word)
            bits[u] = (word >> shift) & 0xffffu;
            // the key of the entry in front
            before[u] = inWords ? bitPrefix[rel >> 5] + __popc(word & ((1u << shift) - 1u)) : keyAll;
        }
        // the key of the window's last entry
        const int32_t lastRel = nEnd - w0 - 1;
        const int32_t keyEnd = bitPrefix[lastRel >> 5] + __popc(rowBits[lastRel >> 5] & (0xffffffffu >> (31 - (lastRel & 31))));
        LdsBarrier();
        // ---- the rows: values times gathered x, summed run by run
        int32_t firstKey = kNoKey, carryKey = kNoKey;
        AccT carrySum = AccT(0);
        constexpr uint32_t kSums = kW / 2;  // 8-byte sums the window's memory holds
        auto park = [&](int32_t key, uint64_t slot) {
            const uint32_t at = static_cast<uint32_t>(key - keyWin);
            if (at < kSums) {
                rowSum[at] = slot;
            }
        };
        auto finish = [&](int32_t key, AccT sum) {
            if (key == firstKey) {
                ends.sum[2 * wave] = AccToSlot(sum);  // the wavefront's first run: it may go on from the one before
            } else {
                park(key, AccToSlot(sum));
            }
        };
#pragma unroll
        for (int u = 0; u < kMaxRounds; ++u) {
            if (rBeg + u < rEnd) {
                const int32_t q = w0 + (rBeg + u) * kBigRound + lane * kLaneRun;
                const uint32_t b = bits[u];
                AccT headSum = AccT(0), run = AccT(0);
                int32_t key = before[u] + static_cast<int32_t>(b & 1u);  // of the lane's first entry
                const int32_t key0 = key;
                bool headOpen = true;
#pragma unroll
                for (int j = 0; j < kLaneRun; ++j) {
                    if (j > 0 && ((b >> j) & 1u) != 0) {
                        if (headOpen) {
                            headSum = run;  // the lane's first run ends here
                            headOpen = false;
                        } else {
                            park(key, AccToSlot(run));  // a run that begins and ends inside the lane
                        }
                        ++key;
                        run = AccT(0);
                    }
                    const uint32_t v4[4] = {vraw[u][j / 4].x, vraw[u][j / 4].y, vraw[u][j / 4].z, vraw[u][j / 4].w};
                    const AccT prod = RawToAcc<AccT, kIntData>(v4[j % 4]) * RawToAcc<AccT, kIntData>(xraw[u][j]);
                    run += q + j < nEnd ? prod : AccT(0);
                }
                if (u == 0) {
                    firstKey = static_cast<int32_t>(__builtin_amdgcn_readfirstlane(key0));
                }
                // `run` is the lane's last run; v becomes the sum of that run's row up to the end of this lane
                uint32_t fresh = (!headOpen || (b & 1u) != 0) ? 1u : 0u;  // it does not go on from the lane before
                AccT v = run;
                if (lane == 0 && fresh == 0) {
                    v += carrySum;
                }
                SegScanStep<kDppRowShr1, 0xf>(v, fresh);
                SegScanStep<kDppRowShr2, 0xf>(v, fresh);
                SegScanStep<kDppRowShr4, 0xf>(v, fresh);
                SegScanStep<kDppRowShr8, 0xf>(v, fresh);
                SegScanStep<kDppRowBcast15, 0xa>(v, fresh);
                SegScanStep<kDppRowBcast31, 0xc>(v, fresh);
                const AccT prevSum = DppMove<kDppWaveShr1, 0xf>(carrySum, v);
                // the row of the lane before ended with that lane (lane 0: the run carried over from the round
                // before; in the wavefront's first round there is none, the wavefront before has that row)
                if ((b & 1u) != 0 && (lane > 0 || u > 0)) {
                    finish(before[u], prevSum);
                }
                if (!headOpen) {
                    finish(key0, (b & 1u) != 0 ? headSum : prevSum + headSum);
                }
                carryKey = static_cast<int32_t>(ReadLane63(static_cast<uint32_t>(key)));
                carrySum = ReadLane63(v);
            }
        }
        if (lane == 0) {
            // to the joining thread its two ends; and in rowSum a mark for both: theirs is not a sum to write out
            SegLeave<AccT>(ends, wave, firstKey, carryKey, firstKey == carryKey, carrySum);
            if (firstKey != kNoKey) {
                park(firstKey, kJoinMark);
                park(carryKey, kJoinMark);
            }
        }
        LdsBarrier();
        if (wave == 0) {
            SegJoinWave<AccT>(ends, kWaves, lane, pendKey, pendSum, outKey);
        }
        const int32_t keyStop = keyEnd - keyWin < static_cast<int32_t>(kSums) ? keyEnd : keyWin + static_cast<int32_t>(kSums) - 1;
        for (int32_t key = keyWin + 1 + tid; key <= keyStop; key += kThreads) {
            const uint64_t sum = rowSum[key - keyWin];
            if (sum != kJoinMark) {
                outKey(key, SlotToAcc<AccT>(sum));
            }
        }
    }
    if (tid == 0 && pendKey != kNoKey) {
        outKey(pendKey, pendSum);
    }
}

// ---- phase 2, streamed --------------------------------------------------------------------------------------
// A wavefront owns a row block of at most 2^10 rows: the rows' sums sit in its 8 KiB of LDS, and it streams the
// block's positions of the (block, panel) order, 512 at a time with the next 1024 on their way: value, row field and
// gathered x (eight positions of a chunk are eight neighbours in panel order, src8 says where).  Nothing is shared
// between wavefronts and nothing waits for another wavefront: sixteen of them a compute unit hide each other's
// loads, and the hardware deals the blocks out as wavefronts finish.  The order of the additions to a row's sum is
// fixed by the layout: instruction by instruction in stream order, and inside an instruction turn by turn
// (StreamTurnsKernel), so that no two lanes ever add to one sum at once.
template <typename ValT, typename OutT>
struct BlockStreamArgs {
    const uint32_t *xg;
    const uint16_t *field;
    const int32_t *src8;
    const BlockMeta *meta;
    const ValT *valD;
    OutT *y;
    const OutT *yIn;
    OpsparseScalar alpha, beta;
    const int32_t *longRows;
    int32_t B, xgEntries;
};

template <typename AccT>
__device__ __forceinline__ void StreamAdd(uint64_t *acc, uint32_t row, AccT t)
{
    if constexpr (std::is_same<AccT, uint32_t>::value) {
        atomicAdd(reinterpret_cast<uint32_t *>(acc + row), t);  // (the low word of the slot)
    } else {
        atomicAdd(reinterpret_cast<double *>(acc + row), t);
    }
}

template <typename ValT, typename OutT, typename AccT>
__global__ __launch_bounds__(kStreamThreads) void SpmvBlockStreamKernel(const BlockStreamArgs<ValT, OutT> a)
{
    constexpr bool kIntData = std::is_same<ValT, int32_t>::value;
    constexpr int kSub = kWave * 4, kStep = 2 * kSub;
    __shared__ __align__(16) uint64_t acc[kStreamRows + kWave];  // (behind the rows: a slot a lane, see below)
    const int lane = threadIdx.x;
    // neighbouring blocks read neighbouring pieces of every panel's xg: they go to one XCD, hence one L2
    const int32_t b = static_cast<int32_t>(XcdContiguousTile(blockIdx.x, gridDim.x));
    if (b >= a.B) {
        return;  // (no barrier anywhere below)
    }
    const BlockMeta m = a.meta[b];
    const int32_t nRows = m.nRows < 0 ? 0 : (m.nRows < kStreamRows ? m.nRows : kStreamRows);
    if (nRows == 0) {
        return;  // a block number that no row maps to
    }
    for (int i = lane; i < kStreamRows; i += kWave) {
        acc[i] = 0;
    }
    for (int32_t l = m.l0 + lane; l < m.l1; l += kWave) {
        const int32_t r = a.longRows[l] - m.row0;  // summed by phase 1 and SpmvLongRowSumKernel
        if (r >= 0 && r < nRows) {
            acc[r] = kJoinMark;
        }
    }
    struct Piece {
        Uint4 v[2], x[2];
        Uint2 f[2];
    };
    struct Sources {
        int32_t at[2];
    };
    const int32_t dBeg = m.dBeg, dEnd = m.dEnd;
    // Where the lane's two runs of four positions of the 512 from `start` sit in panel order.  A wavefront issues
    // its instructions in order: a load whose address waits for another load stalls everything behind it, so these
    // are asked for well before the loads that need them.  Positions behind the block's last: its last four again.
    auto sources = [&](int32_t start) {
        Sources src;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int32_t mine = start + s * kSub + lane * 4;
            const int32_t at = mine < dEnd ? mine : dEnd - 4;  // (a block in the loop has 8 positions at least)
            // (nothing here or in `fetch` may look at what a load brings: that would wait for it, and for every load
            // issued before it)
            src.at[s] = __builtin_nontemporal_load(a.src8 + (at >> 3));
        }
        return src;
    };
    auto fetch = [&](int32_t start, const Sources &from) {
        Piece piece;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int32_t mine = start + s * kSub + lane * 4;
            const int32_t at = mine < dEnd ? mine : dEnd - 4;
            // (in range whatever the table holds; the four loaded may run past the last entry into the 256 bytes
            // that xg has behind it: those are padding positions)
            int32_t src = from.at[s] + (at & 4);
            src = src < 0 ? 0 : (src < a.xgEntries ? src : a.xgEntries);
            piece.v[s] = LoadFourRaw(a.valD + at);
            piece.x[s] = *reinterpret_cast<const Uint4U *>(a.xg + src);
            piece.f[s] = __builtin_nontemporal_load(reinterpret_cast<const Uint2 *>(a.field + at));
        }
        return piece;
    };
    auto process = [&](const Piece &cur, int32_t start) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const uint32_t vr[4] = {cur.v[s].x, cur.v[s].y, cur.v[s].z, cur.v[s].w};
            const uint32_t xr[4] = {cur.x[s].x, cur.x[s].y, cur.x[s].z, cur.x[s].w};
            // positions behind the block's last (a lane then holds the block's last four again): padding
            const bool inside = start + s * kSub + lane * 4 < dEnd;
            const Uint2 fs = inside ? cur.f[s] : Uint2{kStreamPadRow * 0x10001u, kStreamPadRow * 0x10001u};
            const uint32_t fl[4] = {fs.x & 0xffffu, fs.x >> 16, fs.y & 0xffffu, fs.y >> 16};
            uint32_t row[4];
            AccT t[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                row[j] = fl[j] & 0x7ffu;
                t[j] = RawToAcc<AccT, kIntData>(vr[j]) * RawToAcc<AccT, kIntData>(xr[j]);
            }
            const uint32_t first = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row[0])));
            const bool mineSame = row[0] == first && row[1] == first && row[2] == first && row[3] == first;
            if (first != kStreamPadRow && __all(mineSame)) {
                // one row fills the 256 positions: its sum across the lanes in a fixed shape, added once
                AccT sum = (t[0] + t[1]) + (t[2] + t[3]);
#pragma unroll
                for (int off = kWave / 2; off > 0; off >>= 1) {
                    sum += __shfl_xor(sum, off);
                }
                if (lane == 0) {
                    StreamAdd<AccT>(acc, first, sum);
                }
                continue;
            }
            // The first turns: four instructions; then, where the 256 positions hold a row twice in one instruction
            // (most do: a row with many entries has some in every chunk), the later turns, and the 31st and later
            // of a row one lane at a time, in lane order.  A lane whose entry is not on adds to a slot of its own
            // behind the rows' sums instead (nobody reads it): an address select costs less than switching lanes
            // off and on again.
            uint32_t turn[4], latest = 0;
            const uint32_t idle = kStreamRows + lane;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool valid = row[j] != kStreamPadRow;
                turn[j] = valid ? fl[j] >> kStreamRoundShift : 0xffffu;  // (padding: no turn)
                latest = valid && turn[j] > latest ? turn[j] : latest;
                StreamAdd<AccT>(acc, turn[j] == 0 ? row[j] : idle, t[j]);
            }
            if (__any(latest != 0)) {
#pragma nounroll  // (the kernel's code has to stay inside the instruction cache)
                for (uint32_t r = 1; r < kStreamMaxRound; ++r) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        StreamAdd<AccT>(acc, turn[j] == r ? row[j] : idle, t[j]);
                    }
                    if (!__any(latest > r)) {
                        break;
                    }
                }
                if (__any(latest == kStreamMaxRound)) {
#pragma nounroll
                    for (int j = 0; j < 4; ++j) {
                        uint64_t late = __ballot(turn[j] == kStreamMaxRound);
                        while (late != 0) {
                            const int who = __builtin_ctzll(late);
                            if (lane == who) {
                                StreamAdd<AccT>(acc, row[j], t[j]);
                            }
                            late &= late - 1;
                        }
                    }
                }
            }
        }
    };
    if (dBeg < dEnd) {
        // A wavefront issues in order and its loads come back in order.  Piece n is asked for while piece n - 2 is
        // added up, its sources while piece n - 4 is (before that slot's own piece, so that waiting for them does not
        // wait for it): two pieces and two sets of sources are on their way at any time.  Four of each in turn, so
        // that no register a load fills is ever copied (a copy would wait for the load).  Every load is issued
        // whether or not its piece exists (past the end: on the block's last positions): with loads inside branches
        // the compiler can no longer tell which of them a use has to wait for, and waits for all.
        Sources src0 = sources(dBeg), src1 = sources(dBeg + kStep), src2 = sources(dBeg + 2 * kStep),
                src3 = sources(dBeg + 3 * kStep);
        Piece p0 = fetch(dBeg, src0), p1 = fetch(dBeg + kStep, src1), p2, p3;
#define OPSPARSE_STREAM_SLOT(pNow, pAhead, srcAhead, srcFar)      \
    srcFar = sources(start + 4 * kStep);                           \
    pAhead = fetch(start + 2 * kStep, srcAhead);                   \
    process(pNow, start);                                          \
    start += kStep;                                                \
    if (start >= dEnd) {                                           \
        break;                                                     \
    }
        for (int32_t start = dBeg;;) {
            OPSPARSE_STREAM_SLOT(p0, p2, src2, src0)
            OPSPARSE_STREAM_SLOT(p1, p3, src3, src1)
            OPSPARSE_STREAM_SLOT(p2, p0, src0, src2)
            OPSPARSE_STREAM_SLOT(p3, p1, src1, src3)
        }
#undef OPSPARSE_STREAM_SLOT
    }
    const AccT alpha = ReadAcc<AccT>(a.alpha), beta = ReadAcc<AccT>(a.beta);
    for (int32_t i = lane; i < nRows; i += kWave) {
        const uint64_t slot = acc[i];
        if (slot != kJoinMark) {
            StoreOut<OutT, AccT>(a.y, a.yIn, static_cast<int64_t>(m.row0) + i, SlotToAcc<AccT>(slot), alpha, beta);
        }
    }
}

// The long rows of the row blocks that hold more than kInBlockLongRows of them (longDeferred[l] != 0), a wavefront a
// row: y[row] = alpha * (the row's partial sums, added up as phase 2 does) + beta * yIn[row].
template <typename OutT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmvLongRowSumKernel(
    const int32_t *__restrict__ header, const int32_t *__restrict__ longRows, const int32_t *__restrict__ longDeferred,
    const uint64_t *__restrict__ longPartial, int32_t P, OutT *__restrict__ y, const OutT *__restrict__ yIn,
    OpsparseScalar alphaS, OpsparseScalar betaS)
{
    const int lane = threadIdx.x % kWave;
    const int32_t l = static_cast<int32_t>(blockIdx.x) * (kBlockThreads / kWave) + threadIdx.x / kWave;
    if (l >= header[1] || longDeferred[l] == 0) {
        return;
    }
    const AccT sum = LongRowTotal<AccT>(longPartial + static_cast<int64_t>(l) * P, P, lane);
    if (lane == 0) {
        StoreOut<OutT, AccT>(y, yIn, longRows[l], sum, ReadAcc<AccT>(alphaS), ReadAcc<AccT>(betaS));
    }
}

// ------------------------------------------------------------------- host

namespace {

int32_t ValueBytes(int32_t valueType) { return valueType == OPSPARSE_F16 || valueType == OPSPARSE_BF16 ? 2 : 4; }

struct BlockedLayout {
    int32_t P, B, window, passes;
    bool streamed;      // row blocks of 2^10 rows that a wavefront streams (values kept in block order), not windowed
    int32_t rowLog;     // rows of a block at most: 2^rowLog
    int64_t valDOff;    // streamed: the values in block order
    int64_t padded;     // upper bound of the positions in block order
    // op(A) = A^T: the CSR arrays of A^T (= the CSC arrays of A), and with live values the entry of A behind each
    int64_t cscPtrOff, cscIndOff, cscValOff, permOff;
    // used by every launch (the first `resident` bytes)
    int64_t colLocalOff, xgOff, slotOff, src8Off, metaOff, panelStartOff, rowBitsOff, bitPrefixOff, ordRowOff, emptyRowsOff;
    int64_t shortOffsetsOff;  // row offsets without the entries of long rows (with room for long rows, or frozen values)
    int64_t valSOff;          // frozen values: the values phase 2 reads, in row order without those of long rows
    // long rows: row ids, first entry of every (long row, panel) piece, sum of every piece
    int32_t longMinRow;   // rows of at least this many entries are candidates (0: no long-row path)
    int32_t maxLong;      // room for this many
    bool frozenLong;      // the long entries are stored a second time, with their values
    int64_t longRowsOff, longChunkOff, longPartialOff, longDeferredOff;
    int64_t resident;
    // preprocessing only
    int64_t keys0Off, keys1Off, pos0Off, pos1Off, rowOfPosOff, longBeforeOff, longCsrOff, tableOff, scratchOff;
    int64_t srcStartOff, dstStartOff, blockRowOff, blockShortOff, longFirstOff, emptyFlagsOff;
    int64_t transposeWsOff, transposeWsBytes, iotaOff;
    int64_t bytes;
};

// Layout for a product with `rows` outputs and `cols` inputs (op(A) = A^T: the columns of A are the outputs).
// 0 panels: the layout does not apply.
BlockedLayout MakeBlockedLayout(int64_t rows, int64_t cols, int64_t nnz, bool transposed, bool live, int32_t valueType)
{
    BlockedLayout l{};
    if (rows <= 0 || cols <= 0 || nnz <= 0 || nnz > INT32_MAX || rows >= INT32_MAX || cols > INT32_MAX) {
        return l;
    }
    const int64_t P = (cols + kPanelCols - 1) >> kPanelLog;
    static const int64_t minCols = [] {  // tuning override
        const char *env = std::getenv("OPS_SPARSE_BLOCKED_MIN_COLS");
        return env != nullptr ? std::atoll(env) : kMinCols;
    }();
    if (cols <= minCols || nnz < kMinEntries || P > kMaxPanels) {
        return l;
    }
    static const int64_t cutEnv = [] {  // tuning override: the entry window the row blocks are cut by
        const char *env = std::getenv("OPS_SPARSE_BLOCKED_WINDOW");
        return env != nullptr ? std::atoll(env) : 0;
    }();
    int64_t window = cutEnv > 0 ? cutEnv : kRowsWindow * 7 / 8;
    window = window > kMaxBlockEntries / 2 ? kMaxBlockEntries / 2 : window;
    // Values that the layout keeps (frozen values, either op(A)) are kept in block order and streamed by a wavefront
    // a block; values read where the caller has them need the windowed blocks, which read them in row order.
    const bool noStream = std::getenv("OPS_SPARSE_BLOCKED_NO_STREAM") != nullptr;  // tuning switch
    l.streamed = !live && !noStream;
    if (l.streamed) {
        // Streamed blocks are cut by their rows; the entry cut is there for matrices of few, long rows, which would
        // otherwise make fewer blocks than the chip has wavefronts: about 8192 blocks of 4096 entries at least.
        const int64_t byRows = rows >> kStreamRowLog;
        int64_t cut = byRows >= kStreamBlocksWanted / 2 ? kStreamWindow : nnz / (kStreamBlocksWanted - byRows);
        cut = cut < kStreamMinWindow ? kStreamMinWindow : (cut > kStreamWindow ? kStreamWindow : cut);
        cut = cutEnv > 0 ? cutEnv : cut;
        // They pay where a (panel, block) chunk has 16 entries on average (smaller ones are mostly padding, and a
        // block of 2^10 rows has a quarter of the entries of a windowed one: many panels and few entries a row
        // are the windowed blocks' case) and where a row does not put more than 16 entries into a panel on
        // average (such rows meet themselves in every instruction of the stream: 200 000 rows of 300 entries over
        // 10 panels 326 us streamed, 247 us windowed; over 19 panels 234 against 254).
        const int64_t blocks = ((rows + kStreamRows - 1) >> kStreamRowLog) + nnz / cut + 1;
        if (nnz / (P * blocks) < kStreamMinChunkEntries || nnz / rows / P > kStreamMaxRowPanelEntries) {
            l.streamed = false;
        } else {
            window = cut;
        }
    }
    l.rowLog = l.streamed ? kStreamRowLog : kRowBlockLog;
    // The values a launch reads: the caller's own (live values, op(A) = A), the transposed copy (op(A) = A^T), or,
    // for op(A) = A with frozen values, a compact copy without the long rows' values, whose entries are stored a
    // second time with their values.
    const bool frozenCopy = !live && !transposed;
    const bool noLong = std::getenv("OPS_SPARSE_BLOCKED_NO_LONG_ROWS") != nullptr;
    if (!noLong) {
        static const int64_t chunkMean = [] {  // tuning override: entries a long row has per panel at least, on average
            const char *env = std::getenv("OPS_SPARSE_BLOCKED_LONG_MEAN");
            const int64_t v = env != nullptr ? std::atoll(env) : 0;
            return v;
        }();
        // read in place, the pieces are scattered over the arrays and pay from 64 entries (256 bytes of either
        // array); stored again panel by panel they stream
        const int64_t mean = chunkMean > 0 ? chunkMean : (frozenCopy ? kLongChunkMeanFrozen : kLongChunkMean);
        const int64_t floor = frozenCopy ? kLongMinRowFrozen : kLongMinRow;
        int64_t minRow = mean * P > floor ? mean * P : floor;
        minRow = minRow > kLongMaxMinRow ? kLongMaxMinRow : minRow;
        if (frozenCopy && nnz / minRow > 65535) {
            minRow = nnz / 65535 + 1;  // the stored long entries keep their row's number, below nnz / minRow, in 16 bits
        }
        if (minRow <= INT32_MAX && nnz / minRow > 0) {
            l.longMinRow = static_cast<int32_t>(minRow);
            l.maxLong = static_cast<int32_t>(nnz / minRow);
            l.frozenLong = frozenCopy;
        }
    }
    // a block ends behind 2^rowLog rows, behind `window` entries and, where the values are read in place in row
    // order, behind a long row
    const bool cutBehindLong = !l.frozenLong && !l.streamed;
    const int64_t B = ((rows + (int64_t{1} << l.rowLog) - 1) >> l.rowLog) + nnz / window + 1 + (cutBehindLong ? l.maxLong : 0);
    if (P * B + 1 > INT32_MAX || nnz + kLaneEntries * P * B > INT32_MAX - 65536 ||
        nnz / (P * (B - (cutBehindLong ? l.maxLong : 0))) < kMinChunkEntries) {
        return BlockedLayout{};
    }
    l.P = static_cast<int32_t>(P);
    l.B = static_cast<int32_t>(B);
    l.window = static_cast<int32_t>(window);
    int bits = 0;  // the long rows' entries sort as one more panel behind the others, or (stored again) as P more
    while ((int64_t{1} << bits) < (l.maxLong == 0 ? P : (l.frozenLong ? 2 * P : P + 1))) {
        ++bits;
    }
    l.passes = (bits + 3) / 4;
    l.passes = l.passes < 1 ? 1 : l.passes;
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t vb = ValueBytes(valueType);
    int64_t off = 256;  // header: status word of the analysis, counts
    if (transposed) {
        l.cscPtrOff = off; off += align(4 * (rows + 1));
        l.cscIndOff = off; off += align(4 * nnz + 16);
        l.cscValOff = off; off += align(vb * nnz + 16);
        l.permOff = off; off += live ? align(4 * nnz) : 0;
    }
    const int64_t padded = nnz + kLaneEntries * P * B;  // every chunk padded to a multiple of kLaneEntries
    l.padded = padded;
    l.colLocalOff = off; off += align(2 * nnz + 8);
    l.xgOff = off; off += align(4 * nnz) + 256;  // a lane's 16-byte loads of xg may run 7 entries past a chunk
    l.slotOff = off; off += align(2 * padded + 16);  // (the long entries' row numbers behind the block order)
    l.src8Off = off; off += align(4 * (padded / kLaneEntries + 2));
    l.metaOff = off; off += align(static_cast<int64_t>(sizeof(BlockMeta)) * (B + 1));
    l.panelStartOff = off; off += align(4 * (P + 1));
    // (streamed blocks need no row tables, write the rows without entries themselves and keep their values in
    // block order)
    l.rowBitsOff = off; off += l.streamed ? 0 : align(4 * (nnz / 32 + 8 * B + 16));
    l.bitPrefixOff = off; off += l.streamed ? 0 : align(2 * (nnz / 32 + 8 * B + 16));
    l.ordRowOff = off; off += l.streamed ? 0 : align(2 * (rows + 16 * B + 32));
    l.emptyRowsOff = off; off += l.streamed ? 0 : align(4 * rows);
    l.shortOffsetsOff = off; off += (l.maxLong > 0 || frozenCopy) && !l.streamed ? align(4 * (rows + 1)) : 0;
    l.valSOff = off; off += frozenCopy && !l.streamed ? align(vb * nnz + 16) : 0;
    l.valDOff = off; off += l.streamed ? align(vb * padded + 64) : 0;
    l.longRowsOff = off; off += align(4 * static_cast<int64_t>(l.maxLong));
    // in place: first entry of piece (p, l) in the CSR arrays at [p * maxLong + l], p = 0 .. P; stored again: in the
    // sorted order at [p * (maxLong + 1) + l], l = 0 .. L
    l.longChunkOff = off; off += align(4 * (static_cast<int64_t>(l.maxLong) + 1) * (P + 1));
    l.longPartialOff = off; off += align(8 * static_cast<int64_t>(l.maxLong) * P);
    l.longDeferredOff = off; off += align(4 * static_cast<int64_t>(l.maxLong));
    l.resident = off;
    const int64_t scratch0 = off;
    l.keys0Off = off; off += align(4 * nnz);
    l.keys1Off = off; off += align(4 * nnz);
    l.pos0Off = off; off += align(4 * nnz);
    l.pos1Off = off; off += align(4 * nnz);
    l.rowOfPosOff = off; off += align(4 * nnz);
    l.longBeforeOff = off; off += l.maxLong > 0 ? align(4 * rows) : 0;  // long rows among rows 0 .. r
    l.longCsrOff = off; off += l.frozenLong ? align(4 * static_cast<int64_t>(l.maxLong) * (P + 1)) : 0;
    l.srcStartOff = off; off += align(4 * (P * B + 1));
    l.dstStartOff = off; off += align(4 * (P * B + 1));
    l.blockRowOff = off; off += align(4 * (B + 1));
    l.blockShortOff = off; off += align(4 * (B + 1));
    l.longFirstOff = off; off += l.maxLong > 0 ? align(4 * (B + 1)) : 0;
    l.emptyFlagsOff = off; off += l.streamed ? 0 : align(4 * rows);
    if (l.streamed && l.maxLong > 0) {
        l.shortOffsetsOff = off; off += align(4 * (rows + 1));  // (only the analysis reads them)
    }
    l.tableOff = off; off += align(4 * RadixTableInts(nnz));
    int64_t scan = ScanScratchInts(RadixTableInts(nnz));
    scan = ScanScratchInts(P * B + 1) > scan ? ScanScratchInts(P * B + 1) : scan;
    scan = ScanScratchInts(rows + 1) > scan ? ScanScratchInts(rows + 1) : scan;
    l.scratchOff = off; off += align(4 * scan);
    if (transposed) {
        // the transposition comes first and shares the scratch of what follows it
        l.transposeWsOff = scratch0;
        l.transposeWsBytes = static_cast<int64_t>(opsparse_csr2csc_workspace_bytes(cols, rows, nnz));
        l.iotaOff = scratch0 + align(l.transposeWsBytes);
        const int64_t end = l.iotaOff + (live ? align(4 * nnz) : 0);
        off = end > off ? end : off;
    }
    l.bytes = off;
    return l;
}

// Frozen values: the number of its long row, for a long entry at position i of the sorted order, is kept at
// slot16[i + LongRowOfShift]: the block order, which that array serves, ends in front of it (it holds the short
// entries and at most 8 positions of padding for each of the P x B chunks).
int64_t LongRowOfShift(const BlockedLayout &l) { return static_cast<int64_t>(kLaneEntries) * l.P * l.B; }

uint32_t GridOf(int64_t items, int64_t perBlock, int64_t cap)
{
    int64_t g = (items + perBlock - 1) / perBlock;
    g = g < 1 ? 1 : g;
    return static_cast<uint32_t>(g > cap ? cap : g);
}

int32_t ValueTypeOfFlags(int32_t flags)
{
    return (flags & OPSPARSE_BLOCKED_VALUES_F16) != 0    ? OPSPARSE_F16
           : (flags & OPSPARSE_BLOCKED_VALUES_BF16) != 0 ? OPSPARSE_BF16
           : (flags & OPSPARSE_BLOCKED_VALUES_I32) != 0  ? OPSPARSE_I32
                                                         : OPSPARSE_F32;
}

template <typename Fn>
int WithValueType(int32_t valueType, Fn &&fn)
{
    switch (valueType) {
        case OPSPARSE_F32: return fn(float{});
        case OPSPARSE_F16: return fn(Half{});
        case OPSPARSE_BF16: return fn(Bf16{});
        case OPSPARSE_I32: return fn(int32_t{});
        default: return OPSPARSE_E_UNSUPPORTED;
    }
}

}  // namespace

// valType: the type of the caller's values and of x (OPSPARSE_F32 / F16 / BF16 / I32); outType that of y: fp32, or
// the values' own type.  a.rows outputs, a.cols inputs: the caller has exchanged them for op(A) = A^T.
int LaunchBlocked(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType, int32_t computeIsInt)
{
    if (plan.valueType != valType) {
        return OPSPARSE_E_INVALID;  // the plan was made for values of another type
    }
    if ((outType != OPSPARSE_F32 && outType != valType) || (computeIsInt != 0) != (outType == OPSPARSE_I32)) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    const bool transposed = plan.transposed != 0, live = plan.liveValues != 0;
    const BlockedLayout l = MakeBlockedLayout(a.rows, a.cols, a.nnz, transposed, live, valType);
    if (l.P == 0 || plan.numPanels != l.P || plan.numRowBlocks != l.B || plan.entryWindow != l.window) {
        return OPSPARSE_E_INVALID;
    }
    // a launch touches the first `resident` bytes only: the tail served the analysis and may have been handed back
    if (a.ws == nullptr || static_cast<int64_t>(a.wsBytes) < l.resident || plan.bytes != l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    if (plan.numEmptyRows < 0 || plan.numEmptyRows > a.rows || plan.numLongRows < 0 || plan.numLongRows > l.maxLong) {
        return OPSPARSE_E_INVALID;
    }
    if ((plan.streamedBlocks != 0) != l.streamed) {
        return OPSPARSE_E_INVALID;
    }
    auto *base = static_cast<unsigned char *>(a.ws);
    auto ints = [&](int64_t off) { return reinterpret_cast<const int32_t *>(base + off); };
    const auto *colLocal = reinterpret_cast<const uint16_t *>(base + l.colLocalOff);
    const auto *slot16 = reinterpret_cast<const uint16_t *>(base + l.slotOff);
    auto *xg = reinterpret_cast<uint32_t *>(base + l.xgOff);
    const bool frozenCopy = !live && !transposed;
    if (live && !transposed && a.vals == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    if (transposed && live && a.vals == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    // the arrays the kernels read the matrix from
    const int32_t *colInd = transposed ? ints(l.cscIndOff) : a.colInd;
    const void *vals = transposed ? base + l.cscValOff : (frozenCopy ? base + l.valSOff : a.vals);  // (windowed blocks,
                                                                                                    // in-place long rows)
    const bool longRows = plan.numLongRows > 0;
    if (longRows && !l.frozenLong && colInd == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    const int32_t *header = longRows ? ints(0) : nullptr;
    auto *longPartial = reinterpret_cast<uint64_t *>(base + l.longPartialOff);
    // Few panels: several workgroups per panel, so that every CU has one.
    const int32_t splits = l.P >= 192 ? 1 : (256 + l.P - 1) / l.P;
    return WithValueType(valType, [&](auto tag) {
        using ValT = decltype(tag);
        auto run = [&](auto accTag, auto outTag) {
            using AccT = decltype(accTag);
            using OutT = decltype(outTag);
            if (transposed && live) {
                hipLaunchKernelGGL(PermuteValuesKernel<ValT>, dim3(GridOf(a.nnz, kBlockThreads * 4, 65536)),
                                   dim3(kBlockThreads), 0, a.stream, static_cast<const ValT *>(a.vals), ints(l.permOff),
                                   a.nnz, reinterpret_cast<ValT *>(base + l.cscValOff));
            }
            auto gather = [&](auto longSorted) {
                constexpr bool kSorted = decltype(longSorted)::value;
                hipLaunchKernelGGL((SpmvBlockGatherKernel<kSorted, ValT, AccT>), dim3(static_cast<uint32_t>(l.P) * splits),
                                   dim3(kBlkThreads), 0, a.stream, colLocal, static_cast<const ValT *>(a.x), xg,
                                   ints(l.panelStartOff), a.cols, splits, header, ints(l.longChunkOff), colInd,
                                   static_cast<const ValT *>(kSorted ? nullptr : vals), a.nnz, l.P, l.maxLong,
                                   kSorted ? slot16 + LongRowOfShift(l) : static_cast<const uint16_t *>(nullptr), longPartial);
            };
            if (longRows && l.frozenLong) {
                gather(std::true_type{});
            } else {
                gather(std::false_type{});  // (without long rows nothing of the matrix arrays is read)
            }
            if (l.streamed) {
                BlockStreamArgs<ValT, OutT> args{};
                args.xg = xg;
                args.field = slot16;
                args.src8 = ints(l.src8Off);
                args.meta = reinterpret_cast<const BlockMeta *>(base + l.metaOff);
                args.valD = reinterpret_cast<const ValT *>(base + l.valDOff);
                args.y = static_cast<OutT *>(a.y);
                args.yIn = static_cast<const OutT *>(a.yIn);
                args.alpha = a.alpha;
                args.beta = a.beta;
                args.longRows = ints(l.longRowsOff);
                args.B = l.B;
                args.xgEntries = static_cast<int32_t>(a.nnz);
                hipLaunchKernelGGL((SpmvBlockStreamKernel<ValT, OutT, AccT>), dim3(static_cast<uint32_t>(l.B)),
                                   dim3(kStreamThreads), 0, a.stream, args);
                if (longRows) {  // (every long row is left to this kernel)
                    constexpr int kRowsPerBlock = kBlockThreads / kWave;
                    hipLaunchKernelGGL((SpmvLongRowSumKernel<OutT, AccT>),
                                       dim3((plan.numLongRows + kRowsPerBlock - 1) / kRowsPerBlock), dim3(kBlockThreads),
                                       0, a.stream, header, ints(l.longRowsOff), ints(l.longDeferredOff), longPartial,
                                       l.P, static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.alpha, a.beta);
                }
                return CheckLaunch();
            }
            BlockRowsArgs<ValT, OutT> args{};
            args.xg = xg;
            args.slot16 = slot16;
            args.src8 = ints(l.src8Off);
            args.meta = reinterpret_cast<const BlockMeta *>(base + l.metaOff);
            args.rowBits = reinterpret_cast<const uint32_t *>(base + l.rowBitsOff);
            args.bitPrefix = reinterpret_cast<const uint16_t *>(base + l.bitPrefixOff);
            args.ordRow = reinterpret_cast<const uint16_t *>(base + l.ordRowOff);
            args.vals = static_cast<const ValT *>(vals);
            args.y = static_cast<OutT *>(a.y);
            args.yIn = static_cast<const OutT *>(a.yIn);
            args.alpha = a.alpha;
            args.beta = a.beta;
            args.longRows = ints(l.longRowsOff);
            args.longPartial = longPartial;
            args.P = l.P;
            args.xgEntries = static_cast<int32_t>(a.nnz);
            args.valEntries = a.nnz;  // (the compact copy of a frozen plan has room for as many, and 16 bytes more)
            hipLaunchKernelGGL((SpmvBlockRowsKernel<kRowsThreads, ValT, OutT, AccT>), dim3(static_cast<uint32_t>(l.B)),
                               dim3(kRowsThreads), 0, a.stream, args);
            if (plan.numEmptyRows > 0) {
                hipLaunchKernelGGL((SpmvEmptyRowsKernel<OutT, AccT>),
                                   dim3((plan.numEmptyRows + kBlockThreads - 1) / kBlockThreads), dim3(kBlockThreads), 0,
                                   a.stream, ints(l.emptyRowsOff), plan.numEmptyRows, a.rows, static_cast<OutT *>(a.y),
                                   static_cast<const OutT *>(a.yIn), a.alpha, a.beta);
            }
            if (longRows && plan.numDeferredLongRows > 0) {
                constexpr int kRowsPerBlock = kBlockThreads / kWave;
                hipLaunchKernelGGL((SpmvLongRowSumKernel<OutT, AccT>),
                                   dim3((plan.numLongRows + kRowsPerBlock - 1) / kRowsPerBlock), dim3(kBlockThreads), 0,
                                   a.stream, header, ints(l.longRowsOff), ints(l.longDeferredOff), longPartial, l.P,
                                   static_cast<OutT *>(a.y), static_cast<const OutT *>(a.yIn), a.alpha, a.beta);
            }
            return CheckLaunch();
        };
        if constexpr (std::is_same<ValT, int32_t>::value) {
            return computeIsInt != 0 ? run(uint32_t{}, int32_t{}) : run(double{}, float{});
        } else if constexpr (std::is_same<ValT, float>::value) {
            return run(double{}, float{});
        } else {
            return outType == OPSPARSE_F32 ? run(double{}, float{}) : run(double{}, ValT{});
        }
    });
}

}  // namespace opsparse

using namespace opsparse;

extern "C" {

size_t opsparse_spmv_csr_blocked_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags)
{
    const bool t = (flags & OPSPARSE_BLOCKED_TRANSPOSE) != 0, live = (flags & OPSPARSE_BLOCKED_LIVE_VALUES) != 0;
    const int32_t vt = ValueTypeOfFlags(flags);
    return static_cast<size_t>((t ? MakeBlockedLayout(cols, rows, nnz, true, live, vt)
                                  : MakeBlockedLayout(rows, cols, nnz, false, live, vt)).bytes);
}

size_t opsparse_spmv_csr_blocked_resident_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags)
{
    const bool t = (flags & OPSPARSE_BLOCKED_TRANSPOSE) != 0, live = (flags & OPSPARSE_BLOCKED_LIVE_VALUES) != 0;
    const int32_t vt = ValueTypeOfFlags(flags);
    return static_cast<size_t>((t ? MakeBlockedLayout(cols, rows, nnz, true, live, vt)
                                  : MakeBlockedLayout(rows, cols, nnz, false, live, vt)).resident);
}

int opsparse_spmv_csr_blocked_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                      int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                      size_t workspaceBytes, void *scratchSpace, size_t scratchBytes,
                                      OpsparseSpmvPlan *plan, void *stream)
{
    if (plan == nullptr || rowOffsets == nullptr || colInd == nullptr || csrValues == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    const bool transposed = (flags & OPSPARSE_BLOCKED_TRANSPOSE) != 0, live = (flags & OPSPARSE_BLOCKED_LIVE_VALUES) != 0;
    const int32_t valueType = ValueTypeOfFlags(flags);
    const int64_t outputs = transposed ? cols : rows, inputs = transposed ? rows : cols;
    const BlockedLayout l = MakeBlockedLayout(outputs, inputs, nnz, transposed, live, valueType);
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
    // status, number of long rows, their entries, entries of the largest block, long rows summed on their own
    LaunchFillI32(status, 8, 0, s);
    if (transposed) {
        // The CSC arrays of A are the CSR arrays of A^T: from here on the matrix is that copy.
        hipLaunchKernelGGL(CheckColumnsKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s, colInd,
                           nnz, cols, status);
        int32_t bad = 0;
        if (hipMemcpyAsync(&bad, status, sizeof(bad), hipMemcpyDeviceToHost, s) != hipSuccess ||
            hipStreamSynchronize(s) != hipSuccess) {
            (void)hipGetLastError();
            return OPSPARSE_E_LAUNCH;
        }
        if (bad != 0) {
            return OPSPARSE_E_INVALID;  // a column index outside [0, cols)
        }
        const void *srcVals = csrValues;
        void *dstVals = at(l.cscValOff);
        int32_t vb = ValueBytes(valueType);
        if (live) {
            // what travels with an entry is its position in the caller's arrays; the values follow it at every call
            hipLaunchKernelGGL(IotaKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                               ints(l.iotaOff), nnz);
            srcVals = ints(l.iotaOff);
            dstVals = ints(l.permOff);
            vb = 4;
        }
        const int rc = opsparse_csr2csc_launch(rows, cols, nnz, srcVals, rowOffsets, colInd, dstVals, ints(l.cscPtrOff),
                                               ints(l.cscIndOff), vb, 0, at(l.transposeWsOff),
                                               static_cast<size_t>(l.transposeWsBytes), s);
        if (rc != OPSPARSE_OK) {
            return rc;
        }
        rowOffsets = ints(l.cscPtrOff);
        colInd = ints(l.cscIndOff);
        csrValues = at(l.cscValOff);  // (live values: filled at every call; the analysis reads no value then)
    }
    // From here on: `outputs` rows, `inputs` columns, the arrays rowOffsets / colInd / csrValues.
    const bool frozenCopy = !live && !transposed;
    int32_t *keys[2] = {ints(l.keys0Off), ints(l.keys1Off)};
    int32_t *poss[2] = {ints(l.pos0Off), ints(l.pos1Off)};
    int32_t *rowOfPos = ints(l.rowOfPosOff), *table = ints(l.tableOff), *scratch = ints(l.scratchOff);
    int32_t *srcStart = ints(l.srcStartOff), *dstStart = ints(l.dstStartOff);
    int32_t *blockRow = ints(l.blockRowOff);
    auto *colLocal = reinterpret_cast<uint16_t *>(at(l.colLocalOff));
    auto *slot16 = reinterpret_cast<uint16_t *>(at(l.slotOff));

    LaunchExpandRows(rowOffsets, outputs, nnz, 0, rowOfPos, s);
    if (!l.streamed) {
        // the rows without entries, which the windowed row blocks do not see
        int32_t *flags = ints(l.emptyFlagsOff);
        hipLaunchKernelGGL(EmptyRowFlagsKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, outputs, flags);
        LaunchInclusiveScanI32(flags, flags, outputs, 0, scratch, s);
        hipLaunchKernelGGL(EmptyRowListKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           flags, outputs, ints(l.emptyRowsOff), status);
    }
    const int32_t *offsets = rowOffsets;
    int32_t *longBefore = nullptr;
    if (l.maxLong > 0) {
        // Long rows: candidates by length, checked for ascending columns inside [0, cols), numbered, listed.
        longBefore = ints(l.longBeforeOff);
        hipLaunchKernelGGL(LongRowFlagsKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, outputs, l.longMinRow, longBefore);
        hipLaunchKernelGGL(LongRowCheckKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                           rowOffsets, colInd, rowOfPos, nnz, inputs, longBefore);
        LaunchInclusiveScanI32(longBefore, longBefore, outputs, 0, scratch, s);
        hipLaunchKernelGGL(LongRowListKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, longBefore, outputs, l.maxLong, ints(l.longRowsOff), status);
        hipLaunchKernelGGL(LongRowChunksKernel, dim3(GridOf(static_cast<int64_t>(l.maxLong) * (l.P + 1), kBlockThreads, 4096)),
                           dim3(kBlockThreads), 0, s, rowOffsets, colInd, ints(l.longRowsOff), status, l.P, l.maxLong,
                           ints(l.frozenLong ? l.longCsrOff : l.longChunkOff));
        int32_t *shortOffsets = ints(l.shortOffsetsOff);
        hipLaunchKernelGGL(LongRowEntriesKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, longBefore, outputs, shortOffsets);
        LaunchInclusiveScanI32(shortOffsets, shortOffsets, outputs + 1, 0, scratch, s);
        hipLaunchKernelGGL(ShortOffsetsKernel, dim3(GridOf(outputs + 1, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           rowOffsets, outputs, shortOffsets);
        offsets = shortOffsets;  // the row blocks are cut by the entries that stay
    } else if (frozenCopy && !l.streamed) {
        // (a plan with frozen values reads nothing of the caller's arrays at the launches)
        if (hipMemcpyAsync(ints(l.shortOffsetsOff), rowOffsets, sizeof(int32_t) * static_cast<size_t>(outputs + 1),
                           hipMemcpyDeviceToDevice, s) != hipSuccess) {
            (void)hipGetLastError();
            return OPSPARSE_E_LAUNCH;
        }
        offsets = ints(l.shortOffsetsOff);
    }
    // where the values are read in place a long row ends its block, so that a block's other entries are one piece
    const int32_t *cutBehind = (longBefore != nullptr && !l.frozenLong && !l.streamed) ? longBefore : nullptr;
    // Entries in (panel, original position) order: stable 4-bit radix passes over the panel number.
    const int32_t *firstKeys = colInd;
    if (longBefore != nullptr) {
        hipLaunchKernelGGL(LongRowKeysKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s, colInd,
                           rowOfPos, longBefore, nnz, static_cast<int32_t>(l.P) << kPanelLog, l.frozenLong ? 1 : 0, keys[1]);
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
    const int32_t *pos = poss[cur];
    int32_t *chunkKey = keys[1 - cur], *rowOfSrc = poss[1 - cur];
    hipLaunchKernelGGL(BlockedChunkKeysKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                       keys[cur], pos, rowOfPos, offsets, nnz, inputs, l.B, l.window, longBefore,
                       cutBehind != nullptr ? 1 : 0, l.rowLog, colLocal, chunkKey, rowOfSrc, status);
    if (longBefore != nullptr && l.frozenLong) {
        hipLaunchKernelGGL(LongRowPanelsKernel, dim3(GridOf(l.P, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           keys[cur], nnz, l.P, l.maxLong, static_cast<int32_t>(l.P) << kPanelLog, ints(l.longChunkOff));
        hipLaunchKernelGGL(LongRowPiecesKernel, dim3(GridOf(static_cast<int64_t>(l.maxLong) * l.P, kBlockThreads, 8192)),
                           dim3(kBlockThreads), 0, s, pos, nnz, ints(l.longCsrOff), status, l.P, l.maxLong,
                           ints(l.longChunkOff));
    }
    int32_t head[3] = {0, 0, 0};  // status, long rows, their entries
    if (hipMemcpyAsync(head, status, sizeof(head), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    if (head[0] != 0) {
        return OPSPARSE_E_INVALID;  // a column index outside [0, cols)
    }
    const int64_t chunks = static_cast<int64_t>(l.P) * l.B;
    LaunchIndicesToOffsets(chunkKey, nnz, chunks, 0, srcStart, scratch, s);
    hipLaunchKernelGGL(BlockedTablesKernel, dim3(GridOf(chunks, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                       srcStart, l.P, l.B, dstStart);
    LaunchInclusiveScanI32(dstStart + 1, dstStart + 1, chunks, 0, scratch, s);
    // padding positions: the slot kPadSlot, or the row field kStreamPadRow
    LaunchFillI32(reinterpret_cast<int32_t *>(slot16), (l.padded + 1) / 2,
                  static_cast<int32_t>((l.streamed ? kStreamPadRow : kPadSlot) * 0x10001u), s);
    LaunchFillI32(blockRow, l.B + 1, static_cast<int32_t>(outputs), s);
    hipLaunchKernelGGL(BlockedRowBlocksKernel, dim3(GridOf(outputs, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                       offsets, static_cast<int32_t>(outputs), l.window, l.B, cutBehind, l.rowLog, blockRow);
    if (longBefore != nullptr) {
        hipLaunchKernelGGL(BlockedLongFirstKernel, dim3(GridOf(l.B + 1, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                           s, blockRow, longBefore, l.B, ints(l.longFirstOff));
        hipLaunchKernelGGL(BlockedLongDeferKernel, dim3(GridOf(l.B, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0, s,
                           ints(l.longFirstOff), l.B, l.streamed ? 1 : 0, ints(l.longDeferredOff), status);
    }
    const int64_t tableItems = (l.B > l.P ? l.B : l.P) + 1;
    hipLaunchKernelGGL(BlockedBlockTablesKernel, dim3(GridOf(tableItems, kBlockThreads, INT32_MAX)), dim3(kBlockThreads), 0,
                       s, offsets, frozenCopy || l.streamed ? offsets : rowOffsets, blockRow, dstStart, srcStart,
                       longBefore != nullptr ? ints(l.longFirstOff) : nullptr, l.P, l.B, ints(l.blockShortOff),
                       reinterpret_cast<BlockMeta *>(at(l.metaOff)), ints(l.panelStartOff), status);
    if (!l.streamed) {
        hipLaunchKernelGGL(BlockedRowTablesKernel, dim3(static_cast<uint32_t>(l.B)), dim3(kTableThreads), 0, s,
                           reinterpret_cast<const BlockMeta *>(at(l.metaOff)), offsets,
                           reinterpret_cast<uint32_t *>(at(l.rowBitsOff)),
                           reinterpret_cast<uint16_t *>(at(l.bitPrefixOff)),
                           reinterpret_cast<uint16_t *>(at(l.ordRowOff)));
    }
    const int rcScatter = WithValueType(valueType, [&](auto tag) {
        using ValT = decltype(tag);
        if (l.streamed) {
            hipLaunchKernelGGL(StreamScatterKernel<ValT>, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0,
                               s, pos, rowOfSrc, chunkKey, static_cast<const ValT *>(csrValues), srcStart, dstStart,
                               blockRow, nnz, l.P, l.B, slot16, ints(l.src8Off),
                               reinterpret_cast<ValT *>(at(l.valDOff)), static_cast<int32_t *>(nullptr),
                               longBefore != nullptr && l.frozenLong ? reinterpret_cast<uint32_t *>(at(l.xgOff))
                                                                     : nullptr,
                               slot16 + LongRowOfShift(l), longBefore);
            hipLaunchKernelGGL(StreamTurnsKernel, dim3(static_cast<uint32_t>(l.B)), dim3(kTurnThreads), 0, s,
                               reinterpret_cast<const BlockMeta *>(at(l.metaOff)), slot16);
            return OPSPARSE_OK;
        }
        hipLaunchKernelGGL(BlockedScatterKernel<ValT>, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s,
                           pos, rowOfSrc, chunkKey, static_cast<const ValT *>(csrValues), rowOffsets, offsets, srcStart,
                           dstStart, ints(l.blockShortOff), nnz, l.P, l.B, slot16, ints(l.src8Off),
                           frozenCopy ? reinterpret_cast<ValT *>(at(l.valSOff)) : nullptr,
                           longBefore != nullptr && l.frozenLong ? reinterpret_cast<uint32_t *>(at(l.xgOff)) : nullptr,
                           slot16 + LongRowOfShift(l), longBefore);
        return OPSPARSE_OK;
    });
    if (rcScatter != OPSPARSE_OK) {
        return rcScatter;
    }
    int32_t tail[3] = {0, 0, 0};  // entries of the largest row block, long rows summed on their own, rows without entries
    if (hipMemcpyAsync(tail, status + 3, sizeof(tail), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    if (CheckLaunch() != OPSPARSE_OK) {
        return OPSPARSE_E_LAUNCH;
    }
    if (!l.streamed && tail[0] > kMaxBlockEntries) {
        return OPSPARSE_E_UNSUPPORTED;  // a row too long for a block's 16-bit slots that cannot go the long rows' way
    }
    OpsparseSpmvPlan p{};
    p.kernel = OPSPARSE_SPMV_BLOCKED_GATHER;
    p.numPanels = l.P;
    p.panelShift = kPanelLog;
    p.numRowBlocks = l.B;
    p.entryWindow = l.window;
    p.transposed = transposed ? 1 : 0;
    p.liveValues = live ? 1 : 0;
    p.valueType = valueType;
    p.numDeferredLongRows = tail[1];
    p.numEmptyRows = tail[2];
    p.streamedBlocks = l.streamed ? 1 : 0;
    p.numLongRows = head[1];
    p.rows = rows;
    p.nnz = nnz;
    p.bytes = l.bytes;
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmv_csr_blocked_analyse(const int32_t *rowOffsets, const int32_t *colInd, const void *csrValues,
                                      int64_t rows, int64_t cols, int64_t nnz, int32_t flags, void *workspace,
                                      size_t workspaceBytes, OpsparseSpmvPlan *plan, void *stream)
{
    // one piece: the analysis' scratch follows what the launches keep
    const size_t resident = opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz, flags);
    if (resident == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    if (workspace == nullptr || workspaceBytes < resident) {
        return OPSPARSE_E_WORKSPACE;
    }
    return opsparse_spmv_csr_blocked_analyse_split(rowOffsets, colInd, csrValues, rows, cols, nnz, flags, workspace, resident,
                                            static_cast<unsigned char *>(workspace) + resident, workspaceBytes - resident, plan, stream);
}

}  // extern "C"
