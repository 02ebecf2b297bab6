// CSR producers for gfx950: COO rows -> CSR row offsets, CSR row offsets -> COO
// rows, per-row stable sort of CSR column indices with a permutation, and CSR ->
// CSC.  All of it is integer / byte work whose results must be bit-exact, and
// all of it is bound by memory traffic, so the kernels stream their operands
// with coalesced accesses and keep the shuffling in LDS.
//
// They replace the device side of
//   aclsparseXcoo2csr     sparse/coo2csr/arch35/coo2csr_kernel.cpp   (count + prefix sum)
//   aclsparseXcsr2coo     sparse/csr2coo/arch35/csr2coo_kernel.cpp   (row expansion)
//   aclsparseXcsrsort     sparse/csrsort/arch35/csrsort_kernel.cpp   (runs + serial merge)
//   aclsparseCsr2cscEx2   sparse/csr2csc_ex2/arch35/csr2csc_ex2_kernel.cpp (striped counting sort)
// and produce what the reference's CPU goldens produce
// (test/coo2csr/coo2csr_golden.h:44-77, test/csr2coo/csr2coo_golden.h:37-61,
// test/csrsort/arch35/csrsort_golden.h:38-70, test/csr2csc_ex2/csr2csc_ex2_golden.h:50-110).
//
// Building blocks:
//   * a three-kernel inclusive scan of int32 (tile sums, one-workgroup scan of the
//     sums, tile rescan), in place if wanted;
//   * a least-significant-digit radix sort of (key, payload) pairs, four bits a
//     pass.  A thread owns consecutive items of its tile, counts them per digit,
//     the workgroup scans the 16 x 256 counters digit-major, and every item goes to
//     digit base + number of earlier items with its digit: stable by construction;
//   * bitonic sorts of 64-bit (column, position) keys in registers (a wavefront per
//     row of up to 64 entries) and in LDS (a workgroup per row of up to 2048); the
//     position in the low half makes every key distinct, so any correct sort is
//     the stable sort.
#include <climits>
#include <type_traits>
#include <cstdlib>

#include "convert_internal.h"
#include "device_utils.h"

namespace opsparse {

constexpr int kScanItems = 8;                             // consecutive elements a thread scans
constexpr int kScanTile = kBlockThreads * kScanItems;     // elements per workgroup
constexpr int kRadixBits = 4;
constexpr int kRadixDigits = 1 << kRadixBits;
constexpr int kRadixItems = 4;                            // consecutive items a thread ranks
constexpr int kRadixTile = kBlockThreads * kRadixItems;
constexpr int kSortWaveRow = 64;                          // rows up to this length: one wavefront, registers
constexpr int kSortLdsRow = 2048;                         // rows up to this length: one workgroup, LDS
constexpr int kSortListBlocks = 2048;                     // workgroups walking the list of longer rows
constexpr int kSortWideRow = 16384;                       // listed rows longer than this get 1024 lanes instead of 256

// ------------------------------------------------------------------- fill

__global__ __launch_bounds__(kBlockThreads) void FillI32Kernel(int32_t *__restrict__ p, int64_t n, int32_t v)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < n; i += stride) {
        p[i] = v;
    }
}

// ------------------------------------------------------------------- scan

// Exclusive scan of one value per thread over the workgroup; *total gets the sum.  Its barriers order LDS only.
__device__ __forceinline__ int32_t BlockExclusiveScan(int32_t v, int32_t *waveSums /* [4] in LDS */, int32_t *total)
{
    const int32_t lane = threadIdx.x % kWave;
    const int32_t wave = threadIdx.x / kWave;
    int32_t incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int32_t up = __shfl_up(incl, off, kWave);
        if (lane >= off) {
            incl += up;
        }
    }
    if (lane == kWave - 1) {
        waveSums[wave] = incl;
    }
    LdsBarrier();
    int32_t base = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kBlockThreads / kWave; ++w) {
        const int32_t s = waveSums[w];
        base += (w < wave) ? s : 0;
        all += s;
    }
    LdsBarrier();  // waveSums may be reused by the caller's next call
    *total = all;
    return base + incl - v;
}

__global__ __launch_bounds__(kBlockThreads) void ScanTileSumsKernel(const int32_t *__restrict__ in, int64_t n,
                                                                   int32_t *__restrict__ tileSums)
{
    __shared__ int32_t waveSums[kBlockThreads / kWave];
    const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanTile;
    int32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        const int64_t p = base + i * kBlockThreads + threadIdx.x;
        sum += p < n ? in[p] : 0;
    }
    int32_t total;
    (void)BlockExclusiveScan(sum, waveSums, &total);
    if (threadIdx.x == 0) {
        tileSums[blockIdx.x] = total;
    }
}

// One workgroup: tileSums[i] <- sum of tileSums[0..i).
__global__ __launch_bounds__(kBlockThreads) void ScanTileOffsetsKernel(int32_t *__restrict__ tileSums, int64_t numTiles)
{
    __shared__ int32_t waveSums[kBlockThreads / kWave];
    int32_t carry = 0;
    for (int64_t c0 = 0; c0 < numTiles; c0 += kBlockThreads) {
        const int64_t p = c0 + threadIdx.x;
        const int32_t v = p < numTiles ? tileSums[p] : 0;
        int32_t total;
        const int32_t excl = BlockExclusiveScan(v, waveSums, &total);
        if (p < numTiles) {
            tileSums[p] = carry + excl;
        }
        carry += total;
    }
}

// out[i] = add + in[0] + ... + in[i]; out may be in.
__global__ __launch_bounds__(kBlockThreads) void ScanApplyKernel(const int32_t *in, int32_t *out, int64_t n,
                                                                const int32_t *__restrict__ tileOffsets, int32_t add)
{
    __shared__ int32_t waveSums[kBlockThreads / kWave];
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kScanTile + static_cast<int64_t>(threadIdx.x) * kScanItems;
    int32_t v[kScanItems];
    int32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        v[i] = first + i < n ? in[first + i] : 0;
        sum += v[i];
        v[i] = sum;  // inclusive within the thread
    }
    int32_t total;
    const int32_t before = BlockExclusiveScan(sum, waveSums, &total) + tileOffsets[blockIdx.x] + add;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        if (first + i < n) {
            out[first + i] = before + v[i];
        }
    }
}

// ---------------------------------------------------------------- coo2csr

// counts[r + 1] += number of entries with row r (rows outside [0, m) are
// skipped, as the golden does).  A wavefront reads 64 consecutive entries at a
// time; the first lane of every run of equal rows adds the run's length with
// one atomic, so sorted input costs about one atomic per distinct row and
// unsorted input still counts correctly.
__global__ __launch_bounds__(kBlockThreads) void CountRunsKernel(const int32_t *__restrict__ ind, int64_t nnz,
                                                                int64_t m, int32_t base, int32_t *counts)
{
    constexpr int kRounds = 8;
    const int32_t lane = threadIdx.x % kWave;
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * (kBlockThreads / kWave) + threadIdx.x / kWave;
    const int64_t first = wave * (kWave * kRounds);
    // all loads first, unconditionally (a position past the end re-reads the last entry and is not counted): behind
    // the branch around the atomic the compiler would wait for each load before issuing the next
    int32_t raw[kRounds];
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
        const int64_t p = first + r * kWave + lane;
        raw[r] = LoadStream(ind + (p < nnz ? p : nnz - 1));
    }
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
        const int64_t p = first + r * kWave + lane;
        const bool valid = p < nnz;
        // unsigned subtraction, like the reference kernel: no signed overflow on hostile input
        const int32_t row = valid ? static_cast<int32_t>(static_cast<uint32_t>(raw[r]) - static_cast<uint32_t>(base))
                                  : -1;
        const int32_t prev = __shfl_up(row, 1, kWave);
        const bool head = valid && (lane == 0 || prev != row);
        const uint64_t heads = __ballot(head);
        const uint64_t valids = __ballot(valid);
        if (head && row >= 0 && row < m) {
            // the run ends in front of the next head, or with the last valid lane
            const uint64_t later = lane == kWave - 1 ? 0 : (heads >> (lane + 1)) << (lane + 1);
            const int32_t end = later != 0 ? __ffsll(static_cast<long long>(later)) - 1 : __popcll(valids);
            atomicAdd(counts + row + 1, end - lane);
        }
    }
}

// ---------------------------------------------------------------- csr2coo

// A wavefront takes 64 consecutive rows.  Where their bounds chain (every row ends where the next begins, as in
// any well-formed CSR matrix) the 64 rows are one contiguous piece of the output: lane l writes positions
// first + l, first + l + 64, ..., a whole 256-byte line per store instruction, and finds the row of a position
// by walking the wavefront's 65 offsets, kept in LDS, forwards.  Otherwise (a row whose bounds do not describe
// a range inside [0, nnz) is skipped, csr2coo_golden.h:51-53, and rows may overlap or leave gaps) rows of up to
// 16 entries are written by their own lane and a longer row by the whole wavefront, 64 entries per store.
__global__ __launch_bounds__(kBlockThreads) void ExpandRowsKernel(const int32_t *__restrict__ rowPtr, int64_t m,
                                                                 int64_t nnz, int32_t base,
                                                                 int32_t *__restrict__ rowInd)
{
    __shared__ int32_t offs[kBlockThreads / kWave][kWave + 1];
    const int32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int64_t row = (static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x);
    int64_t lo = 0, hi = 0;
    bool bad = false;
    if (row < m) {
        lo = static_cast<int64_t>(rowPtr[row]) - base;
        hi = static_cast<int64_t>(rowPtr[row + 1]) - base;
        if (lo < 0 || hi > nnz || lo > hi) {
            lo = hi = 0;
            bad = true;
        }
    }
    const int32_t value = static_cast<int32_t>(row) + base;
    const int32_t live = __popcll(__ballot(row < m));  // rows of this wavefront: the first `live` lanes
    if (live == 0) {
        return;
    }
    const int64_t nextLo = __shfl_down(lo, 1, kWave);
    const bool chained = !bad && (lane + 1 >= live || hi == nextLo);
    if (__all(chained || lane >= live)) {
        int32_t *mine = offs[wave];
        if (lane < live) {
            mine[lane] = static_cast<int32_t>(lo);
        }
        if (lane == live - 1) {
            mine[live] = static_cast<int32_t>(hi);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int32_t first = mine[0], last = mine[live];
        const int32_t row0 = static_cast<int32_t>(row) - lane + base;
        if (static_cast<int64_t>(last - first) >= 11 * static_cast<int64_t>(live)) {
            // rows of 11 entries and more on average: from one position of a lane to its next (64 further) at most
            // six row ends are passed, and walking past them is cheaper than searching
            int32_t cur = 0;
            for (int32_t p = first + lane; p < last; p += kWave) {
                while (mine[cur + 1] <= p) {  // ends at the latest at cur + 1 == live, whose offset is `last` > p
                    ++cur;
                }
                rowInd[p] = row0 + cur;
            }
        } else {
            for (int32_t p = first + lane; p < last; p += kWave) {
                int32_t a = 0, b = live - 1;  // the last row with mine[row] <= p (mine[0] <= p < mine[live]): 64 candidates
#pragma unroll
                for (int step = 0; step < 6; ++step) {
                    const int32_t mid = (a + b + 1) >> 1;
                    const bool right = mine[mid] <= p;
                    a = right ? mid : a;
                    b = right ? b : mid - 1;
                }
                rowInd[p] = row0 + a;
            }
        }
        return;
    }
    const int64_t len = hi - lo;
    if (len <= 16) {
        for (int64_t j = 0; j < len; ++j) {
            rowInd[lo + j] = value;
        }
    }
    uint64_t longRows = __ballot(len > 16);
    while (longRows != 0) {
        const int32_t src = __ffsll(static_cast<long long>(longRows)) - 1;
        longRows &= longRows - 1;
        const int64_t l = __shfl(lo, src, kWave);
        const int64_t h = __shfl(hi, src, kWave);
        const int32_t v = __shfl(value, src, kWave);
        for (int64_t p = l + lane; p < h; p += kWave) {
            rowInd[p] = v;
        }
    }
}

// ------------------------------------------------------------- radix sort

// Digit of a key for the pass at `shift`.
__device__ __forceinline__ int32_t RadixDigit(int32_t key, int32_t shift)
{
    return static_cast<int32_t>((static_cast<uint32_t>(key) >> shift) & (kRadixDigits - 1));
}

// table[1 + digit * numTiles + tile] = items of that digit in the tile
// (table[0] stays 0: an inclusive scan of the table then leaves, at the same
// place shifted down by one, the first output position of every (digit, tile)).
__global__ __launch_bounds__(kBlockThreads) void RadixCountKernel(const int32_t *__restrict__ keys, int64_t n,
                                                                 int32_t keyBase, int32_t shift,
                                                                 int32_t *__restrict__ table, int64_t numTiles)
{
    __shared__ int32_t hist[kRadixDigits];
    if (threadIdx.x < kRadixDigits) {
        hist[threadIdx.x] = 0;
    }
    __syncthreads();
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kRadixTile + static_cast<int64_t>(threadIdx.x) * kRadixItems;
#pragma unroll
    for (int i = 0; i < kRadixItems; ++i) {
        if (first + i < n) {
            atomicAdd(&hist[RadixDigit(keys[first + i] - keyBase, shift)], 1);
        }
    }
    __syncthreads();
    if (threadIdx.x < kRadixDigits) {
        table[1 + static_cast<int64_t>(threadIdx.x) * numTiles + blockIdx.x] = hist[threadIdx.x];
    }
}

// LDS arrays that one phase reads with lane t at t * 16 + i and another with lane t at d * 256 + t: one unused
// word after every 32 keeps both patterns free of bank conflicts (unpadded, the first puts all lanes on two banks).
__device__ __forceinline__ int32_t Padded(int32_t i)
{
    return i + (i >> 5);
}
constexpr int kCounterSlots = kRadixDigits * kBlockThreads + kRadixDigits * kBlockThreads / 32;

// Exclusive scan, digit-major, of the 16 x 256 per-thread digit counters of a
// workgroup.  counters[d * 256 + t] holds thread t's count of digit d on entry
// and the number of items that sort before thread t's first item of digit d on
// exit.
__device__ __forceinline__ void ScanDigitCounters(int32_t *counters, int32_t *waveSums)
{
    constexpr int kPer = kRadixDigits;  // 4096 counters / 256 threads
    int32_t v[kPer];
    int32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        v[i] = counters[Padded(threadIdx.x * kPer + i)];
        sum += v[i];
    }
    int32_t total;
    int32_t run = BlockExclusiveScan(sum, waveSums, &total);
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        counters[Padded(threadIdx.x * kPer + i)] = run;
        run += v[i];
    }
    LdsBarrier();
}

// What travels with the keys through a pass.  kPayIndex: one int32 per item (a source position; payloadIn ==
// NULL means "the payload of item i is i").  The pair modes carry csr2csc's (row, value) itself, 8 bytes, so that
// no gather by source position is left at the end: kPayPairFirst builds the pair from the row-of-position and
// value arrays (read in order), kPayPair moves it, kPayPairLast writes its two halves to the output arrays.
enum RadixPayload { kPayIndex = 0, kPayPairFirst = 1, kPayPair = 2, kPayPairLast = 3 };

struct RadixPairIo {
    const int32_t *rowSrc;  // kPayPairFirst: row (with the output's index base) of every source position
    const void *valSrc;     //                the values, valueBytes each (0: none)
    int32_t *rowOut;        // kPayPairLast: the sorted rows
    void *valOut;           //               the sorted values
    int32_t valueBytes;
};

struct RadixPair {
    int32_t row;
    uint32_t val;
};

// One pass: items of tile `blockIdx.x` go to prefix[digit][tile] + their rank
// among the tile's items of the same digit.  keyBase is subtracted from the keys
// read (first pass: the index base of the column indices) and the keys are
// written without it.
template <int Mode>
__global__ __launch_bounds__(kBlockThreads) void RadixScatterKernel(
    const int32_t *__restrict__ keysIn, const void *__restrict__ payloadIn, int32_t *__restrict__ keysOut,
    void *__restrict__ payloadOut, int64_t n, int32_t keyBase, int32_t shift, const int32_t *__restrict__ prefix,
    int64_t numTiles, RadixPairIo io)
{
    __shared__ int32_t counters[kCounterSlots];
    __shared__ int32_t waveSums[kBlockThreads / kWave];
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kRadixTile + static_cast<int64_t>(threadIdx.x) * kRadixItems;
    int32_t key[kRadixItems], dig[kRadixItems];
    RadixPair pay[kRadixItems];  // kPayIndex uses .row only
    int32_t cnt[kRadixDigits];
#pragma unroll
    for (int d = 0; d < kRadixDigits; ++d) {
        cnt[d] = 0;
    }
#pragma unroll
    for (int i = 0; i < kRadixItems; ++i) {
        dig[i] = -1;
        pay[i] = RadixPair{0, 0u};
        if (first + i < n) {
            key[i] = keysIn[first + i] - keyBase;
            if (Mode == kPayIndex) {
                pay[i].row = payloadIn != nullptr ? static_cast<const int32_t *>(payloadIn)[first + i]
                                                  : static_cast<int32_t>(first + i);
            } else if (Mode == kPayPairFirst) {
                pay[i].row = io.rowSrc[first + i];
                if (io.valueBytes == 4) {
                    pay[i].val = static_cast<const uint32_t *>(io.valSrc)[first + i];
                } else if (io.valueBytes == 2) {
                    pay[i].val = static_cast<const uint16_t *>(io.valSrc)[first + i];
                } else if (io.valueBytes == 1) {
                    pay[i].val = static_cast<const uint8_t *>(io.valSrc)[first + i];
                }
            } else {
                pay[i] = static_cast<const RadixPair *>(payloadIn)[first + i];
            }
            dig[i] = RadixDigit(key[i], shift);
#pragma unroll
            for (int d = 0; d < kRadixDigits; ++d) {
                cnt[d] += (dig[i] == d) ? 1 : 0;
            }
        }
    }
#pragma unroll
    for (int d = 0; d < kRadixDigits; ++d) {
        counters[Padded(d * kBlockThreads + threadIdx.x)] = cnt[d];
    }
    __syncthreads();
    ScanDigitCounters(counters, waveSums);
#pragma unroll
    for (int i = 0; i < kRadixItems; ++i) {
        if (dig[i] >= 0) {
            // rank inside the tile among items of this digit: the thread's base for the digit, less the
            // digit's own start, plus the thread's earlier items of the digit
            int32_t earlier = 0;
#pragma unroll
            for (int j = 0; j < kRadixItems; ++j) {
                earlier += (j < i && dig[j] == dig[i]) ? 1 : 0;
            }
            const int32_t inTile = counters[Padded(dig[i] * kBlockThreads + threadIdx.x)] -
                                   counters[Padded(dig[i] * kBlockThreads)] + earlier;
            const int64_t dst = static_cast<int64_t>(prefix[static_cast<int64_t>(dig[i]) * numTiles + blockIdx.x]) + inTile;
            keysOut[dst] = key[i];
            if (Mode == kPayPairLast) {
                io.rowOut[dst] = pay[i].row;
                if (io.valueBytes == 4) {
                    static_cast<uint32_t *>(io.valOut)[dst] = pay[i].val;
                } else if (io.valueBytes == 2) {
                    static_cast<uint16_t *>(io.valOut)[dst] = static_cast<uint16_t>(pay[i].val);
                } else if (io.valueBytes == 1) {
                    static_cast<uint8_t *>(io.valOut)[dst] = static_cast<uint8_t>(pay[i].val);
                }
            } else if (Mode == kPayIndex) {
                static_cast<int32_t *>(payloadOut)[dst] = pay[i].row;
            } else {
                static_cast<RadixPair *>(payloadOut)[dst] = pay[i];
            }
        }
    }
}

// ----------------------------------------------- radix sort, 8 bits a pass
// csr2csc's passes.  Sixteen times as many buckets as the 4-bit pass, so a tile's items for one bucket are few:
// written straight from the lanes that hold them they would leave as scattered 12-byte pieces.  The tile is
// therefore ordered by its 8-bit digit inside LDS first and written out in that order: neighbouring lanes then
// write neighbouring addresses of one bucket's run.  What is ordered is one word an item, (digit, slot in the
// tile), by two stable 4-bit splits; the items themselves stay where the loads put them and are fetched by slot at
// the end.  A thread counts its items' digits in one 64-bit register, four bits a digit: the instruction count,
// not the memory system, bounds this kernel, and a counter per digit selected by comparisons costs ten times more.

constexpr int kWideBits = 8;
constexpr int kWideDigits = 1 << kWideBits;
constexpr int kWideItems = 15;                              // items a thread ranks: a 4-bit counter holds them,
                                                            // and an odd stride over LDS has no bank conflicts
constexpr int kWideTile = kBlockThreads * kWideItems;      // 3840
constexpr int kWideSlotBits = 12;
static_assert(kWideTile <= (1 << kWideSlotBits), "a slot number fits its field");
static_assert(kWideDigits == kBlockThreads, "one thread per digit");

// key - keyBase in wrap-around arithmetic (the keys of a COO sort may span the whole int32 range).
__device__ __forceinline__ int32_t Rebased(int32_t key, int32_t keyBase)
{
    return static_cast<int32_t>(static_cast<uint32_t>(key) - static_cast<uint32_t>(keyBase));
}

// A pass's digit: `mask` = 2^bits - 1 with bits <= kWideBits (the passes of a sort share its key bits evenly).
__device__ __forceinline__ int32_t WideDigit(int32_t key, int32_t shift, int32_t mask)
{
    return static_cast<int32_t>((static_cast<uint32_t>(key) >> shift) & static_cast<uint32_t>(mask));
}

// table[1 + digit * numTiles + tile] = items of that digit in the tile (see RadixCountKernel).  A workgroup counts
// kWideCountTiles consecutive tiles and writes their counts of one digit side by side: a tile a workgroup leaves
// the table written four bytes at a time, a cache line for each.
constexpr int kWideCountTiles = 8;

__global__ __launch_bounds__(kBlockThreads) void WideCountKernel(const int32_t *__restrict__ keys, int64_t n,
                                                                int32_t keyBase, int32_t shift, int32_t mask,
                                                                int32_t *__restrict__ table, int64_t numTiles)
{
    __shared__ int32_t hist[kWideCountTiles][kWideDigits];
#pragma unroll
    for (int j = 0; j < kWideCountTiles; ++j) {
        hist[j][threadIdx.x] = 0;
    }
    __syncthreads();
    const int64_t firstTile = static_cast<int64_t>(blockIdx.x) * kWideCountTiles;
    // The keys of a tile are loaded, all of them, a tile ahead of their counting: the compiler keeps a load and the
    // LDS atomic after it in program order, and an atomic straight behind its load is a round trip to memory for
    // every item.  No branch around a load: an item past the end reads the last key and counts for nothing.
    int32_t key[2][kWideItems];
    auto fetch = [&](int j) {
#pragma unroll
        for (int i = 0; i < kWideItems; ++i) {
            const int64_t at = (firstTile + j) * kWideTile + i * kBlockThreads + threadIdx.x;
            key[j & 1][i] = keys[at < n ? at : n - 1];
        }
    };
    fetch(0);
#pragma unroll
    for (int j = 0; j < kWideCountTiles; ++j) {
        if (j + 1 < kWideCountTiles) {
            fetch(j + 1);
        }
#pragma unroll
        for (int i = 0; i < kWideItems; ++i) {
            const int64_t at = (firstTile + j) * kWideTile + i * kBlockThreads + threadIdx.x;
            atomicAdd(&hist[j][WideDigit(Rebased(key[j & 1][i], keyBase), shift, mask)], at < n ? 1 : 0);
        }
    }
    __syncthreads();
    // lanes j = 0 .. kWideCountTiles - 1 of a group write neighbouring tiles of one digit
    constexpr int kDigitsAtOnce = kBlockThreads / kWideCountTiles;
    const int32_t j = threadIdx.x % kWideCountTiles;
#pragma unroll
    for (int d0 = 0; d0 < kWideDigits; d0 += kDigitsAtOnce) {
        const int32_t d = d0 + threadIdx.x / kWideCountTiles;
        if (firstTile + j < numTiles) {
            table[1 + static_cast<int64_t>(d) * numTiles + firstTile + j] = hist[j][d];
        }
    }
}

// Between two passes the n (row, value) pairs lie as n rows followed by n values in the 8 n bytes of their buffer:
// 4-byte stores to a bucket's run, as for the keys (8-byte stores of whole pairs to such short runs took half as
// long again).
template <typename P>
__device__ __forceinline__ auto WideRows(P *pairs)
{
    return reinterpret_cast<std::conditional_t<std::is_const<P>::value, const int32_t, int32_t> *>(pairs);
}
template <typename P>
__device__ __forceinline__ auto WideVals(P *pairs, int64_t n)
{
    return reinterpret_cast<std::conditional_t<std::is_const<P>::value, const uint32_t, uint32_t> *>(pairs) + n;
}

// A tile's items as the loads deliver them, lane t holding slots t, t + 256, ...
struct WideTileRegs {
    int32_t key[kWideItems];
    RadixPair pay[kWideItems];
    int32_t first, next;  // prefix[digit tid][tile] and the entry after it
};

template <int Mode, int VB, bool Full>
__device__ __forceinline__ void WideFetch(WideTileRegs &r, int64_t tile, const int32_t *__restrict__ keysIn,
                                          const RadixPair *__restrict__ pairsIn, int64_t n, int32_t keyBase,
                                          int32_t shift, int32_t mask, const int32_t *__restrict__ prefix,
                                          int64_t numTiles, const RadixPairIo &io)
{
    const int tid = threadIdx.x;
    const int64_t tile0 = tile * kWideTile;
    const int64_t flat = static_cast<int64_t>(tid) * numTiles + tile;
    r.first = prefix[flat];
    r.next = prefix[flat + 1];
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) {
        const int64_t at = tile0 + i * kBlockThreads + tid;
        // a slot past the end gets the largest digit, so that it sorts behind every real item
        r.key[i] = static_cast<int32_t>(static_cast<uint32_t>(mask) << shift);
        r.pay[i] = RadixPair{0, 0u};
        if (Full || at < n) {
            r.key[i] = Rebased(keysIn[at], keyBase);
            if (Mode == kPayPairFirst) {
                r.pay[i].row = io.rowSrc[at];
                if (VB == 4) {
                    r.pay[i].val = static_cast<const uint32_t *>(io.valSrc)[at];
                } else if (VB == 2) {
                    r.pay[i].val = static_cast<const uint16_t *>(io.valSrc)[at];
                } else if (VB == 1) {
                    r.pay[i].val = static_cast<const uint8_t *>(io.valSrc)[at];
                }
            } else {
                r.pay[i] = RadixPair{WideRows(pairsIn)[at], WideVals(pairsIn, n)[at]};
            }
        }
    }
}

struct WideLds {
    int32_t key[kWideTile];
    __align__(8) RadixPair pay[kWideTile];
    uint32_t word[kWideTile];
    int32_t counters[kCounterSlots];
    int32_t waveSums[kBlockThreads / kWave];
    int32_t outOf[kWideDigits];  // output position less slot in the ordered tile, for the items of a digit
};

// Orders the tile held in LDS (key, pay filled, barrier not yet passed) and writes it out.  Ends with the stores
// issued and no barrier behind them.
template <int Mode, int VB, bool Full>
__device__ __forceinline__ void WideOrderAndWrite(WideLds &lds, int32_t first, int32_t next, int64_t tile, int64_t n,
                                                  int32_t shift, int32_t mask, int32_t *__restrict__ keysOut,
                                                  RadixPair *__restrict__ pairsOut, const RadixPairIo &io)
{
    const int tid = threadIdx.x;
    {
        // where the tile's run of digit `tid` starts in the ordered tile, from the lengths of the runs before it
        int32_t total;
        const int32_t start = BlockExclusiveScan(next - first, lds.waveSums, &total);  // has barriers
        lds.outOf[tid] = first - start;
    }
    // a thread takes kWideItems consecutive slots of the current order
    uint32_t word[kWideItems];
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) {
        const int32_t p = tid * kWideItems + i;
        word[i] = (static_cast<uint32_t>(WideDigit(lds.key[p], shift, mask)) << kWideSlotBits) | static_cast<uint32_t>(p);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int32_t at = kWideSlotBits + half * kRadixBits;
        uint64_t packed = 0;  // the thread's count of digit d in bits [4 d, 4 d + 4)
        int32_t earlier[kWideItems];
#pragma unroll
        for (int i = 0; i < kWideItems; ++i) {
            const uint32_t sh = ((word[i] >> at) & (kRadixDigits - 1)) * 4;
            earlier[i] = static_cast<int32_t>((packed >> sh) & 15);
            packed += uint64_t{1} << sh;
        }
#pragma unroll
        for (int d = 0; d < kRadixDigits; ++d) {
            lds.counters[Padded(d * kBlockThreads + tid)] = static_cast<int32_t>((packed >> (4 * d)) & 15);
        }
        LdsBarrier();
        ScanDigitCounters(lds.counters, lds.waveSums);  // counters[d][t]: slots before thread t's first item of d
#pragma unroll
        for (int i = 0; i < kWideItems; ++i) {
            const int32_t d = static_cast<int32_t>((word[i] >> at) & (kRadixDigits - 1));
            lds.word[lds.counters[Padded(d * kBlockThreads + tid)] + earlier[i]] = word[i];
        }
        LdsBarrier();
        if (half == 0) {
#pragma unroll
            for (int i = 0; i < kWideItems; ++i) {
                word[i] = lds.word[tid * kWideItems + i];
            }
        }
    }
    const int64_t tile0 = tile * kWideTile;
    const int32_t valid = Full ? kWideTile : static_cast<int32_t>(n - tile0);
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) {
        const int32_t p = i * kBlockThreads + tid;
        if (Full || p < valid) {  // the real items are the first `valid` slots of the ordered tile
            const uint32_t w = lds.word[p];
            const int32_t slot = static_cast<int32_t>(w & ((1u << kWideSlotBits) - 1));
            const int64_t dst = static_cast<int64_t>(lds.outOf[w >> kWideSlotBits] + p);
            const RadixPair out = lds.pay[slot];
            keysOut[dst] = lds.key[slot];
            if (Mode == kPayPairLast) {
                io.rowOut[dst] = out.row;
                if (VB == 4) {
                    static_cast<uint32_t *>(io.valOut)[dst] = out.val;
                } else if (VB == 2) {
                    static_cast<uint16_t *>(io.valOut)[dst] = static_cast<uint16_t>(out.val);
                } else if (VB == 1) {
                    static_cast<uint8_t *>(io.valOut)[dst] = static_cast<uint8_t>(out.val);
                }
            } else {
                WideRows(pairsOut)[dst] = out.row;
                WideVals(pairsOut, n)[dst] = out.val;
            }
        }
    }
}

template <bool Full>
__device__ __forceinline__ void WideStage(WideLds &lds, const WideTileRegs &r)
{
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) {
        const int32_t p = i * kBlockThreads + threadIdx.x;
        lds.key[p] = r.key[i];
        lds.pay[p] = r.pay[i];
    }
}

// One pass; the payload modes are those of RadixScatterKernel (pairs only), VB the bytes of a value in the arrays
// that the first pass reads and the last one writes (a template parameter: a branch on it among the loads would
// leave the compiler unable to count what is in flight).  prefix is the scanned table:
// prefix[digit * numTiles + tile] is the first output position of the tile's items of that digit, and the entry
// after it, in that same flat order, ends them.  A workgroup takes the full tiles blockIdx.x, blockIdx.x +
// gridDim.x, ... and has the loads of its next tile in flight while it orders and writes the current one (with
// two workgroups on a compute unit and a tile's phases one after another, a tile fetched only when its turn comes
// leaves the memory system idle most of the time: 3.2 TB/s for a pass that does nothing but copy).  The tile that
// the end of the array cuts short is done last, by workgroup 0, with bounds checks.
template <int Mode, int VB>
__global__ __launch_bounds__(kBlockThreads) void WideScatterKernel(
    const int32_t *__restrict__ keysIn, const RadixPair *__restrict__ pairsIn, int32_t *__restrict__ keysOut,
    RadixPair *__restrict__ pairsOut, int64_t n, int32_t keyBase, int32_t shift, int32_t mask,
    const int32_t *__restrict__ prefix, int64_t numTiles, RadixPairIo io)
{
    __shared__ WideLds lds;
    const int64_t fullTiles = n / kWideTile;
    WideTileRegs r;
    // a workgroup's tiles are consecutive: the runs it writes into a bucket follow one another, and the cache line
    // that one run leaves half written is completed by the next from the same compute unit
    const int64_t perBlock = (fullTiles + gridDim.x - 1) / gridDim.x;
    int64_t tile = blockIdx.x * perBlock;
    const int64_t tileEnd = tile + perBlock < fullTiles ? tile + perBlock : fullTiles;
    auto turn = [&]() {
        WideStage<true>(lds, r);
        const int32_t first = r.first, next = r.next;
        // the next tile's loads (the last turn fetches its own tile again rather than branch around the loads:
        // a wait for "all but the stores issued since" needs one straight path)
        const int64_t ahead = tile + 1 < tileEnd ? tile + 1 : tile;
        WideFetch<Mode, VB, true>(r, ahead, keysIn, pairsIn, n, keyBase, shift, mask, prefix, numTiles, io);
        __builtin_amdgcn_sched_barrier(0);  // the loads are issued here, not where the scheduler finds room later
        WideOrderAndWrite<Mode, VB, true>(lds, first, next, tile, n, shift, mask, keysOut, pairsOut, io);
        LdsBarrier();  // the tile's LDS is free again
        ++tile;
    };
    if (tile < tileEnd) {
        WideFetch<Mode, VB, true>(r, tile, keysIn, pairsIn, n, keyBase, shift, mask, prefix, numTiles, io);
        // the first turn stands outside the loop: entered from here, with no stores behind the loads, the loop's
        // wait for the loads would be a wait for everything, the stores of the turn before included
        turn();
        while (tile < tileEnd) {
            turn();
        }
    }
    if (blockIdx.x == 0 && fullTiles < numTiles) {
        WideFetch<Mode, VB, false>(r, fullTiles, keysIn, pairsIn, n, keyBase, shift, mask, prefix, numTiles, io);
        WideStage<false>(lds, r);
        WideOrderAndWrite<Mode, VB, false>(lds, r.first, r.next, fullTiles, n, shift, mask, keysOut, pairsOut, io);
    }
}

// csrsort of a matrix of long rows, between its two sorts: the entries are sorted by column and carry (row,
// permutation value); the second sort is by row and carries (column, permutation value).
__global__ __launch_bounds__(kBlockThreads) void RegroupByRowKernel(const int32_t *__restrict__ colKeys,
                                                                   const RadixPair *__restrict__ rowAndPerm, int64_t n,
                                                                   int32_t colBase, int32_t *__restrict__ rowKeys,
                                                                   RadixPair *__restrict__ colAndPerm)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    if (i < n) {
        const RadixPair in = rowAndPerm[i];
        rowKeys[i] = in.row;
        colAndPerm[i] = RadixPair{colKeys[i] + colBase, in.val};
    }
}

// ---------------------------------------------------------------- csr2csc

// cscRowInd[d] = row of source position pos[d] (+ base); cscVal[d] = csrVal[pos[d]].
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void GatherByPositionKernel(const int32_t *__restrict__ pos,
                                                                       const int32_t *__restrict__ rowOfPos,
                                                                       const T *__restrict__ srcVal, int64_t nnz,
                                                                       int32_t *__restrict__ rowOut,
                                                                       T *__restrict__ valOut)
{
    const int64_t d = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    if (d >= nnz) {
        return;
    }
    const int32_t p = LoadStream(pos + d);
    rowOut[d] = rowOfPos[p];
    if (valOut != nullptr) {
        valOut[d] = srcVal[p];
    }
}

// ---------------------------------------------------------------- csrsort

// Orders by signed column first, position in the row second.
__device__ __forceinline__ uint64_t SortKey(int32_t col, uint32_t idx)
{
    return (static_cast<uint64_t>(static_cast<uint32_t>(col) ^ 0x80000000u) << 32) | idx;
}
__device__ __forceinline__ int32_t SortKeyColumn(uint64_t key)
{
    return static_cast<int32_t>(static_cast<uint32_t>(key >> 32) ^ 0x80000000u);
}

// The value of lane (l ^ J) for every lane l of a wavefront, all of whose lanes are active.  Distances 1, 2, 4
// and 8 stay inside a row of 16 lanes and are data-parallel-primitive moves in the vector ALU (quad permutes,
// rotations of a row); only 16 and 32 go through the LDS crossbar, where every distance went before (the sort of
// a 64-lane group issued 42 such operations and spent its time waiting for them).  `ror4` says whether the
// rotation by 4 or the one by 12 brings lane l the value of lane l ^ 4: found once per thread by sending the
// lane numbers through both, which leaves the direction of the rotation out of the argument.
__device__ __forceinline__ uint32_t DppMove(uint32_t v, int ctrl)
{
    switch (ctrl) {  // the control word is an immediate of the instruction
        case 0xB1: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false));
        case 0x4E: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false));
        case 0x124: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x124, 0xF, 0xF, false));
        case 0x128: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x128, 0xF, 0xF, false));
        default: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x12C, 0xF, 0xF, false));
    }
}

__device__ __forceinline__ bool Ror4IsXor4()
{
    const uint32_t lane = threadIdx.x % kWave;
    return DppMove(lane, 0x124) == (lane ^ 4u);
}

template <int J>
__device__ __forceinline__ uint32_t XorLanes(uint32_t v, bool ror4)
{
    if (J == 1) {
        return DppMove(v, 0xB1);  // quad_perm [1, 0, 3, 2]
    } else if (J == 2) {
        return DppMove(v, 0x4E);  // quad_perm [2, 3, 0, 1]
    } else if (J == 4) {
        const uint32_t a = DppMove(v, 0x124), b = DppMove(v, 0x12C);  // row_ror 4 and 12
        return ror4 ? a : b;
    } else if (J == 8) {
        return DppMove(v, 0x128);  // row_ror 8: the same in either direction
    } else {
        return static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), J, kWave));
    }
}

template <int J>
__device__ __forceinline__ uint64_t XorLanes(uint64_t v, bool ror4)
{
    const uint32_t lo = XorLanes<J>(static_cast<uint32_t>(v), ror4);
    const uint32_t hi = XorLanes<J>(static_cast<uint32_t>(v >> 32), ror4);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

template <int K, int J, typename KeyT>
__device__ __forceinline__ void BitonicStep(KeyT &key, int32_t g, bool ror4)
{
    const KeyT other = XorLanes<J>(key, ror4);
    const bool ascending = (g & K) == 0;
    const bool lower = (g & J) == 0;
    const KeyT mn = key < other ? key : other;
    const KeyT mx = key < other ? other : key;
    key = (ascending == lower) ? mn : mx;
}

template <int K, int J, typename KeyT>
__device__ __forceinline__ void BitonicMerge(KeyT &key, int32_t g, bool ror4)
{
    BitonicStep<K, J>(key, g, ror4);
    if constexpr (J > 1) {
        BitonicMerge<K, J / 2>(key, g, ror4);
    }
}

template <int G, int K, typename KeyT>
__device__ __forceinline__ void BitonicStages(KeyT &key, int32_t g, bool ror4)
{
    BitonicMerge<K, K / 2>(key, g, ror4);
    if constexpr (K < G) {
        BitonicStages<G, K * 2>(key, g, ror4);
    }
}

// Bitonic sort of one key per lane over the G lanes of a group (all 64 lanes of the wavefront take part); `g` is
// the lane's index in its group.  The low bits of a key hold the group lane its entry came from, so all keys
// differ and the sort is the stable one.  Returns the sorted key.
template <int G, typename KeyT>
__device__ __forceinline__ KeyT GroupBitonicSort(KeyT key, int32_t g)
{
    const bool ror4 = Ror4IsXor4();
    BitonicStages<G, 2>(key, g, ror4);
    return key;
}

// Packed: the key is (column << log2 G | lane) in 32 bits, half the moves of the 64-bit key; the launcher takes
// it when every column index of a valid matrix fits (columns outside [0, n) then only lose their order: the
// entries themselves travel by source lane, not inside the key).
// The entry a lane holds of its group's row, sorted within the group: (col, pay) of lane g become those of the
// g-th entry of the sorted row.
template <int G, bool Packed>
__device__ __forceinline__ void SortHeldRow(bool valid, int32_t g, int32_t *col, int32_t *pay)
{
    constexpr int kLog = G == 64 ? 6 : G == 32 ? 5 : G == 16 ? 4 : 3;
    static_assert((1 << kLog) == G, "8, 16, 32 or 64 lanes a row");
    const int32_t lane = threadIdx.x % kWave;
    int32_t from;
    if (Packed) {
        uint32_t key = valid ? (static_cast<uint32_t>(*col) << kLog) | static_cast<uint32_t>(g) : ~0u;  // padding last
        key = GroupBitonicSort<G>(key, g);
        from = (lane - g) + static_cast<int32_t>(key & (G - 1));
    } else {
        uint64_t key = valid ? SortKey(*col, static_cast<uint32_t>(g)) : ~0ull;
        key = GroupBitonicSort<G>(key, g);
        from = (lane - g) + (static_cast<int32_t>(key & 0xffffffffu) & (G - 1));
    }
    *col = __shfl(*col, from, kWave);
    *pay = __shfl(*pay, from, kWave);
}

template <int G, bool Packed>
__device__ __forceinline__ void SortRowInGroup(int64_t begin, int64_t len, int32_t g, int32_t *colInd, int32_t *perm)
{
    const bool valid = g < len;
    int32_t col = 0, pay = 0;
    if (valid) {
        col = colInd[begin + g];
        pay = perm[begin + g];
    }
    SortHeldRow<G, Packed>(valid, g, &col, &pay);
    if (valid) {
        colInd[begin + g] = col;
        perm[begin + g] = pay;
    }
}

// A group of G lanes per row: rows of 2..G entries are sorted in registers (bitonic
// network over the group's lanes); rows of up to 64 entries that do not fit the
// group go to midList (one wavefront each, next kernel), longer rows to longList.
// counters[0] / counters[1] are the two list lengths.  A group takes kSortRowsPerGroup consecutive rows and loads
// all of them before it sorts the first: with a row a group, a wavefront's life was one round trip to memory for
// the offsets, one for the entries and a store, and a million such wavefronts waited more than they moved.
constexpr int kSortRowsPerGroup = 8;

template <int G, bool Packed>
__global__ __launch_bounds__(kBlockThreads) void SortShortRowsKernel(const int32_t *__restrict__ rowPtr, int64_t m,
                                                                    int64_t nnz, int32_t base, int32_t *colInd,
                                                                    int32_t *perm, int32_t *counters,
                                                                    int32_t *__restrict__ midList,
                                                                    int32_t *__restrict__ longList)
{
    constexpr int R = kSortRowsPerGroup;
    const int32_t g = threadIdx.x % G;
    const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlockThreads / G) + threadIdx.x / G) * R;
    int32_t off[R + 1];
#pragma unroll
    for (int r = 0; r <= R; ++r) {
        off[r] = rowPtr[row0 + r <= m ? row0 + r : m];  // (rowPtr has m + 1 entries)
    }
    int64_t begin[R], len[R];
    int32_t col[R], pay[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t row = row0 + r;
        begin[r] = 0;
        len[r] = 0;
        if (row < m) {
            begin[r] = static_cast<int64_t>(off[r]) - base;
            len[r] = static_cast<int64_t>(off[r + 1]) - base - begin[r];
            if (len[r] <= 1 || begin[r] < 0 || begin[r] + len[r] > nnz) {
                len[r] = 0;  // nothing to sort, or bounds that do not describe a range of the arrays
            }
        }
        if (len[r] > G) {
            if (g == 0) {
                if (len[r] <= kSortWaveRow) {
                    midList[atomicAdd(counters, 1)] = static_cast<int32_t>(row);
                } else {
                    longList[atomicAdd(counters + 1, 1)] = static_cast<int32_t>(row);
                }
            }
            len[r] = 0;
        }
        col[r] = 0;
        pay[r] = 0;
        if (g < len[r]) {
            col[r] = colInd[begin[r] + g];
            pay[r] = perm[begin[r] + g];
        }
    }
    // every lane takes part in the shuffles; groups without a row sort padding
#pragma unroll
    for (int r = 0; r < R; ++r) {
        SortHeldRow<G, Packed>(g < len[r], g, &col[r], &pay[r]);
        if (g < len[r]) {
            colInd[begin[r] + g] = col[r];
            perm[begin[r] + g] = pay[r];
        }
    }
}

// Wavefronts walk midList: rows of up to 64 entries, one wavefront each.
template <bool Packed>
__global__ __launch_bounds__(kBlockThreads) void SortMidRowsKernel(const int32_t *__restrict__ rowPtr, int32_t base,
                                                                  int32_t *colInd, int32_t *perm,
                                                                  const int32_t *__restrict__ counters,
                                                                  const int32_t *__restrict__ midList)
{
    const int32_t lane = threadIdx.x % kWave;
    const int32_t count = counters[0];
    const int32_t wavesInGrid = gridDim.x * (kBlockThreads / kWave);
    for (int32_t item = blockIdx.x * (kBlockThreads / kWave) + threadIdx.x / kWave; item < count; item += wavesInGrid) {
        const int32_t row = midList[item];
        const int64_t begin = static_cast<int64_t>(rowPtr[row]) - base;
        const int64_t len = static_cast<int64_t>(rowPtr[row + 1]) - base - begin;
        SortRowInGroup<kWave, Packed>(begin, len, lane, colInd, perm);
    }
}

// Workgroups walk the list of rows longer than 64 entries.  Up to 2048 entries:
// bitonic sort of the keys in LDS.  Longer: a workgroup-local radix sort, four
// bits a pass, between the row and its place in the scratch arrays; thread t
// owns the t-th contiguous part of the row, so the same counter scan as in
// RadixScatterKernel keeps it stable.
template <int kThreads>
__global__ __launch_bounds__(kThreads) void SortListedRowsKernel(const int32_t *__restrict__ rowPtr, int32_t base,
                                                                     int32_t keyBits, int32_t *colInd, int32_t *perm,
                                                                     int32_t *tmpCol, int32_t *tmpPerm,
                                                                     int32_t *listCounts, const int32_t *__restrict__ list,
                                                                     int32_t countSlot, int64_t lenTo,
                                                                     int32_t *__restrict__ longerList)
{
    __shared__ uint64_t keys[kSortLdsRow];                          // 16 KB, doubles as the radix counters
    __shared__ int32_t pays[kSortLdsRow];
    static_assert(sizeof(uint64_t) * kSortLdsRow >= sizeof(int32_t) * 2 * (kThreads / kWave) * kRadixDigits, "counter space");
    int32_t *counters = reinterpret_cast<int32_t *>(keys);

    const int32_t count = listCounts[countSlot];
    for (int32_t item = blockIdx.x; item < count; item += gridDim.x) {
        const int32_t row = list[item];
        const int64_t begin = static_cast<int64_t>(rowPtr[row]) - base;
        const int64_t len = static_cast<int64_t>(rowPtr[row + 1]) - base - begin;
        if (len > lenTo) {
            // too long for this launch: listed for the next one, which runs with more lanes per row
            if (threadIdx.x == 0) {
                longerList[atomicAdd(&listCounts[2], 1)] = row;
            }
            continue;
        }
        if (len <= kSortLdsRow) {
            int32_t npad = 128;
            while (npad < len) {
                npad <<= 1;
            }
            for (int32_t i = threadIdx.x; i < npad; i += kThreads) {
                keys[i] = i < len ? SortKey(colInd[begin + i], static_cast<uint32_t>(i)) : ~0ull;
                pays[i] = i < len ? perm[begin + i] : 0;
            }
            __syncthreads();
            for (int32_t k = 2; k <= npad; k <<= 1) {
                for (int32_t j = k >> 1; j > 0; j >>= 1) {
                    for (int32_t i = threadIdx.x; i < npad; i += kThreads) {
                        const int32_t partner = i ^ j;
                        if (partner > i) {
                            const uint64_t a = keys[i], b = keys[partner];
                            const bool ascending = (i & k) == 0;
                            if ((a > b) == ascending) {
                                keys[i] = b;
                                keys[partner] = a;
                            }
                        }
                    }
                    __syncthreads();
                }
            }
            for (int32_t i = threadIdx.x; i < len; i += kThreads) {
                const uint64_t key = keys[i];
                colInd[begin + i] = SortKeyColumn(key);
                perm[begin + i] = pays[static_cast<uint32_t>(key & 0xffffffffu)];
            }
            __syncthreads();
            continue;
        }
        // Stable 4-bit radix passes over [begin, begin + len) between the row and the scratch arrays.  Wavefront w
        // owns the w-th quarter of the row and walks it 64 consecutive entries at a time, so every load is
        // coalesced.  Counting pass: per-lane digit counts, added up over the wavefront.  Then the first output
        // slot of every (digit, wavefront), digit-major, so that equal digits keep their order.  Scatter pass: the
        // lanes of a round that hold the same digit are found with four ballots, the rank among them is a population
        // count, and a running count per digit carries on from round to round.
        constexpr int kWaves = kThreads / kWave;
        constexpr int kRounds = 8;  // rounds whose loads are issued together
        int32_t *waveDigit = counters;                        // [kWaves][kRadixDigits] counts, then first slots
        int32_t *running = counters + kWaves * kRadixDigits;  // [kWaves][kRadixDigits] entries placed so far
        const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
        const uint64_t below = (uint64_t{1} << lane) - 1;
        const int64_t quarter = (len + kWaves - 1) / kWaves;
        const int64_t lo = begin + wave * quarter < begin + len ? begin + wave * quarter : begin + len;
        const int64_t hi = lo + quarter < begin + len ? lo + quarter : begin + len;
        int32_t *srcCol = colInd, *srcPerm = perm, *dstCol = tmpCol, *dstPerm = tmpPerm;
        for (int32_t shift = 0; shift < keyBits; shift += kRadixBits) {
            int32_t cnt[kRadixDigits];
#pragma unroll
            for (int d = 0; d < kRadixDigits; ++d) {
                cnt[d] = 0;
            }
            for (int64_t p0 = lo + lane; p0 < hi; p0 += kRounds * kWave) {
                int32_t c[kRounds];
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {  // the loads of kRounds rounds issued together
                    const int64_t p = p0 + u * kWave;
                    c[u] = p < hi ? srcCol[p] : -1;
                }
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int32_t dg = p0 + u * kWave < hi ? RadixDigit(c[u] - base, shift) : -1;
#pragma unroll
                    for (int d = 0; d < kRadixDigits; ++d) {
                        cnt[d] += (dg == d) ? 1 : 0;
                    }
                }
            }
#pragma unroll
            for (int d = 0; d < kRadixDigits; ++d) {
                int32_t c = cnt[d];
#pragma unroll
                for (int off = kWave / 2; off > 0; off >>= 1) {
                    c += __shfl_xor(c, off, kWave);
                }
                if (lane == 0) {
                    waveDigit[wave * kRadixDigits + d] = c;
                    running[wave * kRadixDigits + d] = 0;
                }
            }
            __syncthreads();
            if (threadIdx.x == 0) {  // 64 numbers: first slot of (digit, wavefront), digit-major
                int32_t run = 0;
                for (int d = 0; d < kRadixDigits; ++d) {
                    for (int w = 0; w < kWaves; ++w) {
                        const int32_t c = waveDigit[w * kRadixDigits + d];
                        waveDigit[w * kRadixDigits + d] = run;
                        run += c;
                    }
                }
            }
            __syncthreads();
            for (int64_t p0 = lo; p0 < hi; p0 += kRounds * kWave) {
                int32_t c[kRounds], pv[kRounds];
                bool valid[kRounds];
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int64_t p = p0 + u * kWave + lane;
                    valid[u] = p < hi;
                    c[u] = valid[u] ? srcCol[p] : 0;
                    pv[u] = valid[u] ? srcPerm[p] : 0;
                }
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int32_t dg = RadixDigit(c[u] - base, shift);
                    uint64_t same = __ballot(valid[u]);
#pragma unroll
                    for (int b = 0; b < kRadixBits; ++b) {
                        const bool bit = (dg >> b) & 1;
                        const uint64_t votes = __ballot(valid[u] && bit);
                        same &= bit ? votes : ~votes;
                    }
                    const int32_t before = running[wave * kRadixDigits + dg];
                    if (valid[u]) {
                        const int64_t slot = begin + waveDigit[wave * kRadixDigits + dg] + before + __popcll(same & below);
                        dstCol[slot] = c[u];
                        dstPerm[slot] = pv[u];
                        if ((same & below) == 0) {  // the lowest lane of every digit present in this round
                            running[wave * kRadixDigits + dg] = before + __popcll(same);
                        }
                    }
                }
            }
            __threadfence_block();
            __syncthreads();
            int32_t *t = srcCol;
            srcCol = dstCol;
            dstCol = t;
            t = srcPerm;
            srcPerm = dstPerm;
            dstPerm = t;
        }
        if (srcCol != colInd) {  // an odd number of passes left the result in the scratch arrays
            for (int64_t p = begin + threadIdx.x; p < begin + len; p += kThreads) {
                colInd[p] = srcCol[p];
                perm[p] = srcPerm[p];
            }
        }
        __syncthreads();
    }
}

// =============================================================== host side

namespace {

inline int CheckLaunch()
{
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

inline int64_t Align256(int64_t v) { return (v + 255) / 256 * 256; }

inline uint32_t GridFor(int64_t items, int64_t perBlock, int64_t cap = INT32_MAX)
{
    int64_t g = (items + perBlock - 1) / perBlock;
    g = g < 1 ? 1 : g;
    return static_cast<uint32_t>(g > cap ? cap : g);
}

inline int64_t ScanTiles(int64_t count) { return (count + kScanTile - 1) / kScanTile; }

// out[i] = add + in[0..i]; `tiles` holds ScanTiles(count) ints.
void LaunchInclusiveScan(const int32_t *in, int32_t *out, int64_t count, int32_t add, int32_t *tiles, hipStream_t s)
{
    if (count <= 0) {
        return;
    }
    const int64_t numTiles = ScanTiles(count);
    hipLaunchKernelGGL(ScanTileSumsKernel, dim3(static_cast<uint32_t>(numTiles)), dim3(kBlockThreads), 0, s, in, count,
                       tiles);
    hipLaunchKernelGGL(ScanTileOffsetsKernel, dim3(1), dim3(kBlockThreads), 0, s, tiles, numTiles);
    hipLaunchKernelGGL(ScanApplyKernel, dim3(static_cast<uint32_t>(numTiles)), dim3(kBlockThreads), 0, s, in, out,
                       count, tiles, add);
}

void LaunchFill(int32_t *p, int64_t n, int32_t v, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(FillI32Kernel, dim3(GridFor(n, kBlockThreads, 8192)), dim3(kBlockThreads), 0, s, p, n, v);
    }
}

}  // namespace

int64_t ScanScratchInts(int64_t count) { return count <= 0 ? 0 : ScanTiles(count); }

void LaunchInclusiveScanI32(const int32_t *in, int32_t *out, int64_t count, int32_t add, int32_t *scratch, hipStream_t s)
{
    LaunchInclusiveScan(in, out, count, add, scratch, s);
}

void LaunchFillI32(int32_t *p, int64_t n, int32_t v, hipStream_t s)
{
    LaunchFill(p, n, v, s);
}

void LaunchExpandRows(const int32_t *rowPtr, int64_t m, int64_t nnz, int32_t base, int32_t *rowInd, hipStream_t s)
{
    if (m > 0 && nnz > 0) {
        hipLaunchKernelGGL(ExpandRowsKernel, dim3(GridFor(m, kBlockThreads)), dim3(kBlockThreads), 0, s, rowPtr, m, nnz,
                           base, rowInd);
    }
}

int64_t RadixTiles(int64_t n) { return (n + kRadixTile - 1) / kRadixTile; }
int64_t RadixTableInts(int64_t n) { return static_cast<int64_t>(kRadixDigits) * RadixTiles(n) + 1; }

void LaunchRadixPass(const int32_t *keysIn, const int32_t *payIn, int32_t *keysOut, int32_t *payOut, int64_t n,
                     int32_t keyBase, int32_t shift, int32_t *table, int32_t *scratch, hipStream_t s)
{
    if (n <= 0) {
        return;
    }
    const int64_t numTiles = RadixTiles(n);
    const auto grid = dim3(static_cast<uint32_t>(numTiles));
    LaunchFill(table, 1, 0, s);
    hipLaunchKernelGGL(RadixCountKernel, grid, dim3(kBlockThreads), 0, s, keysIn, n, keyBase, shift, table, numTiles);
    LaunchInclusiveScan(table, table, RadixTableInts(n), 0, scratch, s);
    hipLaunchKernelGGL(RadixScatterKernel<kPayIndex>, grid, dim3(kBlockThreads), 0, s, keysIn,
                       static_cast<const void *>(payIn), keysOut, static_cast<void *>(payOut), n, keyBase, shift, table,
                       numTiles, RadixPairIo{});
}

// The same pass carrying csr2csc's (row, value) pairs: mode is one of the pair modes of RadixPayload.
void LaunchRadixPairPass(int mode, const int32_t *keysIn, const void *pairsIn, int32_t *keysOut, void *pairsOut,
                         int64_t n, int32_t keyBase, int32_t shift, int32_t *table, int32_t *scratch,
                         const RadixPairIo &io, hipStream_t s)
{
    if (n <= 0) {
        return;
    }
    const int64_t numTiles = RadixTiles(n);
    const auto grid = dim3(static_cast<uint32_t>(numTiles));
    LaunchFill(table, 1, 0, s);
    hipLaunchKernelGGL(RadixCountKernel, grid, dim3(kBlockThreads), 0, s, keysIn, n, keyBase, shift, table, numTiles);
    LaunchInclusiveScan(table, table, RadixTableInts(n), 0, scratch, s);
    switch (mode) {
        case kPayPairFirst:
            hipLaunchKernelGGL(RadixScatterKernel<kPayPairFirst>, grid, dim3(kBlockThreads), 0, s, keysIn, pairsIn,
                               keysOut, pairsOut, n, keyBase, shift, table, numTiles, io);
            break;
        case kPayPairLast:
            hipLaunchKernelGGL(RadixScatterKernel<kPayPairLast>, grid, dim3(kBlockThreads), 0, s, keysIn, pairsIn,
                               keysOut, pairsOut, n, keyBase, shift, table, numTiles, io);
            break;
        default:
            hipLaunchKernelGGL(RadixScatterKernel<kPayPair>, grid, dim3(kBlockThreads), 0, s, keysIn, pairsIn, keysOut,
                               pairsOut, n, keyBase, shift, table, numTiles, io);
            break;
    }
}

int64_t WideTiles(int64_t n) { return (n + kWideTile - 1) / kWideTile; }
int64_t WideTableInts(int64_t n) { return static_cast<int64_t>(kWideDigits) * WideTiles(n) + 1; }

// Workgroups of the 8-bit scatter pass: two a compute unit, which is what their LDS allows to be resident.
static uint32_t WideScatterBlocks(int64_t n)
{
    static const int64_t resident = [] {
        int dev = 0;
        hipDeviceProp_t prop;
        int64_t cus = 256;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
            prop.multiProcessorCount > 0) {
            cus = prop.multiProcessorCount;
        } else {
            (void)hipGetLastError();
        }
        const char *env = std::getenv("OPS_SPARSE_WIDE_BLOCKS_PER_CU");  // tuning override
        const int64_t perCu = env != nullptr && std::atoi(env) > 0 ? std::atoi(env) : 2;
        return cus * perCu;
    }();
    const int64_t fullTiles = n / kWideTile;
    return static_cast<uint32_t>(fullTiles < 1 ? 1 : (fullTiles < resident ? fullTiles : resident));
}

// One 8-bit pass carrying csr2csc's (row, value) pairs; table: WideTableInts(n) ints.
void LaunchWidePairPass(int mode, const int32_t *keysIn, const void *pairsIn, int32_t *keysOut, void *pairsOut,
                        int64_t n, int32_t keyBase, int32_t shift, int32_t bits, int32_t *table, int32_t *scratch,
                        const RadixPairIo &io, hipStream_t s)
{
    if (n <= 0) {
        return;
    }
    const int32_t mask = (1 << bits) - 1;
    const int64_t numTiles = WideTiles(n);
    const auto *pin = static_cast<const RadixPair *>(pairsIn);
    auto *pout = static_cast<RadixPair *>(pairsOut);
    LaunchFill(table, 1, 0, s);
    hipLaunchKernelGGL(WideCountKernel, dim3(static_cast<uint32_t>((numTiles + kWideCountTiles - 1) / kWideCountTiles)),
                       dim3(kBlockThreads), 0, s, keysIn, n, keyBase, shift, mask, table, numTiles);
    LaunchInclusiveScan(table, table, WideTableInts(n), 0, scratch, s);
    const auto grid = dim3(WideScatterBlocks(n));
#define OPSPARSE_WIDE_SCATTER(MODE, VB)                                                                              \
    hipLaunchKernelGGL((WideScatterKernel<MODE, VB>), grid, dim3(kBlockThreads), 0, s, keysIn, pin, keysOut, pout, n, \
                       keyBase, shift, mask, table, numTiles, io)
#define OPSPARSE_WIDE_SCATTER_BY_VALUE(MODE)                                                                         \
    switch (io.valueBytes) {                                                                                         \
        case 4: OPSPARSE_WIDE_SCATTER(MODE, 4); break;                                                               \
        case 2: OPSPARSE_WIDE_SCATTER(MODE, 2); break;                                                               \
        case 1: OPSPARSE_WIDE_SCATTER(MODE, 1); break;                                                               \
        default: OPSPARSE_WIDE_SCATTER(MODE, 0); break;                                                              \
    }
    switch (mode) {
        case kPayPairFirst:
            OPSPARSE_WIDE_SCATTER_BY_VALUE(kPayPairFirst);
            break;
        case kPayPairLast:
            OPSPARSE_WIDE_SCATTER_BY_VALUE(kPayPairLast);
            break;
        default:
            OPSPARSE_WIDE_SCATTER(kPayPair, 4);
            break;
    }
#undef OPSPARSE_WIDE_SCATTER_BY_VALUE
#undef OPSPARSE_WIDE_SCATTER
}

void LaunchGatherByPosition(const int32_t *pos, const int32_t *rowOfPos, const uint32_t *srcVal, int64_t nnz,
                            int32_t *rowOut, uint32_t *valOut, hipStream_t s)
{
    if (nnz > 0) {
        hipLaunchKernelGGL(GatherByPositionKernel<uint32_t>, dim3(GridFor(nnz, kBlockThreads)), dim3(kBlockThreads), 0,
                           s, pos, rowOfPos, srcVal, nnz, rowOut, valOut);
    }
}

// ptr[0..m] from sorted (or unsorted) indices: zero, count runs, scan.
void LaunchIndicesToOffsets(const int32_t *ind, int64_t nnz, int64_t m, int32_t base, int32_t *ptr, int32_t *tiles,
                            hipStream_t s)
{
    LaunchFill(ptr, m + 1, 0, s);
    if (nnz > 0 && m > 0) {
        hipLaunchKernelGGL(CountRunsKernel, dim3(GridFor(nnz, kBlockThreads * 8)), dim3(kBlockThreads), 0, s, ind, nnz,
                           m, base, ptr);
    }
    LaunchInclusiveScan(ptr, ptr, m + 1, base, tiles, s);
}

namespace {

int32_t KeyBits(int64_t n)
{
    int32_t bits = 1;
    while (bits < 31 && (int64_t{1} << bits) < n) {
        ++bits;
    }
    return bits;
}

struct Csr2CscLayout {
    int64_t keysA, keysB, payA, payB, rowOfPos, table, tiles, bytes;
    int64_t numTiles, tableCount;
};

Csr2CscLayout LayoutCsr2Csc(int64_t n, int64_t nnz)
{
    Csr2CscLayout l{};
    l.numTiles = (nnz + kWideTile - 1) / kWideTile;
    l.tableCount = static_cast<int64_t>(kWideDigits) * l.numTiles + 1;
    int64_t off = 0;
    const int64_t arr = Align256(4 * nnz);
    l.keysA = off; off += arr;
    l.keysB = off; off += arr;
    l.payA = off; off += Align256(8 * nnz);  // (row, value) pairs
    l.payB = off; off += Align256(8 * nnz);
    l.rowOfPos = off; off += arr;
    l.table = off; off += Align256(4 * l.tableCount);
    const int64_t scanCount = l.tableCount > n + 1 ? l.tableCount : n + 1;
    l.tiles = off; off += Align256(4 * ScanTiles(scanCount));
    l.bytes = off;
    return l;
}

}  // namespace
}  // namespace opsparse

using namespace opsparse;

extern "C" {

size_t opsparse_scan_workspace_bytes(int64_t count)
{
    return count <= 0 ? 0 : static_cast<size_t>(Align256(4 * ScanTiles(count)));
}

int opsparse_coo2csr_launch(const int32_t *cooRowInd, int64_t nnz, int64_t m, int32_t *csrRowPtr, int32_t indexBase,
                            void *workspace, size_t workspaceBytes, void *stream)
{
    if (nnz < 0 || m < 0 || nnz > INT32_MAX || m >= INT32_MAX || (indexBase != 0 && indexBase != 1) ||
        csrRowPtr == nullptr || (nnz > 0 && (cooRowInd == nullptr || m == 0))) {
        return OPSPARSE_E_INVALID;
    }
    if (workspace == nullptr || workspaceBytes < opsparse_scan_workspace_bytes(m + 1)) {
        return OPSPARSE_E_WORKSPACE;
    }
    LaunchIndicesToOffsets(cooRowInd, nnz, m, indexBase, csrRowPtr, static_cast<int32_t *>(workspace),
                           static_cast<hipStream_t>(stream));
    return CheckLaunch();
}

int opsparse_csr2coo_launch(const int32_t *csrRowPtr, int64_t nnz, int64_t m, int32_t *cooRowInd, int32_t indexBase,
                            void *stream)
{
    if (nnz < 0 || m < 0 || nnz > INT32_MAX || m > INT32_MAX || (indexBase != 0 && indexBase != 1) ||
        (m == 0 && nnz != 0) || (m > 0 && csrRowPtr == nullptr) || (nnz > 0 && cooRowInd == nullptr)) {
        return OPSPARSE_E_INVALID;
    }
    if (nnz == 0 || m == 0) {
        return OPSPARSE_OK;
    }
    hipLaunchKernelGGL(ExpandRowsKernel, dim3(GridFor(m, kBlockThreads)), dim3(kBlockThreads), 0,
                       static_cast<hipStream_t>(stream), csrRowPtr, m, nnz, indexBase, cooRowInd);
    return CheckLaunch();
}

// Rows of thousands of entries on average: too few rows to occupy the GPU with a workgroup each (one row of 4 M
// entries: 128 ms that way).  The whole matrix is then sorted with the device-wide radix passes, by column and
// after that, stably, by row, 0.1 - 0.2 ms a pass for such sizes.  The mean is known on the host; a matrix of short
// rows with single very long ones among them still takes the per-row kernels.
constexpr int64_t kSortWholeMeanRow = 4096;

static bool SortWhole(int64_t m, int64_t nnz) { return nnz / m >= kSortWholeMeanRow; }

struct SortWholeLayout {
    int64_t keysA, keysB, pairsA, pairsB, rowOfPos, table, tiles, bytes;
};

static SortWholeLayout LayoutSortWhole(int64_t nnz)
{
    SortWholeLayout l{};
    int64_t off = 0;
    l.keysA = off; off += Align256(4 * nnz);
    l.keysB = off; off += Align256(4 * nnz);
    l.pairsA = off; off += Align256(8 * nnz);
    l.pairsB = off; off += Align256(8 * nnz);
    l.rowOfPos = off; off += Align256(4 * nnz);
    l.table = off; off += Align256(4 * RadixTableInts(nnz));
    l.tiles = off; off += Align256(4 * ScanTiles(RadixTableInts(nnz)));
    l.bytes = off;
    return l;
}

size_t opsparse_csrsort_workspace_bytes(int64_t m, int64_t nnz)
{
    if (m <= 0 || nnz <= 0) {
        return 0;
    }
    if (SortWhole(m, nnz)) {
        return static_cast<size_t>(LayoutSortWhole(nnz).bytes);
    }
    return static_cast<size_t>(2 * Align256(4 * nnz) + 256 + 2 * Align256(4 * m));
}

int opsparse_csrsort_launch(int64_t m, int64_t n, int64_t nnz, int32_t indexBase, const int32_t *csrRowPtr,
                            int32_t *csrColInd, int32_t *perm, void *workspace, size_t workspaceBytes, void *stream)
{
    if (m < 0 || n < 0 || nnz < 0 || m > INT32_MAX || nnz > INT32_MAX || (indexBase != 0 && indexBase != 1) ||
        ((m == 0 || n == 0) && nnz != 0)) {
        return OPSPARSE_E_INVALID;
    }
    if (nnz == 0) {
        return OPSPARSE_OK;
    }
    if (csrRowPtr == nullptr || csrColInd == nullptr || perm == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    if (workspace == nullptr || workspaceBytes < opsparse_csrsort_workspace_bytes(m, nnz)) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto *base = static_cast<unsigned char *>(workspace);
    if (SortWhole(m, nnz)) {
        const SortWholeLayout l = LayoutSortWhole(nnz);
        auto at = [&](int64_t off) { return reinterpret_cast<int32_t *>(base + off); };
        int32_t *keys[2] = {at(l.keysA), at(l.keysB)};
        void *pairs[2] = {base + l.pairsA, base + l.pairsB};
        int32_t *rowOfPos = at(l.rowOfPos), *table = at(l.table), *tiles = at(l.tiles);
        hipLaunchKernelGGL(ExpandRowsKernel, dim3(GridFor(m, kBlockThreads)), dim3(kBlockThreads), 0, s, csrRowPtr, m,
                           nnz, indexBase, rowOfPos);  // rows numbered from indexBase: the order is what matters
        // by column, carrying (row, permutation value) ...
        const RadixPairIo in{rowOfPos, perm, nullptr, nullptr, 4};
        const int32_t colPasses = (KeyBits(n) + kRadixBits - 1) / kRadixBits;
        const int32_t *keysIn = csrColInd;
        const void *pairsIn = nullptr;
        int cur = 0;
        for (int32_t pass = 0; pass < colPasses; ++pass) {
            LaunchRadixPairPass(pass == 0 ? kPayPairFirst : kPayPair, keysIn, pairsIn, keys[cur], pairs[cur], nnz,
                                pass == 0 ? indexBase : 0, pass * kRadixBits, table, tiles, in, s);
            keysIn = keys[cur];
            pairsIn = pairs[cur];
            cur ^= 1;
        }
        // ... then, stably, by row, carrying (column, permutation value); the last pass writes both in place
        hipLaunchKernelGGL(RegroupByRowKernel, dim3(GridFor(nnz, kBlockThreads)), dim3(kBlockThreads), 0, s, keysIn,
                           static_cast<const RadixPair *>(pairsIn), nnz, indexBase, keys[cur],
                           static_cast<RadixPair *>(pairs[cur]));
        keysIn = keys[cur];
        pairsIn = pairs[cur];
        cur ^= 1;
        const RadixPairIo out{nullptr, nullptr, csrColInd, perm, 4};
        const int32_t rowPasses = (KeyBits(m + indexBase) + kRadixBits - 1) / kRadixBits;
        for (int32_t pass = 0; pass < rowPasses; ++pass) {
            LaunchRadixPairPass(pass == rowPasses - 1 ? kPayPairLast : kPayPair, keysIn, pairsIn, keys[cur], pairs[cur],
                                nnz, 0, pass * kRadixBits, table, tiles, out, s);
            keysIn = keys[cur];
            pairsIn = pairs[cur];
            cur ^= 1;
        }
        return CheckLaunch();
    }
    const int64_t arr = Align256(4 * nnz);
    auto *tmpCol = reinterpret_cast<int32_t *>(base);
    auto *tmpPerm = reinterpret_cast<int32_t *>(base + arr);
    auto *counters = reinterpret_cast<int32_t *>(base + 2 * arr);
    auto *midList = reinterpret_cast<int32_t *>(base + 2 * arr + 256);
    auto *longList = reinterpret_cast<int32_t *>(base + 2 * arr + 256 + Align256(4 * m));
    LaunchFill(counters, 3, 0, s);
    // Lanes per row from the mean row length: twice the mean, a power of two in [8, 64].
    const int64_t mean2 = 2 * nnz / m;
    const int g = mean2 <= 8 ? 8 : mean2 <= 16 ? 16 : mean2 <= 32 ? 32 : 64;
    const auto shortGrid = dim3(GridFor(m, static_cast<int64_t>(kBlockThreads / g) * kSortRowsPerGroup));
    // 32-bit keys (column and lane packed) where the columns of a valid matrix leave room for the lane number
    auto packedFor = [&](int lanes) {
        int log = 0;
        while ((1 << log) < lanes) {
            ++log;
        }
        return static_cast<int64_t>(n) + indexBase < (int64_t{1} << (32 - log)) - 1;
    };
#define OPSPARSE_SORT_SHORT(G, PACKED)                                                                              \
    hipLaunchKernelGGL((SortShortRowsKernel<G, PACKED>), shortGrid, dim3(kBlockThreads), 0, s, csrRowPtr, m, nnz,    \
                       indexBase, csrColInd, perm, counters, midList, longList)
#define OPSPARSE_SORT_SHORT_G(G)            \
    if (packedFor(G)) {                     \
        OPSPARSE_SORT_SHORT(G, true);       \
    } else {                                \
        OPSPARSE_SORT_SHORT(G, false);      \
    }
    switch (g) {
        case 8: OPSPARSE_SORT_SHORT_G(8); break;
        case 16: OPSPARSE_SORT_SHORT_G(16); break;
        case 32: OPSPARSE_SORT_SHORT_G(32); break;
        default: OPSPARSE_SORT_SHORT_G(64); break;
    }
#undef OPSPARSE_SORT_SHORT_G
#undef OPSPARSE_SORT_SHORT
    if (g < kSortWaveRow) {
        if (packedFor(kWave)) {
            hipLaunchKernelGGL(SortMidRowsKernel<true>, dim3(kSortListBlocks), dim3(kBlockThreads), 0, s, csrRowPtr,
                               indexBase, csrColInd, perm, counters, midList);
        } else {
            hipLaunchKernelGGL(SortMidRowsKernel<false>, dim3(kSortListBlocks), dim3(kBlockThreads), 0, s, csrRowPtr,
                               indexBase, csrColInd, perm, counters, midList);
        }
    }
    // Listed rows of up to kSortWideRow entries: 256 lanes each, many rows at a time.  The few beyond: 1024 lanes
    // each, because the longest of them is what the call waits for (a row of 1 M entries 12.5 -> 6 ms).
    // (the list of the mid rows has been used up by then: its space takes the rows handed on)
    hipLaunchKernelGGL(SortListedRowsKernel<kBlockThreads>, dim3(kSortListBlocks), dim3(kBlockThreads), 0, s, csrRowPtr,
                       indexBase, KeyBits(n), csrColInd, perm, tmpCol, tmpPerm, counters, longList, 1,
                       int64_t{kSortWideRow}, midList);
    hipLaunchKernelGGL(SortListedRowsKernel<1024>, dim3(kSortListBlocks / 4), dim3(1024), 0, s, csrRowPtr, indexBase,
                       KeyBits(n), csrColInd, perm, tmpCol, tmpPerm, counters, midList, 2, int64_t{INT32_MAX},
                       static_cast<int32_t *>(nullptr));
    return CheckLaunch();
}

size_t opsparse_csr2csc_workspace_bytes(int64_t m, int64_t n, int64_t nnz)
{
    if (m <= 0 || n <= 0 || nnz <= 0) {
        return 0;
    }
    return static_cast<size_t>(LayoutCsr2Csc(n, nnz).bytes);
}

int opsparse_csr2csc_launch(int64_t m, int64_t n, int64_t nnz, const void *csrVal, const int32_t *csrRowPtr,
                            const int32_t *csrColInd, void *cscVal, int32_t *cscColPtr, int32_t *cscRowInd,
                            int32_t valueBytes, int32_t indexBase, void *workspace, size_t workspaceBytes,
                            void *stream)
{
    if (m < 0 || n < 0 || nnz < 0 || m > INT32_MAX || n >= INT32_MAX || nnz > INT32_MAX - indexBase ||
        (indexBase != 0 && indexBase != 1) || ((m == 0 || n == 0) && nnz != 0) || cscColPtr == nullptr ||
        (valueBytes != 0 && valueBytes != 1 && valueBytes != 2 && valueBytes != 4)) {
        return OPSPARSE_E_INVALID;
    }
    auto s = static_cast<hipStream_t>(stream);
    if (nnz == 0) {
        LaunchFill(cscColPtr, n + 1, indexBase, s);
        return CheckLaunch();
    }
    if (csrRowPtr == nullptr || csrColInd == nullptr || cscRowInd == nullptr ||
        (valueBytes != 0 && (csrVal == nullptr || cscVal == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    const Csr2CscLayout l = LayoutCsr2Csc(n, nnz);
    if (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto *base = static_cast<unsigned char *>(workspace);
    auto at = [&](int64_t off) { return reinterpret_cast<int32_t *>(base + off); };
    int32_t *keys[2] = {at(l.keysA), at(l.keysB)};
    void *pairs[2] = {base + l.payA, base + l.payB};
    int32_t *rowOfPos = at(l.rowOfPos), *table = at(l.table), *tiles = at(l.tiles);

    // Row index of every source position, with the output's index base.
    hipLaunchKernelGGL(ExpandRowsKernel, dim3(GridFor(m, kBlockThreads)), dim3(kBlockThreads), 0, s, csrRowPtr, m, nnz,
                       indexBase, rowOfPos);

    // Stable sort by column of (column; row, value): the pair travels with its key, 8 bytes a pass and entry more
    // than a source position would, and the last pass writes rows and values where they belong — no gather by
    // position at the end, which cost two cache-line fills per entry (33.5 M entries: 2.9 -> 1.9 ms).
    // Up to eight bits a pass, the tile ordered through LDS before it leaves (33.5 M entries over 2^20 columns:
    // three passes instead of five, 1.2 ms).
    const int32_t keyBits = KeyBits(n);
    int32_t passes = (keyBits + kWideBits - 1) / kWideBits;
    passes = passes < 2 ? 2 : passes;  // a first pass that reads the sources and a last one that writes the outputs
    // the passes share the key's bits evenly (20 bits: 7, 7, 6 rather than 8, 8, 4): the fewer buckets a pass has,
    // the longer the runs its tiles write, and short runs are what the memory side is slow at
    const int32_t perPass = (keyBits + passes - 1) / passes;
    const RadixPairIo io{rowOfPos, csrVal, cscRowInd, cscVal, valueBytes};
    const int32_t *keysIn = csrColInd;
    const void *pairsIn = nullptr;
    int cur = 0;
    for (int32_t pass = 0; pass < passes; ++pass) {
        const int mode = pass == 0 ? kPayPairFirst : (pass == passes - 1 ? kPayPairLast : kPayPair);
        LaunchWidePairPass(mode, keysIn, pairsIn, keys[cur], pairs[cur], nnz, pass == 0 ? indexBase : 0,
                           pass * perPass, perPass, table, tiles, io, s);
        keysIn = keys[cur];
        pairsIn = pairs[cur];
        cur ^= 1;
    }

    // Column offsets from the sorted (zero-based) columns.
    LaunchFill(cscColPtr, n + 1, 0, s);
    hipLaunchKernelGGL(CountRunsKernel, dim3(GridFor(nnz, kBlockThreads * 8)), dim3(kBlockThreads), 0, s, keysIn, nnz,
                       n, 0, cscColPtr);
    LaunchInclusiveScan(cscColPtr, cscColPtr, n + 1, indexBase, tiles, s);
    return CheckLaunch();
}


// ------------------------------------------------------------------ coosort
//
// aclsparseXcoosortByRow / ByColumn (sparse/coosort/arch35/coosort_host.cpp:309-371; the order is the one of
// test/coosort/arch35/coosort_golden.h:52-85): a stable sort of (primary, secondary, P) triples, signed keys,
// ascending in the primary key and, among equal ones, in the secondary.  Least-significant-key first: the 8-bit
// passes of csr2csc over the secondary key, the primary key and P travelling as the pair, then over the primary
// key with the secondary key and P as the pair; the last pass writes the caller's three arrays.  The keys are
// taken relative to their minimum, found on the device first, so that a pass count follows from the range the
// indices really span (one read-back of four integers: the call synchronises its stream once).

}  // extern "C"

namespace opsparse {
namespace {

// range[0..3] = min / max of a[], min / max of b[] (pre-filled with INT32_MAX / INT32_MIN alternately).
__global__ __launch_bounds__(kBlockThreads) void CooRangeKernel(const int32_t *__restrict__ a,
                                                                const int32_t *__restrict__ b, int64_t n,
                                                                int32_t *__restrict__ range)
{
    int32_t lo[2] = {INT32_MAX, INT32_MAX}, hi[2] = {INT32_MIN, INT32_MIN};
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int32_t v[2] = {a[i], b[i]};
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            lo[k] = v[k] < lo[k] ? v[k] : lo[k];
            hi[k] = v[k] > hi[k] ? v[k] : hi[k];
        }
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const int32_t l = __shfl_xor(lo[k], off), h = __shfl_xor(hi[k], off);
            lo[k] = l < lo[k] ? l : lo[k];
            hi[k] = h > hi[k] ? h : hi[k];
        }
    }
    // one set of atomics a workgroup (a set a wavefront of 8192 workgroups took 1.2 ms on four addresses)
    __shared__ int32_t part[kBlockThreads / kWave][4];
    if (threadIdx.x % kWave == 0) {
        int32_t *mine = part[threadIdx.x / kWave];
        mine[0] = lo[0];
        mine[1] = hi[0];
        mine[2] = lo[1];
        mine[3] = hi[1];
    }
    __syncthreads();
    if (threadIdx.x < 4) {
        int32_t v = part[0][threadIdx.x];
        for (int w = 1; w < kBlockThreads / kWave; ++w) {
            const int32_t o = part[w][threadIdx.x];
            v = (threadIdx.x & 1) ? (o > v ? o : v) : (o < v ? o : v);
        }
        if (threadIdx.x & 1) {
            atomicMax(range + threadIdx.x, v);
        } else {
            atomicMin(range + threadIdx.x, v);
        }
    }
}

__global__ __launch_bounds__(kBlockThreads) void CooRangeInitKernel(int32_t *range)
{
    if (threadIdx.x < 4) {
        range[threadIdx.x] = (threadIdx.x & 1) ? INT32_MIN : INT32_MAX;
    }
}

// a[i] += addA, b[i] += addB (wrap-around: the sorted keys come back relative to their minimum).
__global__ __launch_bounds__(kBlockThreads) void CooRebaseKernel(int32_t *__restrict__ a, int32_t *__restrict__ b,
                                                                 int64_t n, int32_t addA, int32_t addB)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        a[i] = static_cast<int32_t>(static_cast<uint32_t>(a[i]) + static_cast<uint32_t>(addA));
        b[i] = static_cast<int32_t>(static_cast<uint32_t>(b[i]) + static_cast<uint32_t>(addB));
    }
}

struct CoosortLayout {
    int64_t range, keysA, keysB, pairsA, pairsB, table, tiles, bytes;
};

CoosortLayout LayoutCoosort(int64_t nnz)
{
    CoosortLayout l{};
    int64_t off = 0;
    l.range = off; off += 256;
    l.keysA = off; off += Align256(4 * nnz);
    l.keysB = off; off += Align256(4 * nnz);
    l.pairsA = off; off += Align256(8 * nnz);
    l.pairsB = off; off += Align256(8 * nnz);
    l.table = off; off += Align256(4 * WideTableInts(nnz));
    l.tiles = off; off += Align256(4 * ScanTiles(WideTableInts(nnz)));
    l.bytes = off;
    return l;
}

// Bits that hold hi - lo (both int32, hi >= lo), at least 1.
int32_t RangeBits(int32_t lo, int32_t hi)
{
    const uint32_t span = static_cast<uint32_t>(hi) - static_cast<uint32_t>(lo);
    int32_t bits = 1;
    while (bits < 32 && (span >> bits) != 0) {
        ++bits;
    }
    return bits;
}

}  // namespace
}  // namespace opsparse

extern "C" {

size_t opsparse_coosort_workspace_bytes(int64_t nnz)
{
    return nnz <= 0 ? 0 : static_cast<size_t>(LayoutCoosort(nnz).bytes);
}

int opsparse_coosort_launch(int64_t nnz, int32_t byRow, int32_t *cooRows, int32_t *cooCols, int32_t *perm,
                            void *workspace, size_t workspaceBytes, void *stream)
{
    if (nnz < 0 || nnz > INT32_MAX) {
        return OPSPARSE_E_INVALID;
    }
    if (nnz == 0) {
        return OPSPARSE_OK;
    }
    if (cooRows == nullptr || cooCols == nullptr || perm == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    const CoosortLayout l = LayoutCoosort(nnz);
    if (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto *base = static_cast<unsigned char *>(workspace);
    auto at = [&](int64_t off) { return reinterpret_cast<int32_t *>(base + off); };
    int32_t *keys[2] = {at(l.keysA), at(l.keysB)};
    void *pairs[2] = {base + l.pairsA, base + l.pairsB};
    int32_t *table = at(l.table), *tiles = at(l.tiles), *range = at(l.range);
    int32_t *primary = byRow != 0 ? cooRows : cooCols, *secondary = byRow != 0 ? cooCols : cooRows;

    hipLaunchKernelGGL(CooRangeInitKernel, dim3(1), dim3(kBlockThreads), 0, s, range);
    hipLaunchKernelGGL(CooRangeKernel, dim3(GridFor(nnz, kBlockThreads * 16, 2048)), dim3(kBlockThreads), 0, s, primary,
                       secondary, nnz, range);
    int32_t r[4] = {0, 0, 0, 0};  // min / max of the primary key, of the secondary key
    if (hipMemcpyAsync(r, range, sizeof(r), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }

    int cur = 0;
    // One key's passes: the first reads (key, pair) from three arrays, the last writes three arrays.
    auto sortBy = [&](const int32_t *keySrc, int32_t keyBase, int32_t bits, const int32_t *pairRowSrc,
                      const void *pairValSrc, int32_t *keyDst, int32_t *pairRowDst, void *pairValDst) {
        int32_t passes = (bits + kWideBits - 1) / kWideBits;
        passes = passes < 2 ? 2 : passes;
        const int32_t perPass = (bits + passes - 1) / passes;
        const RadixPairIo io{pairRowSrc, pairValSrc, pairRowDst, pairValDst, 4};
        const int32_t *keysIn = keySrc;
        const void *pairsIn = nullptr;
        for (int32_t pass = 0; pass < passes; ++pass) {
            const bool last = pass == passes - 1;
            const int mode = pass == 0 ? kPayPairFirst : (last ? kPayPairLast : kPayPair);
            int32_t *keysOut = last ? keyDst : keys[cur];
            LaunchWidePairPass(mode, keysIn, pairsIn, keysOut, pairs[cur], nnz, pass == 0 ? keyBase : 0, pass * perPass,
                               perPass, table, tiles, io, s);
            keysIn = keysOut;
            pairsIn = pairs[cur];
            cur ^= 1;
        }
    };
    // by the secondary key, (primary key, P) as the pair: the result stays in the workspace ...
    int32_t *midKeys = keys[1];                                   // (two or four passes: the last one writes buffer 1
    auto *midRows = static_cast<int32_t *>(pairs[1]);             //  only when their number is even)
    const int32_t bitsS = RangeBits(r[2], r[3]), bitsP = RangeBits(r[0], r[1]);
    const int32_t passesS = (bitsS + kWideBits - 1) / kWideBits < 2 ? 2 : (bitsS + kWideBits - 1) / kWideBits;
    const int lastBuf = (passesS - 1) & 1;                        // buffer the last pass of that stage writes
    midKeys = keys[lastBuf];
    midRows = static_cast<int32_t *>(pairs[lastBuf]);
    uint32_t *midVals = reinterpret_cast<uint32_t *>(pairs[lastBuf]) + nnz;
    sortBy(secondary, r[2], bitsS, primary, perm, midKeys, midRows, midVals);
    // ... then, stably, by the primary key, (secondary key, P) as the pair, into the caller's arrays
    sortBy(midRows, r[0], bitsP, midKeys, midVals, primary, secondary, perm);
    if (r[0] != 0 || r[2] != 0) {
        hipLaunchKernelGGL(CooRebaseKernel, dim3(GridFor(nnz, kBlockThreads * 8)), dim3(kBlockThreads), 0, s, primary,
                           secondary, nnz, r[0], r[2]);
    }
    return CheckLaunch();
}

}  // extern "C"
