// SCATTER_LIVE: y = alpha * A^T x + beta * y for a CSR matrix whose y does not fit a cache, live values.
//
// Takes the place of the reference's transposed kernel, which adds every product to y with an atomic
// (sparse/spmv/arch22/kernels/spmv_kernel.cpp:21-55, SpmvKernelTrans): with scattered columns every such update
// moves a whole line of y for 4 useful bytes.  Here y is only ever updated in LDS, and what goes through memory are
// streams.  It is the mirror image of the blocked-gather layout of op(A) = A: there x, the small operand, is
// brought to the entries through LDS; here the products are brought to y.
//
//   pass 1   a workgroup takes a PIECE of consecutive entries of the caller's arrays (128 KiB of products: 16 384
//            entries of fp32 values, 32 768 of fp16 / bf16): values (as they are at this call) and, from the layout,
//            each entry's row and its slot in the piece sorted by output panel (2^14 columns of A = 128 KiB of fp64
//            sums).  It multiplies by x[row] - consecutive entries share rows, so these loads are as good as linear
//            - drops the product at its slot of a staging area in LDS, and writes the staging area out one (panel,
//            piece) chunk at a time: the products arrive in memory sorted by panel, a panel's in the order of the
//            caller's arrays.  A product is kept exactly: fp64 for fp32 operands, fp32 for 16-bit ones.
//   pass 2   a workgroup takes an output panel: it streams the panel's products and their local columns (2 bytes
//            an entry, from the layout) and adds each product to its column's fp64 sum in LDS with an LDS atomic,
//            then writes y = alpha * sum + beta * y for the panel's columns.
//
// 26 bytes an entry (fp32: 8 read and 8 written, then 10 read) in two linear passes against 8 algorithmic bytes and
// two line transfers of y per entry.  The buffer holds no value of the matrix: csrValues may change between calls,
// the structure may not.  The order of the additions into a column's sum depends on scheduling (the reference's
// atomics on y do too); the products are exact, the sums fp64 and rounded once, so two calls differ at most in the
// last bit of an element, and every element is within an fp32 rounding of the exact result.
//
// Preprocessing (once per structure, on the device): a stable radix sort of the entries on the panel number gives
// the order of the products in memory; because it is stable and a piece is a range of the caller's order, the
// entries of one piece in one panel are a contiguous chunk of it, and a table of chunk sizes, summed both ways,
// gives every chunk's place in memory and in the piece's staging area.
#include <climits>
#include <cstdlib>

#include "convert_internal.h"
#include "device_utils.h"
#include "spmv_internal.h"

namespace opsparse {
namespace scatter_layout {

constexpr int kThreads = 1024;                  // one workgroup a compute unit: it owns 128 KiB of LDS and more
constexpr int kOutLog = 14;                     // columns of A per output panel: 128 KiB of fp64 sums
constexpr int kOutCols = 1 << kOutLog;
constexpr int kStageBytes = 128 << 10;          // the products of a piece staged in LDS
constexpr int kMaxPanels = 2048;                // the chunk tables of a piece in LDS: 16 KiB
constexpr int64_t kMinPanels = 128;             // fewer output panels would leave compute units idle in pass 2
constexpr int64_t kMaxChunks = int64_t{1} << 26;  // panels x pieces: the chunk tables
// A column with more entries than this is left to the ordered layout over the transposed copy, which sums such a
// column as a long row: here all its products would queue for one address of LDS.
constexpr int32_t kMaxColumnEntries = 8192;

typedef float Float4 __attribute__((ext_vector_type(4)));
typedef uint32_t Uint4 __attribute__((ext_vector_type(4)));
typedef unsigned short Ushort4 __attribute__((ext_vector_type(4)));

struct ScatterLayout {
    int32_t P, Q;  // output panels, pieces (0 panels: the layout does not apply)
    int32_t piece;  // entries of a piece
    // what the launches use (the first `resident` bytes)
    int64_t metaOff;       // uint32 per entry: slot in the piece's panel order | (row - first row of the piece) << 16
    int64_t colLocalOff;   // uint16 per product in panel order: column - first column of the panel
    int64_t interOff;      // the products in panel order (fp64 or fp32), rewritten by every call
    int64_t chunkDstOff;   // [Q][P] first position in panel order of the chunk (panel, piece)
    int64_t pieceBaseOff;  // [Q][P + 1] first slot of the chunk in the piece's staging area
    int64_t pieceRowOff;   // [Q] row of the piece's first entry
    int64_t panelStartOff; // [P + 1]
    int64_t resident;
    // the analysis only
    int64_t keys0Off, keys1Off, pay0Off, pay1Off, rowIndOff, dstOfOff, countOff, inclOff, tableOff, scanOff;
    int64_t bytes;
};

int64_t MinPanels()
{
    const char *env = std::getenv("OPS_SPARSE_SCATTER_MIN_PANELS");  // tuning override, read at every call
    return env != nullptr ? std::atoll(env) : kMinPanels;
}

// Bytes of a product that is exact: fp32 x fp32 needs fp64, 16-bit operands fit fp32.
inline int ProductBytes(int32_t valueType)
{
    return valueType == OPSPARSE_F32 ? 8 : 4;
}

int32_t ValueTypeOf(int32_t flags)
{
    return (flags & OPSPARSE_BLOCKED_VALUES_F16) != 0    ? OPSPARSE_F16
           : (flags & OPSPARSE_BLOCKED_VALUES_BF16) != 0 ? OPSPARSE_BF16
                                                         : OPSPARSE_F32;
}

// Layout for A with `rows` rows, `cols` columns (the outputs) and nnz entries of `valueType`.
ScatterLayout MakeLayout(int64_t rows, int64_t cols, int64_t nnz, int32_t valueType)
{
    ScatterLayout l{};
    if (rows <= 0 || cols <= 0 || nnz <= 0 || nnz > INT32_MAX - 65536 || rows >= INT32_MAX || cols > (int64_t{1} << 25)) {
        return l;
    }
    const int64_t P = (cols + kOutCols - 1) >> kOutLog;
    const int pb = ProductBytes(valueType);
    const int64_t piece = kStageBytes / pb;
    const int64_t Q = (nnz + piece - 1) / piece;
    if (P < MinPanels() || P > kMaxPanels || P * Q > kMaxChunks) {
        return l;
    }
    l.P = static_cast<int32_t>(P);
    l.Q = static_cast<int32_t>(Q);
    l.piece = static_cast<int32_t>(piece);
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    int64_t off = 256;  // header: status words of the analysis
    l.metaOff = off; off += align(4 * nnz + 16);
    l.colLocalOff = off; off += align(2 * nnz + 16);   // (pass 2 reads whole groups of four)
    l.interOff = off; off += align(pb * nnz + 64);
    l.chunkDstOff = off; off += align(4 * P * Q);
    l.pieceBaseOff = off; off += align(4 * (P + 1) * Q);
    l.pieceRowOff = off; off += align(4 * Q);
    l.panelStartOff = off; off += align(4 * (P + 1));
    l.resident = off;
    l.keys0Off = off; off += align(4 * nnz);
    l.keys1Off = off; off += align(4 * nnz);
    l.pay0Off = off; off += align(4 * nnz);
    l.pay1Off = off; off += align(4 * nnz);
    l.rowIndOff = off; off += align(4 * nnz);
    l.dstOfOff = off; off += align(4 * nnz);
    l.countOff = off; off += align(4 * (P * Q + 1));
    l.inclOff = off; off += align(4 * (P * Q + 1));
    l.tableOff = off; off += align(4 * RadixTableInts(nnz));
    const int64_t scanA = ScanScratchInts(RadixTableInts(nnz)), scanB = ScanScratchInts(P * Q + 1);
    l.scanOff = off; off += align(4 * (scanA > scanB ? scanA : scanB));
    l.bytes = off;
    return l;
}

inline uint32_t GridOf(int64_t items, int64_t perBlock, int64_t cap)
{
    int64_t g = (items + perBlock - 1) / perBlock;
    g = g > cap ? cap : g;
    return static_cast<uint32_t>(g < 1 ? 1 : g);
}

// ---------------------------------------------------------------------------------------------- analysis kernels

// status[0] |= 1 for a column index outside [0, cols).
__global__ __launch_bounds__(kBlockThreads) void ColumnRangeKernel(const int32_t *__restrict__ colInd, int64_t nnz, int64_t cols,
                                                                   int32_t *__restrict__ status)
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

// A workgroup a panel: status[1] = entries of the fullest column, counted in LDS over the panel's sorted columns.
__global__ __launch_bounds__(kThreads) void ColumnMaxKernel(const uint16_t *__restrict__ colLocal,
                                                            const int32_t *__restrict__ panelStart,
                                                            int32_t *__restrict__ status)
{
    __shared__ int32_t count[kOutCols];
    const int t = threadIdx.x;
    for (int32_t c = t; c < kOutCols; c += kThreads) {
        count[c] = 0;
    }
    __syncthreads();
    const int32_t s0 = panelStart[blockIdx.x], s1 = panelStart[blockIdx.x + 1];
    for (int32_t s = s0 + t; s < s1; s += kThreads) {
        atomicAdd(&count[colLocal[s]], 1);
    }
    __syncthreads();
    int32_t most = 0;
    for (int32_t c = t; c < kOutCols; c += kThreads) {
        most = count[c] > most ? count[c] : most;
    }
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int32_t other = __shfl_xor(most, off, kWave);
        most = other > most ? other : most;
    }
    if (t % kWave == 0 && most > 0) {
        atomicMax(status + 1, most);
    }
}

// From the entries sorted by panel (key = column, payload = entry of the caller's arrays): the local column of every
// product, where every entry's product goes, and the number of entries of every (panel, piece) chunk.  A thread
// takes eight consecutive sorted entries, which mostly share a chunk, and counts a run of them with one atomic.
__global__ __launch_bounds__(kBlockThreads) void ChunkCountKernel(const int32_t *__restrict__ sortedCol,
                                                                  const int32_t *__restrict__ sortedEntry, int64_t nnz, int32_t Q,
                                                                  int32_t piece, uint16_t *__restrict__ colLocal,
                                                                  int32_t *__restrict__ dstOf, int32_t *__restrict__ count)
{
    constexpr int kRun = 8;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * kRun;
    for (int64_t s0 = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * kRun; s0 < nnz; s0 += stride) {
        int64_t chunk = -1;
        int32_t run = 0;
        for (int j = 0; j < kRun && s0 + j < nnz; ++j) {
            const int64_t s = s0 + j;
            const int32_t c = sortedCol[s], i = sortedEntry[s];
            colLocal[s] = static_cast<uint16_t>(c & (kOutCols - 1));
            dstOf[i] = static_cast<int32_t>(s);
            const int64_t at = static_cast<int64_t>(c >> kOutLog) * Q + i / piece;
            if (at != chunk) {
                if (run > 0) {
                    atomicAdd(count + chunk, run);
                }
                chunk = at;
                run = 0;
            }
            ++run;
        }
        if (run > 0) {
            atomicAdd(count + chunk, run);
        }
    }
}

// One wavefront a piece: the chunk tables of the piece from the counts (count[p * Q + q]) and their running sums in
// (panel, piece) order (incl, inclusive), and the row of its first entry.
__global__ __launch_bounds__(kWave) void PieceTablesKernel(const int32_t *__restrict__ count, const int32_t *__restrict__ incl,
                                                           const int32_t *__restrict__ rowInd, int32_t P, int32_t Q, int32_t piece,
                                                           int64_t nnz, int32_t *__restrict__ chunkDst, int32_t *__restrict__ pieceBase,
                                                           int32_t *__restrict__ pieceRow, int32_t *__restrict__ panelStart)
{
    const int32_t q = blockIdx.x;
    const int lane = threadIdx.x;
    int32_t running = 0;
    for (int32_t p0 = 0; p0 < P; p0 += kWave) {
        const int32_t p = p0 + lane;
        const int64_t at = static_cast<int64_t>(p) * Q + q;
        const int32_t c = p < P ? count[at] : 0;
        int32_t sum = c;
        for (int off = 1; off < kWave; off <<= 1) {
            const int32_t up = __shfl_up(sum, off, kWave);
            sum += lane >= off ? up : 0;
        }
        if (p < P) {
            pieceBase[static_cast<int64_t>(q) * (P + 1) + p] = running + sum - c;
            const int32_t first = incl[at] - c;
            chunkDst[static_cast<int64_t>(q) * P + p] = first;
            if (q == 0) {
                panelStart[p] = first;
            }
        }
        running += __shfl(sum, kWave - 1, kWave);
    }
    if (lane == 0) {
        pieceBase[static_cast<int64_t>(q) * (P + 1) + P] = running;
        pieceRow[q] = rowInd[static_cast<int64_t>(q) * piece];
        if (q == 0) {
            panelStart[P] = static_cast<int32_t>(nnz);
        }
    }
}

// meta of every entry: its slot in the piece's staging area and its row relative to the piece's first.
// status[0] |= 2 where a piece spans more than 65 535 rows (runs of empty rows inside it).
__global__ __launch_bounds__(kBlockThreads) void EntryMetaKernel(const int32_t *__restrict__ colInd, const int32_t *__restrict__ rowInd,
                                                                 const int32_t *__restrict__ dstOf, const int32_t *__restrict__ chunkDst,
                                                                 const int32_t *__restrict__ pieceBase,
                                                                 const int32_t *__restrict__ pieceRow, int64_t nnz, int32_t P,
                                                                 int32_t piece, uint32_t *__restrict__ meta,
                                                                 int32_t *__restrict__ status)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    bool wide = false;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const int64_t q = i / piece;
        const int32_t p = colInd[i] >> kOutLog;
        const int32_t slot = pieceBase[q * (P + 1) + p] + dstOf[i] - chunkDst[q * P + p];
        const int32_t rel = rowInd[i] - pieceRow[q];
        wide = wide || rel > 65535;
        meta[i] = static_cast<uint32_t>(slot) | (static_cast<uint32_t>(rel) << 16);
    }
    if (wide) {
        atomicOr(status, 2);
    }
}

// ---------------------------------------------------------------------------------------------- the two passes

template <typename ValT>
__device__ __forceinline__ void LoadFour(const ValT *p, float out[4]);
template <>
__device__ __forceinline__ void LoadFour<float>(const float *p, float out[4])
{
    const Float4U v = __builtin_nontemporal_load(reinterpret_cast<const Float4U *>(p));
    out[0] = v.x, out[1] = v.y, out[2] = v.z, out[3] = v.w;
}
template <>
__device__ __forceinline__ void LoadFour<Half>(const Half *p, float out[4])
{
    const Short4U v = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(p));
    for (int j = 0; j < 4; ++j) {
        const uint16_t bits = v[j];
        Half h;
        __builtin_memcpy(&h, &bits, 2);
        out[j] = static_cast<float>(h);
    }
}
template <>
__device__ __forceinline__ void LoadFour<Bf16>(const Bf16 *p, float out[4])
{
    const Short4U v = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(p));
    for (int j = 0; j < 4; ++j) {
        out[j] = __uint_as_float(static_cast<uint32_t>(v[j]) << 16);
    }
}

template <typename ValT>
__device__ __forceinline__ float WidenOne(ValT v)
{
    return static_cast<float>(ToAcc<double, ValT>(v));
}

// Pass 1: the products of the pieces blockIdx.x, blockIdx.x + gridDim.x, ... written to `inter` in panel order.  One
// workgroup a compute unit (the staging area is most of its LDS), so nothing else would cover the time a piece's
// loads are on their way: the workgroup asks for the next piece's values and slots before it writes the current one
// out (one piece after the other: 309 us on the 8 M x 8 M power-law matrix).
template <typename ValT, typename ProdT>
__global__ __launch_bounds__(kThreads) void ScatterProductsKernel(const ValT *__restrict__ vals, const ValT *__restrict__ x,
                                                                  const uint32_t *__restrict__ meta,
                                                                  const int32_t *__restrict__ chunkDst,
                                                                  const int32_t *__restrict__ pieceBase,
                                                                  const int32_t *__restrict__ pieceRow, int64_t nnz, int32_t P,
                                                                  int32_t Q, ProdT *__restrict__ inter)
{
    constexpr int kPiece = kStageBytes / static_cast<int>(sizeof(ProdT));
    constexpr int kRounds = kPiece / (kThreads * 4);  // a thread takes 4 consecutive entries a round
    __shared__ __align__(16) ProdT stage[kPiece];
    __shared__ int32_t base[kMaxPanels + 1];
    __shared__ int32_t dst[kMaxPanels];
    const int t = threadIdx.x;
    const int wave = t / kWave, lane = t % kWave;
    Uint4 m[kRounds];
    float v[kRounds][4];
    // values and slots of piece q into registers: every load is issued whatever the piece's length (those past its end
    // re-read its first entries and are not used), so that none waits for another
    auto fetch = [&](int32_t q) {
        const int64_t first = static_cast<int64_t>(q) * kPiece;
        const int32_t count = nnz - first < kPiece ? static_cast<int32_t>(nnz - first) : kPiece;
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const int32_t k = (r * kThreads + t) * 4;
            if (k + 4 <= count) {
                m[r] = __builtin_nontemporal_load(reinterpret_cast<const Uint4 *>(meta + first + k));
                LoadFour<ValT>(vals + first + k, v[r]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool in = k + j < count;
                    m[r][j] = in ? meta[first + k + j] : 0u;
                    v[r][j] = in ? WidenOne<ValT>(vals[first + k + j]) : 0.0f;
                }
            }
        }
    };
    int32_t q = blockIdx.x;
    if (q < Q) {
        fetch(q);
    }
    for (; q < Q; q += gridDim.x) {
        const int64_t first = static_cast<int64_t>(q) * kPiece;
        const int32_t count = nnz - first < kPiece ? static_cast<int32_t>(nnz - first) : kPiece;
        for (int32_t p = t; p <= P; p += kThreads) {
            base[p] = pieceBase[static_cast<int64_t>(q) * (P + 1) + p];
        }
        for (int32_t p = t; p < P; p += kThreads) {
            dst[p] = chunkDst[static_cast<int64_t>(q) * P + p];
        }
        const ValT *xRow = x + pieceRow[q];
        float xv[kRounds][4];
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const int32_t k = (r * kThreads + t) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                xv[r][j] = k + j < count ? WidenOne<ValT>(xRow[m[r][j] >> 16]) : 0.0f;
            }
        }
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const int32_t k = (r * kThreads + t) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (k + j < count) {
                    stage[m[r][j] & 0xffffu] = static_cast<ProdT>(v[r][j]) * static_cast<ProdT>(xv[r][j]);
                }
            }
        }
        __syncthreads();
        if (q + static_cast<int32_t>(gridDim.x) < Q) {
            fetch(q + static_cast<int32_t>(gridDim.x));
        }
        // a wavefront a chunk: the piece's products of one panel, contiguous in the staging area and in memory
        // (four chunks at a time, their look-ups and LDS reads issued together, changed nothing: the kernel runs at
        // the rate at which memory takes 256-byte pieces written to 512 places at once, 3.9 TB/s for reads and writes
        // together, where the radix passes of the analysis, with 16 places, reach 2.6)
        for (int32_t p = wave; p < P; p += kThreads / kWave) {
            const int32_t s0 = base[p], s1 = base[p + 1];
            ProdT *out = inter + dst[p];
            for (int32_t k = s0 + lane; k < s1; k += kWave) {
                out[k - s0] = stage[k];
            }
        }
        __syncthreads();
    }
}

// Pass 2: the sums of output panel blockIdx.x, and its part of y.
template <typename OutT, typename ProdT>
__global__ __launch_bounds__(kThreads) void ScatterSumKernel(const ProdT *__restrict__ inter, const uint16_t *__restrict__ colLocal,
                                                             const int32_t *__restrict__ panelStart, OutT *__restrict__ y,
                                                             const OutT *__restrict__ yIn, int64_t cols, OpsparseScalar alphaS,
                                                             OpsparseScalar betaS)
{
    __shared__ __align__(16) double acc[kOutCols];
    const int32_t p = blockIdx.x;
    const int t = threadIdx.x;
    for (int32_t c = t; c < kOutCols; c += kThreads) {
        acc[c] = 0.0;
    }
    __syncthreads();
    const int32_t s0 = panelStart[p], s1 = panelStart[p + 1];
    // groups of four positions (the arrays start at multiples of 256 bytes, so a group is one aligned load each);
    // the first and last group of a panel are shared with its neighbours
    constexpr int kDepth = 4;
    for (int32_t e = (s0 & ~3) + t * 4; e < s1; e += kThreads * 4 * kDepth) {
        typedef ProdT Prod4 __attribute__((ext_vector_type(4)));
        Prod4 v[kDepth];
        Ushort4 c[kDepth];
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int32_t at = e + d * kThreads * 4;
            if (at < s1) {
                v[d] = __builtin_nontemporal_load(reinterpret_cast<const Prod4 *>(inter + at));
                c[d] = __builtin_nontemporal_load(reinterpret_cast<const Ushort4 *>(colLocal + at));
            }
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int32_t at = e + d * kThreads * 4;
            if (at < s1) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (at + j >= s0 && at + j < s1) {
                        atomicAdd(&acc[c[d][j]], static_cast<double>(v[d][j]));
                    }
                }
            }
        }
    }
    __syncthreads();
    const double alpha = ReadScalar<double>(alphaS), beta = ReadScalar<double>(betaS);
    const int64_t c0 = static_cast<int64_t>(p) << kOutLog;
    for (int32_t c = t; c < kOutCols && c0 + c < cols; c += kThreads) {
        double r = alpha * acc[c];
        if (beta != 0.0) {
            r += beta * ToAcc<double, OutT>(yIn[c0 + c]);
        }
        y[c0 + c] = FromAcc<OutT, double>(r);
    }
}

// Compute units of the current device (256 on MI355X), asked once.
int32_t ComputeUnits()
{
    static const int32_t cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            return 256;
        }
        return n;
    }();
    return cus;
}

// a.rows / a.cols: rows and columns of A; x has a.rows elements, y a.cols.
int Launch(const SpmvArgs &a, const OpsparseSpmvPlan &plan, int32_t valType, int32_t outType)
{
    if (plan.valueType != valType || plan.transposed == 0 || plan.liveValues == 0) {
        return OPSPARSE_E_INVALID;  // the plan was made for values of another type, or is not one of these
    }
    if (outType != OPSPARSE_F32 && outType != valType) {
        return OPSPARSE_E_UNSUPPORTED;  // y is fp32, or of the 16-bit type of the values
    }
    const ScatterLayout l = MakeLayout(a.rows, a.cols, a.nnz, valType);
    if (l.P == 0 || plan.numPanels != l.P || plan.numRowBlocks != l.Q || plan.entryWindow != l.piece) {
        return OPSPARSE_E_INVALID;
    }
    if (a.ws == nullptr || static_cast<int64_t>(a.wsBytes) < l.resident || plan.bytes != l.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    if (a.vals == nullptr || a.x == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    auto *base = static_cast<unsigned char *>(a.ws);
    auto ints = [&](int64_t off) { return reinterpret_cast<const int32_t *>(base + off); };
    const auto *meta = reinterpret_cast<const uint32_t *>(base + l.metaOff);
    const auto *colLocal = reinterpret_cast<const uint16_t *>(base + l.colLocalOff);
    void *inter = base + l.interOff;
    auto products = [&](auto valTag, auto prodTag) {
        using ValT = decltype(valTag);
        using ProdT = decltype(prodTag);
        const int32_t grid = l.Q < ComputeUnits() ? l.Q : ComputeUnits();
        hipLaunchKernelGGL((ScatterProductsKernel<ValT, ProdT>), dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0, a.stream,
                           static_cast<const ValT *>(a.vals), static_cast<const ValT *>(a.x), meta, ints(l.chunkDstOff),
                           ints(l.pieceBaseOff), ints(l.pieceRowOff), a.nnz, l.P, l.Q, static_cast<ProdT *>(inter));
    };
    auto sums = [&](auto outTag, auto prodTag) {
        using OutT = decltype(outTag);
        using ProdT = decltype(prodTag);
        hipLaunchKernelGGL((ScatterSumKernel<OutT, ProdT>), dim3(static_cast<uint32_t>(l.P)), dim3(kThreads), 0, a.stream,
                           static_cast<const ProdT *>(inter), colLocal, ints(l.panelStartOff), static_cast<OutT *>(a.y),
                           static_cast<const OutT *>(a.yIn), a.cols, a.alpha, a.beta);
    };
    if (valType == OPSPARSE_F16) {
        products(Half{}, float{});
        if (outType == OPSPARSE_F16) {
            sums(Half{}, float{});
        } else {
            sums(float{}, float{});
        }
    } else if (valType == OPSPARSE_BF16) {
        products(Bf16{}, float{});
        if (outType == OPSPARSE_BF16) {
            sums(Bf16{}, float{});
        } else {
            sums(float{}, float{});
        }
    } else {
        products(float{}, double{});
        sums(float{}, double{});
    }
    return CheckLaunch();
}

}  // namespace scatter_layout
}  // namespace opsparse

using namespace opsparse;
using namespace opsparse::scatter_layout;

extern "C" {

size_t opsparse_spmv_csr_scatter_workspace_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags)
{
    return static_cast<size_t>(MakeLayout(rows, cols, nnz, ValueTypeOf(flags)).bytes);
}

size_t opsparse_spmv_csr_scatter_resident_bytes(int64_t rows, int64_t cols, int64_t nnz, int32_t flags)
{
    return static_cast<size_t>(MakeLayout(rows, cols, nnz, ValueTypeOf(flags)).resident);
}

int opsparse_spmv_csr_scatter_analyse_split(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols,
                                            int64_t nnz, int32_t flags, void *workspace, size_t workspaceBytes,
                                            void *scratchSpace, size_t scratchBytes, OpsparseSpmvPlan *plan, void *stream)
{
    if (plan == nullptr || rowOffsets == nullptr || colInd == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    if ((flags & OPSPARSE_BLOCKED_VALUES_I32) != 0) {
        return OPSPARSE_E_UNSUPPORTED;  // (integer sums wrap: the ordered layout adds them in integers)
    }
    const ScatterLayout l = MakeLayout(rows, cols, nnz, ValueTypeOf(flags));
    if (l.P == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    if (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < l.resident || scratchSpace == nullptr ||
        static_cast<int64_t>(scratchBytes) < l.bytes - l.resident) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    auto *residentBase = static_cast<unsigned char *>(workspace);
    auto *scratchBase = static_cast<unsigned char *>(scratchSpace);
    auto at = [&](int64_t off) { return off < l.resident ? residentBase + off : scratchBase + (off - l.resident); };
    auto ints = [&](int64_t off) { return reinterpret_cast<int32_t *>(at(off)); };
    int32_t *status = ints(0);
    int32_t *keys[2] = {ints(l.keys0Off), ints(l.keys1Off)};
    int32_t *pays[2] = {ints(l.pay0Off), ints(l.pay1Off)};
    int32_t *rowInd = ints(l.rowIndOff), *dstOf = ints(l.dstOfOff), *count = ints(l.countOff), *incl = ints(l.inclOff);
    int32_t *table = ints(l.tableOff), *scan = ints(l.scanOff);
    const int64_t chunks = static_cast<int64_t>(l.P) * l.Q;

    LaunchFillI32(status, 4, 0, s);
    LaunchFillI32(count, chunks + 1, 0, s);
    hipLaunchKernelGGL(ColumnRangeKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s, colInd, nnz, cols,
                       status);
    int32_t seen[2] = {0, 0};
    if (hipMemcpyAsync(seen, status, sizeof(seen), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    if ((seen[0] & 1) != 0) {
        return OPSPARSE_E_INVALID;  // a column index outside [0, cols)
    }
    // Entries in (panel, caller's order) order: stable 4-bit radix passes over the panel number.
    int bits = 0;
    while ((int64_t{1} << bits) < l.P) {
        ++bits;
    }
    const int passes = bits == 0 ? 1 : (bits + 3) / 4;
    const int32_t *keysIn = colInd, *payIn = nullptr;
    for (int k = 0; k < passes; ++k) {
        LaunchRadixPass(keysIn, payIn, keys[k & 1], pays[k & 1], nnz, 0, kOutLog + 4 * k, table, scan, s);
        keysIn = keys[k & 1];
        payIn = pays[k & 1];
    }
    LaunchExpandRows(rowOffsets, rows, nnz, 0, rowInd, s);
    auto *colLocal = reinterpret_cast<uint16_t *>(at(l.colLocalOff));
    hipLaunchKernelGGL(ChunkCountKernel, dim3(GridOf(nnz, kBlockThreads * 8, 16384)), dim3(kBlockThreads), 0, s, keysIn, payIn,
                       nnz, l.Q, l.piece, colLocal, dstOf, count);
    LaunchInclusiveScanI32(count, incl, chunks, 0, scan, s);
    hipLaunchKernelGGL(PieceTablesKernel, dim3(static_cast<uint32_t>(l.Q)), dim3(kWave), 0, s, count, incl, rowInd, l.P, l.Q,
                       l.piece, nnz,
                       ints(l.chunkDstOff), ints(l.pieceBaseOff), ints(l.pieceRowOff), ints(l.panelStartOff));
    hipLaunchKernelGGL(ColumnMaxKernel, dim3(static_cast<uint32_t>(l.P)), dim3(kThreads), 0, s, colLocal,
                       ints(l.panelStartOff), status);
    hipLaunchKernelGGL(EntryMetaKernel, dim3(GridOf(nnz, kBlockThreads, 16384)), dim3(kBlockThreads), 0, s, colInd, rowInd, dstOf,
                       ints(l.chunkDstOff), ints(l.pieceBaseOff), ints(l.pieceRowOff), nnz, l.P, l.piece,
                       reinterpret_cast<uint32_t *>(at(l.metaOff)), status);
    if (hipMemcpyAsync(seen, status, sizeof(seen), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess || CheckLaunch() != OPSPARSE_OK) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    if (seen[1] > kMaxColumnEntries) {
        return OPSPARSE_E_UNSUPPORTED;  // a column that would queue for one address of LDS
    }
    if ((seen[0] & 2) != 0) {
        return OPSPARSE_E_UNSUPPORTED;  // a piece that spans more than 65 535 rows
    }
    OpsparseSpmvPlan p{};
    p.kernel = OPSPARSE_SPMV_SCATTER_LIVE;
    p.rows = rows;
    p.nnz = nnz;
    p.numPanels = l.P;
    p.numRowBlocks = l.Q;
    p.entryWindow = l.piece;
    p.transposed = 1;
    p.liveValues = 1;
    p.valueType = ValueTypeOf(flags);
    p.bytes = l.bytes;
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmv_csr_scatter_analyse(const int32_t *rowOffsets, const int32_t *colInd, int64_t rows, int64_t cols, int64_t nnz,
                                      int32_t flags, void *workspace, size_t workspaceBytes, OpsparseSpmvPlan *plan,
                                      void *stream)
{
    // one piece: the analysis' scratch follows what the launches keep
    const size_t resident = opsparse_spmv_csr_scatter_resident_bytes(rows, cols, nnz, flags);
    if (resident == 0) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    if (workspace == nullptr || workspaceBytes < resident) {
        return OPSPARSE_E_WORKSPACE;
    }
    return opsparse_spmv_csr_scatter_analyse_split(rowOffsets, colInd, rows, cols, nnz, flags, workspace, resident,
                                                   static_cast<unsigned char *>(workspace) + resident,
                                                   workspaceBytes - resident, plan, stream);
}

}  // extern "C"
