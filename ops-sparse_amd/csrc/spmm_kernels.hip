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
// Row-length binning (the counterpart of the reference's greedy row bin
// packing, sparse/spmm/arch35/spmm_csr_mat.cpp:28-66): rows of up to
// kLongRowNnz entries are worked — after Preprocess — in slabs of consecutive
// rows staged through LDS, where every lane group walks an equal share of the
// slab's entries and a row that lies across two shares is cut between them
// (SpmmSlabKernel); without Preprocess a lane group takes one row after the
// other straight from global memory (SpmmRowSplitKernel).  Longer
// rows — the tail of a power-law graph — are cut into segments of kSegmentNnz
// entries, every segment is accumulated by its own lane group into an fp64
// partial row in the workspace, and a fix-up kernel adds a row's partials in
// segment order and applies alpha / beta, so the result does not depend on
// scheduling.
//
// Floating-point products are accumulated in fp64 in stored order and rounded
// once, int8 products in int32 with an int64 saturating epilogue
// (spmm_kernel.cpp:251-266); int8 runs the same kernels with 8 (narrow B: 4)
// bytes of B per lane.  Operands in other layouts — column-major, op(B) = B^T,
// widths or leading dimensions that are not whole vectors — reach these kernels
// as row-major copies staged in the SpMM buffer (DenseRestageKernel, driven by
// spmm_host.cpp); what cannot be staged runs SpmmGeneralKernel in place.
#include <climits>
#include <cstdlib>
#include <type_traits>

#include "device_utils.h"

namespace opsparse {

constexpr int32_t kLongRowNnz = 2048;  // rows longer than this are cut into segments
constexpr int32_t kSegmentNnz = 256;  // entries per segment (128: c5 1.394 ms, 256: 1.378 ms, 512: 1.402 ms)
// Rows a lane group of the row-split kernel takes one after the other, so that a
// workgroup lives long enough to amortise its start-up.  (Two: with four a 5-point mesh takes 120 / 200 / 510 us
// under n = 16 / 32 / 64 instead of 107 / 181 / 431, a 27-point one 313 / 581 us under n = 32 / 64 instead of
// 270 / 459; with one 107 / 212 / 508 and 274 / 492; random columns do not care.)
constexpr int kSpmmRowsPerGroup = 2;

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

// This lane's share of the first L entries of [s, e): entry s + lane, or (0, 0).
template <typename ValT, typename AccT>
__device__ __forceinline__ void LoadFirstChunk(const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
                                               int32_t lane, int32_t s, int32_t e, int32_t *firstCol, float *firstVal)
{
    *firstCol = 0;
    *firstVal = 0.0f;
    if (s + lane < e) {
        *firstCol = LoadStream(colInd + s + lane);
        *firstVal = static_cast<float>(ToAcc<AccT>(LoadStream(vals + s + lane)));
    }
}

// acc[i] += sum over entries p in [s, e) of val[p] * B[colind[p], col + i], in
// stored order.  Called by all L lanes of a group with the same (s, e);
// (firstCol, firstVal) is the lane's LoadFirstChunk result for this range.
template <typename ValT, typename AccT, int V, int L>
__device__ __forceinline__ void AccumulateEntries(const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
                                                  const ValT *__restrict__ B, int64_t ldb, int32_t col, bool active,
                                                  int32_t lane, int32_t s, int32_t e, int32_t firstCol,
                                                  float firstVal, AccT (&acc)[V])
{
    typedef ValT BVec __attribute__((ext_vector_type(V)));
    // Gathers issued back to back, U * 16 bytes in flight per lane.  Eight for the
    // 8-element (fp16) vectors: their fp64 conversion needs the registers, and more
    // resident wavefronts hide more latency than a deeper batch.
    // (sixteen 16-byte gathers a lane cost the row kernel a third of its resident wavefronts: 5-point mesh, n = 64,
    // 432 us with sixteen, 365 with eight; rows of 27 entries 458 and 423; four: rows of 27 under n = 32 314 for 272)
    constexpr int UMAX = 8;
    constexpr int U = L < UMAX ? L : UMAX;
    constexpr int US = U < 8 ? U : 8;   // predicated batch size for the short tail of a row
    for (int32_t p0 = s; p0 < e; p0 += L) {
        // The first L entries come preloaded from the caller (firstCol / firstVal).
        int32_t myCol = firstCol;
        float myVal = firstVal;
        if (p0 != s) {
            myCol = 0;
            myVal = 0.0f;
            if (p0 + lane < e) {
                myCol = LoadStream(colInd + p0 + lane);
                myVal = static_cast<float>(ToAcc<AccT>(LoadStream(vals + p0 + lane)));
            }
        }
        const int32_t cnt = (e - p0 < L) ? e - p0 : L;
        int32_t q0 = 0;
        // Full batches of U entries.
        for (; q0 + U <= cnt; q0 += U) {
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
        // Remaining entries in predicated batches of US; a missing entry adds nothing.
        for (; q0 < cnt; q0 += US) {
            BVec b[US];
            float v[US];
#pragma unroll
            for (int q = 0; q < US; ++q) {
                const bool valid = q0 + q < cnt;
                const int32_t c = __shfl(myCol, (q0 + q) % L, L);
                v[q] = __shfl(myVal, (q0 + q) % L, L);
                if (active && valid) {
                    b[q] = *reinterpret_cast<const BVec *>(B + static_cast<int64_t>(c) * ldb + col);
                }
            }
            if (active) {
#pragma unroll
                for (int q = 0; q < US; ++q) {
                    if (q0 + q < cnt) {
                        const AccT vq = static_cast<AccT>(v[q]);
#pragma unroll
                        for (int i = 0; i < V; ++i) {
                            acc[i] += vq * ToAcc<AccT>(b[q][i]);
                        }
                    }
                }
            }
        }
    }
}

// Rows of at most longRowNnz entries, one lane group per row.
template <typename ValT, typename CT, typename AccT, int V, int L>
__global__ __launch_bounds__(kBlockThreads) void SpmmRowSplitKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, CT *__restrict__ C, int64_t rows, int32_t n, int64_t ldb, int64_t ldc,
    int32_t longRowNnz, OpsparseScalar alphaS, OpsparseScalar betaS, int32_t clampF16)
{
    typedef CT CVec __attribute__((ext_vector_type(V), aligned(16)));
    constexpr int kGroups = kBlockThreads / L;

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));

    const int32_t lane = threadIdx.x % L;
    const int32_t group = threadIdx.x / L;
    const int64_t tile = XcdContiguousTile(blockIdx.x, gridDim.x);
    const int64_t rowBase = tile * (static_cast<int64_t>(kGroups) * kSpmmRowsPerGroup);

    // Row ids, bounds and first entries of all of this group's rows are requested
    // up front, one dependent step per kind for all rows together, instead of a
    // chain of four dependent loads in front of every single row.
    int64_t rowId[kSpmmRowsPerGroup];
    int32_t rowS[kSpmmRowsPerGroup], rowE[kSpmmRowsPerGroup], fCol[kSpmmRowsPerGroup];
    float fVal[kSpmmRowsPerGroup];
#pragma unroll
    for (int it = 0; it < kSpmmRowsPerGroup; ++it) {
        const int64_t slot = rowBase + static_cast<int64_t>(it) * kGroups + group;
        rowId[it] = slot >= rows ? -1 : slot;
    }
#pragma unroll
    for (int it = 0; it < kSpmmRowsPerGroup; ++it) {
        rowS[it] = rowE[it] = 0;
        if (rowId[it] >= 0) {
            rowS[it] = rowOffsets[rowId[it]];
            rowE[it] = rowOffsets[rowId[it] + 1];
        }
    }
#pragma unroll
    for (int it = 0; it < kSpmmRowsPerGroup; ++it) {
        LoadFirstChunk<ValT, AccT>(colInd, vals, lane, rowS[it], rowE[it], &fCol[it], &fVal[it]);
    }

#pragma unroll
    for (int it = 0; it < kSpmmRowsPerGroup; ++it) {
        const int64_t r = rowId[it];
        const int32_t s = rowS[it];
        const int32_t e = rowE[it];
        if (r < 0 || e - s > longRowNnz) {
            continue;  // past the end, or a long row: segment kernel + fix-up write it
        }
        for (int32_t c0 = 0; c0 < n; c0 += L * V) {
            const int32_t col = c0 + lane * V;
            const bool active = col < n;
            AccT acc[V];
#pragma unroll
            for (int i = 0; i < V; ++i) {
                acc[i] = AccT(0);
            }
            AccumulateEntries<ValT, AccT, V, L>(colInd, vals, B, ldb, col, active, lane, s, e, fCol[it], fVal[it],
                                                acc);
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

// ---------------------------------------------------------------- slab path
// The same fast-path operands, rows of at most longRowNnz entries, worked on a
// slab of consecutive rows at a time.  A workgroup copies the slab's (column,
// value) pairs — one contiguous piece of the CSR arrays — and its row bounds
// into LDS, cuts the slab's entries into one run per lane group with about the
// same number of entries each (a run starts at a row's first entry, or inside a
// row of kSplitRowMin entries or more), and every lane group then walks its run
// as one flat sequence of entries: batches of four or eight gathers of B rows,
// two batches in flight, a row's sum written out whenever the sequence crosses a
// row end.  Short rows therefore cost no more than their share of a long one: no
// predicated partial batches, no chain of dependent loads in front of every row.
// The parts of a row cut between runs meet in LDS once the piece has been
// streamed, and the lane group in which the row ends adds them up in the order
// of the entries: the result does not depend on scheduling.  Rows longer than
// longRowNnz are left out (the segment kernels write them); a slab with more
// entries than the LDS holds is worked in several pieces.

constexpr int kSlabCap = 3072;      // entries a workgroup stages in LDS at a time
constexpr int kSlabRowsMax = 255;   // rows whose bounds it stages at a time
// Gathers a lane group issues back to back, two such batches in flight.  Four for
// the 8-element (fp16) vectors, whose widening to fp64 needs the registers: with
// eight the kernel drops to two resident wavefronts per SIMD and runs slower.
template <int V>
struct SlabTuning {
    static constexpr int kBatch = V >= 8 ? 4 : 8;
    static constexpr int kWavesPerSimd = V >= 8 ? 3 : 2;
};
constexpr int kSlabTarget = 2048;   // entries per slab the launcher aims for
// A row of at least kSplitRowMin entries that lies across the boundary between two runs is cut there (neither part
// shorter than kSplitPartMin): the lane group in which it ends adds up the parts.  Without this a row of 250 entries
// makes its run twice as long as the others of its slab, which wait for it (a power-law graph of 2 M rows, mean 16,
// fp16, n = 128: 1.57 -> 1.46 ms), and with it rows of up to 2048 entries are better left to the slabs than cut
// into segments (1.46 -> 1.39 ms; rows of 300, 600 or 2000 entries each run like rows of 64).
constexpr int kSplitRowMin = 16;
constexpr int kSplitPartMin = 4;
static_assert(kLongRowNnz <= kSlabCap, "a row that is not long fits the staging area");

// Small32: B spans less than 4 GiB, so a gather address is the (uniform) base of
// B plus a 32-bit byte offset — one register and one multiply per gather
// instead of a 64-bit multiply-add and a register pair.
template <typename ValT, typename CT, typename AccT, int V, int L, bool Small32>
__device__ __forceinline__ void SlabBody(
    int64_t slab, const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd,
    const ValT *__restrict__ vals, const ValT *__restrict__ B, CT *__restrict__ C, int64_t rows, int32_t n, int64_t ldb,
    int64_t ldc, int32_t rowsPerSlab, const int32_t *__restrict__ slabStart, int32_t longRowNnz,
    OpsparseScalar alphaS, OpsparseScalar betaS, int32_t clampF16, int32_t tileCol0, int32_t tileCols)
{
    typedef ValT BVec __attribute__((ext_vector_type(V)));
    typedef CT CVec __attribute__((ext_vector_type(V), aligned(16)));
    constexpr int kGroups = kBlockThreads / L;
    constexpr int NB = SlabTuning<V>::kBatch;

    // The staged entries; once a piece has been streamed, the same memory takes what every lane group has left of
    // a row that goes on in the next group.
    __shared__ __align__(16) unsigned char stage[kSlabCap * 8];
    int32_t *const entCol = reinterpret_cast<int32_t *>(stage);
    float *const entVal = reinterpret_cast<float *>(stage + kSlabCap * 4);
    AccT *const tailSum = reinterpret_cast<AccT *>(stage);
    static_assert(sizeof(AccT) * kBlockThreads * V <= sizeof(stage), "the parts of cut rows share the staging area");
    __shared__ AccT headSum[kBlockThreads * V];   // a group's sum of the rest of a row that began in an earlier group
    __shared__ int32_t rowAbs[kSlabRowsMax + 1];  // row offsets of the window, as stored
    __shared__ int32_t runRow[kGroups + 1];       // row (window-relative) in which every lane group's run starts,
    __shared__ int32_t runEntry[kGroups + 1];     // and its first entry (piece-relative): past the row's first if cut
    __shared__ int32_t pieceRows;                 // rows of the window that go into this piece
    __shared__ int32_t pieceSplit;                // whether any row of the piece is cut between lane groups

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    const int32_t tid = threadIdx.x;
    const int32_t lane = tid % L;
    const int32_t group = tid / L;
    const int32_t col = tileCol0 + lane * V;  // the workgroup's tile of at most L * V columns of B and C
    const bool active = lane * V < tileCols && col < n;
    const ValT *Bcol = B + col;
    const uint32_t colBytes = static_cast<uint32_t>(col) * static_cast<uint32_t>(sizeof(ValT));
    const uint32_t ldbBytes = static_cast<uint32_t>(ldb) * static_cast<uint32_t>(sizeof(ValT));

    // Slabs of equal work (entries + rows) from the plan's table where there is one, else of equal numbers of rows.
    int64_t rowCur, rowEnd;
    if (slabStart != nullptr) {
        rowCur = slabStart[slab];
        rowEnd = slabStart[slab + 1];
        rowEnd = rowEnd < rows ? rowEnd : rows;  // (the table is the caller's buffer: never past the matrix)
        rowCur = rowCur < 0 ? 0 : rowCur;
    } else {
        rowCur = slab * rowsPerSlab;
        rowEnd = (rowCur + rowsPerSlab < rows) ? rowCur + rowsPerSlab : rows;
    }

    while (rowCur < rowEnd) {  // uniform over the workgroup
        const int32_t win = (rowEnd - rowCur < kSlabRowsMax) ? static_cast<int32_t>(rowEnd - rowCur) : kSlabRowsMax;
        if (tid <= win) {
            rowAbs[tid] = rowOffsets[rowCur + tid];
        }
        if (tid == 0) {
            pieceRows = win;
            pieceSplit = 0;
        }
        __syncthreads();
        const int32_t base = rowAbs[0];
        // The piece ends in front of the first row that is long or no longer fits.
        if (tid < win) {
            const int32_t hi = rowAbs[tid + 1];
            if (hi - rowAbs[tid] > longRowNnz || hi - base > kSlabCap) {
                atomicMin(&pieceRows, tid);
            }
        }
        __syncthreads();
        const int32_t J = pieceRows;
        if (J == 0) {
            rowCur += 1;  // a long row: not this kernel's (longRowNnz <= kSlabCap, so a short row always fits)
            __syncthreads();
            continue;
        }
        const int32_t E = rowAbs[J] - base;
        for (int32_t i = tid; i < E; i += kBlockThreads) {
            entCol[i] = LoadStream(colInd + base + i);
            entVal[i] = static_cast<float>(ToAcc<AccT>(LoadStream(vals + base + i)));
        }
        // A row costs a run its entries (a gather of a row of B each) and one row of C to finish: run g starts at
        // the first row with g * share of that work in front of it.  (Counting entries alone leaves the empty rows
        // of a sparse window to a few lane groups, one row of C after the other: 8 M rows with 0.8 M entries
        // 2.55 ms.)
        if (tid <= kGroups) {
            const int32_t share = (E + J + kGroups - 1) / kGroups;
            int32_t row = J, first = E;
            if (tid < kGroups) {
                const int32_t want = tid * share;
                int32_t lo = 0, hi = J;
                while (lo < hi) {
                    const int32_t mid = (lo + hi) >> 1;
                    if (rowAbs[mid] - base + mid < want) {
                        lo = mid + 1;
                    } else {
                        hi = mid;
                    }
                }
                row = lo;
                first = rowAbs[lo] - base;
                if (lo > 0) {
                    // Row lo - 1 lies across `want`: cut it where entries + rows in front come to `want`.
                    const int32_t rowFirst = rowAbs[lo - 1] - base;
                    const int32_t cut = want - (lo - 1);
                    if (first - rowFirst >= kSplitRowMin && first - cut >= kSplitPartMin) {
                        row = lo - 1;  // (a cut near the row's end goes to the end, one near its start to the start:
                                       // the starts of the runs must not go backwards)
                        if (cut - rowFirst >= kSplitPartMin) {
                            first = cut;
                            pieceSplit = 1;
                        } else {
                            first = rowFirst;
                        }
                    }
                }
            }
            runRow[tid] = row;
            runEntry[tid] = first;
        }
        __syncthreads();

        int32_t cur = runRow[group];             // next row to finish
        const int32_t last = runRow[group + 1];  // first row that this run does not finish
        int32_t f = runEntry[group];             // next entry to consume
        const int32_t fEnd = runEntry[group + 1];
        bool headRow = f > rowAbs[cur] - base;   // the run starts inside row `cur`
        int32_t nextEnd = (cur < last) ? rowAbs[cur + 1] - base : INT32_MAX;

        AccT acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            acc[i] = AccT(0);
        }
        auto writeRow = [&](int32_t row, const AccT(&sum)[V]) {
            CT *out = C + (rowCur + row) * ldc + col;
            CVec res;
            if (betaZero) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    res[i] = Epilogue<CT, AccT>::Apply(sum[i], alpha, beta, true, nullptr, clampF16 != 0);
                }
            } else {
                const CVec old = *reinterpret_cast<const CVec *>(out);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const CT o = old[i];
                    res[i] = Epilogue<CT, AccT>::Apply(sum[i], alpha, beta, false, &o, clampF16 != 0);
                }
            }
            *reinterpret_cast<CVec *>(out) = res;
        };
        // Writes every row of the run that ends at entry position `pos`; the rest of a row that began in an earlier
        // run is kept for the addition of its parts.
        auto finishRows = [&](int32_t pos) {
            while (nextEnd <= pos) {
                if (headRow) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        headSum[tid * V + i] = acc[i];
                    }
                    headRow = false;
                } else if (active) {
                    writeRow(cur, acc);
                }
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    acc[i] = AccT(0);
                }
                ++cur;
                nextEnd = (cur < last) ? rowAbs[cur + 1] - base : INT32_MAX;
            }
        };
        finishRows(f);  // empty rows at the head of the run

        // Gathers are issued unconditionally (a position past the end of the run
        // re-reads the run's last entry with a zero value, a lane past column n reads
        // column 0), so that the compiler can count the loads in flight and wait for
        // one batch while the next stays outstanding.
        BVec bufA[NB], bufB[NB];
        float valA[NB], valB[NB];
        const uint32_t laneBytes = active ? colBytes : 0u;
        const ValT *Blane = active ? Bcol : B;
        auto fetch = [&](int32_t f0, BVec(&buf)[NB], float(&v)[NB]) {
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const int32_t p = f0 + q;
                const int32_t pc = p < fEnd ? p : fEnd - 1;
                const int32_t c = entCol[pc];
                v[q] = p < fEnd ? entVal[pc] : 0.0f;
                if (Small32) {
                    const uint32_t off = static_cast<uint32_t>(c) * ldbBytes + laneBytes;
                    buf[q] = *reinterpret_cast<const BVec *>(reinterpret_cast<const char *>(B) + off);
                } else {
                    buf[q] = *reinterpret_cast<const BVec *>(Blane + static_cast<int64_t>(c) * ldb);
                }
            }
        };
        auto consume = [&](int32_t f0, BVec(&buf)[NB], float(&v)[NB]) {
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const AccT vq = static_cast<AccT>(v[q]);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    acc[i] += vq * ToAcc<AccT>(buf[q][i]);
                }
                finishRows(f0 + q + 1);  // positions past the end finish nothing: every row is done by then
            }
        };
        if (f < fEnd) {
            fetch(f, bufA, valA);
        }
        while (f < fEnd) {
            fetch(f + NB, bufB, valB);  // also when nothing is left: a branch here would hide the load count
            consume(f, bufA, valA);
            f += NB;
            if (f < fEnd) {
                fetch(f + NB, bufA, valA);
                consume(f, bufB, valB);
                f += NB;
            }
        }
        finishRows(fEnd);  // nothing left unless the run has no entry at all
        if (pieceSplit != 0) {  // uniform over the workgroup
            // What a run holds at its end belongs to a row that goes on in the next run (zero if there is none).
            __syncthreads();    // every run is done with the staged entries
#pragma unroll
            for (int i = 0; i < V; ++i) {
                tailSum[tid * V + i] = acc[i];
            }
            __syncthreads();
            const int32_t row = runRow[group];
            const int32_t rowFirst = rowAbs[row] - base;
            if (runEntry[group] > rowFirst && last > row) {
                // Row `row` ends in this run: its parts in the order of the entries, from the run in which it starts.
                int32_t g0 = group - 1;
                while (g0 > 0 && runRow[g0] == row && runEntry[g0] > rowFirst) {
                    --g0;
                }
                AccT sum[V];
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    sum[i] = tailSum[(g0 * L + lane) * V + i];
                }
                for (int32_t g = g0 + 1; g < group; ++g) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        sum[i] += tailSum[(g * L + lane) * V + i];
                    }
                }
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    sum[i] += headSum[tid * V + i];
                }
                if (active) {
                    writeRow(row, sum);
                }
            }
        }
        rowCur += J;
        __syncthreads();   // the next piece overwrites the LDS arrays
    }
}

// One lane group per segment of a long row: partial[seg][0..n) = sum over the
// segment's entries, in fp64.
template <typename ValT, typename AccT, int V, int L>
__device__ __forceinline__ void SegmentBody(int64_t block, const int32_t *__restrict__ rowOffsets,
                                            const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
                                            const ValT *__restrict__ B, int32_t n, int64_t ldb, int32_t numSegments,
                                            const int32_t *__restrict__ segRow, const int32_t *__restrict__ segStart,
                                            AccT *__restrict__ partial, int32_t colBegin, int32_t colEnd)
{
    constexpr int kGroups = kBlockThreads / L;
    const int32_t lane = threadIdx.x % L;
    const int64_t seg = block * kGroups + threadIdx.x / L;
    if (seg >= numSegments) {
        return;
    }
    const int32_t row = segRow[seg];
    const int32_t s = segStart[seg];
    const int32_t rowEnd = rowOffsets[row + 1];
    const int32_t e = (rowEnd - s > kSegmentNnz) ? s + kSegmentNnz : rowEnd;
    int32_t firstCol;
    float firstVal;
    LoadFirstChunk<ValT, AccT>(colInd, vals, lane, s, e, &firstCol, &firstVal);
    for (int32_t c0 = colBegin; c0 < colEnd; c0 += L * V) {
        const int32_t col = c0 + lane * V;
        const bool active = col < colEnd;
        AccT acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            acc[i] = AccT(0);
        }
        AccumulateEntries<ValT, AccT, V, L>(colInd, vals, B, ldb, col, active, lane, s, e, firstCol, firstVal, acc);
        if (active) {
            AccT *out = partial + seg * n + col;
#pragma unroll
            for (int i = 0; i < V; ++i) {
                out[i] = acc[i];
            }
        }
    }
}

template <typename ValT, typename AccT, int V, int L>
__global__ __launch_bounds__(kBlockThreads) void SpmmLongSegmentKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, int32_t n, int64_t ldb, int32_t numSegments, const int32_t *__restrict__ segRow,
    const int32_t *__restrict__ segStart, AccT *__restrict__ partial)
{
    SegmentBody<ValT, AccT, V, L>(blockIdx.x, rowOffsets, colInd, vals, B, n, ldb, numSegments, segRow, segStart, partial,
                                  0, n);
}

// The slab kernel proper.  With long rows (segBlocks > 0) the workgroups of their
// segments are spread evenly among the slab workgroups of the same launch: the
// segment workgroups stream at the gather ceiling and fill the moments in which a
// slab workgroup is between slabs and has no gather in flight.
template <typename ValT, typename CT, typename AccT, int V, int L, bool Small32>
__global__ __launch_bounds__(kBlockThreads, SlabTuning<V>::kWavesPerSimd) void SpmmSlabKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, CT *__restrict__ C, int64_t rows, int32_t n, int64_t ldb, int64_t ldc,
    int32_t rowsPerSlab, const int32_t *__restrict__ slabStart, int32_t longRowNnz, OpsparseScalar alphaS,
    OpsparseScalar betaS, int32_t clampF16, uint32_t segBlocks, int32_t numSegments, const int32_t *__restrict__ segRow,
    const int32_t *__restrict__ segStart, AccT *__restrict__ partial, int32_t tileCols)
{
    // blockIdx.y: which tile of tileCols (<= L * V) columns of B and C.
    const int32_t tileCol0 = static_cast<int32_t>(blockIdx.y) * tileCols;
    int64_t slab;
    if (segBlocks > 0) {
        // workgroup b is a segment workgroup iff floor((b + 1) * segBlocks / total) > floor(b * segBlocks / total)
        const uint64_t before = static_cast<uint64_t>(blockIdx.x) * segBlocks / gridDim.x;
        const uint64_t after = (static_cast<uint64_t>(blockIdx.x) + 1) * segBlocks / gridDim.x;
        if (after > before) {
            SegmentBody<ValT, AccT, V, L>(static_cast<int64_t>(before), rowOffsets, colInd, vals, B, n, ldb, numSegments,
                                          segRow, segStart, partial, tileCol0,
                                          (n - tileCol0 < tileCols) ? n : tileCol0 + tileCols);
            return;
        }
        slab = static_cast<int64_t>(blockIdx.x) - static_cast<int64_t>(before);
    } else {
        slab = XcdContiguousTile(blockIdx.x, gridDim.x);
    }
    SlabBody<ValT, CT, AccT, V, L, Small32>(slab, rowOffsets, colInd, vals, B, C, rows, n, ldb, ldc, rowsPerSlab,
                                            slabStart, longRowNnz, alphaS, betaS, clampF16, tileCol0, tileCols);
}

// One workgroup per long row.  Each of its four wavefronts adds a contiguous
// quarter of the row's partials in segment order (lane = output column), the four
// sums are combined in wavefront order through LDS, then alpha / beta are applied.
// The association order is fixed by the segment table alone, so the result is
// the same on every run.
template <typename CT, typename AccT>
__global__ __launch_bounds__(kBlockThreads) void SpmmLongFixupKernel(
    CT *__restrict__ C, int32_t n, int64_t ldc, int32_t numLongRows, const int32_t *__restrict__ longRows,
    const int32_t *__restrict__ longFirstSeg, const AccT *__restrict__ partial, OpsparseScalar alphaS,
    OpsparseScalar betaS, int32_t clampF16)
{
    constexpr int kWaves = kBlockThreads / kWave;
    __shared__ AccT part[kWaves][kWave];
    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    const int32_t lane = threadIdx.x % kWave;
    const int32_t wave = threadIdx.x / kWave;
    const int64_t j = blockIdx.x;
    const int64_t row = longRows[j];
    const int64_t seg0 = longFirstSeg[j];
    const int64_t seg1 = longFirstSeg[j + 1];
    const int64_t per = (seg1 - seg0 + kWaves - 1) / kWaves;
    const int64_t mine0 = seg0 + wave * per;
    const int64_t mine1 = mine0 + per < seg1 ? mine0 + per : seg1;
    for (int32_t c0 = 0; c0 < n; c0 += kWave) {
        const int32_t col = c0 + lane;
        AccT sum = AccT(0);
        if (col < n) {
            int64_t seg = mine0;
            for (; seg + 16 <= mine1; seg += 16) {  // a row of thousands of segments: sixteen loads in flight
                AccT p[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    p[u] = partial[(seg + u) * n + col];
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    sum += p[u];  // added in segment order
                }
            }
            for (; seg + 4 <= mine1; seg += 4) {  // four loads in flight, added in order
                const AccT p0 = partial[(seg + 0) * n + col];
                const AccT p1 = partial[(seg + 1) * n + col];
                const AccT p2 = partial[(seg + 2) * n + col];
                const AccT p3 = partial[(seg + 3) * n + col];
                sum += p0;
                sum += p1;
                sum += p2;
                sum += p3;
            }
            for (; seg < mine1; ++seg) {
                sum += partial[seg * n + col];
            }
        }
        part[wave][lane] = sum;
        __syncthreads();
        if (wave == 0 && col < n) {
            AccT total = part[0][lane];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                total += part[w][lane];
            }
            CT *out = C + row * ldc + col;
            *out = Epilogue<CT, AccT>::Apply(total, alpha, beta, betaZero, out, clampF16 != 0);
        }
        __syncthreads();
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

// A dense rows x cols matrix copied from one storage order / leading dimension to another, a 32 x 32 tile per
// workgroup through LDS: the tile is read along the source's contiguous direction and written along the
// destination's.  Columns cols .. colsDst-1 of the destination (padding) are written as zero.
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void DenseRestageKernel(const T *__restrict__ src, T *__restrict__ dst,
                                                                    int64_t rows, int64_t cols, int64_t colsDst,
                                                                    int64_t ldSrc, int32_t srcColMajor, int64_t ldDst,
                                                                    int32_t dstColMajor, int64_t tilesAcross)
{
    constexpr int kTile = 32;
    __shared__ T tile[kTile][kTile + 1];  // [row][column]
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) / tilesAcross * kTile;
    const int64_t c0 = static_cast<int64_t>(blockIdx.x) % tilesAcross * kTile;
    const int tx = threadIdx.x % kTile, ty = threadIdx.x / kTile;
    constexpr int kStep = kBlockThreads / kTile;
    for (int i = ty; i < kTile; i += kStep) {
        const int rr = srcColMajor ? tx : i, cc = srcColMajor ? i : tx;
        const int64_t r = r0 + rr, c = c0 + cc;
        T v = T(0);
        if (r < rows && c < cols) {
            v = src[srcColMajor ? r + c * ldSrc : r * ldSrc + c];
        }
        tile[rr][cc] = v;
    }
    __syncthreads();
    for (int i = ty; i < kTile; i += kStep) {
        const int rr = dstColMajor ? tx : i, cc = dstColMajor ? i : tx;
        const int64_t r = r0 + rr, c = c0 + cc;
        if (r < rows && c < colsDst) {
            dst[dstColMajor ? r + c * ldDst : r * ldDst + c] = tile[rr][cc];
        }
    }
}

// The same copy for a destination of at most 32 columns, where a 32 x 32 tile would be mostly padding (1 column:
// 130 us for 4 M rows): a lane a row, the columns one after the other.  Whatever the two orders, the lanes of an
// instruction touch consecutive rows of one column or the short rows of consecutive rows.
// VecSrc / VecDst: that side is row-major with rows of whole, aligned groups of four elements, which then travel
// as one load or store.
template <typename T, bool VecSrc, bool VecDst>
__global__ __launch_bounds__(kBlockThreads) void DenseRestageNarrowKernel(const T *__restrict__ src,
                                                                          T *__restrict__ dst, int64_t rows,
                                                                          int32_t cols, int32_t colsDst, int64_t ldSrc,
                                                                          int32_t srcColMajor, int64_t ldDst,
                                                                          int32_t dstColMajor)
{
    typedef T Vec4 __attribute__((ext_vector_type(4)));
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const T *from = src + (srcColMajor ? r : r * ldSrc);
    T *to = dst + (dstColMajor ? r : r * ldDst);
    const int64_t stepSrc = srcColMajor ? ldSrc : 1, stepDst = dstColMajor ? ldDst : 1;
    for (int32_t c0 = 0; c0 < colsDst; c0 += 4) {
        T v[4];
        if (VecSrc && c0 + 4 <= cols) {
            const Vec4 in = *reinterpret_cast<const Vec4 *>(from + c0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = in[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = c0 + i < cols ? from[(c0 + i) * stepSrc] : T(0);
            }
        }
        if (VecDst) {  // (colsDst is whole groups of four)
            *reinterpret_cast<Vec4 *>(to + c0) = Vec4{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (c0 + i < colsDst) {
                    to[(c0 + i) * stepDst] = v[i];
                }
            }
        }
    }
}

// ------------------------------------------------------------ narrow B
// B of one or two 16-byte pieces a row (4 or 8 fp32 columns, 8 or 16 fp16 ones): a lane group spanning the columns
// would be a lane or two wide, and the kernels above then spend their time on bookkeeping, not on the matrix.  Here
// the product runs like an SpMV whose vector elements are short rows of B.  A persistent workgroup walks over tiles
// of consecutive rows - the slabs of the plan's table, cut (MakeNarrowTiling) so that a tile holds at most
// NarrowEntries(n) entries and its rows times pieces fill the workgroup's lanes a whole number of times.  Per
// tile: every lane takes consecutive (column, value) pairs four at a time as 16-byte loads, gathers their rows of B
// whole and drops them, with the values, into LDS; then one lane group per (row, piece of the row of C) adds up
// its row's products from LDS, in fp64, a lane holding the piece's 4 (fp16: 8) sums.  Three tiles are under way at
// once: while the sums of tile i are made from LDS, the rows of B of tile i + 1 and the entries of tile i + 2 are
// in flight, and the tiles' bounds are read two turns further ahead still, so that no turn of the loop waits for a
// load it has only just asked for.  In LDS the pieces lie so that the lanes of one store instruction - which hold
// entries four apart - write consecutive slots: entry k of a tile is at slot (k mod 4) E / 4 + k / 4 (stored in
// the order of the entries, a wavefront's 64 pieces fell on 8 of the 32 banks).  Lanes past the end of a tile load what the last lane inside it loads and store
// to slots nobody reads: the loop holds no branch that depends on the lane.  Workgroups of one XCD share one
// contiguous range of tiles.
constexpr int kNarrowRows = 1023;    // rows of a tile at most (their offsets pass through LDS)
constexpr int kNarrowMaxRow = 200;   // longest row of a matrix that takes this kernel

// Entries a tile holds at most: a quad a lane.  (Two quads under a one-piece B - 44 KB of LDS, three workgroups a
// compute unit instead of five - run no faster: what counts is the bytes in flight per compute unit.)
constexpr int NarrowEntries(int64_t)
{
    return 1024;
}

// Ragged: rows of B and C of nCols <= W fp32 elements at any leading dimension and 4-byte alignment (3 interleaved
// components a point, say) are read and written where they are, the last piece of a row as 1 - 4 dwords, and sit
// padded with zeros in LDS.  (Through the staging area such operands cost two copies on top: 4 M rows, n = 3,
// 109 us against 71 for n = 4.)
template <typename ValT, typename CT, typename AccT, int W, int G, bool Ragged = false>
__global__ __launch_bounds__(kBlockThreads) void SpmmNarrowKernel(
    const int32_t *__restrict__ rowOffsets, const int32_t *__restrict__ colInd, const ValT *__restrict__ vals,
    const ValT *__restrict__ B, CT *C, uint32_t ldb, uint32_t ldc, const int32_t *__restrict__ slabStart,
    int64_t numSlabs, int64_t nnz, OpsparseScalar alphaS, OpsparseScalar betaS, int32_t clampF16, int32_t nCols)
{
    static_assert(!Ragged || (sizeof(ValT) == 4 && sizeof(CT) == 4), "ragged rows of 4-byte elements");
    typedef int32_t Int2U __attribute__((ext_vector_type(2), aligned(4)));
    typedef int32_t Int4A __attribute__((ext_vector_type(4)));
    constexpr int Q = W * static_cast<int>(sizeof(ValT)) / 16;  // 16-byte pieces of a row of B
    constexpr int kPiece = 16 / static_cast<int>(sizeof(ValT));  // elements of a piece
    constexpr int E = NarrowEntries(W);                          // entries of a tile at most
    constexpr int U = E / (4 * kBlockThreads);                   // quads of entries a lane takes
    static_assert(Q * kPiece == W && (Q == 1 || Q == 2), "one or two whole pieces");
    static_assert(U * 4 * kBlockThreads == E && U >= 1, "whole quads");
    __shared__ __align__(16) unsigned char bRaw[E * Q * 16];
    __shared__ __align__(16) float valLds[E];
    __shared__ int32_t rowLds[kNarrowRows + 1];
    Int4A *const bPieces = reinterpret_cast<Int4A *>(bRaw);
    typedef float Float4A __attribute__((ext_vector_type(4)));

    const AccT alpha = ReadScalar<AccT>(alphaS);
    const AccT beta = ReadScalar<AccT>(betaS);
    const bool betaZero = (beta == AccT(0));
    const int32_t tid = static_cast<int32_t>(threadIdx.x);

    // This XCD's tiles, and this workgroup's stride through them.
    const int32_t slabs = static_cast<int32_t>(numSlabs);  // (below 2^31: the launcher checks)
    const int32_t xcd = static_cast<int32_t>(blockIdx.x % kNumXcd);
    const int32_t perXcd = slabs / kNumXcd, rem = slabs % kNumXcd;
    const int32_t xcdFirst = xcd * perXcd + (xcd < rem ? xcd : rem);
    const int32_t xcdTiles = perXcd + (xcd < rem ? 1 : 0);
    const int32_t stride = (static_cast<int32_t>(gridDim.x) - xcd + kNumXcd - 1) / kNumXcd;  // workgroups on this XCD
    const int32_t t0 = static_cast<int32_t>(blockIdx.x / kNumXcd);
    if (t0 >= xcdTiles) {
        return;
    }
    const int32_t mine = (xcdTiles - t0 + stride - 1) / stride;  // tiles of this workgroup

    struct Tile {
        int32_t r0, r1, first, count;
    };
    auto loadRows = [&](int32_t i, Tile &m) {
        const int32_t slab = xcdFirst + t0 + i * stride;
        m.r0 = slabStart[slab];
        m.r1 = slabStart[slab + 1];
    };
    auto loadEntries = [&](Tile &m) {
        m.first = rowOffsets[m.r0];
        m.count = rowOffsets[m.r1] - m.first;
    };
    // A tile that does not fit - the row offsets changed since the table was made - is summed straight from memory.
    const int32_t nnz32 = static_cast<int32_t>(nnz);
    auto fits = [&](const Tile &m) {
        return m.count >= 0 && m.count <= E && m.r1 - m.r0 <= kNarrowRows && m.first >= 0 &&
               m.first <= nnz32 - m.count;
    };

    Int4U colN[U];
    ValT valN[U][4];
    Int4A piece[U][4][Q];
    float valP[U][4];
    constexpr int kBoundRegs = (kNarrowRows + 1) / kBlockThreads;
    int32_t bnd[kBoundRegs];
    // Requests this lane's entries of a tile that holds any; nothing is waited for.  A quad that would reach past
    // the end of the arrays is read a few entries earlier (nnz >= 4), and issueGather moves its entries into place.
    auto issueQuads = [&](const Tile &m) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if ((u * kBlockThreads + (tid & ~(kWave - 1))) * 4 >= m.count) {
                continue;
            }
            int32_t at = m.first + (u * kBlockThreads + tid) * 4;  // (first + count <= nnz <= INT32_MAX - 4 E)
            at = at + 4 <= nnz32 ? at : nnz32 - 4;
            colN[u] = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(colInd + at));
            if constexpr (sizeof(ValT) == 4) {
                const Int4U v = __builtin_nontemporal_load(reinterpret_cast<const Int4U *>(vals + at));
                __builtin_memcpy(valN[u], &v, 16);
            } else {
                const Short4U v = __builtin_nontemporal_load(reinterpret_cast<const Short4U *>(vals + at));
                __builtin_memcpy(valN[u], &v, 8);
            }
        }
    };
    // Requests the rows of B of the entries issueQuads asked for (waiting for those), and the tile's row offsets.
    // An entry past the tile's end takes the row of B of the tile's first entry.
    auto issueGather = [&](const Tile &m) {
        if (m.first + E > nnz32) {  // the tile that may reach the end of the arrays
#pragma unroll
            for (int u = 0; u < U; ++u) {
                int32_t late = m.first + (u * kBlockThreads + tid) * 4 + 4 - nnz32;  // entries the quad was read early
                late = late > 3 ? 3 : late;
                for (; late > 0; --late) {                                           // (the last lanes of that tile)
                    colN[u] = Int4U{colN[u][1], colN[u][2], colN[u][3], colN[u][3]};
                    valN[u][0] = valN[u][1];
                    valN[u][1] = valN[u][2];
                    valN[u][2] = valN[u][3];
                }
            }
        }
        const int32_t colSafe = __shfl(colN[0][0], 0, kWave);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if ((u * kBlockThreads + (tid & ~(kWave - 1))) * 4 >= m.count) {
                continue;  // a wavefront whose entries all lie past the tile's end
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int32_t k = (u * kBlockThreads + tid) * 4 + i;
                const uint32_t col = static_cast<uint32_t>(k < m.count ? colN[u][i] : colSafe);
                const ValT *bRow = B + static_cast<uint64_t>(col) * ldb;
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    if constexpr (Ragged) {
                        const int32_t have = nCols - q * kPiece;  // elements of this piece that exist (uniform)
                        const int32_t *from = reinterpret_cast<const int32_t *>(bRow + q * kPiece);
                        Int4A p = {0, 0, 0, 0};
                        if (have >= 4) {
                            const Int4U v = *reinterpret_cast<const Int4U *>(from);
                            p = Int4A{v[0], v[1], v[2], v[3]};
                        } else if (have == 3) {  // (two loads: a three-element vector type is loaded as four)
                            const Int2U v = *reinterpret_cast<const Int2U *>(from);
                            p = Int4A{v[0], v[1], from[2], 0};
                        } else if (have == 2) {
                            const Int2U v = *reinterpret_cast<const Int2U *>(from);
                            p = Int4A{v[0], v[1], 0, 0};
                        } else if (have == 1) {
                            p = Int4A{from[0], 0, 0, 0};
                        }
                        piece[u][i][q] = p;
                    } else {
                        piece[u][i][q] = *reinterpret_cast<const Int4A *>(bRow + q * kPiece);
                    }
                }
                valP[u][i] = static_cast<float>(valN[u][i]);
            }
        }
        const int32_t tileRows = m.r1 - m.r0;
#pragma unroll
        for (int b = 0; b < kBoundRegs; ++b) {
            if (b * kBlockThreads <= tileRows) {
                const int32_t rr = b * kBlockThreads + tid;
                bnd[b] = rowOffsets[m.r0 + (rr < tileRows ? rr : tileRows)];
            }
        }
    };

    Tile m0{}, m1{}, m2{}, m3{};
    loadRows(0, m0);
    loadEntries(m0);
    if (mine > 1) {
        loadRows(1, m1);
        loadEntries(m1);
    }
    if (mine > 2) {
        loadRows(2, m2);
        loadEntries(m2);
    }
    if (mine > 3) {
        loadRows(3, m3);
    }
    if (fits(m0) && m0.count > 0) {
        issueQuads(m0);
        issueGather(m0);
    }
    if (mine > 1 && fits(m1) && m1.count > 0) {
        issueQuads(m1);
    }

    constexpr int kGroups = kBlockThreads / G;
    const int32_t lane = tid % G;
    for (int32_t i = 0; i < mine; ++i) {
        Tile m4{};
        if (i + 4 < mine) {
            loadRows(i + 4, m4);
        }
        if (i + 3 < mine) {
            loadEntries(m3);
        }
        const bool staged = fits(m0);
        const int32_t tileRows = m0.r1 - m0.r0;
        if (staged && m0.count > 0) {
#pragma unroll
            for (int b = 0; b < kBoundRegs; ++b) {
                if (b * kBlockThreads <= tileRows) {
                    const int32_t rr = b * kBlockThreads + tid;
                    rowLds[rr < tileRows ? rr : tileRows] = bnd[b];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int32_t k = (u * kBlockThreads + tid) * 4;
                if ((u * kBlockThreads + (tid & ~(kWave - 1))) * 4 >= m0.count) {
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
#pragma unroll
                    for (int q = 0; q < Q; ++q) {
                        bPieces[q * E + e * (E / 4) + (k >> 2)] = piece[u][e][q];
                    }
                }
                *reinterpret_cast<Float4A *>(valLds + k) = Float4A{valP[u][0], valP[u][1], valP[u][2], valP[u][3]};
            }
        }
        LdsBarrier();
        if (i + 1 < mine && fits(m1) && m1.count > 0) {
            issueGather(m1);
        }
        if (i + 2 < mine && fits(m2) && m2.count > 0) {
            issueQuads(m2);
        }

        // one lane group per piece of the tile's rows of C
        const int32_t items = tileRows * Q;
        for (int32_t it = tid / G; it < items; it += kGroups) {
            const int32_t rr = it / Q, q = it % Q;
            AccT acc[kPiece];
#pragma unroll
            for (int c = 0; c < kPiece; ++c) {
                acc[c] = AccT(0);
            }
            if (staged && m0.count > 0) {
                int32_t s = rowLds[rr] - m0.first, e = rowLds[rr + 1] - m0.first;
                s = s < 0 ? 0 : s;
                e = e > m0.count ? m0.count : e;
                for (int32_t k = s + lane; k < e; k += G) {
                    const AccT v = static_cast<AccT>(valLds[k]);
                    const Int4A p = bPieces[q * E + (k & 3) * (E / 4) + (k >> 2)];
                    ValT b[kPiece];
                    __builtin_memcpy(b, &p, 16);
#pragma unroll
                    for (int c = 0; c < kPiece; ++c) {
                        acc[c] += v * ToAcc<AccT>(b[c]);
                    }
                }
            } else {
                const int64_t s = rowOffsets[m0.r0 + rr], e = rowOffsets[m0.r0 + rr + 1];
                for (int64_t k = s + lane; k < e; k += G) {
                    const AccT v = ToAcc<AccT>(vals[k]);
                    const ValT *bRow = B + static_cast<uint64_t>(static_cast<uint32_t>(colInd[k])) * ldb + q * kPiece;
#pragma unroll
                    for (int c = 0; c < kPiece; ++c) {
                        if (!Ragged || q * kPiece + c < nCols) {
                            acc[c] += v * ToAcc<AccT>(bRow[c]);
                        }
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < kPiece; ++c) {
                acc[c] = GroupSum<G>(acc[c]);
            }
            if (lane == 0) {
                CT *out = C + static_cast<uint64_t>(static_cast<uint32_t>(m0.r0 + rr)) * ldc + q * kPiece;
                CT res[kPiece] = {};
                const int32_t have = Ragged ? nCols - q * kPiece : kPiece;  // (uniform but for q)
#pragma unroll
                for (int c = 0; c < kPiece; ++c) {
                    if (c < have) {
                        res[c] = Epilogue<CT, AccT>::Apply(acc[c], alpha, beta, betaZero, out + c, clampF16 != 0);
                    }
                }
                if constexpr (Ragged) {
                    int32_t bits[kPiece];
                    __builtin_memcpy(bits, res, sizeof(bits));
                    int32_t *to = reinterpret_cast<int32_t *>(out);
                    if (have >= 4) {
                        *reinterpret_cast<Int4U *>(to) = Int4U{bits[0], bits[1], bits[2], bits[3]};
                    } else if (have == 3) {
                        *reinterpret_cast<Int2U *>(to) = Int2U{bits[0], bits[1]};
                        to[2] = bits[2];
                    } else if (have == 2) {
                        *reinterpret_cast<Int2U *>(to) = Int2U{bits[0], bits[1]};
                    } else if (have == 1) {
                        to[0] = bits[0];
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < kPiece; ++c) {
                        out[c] = res[c];
                    }
                }
            }
        }
        LdsBarrier();  // everyone is done with the tile before the next one overwrites it; its loads stay in flight
        m0 = m1;
        m1 = m2;
        m2 = m3;
        m3 = m4;
    }
}

// Longest row, number of long rows and number of segments.  stats[0..2] zeroed
// before the launch.
__global__ __launch_bounds__(kBlockThreads) void SpmmRowStatsKernel(const int32_t *__restrict__ rowOffsets,
                                                                    int64_t rows, int32_t *__restrict__ stats)
{
    int32_t best = 0, numLong = 0, numSeg = 0;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
    for (int64_t r = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; r < rows; r += stride) {
        const int32_t len = rowOffsets[r + 1] - rowOffsets[r];
        best = len > best ? len : best;
        if (len > kLongRowNnz) {
            ++numLong;
            numSeg += (len + kSegmentNnz - 1) / kSegmentNnz;
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int32_t other = __shfl_xor(best, off, kWave);
        best = other > best ? other : best;
        numLong += __shfl_xor(numLong, off, kWave);
        numSeg += __shfl_xor(numSeg, off, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        if (best > 0) atomicMax(stats, best);
        if (numLong > 0) {
            atomicAdd(stats + 1, numLong);
            atomicAdd(stats + 2, numSeg);
        }
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
    const OpsparseSpmmPlan *plan;
    void *ws;
};

inline int CheckLaunch()
{
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

inline int64_t Align256(int64_t v) { return (v + 255) / 256 * 256; }

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

// Slabs of the slab kernel: about kSlabTarget entries each, cut where the running count of entries + rows passes
// a multiple of `share` (a row costs its entries and one row of C), so that a matrix whose rows are sorted by
// length is cut as evenly as one whose rows are mixed.  Half as long where no row exceeds 64 entries and B has at
// most 128 columns: 1 M rows of 32, n = 64, 1.215 -> 1.187 ms; 2 M rows of 16 1.245 -> 1.213 ms (with longer rows
// among them the shorter slabs lose: a power-law graph 1.38 -> 1.47 ms; with 256 columns 5.45 -> 5.52 ms).
// The tiles of SpmmNarrowKernel for a B of at most 16 columns under rows of at most kNarrowMaxRow entries.  The
// kernel gives a lane group to every 16-byte piece of a row of C: a tile of R rows and p pieces a row keeps the 256
// lanes busy when R p times the lanes of a group is just below a multiple of 256.  R and the lanes of a group are
// chosen here (for fp32 pieces; fp16 rows have half as many pieces and take twice the lanes), and the slab table
// is cut with share = R (mean + 1): a slab's entries + rows stay below share + maxRow + 1 (SpmmSlabTableKernel),
// so a tile holds about R rows and never more than NarrowEntries(n) entries.
struct NarrowTiling {
    bool ok;
    int64_t share;
    int32_t lanes;  // of a lane group, fp32
};

NarrowTiling MakeNarrowTiling(int64_t rows, int64_t nnz, int32_t maxRow, int64_t n)
{
    NarrowTiling t{};
    if (n < 1 || n > 16 || maxRow < 1 || maxRow > kNarrowMaxRow || rows <= 0 || nnz <= 0) {
        return t;
    }
    const double perRow = static_cast<double>(nnz) / static_cast<double>(rows) + 1.0;  // entries and the row itself
    const double budget = static_cast<double>(NarrowEntries(n) - maxRow);
    const int64_t pieces = (n + 3) / 4;
    for (int32_t lanes = 1; lanes <= 32; lanes *= 2) {
        const int64_t full = 250 / (lanes * pieces);  // rows that fill the lanes once (with a little room)
        if (full < 1) {
            break;
        }
        if (static_cast<double>(full) * perRow > budget) {
            continue;
        }
        int64_t r = full;
        if (lanes == 1) {
            while (r + full <= 3 * full && static_cast<double>(r + full) * perRow <= budget) {
                r += full;  // very short rows: two or three turns of the lanes a tile
            }
        }
        t.ok = true;
        t.share = static_cast<int64_t>(static_cast<double>(r) * perRow);
        t.share = t.share < 1 ? 1 : t.share;
        t.lanes = lanes;
        return t;
    }
    return t;
}

int64_t SlabShare(int64_t rows, int64_t nnz, int32_t maxRow, int64_t n)
{
    static const int64_t fixed =
        std::getenv("OPS_SPARSE_SPMM_SLAB_ENTRIES") != nullptr ? std::atoll(std::getenv("OPS_SPARSE_SPMM_SLAB_ENTRIES")) : 0;
    if (fixed <= 0) {
        const NarrowTiling narrow = MakeNarrowTiling(rows, nnz, maxRow, n);
        if (narrow.ok) {
            return narrow.share;
        }
    }
    const int64_t target = fixed > 0 ? fixed : (maxRow > 0 && maxRow <= 64 && n <= 128 ? kSlabTarget / 2 : kSlabTarget);
    const int64_t t = target < 64 ? 64 : target;
    int64_t rps = nnz > 0 ? t * rows / nnz : 4096;
    rps = rps < 16 ? 16 : (rps > 4096 ? 4096 : rps);
    return t + rps;
}

int64_t SlabCount(int64_t rows, int64_t nnz, int32_t maxRow, int64_t n)
{
    const int64_t share = SlabShare(rows, nnz, maxRow, n);
    return (rows + nnz + share - 1) / share;
}

// Workspace: 256-byte header | first row per slab (+1) | long row ids | first segment per long row (+1) |
// row id per segment | first entry per segment | fp64 partials [segments x n].
void LayoutPlan(OpsparseSpmmPlan *p)
{
    int64_t off = 256;
    p->numSlabs = SlabCount(p->rows, p->nnz, p->maxRowNnz, p->n);  // (maxRowNnz and n set by the caller)
    p->slabStartOff = off;
    // Room for the table of any narrower B: a buffer sized for a wide B serves a narrower one as well.  (The share
    // of a slab depends on the pieces of 16 bytes in a row of B up to four of them, and not on n beyond.)
    int64_t reserveSlabs = 0;
    for (int64_t width : {4, 8, 12, 16, 17}) {
        const int64_t count = SlabCount(p->rows, p->nnz, p->maxRowNnz, width);
        reserveSlabs = count > reserveSlabs ? count : reserveSlabs;
    }
    off = Align256(off + 4 * ((reserveSlabs > p->numSlabs ? reserveSlabs : p->numSlabs) + 1));
    const int64_t slabEnd = off;
    p->longRowsOff = off;
    off = Align256(off + 4 * static_cast<int64_t>(p->numLongRows));
    p->longFirstSegOff = off;
    off = Align256(off + 4 * (static_cast<int64_t>(p->numLongRows) + 1));
    p->segRowOff = off;
    off = Align256(off + 4 * static_cast<int64_t>(p->numSegments));
    p->segStartOff = off;
    off = Align256(off + 4 * static_cast<int64_t>(p->numSegments));
    p->partialOff = off;
    off = Align256(off + 8 * static_cast<int64_t>(p->numSegments) * p->n);
    p->bytes = p->numLongRows > 0 ? off : slabEnd;
}

// slabStart[s] = first row r with rowOffsets[r] + r >= s * share (slabStart[numSlabs] = rows).
__global__ __launch_bounds__(kBlockThreads) void SpmmSlabTableKernel(const int32_t *__restrict__ rowOffsets,
                                                                    int64_t rows, int64_t numSlabs, int64_t share,
                                                                    int32_t *__restrict__ slabStart)
{
    const int64_t s = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (s > numSlabs) {
        return;
    }
    int64_t lo = 0, hi = rows;
    if (s == numSlabs) {
        lo = rows;
    } else {
        const int64_t want = s * share;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (static_cast<int64_t>(rowOffsets[mid]) - rowOffsets[0] + mid < want) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
    }
    slabStart[s] = static_cast<int32_t>(lo);
}

// Tables of the long rows: longRows[i] = row, firstSeg[i] = its first segment (firstSeg[numLongRows] = all
// segments), and for every segment its row and first entry.  `counter` starts at zero.
__global__ __launch_bounds__(kBlockThreads) void SpmmLongTablesKernel(
    const int32_t *__restrict__ rowOffsets, int64_t rows, int32_t numLongRows, int32_t numSegments,
    unsigned long long *__restrict__ counter, int32_t *__restrict__ longRows, int32_t *__restrict__ firstSeg,
    int32_t *__restrict__ segRow, int32_t *__restrict__ segStart)
{
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const int32_t first = rowOffsets[r];
    const int32_t len = rowOffsets[r + 1] - first;
    if (len <= kLongRowNnz) {
        return;
    }
    const int32_t segments = (len + kSegmentNnz - 1) / kSegmentNnz;
    const unsigned long long old = atomicAdd(counter, (1ull << 32) | static_cast<unsigned int>(segments));
    const int64_t index = static_cast<int64_t>(old >> 32);
    const int64_t seg0 = static_cast<int64_t>(old & 0xffffffffull);
    if (index >= numLongRows || seg0 + segments > numSegments) {
        return;  // more long rows than were counted: the host sees it in the counter
    }
    longRows[index] = static_cast<int32_t>(r);
    firstSeg[index] = static_cast<int32_t>(seg0);
    if (index == numLongRows - 1) {
        firstSeg[numLongRows] = static_cast<int32_t>(seg0 + segments);
    }
    for (int32_t j = 0; j < segments; ++j) {
        segRow[seg0 + j] = static_cast<int32_t>(r);
        segStart[seg0 + j] = first + j * kSegmentNnz;
    }
}

// Device reduction of the row lengths into `scratch` (>= 16 bytes), read back
// after a stream synchronisation.
int RowStats(const int32_t *rowOffsets, int64_t rows, int32_t *scratch, hipStream_t s, int32_t out[3])
{
    out[0] = out[1] = out[2] = 0;
    if (rows <= 0) {
        return OPSPARSE_OK;
    }
    if (hipMemsetAsync(scratch, 0, 16, s) != hipSuccess) {
        return OPSPARSE_E_LAUNCH;
    }
    int64_t grid = (rows + kBlockThreads - 1) / kBlockThreads;
    grid = grid > 4096 ? 4096 : grid;
    hipLaunchKernelGGL(SpmmRowStatsKernel, dim3(static_cast<uint32_t>(grid)), dim3(kBlockThreads), 0, s, rowOffsets,
                       rows, scratch);
    if (hipMemcpyAsync(out, scratch, 12, hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    return OPSPARSE_OK;
}

// OPS_SPARSE_SPMM_NO_BINNING: no row is cut into segments; a matrix with rows beyond kLongRowNnz entries then goes
// to the kernel with a lane group a row (for measurements).
bool NoBinning()
{
    const bool force = std::getenv("OPS_SPARSE_SPMM_NO_BINNING") != nullptr;
    return force;
}

template <typename ValT, typename CT, typename AccT, int V, int L>
void LaunchLongRows(const SpmmArgs &a);

template <typename ValT, typename CT, typename AccT, int V, int L>
int LaunchRowSplit(const SpmmArgs &a)
{
    constexpr int kGroups = kBlockThreads / L;
    const bool binned = a.plan != nullptr && a.plan->kernel == OPSPARSE_SPMM_BINNED && a.plan->numLongRows > 0;
    const int64_t rowsPerBlock = static_cast<int64_t>(kGroups) * kSpmmRowsPerGroup;
    const int64_t slots = a.rows;
    const uint32_t grid = static_cast<uint32_t>((slots + rowsPerBlock - 1) / rowsPerBlock);
    if (slots > 0) {
        hipLaunchKernelGGL((SpmmRowSplitKernel<ValT, CT, AccT, V, L>), dim3(grid), dim3(kBlockThreads), 0, a.stream,
                           a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                           static_cast<const ValT *>(a.B), static_cast<CT *>(a.C), slots, static_cast<int32_t>(a.n),
                           a.ldb, a.ldc, binned ? a.plan->longRowNnz : INT32_MAX, a.alpha, a.beta, a.clampF16);
    }
    if (binned) {
        LaunchLongRows<ValT, CT, AccT, V, L>(a);
    }
    return CheckLaunch();
}

// Segment + fix-up kernels for the long rows of a BINNED plan.
template <typename ValT, typename CT, typename AccT, int V, int L>
void LaunchLongRows(const SpmmArgs &a)
{
    constexpr int kGroups = kBlockThreads / L;
    auto *base = static_cast<unsigned char *>(a.ws);
    const auto *longRows = reinterpret_cast<const int32_t *>(base + a.plan->longRowsOff);
    const auto *firstSeg = reinterpret_cast<const int32_t *>(base + a.plan->longFirstSegOff);
    const auto *segRow = reinterpret_cast<const int32_t *>(base + a.plan->segRowOff);
    const auto *segStart = reinterpret_cast<const int32_t *>(base + a.plan->segStartOff);
    auto *partial = reinterpret_cast<AccT *>(base + a.plan->partialOff);
    const int32_t nseg = a.plan->numSegments;
    hipLaunchKernelGGL((SpmmLongSegmentKernel<ValT, AccT, V, L>), dim3((nseg + kGroups - 1) / kGroups),
                       dim3(kBlockThreads), 0, a.stream, a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                       static_cast<const ValT *>(a.B), static_cast<int32_t>(a.n), a.ldb, nseg, segRow, segStart,
                       partial);
    const int32_t nlong = a.plan->numLongRows;
    hipLaunchKernelGGL((SpmmLongFixupKernel<CT, AccT>), dim3(nlong), dim3(kBlockThreads), 0, a.stream,
                       static_cast<CT *>(a.C), static_cast<int32_t>(a.n), a.ldc, nlong, longRows, firstSeg, partial,
                       a.alpha, a.beta, a.clampF16);
}

// The slab kernel needs an analysed matrix (it must know that no row it is given
// exceeds its LDS) and one column tile per lane group.
bool UseSlabKernel(const SpmmArgs &a, int64_t lanesNeeded)
{
    const bool off = std::getenv("OPS_SPARSE_SPMM_NO_SLAB") != nullptr;  // (read at every call: tests switch it)
    if (off || a.plan == nullptr || lanesNeeded > 64 * 65535) {
        return false;
    }
    const bool binned = a.plan->kernel == OPSPARSE_SPMM_BINNED && a.plan->numLongRows > 0;
    if (!binned && a.plan->maxRowNnz > kLongRowNnz) {
        return false;  // (only with OPS_SPARSE_SPMM_NO_BINNING) rows that do not fit the staging area
    }
    return binned || (a.plan->maxRowNnz > 0 && a.plan->maxRowNnz <= kSlabCap);
}

template <typename ValT, typename CT, typename AccT, int V, int L>
int LaunchSlab(const SpmmArgs &a)
{
    const bool binned = a.plan->kernel == OPSPARSE_SPMM_BINNED && a.plan->numLongRows > 0;
    // Slabs of about kSlabTarget entries: of equal work from the plan's table, of equal numbers of rows without it.
    const int64_t target = std::getenv("OPS_SPARSE_SPMM_SLAB_ENTRIES") != nullptr
                                      ? std::atoll(std::getenv("OPS_SPARSE_SPMM_SLAB_ENTRIES"))
                                      : kSlabTarget;
    int64_t rps = a.nnz > 0 ? target * a.rows / a.nnz : 4096;
    rps = rps < 16 ? 16 : (rps > 4096 ? 4096 : rps);
    const bool noTable = std::getenv("OPS_SPARSE_SPMM_NO_SLAB_TABLE") != nullptr;
    const bool table = !noTable && a.plan->slabStartOff > 0 && a.plan->numSlabs > 0;
    const int32_t *slabStart =
        table ? reinterpret_cast<const int32_t *>(static_cast<unsigned char *>(a.ws) + a.plan->slabStartOff) : nullptr;
    const uint32_t grid = table ? static_cast<uint32_t>(a.plan->numSlabs) : static_cast<uint32_t>((a.rows + rps - 1) / rps);
    const int32_t longRowNnz = binned ? a.plan->longRowNnz : kSlabCap;
    const bool small32 = static_cast<uint64_t>(a.k) * static_cast<uint64_t>(a.ldb) * sizeof(ValT) < (1ull << 32);
    // Long rows: their segment workgroups ride in the same launch, the fix-up follows.
    constexpr int kGroups = kBlockThreads / L;
    // More columns than a lane group spans: one workgroup a (slab, tile of columns), the tiles of equal width (a
    // last tile of a few columns would cost a whole pass over the slab: n = 260, 8.2 ms against 5.0 ms).
    // A tile is a whole number of 64-byte pieces of a row of B: four lanes' loads share one (n = 1000 in tiles of
    // 252 columns 27.3 ms, in tiles of 256 25.1 ms).
    const int64_t vecs = (a.n + V - 1) / V;
    const uint32_t colTiles = static_cast<uint32_t>((vecs + L - 1) / L);
    int64_t tileVecs = (vecs + colTiles - 1) / colTiles;
    if (colTiles > 1) {
        tileVecs = (tileVecs + 3) / 4 * 4;  // (L is 64 here)
    }
    const int32_t tileCols = static_cast<int32_t>(tileVecs) * V;
    auto *base = static_cast<unsigned char *>(a.ws);
    const int32_t nseg = binned ? a.plan->numSegments : 0;
    const uint32_t segBlocks = static_cast<uint32_t>((nseg + kGroups - 1) / kGroups);
    const int32_t *segRow = binned ? reinterpret_cast<const int32_t *>(base + a.plan->segRowOff) : nullptr;
    const int32_t *segStart = binned ? reinterpret_cast<const int32_t *>(base + a.plan->segStartOff) : nullptr;
    AccT *partial = binned ? reinterpret_cast<AccT *>(base + a.plan->partialOff) : nullptr;
    auto launch = [&](auto tag) {
        constexpr bool kSmall = decltype(tag)::value;
        hipLaunchKernelGGL((SpmmSlabKernel<ValT, CT, AccT, V, L, kSmall>), dim3(grid + segBlocks, colTiles),
                           dim3(kBlockThreads),
                           0, a.stream, a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                           static_cast<const ValT *>(a.B), static_cast<CT *>(a.C), a.rows, static_cast<int32_t>(a.n),
                           a.ldb, a.ldc, static_cast<int32_t>(rps), slabStart, longRowNnz, a.alpha, a.beta, a.clampF16,
                           segBlocks, nseg, segRow, segStart, partial, tileCols);
    };
    if (small32) {
        launch(std::true_type{});
    } else {
        launch(std::false_type{});
    }
    if (binned) {
        const auto *longRows = reinterpret_cast<const int32_t *>(base + a.plan->longRowsOff);
        const auto *firstSeg = reinterpret_cast<const int32_t *>(base + a.plan->longFirstSegOff);
        const int32_t nlong = a.plan->numLongRows;
        hipLaunchKernelGGL((SpmmLongFixupKernel<CT, AccT>), dim3(nlong), dim3(kBlockThreads), 0, a.stream,
                           static_cast<CT *>(a.C), static_cast<int32_t>(a.n), a.ldc, nlong, longRows, firstSeg, partial,
                           a.alpha, a.beta, a.clampF16);
    }
    return CheckLaunch();
}

// SpmmNarrowKernel for a plan whose slab table was cut for it; W columns: a.n of them, or (Ragged) the a.n columns
// rounded up to whole pieces.
template <typename ValT, typename CT, typename AccT, int W, bool Ragged = false>
int LaunchNarrow(const SpmmArgs &a)
{
    const auto *slabStart =
        reinterpret_cast<const int32_t *>(static_cast<unsigned char *>(a.ws) + a.plan->slabStartOff);
    const NarrowTiling tiling = MakeNarrowTiling(a.plan->rows, a.plan->nnz, a.plan->maxRowNnz, a.plan->n);
    // the tiling counted fp32 pieces: rows of fp16 have half as many, and twice the lanes each
    const int lanes = tiling.lanes * (4 / static_cast<int>(sizeof(ValT)));
    auto launch = [&](auto tag) {
        constexpr int G = decltype(tag)::value;
        static const int fit = [] {
            int blocks = 1;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, SpmmNarrowKernel<ValT, CT, AccT, W, G, Ragged>,
                                                             kBlockThreads, 0) != hipSuccess ||
                blocks < 1) {
                (void)hipGetLastError();
                blocks = 1;
            }
            return blocks;
        }();
        // persistent: the workgroups that fit the device at once walk over all tiles
        const int64_t resident = static_cast<int64_t>(ComputeUnits()) * fit;
        const uint32_t grid = static_cast<uint32_t>(a.plan->numSlabs < resident ? a.plan->numSlabs : resident);
        hipLaunchKernelGGL((SpmmNarrowKernel<ValT, CT, AccT, W, G, Ragged>), dim3(grid), dim3(kBlockThreads), 0,
                           a.stream, a.rowOffsets, a.colInd, static_cast<const ValT *>(a.vals),
                           static_cast<const ValT *>(a.B), static_cast<CT *>(a.C), static_cast<uint32_t>(a.ldb),
                           static_cast<uint32_t>(a.ldc), slabStart, a.plan->numSlabs, a.nnz, a.alpha, a.beta,
                           a.clampF16, static_cast<int32_t>(a.n));
        return CheckLaunch();
    };
    // fp32: 1 .. 32 lanes, fp16: 2 .. 64; with 16 columns (four fp32 pieces in the tiling's count) the tiling stops
    // at 16, because three rows of at most kNarrowMaxRow entries always fit a tile
    constexpr int kMin = 4 / static_cast<int>(sizeof(ValT));
    constexpr int kMax = (W >= 16 ? 16 : 32) * kMin;
    auto pick = [&](auto tag) {
        constexpr int G = decltype(tag)::value;
        if constexpr (G >= kMin && G <= kMax) {
            return launch(tag);
        } else {
            return static_cast<int>(OPSPARSE_E_INVALID);
        }
    };
    switch (lanes) {
        case 1: return pick(std::integral_constant<int, 1>{});
        case 2: return pick(std::integral_constant<int, 2>{});
        case 4: return pick(std::integral_constant<int, 4>{});
        case 8: return pick(std::integral_constant<int, 8>{});
        case 16: return pick(std::integral_constant<int, 16>{});
        case 32: return pick(std::integral_constant<int, 32>{});
        case 64: return pick(std::integral_constant<int, 64>{});
        default: return OPSPARSE_E_INVALID;
    }
}

// Whether a plan's slab table was cut for SpmmNarrowKernel and for as many columns as n rounded up to a multiple of
// four: an analysed matrix of short rows.
bool PlanTakesNarrow(const OpsparseSpmmPlan *plan, const void *workspace, int64_t n, int64_t nnz)
{
    const bool off = std::getenv("OPS_SPARSE_SPMM_NO_NARROW") != nullptr;  // (read at every call: tests switch it)
    if (off || plan == nullptr || workspace == nullptr || n < 1 || n > 16 || nnz < 4 ||
        nnz > INT32_MAX - 4 * NarrowEntries(n) || plan->numSlabs > INT32_MAX / 2 ||
        (plan->n + 3) / 4 != (n + 3) / 4) {
        return false;
    }
    const OpsparseSpmmPlan &p = *plan;
    if (p.kernel == OPSPARSE_SPMM_BINNED || p.numLongRows != 0 || p.slabStartOff <= 0 || p.numSlabs <= 0 ||
        std::getenv("OPS_SPARSE_SPMM_NO_SLAB_TABLE") != nullptr) {
        return false;
    }
    const NarrowTiling tiling = MakeNarrowTiling(p.rows, p.nnz, p.maxRowNnz, p.n);
    return tiling.ok && SlabShare(p.rows, p.nnz, p.maxRowNnz, p.n) == tiling.share;
}

// Whether the product takes SpmmNarrowKernel on whole 16-byte rows of B of one or two pieces.
template <typename ValT>
bool UseNarrowKernel(const SpmmArgs &a)
{
    const int64_t rowBytes = a.n * static_cast<int64_t>(sizeof(ValT));
    if (sizeof(ValT) < 2 || (rowBytes != 16 && rowBytes != 32) || a.ldb > UINT32_MAX || a.ldc > UINT32_MAX ||
        a.plan == nullptr || a.plan->n != a.n) {
        return false;
    }
    return PlanTakesNarrow(a.plan, a.ws, a.n, a.nnz);
}

// ... and on row-major fp32 B and C of at most 8 columns that are not that: another width, leading dimension or
// alignment.  The plan is one for the width rounded up to a multiple of four.
bool UseNarrowRagged(const SpmmArgs &a)
{
    return !a.bColMajor && !a.cColMajor && !a.transB && a.n >= 1 && a.n <= 8 && a.ldb >= a.n && a.ldc >= a.n &&
           a.ldb <= UINT32_MAX && a.ldc <= UINT32_MAX && reinterpret_cast<uintptr_t>(a.B) % 4 == 0 &&
           reinterpret_cast<uintptr_t>(a.C) % 4 == 0 && PlanTakesNarrow(a.plan, a.ws, a.n, a.nnz);
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

// V elements of B per lane and gather.  LMin .. LMax: the widths of lane group that the caller's range of n can ask
// for (the others are not compiled).
template <typename ValT, typename CT, typename AccT, int V, int LMin = 2, int LMax = 64>
int RunTypedV(const SpmmArgs &a)
{
    const bool fast = !a.bColMajor && !a.cColMajor && !a.transB && a.n % V == 0 && a.ldb % V == 0 &&
                      a.ldc % V == 0 && reinterpret_cast<uintptr_t>(a.B) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(a.C) % 16 == 0;
    if constexpr (std::is_same<ValT, float>::value && std::is_same<CT, float>::value) {
        if (!fast && UseNarrowRagged(a)) {
            return a.n <= 4 ? LaunchNarrow<ValT, CT, AccT, 4, true>(a) : LaunchNarrow<ValT, CT, AccT, 8, true>(a);
        }
    }
    if (!fast) {
        return RunGeneral<ValT, CT, AccT>(a);
    }
    const int64_t lanesNeeded = a.n / V;
    if constexpr (V * sizeof(ValT) == 16) {
        if (UseNarrowKernel<ValT>(a)) {
            return lanesNeeded == 1 ? LaunchNarrow<ValT, CT, AccT, V>(a) : LaunchNarrow<ValT, CT, AccT, 2 * V>(a);
        }
    }
    const bool slab = UseSlabKernel(a, lanesNeeded);
    auto launch = [&](auto tag) {
        constexpr int L = decltype(tag)::value;
        if constexpr (L >= LMin && L <= LMax) {
            return slab ? LaunchSlab<ValT, CT, AccT, V, L>(a) : LaunchRowSplit<ValT, CT, AccT, V, L>(a);
        } else {
            return static_cast<int>(OPSPARSE_E_INVALID);  // (n outside the range this V is called for)
        }
    };
    if (lanesNeeded <= 2) return launch(std::integral_constant<int, 2>{});
    if (lanesNeeded <= 4) return launch(std::integral_constant<int, 4>{});
    if (lanesNeeded <= 8) return launch(std::integral_constant<int, 8>{});
    if (lanesNeeded <= 16) return launch(std::integral_constant<int, 16>{});
    if (lanesNeeded <= 32) return launch(std::integral_constant<int, 32>{});
    return launch(std::integral_constant<int, 64>{});
}

template <typename ValT, typename CT, typename AccT>
int RunTyped(const SpmmArgs &a)
{
    return RunTypedV<ValT, CT, AccT, 16 / static_cast<int>(sizeof(ValT))>(a);  // 16 bytes of B per lane
}

}  // namespace
}  // namespace opsparse

using namespace opsparse;

extern "C" {

int opsparse_spmm_csr_workspace_bytes(const int32_t *rowOffsets, int64_t rows, int64_t nnz, int64_t n, void *stream,
                                      size_t *bytes)
{
    if (bytes == nullptr || rows < 0 || nnz < 0 || n < 0 || (rows > 0 && rowOffsets == nullptr)) {
        return OPSPARSE_E_INVALID;
    }
    *bytes = 256;
    if (rows == 0 || nnz <= kLongRowNnz) {
        return OPSPARSE_OK;  // no row can be long
    }
    int32_t *scratch = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&scratch), 256) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    int32_t st[3];
    const int rc = RowStats(rowOffsets, rows, scratch, static_cast<hipStream_t>(stream), st);
    (void)hipFree(scratch);
    if (rc != OPSPARSE_OK) {
        return rc;
    }
    if (NoBinning()) {
        st[1] = st[2] = 0;
    }
    OpsparseSpmmPlan p{};
    p.rows = rows;
    p.nnz = nnz;
    p.n = n;
    p.maxRowNnz = st[0];
    p.numLongRows = st[1];
    p.numSegments = st[2];
    LayoutPlan(&p);
    *bytes = static_cast<size_t>(p.bytes);
    return OPSPARSE_OK;
}

int opsparse_spmm_csr_analyse(const int32_t *rowOffsets, int64_t rows, int64_t nnz, int64_t n, void *workspace,
                              size_t workspaceBytes, int32_t forceKernel, OpsparseSpmmPlan *plan, void *stream)
{
    if (plan == nullptr || rows < 0 || nnz < 0 || n < 0 || (rows > 0 && rowOffsets == nullptr)) {
        return OPSPARSE_E_INVALID;
    }
    if (workspace == nullptr || workspaceBytes < 256) {
        return OPSPARSE_E_WORKSPACE;
    }
    auto s = static_cast<hipStream_t>(stream);
    OpsparseSpmmPlan p{};
    p.kernel = OPSPARSE_SPMM_ROW_SPLIT;
    p.rows = rows;
    p.nnz = nnz;
    p.n = n;
    p.longRowNnz = kLongRowNnz;
    p.segmentNnz = kSegmentNnz;
    p.bytes = 256;
    if (rows == 0 || nnz <= kLongRowNnz || forceKernel == OPSPARSE_SPMM_ROW_SPLIT) {
        *plan = p;
        return OPSPARSE_OK;
    }
    int32_t st[3];
    int rc = RowStats(rowOffsets, rows, static_cast<int32_t *>(workspace), s, st);
    if (rc != OPSPARSE_OK) {
        return rc;
    }
    if (NoBinning()) {
        st[1] = st[2] = 0;
    }
    p.maxRowNnz = st[0];
    p.numLongRows = st[1];
    p.numSegments = st[2];
    LayoutPlan(&p);
    auto *base = static_cast<unsigned char *>(workspace);
    if (static_cast<int64_t>(workspaceBytes) >= p.slabStartOff + 4 * (p.numSlabs + 1)) {
        hipLaunchKernelGGL(SpmmSlabTableKernel, dim3(static_cast<uint32_t>((p.numSlabs + kBlockThreads) / kBlockThreads)),
                           dim3(kBlockThreads), 0, s, rowOffsets, rows, p.numSlabs, SlabShare(rows, nnz, p.maxRowNnz, n),
                           reinterpret_cast<int32_t *>(base + p.slabStartOff));
    } else if (st[1] == 0) {
        p.slabStartOff = 0;  // a 256-byte workspace, which is all a matrix without long rows used to need:
        p.numSlabs = 0;      // slabs of equal numbers of rows then
        p.bytes = 256;
    }
    if (st[1] == 0) {
        p.numLongRows = 0;
        p.numSegments = 0;
        *plan = p;
        return CheckLaunch();
    }
    p.kernel = OPSPARSE_SPMM_BINNED;
    if (static_cast<int64_t>(workspaceBytes) < p.bytes) {
        return OPSPARSE_E_WORKSPACE;
    }
    // The long-row tables are written by one kernel: a long row takes its number among the long rows and its
    // first segment from ONE 64-bit counter (rows in the upper half, segments in the lower), so the two
    // numberings agree and firstSeg is a prefix sum whatever order the rows arrive in.  Nothing but the counter
    // comes back to the host (the reference copies the row offsets to the host and builds its tables there,
    // sparse/spmm/arch35/spmm_csr_mat.cpp:94-136).
    auto *counter = reinterpret_cast<unsigned long long *>(base + 16);
    if (hipMemsetAsync(counter, 0, sizeof(unsigned long long), s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    hipLaunchKernelGGL(SpmmLongTablesKernel, dim3(static_cast<uint32_t>((rows + kBlockThreads - 1) / kBlockThreads)),
                       dim3(kBlockThreads), 0, s, rowOffsets, rows, p.numLongRows, p.numSegments, counter,
                       reinterpret_cast<int32_t *>(base + p.longRowsOff),
                       reinterpret_cast<int32_t *>(base + p.longFirstSegOff),
                       reinterpret_cast<int32_t *>(base + p.segRowOff),
                       reinterpret_cast<int32_t *>(base + p.segStartOff));
    unsigned long long counted = 0;
    if (hipMemcpyAsync(&counted, counter, sizeof(counted), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess) {
        (void)hipGetLastError();
        return OPSPARSE_E_LAUNCH;
    }
    if (counted != ((static_cast<unsigned long long>(p.numLongRows) << 32) | static_cast<unsigned int>(p.numSegments))) {
        return OPSPARSE_E_INVALID;  // the matrix changed between the two passes
    }
    *plan = p;
    return OPSPARSE_OK;
}

int opsparse_spmm_csr_launch(const OpsparseSpmmPlan *plan, const int32_t *rowOffsets, const int32_t *colInd,
                             const void *csrValues, const void *B, void *C, int64_t rows, int64_t k, int64_t n,
                             int64_t nnz, int64_t ldb, int64_t ldc, int32_t bColMajor, int32_t cColMajor,
                             int32_t transB, OpsparseScalar alpha, OpsparseScalar beta, int32_t valType,
                             int32_t cType, void *workspace, size_t workspaceBytes, void *stream)
{
    if (rows < 0 || k < 0 || n < 0 || nnz < 0 || ldb <= 0 || ldc <= 0 || n > INT32_MAX) {
        return OPSPARSE_E_INVALID;
    }
    if (rows == 0 || n == 0) {
        return OPSPARSE_OK;
    }
    if (rowOffsets == nullptr || C == nullptr ||
        (nnz > 0 && (colInd == nullptr || csrValues == nullptr || B == nullptr))) {
        return OPSPARSE_E_INVALID;
    }
    if (plan != nullptr) {
        if (plan->rows != rows || plan->nnz != nnz || (plan->kernel == OPSPARSE_SPMM_BINNED && plan->n != n)) {
            return OPSPARSE_E_INVALID;
        }
        if (plan->kernel == OPSPARSE_SPMM_BINNED &&
            (workspace == nullptr || static_cast<int64_t>(workspaceBytes) < plan->bytes)) {
            return OPSPARSE_E_WORKSPACE;
        }
    }
    SpmmArgs a{rowOffsets, colInd, csrValues, B, C, rows, k, n, nnz, ldb, ldc, bColMajor, cColMajor, transB, 0,
               alpha, beta, static_cast<hipStream_t>(stream), plan, workspace};
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
        // 8 bytes of B per lane, 4 for narrow B: with 16 the sixteen byte extractions and integer multiply-adds
        // per gather outweigh the gather itself (1 M rows of 32, n = 256: 6.1 ms with 16, 1.65 ms with 8, 2.7 ms
        // with 4; n = 16: 0.50 ms with 4, 0.54 ms with 8; the one-column-per-lane kernel 10.6 ms and 0.72 ms).
        if (a.n <= 32) {
            return RunTypedV<int8_t, int32_t, int32_t, 4, 2, 8>(a);   // n / 4 <= 8 lanes
        }
        return RunTypedV<int8_t, int32_t, int32_t, 8, 8, 64>(a);      // n / 8 >= 5 lanes

    }
    return OPSPARSE_E_UNSUPPORTED;
}

int opsparse_spmm_csr_narrow_rows(const OpsparseSpmmPlan *plan, const void *workspace, int64_t n, int64_t nnz,
                                  int32_t valType, int32_t cType)
{
    return valType == OPSPARSE_F32 && cType == OPSPARSE_F32 && n <= 8 && PlanTakesNarrow(plan, workspace, n, nnz) ? 1
                                                                                                                   : 0;
}

int opsparse_dense_restage(const void *src, void *dst, int64_t rows, int64_t cols, int64_t colsDst, int64_t ldSrc,
                           int32_t srcColMajor, int64_t ldDst, int32_t dstColMajor, int32_t elemBytes, void *stream)
{
    if (rows < 0 || cols < 0 || colsDst < cols || ldSrc <= 0 || ldDst <= 0 ||
        (elemBytes != 1 && elemBytes != 2 && elemBytes != 4)) {
        return OPSPARSE_E_INVALID;
    }
    // the source is read through the index formula whatever its ld (a transposed reading of B may overlap);
    // the destination's rows / columns must not
    if (ldDst < (dstColMajor ? rows : colsDst)) {
        return OPSPARSE_E_INVALID;
    }
    if (rows == 0 || colsDst == 0) {
        return OPSPARSE_OK;
    }
    if (src == nullptr || dst == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    auto s = static_cast<hipStream_t>(stream);
    if (colsDst <= 32 && (rows + kBlockThreads - 1) / kBlockThreads <= INT32_MAX) {
        const dim3 narrowGrid(static_cast<uint32_t>((rows + kBlockThreads - 1) / kBlockThreads));
        const uintptr_t group = 4 * static_cast<uintptr_t>(elemBytes);
        const bool vecSrc = !srcColMajor && ldSrc % 4 == 0 && reinterpret_cast<uintptr_t>(src) % group == 0;
        const bool vecDst = !dstColMajor && ldDst % 4 == 0 && colsDst % 4 == 0 &&
                            reinterpret_cast<uintptr_t>(dst) % group == 0;
        auto launch = [&](auto zero) {
            using T = decltype(zero);
            auto kernel = vecSrc ? (vecDst ? DenseRestageNarrowKernel<T, true, true> : DenseRestageNarrowKernel<T, true, false>)
                                 : (vecDst ? DenseRestageNarrowKernel<T, false, true> : DenseRestageNarrowKernel<T, false, false>);
            hipLaunchKernelGGL(kernel, narrowGrid, dim3(kBlockThreads), 0, s, static_cast<const T *>(src),
                               static_cast<T *>(dst), rows, static_cast<int32_t>(cols), static_cast<int32_t>(colsDst),
                               ldSrc, srcColMajor, ldDst, dstColMajor);
        };
        if (elemBytes == 4) {
            launch(uint32_t{});
        } else if (elemBytes == 2) {
            launch(uint16_t{});
        } else {
            launch(uint8_t{});
        }
        return CheckLaunch();
    }
    const int64_t across = (colsDst + 31) / 32, down = (rows + 31) / 32;
    if (across * down > INT32_MAX) {
        return OPSPARSE_E_UNSUPPORTED;
    }
    const dim3 grid(static_cast<uint32_t>(across * down));
    switch (elemBytes) {
        case 4:
            hipLaunchKernelGGL(DenseRestageKernel<uint32_t>, grid, dim3(kBlockThreads), 0, s,
                               static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), rows, cols, colsDst,
                               ldSrc, srcColMajor, ldDst, dstColMajor, across);
            break;
        case 2:
            hipLaunchKernelGGL(DenseRestageKernel<uint16_t>, grid, dim3(kBlockThreads), 0, s,
                               static_cast<const uint16_t *>(src), static_cast<uint16_t *>(dst), rows, cols, colsDst,
                               ldSrc, srcColMajor, ldDst, dstColMajor, across);
            break;
        default:
            hipLaunchKernelGGL(DenseRestageKernel<uint8_t>, grid, dim3(kBlockThreads), 0, s,
                               static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), rows, cols, colsDst,
                               ldSrc, srcColMajor, ldDst, dstColMajor, across);
            break;
    }
    return CheckLaunch();
}

}  // extern "C"
