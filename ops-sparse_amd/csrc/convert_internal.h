// Launchers of the conversion building blocks (convert_kernels.hip) that other
// parts of the library use: the SpMV column-panel and blocked-gather
// preprocessing re-store a CSR matrix with them.  Everything only enqueues work on `s`.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace opsparse {

// Number of int32 the prefix sum over `count` elements needs as scratch.
int64_t ScanScratchInts(int64_t count);

// out[i] = add + in[0] + ... + in[i] (in place allowed).  scratch: ScanScratchInts(count) ints.
void LaunchInclusiveScanI32(const int32_t *in, int32_t *out, int64_t count, int32_t add, int32_t *scratch, hipStream_t s);

// p[0..n) = v.
void LaunchFillI32(int32_t *p, int64_t n, int32_t v, hipStream_t s);

// rowInd[j] = i + base for j in [rowPtr[i], rowPtr[i+1]) - base.
void LaunchExpandRows(const int32_t *rowPtr, int64_t m, int64_t nnz, int32_t base, int32_t *rowInd, hipStream_t s);

// ptr[0..m] = base + prefix sums of the per-index counts of ind[0..nnz) (indices outside [0, m) ignored).
// scratch: ScanScratchInts(m + 1) ints.
void LaunchIndicesToOffsets(const int32_t *ind, int64_t nnz, int64_t m, int32_t base, int32_t *ptr, int32_t *scratch,
                            hipStream_t s);

// One stable 4-bit radix pass over n (key, payload) pairs on digit (key - keyBase) >> shift & 15.
// payIn == NULL: the payload of item i is i.  Keys are written without keyBase.
// table: RadixTableInts(n) ints; afterwards table[d * RadixTiles(n)] is the first output position of digit d.
// scratch: ScanScratchInts(RadixTableInts(n)) ints.
int64_t RadixTiles(int64_t n);
int64_t RadixTableInts(int64_t n);
void LaunchRadixPass(const int32_t *keysIn, const int32_t *payIn, int32_t *keysOut, int32_t *payOut, int64_t n,
                     int32_t keyBase, int32_t shift, int32_t *table, int32_t *scratch, hipStream_t s);

// rowOut[d] = rowOfPos[pos[d]]; valOut[d] = srcVal[pos[d]] (4-byte values; valOut may be NULL).
void LaunchGatherByPosition(const int32_t *pos, const int32_t *rowOfPos, const uint32_t *srcVal, int64_t nnz,
                            int32_t *rowOut, uint32_t *valOut, hipStream_t s);

}  // namespace opsparse
