// Device-side helpers shared by the SpMV and SpMM kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "ops_sparse_hip.h"

namespace opsparse {

constexpr int kWave = 64;          // wavefront width on CDNA
constexpr int kNumXcd = 8;         // accelerator dies, each with a private L2
constexpr int kBlockThreads = 256; // four wavefronts per workgroup

// ---- element conversion --------------------------------------------------
// Floating-point paths accumulate in double: an fp32 x fp32 product is exact
// in fp64, so a row sum carries one rounding per addition at 2^-53 and one
// final rounding to the output type.  Integer paths accumulate in int32 with
// two's-complement wrap-around, like an int32 loop on the host.

// fp16 is the compiler's native _Float16; bf16 is carried as its 16 raw bits
// (the upper half of an fp32), converted by hand with round-to-nearest-even.
typedef _Float16 Half;
struct Bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float Bf16ToFloat(Bf16 v)
{
    return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
}
__device__ __forceinline__ Bf16 FloatToBf16(float f)
{
    uint32_t u = __float_as_uint(f);
    Bf16 r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.bits = static_cast<uint16_t>((u >> 16) | 0x0040u);  // quiet NaN
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        r.bits = static_cast<uint16_t>(u >> 16);
    }
    return r;
}

template <typename AccT, typename T>
__device__ __forceinline__ AccT ToAcc(T v)
{
    return static_cast<AccT>(v);
}
template <>
__device__ __forceinline__ double ToAcc<double, Half>(Half v)
{
    return static_cast<double>(static_cast<float>(v));
}
template <>
__device__ __forceinline__ double ToAcc<double, Bf16>(Bf16 v)
{
    return static_cast<double>(Bf16ToFloat(v));
}

template <typename OutT, typename AccT>
__device__ __forceinline__ OutT FromAcc(AccT v)
{
    return static_cast<OutT>(v);
}
template <>
__device__ __forceinline__ Half FromAcc<Half, double>(double v)
{
    return static_cast<Half>(static_cast<float>(v));
}
template <>
__device__ __forceinline__ Bf16 FromAcc<Bf16, double>(double v)
{
    return FloatToBf16(static_cast<float>(v));
}

// ---- alpha / beta ----------------------------------------------------------

template <typename AccT>
__device__ __forceinline__ AccT ReadScalar(const OpsparseScalar &s)
{
    if (s.devicePtr == nullptr) {
        return static_cast<AccT>(s.value);
    }
    if (s.isInt) {
        return static_cast<AccT>(*static_cast<const int32_t *>(s.devicePtr));
    }
    return static_cast<AccT>(*static_cast<const float *>(s.devicePtr));
}

// ---- streaming loads -------------------------------------------------------
// csrValues / csrColInd are touched exactly once per product, so they are
// loaded with the non-temporal hint and do not displace x / B lines in L2.
// The 4-element vector types are declared 4-byte aligned: a merge-path block
// starts at an arbitrary nnz offset, and gfx950 global loads only need dword
// alignment.

typedef int32_t Int4U __attribute__((ext_vector_type(4), aligned(4)));
typedef float Float4U __attribute__((ext_vector_type(4), aligned(4)));
typedef uint16_t Short4U __attribute__((ext_vector_type(4), aligned(2)));  // four fp16 / bf16 values at any even address

template <typename T>
__device__ __forceinline__ T LoadStream(const T *p)
{
    return __builtin_nontemporal_load(p);
}
template <>
__device__ __forceinline__ Bf16 LoadStream<Bf16>(const Bf16 *p)
{
    Bf16 r;
    r.bits = __builtin_nontemporal_load(&p->bits);
    return r;
}

// ---- workgroup -> tile mapping ----------------------------------------------
// Hardware deals consecutive workgroup ids round-robin to the 8 XCDs.  Tiles
// that are neighbours in the matrix share x / B lines, so give every XCD one
// contiguous range of tiles: its L2 then holds each shared line once instead
// of all 8 L2s fetching it.
__device__ __forceinline__ uint32_t XcdContiguousTile(uint32_t bid, uint32_t numTiles)
{
    const uint32_t xcd = bid % kNumXcd;
    const uint32_t idx = bid / kNumXcd;
    const uint32_t per = numTiles / kNumXcd;
    const uint32_t rem = numTiles % kNumXcd;
    return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// ---- lane-group reduction ----------------------------------------------------
// Sum over the G consecutive lanes a value lives in (G a power of two <= 64).
// Every lane of the group ends with the total.
template <int G, typename T>
__device__ __forceinline__ T GroupSum(T v)
{
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, G);
    }
    return v;
}

template <typename T>
__device__ __forceinline__ T GroupSumDyn(T v, int g)
{
    for (int off = g >> 1; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, kWave);
    }
    return v;
}

// A workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load and store
// the wavefront has in flight; this one leaves them outstanding (a tile's loads issued ahead of their use).
__device__ __forceinline__ void LdsBarrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

}  // namespace opsparse
