// Yard-stick kernels for the measurement harness: what this GPU delivers for a
// plain copy, a plain read and a random 4-byte gather.  They bound what the
// SpMV / SpMM kernels can reach (and the copy kernel calibrates the FETCH_SIZE /
// WRITE_SIZE hardware counters, whose units differ from bytes by a constant).
#include "device_utils.h"

namespace opsparse {

typedef uint32_t Uint4V __attribute__((ext_vector_type(4)));
constexpr int kUnroll = 4;

// dst = src, 16 bytes per lane and step, four independent steps in flight.
__global__ __launch_bounds__(kBlockThreads) void CopyKernel(const Uint4V *__restrict__ src, Uint4V *__restrict__ dst,
                                                            size_t n16)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlockThreads * kUnroll;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlockThreads * kUnroll + threadIdx.x; i < n16; i += stride) {
        Uint4V v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t j = i + static_cast<size_t>(u) * kBlockThreads;
            if (j < n16) {
                v[u] = __builtin_nontemporal_load(src + j);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t j = i + static_cast<size_t>(u) * kBlockThreads;
            if (j < n16) {
                __builtin_nontemporal_store(v[u], dst + j);
            }
        }
    }
}

// Reads src once; the xor of everything goes to sink only if it matches a value
// it cannot have, so nothing is written.
__global__ __launch_bounds__(kBlockThreads) void ReadKernel(const Uint4V *__restrict__ src, size_t n16,
                                                            uint32_t *__restrict__ sink)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlockThreads * kUnroll;
    uint32_t acc = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlockThreads * kUnroll + threadIdx.x; i < n16; i += stride) {
        Uint4V v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t j = i + static_cast<size_t>(u) * kBlockThreads;
            v[u] = j < n16 ? __builtin_nontemporal_load(src + j) : Uint4V{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
        }
    }
    if (acc == 0x9e3779b9u && sink != nullptr) {
        sink[0] = acc;
    }
}

// sum of x[idx[i]]: one independent 4-byte gather per index, indices streamed.
__global__ __launch_bounds__(kBlockThreads) void GatherKernel(const int32_t *__restrict__ idx,
                                                              const float *__restrict__ x, size_t n,
                                                              float *__restrict__ sink)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlockThreads * kUnroll;
    float acc = 0.0f;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlockThreads * kUnroll + threadIdx.x; i < n; i += stride) {
        int32_t c[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t j = i + static_cast<size_t>(u) * kBlockThreads;
            c[u] = j < n ? __builtin_nontemporal_load(idx + j) : -1;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (c[u] >= 0) {
                acc += x[c[u]];
            }
        }
    }
    if (acc == 1.2345e30f && sink != nullptr) {
        sink[0] = acc;
    }
}

inline uint32_t MeasureGrid(size_t items)
{
    size_t grid = (items + static_cast<size_t>(kBlockThreads) * kUnroll - 1) / (static_cast<size_t>(kBlockThreads) * kUnroll);
    grid = grid > 16384 ? 16384 : grid;
    return static_cast<uint32_t>(grid < 1 ? 1 : grid);
}

}  // namespace opsparse

using namespace opsparse;

extern "C" {

int opsparse_copy_launch(const void *src, void *dst, size_t bytes, void *stream)
{
    if (src == nullptr || dst == nullptr || bytes % 16 != 0) {
        return OPSPARSE_E_INVALID;
    }
    if (bytes == 0) {
        return OPSPARSE_OK;
    }
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(CopyKernel, dim3(MeasureGrid(n16)), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const Uint4V *>(src), static_cast<Uint4V *>(dst), n16);
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

int opsparse_read_launch(const void *src, size_t bytes, void *sink, void *stream)
{
    if (src == nullptr || bytes % 16 != 0) {
        return OPSPARSE_E_INVALID;
    }
    if (bytes == 0) {
        return OPSPARSE_OK;
    }
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(ReadKernel, dim3(MeasureGrid(n16)), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const Uint4V *>(src), n16, static_cast<uint32_t *>(sink));
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

int opsparse_gather_launch(const int32_t *indices, const float *x, size_t count, void *sink, void *stream)
{
    if (indices == nullptr || x == nullptr) {
        return OPSPARSE_E_INVALID;
    }
    if (count == 0) {
        return OPSPARSE_OK;
    }
    hipLaunchKernelGGL(GatherKernel, dim3(MeasureGrid(count)), dim3(kBlockThreads), 0,
                       static_cast<hipStream_t>(stream), indices, x, count, static_cast<float *>(sink));
    return hipGetLastError() == hipSuccess ? OPSPARSE_OK : OPSPARSE_E_LAUNCH;
}

}  // extern "C"
