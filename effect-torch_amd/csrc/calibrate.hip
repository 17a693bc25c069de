// Measurement aids: a plain streaming read and a plain copy of known size.
//
// They give (a) the HBM bandwidth this device actually delivers to a kernel of
// the same footprint as a GEMV (the practical ceiling the dequant-GEMV is
// compared with, next to the published peak) and (b) a reference reading for
// hardware counters (FETCH_SIZE / WRITE_SIZE per byte actually moved).
// Nothing on the operator path uses them; the reference has no counterpart.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"

namespace et {
namespace {

// Each workgroup streams a contiguous range with 16-byte loads, four in flight
// per lane. The XOR of everything read leaves through one word per wave, so the
// loads cannot be removed; there is no barrier and no atomic on the way out.
__global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ src, uint32_t quads,
                                                   uint32_t* __restrict__ sink) {
    const uint32_t per_wg = (quads + gridDim.x - 1) / gridDim.x;
    const uint32_t begin = blockIdx.x * per_wg;
    const uint32_t end = min(begin + per_wg, quads);
    uint32_t acc = 0;
    uint32_t i = begin + threadIdx.x;
    for (; i + 3 * 256u < end; i += 4 * 256u) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = src[i + u * 256u];
#pragma unroll
        for (int u = 0; u < 4; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < end; i += 256u) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) acc ^= __shfl_xor(acc, offset);
    if ((threadIdx.x & 63u) == 0) sink[blockIdx.x * 4u + (threadIdx.x >> 6)] = acc;
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src,
                                                   uint4* __restrict__ dst, uint64_t quads) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256ull;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < quads; i += stride) dst[i] = src[i];
}

}  // namespace

hipError_t calibration_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups,
                            hipStream_t stream) {
    if (bytes < 16) return hipSuccess;
    hipLaunchKernelGGL(read_kernel, dim3(workgroups), dim3(256), 0, stream,
                       static_cast<const uint4*>(src), static_cast<uint32_t>(bytes / 16), sink);
    return hipGetLastError();
}

hipError_t calibration_copy(const void* src, void* dst, uint64_t bytes, hipStream_t stream) {
    if (bytes < 16) return hipSuccess;
    const uint64_t quads = bytes / 16;
    uint64_t blocks = (quads + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), quads);
    return hipGetLastError();
}

}  // namespace et
