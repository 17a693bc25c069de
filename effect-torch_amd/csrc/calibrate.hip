// Measurement aids: a plain streaming read and a plain copy of known size.
//
// They give (a) the HBM bandwidth this device actually delivers to a kernel of
// the same footprint as a GEMV (the practical ceiling the dequant-GEMV is
// compared with, next to the published peak) and (b) a reference reading for
// hardware counters (FETCH_SIZE / WRITE_SIZE per byte actually moved).
// Nothing on the operator path uses them; the reference has no counterpart.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "kernels.h"

namespace et {
namespace {

// Each workgroup streams a contiguous range with 16-byte loads, UNROLL in flight per lane.
template <int UNROLL, int THREADS = 256>
__global__ __launch_bounds__(THREADS) void read_kernel(const uint4* __restrict__ src, uint64_t quads,
                                                   uint32_t* __restrict__ sink) {
    const uint64_t per_wg = (quads + gridDim.x - 1) / gridDim.x;
    const uint64_t begin = blockIdx.x * per_wg;
    const uint64_t end = begin + per_wg < quads ? begin + per_wg : quads;
    uint32_t acc = 0;
    uint64_t i = begin + threadIdx.x;
    for (; i + (UNROLL - 1) * static_cast<uint64_t>(THREADS) < end; i += UNROLL * static_cast<uint64_t>(THREADS)) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = src[i + u * static_cast<uint64_t>(THREADS)];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < end; i += static_cast<uint64_t>(THREADS)) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    // The sum is data dependent, so the loads cannot be removed; one word per workgroup leaves.
    __shared__ uint32_t folded;
    if (threadIdx.x == 0) folded = 0;
    __syncthreads();
    atomicXor(&folded, acc);
    __syncthreads();
    if (threadIdx.x == 0) sink[blockIdx.x] = folded;
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
    if (const char* exp = getenv("ET_CAL")) {  // EXPERIMENT HOOK: "unroll,threads"
        int u = 4, t = 256;
        sscanf(exp, "%d,%d", &u, &t);
#define ET_CASE(U, T)                                                                          \
    if (u == U && t == T) {                                                                    \
        hipLaunchKernelGGL((read_kernel<U, T>), dim3(workgroups), dim3(T), 0, stream,          \
                           static_cast<const uint4*>(src), bytes / 16, sink);                  \
        return hipGetLastError();                                                              \
    }
        ET_CASE(8, 256) ET_CASE(16, 256) ET_CASE(4, 512) ET_CASE(8, 512) ET_CASE(4, 1024) ET_CASE(8, 1024)
        ET_CASE(2, 1024) ET_CASE(16, 512) ET_CASE(2, 512) ET_CASE(1, 1024) ET_CASE(16, 64) ET_CASE(32, 64) ET_CASE(8, 64) ET_CASE(8, 128) ET_CASE(16, 128)
#undef ET_CASE
    }
    hipLaunchKernelGGL((read_kernel<4, 256>), dim3(workgroups), dim3(256), 0, stream,
                       static_cast<const uint4*>(src), bytes / 16, sink);
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
