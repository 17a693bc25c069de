// Portable dequant-GEMV for every codec and shape the fast kernels do not cover
// (Q2_K / Q3_K / Q5_K / Q6_K, legacy rows with an odd number of blocks, very
// wide rows), plus the strided-input gather.
//
//     y[v, r] = sum_k x[v, k] * decode(W[r])[k] (+ bias[r])
//
// Same contraction as linear_into (crates/runtime-cpu/src/quantized.rs:419-499)
// with the per-codec decoders of decode_device.h. One wave owns a row; lane l
// decodes columns 4l..4l+3, 4(l+64).., reads the matching activations with one
// 16-byte load per vector (consecutive lanes, consecutive float4s) and the
// wave folds its 64 partial sums with DPP. f32 accumulation, tolerance 1e-3.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "decode_device.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

template <int CODEC, int M>
__global__ __launch_bounds__(256) void gemv_generic_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns) {
    constexpr uint32_t kValues = block_values(CODEC);
    constexpr uint32_t kBytes = block_bytes(CODEC);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t waves = gridDim.x * 4u;
    const uint64_t row_bytes = static_cast<uint64_t>(columns / kValues) * kBytes;
    const uint32_t quads = columns >> 2;
    for (uint32_t row = wave; row < rows; row += waves) {
        const uint8_t* packed = weight + row * row_bytes;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
        for (uint32_t quad = lane; quad < quads; quad += 64u) {
            const uint32_t column = quad << 2;
            const uint32_t block_index = column / kValues;
            float w[4];
            decode4<CODEC>(packed + static_cast<uint64_t>(block_index) * kBytes,
                           column - block_index * kValues, w);
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float4 xv = *reinterpret_cast<const float4*>(x + m * x_row_stride + column);
                acc[m] = fmaf(xv.x, w[0], acc[m]);
                acc[m] = fmaf(xv.y, w[1], acc[m]);
                acc[m] = fmaf(xv.z, w[2], acc[m]);
                acc[m] = fmaf(xv.w, w[3], acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float total = wave_sum(acc[m]);
            if (lane == 0)
                y[static_cast<uint64_t>(m) * rows + row] = bias != nullptr ? total + bias[row] : total;
        }
    }
}

template <int CODEC>
hipError_t launch_generic(const uint8_t* weight, const float* x, uint64_t x_row_stride,
                          const float* bias, float* y, uint32_t rows, uint32_t columns,
                          uint32_t vectors, hipStream_t stream) {
    uint32_t grid = (rows + 3u) / 4u;
    if (grid > 8192u) grid = 8192u;  // 32 waves per CU; the row loop takes the rest
#define ET_LAUNCH(MM)                                                                            \
    hipLaunchKernelGGL((gemv_generic_kernel<CODEC, MM>), dim3(grid), dim3(256), 0, stream, weight, \
                       x, x_row_stride, bias, y, rows, columns)
    switch (vectors) {
        case 1: ET_LAUNCH(1); break;
        case 2: ET_LAUNCH(2); break;
        case 3: ET_LAUNCH(3); break;
        case 4: ET_LAUNCH(4); break;
        default: return hipErrorInvalidValue;
    }
#undef ET_LAUNCH
    return hipGetLastError();
}

__device__ __forceinline__ uint64_t strided_index(const IndexLayout& layout, uint64_t logical) {
    uint64_t source = layout.offset;
    uint64_t remainder = logical;
    for (int d = layout.rank - 1; d >= 0; d--) {
        const uint64_t width = layout.shape[d] > 1 ? layout.shape[d] : 1;
        source += (remainder % width) * layout.strides[d];
        remainder /= width;
    }
    return source;
}

// crates/runtime-cpu/src/tensor.rs:940-953 applied to every element.
__global__ __launch_bounds__(256) void gather_f32_kernel(const float* __restrict__ src,
                                                         IndexLayout layout, uint64_t count,
                                                         float* __restrict__ dst) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count;
         i += stride)
        dst[i] = src[strided_index(layout, i)];
}

}  // namespace

hipError_t gemv_generic(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                        const float* bias, float* y, uint64_t rows, uint64_t columns,
                        uint32_t vectors, hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns);
    switch (codec) {
        case kQ4_0: return launch_generic<kQ4_0>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ8_0: return launch_generic<kQ8_0>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ2_K: return launch_generic<kQ2_K>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ3_K: return launch_generic<kQ3_K>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ4_K: return launch_generic<kQ4_K>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ5_K: return launch_generic<kQ5_K>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ6_K: return launch_generic<kQ6_K>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t gather_f32(const float* src, const IndexLayout& layout, uint64_t count, float* dst,
                      hipStream_t stream) {
    if (count == 0) return hipSuccess;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(gather_f32_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       src, layout, count, dst);
    return hipGetLastError();
}

}  // namespace et
