// int8-activation contraction on the gfx950 matrix cores (stage 2 of the
// int8-activation path; stage 1 is quantize_act.hip).
//
//   Q8_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i qw[n,b,i] * qx[m,b,i])
//   Q4_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i (nib[n,b,i] - 8) * qx[m,b,i])
//   Q4_K:  y[m, n] = sum_g s[m,g] * ( (d*sc_g)[n] * (sum_i nib * qx) - (dmin*m_g)[n] * sumq[m,g] )
// b / g index 32-column blocks; the inner sums are exact int32 and come from
// v_mfma_i32_32x32x32_i8, whose K = 32 is exactly one quantisation block. The
// f32 block-scale epilogue runs on the VALU after every MFMA. The reference has
// no int8 activation path (its Metal prefill kernel decodes to f32 and uses f32
// simdgroup MMA, crates/runtime-metal/src/quantized.rs:1016-1097).
//
// MFMA operand roles: A = activations (tile rows = vectors m), B = weights
// (tile columns = weight rows n). A lane of the 32x32 result then holds one n
// (= lane % 32) and sixteen m (= 8*(r/4) + 4*(lane/32) + r%4), so its weight
// scale is a single value per block and each result register row is written as
// 128 contiguous bytes of y.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct __attribute__((packed, aligned(2))) Bytes16 {
    uint32_t v[4];
};

// One wave owns a 32 (vectors) x 32 (weight rows) tile of y and walks all blocks.
template <int CODEC>
__global__ __launch_bounds__(256) void gemm_i8_kernel(
    const uint8_t* __restrict__ weight, const int8_t* __restrict__ q,
    const float* __restrict__ scale, const int32_t* __restrict__ sum,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t vectors) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t n0 = (blockIdx.x * 4u + wave) * 32u;
    const uint32_t m0 = blockIdx.y * 32u;
    if (n0 >= rows) return;

    // Operand rows of this lane. Rows past the end are clamped for the loads
    // and masked at the stores.
    const uint32_t n = min(n0 + (lane & 31u), rows - 1u);
    const uint32_t m_a = min(m0 + (lane & 31u), vectors - 1u);
    const bool a_valid = m0 + (lane & 31u) < vectors;
    const int8_t* a_row = q + static_cast<uint64_t>(m_a) * columns + 16u * half;

    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    v16i zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0;

    // Scales of the sixteen vectors this lane accumulates: scale[b * stride + m], where
    // stride = vectors rounded up to a whole tile, so the 16-byte loads never leave the array.
    const uint32_t stride = (vectors + 31u) & ~31u;
    auto load_scales = [&](const float* base, float (&out)[16]) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4 v = *reinterpret_cast<const float4*>(base + m0 + 8u * g + 4u * half);
            out[4 * g + 0] = v.x;
            out[4 * g + 1] = v.y;
            out[4 * g + 2] = v.z;
            out[4 * g + 3] = v.w;
        }
    };

    const uint32_t xblocks = columns >> 5;
    if (CODEC == kQ8_0 || CODEC == kQ4_0) {
        constexpr uint32_t kBytes = CODEC == kQ8_0 ? 34u : 18u;
        const uint8_t* w_row = weight + static_cast<uint64_t>(n) * xblocks * kBytes;
        for (uint32_t b = 0; b < xblocks; b++) {
            const uint8_t* block = w_row + b * kBytes;
            v4i bw;
            if (CODEC == kQ8_0) {
                const Bytes16 raw = *reinterpret_cast<const Bytes16*>(block + 2 + 16 * half);
                bw = v4i{static_cast<int>(raw.v[0]), static_cast<int>(raw.v[1]),
                         static_cast<int>(raw.v[2]), static_cast<int>(raw.v[3])};
            } else {
                // element j = low nibble of byte j (j < 16), element j+16 = high nibble:
                // lanes 0-31 take the low nibbles, lanes 32-63 the high ones.
                const Bytes16 raw = *reinterpret_cast<const Bytes16*>(block + 2);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (half ? (raw.v[i] >> 4) : raw.v[i]) & 0x0f0f0f0fu;
                    // (nib - 8) per byte: no borrow across bytes after setting bit 7 first
                    bw[i] = static_cast<int>(((nib | 0x80808080u) - 0x08080808u) ^ 0x80808080u);
                }
            }
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(block));
            v4i ax = *reinterpret_cast<const v4i*>(a_row + 32u * b);
            if (!a_valid) ax = v4i{0, 0, 0, 0};
            const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bw, zero, 0, 0, 0);
            float s[16];
            load_scales(scale + static_cast<uint64_t>(b) * stride, s);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = fmaf(static_cast<float>(c[r]), d * s[r], acc[r]);
        }
    } else {  // Q4_K
        const uint32_t blocks = columns >> 8;
        const uint8_t* w_row = weight + static_cast<uint64_t>(n) * blocks * 144u;
        for (uint32_t sb = 0; sb < blocks; sb++) {
            const uint8_t* block = w_row + sb * 144u;
            const uint4 header = *reinterpret_cast<const uint4*>(block);
            const float d = half_bits_to_float(header.x & 0xffffu);
            const float dmin = half_bits_to_float(header.x >> 16);
            for (uint32_t p = 0; p < 4; p++) {
                const uint4 raw = *reinterpret_cast<const uint4*>(block + 16 + 32 * p + 16 * half);
                const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int side = 0; side < 2; side++) {
                    // scale_min_k4 (crates/runtime-cpu/src/quantized.rs:77-86) for g = 2p + side
                    const uint32_t g = 2u * p + side;
                    const uint32_t shift = 8u * (g & 3u);
                    const uint32_t s0 = (header.y >> shift) & 0xffu;  // scales[g & 3]
                    const uint32_t s1 = (header.z >> shift) & 0xffu;  // scales[4 + (g & 3)]
                    const uint32_t s2 = (header.w >> shift) & 0xffu;  // scales[8 + (g & 3)]
                    const uint32_t sc = g < 4 ? (s0 & 63u) : ((s2 & 0x0fu) | ((s0 >> 6) << 4));
                    const uint32_t mn = g < 4 ? (s1 & 63u) : ((s2 >> 4) | ((s1 >> 6) << 4));
                    const float dl = d * static_cast<float>(sc);
                    const float ml = dmin * static_cast<float>(mn);
                    v4i bw;
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        bw[i] = static_cast<int>((side ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu);
                    const uint32_t b = sb * 8u + g;
                    v4i ax = *reinterpret_cast<const v4i*>(a_row + 32u * b);
                    if (!a_valid) ax = v4i{0, 0, 0, 0};
                    const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bw, zero, 0, 0, 0);
                    float s[16];
                    load_scales(scale + static_cast<uint64_t>(b) * stride, s);
                    const int32_t* sums = sum + static_cast<uint64_t>(b) * stride;
#pragma unroll
                    for (int gr = 0; gr < 4; gr++) {
                        const int4 xs = *reinterpret_cast<const int4*>(sums + m0 + 8u * gr + 4u * half);
                        const int xsum[4] = {xs.x, xs.y, xs.z, xs.w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int r = 4 * gr + j;
                            const float diff =
                                dl * static_cast<float>(c[r]) - ml * static_cast<float>(xsum[j]);
                            acc[r] = fmaf(s[r], diff, acc[r]);
                        }
                    }
                }
            }
        }
    }

    const uint32_t n_out = n0 + (lane & 31u);
    if (n_out < rows) {
        const float b = bias != nullptr ? bias[n_out] : 0.f;
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t m = m0 + 8u * g + 4u * half + j;
                if (m < vectors) y[static_cast<uint64_t>(m) * rows + n_out] = acc[4 * g + j] + b;
            }
    }
}

template <int CODEC>
hipError_t launch(const uint8_t* weight, const int8_t* q, const float* scale, const int32_t* sum,
                  const float* bias, float* y, uint32_t rows, uint32_t columns, uint32_t vectors,
                  hipStream_t stream) {
    const dim3 grid((rows + 127u) / 128u, (vectors + 31u) / 32u);
    hipLaunchKernelGGL(gemm_i8_kernel<CODEC>, grid, dim3(256), 0, stream, weight, q, scale, sum, bias,
                       y, rows, columns, vectors);
    return hipGetLastError();
}

}  // namespace

bool gemm_i8_supported(int32_t codec, uint64_t columns) {
    if (codec == kQ8_0 || codec == kQ4_0) return columns % 32 == 0;
    if (codec == kQ4_K) return columns % 256 == 0;
    return false;
}

hipError_t gemm_i8(int32_t codec, const uint8_t* weight, const int8_t* q, const float* scale,
                   const int32_t* sum, const float* bias, float* y, uint64_t rows, uint64_t columns,
                   uint64_t vectors, hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns),
                   m = static_cast<uint32_t>(vectors);
    switch (codec) {
        case kQ8_0: return launch<kQ8_0>(weight, q, scale, sum, bias, y, n, k, m, stream);
        case kQ4_0: return launch<kQ4_0>(weight, q, scale, sum, bias, y, n, k, m, stream);
        case kQ4_K: return launch<kQ4_K>(weight, q, scale, sum, bias, y, n, k, m, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
