// Arithmetic shared by the stand-alone decode operators (decode_ops.hip) and the activation
// quantisers that apply them on the fly (quantize_act.hip), so that the fused and the separate
// forms produce the same bits. Both translation units are compiled with -ffp-contract=off.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

namespace et {

__device__ __forceinline__ double wave_sum(double v) {
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset);
    return v;
}

constexpr int kRmsHeld = 4;  // float4 vectors of the row a thread keeps in registers between the passes

// First pass of rms_norm_forward_into_impl (crates/runtime-cpu/src/composed.rs:1457-1487) for one
// row and a workgroup of 256: returns 1 / sqrt(mean(x^2) + eps) in f64. The row is read as float4
// (columns % 4 == 0, 16-byte aligned); vector threadIdx.x + 256 j stays in held[j] for j < kRmsHeld.
__device__ __forceinline__ double rms_row_scale(const float* __restrict__ in, uint32_t columns, double eps,
                                                float4 (&held)[kRmsHeld], double (&partial)[4]) {
    const uint32_t vectors = columns / 4;
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < kRmsHeld; j++) {
        const uint32_t i = threadIdx.x + 256 * j;
        held[j] = i < vectors ? reinterpret_cast<const float4*>(in)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < kRmsHeld; j++) {
        const float4 v = held[j];
        sum += (static_cast<double>(v.x) * v.x + static_cast<double>(v.y) * v.y) +
               (static_cast<double>(v.z) * v.z + static_cast<double>(v.w) * v.w);
    }
    for (uint32_t i = threadIdx.x + 256 * kRmsHeld; i < vectors; i += 256) {
        const float4 v = reinterpret_cast<const float4*>(in)[i];
        sum += (static_cast<double>(v.x) * v.x + static_cast<double>(v.y) * v.y) +
               (static_cast<double>(v.z) * v.z + static_cast<double>(v.w) * v.w);
    }
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
    __syncthreads();
    const double mean_square = ((partial[0] + partial[1]) + (partial[2] + partial[3])) / static_cast<double>(columns);
    return 1.0 / sqrt(mean_square + eps);
}

// The weight of an RMS norm: f32, or f16 widened on use (exact), or none (ones). The reference casts
// a half-float parameter to the activations' type in front of the operator; reading the halves here
// gives the same values without the cast's launch.
struct NormWeight {
    const void* data;  // [columns], or null
    int32_t half;      // 0: float, 1: IEEE binary16
};
__device__ __forceinline__ float norm_weight_one(const NormWeight& w, uint32_t i) {
    if (w.data == nullptr) return 1.f;
    if (w.half) return static_cast<float>(static_cast<const _Float16*>(w.data)[i]);
    return static_cast<const float*>(w.data)[i];
}
// elements 4 i .. 4 i + 3 (the array is 16-byte aligned for floats, 8-byte aligned for halves)
__device__ __forceinline__ float4 norm_weight_four(const NormWeight& w, uint32_t i) {
    if (w.data == nullptr) return make_float4(1.f, 1.f, 1.f, 1.f);
    if (w.half) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        const h4 v = static_cast<const h4*>(w.data)[i];
        return make_float4(static_cast<float>(v.x), static_cast<float>(v.y), static_cast<float>(v.z), static_cast<float>(v.w));
    }
    return static_cast<const float4*>(w.data)[i];
}

// Second pass: x * scale * weight in f64, rounded once.
__device__ __forceinline__ float rms_one(float value, double scale, float w) {
    return static_cast<float>(static_cast<double>(value) * scale * static_cast<double>(w));
}
__device__ __forceinline__ float4 rms_four(const float4& v, double scale, const float4& w) {
    return make_float4(rms_one(v.x, scale, w.x), rms_one(v.y, scale, w.y), rms_one(v.z, scale, w.z),
                       rms_one(v.w, scale, w.w));
}

// One pair of rotary_forward_into_impl (crates/runtime-cpu/src/composed.rs:2683-2729): position =
// offset + step, angle = sign * position * theta^(-2 index / head_dim), everything in f64, each
// result rounded once.
__device__ __forceinline__ void rotate_pair(float a_in, float b_in, uint32_t offset, uint32_t step, uint32_t index,
                                            uint32_t head_dim, double theta, double sign, float& lo, float& hi) {
#pragma clang fp contract(off)  // every product and sum rounded on its own, whatever the file's setting
    const double angle = sign * static_cast<double>(static_cast<uint64_t>(offset) + step) *
                         pow(theta, -2.0 * static_cast<double>(index) / static_cast<double>(head_dim));
    double s, c;
    sincos(angle, &s, &c);
    const double a = a_in, b = b_in;
    lo = static_cast<float>(a * c - b * s);
    hi = static_cast<float>(b * c + a * s);
}

// Tensor.silu (packages/core/src/Tensor.ts:1537-1540) times the up projection. Tensor.sigmoid is
// tanh(x / 2) / 2 + 1 / 2, every step rounded to f32 (Tensor.ts:1240-1245).
__device__ __forceinline__ float silu_mul_one(float gate, float up) {
    const float sigmoid = tanhf(gate * 0.5f) * 0.5f + 0.5f;
    return (gate * sigmoid) * up;
}

}  // namespace et
