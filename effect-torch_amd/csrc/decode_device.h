// Per-codec device decoders: decode4<CODEC>(block, e, out) produces the four
// values at positions e..e+3 (e % 4 == 0) of one packed block, following the
// reference's scalar decoders operation by operation
// (crates/runtime-cpu/src/quantized.rs: decode_q2_k :117-138, decode_q3_k
// :142-176, decode_q4_k :180-199, decode_q5_k :203-234, decode_q6_k :238-261;
// Q8_0 / Q4_0 follow the public ggml block layouts, which the reference lacks).
//
// Whether the results are bit-identical to the CPU depends on the including
// translation unit: with floating-point contraction off (as in dequant.hip)
// every multiply and subtract rounds separately, exactly like the reference.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "et_codecs.h"

namespace et {

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    // v_cvt_f32_f16: exact widening, subnormals included.
    union {
        uint16_t u;
        _Float16 h;
    } cvt;
    cvt.u = static_cast<uint16_t>(bits);
    return static_cast<float>(cvt.h);
}

// Little-endian loads at any address (blocks of 18, 34, 110 or 210 bytes are not dword aligned): one
// instruction each instead of a load per byte.
typedef uint16_t __attribute__((aligned(1))) Unaligned16;
typedef uint32_t __attribute__((aligned(1))) Unaligned32;
__device__ __forceinline__ uint32_t load16(const uint8_t* at) { return *reinterpret_cast<const Unaligned16*>(at); }
__device__ __forceinline__ uint32_t load32(const uint8_t* at) { return *reinterpret_cast<const Unaligned32*>(at); }
__device__ __forceinline__ uint32_t byte_of(uint32_t word, int i) { return (word >> (8 * i)) & 0xffu; }

__device__ __forceinline__ float f16_at(const uint8_t* block, uint32_t offset) {
    return f16_bits_to_f32(load16(block + offset));
}

// crates/runtime-cpu/src/quantized.rs:77-86; `scales` = the twelve packed bytes
__device__ __forceinline__ void scale_min_k4(uint32_t index, const uint8_t* scales, uint32_t& scale,
                                             uint32_t& min) {
    const uint32_t shift = 8u * (index & 3u);
    const uint32_t s0 = (load32(scales) >> shift) & 0xffu;      // scales[index & 3]
    const uint32_t s1 = (load32(scales + 4) >> shift) & 0xffu;  // scales[4 + (index & 3)]
    if (index < 4) {
        scale = s0 & 63u;
        min = s1 & 63u;
    } else {
        const uint32_t s2 = (load32(scales + 8) >> shift) & 0xffu;  // scales[8 + (index & 3)]
        scale = (s2 & 0x0fu) | ((s0 >> 6) << 4);
        min = (s2 >> 4) | ((s1 >> 6) << 4);
    }
}

// decode4<CODEC>(block, e, out): the four values at positions e..e+3 (e % 4 == 0)
// of one packed block.
template <int CODEC>
__device__ __forceinline__ void decode4(const uint8_t* block, uint32_t e, float out[4]);

template <>
__device__ __forceinline__ void decode4<kQ8_0>(const uint8_t* block, uint32_t e, float out[4]) {
    const float d = f16_at(block, 0);
    const uint32_t q = load32(block + 2 + e);
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = d * static_cast<float>(static_cast<int8_t>(byte_of(q, i)));
}

template <>
__device__ __forceinline__ void decode4<kQ4_0>(const uint8_t* block, uint32_t e, float out[4]) {
    const float d = f16_at(block, 0);
    const bool high = e >= 16;
    const uint32_t j = high ? e - 16 : e;
    const uint32_t q = load32(block + 2 + j);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t byte = byte_of(q, i);
        const int nib = static_cast<int>(high ? (byte >> 4) : (byte & 0x0fu)) - 8;
        out[i] = d * static_cast<float>(nib);
    }
}

template <>
__device__ __forceinline__ void decode4<kQ2_K>(const uint8_t* block, uint32_t e, float out[4]) {
    // group = half*8 + (shift/2)*2 + q_offset/16, 16 values per group
    const uint32_t group = e >> 4, i0 = e & 15u;
    const uint32_t half = group >> 3, shift = ((group >> 1) & 3u) * 2u, q_offset = (group & 1u) * 16u;
    const uint32_t scale = block[group];
    const float d = f16_at(block, 80), dmin = f16_at(block, 82);
    const float dl = d * static_cast<float>(scale & 0x0fu);
    const float ml = dmin * static_cast<float>(scale >> 4);
    const uint32_t q = load32(block + 16 + half * 32 + q_offset + i0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float prod = dl * static_cast<float>((byte_of(q, i) >> shift) & 3u);
        out[i] = prod - ml;
    }
}

template <>
__device__ __forceinline__ void decode4<kQ3_K>(const uint8_t* block, uint32_t e, float out[4]) {
    const uint32_t group = e >> 4, i0 = e & 15u;
    const uint32_t half = group >> 3, lane = (group >> 1) & 3u, q_offset = (group & 1u) * 16u;
    const uint32_t shift = lane * 2u, mask = 1u << (half * 4u + lane);
    const uint8_t* packed_scales = block + 96;
    const uint32_t low = group < 8 ? (packed_scales[group] & 0x0fu)
                                   : (static_cast<uint32_t>(packed_scales[group - 8]) >> 4);
    const uint32_t high = (static_cast<uint32_t>(packed_scales[8 + (group & 3u)]) >> (2u * (group >> 2))) & 3u;
    const int scale = static_cast<int>(low | (high << 4)) - 32;
    const float d = f16_at(block, 108);
    const float dl = d * static_cast<float>(scale);
    const uint32_t q = load32(block + 32 + half * 32 + q_offset + i0);
    const uint32_t hm = load32(block + q_offset + i0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int low_quant = static_cast<int>((byte_of(q, i) >> shift) & 3u);
        const int high_quant = (byte_of(hm, i) & mask) == 0 ? 4 : 0;
        out[i] = dl * static_cast<float>(low_quant - high_quant);
    }
}

template <>
__device__ __forceinline__ void decode4<kQ4_K>(const uint8_t* block, uint32_t e, float out[4]) {
    const uint32_t group = e >> 5, i0 = e & 31u;
    const uint32_t pair = group >> 1, side = group & 1u;
    uint32_t scale, min;
    scale_min_k4(group, block + 4, scale, min);
    const float d = f16_at(block, 0), dmin = f16_at(block, 2);
    const float dl = d * static_cast<float>(scale);
    const float ml = dmin * static_cast<float>(min);
    const uint32_t q = load32(block + 16 + pair * 32 + i0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t byte = byte_of(q, i);
        const uint32_t quant = side == 0 ? (byte & 0x0fu) : (byte >> 4);
        const float prod = dl * static_cast<float>(quant);
        out[i] = prod - ml;
    }
}

template <>
__device__ __forceinline__ void decode4<kQ5_K>(const uint8_t* block, uint32_t e, float out[4]) {
    const uint32_t group = e >> 5, i0 = e & 31u;
    const uint32_t pair = group >> 1, side = group & 1u;
    uint32_t scale, min;
    scale_min_k4(group, block + 4, scale, min);
    const float d = f16_at(block, 0), dmin = f16_at(block, 2);
    const float dl = d * static_cast<float>(scale);
    const float ml = dmin * static_cast<float>(min);
    const uint32_t high = load32(block + 16 + i0);
    const uint32_t ql = load32(block + 48 + pair * 32 + i0);
    const uint32_t mask = 1u << group;  // 1 << (pair*2 + side)
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t byte = byte_of(ql, i);
        const uint32_t low_quant = side == 0 ? (byte & 0x0fu) : (byte >> 4);
        const uint32_t quant = low_quant + ((byte_of(high, i) & mask) == 0 ? 0u : 16u);
        const float prod = dl * static_cast<float>(quant);
        out[i] = prod - ml;
    }
}

template <>
__device__ __forceinline__ void decode4<kQ6_K>(const uint8_t* block, uint32_t e, float out[4]) {
    // e = half*128 + quarter*32 + index
    const uint32_t half = e >> 7, quarter = (e >> 5) & 3u, i0 = e & 31u;
    const uint32_t ql = load32(block + half * 64 + i0 + ((quarter & 1u) ? 32u : 0u));
    const uint32_t qh = load32(block + 128 + half * 32 + i0);
    const uint32_t scale_index = half * 8u + (i0 >> 4) + quarter * 2u;
    const int scale = static_cast<int8_t>(block[192 + scale_index]);
    const float d = f16_at(block, 208);
    const float ds = d * static_cast<float>(scale);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = byte_of(ql, i);
        const uint32_t nib = (quarter & 2u) ? (lo >> 4) : (lo & 0x0fu);
        const uint32_t hi2 = (byte_of(qh, i) >> (2u * quarter)) & 3u;
        const int quant = static_cast<int>(nib | (hi2 << 4)) - 32;
        out[i] = ds * static_cast<float>(quant);
    }
}

}  // namespace et
