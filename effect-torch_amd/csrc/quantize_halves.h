// The quantiser of gemm_h16's activation tiles for one (vector, 256-column stage), shared by the
// kernels that write such tiles: quantize_act.hip and the epilogue of kv_attention.hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"

namespace et {

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// Activations for gemm_h16: per vector and 256-column stage, X = clamp(rint(x * (2^23 - 1) / amax))
// as two balanced 12-bit halves, X = 4096 * hi + lo with lo in [-2048, 2047], written as the half floats
// hi and lo / 4096 (both exact: integers below 2^11 and a power of two), so that the two products of a
// weight with them add up to X * w / 4096 in one accumulator; unit = amax / (2^23 - 1); xsum[g] = unit * (integer sum of X over sub-block g).
// One wave per (vector, stage): lane `quad` holds columns 4 quad .. 4 quad + 3 of the stage. Blob
// layout: see tile_blob_bytes() in kernels.h.
__device__ __forceinline__ void quantize_halves_store(const float4& in, uint32_t v, uint32_t stage, uint32_t quad,
                                                      uint32_t vector_tiles, uint8_t* __restrict__ tiles) {
#pragma clang fp contract(off)  // the same bits in every file that includes this
    constexpr float kRange = 8388607.f;  // 2^23 - 1
    float amax = fmaxf(fmaxf(fabsf(in.x), fabsf(in.y)), fmaxf(fabsf(in.z), fabsf(in.w)));
    // over the wave: inside rows of 16 lanes with DPP, then the four rows through scalar registers
    amax = fmaxf(amax, dpp_f32<0xB1>(amax));   // quad_perm [1,0,3,2]
    amax = fmaxf(amax, dpp_f32<0x4E>(amax));   // quad_perm [2,3,0,1]
    amax = fmaxf(amax, dpp_f32<0x141>(amax));  // row_half_mirror
    amax = fmaxf(amax, dpp_f32<0x140>(amax));  // row_mirror
    {
        const int bits = __float_as_int(amax);
        amax = fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(bits, 0)),
                           __int_as_float(__builtin_amdgcn_readlane(bits, 16))),
                     fmaxf(__int_as_float(__builtin_amdgcn_readlane(bits, 32)),
                           __int_as_float(__builtin_amdgcn_readlane(bits, 48))));
    }
    const float inv = amax > 0.f ? kRange / amax : 0.f;
    const float values[4] = {in.x, in.y, in.z, in.w};
    int total = 0;
    union {
        _Float16 h[4];
        uint2 words;
    } low, high;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float r = fminf(fmaxf(rintf(values[i] * inv), -kRange), kRange);
        const int q = static_cast<int>(r);
        const int lo = ((q + 2048) & 4095) - 2048;
        total += q;
        low.h[i] = static_cast<_Float16>(static_cast<float>(lo) * (1.0f / 4096.0f));
        high.h[i] = static_cast<_Float16>((q - lo) >> 12);  // exact: q - lo is a multiple of 4096
    }
    total += dpp_i32<0xB1>(total);   // the eight lanes of a 32-column sub-block
    total += dpp_i32<0x4E>(total);
    total += dpp_i32<0x141>(total);
    const float unit = amax / kRange;
    uint8_t* blob = tiles + (static_cast<uint64_t>(stage) * vector_tiles + (v >> 5)) * tile_blob_bytes(2);
    // columns 4 quad .. + 3 = sub-block quad / 8, 16-column half, 8-column part, first or second four
    const uint32_t at = (quad >> 1) * 512u + (v & 31u) * 16u + (quad & 1u) * 8u;
    *reinterpret_cast<uint2*>(blob + at) = low.words;
    *reinterpret_cast<uint2*>(blob + 16384u + at) = high.words;
    float* tables = reinterpret_cast<float*>(blob + 32768u);
    if (quad == 0) tables[v & 31u] = unit;
    if ((quad & 7u) == 0) tables[32u + (quad >> 3) * 32u + (v & 31u)] = unit * static_cast<float>(total);
}

}  // namespace et
