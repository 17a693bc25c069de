// Device helpers shared by the dequant-GEMV kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace et {

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
    union {
        uint16_t u;
        _Float16 h;
    } cvt;
    cvt.u = static_cast<uint16_t>(bits);
    return static_cast<float>(cvt.h);
}

// Sum over the 64 lanes of a wave, returned in every lane.
// Four DPP steps fold each 16-lane row (quad swaps, half-row mirror, row
// mirror); the four row totals are then read as scalars and added in a fixed
// order, so the result does not depend on which lane asks.
__device__ __forceinline__ float wave_sum(float v) {
    int t;
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true);  // row_half_mirror
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true);  // row_mirror
    v += __int_as_float(t);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// LDS slot of the f-th float4 of an activation vector. XOR-ing the low three
// bits with bits 4..6 keeps both access patterns conflict-free: the staging
// writes (consecutive lanes -> consecutive f) and the per-lane reads (lane l
// reads f = 16*l + j or 8*l + j for a fixed j).
__device__ __forceinline__ uint32_t x_slot(uint32_t f) { return f ^ ((f >> 4) & 7u); }

// Stages `vectors` activation rows of `columns` floats into LDS (swizzled).
template <int THREADS>
__device__ __forceinline__ void stage_x(float4* lds, const float* __restrict__ x,
                                        uint64_t x_row_stride, uint32_t columns, int vectors) {
    const uint32_t quads = columns >> 2;
    for (int m = 0; m < vectors; m++) {
        const float4* src = reinterpret_cast<const float4*>(x + m * x_row_stride);
        for (uint32_t f = threadIdx.x; f < quads; f += THREADS) lds[m * quads + x_slot(f)] = src[f];
    }
}

}  // namespace et
