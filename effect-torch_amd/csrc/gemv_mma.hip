// Dequant-GEMV for a few activation vectors (2..8) on the int8 matrix cores of gfx950 (Q4_K, Q5_K, Q4_0, Q8_0):
//     y[v, r] = sum_k x[v, k] * decode(W[r])[k] (+ bias[r])
//
// Same contraction as linear_into (crates/runtime-cpu/src/quantized.rs:419-499) with decode_q4_k
// (:180-199) and decode_q5_k (:203-234) in factored form; Q4_0 and Q8_0 follow the public ggml block layouts. The reference's own GPU
// backend keeps 2..8 vectors in its GEMV family (crates/runtime-metal/src/quantized.rs:1204-1220).
// f32-accurate (23-bit fixed-point activations per 256 columns, exact integer dots).
//
// The kernel is HBM-bound and streams W exactly once, whatever the number of vectors. What a few
// vectors cost on v_dot4 (gemv_limb.hip: 48 dots per vector, row and lane) is here one matrix
// instruction per 32-column block and sixteen rows: v_mfma_i32_16x16x32_i8 with the weights' quants
// as its B operand (sixteen rows of W) and, as its A operand, the three signed-byte limbs of four
// activation vectors in rows 4v + limb (row 4v + 3 is zero). A lane of the result then holds, for its
// weight row and its vector, the three limb dots of the block side by side.
//
// Work split. A workgroup owns a contiguous range of rows (one per compute unit when the matrix
// fits). LOADER waves copy that range into LDS as it lies in memory, with 1 KiB global-to-LDS copies
// taken in turn, a few in flight per wave, and publish how many have landed. Eight CONSUMER waves
// each own one eighth of the columns (two 256-column units at 4096 columns): a consumer quantises its
// own slice of the activation vectors once, keeps the A operands of all its blocks in registers for
// its whole life and walks the rows in groups of sixteen as they land; the eight partial sums of a
// group meet in LDS and the consumer that arrives last adds them in wave order (the same bits on
// every run) and stores y.
//
// LDS image of the weights: rows `pitch` bytes apart, pitch = row bytes + the padding that makes it
// 16 (mod 256), so that the sixteen rows a matrix instruction reads at one column offset lie in
// sixteen different groups of four banks. A copy instruction writes 1 KiB of the image; the lanes
// whose 16 bytes are padding are switched off.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"
#include "lds_handover.h"

namespace et {
namespace {

constexpr int kConsumers = 8;
constexpr uint32_t kLdsBytes = 160u * 1024u;
constexpr uint32_t kGroupRows = 16u;    // rows of W per matrix instruction
// Activations as fixed point: X = rint(x * kLimbRange / max|x|), |X| < 2^22. Adding kLimbMagic to the
// scaled value makes the float's mantissa the integer X + 0x408080 (the sum lies in [2^23, 2^24), where
// floats are the integers): one fused multiply-add quantises, rounds to nearest even and offsets.
constexpr float kLimbRange = 4161000.0f;                // X + 0x8080 stays below 2^22 with room for the reciprocal's ulp
constexpr float kLimbMagic = 12582912.0f + 32896.0f;    // 1.5 * 2^23 + 0x8080

constexpr uint32_t kMostGroups = 4u;    // groups of a range: its rows' partial sums wait in LDS for the end

// Per consumer wave: [limb planes of one vector, 544 bytes apart][sums per vector and 32 columns]
// [units per vector and 256 columns]. Once the A operands are in registers the first part holds the
// wave's partial sums: [group][vector group][lane].
constexpr uint32_t kLimbPitch = 544u;  // 512 bytes of a limb plane + 32: the three planes start in different banks
constexpr uint32_t kSumsAt = 2048u, kUnitsAt = 2560u, kWaveScratch = 2624u;
static_assert(3u * kLimbPitch <= kSumsAt && kMostGroups * 2u * 256u <= kSumsAt, "planes and partial sums share the first part");
struct Control {
    uint32_t landed[8];  // copies of loader w that have landed
    uint32_t summed;     // consumers that have left the partial sums of all their groups
    uint32_t pad[7];
};
static_assert(sizeof(Control) == 64, "sixteen words, zeroed by sixteen lanes");
constexpr uint32_t kControlAt = kLdsBytes - 64u;
constexpr uint32_t kScratchAt = kControlAt - kConsumers * kWaveScratch;  // the image ends below this

__host__ __device__ constexpr uint32_t image_pitch(uint32_t row_bytes) {
    return row_bytes + ((16u - (row_bytes & 255u)) & 255u);
}

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

typedef int v4i __attribute__((ext_vector_type(4)));

#ifdef ET_MMA_PROBES
// timing experiments only: [workgroup][wave][slot] wall-clock stamps (100 MHz)
__device__ uint64_t mma_stamps[1024 * 16 * 16];
#define ET_STAMP(slot)                                                                                          \
    do {                                                                                                        \
        if (PROBE == 4 && lane_id == 0 && blockIdx.x < 1024)                                                    \
            mma_stamps[(blockIdx.x * 16 + wave) * 16 + (slot)] = wall_clock64();                                \
    } while (0)
#else
#define ET_STAMP(slot) do {} while (0)
#endif

__device__ __forceinline__ long pack(uint32_t low, uint32_t high) {
    return static_cast<long>((static_cast<uint64_t>(high) << 32) | low);
}

// 4x3 byte transpose: limb k of four 23-bit values X + 0x408080 (the low three bytes of the words) into
// one dword each. With X = 65536 l2 + 256 l1 + l0 in balanced digits (l0, l1 in [-128, 127], l2 in
// [-64, 63]) the bytes are l0 + 128, l1 + 128 and l2 + 64: flipping the top bit gives the signed limb,
// for the third after another 64 (no byte carries: it is below 128).
__device__ __forceinline__ void split_quad(int x0, int x1, int x2, int x3, uint32_t (&limb)[3]) {
    const uint32_t a = __builtin_amdgcn_perm(x1, x0, 0x05010400u);  // x0.b0 x1.b0 x0.b1 x1.b1
    const uint32_t b = __builtin_amdgcn_perm(x3, x2, 0x05010400u);
    const uint32_t c = __builtin_amdgcn_perm(x1, x0, 0x0c0c0602u);  // x0.b2 x1.b2 0 0
    const uint32_t d = __builtin_amdgcn_perm(x3, x2, 0x0c0c0602u);
    limb[0] = __builtin_amdgcn_perm(b, a, 0x05040100u) ^ 0x80808080u;
    limb[1] = __builtin_amdgcn_perm(b, a, 0x07060302u) ^ 0x80808080u;
    limb[2] = (__builtin_amdgcn_perm(d, c, 0x05040100u) + 0x40404040u) ^ 0x80808080u;
}

// ---------------------------------------------------------------------------
// Codec traits: one 256-column unit (kUnitBytes) of sixteen rows against the A operands.
//   rp     the unit in the lane's row of the LDS image
//   q      the lane's K index: which 8 of a block's 32 columns its operand registers hold
//   a      A operands of the wave's sixteen 32-column blocks, per group of four vectors
//   sums   f32 sums of the lane's vector over the unit's eight blocks (next vector group: + 64 floats)
//   units  value of one unit of limb 0 of the lane's vector in this unit (next vector group: + 8 floats)
// ---------------------------------------------------------------------------
struct Q4KMma {
    static constexpr uint32_t kUnitBytes = 144u;  // one super-block
    static __device__ __forceinline__ uint32_t chunk(uint32_t q) { return q; }
    template <int VG, int UNIT>
    static __device__ __forceinline__ void contract(const uint8_t* rp, uint32_t q, const long (&a)[VG][16],
                                                    const float* sums, const float* units, float (&total)[VG]) {
        const uint4 h = *reinterpret_cast<const uint4*>(rp);
        const float d = half_bits_to_float(h.x & 0xffffu), dmin = half_bits_to_float(h.x >> 16);
        // (scale, min) of the eight sub-blocks, a byte each: crates/runtime-cpu/src/quantized.rs:77-86
        const uint32_t sc[2] = {h.y & 0x3f3f3f3fu, (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u)};
        uint32_t mn[2] = {h.z & 0x3f3f3f3fu, ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u)};
        // keeps the minima packed, a byte-to-float conversion each, instead of a mask per byte
        asm volatile("" : "+v"(mn[0]), "+v"(mn[1]));
        int acc[VG][3];
#pragma unroll
        for (int g = 0; g < VG; g++) acc[g][0] = acc[g][1] = acc[g][2] = 0;
        const v4i zero = {0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            // bytes 8q..8q+7 of the pair: low nibbles = columns 8q.. of sub-block 2p, high = of 2p + 1
            const uint2 w = *reinterpret_cast<const uint2*>(rp + 16 + 32 * p + 8 * q);
            const long lo = pack(w.x & 0x0f0f0f0fu, w.y & 0x0f0f0f0fu);
            const long hi = pack((w.x >> 4) & 0x0f0f0f0fu, (w.y >> 4) & 0x0f0f0f0fu);
            const int s_lo = static_cast<int>((sc[p >> 1] >> (16 * (p & 1))) & 0xffu);
            const int s_hi = static_cast<int>((sc[p >> 1] >> (16 * (p & 1) + 8)) & 0xffu);
#pragma unroll
            for (int g = 0; g < VG; g++) {
                const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * p], lo, zero, 0, 0, 0);
                const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * p + 1], hi, zero, 0, 0, 0);
                // block dots are below 2^17, scales below 2^6: 24-bit multiplies, exact int32 sums
#pragma unroll
                for (int k = 0; k < 3; k++) acc[g][k] += __mul24(c0[k], s_lo) + __mul24(c1[k], s_hi);
            }
        }
        // (the compiler turns these into v_cvt_f32_ubyte0..3)
        const float m0 = static_cast<float>(mn[0] & 0xffu), m1 = static_cast<float>((mn[0] >> 8) & 0xffu);
        const float m2 = static_cast<float>((mn[0] >> 16) & 0xffu), m3 = static_cast<float>(mn[0] >> 24);
        const float m4 = static_cast<float>(mn[1] & 0xffu), m5 = static_cast<float>((mn[1] >> 8) & 0xffu);
        const float m6 = static_cast<float>((mn[1] >> 16) & 0xffu), m7 = static_cast<float>(mn[1] >> 24);
#pragma unroll
        for (int g = 0; g < VG; g++) {
            const float4 s0 = *reinterpret_cast<const float4*>(sums + 64 * g);
            const float4 s1 = *reinterpret_cast<const float4*>(sums + 64 * g + 4);
            float neg = m0 * s0.x;
            neg = fmaf(m1, s0.y, neg);
            neg = fmaf(m2, s0.z, neg);
            neg = fmaf(m3, s0.w, neg);
            neg = fmaf(m4, s1.x, neg);
            neg = fmaf(m5, s1.y, neg);
            neg = fmaf(m6, s1.z, neg);
            neg = fmaf(m7, s1.w, neg);
            float f = static_cast<float>(acc[g][0]);
            f = fmaf(256.0f, static_cast<float>(acc[g][1]), f);
            f = fmaf(65536.0f, static_cast<float>(acc[g][2]), f);
            total[g] += d * (units[8 * g] * f) - dmin * neg;
        }
    }
};

// Q4_0: a unit is four pairs of 18-byte blocks, 36 bytes = 9 dwords each. Block: half-float d, then
// sixteen bytes whose low nibbles are columns 0..15 and whose high nibbles are columns 16..31. The
// lanes with K index q take bytes 8 * (q >> 1) .. + 7, low (q even) or high nibbles: columns
// 16 * (q & 1) + 8 * (q >> 1) .. + 7. value = d * (nibble - 8): the - 8 meets the f32 sums of the
// activations once per block.
struct Q40Mma {
    static constexpr uint32_t kUnitBytes = 144u;  // eight blocks of 18 bytes
    static __device__ __forceinline__ uint32_t chunk(uint32_t q) { return ((q & 1u) << 1) | (q >> 1); }
    template <int VG, int UNIT>
    static __device__ __forceinline__ void contract(const uint8_t* rp, uint32_t q, const long (&a)[VG][16],
                                                    const float* sums, const float* units, float (&total)[VG]) {
        const uint32_t half = q >> 1, shift = (q & 1u) * 4u;
        float pos[VG], corr[VG], s[VG][8];
#pragma unroll
        for (int g = 0; g < VG; g++) {
            pos[g] = corr[g] = 0.f;
            const float4 s0 = *reinterpret_cast<const float4*>(sums + 64 * g);
            const float4 s1 = *reinterpret_cast<const float4*>(sums + 64 * g + 4);
            s[g][0] = s0.x, s[g][1] = s0.y, s[g][2] = s0.z, s[g][3] = s0.w;
            s[g][4] = s1.x, s[g][5] = s1.y, s[g][6] = s1.z, s[g][7] = s1.w;
        }
        const v4i zero = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t* pair = reinterpret_cast<const uint32_t*>(rp + 36 * c);
            const uint32_t* mine = pair + 2 * half;
            // even block: quants at bytes 2..17 of the pair (2 bytes off dword alignment); odd: 20..35
            const uint32_t e0 = mine[0], e1 = mine[1], e2 = mine[2], o0 = mine[5], o1 = mine[6];
            const uint32_t qa0 = __builtin_amdgcn_alignbit(e1, e0, 16), qa1 = __builtin_amdgcn_alignbit(e2, e1, 16);
            const long even = pack((qa0 >> shift) & 0x0f0f0f0fu, (qa1 >> shift) & 0x0f0f0f0fu);
            const long odd = pack((o0 >> shift) & 0x0f0f0f0fu, (o1 >> shift) & 0x0f0f0f0fu);
            const float da = half_bits_to_float(pair[0] & 0xffffu), db = half_bits_to_float(pair[4] >> 16);
#pragma unroll
            for (int g = 0; g < VG; g++) {
                const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * c], even, zero, 0, 0, 0);
                const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * c + 1], odd, zero, 0, 0, 0);
                float f0 = static_cast<float>(c0[0]);
                f0 = fmaf(256.0f, static_cast<float>(c0[1]), f0);
                f0 = fmaf(65536.0f, static_cast<float>(c0[2]), f0);
                float f1 = static_cast<float>(c1[0]);
                f1 = fmaf(256.0f, static_cast<float>(c1[1]), f1);
                f1 = fmaf(65536.0f, static_cast<float>(c1[2]), f1);
                pos[g] = fmaf(db, f1, fmaf(da, f0, pos[g]));
                corr[g] = fmaf(db, s[g][2 * c + 1], fmaf(da, s[g][2 * c], corr[g]));
            }
        }
#pragma unroll
        for (int g = 0; g < VG; g++) total[g] += units[8 * g] * pos[g] - 8.0f * corr[g];
    }
};

// Q5_K (decode_q5_k, crates/runtime-cpu/src/quantized.rs:203-234): Q4_K's layout with a fifth bit per
// value in qh[32] between the scales and the nibbles - bit g of qh[i] belongs to column i of sub-block g.
struct Q5KMma {
    static constexpr uint32_t kUnitBytes = 176u;
    static __device__ __forceinline__ uint32_t chunk(uint32_t q) { return q; }
    template <int VG, int UNIT>
    static __device__ __forceinline__ void contract(const uint8_t* rp, uint32_t q, const long (&a)[VG][16],
                                                    const float* sums, const float* units, float (&total)[VG]) {
        const uint4 h = *reinterpret_cast<const uint4*>(rp);
        const float d = half_bits_to_float(h.x & 0xffffu), dmin = half_bits_to_float(h.x >> 16);
        const uint32_t sc[2] = {h.y & 0x3f3f3f3fu, (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u)};
        uint32_t mn[2] = {h.z & 0x3f3f3f3fu, ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u)};
        asm volatile("" : "+v"(mn[0]), "+v"(mn[1]));
        const uint2 fifth = *reinterpret_cast<const uint2*>(rp + 16 + 8 * q);  // columns 8q..8q+7, all sub-blocks
        int acc[VG][3];
#pragma unroll
        for (int g = 0; g < VG; g++) acc[g][0] = acc[g][1] = acc[g][2] = 0;
        const v4i zero = {0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint2 w = *reinterpret_cast<const uint2*>(rp + 48 + 32 * p + 8 * q);
            const uint32_t fx = fifth.x >> (2 * p), fy = fifth.y >> (2 * p);
            const long lo = pack((w.x & 0x0f0f0f0fu) | ((fx & 0x01010101u) << 4), (w.y & 0x0f0f0f0fu) | ((fy & 0x01010101u) << 4));
            const long hi = pack(((w.x >> 4) & 0x0f0f0f0fu) | ((fx & 0x02020202u) << 3),
                                 ((w.y >> 4) & 0x0f0f0f0fu) | ((fy & 0x02020202u) << 3));
            const int s_lo = static_cast<int>((sc[p >> 1] >> (16 * (p & 1))) & 0xffu);
            const int s_hi = static_cast<int>((sc[p >> 1] >> (16 * (p & 1) + 8)) & 0xffu);
#pragma unroll
            for (int g = 0; g < VG; g++) {
                const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * p], lo, zero, 0, 0, 0);
                const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * p + 1], hi, zero, 0, 0, 0);
                // block dots are below 2^18, scales below 2^6
#pragma unroll
                for (int k = 0; k < 3; k++) acc[g][k] += __mul24(c0[k], s_lo) + __mul24(c1[k], s_hi);
            }
        }
        const float m0 = static_cast<float>(mn[0] & 0xffu), m1 = static_cast<float>((mn[0] >> 8) & 0xffu);
        const float m2 = static_cast<float>((mn[0] >> 16) & 0xffu), m3 = static_cast<float>(mn[0] >> 24);
        const float m4 = static_cast<float>(mn[1] & 0xffu), m5 = static_cast<float>((mn[1] >> 8) & 0xffu);
        const float m6 = static_cast<float>((mn[1] >> 16) & 0xffu), m7 = static_cast<float>(mn[1] >> 24);
#pragma unroll
        for (int g = 0; g < VG; g++) {
            const float4 s0 = *reinterpret_cast<const float4*>(sums + 64 * g);
            const float4 s1 = *reinterpret_cast<const float4*>(sums + 64 * g + 4);
            float neg = m0 * s0.x;
            neg = fmaf(m1, s0.y, neg);
            neg = fmaf(m2, s0.z, neg);
            neg = fmaf(m3, s0.w, neg);
            neg = fmaf(m4, s1.x, neg);
            neg = fmaf(m5, s1.y, neg);
            neg = fmaf(m6, s1.z, neg);
            neg = fmaf(m7, s1.w, neg);
            float f = static_cast<float>(acc[g][0]);
            f = fmaf(256.0f, static_cast<float>(acc[g][1]), f);
            f = fmaf(65536.0f, static_cast<float>(acc[g][2]), f);
            total[g] += d * (units[8 * g] * f) - dmin * neg;
        }
    }
};

// Q8_0: a unit is four pairs of 34-byte blocks, 68 bytes = 17 dwords each. Block: half-float d, then
// 32 signed bytes. The lanes with K index q take columns 8q..8q+7.
struct Q80Mma {
    static constexpr uint32_t kUnitBytes = 272u;
    static __device__ __forceinline__ uint32_t chunk(uint32_t q) { return q; }
    template <int VG, int UNIT>
    static __device__ __forceinline__ void contract(const uint8_t* rp, uint32_t q, const long (&a)[VG][16],
                                                    const float*, const float* units, float (&total)[VG]) {
        float pos[VG];
#pragma unroll
        for (int g = 0; g < VG; g++) pos[g] = 0.f;
        const v4i zero = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t* pair = reinterpret_cast<const uint32_t*>(rp + 68 * c);
            const uint32_t* mine = pair + 2 * q;
            // even block: quants at bytes 2..33 of the pair (2 bytes off dword alignment); odd: 36..67
            const uint32_t e0 = mine[0], e1 = mine[1], e2 = mine[2], o0 = mine[9], o1 = mine[10];
            const long even = pack(__builtin_amdgcn_alignbit(e1, e0, 16), __builtin_amdgcn_alignbit(e2, e1, 16));
            const long odd = pack(o0, o1);
            const float da = half_bits_to_float(pair[0] & 0xffffu), db = half_bits_to_float(pair[8] >> 16);
#pragma unroll
            for (int g = 0; g < VG; g++) {
                const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * c], even, zero, 0, 0, 0);
                const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[g][UNIT * 8 + 2 * c + 1], odd, zero, 0, 0, 0);
                float f0 = static_cast<float>(c0[0]);
                f0 = fmaf(256.0f, static_cast<float>(c0[1]), f0);
                f0 = fmaf(65536.0f, static_cast<float>(c0[2]), f0);
                float f1 = static_cast<float>(c1[0]);
                f1 = fmaf(256.0f, static_cast<float>(c1[1]), f1);
                f1 = fmaf(65536.0f, static_cast<float>(c1[2]), f1);
                pos[g] = fmaf(db, f1, fmaf(da, f0, pos[g]));
            }
        }
#pragma unroll
        for (int g = 0; g < VG; g++) total[g] += units[8 * g] * pos[g];
    }
};

template <class T, int VG, int LOADERS, int DEPTH, int PROBE = 0>
__global__ __launch_bounds__(64 * (kConsumers + LOADERS)) void gemv_mma_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns, uint32_t rows_per_wg,
    uint32_t vectors, uint32_t spin_limit, uint32_t* timeouts) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    static_assert(DEPTH >= 1 && DEPTH <= 8 && LOADERS >= 1 && LOADERS <= 8, "wait_copies_in_flight counts to seven");
    constexpr int VEC = 4 * VG;
    Control* control = reinterpret_cast<Control*>(lds + kControlAt);

    const uint32_t lane_id = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wg_row0 = blockIdx.x * rows_per_wg;
    if (wg_row0 >= rows) return;
    ET_STAMP(0);
    const uint32_t wg_rows = min(rows_per_wg, rows - wg_row0);
    const uint32_t row_units = columns >> 8;
    const uint32_t row_bytes = row_units * T::kUnitBytes;
    const uint32_t pitch = image_pitch(row_bytes);
    const uint32_t image_bytes = (wg_rows - 1u) * pitch + row_bytes;  // ends with the last row's last byte

    if (wave >= static_cast<uint32_t>(kConsumers)) {
        // ---- loaders ----------------------------------------------------------------------------
        const uint32_t loader = wave - kConsumers;
        const uint32_t copies = (image_bytes + 1023u) >> 10;
        const uint32_t mine = copies > loader ? (copies - loader + LOADERS - 1u) / LOADERS : 0u;
        // where this lane's 16 bytes of the wave's next copy lie in the image, and in W (from the range's first byte)
        uint32_t at = loader * 1024u + lane_id * 16u;
        uint32_t row = at / pitch, column = at - row * pitch;
        uint32_t from = row * row_bytes + column;
        constexpr uint32_t kStep = LOADERS * 1024u;  // between two copies of a wave
        const uint32_t step_rows = kStep / pitch, step_columns = kStep - step_rows * pitch;
        const uint32_t step_from = step_rows * row_bytes + step_columns;
        const uint32_t end = wg_rows * row_bytes;  // rows past the range start there
        const uint8_t* source = weight + static_cast<uint64_t>(wg_row0) * row_bytes;
        const uint32_t landed_address = lds_address(&control->landed[loader]);
        uint32_t next = loader;  // number of the wave's next copy
        const auto copy = [&]() {
            // never a copy without a lane: the image ends with bytes of W and padding is shorter than a copy
            if (PROBE != 2 && PROBE != 3 && column < row_bytes && from < end)
                // streamed once: non-temporal (aux bit 1), the caches keep nothing of it
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(source + from),
                                                 reinterpret_cast<uint4*>(lds + next * 1024u), 16, 0, 2);
            next += LOADERS;
            column += step_columns;
            from += step_from;
            if (column >= pitch) {  // into the next row: its padding is not in W
                column -= pitch;
                from += row_bytes - pitch;
            }
        };
        // The first copies wait for the barrier, i.e. until the consumers have issued their activation
        // loads: issued ahead of it they delay those loads, and with them everything else.
        // (measured: issued ahead of the barrier, 0.9 to 1.5 us per launch slower)
        __syncthreads();
        ET_STAMP(1);
        const uint32_t head = min(mine, static_cast<uint32_t>(DEPTH));
        for (uint32_t i = 0; i < head; i++) copy();
        ET_STAMP(2);
        uint32_t landed = 0;
        for (uint32_t i = head; i < mine; i++) {  // only with DEPTH copies in flight
            // the oldest copy in flight has landed: say so, then take its place in the queue
            __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH - 1));
            lds_store_unseen(landed_address, ++landed);
            if (landed == 1u) ET_STAMP(3);
            copy();
        }
        ET_STAMP(4);
        for (uint32_t left = head; left > 0u; left--) {
            wait_copies_in_flight(left - 1u);
            lds_store_unseen(landed_address, ++landed);
        }
        ET_STAMP(5);
        return;
    }

    // ---- consumers --------------------------------------------------------------------------------
    Patience patience{spin_limit, timeouts};
    const uint32_t first_unit = 2u * wave;  // the wave's columns: units first_unit, first_unit + 1
    const uint32_t my_units = row_units > first_unit ? min(2u, row_units - first_unit) : 0u;
    uint8_t* scratch = lds + kScratchAt + wave * kWaveScratch;
    float* sums = reinterpret_cast<float*>(scratch + kSumsAt);    // [vector][block of the slice]
    float* units = reinterpret_cast<float*>(scratch + kUnitsAt);  // [vector][unit of the slice]

    // Activation loads first: nothing of the consumers' may queue behind a copy. Lane j holds columns
    // 8j .. 8j+7 of the slice: chunk j % 4 of block j / 4.
    float4 xv[VEC][2];
    {
        const uint32_t column = first_unit * 256u + lane_id * 8u;
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            xv[v][0] = xv[v][1] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (static_cast<uint32_t>(v) < vectors && column < columns) {
                const float4* p = reinterpret_cast<const float4*>(x + v * x_row_stride + column);
                xv[v][0] = p[0];
                xv[v][1] = p[1];
            }
        }
    }
    if (threadIdx.x < 16) reinterpret_cast<uint32_t*>(control)[threadIdx.x] = 0u;
    __syncthreads();  // the only barrier: the counters are zero before anybody counts
    ET_STAMP(1);

    // 23-bit fixed point per vector and 256-column unit, X = rint(x * kLimbRange / max|x|), in three
    // balanced signed-byte limbs; the limbs go through the wave's scratch into the lanes that hold
    // them as A operands: lane l, as row l % 16 = 4 * vector + limb, K index l / 16.
    long a[VG][16];
#pragma unroll
    for (int g = 0; g < VG; g++)
#pragma unroll
        for (int s = 0; s < 16; s++) a[g][s] = 0;
#pragma unroll
    for (int v = 0; v < VEC; v++) {
        if (static_cast<uint32_t>(v) >= vectors) break;
        const float4 f0 = xv[v][0], f1 = xv[v][1];
        float amax = fmaxf(fmaxf(fabsf(f0.x), fabsf(f0.y)), fabsf(f0.z));  // three-input maxima
        amax = fmaxf(fmaxf(amax, fabsf(f0.w)), fabsf(f1.x));
        amax = fmaxf(fmaxf(amax, fabsf(f1.y)), fabsf(f1.z));
        amax = fmaxf(amax, fabsf(f1.w));
        amax = fmaxf(amax, dpp<0xB1>(amax));   // quad_perm [1,0,3,2]
        amax = fmaxf(amax, dpp<0x4E>(amax));   // quad_perm [2,3,0,1]
        amax = fmaxf(amax, dpp<0x141>(amax));  // row_half_mirror
        amax = fmaxf(amax, dpp<0x140>(amax));  // row_mirror: sixteen lanes = 128 columns
        amax = fmaxf(amax, __shfl_xor(amax, 16));  // the unit's 256 columns
        float total = ((f0.x + f0.y) + (f0.z + f0.w)) + ((f1.x + f1.y) + (f1.z + f1.w));
        total += dpp<0xB1>(total);
        total += dpp<0x4E>(total);  // the block's 32 columns
        // 1 ulp of the reciprocal moves |X| by at most 1, far inside the headroom of the range.
        const bool nonzero = amax >= 1e-30f;
        const float inv = nonzero ? kLimbRange * __builtin_amdgcn_rcpf(amax) : 0.f;
        const float unit = nonzero ? amax * (1.0f / kLimbRange) : 0.f;
        uint32_t low[3], high[3];
        split_quad(__float_as_int(fmaf(f0.x, inv, kLimbMagic)), __float_as_int(fmaf(f0.y, inv, kLimbMagic)),
                   __float_as_int(fmaf(f0.z, inv, kLimbMagic)), __float_as_int(fmaf(f0.w, inv, kLimbMagic)), low);
        split_quad(__float_as_int(fmaf(f1.x, inv, kLimbMagic)), __float_as_int(fmaf(f1.y, inv, kLimbMagic)),
                   __float_as_int(fmaf(f1.z, inv, kLimbMagic)), __float_as_int(fmaf(f1.w, inv, kLimbMagic)), high);
        asm volatile("" ::: "memory");  // the reads of the vector before are done with the planes
#pragma unroll
        for (int k = 0; k < 3; k++)
            *reinterpret_cast<uint2*>(scratch + k * kLimbPitch + lane_id * 8u) = make_uint2(low[k], high[k]);
        if ((lane_id & 3u) == 0u) sums[v * 16 + (lane_id >> 2)] = total;
        if ((lane_id & 31u) == 0u) units[v * 2 + (lane_id >> 5)] = unit;
        asm volatile("" ::: "memory");  // LDS serves a wave in order: written above, read below
        if (((lane_id & 15u) >> 2) == static_cast<uint32_t>(v & 3) && (lane_id & 3u) != 3u) {
            const uint8_t* plane = scratch + (lane_id & 3u) * kLimbPitch + T::chunk(lane_id >> 4) * 8u;
#pragma unroll
            for (int s = 0; s < 16; s++) {
                const uint2 w = *reinterpret_cast<const uint2*>(plane + s * 32);
                a[v >> 2][s] = pack(w.x, w.y);
            }
        }
    }
    asm volatile("" ::: "memory");
    ET_STAMP(2);

    const uint32_t n = lane_id & 15u, q = lane_id >> 4;
    const uint32_t groups = (wg_rows + kGroupRows - 1u) / kGroupRows;
    float* partial = reinterpret_cast<float*>(scratch);  // [group][vector group][lane]
    for (uint32_t group = 0; group < groups; group++) {
        const uint32_t last_row = min(group * kGroupRows + kGroupRows, wg_rows) - 1u;
        const bool landed = await_copies_in_turn<LOADERS>(control->landed, lane_id, (last_row * pitch + row_bytes + 1023u) >> 10, patience);
        ET_STAMP(3 + 3 * group);
        float total[VG];
#pragma unroll
        for (int g = 0; g < VG; g++) total[g] = 0.f;
        if (PROBE != 1 && PROBE != 3 && landed && my_units != 0u) {
            // rows past the end of the range read its last row again and are not stored
            const uint8_t* rp = lds + min(group * kGroupRows + n, wg_rows - 1u) * pitch + first_unit * T::kUnitBytes;
            if (my_units > 1u) {  // both in one block: the second unit's LDS reads overtake the first's arithmetic
                T::template contract<VG, 0>(rp, q, a, sums + q * 16u, units + q * 2u, total);
                T::template contract<VG, 1>(rp + T::kUnitBytes, q, a, sums + q * 16u + 8u, units + q * 2u + 1u, total);
            } else {
                T::template contract<VG, 0>(rp, q, a, sums + q * 16u, units + q * 2u, total);
            }
        }
        ET_STAMP(4 + 3 * group);
#pragma unroll
        for (int g = 0; g < VG; g++) partial[(group * VG + g) * 64u + lane_id] = total[g];
    }
    // The eight partial sums of every (group, vector group) meet here: each consumer adds those of one
    // pair in wave order (the same bits on every run) and stores sixteen rows of four vectors.
    const uint32_t summed_address = lds_address(&control->summed);
    lds_arrive(summed_address, lane_id == 0);
    ET_STAMP(15);
    if (!lds_await(summed_address, kConsumers, patience)) return;
    for (uint32_t pair = wave; pair < groups * VG; pair += kConsumers) {
        const uint32_t group = pair / VG, g = pair - group * VG;
        float value = 0.f;
#pragma unroll
        for (int w = 0; w < kConsumers; w++)
            value += reinterpret_cast<const float*>(lds + kScratchAt + w * kWaveScratch)[pair * 64u + lane_id];
        const uint32_t vector = 4u * g + q, row = group * kGroupRows + n;
        if (vector < vectors && row < wg_rows) {
            if (bias != nullptr) value += bias[wg_row0 + row];
            y[static_cast<uint64_t>(vector) * rows + wg_row0 + row] = value;
        }
    }
    ET_STAMP(14);
}

// Rows of a workgroup's range: a two-hundred-fifty-sixth of the matrix when its image fits LDS (and
// its groups the partial sums' slots); else the matrix is cut into the fewest rounds of 256 ranges that do.
uint32_t range_rows(uint32_t rows, uint32_t row_bytes) {
    const uint32_t pitch = image_pitch(row_bytes);
    const uint32_t most = std::min((kScratchAt - row_bytes) / pitch + 1u, kMostGroups * kGroupRows);
    const uint32_t share = (rows + 255u) / 256u;
    if (share <= most) return share;
    const uint32_t rounds = (share + most - 1u) / most;
    return (rows + 256u * rounds - 1u) / (256u * rounds);
}

template <class T, int VG, int LOADERS, int DEPTH, int PROBE = 0>
hipError_t launch(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias, float* y,
                  uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
    static std::atomic<bool> allowed[64];
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    const auto kernel = gemv_mma_kernel<T, VG, LOADERS, DEPTH, PROBE>;
    if (!allowed[device].load(std::memory_order_acquire)) {
        if (hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes))
            return status;
        allowed[device].store(true, std::memory_order_release);
    }
    HandoverState handover;
    if (hipError_t status = handover_state(&handover)) return status;
    const uint32_t rows_per_wg = range_rows(rows, (columns >> 8) * T::kUnitBytes);
    const uint32_t grid = (rows + rows_per_wg - 1u) / rows_per_wg;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * (kConsumers + LOADERS)), kLdsBytes, stream, weight, x, x_row_stride,
                       bias, y, rows, columns, rows_per_wg, vectors, handover.limit, handover.timeouts);
    return hipGetLastError();
}

template <class T>
hipError_t launch_vectors(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias, float* y,
                          uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
#ifdef ET_MMA_PROBES
    // timing experiments only (never in the product build): ET_HIP_MMA_VARIANT picks a launch shape or a probe
    static const int variant = [] { const char* v = std::getenv("ET_HIP_MMA_VARIANT"); return v ? std::atoi(v) : 0; }();
#define ET_V(N, ...) case N: return launch<T, __VA_ARGS__>(weight, x, x_row_stride, bias, y, rows, columns, vectors, stream)
    if (vectors <= 4) switch (variant) {
        ET_V(1, 1, 8, 4, 1); ET_V(2, 1, 8, 4, 2); ET_V(3, 1, 8, 5); ET_V(4, 1, 8, 6); ET_V(5, 1, 4, 8); ET_V(6, 1, 8, 8);
        ET_V(7, 1, 8, 3); ET_V(8, 1, 4, 6); ET_V(9, 1, 8, 4, 3); ET_V(10, 1, 8, 4, 4);
        default: break;
    } else switch (variant) {
        ET_V(1, 2, 4, 8, 1); ET_V(2, 2, 4, 8, 2); ET_V(3, 2, 8, 4); ET_V(4, 2, 8, 5); ET_V(5, 2, 4, 6); ET_V(6, 2, 2, 8);
        ET_V(9, 2, 4, 8, 3); ET_V(10, 2, 4, 8, 4);
        default: break;
    }
#undef ET_V
#endif
    if (vectors <= 4) return launch<T, 1, 8, 4>(weight, x, x_row_stride, bias, y, rows, columns, vectors, stream);
    // two vector groups keep 64 registers of A operands: twelve waves leave each 168
    return launch<T, 2, 4, 8>(weight, x, x_row_stride, bias, y, rows, columns, vectors, stream);
}

}  // namespace

#ifdef ET_MMA_PROBES
extern "C" int et_hip_mma_stamps(uint64_t* out, uint64_t count) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(mma_stamps), count * 8);
}
#endif

bool gemv_mma_supported(int32_t codec, uint64_t rows, uint64_t columns, uint32_t vectors) {
    if (codec != kQ4_K && codec != kQ4_0 && codec != kQ5_K && codec != kQ8_0) return false;
    if (vectors < 2 || vectors > kGemvMmaMaxVectors) return false;
    // one image row is at most 16 units; the copies are 16 bytes wide (a unit is a multiple of 16 bytes)
    if (columns == 0 || columns % 256 != 0 || columns > 4096) return false;
    // with less than a group of rows to a compute unit most of every matrix instruction is padding
    return rows >= 256u * 8u && rows <= 0xffffffffull;
}

hipError_t gemv_mma(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias,
                    float* y, uint64_t rows, uint64_t columns, uint32_t vectors, hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns);
    if (!gemv_mma_supported(codec, rows, columns, vectors)) return hipErrorInvalidValue;
    switch (codec) {
        case kQ4_K: return launch_vectors<Q4KMma>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ5_K: return launch_vectors<Q5KMma>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ4_0: return launch_vectors<Q40Mma>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ8_0: return launch_vectors<Q80Mma>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
