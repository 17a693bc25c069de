// Dequant-GEMV on integer dot products for gfx950 (the five K-quants, Q4_0, Q8_0; 1-3 vectors):
//     y[v, r] = sum_k x[v, k] * decode(W[r])[k] (+ bias[r])
//
// Same contraction as linear_into (crates/runtime-cpu/src/quantized.rs:419-499)
// with decode_q4_k (:180-199) in factored form; Q4_0 / Q8_0 follow the public
// ggml block layouts. f32-accurate: the result agrees with the scalar f32 loop
// within 1e-3 (in fact to a few 1e-6 relative).
//
// Why integers. The kernel is HBM-bound (0.56 - 1.06 bytes per weight), and on
// CDNA4 the obvious f32 formulation (byte -> float convert + FMA per weight) is
// VALU-bound before it is HBM-bound: ~2.4 vector ops per weight. Here each f32
// activation is converted ONCE per workgroup to a 24-bit fixed-point integer
// with a shared scale per 64 columns, X = rint(x * 127 * 2^16 / max|x|), and X
// is cut into three signed 8-bit limbs,
//     x ~= s * (65536*x1 + 256*x2 + x3),   |residual| <= 6.0e-8 * max|x|,
// i.e. to f32 precision. The weights' quants - already small integers - meet
// the limbs in v_dot4_i32_i8: 4 multiply-adds per op, three ops per four
// weights, exact int32 accumulation. Block scales are applied to the integer
// sums in f32 afterwards. ~1.3 vector ops per weight.
//
// Work split (activation-stationary): a lane owns 64 consecutive columns (one
// 32-byte pair of a Q4_K super-block, or two Q4_0 / Q8_0 blocks), keeps their
// limbs in registers for its whole life, and streams weight rows past them with
// 16-byte loads. A wave covers 4096 columns, NK waves a row; their partial sums
// meet in LDS. A workgroup walks a contiguous range of rows.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdlib>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"
#include "lds_handover.h"

namespace et {
namespace {

constexpr int kChunk = 64;                       // columns a lane owns
constexpr uint32_t kSliceColumns = 64 * kChunk;  // columns a wave covers
constexpr uint32_t kSliceQuads = kSliceColumns / 4;

// Per-vector lane state: the limbs of the lane's 64 activations and their sums.
struct XLimbs {
    int limb[3][16];  // limb[k][j]: bytes = limb k of elements 4j..4j+3 of the chunk;
                      // limb 0 is the least significant (weight 1), limb 2 the most (65536)
    float s;          // value of one unit of limb 0
    float sum[2];     // exact f32 sums of elements 0..31 and 32..63
    // Codecs whose lanes own four separate 16-column runs (Q6_K) use these instead of s / sum:
    float s_pair[2];  // unit of runs 0, 1 and of runs 2, 3 (they lie in two 64-column chunks)
    int bias[4][3];   // -offset * (sum of the limb bytes of run g): where the integer dots start
    float run_sum[4]; // sum of the (quantised) activations of run g, for codecs with block minima
};

constexpr float kLimbRange = 8323072.0f;  // 127 * 2^16: |X| <= this

// LDS slot (in 16-byte units) of limb unit u = 4*chunk + j: the XOR spreads the
// eight lanes that read in one pass over all banks; writes of consecutive dwords
// stay conflict-free because it only permutes within aligned groups of four units.
__device__ __forceinline__ uint32_t limb_slot(uint32_t u) { return u ^ ((u >> 3) & 3u); }

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

struct alignas(16) StageMemory {
    uint32_t limbs[3][kSliceQuads];  // [limb][swizzled dword]
    float unit[64];
    float sum[2][64];
};

// Splits one float4 of a slice into limbs and stores them in LDS. Float4 number f
// of the slice belongs to thread f % THREADS; sixteen consecutive lanes (one DPP
// row) hold one 64-column chunk, so the chunk's maximum and its two 32-column
// sums are folded across lanes with DPP. Must be called by whole waves.
//
// X = rint(x * inv) is an exact integer of at most 24 bits. Adding 0x8080 and
// flipping the top bit of the two low bytes turns its bytes into balanced
// digits: X = 65536*x1 + 256*x2 + x3 with every x_k a signed byte.
__device__ __forceinline__ void stage_quad(StageMemory& stage, float4 v, uint32_t f) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, dpp<0xB1>(amax));   // quad_perm [1,0,3,2]
    amax = fmaxf(amax, dpp<0x4E>(amax));   // quad_perm [2,3,0,1]
    amax = fmaxf(amax, dpp<0x141>(amax));  // row_half_mirror
    amax = fmaxf(amax, dpp<0x140>(amax));  // row_mirror: all 16 lanes hold the chunk's max
    float total = (v.x + v.y) + (v.z + v.w);
    total += dpp<0xB1>(total);
    total += dpp<0x4E>(total);
    total += dpp<0x141>(total);  // sum over the lane's 8-lane half = 32 columns
    // 1 ulp of the reciprocal moves |X| by at most 1, far inside the headroom of the limbs.
    const bool nonzero = amax >= 1e-30f;
    const float inv = nonzero ? kLimbRange * __builtin_amdgcn_rcpf(amax) : 0.f;
    const float unit = nonzero ? amax * (1.0f / kLimbRange) : 0.f;
    const int x0 = static_cast<int>(rintf(v.x * inv)) + 0x8080;
    const int x1 = static_cast<int>(rintf(v.y * inv)) + 0x8080;
    const int x2 = static_cast<int>(rintf(v.z * inv)) + 0x8080;
    const int x3 = static_cast<int>(rintf(v.w * inv)) + 0x8080;
    // 4x3 byte transpose: limb k of the four elements into one dword.
    const uint32_t a = __builtin_amdgcn_perm(x1, x0, 0x05010400u);  // x0.b0 x1.b0 x0.b1 x1.b1
    const uint32_t b = __builtin_amdgcn_perm(x3, x2, 0x05010400u);
    const uint32_t c = __builtin_amdgcn_perm(x1, x0, 0x0c0c0602u);  // x0.b2 x1.b2 0 0
    const uint32_t d = __builtin_amdgcn_perm(x3, x2, 0x0c0c0602u);
    const uint32_t limb0 = __builtin_amdgcn_perm(b, a, 0x05040100u) ^ 0x80808080u;
    const uint32_t limb1 = __builtin_amdgcn_perm(b, a, 0x07060302u) ^ 0x80808080u;
    const uint32_t limb2 = __builtin_amdgcn_perm(d, c, 0x05040100u);
    const uint32_t slot = limb_slot(f >> 2) * 4u + (f & 3u);
    stage.limbs[0][slot] = limb0;
    stage.limbs[1][slot] = limb1;
    stage.limbs[2][slot] = limb2;
    const uint32_t chunk = f >> 4;
    if ((f & 15u) == 0u) stage.unit[chunk] = unit;
    if ((f & 7u) == 0u) stage.sum[(f >> 3) & 1u][chunk] = total;
}

__device__ __forceinline__ void load_limbs(const StageMemory& stage, uint32_t lane, bool active,
                                           XLimbs& out) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint4 v = *reinterpret_cast<const uint4*>(&stage.limbs[k][limb_slot(4u * lane + j) * 4u]);
            out.limb[k][4 * j + 0] = active ? static_cast<int>(v.x) : 0;
            out.limb[k][4 * j + 1] = active ? static_cast<int>(v.y) : 0;
            out.limb[k][4 * j + 2] = active ? static_cast<int>(v.z) : 0;
            out.limb[k][4 * j + 3] = active ? static_cast<int>(v.w) : 0;
        }
    }
    out.s = active ? stage.unit[lane] : 0.f;
    out.sum[0] = active ? stage.sum[0][lane] : 0.f;
    out.sum[1] = active ? stage.sum[1][lane] : 0.f;
}

// s * (D0 + 256*D1 + 65536*D2) for the integer dots D_k of the three limbs.
__device__ __forceinline__ float limb_value(const XLimbs& x, int d0, int d1, int d2) {
    float v = static_cast<float>(d0);
    v = fmaf(256.0f, static_cast<float>(d1), v);
    v = fmaf(65536.0f, static_cast<float>(d2), v);
    return x.s * v;
}

// ---------------------------------------------------------------------------
// Codec traits: what a lane loads per row and how it folds it with the limbs.
// ---------------------------------------------------------------------------

struct Q4KLimb {
    static constexpr uint32_t kBlockColumns = 256u, kBlockBytes = 144u;
    static constexpr bool kLdsCopies = true;     // its weights can come through LDS copies
    static constexpr bool kCopiesInTurn = true;  // ... on gemv_limb_turns_kernel
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_limbs(stage, lane, active, out);
    }
    struct Lane {
        uint32_t offset;  // byte offset of the lane's block within a row
        uint32_t p;       // pair within the block
    };
    struct Data {
        uint4 header;  // d, dmin, scales[12]
        uint4 q[2];    // the pair's 32 bytes of quants
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 144u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        return Lane{(chunk >> 2) * 144u, chunk & 3u};
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;
        data.header = *reinterpret_cast<const uint4*>(base);
        data.q[0] = *reinterpret_cast<const uint4*>(base + 16 + 32 * lane.p);
        data.q[1] = *reinterpret_cast<const uint4*>(base + 32 + 32 * lane.p);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const XLimbs (&x)[M], float (&value)[M]) {
        const uint32_t w[8] = {data.q[0].x, data.q[0].y, data.q[0].z, data.q[0].w,
                               data.q[1].x, data.q[1].y, data.q[1].z, data.q[1].w};
        int lo[M][3], hi[M][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int k = 0; k < 3; k++) lo[m][k] = hi[m][k] = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // low nibbles: elements 4j..4j+3 of sub-block 2p; high nibbles: of sub-block 2p+1
            const int ql = static_cast<int>(w[j] & 0x0f0f0f0fu);
            const int qh = static_cast<int>((w[j] >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    lo[m][k] = __builtin_amdgcn_sdot4(ql, x[m].limb[k][j], lo[m][k], false);
                    hi[m][k] = __builtin_amdgcn_sdot4(qh, x[m].limb[k][8 + j], hi[m][k], false);
                }
        }
        // (scale, min) of sub-blocks 2p, 2p+1: crates/runtime-cpu/src/quantized.rs:77-86
        const uint32_t shift = (lane.p & 1u) * 16u;
        const uint32_t a = data.header.y >> shift, b = data.header.z >> shift, c = data.header.w >> shift;
        uint32_t sc, mn;
        if (lane.p < 2) {
            sc = a & 0x3f3fu;
            mn = b & 0x3f3fu;
        } else {
            sc = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
            mn = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        }
        const float sc_lo = static_cast<float>(sc & 0xffu), sc_hi = static_cast<float>((sc >> 8) & 0xffu);
        const float m_lo = static_cast<float>(mn & 0xffu), m_hi = static_cast<float>((mn >> 8) & 0xffu);
        const float d = half_bits_to_float(data.header.x & 0xffffu);
        const float dmin = half_bits_to_float(data.header.x >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) {
            // sub-block scales first, limb weights second, one f32 scale last
            // (as floats: the dots are below 2^17 and convert exactly; a 32-bit
            // integer multiply would run at quarter rate)
            const float i1 = fmaf(sc_hi, static_cast<float>(hi[m][0]), sc_lo * static_cast<float>(lo[m][0]));
            const float i2 = fmaf(sc_hi, static_cast<float>(hi[m][1]), sc_lo * static_cast<float>(lo[m][1]));
            const float i3 = fmaf(sc_hi, static_cast<float>(hi[m][2]), sc_lo * static_cast<float>(lo[m][2]));
            const float pos = x[m].s * fmaf(65536.0f, i3, fmaf(256.0f, i2, i1));
            const float neg = fmaf(m_lo, x[m].sum[0], m_hi * x[m].sum[1]);
            value[m] = d * pos - dmin * neg;
        }
    }
};

// Q5_K (decode_q5_k, crates/runtime-cpu/src/quantized.rs:203-234): Q4_K's layout with a fifth bit per
// value in qh[32] between the scales and the nibbles - bit g of qh[i] belongs to element i of
// sub-block g. 176 bytes per block, every field 16-byte aligned.
struct Q5KLimb {
    static constexpr uint32_t kBlockColumns = 256u, kBlockBytes = 176u;
    static constexpr bool kLdsCopies = true;     // its weights can come through LDS copies
    static constexpr bool kCopiesInTurn = true;  // ... on gemv_limb_turns_kernel
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_limbs(stage, lane, active, out);
    }
    struct Lane {
        uint32_t offset;  // byte offset of the lane's block within a row
        uint32_t p;       // pair within the block
    };
    struct Data {
        uint4 header;  // d, dmin, scales[12]
        uint4 h[2];    // qh[32]: the fifth bits of all eight sub-blocks
        uint4 q[2];    // the pair's 32 bytes of nibbles
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 176u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        return Lane{(chunk >> 2) * 176u, chunk & 3u};
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;
        data.header = *reinterpret_cast<const uint4*>(base);
        data.h[0] = *reinterpret_cast<const uint4*>(base + 16);
        data.h[1] = *reinterpret_cast<const uint4*>(base + 32);
        data.q[0] = *reinterpret_cast<const uint4*>(base + 48 + 32 * lane.p);
        data.q[1] = *reinterpret_cast<const uint4*>(base + 64 + 32 * lane.p);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const XLimbs (&x)[M], float (&value)[M]) {
        const uint32_t w[8] = {data.q[0].x, data.q[0].y, data.q[0].z, data.q[0].w,
                               data.q[1].x, data.q[1].y, data.q[1].z, data.q[1].w};
        const uint32_t h[8] = {data.h[0].x, data.h[0].y, data.h[0].z, data.h[0].w,
                               data.h[1].x, data.h[1].y, data.h[1].z, data.h[1].w};
        const uint32_t bit = 2u * lane.p;  // sub-blocks 2p and 2p + 1
        int lo[M][3], hi[M][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int k = 0; k < 3; k++) lo[m][k] = hi[m][k] = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // low nibbles: elements 4j..4j+3 of sub-block 2p; high nibbles: of sub-block 2p+1
            const uint32_t fifth = h[j] >> bit;
            const int ql = static_cast<int>((w[j] & 0x0f0f0f0fu) | ((fifth & 0x01010101u) << 4));
            const int qh = static_cast<int>(((w[j] >> 4) & 0x0f0f0f0fu) | ((fifth & 0x02020202u) << 3));
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    lo[m][k] = __builtin_amdgcn_sdot4(ql, x[m].limb[k][j], lo[m][k], false);
                    hi[m][k] = __builtin_amdgcn_sdot4(qh, x[m].limb[k][8 + j], hi[m][k], false);
                }
        }
        // (scale, min) of sub-blocks 2p, 2p+1: crates/runtime-cpu/src/quantized.rs:77-86
        const uint32_t shift = (lane.p & 1u) * 16u;
        const uint32_t a = data.header.y >> shift, b = data.header.z >> shift, c = data.header.w >> shift;
        uint32_t sc, mn;
        if (lane.p < 2) {
            sc = a & 0x3f3fu;
            mn = b & 0x3f3fu;
        } else {
            sc = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
            mn = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        }
        const float sc_lo = static_cast<float>(sc & 0xffu), sc_hi = static_cast<float>((sc >> 8) & 0xffu);
        const float m_lo = static_cast<float>(mn & 0xffu), m_hi = static_cast<float>((mn >> 8) & 0xffu);
        const float d = half_bits_to_float(data.header.x & 0xffffu);
        const float dmin = half_bits_to_float(data.header.x >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) {
            // sub-block scales first, limb weights second, one f32 scale last
            // (as floats: the dots are below 2^17 and convert exactly; a 32-bit
            // integer multiply would run at quarter rate)
            const float i1 = fmaf(sc_hi, static_cast<float>(hi[m][0]), sc_lo * static_cast<float>(lo[m][0]));
            const float i2 = fmaf(sc_hi, static_cast<float>(hi[m][1]), sc_lo * static_cast<float>(lo[m][1]));
            const float i3 = fmaf(sc_hi, static_cast<float>(hi[m][2]), sc_lo * static_cast<float>(lo[m][2]));
            const float pos = x[m].s * fmaf(65536.0f, i3, fmaf(256.0f, i2, i1));
            const float neg = fmaf(m_lo, x[m].sum[0], m_hi * x[m].sum[1]);
            value[m] = d * pos - dmin * neg;
        }
    }
};

struct __attribute__((packed, aligned(4))) Dwords9 {
    uint32_t v[9];
};
struct __attribute__((packed, aligned(4))) Dwords17 {
    uint32_t v[17];
};

// Q4_0: two 18-byte blocks = 36 bytes = 9 dwords (dword aligned when columns % 64 == 0).
struct Q40Limb {
    static constexpr uint32_t kBlockColumns = 32u, kBlockBytes = 18u;
    static constexpr bool kLdsCopies = true;     // its weights can come through LDS copies
    static constexpr bool kCopiesInTurn = true;  // ... on gemv_limb_turns_kernel
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_limbs(stage, lane, active, out);
    }
    struct Lane {
        uint32_t offset;
    };
    struct Data {
        Dwords9 raw;
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 5) * 18u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) { return Lane{chunk * 36u}; }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        data.raw = *reinterpret_cast<const Dwords9*>(row + lane.offset);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane&, const XLimbs (&x)[M],
                                                float (&value)[M]) {
        const uint32_t* w = data.raw.v;
        int da_[M][3], db_[M][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int k = 0; k < 3; k++) da_[m][k] = db_[m][k] = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // block A: bytes 2..17 of the pair (2 bytes off dword alignment); block B: bytes 20..35.
            // Byte j's low nibble is element j, its high nibble element j + 16.
            const uint32_t qa = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
            const uint32_t qb = w[5 + i];
            const int al = static_cast<int>(qa & 0x0f0f0f0fu), ah = static_cast<int>((qa >> 4) & 0x0f0f0f0fu);
            const int bl = static_cast<int>(qb & 0x0f0f0f0fu), bh = static_cast<int>((qb >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    da_[m][k] = __builtin_amdgcn_sdot4(al, x[m].limb[k][i], da_[m][k], false);
                    da_[m][k] = __builtin_amdgcn_sdot4(ah, x[m].limb[k][4 + i], da_[m][k], false);
                    db_[m][k] = __builtin_amdgcn_sdot4(bl, x[m].limb[k][8 + i], db_[m][k], false);
                    db_[m][k] = __builtin_amdgcn_sdot4(bh, x[m].limb[k][12 + i], db_[m][k], false);
                }
        }
        const float da = half_bits_to_float(w[0] & 0xffffu);
        const float db = half_bits_to_float(w[4] >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) {
            // value = d * (nibble - 8): the -8 meets the chunk's activation sums once
            const float va = limb_value(x[m], da_[m][0], da_[m][1], da_[m][2]) - 8.f * x[m].sum[0];
            const float vb = limb_value(x[m], db_[m][0], db_[m][1], db_[m][2]) - 8.f * x[m].sum[1];
            value[m] = da * va + db * vb;
        }
    }
};

// Q8_0: two 34-byte blocks = 68 bytes = 17 dwords (dword aligned when columns % 64 == 0).
struct Q80Limb {
    static constexpr uint32_t kBlockColumns = 32u, kBlockBytes = 34u;
    static constexpr bool kLdsCopies = true;     // its weights can come through LDS copies
    static constexpr bool kCopiesInTurn = true;  // ... on gemv_limb_turns_kernel
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_limbs(stage, lane, active, out);
    }
    struct Lane {
        uint32_t offset;
    };
    struct Data {
        Dwords17 raw;
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 5) * 34u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) { return Lane{chunk * 68u}; }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        data.raw = *reinterpret_cast<const Dwords17*>(row + lane.offset);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane&, const XLimbs (&x)[M],
                                                float (&value)[M]) {
        const uint32_t* w = data.raw.v;
        int da_[M][3], db_[M][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int k = 0; k < 3; k++) da_[m][k] = db_[m][k] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int qa = static_cast<int>(__builtin_amdgcn_alignbit(w[i + 1], w[i], 16));  // bytes 2..33
            const int qb = static_cast<int>(w[9 + i]);                                        // bytes 36..67
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    da_[m][k] = __builtin_amdgcn_sdot4(qa, x[m].limb[k][i], da_[m][k], false);
                    db_[m][k] = __builtin_amdgcn_sdot4(qb, x[m].limb[k][8 + i], db_[m][k], false);
                }
        }
        const float da = half_bits_to_float(w[0] & 0xffffu);
        const float db = half_bits_to_float(w[8] >> 16);
#pragma unroll
        for (int m = 0; m < M; m++)
            value[m] = da * limb_value(x[m], da_[m][0], da_[m][1], da_[m][2]) +
                       db * limb_value(x[m], db_[m][0], db_[m][1], db_[m][2]);
    }
};

// Sixteen bytes from an address that is only 2-byte aligned (odd Q6_K blocks start at 210 * b).
#pragma clang diagnostic ignored "-Walign-mismatch"
typedef uint4 __attribute__((aligned(2))) uint4_a2;
typedef uint2 __attribute__((aligned(2))) uint2_a2;

// Activations of a lane that owns four 16-column runs of a 256-column block (Q2_K, Q3_K, Q6_K):
// lane (block b, half, j) takes runs g = 0..3 = 16-column units 16b + 8*half + 2g + j of the slice.
// OFFSET is what the codec subtracts from every quant: the integer dots start at -OFFSET * (sum of
// the run's limb bytes), so that sum (q - OFFSET) x needs no per-row work.
template <int OFFSET>
__device__ __forceinline__ void load_run_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                     XLimbs& out) {
    const uint32_t first = 16u * (lane >> 2) + 8u * ((lane >> 1) & 1u) + (lane & 1u);
    int totals[4][3];
#pragma unroll
    for (int k = 0; k < 3; k++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 v = *reinterpret_cast<const uint4*>(&stage.limbs[k][limb_slot(first + 2u * g) * 4u]);
            const int words[4] = {static_cast<int>(v.x), static_cast<int>(v.y), static_cast<int>(v.z),
                                  static_cast<int>(v.w)};
            int total = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                out.limb[k][4 * g + i] = active ? words[i] : 0;
                total = __builtin_amdgcn_sdot4(0x01010101, out.limb[k][4 * g + i], total, false);
            }
            totals[g][k] = total;
            out.bias[g][k] = -OFFSET * total;
        }
    }
    const uint32_t chunk = 4u * (lane >> 2) + 2u * ((lane >> 1) & 1u);
    out.s_pair[0] = active ? stage.unit[chunk] : 0.f;
    out.s_pair[1] = active ? stage.unit[chunk + 1u] : 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++)
        out.run_sum[g] = out.s_pair[g >> 1] * fmaf(65536.0f, static_cast<float>(totals[g][2]),
                                                   fmaf(256.0f, static_cast<float>(totals[g][1]),
                                                        static_cast<float>(totals[g][0])));
    out.s = 0.f;
    out.sum[0] = out.sum[1] = 0.f;
}

// Q6_K (decode_q6_k, crates/runtime-cpu/src/quantized.rs:238-261): 210 bytes per 256 values -
// ql[128] low nibbles, qh[64] two high bits, scales[16] int8 per 16 values, d. Value e = half*128 +
// quarter*32 + i of a block is d * scale[half*8 + quarter*2 + i/16] * (q - 32) with
// q = nibble(ql[half*64 + (quarter & 1)*32 + i], quarter >> 1) | ((qh[half*32 + i] >> 2*quarter) & 3) << 4.
// A lane takes (half, j = i / 16) of a block: the four 16-column runs quarter = 0..3, each with ONE
// scale, out of exactly 48 bytes of quants - three 16-byte loads, nothing read twice. Its 64 columns
// are not consecutive, so it gathers its activation limbs run by run (load_activations).
struct Q6KLimb {
    static constexpr uint32_t kBlockColumns = 256u, kBlockBytes = 210u;
    static constexpr bool kLdsCopies = false;    // gemv_limb_kernel only: a share of 14336 rows (56 x 3360 bytes) does not fit LDS
    struct Lane {
        uint32_t offset;  // byte offset of the lane's block within a row
        uint32_t half, j;
    };
    struct Data {
        uint4 qa, qb, qh;  // ql[half*64 + 16j ..], ql[half*64 + 32 + 16j ..], qh[half*32 + 16j ..]
        uint2 scales;      // scales[half*8 .. half*8 + 8]
        uint32_t d;        // f16 bits
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 210u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        return Lane{(chunk >> 2) * 210u, (chunk >> 1) & 1u, chunk & 1u};
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;
        data.qa = *reinterpret_cast<const uint4_a2*>(base + 64u * lane.half + 16u * lane.j);
        data.qb = *reinterpret_cast<const uint4_a2*>(base + 64u * lane.half + 32u + 16u * lane.j);
        data.qh = *reinterpret_cast<const uint4_a2*>(base + 128u + 32u * lane.half + 16u * lane.j);
        data.scales = *reinterpret_cast<const uint2_a2*>(base + 192u + 8u * lane.half);
        data.d = *reinterpret_cast<const uint16_t*>(base + 208u);
    }
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_run_activations<32>(stage, lane, active, out);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const XLimbs (&x)[M], float (&value)[M]) {
        const uint32_t qa[4] = {data.qa.x, data.qa.y, data.qa.z, data.qa.w};
        const uint32_t qb[4] = {data.qb.x, data.qb.y, data.qb.z, data.qb.w};
        const uint32_t qh[4] = {data.qh.x, data.qh.y, data.qh.z, data.qh.w};
        int dot[M][4][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int k = 0; k < 3; k++) dot[m][g][k] = x[m].bias[g][k];  // sum (q - 32) x = sum q x - 32 sum x
#pragma unroll
        for (int g = 0; g < 4; g++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t low = (g & 1) ? qb[i] : qa[i];
                const uint32_t nibbles = ((g & 2) ? (low >> 4) : low) & 0x0f0f0f0fu;
                const uint32_t high = (qh[i] >> (2 * g)) & 0x03030303u;
                const int q = static_cast<int>((high << 4) | nibbles);  // four values 0..63
#pragma unroll
                for (int m = 0; m < M; m++)
#pragma unroll
                    for (int k = 0; k < 3; k++)
                        dot[m][g][k] = __builtin_amdgcn_sdot4(q, x[m].limb[k][4 * g + i], dot[m][g][k], false);
            }
        }
        // scale of run g: signed byte j + 2g of the eight
        const uint32_t shift = 8u * lane.j;
        const auto signed_byte = [](uint32_t word, uint32_t at) {
            return static_cast<float>(static_cast<int>(static_cast<int8_t>(word >> at)));
        };
        const float sc[4] = {signed_byte(data.scales.x, shift), signed_byte(data.scales.x, shift + 16u),
                             signed_byte(data.scales.y, shift), signed_byte(data.scales.y, shift + 16u)};
        const float d = half_bits_to_float(data.d);
#pragma unroll
        for (int m = 0; m < M; m++) {
            float part[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                // the dots are below 2^21 in magnitude and convert exactly
                float limb_sum[3];
#pragma unroll
                for (int k = 0; k < 3; k++)
                    limb_sum[k] = fmaf(sc[2 * h + 1], static_cast<float>(dot[m][2 * h + 1][k]),
                                       sc[2 * h] * static_cast<float>(dot[m][2 * h][k]));
                part[h] = fmaf(65536.0f, limb_sum[2], fmaf(256.0f, limb_sum[1], limb_sum[0]));
            }
            value[m] = d * fmaf(x[m].s_pair[1], part[1], x[m].s_pair[0] * part[0]);
        }
    }
};

// s_pair[0] * (limb-combined, scale-weighted dots of runs 0, 1) + s_pair[1] * (those of runs 2, 3)
template <int M>
__device__ __forceinline__ void combine_runs(const int (&dot)[M][4][3], const float (&sc)[4], const XLimbs (&x)[M],
                                             float (&out)[M]) {
#pragma unroll
    for (int m = 0; m < M; m++) {
        float part[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            float limb_sum[3];
#pragma unroll
            for (int k = 0; k < 3; k++)
                limb_sum[k] = fmaf(sc[2 * h + 1], static_cast<float>(dot[m][2 * h + 1][k]),
                                   sc[2 * h] * static_cast<float>(dot[m][2 * h][k]));
            part[h] = fmaf(65536.0f, limb_sum[2], fmaf(256.0f, limb_sum[1], limb_sum[0]));
        }
        out[m] = fmaf(x[m].s_pair[1], part[1], x[m].s_pair[0] * part[0]);
    }
}

typedef uint4 __attribute__((aligned(4))) uint4_a4;
typedef struct __attribute__((packed, aligned(2))) { uint32_t v[3]; } Dwords3_a2;

// Q2_K (decode_q2_k, crates/runtime-cpu/src/quantized.rs:117-138): 84 bytes per 256 values - scales[16]
// (4-bit scale, 4-bit minimum per 16 values), qs[64] (2-bit quants), d, dmin. Value e = half*128 + 32g +
// 16j + i is d * (scales[8*half + 2g + j] & 15) * ((qs[32*half + 16j + i] >> 2g) & 3) - dmin *
// (scales[..] >> 4). A lane takes (half, j): runs g = 0..3, sixteen bytes of quants.
struct Q2KLimb {
    static constexpr uint32_t kBlockColumns = 256u, kBlockBytes = 84u;
    static constexpr bool kLdsCopies = true;     // gemv_limb_dma_kernel takes this codec; LDS serves the lanes' loads at any alignment
    static constexpr bool kCopiesInTurn = false; // ... on gemv_limb_dma_kernel, whose loaders fold the end of their ranges
    struct Lane {
        uint32_t offset, half, j;
    };
    struct Data {
        uint4 qs;
        uint2 scales;  // scales[8*half .. 8*half + 8]
        uint32_t dd;   // d | dmin << 16 (f16 bits)
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 84u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        return Lane{(chunk >> 2) * 84u, (chunk >> 1) & 1u, chunk & 1u};
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;  // 84 b: dword aligned
        data.qs = *reinterpret_cast<const uint4_a4*>(base + 16u + 32u * lane.half + 16u * lane.j);
        data.scales = *reinterpret_cast<const uint2_a2*>(base + 8u * lane.half);
        data.dd = *reinterpret_cast<const uint32_t*>(base + 80u);
    }
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_run_activations<0>(stage, lane, active, out);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const XLimbs (&x)[M], float (&value)[M]) {
        const uint32_t qs[4] = {data.qs.x, data.qs.y, data.qs.z, data.qs.w};
        int dot[M][4][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int k = 0; k < 3; k++) dot[m][g][k] = 0;
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int q = static_cast<int>((qs[i] >> (2 * g)) & 0x03030303u);
#pragma unroll
                for (int m = 0; m < M; m++)
#pragma unroll
                    for (int k = 0; k < 3; k++)
                        dot[m][g][k] = __builtin_amdgcn_sdot4(q, x[m].limb[k][4 * g + i], dot[m][g][k], false);
            }
        // (scale, minimum) of run g: byte j + 2g of the eight
        const uint32_t shift = 8u * lane.j;
        const uint32_t bytes[4] = {(data.scales.x >> shift) & 0xffu, (data.scales.x >> (shift + 16u)) & 0xffu,
                                   (data.scales.y >> shift) & 0xffu, (data.scales.y >> (shift + 16u)) & 0xffu};
        float sc[4], mn[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            sc[g] = static_cast<float>(bytes[g] & 15u);
            mn[g] = static_cast<float>(bytes[g] >> 4);
        }
        float pos[M];
        combine_runs<M>(dot, sc, x, pos);
        const float d = half_bits_to_float(data.dd & 0xffffu), dmin = half_bits_to_float(data.dd >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float neg = fmaf(mn[3], x[m].run_sum[3],
                                   fmaf(mn[2], x[m].run_sum[2], fmaf(mn[1], x[m].run_sum[1], mn[0] * x[m].run_sum[0])));
            value[m] = d * pos[m] - dmin * neg;
        }
    }
};

// Q3_K (decode_q3_k, crates/runtime-cpu/src/quantized.rs:142-176): 110 bytes per 256 values - hmask[32]
// (third bits), qs[64] (2-bit quants), scales[12] (sixteen 6-bit scales, packed), d. Value e = half*128 +
// 32g + 16j + i is d * (scale[8*half + 2g + j] - 32) * (((qs[32*half + 16j + i] >> 2g) & 3) -
// (hmask[16j + i] bit (4*half + g) ? 0 : 4)). A lane takes (half, j): runs g = 0..3.
struct Q3KLimb {
    static constexpr uint32_t kBlockColumns = 256u, kBlockBytes = 110u;
    // gemv_limb_kernel only. LDS serves the lanes' 2-byte-aligned 16-byte reads, but slowly: through
    // gemv_limb_dma_kernel 14336 x 4096 measured 10.5 us against 9.6.
    static constexpr bool kLdsCopies = false;
    struct Lane {
        uint32_t offset, half, j;
    };
    struct Data {
        uint4 qs, hm;
        uint32_t packed[3];  // scales[12]
        uint32_t d;
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 110u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        return Lane{(chunk >> 2) * 110u, (chunk >> 1) & 1u, chunk & 1u};
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;  // 110 b: odd blocks start 2 bytes off a dword
        data.hm = *reinterpret_cast<const uint4_a2*>(base + 16u * lane.j);
        data.qs = *reinterpret_cast<const uint4_a2*>(base + 32u + 32u * lane.half + 16u * lane.j);
        const Dwords3_a2 packed = *reinterpret_cast<const Dwords3_a2*>(base + 96u);
        data.packed[0] = packed.v[0];
        data.packed[1] = packed.v[1];
        data.packed[2] = packed.v[2];
        data.d = *reinterpret_cast<const uint16_t*>(base + 108u);
    }
    static __device__ __forceinline__ void load_activations(const StageMemory& stage, uint32_t lane, bool active,
                                                            XLimbs& out) {
        load_run_activations<4>(stage, lane, active, out);
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const XLimbs (&x)[M], float (&value)[M]) {
        const uint32_t qs[4] = {data.qs.x, data.qs.y, data.qs.z, data.qs.w};
        const uint32_t hm[4] = {data.hm.x, data.hm.y, data.hm.z, data.hm.w};
        int dot[M][4][3];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int k = 0; k < 3; k++) dot[m][g][k] = x[m].bias[g][k];  // sum (v - 4) x = sum v x - 4 sum x
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t low = (qs[i] >> (2 * g)) & 0x03030303u;
                const uint32_t third = (hm[i] >> (4u * lane.half + g)) & 0x01010101u;
                const int v = static_cast<int>(low | (third << 2));  // four values 0..7
#pragma unroll
                for (int m = 0; m < M; m++)
#pragma unroll
                    for (int k = 0; k < 3; k++)
                        dot[m][g][k] = __builtin_amdgcn_sdot4(v, x[m].limb[k][4 * g + i], dot[m][g][k], false);
            }
        // scale of group G = 8*half + 2g + j: low four bits = nibble `half` of byte 2g + j of scales[0..8],
        // top two bits = bits 2*(2*half + g/2) of byte 8 + 2*(g & 1) + j; minus 32
        float sc[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t word = g < 2 ? data.packed[0] : data.packed[1];
            const uint32_t low = (word >> (8u * (2u * (g & 1) + lane.j) + 4u * lane.half)) & 15u;
            const uint32_t high = (data.packed[2] >> (8u * (2u * (g & 1) + lane.j) + 2u * (2u * lane.half + (g >> 1)))) & 3u;
            sc[g] = static_cast<float>(static_cast<int>(low | (high << 4)) - 32);
        }
        float pos[M];
        combine_runs<M>(dot, sc, x, pos);
        const float d = half_bits_to_float(data.d);
#pragma unroll
        for (int m = 0; m < M; m++) value[m] = d * pos[m];
    }
};

// ---------------------------------------------------------------------------
// The kernel. M vectors, R rows per wave iteration, WAVES waves per workgroup,
// NK waves per row (so WAVES / NK row groups per workgroup).
//
// A 33 MB GEMV lasts only a few microseconds, comparable to a handful of HBM
// round trips, so what counts is how early the whole weight matrix is in
// flight. LOOP = false is the single-shot form: every wave requests ALL its rows
// (R <= 8) as its very first instructions after the activation loads, then
// prepares the activations while the weights travel, then folds the rows as
// they arrive. LOOP = true keeps two R-row buffers in ping-pong for shapes
// whose rows per wave do not fit registers.
// ---------------------------------------------------------------------------
template <class T, int M, int R, int WAVES, int NK, bool LOOP>
__global__ __launch_bounds__(64 * WAVES) void gemv_limb_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t rows_per_wg) {
    constexpr int RG = WAVES / NK;
    constexpr int THREADS = 64 * WAVES;
    constexpr int NI = (kSliceQuads + THREADS - 1) / THREADS;  // float4s per thread and slice
    __shared__ StageMemory stage[M];
    __shared__ float partial[2][RG][NK][R][M];
    const uint32_t lane_id = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t slice = wave % NK;
    const uint32_t group = wave / NK;
    const uint32_t all_quads = columns >> 2;

    // Activation loads first: they are served by L2 and must not queue behind
    // the weight loads (a wave's loads complete in order).
    auto load_x = [&](uint32_t s, float4 (&xv)[M][NI]) {
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const uint32_t f = threadIdx.x + i * THREADS;
                const uint32_t quad = s * kSliceQuads + f;
                xv[m][i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (f < kSliceQuads && quad < all_quads)
                    xv[m][i] = reinterpret_cast<const float4*>(x + m * x_row_stride)[quad];
            }
    };
    float4 xv[M][NI];
    load_x(0, xv);

    const uint32_t chunk = slice * 64u + lane_id;  // which 64-column stretch of the row
    const bool active = chunk < columns / kChunk;
    const typename T::Lane lane = T::lane_setup(active ? chunk : 0u);
    const uint64_t row_bytes = T::row_bytes(columns);

    const uint32_t wg_row0 = blockIdx.x * rows_per_wg;
    const uint32_t wg_row_end = min(wg_row0 + rows_per_wg, rows);
    const uint32_t iterations = LOOP ? (wg_row_end - wg_row0 + RG * R - 1) / (RG * R) : 1u;

    auto load_row = [&](uint32_t it, int r, typename T::Data& data) {
        uint32_t row = wg_row0 + (it * RG + group) * R + r;
        row = min(row, rows - 1);  // rows past the end re-read a valid row and are discarded
        T::load(weight + row * row_bytes, lane, data);
    };
    auto load_rows = [&](uint32_t it, typename T::Data (&data)[R]) {
#pragma unroll
        for (int r = 0; r < R; r++) load_row(it, r, data[r]);
    };

    // Order of the prologue. A wave that issues a load while the CU's memory
    // queue is full stalls, and so does everything behind the load in program
    // order; once the weights of a whole CU are requested the queue stays full
    // for microseconds. The activations, which the whole workgroup needs before
    // the first multiply, therefore go first: (1) activation loads, (2) ONE row
    // of weights, so that HBM has work during the activation round trip,
    // (3) split the activations as soon as they are back, (4) barrier, (5) only
    // then the rest of the rows, which may stall freely.
    typename T::Data current[R];
    load_row(0, 0, current[0]);
    __builtin_amdgcn_sched_barrier(0);

    // Activations: limbs in LDS -> registers, one 4096-column slice at a time.
    XLimbs xr[M];
    for (uint32_t s = 0; s < NK; s++) {
        if (s != 0) {
            __syncthreads();
            load_x(s, xv);
        }
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const uint32_t f = threadIdx.x + i * THREADS;
                if (f < kSliceQuads) stage_quad(stage[m], xv[m][i], f);  // wave-uniform condition
            }
        __syncthreads();
        if (s == slice) {
#pragma unroll
            for (int m = 0; m < M; m++) T::load_activations(stage[m], lane_id, active, xr[m]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // Writes the outputs of iteration `it` from the per-row totals.
    auto write_rows = [&](uint32_t it, const float (&total)[R][M]) {
        const uint32_t row0 = wg_row0 + (it * RG + group) * R;
        if (NK == 1) {
            if (lane_id == 0) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const uint32_t row = row0 + r;
                    if (row < wg_row_end) {
                        const float b = bias != nullptr ? bias[row] : 0.f;
#pragma unroll
                        for (int m = 0; m < M; m++)
                            y[static_cast<uint64_t>(m) * rows + row] =
                                bias != nullptr ? total[r][m] + b : total[r][m];
                    }
                }
            }
        } else {
            const uint32_t parity = it & 1u;
            if (lane_id == 0) {
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int m = 0; m < M; m++) partial[parity][group][slice][r][m] = total[r][m];
            }
            __syncthreads();
            if (slice == 0 && lane_id < R * M) {
                const uint32_t r = lane_id / M, m = lane_id - r * M;
                const uint32_t row = row0 + r;
                if (row < wg_row_end) {
                    float value = 0.f;
                    for (int s = 0; s < NK; s++) value += partial[parity][group][s][r][m];
                    if (bias != nullptr) value += bias[row];
                    y[static_cast<uint64_t>(m) * rows + row] = value;
                }
            }
        }
    };
    auto fold_row = [&](const typename T::Data& data, float (&total)[M]) {
        float value[M];
        T::template fold<M>(data, lane, xr, value);
#pragma unroll
        for (int m = 0; m < M; m++) total[m] = wave_sum(active ? value[m] : 0.f);
    };

    if (!LOOP) {
        // Request row r+1, then fold row r: a request that stalls on a full
        // queue stalls behind useful work, and rows are folded as they arrive.
        float total[R][M];
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (r + 1 < R) load_row(0, r + 1, current[r + 1]);
            __builtin_amdgcn_sched_barrier(0);
            fold_row(current[r], total[r]);
            __builtin_amdgcn_sched_barrier(0);
        }
        write_rows(0, total);
    } else {
        // Two R-row buffers in ping-pong. Row 0 of the first is already on its way.
        typename T::Data other[R];
#pragma unroll
        for (int r = 1; r < R; r++) load_row(0, r, current[r]);
        float total[R][M];
        for (uint32_t it = 0; it < iterations; it += 2) {
            if (it + 1 < iterations) load_rows(it + 1, other);
#pragma unroll
            for (int r = 0; r < R; r++) fold_row(current[r], total[r]);
            write_rows(it, total);
            if (it + 1 < iterations) {
                if (it + 2 < iterations) load_rows(it + 2, current);
#pragma unroll
                for (int r = 0; r < R; r++) fold_row(other[r], total[r]);
                write_rows(it + 1, total);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// The same GEMV with the weights brought in by global-to-LDS copies (one slice: columns <= 4096).
//
// What bounds gemv_limb_kernel is how many bytes a compute unit keeps in flight: a wave requests
// the next row only after it has folded the one before, because a wave that issues a load into a
// full memory queue stalls with all the arithmetic behind it. Here the two jobs are split between
// waves. The workgroup's share of W - a contiguous range of rows, at most 158 KiB - is cut into
// eight contiguous ranges, one per CONSUMER wave; consumer w's range is copied into LDS, as it lies
// in memory, by LOADER wave w with 1 KiB global_load_lds copies (no registers; a loader that stalls
// on a full queue holds nothing up), while the consumers prepare the activations and then fold
// their rows out of LDS as they land. A consumer issues no global load after its activation loads.
//
// Hand-over without barriers (s_barrier would tie the loaders to the consumers' prologue): a
// loader keeps DEPTH copies in flight; before it issues the next one it waits for the oldest
// (loads return in order per wave: one counted s_waitcnt) and publishes in LDS how many of its
// copies have landed; its consumer polls that one word until it covers the next row.
// This kernel serves the 2-bit codec, whose folds are long against its bytes: a loader has issued its
// few copies early and would idle, so once they have all landed it folds the last quarter of its range.
// The other codecs run on gemv_limb_turns_kernel below.
// The consumers meet each other through one LDS counter (`staged`).
// LDS: [the ranges, whole KiB each][...][StageMemory x M][control]; shapes whose ranges would reach
// into the stages stay on gemv_limb_kernel.
// ---------------------------------------------------------------------------
// ET_HIP_GEMV_LDS_COPIES=0 in the environment keeps every shape on gemv_limb_kernel (for A/B timing).
bool gemv_limb_dma_enabled() {
    static const bool enabled = [] {
        const char* value = std::getenv("ET_HIP_GEMV_LDS_COPIES");
        return value == nullptr || value[0] != '0';
    }();
    return enabled;
}

constexpr int kDmaPairs = 8;  // ranges of a share: one loader and one consumer wave each (a workgroup has at most
                              // sixteen waves)
constexpr int kDmaConsumers = kDmaPairs;
constexpr int kDmaDepth = 4;  // copies a loader keeps in flight: more only lengthen the queue, and a loader says that a
                              // copy has landed only when it may issue the copy DEPTH places later
constexpr int kDmaHead = kDmaDepth;  // copies a loader issues before it does anything else, at most eight
                                     // (wait_copies_in_flight). Six and eight measured slower when the 4-bit codec ran
                                     // on this kernel (14336 x 4096: 7.9 and 8.2 against 7.7 us).
constexpr uint32_t kDmaLateEighths = 2;  // share of a range that a loader which only copies folds at the end
constexpr int kDmaThreads = 64 * (kDmaConsumers + kDmaPairs);
constexpr int kTurnConsumers = 11, kTurnLoaders = 5, kTurnDepth = 6;  // gemv_limb_turns_kernel: waves that fold, waves that
                                                                      // copy, copies in flight per loader
static_assert(64 * (kTurnConsumers + kTurnLoaders) == kDmaThreads, "sixteen waves either way");
constexpr uint32_t kDmaLdsBytes = 160u * 1024u;
struct DmaControl {
    uint32_t landed[kDmaPairs];  // copies of loader w that have landed
    uint32_t staged;             // consumers that have written their part of the stages
    uint32_t pad[7];
};
constexpr uint32_t kDmaControlAt = kDmaLdsBytes - 1024u;
static_assert(sizeof(DmaControl) == 64, "sixteen words, zeroed by sixteen lanes");

template <class T, int M, int DEPTH>
__global__ __launch_bounds__(kDmaThreads) void gemv_limb_dma_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t rows_per_wg, uint32_t spin_limit, uint32_t* timeouts) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    Patience patience{spin_limit, timeouts};  // every wait on another wave is bounded (lds_handover.h)
    constexpr uint32_t kStageAt = kDmaControlAt - M * static_cast<uint32_t>(sizeof(StageMemory));
    constexpr int NI = kSliceQuads / (64 * kDmaConsumers);  // float4s per consumer thread and vector
    static_assert(DEPTH <= kDmaHead && kDmaHead <= 8, "the steady loop starts with DEPTH copies in flight; wait_copies_in_flight counts to seven");
    static_assert(!T::kCopiesInTurn, "the other codecs run on gemv_limb_turns_kernel");
    DmaControl* control = reinterpret_cast<DmaControl*>(lds + kDmaControlAt);
    StageMemory* stage = reinterpret_cast<StageMemory*>(lds + kStageAt);

    const uint32_t lane_id = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wg_row0 = blockIdx.x * rows_per_wg;
    if (wg_row0 >= rows) return;
    const uint32_t wg_rows = min(rows_per_wg, rows - wg_row0);
    const uint32_t row_bytes = static_cast<uint32_t>(T::row_bytes(columns));
    const bool consumer = wave < static_cast<uint32_t>(kDmaConsumers);
    // the range this wave works on: rows [first, first + count) of the share, `range_kib` KiB of LDS each
    const uint32_t pair = consumer ? wave : wave - kDmaConsumers;
    const uint32_t per_pair = (rows_per_wg + kDmaPairs - 1u) / kDmaPairs;
    const uint32_t first = min(pair * per_pair, wg_rows);
    const uint32_t count = min(per_pair, wg_rows - first);
    const uint32_t range_kib = (per_pair * row_bytes + 1023u) >> 10;
    uint8_t* range = lds + pair * (range_kib << 10);
    const uint32_t late = count * kDmaLateEighths / 8u;  // rows the loader folds after its last copy

    const uint32_t chunk = lane_id;  // one slice: the lane's 64-column stretch of the row
    const bool active = chunk < columns / kChunk;
    const typename T::Lane lane = T::lane_setup(active ? chunk : 0u);
    XLimbs xr[M];
    // Folds a row of the range that is in registers and stores the result. The loaders keep few copies
    // in flight, so a store finds room in the memory queue.
    const auto fold_row = [&](uint32_t r, const typename T::Data& data) {
        float value[M];
        T::template fold<M>(data, lane, xr, value);
        const uint32_t row = wg_row0 + first + r;
        const float b = bias != nullptr ? bias[row] : 0.f;
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float total = wave_sum(active ? value[m] : 0.f);
            if (lane_id == 0) y[static_cast<uint64_t>(m) * rows + row] = bias != nullptr ? total + b : total;
        }
    };

    float4 xv[M][NI];
    if (consumer) {
        // Activation loads go first in the consumers: nothing of theirs may queue behind a copy.
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const uint32_t quad = threadIdx.x + i * 64u * kDmaConsumers;
                xv[m][i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (quad < (columns >> 2)) xv[m][i] = reinterpret_cast<const float4*>(x + m * x_row_stride)[quad];
            }
        if (threadIdx.x < 16) reinterpret_cast<uint32_t*>(control)[threadIdx.x] = 0u;
        __syncthreads();  // the only barrier: the counters are zero before anybody counts
    } else {
        // ---- loaders ------------------------------------------------------------------------
        const uint32_t bytes = count * row_bytes;
        const uint32_t copies = (bytes + 1023u) >> 10;
        const uint8_t* source = weight + (static_cast<uint64_t>(wg_row0) + first) * row_bytes;
        const uint32_t landed_address = lds_address(&control->landed[pair]);
        const auto copy = [&](uint32_t i) {
            const uint32_t at = i * 1024u + lane_id * 16u;
            if (at < bytes)  // the last copy of a range stops where the range ends
                // streamed once: non-temporal (aux bit 1), the caches keep nothing of it
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(source + at),
                                                 reinterpret_cast<uint4*>(range + i * 1024u), 16, 0, 2);
        };
        // The first copies wait for the barrier, i.e. until the consumers have issued their activation
        // loads: issued ahead of it they delay those loads, and with them every fold, by half a microsecond.
        __syncthreads();
        const uint32_t head = min(copies, static_cast<uint32_t>(kDmaHead));
        for (uint32_t i = 0; i < head; i++) copy(i);
        uint32_t landed = 0, in_flight = head;
        if (in_flight > static_cast<uint32_t>(DEPTH)) {  // down to the steady depth
            __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH));
            landed = in_flight - DEPTH;
            in_flight = DEPTH;
            lds_store_unseen(landed_address, landed);
        }
        for (uint32_t i = head; i < copies; i++) {  // only with DEPTH copies in flight (head = kDmaHead < copies)
            // the oldest copy in flight has landed: say so, then take its place in the queue
            __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH - 1));
            lds_store_unseen(landed_address, ++landed);
            copy(i);
        }
        for (uint32_t left = in_flight; left > 0u; left--) {
            wait_copies_in_flight(left - 1u);
            lds_store_unseen(landed_address, ++landed);
        }
        // nothing of this wave is in flight any more: ordinary LDS reads from here on
        if (late != 0u) {
            lds_await(lds_address(&control->staged), kDmaConsumers, patience);
#pragma unroll
            for (int m = 0; m < M; m++) T::load_activations(stage[m], lane_id, active, xr[m]);
            for (uint32_t r = count - late; r < count; r++) {
                typename T::Data data;
                T::load(range + r * row_bytes, lane, data);
                fold_row(r, data);
            }
        }
        return;
    }

    // ---- consumers ------------------------------------------------------------------------------
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int i = 0; i < NI; i++) stage_quad(stage[m], xv[m][i], threadIdx.x + i * 64u * kDmaConsumers);
    lds_arrive(lds_address(&control->staged), lane_id == 0);
    lds_await(lds_address(&control->staged), kDmaConsumers, patience);
#pragma unroll
    for (int m = 0; m < M; m++) T::load_activations(stage[m], lane_id, active, xr[m]);

    const uint32_t landed_address = lds_address(&control->landed[pair]);
    // Row r needs the copies that hold bytes [0, (r + 1) * row_bytes) of the range. (Reading row r + 1
    // out of LDS ahead of the fold of row r, when it has landed by then, measured slower: the consumers
    // are bound by their arithmetic, two of them and two loaders to a SIMD, not by LDS latency.)
    const uint32_t mine = count - late;  // the last rows are the loader's
    for (uint32_t r = 0; r < mine; r++) {
        lds_await(landed_address, ((r + 1u) * row_bytes + 1023u) >> 10, patience);
        typename T::Data data;
        T::load(range + r * row_bytes, lane, data);
        fold_row(r, data);
    }
}

// The same split of the work with the copies taken in turn (the 4-, 5- and 8-bit codecs): the
// workgroup's share of W is ONE image in LDS, exactly as it lies in memory, whose 1 KiB copies the
// loaders take in turn (copy i is loader i % LOADERS's), so the image lands front to back at the rate of
// all loaders together. Rows are not tied to waves: a consumer that is free takes the next row from a
// counter in LDS, waits until the row's last byte has landed (one poll reads all the loaders' words) and
// folds it. The loaders do nothing but copy: a launch whose loaders read the staged activations while
// their first copies are on the way, to fold a row each at the end, measured half a microsecond slower
// than one whose loaders only copy - and such a launch, with its consumers switched off, runs as fast
// as the same copies alone (Q4_K 14336 x 4096: 6.2 - 6.6 us). What the launch waits for is its folds:
// they start when the activations are in registers (1.3 us after the barrier) and then keep the vector
// ALU busy for about 70 % of the time, so eleven of the sixteen waves fold and five copy, six copies in
// flight each (8 + 8 x 4: 8.2 - 8.4 us, 11 + 5 x 6: 7.9 - 8.1 on the same box; Q4_0 11008 x 4096: 7.1 -> 6.5).
template <class T, int M, int CONSUMERS, int LOADERS, int DEPTH>
__global__ __launch_bounds__(64 * (CONSUMERS + LOADERS)) void gemv_limb_turns_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t rows_per_wg, uint32_t spin_limit, uint32_t* timeouts) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr uint32_t kStageAt = kDmaControlAt - M * static_cast<uint32_t>(sizeof(StageMemory));
    constexpr int kStagers = 8;                            // consumer waves that prepare the activations
    constexpr int NI = kSliceQuads / (64 * kStagers);      // float4s per such thread and vector
    static_assert(DEPTH >= 1 && DEPTH <= 8, "wait_copies_in_flight counts to seven");
    static_assert(CONSUMERS >= kStagers && LOADERS <= kDmaPairs, "eight waves stage; DmaControl has eight loader words");
    DmaControl* control = reinterpret_cast<DmaControl*>(lds + kDmaControlAt);
    StageMemory* stage = reinterpret_cast<StageMemory*>(lds + kStageAt);
    Patience patience{spin_limit, timeouts};  // every wait on another wave is bounded (lds_handover.h)

    const uint32_t lane_id = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wg_row0 = blockIdx.x * rows_per_wg;
    if (wg_row0 >= rows) return;
    const uint32_t wg_rows = min(rows_per_wg, rows - wg_row0);
    const uint32_t row_bytes = static_cast<uint32_t>(T::row_bytes(columns));
    const uint32_t bytes = wg_rows * row_bytes;
    const uint32_t chunk = lane_id;  // one slice: the lane's 64-column stretch of the row
    const bool active = chunk < columns / kChunk;
    const uint32_t staged_address = lds_address(&control->staged);
    const uint32_t next_row_address = lds_address(&control->pad[0]);

    if (wave >= static_cast<uint32_t>(CONSUMERS)) {
        // ---- loaders ------------------------------------------------------------------------
        const uint32_t loader = wave - CONSUMERS;
        const uint32_t copies = (bytes + 1023u) >> 10;
        const uint32_t mine = copies > loader ? (copies - loader + LOADERS - 1u) / LOADERS : 0u;
        const uint8_t* source = weight + static_cast<uint64_t>(wg_row0) * row_bytes + lane_id * 16u;
        const uint32_t landed_address = lds_address(&control->landed[loader]);
        uint32_t at = loader * 1024u;  // of this loader's next copy in the image
        const auto copy = [&]() {
            if (at + lane_id * 16u < bytes)  // the last copy of the image stops where the share ends
                // streamed once: non-temporal (aux bit 1), the caches keep nothing of it
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(source + at),
                                                 reinterpret_cast<uint4*>(lds + at), 16, 0, 2);
            at += LOADERS * 1024u;
        };
        // The first copies wait for the barrier, i.e. until the consumers have issued their activation
        // loads: issued ahead of it they delay those loads, and with them every fold.
        __syncthreads();
        const uint32_t head = min(mine, static_cast<uint32_t>(DEPTH));
        for (uint32_t i = 0; i < head; i++) copy();
        uint32_t landed = 0;
        for (uint32_t i = head; i < mine; i++) {  // only with DEPTH copies in flight
            // the oldest copy in flight has landed: say so, then take its place in the queue
            __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH - 1));
            lds_store_unseen(landed_address, ++landed);
            copy();
        }
        for (uint32_t left = head; left > 0u; left--) {
            wait_copies_in_flight(left - 1u);
            lds_store_unseen(landed_address, ++landed);
        }
        return;
    }

    // ---- consumers ------------------------------------------------------------------------------
    {
        // Activation loads go first: nothing of the consumers' may queue behind a copy.
        float4 xv[M][NI];
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const uint32_t quad = threadIdx.x + i * 64u * kStagers;
                xv[m][i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (wave < kStagers && quad < (columns >> 2))
                    xv[m][i] = reinterpret_cast<const float4*>(x + m * x_row_stride)[quad];
            }
        if (threadIdx.x < 16) reinterpret_cast<uint32_t*>(control)[threadIdx.x] = 0u;
        __syncthreads();  // the only barrier: the counters are zero before anybody counts
        if (wave < kStagers) {
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int i = 0; i < NI; i++) stage_quad(stage[m], xv[m][i], threadIdx.x + i * 64u * kStagers);
            lds_arrive(staged_address, lane_id == 0);
        }
        if (!lds_await(staged_address, kStagers, patience)) return;
    }

    // ---- take a row, wait for it, fold it -------------------------------------------------------
    const typename T::Lane lane = T::lane_setup(active ? chunk : 0u);
    XLimbs xr[M];
#pragma unroll
    for (int m = 0; m < M; m++) T::load_activations(stage[m], lane_id, active, xr[m]);
    for (;;) {
        const uint32_t r = lds_take(next_row_address, lane_id == 0);
        if (r >= wg_rows) break;
        if (!await_copies_in_turn<LOADERS>(control->landed, lane_id, ((r + 1u) * row_bytes + 1023u) >> 10, patience)) break;
        typename T::Data data;
        T::load(lds + r * row_bytes, lane, data);
        float value[M];
        T::template fold<M>(data, lane, xr, value);
        const uint32_t row = wg_row0 + r;
        const float b = bias != nullptr ? bias[row] : 0.f;
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float total = wave_sum(active ? value[m] : 0.f);
            if (lane_id == 0) y[static_cast<uint64_t>(m) * rows + row] = bias != nullptr ? total + b : total;
        }
    }
}

// Whether gemv_limb_dma_kernel takes this shape: one slice of columns, a share per compute unit that
// fits LDS below the activation stages, enough rows per share to occupy the consumers.
template <class T, int M>
bool dma_takes(uint32_t rows, uint32_t columns, uint32_t* rows_per_wg) {
    if (columns > kSliceColumns) return false;
    const uint32_t share = (rows + 255u) / 256u;
    // With fewer than four rows to a range gemv_limb_kernel, which has all of them in flight from its
    // first instructions, is the faster one (Q8_0 4096 x 4096, two rows to a range: 5.1 against 5.5 us).
    if (share < 4u * kDmaPairs) return false;
    const uint64_t row_bytes = (static_cast<uint64_t>(columns) / T::kBlockColumns) * T::kBlockBytes;
    // A loader lane copies 16 bytes: rows that are not whole 16-byte pieces (Q2_K unless columns % 1024 == 0,
    // Q4_0 / Q8_0 unless columns % 256 == 0) would let the last lane of a range read up to 12 bytes past it -
    // for the last range of the matrix, past the weight buffer. Those widths stay on gemv_limb_kernel,
    // which reads exact dwords.
    if (row_bytes % 16u != 0u) return false;
    const uint64_t per_pair = (share + kDmaPairs - 1u) / kDmaPairs;
    const uint64_t range_bytes = ((per_pair * row_bytes + 1023u) / 1024u) * 1024u;  // as laid out in LDS
    const uint64_t stage_at = kDmaControlAt - M * sizeof(StageMemory);
    if (range_bytes * kDmaPairs > stage_at) return false;
    *rows_per_wg = share;
    return true;
}

template <class T, int M>
hipError_t launch_dma(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias,
                      float* y, uint32_t rows, uint32_t columns, uint32_t rows_per_wg, hipStream_t stream) {
    static std::atomic<bool> allowed[64];
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    HandoverState handover;
    if (hipError_t status = handover_state(&handover)) return status;
    const uint32_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
    const auto go = [&](auto kernel, uint32_t threads) -> hipError_t {
        if (!allowed[device].load(std::memory_order_acquire)) {
            if (hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, kDmaLdsBytes))
                return status;
            allowed[device].store(true, std::memory_order_release);
        }
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), kDmaLdsBytes, stream, weight, x, x_row_stride, bias, y,
                           rows, columns, rows_per_wg, handover.limit, handover.timeouts);
        return hipGetLastError();
    };
    if constexpr (T::kCopiesInTurn)
        return go(gemv_limb_turns_kernel<T, M, kTurnConsumers, kTurnLoaders, kTurnDepth>, kDmaThreads);
    else
        return go(gemv_limb_dma_kernel<T, M, kDmaDepth>, kDmaThreads);
}

template <class T, int M, int R, int WAVES, int NK, bool LOOP>
hipError_t launch(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias,
                  float* y, uint32_t rows, uint32_t columns, uint32_t rows_per_wg, hipStream_t stream) {
    const uint32_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL((gemv_limb_kernel<T, M, R, WAVES, NK, LOOP>), dim3(grid), dim3(64 * WAVES), 0,
                       stream, weight, x, x_row_stride, bias, y, rows, columns, rows_per_wg);
    return hipGetLastError();
}

// Picks rows per workgroup and the single-shot depth for WAVES / NK row groups.
template <class T, int M, int WAVES, int NK>
hipError_t launch_rows(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias,
                       float* y, uint32_t rows, uint32_t columns, hipStream_t stream) {
    constexpr uint32_t RG = WAVES / NK;
    // One contiguous range of rows per CU; a wave takes ceil(range / RG) of them.
    const uint32_t share = (rows + 255u) / 256u;
    const uint32_t depth = (share + RG - 1) / RG;
    // Registers bound the single-shot depth: 4 rows with more than 8 waves (128 VGPRs), else 8.
    constexpr uint32_t kMaxDepth = (WAVES > 8 || M > 1) ? 4 : 8;
#define ET_SHOT(D)                                                                               \
    case D:                                                                                      \
        return launch<T, M, D, WAVES, NK, false>(weight, x, x_row_stride, bias, y, rows, columns, \
                                                 RG * D, stream)
    if (depth <= kMaxDepth) {
        switch (depth) {
            ET_SHOT(1);
            ET_SHOT(2);
            ET_SHOT(3);
            ET_SHOT(4);
            default: break;
        }
        if (kMaxDepth == 8) {
            switch (depth) {
                case 5: return launch<T, M, (kMaxDepth == 8 ? 5 : 1), WAVES, NK, false>(weight, x, x_row_stride, bias, y, rows, columns, RG * 5, stream);
                case 6: return launch<T, M, (kMaxDepth == 8 ? 6 : 1), WAVES, NK, false>(weight, x, x_row_stride, bias, y, rows, columns, RG * 6, stream);
                case 7: return launch<T, M, (kMaxDepth == 8 ? 7 : 1), WAVES, NK, false>(weight, x, x_row_stride, bias, y, rows, columns, RG * 7, stream);
                case 8: return launch<T, M, (kMaxDepth == 8 ? 8 : 1), WAVES, NK, false>(weight, x, x_row_stride, bias, y, rows, columns, RG * 8, stream);
                default: break;
            }
        }
    }
#undef ET_SHOT
    // Too many rows per wave for registers: loop with two 2-row buffers.
    const uint32_t rows_per_wg = ((share + RG * 2 - 1) / (RG * 2)) * (RG * 2);
    return launch<T, M, 2, WAVES, NK, true>(weight, x, x_row_stride, bias, y, rows, columns,
                                            rows_per_wg, stream);
}

template <class T, int M>
hipError_t launch_slices(const uint8_t* weight, const float* x, uint64_t x_row_stride,
                         const float* bias, float* y, uint32_t rows, uint32_t columns,
                         hipStream_t stream) {
    const uint32_t slices = (columns + kSliceColumns - 1) / kSliceColumns;
    if constexpr (T::kLdsCopies && M == 1) {  // more vectors need more registers than sixteen waves leave
        uint32_t rows_per_wg = 0;
        if (gemv_limb_dma_enabled() && dma_takes<T, M>(rows, columns, &rows_per_wg))
            return launch_dma<T, M>(weight, x, x_row_stride, bias, y, rows, columns, rows_per_wg, stream);
    }
    if (slices <= 1) {
        return launch_rows<T, M, 8, 1>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    }
    if (slices <= 2) return launch_rows<T, M, 8, 2>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (slices <= 4) return launch_rows<T, M, 8, 4>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (slices <= 8) return launch_rows<T, M, 8, 8>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    return launch_rows<T, M, 16, 16>(weight, x, x_row_stride, bias, y, rows, columns, stream);
}

template <class T>
hipError_t launch_vectors(const uint8_t* weight, const float* x, uint64_t x_row_stride,
                          const float* bias, float* y, uint32_t rows, uint32_t columns,
                          uint32_t vectors, hipStream_t stream) {
    switch (vectors) {
        case 1: return launch_slices<T, 1>(weight, x, x_row_stride, bias, y, rows, columns, stream);
        case 2: return launch_slices<T, 2>(weight, x, x_row_stride, bias, y, rows, columns, stream);
        case 3: return launch_slices<T, 3>(weight, x, x_row_stride, bias, y, rows, columns, stream);
        default: return hipErrorInvalidValue;
    }
}

// One or two vectors per launch (the codecs whose lanes own four runs).
template <class T>
hipError_t launch_pair(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias, float* y,
                       uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
    if (vectors == 1) return launch_slices<T, 1>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (vectors == 2) return launch_slices<T, 2>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    return hipErrorInvalidValue;
}

}  // namespace

uint32_t gemv_limb_max_vectors(int32_t codec) {
    // Q2_K, Q3_K and Q6_K keep 62 and more registers of activation state per vector (48 limb words,
    // 12 dot offsets, 2 units, run sums): three vectors do not fit next to the rows in flight.
    return codec == kQ6_K || codec == kQ3_K || codec == kQ2_K ? 2u : kGemvLimbMaxVectors;
}

bool gemv_limb_copies_through_lds(int32_t codec, uint64_t rows, uint64_t columns, uint32_t vectors) {
    if (vectors != 1 || rows > 0xffffffffull || columns > kSliceColumns || !gemv_limb_dma_enabled()) return false;
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns);
    uint32_t rows_per_wg = 0;
    switch (codec) {
        case kQ4_K: return dma_takes<Q4KLimb, 1>(n, k, &rows_per_wg);
        case kQ5_K: return dma_takes<Q5KLimb, 1>(n, k, &rows_per_wg);
        case kQ4_0: return dma_takes<Q40Limb, 1>(n, k, &rows_per_wg);
        case kQ8_0: return dma_takes<Q80Limb, 1>(n, k, &rows_per_wg);
        case kQ2_K: return dma_takes<Q2KLimb, 1>(n, k, &rows_per_wg);
        default: return false;
    }
}

bool gemv_limb_supported(int32_t codec, uint64_t columns, uint32_t vectors) {
    if (vectors == 0 || vectors > gemv_limb_max_vectors(codec) || columns == 0 || columns > 65536u) return false;
    if (codec == kQ2_K || codec == kQ3_K || codec == kQ4_K || codec == kQ5_K || codec == kQ6_K) return columns % 256 == 0;
    if (codec == kQ4_0 || codec == kQ8_0) return columns % 64 == 0;
    return false;
}

hipError_t gemv_limb(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                     const float* bias, float* y, uint64_t rows, uint64_t columns, uint32_t vectors,
                     hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns);
    switch (codec) {
        case kQ4_K: return launch_vectors<Q4KLimb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ5_K: return launch_vectors<Q5KLimb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ6_K: return launch_pair<Q6KLimb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ3_K: return launch_pair<Q3KLimb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ2_K: return launch_pair<Q2KLimb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ4_0: return launch_vectors<Q40Limb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        case kQ8_0: return launch_vectors<Q80Limb>(weight, x, x_row_stride, bias, y, n, k, vectors, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
