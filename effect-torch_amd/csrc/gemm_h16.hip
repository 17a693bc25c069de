// f32-accurate contraction of Q4_K or Q5_K weights with a batch of activation vectors on the gfx950
// matrix cores, with every operand an exact small integer held in a half float.
//
//   y[m, n] = sum_s  unit[m, s] * d[n, s] * sum_g sum_i (sc_g[n] * nib[n, g, i]) * X[m, g, i]
//           - sum_s  dmin[n, s] * sum_g m_g[n] * xsum[m, g]
// s = 256-column stage (one Q4_K super-block), g = its eight 32-column sub-blocks.
//
// Activations are 24-bit fixed point per vector and stage, X = rint(x * (2^23 - 1) / max|x|), split
// into two balanced 12-bit halves X = 4096 * hi + lo with |lo|, |hi| <= 2048: integers a half float
// holds exactly. The tiles hold hi and lo / 4096 (exact as well: a power of two), so that both halves
// of a sub-block add up in ONE accumulator, hi * w + (lo / 4096) * w = X * w / 4096, and the factor
// 4096 rides on the row scale: one multiply-add per element and stage in the epilogue. On the weight side the 6-bit sub-block scale is folded into the operand:
// sc_g * nib <= 63 * 15 = 945 (Q5_K: 63 * 31 = 1953), exact in a half float as well. Every product (< 2^21) is exact in
// the f32 the matrix core accumulates in, so v_mfma_f32_32x32x16_f16 sums whole super-blocks with
// f32 accumulation error only, and the f32 scales unit[m] * d[n] are applied once per stage instead
// of once per 32-column block: the per-element VALU work, which bounds the int8 kernel with
// three-byte activations (gemm_i8.hip: a convert and multiply-adds per element and block), shrinks
// by the eight blocks of a stage. The contraction computed is linear_into's
// (crates/runtime-cpu/src/quantized.rs:419-499); the reference's own batch kernel decodes weights
// to f32 and uses f32 simdgroup MMA (crates/runtime-metal/src/quantized.rs:1016-1097).
//
// Tiling, operand streams and barriers are those of gemm_i8.hip: a workgroup owns 64 weight rows x
// 32 vectors and walks K in stages; eight consumer waves (four share a 32-row group and split the
// eight sub-blocks of a stage), two loader waves per operand stream that only issue
// global_load_lds copies into LDS rings, one s_barrier per stage.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <type_traits>

#include "decode_math.h"
#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kStageBlocks = 8;
constexpr int kConsumers = 8;
constexpr int kWeightLoaders = 2;
constexpr int kActivationLoaders = 2;
constexpr int kLoaders = kWeightLoaders + kActivationLoaders;
constexpr int kThreads = 64 * (kConsumers + kLoaders);
// RG = 32-row groups per workgroup (2 or 4): the eight consumers are RG groups of 8 / RG waves that
// split the eight sub-blocks of a stage, RG each. Four groups (128 rows) halve the activation bytes a
// workgroup copies per weight row; two groups (64 rows) make twice as many workgroups.
// NARROW = at most sixteen vectors: see Operands.

constexpr float kPlaneRatio = 4096.0f;          // what the accumulators lack: the tiles hold hi and lo / 4096
constexpr uint32_t kBlob = tile_blob_bytes(2);  // in memory and in LDS
constexpr uint32_t kUnitAt = 32768u;            // unit[m]
constexpr uint32_t kSumsAt = 32768u + 128u;     // xsum[g][m]
constexpr int kActivationJobs = kBlob / 1024;
static_assert(kBlob % 1024 == 0, "whole copy instructions");

// (scale, min) of Q4_K sub-block g (crates/runtime-cpu/src/quantized.rs:77-86).
__device__ __forceinline__ void q4k_scale_min(const uint4& header, uint32_t g, uint32_t& sc, uint32_t& mn) {
    const uint32_t shift = 8u * (g & 3u);
    const uint32_t s0 = (header.y >> shift) & 0xffu;
    const uint32_t s1 = (header.z >> shift) & 0xffu;
    const uint32_t s2 = (header.w >> shift) & 0xffu;
    sc = g < 4 ? (s0 & 63u) : ((s2 & 0x0fu) | ((s0 >> 6) << 4));
    mn = g < 4 ? (s1 & 63u) : ((s2 >> 4) | ((s1 >> 6) << 4));
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) {
    return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8);
}

// A row's share of a stage, as it lies in memory: a Q4_K super-block is d, dmin, scales[12], qs[128];
// a Q5_K one d, dmin, scales[12], qh[32] (the fifth bits: bit g of qh[c] belongs to column c of
// sub-block g), qs[128] (crates/runtime-cpu/src/quantized.rs:180-234).
// Super-blocks whose size is not a multiple of sixteen (Q6_K: 210 bytes = ql[128], qh[64], sixteen int8
// scales, d; Q3_K: 110 = hmask[32], qs[64], scales[12], d; Q2_K: 84 = scales[16], qs[64], d, dmin;
// crates/runtime-cpu/src/quantized.rs:117-176, 238-261) get an LDS row of the next multiple: every
// 16-byte chunk holds the stage's bytes at the same offset except the last one, which is taken from the
// stage's last sixteen bytes - so no copy reads past the stage (or the weight buffer). Q3_K and Q6_K
// stages start on 2-byte boundaries; global_load_lds takes such sources, more slowly.
template <int CODEC>
struct Codec {
    static_assert(CODEC == kQ2_K || CODEC == kQ3_K || CODEC == kQ4_K || CODEC == kQ5_K || CODEC == kQ6_K,
                  "the K-quants");
    static constexpr uint32_t kStageBytes = block_bytes(CODEC);            // in memory
    static constexpr uint32_t kRowBytes = (kStageBytes + 15u) / 16u * 16u;  // in LDS
    static constexpr uint32_t kQuantsAt = CODEC == kQ5_K ? 48u : 16u;       // Q4_K / Q5_K
    // where the stage's last sixteen bytes lie in the LDS row: d (and dmin) are read from there
    static constexpr uint32_t kTailAt = kRowBytes - 16u, kTailFrom = kStageBytes - 16u;
    // byte of the stage that LDS byte `within` (a multiple of 16) of the row holds
    static __device__ __forceinline__ uint32_t source_of(uint32_t within) {
        return kRowBytes != kStageBytes && within == kTailAt ? kTailFrom : within;
    }
    // LDS offset of stage byte `at` of the tail
    static constexpr uint32_t in_tail(uint32_t at) { return kTailAt + (at - kTailFrom); }
};

template <int CODEC, int RG, int AX, int AW>
struct Shape {
    static constexpr uint32_t kRowBytes = Codec<CODEC>::kRowBytes;
    static constexpr int kRowGroups = RG, kSplit = kConsumers / RG, kBlocksPerWave = kStageBlocks / kSplit;
    static constexpr uint32_t kRows = 32 * RG;
    static constexpr uint32_t kWeightBytes = kRows * kRowBytes;
    static constexpr int kWeightJobs = kWeightBytes / 1024;
    static_assert(kWeightBytes % 1024 == 0, "whole copy instructions");
    static constexpr int kActivationDepth = AX + 1, kWeightDepth = AW + 1;
    static constexpr uint32_t kWeightRingAt = kActivationDepth * kBlob;
    static constexpr uint32_t kRingBytes = kWeightRingAt + kWeightDepth * kWeightBytes;
    static constexpr int kActivationRounds = (kActivationJobs + kActivationLoaders - 1) / kActivationLoaders;
    static constexpr int kWeightRounds = (kWeightJobs + kWeightLoaders - 1) / kWeightLoaders;
    static constexpr int kActivationWait = (AX - 1) * kActivationRounds < 63 ? (AX - 1) * kActivationRounds : 63;
    static constexpr int kWeightWait = (AW - 1) * kWeightRounds < 63 ? (AW - 1) * kWeightRounds : 63;
    static constexpr uint32_t kExchangeBytes = (kSplit - 1) * kRowGroups * 16 * 64 * 4;
    static constexpr uint32_t kLdsBytes = kRingBytes > kExchangeBytes ? kRingBytes : kExchangeBytes;
};

// Eight nibbles (two dwords of four, one per byte) as eight half floats times `scale`:
// 0x6400 | n is the half float 1024 + n, and (1024 + n) * scale - 1024 * scale, one fused
// multiply-add per pair, is n * scale exactly (1024 * scale <= 64512 is a half float).
template <int OFFSET = 0>
__device__ __forceinline__ v8h nibbles_times(uint32_t first, uint32_t second, v2h scale) {
    // OFFSET is subtracted from every byte first: (1024 + n) * scale - (1024 + OFFSET) * scale
    const v2h offset = {static_cast<_Float16>(1024.0f + OFFSET), static_cast<_Float16>(1024.0f + OFFSET)};
    union {
        uint32_t word[4];
        v2h pair[4];
        v8h all;
    } u;
    u.word[0] = __builtin_amdgcn_perm(0x64646464u, first, 0x04010400u);   // bytes 0, 1
    u.word[1] = __builtin_amdgcn_perm(0x64646464u, first, 0x04030402u);   // bytes 2, 3
    u.word[2] = __builtin_amdgcn_perm(0x64646464u, second, 0x04010400u);
    u.word[3] = __builtin_amdgcn_perm(0x64646464u, second, 0x04030402u);
#pragma unroll
    for (int i = 0; i < 4; i++) u.pair[i] = __builtin_elementwise_fma(u.pair[i], scale, -(offset * scale));
    return u.all;
}

// The matrices of one launch: contractions that share their activations (the q / k / v projections
// of a decode step) run as one grid over the row tiles of all of them.
struct Member {
    const uint8_t* weight;
    const float* bias;
    const float* residual;
    float* y;
    uint32_t rows;
    uint32_t first_tile;  // of the launch's row tiles
};
struct Group {
    Member member[kGemmGroupMost];
    uint32_t count;
    uint32_t row_tiles;  // of all members together
};

// Eight bytes as eight half floats, (n - OFFSET) * scale in two exact steps (for offsets whose product
// with the scale a half float does not hold: 1028 * 31).
template <int OFFSET>
__device__ __forceinline__ v8h bytes_minus_times(uint32_t first, uint32_t second, v2h scale) {
#pragma clang fp contract(off)
    const v2h offset = {static_cast<_Float16>(1024.0f + OFFSET), static_cast<_Float16>(1024.0f + OFFSET)};
    union {
        uint32_t word[4];
        v2h pair[4];
        v8h all;
    } u;
    u.word[0] = __builtin_amdgcn_perm(0x64646464u, first, 0x04010400u);
    u.word[1] = __builtin_amdgcn_perm(0x64646464u, first, 0x04030402u);
    u.word[2] = __builtin_amdgcn_perm(0x64646464u, second, 0x04010400u);
    u.word[3] = __builtin_amdgcn_perm(0x64646464u, second, 0x04030402u);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const v2h centred = u.pair[i] - offset;
        u.pair[i] = centred * scale;
    }
    return u.all;
}

// The activation operands of sub-block b for one lane (matrix row i = in_half, K group = half), two per
// 16-column chunk in the order they are contracted: low and high plane of vector i - or, NARROW (at most
// sixteen vectors), one: rows 0-15 of the matrix are the high plane of vectors 0-15 and rows 16-31 their
// low plane, so one instruction contracts both planes and the two halves of the result are added once
// per stage.
template <bool NARROW>
struct Operands {
    static constexpr int kPlanes = NARROW ? 1 : 2;
    v8h x[2 * kPlanes];
    __device__ __forceinline__ void load(const uint8_t* slot, uint32_t b, uint32_t half, uint32_t in_half) {
        if constexpr (NARROW) {
            const uint8_t* chunk = slot + ((2u * b + half) * 2u) * 512u + (in_half & 15u) * 16u +
                                   (in_half < 16u ? 16384u : 0u);
            x[0] = *reinterpret_cast<const v8h*>(chunk);
            x[1] = *reinterpret_cast<const v8h*>(chunk + 512u);
        } else {
            const uint8_t* chunk = slot + ((2u * b + half) * 2u) * 512u + in_half * 16u;
            x[0] = *reinterpret_cast<const v8h*>(chunk);
            x[1] = *reinterpret_cast<const v8h*>(chunk + 16384u);
            x[2] = *reinterpret_cast<const v8h*>(chunk + 512u);
            x[3] = *reinterpret_cast<const v8h*>(chunk + 16384u + 512u);
        }
    }
    // p += x * (b0 for the first chunk, b1 for the second)
    __device__ __forceinline__ v16f contract(v8h b0, v8h b1, v16f p) const {
#pragma unroll
        for (int i = 0; i < kPlanes; i++) p = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[i], b0, p, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < kPlanes; i++) p = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[kPlanes + i], b1, p, 0, 0, 0);
        return p;
    }
};
// What a stage adds for accumulator r of a lane: the product sum itself, or both planes' halves of it.
template <bool NARROW>
__device__ __forceinline__ float stage_sum(const v16f& p, int r) {
    if constexpr (NARROW) return p[r] + p[r + 8];
    return p[r];
}

// PROBE (measurement only, et_hip_calibration_contraction; results are then meaningless): the same
// kernel with its consumers' arithmetic, or some of its copies, left out - every wave, barrier and
// wait stays.
enum : int { kProbeNone = 0, kProbeNoArithmetic = 1, kProbeNoCopies = 2, kProbeNoWeightCopies = 3, kProbeNoActivationCopies = 4,
              kProbeWeightCopiesOnly = 5, kProbeActivationCopiesOnly = 6 };

template <int CODEC, int RG, int AX, int AW, bool NARROW, int PROBE = kProbeNone>
__global__ __launch_bounds__(kThreads) void gemm_h16_kernel(
    const Group group, const uint8_t* __restrict__ tiles, uint32_t vector_tiles, uint32_t columns,
    uint32_t vectors, uint32_t k_splits, float* __restrict__ partials) {
    using S = Shape<CODEC, RG, AX, AW>;
    constexpr uint32_t kRowBytes = S::kRowBytes, kQuantsAt = Codec<CODEC>::kQuantsAt, kStageBytes = Codec<CODEC>::kStageBytes;
    constexpr int NB = S::kBlocksPerWave;
    constexpr int kSplit = S::kSplit, kRowGroups = S::kRowGroups, kWeightJobs = S::kWeightJobs;
    constexpr uint32_t kRows = S::kRows, kWeightBytes = S::kWeightBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // Workgroups go to the eight XCDs round-robin; all vector tiles and K shares of one row tile
    // run on the same XCD, next to each other in time, so the later ones find the weights in L2.
    const uint32_t xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
    const uint32_t units = vector_tiles * k_splits;
    const uint32_t row_tile = (turn / units) * 8u + xcd;
    const uint32_t tile = (turn % units) % vector_tiles;
    const uint32_t k_share = (turn % units) / vector_tiles;
    if (row_tile >= group.row_tiles) return;
    uint32_t which = 0;
    for (uint32_t i = 1; i < group.count; i++)
        if (row_tile >= group.member[i].first_tile) which = i;
    const Member& member = group.member[which];
    const uint8_t* __restrict__ weight = member.weight;
    const uint32_t rows = member.rows;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t all_stages = columns / 256u;
    const uint32_t share = (all_stages + k_splits - 1u) / k_splits;
    const uint32_t first_stage = k_share * share;  // < all_stages: the launcher leaves no share empty
    const uint32_t stages = min(share, all_stages - first_stage);
    const uint64_t row_bytes = static_cast<uint64_t>(all_stages) * kStageBytes;
    const uint32_t row0 = (row_tile - member.first_tile) * kRows;  // in the member's own rows

    if (wave >= static_cast<uint32_t>(kConsumers + kWeightLoaders)) {
        // ---- activation loaders: linear copies of the stage's blob ----
        const uint32_t loader = wave - (kConsumers + kWeightLoaders);
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);  // past the end: a copy nobody reads
            uint8_t* slot = lds + (stage % S::kActivationDepth) * kBlob;
            const uint8_t* blob = tiles + (static_cast<uint64_t>(first_stage + s) * vector_tiles + tile) * kBlob;
#pragma unroll
            for (int i = 0; i < S::kActivationRounds; i++) {
                uint32_t job = i * kActivationLoaders + loader;
                if (job >= static_cast<uint32_t>(kActivationJobs)) job -= kActivationJobs;
                if constexpr (PROBE == kProbeNoCopies || PROBE == kProbeNoActivationCopies || PROBE == kProbeWeightCopiesOnly) continue;
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(blob + job * 1024u + lane * 16u),
                                                 reinterpret_cast<uint4*>(slot + job * 1024u), 16, 0, 0);
            }
        };
        // Stage 0 on its own: a wave that issues copies into a full memory queue is held there, and with
        // the whole lead requested first this wave reached the first barrier long after stage 0 had landed.
        // (The same for the weight loaders measured no different; 14336 x 4096 with 32 vectors 22.0 -> 21.5 us,
        // 28672 x 4096 33.2 -> 32.2, 4096 x 4096 14.45 -> 14.15.)
        request(0);
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
        __builtin_amdgcn_s_barrier();
        for (uint32_t a = 1; a <= static_cast<uint32_t>(AX); a++) request(a);
        for (uint32_t stage = 1; stage < stages; stage++) {
            __builtin_amdgcn_s_waitcnt(vmcnt_only(S::kActivationWait));  // all but the newest AX - 1 requests
            __builtin_amdgcn_s_barrier();  // "stage is in LDS" / "the slots of stage - 1 are free"
            request(stage + AX);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));  // nothing may still write the ring
        __builtin_amdgcn_s_barrier();               // the consumers' two exchange barriers
        __builtin_amdgcn_s_barrier();
        return;
    }
    if (wave >= static_cast<uint32_t>(kConsumers)) {
        // ---- weight loaders: the stage's bytes of the 64 rows, row after row as in memory ----
        const uint32_t loader = wave - kConsumers;
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);
            uint8_t* region = lds + S::kWeightRingAt + (stage % S::kWeightDepth) * kWeightBytes;
#pragma unroll
            for (int i = 0; i < S::kWeightRounds; i++) {
                uint32_t job = i * kWeightLoaders + loader;
                if (job >= static_cast<uint32_t>(kWeightJobs)) job -= kWeightJobs;
                const uint32_t at = job * 1024u + lane * 16u;
                const uint32_t row = min(row0 + at / kRowBytes, rows - 1u);
                const uint8_t* src = weight + row * row_bytes + static_cast<uint64_t>(first_stage + s) * kStageBytes +
                                     Codec<CODEC>::source_of(at % kRowBytes);
                if constexpr (PROBE == kProbeNoCopies || PROBE == kProbeNoWeightCopies || PROBE == kProbeActivationCopiesOnly) continue;
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                 reinterpret_cast<uint4*>(region + job * 1024u), 16, 0, 0);
            }
        };
        for (uint32_t a = 0; a < static_cast<uint32_t>(AW); a++) request(a);
        for (uint32_t stage = 0; stage < stages; stage++) {
            __builtin_amdgcn_s_waitcnt(vmcnt_only(S::kWeightWait));
            __builtin_amdgcn_s_barrier();
            request(stage + AW);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_s_barrier();
        return;
    }

    // ---- consumer waves ----
    const uint32_t half = lane >> 5, in_half = lane & 31u;
    const uint32_t wave_n = wave % kRowGroups;  // row group
    const uint32_t wave_k = wave / kRowGroups;  // share of the stage's sub-blocks
    const uint32_t n0 = row0 + wave_n * 32u;
    const uint32_t m0 = tile * 32u;
    constexpr int R = NARROW ? 8 : 16;  // vectors a lane accumulates: m = 8 (r / 4) + 4 half + r % 4
    float acc[R];
    v16f acc_min, zero;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        acc_min[r] = 0.f;
        zero[r] = 0.f;
    }
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    for (uint32_t stage = 0; stage < stages; stage++) {
        __builtin_amdgcn_s_barrier();
        const uint8_t* slot = lds + (stage % S::kActivationDepth) * kBlob;
        const uint8_t* region = lds + S::kWeightRingAt + (stage % S::kWeightDepth) * kWeightBytes;
        const uint32_t b_base = wave_k * NB;
        const uint8_t* row_in_slot = region + (wave_n * 32u + in_half) * kRowBytes;  // this lane's weight row
        if constexpr (PROBE == kProbeNoArithmetic || PROBE == kProbeWeightCopiesOnly || PROBE == kProbeActivationCopiesOnly) continue;

        if constexpr (CODEC == kQ3_K) {
            // value = d * (sc - 32) * (v - 4), v = two bits of qs | the hmask bit << 2, a 6-bit scale per 16
            // columns; |(sc - 32) * (v - 4)| <= 128 is exact in a half float. No minimum term.
            const float d_block = half_bits_to_float(*reinterpret_cast<const uint16_t*>(row_in_slot + Codec<CODEC>::in_tail(108u)));
            const float unit = *reinterpret_cast<const float*>(slot + kUnitAt + in_half * 4u);
            const uint4 hm = *reinterpret_cast<const uint4*>(row_in_slot + 16u * half);  // hmask of these columns
            v16f p = zero;
#pragma unroll
            for (int bb = 0; bb < NB; bb++) {
                const uint32_t b = b_base + bb, n = b >> 2, t = b & 3u;
                const uint4 qs = *reinterpret_cast<const uint4*>(row_in_slot + 32u + 32u * n + 16u * half);
                // scale of group 8 n + 2 t + half: nibble n of packed[2 t + half], top bits from packed[8 + ..]
                const uint32_t low_byte = row_in_slot[Codec<CODEC>::in_tail(96u) + 2u * t + half];
                const uint32_t high_byte = row_in_slot[Codec<CODEC>::in_tail(104u) + 2u * (t & 1u) + half];
                const int sc = static_cast<int>(((low_byte >> (4u * n)) & 15u) |
                                                (((high_byte >> (2u * (2u * n + (t >> 1)))) & 3u) << 4)) - 32;
                const uint32_t bit = 4u * n + t;
                const uint32_t w0 = ((qs.x >> (2u * t)) & 0x03030303u) | (((hm.x >> bit) & 0x01010101u) << 2),
                               w1 = ((qs.y >> (2u * t)) & 0x03030303u) | (((hm.y >> bit) & 0x01010101u) << 2),
                               w2 = ((qs.z >> (2u * t)) & 0x03030303u) | (((hm.z >> bit) & 0x01010101u) << 2),
                               w3 = ((qs.w >> (2u * t)) & 0x03030303u) | (((hm.w >> bit) & 0x01010101u) << 2);
                const _Float16 sc_h = static_cast<_Float16>(static_cast<float>(sc));
                const v2h sc2 = {sc_h, sc_h};
                const v8h b0 = bytes_minus_times<4>(w0, w1, sc2), b1 = bytes_minus_times<4>(w2, w3, sc2);
                Operands<NARROW> x;
                x.load(slot, b, half, in_half);
                p = x.contract(b0, b1, p);
            }
            const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? unit : 0.f, half == 0 ? kPlaneRatio * d_block : 0.f,
                                                                 zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] = fmaf(stage_sum<NARROW>(p, r), sd[r], acc[r]);
            continue;
        }
        if constexpr (CODEC == kQ2_K) {
            // value = d * sc * v - dmin * mn with a 4-bit scale and minimum per 16 columns. The minima ride
            // on the matrix cores too: a weight operand that is mn in all sixteen columns sums the
            // activations of the run times mn (acc_min is then the second pair of accumulators).
            const uint32_t dd = *reinterpret_cast<const uint32_t*>(row_in_slot + Codec<CODEC>::in_tail(80u));
            const float d_block = half_bits_to_float(dd & 0xffffu), dmin_block = half_bits_to_float(dd >> 16);
            const float unit = *reinterpret_cast<const float*>(slot + kUnitAt + in_half * 4u);
            v16f p = zero, m = zero;  // products, and the sums of the activations times the minima
#pragma unroll
            for (int bb = 0; bb < NB; bb++) {
                const uint32_t b = b_base + bb, n = b >> 2, t = b & 3u;
                const uint4 qs = *reinterpret_cast<const uint4*>(row_in_slot + 16u + 32u * n + 16u * half);
                const uint32_t both = row_in_slot[2u * b + half];  // scales[8 n + 2 t + half]
                const uint32_t w0 = (qs.x >> (2u * t)) & 0x03030303u, w1 = (qs.y >> (2u * t)) & 0x03030303u,
                               w2 = (qs.z >> (2u * t)) & 0x03030303u, w3 = (qs.w >> (2u * t)) & 0x03030303u;
                const _Float16 sc_h = static_cast<_Float16>(static_cast<float>(both & 15u));
                const _Float16 mn_h = static_cast<_Float16>(static_cast<float>(both >> 4));
                const v2h sc2 = {sc_h, sc_h};
                const v8h b0 = nibbles_times(w0, w1, sc2), b1 = nibbles_times(w2, w3, sc2);
                const v8h bm = {mn_h, mn_h, mn_h, mn_h, mn_h, mn_h, mn_h, mn_h};
                Operands<NARROW> x;
                x.load(slot, b, half, in_half);
                p = x.contract(b0, b1, p);
                m = x.contract(bm, bm, m);
            }
            const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? unit : 0.f, half == 0 ? kPlaneRatio * d_block : 0.f,
                                                                 zero, 0, 0, 0);
            const v16f sm = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? unit : 0.f, half == 0 ? kPlaneRatio * dmin_block : 0.f,
                                                                 zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < R; r++) {
                acc[r] = fmaf(stage_sum<NARROW>(p, r), sd[r], acc[r]);
                acc_min[r] = fmaf(stage_sum<NARROW>(m, r), sm[r], acc_min[r]);
            }
            continue;
        }
        if constexpr (CODEC == kQ6_K) {
            // value = d * sc * (q - 32) with an int8 scale per 16 columns: a lane half's sixteen columns
            // of a 32-column block are one such run. sc * (q - 32) reaches 4096, too wide for a half
            // float, so sc = 16 * s_hi + s_lo (s_lo 0..15, s_hi -8..7) and both parts are contracted:
            // four accumulators, (X_lo, X_hi) x (s_lo, s_hi), joined once per stage.
            const float d_block = half_bits_to_float(*reinterpret_cast<const uint16_t*>(row_in_slot + Codec<CODEC>::in_tail(208u)));
            const float unit = *reinterpret_cast<const float*>(slot + kUnitAt + in_half * 4u);
            v16f p_l = zero, p_h = zero;  // by scale part; both activation halves go into one sum
#pragma unroll
            for (int bb = 0; bb < NB; bb++) {
                const uint32_t b = b_base + bb, n = b >> 2, t = b & 3u;
                // columns 32 t + 16 half .. + 16 of 128-column half n: low four bits in ql[64 n + 32 (t & 1) + l]
                // (high nibbles for t >= 2), bits 4-5 in qh[32 n + l] >> 2 t, l = 16 half .. + 16
                const uint4 ql = *reinterpret_cast<const uint4*>(row_in_slot + 64u * n + 32u * (t & 1u) + 16u * half);
                const uint4 qh = *reinterpret_cast<const uint4*>(row_in_slot + 128u + 32u * n + 16u * half);
                const int sc = *reinterpret_cast<const int8_t*>(row_in_slot + 192u + 8u * n + 2u * t + half);
                const uint32_t low_shift = (t >> 1) * 4u, high_shift = 2u * t;
                const uint32_t w0 = ((ql.x >> low_shift) & 0x0f0f0f0fu) | (((qh.x >> high_shift) & 0x03030303u) << 4),
                               w1 = ((ql.y >> low_shift) & 0x0f0f0f0fu) | (((qh.y >> high_shift) & 0x03030303u) << 4),
                               w2 = ((ql.z >> low_shift) & 0x0f0f0f0fu) | (((qh.z >> high_shift) & 0x03030303u) << 4),
                               w3 = ((ql.w >> low_shift) & 0x0f0f0f0fu) | (((qh.w >> high_shift) & 0x03030303u) << 4);
                const _Float16 s_lo = static_cast<_Float16>(static_cast<float>(sc & 15));
                const _Float16 s_hi = static_cast<_Float16>(static_cast<float>(sc >> 4));
                const v2h lo2 = {s_lo, s_lo}, hi2 = {s_hi, s_hi};
                const v8h bl0 = nibbles_times<32>(w0, w1, lo2), bl1 = nibbles_times<32>(w2, w3, lo2);
                const v8h bh0 = nibbles_times<32>(w0, w1, hi2), bh1 = nibbles_times<32>(w2, w3, hi2);
                Operands<NARROW> x;
                x.load(slot, b, half, in_half);
                p_l = x.contract(bl0, bl1, p_l);
                p_h = x.contract(bh0, bh1, p_h);
            }
            const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? unit : 0.f, half == 0 ? kPlaneRatio * d_block : 0.f,
                                                                 zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < R; r++)
                acc[r] = fmaf(fmaf(16.0f, stage_sum<NARROW>(p_h, r), stage_sum<NARROW>(p_l, r)), sd[r], acc[r]);
            continue;
        }

        const uint4 header = *reinterpret_cast<const uint4*>(row_in_slot);
        const float d_scaled = kPlaneRatio * half_bits_to_float(header.x & 0xffffu);
        const float dmin_block = half_bits_to_float(header.x >> 16);
        uint4 fifth = make_uint4(0u, 0u, 0u, 0u);  // Q5_K: qh of this lane half's sixteen columns
        if constexpr (CODEC == kQ5_K) fifth = *reinterpret_cast<const uint4*>(row_in_slot + 16u + 16u * half);

        // min term: acc_min[m, n] += sum_g (dmin * m_g)[n] * xsum[m, g]; K = 2 per MFMA, lane half h
        // supplies sub-block 2j + h.
#pragma unroll
        for (int jj = 0; jj < NB / 2; jj++) {
            const uint32_t g = b_base + 2u * jj + half;
            uint32_t sc, mn;
            q4k_scale_min(header, g, sc, mn);
            const float a_operand = *reinterpret_cast<const float*>(slot + kSumsAt + g * 128u + in_half * 4u);
            acc_min = __builtin_amdgcn_mfma_f32_32x32x2f32(a_operand, dmin_block * static_cast<float>(mn), acc_min,
                                                           0, 0, 0);
        }

        // The stage's products: both halves of X against sc_g * nib, summed over this wave's sub-blocks.
        // The weight operands of sub-block bb + 1 are prepared (VALU) between the MFMAs of sub-block bb.
        const auto prepare = [&](int bb, v8h& b0, v8h& b1) {
            const uint32_t b = b_base + bb;
            // sub-block 2p + side: low (side 0) or high (side 1) nibbles of the 32 bytes of pair p; this
            // lane half takes bytes 16 * half .. + 16 = columns 16 * half .. + 16 of the sub-block
            const uint4 raw = *reinterpret_cast<const uint4*>(row_in_slot + kQuantsAt + 32u * (b >> 1) + 16u * half);
            const uint32_t shift = (b & 1u) * 4u;
            uint32_t w0 = (raw.x >> shift) & 0x0f0f0f0fu, w1 = (raw.y >> shift) & 0x0f0f0f0fu,
                     w2 = (raw.z >> shift) & 0x0f0f0f0fu, w3 = (raw.w >> shift) & 0x0f0f0f0fu;
            if constexpr (CODEC == kQ5_K) {  // the fifth bit of column c of sub-block b: bit b of qh[c]
                w0 |= ((fifth.x >> b) & 0x01010101u) << 4;
                w1 |= ((fifth.y >> b) & 0x01010101u) << 4;
                w2 |= ((fifth.z >> b) & 0x01010101u) << 4;
                w3 |= ((fifth.w >> b) & 0x01010101u) << 4;
            }
            uint32_t sc, mn;
            q4k_scale_min(header, b, sc, mn);
            const _Float16 sc_h = static_cast<_Float16>(static_cast<float>(sc));
            const v2h sc2 = {sc_h, sc_h};
            b0 = nibbles_times(w0, w1, sc2);
            b1 = nibbles_times(w2, w3, sc2);
        };
        v16f p = zero;
        v8h b0, b1;
        prepare(0, b0, b1);
#pragma unroll
        for (int bb = 0; bb < NB; bb++) {
            Operands<NARROW> x;
            x.load(slot, b_base + bb, half, in_half);
            p = x.contract(b0, b1, p);
            if (bb + 1 < NB) {
                v8h n0, n1;
                prepare(bb + 1, n0, n1);
                b0 = n0;
                b1 = n1;
                constexpr int kMatrix = 2 * Operands<NARROW>::kPlanes;
#pragma unroll
                for (int i = 0; i < kMatrix; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x002, 48 / kMatrix, 0);  // its share of the VALU work
                }
            }
        }
        // unit[m] * d[n] for the sixteen vectors this lane accumulates, m = 8 * (r / 4) + 4 * half + r % 4:
        // four 16-byte LDS reads that every lane of a half shares, sixteen multiplications. (The same
        // products as a rank-1 v_mfma_f32_32x32x2f32 in the result layout cost 64 cycles of the matrix
        // pipe, and matrix and VALU instructions do not run side by side on this device.)
        float sd[R];
#pragma unroll
        for (int j = 0; j < R / 4; j++) {
            const float4 units = *reinterpret_cast<const float4*>(slot + kUnitAt + (8u * j + 4u * half) * 4u);
            sd[4 * j + 0] = units.x * d_scaled;
            sd[4 * j + 1] = units.y * d_scaled;
            sd[4 * j + 2] = units.z * d_scaled;
            sd[4 * j + 3] = units.w * d_scaled;
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = fmaf(stage_sum<NARROW>(p, r), sd[r], acc[r]);
    }

    // ---- combine the sub-block shares, add bias, store ----
    __syncthreads();  // the loaders arrive here with nothing in flight: the ring is free
    float* exchange = reinterpret_cast<float*>(lds);  // [wave_k - 1][wave_n][16][64 lanes]
    if (wave_k > 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
            exchange[(((wave_k - 1u) * kRowGroups + wave_n) * 16 + r) * 64 + lane] = acc[r] - acc_min[r];
    }
    __syncthreads();
    if (wave_k > 0) return;
    const uint32_t n_out = n0 + in_half;
    const float* bias = member.bias;
    const float* residual = member.residual;
    float* y = member.y;
    const float bias_value = bias != nullptr && n_out < rows ? bias[n_out] : 0.f;
    const uint32_t launch_row = row_tile * kRows + wave_n * 32u + in_half;  // among the rows of all members
    const uint64_t launch_rows = static_cast<uint64_t>(group.row_tiles) * kRows;
#pragma unroll
    for (int r = 0; r < R; r++) {
        float value = acc[r] - acc_min[r];
#pragma unroll
        for (int k = 1; k < kSplit; k++) value += exchange[(((k - 1) * kRowGroups + wave_n) * 16 + r) * 64 + lane];
        const uint32_t m = m0 + 8u * (r >> 2) + 4u * half + (r & 3u);
        if (n_out < rows && m < vectors) {
            if (k_splits == 1) {
                // residual may be y itself: every output is read, then written, by this lane only
                const uint64_t at = static_cast<uint64_t>(m) * rows + n_out;
                y[at] = residual != nullptr ? (value + bias_value) + residual[at] : value + bias_value;
            } else {
                partials[(static_cast<uint64_t>(k_share) * vectors + m) * launch_rows + launch_row] = value;
            }
        }
    }
}

// y[m, n] = bias[n] + the K shares in share order (+ residual[m, n], which may be y itself), for every
// member of the launch; partials are [share][vector][launch row], four launch rows per thread (a tile
// of kRows rows belongs to one member).
__global__ __launch_bounds__(256) void reduce_group_kernel(const Group group, const float* __restrict__ partials,
                                                           uint32_t vectors, uint32_t k_splits, uint32_t kRows) {
    const uint64_t launch_rows = static_cast<uint64_t>(group.row_tiles) * kRows;
    const uint64_t item = (static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (item >= launch_rows * vectors) return;
    const uint32_t m = static_cast<uint32_t>(item / launch_rows);
    const uint32_t launch_row = static_cast<uint32_t>(item - m * launch_rows);
    const uint32_t row_tile = launch_row / kRows;
    uint32_t which = 0;
    for (uint32_t i = 1; i < group.count; i++)
        if (row_tile >= group.member[i].first_tile) which = i;
    const Member& member = group.member[which];
    const uint32_t n = launch_row - member.first_tile * kRows;
    if (n >= member.rows) return;
    float4 total = make_float4(0.f, 0.f, 0.f, 0.f);
    const uint64_t share_stride = launch_rows * vectors;
    for (uint32_t k = 0; k < k_splits; k++) {
        const float4 part = *reinterpret_cast<const float4*>(partials + k * share_stride + item);
        if (k == 0) {
            total = part;
        } else {
            total.x += part.x;
            total.y += part.y;
            total.z += part.z;
            total.w += part.w;
        }
    }
    const float sums[4] = {total.x, total.y, total.z, total.w};
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        if (n + i >= member.rows) break;
        const uint64_t at = static_cast<uint64_t>(m) * member.rows + n + i;
        const float with_bias = member.bias != nullptr ? sums[i] + member.bias[n + i] : sums[i];
        member.y[at] = member.residual != nullptr ? with_bias + member.residual[at] : with_bias;
    }
}

// reduce_group_kernel with a rotary embedding behind the sums of the members it names: a thread sums
// the two elements of one rotary pair (of any two neighbouring rows for the other members), adds bias
// and residual as reduce_group_kernel does, rotates with rotary_kernel's arithmetic and stores - the
// bytes of the reduction followed by the rotary launch.
__global__ __launch_bounds__(256) void reduce_group_rotary_kernel(const Group group, const float* __restrict__ partials,
                                                                  uint32_t vectors, uint32_t k_splits, uint32_t kRows,
                                                                  const GemmRotary rotary) {
    const uint64_t launch_rows = static_cast<uint64_t>(group.row_tiles) * kRows;
    const uint64_t item = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= launch_rows / 2 * vectors) return;
    const uint32_t m = static_cast<uint32_t>(item / (launch_rows / 2));
    const uint32_t launch_row = static_cast<uint32_t>(item - m * (launch_rows / 2)) * 2u;
    const uint32_t row_tile = launch_row / kRows;
    uint32_t which = 0;
    for (uint32_t i = 1; i < group.count; i++)
        if (row_tile >= group.member[i].first_tile) which = i;
    const Member& member = group.member[which];
    const uint32_t first_row = member.first_tile * kRows;
    const uint32_t n = launch_row - first_row;  // even
    if (n >= member.rows) return;
    const bool rotate = (rotary.members >> which) & 1u;
    const uint32_t half = rotary.head_dim / 2;
    uint32_t lo = n, hi = n + 1u, index = 0;
    if (rotate) {
        const uint32_t pair = n / 2u, head = pair / half;
        index = pair - head * half;
        lo = rotary.interleaved ? head * rotary.head_dim + 2u * index : head * rotary.head_dim + index;
        hi = rotary.interleaved ? lo + 1u : lo + half;
    }
    const uint64_t share_stride = launch_rows * vectors;
    const auto summed = [&](uint32_t row) {
        const float* first = partials + m * launch_rows + first_row + row;
        float total = first[0];
        for (uint32_t k = 1; k < k_splits; k++) total += first[k * share_stride];
        const float with_bias = member.bias != nullptr ? total + member.bias[row] : total;
        return member.residual != nullptr ? with_bias + member.residual[static_cast<uint64_t>(m) * member.rows + row]
                                          : with_bias;
    };
    float value_lo = summed(lo), value_hi = hi < member.rows ? summed(hi) : 0.f;
    if (rotate) {
        const uint32_t offset = rotary.offsets_len == 1 ? rotary.offsets[0] : rotary.offsets[m];
        rotate_pair(value_lo, value_hi, offset, 0u, index, rotary.head_dim, rotary.theta, rotary.sign, value_lo, value_hi);
    }
    member.y[static_cast<uint64_t>(m) * member.rows + lo] = value_lo;
    if (hi < member.rows) member.y[static_cast<uint64_t>(m) * member.rows + hi] = value_hi;
}

}  // namespace

bool gemm_h16_supported(int32_t codec, uint64_t columns) {
    return (codec == kQ2_K || codec == kQ3_K || codec == kQ4_K || codec == kQ5_K || codec == kQ6_K) &&
           columns % 256 == 0 && columns > 0;
}

GemmGroupGeometry gemm_h16_group_geometry(int32_t codec, const uint64_t* rows, uint32_t count, uint64_t columns,
                                          uint64_t vectors) {
    const uint64_t stages = columns / 256, vector_tiles = (vectors + 31) / 32;
    // The rule of gemm_i8_k_splits: a launch with far fewer workgroups than compute units shares the
    // stages of K out over several workgroups per tile, no share empty.
    const auto shares = [&](uint64_t tiles) -> uint32_t {
        if (tiles == 0 || stages < 2 || tiles >= 192) return 1;
        uint64_t splits = 256 / tiles;
        if (splits > stages) splits = stages;
        if (splits < 2) return 1;
        const uint64_t share = (stages + splits - 1) / splits;
        return static_cast<uint32_t>((stages + share - 1) / share);
    };
    uint64_t small = 0, large = 0;
    for (uint32_t i = 0; i < count; i++) {
        small += (rows[i] + 63) / 64;
        large += (rows[i] + 127) / 128;
    }
    // 128-row workgroups (half the activation copies per weight row) once they fill the device without
    // sharing K. (With K shares they measured slower than 64-row workgroups: 14336 x 4096 with 32 vectors
    // 25.1 against 23.7 us, 4096 x 4096 16.3 against 13.8 us.)
    // (Q6_K: 128 rows of 224 bytes per stage leave no room for a weight ring.)
    if (codec != kQ6_K && large * vector_tiles >= 192) return GemmGroupGeometry{128, large, 1};
    return GemmGroupGeometry{64, small, shares(small * vector_tiles)};
}

uint64_t gemm_h16_group_partial_bytes(int32_t codec, const uint64_t* rows, uint32_t count, uint64_t columns,
                                      uint64_t vectors) {
    const GemmGroupGeometry g = gemm_h16_group_geometry(codec, rows, count, columns, vectors);
    return g.k_splits > 1 ? g.k_splits * vectors * g.row_tiles * g.tile_rows * 4u : 0;
}

namespace {
// The launch that follows a contraction with K shares, unless the caller's next launch sums them itself.
hipError_t sum_shares(const Group& group, const float* partials, uint32_t vectors, uint32_t k_splits, uint32_t tile_rows,
                      hipStream_t stream, bool leave_shares, const GemmRotary* rotary) {
    if (k_splits <= 1 || leave_shares) return hipSuccess;
    if (rotary != nullptr) {
        const uint64_t pairs = static_cast<uint64_t>(group.row_tiles) * tile_rows / 2 * vectors;
        hipLaunchKernelGGL(reduce_group_rotary_kernel, dim3(static_cast<uint32_t>((pairs + 255) / 256)), dim3(256), 0,
                           stream, group, partials, vectors, k_splits, tile_rows, *rotary);
    } else {
        const uint64_t items = static_cast<uint64_t>(group.row_tiles) * tile_rows * vectors / 4;
        hipLaunchKernelGGL(reduce_group_kernel, dim3(static_cast<uint32_t>((items + 255) / 256)), dim3(256), 0, stream,
                           group, partials, vectors, k_splits, tile_rows);
    }
    return hipGetLastError();
}

template <int CODEC, int RG, int AX, int AW, bool NARROW, int PROBE = kProbeNone>
hipError_t launch_tiles(const GemmMember* members, uint32_t count, const uint8_t* tiles, float* partials,
                        uint32_t columns, uint32_t vectors, uint32_t k_splits, hipStream_t stream, bool leave_shares,
                        const GemmRotary* rotary) {
    using S = Shape<CODEC, RG, AX, AW>;
    static_assert(S::kLdsBytes <= 160 * 1024, "LDS of a gfx950 CU: 160 KiB, all of it dynamic here");
    const auto kernel = gemm_h16_kernel<CODEC, RG, AX, AW, NARROW, PROBE>;
    Group group = {};
    group.count = count;
    uint64_t row_tiles = 0;
    for (uint32_t i = 0; i < count; i++) {
        group.member[i] = Member{members[i].weight, members[i].bias, members[i].residual, members[i].y,
                                 static_cast<uint32_t>(members[i].rows), static_cast<uint32_t>(row_tiles)};
        row_tiles += (members[i].rows + S::kRows - 1) / S::kRows;
    }
    if (row_tiles > 0x00ffffffull) return hipErrorInvalidValue;
    group.row_tiles = static_cast<uint32_t>(row_tiles);
    // More than 64 KiB of dynamic LDS has to be allowed once per kernel and device.
    static std::atomic<bool> allowed[64] = {};  // callers may enqueue from several threads; setting twice is harmless
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    if (!allowed[device].load(std::memory_order_acquire)) {
        if (hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, S::kLdsBytes))
            return status;
        allowed[device].store(true, std::memory_order_release);
    }
    const uint32_t vector_tiles = (vectors + 31u) / 32u;
    const uint64_t grid = ((row_tiles + 7u) / 8u) * 8u * vector_tiles * k_splits;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), S::kLdsBytes, stream, group, tiles,
                       vector_tiles, columns, vectors, k_splits, partials);
    if (hipError_t status = hipGetLastError()) return status;
    return sum_shares(group, partials, vectors, k_splits, S::kRows, stream, leave_shares, rotary);
}

// At most sixteen vectors: both planes of a vector ride in one matrix instruction (Operands<true>).
template <int CODEC, int RG, int AX, int AW>
hipError_t launch_group(const GemmMember* members, uint32_t count, const uint8_t* tiles, float* partials,
                        uint32_t columns, uint32_t vectors, uint32_t k_splits, hipStream_t stream, bool leave_shares,
                        const GemmRotary* rotary) {
    if (vectors <= 16u)
        return launch_tiles<CODEC, RG, AX, AW, true>(members, count, tiles, partials, columns, vectors, k_splits, stream,
                                                     leave_shares, rotary);
    return launch_tiles<CODEC, RG, AX, AW, false>(members, count, tiles, partials, columns, vectors, k_splits, stream,
                                                  leave_shares, rotary);
}
}  // namespace

GemmShares gemm_h16_shares_layout(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors) {
    const GemmGroupGeometry g = gemm_h16_group_geometry(codec, &rows, 1, columns, vectors);
    return GemmShares{g.k_splits, g.row_tiles * g.tile_rows};
}

hipError_t gemm_h16_group(int32_t codec, const GemmMember* members, uint32_t count, const uint8_t* tiles,
                          float* partials, uint64_t columns64, uint64_t vectors64, hipStream_t stream,
                          bool leave_shares, const GemmRotary* rotary) {
    if (!gemm_h16_supported(codec, columns64)) return hipErrorInvalidValue;
    if (count == 0 || count > kGemmGroupMost || columns64 % 256 != 0 || columns64 == 0) return hipErrorInvalidValue;
    const uint32_t columns = static_cast<uint32_t>(columns64), vectors = static_cast<uint32_t>(vectors64);
    uint64_t rows[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) {
        if (members[i].rows == 0 || members[i].rows > 0xffffffffull) return hipErrorInvalidValue;
        rows[i] = members[i].rows;
    }
    GemmGroupGeometry g = gemm_h16_group_geometry(codec, rows, count, columns, vectors);
    // the rotary rides on the launch that sums K shares: without shares the caller rotates itself
    if (rotary != nullptr && (g.k_splits == 1 || partials == nullptr)) return hipErrorInvalidValue;
    if (partials == nullptr && g.k_splits > 1) {  // nowhere to keep shares: 64-row workgroups, whole K each
        g = GemmGroupGeometry{64, 0, 1};
    }
    // weight lead: what the activation ring (three slots of 34 KiB) leaves of LDS
    if (codec == kQ6_K)  // 64-row tiles only (gemm_h16_group_geometry): 128 rows of 224 bytes leave no room for a ring
        return launch_group<kQ6_K, 2, 2, 2>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
    if (codec == kQ2_K || codec == kQ3_K) {  // rows of 96 / 112 bytes per stage: room for the longest lead
        if (codec == kQ2_K) {
            if (g.tile_rows == 128)
                return launch_group<kQ2_K, 4, 2, 2>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
            return launch_group<kQ2_K, 2, 2, 3>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
        }
        if (g.tile_rows == 128)
            return launch_group<kQ3_K, 4, 2, 2>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
        // as for Q4_K: three stages of activation lead, one of weights (14336 x 4096 with 32 vectors 28.0 -> 25.9 us)
        return launch_group<kQ3_K, 2, 3, 1>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
    }
    if (codec == kQ5_K) {
        if (g.tile_rows == 128)
            return launch_group<kQ5_K, 4, 2, 1>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
        // three stages of activation lead, one of weights: 158 KiB (14336 x 4096 with 32 vectors 29.9 -> 28.7 us)
        return launch_group<kQ5_K, 2, 3, 1>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
    }
    if (g.tile_rows == 128)
        return launch_group<kQ4_K, 4, 2, 2>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
    // 64-row tiles: two stages of activation lead and three of weights. Timestamps taken inside the kernel
    // show the operands of a stage in LDS well before its barrier with either split of the ring; what the
    // stage waits for is its slowest consumer. (14336 x 4096 with 32 vectors, contraction alone: 20.6 us
    // against 21.7 with three and one; 4096 x 14336 22.5 against 23.6; more loader waves changed nothing.)
    return launch_group<kQ4_K, 2, 2, 3>(members, count, tiles, partials, columns, vectors, g.k_splits, stream, leave_shares, rotary);
}

#ifdef ET_HIP_CALIBRATE  // the measurement library's build of this file: the kernel minus one part, per probe
hipError_t gemm_h16_probe(int probe, const uint8_t* weight, const uint8_t* tiles, float* y, uint64_t rows,
                          uint64_t columns, uint64_t vectors, hipStream_t stream) {
    if (!gemm_h16_supported(kQ4_K, columns) || rows == 0 || rows > 0xffffffffull || vectors == 0 || vectors > 32)
        return hipErrorInvalidValue;
    const GemmGroupGeometry g = gemm_h16_group_geometry(kQ4_K, &rows, 1, columns, vectors);
    if (g.tile_rows != 64 || g.k_splits != 1) return hipErrorInvalidValue;  // the 64-row tiles, whole K each
    const GemmMember one = {weight, nullptr, nullptr, y, rows};
    const uint32_t k = static_cast<uint32_t>(columns), m = static_cast<uint32_t>(vectors);
    const auto run = [&](auto narrow) -> hipError_t {
        constexpr bool N = decltype(narrow)::value;
        switch (probe) {
            case kProbeNone: return launch_tiles<kQ4_K, 2, 2, 3, N>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeNoArithmetic:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeNoArithmetic>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeNoCopies:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeNoCopies>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeNoWeightCopies:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeNoWeightCopies>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeNoActivationCopies:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeNoActivationCopies>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeWeightCopiesOnly:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeWeightCopiesOnly>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            case kProbeActivationCopiesOnly:
                return launch_tiles<kQ4_K, 2, 2, 3, N, kProbeActivationCopiesOnly>(&one, 1, tiles, nullptr, k, m, 1, stream, false, nullptr);
            default: return hipErrorInvalidValue;
        }
    };
    return vectors <= 16 ? run(std::true_type{}) : run(std::false_type{});
}
#endif

hipError_t gemm_h16(int32_t codec, const uint8_t* weight, const uint8_t* tiles, const GemmOutput& out,
                    uint64_t rows, uint64_t columns, uint64_t vectors, hipStream_t stream) {
    const GemmMember one = {weight, out.bias, out.residual, out.y, rows};
    return gemm_h16_group(codec, &one, 1, tiles, out.partials, columns, vectors, stream, out.leave_shares);
}

}  // namespace et
