// Block-scaled int8 contraction on the gfx950 matrix cores, for batches of vectors.
//
//   Q8_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i qw[n,b,i] * qx[m,b,i])
//   Q4_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i (nib[n,b,i] - 8) * qx[m,b,i])
//   Q4_K:  y[m, n] = sum_g (d*sc_g)[n] * s[m,g] * (sum_i nib * qx)  -  sum_g (dmin*m_g)[n] * xf[m,g]
// b / g index 32-column blocks; xf[m, g] is the block's activation sum in f32.
// The inner sums are exact int32 from v_mfma_i32_32x32x32_i8, whose K = 32 is
// exactly one quantisation block. The block scales are applied in f32 after every
// MFMA: the 32x32 tile of scale products s[m] * d[n] is itself a rank-1 matrix
// product and comes from v_mfma_f32_32x32x2f32 in the result layout, so the VALU
// epilogue is one convert and one FMA per element. The Q4_K "min" term is a small
// f32 GEMM of its own (inner dimension K/32) and accumulates on the same f32 MFMA.
//
// Two activation formats feed the same kernel (quantize_act.hip makes both):
//   LIMBS = 1  int8 activations, one scale per vector and 32 columns (the
//              int8-activation mode; tolerance 2e-2 against f32 activations);
//   LIMBS = 3  every activation as a 24-bit fixed-point integer in three
//              balanced signed bytes, X = 65536*x2 + 256*x1 + x0, unit = max|x| /
//              (127 * 2^16) per 32 columns: f32 accuracy. The three limbs of a
//              block go through the matrix core one after the other against the
//              same weight registers and are combined with weights 1, 256, 65536.
// The reference has neither (its Metal prefill kernel decodes weights to f32 and
// uses f32 simdgroup MMA, crates/runtime-metal/src/quantized.rs:1016-1097); the
// contraction computed is linear_into's (crates/runtime-cpu/src/quantized.rs:419-499).
//
// Tiling. A workgroup owns 64 weight rows x 32*MT vectors and walks K in stages of
// eight blocks (256 columns, one Q4_K super-block). Eight consumer waves run the
// MFMAs: four of them share 32 weight rows and split the eight blocks of every
// stage between them; their accumulators meet in LDS at the end.
//
// Operand streams. Four more waves, the loaders, do nothing but copy operands of
// later stages into LDS rings with global_load_lds while the consumers contract
// stage s; one s_barrier per stage joins the groups. Two loaders serve the
// activation ring, two the weight ring: loads return in order per wave, so streams
// with different leads must not share a wave. Activations are re-read by every
// workgroup and come from L2: two stages of lead. Weights come from HBM, and what
// bounds a CU's share of the bandwidth is how many bytes it keeps in flight: their
// ring gets up to three stages of lead.
//   activations  arrive as ready-made stage blobs (see kernels.h): a linear copy;
//   weights      the stage's bytes of the workgroup's rows, row after row as in memory
//                (see WeightLayout for how the consumers read their operands out of them).
// Why separate waves: loads return in order and are counted per wave; a wave that
// mixes global_load_lds with loads into registers gets a full wait (vmcnt 0) from
// the compiler before every use of a loaded register, and a consumer wave whose
// lanes each read another weight row (what the B operand needs) stalls in the address
// unit on every load. The loaders absorb both: they copy along rows, wait with an
// explicit count, and the consumers issue no global loads at all until they store.
//
// The consumers run each stage as a software pipeline over its (block, tile) steps: LDS
// reads one step ahead of the MFMAs, the f32 epilogue one step behind them, so that the
// matrix pipe, the VALU and LDS work on three different steps at a time.
//
// MFMA operand roles: A = activations, B = weights. A lane of the 32x32 result holds
// one weight row n = lane % 32 and sixteen vectors m = 8*(r/4) + 4*(lane/32) + r%4,
// and every result register row is stored as 128 contiguous bytes of y.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// Sixteen bytes at an LDS address that is only a multiple of four (declared 2-byte aligned so that the
// compiler emits one ds_read_b128 instead of two ds_read2_b32).
#pragma clang diagnostic ignored "-Walign-mismatch"
typedef uint4 __attribute__((aligned(2))) LdsQuad;

constexpr int kStageBlocks = 8;  // 32-column blocks per stage
constexpr int kConsumers = 8;    // waves that run the MFMAs: two per SIMD
constexpr int kWeightLoaders = 2;      // waves that only gather weights into LDS
constexpr int kActivationLoaders = 2;  // waves that only copy activation blobs into LDS
constexpr int kLoaders = kWeightLoaders + kActivationLoaders;
constexpr int kThreads = 64 * (kConsumers + kLoaders);
constexpr int kSplit = 4;                         // consumer waves sharing a row group
constexpr int kRowGroups = kConsumers / kSplit;   // 32-row groups per workgroup
constexpr int kBlocksPerWave = kStageBlocks / kSplit;
constexpr uint32_t kRows = 32 * kRowGroups;       // weight rows per workgroup

// (scale, min) of Q4_K sub-block g (crates/runtime-cpu/src/quantized.rs:77-86).
__device__ __forceinline__ void q4k_scale_min(const uint4& header, uint32_t g, float& scale, float& min) {
    const uint32_t shift = 8u * (g & 3u);
    const uint32_t s0 = (header.y >> shift) & 0xffu;  // scales[g & 3]
    const uint32_t s1 = (header.z >> shift) & 0xffu;  // scales[4 + (g & 3)]
    const uint32_t s2 = (header.w >> shift) & 0xffu;  // scales[8 + (g & 3)]
    const uint32_t sc = g < 4 ? (s0 & 63u) : ((s2 & 0x0fu) | ((s0 >> 6) << 4));
    const uint32_t mn = g < 4 ? (s1 & 63u) : ((s2 >> 4) | ((s1 >> 6) << 4));
    scale = static_cast<float>(sc);
    min = static_cast<float>(mn);
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) {
    return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8);
}

// The tile of scale products s[m] * d[n] from v_mfma_f32_32x32x16_bf16, which takes half the
// matrix-core time of the f32 instruction: a half-float row scale is exactly two bfloat16 pieces
// (8 + 3 bits), an f32 vector scale exactly three, and their six products - each exact in the f32
// accumulator - fill six of the eight K slots of the first lane half: rows (d0, d0, d0, 0, d1, d1,
// d1, 0) against vectors (s0, s1, s2, 0, s0, s1, s2, 0). The second lane half holds zeros on the
// row side, so the vector side needs no mask there (scales are finite). The quantiser stores the
// vector pieces next to the scale (kernels.h: pieces[b][m]); kernels that use them copy the pieces
// into LDS in place of the two f32 tables.
union ScaleOperand {
    uint4 words;
    v8bf values;
};
__device__ __forceinline__ ScaleOperand row_scale_pieces(float d, bool first_half) {
    const uint32_t d0 = __float_as_uint(d) >> 16;  // top sixteen bits: the bfloat16 below d
    const uint32_t d1 = __float_as_uint(d - __uint_as_float(d0 << 16)) >> 16;  // exact: at most three bits left
    ScaleOperand operand;
    operand.words = first_half ? make_uint4(d0 | (d0 << 16), d0, d1 | (d1 << 16), d1) : make_uint4(0u, 0u, 0u, 0u);
    return operand;
}
// `pieces` as the quantiser stores them: (s0 | s1 << 16, s2).
__device__ __forceinline__ ScaleOperand vector_scale_pieces(const uint2& pieces) {
    ScaleOperand operand;
    operand.words = make_uint4(pieces.x, pieces.y, pieces.x, pieces.y);
    return operand;
}

// Weight slot in LDS: the stage's bytes of the workgroup's 64 rows, row after row exactly as in
// memory (a row's stage is 144 bytes for Q4_K and Q4_0, 272 for Q8_0: whole 16-byte chunks), so a
// copy instruction's 64 lanes walk along rows and touch about fifteen cache lines. (Gathering one
// chunk per row instead, ready in operand order, touches 32 to 64 lines per instruction and made
// the loaders' issue rate the bound of the whole kernel.) The consumers pick their operands out
// of the rows:
//   Q4_K  16-byte reads at row*144 + {0 (header), 16 + 32*pair + 16*half}: the 144-byte pitch
//         spreads eight consecutive rows over all banks.
//   Q8_0, Q4_0: blocks are 2-byte aligned. A lane reads the five dwords around its block start
//         (+ 16*half for Q8_0): they hold the fp16 scale and the 16 quant bytes behind it, to be
//         shifted by 16 bits for even blocks (block starts alternate between 0 and 2 mod 4).
template <int CODEC>
struct WeightLayout {
    static constexpr uint32_t kBlockBytes = CODEC == kQ8_0 ? 34u : 18u;      // 32-wide codecs
    static constexpr uint32_t kRowBytes = CODEC == kQ8_0 ? 272u : 144u;      // one row's stage
    static constexpr uint32_t kBytes = kRows * kRowBytes;
    static constexpr int kJobs = kBytes / 1024;
    static_assert(kBytes % 1024 == 0, "whole copy instructions");
};

// AX / AW: how many stages the activation / weight stream runs ahead of the MFMAs.
template <int CODEC, int MT, int LIMBS, int AX, int AW>
struct Shape {
    using W = WeightLayout<CODEC>;
    static constexpr uint32_t kBlob = tile_blob_bytes(LIMBS);        // in memory, padded
    static constexpr uint32_t kTile = LIMBS * 8192u + 2048u;          // in LDS: operands and the two f32 tables or the pieces
    // Two rings: activations come from L2 (every workgroup reads the same blobs) and need little
    // lead; weights come from HBM and need as much as LDS allows.
    static constexpr int kActivationDepth = AX + 1, kWeightDepth = AW + 1;
    static constexpr uint32_t kActivationBytes = MT * kTile;            // per slot
    static constexpr uint32_t kWeightRingAt = kActivationDepth * kActivationBytes;
    static constexpr uint32_t kRingBytes = kWeightRingAt + kWeightDepth * W::kBytes;
    // One global_load_lds moves up to 1 KiB per wave. Every loader of a stream issues the same
    // number of copies per stage (for its counted wait): jobs are dealt round-robin and the last
    // round wraps around to the first jobs, copied twice.
    static constexpr int kActivationJobs = kActivationBytes / 1024;
    static constexpr int kActivationRounds = (kActivationJobs + kActivationLoaders - 1) / kActivationLoaders;
    static constexpr int kWeightRounds = (W::kJobs + kWeightLoaders - 1) / kWeightLoaders;
    static_assert(kActivationJobs >= kActivationLoaders && W::kJobs >= kWeightLoaders,
                  "the wrap-around of the last round needs a full first round");
    // vmcnt is a 6-bit counter: a smaller bound only waits for more than necessary.
    static constexpr int kActivationWait = (AX - 1) * kActivationRounds < 63 ? (AX - 1) * kActivationRounds : 63;
    static constexpr int kWeightWait = (AW - 1) * kWeightRounds < 63 ? (AW - 1) * kWeightRounds : 63;
    static constexpr uint32_t kExchangeBytes = (kSplit - 1) * kRowGroups * MT * 16 * 64 * 4;
    static constexpr uint32_t kLdsBytes = kRingBytes > kExchangeBytes ? kRingBytes : kExchangeBytes;
};

template <int CODEC, int MT, int LIMBS, int AX, int AW>
__global__ __launch_bounds__(kThreads) void gemm_i8_kernel(
    const uint8_t* __restrict__ weight, const uint8_t* __restrict__ tiles, uint32_t vector_tiles,
    const float* __restrict__ bias, const float* residual, float* y, uint32_t rows, uint32_t columns,
    uint32_t vectors, uint32_t row_tiles, uint32_t vector_groups, uint32_t k_splits,
    float* __restrict__ partials) {
    using S = Shape<CODEC, MT, LIMBS, AX, AW>;
    using W = WeightLayout<CODEC>;
    constexpr int NB = kBlocksPerWave;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // Workgroups are handed to the eight XCDs round-robin. All vector groups of one row tile
    // go to the same XCD, next to each other in time, so the later ones find the weights in L2.
    const uint32_t xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
    // With k_splits > 1 the stages of K are shared out over that many workgroups per tile, each
    // leaving a partial result for reduce_partials_kernel.
    const uint32_t units = vector_groups * k_splits;
    const uint32_t row_tile = (turn / units) * 8u + xcd;
    const uint32_t vector_group = (turn % units) % vector_groups;
    const uint32_t k_share = (turn % units) / vector_groups;
    if (row_tile >= row_tiles) return;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: uniform branches
    const uint32_t tile0 = vector_group * MT;
    const uint32_t all_stages = columns / 256u;  // whole: columns % 256 == 0
    const uint32_t share = (all_stages + k_splits - 1u) / k_splits;
    const uint32_t first_stage = k_share * share;  // < all_stages: the launcher leaves no share empty
    const uint32_t stages = min(share, all_stages - first_stage);
    const uint64_t row_bytes = static_cast<uint64_t>(columns / block_values(CODEC)) * block_bytes(CODEC);
    const uint32_t row0 = row_tile * kRows;

    if (wave >= static_cast<uint32_t>(kConsumers + kWeightLoaders)) {
        // ---- activation loaders -----------------------------------------------------
        const uint32_t loader = wave - (kConsumers + kWeightLoaders);
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);  // past the end: a copy nobody reads
            uint8_t* slot = lds + (stage % S::kActivationDepth) * S::kActivationBytes;
#pragma unroll
            for (int i = 0; i < S::kActivationRounds; i++) {
                uint32_t job = i * kActivationLoaders + loader;  // 1 KiB of the blobs, as they lie in memory
                if (job >= static_cast<uint32_t>(S::kActivationJobs)) job -= S::kActivationJobs;
                const uint32_t t = job / (S::kTile / 1024u), within = job % (S::kTile / 1024u);
                const uint32_t tile = min(tile0 + t, vector_tiles - 1u);
                // codecs with bfloat16 scale products take the pieces table in place of the two f32 tables
                const uint32_t from = CODEC != kQ4_K && within >= static_cast<uint32_t>(LIMBS) * 8u ? within + 2u : within;
                const uint8_t* src = tiles + (static_cast<uint64_t>(first_stage + s) * vector_tiles + tile) * S::kBlob +
                                     from * 1024u + lane * 16u;
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                 reinterpret_cast<uint4*>(slot + job * 1024u), 16, 0, 0);
            }
        };
        for (uint32_t a = 0; a < static_cast<uint32_t>(AX); a++) request(a);
        for (uint32_t stage = 0; stage < stages; stage++) {
            // Loads return in order: all but the newest AX - 1 requests have landed.
            __builtin_amdgcn_s_waitcnt(vmcnt_only(S::kActivationWait));
            // Passing the barrier says "stage is in LDS" to the consumers and "the slots of
            // stage - 1 are free" to the loaders.
            __builtin_amdgcn_s_barrier();
            request(stage + AX);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));  // nothing may still write the ring
        __builtin_amdgcn_s_barrier();               // the consumers' two exchange barriers
        __builtin_amdgcn_s_barrier();
        return;
    }
    if (wave >= static_cast<uint32_t>(kConsumers)) {
        // ---- weight loaders ---------------------------------------------------------
        const uint32_t loader = wave - kConsumers;
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);
            uint8_t* region = lds + S::kWeightRingAt + (stage % S::kWeightDepth) * W::kBytes;
#pragma unroll
            for (int i = 0; i < S::kWeightRounds; i++) {
                uint32_t job = i * kWeightLoaders + loader;
                if (job >= static_cast<uint32_t>(W::kJobs)) job -= W::kJobs;
                const uint32_t at = job * 1024u + lane * 16u;  // byte of the slot this lane fills
                const uint32_t row = min(row0 + at / W::kRowBytes, rows - 1u);
                const uint8_t* src = weight + row * row_bytes + static_cast<uint64_t>(first_stage + s) * W::kRowBytes +
                                     at % W::kRowBytes;
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

    // ---- consumer waves -----------------------------------------------------------
    const uint32_t half = lane >> 5;
    const uint32_t wave_n = wave % kRowGroups;  // row group
    const uint32_t wave_k = wave / kRowGroups;  // share of the stage's blocks
    const uint32_t n0 = row0 + wave_n * 32u;
    const uint32_t m0 = tile0 * 32u;
    v16f acc[MT];  // a matrix-core register tile: the Q4_K min term accumulates into it directly
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
    // With one limb the integer sums start at the bits of 1.5 * 2^23 instead of zero: a block's sum
    // (|c| <= 32 * 128 * 127 < 2^22) added to those bits IS the float 12582912 + c, so the epilogue turns
    // it into c with one subtraction - exact, and half the issue time of an int-to-float convert.
    constexpr int kFloatBias = 0x4B400000;
    v16i zero_i;
    v16f zero_f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        zero_i[r] = LIMBS == 1 ? kFloatBias : 0;
        zero_f[r] = 0.f;
    }

    for (uint32_t stage = 0; stage < stages; stage++) {
        // A plain s_barrier: __syncthreads() would add a fence the loop does not need.
        __builtin_amdgcn_s_barrier();
        const uint8_t* slot = lds + (stage % S::kActivationDepth) * S::kActivationBytes;
        const uint8_t* region = lds + S::kWeightRingAt + (stage % S::kWeightDepth) * W::kBytes;
        const uint32_t b_base = wave_k * NB;  // first block of this wave inside the stage
        const uint8_t* row_in_slot = region + (wave_n * 32u + (lane & 31u)) * W::kRowBytes;  // this lane's row

        uint4 header = make_uint4(0u, 0u, 0u, 0u);
        float d_block = 0.f, dmin_block = 0.f;
        if constexpr (CODEC == kQ4_K) {
            header = *reinterpret_cast<const uint4*>(row_in_slot);
            d_block = half_bits_to_float(header.x & 0xffffu);
            dmin_block = half_bits_to_float(header.x >> 16);
        }
        if constexpr (CODEC == kQ4_K) {
            // min term: acc[m, n] -= sum_g (dmin * m_g)[n] * xsum[m, g]; K = 2 per MFMA,
            // lane half h supplies sub-block 2j + h. First in the stage: its LDS reads go out with
            // the other operands' and its MFMAs run under the first steps.
#pragma unroll
            for (int jj = 0; jj < NB / 2; jj++) {
                const uint32_t g = b_base + 2u * jj + half;
                float sc, mn;
                q4k_scale_min(header, g, sc, mn);
                const float b_operand = -(dmin_block * mn);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float a_operand = *reinterpret_cast<const float*>(
                        slot + t * S::kTile + LIMBS * 8192u + 1024u + g * 128u + (lane & 31u) * 4u);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_operand, b_operand, acc[t], 0, 0, 0);
                }
            }
        }
        // B operands (16 int8 weights of row n, this lane's half of the block) and block scales
        v4i bw[NB];
        float w_scale[NB];
        // Half-float row scales (Q8_0, Q4_0) go through the bfloat16 instruction; d * sc of Q4_K has
        // seventeen bits and stays on the f32 one.
        constexpr bool kPieces = CODEC != kQ4_K;
        ScaleOperand w_pieces[NB];
#pragma unroll
        for (int bb = 0; bb < NB; bb++) {
            const uint32_t b = b_base + bb;  // block inside the stage
            if constexpr (CODEC == kQ4_K) {
                // sub-block 2p + side: low (side 0) or high (side 1) nibbles of pair p
                const uint4 raw = *reinterpret_cast<const uint4*>(row_in_slot + 16u + 32u * (b >> 1) + 16u * half);
                const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; i++)
                    bw[bb][i] = static_cast<int>(((b & 1u) ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu);
                float sc, mn;
                q4k_scale_min(header, b, sc, mn);
                w_scale[bb] = d_block * sc;
            } else {
                // Five dwords from the dword at or 2 bytes before the block start (+ 16 for the
                // second column half of Q8_0): scale and quants of even blocks start in the low
                // half of the first dword, those of odd blocks in its high half.
                const uint32_t start = b * W::kBlockBytes + (CODEC == kQ8_0 ? 16u * half : 0u);
                const uint32_t* window = reinterpret_cast<const uint32_t*>(row_in_slot + (start & ~3u));
                // The first four as ONE 16-byte LDS read (4-byte aligned: LDS serves it): sixteen lanes of
                // consecutive rows then cover all banks once, where single dwords at the 272- / 144-byte
                // row pitch put four lanes on a bank (config 3 contraction 107.8 -> 103.3 us).
                const uint4 first_four = *reinterpret_cast<const LdsQuad*>(window);
                const uint32_t d0 = first_four.x, d1 = first_four.y, d2 = first_four.z, d3 = first_four.w, d4 = window[4];
                const bool odd = (b & 1u) != 0;  // (row * pitch + b * 34 or 18) & 2, pitch % 4 == 0
                // The scale sits at the block start: for the second half of Q8_0 in another dword.
                const uint32_t scale_word =
                    CODEC == kQ8_0 ? *reinterpret_cast<const uint32_t*>(row_in_slot + ((b * W::kBlockBytes) & ~3u)) : d0;
                w_scale[bb] = half_bits_to_float(odd ? scale_word >> 16 : scale_word & 0xffffu);
                uint32_t words[4];
                words[0] = odd ? d1 : __builtin_amdgcn_alignbit(d1, d0, 16);
                words[1] = odd ? d2 : __builtin_amdgcn_alignbit(d2, d1, 16);
                words[2] = odd ? d3 : __builtin_amdgcn_alignbit(d3, d2, 16);
                words[3] = odd ? d4 : __builtin_amdgcn_alignbit(d4, d3, 16);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if constexpr (CODEC == kQ8_0) {
                        bw[bb][i] = static_cast<int>(words[i]);
                    } else {
                        // element j = low nibble of byte j (j < 16), element j+16 = high nibble: lanes
                        // 0-31 take the low nibbles, lanes 32-63 the high ones; value = nibble - 8,
                        // per byte without borrows between bytes.
                        const uint32_t nib = (half ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu;
                        bw[bb][i] = static_cast<int>(((nib | 0x80808080u) - 0x08080808u) ^ 0x80808080u);
                    }
                }
            }
            // rank-1 operand: only the k = 0 half of the lanes carries a value
            if constexpr (kPieces) w_pieces[bb] = row_scale_pieces(w_scale[bb], half == 0);
            w_scale[bb] = half == 0 ? w_scale[bb] : 0.f;
        }

        // The NB * MT (block, tile) steps of the stage as a software pipeline. Each step reads its
        // A operands (and the activation scales) from LDS one step ahead, issues its MFMAs, and
        // runs the f32 epilogue of an earlier step while they execute: with one limb the previous
        // step's (its integer sums are double-buffered), with three limbs its own (three results of
        // sixteen registers each leave no room for a second set).
        constexpr int kSteps = NB * MT;
        const auto read_step = [&](int step, v4i (&a)[LIMBS], float& x_scale, uint2& x_pieces) {
            const uint32_t b = b_base + step / MT;
            const uint8_t* blob = slot + (step % MT) * S::kTile;
            if constexpr (kPieces)
                x_pieces = *reinterpret_cast<const uint2*>(blob + LIMBS * 8192u + b * 256u + (lane & 31u) * 8u);
            else
                x_scale = *reinterpret_cast<const float*>(blob + LIMBS * 8192u + b * 128u + (lane & 31u) * 4u);
            const uint8_t* chunk = blob + (2u * b + half) * 512u + (lane & 31u) * 16u;
#pragma unroll
            for (int l = 0; l < LIMBS; l++) a[l] = *reinterpret_cast<const v4i*>(chunk + l * 8192u);
        };
        // acc[t] += sd * (c[0] + 256 c[1] + 65536 c[2])
        const auto epilogue = [&](int step, const v16f& sd, const v16i (&c)[LIMBS]) {
            const int t = step % MT;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                if constexpr (LIMBS == 1) {
                    acc[t][r] = fmaf(__int_as_float(c[0][r]) - 12582912.0f, sd[r], acc[t][r]);
                } else {
                    // |c0 + 256 c1| < 2^28 is exact in int32; the top limb joins in f32
                    const float low = static_cast<float>(c[0][r] + (c[1][r] << 8));
                    const float all = fmaf(65536.0f, static_cast<float>(c[2][r]), low);
                    acc[t][r] = fmaf(all, sd[r], acc[t][r]);
                }
            }
        };
        v4i a_next[LIMBS];
        float x_scale_next = 0.f;
        uint2 x_pieces_next = make_uint2(0u, 0u);
        read_step(0, a_next, x_scale_next, x_pieces_next);
        // Scale products s[m] * d[n] for the sixteen vectors this lane accumulates: a rank-1 product in
        // the MFMA result layout.
        const auto scale_products = [&](int bb, float x_scale, const uint2& x_pieces) -> v16f {
            if constexpr (kPieces)
                return __builtin_amdgcn_mfma_f32_32x32x16_bf16(vector_scale_pieces(x_pieces).values, w_pieces[bb].values,
                                                               zero_f, 0, 0, 0);
            else
                return __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? x_scale : 0.f, w_scale[bb], zero_f, 0, 0, 0);
        };
        if constexpr (LIMBS == 1) {
            // Every matrix instruction is followed by half of an epilogue, sixteen VALU instructions that
            // do not depend on it, so the matrix pipe and the VALU run side by side within the wave:
            //   scale products of step s   | the integer sums of step s become floats (in place)
            //   integer MFMA of step s + 1 | acc += sums * scale products of step s
            // The integer sums alternate between two register sets; the scale products need one.
            v16i c_now = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_next[0], bw[0], zero_i, 0, 0, 0);
            float x_scale = x_scale_next;
            uint2 x_pieces = x_pieces_next;
            if (1 < kSteps) read_step(1, a_next, x_scale_next, x_pieces_next);
#pragma unroll
            for (int step = 0; step < kSteps; step++) {
                const int t = step % MT;
                // the matrix instruction first in each half (scheduling barriers: the compiler would put it last)
                __builtin_amdgcn_sched_barrier(0);
                const v16f sd = scale_products(step / MT, x_scale, x_pieces);
                __builtin_amdgcn_sched_barrier(0);
                float sums[16];
#pragma unroll
                for (int r = 0; r < 16; r++) sums[r] = __int_as_float(c_now[r]) - 12582912.0f;
                __builtin_amdgcn_sched_barrier(0);
                if (step + 1 < kSteps) {
                    c_now = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_next[0], bw[(step + 1) / MT], zero_i, 0, 0, 0);
                    x_scale = x_scale_next;
                    x_pieces = x_pieces_next;
                    __builtin_amdgcn_sched_barrier(0);
                    if (step + 2 < kSteps) read_step(step + 2, a_next, x_scale_next, x_pieces_next);
                }
#pragma unroll
                for (int r = 0; r < 16; r++) acc[t][r] = fmaf(sums[r], sd[r], acc[t][r]);
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
#pragma unroll
            for (int step = 0; step < kSteps; step++) {
                const int bb = step / MT;
                const v16f sd = scale_products(bb, x_scale_next, x_pieces_next);
                v16i c[LIMBS];
#pragma unroll
                for (int l = 0; l < LIMBS; l++)
                    c[l] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_next[l], bw[bb], zero_i, 0, 0, 0);
                if (step + 1 < kSteps) read_step(step + 1, a_next, x_scale_next, x_pieces_next);
                __builtin_amdgcn_sched_barrier(0);
                epilogue(step, sd, c);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- combine the K shares, add bias, store ----------------------------------
    __syncthreads();  // the loaders arrive here with nothing in flight: the ring is free
    float* exchange = reinterpret_cast<float*>(lds);  // [wave_k - 1][wave_n][MT * 16][64 lanes]
    if (wave_k > 0) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float value = acc[t][r];
                exchange[((((wave_k - 1u) * kRowGroups + wave_n) * MT + t) * 16 + r) * 64 + lane] = value;
            }
    }
    __syncthreads();
    if (wave_k > 0) return;
    const uint32_t n_out = n0 + (lane & 31u);
    const float bias_value = bias != nullptr && n_out < rows ? bias[n_out] : 0.f;
#pragma unroll
    for (int t = 0; t < MT; t++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float value = acc[t][r];
#pragma unroll
            for (int k = 1; k < kSplit; k++)
                value += exchange[((((k - 1) * kRowGroups + wave_n) * MT + t) * 16 + r) * 64 + lane];
            const uint32_t m = m0 + 32u * t + 8u * (r >> 2) + 4u * half + (r & 3u);
            if (n_out < rows && m < vectors) {
                if (k_splits == 1) {
                    // residual may be y itself: every output is read, then written, by this lane only
                    const uint64_t at = static_cast<uint64_t>(m) * rows + n_out;
                    y[at] = residual != nullptr ? (value + bias_value) + residual[at] : value + bias_value;
                } else
                    partials[(static_cast<uint64_t>(k_share) * vectors + m) * rows + n_out] = value;
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // tile by tile: the sums of all tiles at once do not fit
    }
}

}  // namespace
uint32_t gemm_i8_k_splits(int32_t codec, int limbs, uint64_t rows, uint64_t columns, uint64_t vectors);
namespace {

// y[m, n] = bias[n] + sum over the K shares, in share order (+ residual[m, n], which may be y
// itself); four outputs per thread.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partials,
                                                              const float* __restrict__ bias, const float* residual,
                                                              float* y, uint32_t rows, uint64_t outputs,
                                                              uint32_t k_splits) {
    const uint64_t i = (static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i >= outputs) return;
    if (rows % 4 == 0) {
        const uint32_t n = static_cast<uint32_t>(i % rows);
        float4 total = bias != nullptr ? *reinterpret_cast<const float4*>(bias + n) : make_float4(0.f, 0.f, 0.f, 0.f);
        for (uint32_t k = 0; k < k_splits; k++) {
            const float4 part = *reinterpret_cast<const float4*>(partials + k * outputs + i);
            total.x += part.x;
            total.y += part.y;
            total.z += part.z;
            total.w += part.w;
        }
        if (residual != nullptr) {
            const float4 r = *reinterpret_cast<const float4*>(residual + i);
            total.x += r.x;
            total.y += r.y;
            total.z += r.z;
            total.w += r.w;
        }
        *reinterpret_cast<float4*>(y + i) = total;
    } else {
        for (uint64_t j = i; j < min(i + 4, outputs); j++) {
            float total = bias != nullptr ? bias[j % rows] : 0.f;
            for (uint32_t k = 0; k < k_splits; k++) total += partials[k * outputs + j];
            y[j] = residual != nullptr ? total + residual[j] : total;
        }
    }
}

template <int CODEC, int MT, int LIMBS, int AX, int AW>
hipError_t launch(const uint8_t* weight, const uint8_t* tiles, const GemmOutput& out, uint32_t rows,
                  uint32_t columns, uint32_t vectors, hipStream_t stream) {
    const float* bias = out.bias;
    float* y = out.y;
    float* partials = out.partials;
    using S = Shape<CODEC, MT, LIMBS, AX, AW>;
    static_assert(S::kLdsBytes <= 156 * 1024, "LDS of a gfx950 CU (160 KiB), with a margin");
    const auto kernel = gemm_i8_kernel<CODEC, MT, LIMBS, AX, AW>;
    // More than 64 KiB of dynamic LDS has to be allowed once per kernel and device.
    static std::atomic<bool> allowed[64] = {};  // callers may enqueue from several threads; setting twice is harmless
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    if (!allowed[device].load(std::memory_order_acquire)) {
        if (hipError_t status =
                hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, S::kLdsBytes))
            return status;
        allowed[device].store(true, std::memory_order_release);
    }
    const uint32_t vector_tiles = (vectors + 31u) / 32u;
    const uint32_t vector_groups = (vector_tiles + MT - 1) / MT;
    const uint32_t row_tiles = (rows + kRows - 1) / kRows;
    const uint32_t k_splits = partials != nullptr ? gemm_i8_k_splits(CODEC, LIMBS, rows, columns, vectors) : 1u;
    const uint64_t grid = static_cast<uint64_t>((row_tiles + 7u) / 8u) * 8u * vector_groups * k_splits;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), S::kLdsBytes, stream,
                       weight, tiles, vector_tiles, bias, out.residual, y, rows, columns, vectors, row_tiles,
                       vector_groups, k_splits, partials);
    if (hipError_t status = hipGetLastError()) return status;
    if (k_splits > 1) return reduce_partials(partials, bias, out.residual, y, rows, vectors, k_splits, stream);
    return hipSuccess;
}

// Weight lead (stages) that fills what the activation ring leaves of LDS.
template <int CODEC, int MT, int LIMBS, int AX>
constexpr int weight_lead() {
    constexpr uint32_t tile = LIMBS * 8192u + 2048u;
    constexpr uint32_t left = 156u * 1024u - (AX + 1) * MT * tile;
    constexpr int depth = static_cast<int>(left / WeightLayout<CODEC>::kBytes);
    // the counted wait holds at most 63 copies: (lead - 1) * rounds of a weight loader
    constexpr int rounds = (WeightLayout<CODEC>::kJobs + kWeightLoaders - 1) / kWeightLoaders;
    constexpr int by_counter = 63 / rounds + 1;
    // More than three stages of lead gained nothing in measurements (a small batch waits for the
    // copies' issue time, not their latency) and only delays the first stage.
    constexpr int fits = depth - 1 < by_counter ? depth - 1 : by_counter;
    return fits < 3 ? fits : 3;
}

template <int CODEC, int MT, int LIMBS, int AX>
hipError_t launch_shape(const uint8_t* weight, const uint8_t* tiles, const GemmOutput& out, uint32_t rows,
                        uint32_t columns, uint32_t vectors, hipStream_t stream) {
    constexpr int kWeightLead = weight_lead<CODEC, MT, LIMBS, AX>();
    static_assert(kWeightLead >= 1, "no room for a weight ring");
    return launch<CODEC, MT, LIMBS, AX, kWeightLead>(weight, tiles, out, rows, columns, vectors, stream);
}

template <int CODEC>
hipError_t launch_codec(int limbs, const uint8_t* weight, const uint8_t* tiles, const GemmOutput& out,
                        uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
    // Activations: 26 KiB per stage and 32-vector tile with three limbs, 10 KiB with one; two
    // stages of lead. The weight ring (9 to 20 KiB per stage) takes the rest of LDS.
    // One 32-vector tile per workgroup with three limbs: two tiles of three-limb results do not
    // fit in registers. With one limb four tiles share the weight operands of a step; Q4_K stays at
    // two (four measured slower: 14336 x 4096 with 512 vectors 226 against 170 us - its min-term
    // instructions and a single stage of activation lead).
    // (tiles_per_workgroup() below states the same choice for the launch geometry.)
    if (limbs == 3)
        return launch_shape<CODEC, 1, 3, 2>(weight, tiles, out, rows, columns, vectors, stream);
    if (vectors <= 32)
        return launch_shape<CODEC, 1, 1, 2>(weight, tiles, out, rows, columns, vectors, stream);
    if (vectors <= 64 || CODEC == kQ4_K)
        return launch_shape<CODEC, 2, 1, 2>(weight, tiles, out, rows, columns, vectors, stream);
    return launch_shape<CODEC, 4, 1, 1>(weight, tiles, out, rows, columns, vectors, stream);
}

uint32_t tiles_per_workgroup(int32_t codec, int limbs, uint64_t vectors) {
    if (limbs != 1 || vectors <= 32) return 1;
    if (vectors <= 64 || codec == kQ4_K) return 2;
    return 4;
}

}  // namespace

hipError_t reduce_partials(const float* partials, const float* bias, const float* residual, float* y,
                           uint32_t rows, uint32_t vectors, uint32_t k_splits, hipStream_t stream) {
    const uint64_t outputs = static_cast<uint64_t>(vectors) * rows;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3(static_cast<uint32_t>((outputs + 1023) / 1024)), dim3(256), 0,
                       stream, partials, bias, residual, y, rows, outputs, k_splits);
    return hipGetLastError();
}

bool gemm_i8_supported(int32_t codec, uint64_t columns) {
    // Whole stages of 256 columns, also for the 32-wide codecs.
    return (codec == kQ8_0 || codec == kQ4_0 || codec == kQ4_K) && columns % 256 == 0 && columns > 0;
}

uint32_t gemm_i8_k_splits(int32_t codec, int limbs, uint64_t rows, uint64_t columns, uint64_t vectors) {
    // One workgroup fits a compute unit. A launch with far fewer tiles than the 256 units shares
    // the stages of K out over several workgroups per tile, no share empty.
    const uint64_t vector_tiles = (vectors + 31) / 32, per_group = tiles_per_workgroup(codec, limbs, vectors);
    const uint64_t tiles = ((rows + kRows - 1) / kRows) * ((vector_tiles + per_group - 1) / per_group);
    const uint64_t stages = columns / 256;
    if (tiles == 0 || stages < 2 || tiles >= 192) return 1;
    uint64_t splits = 256 / tiles;
    if (splits > stages) splits = stages;
    if (splits < 2) return 1;
    const uint64_t share = (stages + splits - 1) / splits;
    return static_cast<uint32_t>((stages + share - 1) / share);
}

hipError_t gemm_i8(int32_t codec, int limbs, const uint8_t* weight, const uint8_t* tiles,
                   const GemmOutput& out, uint64_t rows, uint64_t columns, uint64_t vectors,
                   hipStream_t stream) {
    if (limbs != 1 && limbs != 3) return hipErrorInvalidValue;
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns),
                   m = static_cast<uint32_t>(vectors);
    switch (codec) {
        case kQ8_0: return launch_codec<kQ8_0>(limbs, weight, tiles, out, n, k, m, stream);
        case kQ4_0: return launch_codec<kQ4_0>(limbs, weight, tiles, out, n, k, m, stream);
        case kQ4_K: return launch_codec<kQ4_K>(limbs, weight, tiles, out, n, k, m, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
