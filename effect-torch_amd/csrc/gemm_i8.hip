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
// Operand streams. Four more waves, the loaders, do nothing but copy the operands
// of stage s + AHEAD into an LDS ring of AHEAD + 1 slots with global_load_lds while
// the consumers contract stage s; one s_barrier per stage joins the two groups.
//   activations  arrive as ready-made stage blobs (see kernels.h): a linear copy;
//   weights      are gathered so that LDS holds every MFMA B operand where the lane
//                that needs it reads one 16-byte slot at base + 16 * lane: loader lane
//                l fetches the 16 quant bytes of row l % 32 and column half l / 32
//                straight from the packed row (for the 2-byte aligned Q8_0 / Q4_0 blocks:
//                the dword-aligned window around them, see WeightLayout).
// Why separate waves: loads return in order and are counted per wave; a wave that
// mixes global_load_lds with loads into registers gets a full wait (vmcnt 0) from
// the compiler before every use of a loaded register, and a consumer wave whose
// lanes each read another weight row stalls in the address unit for about 64 clocks
// per load. The loaders absorb both: they wait with an explicit count, nothing else
// depends on them, and the consumers issue no global loads at all until they store.
//
// The consumers run each stage as a software pipeline over its (block, tile) steps: LDS
// reads one step ahead of the MFMAs, the f32 epilogue one step behind them, so that the
// matrix pipe, the VALU and LDS work on three different steps at a time.
//
// MFMA operand roles: A = activations, B = weights. A lane of the 32x32 result holds
// one weight row n = lane % 32 and sixteen vectors m = 8*(r/4) + 4*(lane/32) + r%4,
// and every result register row is stored as 128 contiguous bytes of y.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kStageBlocks = 8;  // 32-column blocks per stage
constexpr int kConsumers = 8;    // waves that run the MFMAs: two per SIMD
constexpr int kLoaders = 4;      // waves that only copy operands into LDS: one per SIMD
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

// Weight region of an LDS slot, per codec. "Quant pieces" are 1 KiB: 64 slots of 16 bytes.
//   Q4_K  piece (g, p): slot l = bytes 16*(l/32) .. +16 of nibble pair p of row 32g + l%32.
//         header pieces of 1 KiB, one per two row groups h: slot l = header of row 64h + l.
//   Q8_0, Q4_0: blocks are only 2-byte aligned, and a gather of misaligned 16-byte pieces is
//         served several times slower than an aligned one. So LDS receives the dword-aligned
//         20-byte WINDOW that starts at or 2 bytes before `start` = block + 16 * half
//         (Q8_0) or block (Q4_0): dwords 0..3 in a quant piece, dword 4 in a "tail" piece of
//         256 bytes. The window holds start .. start + 18: the fp16 scale (half 0) and 16
//         quant bytes at start + 2. The consumer shifts by the odd 2 bytes where needed.
//         Q8_0 piece (g, b): slot l = window of row 32g + l%32, block b, column half l/32.
//         Q4_0 piece (g, j): slot l = window of row 32g + l%32, block 2j + l/32 (both nibble halves).
template <int CODEC>
struct WeightLayout {
    static constexpr bool kSuper = CODEC == kQ4_K;
    static constexpr uint32_t kBlockBytes = CODEC == kQ8_0 ? 34u : 18u;  // 32-wide codecs
    static constexpr int kQuantPieces = CODEC == kQ8_0 ? 8 : 4;          // per row group and stage
    static constexpr int kQuantJobs = kRowGroups * kQuantPieces;
    static constexpr int kSmallJobs = kSuper ? kRowGroups / 2 : kQuantJobs;  // headers / tails
    static constexpr uint32_t kSmallBytes = kSuper ? 1024u : 256u;
    static constexpr uint32_t kSmallAt = kQuantJobs * 1024u;  // offset of the small pieces
    static constexpr uint32_t kBytes = kSmallAt + kSmallJobs * kSmallBytes;
    static constexpr int kJobs = kQuantJobs + kSmallJobs;
};

// Start of the window of (row pointer, block index, column half): see WeightLayout.
template <int CODEC>
__device__ __forceinline__ const uint8_t* window_start(const uint8_t* row, uint64_t block, uint32_t half) {
    return row + block * WeightLayout<CODEC>::kBlockBytes + (CODEC == kQ8_0 ? 16u * half : 0u);
}

template <int CODEC, int MT, int LIMBS, int AHEAD>
struct Shape {
    using W = WeightLayout<CODEC>;
    static constexpr int kDepth = AHEAD + 1;
    static constexpr uint32_t kBlob = tile_blob_bytes(LIMBS);        // in memory, padded
    static constexpr uint32_t kTile = LIMBS * 8192u + 2048u;          // in LDS: operands and both tables
    static constexpr uint32_t kActivationBytes = MT * kTile;
    static constexpr uint32_t kSlotBytes = kActivationBytes + W::kBytes;
    // One global_load_lds moves up to 1 KiB per wave.
    static constexpr int kActivationJobs = kActivationBytes / 1024;
    static constexpr int kJobs = kActivationJobs + W::kJobs;
    // Every loader issues the same number of copies per stage (for its counted wait): jobs are
    // dealt round-robin and the last round wraps around to the first jobs, copied twice.
    static constexpr int kRounds = (kJobs + kLoaders - 1) / kLoaders;
    static_assert(kJobs >= kLoaders, "the wrap-around of the last round needs a full first round");
    // vmcnt is a 6-bit counter: a smaller bound only waits for more than necessary.
    static constexpr int kLoaderWait = (AHEAD - 1) * kRounds < 63 ? (AHEAD - 1) * kRounds : 63;
    static constexpr uint32_t kExchangeBytes = (kSplit - 1) * kRowGroups * MT * 16 * 64 * 4;
    static constexpr uint32_t kLdsBytes =
        kDepth * kSlotBytes > kExchangeBytes ? kDepth * kSlotBytes : kExchangeBytes;
};

template <int CODEC, int MT, int LIMBS, int AHEAD>
__global__ __launch_bounds__(kThreads) void gemm_i8_kernel(
    const uint8_t* __restrict__ weight, const uint8_t* __restrict__ tiles, uint32_t vector_tiles,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t vectors, uint32_t row_tiles, uint32_t vector_groups) {
    using S = Shape<CODEC, MT, LIMBS, AHEAD>;
    using W = WeightLayout<CODEC>;
    constexpr int NB = kBlocksPerWave;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // Workgroups are handed to the eight XCDs round-robin. All vector groups of one row tile
    // go to the same XCD, next to each other in time, so the later ones find the weights in L2.
    const uint32_t xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
    const uint32_t row_tile = (turn / vector_groups) * 8u + xcd;
    const uint32_t vector_group = turn % vector_groups;
    if (row_tile >= row_tiles) return;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: uniform branches
    const uint32_t tile0 = vector_group * MT;
    const uint32_t stages = columns / 256u;  // whole: columns % 256 == 0
    // Both loops run a whole number of ring turns; the stages past the end are empty.
    const uint32_t padded_stages = (stages + S::kDepth - 1) / S::kDepth * S::kDepth;
    const uint64_t row_bytes = static_cast<uint64_t>(columns / block_values(CODEC)) * block_bytes(CODEC);
    const uint32_t row0 = row_tile * kRows;

    if (wave >= static_cast<uint32_t>(kConsumers)) {
        // ---- loader waves ---------------------------------------------------------
        const uint32_t loader = wave - kConsumers;
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);  // past the end: a copy nobody reads
            uint8_t* slot = lds + (stage % S::kDepth) * S::kSlotBytes;
#pragma unroll
            for (int i = 0; i < S::kRounds; i++) {
                uint32_t job = i * kLoaders + loader;
                if (job >= static_cast<uint32_t>(S::kJobs)) job -= S::kJobs;
                if (job < static_cast<uint32_t>(S::kActivationJobs)) {
                    // 1 KiB of the activation blobs, as they lie in memory
                    const uint32_t t = job / (S::kTile / 1024u), within = job % (S::kTile / 1024u);
                    const uint32_t tile = min(tile0 + t, vector_tiles - 1u);
                    const uint8_t* src = tiles + (static_cast<uint64_t>(s) * vector_tiles + tile) * S::kBlob +
                                         within * 1024u + lane * 16u;
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                     reinterpret_cast<uint4*>(slot + job * 1024u), 16, 0, 0);
                    continue;
                }
                job -= S::kActivationJobs;
                uint8_t* region = slot + S::kActivationBytes;
                if (job < static_cast<uint32_t>(W::kQuantJobs)) {
                    const uint32_t g = job / W::kQuantPieces, piece = job % W::kQuantPieces;
                    const uint32_t row = min(row0 + 32u * g + (lane & 31u), rows - 1u);
                    const uint8_t* src = weight + row * row_bytes;
                    if constexpr (CODEC == kQ4_K) {
                        src += static_cast<uint64_t>(s) * 144u + 16u + 32u * piece + 16u * (lane >> 5);
                    } else {
                        const uint64_t block = CODEC == kQ8_0 ? static_cast<uint64_t>(s) * kStageBlocks + piece
                                                              : static_cast<uint64_t>(s) * kStageBlocks + 2u * piece + (lane >> 5);
                        src = window_start<CODEC>(src, block, lane >> 5);
                        src -= reinterpret_cast<uintptr_t>(src) & 2u;  // dword aligned
                    }
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                     reinterpret_cast<uint4*>(region + job * 1024u), 16, 0, 0);
                    continue;
                }
                job -= W::kQuantJobs;
                if constexpr (CODEC == kQ4_K) {
                    const uint32_t row = min(row0 + 64u * job + lane, rows - 1u);
                    const uint8_t* src = weight + row * row_bytes + static_cast<uint64_t>(s) * 144u;
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                     reinterpret_cast<uint4*>(region + W::kSmallAt + job * 1024u), 16,
                                                     0, 0);
                } else {
                    // dword 4 of the same windows
                    const uint32_t g = job / W::kQuantPieces, piece = job % W::kQuantPieces;
                    const uint32_t row = min(row0 + 32u * g + (lane & 31u), rows - 1u);
                    const uint64_t block = CODEC == kQ8_0 ? static_cast<uint64_t>(s) * kStageBlocks + piece
                                                          : static_cast<uint64_t>(s) * kStageBlocks + 2u * piece + (lane >> 5);
                    const uint8_t* src = window_start<CODEC>(weight + row * row_bytes, block, lane >> 5);
                    src -= reinterpret_cast<uintptr_t>(src) & 2u;
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(src + 16),
                                                     reinterpret_cast<uint32_t*>(region + W::kSmallAt + job * 256u), 4,
                                                     0, 0);
                }
            }
        };
        for (uint32_t a = 0; a < static_cast<uint32_t>(AHEAD); a++) request(a);
        for (uint32_t stage = 0; stage < padded_stages; stage++) {
            // Loads return in order: all but the newest AHEAD - 1 requests have landed.
            __builtin_amdgcn_s_waitcnt(vmcnt_only(S::kLoaderWait));
            // Passing the barrier says "stage is in LDS" to the consumers and "the slot of
            // stage - 1 is free" to the loaders.
            __builtin_amdgcn_s_barrier();
            request(stage + AHEAD);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));  // nothing may still write the ring
        __builtin_amdgcn_s_barrier();               // the consumers' two exchange barriers
        __builtin_amdgcn_s_barrier();
        return;
    }

    // ---- consumer waves -----------------------------------------------------------
    const uint32_t half = lane >> 5;
    const uint32_t wave_n = wave % kRowGroups;  // row group
    const uint32_t wave_k = wave / kRowGroups;  // share of the stage's blocks
    const uint32_t n0 = row0 + wave_n * 32u;
    const uint32_t m0 = tile0 * 32u;
    // Low address bits of this lane's weight row (the loaders clamp rows the same way).
    const uint32_t row_parity = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>(weight + min(n0 + (lane & 31u), rows - 1u) * row_bytes));

    float acc[MT][16];
    v16f acc_min[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc[t][r] = 0.f;
            acc_min[t][r] = 0.f;
        }
    v16i zero_i;
    v16f zero_f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        zero_i[r] = 0;
        zero_f[r] = 0.f;
    }

    for (uint32_t stage = 0; stage < padded_stages; stage++) {
        // A plain s_barrier: __syncthreads() would add a fence the loop does not need.
        __builtin_amdgcn_s_barrier();
        if (stage >= stages) continue;  // padding of the last ring turn
        const uint8_t* slot = lds + (stage % S::kDepth) * S::kSlotBytes;
        const uint8_t* region = slot + S::kActivationBytes;
        const uint32_t b_base = wave_k * NB;  // first block of this wave inside the stage

        uint4 header = make_uint4(0u, 0u, 0u, 0u);
        float d_block = 0.f, dmin_block = 0.f;
        if constexpr (CODEC == kQ4_K) {
            header = *reinterpret_cast<const uint4*>(region + W::kSmallAt + (wave_n >> 1) * 1024u +
                                                    ((wave_n & 1u) * 32u + (lane & 31u)) * 16u);
            d_block = half_bits_to_float(header.x & 0xffffu);
            dmin_block = half_bits_to_float(header.x >> 16);
        }
        if constexpr (CODEC == kQ4_K) {
            // min term: acc_min[m, n] += sum_g (dmin * m_g)[n] * xsum[m, g]; K = 2 per MFMA,
            // lane half h supplies sub-block 2j + h. First in the stage: its LDS reads go out with
            // the other operands' and its MFMAs run under the first steps.
#pragma unroll
            for (int jj = 0; jj < NB / 2; jj++) {
                const uint32_t g = b_base + 2u * jj + half;
                float sc, mn;
                q4k_scale_min(header, g, sc, mn);
                const float b_operand = dmin_block * mn;
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float a_operand = *reinterpret_cast<const float*>(
                        slot + t * S::kTile + LIMBS * 8192u + 1024u + g * 128u + (lane & 31u) * 4u);
                    acc_min[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_operand, b_operand, acc_min[t], 0, 0, 0);
                }
            }
        }
        // B operands (16 int8 weights of row n, this lane's half of the block) and block scales
        v4i bw[NB];
        float w_scale[NB];
#pragma unroll
        for (int bb = 0; bb < NB; bb++) {
            const uint32_t b = b_base + bb;  // block inside the stage
            if constexpr (CODEC == kQ4_K) {
                // sub-block 2p + side: low (side 0) or high (side 1) nibbles of pair p
                const uint4 raw = *reinterpret_cast<const uint4*>(region + (wave_n * 4u + (b >> 1)) * 1024u + lane * 16u);
                const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; i++)
                    bw[bb][i] = static_cast<int>(((b & 1u) ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu);
                float sc, mn;
                q4k_scale_min(header, b, sc, mn);
                w_scale[bb] = d_block * sc;
            } else {
                // This lane's window: piece and slot as the loaders filled them.
                const uint32_t piece = CODEC == kQ8_0 ? wave_n * 8u + b : wave_n * 4u + (b >> 1);
                const uint32_t in_piece = CODEC == kQ8_0 ? lane : (b & 1u) * 32u + (lane & 31u);
                const uint4 low = *reinterpret_cast<const uint4*>(region + piece * 1024u + in_piece * 16u);
                const uint32_t tail = *reinterpret_cast<const uint32_t*>(region + W::kSmallAt + piece * 256u + in_piece * 4u);
                // The scale sits in the window of column half 0 (for Q4_0 that is this window).
                const uint32_t scale_word =
                    CODEC == kQ8_0 ? *reinterpret_cast<const uint32_t*>(region + piece * 1024u + (lane & 31u) * 16u) : low.x;
                // Do the windows begin 2 bytes before their start? (same arithmetic as the loaders')
                const uint32_t block_at = row_parity + (stage * kStageBlocks + b) * W::kBlockBytes;
                const bool scale_shifted = (block_at & 2u) != 0;
                const bool shifted = ((block_at + (CODEC == kQ8_0 ? 16u * half : 0u)) & 2u) != 0;
                w_scale[bb] = half_bits_to_float(scale_shifted ? scale_word >> 16 : scale_word & 0xffffu);
                // quant bytes: window + 4 if shifted, window + 2 if not
                uint32_t words[4];
                words[0] = shifted ? low.y : __builtin_amdgcn_alignbit(low.y, low.x, 16);
                words[1] = shifted ? low.z : __builtin_amdgcn_alignbit(low.z, low.y, 16);
                words[2] = shifted ? low.w : __builtin_amdgcn_alignbit(low.w, low.z, 16);
                words[3] = shifted ? tail : __builtin_amdgcn_alignbit(tail, low.w, 16);
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
            w_scale[bb] = half == 0 ? w_scale[bb] : 0.f;
        }

        // The NB * MT (block, tile) steps of the stage as a software pipeline. Each step reads its
        // A operands (and the activation scales) from LDS one step ahead, issues its MFMAs, and
        // runs the f32 epilogue of an earlier step while they execute: with one limb the previous
        // step's (its results are double-buffered), with three limbs its own (three results of
        // sixteen registers each leave no room for a second set).
        constexpr int kSteps = NB * MT;
        const auto read_step = [&](int step, v4i (&a)[LIMBS], float& x_scale) {
            const uint32_t b = b_base + step / MT;
            const uint8_t* blob = slot + (step % MT) * S::kTile;
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
                    acc[t][r] = fmaf(static_cast<float>(c[0][r]), sd[r], acc[t][r]);
                } else {
                    // |c0 + 256 c1| < 2^28 is exact in int32; the top limb joins in f32
                    const float low = static_cast<float>(c[0][r] + (c[1][r] << 8));
                    const float all = fmaf(65536.0f, static_cast<float>(c[2][r]), low);
                    acc[t][r] = fmaf(all, sd[r], acc[t][r]);
                }
            }
        };
        v4i a_next[LIMBS];
        float x_scale_next;
        read_step(0, a_next, x_scale_next);
        v16f sd_previous;
        v16i c_previous[LIMBS];
#pragma unroll
        for (int step = 0; step < kSteps; step++) {
            const int bb = step / MT;
            // Scale products s[m] * d[n] for the sixteen vectors this lane accumulates: a rank-1
            // product in the MFMA result layout.
            const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? x_scale_next : 0.f, w_scale[bb],
                                                                 zero_f, 0, 0, 0);
            v16i c[LIMBS];
#pragma unroll
            for (int l = 0; l < LIMBS; l++)
                c[l] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_next[l], bw[bb], zero_i, 0, 0, 0);
            if (step + 1 < kSteps) read_step(step + 1, a_next, x_scale_next);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (LIMBS == 1) {
                if (step > 0) epilogue(step - 1, sd_previous, c_previous);
                sd_previous = sd;
                c_previous[0] = c[0];
            } else {
                epilogue(step, sd, c);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (LIMBS == 1) epilogue(kSteps - 1, sd_previous, c_previous);
    }

    // ---- combine the K shares, add bias, store ----------------------------------
    __syncthreads();  // the loaders arrive here with nothing in flight: the ring is free
    float* exchange = reinterpret_cast<float*>(lds);  // [wave_k - 1][wave_n][MT * 16][64 lanes]
    if (wave_k > 0) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float value = CODEC == kQ4_K ? acc[t][r] - acc_min[t][r] : acc[t][r];
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
            float value = CODEC == kQ4_K ? acc[t][r] - acc_min[t][r] : acc[t][r];
#pragma unroll
            for (int k = 1; k < kSplit; k++)
                value += exchange[((((k - 1) * kRowGroups + wave_n) * MT + t) * 16 + r) * 64 + lane];
            const uint32_t m = m0 + 32u * t + 8u * (r >> 2) + 4u * half + (r & 3u);
            if (n_out < rows && m < vectors) y[static_cast<uint64_t>(m) * rows + n_out] = value + bias_value;
        }
        __builtin_amdgcn_sched_barrier(0);  // tile by tile: the sums of all tiles at once do not fit
    }
}

template <int CODEC, int MT, int LIMBS, int AHEAD>
hipError_t launch(const uint8_t* weight, const uint8_t* tiles, const float* bias, float* y,
                  uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
    using S = Shape<CODEC, MT, LIMBS, AHEAD>;
    static_assert(S::kLdsBytes <= 160 * 1024, "LDS of a gfx950 CU");
    const auto kernel = gemm_i8_kernel<CODEC, MT, LIMBS, AHEAD>;
    // More than 64 KiB of dynamic LDS has to be allowed once per kernel and device.
    static bool allowed[64] = {};
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    if (!allowed[device]) {
        if (hipError_t status =
                hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, S::kLdsBytes))
            return status;
        allowed[device] = true;
    }
    const uint32_t vector_tiles = (vectors + 31u) / 32u;
    const uint32_t vector_groups = (vector_tiles + MT - 1) / MT;
    const uint32_t row_tiles = (rows + kRows - 1) / kRows;
    const uint64_t grid = static_cast<uint64_t>((row_tiles + 7u) / 8u) * 8u * vector_groups;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), S::kLdsBytes, stream,
                       weight, tiles, vector_tiles, bias, y, rows, columns, vectors, row_tiles,
                       vector_groups);
    return hipGetLastError();
}

template <int CODEC>
hipError_t launch_codec(int limbs, const uint8_t* weight, const uint8_t* tiles, const float* bias,
                        float* y, uint32_t rows, uint32_t columns, uint32_t vectors,
                        hipStream_t stream) {
    // The ring depth is what LDS allows: 26 KiB of activations per stage and 32 vectors with
    // three limbs, 10 KiB with one; 9 to 18 KiB of weights.
    if (limbs == 3) {
        constexpr int kAhead = CODEC == kQ8_0 ? 2 : 3;
        // One 32-vector tile per workgroup: two tiles of three-limb results do not fit in registers.
        return launch<CODEC, 1, 3, kAhead>(weight, tiles, bias, y, rows, columns, vectors, stream);
    }
    if (vectors <= 32) return launch<CODEC, 1, 1, 3>(weight, tiles, bias, y, rows, columns, vectors, stream);
    // Q4_K carries a second accumulator (the min term): four tiles of both do not fit in registers.
    if (vectors <= 64 || CODEC == kQ4_K)
        return launch<CODEC, 2, 1, (CODEC == kQ8_0 ? 2 : 3)>(weight, tiles, bias, y, rows, columns, vectors, stream);
    return launch<CODEC, (CODEC == kQ4_K ? 2 : 4), 1, (CODEC == kQ4_K ? 3 : 1)>(weight, tiles, bias, y, rows, columns,
                                                                            vectors, stream);
}

}  // namespace

bool gemm_i8_supported(int32_t codec, uint64_t columns) {
    // Whole stages of 256 columns, also for the 32-wide codecs.
    return (codec == kQ8_0 || codec == kQ4_0 || codec == kQ4_K) && columns % 256 == 0 && columns > 0;
}

hipError_t gemm_i8(int32_t codec, int limbs, const uint8_t* weight, const uint8_t* tiles,
                   const float* bias, float* y, uint64_t rows, uint64_t columns, uint64_t vectors,
                   hipStream_t stream) {
    if (limbs != 1 && limbs != 3) return hipErrorInvalidValue;
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns),
                   m = static_cast<uint32_t>(vectors);
    switch (codec) {
        case kQ8_0: return launch_codec<kQ8_0>(limbs, weight, tiles, bias, y, n, k, m, stream);
        case kQ4_0: return launch_codec<kQ4_0>(limbs, weight, tiles, bias, y, n, k, m, stream);
        case kQ4_K: return launch_codec<kQ4_K>(limbs, weight, tiles, bias, y, n, k, m, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
