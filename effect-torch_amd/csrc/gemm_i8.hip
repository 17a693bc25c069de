// Block-scaled int8 contraction on the gfx950 matrix cores, for 4 or more vectors.
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
// MFMAs: KSPLIT = 4 of them share 32 weight rows and split the eight blocks of every
// stage between them; their accumulators meet in LDS at the end. Two more waves
// only move activations (below).
//
// Streaming. With few vectors the kernel is bound by weight bytes from HBM, and what
// matters is how many bytes each CU keeps in flight. Both operand streams run AHEAD
// stages in front of the MFMAs:
//   activations  arrive as ready-made stage blobs (see kernels.h) and are copied
//                global -> LDS by global_load_lds, 16 bytes per lane, into a ring of
//                AHEAD + 1 slots, by the two loader waves, which do nothing else;
//   weights      never touch LDS: each packed byte is needed by exactly one lane of a
//                consumer wave, which loads it into a ring of AHEAD + 1 register sets.
// The split into loader and consumer waves is what keeps both streams deep. Loads
// return in order and are counted per wave; a wave that mixes global_load_lds with
// loads into registers gets a full wait (vmcnt 0) from the compiler before every use
// of a loaded register, which drains the pipeline once per stage. Kept in separate
// waves, the loaders wait with an explicit count and the consumers' waits are the
// compiler's exact ones. One s_barrier per stage joins the two.
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

// Packed weights one lane holds for NB consecutive blocks of its row (its 16-column half).
template <int CODEC, int NB>
struct StageWeights {
    uint4 q[NB];        // the aligned 20-byte window around the 16 quant bytes: dwords 0..3
    uint32_t tail[NB];  // and dword 4 (dword 3 again if the window is not shifted)
    uint32_t d[NB];     // fp16 bits
};
template <int NB>
struct StageWeights<kQ4_K, NB> {
    uint4 header;     // d, dmin, scales[12]
    uint4 q[NB / 2];  // pair p: bytes 16*half .. +16 of its 32
};

// VMEM instructions load_stage_weights issues (for the counted wait).
template <int CODEC, int NB>
constexpr int weight_loads() {
    return CODEC == kQ4_K ? 1 + NB / 2 : 3 * NB;
}

// first_block: index of the first of the NB 32-column blocks to load.
template <int CODEC, int NB>
__device__ __forceinline__ void load_stage_weights(const uint8_t* row, uint32_t first_block, uint32_t half,
                                                   StageWeights<CODEC, NB>& w) {
    if constexpr (CODEC == kQ4_K) {
        const uint8_t* block = row + static_cast<uint64_t>(first_block >> 3) * 144u;
        const uint32_t first_pair = (first_block & 7u) >> 1;
        w.header = *reinterpret_cast<const uint4*>(block);
#pragma unroll
        for (int p = 0; p < NB / 2; p++)
            w.q[p] = *reinterpret_cast<const uint4*>(block + 16 + 32 * (first_pair + p) + 16 * half);
    } else {
        constexpr uint32_t kBytes = CODEC == kQ8_0 ? 34u : 18u;
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint8_t* block = row + static_cast<uint64_t>(first_block + b) * kBytes;
            // The 16 quant bytes start 2 bytes into a block that is itself only 2-byte aligned.
            // A misaligned 16-byte load is served piecemeal; instead load the aligned 20-byte
            // window around them (4 + 1 dwords); weight_operand() shifts by the 0 or 2 odd bytes.
            // Every dword read holds at least one byte of the block, so no read leaves the buffer's
            // pages: the fifth dword is only fetched when the window is shifted (else the fourth
            // again: a load under a branch would cost the compiler its count of loads in flight).
            const uint8_t* quants = block + (CODEC == kQ8_0 ? 2u + 16u * half : 2u);
            const uint32_t odd = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(quants)) & 3u;  // 0 or 2
            const uint8_t* window = quants - odd;
            w.q[b] = *reinterpret_cast<const uint4*>(window);
            w.tail[b] = *reinterpret_cast<const uint32_t*>(window + (odd ? 16 : 12));
            w.d[b] = *reinterpret_cast<const uint16_t*>(block);
        }
    }
}

// MFMA B operand (16 int8 weights) of local block b for this lane's half.
// The 16 quant bytes out of the aligned window (32-wide codecs).
template <int CODEC, int NB>
__device__ __forceinline__ uint4 window_quants(const StageWeights<CODEC, NB>& w, int b, bool shifted) {
    const uint4 low = w.q[b];
    if (!shifted) return low;
    return make_uint4(__builtin_amdgcn_alignbit(low.y, low.x, 16), __builtin_amdgcn_alignbit(low.z, low.y, 16),
                      __builtin_amdgcn_alignbit(low.w, low.z, 16), __builtin_amdgcn_alignbit(w.tail[b], low.w, 16));
}

// `shifted`: the block's quant bytes start 2 bytes into their aligned window (32-wide codecs).
template <int CODEC, int NB>
__device__ __forceinline__ v4i weight_operand(const StageWeights<CODEC, NB>& w, int b, uint32_t half,
                                              bool shifted) {
    if constexpr (CODEC == kQ8_0) {
        const uint4 q = window_quants<CODEC, NB>(w, b, shifted);
        return v4i{static_cast<int>(q.x), static_cast<int>(q.y), static_cast<int>(q.z), static_cast<int>(q.w)};
    } else if constexpr (CODEC == kQ4_0) {
        // element j = low nibble of byte j (j < 16), element j+16 = high nibble:
        // lanes 0-31 take the low nibbles, lanes 32-63 the high ones; value = nibble - 8.
        const uint4 q = window_quants<CODEC, NB>(w, b, shifted);
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
        v4i out;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t nib = (half ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu;
            // (nib - 8) per byte without borrows between bytes
            out[i] = static_cast<int>(((nib | 0x80808080u) - 0x08080808u) ^ 0x80808080u);
        }
        return out;
    } else {
        // sub-block 2p + side: low (side 0) or high (side 1) nibbles of pair p
        const int p = b >> 1, side = b & 1;
        const uint32_t words[4] = {w.q[p].x, w.q[p].y, w.q[p].z, w.q[p].w};
        v4i out;
#pragma unroll
        for (int i = 0; i < 4; i++)
            out[i] = static_cast<int>((side ? (words[i] >> 4) : words[i]) & 0x0f0f0f0fu);
        return out;
    }
}

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

constexpr int kConsumers = 8;  // waves that run the MFMAs: two per SIMD
constexpr int kLoaders = 2;    // waves that only copy activation blobs into LDS
constexpr int kThreads = 64 * (kConsumers + kLoaders);

template <int CODEC, int MT, int LIMBS, int KSPLIT, int AHEAD>
struct Shape {
    static constexpr int kDepth = AHEAD + 1;
    static constexpr uint32_t kBlob = tile_blob_bytes(LIMBS);
    static constexpr uint32_t kSlotBytes = MT * kBlob;
    // One global_load_lds moves 1 KiB per wave.
    static constexpr int kPieces = kSlotBytes / 1024;
    static constexpr int kRounds = kPieces / kLoaders;
    static_assert(kPieces % kLoaders == 0, "equal shares for the loader waves");
    static constexpr int kBlocksPerWave = kStageBlocks / KSPLIT;
    static constexpr int kRowGroups = kConsumers / KSPLIT;  // 32-row groups per workgroup
    static constexpr uint32_t kRows = 32 * kRowGroups;
    // vmcnt is a 6-bit counter: a smaller bound only waits for more than necessary.
    static constexpr int kLoaderWait = (AHEAD - 1) * kRounds < 63 ? (AHEAD - 1) * kRounds : 63;
    static constexpr uint32_t kExchangeBytes = (KSPLIT - 1) * kRowGroups * MT * 16 * 64 * 4;
    static constexpr uint32_t kLdsBytes =
        kDepth * kSlotBytes > kExchangeBytes ? kDepth * kSlotBytes : kExchangeBytes;
};

template <int CODEC, int MT, int LIMBS, int KSPLIT, int AHEAD>
__global__ __launch_bounds__(kThreads) void gemm_i8_kernel(
    const uint8_t* weight, const uint8_t* __restrict__ tiles, uint32_t vector_tiles,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t vectors, uint32_t row_tiles, uint32_t vector_groups) {
    using S = Shape<CODEC, MT, LIMBS, KSPLIT, AHEAD>;
    constexpr int NB = S::kBlocksPerWave;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // Workgroups are handed to the eight XCDs round-robin. All vector groups of one row tile
    // go to the same XCD, next to each other in time, so the second one finds the weights in L2.
    const uint32_t xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
    const uint32_t row_tile = (turn / vector_groups) * 8u + xcd;
    const uint32_t vector_group = turn % vector_groups;
    if (row_tile >= row_tiles) return;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: uniform branches
    const uint32_t tile0 = vector_group * MT;
    const uint32_t xblocks = columns >> 5;
    const uint32_t stages = xblocks / kStageBlocks;  // whole: columns % 256 == 0
    // Both loops run a whole number of ring turns; the stages past the end are empty.
    const uint32_t padded_stages = (stages + S::kDepth - 1) / S::kDepth * S::kDepth;

    if (wave >= static_cast<uint32_t>(kConsumers)) {
        // ---- loader waves ---------------------------------------------------------
        // Copy the activation blobs of stage s + AHEAD into ring slot (s + AHEAD) % kDepth while
        // the consumers contract stage s. One barrier per stage, matched by the consumers':
        // passing it says "stage s is in LDS" to them and "slot of stage s - 1 is free" to us.
        const uint32_t loader = wave - kConsumers;
        const auto request = [&](uint32_t stage) {
            const uint32_t s = min(stage, stages - 1u);  // past the end: a copy nobody reads
            const uint32_t slot = stage % S::kDepth;
#pragma unroll
            for (int i = 0; i < S::kRounds; i++) {
                const uint32_t piece = i * kLoaders + loader;  // 1 KiB pieces of the slot
                const uint32_t t = piece / (S::kBlob / 1024u), within = piece % (S::kBlob / 1024u);
                const uint32_t tile = min(tile0 + t, vector_tiles - 1u);
                const uint8_t* src = tiles + (static_cast<uint64_t>(s) * vector_tiles + tile) * S::kBlob +
                                     within * 1024u + lane * 16u;
                uint8_t* dst = lds + slot * S::kSlotBytes + piece * 1024u;  // + 16 * lane by the hardware
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src),
                                                 reinterpret_cast<uint4*>(dst), 16, 0, 0);
            }
        };
        for (uint32_t a = 0; a < static_cast<uint32_t>(AHEAD); a++) request(a);
        for (uint32_t stage = 0; stage < padded_stages; stage++) {
            // Loads return in order: all but the newest AHEAD - 1 requests have landed.
            __builtin_amdgcn_s_waitcnt(vmcnt_only(S::kLoaderWait));
            __builtin_amdgcn_s_barrier();
            request(stage + AHEAD);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));  // nothing may still write the ring
        if constexpr (KSPLIT > 1) {
            __builtin_amdgcn_s_barrier();  // the consumers' two exchange barriers
            __builtin_amdgcn_s_barrier();
        }
        return;
    }

    // ---- consumer waves -----------------------------------------------------------
    const uint32_t half = lane >> 5;
    const uint32_t wave_n = wave % S::kRowGroups;
    const uint32_t wave_k = wave / S::kRowGroups;
    const uint32_t n0 = row_tile * S::kRows + wave_n * 32u;
    const uint32_t m0 = tile0 * 32u;

    // This lane's weight row. Rows past the end are clamped for loads, masked at stores.
    const uint32_t n = min(n0 + (lane & 31u), rows - 1u);
    const uint64_t row_bytes = static_cast<uint64_t>(columns / block_values(CODEC)) * block_bytes(CODEC);
    const uint8_t* w_row = weight + n * row_bytes;
    const uint32_t row_parity = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(w_row));

    // Stages are whole (columns % 256 == 0): this wave contracts blocks first .. first + NB of each.
    const auto wave_first = [&](uint32_t stage) { return stage * kStageBlocks + wave_k * NB; };
    // Requests this lane's weights of a stage (past the end: the last stage again, unused).
    const auto request = [&](uint32_t stage, StageWeights<CODEC, NB>& w) {
        load_stage_weights<CODEC, NB>(w_row, wave_first(min(stage, stages - 1u)), half, w);
    };

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

    // Contracts stage `stage` from its LDS slot and the weight registers `w`.
    const auto contract = [&](uint32_t stage, const StageWeights<CODEC, NB>& w) {
        // All NB blocks, or none in the padding of the last ring turn. Written as a count that each
        // block tests on its own: as straight-line code the stage needs more registers than the
        // 168 a wave of this workgroup may hold, and spills.
        const uint32_t first_block = wave_first(stage);
        const uint32_t stage_blocks = first_block < xblocks ? min(xblocks - first_block, static_cast<uint32_t>(NB)) : 0u;
        const uint32_t b_base = wave_k * NB;  // first block of this wave inside the stage
        const uint8_t* base = lds + (stage % S::kDepth) * S::kSlotBytes;
        float d_block = 0.f, dmin_block = 0.f;
        if constexpr (CODEC == kQ4_K) {
            d_block = half_bits_to_float(w.header.x & 0xffffu);
            dmin_block = half_bits_to_float(w.header.x >> 16);
        }
#pragma unroll
        for (int bb = 0; bb < NB; bb++) {
            if (static_cast<uint32_t>(bb) < stage_blocks) {  // wave-uniform
                const uint32_t b = b_base + bb;              // block inside the stage
                bool shifted = false;
                if constexpr (CODEC != kQ4_K) {
                    // parity of the quant bytes' address, as in load_stage_weights()
                    constexpr uint32_t kBytes = CODEC == kQ8_0 ? 34u : 18u;
                    shifted = ((row_parity + (wave_first(stage) + bb) * kBytes + 2u) & 2u) != 0;
                }
                const v4i bw = weight_operand<CODEC, NB>(w, bb, half, shifted);
                float w_scale;
                if constexpr (CODEC == kQ4_K) {
                    float sc, mn;
                    q4k_scale_min(w.header, b, sc, mn);
                    w_scale = d_block * sc;
                } else {
                    w_scale = half_bits_to_float(w.d[bb]);
                }
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const uint8_t* blob = base + t * S::kBlob;
                    // Scale products s[m] * d[n] for the sixteen vectors this lane accumulates: a rank-1
                    // product in the MFMA result layout (only the k = 0 half of the lanes carries values).
                    // One 4-byte LDS read per lane instead of 64 bytes: LDS bandwidth is what this
                    // kernel runs out of first.
                    const float x_scale =
                        *reinterpret_cast<const float*>(blob + LIMBS * 8192u + b * 128u + (lane & 31u) * 4u);
                    const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(half == 0 ? x_scale : 0.f,
                                                                         half == 0 ? w_scale : 0.f, zero_f, 0, 0, 0);
                    const uint8_t* chunk = blob + (2u * b + half) * 512u + (lane & 31u) * 16u;
                    if constexpr (LIMBS == 1) {
                        const v4i ax = *reinterpret_cast<const v4i*>(chunk);
                        const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bw, zero_i, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            acc[t][r] = fmaf(static_cast<float>(c[r]), sd[r], acc[t][r]);
                    } else {
                        const v4i a0 = *reinterpret_cast<const v4i*>(chunk);
                        const v4i a1 = *reinterpret_cast<const v4i*>(chunk + 8192u);
                        const v4i a2 = *reinterpret_cast<const v4i*>(chunk + 16384u);
                        const v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bw, zero_i, 0, 0, 0);
                        const v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bw, zero_i, 0, 0, 0);
                        const v16i c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a2, bw, zero_i, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            // |c0 + 256 c1| < 2^28 is exact in int32; the top limb joins in f32
                            const float low = static_cast<float>(c0[r] + (c1[r] << 8));
                            const float all = fmaf(65536.0f, static_cast<float>(c2[r]), low);
                            acc[t][r] = fmaf(all, sd[r], acc[t][r]);
                        }
                    }
                }
            }
        }
        if constexpr (CODEC == kQ4_K) {
          if (stage_blocks > 0) {
            // min term: acc_min[m, n] += sum_g (dmin * m_g)[n] * xsum[m, g]; K = 2 per MFMA,
            // lane half h supplies sub-block 2j + h.
#pragma unroll
            for (int jj = 0; jj < NB / 2; jj++) {
                const uint32_t g = b_base + 2u * jj + half;
                float sc, mn;
                q4k_scale_min(w.header, g, sc, mn);
                const float b_operand = dmin_block * mn;
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float a_operand = *reinterpret_cast<const float*>(
                        base + t * S::kBlob + LIMBS * 8192u + 1024u + g * 128u + (lane & 31u) * 4u);
                    acc_min[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_operand, b_operand, acc_min[t], 0, 0, 0);
                }
            }
          }
        }
    };

    StageWeights<CODEC, NB> ring[S::kDepth];
#pragma unroll
    for (int a = 0; a < AHEAD; a++) {
        request(a, ring[a]);
        // Oldest stage first: the waits count back from the newest load. (`weight` is not
        // declared __restrict__ so that this compiler barrier orders its loads.)
        asm volatile("" ::: "memory");
    }

    // The ring position of a stage is a compile-time constant only if the loop is unrolled by
    // the ring size. The bodies carry no early exit (stages past the end contract nothing):
    // any extra edge in the loop's control flow makes the compiler assume that fewer loads
    // were issued behind a weight register and wait for more than it has to.
    for (uint32_t s0 = 0; s0 < padded_stages; s0 += S::kDepth) {
#pragma unroll
        for (int d = 0; d < S::kDepth; d++) {
            const uint32_t stage = s0 + d;
            // Stage `stage` is in LDS; every consumer is done with stage - 1.
            // (A plain s_barrier: __syncthreads() adds a fence that waits for every load in flight.)
            __builtin_amdgcn_s_barrier();
            request(stage + AHEAD, ring[(d + AHEAD) % S::kDepth]);
            __builtin_amdgcn_sched_barrier(0);
            contract(stage, ring[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- combine the K shares, add bias, store ----------------------------------
    if constexpr (KSPLIT > 1) {
        __syncthreads();  // the loaders arrive here with nothing in flight: the ring is free
        float* exchange = reinterpret_cast<float*>(lds);  // [wave_k - 1][wave_n][MT * 16][64 lanes]
        if (wave_k > 0) {
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float value = CODEC == kQ4_K ? acc[t][r] - acc_min[t][r] : acc[t][r];
                    exchange[((((wave_k - 1u) * S::kRowGroups + wave_n) * MT + t) * 16 + r) * 64 + lane] = value;
                }
        }
        __syncthreads();
        if (wave_k > 0) return;
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                if constexpr (CODEC == kQ4_K) acc[t][r] -= acc_min[t][r];
#pragma unroll
                for (int k = 1; k < KSPLIT; k++)
                    acc[t][r] += exchange[((((k - 1) * S::kRowGroups + wave_n) * MT + t) * 16 + r) * 64 + lane];
            }
    } else if constexpr (CODEC == kQ4_K) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][r] -= acc_min[t][r];
    }
    const uint32_t n_out = n0 + (lane & 31u);
    if (n_out < rows) {
        const float bias_value = bias != nullptr ? bias[n_out] : 0.f;
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t m = m0 + 32u * t + 8u * (r >> 2) + 4u * half + (r & 3u);
                if (m < vectors) {
                    float value = acc[t][r];
                    if (bias != nullptr) value += bias_value;
                    y[static_cast<uint64_t>(m) * rows + n_out] = value;
                }
            }
    }
}

template <int CODEC, int MT, int LIMBS, int KSPLIT, int AHEAD>
hipError_t launch(const uint8_t* weight, const uint8_t* tiles, const float* bias, float* y,
                  uint32_t rows, uint32_t columns, uint32_t vectors, hipStream_t stream) {
    using S = Shape<CODEC, MT, LIMBS, KSPLIT, AHEAD>;
    static_assert(S::kLdsBytes <= 160 * 1024, "LDS of a gfx950 CU");
    const auto kernel = gemm_i8_kernel<CODEC, MT, LIMBS, KSPLIT, AHEAD>;
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
    const uint32_t row_tiles = (rows + S::kRows - 1) / S::kRows;
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
    // Three limbs: one 32-vector tile per workgroup (28 KiB of activations per stage), 3 stages ahead.
    if (limbs == 3) return launch<CODEC, 1, 3, 4, 3>(weight, tiles, bias, y, rows, columns, vectors, stream);
    if (vectors <= 32) return launch<CODEC, 1, 1, 4, 3>(weight, tiles, bias, y, rows, columns, vectors, stream);
    return launch<CODEC, 2, 1, 4, 2>(weight, tiles, bias, y, rows, columns, vectors, stream);
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
