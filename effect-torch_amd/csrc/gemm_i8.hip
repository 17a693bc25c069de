// Block-scaled int8 contraction on the gfx950 matrix cores, for 4 or more vectors.
//
//   Q8_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i qw[n,b,i] * qx[m,b,i])
//   Q4_0:  y[m, n] = sum_b (d[n,b] * s[m,b]) * (sum_i (nib[n,b,i] - 8) * qx[m,b,i])
//   Q4_K:  y[m, n] = sum_g (d*sc_g)[n] * s[m,g] * (sum_i nib * qx)  -  sum_g (dmin*m_g)[n] * xf[m,g]
// b / g index 32-column blocks; xf[m, g] is the block's activation sum in f32.
// The inner sums are exact int32 from v_mfma_i32_32x32x32_i8, whose K = 32 is
// exactly one quantisation block; the block scales are applied by an f32
// epilogue on the VALU after every MFMA. The Q4_K "min" term is a small f32
// GEMM of its own (inner dimension K/32) and runs on v_mfma_f32_32x32x2f32
// straight into a second accumulator, with no epilogue.
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
// Tiling. A workgroup of four waves owns BN weight rows x BM = 32*MT vectors and
// walks K in stages of eight blocks (256 columns, one Q4_K super-block).
//   KSPLIT = 1: BN = 128, each wave 32 rows, all eight blocks of a stage.
//   KSPLIT = 2: BN = 64, two waves share 32 rows and take four blocks each; their
//               accumulators meet in LDS at the end. Used when there are too few
//               128-row tiles to fill 256 CUs.
// Activations of a stage go global -> registers -> LDS (XOR-swizzled rows, so the
// 16-byte MFMA operand reads are conflict free) one stage ahead of their use.
// Weights never touch LDS: each packed byte is needed by exactly one lane, which
// loads it one stage ahead into registers; MFMA operand roles are A = activations,
// B = weights, so a lane of the 32x32 result holds one weight row (its block
// scale is one value) and sixteen vectors, and every result register row is
// stored as 128 contiguous bytes of y.
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

struct __attribute__((packed, aligned(2))) Bytes16 {
    uint32_t v[4];
};

constexpr int kStageBlocks = 8;                   // 32-column blocks per stage
constexpr int kStageBytes = 32 * kStageBlocks;    // int8 activations per vector and stage
constexpr int kChunksPerRow = kStageBytes / 16;   // 16-byte chunks per vector and stage

// Position of 16-byte chunk c of vector-row m inside its 256-byte LDS row.
__device__ __forceinline__ uint32_t x_chunk_slot(uint32_t m, uint32_t c) { return c ^ (m & 15u); }

// Packed weights one lane holds for NB consecutive blocks of its row (its 16-column half).
template <int CODEC, int NB>
struct StageWeights {
    uint4 q[NB];
    uint32_t d[NB];  // fp16 bits
};
template <int NB>
struct StageWeights<kQ4_K, NB> {
    uint4 header;     // d, dmin, scales[12]
    uint4 q[NB / 2];  // pair p: bytes 16*half .. +16 of its 32
};

// first_block: index of the first 32-column block to load; blocks: how many of the NB exist.
template <int CODEC, int NB>
__device__ __forceinline__ void load_stage_weights(const uint8_t* row, uint32_t first_block,
                                                   uint32_t blocks, uint32_t half,
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
            // Blocks past the end of the row re-read an existing block; they are not used.
            const uint32_t index = b < static_cast<int>(blocks) ? first_block + b : 0u;
            const uint8_t* block = row + static_cast<uint64_t>(index) * kBytes;
            const uint32_t offset = CODEC == kQ8_0 ? 2u + 16u * half : 2u;
            const Bytes16 raw = *reinterpret_cast<const Bytes16*>(block + offset);
            w.q[b] = make_uint4(raw.v[0], raw.v[1], raw.v[2], raw.v[3]);
            w.d[b] = *reinterpret_cast<const uint16_t*>(block);
        }
    }
}

// MFMA B operand (16 int8 weights) of local block b for this lane's half.
template <int CODEC, int NB>
__device__ __forceinline__ v4i weight_operand(const StageWeights<CODEC, NB>& w, int b, uint32_t half) {
    if constexpr (CODEC == kQ8_0) {
        return v4i{static_cast<int>(w.q[b].x), static_cast<int>(w.q[b].y), static_cast<int>(w.q[b].z),
                   static_cast<int>(w.q[b].w)};
    } else if constexpr (CODEC == kQ4_0) {
        // element j = low nibble of byte j (j < 16), element j+16 = high nibble:
        // lanes 0-31 take the low nibbles, lanes 32-63 the high ones; value = nibble - 8.
        const uint32_t words[4] = {w.q[b].x, w.q[b].y, w.q[b].z, w.q[b].w};
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
__device__ __forceinline__ void q4k_scale_min(const uint4& header, int g, float& scale, float& min) {
    const uint32_t shift = 8u * (g & 3);
    const uint32_t s0 = (header.y >> shift) & 0xffu;  // scales[g & 3]
    const uint32_t s1 = (header.z >> shift) & 0xffu;  // scales[4 + (g & 3)]
    const uint32_t s2 = (header.w >> shift) & 0xffu;  // scales[8 + (g & 3)]
    const uint32_t sc = g < 4 ? (s0 & 63u) : ((s2 & 0x0fu) | ((s0 >> 6) << 4));
    const uint32_t mn = g < 4 ? (s1 & 63u) : ((s2 >> 4) | ((s1 >> 6) << 4));
    scale = static_cast<float>(sc);
    min = static_cast<float>(mn);
}

template <int MT, int LIMBS>
struct alignas(16) StageLds {
    uint8_t x[LIMBS][32 * MT][kStageBytes];  // [limb][vector][swizzled chunks]
    float scale[kStageBlocks][32 * MT];
    float xsum[kStageBlocks][32 * MT];
};

template <int CODEC, int MT, int LIMBS, int KSPLIT>
__global__ __launch_bounds__(256) void gemm_i8_kernel(
    const uint8_t* __restrict__ weight, const int8_t* __restrict__ q, uint64_t limb_stride,
    const float* __restrict__ scale, const float* __restrict__ xsum, uint32_t table_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t vectors) {
    constexpr int BM = 32 * MT;
    constexpr int BN = 128 / KSPLIT;
    constexpr int kXChunks = LIMBS * BM * kChunksPerRow;  // 16-byte chunks of a stage
    constexpr int kXPerThread = (kXChunks + 255) / 256;
    constexpr int kTableQuads = kStageBlocks * BM / 4;    // float4s of one table per stage
    constexpr int kTablePerThread = (kTableQuads + 255) / 256;
    constexpr int kBlocksPerWave = kStageBlocks / KSPLIT;
    __shared__ StageLds<MT, LIMBS> lds;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t half = lane >> 5;
    const uint32_t wave_n = KSPLIT == 1 ? wave : (wave & 1u);
    const uint32_t wave_k = KSPLIT == 1 ? 0u : (wave >> 1);
    const uint32_t n0 = blockIdx.x * BN + wave_n * 32u;
    const uint32_t m0 = blockIdx.y * BM;
    const uint32_t xblocks = columns >> 5;
    const uint32_t stages = (xblocks + kStageBlocks - 1) / kStageBlocks;

    // This lane's weight row. Rows past the end are clamped for loads, masked at stores.
    const uint32_t n = min(n0 + (lane & 31u), rows - 1u);
    const uint64_t row_bytes = static_cast<uint64_t>(columns / block_values(CODEC)) * block_bytes(CODEC);
    const uint8_t* w_row = weight + n * row_bytes;

    // ---- staging helpers --------------------------------------------------
    uint4 x_regs[kXPerThread];
    float4 s_regs[kTablePerThread], f_regs[kTablePerThread];
    auto load_x_regs = [&](uint32_t stage) {
        const uint32_t k0 = stage * kStageBytes;
#pragma unroll
        for (int i = 0; i < kXPerThread; i++) {
            const uint32_t c = threadIdx.x + i * 256u;
            x_regs[i] = make_uint4(0u, 0u, 0u, 0u);
            if (c < static_cast<uint32_t>(kXChunks)) {
                const uint32_t limb = c / (BM * kChunksPerRow);
                const uint32_t rest = c - limb * (BM * kChunksPerRow);
                const uint32_t m = rest / kChunksPerRow, chunk = rest % kChunksPerRow;
                const uint32_t column = k0 + 16u * chunk;
                if (m0 + m < vectors && column < columns)
                    x_regs[i] = *reinterpret_cast<const uint4*>(
                        q + limb * limb_stride + static_cast<uint64_t>(m0 + m) * columns + column);
            }
        }
#pragma unroll
        for (int i = 0; i < kTablePerThread; i++) {
            const uint32_t t = threadIdx.x + i * 256u;
            s_regs[i] = f_regs[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (t < static_cast<uint32_t>(kTableQuads)) {
                const uint32_t b = t / (BM / 4), quad = t % (BM / 4);
                const uint32_t block = stage * kStageBlocks + b;
                if (block < xblocks && m0 + 4u * quad < table_stride) {
                    // The tables are padded to a multiple of 32 vectors: whole quads are inside.
                    const uint64_t at = static_cast<uint64_t>(block) * table_stride + m0 + 4u * quad;
                    s_regs[i] = *reinterpret_cast<const float4*>(scale + at);
                    f_regs[i] = *reinterpret_cast<const float4*>(xsum + at);
                }
            }
        }
    };
    auto store_x_regs = [&]() {
#pragma unroll
        for (int i = 0; i < kXPerThread; i++) {
            const uint32_t c = threadIdx.x + i * 256u;
            if (c < static_cast<uint32_t>(kXChunks)) {
                const uint32_t limb = c / (BM * kChunksPerRow);
                const uint32_t rest = c - limb * (BM * kChunksPerRow);
                const uint32_t m = rest / kChunksPerRow, chunk = rest % kChunksPerRow;
                *reinterpret_cast<uint4*>(&lds.x[limb][m][16u * x_chunk_slot(m, chunk)]) = x_regs[i];
            }
        }
#pragma unroll
        for (int i = 0; i < kTablePerThread; i++) {
            const uint32_t t = threadIdx.x + i * 256u;
            if (t < static_cast<uint32_t>(kTableQuads)) {
                const uint32_t b = t / (BM / 4), quad = t % (BM / 4);
                *reinterpret_cast<float4*>(&lds.scale[b][4u * quad]) = s_regs[i];
                *reinterpret_cast<float4*>(&lds.xsum[b][4u * quad]) = f_regs[i];
            }
        }
    };

    // ---- accumulators -------------------------------------------------------
    float acc[MT][16];
    v16f acc_min[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc[t][r] = 0.f;
            acc_min[t][r] = 0.f;
        }
    v16i zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0;

    // Blocks of stage `stage` this wave contracts: wave_first(stage) .. +wave_count(stage).
    const auto wave_first = [&](uint32_t stage) { return stage * kStageBlocks + wave_k * kBlocksPerWave; };
    const auto wave_count = [&](uint32_t stage) {
        const uint32_t first = wave_first(stage);
        return first < xblocks ? min(xblocks - first, static_cast<uint32_t>(kBlocksPerWave)) : 0u;
    };
    StageWeights<CODEC, kBlocksPerWave> w_next;
    load_x_regs(0);
    load_stage_weights<CODEC, kBlocksPerWave>(w_row, wave_first(0), wave_count(0), half, w_next);

    for (uint32_t stage = 0; stage < stages; stage++) {
        __syncthreads();  // the previous stage has been read
        store_x_regs();
        const StageWeights<CODEC, kBlocksPerWave> w = w_next;
        __syncthreads();
        if (stage + 1 < stages) {
            load_x_regs(stage + 1);
            load_stage_weights<CODEC, kBlocksPerWave>(w_row, wave_first(stage + 1), wave_count(stage + 1),
                                                      half, w_next);
        }
        const uint32_t stage_blocks = wave_count(stage);
        const uint32_t b_base = wave_k * kBlocksPerWave;  // first block of this wave inside the stage

        float d_block = 0.f, dmin_block = 0.f;
        if constexpr (CODEC == kQ4_K) {
            d_block = half_bits_to_float(w.header.x & 0xffffu);
            dmin_block = half_bits_to_float(w.header.x >> 16);
        }
#pragma unroll
        for (int bb = 0; bb < kBlocksPerWave; bb++) {
            if (static_cast<uint32_t>(bb) < stage_blocks) {  // wave-uniform
                const uint32_t b = b_base + bb;  // block inside the stage: LDS row and chunk index
                const v4i bw = weight_operand<CODEC, kBlocksPerWave>(w, bb, half);
                float w_scale;
                if constexpr (CODEC == kQ4_K) {
                    float sc, mn;
                    q4k_scale_min(w.header, static_cast<int>(b), sc, mn);
                    w_scale = d_block * sc;
                } else {
                    w_scale = half_bits_to_float(w.d[bb]);
                }
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const uint32_t m = 32u * t + (lane & 31u);
                    // block scales of the sixteen vectors this lane accumulates
                    float sd[16];
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 s4 =
                            *reinterpret_cast<const float4*>(&lds.scale[b][32 * t + 8 * g + 4 * half]);
                        sd[4 * g + 0] = s4.x * w_scale;
                        sd[4 * g + 1] = s4.y * w_scale;
                        sd[4 * g + 2] = s4.z * w_scale;
                        sd[4 * g + 3] = s4.w * w_scale;
                    }
                    const uint32_t slot = 16u * x_chunk_slot(m, 2u * b + half);
                    if constexpr (LIMBS == 1) {
                        const v4i ax = *reinterpret_cast<const v4i*>(&lds.x[0][m][slot]);
                        const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bw, zero, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            acc[t][r] = fmaf(static_cast<float>(c[r]), sd[r], acc[t][r]);
                    } else {
                        const v4i a0 = *reinterpret_cast<const v4i*>(&lds.x[0][m][slot]);
                        const v4i a1 = *reinterpret_cast<const v4i*>(&lds.x[LIMBS > 1 ? 1 : 0][m][slot]);
                        const v4i a2 = *reinterpret_cast<const v4i*>(&lds.x[LIMBS > 2 ? 2 : 0][m][slot]);
                        const v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bw, zero, 0, 0, 0);
                        const v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bw, zero, 0, 0, 0);
                        const v16i c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a2, bw, zero, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            // |c0 + 256 c1| < 2^26 stays exact in int32; the top limb joins in f32
                            const float low = static_cast<float>(c0[r] + (c1[r] << 8));
                            const float all = fmaf(65536.0f, static_cast<float>(c2[r]), low);
                            acc[t][r] = fmaf(all, sd[r], acc[t][r]);
                        }
                    }
                }
            }
        }
        if constexpr (CODEC == kQ4_K) {
            // min term: acc_min[m, n] += sum_g (dmin * m_g)[n] * xsum[m, g], K = 2 per MFMA,
            // lane half h supplies sub-block 2j + h.
#pragma unroll
            for (int jj = 0; jj < 4 / KSPLIT; jj++) {
                const int j = jj + static_cast<int>(wave_k) * (4 / KSPLIT);  // sub-block pair of the stage
                float sc0, mn0, sc1, mn1;
                q4k_scale_min(w.header, 2 * j, sc0, mn0);
                q4k_scale_min(w.header, 2 * j + 1, sc1, mn1);
                const float b_operand = dmin_block * (half ? mn1 : mn0);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float a_operand = lds.xsum[2 * j + half][32 * t + (lane & 31u)];
                    acc_min[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_operand, b_operand, acc_min[t], 0, 0, 0);
                }
            }
        }
    }

    // ---- combine the K halves, add bias, store --------------------------------
    if constexpr (KSPLIT == 2) {
        __syncthreads();
        float* exchange = reinterpret_cast<float*>(&lds);  // [2 (wave_n)][MT*16][64 lanes]
        static_assert(sizeof(StageLds<MT, LIMBS>) >= 2u * MT * 16u * 64u * 4u, "exchange buffer");
        if (wave_k == 1) {
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float value = CODEC == kQ4_K ? acc[t][r] - acc_min[t][r] : acc[t][r];
                    exchange[((wave_n * MT + t) * 16 + r) * 64 + lane] = value;
                }
        }
        __syncthreads();
        if (wave_k == 1) return;
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][r] += exchange[((wave_n * MT + t) * 16 + r) * 64 + lane];
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
                    float value = CODEC == kQ4_K ? acc[t][r] - acc_min[t][r] : acc[t][r];
                    if (bias != nullptr) value += bias_value;
                    y[static_cast<uint64_t>(m) * rows + n_out] = value;
                }
            }
    }
}

template <int CODEC, int MT, int LIMBS, int KSPLIT>
hipError_t launch(const uint8_t* weight, const int8_t* q, uint64_t limb_stride, const float* scale,
                  const float* xsum, uint32_t table_stride, const float* bias, float* y, uint32_t rows,
                  uint32_t columns, uint32_t vectors, hipStream_t stream) {
    constexpr uint32_t BN = 128 / KSPLIT, BM = 32 * MT;
    const dim3 grid((rows + BN - 1) / BN, (vectors + BM - 1) / BM);
    hipLaunchKernelGGL((gemm_i8_kernel<CODEC, MT, LIMBS, KSPLIT>), grid, dim3(256), 0, stream, weight, q,
                       limb_stride, scale, xsum, table_stride, bias, y, rows, columns, vectors);
    return hipGetLastError();
}

template <int CODEC, int LIMBS>
hipError_t launch_shape(const uint8_t* weight, const int8_t* q, uint64_t limb_stride,
                        const float* scale, const float* xsum, uint32_t table_stride,
                        const float* bias, float* y, uint32_t rows, uint32_t columns,
                        uint32_t vectors, hipStream_t stream) {
    // Few vectors: one tile of vectors, 64-row workgroups so that N/64 of them fill the CUs.
    // Many vectors: 128 rows x 64 or 128 vectors per workgroup.
    constexpr int kMaxTiles = LIMBS == 1 ? 4 : 2;  // LDS: 32*MT vectors x 256 B x LIMBS
#define ET_GO(MT, KS) \
    return launch<CODEC, MT, LIMBS, KS>(weight, q, limb_stride, scale, xsum, table_stride, bias, y, rows, columns, vectors, stream)
    const bool few_row_tiles = (rows + 127u) / 128u * ((vectors + 32u * kMaxTiles - 1) / (32u * kMaxTiles)) < 192u;
    if (vectors <= 32) {
        if (few_row_tiles) ET_GO(1, 2);
        ET_GO(1, 1);
    }
    if (vectors <= 64 || kMaxTiles == 2) {
        if (few_row_tiles) ET_GO(2, 2);
        ET_GO(2, 1);
    }
    if constexpr (kMaxTiles == 4) {
        if (vectors <= 96) ET_GO(3, 1);
        ET_GO(4, 1);
    }
#undef ET_GO
    return hipErrorInvalidValue;
}

}  // namespace

bool gemm_i8_supported(int32_t codec, uint64_t columns) {
    if (codec == kQ8_0 || codec == kQ4_0) return columns % 32 == 0 && columns > 0;
    if (codec == kQ4_K) return columns % 256 == 0 && columns > 0;
    return false;
}

hipError_t gemm_i8(int32_t codec, int limbs, const uint8_t* weight, const int8_t* q,
                   uint64_t limb_stride, const float* scale, const float* xsum,
                   uint32_t table_stride, const float* bias, float* y, uint64_t rows,
                   uint64_t columns, uint64_t vectors, hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns),
                   m = static_cast<uint32_t>(vectors);
#define ET_CODEC(C)                                                                                  \
    case C:                                                                                          \
        return limbs == 1 ? launch_shape<C, 1>(weight, q, limb_stride, scale, xsum, table_stride, bias, \
                                               y, n, k, m, stream)                                   \
                          : launch_shape<C, 3>(weight, q, limb_stride, scale, xsum, table_stride, bias, \
                                               y, n, k, m, stream)
    switch (codec) {
        ET_CODEC(kQ8_0);
        ET_CODEC(kQ4_0);
        ET_CODEC(kQ4_K);
        default: return hipErrorInvalidValue;
    }
#undef ET_CODEC
}

}  // namespace et
