// Measurement aids: a plain streaming read, a plain copy of known size, and loops of matrix-core
// instructions that touch no memory.
//
// They give (a) the HBM bandwidth this device actually delivers to a kernel of
// the same footprint as a GEMV (the practical ceiling the dequant-GEMV is
// compared with, next to the published peak), (b) a reference reading for
// hardware counters (FETCH_SIZE / WRITE_SIZE per byte actually moved) and (c) the rate the
// matrix cores sustain on this device for the instructions the batch kernels use, alone and with
// the f32 block-scale epilogue of an int8 contraction whose operands both carry a scale per 32
// columns - the ceiling that arithmetic has whatever feeds it.
// Nothing on the operator path uses them; the reference has no counterpart.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"

namespace et {
namespace {

// Each workgroup streams a contiguous range with 16-byte loads, four in flight
// per lane. The XOR of everything read leaves through one word per wave, so the
// loads cannot be removed; there is no barrier and no atomic on the way out.
__global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ src, uint32_t quads,
                                                   uint32_t* __restrict__ sink) {
    const uint32_t per_wg = (quads + gridDim.x - 1) / gridDim.x;
    const uint32_t begin = blockIdx.x * per_wg;
    const uint32_t end = min(begin + per_wg, quads);
    uint32_t acc = 0;
    uint32_t i = begin + threadIdx.x;
    for (; i + 3 * 256u < end; i += 4 * 256u) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = src[i + u * 256u];
#pragma unroll
        for (int u = 0; u < 4; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < end; i += 256u) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) acc ^= __shfl_xor(acc, offset);
    if ((threadIdx.x & 63u) == 0) sink[blockIdx.x * 4u + (threadIdx.x >> 6)] = acc;
}

// The same read with U loads in flight per lane (and non-temporal loads when STREAMING): if the
// device can deliver more than read_kernel reaches, a deeper queue per wave shows it.
template <int U, bool STREAMING>
__global__ __launch_bounds__(256) void read_deep_kernel(const uint4* __restrict__ src, uint32_t quads,
                                                        uint32_t* __restrict__ sink) {
    const uint32_t per_wg = (quads + gridDim.x - 1) / gridDim.x;
    const uint32_t begin = blockIdx.x * per_wg;
    const uint32_t end = min(begin + per_wg, quads);
    uint32_t acc = 0;
    uint32_t i = begin + threadIdx.x;
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const auto fetch = [&](uint32_t at) {
        if constexpr (STREAMING) {
            const v4u raw = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(src + at));
            return make_uint4(raw.x, raw.y, raw.z, raw.w);
        } else {
            return src[at];
        }
    };
    for (; i + (U - 1) * 256u < end; i += U * 256u) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = fetch(i + u * 256u);
#pragma unroll
        for (int u = 0; u < U; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < end; i += 256u) {
        const uint4 v = fetch(i);
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) acc ^= __shfl_xor(acc, offset);
    if ((threadIdx.x & 63u) == 0) sink[blockIdx.x * 4u + (threadIdx.x >> 6)] = acc;
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8); }

// A read that uses no registers and no arithmetic: every wave only issues 1 KiB global-to-LDS
// copies into its own ring of DEPTH slots and, once the ring is full, waits for the oldest copy
// before it issues the next one - DEPTH KiB in flight per wave for the whole launch. One workgroup
// per compute unit (WAVES * DEPTH <= 128 KiB of LDS); workgroup w takes the w-th contiguous range.
// NT: non-temporal copies (the caches keep nothing of the bytes). RANGES: wave v of a workgroup copies
// the v-th contiguous part of the workgroup's range instead of every WAVES-th KiB of it.
template <int WAVES, int DEPTH, bool NT = false, bool RANGES = false>
__global__ __launch_bounds__(64 * WAVES) void read_lds_kernel(const uint8_t* __restrict__ src, uint32_t kib,
                                                              uint32_t* __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ring[];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t per_wg = (kib + gridDim.x - 1) / gridDim.x;
    const uint32_t begin = blockIdx.x * per_wg;
    const uint32_t end = min(begin + per_wg, kib);
    uint8_t* mine = ring + wave * DEPTH * 1024u;
    const uint32_t per_wave = (per_wg + WAVES - 1) / WAVES;
    // jobs of this wave: begin + wave, begin + wave + WAVES, ... or a contiguous part of the range
    uint32_t job = RANGES ? begin + wave * per_wave : begin + wave, slot = 0;
    const uint32_t last = RANGES ? min(job + per_wave, end) : end;
    for (; job < last; job += RANGES ? 1u : static_cast<uint32_t>(WAVES)) {
        if (slot >= static_cast<uint32_t>(DEPTH)) __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH - 1));  // the slot's last copy has landed
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src + static_cast<uint64_t>(job) * 1024u + lane * 16u),
                                         reinterpret_cast<uint4*>(mine + (slot % DEPTH) * 1024u), 16, 0, NT ? 2 : 0);
        slot += 1;
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __syncthreads();
    // one word of what arrived leaves, so that the copies have an observer
    if (threadIdx.x < 4) sink[(blockIdx.x * 4u + threadIdx.x) % 1024u] = reinterpret_cast<const uint32_t*>(ring)[threadIdx.x * 256u];
}

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src,
                                                   uint4* __restrict__ dst, uint64_t quads) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256ull;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < quads; i += stride) dst[i] = src[i];
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// Every wave runs `iterations` rounds of four independent instructions of one kind and leaves the
// sum of what it accumulated in sink[thread]. Operands are all ones, so the sums are known:
//   kMfmaI8        v_mfma_i32_32x32x32_i8, accumulating: every element ends at 32 * iterations
//   kMfmaI8Scaled  the same instruction from zero, then per element one convert and one multiply-add
//                  with a tile of scale products that v_mfma_f32_32x32x2f32 makes from a scale per
//                  vector and a scale per row (the epilogue of gemm_i8.hip); element = 32 * 0.5 * iterations
//   kMfmaF16       v_mfma_f32_32x32x16_f16, accumulating: 16 * iterations
//   kMfmaF16Small  v_mfma_f32_16x16x32_f16, accumulating: 32 * iterations
//   kMfmaI8ScaledBf16  kMfmaI8Scaled with the scale products from a bfloat16 instruction (see below)
//   kMfmaI8Biased (and ...MatrixOnly, ...ValuOnly)  the step of the int8 batch kernel as it runs now (see below);
//                  element = 32 * 0.5 * iterations (0.5 * iterations per element for ...MatrixOnly's last step only)
template <int KIND>
__global__ __launch_bounds__(256) void mfma_kernel(float* __restrict__ sink, uint32_t iterations) {
    float total = 0.f;
    if constexpr (KIND == kMfmaI8) {
        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
        v16i c[4] = {};
        for (uint32_t it = 0; it < iterations; it++)
#pragma unroll
            for (int k = 0; k < 4; k++) c[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ones, ones, c[k], 0, 0, 0);
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += static_cast<float>(c[k][r]);
    } else if constexpr (KIND == kMfmaI8Scaled) {
        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
        v16i zero_i = {};
        v16f zero_f = {};
        float acc[4][16] = {};
        // only the k = 0 half of the lanes carries a value of the rank-1 product
        const float row_scale = threadIdx.x % 64 < 32 ? 0.5f : 0.f;
        float vector_scale[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        v4i a[4] = {ones, ones, ones, ones};
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // Operands that the compiler cannot prove equal or constant keep four instructions of
                // each kind inside the loop: an empty asm statement per operand, values unchanged.
                asm volatile("" : "+v"(vector_scale[k]));
                asm volatile("" : "+v"(a[k]));
                const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[k], ones, zero_i, 0, 0, 0);
                const v16f sd = __builtin_amdgcn_mfma_f32_32x32x2f32(vector_scale[k], row_scale, zero_f, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[k][r] = fmaf(static_cast<float>(c[r]), sd[r], acc[k][r]);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += acc[k][r];
    } else if constexpr (KIND == kMfmaI8ScaledBf16) {
        // The same arithmetic with the tile of scale products from v_mfma_f32_32x32x16_bf16 (half the
        // matrix-core time of the f32 instruction): the vector's scale as three bfloat16 pieces (exact:
        // 3 x 8 bits), the row's half-float scale as two (8 + 3 bits), their six products in six of
        // the sixteen K slots, every product exact in the f32 accumulator.
        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
        v16i zero_i = {};
        v16f zero_f = {};
        float acc[4][16] = {};
        const bool first_half = threadIdx.x % 64 < 32;
        float vector_scale[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        const float row_value = 0.5f;
        const uint32_t d0 = __float_as_uint(row_value) & 0xffff0000u;
        const uint32_t d1 = __float_as_uint(row_value - __uint_as_float(d0)) >> 16;
        union {
            uint4 words;
            v8bf values;
        } row_operand, vector_operand;
        // K slots 0..5 of the first lane half: (d0, d1, d0, d1, d0, d1) against (s0, s0, s1, s1, s2, s2)
        const uint32_t d_pair = first_half ? (d0 >> 16) | (d1 << 16) : 0u;
        row_operand.words = make_uint4(d_pair, d_pair, d_pair, 0u);
        v4i a[4] = {ones, ones, ones, ones};
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                asm volatile("" : "+v"(vector_scale[k]));
                asm volatile("" : "+v"(a[k]));
                const float s = first_half ? vector_scale[k] : 0.f;
                const uint32_t s0 = __float_as_uint(s) & 0xffff0000u;
                const float rest = s - __uint_as_float(s0);
                const uint32_t s1 = __float_as_uint(rest) & 0xffff0000u;
                const uint32_t s2 = __float_as_uint(rest - __uint_as_float(s1)) >> 16;
                vector_operand.words = make_uint4((s0 >> 16) | s0, (s1 >> 16) | s1, s2 | (s2 << 16), 0u);
                const v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[k], ones, zero_i, 0, 0, 0);
                const v16f sd = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vector_operand.values, row_operand.values, zero_f, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[k][r] = fmaf(static_cast<float>(c[r]), sd[r], acc[k][r]);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += acc[k][r];
    } else if constexpr (KIND == kMfmaI8Biased || KIND == kMfmaI8BiasedMatrixOnly || KIND == kMfmaI8BiasedValuOnly) {
        // The step of gemm_i8.hip's one-limb loop as it is now: the integer sums start at the bits of
        // 1.5 * 2^23 (their bits are then the float 12582912 + sum: one subtraction instead of a convert),
        // the scale products come from v_mfma_f32_32x32x16_bf16 with ready-made operand pieces, and each
        // matrix instruction is followed by sixteen VALU instructions that do not depend on it:
        //   scale products | 16 subtractions;  integer MFMA of the next step | 16 multiply-adds.
        // kMfmaI8BiasedMatrixOnly leaves the VALU instructions out, kMfmaI8BiasedValuOnly the matrix ones
        // (same registers, fed by empty asm statements): together they show how much of the two the
        // device runs side by side.
        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
        v16i bias;
#pragma unroll
        for (int r = 0; r < 16; r++) bias[r] = 0x4B400000;
        v16f zero_f = {};
        float acc[4][16] = {};
        const bool first_half = threadIdx.x % 64 < 32;
        union {
            uint4 words;
            v8bf values;
        } row_operand, vector_operand;
        // 0.5 and 1.0 in bfloat16: K slot 0 of the first lane half carries the product, the rest zeros
        row_operand.words = make_uint4(first_half ? 0x3f00u : 0u, 0u, 0u, 0u);
        uint32_t vector_piece = 0x3f80u;
        v4i a = ones;
        v16i c_now = bias;
        v16f sd = zero_f;
        if constexpr (KIND != kMfmaI8BiasedValuOnly) c_now = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, ones, bias, 0, 0, 0);
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                asm volatile("" : "+v"(vector_piece));
                vector_operand.words = make_uint4(vector_piece, 0u, 0u, 0u);
                asm volatile("" : "+v"(a));
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (KIND != kMfmaI8BiasedValuOnly)
                    sd = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vector_operand.values, row_operand.values, zero_f, 0, 0, 0);
                else
                    asm volatile("" : "+v"(sd));
                if constexpr (KIND == kMfmaI8BiasedMatrixOnly) asm volatile("" : : "v"(sd));  // a use: the instruction stays
                __builtin_amdgcn_sched_barrier(0);
                float sums[16];
                if constexpr (KIND != kMfmaI8BiasedMatrixOnly) {
#pragma unroll
                    for (int r = 0; r < 16; r++) sums[r] = __int_as_float(c_now[r]) - 12582912.0f;
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (KIND != kMfmaI8BiasedValuOnly)
                    c_now = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, ones, bias, 0, 0, 0);
                else
                    asm volatile("" : "+v"(c_now));
                if constexpr (KIND == kMfmaI8BiasedMatrixOnly) asm volatile("" : : "v"(c_now));
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (KIND != kMfmaI8BiasedMatrixOnly) {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[k][r] = fmaf(sums[r], sd[r], acc[k][r]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += acc[k][r];
        if constexpr (KIND == kMfmaI8BiasedMatrixOnly) {  // keep the last results alive
#pragma unroll
            for (int r = 0; r < 16; r++) total += (__int_as_float(c_now[r]) - 12582912.0f) * sd[r];
        }
    } else if constexpr (KIND == kMfmaF16) {
        v8h ones;
#pragma unroll
        for (int i = 0; i < 8; i++) ones[i] = static_cast<_Float16>(1.0f);
        v16f c[4] = {};
        for (uint32_t it = 0; it < iterations; it++)
#pragma unroll
            for (int k = 0; k < 4; k++) c[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, ones, c[k], 0, 0, 0);
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += c[k][r];
    } else {
        v8h ones;
#pragma unroll
        for (int i = 0; i < 8; i++) ones[i] = static_cast<_Float16>(1.0f);
        v4f c[4] = {};
        for (uint32_t it = 0; it < iterations; it++)
#pragma unroll
            for (int k = 0; k < 4; k++) c[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, ones, c[k], 0, 0, 0);
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int r = 0; r < 4; r++) total += c[k][r];
    }
    sink[blockIdx.x * 256u + threadIdx.x] = total;
}

}  // namespace

hipError_t calibration_mfma(int kind, uint32_t iterations, uint32_t workgroups, float* sink, hipStream_t stream) {
    const dim3 grid(workgroups), block(256);
    switch (kind) {
        case kMfmaI8: hipLaunchKernelGGL(mfma_kernel<kMfmaI8>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaI8Scaled: hipLaunchKernelGGL(mfma_kernel<kMfmaI8Scaled>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaF16: hipLaunchKernelGGL(mfma_kernel<kMfmaF16>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaF16Small: hipLaunchKernelGGL(mfma_kernel<kMfmaF16Small>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaI8ScaledBf16: hipLaunchKernelGGL(mfma_kernel<kMfmaI8ScaledBf16>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaI8Biased: hipLaunchKernelGGL(mfma_kernel<kMfmaI8Biased>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaI8BiasedMatrixOnly: hipLaunchKernelGGL(mfma_kernel<kMfmaI8BiasedMatrixOnly>, grid, block, 0, stream, sink, iterations); break;
        case kMfmaI8BiasedValuOnly: hipLaunchKernelGGL(mfma_kernel<kMfmaI8BiasedValuOnly>, grid, block, 0, stream, sink, iterations); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t calibration_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups,
                            hipStream_t stream) {
    if (bytes < 16) return hipSuccess;
    hipLaunchKernelGGL(read_kernel, dim3(workgroups), dim3(256), 0, stream,
                       static_cast<const uint4*>(src), static_cast<uint32_t>(bytes / 16), sink);
    return hipGetLastError();
}

hipError_t calibration_read_variant(int variant, const void* src, uint64_t bytes, uint32_t* sink,
                                    uint32_t workgroups, hipStream_t stream) {
    if (bytes < 1024) return hipSuccess;
    const uint4* quads = static_cast<const uint4*>(src);
    const uint32_t count = static_cast<uint32_t>(bytes / 16);
    constexpr uint32_t kRingBytes = 128u * 1024u;
    const auto launch_lds = [&](auto kernel, uint32_t waves) -> hipError_t {
        if (hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, kRingBytes))
            return status;
        hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(64 * waves), kRingBytes, stream,
                           static_cast<const uint8_t*>(src), static_cast<uint32_t>(bytes / 1024), sink);
        return hipGetLastError();
    };
    switch (variant) {
        case kReadPlain: return calibration_read(src, bytes, sink, workgroups, stream);
        case kReadDeep:
            hipLaunchKernelGGL((read_deep_kernel<16, false>), dim3(workgroups), dim3(256), 0, stream, quads, count, sink);
            break;
        case kReadStreaming:
            hipLaunchKernelGGL((read_deep_kernel<16, true>), dim3(workgroups), dim3(256), 0, stream, quads, count, sink);
            break;
        case kReadLds4: return launch_lds(read_lds_kernel<4, 32>, 4);
        case kReadLds8: return launch_lds(read_lds_kernel<8, 16>, 8);
        case kReadLds8Nt: return launch_lds(read_lds_kernel<8, 16, true>, 8);
        case kReadLds8NtShallow: return launch_lds(read_lds_kernel<8, 4, true>, 8);
        case kReadLds8NtRanges: return launch_lds(read_lds_kernel<8, 16, true, true>, 8);
        case kReadLds8NtRangesShallow: return launch_lds(read_lds_kernel<8, 4, true, true>, 8);
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t calibration_copy(const void* src, void* dst, uint64_t bytes, hipStream_t stream) {
    if (bytes < 16) return hipSuccess;
    const uint64_t quads = bytes / 16;
    uint64_t blocks = (quads + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), quads);
    return hipGetLastError();
}

}  // namespace et
