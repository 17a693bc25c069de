// Activation quantiser: stage 1 of the matrix-core paths.
//
// For each vector v and each 32-column block b:
//     amax  = max |x|                      scale[b, v] = amax / 127
//     inv   = amax > 0 ? 127 / amax : 0    q = clamp(rint(x * inv), -127, 127)
//     sum[b, v] = sum of q (int32)
// Both divisions are IEEE-correct and rint rounds to nearest even, so the
// integers and scales are bit-identical to a CPU evaluation of the same
// formulas. The reference has no int8 activation path; these semantics are
// this library's own. A second variant writes 24-bit fixed-point activations as
// three byte planes (range 127 * 2^16 instead of 127), which the same matrix-core
// kernel contracts limb by limb with f32-level accuracy.
//
// Two output layouts. The public one: q [vectors, columns] int8 row-major, scale and
// sum TRANSPOSED, [columns/32, stride] with stride = vectors rounded up to a multiple
// of 32 (entries at m >= vectors are never written). The one the matrix-core kernel
// streams: a blob per (256-column stage, 32-vector tile) that holds the stage's
// operands in exactly the order the kernel wants them in LDS, so that staging is a
// linear copy (see tile_blob_bytes in kernels.h). Vectors at m >= vectors inside a
// tile are never written and never influence a stored output.
//
// Eight lanes share a block: each loads one float4, the absmax and the sum are
// folded across the eight with DPP, each lane packs its four int8 into a dword.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "decode_math.h"
#include "kernels.h"
#include "quantize_halves.h"

namespace et {
namespace {

// LIMBS = 1: q = clamp(rint(x * 127/amax)), scale = amax / 127.
// LIMBS = 3: X = clamp(rint(x * 8323072/amax)) as three balanced signed bytes
//            (X = 65536*x2 + 256*x1 + x0), scale = amax / 8323072.
// TILED = false: q [vectors, columns], scale and sum transposed tables (the public layout).
// TILED = true:  one blob per (256-column stage, 32-vector tile), see tile_blob_bytes();
//                columns are padded with zeros to whole stages.
template <int LIMBS, bool TILED>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x,
                                                       uint64_t x_row_stride, uint32_t vectors,
                                                       uint32_t columns, int8_t* __restrict__ q,
                                                       float* __restrict__ scale,
                                                       int32_t* __restrict__ sum) {
    constexpr float kRange = LIMBS == 1 ? 127.f : 8323072.f;  // 127 * 2^16
    const uint32_t padded_columns = TILED ? (columns + 255u) & ~255u : columns;
    const uint32_t quads_per_row = padded_columns >> 2;
    const uint32_t vector_tiles = (vectors + 31u) >> 5;
    const uint64_t total = static_cast<uint64_t>(vectors) * quads_per_row;  // multiple of 8
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (uint64_t item = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
         item += stride) {
        const uint32_t v = static_cast<uint32_t>(item / quads_per_row);
        const uint32_t quad = static_cast<uint32_t>(item - static_cast<uint64_t>(v) * quads_per_row);
        float4 in = make_float4(0.f, 0.f, 0.f, 0.f);
        if (4u * quad < columns) in = *reinterpret_cast<const float4*>(x + v * x_row_stride + 4u * quad);
        float amax = fmaxf(fmaxf(fabsf(in.x), fabsf(in.y)), fmaxf(fabsf(in.z), fabsf(in.w)));
        amax = fmaxf(amax, dpp_f32<0xB1>(amax));   // quad_perm [1,0,3,2]
        amax = fmaxf(amax, dpp_f32<0x4E>(amax));   // quad_perm [2,3,0,1]
        amax = fmaxf(amax, dpp_f32<0x141>(amax));  // row_half_mirror: the other quad of the 8
        const float inv = amax > 0.f ? kRange / amax : 0.f;
        int qi[4];
        const float values[4] = {in.x, in.y, in.z, in.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float r = rintf(values[i] * inv);
            r = fminf(fmaxf(r, -kRange), kRange);
            qi[i] = static_cast<int>(r);
        }
        int total_q = (qi[0] + qi[1]) + (qi[2] + qi[3]);
        total_q += dpp_i32<0xB1>(total_q);
        total_q += dpp_i32<0x4E>(total_q);
        total_q += dpp_i32<0x141>(total_q);
        // limb planes: X + 0x808080 = (x2+128)<<16 | (x1+128)<<8 | (x0+128), every x in [-128, 127]
        uint32_t packed[LIMBS];
        if constexpr (LIMBS == 1) {
            packed[0] = (static_cast<uint32_t>(qi[0]) & 0xffu) | ((static_cast<uint32_t>(qi[1]) & 0xffu) << 8) |
                        ((static_cast<uint32_t>(qi[2]) & 0xffu) << 16) |
                        ((static_cast<uint32_t>(qi[3]) & 0xffu) << 24);
        } else {
            uint32_t u[4];
#pragma unroll
            for (int i = 0; i < 4; i++) u[i] = static_cast<uint32_t>(qi[i] + 0x808080);
#pragma unroll
            for (int limb = 0; limb < LIMBS; limb++)
                packed[limb] = (((u[0] >> (8 * limb)) & 0xffu) | (((u[1] >> (8 * limb)) & 0xffu) << 8) |
                                (((u[2] >> (8 * limb)) & 0xffu) << 16) |
                                (((u[3] >> (8 * limb)) & 0xffu) << 24)) ^ 0x80808080u;
        }
        const float unit = amax / kRange;
        if constexpr (TILED) {
            constexpr uint32_t kBlob = tile_blob_bytes(LIMBS);
            const uint32_t stage = quad >> 6, chunk = (quad & 63u) >> 2, dword = quad & 3u;
            uint8_t* blob = reinterpret_cast<uint8_t*>(q) +
                            (static_cast<uint64_t>(stage) * vector_tiles + (v >> 5)) * kBlob;
#pragma unroll
            for (int limb = 0; limb < LIMBS; limb++)
                *reinterpret_cast<uint32_t*>(blob + limb * 8192u + chunk * 512u + (v & 31u) * 16u + dword * 4u) =
                    packed[limb];
            if ((quad & 7u) == 0) {
                float* tables = reinterpret_cast<float*>(blob + LIMBS * 8192u);
                const uint32_t block = (quad & 63u) >> 3;
                tables[block * 32u + (v & 31u)] = unit;
                tables[256u + block * 32u + (v & 31u)] = unit * static_cast<float>(total_q);
                // The scale once more as three bfloat16 pieces whose sum it is exactly (8 bits each),
                // for the kernels that make their scale products on the bfloat16 matrix instruction.
                const uint32_t s0 = __float_as_uint(unit) & 0xffff0000u;
                const float rest = unit - __uint_as_float(s0);
                const uint32_t s1 = __float_as_uint(rest) & 0xffff0000u;
                const uint32_t s2 = __float_as_uint(rest - __uint_as_float(s1));
                reinterpret_cast<uint2*>(tables + 512u)[block * 32u + (v & 31u)] = make_uint2((s0 >> 16) | s1, s2 >> 16);
            }
        } else {
            static_assert(TILED || LIMBS == 1, "the row-major layout is the int8 one");
            reinterpret_cast<uint32_t*>(q)[static_cast<uint64_t>(v) * quads_per_row + quad] = packed[0];
            if ((quad & 7u) == 0) {
                const uint64_t slot = static_cast<uint64_t>(quad >> 3) * ((vectors + 31u) & ~31u) + v;
                scale[slot] = unit;
                if (sum != nullptr) sum[slot] = total_q;
            }
        }
    }
}


// quantize_kernel<LIMBS, true> for large inputs: a workgroup makes ONE blob - a 256-column stage of a
// 32-vector tile - in LDS and writes it out linearly. The kernel above stores every dword where it
// belongs in memory, sixteen bytes at a time in lines 512 bytes apart (measured on 512 x 14336: 29.4 MB
// written for 11.0 MB of blobs); here a wave reads one vector's stage as 1 KiB of consecutive floats and
// the blob leaves as consecutive 16-byte stores. Same arithmetic, same bytes.
// LDS rows of the operand planes have a pitch of 528 bytes (512 + 16): a wave writes one vector's
// dwords into all sixteen chunks at once, and with 512 they would share four banks.
template <int LIMBS>
__global__ __launch_bounds__(256) void quantize_blob_kernel(const float* __restrict__ x, uint64_t x_row_stride,
                                                            uint32_t vectors, uint32_t columns,
                                                            uint8_t* __restrict__ tiles) {
    constexpr float kRange = LIMBS == 1 ? 127.f : 8323072.f;
    constexpr uint32_t kBlob = tile_blob_bytes(LIMBS);
    constexpr uint32_t kPitch = 528u, kPlane = 16u * kPitch, kTablesAt = LIMBS * kPlane;
    constexpr uint32_t kTableBytes = kBlob - LIMBS * 8192u;
    __shared__ __attribute__((aligned(16))) uint8_t blob[kTablesAt + kTableBytes];
    const uint32_t vector_tiles = (vectors + 31u) >> 5;
    const uint32_t stage = blockIdx.x / vector_tiles, tile = blockIdx.x - stage * vector_tiles;
    const uint32_t quad_in_stage = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t quad = stage * 64u + quad_in_stage;  // of the row
    // the tables' padding (behind the pieces) leaves as zeros
    for (uint32_t at = 2048u + 2048u + threadIdx.x * 4u; at < kTableBytes; at += 1024u)
        *reinterpret_cast<uint32_t*>(blob + kTablesAt + at) = 0u;
    float4 in[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {  // a wave takes vectors wave, wave + 4, ...: all loads go out first
        const uint32_t m = 4u * k + wave, v = tile * 32u + m;
        in[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < vectors && 4u * quad < columns) in[k] = *reinterpret_cast<const float4*>(x + v * x_row_stride + 4u * quad);
    }
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const uint32_t m = 4u * k + wave;
        float amax = fmaxf(fmaxf(fabsf(in[k].x), fabsf(in[k].y)), fmaxf(fabsf(in[k].z), fabsf(in[k].w)));
        amax = fmaxf(amax, dpp_f32<0xB1>(amax));
        amax = fmaxf(amax, dpp_f32<0x4E>(amax));
        amax = fmaxf(amax, dpp_f32<0x141>(amax));
        const float inv = amax > 0.f ? kRange / amax : 0.f;
        int qi[4];
        const float values[4] = {in[k].x, in[k].y, in[k].z, in[k].w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float r = rintf(values[i] * inv);
            r = fminf(fmaxf(r, -kRange), kRange);
            qi[i] = static_cast<int>(r);
        }
        int total_q = (qi[0] + qi[1]) + (qi[2] + qi[3]);
        total_q += dpp_i32<0xB1>(total_q);
        total_q += dpp_i32<0x4E>(total_q);
        total_q += dpp_i32<0x141>(total_q);
        const uint32_t chunk = quad_in_stage >> 2, dword = quad_in_stage & 3u;
        uint8_t* slot = blob + chunk * kPitch + m * 16u + dword * 4u;
        if constexpr (LIMBS == 1) {
            *reinterpret_cast<uint32_t*>(slot) = (static_cast<uint32_t>(qi[0]) & 0xffu) | ((static_cast<uint32_t>(qi[1]) & 0xffu) << 8) |
                                                 ((static_cast<uint32_t>(qi[2]) & 0xffu) << 16) |
                                                 ((static_cast<uint32_t>(qi[3]) & 0xffu) << 24);
        } else {
            uint32_t u[4];
#pragma unroll
            for (int i = 0; i < 4; i++) u[i] = static_cast<uint32_t>(qi[i] + 0x808080);
#pragma unroll
            for (int limb = 0; limb < LIMBS; limb++)
                *reinterpret_cast<uint32_t*>(slot + limb * kPlane) =
                    (((u[0] >> (8 * limb)) & 0xffu) | (((u[1] >> (8 * limb)) & 0xffu) << 8) |
                     (((u[2] >> (8 * limb)) & 0xffu) << 16) | (((u[3] >> (8 * limb)) & 0xffu) << 24)) ^ 0x80808080u;
        }
        if ((quad_in_stage & 7u) == 0) {
            const float unit = amax / kRange;
            float* tables = reinterpret_cast<float*>(blob + kTablesAt);
            const uint32_t block = quad_in_stage >> 3;
            tables[block * 32u + m] = unit;
            tables[256u + block * 32u + m] = unit * static_cast<float>(total_q);
            const uint32_t s0 = __float_as_uint(unit) & 0xffff0000u;
            const float rest = unit - __uint_as_float(s0);
            const uint32_t s1 = __float_as_uint(rest) & 0xffff0000u;
            const uint32_t s2 = __float_as_uint(rest - __uint_as_float(s1));
            reinterpret_cast<uint2*>(tables + 512u)[block * 32u + m] = make_uint2((s0 >> 16) | s1, s2 >> 16);
        }
    }
    __syncthreads();
    uint8_t* out = tiles + static_cast<uint64_t>(blockIdx.x) * kBlob;
    for (uint32_t at = threadIdx.x * 16u; at < kBlob; at += 4096u) {
        // the planes without their pitch padding, then the tables as they are
        const uint32_t from = at < LIMBS * 8192u ? (at / 8192u) * kPlane + ((at % 8192u) / 512u) * kPitch + at % 512u
                                                 : kTablesAt + (at - LIMBS * 8192u);
        *reinterpret_cast<uint4*>(out + at) = *reinterpret_cast<const uint4*>(blob + from);
    }
}

// SILU_MUL: the activations are silu(x) * second, element by element (the input of a gated
// feed-forward's down projection), computed on the fly with silu_mul_kernel's arithmetic.
template <bool SILU_MUL>
__global__ __launch_bounds__(64) void quantize_halves_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ second, uint64_t x_row_stride,
                                                             uint32_t vectors, uint32_t stages,
                                                             uint8_t* __restrict__ tiles) {
    const uint32_t vector_tiles = (vectors + 31u) >> 5;
    const uint32_t quad = threadIdx.x;
    for (uint64_t item = blockIdx.x; item < static_cast<uint64_t>(vectors) * stages; item += gridDim.x) {
        const uint32_t v = static_cast<uint32_t>(item / stages), stage = static_cast<uint32_t>(item % stages);
        const uint64_t at = v * x_row_stride + 256u * stage + 4u * quad;
        float4 in = *reinterpret_cast<const float4*>(x + at);
        if constexpr (SILU_MUL) {
            const float4 up = *reinterpret_cast<const float4*>(second + at);
            in = make_float4(silu_mul_one(in.x, up.x), silu_mul_one(in.y, up.y), silu_mul_one(in.z, up.z),
                             silu_mul_one(in.w, up.w));
        }
        quantize_halves_store(in, v, stage, quad, vector_tiles, tiles);
    }
}

// The activations are rms_norm(x) * weight, with rms_norm_kernel's arithmetic and summation order
// (rms_row_scale in decode_math.h: thread t of 256 adds the squares of float4 number t, t + 256, ...
// in that order, the waves' sums meet as ((0 + 1) + (2 + 3))). One workgroup of sixteen waves per
// vector, so that a row of 4096 columns is quantised in one pass, a stage per wave: thread T holds
// float4 number T; the squares go through LDS to the first 256 threads, which add them in
// rms_row_scale's order.
constexpr uint32_t kRmsThreads = 1024;
// The unsummed K shares of a contraction, for the variant that sums them itself: the row it norms is
// y[m, :] = share 0 + share 1 + ... (+ bias) (+ residual[m, :]) in reduce_group_kernel's order, and it
// writes that row to y before it reads it (residual may be y: a float4 is read, then written, by one
// thread).
struct ShareSource {
    const float* shares;     // [count][vectors][launch_rows]
    uint32_t count;
    uint64_t launch_rows, share_stride;
    const float* bias;       // [columns] or null
    const float* residual;   // [vectors, columns] or null
    float* y;                // [vectors, columns]: the summed rows, written before they are normed
};
template <bool SHARES>
__global__ __launch_bounds__(kRmsThreads) void quantize_halves_rms_kernel(const float* x, uint64_t x_row_stride,
                                                                         const ShareSource source,
                                                                         const NormWeight weight, double eps,
                                                                         uint32_t vectors, uint32_t columns,
                                                                         uint8_t* __restrict__ tiles) {
    __shared__ double squares[kRmsThreads];
    __shared__ double partial[4];
    const uint32_t v = blockIdx.x;
    const float4* in = reinterpret_cast<const float4*>(x + v * x_row_stride);
    const uint32_t quads = columns / 4;
    const auto square_sum = [](const float4& f) {
        return (static_cast<double>(f.x) * f.x + static_cast<double>(f.y) * f.y) +
               (static_cast<double>(f.z) * f.z + static_cast<double>(f.w) * f.w);
    };
    float4 held = make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (SHARES) {
        // x is y: every float4 of the row is summed and written once, number T, T + 1024, ... by thread T
        float4* row = reinterpret_cast<float4*>(source.y + v * x_row_stride);
        for (uint32_t i = threadIdx.x; i < quads; i += kRmsThreads) {
            const float* first = source.shares + v * source.launch_rows + 4u * i;
            float4 total = *reinterpret_cast<const float4*>(first);
            for (uint32_t k = 1; k < source.count; k++) {
                const float4 part = *reinterpret_cast<const float4*>(first + k * source.share_stride);
                total.x += part.x;
                total.y += part.y;
                total.z += part.z;
                total.w += part.w;
            }
            if (source.bias != nullptr) {
                const float4 b = reinterpret_cast<const float4*>(source.bias)[i];
                total = make_float4(total.x + b.x, total.y + b.y, total.z + b.z, total.w + b.w);
            }
            if (source.residual != nullptr) {
                const float4 r = reinterpret_cast<const float4*>(source.residual + v * static_cast<uint64_t>(columns))[i];
                total = make_float4(total.x + r.x, total.y + r.y, total.z + r.z, total.w + r.w);
            }
            row[i] = total;
            if (i == threadIdx.x) held = total;
        }
        if (quads > kRmsThreads) __syncthreads();  // the passes below read what other threads wrote
    } else {
        if (threadIdx.x < quads) held = in[threadIdx.x];
    }
    squares[threadIdx.x] = square_sum(held);
    __syncthreads();
    if (threadIdx.x < 256) {
        double sum = 0.0;
#pragma unroll
        for (int j = 0; j < kRmsHeld; j++) sum += squares[threadIdx.x + 256 * j];
        for (uint32_t i = threadIdx.x + 256 * kRmsHeld; i < quads; i += 256) sum += square_sum(in[i]);
        sum = wave_sum(sum);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
    }
    __syncthreads();
    const double mean_square = ((partial[0] + partial[1]) + (partial[2] + partial[3])) / static_cast<double>(columns);
    const double scale = 1.0 / sqrt(mean_square + eps);
    const uint32_t vector_tiles = (vectors + 31u) >> 5, stages = columns >> 8;
    const uint32_t wave = threadIdx.x >> 6, quad = threadIdx.x & 63u;
    if (wave < stages)
        quantize_halves_store(rms_four(held, scale, norm_weight_four(weight, threadIdx.x)), v, wave, quad, vector_tiles, tiles);
    for (uint32_t stage = wave + kRmsThreads / 64u; stage < stages; stage += kRmsThreads / 64u) {
        const uint32_t i = 64u * stage + quad;
        quantize_halves_store(rms_four(in[i], scale, norm_weight_four(weight, i)), v, stage, quad, vector_tiles, tiles);
    }
}

// Small batches are latency-bound: one wave per workgroup spreads them over all CUs.
struct Geometry {
    uint32_t blocks, threads;
};
Geometry geometry_for(uint64_t items) {
    const uint32_t threads = items <= 256u * 1024u ? 64u : 256u;
    const uint64_t blocks = (items + threads - 1) / threads;
    return {static_cast<uint32_t>(blocks > 16384 ? 16384 : blocks), threads};
}

}  // namespace

hipError_t quantize_activations(const float* x, uint64_t x_row_stride, uint64_t vectors,
                                uint64_t columns, int8_t* q, float* scale, int32_t* sum,
                                hipStream_t stream) {
    const uint64_t total = vectors * (columns >> 2);
    if (total == 0) return hipSuccess;
    const Geometry g = geometry_for(total);
    hipLaunchKernelGGL((quantize_kernel<1, false>), dim3(g.blocks), dim3(g.threads), 0, stream, x,
                       x_row_stride, static_cast<uint32_t>(vectors), static_cast<uint32_t>(columns), q,
                       scale, sum);
    return hipGetLastError();
}

hipError_t quantize_tiles(const float* x, uint64_t x_row_stride, uint64_t vectors, uint64_t columns,
                          int limbs, uint8_t* tiles, hipStream_t stream) {
    const uint64_t total = vectors * (((columns + 255) & ~255ull) >> 2);
    if (total == 0) return hipSuccess;
    if (limbs == 2) {
        if (columns % 256 != 0) return hipErrorInvalidValue;
        const uint64_t items = vectors * (columns / 256);
        hipLaunchKernelGGL(quantize_halves_kernel<false>, dim3(static_cast<uint32_t>(items < 65536 ? items : 65536)),
                           dim3(64), 0, stream, x, nullptr, x_row_stride, static_cast<uint32_t>(vectors),
                           static_cast<uint32_t>(columns / 256), tiles);
        return hipGetLastError();
    }
    if (limbs != 1 && limbs != 3) return hipErrorInvalidValue;
    // Enough blobs to occupy the device: a workgroup per blob, assembled in LDS and written once.
    const uint64_t blobs = ((columns + 255) / 256) * ((vectors + 31) / 32);
    if (blobs >= 512 && blobs <= 0x7fffffffull) {
        const dim3 blob_grid(static_cast<uint32_t>(blobs)), blob_block(256);
        if (limbs == 1)
            hipLaunchKernelGGL(quantize_blob_kernel<1>, blob_grid, blob_block, 0, stream, x, x_row_stride,
                               static_cast<uint32_t>(vectors), static_cast<uint32_t>(columns), tiles);
        else
            hipLaunchKernelGGL(quantize_blob_kernel<3>, blob_grid, blob_block, 0, stream, x, x_row_stride,
                               static_cast<uint32_t>(vectors), static_cast<uint32_t>(columns), tiles);
        return hipGetLastError();
    }
    const Geometry g = geometry_for(total);
    const dim3 grid(g.blocks), block(g.threads);
    if (limbs == 1)
        hipLaunchKernelGGL((quantize_kernel<1, true>), grid, block, 0, stream, x, x_row_stride,
                           static_cast<uint32_t>(vectors), static_cast<uint32_t>(columns),
                           reinterpret_cast<int8_t*>(tiles), nullptr, nullptr);
    else
        hipLaunchKernelGGL((quantize_kernel<3, true>), grid, block, 0, stream, x, x_row_stride,
                           static_cast<uint32_t>(vectors), static_cast<uint32_t>(columns),
                           reinterpret_cast<int8_t*>(tiles), nullptr, nullptr);
    return hipGetLastError();
}

hipError_t quantize_tiles_silu_mul(const float* gate, const float* up, uint64_t row_stride, uint64_t vectors,
                                   uint64_t columns, uint8_t* tiles, hipStream_t stream) {
    if (columns % 256 != 0) return hipErrorInvalidValue;
    const uint64_t items = vectors * (columns / 256);
    if (items == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_halves_kernel<true>, dim3(static_cast<uint32_t>(items < 65536 ? items : 65536)),
                       dim3(64), 0, stream, gate, up, row_stride, static_cast<uint32_t>(vectors),
                       static_cast<uint32_t>(columns / 256), tiles);
    return hipGetLastError();
}

hipError_t quantize_tiles_rms_norm(const float* x, uint64_t x_row_stride, const void* weight, int weight_is_half,
                                   double eps, uint64_t vectors, uint64_t columns, uint8_t* tiles, hipStream_t stream) {
    if (columns % 256 != 0 || vectors > 0x7fffffffull) return hipErrorInvalidValue;
    if (vectors == 0 || columns == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_halves_rms_kernel<false>, dim3(static_cast<uint32_t>(vectors)), dim3(kRmsThreads), 0, stream,
                       x, x_row_stride, ShareSource{}, NormWeight{weight, weight_is_half ? 1 : 0}, eps, static_cast<uint32_t>(vectors),
                       static_cast<uint32_t>(columns), tiles);
    return hipGetLastError();
}

hipError_t quantize_tiles_rms_norm_of_shares(const float* shares, uint32_t share_count, uint64_t launch_rows,
                                             const float* bias, const float* residual, float* y, const void* weight,
                                             int weight_is_half, double eps, uint64_t vectors, uint64_t columns,
                                             uint8_t* tiles, hipStream_t stream) {
    if (columns % 256 != 0 || vectors > 0x7fffffffull || share_count == 0 || launch_rows < columns || launch_rows % 4 != 0)
        return hipErrorInvalidValue;
    if (vectors == 0 || columns == 0) return hipSuccess;
    const ShareSource source = {shares, share_count, launch_rows, launch_rows * vectors, bias, residual, y};
    hipLaunchKernelGGL(quantize_halves_rms_kernel<true>, dim3(static_cast<uint32_t>(vectors)), dim3(kRmsThreads), 0, stream,
                       y, columns, source, NormWeight{weight, weight_is_half ? 1 : 0}, eps, static_cast<uint32_t>(vectors),
                       static_cast<uint32_t>(columns), tiles);
    return hipGetLastError();
}

}  // namespace et
