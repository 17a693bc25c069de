// Bit-exact dequantisation of packed GGUF rows on gfx950.
//
// out[p, :] = decode(W[index[p], :]) with every f32 operation rounded exactly
// as the reference's scalar decoders do (crates/runtime-cpu/src/quantized.rs:
// decode_q2_k :117-138, decode_q3_k :142-176, decode_q4_k :180-199,
// decode_q5_k :203-234, decode_q6_k :238-261): `d * scale`, `dmin * min`, then
// `dl * q` and `- ml` as separate multiply and subtract. This translation unit
// is compiled with -ffp-contract=off and carries the pragma below so that no
// multiply-subtract pair is ever fused into an FMA.
//
// The kernel is store-bound (4 output bytes per 0.56-1.06 input bytes), so the
// work split is chosen for the stores: one lane produces four consecutive
// output floats and writes them with a single 16-byte store, which makes every
// wave write 1 KiB of contiguous output. Packed bytes are read through the
// vector L1, where the eight lanes that share a 32-value group hit the same line.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "et_codecs.h"
#include "kernels.h"

#pragma clang fp contract(off)

#include "decode_device.h"

namespace et {
namespace {

// crates/runtime-cpu/src/tensor.rs:940-953, for the index tensor.
__device__ __forceinline__ uint64_t source_index(const IndexLayout& layout, uint64_t logical) {
    if (layout.contiguous) return layout.offset + logical;
    uint64_t source = layout.offset;
    uint64_t remainder = logical;
    for (int d = layout.rank - 1; d >= 0; d--) {
        const uint64_t width = layout.shape[d] > 1 ? layout.shape[d] : 1;
        source += (remainder % width) * layout.strides[d];
        remainder /= width;
    }
    return source;
}

constexpr uint64_t kNoBadIndex = ~0ull;
constexpr uint32_t kChunksPerPass = 4;  // 1024-column chunks a workgroup decodes per pass

__global__ void status_init_kernel(unsigned long long* status) {
    if (threadIdx.x == 0) {
        status[0] = kNoBadIndex;
        status[1] = 0;
    }
}

// Runs after the gather: records the offending index VALUE for the first
// (lowest logical position) bad index, so the host can word the error like
// crates/runtime-cpu/src/quantized.rs:570-583.
__global__ void status_finalize_kernel(const void* indexes, int index_is_i64, IndexLayout layout,
                                       unsigned long long* status) {
    if (threadIdx.x != 0) return;
    const uint64_t position = status[0];
    if (position == kNoBadIndex) return;
    const uint64_t source = source_index(layout, position);
    const long long value = index_is_i64 ? static_cast<const long long*>(indexes)[source]
                                         : static_cast<long long>(static_cast<const uint32_t*>(indexes)[source]);
    status[1] = static_cast<unsigned long long>(value);
}

// One workgroup per (output row, four 1024-column chunks): the row's index is read once per workgroup
// and everything per lane is 32-bit arithmetic (a 64-bit division per item, as a flat grid-stride
// loop over all outputs needs, costs more than the decode itself).
template <int CODEC>
__global__ __launch_bounds__(256) void dequant_rows_kernel(
    const uint8_t* __restrict__ weight, const void* __restrict__ indexes, int index_is_i64,
    IndexLayout layout, uint64_t out_rows, uint64_t table_rows, uint32_t columns,
    uint64_t row_bytes, float* __restrict__ out, unsigned long long* status) {
    constexpr uint32_t kValues = block_values(CODEC);
    constexpr uint32_t kBytes = block_bytes(CODEC);
    const uint32_t chunks = (columns + 1023u) >> 10;
    for (uint64_t p = blockIdx.x; p < out_rows; p += gridDim.x) {
        uint64_t row = p;
        if (indexes != nullptr) {
            const uint64_t source = source_index(layout, p);
            bool bad;
            if (index_is_i64) {
                const long long value = static_cast<const long long*>(indexes)[source];
                bad = value < 0 || static_cast<uint64_t>(value) >= table_rows;
                row = static_cast<uint64_t>(value);
            } else {
                row = static_cast<const uint32_t*>(indexes)[source];
                bad = row >= table_rows;
            }
            if (bad) {
                if (blockIdx.y == 0 && threadIdx.x == 0) atomicMin(status, static_cast<unsigned long long>(p));
                continue;  // skipped, like the reference's Metal kernel
            }
        }
        const uint8_t* packed_row = weight + row * row_bytes;
        float* out_row = out + p * columns;
        // Four chunks per pass, all decoded before the first store: their loads are in flight together.
        for (uint32_t first = blockIdx.y * kChunksPerPass; first < chunks; first += gridDim.y * kChunksPerPass) {
            float values[kChunksPerPass][4];
#pragma unroll
            for (uint32_t u = 0; u < kChunksPerPass; u++) {
                const uint32_t column = ((first + u) << 10) + (threadIdx.x << 2);
                if (column >= columns) continue;  // columns is a multiple of the block width, so of four
                const uint32_t block_index = column / kValues;
                decode4<CODEC>(packed_row + static_cast<uint64_t>(block_index) * kBytes, column - block_index * kValues,
                               values[u]);
            }
#pragma unroll
            for (uint32_t u = 0; u < kChunksPerPass; u++) {
                const uint32_t column = ((first + u) << 10) + (threadIdx.x << 2);
                if (column >= columns) continue;
                *reinterpret_cast<float4*>(out_row + column) =
                    make_float4(values[u][0], values[u][1], values[u][2], values[u][3]);
            }
        }
    }
}

template <int CODEC>
hipError_t launch_dequant(const uint8_t* weight, const void* indexes, int index_is_i64,
                          const IndexLayout& layout, uint64_t out_rows, uint64_t table_rows,
                          uint64_t columns, float* out, void* status, hipStream_t stream) {
    const uint64_t row_bytes = columns / block_values(CODEC) * block_bytes(CODEC);
    if (out_rows == 0 || columns == 0) return hipSuccess;
    // The loops in the kernel take what the grid limits leave over.
    const uint64_t chunks = (((columns + 1023) >> 10) + kChunksPerPass - 1) / kChunksPerPass;
    const uint32_t grid_x = static_cast<uint32_t>(out_rows < (1u << 24) ? out_rows : (1u << 24));
    const uint32_t grid_y = static_cast<uint32_t>(chunks < 1024 ? chunks : 1024);
    auto* status_words = static_cast<unsigned long long*>(status);
    if (indexes != nullptr) {
        hipLaunchKernelGGL(status_init_kernel, dim3(1), dim3(64), 0, stream, status_words);
    }
    hipLaunchKernelGGL(dequant_rows_kernel<CODEC>, dim3(grid_x, grid_y), dim3(256), 0,
                       stream, weight, indexes, index_is_i64, layout, out_rows, table_rows,
                       static_cast<uint32_t>(columns), row_bytes, out, status_words);
    if (indexes != nullptr) {
        hipLaunchKernelGGL(status_finalize_kernel, dim3(1), dim3(64), 0, stream, indexes,
                           index_is_i64, layout, status_words);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t dequantize_rows(int32_t codec, const uint8_t* weight, const void* indexes,
                           int index_is_i64, const IndexLayout& layout, uint64_t out_rows,
                           uint64_t table_rows, uint64_t columns, float* out, void* status,
                           hipStream_t stream) {
    switch (codec) {
        case kQ4_0: return launch_dequant<kQ4_0>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ8_0: return launch_dequant<kQ8_0>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ2_K: return launch_dequant<kQ2_K>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ3_K: return launch_dequant<kQ3_K>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ4_K: return launch_dequant<kQ4_K>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ5_K: return launch_dequant<kQ5_K>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        case kQ6_K: return launch_dequant<kQ6_K>(weight, indexes, index_is_i64, layout, out_rows, table_rows, columns, out, status, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace et
