// The small operators on the decode critical path next to the quantized contraction, for
// gfx950. Each is a plain streaming kernel: the data of a decode step is a few hundred KB, so
// what matters is one launch per operator and full-width loads.
//
//   rms_norm_kernel     rms_norm_forward_into_impl (crates/runtime-cpu/src/composed.rs:1457-1487)
//   rotary_kernel       rotary_forward_into_impl (composed.rs:2683-2729)
//   silu_mul_kernel     Tensor.silu (packages/core/src/Tensor.ts:1537-1540) times the up projection
//   add_kernel          the residual connections (binary add, crates/runtime-cpu/src/ops.rs)
//   argmax_kernel       sample_logits with temperature 0 (crates/runtime/src/sampling.rs:86-103)
//   gather_rows_kernel  index_select along dimension 0 (crates/runtime-cpu/src/indexing.rs:152-187)
//
// The reference computes the first two in f64 and rounds once; so do these kernels (the rows
// are short, f64 costs nothing that shows), which keeps them within one f32 rounding of it.
#include <hip/hip_runtime.h>

#include <cmath>

#include "decode_math.h"
#include "kernels.h"

namespace et {
namespace {

constexpr uint32_t kArgmaxChunk = 4096;  // logits per workgroup of the first stage

// One workgroup of 256 per row. VEC: the row is read as float4 (columns % 4 == 0, 16-byte aligned
// rows); the first four vectors of a thread stay in registers for the second pass.
template <bool VEC>
__global__ __launch_bounds__(256) void rms_norm_kernel(const float* __restrict__ x, const NormWeight weight,
                                                       double eps, float* __restrict__ out, uint32_t columns) {
    __shared__ double partial[4];
    const float* in = x + static_cast<uint64_t>(blockIdx.x) * columns;
    float* row = out + static_cast<uint64_t>(blockIdx.x) * columns;
    if constexpr (VEC) {
        float4 held[kRmsHeld];
        const double scale = rms_row_scale(in, columns, eps, held, partial);
        const uint32_t vectors = columns / 4;
#pragma unroll
        for (int j = 0; j < kRmsHeld; j++) {
            const uint32_t i = threadIdx.x + 256 * j;
            if (i < vectors) reinterpret_cast<float4*>(row)[i] = rms_four(held[j], scale, norm_weight_four(weight, i));
        }
        for (uint32_t i = threadIdx.x + 256 * kRmsHeld; i < vectors; i += 256)
            reinterpret_cast<float4*>(row)[i] =
                rms_four(reinterpret_cast<const float4*>(in)[i], scale, norm_weight_four(weight, i));
    } else {
        double sum = 0.0;
        for (uint32_t i = threadIdx.x; i < columns; i += 256) sum += static_cast<double>(in[i]) * static_cast<double>(in[i]);
        sum = wave_sum(sum);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
        __syncthreads();
        const double mean_square = ((partial[0] + partial[1]) + (partial[2] + partial[3])) / static_cast<double>(columns);
        const double scale = 1.0 / sqrt(mean_square + eps);
        for (uint32_t i = threadIdx.x; i < columns; i += 256) row[i] = rms_one(in[i], scale, norm_weight_one(weight, i));
    }
}

// One thread per (row, step, pair), over one tensor or two of the same steps and head width (the
// queries and the keys of a decode step).
struct RotaryTensor {
    const float* x;
    float* out;
    uint32_t rows_per_batch;
    uint64_t pairs;
};
__global__ __launch_bounds__(256) void rotary_kernel(RotaryTensor first, RotaryTensor second,
                                                     const uint32_t* __restrict__ offsets, uint32_t offsets_len,
                                                     double theta, double sign, int interleaved, uint32_t steps,
                                                     uint32_t head_dim) {
    uint64_t item = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= first.pairs + second.pairs) return;
    const bool in_second = item >= first.pairs;
    if (in_second) item -= first.pairs;
    const float* x = in_second ? second.x : first.x;
    float* out = in_second ? second.out : first.out;
    const uint32_t rows_per_batch = in_second ? second.rows_per_batch : first.rows_per_batch;
    const uint32_t half = head_dim / 2;
    const uint32_t index = static_cast<uint32_t>(item % half);
    const uint64_t row_step = item / half;
    const uint32_t step = static_cast<uint32_t>(row_step % steps);
    const uint64_t row = row_step / steps;
    const uint32_t offset = offsets_len == 1 ? offsets[0] : offsets[row / rows_per_batch];
    const uint64_t base = row_step * head_dim;
    const uint64_t lo = interleaved ? base + 2 * index : base + index;
    const uint64_t hi = interleaved ? base + 2 * index + 1 : base + half + index;
    float rotated_lo, rotated_hi;
    rotate_pair(x[lo], x[hi], offset, step, index, head_dim, theta, sign, rotated_lo, rotated_hi);
    out[lo] = rotated_lo;
    out[hi] = rotated_hi;
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       float* out, uint64_t count, int vectorised) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (vectorised) {
        if (4 * i >= count) return;
        const float4 g = reinterpret_cast<const float4*>(gate)[i], u = reinterpret_cast<const float4*>(up)[i];
        reinterpret_cast<float4*>(out)[i] = make_float4(silu_mul_one(g.x, u.x), silu_mul_one(g.y, u.y),
                                                        silu_mul_one(g.z, u.z), silu_mul_one(g.w, u.w));
    } else if (i < count) {
        out[i] = silu_mul_one(gate[i], up[i]);
    }
}

__global__ __launch_bounds__(256) void add_kernel(const float* a, const float* b,
                                                  float* out, uint64_t count, int vectorised) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (vectorised) {
        if (4 * i >= count) return;
        const float4 x = reinterpret_cast<const float4*>(a)[i], y = reinterpret_cast<const float4*>(b)[i];
        reinterpret_cast<float4*>(out)[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    } else if (i < count) {
        out[i] = a[i] + b[i];
    }
}

// Greedy selection in two launches. Stage 1: one workgroup of 256 per (row, chunk of kArgmaxChunk
// logits) writes the chunk's largest value, its lowest token and the first token that is not
// finite. Stage 2: one wave per row combines the chunks (status[row] = that token + 1, 0 = none).
struct ArgmaxPartial {
    float value;
    uint32_t token, bad;
};

__device__ __forceinline__ void argmax_merge(float& best, uint32_t& token, uint32_t& bad, float other,
                                             uint32_t other_token, uint32_t other_bad) {
    if (other > best || (other == best && other_token < token)) {
        best = other;
        token = other_token;
    }
    bad = min(bad, other_bad);
}

template <bool VEC>
__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, uint32_t columns,
                                                            uint32_t chunks, ArgmaxPartial* __restrict__ partials) {
    __shared__ float best_value[4];
    __shared__ uint32_t best_token[4], bad_token[4];
    const uint32_t chunk = blockIdx.x % chunks, row_index = blockIdx.x / chunks;
    const float* row = logits + static_cast<uint64_t>(row_index) * columns;
    const uint32_t begin = chunk * kArgmaxChunk, end = min(begin + kArgmaxChunk, columns);
    float best = -INFINITY;
    uint32_t token = 0xffffffffu, bad = 0xffffffffu;
    const auto take = [&](float value, uint32_t i) {
        if (!isfinite(value)) bad = min(bad, i);
        if (value > best) {
            best = value;
            token = i;
        }
    };
    if constexpr (VEC) {
        // rows are 16-byte aligned and columns % 4 == 0: four loads of four logits in flight per thread
        constexpr int kLoads = kArgmaxChunk / (4 * 256);
        float4 v[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            const uint32_t i = begin + 4 * (threadIdx.x + 256 * j);
            v[j] = i < end ? *reinterpret_cast<const float4*>(row + i) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            const uint32_t i = begin + 4 * (threadIdx.x + 256 * j);
            if (i < end) {
                take(v[j].x, i);
                take(v[j].y, i + 1);
                take(v[j].z, i + 2);
                take(v[j].w, i + 3);
            }
        }
    } else {
        for (uint32_t i = begin + threadIdx.x; i < end; i += 256) take(row[i], i);
    }
    for (int offset = 32; offset > 0; offset >>= 1)
        argmax_merge(best, token, bad, __shfl_xor(best, offset), __shfl_xor(token, offset), __shfl_xor(bad, offset));
    if ((threadIdx.x & 63) == 0) {
        best_value[threadIdx.x >> 6] = best;
        best_token[threadIdx.x >> 6] = token;
        bad_token[threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) argmax_merge(best, token, bad, best_value[w], best_token[w], bad_token[w]);
        partials[blockIdx.x] = ArgmaxPartial{best, token, bad};
    }
}

__global__ __launch_bounds__(64) void argmax_rows_kernel(const ArgmaxPartial* __restrict__ partials, uint32_t chunks,
                                                         uint32_t* __restrict__ out, uint32_t* __restrict__ status) {
    const ArgmaxPartial* row = partials + static_cast<uint64_t>(blockIdx.x) * chunks;
    float best = -INFINITY;
    uint32_t token = 0xffffffffu, bad = 0xffffffffu;
    for (uint32_t i = threadIdx.x; i < chunks; i += 64) argmax_merge(best, token, bad, row[i].value, row[i].token, row[i].bad);
    for (int offset = 32; offset > 0; offset >>= 1)
        argmax_merge(best, token, bad, __shfl_xor(best, offset), __shfl_xor(token, offset), __shfl_xor(bad, offset));
    if (threadIdx.x == 0) {
        // a row without any finite logit above -inf selects nothing; the status reports it
        out[blockIdx.x] = token == 0xffffffffu ? 0u : token;
        status[blockIdx.x] = bad == 0xffffffffu ? 0u : bad + 1;
    }
}

// One workgroup per gathered row; rows are copied as bytes. status[p] = 0, or the offending
// index + 1 (saturated) when it lies outside the table, in which case the row is left alone.
template <typename Word>
__global__ __launch_bounds__(256) void gather_rows_kernel(const Word* __restrict__ table, uint64_t table_rows,
                                                          uint64_t row_words, const void* __restrict__ indexes,
                                                          int index_is_i64, Word* __restrict__ out,
                                                          unsigned long long* __restrict__ status) {
    const uint64_t p = blockIdx.x;
    const long long id = index_is_i64 ? static_cast<const long long*>(indexes)[p]
                                      : static_cast<long long>(static_cast<const uint32_t*>(indexes)[p]);
    const bool inside = id >= 0 && static_cast<uint64_t>(id) < table_rows;
    if (threadIdx.x == 0) status[p] = inside ? 0ull : (1ull << 63) | (static_cast<unsigned long long>(id) & ~(1ull << 63));
    if (!inside) return;
    const Word* source = table + static_cast<uint64_t>(id) * row_words;
    Word* target = out + p * row_words;
    for (uint64_t i = threadIdx.x; i < row_words; i += 256) target[i] = source[i];
}

// The lookup of a half-float table into f32 rows: index_select followed by the cast the reference's
// graph puts behind it, in one launch (the widening is exact). HALF: IEEE binary16, else bfloat16.
template <bool HALF>
__global__ __launch_bounds__(256) void gather_rows_widen_kernel(const uint16_t* __restrict__ table, uint64_t table_rows,
                                                                uint64_t width, const void* __restrict__ indexes,
                                                                int index_is_i64, float* __restrict__ out,
                                                                unsigned long long* __restrict__ status) {
    const uint64_t p = blockIdx.x;
    const long long id = index_is_i64 ? static_cast<const long long*>(indexes)[p]
                                      : static_cast<long long>(static_cast<const uint32_t*>(indexes)[p]);
    const bool inside = id >= 0 && static_cast<uint64_t>(id) < table_rows;
    if (threadIdx.x == 0) status[p] = inside ? 0ull : (1ull << 63) | (static_cast<unsigned long long>(id) & ~(1ull << 63));
    if (!inside) return;
    const uint16_t* source = table + static_cast<uint64_t>(id) * width;
    float* target = out + p * width;
    const auto widen = [](uint16_t bits) {
        if constexpr (HALF) {
            union {
                uint16_t u;
                _Float16 h;
            } cvt;
            cvt.u = bits;
            return static_cast<float>(cvt.h);
        } else {
            return __uint_as_float(static_cast<uint32_t>(bits) << 16);
        }
    };
    if (width % 4 == 0 && reinterpret_cast<uintptr_t>(source) % 8 == 0 && reinterpret_cast<uintptr_t>(target) % 16 == 0) {
        for (uint64_t i = threadIdx.x; i < width / 4; i += 256) {
            const uint2 raw = reinterpret_cast<const uint2*>(source)[i];
            reinterpret_cast<float4*>(target)[i] =
                make_float4(widen(static_cast<uint16_t>(raw.x)), widen(static_cast<uint16_t>(raw.x >> 16)),
                            widen(static_cast<uint16_t>(raw.y)), widen(static_cast<uint16_t>(raw.y >> 16)));
        }
    } else {
        for (uint64_t i = threadIdx.x; i < width; i += 256) target[i] = widen(source[i]);
    }
}

// kv_prepare's commit (crates/runtime-cpu/src/napi/mod.rs:4511-4517): cursor += advance for the active slots.
__global__ __launch_bounds__(64) void commit_advances_kernel(uint32_t* __restrict__ cursors,
                                                             const uint32_t* __restrict__ advances, uint32_t slots) {
    const uint32_t slot = blockIdx.x * 64u + threadIdx.x;
    if (slot < slots) cursors[slot] += advances[slot];
}

}  // namespace

hipError_t commit_advances(uint32_t* cursors, const uint32_t* advances, uint64_t slots, hipStream_t stream) {
    if (slots == 0) return hipSuccess;
    hipLaunchKernelGGL(commit_advances_kernel, dim3(static_cast<uint32_t>((slots + 63) / 64)), dim3(64), 0, stream, cursors,
                       advances, static_cast<uint32_t>(slots));
    return hipGetLastError();
}

hipError_t gather_rows_widen(const void* table, int table_is_bf16, uint64_t table_rows, uint64_t width, const void* indexes,
                             int index_is_i64, uint64_t count, float* out, void* status, hipStream_t stream) {
    auto* words = static_cast<unsigned long long*>(status);
    if (table_is_bf16)
        hipLaunchKernelGGL(gather_rows_widen_kernel<false>, dim3(static_cast<uint32_t>(count)), dim3(256), 0, stream,
                           static_cast<const uint16_t*>(table), table_rows, width, indexes, index_is_i64, out, words);
    else
        hipLaunchKernelGGL(gather_rows_widen_kernel<true>, dim3(static_cast<uint32_t>(count)), dim3(256), 0, stream,
                           static_cast<const uint16_t*>(table), table_rows, width, indexes, index_is_i64, out, words);
    return hipGetLastError();
}

hipError_t rms_norm(const float* x, const void* weight, int weight_is_half, double eps, float* out, uint64_t rows,
                    uint64_t columns, hipStream_t stream) {
    const auto aligned = [](const void* p, uintptr_t to) { return reinterpret_cast<uintptr_t>(p) % to == 0; };
    const NormWeight w = {weight, weight_is_half ? 1 : 0};
    if (columns % 4 == 0 && aligned(x, 16) && aligned(out, 16) && aligned(weight, weight_is_half ? 8 : 16))
        hipLaunchKernelGGL(rms_norm_kernel<true>, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream, x, w, eps,
                           out, static_cast<uint32_t>(columns));
    else
        hipLaunchKernelGGL(rms_norm_kernel<false>, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream, x, w, eps,
                           out, static_cast<uint32_t>(columns));
    return hipGetLastError();
}

hipError_t rotary(const float* x, const uint32_t* offsets, uint32_t offsets_len, double theta, double sign,
                  int interleaved, float* out, uint64_t batch, uint64_t rows, uint64_t steps, uint64_t head_dim,
                  hipStream_t stream) {
    return rotary_pair(x, out, rows, nullptr, nullptr, 0, offsets, offsets_len, theta, sign, interleaved, batch, steps,
                       head_dim, stream);
}

hipError_t rotary_pair(const float* x, float* out, uint64_t rows, const float* second, float* second_out,
                       uint64_t second_rows, const uint32_t* offsets, uint32_t offsets_len, double theta, double sign,
                       int interleaved, uint64_t batch, uint64_t steps, uint64_t head_dim, hipStream_t stream) {
    const RotaryTensor a = {x, out, static_cast<uint32_t>(rows / batch), rows * steps * (head_dim / 2)};
    const RotaryTensor b = {second, second_out, static_cast<uint32_t>(second_rows / batch),
                            second_rows * steps * (head_dim / 2)};
    const uint64_t pairs = a.pairs + b.pairs;
    if (pairs == 0) return hipSuccess;
    hipLaunchKernelGGL(rotary_kernel, dim3(static_cast<uint32_t>((pairs + 255) / 256)), dim3(256), 0, stream, a, b,
                       offsets, offsets_len, theta, sign, interleaved, static_cast<uint32_t>(steps),
                       static_cast<uint32_t>(head_dim));
    return hipGetLastError();
}

hipError_t silu_mul(const float* gate, const float* up, float* out, uint64_t count, hipStream_t stream) {
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const int vectorised = count % 4 == 0 && aligned(gate) && aligned(up) && aligned(out);
    const uint64_t items = vectorised ? count / 4 : count;
    hipLaunchKernelGGL(silu_mul_kernel, dim3(static_cast<uint32_t>((items + 255) / 256)), dim3(256), 0, stream, gate, up,
                       out, count, vectorised);
    return hipGetLastError();
}

hipError_t add(const float* a, const float* b, float* out, uint64_t count, hipStream_t stream) {
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const int vectorised = count % 4 == 0 && aligned(a) && aligned(b) && aligned(out);
    const uint64_t items = vectorised ? count / 4 : count;
    hipLaunchKernelGGL(add_kernel, dim3(static_cast<uint32_t>((items + 255) / 256)), dim3(256), 0, stream, a, b, out,
                       count, vectorised);
    return hipGetLastError();
}

uint64_t argmax_workspace_bytes(uint64_t rows, uint64_t columns) {
    return rows * ((columns + kArgmaxChunk - 1) / kArgmaxChunk) * sizeof(ArgmaxPartial);
}

hipError_t argmax_rows(const float* logits, uint64_t rows, uint64_t columns, uint32_t* out, uint32_t* status,
                       void* workspace, hipStream_t stream) {
    const uint32_t chunks = static_cast<uint32_t>((columns + kArgmaxChunk - 1) / kArgmaxChunk);
    auto* partials = static_cast<ArgmaxPartial*>(workspace);
    if (columns % 4 == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0)
        hipLaunchKernelGGL(argmax_chunks_kernel<true>, dim3(static_cast<uint32_t>(rows * chunks)), dim3(256), 0, stream,
                           logits, static_cast<uint32_t>(columns), chunks, partials);
    else
        hipLaunchKernelGGL(argmax_chunks_kernel<false>, dim3(static_cast<uint32_t>(rows * chunks)), dim3(256), 0, stream,
                           logits, static_cast<uint32_t>(columns), chunks, partials);
    hipError_t error = hipGetLastError();
    if (error != hipSuccess) return error;
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(static_cast<uint32_t>(rows)), dim3(64), 0, stream, partials, chunks, out,
                       status);
    return hipGetLastError();
}

hipError_t gather_rows(const void* table, uint64_t table_rows, uint64_t row_bytes, const void* indexes,
                       int index_is_i64, uint64_t count, void* out, void* status, hipStream_t stream) {
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    auto* words = static_cast<unsigned long long*>(status);
    if (row_bytes % 16 == 0 && aligned(table) && aligned(out))
        hipLaunchKernelGGL(gather_rows_kernel<uint4>, dim3(static_cast<uint32_t>(count)), dim3(256), 0, stream,
                           static_cast<const uint4*>(table), table_rows, row_bytes / 16, indexes, index_is_i64,
                           static_cast<uint4*>(out), words);
    else if (row_bytes % 2 == 0 && reinterpret_cast<uintptr_t>(table) % 2 == 0 && reinterpret_cast<uintptr_t>(out) % 2 == 0)
        hipLaunchKernelGGL(gather_rows_kernel<uint16_t>, dim3(static_cast<uint32_t>(count)), dim3(256), 0, stream,
                           static_cast<const uint16_t*>(table), table_rows, row_bytes / 2, indexes, index_is_i64,
                           static_cast<uint16_t*>(out), words);
    else
        hipLaunchKernelGGL(gather_rows_kernel<uint8_t>, dim3(static_cast<uint32_t>(count)), dim3(256), 0, stream,
                           static_cast<const uint8_t*>(table), table_rows, row_bytes, indexes, index_is_i64,
                           static_cast<uint8_t*>(out), words);
    return hipGetLastError();
}

}  // namespace et
