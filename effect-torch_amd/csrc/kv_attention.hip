// Paged key/value-cache attention for gfx950: the decode neighbour of the quantized
// contraction. Semantics of kv_attention_into (crates/runtime-cpu/src/napi/mod.rs:3320-3544)
// with the cursor arithmetic of kv_prepare (:3568-3603); block allocation stays with the
// caller, which hands over the block table already sized.
//
//   1. kv_write_kernel     new K / V rows -> slabs (f32, or f16 rounded to nearest even as
//                          SlabWriter::set_f32 does, crates/runtime-cpu/src/pool.rs:72-79)
//   2. kv_attend_kernel    one workgroup per (slot, query token, kv head, context split):
//                          streams the split's K and V rows once for all query heads of the
//                          group, online softmax in f32; writes the output, or (m, l, acc)
//                          partials when the context is split
//      kv_attend_any_kernel  the same for widths / groups the streaming kernel does not cover
//   3. kv_merge_kernel     combines the partials of the splits
//
// Slabs are [max_tokens, kv_heads, width]; the row of logical position p of a slot is
// table[slot][p / block_size] * block_size + p % block_size.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>

#include "kernels.h"

namespace et {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr float kLowest = -1.0e30f;  // "no score yet": finite, so that exp2(kLowest - m) = 0 without NaN

struct KvArgs {
    void* k_slab;
    void* v_slab;
    const uint32_t* table;
    const uint32_t* cursors;
    const uint32_t* advances;
    const float* q;
    const float* k;
    const float* v;
    float* out;
    float* partial;
    unsigned long long* status;
    uint32_t max_tokens, kv_heads, width, block_size;
    int32_t block_shift;  // log2(block_size), or -1 when it is not a power of two
    uint32_t table_stride, active_batch, query_heads, tokens, context_window, window;
    uint32_t splits, max_context;
    float scale_log2;  // scale * log2(e)
};

// status word: (slot << 40 | code << 32 | value); the smallest key wins, which is the first
// failing slot in the reference's iteration order and, inside it, the first check that fails.
__device__ void report(unsigned long long* status, uint32_t slot, uint32_t code, uint32_t value) {
    atomicMin(status, (static_cast<unsigned long long>(slot) << 40) |
                          (static_cast<unsigned long long>(code) << 32) | value);
}

struct Span {
    uint32_t cursor, advance, needed, start;
    bool ok;
};

// kv_prepare (napi/mod.rs:3588-3609) on device-resident cursors.
__device__ Span slot_span(const KvArgs& a, uint32_t slot, bool reporter) {
    Span s;
    s.cursor = a.cursors[slot];
    s.advance = a.advances[slot];
    s.needed = s.cursor + s.advance;
    s.start = a.context_window != 0 && s.needed > a.context_window ? s.needed - a.context_window : 0;
    s.ok = true;
    if (s.advance == 0 || s.advance > a.tokens) {
        if (reporter) report(a.status, slot, kKvBadAdvance, s.advance);
        s.ok = false;
    } else if (s.needed - s.start > a.max_tokens) {
        if (reporter) report(a.status, slot, kKvOverCapacity, s.needed - s.start);
        s.ok = false;
    } else if ((static_cast<uint64_t>(s.needed) + a.block_size - 1) / a.block_size > a.table_stride) {
        if (reporter) report(a.status, slot, kKvShortTable, s.needed);
        s.ok = false;
    } else if (s.needed > a.max_context) {
        if (reporter) report(a.status, slot, kKvOverDeclared, s.needed);
        s.ok = false;
    }
    return s;
}

__device__ __forceinline__ uint32_t block_of(const KvArgs& a, uint32_t position) {
    return a.block_shift >= 0 ? position >> a.block_shift : position / a.block_size;
}
__device__ __forceinline__ uint32_t within_block(const KvArgs& a, uint32_t position) {
    return a.block_shift >= 0 ? position & (a.block_size - 1) : position % a.block_size;
}

__device__ __forceinline__ void slab_store(float* slab, uint64_t at, float value) { slab[at] = value; }
__device__ __forceinline__ void slab_store(__half* slab, uint64_t at, float value) {
    slab[at] = __float2half_rn(value);
}
__device__ __forceinline__ float slab_load(const float* slab, uint64_t at) { return slab[at]; }
__device__ __forceinline__ float slab_load(const __half* slab, uint64_t at) { return __half2float(slab[at]); }

__global__ void kv_status_init_kernel(unsigned long long* status) {
    if (threadIdx.x == 0) {
        status[0] = ~0ull;
        status[1] = 0;
    }
}

__global__ void kv_zero_kernel(float* out, uint64_t count) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) out[i] = 0.f;
}

// Workgroup = (slot, token, kv head); threads run over the width.
template <typename T>
__global__ void kv_write_kernel(const KvArgs a) {
    uint32_t index = blockIdx.x;
    const uint32_t head = index % a.kv_heads;
    index /= a.kv_heads;
    const uint32_t token = index % a.tokens;
    const uint32_t slot = index / a.tokens;
    const Span s = slot_span(a, slot, token == 0 && head == 0 && threadIdx.x == 0);
    if (!s.ok || token >= s.advance) return;
    const uint32_t position = s.cursor + token;
    const uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                       block_of(a, position)]) * a.block_size +
                         within_block(a, position);
    if (row >= a.max_tokens) {
        if (threadIdx.x == 0) report(a.status, slot, kKvBlockOutside, static_cast<uint32_t>(row));
        return;
    }
    const uint64_t source = ((static_cast<uint64_t>(slot) * a.kv_heads + head) * a.tokens + token) * a.width;
    const uint64_t target = (row * a.kv_heads + head) * a.width;
    for (uint32_t column = threadIdx.x; column < a.width; column += blockDim.x) {
        slab_store(static_cast<T*>(a.k_slab), target + column, a.k[source + column]);
        slab_store(static_cast<T*>(a.v_slab), target + column, a.v[source + column]);
    }
}

// Positions a query attends to (napi/mod.rs:3481-3483).
__device__ __forceinline__ void query_range(const KvArgs& a, const Span& s, uint32_t token,
                                            uint32_t& begin, uint32_t& end) {
    end = min(s.cursor + token + 1, s.needed);
    begin = s.start;
    if (a.window != 0) begin = max(end > a.window ? end - a.window : 0u, s.start);
    begin = min(begin, end);
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over the LANES lanes of an aligned group; every lane gets the total.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LANES >= 2) v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]
    if constexpr (LANES >= 4) v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]
    if constexpr (LANES >= 8) v += dpp_f32<0x141>(v);   // row_half_mirror
    if constexpr (LANES >= 16) v += dpp_f32<0x140>(v);  // row_mirror
    if constexpr (LANES >= 32) v += __shfl_xor(v, 16);
    if constexpr (LANES >= 64) v += __shfl_xor(v, 32);
    return v;
}

// Sixteen bytes of a slab row as floats.
template <typename T>
struct Piece;
template <>
struct Piece<float> {
    static constexpr int kDims = 4;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i == 0 ? raw.x : i == 1 ? raw.y : i == 2 ? raw.z : raw.w;
        return __uint_as_float(w);
    }
};
template <>
struct Piece<__half> {
    static constexpr int kDims = 8;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = (i >> 1) == 0 ? raw.x : (i >> 1) == 1 ? raw.y : (i >> 1) == 2 ? raw.z : raw.w;
        return __half2float(__ushort_as_half(static_cast<unsigned short>((i & 1) ? (w >> 16) : (w & 0xffffu))));
    }
};

// Streaming kernel. LPT lanes share one position (each holds Piece<T>::kDims of the width,
// width == LPT * kDims), so a wave covers 64 / LPT positions per load and the workgroup
// 4 * 64 / LPT; U such loads are in flight per step. G query heads of one kv head are
// served from the same K / V registers.
template <typename T, int LPT, int G, int U>
__global__ __launch_bounds__(kThreads) void kv_attend_kernel(const KvArgs a) {
    constexpr int DPL = Piece<T>::kDims;
    constexpr int PPW = 64 / LPT;        // positions per wave per load
    constexpr int PPG = kWaves * PPW;    // per workgroup per load
    constexpr int GROUPS = kWaves * PPW; // independent softmax states in the workgroup
    __shared__ uint32_t rows_of_block[kKvTableEntries];
    __shared__ float merge_m[GROUPS][G];
    __shared__ float merge_l[GROUPS][G];
    __shared__ float merge_acc[GROUPS][G][LPT * DPL + 4];

    uint32_t index = blockIdx.x;
    const uint32_t split = index % a.splits;
    index /= a.splits;
    const uint32_t chunks = (a.query_heads / a.kv_heads) / G;
    const uint32_t chunk = index % chunks;
    index /= chunks;
    const uint32_t kv_head = index % a.kv_heads;
    index /= a.kv_heads;
    const uint32_t token = index % a.tokens;
    const uint32_t slot = index / a.tokens;
    const uint32_t head0 = kv_head * (a.query_heads / a.kv_heads) + chunk * G;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPT, group = wave * PPW + lane / LPT;

    const Span s = slot_span(a, slot, false);
    uint32_t begin, end;
    query_range(a, s, token, begin, end);
    // This split's share, in whole steps.
    const uint32_t length = s.ok ? end - begin : 0;
    uint32_t share = (length + a.splits - 1) / a.splits;
    share = (share + PPG * U - 1) / (PPG * U) * (PPG * U);
    const uint32_t my_begin = min(begin + split * share, end);
    const uint32_t my_end = s.ok ? min(my_begin + share, end) : my_begin;

    // Physical first rows of the blocks this split touches.
    const uint32_t first_block = block_of(a, my_begin);
    if (my_end > my_begin) {
        const uint32_t blocks = block_of(a, my_end - 1) - first_block + 1;
        for (uint32_t i = threadIdx.x; i < blocks && i < kKvTableEntries; i += kThreads) {
            uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                         first_block + i]) * a.block_size;
            if (row + a.block_size > a.max_tokens) {
                // the last block may be cut by the pool's end; positions beyond it are the writer's to report
                if (row >= a.max_tokens) row = 0;
            }
            rows_of_block[i] = static_cast<uint32_t>(row);
        }
    }
    __syncthreads();

    float q[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float* source = a.q + ((static_cast<uint64_t>(slot) * a.query_heads + head0 + g) * a.tokens + token) *
                                        a.width + sub * DPL;
#pragma unroll
        for (int d = 0; d < DPL; d++) q[g][d] = source[d] * a.scale_log2;
    }
    float m[G], l[G], acc[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = kLowest;
        l[g] = 0.f;
#pragma unroll
        for (int d = 0; d < DPL; d++) acc[g][d] = 0.f;
    }

    const uint64_t row_bytes = static_cast<uint64_t>(a.kv_heads) * a.width * sizeof(T);
    const uint64_t lane_offset = (static_cast<uint64_t>(kv_head) * a.width + sub * DPL) * sizeof(T);
    const char* k_base = static_cast<const char*>(a.k_slab) + lane_offset;
    const char* v_base = static_cast<const char*>(a.v_slab) + lane_offset;

    auto fetch = [&](uint32_t step_begin, Piece<T> (&kp)[U], Piece<T> (&vp)[U]) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            // positions past the split's end read its last row again and are masked out below
            const uint32_t position = min(step_begin + u * PPG + group, my_end - 1);
            uint32_t row = rows_of_block[min(block_of(a, position) - first_block, kKvTableEntries - 1u)] +
                           within_block(a, position);
            row = min(row, a.max_tokens - 1);
            kp[u].raw = *reinterpret_cast<const uint4*>(k_base + row * row_bytes);
            vp[u].raw = *reinterpret_cast<const uint4*>(v_base + row * row_bytes);
        }
    };

    if (my_end > my_begin) {
        Piece<T> kp[U], vp[U];
        fetch(my_begin, kp, vp);
        for (uint32_t step = my_begin; step < my_end; step += PPG * U) {
            Piece<T> kn[U], vn[U];
            const bool more = step + PPG * U < my_end;
            if (more) fetch(step + PPG * U, kn, vn);
            float score[G][U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool live = step + u * PPG + group < my_end;
#pragma unroll
                for (int g = 0; g < G; g++) {
                    float part = 0.f;
#pragma unroll
                    for (int d = 0; d < DPL; d++) part = fmaf(q[g][d], kp[u].get(d), part);
                    part = group_sum<LPT>(part);
                    score[g][u] = live ? part : -INFINITY;
                }
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float top = m[g];
#pragma unroll
                for (int u = 0; u < U; u++) top = fmaxf(top, score[g][u]);
                const float keep = __builtin_amdgcn_exp2f(m[g] - top);
                float p[U], total = 0.f;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    p[u] = __builtin_amdgcn_exp2f(score[g][u] - top);
                    total += p[u];
                }
                m[g] = top;
                l[g] = fmaf(l[g], keep, total);
#pragma unroll
                for (int d = 0; d < DPL; d++) {
                    float value = acc[g][d] * keep;
#pragma unroll
                    for (int u = 0; u < U; u++) value = fmaf(p[u], vp[u].get(d), value);
                    acc[g][d] = value;
                }
            }
            if (more) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    kp[u] = kn[u];
                    vp[u] = vn[u];
                }
            }
        }
    }

    // Combine the workgroup's softmax states.
#pragma unroll
    for (int g = 0; g < G; g++) {
        if (sub == 0) {
            merge_m[group][g] = m[g];
            merge_l[group][g] = l[g];
        }
#pragma unroll
        for (int d = 0; d < DPL; d++) merge_acc[group][g][sub * DPL + d] = acc[g][d];
    }
    __syncthreads();
    const uint32_t width = LPT * DPL;
    for (uint32_t item = threadIdx.x; item < G * width; item += kThreads) {
        const uint32_t g = item / width, column = item % width;
        float top = kLowest;
        for (int i = 0; i < GROUPS; i++) top = fmaxf(top, merge_m[i][g]);
        float total = 0.f, value = 0.f;
        for (int i = 0; i < GROUPS; i++) {
            const float weight = __builtin_amdgcn_exp2f(merge_m[i][g] - top);
            total = fmaf(weight, merge_l[i][g], total);
            value = fmaf(weight, merge_acc[i][g][column], value);
        }
        const uint64_t query = (static_cast<uint64_t>(slot) * a.query_heads + head0 + g) * a.tokens + token;
        if (a.splits == 1) {
            if (s.ok) a.out[query * width + column] = value / total;
        } else {
            float* record = a.partial + (query * a.splits + split) * (width + 2);
            record[2 + column] = value;
            if (column == 0) {
                record[0] = top;
                record[1] = total;
            }
        }
    }
}

// One wave per (slot, query head, token, split) for any width up to 64 * kKvAnyWidthPerLane and
// any grouping: lanes run over the width, positions are taken one after another.
template <typename T>
__global__ __launch_bounds__(64) void kv_attend_any_kernel(const KvArgs a) {
    uint32_t index = blockIdx.x;
    const uint32_t split = index % a.splits;
    index /= a.splits;
    const uint32_t token = index % a.tokens;
    index /= a.tokens;
    const uint32_t head = index % a.query_heads;
    const uint32_t slot = index / a.query_heads;
    const uint32_t kv_head = head / (a.query_heads / a.kv_heads);
    const int lane = threadIdx.x;

    const Span s = slot_span(a, slot, false);
    uint32_t begin, end;
    query_range(a, s, token, begin, end);
    const uint32_t length = s.ok ? end - begin : 0;
    const uint32_t share = (length + a.splits - 1) / a.splits;
    const uint32_t my_begin = min(begin + split * share, end);
    const uint32_t my_end = s.ok ? min(my_begin + share, end) : my_begin;

    const uint64_t query = (static_cast<uint64_t>(slot) * a.query_heads + head) * a.tokens + token;
    float q[kKvAnyWidthPerLane], acc[kKvAnyWidthPerLane];
#pragma unroll
    for (int i = 0; i < kKvAnyWidthPerLane; i++) {
        const uint32_t column = lane + 64 * i;
        q[i] = column < a.width ? a.q[query * a.width + column] * a.scale_log2 : 0.f;
        acc[i] = 0.f;
    }
    float m = kLowest, l = 0.f;
    const T* keys = static_cast<const T*>(a.k_slab);
    const T* values = static_cast<const T*>(a.v_slab);
    for (uint32_t position = my_begin; position < my_end; position++) {
        uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                     block_of(a, position)]) * a.block_size +
                       within_block(a, position);
        row = min(row, static_cast<uint64_t>(a.max_tokens - 1));
        const uint64_t at = (row * a.kv_heads + kv_head) * a.width;
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < kKvAnyWidthPerLane; i++) {
            const uint32_t column = lane + 64 * i;
            if (column < a.width) part = fmaf(q[i], slab_load(keys, at + column), part);
        }
        const float score = group_sum<64>(part);
        const float top = fmaxf(m, score);
        const float keep = __builtin_amdgcn_exp2f(m - top), p = __builtin_amdgcn_exp2f(score - top);
        m = top;
        l = fmaf(l, keep, p);
#pragma unroll
        for (int i = 0; i < kKvAnyWidthPerLane; i++) {
            const uint32_t column = lane + 64 * i;
            if (column < a.width) acc[i] = fmaf(p, slab_load(values, at + column), acc[i] * keep);
        }
    }
#pragma unroll
    for (int i = 0; i < kKvAnyWidthPerLane; i++) {
        const uint32_t column = lane + 64 * i;
        if (column >= a.width) continue;
        if (a.splits == 1) {
            if (s.ok) a.out[query * a.width + column] = acc[i] / l;
        } else {
            float* record = a.partial + (query * a.splits + split) * (a.width + 2);
            record[2 + column] = acc[i];
            if (column == 0) {
                record[0] = m;
                record[1] = l;
            }
        }
    }
}

// out[query, :] = sum_s w_s acc_s / sum_s w_s l_s with w_s = exp2(m_s - max m); one wave per query row.
__global__ __launch_bounds__(64) void kv_merge_kernel(const KvArgs a) {
    const uint64_t query = blockIdx.x;
    const uint32_t slot = static_cast<uint32_t>(query / (static_cast<uint64_t>(a.query_heads) * a.tokens));
    const Span s = slot_span(a, slot, false);
    if (!s.ok) return;
    const float* records = a.partial + query * a.splits * (a.width + 2);
    float top = kLowest;
    for (uint32_t i = 0; i < a.splits; i++) top = fmaxf(top, records[i * (a.width + 2)]);
    float total = 0.f;
    for (uint32_t i = 0; i < a.splits; i++)
        total = fmaf(__builtin_amdgcn_exp2f(records[i * (a.width + 2)] - top), records[i * (a.width + 2) + 1], total);
    for (uint32_t column = threadIdx.x; column < a.width; column += 64) {
        float value = 0.f;
        for (uint32_t i = 0; i < a.splits; i++)
            value = fmaf(__builtin_amdgcn_exp2f(records[i * (a.width + 2)] - top),
                         records[i * (a.width + 2) + 2 + column], value);
        a.out[query * a.width + column] = value / total;
    }
}

template <typename T, int LPT, int G>
hipError_t launch_streaming(const KvArgs& a, uint32_t workgroups, hipStream_t stream) {
    constexpr int U = G >= 8 ? 2 : 4;
    hipLaunchKernelGGL((kv_attend_kernel<T, LPT, G, U>), dim3(workgroups), dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

template <typename T, int LPT>
hipError_t launch_streaming_group(const KvArgs& a, int g, uint32_t workgroups, hipStream_t stream) {
    switch (g) {
        case 8: return launch_streaming<T, LPT, 8>(a, workgroups, stream);
        case 4: return launch_streaming<T, LPT, 4>(a, workgroups, stream);
        case 2: return launch_streaming<T, LPT, 2>(a, workgroups, stream);
        default: return launch_streaming<T, LPT, 1>(a, workgroups, stream);
    }
}

template <typename T>
hipError_t launch_streaming_width(const KvArgs& a, int g, uint32_t workgroups, hipStream_t stream) {
    switch (a.width / Piece<T>::kDims) {
        case 32: return launch_streaming_group<T, 32>(a, g, workgroups, stream);
        case 16: return launch_streaming_group<T, 16>(a, g, workgroups, stream);
        default: return launch_streaming_group<T, 8>(a, g, workgroups, stream);
    }
}

// Query heads of one kv head served together by the streaming kernel; 0 = not covered.
int streaming_group(const KvAttention& p) {
    const uint32_t dims = p.slab_is_f16 ? 8 : 4;
    if (p.width % dims != 0) return 0;
    const uint32_t lanes = p.width / dims;
    if (lanes != 8 && lanes != 16 && lanes != 32) return 0;
    const uint32_t group = p.query_heads / p.kv_heads;
    for (int g : {8, 4, 2})
        if (group % g == 0) return g;
    return 1;
}

uint32_t positions_per_step(const KvAttention& p, int g) {
    const uint32_t lanes = p.width / (p.slab_is_f16 ? 8 : 4);
    return kWaves * (64 / lanes) * (g >= 8 ? 2 : 4);
}

}  // namespace

KvLaunchShape kv_attention_shape(const KvAttention& p) {
    KvLaunchShape shape{};
    const int g = streaming_group(p);
    shape.streaming = g != 0;
    const uint64_t rows = static_cast<uint64_t>(p.active_batch) * p.tokens *
                          (shape.streaming ? p.kv_heads * ((p.query_heads / p.kv_heads) / g) : p.query_heads);
    // Enough workgroups for every compute unit several times over, and no split shorter than
    // a few steps; the block list of a split must fit the kernel's table.
    const uint64_t context = p.max_context == 0 ? 1 : p.max_context;
    const uint64_t step = shape.streaming ? positions_per_step(p, g) : 64;
    uint64_t splits = 1;
    const uint64_t wanted = shape.streaming ? 2048 : 4096;
    if (rows < wanted) splits = (wanted + rows - 1) / (rows == 0 ? 1 : rows);
    const uint64_t most = (context + 2 * step - 1) / (2 * step);
    if (splits > most) splits = most;
    if (shape.streaming) {
        // a split's share is rounded up to whole steps and may start inside a block
        const uint64_t room = static_cast<uint64_t>(kKvTableEntries - 2) * p.block_size;
        const uint64_t reach = room > 2 * step ? room - step : step;
        const uint64_t least = (context + reach - 1) / reach;
        if (splits < least) splits = least;
    }
    if (splits == 0) splits = 1;
    shape.splits = static_cast<uint32_t>(splits);
    shape.workgroups = rows * splits;
    const uint64_t queries = static_cast<uint64_t>(p.active_batch) * p.query_heads * p.tokens;
    shape.workspace_bytes = splits > 1 ? queries * splits * (p.width + 2) * sizeof(float) : 0;
    return shape;
}

hipError_t kv_status_init(void* status, hipStream_t stream) {
    hipLaunchKernelGGL(kv_status_init_kernel, dim3(1), dim3(64), 0, stream,
                       static_cast<unsigned long long*>(status));
    return hipGetLastError();
}

hipError_t kv_attention(const KvAttention& p, void* workspace, hipStream_t stream) {
    KvArgs a{};
    a.k_slab = p.k_slab;
    a.v_slab = p.v_slab;
    a.table = p.block_table;
    a.cursors = p.cursors;
    a.advances = p.advances;
    a.q = p.q;
    a.k = p.k;
    a.v = p.v;
    a.out = p.out;
    a.partial = static_cast<float*>(workspace);
    a.status = static_cast<unsigned long long*>(p.status);
    a.max_tokens = p.max_tokens;
    a.kv_heads = p.kv_heads;
    a.width = p.width;
    a.block_size = p.block_size;
    a.block_shift = -1;
    for (int shift = 0; shift < 31; shift++)
        if ((1u << shift) == p.block_size) a.block_shift = shift;
    a.table_stride = p.table_stride;
    a.active_batch = p.active_batch;
    a.query_heads = p.query_heads;
    a.tokens = p.tokens;
    a.context_window = p.context_window;
    a.window = p.window;
    a.scale_log2 = static_cast<float>(p.scale * 1.4426950408889634);
    a.max_context = p.max_context;
    const KvLaunchShape shape = kv_attention_shape(p);
    a.splits = shape.splits;

    // out.fill(0.0) for the slots that are not active (napi/mod.rs:3371).
    const uint64_t per_slot = static_cast<uint64_t>(p.query_heads) * p.tokens * p.width;
    if (p.active_batch < p.batch) {
        const uint64_t count = (p.batch - p.active_batch) * per_slot;
        hipLaunchKernelGGL(kv_zero_kernel, dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, stream,
                           p.out + p.active_batch * per_slot, count);
    }
    if (p.active_batch == 0) return hipGetLastError();

    const uint32_t writers = p.active_batch * p.tokens * p.kv_heads;
    const uint32_t writer_threads = p.width >= 256 ? 256 : p.width > 64 ? 128 : 64;
    if (p.slab_is_f16)
        hipLaunchKernelGGL(kv_write_kernel<__half>, dim3(writers), dim3(writer_threads), 0, stream, a);
    else
        hipLaunchKernelGGL(kv_write_kernel<float>, dim3(writers), dim3(writer_threads), 0, stream, a);
    hipError_t error = hipGetLastError();
    if (error != hipSuccess) return error;

    if (shape.streaming) {
        const int g = streaming_group(p);
        error = p.slab_is_f16
                    ? launch_streaming_width<__half>(a, g, static_cast<uint32_t>(shape.workgroups), stream)
                    : launch_streaming_width<float>(a, g, static_cast<uint32_t>(shape.workgroups), stream);
    } else {
        if (p.slab_is_f16)
            hipLaunchKernelGGL(kv_attend_any_kernel<__half>, dim3(static_cast<uint32_t>(shape.workgroups)),
                               dim3(64), 0, stream, a);
        else
            hipLaunchKernelGGL(kv_attend_any_kernel<float>, dim3(static_cast<uint32_t>(shape.workgroups)),
                               dim3(64), 0, stream, a);
        error = hipGetLastError();
    }
    if (error != hipSuccess) return error;
    if (shape.splits > 1) {
        const uint64_t queries = static_cast<uint64_t>(p.active_batch) * p.query_heads * p.tokens;
        hipLaunchKernelGGL(kv_merge_kernel, dim3(static_cast<uint32_t>(queries)), dim3(64), 0, stream, a);
        error = hipGetLastError();
    }
    return error;
}

}  // namespace et
