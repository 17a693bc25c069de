// Paged key/value-cache attention for gfx950: the decode neighbour of the quantized
// contraction. Semantics of kv_attention_into (crates/runtime-cpu/src/napi/mod.rs:3320-3544)
// with the cursor arithmetic of kv_prepare (:3568-3603); block allocation stays with the
// caller, which hands over the block table already sized.
//
//   1. kv_attend_kernel    one workgroup per (slot, query token, kv head, context split):
//                          streams the split's cached K and V rows once for all query heads
//                          of the group, takes the new rows straight from the k / v inputs
//                          (rounded as the slab stores them) and appends them to the slabs
//                          (f32, or f16 rounded to nearest even as SlabWriter::set_f32 does,
//                          crates/runtime-cpu/src/pool.rs:72-79); online softmax in f32;
//                          writes the output, or (m, l, acc) partials when the context is split
//      kv_attend_any_kernel  the same for widths / groups the streaming kernel does not cover
//   2. kv_merge_kernel     combines the partials of the splits
//      (Letting the last split to finish combine them inside the attend kernel was measured: the
//      device-wide fences it needs cost far more than this second launch.)
//
// The reference writes the new rows first and attends afterwards (napi/mod.rs:3393-3544); here
// no workgroup reads a new row back from the slab, so one launch does both.
//
// Slabs are [max_tokens, kv_heads, width]; the row of logical position p of a slot is
// table[slot][p / block_size] * block_size + p % block_size.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "decode_math.h"
#include "et_hip.h"
#include "kernels.h"
#include "quantize_halves.h"

namespace et {
namespace {

constexpr uint32_t kNoBlock = 0xffffffffu;
constexpr float kLowest = -1.0e30f;  // "no score yet": finite, so that exp2(kLowest - m) = 0 without NaN

// Element types of a slab besides float and __half.
struct Bf16 {
    uint16_t bits;
};
struct U8 {  // the int8-quantized tier: byte = round(x / scale) + 128, one f32 scale per row and head
    uint8_t byte;
};

struct KvArgs {
    void* k_slab;
    void* v_slab;
    float* k_scales;  // [max_tokens, kv_heads], the U8 tier only
    float* v_scales;
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
    uint8_t* prepared;       // see KvAttention::prepared; null = none, or a quantiser launch follows
    uint32_t vector_tiles;   // of the prepared activations: ceil(batch / 32)
    KvProjected projected;   // see KvAttention::projected; shares == null: q, k, v above
};

struct Span {
    uint32_t cursor, advance, needed, start;
    uint32_t code;   // the first check of kv_prepare that fails, 0 = none
    uint64_t value;  // what that check reports; cursor + advance needs 33 bits
    bool ok;
};

// kv_prepare (napi/mod.rs:3588-3609) on device-resident cursors.
__device__ Span slot_span(const KvArgs& a, uint32_t slot) {
    Span s;
    s.cursor = a.cursors[slot];
    s.advance = a.advances[slot];
    // The reference adds in usize and cannot wrap; a cursor near 2^32 (an idle slot's -1) must fail
    // a check here, before any table access, instead of wrapping to a small context.
    const uint64_t needed = static_cast<uint64_t>(s.cursor) + s.advance;
    const uint64_t start = a.context_window != 0 && needed > a.context_window ? needed - a.context_window : 0;
    s.code = 0;
    s.value = 0;
    if (s.advance == 0 || s.advance > a.tokens) {
        s.code = kKvBadAdvance;
        s.value = s.advance;
    } else if (needed - start > a.max_tokens) {
        s.code = kKvOverCapacity;
        s.value = needed - start;
    } else if ((needed + a.block_size - 1) / a.block_size > a.table_stride) {
        s.code = kKvShortTable;
        s.value = needed;
    } else if (needed > a.max_context) {  // max_context is 32 bits wide: passing means no wrap below
        s.code = kKvOverDeclared;
        s.value = needed;
    }
    s.ok = s.code == 0;
    s.needed = s.ok ? static_cast<uint32_t>(needed) : 0;
    s.start = s.ok ? static_cast<uint32_t>(start) : 0;
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
// the value a slab of this type holds after storing `value`
__device__ __forceinline__ float slab_round(const float*, float value) { return value; }
__device__ __forceinline__ float slab_round(const __half*, float value) {
    return __half2float(__float2half_rn(value));
}
__device__ __forceinline__ float slab_load(const float* slab, uint64_t at) { return slab[at]; }
__device__ __forceinline__ float slab_load(const __half* slab, uint64_t at) { return __half2float(slab[at]); }
// bf16::from_f32 (half 2.7.1): NaN keeps its top bits and gets a quiet bit, else round to nearest even.
__device__ __forceinline__ uint32_t bf16_bits(float value) {
    const uint32_t x = __float_as_uint(value);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (x >> 16) | 0x0040u;
    return (x + 0x7fffu + ((x >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ void slab_store(Bf16* slab, uint64_t at, float value) {
    slab[at].bits = static_cast<uint16_t>(bf16_bits(value));
}
__device__ __forceinline__ float slab_round(const Bf16*, float value) { return __uint_as_float(bf16_bits(value) << 16); }
__device__ __forceinline__ float slab_load(const Bf16* slab, uint64_t at) {
    return __uint_as_float(static_cast<uint32_t>(slab[at].bits) << 16);
}
// The U8 tier (napi/mod.rs:3397-3437, :3467-3478): scale = max|x| / 127 + 1e-12 over the row of a
// head, byte = clamp(round(x / scale), +-127) + 128 (halves away from zero), value = (byte - 128) * scale.
__device__ __forceinline__ float u8_scale(float row_maximum) { return row_maximum / 127.0f + 1e-12f; }
__device__ __forceinline__ uint32_t u8_byte(float value, float scale) {
    return static_cast<uint32_t>(fminf(fmaxf(roundf(value / scale), -127.0f), 127.0f) + 128.0f);
}
__device__ __forceinline__ float u8_value(uint32_t byte, float scale) {
    return (static_cast<float>(byte) - 128.0f) * scale;
}

__global__ void kv_zero_kernel(float* out, uint64_t count, unsigned long long* status, uint32_t slots) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) out[i] = 0.f;
    if (i < slots) status[i] = 0;
}

// The status word of a slot: 0, or code << 56 | value. Written by one wave per slot, which also
// checks that the rows of the new positions lie inside the pool.
__device__ void write_slot_status(const KvArgs& a, uint32_t slot, const Span& s, int lane) {
    uint32_t code = s.code;
    uint64_t value = s.value;
    if (s.ok) {
        uint32_t worst = 0;
        for (uint32_t token = lane; token < s.advance; token += 64) {
            const uint32_t position = s.cursor + token;
            const uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                               block_of(a, position)]) * a.block_size +
                                 within_block(a, position);
            if (row >= a.max_tokens) worst = max(worst, static_cast<uint32_t>(min(row, uint64_t{0xffffffffu})));
        }
        for (int offset = 32; offset > 0; offset >>= 1) worst = max(worst, __shfl_xor(worst, offset));
        if (worst != 0) {
            code = kKvBlockOutside;
            value = worst;
        }
    }
    if (lane == 0) a.status[slot] = (static_cast<unsigned long long>(code) << 56) | value;
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

template <int LANES>
__device__ __forceinline__ float group_max(float v) {
    if constexpr (LANES >= 2) v = fmaxf(v, dpp_f32<0xB1>(v));
    if constexpr (LANES >= 4) v = fmaxf(v, dpp_f32<0x4E>(v));
    if constexpr (LANES >= 8) v = fmaxf(v, dpp_f32<0x141>(v));
    if constexpr (LANES >= 16) v = fmaxf(v, dpp_f32<0x140>(v));
    if constexpr (LANES >= 32) v = fmaxf(v, __shfl_xor(v, 16));
    if constexpr (LANES >= 64) v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}

// Sixteen bytes of a slab row as floats.
template <typename T>
struct Piece;
template <>
struct Piece<float> {
    static constexpr int kDims = 4;
    static constexpr int kElementBytes = 4;
    static constexpr bool kScaled = false;
    using Raw = uint4;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i == 0 ? raw.x : i == 1 ? raw.y : i == 2 ? raw.z : raw.w;
        return __uint_as_float(w);
    }
    // what the slab would hold for these input values (LANES lanes share the row of a head)
    template <int LANES>
    __device__ __forceinline__ void from_input(const float* source) {
        raw = *reinterpret_cast<const uint4*>(source);
    }
};
template <>
struct Piece<__half> {
    static constexpr int kDims = 8;
    static constexpr int kElementBytes = 2;
    static constexpr bool kScaled = false;
    using Raw = uint4;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = (i >> 1) == 0 ? raw.x : (i >> 1) == 1 ? raw.y : (i >> 1) == 2 ? raw.z : raw.w;
        return __half2float(__ushort_as_half(static_cast<unsigned short>((i & 1) ? (w >> 16) : (w & 0xffffu))));
    }
    template <int LANES>
    __device__ __forceinline__ void from_input(const float* source) {
        const float4 low = *reinterpret_cast<const float4*>(source);
        const float4 high = *reinterpret_cast<const float4*>(source + 4);
        const auto pack = [](float x, float y) {
            return static_cast<uint32_t>(__half_as_ushort(__float2half_rn(x))) |
                   (static_cast<uint32_t>(__half_as_ushort(__float2half_rn(y))) << 16);
        };
        raw = make_uint4(pack(low.x, low.y), pack(low.z, low.w), pack(high.x, high.y), pack(high.z, high.w));
    }
};
template <>
struct Piece<Bf16> {
    static constexpr int kDims = 8;
    static constexpr int kElementBytes = 2;
    static constexpr bool kScaled = false;
    using Raw = uint4;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = (i >> 1) == 0 ? raw.x : (i >> 1) == 1 ? raw.y : (i >> 1) == 2 ? raw.z : raw.w;
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    template <int LANES>
    __device__ __forceinline__ void from_input(const float* source) {
        const float4 low = *reinterpret_cast<const float4*>(source);
        const float4 high = *reinterpret_cast<const float4*>(source + 4);
        const auto pack = [](float x, float y) { return bf16_bits(x) | (bf16_bits(y) << 16); };
        raw = make_uint4(pack(low.x, low.y), pack(low.z, low.w), pack(high.x, high.y), pack(high.z, high.w));
    }
};
// The u8 tier takes eight bytes per lane, not sixteen: a head of width 128 then spans sixteen lanes,
// the shape the reduce-scatter softmax (attend_step_scatter) is built for.
template <>
struct Piece<U8> {
    static constexpr int kDims = 8;
    static constexpr int kElementBytes = 1;
    static constexpr bool kScaled = true;
    using Raw = uint2;
    uint2 raw;
    float scale;  // of the row and head these bytes belong to
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = (i >> 2) == 0 ? raw.x : raw.y;
        // (byte - 128) * scale, one rounding: -128 * scale is exact
        return fmaf(static_cast<float>((w >> (8 * (i & 3))) & 0xffu), scale, -128.0f * scale);
    }
    template <int LANES>
    __device__ __forceinline__ void from_input(const float* source) {
        const float4 low = *reinterpret_cast<const float4*>(source);
        const float4 high = *reinterpret_cast<const float4*>(source + 4);
        const float values[8] = {low.x, low.y, low.z, low.w, high.x, high.y, high.z, high.w};
        float maximum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) maximum = fmaxf(maximum, fabsf(values[i]));
        scale = u8_scale(group_max<LANES>(maximum));
        uint32_t words[2];
#pragma unroll
        for (int j = 0; j < 2; j++)
            words[j] = u8_byte(values[4 * j], scale) | (u8_byte(values[4 * j + 1], scale) << 8) |
                       (u8_byte(values[4 * j + 2], scale) << 16) | (u8_byte(values[4 * j + 3], scale) << 24);
        raw = make_uint2(words[0], words[1]);
    }
};

// A cached row is read once per launch: non-temporal loads, so that the caches keep nothing of it
// (measured on plain reads of this device: 7.1 against 6.2 TB/s on 1 GiB).
__device__ __forceinline__ uint4 load_streamed(const uint4* source) {
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const v4u raw = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(source));
    return make_uint4(raw.x, raw.y, raw.z, raw.w);
}
__device__ __forceinline__ uint2 load_streamed(const uint2* source) {
    typedef uint32_t v2u __attribute__((ext_vector_type(2)));
    const v2u raw = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(source));
    return make_uint2(raw.x, raw.y);
}

// One step of the online softmax over U positions per lane group: scores of the G query heads
// against kp[], then the running maximum, denominator and value sums.
template <typename T, int LPT, int G, int U>
__device__ __forceinline__ void attend_step(const float (&q)[G][Piece<T>::kDims], const Piece<T> (&kp)[U],
                                            const Piece<T> (&vp)[U], const bool (&live)[U], float (&m)[G],
                                            float (&l)[G], float (&acc)[G][Piece<T>::kDims]) {
    constexpr int DPL = Piece<T>::kDims;
    float score[G][U];
#pragma unroll
    for (int u = 0; u < U; u++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            float part = 0.f;
#pragma unroll
            for (int d = 0; d < DPL; d++) part = fmaf(q[g][d], kp[u].get(d), part);
            part = group_sum<LPT>(part);
            score[g][u] = live[u] ? part : -INFINITY;
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
}

// Softmax state of the scatter step: the lanes r = sub % 16 of a 16-lane row with
// r / (16 / G) == g hold the running maximum and denominator of query head g.
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) { return fmaxf(v, dpp_f32<CTRL>(v)); }

template <int LANES>
__device__ __forceinline__ float block_max(float v) {
    if constexpr (LANES >= 2) v = dpp_max<0xB1>(v);
    if constexpr (LANES >= 4) v = dpp_max<0x4E>(v);
    if constexpr (LANES >= 8) v = dpp_max<0x141>(v);
    if constexpr (LANES >= 16) v = dpp_max<0x140>(v);
    return v;
}

__device__ __forceinline__ float from_lane(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(lane << 2, __float_as_int(v)));
}

// One stage of the reduce-scatter over a 16-lane row: partners (DPP pattern CTRL) differ in
// bit BIT of the lane number; each keeps the half of the values whose index has its own bit
// and adds the partner's copy of that half. With one value left the stage is a plain sum.
template <int CTRL, int BIT, int N>
__device__ __forceinline__ void scatter_stage(float (&w)[16], int r) {
    if constexpr (N > 1) {
        const bool upper = (r >> BIT) & 1;
#pragma unroll
        for (int k = 0; k < N / 2; k++) {
            const float mine = upper ? w[N / 2 + k] : w[k];
            const float theirs = upper ? w[k] : w[N / 2 + k];
            w[k] = mine + dpp_f32<CTRL>(theirs);
        }
    } else {
        w[0] += dpp_f32<CTRL>(w[0]);
    }
}

// The same step as attend_step for LPT >= 16, with less arithmetic: the G * U partial scores are
// reduce-scattered over the 16 lanes of a row (lane r ends with the total of pair r / R,
// R = 16 / (G * U)), every lane does the softmax arithmetic of its own pair only, and the
// weights come back to all lanes through the LDS crossbar. `first` is the position of u = 0.
template <typename T, int LPT, int G, int U>
__device__ __forceinline__ void attend_step_scatter(const float (&q)[G][Piece<T>::kDims], const Piece<T> (&kp)[U],
                                                    const Piece<T> (&vp)[U], uint32_t first, uint32_t stride,
                                                    uint32_t end, int lane, float& m, float& l,
                                                    float (&acc)[G][Piece<T>::kDims]) {
    constexpr int DPL = Piece<T>::kDims;
    constexpr int N = G * U;       // pairs (query head, position)
    constexpr int R = 16 / N;      // lanes holding the same pair
    constexpr int BLOCK = 16 / G;  // lanes of one query head
    static_assert(N <= 16 && LPT >= 16, "scatter step: at most 16 pairs over rows of 16 lanes");
    const int r = lane & 15;
    float w[16];
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            float part = 0.f;
#pragma unroll
            for (int d = 0; d < DPL; d++) part = fmaf(q[g][d], kp[u].get(d), part);
            if constexpr (LPT >= 32) part += from_lane(part, lane ^ 16);
            w[g * U + u] = part;
        }
    }
    scatter_stage<0x140, 3, N>(w, r);
    scatter_stage<0x141, 2, (N > 1 ? N / 2 : 1)>(w, r);
    scatter_stage<0x4E, 1, (N > 2 ? N / 4 : 1)>(w, r);
    scatter_stage<0xB1, 0, (N > 4 ? N / 8 : 1)>(w, r);
    const int u = (r / R) % U;
    const float score = first + u * stride < end ? w[0] : -INFINITY;
    const float top = fmaxf(m, block_max<BLOCK>(score));
    const float keep = __builtin_amdgcn_exp2f(m - top);
    const float p = __builtin_amdgcn_exp2f(score - top);
    float total = p;
    if constexpr (BLOCK >= 2) total += dpp_f32<0xB1>(total);
    if constexpr (BLOCK >= 4) total += dpp_f32<0x4E>(total);
    if constexpr (BLOCK >= 8) total += dpp_f32<0x141>(total);
    if constexpr (BLOCK >= 16) total += dpp_f32<0x140>(total);
    l = fmaf(l, keep, total * (1.0f / R));
    m = top;
    const int row = lane & ~15;
    if (__builtin_amdgcn_ballot_w64(keep != 1.0f) != 0) {  // some maximum moved: rescale the sums
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float factor = from_lane(keep, row + g * BLOCK);
#pragma unroll
            for (int d = 0; d < DPL; d++) acc[g][d] *= factor;
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int uu = 0; uu < U; uu++) {
            const float weight = from_lane(p, row + (g * U + uu) * R);
#pragma unroll
            for (int d = 0; d < DPL; d++) acc[g][d] = fmaf(weight, vp[uu].get(d), acc[g][d]);
        }
    }
}

// out[query, column] = sum_i w_i acc_i / sum_i w_i l_i with w_i = exp2(m_i - max m) over the
// partial records of the context splits.
__device__ __forceinline__ void merge_splits(const KvArgs& a, uint64_t query, uint32_t column) {
    const uint32_t stride = a.width + 2;
    const float* records = a.partial + query * a.splits * stride;
    float top = kLowest, total = 0.f, value = 0.f;
#pragma unroll 4
    for (uint32_t i = 0; i < a.splits; i++) {
        const float m = records[i * stride], l = records[i * stride + 1], part = records[i * stride + 2 + column];
        const float next = fmaxf(top, m);
        const float keep = __builtin_amdgcn_exp2f(top - next), weight = __builtin_amdgcn_exp2f(m - next);
        total = fmaf(total, keep, weight * l);
        value = fmaf(value, keep, weight * part);
        top = next;
    }
    a.out[query * a.width + column] = value / total;
}

// Streaming kernel. LPT lanes share one position (each holds Piece<T>::kDims of the width,
// width == LPT * kDims), so a wave covers 64 / LPT positions per load and the workgroup
// WAVES * 64 / LPT; U such loads are in flight per step. G query heads of one kv head are
// served from the same K / V registers. WAVES = 8 when the launch has enough rows of queries to give
// every compute unit a workgroup without splitting the context (no partial records, no merge
// launch), else 4.
// q of the workgroup's G heads, then k and v of its kv head, for one slot, from the K shares of the
// projection: the sums in share order, the bias, the rotary pairs of q and k - what
// reduce_group_rotary_kernel (gemm_h16.hip) stores. out: [(G + 2)][width] floats in LDS.
template <int G>
__device__ void project_rows(const KvArgs& a, uint32_t slot, uint32_t head0, uint32_t kv_head, float* out,
                             uint32_t threads) {
    const KvProjected& s = a.projected;
    const uint32_t width = a.width, half = width / 2;
    const uint64_t share_stride = s.launch_rows * s.vectors;
    const auto summed = [&](uint32_t first_row, const float* bias, uint32_t row) {
        const float* first = s.shares + static_cast<uint64_t>(slot) * s.launch_rows + first_row + row;
        float total = first[0];
        for (uint32_t k = 1; k < s.count; k++) total += first[k * share_stride];
        return bias != nullptr ? total + bias[row] : total;
    };
    const uint32_t offset = s.offsets_len == 1 ? s.offsets[0] : s.offsets[slot];
    const uint32_t rotated = (G + 1) * half;  // the pairs of the G query heads, then of the key head
    for (uint32_t item = threadIdx.x; item < rotated + width; item += threads) {
        if (item < rotated) {
            const uint32_t h = item / half, index = item - h * half;
            const uint32_t head = h < G ? head0 + h : kv_head;
            const uint32_t first_row = h < G ? s.q_row : s.k_row;
            const float* bias = h < G ? s.q_bias : s.k_bias;
            const uint32_t lo = s.interleaved ? 2u * index : index, hi = s.interleaved ? lo + 1u : lo + half;
            float value_lo = summed(first_row, bias, head * width + lo);
            float value_hi = summed(first_row, bias, head * width + hi);
            rotate_pair(value_lo, value_hi, offset, 0u, index, width, s.theta, s.sign, value_lo, value_hi);
            out[h * width + lo] = value_lo;
            out[h * width + hi] = value_hi;
        } else {
            const uint32_t d = item - rotated;
            out[(G + 1) * width + d] = summed(s.v_row, s.v_bias, kv_head * width + d);
        }
    }
}

// PROJECTED: q, k, v arrive as the K shares of their projections (KvArgs::projected, one token per slot).
template <typename T, int LPT, int G, int U, int WAVES, bool PROJECTED>
__global__ __launch_bounds__(64 * WAVES) void kv_attend_kernel(const KvArgs a) {
    constexpr int kWaves = WAVES;
    constexpr int kThreads = 64 * WAVES;
    constexpr int DPL = Piece<T>::kDims;
    constexpr int PPW = 64 / LPT;        // positions per wave per load
    constexpr int PPG = kWaves * PPW;    // per workgroup per load
    constexpr int GROUPS = kWaves * PPW; // independent softmax states in the workgroup
    __shared__ uint32_t rows_of_block[kKvTableEntries];
    __shared__ float merge_m[GROUPS][G];
    __shared__ float merge_l[GROUPS][G];
    __shared__ float merge_acc[GROUPS][G][LPT * DPL + 4];
    __shared__ __attribute__((aligned(16))) float projected[PROJECTED ? (G + 2) * LPT * DPL : 4];  // q of the G heads, k, v

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

    const Span s = slot_span(a, slot);
    if (token == 0 && kv_head == 0 && chunk == 0 && split == 0 && wave == 0) write_slot_status(a, slot, s, lane);
    uint32_t begin, end;
    query_range(a, s, token, begin, end);
    // This split's share, in whole steps.
    const uint32_t length = s.ok ? end - begin : 0;
    uint32_t share = (length + a.splits - 1) / a.splits;
    share = (share + PPG * U - 1) / (PPG * U) * (PPG * U);
    const uint32_t my_begin = min(begin + split * share, end);
    const uint32_t my_end = s.ok ? min(my_begin + share, end) : my_begin;
    // Positions below the cursor are cached rows; the others arrive with this call.
    const uint32_t cached_end = min(my_end, max(my_begin, s.cursor));

    // Physical first rows of the blocks this split touches.
    const uint32_t first_block = block_of(a, my_begin);
    if (my_end > my_begin) {
        const uint32_t blocks = block_of(a, my_end - 1) - first_block + 1;
        for (uint32_t i = threadIdx.x; i < blocks && i < kKvTableEntries; i += kThreads) {
            uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                         first_block + i]) * a.block_size;
            // a block outside the pool is reported by the slot's status; it is neither read nor written
            rows_of_block[i] = row >= a.max_tokens ? kNoBlock : static_cast<uint32_t>(row);
        }
    }
    constexpr bool from_shares = PROJECTED;
    if constexpr (from_shares) project_rows<G>(a, slot, head0, kv_head, projected, kThreads);
    __syncthreads();

    float q[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        if constexpr (from_shares) {
#pragma unroll
            for (int d = 0; d < DPL; d++) q[g][d] = projected[g * (LPT * DPL) + sub * DPL + d] * a.scale_log2;
        } else {
            const float* source = a.q + ((static_cast<uint64_t>(slot) * a.query_heads + head0 + g) * a.tokens + token) *
                                            a.width + sub * DPL;
#pragma unroll
            for (int d = 0; d < DPL; d++) q[g][d] = source[d] * a.scale_log2;
        }
    }
    // Softmax state: per query head in every lane (rows of 8 lanes), or spread over the 16 lanes of a
    // row, lane r holding head r / (16 / G) (see attend_step_scatter).
    constexpr bool kScatter = LPT >= 16;
    float m[G], l[G], acc[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = kLowest;
        l[g] = 0.f;
#pragma unroll
        for (int d = 0; d < DPL; d++) acc[g][d] = 0.f;
    }

    const uint64_t row_bytes = static_cast<uint64_t>(a.kv_heads) * a.width * Piece<T>::kElementBytes;
    const uint64_t lane_offset = (static_cast<uint64_t>(kv_head) * a.width + sub * DPL) * Piece<T>::kElementBytes;
    char* k_base = static_cast<char*>(a.k_slab) + lane_offset;
    char* v_base = static_cast<char*>(a.v_slab) + lane_offset;
    const auto row_of = [&](uint32_t position) {
        const uint32_t base = rows_of_block[min(block_of(a, position) - first_block, kKvTableEntries - 1u)];
        return base == kNoBlock ? 0u : min(base + within_block(a, position), a.max_tokens - 1);
    };

    if (cached_end > my_begin) {
        const auto fetch = [&](uint32_t step_begin, Piece<T> (&kp)[U], Piece<T> (&vp)[U]) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                // positions past the end read the last cached row again and are masked out below
                const uint32_t row = row_of(min(step_begin + u * PPG + group, cached_end - 1));
                kp[u].raw = load_streamed(reinterpret_cast<const typename Piece<T>::Raw*>(k_base + row * row_bytes));
                vp[u].raw = load_streamed(reinterpret_cast<const typename Piece<T>::Raw*>(v_base + row * row_bytes));
                if constexpr (Piece<T>::kScaled) {
                    kp[u].scale = a.k_scales[static_cast<uint64_t>(row) * a.kv_heads + kv_head];
                    vp[u].scale = a.v_scales[static_cast<uint64_t>(row) * a.kv_heads + kv_head];
                }
            }
        };
        const auto consume = [&](uint32_t step, const Piece<T> (&kp)[U], const Piece<T> (&vp)[U]) {
            if constexpr (kScatter) {
                attend_step_scatter<T, LPT, G, U>(q, kp, vp, step + group, PPG, cached_end, lane, m[0], l[0], acc);
            } else {
                bool live[U];
#pragma unroll
                for (int u = 0; u < U; u++) live[u] = step + u * PPG + group < cached_end;
                attend_step<T, LPT, G, U>(q, kp, vp, live, m, l, acc);
            }
        };
        // two register sets take turns: one is consumed while the other one's loads are in flight
        constexpr uint32_t kStep = PPG * U;
        Piece<T> ka[U], va[U], kb[U], vb[U];
        fetch(my_begin, ka, va);
        for (uint32_t step = my_begin; step < cached_end; step += 2 * kStep) {
            if (step + kStep < cached_end) fetch(step + kStep, kb, vb);
            consume(step, ka, va);
            if (step + kStep >= cached_end) break;
            if (step + 2 * kStep < cached_end) fetch(step + 2 * kStep, ka, va);
            consume(step + kStep, kb, vb);
        }
    }
    // The new positions of this split: from the inputs, as the slab will hold them. The workgroup
    // whose query token is the new position itself (chunk 0) appends the row to the slabs.
    for (uint32_t step = cached_end; step < my_end; step += PPG) {
        const uint32_t position = step + group;
        const bool live[1] = {position < my_end};
        const uint32_t arrival = min(position, my_end - 1) - s.cursor;
        const uint64_t source = ((static_cast<uint64_t>(slot) * a.kv_heads + kv_head) * a.tokens + arrival) *
                                    a.width + sub * DPL;
        Piece<T> kp[1], vp[1];
        if constexpr (from_shares) {
            kp[0].template from_input<LPT>(projected + G * (LPT * DPL) + sub * DPL);
            vp[0].template from_input<LPT>(projected + (G + 1) * (LPT * DPL) + sub * DPL);
        } else {
            kp[0].template from_input<LPT>(a.k + source);
            vp[0].template from_input<LPT>(a.v + source);
        }
        if (live[0] && arrival == token && chunk == 0) {
            const uint32_t base = rows_of_block[min(block_of(a, position) - first_block, kKvTableEntries - 1u)];
            const uint32_t row = base + within_block(a, position);
            if (base != kNoBlock && row < a.max_tokens) {
                *reinterpret_cast<typename Piece<T>::Raw*>(k_base + row * row_bytes) = kp[0].raw;
                *reinterpret_cast<typename Piece<T>::Raw*>(v_base + row * row_bytes) = vp[0].raw;
                if constexpr (Piece<T>::kScaled) {
                    if (sub == 0) {
                        a.k_scales[static_cast<uint64_t>(row) * a.kv_heads + kv_head] = kp[0].scale;
                        a.v_scales[static_cast<uint64_t>(row) * a.kv_heads + kv_head] = vp[0].scale;
                    }
                }
            }
        }
        if constexpr (kScatter)
            attend_step_scatter<T, LPT, G, 1>(q, kp, vp, position, PPG, my_end, lane, m[0], l[0], acc);
        else
            attend_step<T, LPT, G, 1>(q, kp, vp, live, m, l, acc);
    }

    // Combine the workgroup's softmax states.
#pragma unroll
    for (int g = 0; g < G; g++) {
        if constexpr (kScatter) {
            if (sub == g * (16 / G)) {
                merge_m[group][g] = m[0];
                merge_l[group][g] = l[0];
            }
        } else if (sub == 0) {
            merge_m[group][g] = m[g];
            merge_l[group][g] = l[g];
        }
#pragma unroll
        for (int d = 0; d < DPL; d++) merge_acc[group][g][sub * DPL + d] = acc[g][d];
    }
    __syncthreads();
    const uint32_t width = LPT * DPL;
    // The G heads of this workgroup are G * width neighbouring columns of the slot's row of activations
    // for the contraction that follows; where they are whole 256-column stages the rows' tiles are
    // quantised here, from the values just stored (a skipped slot: from what the destination holds).
    __shared__ __attribute__((aligned(16))) float row_part[G * width];
    const bool quantise = a.prepared != nullptr && (G * width) % 256 == 0;
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
            const float result = value / total;
            if (s.ok) a.out[query * width + column] = result;
            if (quantise) row_part[item] = s.ok ? result : a.out[query * width + column];
        } else {
            float* record = a.partial + (query * a.splits + split) * (width + 2);
            record[2 + column] = value;
            if (column == 0) {
                record[0] = top;
                record[1] = total;
            }
        }
    }
    if (quantise && a.splits == 1) {  // uniform: the launcher sets `prepared` only for one token per slot
        __syncthreads();
        const uint32_t wave = threadIdx.x >> 6, quad = threadIdx.x & 63u;
        if (wave < G * width / 256u) {
            const float4 in = *reinterpret_cast<const float4*>(&row_part[wave * 256u + 4u * quad]);
            quantize_halves_store(in, slot, (head0 * width) / 256u + wave, quad, a.vector_tiles, a.prepared);
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
    const uint32_t group_size = a.query_heads / a.kv_heads;
    const uint32_t kv_head = head / group_size;
    const int lane = threadIdx.x;

    const Span s = slot_span(a, slot);
    if (token == 0 && head == 0 && split == 0) write_slot_status(a, slot, s, lane);
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
    T* keys = static_cast<T*>(a.k_slab);
    T* values = static_cast<T*>(a.v_slab);
    for (uint32_t position = my_begin; position < my_end; position++) {
        uint64_t row = static_cast<uint64_t>(a.table[static_cast<uint64_t>(slot) * a.table_stride +
                                                     block_of(a, position)]) * a.block_size +
                       within_block(a, position);
        const bool inside = row < a.max_tokens;
        row = min(row, static_cast<uint64_t>(a.max_tokens - 1));
        const uint64_t at = (row * a.kv_heads + kv_head) * a.width;
        // A new position comes from the inputs, rounded as the slab stores it; the first query head
        // of the group whose token is that position appends it.
        const bool arriving = position >= s.cursor;
        const uint32_t arrival = arriving ? position - s.cursor : 0;
        const uint64_t source = ((static_cast<uint64_t>(slot) * a.kv_heads + kv_head) * a.tokens + arrival) * a.width;
        const bool appends = arriving && arrival == token && head % group_size == 0 && inside;
        float key[kKvAnyWidthPerLane], value[kKvAnyWidthPerLane];
        float part = 0.f;
        if constexpr (std::is_same<T, U8>::value) {
            // the row's scales: of the cached row, or what the write computes for the arriving one
            float k_scale, v_scale;
            if (arriving) {
                float k_top = 0.f, v_top = 0.f;
#pragma unroll
                for (int i = 0; i < kKvAnyWidthPerLane; i++) {
                    const uint32_t column = lane + 64 * i;
                    if (column < a.width) {
                        k_top = fmaxf(k_top, fabsf(a.k[source + column]));
                        v_top = fmaxf(v_top, fabsf(a.v[source + column]));
                    }
                }
                k_scale = u8_scale(group_max<64>(k_top));
                v_scale = u8_scale(group_max<64>(v_top));
                if (appends && lane == 0) {
                    a.k_scales[row * a.kv_heads + kv_head] = k_scale;
                    a.v_scales[row * a.kv_heads + kv_head] = v_scale;
                }
            } else {
                k_scale = a.k_scales[row * a.kv_heads + kv_head];
                v_scale = a.v_scales[row * a.kv_heads + kv_head];
            }
#pragma unroll
            for (int i = 0; i < kKvAnyWidthPerLane; i++) {
                const uint32_t column = lane + 64 * i;
                key[i] = value[i] = 0.f;
                if (column < a.width) {
                    uint32_t k_byte, v_byte;
                    if (arriving) {
                        k_byte = u8_byte(a.k[source + column], k_scale);
                        v_byte = u8_byte(a.v[source + column], v_scale);
                        if (appends) {
                            keys[at + column].byte = static_cast<uint8_t>(k_byte);
                            values[at + column].byte = static_cast<uint8_t>(v_byte);
                        }
                    } else {
                        k_byte = keys[at + column].byte;
                        v_byte = values[at + column].byte;
                    }
                    key[i] = u8_value(k_byte, k_scale);
                    value[i] = u8_value(v_byte, v_scale);
                    part = fmaf(q[i], key[i], part);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < kKvAnyWidthPerLane; i++) {
                const uint32_t column = lane + 64 * i;
                key[i] = value[i] = 0.f;
                if (column < a.width) {
                    if (arriving) {
                        key[i] = slab_round(keys, a.k[source + column]);
                        value[i] = slab_round(values, a.v[source + column]);
                        if (appends) {
                            slab_store(keys, at + column, a.k[source + column]);
                            slab_store(values, at + column, a.v[source + column]);
                        }
                    } else {
                        key[i] = slab_load(keys, at + column);
                        value[i] = slab_load(values, at + column);
                    }
                    part = fmaf(q[i], key[i], part);
                }
            }
        }
        const float score = group_sum<64>(part);
        const float top = fmaxf(m, score);
        const float keep = __builtin_amdgcn_exp2f(m - top), p = __builtin_amdgcn_exp2f(score - top);
        m = top;
        l = fmaf(l, keep, p);
#pragma unroll
        for (int i = 0; i < kKvAnyWidthPerLane; i++) acc[i] = fmaf(p, value[i], acc[i] * keep);
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

// Combines the partial records of the context splits: a workgroup per query row, a thread per column.
__global__ void kv_merge_kernel(const KvArgs a) {
    const uint64_t query = blockIdx.x;
    const uint32_t slot = static_cast<uint32_t>(query / (static_cast<uint64_t>(a.query_heads) * a.tokens));
    if (!slot_span(a, slot).ok) return;
    for (uint32_t column = threadIdx.x; column < a.width; column += blockDim.x) merge_splits(a, query, column);
}

template <typename T, int LPT, int G>
hipError_t launch_streaming(const KvArgs& a, uint32_t workgroups, int waves, hipStream_t stream) {
    constexpr int U = G >= 8 ? 2 : 4;
    if (a.projected.shares != nullptr) {
        if (waves == 8)
            hipLaunchKernelGGL((kv_attend_kernel<T, LPT, G, U, 8, true>), dim3(workgroups), dim3(512), 0, stream, a);
        else
            hipLaunchKernelGGL((kv_attend_kernel<T, LPT, G, U, 4, true>), dim3(workgroups), dim3(256), 0, stream, a);
    } else if (waves == 8) {
        hipLaunchKernelGGL((kv_attend_kernel<T, LPT, G, U, 8, false>), dim3(workgroups), dim3(512), 0, stream, a);
    } else {
        hipLaunchKernelGGL((kv_attend_kernel<T, LPT, G, U, 4, false>), dim3(workgroups), dim3(256), 0, stream, a);
    }
    return hipGetLastError();
}

template <typename T, int LPT>
hipError_t launch_streaming_group(const KvArgs& a, int g, uint32_t workgroups, int waves, hipStream_t stream) {
    switch (g) {
        case 8: return launch_streaming<T, LPT, 8>(a, workgroups, waves, stream);
        case 4: return launch_streaming<T, LPT, 4>(a, workgroups, waves, stream);
        case 2: return launch_streaming<T, LPT, 2>(a, workgroups, waves, stream);
        default: return launch_streaming<T, LPT, 1>(a, workgroups, waves, stream);
    }
}

template <typename T>
hipError_t launch_streaming_width(const KvArgs& a, int g, uint32_t workgroups, int waves, hipStream_t stream) {
    switch (a.width / Piece<T>::kDims) {
        case 32: return launch_streaming_group<T, 32>(a, g, workgroups, waves, stream);
        case 16: return launch_streaming_group<T, 16>(a, g, workgroups, waves, stream);
        default: return launch_streaming_group<T, 8>(a, g, workgroups, waves, stream);
    }
}

// Query heads of one kv head served together by the streaming kernel; 0 = not covered.
// Elements of a slab row one lane takes (sixteen bytes; eight for the u8 tier).
uint32_t piece_dims(const KvAttention& p) { return p.slab_dtype == ET_DTYPE_F32 ? 4 : 8; }

int streaming_group(const KvAttention& p) {
    const uint32_t dims = piece_dims(p);
    if (p.width % dims != 0) return 0;
    const uint32_t lanes = p.width / dims;
    if (lanes != 8 && lanes != 16 && lanes != 32) return 0;
    const uint32_t group = p.query_heads / p.kv_heads;
    for (int g : {8, 4, 2})
        if (group % g == 0) return g;
    return 1;
}

uint32_t positions_per_step(const KvAttention& p, int g, int waves) {
    const uint32_t lanes = p.width / piece_dims(p);
    return waves * (64 / lanes) * (g >= 8 ? 2 : 4);
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
    // A compute unit keeps eight waves of the streaming kernel resident: two workgroups of four, or
    // one of eight. With all workgroups resident at once none waits for a second round (measured for 32
    // slots x 8 kv heads at context 2048: 512 x 4 waves 58.9 us, 1024 x 4 waves 63.7, 256 x 8 waves
    // without any split - no partial records, no merge launch - 55.6). Eight waves need enough rows
    // of queries to go round without splitting.
    shape.waves = shape.streaming && rows >= 128 ? 8 : 4;
    const uint64_t step = shape.streaming ? positions_per_step(p, g, shape.waves) : 64;
    uint64_t splits = 1;
    const uint64_t wanted = shape.streaming ? (shape.waves == 8 ? 256 : 512) : 4096;
    if (rows < wanted) splits = shape.streaming ? wanted / (rows == 0 ? 1 : rows)
                                                : (wanted + rows - 1) / (rows == 0 ? 1 : rows);
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

hipError_t kv_attention(const KvAttention& p, void* workspace, hipStream_t stream) {
    KvArgs a{};
    a.k_slab = p.k_slab;
    a.v_slab = p.v_slab;
    a.k_scales = p.k_scales;
    a.v_scales = p.v_scales;
    a.table = p.block_table;
    a.cursors = p.cursors;
    a.advances = p.advances;
    a.q = p.q;
    a.k = p.k;
    a.v = p.v;
    a.out = p.out;
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
    a.partial = static_cast<float*>(workspace);
    // The streaming kernel quantises the rows itself when it writes them in one piece (no context
    // splits), every slot is active and its heads are whole stages; else a quantiser launch follows.
    const bool fused_tiles = p.prepared != nullptr && p.tokens == 1 && shape.streaming && shape.splits == 1 &&
                             p.active_batch == p.batch &&
                             (static_cast<uint64_t>(streaming_group(p)) * p.width) % 256 == 0;
    a.prepared = fused_tiles ? p.prepared : nullptr;
    a.vector_tiles = (p.batch + 31u) / 32u;
    a.projected = p.projected;
    if (p.projected.shares != nullptr && !(shape.streaming && p.tokens == 1)) return hipErrorInvalidValue;
    const auto finish = [&](hipError_t error) -> hipError_t {
        if (error != hipSuccess || p.prepared == nullptr || fused_tiles || p.batch == 0) return error;
        const uint64_t columns = static_cast<uint64_t>(p.query_heads) * p.width;
        return quantize_tiles(p.out, columns, p.batch, columns, 2, p.prepared, stream);
    };

    // out.fill(0.0) for the slots that are not active (napi/mod.rs:3371); their status words too.
    const uint64_t per_slot = static_cast<uint64_t>(p.query_heads) * p.tokens * p.width;
    if (p.active_batch < p.batch) {
        const uint64_t count = (p.batch - p.active_batch) * per_slot;
        hipLaunchKernelGGL(kv_zero_kernel, dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, stream,
                           p.out + p.active_batch * per_slot, count, a.status + p.active_batch,
                           p.batch - p.active_batch);
    }
    if (p.active_batch == 0) return finish(hipGetLastError());

    hipError_t error;
    if (shape.streaming) {
        const int g = streaming_group(p);
        const uint32_t workgroups = static_cast<uint32_t>(shape.workgroups);
        switch (p.slab_dtype) {
            case ET_DTYPE_F16: error = launch_streaming_width<__half>(a, g, workgroups, shape.waves, stream); break;
            case ET_DTYPE_BF16: error = launch_streaming_width<Bf16>(a, g, workgroups, shape.waves, stream); break;
            case ET_DTYPE_U8: error = launch_streaming_width<U8>(a, g, workgroups, shape.waves, stream); break;
            default: error = launch_streaming_width<float>(a, g, workgroups, shape.waves, stream); break;
        }
    } else {
        const dim3 grid(static_cast<uint32_t>(shape.workgroups));
        switch (p.slab_dtype) {
            case ET_DTYPE_F16: hipLaunchKernelGGL(kv_attend_any_kernel<__half>, grid, dim3(64), 0, stream, a); break;
            case ET_DTYPE_BF16: hipLaunchKernelGGL(kv_attend_any_kernel<Bf16>, grid, dim3(64), 0, stream, a); break;
            case ET_DTYPE_U8: hipLaunchKernelGGL(kv_attend_any_kernel<U8>, grid, dim3(64), 0, stream, a); break;
            default: hipLaunchKernelGGL(kv_attend_any_kernel<float>, grid, dim3(64), 0, stream, a); break;
        }
        error = hipGetLastError();
    }
    if (error != hipSuccess) return error;
    if (shape.splits > 1) {
        const uint64_t queries = static_cast<uint64_t>(p.active_batch) * p.query_heads * p.tokens;
        const uint32_t threads = p.width > 128 ? 256 : p.width > 64 ? 128 : 64;
        hipLaunchKernelGGL(kv_merge_kernel, dim3(static_cast<uint32_t>(queries)), dim3(threads), 0, stream, a);
        error = hipGetLastError();
    }
    return finish(error);
}

}  // namespace et
