// Activation-stationary dequant-GEMV for gfx950 (Q4_K, Q4_0, Q8_0):
//     y[v, r] = sum_k x[v, k] * decode(W[r])[k] (+ bias[r]),   1 <= v <= 4 per launch.
//
// Computes what linear_into (crates/runtime-cpu/src/quantized.rs:419-499)
// computes, with f32 accumulation but in factored form (block scales applied to
// per-lane partial sums), so results agree with the scalar loop within 1e-3,
// not bit for bit. Q4_K follows decode_q4_k (:180-199):
//     y = sum_blocks d * sum_g sc_g * (sum_i q_gi x_gi) - dmin * sum_g m_g * (sum_i x_gi).
// Q4_0 / Q8_0 follow the public ggml block layouts (not in the reference).
//
// The kernel is HBM-bound on the packed weights (0.56 - 1.06 bytes per weight
// against 2 flops), so the design minimises everything that is not a weight
// byte: each lane owns a fixed stretch of XW columns of the activation vector,
// loads it ONCE into registers (staged through LDS so the global reads are
// coalesced), and then streams weight rows past it with 16-byte loads. A wave
// covers 64*XW columns of a row; NK waves cover the whole row and combine their
// partial sums in LDS. Rows are dealt to workgroups in contiguous ranges so that
// each workgroup walks HBM sequentially.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "et_codecs.h"
#include "gemv_common.h"
#include "kernels.h"

namespace et {
namespace {

// ---------------------------------------------------------------------------
// Codec traits. Each describes what one lane owns and how it folds one row's
// bytes into per-vector partial sums.
//   XW            activation floats a lane owns per vector
//   Lane          lane-constant geometry
//   Data          the bytes a lane loads per row
//   x_quad(l, j)  index (within the wave's slice, in float4s) of the j-th float4
//                 the lane owns
// ---------------------------------------------------------------------------

// Unpacks the (scale, min) of sub-blocks 2p and 2p+1 from the 12 scale bytes of
// a Q4_K block (crates/runtime-cpu/src/quantized.rs:77-86), for a lane-constant p.
__device__ __forceinline__ void q4k_pair_scales(const uint4& header, uint32_t p, float& sc_lo,
                                                float& sc_hi, float& m_lo, float& m_hi) {
    const uint32_t shift = (p & 1u) * 16u;
    const uint32_t a = header.y >> shift;  // scales[0..3], bytes 2(p&1) and 2(p&1)+1
    const uint32_t b = header.z >> shift;  // scales[4..7]
    const uint32_t c = header.w >> shift;  // scales[8..11]
    uint32_t sc, mn;
    if (p < 2) {
        sc = a & 0x3f3fu;
        mn = b & 0x3f3fu;
    } else {
        sc = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        mn = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
    }
    sc_lo = static_cast<float>(sc & 0xffu);
    sc_hi = static_cast<float>((sc >> 8) & 0xffu);
    m_lo = static_cast<float>(mn & 0xffu);
    m_hi = static_cast<float>((mn >> 8) & 0xffu);
}

// One dword of 4-bit quants: its 4 low nibbles meet x[lo_base + t], its 4 high
// nibbles x[hi_base + t].
template <int M, int XW>
__device__ __forceinline__ void nibble_dot(uint32_t w, const float (&x)[M][XW], int lo_base,
                                           int hi_base, float (&s_lo)[M], float (&s_hi)[M]) {
    uint32_t lo = w & 0x0f0f0f0fu;
    uint32_t hi = (w >> 4) & 0x0f0f0f0fu;
    // Keep the two masked dwords opaque: each byte then converts with a single
    // v_cvt_f32_ubyteN instead of a bit-field extract plus a convert.
    asm("" : "+v"(lo));
    asm("" : "+v"(hi));
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const float ql = static_cast<float>((lo >> (8 * t)) & 0xffu);
        const float qh = static_cast<float>((hi >> (8 * t)) & 0xffu);
#pragma unroll
        for (int m = 0; m < M; m++) {
            s_lo[m] = fmaf(ql, x[m][lo_base + t], s_lo[m]);
            s_hi[m] = fmaf(qh, x[m][hi_base + t], s_hi[m]);
        }
    }
}

// Q4_K. FULL: a lane owns one 32-byte pair of a super-block = 64 columns (32 low
// nibbles = sub-block 2p, 32 high nibbles = sub-block 2p+1). HALF: 16 of those
// bytes = 16 + 16 columns, to halve the registers per vector.
template <bool HALF>
struct Q4KTraits {
    static constexpr int XW = HALF ? 32 : 64;
    struct Lane {
        uint32_t offset;  // byte offset of the lane's block within a row
        uint32_t piece;   // first 16-byte piece of qs the lane owns (0..7)
        uint32_t p;       // pair within the block
    };
    struct Data {
        uint4 header;
        uint4 q[HALF ? 1 : 2];
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 8) * 144u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) {
        Lane lane;
        const uint32_t block = HALF ? chunk >> 3 : chunk >> 2;
        lane.piece = HALF ? (chunk & 7u) : ((chunk & 3u) * 2u);
        lane.p = lane.piece >> 1;
        lane.offset = block * 144u;
        return lane;
    }
    static __device__ __forceinline__ uint32_t x_quad(uint32_t l, int j) {
        // FULL: 16 consecutive float4s. HALF: two runs of 4 float4s, 8 float4s apart.
        return HALF ? (8u * l - 4u * (l & 1u) + (j & 3) + 8u * (j >> 2)) : (16u * l + j);
    }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        const uint8_t* base = row + lane.offset;
        data.header = *reinterpret_cast<const uint4*>(base);
        data.q[0] = *reinterpret_cast<const uint4*>(base + 16 + 16 * lane.piece);
        if (!HALF) data.q[HALF ? 0 : 1] = *reinterpret_cast<const uint4*>(base + 32 + 16 * lane.piece);
    }
    // Lane-constant sums of the owned activations: [0] low run, [1] high run.
    template <int M>
    static __device__ __forceinline__ void x_sums(const float (&x)[M][XW], float (&sums)[M][2]) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            float lo = 0.f, hi = 0.f;
#pragma unroll
            for (int i = 0; i < XW / 2; i++) {
                lo += x[m][i];
                hi += x[m][XW / 2 + i];
            }
            sums[m][0] = lo;
            sums[m][1] = hi;
        }
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane& lane,
                                                const float (&x)[M][XW], const float (&sums)[M][2],
                                                float (&value)[M]) {
        float s_lo[M], s_hi[M];
#pragma unroll
        for (int m = 0; m < M; m++) s_lo[m] = s_hi[m] = 0.f;
#pragma unroll
        for (int u = 0; u < (HALF ? 1 : 2); u++) {
            nibble_dot<M, XW>(data.q[u].x, x, 16 * u + 0, XW / 2 + 16 * u + 0, s_lo, s_hi);
            nibble_dot<M, XW>(data.q[u].y, x, 16 * u + 4, XW / 2 + 16 * u + 4, s_lo, s_hi);
            nibble_dot<M, XW>(data.q[u].z, x, 16 * u + 8, XW / 2 + 16 * u + 8, s_lo, s_hi);
            nibble_dot<M, XW>(data.q[u].w, x, 16 * u + 12, XW / 2 + 16 * u + 12, s_lo, s_hi);
        }
        float sc_lo, sc_hi, m_lo, m_hi;
        q4k_pair_scales(data.header, lane.p, sc_lo, sc_hi, m_lo, m_hi);
        const float d = half_bits_to_float(data.header.x & 0xffffu);
        const float dmin = half_bits_to_float(data.header.x >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float pos = sc_lo * s_lo[m] + sc_hi * s_hi[m];
            const float neg = m_lo * sums[m][0] + m_hi * sums[m][1];
            value[m] = d * pos - dmin * neg;
        }
    }
};

struct __attribute__((packed, aligned(4))) Dwords9 {
    uint32_t v[9];
};
struct __attribute__((packed, aligned(4))) Dwords17 {
    uint32_t v[17];
};

// Q4_0: a lane owns two consecutive 18-byte blocks = 36 bytes = 64 columns. The
// pair is dword aligned (rows are a multiple of 36 bytes when columns % 64 == 0);
// the first block's quants sit 2 bytes off dword alignment and are realigned
// with funnel shifts. value = d * (nibble - 8): the -8 is applied to the lane's
// activation sum once, not per weight.
struct Q40Traits {
    static constexpr int XW = 64;
    struct Lane {
        uint32_t offset;
    };
    struct Data {
        Dwords9 raw;
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 5) * 18u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) { return Lane{chunk * 36u}; }
    static __device__ __forceinline__ uint32_t x_quad(uint32_t l, int j) { return 16u * l + j; }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        data.raw = *reinterpret_cast<const Dwords9*>(row + lane.offset);
    }
    template <int M>
    static __device__ __forceinline__ void x_sums(const float (&x)[M][XW], float (&sums)[M][2]) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            float a = 0.f, b = 0.f;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                a += x[m][i];
                b += x[m][32 + i];
            }
            sums[m][0] = a;
            sums[m][1] = b;
        }
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane&,
                                                const float (&x)[M][XW], const float (&sums)[M][2],
                                                float (&value)[M]) {
        const uint32_t* w = data.raw.v;
        float s_a[M], s_b[M];
#pragma unroll
        for (int m = 0; m < M; m++) s_a[m] = s_b[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // block A: bytes 2..17 of the pair; element j = low nibble of byte j, j+16 = high.
            const uint32_t qa = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
            nibble_dot<M, XW>(qa, x, 4 * i, 16 + 4 * i, s_a, s_a);
            // block B: bytes 20..35, dword aligned.
            nibble_dot<M, XW>(w[5 + i], x, 32 + 4 * i, 48 + 4 * i, s_b, s_b);
        }
        const float da = half_bits_to_float(w[0] & 0xffffu);
        const float db = half_bits_to_float(w[4] >> 16);
#pragma unroll
        for (int m = 0; m < M; m++)
            value[m] = da * (s_a[m] - 8.f * sums[m][0]) + db * (s_b[m] - 8.f * sums[m][1]);
    }
};

// Q8_0: a lane owns two consecutive 34-byte blocks = 68 bytes = 64 columns
// (dword aligned when columns % 64 == 0).
struct Q80Traits {
    static constexpr int XW = 64;
    struct Lane {
        uint32_t offset;
    };
    struct Data {
        Dwords17 raw;
    };
    static __device__ __forceinline__ uint64_t row_bytes(uint32_t columns) {
        return static_cast<uint64_t>(columns >> 5) * 34u;
    }
    static __device__ __forceinline__ Lane lane_setup(uint32_t chunk) { return Lane{chunk * 68u}; }
    static __device__ __forceinline__ uint32_t x_quad(uint32_t l, int j) { return 16u * l + j; }
    static __device__ __forceinline__ void load(const uint8_t* row, const Lane& lane, Data& data) {
        data.raw = *reinterpret_cast<const Dwords17*>(row + lane.offset);
    }
    template <int M>
    static __device__ __forceinline__ void x_sums(const float (&)[M][XW], float (&)[M][2]) {}
    template <int M>
    static __device__ __forceinline__ void byte_dot(uint32_t w, const float (&x)[M][XW], int base,
                                                    float (&s)[M]) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const float q = static_cast<float>(static_cast<int>(static_cast<int8_t>(w >> (8 * t))));
#pragma unroll
            for (int m = 0; m < M; m++) s[m] = fmaf(q, x[m][base + t], s[m]);
        }
    }
    template <int M>
    static __device__ __forceinline__ void fold(const Data& data, const Lane&,
                                                const float (&x)[M][XW], const float (&)[M][2],
                                                float (&value)[M]) {
        const uint32_t* w = data.raw.v;
        float s_a[M], s_b[M];
#pragma unroll
        for (int m = 0; m < M; m++) s_a[m] = s_b[m] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t qa = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);  // bytes 2..33
            byte_dot<M>(qa, x, 4 * i, s_a);
            byte_dot<M>(w[9 + i], x, 32 + 4 * i, s_b);  // bytes 36..67
        }
        const float da = half_bits_to_float(w[0] & 0xffffu);
        const float db = half_bits_to_float(w[8] >> 16);
#pragma unroll
        for (int m = 0; m < M; m++) value[m] = da * s_a[m] + db * s_b[m];
    }
};

// ---------------------------------------------------------------------------
// The kernel. M vectors, R rows per wave iteration, WAVES waves per workgroup,
// NK waves per row (so WAVES / NK row groups per workgroup).
// ---------------------------------------------------------------------------
template <class T, int M, int R, int WAVES, int NK>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(
    const uint8_t* __restrict__ weight, const float* __restrict__ x, uint64_t x_row_stride,
    const float* __restrict__ bias, float* __restrict__ y, uint32_t rows, uint32_t columns,
    uint32_t rows_per_wg) {
    constexpr int RG = WAVES / NK;
    constexpr int XW = T::XW;
    constexpr uint32_t SLICE_QUADS = 64u * XW / 4u;  // float4s of one wave-wide slice
    __shared__ float4 x_stage[M * SLICE_QUADS];
    __shared__ float partial[2][RG][NK][R][M];
    const uint32_t lane_id = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t slice = wave % NK;
    const uint32_t group = wave / NK;

    const uint32_t chunk = slice * 64u + lane_id;  // which XW-column stretch of the row
    const bool active = chunk < columns / XW;
    const typename T::Lane lane = T::lane_setup(active ? chunk : 0u);
    const uint64_t row_bytes = T::row_bytes(columns);

    const uint32_t wg_row0 = blockIdx.x * rows_per_wg;
    const uint32_t wg_row_end = min(wg_row0 + rows_per_wg, rows);
    const uint32_t iterations = (wg_row_end - wg_row0 + RG * R - 1) / (RG * R);

    auto load_rows = [&](uint32_t it, typename T::Data (&data)[R]) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t row = wg_row0 + (it * RG + group) * R + r;
            row = min(row, rows - 1);  // rows past the end re-read a valid row and are discarded
            T::load(weight + row * row_bytes, lane, data[r]);
        }
    };

    // Start the first weight loads before touching the activations.
    typename T::Data current[R];
    load_rows(0, current);

    // Activations: global -> LDS (coalesced, swizzled) -> registers, one slice at a time.
    float xr[M][XW];
    for (uint32_t s = 0; s < NK; s++) {
        const uint32_t first_quad = s * SLICE_QUADS;
        const uint32_t all_quads = columns >> 2;
        const uint32_t quads = min(SLICE_QUADS, all_quads - min(all_quads, first_quad));
        if (s != 0) __syncthreads();
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float4* src = reinterpret_cast<const float4*>(x + m * x_row_stride) + first_quad;
            for (uint32_t f = threadIdx.x; f < quads; f += 64 * WAVES)
                x_stage[m * SLICE_QUADS + x_slot(f)] = src[f];
        }
        __syncthreads();
        if (s == slice) {
#pragma unroll
            for (int m = 0; m < M; m++) {
#pragma unroll
                for (int j = 0; j < XW / 4; j++) {
                    const float4 v = active ? x_stage[m * SLICE_QUADS + x_slot(T::x_quad(lane_id, j))]
                                            : make_float4(0.f, 0.f, 0.f, 0.f);
                    xr[m][4 * j + 0] = v.x;
                    xr[m][4 * j + 1] = v.y;
                    xr[m][4 * j + 2] = v.z;
                    xr[m][4 * j + 3] = v.w;
                }
            }
        }
    }
    float sums[M][2];
    T::template x_sums<M>(xr, sums);

    // Folds the rows held in `data` (iteration `it`) and writes their outputs.
    auto process = [&](uint32_t it, const typename T::Data (&data)[R]) {
        float total[R][M];
#pragma unroll
        for (int r = 0; r < R; r++) {
            float value[M];
            T::template fold<M>(data[r], lane, xr, sums, value);
#pragma unroll
            for (int m = 0; m < M; m++) total[r][m] = wave_sum(active ? value[m] : 0.f);
        }
        const uint32_t row0 = wg_row0 + (it * RG + group) * R;
        if (NK == 1) {
            if (lane_id == 0) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const uint32_t row = row0 + r;
                    if (row < wg_row_end) {
                        const float b = bias != nullptr ? bias[row] : 0.f;
#pragma unroll
                        for (int m = 0; m < M; m++)
                            y[static_cast<uint64_t>(m) * rows + row] =
                                bias != nullptr ? total[r][m] + b : total[r][m];
                    }
                }
            }
        } else {
            const uint32_t parity = it & 1u;
            if (lane_id == 0) {
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int m = 0; m < M; m++) partial[parity][group][slice][r][m] = total[r][m];
            }
            __syncthreads();
            if (slice == 0 && lane_id < R * M) {
                const uint32_t r = lane_id / M, m = lane_id - r * M;
                const uint32_t row = row0 + r;
                if (row < wg_row_end) {
                    float value = 0.f;
                    for (int s = 0; s < NK; s++) value += partial[parity][group][s][r][m];
                    if (bias != nullptr) value += bias[row];
                    y[static_cast<uint64_t>(m) * rows + row] = value;
                }
            }
        }
    };

    // Two row buffers in ping-pong: the loads of iteration it+1 are in flight
    // while iteration it is folded.
    typename T::Data other[R];
    for (uint32_t it = 0; it < iterations; it += 2) {
        if (it + 1 < iterations) load_rows(it + 1, other);
        process(it, current);
        if (it + 1 < iterations) {
            if (it + 2 < iterations) load_rows(it + 2, current);
            process(it + 1, other);
        }
    }
}

template <class T, int M, int R, int WAVES, int NK>
hipError_t launch(const uint8_t* weight, const float* x, uint64_t x_row_stride, const float* bias,
                  float* y, uint32_t rows, uint32_t columns, hipStream_t stream, uint32_t rpw = 0) {
    constexpr int RG = WAVES / NK;
    // One contiguous range of rows per CU, rounded to whole iterations.
    uint32_t rows_per_wg = rpw ? rpw : (rows + 255u) / 256u;
    rows_per_wg = ((rows_per_wg + RG * R - 1) / (RG * R)) * (RG * R);
    const uint32_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL((gemv_kernel<T, M, R, WAVES, NK>), dim3(grid), dim3(64 * WAVES), 0, stream,
                       weight, x, x_row_stride, bias, y, rows, columns, rows_per_wg);
    return hipGetLastError();
}

template <class T, int M, int R>
hipError_t launch_slices(const uint8_t* weight, const float* x, uint64_t x_row_stride,
                         const float* bias, float* y, uint32_t rows, uint32_t columns,
                         hipStream_t stream) {
    const uint32_t slice_columns = 64u * T::XW;
    const uint32_t slices = (columns + slice_columns - 1) / slice_columns;
    if (slices <= 1) return launch<T, M, R, 4, 1>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (slices <= 2) return launch<T, M, R, 4, 2>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (slices <= 4) return launch<T, M, R, 4, 4>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    if (slices <= 8) return launch<T, M, R, 8, 8>(weight, x, x_row_stride, bias, y, rows, columns, stream);
    return launch<T, M, R, 16, 16>(weight, x, x_row_stride, bias, y, rows, columns, stream);
}

}  // namespace

uint32_t gemv_fast_max_vectors(int32_t codec) { return codec == kQ4_K ? 4u : 2u; }

bool gemv_fast_supported(int32_t codec, uint64_t columns, uint32_t vectors) {
    if (vectors == 0 || vectors > gemv_fast_max_vectors(codec)) return false;
    switch (codec) {
        case kQ4_K:
            // 16 waves x (4096 | 2048) columns per launch
            return columns % 256 == 0 && columns <= (vectors <= 2 ? 65536u : 32768u);
        case kQ4_0:
        case kQ8_0:
            return columns % 64 == 0 && columns <= 65536u;
        default:
            return false;
    }
}

hipError_t gemv_fast(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                     const float* bias, float* y, uint64_t rows, uint64_t columns, uint32_t vectors,
                     hipStream_t stream) {
    const uint32_t n = static_cast<uint32_t>(rows), k = static_cast<uint32_t>(columns);
    if (codec == kQ4_K && vectors == 1 && k <= 4096 && getenv("ET_EXP")) {  // EXPERIMENT HOOK
        int w = 4, r = 2, rpw = 0;
        sscanf(getenv("ET_EXP"), "%d,%d,%d", &w, &r, &rpw);
        using T = Q4KTraits<false>;
        if (w == 4 && r == 2) return launch<T, 1, 2, 4, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 4 && r == 1) return launch<T, 1, 1, 4, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 4 && r == 4) return launch<T, 1, 4, 4, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 8 && r == 2) return launch<T, 1, 2, 8, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 8 && r == 1) return launch<T, 1, 1, 8, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 8 && r == 4) return launch<T, 1, 4, 8, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 16 && r == 1) return launch<T, 1, 1, 16, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 12 && r == 1) return launch<T, 1, 1, 12, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        if (w == 12 && r == 2) return launch<T, 1, 2, 12, 1>(weight, x, x_row_stride, bias, y, n, k, stream, rpw);
        return hipErrorInvalidValue;
    }
    if (codec == kQ4_K) {
        switch (vectors) {
            case 1: return launch_slices<Q4KTraits<false>, 1, 2>(weight, x, x_row_stride, bias, y, n, k, stream);
            case 2: return launch_slices<Q4KTraits<false>, 2, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            case 3: return launch_slices<Q4KTraits<true>, 3, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            case 4: return launch_slices<Q4KTraits<true>, 4, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            default: return hipErrorInvalidValue;
        }
    }
    if (codec == kQ4_0) {
        switch (vectors) {
            case 1: return launch_slices<Q40Traits, 1, 2>(weight, x, x_row_stride, bias, y, n, k, stream);
            case 2: return launch_slices<Q40Traits, 2, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            default: return hipErrorInvalidValue;
        }
    }
    if (codec == kQ8_0) {
        switch (vectors) {
            case 1: return launch_slices<Q80Traits, 1, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            case 2: return launch_slices<Q80Traits, 2, 1>(weight, x, x_row_stride, bias, y, n, k, stream);
            default: return hipErrorInvalidValue;
        }
    }
    return hipErrorInvalidValue;
}

}  // namespace et
