// Launchers of the gfx950 kernels. Host-callable; every function enqueues on
// `stream` and returns the launch status without synchronising.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>

namespace et {

constexpr int kMaxRank = 8;

// Strided view of an index (or input) tensor, passed to kernels by value.
struct IndexLayout {
    int32_t rank;
    int32_t contiguous;
    uint64_t offset;
    uint64_t shape[kMaxRank];
    uint64_t strides[kMaxRank];
};

// ---- dequant.hip -----------------------------------------------------------
// out[p, :] = decode(W[index[p], :]); indexes == nullptr decodes rows 0..out_rows.
hipError_t dequantize_rows(int32_t codec, const uint8_t* weight, const void* indexes,
                           int index_is_i64, const IndexLayout& layout, uint64_t out_rows,
                           uint64_t table_rows, uint64_t columns, float* out, void* status,
                           hipStream_t stream);

// ---- gemv_generic.hip (gather) ------------------------------------------------
// dst[i] = src[source_index(layout, i)] for i < count (f32): densifies a
// strided activation view into the workspace.
hipError_t gather_f32(const float* src, const IndexLayout& layout, uint64_t count, float* dst,
                      hipStream_t stream);

// ---- gemv_limb.hip: dequant-GEMV on v_dot4_i32_i8 over 3-limb activations -----
// y[v, r] = sum_k x[v, k] * decode(W[r])[k] (+ bias[r]) for v < vectors; f32-accurate.
// x rows must be 16-byte aligned (x pointer and x_row_stride * 4).
constexpr uint32_t kGemvLimbMaxVectors = 3;
uint32_t gemv_limb_max_vectors(int32_t codec);  // per launch: 3, or 2 for Q6_K
bool gemv_limb_supported(int32_t codec, uint64_t columns, uint32_t vectors);
// whether that launch takes its weights through LDS copies issued by loader waves
// (gemv_limb_turns_kernel, or gemv_limb_dma_kernel for the 2-bit codec)
bool gemv_limb_copies_through_lds(int32_t codec, uint64_t rows, uint64_t columns, uint32_t vectors);
hipError_t gemv_limb(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                     const float* bias, float* y, uint64_t rows, uint64_t columns, uint32_t vectors,
                     hipStream_t stream);

// ---- gemv_mma.hip: dequant-GEMV for 2..8 vectors on v_mfma_i32_16x16x32_i8 (Q4_K, Q5_K, Q4_0, Q8_0) ----
// W is streamed once through LDS whatever the number of vectors; f32-accurate like gemv_limb.
// x rows must be 16-byte aligned (x pointer and x_row_stride * 4).
constexpr uint32_t kGemvMmaMaxVectors = 8;
bool gemv_mma_supported(int32_t codec, uint64_t rows, uint64_t columns, uint32_t vectors);
hipError_t gemv_mma(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                    const float* bias, float* y, uint64_t rows, uint64_t columns, uint32_t vectors,
                    hipStream_t stream);

// ---- gemv_generic.hip: every codec, any whole number of blocks, vectors <= 4 ----
constexpr uint32_t kGemvGenericMaxVectors = 4;
hipError_t gemv_generic(int32_t codec, const uint8_t* weight, const float* x, uint64_t x_row_stride,
                        const float* bias, float* y, uint64_t rows, uint64_t columns,
                        uint32_t vectors, hipStream_t stream);

// ---- quantize_act.hip --------------------------------------------------------
// Public layout: q [vectors, columns] int8, scale = max|x| / 127 per vector and 32 columns,
// scale and sum (int32 block sums, may be null) TRANSPOSED: [columns/32, round_up(vectors, 32)].
hipError_t quantize_activations(const float* x, uint64_t x_row_stride, uint64_t vectors,
                                uint64_t columns, int8_t* q, float* scale, int32_t* sum,
                                hipStream_t stream);

// Tiled layout for gemm_i8: blob (stage s, tile t) at ((s * tiles) + t) * tile_blob_bytes(limbs),
// stages = ceil(columns / 256), tiles = ceil(vectors / 32). Inside a blob:
//   limb l, 16-column chunk c (0..15), vector m (0..31): 16 int8 at  l*8192 + c*512 + m*16
//   scale[block b (0..7)][m] f32 at  limbs*8192 + b*128 + m*4
//   xsum [b][m] f32 (scale * integer block sum) at  limbs*8192 + 1024 + b*128 + m*4
//   pieces[b][m]: the scale as three bfloat16 values whose sum it is exactly, (s0 | s1 << 16, s2),
//                 8 bytes at  limbs*8192 + 2048 + b*256 + m*8
// in all a multiple of 4096 bytes.
// limbs = 1: int8 activations, scale = max|x| / 127.
// limbs = 3: 24-bit fixed point in three balanced signed bytes, scale = max|x| / (127 * 65536).
// limbs = 2 is the layout of gemm_h16: 24-bit fixed point per vector and 256-column stage in two
// balanced 12-bit halves, each a half float:
//   half l (0: low / 4096, 1: high), 8-column part c (0..31), vector m: 8 half floats at  l*16384 + c*512 + m*16
//   unit[m] f32 (max|x| / (2^23 - 1)) at  32768 + m*4
//   xsum[sub-block g (0..7)][m] f32 at  32768 + 128 + g*128 + m*4
// and padding up to 34 KiB.
constexpr uint32_t tile_blob_bytes(int limbs) { return limbs == 1 ? 12288u : limbs == 2 ? 34816u : 28672u; }
constexpr uint64_t tile_workspace_bytes(int limbs, uint64_t vectors, uint64_t columns) {
    return ((columns + 255) / 256) * ((vectors + 31) / 32) * tile_blob_bytes(limbs);
}
hipError_t quantize_tiles(const float* x, uint64_t x_row_stride, uint64_t vectors, uint64_t columns,
                          int limbs, uint8_t* tiles, hipStream_t stream);
// The limbs = 2 tiles of silu(gate) * up / of rms_norm(x) * weight (weight may be null), computed
// on the fly with the arithmetic of silu_mul() / rms_norm() below: the same bits as the operator
// followed by quantize_tiles, one launch less. columns % 256 == 0, 16-byte aligned rows.
hipError_t quantize_tiles_silu_mul(const float* gate, const float* up, uint64_t row_stride, uint64_t vectors,
                                   uint64_t columns, uint8_t* tiles, hipStream_t stream);
// weight: [columns] floats, or half floats (weight_is_half; widened on use), or null.
hipError_t quantize_tiles_rms_norm(const float* x, uint64_t x_row_stride, const void* weight, int weight_is_half,
                                   double eps, uint64_t vectors, uint64_t columns, uint8_t* tiles, hipStream_t stream);
// The same with x = y computed in the same launch from the unsummed K shares of a contraction:
// y[m, n] = shares in share order (+ bias[n]) (+ residual[m, n], which may be y itself), written to
// y [vectors, columns] - the bytes reduce_group_kernel writes - and then normed and quantised.
hipError_t quantize_tiles_rms_norm_of_shares(const float* shares, uint32_t share_count, uint64_t launch_rows,
                                             const float* bias, const float* residual, float* y, const void* weight,
                                             int weight_is_half, double eps, uint64_t vectors, uint64_t columns,
                                             uint8_t* tiles, hipStream_t stream);

// ---- gemm_i8.hip: matrix-core contraction over quantised activation tiles ---------
bool gemm_i8_supported(int32_t codec, uint64_t columns);
// From this many vectors on, f32-mode requests use the matrix cores (3-limb activations):
// measured on MI355X, two launches of the 3-vector GEMV are still faster below it.
constexpr uint32_t kGemmMinVectors = 7;
// Launches with few output tiles share K out over this many workgroups per tile (1 = no sharing);
// `partials` then holds k_splits * vectors * rows floats. partials == nullptr: never share.
uint32_t gemm_i8_k_splits(int32_t codec, int limbs, uint64_t rows, uint64_t columns, uint64_t vectors);
struct GemmOutput {
    const float* bias;      // [rows] or null
    const float* residual;  // [vectors, rows] added to the result, or null; may be y itself
    float* y;               // [vectors, rows]
    float* partials;        // see gemm_i8_k_splits, or null
    // gemm_h16 only: leave the K shares in `partials` unsummed ([share][vector][launch row], see
    // gemm_h16_shares_layout) for a consumer that sums them itself; bias, residual and y are then unused.
    bool leave_shares = false;
};
hipError_t gemm_i8(int32_t codec, int limbs, const uint8_t* weight, const uint8_t* tiles,
                   const GemmOutput& out, uint64_t rows, uint64_t columns, uint64_t vectors,
                   hipStream_t stream);
// y = bias + the k_splits partial results in share order (+ residual); the second kernel of a launch
// that shared K out.
hipError_t reduce_partials(const float* partials, const float* bias, const float* residual, float* y,
                           uint32_t rows, uint32_t vectors, uint32_t k_splits, hipStream_t stream);

// ---- gemm_h16.hip: Q4_K, Q5_K and Q6_K on the half-float matrix cores, exact integer operands (limbs = 2 tiles) ----
bool gemm_h16_supported(int32_t codec, uint64_t columns);
hipError_t gemm_h16(int32_t codec, const uint8_t* weight, const uint8_t* tiles, const GemmOutput& out,
                    uint64_t rows, uint64_t columns, uint64_t vectors, hipStream_t stream);
// Several matrices of one codec and the same width against the same activation tiles in one launch (the q / k /
// v projections of a decode step): the grid runs over the row tiles of all of them, and K is shared
// out by the rule of gemm_i8_k_splits for that many tiles. `partials` holds
// gemm_h16_group_partial_bytes(...) bytes when that is not zero.
constexpr uint32_t kGemmGroupMost = 4;
struct GemmMember {
    const uint8_t* weight;
    const float* bias;      // [rows] or null
    const float* residual;  // [vectors, rows] or null; may be y
    float* y;               // [vectors, rows]
    uint64_t rows;
};
// Rows per workgroup (64 or 128), row tiles of that height over all members, K shares.
struct GemmGroupGeometry {
    uint32_t tile_rows;
    uint64_t row_tiles;
    uint32_t k_splits;
};
GemmGroupGeometry gemm_h16_group_geometry(int32_t codec, const uint64_t* rows, uint32_t count, uint64_t columns,
                                          uint64_t vectors);
uint64_t gemm_h16_group_partial_bytes(int32_t codec, const uint64_t* rows, uint32_t count, uint64_t columns,
                                      uint64_t vectors);
// A rotary embedding applied to some members of a group launch in the launch that sums their K
// shares: member i with bit i of `members` set is [vectors, rows / head_dim heads, 1 step, head_dim]
// at positions offsets[0] or offsets[vector] (rotary_kernel's arithmetic, decode_math.h).
struct GemmRotary {
    uint32_t members;
    const uint32_t* offsets;
    uint32_t offsets_len;
    double theta, sign;
    int interleaved;
    uint32_t head_dim;
};
hipError_t gemm_h16_group(int32_t codec, const GemmMember* members, uint32_t count, const uint8_t* tiles,
                          float* partials, uint64_t columns, uint64_t vectors, hipStream_t stream,
                          bool leave_shares = false, const GemmRotary* rotary = nullptr);
// Measurement only (et_hip_calibration_contraction): the Q4_K kernel of 64-row tiles without K shares
// as it is (probe 0), without its consumers' arithmetic (1), without its copies (2), without the weight
// (3) or the activation copies (4), with the weight (5) or the activation copies (6) and nothing else; at
// most 32 vectors. y receives meaningless values for probes > 0.
hipError_t gemm_h16_probe(int probe, const uint8_t* weight, const uint8_t* tiles, float* y, uint64_t rows,
                          uint64_t columns, uint64_t vectors, hipStream_t stream);
// Where a one-matrix launch with K shares leaves them: share k, vector m, row n at
// partials[(k * vectors + m) * launch_rows + n].
struct GemmShares {
    uint32_t count;        // 1: the launch does not share K
    uint64_t launch_rows;  // rows rounded up to whole tiles
};
GemmShares gemm_h16_shares_layout(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors);

// ---- kv_attention.hip: paged key/value-cache attention ---------------------------
constexpr int kKvTableEntries = 1024;     // blocks one context split of the streaming kernel may touch
constexpr int kKvAnyWidthPerLane = 8;     // the any-width kernel covers head widths up to 64 * 8
// The device status block holds one word per slot: 0, or code << 56 | value (56 bits of value).
enum : uint32_t {
    kKvBadAdvance = 1,    // value = the advance
    kKvOverCapacity = 2,  // value = live context
    kKvShortTable = 3,    // value = cursor + advance
    kKvOverDeclared = 4,  // value = cursor + advance, above the caller's max_context
    kKvBlockOutside = 5,  // value = physical row
};
// q, k and v of a decode step as the unsummed K shares of the group launch that projected them
// (gemm_h16_group with leave_shares): share s of vector m, launch row n at
// shares[(s * vectors + m) * launch_rows + n]; the projections start at launch rows q_row, k_row, v_row.
struct KvProjected {
    const float* shares;  // null: q, k, v arrive as tensors
    uint32_t count, vectors;
    uint64_t launch_rows;
    uint32_t q_row, k_row, v_row;
    const float* q_bias;  // [query_heads * width], or null
    const float* k_bias;  // [kv_heads * width], or null
    const float* v_bias;
    const uint32_t* offsets;  // rotary positions of q and k: 1 or `vectors` device words
    uint32_t offsets_len;
    int32_t interleaved;
    double theta, sign;
};
struct KvAttention {
    void* k_slab;
    void* v_slab;
    int32_t slab_dtype;  // ET_DTYPE_F32, _F16, _BF16 or _U8 (the int8-quantized tier)
    float* k_scales;     // [max_tokens, kv_heads], ET_DTYPE_U8 only
    float* v_scales;
    uint32_t max_tokens, kv_heads, width, block_size;
    const uint32_t* block_table;  // [batch, table_stride]
    uint32_t table_stride;
    const uint32_t* cursors;      // [batch]
    const uint32_t* advances;     // [batch]
    uint32_t batch, active_batch, query_heads, tokens;
    uint32_t context_window, window, max_context;
    const float* q;               // [batch, query_heads, tokens, width]
    const float* k;               // [batch, kv_heads, tokens, width]
    const float* v;
    double scale;
    float* out;                   // like q
    void* status;                 // 8 bytes per slot, written by the call
    // Optional (tokens == 1): `out` seen as activations [batch, query_heads * width], quantised into
    // gemm_h16's tiles (quantize_tiles with two halves) - by the attention kernel itself where one
    // workgroup holds whole 256-column stages of a row, by a quantiser launch otherwise.
    uint8_t* prepared = nullptr;
    // Optional (tokens == 1, a shape the streaming kernel takes): q, k, v above are unused; every workgroup
    // sums the shares of the rows it needs, adds the biases and rotates q and k - the bytes of
    // reduce_group_rotary_kernel - before it attends (kv_attention returns hipErrorInvalidValue for other shapes).
    KvProjected projected = {};
};
struct KvLaunchShape {
    bool streaming;
    int waves;  // per workgroup of the streaming kernel: 4 or 8
    uint32_t splits;
    uint64_t workgroups;
    uint64_t workspace_bytes;
};
KvLaunchShape kv_attention_shape(const KvAttention& p);
// Attends, appends the new rows, merges; `workspace` holds kv_attention_shape(p).workspace_bytes.
hipError_t kv_attention(const KvAttention& p, void* workspace, hipStream_t stream);

// ---- decode_ops.hip: the small operators next to the contraction in a decode step ----
// Dense f32 rows; weight: [columns] floats, or half floats (weight_is_half), or null. rows, columns < 2^32.
hipError_t rms_norm(const float* x, const void* weight, int weight_is_half, double eps, float* out, uint64_t rows,
                    uint64_t columns, hipStream_t stream);
// cursors[slot] += advances[slot] for slot < slots: the commit of a decode step.
hipError_t commit_advances(uint32_t* cursors, const uint32_t* advances, uint64_t slots, hipStream_t stream);
// gather_rows for a table of half floats (or bfloat16) into f32 rows.
hipError_t gather_rows_widen(const void* table, int table_is_bf16, uint64_t table_rows, uint64_t width, const void* indexes,
                             int index_is_i64, uint64_t count, float* out, void* status, hipStream_t stream);
// x, out: [rows, steps, head_dim]; offsets: 1 or `batch` device words; rows % batch == 0.
hipError_t rotary(const float* x, const uint32_t* offsets, uint32_t offsets_len, double theta, double sign,
                  int interleaved, float* out, uint64_t batch, uint64_t rows, uint64_t steps, uint64_t head_dim,
                  hipStream_t stream);
// The same for two tensors of the same batch, steps and head width in one launch (rows = elements /
// (steps * head_dim) of each).
hipError_t rotary_pair(const float* x, float* out, uint64_t rows, const float* second, float* second_out,
                       uint64_t second_rows, const uint32_t* offsets, uint32_t offsets_len, double theta, double sign,
                       int interleaved, uint64_t batch, uint64_t steps, uint64_t head_dim, hipStream_t stream);
hipError_t add(const float* a, const float* b, float* out, uint64_t count, hipStream_t stream);
hipError_t silu_mul(const float* gate, const float* up, float* out, uint64_t count, hipStream_t stream);
// out[row] = greedy token; status[row] = 0, or 1 + the first token whose logit is not finite.
// `workspace` holds argmax_workspace_bytes(rows, columns), 4-byte aligned.
uint64_t argmax_workspace_bytes(uint64_t rows, uint64_t columns);
hipError_t argmax_rows(const float* logits, uint64_t rows, uint64_t columns, uint32_t* out, uint32_t* status,
                       void* workspace, hipStream_t stream);
// out[p, :] = table[indexes[p], :] as bytes; status[p] (8 bytes each) = 0, or bit 63 | the index.
hipError_t gather_rows(const void* table, uint64_t table_rows, uint64_t row_bytes, const void* indexes,
                       int index_is_i64, uint64_t count, void* out, void* status, hipStream_t stream);

// ---- calibrate.hip: measurement aids (plain read / copy of known size, matrix-core loops) -------
// sink must hold 4 * `workgroups` words; bytes < 2^36.
hipError_t calibration_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups,
                            hipStream_t stream);
enum : int {
    kReadPlain = 0, kReadDeep = 1, kReadStreaming = 2, kReadLds4 = 3, kReadLds8 = 4, kReadLds8Nt = 5,
    kReadLds8NtShallow = 6, kReadLds8NtRanges = 7, kReadLds8NtRangesShallow = 8
};
hipError_t calibration_read_variant(int variant, const void* src, uint64_t bytes, uint32_t* sink,
                                    uint32_t workgroups, hipStream_t stream);
hipError_t calibration_copy(const void* src, void* dst, uint64_t bytes, hipStream_t stream);
// Loops of matrix-core instructions without memory traffic: four waves per workgroup, four
// independent instructions per wave and round; sink gets one float per thread (256 * workgroups).
enum : int { kMfmaI8 = 0, kMfmaI8Scaled = 1, kMfmaF16 = 2, kMfmaF16Small = 3, kMfmaI8ScaledBf16 = 4,
              kMfmaI8Biased = 5, kMfmaI8BiasedMatrixOnly = 6, kMfmaI8BiasedValuOnly = 7 };
hipError_t calibration_mfma(int kind, uint32_t iterations, uint32_t workgroups, float* sink, hipStream_t stream);

}  // namespace et
