/*
 * CPU oracle for the block-quantized weight x activation contraction.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing on the product path (the HIP library and
 * its host layer) may include, link or call this. It is the checker used by
 * the test-suite, by the smoke check and by the benchmark's CPU-baseline leg.
 *
 * Every routine is a plain-C restatement of the reference's scalar CPU
 * algorithm; each cites the reference lines it follows. Build with
 * -ffp-contract=off and without -ffast-math: the reference rounds every f32
 * multiply, add and subtract separately.
 *
 * Pin status (what fixes each function besides "it was retyped"):
 *   et_oracle_fp16_to_f32      all 65536 codes vs numpy float16->float32; fixture constants
 *   et_oracle_scale_min_k4     reference fixtures (low branch); inverse-packer brute force
 *                              over all 64x64 pairs at all 8 positions (both branches)
 *   et_oracle_decode_block     Q2_K..Q6_K: the reference's five fixture tables (exact);
 *                              pack->decode round trips against closed forms on random
 *                              fields (element order, high-bit branch, signed scales)
 *                              Q8_0 / Q4_0: NOT in the reference. Public ggml layout only;
 *                              round trip with an independent packer. PARITY UNPINNED
 *                              by the reference.
 *   et_oracle_linear_into      reference KATs [4096.5, 4095.5, 512.5, 511.5] and [2048 x3];
 *                              x = e_k selects one decoded weight exactly; x = ones gives the
 *                              sequential row sum; strided views equal their dense copies
 *   et_oracle_embedding_into   reference KAT (Q5_K, rows [1,1], u32 and i64); index errors
 *   et_oracle_quantize_q8 /    NOT in the reference (it has no int8 activation path).
 *   et_oracle_linear_q8_into   Builder-defined; pinned by an int64 brute-force dot on tiny
 *                              inputs and by |err| <= 2e-2 against et_oracle_linear_into.
 *                              PARITY UNPINNED by the reference.
 */
#ifndef ET_ORACLE_H
#define ET_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGML tensor type codes. 10..14 are the reference's GgmlKQuant
 * (crates/runtime/src/gguf.rs:199-205, codes at gguf.rs:278-291); 2 and 8 are
 * the legacy ggml formats the reference does not implement. */
enum {
    ET_ORACLE_Q4_0 = 2,
    ET_ORACLE_Q8_0 = 8,
    ET_ORACLE_Q2_K = 10,
    ET_ORACLE_Q3_K = 11,
    ET_ORACLE_Q4_K = 12,
    ET_ORACLE_Q5_K = 13,
    ET_ORACLE_Q6_K = 14
};

/* Dense-or-strided view of a caller-owned buffer, in elements. strides == NULL
 * means row-major contiguous (offset still applies). Mirrors the reference's
 * Layout as consumed by source_index (crates/runtime-cpu/src/tensor.rs:940-953). */
typedef struct {
    int rank;
    const size_t* shape;
    const size_t* strides; /* may be NULL */
    size_t offset;
} et_oracle_layout;

const char* et_oracle_codec_name(int codec);
size_t et_oracle_block_values(int codec); /* 256 for K-quants, 32 for Q8_0/Q4_0, 0 = unknown */
size_t et_oracle_block_bytes(int codec);  /* 0 = unknown */
/* 0 when columns is not a multiple of the block width or on overflow. */
size_t et_oracle_encoded_row_bytes(int codec, size_t columns);

float et_oracle_fp16_to_f32(uint16_t bits);
void et_oracle_scale_min_k4(size_t index, const uint8_t* scales12, uint8_t* scale, uint8_t* min);

/* Decodes one packed block into block_values(codec) floats. Returns 0, or -1
 * with a message in err when block_len is not the codec's block size. */
int et_oracle_decode_block(int codec, const uint8_t* block, size_t block_len, float* out,
                           char* err, size_t err_len);

size_t et_oracle_source_index(const et_oracle_layout* layout, size_t logical);

/* y[v*rows + r] = (sum over blocks, lanes in order) x[v, k] * decode(W[r])[k] (+ bias[r]).
 * cancel may be NULL; a non-zero *cancel yields -2 and "operation aborted".
 * Returns 0 on success, -1 on a validation error (message in err). */
int et_oracle_linear_into(int codec, size_t rows, size_t columns, const float* x,
                          const et_oracle_layout* x_layout, const uint8_t* weight,
                          size_t weight_bytes, const float* bias,
                          const et_oracle_layout* bias_layout, float* y,
                          const volatile int32_t* cancel, char* err, size_t err_len);

/* Same loop, rows [row_begin, row_end) only, x dense [vectors, columns];
 * y is still indexed [v*rows + r]. Used to time and to check row subsets. */
int et_oracle_linear_rows(int codec, size_t rows, size_t columns, size_t vectors, const float* x,
                          const uint8_t* weight, const float* bias, float* y, size_t row_begin,
                          size_t row_end);

/* out[p, :] = decode(W[index[p], :]). index_is_i64 selects int64_t vs uint32_t. */
int et_oracle_embedding_into(int codec, size_t rows, size_t columns, const void* indexes,
                             int index_is_i64, const et_oracle_layout* index_layout, size_t count,
                             const uint8_t* weight, size_t weight_bytes, float* out,
                             const volatile int32_t* cancel, char* err, size_t err_len);

/* int8 activation quantizer, per vector and per 32 columns:
 *   amax = max|x|; scale = amax / 127; inv = amax > 0 ? 127 / amax : 0;
 *   q = clamp(rint(x * inv), -127, 127); sum = sum of q (int32). */
void et_oracle_quantize_q8(size_t vectors, size_t columns, const float* x, int8_t* q, float* scale,
                           int32_t* sum);

/* int8-activation contraction for Q8_0, Q4_0 and Q4_K weights over
 * pre-quantized activations, rows [row_begin, row_end). */
int et_oracle_linear_q8_rows(int codec, size_t rows, size_t columns, size_t vectors,
                             const int8_t* q, const float* scale, const int32_t* sum,
                             const uint8_t* weight, const float* bias, float* y, size_t row_begin,
                             size_t row_end);

#ifdef __cplusplus
}
#endif
#endif
