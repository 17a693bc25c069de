/*
 * CPU oracle: plain-C restatement of the reference's scalar quantized kernels.
 * TEST INFRASTRUCTURE ONLY - see et_oracle.h for who may use it and for the
 * pin status of every function.
 *
 * Compile: gcc -O2 -ffp-contract=off -fno-fast-math (no FMA contraction, no
 * reassociation), so each f32 operation rounds exactly once, like the
 * reference's Rust `f32` arithmetic.
 */
#include "et_oracle.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

/* ---- codec tables: crates/runtime/src/gguf.rs:199-251 and
 *      crates/runtime-cpu/src/quantized.rs:60-68. Q8_0/Q4_0: public ggml layout. */

const char* et_oracle_codec_name(int codec) {
    switch (codec) {
        case ET_ORACLE_Q4_0: return "Q4_0";
        case ET_ORACLE_Q8_0: return "Q8_0";
        case ET_ORACLE_Q2_K: return "Q2_K";
        case ET_ORACLE_Q3_K: return "Q3_K";
        case ET_ORACLE_Q4_K: return "Q4_K";
        case ET_ORACLE_Q5_K: return "Q5_K";
        case ET_ORACLE_Q6_K: return "Q6_K";
        default: return "?";
    }
}

size_t et_oracle_block_values(int codec) {
    switch (codec) {
        case ET_ORACLE_Q4_0:
        case ET_ORACLE_Q8_0: return 32;
        case ET_ORACLE_Q2_K:
        case ET_ORACLE_Q3_K:
        case ET_ORACLE_Q4_K:
        case ET_ORACLE_Q5_K:
        case ET_ORACLE_Q6_K: return 256;
        default: return 0;
    }
}

size_t et_oracle_block_bytes(int codec) {
    switch (codec) {
        case ET_ORACLE_Q4_0: return 18;
        case ET_ORACLE_Q8_0: return 34;
        case ET_ORACLE_Q2_K: return 84;
        case ET_ORACLE_Q3_K: return 110;
        case ET_ORACLE_Q4_K: return 144;
        case ET_ORACLE_Q5_K: return 176;
        case ET_ORACLE_Q6_K: return 210;
        default: return 0;
    }
}

/* gguf.rs:245-250: None unless columns is a multiple of the block; checked multiply. */
size_t et_oracle_encoded_row_bytes(int codec, size_t columns) {
    size_t values = et_oracle_block_values(codec);
    size_t bytes = et_oracle_block_bytes(codec);
    if (values == 0 || columns % values != 0) return 0;
    size_t blocks = columns / values;
    if (blocks != 0 && bytes > SIZE_MAX / blocks) return 0;
    return blocks * bytes;
}

/* ---- fp16: quantized.rs:71-73 calls half 2.7.1 f16::from_bits(..).to_f32(),
 * which is the exact IEEE binary16 -> binary32 widening (NaNs come out quiet
 * with the payload shifted left by 13). */
float et_oracle_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            /* subnormal: value = man * 2^-24; normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 0x1f) {
        bits = man == 0 ? (sign | 0x7f800000u) : (sign | 0x7fc00000u | (man << 13));
    } else {
        bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &bits, sizeof out);
    return out;
}

static float fp16_at(const uint8_t* block, size_t offset) {
    return et_oracle_fp16_to_f32((uint16_t)(block[offset] | ((uint16_t)block[offset + 1] << 8)));
}

/* quantized.rs:77-86 */
void et_oracle_scale_min_k4(size_t index, const uint8_t* scales, uint8_t* scale, uint8_t* min) {
    if (index < 4) {
        *scale = scales[index] & 63;
        *min = scales[index + 4] & 63;
    } else {
        *scale = (uint8_t)((scales[index + 4] & 0x0f) | ((scales[index - 4] >> 6) << 4));
        *min = (uint8_t)((scales[index + 4] >> 4) | ((scales[index] >> 6) << 4));
    }
}

/* quantized.rs:117-138 */
static void decode_q2_k(const uint8_t* block, float* output) {
    const uint8_t* scales = block;
    const uint8_t* quants = block + 16;
    float d = fp16_at(block, 80);
    float dmin = fp16_at(block, 82);
    size_t group = 0;
    for (size_t half = 0; half < 2; half++) {
        const uint8_t* q = quants + half * 32;
        for (unsigned shift = 0; shift < 8; shift += 2) {
            for (size_t q_offset = 0; q_offset < 32; q_offset += 16) {
                uint8_t scale = scales[group];
                float dl = d * (float)(scale & 0x0f);
                float ml = dmin * (float)(scale >> 4);
                float* out = output + group * 16;
                for (size_t i = 0; i < 16; i++) {
                    float prod = dl * (float)((q[q_offset + i] >> shift) & 3);
                    out[i] = prod - ml;
                }
                group++;
            }
        }
    }
}

/* quantized.rs:142-176 */
static void decode_q3_k(const uint8_t* block, float* output) {
    const uint8_t* hmask = block;
    const uint8_t* quants = block + 32;
    const uint8_t* packed_scales = block + 96;
    float d = fp16_at(block, 108);
    size_t group = 0;
    for (size_t half = 0; half < 2; half++) {
        const uint8_t* q = quants + half * 32;
        for (unsigned lane = 0; lane < 4; lane++) {
            unsigned shift = lane * 2;
            uint8_t mask = (uint8_t)(1u << (half * 4 + lane));
            for (size_t q_offset = 0; q_offset < 32; q_offset += 16) {
                uint8_t low = group < 8 ? (packed_scales[group] & 0x0f)
                                        : (uint8_t)(packed_scales[group - 8] >> 4);
                uint8_t high = (packed_scales[8 + group % 4] >> (2 * (group / 4))) & 3;
                int scale = (int)(uint8_t)(low | (high << 4)) - 32;
                float dl = d * (float)scale;
                float* out = output + group * 16;
                for (size_t i = 0; i < 16; i++) {
                    int low_quant = (q[q_offset + i] >> shift) & 3;
                    int high_quant = (hmask[q_offset + i] & mask) == 0 ? 4 : 0;
                    out[i] = dl * (float)(low_quant - high_quant);
                }
                group++;
            }
        }
    }
}

/* quantized.rs:180-199 */
static void decode_q4_k(const uint8_t* block, float* output) {
    float d = fp16_at(block, 0);
    float dmin = fp16_at(block, 2);
    const uint8_t* scales = block + 4;
    const uint8_t* quants = block + 16;
    for (size_t pair = 0; pair < 4; pair++) {
        const uint8_t* q = quants + pair * 32;
        for (size_t side = 0; side < 2; side++) {
            size_t group = pair * 2 + side;
            uint8_t scale, min;
            et_oracle_scale_min_k4(group, scales, &scale, &min);
            float dl = d * (float)scale;
            float ml = dmin * (float)min;
            float* out = output + group * 32;
            for (size_t i = 0; i < 32; i++) {
                uint8_t quant = side == 0 ? (q[i] & 0x0f) : (uint8_t)(q[i] >> 4);
                float prod = dl * (float)quant;
                out[i] = prod - ml;
            }
        }
    }
}

/* quantized.rs:203-234 */
static void decode_q5_k(const uint8_t* block, float* output) {
    float d = fp16_at(block, 0);
    float dmin = fp16_at(block, 2);
    const uint8_t* scales = block + 4;
    const uint8_t* high = block + 16;
    const uint8_t* low = block + 48;
    for (size_t pair = 0; pair < 4; pair++) {
        const uint8_t* ql = low + pair * 32;
        uint8_t masks[2] = {(uint8_t)(1u << (pair * 2)), (uint8_t)(1u << (pair * 2 + 1))};
        for (size_t side = 0; side < 2; side++) {
            size_t group = pair * 2 + side;
            uint8_t scale, min;
            et_oracle_scale_min_k4(group, scales, &scale, &min);
            float dl = d * (float)scale;
            float ml = dmin * (float)min;
            float* out = output + group * 32;
            for (size_t i = 0; i < 32; i++) {
                uint8_t low_quant = side == 0 ? (ql[i] & 0x0f) : (uint8_t)(ql[i] >> 4);
                uint8_t quant = (uint8_t)(low_quant + ((high[i] & masks[side]) == 0 ? 0 : 16));
                float prod = dl * (float)quant;
                out[i] = prod - ml;
            }
        }
    }
}

/* quantized.rs:238-261. Note the product order: (d * scale) * quant. */
static void decode_q6_k(const uint8_t* block, float* output) {
    const uint8_t* low = block;
    const uint8_t* high = block + 128;
    float d = fp16_at(block, 208);
    for (size_t half = 0; half < 2; half++) {
        const uint8_t* ql = low + half * 64;
        const uint8_t* qh = high + half * 32;
        for (size_t i = 0; i < 32; i++) {
            size_t scale_lane = i / 16;
            uint8_t quants[4] = {
                (uint8_t)((ql[i] & 0x0f) | (((qh[i] >> 0) & 3) << 4)),
                (uint8_t)((ql[i + 32] & 0x0f) | (((qh[i] >> 2) & 3) << 4)),
                (uint8_t)((ql[i] >> 4) | (((qh[i] >> 4) & 3) << 4)),
                (uint8_t)((ql[i + 32] >> 4) | (((qh[i] >> 6) & 3) << 4)),
            };
            for (size_t quarter = 0; quarter < 4; quarter++) {
                size_t scale_index = half * 8 + scale_lane + quarter * 2;
                int8_t scale = (int8_t)block[192 + scale_index];
                int quant = (int)quants[quarter] - 32;
                float ds = d * (float)scale;
                output[half * 128 + quarter * 32 + i] = ds * (float)quant;
            }
        }
    }
}

/* Public ggml block_q8_0: fp16 d @0, int8 qs[32] @2; value = d * qs[i].
 * Not in the reference. */
static void decode_q8_0(const uint8_t* block, float* output) {
    float d = fp16_at(block, 0);
    for (size_t i = 0; i < 32; i++) output[i] = d * (float)(int8_t)block[2 + i];
}

/* Public ggml block_q4_0: fp16 d @0, qs[16] @2; element j is the low nibble of
 * qs[j], element j+16 the high nibble; value = d * (nibble - 8). Not in the reference. */
static void decode_q4_0(const uint8_t* block, float* output) {
    float d = fp16_at(block, 0);
    for (size_t j = 0; j < 16; j++) {
        output[j] = d * (float)((int)(block[2 + j] & 0x0f) - 8);
        output[j + 16] = d * (float)((int)(block[2 + j] >> 4) - 8);
    }
}

static void decode_unchecked(int codec, const uint8_t* block, float* output) {
    switch (codec) {
        case ET_ORACLE_Q4_0: decode_q4_0(block, output); break;
        case ET_ORACLE_Q8_0: decode_q8_0(block, output); break;
        case ET_ORACLE_Q2_K: decode_q2_k(block, output); break;
        case ET_ORACLE_Q3_K: decode_q3_k(block, output); break;
        case ET_ORACLE_Q4_K: decode_q4_k(block, output); break;
        case ET_ORACLE_Q5_K: decode_q5_k(block, output); break;
        case ET_ORACLE_Q6_K: decode_q6_k(block, output); break;
        default: break;
    }
}

/* quantized.rs:90-111 */
int et_oracle_decode_block(int codec, const uint8_t* block, size_t block_len, float* out,
                           char* err, size_t err_len) {
    size_t expected = et_oracle_block_bytes(codec);
    if (expected == 0 || block_len != expected) {
        if (err != NULL && err_len > 0)
            snprintf(err, err_len, "%s block has %zu bytes, expected %zu",
                     et_oracle_codec_name(codec), block_len, expected);
        return -1;
    }
    decode_unchecked(codec, block, out);
    return 0;
}

/* crates/runtime-cpu/src/tensor.rs:940-953 */
static int layout_is_contiguous(const et_oracle_layout* layout) {
    if (layout->strides == NULL) return 1;
    size_t expected = 1;
    for (int d = layout->rank - 1; d >= 0; d--) {
        if (layout->shape[d] != 1 && layout->strides[d] != expected) return 0;
        expected *= layout->shape[d];
    }
    return 1;
}

size_t et_oracle_source_index(const et_oracle_layout* layout, size_t logical) {
    if (layout_is_contiguous(layout)) return layout->offset + logical;
    size_t source = layout->offset;
    size_t remainder = logical;
    for (int d = layout->rank - 1; d >= 0; d--) {
        size_t width = layout->shape[d] > 1 ? layout->shape[d] : 1;
        size_t coordinate = remainder % width;
        remainder /= width;
        source += coordinate * layout->strides[d];
    }
    return source;
}

static int fail(char* err, size_t err_len, const char* message) {
    if (err != NULL && err_len > 0) snprintf(err, err_len, "%s", message);
    return -1;
}

/* cancellation: quantized.rs:451-453 */
static int aborted(char* err, size_t err_len) {
    fail(err, err_len, "operation aborted");
    return -2;
}

/* quantized.rs:419-499 (execute) with the checks of :266-292 and :367-415
 * reduced to what a raw-pointer interface can express. */
int et_oracle_linear_into(int codec, size_t rows, size_t columns, const float* x,
                          const et_oracle_layout* x_layout, const uint8_t* weight,
                          size_t weight_bytes, const float* bias,
                          const et_oracle_layout* bias_layout, float* y,
                          const volatile int32_t* cancel, char* err, size_t err_len) {
    char message[160];
    if (x_layout->rank < 2) return fail(err, err_len, "quantized_linear: input must be rank >= 2 f32");
    if (x_layout->shape[x_layout->rank - 1] != columns)
        return fail(err, err_len, "quantized_linear: input does not match the immutable plan");
    size_t encoded_row_bytes = et_oracle_encoded_row_bytes(codec, columns);
    if (encoded_row_bytes == 0 && columns != 0) {
        snprintf(message, sizeof message, "quantized_linear: logical row width %zu is invalid for %s",
                 columns, et_oracle_codec_name(codec));
        return fail(err, err_len, message);
    }
    if (encoded_row_bytes != 0 && rows > SIZE_MAX / encoded_row_bytes)
        return fail(err, err_len, "quantized_linear: packed weight byte size overflow");
    if (weight_bytes != rows * encoded_row_bytes) {
        snprintf(message, sizeof message,
                 "quantized_linear: expected exact contiguous packed %s weight [%zu, %zu] u8",
                 et_oracle_codec_name(codec), rows, encoded_row_bytes);
        return fail(err, err_len, message);
    }
    size_t vectors = 1;
    for (int d = 0; d < x_layout->rank - 1; d++) vectors *= x_layout->shape[d];
    size_t block_values = et_oracle_block_values(codec);
    size_t block_bytes = et_oracle_block_bytes(codec);
    size_t blocks = columns / block_values;
    float decoded[256];
    for (size_t vector = 0; vector < vectors; vector++) {
        for (size_t row = 0; row < rows; row++) {
            if (cancel != NULL && *cancel != 0) return aborted(err, err_len);
            size_t row_start = row * encoded_row_bytes;
            float sum = 0.0f;
            for (size_t block_index = 0; block_index < blocks; block_index++) {
                if (cancel != NULL && *cancel != 0)
                    return aborted(err, err_len);
                decode_unchecked(codec, weight + row_start + block_index * block_bytes, decoded);
                size_t input_start = vector * columns + block_index * block_values;
                for (size_t lane = 0; lane < block_values; lane++) {
                    size_t input_index = et_oracle_source_index(x_layout, input_start + lane);
                    float prod = x[input_index] * decoded[lane];
                    sum += prod;
                }
            }
            if (bias != NULL) sum += bias[et_oracle_source_index(bias_layout, row)];
            y[vector * rows + row] = sum;
        }
    }
    return 0;
}

int et_oracle_linear_rows(int codec, size_t rows, size_t columns, size_t vectors, const float* x,
                          const uint8_t* weight, const float* bias, float* y, size_t row_begin,
                          size_t row_end) {
    size_t encoded_row_bytes = et_oracle_encoded_row_bytes(codec, columns);
    if (encoded_row_bytes == 0 || row_end > rows) return -1;
    size_t block_values = et_oracle_block_values(codec);
    size_t block_bytes = et_oracle_block_bytes(codec);
    size_t blocks = columns / block_values;
    float decoded[256];
    for (size_t vector = 0; vector < vectors; vector++) {
        for (size_t row = row_begin; row < row_end; row++) {
            const uint8_t* packed = weight + row * encoded_row_bytes;
            float sum = 0.0f;
            for (size_t block_index = 0; block_index < blocks; block_index++) {
                decode_unchecked(codec, packed + block_index * block_bytes, decoded);
                const float* input = x + vector * columns + block_index * block_values;
                for (size_t lane = 0; lane < block_values; lane++) {
                    float prod = input[lane] * decoded[lane];
                    sum += prod;
                }
            }
            if (bias != NULL) sum += bias[row];
            y[vector * rows + row] = sum;
        }
    }
    return 0;
}

/* quantized.rs:546-616 */
int et_oracle_embedding_into(int codec, size_t rows, size_t columns, const void* indexes,
                             int index_is_i64, const et_oracle_layout* index_layout, size_t count,
                             const uint8_t* weight, size_t weight_bytes, float* out,
                             const volatile int32_t* cancel, char* err, size_t err_len) {
    char message[160];
    size_t encoded_row_bytes = et_oracle_encoded_row_bytes(codec, columns);
    if (encoded_row_bytes == 0 && columns != 0) {
        snprintf(message, sizeof message,
                 "quantized_embedding: logical row width %zu is invalid for %s", columns,
                 et_oracle_codec_name(codec));
        return fail(err, err_len, message);
    }
    if (encoded_row_bytes != 0 && rows > SIZE_MAX / encoded_row_bytes)
        return fail(err, err_len, "quantized_embedding: packed weight byte size overflow");
    if (weight_bytes != rows * encoded_row_bytes) {
        snprintf(message, sizeof message,
                 "quantized_embedding: expected exact contiguous packed %s weight [%zu, %zu] u8",
                 et_oracle_codec_name(codec), rows, encoded_row_bytes);
        return fail(err, err_len, message);
    }
    size_t block_values = et_oracle_block_values(codec);
    size_t block_bytes = et_oracle_block_bytes(codec);
    size_t blocks = columns / block_values;
    for (size_t logical_index = 0; logical_index < count; logical_index++) {
        if (cancel != NULL && *cancel != 0) return aborted(err, err_len);
        size_t source = et_oracle_source_index(index_layout, logical_index);
        size_t row;
        if (index_is_i64) {
            int64_t value = ((const int64_t*)indexes)[source];
            if (value < 0) {
                snprintf(message, sizeof message, "quantized_embedding: index %lld is outside 0..%zu",
                         (long long)value, rows);
                return fail(err, err_len, message);
            }
            row = (size_t)value;
        } else {
            row = ((const uint32_t*)indexes)[source];
        }
        if (row >= rows) {
            snprintf(message, sizeof message, "quantized_embedding: index %zu is outside 0..%zu", row,
                     rows);
            return fail(err, err_len, message);
        }
        for (size_t block_index = 0; block_index < blocks; block_index++) {
            if (cancel != NULL && *cancel != 0) return aborted(err, err_len);
            decode_unchecked(codec, weight + row * encoded_row_bytes + block_index * block_bytes,
                             out + logical_index * columns + block_index * block_values);
        }
    }
    return 0;
}

/* ---- int8-activation path. The reference has none (its only int8 is a
 * KV-cache storage tier); these semantics are this build's own. ---- */

void et_oracle_quantize_q8(size_t vectors, size_t columns, const float* x, int8_t* q, float* scale,
                           int32_t* sum) {
    size_t blocks = columns / 32;
    for (size_t v = 0; v < vectors; v++) {
        for (size_t b = 0; b < blocks; b++) {
            const float* in = x + v * columns + b * 32;
            float amax = 0.0f;
            for (size_t i = 0; i < 32; i++) {
                float a = fabsf(in[i]);
                if (a > amax) amax = a;
            }
            float s = amax / 127.0f;
            float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            int32_t total = 0;
            for (size_t i = 0; i < 32; i++) {
                float r = rintf(in[i] * inv);
                if (r > 127.0f) r = 127.0f;
                if (r < -127.0f) r = -127.0f;
                int8_t value = (int8_t)r;
                q[v * columns + b * 32 + i] = value;
                total += value;
            }
            scale[v * blocks + b] = s;
            if (sum != NULL) sum[v * blocks + b] = total;
        }
    }
}

int et_oracle_linear_q8_rows(int codec, size_t rows, size_t columns, size_t vectors,
                             const int8_t* q, const float* scale, const int32_t* sum,
                             const uint8_t* weight, const float* bias, float* y, size_t row_begin,
                             size_t row_end) {
    size_t encoded_row_bytes = et_oracle_encoded_row_bytes(codec, columns);
    if (encoded_row_bytes == 0 || row_end > rows) return -1;
    if (codec != ET_ORACLE_Q8_0 && codec != ET_ORACLE_Q4_0 && codec != ET_ORACLE_Q4_K) return -1;
    size_t xblocks = columns / 32;
    for (size_t v = 0; v < vectors; v++) {
        const int8_t* xq = q + v * columns;
        const float* xs = scale + v * xblocks;
        const int32_t* xsum = sum + v * xblocks;
        for (size_t row = row_begin; row < row_end; row++) {
            const uint8_t* packed = weight + row * encoded_row_bytes;
            float acc = 0.0f;
            if (codec == ET_ORACLE_Q8_0) {
                for (size_t b = 0; b < xblocks; b++) {
                    const uint8_t* block = packed + b * 34;
                    int32_t dot = 0;
                    for (size_t i = 0; i < 32; i++) dot += (int32_t)(int8_t)block[2 + i] * xq[b * 32 + i];
                    float ds = fp16_at(block, 0) * xs[b];
                    float term = ds * (float)dot;
                    acc += term;
                }
            } else if (codec == ET_ORACLE_Q4_0) {
                for (size_t b = 0; b < xblocks; b++) {
                    const uint8_t* block = packed + b * 18;
                    int32_t dot = 0;
                    for (size_t j = 0; j < 16; j++) {
                        dot += ((int32_t)(block[2 + j] & 0x0f) - 8) * xq[b * 32 + j];
                        dot += ((int32_t)(block[2 + j] >> 4) - 8) * xq[b * 32 + j + 16];
                    }
                    float ds = fp16_at(block, 0) * xs[b];
                    float term = ds * (float)dot;
                    acc += term;
                }
            } else {
                for (size_t sb = 0; sb < columns / 256; sb++) {
                    const uint8_t* block = packed + sb * 144;
                    float d = fp16_at(block, 0);
                    float dmin = fp16_at(block, 2);
                    for (size_t g = 0; g < 8; g++) {
                        uint8_t sc, m;
                        et_oracle_scale_min_k4(g, block + 4, &sc, &m);
                        const uint8_t* qs = block + 16 + (g / 2) * 32;
                        size_t b = sb * 8 + g;
                        int32_t dot = 0;
                        for (size_t i = 0; i < 32; i++) {
                            int32_t nib = (g & 1) == 0 ? (qs[i] & 0x0f) : (qs[i] >> 4);
                            dot += nib * xq[b * 32 + i];
                        }
                        float dl = d * (float)sc;
                        float ml = dmin * (float)m;
                        float pos = dl * (float)dot;
                        float neg = ml * (float)xsum[b];
                        float diff = pos - neg;
                        float term = xs[b] * diff;
                        acc += term;
                    }
                }
            }
            if (bias != NULL) acc += bias[row];
            y[v * rows + row] = acc;
        }
    }
    return 0;
}
