/* See et_oracle_kv.h. Plain C restatement of the reference's paged KV attention. */
#include "et_oracle_kv.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

float et_oracle_fp16_to_f32(uint16_t h); /* et_oracle.c */

/* f16::from_f32 (half 2.7.1): round to nearest, ties to even; overflow to infinity;
 * subnormal results; NaN keeps its sign and gets a quiet payload bit. */
uint16_t et_oracle_f32_to_fp16(float value) {
    uint32_t x;
    memcpy(&x, &value, sizeof x);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t exponent = (x >> 23) & 0xffu;
    uint32_t mantissa = x & 0x7fffffu;
    if (exponent == 0xffu) { /* infinity or NaN */
        if (mantissa == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (mantissa >> 13));
    }
    const int32_t unbiased = (int32_t)exponent - 127;
    if (unbiased > 15) return (uint16_t)(sign | 0x7c00u); /* overflow */
    if (unbiased >= -14) {                                 /* normal result */
        uint32_t half = ((uint32_t)(unbiased + 15) << 10) | (mantissa >> 13);
        const uint32_t rest = mantissa & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (half & 1u))) half++; /* may carry into the exponent */
        return (uint16_t)(sign | half);
    }
    if (unbiased < -25) return (uint16_t)sign; /* below half of the smallest subnormal */
    /* subnormal result: value = m * 2^-24 with m = round(1.mantissa * 2^(unbiased + 24)) */
    mantissa |= 0x800000u;
    const int shift = -unbiased - 1; /* 14 .. 24: bits dropped from the 24-bit significand */
    uint32_t half = mantissa >> shift;
    const uint32_t rest = mantissa & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rest > halfway || (rest == halfway && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

/* bf16::from_f32 (half 2.7.1): NaN keeps its top bits and gets a quiet bit; otherwise round to
 * nearest even on the sixteen dropped bits. */
uint16_t et_oracle_f32_to_bf16(float value) {
    uint32_t x;
    memcpy(&x, &value, sizeof x);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    const uint32_t round_bit = 0x00008000u;
    if ((x & round_bit) != 0 && (x & (3u * round_bit - 1u)) != 0) return (uint16_t)((x >> 16) + 1u);
    return (uint16_t)(x >> 16);
}

static float bf16_to_f32(uint16_t bits) {
    const uint32_t x = (uint32_t)bits << 16;
    float value;
    memcpy(&value, &x, sizeof value);
    return value;
}

static int fail(char* err, size_t err_len, const char* message) {
    if (err != NULL && err_len > 0) snprintf(err, err_len, "%s", message);
    return -1;
}

/* SlabReader::get_f32 (pool.rs) and, for the u8 tier, `cached` (napi/mod.rs:3467-3478):
 * (raw - 128) * scale of the row and head. */
static float slab_get(int dtype, const void* slab, const float* scales, size_t index, size_t width) {
    if (dtype == 0) return ((const float*)slab)[index];
    if (dtype == 2) return et_oracle_fp16_to_f32(((const uint16_t*)slab)[index]);
    if (dtype == 3) return bf16_to_f32(((const uint16_t*)slab)[index]);
    return ((float)((const uint8_t*)slab)[index] - 128.0f) * scales[index / width];
}

static void slab_set(int dtype, void* slab, size_t index, float value) {
    if (dtype == 0)
        ((float*)slab)[index] = value;
    else if (dtype == 2)
        ((uint16_t*)slab)[index] = et_oracle_f32_to_fp16(value);
    else
        ((uint16_t*)slab)[index] = et_oracle_f32_to_bf16(value);
}

/* The u8 tier's write (napi/mod.rs:3397-3437): one scale per row and head, max|x| / 127 + 1e-12,
 * bytes round(x / scale) clamped to +-127, plus 128. f32::round rounds halves away from zero. */
static void slab_set_row_u8(uint8_t* slab, float* scales, size_t row_head, const float* values, size_t width) {
    float maximum = 0.0f;
    for (size_t column = 0; column < width; column++) {
        const float magnitude = fabsf(values[column]);
        if (magnitude > maximum) maximum = magnitude; /* f32::max ignores a NaN operand the same way */
    }
    const float scale = maximum / 127.0f + 1e-12f;
    scales[row_head] = scale;
    for (size_t column = 0; column < width; column++) {
        float value = roundf(values[column] / scale);
        if (value < -127.0f) value = -127.0f;
        if (value > 127.0f) value = 127.0f;
        slab[row_head * width + column] = (uint8_t)(value + 128.0f);
    }
}

int et_oracle_kv_attention(int slab_dtype, void* k_slab, void* v_slab, size_t max_tokens,
                           size_t kv_heads, size_t width, size_t block_size,
                           const uint32_t* block_table, size_t table_stride,
                           const uint32_t* cursors, const uint32_t* advances, size_t batch,
                           size_t active_batch, size_t query_heads, size_t tokens, const float* q,
                           const float* k, const float* v, double scale, size_t context_window, size_t window,
                           float* out, char* err, size_t err_len) {
    return et_oracle_kv_attention_scaled(slab_dtype, k_slab, v_slab, NULL, NULL, max_tokens, kv_heads, width,
                                         block_size, block_table, table_stride, cursors, advances, batch,
                                         active_batch, query_heads, tokens, q, k, v, scale, context_window, window,
                                         out, err, err_len);
}

int et_oracle_kv_attention_scaled(int slab_dtype, void* k_slab, void* v_slab, float* k_scales, float* v_scales,
                                  size_t max_tokens, size_t kv_heads, size_t width, size_t block_size,
                                  const uint32_t* block_table, size_t table_stride,
                                  const uint32_t* cursors, const uint32_t* advances, size_t batch,
                                  size_t active_batch, size_t query_heads, size_t tokens, const float* q,
                                  const float* k, const float* v, double scale, size_t context_window,
                                  size_t window, float* out, char* err, size_t err_len) {
    if (slab_dtype != 0 && slab_dtype != 2 && slab_dtype != 3 && slab_dtype != 4)
        return fail(err, err_len, "kv attention: unsupported slab dtype");
    if (slab_dtype == 4 && (k_scales == NULL || v_scales == NULL))
        return fail(err, err_len, "kv attention: the u8 tier needs its scale slabs");
    /* napi/mod.rs:3347-3360 */
    if (kv_heads == 0 || query_heads % kv_heads != 0)
        return fail(err, err_len, "kv attention: incompatible grouped-query q/k/v shapes");
    if (active_batch > batch) return fail(err, err_len, "kv attention: active batch exceeds batch");
    memset(out, 0, batch * query_heads * tokens * width * sizeof(float)); /* :3371 out.fill(0.0) */
    double* weights = NULL;
    size_t weight_capacity = 0;
    for (size_t b = 0; b < active_batch; b++) {
        /* kv_prepare, :3588-3603 */
        const size_t cursor = cursors[b], advance = advances[b];
        if (advance == 0 || advance > tokens) {
            char message[128];
            snprintf(message, sizeof message, "kv attention: advance %zu out of range for chunk length %zu",
                     advance, tokens);
            { free(weights); return fail(err, err_len, message); }
        }
        const size_t needed = cursor + advance;
        const size_t start = context_window != 0 ? (needed > context_window ? needed - context_window : 0) : 0;
        if (needed - start > max_tokens) { free(weights); return fail(err, err_len, "kv attention: live context exceeds pool capacity"); }
        if ((needed + block_size - 1) / block_size > table_stride)
            { free(weights); return fail(err, err_len, "kv attention: block table too short"); }
        const uint32_t* blocks = block_table + b * table_stride;
        /* write first, :3393-3458 (f32 / half slabs) */
        for (size_t token = 0; token < advance; token++) {
            const size_t position = cursor + token;
            const size_t row = (size_t)blocks[position / block_size] * block_size + position % block_size;
            if (row >= max_tokens) { free(weights); return fail(err, err_len, "kv attention: block outside the pool"); }
            for (size_t head = 0; head < kv_heads; head++) {
                const size_t logical_row = ((b * kv_heads + head) * tokens + token) * width;
                if (slab_dtype == 4) {
                    slab_set_row_u8((uint8_t*)k_slab, k_scales, row * kv_heads + head, k + logical_row, width);
                    slab_set_row_u8((uint8_t*)v_slab, v_scales, row * kv_heads + head, v + logical_row, width);
                    continue;
                }
                for (size_t column = 0; column < width; column++) {
                    slab_set(slab_dtype, k_slab, (row * kv_heads + head) * width + column, k[logical_row + column]);
                    slab_set(slab_dtype, v_slab, (row * kv_heads + head) * width + column, v[logical_row + column]);
                }
            }
        }
        /* then attend, :3476-3542: three passes in f64 per (head, query) */
        for (size_t head = 0; head < query_heads; head++) {
            const size_t kv_head = head / (query_heads / kv_heads);
            for (size_t query = 0; query < tokens; query++) {
                size_t end = cursor + query + 1;
                if (end > needed) end = needed;
                size_t begin = start;
                if (window != 0) {
                    const size_t low = end > window ? end - window : 0;
                    begin = low > start ? low : start;
                }
                const float* q_row = q + ((b * query_heads + head) * tokens + query) * width;
                double maximum = -INFINITY;
                for (size_t position = begin; position < end; position++) {
                    const size_t row = (size_t)blocks[position / block_size] * block_size + position % block_size;
                    double score = 0.0;
                    for (size_t column = 0; column < width; column++)
                        score += (double)q_row[column] *
                                 (double)slab_get(slab_dtype, k_slab, k_scales, (row * kv_heads + kv_head) * width + column, width);
                    if (score * scale > maximum) maximum = score * scale;
                }
                /* The reference recomputes every score in the second pass and again per output column
                 * (:3497-3536); the recomputation yields bit-identical f64 values, so the weights are
                 * kept from the second pass. */
                if (end - begin > weight_capacity) {
                    free(weights);
                    weight_capacity = 2 * (end - begin);
                    weights = (double*)malloc(weight_capacity * sizeof(double));
                    if (weights == NULL) return fail(err, err_len, "kv attention: out of memory");
                }
                double denominator = 0.0;
                for (size_t position = begin; position < end; position++) {
                    const size_t row = (size_t)blocks[position / block_size] * block_size + position % block_size;
                    double score = 0.0;
                    for (size_t column = 0; column < width; column++)
                        score += (double)q_row[column] *
                                 (double)slab_get(slab_dtype, k_slab, k_scales, (row * kv_heads + kv_head) * width + column, width);
                    weights[position - begin] = exp(score * scale - maximum);
                    denominator += weights[position - begin];
                }
                float* out_row = out + ((b * query_heads + head) * tokens + query) * width;
                for (size_t column = 0; column < width; column++) {
                    double result = 0.0;
                    for (size_t position = begin; position < end; position++) {
                        const size_t row = (size_t)blocks[position / block_size] * block_size + position % block_size;
                        result += weights[position - begin] *
                                  (double)slab_get(slab_dtype, v_slab, v_scales, (row * kv_heads + kv_head) * width + column, width);
                    }
                    out_row[column] = (float)(result / denominator);
                }
            }
        }
    }
    free(weights);
    return 0;
}
