/* See et_oracle_ops.h. Plain C restatements; test infrastructure only. */
#include "et_oracle_ops.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

static int fail(char* err, size_t err_len, const char* message) {
    if (err != NULL && err_len != 0) snprintf(err, err_len, "%s", message);
    return -1;
}

/* composed.rs:1469-1486 */
void et_oracle_rms_norm(const float* x, const float* weight, double eps, float* out, size_t rows,
                        size_t columns) {
    for (size_t row = 0; row < rows; row++) {
        const float* in = x + row * columns;
        double mean_square = 0.0;
        for (size_t i = 0; i < columns; i++) mean_square += (double)in[i] * (double)in[i];
        const double scale = 1.0 / sqrt(mean_square / (double)columns + eps);
        for (size_t i = 0; i < columns; i++) {
            const double w = weight != NULL ? (double)weight[i] : 1.0;
            out[row * columns + i] = (float)((double)in[i] * scale * w);
        }
    }
}

/* composed.rs:2683-2729, checks :2742-2754 */
int et_oracle_rotary(const float* x, const uint32_t* offsets, size_t offsets_len, double theta,
                     double sign, int layout, float* out, size_t batch, size_t rows, size_t steps,
                     size_t head_dim, char* err, size_t err_len) {
    if (head_dim % 2 != 0)
        return fail(err, err_len, "rotary: expected a float rank >= 2 tensor with even head dimension");
    if (offsets_len != 1 && offsets_len != batch) {
        char message[96];
        snprintf(message, sizeof message, "rotary embedding: %zu offsets for batch %zu", offsets_len, batch);
        return fail(err, err_len, message);
    }
    if (batch == 0 || rows % batch != 0) return fail(err, err_len, "rotary: rows are not a multiple of the batch");
    const size_t rows_per_batch = rows / batch, half = head_dim / 2;
    for (size_t row = 0; row < rows; row++) {
        const size_t offset = offsets_len == 1 ? offsets[0] : offsets[row / rows_per_batch];
        for (size_t step = 0; step < steps; step++) {
            const size_t base = (row * steps + step) * head_dim;
            for (size_t index = 0; index < half; index++) {
                const double angle =
                    sign * (double)(offset + step) * pow(theta, -2.0 * (double)index / (double)head_dim);
                const double s = sin(angle), c = cos(angle);
                const size_t first = layout == 0 ? base + index : base + 2 * index;
                const size_t second = layout == 0 ? base + half + index : base + 2 * index + 1;
                const double a = (double)x[first], b = (double)x[second];
                out[first] = (float)(a * c - b * s);
                out[second] = (float)(b * c + a * s);
            }
        }
    }
    return 0;
}

void et_oracle_silu_mul(const float* gate, const float* up, float* out, size_t count) {
    for (size_t i = 0; i < count; i++) {
        const float half = gate[i] / 2.0f;            /* Tensor.ts:1242-1243 */
        const float t = tanhf(half);                  /* ops.rs:919 */
        const float sigmoid = t / 2.0f + 0.5f;        /* Tensor.ts:1244 */
        const float silu = gate[i] * sigmoid;         /* Tensor.ts:1539 */
        out[i] = silu * up[i];
    }
}

void et_oracle_add(const float* a, const float* b, float* out, size_t count) {
    for (size_t i = 0; i < count; i++) out[i] = a[i] + b[i];
}

/* sampling.rs:86-103 */
int et_oracle_argmax(const float* logits, size_t rows, size_t columns, uint32_t* out, char* err,
                     size_t err_len) {
    if (columns == 0) return fail(err, err_len, "sample: logits must be non-empty");
    for (size_t row = 0; row < rows; row++) {
        size_t selected = 0;
        double best = -INFINITY;
        for (size_t token = 0; token < columns; token++) {
            const double value = (double)logits[row * columns + token];
            if (!isfinite(value)) {
                char message[96];
                snprintf(message, sizeof message, "sample: logit %zu is not finite", token);
                return fail(err, err_len, message);
            }
            if (value > best) {
                best = value;
                selected = token;
            }
        }
        out[row] = (uint32_t)selected;
    }
    return 0;
}

/* indexing.rs:162-183 for a row-major table selected along dimension 0 */
int et_oracle_gather_rows(const void* table, size_t table_rows, size_t row_bytes,
                          const int64_t* indexes, size_t count, void* out, char* err,
                          size_t err_len) {
    for (size_t p = 0; p < count; p++) {
        if (indexes[p] < 0 || (uint64_t)indexes[p] >= table_rows) {
            char message[128];
            snprintf(message, sizeof message, "index_select: index %lld is out of bounds for extent %zu",
                     (long long)indexes[p], table_rows);
            return fail(err, err_len, message);
        }
        memcpy((char*)out + p * row_bytes, (const char*)table + (size_t)indexes[p] * row_bytes, row_bytes);
    }
    return 0;
}
