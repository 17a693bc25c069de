/*
 * CPU oracle for the small operators on the decode critical path next to the
 * quantized contraction. TEST INFRASTRUCTURE ONLY, like et_oracle.h.
 *
 * Pin status (tests/test_oracle_ops_pins.py):
 *   et_oracle_rms_norm    rms_norm_forward_into_impl (crates/runtime-cpu/src/composed.rs:1457-1487):
 *                         the reference's test vectors (packages/core/test/Tensor.test.ts:462-481)
 *                         against the closed form evaluated in numpy f64; unit weight and a
 *                         constant row give sign(x) / sqrt(1 + eps / x^2) exactly in f64
 *   et_oracle_rotary      rotary_forward_into_impl (composed.rs:2683-2729): the reference's test
 *                         (composed.rs:6393-6466: both layouts, inverse rotation, rank-2 input) at
 *                         its 2e-6; norm preservation of every pair; angle 0 is the identity;
 *                         per-batch offsets against one call per batch entry
 *   et_oracle_silu_mul    Tensor.silu (packages/core/src/Tensor.ts:1537-1540) over Tensor.sigmoid
 *                         (:1240-1245: tanh(x / 2) / 2 + 1 / 2, every step rounded to f32, tanh =
 *                         the platform's f32 tanh, crates/runtime-cpu/src/ops.rs:919) times `up`:
 *                         against x / (1 + exp(-x)) * up in f64 within 1e-6 relative. The last
 *                         bits depend on the platform's tanhf: PARITY UNPINNED at the bit level.
 *   et_oracle_argmax      sample_logits with temperature 0 (crates/runtime/src/sampling.rs:86-103):
 *                         the reference's tie test ([1, 4, 4, 2] -> 1, :223-238), numpy argmax on
 *                         random rows, the non-finite error message
 *   et_oracle_add         elementwise f32 sum (the residual connections; ops.rs binary add): IEEE
 *                         addition, identical to numpy's
 *   et_oracle_gather_rows index_select along dimension 0 (crates/runtime-cpu/src/indexing.rs:152-187):
 *                         numpy fancy indexing; the out-of-bounds message
 */
#ifndef ET_ORACLE_OPS_H
#define ET_ORACLE_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* out[r, i] = f32(x[r, i] * (1 / sqrt(mean(x[r]^2) + eps)) * weight[i]) in f64; weight may be NULL. */
void et_oracle_rms_norm(const float* x, const float* weight, double eps, float* out, size_t rows,
                        size_t columns);

/* x and out are [rows, steps, head_dim]; the batch entry of a row is row / (rows / batch);
 * offsets has 1 or `batch` entries. layout 0 = HalfSplit (i, i + d/2), 1 = InterleavedPairs
 * (2i, 2i + 1). Returns 0, or -1 with the reference's message. */
int et_oracle_rotary(const float* x, const uint32_t* offsets, size_t offsets_len, double theta,
                     double sign, int layout, float* out, size_t batch, size_t rows, size_t steps,
                     size_t head_dim, char* err, size_t err_len);

/* out = (gate * (tanhf(gate / 2) / 2 + 0.5)) * up, every operation rounded to f32. */
void et_oracle_silu_mul(const float* gate, const float* up, float* out, size_t count);

/* out = a + b, f32. */
void et_oracle_add(const float* a, const float* b, float* out, size_t count);

/* Greedy token per row; 0, or -1 with "sample: logit {token} is not finite" for the first row
 * that holds one. */
int et_oracle_argmax(const float* logits, size_t rows, size_t columns, uint32_t* out, char* err,
                     size_t err_len);

/* out[p, :] = table[indexes[p], :] for rows of `row_bytes` bytes; 0, or -1 with
 * "index_select: index {id} is out of bounds for extent {rows}". */
int et_oracle_gather_rows(const void* table, size_t table_rows, size_t row_bytes,
                          const int64_t* indexes, size_t count, void* out, char* err,
                          size_t err_len);

#ifdef __cplusplus
}
#endif
#endif
