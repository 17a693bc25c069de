/*
 * CPU oracle for paged key/value-cache attention (the decode neighbour of the
 * quantized contraction). TEST INFRASTRUCTURE ONLY, like et_oracle.h.
 *
 * Restates kv_attention_into (crates/runtime-cpu/src/napi/mod.rs:3320-3544) with
 * the cursor arithmetic of kv_prepare (:3568-3615). Block allocation stays with
 * the caller: the block table comes in already sized.
 *
 * Pin status:
 *   et_oracle_f32_to_fp16     all finite and special f32 patterns of a 2^20 sweep plus edge
 *                             cases against numpy float32 -> float16 (round to nearest even,
 *                             what half::f16::from_f32 implements)
 *   et_oracle_f32_to_bf16     a 2^20 sweep plus edge cases against torch's float32 -> bfloat16
 *                             (round to nearest even, what half::bf16::from_f32 implements)
 *   bf16 / u8 tiers           the reference tests them only through a whole model (packages/core/test/
 *                             Inference.test.ts:509-550: logits of a bf16 / int8 pool within 6e-2 /
 *                             1e-1 of the f32 model's), so here: attention over such a pool against
 *                             the f32 pool on the same inputs within the quantisation step;
 *                             closed forms: a row of equal magnitudes stores +-127 and scale
 *                             max / 127 + 1e-12, dequantised values are within half a step of
 *                             the input, halves round away from zero; PARITY UNPINNED by a
 *                             reference vector: its tests hold none for this tier
 *   et_oracle_kv_attention    the reference's own test (napi/mod.rs:4963-5051: one slot,
 *                             cursor 0, advance 3, two kv heads of width 4, block size 4,
 *                             q = 0..47, k = 0.24.., v = 0.48.., scale 0.5) against an
 *                             independent causal softmax attention in numpy f64 at the
 *                             reference's 1e-6; closed forms (equal scores -> mean of V, one
 *                             position -> that V row, shift invariance of the scores);
 *                             paging (permuted block tables give the same output); windowing
 *                             against the dense formula; inactive slots stay zero
 */
#ifndef ET_ORACLE_KV_H
#define ET_ORACLE_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* binary32 -> binary16 bits, round to nearest even (pool.rs:72-79 stores through f16::from_f32). */
uint16_t et_oracle_f32_to_fp16(float value);

/* binary32 -> bfloat16 bits, round to nearest even (bf16::from_f32). */
uint16_t et_oracle_f32_to_bf16(float value);

/* slab_dtype: 0 = f32, 2 = f16, 3 = bf16, 4 = u8 - the int8-quantized tier, which needs
 * et_oracle_kv_attention_scaled (the DType order of crates/runtime/src/dtype.rs:13-21). Slabs are [max_tokens, kv_heads, width].
 * block_table[slot * table_stride + i] = physical block of logical block i of that slot.
 * q is [batch, query_heads, tokens, width], k and v [batch, kv_heads, tokens, width], all f32,
 * out like q. context_window is the pool's sliding window (kv_prepare's `start`, :3599), window
 * the operator's own (:3482-3483); 0 means none for either. Writes the new rows first, then attends.
 * Returns 0, or -1 with a message in err. */
int et_oracle_kv_attention(int slab_dtype, void* k_slab, void* v_slab, size_t max_tokens,
                           size_t kv_heads, size_t width, size_t block_size,
                           const uint32_t* block_table, size_t table_stride,
                           const uint32_t* cursors, const uint32_t* advances, size_t batch,
                           size_t active_batch, size_t query_heads, size_t tokens, const float* q,
                           const float* k, const float* v, double scale, size_t context_window, size_t window,
                           float* out, char* err, size_t err_len);

/* The same with the scale slabs of the u8 tier ([max_tokens, kv_heads] f32 each, written with the
 * rows; NULL for the other dtypes): napi/mod.rs:3397-3437 (write) and :3467-3478 (read). */
int et_oracle_kv_attention_scaled(int slab_dtype, void* k_slab, void* v_slab, float* k_scales, float* v_scales,
                                  size_t max_tokens, size_t kv_heads, size_t width, size_t block_size,
                                  const uint32_t* block_table, size_t table_stride,
                                  const uint32_t* cursors, const uint32_t* advances, size_t batch,
                                  size_t active_batch, size_t query_heads, size_t tokens, const float* q,
                                  const float* k, const float* v, double scale, size_t context_window,
                                  size_t window, float* out, char* err, size_t err_len);

#ifdef __cplusplus
}
#endif
#endif
