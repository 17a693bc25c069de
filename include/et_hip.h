/*
 * et_hip.h - C ABI of the MI355X (gfx950) quantized-GGUF matmul backend.
 *
 * This is the boundary a `runtime-hip` backend crate binds over FFI. It mirrors
 * the per-operator free-function pair every backend crate of the reference
 * exposes to its executable: a *plan* step that validates geometry and freezes
 * an immutable requirements object, and an allocation-free *execute* step that
 * re-validates against the plan and runs (CPU) or enqueues (GPU):
 *
 *   reference (crates/runtime-cpu/src/quantized.rs)        this header
 *   ------------------------------------------------       ---------------------------------
 *   linear_requirements            :297-336                et_hip_linear_requirements
 *   linear_into                    :419-499                et_hip_linear_into
 *   embedding_requirements         :340-365                et_hip_embedding_requirements
 *   embedding_into                 :546-616                et_hip_embedding_into (+ _status_check)
 *   GgmlKQuant::encoded_row_bytes  crates/runtime/src/gguf.rs:245-250   et_hip_encoded_row_bytes
 *   warm_linear_exact              crates/runtime-metal/src/quantized.rs:1226   (done inside the plan step)
 *   isAvailable                    packages/backend-cpu/src/internal/native-addon.ts:266   et_hip_is_available
 *
 * Conventions
 *   - All `data` pointers are DEVICE pointers to caller-owned, pre-allocated
 *     memory. No entry point allocates or frees device memory; execute entry
 *     points allocate nothing at all. Scratch comes in as `workspace`.
 *   - Execute entry points ENQUEUE on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream) and return without synchronising.
 *   - Return value 0 = ok; otherwise an et_status whose categories follow the
 *     reference's BackendError taxonomy (crates/runtime/src/error.rs:25-68).
 *     The message, worded like the reference's `Err(String)`, is available
 *     from et_hip_last_error() on the calling thread.
 *   - `cancel` is an optional host flag (the reference's CancellationFlag,
 *     crates/runtime/src/cancellation.rs:18-35). It is polled before anything
 *     is enqueued and again between the launches of one call (quantiser,
 *     contraction, reduction; one GEMV launch after the other), where the
 *     reference polls between rows and blocks (quantized.rs:451,459); a set
 *     flag yields ET_ERR_CANCELLED / "operation aborted". Kernels already
 *     enqueued are not pre-empted.
 *   - No C++ exception crosses this boundary.
 */
#ifndef ET_HIP_H
#define ET_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGML tensor type codes. 10..14 = the reference's GgmlKQuant
 * (crates/runtime/src/gguf.rs:199-205, codes :278-291). 2 and 8 are the legacy
 * ggml block formats, which the reference does not implement. */
typedef enum {
    ET_CODEC_Q4_0 = 2,
    ET_CODEC_Q8_0 = 8,
    ET_CODEC_Q2_K = 10,
    ET_CODEC_Q3_K = 11,
    ET_CODEC_Q4_K = 12,
    ET_CODEC_Q5_K = 13,
    ET_CODEC_Q6_K = 14
} et_codec;

/* Element types, in the order of the reference's DType (crates/runtime/src/dtype.rs:13-21). */
typedef enum {
    ET_DTYPE_F32 = 0,
    ET_DTYPE_F64 = 1,
    ET_DTYPE_F16 = 2,
    ET_DTYPE_BF16 = 3,
    ET_DTYPE_U8 = 4,
    ET_DTYPE_U32 = 5,
    ET_DTYPE_I64 = 6
} et_dtype;

typedef enum {
    ET_OK = 0,
    ET_ERR_UNSUPPORTED = 1, /* geometry / dtype / layout the operator does not accept */
    ET_ERR_EXECUTION = 2,   /* a HIP call failed, or operands do not match the frozen plan */
    ET_ERR_CANCELLED = 3,   /* "operation aborted" */
    ET_ERR_UNAVAILABLE = 4, /* no usable gfx950 device */
    ET_ERR_INVALID = 5      /* NULL where a pointer is required, unknown enum value */
} et_status;

/* How activations enter the contraction. */
typedef enum {
    ET_ACT_F32 = 0, /* f32 activations, f32 accumulate; tolerance 1e-3 against the CPU path */
    ET_ACT_INT8 = 1 /* activations quantised on the fly to int8 per 32 columns with an f32
                       absmax scale, int8 MFMA, f32 block-scale epilogue; tolerance 2e-2.
                       The reference has no such mode. Codecs: Q8_0, Q4_0 and Q4_K (whole
                       256-column stages); a plan for Q2_K, Q3_K, Q5_K or Q6_K in this mode is
                       refused with ET_ERR_UNSUPPORTED ("int8 activation mode is not available
                       for ...") - their batches run in ET_ACT_F32. */
} et_activation_mode;

/* A strided view of caller-owned storage, in ELEMENTS - the reference's Tensor
 * = buffer + Layout{shape, strides, offset} (crates/runtime/src/layout.rs).
 * `strides == NULL` means row-major contiguous. */
typedef struct {
    const void* data;       /* device pointer to the start of the STORAGE (not of the view) */
    int32_t dtype;          /* et_dtype */
    int32_t rank;
    const uint64_t* shape;  /* host array, `rank` entries */
    const uint64_t* strides; /* host array, `rank` entries, or NULL */
    uint64_t offset;        /* view offset into the storage */
} et_tensor;

typedef struct et_linear_plan et_linear_plan;       /* opaque, immutable, host memory */
typedef struct et_embedding_plan et_embedding_plan; /* opaque, immutable, host memory */

/* ---- availability and codec tables -------------------------------------- */

/* 1 when a gfx950 device is visible and the library's kernels can run on it.
 * cf. isAvailable (packages/backend-cpu/src/internal/native-addon.ts:266). */
int et_hip_is_available(void);

/* "Q4_K", ... or NULL. cf. GgmlKQuant::name (crates/runtime/src/gguf.rs:208-217). */
const char* et_hip_codec_name(int32_t codec);
/* Values per block (256 for K-quants, 32 for Q8_0 / Q4_0); 0 = unknown codec. */
uint64_t et_hip_block_values(int32_t codec);
/* Bytes per block. cf. block_bytes (crates/runtime-cpu/src/quantized.rs:60-68). */
uint64_t et_hip_block_bytes(int32_t codec);
/* Packed bytes of one logical row; 0 when `columns` is not a whole number of
 * blocks or the product overflows. cf. GgmlKQuant::encoded_row_bytes
 * (crates/runtime/src/gguf.rs:245-250). */
uint64_t et_hip_encoded_row_bytes(int32_t codec, uint64_t columns);

/* ---- quantized_linear ---------------------------------------------------- */

/* Plan step = linear_requirements (crates/runtime-cpu/src/quantized.rs:297-336)
 * + kernel selection by (codec, vectors, mode) (cf. linear_kernel_kind,
 * crates/runtime-metal/src/quantized.rs:1204-1220).
 *   input  f32, rank >= 2, trailing width = columns, any strides
 *   weight u8, exactly [rows, encoded_row_bytes], contiguous, offset 0
 *   bias   NULL or f32 [rows]
 * Only metadata is read; `data` pointers may be NULL here. */
int et_hip_linear_requirements(const et_tensor* input, const et_tensor* weight,
                               const et_tensor* bias, int32_t codec, uint64_t rows,
                               uint64_t columns, int32_t activation_mode, et_linear_plan** out);

void et_hip_linear_plan_destroy(et_linear_plan* plan);

/* Plan queries (QuantizedRequirements, crates/runtime-cpu/src/quantized.rs:35-42;
 * LinearRequirements, crates/runtime-metal/src/quantized.rs:45-68). */
int32_t et_hip_linear_plan_output_rank(const et_linear_plan* plan);
/* Writes output_rank entries. */
void et_hip_linear_plan_output_shape(const et_linear_plan* plan, uint64_t* shape);
uint64_t et_hip_linear_plan_vectors(const et_linear_plan* plan);
uint64_t et_hip_linear_plan_output_bytes(const et_linear_plan* plan);
/* Device scratch the execute step needs (int8 activations, gathered strided
 * input); the caller allocates at least this many bytes, 256-byte aligned. May be 0. */
uint64_t et_hip_linear_plan_workspace_bytes(const et_linear_plan* plan);
/* Name of the selected kernel variant, for profiles and diagnostics. */
const char* et_hip_linear_plan_kernel(const et_linear_plan* plan);
/* Algorithmic bytes of one execution: packed weight + f32 input + f32 output (+ bias). */
uint64_t et_hip_linear_plan_algorithmic_bytes(const et_linear_plan* plan);

/* Execute step = linear_into (crates/runtime-cpu/src/quantized.rs:419-499):
 * re-validates the operands against the plan (validate_linear_execution,
 * :367-415), then enqueues. destination: f32, contiguous, offset 0, shape =
 * input shape with the trailing dim replaced by rows. */
int et_hip_linear_into(const et_linear_plan* plan, const et_tensor* input, const et_tensor* weight,
                       const et_tensor* bias, const et_tensor* destination, void* workspace,
                       uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel);

/* Raw-pointer form of the same pair for callers that hold dense buffers:
 * x is [vectors, columns] f32 with `x_row_stride` elements between vectors,
 * y is dense [vectors, rows] f32. Same validation of (codec, rows, columns). */
int et_hip_linear_plan_create(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors,
                              int32_t has_bias, int32_t activation_mode, et_linear_plan** out);
int et_hip_linear_enqueue(const et_linear_plan* plan, const float* x, uint64_t x_row_stride,
                          const uint8_t* weight, const float* bias, float* y, void* workspace,
                          uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel);

/* et_hip_linear_enqueue without a workspace argument: the scratch memory the kernels need
 * (activation tiles, K-share partials, the dense copy of strided rows) is a device array inside the
 * library, ET_HIP_STATIC_WORKSPACE_BYTES per GPU, held from its first use on that GPU until the
 * process ends. It has no counterpart in the reference; it exists for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The call allocates nothing and frees nothing. A plan whose et_hip_linear_plan_workspace_bytes
 * exceeds the array is refused (ET_ERR_UNSUPPORTED, "... the static workspace holds ..."): such
 * callers bring their own workspace to et_hip_linear_enqueue. Every call on a GPU uses the same
 * array: calls that overlap in time on one GPU race on it - serialise them (one stream, or events).
 * Results are those of et_hip_linear_enqueue, bit for bit. The array's device address is looked up
 * when a plan is made on that GPU (et_hip_linear_plan_create / et_hip_linear_requirements), not by
 * this call, so that the call may be recorded into a stream capture: make the plan, with the GPU
 * current, before the capture begins. */
#define ET_HIP_STATIC_WORKSPACE_BYTES (16u << 20)
int et_hip_linear_enqueue_static_workspace(const et_linear_plan* plan, const float* x, uint64_t x_row_stride,
                                           const uint8_t* weight, const float* bias, float* y, void* stream,
                                           const volatile int32_t* cancel);

/* Contractions that share their activations (q / k / v, gate / up of a decode step) can share the
 * quantised form the matrix-core kernels consume: prepare it once, then enqueue every plan of the
 * same columns, vectors and activation mode from it. `residual` (dense [vectors, rows], may be y
 * itself) is added to the result in the kernel's epilogue, which saves the separate sum of a
 * residual connection. Only plans whose kernel runs on the matrix cores have a prepared form
 * (et_hip_linear_plan_prepared_input_bytes > 0); the others return ET_ERR_UNSUPPORTED here and
 * use et_hip_linear_enqueue. No counterpart in the reference, whose executor runs one operator
 * at a time. */
uint64_t et_hip_linear_plan_prepared_input_bytes(const et_linear_plan* plan);
int et_hip_linear_prepare_input(const et_linear_plan* plan, const float* x, uint64_t x_row_stride,
                                void* prepared, uint64_t prepared_bytes, void* stream);
/* The prepared input of an operator's RESULT, without the operator's own launch or its f32 output:
 * the activations are computed element by element while they are quantised, with the arithmetic of
 * the stand-alone operator, so the prepared bytes are those of the operator followed by
 * et_hip_linear_prepare_input. Kinds: ET_PREPARE_RMS_NORM, rms_norm(x) * second (second = the
 * weight [columns], or NULL; et_hip_rms_norm_into, crates/runtime-cpu/src/composed.rs:1491-1533),
 * and ET_PREPARE_SILU_MUL, silu(x) * second (second = the up projection, laid out like x;
 * et_hip_silu_mul_into). ET_PREPARE_PLAIN is et_hip_linear_prepare_input. Only plans with
 * et_hip_linear_plan_fused_prepare(plan) != 0 take the first two; the others return
 * ET_ERR_UNSUPPORTED and the caller runs the operator itself. No counterpart in the reference,
 * whose executor runs one operator at a time. */
typedef enum { ET_PREPARE_PLAIN = 0, ET_PREPARE_RMS_NORM = 1, ET_PREPARE_SILU_MUL = 2 } et_prepare_kind;
typedef struct et_prepare_source {
    int32_t kind;           /* et_prepare_kind */
    const float* x;         /* [vectors, columns] f32, rows x_row_stride elements apart, 16-byte aligned */
    uint64_t x_row_stride;
    const void* second;     /* see the kinds above; f32 [..] */
    double eps;             /* ET_PREPARE_RMS_NORM */
    int32_t second_dtype;   /* ET_DTYPE_F32 (0), or ET_DTYPE_F16 for an rms norm weight held as half floats: it is
                               widened on use, the cast the reference's graph puts in front of the operator */
} et_prepare_source;
int et_hip_linear_plan_fused_prepare(const et_linear_plan* plan);
int et_hip_linear_prepare_input_from(const et_linear_plan* plan, const et_prepare_source* source,
                                     void* prepared, uint64_t prepared_bytes, void* stream);
/* Up to four contractions from the same prepared input in ONE launch: the q / k / v projections of
 * a decode step are three small matrices, each of which alone leaves most of the device idle.
 * The grid runs over the 64-row tiles of all members; results are those of
 * et_hip_linear_enqueue_prepared per member up to the order of the K shares (the same order on
 * every run). Every plan must have et_hip_linear_plan_fused_prepare(plan) != 0 and share columns
 * and vectors; weights / biases / residuals / ys hold one device pointer per plan (biases and
 * residuals may be NULL, or hold NULL entries). The workspace is the group's own:
 * et_hip_linear_group_workspace_bytes. No counterpart in the reference. */
int et_hip_linear_group_workspace_bytes(const et_linear_plan* const* plans, uint32_t count, uint64_t* bytes);
int et_hip_linear_enqueue_prepared_group(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                         const uint8_t* const* weights, const float* const* biases,
                                         const float* const* residuals, float* const* ys, void* workspace,
                                         uint64_t workspace_bytes, void* stream,
                                         const volatile int32_t* cancel);

/* et_hip_linear_enqueue_prepared_group for a group that shares K over workgroups, WITHOUT the launch
 * that sums the shares: `workspace` keeps them, `layout` says where, and the launch that takes the
 * results (et_hip_kv_attention_projected_into for the q / k / v projections of a decode step) sums
 * the rows it needs itself, in share order - one launch less. Biases and residuals are the summing
 * launch's business. ET_ERR_UNSUPPORTED for a group that does not share K
 * (et_hip_linear_group_shares_layout: count <= 1). No counterpart in the reference. */
#define ET_HIP_LINEAR_GROUP_MOST 4
typedef struct et_group_shares {
    const float* shares;   /* share s of vector m, launch row n: shares[(s * vectors + m) * launch_rows + n] */
    uint32_t count;        /* K shares; <= 1: the group does not share K */
    uint64_t vectors;
    uint64_t launch_rows;  /* the members' rows, each member rounded up to whole tiles */
    uint64_t first_row[ET_HIP_LINEAR_GROUP_MOST];  /* launch row of row 0 of plans[i] */
} et_group_shares;
/* The layout alone (shares = NULL): what the plans decide, for a caller that chooses its path. */
int et_hip_linear_group_shares_layout(const et_linear_plan* const* plans, uint32_t count,
                                      et_group_shares* layout);
int et_hip_linear_enqueue_prepared_group_shares(const et_linear_plan* const* plans, uint32_t count,
                                                const void* prepared, const uint8_t* const* weights,
                                                void* workspace, uint64_t workspace_bytes,
                                                et_group_shares* layout, void* stream,
                                                const volatile int32_t* cancel);

int et_hip_linear_enqueue_prepared(const et_linear_plan* plan, const void* prepared,
                                   const uint8_t* weight, const float* bias, const float* residual,
                                   float* y, void* workspace, uint64_t workspace_bytes, void* stream,
                                   const volatile int32_t* cancel);

/* et_hip_linear_enqueue_prepared, then the prepared input of rms_norm(y) * norm_weight for the
 * contraction that comes next (`next`: columns = this plan's rows, the same vectors,
 * et_hip_linear_plan_fused_prepare(next) != 0) - the residual stream of a transformer layer: y = x W
 * + residual, then the next block's norm. y and next_prepared receive the bytes of
 * et_hip_linear_enqueue_prepared followed by et_hip_linear_prepare_input_from(ET_PREPARE_RMS_NORM).
 * Where this plan shares K over workgroups, the launch that would only sum the shares sums them,
 * writes y, norms and quantises: one launch less. Other plans run the two steps one after the
 * other. norm_weight: [rows] f32 or f16 (norm_weight_dtype: ET_DTYPE_F32 / ET_DTYPE_F16; halves are
 * widened on use) or NULL. No counterpart in the reference, whose executor runs one operator at a time. */
int et_hip_linear_enqueue_prepared_then_norm(const et_linear_plan* plan, const void* prepared,
                                             const uint8_t* weight, const float* bias, const float* residual,
                                             float* y, void* workspace, uint64_t workspace_bytes,
                                             const et_linear_plan* next, const void* norm_weight,
                                             int32_t norm_weight_dtype, double eps, void* next_prepared,
                                             uint64_t next_prepared_bytes, void* stream,
                                             const volatile int32_t* cancel);

/* ---- quantized_embedding (= bit-exact dequantisation of selected rows) ---- */

/* Plan step = embedding_requirements (crates/runtime-cpu/src/quantized.rs:340-365).
 * indexes: u32 or i64, any shape and strides. */
int et_hip_embedding_requirements(const et_tensor* indexes, const et_tensor* weight, int32_t codec,
                                  uint64_t rows, uint64_t columns, et_embedding_plan** out);
void et_hip_embedding_plan_destroy(et_embedding_plan* plan);
int32_t et_hip_embedding_plan_output_rank(const et_embedding_plan* plan);
void et_hip_embedding_plan_output_shape(const et_embedding_plan* plan, uint64_t* shape);
uint64_t et_hip_embedding_plan_output_bytes(const et_embedding_plan* plan);

/* Execute step = embedding_into (crates/runtime-cpu/src/quantized.rs:546-616).
 * destination: f32 [indexes.., columns], contiguous, offset 0. Every value is
 * bit-identical to the CPU decode. An index outside 0..rows cannot fail the
 * call (the kernel is already enqueued): the row is skipped and the device
 * `status` block (ET_HIP_STATUS_BYTES bytes, zeroed by this call on `stream`)
 * records it, as the reference's Metal backend does
 * (crates/runtime-metal/src/quantized.rs:1103-1129). `status` may be NULL when
 * `indexes` is NULL (= decode every row in order). */
#define ET_HIP_STATUS_BYTES 16
int et_hip_embedding_into(const et_embedding_plan* plan, const et_tensor* indexes,
                          const et_tensor* weight, const et_tensor* destination, void* status,
                          void* stream, const volatile int32_t* cancel);
/* After the stream has completed and `status` has been copied to the host:
 * 0, or ET_ERR_EXECUTION with "quantized_embedding: index {i} is outside 0..{rows}"
 * (crates/runtime-cpu/src/quantized.rs:570-583). */
int et_hip_embedding_status_check(const et_embedding_plan* plan, const void* status_host);

/* Raw-pointer dequantisation of whole rows: out[r, :] = decode(W[r, :]) for
 * r in [0, rows). Bit-exact. cf. decode_block (crates/runtime-cpu/src/quantized.rs:90-111). */
int et_hip_dequantize_rows(int32_t codec, uint64_t rows, uint64_t columns, const uint8_t* weight,
                           float* out, void* stream);

/* ---- paged key/value-cache attention ---------------------------------------
 *
 * The decode neighbour of quantized_linear: kv_attention_into
 * (crates/runtime-cpu/src/napi/mod.rs:3320-3544). The caller keeps what the
 * reference keeps on the host - block allocation, eviction, the cursors'
 * advance between steps (kv_prepare / kv_evict, :3568-3627) - and hands over
 * the state of one layer as device arrays. */

/* One layer of a KvContext (napi/mod.rs:2656-2664) over its pool (PoolInner,
 * :2501-2513; slabs crates/runtime-cpu/src/pool.rs). All pointers are device
 * pointers. */
typedef struct {
    void* k_slab;                /* [max_tokens, kv_heads, head_dim] of slab_dtype; written and read */
    void* v_slab;
    int32_t slab_dtype;          /* ET_DTYPE_F32, ET_DTYPE_F16, ET_DTYPE_BF16, or ET_DTYPE_U8: the
                                    int8-quantized tier (napi/mod.rs:3397-3437), byte = round(x / scale) +
                                    128 with one f32 scale per row and head in k_scales / v_scales */
    uint64_t max_tokens;         /* pool.max_tokens */
    uint64_t kv_heads;           /* pool.kv_heads */
    uint64_t head_dim;           /* pool.head_dim */
    uint64_t block_size;         /* pool.block_size */
    const uint32_t* block_table; /* [slots, table_stride]: SeqState.blocks of every slot, already
                                    grown to cover cursor + advance */
    uint64_t table_stride;
    const uint32_t* cursors;     /* [slots] SeqState.cursor */
    const uint32_t* advances;    /* [slots] SeqState.advance */
    uint64_t slots;              /* context.slots.len() = the batch of q */
    uint64_t active_batch;       /* context.active_batch: slots beyond it get zeros */
    uint64_t context_window;     /* context.window, 0 = none */
    uint64_t max_context;        /* host-side upper bound of cursor + advance over the active slots;
                                    it sizes the launch and the workspace */
    float* k_scales;             /* [max_tokens, kv_heads] f32, ET_DTYPE_U8 only (pool.scales[2 * layer],
                                    napi/mod.rs:3727-3734); written with the rows; NULL otherwise */
    float* v_scales;
} et_kv_layer;

/* Device scratch et_hip_kv_attention_into needs for these sizes (partial results
 * of the context splits); may be 0. */
uint64_t et_hip_kv_attention_workspace_bytes(const et_kv_layer* layer, uint64_t query_heads,
                                             uint64_t tokens);

/* = kv_attention_into (napi/mod.rs:3320-3544): appends `advance` rows of k / v
 * per active slot to the slabs, then attends causally over each slot's cached
 * context (grouped-query: query head h reads kv head h / (query_heads /
 * kv_heads)) with softmax(q.k * scale) in f32 (the reference accumulates in
 * f64; results agree to 1e-4).
 *   q [.., query_heads, tokens, head_dim], k and v [.., kv_heads, tokens, head_dim],
 *   destination like q: f32, rank >= 4, contiguous; the leading dims multiply to `slots`.
 *   window: the operator's own sliding window, 0 = none.
 * The cursors live on the device, so the checks of kv_prepare that depend on
 * them cannot fail this call: a slot that fails one is skipped and the device
 * `status` block (8 bytes per slot, every word written by this call) records it
 * for et_hip_kv_attention_status_check. */
#define ET_HIP_KV_STATUS_BYTES(slots) (8 * (uint64_t)(slots))
int et_hip_kv_attention_into(const et_kv_layer* layer, const et_tensor* q, const et_tensor* k,
                             const et_tensor* v, double scale, uint64_t window,
                             const et_tensor* destination, void* workspace,
                             uint64_t workspace_bytes, void* status, void* stream,
                             const volatile int32_t* cancel);
/* et_hip_kv_attention_into for one token per slot, then the prepared input of the contraction that
 * takes the result as its activations (`consumer`: et_hip_linear_plan_fused_prepare != 0, vectors =
 * slots, columns = query_heads * head_dim - the output projection of a decode step): destination and
 * `prepared` receive the bytes of et_hip_kv_attention_into followed by et_hip_linear_prepare_input.
 * Where a workgroup of the attention kernel holds whole 256-column stages of a row and the context is
 * not split, it quantises them in its epilogue (one launch less); otherwise the quantiser launch
 * follows. No counterpart in the reference, whose executor runs one operator at a time. */
int et_hip_kv_attention_prepared_into(const et_kv_layer* layer, const et_tensor* q, const et_tensor* k,
                                      const et_tensor* v, double scale, uint64_t window,
                                      const et_tensor* destination, void* workspace,
                                      uint64_t workspace_bytes, void* status, const et_linear_plan* consumer,
                                      void* prepared, uint64_t prepared_bytes, void* stream,
                                      const volatile int32_t* cancel);
/* et_hip_kv_attention_prepared_into for a decode step whose q, k and v are still the unsummed K
 * shares of their projections (et_hip_linear_enqueue_prepared_group_shares): every workgroup of the
 * attention kernel first sums the shares of the rows it needs in share order, adds the biases and
 * rotates q and k at `offsets` (rotary_forward_into's arithmetic, composed.rs:2683-2729) - the bytes
 * et_hip_linear_enqueue_prepared_group_then_rotary leaves in q, k and v - then appends and attends
 * as et_hip_kv_attention_into does with those tensors. One token per slot; destination
 * [.., query_heads, 1, head_dim]. `consumer` / `prepared` as in et_hip_kv_attention_prepared_into, or
 * NULL / NULL / 0. ET_ERR_UNSUPPORTED for geometries the streaming attention kernel does not take
 * (et_hip_kv_attention_kernel names another one): such callers sum and rotate first. No counterpart
 * in the reference, whose executor runs one operator at a time. */
typedef struct et_kv_projected {
    et_group_shares shares;            /* vectors = slots */
    uint32_t q_member, k_member, v_member;  /* which plans of the group are q, k and v */
    const float* q_bias;               /* [query_heads * head_dim] device floats, or NULL */
    const float* k_bias;               /* [kv_heads * head_dim], or NULL */
    const float* v_bias;
    const uint32_t* offsets;           /* rotary positions: DEVICE array of 1 or `slots` u32 (the cursors) */
    uint64_t offsets_len;
    double theta, sign;
    int32_t layout;                    /* et_rotary_layout */
} et_kv_projected;
int et_hip_kv_attention_projected_into(const et_kv_layer* layer, const et_kv_projected* projected,
                                       double scale, uint64_t window, const et_tensor* destination,
                                       void* workspace, uint64_t workspace_bytes, void* status,
                                       const et_linear_plan* consumer, void* prepared,
                                       uint64_t prepared_bytes, void* stream,
                                       const volatile int32_t* cancel);
/* After the stream has completed and `status` has been copied to the host: 0, or
 * ET_ERR_EXECUTION with the reference's message for the first failing slot, e.g.
 * "kv attention: advance {a} out of range for chunk length {tokens}"
 * (napi/mod.rs:3590-3594). */
int et_hip_kv_attention_status_check(const et_kv_layer* layer, uint64_t tokens,
                                     const void* status_host);
/* The commit of a step (crates/runtime-cpu/src/napi/mod.rs:4511-4517): cursor += advance for the
 * layer's active slots, on the device, after the step's last attention call - so that a decode loop
 * replays one captured graph per step without a host round trip. Writes layer->cursors (the caller's
 * array, as everything the struct points to). Layers that share their cursor array are committed by
 * one call. */
int et_hip_kv_commit(const et_kv_layer* layer, void* stream);

/* Name of the kernel variant these sizes select, for profiles and diagnostics. */
const char* et_hip_kv_attention_kernel(const et_kv_layer* layer, uint64_t query_heads,
                                       uint64_t tokens);

/* ---- the small operators of a decode step ---------------------------------
 *
 * RMS norm, rotary embedding, SiLU(gate) * up, greedy token selection and the
 * dense embedding lookup sit between the contractions of every decode step.
 * All take contiguous tensors and enqueue one kernel on `stream`. */

/* = rms_norm_forward_into (crates/runtime-cpu/src/composed.rs:1491-1533) for
 * f32: out = x * (1 / sqrt(mean(x^2) + eps)) * weight over the last dimension,
 * in f64, rounded once. weight: NULL or [columns], f32 - or f16, widened on use: the
 * reference wants the weight in the activations' type (composed.rs:700-705) and a model
 * whose norms are stored as half floats casts them in front of the operator; here the
 * operator reads the halves itself (the widening is exact, the result the same). */
int et_hip_rms_norm_into(const et_tensor* x, const et_tensor* weight, double eps,
                         const et_tensor* destination, void* stream);

/* RotaryLayout (the pairs one angle rotates): (i, i + d/2) or (2i, 2i + 1). */
typedef enum { ET_ROTARY_HALF_SPLIT = 0, ET_ROTARY_INTERLEAVED_PAIRS = 1 } et_rotary_layout;
/* = rotary_forward_into (composed.rs:2735-2772) for f32 [.., steps, head_dim]:
 * position = offset + step, angle = sign * position * theta^(-2i / head_dim),
 * in f64, rounded once. `offsets` is a DEVICE array of 1 or batch (= shape[0], 1
 * for rank 2) u32 entries - in a decode step, the kv cursors. */
int et_hip_rotary_into(const et_tensor* x, const uint32_t* offsets, uint64_t offsets_len,
                       double theta, double sign, int32_t layout, const et_tensor* destination,
                       void* stream);
/* The same for two tensors of one batch, steps and head_dim at the same offsets - the queries and
 * the keys of a decode step - in one launch; each result is et_hip_rotary_into's. */
int et_hip_rotary_pair_into(const et_tensor* x, const et_tensor* second, const uint32_t* offsets,
                            uint64_t offsets_len, double theta, double sign, int32_t layout,
                            const et_tensor* destination, const et_tensor* second_destination,
                            void* stream);
/* et_hip_linear_enqueue_prepared_group, then et_hip_rotary_into in place on the results of the
 * members whose bit is set in `members` (bit i = plans[i]), each seen as [vectors, rows / head_dim,
 * 1, head_dim] at offsets[0] or offsets[vector] - the q and k projections of a decode step at the
 * slots' cursors. The ys receive the bytes of the two steps. Where the group shares K over
 * workgroups, the launch that sums the shares also rotates (one launch less); other groups run the
 * steps one after the other. No counterpart in the reference, whose executor runs one operator at a
 * time. */
typedef struct et_rotary_after {
    uint32_t members;
    const uint32_t* offsets;   /* DEVICE array of 1 or `vectors` u32 */
    uint64_t offsets_len;
    double theta, sign;
    int32_t layout;            /* et_rotary_layout */
    uint64_t head_dim;
} et_rotary_after;
int et_hip_linear_enqueue_prepared_group_then_rotary(const et_linear_plan* const* plans, uint32_t count,
                                                     const void* prepared, const uint8_t* const* weights,
                                                     const float* const* biases, const float* const* residuals,
                                                     float* const* ys, void* workspace, uint64_t workspace_bytes,
                                                     const et_rotary_after* rotary, void* stream,
                                                     const volatile int32_t* cancel);

/* out = a + b, f32, same shapes (the residual connections; the reference's binary
 * add without broadcasting, crates/runtime-cpu/src/ops.rs). `destination` may be `a`. */
int et_hip_add_into(const et_tensor* a, const et_tensor* b, const et_tensor* destination,
                    void* stream);

/* out = silu(gate) * up with silu(x) = x * (tanh(x / 2) / 2 + 1 / 2), f32, every
 * step rounded (Tensor.silu over Tensor.sigmoid, packages/core/src/Tensor.ts:1537-1540,
 * :1240-1245; the reference builds it from four elementwise nodes). */
int et_hip_silu_mul_into(const et_tensor* gate, const et_tensor* up, const et_tensor* destination,
                         void* stream);

/* = sample_logits with temperature 0 (crates/runtime/src/sampling.rs:86-103) for
 * every row of f32 logits [.., vocabulary]: the largest logit, the lowest token
 * among equals. tokens: device u32 [rows]. workspace: device scratch of
 * et_hip_greedy_workspace_bytes(rows, vocabulary), 4-byte aligned (the rows are
 * scanned in chunks by many workgroups). A logit that is not finite cannot fail
 * the call; `status` (device, 4 bytes per row, written by the call) records it
 * for et_hip_greedy_status_check ("sample: logit {token} is not finite"). */
uint64_t et_hip_greedy_workspace_bytes(uint64_t rows, uint64_t vocabulary);
int et_hip_greedy_tokens_into(const et_tensor* logits, uint32_t* tokens, void* workspace,
                              uint64_t workspace_bytes, void* status, void* stream);
int et_hip_greedy_status_check(uint64_t rows, const void* status_host);

/* = index_select_into along dimension 0 (crates/runtime-cpu/src/indexing.rs:396-430)
 * of a [rows, width] table of any element type: destination[p, :] =
 * table[indexes[p], :] (the dense embedding lookup; f16 tables stay f16). An f32
 * destination for an f16 / bf16 table receives the rows widened (exact): the lookup and
 * the cast a model with a half-float table puts behind it, in one launch.
 * indexes: u32 or i64, any shape, contiguous; destination [count, width].
 * `status`: device, 8 bytes per index, written by the call; an index outside
 * the table leaves its row alone and et_hip_gather_rows_status_check returns
 * "index_select: index {id} is out of bounds for extent {rows}". */
int et_hip_gather_rows_into(const et_tensor* table, const et_tensor* indexes,
                            const et_tensor* destination, void* status, void* stream);
int et_hip_gather_rows_status_check(uint64_t table_rows, uint64_t count, const void* status_host);

/* ---- GGUF v3 files: the on-disk format that feeds the contraction ----------
 *
 * = parse_gguf / read_gguf_tensor_into (crates/runtime/src/gguf.rs:682-957,
 * :959-994): the header is parsed with the reference's validation, resource
 * limits and messages ("gguf: ..."); tensor payloads are validated for range and
 * overlap, not read. Beyond the reference's F32 and K-quant tensors, GGML type
 * codes 2 (Q4_0) and 8 (Q8_0) are accepted. Host calls; only the upload touches
 * the device. */
typedef struct et_gguf et_gguf; /* opaque; owns the open file */

/* ET_ERR_UNSUPPORTED = the file violates the format or a limit
 * (GgufParseError::Invalid), ET_ERR_EXECUTION = I/O failed, ET_ERR_CANCELLED. */
int et_hip_gguf_open(const char* path, const volatile int32_t* cancel, et_gguf** out);
void et_hip_gguf_close(et_gguf* file);
const char* et_hip_gguf_architecture(const et_gguf* file); /* general.architecture */

/* The metadata table in file order. Types are the GGUF value type codes: 0 u8, 1 i8,
 * 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array, 10 u64, 11 i64, 12 f64. */
uint64_t et_hip_gguf_metadata_count(const et_gguf* file);
int64_t et_hip_gguf_metadata_find(const et_gguf* file, const char* key); /* index or -1 */
const char* et_hip_gguf_metadata_key(const et_gguf* file, uint64_t index);
uint64_t et_hip_gguf_metadata_key_length(const et_gguf* file, uint64_t index); /* bytes; a key may hold NULs */
int32_t et_hip_gguf_metadata_type(const et_gguf* file, uint64_t index);
int32_t et_hip_gguf_metadata_element_type(const et_gguf* file, uint64_t index); /* arrays, else = type */
uint64_t et_hip_gguf_metadata_length(const et_gguf* file, uint64_t index);      /* elements; 1 for a scalar */
/* Element `element` of entry `index`: unsigned / bool, signed, real (f32 widened exactly) or
 * string (not NUL-terminated inside: `*length` bytes). Non-zero when the entry is of another kind. */
int et_hip_gguf_metadata_unsigned(const et_gguf* file, uint64_t index, uint64_t element, uint64_t* out);
int et_hip_gguf_metadata_signed(const et_gguf* file, uint64_t index, uint64_t element, int64_t* out);
int et_hip_gguf_metadata_real(const et_gguf* file, uint64_t index, uint64_t element, double* out);
const char* et_hip_gguf_metadata_string(const et_gguf* file, uint64_t index, uint64_t element,
                                        uint64_t* length);

/* GgufTensorDescriptor (gguf.rs:319-341). */
typedef struct {
    const char* name;
    uint64_t name_length;      /* bytes */
    int32_t format;            /* GGML type code: 0 F32, 2 Q4_0, 8 Q8_0, 10..14 Q2_K..Q6_K (= et_codec) */
    int32_t logical_rank;
    uint64_t logical_shape[4]; /* row-major */
    int32_t physical_rank;     /* F32: the logical shape; quantized: [rows, encoded_row_bytes] */
    uint64_t physical_shape[4];
    uint64_t data_offset;      /* absolute file offset */
    uint64_t byte_len;
} et_gguf_tensor;
uint64_t et_hip_gguf_tensor_count(const et_gguf* file);
int64_t et_hip_gguf_tensor_find(const et_gguf* file, const char* name); /* index or -1 */
int et_hip_gguf_tensor_at(const et_gguf* file, uint64_t index, et_gguf_tensor* out);

/* = read_gguf_tensor_into (gguf.rs:959-994): exactly byte_len bytes into host memory. */
int et_hip_gguf_read_tensor_into(const et_gguf* file, uint64_t index, void* destination,
                                 uint64_t destination_bytes, const volatile int32_t* cancel);
/* The same bytes into DEVICE memory: 8 MiB positioned reads into two pinned buffers (allocated
 * at the first upload, owned by the file object) alternate with asynchronous copies on `stream`;
 * returns when the tensor is in place. A quantized tensor arrives as the [rows,
 * encoded_row_bytes] u8 matrix et_hip_linear_requirements takes as `weight`. */
int et_hip_gguf_upload_tensor(et_gguf* file, uint64_t index, void* device_destination,
                              uint64_t destination_bytes, void* stream,
                              const volatile int32_t* cancel);

/* ---- int8 activation quantiser (stage 1 of ET_ACT_INT8) ------------------- */

/* The activation quantiser on its own, exposed so that tests can check the
 * stage separately: q is int8 [vectors, columns]; scale (f32) and sum (i32, may
 * be NULL) are TRANSPOSED tables [columns/32, stride] with stride = vectors
 * rounded up to a multiple of 32 (entries at m >= vectors are not written).
 *   amax = max|x| over the 32-block; scale = amax / 127;
 *   q = clamp(rint(x * (amax > 0 ? 127 / amax : 0)), -127, 127); sum = sum of q.
 * No counterpart in the reference. */
int et_hip_quantize_activations(const float* x, uint64_t x_row_stride, uint64_t vectors,
                                uint64_t columns, int8_t* q, float* scale, int32_t* sum,
                                void* stream);

/* ---- errors -------------------------------------------------------------- */

/* Message of the last failed call on this thread ("" if none). */
const char* et_hip_last_error(void);

/* The GEMV kernels whose loader waves hand rows over to consumer waves through LDS bound every
 * such wait: a wave that has polled a fixed number of times (about a second) gives up, and every
 * wave of the launch still reaches its end. `*count` receives how many waves of this process have
 * done so on the current device (0 on a healthy run; results of a launch that counted are
 * meaningless). Synchronises with the device. No counterpart in the reference: its kernels have
 * no cross-thread waits. */
int et_hip_handover_timeouts(uint64_t* count);
/* Test hook: the number of polls after which a wave gives up such a wait, for the launches that
 * follow. 0 makes every wait that is not already satisfied give up at once, so that a test can see
 * every wave leave the kernel; ET_HIP_HANDOVER_DEFAULT_SPIN_LIMIT restores the library's own value. */
#define ET_HIP_HANDOVER_DEFAULT_SPIN_LIMIT 0xffffffffu
void et_hip_test_set_handover_spin_limit(uint32_t limit);

#ifdef __cplusplus
}
#endif
#endif /* ET_HIP_H */
