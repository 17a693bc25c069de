// Host side of the quantized operators: the plan / execute pair a backend
// crate of the reference exposes to its executable, restated over device
// buffers. Names, argument meaning and error text follow
// crates/runtime-cpu/src/quantized.rs (linear_requirements :297-336,
// validate_linear_execution :367-415, linear_into :419-499,
// embedding_requirements :340-365, embedding_into :546-616).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "et_hip.h"

namespace et {
namespace quantized {

// Reference Tensor = storage + Layout (crates/runtime/src/layout.rs).
struct TensorView {
    const void* data = nullptr;
    int32_t dtype = ET_DTYPE_F32;
    std::vector<uint64_t> shape;
    std::vector<uint64_t> strides;  // always materialised
    uint64_t offset = 0;

    static bool from_c(const et_tensor* tensor, TensorView* out, std::string* error);
    bool is_contiguous() const;  // Layout::is_contiguous, layout.rs:110-124
};

enum class LinearKernel {
    kNone,         // empty output: nothing is enqueued
    kGemvLimb,     // dequant-GEMV on integer dot products (gemv_limb.hip)
    kGemvGeneric,  // portable dequant-GEMV (gemv_generic.hip)
    kGemvMma,      // 2..8 vectors in one pass over W on the int8 matrix cores (gemv_mma.hip)
    kGemmI8,       // int8 activations: quantize_act.hip + gemm_i8.hip
    kGemmLimb,     // f32-accurate 3-limb activations on the same matrix-core kernel
    kGemmHalf,     // f32-accurate two-half activations on the half-float matrix cores (gemm_h16)
};

}  // namespace quantized
}  // namespace et

// The opaque plan types of the C ABI.
struct et_linear_plan {
    int32_t codec;
    uint64_t rows, columns, encoded_row_bytes;
    bool has_bias;
    int32_t activation_mode;
    std::vector<uint64_t> input_shape;   // empty for plans made from raw sizes
    std::vector<uint64_t> output_shape;
    uint64_t vectors;
    uint64_t output_bytes;
    et::quantized::LinearKernel kernel;
    uint32_t vectors_per_launch;
    std::string kernel_label;              // kGemvLimb plans: what the launches of one call are (kernel_name)
    // workspace sections (byte offsets), all 256-byte aligned
    uint64_t gather_offset, gather_bytes;  // densified f32 input
    uint64_t bias_offset;                  // densified f32 bias
    uint64_t q_offset;                     // quantised activation tiles (matrix-core kernels)
    uint64_t partial_offset;               // partial results of the K shares (0 splits: unused)
    uint32_t k_splits;
    uint64_t workspace_bytes;
};

struct et_embedding_plan {
    int32_t codec;
    uint64_t rows, columns, encoded_row_bytes;
    std::vector<uint64_t> index_shape;
    int32_t index_dtype;
    std::vector<uint64_t> output_shape;
    uint64_t count;
    uint64_t output_bytes;
};

namespace et {
namespace quantized {

// Every function returns an et_status and, on failure, leaves the message in *error.
int linear_requirements(const TensorView& input, const TensorView& weight, const TensorView* bias,
                        int32_t codec, uint64_t rows, uint64_t columns, int32_t activation_mode,
                        et_linear_plan* plan, std::string* error);
// Resolves the device addresses of the library's own device symbols on the current device (a no-op
// without a device). Called when a plan is made, so that no launch has to do it - a launch may be
// recorded into a stream capture, where such a lookup does not belong.
void warm_device_symbols();
int linear_plan_from_sizes(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors,
                           bool has_bias, int32_t activation_mode, et_linear_plan* plan,
                           std::string* error);
int linear_into(const et_linear_plan& plan, const TensorView& input, const TensorView& weight,
                const TensorView* bias, const TensorView& destination, void* workspace,
                uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                std::string* error);
int linear_enqueue(const et_linear_plan& plan, const float* x, uint64_t x_row_stride,
                   const uint8_t* weight, const float* bias, float* y, void* workspace,
                   uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                   std::string* error);

// The quantised form of the activations a matrix-core plan consumes, made once and shared by every
// plan of the same columns, vectors and activation mode; 0 bytes when the plan's kernel reads x itself.
uint64_t prepared_input_bytes(const et_linear_plan& plan);
int linear_prepare_input(const et_linear_plan& plan, const float* x, uint64_t x_row_stride, void* prepared,
                         uint64_t prepared_bytes, void* stream, std::string* error);
// The prepared input of rms_norm(x) * second or silu(x) * second (et_prepare_source in et_hip.h):
// only for plans whose prepared form has a quantiser that applies the operator on the fly.
bool fused_prepare(const et_linear_plan& plan);
int linear_prepare_input_from(const et_linear_plan& plan, const et_prepare_source& source, void* prepared,
                              uint64_t prepared_bytes, void* stream, std::string* error);
// Several plans of the same columns and vectors against one prepared input in one launch (see
// et_hip_linear_enqueue_prepared_group in et_hip.h).
// linear_enqueue with the workspace in a device array of the library's own (static_workspace.cpp): for
// callers that cannot allocate. Plans that need more than ET_HIP_STATIC_WORKSPACE_BYTES are refused.
int linear_enqueue_static_workspace(const et_linear_plan& plan, const float* x, uint64_t x_row_stride,
                                    const uint8_t* weight, const float* bias, float* y, void* stream,
                                    const volatile int32_t* cancel, std::string* error);
int linear_group_workspace_bytes(const et_linear_plan* const* plans, uint32_t count, uint64_t* bytes, std::string* error);
int linear_enqueue_prepared_group(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                  const uint8_t* const* weights, const float* const* biases,
                                  const float* const* residuals, float* const* ys, void* workspace,
                                  uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                                  std::string* error);
// y = W x (+ bias) (+ residual, which may be y itself) from a prepared input.
// linear_enqueue_prepared_group, then a rotary embedding of the members named by `rotary.members`
// (see et_hip_linear_enqueue_prepared_group_then_rotary in et_hip.h).
int linear_enqueue_prepared_group_then_rotary(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                              const uint8_t* const* weights, const float* const* biases,
                                              const float* const* residuals, float* const* ys, void* workspace,
                                              uint64_t workspace_bytes, const et_rotary_after& rotary, void* stream,
                                              const volatile int32_t* cancel, std::string* error);
// The group's launch without the one that sums its K shares (see et_hip_linear_enqueue_prepared_group_shares
// in et_hip.h); prepared == nullptr: the layout only.
int linear_enqueue_prepared_group_shares(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                         const uint8_t* const* weights, void* workspace, uint64_t workspace_bytes,
                                         et_group_shares* layout, bool launch, void* stream,
                                         const volatile int32_t* cancel, std::string* error);
int linear_enqueue_prepared(const et_linear_plan& plan, const void* prepared, const uint8_t* weight, const float* bias,
                            const float* residual, float* y, void* workspace, uint64_t workspace_bytes, void* stream,
                            const volatile int32_t* cancel, std::string* error);
// linear_enqueue_prepared, then the prepared input of rms_norm(y) * norm_weight for `next` (see
// et_hip_linear_enqueue_prepared_then_norm in et_hip.h).
int linear_enqueue_prepared_then_norm(const et_linear_plan& plan, const void* prepared, const uint8_t* weight,
                                      const float* bias, const float* residual, float* y, void* workspace,
                                      uint64_t workspace_bytes, const et_linear_plan& next, const void* norm_weight,
                                      int32_t norm_weight_dtype,
                                      double eps, void* next_prepared, uint64_t next_prepared_bytes, void* stream,
                                      const volatile int32_t* cancel, std::string* error);

int embedding_requirements(const TensorView& indexes, const TensorView& weight, int32_t codec,
                           uint64_t rows, uint64_t columns, et_embedding_plan* plan,
                           std::string* error);
int embedding_into(const et_embedding_plan& plan, const TensorView& indexes,
                   const TensorView& weight, const TensorView& destination, void* status,
                   void* stream, const volatile int32_t* cancel, std::string* error);
int embedding_status_check(const et_embedding_plan& plan, const void* status_host,
                           std::string* error);

const char* kernel_name(const et_linear_plan& plan);

}  // namespace quantized
}  // namespace et
