// extern "C" surface of libet_hip.so (declared in include/et_hip.h). Thin
// wrappers: convert descriptors, catch every C++ exception, keep the last
// error message per thread.
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <exception>
#include <new>
#include <string>

#include "et_codecs.h"
#include "et_hip.h"
#include "kernels.h"
#include "lds_handover.h"
#include "decode_host.h"
#include "gguf.h"
#include "kv_cache.h"
#include "quantized.h"

namespace {

thread_local std::string g_last_error;

int set_error(int status, const std::string& message) {
    g_last_error = message;
    return status;
}

template <class F>
int guarded(F&& body) {
    try {
        std::string error;
        const int status = body(&error);
        if (status != ET_OK) g_last_error = error;
        return status;
    } catch (const std::bad_alloc&) {
        return set_error(ET_ERR_EXECUTION, "out of host memory");
    } catch (const std::exception& e) {
        return set_error(ET_ERR_EXECUTION, e.what());
    } catch (...) {
        return set_error(ET_ERR_EXECUTION, "unknown C++ exception");
    }
}

using et::quantized::TensorView;

int gguf_failure(const et::gguf::Error& error) {
    g_last_error = error.message;
    switch (error.kind) {
        case et::gguf::Failure::kInvalid: return ET_ERR_UNSUPPORTED;
        case et::gguf::Failure::kCancelled: return ET_ERR_CANCELLED;
        default: return ET_ERR_EXECUTION;
    }
}

}  // namespace

extern "C" {

int et_hip_is_available(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    hipDeviceProp_t props;
    if (hipGetDeviceProperties(&props, device) != hipSuccess) return 0;
    return std::strncmp(props.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

const char* et_hip_codec_name(int32_t codec) { return et::codec_name(codec); }
uint64_t et_hip_block_values(int32_t codec) { return et::block_values(codec); }
uint64_t et_hip_block_bytes(int32_t codec) { return et::block_bytes(codec); }

uint64_t et_hip_encoded_row_bytes(int32_t codec, uint64_t columns) {
    const uint64_t values = et::block_values(codec);
    if (values == 0 || columns % values != 0) return 0;
    const uint64_t blocks = columns / values;
    const uint64_t bytes = et::block_bytes(codec);
    if (blocks != 0 && bytes > UINT64_MAX / blocks) return 0;
    return blocks * bytes;
}

int et_hip_linear_requirements(const et_tensor* input, const et_tensor* weight, const et_tensor* bias,
                               int32_t codec, uint64_t rows, uint64_t columns,
                               int32_t activation_mode, et_linear_plan** out) {
    return guarded([&](std::string* error) -> int {
        if (out == nullptr) {
            *error = "quantized_linear: output plan pointer is NULL";
            return ET_ERR_INVALID;
        }
        *out = nullptr;
        TensorView in, w, b;
        if (!TensorView::from_c(input, &in, error) || !TensorView::from_c(weight, &w, error) ||
            (bias != nullptr && !TensorView::from_c(bias, &b, error))) {
            *error = "quantized_linear: " + *error;
            return ET_ERR_INVALID;
        }
        auto* plan = new et_linear_plan();
        const int status = et::quantized::linear_requirements(in, w, bias ? &b : nullptr, codec, rows,
                                                              columns, activation_mode, plan, error);
        if (status != ET_OK) {
            delete plan;
            return status;
        }
        *out = plan;
        return ET_OK;
    });
}

int et_hip_linear_plan_create(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors,
                              int32_t has_bias, int32_t activation_mode, et_linear_plan** out) {
    return guarded([&](std::string* error) -> int {
        if (out == nullptr) {
            *error = "quantized_linear: output plan pointer is NULL";
            return ET_ERR_INVALID;
        }
        *out = nullptr;
        auto* plan = new et_linear_plan();
        const int status = et::quantized::linear_plan_from_sizes(codec, rows, columns, vectors,
                                                                 has_bias != 0, activation_mode, plan,
                                                                 error);
        if (status != ET_OK) {
            delete plan;
            return status;
        }
        *out = plan;
        return ET_OK;
    });
}

void et_hip_linear_plan_destroy(et_linear_plan* plan) { delete plan; }

int32_t et_hip_linear_plan_output_rank(const et_linear_plan* plan) {
    return plan ? static_cast<int32_t>(plan->output_shape.size()) : 0;
}
void et_hip_linear_plan_output_shape(const et_linear_plan* plan, uint64_t* shape) {
    if (plan == nullptr || shape == nullptr) return;
    for (size_t d = 0; d < plan->output_shape.size(); d++) shape[d] = plan->output_shape[d];
}
uint64_t et_hip_linear_plan_vectors(const et_linear_plan* plan) { return plan ? plan->vectors : 0; }
uint64_t et_hip_linear_plan_output_bytes(const et_linear_plan* plan) {
    return plan ? plan->output_bytes : 0;
}
uint64_t et_hip_linear_plan_workspace_bytes(const et_linear_plan* plan) {
    return plan ? plan->workspace_bytes : 0;
}
const char* et_hip_linear_plan_kernel(const et_linear_plan* plan) {
    return plan ? et::quantized::kernel_name(*plan) : "";
}
uint64_t et_hip_linear_plan_algorithmic_bytes(const et_linear_plan* plan) {
    if (plan == nullptr) return 0;
    return plan->rows * plan->encoded_row_bytes + 4 * plan->vectors * plan->columns +
           4 * plan->vectors * plan->rows + (plan->has_bias ? 4 * plan->rows : 0);
}

int et_hip_linear_into(const et_linear_plan* plan, const et_tensor* input, const et_tensor* weight,
                       const et_tensor* bias, const et_tensor* destination, void* workspace,
                       uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        TensorView in, w, b, dst;
        if (!TensorView::from_c(input, &in, error) || !TensorView::from_c(weight, &w, error) ||
            (bias != nullptr && !TensorView::from_c(bias, &b, error)) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "quantized_linear: " + *error;
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_into(*plan, in, w, bias ? &b : nullptr, dst, workspace,
                                          workspace_bytes, stream, cancel, error);
    });
}

int et_hip_linear_enqueue(const et_linear_plan* plan, const float* x, uint64_t x_row_stride,
                          const uint8_t* weight, const float* bias, float* y, void* workspace,
                          uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_enqueue(*plan, x, x_row_stride, weight, bias, y, workspace,
                                             workspace_bytes, stream, cancel, error);
    });
}

int et_hip_linear_enqueue_static_workspace(const et_linear_plan* plan, const float* x, uint64_t x_row_stride,
                                           const uint8_t* weight, const float* bias, float* y, void* stream,
                                           const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_enqueue_static_workspace(*plan, x, x_row_stride, weight, bias, y, stream, cancel,
                                                              error);
    });
}

uint64_t et_hip_linear_plan_prepared_input_bytes(const et_linear_plan* plan) {
    return plan ? et::quantized::prepared_input_bytes(*plan) : 0;
}

int et_hip_linear_prepare_input(const et_linear_plan* plan, const float* x, uint64_t x_row_stride, void* prepared,
                                uint64_t prepared_bytes, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_prepare_input(*plan, x, x_row_stride, prepared, prepared_bytes, stream, error);
    });
}

int et_hip_linear_plan_fused_prepare(const et_linear_plan* plan) {
    return plan != nullptr && et::quantized::fused_prepare(*plan) ? 1 : 0;
}

int et_hip_linear_prepare_input_from(const et_linear_plan* plan, const et_prepare_source* source, void* prepared,
                                     uint64_t prepared_bytes, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr || source == nullptr) {
            *error = "quantized_linear: plan or source is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_prepare_input_from(*plan, *source, prepared, prepared_bytes, stream, error);
    });
}

int et_hip_linear_group_workspace_bytes(const et_linear_plan* const* plans, uint32_t count, uint64_t* bytes) {
    return guarded([&](std::string* error) -> int {
        if (bytes == nullptr) {
            *error = "quantized_linear: bytes is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_group_workspace_bytes(plans, count, bytes, error);
    });
}

int et_hip_linear_enqueue_prepared_group(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                         const uint8_t* const* weights, const float* const* biases,
                                         const float* const* residuals, float* const* ys, void* workspace,
                                         uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        return et::quantized::linear_enqueue_prepared_group(plans, count, prepared, weights, biases, residuals, ys,
                                                            workspace, workspace_bytes, stream, cancel, error);
    });
}

int et_hip_linear_enqueue_prepared(const et_linear_plan* plan, const void* prepared, const uint8_t* weight,
                                   const float* bias, const float* residual, float* y, void* workspace,
                                   uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_enqueue_prepared(*plan, prepared, weight, bias, residual, y, workspace,
                                                      workspace_bytes, stream, cancel, error);
    });
}

int et_hip_linear_enqueue_prepared_group_then_rotary(const et_linear_plan* const* plans, uint32_t count,
                                                     const void* prepared, const uint8_t* const* weights,
                                                     const float* const* biases, const float* const* residuals,
                                                     float* const* ys, void* workspace, uint64_t workspace_bytes,
                                                     const et_rotary_after* rotary, void* stream,
                                                     const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (rotary == nullptr) {
            *error = "rotary: NULL descriptor";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_enqueue_prepared_group_then_rotary(plans, count, prepared, weights, biases, residuals,
                                                                        ys, workspace, workspace_bytes, *rotary, stream,
                                                                        cancel, error);
    });
}

int et_hip_linear_group_shares_layout(const et_linear_plan* const* plans, uint32_t count, et_group_shares* layout) {
    return guarded([&](std::string* error) -> int {
        return et::quantized::linear_enqueue_prepared_group_shares(plans, count, nullptr, nullptr, nullptr, 0, layout,
                                                                   false, nullptr, nullptr, error);
    });
}

int et_hip_linear_enqueue_prepared_group_shares(const et_linear_plan* const* plans, uint32_t count,
                                                const void* prepared, const uint8_t* const* weights,
                                                void* workspace, uint64_t workspace_bytes, et_group_shares* layout,
                                                void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        return et::quantized::linear_enqueue_prepared_group_shares(plans, count, prepared, weights, workspace,
                                                                   workspace_bytes, layout, true, stream, cancel, error);
    });
}

int et_hip_linear_enqueue_prepared_then_norm(const et_linear_plan* plan, const void* prepared,
                                             const uint8_t* weight, const float* bias, const float* residual,
                                             float* y, void* workspace, uint64_t workspace_bytes,
                                             const et_linear_plan* next, const void* norm_weight,
                                             int32_t norm_weight_dtype, double eps, void* next_prepared,
                                             uint64_t next_prepared_bytes, void* stream,
                                             const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr || next == nullptr) {
            *error = "quantized_linear: plan is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::linear_enqueue_prepared_then_norm(*plan, prepared, weight, bias, residual, y, workspace,
                                                                workspace_bytes, *next, norm_weight, norm_weight_dtype, eps,
                                                                next_prepared,
                                                                next_prepared_bytes, stream, cancel, error);
    });
}

int et_hip_embedding_requirements(const et_tensor* indexes, const et_tensor* weight, int32_t codec,
                                  uint64_t rows, uint64_t columns, et_embedding_plan** out) {
    return guarded([&](std::string* error) -> int {
        if (out == nullptr) {
            *error = "quantized_embedding: output plan pointer is NULL";
            return ET_ERR_INVALID;
        }
        *out = nullptr;
        TensorView idx, w;
        if (!TensorView::from_c(indexes, &idx, error) || !TensorView::from_c(weight, &w, error)) {
            *error = "quantized_embedding: " + *error;
            return ET_ERR_INVALID;
        }
        auto* plan = new et_embedding_plan();
        const int status =
            et::quantized::embedding_requirements(idx, w, codec, rows, columns, plan, error);
        if (status != ET_OK) {
            delete plan;
            return status;
        }
        *out = plan;
        return ET_OK;
    });
}

void et_hip_embedding_plan_destroy(et_embedding_plan* plan) { delete plan; }
int32_t et_hip_embedding_plan_output_rank(const et_embedding_plan* plan) {
    return plan ? static_cast<int32_t>(plan->output_shape.size()) : 0;
}
void et_hip_embedding_plan_output_shape(const et_embedding_plan* plan, uint64_t* shape) {
    if (plan == nullptr || shape == nullptr) return;
    for (size_t d = 0; d < plan->output_shape.size(); d++) shape[d] = plan->output_shape[d];
}
uint64_t et_hip_embedding_plan_output_bytes(const et_embedding_plan* plan) {
    return plan ? plan->output_bytes : 0;
}

int et_hip_embedding_into(const et_embedding_plan* plan, const et_tensor* indexes,
                          const et_tensor* weight, const et_tensor* destination, void* status,
                          void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr) {
            *error = "quantized_embedding: plan is NULL";
            return ET_ERR_INVALID;
        }
        TensorView idx, w, dst;
        if (!TensorView::from_c(indexes, &idx, error) || !TensorView::from_c(weight, &w, error) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "quantized_embedding: " + *error;
            return ET_ERR_INVALID;
        }
        return et::quantized::embedding_into(*plan, idx, w, dst, status, stream, cancel, error);
    });
}

int et_hip_embedding_status_check(const et_embedding_plan* plan, const void* status_host) {
    return guarded([&](std::string* error) -> int {
        if (plan == nullptr || status_host == nullptr) {
            *error = "quantized_embedding: plan or status is NULL";
            return ET_ERR_INVALID;
        }
        return et::quantized::embedding_status_check(*plan, status_host, error);
    });
}

int et_hip_dequantize_rows(int32_t codec, uint64_t rows, uint64_t columns, const uint8_t* weight,
                           float* out, void* stream) {
    return guarded([&](std::string* error) -> int {
        const char* name = et::codec_name(codec);
        if (name == nullptr) {
            *error = "dequantize_rows: unknown codec " + std::to_string(codec);
            return ET_ERR_INVALID;
        }
        if (et_hip_encoded_row_bytes(codec, columns) == 0 && columns != 0) {
            *error = "dequantize_rows: logical row width " + std::to_string(columns) +
                     " is invalid for " + name;
            return ET_ERR_UNSUPPORTED;
        }
        if (rows == 0 || columns == 0) return ET_OK;
        if (weight == nullptr || out == nullptr || reinterpret_cast<uintptr_t>(out) % 16 != 0) {
            *error = "dequantize_rows: operands must be non-NULL and the output 16-byte aligned";
            return ET_ERR_INVALID;
        }
        et::IndexLayout layout;
        std::memset(&layout, 0, sizeof layout);
        layout.contiguous = 1;
        const hipError_t status = et::dequantize_rows(codec, weight, nullptr, 0, layout, rows, rows,
                                                      columns, out, nullptr,
                                                      static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("dequantize_rows: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

uint64_t et_hip_kv_attention_workspace_bytes(const et_kv_layer* layer, uint64_t query_heads,
                                             uint64_t tokens) {
    uint64_t bytes = 0;
    guarded([&](std::string* error) -> int {
        if (layer == nullptr) {
            *error = "kv attention: layer is NULL";
            return ET_ERR_INVALID;
        }
        return et::kv::workspace_bytes(*layer, query_heads, tokens, &bytes, error);
    });
    return bytes;
}

const char* et_hip_kv_attention_kernel(const et_kv_layer* layer, uint64_t query_heads, uint64_t tokens) {
    return layer ? et::kv::kernel_name(*layer, query_heads, tokens) : "";
}

int et_hip_kv_attention_into(const et_kv_layer* layer, const et_tensor* q, const et_tensor* k,
                             const et_tensor* v, double scale, uint64_t window,
                             const et_tensor* destination, void* workspace, uint64_t workspace_bytes,
                             void* status, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (layer == nullptr) {
            *error = "kv attention: layer is NULL";
            return ET_ERR_INVALID;
        }
        TensorView qv, kv, vv, dst;
        if (!TensorView::from_c(q, &qv, error) || !TensorView::from_c(k, &kv, error) ||
            !TensorView::from_c(v, &vv, error) || !TensorView::from_c(destination, &dst, error)) {
            *error = "kv attention: " + *error;
            return ET_ERR_INVALID;
        }
        return et::kv::attention_into(*layer, qv, kv, vv, scale, window, dst, workspace, workspace_bytes,
                                      status, stream, cancel, error);
    });
}

int et_hip_kv_attention_prepared_into(const et_kv_layer* layer, const et_tensor* q, const et_tensor* k,
                                      const et_tensor* v, double scale, uint64_t window,
                                      const et_tensor* destination, void* workspace, uint64_t workspace_bytes,
                                      void* status, const et_linear_plan* consumer, void* prepared,
                                      uint64_t prepared_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (layer == nullptr || consumer == nullptr) {
            *error = "kv attention: layer or plan is NULL";
            return ET_ERR_INVALID;
        }
        TensorView qv, kv, vv, dst;
        if (!TensorView::from_c(q, &qv, error) || !TensorView::from_c(k, &kv, error) ||
            !TensorView::from_c(v, &vv, error) || !TensorView::from_c(destination, &dst, error)) {
            *error = "kv attention: " + *error;
            return ET_ERR_INVALID;
        }
        return et::kv::attention_into(*layer, qv, kv, vv, scale, window, dst, workspace, workspace_bytes, status,
                                      stream, cancel, error, consumer, prepared, prepared_bytes);
    });
}

int et_hip_kv_attention_projected_into(const et_kv_layer* layer, const et_kv_projected* projected, double scale,
                                       uint64_t window, const et_tensor* destination, void* workspace,
                                       uint64_t workspace_bytes, void* status, const et_linear_plan* consumer,
                                       void* prepared, uint64_t prepared_bytes, void* stream,
                                       const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (layer == nullptr || projected == nullptr) {
            *error = "kv attention: layer or projection is NULL";
            return ET_ERR_INVALID;
        }
        TensorView dst;
        if (!TensorView::from_c(destination, &dst, error)) {
            *error = "kv attention: " + *error;
            return ET_ERR_INVALID;
        }
        return et::kv::attention_projected_into(*layer, *projected, scale, window, dst, workspace, workspace_bytes,
                                                status, stream, cancel, error, consumer, prepared, prepared_bytes);
    });
}

int et_hip_kv_attention_status_check(const et_kv_layer* layer, uint64_t tokens, const void* status_host) {
    return guarded([&](std::string* error) -> int {
        if (layer == nullptr || status_host == nullptr) {
            *error = "kv attention: layer or status is NULL";
            return ET_ERR_INVALID;
        }
        return et::kv::status_check(*layer, tokens, status_host, error);
    });
}

int et_hip_kv_commit(const et_kv_layer* layer, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (layer == nullptr || layer->cursors == nullptr || layer->advances == nullptr) {
            *error = "kv commit: layer, cursors or advances is NULL";
            return ET_ERR_INVALID;
        }
        if (layer->active_batch > layer->slots) {
            *error = "kv commit: active batch " + std::to_string(layer->active_batch) + " exceeds " +
                     std::to_string(layer->slots) + " slots";
            return ET_ERR_INVALID;
        }
        const hipError_t status = et::commit_advances(const_cast<uint32_t*>(layer->cursors), layer->advances,
                                                      layer->active_batch, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("kv commit: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

int et_hip_rms_norm_into(const et_tensor* x, const et_tensor* weight, double eps, const et_tensor* destination,
                         void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView xv, wv, dst;
        if (!TensorView::from_c(x, &xv, error) || (weight != nullptr && !TensorView::from_c(weight, &wv, error)) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "rms_norm: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::rms_norm_into(xv, weight ? &wv : nullptr, eps, dst, stream, error);
    });
}

int et_hip_rotary_into(const et_tensor* x, const uint32_t* offsets, uint64_t offsets_len, double theta,
                       double sign, int32_t layout, const et_tensor* destination, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView xv, dst;
        if (!TensorView::from_c(x, &xv, error) || !TensorView::from_c(destination, &dst, error)) {
            *error = "rotary: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::rotary_into(xv, offsets, offsets_len, theta, sign, layout, dst, stream, error);
    });
}

int et_hip_rotary_pair_into(const et_tensor* x, const et_tensor* second, const uint32_t* offsets, uint64_t offsets_len,
                            double theta, double sign, int32_t layout, const et_tensor* destination,
                            const et_tensor* second_destination, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView xv, sv, dst, sdst;
        if (!TensorView::from_c(x, &xv, error) || !TensorView::from_c(second, &sv, error) ||
            !TensorView::from_c(destination, &dst, error) || !TensorView::from_c(second_destination, &sdst, error)) {
            *error = "rotary: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::rotary_pair_into(xv, sv, offsets, offsets_len, theta, sign, layout, dst, sdst, stream, error);
    });
}

int et_hip_add_into(const et_tensor* a, const et_tensor* b, const et_tensor* destination, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView av, bv, dst;
        if (!TensorView::from_c(a, &av, error) || !TensorView::from_c(b, &bv, error) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "add: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::add_into(av, bv, dst, stream, error);
    });
}

int et_hip_silu_mul_into(const et_tensor* gate, const et_tensor* up, const et_tensor* destination, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView gv, uv, dst;
        if (!TensorView::from_c(gate, &gv, error) || !TensorView::from_c(up, &uv, error) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "silu_mul: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::silu_mul_into(gv, uv, dst, stream, error);
    });
}

uint64_t et_hip_greedy_workspace_bytes(uint64_t rows, uint64_t vocabulary) {
    return et::decode::greedy_workspace_bytes(rows, vocabulary);
}

int et_hip_greedy_tokens_into(const et_tensor* logits, uint32_t* tokens, void* workspace, uint64_t workspace_bytes,
                              void* status, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView lv;
        if (!TensorView::from_c(logits, &lv, error)) {
            *error = "sample: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::greedy_tokens_into(lv, tokens, workspace, workspace_bytes, status, stream, error);
    });
}

int et_hip_greedy_status_check(uint64_t rows, const void* status_host) {
    return guarded([&](std::string* error) -> int {
        if (status_host == nullptr && rows != 0) {
            *error = "sample: status is NULL";
            return ET_ERR_INVALID;
        }
        return et::decode::greedy_status_check(rows, status_host, error);
    });
}

int et_hip_gather_rows_into(const et_tensor* table, const et_tensor* indexes, const et_tensor* destination,
                            void* status, void* stream) {
    return guarded([&](std::string* error) -> int {
        TensorView tv, iv, dst;
        if (!TensorView::from_c(table, &tv, error) || !TensorView::from_c(indexes, &iv, error) ||
            !TensorView::from_c(destination, &dst, error)) {
            *error = "index_select: " + *error;
            return ET_ERR_INVALID;
        }
        return et::decode::gather_rows_into(tv, iv, dst, status, stream, error);
    });
}

int et_hip_gather_rows_status_check(uint64_t table_rows, uint64_t count, const void* status_host) {
    return guarded([&](std::string* error) -> int {
        if (status_host == nullptr && count != 0) {
            *error = "index_select: status is NULL";
            return ET_ERR_INVALID;
        }
        return et::decode::gather_rows_status_check(table_rows, count, status_host, error);
    });
}

int et_hip_gguf_open(const char* path, const volatile int32_t* cancel, et_gguf** out) {
    return guarded([&](std::string* error) -> int {
        if (path == nullptr || out == nullptr) {
            *error = "gguf: path or output pointer is NULL";
            return ET_ERR_INVALID;
        }
        *out = nullptr;
        et::gguf::Error failure;
        et::gguf::File* file = et::gguf::open(path, cancel, &failure);
        if (file == nullptr) {
            const int status = gguf_failure(failure);
            *error = failure.message;
            return status;
        }
        *out = reinterpret_cast<et_gguf*>(file);
        return ET_OK;
    });
}

}  // extern "C"
namespace {
const et::gguf::File* as_file(const et_gguf* file) { return reinterpret_cast<const et::gguf::File*>(file); }
const et::gguf::Entry* entry_at(const et_gguf* file, uint64_t index) {
    return file != nullptr && index < as_file(file)->metadata.size() ? &as_file(file)->metadata[index] : nullptr;
}
}  // namespace
extern "C" {

void et_hip_gguf_close(et_gguf* file) { delete reinterpret_cast<et::gguf::File*>(file); }
const char* et_hip_gguf_architecture(const et_gguf* file) { return file ? as_file(file)->architecture.c_str() : ""; }
uint64_t et_hip_gguf_metadata_count(const et_gguf* file) { return file ? as_file(file)->metadata.size() : 0; }
int64_t et_hip_gguf_metadata_find(const et_gguf* file, const char* key) {
    if (file == nullptr || key == nullptr) return -1;
    const auto& metadata = as_file(file)->metadata;
    for (size_t i = 0; i < metadata.size(); i++)
        if (metadata[i].key == key) return static_cast<int64_t>(i);
    return -1;
}
const char* et_hip_gguf_metadata_key(const et_gguf* file, uint64_t index) {
    const auto* entry = entry_at(file, index);
    return entry ? entry->key.c_str() : nullptr;
}
uint64_t et_hip_gguf_metadata_key_length(const et_gguf* file, uint64_t index) {
    const auto* entry = entry_at(file, index);
    return entry ? entry->key.size() : 0;
}
int32_t et_hip_gguf_metadata_type(const et_gguf* file, uint64_t index) {
    const auto* entry = entry_at(file, index);
    return entry ? static_cast<int32_t>(entry->value.type) : -1;
}
int32_t et_hip_gguf_metadata_element_type(const et_gguf* file, uint64_t index) {
    const auto* entry = entry_at(file, index);
    if (entry == nullptr) return -1;
    return static_cast<int32_t>(entry->value.type == 9 ? entry->value.element_type : entry->value.type);
}
uint64_t et_hip_gguf_metadata_length(const et_gguf* file, uint64_t index) {
    const auto* entry = entry_at(file, index);
    return entry ? entry->value.length() : 0;
}
int et_hip_gguf_metadata_unsigned(const et_gguf* file, uint64_t index, uint64_t element, uint64_t* out) {
    const auto* entry = entry_at(file, index);
    if (entry == nullptr || out == nullptr || element >= entry->value.integers.size()) return ET_ERR_INVALID;
    *out = entry->value.integers[element];
    return ET_OK;
}
int et_hip_gguf_metadata_signed(const et_gguf* file, uint64_t index, uint64_t element, int64_t* out) {
    const auto* entry = entry_at(file, index);
    if (entry == nullptr || out == nullptr || element >= entry->value.signed_integers.size()) return ET_ERR_INVALID;
    *out = entry->value.signed_integers[element];
    return ET_OK;
}
int et_hip_gguf_metadata_real(const et_gguf* file, uint64_t index, uint64_t element, double* out) {
    const auto* entry = entry_at(file, index);
    if (entry == nullptr || out == nullptr || element >= entry->value.reals.size()) return ET_ERR_INVALID;
    *out = entry->value.reals[element];
    return ET_OK;
}
const char* et_hip_gguf_metadata_string(const et_gguf* file, uint64_t index, uint64_t element, uint64_t* length) {
    const auto* entry = entry_at(file, index);
    if (entry == nullptr || element >= entry->value.strings.size()) return nullptr;
    if (length != nullptr) *length = entry->value.strings[element].size();
    return entry->value.strings[element].c_str();
}

uint64_t et_hip_gguf_tensor_count(const et_gguf* file) { return file ? as_file(file)->tensors.size() : 0; }
int64_t et_hip_gguf_tensor_find(const et_gguf* file, const char* name) {
    if (file == nullptr || name == nullptr) return -1;
    const auto& tensors = as_file(file)->tensors;
    for (size_t i = 0; i < tensors.size(); i++)
        if (tensors[i].name == name) return static_cast<int64_t>(i);
    return -1;
}
int et_hip_gguf_tensor_at(const et_gguf* file, uint64_t index, et_gguf_tensor* out) {
    if (file == nullptr || out == nullptr || index >= as_file(file)->tensors.size())
        return set_error(ET_ERR_INVALID, "gguf: tensor index out of range");
    const et::gguf::Tensor& tensor = as_file(file)->tensors[index];
    std::memset(out, 0, sizeof *out);
    out->name = tensor.name.c_str();
    out->name_length = tensor.name.size();
    out->format = static_cast<int32_t>(tensor.format);
    out->logical_rank = static_cast<int32_t>(tensor.logical_shape.size());
    for (size_t d = 0; d < tensor.logical_shape.size(); d++) out->logical_shape[d] = tensor.logical_shape[d];
    out->physical_rank = static_cast<int32_t>(tensor.physical_shape.size());
    for (size_t d = 0; d < tensor.physical_shape.size(); d++) out->physical_shape[d] = tensor.physical_shape[d];
    out->data_offset = tensor.data_offset;
    out->byte_len = tensor.byte_len;
    return ET_OK;
}

int et_hip_gguf_read_tensor_into(const et_gguf* file, uint64_t index, void* destination,
                                 uint64_t destination_bytes, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (file == nullptr || index >= as_file(file)->tensors.size() || (destination == nullptr && destination_bytes != 0)) {
            *error = "gguf: file, tensor index or destination is invalid";
            return ET_ERR_INVALID;
        }
        et::gguf::Error failure;
        if (et::gguf::read_tensor(*as_file(file), as_file(file)->tensors[index], destination, destination_bytes, cancel,
                                  &failure))
            return ET_OK;
        const int status = gguf_failure(failure);
        *error = failure.message;
        return status;
    });
}

int et_hip_gguf_upload_tensor(et_gguf* file, uint64_t index, void* device_destination,
                              uint64_t destination_bytes, void* stream, const volatile int32_t* cancel) {
    return guarded([&](std::string* error) -> int {
        if (file == nullptr || index >= as_file(file)->tensors.size() ||
            (device_destination == nullptr && destination_bytes != 0)) {
            *error = "gguf: file, tensor index or destination is invalid";
            return ET_ERR_INVALID;
        }
        auto* owner = reinterpret_cast<et::gguf::File*>(file);
        et::gguf::Error failure;
        if (et::gguf::upload_tensor(*owner, owner->tensors[index], device_destination, destination_bytes, stream, cancel,
                                    &failure))
            return ET_OK;
        const int status = gguf_failure(failure);
        *error = failure.message;
        return status;
    });
}

int et_hip_quantize_activations(const float* x, uint64_t x_row_stride, uint64_t vectors,
                                uint64_t columns, int8_t* q, float* scale, int32_t* sum,
                                void* stream) {
    return guarded([&](std::string* error) -> int {
        if (columns % 32 != 0) {
            *error = "quantize_activations: columns must be a multiple of 32";
            return ET_ERR_UNSUPPORTED;
        }
        if (vectors == 0 || columns == 0) return ET_OK;
        if (x == nullptr || q == nullptr || scale == nullptr ||
            reinterpret_cast<uintptr_t>(x) % 16 != 0 || x_row_stride % 4 != 0 ||
            reinterpret_cast<uintptr_t>(q) % 4 != 0) {
            *error = "quantize_activations: operands must be non-NULL and 16-byte aligned";
            return ET_ERR_INVALID;
        }
        const hipError_t status = et::quantize_activations(x, x_row_stride, vectors, columns, q, scale,
                                                           sum, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("quantize_activations: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

const char* et_hip_last_error(void) { return g_last_error.c_str(); }

int et_hip_handover_timeouts(uint64_t* count) {
    return guarded([&](std::string* error) -> int {
        if (count == nullptr) {
            *error = "handover_timeouts: count is NULL";
            return ET_ERR_INVALID;
        }
        uint32_t word = 0;
        if (hipError_t status = et::handover_timeouts(&word)) {
            *error = std::string("handover_timeouts: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        *count = word;
        return ET_OK;
    });
}

void et_hip_test_set_handover_spin_limit(uint32_t limit) {
    et::handover_set_spin_limit(limit == ET_HIP_HANDOVER_DEFAULT_SPIN_LIMIT ? et::kHandoverSpinLimit : limit);
}

}  // extern "C"
