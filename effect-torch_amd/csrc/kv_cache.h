// Host side of paged key/value-cache attention: validation in the reference's
// order and wording (crates/runtime-cpu/src/napi/mod.rs:3320-3369, :3568-3609),
// then the launch.
#pragma once

#include <cstdint>
#include <string>

#include "et_hip.h"
#include "quantized.h"

namespace et {
namespace kv {

// Every function returns an et_status and, on failure, leaves the message in *error.
int workspace_bytes(const et_kv_layer& layer, uint64_t query_heads, uint64_t tokens, uint64_t* bytes,
                    std::string* error);
int attention_into(const et_kv_layer& layer, const quantized::TensorView& q, const quantized::TensorView& k,
                   const quantized::TensorView& v, double scale, uint64_t window,
                   const quantized::TensorView& destination, void* workspace, uint64_t workspace_bytes,
                   void* status, void* stream, const volatile int32_t* cancel, std::string* error,
                   const et_linear_plan* consumer = nullptr, void* prepared = nullptr, uint64_t prepared_bytes = 0,
                   const et_kv_projected* projected = nullptr);
// attention_into for one token per slot with q, k and v still the K shares of their projections
// (see et_hip_kv_attention_projected_into in et_hip.h).
int attention_projected_into(const et_kv_layer& layer, const et_kv_projected& projected, double scale, uint64_t window,
                             const quantized::TensorView& destination, void* workspace, uint64_t workspace_bytes,
                             void* status, void* stream, const volatile int32_t* cancel, std::string* error,
                             const et_linear_plan* consumer, void* prepared, uint64_t prepared_bytes);
int status_check(const et_kv_layer& layer, uint64_t tokens, const void* status_host, std::string* error);
const char* kernel_name(const et_kv_layer& layer, uint64_t query_heads, uint64_t tokens);

}  // namespace kv
}  // namespace et
