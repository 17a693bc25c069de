// Host side of the decode-neighbour operators: the reference's validation and messages, then
// the launch (kernels in decode_ops.hip).
#pragma once

#include <cstdint>
#include <string>

#include "et_hip.h"
#include "quantized.h"

namespace et {
namespace decode {

using quantized::TensorView;

// Every function returns an et_status and, on failure, leaves the message in *error.
int rms_norm_into(const TensorView& x, const TensorView* weight, double eps, const TensorView& destination,
                  void* stream, std::string* error);
int rotary_into(const TensorView& x, const uint32_t* offsets, uint64_t offsets_len, double theta, double sign,
                int32_t layout, const TensorView& destination, void* stream, std::string* error);
int rotary_pair_into(const TensorView& x, const TensorView& second, const uint32_t* offsets, uint64_t offsets_len,
                     double theta, double sign, int32_t layout, const TensorView& destination,
                     const TensorView& second_destination, void* stream, std::string* error);
int add_into(const TensorView& a, const TensorView& b, const TensorView& destination, void* stream,
             std::string* error);
int silu_mul_into(const TensorView& gate, const TensorView& up, const TensorView& destination, void* stream,
                  std::string* error);
uint64_t greedy_workspace_bytes(uint64_t rows, uint64_t vocabulary);
int greedy_tokens_into(const TensorView& logits, uint32_t* tokens, void* workspace, uint64_t workspace_bytes,
                       void* status, void* stream, std::string* error);
int greedy_status_check(uint64_t rows, const void* status_host, std::string* error);
int gather_rows_into(const TensorView& table, const TensorView& indexes, const TensorView& destination,
                     void* status, void* stream, std::string* error);
int gather_rows_status_check(uint64_t table_rows, uint64_t count, const void* status_host, std::string* error);

}  // namespace decode
}  // namespace et
