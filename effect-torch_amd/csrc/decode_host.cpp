#include "decode_host.h"

#include <hip/hip_runtime_api.h>

#include <cstring>

#include "kernels.h"

namespace et {
namespace decode {
namespace {

int fail(std::string* error, int status, const std::string& message) {
    *error = message;
    return status;
}

uint64_t numel(const TensorView& t) {
    uint64_t total = 1;
    for (uint64_t d : t.shape) total *= d;
    return total;
}

const float* f32_data(const TensorView& t) { return static_cast<const float*>(t.data) + t.offset; }
float* f32_out(const TensorView& t) { return const_cast<float*>(static_cast<const float*>(t.data)) + t.offset; }

int launched(hipError_t status, const char* what, std::string* error) {
    if (status == hipSuccess) return ET_OK;
    return fail(error, ET_ERR_EXECUTION, std::string(what) + ": HIP error: " + hipGetErrorString(status));
}

constexpr uint64_t kLimit = 0xffffffffull;

}  // namespace

// rms_norm_forward_requirements (composed.rs:690-715) + rms_norm_forward_into (:1491-1533)
int rms_norm_into(const TensorView& x, const TensorView* weight, double eps, const TensorView& destination,
                  void* stream, std::string* error) {
    if (x.dtype != ET_DTYPE_F32) return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: only f32 tensors are supported");
    if (x.shape.empty()) return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: input must have rank at least 1");
    const uint64_t columns = x.shape.back(), elements = numel(x);
    if (columns == 0 || elements == 0)
        return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: zero-sized dimensions are unsupported");
    // composed.rs:700-705 wants the weight in the input's type; a half-float weight is widened on use
    if (weight != nullptr && ((weight->dtype != x.dtype && weight->dtype != ET_DTYPE_F16) ||
                              weight->shape != std::vector<uint64_t>{columns}))
        return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: weight must match the last dimension and dtype");
    if (destination.dtype != x.dtype || destination.shape != x.shape)
        return fail(error, ET_ERR_EXECUTION, "rms_norm output: destination does not match the input shape");
    if (!x.is_contiguous() || !destination.is_contiguous() || (weight != nullptr && !weight->is_contiguous()))
        return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: operands must be contiguous");
    if (columns > kLimit || elements / columns > 0x7fffffffull)
        return fail(error, ET_ERR_UNSUPPORTED, "rms_norm: geometry exceeds the launch limits");
    if (x.data == nullptr || destination.data == nullptr || (weight != nullptr && weight->data == nullptr))
        return fail(error, ET_ERR_INVALID, "rms_norm: NULL device pointer");
    const bool half = weight != nullptr && weight->dtype == ET_DTYPE_F16;
    const void* w = weight == nullptr ? nullptr
                    : half            ? static_cast<const void*>(static_cast<const uint16_t*>(weight->data) + weight->offset)
                                      : static_cast<const void*>(f32_data(*weight));
    return launched(rms_norm(f32_data(x), w, half ? 1 : 0, eps, f32_out(destination), elements / columns, columns,
                             static_cast<hipStream_t>(stream)),
                    "rms_norm", error);
}

namespace {
struct RotaryShape {
    uint64_t batch, rows, steps, head_dim, elements;
};
// The checks of rotary_forward_into (composed.rs:2735-2772) for one tensor.
int rotary_shape(const TensorView& x, uint64_t offsets_len, const TensorView& destination, RotaryShape* shape,
                 std::string* error) {
    const size_t rank = x.shape.size();
    if (rank < 2 || x.shape[rank - 1] % 2 != 0 || x.dtype != ET_DTYPE_F32)
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: expected a float rank >= 2 tensor with even head dimension");
    shape->batch = rank == 2 ? 1 : x.shape[0];
    if (offsets_len != 1 && offsets_len != shape->batch)
        return fail(error, ET_ERR_UNSUPPORTED, "rotary embedding: " + std::to_string(offsets_len) +
                                                   " offsets for batch " + std::to_string(shape->batch));
    if (destination.dtype != x.dtype || destination.shape != x.shape)
        return fail(error, ET_ERR_EXECUTION, "rotary output: destination does not match the input shape");
    if (!x.is_contiguous() || !destination.is_contiguous())
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: operands must be contiguous");
    shape->steps = x.shape[rank - 2];
    shape->head_dim = x.shape[rank - 1];
    shape->elements = numel(x);
    shape->rows = shape->elements == 0 ? 0 : shape->elements / (shape->steps * shape->head_dim);
    if (shape->elements != 0 && (shape->steps > kLimit || shape->head_dim > kLimit || shape->rows / shape->batch > kLimit ||
                                 shape->elements / 2 > (0x7fffffffull << 8)))
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: geometry exceeds the launch limits");
    if (shape->elements != 0 && (x.data == nullptr || destination.data == nullptr))
        return fail(error, ET_ERR_INVALID, "rotary: NULL device pointer");
    return ET_OK;
}
}  // namespace

// rotary_forward_into (composed.rs:2735-2772)
int rotary_into(const TensorView& x, const uint32_t* offsets, uint64_t offsets_len, double theta, double sign,
                int32_t layout, const TensorView& destination, void* stream, std::string* error) {
    if (layout != ET_ROTARY_HALF_SPLIT && layout != ET_ROTARY_INTERLEAVED_PAIRS)
        return fail(error, ET_ERR_INVALID, "rotary: unknown layout " + std::to_string(layout));
    RotaryShape shape;
    if (int rc = rotary_shape(x, offsets_len, destination, &shape, error)) return rc;
    if (shape.elements == 0) return ET_OK;
    if (offsets == nullptr) return fail(error, ET_ERR_INVALID, "rotary: NULL device pointer");
    return launched(rotary(f32_data(x), offsets, static_cast<uint32_t>(offsets_len), theta, sign,
                           layout == ET_ROTARY_INTERLEAVED_PAIRS, f32_out(destination), shape.batch, shape.rows,
                           shape.steps, shape.head_dim, static_cast<hipStream_t>(stream)),
                    "rotary", error);
}

// Two tensors at the same positions (the queries and the keys of a step) in one launch.
int rotary_pair_into(const TensorView& x, const TensorView& second, const uint32_t* offsets, uint64_t offsets_len,
                     double theta, double sign, int32_t layout, const TensorView& destination,
                     const TensorView& second_destination, void* stream, std::string* error) {
    if (layout != ET_ROTARY_HALF_SPLIT && layout != ET_ROTARY_INTERLEAVED_PAIRS)
        return fail(error, ET_ERR_INVALID, "rotary: unknown layout " + std::to_string(layout));
    RotaryShape a, b;
    if (int rc = rotary_shape(x, offsets_len, destination, &a, error)) return rc;
    if (int rc = rotary_shape(second, offsets_len, second_destination, &b, error)) return rc;
    if (a.batch != b.batch || a.steps != b.steps || a.head_dim != b.head_dim)
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: both tensors must share batch, steps and head dimension");
    if (a.elements == 0 && b.elements == 0) return ET_OK;
    if (offsets == nullptr) return fail(error, ET_ERR_INVALID, "rotary: NULL device pointer");
    if ((a.elements + b.elements) / 2 > (0x7fffffffull << 8))
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: geometry exceeds the launch limits");
    return launched(rotary_pair(f32_data(x), f32_out(destination), a.rows, f32_data(second), f32_out(second_destination),
                                b.rows, offsets, static_cast<uint32_t>(offsets_len), theta, sign,
                                layout == ET_ROTARY_INTERLEAVED_PAIRS, a.batch, a.steps, a.head_dim,
                                static_cast<hipStream_t>(stream)),
                    "rotary", error);
}

int add_into(const TensorView& a, const TensorView& b, const TensorView& destination, void* stream,
             std::string* error) {
    if (a.dtype != ET_DTYPE_F32 || b.dtype != ET_DTYPE_F32 || destination.dtype != ET_DTYPE_F32)
        return fail(error, ET_ERR_UNSUPPORTED, "add: only f32 tensors are supported");
    if (a.shape != b.shape || destination.shape != a.shape)
        return fail(error, ET_ERR_UNSUPPORTED, "add: both operands and the destination must have one shape");
    if (!a.is_contiguous() || !b.is_contiguous() || !destination.is_contiguous())
        return fail(error, ET_ERR_UNSUPPORTED, "add: operands must be contiguous");
    const uint64_t count = numel(a);
    if (count == 0) return ET_OK;
    if (count > (0x7fffffffull << 8)) return fail(error, ET_ERR_UNSUPPORTED, "add: geometry exceeds the launch limits");
    if (a.data == nullptr || b.data == nullptr || destination.data == nullptr)
        return fail(error, ET_ERR_INVALID, "add: NULL device pointer");
    return launched(add(f32_data(a), f32_data(b), f32_out(destination), count, static_cast<hipStream_t>(stream)), "add",
                    error);
}

int silu_mul_into(const TensorView& gate, const TensorView& up, const TensorView& destination, void* stream,
                  std::string* error) {
    if (gate.dtype != ET_DTYPE_F32 || up.dtype != ET_DTYPE_F32 || destination.dtype != ET_DTYPE_F32)
        return fail(error, ET_ERR_UNSUPPORTED, "silu_mul: only f32 tensors are supported");
    if (gate.shape != up.shape || destination.shape != gate.shape)
        return fail(error, ET_ERR_UNSUPPORTED, "silu_mul: gate, up and the destination must have one shape");
    if (!gate.is_contiguous() || !up.is_contiguous() || !destination.is_contiguous())
        return fail(error, ET_ERR_UNSUPPORTED, "silu_mul: operands must be contiguous");
    const uint64_t count = numel(gate);
    if (count == 0) return ET_OK;
    if (count > (0x7fffffffull << 8)) return fail(error, ET_ERR_UNSUPPORTED, "silu_mul: geometry exceeds the launch limits");
    if (gate.data == nullptr || up.data == nullptr || destination.data == nullptr)
        return fail(error, ET_ERR_INVALID, "silu_mul: NULL device pointer");
    return launched(silu_mul(f32_data(gate), f32_data(up), f32_out(destination), count, static_cast<hipStream_t>(stream)),
                    "silu_mul", error);
}

// validate (crates/runtime/src/sampling.rs:42-57) + the greedy branch (:86-103)
uint64_t greedy_workspace_bytes(uint64_t rows, uint64_t vocabulary) { return argmax_workspace_bytes(rows, vocabulary); }

int greedy_tokens_into(const TensorView& logits, uint32_t* tokens, void* workspace, uint64_t workspace_bytes,
                       void* status, void* stream, std::string* error) {
    if (logits.dtype != ET_DTYPE_F32 || logits.shape.empty())
        return fail(error, ET_ERR_UNSUPPORTED, "sample: logits must be an f32 tensor of rank at least 1");
    const uint64_t columns = logits.shape.back();
    if (columns == 0) return fail(error, ET_ERR_UNSUPPORTED, "sample: logits must be non-empty");
    if (columns > 1048576)
        return fail(error, ET_ERR_UNSUPPORTED, "sample: vocabulary " + std::to_string(columns) + " exceeds limit 1048576");
    if (!logits.is_contiguous()) return fail(error, ET_ERR_UNSUPPORTED, "sample: logits must be contiguous");
    const uint64_t rows = numel(logits) / columns;
    if (rows == 0) return ET_OK;
    if (rows > 0x7fffffffull) return fail(error, ET_ERR_UNSUPPORTED, "sample: too many rows");
    const uint64_t need = argmax_workspace_bytes(rows, columns);
    if (workspace_bytes < need)
        return fail(error, ET_ERR_EXECUTION, "sample: workspace of " + std::to_string(workspace_bytes) +
                                                 " bytes is smaller than the " + std::to_string(need) + " required");
    if (logits.data == nullptr || tokens == nullptr || status == nullptr || workspace == nullptr)
        return fail(error, ET_ERR_INVALID, "sample: NULL device pointer");
    return launched(argmax_rows(f32_data(logits), rows, columns, tokens, static_cast<uint32_t*>(status), workspace,
                                static_cast<hipStream_t>(stream)),
                    "sample", error);
}

int greedy_status_check(uint64_t rows, const void* status_host, std::string* error) {
    for (uint64_t row = 0; row < rows; row++) {
        uint32_t word;
        std::memcpy(&word, static_cast<const char*>(status_host) + 4 * row, sizeof word);
        if (word != 0)  // sampling.rs:94-96
            return fail(error, ET_ERR_EXECUTION, "sample: logit " + std::to_string(word - 1) + " is not finite");
    }
    return ET_OK;
}

// index_select_into along dimension 0 of a [rows, width] table (crates/runtime-cpu/src/indexing.rs:396-430)
int gather_rows_into(const TensorView& table, const TensorView& indexes, const TensorView& destination,
                     void* status, void* stream, std::string* error) {
    if (table.shape.size() != 2)
        return fail(error, ET_ERR_UNSUPPORTED, "index_select: the table must be [rows, width]");
    uint64_t element = 0;
    switch (table.dtype) {
        case ET_DTYPE_F32: case ET_DTYPE_U32: element = 4; break;
        case ET_DTYPE_F16: case ET_DTYPE_BF16: element = 2; break;
        case ET_DTYPE_F64: case ET_DTYPE_I64: element = 8; break;
        case ET_DTYPE_U8: element = 1; break;
        default: return fail(error, ET_ERR_UNSUPPORTED, "index_select: unknown table dtype");
    }
    if (indexes.dtype != ET_DTYPE_U32 && indexes.dtype != ET_DTYPE_I64)
        return fail(error, ET_ERR_UNSUPPORTED, "index_select: indexes must be u32 or i64");
    const uint64_t count = numel(indexes), width = table.shape[1];
    const bool widen = destination.dtype == ET_DTYPE_F32 && (table.dtype == ET_DTYPE_F16 || table.dtype == ET_DTYPE_BF16);
    if ((destination.dtype != table.dtype && !widen) || destination.shape.size() != 2)
        return fail(error, ET_ERR_EXECUTION, "index_select destination rank mismatch: expected 2, got " +
                                                 std::to_string(destination.shape.size()));
    if (destination.shape[0] != count)
        return fail(error, ET_ERR_EXECUTION, "index_select destination shape mismatch at dimension 0: expected " +
                                                 std::to_string(count) + ", got " + std::to_string(destination.shape[0]));
    if (destination.shape[1] != width)
        return fail(error, ET_ERR_EXECUTION, "index_select destination shape mismatch at dimension 1: expected " +
                                                 std::to_string(width) + ", got " + std::to_string(destination.shape[1]));
    if (!table.is_contiguous() || !indexes.is_contiguous() || !destination.is_contiguous())
        return fail(error, ET_ERR_UNSUPPORTED, "index_select: operands must be contiguous");
    if (count == 0 || width == 0) return ET_OK;
    if (count > 0x7fffffffull) return fail(error, ET_ERR_UNSUPPORTED, "index_select: too many indexes");
    if (table.data == nullptr || indexes.data == nullptr || destination.data == nullptr || status == nullptr)
        return fail(error, ET_ERR_INVALID, "index_select: NULL device pointer");
    const char* source = static_cast<const char*>(table.data) + table.offset * element;
    char* target = const_cast<char*>(static_cast<const char*>(destination.data)) + destination.offset * (widen ? 4 : element);
    const bool wide = indexes.dtype == ET_DTYPE_I64;
    const char* ids = static_cast<const char*>(indexes.data) + indexes.offset * (wide ? 8 : 4);
    if (widen)
        return launched(gather_rows_widen(source, table.dtype == ET_DTYPE_BF16 ? 1 : 0, table.shape[0], width, ids,
                                          wide ? 1 : 0, count, reinterpret_cast<float*>(target), status,
                                          static_cast<hipStream_t>(stream)),
                        "index_select", error);
    return launched(gather_rows(source, table.shape[0], width * element, ids, wide ? 1 : 0, count, target, status,
                                static_cast<hipStream_t>(stream)),
                    "index_select", error);
}

int gather_rows_status_check(uint64_t table_rows, uint64_t count, const void* status_host, std::string* error) {
    for (uint64_t p = 0; p < count; p++) {
        unsigned long long word;
        std::memcpy(&word, static_cast<const char*>(status_host) + 8 * p, sizeof word);
        if (word == 0) continue;
        // bit 63 marks the report; bits 0..62 are the index, bit 62 standing for its sign
        long long id = static_cast<long long>(word & ~(1ull << 63));
        if (word & (1ull << 62)) id = static_cast<long long>(word | (1ull << 63));
        return fail(error, ET_ERR_EXECUTION, "index_select: index " + std::to_string(id) +
                                                 " is out of bounds for extent " + std::to_string(table_rows));
    }
    return ET_OK;
}

}  // namespace decode
}  // namespace et
