// Host side of the quantized operators (plan + execute). See quantized.h.
#include "quantized.h"

#include <hip/hip_runtime_api.h>

#include <cstring>
#include <initializer_list>
#include <limits>
#include <sstream>

#include "et_codecs.h"
#include "kernels.h"

namespace et {
namespace quantized {
namespace {

constexpr uint64_t kMax = std::numeric_limits<uint64_t>::max();

bool checked_mul(uint64_t a, uint64_t b, uint64_t* out) {
    if (a != 0 && b > kMax / a) return false;
    *out = a * b;
    return true;
}

// checked_product, crates/runtime-cpu/src/quantized.rs:44-49
bool checked_product(const std::vector<uint64_t>& values, uint64_t* out) {
    uint64_t total = 1;
    for (uint64_t value : values)
        if (!checked_mul(total, value, &total)) return false;
    *out = total;
    return true;
}

const char* dtype_name(int32_t dtype) {  // DType::name, crates/runtime/src/dtype.rs:38-48
    switch (dtype) {
        case ET_DTYPE_F32: return "f32";
        case ET_DTYPE_F64: return "f64";
        case ET_DTYPE_F16: return "f16";
        case ET_DTYPE_BF16: return "bf16";
        case ET_DTYPE_U8: return "u8";
        case ET_DTYPE_U32: return "u32";
        case ET_DTYPE_I64: return "i64";
        default: return "?";
    }
}

// Rust's `{:?}` of a slice of integers: "[2, 512]".
std::string debug_shape(const std::vector<uint64_t>& shape) {
    std::ostringstream out;
    out << "[";
    for (size_t i = 0; i < shape.size(); i++) out << (i ? ", " : "") << shape[i];
    out << "]";
    return out.str();
}

int fail(std::string* error, int status, const std::string& message) {
    if (error != nullptr) *error = message;
    return status;
}

uint64_t align_up(uint64_t value, uint64_t alignment) {
    return (value + alignment - 1) / alignment * alignment;
}

// GgmlKQuant::encoded_row_bytes (crates/runtime/src/gguf.rs:245-250): false = None.
bool encoded_row_bytes(int32_t codec, uint64_t columns, uint64_t* out) {
    const uint64_t values = block_values(codec);
    if (values == 0 || columns % values != 0) return false;
    return checked_mul(columns / values, block_bytes(codec), out);
}

// validate_weight, crates/runtime-cpu/src/quantized.rs:266-292
int validate_weight(const char* operation, const TensorView& weight, int32_t codec, uint64_t rows,
                    uint64_t columns, uint64_t* row_bytes, std::string* error) {
    const char* name = codec_name(codec);
    if (name == nullptr)
        return fail(error, ET_ERR_INVALID,
                    std::string(operation) + ": unknown codec " + std::to_string(codec));
    if (!encoded_row_bytes(codec, columns, row_bytes))
        return fail(error, ET_ERR_UNSUPPORTED,
                    std::string(operation) + ": logical row width " + std::to_string(columns) +
                        " is invalid for " + name);
    uint64_t total;
    if (!checked_mul(rows, *row_bytes, &total))
        return fail(error, ET_ERR_UNSUPPORTED,
                    std::string(operation) + ": packed weight byte size overflow");
    if (weight.dtype != ET_DTYPE_U8 || weight.shape.size() != 2 || weight.shape[0] != rows ||
        weight.shape[1] != *row_bytes || !weight.is_contiguous() || weight.offset != 0)
        return fail(error, ET_ERR_UNSUPPORTED,
                    std::string(operation) + ": expected exact contiguous packed " + name +
                        " weight [" + std::to_string(rows) + ", " + std::to_string(*row_bytes) +
                        "] u8");
    return ET_OK;
}

// Chooses the kernel for (codec, columns, vectors, mode) and lays out the workspace.
// cf. linear_kernel_kind, crates/runtime-metal/src/quantized.rs:1204-1220.
int select_kernel(et_linear_plan* plan, std::string* error) {
    plan->gather_offset = plan->gather_bytes = 0;
    plan->q_offset = plan->bias_offset = plan->partial_offset = 0;
    plan->k_splits = 1;
    plan->workspace_bytes = 0;
    plan->vectors_per_launch = 0;
    if (plan->vectors == 0 || plan->rows == 0) {
        plan->kernel = LinearKernel::kNone;
        return ET_OK;
    }
    if (plan->rows > 0xffffffffull || plan->columns > 0xffffffffull || plan->vectors > 0xffffffffull)
        return fail(error, ET_ERR_UNSUPPORTED,
                    "quantized_linear: rows, columns and vectors must each fit 32 bits");
    // The workspace, part after part, each at a multiple of 256 bytes. Every size is a checked product
    // (rows, columns and vectors each fit 32 bits, their products times a byte count need not fit 64):
    // one that overflows leaves `fits` false and the plan is refused below.
    uint64_t cursor = 0;
    bool fits = true;
    const auto take = [&](std::initializer_list<uint64_t> factors) -> uint64_t {  // offset of a part of prod(factors) bytes
        const uint64_t offset = cursor;
        uint64_t bytes = 0;
        if (!fits || !checked_product(std::vector<uint64_t>(factors), &bytes) || bytes > kMax - 255 - cursor) {
            fits = false;
            return 0;
        }
        cursor = align_up(cursor + bytes, 256);
        return offset;
    };
    // Space to densify a strided or misaligned f32 input.
    plan->gather_offset = take({plan->vectors, plan->columns, 4});
    plan->gather_bytes = fits ? plan->vectors * plan->columns * 4u : 0;
    plan->bias_offset = take({plan->rows, 4});  // dense copy of a strided bias
    const auto plan_matrix_core = [&](LinearKernel kernel, int limbs) {
        plan->kernel = kernel;
        // activation tiles, see tile_blob_bytes(): one blob per 256-column stage and 32-vector tile
        plan->q_offset = take({(plan->columns + 255) / 256, (plan->vectors + 31) / 32, tile_blob_bytes(limbs)});
        if (limbs == 2) {  // gemm_h16 chooses its own tile height and keeps partial results by whole tiles
            const GemmGroupGeometry g = gemm_h16_group_geometry(plan->codec, &plan->rows, 1, plan->columns, plan->vectors);
            plan->k_splits = g.k_splits;
            if (plan->k_splits > 1) plan->partial_offset = take({g.k_splits, plan->vectors, g.row_tiles, g.tile_rows, 4});
            return;
        }
        plan->k_splits = gemm_i8_k_splits(plan->codec, limbs, plan->rows, plan->columns, plan->vectors);
        if (plan->k_splits > 1) plan->partial_offset = take({plan->k_splits, plan->vectors, plan->rows, 4});
    };
    if (plan->activation_mode == ET_ACT_INT8) {
        if (!gemm_i8_supported(plan->codec, plan->columns))
            return fail(error, ET_ERR_UNSUPPORTED,
                        std::string("quantized_linear: int8 activation mode is not available for ") +
                            codec_name(plan->codec));
        plan_matrix_core(LinearKernel::kGemmI8, 1);
    } else if (plan->activation_mode == ET_ACT_F32) {
        const uint32_t limb_most = gemv_limb_max_vectors(plan->codec);
        const uint32_t limb_launch = static_cast<uint32_t>(plan->vectors < limb_most ? plan->vectors : limb_most);
        if (plan->vectors >= 2 && plan->vectors <= kGemvMmaMaxVectors &&
            gemv_mma_supported(plan->codec, plan->rows, plan->columns, static_cast<uint32_t>(plan->vectors))) {
            // the small-batch regime of the reference's GPU backend (runtime-metal/src/quantized.rs:1204-1220):
            // one pass over W for all the vectors
            plan->kernel = LinearKernel::kGemvMma;
            plan->vectors_per_launch = kGemvMmaMaxVectors;
        } else if (plan->vectors >= kGemmMinVectors && gemm_h16_supported(plan->codec, plan->columns)) {
            plan_matrix_core(LinearKernel::kGemmHalf, 2);
        } else if (plan->vectors >= kGemmMinVectors && gemm_i8_supported(plan->codec, plan->columns)) {
            plan_matrix_core(LinearKernel::kGemmLimb, 3);
        } else if (gemv_limb_supported(plan->codec, plan->columns, limb_launch)) {
            plan->kernel = LinearKernel::kGemvLimb;
            plan->vectors_per_launch = limb_launch;
            // One call is vectors / limb_launch launches of limb_launch vectors and one of the rest; a
            // launch of one vector may take its weights through LDS copies. The name says all of it.
            const auto launch_name = [&](uint64_t vectors) {
                return std::string(gemv_limb_copies_through_lds(plan->codec, plan->rows, plan->columns,
                                                                static_cast<uint32_t>(vectors))
                                       ? "gemv_limb_dma"
                                       : "gemv_limb");
            };
            const uint64_t whole = plan->vectors / limb_launch, rest = plan->vectors % limb_launch;
            plan->kernel_label = launch_name(limb_launch);
            if (whole > 1) plan->kernel_label += " x" + std::to_string(whole);
            if (rest != 0) plan->kernel_label += "+" + launch_name(rest);
        } else {
            plan->kernel = LinearKernel::kGemvGeneric;
            plan->vectors_per_launch = kGemvGenericMaxVectors;
        }
    } else {
        return fail(error, ET_ERR_INVALID, "quantized_linear: unknown activation mode " +
                                               std::to_string(plan->activation_mode));
    }
    if (!fits) return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: workspace byte size overflow");
    plan->workspace_bytes = cursor;
    return ET_OK;
}

hipStream_t as_stream(void* stream) { return static_cast<hipStream_t>(stream); }

int hip_failure(std::string* error, const char* operation, hipError_t status) {
    return fail(error, ET_ERR_EXECUTION,
                std::string(operation) + ": HIP error: " + hipGetErrorString(status));
}

bool cancelled(const volatile int32_t* cancel) { return cancel != nullptr && *cancel != 0; }

// A view is "row-dense" when it can be read as [vectors, columns] with unit
// trailing stride and one common stride between consecutive vectors.
bool row_dense(const TensorView& input, uint64_t* row_stride) {
    const size_t rank = input.shape.size();
    const uint64_t columns = input.shape[rank - 1];
    if (columns > 1 && input.strides[rank - 1] != 1) return false;
    bool have = false;
    uint64_t stride = columns, expected = 0;
    for (size_t d = rank - 1; d-- > 0;) {
        if (input.shape[d] == 1) continue;
        if (!have) {
            have = true;
            stride = input.strides[d];
            if (!checked_mul(stride, input.shape[d], &expected)) return false;
        } else {
            if (input.strides[d] != expected) return false;
            if (!checked_mul(expected, input.shape[d], &expected)) return false;
        }
    }
    *row_stride = stride;
    return true;
}

IndexLayout make_layout(const TensorView& view) {
    IndexLayout layout;
    std::memset(&layout, 0, sizeof layout);
    layout.rank = static_cast<int32_t>(view.shape.size());
    layout.contiguous = view.is_contiguous() ? 1 : 0;
    layout.offset = view.offset;
    for (size_t d = 0; d < view.shape.size(); d++) {
        layout.shape[d] = view.shape[d];
        layout.strides[d] = view.strides[d];
    }
    return layout;
}

}  // namespace

bool TensorView::from_c(const et_tensor* tensor, TensorView* out, std::string* error) {
    if (tensor == nullptr) {
        if (error) *error = "tensor descriptor is NULL";
        return false;
    }
    if (tensor->rank < 0 || tensor->rank > kMaxRank || (tensor->rank > 0 && tensor->shape == nullptr)) {
        if (error) *error = "tensor rank must be 0.." + std::to_string(kMaxRank) + " with a shape array";
        return false;
    }
    out->data = tensor->data;
    out->dtype = tensor->dtype;
    out->offset = tensor->offset;
    out->shape.assign(tensor->shape, tensor->shape + tensor->rank);
    if (tensor->strides != nullptr) {
        out->strides.assign(tensor->strides, tensor->strides + tensor->rank);
    } else {
        // Layout::contiguous, crates/runtime/src/layout.rs:53-67
        out->strides.assign(tensor->rank, 0);
        uint64_t acc = 1;
        for (int d = tensor->rank - 1; d >= 0; d--) {
            out->strides[d] = acc;
            if (d != 0 && !checked_mul(acc, out->shape[d], &acc)) {
                if (error) *error = "layout stride overflow";
                return false;
            }
        }
    }
    return true;
}

bool TensorView::is_contiguous() const {
    uint64_t acc = 1;
    for (size_t d = shape.size(); d-- > 0;) {
        if (shape[d] != 1 && strides[d] != acc) return false;
        if (d != 0 && !checked_mul(acc, shape[d], &acc)) return false;
    }
    return true;
}

const char* kernel_name(const et_linear_plan& plan) {
    switch (plan.kernel) {
        case LinearKernel::kNone: return "none";
        case LinearKernel::kGemvLimb: return plan.kernel_label.c_str();
        case LinearKernel::kGemvGeneric: return "gemv_generic";
        case LinearKernel::kGemvMma: return "gemv_mma";
        case LinearKernel::kGemmI8:
            return plan.k_splits > 1 ? "quantize_act+gemm_i8+reduce" : "quantize_act+gemm_i8";
        case LinearKernel::kGemmLimb:
            return plan.k_splits > 1 ? "quantize_limbs+gemm_i8+reduce" : "quantize_limbs+gemm_i8";
        case LinearKernel::kGemmHalf:
            return plan.k_splits > 1 ? "quantize_halves+gemm_h16+reduce" : "quantize_halves+gemm_h16";
    }
    return "?";
}

int linear_requirements(const TensorView& input, const TensorView& weight, const TensorView* bias,
                        int32_t codec, uint64_t rows, uint64_t columns, int32_t activation_mode,
                        et_linear_plan* plan, std::string* error) {
    warm_device_symbols();
    if (input.dtype != ET_DTYPE_F32 || input.shape.size() < 2)
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: input must be rank >= 2 f32");
    if (input.shape.back() != columns)
        return fail(error, ET_ERR_UNSUPPORTED,
                    "quantized_linear: expected input trailing width " + std::to_string(columns) +
                        ", got " + debug_shape(input.shape));
    uint64_t elements;
    if (!checked_product(input.shape, &elements))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: element count overflow");
    uint64_t row_bytes = 0;
    if (int status = validate_weight("quantized_linear", weight, codec, rows, columns, &row_bytes, error))
        return status;
    if (bias != nullptr) {
        if (bias->dtype != ET_DTYPE_F32 || bias->shape.size() != 1 || bias->shape[0] != rows)
            return fail(error, ET_ERR_UNSUPPORTED,
                        "quantized_linear: bias must be [" + std::to_string(rows) + "] f32, got " +
                            debug_shape(bias->shape) + " " + dtype_name(bias->dtype));
    }
    plan->codec = codec;
    plan->rows = rows;
    plan->columns = columns;
    plan->encoded_row_bytes = row_bytes;
    plan->has_bias = bias != nullptr;
    plan->activation_mode = activation_mode;
    plan->input_shape = input.shape;
    plan->output_shape = input.shape;
    plan->output_shape.back() = rows;
    uint64_t out_elements;
    if (!checked_product(plan->output_shape, &out_elements))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: element count overflow");
    if (!checked_mul(out_elements, 4, &plan->output_bytes))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: output byte size overflow");
    std::vector<uint64_t> leading(input.shape.begin(), input.shape.end() - 1);
    if (!checked_product(leading, &plan->vectors))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: element count overflow");
    return select_kernel(plan, error);
}

int linear_plan_from_sizes(int32_t codec, uint64_t rows, uint64_t columns, uint64_t vectors,
                           bool has_bias, int32_t activation_mode, et_linear_plan* plan,
                           std::string* error) {
    warm_device_symbols();
    TensorView input;
    input.dtype = ET_DTYPE_F32;
    input.shape = {vectors, columns};
    input.strides = {columns, 1};
    uint64_t row_bytes = 0;
    TensorView weight;
    weight.dtype = ET_DTYPE_U8;
    if (!encoded_row_bytes(codec, columns, &row_bytes)) row_bytes = 0;  // reported by validate_weight
    weight.shape = {rows, row_bytes};
    weight.strides = {row_bytes, 1};
    TensorView bias;
    bias.dtype = ET_DTYPE_F32;
    bias.shape = {rows};
    bias.strides = {1};
    return linear_requirements(input, weight, has_bias ? &bias : nullptr, codec, rows, columns,
                               activation_mode, plan, error);
}

namespace {
bool on_matrix_cores(const et_linear_plan& plan) {
    return plan.kernel == LinearKernel::kGemmI8 || plan.kernel == LinearKernel::kGemmLimb ||
           plan.kernel == LinearKernel::kGemmHalf;
}
int limbs_of(const et_linear_plan& plan) {
    return plan.kernel == LinearKernel::kGemmI8 ? 1 : plan.kernel == LinearKernel::kGemmHalf ? 2 : 3;
}
// The contraction over prepared activation tiles, on whichever matrix-core kernel the plan chose.
hipError_t contract_tiles(const et_linear_plan& plan, const uint8_t* weight, const uint8_t* tiles,
                          const GemmOutput& out, hipStream_t stream) {
    if (plan.kernel == LinearKernel::kGemmHalf)
        return gemm_h16(plan.codec, weight, tiles, out, plan.rows, plan.columns, plan.vectors, stream);
    return gemm_i8(plan.codec, limbs_of(plan), weight, tiles, out, plan.rows, plan.columns, plan.vectors, stream);
}
}  // namespace

uint64_t prepared_input_bytes(const et_linear_plan& plan) {
    return on_matrix_cores(plan) ? tile_workspace_bytes(limbs_of(plan), plan.vectors, plan.columns) : 0;
}

int linear_prepare_input(const et_linear_plan& plan, const float* x, uint64_t x_row_stride, void* prepared,
                         uint64_t prepared_bytes, void* stream, std::string* error) {
    if (!on_matrix_cores(plan))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: this plan's kernel takes the activations as they are");
    if (prepared == nullptr || prepared_bytes < prepared_input_bytes(plan))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: prepared-input buffer of " + std::to_string(prepared_bytes) +
                                                 " bytes is smaller than the " + std::to_string(prepared_input_bytes(plan)) +
                                                 " required");
    if (x == nullptr || reinterpret_cast<uintptr_t>(x) % 16 != 0 || x_row_stride % 4 != 0 || x_row_stride < plan.columns ||
        reinterpret_cast<uintptr_t>(prepared) % 16 != 0)
        return fail(error, ET_ERR_INVALID, "quantized_linear: activations and prepared input must be 16-byte aligned rows");
    if (hipError_t status = quantize_tiles(x, x_row_stride, plan.vectors, plan.columns, limbs_of(plan),
                                           static_cast<uint8_t*>(prepared), as_stream(stream)))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

bool fused_prepare(const et_linear_plan& plan) { return plan.kernel == LinearKernel::kGemmHalf; }

int linear_prepare_input_from(const et_linear_plan& plan, const et_prepare_source& source, void* prepared,
                              uint64_t prepared_bytes, void* stream, std::string* error) {
    if (source.kind == ET_PREPARE_PLAIN)
        return linear_prepare_input(plan, source.x, source.x_row_stride, prepared, prepared_bytes, stream, error);
    if (source.kind != ET_PREPARE_RMS_NORM && source.kind != ET_PREPARE_SILU_MUL)
        return fail(error, ET_ERR_INVALID, "quantized_linear: unknown prepared-input kind " + std::to_string(source.kind));
    if (!fused_prepare(plan))
        return fail(error, ET_ERR_UNSUPPORTED,
                    "quantized_linear: this plan's prepared input cannot be computed from an operator on the fly");
    if (prepared == nullptr || prepared_bytes < prepared_input_bytes(plan))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: prepared-input buffer of " + std::to_string(prepared_bytes) +
                                                 " bytes is smaller than the " + std::to_string(prepared_input_bytes(plan)) +
                                                 " required");
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool half_weight = source.kind == ET_PREPARE_RMS_NORM && source.second_dtype == ET_DTYPE_F16;
    if (source.second_dtype != ET_DTYPE_F32 && !half_weight)
        return fail(error, ET_ERR_UNSUPPORTED,
                    "quantized_linear: the second operand must be f32 (an rms norm weight may be f16)");
    const bool second_aligned = half_weight ? reinterpret_cast<uintptr_t>(source.second) % 8 == 0 : aligned(source.second);
    if (source.x == nullptr || !aligned(source.x) || source.x_row_stride % 4 != 0 || source.x_row_stride < plan.columns ||
        !aligned(prepared) || !second_aligned || (source.kind == ET_PREPARE_SILU_MUL && source.second == nullptr))
        return fail(error, ET_ERR_INVALID, "quantized_linear: activations and prepared input must be 16-byte aligned rows");
    hipError_t status;
    if (source.kind == ET_PREPARE_RMS_NORM) {
        if (!(source.eps == source.eps))
            return fail(error, ET_ERR_INVALID, "quantized_linear: rms norm epsilon is not a number");
        status = quantize_tiles_rms_norm(source.x, source.x_row_stride, source.second, half_weight ? 1 : 0, source.eps,
                                         plan.vectors, plan.columns, static_cast<uint8_t*>(prepared), as_stream(stream));
    } else {
        status = quantize_tiles_silu_mul(source.x, static_cast<const float*>(source.second), source.x_row_stride,
                                         plan.vectors, plan.columns, static_cast<uint8_t*>(prepared), as_stream(stream));
    }
    if (status != hipSuccess) return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

namespace {
// What a group launch needs of its members: the same prepared input, all on gemm_h16.
int check_group(const et_linear_plan* const* plans, uint32_t count, std::string* error) {
    if (plans == nullptr || count == 0 || count > kGemmGroupMost)
        return fail(error, ET_ERR_INVALID, "quantized_linear: a group holds 1 to " + std::to_string(kGemmGroupMost) + " plans");
    for (uint32_t i = 0; i < count; i++) {
        if (plans[i] == nullptr) return fail(error, ET_ERR_INVALID, "quantized_linear: plan is NULL");
        if (plans[i]->kernel != LinearKernel::kGemmHalf)
            return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: this plan's kernel has no group launch");
        if (plans[i]->columns != plans[0]->columns || plans[i]->vectors != plans[0]->vectors ||
            plans[i]->codec != plans[0]->codec)
            return fail(error, ET_ERR_INVALID, "quantized_linear: the plans of a group must share columns and vectors and codec");
    }
    return ET_OK;
}
uint64_t group_partial_bytes(const et_linear_plan* const* plans, uint32_t count) {
    uint64_t rows[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) rows[i] = plans[i]->rows;
    return gemm_h16_group_partial_bytes(plans[0]->codec, rows, count, plans[0]->columns, plans[0]->vectors);
}
}  // namespace

int linear_group_workspace_bytes(const et_linear_plan* const* plans, uint32_t count, uint64_t* bytes, std::string* error) {
    if (int rc = check_group(plans, count, error)) return rc;
    *bytes = group_partial_bytes(plans, count);
    return ET_OK;
}

int linear_enqueue_prepared_group(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                  const uint8_t* const* weights, const float* const* biases,
                                  const float* const* residuals, float* const* ys, void* workspace,
                                  uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                                  std::string* error) {
    if (int rc = check_group(plans, count, error)) return rc;
    if (weights == nullptr || ys == nullptr || prepared == nullptr)
        return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
    GemmMember members[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) {
        const float* bias = biases != nullptr ? biases[i] : nullptr;
        if ((bias != nullptr) != plans[i]->has_bias)
            return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias presence does not match the immutable plan");
        if (weights[i] == nullptr || ys[i] == nullptr)
            return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
        members[i] = GemmMember{weights[i], bias, residuals != nullptr ? residuals[i] : nullptr, ys[i], plans[i]->rows};
    }
    if (cancel != nullptr && *cancel != 0) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (plans[0]->vectors == 0) return ET_OK;
    const uint64_t need = group_partial_bytes(plans, count);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                                                 " bytes is smaller than the " + std::to_string(need) + " the group needs");
    if (hipError_t status = gemm_h16_group(plans[0]->codec, members, count, static_cast<const uint8_t*>(prepared),
                                           need > 0 ? static_cast<float*>(workspace) : nullptr, plans[0]->columns,
                                           plans[0]->vectors, as_stream(stream)))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

int linear_enqueue_prepared_group_then_rotary(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                              const uint8_t* const* weights, const float* const* biases,
                                              const float* const* residuals, float* const* ys, void* workspace,
                                              uint64_t workspace_bytes, const et_rotary_after& rotary, void* stream,
                                              const volatile int32_t* cancel, std::string* error) {
    if (int rc = check_group(plans, count, error)) return rc;
    if (rotary.layout != ET_ROTARY_HALF_SPLIT && rotary.layout != ET_ROTARY_INTERLEAVED_PAIRS)
        return fail(error, ET_ERR_INVALID, "rotary: unknown layout " + std::to_string(rotary.layout));
    const uint64_t vectors = plans[0]->vectors;
    if (rotary.head_dim == 0 || rotary.head_dim % 2 != 0 || rotary.head_dim > 0xffffffffull)
        return fail(error, ET_ERR_UNSUPPORTED, "rotary: expected a float rank >= 2 tensor with even head dimension");
    if (rotary.offsets_len != 1 && rotary.offsets_len != vectors)
        return fail(error, ET_ERR_UNSUPPORTED, "rotary embedding: " + std::to_string(rotary.offsets_len) +
                                                   " offsets for batch " + std::to_string(vectors));
    if (rotary.members >> count != 0) return fail(error, ET_ERR_INVALID, "rotary: the group has no such member");
    for (uint32_t i = 0; i < count; i++)
        if (((rotary.members >> i) & 1u) && plans[i]->rows % rotary.head_dim != 0)
            return fail(error, ET_ERR_UNSUPPORTED, "rotary: " + std::to_string(plans[i]->rows) +
                                                       " rows are not whole heads of " + std::to_string(rotary.head_dim));
    if (rotary.members != 0 && vectors != 0 && rotary.offsets == nullptr)
        return fail(error, ET_ERR_INVALID, "rotary: NULL device pointer");
    uint64_t rows[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) rows[i] = plans[i]->rows;
    const bool shares =
        gemm_h16_group_geometry(plans[0]->codec, rows, count, plans[0]->columns, vectors).k_splits > 1 && rotary.members != 0;
    if (!shares) {
        // no second launch to ride on: the group, then the rotary launches
        if (int rc = linear_enqueue_prepared_group(plans, count, prepared, weights, biases, residuals, ys, workspace,
                                                   workspace_bytes, stream, cancel, error))
            return rc;
        for (uint32_t i = 0; i < count && vectors != 0; i++)
            if ((rotary.members >> i) & 1u)
                if (hipError_t status = et::rotary(ys[i], rotary.offsets, static_cast<uint32_t>(rotary.offsets_len), rotary.theta,
                                                   rotary.sign, rotary.layout == ET_ROTARY_INTERLEAVED_PAIRS, ys[i], vectors,
                                                   vectors * (plans[i]->rows / rotary.head_dim), 1, rotary.head_dim,
                                                   as_stream(stream)))
                    return hip_failure(error, "rotary", status);
        return ET_OK;
    }
    if (weights == nullptr || ys == nullptr || prepared == nullptr)
        return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
    GemmMember members[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) {
        const float* bias = biases != nullptr ? biases[i] : nullptr;
        if ((bias != nullptr) != plans[i]->has_bias)
            return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias presence does not match the immutable plan");
        if (weights[i] == nullptr || ys[i] == nullptr)
            return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
        members[i] = GemmMember{weights[i], bias, residuals != nullptr ? residuals[i] : nullptr, ys[i], plans[i]->rows};
    }
    if (cancel != nullptr && *cancel != 0) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (vectors == 0) return ET_OK;
    const uint64_t need = group_partial_bytes(plans, count);
    if (workspace == nullptr || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                                                 " bytes is smaller than the " + std::to_string(need) + " the group needs");
    const GemmRotary after = {rotary.members, rotary.offsets, static_cast<uint32_t>(rotary.offsets_len), rotary.theta,
                              rotary.sign, rotary.layout == ET_ROTARY_INTERLEAVED_PAIRS,
                              static_cast<uint32_t>(rotary.head_dim)};
    if (hipError_t status = gemm_h16_group(plans[0]->codec, members, count, static_cast<const uint8_t*>(prepared),
                                           static_cast<float*>(workspace), plans[0]->columns, vectors, as_stream(stream),
                                           false, &after))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

int linear_enqueue_prepared_group_shares(const et_linear_plan* const* plans, uint32_t count, const void* prepared,
                                         const uint8_t* const* weights, void* workspace, uint64_t workspace_bytes,
                                         et_group_shares* layout, bool launch, void* stream,
                                         const volatile int32_t* cancel, std::string* error) {
    if (int rc = check_group(plans, count, error)) return rc;
    if (layout == nullptr) return fail(error, ET_ERR_INVALID, "quantized_linear: NULL layout");
    static_assert(ET_HIP_LINEAR_GROUP_MOST == kGemmGroupMost, "the header's bound is the kernel's");
    uint64_t rows[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) rows[i] = plans[i]->rows;
    const uint64_t vectors = plans[0]->vectors;
    const GemmGroupGeometry g = gemm_h16_group_geometry(plans[0]->codec, rows, count, plans[0]->columns, vectors);
    *layout = et_group_shares{};
    layout->count = g.k_splits;
    layout->vectors = vectors;
    layout->launch_rows = g.row_tiles * g.tile_rows;
    uint64_t first = 0;
    for (uint32_t i = 0; i < count; i++) {
        layout->first_row[i] = first;
        first += (rows[i] + g.tile_rows - 1) / g.tile_rows * g.tile_rows;
    }
    if (!launch) return ET_OK;
    if (g.k_splits <= 1) return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: this group does not share K over workgroups");
    if (weights == nullptr || prepared == nullptr) return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
    GemmMember members[kGemmGroupMost];
    for (uint32_t i = 0; i < count; i++) {
        if (weights[i] == nullptr) return fail(error, ET_ERR_INVALID, "quantized_linear: NULL device pointer");
        members[i] = GemmMember{weights[i], nullptr, nullptr, nullptr, plans[i]->rows};
    }
    if (cancel != nullptr && *cancel != 0) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    const uint64_t need = group_partial_bytes(plans, count);
    if (workspace == nullptr || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                                                 " bytes is smaller than the " + std::to_string(need) + " the group needs");
    layout->shares = static_cast<const float*>(workspace);
    if (vectors == 0) return ET_OK;
    if (hipError_t status = gemm_h16_group(plans[0]->codec, members, count, static_cast<const uint8_t*>(prepared),
                                           static_cast<float*>(workspace), plans[0]->columns, vectors, as_stream(stream),
                                           true))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

int linear_enqueue_prepared(const et_linear_plan& plan, const void* prepared, const uint8_t* weight, const float* bias,
                            const float* residual, float* y, void* workspace, uint64_t workspace_bytes, void* stream,
                            const volatile int32_t* cancel, std::string* error) {
    if (!on_matrix_cores(plan))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: this plan's kernel takes the activations as they are");
    if ((bias != nullptr) != plan.has_bias)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias does not match the immutable plan");
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (prepared == nullptr || weight == nullptr || y == nullptr)
        return fail(error, ET_ERR_INVALID, "quantized_linear: NULL operand");
    float* partials = nullptr;
    if (plan.k_splits > 1) {
        if (workspace == nullptr || workspace_bytes < plan.workspace_bytes)
            return fail(error, ET_ERR_EXECUTION, "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                                                     " bytes is smaller than the planned " +
                                                     std::to_string(plan.workspace_bytes));
        partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + plan.partial_offset);
    }
    if (hipError_t status = contract_tiles(plan, weight, static_cast<const uint8_t*>(prepared),
                                           GemmOutput{bias, residual, y, partials}, as_stream(stream)))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

int linear_enqueue_prepared_then_norm(const et_linear_plan& plan, const void* prepared, const uint8_t* weight,
                                      const float* bias, const float* residual, float* y, void* workspace,
                                      uint64_t workspace_bytes, const et_linear_plan& next, const void* norm_weight,
                                      int32_t norm_weight_dtype, double eps, void* next_prepared,
                                      uint64_t next_prepared_bytes, void* stream, const volatile int32_t* cancel,
                                      std::string* error) {
    if (next.columns != plan.rows || next.vectors != plan.vectors)
        return fail(error, ET_ERR_INVALID,
                    "quantized_linear: the next contraction must take this one's result: " + std::to_string(plan.vectors) +
                        " x " + std::to_string(plan.rows) + " against " + std::to_string(next.vectors) + " x " +
                        std::to_string(next.columns));
    if (!fused_prepare(next))
        return fail(error, ET_ERR_UNSUPPORTED,
                    "quantized_linear: this plan's prepared input cannot be computed from an operator on the fly");
    if (!(eps == eps)) return fail(error, ET_ERR_INVALID, "quantized_linear: rms norm epsilon is not a number");
    if (norm_weight_dtype != ET_DTYPE_F32 && norm_weight_dtype != ET_DTYPE_F16)
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_linear: an rms norm weight must be f32 or f16");
    const bool half_weight = norm_weight_dtype == ET_DTYPE_F16;
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (y == nullptr || !aligned(y) || !aligned(residual) || !aligned(bias) ||
        reinterpret_cast<uintptr_t>(norm_weight) % (half_weight ? 8 : 16) != 0 || !aligned(next_prepared))
        return fail(error, ET_ERR_INVALID, "quantized_linear: activations and prepared input must be 16-byte aligned rows");
    if (next_prepared == nullptr || next_prepared_bytes < prepared_input_bytes(next))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: prepared-input buffer of " + std::to_string(next_prepared_bytes) +
                                                 " bytes is smaller than the " + std::to_string(prepared_input_bytes(next)) +
                                                 " required");
    // Only a gemm_h16 launch with K shares has a second launch to fold the norm into; every other
    // plan runs the two steps one after the other.
    const bool shares = plan.kernel == LinearKernel::kGemmHalf && plan.k_splits > 1;
    if (!shares) {
        if (int status = linear_enqueue_prepared(plan, prepared, weight, bias, residual, y, workspace, workspace_bytes, stream,
                                                 cancel, error))
            return status;
        et_prepare_source source = {};
        source.kind = ET_PREPARE_RMS_NORM;
        source.x = y;
        source.x_row_stride = plan.rows;
        source.second = norm_weight;
        source.second_dtype = norm_weight_dtype;
        source.eps = eps;
        return linear_prepare_input_from(next, source, next_prepared, next_prepared_bytes, stream, error);
    }
    if ((bias != nullptr) != plan.has_bias)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias does not match the immutable plan");
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (prepared == nullptr || weight == nullptr) return fail(error, ET_ERR_INVALID, "quantized_linear: NULL operand");
    if (workspace == nullptr || workspace_bytes < plan.workspace_bytes)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                                                 " bytes is smaller than the planned " + std::to_string(plan.workspace_bytes));
    float* partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + plan.partial_offset);
    const GemmShares layout = gemm_h16_shares_layout(plan.codec, plan.rows, plan.columns, plan.vectors);
    if (layout.count != plan.k_splits) return fail(error, ET_ERR_EXECUTION, "quantized_linear: K shares do not match the plan");
    GemmOutput out = {bias, residual, y, partials};
    out.leave_shares = true;
    if (hipError_t status = contract_tiles(plan, weight, static_cast<const uint8_t*>(prepared), out, as_stream(stream)))
        return hip_failure(error, "quantized_linear", status);
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (hipError_t status = quantize_tiles_rms_norm_of_shares(partials, layout.count, layout.launch_rows, bias, residual, y,
                                                              norm_weight, half_weight ? 1 : 0, eps, plan.vectors, plan.rows,
                                                              static_cast<uint8_t*>(next_prepared), as_stream(stream)))
        return hip_failure(error, "quantized_linear", status);
    return ET_OK;
}

int linear_enqueue(const et_linear_plan& plan, const float* x, uint64_t x_row_stride,
                   const uint8_t* weight, const float* bias, float* y, void* workspace,
                   uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                   std::string* error) {
    if ((bias != nullptr) != plan.has_bias)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias does not match the immutable plan");
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (plan.kernel == LinearKernel::kNone) return ET_OK;  // empty output: no dispatch
    if (x == nullptr || weight == nullptr || y == nullptr)
        return fail(error, ET_ERR_INVALID, "quantized_linear: NULL operand");
    hipStream_t s = as_stream(stream);
    auto* scratch = static_cast<uint8_t*>(workspace);
    // every part of the workspace starts at a multiple of 256 bytes and is read in 16-byte pieces
    if (scratch != nullptr && reinterpret_cast<uintptr_t>(scratch) % 16 != 0)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: the workspace must be 16-byte aligned");

    // The kernels read activations with 16-byte loads.
    const bool aligned = (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (x_row_stride % 4 == 0) &&
                         x_row_stride >= plan.columns;
    if (!aligned) {
        if (scratch == nullptr || workspace_bytes < plan.gather_offset + plan.gather_bytes)
            return fail(error, ET_ERR_EXECUTION,
                        "quantized_linear: input rows are not 16-byte aligned and the workspace (" +
                            std::to_string(workspace_bytes) + " bytes) cannot hold a dense copy");
        IndexLayout layout;
        std::memset(&layout, 0, sizeof layout);
        layout.rank = 2;
        layout.shape[0] = plan.vectors;
        layout.shape[1] = plan.columns;
        layout.strides[0] = x_row_stride;
        layout.strides[1] = 1;
        float* dense = reinterpret_cast<float*>(scratch + plan.gather_offset);
        if (hipError_t status = gather_f32(x, layout, plan.vectors * plan.columns, dense, s))
            return hip_failure(error, "quantized_linear", status);
        x = dense;
        x_row_stride = plan.columns;
    }

    if (on_matrix_cores(plan)) {
        if (scratch == nullptr || workspace_bytes < plan.workspace_bytes)
            return fail(error, ET_ERR_EXECUTION,
                        "quantized_linear: workspace of " + std::to_string(workspace_bytes) +
                            " bytes is smaller than the planned " +
                            std::to_string(plan.workspace_bytes));
        auto* tiles = scratch + plan.q_offset;
        if (hipError_t status =
                quantize_tiles(x, x_row_stride, plan.vectors, plan.columns, limbs_of(plan), tiles, s))
            return hip_failure(error, "quantized_linear", status);
        // between the launches of one call, as the reference polls between rows (quantized.rs:451,459)
        if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
        float* partials = plan.k_splits > 1 ? reinterpret_cast<float*>(scratch + plan.partial_offset) : nullptr;
        if (hipError_t status = contract_tiles(plan, weight, tiles, GemmOutput{bias, nullptr, y, partials}, s))
            return hip_failure(error, "quantized_linear", status);
        return ET_OK;
    }

    for (uint64_t v0 = 0; v0 < plan.vectors; v0 += plan.vectors_per_launch) {
        if (v0 != 0 && cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
        const uint32_t count = static_cast<uint32_t>(
            plan.vectors - v0 < plan.vectors_per_launch ? plan.vectors - v0 : plan.vectors_per_launch);
        const float* xv = x + v0 * x_row_stride;
        float* yv = y + v0 * plan.rows;
        hipError_t status;
        if (plan.kernel == LinearKernel::kGemvMma)
            status = gemv_mma(plan.codec, weight, xv, x_row_stride, bias, yv, plan.rows, plan.columns, count, s);
        else if (plan.kernel == LinearKernel::kGemvLimb && gemv_limb_supported(plan.codec, plan.columns, count))
            status = gemv_limb(plan.codec, weight, xv, x_row_stride, bias, yv, plan.rows, plan.columns,
                               count, s);
        else
            status = gemv_generic(plan.codec, weight, xv, x_row_stride, bias, yv, plan.rows,
                                  plan.columns, count, s);
        if (status != hipSuccess) return hip_failure(error, "quantized_linear", status);
    }
    return ET_OK;
}

// validate_linear_execution + linear_into, crates/runtime-cpu/src/quantized.rs:367-499
int linear_into(const et_linear_plan& plan, const TensorView& input, const TensorView& weight,
                const TensorView* bias, const TensorView& destination, void* workspace,
                uint64_t workspace_bytes, void* stream, const volatile int32_t* cancel,
                std::string* error) {
    if (input.dtype != ET_DTYPE_F32 || input.shape.size() < 2 || input.shape.back() != plan.columns)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: input does not match the immutable plan");
    std::vector<uint64_t> leading(input.shape.begin(), input.shape.end() - 1);
    uint64_t vectors;
    if (!checked_product(leading, &vectors))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: element count overflow");
    uint64_t output_elements, output_bytes;
    if (!checked_mul(vectors, plan.rows, &output_elements))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: output element count overflow");
    if (!checked_mul(output_elements, 4, &output_bytes))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: output byte size overflow");
    uint64_t row_bytes;
    if (int status = validate_weight("quantized_linear", weight, plan.codec, plan.rows, plan.columns,
                                     &row_bytes, error))
        return status;
    if ((bias != nullptr) != plan.has_bias ||
        (bias != nullptr && (bias->dtype != ET_DTYPE_F32 || bias->shape.size() != 1 ||
                             bias->shape[0] != plan.rows)))
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: bias does not match the immutable plan");
    bool shape_ok = destination.dtype == ET_DTYPE_F32 &&
                    destination.shape.size() == input.shape.size() &&
                    destination.shape.back() == plan.rows;
    for (size_t d = 0; shape_ok && d + 1 < input.shape.size(); d++)
        shape_ok = destination.shape[d] == input.shape[d];
    if (!shape_ok)
        return fail(error, ET_ERR_EXECUTION,
                    "quantized_linear: destination does not match the logical node shape");
    // The plan froze the vector count through its shapes; a different count needs a new plan.
    if (vectors != plan.vectors)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: input does not match the immutable plan");
    // CpuDestination is an exclusive dense output (crates/runtime-cpu/src/tensor.rs:743-760).
    if (!destination.is_contiguous() || destination.offset != 0)
        return fail(error, ET_ERR_EXECUTION, "quantized_linear: destination must be contiguous with zero offset");
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (plan.kernel == LinearKernel::kNone) return ET_OK;

    hipStream_t s = as_stream(stream);
    const float* x = static_cast<const float*>(input.data);
    uint64_t x_row_stride = plan.columns;
    const float* bias_data = nullptr;
    if (bias != nullptr) {
        // bias[source_index(layout, row)]: a strided [rows] view is densified too.
        if (bias->is_contiguous()) {
            bias_data = static_cast<const float*>(bias->data) + bias->offset;
        } else {
            auto* scratch = static_cast<uint8_t*>(workspace);
            if (scratch == nullptr || workspace_bytes < plan.workspace_bytes)
                return fail(error, ET_ERR_EXECUTION,
                            "quantized_linear: strided bias needs the planned workspace of " +
                                std::to_string(plan.workspace_bytes) + " bytes");
            float* dense = reinterpret_cast<float*>(scratch + plan.bias_offset);
            if (hipError_t status = gather_f32(static_cast<const float*>(bias->data),
                                               make_layout(*bias), plan.rows, dense, s))
                return hip_failure(error, "quantized_linear", status);
            bias_data = dense;
        }
    }
    uint64_t stride;
    if (row_dense(input, &stride)) {
        x = static_cast<const float*>(input.data) + input.offset;
        x_row_stride = stride;
    } else {
        auto* scratch = static_cast<uint8_t*>(workspace);
        if (scratch == nullptr || workspace_bytes < plan.gather_offset + plan.gather_bytes)
            return fail(error, ET_ERR_EXECUTION,
                        "quantized_linear: strided input needs a workspace of at least " +
                            std::to_string(plan.gather_offset + plan.gather_bytes) + " bytes");
        float* dense = reinterpret_cast<float*>(scratch + plan.gather_offset);
        const IndexLayout layout = make_layout(input);
        if (hipError_t status = gather_f32(static_cast<const float*>(input.data), layout,
                                           plan.vectors * plan.columns, dense, s))
            return hip_failure(error, "quantized_linear", status);
        x = dense;
        x_row_stride = plan.columns;
    }
    return linear_enqueue(plan, x, x_row_stride, static_cast<const uint8_t*>(weight.data), bias_data,
                          static_cast<float*>(const_cast<void*>(destination.data)), workspace,
                          workspace_bytes, stream, cancel, error);
}

int embedding_requirements(const TensorView& indexes, const TensorView& weight, int32_t codec,
                           uint64_t rows, uint64_t columns, et_embedding_plan* plan,
                           std::string* error) {
    if (indexes.dtype != ET_DTYPE_U32 && indexes.dtype != ET_DTYPE_I64)
        return fail(error, ET_ERR_UNSUPPORTED,
                    std::string("quantized_embedding: indexes must be u32 or i64, got ") +
                        dtype_name(indexes.dtype));
    uint64_t count;
    if (!checked_product(indexes.shape, &count))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_embedding: element count overflow");
    uint64_t row_bytes = 0;
    if (int status = validate_weight("quantized_embedding", weight, codec, rows, columns, &row_bytes, error))
        return status;
    if (columns > 0xffff0000ull)  // the kernel counts columns, in chunks of 1024, in 32 bits
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_embedding: columns must fit 32 bits");
    plan->codec = codec;
    plan->rows = rows;
    plan->columns = columns;
    plan->encoded_row_bytes = row_bytes;
    plan->index_shape = indexes.shape;
    plan->index_dtype = indexes.dtype;
    plan->output_shape = indexes.shape;
    plan->output_shape.push_back(columns);
    plan->count = count;
    uint64_t out_elements;
    if (!checked_product(plan->output_shape, &out_elements))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_embedding: element count overflow");
    if (!checked_mul(out_elements, 4, &plan->output_bytes))
        return fail(error, ET_ERR_UNSUPPORTED, "quantized_embedding: output byte size overflow");
    return ET_OK;
}

// validate_embedding_execution + embedding_into, crates/runtime-cpu/src/quantized.rs:501-616
int embedding_into(const et_embedding_plan& plan, const TensorView& indexes,
                   const TensorView& weight, const TensorView& destination, void* status,
                   void* stream, const volatile int32_t* cancel, std::string* error) {
    if (indexes.dtype != ET_DTYPE_U32 && indexes.dtype != ET_DTYPE_I64)
        return fail(error, ET_ERR_EXECUTION, "quantized_embedding: indexes do not match the immutable plan");
    uint64_t count;
    if (!checked_product(indexes.shape, &count))
        return fail(error, ET_ERR_EXECUTION, "quantized_embedding: element count overflow");
    uint64_t output_elements, output_bytes;
    if (!checked_mul(count, plan.columns, &output_elements))
        return fail(error, ET_ERR_EXECUTION, "quantized_embedding: output element count overflow");
    if (!checked_mul(output_elements, 4, &output_bytes))
        return fail(error, ET_ERR_EXECUTION, "quantized_embedding: output byte size overflow");
    uint64_t row_bytes;
    if (int rc = validate_weight("quantized_embedding", weight, plan.codec, plan.rows, plan.columns,
                                 &row_bytes, error))
        return rc;
    bool shape_ok = destination.dtype == ET_DTYPE_F32 &&
                    destination.shape.size() == indexes.shape.size() + 1 &&
                    destination.shape.back() == plan.columns;
    for (size_t d = 0; shape_ok && d < indexes.shape.size(); d++)
        shape_ok = destination.shape[d] == indexes.shape[d];
    if (!shape_ok)
        return fail(error, ET_ERR_EXECUTION,
                    "quantized_embedding: destination does not match the logical node shape");
    if (!destination.is_contiguous() || destination.offset != 0)
        return fail(error, ET_ERR_EXECUTION,
                    "quantized_embedding: destination must be contiguous with zero offset");
    if (cancelled(cancel)) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    if (count == 0 || plan.columns == 0) return ET_OK;
    if (status == nullptr)
        return fail(error, ET_ERR_INVALID, "quantized_embedding: a device status block is required");
    if (reinterpret_cast<uintptr_t>(destination.data) % 16 != 0)
        return fail(error, ET_ERR_EXECUTION, "quantized_embedding: destination must be 16-byte aligned");
    const IndexLayout layout = make_layout(indexes);
    if (hipError_t rc = dequantize_rows(plan.codec, static_cast<const uint8_t*>(weight.data),
                                        indexes.data, indexes.dtype == ET_DTYPE_I64 ? 1 : 0, layout,
                                        count, plan.rows, plan.columns,
                                        static_cast<float*>(const_cast<void*>(destination.data)), status,
                                        as_stream(stream)))
        return hip_failure(error, "quantized_embedding", rc);
    return ET_OK;
}

int embedding_status_check(const et_embedding_plan& plan, const void* status_host,
                           std::string* error) {
    uint64_t words[2];
    std::memcpy(words, status_host, sizeof words);
    if (words[0] == kMax) return ET_OK;
    // crates/runtime-cpu/src/quantized.rs:570-583: i64 values print signed, u32 unsigned.
    const long long value = static_cast<long long>(words[1]);
    return fail(error, ET_ERR_EXECUTION,
                "quantized_embedding: index " + std::to_string(value) + " is outside 0.." +
                    std::to_string(plan.rows));
}

}  // namespace quantized
}  // namespace et
