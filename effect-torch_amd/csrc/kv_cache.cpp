#include "kv_cache.h"

#include <hip/hip_runtime_api.h>

#include <cstring>

#include "kernels.h"

namespace et {
namespace kv {
namespace {

int fail(std::string* error, int status, const std::string& message) {
    *error = message;
    return status;
}

constexpr uint64_t kLimit = 0xffffffffull;

// Geometry of the layer alone; `p` receives what the kernels need of it.
int layer_geometry(const et_kv_layer& layer, KvAttention* p, std::string* error) {
    // NativeKvPool::new (napi/mod.rs:3652-3658)
    if (layer.slab_dtype != ET_DTYPE_F32 && layer.slab_dtype != ET_DTYPE_F16 && layer.slab_dtype != ET_DTYPE_BF16 &&
        layer.slab_dtype != ET_DTYPE_U8)
        return fail(error, ET_ERR_UNSUPPORTED, "kv pool: dtype must be f32, f16, bf16 or u8 (int8-quantized)");
    if (layer.kv_heads == 0 || layer.head_dim == 0 || layer.block_size == 0 || layer.max_tokens == 0)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: empty pool geometry");
    if (layer.max_tokens > kLimit || layer.kv_heads > kLimit || layer.head_dim > kLimit ||
        layer.block_size > kLimit || layer.table_stride > kLimit || layer.slots >= (1ull << 24) ||
        layer.max_context > kLimit || layer.context_window > kLimit)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: geometry exceeds 32-bit positions");
    if (layer.block_size > layer.max_tokens)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: pool smaller than one block");
    if (layer.active_batch > layer.slots)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: active batch " + std::to_string(layer.active_batch) +
                                                   " exceeds " + std::to_string(layer.slots) + " kv slots");
    p->slab_dtype = layer.slab_dtype;
    p->max_tokens = static_cast<uint32_t>(layer.max_tokens);
    p->kv_heads = static_cast<uint32_t>(layer.kv_heads);
    p->width = static_cast<uint32_t>(layer.head_dim);
    p->block_size = static_cast<uint32_t>(layer.block_size);
    p->table_stride = static_cast<uint32_t>(layer.table_stride);
    p->batch = static_cast<uint32_t>(layer.slots);
    p->active_batch = static_cast<uint32_t>(layer.active_batch);
    p->context_window = static_cast<uint32_t>(layer.context_window);
    p->max_context = static_cast<uint32_t>(layer.max_context);
    return ET_OK;
}

int query_geometry(uint64_t query_heads, uint64_t tokens, KvAttention* p, std::string* error) {
    if (p->kv_heads == 0 || query_heads % p->kv_heads != 0 || query_heads == 0)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: incompatible grouped-query q/k/v shapes");
    if (query_heads > kLimit || tokens > kLimit || tokens == 0)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: geometry exceeds 32-bit positions");
    if (p->width > 64u * kKvAnyWidthPerLane)
        return fail(error, ET_ERR_UNSUPPORTED,
                    "kv attention: head width " + std::to_string(p->width) + " is above " +
                        std::to_string(64 * kKvAnyWidthPerLane));
    p->query_heads = static_cast<uint32_t>(query_heads);
    p->tokens = static_cast<uint32_t>(tokens);
    return ET_OK;
}

uint64_t product(const std::vector<uint64_t>& shape, size_t from, size_t to) {
    uint64_t total = 1;
    for (size_t d = from; d < to; d++) total *= shape[d];
    return total;
}

}  // namespace

int workspace_bytes(const et_kv_layer& layer, uint64_t query_heads, uint64_t tokens, uint64_t* bytes,
                    std::string* error) {
    KvAttention p{};
    int status = layer_geometry(layer, &p, error);
    if (status == ET_OK) status = query_geometry(query_heads, tokens, &p, error);
    if (status != ET_OK) return status;
    *bytes = kv_attention_shape(p).workspace_bytes;
    return ET_OK;
}

const char* kernel_name(const et_kv_layer& layer, uint64_t query_heads, uint64_t tokens) {
    KvAttention p{};
    std::string error;
    if (layer_geometry(layer, &p, &error) != ET_OK || query_geometry(query_heads, tokens, &p, &error) != ET_OK)
        return "";
    const KvLaunchShape shape = kv_attention_shape(p);
    if (shape.streaming) return shape.splits > 1 ? "kv_attend+kv_merge" : "kv_attend";
    return shape.splits > 1 ? "kv_attend_any+kv_merge" : "kv_attend_any";
}

int attention_into(const et_kv_layer& layer, const quantized::TensorView& q, const quantized::TensorView& k,
                   const quantized::TensorView& v, double scale, uint64_t window,
                   const quantized::TensorView& destination, void* workspace, uint64_t workspace_bytes,
                   void* status, void* stream, const volatile int32_t* cancel, std::string* error,
                   const et_linear_plan* consumer, void* prepared, uint64_t prepared_bytes,
                   const et_kv_projected* projected) {
    // napi/mod.rs:3331-3344
    const size_t rank = q.shape.size();
    if (rank < 4 || q.dtype != ET_DTYPE_F32 || k.dtype != ET_DTYPE_F32 || v.dtype != ET_DTYPE_F32 ||
        k.shape.size() != rank || v.shape.size() != rank || destination.shape != q.shape ||
        destination.dtype != ET_DTYPE_F32)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: expected matching rank-4-or-higher f32 tensors");
    const uint64_t batch = product(q.shape, 0, rank - 3);
    const uint64_t query_heads = q.shape[rank - 3], tokens = q.shape[rank - 2], width = q.shape[rank - 1];
    const uint64_t kv_heads = k.shape[rank - 3];
    // :3353-3365
    bool compatible = v.shape[rank - 3] == kv_heads && kv_heads != 0 && query_heads % kv_heads == 0 &&
                      k.shape[rank - 2] == tokens && v.shape[rank - 2] == tokens &&
                      k.shape[rank - 1] == width && v.shape[rank - 1] == width;
    for (size_t d = 0; d + 3 < rank; d++)
        compatible = compatible && k.shape[d] == q.shape[d] && v.shape[d] == q.shape[d];
    if (!compatible) return fail(error, ET_ERR_UNSUPPORTED, "kv attention: incompatible grouped-query q/k/v shapes");
    // :3366-3371
    if (batch != layer.slots)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: batch " + std::to_string(batch) +
                                                   " does not match " + std::to_string(layer.slots) + " kv slots");
    // kv_prepare, :3583-3588
    if (kv_heads != layer.kv_heads || width != layer.head_dim)
        return fail(error, ET_ERR_UNSUPPORTED,
                    "kv attention: layer shape [" + std::to_string(kv_heads) + ", " + std::to_string(width) +
                        "] does not match pool geometry [" + std::to_string(layer.kv_heads) + ", " +
                        std::to_string(layer.head_dim) + "]");
    KvAttention p{};
    int code = layer_geometry(layer, &p, error);
    if (code == ET_OK) code = query_geometry(query_heads, tokens, &p, error);
    if (code != ET_OK) return code;
    if (window > kLimit) return fail(error, ET_ERR_UNSUPPORTED, "kv attention: geometry exceeds 32-bit positions");
    if (!q.is_contiguous() || !k.is_contiguous() || !v.is_contiguous() || !destination.is_contiguous())
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: q, k, v and the destination must be contiguous");
    if (batch == 0) return ET_OK;
    if (status == nullptr) return fail(error, ET_ERR_INVALID, "kv attention: status block is NULL");
    if (layer.k_slab == nullptr || layer.v_slab == nullptr || layer.block_table == nullptr ||
        layer.cursors == nullptr || layer.advances == nullptr || destination.data == nullptr ||
        (projected == nullptr && (q.data == nullptr || k.data == nullptr || v.data == nullptr)))
        return fail(error, ET_ERR_INVALID, "kv attention: NULL device pointer");
    if (layer.slab_dtype == ET_DTYPE_U8 &&
        (layer.k_scales == nullptr || layer.v_scales == nullptr || reinterpret_cast<uintptr_t>(layer.k_scales) % 4 != 0 ||
         reinterpret_cast<uintptr_t>(layer.v_scales) % 4 != 0))
        return fail(error, ET_ERR_INVALID, "kv attention: the u8 tier needs its f32 scale slabs");
    p.k_slab = layer.k_slab;
    p.v_slab = layer.v_slab;
    p.k_scales = layer.slab_dtype == ET_DTYPE_U8 ? layer.k_scales : nullptr;
    p.v_scales = layer.slab_dtype == ET_DTYPE_U8 ? layer.v_scales : nullptr;
    p.block_table = layer.block_table;
    p.cursors = layer.cursors;
    p.advances = layer.advances;
    p.window = static_cast<uint32_t>(window);
    if (projected == nullptr) {
        p.q = static_cast<const float*>(q.data) + q.offset;
        p.k = static_cast<const float*>(k.data) + k.offset;
        p.v = static_cast<const float*>(v.data) + v.offset;
    } else {
        // the projections as the group launch left them: shares of rows [q | k | v], each from its own first row
        const et_group_shares& s = projected->shares;
        const uint64_t q_rows = query_heads * width, kv_rows = kv_heads * width;
        if (tokens != 1) return fail(error, ET_ERR_UNSUPPORTED, "kv attention: projections as K shares take one token per slot");
        if (s.shares == nullptr || reinterpret_cast<uintptr_t>(s.shares) % 4 != 0 || s.count == 0 || s.count > kLimit ||
            s.vectors != batch || s.launch_rows > kLimit || projected->q_member >= ET_HIP_LINEAR_GROUP_MOST ||
            projected->k_member >= ET_HIP_LINEAR_GROUP_MOST || projected->v_member >= ET_HIP_LINEAR_GROUP_MOST)
            return fail(error, ET_ERR_INVALID, "kv attention: the K shares do not describe [" + std::to_string(batch) +
                                                   "] projected vectors");
        const uint64_t q_row = s.first_row[projected->q_member], k_row = s.first_row[projected->k_member],
                       v_row = s.first_row[projected->v_member];
        // a projection ends where the next member of the launch (or the launch) does
        const auto room = [&](uint64_t first) {
            uint64_t end = s.launch_rows;
            for (uint64_t other : s.first_row)
                if (other > first && other < end) end = other;
            return first <= end ? end - first : 0;
        };
        if (q_rows > room(q_row) || kv_rows > room(k_row) || kv_rows > room(v_row) || k_row == v_row || q_row == k_row ||
            q_row == v_row)
            return fail(error, ET_ERR_INVALID, "kv attention: the projections do not fit the rows of the shares");
        if (projected->layout != ET_ROTARY_HALF_SPLIT && projected->layout != ET_ROTARY_INTERLEAVED_PAIRS)
            return fail(error, ET_ERR_INVALID, "rotary: unknown layout " + std::to_string(projected->layout));
        if (width % 2 != 0)
            return fail(error, ET_ERR_UNSUPPORTED, "rotary: expected a float rank >= 2 tensor with even head dimension");
        if (projected->offsets_len != 1 && projected->offsets_len != batch)
            return fail(error, ET_ERR_UNSUPPORTED, "rotary embedding: " + std::to_string(projected->offsets_len) +
                                                       " offsets for batch " + std::to_string(batch));
        if (projected->offsets == nullptr) return fail(error, ET_ERR_INVALID, "rotary: NULL device pointer");
        p.projected = KvProjected{s.shares, s.count, static_cast<uint32_t>(batch), s.launch_rows,
                                  static_cast<uint32_t>(q_row), static_cast<uint32_t>(k_row), static_cast<uint32_t>(v_row),
                                  projected->q_bias, projected->k_bias, projected->v_bias, projected->offsets,
                                  static_cast<uint32_t>(projected->offsets_len),
                                  projected->layout == ET_ROTARY_INTERLEAVED_PAIRS ? 1 : 0, projected->theta, projected->sign};
    }
    p.out = const_cast<float*>(static_cast<const float*>(destination.data)) + destination.offset;
    p.scale = scale;
    p.status = status;
    if (consumer != nullptr) {
        // the result as the activations of the contraction that follows: one row per slot
        if (tokens != 1 || consumer->columns != query_heads * width || consumer->vectors != batch)
            return fail(error, ET_ERR_UNSUPPORTED,
                        "kv attention: the prepared input of a contraction takes one token per slot and [" +
                            std::to_string(batch) + ", " + std::to_string(query_heads * width) + "] activations");
        if (!quantized::fused_prepare(*consumer))
            return fail(error, ET_ERR_UNSUPPORTED,
                        "quantized_linear: this plan's prepared input cannot be computed from an operator on the fly");
        if (prepared == nullptr || reinterpret_cast<uintptr_t>(prepared) % 16 != 0 ||
            prepared_bytes < quantized::prepared_input_bytes(*consumer))
            return fail(error, ET_ERR_EXECUTION, "quantized_linear: prepared-input buffer of " + std::to_string(prepared_bytes) +
                                                     " bytes is smaller than the " +
                                                     std::to_string(quantized::prepared_input_bytes(*consumer)) + " required");
        if (reinterpret_cast<uintptr_t>(p.out) % 16 != 0)
            return fail(error, ET_ERR_INVALID, "quantized_linear: activations and prepared input must be 16-byte aligned rows");
        p.prepared = static_cast<uint8_t*>(prepared);
    }
    const KvLaunchShape shape = kv_attention_shape(p);
    if (projected != nullptr && !shape.streaming)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: this geometry's kernel takes q, k and v as tensors");
    if (shape.streaming) {
        // the streaming kernel moves 16 bytes per lane
        const auto misaligned = [](const void* pointer) { return reinterpret_cast<uintptr_t>(pointer) % 16 != 0; };
        if (misaligned(p.k_slab) || misaligned(p.v_slab))
            return fail(error, ET_ERR_INVALID, "kv attention: slabs must be 16-byte aligned");
    }
    if (shape.workgroups > 0x7fffffffull)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: launch exceeds the grid limit");
    if (workspace_bytes < shape.workspace_bytes || (shape.workspace_bytes != 0 && workspace == nullptr))
        return fail(error, ET_ERR_EXECUTION,
                    "kv attention: workspace of " + std::to_string(workspace_bytes) + " bytes is smaller than the " +
                        std::to_string(shape.workspace_bytes) + " required");
    if (cancel != nullptr && *cancel != 0) return fail(error, ET_ERR_CANCELLED, "operation aborted");
    const hipError_t launched = kv_attention(p, workspace, static_cast<hipStream_t>(stream));
    if (launched != hipSuccess)
        return fail(error, ET_ERR_EXECUTION, std::string("kv attention: HIP error: ") + hipGetErrorString(launched));
    return ET_OK;
}

int attention_projected_into(const et_kv_layer& layer, const et_kv_projected& projected, double scale, uint64_t window,
                             const quantized::TensorView& destination, void* workspace, uint64_t workspace_bytes,
                             void* status, void* stream, const volatile int32_t* cancel, std::string* error,
                             const et_linear_plan* consumer, void* prepared, uint64_t prepared_bytes) {
    // q is the destination's shape; k and v that of the layer's heads, one token each
    const size_t rank = destination.shape.size();
    if (rank < 4 || destination.dtype != ET_DTYPE_F32)
        return fail(error, ET_ERR_UNSUPPORTED, "kv attention: expected matching rank-4-or-higher f32 tensors");
    quantized::TensorView q = destination, k = destination;
    q.data = nullptr;
    k.data = nullptr;
    k.offset = 0;
    k.shape[rank - 3] = layer.kv_heads;
    uint64_t stride = 1;
    for (size_t d = rank; d-- > 0;) {  // contiguous
        k.strides[d] = stride;
        stride *= k.shape[d];
    }
    return attention_into(layer, q, k, k, scale, window, destination, workspace, workspace_bytes, status, stream, cancel,
                          error, consumer, prepared, prepared_bytes, &projected);
}

int status_check(const et_kv_layer& layer, uint64_t tokens, const void* status_host, std::string* error) {
    // the first failing slot, as the reference's loop over the slots would meet it
    unsigned long long word = 0;
    uint64_t slot = 0;
    for (; slot < layer.slots && word == 0; slot++)
        std::memcpy(&word, static_cast<const char*>(status_host) + 8 * slot, sizeof word);
    if (word == 0) return ET_OK;
    slot -= 1;
    const uint64_t code = word >> 56, value = word & 0x00ffffffffffffffull;
    switch (code) {
        case kKvBadAdvance:  // napi/mod.rs:3590-3594
            return fail(error, ET_ERR_EXECUTION,
                        "kv attention: advance " + std::to_string(value) + " out of range for chunk length " +
                            std::to_string(tokens));
        case kKvOverCapacity:  // :3597-3603
            return fail(error, ET_ERR_EXECUTION,
                        "kv attention: live context " + std::to_string(value) + " exceeds pool capacity " +
                            std::to_string(layer.max_tokens));
        case kKvShortTable:
            return fail(error, ET_ERR_EXECUTION,
                        "kv attention: block table of slot " + std::to_string(slot) + " does not cover " +
                            std::to_string(value) + " tokens");
        case kKvOverDeclared:
            return fail(error, ET_ERR_EXECUTION,
                        "kv attention: slot " + std::to_string(slot) + " needs " + std::to_string(value) +
                            " tokens, above the declared max_context " + std::to_string(layer.max_context));
        case kKvBlockOutside:
            return fail(error, ET_ERR_EXECUTION,
                        "kv attention: slot " + std::to_string(slot) + " maps to row " + std::to_string(value) +
                            " outside the pool of " + std::to_string(layer.max_tokens));
        default:
            return fail(error, ET_ERR_EXECUTION, "kv attention: unknown device status " + std::to_string(word));
    }
}

}  // namespace kv
}  // namespace et
