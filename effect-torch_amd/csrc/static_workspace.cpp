// quantized_linear for callers that cannot allocate device memory and bring no workspace:
// et_hip_linear_enqueue with the workspace in a device array that the library's code object
// carries. Code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc
// are who it is for; the reference has no counterpart (its backends own their scratch).
//
// `scratch` is ONE array per GPU, held from the first use of the library on that GPU until the
// process ends, and every call on a GPU uses it: calls that overlap in time on one GPU (two
// streams, two threads) race on it and must be serialised by the caller. A call needs the bytes
// et_hip_linear_plan_workspace_bytes reports for its plan; plans that need more than
// ET_HIP_STATIC_WORKSPACE_BYTES are refused. What a call finds in the array is what the last call
// left there: the kernels write every byte they later read (activation tiles, K-share partials,
// the dense copy of strided input rows), nothing has to start at zero.
#include <hip/hip_runtime.h>

#include <atomic>
#include <string>

#include "et_hip.h"
#include "lds_handover.h"
#include "quantized.h"

static __device__ __align__(256) uint8_t scratch[ET_HIP_STATIC_WORKSPACE_BYTES];

namespace et {
namespace {

constexpr int kMostDevices = 64;
std::atomic<uint8_t*> g_scratch_of[kMostDevices];

// The array's address on the current device. In host code `scratch` is only a handle for the
// runtime, not a device address: the address comes from hipGetSymbolAddress, once per device (each
// GPU holds its own copy of the array at its own address), and only that pointer is used afterwards.
int scratch_pointer(uint8_t** out, std::string* error) {
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) {
        *error = std::string("quantized_linear: hipGetDevice: ") + hipGetErrorString(status);
        return ET_ERR_EXECUTION;
    }
    if (device < 0 || device >= kMostDevices) {
        *error = "quantized_linear: device " + std::to_string(device) + " is outside 0.." + std::to_string(kMostDevices);
        return ET_ERR_UNSUPPORTED;
    }
    uint8_t* pointer = g_scratch_of[device].load(std::memory_order_acquire);
    if (pointer == nullptr) {
        void* address = nullptr;
        if (hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch))) {
            *error = std::string("quantized_linear: hipGetSymbolAddress(scratch): ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        if (address == nullptr || reinterpret_cast<uintptr_t>(address) % 256 != 0) {
            *error = "quantized_linear: the static workspace has no usable device address";
            return ET_ERR_EXECUTION;
        }
        pointer = static_cast<uint8_t*>(address);
        g_scratch_of[device].store(pointer, std::memory_order_release);  // every thread would store the same value
    }
    *out = pointer;
    return ET_OK;
}

}  // namespace

namespace quantized {

void warm_device_symbols() {
    // Looks up, outside any stream capture, the device addresses that launches need later: the static
    // workspace's and the hand-over status word's (hipGetSymbolAddress may load the code object).
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();  // no device: plans can still be made (and checked) on the host
        return;
    }
    uint8_t* pointer = nullptr;
    std::string ignored;
    (void)scratch_pointer(&pointer, &ignored);
    HandoverState handover;
    (void)handover_state(&handover);
    (void)hipGetLastError();
}

int linear_enqueue_static_workspace(const et_linear_plan& plan, const float* x, uint64_t x_row_stride,
                                    const uint8_t* weight, const float* bias, float* y, void* stream,
                                    const volatile int32_t* cancel, std::string* error) {
    const uint64_t needed = plan.workspace_bytes;
    if (needed > ET_HIP_STATIC_WORKSPACE_BYTES) {
        *error = "quantized_linear: this plan needs a workspace of " + std::to_string(needed) +
                 " bytes, the static workspace holds " + std::to_string(ET_HIP_STATIC_WORKSPACE_BYTES) +
                 "; use et_hip_linear_enqueue with a workspace of the caller's";
        return ET_ERR_UNSUPPORTED;
    }
    uint8_t* pointer = nullptr;
    if (int status = scratch_pointer(&pointer, error)) return status;
    return linear_enqueue(plan, x, x_row_stride, weight, bias, y, pointer, ET_HIP_STATIC_WORKSPACE_BYTES, stream, cancel,
                          error);
}

}  // namespace quantized
}  // namespace et
