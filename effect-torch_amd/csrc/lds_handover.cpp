// Host side of lds_handover.h: the device word that counts abandoned waits and the poll limit.
#include "lds_handover.h"

#include <atomic>
#include <mutex>

namespace et {
namespace {

__device__ uint32_t handover_timeout_count = 0;

std::atomic<uint32_t> spin_limit{kHandoverSpinLimit};
std::mutex lookup;
uint32_t* word_of_device[64] = {};

}  // namespace

hipError_t handover_state(HandoverState* state) {
    int device = 0;
    if (hipError_t status = hipGetDevice(&device)) return status;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lookup);
    if (word_of_device[device] == nullptr) {
        void* address = nullptr;
        // every device holds its own copy of the word at its own address
        if (hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(handover_timeout_count))) return status;
        word_of_device[device] = static_cast<uint32_t*>(address);
    }
    state->timeouts = word_of_device[device];
    state->limit = spin_limit.load(std::memory_order_relaxed);
    return hipSuccess;
}

void handover_set_spin_limit(uint32_t limit) { spin_limit.store(limit, std::memory_order_relaxed); }

hipError_t handover_timeouts(uint32_t* count) {
    HandoverState state;
    if (hipError_t status = handover_state(&state)) return status;
    return hipMemcpy(count, state.timeouts, sizeof *count, hipMemcpyDeviceToHost);
}

}  // namespace et
