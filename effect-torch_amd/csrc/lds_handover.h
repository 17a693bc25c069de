// Hand-over words in LDS between waves of one workgroup, for kernels whose loader waves keep
// global-to-LDS copies in flight (gemv_limb_dma_kernel, gemv_mma_kernel).
//
// The words are accessed through their LDS addresses with instructions the compiler does not look
// into. LDS serves a wave's requests in order, so "data, then counter" needs no fence; an acquire /
// release at workgroup scope - or any LDS access the compiler can see next to global-to-LDS copies,
// whose destinations it cannot tell from other LDS addresses - would make it wait for every
// outstanding copy (vmcnt 0), exactly what a loader with copies in flight must not do. These accesses
// touch control words only, where no copy lands.
//
// Every wait is bounded: a wave that has polled `limit` times without seeing its count gives up,
// records that in a device word the host can read (Handover::timeouts) and stops waiting for
// anything from then on, so that every wave of the grid reaches the end of the kernel whatever the
// other waves do. The results of such a launch are meaningless; the host reports it as an error.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace et {

// Polls a wave spends on one wait before it gives up: far above any wait of a working launch (a
// whole kernel lasts tens of microseconds, a poll a few hundred cycles), below a second in all.
constexpr uint32_t kHandoverSpinLimit = 1u << 21;

// Device word that counts abandoned waits since the process started (per device), and the limit the
// kernels run with. handover_state() returns both for the current device.
struct HandoverState {
    uint32_t* timeouts;  // device address
    uint32_t limit;
};
hipError_t handover_state(HandoverState* state);
// Test hook: the limit of the launches that follow (0: every wait gives up at once).
void handover_set_spin_limit(uint32_t limit);
// Reads the device word (synchronises with the device).
hipError_t handover_timeouts(uint32_t* count);

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8); }

__device__ __forceinline__ uint32_t lds_address(const void* pointer) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(pointer));  // low half of the flat address
}
__device__ __forceinline__ void lds_store_unseen(uint32_t address, uint32_t value) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(address), "v"(value) : "memory");
}
__device__ __forceinline__ uint32_t lds_read_unseen(uint32_t address) {
    uint32_t value;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(value) : "v"(address) : "memory");
    return value;
}
__device__ __forceinline__ uint32_t lds_count(uint32_t address) {
    return __builtin_amdgcn_readfirstlane(lds_read_unseen(address));
}
__device__ __forceinline__ void lds_arrive(uint32_t address, bool one_lane) {
    // this wave's LDS writes are complete (and the compiler keeps them above this line)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (one_lane) asm volatile("ds_add_u32 %0, %1" : : "v"(address), "v"(1u) : "memory");
}

// Takes the next number from a counter in LDS (what the word held; the word grows by one). Wave-uniform.
__device__ __forceinline__ uint32_t lds_take(uint32_t address, bool one_lane) {
    uint32_t old = 0u;
    if (one_lane) asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=v"(old) : "v"(address), "v"(1u) : "memory");
    return __builtin_amdgcn_readfirstlane(old);
}

// What a wave remembers of its waits.
struct Patience {
    uint32_t limit;      // polls per wait; 0 once a wait has been abandoned
    uint32_t* timeouts;  // device word
    __device__ __forceinline__ void give_up() {
        if ((threadIdx.x & 63u) == 0u && timeouts != nullptr) atomicAdd(timeouts, 1u);
        timeouts = nullptr;  // counted once per wave
        limit = 0u;
    }
};

// Waits until the word at `address` is at least `count`. Returns false when the wave gave up.
__device__ __forceinline__ bool lds_await(uint32_t address, uint32_t count, Patience& patience) {
    for (uint32_t polls = 0;; polls++) {
        if (lds_count(address) >= count) return true;
        if (polls >= patience.limit) break;
        __builtin_amdgcn_s_sleep(1);
    }
    patience.give_up();
    return false;
}

// Waits until the first `need` copies of an image have landed whose copies LOADERS loader waves take in
// turn (copy i is loader i % LOADERS's; landed[j] counts loader j's). One poll reads all the loaders'
// words, a lane each. Returns false when the wave gave up.
template <int LOADERS>
__device__ __forceinline__ bool await_copies_in_turn(const uint32_t* landed, uint32_t lane_id, uint32_t need,
                                                     Patience& patience) {
    const uint32_t loader = lane_id < LOADERS ? lane_id : LOADERS - 1;
    const uint32_t wanted = need > loader ? (need - loader + LOADERS - 1) / LOADERS : 0u;
    const uint32_t address = lds_address(&landed[loader]);
    for (uint32_t polls = 0;; polls++) {
        const uint32_t have = lds_read_unseen(address);
        if (__builtin_amdgcn_ballot_w64(have < wanted) == 0ull) return true;
        if (polls >= patience.limit) break;
        __builtin_amdgcn_s_sleep(1);
    }
    patience.give_up();
    return false;
}

// Waits until at most `left` (wave-uniform, below eight) of this wave's copies are in flight: the
// count of s_waitcnt is an immediate, so one instruction per value.
__device__ __forceinline__ void wait_copies_in_flight(uint32_t left) {
    switch (left) {
        case 0: __builtin_amdgcn_s_waitcnt(vmcnt_only(0)); break;
        case 1: __builtin_amdgcn_s_waitcnt(vmcnt_only(1)); break;
        case 2: __builtin_amdgcn_s_waitcnt(vmcnt_only(2)); break;
        case 3: __builtin_amdgcn_s_waitcnt(vmcnt_only(3)); break;
        case 4: __builtin_amdgcn_s_waitcnt(vmcnt_only(4)); break;
        case 5: __builtin_amdgcn_s_waitcnt(vmcnt_only(5)); break;
        case 6: __builtin_amdgcn_s_waitcnt(vmcnt_only(6)); break;
        case 7: __builtin_amdgcn_s_waitcnt(vmcnt_only(7)); break;
        default: break;
    }
}

}  // namespace et
