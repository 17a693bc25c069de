// Codec tables shared by host and device code.
//
// Block sizes follow the reference's GgmlKQuant table
// (crates/runtime/src/gguf.rs:233-241, duplicated in
// crates/runtime-cpu/src/quantized.rs:60-68). Q8_0 and Q4_0 are the public ggml
// legacy layouts; the reference does not implement them.
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#define ET_HD __host__ __device__
#else
#define ET_HD
#endif

namespace et {

enum Codec : int32_t {
    kQ4_0 = 2,
    kQ8_0 = 8,
    kQ2_K = 10,
    kQ3_K = 11,
    kQ4_K = 12,
    kQ5_K = 13,
    kQ6_K = 14,
};

ET_HD constexpr bool codec_known(int32_t codec) {
    return codec == kQ4_0 || codec == kQ8_0 || (codec >= kQ2_K && codec <= kQ6_K);
}

// Logical values per packed block.
ET_HD constexpr uint32_t block_values(int32_t codec) {
    return (codec == kQ4_0 || codec == kQ8_0) ? 32u : (codec >= kQ2_K && codec <= kQ6_K) ? 256u : 0u;
}

// Packed bytes per block.
ET_HD constexpr uint32_t block_bytes(int32_t codec) {
    switch (codec) {
        case kQ4_0: return 18;
        case kQ8_0: return 34;
        case kQ2_K: return 84;
        case kQ3_K: return 110;
        case kQ4_K: return 144;
        case kQ5_K: return 176;
        case kQ6_K: return 210;
        default: return 0;
    }
}

inline const char* codec_name(int32_t codec) {
    switch (codec) {
        case kQ4_0: return "Q4_0";
        case kQ8_0: return "Q8_0";
        case kQ2_K: return "Q2_K";
        case kQ3_K: return "Q3_K";
        case kQ4_K: return "Q4_K";
        case kQ5_K: return "Q5_K";
        case kQ6_K: return "Q6_K";
        default: return nullptr;
    }
}

}  // namespace et
