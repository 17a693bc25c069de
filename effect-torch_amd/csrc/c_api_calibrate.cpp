// extern "C" surface of libet_hip_calibrate.so (declared in include/et_hip_calibrate.h): the
// measurement aids, apart from the operators' library. Same conventions as c_api.cpp: no exception
// crosses the boundary, the message of a failure is kept per thread.
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <exception>
#include <new>
#include <string>

#include "et_hip.h"
#include "et_hip_calibrate.h"
#include "kernels.h"

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

}  // namespace

extern "C" {

int et_hip_calibration_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups,
                            void* stream) {
    return guarded([&](std::string* error) -> int {
        if (src == nullptr || sink == nullptr || workgroups == 0 || (bytes >> 36) != 0 ||
            reinterpret_cast<uintptr_t>(src) % 16 != 0) {
            *error = "calibration_read: source must be 16-byte aligned, sink non-NULL, workgroups > 0";
            return ET_ERR_INVALID;
        }
        const hipError_t status =
            et::calibration_read(src, bytes, sink, workgroups, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("calibration_read: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

int et_hip_calibration_read_variant(int32_t variant, const void* src, uint64_t bytes, uint32_t* sink,
                                    uint32_t workgroups, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (src == nullptr || sink == nullptr || workgroups == 0 || workgroups > 65536 || (bytes >> 36) != 0 ||
            reinterpret_cast<uintptr_t>(src) % 16 != 0 || variant < ET_READ_PLAIN || variant > ET_READ_LDS_8_NT_RANGES_SHALLOW) {
            *error = "calibration_read_variant: variant 0..8, source 16-byte aligned, sink non-NULL, "
                     "1 <= workgroups <= 65536";
            return ET_ERR_INVALID;
        }
        const hipError_t status =
            et::calibration_read_variant(variant, src, bytes, sink, workgroups, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("calibration_read_variant: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

int et_hip_calibration_copy(const void* src, void* dst, uint64_t bytes, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (src == nullptr || dst == nullptr || reinterpret_cast<uintptr_t>(src) % 16 != 0 ||
            reinterpret_cast<uintptr_t>(dst) % 16 != 0) {
            *error = "calibration_copy: buffers must be non-NULL and 16-byte aligned";
            return ET_ERR_INVALID;
        }
        const hipError_t status =
            et::calibration_copy(src, dst, bytes, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("calibration_copy: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

int et_hip_calibration_mfma(int32_t kind, uint32_t iterations, uint32_t workgroups, float* sink, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (sink == nullptr || workgroups == 0 || workgroups > 65536 || iterations == 0 || iterations > (1u << 20) ||
            kind < ET_MFMA_I8 || kind > ET_MFMA_I8_BIASED_VALU_ONLY) {
            *error = "calibration_mfma: kind 0..7, 1 <= iterations <= 2^20, 1 <= workgroups <= 65536, sink non-NULL";
            return ET_ERR_INVALID;
        }
        const hipError_t status = et::calibration_mfma(kind, iterations, workgroups, sink, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) {
            *error = std::string("calibration_mfma: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

int et_hip_calibration_contraction(int32_t probe, const void* weight, const void* prepared, float* y, uint64_t rows,
                                   uint64_t columns, uint64_t vectors, void* stream) {
    return guarded([&](std::string* error) -> int {
        if (weight == nullptr || prepared == nullptr || y == nullptr || probe < ET_CONTRACTION_WHOLE ||
            probe > ET_CONTRACTION_ACTIVATION_COPIES_ONLY || reinterpret_cast<uintptr_t>(prepared) % 16 != 0) {
            *error = "calibration_contraction: probe 0..6, operands non-NULL, prepared input 16-byte aligned";
            return ET_ERR_INVALID;
        }
        const hipError_t status =
            et::gemm_h16_probe(probe, static_cast<const uint8_t*>(weight), static_cast<const uint8_t*>(prepared), y, rows,
                               columns, vectors, static_cast<hipStream_t>(stream));
        if (status == hipErrorInvalidValue) {
            *error = "calibration_contraction: a Q4_K shape of 64-row tiles without K shares and at most 32 vectors";
            return ET_ERR_UNSUPPORTED;
        }
        if (status != hipSuccess) {
            *error = std::string("calibration_contraction: HIP error: ") + hipGetErrorString(status);
            return ET_ERR_EXECUTION;
        }
        return ET_OK;
    });
}

const char* et_hip_calibration_last_error(void) { return g_last_error.c_str(); }

}  // extern "C"
