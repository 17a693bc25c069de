/* Measurement aids: plain reads, a plain copy, matrix-core loops and the batched contraction taken apart.
 *
 * These entry points live in a library of their own, libet_hip_calibrate.so, apart from the
 * operator boundary (et_hip.h, libet_hip.so): they mirror nothing in the reference and nothing on
 * the operator path calls them. The benchmark's calibrate_* workloads and two tests load it to put
 * the rates this device sustains next to the published peaks and to calibrate hardware counters
 * against a known number of bytes. Failures return an et_status (et_hip.h); the message is
 * et_hip_calibration_last_error() on the calling thread.
 */
#ifndef ET_HIP_CALIBRATE_H
#define ET_HIP_CALIBRATE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming read (`workgroups` workgroups of 256 lanes, each a
 * contiguous range, 16-byte loads; `sink` receives four words per workgroup; at
 * most 2^36 bytes) and a
 * plain 16-byte copy, both of `bytes` rounded down to 16. They measure the
 * bandwidth this device delivers to a kernel of a given footprint and calibrate
 * hardware counters against a known number of bytes. They have no counterpart
 * in the reference and are not part of the operator path. */
int et_hip_calibration_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups,
                            void* stream);

/* The same read by other kernels, to tell what the device delivers from what one read kernel
 * reaches. `sink` holds at least 4 * workgroups words (at least 1024 for the LDS variants).
 *   ET_READ_PLAIN     et_hip_calibration_read: four 16-byte loads in flight per lane, then the next four
 *   ET_READ_DEEP      sixteen 16-byte loads in flight per lane
 *   ET_READ_STREAMING ET_READ_DEEP with non-temporal loads
 *   ET_READ_LDS_4 / ET_READ_LDS_8   one workgroup of 4 / 8 waves per `workgroups` entry that only issue
 *                     1 KiB global-to-LDS copies (no registers, no arithmetic), each wave keeping
 *                     32 / 16 KiB of copies in flight in a ring of LDS slots.
 * ET_READ_LDS_8_NT: ET_READ_LDS_8 with non-temporal copies; _NT_SHALLOW: the same with 4 KiB in
 *                     flight per wave; _NT_RANGES: every wave copies its own contiguous eighth of the
 *                     workgroup's range instead of every eighth KiB of it; _NT_RANGES_SHALLOW: both. */
enum {
    ET_READ_PLAIN = 0, ET_READ_DEEP = 1, ET_READ_STREAMING = 2, ET_READ_LDS_4 = 3, ET_READ_LDS_8 = 4,
    ET_READ_LDS_8_NT = 5, ET_READ_LDS_8_NT_SHALLOW = 6, ET_READ_LDS_8_NT_RANGES = 7,
    ET_READ_LDS_8_NT_RANGES_SHALLOW = 8
};
int et_hip_calibration_read_variant(int32_t variant, const void* src, uint64_t bytes, uint32_t* sink,
                                    uint32_t workgroups, void* stream);
int et_hip_calibration_copy(const void* src, void* dst, uint64_t bytes, void* stream);

/* Loops of matrix-core instructions that touch no memory: `workgroups` workgroups of four waves,
 * every wave `iterations` rounds of four independent instructions of one kind, all operands ones;
 * `sink` receives one float per thread (256 * workgroups), the sum of what the thread accumulated.
 * ET_MFMA_I8: v_mfma_i32_32x32x32_i8 (65 536 operations each); ET_MFMA_I8_SCALED: the same
 * instruction followed by the f32 epilogue of a contraction whose operands both carry a scale per 32
 * columns (a tile of scale products from v_mfma_f32_32x32x2f32, one convert and one multiply-add per
 * element); ET_MFMA_F16: v_mfma_f32_32x32x16_f16 (32 768 operations); ET_MFMA_F16_16X16:
 * v_mfma_f32_16x16x32_f16 (16 384); ET_MFMA_I8_SCALED_BF16: ET_MFMA_I8_SCALED with the scale products from
 * v_mfma_f32_32x32x16_bf16 (scales split into exact bfloat16 pieces); ET_MFMA_I8_BIASED: the step of the
 * int8 batch kernel as it runs now (integer sums that start at the bits of 1.5 * 2^23, one subtraction and
 * one multiply-add per element, each matrix instruction followed by half of them), ..._MATRIX_ONLY and
 * ..._VALU_ONLY its matrix and its VALU instructions alone. They measure what the matrix cores of this device sustain, the
 * ceiling the batch kernels are compared with next to the published peak. No counterpart in the
 * reference, not part of the operator path. */
enum { ET_MFMA_I8 = 0, ET_MFMA_I8_SCALED = 1, ET_MFMA_F16 = 2, ET_MFMA_F16_16X16 = 3, ET_MFMA_I8_SCALED_BF16 = 4,
       ET_MFMA_I8_BIASED = 5, ET_MFMA_I8_BIASED_MATRIX_ONLY = 6, ET_MFMA_I8_BIASED_VALU_ONLY = 7 };
int et_hip_calibration_mfma(int32_t kind, uint32_t iterations, uint32_t workgroups, float* sink, void* stream);

/* The batched Q4_K contraction (64-row tiles, at most 32 vectors, a shape that does not share K over
 * workgroups, e.g. 14336 x 4096) taken apart: the kernel as the operator path launches it
 * (ET_CONTRACTION_WHOLE), without its consumer waves' arithmetic (every copy, wait and barrier stays),
 * without its copies (arithmetic and barriers stay), without the weight or the activation copies
 * alone, and with the weight or the activation copies and no arithmetic. `prepared` is what et_hip_linear_prepare_input left for a plan of these sizes; y
 * [vectors, rows] receives the result for ET_CONTRACTION_WHOLE and meaningless values otherwise.
 * The durations say which of the two - the path into LDS or the instruction stream - a change has
 * to shorten. No counterpart in the reference, not part of the operator path. */
enum { ET_CONTRACTION_WHOLE = 0, ET_CONTRACTION_NO_ARITHMETIC = 1, ET_CONTRACTION_NO_COPIES = 2,
       ET_CONTRACTION_NO_WEIGHT_COPIES = 3, ET_CONTRACTION_NO_ACTIVATION_COPIES = 4,
       ET_CONTRACTION_WEIGHT_COPIES_ONLY = 5, ET_CONTRACTION_ACTIVATION_COPIES_ONLY = 6 };
int et_hip_calibration_contraction(int32_t probe, const void* weight, const void* prepared, float* y,
                                   uint64_t rows, uint64_t columns, uint64_t vectors, void* stream);

const char* et_hip_calibration_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* ET_HIP_CALIBRATE_H */
