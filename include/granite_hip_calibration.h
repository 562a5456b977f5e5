/*
 * granite_hip_calibration.h -- C ABI of libgranite_hip_calibration.so, a measurement aid
 * that ships beside the attention library and is not part of it.  Nothing on the attention
 * path calls it and it has no counterpart in the reference; bench.py's
 * `--workload mfma_calibration` uses it to say what the matrix cores of an MI355X reach
 * (a) with nothing else running and (b) with the other instructions an attention inner
 * loop issues per MFMA beside them, which is the rate an MFMA-bound kernel can be compared
 * with next to the published peak.
 */
#ifndef GRANITE_HIP_CALIBRATION_H
#define GRANITE_HIP_CALIBRATION_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One timed launch of a kernel that issues MFMAs on register operands, one workgroup per
 * compute unit, `waves_per_simd` (1 or 2) waves per SIMD, `iterations` passes of 16
 * v_mfma_f32_32x32x16_f16 (shape 32) or 32 v_mfma_f32_16x16x32_f16 (shape 16) per wave.
 * After every MFMA a wave also issues `fma_per_mfma` float FMAs, `exp_per_mfma` v_exp_f32
 * and `lds_reads_per_mfma` 16-byte LDS reads per lane (conflict free; the data read is the
 * next MFMAs' A operand).  Supported mixes: shape 16 with (0, 0, 0); shape 32 with
 * (fma, exp, lds) in {(0,0,0), (4,0,0), (8,0,0), (0,1,0), (3,1,0), (0,0,1), (3,1,1)}.
 * operands_f16: device memory, n_halves (a multiple of 8, at least 16384) fp16 values: zeros
 * keep the part at its peak clock, values that look like data run it into its power limit.
 * Three untimed launches come first so that the clock is the one under load.  *flops
 * receives the MFMA flops of the timed launch, *milliseconds its duration (HIP events on the
 * default stream of `device`).  Returns 0, -1 for an argument it rejects, or a hipError_t. */
int granite_hip_cal_mfma_rate(int device, const void *operands_f16, uint64_t n_halves,
                              uint32_t iterations, int shape, int waves_per_simd,
                              int fma_per_mfma, int exp_per_mfma, int lds_reads_per_mfma,
                              double *flops, float *milliseconds);

/* The same with the mix given per PAIR of MFMAs (so that half an instruction per MFMA can be
 * asked for: an LDS operand that feeds two MFMAs) and with scalar instructions in it:
 * after every pair a wave issues fma_per_pair float FMAs, exp_per_pair v_exp_f32,
 * lds_reads_per_pair LDS operand reads and salu_per_pair scalar additions, the larger half
 * of each after the first MFMA of the pair (an MFMA with two reads gets its operand as two
 * 8-byte reads, as a V^T operand is read; with one as a 16-byte read).  Supported
 * (fma, exp, lds, salu), shape 32: (0,0,0,0) (8,0,0,0) (16,0,0,0) (0,2,0,0) (6,2,0,0) (0,0,2,0)
 * (6,2,2,0) (6,2,1,0) (6,2,3,0) and the mixes that the hardware counters report for the two
 * prefill kernels, (6,2,3,4) for attention_tiles_dma_kernel and (8,2,3,6) for
 * attention_tiles_kernel, and (7,2,1,2), a 64-rows-per-wave form; shape 16 with (0,0,0,0).  All-zero operands run an
 * instantiation of their own, so that a kernel trace tells them apart.  Everything else as
 * above. */
int granite_hip_cal_mfma_mix(int device, const void *operands_f16, uint64_t n_halves,
                             uint32_t iterations, int shape, int waves_per_simd,
                             int fma_per_pair, int exp_per_pair, int lds_reads_per_pair,
                             int salu_per_pair, double *flops, float *milliseconds);

#ifdef __cplusplus
}
#endif
#endif /* GRANITE_HIP_CALIBRATION_H */
