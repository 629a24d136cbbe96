/* lten_hip_measure.h — calibration kernels behind the roofline figures (liblten_hip_measure.so).
 *
 * NOT part of the drop-in surface: nothing here replaces an l-ten interface, l-ten never calls it, and the product
 * library liblten_hip.so neither contains nor needs it.  bench.py and the profile commands use it to state measured
 * fractions against what this part sustains, beside the published peaks.  Everything runs on the null stream;
 * return value 0 on success, else a message is available from lten_measure_last_error().
 */
#ifndef LTEN_HIP_MEASURE_H
#define LTEN_HIP_MEASURE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* lten_measure_last_error(void);

/* The MFMA issue rate sustained by a kernel that does nothing else.  kind 0: int8 32x32x32 in tera-ops/s; kind 1: fp32
 * 32x32x2 in TFLOP/s; kinds 2 and 3: the same two on uniform pseudo-random operands that change with every MFMA;
 * 1..8 wavefronts per SIMD. */
int lten_measure_mfma_peak(int kind, int waves_per_simd, float* tera_per_s);
/* The int8 loop on operands taken from a product's own matrices (device pointers, 16-byte aligned, `bytes` each):
 * a_u8 holds uint8 activations (sign-flipped in registers, as the GEMM does), b_i8 prepared int8 weights.  The rate
 * the matrix pipes alone sustain on data of that distribution. */
int lten_measure_mfma_peak_operands(const void* a_u8, const void* b_i8, uint64_t bytes, int waves_per_simd, float* tera_per_s);
/* After an int8 measurement: shader clocks per MFMA as one wavefront sees them, and the shader clock in MHz over the
 * loop (shader clock counter against the 100 MHz wall clock). */
int lten_measure_last_clocks(double* cycles_per_mfma, double* shader_mhz);
/* A plain copy with 16-byte accesses: 2 * bytes of HBM traffic, for scaling profiler byte counters. */
int lten_measure_copy(const void* device_src, void* device_dst, uint64_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* LTEN_HIP_MEASURE_H */
