/*
 * Measurement aid, not part of the runtime's C-ABI: what the matrix cores of
 * device 0 deliver with nothing else going on.  Built into a library of its
 * own (libom_mi355x_measure.so) that only the benchmark and one GPU test load;
 * nothing that a compiled model calls lives here.
 */
#ifndef OM_MI355X_MFMA_CEILING_H
#define OM_MI355X_MFMA_CEILING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Every SIMD of every CU issues v_mfma_i32_32x32x32_i8 back to back from
 * registers for a few milliseconds, no memory traffic.  random_operands = 0:
 * operands of small constants (few bits toggle); 1: operands of random bytes,
 * as a quantized model's are.  Returns 0 and fills *tops (10^12 int8
 * operations per second over the device) and *clock_ghz (the shader clock that
 * rate corresponds to at one such MFMA per 32 clocks and SIMD), or the HIP
 * error code of the call that failed.  Under random operands the device lowers
 * its clock, and no int8 GEMM can exceed what this reports. */
int om_mi355x_measure_mfma_ceiling(int64_t random_operands, double *tops,
    double *clock_ghz);

#ifdef __cplusplus
}
#endif
#endif
