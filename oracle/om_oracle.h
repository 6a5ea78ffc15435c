/*
 * CPU oracle for the onnx-mlir int8 quantized-inference path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing that ships may call into this library:
 * it exists so that tests, the smoke check and the benchmark's CPU-baseline
 * leg can compare the HIP path against an independent restatement of what the
 * reference's CPU lowering computes.
 *
 * Every function restates, operation for operation, the arithmetic that the
 * reference's ONNX->Krnl lowering emits (each op is a single IEEE-754 binary32
 * operation or a two's-complement int32 operation, so a C restatement compiled
 * with -ffp-contract=off -fno-fast-math is bit-identical by construction).
 * The reference file:line each function follows is cited in om_oracle.c.
 *
 * Parity status per function (what pins it is listed in om_oracle.c):
 *   om_oracle_rne, quantize (per-tensor), dequantize (per-tensor),
 *   dynamic_quantize, matmul_integer, qlinear_matmul, dequant_epilogue, relu:
 *   pinned by the reference's enabled ONNX node-test vectors, its constant-
 *   propagation lit answers and closed forms.
 *   quantize / dequantize PER-AXIS: "parity unpinned" -- the reference's CPU
 *   lowering asserts on per-axis scales, so there is no reference output; the
 *   per-tensor formula is applied with scale[c], zp[c] and checked against the
 *   ONNX operator specification's per-axis node vectors only.
 *   gelu: "parity unpinned" at the bit level -- the reference expands erf
 *   with a polynomial approximation pass of the compiler it is built on, not
 *   held in its tree, and stores no Gelu outputs; libm's erff stands in, and
 *   comparisons with this function carry a tolerance of a few units in the
 *   last place of erf.
 */
#ifndef OM_ORACLE_H
#define OM_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element kinds for the quantized side. */
enum { OM_ORACLE_U8 = 0, OM_ORACLE_I8 = 1, OM_ORACLE_I32 = 2 };

/* Compiler options that change the quantize arithmetic (bits of `mode`). */
enum { OM_ORACLE_RECIPROCAL = 1, OM_ORACLE_NO_ZERO_POINT = 2 };

/* QLinearMatMul narrowing modes. */
enum { OM_ORACLE_WRAP = 0, OM_ORACLE_SATURATE = 1 };

float om_oracle_rne(float x);
/* Values among the `count` bit patterns from `first_bits` on that
 * om_oracle_rne and rintf round differently (0 expected). */
int64_t om_oracle_rne_sweep(uint32_t first_bits, int64_t count);

/* y = cast(clip(rne(x / scale) + zp)).  The tensor is viewed as
 * [outer, channels, inner]; scale/zp have `channels` entries (channels == 1
 * and inner == n for per-tensor).  zp may be NULL (no zero point).
 * qkind: OM_ORACLE_U8 or OM_ORACLE_I8; zp points at elements of that kind. */
void om_oracle_quantize_linear(const float *x, int64_t outer, int64_t channels,
    int64_t inner, const float *scale, const void *zp, int qkind, void *y);

/* y = (f32(x) - f32(zp)) * scale; xkind U8 / I8 / I32, zp of the same kind. */
void om_oracle_dequantize_linear(const void *x, int xkind, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    float *y);

/* NaN-ignoring full-tensor min / max (init +inf / -inf). */
void om_oracle_minmax(const float *x, int64_t n, float *mn, float *mx);

/* scale / zero point from min / max. */
void om_oracle_dynamic_params(
    float xmin, float xmax, float *scale, float *zp_f32, uint8_t *zp_u8);

/* DynamicQuantizeLinear: y u8[n], scale f32, zp u8. */
void om_oracle_dynamic_quantize_linear(
    const float *x, int64_t n, uint8_t *y, float *scale, uint8_t *zp);

/* MatMulInteger: Y[M,N] = (A - a_zp) x (B - b_zp), int32 wrap.
 * akind / bkind: U8 or I8.  a_zp: NULL, 1 entry, or M entries (per row);
 * b_zp: NULL, 1 entry, or N entries (per column); kinds follow A / B.
 * This entry is a plain triple loop. */
void om_oracle_matmul_integer(const void *A, int akind, const void *B,
    int bkind, int64_t M, int64_t K, int64_t N, const void *a_zp,
    int64_t a_zp_len, const void *b_zp, int64_t b_zp_len, int32_t *Y);

/* Same result as om_oracle_matmul_integer, organised as the reference's CPU
 * code is: int32 copies of A and B are materialised in separate passes, the
 * zero points are subtracted in separate passes, the result is zeroed and an
 * int32 GEMM blocked 4x8x8 runs with OpenMP over row tiles.  Used as the timed
 * CPU baseline. */
void om_oracle_matmul_integer_passes(const void *A, int akind, const void *B,
    int bkind, int64_t M, int64_t K, int64_t N, const void *a_zp,
    int64_t a_zp_len, const void *b_zp, int64_t b_zp_len, int32_t *Y);

/* QLinearMatMul.  a/b/y kinds U8 or I8 (zero points follow their tensor's
 * kind).  mode WRAP is what the reference computes, SATURATE what the ONNX
 * specification says. */
void om_oracle_qlinear_matmul(const void *A, int akind, float a_scale,
    const void *a_zp, int64_t a_zp_len, const void *B, int bkind,
    float b_scale, const void *b_zp, int64_t b_zp_len, float y_scale,
    const void *y_zp, int ykind, int64_t M, int64_t K, int64_t N, int mode,
    void *Y);

/* QuantizeLinear / DynamicQuantizeLinear as compiled with --enable-fast-math
 * (mode & 1: x * (1 / scale)) and / or --disable-quantization-zero-point
 * (mode & 2).  mode 0 equals the functions without the suffix. */
void om_oracle_quantize_linear_mode(const float *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    int qkind, void *y, int mode);
void om_oracle_dynamic_quantize_linear_mode(const float *x, int64_t n,
    uint8_t *y, float *scale, uint8_t *zp, int mode);

/* out[i,j] = f32(acc[i,j]) * (a_scale * b_scale[j or 0]). */
void om_oracle_dequant_epilogue(const int32_t *acc, int64_t M, int64_t N,
    float a_scale, const float *b_scale, int64_t b_scale_len, float *out);

/* out[i] = max(0, x[i]); NaN -> 0. */
void om_oracle_relu(const float *x, int64_t n, float *out);

/* out[i] = (0.5 * x[i]) * (1 + erf(x[i] * f32(1 / sqrt 2))), erf by libm. */
void om_oracle_gelu(const float *x, int64_t n, float *out);

/* The reference's pass structure for Q / DQ / DQL with OpenMP, used only as
 * the timed CPU baseline (results identical to the functions above). */
void om_oracle_quantize_linear_omp(const float *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    int qkind, void *y);
void om_oracle_dequantize_linear_omp(const void *x, int xkind, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    float *y);
void om_oracle_dynamic_quantize_linear_omp(
    const float *x, int64_t n, uint8_t *y, float *scale, uint8_t *zp);

int om_oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
