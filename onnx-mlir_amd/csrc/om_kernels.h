// Internal interface between the runtime (OMTensor marshalling, residency)
// and the gfx950 kernels.  Everything here works on GPU pointers only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace om {

enum QKind : int { kU8 = 0, kI8 = 1, kI32 = 2 };
enum Epilogue : int { kEpiI32 = 0, kEpiF32 = 1, kEpiQ8 = 2 };
enum NarrowMode : int { kWrap = 0, kSaturate = 1 };

// ---- quantize / dequantize (HBM-bound streaming kernels) ------------------
// The tensor is viewed as [outer, channels, inner]; scale / zp have `channels`
// entries.  channels == 1 is the per-tensor case.  zp may be null.
// reciprocal: quantize as the reference does when compiled with
// --enable-fast-math, x * (1 / scale) in place of x / scale.
hipError_t launch_quantize(hipStream_t s, const float *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    bool is_signed, void *y, bool reciprocal = false);

hipError_t launch_dequantize(hipStream_t s, const void *x, QKind xkind,
    int64_t outer, int64_t channels, int64_t inner, const float *scale,
    const void *zp, float *y);

// Scratch a DynamicQuantizeLinear launch needs: per-block partial min / max
// and an arrival counter of the two-launch path, which must be zero before the
// first launch (the kernel leaves it zero), and the per-block slots of the
// one-launch kernel.
struct DqlScratch {
  float *partial_min; // [max_blocks]
  float *partial_max; // [max_blocks]
  unsigned *counter;  // [16], zeroed once: [0] two-pass arrivals, [8] set if
                      // the exchange of the one-launch kernel ever timed out
  int grid_blocks;    // dql_grid_blocks(), or 0 to disable the one-launch path
  unsigned spin_limit; // polls a thread of the one-launch kernel waits for
                       // another block's result before giving up
  unsigned long long *grid_slots; // [2 * max_blocks], 16-byte aligned,
                      // zeroed once: per block two words, (launch number
                      // << 32 | float bits) of its min and of its max
  unsigned epoch;     // launch number of the one-launch kernel (host side)
  int max_blocks;     // capacity of partial_min / partial_max and blocks
                      // that grid_slots has room for (at most kDqlMaxBlocks)
  // Two-launch path only (sets grid_blocks to 0 for the call).
  DqlScratch two_launch() const {
    DqlScratch s = *this;
    s.grid_blocks = 0;
    return s;
  }
};
// Blocks of the one-launch DynamicQuantizeLinear kernel that fit the current
// device at once (0 if it cannot run here).
int dql_grid_blocks();
constexpr int kDqlMaxBlocks = 4096;

// y u8[n], scale f32[1], zp u8[1].  If y_shift is true the stored bytes are
// y ^ 0x80 (the value minus 128 as int8), the form the GEMM consumes, and
// row sums are not needed because they are not produced here.
// mode: bits of OM_MI355X_QUANT_* (reciprocal quotient, no zero point); any
// mode but 0 takes the small-tensor kernel or the two-launch path.
hipError_t launch_dynamic_quantize(hipStream_t s, DqlScratch &scratch,
    const float *x, int64_t n, uint8_t *y, float *scale, uint8_t *zp,
    bool y_shift, int mode = 0);
constexpr int kQuantReciprocal = 1, kQuantNoZeroPoint = 2;

// Minimum and maximum of a tensor handed from the op that produced it to the
// DynamicQuantizeLinear that consumes it: limits[0] = min, limits[1] = max
// over all elements with NaN ignored, zero not yet included (what the
// reference's two reductions give,
// src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:100-110).
struct QuantLimits {
  const float *limits; // null: not known
  float *scale_out;    // where the derived scale and zero point go
  uint8_t *zp_out;
  int no_zp;           // kQuantNoZeroPoint
};
hipError_t launch_quantize_from_limits(hipStream_t s, const float *x, int64_t n,
    const float *limits, uint8_t *y, float *scale, uint8_t *zp, bool y_shift,
    int mode = 0);
hipError_t launch_minmax_limits(hipStream_t s, DqlScratch &scratch,
    const float *x, int64_t n, float *limits_out);

// The tagged-slot exchange between the blocks of one launch (k_dql_grid, the
// fused layer of k_gemm_i8_flight).  At most one kernel that uses it may be in
// flight per process: two of them dispatched at the same time from different
// streams could each hold part of the device and wait for the rest.
// dql_exchange_begin returns false when the exchange is switched off
// (scratch.grid_blocks == 0) or the last such kernel was launched on another
// stream that is still busy; otherwise it fills `x` with this launch's number
// and the slots, and holds a lock until dql_exchange_end, which the caller
// calls right after queuing its kernel on `s` (launched: whether it did).
struct GridExchange {
  unsigned long long *slots;
  unsigned epoch;
  unsigned *failed;
  unsigned spin_limit;
};
bool dql_exchange_begin(hipStream_t s, DqlScratch &scratch, GridExchange &x);
void dql_exchange_end(hipStream_t s, bool launched);

// Call before destroying a stream that launch_dynamic_quantize was given.
void dql_forget_stream(hipStream_t s);

// ---- int8 GEMM ------------------------------------------------------------
// B [K,N] row-major (u8 or i8) -> Bp, Npad * Kpad bytes of int8 in MFMA
// operand order: Bp[n/32][k/64][half step][lane][16 B], u8 shifted to int8
// by -128, zero filled outside [N,K]; colsum[n] = sum_k of the int8 values
// written (int32), colsum has Npad entries.
constexpr int kGemmBK = 64;    // K granularity of the packed operand
constexpr int kGemmBN = 256;   // N granularity of the packed operand (largest tile)
inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

hipError_t launch_pack_b(hipStream_t s, const void *B, bool b_unsigned,
    int64_t K, int64_t N, int8_t *Bp, int32_t *colsum);

struct GemmArgs {
  // If set (see gemm_quantizes_rows): the activation as f32 [M,K]; the kernel
  // quantizes it itself as DynamicQuantizeLinear would (A, a_zp and a_scale
  // are then not read).  `dql`: the scratch whose exchange slots the blocks
  // use where they have to agree on minimum and maximum across the grid.
  const float *X;
  DqlScratch *dql;
  const void *A;       // [M,K] row-major, u8 or i8
  bool a_unsigned;     // A holds u8
  bool a_preshifted;   // A already holds (u8 - 128) as int8; offsets as for u8
  const int8_t *Bp;    // B in MFMA operand order (launch_pack_b)
  bool b_unsigned;     // original B was u8 (packed values are B - 128)
  int64_t M, K, N;
  const void *a_zp;    // element type follows A; may be null
  int64_t a_zp_len;    // 0, 1 or M
  const void *b_zp;    // element type follows B; may be null
  int64_t b_zp_len;    // 0, 1 or N
  const int32_t *colsum; // sum_k B' per column (Npad entries)
  Epilogue epi;
  // kEpiF32: out = f32(acc) * (a_scale[0] * b_scale[j or 0]) [+ bias[j or 0]]
  // kEpiQ8 : s = (a_scale[0]*b_scale[0]) / y_scale[0];
  //          out = narrow(i32(rne(f32(acc) * s)) + y_zp)
  const float *a_scale;
  const float *b_scale;
  int64_t b_scale_len; // 1 or N
  const float *y_scale;
  const void *y_zp;
  const float *bias;   // kEpiF32 only; may be null
  int64_t bias_len;    // 1 or N
  // kEpiF32 only: onnx.Relu on the result, max(0, x) with a NaN giving 0
  // (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:746-754).
  bool relu;
  // kEpiF32 only: onnx.Gelu (approximate = "none") on the result instead,
  // applied by a pass of its own after the product.
  bool gelu;
  bool y_unsigned;
  NarrowMode narrow;
  void *out;           // i32 / f32 / u8|i8 [M,N]
  // kEpiF32 only, optional: receives minimum and maximum of `out` (see
  // QuantLimits) for the DynamicQuantizeLinear that reads it next.  Kernels
  // that can, reduce them in their epilogue (partial results and arrival
  // counter in `dql`, which must be set); behind the others a pass over `out`
  // does.
  float *y_limits;
  // With X, optional: minimum and maximum of X as an earlier product's
  // y_limits gave them; the kernel then does not look for them.
  const float *x_limits;
};

hipError_t launch_gemm(hipStream_t s, const GemmArgs &g);
// Name of the kernel the calling thread's last launch_gemm chose.
const char *last_gemm_kernel();

// Whether launch_gemm can take an f32 activation of this shape in GemmArgs::X:
// 0 no; 1 yes, every block quantizes the rows for itself; 2 yes, the blocks
// agree on minimum and maximum through the exchange slots of GemmArgs::dql
// (one-launch rules of DynamicQuantizeLinear apply: launch_gemm answers
// hipErrorNotReady when the exchange cannot be used right now -- the caller
// then quantizes with DynamicQuantizeLinear and passes A -- and a block that
// gives up waiting raises the scratch's flag).
int gemm_quantizes_rows(int64_t M, int64_t K, int64_t N, const void *x);
// Whether the caller should hand `a` over as rows of round_up(K, 16) bytes
// made by launch_pad_rows (few rows, K % 16 != 0 or a misaligned start), and
// pass that length as K.  a_zp: the rows' zero point(s) on the GPU (null: 0),
// one or one per row; stored_minus_128: rows hold (u8 - 128).
bool gemm_pads_rows(int64_t M, int64_t K, const void *a);
hipError_t launch_pad_rows(hipStream_t s, const void *a, int64_t M, int64_t K,
    const void *a_zp, int64_t a_zp_len, bool stored_minus_128, void *out);

// Fill n 32-bit words with v.
hipError_t launch_fill_u32(hipStream_t s, uint32_t *p, int64_t n, uint32_t v);

#if defined(__HIPCC__)
// ---- device arithmetic shared by the quantize and GEMM kernels ------------
// One element of QuantizeLinear, operation for operation as the reference's
// generated code (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp
// :119-144): IEEE divide, round half to even, separate add of the zero point,
// maxnum then minnum (NaN -> lower bound), float -> integer.
//
// The divide.  x / s correctly rounded costs eleven vector instructions
// (scaling of operands near the ends of the exponent range, a reciprocal
// estimate, two refinement steps, the final correction and fix-up).  When the
// reciprocal r = RN(1 / s) is at hand -- computed once per scale with that
// same divide -- a single correction step gives the correctly rounded quotient:
//     q0 = RN(x * r);  e = x - q0 * s (exact in one fma);  q = RN(q0 + e * r)
// (Markstein's theorem: a faithful q0 and a correctly rounded r suffice), as
// long as nothing under- or overflows on the way.  That holds for "tame"
// scales, 2^-96 <= s <= 2^96, and quotients of magnitude 2^-3 .. 2^10; a
// smaller quotient may be off by an ulp, which cannot change its rounding to
// the integer 0, and q0 is clamped to +-1024 first, so that a larger one (or
// an infinite x, for which e would be a NaN) stays beyond +-1023, where the
// 8-bit result saturates whatever the zero point; a NaN x stays a NaN.
// quotient<true> therefore gives the same 8-bit result as x / s for every x,
// in four instructions.  Checked against the divide on the CPU
// (tests/quotient_check.c: random pairs and every neighbour of a rounding
// boundary, no difference in 2.9e10 pairs) and on the GPU by the boundary test
// of the parity suite.  Any other scale (zero,
// negative, denormal, huge, infinite, NaN) takes quotient<false>, the divide.
__device__ __forceinline__ bool scale_is_tame(float s) {
  return s >= 0x1p-96f && s <= 0x1p96f;
}
// QMODE 0: the divide; 1: the corrected reciprocal form above (same result);
// 2: x * r and nothing else -- what the reference computes when it is
// compiled with --enable-fast-math at -O3
// (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:43-44,119-132),
// a different result by design, for any scale.
template <int QMODE>
__device__ __forceinline__ float quotient(float x, float s, float r) {
  if (QMODE == 0)
    return x / s;
  if (QMODE == 2)
    return x * r;
  const float q0 =
      __builtin_fminf(__builtin_fmaxf(x * r, -1024.0f), 1024.0f);
  const float e = __builtin_fmaf(-q0, s, x);
  return __builtin_fmaf(e, r, q0);
}

// rne(x / s) + zp, not yet clamped.
template <bool HAS_ZP, int QMODE>
__device__ __forceinline__ float quant_value(
    float x, float s, float r, float zpf) {
  float v = __builtin_rintf(quotient<QMODE>(x, s, r));
  if (HAS_ZP)
    v = v + zpf;
  return v;
}

template <bool SIGNED, bool HAS_ZP, int QMODE = 0>
__device__ __forceinline__ uint32_t quant_one(
    float x, float s, float zpf, float r = 0.0f) {
  const float v = quant_value<HAS_ZP, QMODE>(x, s, r, zpf);
  if (SIGNED) {
    float c = __builtin_fminf(__builtin_fmaxf(v, -128.0f), 127.0f);
    return (uint32_t)((int32_t)c) & 0xFFu;
  }
  float c = __builtin_fminf(__builtin_fmaxf(v, 0.0f), 255.0f);
  return (uint32_t)c;
}

// Four values into the bytes of one word.  Unsigned: v_cvt_pk_u8_f32 converts
// with saturation to 0 .. 255 and writes the byte in place; its input is
// already an integer (or an infinity, which saturates, or a NaN, which gives
// 0 = the lower bound, as maxnum-then-minnum does), so its own rounding never
// acts.
template <bool SIGNED, bool HAS_ZP, int FAST>
__device__ __forceinline__ uint32_t quant_pack4(float x0, float x1, float x2,
    float x3, float s0, float s1, float s2, float s3, float r0, float r1,
    float r2, float r3, float z0, float z1, float z2, float z3) {
  if (SIGNED) {
    return quant_one<true, HAS_ZP, FAST>(x0, s0, z0, r0) |
           (quant_one<true, HAS_ZP, FAST>(x1, s1, z1, r1) << 8) |
           (quant_one<true, HAS_ZP, FAST>(x2, s2, z2, r2) << 16) |
           (quant_one<true, HAS_ZP, FAST>(x3, s3, z3, r3) << 24);
  }
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      quant_value<HAS_ZP, FAST>(x0, s0, r0, z0), 0, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      quant_value<HAS_ZP, FAST>(x1, s1, r1, z1), 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      quant_value<HAS_ZP, FAST>(x2, s2, r2, z2), 2, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      quant_value<HAS_ZP, FAST>(x3, s3, r3, z3), 3, w);
  return w;
}

// minnum / maxnum from +inf / -inf (src/Conversion/ONNXToKrnl/Math/
// Reduction.cpp:529-548); the order of a min / max reduction does not change
// its value, so lanes, waves and blocks may combine in any order.
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    v = __builtin_fminf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    v = __builtin_fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Scale and zero point of DynamicQuantizeLinear from min / max
// (src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:43-84).
// no_zp: compiled with --disable-quantization-zero-point, the zero point is 0
// (DynamicQuantizeLinear.cpp:75-84); adding that 0 changes no result.
__device__ __forceinline__ void dynamic_params(
    float xmin, float xmax, float &scale, float &zpf, bool no_zp = false) {
  const float mx = __builtin_fmaxf(xmax, 0.0f);
  const float mn = __builtin_fminf(xmin, 0.0f);
  const float xdiff = mx - mn;
  const float bound = 255.0f - 0.0f;
  scale = xdiff / bound;
  const float inter = 0.0f - mn / scale;
  const float sat = __builtin_fminf(__builtin_fmaxf(inter, 0.0f), 255.0f);
  zpf = no_zp ? 0.0f : __builtin_rintf(sat);
}
#endif

} // namespace om
