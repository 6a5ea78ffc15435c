// Definitions shared by the int8 GEMM kernels of gemm_kernels.hip and
// gemm_wreg.hip: vector types, the epilogue's parameter block and small device
// helpers.  Device code only; include inside namespace om.
#pragma once

#include "om_kernels.h"

#include <type_traits>
#include <utility>

namespace om {
namespace gemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v4i_any __attribute__((ext_vector_type(4), aligned(1)));
enum : int { kLoadBytes = 0, kLoadAligned = 1, kLoadAny = 2 };
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BK = kGemmBK;

// Cache policy operand of the buffer stores that carry results: sc1, the
// store is written through to memory when it is issued instead of staying
// dirty in L2 until the kernel ends (2 would be nontemporal, 0 plain).
constexpr int kAuxThrough = 16;
constexpr int kAuxStream = 2;

// Byte offset of 16-byte chunk `c` (0..3) of tile row `r` (row = 64 bytes).
__device__ __forceinline__ int lds_off(int r, int c) {
  return r * BK + ((c ^ ((r >> 2) & 3)) << 4);
}

// A pointer that is the same in every lane, pinned to scalar registers: the
// compiler then addresses memory as (scalar base + 32-bit lane offset) and
// cannot turn base + offset into a per-lane pointer that it advances with
// vector adds.
// A 32-bit lane offset whose widening to 64 bits stays next to its use: hoisted
// out of a loop it would arrive as a 64-bit register pair, and the load would
// then take the per-lane 64-bit address form.
__device__ __forceinline__ uint32_t lane_offset(uint32_t o) {
  asm volatile("" : "+v"(o));
  return o;
}

template <typename T>
__device__ __forceinline__ T *scalar_ptr(T *p) {
  const uint64_t a = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return (T *)(((uint64_t)hi << 32) | lo);
}

// Barrier that orders LDS accesses only; global loads already issued keep
// flying across it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Where a kernel with the f32 epilogue leaves minimum and maximum of what it
// stored (GemmArgs::y_limits): `out`, null when not asked for; one partial
// pair per block; an arrival counter that is zero between launches.
struct LimitsOut {
  float *out;
  float *part_min, *part_max;
  unsigned *counter;
};

struct EpiParams {
  LimitsOut limits;
  // Kernels that quantize an f32 activation themselves (GemmArgs::X): its
  // minimum and maximum when the caller knows them (GemmArgs::x_limits), so
  // that they are not looked for; null otherwise.
  const float *x_limits;
  const void *a_zp;
  int64_t a_zp_len;
  const void *b_zp;
  int64_t b_zp_len;
  bool need_rowsum;      // B carries an offset: row sums of A' are needed
  const int32_t *colsum;
  const float *a_scale;
  const float *b_scale;
  int64_t b_scale_len;
  const float *y_scale;
  const void *y_zp;
  const float *bias;     // kEpiF32: added after the scaling; null = none
  int64_t bias_len;      // 1 or N
  float floor;           // kEpiF32: relu_floor(whether onnx.Relu follows)
  void *out;
  bool b_unsigned;
  bool y_unsigned;
  int narrow;
};

// Called once by every thread of a block of `nwaves` waves (the waves that are
// still running, in uniform control flow) with the minimum and maximum of the
// elements it stored, NaN ignored (+inf / -inf if it stored none).  The block's
// pair goes to its slot; the block that arrives last folds all slots and
// writes L.out[0..1] (the scheme of DynamicQuantizeLinear's reduction kernel:
// partials as device-scope atomic stores, a ticket drawn after they have been
// acknowledged, the counter put back to zero by the last block).
// lds: 2 * nwaves + 1 words nobody else uses any more; sync: a barrier of the
// calling waves that orders LDS.
template <typename Sync>
__device__ __forceinline__ void block_publish_limits(float lo, float hi,
    const LimitsOut &L, float *lds, int wave, int lane, int nwaves, Sync sync) {
  lo = wave_min(lo);
  hi = wave_max(hi);
  if (lane == 0) {
    lds[wave] = lo;
    lds[nwaves + wave] = hi;
  }
  sync();
  if (wave == 0 && lane == 0) {
    for (int w = 1; w < nwaves; ++w) {
      lo = __builtin_fminf(lo, lds[w]);
      hi = __builtin_fmaxf(hi, lds[nwaves + w]);
    }
    __hip_atomic_store(&L.part_min[blockIdx.x], lo, __ATOMIC_RELAXED,
        __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&L.part_max[blockIdx.x], hi, __ATOMIC_RELAXED,
        __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): both stores acknowledged
    const unsigned ticket = __hip_atomic_fetch_add(
        L.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    lds[2 * nwaves] = ticket == gridDim.x - 1 ? 1.0f : 0.0f;
  }
  sync();
  if (lds[2 * nwaves] == 0.0f)
    return;
  // the last block to arrive
  lo = __builtin_inff();
  hi = -__builtin_inff();
  for (unsigned i = wave * 64 + lane; i < gridDim.x; i += nwaves * 64) {
    lo = __builtin_fminf(lo, __hip_atomic_load(&L.part_min[i], __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT));
    hi = __builtin_fmaxf(hi, __hip_atomic_load(&L.part_max[i], __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT));
  }
  lo = wave_min(lo);
  hi = wave_max(hi);
  sync(); // (everyone has read the flag)
  if (lane == 0) {
    lds[wave] = lo;
    lds[nwaves + wave] = hi;
  }
  sync();
  if (wave == 0 && lane == 0) {
    for (int w = 1; w < nwaves; ++w) {
      lo = __builtin_fminf(lo, lds[w]);
      hi = __builtin_fmaxf(hi, lds[nwaves + w]);
    }
    L.out[0] = lo;
    L.out[1] = hi;
    __hip_atomic_store(L.counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// onnx.Relu as the reference lowers it: max(0, x) with the maximum that
// returns the other operand for a NaN
// (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:746-754), so NaN -> 0; a
// negative zero becomes +0.
// Done as one maximum per element whether or not a Relu is asked for: against
// `floor` = 0 when it is, and against a NaN when it is not -- that maximum
// (v_max_f32) returns its other operand unchanged, negative zero included, and
// a NaN only when both are.
__device__ __forceinline__ float relu_f32(float f, float floor) {
  return __builtin_fmaxf(f, floor);
}
inline float relu_floor(bool relu) {
  return relu ? 0.0f : __builtin_nanf("");
}

// onnx.Gelu with approximate = "none" as the reference lowers it
// (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:374-388): (0.5 * x) *
// (1 + erf(x * f32(1 / sqrt 2))), every operation rounded to f32, in this
// order.  The reference's erf is a polynomial approximation that the compiler
// it is built on expands (src/Conversion/KrnlToLLVM/ConvertKrnlToLLVM.cpp:
// 223-225), so no erf reproduces its last bits; this one is
//   erf(m) = sign(m) * (1 - 2^(t * p(t))),  t = min(|m|, 3.925),
// with p of degree 7 fitted (minimax in the error of erf) to log2(erfc(t)) / t
// on [0, 3.925] and the hardware's base-2 exponential: eight multiply-adds, an
// exponential and a subtraction.  Past 3.925, erf rounds to 1 in f32.  Error of
// erf: below 1.5e-7 absolute (0.63 * 2^-22) over the whole line with every
// rounding at its worst, the exponential's one unit in the last place
// included; Gelu needs it absolute, not relative, because the sum 1 + erf is
// what gets multiplied.  Every kernel that applies Gelu calls this function,
// so the result does not depend on which kernel a shape takes.  A NaN gives a
// NaN (through 0.5 * x), +inf gives +inf and -inf gives -inf * 0 = NaN, as the
// formula does.
__device__ __forceinline__ float gelu_erf_f32(float m) {
  const float t = __builtin_fminf(__builtin_fabsf(m), 3.925f);
  float p = -0x1.740ee2p-15f;
  p = __builtin_fmaf(p, t, 0x1.ca2b3ap-12f);
  p = __builtin_fmaf(p, t, -0x1.7ed47ep-10f);
  p = __builtin_fmaf(p, t, -0x1.b09ff2p-11f);
  p = __builtin_fmaf(p, t, 0x1.cfb2b8p-6f);
  p = __builtin_fmaf(p, t, -0x1.302440p-3f);
  p = __builtin_fmaf(p, t, -0x1.d639d0p-1f);
  p = __builtin_fmaf(p, t, -0x1.a0beaap+0f);
  const float e = __builtin_amdgcn_exp2f(p * t);
  return __builtin_copysignf(1.0f - e, m);
}
__device__ __forceinline__ float gelu_f32(float x) {
  const float half_x = 0.5f * x;
  const float e = gelu_erf_f32(x * 0.70710678118654752440f);
  return half_x * (1.0f + e);
}

__device__ __forceinline__ int32_t load_zp_i32(
    const void *p, bool is_unsigned, int64_t i) {
  return is_unsigned ? (int32_t)((const uint8_t *)p)[i]
                     : (int32_t)((const int8_t *)p)[i];
}

// Sum of the 16 int8 values of an MFMA A operand register group (one lane:
// one row, 16 consecutive K bytes).  Kernels add these up over K when the
// epilogue needs rowsum(A'), i.e. when B carries an offset.
__device__ __forceinline__ int32_t frag_rowsum(v4i f) {
  int32_t s = __builtin_amdgcn_sdot4(f.x, 0x01010101, 0, false);
  s = __builtin_amdgcn_sdot4(f.y, 0x01010101, s, false);
  s = __builtin_amdgcn_sdot4(f.z, 0x01010101, s, false);
  return __builtin_amdgcn_sdot4(f.w, 0x01010101, s, false);
}


// Calls f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int,
// N - 1>{}): a loop whose index is a compile-time constant in the body.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(
    F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// k_gemm_i8_wreg (gemm_wreg.hip): whether it takes this problem (wreg_ok),
// whether it is the faster kernel for it (wreg_pays), and its launch.
bool wreg_ok(const GemmArgs &g);
bool wreg_pays(int64_t M, int64_t N);
hipError_t launch_gemm_wreg(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode);

// k_gemm_i8_flight (gemm_flight.hip): problems that one round of blocks covers,
// K a multiple of 256 up to 1024.  The _dq forms take the f32 activation of a dynamically
// quantized layer (GemmArgs::X) and quantize it in the same launch; the launch
// returns hipErrorNotReady when the exchange between blocks cannot be used
// right now (the caller quantizes with a launch of its own instead).
bool flight_ok(const GemmArgs &g, int a_mode);
hipError_t launch_gemm_flight(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode);
bool flight_quantizes_rows(int64_t M, int64_t K, int64_t N, const void *x);
hipError_t launch_gemm_flight_dq(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, DqlScratch &scratch);

} // namespace gemm
} // namespace om
