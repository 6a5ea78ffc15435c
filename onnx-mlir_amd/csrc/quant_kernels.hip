// QuantizeLinear / DequantizeLinear / DynamicQuantizeLinear for gfx950.
//
// All three are HBM-bound streaming kernels: every lane moves 16 bytes per
// memory instruction on the wide side (float4) and 4 bytes on the narrow side
// (four packed 8-bit values), consecutive lanes touch consecutive addresses,
// and several loads are issued before the first use so that enough bytes are
// in flight to cover HBM latency.
//
// Arithmetic follows the reference's generated code operation for operation
// (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:119-144):
//   t = x / scale          IEEE-754 correctly rounded quotient: the divide, or
//                          for scales of ordinary magnitude a reciprocal
//                          multiply with an exact correction step that gives
//                          the same bits (quotient<> in om_kernels.h)
//   r = roundEven(t)       v_rndne_f32 == the reference's floor-based
//                          emulation (src/Dialect/Mlir/DialectBuilder.cpp
//                          :291-332) for every input, up to the sign of zero
//   r = r + zp             separate add (no FMA contraction: -ffp-contract=off)
//   c = min(max(r,lo),hi)  maxnum then minnum: NaN -> lo
//   y = trunc_i8(fpto[us]i(c))
// Denormals are kept (the file is built with -fno-gpu-flush-denormals-to-zero).

#include "om_kernels.h"

#include <mutex>
#include <type_traits>

#include <stdlib.h>

namespace om {

namespace {

constexpr int kThreads = 256;

typedef float f4a __attribute__((ext_vector_type(4)));
typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));
typedef int32_t i4u __attribute__((ext_vector_type(4), aligned(4)));

// A store that is written through to memory when it is issued (sc1) instead
// of staying dirty in L2 until the kernel ends, when the write-back of all of
// a kernel's results would be its last microseconds; unlike a streaming store
// it leaves the data where a kernel that reads it next finds it quickly.
__device__ __forceinline__ void store_through_u32(uint32_t *p, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

// Stores of the large quantize / dequantize kernels.  8-bit results are
// written through: per-tensor quantize of 256 Mi elements 83.0 -> 84.8 % of HBM
// peak, ragged per-axis 83.4 -> 87.8 %, DynamicQuantizeLinear 84.0 -> 85.0 %
// (streaming stores: 7 - 14 % slower than plain ones).  For the f32 results of
// dequantize, streaming and written-through stores measure the same, 3.5 %
// ahead of plain ones.
template <typename V>
__device__ __forceinline__ void dq_store(V o, V *p) {
  __builtin_nontemporal_store(o, p);
}
__device__ __forceinline__ void q_store(void *p, uint32_t v) {
  store_through_u32((uint32_t *)p, v);
}

template <bool SIGNED>
__device__ __forceinline__ float load_zp_f32(const void *zp, int64_t i) {
  // int -> f32 through a 32-bit integer of the same signedness
  // (src/Dialect/Mlir/DialectBuilder.cpp:979-995).
  if (SIGNED)
    return (float)(int32_t)((const int8_t *)zp)[i];
  return (float)(uint32_t)((const uint8_t *)zp)[i];
}

// Four elements that share one scale; r = 1 / s is used when FAST (only for
// a tame s, see scale_is_tame).
template <bool SIGNED, bool HAS_ZP, int FAST, typename V4>
__device__ __forceinline__ uint32_t quant_four(
    V4 v, float s, float r, float zpf, uint32_t flip) {
  return quant_pack4<SIGNED, HAS_ZP, FAST>(
             v.x, v.y, v.z, v.w, s, s, s, s, r, r, r, r, zpf, zpf, zpf, zpf) ^
         flip;
}
// Four elements with a scale each (four adjacent columns of a per-axis op).
template <bool SIGNED, bool HAS_ZP, int FAST, typename V4>
__device__ __forceinline__ uint32_t quant_cols(V4 v, const float (&s)[4],
    const float (&r)[4], const float (&z)[4]) {
  return quant_pack4<SIGNED, HAS_ZP, FAST>(v.x, v.y, v.z, v.w, s[0], s[1], s[2],
      s[3], r[0], r[1], r[2], r[3], z[0], z[1], z[2], z[3]);
}
// Whether every lane of the wave holds tame scales: the kernels pick the
// short quotient by a branch the whole wave takes together.
__device__ __forceinline__ bool wave_all(bool p) {
  return __builtin_amdgcn_ballot_w64(!p) == 0;
}

// ---- per-tensor quantize over a flat array -------------------------------
// x must be 16-byte aligned and y 4-byte aligned.  Each block handles
// kThreads*UNROLL float4 per step; `flip` is 0, or 0x80808080 to store the
// result minus 128 as int8.
constexpr int kUnroll = 4;
constexpr int kRowUnroll = 8; // rows in flight per thread in the row-walking per-axis kernels

// Scale and zero point of a per-tensor quantize kernel: read from memory, or
// -- when the caller knows minimum and maximum of x (QuantLimits) -- derived
// from those as DynamicQuantizeLinear derives them, by every block for itself,
// and written to where the GEMM that follows reads them by the first block.
template <bool SIGNED, bool HAS_ZP>
__device__ __forceinline__ void quant_params(const float *__restrict__ scale_p,
    const void *__restrict__ zp_p, const QuantLimits &lim, bool first_block,
    float &s, float &zpf) {
  if (lim.limits) { // (the same for every thread)
    dynamic_params(lim.limits[0], lim.limits[1], s, zpf, lim.no_zp != 0);
    if (first_block && threadIdx.x == 0) {
      lim.scale_out[0] = s;
      lim.zp_out[0] = (uint8_t)(uint32_t)zpf;
    }
  } else {
    s = scale_p[0];
    zpf = HAS_ZP ? load_zp_f32<SIGNED>(zp_p, 0) : 0.0f;
  }
}

template <bool SIGNED, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_quant_flat(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n,
    const float *__restrict__ scale_p, const void *__restrict__ zp_p,
    uint32_t flip, QuantLimits lim) {
  const int64_t nvec = n >> 2;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const int64_t step = (int64_t)gridDim.x * (kThreads * kUnroll);
  const int64_t base0 = (int64_t)blockIdx.x * (kThreads * kUnroll);
  // The block's first vectors are requested before scale and zero point are
  // (no branch around them: one past the end is the last one again, and is
  // not stored): the parameters first would put a memory round trip of their
  // own in front of the data's.
  f4a v[kUnroll];
  auto request = [&](int64_t base) {
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      const int64_t idx = base + j * kThreads + threadIdx.x;
      v[j] = __builtin_nontemporal_load(&x4[idx < nvec ? idx : nvec - 1]);
    }
  };
  if (base0 < nvec) // (the same for the whole block; implies nvec > 0)
    request(base0);
  __builtin_amdgcn_sched_barrier(0);
  float s, zpf;
  quant_params<SIGNED, HAS_ZP>(scale_p, zp_p, lim, blockIdx.x == 0, s, zpf);
  const float r = 1.0f / s;
  auto body = [&](auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
    for (int64_t base = base0; base < nvec; base += step) {
      if (base != base0)
        request(base);
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        const int64_t idx = base + j * kThreads + threadIdx.x;
        if (idx < nvec)
          q_store(&y4[idx], quant_four<SIGNED, HAS_ZP, FAST>(v[j], s, r, zpf, flip));
      }
    }
  };
  if (scale_is_tame(s)) // the same for every thread
    body(std::true_type{});
  else
    body(std::false_type{});
  // Up to three trailing elements.
  if (blockIdx.x == 0) {
    int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n)
      y[e] = (uint8_t)(quant_one<SIGNED, HAS_ZP>(x[e], s, zpf) ^ (flip & 0xFFu));
  }
}

// The same op with the launch shape of the row-walking kernels below, for
// tensors of 4 Mi elements and more: the flat array is cut into runs of
// kTileRun float4, a block takes kThreads adjacent float4 of kTileRows
// consecutive runs (one trip, all loads before the first store).  Measured
// against k_quant_flat, whose blocks walk contiguous KiB: 256 Mi elements 6.6
// against 6.2 TB/s (DynamicQuantizeLinear, whose second pass this is, 6.73
// against 6.49), 64 Mi 6.2 against 5.9, 12 Mi 5.3 against 5.0, 8 Mi the same.
constexpr int kTileRun = 8192, kTileRows = 8;

template <bool SIGNED, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_quant_tiled(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n,
    const float *__restrict__ scale_p, const void *__restrict__ zp_p,
    uint32_t flip, QuantLimits lim) {
  const int64_t nvec = n >> 2; // >= 1: the kernel is for large tensors
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const int64_t first = (int64_t)blockIdx.y * kTileRows * kTileRun +
                        (int64_t)blockIdx.x * kThreads + threadIdx.x;
  // The vectors are requested before scale and zero point are, and without a
  // branch around any of them (one past the end is the last one again, and is
  // not stored): a block lives for one memory round trip, and parameters
  // loaded first -- a scalar load that the zero point's load waits for, and a
  // wait for that one -- made it two and a half (83 % of HBM peak against
  // 88 % for the per-axis kernel, which asks for its rows first).
  f4a v[kTileRows];
#pragma unroll
  for (int j = 0; j < kTileRows; ++j) {
    const int64_t idx = first + (int64_t)j * kTileRun;
    v[j] = __builtin_nontemporal_load(&x4[idx < nvec ? idx : nvec - 1]);
  }
  __builtin_amdgcn_sched_barrier(0);
  float s, zpf;
  quant_params<SIGNED, HAS_ZP>(
      scale_p, zp_p, lim, blockIdx.x == 0 && blockIdx.y == 0, s, zpf);
  const float r = 1.0f / s;
  const bool tame = scale_is_tame(s); // the same for every thread
  auto store = [&](auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
    for (int j = 0; j < kTileRows; ++j) {
      const int64_t idx = first + (int64_t)j * kTileRun;
      if (idx < nvec) {
        q_store(&y4[idx], quant_four<SIGNED, HAS_ZP, FAST>(v[j], s, r, zpf, flip));
      }
    }
  };
  if (tame)
    store(std::true_type{});
  else
    store(std::false_type{});
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n)
      y[e] = (uint8_t)(quant_one<SIGNED, HAS_ZP>(x[e], s, zpf) ^ (flip & 0xFFu));
  }
}

// ---- per-axis quantize, axis is the innermost dimension -------------------
// View [rows, C]; each thread owns four fixed columns, keeps their scale and
// zero point in registers and walks down `rows_per_block` rows.  Row starts
// need not be 16-byte aligned (C % 4 != 0): loads are dword-aligned float4,
// the 4-byte store may sit at any byte address.
// VEC: every thread's four columns lie inside the tensor (C % 4 == 0), `scale`
// is 16-byte and `zp` 4-byte aligned: scale and zero point then come as one
// load each.  Reciprocals and the conversion of the zero points wait until the
// first rows have been requested.
template <bool SIGNED, bool HAS_ZP, bool VEC>
__global__ __launch_bounds__(kThreads) void k_quant_lastaxis(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t rows,
    int64_t C, const float *__restrict__ scale, const void *__restrict__ zp,
    int rows_per_block) {
  const int64_t c0 = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  if (c0 >= C)
    return;
  const int ncol = VEC ? 4 : ((C - c0 >= 4) ? 4 : (int)(C - c0));
  float s[4], z[4], rc[4];
  uint32_t zraw[4] = {0, 0, 0, 0};
  if (VEC) {
    const f4a sv = *(const f4a *)(scale + c0);
    s[0] = sv.x;
    s[1] = sv.y;
    s[2] = sv.z;
    s[3] = sv.w;
    if (HAS_ZP) {
      const uint32_t w = *(const uint32_t *)((const uint8_t *)zp + c0);
      zraw[0] = w & 0xFFu;
      zraw[1] = (w >> 8) & 0xFFu;
      zraw[2] = (w >> 16) & 0xFFu;
      zraw[3] = w >> 24;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t c = c0 + (j < ncol ? j : 0);
      s[j] = scale[c];
      zraw[j] = HAS_ZP ? (uint32_t)((const uint8_t *)zp)[c] : 0u;
    }
  }
  auto derive = [&]() { // what follows from scale and zero point
    bool tame = true;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      rc[j] = 1.0f / s[j];
      tame = tame && scale_is_tame(s[j]);
      z[j] = HAS_ZP ? (SIGNED ? (float)(int32_t)(int8_t)zraw[j]
                              : (float)zraw[j])
                    : 0.0f;
    }
    return wave_all(tame);
  };
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end =
      (r_begin + rows_per_block < rows) ? r_begin + rows_per_block : rows;
  if (ncol == 4) {
    int64_t r = r_begin;
    f4u v[kRowUnroll];
    auto request = [&](int64_t r0) {
#pragma unroll
      for (int j = 0; j < kRowUnroll; ++j)
        v[j] = __builtin_nontemporal_load((const f4u *)(x + (r0 + j) * C + c0));
    };
    auto finish = [&](int64_t r0, auto fast_c) {
      constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
      for (int j = 0; j < kRowUnroll; ++j)
        q_store(y + (r0 + j) * C + c0,
            quant_cols<SIGNED, HAS_ZP, FAST>(v[j], s, rc, z));
    };
    auto rest = [&](auto fast_c) {
      constexpr bool FAST = decltype(fast_c)::value;
      for (; r + kRowUnroll <= r_end; r += kRowUnroll) {
        request(r);
        finish(r, fast_c);
      }
      for (; r < r_end; ++r) {
        f4u v1 = *(const f4u *)(x + r * C + c0);
        *(u32_a1 *)(y + r * C + c0) =
            quant_cols<SIGNED, HAS_ZP, FAST>(v1, s, rc, z);
      }
    };
    const bool first = r + kRowUnroll <= r_end;
    if (first)
      request(r);
    if (derive()) {
      if (first) {
        finish(r, std::true_type{});
        r += kRowUnroll;
      }
      rest(std::true_type{});
    } else {
      if (first) {
        finish(r, std::false_type{});
        r += kRowUnroll;
      }
      rest(std::false_type{});
    }
  } else {
    derive();
    for (int64_t r = r_begin; r < r_end; ++r)
      for (int j = 0; j < ncol; ++j)
        y[r * C + c0 + j] =
            (uint8_t)quant_one<SIGNED, HAS_ZP>(x[r * C + c0 + j], s[j], z[j]);
  }
}

// ---- per-axis quantize, innermost axis, rows not 16-byte aligned -----------
// When C % 4 != 0 the rows of a [rows, C] tensor start at odd alignments and
// the row-walking kernel above would issue misaligned 16-byte loads and
// misaligned 4-byte stores.  This kernel works on the flat array cut into
// aligned vectors of four elements.  Vector i covers columns (4 i + e) mod C,
// which repeats every C / gcd(C, 4) vectors (every four rows when C is odd).
// `period` is a multiple of that, so a thread that takes vectors v, v +
// period, v + 2 period, ... meets the same four columns each time: it loads
// their scales and zero points once, like the row-walking kernel, and every
// data access is aligned and coalesced.
// Scale and raw zero point of the four columns c, c+1, c+2, c+3 (mod C) that
// a thread of the periodic kernels keeps to.  Unless they wrap around the end
// of a row (one thread in C / 4 does) they are adjacent: one 16-byte load at a
// 4-byte aligned address and one 4-byte load at any address, issued before
// anything waits; the wrapping lanes redo theirs element by element in
// periodic_params_fix, which the kernels call after their first vectors have
// been requested.  Needs C >= 4 (VEC); otherwise element by element at once.
template <bool HAS_ZP, bool VEC>
__device__ __forceinline__ void periodic_params(const float *__restrict__ scale,
    const void *__restrict__ zp, uint32_t c, uint32_t C, float (&s)[4],
    uint32_t (&zraw)[4]) {
  if (VEC) {
    const uint32_t cb = (c + 4 > C) ? 0u : c;
    const f4u sv = *(const f4u *)(scale + cb);
    s[0] = sv.x;
    s[1] = sv.y;
    s[2] = sv.z;
    s[3] = sv.w;
    const uint32_t w =
        HAS_ZP ? *(const u32_a1 *)((const uint8_t *)zp + cb) : 0u;
    zraw[0] = w & 0xFFu;
    zraw[1] = (w >> 8) & 0xFFu;
    zraw[2] = (w >> 16) & 0xFFu;
    zraw[3] = w >> 24;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[e] = scale[c];
      zraw[e] = HAS_ZP ? (uint32_t)((const uint8_t *)zp)[c] : 0u;
      c = (c + 1 == C) ? 0 : c + 1;
    }
  }
}
template <bool HAS_ZP, bool VEC>
__device__ __forceinline__ void periodic_params_fix(
    const float *__restrict__ scale, const void *__restrict__ zp, uint32_t c,
    uint32_t C, float (&s)[4], uint32_t (&zraw)[4]) {
  if (VEC && c + 4 > C) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[e] = scale[c];
      zraw[e] = HAS_ZP ? (uint32_t)((const uint8_t *)zp)[c] : 0u;
      c = (c + 1 == C) ? 0 : c + 1;
    }
  }
}

template <bool SIGNED, bool HAS_ZP, bool VEC>
__global__ __launch_bounds__(kThreads) void k_quant_periodic(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n, uint32_t C,
    int64_t period, const float *__restrict__ scale,
    const void *__restrict__ zp, int periods_per_block) {
  const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t nvec = n >> 2;
  if (v >= period)
    return;
  // Scales and zero points as loaded; reciprocals and conversions wait until
  // the first vectors have been requested.
  float s[4], z[4], rc[4];
  uint32_t zraw[4];
  const uint32_t c_first = (uint32_t)(((uint64_t)v * 4) % C);
  periodic_params<HAS_ZP, VEC>(scale, zp, c_first, C, s, zraw);
  auto derive = [&]() {
    periodic_params_fix<HAS_ZP, VEC>(scale, zp, c_first, C, s, zraw);
    bool tame = true;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      rc[e] = 1.0f / s[e];
      tame = tame && scale_is_tame(s[e]);
      z[e] = HAS_ZP ? (SIGNED ? (float)(int32_t)(int8_t)zraw[e]
                              : (float)zraw[e])
                    : 0.0f;
    }
    return wave_all(tame);
  };
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  int64_t idx = (int64_t)blockIdx.y * periods_per_block * period + v;
  const int64_t end = idx + (int64_t)periods_per_block * period;
  const int64_t stop = end < nvec ? end : nvec;
  f4a q[kRowUnroll];
  auto request = [&](int64_t i0) {
#pragma unroll
    for (int j = 0; j < kRowUnroll; ++j)
      q[j] = __builtin_nontemporal_load(&x4[i0 + j * period]);
  };
  auto finish = [&](int64_t i0, auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
    for (int j = 0; j < kRowUnroll; ++j)
      q_store(&y4[i0 + j * period], quant_cols<SIGNED, HAS_ZP, FAST>(q[j], s, rc, z));
  };
  auto rest = [&](auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
    for (; idx + (kRowUnroll - 1) * period < stop;
         idx += kRowUnroll * period) {
      request(idx);
      finish(idx, fast_c);
    }
    for (; idx < stop; idx += period)
      y4[idx] = quant_cols<SIGNED, HAS_ZP, FAST>(x4[idx], s, rc, z);
  };
  const bool first = idx + (kRowUnroll - 1) * period < stop;
  if (first)
    request(idx);
  if (derive()) {
    if (first) {
      finish(idx, std::true_type{});
      idx += kRowUnroll * period;
    }
    rest(std::true_type{});
  } else {
    if (first) {
      finish(idx, std::false_type{});
      idx += kRowUnroll * period;
    }
    rest(std::false_type{});
  }
  // the up to three elements after the last whole vector
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    const int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n) {
      const uint32_t ce = (uint32_t)(e % C);
      const float zf = HAS_ZP ? load_zp_f32<SIGNED>(zp, ce) : 0.0f;
      y[e] = (uint8_t)quant_one<SIGNED, HAS_ZP>(x[e], scale[ce], zf);
    }
  }
}

// ---- general [outer, channels, inner] quantize ---------------------------
// One block row per (outer, channel) pair; the scale is uniform over a run of
// `inner` elements.  Used when the axis is not the innermost dimension, and as
// the fallback for misaligned per-tensor buffers.
// ---- per-axis, axis not innermost, inner % 4 == 0 -------------------------
// [outer, channels, inner] with the axis in the middle (per-channel scales of
// an NCHW tensor): a slab of `inner` consecutive elements shares one scale and
// the slabs lie back to back, so the tensor is walked as the flat array of
// float4 it is.  A block takes kThreads * U consecutive float4 in one
// trip; a thread finds the slab and channel of its first float4 by division
// and steps on from there (kThreads float4 further = `adv` whole slabs and
// `rem` float4), so that any further ones cost a few integer operations.
// float4 per thread: measured on 100 MB tensors, rotating over six of them,
// quantize / dequantize in TB/s: 1: 5.0 / 5.1; 2: 4.7 / 5.2; 4: 4.1 / 4.75;
// 8: 4.2 / 4.6.
constexpr int kSlabQuantPerThread = 1, kSlabDequantPerThread = 2;
struct SlabStep {
  uint32_t iv;       // float4 per slab
  uint32_t channels;
  uint32_t adv, rem; // kThreads == adv * iv + rem
};

__device__ __forceinline__ void slab_advance(
    const SlabStep &st, uint32_t &col, uint32_t &c) {
  col += st.rem;
  uint32_t add = st.adv;
  if (col >= st.iv) {
    col -= st.iv;
    ++add;
  }
  c += add;
  if (c >= st.channels)
    c %= st.channels;
}

template <bool SIGNED, bool HAS_ZP, int U>
__global__ __launch_bounds__(kThreads) void k_quant_slabs(
    const float *__restrict__ x, uint8_t *__restrict__ y, uint32_t nvec,
    SlabStep st, const float *__restrict__ scale,
    const void *__restrict__ zp) {
  const uint32_t first = blockIdx.x * (uint32_t)(kThreads * U) + threadIdx.x;
  if (first >= nvec)
    return;
  const uint32_t slab = first / st.iv;
  uint32_t col = first - slab * st.iv;
  uint32_t c = slab % st.channels;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  f4a v[U];
  float s[U], z[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const uint32_t idx = first + j * kThreads;
    if (idx < nvec) {
      v[j] = __builtin_nontemporal_load(&x4[idx]);
      s[j] = scale[c];
      z[j] = HAS_ZP ? load_zp_f32<SIGNED>(zp, c) : 0.0f;
    }
    slab_advance(st, col, c);
  }
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const uint32_t idx = first + j * kThreads;
    if (idx < nvec) {
      // a scale per float4: the reciprocal costs a divide, the four elements
      // then save three
      if (wave_all(scale_is_tame(s[j])))
        y4[idx] = quant_four<SIGNED, HAS_ZP, true>(
            v[j], s[j], 1.0f / s[j], z[j], 0u);
      else
        y4[idx] = quant_four<SIGNED, HAS_ZP, false>(v[j], s[j], 0.0f, z[j], 0u);
    }
  }
}

// Per-tensor quantize with the quotient taken as x * (1 / scale), the form
// the reference's code has under --enable-fast-math (quotient<2>): blocks of
// two float4 per thread, one trip; x 16-byte and y 4-byte aligned.
template <bool SIGNED, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_quant_flat_reciprocal(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n,
    const float *__restrict__ scale_p, const void *__restrict__ zp_p,
    uint32_t flip) {
  const int64_t nvec = n >> 2;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * 2) + threadIdx.x;
  f4a v[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    if (base + j * kThreads < nvec)
      v[j] = __builtin_nontemporal_load(&x4[base + j * kThreads]);
  const float s = scale_p[0];
  const float r = 1.0f / s;
  const float zpf = HAS_ZP ? load_zp_f32<SIGNED>(zp_p, 0) : 0.0f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
    if (base + j * kThreads < nvec)
      q_store(&y4[base + j * kThreads],
          quant_four<SIGNED, HAS_ZP, 2>(v[j], s, r, zpf, flip));
  if (blockIdx.x == 0) {
    const int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n)
      y[e] = (uint8_t)(quant_one<SIGNED, HAS_ZP, 2>(x[e], s, zpf, r) ^ (flip & 0xFFu));
  }
}

// ---- per-axis on an inner axis whose slabs are not whole float4 --------------
// [outer, channels, inner] with inner >= 4 and inner % 4 != 0 (an NCHW
// activation with 7 x 7 or 57 x 57 pixels a channel): the flat array is walked
// in aligned float4 all the same; the four elements of a vector lie in at most
// two consecutive slabs, so a thread finds the channel of its first element
// (one 32-bit division by `inner`, one remainder by `channels`), takes the
// parameters of that channel and of the next, and picks per element.  Blocks
// of two vectors per thread, one trip.  x 16-byte and y 4-byte aligned (the
// other way round for dequantize), fewer than 2^32 elements.
struct GatherPos {
  uint32_t ca, cb; // channel of the vector's first element, and the one after
  uint32_t na;     // how many of the four elements belong to ca
};
__device__ __forceinline__ GatherPos gather_pos(
    uint32_t e0, uint32_t channels, uint32_t inner) {
  const uint32_t slab = e0 / inner;
  const uint32_t left = inner - (e0 - slab * inner); // elements to the slab's end
  GatherPos p;
  p.ca = slab % channels;
  p.cb = p.ca + 1 == channels ? 0 : p.ca + 1;
  p.na = left < 4 ? left : 4;
  return p;
}

// QMODE2: the reference's fast-math form (quotient<2>); otherwise the divide,
// or its corrected-reciprocal equivalent when every scale in the wave is tame.
template <bool SIGNED, bool HAS_ZP, bool QMODE2>
__global__ __launch_bounds__(kThreads) void k_quant_gather(
    const float *__restrict__ x, uint8_t *__restrict__ y, uint32_t n,
    uint32_t channels, uint32_t inner, const float *__restrict__ scale,
    const void *__restrict__ zp) {
  const uint32_t nvec = n >> 2;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const uint32_t base = blockIdx.x * (uint32_t)(kThreads * 2) + threadIdx.x;
  f4a v[2];
  GatherPos pos[2];
  float sa[2], sb[2], za[2], zb[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t idx = base + j * kThreads;
    if (idx < nvec)
      v[j] = __builtin_nontemporal_load(&x4[idx]);
    pos[j] = gather_pos((idx < nvec ? idx : 0) << 2, channels, inner);
    sa[j] = scale[pos[j].ca];
    sb[j] = scale[pos[j].cb];
    za[j] = HAS_ZP ? load_zp_f32<SIGNED>(zp, pos[j].ca) : 0.0f;
    zb[j] = HAS_ZP ? load_zp_f32<SIGNED>(zp, pos[j].cb) : 0.0f;
  }
  auto finish = [&](auto qmode_c) {
    constexpr int QM = decltype(qmode_c)::value;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t idx = base + j * kThreads;
      if (idx >= nvec)
        continue;
      const float ra = 1.0f / sa[j], rb = 1.0f / sb[j];
      float s[4], r[4], z[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const bool first = (uint32_t)k < pos[j].na;
        s[k] = first ? sa[j] : sb[j];
        r[k] = first ? ra : rb;
        z[k] = first ? za[j] : zb[j];
      }
      q_store(&y4[idx], quant_cols<SIGNED, HAS_ZP, QM>(v[j], s, r, z));
    }
  };
  if (QMODE2) {
    finish(std::integral_constant<int, 2>{});
  } else {
    const bool tame = scale_is_tame(sa[0]) && scale_is_tame(sb[0]) &&
                      scale_is_tame(sa[1]) && scale_is_tame(sb[1]);
    if (wave_all(tame))
      finish(std::integral_constant<int, 1>{});
    else
      finish(std::integral_constant<int, 0>{});
  }
  if (blockIdx.x == 0) {
    const uint32_t e = (nvec << 2) + threadIdx.x;
    if (e < n) {
      const uint32_t c = (e / inner) % channels;
      const float s1 = scale[c];
      const float z1 = HAS_ZP ? load_zp_f32<SIGNED>(zp, c) : 0.0f;
      y[e] = (uint8_t)quant_one<SIGNED, HAS_ZP, QMODE2 ? 2 : 0>(x[e], s1, z1, 1.0f / s1);
    }
  }
}

// The same form with a scale per column of a [rows, C] tensor (per-axis on the
// last axis): a thread takes four consecutive elements of the flat array,
// finds their columns (one 32-bit remainder, then steps with wrap-around) and
// gathers scale and zero point for each; x 16-byte and y 4-byte aligned, fewer
// than 2^32 elements.
template <bool SIGNED, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_quant_lastaxis_reciprocal(
    const float *__restrict__ x, uint8_t *__restrict__ y, uint32_t n,
    uint32_t C, const float *__restrict__ scale, const void *__restrict__ zp) {
  const uint32_t nvec = n >> 2;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const uint32_t base = blockIdx.x * (uint32_t)(kThreads * 2) + threadIdx.x;
  f4a v[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    if (base + j * kThreads < nvec)
      v[j] = __builtin_nontemporal_load(&x4[base + j * kThreads]);
  auto one = [&](float xe, uint32_t c) {
    const float s = scale[c];
    const float zpf = HAS_ZP ? load_zp_f32<SIGNED>(zp, c) : 0.0f;
    return quant_one<SIGNED, HAS_ZP, 2>(xe, s, zpf, 1.0f / s);
  };
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t idx = base + j * kThreads;
    if (idx < nvec) {
      uint32_t c[4];
      c[0] = (idx << 2) % C;
#pragma unroll
      for (int k = 1; k < 4; ++k)
        c[k] = c[k - 1] + 1 == C ? 0 : c[k - 1] + 1;
      q_store(&y4[idx], one(v[j].x, c[0]) | (one(v[j].y, c[1]) << 8) |
                            (one(v[j].z, c[2]) << 16) | (one(v[j].w, c[3]) << 24));
    }
  }
  if (blockIdx.x == 0) {
    const uint32_t e = (nvec << 2) + threadIdx.x;
    if (e < n)
      y[e] = (uint8_t)one(x[e], e % C);
  }
}

template <bool SIGNED, bool HAS_ZP, bool RECIP = false>
__global__ __launch_bounds__(kThreads) void k_quant_general(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t channels,
    int64_t inner, const float *__restrict__ scale,
    const void *__restrict__ zp, int64_t oc_total, uint32_t flip = 0) {
  // flip: 0, or 0x80 to store the values minus 128 (see k_quant_flat)
  for (int64_t oc = blockIdx.y; oc < oc_total; oc += gridDim.y) {
    const int64_t c = oc % channels;
    const float s = scale[c];
    const float r = 1.0f / s;
    const float zpf = HAS_ZP ? load_zp_f32<SIGNED>(zp, c) : 0.0f;
    const float *__restrict__ xr = x + oc * inner;
    uint8_t *__restrict__ yr = y + oc * inner;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < inner;
         i += (int64_t)gridDim.x * kThreads)
      yr[i] = (uint8_t)(quant_one<SIGNED, HAS_ZP, RECIP ? 2 : 0>(xr[i], s, zpf, r) ^
                        (flip & 0xFFu));
  }
}

// ---- dequantize -----------------------------------------------------------
// y = (f32(x) - f32(zp)) * scale  (src/Conversion/ONNXToKrnl/Math/
// Elementwise.cpp:1439-1461): int->f32 conversion, subtract, multiply, each
// rounded once.
template <int KIND>
__device__ __forceinline__ float q_to_f32(uint32_t byte_or_word) {
  if (KIND == kU8)
    return (float)(byte_or_word & 0xFFu);
  if (KIND == kI8)
    return (float)(int32_t)(int8_t)(byte_or_word & 0xFFu);
  return (float)(int32_t)byte_or_word;
}

template <int KIND>
__device__ __forceinline__ float load_q_zp_f32(const void *zp, int64_t i) {
  if (KIND == kU8)
    return (float)(uint32_t)((const uint8_t *)zp)[i];
  if (KIND == kI8)
    return (float)(int32_t)((const int8_t *)zp)[i];
  return (float)((const int32_t *)zp)[i];
}

template <bool HAS_ZP>
__device__ __forceinline__ float dq_one(float xf, float s, float zpf) {
  if (HAS_ZP)
    xf = xf - zpf;
  return xf * s;
}

// 8-bit input, flat: each lane reads one dword (4 values) and writes one
// float4; x 4-byte aligned, y 16-byte aligned.  A block takes kThreads * U
// vectors and ends: no loop, the vectors requested before scale and zero point
// are (a block lives for one memory round trip; loading the parameters first
// makes that two), and U = 2.  Measured on 256 Mi elements, % of HBM peak:
// U = 2 with this order 83.7, parameters first 77.8, inside a grid-stride loop
// 73.0; U = 4 with this order 77.8, parameters first 66; U = 1 71; U = 8 70.
constexpr int kDequantFlatU = 2;
template <int KIND, bool HAS_ZP, int U>
__global__ __launch_bounds__(kThreads) void k_dequant8_flat(
    const uint8_t *__restrict__ x, float *__restrict__ y, int64_t n,
    const float *__restrict__ scale_p, const void *__restrict__ zp_p) {
  const int64_t nvec = n >> 2;
  const uint32_t *__restrict__ x4 = (const uint32_t *)x;
  f4a *__restrict__ y4 = (f4a *)y;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * U) + threadIdx.x;
  uint32_t w[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const int64_t idx = base + j * kThreads;
    w[j] = idx < nvec ? __builtin_nontemporal_load(&x4[idx]) : 0u;
  }
  const float s = scale_p[0];
  const float zpf = HAS_ZP ? load_q_zp_f32<KIND>(zp_p, 0) : 0.0f;
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const int64_t idx = base + j * kThreads;
    if (idx < nvec) {
      f4a o;
      o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j]), s, zpf);
      o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 8), s, zpf);
      o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 16), s, zpf);
      o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 24), s, zpf);
      dq_store(o, &y4[idx]);
    }
  }
  if (blockIdx.x == 0) {
    int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n)
      y[e] = dq_one<HAS_ZP>(q_to_f32<KIND>(x[e]), s, zpf);
  }
}

// Axis innermost: four fixed columns per thread.  8-bit input is read as one
// dword at any byte address, 32-bit input as a dword-aligned int4.
template <int KIND>
__device__ __forceinline__ void load_four_q(
    const void *x, int64_t elem, uint32_t (&q)[4]) {
  if (KIND == kI32) {
    i4u v = __builtin_nontemporal_load((const i4u *)((const int32_t *)x + elem));
    q[0] = (uint32_t)v.x;
    q[1] = (uint32_t)v.y;
    q[2] = (uint32_t)v.z;
    q[3] = (uint32_t)v.w;
  } else {
    uint32_t w =
        __builtin_nontemporal_load((const u32_a1 *)((const uint8_t *)x + elem));
    q[0] = w & 0xFFu;
    q[1] = (w >> 8) & 0xFFu;
    q[2] = (w >> 16) & 0xFFu;
    q[3] = w >> 24;
  }
}

template <int KIND>
__device__ __forceinline__ uint32_t load_one_q(const void *x, int64_t elem) {
  if (KIND == kI32)
    return (uint32_t)((const int32_t *)x)[elem];
  return ((const uint8_t *)x)[elem];
}

// Scale and zero point of four adjacent columns.  When the four lie inside the
// tensor and their addresses allow it they come as one 16-byte and one 4-byte
// load (8-bit zero points), not eight loads: a block of the row-walking
// kernels lives for eight rows only, and what it loads before its first row
// is a visible part of its life.  The zero points are returned as loaded;
// zp_to_f32 converts them, which the kernels do after they have requested
// their first rows (a conversion before that would make those requests wait
// for the zero points to arrive).
template <int KIND>
struct ColParams {
  float s[4];
  uint32_t zraw[4]; // 8-bit kinds: the byte in the low bits; i32: the word
};
// VEC: the launcher has checked that every thread's four columns lie inside
// the tensor (C % 4 == 0) and that `scale` is 16-byte and `zp` 4-byte aligned,
// so the vector loads need no test here -- a branch around them would make
// the code after it wait for them.
template <int KIND, bool HAS_ZP, bool VEC>
__device__ __forceinline__ void load_col_params(const float *__restrict__ scale,
    const void *__restrict__ zp, int64_t c0, int ncol, ColParams<KIND> &p) {
  if (VEC) {
    const f4a v = *(const f4a *)(scale + c0);
    p.s[0] = v.x;
    p.s[1] = v.y;
    p.s[2] = v.z;
    p.s[3] = v.w;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      p.s[j] = scale[c0 + (j < ncol ? j : 0)];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
    p.zraw[j] = 0;
  if (!HAS_ZP)
    return;
  if (KIND != kI32 && VEC) {
    const uint32_t w = *(const uint32_t *)((const uint8_t *)zp + c0);
    p.zraw[0] = w & 0xFFu;
    p.zraw[1] = (w >> 8) & 0xFFu;
    p.zraw[2] = (w >> 16) & 0xFFu;
    p.zraw[3] = w >> 24;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t c = c0 + (j < ncol ? j : 0);
      p.zraw[j] = KIND == kI32 ? (uint32_t)((const int32_t *)zp)[c]
                               : (uint32_t)((const uint8_t *)zp)[c];
    }
  }
}
template <int KIND, bool HAS_ZP>
__device__ __forceinline__ void zp_to_f32(
    const ColParams<KIND> &p, float (&z)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j)
    z[j] = HAS_ZP ? q_to_f32<KIND>(p.zraw[j]) : 0.0f;
}

template <int KIND, bool HAS_ZP, bool VEC>
__global__ __launch_bounds__(kThreads) void k_dequant_lastaxis(
    const void *__restrict__ x, float *__restrict__ y, int64_t rows, int64_t C,
    const float *__restrict__ scale, const void *__restrict__ zp,
    int rows_per_block) {
  const int64_t c0 = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  if (c0 >= C)
    return;
  const int ncol = VEC ? 4 : ((C - c0 >= 4) ? 4 : (int)(C - c0));
  ColParams<KIND> cp;
  load_col_params<KIND, HAS_ZP, VEC>(scale, zp, c0, ncol, cp);
  const float(&s)[4] = cp.s;
  float z[4];
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end =
      (r_begin + rows_per_block < rows) ? r_begin + rows_per_block : rows;
  if (ncol == 4) {
    int64_t r = r_begin;
    uint32_t q[kRowUnroll][4];
    auto request = [&](int64_t r0) {
#pragma unroll
      for (int j = 0; j < kRowUnroll; ++j)
        load_four_q<KIND>(x, (r0 + j) * C + c0, q[j]);
    };
    auto finish = [&](int64_t r0) {
#pragma unroll
      for (int j = 0; j < kRowUnroll; ++j) {
        f4u o;
        o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(q[j][0]), s[0], z[0]);
        o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(q[j][1]), s[1], z[1]);
        o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(q[j][2]), s[2], z[2]);
        o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(q[j][3]), s[3], z[3]);
        // streaming store: measured 3.5 % faster here (and 14 % slower for
        // the 4-byte stores of the quantize kernel, which keeps plain ones)
        __builtin_nontemporal_store(o, (f4u *)(y + (r0 + j) * C + c0));
      }
    };
    // the first rows are requested before the zero points are converted
    const bool first = r + kRowUnroll <= r_end;
    if (first)
      request(r);
    zp_to_f32<KIND, HAS_ZP>(cp, z);
    if (first) {
      finish(r);
      r += kRowUnroll;
    }
    for (; r + kRowUnroll <= r_end; r += kRowUnroll) {
      request(r);
      finish(r);
    }
    for (; r < r_end; ++r) {
      uint32_t q1[4];
      load_four_q<KIND>(x, r * C + c0, q1);
      f4u o;
      o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(q1[0]), s[0], z[0]);
      o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(q1[1]), s[1], z[1]);
      o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(q1[2]), s[2], z[2]);
      o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(q1[3]), s[3], z[3]);
      *(f4u *)(y + r * C + c0) = o;
    }
  } else {
    zp_to_f32<KIND, HAS_ZP>(cp, z);
    for (int64_t r = r_begin; r < r_end; ++r)
      for (int j = 0; j < ncol; ++j)
        y[r * C + c0 + j] = dq_one<HAS_ZP>(
            q_to_f32<KIND>(load_one_q<KIND>(x, r * C + c0 + j)), s[j], z[j]);
  }
}

// 8-bit input, innermost axis, C a power of two from 2 Ki to 32 Ki, x 4-byte,
// y and scale 16-byte, zp 4-byte aligned: block (bx, by) takes R = 2 rows of
// kThreads * 4 columns and ends.  The rows are requested first, scale and
// zero point after them: a block lives for one memory round trip, and
// parameters loaded (and converted) first would make that two.  % of HBM
// peak, k_dequant_lastaxis (8 rows per block) -> this: [8192, 32768] 76.4 ->
// 79.8, [16384, 16384] 76 -> 79, [32768, 8192] 76 -> 79, [131072, 2048] 75 ->
// 78, [65536, 4096] the same.  Only for these row lengths: with any other the
// column blocks of a row move from XCD to XCD between rows and blocks this
// short lose 6 - 9 points ([10922, 24576] 75.5 -> 68.5, [8192, 28672] 74 -> 66),
// and rows of 64 Ki elements gain nothing.
constexpr int kDequantRowsR = 2;
inline bool dequant_rows_ok(int64_t rows, int64_t C) {
  return C >= 2048 && C <= 32768 && (C & (C - 1)) == 0 &&
         (rows + kDequantRowsR - 1) / kDequantRowsR <= 65535;
}
template <int KIND, bool HAS_ZP, int R>
__global__ __launch_bounds__(kThreads) void k_dequant8_rows(
    const uint8_t *__restrict__ x, float *__restrict__ y, int64_t rows,
    int64_t C, const float *__restrict__ scale, const void *__restrict__ zp) {
  const int64_t c0 = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  if (c0 >= C)
    return;
  const int64_t r0 = (int64_t)blockIdx.y * R;
  uint32_t w[R];
#pragma unroll
  for (int j = 0; j < R; ++j)
    w[j] = r0 + j < rows ? __builtin_nontemporal_load(
                               (const uint32_t *)(x + (r0 + j) * C + c0))
                         : 0u;
  const f4a sv = *(const f4a *)(scale + c0);
  float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (HAS_ZP) {
    const uint32_t zw = *(const uint32_t *)((const uint8_t *)zp + c0);
    z[0] = q_to_f32<KIND>(zw);
    z[1] = q_to_f32<KIND>(zw >> 8);
    z[2] = q_to_f32<KIND>(zw >> 16);
    z[3] = q_to_f32<KIND>(zw >> 24);
  }
#pragma unroll
  for (int j = 0; j < R; ++j) {
    if (r0 + j >= rows)
      break;
    f4a o;
    o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j]), sv.x, z[0]);
    o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 8), sv.y, z[1]);
    o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 16), sv.z, z[2]);
    o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 24), sv.w, z[3]);
    dq_store(o, (f4a *)(y + (r0 + j) * C + c0));
  }
}

// 8-bit input, innermost axis, C % 4 != 0: aligned vectors of the flat array,
// each thread on a fixed set of four columns (see k_quant_periodic).
template <int KIND, bool HAS_ZP, bool VEC>
__global__ __launch_bounds__(kThreads) void k_dequant8_periodic(
    const uint8_t *__restrict__ x, float *__restrict__ y, int64_t n, uint32_t C,
    int64_t period, const float *__restrict__ scale,
    const void *__restrict__ zp, int periods_per_block) {
  const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t nvec = n >> 2;
  if (v >= period)
    return;
  // Scales and zero points as loaded; the zero points are converted after the
  // first rows have been requested (a conversion here would make those
  // requests wait for the zero points to arrive).
  float s[4], z[4];
  uint32_t zraw[4];
  const uint32_t c_first = (uint32_t)(((uint64_t)v * 4) % C);
  periodic_params<HAS_ZP, VEC>(scale, zp, c_first, C, s, zraw);
  const uint32_t *__restrict__ x4 = (const uint32_t *)x;
  f4a *__restrict__ y4 = (f4a *)y;
  int64_t idx = (int64_t)blockIdx.y * periods_per_block * period + v;
  const int64_t end = idx + (int64_t)periods_per_block * period;
  const int64_t stop = end < nvec ? end : nvec;
  uint32_t w[kRowUnroll];
  auto request = [&](int64_t i0) {
#pragma unroll
    for (int j = 0; j < kRowUnroll; ++j)
      w[j] = __builtin_nontemporal_load(&x4[i0 + j * period]);
  };
  auto finish = [&](int64_t i0) {
#pragma unroll
    for (int j = 0; j < kRowUnroll; ++j) {
      f4a o;
      o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j]), s[0], z[0]);
      o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 8), s[1], z[1]);
      o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 16), s[2], z[2]);
      o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 24), s[3], z[3]);
      __builtin_nontemporal_store(o, &y4[i0 + j * period]);
    }
  };
  const bool first = idx + (kRowUnroll - 1) * period < stop;
  if (first)
    request(idx);
  periodic_params_fix<HAS_ZP, VEC>(scale, zp, c_first, C, s, zraw);
#pragma unroll
  for (int e = 0; e < 4; ++e)
    z[e] = HAS_ZP ? q_to_f32<KIND>(zraw[e]) : 0.0f;
  if (first) {
    finish(idx);
    idx += kRowUnroll * period;
  }
  for (; idx + (kRowUnroll - 1) * period < stop; idx += kRowUnroll * period) {
    request(idx);
    finish(idx);
  }
  for (; idx < stop; idx += period) {
    const uint32_t w1 = x4[idx];
    f4a o;
    o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w1), s[0], z[0]);
    o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w1 >> 8), s[1], z[1]);
    o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w1 >> 16), s[2], z[2]);
    o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w1 >> 24), s[3], z[3]);
    y4[idx] = o;
  }
  // the up to three elements after the last whole vector
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    const int64_t e = (nvec << 2) + threadIdx.x;
    if (e < n) {
      const uint32_t ce = (uint32_t)(e % C);
      const float zf = HAS_ZP ? load_q_zp_f32<KIND>(zp, ce) : 0.0f;
      y[e] = dq_one<HAS_ZP>(q_to_f32<KIND>(x[e]), scale[ce], zf);
    }
  }
}

// ---- per-axis, innermost axis, rows off the cache lines --------------------
// (k_dequant8_rowtable, k_quant_rowtable: 8-bit on the quantized side, rows of
// about 4 Ki elements and more whose float rows do not start on a 128-byte
// line, C % 32 != 0.)
// Every access is an aligned 4-element vector of the flat array AND every
// wave's piece of a row starts on a cache line on both sides, with the rows of
// a block next to each other in memory.  A wave that writes its 1 KiB starting
// 16 or 32 bytes into a line costs 12 % of the whole kernel (k_dequant_lastaxis
// on rows that are only 16-byte aligned: 67 % of HBM peak against 76 %), and
// so do strides of megabytes between a thread's accesses, which is what
// keeping a thread's columns fixed takes when rows are not aligned
// (k_dequant8_periodic).  Row r is taken to start at the next multiple of
// kRtAlign elements at or after r * C (the elements before that go with row
// r - 1, whose columns wrap around); block (bx, by) takes elements
// [bx * kRtCols, + kRtCols) after that start in each of its kRtRows rows.
// Which columns a thread meets therefore moves from row to row, by less than
// kRtAlign: scale and zero point of the block's kRtCols + kRtAlign columns sit
// in LDS and are read from there for every vector.
constexpr int kRtRows = 8; // rows per block (4: 2 points less, 2: 8 less, 16: 6 less)
constexpr int kRtCols = kThreads * 4;
constexpr int kRtAlign = 128;
constexpr int kRtTable = kRtCols + kRtAlign;
// Shortest row: a block's columns wrap around at most once, and the table
// fill per block stays small against the rows it serves.
constexpr int64_t kRtMinC = 4 * kRtCols - kRtAlign;

// Launch shape.  Blocks are numbered so that the hardware's round-robin of
// consecutive block ids over the 8 XCDs hands each XCD whole row groups (all
// column blocks of rows 8 by .. 8 by + 7, then those of row group by + 8, ..),
// when a row group has at most kRtGroupedMax column blocks; longer rows run
// column block first.  Dequantize, % of HBM peak, column first / row groups
// per XCD, on one device: [8191, 32767] 62 / 74 (column first loses 10 points
// wherever the row pitch is within a few elements of a multiple of 32 Ki, and
// at some other pitches; DRAM write-credit stalls double there),
// [16384, 16380] 74 / 74.5, [65528, 4095] 72 / 72, [4096, 65535] 74.5 / 73.5,
// [2048, 131071] 74 / 67.  Quantize: [8191, 32767] 72 / 83.6, [16384, 16383]
// 80 / 83.8, [4096, 65535] 82.6 / 83.4, [2048, 131071] 82.5 / 78.6.
constexpr int kRtGroupedMax = 48;
struct RtGrid {
  int gx, gy;   // column blocks of a row group, row groups
  int grouped;  // 1: row groups dealt to the XCDs
};
RtGrid rt_grid(int64_t rows, int64_t C) {
  RtGrid g;
  g.gx = (int)((C + kRtAlign - 1 + kRtCols - 1) / kRtCols);
  g.gy = (int)((rows + kRtRows - 1) / kRtRows);
  g.grouped = g.gx <= kRtGroupedMax;
  return g;
}
bool rt_ok(int64_t rows, int64_t C) {
  return C >= kRtMinC && C % 32 != 0 && rows >= kRtRows &&
         C < ((int64_t)1 << 31) &&
         ((rows + kRtRows - 1) / kRtRows) *
                 ((C + kRtAlign - 1 + kRtCols - 1) / kRtCols) <
             ((int64_t)1 << 31);
}
__device__ __forceinline__ void rt_block(const RtGrid &g, int &bx, int &by) {
  const int id = blockIdx.x;
  const int full = g.grouped ? g.gy / 8 * 8 : 0; // row groups in sets of 8
  if (id < full * g.gx) {
    by = 8 * (id / (8 * g.gx)) + (id & 7);
    bx = (id % (8 * g.gx)) >> 3;
  } else {
    const int rest = id - full * g.gx;
    by = full + rest / g.gx;
    bx = rest % g.gx;
  }
}
// First element of row r in this scheme (r == rows: the end of the last row);
// nvec4 = the elements that whole vectors cover.
__device__ __forceinline__ int64_t rt_row_start(int64_t r, uint32_t C, int64_t nvec4) {
  const int64_t e = (r * (int64_t)C + (kRtAlign - 1)) & ~(int64_t)(kRtAlign - 1);
  return e < nvec4 ? e : nvec4;
}

// Scale and zero point of the four columns from c on (a column past C - 1
// stands for the one C before it).  rt_load_cols only issues loads, without a
// branch, so that a caller's loads all leave before anything waits; where the
// four columns run over the end of the row it loads the last four of the row
// instead and rt_fix_cols then fetches the right ones.
typedef float f4u4 __attribute__((ext_vector_type(4), aligned(4)));
struct RtCols {
  f4a s;
  uint32_t z; // four bytes
};
__device__ __forceinline__ uint32_t rt_wrap(uint32_t c, uint32_t C) {
  c = c >= C ? c - C : c;
  return c >= C ? c - C : c;
}
template <bool HAS_ZP>
__device__ __forceinline__ RtCols rt_load_cols(const float *__restrict__ scale,
    const void *__restrict__ zp, uint32_t c, uint32_t C) {
  c = rt_wrap(c, C);
  const uint32_t cs = c + 3 < C ? c : C - 4;
  RtCols p;
  p.s = *(const f4u4 *)(scale + cs);
  p.z = HAS_ZP ? *(const u32_a1 *)((const uint8_t *)zp + cs) : 0u;
  return p;
}
template <bool HAS_ZP>
__device__ __forceinline__ void rt_fix_cols(RtCols &p,
    const float *__restrict__ scale, const void *__restrict__ zp, uint32_t c,
    uint32_t C) {
  c = rt_wrap(c, C);
  if (c + 3 < C)
    return;
  const uint8_t *zb = (const uint8_t *)zp;
  uint32_t ce[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    ce[e] = c + e >= C ? c + e - C : c + e;
  p.s.x = scale[ce[0]];
  p.s.y = scale[ce[1]];
  p.s.z = scale[ce[2]];
  p.s.w = scale[ce[3]];
  if (HAS_ZP)
    p.z = (uint32_t)zb[ce[0]] | (uint32_t)zb[ce[1]] << 8 |
          (uint32_t)zb[ce[2]] << 16 | (uint32_t)zb[ce[3]] << 24;
}
// The zero points of the four columns from `first` on (counted from col0).
template <int KIND>
__device__ __forceinline__ void rt_zps(
    const uint32_t *sZ, int first, float (&z)[4]) {
  const uint32_t zw = __builtin_amdgcn_alignbyte(
      sZ[(first >> 2) + 1], sZ[first >> 2], (uint32_t)(first & 3));
  z[0] = q_to_f32<KIND>(zw);
  z[1] = q_to_f32<KIND>(zw >> 8);
  z[2] = q_to_f32<KIND>(zw >> 16);
  z[3] = q_to_f32<KIND>(zw >> 24);
}

template <int KIND, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_dequant8_rowtable(
    const uint8_t *__restrict__ x, float *__restrict__ y, int64_t n,
    int64_t rows, uint32_t C, const float *__restrict__ scale,
    const void *__restrict__ zp, RtGrid g) {
  __shared__ __attribute__((aligned(16))) float sS[kRtTable];
  __shared__ uint32_t sZ[kRtTable / 4 + 1];
  const int t = threadIdx.x;
  int bx, by;
  rt_block(g, bx, by);
  const uint32_t col0 = bx * (uint32_t)kRtCols;
  const int64_t nvec4 = (n >> 2) << 2;
  const int64_t r0 = (int64_t)by * kRtRows;
  const uint32_t *__restrict__ x4 = (const uint32_t *)x;
  f4a *__restrict__ y4 = (f4a *)y;
  uint32_t w[kRtRows];
  int64_t vec[kRtRows]; // the thread's vector in row r0 + j, or -1
  int first[kRtRows];   // its first column in that row, counted from col0
  auto request = [&]() {
#pragma unroll
    for (int j = 0; j < kRtRows; ++j) {
      const int64_t r = r0 + j;
      const int64_t s0 = rt_row_start(r, C, nvec4);
      const int64_t e = s0 + col0 + 4 * t;
      const bool ok = r < rows && e < rt_row_start(r + 1, C, nvec4);
      vec[j] = ok ? (e >> 2) : -1;
      first[j] = (int)(s0 - r * (int64_t)C) + 4 * t;
      w[j] = ok ? __builtin_nontemporal_load(&x4[e >> 2]) : 0u;
    }
  };
  auto finish = [&]() {
#pragma unroll
    for (int j = 0; j < kRtRows; ++j) {
      if (vec[j] < 0)
        continue;
      const f4a sv = *(const f4u4 *)&sS[first[j]];
      float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (HAS_ZP)
        rt_zps<KIND>(sZ, first[j], z);
      f4a o;
      o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j]), sv.x, z[0]);
      o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 8), sv.y, z[1]);
      o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 16), sv.z, z[2]);
      o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 24), sv.w, z[3]);
      dq_store(o, &y4[vec[j]]);
    }
  };
  // The rows are requested before the tables are: the tables' loads would
  // otherwise stand between the block's start and its first row.
  request();
  // The tables: columns col0 + 4 t .. + 3 from every thread, and the
  // kRtAlign columns after those from the first threads (plus one more word
  // of zero points, which a read of four bytes may reach into).  Every thread
  // issues both loads, so that no branch separates them from the rows'.
  const int t1 = t <= kRtAlign / 4 ? t : 0;
  RtCols p0 = rt_load_cols<HAS_ZP>(scale, zp, col0 + 4 * t, C);
  RtCols p1 = rt_load_cols<HAS_ZP>(scale, zp, col0 + kRtCols + 4 * t1, C);
  rt_fix_cols<HAS_ZP>(p0, scale, zp, col0 + 4 * t, C);
  rt_fix_cols<HAS_ZP>(p1, scale, zp, col0 + kRtCols + 4 * t1, C);
  *(f4a *)&sS[4 * t] = p0.s;
  if (HAS_ZP)
    sZ[t] = p0.z;
  if (t <= kRtAlign / 4) {
    if (t < kRtAlign / 4)
      *(f4a *)&sS[kRtCols + 4 * t] = p1.s;
    if (HAS_ZP)
      sZ[kThreads + t] = p1.z;
  }
  __syncthreads();
  finish();
  // the up to three elements after the last whole vector
  if (bx == 0 && by == 0) {
    const int64_t e = nvec4 + t;
    if (e < n) {
      const uint32_t ce = (uint32_t)(e % C);
      const float zf = HAS_ZP ? load_q_zp_f32<KIND>(zp, ce) : 0.0f;
      y[e] = dq_one<HAS_ZP>(q_to_f32<KIND>(x[e]), scale[ce], zf);
    }
  }
}

// The quantize counterpart: aligned float4 loads, one 4-byte store; the table
// also holds the reciprocals of the scales (see quotient()).  % of HBM peak,
// k_quant_periodic -> this: [8191, 32767] 77.9 -> 83.6, [8192, 32764] 80.0 ->
// 83.4, [16384, 16383] 82.1 -> 83.8, [65528, 4095] 79.5 -> 80.0, [4096, 65535]
// 69.2 -> 83.4, [2048, 131071] 68.2 -> 82.5.
template <bool SIGNED, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_quant_rowtable(
    const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n,
    int64_t rows, uint32_t C, const float *__restrict__ scale,
    const void *__restrict__ zp, RtGrid g) {
  __shared__ __attribute__((aligned(16))) float sS[kRtTable];
  __shared__ __attribute__((aligned(16))) float sR[kRtTable];
  __shared__ uint32_t sZ[kRtTable / 4 + 1];
  constexpr int KIND = SIGNED ? kI8 : kU8;
  const int t = threadIdx.x;
  int bx, by;
  rt_block(g, bx, by);
  const uint32_t col0 = bx * (uint32_t)kRtCols;
  const int64_t nvec4 = (n >> 2) << 2;
  const int64_t r0 = (int64_t)by * kRtRows;
  const f4a *__restrict__ x4 = (const f4a *)x;
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  f4a v[kRtRows];
  int64_t vec[kRtRows];
  int first[kRtRows];
#pragma unroll
  for (int j = 0; j < kRtRows; ++j) {
    const int64_t r = r0 + j;
    const int64_t s0 = rt_row_start(r, C, nvec4);
    const int64_t e = s0 + col0 + 4 * t;
    const bool ok = r < rows && e < rt_row_start(r + 1, C, nvec4);
    vec[j] = ok ? (e >> 2) : -1;
    first[j] = (int)(s0 - r * (int64_t)C) + 4 * t;
    const f4a zero = {0.0f, 0.0f, 0.0f, 0.0f};
    v[j] = ok ? __builtin_nontemporal_load(&x4[e >> 2]) : zero;
  }
  const int t1 = t <= kRtAlign / 4 ? t : 0;
  RtCols p0 = rt_load_cols<HAS_ZP>(scale, zp, col0 + 4 * t, C);
  RtCols p1 = rt_load_cols<HAS_ZP>(scale, zp, col0 + kRtCols + 4 * t1, C);
  rt_fix_cols<HAS_ZP>(p0, scale, zp, col0 + 4 * t, C);
  rt_fix_cols<HAS_ZP>(p1, scale, zp, col0 + kRtCols + 4 * t1, C);
  bool mine = scale_is_tame(p0.s.x) && scale_is_tame(p0.s.y) &&
              scale_is_tame(p0.s.z) && scale_is_tame(p0.s.w);
  {
    f4a r;
    r.x = 1.0f / p0.s.x;
    r.y = 1.0f / p0.s.y;
    r.z = 1.0f / p0.s.z;
    r.w = 1.0f / p0.s.w;
    *(f4a *)&sS[4 * t] = p0.s;
    *(f4a *)&sR[4 * t] = r;
  }
  if (HAS_ZP)
    sZ[t] = p0.z;
  if (t <= kRtAlign / 4) {
    if (t < kRtAlign / 4) {
      mine = mine && scale_is_tame(p1.s.x) && scale_is_tame(p1.s.y) &&
             scale_is_tame(p1.s.z) && scale_is_tame(p1.s.w);
      f4a r;
      r.x = 1.0f / p1.s.x;
      r.y = 1.0f / p1.s.y;
      r.z = 1.0f / p1.s.z;
      r.w = 1.0f / p1.s.w;
      *(f4a *)&sS[kRtCols + 4 * t] = p1.s;
      *(f4a *)&sR[kRtCols + 4 * t] = r;
    }
    if (HAS_ZP)
      sZ[kThreads + t] = p1.z;
  }
  const bool tame = __syncthreads_and(mine) != 0; // the same for the whole block
  auto finish = [&](auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
    for (int j = 0; j < kRtRows; ++j) {
      if (vec[j] < 0)
        continue;
      const f4a sv = *(const f4u4 *)&sS[first[j]];
      const f4a rv = *(const f4u4 *)&sR[first[j]];
      const float s[4] = {sv.x, sv.y, sv.z, sv.w};
      const float rc[4] = {rv.x, rv.y, rv.z, rv.w};
      float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (HAS_ZP)
        rt_zps<KIND>(sZ, first[j], z);
      q_store(&y4[vec[j]], quant_cols<SIGNED, HAS_ZP, FAST>(v[j], s, rc, z));
    }
  };
  if (tame)
    finish(std::true_type{});
  else
    finish(std::false_type{});
  if (bx == 0 && by == 0) {
    const int64_t e = nvec4 + t;
    if (e < n) {
      const uint32_t ce = (uint32_t)(e % C);
      const float zf = HAS_ZP ? load_zp_f32<SIGNED>(zp, ce) : 0.0f;
      y[e] = (uint8_t)quant_one<SIGNED, HAS_ZP>(x[e], scale[ce], zf);
    }
  }
}

// Any element kind, [outer, channels, inner]: one element per lane.
// The dequantize counterpart of k_quant_slabs (8-bit input).
template <int KIND, bool HAS_ZP, int U>
__global__ __launch_bounds__(kThreads) void k_dequant8_slabs(
    const uint8_t *__restrict__ x, float *__restrict__ y, uint32_t nvec,
    SlabStep st, const float *__restrict__ scale,
    const void *__restrict__ zp) {
  const uint32_t first = blockIdx.x * (uint32_t)(kThreads * U) + threadIdx.x;
  if (first >= nvec)
    return;
  const uint32_t slab = first / st.iv;
  uint32_t col = first - slab * st.iv;
  uint32_t c = slab % st.channels;
  const uint32_t *__restrict__ x4 = (const uint32_t *)x;
  f4a *__restrict__ y4 = (f4a *)y;
  uint32_t w[U];
  float s[U], z[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const uint32_t idx = first + j * kThreads;
    if (idx < nvec) {
      w[j] = __builtin_nontemporal_load(&x4[idx]);
      s[j] = scale[c];
      z[j] = HAS_ZP ? load_q_zp_f32<KIND>(zp, c) : 0.0f;
    }
    slab_advance(st, col, c);
  }
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const uint32_t idx = first + j * kThreads;
    if (idx < nvec) {
      f4a o;
      o.x = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j]), s[j], z[j]);
      o.y = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 8), s[j], z[j]);
      o.z = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 16), s[j], z[j]);
      o.w = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> 24), s[j], z[j]);
      __builtin_nontemporal_store(o, &y4[idx]);
    }
  }
}

// The dequantize side of k_quant_gather: one dword of four 8-bit values in,
// one float4 out, parameters of two consecutive channels picked per element.
template <int KIND, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_dequant8_gather(
    const uint8_t *__restrict__ x, float *__restrict__ y, uint32_t n,
    uint32_t channels, uint32_t inner, const float *__restrict__ scale,
    const void *__restrict__ zp) {
  const uint32_t nvec = n >> 2;
  const uint32_t *__restrict__ x4 = (const uint32_t *)x;
  f4a *__restrict__ y4 = (f4a *)y;
  const uint32_t base = blockIdx.x * (uint32_t)(kThreads * 2) + threadIdx.x;
  uint32_t w[2];
  GatherPos pos[2];
  float sa[2], sb[2], za[2], zb[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t idx = base + j * kThreads;
    w[j] = idx < nvec ? __builtin_nontemporal_load(&x4[idx]) : 0u;
    pos[j] = gather_pos((idx < nvec ? idx : 0) << 2, channels, inner);
    sa[j] = scale[pos[j].ca];
    sb[j] = scale[pos[j].cb];
    za[j] = HAS_ZP ? load_q_zp_f32<KIND>(zp, pos[j].ca) : 0.0f;
    zb[j] = HAS_ZP ? load_q_zp_f32<KIND>(zp, pos[j].cb) : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t idx = base + j * kThreads;
    if (idx >= nvec)
      continue;
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool first = (uint32_t)k < pos[j].na;
      o[k] = dq_one<HAS_ZP>(q_to_f32<KIND>(w[j] >> (8 * k)),
          first ? sa[j] : sb[j], first ? za[j] : zb[j]);
    }
    dq_store((f4a){o[0], o[1], o[2], o[3]}, &y4[idx]);
  }
  if (blockIdx.x == 0) {
    const uint32_t e = (nvec << 2) + threadIdx.x;
    if (e < n) {
      const uint32_t c = (e / inner) % channels;
      y[e] = dq_one<HAS_ZP>(q_to_f32<KIND>(x[e]), scale[c],
          HAS_ZP ? load_q_zp_f32<KIND>(zp, c) : 0.0f);
    }
  }
}

template <int KIND, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void k_dequant_general(
    const void *__restrict__ x, float *__restrict__ y, int64_t channels,
    int64_t inner, const float *__restrict__ scale,
    const void *__restrict__ zp, int64_t oc_total) {
  for (int64_t oc = blockIdx.y; oc < oc_total; oc += gridDim.y) {
    const int64_t c = oc % channels;
    const float s = scale[c];
    const float zpf = HAS_ZP ? load_q_zp_f32<KIND>(zp, c) : 0.0f;
    float *__restrict__ yr = y + oc * inner;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < inner;
         i += (int64_t)gridDim.x * kThreads) {
      uint32_t raw;
      if (KIND == kI32)
        raw = (uint32_t)((const int32_t *)x)[oc * inner + i];
      else
        raw = ((const uint8_t *)x)[oc * inner + i];
      yr[i] = dq_one<HAS_ZP>(q_to_f32<KIND>(raw), s, zpf);
    }
  }
}

// ---- DynamicQuantizeLinear: min / max reduction ---------------------------
__device__ __forceinline__ void block_minmax(float &lo, float &hi) {
  __shared__ float s_lo[kThreads / 64], s_hi[kThreads / 64];
  lo = wave_min(lo);
  hi = wave_max(hi);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    s_lo[wave] = lo;
    s_hi[wave] = hi;
  }
  __syncthreads();
  lo = s_lo[0];
  hi = s_hi[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) {
    lo = __builtin_fminf(lo, s_lo[w]);
    hi = __builtin_fmaxf(hi, s_hi[w]);
  }
  __syncthreads();
}

__global__ __launch_bounds__(kThreads) void k_minmax_params(
    const float *__restrict__ x, int64_t n, float *partial_min,
    float *partial_max, unsigned *counter, float *__restrict__ scale_out,
    uint8_t *__restrict__ zp_out, int no_zp,
    float *__restrict__ limits_out = nullptr) {
  // limits_out: minimum and maximum themselves go there (NaN ignored, 0 not
  // yet included) in place of the parameters derived from them.
  float lo = __builtin_inff(), hi = -__builtin_inff();
  const int64_t nvec = n >> 2;
  const f4a *__restrict__ x4 = (const f4a *)x;
  const bool aligned = (((uintptr_t)x) & 15) == 0;
  if (aligned) {
    // Read-only pass: eight 16-byte loads in flight per lane, streamed past
    // the caches (the data is not touched again before the quantize pass has
    // walked the whole tensor).
    constexpr int kMU = 8;
    const int64_t step = (int64_t)gridDim.x * (kThreads * kMU);
    for (int64_t base = (int64_t)blockIdx.x * (kThreads * kMU);
         base < nvec; base += step) {
      f4a v[kMU];
#pragma unroll
      for (int j = 0; j < kMU; ++j) {
        const int64_t idx = base + j * kThreads + threadIdx.x;
        if (idx < nvec)
          v[j] = __builtin_nontemporal_load(&x4[idx]);
        else
          v[j] = (f4a){__builtin_nanf(""), __builtin_nanf(""),
              __builtin_nanf(""), __builtin_nanf("")};
      }
#pragma unroll
      for (int j = 0; j < kMU; ++j) {
        // The NaN filler above is neutral: minnum / maxnum ignore NaN.
        lo = __builtin_fminf(lo, __builtin_fminf(__builtin_fminf(v[j].x, v[j].y),
                                     __builtin_fminf(v[j].z, v[j].w)));
        hi = __builtin_fmaxf(hi, __builtin_fmaxf(__builtin_fmaxf(v[j].x, v[j].y),
                                     __builtin_fmaxf(v[j].z, v[j].w)));
      }
    }
    if (blockIdx.x == 0) {
      const int64_t e = (nvec << 2) + threadIdx.x;
      if (e < n) {
        lo = __builtin_fminf(lo, x[e]);
        hi = __builtin_fmaxf(hi, x[e]);
      }
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * kThreads) {
      lo = __builtin_fminf(lo, x[i]);
      hi = __builtin_fmaxf(hi, x[i]);
    }
  }
  block_minmax(lo, hi);

  __shared__ bool s_last;
  if (threadIdx.x == 0) {
    __hip_atomic_store(&partial_min[blockIdx.x], lo, __ATOMIC_RELAXED,
        __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&partial_max[blockIdx.x], hi, __ATOMIC_RELAXED,
        __HIP_MEMORY_SCOPE_AGENT);
    // The partials are device-scope atomic stores, performed where every
    // XCD sees them, and the last block reads them with device-scope atomic
    // loads: nothing has to be written back or invalidated in any cache.  The
    // ticket only has to be drawn after this block's two stores have
    // completed.  A workgroup-scope release does not wait for that (the
    // stores and the ticket may travel to different memory channels), so the
    // wait is explicit: vmcnt(0) returns once both stores are acknowledged.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    const unsigned ticket = __hip_atomic_fetch_add(
        counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    s_last = (ticket == gridDim.x - 1);
  }
  __syncthreads();
  if (!s_last)
    return;
  // Last block to arrive: every other block drew its ticket after its
  // partials had landed.  Fold them and derive the parameters.
  lo = __builtin_inff();
  hi = -__builtin_inff();
  for (unsigned i = threadIdx.x; i < gridDim.x; i += kThreads) {
    lo = __builtin_fminf(lo, __hip_atomic_load(&partial_min[i],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    hi = __builtin_fmaxf(hi, __hip_atomic_load(&partial_max[i],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  }
  block_minmax(lo, hi);
  if (threadIdx.x == 0) {
    if (limits_out) {
      limits_out[0] = lo;
      limits_out[1] = hi;
    } else {
      float scale, zpf;
      dynamic_params(lo, hi, scale, zpf, no_zp != 0);
      scale_out[0] = scale;
      zp_out[0] = (uint8_t)(uint32_t)zpf;
    }
    __hip_atomic_store(
        counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Small tensors (the activations of a decode step): one block does the whole
// op -- every thread keeps its elements in registers across the min / max
// reduction, so x is read once and there is a single launch.
constexpr int kSmallThreads = 1024;
constexpr int kSmallPerThread = 16; // float4 x 4
// One block does not scale further: with 16 float4 per thread (64 Ki
// elements) it takes 11.3 us against 7.1 us for the two launches of the
// general path, at 48 Ki 9.0 against 7.0; only around 24 Ki it is ahead (5.8
// against 6.8).
constexpr int64_t kSmallMax = (int64_t)kSmallThreads * kSmallPerThread;

__global__ __launch_bounds__(kSmallThreads) void k_dql_small(
    const float *__restrict__ x, int64_t n, uint8_t *__restrict__ y,
    float *__restrict__ scale_out, uint8_t *__restrict__ zp_out,
    uint32_t flip, int mode) {
  __shared__ float s_lo[kSmallThreads / 64], s_hi[kSmallThreads / 64];
  float v[kSmallPerThread];
  float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < kSmallPerThread; ++j) {
    const int64_t e = (int64_t)j * kSmallThreads + threadIdx.x;
    v[j] = e < n ? x[e] : __builtin_nanf(""); // NaN is neutral for minnum/maxnum
    lo = __builtin_fminf(lo, v[j]);
    hi = __builtin_fmaxf(hi, v[j]);
  }
  lo = wave_min(lo);
  hi = wave_max(hi);
  if ((threadIdx.x & 63) == 0) {
    s_lo[threadIdx.x >> 6] = lo;
    s_hi[threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  lo = s_lo[0];
  hi = s_hi[0];
#pragma unroll
  for (int w = 1; w < kSmallThreads / 64; ++w) {
    lo = __builtin_fminf(lo, s_lo[w]);
    hi = __builtin_fmaxf(hi, s_hi[w]);
  }
  float scale, zpf;
  dynamic_params(lo, hi, scale, zpf, (mode & kQuantNoZeroPoint) != 0);
  if (threadIdx.x == 0) {
    scale_out[0] = scale;
    zp_out[0] = (uint8_t)(uint32_t)zpf;
  }
  const float recip = 1.0f / scale;
  auto store = [&](auto qmode_c) {
    constexpr int QMODE = decltype(qmode_c)::value;
#pragma unroll
    for (int j = 0; j < kSmallPerThread; ++j) {
      const int64_t e = (int64_t)j * kSmallThreads + threadIdx.x;
      if (e < n)
        y[e] = (uint8_t)(quant_one<false, true, QMODE>(v[j], scale, zpf, recip) ^
                         (flip & 0xFFu));
    }
  };
  // (the same branch for every thread)
  if (mode & kQuantReciprocal)
    store(std::integral_constant<int, 2>{});
  else if (scale_is_tame(scale))
    store(std::integral_constant<int, 1>{});
  else
    store(std::integral_constant<int, 0>{});
}

// Mid-sized tensors (up to 32 float4 per thread of a grid that fills the
// device once, 16 Mi elements): the whole op in one launch.  Every thread keeps
// its elements in registers while the blocks exchange their minima and maxima,
// so x is read once, nothing but the result is written, and there is one
// launch instead of two.  The grid is one block per CU, and the launcher keeps
// at most one such kernel in flight, so its blocks become resident together
// as soon as older work has drained (a cooperative launch would guarantee
// that, but costs about 30 us per launch on this platform).  The wait for the
// other blocks is bounded all the same: a block that gives up raises `failed`
// and writes nothing.
//
// Where the time goes, [4096, 768] / [4096, 3072] on MI355X, microseconds
// since the first block started (median block): own minimum and maximum known
// 1.4 / 5.4 (the loads: latency, then 6 TB/s), everybody's known 3.8 / 8.1,
// last wave done 4.6 / 10.4, next launch can start 6.1 / 15.5.  Blocks of
// eight waves rather than sixteen start and reduce faster.  Quantizing is
// bound by the vector units, not by memory (at sixteen instructions per
// element the last wave finished 4 us after the first: the four-instruction
// quotient of om_kernels.h is what shortened it).  Plain loads: streaming
// loads make a loop of nothing but this kernel on one tensor 1.5 us faster at
// [4096, 3072], but the same kernel 5 us slower when a GEMM runs between its
// launches (20.9 against 15.3 us in a kernel trace of the fused layer).
// Stores written through (store_through_u32): with plain stores the kernel
// ends with the write-back of its 12 MB result (15.4 against 13.9 us), and
// streaming stores slow down the GEMM that reads the result next by 3 us.
constexpr int kGridThreads = 512;
constexpr int kGridMaxPerThread = 32; // float4

template <int NV>
__global__ __launch_bounds__(kGridThreads) void k_dql_grid(
    const float *__restrict__ x, int64_t n, uint8_t *__restrict__ y,
    float *__restrict__ scale_out, uint8_t *__restrict__ zp_out, uint32_t flip,
    unsigned long long *slots, unsigned epoch, unsigned *failed,
    unsigned spin_limit) {
  constexpr int kWaves = kGridThreads / 64;
  __shared__ float s_lo[kWaves], s_hi[kWaves];
  __shared__ int s_ok;
  const int64_t nvec = n >> 2;
  const int64_t total = (int64_t)gridDim.x * kGridThreads;
  const int64_t gtid = (int64_t)blockIdx.x * kGridThreads + threadIdx.x;
  const f4a *__restrict__ x4 = (const f4a *)x;
  const f4a nan4 = {__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""),
      __builtin_nanf("")};

  f4a v[NV];
  float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int64_t idx = (int64_t)j * total + gtid;
    // NaN is neutral for minnum / maxnum
    v[j] = idx < nvec ? x4[idx] : nan4;
  }
  // the up to three elements after the last whole float4
  const int64_t te = (nvec << 2) + gtid;
  const float tail = (gtid < 3 && te < n) ? x[te] : __builtin_nanf("");
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    lo = __builtin_fminf(lo, __builtin_fminf(__builtin_fminf(v[j].x, v[j].y),
                                 __builtin_fminf(v[j].z, v[j].w)));
    hi = __builtin_fmaxf(hi, __builtin_fmaxf(__builtin_fmaxf(v[j].x, v[j].y),
                                 __builtin_fmaxf(v[j].z, v[j].w)));
  }
  lo = __builtin_fminf(lo, tail);
  hi = __builtin_fmaxf(hi, tail);

  // The block's own result, and the flag of the exchange.
  lo = wave_min(lo);
  hi = wave_max(hi);
  if ((threadIdx.x & 63) == 0) {
    s_lo[threadIdx.x >> 6] = lo;
    s_hi[threadIdx.x >> 6] = hi;
  }
  if (threadIdx.x == 0)
    s_ok = 1;
  __syncthreads();

  // Grid-wide exchange in two memory round trips.  Block b publishes
  // (tag, min) and (tag, max), tag being this launch's number, as two 64-bit
  // device-scope atomic stores into its own 16-byte slot: value and "it is
  // there" travel in one word, so no fence and no arrival counter are needed,
  // and nothing has to be reset between launches.  Every block then reads all
  // slots, one slot per thread so that all of a block's reads are in flight
  // together (a thread that polled four slots one after the other made the
  // exchange 1.3 us longer), each thread polling until both words carry the
  // tag.  The 16-byte read is one request to the slot's cache line, past the
  // caches that other XCDs do not see (sc1); each of its 8-byte halves was
  // written by one atomic store and is checked on its own.  All blocks fold
  // the same values, in an order that does not matter for min / max, so all
  // agree.  The wait is bounded: a thread that gives up makes its block raise
  // `failed` and write nothing.
  if (threadIdx.x == 0) {
    float bl = s_lo[0], bh = s_hi[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      bl = __builtin_fminf(bl, s_lo[w]);
      bh = __builtin_fmaxf(bh, s_hi[w]);
    }
    const unsigned long long tag = (unsigned long long)epoch << 32;
    __hip_atomic_store(&slots[2 * blockIdx.x], tag | __float_as_uint(bl),
        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&slots[2 * blockIdx.x + 1], tag | __float_as_uint(bh),
        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads(); // s_lo / s_hi are reused below
  typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
  bool ok = true;
  lo = __builtin_inff();
  hi = -__builtin_inff();
  for (unsigned i = threadIdx.x; i < gridDim.x; i += kGridThreads) {
    u64x2 w = {0, 0};
    bool got = false;
    for (unsigned spin = 0; spin < spin_limit; ++spin) {
      asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                   : "=v"(w)
                   : "v"(&slots[2 * i])
                   : "memory");
      if ((unsigned)(w.x >> 32) == epoch && (unsigned)(w.y >> 32) == epoch) {
        got = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    ok = ok && got;
    lo = __builtin_fminf(lo, __uint_as_float((unsigned)w.x));
    hi = __builtin_fmaxf(hi, __uint_as_float((unsigned)w.y));
  }
  // only the waves that had a slot to poll take part in the fold
  const unsigned pollers = gridDim.x < (unsigned)kGridThreads
                               ? (gridDim.x + 63) / 64
                               : (unsigned)kWaves;
  if ((threadIdx.x >> 6) < pollers) {
    lo = wave_min(lo);
    hi = wave_max(hi);
    if (!wave_all(ok) && (threadIdx.x & 63) == 0)
      s_ok = 0;
    if ((threadIdx.x & 63) == 0) {
      s_lo[threadIdx.x >> 6] = lo;
      s_hi[threadIdx.x >> 6] = hi;
    }
  }
  __syncthreads();
  if (!s_ok) {
    if (threadIdx.x == 0)
      __hip_atomic_store(
          failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  lo = s_lo[0];
  hi = s_hi[0];
  for (unsigned w = 1; w < pollers; ++w) {
    lo = __builtin_fminf(lo, s_lo[w]);
    hi = __builtin_fmaxf(hi, s_hi[w]);
  }

  float scale, zpf;
  dynamic_params(lo, hi, scale, zpf);
  if (gtid == 0) {
    scale_out[0] = scale;
    zp_out[0] = (uint8_t)(uint32_t)zpf;
  }
  uint32_t *__restrict__ y4 = (uint32_t *)y;
  const float recip = 1.0f / scale;
  auto store = [&](auto fast_c) {
    constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t idx = (int64_t)j * total + gtid;
      if (idx < nvec) {
        const uint32_t q = quant_four<false, true, FAST>(v[j], scale, recip, zpf, flip);
        // written through (see store_through_u32): 15.4 -> 13.9 us at
        // [4096, 3072], and the GEMM that reads the result next gains too
        store_through_u32(y4 + idx, q);
      }
    }
  };
  if (scale_is_tame(scale)) // the same for every thread
    store(std::true_type{});
  else
    store(std::false_type{});
  if (gtid < 3 && te < n)
    y[te] = (uint8_t)(quant_one<false, true>(tail, scale, zpf) ^ (flip & 0xFFu));
}

__global__ __launch_bounds__(kThreads) void k_fill_u32(
    uint32_t *__restrict__ p, int64_t n, uint32_t v) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads)
    p[i] = v;
}

// Blocks of a grid-stride kernel: never more than the work needs, at most
// `cap`.  The cap that streams fastest differs per kernel (measured on a 1 GiB
// tensor, blocks of 256 threads x 4 vectors): per-tensor quantize 4096 blocks
// 5.52 TB/s, 16384 5.68, 65536 5.64; per-tensor dequantize 4096 blocks 5.47,
// 16384 5.81, 65536 6.09, 262144 6.10.
constexpr int64_t kGridCapDefault = 256 * 16;
constexpr int64_t kGridCapQuantFlat = 16384;
inline int stream_grid(
    int64_t work_items, int64_t per_block, int64_t cap = kGridCapDefault) {
  int64_t need = (work_items + per_block - 1) / per_block;
  if (need < 1)
    need = 1;
  return (int)(need < cap ? need : cap);
}

// Rows (or periods) a block of the row-walking kernels takes: `trips` trips
// of the unrolled loop.  Many short blocks keep more of the tensor's pages in
// flight than few long ones.  Measured on [8192, 32768] (quantize /
// dequantize, TB/s): 8 rows per block 6.49 / 5.97, 16 rows 6.23 / 5.94, 32
// rows 6.02 / 5.59, 64 rows 5.62 (dequantize with 4 rows in flight and 4 rows
// per block: 5.41, with 16 in flight: 5.94); on [8191, 32767], where a block
// walks periods of the flat array: 8 periods 5.72 / 5.11, 16 periods 5.77 /
// 5.37.
void rows_per_block(
    int64_t rows, int trips, int64_t &rpb, int64_t &row_blocks) {
  rpb = trips * kRowUnroll;
  row_blocks = (rows + rpb - 1) / rpb;
  if (row_blocks > 65535) {
    rpb = (rows + 65534) / 65535;
    row_blocks = (rows + rpb - 1) / rpb;
  }
  if (row_blocks < 1)
    row_blocks = 1;
}

// Whether the slab kernels take [outer, channels, inner]: whole float4 per
// slab, 32-bit indices, and slabs long enough for the thread's step from one
// float4 to the next to stay a handful of operations.
bool slabs_ok(int64_t n, int64_t channels, int64_t inner) {
  return channels > 1 && inner % 4 == 0 && inner >= 64 &&
         n < ((int64_t)1 << 32) && channels < ((int64_t)1 << 31);
}
SlabStep slab_step(int64_t channels, int64_t inner) {
  SlabStep st;
  st.iv = (uint32_t)(inner >> 2);
  st.channels = (uint32_t)channels;
  st.adv = (uint32_t)kThreads / st.iv;
  st.rem = (uint32_t)kThreads % st.iv;
  return st;
}

// Launch shape of the periodic kernels: `period` is the column period of the
// 4-element vectors (C / gcd(C, 4)), repeated until it is a multiple of 4 and
// spans at least four blocks' worth of threads; grid.x covers one period,
// grid.y splits the periods, `trips` * kRowUnroll to a block.  Measured on
// [8191, 32767] (quantize / dequantize, TB/s) by the multiple the period is
// padded to and the trips: 8 and 2: 5.76 / 5.36; 4 and 2: 5.93 / 5.49; 4 and
// 1: 6.02 / 5.20; 2 and 1: 6.03 / 5.26; 1 and 1: 6.01 / 5.14; 1 and 2: 5.89 /
// 4.90.  A multiple of 4 float4 keeps a thread's accesses at the same
// position within a 64-byte segment from one period to the next; quantize
// then does best with one trip per block, dequantize with two.
struct PeriodicGrid {
  dim3 grid;
  int64_t period;
  int per_block;
};
PeriodicGrid periodic_grid(int64_t nvec, int64_t C, int trips) {
  const int64_t g = (C % 4 == 0) ? 4 : (C % 2 == 0) ? 2 : 1; // gcd(C, 4)
  int64_t period = C / g; // float4 until the columns repeat
  while (period % 4 != 0)
    period *= 2;
  const int64_t want = 4 * kThreads;
  if (period < want)
    period *= (want + period - 1) / period;
  const int64_t gx = (period + kThreads - 1) / kThreads;
  const int64_t periods = (nvec + period - 1) / period;
  int64_t per_block, gy;
  rows_per_block(periods, trips, per_block, gy);
  PeriodicGrid pg;
  pg.grid = dim3((unsigned)gx, (unsigned)gy);
  pg.period = period;
  pg.per_block = (int)per_block;
  return pg;
}

// Row lengths the periodic kernels are for: rows that are not whole float4
// (a thread's columns differ from row to row), and short rows of whole float4
// (fewer than 256 columns), which would leave most of a block of the
// row-walking kernels without a column to work on ([1 Mi, 4]: 0.31 TB/s there).
bool periodic_pays(int64_t C) { return C % 4 != 0 || C < 256; }

// Shapes the gathering kernels take: per-axis on an inner axis, slabs of at
// least four elements (a vector then spans two channels at most), everything
// indexable in 32 bits.
bool gather_ok(int64_t n, int64_t channels, int64_t inner) {
  return channels > 1 && inner >= 4 && n < ((int64_t)1 << 32);
}
unsigned gather_grid(int64_t n) {
  const int64_t blocks = ((n >> 2) + kThreads * 2 - 1) / (kThreads * 2);
  return (unsigned)(blocks > 0 ? blocks : 1);
}

// Scale and zero point from known limits, as a launch of its own (in front of
// the quantize kernels that read them from memory).
__global__ void k_params_from_limits(QuantLimits lim) {
  float s, zpf;
  dynamic_params(lim.limits[0], lim.limits[1], s, zpf, lim.no_zp != 0);
  lim.scale_out[0] = s;
  lim.zp_out[0] = (uint8_t)(uint32_t)zpf;
}

template <bool SIGNED>
hipError_t quantize_dispatch(hipStream_t st, const float *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    void *y, uint32_t flip, bool reciprocal = false,
    const QuantLimits *limits = nullptr) {
  const int64_t n = outer * channels * inner;
  if (n == 0)
    return hipSuccess;
  uint8_t *yo = (uint8_t *)y;
  const bool has_zp = zp != nullptr;
  // Limits of x in place of scale and zero point (per tensor, u8): the two
  // streaming kernels derive the parameters themselves; in front of any other
  // kernel a launch of one thread does.
  QuantLimits lim = {};
  if (limits) {
    const bool aligned =
        ((((uintptr_t)x) & 15) == 0) && ((((uintptr_t)y) & 3) == 0);
    if (channels == 1 && !reciprocal && aligned && !SIGNED && has_zp) {
      lim = *limits;
    } else {
      k_params_from_limits<<<1, 1, 0, st>>>(*limits);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess)
        return e;
    }
  }
  if (reciprocal) {
    // The reference's fast-math form, x * (1 / scale): a kernel of its own
    // for the per-tensor case, the general kernel for everything else.
    const bool aligned =
        ((((uintptr_t)x) & 15) == 0) && ((((uintptr_t)y) & 3) == 0);
    const int64_t blocks = ((n >> 2) + kThreads * 2 - 1) / (kThreads * 2);
    if (channels == 1 && aligned && blocks < ((int64_t)1 << 31)) {
      const unsigned grid = (unsigned)(blocks > 0 ? blocks : 1);
      if (has_zp)
        k_quant_flat_reciprocal<SIGNED, true>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip);
      else
        k_quant_flat_reciprocal<SIGNED, false>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip);
      return hipGetLastError();
    }
    // (values stored minus 128 exist per tensor only: the rows of the fused
    // layer; misaligned, they take the general kernel below)
    if (flip != 0 && channels != 1)
      return hipErrorInvalidValue;
    if (channels > 1 && inner == 1 && aligned && n < ((int64_t)1 << 32)) {
      const unsigned grid = (unsigned)(blocks > 0 ? blocks : 1);
      if (has_zp)
        k_quant_lastaxis_reciprocal<SIGNED, true><<<grid, kThreads, 0, st>>>(
            x, yo, (uint32_t)n, (uint32_t)channels, scale, zp);
      else
        k_quant_lastaxis_reciprocal<SIGNED, false><<<grid, kThreads, 0, st>>>(
            x, yo, (uint32_t)n, (uint32_t)channels, scale, zp);
      return hipGetLastError();
    }
    if (aligned && gather_ok(n, channels, inner)) {
      const unsigned grid = gather_grid(n);
      if (has_zp)
        k_quant_gather<SIGNED, true, true><<<grid, kThreads, 0, st>>>(x, yo,
            (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
      else
        k_quant_gather<SIGNED, false, true><<<grid, kThreads, 0, st>>>(x, yo,
            (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
      return hipGetLastError();
    }
    if (channels == 1) {
      outer = 1;
      inner = n;
    }
    const int64_t oc = outer * channels;
    const int64_t gy = oc < 4096 ? oc : 4096;
    int64_t gx = (inner + kThreads - 1) / kThreads;
    const int64_t cap = (4096 + gy - 1) / gy;
    gx = gx > cap ? cap : (gx < 1 ? 1 : gx);
    dim3 grid((unsigned)gx, (unsigned)gy);
    if (has_zp)
      k_quant_general<SIGNED, true, true>
          <<<grid, kThreads, 0, st>>>(x, yo, channels, inner, scale, zp, oc, flip);
    else
      k_quant_general<SIGNED, false, true>
          <<<grid, kThreads, 0, st>>>(x, yo, channels, inner, scale, zp, oc, flip);
    return hipGetLastError();
  }
  if (channels == 1) {
    const bool aligned =
        ((((uintptr_t)x) & 15) == 0) && ((((uintptr_t)y) & 3) == 0);
    const int64_t tile_rows =
        ((n >> 2) + kTileRun - 1) / kTileRun; // runs of the tiled kernel
    const int64_t tile_gy = (tile_rows + kTileRows - 1) / kTileRows;
    if (aligned && tile_gy >= 16 && tile_gy <= 65535) {
      const dim3 grid(kTileRun / kThreads, (unsigned)tile_gy);
      if (has_zp)
        k_quant_tiled<SIGNED, true>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip, lim);
      else
        k_quant_tiled<SIGNED, false>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip, lim);
      return hipGetLastError();
    }
    if (aligned) {
      const int grid =
          stream_grid(n >> 2, kThreads * kUnroll, kGridCapQuantFlat);
      if (has_zp)
        k_quant_flat<SIGNED, true>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip, lim);
      else
        k_quant_flat<SIGNED, false>
            <<<grid, kThreads, 0, st>>>(x, yo, n, scale, zp, flip, lim);
      return hipGetLastError();
    }
    // Misaligned buffers: treat as one long run.
    outer = 1;
    inner = n;
    if (flip != 0) {
      // (the rows of the fused layer, stored minus 128: the general kernel)
      int64_t gx = (n + kThreads - 1) / kThreads;
      gx = gx > 4096 ? 4096 : gx;
      if (has_zp)
        k_quant_general<SIGNED, true><<<dim3((unsigned)gx, 1), kThreads, 0, st>>>(
            x, yo, 1, n, scale, zp, 1, flip);
      else
        k_quant_general<SIGNED, false><<<dim3((unsigned)gx, 1), kThreads, 0, st>>>(
            x, yo, 1, n, scale, zp, 1, flip);
      return hipGetLastError();
    }
  }
  if (flip != 0)
    return hipErrorInvalidValue;
  if (inner == 1 && rt_ok(outer, channels) && ((((uintptr_t)x) & 15) == 0) &&
      ((((uintptr_t)y) & 3) == 0) && ((((uintptr_t)scale) & 3) == 0)) {
    const RtGrid g = rt_grid(outer, channels);
    const unsigned grid = (unsigned)g.gx * (unsigned)g.gy;
    if (has_zp)
      k_quant_rowtable<SIGNED, true><<<grid, kThreads, 0, st>>>(
          x, yo, n, outer, (uint32_t)channels, scale, zp, g);
    else
      k_quant_rowtable<SIGNED, false><<<grid, kThreads, 0, st>>>(
          x, yo, n, outer, (uint32_t)channels, scale, zp, g);
    return hipGetLastError();
  }
  if (inner == 1 && channels > 1 && periodic_pays(channels) &&
      channels < ((int64_t)1 << 31) && ((((uintptr_t)x) & 15) == 0) &&
      ((((uintptr_t)y) & 3) == 0) && (n >> 2) > 0) {
    const PeriodicGrid pg = periodic_grid(n >> 2, channels, 1);
    const bool vec = channels >= 4 && ((((uintptr_t)scale) & 3) == 0);
    if (has_zp && vec)
      k_quant_periodic<SIGNED, true, true><<<pg.grid, kThreads, 0, st>>>(
          x, yo, n, (uint32_t)channels, pg.period, scale, zp, pg.per_block);
    else if (has_zp)
      k_quant_periodic<SIGNED, true, false><<<pg.grid, kThreads, 0, st>>>(
          x, yo, n, (uint32_t)channels, pg.period, scale, zp, pg.per_block);
    else if (vec)
      k_quant_periodic<SIGNED, false, true><<<pg.grid, kThreads, 0, st>>>(
          x, yo, n, (uint32_t)channels, pg.period, scale, zp, pg.per_block);
    else
      k_quant_periodic<SIGNED, false, false><<<pg.grid, kThreads, 0, st>>>(
          x, yo, n, (uint32_t)channels, pg.period, scale, zp, pg.per_block);
    return hipGetLastError();
  }
  if (inner == 1 && channels > 1) {
    const int64_t rows = outer, C = channels;
    const int64_t col_blocks = (C + kThreads * 4 - 1) / (kThreads * 4);
    int64_t rpb, row_blocks;
    rows_per_block(rows, 1, rpb, row_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)row_blocks);
    const bool vec = C % 4 == 0 && ((((uintptr_t)scale) & 15) == 0) &&
                     (!has_zp || ((((uintptr_t)zp) & 3) == 0));
    if (has_zp && vec)
      k_quant_lastaxis<SIGNED, true, true>
          <<<grid, kThreads, 0, st>>>(x, yo, rows, C, scale, zp, (int)rpb);
    else if (has_zp)
      k_quant_lastaxis<SIGNED, true, false>
          <<<grid, kThreads, 0, st>>>(x, yo, rows, C, scale, zp, (int)rpb);
    else if (vec)
      k_quant_lastaxis<SIGNED, false, true>
          <<<grid, kThreads, 0, st>>>(x, yo, rows, C, scale, zp, (int)rpb);
    else
      k_quant_lastaxis<SIGNED, false, false>
          <<<grid, kThreads, 0, st>>>(x, yo, rows, C, scale, zp, (int)rpb);
    return hipGetLastError();
  }
  // General [outer, channels, inner].
  if (slabs_ok(n, channels, inner) && ((((uintptr_t)x) & 15) == 0) &&
      ((((uintptr_t)y) & 3) == 0)) {
    const SlabStep step = slab_step(channels, inner);
    const uint32_t nvec = (uint32_t)(n >> 2);
    constexpr int per_block = kThreads * kSlabQuantPerThread;
    const unsigned grid = (unsigned)((nvec + per_block - 1) / per_block);
    if (has_zp)
      k_quant_slabs<SIGNED, true, kSlabQuantPerThread>
          <<<grid, kThreads, 0, st>>>(x, yo, nvec, step, scale, zp);
    else
      k_quant_slabs<SIGNED, false, kSlabQuantPerThread>
          <<<grid, kThreads, 0, st>>>(x, yo, nvec, step, scale, zp);
    return hipGetLastError();
  }
  if (gather_ok(n, channels, inner) && ((((uintptr_t)x) & 15) == 0) &&
      ((((uintptr_t)y) & 3) == 0)) {
    const unsigned grid = gather_grid(n);
    if (has_zp)
      k_quant_gather<SIGNED, true, false><<<grid, kThreads, 0, st>>>(x, yo,
          (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
    else
      k_quant_gather<SIGNED, false, false><<<grid, kThreads, 0, st>>>(x, yo,
          (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
    return hipGetLastError();
  }
  const int64_t oc = outer * channels;
  const int64_t gy = oc < 4096 ? oc : 4096;
  int64_t gx = (inner + kThreads - 1) / kThreads;
  const int64_t cap = (4096 + gy - 1) / gy;
  if (gx > cap)
    gx = cap;
  if (gx < 1)
    gx = 1;
  dim3 grid((unsigned)gx, (unsigned)gy);
  if (has_zp)
    k_quant_general<SIGNED, true>
        <<<grid, kThreads, 0, st>>>(x, yo, channels, inner, scale, zp, oc);
  else
    k_quant_general<SIGNED, false>
        <<<grid, kThreads, 0, st>>>(x, yo, channels, inner, scale, zp, oc);
  return hipGetLastError();
}

template <int KIND>
hipError_t dequantize_dispatch(hipStream_t st, const void *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    float *y) {
  const int64_t n = outer * channels * inner;
  if (n == 0)
    return hipSuccess;
  const bool has_zp = zp != nullptr;
  if (KIND != kI32 && channels == 1 && ((((uintptr_t)x) & 3) == 0) &&
      ((((uintptr_t)y) & 15) == 0)) {
    const uint8_t *xi = (const uint8_t *)x;
    const int64_t per_block = kThreads * kDequantFlatU;
    const int64_t blocks = ((n >> 2) + per_block - 1) / per_block;
    if (blocks < ((int64_t)1 << 31)) {
      const unsigned grid = (unsigned)(blocks < 1 ? 1 : blocks);
      if (has_zp)
        k_dequant8_flat<KIND, true, kDequantFlatU>
            <<<grid, kThreads, 0, st>>>(xi, y, n, scale, zp);
      else
        k_dequant8_flat<KIND, false, kDequantFlatU>
            <<<grid, kThreads, 0, st>>>(xi, y, n, scale, zp);
      return hipGetLastError();
    }
  }
  if (KIND != kI32 && inner == 1 && rt_ok(outer, channels) &&
      ((((uintptr_t)x) & 3) == 0) && ((((uintptr_t)y) & 15) == 0) &&
      ((((uintptr_t)scale) & 3) == 0)) {
    constexpr int K8 = KIND == kI32 ? kU8 : KIND;
    const RtGrid g = rt_grid(outer, channels);
    const unsigned grid = (unsigned)g.gx * (unsigned)g.gy;
    if (has_zp)
      k_dequant8_rowtable<K8, true><<<grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, outer, (uint32_t)channels, scale, zp, g);
    else
      k_dequant8_rowtable<K8, false><<<grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, outer, (uint32_t)channels, scale, zp, g);
    return hipGetLastError();
  }
  if (KIND != kI32 && inner == 1 && channels > 1 && periodic_pays(channels) &&
      channels < ((int64_t)1 << 31) && ((((uintptr_t)x) & 3) == 0) &&
      ((((uintptr_t)y) & 15) == 0) && (n >> 2) > 0) {
    constexpr int K8 = KIND == kI32 ? kU8 : KIND;
    const PeriodicGrid pg = periodic_grid(n >> 2, channels, 2);
    const bool vec = channels >= 4 && ((((uintptr_t)scale) & 3) == 0);
    if (has_zp && vec)
      k_dequant8_periodic<K8, true, true><<<pg.grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, (uint32_t)channels, pg.period, scale, zp,
          pg.per_block);
    else if (has_zp)
      k_dequant8_periodic<K8, true, false><<<pg.grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, (uint32_t)channels, pg.period, scale, zp,
          pg.per_block);
    else if (vec)
      k_dequant8_periodic<K8, false, true><<<pg.grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, (uint32_t)channels, pg.period, scale, zp,
          pg.per_block);
    else
      k_dequant8_periodic<K8, false, false><<<pg.grid, kThreads, 0, st>>>(
          (const uint8_t *)x, y, n, (uint32_t)channels, pg.period, scale, zp,
          pg.per_block);
    return hipGetLastError();
  }
  if (inner == 1 && channels > 1) {
    const int64_t rows = outer, C = channels;
    const int64_t col_blocks = (C + kThreads * 4 - 1) / (kThreads * 4);
    int64_t rpb, row_blocks;
    rows_per_block(rows, 1, rpb, row_blocks);
    dim3 grid((unsigned)col_blocks, (unsigned)row_blocks);
    const bool vec = C % 4 == 0 && ((((uintptr_t)scale) & 15) == 0) &&
                     (!has_zp || ((((uintptr_t)zp) & 3) == 0));
    if (KIND != kI32 && vec && ((((uintptr_t)x) & 3) == 0) &&
        ((((uintptr_t)y) & 15) == 0) && dequant_rows_ok(rows, C)) {
      constexpr int K8 = KIND == kI32 ? kU8 : KIND;
      dim3 g2((unsigned)col_blocks,
          (unsigned)((rows + kDequantRowsR - 1) / kDequantRowsR));
      if (has_zp)
        k_dequant8_rows<K8, true, kDequantRowsR><<<g2, kThreads, 0, st>>>(
            (const uint8_t *)x, y, rows, C, scale, zp);
      else
        k_dequant8_rows<K8, false, kDequantRowsR><<<g2, kThreads, 0, st>>>(
            (const uint8_t *)x, y, rows, C, scale, zp);
      return hipGetLastError();
    }
    if (has_zp && vec)
      k_dequant_lastaxis<KIND, true, true>
          <<<grid, kThreads, 0, st>>>(x, y, rows, C, scale, zp, (int)rpb);
    else if (has_zp)
      k_dequant_lastaxis<KIND, true, false>
          <<<grid, kThreads, 0, st>>>(x, y, rows, C, scale, zp, (int)rpb);
    else if (vec)
      k_dequant_lastaxis<KIND, false, true>
          <<<grid, kThreads, 0, st>>>(x, y, rows, C, scale, zp, (int)rpb);
    else
      k_dequant_lastaxis<KIND, false, false>
          <<<grid, kThreads, 0, st>>>(x, y, rows, C, scale, zp, (int)rpb);
    return hipGetLastError();
  }
  if (channels == 1) {
    outer = 1;
    inner = n;
  }
  if (KIND != kI32 && slabs_ok(n, channels, inner) &&
      ((((uintptr_t)x) & 3) == 0) && ((((uintptr_t)y) & 15) == 0)) {
    const SlabStep step = slab_step(channels, inner);
    const uint32_t nvec = (uint32_t)(n >> 2);
    constexpr int per_block = kThreads * kSlabDequantPerThread;
    const unsigned grid = (unsigned)((nvec + per_block - 1) / per_block);
    if (has_zp)
      k_dequant8_slabs<(KIND == kI32 ? kU8 : KIND), true, kSlabDequantPerThread>
          <<<grid, kThreads, 0, st>>>(
              (const uint8_t *)x, y, nvec, step, scale, zp);
    else
      k_dequant8_slabs<(KIND == kI32 ? kU8 : KIND), false, kSlabDequantPerThread>
          <<<grid, kThreads, 0, st>>>(
              (const uint8_t *)x, y, nvec, step, scale, zp);
    return hipGetLastError();
  }
  if (KIND != kI32 && gather_ok(n, channels, inner) &&
      ((((uintptr_t)x) & 3) == 0) && ((((uintptr_t)y) & 15) == 0)) {
    const unsigned grid = gather_grid(n);
    constexpr int K8 = KIND == kI32 ? kU8 : KIND;
    if (has_zp)
      k_dequant8_gather<K8, true><<<grid, kThreads, 0, st>>>((const uint8_t *)x,
          y, (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
    else
      k_dequant8_gather<K8, false><<<grid, kThreads, 0, st>>>((const uint8_t *)x,
          y, (uint32_t)n, (uint32_t)channels, (uint32_t)inner, scale, zp);
    return hipGetLastError();
  }
  const int64_t oc = outer * channels;
  const int64_t gy = oc < 4096 ? oc : 4096;
  int64_t gx = (inner + kThreads - 1) / kThreads;
  const int64_t cap = (4096 + gy - 1) / gy;
  if (gx > cap)
    gx = cap;
  if (gx < 1)
    gx = 1;
  dim3 grid((unsigned)gx, (unsigned)gy);
  if (has_zp)
    k_dequant_general<KIND, true>
        <<<grid, kThreads, 0, st>>>(x, y, channels, inner, scale, zp, oc);
  else
    k_dequant_general<KIND, false>
        <<<grid, kThreads, 0, st>>>(x, y, channels, inner, scale, zp, oc);
  return hipGetLastError();
}

} // namespace

hipError_t launch_quantize(hipStream_t s, const float *x, int64_t outer,
    int64_t channels, int64_t inner, const float *scale, const void *zp,
    bool is_signed, void *y, bool reciprocal) {
  if (is_signed)
    return quantize_dispatch<true>(
        s, x, outer, channels, inner, scale, zp, y, 0u, reciprocal);
  return quantize_dispatch<false>(
      s, x, outer, channels, inner, scale, zp, y, 0u, reciprocal);
}

hipError_t launch_dequantize(hipStream_t s, const void *x, QKind xkind,
    int64_t outer, int64_t channels, int64_t inner, const float *scale,
    const void *zp, float *y) {
  switch (xkind) {
  case kU8:
    return dequantize_dispatch<kU8>(s, x, outer, channels, inner, scale, zp, y);
  case kI8:
    return dequantize_dispatch<kI8>(s, x, outer, channels, inner, scale, zp, y);
  default:
    return dequantize_dispatch<kI32>(
        s, x, outer, channels, inner, scale, zp, y);
  }
}

namespace {
std::mutex g_grid_mutex;
hipStream_t g_grid_stream = nullptr; // stream of the last such launch
} // namespace

hipError_t launch_dynamic_quantize(hipStream_t s, DqlScratch &scratch,
    const float *x, int64_t n, uint8_t *y, float *scale, uint8_t *zp,
    bool y_shift, int mode) {
  if (n <= kSmallMax) { // n == 0 included: scale and zero point are written
    k_dql_small<<<1, kSmallThreads, 0, s>>>(
        x, n, y, scale, zp, y_shift ? 0x80808080u : 0u, mode);
    return hipGetLastError();
  }
  // One launch when the tensor fits the registers of a grid that is resident
  // all at once (one block per CU).
  if (mode == 0 && scratch.grid_blocks > 0 && ((((uintptr_t)x) & 15) == 0) &&
      ((((uintptr_t)y) & 3) == 0)) {
    const int64_t total = (int64_t)scratch.grid_blocks * kGridThreads;
    const int64_t nvec = n >> 2;
    void (*fn_launch)(const float *, int64_t, uint8_t *, float *, uint8_t *,
        uint32_t, unsigned long long *, unsigned, unsigned *, unsigned) =
        nullptr;
    // Up to two float4 per thread of the whole grid the launch takes only as
    // many blocks as that needs: the fewer blocks, the shorter the exchange
    // (64 Ki elements: 16 blocks 5.4 us, 4 blocks of 4 float4 per thread 7.0,
    // the two launches of the general path 8.1; 512 Ki: 128 blocks 7.2
    // against 8.2 for 256 blocks of 4 per thread; 96 Ki: 6.1 against 8.1).
    int64_t blocks = scratch.grid_blocks; // <= scratch.max_blocks
    if (nvec <= 2 * total) {
      fn_launch = k_dql_grid<2>;
      blocks = (nvec + 2 * kGridThreads - 1) / (2 * kGridThreads);
    } else if (nvec <= 8 * total)
      fn_launch = k_dql_grid<8>;
    else if (nvec <= kGridMaxPerThread * total)
      fn_launch = k_dql_grid<kGridMaxPerThread>;
    if (fn_launch) {
      const uint32_t flip = y_shift ? 0x80808080u : 0u;
      // If the previous kernel of this kind was launched on another stream and
      // that stream is still busy, this call takes the two-launch path.
      GridExchange ex;
      if (dql_exchange_begin(s, scratch, ex)) {
        hipLaunchKernelGGL(fn_launch, dim3((unsigned)blocks),
            dim3(kGridThreads), 0, s, x, n, y, scale, zp, flip, ex.slots,
            ex.epoch, ex.failed, ex.spin_limit);
        const hipError_t e = hipGetLastError();
        dql_exchange_end(s, e == hipSuccess);
        return e;
      }
    }
  }
  // A read-only reduction streams fastest with few, long-lived blocks
  // (measured on 1 GiB: 512 blocks 6.3 TB/s for the whole op, 4096 blocks
  // 5.9), the opposite of the kernels that also store.
  const int grid = stream_grid(
      n >> 2, kThreads * 8, scratch.max_blocks < 512 ? scratch.max_blocks : 512);
  k_minmax_params<<<grid, kThreads, 0, s>>>(x, n, scratch.partial_min,
      scratch.partial_max, scratch.counter, scale, zp,
      (mode & kQuantNoZeroPoint) ? 1 : 0);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return e;
  // Second pass: the ordinary per-tensor quantize with the parameters just
  // written (the u8 zero point converted back to f32 is the float zero point
  // the reference adds: it is an integer in [0, 255]).
  return quantize_dispatch<false>(s, x, 1, 1, n, scale, zp, y,
      y_shift ? 0x80808080u : 0u, (mode & kQuantReciprocal) != 0);
}

// DynamicQuantizeLinear of a tensor whose minimum and maximum are known:
// limits[0..1] on the GPU, as launch_minmax_limits or a GEMM's epilogue
// (GemmArgs::y_limits) wrote them.  One pass over x.
hipError_t launch_quantize_from_limits(hipStream_t s, const float *x, int64_t n,
    const float *limits, uint8_t *y, float *scale, uint8_t *zp, bool y_shift,
    int mode) {
  QuantLimits lim = {limits, scale, zp, (mode & kQuantNoZeroPoint) ? 1 : 0};
  if (n == 0) { // scale and zero point are written all the same
    k_params_from_limits<<<1, 1, 0, s>>>(lim);
    return hipGetLastError();
  }
  return quantize_dispatch<false>(s, x, 1, 1, n, scale, zp, y,
      y_shift ? 0x80808080u : 0u, (mode & kQuantReciprocal) != 0, &lim);
}

// Minimum and maximum of x (NaN ignored; +inf / -inf for an empty tensor)
// into limits_out[0..1]: the first pass of DynamicQuantizeLinear by itself.
hipError_t launch_minmax_limits(hipStream_t s, DqlScratch &scratch,
    const float *x, int64_t n, float *limits_out) {
  const int grid = stream_grid(
      n >> 2, kThreads * 8, scratch.max_blocks < 512 ? scratch.max_blocks : 512);
  k_minmax_params<<<grid, kThreads, 0, s>>>(x, n, scratch.partial_min,
      scratch.partial_max, scratch.counter, nullptr, nullptr, 0, limits_out);
  return hipGetLastError();
}

bool dql_exchange_begin(hipStream_t s, DqlScratch &scratch, GridExchange &x) {
  if (scratch.grid_blocks <= 0)
    return false;
  g_grid_mutex.lock();
  // (same stream: the previous kernel finishes before the next one starts;
  // streams of this library live as long as their threads)
  if (g_grid_stream && g_grid_stream != s &&
      hipStreamQuery(g_grid_stream) != hipSuccess) {
    (void)hipGetLastError();
    g_grid_mutex.unlock();
    return false;
  }
  if (++scratch.epoch == 0) // 0 is what untouched slots hold
    scratch.epoch = 1;
  x.slots = scratch.grid_slots; // 16-byte aligned
  x.epoch = scratch.epoch;
  x.failed = scratch.counter + 8;
  x.spin_limit = scratch.spin_limit;
  return true;
}

void dql_exchange_end(hipStream_t s, bool launched) {
  if (launched)
    g_grid_stream = s;
  g_grid_mutex.unlock();
}

void dql_forget_stream(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g_grid_mutex);
  if (g_grid_stream == s)
    g_grid_stream = nullptr; // the caller has synchronised it
}

hipError_t launch_fill_u32(hipStream_t s, uint32_t *p, int64_t n, uint32_t v) {
  if (n == 0)
    return hipSuccess;
  k_fill_u32<<<stream_grid(n, kThreads * 4), kThreads, 0, s>>>(p, n, v);
  return hipGetLastError();
}

int dql_grid_blocks() {
  // Blocks of k_dql_grid that are resident at once: one per CU if the
  // occupancy calculator agrees that one fits (32 float4 per thread).
  int dev = 0, cus = 0, per = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) !=
          hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &per, k_dql_grid<kGridMaxPerThread>, kGridThreads, 0) != hipSuccess)
    return 0;
  if (per < 1 || cus < 1)
    return 0;
  return cus < kDqlMaxBlocks ? cus : kDqlMaxBlocks;
}

} // namespace om
