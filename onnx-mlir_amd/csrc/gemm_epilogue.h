// The epilogue shared by the tile GEMM kernels (gemm_kernels.hip,
// gemm_flight.hip): zero-point correction in int32 and the op's output
// conversion, fused into the store.  Device code only.
#pragma once

#include "gemm_common.h"

namespace om {
namespace gemm {

// Epilogue shared by the GEMM kernels: applies the zero-point correction and
// the op's output conversion to a wave's TM x TN grid of 32x32 accumulator
// tiles whose top-left element is (mrow0, ncol0).
// 32x32 accumulator layout: lane holds column (lane & 31); register r holds
// row 8*(r/4) + 4*(lane/32) + (r%4).
//
// The code is kept free of branches around memory operations: every load is
// unconditional (indices clamped, absent operands redirected to valid memory
// and masked afterwards) and all loads precede the stores, so the stores can
// be issued back to back without waiting on one another.
// bj: the bias of the column, or -0.0f, which leaves every value (both zeros
// included) as it is.
template <int EPI>
__device__ __forceinline__ void store_one(const EpiParams &ep, int64_t o,
    uint32_t y, float sj, int32_t yz, float bj) {
  if (EPI == kEpiI32) {
    ((int32_t *)ep.out)[o] = (int32_t)y;
  } else if (EPI == kEpiF32) {
    const float f = (float)(int32_t)y * sj + bj;
    ((float *)ep.out)[o] = relu_f32(f, ep.floor);
  } else {
    const float f = (float)(int32_t)y * sj;
    const int32_t q = (int32_t)__builtin_rintf(f);
    int32_t v = (int32_t)((uint32_t)q + (uint32_t)yz);
    if (ep.narrow == kSaturate) {
      const int32_t lo = ep.y_unsigned ? 0 : -128;
      const int32_t hi = ep.y_unsigned ? 255 : 127;
      v = v < lo ? lo : (v > hi ? hi : v);
    }
    ((uint8_t *)ep.out)[o] = (uint8_t)(v & 0xFF);
  }
}

template <int TM, int TN, int A_MODE, int EPI, int AUX32 = kAuxStream>
__device__ __forceinline__ void gemm_epilogue(v16i (&acc)[TM][TN],
    const int32_t (&rsp)[TM], int mrow0, int ncol0, int M, int N, int K,
    const EpiParams &ep) {
  const int lane = threadIdx.x & 63;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const bool B_UNSIGNED = ep.b_unsigned;
  constexpr bool A_OFF = (A_MODE != 0);
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = B_UNSIGNED ? 128 : 0;

  int32_t yz = 0;
  float a_scale = 0.0f, y_scale = 1.0f;
  if (EPI == kEpiQ8) {
    yz = load_zp_i32(ep.y_zp, ep.y_unsigned, 0);
    y_scale = ep.y_scale[0];
  }
  if (EPI != kEpiI32)
    a_scale = ep.a_scale[0];

  // Absent operands read from colsum (always valid) and are masked to zero.
  const bool has_bzp = ep.b_zp_len > 0;
  const void *bzp_ptr = has_bzp ? ep.b_zp : (const void *)ep.colsum;
  const bool has_azp = ep.a_zp_len > 0;
  const void *azp_ptr = has_azp ? ep.a_zp : (const void *)ep.colsum;
  const bool per_row = ep.a_zp_len > 1;
  const bool has_rs = ep.need_rowsum;
  // rsp[i]: this lane's share of rowsum(A') for row (lane % 32) of row tile i
  // (the two lanes of a row each saw every other 16-byte chunk of K).  After
  // the fold, lane l and lane l+32 both hold the whole sum of row l % 32.
  int32_t rsf[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
    rsf[i] = has_rs ? rsp[i] + __shfl_xor(rsp[i], 32, 64) : 0;

  int n_[TN];
  int32_t db[TN], cs[TN];
  float sj[TN], bj[TN];
  const bool has_bias = EPI == kEpiF32 && ep.bias != nullptr;
  const float *bias_ptr = has_bias ? ep.bias : (const float *)ep.colsum;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    n_[j] = ncol0 + j * 32 + l32;
    const int nc = n_[j] < N ? n_[j] : N - 1;
    // the product is rounded before the bias is added, as Mul then Add are
    const float bv = bias_ptr[has_bias && ep.bias_len > 1 ? nc : 0];
    bj[j] = has_bias ? bv : -0.0f;
    const int32_t bz =
        load_zp_i32(bzp_ptr, B_UNSIGNED, ep.b_zp_len > 1 ? nc : 0);
    db[j] = ob - (has_bzp ? bz : 0);
    cs[j] = ep.colsum[nc];
    sj[j] = 0.0f;
    // a_scale * b_scale[j] first, then one multiply per element; for the
    // requantize (a_scale * b_scale) / y_scale, in this order
    // (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:127).
    if (EPI != kEpiI32) {
      sj[j] = a_scale * ep.b_scale[ep.b_scale_len == 1 ? 0 : nc];
      if (EPI == kEpiQ8)
        sj[j] = sj[j] / y_scale;
    }
  }

  const int32_t az0 = load_zp_i32(azp_ptr, A_OFF, 0);
  const int32_t da0 = oa - (has_azp ? az0 : 0);
  __builtin_amdgcn_sched_barrier(0);

  if (!per_row) {
    // Common case: one zero point for all rows.  The correction is one value
    // per column, computed once per lane, plus db[j] * rowsum(row) when B
    // carries an offset.
    uint32_t cj[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      cj[j] = (uint32_t)da0 * (uint32_t)cs[j] +
              (uint32_t)K * (uint32_t)da0 * (uint32_t)db[j];

    // mrow0 and ncol0 are the same for every lane of the wave (callers derive
    // them from a scalar wave index), so this test and the row addresses below
    // are scalar work.
    const bool full = (mrow0 + 32 * TM <= M) && (ncol0 + 32 * TN <= N) &&
                      (int64_t)N * (32 * TM + 8) * 4 < ((int64_t)1 << 31);
    constexpr int ES = (EPI == kEpiQ8) ? 1 : 4;
    char *const base =
        (char *)ep.out + ((int64_t)mrow0 * N + ncol0) * (int64_t)ES;
    const uint32_t loff =
        ((uint32_t)(4 * lh) * (uint32_t)N + (uint32_t)l32) * (uint32_t)ES;
    // One element: row tile i, register r (row 8*(r/4) + 4*lh + r%4 of the
    // tile), column tile j.  RS: add the row-sum term.
    // Results leave through buffer stores on a descriptor that starts at the
    // wave tile's first element (offsets then fit 32 bits: `full` below also
    // asks for that), written through to memory as they are issued (sc1)
    // instead of sitting in L2 until the kernel ends: the write-back of the
    // whole result at the end of the kernel is otherwise the kernel's last
    // microsecond or two (4096 x 768 x 3072 with f32 results, weights in
    // registers: plain stores 15.9 us, streaming 15.0, written through 13.8;
    // the 8-bit activations of DynamicQuantizeLinear [4096, 3072]: 15.4 ->
    // 13.9 us, and the GEMM that reads them next is not slowed down as it is
    // by streaming stores) -- but only when a wave's 128-byte row pieces are
    // whole lines.  With a row pitch that is no multiple of 128 bytes every
    // piece straddles two lines, and sending the parts to memory one by one
    // costs far more than letting L2 put the lines together (N = 3070:
    // 28.0 us streaming, 19.4 us plain).
    const __amdgpu_buffer_rsrc_t orsrc =
        __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7FFFFFFF, 0x00020000);
    auto emit = [&](auto rs_c, auto stream_c, int i, int r, int j,
                    int32_t rs_row, int32_t rowb) {
      uint32_t y = (uint32_t)acc[i][j][r] + cj[j];
      if (decltype(rs_c)::value)
        y += (uint32_t)db[j] * (uint32_t)rs_row;
      const int voff = (int)(loff + (uint32_t)(j * 32 * ES));
      // 8-bit results: written through.  32-bit results: the caller's choice
      // (streaming for the 128-wide tiles, 4096 x 768 x 768 7.4 us against 7.8
      // written through; written through for k_gemm_i8_bs, 2048 x 4096 x 11008
      // 93.9 us against 94.5 streaming).
      constexpr int kAux = !decltype(stream_c)::value ? 0
                           : EPI == kEpiQ8            ? kAuxThrough
                                                      : AUX32;
      if (EPI == kEpiI32) {
        __builtin_amdgcn_raw_buffer_store_b32((int)y, orsrc, voff, rowb, kAux);
      } else if (EPI == kEpiF32) {
        float f = (float)(int32_t)y * sj[j] + bj[j];
        f = relu_f32(f, ep.floor);
        __builtin_amdgcn_raw_buffer_store_b32(
            (int)__float_as_uint(f), orsrc, voff, rowb, kAux);
      } else {
        const float f = (float)(int32_t)y * sj[j];
        int32_t v =
            (int32_t)((uint32_t)(int32_t)__builtin_rintf(f) + (uint32_t)yz);
        if (ep.narrow == kSaturate) {
          const int32_t lo = ep.y_unsigned ? 0 : -128;
          const int32_t hi = ep.y_unsigned ? 255 : 127;
          v = v < lo ? lo : (v > hi ? hi : v);
        }
        __builtin_amdgcn_raw_buffer_store_b8(
            (unsigned char)(v & 0xFF), orsrc, voff, rowb, kAux);
      }
    };
    auto whole = [&](auto rs_c, auto stream_c) {
      // Whole grid inside the matrix: no bounds tests, and every address is
      // (scalar row base) + (one 32-bit lane offset) + constant, so a store
      // costs the few vector instructions that produce its value.
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rr = 8 * (r >> 2) + 4 * lh + (r & 3);
          const int32_t rs_row =
              decltype(rs_c)::value ? __shfl(rsf[i], rr, 64) : 0;
          const int32_t rowb =
              (int32_t)((i * 32 + 8 * (r >> 2) + (r & 3)) * N * ES);
#pragma unroll
          for (int j = 0; j < TN; ++j)
            emit(rs_c, stream_c, i, r, j, rs_row, rowb);
        }
      }
    };
    if (full) {
      const bool whole_lines = ((int64_t)N * ES) % 128 == 0;
      if (has_rs) {
        if (whole_lines)
          whole(std::true_type{}, std::true_type{});
        else
          whole(std::true_type{}, std::false_type{});
      } else {
        if (whole_lines)
          whole(std::false_type{}, std::true_type{});
        else
          whole(std::false_type{}, std::false_type{});
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mbase = mrow0 + i * 32 + 4 * lh;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int rr = 8 * (r >> 2) + 4 * lh + (r & 3);
        const int m = mbase + 8 * (r >> 2) + (r & 3);
        const int32_t rs_row = __shfl(rsf[i], rr, 64);
        const int64_t orow = (int64_t)m * N;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint32_t y = (uint32_t)acc[i][j][r] + cj[j] +
                             (uint32_t)db[j] * (uint32_t)rs_row;
          if (m < M && n_[j] < N)
            store_one<EPI>(ep, orow + n_[j], y, sj[j], yz, bj[j]);
        }
      }
    }
    return;
  }

  // Per-row zero points: four rows at a time, to keep the register footprint
  // of this rarely taken path small.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int mbase = mrow0 + i * 32 + 4 * lh;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      int32_t da[4], rs[4];
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int m = mbase + 8 * rg + rr;
        const int mc = m < M ? m : M - 1;
        const int32_t az = load_zp_i32(azp_ptr, A_OFF, per_row ? mc : 0);
        da[rr] = oa - (has_azp ? az : 0);
        rs[rr] = __shfl(rsf[i], 8 * rg + 4 * lh + rr, 64);
      }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int r = rg * 4 + rr;
        const int m = mbase + 8 * rg + rr;
        const int64_t orow = (int64_t)m * N;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          uint32_t y = (uint32_t)acc[i][j][r];
          y += (uint32_t)da[rr] * (uint32_t)cs[j];
          y += (uint32_t)db[j] * (uint32_t)rs[rr];
          y += (uint32_t)K * (uint32_t)da[rr] * (uint32_t)db[j];
          if (m < M && n_[j] < N)
            store_one<EPI>(ep, orow + n_[j], y, sj[j], yz, bj[j]);
        }
      }
    }
  }
}

} // namespace gemm
} // namespace om
