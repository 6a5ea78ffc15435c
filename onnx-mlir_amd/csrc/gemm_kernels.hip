// int8 GEMM for gfx950 on the matrix cores (v_mfma_i32_32x32x32_i8), with the
// zero-point correction applied exactly in int32 and the epilogues of
// MatMulInteger (int32), MatMulInteger+Cast+Mul (f32) and QLinearMatMul
// (8-bit requantize) fused into the store.
//
// What is computed (src/Conversion/ONNXToKrnl/Math/MatMulInteger.cpp:59-90,
// src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:88-138):
//     Y[i,j] = sum_k (A[i,k] - az[i]) * (B[k,j] - bz[j])        (mod 2^32)
// The matrix cores multiply signed 8-bit values, so an unsigned operand is
// moved to int8 by subtracting 128 (XOR 0x80): A = A' + oa, B = B' + ob with
// oa, ob in {0, 128}.  With da[i] = oa - az[i] and db[j] = ob - bz[j]
//     Y[i,j] = sum_k A'B' + db[j]*rowsum(A')[i] + da[i]*colsum(B')[j]
//              + K*da[i]*db[j]                                  (mod 2^32)
// which is exact because int32 addition and multiplication wrap.
//
// Layout: A is used as given ([M,K] row-major, K contiguous).  B is packed
// once into Bt [Npad,Kpad] int8 (K contiguous, zero filled), so both MFMA
// operands are read as 16 consecutive K bytes per lane.
//
// Kernels (all walk K in steps of 64 bytes; LDS rows are 64 bytes and the
// 16-byte chunk index is XOR-swizzled with bits 2..3 of the row, so operand
// reads and tile writes are bank-conflict free):
//   k_gemm_i8_dma     tiles copied from global memory straight into a ring of
//                     three LDS stages (no register staging); the default
//   k_gemm_i8         tiles staged through registers, LDS double buffered;
//                     also the byte-wise path for odd K or a misaligned A
//   k_gemm_i8_stream  A read from a fragment-packed copy straight into MFMA
//                     operand registers, only Bt through LDS; large problems
//   k_gemm_i8_skinny  M <= 16: weight streaming, K split over the waves

#include "om_kernels.h"

#include <stdlib.h>

#include <type_traits>

namespace om {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BK = kGemmBK;

// Byte offset of 16-byte chunk `c` (0..3) of tile row `r` (row = 64 bytes).
__device__ __forceinline__ int lds_off(int r, int c) {
  return r * BK + ((c ^ ((r >> 2) & 3)) << 4);
}

// Barrier that orders LDS accesses only; global loads already issued keep
// flying across it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct EpiParams {
  const void *a_zp;
  int64_t a_zp_len;
  const void *b_zp;
  int64_t b_zp_len;
  const int32_t *rowsum;
  const int32_t *colsum;
  const float *a_scale;
  const float *b_scale;
  int64_t b_scale_len;
  const float *y_scale;
  const void *y_zp;
  void *out;
  bool b_unsigned;
  bool y_unsigned;
  int narrow;
  int group;   // tile rows per scheduling group
  int xcd;     // renumber workgroups per XCD
};

__device__ __forceinline__ int32_t load_zp_i32(
    const void *p, bool is_unsigned, int64_t i) {
  return is_unsigned ? (int32_t)((const uint8_t *)p)[i]
                     : (int32_t)((const int8_t *)p)[i];
}

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
template <int EPI>
__device__ __forceinline__ void store_one(const EpiParams &ep, int64_t o,
    uint32_t y, float sj, int32_t yz) {
  if (EPI == kEpiI32) {
    ((int32_t *)ep.out)[o] = (int32_t)y;
  } else if (EPI == kEpiF32) {
    ((float *)ep.out)[o] = (float)(int32_t)y * sj;
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

template <int TM, int TN, int A_MODE, int EPI>
__device__ __forceinline__ void gemm_epilogue(v16i (&acc)[TM][TN], int mrow0,
    int ncol0, int M, int N, int K, const EpiParams &ep) {
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
  const bool has_rs = ep.rowsum != nullptr;
  const int32_t *rs_ptr = has_rs ? ep.rowsum : ep.colsum;

  int n_[TN];
  int32_t db[TN], cs[TN];
  float sj[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    n_[j] = ncol0 + j * 32 + l32;
    const int nc = n_[j] < N ? n_[j] : N - 1;
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

  if (!per_row && !has_rs) {
    // Common case: one zero point for all rows and no offset on B.  The whole
    // correction is then one value per column, computed once per lane.
    uint32_t cj[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      cj[j] = (uint32_t)da0 * (uint32_t)cs[j] +
              (uint32_t)K * (uint32_t)da0 * (uint32_t)db[j];

    // mrow0 and ncol0 are the same for every lane of the wave (callers derive
    // them from a scalar wave index), so this test and the row addresses below
    // are scalar work.
    const bool full = (mrow0 + 32 * TM <= M) && (ncol0 + 32 * TN <= N);
    if (full) {
      // Whole grid inside the matrix: no bounds tests, and every address is
      // (scalar row base) + (one 32-bit lane offset) + constant, so a store
      // costs the two or three vector instructions that produce its value.
      constexpr int ES = (EPI == kEpiQ8) ? 1 : 4;
      char *const base =
          (char *)ep.out + ((int64_t)mrow0 * N + ncol0) * (int64_t)ES;
      const uint32_t loff =
          ((uint32_t)(4 * lh) * (uint32_t)N + (uint32_t)l32) * (uint32_t)ES;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t rowb =
              (int64_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * N * (int64_t)ES;
          char *const rowp = base + rowb;
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const uint32_t y = (uint32_t)acc[i][j][r] + cj[j];
            char *const q = rowp + loff + (uint32_t)(j * 32 * ES);
            // Streaming stores: the result is not read again by this kernel,
            // and keeping it out of the way in L2 leaves the A and Bt panels
            // cached for the blocks still in their K loop (measured faster).
            if (EPI == kEpiI32) {
              __builtin_nontemporal_store((int32_t)y, (int32_t *)q);
            } else if (EPI == kEpiF32) {
              __builtin_nontemporal_store(
                  (float)(int32_t)y * sj[j], (float *)q);
            } else {
              const float f = (float)(int32_t)y * sj[j];
              int32_t v = (int32_t)((uint32_t)(int32_t)__builtin_rintf(f) +
                                    (uint32_t)yz);
              if (ep.narrow == kSaturate) {
                const int32_t lo = ep.y_unsigned ? 0 : -128;
                const int32_t hi = ep.y_unsigned ? 255 : 127;
                v = v < lo ? lo : (v > hi ? hi : v);
              }
              *(uint8_t *)q = (uint8_t)(v & 0xFF);
            }
          }
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mbase = mrow0 + i * 32 + 4 * lh;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mbase + 8 * (r >> 2) + (r & 3);
        const int64_t orow = (int64_t)m * N;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint32_t y = (uint32_t)acc[i][j][r] + cj[j];
          if (m < M && n_[j] < N)
            store_one<EPI>(ep, orow + n_[j], y, sj[j], yz);
        }
      }
    }
    return;
  }

  // Per-row zero points and / or row sums: four rows at a time, to keep the
  // register footprint of this rarely taken path small.
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
        const int32_t rv = rs_ptr[has_rs ? mc : 0];
        rs[rr] = has_rs ? rv : 0;
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
            store_one<EPI>(ep, orow + n_[j], y, sj[j], yz);
        }
      }
    }
  }
}


// BM x BN block tile, WGM x WGN waves, each wave a (BM/WGM) x (BN/WGN) tile
// made of 32x32 MFMA tiles.
// A_MODE: 0 = int8 as is, 1 = uint8 (XOR 0x80 while staging), 2 = already
// shifted (stored as u8-128) -- offsets as for uint8, no XOR.
// ALIGNED: K % 64 == 0 and A 16-byte aligned (vector loads), else byte loads.
template <int BM, int BN, int WGM, int WGN, int MINB, int A_MODE, int EPI,
    bool ALIGNED>
__global__ __launch_bounds__(WGM *WGN * 64, MINB) void k_gemm_i8(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bt, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  constexpr int THREADS = WGM * WGN * 64;
  constexpr int WTM = BM / WGM, WTN = BN / WGN; // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;   // MFMA tiles per wave
  constexpr int CH_A = BM * 4 / THREADS;        // 16-byte chunks per thread
  constexpr int CH_B = BN * 4 / THREADS;
  static_assert(BM * 4 % THREADS == 0 && BN * 4 % THREADS == 0, "tile/threads");

  __shared__ __attribute__((aligned(16))) uint8_t sA[2][BM * BK];
  __shared__ __attribute__((aligned(16))) uint8_t sB[2][BN * BK];

  // Tile order.  Consecutive workgroup ids are dealt round-robin to the 8
  // XCDs, each with its own L2; renumber so that one XCD gets a contiguous
  // range, then walk that range in groups of 8 tile rows so the tiles resident
  // on an XCD share a few A panels and Bt panels.
  int pid = blockIdx.x;
  {
    const int nb = gridDim.x;
    const int per = nb >> 3;
    if (per > 0 && pid < per * 8)
      pid = (pid & 7) * per + (pid >> 3);
  }
  constexpr int GROUP = 8;
  const int in_group = GROUP * tiles_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
  const int tm = first_m + (pid % in_group) % gsize;
  const int tn = (pid % in_group) / gsize;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // wave index as a scalar: everything derived from it (tile origin, LDS
  // bases, output rows) then lives in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;


  constexpr int kFill = (A_MODE == 1) ? (int)0x80808080 : 0;

  // Global loads only fetch; uint8 data is shifted to int8 after it is read
  // back from LDS.  In the byte-wise path chunks outside [M,K] are filled with
  // the byte that the shift maps to 0.
  auto load_global = [&](int k0, v4i(&ra)[CH_A], v4i(&rb)[CH_B]) {
#pragma unroll
    for (int h = 0; h < CH_A; ++h) {
      const int q = tid + h * THREADS;
      const int r = q >> 2, c = q & 3;
      const int gm = m0 + r;
      const int gk = k0 + c * 16;
      v4i v = {kFill, kFill, kFill, kFill};
      if (ALIGNED) {
        // K % 64 == 0, so every chunk lies inside its row.  Rows past M are
        // clamped to the last row: they only feed output rows that are never
        // stored, and an unconditional load lets the hardware counter of
        // outstanding loads be waited on exactly (a load under a branch
        // would force a full drain).
        const int gmc = gm < M ? gm : M - 1;
        v = *(const v4i *)(A + (int64_t)gmc * K + gk);
      } else {
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int b = 0; b < 16; ++b) {
          const int kk = gk + b;
          uint32_t byte = (uint32_t)kFill & 0xFFu;
          if (gm < M && kk < K)
            byte = A[(int64_t)gm * K + kk];
          w[b >> 2] |= byte << ((b & 3) * 8);
        }
        v = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
      }
      ra[h] = v;
    }
#pragma unroll
    for (int h = 0; h < CH_B; ++h) {
      const int q = tid + h * THREADS;
      const int r = q >> 2, c = q & 3;
      // Bt is padded to [Npad, Kpad]: always in bounds and aligned.
      rb[h] = *(const v4i *)(Bt + (int64_t)(n0 + r) * Kpad + k0 + c * 16);
    }
  };
  auto store_lds = [&](int buf, const v4i(&ra)[CH_A], const v4i(&rb)[CH_B]) {
#pragma unroll
    for (int h = 0; h < CH_A; ++h) {
      const int q = tid + h * THREADS;
      *(v4i *)(&sA[buf][lds_off(q >> 2, q & 3)]) = ra[h];
    }
#pragma unroll
    for (int h = 0; h < CH_B; ++h) {
      const int q = tid + h * THREADS;
      *(v4i *)(&sB[buf][lds_off(q >> 2, q & 3)]) = rb[h];
    }
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  const int l32 = lane & 31;
  const int lh = lane >> 5;

  auto compute = [&](int buf) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c = s * 2 + lh;
      v4i fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        fa[i] = *(const v4i *)(&sA[buf][lds_off(wm * WTM + i * 32 + l32, c)]);
        // uint8 -> int8 (minus 128) on the operand registers: VALU work that
        // runs beside the MFMAs and keeps the staging path free of any use
        // of freshly loaded data.
        if (A_MODE == 1)
          fa[i] ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
              (int)0x80808080};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = *(const v4i *)(&sB[buf][lds_off(wn * WTN + j * 32 + l32, c)]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
              fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  };

  // Every load and LDS store below is unconditional (steps past the end are
  // clamped to the last step and their data is never consumed): with no
  // branch around a load the compiler can wait for exactly the register set
  // it is about to store and leave the other set's loads in flight.
  const int KT = Kpad / BK;
  const int klast = (KT - 1) * BK;
  auto kclamp = [&](int step) { return step < KT ? step * BK : klast; };
  v4i ra0[CH_A], rb0[CH_B], ra1[CH_A], rb1[CH_B];
  load_global(0, ra0, rb0);
  load_global(kclamp(1), ra1, rb1);
  store_lds(0, ra0, rb0);
  load_global(kclamp(2), ra0, rb0);
  lds_barrier();

  int kt = 0;
  while (true) {
    // even step: MFMAs on buffer 0; step kt+1 goes to buffer 1 from set 1,
    // then set 1 fetches step kt+3.
    compute(0);
    __builtin_amdgcn_sched_barrier(0);
    store_lds(1, ra1, rb1);
    load_global(kclamp(kt + 3), ra1, rb1);
    lds_barrier();
    if (++kt >= KT)
      break;
    compute(1);
    __builtin_amdgcn_sched_barrier(0);
    store_lds(0, ra0, rb0);
    load_global(kclamp(kt + 3), ra0, rb0);
    lds_barrier();
    if (++kt >= KT)
      break;
  }
  gemm_epilogue<TM, TN, A_MODE, EPI>(
      acc, m0 + wm * WTM, n0 + wn * WTN, M, N, K, ep);
}

// ---- GEMM, tiles copied from global memory straight into LDS --------------
// gfx950 can write a 16-byte global load into LDS without passing through
// vector registers (global_load_lds_dwordx4): LDS address = M0 + lane * 16, so
// one wave instruction fills 1 KiB of consecutive LDS and the per-lane global
// address decides what lands where.  That removes the register staging, the
// ds_write instructions and the wait that tied them to the loads; a wave only
// issues the copies, waits for its own to land, and meets the others at one
// barrier per K step.
//
// LDS holds a ring of three stages (A tile + Bt tile of one 64-byte K step
// each, same XOR-swizzled row layout as above).  In step k a wave
//   waits until its copies for step k have landed (those for k+1 stay in
//   flight), passes the barrier -- now every wave's step-k data is in LDS and
//   every wave is done reading stage (k-1)%3 --,
//   issues its copies for step k+2 into stage (k-1)%3,
//   reads the operands of stage k%3 and runs the MFMAs.
// The operand reads are written as inline assembly: the compiler would make
// every LDS read wait for all outstanding copies into LDS, whichever stage
// they target.  The counts waited for below are therefore explicit.
template <int BN, int NSTAGE, int MINB, int A_MODE, int EPI>
__global__ __launch_bounds__(256, MINB) void k_gemm_i8_dma(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bt, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  // 2 x 2 waves, each a 64 x (BN/2) tile.
  constexpr int BM = 128, WTM = 64, WTN = BN / 2, TM = 2, TN = WTN / 32;
  static_assert(BN == 128 || BN == 64, "tile width");
  constexpr int STAGE = (BM + BN) * BK;
  constexpr int CB = BN / 64;      // Bt copies per wave and step
  constexpr int CPW = 2 + CB;      // copies per wave and step
  __shared__ __attribute__((aligned(1024))) uint8_t sm[NSTAGE * STAGE];

  int pid = blockIdx.x;
  {
    const int nb = gridDim.x;
    const int per = nb >> 3;
    if (per > 0 && pid < per * 8)
      pid = (pid & 7) * per + (pid >> 3);
  }
  constexpr int GROUP = 8;
  const int in_group = GROUP * tiles_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
  const int tm = first_m + (pid % in_group) % gsize;
  const int tn = (pid % in_group) / gsize;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31;
  const int lh = lane >> 5;

  // Copy addressing.  Copy instruction j of a tile fills LDS bytes
  // [j*1024, (j+1)*1024): lane -> row j*16 + lane/4, chunk position lane%4,
  // which holds chunk (lane%4) ^ ((row/4)%4) = (lane%4) ^ ((lane/16)%4) of the
  // row.  A wave issues copies 2*wave, 2*wave+1 of A and CB consecutive copies
  // of Bt.
  const int crow = lane >> 2;
  const int cchunk = (lane & 3) ^ ((lane >> 4) & 3);
  const uint8_t *ga[2];
  const int8_t *gb[CB];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = (wave * 2 + h) * 16 + crow;
    const int gm = (m0 + r < M) ? m0 + r : M - 1; // rows past M: never stored
    ga[h] = A + (int64_t)gm * K + cchunk * 16;
  }
#pragma unroll
  for (int h = 0; h < CB; ++h) {
    const int r = (wave * CB + h) * 16 + crow;
    gb[h] = Bt + (int64_t)(n0 + r) * Kpad + cchunk * 16;
  }
  typedef __attribute__((address_space(3))) void *lds_ptr;
  typedef const __attribute__((address_space(1))) void *glb_ptr;
  auto copy_step = [&](int k0, int stage) {
    uint8_t *base = sm + stage * STAGE;
#pragma unroll
    for (int h = 0; h < 2; ++h)
      __builtin_amdgcn_global_load_lds((glb_ptr)(ga[h] + k0),
          (lds_ptr)(base + (wave * 2 + h) * 1024), 16, 0, 0);
#pragma unroll
    for (int h = 0; h < CB; ++h)
      __builtin_amdgcn_global_load_lds((glb_ptr)(gb[h] + k0),
          (lds_ptr)(base + BM * BK + (wave * CB + h) * 1024), 16, 0, 0);
  };

  // Operand addressing: sub-step s (0,1) of a stage uses chunk 2*s + lane/32 of
  // row (wave tile row + lane%32); MFMA tile i adds 32 rows = 2048 bytes.
  const unsigned sm_base = (unsigned)(uintptr_t)(lds_ptr)sm;
  unsigned ra[2], rb[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    ra[s] = sm_base + lds_off(wm * WTM + l32, s * 2 + lh);
    rb[s] = sm_base + BM * BK + lds_off(wn * WTN + l32, s * 2 + lh);
  }

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  const int KT = Kpad / BK;
  const int klast = (KT - 1) * BK;
  auto kclamp = [&](int step) { return step < KT ? step * BK : klast; };
#pragma unroll
  for (int p = 0; p < NSTAGE - 1; ++p)
    copy_step(kclamp(p), p);

  // One LDS read of an MFMA operand.  Kept opaque to the compiler, see above;
  // lds_wait<n>() makes the operands it is given valid once at most n reads
  // are still outstanding (reads complete in order).
  auto lds_read = [](v4i &f, unsigned addr, auto off) {
    asm volatile("ds_read_b128 %0, %1 offset:%2"
                 : "=v"(f)
                 : "v"(addr), "n"(decltype(off)::value)
                 : "memory");
  };

  int stage = 0; // kt % NSTAGE
  for (int kt = 0; kt < KT; ++kt) {
    const int prev = (stage == 0) ? NSTAGE - 1 : stage - 1;
    // Own copies of step kt have landed; those of the NSTAGE-2 steps after it
    // may still be in flight.
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((NSTAGE - 2) * CPW));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    copy_step(kclamp(kt + NSTAGE - 1), prev);
    __builtin_amdgcn_sched_barrier(0);
    const unsigned soff = (unsigned)(stage * STAGE);
    v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    using O0 = std::integral_constant<int, 0>;
    using O1 = std::integral_constant<int, 2048>;
    lds_read(fa0[0], ra[0] + soff, O0{});
    lds_read(fa0[1], ra[0] + soff, O1{});
    lds_read(fb0[0], rb[0] + soff, O0{});
    if (TN == 2)
      lds_read(fb0[TN - 1], rb[0] + soff, O1{});
    lds_read(fa1[0], ra[1] + soff, O0{});
    lds_read(fa1[1], ra[1] + soff, O1{});
    lds_read(fb1[0], rb[1] + soff, O0{});
    if (TN == 2)
      lds_read(fb1[TN - 1], rb[1] + soff, O1{});
    if (TN == 2)
      asm volatile("s_waitcnt lgkmcnt(4)"
                   : "+v"(fa0[0]), "+v"(fa0[1]), "+v"(fb0[0]), "+v"(fb0[TN - 1])
                   :
                   : "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(3)"
                   : "+v"(fa0[0]), "+v"(fa0[1]), "+v"(fb0[0])
                   :
                   : "memory");
    if (A_MODE == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa0[i] ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
            (int)0x80808080};
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa0[i], fb0[j], acc[i][j], 0, 0, 0);
    if (TN == 2)
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(fa1[0]), "+v"(fa1[1]), "+v"(fb1[0]), "+v"(fb1[TN - 1])
                   :
                   : "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(fa1[0]), "+v"(fa1[1]), "+v"(fb1[0])
                   :
                   : "memory");
    if (A_MODE == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa1[i] ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
            (int)0x80808080};
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa1[i], fb1[j], acc[i][j], 0, 0, 0);
    stage = (stage == NSTAGE - 1) ? 0 : stage + 1;
  }
  // Copies past the last step are still landing in LDS; nothing reads them,
  // but the block must not release its LDS before they are done.
  __builtin_amdgcn_s_waitcnt(0x0F70);

  gemm_epilogue<TM, TN, A_MODE, EPI>(
      acc, m0 + wm * WTM, n0 + wn * WTN, M, N, K, ep);
}

// ---- GEMM, A streamed to registers ----------------------------------------
// LDS stores are the scarcest on-chip resource of a CU (about a third of the
// LDS read rate), so this kernel keeps A out of LDS altogether.  The four
// waves of a block are stacked along M: a wave owns 32*TM rows that no other
// wave needs, and reads its A operands straight from global memory in MFMA
// operand layout (lane = row, 16 K-bytes per lane).  Only the Bt tile, which
// all four waves share, goes through LDS: a ring of three 64-byte-deep stages.
//
// Global loads run D steps ahead in registers (D register sets, loop unrolled
// by D so that every set is addressed statically).  Per K step (64 bytes) a
// wave issues, in this order,
//   ds_read  B operands of sub-step 1 (this step's stage)
//   MFMAs of sub-step 0; A registers of sub-step 0 are refilled for step +D
//   ds_write the staged Bt chunk of step +2 into its stage; refetch step +2+D
//   ds_read  B operands of sub-step 0 of step +1 (stage published one barrier
//            ago -- this is what the third stage buys: nothing waits on LDS
//            right after the barrier)
//   MFMAs of sub-step 1; A registers of sub-step 1 are refilled for step +D
//   one LDS-only barrier
// All loads are unconditional (clamped), so every wait is an exact count.
template <int TM, int TN, int D, int A_MODE, int EPI>
__global__ __launch_bounds__(256, (TM == 1 ? 2 : 1)) void k_gemm_i8_stream(
    const uint8_t *__restrict__ Ap, const int8_t *__restrict__ Bt, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  constexpr int BM = 4 * 32 * TM, BN = 32 * TN;
  constexpr int CH_B = BN * 4 / 256; // 16-byte chunks of Bt per thread, per step
  static_assert(BN * 4 % 256 == 0, "BN must be a multiple of 64");
  constexpr int STAGE = BN * BK;

  __shared__ __attribute__((aligned(16))) uint8_t sB[3 * STAGE];

  int pid = blockIdx.x;
  if (ep.xcd) {
    const int nb = gridDim.x;
    const int per = nb >> 3;
    if (per > 0 && pid < per * 8)
      pid = (pid & 7) * per + (pid >> 3);
  }
  const int GROUP = ep.group;
  const int in_group = GROUP * tiles_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
  const int tm = first_m + (pid % in_group) % gsize;
  const int tn = (pid % in_group) / gsize;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int mrow0 = m0 + wave * 32 * TM;

  const int KT = Kpad / BK;
  const int klast = (KT - 1) * BK;
  auto kclamp = [&](int step) { return step < KT ? step * BK : klast; };

  // A operand pointers into the fragment-packed copy of A (see k_pack_a): the
  // operand of MFMA row tile mt, step ks, half step sub is one contiguous KiB,
  // 16 bytes per lane.  Row tiles past the last one are clamped (they only
  // feed output rows that are never stored).
  const uint8_t *__restrict__ arow[TM];
  {
    const int mt_max = (M + 31) / 32 - 1;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      int mt = (mrow0 >> 5) + i;
      mt = mt < mt_max ? mt : mt_max;
      arow[i] = Ap + (int64_t)mt * KT * 2048 + lane * 16;
    }
  }
  // Bt staging pointers: chunk q -> row q>>2, 16-byte chunk q&3.
  const int8_t *__restrict__ brow[CH_B];
  int bdst[CH_B];
#pragma unroll
  for (int h = 0; h < CH_B; ++h) {
    const int q = tid + h * 256;
    // Bt has round_up(N, kGemmBN) rows; a tile whose width does not divide
    // that may reach past it: clamp (those columns are never stored).
    const int npad = (N + kGemmBN - 1) / kGemmBN * kGemmBN;
    int bn = n0 + (q >> 2);
    bn = bn < npad ? bn : npad - 1;
    brow[h] = Bt + (int64_t)bn * Kpad + (q & 3) * 16;
    bdst[h] = lds_off(q >> 2, q & 3);
  }

  // k0 is a byte offset along K (64 per step); a step of packed A is 2 KiB.
  auto load_a = [&](int k0, int sub, v4i(&ra)[TM]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      ra[i] = *(const v4i *)(arow[i] + k0 * 32 + sub * 1024);
  };
  auto load_b = [&](int k0, v4i(&rb)[CH_B]) {
#pragma unroll
    for (int h = 0; h < CH_B; ++h)
      rb[h] = *(const v4i *)(brow[h] + k0);
  };
  auto write_b = [&](int stage, const v4i(&rb)[CH_B]) {
#pragma unroll
    for (int h = 0; h < CH_B; ++h)
      *(v4i *)(&sB[stage * STAGE + bdst[h]]) = rb[h];
  };
  auto read_frag = [&](int stage, int sub, v4i(&fb)[TN]) {
    const int c = sub * 2 + lh;
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *(const v4i *)(&sB[stage * STAGE + lds_off(j * 32 + l32, c)]);
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  auto mfma_sub = [&](const v4i(&ra)[TM], const v4i(&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            ra[i], fb[j], acc[i][j], 0, 0, 0);
    }
  };

  // D register sets: as[u][sub] holds A of a step with (step % D) == u;
  // bs[u] holds the staged Bt chunk of the step two ahead of that.
  v4i as[D][2][TM];
  v4i bs[D][CH_B];
  v4i f0[TN], f1[TN];

  // Prologue.  Bt of steps 0 and 1 goes to stages 0 and 1 through bs[0],
  // bs[1]; then bs[u] is filled with step 2+u.  as[u] is filled with step u.
  load_b(0, bs[0]);
  load_b(kclamp(1), bs[D > 1 ? 1 : 0]);
#pragma unroll
  for (int u = 0; u < D; ++u) {
    load_a(kclamp(u), 0, as[u][0]);
    load_a(kclamp(u), 1, as[u][1]);
  }
  write_b(0, bs[0]);
  if (D > 1)
    write_b(1, bs[1]);
  else {
    load_b(kclamp(1), bs[0]);
    write_b(1, bs[0]);
  }
#pragma unroll
  for (int u = 0; u < D; ++u)
    load_b(kclamp(2 + u), bs[u]);
  lds_barrier();
  read_frag(0, 0, f0);

  int kt = 0;
  int st0 = 0, st1 = 1, st2 = 2; // stages of steps kt, kt+1, kt+2
  bool done = false;
  while (!done) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      read_frag(st0, 1, f1);
      mfma_sub(as[u][0], f0);
      load_a(kclamp(kt + D), 0, as[u][0]);
      write_b(st2, bs[u]);
      load_b(kclamp(kt + 2 + D), bs[u]);
      read_frag(st1, 0, f0);
      mfma_sub(as[u][1], f1);
      load_a(kclamp(kt + D), 1, as[u][1]);
      lds_barrier();
      if (++kt >= KT) {
        done = true;
        break;
      }
      const int t = st0;
      st0 = st1;
      st1 = st2;
      st2 = t;
    }
  }

  gemm_epilogue<TM, TN, A_MODE, EPI>(acc, mrow0, n0, M, N, K, ep);
}

// ---- skinny GEMM (M <= 16): weight streaming -------------------------------
// With at most 16 rows the product is bound by reading the weights once, so
// the kernel is organised around keeping many KiB of Bt in flight per CU and
// nothing else: a block owns 32 output columns, its 8 waves split K between
// them, and each wave streams its slice of the 32 Bt rows straight from
// global memory into v_mfma_i32_16x16x64_i8 operands (lane = column, 16
// K-bytes per lane; a wave instruction reads 16 rows x 64 contiguous bytes).
// The tiny A operand (rows padded to 16 with zeros) comes from L2.  The eight
// partial 16x32 results are summed through LDS and the usual epilogue runs on
// the sum.  No LDS staging, no barrier in the K loop.
template <int NG, int A_MODE, int EPI>
__global__ __launch_bounds__(512) void k_gemm_i8_skinny(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bt, int M, int N,
    int K, int Kpad, EpiParams ep) {
  constexpr int WAVES = 8, U = 8;
  __shared__ int32_t part[WAVES][NG][4][64];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int lq = lane >> 4; // K quarter of the 64-byte step
  const int n0 = blockIdx.x * 16 * NG;

  const int KT = Kpad / BK;
  const int per = (KT + WAVES - 1) / WAVES;
  const int kt_begin = wave * per;
  const int kt_end = (kt_begin + per < KT) ? kt_begin + per : KT;

  // Row l16 of A (clamped; rows >= M are zeroed after the load).
  const bool row_ok = l16 < M;
  const uint8_t *__restrict__ ap =
      A + (int64_t)(row_ok ? l16 : 0) * K + (lq * 16 < K ? lq * 16 : 0);
  const int8_t *__restrict__ bp0 = Bt + (int64_t)(n0 + l16) * Kpad + lq * 16;
  const int8_t *__restrict__ bp1 = bp0 + (int64_t)(NG > 1 ? 16 : 0) * Kpad;
  const int klim = K - lq * 16; // chunks starting at or past this are absent

  v4i acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
  constexpr int kFill = (A_MODE == 1) ? (int)0x80808080 : 0;
  for (int kt = kt_begin; kt < kt_end; kt += U) {
    v4i a[U], b0[U], b1[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // steps past this wave's slice reload its last step and are discarded
      const int s = (kt + u < kt_end) ? kt + u : kt_end - 1;
      const int k0 = s * BK;
      const int ka = (k0 < klim) ? k0 : 0; // in bounds whatever K is
      a[u] = *(const v4i *)(ap + ka);
      if (!(row_ok && k0 < klim))
        a[u] = (v4i){kFill, kFill, kFill, kFill};
      b0[u] = *(const v4i *)(bp0 + k0);
      if (NG > 1)
        b1[u] = *(const v4i *)(bp1 + k0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (kt + u < kt_end) {
        v4i av = a[u];
        if (A_MODE == 1)
          av ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
              (int)0x80808080};
        acc0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, b0[u], acc0, 0, 0, 0);
        if (NG > 1)
          acc1 =
              __builtin_amdgcn_mfma_i32_16x16x64_i8(av, b1[u], acc1, 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    part[wave][0][r][lane] = acc0[r];
    if (NG > 1)
      part[wave][1][r][lane] = acc1[r];
  }
  __syncthreads();

  // 16x16 accumulator layout: lane holds column (lane & 15); register r holds
  // row 4*(lane/16) + r.  Thread t finishes element (g, r, lane) = t.
  const int g = tid >> 8, r = (tid >> 6) & 3;
  if (g >= NG)
    return;
  uint32_t y = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w)
    y += (uint32_t)part[w][g][r][lane];
  const int m = 4 * lq + r;
  const int n = n0 + g * 16 + l16;
  if (m >= M || n >= N)
    return;

  constexpr bool A_OFF = (A_MODE != 0);
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = ep.b_unsigned ? 128 : 0;
  int32_t da = oa, db = ob, rs = 0;
  if (ep.a_zp_len > 0)
    da = oa - load_zp_i32(ep.a_zp, A_OFF, ep.a_zp_len > 1 ? m : 0);
  if (ep.b_zp_len > 0)
    db = ob - load_zp_i32(ep.b_zp, ep.b_unsigned, ep.b_zp_len > 1 ? n : 0);
  if (ep.rowsum)
    rs = ep.rowsum[m];
  y += (uint32_t)da * (uint32_t)ep.colsum[n];
  y += (uint32_t)db * (uint32_t)rs;
  y += (uint32_t)K * (uint32_t)da * (uint32_t)db;
  float sj = 0.0f;
  int32_t yz = 0;
  if (EPI != kEpiI32) {
    sj = ep.a_scale[0] * ep.b_scale[ep.b_scale_len == 1 ? 0 : n];
    if (EPI == kEpiQ8) {
      sj = sj / ep.y_scale[0];
      yz = load_zp_i32(ep.y_zp, ep.y_unsigned, 0);
    }
  }
  store_one<EPI>(ep, (int64_t)m * N + n, y, sj, yz);
}

// ---- pack B ---------------------------------------------------------------
// One block transposes a 64(k) x 64(n) tile through LDS and adds the tile's
// column sums into colsum with int32 atomics (integer adds commute, so the
// result does not depend on arrival order).
constexpr int PT = 64;

template <bool B_UNSIGNED>
__global__ __launch_bounds__(256) void k_pack_b(const uint8_t *__restrict__ B,
    int64_t K, int64_t N, int64_t Kpad, int8_t *__restrict__ Bt,
    int32_t *__restrict__ colsum) {
  __shared__ uint8_t tile[PT][PT + 4];
  const int64_t k0 = (int64_t)blockIdx.y * PT;
  const int64_t n0 = (int64_t)blockIdx.x * PT;
  const int tid = threadIdx.x;
  // Read: thread -> row k = tid/4, 16 columns starting at (tid%4)*16.
  {
    const int kr = tid >> 2;
    const int nc = (tid & 3) * 16;
    const int64_t k = k0 + kr;
#pragma unroll
    for (int b = 0; b < 16; ++b) {
      const int64_t n = n0 + nc + b;
      uint8_t v = B_UNSIGNED ? 0x80 : 0;
      if (k < K && n < N)
        v = B[k * N + n];
      if (B_UNSIGNED)
        v ^= 0x80;
      tile[kr][nc + b] = v;
    }
  }
  __syncthreads();
  // Write: thread -> column n = tid/4, 16 k values starting at (tid%4)*16.
  {
    const int nr = tid >> 2;
    const int kc = (tid & 3) * 16;
    uint32_t w[4] = {0, 0, 0, 0};
    int32_t sum = 0;
#pragma unroll
    for (int b = 0; b < 16; ++b) {
      const uint8_t v = tile[kc + b][nr];
      sum += (int32_t)(int8_t)v;
      w[b >> 2] |= (uint32_t)v << ((b & 3) * 8);
    }
    const int64_t n = n0 + nr;
    // Bt has Npad >= gridDim.x*64 rows and Kpad >= gridDim.y*64 columns.
    *(v4i *)(Bt + n * Kpad + k0 + kc) =
        (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    // Fold the four k-chunks of this column (lanes 4n..4n+3) before the atomic.
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    if ((tid & 3) == 0 && sum != 0)
      atomicAdd(&colsum[n], sum);
  }
}

// ---- pack A ---------------------------------------------------------------
// Rewrites A [M,K] (row-major) in MFMA operand order for k_gemm_i8_stream:
//   Ap[mt][ks][sub][lane][16 bytes],  lane = half*32 + row,
//   bytes = A[mt*32 + row][ks*64 + (sub*2 + half)*16 .. +16]
// so that a wave fetches one operand (32 rows x 32 K-bytes... x 2 halves) as a
// single contiguous KiB.  uint8 is moved to int8 (minus 128) on the way and
// everything outside [M,K] is zero in that domain, which also makes K that is
// not a multiple of 64 (or 16) legal for the fast kernel.
// A block handles one 32-row tile and four K steps (256 bytes of each row):
// eight consecutive threads read 128 contiguous bytes of a row.
template <bool A_UNSIGNED, bool ALIGNED>
__global__ __launch_bounds__(256) void k_pack_a(const uint8_t *__restrict__ A,
    int64_t M, int64_t K, int KT, uint8_t *__restrict__ Ap) {
  const int mt = blockIdx.y;
  const int ks0 = blockIdx.x * 4;
  const int tid = threadIdx.x;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = tid >> 3;
    const int c16 = (tid & 7) + 8 * h; // 16-byte chunk within the 256 bytes
    const int ks = ks0 + (c16 >> 2);
    if (ks >= KT)
      continue;
    const int c = c16 & 3;
    const int64_t m = (int64_t)mt * 32 + row;
    const int64_t k = (int64_t)ks * 64 + c * 16;
    v4i v = {0, 0, 0, 0};
    if (ALIGNED) {
      if (m < M && k < K) {
        v = *(const v4i *)(A + m * K + k);
        if (A_UNSIGNED)
          v ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
              (int)0x80808080};
      }
    } else {
      uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 16; ++b) {
        uint32_t byte = 0;
        if (m < M && k + b < K) {
          byte = A[m * K + k + b];
          if (A_UNSIGNED)
            byte ^= 0x80u;
        }
        w[b >> 2] |= byte << ((b & 3) * 8);
      }
      v = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
    const int sub = c >> 1, half = c & 1;
    const int64_t o =
        ((((int64_t)mt * KT + ks) * 2 + sub) * 64 + half * 32 + row) * 16;
    *(v4i *)(Ap + o) = v;
  }
}

// rowsum[m] = sum_k A'[m,k]; one wave per row.
template <bool A_UNSIGNED>
__global__ __launch_bounds__(256) void k_rowsum_a(
    const uint8_t *__restrict__ A, int64_t M, int64_t K,
    int32_t *__restrict__ rowsum) {
  const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M)
    return;
  const int lane = threadIdx.x & 63;
  const uint8_t *__restrict__ row = A + m * K;
  int32_t sum = 0;
  for (int64_t k = lane; k < K; k += 64) {
    const uint8_t v = row[k];
    sum += A_UNSIGNED ? ((int32_t)v - 128) : (int32_t)(int8_t)v;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    sum += __shfl_xor(sum, off, 64);
  if (lane == 0)
    rowsum[m] = sum;
}

// ---- launch ---------------------------------------------------------------

template <int BM, int BN, int WGM, int WGN, int MINB, int A_MODE, int EPI>
hipError_t gemm_launch_tile(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  const int tiles_m = (int)((g.M + BM - 1) / BM);
  const int tiles_n = (int)((g.N + BN - 1) / BN);
  const dim3 grid((unsigned)(tiles_m * tiles_n));
  constexpr int threads = WGM * WGN * 64;
  k_gemm_i8<BM, BN, WGM, WGN, MINB, A_MODE, EPI, true>
      <<<grid, threads, 0, st>>>((const uint8_t *)g.A, g.Bt, (int)g.M,
          (int)g.N, (int)g.K, Kpad, ep, tiles_m, tiles_n);
  return hipGetLastError();
}

hipError_t launch_pack_a(hipStream_t st, const void *A, bool a_unsigned,
    int64_t M, int64_t K, uint8_t *Ap) {
  const int KT = (int)(round_up(K > 0 ? K : 1, kGemmBK) / kGemmBK);
  const int MT = (int)((M + 31) / 32);
  const bool aligned = (K % 16 == 0) && ((((uintptr_t)A) & 15) == 0);
  dim3 grid((unsigned)((KT + 3) / 4), (unsigned)MT);
  if (a_unsigned) {
    if (aligned)
      k_pack_a<true, true><<<grid, 256, 0, st>>>(
          (const uint8_t *)A, M, K, KT, Ap);
    else
      k_pack_a<true, false><<<grid, 256, 0, st>>>(
          (const uint8_t *)A, M, K, KT, Ap);
  } else {
    if (aligned)
      k_pack_a<false, true><<<grid, 256, 0, st>>>(
          (const uint8_t *)A, M, K, KT, Ap);
    else
      k_pack_a<false, false><<<grid, 256, 0, st>>>(
          (const uint8_t *)A, M, K, KT, Ap);
  }
  return hipGetLastError();
}

template <int TM, int TN, int D, int A_MODE, int EPI>
hipError_t gemm_launch_stream(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  constexpr int BM = 4 * 32 * TM, BN = 32 * TN;
  const int tiles_m = (int)((g.M + BM - 1) / BM);
  const int tiles_n = (int)((g.N + BN - 1) / BN);
  k_gemm_i8_stream<TM, TN, D, A_MODE, EPI>
      <<<dim3((unsigned)(tiles_m * tiles_n)), 256, 0, st>>>(g.a_pack, g.Bt,
          (int)g.M, (int)g.N, (int)g.K, Kpad, ep, tiles_m, tiles_n);
  return hipGetLastError();
}

// Kernel / tile configurations.
enum TileCfg : int {
  kT128x128 = 0, // k_gemm_i8, BM x BN
  kT256x128 = 1,
  kS256x192 = 2, // k_gemm_i8_stream (needs the packed copy of A)
  kS256x128 = 3,
  kS128x192 = 4,
  kS128x128 = 5,
  kD128x128 = 6, // k_gemm_i8_dma (tiles copied straight into LDS)
  kD128x64 = 7,
  kNumCfg = 8
};

bool cfg_is_stream(int c) {
  return c == kS256x192 || c == kS256x128 || c == kS128x192 || c == kS128x128;
}

// Tile choice.  Each configuration is costed as (rounds of tiles over the 256
// CUs) x (tile area), i.e. matrix-core time including the idle tail of the
// last round; among near-equal costs the larger tile wins (fewer LDS and L2
// bytes per MFMA).  The streamed-A kernels are only eligible when the caller
// provided the buffer for the packed copy of A.
int choose_tile(const GemmArgs &g) {
  // Override for tests and tuning: OM_MI355X_GEMM_TILE=<TileCfg value>.
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (force && force[0]) {
    const int c = atoi(force);
    if (c >= 0 && c < kNumCfg && (!cfg_is_stream(c) || g.a_pack))
      return c;
  }
  struct Cand {
    int cfg, bm, bn, per_cu;
  };
  static const Cand cands[] = {{kS256x192, 256, 192, 1}, {kS256x128, 256, 128, 1},
      {kS128x192, 128, 192, 2}, {kS128x128, 128, 128, 2}};
  // Measured on MI355X (4096 x 768 x 3072 and its siblings): the kernel that
  // copies tiles straight into LDS beats the register-staged one on every
  // shape below the streamed-A threshold, with 128 x 128 tiles even when they
  // leave some CUs without a block.
  if (!g.a_pack)
    return kD128x128;
  int best = kS128x128;
  double best_cost = 1e300;
  for (const Cand &c : cands) {
    const int64_t tiles =
        ((g.M + c.bm - 1) / c.bm) * ((g.N + c.bn - 1) / c.bn);
    const int64_t slots = 256 * c.per_cu;
    const int64_t rounds = (tiles + slots - 1) / slots;
    // two co-resident tiles share a CU's matrix cores
    double cost = (double)rounds * c.per_cu * c.bm * c.bn;
    // small tiles pay more LDS / L2 traffic per MFMA
    cost *= 1.0 + 24.0 / c.bm + 24.0 / c.bn;
    if (cost < best_cost) {
      best_cost = cost;
      best = c.cfg;
    }
  }
  return best;
}

template <int A_MODE, int EPI>
hipError_t gemm_launch_cfg(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (g.M <= 16 && g.K % 16 == 0 && ((((uintptr_t)g.A) & 15) == 0) &&
      !(force && force[0])) {
    // 32 columns per block halves the reads of A (measured faster whenever
    // that still gives every CU a block); 16 columns for narrower outputs.
    if ((g.N + 31) / 32 >= 256)
      k_gemm_i8_skinny<2, A_MODE, EPI>
          <<<dim3((unsigned)((g.N + 31) / 32)), 512, 0, st>>>(
              (const uint8_t *)g.A, g.Bt, (int)g.M, (int)g.N, (int)g.K, Kpad,
              ep);
    else
      k_gemm_i8_skinny<1, A_MODE, EPI>
          <<<dim3((unsigned)((g.N + 15) / 16)), 512, 0, st>>>(
              (const uint8_t *)g.A, g.Bt, (int)g.M, (int)g.N, (int)g.K, Kpad,
              ep);
    return hipGetLastError();
  }
  const int cfg = choose_tile(g);
  if (cfg_is_stream(cfg)) {
    // A_MODE 1 (raw uint8) is shifted to int8 by the pack; 0 and 2 are copied.
    hipError_t e = launch_pack_a(st, g.A, A_MODE == 1, g.M, g.K, g.a_pack);
    if (e != hipSuccess)
      return e;
    switch (cfg) {
    case kS256x192:
      return gemm_launch_stream<2, 6, 3, A_MODE, EPI>(st, g, ep, Kpad);
    case kS256x128:
      return gemm_launch_stream<2, 4, 3, A_MODE, EPI>(st, g, ep, Kpad);
    case kS128x192:
      return gemm_launch_stream<1, 6, 4, A_MODE, EPI>(st, g, ep, Kpad);
    default:
      return gemm_launch_stream<1, 4, 4, A_MODE, EPI>(st, g, ep, Kpad);
    }
  }
  const bool aligned = (g.K % 64 == 0) && ((((uintptr_t)g.A) & 15) == 0);
  if (!aligned) {
    // Byte-wise staging of A for odd K or a misaligned A.
    const int tiles_m = (int)((g.M + 127) / 128);
    const int tiles_n = (int)((g.N + 127) / 128);
    k_gemm_i8<128, 128, 2, 2, 2, A_MODE, EPI, false>
        <<<dim3((unsigned)(tiles_m * tiles_n)), 256, 0, st>>>(
            (const uint8_t *)g.A, g.Bt, (int)g.M, (int)g.N, (int)g.K, Kpad, ep,
            tiles_m, tiles_n);
    return hipGetLastError();
  }
  if (cfg == kD128x128 || cfg == kD128x64) {
    const int bn = (cfg == kD128x128) ? 128 : 64;
    const int tiles_m = (int)((g.M + 127) / 128);
    const int tiles_n = (int)((g.N + bn - 1) / bn);
    const dim3 grid((unsigned)(tiles_m * tiles_n));
    const uint8_t *A = (const uint8_t *)g.A;
    if (cfg == kD128x128)
      k_gemm_i8_dma<128, 3, 3, A_MODE, EPI><<<grid, 256, 0, st>>>(A, g.Bt,
          (int)g.M, (int)g.N, (int)g.K, Kpad, ep, tiles_m, tiles_n);
    else
      k_gemm_i8_dma<64, 3, 4, A_MODE, EPI><<<grid, 256, 0, st>>>(A, g.Bt,
          (int)g.M, (int)g.N, (int)g.K, Kpad, ep, tiles_m, tiles_n);
    return hipGetLastError();
  }
  if (cfg == kT256x128)
    return gemm_launch_tile<256, 128, 2, 2, 2, A_MODE, EPI>(st, g, ep, Kpad);
  return gemm_launch_tile<128, 128, 2, 2, 3, A_MODE, EPI>(st, g, ep, Kpad);
}

template <int A_MODE>
hipError_t gemm_launch_epi(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  switch (g.epi) {
  case kEpiI32:
    return gemm_launch_cfg<A_MODE, kEpiI32>(st, g, ep, Kpad);
  case kEpiF32:
    return gemm_launch_cfg<A_MODE, kEpiF32>(st, g, ep, Kpad);
  default:
    return gemm_launch_cfg<A_MODE, kEpiQ8>(st, g, ep, Kpad);
  }
}

} // namespace

hipError_t launch_pack_b(hipStream_t s, const void *B, bool b_unsigned,
    int64_t K, int64_t N, int8_t *Bt, int32_t *colsum) {
  const int64_t Kpad = round_up(K, kGemmBK);
  const int64_t Npad = round_up(N, kGemmBN);
  hipError_t e = launch_fill_u32(s, (uint32_t *)colsum, Npad, 0u);
  if (e != hipSuccess)
    return e;
  // kGemmBK and kGemmBN are multiples of the 64 x 64 pack tile, so the grid
  // covers [Npad, Kpad] exactly and every byte of Bt is written.
  dim3 grid((unsigned)(Npad / PT), (unsigned)(Kpad / PT));
  if (b_unsigned)
    k_pack_b<true><<<grid, 256, 0, s>>>(
        (const uint8_t *)B, K, N, Kpad, Bt, colsum);
  else
    k_pack_b<false><<<grid, 256, 0, s>>>(
        (const uint8_t *)B, K, N, Kpad, Bt, colsum);
  return hipGetLastError();
}

size_t gemm_a_pack_bytes(int64_t M, int64_t K, int64_t N) {
  // The packed copy pays off once there are enough rows and columns for the
  // large tiles; below that the kernels that stage A through LDS are used.
  if (M < 128 || N < 128 || K < 64)
    return 0;
  // Measured on MI355X: below ~3e10 multiply-accumulates the extra pass over A
  // and the single round of large tiles cost more than they save.
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (!(force && force[0]) && (double)M * (double)N * (double)K < 3e10)
    return 0;
  const int64_t KT = round_up(K, kGemmBK) / kGemmBK;
  const int64_t MT = (M + 31) / 32;
  return (size_t)(MT * KT * 2048);
}

hipError_t launch_rowsum_a(hipStream_t s, const void *A, bool a_unsigned,
    int64_t M, int64_t K, int32_t *rowsum) {
  if (M == 0)
    return hipSuccess;
  const unsigned grid = (unsigned)((M + 3) / 4);
  if (a_unsigned)
    k_rowsum_a<true><<<grid, 256, 0, s>>>((const uint8_t *)A, M, K, rowsum);
  else
    k_rowsum_a<false><<<grid, 256, 0, s>>>((const uint8_t *)A, M, K, rowsum);
  return hipGetLastError();
}

hipError_t launch_gemm(hipStream_t s, const GemmArgs &g) {
  if (g.M == 0 || g.N == 0)
    return hipSuccess;
  if (g.M > INT32_MAX || g.N > INT32_MAX || g.K > INT32_MAX ||
      g.M * g.N > ((int64_t)1 << 40))
    return hipErrorInvalidValue;
  const int Kpad = (int)round_up(g.K > 0 ? g.K : 1, kGemmBK);
  EpiParams ep;
  ep.a_zp = g.a_zp;
  ep.a_zp_len = g.a_zp ? g.a_zp_len : 0;
  ep.b_zp = g.b_zp;
  ep.b_zp_len = g.b_zp ? g.b_zp_len : 0;
  ep.rowsum = g.rowsum;
  ep.colsum = g.colsum;
  ep.a_scale = g.a_scale;
  ep.b_scale = g.b_scale;
  ep.b_scale_len = g.b_scale_len;
  ep.y_scale = g.y_scale;
  ep.y_zp = g.y_zp;
  ep.out = g.out;
  ep.b_unsigned = g.b_unsigned;
  ep.y_unsigned = g.y_unsigned;
  ep.narrow = (int)g.narrow;
  ep.group = 8;
  ep.xcd = 1;
  const int a_mode = g.a_preshifted ? 2 : (g.a_unsigned ? 1 : 0);
  switch (a_mode) {
  case 0:
    return gemm_launch_epi<0>(s, g, ep, Kpad);
  case 1:
    return gemm_launch_epi<1>(s, g, ep, Kpad);
  default:
    return gemm_launch_epi<2>(s, g, ep, Kpad);
  }
}


} // namespace om
