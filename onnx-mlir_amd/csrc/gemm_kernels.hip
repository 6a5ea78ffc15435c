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
// Pipeline: a block owns a BM x BN tile of Y and walks K in steps of 64 bytes.
// Global loads run two steps ahead of the MFMAs in registers (two register
// sets), LDS is double buffered, and the block barrier only orders LDS traffic
// so the global loads stay in flight across it.  LDS rows are 64 bytes; the
// 16-byte chunk index is XOR-swizzled with bits 2..3 of the row so that both
// ds_write_b128 (staging) and ds_read_b128 (MFMA operands) are bank-conflict
// free.

#include "om_kernels.h"

#include <stdlib.h>

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
};

__device__ __forceinline__ int32_t load_zp_i32(
    const void *p, bool is_unsigned, int64_t i) {
  return is_unsigned ? (int32_t)((const uint8_t *)p)[i]
                     : (int32_t)((const int8_t *)p)[i];
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
  const int wave = tid >> 6;
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
#if defined(OM_EXP) && (OM_EXP & 2)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j][0] += fa[i].x ^ fb[j].y;
#else
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
              fa[i], fb[j], acc[i][j], 0, 0, 0);
#endif
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
#if !(defined(OM_EXP) && (OM_EXP & 1))
    load_global(kclamp(kt + 3), ra1, rb1);
#endif
    lds_barrier();
    if (++kt >= KT)
      break;
    compute(1);
    __builtin_amdgcn_sched_barrier(0);
    store_lds(0, ra0, rb0);
#if !(defined(OM_EXP) && (OM_EXP & 1))
    load_global(kclamp(kt + 3), ra0, rb0);
#endif
    lds_barrier();
    if (++kt >= KT)
      break;
  }

  // ---- epilogue ----------------------------------------------------------
  // 32x32 accumulator layout: lane holds column (lane & 31); register r holds
  // row 8*(r/4) + 4*(lane/32) + (r%4).
  const bool B_UNSIGNED = ep.b_unsigned;
  const bool Y_UNSIGNED = ep.y_unsigned;
  const int NARROW = ep.narrow;
  constexpr bool A_OFF = (A_MODE != 0);
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = B_UNSIGNED ? 128 : 0;
  const bool a_uns = A_OFF;

  int32_t yz = 0;
  float a_scale = 0.0f;
  if (EPI == kEpiQ8)
    yz = load_zp_i32(ep.y_zp, Y_UNSIGNED, 0);
  if (EPI == kEpiF32)
    a_scale = ep.a_scale[0];

  // Everything the epilogue reads is loaded into registers before the first
  // store: a load placed after a store to possibly aliasing memory would have
  // to wait for it.
  int n_[TN];
  bool n_ok[TN];
  int32_t db[TN], cs[TN];
  float sj[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    n_[j] = n0 + wn * WTN + j * 32 + l32;
    n_ok[j] = n_[j] < N;
    db[j] = ob;
    cs[j] = 0;
    sj[j] = 0.0f;
    if (n_ok[j]) {
      if (ep.b_zp_len > 0)
        db[j] = ob - load_zp_i32(
                         ep.b_zp, B_UNSIGNED, ep.b_zp_len == 1 ? 0 : n_[j]);
      cs[j] = ep.colsum[n_[j]];
      // a_scale * b_scale[j] first, then one multiply per element; for the
      // requantize (a_scale * b_scale) / y_scale, in this order
      // (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:127).
      if (EPI == kEpiF32)
        sj[j] = a_scale * ep.b_scale[ep.b_scale_len == 1 ? 0 : n_[j]];
      if (EPI == kEpiQ8)
        sj[j] = (ep.a_scale[0] * ep.b_scale[ep.b_scale_len == 1 ? 0 : n_[j]]) /
                ep.y_scale[0];
    }
  }
  const int32_t az0 = ep.a_zp_len > 0 ? load_zp_i32(ep.a_zp, a_uns, 0) : 0;
  const bool per_row = ep.a_zp_len > 1;
  const bool has_rs = ep.rowsum != nullptr;

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int mbase = m0 + wm * WTM + i * 32 + 4 * lh;
    int32_t da[16], rs[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = mbase + 8 * (r >> 2) + (r & 3);
      da[r] = oa - az0;
      rs[r] = 0;
      if (m < M) {
        if (per_row)
          da[r] = oa - load_zp_i32(ep.a_zp, a_uns, m);
        if (has_rs)
          rs[r] = ep.rowsum[m];
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mbase + 8 * (r >> 2) + (r & 3);
        if (!(n_ok[j] && m < M))
          continue;
        uint32_t y = (uint32_t)acc[i][j][r];
        y += (uint32_t)da[r] * (uint32_t)cs[j];
        y += (uint32_t)db[j] * (uint32_t)rs[r];
        y += (uint32_t)K * (uint32_t)da[r] * (uint32_t)db[j];
        const int64_t o = (int64_t)m * N + n_[j];
        if (EPI == kEpiI32) {
          ((int32_t *)ep.out)[o] = (int32_t)y;
        } else if (EPI == kEpiF32) {
          ((float *)ep.out)[o] = (float)(int32_t)y * sj[j];
        } else {
          const float f = (float)(int32_t)y * sj[j];
          const int32_t q = (int32_t)__builtin_rintf(f);
          int32_t v = (int32_t)((uint32_t)q + (uint32_t)yz);
          if (NARROW == kSaturate) {
            if (Y_UNSIGNED)
              v = v < 0 ? 0 : (v > 255 ? 255 : v);
            else
              v = v < -128 ? -128 : (v > 127 ? 127 : v);
          }
          ((uint8_t *)ep.out)[o] = (uint8_t)(v & 0xFF);
        }
      }
    }
  }
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
enum TileCfg : int { kT128x128 = 0, kT256x128 = 1, kT256x256 = 2 };

template <int BM, int BN, int WGM, int WGN, int MINB, int A_MODE, int EPI>
hipError_t gemm_launch_tile(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  const int tiles_m = (int)((g.M + BM - 1) / BM);
  const int tiles_n = (int)((g.N + BN - 1) / BN);
  const dim3 grid((unsigned)(tiles_m * tiles_n));
  constexpr int threads = WGM * WGN * 64;
  static const char *pad_env = getenv("OM_MI355X_GEMM_LDS_PAD");
  const size_t pad = pad_env ? (size_t)atoi(pad_env) : 0;
  k_gemm_i8<BM, BN, WGM, WGN, MINB, A_MODE, EPI, true>
      <<<grid, threads, pad, st>>>((const uint8_t *)g.A, g.Bt, (int)g.M,
          (int)g.N, (int)g.K, Kpad, ep, tiles_m, tiles_n);
  return hipGetLastError();
}

// Tile choice.  Small-K or small problems want many small tiles (several
// resident per CU hide each other's latency and store phases); large problems
// want the big tiles' higher MFMA-per-LDS-byte ratio.
int choose_tile(const GemmArgs &g) {
  static const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (force && force[0] >= '0' && force[0] <= '2')
    return force[0] - '0';
  const int64_t t128 = ((g.M + 127) / 128) * ((g.N + 127) / 128);
  if (t128 < 3 * 256 || g.K < 1024)
    return kT128x128;
  return kT256x128;
}

template <int A_MODE, int EPI>
hipError_t gemm_launch_cfg(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
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
  switch (choose_tile(g)) {
  case kT256x256:
    return gemm_launch_tile<256, 256, 2, 4, 1, A_MODE, EPI>(st, g, ep, Kpad);
  case kT256x128:
    return gemm_launch_tile<256, 128, 2, 2, 2, A_MODE, EPI>(st, g, ep, Kpad);
  default:
    return gemm_launch_tile<128, 128, 2, 2, 3, A_MODE, EPI>(st, g, ep, Kpad);
  }
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
