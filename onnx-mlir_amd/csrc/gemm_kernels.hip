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
// operands are read as 16 consecutive K bytes per lane.  Tiles go through LDS
// with an XOR swizzle of the 16-byte chunk index so that ds_read_b128 and
// ds_write_b128 are bank-conflict free.

#include "om_kernels.h"

namespace om {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = kGemmBN, BK = kGemmBK;
constexpr int kGemmThreads = 256;

// Byte offset of 16-byte chunk `c` (0..3) of tile row `r` (row = 64 bytes).
// Rows r, r+4, r+8, r+12 share a bank group; XOR with (r>>2)&3 spreads them.
__device__ __forceinline__ int lds_off(int r, int c) {
  return r * BK + ((c ^ ((r >> 2) & 3)) << 4);
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

// A_MODE: 0 = int8 as is, 1 = uint8 (XOR 0x80 while staging), 2 = already
// shifted (stored as u8-128) -- offsets as for uint8, no XOR.
// ALIGNED: K % 16 == 0 and A 16-byte aligned (vector loads), else byte loads.
template <int A_MODE, int EPI, bool ALIGNED>
__global__ __launch_bounds__(kGemmThreads) void k_gemm_i8(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bt, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  const bool B_UNSIGNED = ep.b_unsigned;
  const bool Y_UNSIGNED = ep.y_unsigned;
  const int NARROW = ep.narrow;
  __shared__ __attribute__((aligned(16))) uint8_t sA[2][BM * BK];
  __shared__ __attribute__((aligned(16))) uint8_t sB[2][BN * BK];

  // Tile order: consecutive blocks walk down M inside a band of N, so the
  // blocks resident at one time share a few Bt tiles and the A panel.
  const int pid = blockIdx.x;
  const int tm = pid % tiles_m;
  const int tn = pid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1; // 2 x 2 waves, 64 x 64 each

  // Staging map: thread -> (row, 16-byte chunk) twice per operand.
  const int lc = tid & 3;
  const int lr = tid >> 2; // 0..63

  v4i ra[2], rb[2];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lr + h * 64;
      const int gm = m0 + r;
      const int gk = k0 + lc * 16;
      v4i v = {0, 0, 0, 0};
      if (ALIGNED) {
        // K % 16 == 0: a chunk is either wholly inside the row or absent.
        // Absent chunks and rows >= M stay 0 in the int8 domain.
        if (gm < M && gk < K) {
          v = *(const v4i *)(A + (int64_t)gm * K + gk);
          if (A_MODE == 1)
            v ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
                (int)0x80808080};
        }
      } else {
        uint32_t w[4] = {0, 0, 0, 0};
        if (gm < M) {
#pragma unroll
          for (int b = 0; b < 16; ++b) {
            const int kk = gk + b;
            uint32_t byte = 0;
            if (kk < K) {
              byte = A[(int64_t)gm * K + kk];
              if (A_MODE == 1)
                byte ^= 0x80u;
            }
            w[b >> 2] |= byte << ((b & 3) * 8);
          }
        }
        v = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
      }
      ra[h] = v;
      // Bt is padded to [Npad, Kpad]: always in bounds and aligned.
      rb[h] = *(const v4i *)(Bt + (int64_t)(n0 + r) * Kpad + gk);
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lr + h * 64;
      *(v4i *)(&sA[buf][lds_off(r, lc)]) = ra[h];
      *(v4i *)(&sB[buf][lds_off(r, lc)]) = rb[h];
    }
  };

  v16i acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  const int kt_total = Kpad / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int l32 = lane & 31;
  const int lh = lane >> 5;

  for (int kt = 0; kt < kt_total; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < kt_total)
      load_global((kt + 1) * BK);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c = s * 2 + lh;
      v4i fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        fa[i] = *(const v4i *)(&sA[buf][lds_off(wm * 64 + i * 32 + l32, c)]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        fb[j] = *(const v4i *)(&sB[buf][lds_off(wn * 64 + j * 32 + l32, c)]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
              fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < kt_total)
      store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------
  // 32x32 accumulator layout: lane holds column (lane & 31); register r holds
  // row 8*(r/4) + 4*(lane/32) + (r%4).
  constexpr bool A_OFF = (A_MODE != 0);
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = B_UNSIGNED ? 128 : 0;
  const bool a_uns = A_OFF;

  float s_q = 0.0f;
  int32_t yz = 0;
  float a_scale = 0.0f;
  if (EPI == kEpiQ8) {
    // (a_scale * b_scale) / y_scale: two roundings, in this order
    // (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:127).
    s_q = (ep.a_scale[0] * ep.b_scale[0]) / ep.y_scale[0];
    yz = load_zp_i32(ep.y_zp, Y_UNSIGNED, 0);
  }
  if (EPI == kEpiF32)
    a_scale = ep.a_scale[0];

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + l32;
    const bool n_ok = n < N;
    int32_t db = ob, cs = 0;
    float sj = 0.0f;
    if (n_ok) {
      if (ep.b_zp_len > 0)
        db = ob - load_zp_i32(ep.b_zp, B_UNSIGNED, ep.b_zp_len == 1 ? 0 : n);
      cs = ep.colsum[n];
      if (EPI == kEpiF32)
        sj = a_scale * ep.b_scale[ep.b_scale_len == 1 ? 0 : n];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (!(n_ok && m < M))
          continue;
        int32_t da = oa;
        if (ep.a_zp_len > 0)
          da = oa - load_zp_i32(ep.a_zp, a_uns, ep.a_zp_len == 1 ? 0 : m);
        uint32_t y = (uint32_t)acc[i][j][r];
        y += (uint32_t)da * (uint32_t)cs;
        if (ep.rowsum)
          y += (uint32_t)db * (uint32_t)ep.rowsum[m];
        y += (uint32_t)K * (uint32_t)da * (uint32_t)db;
        const int64_t o = (int64_t)m * N + n;
        if (EPI == kEpiI32) {
          ((int32_t *)ep.out)[o] = (int32_t)y;
        } else if (EPI == kEpiF32) {
          ((float *)ep.out)[o] = (float)(int32_t)y * sj;
        } else {
          const float f = (float)(int32_t)y * s_q;
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

template <int A_MODE, int EPI>
hipError_t gemm_launch_aligned(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int Kpad, int tiles_m, int tiles_n) {
  const bool aligned = (g.K % 16 == 0) && ((((uintptr_t)g.A) & 15) == 0);
  const dim3 grid((unsigned)(tiles_m * tiles_n));
  if (aligned)
    k_gemm_i8<A_MODE, EPI, true><<<grid, kGemmThreads, 0, st>>>(
        (const uint8_t *)g.A, g.Bt, (int)g.M, (int)g.N, (int)g.K, Kpad, ep,
        tiles_m, tiles_n);
  else
    k_gemm_i8<A_MODE, EPI, false><<<grid, kGemmThreads, 0, st>>>(
        (const uint8_t *)g.A, g.Bt, (int)g.M, (int)g.N, (int)g.K, Kpad, ep,
        tiles_m, tiles_n);
  return hipGetLastError();
}

template <int A_MODE>
hipError_t gemm_launch_epi(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int Kpad, int tiles_m, int tiles_n) {
  switch (g.epi) {
  case kEpiI32:
    return gemm_launch_aligned<A_MODE, kEpiI32>(
        st, g, ep, Kpad, tiles_m, tiles_n);
  case kEpiF32:
    return gemm_launch_aligned<A_MODE, kEpiF32>(
        st, g, ep, Kpad, tiles_m, tiles_n);
  default:
    return gemm_launch_aligned<A_MODE, kEpiQ8>(
        st, g, ep, Kpad, tiles_m, tiles_n);
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
  const int tiles_m = (int)((g.M + BM - 1) / BM);
  const int tiles_n = (int)((g.N + BN - 1) / BN);
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
    return gemm_launch_epi<0>(s, g, ep, Kpad, tiles_m, tiles_n);
  case 1:
    return gemm_launch_epi<1>(s, g, ep, Kpad, tiles_m, tiles_n);
  default:
    return gemm_launch_epi<2>(s, g, ep, Kpad, tiles_m, tiles_n);
  }
}

} // namespace om
