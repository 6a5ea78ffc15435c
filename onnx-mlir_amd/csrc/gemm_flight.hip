// int8 GEMM for gfx950 for problems that one round of blocks covers
// (k_gemm_i8_flight): everything a block needs is requested at once.
//
// A small product -- a [128, 768] activation against [768, 768] weights, a
// 512 x 1024 x 4096 QLinearMatMul -- is one tile per CU and a dozen K steps.
// A pipelined K loop that keeps two or three steps in flight then pays the
// memory latency once per step or two (16 steps of ~0.35 us on top of the
// launch: 8 us for work that the matrix cores do in under one).  Here a block
// asks for all of its operands before it waits for any of them: the weights of
// a wave's 32 columns for all of K go straight into registers (Bp is stored in
// that order, see gemm_kernels.hip), the block's rows of A for all of K are
// copied into LDS without passing through registers, and the K loop that
// follows touches LDS and registers only.  K is limited by the registers (K <=
// 1024: 128 per lane for the weights) and must be a multiple of 256.
//
// DQ: the whole dynamically quantized layer in one launch
// (DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul,
// src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:86-158 and
// src/Conversion/ONNXToKrnl/Math/MatMulInteger.cpp:59-90).  The activation
// arrives as f32 X[M,K].  A block loads its 32 rows into registers; the
// blocks of a row region split those rows between them for the minimum and
// maximum (a block reduces the K columns c with (c / 32) % G == its share),
// publish them in the tagged slots that DynamicQuantizeLinear's one-launch
// kernel uses, read everybody's, derive scale and zero point (every block the
// same), quantize their rows into LDS and multiply.  No block reads more of X
// than the rows it multiplies, and the weights arrive while the blocks wait
// for one another.
//
// A in LDS: [row tile of 32][K group of 256 bytes][row][256 bytes]; within a
// row's 256 bytes the 16-byte chunk c sits at position c ^ (row % 16), so the
// lanes of an operand read (rows 0..31, the same chunk of each) fall into
// different banks, and a copy instruction (1 KiB of consecutive LDS) is four
// rows of one K group: 256 contiguous bytes of each row of A.

#include "gemm_common.h"
#include "gemm_epilogue.h"

namespace om {
namespace gemm {

namespace {

constexpr int kFlightKH = 32;   // K steps of 32 bytes a wave's registers hold
constexpr int kFlightWaves = 4; // column tiles (of 32) per block
constexpr int kFlightGroup = 8; // operand reads issued together

struct FlightDq {
  const float *X;            // [M, K] f32
  unsigned long long *slots; // tagged (launch number, value) slots
  unsigned epoch;
  unsigned *failed;
  unsigned spin_limit;
  int share_groups; // G: blocks of a row region that split its min / max
  int col_blocks;   // blocks per row region
};

// KG: K / 256 (a template argument: every loop over K is unrolled and has no
// branch).  nr: row tiles of 32 per block; the block's LDS, nr * KG * 8 KiB, is
// sized at launch.
template <int KG, bool A_OFF, bool DQ, int EPI>
__global__ __launch_bounds__(kFlightWaves * 64, 1) void k_gemm_i8_flight(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
    EpiParams ep, uint32_t flip, int nr, int regions_n, int bp_tiles,
    FlightDq dq) {
  constexpr int WAVES = kFlightWaves, KH = 8 * KG, K = 256 * KG, G8 = kFlightGroup;
  constexpr int KHMAX = KH;
  static_assert(KH <= kFlightKH, "registers");
  static_assert(!DQ || (A_OFF && EPI == kEpiF32), "fused layer");
  extern __shared__ __attribute__((aligned(1024))) uint8_t sA[];
  const int ROWS = 32 * nr;
  __shared__ float s_lo[WAVES], s_hi[WAVES];
  __shared__ int s_ok;
  __shared__ float s_scale;
  __shared__ __attribute__((aligned(4))) uint8_t s_zp[4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int rm = blockIdx.x / regions_n, rn = blockIdx.x % regions_n;
  const int row0 = rm * ROWS;
  const int ct = rn * WAVES + wave; // the wave's column tile

  typedef __attribute__((address_space(3))) void *lds_ptr;
  typedef const __attribute__((address_space(1))) void *glb_ptr;

  // ---- everything is requested here ----------------------------------------
  typedef float f4 __attribute__((ext_vector_type(4)));
  f4 x[DQ ? KHMAX : 1];
  if (DQ) {
    // Thread (row r = tid / 8, position p = tid % 8) takes float4 p + 8 j of
    // its row, j < K / 32: a wave instruction reads 8 rows x 128 bytes, whole
    // cache lines.  Register slot i holds j = ((i / S + share) % G) + G * (i % S)
    // with S = (K / 32) / G, so that slots 0 .. S-1 are the block's own share
    // of the minimum / maximum and arrive first.
    const int r = tid >> 3;
    const int row = row0 + r < M ? row0 + r : M - 1;
    const f4 *__restrict__ xr = (const f4 *)(dq.X + (int64_t)row * K) + (tid & 7);
    const int G = dq.share_groups, S = KH / G;
    int a = 0, b = 0; // i / S, i % S
#pragma unroll
    for (int i = 0; i < KHMAX; ++i) {
      int g = a + (rn % G);
      g = g >= G ? g - G : g;
      x[i] = xr[8 * (g + G * b)];
      if (++b == S) {
        b = 0;
        ++a;
      }
    }
  } else {
    // A copy instruction fills 1 KiB of consecutive LDS, 16 bytes per lane:
    // rows 4 q .. 4 q + 3 (q < 8) of K group cg of row tile t.  Lane l is
    // position l % 16 of row 4 q + l / 16 and fetches the chunk that belongs
    // there.  Wave w issues q = w and w + 4 of every (t, cg).  Rows past M
    // are copies of the last row and are never stored.
    const int rl = lane >> 4;
#pragma unroll 1
    for (int t = 0; t < nr; ++t) {
#pragma unroll
      for (int cg = 0; cg < KG; ++cg) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int q = wave + 4 * h;
          const int r = 4 * q + rl; // row within the tile
          const int c = (lane & 15) ^ (r & 15);
          int row = row0 + 32 * t + r;
          row = row < M ? row : M - 1;
          __builtin_amdgcn_global_load_lds(
              (glb_ptr)(A + (int64_t)row * K + cg * 256 + c * 16),
              (lds_ptr)(sA + ((t * KG + cg) * 8 + q) * 1024), 16, 0, 0);
        }
      }
    }
  }
  v4i b[KHMAX];
  {
    // column tiles past the packed weights (the last region of a ragged N)
    // read the last tile and are not stored
    const int ctc = ct < bp_tiles ? ct : bp_tiles - 1;
    const int8_t *const bp = Bp + (int64_t)ctc * KH * 1024 + lane * 16;
#pragma unroll
    for (int s = 0; s < KH; ++s)
      b[s] = *(const v4i *)(bp + s * 1024);
  }

  if (DQ) {
    // ---- minimum / maximum of the block's share, exchange, quantize ---------
    const int G = dq.share_groups, S = KH / G;
    const bool row_in = row0 + (tid >> 3) < M;
    float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < KHMAX; ++i) {
      if (i < S) {
        lo = __builtin_fminf(lo, __builtin_fminf(__builtin_fminf(x[i].x, x[i].y),
                                     __builtin_fminf(x[i].z, x[i].w)));
        hi = __builtin_fmaxf(hi, __builtin_fmaxf(__builtin_fmaxf(x[i].x, x[i].y),
                                     __builtin_fmaxf(x[i].z, x[i].w)));
      }
    }
    if (!row_in) { // a copy of the last row: in another block's share already
      lo = __builtin_inff();
      hi = -__builtin_inff();
    }
    lo = wave_min(lo);
    hi = wave_max(hi);
    if (lane == 0) {
      s_lo[wave] = lo;
      s_hi[wave] = hi;
    }
    if (tid == 0)
      s_ok = 1;
    __syncthreads();
    // Publishers: the first G blocks of every row region (with G == 1 every
    // block of the region holds the same values and the first one publishes).
    const int nslots = (int)(gridDim.x / dq.col_blocks) * G;
    if (tid == 0 && rn < G) {
      float bl = s_lo[0], bh = s_hi[0];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        bl = __builtin_fminf(bl, s_lo[w]);
        bh = __builtin_fmaxf(bh, s_hi[w]);
      }
      const unsigned long long tag = (unsigned long long)dq.epoch << 32;
      const int slot = rm * G + rn;
      __hip_atomic_store(&dq.slots[2 * slot], tag | __float_as_uint(bl),
          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&dq.slots[2 * slot + 1], tag | __float_as_uint(bh),
          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    // Everybody's: one slot per thread (nslots <= 256), polled until both
    // words carry this launch's number; bounded (see k_dql_grid).
    typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
    bool ok = true;
    lo = __builtin_inff();
    hi = -__builtin_inff();
    if (tid < nslots) {
      u64x2 w = {0, 0};
      bool got = false;
      for (unsigned spin = 0; spin < dq.spin_limit; ++spin) {
        asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=v"(w)
                     : "v"(&dq.slots[2 * tid])
                     : "memory");
        if ((unsigned)(w.x >> 32) == dq.epoch && (unsigned)(w.y >> 32) == dq.epoch) {
          got = true;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
      ok = got;
      lo = __uint_as_float((unsigned)w.x);
      hi = __uint_as_float((unsigned)w.y);
    }
    lo = wave_min(lo);
    hi = wave_max(hi);
    const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
    if (lane == 0) {
      s_lo[wave] = lo;
      s_hi[wave] = hi;
      if (!all_ok)
        s_ok = 0;
    }
    __syncthreads();
    if (!s_ok) {
      if (tid == 0)
        __hip_atomic_store(
            dq.failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    lo = s_lo[0];
    hi = s_hi[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      lo = __builtin_fminf(lo, s_lo[w]);
      hi = __builtin_fmaxf(hi, s_hi[w]);
    }
    float scale, zpf;
    dynamic_params(lo, hi, scale, zpf);
    if (tid == 0) {
      s_scale = scale;
      s_zp[0] = (uint8_t)(uint32_t)zpf;
    }
    // The 8-bit rows, minus 128, into LDS at the operand layout's positions.
    const float recip = 1.0f / scale;
    const int r = tid >> 3;
    const int p = tid & 7;
    uint8_t *const rowp = sA + r * 256 + (p & 3) * 4;
    auto quantize = [&](auto fast_c) {
      constexpr int FAST = decltype(fast_c)::value ? 1 : 0;
      int a = 0, bq = 0;
#pragma unroll
      for (int i = 0; i < KHMAX; ++i) {
        int g = a + (rn % G);
        g = g >= G ? g - G : g;
        const int j = g + G * bq;
        // float4 p + 8 j of the row: K group j / 8, chunk 2 (j % 8) + p / 4
        const int c = 2 * (j & 7) + (p >> 2);
        const uint32_t q = quant_pack4<false, true, FAST>(x[i].x, x[i].y,
            x[i].z, x[i].w, scale, scale, scale, scale, recip, recip, recip,
            recip, zpf, zpf, zpf, zpf);
        *(uint32_t *)(rowp + (j >> 3) * 8192 + ((c ^ (r & 15)) << 4)) =
            q ^ 0x80808080u;
        if (++bq == S) {
          bq = 0;
          ++a;
        }
      }
    };
    if (scale_is_tame(scale)) // the same for every thread
      quantize(std::true_type{});
    else
      quantize(std::false_type{});
    __syncthreads();
  } else {
    __builtin_amdgcn_s_waitcnt(0x0F70); // this wave's copies have landed
    __builtin_amdgcn_s_barrier();
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop: LDS and registers only -----------------------------------------
  // Lane (row l32, half lh) takes chunk 2 s + lh of its row in step s.  With
  // s = 8 g + v that is chunk 2 v + lh of K group g, at byte
  // 8192 g + 256 l32 + ((32 v + 16 lh) ^ (16 (l32 % 16))) of the row tile:
  // eight lane addresses, one per v, and an immediate per g.
  unsigned aaddr[8];
  {
    const unsigned arow = (unsigned)(uintptr_t)(lds_ptr)sA + l32 * 256;
    const unsigned xh = (unsigned)((16 * lh) ^ (16 * (l32 & 15)));
#pragma unroll
    for (int v = 0; v < 8; ++v)
      aaddr[v] = arow + ((unsigned)(32 * v) ^ xh);
  }
  const v4i flip4 = {(int)flip, (int)flip, (int)flip, (int)flip};
  const bool need_rs = ep.need_rowsum;
  EpiParams epl = ep;
  if (DQ) {
    epl.a_scale = &s_scale;
    epl.a_zp = s_zp;
    epl.a_zp_len = 1;
  }
#pragma unroll 1
  for (int t = 0; t < nr; ++t) {
    v16i acc[1][1];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      acc[0][0][r] = 0;
    int32_t rsp[1] = {0};
    v4i fa[2][G8];
    auto read_group = [&](auto gc) { // the reads of steps 8 g .. 8 g + 7
      constexpr int g = decltype(gc)::value;
      static_for<G8>([&](auto vc) {
        constexpr int v = decltype(vc)::value;
        v4i &f = fa[g & 1][v];
        const unsigned addr = aaddr[v];
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(f)
                     : "v"(addr), "n"(8192 * g)
                     : "memory");
      });
    };
    read_group(std::integral_constant<int, 0>{});
    static_for<KG>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      constexpr bool more = g + 1 < KG;
      if constexpr (more)
        read_group(std::integral_constant<int, g + 1>{});
      static_for<G8>([&](auto vc) {
        constexpr int v = decltype(vc)::value;
        v4i &f = fa[g & 1][v];
        // reads complete in order: this one has landed when at most the
        // later ones of its group, and the next group's, are outstanding
        asm volatile("s_waitcnt lgkmcnt(%1)"
                     : "+v"(f)
                     : "n"(G8 - 1 - v + (more ? G8 : 0))
                     : "memory");
        const v4i av = f ^ flip4;
        if (need_rs)
          rsp[0] += frag_rowsum(av);
        acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            av, b[g * G8 + v], acc[0][0], 0, 0, 0);
      });
    });
    gemm_epilogue<1, 1, A_OFF ? 2 : 0, EPI, kAuxThrough>(
        acc, rsp, row0 + 32 * t, ct * 32, M, N, K, epl);
#pragma unroll
    for (int v = 0; v < 8; ++v)
      aaddr[v] += KG * 8192;
  }
}

// A block's LDS beyond the default limit has to be asked for, once per kernel.
template <typename Kern>
hipError_t flight_allow_lds(Kern kern) {
  static const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
      hipFuncAttributeMaxDynamicSharedMemorySize, 4 * kFlightKH * 32 * 32);
  return e;
}

template <int KG, bool A_OFF, int EPI>
hipError_t flight_launch(hipStream_t st, const GemmArgs &g, const EpiParams &ep,
    uint32_t flip, int nr) {
  const int ntiles = (int)((g.N + 31) / 32);
  const int regions_n = (ntiles + kFlightWaves - 1) / kFlightWaves;
  const int regions_m = (int)((g.M + 32 * nr - 1) / (32 * nr));
  const int bp_tiles = (int)(round_up(g.N, kGemmBN) / 32);
  const FlightDq none = {};
  auto kern = k_gemm_i8_flight<KG, A_OFF, false, EPI>;
  hipError_t e = flight_allow_lds(kern);
  if (e != hipSuccess)
    return e;
  kern<<<dim3((unsigned)(regions_m * regions_n)), dim3(kFlightWaves * 64),
      (size_t)nr * KG * 8192, st>>>((const uint8_t *)g.A, g.Bp, (int)g.M,
      (int)g.N, ep, flip, nr, regions_n, bp_tiles, none);
  return hipGetLastError();
}

template <bool A_OFF, int EPI>
hipError_t flight_launch_kg(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, uint32_t flip, int nr) {
  switch (g.K / 256) {
  case 2:
    return flight_launch<2, A_OFF, EPI>(st, g, ep, flip, nr);
  case 3:
    return flight_launch<3, A_OFF, EPI>(st, g, ep, flip, nr);
  case 4:
    return flight_launch<4, A_OFF, EPI>(st, g, ep, flip, nr);
  default:
    return hipErrorInvalidValue;
  }
}

template <int KG>
hipError_t flight_launch_dq(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int regions_m, int regions_n, int bp_tiles,
    const FlightDq &dq) {
  auto kern = k_gemm_i8_flight<KG, true, true, kEpiF32>;
  hipError_t e = flight_allow_lds(kern);
  if (e != hipSuccess)
    return e;
  kern<<<dim3((unsigned)(regions_m * regions_n)), dim3(kFlightWaves * 64),
      (size_t)KG * 8192, st>>>(nullptr, g.Bp, (int)g.M, (int)g.N, ep, 0u, 1,
      regions_n, bp_tiles, dq);
  return hipGetLastError();
}

int flight_cus() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess)
      return 0;
    return n;
  }();
  return cus;
}

bool flight_k_ok(int64_t K) { return K >= 512 && K <= 32 * kFlightKH && K % 256 == 0; }

} // namespace

// Row tiles per block for this problem: the fewest with which one round of
// blocks (one block per CU) covers it; 0 if the kernel does not take it.
int flight_row_tiles(const GemmArgs &g) {
  if (!flight_k_ok(g.K) || g.M < 1 || g.X || ((((uintptr_t)g.A) & 15) != 0))
    return 0;
  const int64_t regions_n = ((g.N + 31) / 32 + kFlightWaves - 1) / kFlightWaves;
  const int cus = flight_cus();
  for (int nr = 1; nr <= 4; nr *= 2)
    if (((g.M + 32 * nr - 1) / (32 * nr)) * regions_n <= cus)
      return nr;
  return 0;
}

hipError_t launch_gemm_flight(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode) {
  const int nr = flight_row_tiles(g);
  if (nr == 0)
    return hipErrorInvalidValue;
  const uint32_t flip = a_mode == 1 ? 0x80808080u : 0u;
  if (a_mode == 0) {
    switch (g.epi) {
    case kEpiI32:
      return flight_launch_kg<false, kEpiI32>(st, g, ep, flip, nr);
    case kEpiF32:
      return flight_launch_kg<false, kEpiF32>(st, g, ep, flip, nr);
    default:
      return flight_launch_kg<false, kEpiQ8>(st, g, ep, flip, nr);
    }
  }
  switch (g.epi) {
  case kEpiI32:
    return flight_launch_kg<true, kEpiI32>(st, g, ep, flip, nr);
  case kEpiF32:
    return flight_launch_kg<true, kEpiF32>(st, g, ep, flip, nr);
  default:
    return flight_launch_kg<true, kEpiQ8>(st, g, ep, flip, nr);
  }
}

// The fused layer in one launch: 32 rows per block, and every block of the
// grid resident at once (they wait for one another).
bool flight_quantizes_rows(int64_t M, int64_t K, int64_t N, const void *x) {
  if (!flight_k_ok(K) || M < 1 || ((((uintptr_t)x) & 15) != 0))
    return false;
  const int64_t regions_n = ((N + 31) / 32 + kFlightWaves - 1) / kFlightWaves;
  const int cus = flight_cus();
  return ((M + 31) / 32) * regions_n <= (cus < 256 ? cus : 256);
}

hipError_t launch_gemm_flight_dq(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, DqlScratch &scratch) {
  if (!g.X || g.epi != kEpiF32 || !flight_quantizes_rows(g.M, g.K, g.N, g.X))
    return hipErrorInvalidValue;
  const int ntiles = (int)((g.N + 31) / 32);
  const int regions_n = (ntiles + kFlightWaves - 1) / kFlightWaves;
  const int regions_m = (int)((g.M + 31) / 32);
  const int bp_tiles = (int)(round_up(g.N, kGemmBN) / 32);
  if (2 * regions_m * regions_n > 2 * scratch.max_blocks)
    return hipErrorInvalidValue;
  FlightDq dq = {};
  dq.X = g.X;
  dq.col_blocks = regions_n;
  // the largest number of blocks of a row region, a divisor of the K steps,
  // that can share the region's minimum / maximum between them
  const int KH = (int)(g.K / 32);
  dq.share_groups = 1;
  for (int d = 1; d <= regions_n && d <= KH; ++d)
    if (KH % d == 0)
      dq.share_groups = d;
  GridExchange ex;
  if (!dql_exchange_begin(st, scratch, ex))
    return hipErrorNotReady; // another stream's exchange may be running
  dq.slots = ex.slots;
  dq.epoch = ex.epoch;
  dq.failed = ex.failed;
  dq.spin_limit = ex.spin_limit;
  hipError_t e;
  switch (g.K / 256) {
  case 2:
    e = flight_launch_dq<2>(st, g, ep, regions_m, regions_n, bp_tiles, dq);
    break;
  case 3:
    e = flight_launch_dq<3>(st, g, ep, regions_m, regions_n, bp_tiles, dq);
    break;
  default:
    e = flight_launch_dq<4>(st, g, ep, regions_m, regions_n, bp_tiles, dq);
    break;
  }
  dql_exchange_end(st, e == hipSuccess);
  return e;
}

} // namespace gemm
} // namespace om
