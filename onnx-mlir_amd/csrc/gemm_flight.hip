// int8 GEMM for gfx950 for problems that one round of blocks covers
// (k_gemm_i8_flight, k_gemm_i8_flight_dq): everything a block needs is
// requested at once.
//
// A small product -- a [128, 768] activation against [768, 768] weights, a
// 512 x 1024 x 4096 QLinearMatMul -- is at most one tile per CU and a dozen K
// steps.  A pipelined K loop that keeps two or three steps in flight pays the
// memory latency once per step or two (16 steps of ~0.35 us on top of the
// launch: 8 us for work that the matrix cores do in under one).  Here a block
// asks for all of its operands before it waits for any of them: the weights of
// a wave's 32 columns for all of K go straight into registers (Bp is stored in
// that order, see gemm_kernels.hip), the block's rows of A for all of K pass
// through registers into LDS (uint8 becomes int8 on the way), and the K loop
// that follows touches LDS and registers only.  K is limited by the registers
// (K <= 1024: 128 per lane for the weights) and must be a multiple of 256.
//
// What bounds such a launch is the path into the CU: it takes in about 64
// bytes per clock (130 B/ns), and a load instruction is not issued before the
// ones in front of it have been through.  512 x 1024 x 4096 on 256 CUs is
// 192 KB per CU however it is tiled -- 1.45 us -- so the launcher picks, among
// the block shapes that cover the problem in one round, the one with the
// fewest bytes per block.
//
// What the compiler must see, and not see (each of these was a measured
// microsecond):
//  - every load is an ordinary one in program order; the compiler then puts
//    a wait for exactly the loads up to the one used in front of each use.
//    Loads it cannot count (inline asm) make it wait for everything at the
//    first use of anything, and their destination registers are not safe.
//  - no flat load (a pointer that went through an integer): while one is
//    outstanding every wait is for all loads;
//  - a value loaded from an address that is the same in all lanes is moved
//    to a scalar register right behind the load, which waits for it: such
//    loads index with an opaque zero;
//  - byte loads are widened right behind the load: zero points are loaded as
//    the aligned word that holds them;
//  - barriers are s_barrier behind a wait for LDS only (lds_sync): a
//    workgroup fence waits for the global loads in flight as well;
//  - branches that only some waves take, with loads in them, merge into a
//    wait for the shortest count: the multiplying and the polling waves of
//    the fused kernel run the rest of the kernel in separate branches.
// One wave per SIMD: vector instructions are not hidden behind anything, a
// wave issues about one per four clocks, so their number is what a phase
// costs; between two MFMAs each costs its issue time on top (a wait
// instruction about eight clocks).
//
// k_gemm_i8_flight_dq: the whole dynamically quantized layer in one launch
// (DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul,
// src/Conversion/ONNXToKrnl/Quantization/DynamicQuantizeLinear.cpp:86-158 and
// src/Conversion/ONNXToKrnl/Math/MatMulInteger.cpp:59-90).  The activation
// arrives as f32 X[M,K].  A block of eight waves owns 8, 16 or 32 rows and up
// to 128 columns.  All of its rows are requested at once, its share of them
// first (the blocks of a row region split the region's columns between them);
// it reduces the share and publishes minimum and maximum in the tagged slots
// that DynamicQuantizeLinear's one-launch kernel uses; then it requests its
// weights, which arrive while the blocks wait for one another; then every
// block reads all slots, derives scale and zero point (every block the same),
// quantizes its rows into LDS and multiplies.  No block reads more of X than
// the rows it multiplies.
//
// A in LDS: [row tile of 32][K group of 256 bytes][row][256 bytes]; within a
// row's 256 bytes the 16-byte chunk c sits at position c ^ (row % 16), so the
// lanes of an operand read (rows 0..31, the same chunk of each) fall into
// different banks, and a staging store (1 KiB of consecutive LDS) is four
// rows of one K group: 256 contiguous bytes of each row of A.

#include "gemm_common.h"
#include "gemm_epilogue.h"

namespace om {
namespace gemm {

namespace {

#ifdef FLIGHT_TIMING
// Measurement build (measure/flight_timeline.py): wave 0 of every block reads
// the 100 MHz clock at fixed points, slots 0..7, and the cycle counter on entry
// and at the end, slots 10 and 11; written out when the kernel ends
// (om_dev_flight_ts reads them).
constexpr int kFlightTsSlots = 12;
__device__ unsigned long long flight_ts[1024 * kFlightTsSlots];
#define FLIGHT_TS(i)                                                           \
  if (wave == 0)                                                               \
  ts[i] = __builtin_amdgcn_s_memrealtime()
#define FLIGHT_TS_DECL                                                         \
  unsigned long long ts[kFlightTsSlots] = {};                                  \
  ts[10] = __builtin_readcyclecounter()
#define FLIGHT_TS_WRITE                                                        \
  ts[11] = __builtin_readcyclecounter();                                       \
  if (wave == 0 && lane == 0 && blockIdx.x < 1024)                             \
    for (int i_ = 0; i_ < kFlightTsSlots; ++i_)                                \
  flight_ts[blockIdx.x * kFlightTsSlots + i_] = ts[i_]
#else
#define FLIGHT_TS(i)
#define FLIGHT_TS_DECL
#define FLIGHT_TS_WRITE
#endif

constexpr int kFlightMaxKG = 4;  // K / 256 at most: 128 registers of weights
constexpr int kFlightMaxTiles = 2;

typedef __attribute__((address_space(3))) void *lds_ptr;
typedef const __attribute__((address_space(1))) void *glb_ptr;

// Block-wide barrier that orders LDS accesses and nothing else: this wave's LDS
// operations have completed, and memory operations on global memory (loads
// still arriving, copies into LDS of later pieces, stores on their way out)
// keep flying across it.  (A workgroup fence, even one restricted to LDS, makes
// the compiler wait for every outstanding vector memory operation as soon as
// the kernel contains copies from global memory into LDS.)
__device__ __forceinline__ void lds_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
}

// Sum over the 16 lanes of a DPP row (lanes 16 k .. 16 k + 15); every lane
// gets the total.
__device__ __forceinline__ int32_t row16_sum(int32_t v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true); // row_half_mirror
  v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true); // row_mirror
  return v;
}

// Minimum / maximum over the wave, every lane gets the result: within the
// rows of 16 lanes by DPP, across the four rows through scalar registers (a
// butterfly of __shfl_xor is six dependent LDS-crossbar round trips).
template <bool MAX>
__device__ __forceinline__ float wave_fold(float v) {
  auto op = [](float a, float b) {
    return MAX ? __builtin_fmaxf(a, b) : __builtin_fminf(a, b);
  };
  auto dpp = [](float a, auto ctrl) {
    return __int_as_float(__builtin_amdgcn_update_dpp(
        0, __float_as_int(a), decltype(ctrl)::value, 0xF, 0xF, true));
  };
  v = op(v, dpp(v, std::integral_constant<int, 0xB1>{}));  // quad_perm [1,0,3,2]
  v = op(v, dpp(v, std::integral_constant<int, 0x4E>{}));  // quad_perm [2,3,0,1]
  v = op(v, dpp(v, std::integral_constant<int, 0x141>{})); // row_half_mirror
  v = op(v, dpp(v, std::integral_constant<int, 0x140>{})); // row_mirror
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return op(op(r0, r1), op(r2, r3));
}

// The per-column operands of the epilogue and its scalars, as they come out
// of memory.  Loaded before everything else so that their latency is spent
// behind the operand loads; turned into FlightEpi once they are needed.
struct FlightRaw {
  float as, bs, ys, bias;
  int32_t yz, az, bz, cs;
  int yz_sh, az_sh, bz_sh; // where in the loaded word each zero point's byte is
};

// The aligned word that holds the byte at p + i: a byte load would be widened
// right behind the load, which is a use of it, and the wave would wait there.
__device__ __forceinline__ int32_t flight_load_byte_word(
    const void *p, int i, int &shift) {
  // (pointer arithmetic only: through an integer the pointer would lose its
  // address space and the load become a flat one)
  const int at = (int)(((uintptr_t)p + (uintptr_t)(uint32_t)i) & 3);
  shift = at * 8;
  return *(const int32_t *)((const char *)p + (i - at));
}

template <int EPI>
__device__ __forceinline__ FlightRaw flight_load_params(
    const EpiParams &ep, bool a_off, int nc) {
  // absent operands read from colsum (always valid) and are masked later
  const bool has_bzp = ep.b_zp_len > 0;
  const void *bzp_ptr = has_bzp ? ep.b_zp : (const void *)ep.colsum;
  const bool has_azp = ep.a_zp_len > 0;
  const void *azp_ptr = has_azp ? ep.a_zp : (const void *)ep.colsum;
  const bool has_bias = EPI == kEpiF32 && ep.bias != nullptr;
  const float *bias_ptr = has_bias ? ep.bias : (const float *)ep.colsum;
  const float *as_ptr =
      (EPI != kEpiI32 && ep.a_scale) ? ep.a_scale : (const float *)ep.colsum;
  const float *bs_ptr = EPI != kEpiI32 ? ep.b_scale : (const float *)ep.colsum;
  const float *ys_ptr = EPI == kEpiQ8 ? ep.y_scale : (const float *)ep.colsum;
  const void *yz_ptr = EPI == kEpiQ8 ? ep.y_zp : (const void *)ep.colsum;
  // A zero the compiler cannot see through: a value loaded from an address
  // that is the same in every lane would be moved to a scalar register right
  // after the load, and the wave would wait there for every load it has
  // issued.  These stay vector registers until the epilogue.
  int vz = 0;
  asm volatile("" : "+v"(vz));
  FlightRaw r;
  r.as = as_ptr[vz];
  r.bs = bs_ptr[(EPI != kEpiI32 && ep.b_scale_len > 1) ? nc : vz];
  r.ys = ys_ptr[vz];
  // (the zero points as the bytes they are; flight_epi gives them their sign)
  r.yz = flight_load_byte_word(yz_ptr, vz, r.yz_sh);
  r.az = flight_load_byte_word(azp_ptr, vz, r.az_sh);
  r.bz = flight_load_byte_word(bzp_ptr, ep.b_zp_len > 1 ? nc : vz, r.bz_sh);
  r.cs = ep.colsum[nc];
  r.bias = bias_ptr[has_bias && ep.bias_len > 1 ? nc : 0];
  return r;
}

// Keeps every use of the parameters behind this point (the compiler would
// otherwise decode them, and wait for them, as early as it can: in front of
// the K loop, where that wait covers the weights as well).
__device__ __forceinline__ void flight_params_not_before(FlightRaw &r) {
  __builtin_amdgcn_sched_barrier(0); // (nor the K loop's last steps behind it)
  asm volatile(""
               : "+v"(r.as), "+v"(r.bs), "+v"(r.ys), "+v"(r.bias), "+v"(r.yz),
               "+v"(r.az), "+v"(r.bz), "+v"(r.cs));
  r.yz = (r.yz >> r.yz_sh) & 0xff;
  r.az = (r.az >> r.az_sh) & 0xff;
  r.bz = (r.bz >> r.bz_sh) & 0xff;
}

// What the epilogue needs per lane (its column) once the parameters are in.
struct FlightEpi {
  uint32_t cj; // da0 * colsum[j] + K * da0 * db[j]
  int32_t db;  // offset of B's column: its -128 shift minus its zero point
  float sj;    // a_scale * b_scale[j] (/ y_scale)
  float bj;    // bias[j], or -0.0f
  int32_t yz;
};

// a_scale / a_zp: the values to use (the fused layer computes them itself).
template <int EPI>
__device__ __forceinline__ FlightEpi flight_epi(const EpiParams &ep,
    const FlightRaw &r, bool a_off, int K, float a_scale, int32_t a_zp) {
  FlightEpi e;
  const int32_t oa = a_off ? 128 : 0;
  const int32_t ob = ep.b_unsigned ? 128 : 0;
  const int32_t da0 = oa - a_zp;
  const int32_t bz = ep.b_unsigned ? r.bz : (int32_t)(int8_t)r.bz;
  e.db = ob - (ep.b_zp_len > 0 ? bz : 0);
  e.cj = (uint32_t)da0 * (uint32_t)r.cs +
         (uint32_t)K * (uint32_t)da0 * (uint32_t)e.db;
  e.sj = 0.0f;
  e.yz = 0;
  if (EPI != kEpiI32) {
    // a_scale * b_scale[j] first, then one multiply per element; for the
    // requantize (a_scale * b_scale) / y_scale, in this order
    // (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:127).
    e.sj = a_scale * r.bs;
    if (EPI == kEpiQ8) {
      e.sj = e.sj / r.ys;
      e.yz = ep.y_unsigned ? r.yz : (int32_t)(int8_t)r.yz;
    }
  }
  e.bj = (EPI == kEpiF32 && ep.bias != nullptr) ? r.bias : -0.0f;
  return e;
}

// One finished 32 x 32 tile of a wave: zero-point correction, the op's output
// conversion, store.  Lane (column n = ncol0 + lane % 32, half lh) holds in
// register r the row 8 (r / 4) + 4 lh + r % 4 of the tile.  Only the first
// `rows` rows of the tile are the block's.  rs: LDS words with rowsum(A') of
// the tile's 32 rows (they only matter if B carries an offset: without one
// they are multiplied by zero, whatever they hold).  Results leave through
// range-checked buffer stores on a descriptor that covers exactly the M x N
// output: rows past M fall off its end, columns past N and rows that are not
// the block's get an offset that is out of range for every row (the hardware
// checks the sum of the lane's offset and the scalar row offset).
// act: 0 none / Relu by EpiParams::floor, 2 Gelu.
// 8-bit results in whole 16-byte pieces (N % 16 == 0, aligned output) pass
// through `stage` (32 rows x 32 * waves bytes) so that a lane stores 16 bytes
// of one row and the block's waves together write whole lines; every wave of
// the block must then call this together.
// (One wave per SIMD: nothing hides the latency of these instructions, so
// their number is what the epilogue costs.  No branch per element.)
template <int EPI>
__device__ __forceinline__ void flight_store_tile(const v16i &acc,
    const FlightEpi &e, const EpiParams &ep, const int32_t *rs, int mrow0,
    int rows, int ncol0_block, int wave, int waves, int lane, int M, int N,
    int act, uint8_t *stage, bool q8_lines, float &lim_lo, float &lim_hi) {
  // lim_lo / lim_hi: running minimum and maximum of the f32 results this lane
  // has stored (only kept when the caller asked for them, ep.limits.out)
  constexpr int ES = (EPI == kEpiQ8) ? 1 : 4;
  const int l32 = lane & 31, lh = lane >> 5;
  const int n = ncol0_block + wave * 32 + l32;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      ep.out, 0, (int)((uint32_t)M * (uint32_t)N * (uint32_t)ES), 0x00020000);
  const uint32_t toff =
      n < N ? ((uint32_t)(mrow0 + 4 * lh) * (uint32_t)N + (uint32_t)n) * (uint32_t)ES
            : 0x80000000u;
  // this lane's results before the output conversion
  // (|rowsum| <= 128 K and |db| < 512 fit 24 bits: a full-rate multiply)
  uint32_t y[16];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const v4i w = *(const v4i *)(rs + 8 * g + 4 * lh);
    y[4 * g + 0] = (uint32_t)acc[4 * g + 0] + e.cj + (uint32_t)__mul24(e.db, w.x);
    y[4 * g + 1] = (uint32_t)acc[4 * g + 1] + e.cj + (uint32_t)__mul24(e.db, w.y);
    y[4 * g + 2] = (uint32_t)acc[4 * g + 2] + e.cj + (uint32_t)__mul24(e.db, w.z);
    y[4 * g + 3] = (uint32_t)acc[4 * g + 3] + e.cj + (uint32_t)__mul24(e.db, w.w);
  }
  if (EPI != kEpiQ8) {
    if (EPI == kEpiF32) {
      float f[16];
#pragma unroll
      for (int r = 0; r < 16; ++r)
        f[r] = (float)(int32_t)y[r] * e.sj + e.bj;
      if (act == 2) { // (the same for every lane)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          y[r] = __float_as_uint(gelu_f32(f[r]));
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          y[r] = __float_as_uint(relu_f32(f[r], ep.floor));
      }
      if (ep.limits.out != nullptr) { // (the same for every lane)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (8 * (r >> 2) >= rows)
            continue;
          // rows of the tile that are not the block's count as NaN: ignored
          const bool mine = 8 * (r >> 2) + (r & 3) + 4 * lh < rows;
          const float v = mine ? __uint_as_float(y[r]) : __builtin_nanf("");
          lim_lo = __builtin_fminf(lim_lo, v);
          lim_hi = __builtin_fmaxf(lim_hi, v);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int rr = 8 * (r >> 2) + (r & 3); // + 4 lh: the row within the tile
      if (8 * (r >> 2) >= rows) // (the same for every lane) not the block's rows
        continue;
      const int voff = (int)(rr + 4 * lh < rows ? toff : 0x80000000u);
      const int soff = rr * N * ES; // the same for every lane
      __builtin_amdgcn_raw_buffer_store_b32((int)y[r], rsrc, voff, soff, kAuxThrough);
    }
    return;
  }
  // 8-bit: wrapping keeps the low byte, which the byte store does by itself;
  // saturating clamps first
  const bool sat = ep.narrow == kSaturate;
  const int32_t sat_lo = !sat ? INT32_MIN : ep.y_unsigned ? 0 : -128;
  const int32_t sat_hi = !sat ? INT32_MAX : ep.y_unsigned ? 255 : 127;
  const int32_t sat_hi_v = sat_hi; // (an instruction reads one scalar register)
  int32_t v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float f = (float)(int32_t)y[r] * e.sj;
    v[r] = (int32_t)((uint32_t)(int32_t)__builtin_rintf(f) + (uint32_t)e.yz);
    // (one instruction; bounds that do nothing when the result wraps)
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(v[r]) : "v"(v[r]), "s"(sat_lo), "v"(sat_hi_v));
  }
  if (!q8_lines) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int rr = 8 * (r >> 2) + (r & 3);
      if (8 * (r >> 2) >= rows)
        continue;
      const int voff = (int)(rr + 4 * lh < rows ? toff : 0x80000000u);
      __builtin_amdgcn_raw_buffer_store_b8((uint8_t)v[r], rsrc, voff, rr * N, 0);
    }
    return;
  }
  const int pitch = 32 * waves;
  uint8_t *const my_stage = stage + 4 * lh * pitch + wave * 32 + l32;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    my_stage[(8 * (r >> 2) + (r & 3)) * pitch] = (uint8_t)v[r];
  lds_sync();
  // lane -> 16 bytes of one row: 2 * waves lanes a row, 32 / waves rows a wave
  const int row = wave * (32 / waves) + lane / (2 * waves);
  const int c16 = lane % (2 * waves);
  const v4i w = *(const v4i *)(stage + row * pitch + c16 * 16);
  const int col = ncol0_block + c16 * 16;
  const uint32_t off = (col < N && row < rows)
                           ? (uint32_t)(mrow0 + row) * (uint32_t)N + (uint32_t)col
                           : 0x80000000u;
  __builtin_amdgcn_raw_buffer_store_b128(w, rsrc, (int)off, 0, kAuxThrough);
}

// The K loop of one wave: LDS and registers only -- one LDS read and one MFMA a
// step and nothing else.  (A wave does not issue while one of its MFMAs is being
// fed, 32 clocks; vector instructions between the MFMAs of a wave add their
// time to the loop instead of hiding in it.  Measured with one wave per SIMD:
// 32 clocks an MFMA with two independent accumulators, 44 with one, 71 with
// eight vector instructions in between.)
//
// Lane (row l32, half lh) takes chunk 2 s + lh of its row in step s.  With
// s = 8 g + v that is chunk 2 v + lh of K group g, at byte 8192 g + 256 l32 +
// ((32 v + 16 lh) ^ (16 (l32 % 16))) of the row tile: eight lane addresses
// (aaddr), one per v, and an immediate per g.
//
// Two independent accumulators, because an MFMA that adds to the result of
// the one before it waits for that result.  NT == 2: two row tiles (the second
// KG * 8 KiB after the first), each over all of K, sharing the weights.
// NT == 1: one row tile, even steps into acc[0], odd steps into acc[1]; the
// caller adds them.  Operand reads run a batch of four steps ahead; they
// complete in order, and the counts below say how many may still be
// outstanding when one is used.
// The weights may still be arriving when the loop starts: they were requested
// in order of K, and the compiler puts the wait for each in front of its MFMA.
template <int KG, int NT>
__device__ __forceinline__ void flight_kloop(const unsigned (&aaddr)[8],
    const v4i (&b)[8 * KG], v16i (&acc)[2]) {
  constexpr int BS = 4, NB = 8 * KG / BS;
  v4i fa[2][NT][BS];
  auto read_batch = [&](auto kc) {
    constexpr int k = decltype(kc)::value;
    static_for<BS>([&](auto vc) {
      static_for<NT>([&](auto tc) {
        constexpr int s = BS * k + decltype(vc)::value, t = decltype(tc)::value;
        v4i &f = fa[k & 1][t][decltype(vc)::value];
        const unsigned addr = aaddr[s % 8];
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(f)
                     : "v"(addr), "n"(8192 * (s / 8) + t * KG * 8192)
                     : "memory");
      });
    });
  };
  read_batch(std::integral_constant<int, 0>{});
  static_for<NB>([&](auto kc) {
    constexpr int k = decltype(kc)::value;
    constexpr bool more = k + 1 < NB;
    if constexpr (more)
      read_batch(std::integral_constant<int, k + 1>{});
    // One wait for the batch's operand reads (the next batch's stay
    // outstanding) and one for its weights: a wait instruction between two
    // MFMAs costs about eight clocks, a quarter of an MFMA.
    v4i &f0 = fa[k & 1][0][0], &f1 = fa[k & 1][0][1], &f2 = fa[k & 1][0][2],
        &f3 = fa[k & 1][0][3];
    if constexpr (NT == 2) {
      v4i &g0 = fa[k & 1][1][0], &g1 = fa[k & 1][1][1], &g2 = fa[k & 1][1][2],
          &g3 = fa[k & 1][1][3];
      asm volatile("s_waitcnt lgkmcnt(%8)"
                   : "+v"(f0), "+v"(g0), "+v"(f1), "+v"(g1), "+v"(f2), "+v"(g2),
                   "+v"(f3), "+v"(g3)
                   : "n"(more ? BS * NT : 0)
                   : "memory");
    } else {
      asm volatile("s_waitcnt lgkmcnt(%4)"
                   : "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3)
                   : "n"(more ? BS * NT : 0)
                   : "memory");
    }
    // (a use of the batch's last weights: the compiler waits for them here,
    // and with them for the batch's others, which were requested earlier)
    const v4i &b_last = b[BS * k + BS - 1];
    asm volatile("" : : "v"(b_last));
    static_for<BS>([&](auto vc) {
      static_for<NT>([&](auto tc) {
        constexpr int v = decltype(vc)::value, t = decltype(tc)::value;
        constexpr int s = BS * k + v;
        constexpr int c = NT == 2 ? t : (s & 1);
        v4i &f = fa[k & 1][t][v];
        acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f, b[s], acc[c], 0, 0, 0);
      });
    });
  });
}

// ---------------------------------------------------------------------------
// KG: K / 256 (a template argument: every loop over K is unrolled and has no
// branch).  FLIP: A holds uint8 and becomes int8 (minus 128) on its way into
// LDS; flags: bit 0, A' = A - 128 (FLIP, or A was stored that way); bit 1,
// onnx.Gelu on the f32 result.
// A block is WAVES column tiles side by side and NR row tiles of 32 one after
// the other (1 or 2, 2 NR <= WAVES).  Its rows of A are
// 8 nr groups of four rows; wave w brings groups w, w + waves, .. (two or four:
// with the weights, up to 192 registers of operands in flight) through its
// registers into LDS: uint8 becomes int8 (minus 128) on the
// way, and the row sums of A' are taken there if B carries an offset -- vector
// work on data that arrives first, done while the weights are still arriving,
// so that the K loop stays free of it.
// Every load is one the compiler sees, in program order A, Bp in order of K,
// parameters: it puts in front of each use a wait for exactly the loads up to
// the one used, and the K loop starts while the weights are still arriving.
// LDS: nr * KG * 8 KiB + 512 + 2 * waves KiB.
// ---------------------------------------------------------------------------
template <int KG, bool FLIP, int EPI, int NR, int WAVES>
__global__ __launch_bounds__(64 * WAVES, 1)
__attribute__((amdgpu_waves_per_eu(1, 1))) void k_gemm_i8_flight(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
    EpiParams ep, int flags, int regions_n, int bp_tiles) {
  constexpr int KH = 8 * KG, K = 256 * KG;
  constexpr int nr = NR, waves = WAVES;
  constexpr int P = (8 * NR) / WAVES; // groups of four rows a wave stages
  static_assert(KG >= 1 && KG <= kFlightMaxKG, "registers");
  static_assert(NR <= kFlightMaxTiles && (P == 2 || P == 4), "registers");
  const bool A_OFF = (flags & 1) != 0; // flags: 1 a_off, 2 onnx.Gelu on the f32 result
  const int act = (flags & 2) ? 2 : 0;
  extern __shared__ __attribute__((aligned(1024))) uint8_t sA[];
  int32_t *const s_rs = (int32_t *)(sA + nr * KG * 8192); // [32 * nr] row sums
  uint8_t *const stage = (uint8_t *)(s_rs + 32 * kFlightMaxTiles);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int rm = blockIdx.x / regions_n, rn = blockIdx.x % regions_n;
  const int row0 = rm * 32 * nr;
  const int ct = rn * waves + wave; // the wave's column tile
  FLIGHT_TS_DECL;
  FLIGHT_TS(0);

  // ---- everything is requested here ----------------------------------------
  const bool need_rs = ep.need_rowsum;
  // Group g of the block is rows 4 g .. 4 g + 3 (of row tile g / 8); for each
  // K group it is 1 KiB of LDS, 16 bytes per lane: lane l is position l % 16 of
  // row 4 g + l / 16 and holds the chunk that belongs there.  Rows past M are
  // copies of the last row and are never stored.
  const int rl = lane >> 4;
  v4i a[P][KG];
  auto request_rows = [&](auto hc) __attribute__((always_inline)) {
    constexpr int h = decltype(hc)::value;
    const int r = 4 * (wave + h * waves) + rl; // row within the block
    const int c = (lane & 15) ^ (r & 15);
    int row = row0 + r;
    row = row < M ? row : M - 1;
    const uint8_t *const src = A + (int64_t)row * K + c * 16;
#pragma unroll
    for (int cg = 0; cg < KG; ++cg) {
      a[h][cg] = *(const v4i *)(src + cg * 256);
      __builtin_amdgcn_sched_barrier(0); // in this order
    }
  };
  static_for<P>([&](auto hc) { request_rows(hc); });
  __builtin_amdgcn_sched_barrier(0);
  v4i b[KH];
  // column tiles past the packed weights (the last region of a ragged N)
  // read the last tile and are not stored
  const int ctc = ct < bp_tiles ? ct : bp_tiles - 1;
  const int8_t *const bp = Bp + (int64_t)ctc * KH * 1024 + lane * 16;
  auto request_weights = [&](auto from_c, auto to_c) __attribute__((always_inline)) {
    constexpr int FROM = decltype(from_c)::value, TO = decltype(to_c)::value;
    static_for<TO - FROM>([&](auto sc) {
      constexpr int s = FROM + decltype(sc)::value;
      b[s] = *(const v4i *)(bp + s * 1024);
      __builtin_amdgcn_sched_barrier(0); // in this order
    });
  };
  // The rows into LDS.
  auto stage_rows = [&](auto hc) __attribute__((always_inline)) {
    constexpr int h = decltype(hc)::value;
    const int g = wave + h * waves;
    uint8_t *const dst = sA + (g >> 3) * (KG * 8192) + (g & 7) * 1024 + lane * 16;
    int32_t sum = 0;
#pragma unroll
    for (int cg = 0; cg < KG; ++cg) {
      v4i v = a[h][cg];
      if (FLIP)
        v ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
            (int)0x80808080};
      *(v4i *)(dst + cg * 8192) = v;
      if (need_rs) // (the same for every wave)
        sum += frag_rowsum(v);
    }
    if (need_rs) {
      // the 16 lanes of a row hold all of its chunks: no other wave and no
      // other group adds to this row's sum
      sum = row16_sum(sum);
      if ((lane & 15) == 0)
        s_rs[4 * g + rl] = sum;
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // A wave issues a load only when the ones before it have been taken in, so
  // the requests for the weights take as long as the weights take to arrive,
  // and the rows, requested first, land halfway through.  They are staged
  // between the requests, not after them: the K loop can then start as soon
  // as the last request is out, and follows the weights as they arrive.
  typedef std::integral_constant<int, 0> c0;
  typedef std::integral_constant<int, KH / 2> c_half;
  typedef std::integral_constant<int, 3 * KH / 4> c_3q;
  typedef std::integral_constant<int, KH> c_all;
  request_weights(c0{}, c_half{});
  FLIGHT_TS(1);
  static_for<P / 2>([&](auto hc) { stage_rows(hc); });
  FLIGHT_TS(2);
  request_weights(c_half{}, c_3q{});
  static_for<P / 2>([&](auto hc) {
    stage_rows(std::integral_constant<int, P / 2 + decltype(hc)::value>{});
  });
  request_weights(c_3q{}, c_all{});
  // The epilogue's parameters, requested last and first used after the K loop
  // (a use before that would wait for the weights, which were requested before
  // them).
  const int n = ct * 32 + l32;
  FlightRaw raw = flight_load_params<EPI>(ep, A_OFF, n < N ? n : N - 1);
  __builtin_amdgcn_sched_barrier(0);
  FLIGHT_TS(3);
  lds_sync(); // every wave's rows (and row sums) are in LDS
  __builtin_amdgcn_sched_barrier(0);
  FLIGHT_TS(4);

  unsigned aaddr[8];
  {
    const unsigned arow = (unsigned)(uintptr_t)(lds_ptr)sA + l32 * 256;
    const unsigned xh = (unsigned)((16 * lh) ^ (16 * (l32 & 15)));
#pragma unroll
    for (int v = 0; v < 8; ++v)
      aaddr[v] = arow + ((unsigned)(32 * v) ^ xh);
  }
  const bool q8_lines = EPI == kEpiQ8 && (N & 15) == 0 &&
                        ((((uintptr_t)ep.out) & 15) == 0);
  const v16i acc_zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float lim_lo = __builtin_inff(), lim_hi = -__builtin_inff();
  auto finish = [&](const v16i &acc, const FlightEpi &e, int t)
                    __attribute__((always_inline)) {
    flight_store_tile<EPI>(acc, e, ep, s_rs + 32 * t, row0 + 32 * t, 32,
        rn * waves * 32, wave, waves, lane, M, N, act,
        stage + (t & 1) * 1024 * waves, q8_lines, lim_lo, lim_hi);
  };
  auto epi_params = [&]() __attribute__((always_inline)) {
    flight_params_not_before(raw);
    return flight_epi<EPI>(ep, raw, A_OFF, K, raw.as,
        ep.a_zp_len > 0 ? (A_OFF ? raw.az : (int32_t)(int8_t)raw.az) : 0);
  };
  v16i acc[2] = {acc_zero, acc_zero};
  // (the weights are still arriving)
  flight_kloop<KG, NR>(aaddr, b, acc);
  // (A use of every weight register behind the loop: without it the compiler
  // hands a step's registers to the operand reads of the steps after it, and
  // the loop runs a tenth slower.)
#pragma unroll
  for (int s = 0; s < KH; ++s)
    asm volatile("" : : "v"(b[s]));
  if (NR == 1) {
#pragma unroll
    for (int r = 0; r < 16; ++r)
      acc[0][r] += acc[1][r];
  }
  FLIGHT_TS(5);
  const FlightEpi e = epi_params();
  finish(acc[0], e, 0);
  if (NR == 2)
    finish(acc[1], e, 1);
  if (EPI == kEpiF32 && ep.limits.out != nullptr) { // (the same for every wave)
    // rows past M are copies of the last row; columns past N are nobody's
    if (n >= N) {
      lim_lo = __builtin_inff();
      lim_hi = -__builtin_inff();
    }
    lds_sync(); // (the staging area is free)
    block_publish_limits(lim_lo, lim_hi, ep.limits, (float *)stage, wave, lane,
        waves, [] { lds_sync(); });
  }
#ifdef FLIGHT_TIMING
  FLIGHT_TS(6);
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  FLIGHT_TS(7);
  FLIGHT_TS_WRITE;
#endif
}

// ---------------------------------------------------------------------------
// The dynamically quantized layer in one launch.  A block is eight waves; it
// owns R = 8 << RSH rows of X and 32 * mwaves columns (mwaves <= 4: the waves
// that multiply; all eight load and quantize X, which is what takes the time,
// and the last four poll the exchange slots).
// Thread (row r = tid / TPR, position p = tid % TPR, TPR = 512 / R) takes
// float4 p + TPR j of its row, j < NJ = (K / 4) / TPR.  Register slot i holds
// j = ((i / S + share) % G) + G * (i % S) with S = NJ / G: slots 0 .. S-1 are
// the block's own share of its row region's minimum / maximum, the columns
// the region's other blocks do not reduce.
//
// Order of the memory operations: the rows, the share first (loads complete in
// order, so the share is there before the rest); [publication]; the epilogue's
// parameters; then the weights in the waves that multiply and the poll of the
// slots in the last four waves.  The weights arrive while the blocks wait for
// one another and quantize.
// ---------------------------------------------------------------------------
struct FlightDq {
  const float *X;            // [M, K] f32
  unsigned long long *slots; // tagged (launch number, value) slots
  unsigned epoch;
  unsigned *failed;
  unsigned spin_limit;
  int share_groups; // G: blocks of a row region that split its min / max
  int mwaves;       // waves that multiply: 32 * mwaves columns per block
  int act;          // 0 none / Relu by EpiParams::floor, 2 Gelu
};

template <int KG, int RSH>
__global__ __launch_bounds__(512, 1) void k_gemm_i8_flight_dq(
    const int8_t *__restrict__ Bp, int M, int N, EpiParams ep, int regions_n,
    int bp_tiles, FlightDq dq) {
  constexpr int KH = 8 * KG, K = 256 * KG;
  constexpr int WAVES = 8, T = 64 * WAVES;
  constexpr int R = 8 << RSH;         // rows of the block
  constexpr int TPR = T / R;          // threads per row: 64, 32 or 16
  constexpr int NJ = (K / 4) / TPR;   // float4 per thread: KG, 2 KG or 4 KG
  static_assert(RSH >= 0 && RSH <= 2, "rows");
  extern __shared__ __attribute__((aligned(1024))) uint8_t sA[]; // one row tile
  int32_t *const s_rs = (int32_t *)(sA + KG * 8192); // [32]
  __shared__ float s_lo[WAVES], s_hi[WAVES];
  __shared__ int s_ok;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mwaves = dq.mwaves;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int rm = blockIdx.x / regions_n, rn = blockIdx.x % regions_n;
  const int row0 = rm * R;
  const bool multiplies = wave < mwaves;
  const int ct = rn * mwaves + (multiplies ? wave : 0);
  FLIGHT_TS_DECL;
  FLIGHT_TS(0);

  typedef float f4 __attribute__((ext_vector_type(4)));
  const int r = tid / TPR, p = tid % TPR;
  const bool row_in = row0 + r < M;
  const f4 *__restrict__ xr =
      (const f4 *)(dq.X + (int64_t)(row_in ? row0 + r : M - 1) * K) + p;
  const int G = dq.share_groups, S = NJ / G, share = rn % G;
  // j of register slot i, as scalar arithmetic
  int jof[NJ];
  {
    int a = 0, bb = 0;
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
      int g = a + share;
      g = g >= G ? g - G : g;
      jof[i] = g + G * bb;
      if (++bb == S) {
        bb = 0;
        ++a;
      }
    }
  }
  // ---- the block's rows, its share of the minimum / maximum first ---------------
  f4 x[NJ];
#pragma unroll
  for (int i = 0; i < NJ; ++i)
    x[i] = xr[TPR * jof[i]];
  __builtin_amdgcn_sched_barrier(0);
  float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < NJ; ++i) {
    if (i < S) {
      lo = __builtin_fminf(lo, __builtin_fminf(__builtin_fminf(x[i].x, x[i].y),
                                   __builtin_fminf(x[i].z, x[i].w)));
      hi = __builtin_fmaxf(hi, __builtin_fmaxf(__builtin_fmaxf(x[i].x, x[i].y),
                                   __builtin_fmaxf(x[i].z, x[i].w)));
    }
  }
  if (!row_in) { // a copy of the last row, which its own block reduces
    lo = __builtin_inff();
    hi = -__builtin_inff();
  }
  lo = wave_fold<false>(lo);
  hi = wave_fold<true>(hi);
  if (lane == 0) {
    s_lo[wave] = lo;
    s_hi[wave] = hi;
  }
  if (tid == 0)
    s_ok = 1;
  if (tid < 32)
    s_rs[tid] = 0;
  lds_sync();
  // The caller knows minimum and maximum of X (from the layer before): nothing
  // is published and nobody polls.
  const bool known = ep.x_limits != nullptr;
  // Publishers: the first G blocks of every row region.
  const int nslots = (int)(gridDim.x / regions_n) * G; // <= 256
  if (tid == 0 && rn < G && !known) {
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
  FLIGHT_TS(1);
  __builtin_amdgcn_sched_barrier(0);

  // ---- the epilogue's parameters ------------------------------------------------
  const int n = ct * 32 + l32;
  FlightRaw raw = flight_load_params<kEpiF32>(ep, true, n < N ? n : N - 1);
  const bool need_rs = ep.need_rowsum;
  lds_sync(); // s_lo / s_hi are reused below
  __builtin_amdgcn_sched_barrier(0);

  // ---- the weights; the poll ---------------------------------------------------------
  // The waves that multiply (the first mwaves <= 4) request their weights.  The
  // last four waves poll: one slot per thread (nslots <= 256), until both
  // words carry this launch's number; bounded (see k_dql_grid).  Each word was
  // written by one atomic store and is read by one atomic load, past the
  // caches that other XCDs do not see.  A polling wave has no weights on their
  // way, so its answer does not queue behind them.
  // The two kinds of waves run the rest of the kernel in separate branches
  // (with the same barriers): the compiler counts the loads a wave has in
  // flight per branch, and in common code it would make the multiplying
  // waves wait for their weights wherever the others have nothing to wait for.
  float scale = 0.0f, zpf = 0.0f;
  // Once the poll is over: scale and zero point, the block's rows as 8-bit
  // values minus 128 into LDS.  float4 c4 = p + TPR j of row r: bytes 4 c4 .. of
  // the row, K group c4 / 64, chunk (c4 % 64) / 4 at position chunk ^ (r % 16).
  // False if the exchange gave up.
  auto rows_to_lds = [&]() __attribute__((always_inline)) {
    FLIGHT_TS(2);
    lds_sync();
    if (!s_ok) {
      // (the loads of the weights still in flight are waited for at the end of
      // the program like any others)
      if (tid == 0)
        __hip_atomic_store(
            dq.failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    float xlo = s_lo[0], xhi = s_hi[0];
#pragma unroll
    for (int w2 = 1; w2 < 4; ++w2) { // what the four polling waves found
      xlo = __builtin_fminf(xlo, s_lo[w2]);
      xhi = __builtin_fmaxf(xhi, s_hi[w2]);
    }
    if (known) {
      xlo = ep.x_limits[0];
      xhi = ep.x_limits[1];
    }
    FLIGHT_TS(3);
    dynamic_params(xlo, xhi, scale, zpf);
    const float recip = 1.0f / scale;
    uint8_t *const rowp = sA + r * 256 + (p & 3) * 4;
    int32_t sum = 0;
    auto quantize = [&](auto fast_c) __attribute__((always_inline)) {
      constexpr int FAST = decltype(fast_c)::value ? 1 : 0;
#pragma unroll
      for (int i = 0; i < NJ; ++i) {
        const int c4 = p + TPR * jof[i];
        const int c = (c4 & 63) >> 2;
        const uint32_t q =
            quant_pack4<false, true, FAST>(x[i].x, x[i].y, x[i].z, x[i].w, scale,
                scale, scale, scale, recip, recip, recip, recip, zpf, zpf, zpf,
                zpf) ^
            0x80808080u;
        *(uint32_t *)(rowp + (c4 >> 6) * 8192 + ((c ^ (r & 15)) << 4)) = q;
        sum = __builtin_amdgcn_sdot4((int)q, 0x01010101, sum, false);
      }
    };
    if (scale_is_tame(scale)) // the same for every thread
      quantize(std::true_type{});
    else
      quantize(std::false_type{});
    if (need_rs) {
      // the TPR threads of a row are 1, 2 or 4 DPP rows of 16 lanes
      sum = row16_sum(sum);
      if ((p & 15) == 0)
        atomicAdd(&s_rs[r], sum);
    }
    lds_sync();
    FLIGHT_TS(4);
    return true;
  };
  if (!multiplies) { // (the same for the whole wave)
    if (wave >= 4 && !known) {
      const int slot = tid - 256;
      const bool polls = slot < nslots;
      const unsigned long long *const slot_p = &dq.slots[2 * (polls ? slot : 0)];
      unsigned long long w0 = 0, w1 = 0;
      bool got = !polls;
      for (unsigned spin = 0; !got && spin < dq.spin_limit; ++spin) {
        if (spin)
          __builtin_amdgcn_s_sleep(1);
        w0 = __hip_atomic_load(slot_p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w1 = __hip_atomic_load(slot_p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        got = (unsigned)(w0 >> 32) == dq.epoch && (unsigned)(w1 >> 32) == dq.epoch;
      }
      lo = polls ? __uint_as_float((unsigned)w0) : __builtin_inff();
      hi = polls ? __uint_as_float((unsigned)w1) : -__builtin_inff();
      lo = wave_fold<false>(lo);
      hi = wave_fold<true>(hi);
      const bool all_ok = __builtin_amdgcn_ballot_w64(!got) == 0;
      if (lane == 0) {
        s_lo[wave - 4] = lo;
        s_hi[wave - 4] = hi;
        if (!all_ok)
          s_ok = 0;
      }
    }
    (void)rows_to_lds();
    return;
  }
  v4i b[KH];
  {
    const int ctc = ct < bp_tiles ? ct : bp_tiles - 1;
    const int8_t *const bp = Bp + (int64_t)ctc * KH * 1024 + lane * 16;
#pragma unroll
    for (int s = 0; s < KH; ++s) {
      b[s] = *(const v4i *)(bp + s * 1024);
      __builtin_amdgcn_sched_barrier(0); // in this order
    }
  }
  if (!rows_to_lds()) {
#ifdef FLIGHT_TIMING
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#endif
    return;
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop ---------------------------------------------------------------------
  unsigned aaddr[8];
  {
    const unsigned arow = (unsigned)(uintptr_t)(lds_ptr)sA + l32 * 256;
    const unsigned xh = (unsigned)((16 * lh) ^ (16 * (l32 & 15)));
#pragma unroll
    for (int v = 0; v < 8; ++v)
      aaddr[v] = arow + ((unsigned)(32 * v) ^ xh);
  }
  v16i accs[2] = {{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0},
      {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}};
  flight_kloop<KG, 1>(aaddr, b, accs);
  v16i acc;
#pragma unroll
  for (int r2 = 0; r2 < 16; ++r2)
    acc[r2] = accs[0][r2] + accs[1][r2];
  FLIGHT_TS(5);
  flight_params_not_before(raw);
  const FlightEpi e =
      flight_epi<kEpiF32>(ep, raw, true, K, scale, (int32_t)(uint32_t)zpf);
  float lim_lo = __builtin_inff(), lim_hi = -__builtin_inff();
  flight_store_tile<kEpiF32>(acc, e, ep, s_rs, row0, R, rn * mwaves * 32, wave,
      mwaves, lane, M, N, dq.act, nullptr, false, lim_lo, lim_hi);
  if (ep.limits.out != nullptr) { // (the same for every wave)
    // Rows past M are copies of the last row; columns past N are nobody's.
    // Only the multiplying waves are still running: the barrier counts them.
    if (n >= N) {
      lim_lo = __builtin_inff();
      lim_hi = -__builtin_inff();
    }
    lds_sync(); // (the row sums have been read)
    block_publish_limits(lim_lo, lim_hi, ep.limits, (float *)s_rs, wave, lane,
        mwaves, [] { lds_sync(); });
  }
#ifdef FLIGHT_TIMING
  FLIGHT_TS(6);
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  FLIGHT_TS(7);
  FLIGHT_TS_WRITE;
#endif
}

// A block's LDS beyond the default limit has to be asked for, once per kernel.
template <typename Kern>
hipError_t flight_allow_lds(Kern kern) {
  static const hipError_t e =
      hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
          hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
  return e;
}

struct FlightShape {
  int nr, waves; // row tiles per block, column tiles per block
  int64_t blocks;
};

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

bool flight_k_ok(int64_t K) {
  return K >= 512 && K <= 256 * kFlightMaxKG && K % 256 == 0;
}

// Among the block shapes that cover the problem with at most one block per
// CU, the one that brings the fewest bytes into a CU; with equal bytes the one
// with more waves per block.  (2 nr <= waves: a wave stages at most four
// groups of four rows.)
FlightShape flight_shape(int64_t M, int64_t N) {
  FlightShape best = {0, 0, 0};
  int64_t best_bytes = 0;
  const int cus = flight_cus();
  for (int nr = 1; nr <= kFlightMaxTiles; nr *= 2)
    for (int w = 2 * nr; w <= 4; w *= 2) {
      const int64_t blocks =
          ((M + 32 * nr - 1) / (32 * nr)) * ((N + 32 * w - 1) / (32 * w));
      if (blocks > cus)
        continue;
      const int64_t bytes = 32 * nr + 32 * w; // times K
      if (best.nr == 0 || bytes < best_bytes ||
          (bytes == best_bytes && w > best.waves)) {
        best = FlightShape{nr, w, blocks};
        best_bytes = bytes;
      }
    }
  return best;
}

template <int KG, bool FLIP, int EPI, int NR, int WAVES>
hipError_t flight_launch(hipStream_t st, const GemmArgs &g, const EpiParams &ep,
    int a_mode) {
  const int regions_n = (int)((g.N + 32 * WAVES - 1) / (32 * WAVES));
  const int regions_m = (int)((g.M + 32 * NR - 1) / (32 * NR));
  const int bp_tiles = (int)(round_up(g.N, kGemmBN) / 32);
  auto kern = k_gemm_i8_flight<KG, FLIP, EPI, NR, WAVES>;
  hipError_t e = flight_allow_lds(kern);
  if (e != hipSuccess)
    return e;
  const size_t lds = (size_t)NR * KG * 8192 + 4 * 32 * kFlightMaxTiles +
                     2 * 1024 * (size_t)WAVES;
  kern<<<dim3((unsigned)(regions_m * regions_n)), dim3(64 * WAVES), lds, st>>>(
      (const uint8_t *)g.A, g.Bp, (int)g.M, (int)g.N, ep,
      (a_mode != 0 ? 1 : 0) | (EPI == kEpiF32 && g.gelu ? 2 : 0), regions_n,
      bp_tiles);
  return hipGetLastError();
}

template <int KG, bool FLIP, int EPI>
hipError_t flight_launch_shape(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode, const FlightShape &sh) {
  if (sh.nr == 2)
    return flight_launch<KG, FLIP, EPI, 2, 4>(st, g, ep, a_mode);
  if (sh.waves == 2)
    return flight_launch<KG, FLIP, EPI, 1, 2>(st, g, ep, a_mode);
  return flight_launch<KG, FLIP, EPI, 1, 4>(st, g, ep, a_mode);
}

template <bool FLIP, int EPI>
hipError_t flight_launch_kg(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode, const FlightShape &sh) {
  switch (g.K / 256) {
  case 2:
    return flight_launch_shape<2, FLIP, EPI>(st, g, ep, a_mode, sh);
  case 3:
    return flight_launch_shape<3, FLIP, EPI>(st, g, ep, a_mode, sh);
  case 4:
    return flight_launch_shape<4, FLIP, EPI>(st, g, ep, a_mode, sh);
  default:
    return hipErrorInvalidValue;
  }
}

template <bool FLIP>
hipError_t flight_launch_epi(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode, const FlightShape &sh) {
  switch (g.epi) {
  case kEpiI32:
    return flight_launch_kg<FLIP, kEpiI32>(st, g, ep, a_mode, sh);
  case kEpiF32:
    return flight_launch_kg<FLIP, kEpiF32>(st, g, ep, a_mode, sh);
  default:
    return flight_launch_kg<FLIP, kEpiQ8>(st, g, ep, a_mode, sh);
  }
}

// Block shape of the fused layer: R = 8 << rsh rows, 32 * mwaves columns.
// Among the shapes whose grid is resident at once, the one that brings the
// fewest bytes into a CU (4 R + 32 mwaves, times K); nothing if there is none.
struct FlightDqShape {
  int rsh, mwaves;
};
bool flight_dq_shape(int64_t M, int64_t N, FlightDqShape &best) {
  const int cus = flight_cus() < 256 ? flight_cus() : 256;
  int64_t best_bytes = 0;
  bool found = false;
  for (int rsh = 0; rsh <= 2; ++rsh)
    for (int w = 1; w <= 4; w *= 2) {
      const int64_t R = 8 << rsh;
      if (((M + R - 1) / R) * ((N + 32 * w - 1) / (32 * w)) > cus)
        continue;
      const int64_t bytes = 4 * R + 32 * w;
      if (!found || bytes < best_bytes) {
        best = FlightDqShape{rsh, w};
        best_bytes = bytes;
        found = true;
      }
    }
  return found;
}

template <int KG, int RSH>
hipError_t flight_launch_dq(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, const FlightDq &dq) {
  const int regions_n = (int)((g.N + 32 * dq.mwaves - 1) / (32 * dq.mwaves));
  const int regions_m = (int)((g.M + (8 << RSH) - 1) / (8 << RSH));
  const int bp_tiles = (int)(round_up(g.N, kGemmBN) / 32);
  auto kern = k_gemm_i8_flight_dq<KG, RSH>;
  hipError_t e = flight_allow_lds(kern);
  if (e != hipSuccess)
    return e;
  kern<<<dim3((unsigned)(regions_m * regions_n)), dim3(512),
      (size_t)KG * 8192 + 128, st>>>(g.Bp, (int)g.M, (int)g.N, ep, regions_n,
      bp_tiles, dq);
  return hipGetLastError();
}

template <int KG>
hipError_t flight_launch_dq_rows(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int rsh, const FlightDq &dq) {
  switch (rsh) {
  case 0:
    return flight_launch_dq<KG, 0>(st, g, ep, dq);
  case 1:
    return flight_launch_dq<KG, 1>(st, g, ep, dq);
  default:
    return flight_launch_dq<KG, 2>(st, g, ep, dq);
  }
}

} // namespace

// Whether k_gemm_i8_flight takes this problem (a_mode as in launch_gemm: 0 int8,
// 1 uint8, 2 stored minus 128).  One zero point per row of A is left to the
// other kernels.
bool flight_ok(const GemmArgs &g, int a_mode) {
  if (!flight_k_ok(g.K) || g.M < 1 || g.X || ((((uintptr_t)g.A) & 15) != 0) ||
      g.M * g.N >= ((int64_t)1 << 29) || (g.a_zp != nullptr && g.a_zp_len > 1))
    return false;
  return flight_shape(g.M, g.N).nr > 0;
}

hipError_t launch_gemm_flight(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode) {
  if (!flight_ok(g, a_mode))
    return hipErrorInvalidValue;
  const FlightShape sh = flight_shape(g.M, g.N);
  return a_mode == 1 ? flight_launch_epi<true>(st, g, ep, a_mode, sh)
                     : flight_launch_epi<false>(st, g, ep, a_mode, sh);
}

// The fused layer in one launch: every block of the grid resident at once
// (they wait for one another).
bool flight_quantizes_rows(int64_t M, int64_t K, int64_t N, const void *x) {
  if (!flight_k_ok(K) || M < 1 || N < 1 || ((((uintptr_t)x) & 15) != 0) ||
      M * N >= ((int64_t)1 << 29))
    return false;
  FlightDqShape sh;
  return flight_dq_shape(M, N, sh);
}

hipError_t launch_gemm_flight_dq(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, DqlScratch &scratch) {
  FlightDqShape sh;
  if (!g.X || g.epi != kEpiF32 || !flight_quantizes_rows(g.M, g.K, g.N, g.X) ||
      !flight_dq_shape(g.M, g.N, sh))
    return hipErrorInvalidValue;
  const int R = 8 << sh.rsh;
  const int regions_n = (int)((g.N + 32 * sh.mwaves - 1) / (32 * sh.mwaves));
  const int regions_m = (int)((g.M + R - 1) / R);
  if (regions_m * regions_n > scratch.max_blocks)
    return hipErrorInvalidValue;
  FlightDq dq = {};
  dq.X = g.X;
  dq.act = g.gelu ? 2 : 0;
  dq.mwaves = sh.mwaves;
  // the largest number of blocks of a row region, a divisor of the float4s a
  // thread holds, that can share the region's minimum / maximum between them
  const int NJ = (int)(g.K / 4) / (512 / R);
  dq.share_groups = 1;
  for (int d = 1; d <= regions_n && d <= NJ; ++d)
    if (NJ % d == 0)
      dq.share_groups = d;
  // (minimum and maximum of X known: the blocks do not wait for one another,
  // and the kernel is like any other)
  const bool exchanges = ep.x_limits == nullptr;
  GridExchange ex = {};
  if (exchanges && !dql_exchange_begin(st, scratch, ex))
    return hipErrorNotReady; // the exchange is off or another stream's runs
  dq.slots = ex.slots;
  dq.epoch = ex.epoch;
  dq.failed = ex.failed;
  dq.spin_limit = ex.spin_limit;
  hipError_t e;
  switch (g.K / 256) {
  case 2:
    e = flight_launch_dq_rows<2>(st, g, ep, sh.rsh, dq);
    break;
  case 3:
    e = flight_launch_dq_rows<3>(st, g, ep, sh.rsh, dq);
    break;
  default:
    e = flight_launch_dq_rows<4>(st, g, ep, sh.rsh, dq);
    break;
  }
  if (exchanges)
    dql_exchange_end(st, e == hipSuccess);
  return e;
}

} // namespace gemm
} // namespace om

#ifdef FLIGHT_TIMING
extern "C" int om_dev_flight_ts(void *out, size_t bytes) {
  (void)hipDeviceSynchronize();
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(om::gemm::flight_ts),
      bytes < sizeof(om::gemm::flight_ts) ? bytes : sizeof(om::gemm::flight_ts));
}
#endif
