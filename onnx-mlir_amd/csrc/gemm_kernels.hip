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
// once into Bp, the order in which the matrix cores consume it (k_pack_b):
//   Bp[nt][ks][sub][lane][16 bytes], nt = column / 32, ks = K step of 64
//   bytes, sub = half step; lane l holds, for column nt*32 + l%32, the 16 K
//   bytes starting at ks*64 + (sub*2 + l/32)*16
// int8 (u8 shifted by -128), zero filled up to [Npad, Kpad].  The operand of
// one MFMA is one contiguous KiB, 16 bytes per lane, whether it is loaded
// into registers or copied into LDS.
//
// Kernels (all walk K in steps of 64 bytes):
//   k_gemm_i8_bs         Bp read straight into MFMA operand registers, only
//                        the A tile goes through LDS (copied there without
//                        passing through registers); more than one tile per CU
//   k_gemm_i8_dma        A and Bp tiles copied from global memory straight
//                        into a ring of three LDS stages; up to one tile per CU
//   k_gemm_i8            tiles staged through registers, LDS double buffered;
//                        also the general path: any K, any alignment of A
//   k_gemm_i8_skinny_bp  M <= 32: weight streaming, K split over the waves
// A tiles in LDS have 64-byte rows whose 16-byte chunk index is XOR-swizzled
// with bits 2..3 of the row (bank-conflict free writes and operand reads); Bp
// tiles in LDS keep their global order.

#include "gemm_common.h"
#include "gemm_epilogue.h"

#include <stdlib.h>

namespace om {

using namespace gemm;

namespace {

// BM x BN block tile, WGM x WGN waves, each wave a (BM/WGM) x (BN/WGN) tile
// made of 32x32 MFMA tiles.
// A_MODE: 0 = int8 as is, 1 = uint8 (XOR 0x80 while staging), 2 = already
// shifted (stored as u8-128) -- offsets as for uint8, no XOR.
// A_LOAD: kLoadAligned = K % 64 == 0 and A 16-byte aligned (plain vector
// loads); kLoadAny = any K and alignment, at least 16 bytes of A (16-byte
// loads at byte addresses, the bytes past the end of a row replaced); kLoadBytes
// = byte loads (an A of fewer than 16 bytes, K = 0).
template <int BM, int BN, int WGM, int WGN, int MINB, int A_MODE, int EPI,
    int A_LOAD>
__global__ __launch_bounds__(WGM *WGN * 64, MINB) void k_gemm_i8(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
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
  // on an XCD share a few A panels and Bp panels.
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
  const int KTs = Kpad / BK; // K steps: stride between column tiles of Bp

  // Global loads only fetch; uint8 data is shifted to int8 after it is read
  // back from LDS.  In the general paths bytes outside [M,K] are replaced by
  // the byte that the shift maps to 0.
  auto load_global = [&](int k0, v4i(&ra)[CH_A], v4i(&rb)[CH_B]) {
#pragma unroll
    for (int h = 0; h < CH_A; ++h) {
      const int q = tid + h * THREADS;
      const int r = q >> 2, c = q & 3;
      const int gm = m0 + r;
      const int gk = k0 + c * 16;
      v4i v = {kFill, kFill, kFill, kFill};
      if (A_LOAD == kLoadAligned) {
        // K % 64 == 0, so every chunk lies inside its row.  Rows past M are
        // clamped to the last row: they only feed output rows that are never
        // stored, and an unconditional load lets the hardware counter of
        // outstanding loads be waited on exactly (a load under a branch
        // would force a full drain).
        const int gmc = gm < M ? gm : M - 1;
        v = *(const v4i *)(A + (int64_t)gmc * K + gk);
      } else if (A_LOAD == kLoadAny) {
        // One 16-byte load per chunk at whatever address the chunk has.  The
        // chunk at the end of a row holds K - gk < 16 of its bytes; the rest
        // (the next row's, or nothing: the load is moved back to end with the
        // buffer and its bytes shifted down) become the fill byte.  Chunks
        // outside [M, K] load the first 16 bytes and keep none of them.
        const bool valid = gm < M && gk < K;
        const int64_t total = (int64_t)M * K;
        const int64_t off = valid ? (int64_t)gm * K + gk : 0;
        const int len = valid ? (K - gk < 16 ? K - gk : 16) : 0;
        const int64_t off2 = off + 16 <= total ? off : total - 16;
        const int sh = (int)(off - off2) * 8; // bits to shift down, < 128
        const v4i_any raw = *(const v4i_any *)(A + off2);
        uint64_t lo = (uint32_t)raw.x | ((uint64_t)(uint32_t)raw.y << 32);
        uint64_t hi = (uint32_t)raw.z | ((uint64_t)(uint32_t)raw.w << 32);
        if (sh >= 64) {
          lo = hi;
          hi = 0;
        }
        const int s1 = sh & 63;
        if (s1) {
          lo = (lo >> s1) | (hi << (64 - s1));
          hi >>= s1;
        }
        const uint64_t fill64 =
            (uint32_t)kFill | ((uint64_t)(uint32_t)kFill << 32);
        const uint64_t mlo =
            len >= 8 ? ~(uint64_t)0 : (((uint64_t)1 << (8 * len)) - 1);
        const uint64_t mhi =
            len >= 16 ? ~(uint64_t)0
                      : (len > 8 ? (((uint64_t)1 << (8 * (len - 8))) - 1) : 0);
        lo = (lo & mlo) | (fill64 & ~mlo);
        hi = (hi & mhi) | (fill64 & ~mhi);
        v = (v4i){(int)(uint32_t)lo, (int)(uint32_t)(lo >> 32),
            (int)(uint32_t)hi, (int)(uint32_t)(hi >> 32)};
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
      // Chunk q of the stage's Bp tile: KiB q/64 is (column tile (q/64)/2,
      // half step (q/64)%2), 16 bytes per lane.  Bp is padded to
      // [Npad, Kpad]: always in bounds and aligned.
      const int q = tid + h * THREADS;
      const int ci = q >> 6;
      rb[h] = *(const v4i *)(Bp +
                             ((int64_t)((n0 >> 5) + (ci >> 1)) * KTs +
                                 (k0 >> 6)) * 2048 +
                             (ci & 1) * 1024 + (q & 63) * 16);
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
      *(v4i *)(&sB[buf][q * 16]) = rb[h];
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
  const bool need_rs = ep.need_rowsum;
  int32_t rsp[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
    rsp[i] = 0;

  // Operands of half step s (32 of the stage's 64 K bytes) of this wave's tile.
  auto read_frags = [&](int buf, int s2, v4i(&fa)[TM], v4i(&fb)[TN]) {
    const int c = s2 * 2 + lh;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *(const v4i *)(&sA[buf][lds_off(wm * WTM + i * 32 + l32, c)]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *(const v4i *)(&sB[buf][(((wn * TN + j) * 2 + s2) * 64 + lane) *
                                      16]);
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

  // One K step on LDS buffer `buf`: request all operands of the step, put the
  // next step's tile (already in registers) into the other buffer -- every
  // wave finished reading that one before the last barrier --, refill those
  // registers two steps ahead, then run the MFMAs of both half steps.  RS is
  // whether row sums of A are needed, fixed outside the loop so that the loop
  // body has no branch.
  auto k_step = [&](int buf, v4i(&ra)[CH_A], v4i(&rb)[CH_B], int knext,
                    auto RS) {
    v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    read_frags(buf, 0, fa0, fb0);
    read_frags(buf, 1, fa1, fb1);
    __builtin_amdgcn_sched_barrier(0);
    store_lds(buf ^ 1, ra, rb);
    load_global(knext, ra, rb);
    __builtin_amdgcn_sched_barrier(0);
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080,
        (int)0x80808080};
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      // uint8 -> int8 (minus 128) on the operand registers: VALU work that
      // runs beside the MFMAs
      if (A_MODE == 1)
        fa0[i] ^= flip;
      if (decltype(RS)::value)
        rsp[i] += frag_rowsum(fa0[i]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa0[i], fb0[j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (A_MODE == 1)
        fa1[i] ^= flip;
      if (decltype(RS)::value)
        rsp[i] += frag_rowsum(fa1[i]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa1[i], fb1[j], acc[i][j], 0, 0, 0);
    lds_barrier();
  };
  auto k_loop = [&](auto RS) {
    int kt = 0;
    while (true) {
      k_step(0, ra1, rb1, kclamp(kt + 3), RS);
      if (++kt >= KT)
        break;
      k_step(1, ra0, rb0, kclamp(kt + 3), RS);
      if (++kt >= KT)
        break;
    }
  };
  if (need_rs)
    k_loop(std::true_type{});
  else
    k_loop(std::false_type{});
  gemm_epilogue<TM, TN, A_MODE, EPI>(
      acc, rsp, m0 + wm * WTM, n0 + wn * WTN, M, N, K, ep);
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
// LDS holds a ring of three stages (A tile + Bp tile of one 64-byte K step
// each; the A tile in the XOR-swizzled row layout, the Bp tile as it is in
// global memory).  In step k a wave
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
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  // 2 x 2 waves, each a 64 x (BN/2) tile.
  constexpr int BM = 128, WTM = 64, WTN = BN / 2, TM = 2, TN = WTN / 32;
  static_assert(BN == 128 || BN == 64, "tile width");
  constexpr int STAGE = (BM + BN) * BK;
  constexpr int CB = BN / 64;      // Bp copies per wave and step
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

  // Copy addressing.  Copy instruction j of the A tile fills LDS bytes
  // [j*1024, (j+1)*1024): lane -> row j*16 + lane/4, chunk position lane%4,
  // which holds chunk (lane%4) ^ ((row/4)%4) = (lane%4) ^ ((lane/16)%4) of the
  // row.  Copy instruction c of the Bp tile moves KiB c of the stage, which
  // is (column tile c/2, half step c%2), unchanged.  A wave issues copies
  // 2*wave, 2*wave+1 of A and CB consecutive copies of Bp.
  const int KT = Kpad / BK;
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
    const int c = wave * CB + h;
    gb[h] = Bp + (int64_t)((n0 >> 5) + (c >> 1)) * KT * 2048 + (c & 1) * 1024 +
            lane * 16;
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
      __builtin_amdgcn_global_load_lds((glb_ptr)(gb[h] + k0 * 32),
          (lds_ptr)(base + BM * BK + (wave * CB + h) * 1024), 16, 0, 0);
  };

  // Operand addressing: sub-step s (0,1) of a stage uses chunk 2*s + lane/32 of
  // row (wave tile row + lane%32); MFMA tile i adds 32 rows = 2048 bytes.
  const unsigned sm_base = (unsigned)(uintptr_t)(lds_ptr)sm;
  unsigned ra[2], rb[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    ra[s] = sm_base + lds_off(wm * WTM + l32, s * 2 + lh);
    rb[s] = sm_base + BM * BK + ((wn * TN * 2 + s) * 64 + lane) * 16;
  }

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

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

  const bool need_rs = ep.need_rowsum;
  int32_t rsp[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
    rsp[i] = 0;

  int stage = 0; // kt % NSTAGE
  // Whether row sums of A are needed is fixed here, outside the loop, so that
  // the loop body has no branch.
  auto k_loop = [&](auto RS) {
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
      if (decltype(RS)::value) {
  #pragma unroll
        for (int i = 0; i < TM; ++i)
          rsp[i] += frag_rowsum(fa0[i]);
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
      if (decltype(RS)::value) {
  #pragma unroll
        for (int i = 0; i < TM; ++i)
          rsp[i] += frag_rowsum(fa1[i]);
      }
  #pragma unroll
      for (int i = 0; i < TM; ++i)
  #pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
              fa1[i], fb1[j], acc[i][j], 0, 0, 0);
      stage = (stage == NSTAGE - 1) ? 0 : stage + 1;
    }
  };
  if (need_rs)
    k_loop(std::true_type{});
  else
    k_loop(std::false_type{});
  // Copies past the last step are still landing in LDS; nothing reads them,
  // but the block must not release its LDS before they are done.
  __builtin_amdgcn_s_waitcnt(0x0F70);

  gemm_epilogue<TM, TN, A_MODE, EPI>(
      acc, rsp, m0 + wm * WTM, n0 + wn * WTN, M, N, K, ep);
}

// ---- GEMM, Bp streamed to registers -----------------------------------------
// The right-hand side is stored in exactly the order the matrix cores consume
// it: the operand of column tile nt, K step ks, half step sub is one
// contiguous KiB, 16 bytes per lane.  The four waves of a block sit side by
// side along N; each owns 32*TN columns that no other wave needs and loads
// their operands from Bp straight into registers, D steps ahead.  Only the A
// tile, which all four waves share, goes through LDS, and it gets there
// without passing through registers (see k_gemm_i8_dma).  Per K step a block
// therefore moves half as many bytes into LDS as that kernel, and the copy
// path into LDS is what bounds it.
//
// PIPE (needs NST >= 4) reads the operands of each half step one half step
// early, see the loop.
//
// Per step, in this order (so that the explicit wait below can count):
//   wait for own A copies of this step, barrier
//   LDS reads of the A operands (both half steps), MFMAs of half step 0,
//   refill its Bp registers for step +D, MFMAs of half step 1, refill,
//   A copies for step +NST-1 into the stage that was read in the last step.
template <int TM, int TN, int D, int NST, int MINB, bool PIPE, int A_MODE,
    int EPI, bool RS>
__global__ __launch_bounds__(256, MINB) void k_gemm_i8_bs(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
    int K, int Kpad, EpiParams ep, int tiles_m, int tiles_n) {
  constexpr int BM = 32 * TM, BN = 4 * 32 * TN;
  constexpr int STAGE = BM * BK;
  constexpr int CA = BM / 64; // A copies (1 KiB each) per wave and step
  static_assert(BM % 64 == 0, "tile height");
  // The only depths this kernel has been validated with on the device.
  static_assert(NST == 4 && D == 4, "stages");
  __shared__ __attribute__((aligned(1024))) uint8_t sm[NST * STAGE];

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
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int ncol0 = n0 + wave * 32 * TN;

  const int KT = Kpad / BK;
  const int klast = KT - 1;
  auto sclamp = [&](int step) { return step < KT ? step : klast; };

  // A copies: copy j of a step fills LDS bytes [j*1024, (j+1)*1024) of the
  // stage, lane -> row j*16 + lane/4, holding chunk (lane%4) ^ ((lane/16)%4).
  const int crow = lane >> 2;
  const int cchunk = (lane & 3) ^ ((lane >> 4) & 3);
  // Scalar base (tile origin + K step) plus a 32-bit lane offset that does not
  // change from step to step: no vector address arithmetic in the loop.
  const uint8_t *const abase = A + (int64_t)m0 * K;
  uint32_t ga[CA];
#pragma unroll
  for (int h = 0; h < CA; ++h) {
    const int r = (wave * CA + h) * 16 + crow;
    const int rc = (m0 + r < M) ? r : M - 1 - m0; // rows past M: never stored
    ga[h] = (uint32_t)rc * (uint32_t)K + (uint32_t)cchunk * 16u;
  }
  typedef __attribute__((address_space(3))) void *lds_ptr;
  typedef const __attribute__((address_space(1))) void *glb_ptr;
  auto copy_a = [&](int step, int stage) {
    uint8_t *base = sm + stage * STAGE + wave * CA * 1024;
    const uint8_t *const src = scalar_ptr(abase + step * BK);
#pragma unroll
    for (int h = 0; h < CA; ++h)
      __builtin_amdgcn_global_load_lds((glb_ptr)(src + lane_offset(ga[h])),
          (lds_ptr)(base + h * 1024), 16, 0, 0);
  };

  // Bp operands of this wave's column tiles, by buffer addressing: one
  // descriptor in scalar registers, a 32-bit lane offset, and the step as a
  // scalar offset.  The loads are written as inline assembly because the
  // compiler, which cannot count memory operations across the loop's back
  // edge, would otherwise wait for every outstanding one (vmcnt(0)) before
  // the first use of these registers in each trip, draining the prefetch.  No
  // wait of their own is needed: a step's operands were requested D >= 2 steps
  // earlier, and the wait for the A copies at the top of each step covers
  // everything issued up to two steps before it.
  v4i brsrc;
  {
    const uint64_t a = (uint64_t)(Bp + (int64_t)(ncol0 >> 5) * KT * 2048);
    brsrc.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    brsrc.y = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu));
    brsrc.z = __builtin_amdgcn_readfirstlane(TN * KT * 2048); // bytes covered
    brsrc.w = 0x00020000; // raw buffer, 32-bit elements
  }
  int boff[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
    boff[j] = j * KT * 2048 + lane * 16;
  auto load_b = [&](int step, int sub, v4i(&fb)[TN]) {
    const int soff = step * 2048 + sub * 1024;
#pragma unroll
    for (int j = 0; j < TN; ++j)
      asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"
                   : "=v"(fb[j])
                   : "v"(boff[j]), "s"(brsrc), "s"(soff)
                   : "memory");
  };

  // A operand reads: half step s uses chunk 2*s + lane/32 of row lane%32 of
  // MFMA row tile i (2048 bytes apart).
  const unsigned sm_base = (unsigned)(uintptr_t)(lds_ptr)sm;
  unsigned ra[2];
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2)
    ra[s2] = sm_base + lds_off(l32, s2 * 2 + lh);
  auto lds_read = [](v4i &f, unsigned addr, auto off) {
    asm volatile("ds_read_b128 %0, %1 offset:%2"
                 : "=v"(f)
                 : "v"(addr), "n"(decltype(off)::value)
                 : "memory");
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  // Prologue: A of steps 0..NST-2 on their way into stages 0..NST-2, then Bp
  // of steps 0..D-1 into the D register sets.
#pragma unroll
  for (int p2 = 0; p2 < NST - 1; ++p2)
    copy_a(sclamp(p2), p2);
  v4i bs[D][2][TN];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    load_b(sclamp(u), 0, bs[u][0]);
    load_b(sclamp(u), 1, bs[u][1]);
  }
  __builtin_amdgcn_sched_barrier(0);

  // Memory operations a wave issues per step, and how many of them are
  // younger than the A copies it has to wait for at the top of a step.  The A
  // copies are the last operations of a step, so those of step k were
  // followed by NST-2 whole steps when step k starts.  The first steps have
  // issued more (the prologue), never fewer.
  constexpr int PER_STEP = CA + 2 * TN;
  constexpr int AHEAD = PIPE ? 1 : 0; // PIPE waits for the copies of step k+1
  constexpr int YOUNGER = (NST - 2 - AHEAD) * PER_STEP;
  static_assert(YOUNGER < 64 && NST - 2 - AHEAD >= 0 && D >= NST - 2,
      "wait count");
  // Step 0: the prologue asks for the rows of NST - 1 steps first and for the
  // weights after them, so the weights of step 0 are followed by those of the
  // other D - 1 steps only, and the first wait must not let more than that
  // many operations stand.  (An instantiation with six stages and D = 4 did:
  // it multiplied with registers whose loads were still in flight.)
  static_assert(2 * TN * (D - 1) >= YOUNGER, "step 0 would not wait for its weights");
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080,
      (int)0x80808080};
  using O = std::integral_constant<int, 0>;

  // RS: row sums of A are needed (B carries an offset); a template argument
  // so that the loop body has no branch.
  constexpr bool need_rs = RS;
  int32_t rsp[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
    rsp[i] = 0;

  int kt = 0;
  int stage = 0;
  bool done = false;
  if constexpr (!PIPE) {
    while (!done) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        __builtin_amdgcn_s_waitcnt(
            0x0F70 | (YOUNGER & 15) | ((YOUNGER >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const unsigned soff = (unsigned)(stage * STAGE);
        v4i fa0[TM], fa1[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          lds_read(fa0[i], ra[0] + soff + i * 2048, O{});
#pragma unroll
        for (int i = 0; i < TM; ++i)
          lds_read(fa1[i], ra[1] + soff + i * 2048, O{});
        // first half landed (reads complete in order); the empty statements
        // make the registers count as written here, after the wait
        asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(TM) : "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i)
          asm volatile("" : "+v"(fa0[i]));
        if (A_MODE == 1) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa0[i] ^= flip;
        }
        if (need_rs) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            rsp[i] += frag_rowsum(fa0[i]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                fa0[i], bs[u][0][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_b(sclamp(kt + D), 0, bs[u][0]);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i)
          asm volatile("" : "+v"(fa1[i]));
        if (A_MODE == 1) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa1[i] ^= flip;
        }
        if (need_rs) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            rsp[i] += frag_rowsum(fa1[i]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                fa1[i], bs[u][1][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_b(sclamp(kt + D), 1, bs[u][1]);
        __builtin_amdgcn_sched_barrier(0);
        // The stage read in the previous step is free: every wave passed this
        // step's barrier after finishing those reads.
        copy_a(sclamp(kt + NST - 1), stage == 0 ? NST - 1 : stage - 1);
        __builtin_amdgcn_sched_barrier(0);
        stage = (stage == NST - 1) ? 0 : stage + 1;
        if (++kt >= KT) {
          done = true;
          break;
        }
      }
    }
  } else {
    // Software-pipelined operand reads: the barrier at the top of step k
    // publishes stage k+1, so the first-half operands of step k+1 can be read
    // while the second-half MFMAs of step k run, and the second-half operands
    // of step k while its first-half MFMAs run.  No MFMA waits on an LDS read
    // issued just before it.
    {
      constexpr int P0 = (NST - 2) * CA + 2 * D * TN; // younger than step 0's
      static_assert(P0 < 64, "wait count");
      __builtin_amdgcn_s_waitcnt(0x0F70 | (P0 & 15) | ((P0 >> 4) << 14));
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    v4i fa0[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
      lds_read(fa0[i], ra[0] + i * 2048, O{});
    while (!done) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        __builtin_amdgcn_s_waitcnt(
            0x0F70 | (YOUNGER & 15) | ((YOUNGER >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const unsigned soff = (unsigned)(stage * STAGE);
        const int nstage = (stage == NST - 1) ? 0 : stage + 1;
        const unsigned noff = (unsigned)(nstage * STAGE);
        v4i fa1[TM], fn0[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          lds_read(fa1[i], ra[1] + soff + i * 2048, O{});
        // the first-half operands were requested a step ago
        asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(TM) : "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i)
          asm volatile("" : "+v"(fa0[i]));
        if (A_MODE == 1) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa0[i] ^= flip;
        }
        if (need_rs) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            rsp[i] += frag_rowsum(fa0[i]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                fa0[i], bs[u][0][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_b(sclamp(kt + D), 0, bs[u][0]);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i)
          asm volatile("" : "+v"(fa1[i]));
#pragma unroll
        for (int i = 0; i < TM; ++i)
          lds_read(fn0[i], ra[0] + noff + i * 2048, O{});
        if (A_MODE == 1) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa1[i] ^= flip;
        }
        if (need_rs) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            rsp[i] += frag_rowsum(fa1[i]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                fa1[i], bs[u][1][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_b(sclamp(kt + D), 1, bs[u][1]);
        __builtin_amdgcn_sched_barrier(0);
        copy_a(sclamp(kt + NST - 1), stage == 0 ? NST - 1 : stage - 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa0[i] = fn0[i];
        stage = nstage;
        if (++kt >= KT) {
          done = true;
          break;
        }
      }
    }
    // the operands requested for the step after the last one
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
  }
  // A copies past the last step are still landing in LDS.
  __builtin_amdgcn_s_waitcnt(0x0F70);

  gemm_epilogue<TM, TN, A_MODE, EPI, kAuxThrough>(
      acc, rsp, m0, ncol0, M, N, K, ep);
}

// ---- skinny GEMM (M <= 64): weight streaming -------------------------------
// With few rows the product is bound by reading the weights once (32 rows
// per MFMA row tile, TR = 1 or 2 tiles against the same Bp operands), so
// the kernel is organised around keeping many KiB of Bp in flight per CU and
// nothing else: a block owns one 32-column tile, whose operands for all of K
// are one contiguous run of Bp (2 KiB per K step); its 8 waves take
// contiguous slices of K, and every Bp load is a fully coalesced KiB.  A (at
// most 32 rows, zero rows above M) is read from L2 in operand layout.  The
// eight partial 32x32 results are summed through LDS.  No LDS staging, no
// barrier in the K loop.
//
// DQ: the activation arrives as f32 X[M,K] (at most kSkinnyDqBytes elements)
// and every block quantizes it itself, exactly as DynamicQuantizeLinear
// would: minimum and maximum over all of X, scale and zero point from them,
// the 8-bit values minus 128 into LDS, from where the K loop takes its A
// operands.  That is 16 KiB of reads from L2 per block for one row of 4096,
// in place of a launch of its own in front of this one.  Whole layer with
// 4096 x 11008 weights, this kernel against DynamicQuantizeLinear (5.4 us by
// itself at these sizes) in front of it: 1 row 8.9 / 10.6 us, 4 rows 10.7 /
// 12.9, 5 rows 11.7 / 13.5, 6 rows 12.9 / 13.6, 8 rows 15.2 / 13.9: the cost
// grows with every row that every block reads.  With the four-instruction
// quotient the same comparison reads 4 rows 9.7 / 12.4, 6 rows 10.4 / 12.5,
// 8 rows 11.2 / 12.6, 16 rows 14 / 13.2: the limit is eight rows of 4096.
// Requesting the first Bp operands before the rows are quantized did
// not shorten it, and neither did rows K + 16 bytes apart in LDS (no two
// lanes' 16-byte reads in the same banks): 4 rows 10.7 -> 11.7 us, 8 rows
// 15.2 -> 17.1 us with the index arithmetic that takes.
//
// Tried and dropped: one launch in which the first blocks of the grid quantize
// X between them (8192 elements each), publish the result through global
// memory, and every block waits for it with all its weights already
// requested.  While the 45 MB weight stream saturates HBM every dependent
// memory step of that chain -- the load of X, the exchange of minima and
// maxima, the acknowledgement of the quantized rows, the "done" exchange, the
// copy of the rows into LDS, the polling wave's own weights -- takes 1.2 to
// 2 us: 16 rows 15.0 us (rows seen at 8.0 us, K loop over at 11.4 us), 4 rows
// 12.5 us, 1 row 11.8 us, all slower than what they would replace.
constexpr int kSkinnyDqBytes = 32768;
// Whether k_gemm_i8_skinny_bp can quantize this activation itself (DQ).
bool skinny_quantizes_rows(int64_t M, int64_t K, const void *x) {
  return M >= 1 && M <= 32 && K > 0 && K % 16 == 0 &&
         M * K <= kSkinnyDqBytes && ((((uintptr_t)x) & 15) == 0);
}

// DQ: 0, or the float4 of X a thread takes when the block quantizes X itself
// (4, 8 or 16: up to 8192, 16384 or kSkinnyDqBytes elements).
template <int A_MODE, int EPI, int DQ, int TR, bool STG>
__global__ __launch_bounds__(512) void k_gemm_i8_skinny_bp(
    const uint8_t *__restrict__ A, const float *__restrict__ X,
    const int8_t *__restrict__ Bp, int M, int N, int K, int Kpad,
    EpiParams ep) {
  // TR row tiles of 32 (M <= 32 * TR); with two of them a wave keeps half as
  // many K steps in flight, to stay within the same registers.
  constexpr int WAVES = 8, U = (TR == 1) ? 4 : 2;
  static_assert(!DQ || A_MODE == 2, "quantized rows are stored minus 128");
  static_assert(TR == 1 || (TR == 2 && !DQ), "row tiles");
  static_assert(!(DQ && STG), "quantized rows are in LDS already");
  // STG: A rows from global memory pass through a piece of LDS private to
  // the wave: a load instruction takes whole rows of the batch of U steps (CPR
  // 16-byte chunks each, so every cache line it touches is used completely),
  // the MFMA operands -- 32 bytes of each of 32 rows -- are read back from
  // there.  Loading the operands straight from global memory touches 32
  // lines per instruction for 32 bytes each, and the eight waves' lines do
  // not stay in the CU's cache until their other three quarters are wanted
  // (K=4096 N=11008, 32 rows: 12.6 us that way, 9.1 us with loads of whole
  // lines).  Rows lie CPR * 16 + 16 bytes apart in LDS, which spreads the
  // rows of one operand read over the banks.  Up to 4 rows the direct loads
  // are kept: the lanes of the rows that are not there fetch nothing, and
  // the way through LDS costs more than it saves (1 row 7.7 against 8.3 us,
  // 4 rows 8.1 / 8.4, 16 rows 9.4 / 8.7, 32 rows 12.6 / 9.6).
  constexpr int CPR = U * 4;
  constexpr int kPitch = CPR * 16 + 16;
  constexpr int kStageWave = 32 * TR * kPitch;
  constexpr int kPartBytes = WAVES * 16 * 64 * 4;
  constexpr int kLdsBytes = (STG && WAVES * kStageWave > kPartBytes)
                                ? WAVES * kStageWave
                                : kPartBytes;
  // The staged rows, and the rows quantized here (DQ), share the memory of
  // the partial sums, which are not written before every wave has left the
  // K loop.
  __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kLdsBytes];
  int32_t(*const part)[16][64] = (int32_t(*)[16][64])lds_raw;
  __shared__ int32_t part_rs[WAVES][64];
  static_assert(kPartBytes >= kSkinnyDqBytes, "quantized rows fit");
  uint8_t *const aq = lds_raw;
  __shared__ float s_lo[WAVES], s_hi[WAVES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int nt = blockIdx.x;

  const int KT = Kpad / BK;
  const int per = (KT + WAVES - 1) / WAVES;
  const int kt_begin = wave * per;
  const int kt_end = (kt_begin + per < KT) ? kt_begin + per : KT;

  float dq_scale = 0.0f;
  int32_t dq_zp = 0;
  if (DQ) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int NV = DQ > 0 ? DQ : 1; // float4 per thread
    static_assert(DQ * 4 * WAVES * 64 <= kSkinnyDqBytes, "quantized rows fit");
    const int nvec = (M * K) >> 2; // K % 16 == 0, M * K <= kSkinnyDqBytes
    const f4 *__restrict__ x4 = (const f4 *)X;
    f4 v[NV];
    float lo = __builtin_inff(), hi = -__builtin_inff();
    const float nan = __builtin_nanf(""); // neutral for minnum / maxnum
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = j * (WAVES * 64) + tid;
      v[j] = e < nvec ? x4[e] : (f4){nan, nan, nan, nan};
      lo = __builtin_fminf(__builtin_fminf(lo, v[j].x),
          __builtin_fminf(__builtin_fminf(v[j].y, v[j].z), v[j].w));
      hi = __builtin_fmaxf(__builtin_fmaxf(hi, v[j].x),
          __builtin_fmaxf(__builtin_fmaxf(v[j].y, v[j].z), v[j].w));
    }
    if (ep.x_limits) { // (the same for every thread) known from the layer before
      lo = ep.x_limits[0];
      hi = ep.x_limits[1];
    } else {
      lo = wave_min(lo);
      hi = wave_max(hi);
      if (lane == 0) {
        s_lo[wave] = lo;
        s_hi[wave] = hi;
      }
      __syncthreads();
      lo = s_lo[0];
      hi = s_hi[0];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        lo = __builtin_fminf(lo, s_lo[w]);
        hi = __builtin_fmaxf(hi, s_hi[w]);
      }
    }
    float zpf;
    dynamic_params(lo, hi, dq_scale, zpf);
    dq_zp = (int32_t)(uint32_t)zpf;
    const float recip = 1.0f / dq_scale;
    auto quantize = [&](auto fast_c) {
      constexpr bool FAST = decltype(fast_c)::value;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int e = j * (WAVES * 64) + tid;
        if (e < nvec) {
          const uint32_t q = quant_pack4<false, true, FAST>(v[j].x, v[j].y,
              v[j].z, v[j].w, dq_scale, dq_scale, dq_scale, dq_scale, recip,
              recip, recip, recip, zpf, zpf, zpf, zpf);
          ((uint32_t *)aq)[e] = q ^ 0x80808080u;
        }
      }
    };
    if (scale_is_tame(dq_scale)) // the same for every thread
      quantize(std::true_type{});
    else
      quantize(std::false_type{});
    __syncthreads();
  }

  bool row_ok[TR];
  const uint8_t *__restrict__ ap[TR];
#pragma unroll
  for (int t = 0; t < TR; ++t) {
    row_ok[t] = t * 32 + l32 < M;
    ap[t] = (DQ ? (const uint8_t *)aq : A) +
            (int64_t)(row_ok[t] ? t * 32 + l32 : 0) * K;
  }
  const int8_t *__restrict__ bp = Bp + (int64_t)nt * KT * 2048 + lane * 16;
  constexpr int kFill = (A_MODE == 1) ? (int)0x80808080 : 0;

  v16i acc[TR];
#pragma unroll
  for (int t = 0; t < TR; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      acc[t][r] = 0;
  const bool need_rs = ep.need_rowsum;
  int32_t rsp[TR]; // this lane's share of rowsum(A') of row t*32 + lane % 32
#pragma unroll
  for (int t = 0; t < TR; ++t)
    rsp[t] = 0;
  for (int kt = kt_begin; kt < kt_end; kt += U) {
    v4i a[TR][U][2], b[U][2];
    constexpr int RPI = 64 / CPR;       // rows per load instruction
    constexpr int NLD = 32 * TR / RPI;  // load instructions per batch
    v4i ar[NLD];
    if (STG) {
      const int ld_chunk = lane % CPR;
      const int step = kt + ld_chunk / 4;
      const int k0 = step * BK + (ld_chunk & 3) * 16;
      const bool k_in = step < kt_end && k0 < K; // K % 16 == 0: a chunk is in or out
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        const int row = j * RPI + lane / CPR;
        const bool in = k_in && row < M;
        ar[j] = *(const v4i *)(A + (in ? (int64_t)row * K + k0 : 0));
        if (!in)
          ar[j] = (v4i){kFill, kFill, kFill, kFill};
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // steps past this wave's slice reload its last step and are discarded
      const int s = (kt + u < kt_end) ? kt + u : kt_end - 1;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        if (!STG) {
          const int k0 = s * BK + (sub * 2 + lh) * 16;
#pragma unroll
          for (int t = 0; t < TR; ++t) {
            const bool in = row_ok[t] && k0 < K;
            a[t][u][sub] = *(const v4i *)(ap[t] + (in ? k0 : 0));
            if (!in)
              a[t][u][sub] = (v4i){kFill, kFill, kFill, kFill};
          }
        }
        b[u][sub] = *(const v4i *)(bp + (int64_t)s * 2048 + sub * 1024);
      }
    }
    if (STG) {
      // Through the wave's own piece of LDS into operand order.  The LDS
      // instructions of a wave execute in order; the fences keep the compiler
      // from moving the reads above the writes of other lanes, and the next
      // batch's writes above these reads.
      uint8_t *const stg = lds_raw + wave * kStageWave;
#pragma unroll
      for (int j = 0; j < NLD; ++j)
        *(v4i *)(stg + (j * RPI + lane / CPR) * kPitch + (lane % CPR) * 16) =
            ar[j];
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
          for (int t = 0; t < TR; ++t)
            a[t][u][sub] = *(const v4i *)(stg + (t * 32 + l32) * kPitch +
                                          (u * 4 + sub * 2 + lh) * 16);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (kt + u < kt_end) {
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
          for (int t = 0; t < TR; ++t) {
            v4i av = a[t][u][sub];
            if (A_MODE == 1)
              av ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
                  (int)0x80808080};
            if (need_rs)
              rsp[t] += frag_rowsum(av);
            acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                av, b[u][sub], acc[t], 0, 0, 0);
          }
        }
      }
    }
  }
  __syncthreads(); // every wave is done reading its rows from LDS

  // 32x32 accumulator layout: lane holds column (lane & 31); register r holds
  // row 8*(r/4) + 4*(lane/32) + r%4.  Thread t finishes elements (r, lane)
  // with r = t / 64 and r + 8.
  constexpr bool A_OFF = (A_MODE != 0);
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = ep.b_unsigned ? 128 : 0;
  const int n = nt * 32 + l32;
  const bool col_ok = n < N;
  const int nc = col_ok ? n : 0; // columns past N: computed on column 0, not stored
  int32_t db = ob;
  if (ep.b_zp_len > 0)
    db = ob - load_zp_i32(ep.b_zp, ep.b_unsigned, ep.b_zp_len > 1 ? nc : 0);
  const int32_t cs = ep.colsum[nc];
  float sj = 0.0f, bj = -0.0f;
  int32_t yz = 0;
  if (EPI == kEpiF32 && ep.bias != nullptr)
    bj = ep.bias[ep.bias_len > 1 ? nc : 0];
  if (EPI != kEpiI32) {
    sj = (DQ ? dq_scale : ep.a_scale[0]) *
         ep.b_scale[ep.b_scale_len == 1 ? 0 : nc];
    if (EPI == kEpiQ8) {
      sj = sj / ep.y_scale[0];
      yz = load_zp_i32(ep.y_zp, ep.y_unsigned, 0);
    }
  }
  // One row tile at a time through the partial-sum buffers.
#pragma unroll
  for (int t = 0; t < TR; ++t) {
    if (t > 0)
      __syncthreads(); // the sums of the tile before have been read
#pragma unroll
    for (int r = 0; r < 16; ++r)
      part[wave][r][lane] = acc[t][r];
    part_rs[wave][lane] = rsp[t];
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = (tid >> 6) + h * 8;
      const int ml = 8 * (r >> 2) + 4 * lh + (r & 3); // row within the tile
      const int m = t * 32 + ml;
      if (m >= M || !col_ok)
        continue;
      uint32_t y = 0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w)
        y += (uint32_t)part[w][r][lane];
      int32_t da = oa, rs = 0;
      if (DQ)
        da = oa - dq_zp;
      else if (ep.a_zp_len > 0)
        da = oa - load_zp_i32(ep.a_zp, A_OFF, ep.a_zp_len > 1 ? m : 0);
      if (need_rs) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w)
          rs += part_rs[w][ml] + part_rs[w][ml + 32];
      }
      y += (uint32_t)da * (uint32_t)cs;
      y += (uint32_t)db * (uint32_t)rs;
      y += (uint32_t)K * (uint32_t)da * (uint32_t)db;
      store_one<EPI>(ep, (int64_t)m * N + n, y, sj, yz, bj);
    }
  }
}

// ---- pack B ---------------------------------------------------------------
// One block transposes a 64(k) x 64(n) tile of B [K,N] through LDS, writes it
// in MFMA operand order (see the top of the file) and adds the tile's column
// sums into colsum with int32 atomics (integer adds commute, so the result
// does not depend on arrival order).
constexpr int PT = 64;

template <bool B_UNSIGNED>
__global__ __launch_bounds__(256) void k_pack_b(const uint8_t *__restrict__ B,
    int64_t K, int64_t N, int KT, int8_t *__restrict__ Bp,
    int32_t *__restrict__ colsum) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[PT][PT + 4];
  const int ks = blockIdx.y; // K step of 64
  const int64_t k0 = (int64_t)ks * PT;
  const int64_t n0 = (int64_t)blockIdx.x * PT;
  const int tid = threadIdx.x;
  // Read: thread -> row k = tid/4, 16 columns starting at (tid%4)*16.
  {
    const int kr = tid >> 2;
    const int nc = (tid & 3) * 16;
    const int64_t k = k0 + kr;
    // Rows that start on 16-byte boundaries (N % 16 == 0, aligned B): one
    // 16-byte load per thread; otherwise, and at the edges, byte by byte.
    const bool rows_aligned = ((N & 15) == 0) && ((((uintptr_t)B) & 15) == 0);
    if (rows_aligned && k < K && n0 + nc + 16 <= N) {
      v4i q = *(const v4i *)(B + k * N + n0 + nc);
      if (B_UNSIGNED)
        q ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080,
            (int)0x80808080};
      // row stride 68 and nc % 16 == 0: 4-byte aligned
      uint32_t *dst = (uint32_t *)&tile[kr][nc];
      dst[0] = (uint32_t)q.x;
      dst[1] = (uint32_t)q.y;
      dst[2] = (uint32_t)q.z;
      dst[3] = (uint32_t)q.w;
    } else {
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
  }
  __syncthreads();
  // Write: thread -> column n = tid/4, 16-byte chunk c = tid%4 of the step.
  {
    const int nr = tid >> 2;
    const int c = tid & 3;
    uint32_t w[4] = {0, 0, 0, 0};
    int32_t sum = 0;
#pragma unroll
    for (int b = 0; b < 16; ++b) {
      const uint8_t v = tile[c * 16 + b][nr];
      sum += (int32_t)(int8_t)v;
      w[b >> 2] |= (uint32_t)v << ((b & 3) * 8);
    }
    const int64_t n = n0 + nr;
    // The grid covers [Npad, Kpad] exactly: every byte of Bp is written.
    const int64_t o =
        ((((n >> 5) * KT + ks) * 2 + (c >> 1)) * 64 + (c & 1) * 32 + (n & 31)) *
        16;
    *(v4i *)(Bp + o) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    // Fold the four k-chunks of this column (lanes 4n..4n+3) before the atomic.
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    if ((tid & 3) == 0 && sum != 0)
      atomicAdd(&colsum[n], sum);
  }
}

// ---- launch ---------------------------------------------------------------

// Kernel / tile configurations.
enum TileCfg : int {
  kT128x128 = 0, // k_gemm_i8: register-staged tiles (and the general path)
  kD128x128 = 1, // k_gemm_i8_dma: tiles copied straight into LDS
  kB128x256 = 2, // k_gemm_i8_bs: Bp straight into registers
  kD128x64 = 3,  // k_gemm_i8_dma with 128 x 64 tiles
  kW128x384 = 4, // k_gemm_i8_wreg: weights in registers, 12 waves of 32 columns
  kFlight = 5,   // k_gemm_i8_flight: one round of blocks, all operands requested at once
  kNumCfg = 6
};

// Kernel choice for problems with more than 32 rows, K % 64 == 0 and a
// 16-byte aligned A (anything else takes the general path of k_gemm_i8).
// Measured on MI355X over the BERT-base and Llama-7B layer shapes and square
// problems up to 8192: a 128 x 256 tile of k_gemm_i8_bs costs about 1.7 times
// a 128 x 128 tile of k_gemm_i8_dma, so it wins when it needs at most half as
// many rounds over the 256 CUs and fills at least one round.  When 128 x 128
// tiles cover at most half the CUs, 128 x 64 tiles spread the work over twice
// as many (512x1024x4096: 10.1 -> 8.8 us); with 192 tiles for 256 CUs the
// half-width tiles lose (4096x768x768 7.2 -> 7.6 us, 4096x3072x768 18.6 ->
// 19.4 us).
// Override for tests and tuning: OM_MI355X_GEMM_TILE=<TileCfg value>.
int choose_tile(int64_t M, int64_t N, int64_t K) {
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (force && force[0]) {
    const int c = atoi(force);
    if (c >= 0 && c < kNumCfg)
      return c;
  }
  const int64_t tm = (M + 127) / 128;
  const int64_t t128 = tm * ((N + 127) / 128);
  const int64_t t256 = tm * ((N + 255) / 256);
  const int64_t r128 = (t128 + 255) / 256, r256 = (t256 + 255) / 256;
  // (k_gemm_i8_bs only with whole trips of its four-step loop body, K % 256
  // == 0: the step counts it runs with in production -- K = 2048, 4096, 11008
  // -- and is validated at.  Other K take the 128 x 128 tiles, a few percent
  // slower on such shapes.)
  if (t256 >= 256 && r256 * 17 < r128 * 10 && K % (4 * kGemmBK) == 0)
    return kB128x256;
  if (N > 64 && t128 <= 128)
    return kD128x64;
  return kD128x128;
}

bool gemm_fast_path(int64_t M, int64_t K, const void *A) {
  // K == 0 (an empty sum) has no bytes of A to read: only the general path
  // checks every address against K.
  return M > 16 && K > 0 && K % 64 == 0 && ((((uintptr_t)A) & 15) == 0);
}

// Name of the kernel the calling thread's last launch_gemm chose (for tests
// and reports).
thread_local const char *t_last_kernel = "";
// Whether that kernel applied the onnx.Gelu asked for to its results itself
// (launch_gemm runs the pass over the output when it did not).
thread_local bool t_gelu_applied = false;
// Whether that kernel wrote GemmArgs::y_limits itself (launch_gemm runs the
// reduction over the output when it did not).
thread_local bool t_limits_written = false;

template <int A_MODE, int EPI>
hipError_t gemm_launch_cfg(
    hipStream_t st, const GemmArgs &g, const EpiParams &ep, int Kpad) {
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  const uint8_t *A = (const uint8_t *)g.A;
  const int M = (int)g.M, N = (int)g.N, K = (int)g.K;
  if (g.X) {
    // rows quantized inside the kernel (the caller asked gemm_quantizes_rows)
    if (A_MODE != 2 || !gemm_quantizes_rows(g.M, g.K, g.N, g.X))
      return hipErrorInvalidValue;
    if (!skinny_quantizes_rows(g.M, g.K, g.X)) {
      // more rows than every block can quantize for itself: the blocks share
      // the minimum / maximum through the exchange slots
      if (EPI != kEpiF32 || !g.dql)
        return hipErrorInvalidValue;
      t_last_kernel = "k_gemm_i8_flight (rows quantized in the kernel)";
      t_gelu_applied = g.gelu; // this kernel applies it to its results
      t_limits_written = ep.limits.out != nullptr; // and reduces their limits
      return launch_gemm_flight_dq(st, g, ep, *g.dql);
    }
    if constexpr (A_MODE == 2) {
      t_last_kernel = "k_gemm_i8_skinny_bp (rows quantized in the kernel)";
      const dim3 grid((unsigned)((g.N + 31) / 32));
      const int64_t elements = g.M * g.K;
      if (elements <= 4 * 4 * 512)
        k_gemm_i8_skinny_bp<2, EPI, 4, 1, false>
            <<<grid, 512, 0, st>>>(nullptr, g.X, g.Bp, M, N, K, Kpad, ep);
      else if (elements <= 8 * 4 * 512)
        k_gemm_i8_skinny_bp<2, EPI, 8, 1, false>
            <<<grid, 512, 0, st>>>(nullptr, g.X, g.Bp, M, N, K, Kpad, ep);
      else
        k_gemm_i8_skinny_bp<2, EPI, 16, 1, false>
            <<<grid, 512, 0, st>>>(nullptr, g.X, g.Bp, M, N, K, Kpad, ep);
    }
    return hipGetLastError();
  }
  // Up to 64 rows the weight-streaming kernel is ahead of every tile kernel
  // (K=4096 N=11008: M=33 11.6 against 17.2 us, M=48 12.3 / 17.7; K=11008
  // N=4096 M=64: 15.0 / 37.7; K=768 N=3072 M=64: 4.2 / 6.0).
  const bool skinny_rows = g.M <= 64;
  if (skinny_rows && g.K > 0 && g.K % 16 == 0 && ((((uintptr_t)g.A) & 15) == 0) &&
      !(force && force[0])) {
    const dim3 grid((unsigned)((g.N + 31) / 32));
    t_last_kernel = "k_gemm_i8_skinny_bp";
    if (g.M <= 4)
      k_gemm_i8_skinny_bp<A_MODE, EPI, 0, 1, false>
          <<<grid, 512, 0, st>>>(A, nullptr, g.Bp, M, N, K, Kpad, ep);
    else if (g.M <= 32)
      k_gemm_i8_skinny_bp<A_MODE, EPI, 0, 1, true>
          <<<grid, 512, 0, st>>>(A, nullptr, g.Bp, M, N, K, Kpad, ep);
    else
      k_gemm_i8_skinny_bp<A_MODE, EPI, 0, 2, true>
          <<<grid, 512, 0, st>>>(A, nullptr, g.Bp, M, N, K, Kpad, ep);
    return hipGetLastError();
  }
  const int tiles_m = (int)((g.M + 127) / 128);
  const int tiles_n128 = (int)((g.N + 127) / 128);
  if (!gemm_fast_path(g.M, g.K, g.A)) {
    // Any K, any alignment of A (and the forced configurations of the tests
    // when M <= 16); byte loads only for an A of fewer than 16 bytes.
    t_last_kernel = "k_gemm_i8 (any K, any alignment)";
    if (g.M * g.K >= 16)
      k_gemm_i8<128, 128, 2, 2, 2, A_MODE, EPI, kLoadAny>
          <<<dim3((unsigned)(tiles_m * tiles_n128)), 256, 0, st>>>(
              A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n128);
    else
      k_gemm_i8<128, 128, 2, 2, 2, A_MODE, EPI, kLoadBytes>
          <<<dim3((unsigned)(tiles_m * tiles_n128)), 256, 0, st>>>(
              A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n128);
    return hipGetLastError();
  }
  const int cfg = choose_tile(g.M, g.N, g.K);
  // One round of blocks with everything requested at once: small problems,
  // where a pipelined K loop would pay the memory latency step after step
  // (512 x 1024 x 4096 QLinearMatMul: 8.2 us in 128 x 64 tiles of
  // k_gemm_i8_dma; 128 x 768 x 768: 7.0 us).
  if ((cfg == kFlight || !(force && force[0])) && flight_ok(g, A_MODE)) {
    t_last_kernel = "k_gemm_i8_flight (one round, operands requested at once)";
    t_gelu_applied = EPI == kEpiF32 && g.gelu; // this kernel applies it itself
    t_limits_written = EPI == kEpiF32 && ep.limits.out != nullptr;
    return launch_gemm_flight(st, g, ep, A_MODE);
  }
  // Weights in registers: K = 768 (the projections of a BERT-base layer)
  // when the problem fills the device with its 128 x 384 blocks.
  const bool forced = force && force[0];
  if (wreg_ok(g) && (cfg == kW128x384 || (!forced && wreg_pays(g.M, g.N)))) {
    t_last_kernel = "k_gemm_i8_wreg (weights in registers, 128x384 blocks)";
    t_gelu_applied = g.epi == kEpiF32 && g.gelu; // this kernel applies it to its results
    // (the limits of y: in the kernel for the f32 results of a fused layer)
    t_limits_written = A_MODE == 2 && EPI == kEpiF32 && ep.limits.out != nullptr;
    return launch_gemm_wreg(st, g, ep, A_MODE);
  }
  switch (cfg) {
  case kB128x256: {
    const int tiles_n = (int)((g.N + 255) / 256);
    t_last_kernel = "k_gemm_i8_bs (128x256 tiles)";
    if (ep.need_rowsum)
      k_gemm_i8_bs<4, 2, 4, 4, 2, true, A_MODE, EPI, true>
          <<<dim3((unsigned)(tiles_m * tiles_n)), 256, 0, st>>>(
              A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n);
    else
      k_gemm_i8_bs<4, 2, 4, 4, 2, true, A_MODE, EPI, false>
          <<<dim3((unsigned)(tiles_m * tiles_n)), 256, 0, st>>>(
              A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n);
    break;
  }
  case kD128x64: {
    const int tiles_n64 = (int)((g.N + 63) / 64);
    t_last_kernel = "k_gemm_i8_dma (128x64 tiles)";
    k_gemm_i8_dma<64, 3, 3, A_MODE, EPI>
        <<<dim3((unsigned)(tiles_m * tiles_n64)), 256, 0, st>>>(
            A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n64);
    break;
  }
  case kW128x384: // (forced, on a shape that kernel does not take)
  case kFlight:
  case kD128x128:
    t_last_kernel = "k_gemm_i8_dma (128x128 tiles)";
    k_gemm_i8_dma<128, 3, 3, A_MODE, EPI>
        <<<dim3((unsigned)(tiles_m * tiles_n128)), 256, 0, st>>>(
            A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n128);
    break;
  default:
    t_last_kernel = "k_gemm_i8 (128x128 tiles through registers)";
    k_gemm_i8<128, 128, 2, 2, 3, A_MODE, EPI, kLoadAligned>
        <<<dim3((unsigned)(tiles_m * tiles_n128)), 256, 0, st>>>(
            A, g.Bp, M, N, K, Kpad, ep, tiles_m, tiles_n128);
    break;
  }
  return hipGetLastError();
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

// Rows of A copied to a pitch of Kp >= K bytes, the bytes past K set to the
// row's zero point (exclusive-ored with `flip`: 0x80 for rows stored minus
// 128): an element equal to its zero point stands for the real value 0, so a
// product over the Kp bytes equals the product over the K (see
// gemm_pads_rows).  One thread per byte; at most 64 rows.
__global__ __launch_bounds__(256) void k_pad_rows(const uint8_t *__restrict__ A,
    int M, int K, int Kp, const uint8_t *__restrict__ zp, int zp_len,
    uint8_t flip, uint8_t *__restrict__ out) {
  const int r = blockIdx.y;
  const uint8_t fill =
      (uint8_t)((zp && zp_len > 0 ? zp[zp_len > 1 ? r : 0] : 0) ^ flip);
  for (int c = blockIdx.x * 256 + threadIdx.x; c < Kp; c += gridDim.x * 256)
    out[(int64_t)r * Kp + c] = c < K ? A[(int64_t)r * K + c] : fill;
}

} // namespace

// Few rows whose length is no multiple of 16 bytes, or that do not start on a
// 16-byte boundary, would fall to the tile kernels, which take several times
// as long on such shapes (16 x 4100 x 11008: 41 us against 9 us).  The
// runtime copies them to an aligned buffer with rows of round_up(K, 16) bytes
// instead, the tail of each row filled with its zero point, and multiplies
// with that K: (a - a_zp) is zero there, so the products, the row sums and the
// K * (a offset) * (b offset) term of the zero-point algebra are those of the
// original rows, bit for bit.
bool gemm_pads_rows(int64_t M, int64_t K, const void *a) {
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  return M >= 1 && M <= 64 && K >= 1 &&
         (K % 16 != 0 || ((((uintptr_t)a) & 15) != 0)) &&
         !(force && force[0]);
}

hipError_t launch_pad_rows(hipStream_t s, const void *a, int64_t M, int64_t K,
    const void *a_zp, int64_t a_zp_len, bool stored_minus_128, void *out) {
  const int64_t Kp = round_up(K, 16);
  if (M < 1 || M > 64 || Kp > INT32_MAX)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)((Kp + 1023) / 1024), (unsigned)M);
  k_pad_rows<<<grid, 256, 0, s>>>((const uint8_t *)a, (int)M, (int)K, (int)Kp,
      (const uint8_t *)a_zp, (int)a_zp_len, stored_minus_128 ? 0x80 : 0,
      (uint8_t *)out);
  return hipGetLastError();
}

hipError_t launch_pack_b(hipStream_t s, const void *B, bool b_unsigned,
    int64_t K, int64_t N, int8_t *Bp, int32_t *colsum) {
  const int64_t Kpad = round_up(K > 0 ? K : 1, kGemmBK);
  const int64_t Npad = round_up(N, kGemmBN);
  hipError_t e = launch_fill_u32(s, (uint32_t *)colsum, Npad, 0u);
  if (e != hipSuccess)
    return e;
  // kGemmBK and kGemmBN are multiples of the 64 x 64 pack tile, so the grid
  // covers [Npad, Kpad] exactly and every byte of Bp is written.
  const int KT = (int)(Kpad / kGemmBK);
  dim3 grid((unsigned)(Npad / PT), (unsigned)(Kpad / PT));
  if (b_unsigned)
    k_pack_b<true><<<grid, 256, 0, s>>>(
        (const uint8_t *)B, K, N, KT, Bp, colsum);
  else
    k_pack_b<false><<<grid, 256, 0, s>>>(
        (const uint8_t *)B, K, N, KT, Bp, colsum);
  return hipGetLastError();
}

int gemm_quantizes_rows(int64_t M, int64_t K, int64_t N, const void *x) {
  const char *force = getenv("OM_MI355X_GEMM_TILE");
  if (force && force[0])
    return 0;
  if (skinny_quantizes_rows(M, K, x))
    return 1;
  return flight_quantizes_rows(M, K, N, x) ? 2 : 0;
}

const char *last_gemm_kernel() { return t_last_kernel; }

namespace {
// onnx.Gelu (gelu_f32) in place over n floats, for the kernels that do not
// apply it to their results themselves; y 16-byte aligned or not (the edges
// go one by one).
__global__ __launch_bounds__(256) void k_gelu_inplace(float *__restrict__ y,
    int64_t n) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const int64_t head = (4 - (int64_t)((((uintptr_t)y) >> 2) & 3)) & 3; // floats before the first aligned vector
  const int64_t lead = head < n ? head : n;
  f4 *const y4 = (f4 *)(y + lead);
  const int64_t nvec = (n - lead) >> 2;
  const int64_t base = (int64_t)blockIdx.x * 512 + threadIdx.x;
  f4 v[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t i = base + j * 256;
    const f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    v[j] = i < nvec ? y4[i] : zero;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t i = base + j * 256;
    if (i < nvec) {
      f4 o;
      o.x = gelu_f32(v[j].x);
      o.y = gelu_f32(v[j].y);
      o.z = gelu_f32(v[j].z);
      o.w = gelu_f32(v[j].w);
      y4[i] = o;
    }
  }
  if (blockIdx.x == 0) {
    // up to three floats before the first vector and after the last one
    const int64_t t = threadIdx.x;
    if (t < lead)
      y[t] = gelu_f32(y[t]);
    const int64_t tail = lead + (nvec << 2) + t;
    if (t < 4 && tail < n)
      y[tail] = gelu_f32(y[tail]);
  }
}
} // namespace

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
  ep.need_rowsum = g.b_unsigned || (g.b_zp != nullptr && g.b_zp_len > 0);
  ep.colsum = g.colsum;
  ep.a_scale = g.a_scale;
  ep.b_scale = g.b_scale;
  ep.b_scale_len = g.b_scale_len;
  ep.y_scale = g.y_scale;
  ep.y_zp = g.y_zp;
  ep.bias = g.epi == kEpiF32 ? g.bias : nullptr;
  ep.bias_len = g.bias_len;
  ep.x_limits = g.X ? g.x_limits : nullptr;
  ep.limits = LimitsOut{};
  if (g.y_limits) // (slot [4] of the counters: [0] is DynamicQuantizeLinear's)
    ep.limits = LimitsOut{g.y_limits, g.dql->partial_min, g.dql->partial_max,
        g.dql->counter + 4};
  ep.floor = relu_floor(g.epi == kEpiF32 && g.relu);
  ep.out = g.out;
  ep.b_unsigned = g.b_unsigned;
  ep.y_unsigned = g.y_unsigned;
  ep.narrow = (int)g.narrow;
  const int a_mode = (g.X || g.a_preshifted) ? 2 : (g.a_unsigned ? 1 : 0);
  t_gelu_applied = false;
  t_limits_written = false;
  if (g.y_limits && (g.epi != kEpiF32 || !g.dql))
    return hipErrorInvalidValue;
  hipError_t e;
  switch (a_mode) {
  case 0:
    e = gemm_launch_epi<0>(s, g, ep, Kpad);
    break;
  case 1:
    e = gemm_launch_epi<1>(s, g, ep, Kpad);
    break;
  default:
    e = gemm_launch_epi<2>(s, g, ep, Kpad);
    break;
  }
  if (e == hipSuccess && g.epi == kEpiF32 && g.gelu && !t_gelu_applied) {
    // onnx.Gelu on the result, as a pass of its own over the f32 output
    const int64_t n = g.M * g.N;
    const int64_t per_block = 256 * 2 * 4;
    k_gelu_inplace<<<(unsigned)((n + per_block - 1) / per_block), 256, 0, s>>>(
        (float *)g.out, n);
    e = hipGetLastError();
  }
  if (e == hipSuccess && g.y_limits && !t_limits_written)
    e = launch_minmax_limits(s, *g.dql, (const float *)g.out, g.M * g.N, g.y_limits);
  return e;
}


} // namespace om
