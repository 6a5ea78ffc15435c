// int8 GEMM for gfx950 with the weights held in registers (k_gemm_i8_wreg):
// the kernel for products whose K fits a wave's registers, such as the
// K = 768 projections of a BERT-base layer.  Same arithmetic and operand
// layouts as the kernels of gemm_kernels.hip (A [M,K] row-major, Bp in MFMA
// operand order, zero-point correction in int32, epilogues fused into the
// store); see the top of that file.
//
// A wave owns one column tile (32 columns) and keeps its operands for ALL of K
// in registers: K = 768 is 96 registers per lane, loaded from Bp with 24
// perfectly coalesced KiB loads (Bp is stored in exactly that order).  The
// WAVES waves of a block sit side by side along N and walk together over NR row
// tiles of 32 rows.  A row tile for all of K is one contiguous piece of A
// (32 * K bytes, as K is the row pitch); it is copied into LDS once per block
// without passing through registers, and every wave reads its MFMA operands
// from there: the only traffic inside the K loop is one LDS read of 16 bytes
// per lane and MFMA.  With 12 waves and 4 row tiles a block makes 128 x 384
// results from 96 KB of A and 288 KB of Bp, each byte of which it moves
// exactly once: 384 KB per CU for 4096 x 768 x 3072 against 590 KB with
// 128 x 128 tiles, none of it through the slow path for operands (16-byte
// pieces of many rows per instruction).
//
// Results leave the block tile by tile while the next tile is being computed:
// the conversion and the store of the finished tile's 16 elements per lane are
// spread, one per K step, between the MFMAs of the next tile (two accumulator
// sets), so the matrix cores do not wait for the epilogue and the output is
// written in a steady stream instead of in a burst at the end.  32-bit results
// go straight to memory, a 128-byte line per row and wave.  8-bit results are
// first gathered in LDS, the whole 32 x (32 WAVES) tile of the block, and
// leave one K loop later in 16-byte pieces of whole lines, one store per
// wave and tile.
//
// A tile in LDS: row r at r * K, its 16-byte chunk c at position
// c ^ (r % 16): the lanes of an operand read (16 rows at a time, the same
// chunk of each) then fall into different banks.  The copy puts the chunks
// there by choosing which global chunk each lane fetches; its LDS side is
// linear.
//
// Order of a wave's memory operations, which the explicit waits count on
// (operations complete in the order they were issued): per-column parameters,
// the copy of row tile 0 (CPT instructions), the loads of Bp (KH), the copies
// of tiles 1..NR-1; later only stores, 16 per tile (one for 8-bit results).  "Tile u has landed" = at
// most [what was issued after its copies] operations are outstanding.  Every
// block copies and computes all NR tiles (rows past M are copies of the last
// row and are not stored), so the counts hold for every block.

#include "gemm_common.h"

namespace om {
namespace gemm {

namespace {

#ifdef WREG_TIMING
// Development build: clock readings of block 0's waves at fixed points,
// kept in registers and written out when the kernel ends.
__device__ unsigned long long wreg_ts[16 * 16];
#define WREG_TS(i) ts[i] = __builtin_readcyclecounter()
#else
#define WREG_TS(i)
#endif

// Memory operations a wave has issued after its copies of tile t + 1 when it
// waits for them in tile t, at K step WAIT_STEP: the copies of the tiles after
// that, the loads of Bp issued in tile 0 (one per step), the stores of the
// tiles before t (16 each) and those of tile t so far (one per step from
// EPI_FIRST on).  STAGED (8-bit results, gathered in LDS): one store per
// tile, issued in the tile's last step, after the wait.
template <int KH, int CPT, int NR, int B_FIRST, int WAIT_STEP, int EPI_FIRST, bool STAGED>
struct WregNeed {
  static constexpr int at(int t) {
    const int b_late = KH - B_FIRST;
    const int b_seen = t > 0 ? b_late : (WAIT_STEP < b_late ? WAIT_STEP : b_late);
    const int here = WAIT_STEP - EPI_FIRST < 16 ? WAIT_STEP - EPI_FIRST : 16;
    const int stores = t == 0 ? 0 : STAGED ? t - 1 : 16 * (t - 1) + here;
    return CPT * (NR - 2 - t) + b_seen + stores;
  }
};
// LDS operations issued between the steps `from` (after its operand read) and
// `to` (before its operand read) of a tile other than the block's first by
// the staged epilogue: one write per step from epi_first on, 16 in all, each
// at the end of its step.
constexpr int wreg_staged_writes(int from, int to, int epi_first) {
  int x = 0;
  for (int j = from; j < to; ++j)
    if (j >= epi_first && j < epi_first + 16)
      ++x;
  return x;
}
// LDS operations issued after the read for step s when step s waits for it:
// the pf reads ahead of it, the fix-up's fix_ops reads (issued in step
// fix_read) and as many writes (step fix_write) while they are among those,
// and, with `staged` (the staged epilogue, in a tile that has a finished one
// to store), its writes of the pf steps before and its read of the gathered
// tile, issued in step flush_read.
constexpr int wreg_younger(int s, int pf, int fix_ops, int fix_read, int fix_write,
    bool staged, int epi_first, int flush_read) {
  int x = pf;
  if (s >= fix_read && s < fix_read + pf)
    x += fix_ops;
  if (s >= fix_write && s < fix_write + pf)
    x += fix_ops;
  if (staged) {
    x += wreg_staged_writes(s - pf, s, epi_first);
    if (s >= flush_read && s < flush_read + pf)
      x += 1;
  }
  return x;
}

// LIM: minimum and maximum of the (f32) results are kept per lane while they
// are stored and reduced over the grid when the block ends (EpiParams::limits).
template <int KH, int WAVES, int NR, int A_MODE, int EPI, bool STREAM, int ACT,
    bool LIM = false>
__global__ __launch_bounds__(WAVES * 64, 1) void k_gemm_i8_wreg(
    const uint8_t *__restrict__ A, const int8_t *__restrict__ Bp, int M, int N,
    EpiParams ep, int regions_m, int regions_n, int bp_tiles) {
  constexpr int K = 32 * KH;
  constexpr int CPR = K / 16;           // 16-byte chunks per row of A
  constexpr int CPT = KH / WAVES;       // copy instructions per wave and tile
  constexpr int TILE_BYTES = KH * 1024; // a column tile of Bp, a row tile of A
  constexpr int PF = 3;                 // operand reads in flight
  // Operand register sets.  The read issued in step s lands on the set of
  // the MFMA issued in step s - 1, long after that MFMA has fetched its
  // operands (an LDS read takes far longer than an MFMA's operand fetch).
  constexpr int NB = PF + 1;
  constexpr int ES = (EPI == kEpiQ8) ? 1 : 4;
  constexpr int kEpiFirst = 2;          // K step in which a tile's stores begin
  // uint8 A: the bytes of a tile are turned into int8 (minus 128) in LDS, by
  // the wave that copied them, in two K steps of the tile before.
  constexpr bool FIX = (A_MODE == 1);
  constexpr int kFixRead = 12, kFixWrite = 16;
  // Loads of Bp issued before the first tile starts; the rest follow one per
  // K step of tile 0, ahead of the MFMA that needs them.
  constexpr int kBFirst = 8;
  static_assert(KH % WAVES == 0 && KH - PF >= kEpiFirst + 16 && KH % NB == 0 &&
                    CPR % 16 == 0 && KH % 8 == 0 && kFixWrite >= kFixRead + PF &&
                    kFixWrite + PF <= KH - PF && kFixRead >= kEpiFirst,
      "shape");
  constexpr int kWaitStep = FIX ? kFixRead : KH - PF;
  // 8-bit results are gathered in LDS, a 32 x (32 WAVES) tile of the block at
  // a time, and leave in whole 128-byte lines, 16 bytes a lane: a wave's own
  // part of a row is 32 bytes, and the memory system takes as long over a
  // 32-byte piece as over a line.  Two tiles: one is being filled (one byte
  // a lane and K step) while the one before it is read back and stored.
  constexpr bool STAGED = (EPI == kEpiQ8);
  constexpr int kStagePitch = 32 * WAVES + 16; // rows 4 apart: different banks
  constexpr int kStageBytes = 32 * kStagePitch;
  constexpr int kStageAt = (NR + 1) * TILE_BYTES;
  constexpr int kFlushRead = KH - PF;   // step: behind the tile's barrier
  static_assert(!STAGED || (kEpiFirst + 16 <= kFlushRead && (32 * WAVES) % 16 == 0 &&
                               kStageAt + 2 * kStageBytes <= 160 * 1024),
      "staged epilogue");
  using Need = WregNeed<KH, CPT, NR, kBFirst, kWaitStep, kEpiFirst, STAGED>;
  static_assert(kBFirst + CPT * (NR - 1) <= 63 && Need::at(NR - 2) <= 63, "counter");
  // (+ one spare tile: the reads that run ahead of the last tile's last steps)
  __shared__ __attribute__((aligned(1024)))
  uint8_t sA[(NR + 1) * TILE_BYTES + (STAGED ? 2 * kStageBytes : 0)];

#ifdef WREG_TIMING
  unsigned long long ts[16] = {};
#endif
  WREG_TS(0);
  // Block order: consecutive ids go round-robin to the 8 XCDs (each with its
  // own L2); renumbered so that an XCD gets a contiguous range, walked in
  // groups of 8 row regions: the blocks resident on an XCD share a few
  // panels of A and of Bp.
  int pid = blockIdx.x;
  {
    const int nb = gridDim.x;
    const int per = nb >> 3;
    if (per > 0 && pid < per * 8)
      pid = (pid & 7) * per + (pid >> 3);
  }
  constexpr int GROUP = 8;
  const int in_group = GROUP * regions_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int gsize = (regions_m - first_m < GROUP) ? regions_m - first_m : GROUP;
  const int rm = first_m + (pid % in_group) % gsize;
  const int rn = (pid % in_group) / gsize;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int row0 = rm * (32 * NR);       // first row of the block
  const int ct = rn * WAVES + wave;      // the wave's column tile
  const int n = ct * 32 + l32;           // the lane's column
  const int nc = n < N ? n : N - 1;

  // ---- per-column parameters: loaded first, used after the first wait -------
  constexpr bool A_OFF = (A_MODE != 0);
  const bool has_bzp = ep.b_zp_len > 0;
  const void *bzp_ptr = has_bzp ? ep.b_zp : (const void *)ep.colsum;
  const bool has_azp = ep.a_zp_len > 0;
  const void *azp_ptr = has_azp ? ep.a_zp : (const void *)ep.colsum;
  const bool has_bias = EPI == kEpiF32 && ep.bias != nullptr;
  const float *bias_ptr = has_bias ? ep.bias : (const float *)ep.colsum;
  const float *as_ptr = EPI != kEpiI32 ? ep.a_scale : (const float *)ep.colsum;
  const float *bs_ptr = EPI != kEpiI32 ? ep.b_scale : (const float *)ep.colsum;
  const float *ys_ptr = EPI == kEpiQ8 ? ep.y_scale : (const float *)ep.colsum;
  const void *yz_ptr = EPI == kEpiQ8 ? ep.y_zp : (const void *)ep.colsum;
  const float raw_as = as_ptr[0];
  const float raw_bs = bs_ptr[(EPI != kEpiI32 && ep.b_scale_len > 1) ? nc : 0];
  const float raw_ys = ys_ptr[0];
  const int32_t raw_yz = load_zp_i32(yz_ptr, ep.y_unsigned, 0);
  const int32_t raw_az = load_zp_i32(azp_ptr, A_OFF, 0);
  const int32_t raw_bz =
      load_zp_i32(bzp_ptr, ep.b_unsigned, ep.b_zp_len > 1 ? nc : 0);
  const int32_t raw_cs = ep.colsum[nc];
  const float raw_bias = bias_ptr[has_bias && ep.bias_len > 1 ? nc : 0];
  __builtin_amdgcn_sched_barrier(0);

  // ---- copies of A into LDS, loads of Bp into registers --------------------
  typedef __attribute__((address_space(3))) void *lds_ptr;
  // Copy instruction j of a tile fills LDS chunks [64 j, 64 j + 64): chunk q is
  // position q % CPR of row q / CPR and holds chunk (q % CPR) ^ (row % 16).
  // (A buffer load, not a global one: the compiler takes a global load into
  // LDS for an operation that may complete out of order with everything else
  // and from then on waits for ALL outstanding memory operations wherever it
  // waits for one, which the loads of Bp in tile 0 make it do.)
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(A), 0, (int)((uint32_t)M * (uint32_t)K), 0x00020000);
  auto copy_tile = [&](int t) {
#pragma unroll
    for (int jj = 0; jj < CPT; ++jj) {
      const int q = 64 * (wave * CPT + jj) + lane;
      const int r = q / CPR;
      const int c = (q % CPR) ^ (r & 15);
      int row = row0 + t * 32 + r;
      row = row < M ? row : M - 1; // rows past M: never stored
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc,
          (lds_ptr)(sA + t * TILE_BYTES + (wave * CPT + jj) * 1024), 16,
          (int)((uint32_t)row * (uint32_t)K + (uint32_t)(c * 16)), 0, 0, 0);
    }
  };
  copy_tile(0);
  __builtin_amdgcn_sched_barrier(0);
  v4i b[KH];
  const int ctc = ct < bp_tiles ? ct : bp_tiles - 1; // tiles past Bp: not stored
  const int8_t *const bp = Bp + (int64_t)ctc * TILE_BYTES + lane * 16;
#pragma unroll
  for (int s2 = 0; s2 < kBFirst; ++s2)
    b[s2] = *(const v4i *)(bp + s2 * 1024);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int t = 1; t < NR; ++t)
    copy_tile(t);
  __builtin_amdgcn_sched_barrier(0);

  // LDS address of the chunks this wave copies (those it also fixes up)
  unsigned own = (unsigned)(uintptr_t)(lds_ptr)sA + wave * (CPT * 1024) + lane * 16;
  // Turns the wave's own chunks of the tile at `own + TILE_OFF` into int8.
  v4i fx[CPT];
  auto fix_read = [&](auto offc) {
    static_for<CPT>([&](auto jc) {
      constexpr int jj = decltype(jc)::value;
      v4i &f = fx[jj];
      const unsigned addr = own;
      asm volatile("ds_read_b128 %0, %1 offset:%2"
                   : "=v"(f)
                   : "v"(addr), "n"(decltype(offc)::value + jj * 1024)
                   : "memory");
    });
  };
  auto fix_write = [&](auto offc, auto waitc) {
    {
      v4i &f0 = fx[0];
      v4i &f1 = fx[CPT - 1];
      asm volatile("s_waitcnt lgkmcnt(%2)"
                   : "+v"(f0), "+v"(f1)
                   : "n"(decltype(waitc)::value)
                   : "memory");
    }
    static_for<CPT>([&](auto jc) {
      constexpr int jj = decltype(jc)::value;
      const v4i f = fx[jj] ^ (v4i){(int)0x80808080, (int)0x80808080,
                                 (int)0x80808080, (int)0x80808080};
      const unsigned addr = own;
      asm volatile("ds_write_b128 %0, %1 offset:%2"
                   :
                   : "v"(addr), "v"(f), "n"(decltype(offc)::value + jj * 1024)
                   : "memory");
    });
  };

  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kBFirst + CPT * (NR - 1)) : "memory");
  if (FIX) {
    static_assert(CPT <= 2, "fix_write waits on two registers");
    fix_read(std::integral_constant<int, 0>{});
    fix_write(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
  }
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  WREG_TS(1); // tile 0 of A has landed

  // Every load issued before the copies has completed: the parameters.
  const int32_t oa = A_OFF ? 128 : 0;
  const int32_t ob = ep.b_unsigned ? 128 : 0;
  int32_t yz = 0;
  float sj = 0.0f;
  if (EPI != kEpiI32) {
    // a_scale * b_scale[j] first, then one multiply per element; for the
    // requantize (a_scale * b_scale) / y_scale, in this order
    // (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:127).
    sj = raw_as * raw_bs;
    if (EPI == kEpiQ8) {
      sj = sj / raw_ys;
      yz = raw_yz;
    }
  }
  const int32_t da0 = oa - (has_azp ? raw_az : 0);
  const int32_t dbj = ob - (has_bzp ? raw_bz : 0);
  // The row-sum term db[j] * rowsum(A') is not computed here: the kernel is
  // used when B carries no offset (dbj == 0).
  const uint32_t cj = (uint32_t)da0 * (uint32_t)raw_cs +
                      (uint32_t)K * (uint32_t)da0 * (uint32_t)dbj;
  const float bj = has_bias ? raw_bias : -0.0f; // -0.0f changes no value

  // ---- operand reads -------------------------------------------------------
  // Lane (row r = lane % 32, half h = lane / 32) takes chunk c = 2 s + h of
  // its row in step s, stored at position c ^ (r % 16): byte offset
  // r * K + ((32 s) ^ xh), xh = 16 h ^ 16 (r % 16) < 256.  With s = 8 u + v
  // that is 256 u + ((32 v) ^ xh): eight lane addresses, one per v, and an
  // immediate offset per u.  The tiles lie back to back, so "PF steps ahead"
  // is the same whether it stays in the tile or reaches into the next one
  // (+ TILE_BYTES).
  unsigned aaddr[8];
  {
    const unsigned arow = (unsigned)(uintptr_t)(lds_ptr)sA + l32 * K;
    const unsigned xh = (unsigned)((16 * lh) ^ (16 * (l32 & 15)));
#pragma unroll
    for (int v = 0; v < 8; ++v)
      aaddr[v] = arow + ((unsigned)(32 * v) ^ xh);
  }
  v4i fa[NB];
  auto aread = [&](auto sc) { // the read for step SC of the current tile
    constexpr int SC = decltype(sc)::value;
    v4i &f = fa[SC % NB]; // (named here: asm operands alone do not capture)
    const unsigned addr = aaddr[SC % 8];
    asm volatile("ds_read_b128 %0, %1 offset:%2"
                 : "=v"(f)
                 : "v"(addr),
                 "n"(256 * ((SC % KH) / 8) + (SC >= KH ? TILE_BYTES : 0))
                 : "memory");
  };

  // ---- output addressing ---------------------------------------------------
  // Results are written with buffer stores: the descriptor covers exactly the
  // M x N output, so an element of a row past M (its offset is past the end)
  // is dropped by the hardware's range check, and the lanes of a column past
  // N get an offset that is out of range for every row.  No store needs a
  // branch, and blocks at the edge of the matrix run the same code as the rest.
  // No offset wraps around into the buffer: the output has at most 2^31
  // bytes and the rows of a block fewer than 2^30 (wreg_ok), so a row past M
  // stays below 2^32 and the offsets of a column past N, which start at 2^31,
  // do too.
  const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      ep.out, 0, (int)((uint32_t)M * (uint32_t)N * (uint32_t)ES), 0x00020000);
  // offset of (first row of the finished tile + 4 * lh, column of the lane)
  uint32_t toff = n < N ? ((uint32_t)(row0 + 4 * lh) * (uint32_t)N + (uint32_t)n) *
                              (uint32_t)ES
                        : 0x80000000u;
  const uint32_t tile_pitch = 32u * (uint32_t)N * (uint32_t)ES;
  // Staged: where the lane puts its bytes (row 4 * lh of the tile being
  // filled, its own column), and what it stores of a gathered tile: piece
  // idx % (2 WAVES) of row idx / (2 WAVES), idx = its number in the block.
  unsigned saddr = (unsigned)(uintptr_t)(lds_ptr)sA + kStageAt +
                   4 * lh * kStagePitch + wave * 32 + l32;
  int stage_row0 = row0 * N; // offset of the gathered tile's first row
  auto flush_read = [&](v4i &dst, int buf) {
    // (the lane's number is read again here rather than kept in a register)
    const int idx = wave * 64 + (int)__builtin_amdgcn_mbcnt_hi(
                                    ~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int frow = idx / (2 * WAVES);
    const int fch = idx - frow * (2 * WAVES);
    const unsigned addr = (unsigned)(uintptr_t)(lds_ptr)sA + kStageAt +
                          buf * kStageBytes + frow * kStagePitch + fch * 16;
    asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(addr) : "memory");
  };
  auto flush_store = [&](const v4i &src) {
    const int idx = wave * 64 + (int)__builtin_amdgcn_mbcnt_hi(
                                    ~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int frow = idx / (2 * WAVES);
    const int fch = idx - frow * (2 * WAVES);
    const int col = rn * (32 * WAVES) + fch * 16;
    const uint32_t off =
        col < N ? (uint32_t)(stage_row0 + frow * N + col) : 0x80000000u;
    __builtin_amdgcn_raw_buffer_store_b128(
        src, out_rsrc, (int)off, 0, STREAM ? kAuxThrough : 0);
  };

  const bool sat = EPI == kEpiQ8 && ep.narrow == kSaturate;
  const int32_t sat_lo = !sat ? INT32_MIN : ep.y_unsigned ? 0 : -128;
  int32_t sat_hi = !sat ? INT32_MAX : ep.y_unsigned ? 255 : 127;
  // (kept in a vector register: the clamp takes one scalar operand, and the
  // compiler would otherwise move the other one over before every element)
  if (EPI == kEpiQ8)
    asm volatile("v_mov_b32 %0, %1" : "=v"(sat_hi) : "s"(sat_hi));

  static_assert(!LIM || EPI == kEpiF32, "limits of f32 results");
  // (rows past M are copies of row M - 1, whose results they repeat: they
  // change neither limit; the lanes of a column past N are taken out at the end)
  float lim_lo = __builtin_inff(), lim_hi = -__builtin_inff();
  v16i acc, accp; // the tile being computed, the finished one before it
  // One element of the finished tile: register r.
  auto emit = [&](auto rc) {
    constexpr int r = decltype(rc)::value;
    const uint32_t y = (uint32_t)accp[r] + cj;
    constexpr int row = 8 * (r >> 2) + (r & 3); // + 4 * lh
    const int soff = row * N * ES; // the same for every lane: a scalar offset
    constexpr int kAux = STREAM ? kAuxThrough : 0;
    if (EPI == kEpiI32) {
      __builtin_amdgcn_raw_buffer_store_b32((int)y, out_rsrc, (int)toff, soff, kAux);
    } else if (EPI == kEpiF32) {
      float f = (float)(int32_t)y * sj + bj;
      // compiled in only where asked for: the loop has no slot to spare
      if (ACT == 1)
        f = relu_f32(f, 0.0f);
      else if (ACT == 2)
        f = gelu_f32(f);
      if (LIM) {
        // A NaN is ignored (the instructions return their other operand), as
        // DynamicQuantizeLinear's reductions ignore it.  Written as
        // instructions in place: the compiler moves minnum / maxnum calls to
        // the end of the tile and keeps the tile's sixteen results until then.
        float &lo = lim_lo, &hi = lim_hi;
        asm volatile("v_min_f32 %0, %0, %2\n\tv_max_f32 %1, %1, %2"
                     : "+v"(lo), "+v"(hi)
                     : "v"(f));
      }
      __builtin_amdgcn_raw_buffer_store_b32(
          (int)__float_as_uint(f), out_rsrc, (int)toff, soff, kAux);
    } else {
      const float f = (float)(int32_t)y * sj;
      int32_t v =
          (int32_t)((uint32_t)(int32_t)__builtin_rintf(f) + (uint32_t)yz);
      // one instruction, no branch: bounds that do nothing when the result
      // wraps (the byte store keeps the low byte by itself)
      // (named here: asm operands alone do not capture)
      const int32_t lo = sat_lo, hi = sat_hi;
      const unsigned at = saddr;
      asm("v_med3_i32 %0, %1, %2, %3" : "=v"(v) : "v"(v), "s"(lo), "v"(hi));
      asm volatile("ds_write_b8 %0, %1 offset:%2"
                   :
                   : "v"(at), "v"(v), "n"(row * kStagePitch)
                   : "memory");
    }
  };

  // Waits until this wave's copies of tile t + 1 have landed; runs in tile t.
  auto next_tile_landed = [&](int t) {
    static_for<NR - 1>([&](auto uc) {
      constexpr int U = decltype(uc)::value;
      if (t == U)
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(Need::at(U)) : "memory");
    });
  };

  // The K loop of tile t.  FIRST: tile 0, which has no finished tile to store
  // and issues the remaining loads of Bp.
  auto tile = [&](auto firstc, int t) {
    constexpr bool FIRST = decltype(firstc)::value;
    constexpr bool ST = STAGED && !FIRST; // a finished tile passes through LDS
    v4i gathered;
    static_for<KH>([&](auto sc) {
      constexpr int s2 = decltype(sc)::value;
      if constexpr (FIX && s2 == kFixRead) {
        next_tile_landed(t);
        fix_read(std::integral_constant<int, TILE_BYTES>{});
      }
      if constexpr (FIX && s2 == kFixWrite) // operations issued since the reads
        fix_write(std::integral_constant<int, TILE_BYTES>{},
            std::integral_constant<int,
                kFixWrite - kFixRead +
                    (ST ? wreg_staged_writes(kFixRead, kFixWrite, kEpiFirst) : 0)>{});
      if constexpr (s2 == KH - PF) {
        if (FIX) // the fix-up's writes are done: operations issued since them
          asm volatile("s_waitcnt lgkmcnt(%0)"
                       :
                       : "n"(KH - PF - kFixWrite +
                             (ST ? wreg_staged_writes(kFixWrite, KH - PF, kEpiFirst) : 0))
                       : "memory");
        else
          next_tile_landed(t);
        // (the bytes of the finished tile were written before the operand read
        // that step s2 - 1 waited for: every wave's are in LDS behind the barrier)
        __builtin_amdgcn_s_barrier();
        if constexpr (ST)
          flush_read(gathered, (t - 1) & 1);
      }
#ifndef WREG_ABL_NO_LDS
      aread(std::integral_constant<int, s2 + PF>{});
#endif
      {
        v4i &f = fa[s2 % NB];
        asm volatile("s_waitcnt lgkmcnt(%1)"
                     : "+v"(f)
                     : "n"(wreg_younger(s2, PF, FIX ? CPT : 0, kFixRead, kFixWrite, ST,
                         kEpiFirst, kFlushRead))
                     : "memory");
      }
#ifdef WREG_ABL_NO_MFMA
      if constexpr (s2 == 0)
        acc = (v16i){fa[0].x, b[s2].x, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      else
        acc[s2 % 16] += fa[s2 % NB].x + b[s2].y;
#else
      if constexpr (s2 == 0) {
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa[s2 % NB], b[s2], zero, 0, 0, 0);
      } else {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(
            fa[s2 % NB], b[s2], acc, 0, 0, 0);
      }
#endif
      if constexpr (FIRST && s2 + kBFirst < KH)
        b[s2 + kBFirst] = *(const v4i *)(bp + (s2 + kBFirst) * 1024);
      // The finished tile leaves, one element per step.
#ifndef WREG_ABL_NO_EPI
      if constexpr (!FIRST && s2 >= kEpiFirst && s2 < kEpiFirst + 16)
        emit(std::integral_constant<int, s2 - kEpiFirst>{});
      if constexpr (ST && s2 == KH - 1) {
        // the operand reads of the steps since are younger than the read of
        // the gathered tile
        asm volatile("s_waitcnt lgkmcnt(%1)"
                     : "+v"(gathered)
                     : "n"(KH - kFlushRead)
                     : "memory");
        flush_store(gathered);
      }
#endif
      __builtin_amdgcn_sched_barrier(0);
    });
    // This tile is finished: its sums become the previous tile's, the operand
    // reads and the output rows move on.  (fa is indexed by the step within
    // the tile: KH is a multiple of NB, so the ring carries over.)
    accp = acc;
    if constexpr (!FIRST) {
      toff += tile_pitch;
      if (STAGED) { // the other staging tile, the next 32 rows
        saddr += ((t - 1) & 1) ? -kStageBytes : kStageBytes;
        stage_row0 += 32 * N;
      }
    }
    // (in place: written as plain additions the compiler keeps the eight
    // addresses of tile 0 and makes eight more per tile from them)
    static_for<8>([&](auto vc) {
      unsigned &a = aaddr[decltype(vc)::value];
      asm volatile("v_add_u32_e32 %0, %1, %0" : "+v"(a) : "n"(TILE_BYTES));
    });
    own += TILE_BYTES;
    __builtin_amdgcn_sched_barrier(0);
  };

  static_for<PF>([&](auto sc) { aread(sc); });
  tile(std::true_type{}, 0);
  WREG_TS(2);
#pragma unroll 1
  for (int t = 1; t < NR; ++t) {
    tile(std::false_type{}, t);
#ifdef WREG_TIMING
    static_for<NR>([&](auto uc) {
      if (t == decltype(uc)::value)
        WREG_TS(2 + decltype(uc)::value);
    });
#endif
  }
  // the last tile
  static_for<16>([&](auto rc) { emit(rc); });
  asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); // reads past the last tile
  if (STAGED) {
    v4i gathered;
    __builtin_amdgcn_s_barrier();
    flush_read(gathered, (NR - 1) & 1);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(gathered) : : "memory");
    flush_store(gathered);
  }
  if constexpr (LIM) {
    if (n >= N) {
      lim_lo = __builtin_inff();
      lim_hi = -__builtin_inff();
    }
    // (the tiles in LDS are not read any more; behind a barrier their place
    // is free)
    __syncthreads();
    block_publish_limits(lim_lo, lim_hi, ep.limits, (float *)sA, wave, lane, WAVES,
        [] { __syncthreads(); });
  }
#ifdef WREG_TIMING
  WREG_TS(2 + NR);
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  WREG_TS(3 + NR); // every store acknowledged
  if (blockIdx.x == 0 && lane == 0)
    for (int i = 0; i < 16; ++i)
      wreg_ts[wave * 16 + i] = ts[i];
#endif
}

// Shapes the kernel is built for.
constexpr int kWregKH = 24, kWregWaves = 12, kWregNR = 4;

// ACT: 0 = none, 1 = Relu, 2 = Gelu on the f32 result
template <int A_MODE, int EPI, int ACT = 0>
hipError_t wreg_launch(hipStream_t st, const GemmArgs &g, const EpiParams &ep) {
  const int M = (int)g.M, N = (int)g.N;
  const int regions_m = (int)((g.M + 32 * kWregNR - 1) / (32 * kWregNR));
  const int ntiles = (int)((g.N + 31) / 32);
  const int regions_n = (ntiles + kWregWaves - 1) / kWregWaves;
  const int bp_tiles = (int)(round_up(g.N, kGemmBN) / 32);
  // Minimum and maximum of the results (EpiParams::limits) are taken in the
  // kernel for the f32 results of a fused layer (its activations arrive
  // stored minus 128: A_MODE 2); elsewhere a pass over y takes them.
  if constexpr (A_MODE == 2 && EPI == kEpiF32) {
    if (ep.limits.out != nullptr) {
      k_gemm_i8_wreg<kWregKH, kWregWaves, kWregNR, A_MODE, EPI, true, ACT, true>
          <<<dim3((unsigned)(regions_m * regions_n)), dim3(kWregWaves * 64), 0, st>>>(
              (const uint8_t *)g.A, g.Bp, M, N, ep, regions_m, regions_n, bp_tiles);
      return hipGetLastError();
    }
  }
  k_gemm_i8_wreg<kWregKH, kWregWaves, kWregNR, A_MODE, EPI, true, ACT>
      <<<dim3((unsigned)(regions_m * regions_n)), dim3(kWregWaves * 64), 0, st>>>(
          (const uint8_t *)g.A, g.Bp, M, N, ep, regions_m, regions_n, bp_tiles);
  return hipGetLastError();
}

} // namespace

bool wreg_ok(const GemmArgs &g) {
  const int64_t es = g.epi == kEpiQ8 ? 1 : 4;
  if (g.M * g.N * es > ((int64_t)1 << 31) ||
      32 * kWregNR * g.N * es >= ((int64_t)1 << 30) || g.M * g.K >= ((int64_t)1 << 32))
    return false;
  const bool rowsum = g.b_unsigned || (g.b_zp != nullptr && g.b_zp_len > 0);
  // (8-bit results leave in 16-byte pieces of whole 128-byte lines)
  return g.K == 32 * kWregKH && g.a_zp_len <= 1 && !g.X && !rowsum &&
         ((((uintptr_t)g.A) & 15) == 0) && (g.N * es) % 128 == 0 &&
         (g.epi != kEpiQ8 || (((uintptr_t)g.out) & 15) == 0) &&
         (g.epi == kEpiF32 || g.epi == kEpiI32 || g.epi == kEpiQ8);
}

// One block per CU and round: the kernel pays when its blocks fill at least
// 70 % of the CUs of the rounds they take (measured on MI355X, 256 CUs:
// 4096 x 768 x 3072, 256 blocks: 14.7 us against 17.4 us for 128 x 128 tiles;
// x 2304, 192 blocks: 12.1 against 15.5; x 768, 64 blocks: slower).
bool wreg_pays(int64_t M, int64_t N) {
  const int64_t blocks = ((M + 32 * kWregNR - 1) / (32 * kWregNR)) *
                         ((N + 32 * kWregWaves - 1) / (32 * kWregWaves));
  const int64_t rounds = (blocks + 255) / 256;
  return blocks * 10 >= rounds * 256 * 7;
}

hipError_t launch_gemm_wreg(hipStream_t st, const GemmArgs &g,
    const EpiParams &ep, int a_mode) {
  if (!wreg_ok(g))
    return hipErrorInvalidValue;
#ifdef OM_WREG_DEV
  return a_mode == 1 ? wreg_launch<1, kEpiF32>(st, g, ep) : hipErrorInvalidValue;
#else
  const bool f32 = g.epi == kEpiF32;
  const int act = !f32 ? 0 : g.relu ? 1 : g.gelu ? 2 : 0;
  if (g.epi == kEpiQ8)
    return a_mode == 0   ? wreg_launch<0, kEpiQ8>(st, g, ep)
           : a_mode == 1 ? wreg_launch<1, kEpiQ8>(st, g, ep)
                         : wreg_launch<2, kEpiQ8>(st, g, ep);
  switch (a_mode * 4 + (f32 ? act : 3)) {
  case 0:
    return wreg_launch<0, kEpiF32>(st, g, ep);
  case 1:
    return wreg_launch<0, kEpiF32, 1>(st, g, ep);
  case 2:
    return wreg_launch<0, kEpiF32, 2>(st, g, ep);
  case 3:
    return wreg_launch<0, kEpiI32>(st, g, ep);
  case 4:
    return wreg_launch<1, kEpiF32>(st, g, ep);
  case 5:
    return wreg_launch<1, kEpiF32, 1>(st, g, ep);
  case 6:
    return wreg_launch<1, kEpiF32, 2>(st, g, ep);
  case 7:
    return wreg_launch<1, kEpiI32>(st, g, ep);
  case 8:
    return wreg_launch<2, kEpiF32>(st, g, ep);
  case 9:
    return wreg_launch<2, kEpiF32, 1>(st, g, ep);
  case 10:
    return wreg_launch<2, kEpiF32, 2>(st, g, ep);
  case 11:
    return wreg_launch<2, kEpiI32>(st, g, ep);
  default:
    return hipErrorInvalidValue;
  }
#endif
}

} // namespace gemm
} // namespace om
