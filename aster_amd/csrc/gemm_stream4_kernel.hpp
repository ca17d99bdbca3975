// Stream kernel for MXFP4 operands (e2m1 nibbles, one e8m0 scale per 32 K-elements of a
// row, both operands): the staging, swizzle, tile map and epilogue of the fp8 stream kernel
// with v_mfma_scale_f32_16x16x128_f8f6f4 (cbsz = blgp = 4) as the inner instruction.
//
// A K-step is a 128-byte row slice = 256 fp4 elements = two MFMAs per 16x16 tile.  The
// operand of one MFMA is 16 bytes per lane = one 32-element scale block; lane (i, q) takes
// granule q of its row for the first MFMA and granule 4+q for the second (the same two
// reads as the fp8 kernel), with the scales of blocks q and 4+q.
//
// Scales travel through LDS as well: the 8 e8m0 bytes of a row and K-step are half a
// 16-byte granule, so one transfer instruction per wave brings the scales of 64 rows for
// TWO K-steps (a chunk), two K-steps ahead of their first use.  The wave that fetched a
// granule re-packs it in place, one trip after it landed, into byte pairs {block q,
// block 4+q}: a reading lane then needs one 16-bit LDS read per 16-row tile and K-step,
// and the two MFMAs pick bytes 0 and 1 of that register with op_sel, with no per-lane
// shifts.  (Fetching the scale bytes from global memory in the loop costs one vector
// memory instruction per tile and K-step, which the address unit cannot absorb next to the
// tile transfers, and their latency sits in front of the MFMAs.)
//
// LDS: two A slots and two B slots of 32 KiB (K-step k in slot k mod 2), 8 KiB of A scales
// and 8 KiB of B scales (chunk c in buffer c mod 2).  The barrier of a trip sits behind
// the last read of B(k): it certifies everything transferred for K-step k+1 and frees the
// slots of K-step k, whose refills (K-step k+2) are issued right behind it.
//
// Wave grid: 2 x 4 (eight waves, wave tile 128 x 64, two waves per SIMD) is the default; 2 x 2
// (four waves, one per SIMD, 128 x 128 of C each, a third fewer LDS reads per MFMA) is built as
// well and is slower: with one wave per SIMD nothing covers a wave's wait at the barrier.
// Either way the accumulators live in the accumulation registers (64 or 32 tiles x 4), which
// leaves the architectural registers to fragments, scales and addresses; with one pool of 256
// registers the eight-wave form does not allocate.
#pragma once
#include "gemm_stream_kernel.hpp"

// Register file half of the accumulators: accumulation registers.
#define ACC_CONSTRAINT(x) "+a"(x)

namespace astergemm {
namespace {

// WALK: the workgroup takes tiles bid, bid + stride, ... below `total` as one long K loop: the
// last two trips of a tile bring in K-steps 0 and 1 (and scale chunks 0 and 1) of the next tile
// where a longer row would have brought K-steps nk and nk+1, so the next tile starts with its
// operands in LDS, and the epilogue in between touches no ring memory.  Needs nk % 4 == 0 (slot
// and scale-buffer parities carry over).
template <int DT, int OUT, int BM, int BN, int WM, int WN, bool WALK = false>
__device__ __forceinline__ void gemm_stream4_body(const GemmArgs& p, int bid, int stride = 0,
                                                  int total = 0) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr int SLOT = BM * kRowBytes;  // 32 KiB: one operand half of one K-step
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 1 KiB transfers per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  constexpr int NMF = TM * TN;          // slots per trip (two MFMAs each)
  constexpr int BAR = (TN - 2) * TM + 4;  // slots of a trip issued ahead of its barrier
  constexpr int NSR = BM / 64;          // scale transfers per operand and chunk (64 rows each)
  constexpr int NSC = 2 * NSR / NW;     // scale transfers per wave and chunk
  constexpr int SC_A = 4 * SLOT;        // A scales: [2 buffers][256 rows][16 bytes]
  constexpr int SC_B = SC_A + 2 * BM * 16;
  static_assert(BM == BN, "the ring holds equal A and B halves");
  static_assert(DT == ASTERGEMM_MXFP4, "fp4 operands");
  static_assert(BM % (8 * NW) == 0 && (8 * NW) % 16 == 0, "tile rows per wave");
  static_assert(TM % 2 == 0 && TM >= 4 && TN >= 2 && (2 * NSR) % NW == 0 && NSC >= 1,
                "side-instruction schedule below");
  static_assert(BM % 64 == 0, "scale transfers cover 64 rows each");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;

  // ---- global -> LDS, tiles: identical to the other stream kernels ---------------------------
  const int lane = threadIdx.x & 63;
  const int lrow = lane >> 3;
  const int g_lane = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
  const unsigned a_off = (unsigned)(lrow * (int)p.lda_bytes + g_lane * 16);
  const unsigned b_off = (unsigned)(lrow * (int)p.ldb_bytes + g_lane * 16);
  const int nk = p.ksteps;

  // what depends on the tile: where its rows start and where its transfers read
  struct Src {
    int row0, col0;
    const uint8_t* a[LH];
    const uint8_t* b[LH];
    const uint8_t* sc[NSC];
    unsigned sc_off[NSC];
  };
  uint8_t* sc_lds[NSC];
#pragma unroll
  for (int i = 0; i < NSC; ++i) sc_lds[i] = lds + (wave + i * NW < NSR ? SC_A : SC_B) + ((wave + i * NW) % NSR) * 64 * 16;
  auto load_tile = [&](int id, Src& t) {
    int tile_m, tile_n;
    map_tile(id, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
    t.row0 = tile_m * BM, t.col0 = tile_n * BN;
    if constexpr (WALK) {
      // whole tiles: transfer j starts 8 * NW rows behind transfer j - 1, one base is enough
      t.a[0] = p.A + (int64_t)(t.row0 + wave * 8) * p.lda_bytes;
      t.b[0] = p.B + (int64_t)(t.col0 + wave * 8) * p.ldb_bytes;
    } else {
      group_bases<Plan>(p.A, p.lda_bytes, t.row0, wave, p.M, t.a);
      group_bases<Plan>(p.B, p.ldb_bytes, t.col0, wave, p.N, t.b);
    }
    // scales: transfer x = wave + i * NW (0..7): x < 4 covers A rows [64x, +64), else B rows
    // [64(x-4), +64); lane L brings the 16 scale bytes of row L for chunk c (K-steps 2c and
    // 2c+1) to [buffer c mod 2][row][16]
#pragma unroll
    for (int i = 0; i < NSC; ++i) {
      const int x = wave + i * NW;
      const bool is_a = x < NSR;
      t.sc[i] = is_a ? p.mx_a + (int64_t)t.row0 * p.mx_ld : p.mx_b + (int64_t)t.col0 * p.mx_ld;
      // rows past the end of an edge tile re-read the operand's last row
      const int first = is_a ? t.row0 : t.col0, rows = is_a ? p.M : p.N;
      int r = (x % NSR) * 64 + lane;
      if constexpr (!WALK) r = first + r < rows ? r : rows - 1 - first;  // the walk has whole tiles
      t.sc_off[i] = (unsigned)(r * p.mx_ld);
    }
  };
  Src cur;
  load_tile(bid, cur);

  auto g2s = [&](const uint8_t* base, unsigned voff, uint8_t* dst) {
    const unsigned m0v = (unsigned)(size_t)AG_LDS(dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(base)
                 : "memory", "m0");
  };
  // K-step k of tile t into ring slot `slot` (A: 0..1, B: 2..3)
  auto issue_a1 = [&](const Src& t, int k, int slot, int j) {
    const uint8_t* base = WALK ? t.a[0] + (int64_t)j * (8 * NW) * p.lda_bytes : t.a[j];
    g2s(base + (int64_t)k * kRowBytes, a_off, lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  auto issue_b1 = [&](const Src& t, int k, int slot, int j) {
    const uint8_t* base = WALK ? t.b[0] + (int64_t)j * (8 * NW) * p.ldb_bytes : t.b[j];
    g2s(base + (int64_t)k * kRowBytes, b_off, lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  // scale chunk c of tile t into scale buffer `buf`
  auto issue_scales = [&](const Src& t, int c, int buf) {
#pragma unroll
    for (int i = 0; i < NSC; ++i) g2s(t.sc[i] + c * 16, t.sc_off[i], sc_lds[i] + buf * BM * 16);
  };
  // in place: bytes b[0..15] of this lane's row -> pairs {b[8h+q], b[8h+4+q]}, h = K-step
  // parity, q = 0..3
  auto repack_scales = [&](int c) {
#pragma unroll
    for (int i = 0; i < NSC; ++i) {
      i32x4* cell = (i32x4*)(sc_lds[i] + (c & 1) * BM * 16 + lane * 16);
      const i32x4 v = *cell;
      i32x4 r;
      // v_perm_b32(hi, lo, sel): selector bytes 0-3 index lo, 4-7 index hi
      r.x = (int)__builtin_amdgcn_perm((unsigned)v.y, (unsigned)v.x, 0x05010400u);  // q = 0, 1
      r.y = (int)__builtin_amdgcn_perm((unsigned)v.y, (unsigned)v.x, 0x07030602u);  // q = 2, 3
      r.z = (int)__builtin_amdgcn_perm((unsigned)v.w, (unsigned)v.z, 0x05010400u);
      r.w = (int)__builtin_amdgcn_perm((unsigned)v.w, (unsigned)v.z, 0x07030602u);
      *cell = r;
    }
  };

  // ---- LDS -> fragments ---------------------------------------------------------------------
  const int li = lane & 15, lq = lane >> 4;
  const unsigned rd0 = (unsigned)(li * kRowBytes + ((lq ^ (li >> 1)) << 4));
  const unsigned rd1 = (unsigned)(li * kRowBytes + (((4 + lq) ^ (li >> 1)) << 4));
  const unsigned a_rd = (unsigned)(wm * TM * 16 * kRowBytes);
  const unsigned b_rd = (unsigned)(wn * TN * 16 * kRowBytes);
  // scale pair of lane (i, q) inside a 16-row tile: row i, byte 2q (+ 8 for odd K-steps)
  const unsigned sc_rd = (unsigned)(li * 16 + lq * 2);
  const unsigned sa_rd = (unsigned)(SC_A + wm * TM * 16 * 16);
  const unsigned sb_rd = (unsigned)(SC_B + wn * TN * 16 * 16);

  i32x4 fa_lo[TM], fa_hi[TM], fb_lo[2], fb_hi[2];
  int sa[TM], sb[2];
  // K-step k: tiles in slot k mod 2 (+2 for B), scales in buffer (k/2) mod 2 at byte 8*(k mod 2)
  auto read_b = [&](int k, auto nn) {
    constexpr int N = decltype(nn)::value;
    const uint8_t* s = lds + ((unsigned)((2 + (k & 1)) * SLOT) + b_rd);
    fb_lo[N & 1] = *(const i32x4*)(s + rd0 + N * 16 * kRowBytes);
    fb_hi[N & 1] = *(const i32x4*)(s + rd1 + N * 16 * kRowBytes);
  };
  auto read_sb = [&](int k, auto nn) {
    constexpr int N = decltype(nn)::value;
    const uint8_t* s = lds + ((unsigned)(((k >> 1) & 1) * BM * 16 + (k & 1) * 8) + sb_rd);
    sb[N & 1] = *(const unsigned short*)(s + sc_rd + N * 16 * 16);
  };
  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      // Accumulators live in the accumulation half of the register file (the "a"
      // constraint makes the compiler use that form of the MFMAs), which leaves the 128
      // architectural registers to fragments, scales and addresses; one pool of 256 does
      // not allocate without spilling here.  Opaque to the optimiser as well: otherwise the
      // first MFMA of every tile reads one shared zero tuple and writes a fresh one.
      asm volatile("" : ACC_CONSTRAINT(acc[m][n]));
    }

  // ---- prologue: scales of chunks 0 and 1 and tiles of K-steps 0 and 1 issued; chunk 0
  // re-packed; A-row fragments and the first B-row fragment of K-step 0 read --------------------
  issue_scales(cur, 0, 0);
#pragma unroll
  for (int j = 0; j < LH; ++j) issue_a1(cur, 0, 0, j);
#pragma unroll
  for (int j = 0; j < LH; ++j) issue_b1(cur, 0, 2, j);
  if (nk > 2) issue_scales(cur, 1, 1);
  if (nk > 1) {
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_a1(cur, 1, 1, j);
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_b1(cur, 1, 3, j);
  }
  // the first transfer (scales of chunk 0) has landed for this wave: re-pack it
  if (nk > 2) __builtin_amdgcn_s_waitcnt(waitcnt_imm(4 * LH + NSC, 15));
  else if (nk > 1) __builtin_amdgcn_s_waitcnt(waitcnt_imm(4 * LH, 15));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LH, 15));
  asm volatile("" ::: "memory");
  repack_scales(0);
  // tiles of K-step 0 landed, everybody's scales re-packed
  if (nk > 1) __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LH, 0));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // fragments of K-step 0 (slot 0, scale buffer 0): all A rows and the first B row
  auto first_reads = [&]() {
    using K0 = std::integral_constant<int, 0>;
    read_b(0, K0{});
    read_sb(0, K0{});
    const uint8_t* s = lds + a_rd;
    const uint8_t* ps = lds + sa_rd + sc_rd;
    if constexpr (WALK) {
      // used once per tile: recomputed from a lane index the optimiser cannot see through,
      // instead of living in a register (or a spill slot) across the K loop
      int l2;
      asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l2));
      ps = lds + sa_rd + (unsigned)((l2 & 15) * 16 + (l2 >> 4) * 2);
    }
    static_for<0, TM>([&](auto mc) {
      constexpr int m = decltype(mc)::value;
      fa_lo[m] = *(const i32x4*)(s + rd0 + m * 16 * kRowBytes);
      fa_hi[m] = *(const i32x4*)(s + rd1 + m * 16 * kRowBytes);
      sa[m] = *(const unsigned short*)(ps + m * 16 * 16);
    });
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- K loop: trip k multiplies K-step k; pair i = (n, m) is the two MFMAs of tile (m, n) ----
  // (slot numbers for TM = 8; group n is slots 8n .. 8n+7)
  //   slot 8n, 8n+1      + B-row fragment n+1 of K-step k and its scales (n < TN-1)
  //   slot 4             (odd k) re-pack the scale granules of chunk (k+1)/2 that this wave
  //                      brought in and that the previous barrier certified
  //   after slot BAR-1   wait for every transfer and every LDS access of this wave; barrier:
  //                      certifies tiles of K-step k+1 (and re-packed scales), frees K-step k
  //   slot BAR..BAR+LH-1 + transfers of B(k+2) and A(k+2) into the slots of K-step k
  //   slot BAR+LH-1      (odd k) + scale transfers of chunk (k+3)/2 (K-steps k+3, k+4)
  //   last group         + B-row fragment 0 of K-step k+1 and its scales, and A-row
  //                      fragment m of K-step k+1 and its scales behind the MFMAs of tile m
  // FIRST: pairs 0..BAR-1 and the barrier; else pairs BAR..31 (the loop body is the second
  // part of trip k followed by the first part of trip k+1, so that the loop header follows
  // the full wait and the compiler's own wait counts inside the body stay exact).
  // Every condition of a part is a compile-time flag, so that each part is straight-line
  // code: ODD = k is odd; LD = K-step k+2 exists (tile transfers); RD = K-step k+1 exists
  // (reads, re-pack, barrier); SC = K-step k+3 exists (scale transfer, odd trips only).
  // Tile transfers read tile `lt` at K-step k + 2 - kshift, scale transfers tile `lsc` at chunk
  // (k + 3) / 2 - cshift: both shifts are 0 inside a tile; when the last trips of a tile bring
  // in the next one they are nk and nk / 2.  Where transfers land, and everything that is
  // read, follows k alone.
  // GUARD: two wait states in front of every MFMA.  The MFMAs are inline asm, which the
  // compiler's hazard recogniser does not look into: where it places a register copy right in
  // front of one (it does in the straight-line parts of the tile walk, not in the K loop), the
  // MFMA would read the register before the copy has landed.
  constexpr int NST = TM * 2 * (OUT == ASTERGEMM_F32 ? 2 : 1);  // stores of walk_epilogue per wave
  bool stores_behind = false;
  auto part = [&](int k, auto first, auto odd_c, auto ld_c, auto rd_c, auto sc_c, const Src& lt,
                  int kshift, const Src& lsc, int cshift, auto guard_c) {
    constexpr bool GUARD = decltype(guard_c)::value != 0;
    // trip 0 of the tile walk: the stores of the previous tile's epilogue are younger than every
    // transfer this barrier has to certify, so they may stay outstanding
    constexpr bool AFTER_STORES = decltype(guard_c)::value == 2;
    constexpr bool FIRST = decltype(first)::value;
    constexpr bool odd = decltype(odd_c)::value;
    constexpr bool do_ld = decltype(ld_c)::value;
    constexpr bool do_rd = decltype(rd_c)::value;
    constexpr bool do_sc = decltype(sc_c)::value;
    const uint8_t *ra0 = nullptr, *ra1 = nullptr, *ras = nullptr;  // set right before first use
    static_for<(FIRST ? 0 : BAR), (FIRST ? BAR : NMF)>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int n = I / TM;
      // Slots come in couples over two A-row tiles: the even slot issues the first MFMA
      // (granule q) of tiles m0 and m0+1, the odd slot their second MFMA (granule 4+q), so
      // that the two MFMAs on one accumulator are never back to back.
      constexpr int m0 = (I % TM) & ~1;
      constexpr bool HI = (I & 1) != 0;
      static_for<0, 2>([&](auto jc) {
        constexpr int m = m0 + decltype(jc)::value;
        const i32x4 b4 = HI ? fb_hi[n & 1] : fb_lo[n & 1];
        const i32x4 a4 = HI ? fa_hi[m] : fa_lo[m];
        // cbsz = blgp = 4: both operands e2m1 (four registers each); op_sel picks byte 0
        // (blocks q) or byte 1 (blocks 4+q) of the scale registers.  Written as asm to tie
        // the destination to the accumulator: the compiler otherwise lets the two MFMAs of
        // a trip rotate an accumulator through fresh registers, which costs copies at the
        // loop edge and more registers than there are.  Same destination and addend is also
        // the form the hardware chains without software wait states.
#define AG_MFMA4(PRE, SEL)                                                              \
  asm volatile(PRE "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 " SEL       \
               "op_sel_hi:[0,0,0] cbsz:4 blgp:4"                                         \
               : ACC_CONSTRAINT(acc[m][n])                                               \
               : "v"(b4), "v"(a4), "v"(sb[n & 1]), "v"(sa[m]))
        if constexpr (GUARD) {
          if constexpr (!HI) AG_MFMA4("s_nop 1\n\t", "");
          else AG_MFMA4("s_nop 1\n\t", "op_sel:[1,1,0] ");
        } else {
          if constexpr (!HI) AG_MFMA4("", "");
          else AG_MFMA4("", "op_sel:[1,1,0] ");
        }
#undef AG_MFMA4
        // ---- one or two side instructions behind every MFMA --------------------------------
        if constexpr (decltype(jc)::value == 0) {
          if constexpr (I % TM == 0 && n + 1 < TN) read_b(k, std::integral_constant<int, n + 1>{});
          if constexpr (I % TM == 1 && n + 1 < TN) read_sb(k, std::integral_constant<int, n + 1>{});
          if constexpr (I == 4) {
            if (odd && do_rd) repack_scales((k + 1) >> 1);
          }
          if constexpr (I >= BAR && I < BAR + LH) {
            if (do_ld) issue_b1(lt, k + 2 - kshift, 2 + (k & 1), I - BAR);
          }
          if constexpr (I == (TN - 1) * TM) {
            const int kn = k + 1;
            const uint8_t* s = lds + ((unsigned)((kn & 1) * SLOT) + a_rd);
            ra0 = s + rd0;
            ra1 = s + rd1;
            ras = lds + ((unsigned)(((kn >> 1) & 1) * BM * 16 + (kn & 1) * 8) + sa_rd) + sc_rd;
            if (do_rd) read_b(k + 1, std::integral_constant<int, 0>{});
          }
          if constexpr (I == (TN - 1) * TM + 1) {
            if (do_rd) read_sb(k + 1, std::integral_constant<int, 0>{});
          }
        } else {
          if constexpr (I >= BAR && I < BAR + LH) {
            if (do_ld) issue_a1(lt, k + 2 - kshift, k & 1, I - BAR);
          }
          if constexpr (I == BAR + LH - 1) {
            // chunk (k+3)/2 covers K-steps k+3 and k+4; its buffer held chunk (k-1)/2
            // (K-steps k-1 and k), last read before this trip's barrier
            if (odd && do_sc) issue_scales(lsc, ((k + 3) >> 1) - cshift, ((k + 3) >> 1) & 1);
          }
        }
        // refill in place for K-step k+1: the first-MFMA operands of a couple are dead after
        // its even slot, the second-MFMA operands and the scales after its odd slot
        if constexpr (I >= (TN - 1) * TM) {
          if (do_rd) {
            if constexpr (!HI) {
              fa_lo[m] = *(const i32x4*)(ra0 + m * 16 * kRowBytes);
            } else {
              fa_hi[m] = *(const i32x4*)(ra1 + m * 16 * kRowBytes);
              sa[m] = *(const unsigned short*)(ras + m * 16 * 16);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (I == BAR - 1) {
        if (do_rd) {
          if constexpr (AFTER_STORES) {
            if (stores_behind) __builtin_amdgcn_s_waitcnt(waitcnt_imm(NST, 0));
            else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
          } else {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
          }
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };
  static_assert(BAR > (TN - 2) * TM + 1 && BAR + LH <= NMF, "schedule positions");
  using T = std::true_type;
  using F = std::false_type;
  using G0 = std::integral_constant<int, 0>;  // guard_c: no wait states in front of the MFMAs
  using G1 = std::integral_constant<int, 1>;  // two wait states
  using G2 = std::integral_constant<int, 2>;  // two wait states, trip 0 of the tile walk
  // nk is even.  part(k, first-half?, odd, LD, RD, SC, tile source, K shift, scale source, chunk shift)
  if constexpr (!WALK) {
    first_reads();
    int k = 0;
    part(0, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
#pragma unroll 1
    for (; k + 4 < nk; k += 2) {
      part(k, F{}, F{}, T{}, T{}, F{}, cur, 0, cur, 0, G0{});
      part(k + 1, T{}, T{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
      part(k + 1, F{}, T{}, T{}, T{}, T{}, cur, 0, cur, 0, G0{});
      part(k + 2, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
    }
    if (nk >= 4) {  // k = nk - 4: the last scale chunk is already on its way
      part(k, F{}, F{}, T{}, T{}, F{}, cur, 0, cur, 0, G0{});
      part(k + 1, T{}, T{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
      part(k + 1, F{}, T{}, T{}, T{}, F{}, cur, 0, cur, 0, G0{});
      part(k + 2, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
      k += 2;
    }
    // k = nk - 2: nothing left to transfer; the last trip has nothing left to read
    part(k, F{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
    part(k + 1, T{}, T{}, F{}, F{}, F{}, cur, 0, cur, 0, G0{});
    part(k + 1, F{}, T{}, F{}, F{}, F{}, cur, 0, cur, 0, G0{});
    __builtin_amdgcn_sched_barrier(0);
    stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, cur.row0, cur.col0);
  } else {
    // One path for every tile, so that the accumulators never meet a join: the last tile of a
    // workgroup brings in its own first two K-steps again, into slots nothing reads any more.
    int tile = bid;
    for (;;) {
      // zeroed here, not behind the epilogue: nothing of the accumulators crosses the back edge.
      // The zero is made here as well (opaque, so that it is not kept across the loop in
      // registers the loop does not have).
      float z;
      asm volatile("v_mov_b32 %0, 0" : "=v"(z));
      const f32x4 zero = {z, z, z, z};
#pragma unroll
      for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int n = 0; n < TN; ++n) {
          acc[m][n] = zero;
          asm volatile("" : ACC_CONSTRAINT(acc[m][n]));
        }
      // what the barrier of the last trip (the prologue, for the first tile) certified
      first_reads();
      int k = 0;
      part(0, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G2{});
#pragma unroll 1
      for (; k + 4 < nk; k += 2) {
        part(k, F{}, F{}, T{}, T{}, F{}, cur, 0, cur, 0, G0{});
        part(k + 1, T{}, T{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
        part(k + 1, F{}, T{}, T{}, T{}, T{}, cur, 0, cur, 0, G0{});
        part(k + 2, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G0{});
      }
      // k = nk - 4 (nk % 4 == 0, so nk >= 4): chunk nk / 2 is chunk 0 of the next tile, K-steps
      // nk and nk + 1 are its K-steps 0 and 1; the last trip keeps its barrier (which certifies
      // K-step 0 and the re-packed scales of the next tile) but reads nothing: fragments held
      // across the epilogue would not fit in the registers next to it
      const bool more = tile + stride < total;
      Src nxt;
      load_tile(more ? tile + stride : tile, nxt);
      part(k, F{}, F{}, T{}, T{}, F{}, cur, 0, cur, 0, G1{});
      part(k + 1, T{}, T{}, F{}, T{}, F{}, cur, 0, cur, 0, G1{});
      part(k + 1, F{}, T{}, T{}, T{}, T{}, cur, 0, nxt, nk >> 1, G1{});
      part(k + 2, T{}, F{}, F{}, T{}, F{}, cur, 0, cur, 0, G1{});
      k += 2;
      part(k, F{}, F{}, T{}, T{}, F{}, nxt, nk, nxt, nk >> 1, G1{});
      part(k + 1, T{}, T{}, F{}, T{}, F{}, cur, 0, cur, 0, G1{});
      part(k + 1, F{}, T{}, T{}, F{}, T{}, nxt, nk, nxt, nk >> 1, G1{});
      __builtin_amdgcn_sched_barrier(0);
      walk_epilogue<OUT, TM, TN>(p, acc, lds + SC_B + 2 * BM * 16 + wave * 2048,
                                 cur.row0 + wm * TM * 16, cur.col0 + wn * TN * 16);
      __builtin_amdgcn_sched_barrier(0);
      if (!more) break;
      cur = nxt;
      tile += stride;
      stores_behind = true;
    }
    // the transfers the last tile issued into the ring must have landed before the workgroup
    // gives its LDS back
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream4_kernel(const GemmArgs p) {
  gemm_stream4_body<DT, OUT, BM, BN, WM, WN>(p, blockIdx.x);
}

// Tile walk: gridDim.x workgroups (one per CU) share the tiles_m x tiles_n tiles round-robin.
template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream4_walk_kernel(const GemmArgs p) {
  gemm_stream4_body<DT, OUT, BM, BN, WM, WN, true>(p, blockIdx.x, gridDim.x, p.tiles_m * p.tiles_n);
}

// Split K (see gemm_stream_splitk_kernel): copy s of the tile grid multiplies K steps
// [s * p.ksteps, (s + 1) * p.ksteps) into plane s of the fp32 workspace.  A 128-byte step of
// nibbles has 8 e8m0 bytes per row; ranges are an even number of steps, so the scale planes
// stay on the 16-byte granules the kernel fetches.
template <int DT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream4_splitk_kernel(const GemmArgs p) {
  const int tiles = p.tiles_m * p.tiles_n;
  const int ks = blockIdx.x / tiles;
  GemmArgs q = p;
  q.A = p.A + (int64_t)ks * p.ksteps * kRowBytes;
  q.B = p.B + (int64_t)ks * p.ksteps * kRowBytes;
  q.mx_a = p.mx_a + (int64_t)ks * p.ksteps * 8;
  q.mx_b = p.mx_b + (int64_t)ks * p.ksteps * 8;
  q.C = p.workspace + (int64_t)ks * p.M * p.N;
  gemm_stream4_body<DT, ASTERGEMM_F32, BM, BN, WM, WN>(q, blockIdx.x - ks * tiles);
}

}  // namespace
}  // namespace astergemm
#undef ACC_CONSTRAINT
