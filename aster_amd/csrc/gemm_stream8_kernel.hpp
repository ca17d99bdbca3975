// Stream kernel for fp8 e4m3 operands: the staging, swizzle, tile map and epilogue of
// gemm_stream_kernel.hpp with v_mfma_scale_f32_16x16x128_f8f6f4 as the inner instruction.
//
// One K-step is a 128-byte row slice = 128 fp8 elements = ONE MFMA per 16x16 tile, whose
// operand is 32 bytes per lane.  The dot product does not care in which order the 128
// K positions are visited as long as both operands agree, so lane (i, q) takes granules
// q and 4+q of its row (the two 16-byte reads the 16-bit kernel makes for its two
// k-substeps) instead of the contiguous bytes [32q, 32q+32).
//
// Registers decide the structure.  128 accumulators leave room for about 90 fragment
// registers, and a full K-step of fragments is 8 x 8 (A rows) + 4 x 8 (B rows) = 96 in
// eight-register tuples, which does not allocate.  With the n-outer MFMA order (B-row
// fragment as srcA, held for eight instructions) a B-row fragment is needed for one
// group of eight MFMAs only, so B-row fragments live in a ring of two and are read one
// group ahead; the eight A-row fragments stay resident and are refilled in place for
// the next K-step as they die during the last group (next use eight MFMAs later).
// The workgroup barrier of a trip sits after MFMA 19: behind the last read of B(k) (at
// MFMA 16) and ahead of the first read of K-step k+1 (at MFMA 24), so one barrier both
// certifies A(k+1), B(k+1) and frees B(k).  The ring is three A slots (k mod 3) and two
// B slots (k mod 2); B is transferred one K-step ahead and A two, 96 KiB in flight, as in
// the 16-bit kernel.  Slot offsets are scalars that rotate from trip to trip, so the loop
// body is a single trip (the register allocator does not cope with six unrolled ones at
// this register pressure).
//
// WALK: one workgroup per CU takes tiles bid, bid + stride, ... below `total` in one launch.  When
// the K loop of a tile is over and every wave has left the ring (one barrier), the first two
// K-steps of the next tile are requested into slots A0, A1, B0, B1 and arrive while the
// epilogue runs out of the third A slot (4 KiB per wave, no barrier); the epilogue's stores are
// left in flight: the waits of the next tile's start count them as still outstanding (the
// vector-memory counter retires in issue order), so only the barrier of trip 1, whose transfers
// were requested behind the stores, waits for them.  Whole tiles, whole K-steps, at least four.
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT, int BM, int BN, int WM, int WN, bool WALK = false>
__device__ __forceinline__ void gemm_stream8_body(const GemmArgs& p, int bid, int stride = 0,
                                                  int total = 0) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr int SLOT = BM * kRowBytes;  // 32 KiB: one operand half of one K-step
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 1 KiB transfers per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  constexpr int NMF = TM * TN;
  // MFMAs of a trip issued ahead of its barrier: behind the last read of B(k), at MFMA
  // (TN-2)*TM, and not behind the first read of K-step k+1, at MFMA (TN-1)*TM
  constexpr int BAR = (TN - 2) * TM + (TM == 8 ? 4 : 1);
  static_assert(BM == BN, "the ring holds equal A and B halves");
  static_assert(DT == ASTERGEMM_FP8_E4M3, "fp8 operands");
  static_assert(BM % (8 * NW) == 0 && (8 * NW) % 16 == 0, "tile rows per wave");
  static_assert((TM == 8 || TM == 4) && TN == 4 && LH == 4, "side-instruction schedule below");
  // vector stores of one wave's walk epilogue (two per 16-row slab and 128 bytes of row)
  constexpr int NST = TM * 2 * (OUT == ASTERGEMM_F32 ? 2 : 1);
  static_assert(2 * LH + NST <= 63, "the counted waits fit the vmcnt field");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  // Eight waves: waves w and w + 4 share a SIMD.  The upper four get the higher issue priority,
  // so that of the two the same one wins whenever both are ready (measured on 8192^3: 350-352 us
  // without, 343-346 with; no difference for the 16-bit and MXFP4 kernels, which do not do it).
  if constexpr (NW == 8) {
    if (wave >= 4) __builtin_amdgcn_s_setprio(1);
  }

  // ---- global -> LDS: identical to the 16-bit stream kernel --------------------------------
  const int lane = threadIdx.x & 63;
  const int lrow = lane >> 3;
  const int g_lane = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
  const unsigned a_off = (unsigned)(lrow * (int)p.lda_bytes + g_lane * 16);
  const unsigned b_off = (unsigned)(lrow * (int)p.ldb_bytes + g_lane * 16);
  // what depends on the tile
  int row0, col0;
  const uint8_t* a_base[LH];
  const uint8_t* b_base[LH];
  auto set_tile = [&](int id) {
    int tile_m, tile_n;
    map_tile(id, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
    row0 = tile_m * BM, col0 = tile_n * BN;
    if constexpr (WALK) {
      // whole tiles: transfer j starts 8 * NW rows behind transfer j - 1, one base is enough
      a_base[0] = p.A + (int64_t)(row0 + wave * 8) * p.lda_bytes;
      b_base[0] = p.B + (int64_t)(col0 + wave * 8) * p.ldb_bytes;
    } else {
      group_bases<Plan>(p.A, p.lda_bytes, row0, wave, p.M, a_base);
      group_bases<Plan>(p.B, p.ldb_bytes, col0, wave, p.N, b_base);
    }
  };
  set_tile(bid);
  const int nk = p.ksteps - (p.tail_granules ? 1 : 0);  // whole 128-byte steps

  auto g2s = [&](const uint8_t* base, unsigned voff, uint8_t* dst) {
    const unsigned m0v = (unsigned)(size_t)AG_LDS(dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(base)
                 : "memory", "m0");
  };
  auto issue_a1 = [&](int k, int slot, int j) {  // slot: 0..2
    const uint8_t* base = WALK ? a_base[0] + (int64_t)j * (8 * NW) * p.lda_bytes : a_base[j];
    g2s(base + (int64_t)k * kRowBytes, a_off, lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  auto issue_b1 = [&](int k, int slot, int j) {  // slot: 3..4
    const uint8_t* base = WALK ? b_base[0] + (int64_t)j * (8 * NW) * p.ldb_bytes : b_base[j];
    g2s(base + (int64_t)k * kRowBytes, b_off, lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  auto issue_a = [&](int k, int slot) {
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_a1(k, slot, j);
  };
  auto issue_b = [&](int k, int slot) {
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_b1(k, slot, j);
  };

  // ---- LDS -> fragments ---------------------------------------------------------------------
  // lane (i, q) reads granule q (half 0) and granule 4+q (half 1) of row i of a 16-row block;
  // the wave's row block and the ring slot are scalar offsets added per read
  const int li = lane & 15, lq = lane >> 4;
  const unsigned rd0 = (unsigned)(li * kRowBytes + ((lq ^ (li >> 1)) << 4));
  const unsigned rd1 = (unsigned)(li * kRowBytes + (((4 + lq) ^ (li >> 1)) << 4));
  const unsigned a_rd = (unsigned)(wm * TM * 16 * kRowBytes);
  const unsigned b_rd = (unsigned)(wn * TN * 16 * kRowBytes);

  // slot of A(k) / B(k)
  auto a_slot = [](int k) { return k % 3; };
  auto b_slot = [](int k) { return 3 + k % 2; };

  i32x8 fa[TM], fbr[2];
  // B-row fragment N out of ring slot `slot` -> fbr[N & 1]; A-row fragment M -> fa[M]: two
  // 16-byte reads that together make the 32-byte operand
  auto read_b = [&](int slot, auto nn) {
    constexpr int N = decltype(nn)::value;
    const uint8_t* sb = lds + ((unsigned)(slot * SLOT) + b_rd);
    const i32x4 lo = *(const i32x4*)(sb + rd0 + N * 16 * kRowBytes);
    const i32x4 hi = *(const i32x4*)(sb + rd1 + N * 16 * kRowBytes);
    fbr[N & 1] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  auto read_a = [&](auto mm, const uint8_t* p0, const uint8_t* p1) {
    constexpr int M = decltype(mm)::value;
    const i32x4 lo = *(const i32x4*)(p0 + M * 16 * kRowBytes);
    const i32x4 hi = *(const i32x4*)(p1 + M * 16 * kRowBytes);
    fa[M] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  f32x4 acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
      for (int n = 0; n < TN; ++n) {
        acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
        // opaque to the optimiser: otherwise the first MFMA of every tile reads one shared
        // zero tuple and writes a fresh one, and 128 accumulators + 4 no longer fit
        asm volatile("" : "+v"(acc[m][n]));
      }
  };
  using K0 = std::integral_constant<int, 0>;
  // A-row fragments and the first B-row fragment of K-step 0 (slots 0 and 3)
  auto first_reads = [&]() {
    read_b(b_slot(0), K0{});
    const uint8_t* sa = lds + ((unsigned)(a_slot(0) * SLOT) + a_rd);
    const uint8_t* p0 = sa + rd0;
    const uint8_t* p1 = sa + rd1;
    static_for<0, TM>([&](auto m) { read_a(m, p0, p1); });
  };
  bool stores_behind = false;  // walk: the previous tile's stores are still counted

  // ---- prologue: A(0) B(0) A(1) B(1) issued; A-row fragments and the first B-row fragment
  // of K-step 0 read -----------------------------------------------------------------------------
  if constexpr (!WALK) zero_acc();
  issue_a(0, a_slot(0));
  issue_b(0, b_slot(0));
  if constexpr (!WALK) {
    if (nk > 1) {
      issue_a(1, a_slot(1));
      issue_b(1, b_slot(1));
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LH, 15));
    } else {
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    first_reads();
    __builtin_amdgcn_sched_barrier(0);
  } else {
    issue_a(1, a_slot(1));
    issue_b(1, b_slot(1));
  }

  // ---- K loop: trip k multiplies K-step k ------------------------------------------------------
  //   MFMA  0         + B-row fragment 1 of K-step k          (8: fragment 2, 16: fragment 3)
  //   MFMA  2.. 5     + transfers of A(k+2) into the slot of A(k-1)
  //   after MFMA 19   wait until A(k+1), B(k+1) have landed (A(k+2) may be in flight) and every
  //                   LDS read has returned; barrier: certifies K-step k+1, frees B(k)
  //   MFMA 20..23     + transfers of B(k+2) into the slot of B(k)
  //   MFMA 24         + B-row fragment 0 of K-step k+1
  //   MFMA 24+m       + A-row fragment m of K-step k+1
  // The loop is rotated: its body is MFMAs 20..31 of trip k followed by MFMAs 0..19 of trip
  // k+1, so that the loop header comes right after the full wait and the barrier and the
  // compiler's own wait counts inside the body stay exact.
  // ia = k mod 3, ib = k mod 2.  FIRST: MFMAs 0..BAR-1 and the barrier; else MFMAs BAR..31.
  // W0: trip 0 of a walked tile, whose barrier may leave the previous tile's stores in flight
  auto part = [&](int k, int ia, int ib, auto first, auto steady, auto w0) {
    constexpr bool FIRST = decltype(first)::value;
    constexpr bool STEADY = decltype(steady)::value;
    constexpr bool W0 = decltype(w0)::value;
    const bool do_ld = STEADY || k + 2 < nk;
    const bool do_rd = STEADY || k + 1 < nk;
    const int a_next = ia == 2 ? 0 : ia + 1;       // slot of A(k+1)
    const int a_ld = ia == 0 ? 2 : ia - 1;         // slot of A(k+2) = slot of A(k-1)
    const int b_cur = 3 + ib, b_next = 3 + (ib ^ 1);
    const uint8_t *ra0 = nullptr, *ra1 = nullptr;  // set right before their first use
    static_for<(FIRST ? 0 : BAR), (FIRST ? BAR : NMF)>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int n = I / TM, m = I % TM;
      // cbsz = blgp = 0: both operands OCP e4m3; zero scale operands select the unscaled form
      acc[m][n] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fbr[n & 1], fa[m], acc[m][n], 0,
                                                                   0, 0, 0, 0, 0);
      if constexpr (m == 0 && n + 1 < TN) read_b(b_cur, std::integral_constant<int, n + 1>{});
      if constexpr (I >= 2 && I < 2 + LH) {
        if (do_ld) issue_a1(k + 2, a_ld, I - 2);
      }
      if constexpr (I == BAR - 1) {
        __builtin_amdgcn_sched_barrier(0);
        if (do_rd) {
          if constexpr (W0) {
            // younger than A(1), B(1): the stores, then the LH transfers of A(2)
            if (stores_behind) __builtin_amdgcn_s_waitcnt(waitcnt_imm(LH + NST, 0));
            else __builtin_amdgcn_s_waitcnt(waitcnt_imm(LH, 0));
          } else if constexpr (STEADY) {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(LH, 0));
          } else {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
          }
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
      }
      if constexpr (I >= BAR && I < BAR + LH) {
        if (do_ld) issue_b1(k + 2, b_cur, I - BAR);
      }
      if constexpr (I == (TN - 1) * TM) {
        const uint8_t* sa = lds + ((unsigned)(a_next * SLOT) + a_rd);
        ra0 = sa + rd0;
        ra1 = sa + rd1;
      }
      if constexpr (I >= (TN - 1) * TM) {
        if (do_rd) {
          if constexpr (m == 0) read_b(b_next, std::integral_constant<int, 0>{});
          read_a(std::integral_constant<int, m>{}, ra0, ra1);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  static_assert(BAR > 2 + LH && BAR > (TN - 2) * TM && BAR <= (TN - 1) * TM && BAR + LH <= NMF,
                "schedule positions");
  using T = std::true_type;
  using F = std::false_type;
  // the K loop of one tile, from MFMA 0 of trip 0 to the last MFMA
  auto k_loop = [&](auto w0) {
    int k = 0, ia = 0, ib = 0;
    part(0, 0, 0, T{}, w0, w0);  // a walked tile has K-steps 1 and 2 to read and to request
#pragma unroll 1
    for (; k + 3 < nk; ++k) {
      part(k, ia, ib, F{}, T{}, F{});
      ia = ia == 2 ? 0 : ia + 1;
      ib ^= 1;
      part(k + 1, ia, ib, T{}, T{}, F{});
    }
#pragma unroll 1
    for (; k < nk; ++k) {
      part(k, ia, ib, F{}, F{}, F{});
      ia = ia == 2 ? 0 : ia + 1;
      ib ^= 1;
      if (k + 1 < nk) part(k + 1, ia, ib, T{}, F{}, F{});
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (!WALK) {
    k_loop(F{});
    if (p.tail_granules) stream_k_tail<DT, BM, BN, WM, WN>(p, acc, wave, row0, col0, nk);
    stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, row0, col0);
  } else {
    // One path for every tile (the accumulators never meet a join): the last tile of a workgroup
    // requests its own first two K-steps again, into slots nothing reads any more.
    int tile = bid;
    for (;;) {
      zero_acc();
      // A(0), B(0) have landed; A(1), B(1) and, behind them, the stores may be in flight
      if (stores_behind) __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LH + NST, 15));
      else __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LH, 15));
      // also: every wave is through its epilogue, whose staging memory trip 0 gives to A(2)
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      first_reads();
      __builtin_amdgcn_sched_barrier(0);
      k_loop(T{});
      // every wave has left the ring before anything is requested into it
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      const bool more = tile + stride < total;
      const int wrow0 = row0 + wm * TM * 16, wcol0 = col0 + wn * TN * 16;
      set_tile(more ? tile + stride : tile);
      issue_a(0, a_slot(0));
      issue_b(0, b_slot(0));
      issue_a(1, a_slot(1));
      issue_b(1, b_slot(1));
      __builtin_amdgcn_sched_barrier(0);
      walk_epilogue<OUT, TM, TN>(p, acc, lds + 2 * SLOT + wave * 4096, wrow0, wcol0);
      __builtin_amdgcn_sched_barrier(0);
      if (!more) break;
      tile += stride;
      stores_behind = true;
    }
    // the transfers the last tile requested must have landed before the workgroup gives its
    // LDS back
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream8_kernel(const GemmArgs p) {
  gemm_stream8_body<DT, OUT, BM, BN, WM, WN>(p, blockIdx.x);
}

// Tile walk: grid = one workgroup per CU, workgroup b takes tiles b, b + grid, ...
template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream8_walk_kernel(const GemmArgs p) {
  gemm_stream8_body<DT, OUT, BM, BN, WM, WN, true>(p, blockIdx.x, gridDim.x,
                                                  p.tiles_m * p.tiles_n);
}

// Split K (see gemm_stream_splitk_kernel): copy s of the tile grid multiplies K steps
// [s * p.ksteps, (s + 1) * p.ksteps) into plane s of the fp32 workspace; the tensor scales are
// applied by the kernel that adds the planes.
template <int DT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream8_splitk_kernel(const GemmArgs p) {
  const int tiles = p.tiles_m * p.tiles_n;
  const int ks = blockIdx.x / tiles;
  GemmArgs q = p;
  q.A = p.A + (int64_t)ks * p.ksteps * kRowBytes;
  q.B = p.B + (int64_t)ks * p.ksteps * kRowBytes;
  q.C = p.workspace + (int64_t)ks * p.M * p.N;
  gemm_stream8_body<DT, ASTERGEMM_F32, BM, BN, WM, WN>(q, blockIdx.x - ks * tiles);
}

}  // namespace
}  // namespace astergemm
