// MFMA tile kernel with whole-cache-line staging and register double-buffered
// fragments, for gfx950: C[M,N] = epi(A[M,K] * B[N,K]^T), 16-bit operands.
//
// What measurement on MI355X says this kernel has to respect:
//   * the vector L1 moves 64 B/clk/CU and is charged per cache line touched, so
//     a global->LDS transfer should cover whole 128-byte lines (8 rows x 128 B per
//     wave instruction); 64-byte row slices cost twice the L1 time per byte;
//   * with realistic operand bits the matrix cores are power limited: back-to-back
//     v_mfma_f32_16x16x32_bf16 on random data sustain ~1.75 PFLOP/s when srcA
//     changes on every instruction and ~1.92 PFLOP/s when srcA is held for eight
//     instructions in a row, so the inner loop is ordered n-outer / m-inner with
//     the B-row fragment as srcA;
//   * ds_read_b128 serves 16 lanes per cycle (256 B/clk) when conflict-free,
//     ds_read_b64 only a quarter of that.
//   * a 64 KiB K-step of transfers issued at once needs ~2150 shader clocks until
//     the last byte is in LDS (about half latency, half L1 transfer time), more
//     than the 2048 clocks the matrix cores need for that K-step; and under MFMA
//     load the shader clock, which also clocks L1 and L2, drops to ~1.7 GHz.
// Structure: 256x256 workgroup tile, K-step = 128 bytes of a row.  LDS is a ring of
// five 32 KiB slots (all 160 KiB), each holding the A half or the B half of one
// K-step: A(k) in slot 2k mod 5, B(k) in slot (2k+1) mod 5.  When K-step k has been
// read into registers its two slots are refilled with B(k+2) and A(k+3), so 96 KiB
// are in flight and the half that is needed first, B(k+1), was the first in the
// queue a whole K-step earlier.  Each K-step is two MFMA k-substeps; the fragments
// of substep j+1 are read from LDS before the MFMAs of substep j are issued; one
// barrier per K-step.  The reference's equivalent pieces: direct-to-LDS staging
// (python/aster/dialects/kernel_builder_with_layouts.py:371-481), fragment reads
// (contrib/kittens/library/lds_mfma_16x64_b.mlir), the (k, m, n) MFMA loop
// (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:296-306).
#pragma once
#include <type_traits>

#include "gemm_tile_kernel.hpp"
#include "stream_load_plan.inc"

namespace astergemm {
namespace {

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// ---- epilogue shared by the stream kernels -------------------------------------------------
// Scale, bias and cast in registers, then turn each 16-row slab of the wave tile
// around in LDS so that every lane stores 16 contiguous bytes and every store
// instruction covers whole 128-byte lines of C.  (A lane owns 4 consecutive
// columns of one row per MFMA tile; stored directly that is 8 bytes per lane and
// 32-byte pieces per row, which costs ~7 % of the kernel.)  The lane id is
// recomputed here, opaque to the optimiser, so that no lane-derived value has to
// stay in a VGPR across the K loop.
// Scalar bases of a wave's LH row groups (8 rows each, 8 * NW rows apart) for the global->LDS
// transfers.  Operand heights are multiples of 8, so a group lies either inside the matrix or
// wholly past its end; the latter re-read the last 8 rows (their products land in output rows
// or columns the epilogue does not store).
template <class Plan>
__device__ __forceinline__ void group_bases(const uint8_t* mat, int64_t ld_bytes, int tile_row0, int wave,
                                            int rows, const uint8_t* (&out)[Plan::LH]) {
#pragma unroll
  for (int j = 0; j < Plan::LH; ++j) {
    int r = tile_row0 + Plan::first_row(wave, j);
    r = r < rows - Plan::TILE_ROWS ? r : rows - Plan::TILE_ROWS;
    out[j] = mat + (int64_t)r * ld_bytes;
  }
}

// K tail: when a row does not end on a 128-byte step, the K loop runs over the whole steps and
// the remaining 1..7 granules (16 bytes each) are multiplied here, once per tile, straight from
// global memory: lane (li, lq) loads the granules it would have read from LDS (s * 4 + lq for
// the 16-bit types, lq and 4 + lq for fp8) when they exist and takes zeros otherwise.  The lane
// index is recomputed, opaque to the optimiser, so that nothing here lives across the K loop.
template <int DT, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void stream_k_tail(const GemmArgs& p,
                                              f32x4 (&acc)[BM / WM / 16][BN / WN / 16], int wave,
                                              int row0, int col0, int nfull) {
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr int SUB = Enc<DT>::kSub, GR = Enc<DT>::kGran;
  int lane_t;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_t));
  const int li = lane_t & 15, lq = lane_t >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int tg = p.tail_granules;
  const int64_t koff = (int64_t)nfull * kRowBytes;
  const i32x4 zero = {0, 0, 0, 0};
#pragma unroll
  for (int s = 0; s < SUB; ++s) {
    i32x4 fbt[TN][GR], fat[TM][GR];
#pragma unroll
    for (int g = 0; g < GR; ++g) {
      const int gran = (SUB == 2 ? s : g) * 4 + lq;
      const bool live = gran < tg;
#pragma unroll
      for (int n = 0; n < TN; ++n) {
        int r = col0 + (wn * TN + n) * 16 + li;
        r = r < p.N ? r : p.N - 1;
        fbt[n][g] = live ? *(const i32x4*)(p.B + (int64_t)r * p.ldb_bytes + koff + gran * 16) : zero;
      }
#pragma unroll
      for (int m = 0; m < TM; ++m) {
        int r = row0 + (wm * TM + m) * 16 + li;
        r = r < p.M ? r : p.M - 1;
        fat[m][g] = live ? *(const i32x4*)(p.A + (int64_t)r * p.lda_bytes + koff + gran * 16) : zero;
      }
    }
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
      for (int n = 0; n < TN; ++n) acc[m][n] = mfma_step<DT>(fbt[n], fat[m], acc[m][n], 0, 0);
  }
}

template <int OUT, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void stream_epilogue(const GemmArgs& p,
                                                f32x4 (&acc)[BM / WM / 16][BN / WN / 16],
                                                uint8_t* lds, int wave, int row0, int col0) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr int SLOT = BM * kRowBytes;
  constexpr int NSLOT = 5;
  const int wm = wave / WN, wn = wave % WN;
  int lane_e;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
  const int li_e = lane_e & 15, lq_e = lane_e >> 4;
  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  constexpr int OB = (OUT == ASTERGEMM_F32) ? 4 : 2;  // bytes per output element
  constexpr int WCOLS = TN * 16;                      // columns of the wave tile
  constexpr int ROWB = WCOLS * OB;                    // bytes of one slab row
  constexpr int PITCH = ROWB + 16;                    // padded LDS pitch
  constexpr int SLAB = 16 * PITCH;
  constexpr int CHUNKS = 16 * ROWB / 16;              // 16-byte chunks per slab
  static_assert(CHUNKS % 64 == 0, "whole store instructions per slab");
  static_assert(2 * SLAB * NW <= NSLOT * SLOT, "staging fits in the ring");
  // every wave is done reading fragments before LDS is reused
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  uint8_t* stage = lds + wave * 2 * SLAB;
  const int wrow0 = row0 + wm * TM * 16, wcol0 = col0 + wn * WCOLS;
  float bias_v[TN][4];
#pragma unroll
  for (int n = 0; n < TN; ++n)
#pragma unroll
    for (int e = 0; e < 4; ++e)
    {
      int col = wcol0 + n * 16 + 4 * lq_e + e;
      col = col < p.N ? col : p.N - 1;
      bias_v[n][e] = p.bias ? p.bias[col] : 0.f;
    }
#pragma unroll
  for (int m = 0; m < TM; ++m) {
    uint8_t* slab = stage + (m & 1) * SLAB;
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      f32x4 v = acc[m][n] * scale;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += bias_v[n][e];
      uint8_t* dst = slab + li_e * PITCH + (n * 16 + 4 * lq_e) * OB;
      if constexpr (OUT == ASTERGEMM_F32) {
        *(f32x4*)dst = v;
      } else {
        const u16x4 h = cast4_16<OUT>(v);
        *(u16x4*)dst = h;
      }
    }
#pragma unroll
    for (int t = 0; t < CHUNKS / 64; ++t) {
      const int c = t * 64 + lane_e;
      const int r = c / (ROWB / 16), cc = c % (ROWB / 16);
      const i32x4 d = *(const i32x4*)(slab + r * PITCH + cc * 16);
      uint8_t* out = (uint8_t*)p.C + ((int64_t)(wrow0 + m * 16 + r) * p.ldc + wcol0) * OB + cc * 16;
      // edge tiles: N is a multiple of 8, so a 16-byte chunk is inside a row or past its end
      if (wrow0 + m * 16 + r < p.M && wcol0 + cc * (16 / OB) < p.N)
        __builtin_nontemporal_store(d, (i32x4*)out);
    }
  }
}

// Epilogue of the tile walk: a wave stages its 16-row slabs in 2 KiB of its own, which the
// ring (already receiving the next tile) does not use, so no barrier is needed: LDS operations of
// one wave execute in order.  A slab row is 128 bytes (64 16-bit or 32 fp32 columns), 16-byte
// granule g of row r sits at granule g ^ (r & 7).  M and N are whole tiles.
template <int OUT, int TM, int TN>
__device__ __forceinline__ void walk_epilogue(const GemmArgs& p, f32x4 (&acc)[TM][TN], uint8_t* stage,
                                              int wrow0, int wcol0) {
  static_assert(TN == 4, "64 columns per wave");
  float scale = 1.0f;  // fetched per tile (scalar loads): nothing to keep across the K loop
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  int lane;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
  const int li = lane & 15, lq = lane >> 4;
  constexpr int OB = (OUT == ASTERGEMM_F32) ? 4 : 2;
  constexpr int PASSES = 64 * OB / 128;          // 128-byte column ranges of the wave tile
  constexpr int TPP = TN / PASSES;               // 16-column tiles per pass
  float bias_v[TN][4];
#pragma unroll
  for (int n = 0; n < TN; ++n)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      int col = wcol0 + n * 16 + 4 * lq + e;
      col = col < p.N ? col : p.N - 1;
      bias_v[n][e] = p.bias ? p.bias[col] : 0.f;
    }
#pragma unroll
  for (int m = 0; m < TM; ++m) {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
#pragma unroll
      for (int t = 0; t < TPP; ++t) {
        const int n = ps * TPP + t;
        f32x4 v = acc[m][n] * scale;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += bias_v[n][e];
        if constexpr (OUT == ASTERGEMM_F32) {
          *(f32x4*)(stage + li * 128 + (((t * 4 + lq) ^ (li & 7)) << 4)) = v;
        } else {
          const u16x4 h = cast4_16<OUT>(v);
          *(u16x4*)(stage + li * 128 + (((t * 2 + (lq >> 1)) ^ (li & 7)) << 4) + (lq & 1) * 8) = h;
        }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int c = t * 64 + lane;
        const int r = c >> 3, cc = c & 7;
        const i32x4 d = *(const i32x4*)(stage + r * 128 + ((cc ^ (r & 7)) << 4));
        const int col = wcol0 + (ps * 128 + cc * 16) / OB;
        uint8_t* out = (uint8_t*)p.C + ((int64_t)(wrow0 + m * 16 + r) * p.ldc + col) * OB;
        // whole tiles only (the launcher checks): every store is issued, so that the count
        // the next tile's first barrier leaves outstanding is exact
        __builtin_nontemporal_store(d, (i32x4*)out);
      }
    }
  }
}

// acc += srcA * srcB for the 16-bit types.  AX: the accumulator lives in the accumulation
// half of the register file and destination and addend are tied (a four-wave workgroup owns
// 256 architectural + 256 accumulation registers per wave; only the constraint makes the
// compiler use the latter, and the tie keeps it from rotating accumulators through copies).
template <int DT, bool AX>
__device__ __forceinline__ void stream_mma(const i32x4& a, const i32x4& b, f32x4& acc) {
  if constexpr (!AX) {
    acc = mfma_step<DT>(&a, &b, acc, 0, 0);
  } else if constexpr (DT == ASTERGEMM_BF16) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  } else {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN, int NSLOT = 5>
__device__ __forceinline__ void gemm_stream_body(const GemmArgs& p, int bid) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;
  constexpr int TN = BN / WN / 16;
  constexpr int SLOT = BM * kRowBytes;  // 32 KiB: one operand half of one K-step
  // Ring of NSLOT = 2 D + 1 slots: A(k) in slot 2k mod NSLOT, B(k) in slot 2k + 1 mod NSLOT; while
  // K-step k is multiplied, B(k + D) and A(k + D + 1) are requested.  Five slots (D = 2) fill the
  // LDS of a CU at 256 x 256; the 128 x 128 form is also built with nine (D = 4, 144 KiB) for
  // grids of at most one workgroup per CU, where the bytes in flight per CU bound the speed.
  static_assert(NSLOT % 2 == 1 && NSLOT >= 5, "odd ring");
  constexpr int D = (NSLOT - 1) / 2;
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 1 KiB (8 rows x 128 B) transfers per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  constexpr bool AX = NW == 4;          // one wave per SIMD: accumulators in accumulation registers
  static_assert(BM == BN, "the ring holds equal A and B halves");
  static_assert(DT == ASTERGEMM_BF16 || DT == ASTERGEMM_F16, "16-bit operands");
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows per wave");
  static_assert((8 * NW) % 16 == 0, "swizzle phase must not depend on the transfer index");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  int tile_m, tile_n;
  map_tile(bid, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;

  // ---- global -> LDS (same layout as gemm_tile_body: 128-byte rows, granule
  // index XOR ((row >> 1) & 7)).  Only whole tiles and whole K-steps come here, so
  // one per-lane offset serves every transfer and the row block of transfer j goes
  // into the scalar base.
  const int lrow = lane >> 3;
  const int g_lane = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
  const unsigned a_off = (unsigned)(lrow * (int)p.lda_bytes + g_lane * 16);
  const unsigned b_off = (unsigned)(lrow * (int)p.ldb_bytes + g_lane * 16);
  const uint8_t* a_base[LH];
  const uint8_t* b_base[LH];
  group_bases<Plan>(p.A, p.lda_bytes, row0, wave, p.M, a_base);
  group_bases<Plan>(p.B, p.ldb_bytes, col0, wave, p.N, b_base);
  const int nk = p.ksteps - (p.tail_granules ? 1 : 0);  // whole 128-byte steps

  // 64 lanes x 16 bytes from (scalar base + per-lane offset) to LDS at M0 + lane*16.
  // Written as asm to keep the scalar-base form; vmcnt is tracked by hand.
  auto g2s = [&](const uint8_t* base, unsigned voff, uint8_t* dst) {
    const unsigned m0v = (unsigned)(size_t)AG_LDS(dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(base)
                 : "memory", "m0");
  };
  // transfer j (0..LH-1) of this wave for the A / B half of K-step k
  auto issue_a1 = [&](int k, int slot, int j) {
    g2s(a_base[j] + (int64_t)k * kRowBytes, a_off,
        lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  auto issue_b1 = [&](int k, int slot, int j) {
    g2s(b_base[j] + (int64_t)k * kRowBytes, b_off,
        lds + slot * SLOT + Plan::lds_offset(wave, j));
  };
  auto issue_a = [&](int k, int slot) {
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_a1(k, slot, j);
  };
  auto issue_b = [&](int k, int slot) {
#pragma unroll
    for (int j = 0; j < LH; ++j) issue_b1(k, slot, j);
  };

  // ---- LDS -> fragments -------------------------------------------------------------
  const int li = lane & 15, lq = lane >> 4;
  unsigned rd_off[2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
    rd_off[s] = (unsigned)(li * kRowBytes + (((s * 4 + lq) ^ (li >> 1)) << 4));
  const unsigned a_rd = (unsigned)(wm * TM * 16 * kRowBytes);
  const unsigned b_rd = (unsigned)(wn * TN * 16 * kRowBytes);

  // KM = k mod NSLOT fixes the ring slots of K-step k at compile time.
  i32x4 fa[2][TM], fb[2][TN];
  auto read_frags = [&](auto kmod, auto sub) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int S = decltype(sub)::value;
    const uint8_t* sa = lds + ((2 * KM) % NSLOT) * SLOT;
    const uint8_t* sb = lds + ((2 * KM + 1) % NSLOT) * SLOT;
#pragma unroll
    for (int n = 0; n < TN; ++n)
      fb[S][n] = *(const i32x4*)(sb + b_rd + n * 16 * kRowBytes + rd_off[S]);
#pragma unroll
    for (int m = 0; m < TM; ++m)
      fa[S][m] = *(const i32x4*)(sa + a_rd + m * 16 * kRowBytes + rd_off[S]);
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (AX) asm volatile("" : "+a"(acc[m][n]));
    }

  // fragment I of substep S of the K-step with ring position KM: I < TN is B tile I,
  // else A tile I - TN
  auto read_one = [&](auto kmod, auto sub, auto idx) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int S = decltype(sub)::value;
    constexpr int I = decltype(idx)::value;
    if constexpr (I < TN) {
      const uint8_t* sb = lds + ((2 * KM + 1) % NSLOT) * SLOT;
      fb[S][I] = *(const i32x4*)(sb + b_rd + I * 16 * kRowBytes + rd_off[S]);
    } else {
      const uint8_t* sa = lds + ((2 * KM) % NSLOT) * SLOT;
      fa[S][I - TN] = *(const i32x4*)(sa + a_rd + (I - TN) * 16 * kRowBytes + rd_off[S]);
    }
  };

  // srcA = B-row fragment, held for TM instructions in a row; lane owns
  // C[m = lane % 16][4 consecutive n].
  auto mfmas = [&](auto sub) {
    constexpr int S = decltype(sub)::value;
#pragma unroll
    for (int n = 0; n < TN; ++n)
#pragma unroll
      for (int m = 0; m < TM; ++m)
        stream_mma<DT, AX>(fb[S][n], fa[S][m], acc[m][n]);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // ---- prologue: A(0) B(0) ... A(D-1) B(D-1) A(D) in flight, both fragment sets of K-step 0
  // read, first substep multiplied -----------------------------------------------------------
  static_for<0, D>([&](auto ic) {
    constexpr int I = decltype(ic)::value;
    if (nk > I) {
      issue_a(I, (2 * I) % NSLOT);
      issue_b(I, (2 * I + 1) % NSLOT);
    }
  });
  if (nk > D) issue_a(D, (2 * D) % NSLOT);
  {
    // groups of LH transfers issued; all but the first two (A(0), B(0)) may stay in flight
    const int groups = 2 * (nk < D ? nk : D) + (nk > D ? 1 : 0);
    static_for<2, 2 * D + 2>([&](auto gc) {
      constexpr int G = decltype(gc)::value;
      if (groups == G) __builtin_amdgcn_s_waitcnt(waitcnt_imm((G - 2) * LH, 15));
    });
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  using K0 = std::integral_constant<int, 0>;
  read_frags(K0{}, S0{});
  read_frags(K0{}, S1{});
  __builtin_amdgcn_sched_barrier(0);
  mfmas(S0{});
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop ------------------------------------------------------------------------------
  // One trip finishes K-step k (substep 1) and starts K-step k+1 (substep 0).  It
  // begins with a wait and a barrier: A(k+1) and B(k+1) have landed for everybody
  // (only A(k+2) ... A(k+D) may still be in flight) and every fragment of K-step k is in
  // registers, which frees its two slots for B(k+D) and A(k+D+1).
  // Inside a trip nothing is issued in bursts: a wave that is stuck pushing loads
  // into a full address queue, or reads into a full LDS queue, cannot issue MFMAs.
  // So every MFMA is followed by at most one LDS read or one global->LDS transfer:
  // block 1 (substep 1 of K-step k) carries the reads of substep 0 of K-step k+1 and
  // the transfers of B(k+D), which is needed first; block 2 carries the reads of
  // substep 1 and the transfers of A(k+D+1).
  auto trip = [&](int k, auto kmod, auto steady) {
    constexpr int KM = decltype(kmod)::value;
    constexpr bool STEADY = decltype(steady)::value;
    using KN = std::integral_constant<int, (KM + 1) % NSLOT>;
    constexpr int NF = TM + TN;      // fragments per substep
    constexpr int NMF = TM * TN;     // MFMAs per substep
    static_assert(NF + LH <= NMF, "one side instruction per MFMA");
    static_assert((2 * D - 3) * LH <= 63, "vmcnt field");
    if constexpr (STEADY) __builtin_amdgcn_s_waitcnt(waitcnt_imm((2 * D - 3) * LH, 0));
    else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const bool do_b = STEADY || k + D < nk;
    const bool do_a = STEADY || k + D + 1 < nk;
    static_for<0, NMF>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int n = I / TM, m = I % TM;
      stream_mma<DT, AX>(fb[1][n], fa[1][m], acc[m][n]);
      if constexpr (I < LH) {
        if (do_b) issue_b1(k + D, (2 * KM) % NSLOT, I);
      }
      if constexpr (I >= LH && I < LH + NF) read_one(KN{}, S0{}, std::integral_constant<int, I - LH>{});
      __builtin_amdgcn_sched_barrier(0);
    });
    static_for<0, NMF>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int n = I / TM, m = I % TM;
      stream_mma<DT, AX>(fb[0][n], fa[0][m], acc[m][n]);
      if constexpr (I < NF) read_one(KN{}, S1{}, std::integral_constant<int, I>{});
      if constexpr (I >= NF && I < NF + LH) {
        if (do_a) issue_a1(k + D + 1, (2 * KM + 1) % NSLOT, I - NF);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  using T = std::true_type;
  using F = std::false_type;
  int k = 0;
  // steady: K-steps up to k + (NSLOT - 1) + D + 1 exist for the whole group of NSLOT trips
  for (; k + NSLOT + D + 1 <= nk; k += NSLOT)
    static_for<0, NSLOT>([&](auto ic) { trip(k + decltype(ic)::value, ic, T{}); });
  for (; k + 1 < nk; k += NSLOT)
    static_for<0, NSLOT>([&](auto ic) {
      if (k + decltype(ic)::value + 1 < nk) trip(k + decltype(ic)::value, ic, F{});
    });
  __builtin_amdgcn_sched_barrier(0);
  mfmas(S1{});

  if constexpr (WM * WN == 8 || BM == 128) {  // four waves on 256 x 256 have no registers to spare
    if (p.tail_granules) stream_k_tail<DT, BM, BN, WM, WN>(p, acc, wave, row0, col0, nk);
  }
  stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, row0, col0);
}

template <int DT, int OUT, int BM, int BN, int WM, int WN, int NSLOT = 5>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream_kernel(const GemmArgs p) {
  gemm_stream_body<DT, OUT, BM, BN, WM, WN, NSLOT>(p, blockIdx.x);
}

// Split K: the grid is p.split_k copies of the tile grid; copy s multiplies K steps
// [s * p.ksteps, (s + 1) * p.ksteps) of every row and leaves its fp32 sums in plane s of the
// workspace [split_k][M][N] (no scale, no bias: the kernel that adds the planes applies them).
// For few output tiles and long rows, where the tile grid alone leaves most CUs idle.
template <int DT, int BM, int BN, int WM, int WN, int NSLOT = 5>
__global__ __launch_bounds__(WM* WN * 64) void gemm_stream_splitk_kernel(const GemmArgs p) {
  const int tiles = p.tiles_m * p.tiles_n;
  const int ks = blockIdx.x / tiles;
  GemmArgs q = p;
  q.A = p.A + (int64_t)ks * p.ksteps * kRowBytes;
  q.B = p.B + (int64_t)ks * p.ksteps * kRowBytes;
  q.C = p.workspace + (int64_t)ks * p.M * p.N;
  gemm_stream_body<DT, ASTERGEMM_F32, BM, BN, WM, WN, NSLOT>(q, blockIdx.x - ks * tiles);
}

}  // namespace
}  // namespace astergemm
