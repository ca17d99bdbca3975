// MXFP4 stream kernel with B straight from global memory into MFMA operand registers and the
// e8m0 planes of BOTH operands in lane order: gemm_stream4db_kernel.hpp (128 x 256 workgroup tile,
// four waves in a 1 x 4 grid, two workgroups per CU; the reference's direct-B geometry,
// contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:75-324) without any
// scale traffic through LDS, and with every load of the K loop counted by hand.
//
// Layouts (B pre-shuffled once, A's plane written in this order by the quantiser):
//   B payload, "step order" (astergemm_shuffle_weight_8): 1 KiB chunks; chunk
//     ((nb * steps + s) * 2 + u) holds for rows 16 nb .. 16 nb + 15 and 128-byte step s the
//     granules 4 u .. 4 u + 3: lane L = 16 q + n finds at byte 16 L granule 4 u + q of row
//     16 nb + n, the operand of MFMA u of that step.
//   B e8m0 plane, "lane order" (astergemm_shuffle_scales_e8m0_lanes): 512-byte chunks; chunk
//     (nb4 * steps + s), byte 8 L + 2 t + h of lane L = 16 q + i = scale of block 4 h + q of row
//     64 nb4 + 16 t + i.
//   A e8m0 plane, "lane order in groups of 128 rows" (astergemm_shuffle_scales_e8m0_lanes128):
//     1 KiB chunks; chunk (g * steps + s), byte 16 L + 2 t + h = scale of block 4 h + q of row
//     128 g + 16 t + i; the plane holds whole groups (padded past M).
//   A payload row-major, through an LDS ring of four K-steps as in the other stream kernels.
// Per wave and K-step: one 8-byte load brings B's scales, one 16-byte load A's, and the MFMAs
// select their byte with op_sel / op_sel_hi (scale operand form: reference
// test/Dialect/AMDGCN/cdna4-scaled-mfma.mlir:37-47).
//
// MFMA order is m-outer per half K-step: m-step T = 8 u + m multiplies A fragment (m, u), read
// from LDS three m-steps ahead into a ring of four, with the four B fragments of half u.  B and
// the scales are two K-steps ahead in registers.  One barrier per K-step, three m-steps before
// its end: it certifies A(k+1) and, all reads of A(k) having been issued, frees slot k mod 4.
//
// Why every load is inline assembly: the compiler does not see the global->LDS transfers of A,
// so a wait it inserts for a B load uses a count that is too small by the transfers behind that
// load; it then forces transfers requested one K-step earlier although the ring gives them
// three.  With the counts below a wait never covers more than what it needs (loads retire in
// issue order).
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT>
__device__ __forceinline__ void gemm_stream4dbl_body(const GemmArgs& p, int bid) {
  constexpr int BM = 128, BN = 256, WM = 1, WN = 4;
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;      // 8
  constexpr int TN = BN / WN / 16;      // 4
  constexpr int SLOT = BM * kRowBytes;  // 16 KiB: A rows of one K-step
  constexpr int NSLOT = 4;              // A ring
  constexpr int NBUF = 4;               // B register buffers of half a K-step each
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 4 transfers of 1 KiB per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  constexpr int RA = 4;                 // A fragment ring
  constexpr int MS = 2 * TM;            // m-steps per K-step
  constexpr int BAR = MS - (RA - 1);    // m-step whose first MFMA follows the barrier
  static_assert(DT == ASTERGEMM_MXFP4, "fp4 operands");
  static_assert(MS % RA == 0 && TN == 4 && LH == 4, "side-instruction schedule below");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave;

  int tile_m, tile_n;
  map_tile(bid, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const int nk = p.ksteps;  // even (the launcher checks)

  // ---- A: global -> LDS, as in the other stream kernels ----------------------------------------
  const int lrow = lane >> 3;
  const int g_lane = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
  const unsigned a_off = (unsigned)(lrow * (int)p.lda_bytes + g_lane * 16);
  const uint8_t* a_base[LH];
  group_bases<Plan>(p.A, p.lda_bytes, row0, wave, p.M, a_base);
  auto g2s = [&](const uint8_t* base, unsigned voff, uint8_t* dst) {
    const unsigned m0v = (unsigned)(size_t)AG_LDS(dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(base)
                 : "memory", "m0");
  };
  auto issue_a1 = [&](int k, int slot, int j) {
    g2s(a_base[j] + (int64_t)k * kRowBytes, a_off,
        lds + slot * SLOT + Plan::lds_offset(wave, j));
  };

  // ---- B and the scale planes: global -> registers.  One raw buffer resource each; a load is
  // resource + scalar offset + per-lane offset.  The hardware's range check does not cover the
  // scalar offset, so the block indices of an edge tile are clamped to the last 16-row block of
  // B and the last 64-row group of its plane (those columns are never stored); A's plane holds
  // whole 128-row groups. ----------------------------------------------------------------------------
  const unsigned chunk_row = (unsigned)(p.K >> 7) * 1024u;  // bytes of 16 rows of B (K/2 per row)
  auto rsrc_of = [](const void* ptr, unsigned bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)ptr;
    return i32x4{(int)(unsigned)a, (int)((unsigned)(a >> 32) & 0xffffu), (int)bytes, 0x00020000};
  };
  const i32x4 b_rsrc = rsrc_of(p.B, (unsigned)(p.N >> 4) * chunk_row);
  const i32x4 sb_rsrc = rsrc_of(p.mx_b, (unsigned)(p.N >> 6) * (unsigned)nk * 512u);
  const i32x4 sa_rsrc = rsrc_of(p.mx_a, (unsigned)p.tiles_m * (unsigned)nk * 1024u);
  unsigned b_tile[TN];
#pragma unroll
  for (int n = 0; n < TN; ++n) {
    int nb = (col0 >> 4) + wn * TN + n;
    const int last = (p.N >> 4) - 1;
    nb = nb < last ? nb : last;
    b_tile[n] = __builtin_amdgcn_readfirstlane((unsigned)nb * chunk_row);
  }
  int sg = (col0 >> 6) + wn;
  sg = sg < (p.N >> 6) - 1 ? sg : (p.N >> 6) - 1;
  const unsigned sb_tile = __builtin_amdgcn_readfirstlane((unsigned)sg * (unsigned)nk * 512u);
  const unsigned sa_tile = __builtin_amdgcn_readfirstlane((unsigned)tile_m * (unsigned)nk * 1024u);
  const unsigned b_lane = (unsigned)lane * 16, s_lane = (unsigned)lane * 8;
  typedef int i32x2 __attribute__((ext_vector_type(2)));
  i32x4 fb[NBUF][TN];
  i32x2 sbk[NBUF];  // B scales of K-step k in sbk[k mod 4]: tiles 2 d, 2 d + 1 in dword d
  i32x4 sak[NBUF];  // A scales of K-step k in sak[k mod 4]: tiles 2 d, 2 d + 1 in dword d
  auto load_b1 = [&](int j, auto buf, auto nc) {  // substep j = 2 k + u
    constexpr int BI = decltype(buf)::value;
    constexpr int n = decltype(nc)::value;
    const unsigned soff = b_tile[n] + (unsigned)j * 1024u;
    i32x4& dst = fb[BI][n];
    const unsigned voff = b_lane;
    const i32x4 rsrc = b_rsrc;
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff));
  };
  auto load_sb = [&](int k, auto buf) {
    constexpr int KB = decltype(buf)::value;
    const unsigned soff = sb_tile + (unsigned)k * 512u;
    i32x2& dst = sbk[KB];
    const unsigned voff = s_lane;
    const i32x4 rsrc = sb_rsrc;
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff));
  };
  auto load_sa = [&](int k, auto buf) {
    constexpr int KB = decltype(buf)::value;
    const unsigned soff = sa_tile + (unsigned)k * 1024u;
    i32x4& dst = sak[KB];
    const unsigned voff = b_lane;
    const i32x4 rsrc = sa_rsrc;
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff));
  };

  // ---- A: LDS -> fragment ring ---------------------------------------------------------------------
  const int li = lane & 15, lq = lane >> 4;
  typedef const __attribute__((address_space(3))) i32x4* lvec_t;
  unsigned rd_addr[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    rd_addr[s] = (unsigned)(size_t)AG_LDS(lds) + (unsigned)(li * kRowBytes + (((s * 4 + lq) ^ (li >> 1)) << 4));
    asm volatile("" : "+v"(rd_addr[s]));
  }
  i32x4 fa[RA];
  // fragment of m-step T (half T / TM, tile T % TM) of the K-step in ring slot KS
  auto read_a = [&](auto kslot, auto tt) {
    constexpr int KS = decltype(kslot)::value;
    constexpr int T = decltype(tt)::value;
    constexpr int OFF = KS * SLOT + (T % TM) * 16 * kRowBytes;
    fa[T % RA] = *(lvec_t)(size_t)(rd_addr[T / TM] + (unsigned)OFF);
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[m][n]));
    }

  // ---- prologue: B halves 0..3, the scales of K-steps 0 and 1, A(0..3) ------------------------------
  static_for<0, NBUF>([&](auto bc) {
    constexpr int J = decltype(bc)::value;
    if (J < 2 * nk) {
      static_for<0, TN>([&](auto nc) { load_b1(J, bc, nc); });
    }
  });
  load_sb(0, std::integral_constant<int, 0>{});
  load_sa(0, std::integral_constant<int, 0>{});
  load_sb(1, std::integral_constant<int, 1>{});
  load_sa(1, std::integral_constant<int, 1>{});
#pragma unroll
  for (int k = 0; k < NSLOT; ++k) {
    if (k < nk) {
#pragma unroll
      for (int j = 0; j < LH; ++j) issue_a1(k, k, j);
    }
  }
  // A(0) and everything older (B and the scales of K-steps 0 and 1) has landed when only the
  // transfers of A(1..3) may be in flight
  if (nk >= NSLOT) __builtin_amdgcn_s_waitcnt(waitcnt_imm((NSLOT - 1) * LH, 15));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  using K0 = std::integral_constant<int, 0>;
  static_for<0, RA - 1>([&](auto tc) { read_a(K0{}, tc); });
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop: trip k multiplies K-step k.  KM = k mod 4 fixes the A slot, the B buffers and
  // the scale registers at compile time.  VMW = loads that may still be in flight at the barrier;
  // VB0 / VB1 = loads that may still be in flight when tile 0 of the first / second half of B(k)
  // is needed (tile n: n fewer); NA, NB, NX: the trip requests A(k+4), requests B and the scales
  // of K-step k + 2, has a trip behind it.  VMW < 0: none of this is known at compile time;
  // every wait is for all loads and the requests are decided at run time. ----------------------------
  auto trip = [&](int k, auto kmod, auto vmw_c, auto vb0_c, auto vb1_c, auto na_c, auto nb_c, auto nx_c) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int VMW = decltype(vmw_c)::value;
    constexpr int VB0 = decltype(vb0_c)::value, VB1 = decltype(vb1_c)::value;
    constexpr bool KNOWN = VMW >= 0;
    using KS = std::integral_constant<int, KM>;
    using KN = std::integral_constant<int, (KM + 1) % NSLOT>;
    const bool has_next = KNOWN ? decltype(nx_c)::value : k + 1 < nk;
    const bool do_a = KNOWN ? decltype(na_c)::value : k + NSLOT < nk;
    const bool do_b = KNOWN ? decltype(nb_c)::value : k + 2 < nk;
    static_for<0, MS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      constexpr int U = T / TM, m = T % TM;
      constexpr int BI = (2 * KM + U) % NBUF;          // B buffer of this half
      using BIc = std::integral_constant<int, BI>;
      if constexpr (T == BAR) {
        if (has_next) {
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(KNOWN ? VMW : 0, 15));
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<0, TN>([&](auto nc) {
        constexpr int n = decltype(nc)::value;
        if constexpr (m == 0) {
          // tile n of this half of B(k); with tile 0 of the first half come the scales, which
          // were requested in front of it
          constexpr int VB = (U == 0 ? VB0 : VB1) - n;
          static_assert(!KNOWN || VB >= 0, "wait counts");
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(KNOWN ? VB : 0, 15));
          // the registers hold the loaded bytes from here on, not before
          asm volatile("" : "+v"(fb[BI][n]));
          if constexpr (U == 0 && n == 0) asm volatile("" : "+v"(sbk[KM]), "+v"(sak[KM]));
        }
        // scale bytes: B pairs {q, 4+q} of tiles 2 d, 2 d + 1 in the four bytes of sbk[KM][d]
        // -> byte 2 (n & 1) + U; A pairs the same way in sak[KM][m >> 1] -> byte 2 (m & 1) + U
#define AG_MFMA4DBL(SEL)                                                                    \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 " SEL " cbsz:4 blgp:4" \
               : "+a"(acc[m][n])                                                            \
               : "v"(fb[BI][n]), "v"(fa[T % RA]), "v"(sbk[KM][n >> 1]), "v"(sak[KM][m >> 1]))
        if constexpr ((m & 1) == 0) {
          if constexpr (U == 0 && (n & 1) == 0) AG_MFMA4DBL("op_sel:[0,0,0] op_sel_hi:[0,0,0]");
          else if constexpr (U == 0) AG_MFMA4DBL("op_sel:[0,0,0] op_sel_hi:[1,0,0]");
          else if constexpr ((n & 1) == 0) AG_MFMA4DBL("op_sel:[1,1,0] op_sel_hi:[0,0,0]");
          else AG_MFMA4DBL("op_sel:[1,1,0] op_sel_hi:[1,0,0]");
        } else {
          if constexpr (U == 0 && (n & 1) == 0) AG_MFMA4DBL("op_sel:[0,0,0] op_sel_hi:[0,1,0]");
          else if constexpr (U == 0) AG_MFMA4DBL("op_sel:[0,0,0] op_sel_hi:[1,1,0]");
          else if constexpr ((n & 1) == 0) AG_MFMA4DBL("op_sel:[1,1,0] op_sel_hi:[0,1,0]");
          else AG_MFMA4DBL("op_sel:[1,1,0] op_sel_hi:[1,1,0]");
        }
#undef AG_MFMA4DBL
        // ---- at most two side instructions behind an MFMA ---------------------------------------
        if constexpr (n == 0) {
          // the fragment three m-steps ahead: this K-step's, or behind the barrier the next one's
          if constexpr (T + RA - 1 < MS) read_a(KS{}, std::integral_constant<int, T + RA - 1>{});
          else if (has_next) read_a(KN{}, std::integral_constant<int, T + RA - 1 - MS>{});
        }
        // A(k+4) into the slot this K-step leaves: transfers 0..2 at m-step BAR, 3 at BAR + 1
        if constexpr (T == BAR && n >= 1) {
          if (do_a) issue_a1(k + NSLOT, KM, n - 1);
        }
        if constexpr (T == BAR + 1 && n == 1) {
          if (do_a) issue_a1(k + NSLOT, KM, 3);
        }
        // last m-step of a half: tile n of this buffer is done with MFMA (m = 7, n).  The scales
        // of K-step k + 2 go first in the first half's batch.
        if constexpr (m == TM - 1) {
          if constexpr (U == 0 && n == 0) {
            if (do_b) {
              load_sb(k + 2, std::integral_constant<int, (KM + 2) % NBUF>{});
              load_sa(k + 2, std::integral_constant<int, (KM + 2) % NBUF>{});
            }
          }
          if (do_b) load_b1(2 * (k + 2) + U, BIc{}, nc);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  // Loads of a full trip in issue order: B's scales, A's scales and 4 B loads (m-step 7, first
  // half), behind the barrier 4 A transfers (m-steps 13, 14), then 4 B loads (m-step 15): TL = 14,
  // of which TB = 6 in front of the barrier.
  //   First half of B(k), tile 0: requested in trip k - 2 behind the two scale loads; behind it
  //     3 B loads, 4 transfers and 4 B loads of that trip and the loads of trip k - 1.
  //   Second half, tile 0: behind it 3 B loads of trip k - 2, the loads of trip k - 1 and the
  //     first batch of this trip.
  //   A(k+1) at the barrier, requested in trip k - 3: behind it the 4 B loads of that trip's
  //     second half, two trips and the first batch of this one.  Trips 0..2: A(k+1) was
  //     requested in the prologue, followed there by A(k+2..3).
  //   B(0), B(1) and their scales have landed before the loop (the prologue's wait): the counts
  //     of the steady state are above what can be in flight in trips 0 and 1.
  // The last four trips t0..t3 = nk - 4 .. nk - 1 request no A and only t0, t1 request B
  // (10 loads each).
  constexpr int TL = 14, TB = 6;
  constexpr int VB0_S = 3 + LH + TN + TL, VB1_S = 3 + TL + TB, VMW_S = TN + 2 * TL + TB;
  using T_ = std::true_type;
  using F_ = std::false_type;
  auto group = [&](int k0, auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int VM = (FIRST && I <= NSLOT - 2) ? (NSLOT - 2 - I) * LH + TL * I + TB : VMW_S;
      trip(k0 + I, ic, std::integral_constant<int, VM>{}, std::integral_constant<int, VB0_S>{},
           std::integral_constant<int, VB1_S>{}, T_{}, T_{}, T_{});
    });
  };
  auto last_group = [&](int k0) {
    constexpr int NB = TB + TN;  // loads of a trip that requests no A
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      // t0: everything behind is steady.  t1: trip t0 behind B(t1) had no transfers.  t2: B(t2)
      // was requested in t0, behind it t0's second half and t1.  t3: requested in t1, nothing since.
      constexpr int VB0 = I == 0 ? VB0_S : I == 1 ? 3 + LH + TN + NB : I == 2 ? 3 + TN + NB : 3 + TN;
      constexpr int VB1 = I == 0 ? VB1_S : I == 1 ? 3 + NB + TB : I == 2 ? 3 + NB : 3;
      constexpr int VM = I == 0 ? VMW_S : I == 1 ? TN + TL + NB + TB : TN + 2 * NB;
      trip(k0 + I, ic, std::integral_constant<int, VM>{}, std::integral_constant<int, VB0>{},
           std::integral_constant<int, VB1>{}, F_{}, std::integral_constant<bool, (I < 2)>{},
           std::integral_constant<bool, (I < 3)>{});
    });
  };
  using NEG = std::integral_constant<int, -1>;
  int k = 0;
  // a steady group of four trips requests A up to K-step k + 7, B and scales up to K-step k + 5
  if (nk >= 2 * NSLOT) {
    group(0, T_{});
#pragma unroll 1
    for (k = NSLOT; k + 2 * NSLOT <= nk; k += NSLOT) group(k, F_{});
    if (k + NSLOT == nk) {
      last_group(k);
      k = nk;
    }
  }
#pragma unroll 1
  for (; k < nk; k += NSLOT) {
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      if (I == 0 || k + I < nk) trip(k + I, ic, NEG{}, NEG{}, NEG{}, F_{}, F_{}, F_{});
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, row0, col0);
}

template <int DT, int OUT>
__global__ __launch_bounds__(256, 2) void gemm_stream4dbl_kernel(const GemmArgs p) {
  gemm_stream4dbl_body<DT, OUT>(p, blockIdx.x);
}

}  // namespace
}  // namespace astergemm
