// MXFP4 stream kernel with B straight from global memory into MFMA operand registers: the
// structure of gemm_streamdb_kernel.hpp at the reference's own best geometry (128 x 256 workgroup
// tile, four waves in a 1 x 4 grid, two workgroups per CU; contrib/kittens/test/
// test_102_gemm_python_multitile_g2s_directb_cdna4.py:75-324) with
// v_mfma_scale_f32_16x16x128_f8f6f4 (cbsz = blgp = 4) as the inner instruction.
//
// Why for fp4: the LDS kernel (gemm_stream4_kernel.hpp) has room for two K-steps of A and B in
// the 160 KiB, so every transfer is waited for one K-step after it was requested, by all eight
// waves at one barrier.  Here LDS holds only A, 16 KiB per K-step: a ring of four slots, A(k+4)
// requested when K-step k has been read, and B is two K-steps ahead in registers; a workgroup is
// four waves and 68 KiB, two share a CU and cover each other's barrier waits.
//
// B layouts (pre-shuffled by the host, astergemm_shuffle_weight_8 and
// astergemm_shuffle_scales_e8m0_lanes):
//   payload, "step order": 1 KiB chunks; chunk ((nb * steps + s) * 2 + u) holds for rows
//     16 nb .. 16 nb + 15 and 128-byte step s the granules 4 u .. 4 u + 3: lane L = 16 q + n finds
//     at byte 16 L granule 4 u + q of row 16 nb + n, the operand of MFMA u of that step.
//   e8m0 plane, "lane order": 512-byte chunks; chunk (nb4 * steps + s) holds for rows
//     64 nb4 .. 64 nb4 + 63 and step s, at byte 8 L + 2 t + h of lane L = 16 q + i, the scale of
//     block 4 h + q of row 64 nb4 + 16 t + i: one 8-byte load per wave and K-step brings the
//     scales of the wave's four B tiles, and the MFMAs select their byte with op_sel.
// A and its e8m0 plane are row-major.  A's scales go through LDS as in the LDS kernel (16 bytes
// per row = one chunk of two K-steps, re-packed into byte pairs {block q, block 4 + q}, here
// one plane of 8 bytes per row for each of the two K-steps), but by
// ordinary loads: a lane fetches one row's granule, re-packs it in registers and writes it
// (waves 2 and 3 repeat what waves 0 and 1 do, which keeps the loop free of branches), so that
// only the A tile transfers are counted by hand.
//
// MFMA order is m-outer per half K-step: m-step T = 8 u + m multiplies A fragment (m, u), read
// from LDS three m-steps ahead into a ring of four, with the four B fragments of half u.
// One barrier per K-step, three m-steps before its end: it certifies A(k+1) and, all reads of
// A(k) having been issued, frees slot k mod 4.
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT>
__device__ __forceinline__ void gemm_stream4db_body(const GemmArgs& p, int bid) {
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
  constexpr int SC_A = NSLOT * SLOT;    // A scales: [2 buffers][2 K-step parities][128 rows][8 bytes]
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
  const int nk = p.ksteps;  // even (the launcher checks): a scale chunk is two K-steps

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

  // ---- A scales: a wave brings chunk c (K-steps 2c, 2c+1) of 64 rows, lane L the 16 bytes of
  // row 64 (w & 1) + L, re-packed into pairs {b[8h+q], b[8h+4+q]} (h = K-step parity) -------------
  int sc_row = row0 + (wave & 1) * 64 + lane;
  sc_row = sc_row < p.M ? sc_row : p.M - 1;  // rows past the end of an edge tile re-read the last
  const uint8_t* sc_src = p.mx_a + (int64_t)sc_row * p.mx_ld;
  uint8_t* sc_dst = lds + SC_A + ((wave & 1) * 64 + lane) * 8;
  i32x4 sc_raw = {0, 0, 0, 0};
  auto load_scales = [&](int c) { sc_raw = *(const i32x4*)(sc_src + c * 16); };
  auto store_scales = [&](int c) {
    i32x4 r;
    // v_perm_b32(hi, lo, sel): selector bytes 0-3 index lo, 4-7 index hi
    r.x = (int)__builtin_amdgcn_perm((unsigned)sc_raw.y, (unsigned)sc_raw.x, 0x05010400u);
    r.y = (int)__builtin_amdgcn_perm((unsigned)sc_raw.y, (unsigned)sc_raw.x, 0x07030602u);
    r.z = (int)__builtin_amdgcn_perm((unsigned)sc_raw.w, (unsigned)sc_raw.z, 0x05010400u);
    r.w = (int)__builtin_amdgcn_perm((unsigned)sc_raw.w, (unsigned)sc_raw.z, 0x07030602u);
    // the pairs of a K-step parity lie 8 bytes apart from row to row: the 16 rows of a tile are
    // 128 contiguous bytes, which 64 lanes read without a bank conflict
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    *(i32x2*)(sc_dst + (c & 1) * BM * 16) = i32x2{r.x, r.y};
    *(i32x2*)(sc_dst + (c & 1) * BM * 16 + BM * 8) = i32x2{r.z, r.w};
  };

  // ---- B: global -> registers.  One buffer resource over the payload and one over the scale
  // plane; a load is resource + scalar offset + per-lane offset.  The hardware's range check does
  // not cover the scalar offset, so the block indices of an edge tile are clamped to the last
  // 16-row block of B and the last 64-row group of the plane (those columns are never stored). ------
  const unsigned chunk_row = (unsigned)(p.K >> 7) * 1024u;  // bytes of 16 rows of B (K/2 per row)
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.B, 0, (int)((unsigned)(p.N >> 4) * chunk_row), 0x00020000);
  const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.mx_b, 0, (int)((unsigned)(p.N >> 6) * (unsigned)nk * 512u), 0x00020000);
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
  const unsigned s_tile = __builtin_amdgcn_readfirstlane((unsigned)sg * (unsigned)nk * 512u);
  const unsigned b_lane = (unsigned)lane * 16, s_lane = (unsigned)lane * 8;
  i32x4 fb[NBUF][TN];
  int sbk[NBUF][2];  // scales of K-step k in sbk[k mod 4]
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  auto load_b1 = [&](int j, auto buf, int n) {  // substep j = 2 k + u
    constexpr int BI = decltype(buf)::value;
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_lane,
                                                          (int)(b_tile[n] + (unsigned)j * 1024u), 0);
    fb[BI][n] = __builtin_bit_cast(i32x4, v);
  };
  auto load_sb = [&](int k, auto buf) {
    constexpr int KB = decltype(buf)::value;
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, (int)s_lane,
                                                         (int)(s_tile + (unsigned)k * 512u), 0);
    sbk[KB][0] = (int)v.x;
    sbk[KB][1] = (int)v.y;
  };

  // ---- A: LDS -> fragment ring ---------------------------------------------------------------------
  const int li = lane & 15, lq = lane >> 4;
  typedef const __attribute__((address_space(3))) i32x4* lvec_t;
  typedef const __attribute__((address_space(3))) unsigned short* lu16_t;
  unsigned rd_addr[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    rd_addr[s] = (unsigned)(size_t)AG_LDS(lds) + (unsigned)(li * kRowBytes + (((s * 4 + lq) ^ (li >> 1)) << 4));
    asm volatile("" : "+v"(rd_addr[s]));
  }
  unsigned sc_addr = (unsigned)(size_t)AG_LDS(lds) + (unsigned)(SC_A + li * 8 + lq * 2);
  asm volatile("" : "+v"(sc_addr));
  i32x4 fa[RA];
  int sa[TM];
  // fragment of m-step T (half T / TM, tile T % TM) of the K-step in ring slot KS; with the first
  // half comes the tile's scale pair (scale buffer (k / 2) mod 2, parity plane k mod 2)
  auto read_a = [&](auto kslot, auto tt) {
    constexpr int KS = decltype(kslot)::value;
    constexpr int T = decltype(tt)::value;
    constexpr int OFF = KS * SLOT + (T % TM) * 16 * kRowBytes;
    fa[T % RA] = *(lvec_t)(size_t)(rd_addr[T / TM] + (unsigned)OFF);
    if constexpr (T < TM) {
      constexpr int SOFF = ((KS >> 1) & 1) * BM * 16 + (KS & 1) * BM * 8 + T * 16 * 8;
      sa[T] = *(lu16_t)(size_t)(sc_addr + (unsigned)SOFF);
    }
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[m][n]));
    }

  // ---- prologue: B halves 0..3 and their scales, A(0..3), scale chunks 0 and 1 --------------------
  static_for<0, NBUF>([&](auto bc) {
    constexpr int J = decltype(bc)::value;
    if (J < 2 * nk) {
#pragma unroll
      for (int n = 0; n < TN; ++n) load_b1(J, bc, n);
    }
  });
  load_sb(0, std::integral_constant<int, 0>{});
  load_sb(1, std::integral_constant<int, 1>{});
  load_scales(0);
  store_scales(0);
  if (nk > 2) {
    load_scales(1);
    store_scales(1);
  }
  asm volatile("" ::: "memory");
#pragma unroll
  for (int k = 0; k < NSLOT; ++k) {
    if (k < nk) {
#pragma unroll
      for (int j = 0; j < LH; ++j) issue_a1(k, k, j);
    }
  }
  // A(0) is older than the transfers of A(1..3): only those may still be in flight; the scale
  // writes of this wave have been issued (LDS operations of a wave complete in order)
  if (nk >= NSLOT) __builtin_amdgcn_s_waitcnt(waitcnt_imm((NSLOT - 1) * LH, 0));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  using K0 = std::integral_constant<int, 0>;
  static_for<0, RA - 1>([&](auto tc) { read_a(K0{}, tc); });
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop: trip k multiplies K-step k.  KM = k mod 4 fixes the A slot, the B buffers and
  // the scale registers at compile time; VMW = loads that may still be in flight at the barrier
  // (0 = wait for all). ---------------------------------------------------------------------------------
  auto trip = [&](int k, auto kmod, auto vmw_c) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int VMW = decltype(vmw_c)::value;
    constexpr bool STEADY = VMW > 0;
    using KS = std::integral_constant<int, KM>;
    using KN = std::integral_constant<int, (KM + 1) % NSLOT>;
    constexpr bool ODD = (KM & 1) != 0;
    const bool has_next = STEADY || k + 1 < nk;
    const bool do_a = STEADY || k + NSLOT < nk;
    const bool do_b = STEADY || k + 2 < nk;   // K-step k + 2 exists: both halves and the scales
    const bool do_sc = STEADY || k + 3 < nk;  // odd k: chunk (k + 3) / 2 exists
    static_for<0, MS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      constexpr int U = T / TM, m = T % TM;
      constexpr int BI = (2 * KM + U) % NBUF;          // B buffer of this half
      using BIc = std::integral_constant<int, BI>;
      if constexpr (T == BAR) {
        if (has_next) {
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(VMW, 15));
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<0, TN>([&](auto nc) {
        constexpr int n = decltype(nc)::value;
        // scale bytes: A pair {q, 4+q} in bytes 0, 1 of sa[m] -> byte U; B pairs of tiles
        // 2 d, 2 d + 1 in the four bytes of sbk[KM][d] -> byte 2 (n & 1) + U
#define AG_MFMA4DB(SEL)                                                                     \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 " SEL " cbsz:4 blgp:4" \
               : "+a"(acc[m][n])                                                            \
               : "v"(fb[BI][n]), "v"(fa[T % RA]), "v"(sbk[KM][n >> 1]), "v"(sa[m]))
        if constexpr (U == 0 && (n & 1) == 0) AG_MFMA4DB("op_sel:[0,0,0] op_sel_hi:[0,0,0]");
        else if constexpr (U == 0) AG_MFMA4DB("op_sel:[0,0,0] op_sel_hi:[1,0,0]");
        else if constexpr ((n & 1) == 0) AG_MFMA4DB("op_sel:[1,1,0] op_sel_hi:[0,0,0]");
        else AG_MFMA4DB("op_sel:[1,1,0] op_sel_hi:[1,0,0]");
#undef AG_MFMA4DB
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
        // odd trips: chunk (k + 3) / 2 is fetched behind the barrier that freed its buffer (last
        // read at m-step 4 of this trip) and written at m-step 4 of the next odd trip, nine
        // m-steps ahead of the barrier behind which it is first read.  Written there and not
        // earlier because the compiler's wait for the fetched granule counts only the loads it
        // sees: one trip after the fetch it would also force the A transfers requested beside
        // it, two trips after it forces nothing that is not needed by then anyway.
        if constexpr (ODD && T == 4 && n == 2) {
          if (STEADY || k + 1 < nk) {
            if (k > 1) store_scales((k + 1) >> 1);
          }
        }
        if constexpr (ODD && T == BAR + 1 && n == 2) {
          if (do_sc) load_scales((k + 3) >> 1);
        }
        // last m-step of a half: tile n of this buffer is done with MFMA (m = 7, n).  The B
        // scales of K-step k + 2 go first in the first half's batch, so that the wait for them
        // two trips on has this batch and a whole trip of loads behind it.
        if constexpr (m == TM - 1) {
          if constexpr (U == 0 && n == 0) {
            if (do_b) load_sb(k + 2, std::integral_constant<int, (KM + 2) % NBUF>{});
          }
          if (do_b) load_b1(2 * (k + 2) + U, BIc{}, n);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  // Loads of a trip in issue order: one B-scale load and 4 B loads (first half, m-step 7), the
  // barrier, 4 A transfers (m-steps 13, 14), on odd trips one A-scale load, 4 B loads (m-step 15).
  // Younger than the transfers of A(k+1) at the barrier of trip k, steady state, counted from
  // below (a smaller count only waits for loads that are older and long complete): 4 behind them
  // in trip k - 3, 13 in each of the two trips between, 5 of trip k; the A-scale loads of odd
  // trips are not counted.  Trips 0..2: A(k+1) was requested in the prologue, followed there by
  // A(k+2..3) and here by 13 loads per earlier trip and 5 of this one.
  constexpr int VM_STEADY = 4 + 2 * 13 + 5;
  auto group = [&](int k0, auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int VM = (FIRST && I <= NSLOT - 2) ? (NSLOT - 2 - I) * LH + 13 * I + 5 : VM_STEADY;
      trip(k0 + I, ic, std::integral_constant<int, VM>{});
    });
  };
  using WZ = std::integral_constant<int, 0>;
  int k = 0;
  // a steady group of four trips requests A up to K-step k + 7, B and scales up to K-step k + 5
  // and scale chunk (k + 6) / 2
  if (nk >= 2 * NSLOT) {
    group(0, std::true_type{});
#pragma unroll 1
    for (k = NSLOT; k + 2 * NSLOT <= nk; k += NSLOT) group(k, std::false_type{});
  }
#pragma unroll 1
  for (; k < nk; k += NSLOT) {
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      if (I == 0 || k + I < nk) trip(k + I, ic, WZ{});
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, row0, col0);
}

template <int DT, int OUT>
__global__ __launch_bounds__(256, 2) void gemm_stream4db_kernel(const GemmArgs p) {
  gemm_stream4db_body<DT, OUT>(p, blockIdx.x);
}

}  // namespace
}  // namespace astergemm
