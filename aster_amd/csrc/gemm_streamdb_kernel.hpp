// Stream kernel with B straight from global memory into MFMA operand registers ("direct B"),
// 16-bit operands, 256x256 workgroup tile with 2x4 waves or 128x256 with 1x4 waves (the
// reference's own best mapping: no two waves of a workgroup fetch the same B, two workgroups
// of four waves per CU): the operand path of the reference's best
// gfx950 kernel (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:75-324:
// A through LDS by direct-to-LDS transfers, B pre-shuffled on the host so that one
// global_load_dwordx4 per lane is an MFMA operand) on this build's staging, swizzle, tile map
// and epilogue.
//
// B layout ("K8 order", astergemm_shuffle_weight_k8_16): chunks of 1 KiB, chunk (nb, kb) holds
// rows 16 nb .. 16 nb + 15 and K elements 32 kb .. 32 kb + 31; lane L = 16 g + n of a wave finds
// at byte 16 L of the chunk the eight consecutive K elements 32 kb + 8 g .. + 7 of row 16 nb + n,
// which is what v_mfma_f32_16x16x32 wants from lane L, and what a ds_read_b128 of granule
// 4 s + g of a 128-byte LDS row gives the same lane for A.  (The reference's shuffle_weight
// pairs K elements {4g..4g+3} and {16+4g..16+4g+3}, the order of two ds_read_b64; 16-byte LDS
// reads are four times as fast on this chip, so the B order follows them.)
//
// What changes against gemm_stream_body:
//   * LDS holds only A: a ring of five 32 KiB slots, A(k) in slot k mod 5, A(k+5) requested when
//     K-step k has been read; LDS reads per MFMA drop from 12/32 to 8/32 and LDS writes halve.
//   * B fragments live in five register buffers of one MFMA substep each (4 tiles x 4
//     registers); the buffer of substep j is refilled with substep j + 5 as its last MFMAs
//     issue, two K-steps before the data is needed.  The two waves that share B columns
//     (wave rows 0 and 1) fetch the same lines; the second fetch is an L1 / L2 hit.
//   * MFMA order is m-outer: an A fragment is read from LDS three m-steps ahead into a ring of
//     four, multiplied with the four B fragments and dropped, so A fragments cost 16 registers
//     instead of 64 and the B buffers fit (128 accumulation registers; 80 + 16 architectural).
//   * one barrier per K-step, three m-steps before its end: it certifies A(k+1) (every wave has
//     waited for its own transfers) and, since all reads of A(k) have been issued by then,
//     frees slot k mod 5.
// vmcnt bookkeeping: per K-step a wave issues, in this order, 4 B loads (end of substep 0),
// 4 A transfers (behind the barrier), 4 B loads (end of substep 1).  The B loads are ordinary
// loads (the compiler waits for them itself, conservatively, because it does not see the
// transfers); the wait in front of the barrier is counted by hand.
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT, int NSLOT, int NBUF, int WM>
__device__ __forceinline__ void gemm_streamdb_body(const GemmArgs& p, int bid) {
  constexpr int BM = 128 * WM, BN = 256, WN = 4;
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;      // 8
  constexpr int TN = BN / WN / 16;      // 4
  constexpr int SLOT = BM * kRowBytes;  // 32 (16) KiB: A rows of one K-step
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 4 transfers of 1 KiB per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  // NSLOT A slots in LDS, NBUF B register buffers of one MFMA substep each; the loop is unrolled
  // over NSLOT trips, after which slot and buffer numbers repeat
  static_assert(NBUF == NSLOT || NBUF == 2 * NSLOT, "buffer numbers repeat with the slots");
  // (three slots and six buffers, which waits for B a K-step later, was measured at the same
  // speed and is not built)
  static_assert(NSLOT == 5 && NBUF == 5, "the configuration that is tested");
  constexpr int AHEAD = NSLOT > (NBUF + 2) / 2 ? NSLOT : (NBUF + 2) / 2;  // K-steps requested ahead
  constexpr int RA = 4;                 // A fragment ring
  constexpr int MS = 2 * TM;            // m-steps per K-step
  constexpr int BAR = MS - (RA - 1);    // m-step whose first slot carries the barrier
  static_assert(DT == ASTERGEMM_BF16 || DT == ASTERGEMM_F16, "16-bit operands");
  static_assert(WM == 1 || WM == 2, "one or two wave rows of 128 rows each");
  static_assert(MS % RA == 0, "the A fragment ring is in phase at every K-step");
  static_assert(TN == 4 && LH == 4, "side-instruction schedule below");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  int tile_m, tile_n;
  map_tile(bid, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const int nk = p.ksteps;

  // ---- A: global -> LDS, as in gemm_stream_body ------------------------------------------------
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

  // ---- B: global -> registers.  Scalar base of the wave's n-tile `n` (16 rows of B, clamped to
  // the last 16 rows for edge tiles), substep j at + j KiB, lane at + 16 lane. ---------------------
  // One buffer resource over the whole of B; a load is resource + scalar offset (n-tile and
  // substep) + per-lane offset, so no address lives in vector registers.
  const unsigned chunk_row = (unsigned)(p.K >> 5) * 1024u;  // bytes of 16 rows of B
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.B, 0, (int)((unsigned)(p.N >> 4) * chunk_row), 0x00020000);
  unsigned b_tile[TN];
#pragma unroll
  for (int n = 0; n < TN; ++n) {
    int nb = (col0 >> 4) + wn * TN + n;
    const int last = (p.N >> 4) - 1;
    nb = nb < last ? nb : last;
    b_tile[n] = __builtin_amdgcn_readfirstlane((unsigned)nb * chunk_row);
  }
  const unsigned b_lane = (unsigned)lane * 16;
  i32x4 fb[NBUF][TN];
  auto load_b1 = [&](int j, auto buf, int n) {
    constexpr int BI = decltype(buf)::value;
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_lane,
                                                          (int)(b_tile[n] + (unsigned)j * 1024u), 0);
    fb[BI][n] = __builtin_bit_cast(i32x4, v);
  };

  // ---- A: LDS -> fragment ring -------------------------------------------------------------------
  const int li = lane & 15, lq = lane >> 4;
  // LDS byte address of this lane's granule in row 0 of the wave's A rows, per substep and per
  // 64 KiB of the ring (a ds_read offset field holds 16 bits): six registers, opaque to the
  // optimiser so that it does not keep one hoisted address per read instead
  typedef const __attribute__((address_space(3))) i32x4* lvec_t;
  constexpr int NG = (NSLOT * SLOT + 65535) / 65536;
  unsigned rd_addr[NG][2];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      rd_addr[g][s] = (unsigned)(size_t)AG_LDS(lds) + (unsigned)(g * 65536) +
                      (unsigned)(li * kRowBytes + (((s * 4 + lq) ^ (li >> 1)) << 4)) +
                      (unsigned)(wm * TM * 16 * kRowBytes);
      asm volatile("" : "+v"(rd_addr[g][s]));
    }
  i32x4 fa[RA];
  // fragment of m-step T (substep T / TM, tile T % TM) of the K-step in ring slot KS
  auto read_a = [&](auto kslot, auto tt) {
    constexpr int KS = decltype(kslot)::value;
    constexpr int T = decltype(tt)::value;
    constexpr int OFF = KS * SLOT + (T % TM) * 16 * kRowBytes;
    fa[T % RA] = *(lvec_t)(size_t)(rd_addr[OFF >> 16][T / TM] + (unsigned)(OFF & 65535));
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      // accumulators in the accumulation half of the register file, destination tied to the
      // addend: 128 architectural registers stay for the B buffers, the A ring and addresses
      asm volatile("" : "+a"(acc[m][n]));
    }

  // ---- prologue: B substeps 0..4 and A(0..4) requested; A(0) landed; first fragments read -------
  static_for<0, NBUF>([&](auto bc) {
    constexpr int J = decltype(bc)::value;
    if (J < 2 * nk) {
#pragma unroll
      for (int n = 0; n < TN; ++n) load_b1(J, bc, n);
    }
  });
  asm volatile("" ::: "memory");
#pragma unroll
  for (int k = 0; k < NSLOT; ++k) {
    if (k < nk) {
#pragma unroll
      for (int j = 0; j < LH; ++j) issue_a1(k, k, j);
    }
  }
  // A(0) is older than the transfers of A(1..NSLOT-1): only those may still be in flight
  if (nk >= NSLOT) __builtin_amdgcn_s_waitcnt(waitcnt_imm((NSLOT - 1) * LH, 15));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  using K0 = std::integral_constant<int, 0>;
  static_for<0, RA - 1>([&](auto tc) { read_a(K0{}, tc); });
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop: trip k multiplies K-step k.  KM = k mod 5 fixes the A slot and the B buffers at
  // compile time; VMW = loads that may still be in flight at the barrier (0 = wait for all). -----
  auto trip = [&](int k, auto kmod, auto vmw_c) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int VMW = decltype(vmw_c)::value;
    constexpr bool STEADY = VMW > 0;
    using KS = std::integral_constant<int, KM>;
    using KN = std::integral_constant<int, (KM + 1) % NSLOT>;
    const bool has_next = STEADY || k + 1 < nk;
    const bool do_a = STEADY || k + NSLOT < nk;
    static_for<0, MS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      constexpr int S = T / TM, m = T % TM;
      constexpr int BI = (2 * KM + S) % NBUF;          // B buffer of this substep
      using BIc = std::integral_constant<int, BI>;
      const int j = 2 * k + S;                         // substep index along K
      const bool do_b = STEADY || j + NBUF < 2 * nk;
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
        stream_mma<DT, true>(fb[BI][n], fa[T % RA], acc[m][n]);
        // ---- at most two side instructions behind an MFMA -------------------------------------
        if constexpr (n == 0) {
          // the fragment three m-steps ahead: this K-step's, or behind the barrier the next one's
          if constexpr (T + RA - 1 < MS) read_a(KS{}, std::integral_constant<int, T + RA - 1>{});
          else if (has_next) read_a(KN{}, std::integral_constant<int, T + RA - 1 - MS>{});
        }
        // A(k+5) into the slot this K-step leaves: transfers 0..2 at m-step BAR, 3 at BAR + 1
        if constexpr (T == BAR && n >= 1) {
          if (do_a) issue_a1(k + NSLOT, KM, n - 1);
        }
        if constexpr (T == BAR + 1 && n == 1) {
          if (do_a) issue_a1(k + NSLOT, KM, 3);
        }
        // last m-step of a substep: tile n of this buffer is done with MFMA (m = 7, n)
        if constexpr (m == TM - 1) {
          if (do_b) load_b1(j + NBUF, BIc{}, n);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  // loads younger than the transfers of A(k+1) at the barrier of trip k, steady state: the 4 B
  // loads that followed them in trip k+1-NSLOT, 12 loads in each of the NSLOT-2 trips between,
  // 4 B loads of trip k.  Trips 0..NSLOT-2: A(k+1) was requested in the prologue, followed there
  // by A(k+2..NSLOT-1) and here by 12 loads per earlier trip and 4 of this one.
  constexpr int VM_STEADY = 4 + (NSLOT - 2) * 12 + 4;
  auto group = [&](int k0, auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int VM = (FIRST && I <= NSLOT - 2) ? (NSLOT - 2 - I) * LH + 12 * I + 4 : VM_STEADY;
      trip(k0 + I, ic, std::integral_constant<int, VM>{});
    });
  };
  using WZ = std::integral_constant<int, 0>;
  int k = 0;
  // a steady group of NSLOT trips requests A up to K-step k + 2 NSLOT - 1 and B up to substep
  // 2 (k + NSLOT - 1) + 1 + NBUF
  if (nk >= NSLOT + AHEAD) {
    group(0, std::true_type{});
    // (entered only from the group above: the compiler's own wait counts for the B loads then
    // see the same history on both ways into the loop header and stay exact)
#pragma unroll 1
    for (k = NSLOT; k + NSLOT + AHEAD <= nk; k += NSLOT) group(k, std::false_type{});
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

// WM = 1: four waves and 80 KiB per workgroup, two workgroups per CU (at most 256 registers per
// wave, which the second launch bound asks for)
template <int DT, int OUT, int NSLOT, int NBUF, int WM = 2>
__global__ __launch_bounds__(WM * 256, 2) void gemm_streamdb_kernel(const GemmArgs p) {
  gemm_streamdb_body<DT, OUT, NSLOT, NBUF, WM>(p, blockIdx.x);
}

}  // namespace
}  // namespace astergemm
