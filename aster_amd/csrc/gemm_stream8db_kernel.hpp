// fp8 (e4m3) stream kernel with B straight from global memory into MFMA operand registers: the
// structure of gemm_stream4db_kernel.hpp (128 x 256 workgroup tile, four waves in a 1 x 4 grid,
// two workgroups per CU; the reference's direct-B geometry, contrib/kittens/test/
// test_102_gemm_python_multitile_g2s_directb_cdna4.py:75-324) with the unscaled
// v_mfma_f32_16x16x128_f8f6f4 as the inner instruction.
//
// B is pre-shuffled into step order (astergemm_shuffle_weight_8): 1 KiB chunks, chunk
// ((nb * steps + s) * 2 + u) holds for rows 16 nb .. 16 nb + 15 and 128-byte step s the granules
// 4 u .. 4 u + 3; lane L = 16 q + n finds at byte 16 L granule 4 u + q of row 16 nb + n.  The
// 32-byte operand of a lane is {granule q, granule 4 + q}: the loads of chunks u = 0 and u = 1.
// A is row-major and goes through an LDS ring of four K-steps as in the other stream kernels.
//
// MFMA order is m-outer: m-step m multiplies A fragment m, read from LDS three m-steps ahead into
// a ring of four, with the four B fragments of the K-step.  B is two K-steps ahead in two
// register buffers; tile n of a buffer is re-loaded behind its last MFMA (m = 7).  One barrier
// per K-step, three m-steps before its end: it certifies A(k+1) and, all reads of A(k) having
// been issued, frees slot k mod 4 for A(k+4).
//
// Every load of the loop is counted by hand (loads retire in issue order): the B loads are
// inline assembly like the A transfers, because the compiler, which does not see the transfers,
// would wait for B(k) with a count that also forces the transfers of the trip before, requested
// only three m-steps earlier.
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT>
__device__ __forceinline__ void gemm_stream8db_body(const GemmArgs& p, int bid) {
  constexpr int BM = 128, BN = 256, WM = 1, WN = 4;
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;      // 8
  constexpr int TN = BN / WN / 16;      // 4
  constexpr int SLOT = BM * kRowBytes;  // 16 KiB: A rows of one K-step
  constexpr int NSLOT = 4;              // A ring
  constexpr int NBUF = 2;               // B register buffers of one K-step each
  using Plan = StreamLoadPlan<BM, NW>;  // the staging as a cooperative load plan (stream_load_plan.inc)
  constexpr int LH = Plan::LH;       // 4 transfers of 1 KiB per wave and slot
  static_assert(Plan::TILE_ROWS == 8 && Plan::TILE_LDS_BYTES == 8 * kRowBytes, "transfer tile");
  constexpr int RA = 4;                 // A fragment ring
  constexpr int MS = TM;                // m-steps per K-step
  constexpr int BAR = MS - (RA - 1);    // m-step whose first MFMA follows the barrier
  constexpr int TRIP_LOADS = LH + 2 * TN;  // loads of one trip: the A transfers, then the B loads
  static_assert(DT == ASTERGEMM_FP8_E4M3, "fp8 operands");
  static_assert(TN == 4 && LH == 4 && BAR + 1 < MS - 1, "side-instruction schedule below");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave;

  int tile_m, tile_n;
  map_tile(bid, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const int nk = p.ksteps;

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

  // ---- B: global -> registers.  A raw buffer over the payload; a load is resource + scalar
  // offset + lane offset + the chunk's immediate.  The hardware's range check covers the lane
  // offset and the immediate only, not the scalar offset, so the 16-row block index of an edge
  // tile is clamped to the last block of B here (those columns are never stored). ------------------
  const unsigned chunk_row = (unsigned)nk * 2048u;  // bytes of 16 rows of B
  const uint64_t b_addr = (uint64_t)(uintptr_t)p.B;
  const i32x4 b_rsrc = {(int)(unsigned)b_addr, (int)((unsigned)(b_addr >> 32) & 0xffffu),
                        (int)((unsigned)(p.N >> 4) * chunk_row), 0x00020000};
  unsigned b_tile[TN];
#pragma unroll
  for (int n = 0; n < TN; ++n) {
    int nb = (col0 >> 4) + wn * TN + n;
    const int last = (p.N >> 4) - 1;
    nb = nb < last ? nb : last;
    b_tile[n] = __builtin_amdgcn_readfirstlane((unsigned)nb * chunk_row);
  }
  const unsigned b_lane = (unsigned)lane * 16;
  i32x4 fbl[NBUF][TN][2];
  auto load_b1 = [&](int k, auto buf, auto nc) {
    constexpr int KB = decltype(buf)::value;
    constexpr int n = decltype(nc)::value;
    const unsigned soff = b_tile[n] + (unsigned)k * 2048u;
    // named outside the asm statements so that the generic lambda captures them
    i32x4 &lo = fbl[KB][n][0], &hi = fbl[KB][n][1];
    const unsigned voff = b_lane;
    const i32x4 rsrc = b_rsrc;
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(lo) : "v"(voff), "s"(rsrc), "s"(soff));
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:1024"
                 : "=v"(hi)
                 : "v"(voff), "s"(rsrc), "s"(soff));
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
  i32x8 fa[RA];
  auto read_a = [&](auto kslot, auto tt) {
    constexpr int KS = decltype(kslot)::value;
    constexpr int T = decltype(tt)::value;
    constexpr int OFF = KS * SLOT + T * 16 * kRowBytes;
    const i32x4 lo = *(lvec_t)(size_t)(rd_addr[0] + (unsigned)OFF);
    const i32x4 hi = *(lvec_t)(size_t)(rd_addr[1] + (unsigned)OFF);
    fa[T % RA] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[m][n]));
    }

  // ---- prologue: B(0), B(1), then A(0..3) ----------------------------------------------------------
  static_for<0, NBUF>([&](auto bc) {
    constexpr int J = decltype(bc)::value;
    if (J < nk) {
      static_for<0, TN>([&](auto nc) { load_b1(J, bc, nc); });
    }
  });
#pragma unroll
  for (int k = 0; k < NSLOT; ++k) {
    if (k < nk) {
#pragma unroll
      for (int j = 0; j < LH; ++j) issue_a1(k, k, j);
    }
  }
  // A(0) and everything older (B(0), B(1)) has landed when only A(1..3) may be in flight
  if (nk >= NSLOT) __builtin_amdgcn_s_waitcnt(waitcnt_imm((NSLOT - 1) * LH, 15));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  using K0 = std::integral_constant<int, 0>;
  static_for<0, RA - 1>([&](auto tc) { read_a(K0{}, tc); });
  __builtin_amdgcn_sched_barrier(0);

  // ---- K loop: trip k multiplies K-step k.  KM = k mod 4 fixes the A slot and the B buffer at
  // compile time.  VMW = loads that may still be in flight at the barrier, VMB = loads behind
  // the batch of B(k) that may still be in flight at the trip's first MFMAs; NA, NB, NX: the
  // trip requests A(k+4), requests B(k+2), has a trip behind it.  VMW < 0: none of this is known
  // at compile time; every wait is for all loads and the requests are decided at run time. ---------
  auto trip = [&](int k, auto kmod, auto vmw_c, auto vmb_c, auto na_c, auto nb_c, auto nx_c) {
    constexpr int KM = decltype(kmod)::value;
    constexpr int VMW = decltype(vmw_c)::value;
    constexpr int VMB = decltype(vmb_c)::value;
    constexpr bool KNOWN = VMW >= 0;
    constexpr int KB = KM % NBUF;
    using KS = std::integral_constant<int, KM>;
    using KN = std::integral_constant<int, (KM + 1) % NSLOT>;
    using KBc = std::integral_constant<int, KB>;
    const bool has_next = KNOWN ? decltype(nx_c)::value : k + 1 < nk;
    const bool do_a = KNOWN ? decltype(na_c)::value : k + NSLOT < nk;
    const bool do_b = KNOWN ? decltype(nb_c)::value : k + NBUF < nk;
    static_for<0, MS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
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
        if constexpr (T == 0) {
          // B(k) tile n: younger than its second load are the rest of its batch and VMB more
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(KNOWN ? 2 * (TN - 1 - n) + VMB : 0, 15));
          // the registers hold the loaded bytes from here on, not before
          i32x4 &l0 = fbl[KB][n][0], &h0 = fbl[KB][n][1];
          asm volatile("" : "+v"(l0), "+v"(h0));
        }
        const i32x4 lo = fbl[KB][n][0], hi = fbl[KB][n][1];
        const i32x8 fb = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        // cbsz = blgp = 0: both operands OCP e4m3; accumulated in place in the AGPRs
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0"
                     : "+a"(acc[T][n])
                     : "v"(fb), "v"(fa[T % RA]));
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
        // last m-step: tile n of this buffer is done with MFMA (m = 7, n)
        if constexpr (T == MS - 1) {
          if (do_b) load_b1(k + NBUF, KBc{}, nc);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  // Loads of a full trip in issue order: behind the barrier the 4 A transfers (m-steps 5, 6),
  // then the 8 B loads (m-step 7).
  //   B(k), requested at the end of trip k - 2: behind its batch come the loads of trip k - 1.
  //   A(k+1) at the barrier of trip k, requested in trip k - 3: behind it the 8 B loads of that
  //   trip and the loads of trips k - 2 and k - 1.  Trips 0..2: A(k+1) was requested in the
  //   prologue, followed there by A(k+2..3) and here by 12 loads per earlier trip.
  // The last four trips (K-steps nk - 4 .. nk - 1 = trips t0 .. t3) request no A and only t0, t1
  // request B (8 loads each), so B(t1), B(t2) have 8 loads behind their batch and B(t3) none,
  // and the barriers of t1, t2 have 8 + 12 + 8 and 8 + 8 + 8 behind A(k+1).
  constexpr int VM_STEADY = 2 * TN + 2 * TRIP_LOADS;
  using T_ = std::true_type;
  using F_ = std::false_type;
  auto group = [&](int k0, auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int VM = (FIRST && I <= NSLOT - 2) ? (NSLOT - 2 - I) * LH + TRIP_LOADS * I : VM_STEADY;
      trip(k0 + I, ic, std::integral_constant<int, VM>{}, std::integral_constant<int, TRIP_LOADS>{},
           T_{}, T_{}, T_{});
    });
  };
  auto last_group = [&](int k0) {
    static_for<0, NSLOT>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int VM = I == 0 ? VM_STEADY : I == 1 ? 2 * TN + TRIP_LOADS + 2 * TN : 3 * 2 * TN;
      constexpr int VB = I == 0 ? TRIP_LOADS : I == 3 ? 0 : 2 * TN;
      trip(k0 + I, ic, std::integral_constant<int, VM>{}, std::integral_constant<int, VB>{}, F_{},
           std::integral_constant<bool, (I < 2)>{}, std::integral_constant<bool, (I < 3)>{});
    });
  };
  using NEG = std::integral_constant<int, -1>;
  int k = 0;
  // a steady group of four trips requests A up to K-step k + 7 and B up to K-step k + 5
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
      if (I == 0 || k + I < nk) trip(k + I, ic, NEG{}, NEG{}, F_{}, F_{}, F_{});
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  stream_epilogue<OUT, BM, BN, WM, WN>(p, acc, lds, wave, row0, col0);
}

template <int DT, int OUT>
__global__ __launch_bounds__(256, 2) void gemm_stream8db_kernel(const GemmArgs p) {
  gemm_stream8db_body<DT, OUT>(p, blockIdx.x);
}

}  // namespace
}  // namespace astergemm
