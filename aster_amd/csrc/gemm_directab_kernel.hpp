// GEMM with BOTH operands straight from global memory into MFMA operand registers ("direct
// AB"), 16-bit operands, no LDS at all: the operand path of the reference's
// `gemm_f16_direct_ab` template (contrib/kittens/test/gemm_16x32_f16_k_loop_helpers_direct_ab.mlir:
// 1-128, selected by `operand_path = direct_ab`, contrib/kittens/gemm_config.py:213-276;
// the caller pre-shuffles A as well as B, test_perf_001_gemm_fp16_weak_scaled.py:252-254).
//
// Operand layout: A [M, K] and B [N, K] both in the reference's `shuffle_weight` order
// (astergemm_shuffle_weight_16): chunks of 1 KiB, chunk (rb, kb) holds rows 16 rb .. 16 rb + 15
// and K elements 32 kb .. 32 kb + 31; lane L = 16 g + r of a wave finds at byte 16 L of the
// chunk the K elements {4g .. 4g+3} and {16+4g .. 16+4g+3} of row 16 rb + r.  That is the
// pairing of two 16x16x16 MFMAs in the reference; here the eight values go into ONE
// v_mfma_f32_16x16x32, which multiplies lane group g of one operand with lane group g of the
// other: since A and B carry the same K permutation, the sum over K is the same sum.
//
// Geometry: a wave owns TM x TN tiles of 16 x 16 (128 x 64 by default), a workgroup WM x WN
// waves.  Per chunk column a wave issues TM + TN loads of 1 KiB for TM * TN MFMAs; the waves
// of a workgroup that share rows of an operand fetch the same lines, which the vector L1
// serves.  NB - 1 chunk columns are in flight in a ring of NB register buffers, refilled one load
// behind every second MFMA; every load is an ordinary
// buffer load, so the compiler's own vmcnt bookkeeping is exact.  Rows past M or N are clamped
// to the last 16-row block (buffer loads check voffset against the resource, not the scalar
// offset) and not stored.  There is no barrier: one per chunk column, to keep the waves that
// share lines together in the L1, was measured slower (bf16 8192^3: 828 against 776 us).
#pragma once
#include "gemm_stream_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT, int TM, int TN, int WM, int WN, int NB>
__global__ __launch_bounds__(WM* WN * 64) void gemm_directab_kernel(const GemmArgs p) {
  constexpr int BM = TM * 16 * WM, BN = TN * 16 * WN;
  // accumulators in the accumulation half of the register file, destination tied to the addend
  // (left to itself the compiler moves them through architectural registers around every MFMA)
  constexpr bool AX = true;
  static_assert(DT == ASTERGEMM_BF16 || DT == ASTERGEMM_F16, "16-bit operands");
  static_assert(NB >= 2 && NB <= 4, "ring of register buffers");

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM + wm * TM * 16, col0 = tile_n * BN + wn * TN * 16;
  const int nk = p.K >> 5;  // chunk columns

  const unsigned chunk_row = (unsigned)nk * 1024u;  // bytes of 16 rows of an operand
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.A, 0, (int)((unsigned)(p.M >> 4) * chunk_row), 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.B, 0, (int)((unsigned)(p.N >> 4) * chunk_row), 0x00020000);
  unsigned a_tile[TM], b_tile[TN];
#pragma unroll
  for (int m = 0; m < TM; ++m) {
    int rb = (row0 >> 4) + m;
    const int last = (p.M >> 4) - 1;
    rb = rb < last ? rb : last;
    a_tile[m] = __builtin_amdgcn_readfirstlane((unsigned)rb * chunk_row);
  }
#pragma unroll
  for (int n = 0; n < TN; ++n) {
    int nb = (col0 >> 4) + n;
    const int last = (p.N >> 4) - 1;
    nb = nb < last ? nb : last;
    b_tile[n] = __builtin_amdgcn_readfirstlane((unsigned)nb * chunk_row);
  }
  const int v_lane = lane * 16;

  i32x4 fa[NB][TM], fb[NB][TN];
  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  // One 1 KiB load of chunk column kb (clamped: the last trips of the loop request columns past
  // the end, whose data is never multiplied) into buffer BI, in the order the MFMAs need them:
  // B tile 0, the TM tiles of A, the other B tiles.
  auto load_one = [&](int kb, auto buf, auto idx) {
    constexpr int BI = decltype(buf)::value;
    constexpr int J = decltype(idx)::value;
    const unsigned kk = (unsigned)(kb < nk ? kb : nk - 1) * 1024u;
    if constexpr (J == 0 || J > TM) {
      constexpr int n = J == 0 ? 0 : J - TM;
      fb[BI][n] = __builtin_bit_cast(
          i32x4, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(b_rsrc, v_lane, (int)(b_tile[n] + kk), 0));
    } else {
      constexpr int m = J - 1;
      fa[BI][m] = __builtin_bit_cast(
          i32x4, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(a_rsrc, v_lane, (int)(a_tile[m] + kk), 0));
    }
  };
  constexpr int NL = TM + TN;   // loads per chunk column
  constexpr int NMF = TM * TN;  // MFMAs per chunk column
  static_assert(2 * NL <= NMF, "one load behind every second MFMA");

  // prologue: columns 0 .. NB-2 in flight
  static_for<0, NB - 1>([&](auto ic) {
    static_for<0, NL>([&](auto jc) { load_one(decltype(ic)::value, ic, jc); });
  });
  // Trip (kb, i) multiplies buffer i (column kb + i) and, behind every second MFMA, requests one
  // load of column kb + i + NB - 1 into the buffer the previous trip has finished with.
  // srcA = B-row fragment, held for TM instructions in a row; lane owns C[m = lane % 16][4
  // consecutive n].
  auto trip = [&](int kb, auto buf, bool refill) {
    constexpr int BI = decltype(buf)::value;
    using Next = std::integral_constant<int, (BI + NB - 1) % NB>;
    static_for<0, NMF>([&](auto ic) {
      constexpr int I = decltype(ic)::value;
      constexpr int n = I / TM, m = I % TM;
      stream_mma<DT, AX>(fb[BI][n], fa[BI][m], acc[m][n]);
      if constexpr (I % 2 == 0 && I / 2 < NL) {
        if (refill) load_one(kb + BI + NB - 1, Next{}, std::integral_constant<int, I / 2>{});
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  int kb = 0;
  for (; kb + NB <= nk; kb += NB) static_for<0, NB>([&](auto ic) { trip(kb, ic, true); });
  // the ring is in phase 0 again: the remaining nk % NB columns sit in buffers 0 ..
  static_for<0, NB - 1>([&](auto ic) {
    if (kb + decltype(ic)::value < nk) trip(kb, ic, false);
  });

  // ---- epilogue: straight from the accumulators, 4 consecutive columns per lane ---------------
  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  const int li = lane & 15, lq = lane >> 4;
  constexpr int OB = (OUT == ASTERGEMM_F32) ? 4 : 2;
#pragma unroll
  for (int n = 0; n < TN; ++n) {
    const int col = col0 + n * 16 + 4 * lq;
    if (col >= p.N) continue;  // N is a multiple of 16: the four columns are inside or outside
    float bias_v[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
      for (int e = 0; e < 4; ++e) bias_v[e] = p.bias[col + e];
    }
#pragma unroll
    for (int m = 0; m < TM; ++m) {
      const int row = row0 + m * 16 + li;
      if (row >= p.M) continue;
      f32x4 v = acc[m][n] * scale;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += bias_v[e];
      uint8_t* out = (uint8_t*)p.C + ((int64_t)row * p.ldc + col) * OB;
      if constexpr (OUT == ASTERGEMM_F32) {
        __builtin_nontemporal_store(v, (f32x4*)out);
      } else {
        const u16x4 h = cast4_16<OUT>(v);
        __builtin_nontemporal_store(h, (u16x4*)out);
      }
    }
  }
}

}  // namespace
}  // namespace astergemm
