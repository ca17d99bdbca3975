// Deep-pipelined MFMA tile kernel for gfx950: C[M,N] = epi(A[M,K] * B[N,K]^T).
//
// Measured on MI355X, a global->LDS transfer that hits in L2 takes about 0.9 us
// from issue to data-in-LDS, the same time the matrix cores need for a 256x256
// tile step of 128 bytes of K.  A two-stage ring (load step k+1 while computing
// step k) therefore stalls on every step.  This kernel cuts the K loop into
// 64-byte sub-steps (32 bf16/f16, 64 fp8, 128 fp4 elements of a row), keeps a
// ring of four 32 KiB LDS stages and issues the transfer for sub-step i+4 while
// computing sub-step i, so three sub-steps of matrix work cover the latency.
// MFMA operand fragments are double-buffered in registers: the ds_reads of
// sub-step i+1 are issued before the MFMAs of sub-step i.
//
// Per sub-step one MFMA K-step per tile pair in every encoding:
//   bf16/f16  v_mfma_f32_16x16x32       lane (r=lane%16, q=lane/16) <- granule q
//   fp8       v_mfma_f32_32x32x64_f8f6f4 lane (r=lane%32, q=lane/32) <- granules 2q, 2q+1
//   fp4       v_mfma_scale_f32_16x16x128_f8f6f4 (cbsz=blgp=4)        <- granule q
// LDS stage layout: rows of 64 bytes, 16-byte granule index XOR f(row) with
// f(row) = (-(row >> 2)) & 3.  The reference's direct-to-LDS kernels use
// Swizzle(2, 4, 4), i.e. f(row) = (row >> 2) & 3
// (contrib/kittens/test/test_102_gemm_python_multitile_g2s_lds_cdna4.py:142), which
// is conflict-free for their ds_read_b64; a ds_read_b128 is served 16 lanes at a
// time in the lane groups {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31}
// (and the same +32), and under that grouping (row >> 2) & 3 is a two-way bank
// conflict (measured: SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE) while
// (-(row >> 2)) & 3 is conflict-free.  The swizzle is applied through the global
// source address because the LDS side of global_load_lds is linear
// (python/aster/dialects/kernel_builder_with_layouts.py:401-416).
// The stage-per-op-class picture of the reference's pipeline strategies
// (contrib/kittens/test/kittens_helpers.py:137-157) maps onto this as
// A_LOAD = B_LOAD = 0, LDS_READ = 3, COMPUTE = 4.
#pragma once
#include <type_traits>

#include "gemm_tile_kernel.hpp"

namespace astergemm {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kSubBytes = 64;  // bytes of one operand row per sub-step
constexpr int kStages = 4;

template <int DT>
struct PipeEnc {
  static constexpr bool k32 = (DT == ASTERGEMM_FP8_E4M3);  // 32x32 tiles
  static constexpr int kTile = k32 ? 32 : 16;              // rows per MFMA tile
  static constexpr int kGran = k32 ? 2 : 1;                // 16-byte granules per fragment
  static constexpr int kAccRegs = k32 ? 16 : 4;
};

template <int DT>
struct AccT {
  using type = f32x4;
};
template <>
struct AccT<ASTERGEMM_FP8_E4M3> {
  using type = f32x16;
};

template <int DT>
__device__ __forceinline__ typename AccT<DT>::type pipe_mfma(const i32x4* a, const i32x4* b,
                                                              typename AccT<DT>::type c, int sa,
                                                              int sb) {
  if constexpr (DT == ASTERGEMM_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  } else if constexpr (DT == ASTERGEMM_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  } else if constexpr (DT == ASTERGEMM_FP8_E4M3) {
    i32x8 av = {a[0].x, a[0].y, a[0].z, a[0].w, a[1].x, a[1].y, a[1].z, a[1].w};
    i32x8 bv = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 0, 0, 0, 0, 0, 0);
  } else {
    i32x8 av = {a[0].x, a[0].y, a[0].z, a[0].w, 0, 0, 0, 0};
    i32x8 bv = {b[0].x, b[0].y, b[0].z, b[0].w, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 4, 4, 0, sa, 0, sb);
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void gemm_pipe_body(const GemmArgs& p) {
  using Acc = typename AccT<DT>::type;
  constexpr int NW = WM * WN;
  constexpr int TR = PipeEnc<DT>::kTile;
  constexpr int TM = BM / WM / TR;  // MFMA tiles per wave along M
  constexpr int TN = BN / WN / TR;
  constexpr int KG = PipeEnc<DT>::kGran;
  constexpr int STAGE_A = BM * kSubBytes;
  constexpr int STAGE = (BM + BN) * kSubBytes;
  constexpr int LA = BM / 16 / NW;  // 1 KiB (16-row) transfers per wave and stage
  constexpr int LB = BN / 16 / NW;
  constexpr int LOADS = LA + LB;    // global->LDS instructions per wave and stage
  static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile rows per wave");
  static_assert(DT != ASTERGEMM_MXFP4, "fp4 scales are not staged by this kernel yet");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  int tile_m, tile_n;
  map_tile(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;

  // ---- global -> LDS: transfer j of this wave fills rows [(j*NW + wave)*16, +16);
  // lane i writes (row i/4, slot i%4) and fetches granule slot ^ ((-(row >> 2)) & 3).
  const uint8_t* a_base = p.A + (int64_t)row0 * p.lda_bytes;
  const uint8_t* b_base = p.B + (int64_t)col0 * p.ldb_bytes;
  const int g_lane = (lane & 3) ^ ((-(lane >> 4)) & 3);
  unsigned a_off[LA], b_off[LB];
#pragma unroll
  for (int j = 0; j < LA; ++j) {
    const int r = (j * NW + wave) * 16 + (lane >> 2);
    const int rr = (row0 + r < p.M) ? r : (p.M - 1 - row0);
    a_off[j] = (unsigned)(rr * (int)p.lda_bytes + g_lane * 16);
  }
#pragma unroll
  for (int j = 0; j < LB; ++j) {
    const int r = (j * NW + wave) * 16 + (lane >> 2);
    const int rr = (col0 + r < p.N) ? r : (p.N - 1 - col0);
    b_off[j] = (unsigned)(rr * (int)p.ldb_bytes + g_lane * 16);
  }
  const int nsub = p.ksteps;  // sub-steps of 64 bytes
  const bool live_tail = g_lane < p.tail_granules;

  // One 1 KiB transfer: 64 lanes x 16 bytes from (uniform base + per-lane offset)
  // to LDS at M0 + lane * 16.  Written as asm so the address stays in the
  // scalar-base + 32-bit-offset form; completion is tracked with vmcnt by hand.
  auto g2s = [&](const uint8_t* base, unsigned voff, uint8_t* dst) {
    const unsigned m0v = (unsigned)(size_t)AG_LDS(dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(base)
                 : "memory", "m0");
  };
  auto issue = [&](int s, int buf) {
    const uint8_t* ga = a_base + (int64_t)s * kSubBytes;
    const uint8_t* gb = b_base + (int64_t)s * kSubBytes;
    uint8_t* la = lds + buf * STAGE + wave * 16 * kSubBytes;
    uint8_t* lb = la + STAGE_A;
#pragma unroll
    for (int j = 0; j < LA; ++j) g2s(ga, a_off[j], la + j * NW * 16 * kSubBytes);
#pragma unroll
    for (int j = 0; j < LB; ++j) g2s(gb, b_off[j], lb + j * NW * 16 * kSubBytes);
  };
  // Last sub-step of a row that does not fill 64 bytes: granules past the end of
  // the row come from a block of zeros.
  auto issue_tail = [&](int s, int buf) {
    const uint8_t* ga = a_base + (int64_t)s * kSubBytes;
    const uint8_t* gb = b_base + (int64_t)s * kSubBytes;
    uint8_t* la = lds + buf * STAGE + wave * 16 * kSubBytes;
    uint8_t* lb = la + STAGE_A;
#pragma unroll
    for (int j = 0; j < LA; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(live_tail ? ga + a_off[j] : g_zero16),
                                       AG_LDS(la + j * NW * 16 * kSubBytes), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < LB; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(live_tail ? gb + b_off[j] : g_zero16),
                                       AG_LDS(lb + j * NW * 16 * kSubBytes), 16, 0, 0);
  };
  auto issue_any = [&](int s, int buf) {
    if (p.tail_granules != 0 && s == nsub - 1) issue_tail(s, buf);
    else issue(s, buf);
  };

  // ---- LDS -> fragments ---------------------------------------------------------
  const int lr = lane % TR, lq = lane / TR;
  unsigned rd_off[KG];
#pragma unroll
  for (int h = 0; h < KG; ++h) {
    const int g = (KG == 2) ? (2 * lq + h) : lq;
    rd_off[h] = (unsigned)(lr * kSubBytes + ((g ^ ((-(lr >> 2)) & 3)) << 4));
  }
  const unsigned a_rd = (unsigned)(wm * TM * TR * kSubBytes);
  const unsigned b_rd = (unsigned)(STAGE_A + wn * TN * TR * kSubBytes);

  i32x4 fa[2][TM][KG], fb[2][TN][KG];
  auto read_frags = [&](int buf, auto parity) {
    constexpr int P = decltype(parity)::value;
    const uint8_t* st = lds + buf * STAGE;
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
      for (int h = 0; h < KG; ++h)
        fa[P][m][h] = *(const i32x4*)(st + a_rd + m * TR * kSubBytes + rd_off[h]);
#pragma unroll
    for (int n = 0; n < TN; ++n)
#pragma unroll
      for (int h = 0; h < KG; ++h)
        fb[P][n][h] = *(const i32x4*)(st + b_rd + n * TR * kSubBytes + rd_off[h]);
  };

  Acc acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n)
#pragma unroll
      for (int e = 0; e < PipeEnc<DT>::kAccRegs; ++e) acc[m][n][e] = 0.f;

  // ---- prologue: stages 0..3 in flight, fragments of sub-step 0 in registers ----
#pragma unroll
  for (int s = 0; s < kStages; ++s)
    if (s < nsub) issue_any(s, s);
  if (nsub > 3) __builtin_amdgcn_s_waitcnt(waitcnt_imm(3 * LOADS, 15));
  else if (nsub > 2) __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LOADS, 15));
  else if (nsub > 1) __builtin_amdgcn_s_waitcnt(waitcnt_imm(1 * LOADS, 15));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_frags(0, std::integral_constant<int, 0>{});

  // One sub-step; U = i % 4 is the ring slot of stage i, known at compile time.
  // STEADY: at least four more sub-steps follow, so nothing is conditional.
  auto step = [&](int i, auto uu, auto steady) {
    constexpr int U = decltype(uu)::value;
    constexpr bool STEADY = decltype(steady)::value;
    // stage i+1 landed (this wave's part); fragments of sub-step i arrived, so
    // ring slot U may be overwritten once everybody is past the barrier.
    if (STEADY || i + 3 < nsub) __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LOADS, 0));
    else if (i + 2 < nsub) __builtin_amdgcn_s_waitcnt(waitcnt_imm(1 * LOADS, 0));
    else __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (STEADY) issue(i + kStages, U);
    else if (i + kStages < nsub) issue_any(i + kStages, U);
    if (STEADY || i + 1 < nsub)
      read_frags((U + 1) % kStages, std::integral_constant<int, (U + 1) & 1>{});
    // Keep the order "reads of sub-step i+1, then MFMAs of sub-step i": the
    // scheduler would otherwise sink each read next to its first use and wait.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
      for (int n = 0; n < TN; ++n)
        acc[m][n] = pipe_mfma<DT>(fb[U & 1][n], fa[U & 1][m], acc[m][n], 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  using T = std::true_type;
  using F = std::false_type;
  int i = 0;
  for (; i + 2 * kStages < nsub; i += kStages) {
    step(i, std::integral_constant<int, 0>{}, T{});
    step(i + 1, std::integral_constant<int, 1>{}, T{});
    step(i + 2, std::integral_constant<int, 2>{}, T{});
    step(i + 3, std::integral_constant<int, 3>{}, T{});
  }
  for (; i < nsub; i += kStages) {
    step(i, std::integral_constant<int, 0>{}, F{});
    if (i + 1 < nsub) step(i + 1, std::integral_constant<int, 1>{}, F{});
    if (i + 2 < nsub) step(i + 2, std::integral_constant<int, 2>{}, F{});
    if (i + 3 < nsub) step(i + 3, std::integral_constant<int, 3>{}, F{});
  }

  // ---- epilogue -------------------------------------------------------------------
  // srcA = B rows, srcB = A rows: lane owns C[m = lane % TR][4 consecutive n].
  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  const bool vec_ok = (p.ldc & 3) == 0;
#pragma unroll
  for (int m = 0; m < TM; ++m) {
    const int row = row0 + (wm * TM + m) * TR + lr;
#pragma unroll
    for (int n = 0; n < TN; ++n) {
#pragma unroll
      for (int v4 = 0; v4 < PipeEnc<DT>::kAccRegs / 4; ++v4) {
        // 16x16: n = 4*lq + e.  32x32: n = 8*v4 + 4*lq + e.
        const int col = col0 + (wn * TN + n) * TR + (TR == 32 ? 8 * v4 : 0) + 4 * lq;
        if (row < p.M && col < p.N) {
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[m][n][v4 * 4 + e] * scale;
          const int ncols = (p.N - col) < 4 ? (p.N - col) : 4;
          if (p.bias) {
            for (int r = 0; r < ncols; ++r) v[r] += p.bias[col + r];
          }
          store4<OUT>(p.C, (int64_t)row * p.ldc + col, v, vec_ok, ncols);
        }
      }
    }
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_pipe_kernel(const GemmArgs p) {
  gemm_pipe_body<DT, OUT, BM, BN, WM, WN>(p);
}

}  // namespace
}  // namespace astergemm
