// LDS-staged MFMA tile kernels for gfx950 (CDNA4): C[M,N] = epi(A[M,K] * B[N,K]^T).
//
// One kernel body serves four operand encodings because they share one byte
// geometry: a K-step is 128 bytes of an operand row (64 bf16/f16, 128 fp8,
// 256 fp4), which the matrix core consumes in 32 cycles per 16x16 tile pair in
// every encoding (2 x 16x16x32 for 16-bit, 1 x 16x16x128 for fp8, 2 x 16x16x128
// for fp4).
//
// What the reference does for the same job, as generated AMDGCN:
//   * global -> LDS with `buffer_load_dwordx4 ... lds`, XOR-swizzled through the
//     global source address because the LDS side of that instruction is linear
//     (python/aster/dialects/kernel_builder_with_layouts.py:371-481,
//      contrib/kittens/test/test_102_gemm_python_multitile_g2s_lds_cdna4.py:142);
//   * LDS -> VGPR MFMA fragments (contrib/kittens/library/lds_mfma_16x64_b.mlir);
//   * v_mfma_f32_16x16x32_f16 inner loop over (k, m, n) tiles with AGPR
//     accumulators (test_102_..._g2s_directb_cdna4.py:296-306);
//   * row-major workgroup -> (m, n) tile mapping (same file :201-203).
// Here: 128-byte LDS rows, 16-byte granule index XOR ((row >> 1) & 7) so that a
// ds_read_b128 of 16 rows x one granule touches 16 distinct 16-byte bank groups;
// fragments are read with ds_read_b128; accumulators are computed transposed
// (srcA = B rows, srcB = A rows) so each lane owns 4 consecutive columns of one
// C row and the epilogue stores 8/16-byte vectors.
#pragma once
#include "astergemm_internal.h"

namespace astergemm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

#define AG_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define AG_GLOBAL(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int kRowBytes = 128;  // bytes of one operand row per K-step

// Source of the 16-byte transfers that lie past the end of a row.
__device__ __attribute__((aligned(16))) const uint8_t g_zero16[16] = {0};

// s_waitcnt immediate for gfx9: vmcnt[3:0]|[15:14], expcnt[6:4], lgkmcnt[11:8].
constexpr int waitcnt_imm(int vm, int lgkm) {
  return (vm & 0xF) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 0xF) << 8);
}

__device__ __forceinline__ float bf16_bits_to_f32(unsigned short b) {
  return __builtin_bit_cast(float, (unsigned)b << 16);
}

// fp32 -> bf16 round-to-nearest-even, NaN kept quiet.
// Four fp32 values to four 16-bit outputs, round to nearest even, with the hardware
// converters (v_cvt_pk_bf16_f32 / v_cvt_f16_f32): the integer bf16 rounding sequence is six
// VALU operations per element, which made the epilogue of a 256x256 tile VALU bound.
template <int OUT>
__device__ __forceinline__ u16x4 cast4_16(f32x4 v) {
  if constexpr (OUT == ASTERGEMM_BF16) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(u16x4, __builtin_convertvector(v, bf16x4_t));
  } else {
    typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(u16x4, __builtin_convertvector(v, f16x4_t));
  }
}

// Hardware hands workgroup b to XCD b % 8.  Give each XCD one contiguous run of
// the logical tile order, then walk that order in groups of `group_m` tile rows
// (column-major inside a group) so the 32 workgroups resident on an XCD share
// A and B panels through that XCD's L2.
__device__ __forceinline__ void map_tile(int bid, int tiles_m, int tiles_n,
                                         int group_m, int& tm, int& tn) {
  if (group_m < 0) {
    // band order (tiles_m % 8 == 0, tiles_n % 8 == 0): all eight XCDs work on the same band of
    // eight tile rows, XCD x on its own tiles_n / 8 tile columns of it, so that a band of A is
    // fetched from HBM once and reaches the other seven XCDs from the last-level cache
    const int xcd = bid & 7, idx = bid >> 3;
    const int cols = tiles_n >> 3;               // tile columns of an XCD
    const int per_band = 8 * cols;               // tiles of an XCD in one band
    const int band = idx / per_band, j = idx - band * per_band;
    tm = band * 8 + (j & 7);
    tn = xcd * cols + (j >> 3);
    return;
  }
  const int total = tiles_m * tiles_n;
  const int q = total >> 3, rem = total & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  const int logical = xcd * q + (xcd < rem ? xcd : rem) + idx;
  const int gsz = group_m * tiles_n;
  const int g = logical / gsz;
  const int first_m = g * group_m;
  const int rows = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int r = logical - g * gsz;
  tm = first_m + r % rows;
  tn = r / rows;
}

template <int DT>
struct Enc {
  // MFMA k-substeps per 128-byte row chunk and 16-byte granules per fragment.
  static constexpr int kSub = (DT == ASTERGEMM_FP8_E4M3) ? 1 : 2;
  static constexpr int kGran = (DT == ASTERGEMM_FP8_E4M3) ? 2 : 1;
  static constexpr int kElemsPerStep =
      (DT == ASTERGEMM_FP8_E4M3) ? 128 : (DT == ASTERGEMM_MXFP4 ? 256 : 64);
};

// One MFMA: acc += srcA(16 x k) * srcB(k x 16), operands as raw dwords.
template <int DT>
__device__ __forceinline__ f32x4 mfma_step(const i32x4* a, const i32x4* b, f32x4 c,
                                           int sa, int sb) {
  if constexpr (DT == ASTERGEMM_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  } else if constexpr (DT == ASTERGEMM_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  } else if constexpr (DT == ASTERGEMM_FP8_E4M3) {
    i32x8 av = {a[0].x, a[0].y, a[0].z, a[0].w, a[1].x, a[1].y, a[1].z, a[1].w};
    i32x8 bv = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
    // cbsz = blgp = 0: both operands OCP e4m3; zero scale operands select the
    // unscaled form of the instruction.
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 0, 0, 0, 0, 0, 0);
  } else {
    i32x8 av = {a[0].x, a[0].y, a[0].z, a[0].w, 0, 0, 0, 0};
    i32x8 bv = {b[0].x, b[0].y, b[0].z, b[0].w, 0, 0, 0, 0};
    // cbsz = blgp = 4: both operands e2m1; byte 0 of sa / sb is the e8m0 scale
    // of this lane's 32 K-elements.
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 4, 4, 0, sa, 0, sb);
  }
}

template <int OUT>
__device__ __forceinline__ void store4(void* C, int64_t idx, f32x4 v, bool vec_ok,
                                       int ncols) {
  if constexpr (OUT == ASTERGEMM_F32) {
    float* p = (float*)C + idx;
    if (vec_ok && ncols == 4) {
      *(f32x4*)p = v;
    } else {
      for (int r = 0; r < ncols; ++r) p[r] = v[r];
    }
  } else {
    const u16x4 hv4 = cast4_16<OUT>(v);
    const unsigned short h[4] = {hv4.x, hv4.y, hv4.z, hv4.w};
    unsigned short* p = (unsigned short*)C + idx;
    if (vec_ok && ncols == 4) {
      u16x4 hv = {h[0], h[1], h[2], h[3]};
      *(u16x4*)p = hv;
    } else {
      for (int r = 0; r < ncols; ++r) p[r] = h[r];
    }
  }
}

template <int DT, int OUT, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void gemm_tile_body(const GemmArgs& p) {
  constexpr int NW = WM * WN;
  constexpr int TM = BM / WM / 16;  // 16-row MFMA tiles per wave along M
  constexpr int TN = BN / WN / 16;
  constexpr int STAGE_A = BM * kRowBytes;
  constexpr int STAGE = (BM + BN) * kRowBytes;
  constexpr int LA = BM / 8 / NW;  // 1 KiB (8-row) global->LDS transfers per wave
  constexpr int LB = BN / 8 / NW;
  constexpr int KSUB = Enc<DT>::kSub;
  constexpr int KGRAN = Enc<DT>::kGran;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows per wave");
  static_assert((8 * NW) % 16 == 0, "swizzle phase must not depend on the transfer index");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  int tile_m, tile_n;
  map_tile(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
  const int row0 = tile_m * BM, col0 = tile_n * BN;

  // ---- global -> LDS addressing -------------------------------------------
  // Transfer j of this wave fills tile rows [j*8*NW + wave*8, +8): lane i writes
  // LDS slot (row = i/8, granule slot = i%8) and therefore fetches the global
  // granule (slot ^ ((row >> 1) & 7)) of that row.  Rows past M / N are clamped
  // to the last valid row; their products are never stored.
  const uint8_t* a_base = p.A + (int64_t)row0 * p.lda_bytes;
  const uint8_t* b_base = p.B + (int64_t)col0 * p.ldb_bytes;
  unsigned a_off[LA], b_off[LB];
  int g_lane;  // K granule (0..7) of a row that this lane moves; same for every transfer
  {
    const int lrow = lane >> 3, slot = lane & 7;
    g_lane = slot ^ (((wave * 8 + lrow) >> 1) & 7);
#pragma unroll
    for (int j = 0; j < LA; ++j) {
      const int r = j * 8 * NW + wave * 8 + lrow;
      const int g = slot ^ ((r >> 1) & 7);
      const int rr = (row0 + r < p.M) ? r : (p.M - 1 - row0);
      a_off[j] = (unsigned)(rr * (int)p.lda_bytes + g * 16);
    }
#pragma unroll
    for (int j = 0; j < LB; ++j) {
      const int r = j * 8 * NW + wave * 8 + lrow;
      const int g = slot ^ ((r >> 1) & 7);
      const int rr = (col0 + r < p.N) ? r : (p.N - 1 - col0);
      b_off[j] = (unsigned)(rr * (int)p.ldb_bytes + g * 16);
    }
  }

  auto issue_loads = [&](int kt, int stage) {
    const uint8_t* ga = a_base + (int64_t)kt * kRowBytes;
    const uint8_t* gb = b_base + (int64_t)kt * kRowBytes;
    uint8_t* la = lds + stage * STAGE + wave * 8 * kRowBytes;
    uint8_t* lb = la + STAGE_A;
#pragma unroll
    for (int j = 0; j < LA; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(ga + a_off[j]),
                                       AG_LDS(la + j * 8 * NW * kRowBytes), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < LB; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(gb + b_off[j]),
                                       AG_LDS(lb + j * 8 * NW * kRowBytes), 16, 0, 0);
  };
  // Last K-step of a row that does not fill 128 bytes: granules past the end of
  // the row are fetched from a block of zeros instead, so they add nothing.
  auto issue_tail_loads = [&](int kt, int stage) {
    const uint8_t* ga = a_base + (int64_t)kt * kRowBytes;
    const uint8_t* gb = b_base + (int64_t)kt * kRowBytes;
    uint8_t* la = lds + stage * STAGE + wave * 8 * kRowBytes;
    uint8_t* lb = la + STAGE_A;
    const bool live = g_lane < p.tail_granules;
#pragma unroll
    for (int j = 0; j < LA; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(live ? ga + a_off[j] : g_zero16),
                                       AG_LDS(la + j * 8 * NW * kRowBytes), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < LB; ++j)
      __builtin_amdgcn_global_load_lds(AG_GLOBAL(live ? gb + b_off[j] : g_zero16),
                                       AG_LDS(lb + j * 8 * NW * kRowBytes), 16, 0, 0);
  };
  auto stage_step = [&](int kt, int stage) {
    if (p.tail_granules != 0 && kt == p.ksteps - 1) issue_tail_loads(kt, stage);
    else issue_loads(kt, stage);
  };

  // ---- LDS -> fragment addressing ------------------------------------------
  // Lane (li = lane%16, lq = lane/16) owns row li of a 16-row tile and, for
  // k-substep s, granule s*4+lq (16-bit, fp4) or granules 2*lq, 2*lq+1 (fp8).
  const int li = lane & 15, lq = lane >> 4;
  unsigned rd_off[KSUB][KGRAN];
#pragma unroll
  for (int s = 0; s < KSUB; ++s)
#pragma unroll
    for (int h = 0; h < KGRAN; ++h) {
      const int g = (KGRAN == 2) ? (2 * lq + h) : (s * 4 + lq);
      rd_off[s][h] = (unsigned)(li * kRowBytes + ((g ^ (li >> 1)) << 4));
    }
  const unsigned a_rd = (unsigned)(wm * TM * 16 * kRowBytes);
  const unsigned b_rd = (unsigned)(STAGE_A + wn * TN * 16 * kRowBytes);

  // MX scale rows (fp4 only): lane reads the 8 e8m0 bytes of its row for this
  // K-step and shifts its own byte down.
  const uint8_t* mxa_row[DT == ASTERGEMM_MXFP4 ? TM : 1];
  const uint8_t* mxb_row[DT == ASTERGEMM_MXFP4 ? TN : 1];
  if constexpr (DT == ASTERGEMM_MXFP4) {
#pragma unroll
    for (int m = 0; m < TM; ++m) {
      int r = row0 + wm * TM * 16 + m * 16 + li;
      r = r < p.M ? r : p.M - 1;
      mxa_row[m] = p.mx_a + (int64_t)r * p.mx_ld;
    }
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      int r = col0 + wn * TN * 16 + n * 16 + li;
      r = r < p.N ? r : p.N - 1;
      mxb_row[n] = p.mx_b + (int64_t)r * p.mx_ld;
    }
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int m = 0; m < TM; ++m)
#pragma unroll
    for (int n = 0; n < TN; ++n) acc[m][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  // MX scales of a K-step are fetched one step ahead and ahead of that step's tile
  // transfers in issue order, so that waiting for them (loads return in order) neither
  // exposes their latency nor drains the transfers of the next stage.
  i32x2 sa[DT == ASTERGEMM_MXFP4 ? TM : 1], sb[DT == ASTERGEMM_MXFP4 ? TN : 1];
  i32x2 sa_nx[DT == ASTERGEMM_MXFP4 ? TM : 1], sb_nx[DT == ASTERGEMM_MXFP4 ? TN : 1];
  auto load_scales = [&](int kt) {
    if constexpr (DT == ASTERGEMM_MXFP4) {
#pragma unroll
      for (int m = 0; m < TM; ++m) sa_nx[m] = *(const i32x2*)(mxa_row[m] + kt * 8);
#pragma unroll
      for (int n = 0; n < TN; ++n) sb_nx[n] = *(const i32x2*)(mxb_row[n] + kt * 8);
    }
  };
  load_scales(0);
  stage_step(0, 0);

  for (int kt = 0; kt < p.ksteps; ++kt) {
    // All of this wave's transfers for step kt have landed; after the barrier
    // everybody's have, and everybody is done reading the other stage.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
    __syncthreads();
    if constexpr (DT == ASTERGEMM_MXFP4) {
#pragma unroll
      for (int m = 0; m < TM; ++m) sa[m] = sa_nx[m];
#pragma unroll
      for (int n = 0; n < TN; ++n) sb[n] = sb_nx[n];
    }
    if (kt + 1 < p.ksteps) {
      load_scales(kt + 1);
      stage_step(kt + 1, (kt + 1) & 1);
    }

    const uint8_t* st = lds + (kt & 1) * STAGE;
#pragma unroll
    for (int s = 0; s < KSUB; ++s) {
      i32x4 af[TM][KGRAN], bf[TN][KGRAN];
#pragma unroll
      for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int h = 0; h < KGRAN; ++h)
          af[m][h] = *(const i32x4*)(st + a_rd + m * 16 * kRowBytes + rd_off[s][h]);
#pragma unroll
      for (int n = 0; n < TN; ++n)
#pragma unroll
        for (int h = 0; h < KGRAN; ++h)
          bf[n][h] = *(const i32x4*)(st + b_rd + n * 16 * kRowBytes + rd_off[s][h]);
#pragma unroll
      for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int n = 0; n < TN; ++n) {
          int xa = 0, xb = 0;
          if constexpr (DT == ASTERGEMM_MXFP4) {
            xa = (int)((unsigned)(s ? sa[m].y : sa[m].x) >> (8 * lq));
            xb = (int)((unsigned)(s ? sb[n].y : sb[n].x) >> (8 * lq));
          }
          acc[m][n] = mfma_step<DT>(bf[n], af[m], acc[m][n], xb, xa);
        }
    }
  }

  // ---- epilogue: scale, bias, cast, vector store ----------------------------
  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  const bool vec_ok = (p.ldc & 3) == 0;
#pragma unroll
  for (int m = 0; m < TM; ++m) {
    const int row = row0 + (wm * TM + m) * 16 + li;
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      const int col = col0 + (wn * TN + n) * 16 + 4 * lq;
      if (row < p.M && col < p.N) {
        f32x4 v = acc[m][n] * scale;
        const int ncols = (p.N - col) < 4 ? (p.N - col) : 4;
        if (p.bias) {
          for (int r = 0; r < ncols; ++r) v[r] += p.bias[col + r];
        }
        store4<OUT>(p.C, (int64_t)row * p.ldc + col, v, vec_ok, ncols);
      }
    }
  }
}


template <int DT, int OUT, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_tile_kernel(const GemmArgs p) {
  gemm_tile_body<DT, OUT, BM, BN, WM, WN>(p);
}

}  // namespace
}  // namespace astergemm
