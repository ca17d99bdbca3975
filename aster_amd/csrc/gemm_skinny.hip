// Weight-streaming GEMM for decode shapes (M <= 64): C[M,N] = epi(A[M,K] * B[N,K]^T)
// with B (the weights, N x K) read exactly once from HBM.
//
// The reference has no skinny path (its kernels are all WG-tiled, LDS-staged:
// contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py); the
// closest thing is its "direct-B" operand path, where each lane's 16-byte global
// load IS its MFMA B operand (contrib/kittens/test/kittens_helpers.py:90-119).
// This kernel uses that idea without a host pre-shuffle: lane (i = lane%16,
// q = lane/16) loads bytes [16q, 16q+16) of every 64-byte K chunk of weight row
// n0+i straight into the srcA operand of v_mfma_f32_16x16x32_{bf16,f16}; the
// activations take the same K positions as srcB, so the K permutation cancels.
// It is HBM-bound: no LDS for weights, many 16-byte loads in flight per wave,
// K split over the waves of a workgroup and reduced through LDS.
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "astergemm_internal.h"

namespace astergemm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned short sk_f32_to_bf16(float f) {
  unsigned u = __builtin_bit_cast(unsigned, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}

// C[m][n .. n + ncols) = cast(v): the four neighbours one lane owns; one vector store where the
// row pitch keeps it aligned and all four columns exist.
template <int OUT>
__device__ __forceinline__ void sk_store_row4(void* C, int64_t ldc, int m, int n, const f32x4& v, int ncols) {
  const int64_t idx = (int64_t)m * ldc + n;
  const bool vec_ok = (ldc & 3) == 0 && ncols == 4;
  if constexpr (OUT == ASTERGEMM_F32) {
    float* o = (float*)C + idx;
    if (vec_ok) *(f32x4*)o = v;
    else
      for (int r = 0; r < ncols; ++r) o[r] = v[r];
  } else {
    unsigned short h[4];
    for (int r = 0; r < 4; ++r) {
      if constexpr (OUT == ASTERGEMM_BF16) h[r] = sk_f32_to_bf16(v[r]);
      else {
        const _Float16 hh = (_Float16)v[r];
        h[r] = __builtin_bit_cast(unsigned short, hh);
      }
    }
    unsigned short* o = (unsigned short*)C + idx;
    if (vec_ok) *(u16x4*)o = u16x4{h[0], h[1], h[2], h[3]};
    else
      for (int r = 0; r < ncols; ++r) o[r] = h[r];
  }
}

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <int DT>
__device__ __forceinline__ f32x4 sk_mfma(i32x4 a, i32x4 b, f32x4 c) {
  if constexpr (DT == ASTERGEMM_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// MT: 16-row activation tiles (M <= 16*MT); NB: 16-row weight blocks per
// workgroup; KW: waves splitting K; U: 64-byte K chunks in flight per wave.
template <int DT, int OUT, int MT, int NB, int KW, int U>
__global__ __launch_bounds__(KW * 64) void gemm_skinny_kernel(const GemmArgs p) {
  __shared__ f32x4 red[KW][MT * NB][64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  const int n0 = blockIdx.x * (NB * 16);

  // K slice of this wave, in 64-byte chunks (32 elements).
  const int chunks = p.K >> 5;
  const int per = (chunks + KW - 1) / KW;
  const int c_lo = wave * per;
  const int c_hi = (c_lo + per) < chunks ? (c_lo + per) : chunks;

  const uint8_t* wrow[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    int n = n0 + b * 16 + li;
    n = n < p.N ? n : p.N - 1;
    wrow[b] = p.B + (int64_t)n * p.ldb_bytes + lq * 16;
  }
  const uint8_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int m = t * 16 + li;
    m = m < p.M ? m : p.M - 1;
    xrow[t] = p.A + (int64_t)m * p.lda_bytes + lq * 16;
  }

  f32x4 acc[MT][NB];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[t][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  int c = c_lo;
  for (; c + U <= c_hi; c += U) {
    i32x4 w[U][NB], x[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int b = 0; b < NB; ++b)
        w[u][b] = __builtin_nontemporal_load((const i32x4*)(wrow[b] + (int64_t)(c + u) * 64));
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) x[u][t] = *(const i32x4*)(xrow[t] + (int64_t)(c + u) * 64);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[t][b] = sk_mfma<DT>(w[u][b], x[u][t], acc[t][b]);
  }
  for (; c < c_hi; ++c) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const i32x4 w = __builtin_nontemporal_load((const i32x4*)(wrow[b] + (int64_t)c * 64));
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const i32x4 x = *(const i32x4*)(xrow[t] + (int64_t)c * 64);
        acc[t][b] = sk_mfma<DT>(w, x, acc[t][b]);
      }
    }
  }

  // ---- reduce the KW partial sums through LDS --------------------------------
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int b = 0; b < NB; ++b) red[wave][t * NB + b][lane] = acc[t][b];
  __syncthreads();

  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;
  // Lane l of tile (t, b) owns C[t*16 + l%16][n0 + b*16 + 4*(l/16) + 0..3].
  for (int e = threadIdx.x; e < MT * NB * 64; e += KW * 64) {
    const int tb = e >> 6, l = e & 63;
    f32x4 v = red[0][tb][l];
#pragma unroll
    for (int k = 1; k < KW; ++k) v += red[k][tb][l];
    const int t = tb / NB, b = tb % NB;
    const int m = t * 16 + (l & 15);
    const int n = n0 + b * 16 + 4 * (l >> 4);
    if (m >= p.M || n >= p.N) continue;
    v *= scale;
    const int ncols = (p.N - n) < 4 ? (p.N - n) : 4;
    if (p.bias)
      for (int r = 0; r < ncols; ++r) v[r] += p.bias[n + r];
    sk_store_row4<OUT>(p.C, p.ldc, m, n, v, ncols);
  }
}

// ---- M <= 16: activations resident in registers, one persistent workgroup per CU ----
//
// The kernel above re-reads the activation rows from L2 for every 16 weight rows and
// fetches weights as 16 rows x 64 bytes per instruction (half cache lines), which
// holds M = 16 near 2.9 TB/s.  Here the eight waves of a workgroup split K into
// eight contiguous slices; a wave loads its slice of x once, straight into MFMA
// operand registers, and then streams a contiguous range of weight rows (N is split
// evenly over the grid in multiples of 8 rows, so no workgroup carries a whole extra
// 16-row block).  Weights are fetched with non-temporal loads of 8 rows x 128 bytes
// per instruction (whole cache lines), written to a wave-private LDS buffer and read
// back in MFMA operand order; same-wave LDS operations execute in order, so the
// transposition needs no barrier.  The partial 16x16 tiles of the eight waves are
// summed through LDS once per four 16-row blocks.  All weight loads are unconditional
// so that the wait counts stay exact: rows past the end of the range are clamped to
// the last valid one (the same lines, in the same instruction), and the two units
// prefetched past the last block read the first line of x instead, because weight
// lines are fetched non-temporally and would come from HBM a second time.
//
// SPB = 128-byte steps per wave and block = K / 512; a unit of work is four steps
// (eight loads, eight MFMAs) and two units are kept in flight per wave.
//
// Rows of 4 KiB (SPB = 4: a unit is a wave's whole 512-byte slice of 16 rows) are fetched as
// 2 rows x 512 contiguous bytes per instruction instead of 8 rows x 128 bytes: measured back to
// back over rotating weight sets, M = 16, 8 rows x 128 -> 2 rows x 512: fp8 14336 x 4096 14.2 ->
// 12.7 us, fp8 28672 x 4096 25.5 -> 22.1, bf16 28672 x 2048 25.4 -> 22.7.  On longer rows, where a
// unit is half or a quarter of the slice, the same change loses 3-5 % (bf16 14336 x 4096 20.6 ->
// 21.6 us, x 8192 38.0 -> 39.2, fp8 x 8192 20.9 -> 21.5), and so does one row x 1 KiB per
// instruction with a block per LDS pass (bf16 14336 x 4096 21.6): they keep 8 rows x 128 bytes.
template <int DT, int OUT, int SPB>
__global__ __launch_bounds__(512) void gemm_skinny_reg_kernel(const GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr int KW = 8;
  constexpr int UPB = SPB / 4;                   // units per block
  constexpr int slice = SPB * 128;               // bytes of every row owned by one wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  uint8_t* tbuf = slds + wave * 8192;            // 4 steps x 2 KiB, private to the wave
  constexpr int NBS = 4;                         // blocks between workgroup barriers
  f32x4* red = (f32x4*)(slds + KW * 8192);       // [2][NBS][KW][64]

  // rows [r0, r1) of the weight matrix belong to this workgroup
  const int g = gridDim.x;
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = blockIdx.x * per;
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nblk = (r1 - r0 + 15) >> 4;
  const int total = nblk * UPB;

  // load: lane -> row (lane >> 3) of an 8-row half block, 16-byte piece (lane & 7)
  const int lrow = lane >> 3, lpiece = lane & 7;
  const uint8_t* wbase = p.B + wave * slice + lpiece * 16;
  constexpr bool CONTIG = UPB == 1;              // 2 rows x 512 contiguous bytes per instruction
  const int hi = lane >> 5, p32 = lane & 31;     // CONTIG: row of the pair, piece of its 512 bytes
  auto issue = [&](int j, i32x4(&dst)[8]) {      // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {              // instruction i: rows 2 i and 2 i + 1 of the block
        const int nh = r0 + blk * 16 + 2 * i;
        int n = nh + hi;
        n = n < r1 ? n : r1 - 1;
        const uint8_t* src = p.B + wave * slice + (int64_t)n * p.ldb_bytes + p32 * 16;
        if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
        dst[i] = __builtin_nontemporal_load((const i32x4*)src);
      }
      return;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int nh = r0 + blk * 16 + h * 8;
      int n = nh + lrow;
      n = n < r1 ? n : r1 - 1;
      const uint8_t* src = wbase + (int64_t)n * p.ldb_bytes + t * 512;
      if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
#pragma unroll
      for (int s = 0; s < 4; ++s)
        dst[s * 2 + h] = __builtin_nontemporal_load((const i32x4*)(src + s * 128));
    }
  };

  // LDS transposition: 128-byte rows, 16-byte piece index XOR (row & 7)
  const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);          // + h * 1024 + s * 2048
  const int rd_off = li * 128;                                     // + ((4u + lq) ^ (li & 7)) * 16
  // stash: registers of one unit -> the wave's LDS buffer (frees the registers)
  auto stash = [&](const i32x4(&src)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = src[i];
  };
  // the same LDS layout from the CONTIG load pattern: register i holds, for row r = 2 i + hi,
  // piece p32 of the 512 bytes = piece (p32 & 7) of step (p32 >> 3)
  const int wr_c = (p32 >> 3) * 2048 + hi * 128;
  const int pch = ((p32 & 7) ^ hi) << 4;
  auto stash_w = [&](const i32x4(&src)[8]) {
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *(i32x4*)(tbuf + wr_c + (i >> 2) * 1024 + (i & 3) * 256 + (pch ^ ((i & 3) << 5))) = src[i];
    } else {
      stash(src);
    }
  };
  auto operand = [&](int s, int u) {             // MFMA operand (row li, K piece 4u + lq) of step s
    return *(const i32x4*)(tbuf + s * 2048 + rd_off + (((4 * u + lq) ^ (li & 7)) << 4));
  };

  // x: operand registers for the SPB*2 MFMAs of a block, fetched like the weights
  // (whole lines, then through the LDS buffer) but cacheable: every workgroup reads
  // them.  The loads of the first two units go out ahead of the first weight loads
  // and are consumed while those are in flight.
  i32x4 x[SPB * 2];
  auto x_load = [&](int t, i32x4(&dst)[8]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int m = h * 8 + lrow;
      m = m < p.M ? m : p.M - 1;
      const uint8_t* src = p.A + (int64_t)m * p.lda_bytes + wave * slice + t * 512 + lpiece * 16;
#pragma unroll
      for (int s = 0; s < 4; ++s) dst[s * 2 + h] = *(const i32x4*)(src + s * 128);
    }
  };
  auto x_keep = [&](auto T, const i32x4(&src)[8]) {
    constexpr int t = decltype(T)::value;
    stash(src);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[t * 8 + i] = operand(i >> 1, i & 1);
  };
  i32x4 w0[8], w1[8];
  {
    i32x4 xa[8], xb[8];
    x_load(0, xa);
    if constexpr (UPB > 1) x_load(1, xb);
    __builtin_amdgcn_sched_barrier(0);
    issue(0, w0);
    issue(1, w1);
    __builtin_amdgcn_sched_barrier(0);
    x_keep(std::integral_constant<int, 0>{}, xa);
    if constexpr (UPB > 1) x_keep(std::integral_constant<int, 1>{}, xb);
    static_for<2, UPB>([&](auto T) {
      x_load(decltype(T)::value, xa);
      x_keep(T, xa);
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  int parity = 0;

  // Partial tiles go to red[parity][block % NBS][wave]; the workgroup meets only once
  // per NBS blocks, then wave b sums and stores block b of the group.
  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
    red[((parity * NBS + slot) * KW + wave) * 64 + lane] = acc;
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave <= slot) {
      const f32x4* src = red + ((parity * NBS + wave) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = li, n = r0 + (blk - slot + wave) * 16 + 4 * lq;
      if (m < p.M && n < r1) {
        v *= scale;
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        if (p.bias)
          for (int r = 0; r < ncols; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, ncols);
      }
    }
    parity ^= 1;
  };

  // T = unit index inside the block (compile time: selects the x registers)
  auto mma = [&](int blk, auto T) {
    constexpr int t = decltype(T)::value;
    if constexpr (DT == ASTERGEMM_FP8_E4M3) {
      // one 16x16x128 MFMA per 128-byte step: a lane's 32 operand bytes are pieces lq and
      // 4 + lq of the row, for the weights and the activations alike
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const i32x4 lo = operand(s, 0), hi = operand(s, 1);
        const i32x4 xl = x[t * 8 + 2 * s], xh = x[t * 8 + 2 * s + 1];
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]},
            i32x8{xl[0], xl[1], xl[2], xl[3], xh[0], xh[1], xh[2], xh[3]}, acc, 0, 0, 0, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc = sk_mfma<DT>(operand(i >> 1, i & 1), x[t * 8 + i], acc);
      }
    }
    if (t == UPB - 1) block_end(blk);
  };

  // TRIP flat steps per trip so that register sets and x indices are static
  constexpr int TRIP = UPB < 2 ? 2 : UPB;
  int j = 0;
  for (; j + TRIP <= total; j += TRIP) {
    const int blk = j / UPB;
    static_for<0, TRIP / 2>([&](auto I) {
      constexpr int i = decltype(I)::value * 2;
      // each register set is refilled as soon as its unit has been written to LDS;
      // the scheduler must not move the loads across the units they overlap with
      stash_w(w0);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 2, w0);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + i / UPB, std::integral_constant<int, i % UPB>{});
      __builtin_amdgcn_sched_barrier(0);
      stash_w(w1);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w1);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + (i + 1) / UPB, std::integral_constant<int, (i + 1) % UPB>{});
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  if (j < total) {  // UPB == 1, odd block count
    stash_w(w0);
    mma(j / UPB, std::integral_constant<int, 0>{});
  }
}

template <int DT, int OUT, int SPB>
int launch_skinny_reg_t(const GemmArgs& a, hipStream_t s) {
  auto k = gemm_skinny_reg_kernel<DT, OUT, SPB>;
  constexpr int lds = 8 * 8192 + 2 * 4 * 8 * 64 * 16;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  const int nblocks = (int)((a.N + 15) / 16);
  const int g = nblocks < cus ? nblocks : cus;
  AG_LAUNCH_KERNEL(k, dim3(g), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

// ---- M <= 16, MXFP4 weights and activations ---------------------------------------------
//
// The resident-activation kernel for e2m1 nibbles with e8m0 block scales.  A 128-byte step of
// a row is 256 elements = two v_mfma_scale_f32_16x16x128_f8f6f4 (cbsz = blgp = 4), each taking
// one 16-byte piece (32 elements, one scale byte) per lane: piece 4u + lq of the step, for the
// weights and the activations alike.  The scale bytes of a step are 8 consecutive bytes of the
// row's scale plane; a lane loads them with the unit's weights (two dwords per step, the same
// address for the four lanes that share a row) and shifts its own byte down to byte 0, which is
// the byte the instruction reads.  The activations' scale bytes are shifted once and stay in
// registers with the activations.
// SPB = 128-byte steps per wave and row (K / 2048), SU = steps per unit (4, or 2 at K = 4096).
template <int OUT, int SPB, int SU>
__global__ __launch_bounds__(512) void gemm_skinny_fp4_kernel(const GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr int KW = 8;
  constexpr int UPB = SPB / SU;                  // units per block
  constexpr int NL = 2 * SU;                     // loads per unit
  constexpr int slice = SPB * 128;               // bytes of every row owned by one wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  uint8_t* tbuf = slds + wave * 8192;            // SU steps x 2 KiB, private to the wave
  constexpr int NBS = 4;                         // blocks between workgroup barriers
  f32x4* red = (f32x4*)(slds + KW * 8192);       // [2][NBS][KW][64]

  const int g = gridDim.x;
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = blockIdx.x * per;
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nblk = (r1 - r0 + 15) >> 4;
  const int total = nblk * UPB;

  const int lrow = lane >> 3, lpiece = lane & 7;
  const uint8_t* wbase = p.B + wave * slice + lpiece * 16;
  const uint8_t* sbase = p.mx_b + wave * (SPB * 8);       // this wave's scale bytes of a row
  // a unit that is the wave's whole slice of a row (UPB == 1) is fetched as R rows x SU * 128
  // contiguous bytes per instruction instead of 8 rows x 128 bytes (see gemm_skinny_reg_kernel)
  constexpr bool CONTIG = UPB == 1;
  constexpr int R = 16 / NL, LPR = 64 / R;       // rows per instruction, lanes (pieces) per row
  const int rsel = lane / LPR, pidx = lane % LPR;
  auto issue = [&](int j, i32x4(&dst)[NL], i32x2(&sc)[SU]) {  // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {             // instruction i: rows R i .. R i + R - 1 of the block
        const int nh = r0 + blk * 16 + R * i;
        int n = nh + rsel;
        n = n < r1 ? n : r1 - 1;
        const uint8_t* src = p.B + wave * slice + (int64_t)n * p.ldb_bytes + pidx * 16;
        if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
        dst[i] = __builtin_nontemporal_load((const i32x4*)src);
      }
    }
#pragma unroll
    for (int h = 0; h < (CONTIG ? 0 : 2); ++h) {
      const int nh = r0 + blk * 16 + h * 8;
      int n = nh + lrow;
      n = n < r1 ? n : r1 - 1;
      const uint8_t* src = wbase + (int64_t)n * p.ldb_bytes + t * (SU * 128);
      if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
#pragma unroll
      for (int s = 0; s < SU; ++s)
        dst[s * 2 + h] = __builtin_nontemporal_load((const i32x4*)(src + s * 128));
    }
    int n = r0 + blk * 16 + li;                  // the row this lane multiplies
    n = n < r1 ? n : r1 - 1;
    const uint8_t* ssrc = sbase + (int64_t)n * p.mx_ld + t * (SU * 8);
#pragma unroll
    for (int s = 0; s < SU; ++s) sc[s] = *(const i32x2*)(ssrc + s * 8);
  };

  const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);
  const int rd_off = li * 128;
  auto stash = [&](const i32x4(&src)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i)
      *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = src[i];
  };
  // the same LDS layout from the CONTIG load pattern: register i holds, for row r = R i + rsel,
  // piece (pidx & 7) of step (pidx >> 3)
  const int wr_c = (pidx >> 3) * 2048 + rsel * 128;
  const int pch = ((pidx & 7) ^ rsel) << 4;
  auto stash_w = [&](const i32x4(&src)[NL]) {
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int rr = R * i;                    // compile time after unrolling
        *(i32x4*)(tbuf + wr_c + (rr >> 3) * 1024 + (rr & 7) * 128 + (pch ^ ((rr & 7) << 4))) = src[i];
      }
    } else {
      stash(src);
    }
  };
  auto operand = [&](int s, int u) {             // piece 4u + lq of step s, row li
    return *(const i32x4*)(tbuf + s * 2048 + rd_off + (((4 * u + lq) ^ (li & 7)) << 4));
  };

  // x and its scales: operand registers for the SPB * 2 MFMAs of a block
  i32x4 x[SPB * 2];
  int xs[SPB * 2];
  {
    const int m = li < p.M ? li : p.M - 1;
    const uint8_t* xsrc = p.mx_a + (int64_t)m * p.mx_ld + wave * (SPB * 8);
#pragma unroll
    for (int s = 0; s < SPB; ++s) {
      const i32x2 v = *(const i32x2*)(xsrc + s * 8);
      xs[s * 2] = (int)((unsigned)v[0] >> (8 * lq));
      xs[s * 2 + 1] = (int)((unsigned)v[1] >> (8 * lq));
    }
  }
  auto x_load = [&](int t, i32x4(&dst)[NL]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int m = h * 8 + lrow;
      m = m < p.M ? m : p.M - 1;
      const uint8_t* src = p.A + (int64_t)m * p.lda_bytes + wave * slice + t * (SU * 128) + lpiece * 16;
#pragma unroll
      for (int s = 0; s < SU; ++s) dst[s * 2 + h] = *(const i32x4*)(src + s * 128);
    }
  };
  i32x4 w0[NL], w1[NL];
  i32x2 s0[SU], s1[SU];
  {
    i32x4 xa[NL];
    issue(0, w0, s0);
    issue(1, w1, s1);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, UPB>([&](auto T) {
      constexpr int t = decltype(T)::value;
      x_load(t, xa);
      stash(xa);
#pragma unroll
      for (int i = 0; i < NL; ++i) x[t * NL + i] = operand(i >> 1, i & 1);
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  int parity = 0;

  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
    red[((parity * NBS + slot) * KW + wave) * 64 + lane] = acc;
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave <= slot) {
      const f32x4* src = red + ((parity * NBS + wave) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = li, n = r0 + (blk - slot + wave) * 16 + 4 * lq;
      if (m < p.M && n < r1) {
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        if (p.bias)
          for (int r = 0; r < ncols; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, ncols);
      }
    }
    parity ^= 1;
  };

  // T = unit index inside the block (compile time: selects the x registers); sc = the unit's
  // weight scale dwords, this lane's byte already in byte 0
  auto mma = [&](int blk, auto T, const int (&sc)[NL]) {
    constexpr int t = decltype(T)::value;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const i32x4 w = operand(i >> 1, i & 1);
      const i32x4 xv = x[t * NL + i];
      acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
          i32x8{w[0], w[1], w[2], w[3], 0, 0, 0, 0}, i32x8{xv[0], xv[1], xv[2], xv[3], 0, 0, 0, 0},
          acc, 4, 4, 0, sc[i], 0, xs[t * NL + i]);
    }
    if (t == UPB - 1) block_end(blk);
  };
  auto take_scales = [&](const i32x2(&src)[SU], int (&dst)[NL]) {
#pragma unroll
    for (int s = 0; s < SU; ++s) {
      dst[s * 2] = (int)((unsigned)src[s][0] >> (8 * lq));
      dst[s * 2 + 1] = (int)((unsigned)src[s][1] >> (8 * lq));
    }
  };

  constexpr int TRIP = UPB < 2 ? 2 : UPB;
  int j = 0;
  int sc[NL];
  for (; j + TRIP <= total; j += TRIP) {
    const int blk = j / UPB;
    static_for<0, TRIP / 2>([&](auto I) {
      constexpr int i = decltype(I)::value * 2;
      stash_w(w0);
      take_scales(s0, sc);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 2, w0, s0);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + i / UPB, std::integral_constant<int, i % UPB>{}, sc);
      __builtin_amdgcn_sched_barrier(0);
      stash_w(w1);
      take_scales(s1, sc);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w1, s1);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + (i + 1) / UPB, std::integral_constant<int, (i + 1) % UPB>{}, sc);
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  if (j < total) {  // UPB == 1, odd block count
    stash_w(w0);
    take_scales(s0, sc);
    mma(j / UPB, std::integral_constant<int, 0>{}, sc);
  }
}

template <int OUT, int SPB, int SU>
int launch_skinny_fp4_t(const GemmArgs& a, hipStream_t s) {
  auto k = gemm_skinny_fp4_kernel<OUT, SPB, SU>;
  constexpr int lds = 8 * 8192 + 2 * 4 * 8 * 64 * 16;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  const int nblocks = (int)((a.N + 15) / 16);
  const int g = nblocks < cus ? nblocks : cus;
  AG_LAUNCH_KERNEL(k, dim3(g), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

template <int OUT>
int launch_skinny_fp4(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  switch (a.K) {  // eight waves x SPB steps of 256 elements
    case 4096: return launch_skinny_fp4_t<OUT, 2, 2>(a, s);
    case 8192: return launch_skinny_fp4_t<OUT, 4, 4>(a, s);
    case 16384: return launch_skinny_fp4_t<OUT, 8, 4>(a, s);
  }
  return (int)hipErrorInvalidValue;
}

const char* check_skinny_fp4(const astergemm_config& c) {
  if (c.M > 16) return "resident-activation MXFP4 path needs M <= 16";
  if (c.K != 4096 && c.K != 8192 && c.K != 16384)
    return "resident-activation MXFP4 path needs K = 4096, 8192 or 16384";
  return nullptr;
}

#define AG_SKINNY_FP4(name, OUT)                                                           \
  Variant {                                                                                \
    name, ASTERGEMM_KERNEL_SKINNY, ASTERGEMM_MXFP4, OUT, 16, 16, 512, 1, 8, 1, 3,           \
        8 * 8192 + 65536, (const void*)gemm_skinny_fp4_kernel<OUT, 2, 2>,                  \
        launch_skinny_fp4<OUT>, check_skinny_fp4                                           \
  }

// ---- rows cut into K ranges: partial sums, their workspace and the kernel that adds them ---

// out[m][n..n+3] = cast(scale * sum over K ranges of partial[s][m][n..] + bias), ranges added in
// index order; a thread takes four neighbours and has all of a pass's loads in flight at once
template <int OUT>
__global__ __launch_bounds__(256) void skinny_splitk_reduce_kernel(const float* ws, int S, int M,
                                                                   int N, int64_t ldc,
                                                                   const float* scale_a,
                                                                   const float* scale_b,
                                                                   const float* bias, void* C) {
  float scale = 1.0f;
  if (scale_a) scale *= *scale_a;
  if (scale_b) scale *= *scale_b;
  const int cg = (N + 3) >> 2;                     // groups of four columns per row
  const int64_t plane = (int64_t)M * N;
  const bool vec = (N & 3) == 0;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < (int64_t)M * cg;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int m = (int)(i / cg), n = (int)(i - (int64_t)m * cg) * 4;
    const int ncols = (N - n) < 4 ? (N - n) : 4;
    const float* src = ws + (int64_t)m * N + n;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < S; s0 += 8) {
      f32x4 t[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const int sc = (s0 + s) < S ? (s0 + s) : S - 1;
        const float* q = src + sc * plane;
        if (vec) t[s] = *(const f32x4*)q;
        else
          for (int r = 0; r < 4; ++r) t[s][r] = r < ncols ? q[r] : 0.f;
      }
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s0 + s < S) v += t[s];
    }
    v *= scale;
    if (bias)
      for (int r = 0; r < ncols; ++r) v[r] += bias[n + r];
    sk_store_row4<OUT>(C, ldc, m, n, v, ncols);
  }
}

template <int OUT>
void launch_splitk_reduce(const GemmArgs& a, int S, hipStream_t s) {
  const int64_t total = (int64_t)a.M * ((a.N + 3) / 4);
  const int rg = (int)((total + 255) / 256 < 2048 ? (total + 255) / 256 : 2048);
  AG_LAUNCH_KERNEL(skinny_splitk_reduce_kernel<OUT>, dim3(rg), dim3(256), 0, s, a.workspace, S,
                     a.M, a.N, a.ldc, a.scale_a, a.scale_b, a.bias, a.C);
}

// fp32 scratch for the K-split partial sums when the caller brings none: one buffer per
// (device, stream), so launches on different streams never share one; launches on one stream are
// ordered and reuse it.  A buffer that is too small is replaced by one at least twice its size
// and stays allocated (kernels already enqueued, or being enqueued by another host thread, keep a
// valid pointer), so the retired buffers together stay below the size of the live one; nothing
// is released before the process ends.
struct SplitWorkspace {
  float* ptr = nullptr;
  size_t bytes = 0;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, SplitWorkspace> g_ws;
std::vector<float*> g_ws_retired;

int splitk_workspace(size_t bytes, hipStream_t stream, float** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return (int)hipGetLastError();
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  SplitWorkspace& w = g_ws[{dev, stream}];
  if (bytes > w.bytes) {
    size_t want = bytes < ((size_t)8 << 20) ? ((size_t)8 << 20) : bytes;
    if (want < 2 * w.bytes) want = 2 * w.bytes;
    float* fresh = nullptr;
    if (hipMalloc((void**)&fresh, want) != hipSuccess) return (int)hipGetLastError();
    if (w.ptr) g_ws_retired.push_back(w.ptr);
    w.ptr = fresh;
    w.bytes = want;
  }
  *out = w.ptr;
  return 0;
}

// Gives back the workspace of a stream that is about to be destroyed.  The caller has
// synchronised the stream: nothing enqueued on it can still use the buffer.
void splitk_workspace_drop(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_ws.find({dev, stream});
  if (it == g_ws.end()) return;
  if (it->second.ptr) (void)hipFree(it->second.ptr);
  g_ws.erase(it);
}

// Grid of the K-range decode kernels: S K ranges x R row ranges, one workgroup per CU; with
// mh = 2 two workgroups share a row range, in whole pairs on each of the 8 XCDs.  The launchers
// and the description of a variant both come here.
struct KRangeGrid {
  int mh, rows, grid;
};
inline KRangeGrid krange_grid(int mh, int64_t N, int S, int cus) {
  KRangeGrid g;
  g.mh = mh;
  const int nblocks = (int)((N + 15) / 16);
  const int slots = g.mh == 2 ? (cus / 16) * 8 : cus;
  int R = slots / S;
  g.rows = R < 1 ? 1 : (R > nblocks ? nblocks : R);
  g.grid = g.mh * S * g.rows;
  if (g.mh == 2) g.grid = (g.grid + 15) & ~15;
  return g;
}

// The MXFP4 kernel above with two activation tiles per wave and, for M > 32, two workgroups
// per weight row range (see gemm_skinny_regm_kernel).
template <int OUT, int SPB, int SU, int MT, int MH>
__global__ __launch_bounds__(512) void gemm_skinny_fp4m_kernel(const GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr int KW = 8;
  constexpr int UPB = SPB / SU;                  // units per block
  constexpr int NL = 2 * SU;                     // loads per unit
  constexpr int slice = SPB * 128;               // bytes of every row owned by one wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  uint8_t* tbuf = slds + wave * 8192;            // SU steps x 2 KiB, private to the wave
  constexpr int NBS = 2;                         // blocks between workgroup barriers
  f32x4* red = (f32x4*)(slds + KW * 8192);       // [2][NBS][MT][KW][64]

  // block b runs on XCD b % 8; with MH = 2 blocks b and b + 8 share a row range.  Rows longer
  // than the 8 waves' slices are cut into p.split_k K ranges (see gemm_skinny_regm_kernel): a
  // workgroup takes one K range of one of p.tiles_n row ranges; a wave whose slice lies
  // behind the row's end multiplies zeros with unit scales.
  const int q = blockIdx.x >> 3;
  const int half = MH == 2 ? (q & 1) : 0;
  const int idx = MH == 2 ? ((q >> 1) << 3) | (blockIdx.x & 7) : (int)blockIdx.x;
  const int g = p.tiles_n;                       // row ranges
  if (idx >= g * p.split_k) return;
  const int ks = idx / g, rid = idx - ks * g;
  const int64_t koff = (int64_t)ks * (KW * slice);
  const bool dead = koff + (wave + 1) * slice > p.K / 2;
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = rid * per;
  const int m0 = half * MT * 16;                 // first activation row of this workgroup
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nblk = (r1 - r0 + 15) >> 4;
  const int total = nblk * UPB;

  const int lrow = lane >> 3, lpiece = lane & 7;
  const uint8_t* wbase = p.B + koff + wave * slice + lpiece * 16;
  const uint8_t* sbase = p.mx_b + koff / 16 + wave * (SPB * 8);  // this wave's scale bytes of a row
  // a unit that is the wave's whole slice of a row (UPB == 1): R rows x SU * 128 contiguous bytes
  // per instruction instead of 8 rows x 128 bytes (see gemm_skinny_reg_kernel)
  constexpr bool CONTIG = UPB == 1;
  constexpr int R = 16 / NL, LPR = 64 / R;       // rows per instruction, lanes (pieces) per row
  const int rsel = lane / LPR, pidx = lane % LPR;
  auto issue = [&](int j, i32x4(&dst)[NL], i32x2(&sc)[SU]) {  // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    if (dead) {
#pragma unroll
      for (int i = 0; i < NL; ++i) dst[i] = i32x4{0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < SU; ++s) sc[s] = i32x2{0x7F7F7F7F, 0x7F7F7F7F};
      return;
    }
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {             // instruction i: rows R i .. R i + R - 1 of the block
        const int nh = r0 + blk * 16 + R * i;
        int n = nh + rsel;
        n = n < r1 ? n : r1 - 1;
        const uint8_t* src = p.B + koff + wave * slice + (int64_t)n * p.ldb_bytes + pidx * 16;
        if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
        dst[i] = __builtin_nontemporal_load((const i32x4*)src);
      }
    }
#pragma unroll
    for (int h = 0; h < (CONTIG ? 0 : 2); ++h) {
      const int nh = r0 + blk * 16 + h * 8;
      int n = nh + lrow;
      n = n < r1 ? n : r1 - 1;
      const uint8_t* src = wbase + (int64_t)n * p.ldb_bytes + t * (SU * 128);
      if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
#pragma unroll
      for (int s = 0; s < SU; ++s)
        dst[s * 2 + h] = __builtin_nontemporal_load((const i32x4*)(src + s * 128));
    }
    int n = r0 + blk * 16 + li;                  // the row this lane multiplies
    n = n < r1 ? n : r1 - 1;
    const uint8_t* ssrc = sbase + (int64_t)n * p.mx_ld + t * (SU * 8);
#pragma unroll
    for (int s = 0; s < SU; ++s) sc[s] = *(const i32x2*)(ssrc + s * 8);
  };

  const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);
  const int rd_off = li * 128;
  auto stash = [&](const i32x4(&src)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i)
      *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = src[i];
  };
  const int wr_c = (pidx >> 3) * 2048 + rsel * 128;
  const int pch = ((pidx & 7) ^ rsel) << 4;
  auto stash_w = [&](const i32x4(&src)[NL]) {
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int rr = R * i;                    // compile time after unrolling
        *(i32x4*)(tbuf + wr_c + (rr >> 3) * 1024 + (rr & 7) * 128 + (pch ^ ((rr & 7) << 4))) = src[i];
      }
    } else {
      stash(src);
    }
  };
  auto operand = [&](int s, int u) {             // piece 4u + lq of step s, row li
    return *(const i32x4*)(tbuf + s * 2048 + rd_off + (((4 * u + lq) ^ (li & 7)) << 4));
  };

  // x and its scales: operand registers for the SPB * 2 MFMAs of a block
  i32x4 x[MT][SPB * 2];
  int xs[MT][SPB * 2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = m0 + mt * 16 + li;
    m = m < p.M ? m : p.M - 1;
    const uint8_t* xsrc = p.mx_a + (int64_t)m * p.mx_ld + koff / 16 + wave * (SPB * 8);
#pragma unroll
    for (int s = 0; s < SPB; ++s) {
      const i32x2 v = dead ? i32x2{0x7F7F7F7F, 0x7F7F7F7F} : *(const i32x2*)(xsrc + s * 8);
      xs[mt][s * 2] = (int)((unsigned)v[0] >> (8 * lq));
      xs[mt][s * 2 + 1] = (int)((unsigned)v[1] >> (8 * lq));
    }
  }
  auto x_load = [&](int mt, int t, i32x4(&dst)[NL]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int m = m0 + mt * 16 + h * 8 + lrow;
      m = m < p.M ? m : p.M - 1;
      const uint8_t* src =
          p.A + (int64_t)m * p.lda_bytes + koff + wave * slice + t * (SU * 128) + lpiece * 16;
#pragma unroll
      for (int s = 0; s < SU; ++s)
        dst[s * 2 + h] = dead ? i32x4{0, 0, 0, 0} : *(const i32x4*)(src + s * 128);
    }
  };
  i32x4 w0[NL], w1[NL];
  i32x2 s0[SU], s1[SU];
  {
    i32x4 xa[NL];
    issue(0, w0, s0);
    issue(1, w1, s1);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, MT * UPB>([&](auto T) {
      constexpr int mt = decltype(T)::value / UPB, t = decltype(T)::value % UPB;
      x_load(mt, t, xa);
      stash(xa);
#pragma unroll
      for (int i = 0; i < NL; ++i) x[mt][t * NL + i] = operand(i >> 1, i & 1);
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int parity = 0;

  // wave w sums and stores tile w % MT of block w / MT of the group
  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      red[(((parity * NBS + slot) * MT + mt) * KW + wave) * 64 + lane] = acc[mt];
      acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave < (slot + 1) * MT) {
      const int rb = wave / MT, rt = wave % MT;
      const f32x4* src = red + (((parity * NBS + rb) * MT + rt) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = m0 + rt * 16 + li, n = r0 + (blk - slot + rb) * 16 + 4 * lq;
      if (m < p.M && n < r1 && p.split_k > 1) {
        // sums over this K range only: [range][M][N] fp32, added up by the reduce kernel
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        float* o = p.workspace + ((int64_t)ks * p.M + m) * p.N + n;
        if ((p.N & 3) == 0 && ncols == 4) *(f32x4*)o = v;
        else
          for (int r = 0; r < ncols; ++r) o[r] = v[r];
      } else if (m < p.M && n < r1) {
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        if (p.bias)
          for (int r = 0; r < ncols; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, ncols);
      }
    }
    parity ^= 1;
  };

  // T = unit index inside the block (compile time: selects the x registers); sc = the unit's
  // weight scale dwords, this lane's byte already in byte 0
  auto mma = [&](int blk, auto T, const int (&sc)[NL]) {
    constexpr int t = decltype(T)::value;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const i32x4 w = operand(i >> 1, i & 1);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const i32x4 xv = x[mt][t * NL + i];
        acc[mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8{w[0], w[1], w[2], w[3], 0, 0, 0, 0},
            i32x8{xv[0], xv[1], xv[2], xv[3], 0, 0, 0, 0}, acc[mt], 4, 4, 0, sc[i], 0,
            xs[mt][t * NL + i]);
      }
    }
    if (t == UPB - 1) block_end(blk);
  };
  auto take_scales = [&](const i32x2(&src)[SU], int (&dst)[NL]) {
#pragma unroll
    for (int s = 0; s < SU; ++s) {
      dst[s * 2] = (int)((unsigned)src[s][0] >> (8 * lq));
      dst[s * 2 + 1] = (int)((unsigned)src[s][1] >> (8 * lq));
    }
  };

  constexpr int TRIP = UPB < 2 ? 2 : UPB;
  int j = 0;
  int sc[NL];
  for (; j + TRIP <= total; j += TRIP) {
    const int blk = j / UPB;
    static_for<0, TRIP / 2>([&](auto I) {
      constexpr int i = decltype(I)::value * 2;
      stash_w(w0);
      take_scales(s0, sc);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 2, w0, s0);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + i / UPB, std::integral_constant<int, i % UPB>{}, sc);
      __builtin_amdgcn_sched_barrier(0);
      stash_w(w1);
      take_scales(s1, sc);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w1, s1);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + (i + 1) / UPB, std::integral_constant<int, (i + 1) % UPB>{}, sc);
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  if (j < total) {  // UPB == 1, odd block count
    stash_w(w0);
    take_scales(s0, sc);
    mma(j / UPB, std::integral_constant<int, 0>{}, sc);
  }
}

// K ranges for an MXFP4 row of `rb` bytes of nibbles: ranges of 4 KiB when the row is a whole
// number of them, else of 2 KiB in 256-byte slices, the last one possibly short; 0 when the
// row is shorter than 2 KiB, not whole slices, or needs more than 16 ranges.
__host__ inline int skinny_fp4_split_of(int64_t rb, int* spb) {
  if (rb < 2048) return 0;
  if (rb % 4096 == 0 && rb / 4096 <= 16) return *spb = 4, (int)(rb / 4096);
  if (rb % 256 == 0 && (rb + 2047) / 2048 <= 16) return *spb = 2, (int)((rb + 2047) / 2048);
  return 0;
}

template <int OUT, int SPB, int SU, int MT, int MH>
int launch_skinny_fp4m_t(const GemmArgs& a0, int S, hipStream_t s) {
  auto k = gemm_skinny_fp4m_kernel<OUT, SPB, SU, MT, MH>;
  constexpr int lds = 8 * 8192 + 2 * 2 * MT * 8 * 64 * 16;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  GemmArgs a = a0;
  const KRangeGrid kg = krange_grid(MH, a.N, S, cus);
  a.tiles_n = kg.rows;
  a.split_k = S;
  if (S > 1 && !a.workspace) {
    if (int rc = splitk_workspace((size_t)S * a.M * a.N * sizeof(float), s, &a.workspace)) return rc;
  }
  AG_LAUNCH_KERNEL(k, dim3(kg.grid), dim3(512), lds, s, a);
  // the partial sums must exist before anything adds them: a failed launch ends here
  if (const hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
  if (S > 1) launch_splitk_reduce<OUT>(a, S, s);
  return (int)hipGetLastError();
}

template <int OUT>
int launch_skinny_fp4m(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  int spb = 0;
  const int S = skinny_fp4_split_of(a.K / 2, &spb);
  if (S == 0) return (int)hipErrorInvalidValue;
  if (a.M <= 16)
    return spb == 4 ? launch_skinny_fp4m_t<OUT, 4, 4, 1, 1>(a, S, s)
                    : launch_skinny_fp4m_t<OUT, 2, 2, 1, 1>(a, S, s);
  if (a.M <= 32)
    return spb == 4 ? launch_skinny_fp4m_t<OUT, 4, 4, 2, 1>(a, S, s)
                    : launch_skinny_fp4m_t<OUT, 2, 2, 2, 1>(a, S, s);
  return spb == 4 ? launch_skinny_fp4m_t<OUT, 4, 4, 2, 2>(a, S, s)
                  : launch_skinny_fp4m_t<OUT, 2, 2, 2, 2>(a, S, s);
}

const char* check_skinny_fp4m(const astergemm_config& c) {
  if (c.M > 64) return "resident-activation MXFP4 path needs M <= 64";
  int spb = 0;
  if (skinny_fp4_split_of(c.K / 2, &spb) == 0)
    return "resident-activation MXFP4 path needs K >= 4096, a multiple of 512, at most 65536 "
           "(131072 in multiples of 8192)";
  return nullptr;
}

int splits_skinny_fp4m(const astergemm_config& c) {
  int spb = 0;
  const int S = skinny_fp4_split_of(c.K / 2, &spb);
  return S < 1 ? 1 : S;
}
int grid_skinny_fp4m(const astergemm_config& c, int cus) {
  return krange_grid(c.M > 32 ? 2 : 1, c.N, splits_skinny_fp4m(c), cus).grid;
}

#define AG_SKINNY_FP4M(name, OUT)                                                          \
  Variant {                                                                                \
    name, ASTERGEMM_KERNEL_SKINNY, ASTERGEMM_MXFP4, OUT, 64, 16, 512, 1, 8, 1, 2,           \
        8 * 8192 + 65536, (const void*)gemm_skinny_fp4m_kernel<OUT, 2, 2, 2, 2>,           \
        launch_skinny_fp4m<OUT>, check_skinny_fp4m, ASTERGEMM_OPERAND_LDS,                 \
        splits_skinny_fp4m, grid_skinny_fp4m                                               \
  }

// ---- 16 < M <= 64: the same persistent kernel with two activation tiles per wave --------
//
// A wave still owns a K slice of every row, now for 32 activation rows: MT * SPB * 2 = 128
// operand registers at K = 4096, half of what a wave of an eight-wave workgroup can hold,
// so 32 rows is the limit (64 rows x 8 KB would be the whole register file of the CU).
// Every weight operand read back from the wave's LDS buffer feeds MT MFMAs; the partial
// tiles of a row block are reduced after every block, tile mt by wave mt.
// M > 32 has two forms.  Rows of exactly 8 KiB (and rows of more than 64 KiB): MH = 2, two
// workgroups on the same XCD (block ids 8 apart) take the same weight rows and one half of the
// activation rows each, the second read of a weight line served by that XCD's L2 (bf16 64 x
// 14336 x 4096: 29.5 us).  Other rows take four activation tiles per wave (MT = 4) on K ranges
// of 4 KiB (SPB = 4: the same 128 operand registers): one workgroup covers all 64 rows and
// every weight byte is fetched once and multiplied four times (64 x 14336 x 8192: 52 us
// against 63 for split K on the tile kernel); a 4 KiB row is a single range.  On an 8 KiB row
// that form would pay for a workspace pass the paired form does not need (33.0 against
// 29.5 us).
template <int DT, int OUT, int SPB, int MT, int MH>
__global__ __launch_bounds__(512) void gemm_skinny_regm_kernel(const GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr int KW = 8;
  constexpr int UPB = SPB / 4;                   // units per block
  constexpr int slice = SPB * 128;               // bytes of every row owned by one wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  uint8_t* tbuf = slds + wave * 8192;            // 4 steps x 2 KiB, private to the wave
  constexpr int NBS = MT >= 4 ? 1 : 2;           // blocks between workgroup barriers (NBS * MT <= 8)
  f32x4* red = (f32x4*)(slds + KW * 8192);       // [2][NBS][MT][KW][64]

  // block b runs on XCD b % 8; with MH = 2 blocks b and b + 8 share a row range.
  // Rows longer than the 8 waves' slices are cut into p.split_k K ranges: a workgroup takes
  // one K range of one of p.tiles_n row ranges and leaves fp32 partial sums in the workspace.
  const int q = blockIdx.x >> 3;
  const int half = MH == 2 ? (q & 1) : 0;
  const int idx = MH == 2 ? ((q >> 1) << 3) | (blockIdx.x & 7) : (int)blockIdx.x;
  const int g = p.tiles_n;                       // row ranges
  if (idx >= g * p.split_k) return;
  const int ks = idx / g, rid = idx - ks * g;
  const int64_t koff = (int64_t)ks * (KW * slice);
  // the last K range may end inside the workgroup's span: a wave whose slice lies behind the
  // row's end multiplies zeros (rows are whole slices long, the launcher checks)
  const bool dead = koff + (wave + 1) * slice > (DT == ASTERGEMM_FP8_E4M3 ? p.K : 2 * p.K);
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = rid * per;
  const int m0 = half * MT * 16;                 // first activation row of this workgroup
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nblk = (r1 - r0 + 15) >> 4;
  const int total = nblk * UPB;

  const int lrow = lane >> 3, lpiece = lane & 7;
  const uint8_t* wbase = p.B + koff + wave * slice + lpiece * 16;
  // a unit that is the wave's whole slice of a row (UPB == 1): 2 rows x 512 contiguous bytes per
  // instruction instead of 8 rows x 128 bytes (see gemm_skinny_reg_kernel)
  constexpr bool CONTIG = UPB == 1;
  const int hi = lane >> 5, p32 = lane & 31;
  auto issue = [&](int j, i32x4(&dst)[8]) {      // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    if (dead) {                                    // zeros, so that nothing non-finite gets in
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = i32x4{0, 0, 0, 0};
      return;
    }
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {              // instruction i: rows 2 i and 2 i + 1 of the block
        const int nh = r0 + blk * 16 + 2 * i;
        int n = nh + hi;
        n = n < r1 ? n : r1 - 1;
        const uint8_t* src = p.B + koff + wave * slice + (int64_t)n * p.ldb_bytes + p32 * 16;
        if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
        dst[i] = __builtin_nontemporal_load((const i32x4*)src);
      }
      return;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int nh = r0 + blk * 16 + h * 8;
      int n = nh + lrow;
      n = n < r1 ? n : r1 - 1;
      const uint8_t* src = wbase + (int64_t)n * p.ldb_bytes + t * 512;
      if (j >= total || nh >= r1) src = p.A + lpiece * 16;  // nothing to fetch: a line that stays in L2
#pragma unroll
      for (int s = 0; s < 4; ++s)
        dst[s * 2 + h] = __builtin_nontemporal_load((const i32x4*)(src + s * 128));
    }
  };

  const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);
  const int rd_off = li * 128;
  auto stash = [&](const i32x4(&src)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = src[i];
  };
  const int wr_c = (p32 >> 3) * 2048 + hi * 128;
  const int pch = ((p32 & 7) ^ hi) << 4;
  auto stash_w = [&](const i32x4(&src)[8]) {
    if constexpr (CONTIG) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *(i32x4*)(tbuf + wr_c + (i >> 2) * 1024 + (i & 3) * 256 + (pch ^ ((i & 3) << 5))) = src[i];
    } else {
      stash(src);
    }
  };
  auto operand = [&](int s, int u) {
    return *(const i32x4*)(tbuf + s * 2048 + rd_off + (((4 * u + lq) ^ (li & 7)) << 4));
  };

  // x: MT * UPB units, fetched like the weights (whole lines, through the LDS buffer) but
  // cacheable; two units in flight, behind the first two weight units.
  i32x4 x[MT][SPB * 2];
  auto x_load = [&](int xi, i32x4(&dst)[8]) {    // xi = mt * UPB + t
    const int mt = xi / UPB, t = xi % UPB;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int m = m0 + mt * 16 + h * 8 + lrow;
      m = m < p.M ? m : p.M - 1;
      const uint8_t* src =
          p.A + (int64_t)m * p.lda_bytes + koff + wave * slice + t * 512 + lpiece * 16;
#pragma unroll
      for (int s = 0; s < 4; ++s)
        dst[s * 2 + h] = dead ? i32x4{0, 0, 0, 0} : *(const i32x4*)(src + s * 128);
    }
  };
  i32x4 w0[8], w1[8];
  {
    i32x4 xa[8], xb[8];
    issue(0, w0);
    issue(1, w1);
    __builtin_amdgcn_sched_barrier(0);
    x_load(0, xa);
    x_load(1, xb);
    static_for<0, MT * UPB>([&](auto I) {
      constexpr int xi = decltype(I)::value;
      constexpr int mt = xi / UPB, t = xi % UPB;
      if constexpr (xi % 2 == 0) stash(xa); else stash(xb);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[mt][t * 8 + i] = operand(i >> 1, i & 1);
      if constexpr (xi + 2 < MT * UPB) {
        if constexpr (xi % 2 == 0) x_load(xi + 2, xa); else x_load(xi + 2, xb);
      }
    });
  }
  __builtin_amdgcn_sched_barrier(0);

  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int parity = 0;

  // Partial tiles go to red[parity][block % NBS][mt][wave]; the workgroup meets once per NBS
  // blocks, then wave w sums and stores tile w % MT of block w / MT of the group.
  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      red[(((parity * NBS + slot) * MT + mt) * KW + wave) * 64 + lane] = acc[mt];
      acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave < (slot + 1) * MT) {
      const int rb = wave / MT, rt = wave % MT;
      const f32x4* src = red + (((parity * NBS + rb) * MT + rt) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = m0 + rt * 16 + li, n = r0 + (blk - slot + rb) * 16 + 4 * lq;
      if (m < p.M && n < r1 && p.split_k > 1) {
        // partial sums of this K range: [split][M][N] fp32, finished by the reduce kernel
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        float* o = p.workspace + ((int64_t)ks * p.M + m) * p.N + n;
        if ((p.N & 3) == 0 && ncols == 4) *(f32x4*)o = v;
        else
          for (int r = 0; r < ncols; ++r) o[r] = v[r];
      } else if (m < p.M && n < r1) {
        v *= scale;
        const int ncols = (r1 - n) < 4 ? (r1 - n) : 4;
        if (p.bias)
          for (int r = 0; r < ncols; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, ncols);
      }
    }
    parity ^= 1;
  };

  auto mma = [&](int blk, auto T) {
    constexpr int t = decltype(T)::value;
    if constexpr (DT == ASTERGEMM_FP8_E4M3) {
      // one 16x16x128 MFMA per 128-byte step and activation tile (pieces lq and 4 + lq)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const i32x4 lo = operand(s, 0), hi = operand(s, 1);
        const i32x8 w = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const i32x4 xl = x[mt][t * 8 + 2 * s], xh = x[mt][t * 8 + 2 * s + 1];
          acc[mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              w, i32x8{xl[0], xl[1], xl[2], xl[3], xh[0], xh[1], xh[2], xh[3]}, acc[mt], 0, 0, 0,
              0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const i32x4 w = operand(i >> 1, i & 1);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = sk_mfma<DT>(w, x[mt][t * 8 + i], acc[mt]);
      }
    }
    if (t == UPB - 1) block_end(blk);
  };

  constexpr int TRIP = UPB < 2 ? 2 : UPB;
  int j = 0;
  for (; j + TRIP <= total; j += TRIP) {
    const int blk = j / UPB;
    static_for<0, TRIP / 2>([&](auto I) {
      constexpr int i = decltype(I)::value * 2;
      stash_w(w0);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 2, w0);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + i / UPB, std::integral_constant<int, i % UPB>{});
      __builtin_amdgcn_sched_barrier(0);
      stash_w(w1);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w1);
      __builtin_amdgcn_sched_barrier(0);
      mma(blk + (i + 1) / UPB, std::integral_constant<int, (i + 1) % UPB>{});
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  if (j < total) {  // UPB == 1, odd block count
    stash_w(w0);
    mma(j / UPB, std::integral_constant<int, 0>{});
  }
}

// K ranges for a row of `rb` bytes: rb / 8 KiB when that is whole (one range: the eight
// waves' 1 KiB slices cover the row), else ranges of 4 KiB in 512-byte slices, the last one
// possibly short; 0 when the row is not a whole number of slices or needs over 16 ranges.
__host__ inline int skinny_split_of(int64_t rb, int* spb) {
  if (rb < 4096) return 0;                       // most waves would idle: the generic kernel
  if (rb % 8192 == 0 && rb / 8192 <= 16) return *spb = 8, (int)(rb / 8192);
  if (rb % 512 == 0 && (rb + 4095) / 4096 <= 16) return *spb = 4, (int)((rb + 4095) / 4096);
  return 0;
}

// How the decode kernel of up to 64 rows runs a problem: K ranges, steps per wave and range,
// activation tiles per wave, workgroups per row range.  Shared by the launcher, the workspace
// size and the reported grid.
struct RegmPlan {
  int S = 0, spb = 0, mt = 0, mh = 0;
};
inline RegmPlan regm_plan_of(int64_t M, int64_t rb) {
  RegmPlan r;
  int spb = 0;
  const int S = skinny_split_of(rb, &spb);
  if (S == 0) return r;
  if (M > 32 && rb != 8192 && rb % 512 == 0 && (rb + 4095) / 4096 <= 16) {
    r.S = (int)((rb + 4095) / 4096), r.spb = 4, r.mt = 4, r.mh = 1;
    return r;
  }
  r.S = S, r.spb = spb;
  r.mt = (M <= 16 && S > 1) ? 1 : 2;
  r.mh = M > 32 ? 2 : 1;
  return r;
}

template <int DT, int OUT, int SPB, int MT, int MH>
int launch_skinny_regm_t(const GemmArgs& a0, int S, hipStream_t s) {
  auto k = gemm_skinny_regm_kernel<DT, OUT, SPB, MT, MH>;
  constexpr int lds = 8 * 8192 + 2 * (MT >= 4 ? 1 : 2) * MT * 8 * 64 * 16;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  GemmArgs a = a0;
  const KRangeGrid kg = krange_grid(MH, a.N, S, cus);
  a.tiles_n = kg.rows;
  a.split_k = S;
  if (S > 1 && !a.workspace) {
    if (int rc = splitk_workspace((size_t)S * a.M * a.N * sizeof(float), s, &a.workspace)) return rc;
  }
  AG_LAUNCH_KERNEL(k, dim3(kg.grid), dim3(512), lds, s, a);
  // the partial sums must exist before anything adds them: a failed launch ends here
  if (const hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
  if (S > 1) launch_splitk_reduce<OUT>(a, S, s);
  return (int)hipGetLastError();
}

template <int DT, int OUT>
int launch_skinny_regm(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  const RegmPlan r = regm_plan_of(a.M, row_bytes(DT, a.K));
  if (r.S == 0) return (int)hipErrorInvalidValue;
  if (r.mt == 4) return launch_skinny_regm_t<DT, OUT, 4, 4, 1>(a, r.S, s);
  if (r.mt == 1)
    return r.spb == 8 ? launch_skinny_regm_t<DT, OUT, 8, 1, 1>(a, r.S, s)
                      : launch_skinny_regm_t<DT, OUT, 4, 1, 1>(a, r.S, s);
  if (r.mh == 1)
    return r.spb == 8 ? launch_skinny_regm_t<DT, OUT, 8, 2, 1>(a, r.S, s)
                      : launch_skinny_regm_t<DT, OUT, 4, 2, 1>(a, r.S, s);
  return r.spb == 8 ? launch_skinny_regm_t<DT, OUT, 8, 2, 2>(a, r.S, s)
                    : launch_skinny_regm_t<DT, OUT, 4, 2, 2>(a, r.S, s);
}

const char* check_skinny_regm(const astergemm_config& c) {
  if (c.M > 64) return "resident-activation path needs M <= 64";
  int spb = 0;
  if (skinny_split_of(row_bytes(c.dtype_ab, c.K), &spb) == 0)
    return c.dtype_ab == ASTERGEMM_FP8_E4M3
               ? "resident-activation path for fp8 needs K >= 4096, a multiple of 512, at most 65536 "
                 "(131072 in multiples of 8192)"
               : "resident-activation path needs K >= 2048, a multiple of 256, at most 32768 (65536 in "
                 "multiples of 4096)";
  return nullptr;
}

int splits_skinny_regm(const astergemm_config& c) {
  const RegmPlan r = regm_plan_of(c.M, row_bytes(c.dtype_ab, c.K));
  return r.S < 1 ? 1 : r.S;
}
int grid_skinny_regm(const astergemm_config& c, int cus) {
  const RegmPlan r = regm_plan_of(c.M, row_bytes(c.dtype_ab, c.K));
  return krange_grid(r.mh < 1 ? 1 : r.mh, c.N, r.S < 1 ? 1 : r.S, cus).grid;
}

#define AG_SKINNY_LDSM(name, DT, OUT)                                                      \
  Variant {                                                                                \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 64, 16, 512, 1, 8, 1, 2, 8 * 8192 + 65536,      \
        (const void*)gemm_skinny_regm_kernel<DT, OUT, 8, 2, 2>, launch_skinny_regm<DT, OUT>, \
        check_skinny_regm, ASTERGEMM_OPERAND_LDS, splits_skinny_regm, grid_skinny_regm     \
  }

template <int DT, int OUT>
int launch_skinny_reg(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  switch (row_bytes(DT, a.K)) {  // eight waves x SPB steps of 128 bytes
    case 4096: return launch_skinny_reg_t<DT, OUT, 4>(a, s);
    case 8192: return launch_skinny_reg_t<DT, OUT, 8>(a, s);
    case 16384: return launch_skinny_reg_t<DT, OUT, 16>(a, s);
  }
  return (int)hipErrorInvalidValue;
}

const char* check_skinny_reg(const astergemm_config& c) {
  if (c.M > 16) return "resident-activation path needs M <= 16";
  const int64_t rb = row_bytes(c.dtype_ab, c.K);
  if (rb != 4096 && rb != 8192 && rb != 16384)
    return c.dtype_ab == ASTERGEMM_FP8_E4M3
               ? "resident-activation path needs K = 4096, 8192 or 16384 for fp8"
               : "resident-activation path needs K = 2048, 4096 or 8192";
  return nullptr;
}

#define AG_SKINNY_LDS(name, DT, OUT)                                                       \
  Variant {                                                                                \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 16, 16, 512, 1, 8, 1, 3, 8 * 8192 + 65536,      \
        (const void*)gemm_skinny_reg_kernel<DT, OUT, 8>, launch_skinny_reg<DT, OUT>,       \
        check_skinny_reg                                                                   \
  }

// ---- M <= 16, B pre-shuffled (operand path "direct B") ---------------------------------
//
// B arrives in the order of the reference's shuffle_weight
// (contrib/kittens/test/kittens_helpers.py:90-119): 1 KiB chunks (16 weight rows x 32 K
// elements), chunk (nb, kb) at ((nb * K/32 + kb) * 1024), inside it lane d = 16*g + n holds
// B[16 nb + n][32 kb + 4g .. 4g+3] and B[16 nb + n][32 kb + 16 + 4g .. +3].  A wave's 16-byte
// load per lane of one chunk therefore IS its MFMA operand and is 1 KiB contiguous; the
// eight waves take the chunks of a row block round robin, so a workgroup sweeps its part of B
// front to back.  No LDS transposition; x is gathered once
// into registers in the same K order.  Everything else (persistent grid, N split in
// multiples of 8 rows, two units in flight, reduction through LDS every four row blocks) is
// as in the kernel above.
// CPW = chunks per wave and row block = K / 256.
template <int DT, int OUT, int CPW>
__global__ __launch_bounds__(512) void gemm_skinny_direct_kernel(const GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr int KW = 8;
  constexpr int UPB = CPW / 8;                   // units (8 chunks) per wave and row block
  constexpr int NBS = 4;                         // row blocks between workgroup barriers
  static_assert(CPW % 8 == 0, "whole units");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  f32x4* red = (f32x4*)slds;                     // [2][NBS][KW][64]

  // rows [r0, r1) of the weight matrix belong to this workgroup (multiples of 8: a row
  // block at either end may be half of a 16-row chunk)
  const int g = gridDim.x;
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = blockIdx.x * per;
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nb0 = r0 >> 4;
  const int nblk = ((r1 - 1) >> 4) - nb0 + 1;
  const int total = nblk * UPB;
  const int64_t blk_bytes = (int64_t)(p.K >> 5) * 1024;   // all chunks of one row block

  const uint8_t* wbase = p.B + (int64_t)nb0 * blk_bytes + (int64_t)wave * CPW * 1024 + lane * 16;
  const uint8_t* idle = p.A + lane * 16;  // nothing to fetch: lines that stay in L2
  auto issue = [&](int j, i32x4(&dst)[8]) {      // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    const int n = (nb0 + blk) * 16 + li;
    const bool dead = j >= total || n < r0 || n >= r1;
    const uint8_t* src = dead ? idle : wbase + (int64_t)blk * blk_bytes + t * 8192;
    const int step = dead ? 0 : 1024;            // idle lanes re-read one line of x
#pragma unroll
    for (int u = 0; u < 8; ++u) dst[u] = __builtin_nontemporal_load((const i32x4*)(src + u * step));
  };

  // x operands in the K order of the shuffle: row li, elements 4q..4q+3 and 16+4q..16+4q+3 of
  // every 32-element block of this wave's slice.  Fetched as whole lines (8 rows x 128 bytes
  // per instruction; 8-byte gathers straight from global memory are four times the requests
  // and cost ~4 us at the start of the kernel) and turned around in a wave-private LDS
  // buffer: 128-byte rows, 16-byte granule index XOR (row & 7).
  i32x4 x[CPW];
  {
    uint8_t* tbuf = slds + 2 * NBS * KW * 1024 + wave * 8192;
    const int lrow = lane >> 3, lpiece = lane & 7;
    const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);
    static_for<0, UPB>([&](auto T) {
      constexpr int t = decltype(T)::value;
      i32x4 xw[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int m = h * 8 + lrow;
        m = m < p.M ? m : p.M - 1;
        const uint8_t* src =
            p.A + (int64_t)m * p.lda_bytes + (int64_t)wave * CPW * 64 + t * 512 + lpiece * 16;
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) xw[s2 * 2 + h] = *(const i32x4*)(src + s2 * 128);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = xw[i];
#pragma unroll
      for (int c = 0; c < 8; ++c) {               // chunk c of this unit: line c/2, half c&1
        const uint8_t* row = tbuf + (c >> 1) * 2048 + li * 128 + (lq & 1) * 8;
        const int g_lo = (c & 1) * 4 + (lq >> 1), g_hi = g_lo + 2;
        const i32x2 lo = *(const i32x2*)(row + ((g_lo ^ (li & 7)) << 4));
        const i32x2 hi = *(const i32x2*)(row + ((g_hi ^ (li & 7)) << 4));
        x[t * 8 + c] = i32x4{lo.x, lo.y, hi.x, hi.y};
      }
    });
  }
  __builtin_amdgcn_sched_barrier(0);
  // three register sets: the loaded registers are the MFMA operands themselves, so a set is
  // busy until its MFMAs have issued; with three, two units stay in flight behind the one
  // being multiplied
  i32x4 w0[8], w1[8], w2[8];
  issue(0, w0);
  issue(1, w1);
  issue(2, w2);
  __builtin_amdgcn_sched_barrier(0);

  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  int parity = 0;
  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
    red[((parity * NBS + slot) * KW + wave) * 64 + lane] = acc;
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave <= slot) {
      const f32x4* src = red + ((parity * NBS + wave) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = li, n = (nb0 + blk - slot + wave) * 16 + 4 * lq;
      if (m < p.M && n >= r0 && n < r1) {
        v *= scale;
        if (p.bias)
          for (int r = 0; r < 4; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, 4);
      }
    }
    parity ^= 1;
  };
  // T = unit index inside the row block (compile time: selects the x registers)
  auto mma = [&](int blk, auto T, const i32x4(&src)[8]) {
    constexpr int t = decltype(T)::value;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc = sk_mfma<DT>(src[u], x[t * 8 + u], acc);
    if (t == UPB - 1) block_end(blk);
  };

  // flat steps in groups of lcm(3, UPB) so that register set and x indices are static
  constexpr int TRIP = (UPB % 3 == 0) ? UPB : 3 * UPB;
  auto step = [&](int j, auto IC) {
    constexpr int i = decltype(IC)::value;
    auto body = [&](i32x4(&w)[8]) {
      mma((j + i) / UPB, std::integral_constant<int, i % UPB>{}, w);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w);
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (i % 3 == 0) body(w0);
    else if constexpr (i % 3 == 1) body(w1);
    else body(w2);
  };
  int j = 0;
  for (; j + TRIP <= total; j += TRIP) static_for<0, TRIP>([&](auto IC) { step(j, IC); });
  // remainder: fewer than TRIP steps, j is a multiple of TRIP (so of 3 and of UPB)
  static_for<0, TRIP>([&](auto IC) {
    if (j + decltype(IC)::value < total) step(j, IC);
  });
}

template <int DT, int OUT, int CPW>
int launch_skinny_direct_t(const GemmArgs& a, hipStream_t s) {
  auto k = gemm_skinny_direct_kernel<DT, OUT, CPW>;
  constexpr int lds = 2 * 4 * 8 * 64 * 16 + 8 * 8192;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  const int nblocks = (int)((a.N + 15) / 16);
  const int g = nblocks < cus ? nblocks : cus;
  AG_LAUNCH_KERNEL(k, dim3(g), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

template <int DT, int OUT>
int launch_skinny_direct(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  switch (a.K) {
    case 2048: return launch_skinny_direct_t<DT, OUT, 8>(a, s);
    case 4096: return launch_skinny_direct_t<DT, OUT, 16>(a, s);
    case 8192: return launch_skinny_direct_t<DT, OUT, 32>(a, s);
  }
  return (int)hipErrorInvalidValue;
}

const char* check_skinny_direct(const astergemm_config& c) {
  if (c.M > 16) return "pre-shuffled B is supported for M <= 16";
  if (c.K != 2048 && c.K != 4096 && c.K != 8192)
    return "pre-shuffled B is supported for K = 2048, 4096 or 8192";
  if (c.N % 16 != 0) return "pre-shuffled B needs N % 16 == 0";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  return nullptr;
}

#define AG_SKINNY_DIRECT(name, DT, OUT)                                                     \
  Variant {                                                                                 \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 16, 16, 512, 1, 8, 1, 1, 131072,                \
        (const void*)gemm_skinny_direct_kernel<DT, OUT, 16>, launch_skinny_direct<DT, OUT>, \
        check_skinny_direct, ASTERGEMM_OPERAND_DIRECT_B                                     \
  }

// ---- M <= 16, fp8 or MXFP4 weights pre-shuffled (operand path "direct B") ------------------
//
// The same idea for the one-byte and nibble types, whose MFMA (16x16x128) takes pieces lq and
// 4 + lq of a 128-byte step of a row: B arrives in STEP ORDER (astergemm_shuffle_weight_8),
// row block nb (16 rows), step s, half u in one KiB at ((nb * steps + s) * 2 + u) * 1024, lane
// 16 q + n of a wave finding bytes [(4u + q) * 16, + 16) of row 16 nb + n, step s, at byte
// 16 (16 q + n).  A lane's 16-byte load of a KiB is therefore its operand piece (fp8: the two
// halves of a step are the two halves of one operand; MXFP4: one operand each), a unit of SU
// steps is 2 SU KiB in a row, and a wave's slice of a row block (SPB steps) is contiguous.
// The MXFP4 scale plane arrives in the matching order (astergemm_shuffle_scales_e8m0): the
// 8 e8m0 bytes of row 16 nb + n, step s at (nb * steps + s) * 128 + 8 n, so the scales a wave
// needs for a step are one line.  Activations are plain row-major and go through the wave's
// LDS buffer once, as in gemm_skinny_reg_kernel / gemm_skinny_fp4_kernel; persistent grid, N in
// multiples of 8 rows, three register sets (a loaded register is the operand, so a set is busy
// until its MFMAs have issued), reduction through LDS every four row blocks.
// SPB = steps per wave and row (row bytes / 1024), SU = steps per unit.
template <int DT, int OUT, int SPB, int SU>
__global__ __launch_bounds__(512) void gemm_skinny_directb_kernel(const GemmArgs p) {
  static_assert(DT == ASTERGEMM_FP8_E4M3 || DT == ASTERGEMM_MXFP4, "one-byte and nibble operands");
  extern __shared__ __attribute__((aligned(1024))) uint8_t slds[];
  constexpr bool FP4 = DT == ASTERGEMM_MXFP4;
  constexpr int KW = 8;
  constexpr int UPB = SPB / SU;                  // units per row block
  constexpr int NL = 2 * SU;                     // loads (KiB) per unit
  constexpr int NBS = 4;                         // row blocks between workgroup barriers
  static_assert(SPB % SU == 0, "whole units");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lq = lane >> 4;
  f32x4* red = (f32x4*)slds;                     // [2][NBS][KW][64]
  uint8_t* tbuf = slds + 2 * NBS * KW * 1024 + wave * 8192;  // the activations' way into operand order

  const int g = gridDim.x;
  const int per = (((p.N + g - 1) / g) + 7) & ~7;
  const int r0 = blockIdx.x * per;
  const int r1 = (r0 + per) < p.N ? (r0 + per) : p.N;
  if (r0 >= p.N) return;
  const int nb0 = r0 >> 4;
  const int nblk = ((r1 - 1) >> 4) - nb0 + 1;
  const int total = nblk * UPB;
  const int64_t steps = (int64_t)SPB * KW;       // 128-byte steps of a row
  const int64_t blk_bytes = steps * 2048;        // payload of one row block

  const uint8_t* wbase = p.B + (int64_t)nb0 * blk_bytes + (int64_t)wave * SPB * 2048 + lane * 16;
  const uint8_t* sbase = FP4 ? p.mx_b + ((int64_t)nb0 * steps + wave * SPB) * 128 + li * 8 : nullptr;
  const uint8_t* idle = p.A + lane * 16;         // nothing to fetch: lines that stay in L2
  auto issue = [&](int j, i32x4(&dst)[NL], i32x2(&sc)[SU]) {  // flat index j = block * UPB + t
    int blk = j / UPB;
    const int t = j % UPB;
    blk = blk < nblk ? blk : nblk - 1;
    const int n = (nb0 + blk) * 16 + li;
    const bool dead = j >= total || n < r0 || n >= r1;
    const uint8_t* src = dead ? idle : wbase + (int64_t)blk * blk_bytes + t * (NL * 1024);
    const int step = dead ? 0 : 1024;            // idle lanes re-read one line of x
#pragma unroll
    for (int u = 0; u < NL; ++u) dst[u] = __builtin_nontemporal_load((const i32x4*)(src + u * step));
    if constexpr (FP4) {
      // scale bytes of a row of the block exist even where the row belongs to a neighbour
      const uint8_t* ssrc = sbase + ((int64_t)blk * steps + t * SU) * 128;
#pragma unroll
      for (int s2 = 0; s2 < SU; ++s2) sc[s2] = *(const i32x2*)(ssrc + s2 * 128);
    }
  };

  // x (and its scales): operand registers for the SPB * 2 pieces of a row block, fetched as
  // whole lines and turned around in the wave's LDS buffer
  i32x4 x[SPB * 2];
  int xs[FP4 ? SPB * 2 : 1];
  {
    const int lrow = lane >> 3, lpiece = lane & 7;
    const int wr_off = lrow * 128 + ((lpiece ^ lrow) << 4);
    if constexpr (FP4) {
      const int m = li < p.M ? li : p.M - 1;
      const uint8_t* xsrc = p.mx_a + (int64_t)m * p.mx_ld + wave * (SPB * 8);
#pragma unroll
      for (int s2 = 0; s2 < SPB; ++s2) {
        const i32x2 v = *(const i32x2*)(xsrc + s2 * 8);
        xs[s2 * 2] = (int)((unsigned)v[0] >> (8 * lq));
        xs[s2 * 2 + 1] = (int)((unsigned)v[1] >> (8 * lq));
      }
    }
    static_for<0, UPB>([&](auto T) {
      constexpr int t = decltype(T)::value;
      i32x4 xw[NL];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int m = h * 8 + lrow;
        m = m < p.M ? m : p.M - 1;
        const uint8_t* src =
            p.A + (int64_t)m * p.lda_bytes + (int64_t)wave * SPB * 128 + t * (SU * 128) + lpiece * 16;
#pragma unroll
        for (int s2 = 0; s2 < SU; ++s2) xw[s2 * 2 + h] = *(const i32x4*)(src + s2 * 128);
      }
#pragma unroll
      for (int i = 0; i < NL; ++i)
        *(i32x4*)(tbuf + (i >> 1) * 2048 + (i & 1) * 1024 + wr_off) = xw[i];
#pragma unroll
      for (int i = 0; i < NL; ++i)               // piece 4u + lq of step s: i = 2 s + u
        x[t * NL + i] = *(const i32x4*)(tbuf + (i >> 1) * 2048 + li * 128 +
                                        (((4 * (i & 1) + lq) ^ (li & 7)) << 4));
    });
  }
  __builtin_amdgcn_sched_barrier(0);
  i32x4 w0[NL], w1[NL], w2[NL];
  i32x2 s0[SU], s1[SU], s2r[SU];
  issue(0, w0, s0);
  issue(1, w1, s1);
  issue(2, w2, s2r);
  __builtin_amdgcn_sched_barrier(0);

  float scale = 1.0f;
  if (p.scale_a) scale *= *p.scale_a;
  if (p.scale_b) scale *= *p.scale_b;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  int parity = 0;
  auto block_end = [&](int blk) {
    const int slot = blk & (NBS - 1);
    red[((parity * NBS + slot) * KW + wave) * 64 + lane] = acc;
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (slot != NBS - 1 && blk != nblk - 1) return;
    __syncthreads();
    if (wave <= slot) {
      const f32x4* src = red + ((parity * NBS + wave) * KW) * 64 + lane;
      f32x4 v = src[0];
#pragma unroll
      for (int k = 1; k < KW; ++k) v += src[k * 64];
      const int m = li, n = (nb0 + blk - slot + wave) * 16 + 4 * lq;
      if (m < p.M && n >= r0 && n < r1) {
        v *= scale;
        if (p.bias)
          for (int r = 0; r < 4; ++r) v[r] += p.bias[n + r];
        sk_store_row4<OUT>(p.C, p.ldc, m, n, v, 4);
      }
    }
    parity ^= 1;
  };
  // T = unit index inside the row block (compile time: selects the x registers)
  auto mma = [&](int blk, auto T, const i32x4(&w)[NL], const i32x2(&sc)[SU]) {
    constexpr int t = decltype(T)::value;
    if constexpr (FP4) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {             // i = 2 s + u: scale byte 4u + lq of step s
        const int ws = (int)((unsigned)sc[i >> 1][i & 1] >> (8 * lq));
        const i32x4 xv = x[t * NL + i];
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8{w[i][0], w[i][1], w[i][2], w[i][3], 0, 0, 0, 0},
            i32x8{xv[0], xv[1], xv[2], xv[3], 0, 0, 0, 0}, acc, 4, 4, 0, ws, 0, xs[t * NL + i]);
      }
    } else {
#pragma unroll
      for (int s2 = 0; s2 < SU; ++s2) {
        const i32x4 lo = w[2 * s2], hi = w[2 * s2 + 1];
        const i32x4 xl = x[t * NL + 2 * s2], xh = x[t * NL + 2 * s2 + 1];
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]},
            i32x8{xl[0], xl[1], xl[2], xl[3], xh[0], xh[1], xh[2], xh[3]}, acc, 0, 0, 0, 0, 0, 0);
      }
    }
    if (t == UPB - 1) block_end(blk);
  };

  // flat steps in groups of lcm(3, UPB) so that register set and x indices are static
  constexpr int TRIP = (UPB % 3 == 0) ? UPB : 3 * UPB;
  auto step = [&](int j, auto IC) {
    constexpr int i = decltype(IC)::value;
    auto body = [&](i32x4(&w)[NL], i32x2(&sc)[SU]) {
      mma((j + i) / UPB, std::integral_constant<int, i % UPB>{}, w, sc);
      __builtin_amdgcn_sched_barrier(0);
      issue(j + i + 3, w, sc);
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (i % 3 == 0) body(w0, s0);
    else if constexpr (i % 3 == 1) body(w1, s1);
    else body(w2, s2r);
  };
  int j = 0;
  for (; j + TRIP <= total; j += TRIP) static_for<0, TRIP>([&](auto IC) { step(j, IC); });
  // remainder: fewer than TRIP steps, j is a multiple of TRIP (so of 3 and of UPB)
  static_for<0, TRIP>([&](auto IC) {
    if (j + decltype(IC)::value < total) step(j, IC);
  });
}

template <int DT, int OUT, int SPB, int SU>
int launch_skinny_directb_t(const GemmArgs& a, hipStream_t s) {
  auto k = gemm_skinny_directb_kernel<DT, OUT, SPB, SU>;
  constexpr int lds = 2 * 4 * 8 * 64 * 16 + 8 * 8192;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  // what the kernel's indexing assumes: whole row blocks, packed rows of SPB * 8 steps
  if (a.N % 16 != 0 || row_bytes(DT, a.K) != (int64_t)SPB * 1024 || a.ldb_bytes != row_bytes(DT, a.K))
    return (int)hipErrorInvalidValue;
  if (DT == ASTERGEMM_MXFP4 && (((uintptr_t)a.mx_b | (uintptr_t)a.mx_a) & 7) != 0)
    return (int)hipErrorInvalidValue;
  const int nblocks = (int)(a.N / 16);
  const int g = nblocks < cus ? nblocks : cus;
  AG_LAUNCH_KERNEL(k, dim3(g), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

template <int DT, int OUT>
int launch_skinny_directb(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  switch (row_bytes(DT, a.K)) {
    case 2048: return launch_skinny_directb_t<DT, OUT, 2, 2>(a, s);
    case 4096: return launch_skinny_directb_t<DT, OUT, 4, 4>(a, s);
    case 8192: return launch_skinny_directb_t<DT, OUT, 8, 4>(a, s);
  }  // 16 KiB rows: 128 activation registers next to three weight sets do not allocate
  return (int)hipErrorInvalidValue;
}

const char* check_skinny_directb(const astergemm_config& c) {
  if (c.M > 16) return "pre-shuffled B is supported for M <= 16";
  const int64_t rb = row_bytes(c.dtype_ab, c.K);
  if (rb != 2048 && rb != 4096 && rb != 8192)
    return c.dtype_ab == ASTERGEMM_MXFP4 ? "pre-shuffled MXFP4 B is supported for K = 4096, 8192 or 16384"
                                          : "pre-shuffled fp8 B is supported for K = 2048, 4096 or 8192";
  if (c.N % 16 != 0) return "pre-shuffled B needs N % 16 == 0";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  return nullptr;
}

#define AG_SKINNY_DIRECTB(name, DT, OUT)                                                      \
  Variant {                                                                                   \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 16, 16, 512, 1, 8, 1, 1, 131072,                  \
        (const void*)gemm_skinny_directb_kernel<DT, OUT, 4, 4>, launch_skinny_directb<DT, OUT>, \
        check_skinny_directb, ASTERGEMM_OPERAND_DIRECT_B                                      \
  }

template <int DT, int OUT, int MT, int NB, int KW, int U>
int launch_skinny(const GemmArgs& a, int grid, hipStream_t s) {
  AG_LAUNCH_KERNEL((gemm_skinny_kernel<DT, OUT, MT, NB, KW, U>), dim3(grid), dim3(KW * 64), 0,
                     s, a);
  return (int)hipGetLastError();
}

const char* check_skinny(const astergemm_config& c) {
  if (c.K % 32 != 0) return "skinny path needs K % 32 == 0";
  if (c.M > 64) return "skinny path needs M <= 64";
  return nullptr;
}

// tile_m = 16*MT (rows of A covered), tile_n = 16*NB, waves_n = KW (K split).
#define AG_SKINNY(name, DT, OUT, MT, NB, KW, U)                                           \
  Variant {                                                                               \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 16 * MT, 16 * NB, 64 * U, 1, KW, 1, 0,        \
        KW * MT * NB * 1024, (const void*)gemm_skinny_kernel<DT, OUT, MT, NB, KW, U>,      \
        launch_skinny<DT, OUT, MT, NB, KW, U>, check_skinny                               \
  }

#define AG_SKINNY_SET(prefix, DT, OUTN, OUT)                                      \
  AG_SKINNY(prefix "_m16_" OUTN, DT, OUT, 1, 1, 4, 8),                            \
      AG_SKINNY(prefix "_m32_" OUTN, DT, OUT, 2, 1, 4, 8),                        \
      AG_SKINNY(prefix "_m64_" OUTN, DT, OUT, 4, 1, 4, 4)

// Wider variants for M = 17..64: a workgroup covers 64 weight rows, so the activations
// are re-read from L2 once per 64 rows instead of once per 16 (at M = 64 the activation
// traffic of the narrow variant is four times the weight traffic).  rank 1: preferred.
#define AG_SKINNY_WIDE(name, DT, OUT, MT, NB, KW, U)                                      \
  Variant {                                                                               \
    name, ASTERGEMM_KERNEL_SKINNY, DT, OUT, 16 * MT, 16 * NB, 64 * U, 1, KW, 1, 1,        \
        KW * MT * NB * 1024, (const void*)gemm_skinny_kernel<DT, OUT, MT, NB, KW, U>,      \
        launch_skinny<DT, OUT, MT, NB, KW, U>, check_skinny                               \
  }
#define AG_SKINNY_WIDE_SET(prefix, DT, OUTN, OUT)                                 \
  AG_SKINNY_WIDE(prefix "_m32n64_" OUTN, DT, OUT, 2, 4, 4, 2),                    \
      AG_SKINNY_WIDE(prefix "_m64n64_" OUTN, DT, OUT, 4, 4, 4, 1)

const Variant kSkinnyVariants[] = {
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "f32", ASTERGEMM_F32),
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "f16", ASTERGEMM_F16),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "f32", ASTERGEMM_F32),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "f16", ASTERGEMM_F16),
    AG_SKINNY_WIDE_SET("skinny_bf16", ASTERGEMM_BF16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_WIDE_SET("skinny_bf16", ASTERGEMM_BF16, "f32", ASTERGEMM_F32),
    AG_SKINNY_WIDE_SET("skinny_bf16", ASTERGEMM_BF16, "f16", ASTERGEMM_F16),
    AG_SKINNY_WIDE_SET("skinny_f16", ASTERGEMM_F16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_WIDE_SET("skinny_f16", ASTERGEMM_F16, "f32", ASTERGEMM_F32),
    AG_SKINNY_WIDE_SET("skinny_f16", ASTERGEMM_F16, "f16", ASTERGEMM_F16),
    AG_SKINNY_LDS("skinnyx_bf16_m16_bf16", ASTERGEMM_BF16, ASTERGEMM_BF16),
    AG_SKINNY_LDS("skinnyx_bf16_m16_f32", ASTERGEMM_BF16, ASTERGEMM_F32),
    AG_SKINNY_LDS("skinnyx_bf16_m16_f16", ASTERGEMM_BF16, ASTERGEMM_F16),
    AG_SKINNY_LDS("skinnyx_f16_m16_bf16", ASTERGEMM_F16, ASTERGEMM_BF16),
    AG_SKINNY_LDS("skinnyx_f16_m16_f32", ASTERGEMM_F16, ASTERGEMM_F32),
    AG_SKINNY_LDS("skinnyx_f16_m16_f16", ASTERGEMM_F16, ASTERGEMM_F16),
    AG_SKINNY_LDSM("skinnyx_bf16_m64_bf16", ASTERGEMM_BF16, ASTERGEMM_BF16),
    AG_SKINNY_LDSM("skinnyx_bf16_m64_f32", ASTERGEMM_BF16, ASTERGEMM_F32),
    AG_SKINNY_LDSM("skinnyx_bf16_m64_f16", ASTERGEMM_BF16, ASTERGEMM_F16),
    AG_SKINNY_LDSM("skinnyx_f16_m64_bf16", ASTERGEMM_F16, ASTERGEMM_BF16),
    AG_SKINNY_LDSM("skinnyx_f16_m64_f32", ASTERGEMM_F16, ASTERGEMM_F32),
    AG_SKINNY_LDSM("skinnyx_f16_m64_f16", ASTERGEMM_F16, ASTERGEMM_F16),
    AG_SKINNY_LDSM("skinnyx_fp8_m64_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_SKINNY_LDSM("skinnyx_fp8_m64_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_SKINNY_LDSM("skinnyx_fp8_m64_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_SKINNY_LDS("skinnyx_fp8_m16_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_SKINNY_LDS("skinnyx_fp8_m16_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_SKINNY_LDS("skinnyx_fp8_m16_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_SKINNY_FP4M("skinnyx_mxfp4_m64_bf16", ASTERGEMM_BF16),
    AG_SKINNY_FP4M("skinnyx_mxfp4_m64_f32", ASTERGEMM_F32),
    AG_SKINNY_FP4M("skinnyx_mxfp4_m64_f16", ASTERGEMM_F16),
    AG_SKINNY_FP4("skinnyx_mxfp4_m16_bf16", ASTERGEMM_BF16),
    AG_SKINNY_FP4("skinnyx_mxfp4_m16_f32", ASTERGEMM_F32),
    AG_SKINNY_FP4("skinnyx_mxfp4_m16_f16", ASTERGEMM_F16),
    AG_SKINNY_DIRECT("skinnyd_bf16_m16_bf16", ASTERGEMM_BF16, ASTERGEMM_BF16),
    AG_SKINNY_DIRECT("skinnyd_bf16_m16_f32", ASTERGEMM_BF16, ASTERGEMM_F32),
    AG_SKINNY_DIRECT("skinnyd_bf16_m16_f16", ASTERGEMM_BF16, ASTERGEMM_F16),
    AG_SKINNY_DIRECT("skinnyd_f16_m16_bf16", ASTERGEMM_F16, ASTERGEMM_BF16),
    AG_SKINNY_DIRECT("skinnyd_f16_m16_f32", ASTERGEMM_F16, ASTERGEMM_F32),
    AG_SKINNY_DIRECT("skinnyd_f16_m16_f16", ASTERGEMM_F16, ASTERGEMM_F16),
    AG_SKINNY_DIRECTB("skinnyd_fp8_m16_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_SKINNY_DIRECTB("skinnyd_fp8_m16_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_SKINNY_DIRECTB("skinnyd_fp8_m16_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_SKINNY_DIRECTB("skinnyd_mxfp4_m16_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_SKINNY_DIRECTB("skinnyd_mxfp4_m16_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_SKINNY_DIRECTB("skinnyd_mxfp4_m16_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
};

}  // namespace

int num_skinny_variants() {
  return (int)(sizeof(kSkinnyVariants) / sizeof(kSkinnyVariants[0]));
}
const Variant* skinny_variants() { return kSkinnyVariants; }

int splitk_workspace_for(size_t bytes, hipStream_t stream, float** out) {
  return splitk_workspace(bytes, stream, out);
}

void splitk_workspace_release(hipStream_t stream) { splitk_workspace_drop(stream); }

int splitk_reduce(int out_dtype, const GemmArgs& a, int splits, hipStream_t stream) {
  switch (out_dtype) {
    case ASTERGEMM_F32: launch_splitk_reduce<ASTERGEMM_F32>(a, splits, stream); break;
    case ASTERGEMM_BF16: launch_splitk_reduce<ASTERGEMM_BF16>(a, splits, stream); break;
    case ASTERGEMM_F16: launch_splitk_reduce<ASTERGEMM_F16>(a, splits, stream); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

}  // namespace astergemm
