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
#include "astergemm_internal.h"

namespace astergemm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned short sk_f32_to_bf16(float f) {
  unsigned u = __builtin_bit_cast(unsigned, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
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
  const bool vec_ok = (p.ldc & 3) == 0;
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
    const int64_t idx = (int64_t)m * p.ldc + n;
    if constexpr (OUT == ASTERGEMM_F32) {
      float* o = (float*)p.C + idx;
      if (vec_ok && ncols == 4) *(f32x4*)o = v;
      else
        for (int r = 0; r < ncols; ++r) o[r] = v[r];
    } else {
      unsigned short h[4];
      for (int r = 0; r < 4; ++r) {
        if constexpr (OUT == ASTERGEMM_BF16) h[r] = sk_f32_to_bf16(v[r]);
        else {
          _Float16 hh = (_Float16)v[r];
          h[r] = __builtin_bit_cast(unsigned short, hh);
        }
      }
      unsigned short* o = (unsigned short*)p.C + idx;
      if (vec_ok && ncols == 4) *(u16x4*)o = u16x4{h[0], h[1], h[2], h[3]};
      else
        for (int r = 0; r < ncols; ++r) o[r] = h[r];
    }
  }
}

template <int DT, int OUT, int MT, int NB, int KW, int U>
int launch_skinny(const GemmArgs& a, int grid, hipStream_t s) {
  hipLaunchKernelGGL((gemm_skinny_kernel<DT, OUT, MT, NB, KW, U>), dim3(grid), dim3(KW * 64), 0,
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

const Variant kSkinnyVariants[] = {
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "f32", ASTERGEMM_F32),
    AG_SKINNY_SET("skinny_bf16", ASTERGEMM_BF16, "f16", ASTERGEMM_F16),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "bf16", ASTERGEMM_BF16),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "f32", ASTERGEMM_F32),
    AG_SKINNY_SET("skinny_f16", ASTERGEMM_F16, "f16", ASTERGEMM_F16),
};

}  // namespace

int num_skinny_variants() {
  return (int)(sizeof(kSkinnyVariants) / sizeof(kSkinnyVariants[0]));
}
const Variant* skinny_variants() { return kSkinnyVariants; }

}  // namespace astergemm
