// Operand quantisers for the fp8 and MXFP4 GEMM paths: fp32 / bf16 / f16 -> OCP e4m3 with a
// per-tensor absmax scale, and -> MXFP4 (e2m1 nibbles + one e8m0 byte per 32 elements).
//
// These produce, on the device, exactly the bytes the GEMM kernels consume (operand
// layouts of astergemm_config: row-major, e2m1 low nibble first, scales [rows, K/32]).
// The e4m3 rounding follows the converter the reference's tests hold
// (f32_to_fp8_e4m3(val, fnuz=False), test/integration/test_conversion_pack_e2e.py:91-167:
// bias 7, round to nearest even with carry into the exponent, saturation to 0x7E = 448,
// NaN and infinities to S|0x7F, signed zero), with the subnormal range rounded to nearest
// even as the hardware converter does.  The MX block format is the one the scaled MFMA
// expects (v_mfma_scale_f32_16x16x128_f8f6f4, e8m0 scale per 32 K-elements).
// Both are HBM-bound byte work: one pass over the source (two for the per-tensor scale).
#include <type_traits>

#include "astergemm_internal.h"

namespace astergemm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
// Vector elements are passed by value (__float_as_uint) before their bits are taken: a bit
// cast applied to the element expression itself read element 0 for every index.

// fp32 -> e4m3 code, round to nearest even, saturating: |x| > 448 -> 0x7E, NaN / inf -> 0x7F.
// Normal range (|x| >= 2^-6): round the fp32 bit pattern to 3 fraction bits in integer
// arithmetic (a carry out of the fraction flows into the exponent) and re-bias 127 -> 7.
// Below that the codes are multiples of 2^-9: adding 2^14 makes the fp32 adder round |x| to
// that grid, ties to even, and leaves the code in the low bits of the sum.
__device__ __forceinline__ unsigned e4m3_rne_sat(float x) {
  const unsigned b = __float_as_uint(x);
  const unsigned s = (b >> 24) & 0x80u;
  const unsigned m = b & 0x7FFFFFFFu;
  unsigned code;
  if (m >= 0x3C800000u) {  // 2^-6
    code = ((m + 0x7FFFFu + ((m >> 20) & 1u)) >> 20) - ((127u - 7u) << 3);
    code = code > 0x7Eu ? 0x7Eu : code;
    code = m >= 0x7F800000u ? 0x7Fu : code;
  } else {
    code = __float_as_uint(__uint_as_float(m) + 16384.0f) & 0xFu;
  }
  return s | code;
}

// fp32 -> e2m1 code (0..15): nearest value of {0, .5, 1, 1.5, 2, 3, 4, 6}, ties to the code
// with an even index, saturation to 6, NaN -> S|7.  Same two tricks: one fraction bit kept
// for |x| >= 1, the grid of 0.5 below (2^22 has an ulp of 0.5).
__device__ __forceinline__ unsigned e2m1_rne_sat(float x) {
  const unsigned b = __float_as_uint(x);
  const unsigned s = (b >> 28) & 0x8u;
  const unsigned m = b & 0x7FFFFFFFu;
  unsigned code;
  if (m >= 0x3F800000u) {  // 1.0
    code = ((m + 0x1FFFFFu + ((m >> 22) & 1u)) >> 22) - ((127u - 1u) << 1);
    code = code > 7u ? 7u : code;
  } else {
    code = __float_as_uint(__uint_as_float(m) + 4194304.0f) & 0x3u;
  }
  return s | code;
}

__global__ void zero_u32_kernel(unsigned* p) { *p = 0u; }

// Source element types: fp32, or the 16-bit types a GEMM of this library writes (both widen
// to fp32 exactly, so quantising them equals quantising the widened values).
template <int SRC>
struct Src {
  static constexpr int kBytes = SRC == ASTERGEMM_F32 ? 4 : 2;
};
template <int SRC>
__device__ __forceinline__ float widen(unsigned short h) {
  if constexpr (SRC == ASTERGEMM_BF16) return __uint_as_float((unsigned)h << 16);
  else return (float)__builtin_bit_cast(_Float16, h);
}
// four consecutive elements (16 or 8 bytes, naturally aligned) as fp32
template <int SRC>
__device__ __forceinline__ f32x4 load4(const void* base, int64_t group) {
  if constexpr (SRC == ASTERGEMM_F32) {
    return __builtin_nontemporal_load((const f32x4*)base + group);
  } else {
    typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
    const u16x4 h = __builtin_nontemporal_load((const u16x4*)base + group);
    return f32x4{widen<SRC>(h[0]), widen<SRC>(h[1]), widen<SRC>(h[2]), widen<SRC>(h[3])};
  }
}
template <int SRC>
__device__ __forceinline__ float load1(const void* base, int64_t i) {
  if constexpr (SRC == ASTERGEMM_F32) return ((const float*)base)[i];
  else return widen<SRC>(((const unsigned short*)base)[i]);
}

// max over |x| as unsigned bits (non-negative floats order like their bit patterns; NaNs
// compare above infinity and so survive the maximum, as they do in numpy's max).  Four
// independent loads per trip; one atomic per workgroup.
template <int SRC>
__global__ __launch_bounds__(256) void absmax_kernel(const void* __restrict__ src, int64_t n,
                                                     unsigned* __restrict__ out) {
  __shared__ unsigned wave_max[4];
  unsigned m = 0;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t n4 = n >> 2;
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  auto fold = [&](const f32x4 v) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned b = __float_as_uint(v[e]) & 0x7FFFFFFFu;
      m = b > m ? b : m;
    }
  };
  for (; i + 3 * stride < n4; i += 4 * stride) {
    const f32x4 v0 = load4<SRC>(src, i);
    const f32x4 v1 = load4<SRC>(src, i + stride);
    const f32x4 v2 = load4<SRC>(src, i + 2 * stride);
    const f32x4 v3 = load4<SRC>(src, i + 3 * stride);
    fold(v0), fold(v1), fold(v2), fold(v3);
  }
  for (; i < n4; i += stride) fold(load4<SRC>(src, i));
  for (int64_t j = (n4 << 2) + blockIdx.x * (int64_t)blockDim.x + threadIdx.x; j < n; j += stride) {
    const unsigned b = __float_as_uint(load1<SRC>(src, j)) & 0x7FFFFFFFu;
    m = b > m ? b : m;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned o = (unsigned)__shfl_xor((int)m, off, 64);
    m = o > m ? o : m;
  }
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) m = wave_max[w] > m ? wave_max[w] : m;
    if (m != 0) atomicMax(out, m);
  }
}

// scale = absmax / 448 in fp32, 1.0 when absmax is zero (or NaN)
__global__ void fp8_scale_kernel(const unsigned* amax_bits, float* scale) {
  const float a = __builtin_bit_cast(float, *amax_bits);
  *scale = (a > 0.0f) ? a / 448.0f : 1.0f;
}

template <int SRC>
__global__ __launch_bounds__(256) void quantize_fp8_kernel(const void* __restrict__ src, int64_t n,
                                                           const float* __restrict__ scale,
                                                           uint8_t* __restrict__ dst) {
  const float s = *scale;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t n4 = n >> 2;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += stride) {
    const f32x4 v = load4<SRC>(src, i);
    unsigned w = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) w |= e4m3_rne_sat(v[e] / s) << (8 * e);
    ((unsigned*)dst)[i] = w;
  }
  for (int64_t i = (n4 << 2) + blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (uint8_t)e4m3_rne_sat(load1<SRC>(src, i) / s);
}

// Eight lanes per 32-element block: a lane loads 16 bytes (4 elements), so one wave-wide load
// covers 1 KB of contiguous source (8 blocks); four such loads are in flight per trip.  The
// block maximum goes round the 8 lanes with three exchanges; every lane then encodes its 4
// elements (2 bytes out) and lane 0 of the group writes the scale byte.  CONTIG: ld == K, so
// block t sits at element 32 t and no (row, column) split is needed.
// LANES: the scale byte of block c of row r goes where astergemm_shuffle_scales_e8m0_lanes128 puts
// it (groups of 128 rows, one KiB per group and 8-block step).
template <int SRC, bool CONTIG, bool LANES = false>
__global__ __launch_bounds__(256) void quantize_mxfp4_kernel(const void* __restrict__ src,
                                                             int64_t nblocks, unsigned bpr,
                                                             int64_t ld,
                                                             uint8_t* __restrict__ packed,
                                                             uint8_t* __restrict__ scales) {
  constexpr int U = 4;
  const int lane = threadIdx.x & 63, g = lane >> 3, l8 = lane & 7;
  const int64_t nwaves = (int64_t)gridDim.x * 4;
  for (int64_t base = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (8 * U); base < nblocks;
       base += nwaves * (8 * U)) {
    f32x4 v[U];
    int64_t t[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      t[u] = base + u * 8 + g;
      live[u] = t[u] < nblocks;
      if (!live[u]) t[u] = nblocks - 1;  // stay inside the source; nothing is stored
      int64_t off;
      if (CONTIG) {
        off = t[u] * 32;
      } else {
        const unsigned r = (unsigned)t[u] / bpr, c = (unsigned)t[u] - r * bpr;
        off = (int64_t)r * ld + (int64_t)c * 32;
      }
      v[u] = load4<SRC>((const uint8_t*)src + off * Src<SRC>::kBytes, l8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      unsigned mb = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned b = __float_as_uint(v[u][e]) & 0x7FFFFFFFu;
        mb = b > mb ? b : mb;
      }
#pragma unroll
      for (int off = 1; off < 8; off <<= 1) {
        const unsigned o = (unsigned)__shfl_xor((int)mb, off, 64);
        mb = o > mb ? o : mb;
      }
      // shared exponent = floor(log2(absmax)) - 2; an all-zero block gets exponent 0, a block
      // holding NaN / inf gets scale byte 0xFF and its elements are scaled by 2^2
      const bool bad = mb >= 0x7F800000u;
      int fl;
      if (mb == 0 || bad) fl = bad ? 0 : 2;                    // -> shared 0 (zero) / -2 (bad)
      else if (mb >= 0x00800000u) fl = (int)(mb >> 23) - 127;  // normal
      else fl = -149 + (31 - __builtin_clz(mb));               // fp32 subnormal
      int sbyte = (fl - 2) + 127;
      sbyte = sbyte < 0 ? 0 : (sbyte > 254 ? 254 : sbyte);
      const int shift = -(sbyte - 127);
      unsigned w = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // exact scaling by a power of two in two steps (|shift| can exceed the fp32 exponent
        // range of a single factor)
        const float q = ldexpf(ldexpf(v[u][e], shift / 2), shift - shift / 2);
        w |= e2m1_rne_sat(q) << (4 * e);
      }
      if (live[u]) {
        *(unsigned short*)(packed + t[u] * 16 + l8 * 2) = (unsigned short)w;
        if (l8 == 0) {
          int64_t so = t[u];
          if constexpr (LANES) {
            const unsigned r = (unsigned)t[u] / bpr, c = (unsigned)t[u] - r * bpr;
            // (group, step, q, i, tile, h): block c = 8 step + 4 h + q, row r = 128 group + 16 tile + i
            so = ((int64_t)(r >> 7) * (bpr >> 3) + (c >> 3)) * 1024 +
                 (((c & 3) * 16 + (r & 15)) * 16 + ((r >> 4) & 7) * 2 + ((c >> 2) & 1));
          }
          scales[so] = bad ? (uint8_t)0xFF : (uint8_t)sbyte;
        }
      }
    }
  }
}

// workgroups of 256 threads for `work_items` thread-items, at most 8 per compute unit
int blocks_for(int64_t work_items) {
  const int64_t b = (work_items + 255) / 256, cap = 256 * 8;
  return (int)(b < 1 ? 1 : (b > cap ? cap : b));
}

}  // namespace
}  // namespace astergemm

using namespace astergemm;

namespace {
bool src_ok(int dt) { return dt == ASTERGEMM_F32 || dt == ASTERGEMM_BF16 || dt == ASTERGEMM_F16; }

// Calls f with the source type as a compile-time constant.
template <class F>
void with_src(int dt, F&& f) {
  switch (dt) {
    case ASTERGEMM_F32: f(std::integral_constant<int, ASTERGEMM_F32>{}); break;
    case ASTERGEMM_BF16: f(std::integral_constant<int, ASTERGEMM_BF16>{}); break;
    default: f(std::integral_constant<int, ASTERGEMM_F16>{}); break;
  }
}
}  // namespace

extern "C" int astergemm_absmax(const void* dSrc, int src_dtype, int64_t n, float* dAbsmax,
                                void* stream) {
  if ((!dSrc && n > 0) || !dAbsmax || n < 0 || (((uintptr_t)dSrc) & 15) || !src_ok(src_dtype)) {
    set_error("astergemm_absmax: bad argument (source F32, BF16 or F16, 16-byte aligned)");
    return ASTERGEMM_EINVAL;
  }
  hipStream_t s = (hipStream_t)stream;
  (void)hipGetLastError();  // only this call's launches are reported below
  hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(1), 0, s, (unsigned*)dAbsmax);
  if (n > 0)
    with_src(src_dtype, [&](auto T) {
      hipLaunchKernelGGL(absmax_kernel<decltype(T)::value>, dim3(blocks_for(n / 4 + 1)), dim3(256),
                         0, s, dSrc, n, (unsigned*)dAbsmax);
    });
  AG_HIP(hipGetLastError());
  return 0;
}

extern "C" int astergemm_quantize_fp8_tensor(const void* dSrc, int src_dtype, int64_t n,
                                             uint8_t* dDst, float* dScale, void* stream) {
  if ((!dSrc && n > 0) || (!dDst && n > 0) || !dScale || n < 0 || (((uintptr_t)dSrc) & 15) ||
      (((uintptr_t)dDst) & 3) || !src_ok(src_dtype)) {
    set_error("astergemm_quantize_fp8_tensor: bad argument (source F32, BF16 or F16, 16-byte "
              "aligned; dDst 4-byte aligned)");
    return ASTERGEMM_EINVAL;
  }
  hipStream_t s = (hipStream_t)stream;
  // dScale doubles as the absmax accumulator: bits of a non-negative float
  if (int rc = astergemm_absmax(dSrc, src_dtype, n, dScale, stream)) return rc;
  hipLaunchKernelGGL(fp8_scale_kernel, dim3(1), dim3(1), 0, s, (const unsigned*)dScale, dScale);
  if (n > 0)
    with_src(src_dtype, [&](auto T) {
      hipLaunchKernelGGL(quantize_fp8_kernel<decltype(T)::value>, dim3(blocks_for(n / 4 + 1)),
                         dim3(256), 0, s, dSrc, n, dScale, dDst);
    });
  AG_HIP(hipGetLastError());
  return 0;
}

extern "C" int astergemm_quantize_mxfp4_ex(const void* dSrc, int src_dtype, int64_t rows, int64_t K,
                                           int64_t ld_src, uint8_t* dPacked, uint8_t* dScales,
                                           int scales_layout, void* stream) {
  if (ld_src == 0) ld_src = K;
  const bool lanes = scales_layout == ASTERGEMM_MX_LANES128;
  if (rows < 0 || K < 0 || K % 32 != 0 || ld_src < K || ld_src % 8 != 0 || !src_ok(src_dtype) ||
      ((rows > 0 && K > 0) && (!dSrc || !dPacked || !dScales)) || (((uintptr_t)dSrc) & 15) ||
      (((uintptr_t)dPacked) & 15) || (!lanes && scales_layout != ASTERGEMM_MX_ROWS) ||
      (lanes && (K % 256 != 0 || (((uintptr_t)dScales) & 15)))) {
    set_error("astergemm_quantize_mxfp4: need a source of F32, BF16 or F16, K %% 32 == 0, "
              "ld_src >= K, ld_src %% 8 == 0, dSrc and dPacked 16-byte aligned; scales in lane "
              "order: K %% 256 == 0 and dScales 16-byte aligned");
    return ASTERGEMM_EINVAL;
  }
  if (rows == 0 || K == 0) return 0;
  const int64_t nblocks = rows * (K / 32);
  if (nblocks >= (int64_t)1 << 31) {
    set_error("astergemm_quantize_mxfp4: more than 2^31 blocks");
    return ASTERGEMM_EINVAL;
  }
  const dim3 grid(blocks_for(nblocks * 2));  // a workgroup takes 128 blocks per trip
  (void)hipGetLastError();
  with_src(src_dtype, [&](auto T) {
    constexpr int SRC = decltype(T)::value;
    auto go = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, dSrc, nblocks,
                         (unsigned)(K / 32), ld_src, dPacked, dScales);
    };
    if (lanes) {
      if (ld_src == K) go(quantize_mxfp4_kernel<SRC, true, true>);
      else go(quantize_mxfp4_kernel<SRC, false, true>);
    } else {
      if (ld_src == K) go(quantize_mxfp4_kernel<SRC, true, false>);
      else go(quantize_mxfp4_kernel<SRC, false, false>);
    }
  });
  AG_HIP(hipGetLastError());
  return 0;
}

extern "C" int astergemm_quantize_mxfp4(const void* dSrc, int src_dtype, int64_t rows, int64_t K,
                                        int64_t ld_src, uint8_t* dPacked, uint8_t* dScales,
                                        void* stream) {
  return astergemm_quantize_mxfp4_ex(dSrc, src_dtype, rows, K, ld_src, dPacked, dScales,
                                     ASTERGEMM_MX_ROWS, stream);
}

// ---- pre-shuffle of weights on the device ----------------------------------------------------
//
// Every pre-shuffled layout is a permutation of fixed-size units inside blocks of 16 (64) rows:
// thread t writes destination unit t, fetched from where the host functions of the same name
// take it.  MODE 0: 16-bit, the reference's shuffle_weight order (units of 8 bytes);
// 1: 16-bit, K8 order (16 bytes); 2: byte rows in step order (16 bytes); 3: e8m0 plane in
// step order (8 bytes); 4: e8m0 plane in lane order (1 byte).
namespace astergemm {
namespace {

template <int MODE>
__global__ __launch_bounds__(256) void preshuffle_kernel(const uint8_t* __restrict__ src,
                                                         uint8_t* __restrict__ dst, int64_t units,
                                                         int64_t rb) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= units) return;
  if constexpr (MODE == 0) {
    // dst (nb, kb, g, n, kh) <- src (nb, n, kb, kh, g), units of 4 elements
    const int64_t kblocks = rb / 64;
    const int kh = (int)(t & 1), n = (int)((t >> 1) & 15), g = (int)((t >> 5) & 3);
    const int64_t kb = (t >> 7) % kblocks, nb = (t >> 7) / kblocks;
    *(uint2*)(dst + t * 8) = *(const uint2*)(src + (nb * 16 + n) * rb + kb * 64 + kh * 32 + g * 8);
  } else if constexpr (MODE == 1) {
    // dst (nb, kb, g, n) <- src (nb, n, kb, g), units of 8 elements
    const int64_t kblocks = rb / 64;
    const int n = (int)(t & 15), g = (int)((t >> 4) & 3);
    const int64_t kb = (t >> 6) % kblocks, nb = (t >> 6) / kblocks;
    *(uint4*)(dst + t * 16) = *(const uint4*)(src + (nb * 16 + n) * rb + kb * 64 + g * 16);
  } else if constexpr (MODE == 2) {
    // dst (nb, step, u, q, n) <- src (nb, n, step, 4u + q), units of 16 bytes
    const int64_t steps = rb / 128;
    const int n = (int)(t & 15), q = (int)((t >> 4) & 3), u = (int)((t >> 6) & 1);
    const int64_t st = (t >> 7) % steps, nb = (t >> 7) / steps;
    *(uint4*)(dst + t * 16) = *(const uint4*)(src + (nb * 16 + n) * rb + st * 128 + (4 * u + q) * 16);
  } else if constexpr (MODE == 3) {
    // dst (nb, step, n) <- src (nb, n, step), units of 8 bytes; rb = K / 32 bytes
    const int64_t steps = rb / 8;
    const int n = (int)(t & 15);
    const int64_t st = (t >> 4) % steps, nb = (t >> 4) / steps;
    *(uint2*)(dst + t * 8) = *(const uint2*)(src + (nb * 16 + n) * rb + st * 8);
  } else if constexpr (MODE == 4) {
    // dst (nb4, step, q, i, tile, h) <- src (nb4, tile, i, step, 4h + q), bytes; rb = K / 32 bytes
    const int64_t steps = rb / 8;
    const int h = (int)(t & 1), tl = (int)((t >> 1) & 3), i = (int)((t >> 3) & 15), q = (int)((t >> 7) & 3);
    const int64_t st = (t >> 9) % steps, nb4 = (t >> 9) / steps;
    dst[t] = src[(nb4 * 64 + tl * 16 + i) * rb + st * 8 + 4 * h + q];
  }
}

// A's plane into lane order in groups of 128 rows: dst (g, step, q, i, tile, h) <- src (g, tile, i,
// step, 4h + q), one byte per thread; rows past `rows` get 127 (scale 1)
__global__ __launch_bounds__(256) void preshuffle_scales_a_kernel(const uint8_t* __restrict__ src,
                                                                  uint8_t* __restrict__ dst,
                                                                  int64_t units, int64_t rb, int64_t rows) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= units) return;
  const int64_t steps = rb / 8;
  const int h = (int)(t & 1), tl = (int)((t >> 1) & 7), i = (int)((t >> 4) & 15), q = (int)((t >> 8) & 3);
  const int64_t st = (t >> 10) % steps, g = (t >> 10) / steps;
  const int64_t row = g * 128 + tl * 16 + i;
  dst[t] = row < rows ? src[row * rb + st * 8 + 4 * h + q] : (uint8_t)127;
}

template <int MODE>
int preshuffle_launch(const void* src, void* dst, int64_t bytes, int unit, int64_t row_bytes_,
                      hipStream_t s) {
  const int64_t units = bytes / unit;
  if (units == 0) return 0;
  if ((units + 255) / 256 >= (int64_t)1 << 31) {
    set_error("astergemm_preshuffle: matrix too large");
    return ASTERGEMM_EINVAL;
  }
  (void)hipGetLastError();
  hipLaunchKernelGGL(preshuffle_kernel<MODE>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s,
                     (const uint8_t*)src, (uint8_t*)dst, units, row_bytes_);
  AG_HIP(hipGetLastError());
  return 0;
}

}  // namespace
}  // namespace astergemm

extern "C" int astergemm_preshuffle(int dtype_ab, int operand_path, int64_t N, int64_t K,
                                    const void* dSrc, void* dDst, const uint8_t* dMxSrc,
                                    uint8_t* dMxDst, void* stream) {
  using namespace astergemm;
  const bool is16 = dtype_ab == ASTERGEMM_F16 || dtype_ab == ASTERGEMM_BF16;
  const bool fp4 = dtype_ab == ASTERGEMM_MXFP4;
  if (!is16 && !fp4 && dtype_ab != ASTERGEMM_FP8_E4M3) {
    set_error("astergemm_preshuffle: dtype_ab must be F16, BF16, FP8_E4M3 or MXFP4");
    return ASTERGEMM_EINVAL;
  }
  // DIRECT_AB: one call per operand (A [M, K] or B [N, K]), both in DIRECT_B's 16-bit order
  if (operand_path == ASTERGEMM_OPERAND_DIRECT_AB && is16) operand_path = ASTERGEMM_OPERAND_DIRECT_B;
  if (operand_path != ASTERGEMM_OPERAND_DIRECT_B && operand_path != ASTERGEMM_OPERAND_DIRECT_B_K8) {
    set_error("astergemm_preshuffle: operand_path must be DIRECT_B, DIRECT_B_K8 or (16-bit "
              "operands) DIRECT_AB");
    return ASTERGEMM_EINVAL;
  }
  const bool k8 = operand_path == ASTERGEMM_OPERAND_DIRECT_B_K8;
  const int64_t rb = row_bytes(dtype_ab, K);
  const int64_t rows_mod = (fp4 && k8) ? 64 : 16;
  if (N < 0 || K < 0 || N % rows_mod != 0 || (is16 ? K % 32 != 0 : rb % 128 != 0) ||
      (N > 0 && K > 0 && (!dSrc || !dDst || dSrc == dDst)) || ((((uintptr_t)dSrc) | ((uintptr_t)dDst)) & 15) ||
      (fp4 && N > 0 && K > 0 && (!dMxSrc || !dMxDst || dMxSrc == dMxDst ||
                                 ((((uintptr_t)dMxSrc) | ((uintptr_t)dMxDst)) & 7)))) {
    set_error("astergemm_preshuffle: need N %% %d == 0, rows of whole %s, distinct 16-byte aligned "
              "source and destination (MXFP4: and distinct 8-byte aligned scale planes)",
              (int)rows_mod, is16 ? "32-element blocks" : "128-byte steps");
    return ASTERGEMM_EINVAL;
  }
  if (N == 0 || K == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (is16) rc = k8 ? preshuffle_launch<1>(dSrc, dDst, N * rb, 16, rb, s)
                    : preshuffle_launch<0>(dSrc, dDst, N * rb, 8, rb, s);
  else rc = preshuffle_launch<2>(dSrc, dDst, N * rb, 16, rb, s);
  if (rc != 0 || !fp4) return rc;
  return k8 ? preshuffle_launch<4>(dMxSrc, dMxDst, N * (K / 32), 1, K / 32, s)
            : preshuffle_launch<3>(dMxSrc, dMxDst, N * (K / 32), 8, K / 32, s);
}

extern "C" int astergemm_preshuffle_scales_a(int64_t M, int64_t K, const uint8_t* dMxSrc,
                                             uint8_t* dMxDst, void* stream) {
  using namespace astergemm;
  if (M < 0 || K < 0 || K % 256 != 0 || (M > 0 && K > 0 && (!dMxSrc || !dMxDst || dMxSrc == dMxDst)) ||
      ((((uintptr_t)dMxSrc) | ((uintptr_t)dMxDst)) & 15)) {
    set_error("astergemm_preshuffle_scales_a: need K %% 256 == 0 and distinct 16-byte aligned planes");
    return ASTERGEMM_EINVAL;
  }
  const int64_t units = astergemm_mx_lanes128_bytes(M, K);
  if (units == 0) return 0;
  if ((units + 255) / 256 >= (int64_t)1 << 31) {
    set_error("astergemm_preshuffle_scales_a: plane too large");
    return ASTERGEMM_EINVAL;
  }
  (void)hipGetLastError();
  hipLaunchKernelGGL(preshuffle_scales_a_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, dMxSrc, dMxDst, units, K / 32, M);
  AG_HIP(hipGetLastError());
  return 0;
}
