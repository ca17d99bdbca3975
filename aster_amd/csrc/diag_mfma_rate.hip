// Diagnostic, not part of the GEMM path: the MFMA rate the chip reaches on given operand values
// with nothing else going on -- a loop of independent MFMAs over registers that were filled once
// from a sample of the caller's operand bytes.  No LDS, no memory traffic, no waits: what is left
// is the matrix pipe under the board's power limit, and that depends on the values (with zeros
// the loop runs close to the published peak, with N(0, 0.02) bf16 data it settles near 70 % of
// it).  The loop is ordered like the GEMM kernels' inner loops (the first operand is held for
// four instructions in a row, the second changes every instruction), so its rate is a measured
// reference to read a kernel's TFLOP/s against next to the published peak; it is not a proven
// upper bound (another operand order or register pattern may draw less power).  Shape of the
// loop: 32 independent accumulators per wave from eight + four operand fragments, one operand
// held for eight instructions -- the register picture of a 128 x 64 wave tile; a loop with 16
// accumulators from four + four fragments issues ~8 % fewer MFMAs per clock even on zeros and
// reads 15 % low on random data.  The instruction
// per dtype is the one the GEMM kernels use: v_mfma_f32_16x16x32_{bf16,f16} and
// v_mfma_scale_f32_16x16x128_f8f6f4 (fp8, fp4 with unit scales), the reference's
// (include/aster/Dialect/AMDGCN/IR/Instructions/MMA.td:792).
#include "astergemm_internal.h"

namespace astergemm {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

constexpr int kAcc = 32;  // independent accumulators per wave: eight A x four B operands, a 128 x 64 wave tile

template <int DT>
__global__ __launch_bounds__(512) void mfma_rate_kernel(const i32x4* sample, int64_t n16,
                                                           int iters, float* sink) {
  const int64_t t = (int64_t)blockIdx.x * 512 + threadIdx.x;
  constexpr int R = (DT == ASTERGEMM_FP8_E4M3) ? 2 : 1;  // 16-byte registers per operand
  i32x4 a[8][R], b[4][R];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < R; ++r) a[i][r] = sample[(t * 24 + i * R + r) % n16];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < R; ++r) b[i][r] = sample[(t * 24 + 16 + i * R + r) % n16];
  f32x4 acc[kAcc];
#pragma unroll
  for (int i = 0; i < kAcc; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kAcc; ++i) {
      const int ia = i >> 3, ib = i & 7;  // first operand (one of four) held for eight instructions
      if constexpr (DT == ASTERGEMM_BF16) {
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, b[ia][0]),
                                                          __builtin_bit_cast(bf16x8_t, a[ib][0]),
                                                          acc[i], 0, 0, 0);
      } else if constexpr (DT == ASTERGEMM_F16) {
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, b[ia][0]),
                                                         __builtin_bit_cast(f16x8_t, a[ib][0]),
                                                         acc[i], 0, 0, 0);
      } else if constexpr (DT == ASTERGEMM_FP8_E4M3) {
        const i32x4 al = b[ia][0], ah = b[ia][1], bl = a[ib][0], bh = a[ib][1];
        acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8_t{al[0], al[1], al[2], al[3], ah[0], ah[1], ah[2], ah[3]},
            i32x8_t{bl[0], bl[1], bl[2], bl[3], bh[0], bh[1], bh[2], bh[3]}, acc[i], 0, 0, 0, 0, 0,
            0);
      } else {  // fp4: 128 nibbles per lane in four registers, unit e8m0 scales
        const i32x4 al = b[ia][0], bl = a[ib][0];
        acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            i32x8_t{al[0], al[1], al[2], al[3], 0, 0, 0, 0},
            i32x8_t{bl[0], bl[1], bl[2], bl[3], 0, 0, 0, 0}, acc[i], 4, 4, 0, 127, 0, 127);
      }
    }
  }
  f32x4 s = acc[0];
#pragma unroll
  for (int i = 1; i < kAcc; ++i) s += acc[i];
  sink[t] = s[0] + s[1] + s[2] + s[3];
}

template <int DT>
int run_mfma_rate(const void* sample, int64_t bytes, int target_ms, double* tflops, hipStream_t s) {
  int dev = 0;
  hipDeviceProp_t prop;
  AG_HIP(hipGetDevice(&dev));
  AG_HIP(hipGetDeviceProperties(&prop, dev));
  const int wgs = prop.multiProcessorCount;  // one workgroup of eight waves per CU, two per SIMD
  float* sink = nullptr;
  AG_HIP(hipMalloc((void**)&sink, (size_t)wgs * 512 * sizeof(float)));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = 0;
  auto fail = [&](hipError_t e, const char* what) {
    rc = hip_fail(e, what, __FILE__, __LINE__);
  };
  const double flop_per_iter =
      (double)wgs * 8 * kAcc * 2.0 * 16 * 16 * (DT == ASTERGEMM_BF16 || DT == ASTERGEMM_F16 ? 32 : 128);
  hipError_t e;
  if ((e = hipEventCreate(&e0)) != hipSuccess) fail(e, "hipEventCreate");
  if (!rc && (e = hipEventCreate(&e1)) != hipSuccess) fail(e, "hipEventCreate");
  // a short launch to size the timed ones (about 10 ms each), then launches until the target
  int iters = 2000;
  float ms = 0.f;
  double total_ms = 0.0, total_flop = 0.0;
  for (int pass = 0; !rc && pass < 2; ++pass) {
    const int launches = pass == 0 ? 1 : (target_ms + 9) / 10;
    for (int l = 0; !rc && l < launches; ++l) {
      if ((e = hipEventRecord(e0, s)) != hipSuccess) { fail(e, "hipEventRecord"); break; }
      hipLaunchKernelGGL(mfma_rate_kernel<DT>, dim3(wgs), dim3(512), 0, s, (const i32x4*)sample,
                         bytes / 16, iters, sink);
      if ((e = hipGetLastError()) != hipSuccess) { fail(e, "mfma_rate_kernel"); break; }
      if ((e = hipEventRecord(e1, s)) != hipSuccess) { fail(e, "hipEventRecord"); break; }
      if ((e = hipEventSynchronize(e1)) != hipSuccess) { fail(e, "hipEventSynchronize"); break; }
      if ((e = hipEventElapsedTime(&ms, e0, e1)) != hipSuccess) { fail(e, "hipEventElapsedTime"); break; }
      if (pass == 1) {
        total_ms += ms;
        total_flop += flop_per_iter * iters;
      }
    }
    if (pass == 0 && !rc) {
      const double want = 10.0 * iters / (ms > 0.01f ? ms : 0.01f);
      iters = want < 1000 ? 1000 : (want > 4e6 ? 4000000 : (int)want);
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  if (rc) return rc;
  *tflops = total_flop / total_ms * 1e-9;
  return 0;
}

}  // namespace
}  // namespace astergemm

using namespace astergemm;

extern "C" int astergemm_diag_mfma_rate(int dtype_ab, const void* dSample, int64_t sample_bytes,
                                      int target_ms, double* tflops, void* stream) {
  if (!dSample || !tflops || sample_bytes < 4096 || (sample_bytes & 15) ||
      ((uintptr_t)dSample & 15) || target_ms <= 0 || target_ms > 10000) {
    set_error("astergemm_diag_mfma_rate: need a 16-byte aligned sample of at least 4096 bytes (a "
              "multiple of 16) and 0 < target_ms <= 10000");
    return ASTERGEMM_EINVAL;
  }
  (void)hipGetLastError();
  hipStream_t s = (hipStream_t)stream;
  switch (dtype_ab) {
    case ASTERGEMM_BF16: return run_mfma_rate<ASTERGEMM_BF16>(dSample, sample_bytes, target_ms, tflops, s);
    case ASTERGEMM_F16: return run_mfma_rate<ASTERGEMM_F16>(dSample, sample_bytes, target_ms, tflops, s);
    case ASTERGEMM_FP8_E4M3:
      return run_mfma_rate<ASTERGEMM_FP8_E4M3>(dSample, sample_bytes, target_ms, tflops, s);
    case ASTERGEMM_MXFP4: return run_mfma_rate<ASTERGEMM_MXFP4>(dSample, sample_bytes, target_ms, tflops, s);
  }
  set_error("astergemm_diag_mfma_rate: dtype_ab must be F16, BF16, FP8_E4M3 or MXFP4");
  return ASTERGEMM_EINVAL;
}
