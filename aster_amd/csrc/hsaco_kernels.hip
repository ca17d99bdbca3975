// Code-object entry points: the tile kernel behind `extern "C"` names, built with
// `hipcc --genco` into astergemm_kernels.hsaco so that a generic module launcher
// (hipModuleLoadData + hipModuleLaunchKernel, i.e. the reference's execute_hsaco,
// python/aster/execution/core.py:605-717) can run it.  The reference's GEMM code
// objects take three pointers and bake the sizes in
// (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:150-156);
// these take the sizes as trailing int32 arguments.  Launch with a 1-D grid of
// ceil(M/128) * ceil(N/128) workgroups, 256 threads, 65536 bytes of dynamic LDS.
#include "gemm_tile_kernel.hpp"

using namespace astergemm;

namespace {
__device__ __forceinline__ GemmArgs make_args(const void* A, const void* B, void* C, int M, int N,
                                              int K, int elt_bytes) {
  GemmArgs a = {};
  a.A = (const uint8_t*)A;
  a.B = (const uint8_t*)B;
  a.C = C;
  a.lda_bytes = a.ldb_bytes = (int64_t)K * elt_bytes;
  a.ldc = N;
  a.M = M;
  a.N = N;
  a.K = K;
  const int kb = K * elt_bytes;
  a.ksteps = (kb + 127) / 128;
  a.tail_granules = (kb % 128) / 16;
  a.tiles_m = (M + 127) / 128;
  a.tiles_n = (N + 127) / 128;
  a.group_m = 8;
  return a;
}
}  // namespace

// C[M,N] (f32) = A[M,K] (f16) * B[N,K]^T (f16); K % 8 == 0.
extern "C" __global__ __launch_bounds__(256) void gemm_cdna4(const void* A, const void* B,
                                                             void* C, int M, int N, int K) {
  gemm_tile_body<ASTERGEMM_F16, ASTERGEMM_F32, 128, 128, 2, 2>(make_args(A, B, C, M, N, K, 2));
}

// Same with bf16 operands and bf16 output.
extern "C" __global__ __launch_bounds__(256) void gemm_cdna4_bf16(const void* A, const void* B,
                                                                  void* C, int M, int N, int K) {
  gemm_tile_body<ASTERGEMM_BF16, ASTERGEMM_BF16, 128, 128, 2, 2>(make_args(A, B, C, M, N, K, 2));
}
