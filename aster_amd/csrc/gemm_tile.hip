// Variant table and launchers of the LDS-staged MFMA tile kernels
// (device code: gemm_tile_kernel.hpp).
#include "gemm_pipe_kernel.hpp"
#include "gemm_stream_kernel.hpp"
#include "gemm_stream8_kernel.hpp"
#include "gemm_stream4_kernel.hpp"

namespace astergemm {
namespace {

// ---- host side: variant table ------------------------------------------------
template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_tile(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 2 * (BM + BN) * kRowBytes;
  auto k = gemm_tile_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)k,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_tile(const astergemm_config& c) {
  const int64_t kb = row_bytes(c.dtype_ab, c.K);
  if (c.dtype_ab == ASTERGEMM_MXFP4) {
    if (kb % kRowBytes != 0) return "MXFP4 needs K % 256 == 0";
  } else if (kb % 16 != 0) {
    return "K must cover a whole number of 16-byte granules";
  }
  return nullptr;
}

#define AG_TILE(name, DT, OUT, BM, BN, WM, WN)                                   \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, BM, BN, kRowBytes, WM, WN, 2, 1,       \
        2 * (BM + BN) * kRowBytes,                                               \
        (const void*)gemm_tile_kernel<DT, OUT, BM, BN, WM, WN>,                  \
        launch_tile<DT, OUT, BM, BN, WM, WN>, check_tile                         \
  }

#define AG_TILE_SET(prefix, DT)                                                        \
  AG_TILE(prefix "_256x256_w2x4_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 4),            \
      AG_TILE(prefix "_256x256_w2x4_f32", DT, ASTERGEMM_F32, 256, 256, 2, 4),          \
      AG_TILE(prefix "_256x256_w2x4_f16", DT, ASTERGEMM_F16, 256, 256, 2, 4),          \
      AG_TILE(prefix "_128x128_w2x2_bf16", DT, ASTERGEMM_BF16, 128, 128, 2, 2),        \
      AG_TILE(prefix "_128x128_w2x2_f32", DT, ASTERGEMM_F32, 128, 128, 2, 2),          \
      AG_TILE(prefix "_128x128_w2x2_f16", DT, ASTERGEMM_F16, 128, 128, 2, 2),          \
      AG_TILE(prefix "_128x64_w2x2_bf16", DT, ASTERGEMM_BF16, 128, 64, 2, 2),          \
      AG_TILE(prefix "_128x64_w2x2_f32", DT, ASTERGEMM_F32, 128, 64, 2, 2),            \
      AG_TILE(prefix "_128x64_w2x2_f16", DT, ASTERGEMM_F16, 128, 64, 2, 2),            \
      AG_TILE(prefix "_64x64_w2x2_bf16", DT, ASTERGEMM_BF16, 64, 64, 2, 2),            \
      AG_TILE(prefix "_64x64_w2x2_f32", DT, ASTERGEMM_F32, 64, 64, 2, 2),              \
      AG_TILE(prefix "_64x64_w2x2_f16", DT, ASTERGEMM_F16, 64, 64, 2, 2)

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_pipe(const GemmArgs& a0, int grid, hipStream_t s) {
  constexpr int lds = kStages * (BM + BN) * kSubBytes;
  auto k = gemm_pipe_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)k,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  // This kernel counts K in 64-byte sub-steps.
  GemmArgs a = a0;
  const int64_t kb = row_bytes(DT, a.K);
  a.ksteps = (int32_t)((kb + kSubBytes - 1) / kSubBytes);
  a.tail_granules = (int32_t)((kb % kSubBytes) / 16);
  hipLaunchKernelGGL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

#define AG_PIPE(name, DT, OUT, BM, BN, WM, WN)                                   \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, BM, BN, kSubBytes, WM, WN, kStages, 0, \
        kStages * (BM + BN) * kSubBytes,                                         \
        (const void*)gemm_pipe_kernel<DT, OUT, BM, BN, WM, WN>,                  \
        launch_pipe<DT, OUT, BM, BN, WM, WN>, check_tile                         \
  }

#define AG_PIPE_SET(prefix, DT)                                                        \
  AG_PIPE(prefix "_256x256_w2x4_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 4),            \
      AG_PIPE(prefix "_256x256_w2x4_f32", DT, ASTERGEMM_F32, 256, 256, 2, 4),          \
      AG_PIPE(prefix "_256x256_w2x4_f16", DT, ASTERGEMM_F16, 256, 256, 2, 4),          \
      AG_PIPE(prefix "_256x256_w2x2_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 2)

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_stream(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 5 * BM * kRowBytes;
  auto k = gemm_stream_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)k,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

// Whole 256x256 tiles and whole 128-byte K-steps only; other shapes go to the
// general tile kernel.
const char* check_stream(const astergemm_config& c) {
  // edge tiles are handled in units of 8 operand rows and 16-byte output chunks
  if (c.M % 8 != 0 || c.N % 8 != 0 || c.M < 8 || c.N < 8) return "M and N must be multiples of 8";
  // a K tail of 1..7 granules is multiplied after the loop; at least one whole step is needed
  if (row_bytes(c.dtype_ab, c.K) % 16 != 0) return "K must cover a whole number of 16-byte granules";
  if (row_bytes(c.dtype_ab, c.K) < kRowBytes) return "K must cover at least one 128-byte row chunk";
  if (c.ldc % 8 != 0) return "ldc must be a multiple of 8 elements";
  return nullptr;
}

const char* check_stream_whole_k(const astergemm_config& c) {
  if (const char* why = check_stream(c)) return why;
  if (row_bytes(c.dtype_ab, c.K) % kRowBytes != 0) return "K must fill whole 128-byte row chunks";
  return nullptr;
}

#define AG_STREAM(name, DT, OUT, BM, BN, WM, WN)                                 \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, BM, BN, kRowBytes, WM, WN, 3,          \
        (WM * WN == 8 || BM == 128) ? 2 : 0, 5 * BM * kRowBytes,                \
        (const void*)gemm_stream_kernel<DT, OUT, BM, BN, WM, WN>,                \
        launch_stream<DT, OUT, BM, BN, WM, WN>,                                  \
        (WM * WN == 8 || BM == 128) ? check_stream : check_stream_whole_k        \
  }

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_stream8(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 5 * BM * kRowBytes;
  auto k = gemm_stream8_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)k,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

#define AG_STREAM8(name, DT, OUT)                                                \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 4, 3, 2,       \
        5 * 256 * kRowBytes,                                                     \
        (const void*)gemm_stream8_kernel<DT, OUT, 256, 256, 2, 4>,               \
        launch_stream8<DT, OUT, 256, 256, 2, 4>, check_stream                    \
  }
#define AG_STREAM8_128(name, DT, OUT)                                            \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 128, kRowBytes, 2, 2, 3, 2,       \
        5 * 128 * kRowBytes,                                                     \
        (const void*)gemm_stream8_kernel<DT, OUT, 128, 128, 2, 2>,               \
        launch_stream8<DT, OUT, 128, 128, 2, 2>, check_stream                    \
  }

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_stream4(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 4 * BM * kRowBytes + 4 * BM * 16;
  // the scale planes are fetched in 16-byte granules
  if ((((uintptr_t)a.mx_a | (uintptr_t)a.mx_b) & 15) != 0 || a.mx_ld % 16 != 0)
    return (int)hipErrorInvalidValue;
  auto k = gemm_stream4_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)k,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

// Whole 256x256 tiles and an even number of 256-element K-steps (scales move in 16-byte
// granules = two K-steps of a row).
const char* check_stream4(const astergemm_config& c) {
  if (const char* why = check_stream_whole_k(c)) return why;
  if (c.K % 512 != 0) return "K must be a multiple of 512";
  return nullptr;
}

#define AG_STREAM4(name, DT, OUT)                                                \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 2, 2, 2,       \
        4 * 256 * kRowBytes + 4 * 256 * 16,                                      \
        (const void*)gemm_stream4_kernel<DT, OUT, 256, 256, 2, 2>,               \
        launch_stream4<DT, OUT, 256, 256, 2, 2>, check_stream4                   \
  }
#define AG_STREAM4_128(name, DT, OUT)                                            \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 128, kRowBytes, 2, 2, 2, 2,       \
        4 * 128 * kRowBytes + 4 * 128 * 16,                                      \
        (const void*)gemm_stream4_kernel<DT, OUT, 128, 128, 2, 2>,               \
        launch_stream4<DT, OUT, 128, 128, 2, 2>, check_stream4                   \
  }

#define AG_STREAM_SET(prefix, DT)                                                      \
  AG_STREAM(prefix "_256x256_w2x4_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 4),          \
      AG_STREAM(prefix "_256x256_w2x4_f32", DT, ASTERGEMM_F32, 256, 256, 2, 4),        \
      AG_STREAM(prefix "_256x256_w2x4_f16", DT, ASTERGEMM_F16, 256, 256, 2, 4),        \
      AG_STREAM(prefix "_256x256_w2x2_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 2),        \
      AG_STREAM(prefix "_128x128_w2x2_bf16", DT, ASTERGEMM_BF16, 128, 128, 2, 2),        \
      AG_STREAM(prefix "_128x128_w2x2_f32", DT, ASTERGEMM_F32, 128, 128, 2, 2),          \
      AG_STREAM(prefix "_128x128_w2x2_f16", DT, ASTERGEMM_F16, 128, 128, 2, 2)

const Variant kTileVariants[] = {
    AG_TILE_SET("tile_bf16", ASTERGEMM_BF16),
    AG_TILE_SET("tile_f16", ASTERGEMM_F16),
    AG_TILE_SET("tile_fp8", ASTERGEMM_FP8_E4M3),
    AG_TILE_SET("tile_mxfp4", ASTERGEMM_MXFP4),
    AG_PIPE_SET("pipe_bf16", ASTERGEMM_BF16),
    AG_PIPE_SET("pipe_f16", ASTERGEMM_F16),
    AG_PIPE_SET("pipe_fp8", ASTERGEMM_FP8_E4M3),
    AG_STREAM_SET("stream_bf16", ASTERGEMM_BF16),
    AG_STREAM_SET("stream_f16", ASTERGEMM_F16),
    AG_STREAM8("stream_fp8_256x256_w2x4_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_STREAM8("stream_fp8_256x256_w2x4_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_STREAM8("stream_fp8_256x256_w2x4_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
};

}  // namespace

int num_tile_variants() { return (int)(sizeof(kTileVariants) / sizeof(kTileVariants[0])); }
const Variant* tile_variants() { return kTileVariants; }

}  // namespace astergemm
