// Stream kernels (whole-ring, hand-scheduled MFMA loops) for f16 / bf16, fp8 and MXFP4:
// launchers, shape checks and the variant table.  Kept apart from gemm_tile.hip so that the
// two halves of the kernel set compile side by side.
#include "gemm_stream_kernel.hpp"
#include "gemm_stream8_kernel.hpp"
#include "gemm_stream4_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_stream(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 5 * BM * kRowBytes;
  auto k = gemm_stream_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
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

// ---- split K on the 128x128 kernel --------------------------------------------------------
//
// KIND 0: 16-bit operands, 1: fp8, 2: MXFP4 (ranges of an even number of steps)
template <int KIND, int DT, int OUT>
int launch_stream_splitk(const GemmArgs& a0, int grid, hipStream_t s) {
  (void)grid;
  constexpr int lds = KIND == 2 ? 4 * 128 * kRowBytes + 4 * 128 * 16 : 5 * 128 * kRowBytes;
  void (*k)(const GemmArgs);
  if constexpr (KIND == 0) k = gemm_stream_splitk_kernel<DT, 128, 128, 2, 2>;
  else if constexpr (KIND == 1) k = gemm_stream8_splitk_kernel<DT, 128, 128, 2, 2>;
  else k = gemm_stream4_splitk_kernel<DT, 128, 128, 2, 2>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  if constexpr (KIND == 2) {
    if ((((uintptr_t)a0.mx_a | (uintptr_t)a0.mx_b) & 15) != 0 || a0.mx_ld % 16 != 0)
      return (int)hipErrorInvalidValue;
  }
  const int tiles = a0.tiles_m * a0.tiles_n;
  const int S = stream_split_of(tiles, a0.ksteps, KIND == 2);
  if (S == 0) return (int)hipErrorInvalidValue;
  GemmArgs a = a0;
  if (!a.workspace) {
    if (int rc = splitk_workspace_for((size_t)S * a.M * a.N * sizeof(float), s, &a.workspace))
      return rc;
  }
  GemmArgs part = a;           // what the K-range workgroups see: fp32 planes, no epilogue terms
  part.split_k = S;
  part.ksteps = a.ksteps / S;
  part.ldc = a.N;
  part.scale_a = part.scale_b = part.bias = nullptr;
  hipLaunchKernelGGL(k, dim3(tiles * S), dim3(256), lds, s, part);
  return splitk_reduce(OUT, a, S, s);
}

const char* check_stream_splitk(const astergemm_config& c) {
  if (const char* why = check_stream_whole_k(c)) return why;
  if (c.dtype_ab == ASTERGEMM_MXFP4 && c.K % 512 != 0) return "K must be a multiple of 512";
  const int64_t tiles = ((c.M + 127) / 128) * ((c.N + 127) / 128);
  // shorter rows: the unsplit 64 x 64 kernels are ahead (fp8 256x4096x4096: 15.2 against 19.8 us)
  const int64_t min_steps = c.dtype_ab == ASTERGEMM_MXFP4 ? 32 : 64;
  if (row_bytes(c.dtype_ab, c.K) / kRowBytes < min_steps)
    return "split K needs rows of at least 8 KiB (4 KiB for MXFP4)";
  if (stream_split_of(tiles, row_bytes(c.dtype_ab, c.K) / kRowBytes,
                      c.dtype_ab == ASTERGEMM_MXFP4) == 0)
    return "split K needs at most 128 output tiles of 128 x 128 and a K that divides into 2..16 "
           "ranges of 8 or more 128-byte steps (an even number of steps for MXFP4)";
  if (c.M * c.N > ((int64_t)1 << 26)) return "split K workspace would pass 4 GiB";
  return nullptr;
}

int splits_stream_splitk(const astergemm_config& c) {
  const int64_t tiles = ((c.M + 127) / 128) * ((c.N + 127) / 128);
  const int S = stream_split_of(tiles, row_bytes(c.dtype_ab, c.K) / kRowBytes,
                                c.dtype_ab == ASTERGEMM_MXFP4);
  return S < 1 ? 1 : S;
}

#define AG_STREAM_SPLITK(name, KIND, DT, OUT, LDS, FUNC)                         \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 128, kRowBytes, 2, 2, 3, 4, LDS,  \
        (const void*)FUNC<DT, 128, 128, 2, 2>, launch_stream_splitk<KIND, DT, OUT>, \
        check_stream_splitk, ASTERGEMM_OPERAND_LDS, splits_stream_splitk         \
  }
#define AG_STREAM_SPLITK_SET(prefix, KIND, DT, LDS, FUNC)                        \
  AG_STREAM_SPLITK(prefix "_128x128_w2x2_bf16", KIND, DT, ASTERGEMM_BF16, LDS, FUNC),   \
      AG_STREAM_SPLITK(prefix "_128x128_w2x2_f32", KIND, DT, ASTERGEMM_F32, LDS, FUNC), \
      AG_STREAM_SPLITK(prefix "_128x128_w2x2_f16", KIND, DT, ASTERGEMM_F16, LDS, FUNC)

template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_stream8(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 5 * BM * kRowBytes;
  auto k = gemm_stream8_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
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
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
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

const Variant kStreamVariants[] = {
    AG_STREAM_SET("stream_bf16", ASTERGEMM_BF16),
    AG_STREAM_SPLITK_SET("splitk_bf16", 0, ASTERGEMM_BF16, 5 * 128 * kRowBytes, gemm_stream_splitk_kernel),
    AG_STREAM_SPLITK_SET("splitk_f16", 0, ASTERGEMM_F16, 5 * 128 * kRowBytes, gemm_stream_splitk_kernel),
    AG_STREAM_SPLITK_SET("splitk_fp8", 1, ASTERGEMM_FP8_E4M3, 5 * 128 * kRowBytes,
                         gemm_stream8_splitk_kernel),
    AG_STREAM_SPLITK_SET("splitk_mxfp4", 2, ASTERGEMM_MXFP4, 4 * 128 * kRowBytes + 4 * 128 * 16,
                         gemm_stream4_splitk_kernel),
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

int num_stream_variants() { return (int)(sizeof(kStreamVariants) / sizeof(kStreamVariants[0])); }
const Variant* stream_variants() { return kStreamVariants; }

}  // namespace astergemm
