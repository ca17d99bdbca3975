// Variant table and launchers of the LDS-staged MFMA tile kernels
// (device code: gemm_tile_kernel.hpp).
#include "gemm_tile_kernel.hpp"

namespace astergemm {
namespace {

// ---- host side: variant table ------------------------------------------------
template <int DT, int OUT, int BM, int BN, int WM, int WN>
int launch_tile(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 2 * (BM + BN) * kRowBytes;
  auto k = gemm_tile_kernel<DT, OUT, BM, BN, WM, WN>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
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

const Variant kTileVariants[] = {
    AG_TILE_SET("tile_bf16", ASTERGEMM_BF16),
    AG_TILE_SET("tile_f16", ASTERGEMM_F16),
    AG_TILE_SET("tile_fp8", ASTERGEMM_FP8_E4M3),
    AG_TILE_SET("tile_mxfp4", ASTERGEMM_MXFP4),
};

}  // namespace

int num_tile_variants() { return (int)(sizeof(kTileVariants) / sizeof(kTileVariants[0])); }
const Variant* tile_variants() { return kTileVariants; }

}  // namespace astergemm
