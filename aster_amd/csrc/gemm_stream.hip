// Stream kernels (whole-ring, hand-scheduled MFMA loops) for f16 / bf16, fp8 and MXFP4:
// launchers, shape checks and the variant table.  Kept apart from gemm_tile.hip so that the
// two halves of the kernel set compile side by side.
#include <vector>

#include "gemm_stream_kernel.hpp"
#include "gemm_stream8_kernel.hpp"
#include "gemm_stream4_kernel.hpp"
#include "gemm_streamdb_kernel.hpp"
#include "gemm_stream4db_kernel.hpp"
#include "gemm_stream4dbl_kernel.hpp"
#include "gemm_stream8db_kernel.hpp"
#include "gemm_directab_kernel.hpp"

namespace astergemm {
namespace {

template <int DT, int OUT, int BM, int BN, int WM, int WN, int NSLOT = 5>
int launch_stream(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = NSLOT * BM * kRowBytes;
  auto k = gemm_stream_kernel<DT, OUT, BM, BN, WM, WN, NSLOT>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
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

// The 128 x 128 kernel with a ring of nine slots (144 KiB of LDS, one workgroup per CU): four
// K-steps requested ahead instead of two.  For grids of at most one workgroup per CU with two or
// more tile rows, where nothing else covers a workgroup's waits (bf16, five -> nine slots:
// 256 x 14336 x 4096 37.7-38.7 -> 33.7-34.4 us, 384 x 8192 x 4096 34.4 -> 31.0, 2048^3 23.3 ->
// 21.2, 1024 x 4096 x 4096 36.9 -> 35.5; one tile row, which is HBM-bound on B alone, loses:
// 128 x 28672 x 4096 39.8 -> 41.8; eight waves instead of four: level).
const char* check_stream_ring9(const astergemm_config& c) {
  if (const char* why = check_stream(c)) return why;
  int cus = device_cus();
  if (cus <= 0) cus = 256;  // no device to ask: describe the MI355X
  const int64_t tm = (c.M + 127) / 128, tn = (c.N + 127) / 128;
  if (tm < 2) return "the nine-slot ring pays from two tile rows on";
  if (tm * tn > cus) return "the nine-slot ring takes the LDS of a CU: at most one workgroup per CU";
  if (row_bytes(c.dtype_ab, c.K) < 16 * kRowBytes) return "the nine-slot ring needs 16 K-steps or more";
  return nullptr;
}
#define AG_STREAM_RING9(name, DT, OUT)                                           \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 128, kRowBytes, 2, 2, 5, 3,       \
        9 * 128 * kRowBytes,                                                     \
        (const void*)gemm_stream_kernel<DT, OUT, 128, 128, 2, 2, 9>,             \
        launch_stream<DT, OUT, 128, 128, 2, 2, 9>, check_stream_ring9            \
  }
#define AG_STREAM_RING9_SET(prefix, DT)                                          \
  AG_STREAM_RING9(prefix "_128x128_w2x2_ring9_bf16", DT, ASTERGEMM_BF16),        \
      AG_STREAM_RING9(prefix "_128x128_w2x2_ring9_f32", DT, ASTERGEMM_F32),      \
      AG_STREAM_RING9(prefix "_128x128_w2x2_ring9_f16", DT, ASTERGEMM_F16)

// ---- B pre-shuffled, loaded straight into MFMA operands (gemm_streamdb_kernel.hpp) ---------
template <int DT, int OUT, int NSLOT, int NBUF, int WM>
int launch_streamdb(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 5 * 128 * WM * kRowBytes;  // the epilogue stages through the ring
  auto k = gemm_streamdb_kernel<DT, OUT, NSLOT, NBUF, WM>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  // what the kernel's indexing assumes: whole 16-row blocks of B and whole K-steps
  if (a.N % 16 != 0 || a.N < 16 || a.M < 8 || a.M % 8 != 0 || a.K % 64 != 0 || a.tail_granules != 0 ||
      a.ldb_bytes != (int64_t)a.K * 2)
    return (int)hipErrorInvalidValue;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * 256), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_streamdb(const astergemm_config& c) {
  if (c.M % 8 != 0 || c.M < 8) return "M must be a multiple of 8";
  if (c.N % 16 != 0 || c.N < 16) return "pre-shuffled B needs N % 16 == 0";
  if (c.K % 64 != 0) return "pre-shuffled B in K8 order needs K % 64 == 0";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  if (c.ldc % 8 != 0) return "ldc must be a multiple of 8 elements";
  if (c.N * c.K * 2 >= ((int64_t)1 << 32)) return "pre-shuffled B must stay below 4 GiB";
  return nullptr;
}

#define AG_STREAMDB(name, DT, OUT, NSLOT, NBUF, WM, RANK)                        \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128 * WM, 256, kRowBytes, WM, 4, NSLOT, RANK, \
        5 * 128 * WM * kRowBytes,                                                \
        (const void*)gemm_streamdb_kernel<DT, OUT, NSLOT, NBUF, WM>,             \
        launch_streamdb<DT, OUT, NSLOT, NBUF, WM>, check_streamdb,               \
        ASTERGEMM_OPERAND_DIRECT_B_K8                                            \
  }

// ---- A and B pre-shuffled, both loaded straight into MFMA operands, no LDS
// (gemm_directab_kernel.hpp) --------------------------------------------------------------------
template <int DT, int OUT, int TM, int TN, int WM, int WN, int NB>
int launch_directab(const GemmArgs& a, int grid, hipStream_t s) {
  auto k = gemm_directab_kernel<DT, OUT, TM, TN, WM, WN, NB>;
  // what the kernel's indexing assumes: whole 16-row blocks of both operands, whole 32-element
  // chunk columns, both operands packed
  if (a.M % 16 != 0 || a.M < 16 || a.N % 16 != 0 || a.N < 16 || a.K % 32 != 0 || a.K < 32 ||
      a.lda_bytes != (int64_t)a.K * 2 || a.ldb_bytes != (int64_t)a.K * 2)
    return (int)hipErrorInvalidValue;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * WN * 64), 0, s, a);
  return (int)hipGetLastError();
}

const char* check_directab(const astergemm_config& c) {
  if (c.M % 16 != 0 || c.M < 16) return "pre-shuffled A needs M % 16 == 0";
  if (c.N % 16 != 0 || c.N < 16) return "pre-shuffled B needs N % 16 == 0";
  if (c.K % 32 != 0) return "pre-shuffled operands need K % 32 == 0";
  if (c.lda != 0 && c.lda != c.K) return "pre-shuffled A is packed (lda = K)";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  if (c.ldc % 4 != 0) return "ldc must be a multiple of 4 elements";
  if (c.M * c.K * 2 >= ((int64_t)1 << 32) || c.N * c.K * 2 >= ((int64_t)1 << 32))
    return "pre-shuffled operands must stay below 4 GiB each";
  return nullptr;
}

#define AG_DIRECTAB(name, DT, OUT, TM, TN, WM, WN, NB, RANK)                     \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, TM * 16 * WM, TN * 16 * WN, 64, WM, WN, NB, RANK, 0, \
        (const void*)gemm_directab_kernel<DT, OUT, TM, TN, WM, WN, NB>,          \
        launch_directab<DT, OUT, TM, TN, WM, WN, NB>, check_directab,            \
        ASTERGEMM_OPERAND_DIRECT_AB                                              \
  }
#define AG_DIRECTAB_SET(prefix, DT)                                                        \
  AG_DIRECTAB(prefix "_128x256_w1x4_bf16", DT, ASTERGEMM_BF16, 8, 4, 1, 4, 4, 1),          \
      AG_DIRECTAB(prefix "_128x256_w1x4_f32", DT, ASTERGEMM_F32, 8, 4, 1, 4, 4, 1),        \
      AG_DIRECTAB(prefix "_128x256_w1x4_f16", DT, ASTERGEMM_F16, 8, 4, 1, 4, 4, 1),        \
      AG_DIRECTAB(prefix "_256x256_w2x2_bf16", DT, ASTERGEMM_BF16, 8, 8, 2, 2, 3, 2),      \
      AG_DIRECTAB(prefix "_256x256_w2x2_f32", DT, ASTERGEMM_F32, 8, 8, 2, 2, 3, 2),        \
      AG_DIRECTAB(prefix "_256x256_w2x2_f16", DT, ASTERGEMM_F16, 8, 8, 2, 2, 3, 2)

// ---- MXFP4, B pre-shuffled (payload in step order, scale plane in lane order) and loaded
// straight into MFMA operands: 128 x 256 tiles, four waves (gemm_stream4db_kernel.hpp) ---------
template <int DT, int OUT, bool SAL>
int launch_stream4db(const GemmArgs& a, int grid, hipStream_t s) {
  // SAL: A's e8m0 plane in lane order as well (gemm_stream4dbl_kernel.hpp), nothing but A in LDS
  constexpr int lds = 4 * 128 * kRowBytes + (SAL ? 0 : 2 * 128 * 16);
  void (*k)(const GemmArgs);
  if constexpr (SAL) k = gemm_stream4dbl_kernel<DT, OUT>;
  else k = gemm_stream4db_kernel<DT, OUT>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  // what the kernel's indexing assumes: whole 64-row groups of B, an even number of whole
  // K-steps, packed B, A scale rows fetched in 16-byte granules
  if (a.N % 64 != 0 || a.N < 64 || a.M < 8 || a.M % 8 != 0 || a.K % 512 != 0 || a.tail_granules != 0 ||
      a.ldb_bytes != (int64_t)a.K / 2 || (((uintptr_t)a.mx_a | (uintptr_t)a.mx_b) & 15) != 0 ||
      a.mx_ld % 16 != 0)
    return (int)hipErrorInvalidValue;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(256), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_stream4db(const astergemm_config& c) {
  if (c.M % 8 != 0 || c.M < 8) return "M must be a multiple of 8";
  if (c.N % 64 != 0 || c.N < 64) return "the pre-shuffled scale plane needs N % 64 == 0";
  if (c.K % 512 != 0) return "K must be a multiple of 512";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  if (c.ldc % 8 != 0) return "ldc must be a multiple of 8 elements";
  if (c.N * (c.K / 2) >= ((int64_t)1 << 32)) return "pre-shuffled B must stay below 4 GiB";
  return nullptr;
}

#define AG_STREAM4DB(name, DT, OUT, SAL)                                         \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 256, kRowBytes, 1, 4, 4, 2,       \
        4 * 128 * kRowBytes + (SAL ? 0 : 2 * 128 * 16),                          \
        SAL ? (const void*)gemm_stream4dbl_kernel<DT, OUT>                       \
            : (const void*)gemm_stream4db_kernel<DT, OUT>,                       \
        launch_stream4db<DT, OUT, SAL>, check_stream4db,                         \
        ASTERGEMM_OPERAND_DIRECT_B_K8, nullptr, nullptr,                         \
        SAL ? ASTERGEMM_MX_LANES128 : ASTERGEMM_MX_ROWS                          \
  }

// ---- fp8, B pre-shuffled into step order and loaded straight into MFMA operands: 128 x 256
// tiles, four waves (gemm_stream8db_kernel.hpp) -------------------------------------------------
template <int DT, int OUT>
int launch_stream8db(const GemmArgs& a, int grid, hipStream_t s) {
  constexpr int lds = 4 * 128 * kRowBytes;
  auto k = gemm_stream8db_kernel<DT, OUT>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  // what the kernel's indexing assumes: whole 16-row blocks of B, whole K-steps, packed B
  if (a.N % 16 != 0 || a.N < 16 || a.M < 8 || a.M % 8 != 0 || a.K % 128 != 0 || a.tail_granules != 0 ||
      a.ldb_bytes != (int64_t)a.K)
    return (int)hipErrorInvalidValue;
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(256), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_stream8db(const astergemm_config& c) {
  if (c.M % 8 != 0 || c.M < 8) return "M must be a multiple of 8";
  if (c.N % 16 != 0 || c.N < 16) return "pre-shuffled B needs N % 16 == 0";
  if (c.K % 128 != 0) return "pre-shuffled fp8 B needs K % 128 == 0";
  if (c.ldb != 0 && c.ldb != c.K) return "pre-shuffled B is packed (ldb = K)";
  if (c.ldc % 8 != 0) return "ldc must be a multiple of 8 elements";
  if (c.N * c.K >= ((int64_t)1 << 32)) return "pre-shuffled B must stay below 4 GiB";
  return nullptr;
}

#define AG_STREAM8DB(name, DT, OUT)                                              \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 256, kRowBytes, 1, 4, 4, 2,       \
        4 * 128 * kRowBytes,                                                     \
        (const void*)gemm_stream8db_kernel<DT, OUT>, launch_stream8db<DT, OUT>,  \
        check_stream8db, ASTERGEMM_OPERAND_DIRECT_B_K8                           \
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
  AG_LAUNCH_KERNEL(k, dim3(tiles * S), dim3(256), lds, s, part);
  // the partial sums must exist before anything adds them: a failed launch ends here
  if (const hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
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
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
  return (int)hipGetLastError();
}

// The 256 x 256 fp8 kernel as a tile walk (see gemm_stream8_body): one workgroup per CU.
template <int DT, int OUT>
int launch_stream8_walk(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  constexpr int lds = 5 * 256 * kRowBytes;
  // what the kernel assumes: whole tiles (its epilogue stores without bounds checks), whole
  // K-steps and enough of them for the steady form of trip 0
  if (a.M % 256 != 0 || a.N % 256 != 0 || a.tail_granules != 0 || a.ksteps < 4)
    return (int)hipErrorInvalidValue;
  auto k = gemm_stream8_walk_kernel<DT, OUT, 256, 256, 2, 4>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  const int tiles = a.tiles_m * a.tiles_n;
  AG_LAUNCH_KERNEL(k, dim3(tiles < cus ? tiles : cus), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_stream8_walk(const astergemm_config& c) {
  if (const char* why = check_stream_whole_k(c)) return why;
  if (c.K < 512) return "the tile walk needs at least four K-steps";
  if (c.M % 256 != 0 || c.N % 256 != 0) return "the tile walk needs M and N to be multiples of 256";
  int cus = device_cus();
  if (cus <= 0) cus = 256;                       // no device to ask: describe the MI355X
  if (((c.M + 255) / 256) * ((c.N + 255) / 256) <= cus)
    return "the tile walk pays from two tiles per workgroup on";
  return nullptr;
}

int grid_stream_walk(const astergemm_config& c, int cus) {
  const int64_t tiles = ((c.M + 255) / 256) * ((c.N + 255) / 256);
  if (cus <= 0) cus = 256;
  return (int)(tiles > cus ? cus : tiles);
}

#define AG_STREAM8_WALK(name, DT, OUT, RANK)                                     \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 4, 3, RANK,    \
        5 * 256 * kRowBytes,                                                     \
        (const void*)gemm_stream8_walk_kernel<DT, OUT, 256, 256, 2, 4>,          \
        launch_stream8_walk<DT, OUT>, check_stream8_walk, ASTERGEMM_OPERAND_LDS, \
        nullptr, grid_stream_walk                                                \
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
  AG_LAUNCH_KERNEL(k, dim3(grid), dim3(WM * WN * 64), lds, s, a);
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
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 2, 2, 1,       \
        4 * 256 * kRowBytes + 4 * 256 * 16,                                      \
        (const void*)gemm_stream4_kernel<DT, OUT, 256, 256, 2, 2>,               \
        launch_stream4<DT, OUT, 256, 256, 2, 2>, check_stream4                   \
  }
// The same kernel with eight waves (2 x 4, wave tile 128 x 64, two waves per SIMD): with the
// accumulators in the accumulation registers it allocates without spills (128 + 116), and a
// second wave on every SIMD covers the waits of the first.  p50, one box, four -> eight waves:
// 4096 x 14336 x 4096 134.2 -> 125.3 us, 8192^3 246.8 -> 243.1, 16384 x 16384 x 4096 550.5 ->
// 533.3, 4096^3 38.1 -> 37.3; the same bits.  Preferred (rank 2 over 1).
#define AG_STREAM4_W8(name, DT, OUT, RANK)                                       \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 4, 2, RANK,    \
        4 * 256 * kRowBytes + 4 * 256 * 16,                                      \
        (const void*)gemm_stream4_kernel<DT, OUT, 256, 256, 2, 4>,               \
        launch_stream4<DT, OUT, 256, 256, 2, 4>, check_stream4                   \
  }
// Tile walk: one workgroup per CU takes its tiles round-robin as one long K loop, the next
// tile's first K-steps arriving during the last trips and the epilogue of the current one
// (see gemm_stream4_body).  16 KiB of LDS outside the ring stage the epilogue.
template <int DT, int OUT>
int launch_stream4_walk(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  constexpr int lds = 4 * 256 * kRowBytes + 4 * 256 * 16 + 8 * 2048;
  if ((((uintptr_t)a.mx_a | (uintptr_t)a.mx_b) & 15) != 0 || a.mx_ld % 16 != 0)
    return (int)hipErrorInvalidValue;
  // what the kernel assumes: slot parities that carry over from tile to tile, and whole tiles
  // (its epilogue stores without bounds checks)
  if (a.ksteps % 4 != 0 || a.M % 256 != 0 || a.N % 256 != 0) return (int)hipErrorInvalidValue;
  auto k = gemm_stream4_walk_kernel<DT, OUT, 256, 256, 2, 4>;
  static std::atomic<uint64_t> attr_devs{0};
  if (int e = lds_attr_once(attr_devs, (const void*)k, lds)) return e;
  const int cus = device_cus();
  if (cus <= 0) return (int)hipErrorNoDevice;
  const int tiles = a.tiles_m * a.tiles_n;
  AG_LAUNCH_KERNEL(k, dim3(tiles < cus ? tiles : cus), dim3(512), lds, s, a);
  return (int)hipGetLastError();
}

const char* check_stream4_walk(const astergemm_config& c) {
  if (const char* why = check_stream4(c)) return why;
  if (c.K % 1024 != 0) return "the tile walk needs K to be a multiple of 1024";
  if (c.M % 256 != 0 || c.N % 256 != 0) return "the tile walk needs M and N to be multiples of 256";
  int cus = device_cus();
  if (cus <= 0) cus = 256;                       // no device to ask: describe the MI355X
  if (((c.M + 255) / 256) * ((c.N + 255) / 256) <= cus)
    return "the tile walk pays from two tiles per workgroup on";
  return nullptr;
}

int grid_stream4_walk(const astergemm_config& c, int cus) {
  const int64_t tiles = ((c.M + 255) / 256) * ((c.N + 255) / 256);
  if (cus <= 0) cus = 256;
  return (int)(tiles > cus ? cus : tiles);
}

#define AG_STREAM4_WALK(name, DT, OUT)                                           \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, 2, 4, 2, 3,       \
        4 * 256 * kRowBytes + 4 * 256 * 16 + 8 * 2048,                           \
        (const void*)gemm_stream4_walk_kernel<DT, OUT, 256, 256, 2, 4>,          \
        launch_stream4_walk<DT, OUT>, check_stream4_walk, ASTERGEMM_OPERAND_LDS, \
        nullptr, grid_stream4_walk                                               \
  }
#define AG_STREAM4_128(name, DT, OUT)                                            \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 128, 128, kRowBytes, 2, 2, 2, 2,       \
        4 * 128 * kRowBytes + 4 * 128 * 16,                                      \
        (const void*)gemm_stream4_kernel<DT, OUT, 128, 128, 2, 2>,               \
        launch_stream4<DT, OUT, 128, 128, 2, 2>, check_stream4                   \
  }

// ---- whole rounds of 256 x 256 tiles, the rest in 128 x 128 tiles ---------------------------
//
// One workgroup of the 256 x 256 kernels runs per CU, so a tile count that is not a multiple of
// the CU count leaves the last round partly empty (4096 x 14336: 896 tiles on 256 CUs = 3.5
// rounds, paid as 4).  The problem is cut along N or M: the part whose 256 x 256 tiles fill
// whole rounds goes to the 256 x 256 kernel, the remaining columns (or rows) to the 128 x 128
// kernel of the same family, two workgroups per CU, right behind it on the same stream.
// Measured on 4096 x 14336 x 4096, p50 on one box, 256 x 256 alone -> with the cut: MXFP4 136.3 ->
// 134.7 us, bf16 350.2 -> 343.4 us, fp8 179.2 -> 180.0 us (128 x 128 alone: 141.9, 393.7, 203.5).
// The gain is far below the 12 % of the empty half round: the chip is power limited, and the CUs
// that stay busy in a half-empty round run at a higher clock.
struct TailSplit {
  int along = 0;      // 0 = no split, 1 = along N, 2 = along M
  int64_t first = 0;  // columns (rows) of the 256 x 256 part
};

inline TailSplit tail_split_of(int64_t M, int64_t N, int cus) {
  TailSplit best;
  if (cus <= 0) cus = 256;
  const int64_t tm = (M + 255) / 256, tn = (N + 255) / 256;
  const double whole = (double)((tm * tn + cus - 1) / cus);
  double best_cost = whole * 0.93;  // a split has to save at least 7 %
  for (int along = 1; along <= 2; ++along) {
    const int64_t cut_tiles = along == 1 ? tn : tm, other = along == 1 ? tm : tn;
    const int64_t extent = along == 1 ? N : M;
    // the largest number of tile columns (rows) that gives whole rounds
    for (int64_t t1 = cut_tiles - 1; t1 >= 1; --t1) {
      if ((t1 * other) % cus != 0) continue;
      const int64_t rest = extent - t1 * 256;
      const int64_t rest128 = (rest + 127) / 128 * (((along == 1 ? M : N) + 127) / 128);
      const double cost = (double)(t1 * other / cus) +
                          0.55 * (double)((rest128 + 2 * cus - 1) / (2 * cus));
      if (cost < best_cost) {
        best_cost = cost;
        best.along = along;
        best.first = t1 * 256;
      }
      break;
    }
  }
  return best;
}

// the two sub-problems of a split: `part1` the first `ts.first` columns (rows), `part2` the rest
inline void tail_parts(const GemmArgs& a, const TailSplit& ts, int out_bytes, GemmArgs* part1,
                       GemmArgs* part2) {
  *part1 = a;
  *part2 = a;
  if (ts.along == 1) {
    part1->N = (int32_t)ts.first;
    part2->N = a.N - (int32_t)ts.first;
    part2->B = a.B + ts.first * a.ldb_bytes;
    if (a.mx_b) part2->mx_b = a.mx_b + ts.first * a.mx_ld;
    if (a.bias) part2->bias = a.bias + ts.first;
    part2->C = (uint8_t*)a.C + ts.first * out_bytes;
  } else {
    part1->M = (int32_t)ts.first;
    part2->M = a.M - (int32_t)ts.first;
    part2->A = a.A + ts.first * a.lda_bytes;
    if (a.mx_a) part2->mx_a = a.mx_a + ts.first * a.mx_ld;
    part2->C = (uint8_t*)a.C + ts.first * a.ldc * out_bytes;
  }
  part1->tiles_m = (part1->M + 255) / 256;
  part1->tiles_n = (part1->N + 255) / 256;
  part2->tiles_m = (part2->M + 127) / 128;
  part2->tiles_n = (part2->N + 127) / 128;
  // the tile order is a property of each part's own tile grid (see map_tile)
  part1->group_m = (part1->tiles_m % 8 == 0 && part1->tiles_n % 32 == 0) ? -1 : 8;
  part2->group_m = (part2->tiles_m % 8 == 0 && part2->tiles_n % 32 == 0) ? -1 : 8;
}

// KIND 0: 16-bit operands, 1: fp8, 2: MXFP4
template <int KIND, int DT, int OUT>
int launch_stream_tail(const GemmArgs& a, int grid, hipStream_t s) {
  (void)grid;
  const TailSplit ts = tail_split_of(a.M, a.N, device_cus());
  if (ts.along == 0) return (int)hipErrorInvalidValue;
  GemmArgs p1, p2;
  tail_parts(a, ts, OUT == ASTERGEMM_F32 ? 4 : 2, &p1, &p2);
  const int g1 = p1.tiles_m * p1.tiles_n, g2 = p2.tiles_m * p2.tiles_n;
  int rc;
  if constexpr (KIND == 0) {
    if ((rc = launch_stream<DT, OUT, 256, 256, 2, 4>(p1, g1, s)) != 0) return rc;
    return launch_stream<DT, OUT, 128, 128, 2, 2>(p2, g2, s);
  } else if constexpr (KIND == 1) {
    // the whole rounds as a tile walk where its conditions hold (see launch_stream8_walk)
    const bool walk = p1.M % 256 == 0 && p1.N % 256 == 0 && p1.tail_granules == 0 &&
                      p1.ksteps >= 4 && g1 > device_cus();
    rc = walk ? launch_stream8_walk<DT, OUT>(p1, g1, s) : launch_stream8<DT, OUT, 256, 256, 2, 4>(p1, g1, s);
    if (rc != 0) return rc;
    return launch_stream8<DT, OUT, 128, 128, 2, 2>(p2, g2, s);
  } else {
    // the whole rounds as a tile walk where its conditions hold (see launch_stream4_walk)
    const bool walk = p1.ksteps % 4 == 0 && p1.M % 256 == 0 && p1.N % 256 == 0 && g1 > device_cus();
    rc = walk ? launch_stream4_walk<DT, OUT>(p1, g1, s) : launch_stream4<DT, OUT, 256, 256, 2, 4>(p1, g1, s);
    if (rc != 0) return rc;
    return launch_stream4<DT, OUT, 128, 128, 2, 2>(p2, g2, s);
  }
}

const char* check_stream_tail(const astergemm_config& c) {
  if (c.dtype_ab == ASTERGEMM_MXFP4) {
    if (const char* why = check_stream4(c)) return why;
  } else if (const char* why = check_stream(c)) {
    return why;
  }
  if (tail_split_of(c.M, c.N, device_cus()).along == 0)
    return "no cut along M or N gives whole rounds of 256 x 256 tiles plus a cheaper rest";
  return nullptr;
}

int grid_stream_tail(const astergemm_config& c, int cus) {
  const TailSplit ts = tail_split_of(c.M, c.N, cus);
  if (ts.along == 0) return (int)(((c.M + 255) / 256) * ((c.N + 255) / 256));
  const int64_t m1 = ts.along == 2 ? ts.first : c.M, n1 = ts.along == 1 ? ts.first : c.N;
  const int64_t m2 = ts.along == 2 ? c.M - ts.first : c.M, n2 = ts.along == 1 ? c.N - ts.first : c.N;
  int64_t g1 = ((m1 + 255) / 256) * ((n1 + 255) / 256);
  // MXFP4, fp8: the whole rounds run as a tile walk, one workgroup per CU (see launch_stream_tail)
  if (cus <= 0) cus = 256;
  if (c.dtype_ab == ASTERGEMM_MXFP4 && c.K % 1024 == 0 && m1 % 256 == 0 && n1 % 256 == 0 && g1 > cus)
    g1 = cus;
  if (c.dtype_ab == ASTERGEMM_FP8_E4M3 && c.K % 128 == 0 && c.K >= 512 && m1 % 256 == 0 &&
      n1 % 256 == 0 && g1 > cus)
    g1 = cus;
  return (int)(g1 + ((m2 + 127) / 128) * ((n2 + 127) / 128));
}

// rank 3: preferred over the plain 256 x 256 kernel wherever its check passes
#define AG_STREAM_TAIL(name, KIND, DT, OUT, WM, WN, LDS, FUNC)                   \
  Variant {                                                                      \
    name, ASTERGEMM_KERNEL_TILE, DT, OUT, 256, 256, kRowBytes, WM, WN, 3, 3, LDS, \
        (const void*)FUNC<DT, OUT, 256, 256, WM, WN>, launch_stream_tail<KIND, DT, OUT>, \
        check_stream_tail, ASTERGEMM_OPERAND_LDS, nullptr, grid_stream_tail      \
  }
#define AG_STREAM_TAIL_SET(prefix, KIND, DT, WM, WN, LDS, FUNC)                  \
  AG_STREAM_TAIL(prefix "_bf16", KIND, DT, ASTERGEMM_BF16, WM, WN, LDS, FUNC),   \
      AG_STREAM_TAIL(prefix "_f32", KIND, DT, ASTERGEMM_F32, WM, WN, LDS, FUNC), \
      AG_STREAM_TAIL(prefix "_f16", KIND, DT, ASTERGEMM_F16, WM, WN, LDS, FUNC)

#define AG_STREAM_SET(prefix, DT)                                                      \
  AG_STREAM(prefix "_256x256_w2x4_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 4),          \
      AG_STREAM(prefix "_256x256_w2x4_f32", DT, ASTERGEMM_F32, 256, 256, 2, 4),        \
      AG_STREAM(prefix "_256x256_w2x4_f16", DT, ASTERGEMM_F16, 256, 256, 2, 4),        \
      AG_STREAM(prefix "_256x256_w2x2_bf16", DT, ASTERGEMM_BF16, 256, 256, 2, 2),        \
      AG_STREAM(prefix "_128x128_w2x2_bf16", DT, ASTERGEMM_BF16, 128, 128, 2, 2),        \
      AG_STREAM(prefix "_128x128_w2x2_f32", DT, ASTERGEMM_F32, 128, 128, 2, 2),          \
      AG_STREAM(prefix "_128x128_w2x2_f16", DT, ASTERGEMM_F16, 128, 128, 2, 2)

// The table is compiled in four parts (this file once per AG_STREAM_PART: bf16, fp8, MXFP4 and f16
// operands), so that the parts build side by side and work on one family recompiles one part.
#ifndef AG_STREAM_PART
#error "compile with -DAG_STREAM_PART=0, 1, 2 or 3"
#endif

const Variant kStreamVariants[] = {
#if AG_STREAM_PART == 0 || AG_STREAM_PART == 3
#if AG_STREAM_PART == 0
#define AG_P16 ASTERGEMM_BF16
#define AG_N16(x) x "_bf16"
#else
#define AG_P16 ASTERGEMM_F16
#define AG_N16(x) x "_f16"
#endif
    AG_STREAM_SET(AG_N16("stream"), AG_P16),
    AG_STREAM_SPLITK_SET(AG_N16("splitk"), 0, AG_P16, 5 * 128 * kRowBytes, gemm_stream_splitk_kernel),
    AG_STREAMDB(AG_N16("streamdb") "_256x256_w2x4_bf16", AG_P16, ASTERGEMM_BF16, 5, 5, 2, 2),
    AG_STREAMDB(AG_N16("streamdb") "_256x256_w2x4_f32", AG_P16, ASTERGEMM_F32, 5, 5, 2, 2),
    AG_STREAMDB(AG_N16("streamdb") "_256x256_w2x4_f16", AG_P16, ASTERGEMM_F16, 5, 5, 2, 2),
    AG_STREAMDB(AG_N16("streamdb") "_128x256_w1x4_bf16", AG_P16, ASTERGEMM_BF16, 5, 5, 1, 1),
    AG_STREAMDB(AG_N16("streamdb") "_128x256_w1x4_f32", AG_P16, ASTERGEMM_F32, 5, 5, 1, 1),
    AG_STREAMDB(AG_N16("streamdb") "_128x256_w1x4_f16", AG_P16, ASTERGEMM_F16, 5, 5, 1, 1),
    AG_STREAM_TAIL_SET(AG_N16("stream") "_256x256_w2x4_tail128", 0, AG_P16, 2, 4, 5 * 256 * kRowBytes,
                       gemm_stream_kernel),
    AG_STREAM_RING9_SET(AG_N16("stream"), AG_P16),
    AG_DIRECTAB_SET(AG_N16("directab"), AG_P16),
#elif AG_STREAM_PART == 1
    AG_STREAM_SPLITK_SET("splitk_fp8", 1, ASTERGEMM_FP8_E4M3, 5 * 128 * kRowBytes,
                         gemm_stream8_splitk_kernel),
    AG_STREAM_TAIL_SET("stream_fp8_256x256_w2x4_tail128", 1, ASTERGEMM_FP8_E4M3, 2, 4,
                       5 * 256 * kRowBytes, gemm_stream8_kernel),
    AG_STREAM8("stream_fp8_256x256_w2x4_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_STREAM8("stream_fp8_256x256_w2x4_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_STREAM8("stream_fp8_256x256_w2x4_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_STREAM8_WALK("stream_fp8_256x256_w2x4_walk_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16, 3),
    AG_STREAM8_WALK("stream_fp8_256x256_w2x4_walk_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32, 3),
    AG_STREAM8_WALK("stream_fp8_256x256_w2x4_walk_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16, 3),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_STREAM8_128("stream_fp8_128x128_w2x2_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
    AG_STREAM8DB("streamdb_fp8_128x256_w1x4_bf16", ASTERGEMM_FP8_E4M3, ASTERGEMM_BF16),
    AG_STREAM8DB("streamdb_fp8_128x256_w1x4_f32", ASTERGEMM_FP8_E4M3, ASTERGEMM_F32),
    AG_STREAM8DB("streamdb_fp8_128x256_w1x4_f16", ASTERGEMM_FP8_E4M3, ASTERGEMM_F16),
#else
    AG_STREAM_SPLITK_SET("splitk_mxfp4", 2, ASTERGEMM_MXFP4, 4 * 128 * kRowBytes + 4 * 128 * 16,
                         gemm_stream4_splitk_kernel),
    AG_STREAM_TAIL_SET("stream_mxfp4_256x256_w2x4_tail128", 2, ASTERGEMM_MXFP4, 2, 4,
                       4 * 256 * kRowBytes + 4 * 256 * 16, gemm_stream4_kernel),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_STREAM4("stream_mxfp4_256x256_w2x2_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
    AG_STREAM4_W8("stream_mxfp4_256x256_w2x4_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16, 2),
    AG_STREAM4_W8("stream_mxfp4_256x256_w2x4_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32, 2),
    AG_STREAM4_W8("stream_mxfp4_256x256_w2x4_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16, 2),
    AG_STREAM4_WALK("stream_mxfp4_256x256_w2x4_walk_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_STREAM4_WALK("stream_mxfp4_256x256_w2x4_walk_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_STREAM4_WALK("stream_mxfp4_256x256_w2x4_walk_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16, false),
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32, false),
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16, false),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32),
    AG_STREAM4_128("stream_mxfp4_128x128_w2x2_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16),
    // the same with A's e8m0 plane in lane order (mx_a_layout = ASTERGEMM_MX_LANES128)
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_sal_bf16", ASTERGEMM_MXFP4, ASTERGEMM_BF16, true),
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_sal_f32", ASTERGEMM_MXFP4, ASTERGEMM_F32, true),
    AG_STREAM4DB("streamdb_mxfp4_128x256_w1x4_sal_f16", ASTERGEMM_MXFP4, ASTERGEMM_F16, true),
#endif
};

}  // namespace

#define AG_CAT_(a, b) a##b
#define AG_CAT(a, b) AG_CAT_(a, b)
const Variant* AG_CAT(stream_variants_part, AG_STREAM_PART)(int* count) {
  *count = (int)(sizeof(kStreamVariants) / sizeof(kStreamVariants[0]));
  return kStreamVariants;
}

#if AG_STREAM_PART == 0
const Variant* stream_variants_part1(int* count);
const Variant* stream_variants_part2(int* count);
const Variant* stream_variants_part3(int* count);

// the four parts as one table: bf16, f16, fp8, MXFP4
static const std::vector<Variant>& all_stream_variants() {
  static const std::vector<Variant> all = [] {
    std::vector<Variant> v;
    int n = 0;
    const Variant* p = stream_variants_part0(&n);
    v.insert(v.end(), p, p + n);
    p = stream_variants_part3(&n);
    v.insert(v.end(), p, p + n);
    p = stream_variants_part1(&n);
    v.insert(v.end(), p, p + n);
    p = stream_variants_part2(&n);
    v.insert(v.end(), p, p + n);
    return v;
  }();
  return all;
}
int num_stream_variants() { return (int)all_stream_variants().size(); }
const Variant* stream_variants() { return all_stream_variants().data(); }
#endif

}  // namespace astergemm
