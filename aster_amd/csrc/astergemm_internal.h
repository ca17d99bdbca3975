// Internal declarations shared by the HIP translation units of libastergemm.
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "astergemm.h"

namespace astergemm {

// Arguments of every GEMM kernel (passed by value as one kernarg struct).
struct GemmArgs {
  const uint8_t* A;      // [M, lda_bytes]
  const uint8_t* B;      // [N, ldb_bytes]
  void* C;               // [M, ldc] elements of the output type
  const float* scale_a;  // per-tensor scales (device) or nullptr
  const float* scale_b;
  const float* bias;     // [N] or nullptr
  const uint8_t* mx_a;   // e8m0 [M, mx_ld] or nullptr
  const uint8_t* mx_b;   // e8m0 [N, mx_ld]
  int64_t lda_bytes, ldb_bytes;
  int64_t ldc;           // elements
  int32_t mx_ld;         // bytes per row of the e8m0 planes (= K/32)
  int32_t M, N, K;       // K in elements
  int32_t ksteps;        // K-loop trip count (128 bytes of a row per step)
  int32_t tail_granules; // valid 16-byte granules of the last step, 0 = all 8
  int32_t tiles_m, tiles_n;
  int32_t group_m;       // tile rows per rasterisation group; < 0: band order (see map_tile)
  int32_t split_k;       // skinny path: K slices per output row block
  float* workspace;      // fp32 partials [split_k][M][N] when a row is cut into K ranges; set by
                         // the caller of a launcher = use this buffer, null = the library's own
};

// Bytes of one operand row covering `k` elements.
__host__ __device__ inline int64_t row_bytes(int dtype, int64_t k) {
  switch (dtype) {
    case ASTERGEMM_F16:
    case ASTERGEMM_BF16: return k * 2;
    case ASTERGEMM_FP8_E4M3: return k;
    case ASTERGEMM_MXFP4: return k / 2;
    default: return k * 4;
  }
}

inline int out_elt_bytes(int dtype) { return dtype == ASTERGEMM_F32 ? 4 : 2; }

// One entry of the variant table (filled in by gemm_tile.hip / gemm_skinny.hip).
struct Variant {
  const char* name;
  int family;
  int dtype_ab;      // -1 = any 16-bit float (F16 and BF16 share a kernel body)
  int dtype_c;
  int tile_m, tile_n, tile_k_bytes;
  int waves_m, waves_n;
  int stages;
  int rank;          // preference among variants of equal tile size (higher wins)
  int lds_bytes;
  const void* func;  // device function symbol, for hipFuncGetAttributes
  // Launches the kernel; returns a hipError_t as int.
  int (*launch)(const GemmArgs& a, int grid, hipStream_t s);
  // Host-side shape check: nullptr when ok, else a reason.
  const char* (*check)(const astergemm_config& c);
  // B operand form this variant reads (astergemm_operand_path); plain row-major by default.
  int operand_path = 0;
  // K ranges the launcher cuts the rows of this problem into (1 = none): the launch then needs
  // splits * M * N * 4 bytes of fp32 workspace.  nullptr = never splits.
  int (*splits)(const astergemm_config& c) = nullptr;
  // Grid the launcher uses when it is not the number of output tiles (persistent kernels);
  // `cus` = compute units of the current device.  nullptr = tiles (times splits).
  int (*grid)(const astergemm_config& c, int cus) = nullptr;
  // Layout of A's e8m0 plane this variant reads (astergemm_mx_layout); row-major by default.
  int mx_a_layout = 0;
};

// Compute units of the current device (0 when there is none), cached per device ordinal.
int device_cus();

// State of the launcher call in progress on this thread, set by the entry points in
// astergemm_api.hip: the stream the kernels go to, and whether this is astergemm_prepare (every
// one-time step of the launcher runs, the kernels themselves are not launched).
struct LaunchContext {
  hipStream_t stream = nullptr;
  bool prepare_only = false;
};
LaunchContext& launch_context();

// Every GEMM kernel launch of the library goes through this macro.
#define AG_LAUNCH_KERNEL(...)                                                   \
  do {                                                                          \
    if (!::astergemm::launch_context().prepare_only) hipLaunchKernelGGL(__VA_ARGS__); \
  } while (0)

// Raises a kernel's dynamic-LDS limit once per device; `devs` is a static of the launcher with
// one bit per device ordinal.  Returns 0 or a hipError_t.  Changing a function attribute is not
// a stream operation: when the kernel's first launch on a device arrives while the stream is
// being captured into a graph, the launcher refuses (hipErrorStreamCaptureUnsupported) instead
// of touching the runtime from inside the capture; astergemm_prepare does this step ahead of time.
inline int lds_attr_once(std::atomic<uint64_t>& devs, const void* func, int lds_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return (int)hipGetLastError();
  const uint64_t bit = (uint64_t)1 << (dev & 63);
  if (devs.load(std::memory_order_acquire) & bit) return 0;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(launch_context().stream, &st) != hipSuccess ||
      st != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return (int)hipErrorStreamCaptureUnsupported;
  }
  const hipError_t e = hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e != hipSuccess) return (int)e;
  devs.fetch_or(bit, std::memory_order_release);
  return 0;
}

int num_tile_variants();
const Variant* tile_variants();
int num_stream_variants();
const Variant* stream_variants();
int num_skinny_variants();
const Variant* skinny_variants();

// K ranges for `tiles` output tiles and rows of `ksteps` 128-byte steps: the largest divisor
// S of ksteps (2..16, ranges of at least 8 steps) with tiles * S <= 256, one workgroup per CU
// of a 256-CU part; 0 if there is none.  Measured on MI355X (bf16 and fp8, 32 to 128 tiles,
// 64 to 224 steps): filling the CUs once beats filling them twice by 5-15 % (32 tiles x 224
// steps: 32.3 us with 8 ranges, 37.4 with 16, 61.3 with 2; unsplit 103), and split K is ahead
// of the best unsplit kernel wherever this returns a value and rows are 8 KiB or longer.
inline int stream_split_of(int64_t tiles, int64_t ksteps, bool even_ranges = false) {
  int best = 0;
  for (int S = 2; S <= 16; ++S) {
    if (ksteps % S != 0 || ksteps / S < 8 || tiles * S > 256) continue;
    if (even_ranges && (ksteps / S) % 2 != 0) continue;
    best = S;
  }
  // ranges of 64 steps and more: twice as many, two workgroups per CU, is ahead (128 tiles x
  // 224 steps: 64.8 us with 4 ranges, 67-77 with 2)
  if (best && ksteps / best >= 64 && best * 2 <= 16 && ksteps % (best * 2) == 0 &&
      tiles * best * 2 <= 512 && !(even_ranges && (ksteps / (best * 2)) % 2 != 0))
    best *= 2;
  return best;
}

// Split-K support shared by the decode and the tile kernels (gemm_skinny.hip): the fp32
// workspace of a (device, stream), and the kernel that adds `splits` planes [M][N] of
// a.workspace in index order, applies a's scales and bias and stores a.C in `out_dtype`.
int splitk_workspace_for(size_t bytes, hipStream_t stream, float** out);
// Frees the workspace of a (synchronised) stream that is about to be destroyed.
void splitk_workspace_release(hipStream_t stream);
int splitk_reduce(int out_dtype, const GemmArgs& a, int splits, hipStream_t stream);

void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what, const char* file, int line);

#define AG_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t _e = (expr);                                            \
    if (_e != hipSuccess) return hip_fail(_e, #expr, __FILE__, __LINE__); \
  } while (0)

}  // namespace astergemm
