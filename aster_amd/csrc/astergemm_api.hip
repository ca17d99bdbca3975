// Host side of libastergemm: variant selection, launch, event timing, and the
// thin HIP runtime seam.  Everything exported is declared in include/astergemm.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

#include "astergemm_internal.h"

namespace astergemm {

static thread_local char g_err[512] = "";
static thread_local int g_choose_rc = 0;  // why choose() returned nullptr

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// Same message shape as the reference's HIP error exceptions
// ("file:line - hipGetErrorString", python/lib/RuntimeModule.cpp:126-134).
int hip_fail(hipError_t e, const char* what, const char* file, int line) {
  set_error("%s:%d - %s (%s)", file, line, hipGetErrorString(e), what);
  return ASTERGEMM_EHIP;
}

LaunchContext& launch_context() {
  static thread_local LaunchContext ctx;
  return ctx;
}

// Sets the launch context for the launcher calls of one entry point and clears it on return.
struct LaunchScope {
  explicit LaunchScope(void* stream, bool prepare_only = false) {
    launch_context().stream = (hipStream_t)stream;
    launch_context().prepare_only = prepare_only;
  }
  ~LaunchScope() { launch_context() = LaunchContext{}; }
};

// The error text of a launcher's status; a first launch refused inside a capture says what to do.
int launch_fail(int e, const char* name, const char* file, int line) {
  if ((hipError_t)e == hipErrorStreamCaptureUnsupported) {
    set_error("%s: the first launch of a kernel on a device sets a function attribute, which cannot "
              "happen while the stream is being captured; call astergemm_prepare(cfg) (or launch "
              "once eagerly) before the capture", name);
    return ASTERGEMM_EHIP;
  }
  return hip_fail((hipError_t)e, name, file, line);
}

// Compute units of the current device (0 when there is none), cached per device ordinal.
int device_cus() {
  static std::atomic<int> cus[64];
  static std::atomic<bool> init{false};
  static std::mutex init_mutex;
  if (!init.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(init_mutex);
    if (!init.load()) {
      for (auto& c : cus) c.store(-1);
      init.store(true, std::memory_order_release);
    }
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  std::atomic<int>& slot = cus[dev & 63];
  int n = slot.load();
  if (n < 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) == hipSuccess)
      n = prop.multiProcessorCount;
    else
      (void)hipGetLastError(), n = 0;
    slot.store(n);
  }
  return n;
}

namespace {

int total_variants() {
  return num_tile_variants() + num_stream_variants() + num_skinny_variants();
}

const Variant* variant_at(int index) {
  if (index < 0) return nullptr;
  if (index < num_tile_variants()) return tile_variants() + index;
  index -= num_tile_variants();
  if (index < num_stream_variants()) return stream_variants() + index;
  index -= num_stream_variants();
  if (index < num_skinny_variants()) return skinny_variants() + index;
  return nullptr;
}

bool variant_matches_types(const Variant& v, const astergemm_config& c) {
  return v.dtype_ab == c.dtype_ab && v.dtype_c == c.dtype_c && v.operand_path == c.operand_path &&
         v.mx_a_layout == c.mx_a_layout;
}

const char* validate_problem(const astergemm_config& c) {
  if (c.M < 0 || c.N < 0 || c.K <= 0) return "M, N must be >= 0 and K > 0";
  if (c.M > INT32_MAX || c.N > INT32_MAX || c.K > INT32_MAX) return "dimension exceeds int32";
  if (c.dtype_ab < ASTERGEMM_F16 || c.dtype_ab > ASTERGEMM_MXFP4) return "bad dtype_ab";
  if (c.dtype_c != ASTERGEMM_F32 && c.dtype_c != ASTERGEMM_BF16 && c.dtype_c != ASTERGEMM_F16)
    return "dtype_c must be F32, BF16 or F16";
  if (c.scale_mode < ASTERGEMM_SCALE_NONE || c.scale_mode > ASTERGEMM_SCALE_MX32)
    return "bad scale_mode";
  if (c.operand_path < ASTERGEMM_OPERAND_LDS || c.operand_path > ASTERGEMM_OPERAND_DIRECT_AB)
    return "bad operand_path";
  if (c.mx_a_layout != ASTERGEMM_MX_ROWS &&
      (c.mx_a_layout != ASTERGEMM_MX_LANES128 || c.dtype_ab != ASTERGEMM_MXFP4))
    return "bad mx_a_layout (LANES128 goes with MXFP4 operands)";
  if ((c.dtype_ab == ASTERGEMM_MXFP4) != (c.scale_mode == ASTERGEMM_SCALE_MX32))
    return "MXFP4 operands and SCALE_MX32 go together";
  if (c.dtype_ab == ASTERGEMM_MXFP4 && c.K % 32 != 0) return "MXFP4 needs K % 32 == 0";
  const int64_t lda = c.lda ? c.lda : c.K, ldb = c.ldb ? c.ldb : c.K, ldc = c.ldc ? c.ldc : c.N;
  if (lda < c.K || ldb < c.K || ldc < c.N) return "leading dimension smaller than the row";
  if (row_bytes(c.dtype_ab, lda) % 16 != 0 || row_bytes(c.dtype_ab, ldb) % 16 != 0)
    return "row pitch of A and B must be a multiple of 16 bytes";
  if (row_bytes(c.dtype_ab, lda) * 256 >= (int64_t)1 << 31 ||
      row_bytes(c.dtype_ab, ldb) * 256 >= (int64_t)1 << 31)
    return "row pitch too large for 32-bit tile offsets";
  return nullptr;
}

// The last selections of this thread: a serving loop calls the entry points with the same few
// configs over and over, and walking the variant table with its shape checks costs about 5 us of
// host time a call.  A selection depends on the config and, through the CU count, on the device.
struct ChoiceCacheEntry {
  astergemm_config cfg;
  int dev;
  int index;
};
constexpr int kChoiceCache = 16;
thread_local ChoiceCacheEntry g_choice_cache[kChoiceCache];
thread_local int g_choice_cache_used = 0, g_choice_cache_next = 0;

int current_device_or_minus_one() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    dev = -1;
  }
  return dev;
}

const Variant* choose_uncached(const astergemm_config& c, int* index_out);

// Picks the variant for cfg; on failure returns nullptr with the error set.
const Variant* choose(const astergemm_config& c, int* index_out) {
  const int dev = current_device_or_minus_one();
  for (int i = 0; i < g_choice_cache_used; ++i) {
    const ChoiceCacheEntry& e = g_choice_cache[i];
    if (e.dev == dev && memcmp(&e.cfg, &c, sizeof(c)) == 0) {
      if (index_out) *index_out = e.index;
      return variant_at(e.index);
    }
  }
  int index = -1;
  const Variant* v = choose_uncached(c, &index);
  if (!v) return nullptr;  // refusals are not remembered: the message is made again
  ChoiceCacheEntry& e = g_choice_cache[g_choice_cache_next];
  memcpy(&e.cfg, &c, sizeof(c));
  e.dev = dev;
  e.index = index;
  g_choice_cache_next = (g_choice_cache_next + 1) % kChoiceCache;
  if (g_choice_cache_used < kChoiceCache) ++g_choice_cache_used;
  if (index_out) *index_out = index;
  return v;
}

const Variant* choose_uncached(const astergemm_config& c, int* index_out) {
  g_choose_rc = ASTERGEMM_ENOTSUP;
  if (const char* why = validate_problem(c)) {
    set_error("astergemm: invalid config: %s", why);
    g_choose_rc = ASTERGEMM_EINVAL;
    return nullptr;
  }
  if (c.variant != 0) {
    const Variant* v = variant_at(c.variant - 1);
    if (!v || !variant_matches_types(*v, c)) {
      set_error("astergemm: variant %d does not exist for these dtypes", c.variant);
      return nullptr;
    }
    if (const char* why = v->check(c)) {
      set_error("astergemm: variant %s: %s", v->name, why);
      return nullptr;
    }
    if (index_out) *index_out = c.variant - 1;
    return v;
  }
  const bool is16 = c.dtype_ab == ASTERGEMM_F16 || c.dtype_ab == ASTERGEMM_BF16;
  int family = c.family;
  if (family == ASTERGEMM_KERNEL_AUTO)
    family = ((is16 && c.M <= 64 && c.K % 32 == 0) ||
              // fp8 / MXFP4: only the resident-activation kernels, whose waves take whole
              // slices of a row in at most 16 K ranges
              ((c.dtype_ab == ASTERGEMM_FP8_E4M3 || c.dtype_ab == ASTERGEMM_MXFP4) && c.M <= 64 &&
               c.K >= 4096 &&
               ((c.K % 512 == 0 && c.K <= 16 * 4096) || (c.K % 8192 == 0 && c.K <= 16 * 8192))))
                 ? ASTERGEMM_KERNEL_SKINNY
                 : ASTERGEMM_KERNEL_TILE;
  // 32 < M <= 64 on rows of more than 32 KiB: the decode kernel's K ranges of 4 KiB leave more
  // partial sums than split K on the 128 x 128 kernel (bf16 64x8192x28672: 107 against 94 us;
  // 64x4096x28672 level at 57.5 against 58.5); up to 32 KiB the decode kernel is ahead
  // (64x8192x16384: 60 against 81 us, 64x14336x8192: 53 against 63, fp8 64x8192x28672: 56
  // against 60)
  if (c.family == ASTERGEMM_KERNEL_AUTO && family == ASTERGEMM_KERNEL_SKINNY && c.M > 32 &&
      (is16 || c.dtype_ab == ASTERGEMM_FP8_E4M3) && row_bytes(c.dtype_ab, c.K) > 32768) {
    for (int i = 0; i < total_variants(); ++i) {
      const Variant* v = variant_at(i);
      if (v->family == ASTERGEMM_KERNEL_TILE && v->rank == 4 && variant_matches_types(*v, c) &&
          v->check(c) == nullptr) {
        family = ASTERGEMM_KERNEL_TILE;
        break;
      }
    }
  }
  if (c.operand_path == ASTERGEMM_OPERAND_DIRECT_B) family = ASTERGEMM_KERNEL_SKINNY;
  if (c.operand_path == ASTERGEMM_OPERAND_DIRECT_B_K8) family = ASTERGEMM_KERNEL_TILE;
  if (c.operand_path == ASTERGEMM_OPERAND_DIRECT_AB) family = ASTERGEMM_KERNEL_TILE;

  const Variant* best = nullptr;
  int best_index = -1;
  const char* last_why = nullptr;  // reason given by the first variant that refused
  for (int i = 0; i < total_variants(); ++i) {
    const Variant* v = variant_at(i);
    if (v->family != family || !variant_matches_types(*v, c)) continue;
    if (const char* why = v->check(c)) {
      if (!last_why) last_why = why;
      continue;
    }
    if (c.wg_tile_m && c.wg_tile_m != v->tile_m) continue;
    if (c.wg_tile_n && c.wg_tile_n != v->tile_n) continue;
    if (c.waves_m && c.waves_m != v->waves_m) continue;
    if (c.waves_n && c.waves_n != v->waves_n) continue;
    bool better = false;
    if (!best) {
      better = true;
    } else if (family == ASTERGEMM_KERNEL_SKINNY) {
      // among the variants that cover M: the resident-activation kernels (rank >= 2) by
      // rank, otherwise the smallest activation tile, rank breaking ties
      const bool fits = v->tile_m >= c.M, best_fits = best->tile_m >= c.M;
      if (fits != best_fits) better = fits;
      else if (!fits) better = v->tile_m > best->tile_m;
      else if (v->rank >= 2 || best->rank >= 2) better = v->rank > best->rank;
      else better = v->tile_m < best->tile_m || (v->tile_m == best->tile_m && v->rank > best->rank);
    } else if (c.operand_path == ASTERGEMM_OPERAND_DIRECT_AB) {
      // both operands straight into registers: the 256 x 256 form (128 x 128 per wave, half the
      // L1 requests per MFMA) once it nearly fills the chip, else the 128 x 256 form (bf16 8192^3
      // 776 against 950 us, 4096^3 125 against 144, 4096 x 14336 x 4096 456 against 495;
      // 2048^3, 64 tiles: 52.7 against 36.0)
      auto wgs = [&](const Variant* x) {
        return ((c.M + x->tile_m - 1) / x->tile_m) * ((c.N + x->tile_n - 1) / x->tile_n);
      };
      const Variant* big = v->tile_m > best->tile_m ? v : best;
      const Variant* want = wgs(big) >= 200 ? big : (big == v ? best : v);
      better = want == v;
    } else if (c.operand_path == ASTERGEMM_OPERAND_DIRECT_B_K8) {
      // pre-shuffled B straight into operands: the 128 x 256 form (four waves side by side, two
      // workgroups per CU, no B line fetched by two waves) is ahead of the 256 x 256 form on
      // every shape measured (8192^3 744 against 757 us, 16384 x 16384 x 4096 1508 against 1566,
      // 4096 x 14336 x 4096 336 against 370, 2048^3 29.5 against 45.5)
      better = v->tile_m < best->tile_m;
    } else {
      // Measured on MI355X (256 CUs): the 256 x 256 kernels (one workgroup per CU) win once
      // they nearly fill the chip; below that the 128 x 128 stream kernel (rank 2, two
      // workgroups per CU) from about 0.8 workgroups per CU on, else the largest tile that
      // still gives about two workgroups per CU; for tiny problems the smallest tile.
      auto wgs = [&](const Variant* x) {
        return ((c.M + x->tile_m - 1) / x->tile_m) * ((c.N + x->tile_n - 1) / x->tile_n);
      };
      // 256 x 256 from 220 workgroups on (bf16 1024 x 14336 x 4096, 224 tiles: 85.6 us against
      // 103.9 for 896 tiles of 128 x 128); already from 140 on when the last round of the
      // 128 x 128 stream kernel (512 workgroups fill the chip) would be less than about a
      // third full.  The 128 x 128 stream kernel from 200 workgroups on,
      // from 128 on when rows are long (8 KiB and more: few prologues per byte streamed).
      const int64_t g128 = ((c.M + 127) / 128) * ((c.N + 127) / 128);
      const bool ragged_128 = g128 > 512 && g128 % 512 != 0 && g128 % 512 < 180;
      const int thr256 = ragged_128 ? 140 : 220;
      // MXFP4: the generic tile kernels are weak next to the stream kernels, so the 128 x 128
      // stream kernel from 16 workgroups on when K >= 4096, and instead of the 256 x 256 one
      // (long prologue: two K-steps and their scales) when K < 4096
      const bool fp4 = c.dtype_ab == ASTERGEMM_MXFP4;
      const int thr128s = fp4 ? (c.K >= 4096 ? 16 : 200)
                              : (row_bytes(c.dtype_ab, c.K) >= 8192 ? 128 : 200);
      auto tier = [&](const Variant* x) {
        const int area = x->tile_m * x->tile_n;
        // split K (rank 4) only passes its check where it was measured ahead of every
        // unsplit kernel: few output tiles, long rows
        if (x->rank == 4) return 3;
        // (not the tile walk and the whole-rounds form, rank 3, which pay that prologue once per
        // workgroup, from about two tiles of K = 2048 per CU on: 8192 x 8192 x 1024 51 against
        // 57 us, 16384 x 16384 x 1024 180 against 210, 8192 x 8192 x 2048 74 against 84,
        // 4096 x 8192 x 2048 42 against 45; below that level or behind: 4096 x 8192 x 1024 30.6
        // against 29.8, 4096 x 6144 x 1024 24.0 against 21.8)
        const bool walk_pays = x->rank == 3 && wgs(x) * c.K >= (int64_t)512 * 2048;
        if (area >= 256 * 256 && fp4 && c.K < 4096 && c.K % 512 == 0 && !walk_pays) return -1;
        if (area >= 256 * 256) return wgs(x) >= thr256 ? 2 : -1;
        return wgs(x) >= ((x->rank >= 2) ? thr128s : 448) ? 1 : 0;
      };
      const int tv = tier(v), tb = tier(best);
      const int area = v->tile_m * v->tile_n, best_area = best->tile_m * best->tile_n;
      if (tv != tb) better = tv > tb;
      else if (area != best_area) better = (tv >= 1) ? area > best_area : area < best_area;
      else better = v->rank > best->rank;
    }
    if (better) {
      best = v;
      best_index = i;
    }
  }
  if (!best) {
    set_error("astergemm: no kernel variant for this config (%s)",
              last_why ? last_why : "no variant with these dtypes");
    return nullptr;
  }
  if (family == ASTERGEMM_KERNEL_SKINNY && best->tile_m < c.M) {
    set_error("astergemm: skinny path covers M <= %d, got M=%lld", best->tile_m, (long long)c.M);
    return nullptr;
  }
  if (index_out) *index_out = best_index;
  return best;
}

// K ranges the launcher of `v` cuts this problem into, and the fp32 workspace that takes.
int splits_of(const Variant& v, const astergemm_config& c) { return v.splits ? v.splits(c) : 1; }
size_t workspace_need(const Variant& v, const astergemm_config& c) {
  const int S = splits_of(v, c);
  return S > 1 ? (size_t)S * (size_t)c.M * (size_t)c.N * sizeof(float) : 0;
}

int grid_of(const Variant& v, const astergemm_config& c) {
  if (v.grid) return v.grid(c, device_cus());
  if (v.family == ASTERGEMM_KERNEL_SKINNY) {
    const int blocks = (int)((c.N + v.tile_n - 1) / v.tile_n);
    // the resident-activation kernels (8 waves) are persistent: at most one workgroup per CU
    if (v.waves_n == 8 && device_cus() > 0 && blocks > device_cus()) return device_cus();
    return blocks;
  }
  const int64_t tiles = ((c.M + v.tile_m - 1) / v.tile_m) * ((c.N + v.tile_n - 1) / v.tile_n);
  return (int)(tiles * splits_of(v, c));  // split K: one copy of the tile grid per K range
}

int64_t algorithmic_bytes(const astergemm_config& c) {
  int64_t b = row_bytes(c.dtype_ab, c.K) * (c.M + c.N) + c.M * c.N * out_elt_bytes(c.dtype_c);
  if (c.scale_mode == ASTERGEMM_SCALE_MX32) b += (c.M + c.N) * (c.K / 32);
  if (c.scale_mode == ASTERGEMM_SCALE_TENSOR) b += 8;
  if (c.has_bias) b += c.N * 4;
  return b;
}

void describe(const Variant& v, int index, const astergemm_config& c, astergemm_kernel_info* o) {
  memset(o, 0, sizeof(*o));
  o->variant = index + 1;
  o->family = v.family;
  o->grid_x = grid_of(v, c);
  o->block_x = v.waves_m * v.waves_n * 64;
  o->lds_bytes = v.lds_bytes;
  o->wg_tile_m = v.tile_m;
  o->wg_tile_n = v.tile_n;
  const int eb2 = (int)row_bytes(c.dtype_ab, 2);  // bytes of two elements (fp4-safe)
  o->wg_tile_k = eb2 ? v.tile_k_bytes * 2 / eb2 : 0;
  o->waves_m = v.waves_m;
  o->waves_n = v.waves_n;
  o->pipeline_stages = v.stages;
  o->flops = 2 * c.M * c.N * c.K;
  o->bytes = algorithmic_bytes(c);
  snprintf(o->name, sizeof(o->name), "%s", v.name);
  hipFuncAttributes fa;
  if (hipFuncGetAttributes(&fa, v.func) == hipSuccess) {
    o->vgprs = fa.numRegs;
    o->agprs = 0;
  } else {
    (void)hipGetLastError();
  }
}

int build_args(const Variant& v, const astergemm_config& c, const astergemm_operands& ops,
               GemmArgs* a) {
  if (!ops.dA || !ops.dB || !ops.dC) {
    set_error("astergemm: dA, dB and dC must be non-null");
    return ASTERGEMM_EINVAL;
  }
  if ((((uintptr_t)ops.dA) | ((uintptr_t)ops.dB)) & 15) {
    set_error("astergemm: dA and dB must be 16-byte aligned");
    return ASTERGEMM_EINVAL;
  }
  if (((uintptr_t)ops.dC) & 15) {
    set_error("astergemm: dC must be 16-byte aligned");
    return ASTERGEMM_EINVAL;
  }
  if (c.scale_mode == ASTERGEMM_SCALE_MX32 && (!ops.dMxA || !ops.dMxB)) {
    set_error("astergemm: SCALE_MX32 needs dMxA and dMxB");
    return ASTERGEMM_EINVAL;
  }
  if (c.mx_a_layout == ASTERGEMM_MX_LANES128 && (((uintptr_t)ops.dMxA) & 15)) {
    set_error("astergemm: dMxA in lane order must be 16-byte aligned");
    return ASTERGEMM_EINVAL;
  }
  if (c.scale_mode == ASTERGEMM_SCALE_MX32 && ((((uintptr_t)ops.dMxA) | ((uintptr_t)ops.dMxB)) & 7)) {
    set_error("astergemm: dMxA and dMxB must be 8-byte aligned");
    return ASTERGEMM_EINVAL;
  }
  if (c.scale_mode == ASTERGEMM_SCALE_TENSOR && (!ops.dScaleA || !ops.dScaleB)) {
    set_error("astergemm: SCALE_TENSOR needs dScaleA and dScaleB");
    return ASTERGEMM_EINVAL;
  }
  if (c.has_bias && !ops.dBias) {
    set_error("astergemm: has_bias set but dBias is null");
    return ASTERGEMM_EINVAL;
  }
  memset(a, 0, sizeof(*a));
  a->A = (const uint8_t*)ops.dA;
  a->B = (const uint8_t*)ops.dB;
  a->C = ops.dC;
  if (c.scale_mode == ASTERGEMM_SCALE_TENSOR) {
    a->scale_a = ops.dScaleA;
    a->scale_b = ops.dScaleB;
  }
  if (c.scale_mode == ASTERGEMM_SCALE_MX32) {
    a->mx_a = ops.dMxA;
    a->mx_b = ops.dMxB;
    a->mx_ld = (int32_t)(c.K / 32);
  }
  a->bias = c.has_bias ? ops.dBias : nullptr;
  a->lda_bytes = row_bytes(c.dtype_ab, c.lda ? c.lda : c.K);
  a->ldb_bytes = row_bytes(c.dtype_ab, c.ldb ? c.ldb : c.K);
  a->ldc = c.ldc ? c.ldc : c.N;
  a->M = (int32_t)c.M;
  a->N = (int32_t)c.N;
  a->K = (int32_t)c.K;
  a->ksteps = (int32_t)((row_bytes(c.dtype_ab, c.K) + 127) / 128);
  a->tail_granules = (int32_t)((row_bytes(c.dtype_ab, c.K) % 128) / 16);
  a->tiles_m = (int32_t)((c.M + v.tile_m - 1) / v.tile_m);
  a->tiles_n = (int32_t)((c.N + v.tile_n - 1) / v.tile_n);
  // tile order (map_tile): groups of 8 tile rows inside one contiguous run per XCD; where the
  // tile grid divides, band order instead (all XCDs on one band of 8 tile rows, 8 x 4 tiles per
  // XCD and round as before): 8192^3 bf16 +0.5 %, fp8 +1.3 %, 16384 x 16384 x 4096 fp8 +1.2 %,
  // MXFP4 +1.5 %, bf16 -0.1 %, same process
  a->group_m = (a->tiles_m % 8 == 0 && a->tiles_n % 32 == 0) ? -1 : 8;
  a->split_k = 1;
  // rows cut into K ranges: the caller's workspace when one is given, else the library's own
  if (ops.dWorkspace) {
    const size_t need = workspace_need(v, c);
    if (ops.workspace_bytes < need) {
      set_error("astergemm: workspace of %zu bytes given, %s needs %zu for this config",
                (size_t)ops.workspace_bytes, v.name, need);
      return ASTERGEMM_EINVAL;
    }
    if (((uintptr_t)ops.dWorkspace) & 15) {
      set_error("astergemm: dWorkspace must be 16-byte aligned");
      return ASTERGEMM_EINVAL;
    }
    if (need) a->workspace = (float*)ops.dWorkspace;
  }
  return 0;
}

// ---- the entry point that allocates nothing ------------------------------------------------
// Partial sums of rows cut into K ranges go to this array instead of an allocation.  Its name is
// a host-side handle only: the device address is looked up once per device.
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[ASTERGEMM_NOALLOC_SCRATCH_BYTES];
std::atomic<void*> g_scratch_ptr[64];

// Device address of `scratch` on the current device (looked up on first use), or nullptr with
// the error set.
void* scratch_address() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    hip_fail(hipGetLastError(), "hipGetDevice", __FILE__, __LINE__);
    return nullptr;
  }
  std::atomic<void*>& slot = g_scratch_ptr[dev & 63];
  void* p = slot.load(std::memory_order_acquire);
  if (!p) {
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      hip_fail(e, "hipGetSymbolAddress(scratch)", __FILE__, __LINE__);
      return nullptr;
    }
    slot.store(p, std::memory_order_release);
  }
  return p;
}

// Start / stop events of a timed region; destroyed on every return path.
struct EventPair {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t create() {
    hipError_t e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    return e;
  }
  ~EventPair() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
};
struct DeviceBuffer {
  void* ptr = nullptr;
  ~DeviceBuffer() {
    if (ptr) (void)hipFree(ptr);
  }
};

// Streams a scratch buffer so the next launch finds the last-level cache cold;
// the reference's flush kernel does the same with a global_load_dword loop
// (python/aster/execution/flush_llc.py:25-120).
__global__ void flush_llc_kernel(uint32_t* buf, size_t words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < words; i += stride) buf[i] = buf[i] + 1u;
}

}  // namespace
}  // namespace astergemm

using namespace astergemm;

extern "C" {

int astergemm_abi_version(void) { return ASTERGEMM_ABI_VERSION; }
const char* astergemm_last_error(void) { return g_err; }

int astergemm_variant_count(void) { return total_variants(); }

int astergemm_variant_info(int index, const astergemm_config* cfg, astergemm_kernel_info* out) {
  if (!cfg || !out) {
    set_error("astergemm_variant_info: null argument");
    return ASTERGEMM_EINVAL;
  }
  const Variant* v = variant_at(index);
  if (!v) {
    set_error("astergemm_variant_info: index %d out of range", index);
    return ASTERGEMM_EINVAL;
  }
  describe(*v, index, *cfg, out);
  return 0;
}

int astergemm_select(const astergemm_config* cfg, astergemm_kernel_info* out) {
  if (!cfg || !out) {
    set_error("astergemm_select: null argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  describe(*v, index, *cfg, out);
  return 0;
}

int astergemm_run(const astergemm_config* cfg, const astergemm_operands* ops, void* stream) {
  if (!cfg || !ops) {
    set_error("astergemm_run: null argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  if (cfg->M == 0 || cfg->N == 0) return 0;
  GemmArgs a;
  if (int rc = build_args(*v, *cfg, *ops, &a)) return rc;
  (void)hipGetLastError();  // the launchers report hipGetLastError(): drop what an earlier call left
  LaunchScope scope(stream);
  const int e = v->launch(a, grid_of(*v, *cfg), (hipStream_t)stream);
  if (e != 0) return launch_fail(e, v->name, __FILE__, __LINE__);
  return 0;
}

int astergemm_prepare(const astergemm_config* cfg) {
  if (!cfg) {
    set_error("astergemm_prepare: null argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  if (device_cus() <= 0) {
    set_error("astergemm_prepare: no HIP device");
    return ASTERGEMM_ENODEV;
  }
  void* scratch_ptr = scratch_address();
  if (!scratch_ptr) return ASTERGEMM_EHIP;
  if (cfg->M == 0 || cfg->N == 0) return 0;
  // The launcher runs with every one-time step (function attributes, cached device facts) and
  // without the kernel launches; the operands are never read.  Partial sums, where the config
  // has any, point at the built-in scratch when they fit, so that nothing is allocated either.
  GemmArgs a;
  astergemm_operands o;
  memset(&o, 0, sizeof(o));
  o.dA = o.dB = o.dC = scratch_ptr;
  o.dScaleA = o.dScaleB = o.dBias = (const float*)scratch_ptr;
  o.dMxA = o.dMxB = (const uint8_t*)scratch_ptr;
  if (workspace_need(*v, *cfg) <= (size_t)ASTERGEMM_NOALLOC_SCRATCH_BYTES) {
    o.dWorkspace = scratch_ptr;
    o.workspace_bytes = (size_t)ASTERGEMM_NOALLOC_SCRATCH_BYTES;
  }
  if (int rc = build_args(*v, *cfg, o, &a)) return rc;
  (void)hipGetLastError();
  LaunchScope scope(nullptr, /*prepare_only=*/true);
  const int e = v->launch(a, grid_of(*v, *cfg), nullptr);
  if (e != 0) return launch_fail(e, v->name, __FILE__, __LINE__);
  return 0;
}

int astergemm_workspace_bytes(const astergemm_config* cfg, size_t* bytes) {
  if (!cfg || !bytes) {
    set_error("astergemm_workspace_bytes: null argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  *bytes = (cfg->M == 0 || cfg->N == 0) ? 0 : workspace_need(*v, *cfg);
  return 0;
}

int astergemm_run_noalloc(const astergemm_config* cfg, const astergemm_operands* ops,
                          void* stream) {
  if (!cfg || !ops) {
    set_error("astergemm_run_noalloc: null argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  if (cfg->M == 0 || cfg->N == 0) return 0;
  const size_t need = workspace_need(*v, *cfg);
  if (need > (size_t)ASTERGEMM_NOALLOC_SCRATCH_BYTES) {
    set_error("astergemm_run_noalloc: %s needs %zu bytes of partial sums for this config, the "
              "built-in scratch holds %zu; use astergemm_run with a workspace",
              v->name, need, (size_t)ASTERGEMM_NOALLOC_SCRATCH_BYTES);
    return ASTERGEMM_EINVAL;
  }
  astergemm_operands o = *ops;
  o.dWorkspace = nullptr;
  o.workspace_bytes = 0;
  if (need) {
    void* p = scratch_address();
    if (!p) return ASTERGEMM_EHIP;
    o.dWorkspace = p;
    o.workspace_bytes = (size_t)ASTERGEMM_NOALLOC_SCRATCH_BYTES;
  }
  GemmArgs a;
  if (int rc = build_args(*v, *cfg, o, &a)) return rc;
  (void)hipGetLastError();
  LaunchScope scope(stream);
  const int e = v->launch(a, grid_of(*v, *cfg), (hipStream_t)stream);
  if (e != 0) return launch_fail(e, v->name, __FILE__, __LINE__);
  return 0;
}

int astergemm_bench_rotate(const astergemm_config* cfg, const astergemm_operands* ops, int n_ops,
                           int iters, int64_t* total_ns, void* stream) {
  if (!cfg || !ops || !total_ns || iters <= 0 || n_ops <= 0) {
    set_error("astergemm_bench_rotate: bad argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  *total_ns = 0;
  if (cfg->M == 0 || cfg->N == 0) return 0;
  std::vector<GemmArgs> args((size_t)n_ops);
  for (int i = 0; i < n_ops; ++i)
    if (int rc = build_args(*v, *cfg, ops[i], &args[(size_t)i])) return rc;
  hipStream_t s = (hipStream_t)stream;
  LaunchScope scope(stream);
  const int grid = grid_of(*v, *cfg);
  EventPair ev;
  AG_HIP(ev.create());
  int le = (int)hipEventRecord(ev.e0, s);
  (void)hipGetLastError();
  for (int i = 0; i < iters && le == 0; ++i) le = v->launch(args[(size_t)(i % n_ops)], grid, s);
  if (le == 0) le = (int)hipEventRecord(ev.e1, s);
  if (le == 0) le = (int)hipEventSynchronize(ev.e1);
  float ms = 0.f;
  if (le == 0) le = (int)hipEventElapsedTime(&ms, ev.e0, ev.e1);
  if (le != 0) return hip_fail((hipError_t)le, v->name, __FILE__, __LINE__);
  *total_ns = (int64_t)((double)ms * 1e6);
  return 0;
}

int astergemm_bench_graph(const astergemm_config* cfg, const astergemm_operands* ops, int n_ops,
                          int launches, int replays, int64_t* total_ns) {
  if (!cfg || !ops || !total_ns || launches <= 0 || launches > 4096 || replays <= 0 || n_ops <= 0) {
    set_error("astergemm_bench_graph: bad argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  *total_ns = 0;
  if (cfg->M == 0 || cfg->N == 0) return 0;
  std::vector<GemmArgs> args((size_t)n_ops);
  for (int i = 0; i < n_ops; ++i)
    if (int rc = build_args(*v, *cfg, ops[i], &args[(size_t)i])) return rc;
  const int grid = grid_of(*v, *cfg);
  // a stream of this call's own (default priority), so that the capture sees nothing else
  hipStream_t s = nullptr;
  AG_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  EventPair ev;
  int le = (int)ev.create();
  {
    LaunchScope scope(s);
    // one eager launch first: function attributes, and the partial-sum workspace of this stream
    // where the config has one, are one-time steps that may not happen inside a capture
    (void)hipGetLastError();
    if (le == 0) le = v->launch(args[0], grid, s);
    if (le == 0) le = (int)hipStreamSynchronize(s);
    if (le == 0) {
      le = (int)hipStreamBeginCapture(s, hipStreamCaptureModeGlobal);
      if (le == 0) {
        int ce = 0;
        for (int i = 0; i < launches && ce == 0; ++i) ce = v->launch(args[(size_t)(i % n_ops)], grid, s);
        le = (int)hipStreamEndCapture(s, &graph);  // always ended, also after a refused launch
        if (ce != 0) le = ce;
      }
    }
  }
  if (le == 0) le = (int)hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (le == 0) le = (int)hipGraphLaunch(exec, s);  // untimed: the first replay uploads the graph
  if (le == 0) le = (int)hipStreamSynchronize(s);
  if (le == 0) le = (int)hipEventRecord(ev.e0, s);
  for (int r = 0; r < replays && le == 0; ++r) le = (int)hipGraphLaunch(exec, s);
  if (le == 0) le = (int)hipEventRecord(ev.e1, s);
  if (le == 0) le = (int)hipEventSynchronize(ev.e1);
  float ms = 0.f;
  if (le == 0) le = (int)hipEventElapsedTime(&ms, ev.e0, ev.e1);
  if (exec) (void)hipGraphExecDestroy(exec);
  if (graph) (void)hipGraphDestroy(graph);
  (void)hipStreamSynchronize(s);
  splitk_workspace_release(s);  // the partial-sum workspace this stream may have been given
  (void)hipStreamDestroy(s);
  if (le != 0) return hip_fail((hipError_t)le, v->name, __FILE__, __LINE__);
  *total_ns = (int64_t)((double)ms * 1e6);
  return 0;
}

int astergemm_tune(const astergemm_config* cfg, const astergemm_operands* ops, int iters,
                   int* best_variant, int64_t* best_ns, void* stream) {
  if (!cfg || !ops || !best_variant || iters <= 0) {
    set_error("astergemm_tune: bad argument");
    return ASTERGEMM_EINVAL;
  }
  if (const char* why = validate_problem(*cfg)) {
    set_error("astergemm: invalid config: %s", why);
    return ASTERGEMM_EINVAL;
  }
  *best_variant = 0;
  if (best_ns) *best_ns = 0;
  hipStream_t s = (hipStream_t)stream;
  LaunchScope scope(stream);
  EventPair ev;
  AG_HIP(ev.create());
  hipEvent_t e0 = ev.e0, e1 = ev.e1;
  double best = 0.0;
  int rc = 0;
  for (int i = 0; i < total_variants() && rc == 0; ++i) {
    const Variant* v = variant_at(i);
    // every variant that can run the config: right types, family if one is asked for, shape
    // check passed, activation tile covering M on the weight-streaming path
    if (!variant_matches_types(*v, *cfg) || v->check(*cfg)) continue;
    if (cfg->family != ASTERGEMM_KERNEL_AUTO && cfg->family != v->family) continue;
    if (v->family == ASTERGEMM_KERNEL_SKINNY && v->tile_m < cfg->M) continue;
    if (cfg->M == 0 || cfg->N == 0) {
      *best_variant = i + 1;
      break;
    }
    // a caller's workspace too small for this variant's K ranges: the variant is skipped, the
    // tune goes on with the others
    if (ops->dWorkspace && ops->workspace_bytes < workspace_need(*v, *cfg)) continue;
    GemmArgs a;
    if ((rc = build_args(*v, *cfg, *ops, &a)) != 0) break;
    const int grid = grid_of(*v, *cfg);
    (void)hipGetLastError();
    int le = 0;
    for (int w = 0; w < 2 && le == 0; ++w) le = v->launch(a, grid, s);  // warm-up
    if (le == 0) le = (int)hipEventRecord(e0, s);
    for (int k = 0; k < iters && le == 0; ++k) le = v->launch(a, grid, s);
    if (le == 0) le = (int)hipEventRecord(e1, s);
    if (le == 0) le = (int)hipEventSynchronize(e1);
    float ms = 0.f;
    if (le == 0) le = (int)hipEventElapsedTime(&ms, e0, e1);
    if (le != 0) {
      rc = hip_fail((hipError_t)le, v->name, __FILE__, __LINE__);
      break;
    }
    if (*best_variant == 0 || ms < best) {
      best = ms;
      *best_variant = i + 1;
    }
  }
  if (rc != 0) return rc;
  if (*best_variant == 0) {
    set_error("astergemm_tune: no kernel variant can run this config");
    return ASTERGEMM_ENOTSUP;
  }
  if (best_ns) *best_ns = (int64_t)(best * 1e6 / iters);
  return 0;
}

int astergemm_bench(const astergemm_config* cfg, const astergemm_operands* ops, int iters,
                    int64_t* times_ns, int64_t flush_bytes, void* stream) {
  if (!cfg || !ops || !times_ns || iters <= 0) {
    set_error("astergemm_bench: bad argument");
    return ASTERGEMM_EINVAL;
  }
  int index = -1;
  const Variant* v = choose(*cfg, &index);
  if (!v) return g_choose_rc;
  if (cfg->M == 0 || cfg->N == 0) {
    for (int i = 0; i < iters; ++i) times_ns[i] = 0;
    return 0;
  }
  GemmArgs a;
  if (int rc = build_args(*v, *cfg, *ops, &a)) return rc;
  hipStream_t s = (hipStream_t)stream;
  LaunchScope scope(stream);
  const int grid = grid_of(*v, *cfg);

  DeviceBuffer flush_buf;
  uint32_t* flush = nullptr;
  if (flush_bytes > 0) {
    AG_HIP(hipMalloc(&flush_buf.ptr, (size_t)flush_bytes));
    flush = (uint32_t*)flush_buf.ptr;
    AG_HIP(hipMemsetAsync(flush, 0, (size_t)flush_bytes, s));
  }
  EventPair ev;
  AG_HIP(ev.create());
  hipEvent_t e0 = ev.e0, e1 = ev.e1;
  int rc = 0;
  (void)hipGetLastError();  // the launchers report hipGetLastError()
  for (int i = 0; i < iters && rc == 0; ++i) {
    if (flush) {
      hipLaunchKernelGGL(flush_llc_kernel, dim3(2048), dim3(256), 0, s, flush,
                         (size_t)flush_bytes / 4);
      // a flush that did not launch would give warm-cache times labelled as flushed
      const hipError_t fe = hipGetLastError();
      if (fe != hipSuccess) return hip_fail(fe, "flush_llc_kernel", __FILE__, __LINE__);
    }
    hipError_t e = hipEventRecord(e0, s);
    int le = (e == hipSuccess) ? v->launch(a, grid, s) : (int)e;
    if (le == 0) le = (int)hipEventRecord(e1, s);
    if (le == 0) le = (int)hipEventSynchronize(e1);
    float ms = 0.f;
    if (le == 0) le = (int)hipEventElapsedTime(&ms, e0, e1);
    if (le != 0) {
      rc = hip_fail((hipError_t)le, v->name, __FILE__, __LINE__);
      break;
    }
    times_ns[i] = (int64_t)((double)ms * 1e6);
  }
  return rc;
}

int astergemm_shuffle_weight_16(const uint16_t* src, uint16_t* dst, int64_t N, int64_t K) {
  if (!src || !dst || N < 0 || K < 0 || N % 16 != 0 || K % 32 != 0) {
    set_error("astergemm_shuffle_weight_16: need N %% 16 == 0 and K %% 32 == 0");
    return ASTERGEMM_EINVAL;
  }
  // dst index order (nb, kb, lane_group, n_lane, kh, k_within) <- src (nb, n_lane, kb, kh,
  // lane_group, k_within): each lane's 8 contiguous elements are its two 16x16x16 K-steps.
  const int64_t kblocks = K / 32;
  int64_t o = 0;
  for (int64_t nb = 0; nb < N / 16; ++nb)
    for (int64_t kb = 0; kb < kblocks; ++kb)
      for (int g = 0; g < 4; ++g)
        for (int nl = 0; nl < 16; ++nl)
          for (int kh = 0; kh < 2; ++kh)
            for (int kw = 0; kw < 4; ++kw)
              dst[o++] = src[(nb * 16 + nl) * K + kb * 32 + kh * 16 + g * 4 + kw];
  return 0;
}

int astergemm_shuffle_weight_k8_16(const uint16_t* src, uint16_t* dst, int64_t N, int64_t K) {
  if (!src || !dst || N < 0 || K < 0 || N % 16 != 0 || K % 32 != 0) {
    set_error("astergemm_shuffle_weight_k8_16: need N %% 16 == 0 and K %% 32 == 0");
    return ASTERGEMM_EINVAL;
  }
  // dst order (nb, kb, lane group g, row n, 8 consecutive K) <- src (nb, n, kb, g, k)
  const int64_t kblocks = K / 32;
  int64_t o = 0;
  for (int64_t nb = 0; nb < N / 16; ++nb)
    for (int64_t kb = 0; kb < kblocks; ++kb)
      for (int g = 0; g < 4; ++g)
        for (int nl = 0; nl < 16; ++nl)
          for (int kw = 0; kw < 8; ++kw) dst[o++] = src[(nb * 16 + nl) * K + kb * 32 + g * 8 + kw];
  return 0;
}

int astergemm_shuffle_weight_8(const uint8_t* src, uint8_t* dst, int64_t N, int64_t row_bytes_) {
  if (!src || !dst || N < 0 || row_bytes_ < 0 || N % 16 != 0 || row_bytes_ % 128 != 0) {
    set_error("astergemm_shuffle_weight_8: need N %% 16 == 0 and rows of whole 128-byte steps");
    return ASTERGEMM_EINVAL;
  }
  // dst order (nb, step, half u, lane group q, row n, 16 bytes) <- src (nb, n, step, 4u + q, 16 bytes)
  const int64_t steps = row_bytes_ / 128;
  uint8_t* o = dst;
  for (int64_t nb = 0; nb < N / 16; ++nb)
    for (int64_t st = 0; st < steps; ++st)
      for (int u = 0; u < 2; ++u)
        for (int q = 0; q < 4; ++q)
          for (int nl = 0; nl < 16; ++nl, o += 16)
            memcpy(o, src + (nb * 16 + nl) * row_bytes_ + st * 128 + (4 * u + q) * 16, 16);
  return 0;
}

int astergemm_shuffle_scales_e8m0(const uint8_t* src, uint8_t* dst, int64_t N, int64_t K) {
  if (!src || !dst || N < 0 || K < 0 || N % 16 != 0 || K % 256 != 0) {
    set_error("astergemm_shuffle_scales_e8m0: need N %% 16 == 0 and K %% 256 == 0");
    return ASTERGEMM_EINVAL;
  }
  // dst order (nb, step, row n, 8 bytes) <- src (nb, n, step, 8 bytes)
  const int64_t steps = K / 256, ld = K / 32;
  uint8_t* o = dst;
  for (int64_t nb = 0; nb < N / 16; ++nb)
    for (int64_t st = 0; st < steps; ++st)
      for (int nl = 0; nl < 16; ++nl, o += 8) memcpy(o, src + (nb * 16 + nl) * ld + st * 8, 8);
  return 0;
}

int astergemm_shuffle_scales_e8m0_lanes(const uint8_t* src, uint8_t* dst, int64_t N, int64_t K) {
  if (!src || !dst || N < 0 || K < 0 || N % 64 != 0 || K % 256 != 0) {
    set_error("astergemm_shuffle_scales_e8m0_lanes: need N %% 64 == 0 and K %% 256 == 0");
    return ASTERGEMM_EINVAL;
  }
  // dst order (nb4, step, lane group q, row i, tile t, half h) <- src (nb4, t, i, step, 4 h + q)
  const int64_t steps = K / 256, ld = K / 32;
  uint8_t* o = dst;
  for (int64_t nb4 = 0; nb4 < N / 64; ++nb4)
    for (int64_t st = 0; st < steps; ++st)
      for (int q = 0; q < 4; ++q)
        for (int i = 0; i < 16; ++i)
          for (int t = 0; t < 4; ++t)
            for (int h = 0; h < 2; ++h)
              *o++ = src[(nb4 * 64 + t * 16 + i) * ld + st * 8 + 4 * h + q];
  return 0;
}

int64_t astergemm_mx_lanes128_bytes(int64_t M, int64_t K) {
  if (M < 0 || K < 0) return 0;
  return ((M + 127) / 128) * (K / 256) * 1024;
}

int astergemm_shuffle_scales_e8m0_lanes128(const uint8_t* src, uint8_t* dst, int64_t M, int64_t K) {
  if (!src || !dst || M < 0 || K < 0 || K % 256 != 0) {
    set_error("astergemm_shuffle_scales_e8m0_lanes128: need K %% 256 == 0");
    return ASTERGEMM_EINVAL;
  }
  // dst order (group g, step, lane group q, row i, tile t, half h) <- src (g, t, i, step, 4 h + q);
  // rows past M: 127
  const int64_t steps = K / 256, ld = K / 32;
  uint8_t* o = dst;
  for (int64_t g = 0; g < (M + 127) / 128; ++g)
    for (int64_t st = 0; st < steps; ++st)
      for (int q = 0; q < 4; ++q)
        for (int i = 0; i < 16; ++i)
          for (int t = 0; t < 8; ++t)
            for (int h = 0; h < 2; ++h) {
              const int64_t row = g * 128 + t * 16 + i;
              *o++ = row < M ? src[row * ld + st * 8 + 4 * h + q] : (uint8_t)127;
            }
  return 0;
}

/* ---- runtime seam --------------------------------------------------------- */

int aster_rt_init(void) {
  int n = 0;
  AG_HIP(hipGetDeviceCount(&n));
  if (n <= 0) {
    set_error("aster_rt_init: no HIP device");
    return ASTERGEMM_ENODEV;
  }
  // the built-in scratch of astergemm_run_noalloc, for the device that is current now
  if (!scratch_address()) return ASTERGEMM_EHIP;
  return 0;
}
int aster_rt_peek_at_last_error(void) { return (int)hipPeekAtLastError(); }
int aster_rt_clear_last_error(void) { return (int)hipGetLastError(); }
int aster_rt_get_device_count(int* count) {
  AG_HIP(hipGetDeviceCount(count));
  return 0;
}
int aster_rt_set_device(int device) {
  AG_HIP(hipSetDevice(device));
  return 0;
}
int aster_rt_get_device(int* device) {
  AG_HIP(hipGetDevice(device));
  return 0;
}
int aster_rt_device_reset(void) {
  AG_HIP(hipDeviceReset());
  return 0;
}
int aster_rt_device_synchronize(void) {
  AG_HIP(hipDeviceSynchronize());
  return 0;
}
int aster_rt_get_device_props(int device, astergemm_device_props* out) {
  if (!out) {
    set_error("aster_rt_get_device_props: null out");
    return ASTERGEMM_EINVAL;
  }
  hipDeviceProp_t p;
  AG_HIP(hipGetDeviceProperties(&p, device));
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s", p.name);
  snprintf(out->gcn_arch_name, sizeof(out->gcn_arch_name), "%s", p.gcnArchName);
  out->warp_size = p.warpSize;
  out->lds_per_cu = (int32_t)p.sharedMemPerBlock;
  out->regs_per_multiprocessor = p.regsPerMultiprocessor;
  out->multiprocessor_count = p.multiProcessorCount;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->max_threads_per_multiprocessor = p.maxThreadsPerMultiProcessor;
  out->asic_revision = p.asicRevision;
  out->cluster_launch = 0;
  out->total_global_mem = (int64_t)p.totalGlobalMem;
  out->clock_rate_khz = p.clockRate;
  out->l2_cache_bytes = p.l2CacheSize;
  return 0;
}
int aster_rt_malloc(void** dptr, size_t bytes) {
  AG_HIP(hipMalloc(dptr, bytes));
  return 0;
}
int aster_rt_free(void* dptr) {
  AG_HIP(hipFree(dptr));
  return 0;
}
int aster_rt_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  AG_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return 0;
}
int aster_rt_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  AG_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return 0;
}
int aster_rt_memcpy_d2d(void* dst, const void* src, size_t bytes) {
  AG_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
  return 0;
}
int aster_rt_memset(void* dst, int value, size_t bytes) {
  AG_HIP(hipMemset(dst, value, bytes));
  return 0;
}
int aster_rt_module_load_data(const void* image, size_t bytes, void** module) {
  (void)bytes;
  hipModule_t m;
  AG_HIP(hipModuleLoadData(&m, image));
  *module = (void*)m;
  return 0;
}
int aster_rt_module_get_function(void* module, const char* name, void** fn) {
  hipFunction_t f;
  AG_HIP(hipModuleGetFunction(&f, (hipModule_t)module, name));
  *fn = (void*)f;
  return 0;
}
int aster_rt_module_unload(void* module) {
  AG_HIP(hipModuleUnload((hipModule_t)module));
  return 0;
}
int aster_rt_module_launch_kernel(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                                  unsigned by, unsigned bz, unsigned shared_bytes, void* stream,
                                  void** kernel_params) {
  AG_HIP(hipModuleLaunchKernel((hipFunction_t)fn, gx, gy, gz, bx, by, bz, shared_bytes,
                               (hipStream_t)stream, kernel_params, nullptr));
  return 0;
}
int aster_rt_function_free(void* fn) {
  // a hipFunction_t belongs to its module and goes with aster_rt_module_unload; the reference
  // frees only the heap cell its binding wrapped the handle in (RuntimeModule.cpp:221-226)
  (void)fn;
  return 0;
}
int aster_rt_module_launch_kernel_ex(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                                     unsigned by, unsigned bz, unsigned cx, unsigned cy,
                                     unsigned cz, unsigned shared_bytes, void* stream,
                                     void** kernel_params) {
  // cluster launches do not exist on gfx950: a cluster of (1,1,1) is a plain launch
  if (cx > 1 || cy > 1 || cz > 1) {
    set_error("aster_rt_module_launch_kernel_ex: cluster launch (%u,%u,%u) is not supported on "
              "gfx950", cx, cy, cz);
    return ASTERGEMM_ENOTSUP;
  }
  return aster_rt_module_launch_kernel(fn, gx, gy, gz, bx, by, bz, shared_bytes, stream,
                                       kernel_params);
}
int aster_rt_event_create(void** event) {
  hipEvent_t e;
  AG_HIP(hipEventCreate(&e));
  *event = (void*)e;
  return 0;
}
int aster_rt_event_destroy(void* event) {
  AG_HIP(hipEventDestroy((hipEvent_t)event));
  return 0;
}
int aster_rt_event_record(void* event, void* stream) {
  AG_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return 0;
}
int aster_rt_event_synchronize(void* event) {
  AG_HIP(hipEventSynchronize((hipEvent_t)event));
  return 0;
}
int aster_rt_event_elapsed_ms(void* start, void* stop, float* ms) {
  AG_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}
int aster_rt_stream_create(void** stream) {
  hipStream_t s;
  AG_HIP(hipStreamCreate(&s));
  *stream = (void*)s;
  return 0;
}
int aster_rt_stream_destroy(void* stream) {
  AG_HIP(hipStreamDestroy((hipStream_t)stream));
  return 0;
}
int aster_rt_stream_synchronize(void* stream) {
  AG_HIP(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}

}  // extern "C"
