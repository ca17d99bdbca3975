/*
 * astergemm.h -- C-ABI of the MI355X (gfx950) GEMM hot path.
 *
 * One shared library (libastergemm.so) exports everything below with C
 * linkage: plain pointers, sizes and PODs only.  It replaces two seams of the
 * reference:
 *
 *   1. the nanobind HIP wrapper `_runtime_module`
 *      (reference: python/lib/RuntimeModule.cpp:140-418) -- the `aster_rt_*`
 *      functions are its hip_* functions one for one, so the reference's
 *      `execute_hsaco` (python/aster/execution/core.py:605-717) can be bound
 *      to them unchanged;
 *   2. the per-config `compile_*` / `execute_*_hsaco` pair of every GEMM
 *      generator (reference: contrib/kittens/test/
 *      test_102_gemm_python_multitile_g2s_directb_cdna4.py:420-467) -- the
 *      `astergemm_*` functions select a pre-built hand-written kernel for a
 *      problem + mapping and launch / time it.
 *
 * Conventions: every function returns 0 on success and a negative
 * ASTERGEMM_E* code on failure; nothing throws; the message of the last
 * failure on the calling thread is returned by astergemm_last_error().
 * All buffers are owned by the caller.  Decode shapes (M <= 64) whose rows are
 * not 4 or 8 KiB long, and shapes with at most 128 output tiles of 128 x 128
 * and long rows, are computed in K ranges whose fp32 partial sums need a
 * workspace: astergemm_workspace_bytes() says how much, and
 * astergemm_operands.dWorkspace brings it.  Without one the library falls back
 * to a buffer of its own, one per (device, stream), allocated on the first such
 * call (that call therefore cannot be captured into a graph), replaced by a
 * larger one when needed and kept until the process ends.  Calls on different
 * streams may run
 * concurrently; calls on one stream are ordered by it.  Pointers named d*
 * are device pointers.  Launches go to the stream that is passed (NULL = the null
 * stream, which is what the reference uses everywhere).
 */
#ifndef ASTERGEMM_H_
#define ASTERGEMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ASTERGEMM_ABI_VERSION 3

/* ---- error codes ------------------------------------------------------ */
#define ASTERGEMM_OK 0
#define ASTERGEMM_EINVAL (-22)   /* bad argument / unsupported shape       */
#define ASTERGEMM_ENOTSUP (-95)  /* no kernel variant for this config      */
#define ASTERGEMM_EHIP (-5)      /* a HIP runtime call failed              */
#define ASTERGEMM_ENODEV (-19)   /* no gfx950 device                       */

/* ---- element types ----------------------------------------------------- */
/* The reference's GemmSpec carries only elt_bytes_a/b/c (f16 x f16 -> f32,
 * contrib/kittens/gemm_config.py:115-118); the build adds the storage types
 * of the other four configurations. */
typedef enum astergemm_dtype {
  ASTERGEMM_F16 = 0,      /* IEEE binary16                                  */
  ASTERGEMM_BF16 = 1,     /* bfloat16                                       */
  ASTERGEMM_FP8_E4M3 = 2, /* OCP e4m3 (bias 7, max 448, NaN 0x7F)           */
  ASTERGEMM_MXFP4 = 3,    /* OCP e2m1, two per byte (low nibble first), with
                             one e8m0 scale byte per 32 K-elements          */
  ASTERGEMM_F32 = 4       /* output only                                    */
} astergemm_dtype;

typedef enum astergemm_scale_mode {
  ASTERGEMM_SCALE_NONE = 0,
  ASTERGEMM_SCALE_TENSOR = 1, /* one fp32 per operand, read from device     */
  ASTERGEMM_SCALE_MX32 = 2    /* e8m0 byte per (row, 32-wide K block)       */
} astergemm_scale_mode;

typedef enum astergemm_kernel_family {
  ASTERGEMM_KERNEL_AUTO = 0,
  ASTERGEMM_KERNEL_TILE = 1,  /* LDS-staged MFMA tile kernel                */
  ASTERGEMM_KERNEL_SKINNY = 2 /* weight-streaming kernel for M <= 64        */
} astergemm_kernel_family;

/* The reference's GemmMappingSpec.operand_path (gemm_config.py:213-276): with
 * "direct_b" the host pre-shuffles B with shuffle_weight
 * (contrib/kittens/test/kittens_helpers.py:90-119) so that a lane's 16-byte
 * global load is its MFMA operand and B never passes through LDS.            */
typedef enum astergemm_operand_path {
  ASTERGEMM_OPERAND_LDS = 0,      /* B[N, ldb] row-major as described below   */
  ASTERGEMM_OPERAND_DIRECT_B = 1, /* B packed [N, K] and pre-shuffled: 16-bit
                                     operands with astergemm_shuffle_weight_16,
                                     the reference's order; fp8 and MXFP4
                                     payloads with astergemm_shuffle_weight_8
                                     (MXFP4: dMxB pre-shuffled as well, with
                                     astergemm_shuffle_scales_e8m0).  The
                                     decode kernels, M <= 16                 */
  ASTERGEMM_OPERAND_DIRECT_B_K8 = 2, /* B packed [N, K] and pre-shuffled for the
                                     stream kernels that load B straight into
                                     MFMA operands.  MXFP4: payload with
                                     astergemm_shuffle_weight_8, dMxB with
                                     astergemm_shuffle_scales_e8m0_lanes
                                     (128 x 256 tiles, N % 64 == 0,
                                     K % 512 == 0).  fp8: with
                                     astergemm_shuffle_weight_8, the same
                                     bytes as DIRECT_B (128 x 256 tiles,
                                     N % 16 == 0, K % 128 == 0).  16-bit
                                     operands: with
                                     astergemm_shuffle_weight_k8_16: 8
                                     consecutive K per lane, the order of the
                                     16x16x32 MFMA and of 16-byte LDS reads
                                     (the 128 x 256 and 256 x 256 stream
                                     kernel, N % 16 == 0, K % 64 == 0)       */
  ASTERGEMM_OPERAND_DIRECT_AB = 3 /* 16-bit operands: A packed [M, K] AND B
                                     packed [N, K], both pre-shuffled with
                                     astergemm_shuffle_weight_16 (the
                                     reference's order: its direct_ab
                                     template shuffles both operands alike,
                                     test_perf_001_gemm_fp16_weak_scaled.py:
                                     252-254); neither passes through LDS
                                     (M % 16 == 0, N % 16 == 0,
                                     K % 32 == 0)                             */
} astergemm_operand_path;

/* Layout of the e8m0 plane of the ACTIVATIONS (A) of an MXFP4 GEMM.  The
 * reference has no scaled-MFMA GEMM; the operand form being matched is the
 * scale register of v_mfma_scale_f32_16x16x128_f8f6f4
 * (test/Dialect/AMDGCN/cdna4-scaled-mfma.mlir:37-47). */
typedef enum astergemm_mx_layout {
  ASTERGEMM_MX_ROWS = 0,     /* [M, K/32] bytes, row-major                      */
  ASTERGEMM_MX_LANES128 = 1  /* lane order in groups of 128 rows, padded to
                                whole groups: astergemm_shuffle_scales_e8m0_lanes128
                                / astergemm_quantize_mxfp4_ex.  Read by the
                                ASTERGEMM_OPERAND_DIRECT_B_K8 MXFP4 stream
                                kernel with one 16-byte load per wave and
                                256-element step, instead of a pass through
                                LDS                                            */
} astergemm_mx_layout;

/* ---- problem + mapping --------------------------------------------------
 * C[M,N] = epilogue( sum_k A[M,K] * B[N,K] )      (B is stored N x K, i.e.
 * "column-major K x N"; reference: gemm_config.py:94, 109).
 * Mirrors GemmSpec (gemm_config.py:90-205) and the subset of
 * GemmMappingSpec (gemm_config.py:213-276) that selects a kernel variant.
 * A zero in a mapping field means "library default".                      */
typedef struct astergemm_config {
  int64_t M, N, K;       /* K in elements (for MXFP4: e2m1 elements)        */
  int64_t lda, ldb, ldc; /* row pitch in elements; 0 = packed (K, K, N)     */
  int32_t dtype_ab;      /* astergemm_dtype of A and B                      */
  int32_t dtype_c;       /* F32, BF16 or F16                                */
  int32_t scale_mode;    /* astergemm_scale_mode                            */
  int32_t has_bias;      /* fp32 bias[N] added after scaling                */
  /* mapping (all optional) */
  int32_t family;        /* astergemm_kernel_family                         */
  int32_t wg_tile_m;     /* = num_tiles_per_workgroup[M] * mfma_m           */
  int32_t wg_tile_n;     /* = num_tiles_per_workgroup[N] * mfma_n           */
  int32_t waves_m;       /* num_waves_per_workgroup[M]                      */
  int32_t waves_n;       /* num_waves_per_workgroup[N]                      */
  int32_t variant;       /* explicit variant id from astergemm_variant_*,
                            or 0                                             */
  int32_t operand_path;  /* astergemm_operand_path: how B (DIRECT_AB: and A)
                            is stored                                       */
  int32_t mx_a_layout;   /* astergemm_mx_layout: how A's e8m0 plane is stored
                            (SCALE_MX32 only; B's follows operand_path)      */
  int32_t reserved[4];
} astergemm_config;

/* What astergemm_select() reports back; the reference gets the same facts by
 * parsing the generated asm (`parse_asm_kernel_resources`,
 * python/aster/compiler/metadata.py) and from cfg.num_workgroups/num_threads. */
typedef struct astergemm_kernel_info {
  int32_t variant;        /* id usable in astergemm_config.variant           */
  int32_t family;
  int32_t grid_x;         /* 1-D grid, like every reference GEMM             */
  int32_t block_x;
  int32_t lds_bytes;
  int32_t vgprs, agprs;   /* from hipFuncGetAttributes; agprs is 0 when the
                             runtime reports only the unified count          */
  int32_t wg_tile_m, wg_tile_n, wg_tile_k;
  int32_t waves_m, waves_n;
  int32_t pipeline_stages;
  int64_t flops;          /* 2*M*N*K                                         */
  int64_t bytes;          /* algorithmic bytes: A + B (+ scales) + C         */
  char name[64];
} astergemm_kernel_info;

/* Device operands of one GEMM call. Unused pointers are NULL. */
typedef struct astergemm_operands {
  const void* dA;          /* [M, lda]                                        */
  const void* dB;          /* [N, ldb]                                        */
  void* dC;                /* [M, ldc]                                        */
  const float* dScaleA;    /* SCALE_TENSOR: 1 fp32 on device                  */
  const float* dScaleB;
  const uint8_t* dMxA;     /* SCALE_MX32: [M, K/32] e8m0 bytes, row-major     */
  const uint8_t* dMxB;     /*             [N, K/32]                           */
  const float* dBias;      /* [N] fp32                                        */
  void* dWorkspace;        /* fp32 partial sums of K ranges, 16-byte aligned,
                              at least astergemm_workspace_bytes(); NULL = the
                              library's own buffer                            */
  size_t workspace_bytes;  /* size of dWorkspace                              */
} astergemm_operands;

/* reference: hip_get_device_props dict (RuntimeModule.cpp:166-191) */
typedef struct astergemm_device_props {
  char name[128];
  char gcn_arch_name[64];
  int32_t warp_size;
  int32_t lds_per_cu;
  int32_t regs_per_multiprocessor;
  int32_t multiprocessor_count;
  int32_t max_threads_per_block;
  int32_t max_threads_per_multiprocessor;
  int32_t asic_revision;
  int32_t cluster_launch;
  int64_t total_global_mem;
  int32_t clock_rate_khz;
  int32_t l2_cache_bytes;
} astergemm_device_props;

/* ---- library ----------------------------------------------------------- */
int astergemm_abi_version(void);
const char* astergemm_last_error(void);

/* ---- GEMM path ---------------------------------------------------------- */
/* Replaces compile_fn: pick the kernel variant for cfg and describe it.     */
int astergemm_select(const astergemm_config* cfg, astergemm_kernel_info* out);
/* Number of built variants and a description of variant `index`
 * (0 <= index < count) instantiated for cfg's problem.                      */
int astergemm_variant_count(void);
int astergemm_variant_info(int index, const astergemm_config* cfg,
                           astergemm_kernel_info* out);
/* One asynchronous launch on `stream` (hipStream_t, NULL = null stream).    */
int astergemm_run(const astergemm_config* cfg, const astergemm_operands* ops,
                  void* stream);
/* Bytes of fp32 workspace astergemm_run needs for cfg with the variant it
 * selects (0 for most shapes: only rows cut into K ranges need one).  The
 * reference's kernels have no workspace (every kernel takes exactly A, B, C:
 * test_102_gemm_python_multitile_g2s_directb_cdna4.py:150-156); this is the
 * caller-owned form of what split K adds here.                              */
int astergemm_workspace_bytes(const astergemm_config* cfg, size_t* bytes);

/* astergemm_run for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): it
 * never calls hipMalloc / hipFree or an allocating routine.  No counterpart in
 * the reference.  ops->dWorkspace is ignored: the partial sums of K ranges go
 * to a scratch array built into the library, ASTERGEMM_NOALLOC_SCRATCH_BYTES
 * per device, held until the process ends; a config that needs more is refused
 * with ASTERGEMM_EINVAL.  Every call on a device shares that array, whatever
 * its stream: calls that overlap on one device race (calls on one stream are
 * ordered and safe).  Nothing in the array has to start at zero: every launch
 * writes all the planes it later adds.  The array's address is looked up on
 * the first call on a device, or by aster_rt_init / astergemm_prepare for the
 * current device.  A kernel's FIRST launch on a device also sets a function
 * attribute and is refused while the stream is being captured: call
 * astergemm_prepare(cfg) (below) or launch the config once eagerly before
 * capturing it.                                                              */
#define ASTERGEMM_NOALLOC_SCRATCH_BYTES (16u << 20)
int astergemm_run_noalloc(const astergemm_config* cfg, const astergemm_operands* ops,
                          void* stream);

/* Does, for the kernel `cfg` selects on the current device, everything a first
 * launch does apart from launching: raises the kernel's dynamic-LDS limit
 * (hipFuncSetAttribute), caches the device's compute-unit count and looks up
 * the address of the built-in scratch.  None of these is a stream operation,
 * so they must not happen inside a stream capture: astergemm_run and
 * astergemm_run_noalloc REFUSE a kernel's first launch on a device when the
 * stream is being captured (ASTERGEMM_EHIP, the message names this function).
 * Call it once per config and device before capturing (an eager launch of the
 * same config does the same).  Allocates nothing when the config's partial
 * sums fit the built-in scratch; reads no operand.  No counterpart in the
 * reference, whose kernels carry their LDS size in the code object. */
int astergemm_prepare(const astergemm_config* cfg);

/* Replaces execute_fn's timed loop (execution/core.py:690-703): `iters`
 * launches, each bracketed by its own HIP event pair on `stream`;
 * times_ns[i] = int(ms * 1e6).  If flush_bytes > 0 a streaming kernel over a
 * scratch buffer of that size runs before every start event (the reference's
 * FlushLLC hook, python/aster/execution/flush_llc.py:25-120).               */
int astergemm_bench(const astergemm_config* cfg, const astergemm_operands* ops,
                    int iters, int64_t* times_ns, int64_t flush_bytes,
                    void* stream);

/* Steady-state timing for launches too short for an event pair each (an event
 * pair around an empty kernel reads ~6 us on MI355X): `iters` launches go out
 * back to back between ONE event pair, launch i using operand set
 * ops[i % n_ops]; *total_ns = int(ms * 1e6) for all of them.  With enough
 * distinct weight buffers (n_ops * bytes of B well above the 256 MiB last-level
 * cache) every launch streams its weights from HBM, which is what the
 * reference's FlushLLC hook is for (python/aster/execution/flush_llc.py:25-60).
 * No counterpart in the reference: its harness times every launch separately. */
int astergemm_bench_rotate(const astergemm_config* cfg, const astergemm_operands* ops,
                           int n_ops, int iters, int64_t* total_ns, void* stream);

/* The same launches as nodes of a HIP graph: `launches` launches (launch i on
 * ops[i % n_ops]) are captured once on a stream of the call's own, after one
 * eager launch that does the config's one-time steps, and the graph is replayed
 * `replays` times between one event pair after one untimed replay;
 * *total_ns covers launches * replays launches.  What a serving loop that
 * replays a captured decode step pays per GEMM.  No counterpart in the
 * reference.                                                                  */
int astergemm_bench_graph(const astergemm_config* cfg, const astergemm_operands* ops,
                          int n_ops, int launches, int replays, int64_t* total_ns);

/* Measures every variant that can run cfg on the given operands (`iters`
 * back-to-back launches between one event pair each, after two warm-up
 * launches) and returns the fastest: *best_variant is what cfg->variant takes
 * to pin it, *best_ns (may be NULL) its time per launch.  cfg->family
 * restricts the candidates when it is not AUTO; cfg->variant is ignored.  dC
 * is overwritten by every candidate.  This is the reference's sweep step
 * (run_single over a list of mappings, bench_harness.py:1738-1850, feeding
 * tools/perf_best_known_update.py) on the prebuilt variants. */
int astergemm_tune(const astergemm_config* cfg, const astergemm_operands* ops, int iters,
                   int* best_variant, int64_t* best_ns, void* stream);

/* Host pre-shuffle of B[N,K] 2-byte elements into per-lane MFMA order
 * (reference: shuffle_weight, contrib/kittens/test/kittens_helpers.py:90-119). */
int astergemm_shuffle_weight_16(const uint16_t* src, uint16_t* dst, int64_t N,
                                int64_t K);
/* The same pre-shuffle for the 16x16x32 MFMA of gfx950 read with 16-byte
 * operand loads: chunk (nb, kb) of 1 KiB holds rows 16 nb .. + 15 and K
 * elements 32 kb .. + 31, lane 16 g + n of a wave finds its eight consecutive
 * K elements 32 kb + 8 g .. + 7 of row 16 nb + n at byte 16 (16 g + n).  The
 * reference's shuffle_weight (kittens_helpers.py:90-119) pairs the K elements
 * {4g..4g+3} and {16+4g..16+4g+3} instead, because its kernels read A with two
 * ds_read_b64 (test_102_gemm_python_multitile_g2s_directb_cdna4.py:178-188). */
int astergemm_shuffle_weight_k8_16(const uint16_t* src, uint16_t* dst, int64_t N,
                                   int64_t K);

/* The pre-shuffle for the one-byte and nibble types (fp8 e4m3, MXFP4 payload),
 * whose 16x16x128 MFMA takes the 16-byte pieces q and 4 + q of a 128-byte step
 * of a row: rows of `row_bytes` bytes (K for fp8, K / 2 for MXFP4; whole
 * 128-byte steps), N % 16 == 0.  Row block nb (16 rows), step s, half u is one
 * KiB at ((nb * steps + s) * 2 + u) * 1024 in which lane 16 q + n of a wave
 * finds bytes [(4u + q) * 16, + 16) of row 16 nb + n, step s, at byte
 * 16 (16 q + n).  The reference has no counterpart for these types; it is the
 * generalisation of its shuffle_weight (kittens_helpers.py:90-119) to the
 * operand order of v_mfma_scale_f32_16x16x128_f8f6f4. */
int astergemm_shuffle_weight_8(const uint8_t* src, uint8_t* dst, int64_t N, int64_t row_bytes);
/* The e8m0 plane [N, K/32] of pre-shuffled MXFP4 weights in the matching
 * order: the 8 scale bytes of row 16 nb + n, step s (256 elements) at
 * (nb * steps + s) * 128 + 8 n.  N % 16 == 0, K % 256 == 0. */
int astergemm_shuffle_scales_e8m0(const uint8_t* src, uint8_t* dst, int64_t N, int64_t K);
/* The e8m0 plane [N, K/32] of pre-shuffled MXFP4 weights in lane order, for
 * the stream kernel that loads B straight into MFMA operands
 * (ASTERGEMM_OPERAND_DIRECT_B_K8): rows in groups of 64 (four 16-row tiles, the
 * columns of one wave), group nb4 and step s (256 elements) are 512 bytes at
 * (nb4 * steps + s) * 512 in which lane L = 16 q + i of a wave finds, at byte
 * 8 L + 2 t + h, the scale of block 4 h + q of row 64 nb4 + 16 t + i: one
 * 8-byte load per lane brings the scale bytes of both MFMAs of a step for the
 * wave's four tiles.  N % 64 == 0, K % 256 == 0.  No counterpart in the
 * reference (it has no scaled MFMA kernels). */
int astergemm_shuffle_scales_e8m0_lanes(const uint8_t* src, uint8_t* dst, int64_t N, int64_t K);

/* The e8m0 plane of MXFP4 ACTIVATIONS [M, K/32] in lane order
 * (ASTERGEMM_MX_LANES128): rows in groups of 128 (the eight 16-row tiles a wave
 * of the 128 x 256 stream kernel multiplies), per group and 256-element step one
 * KiB in which lane L = 16 q + i finds, at byte 16 L + 2 t + h, the scale of
 * block 4 h + q of row 128 g + 16 t + i.  M need not be a multiple of 128: the
 * destination holds astergemm_mx_lanes128_bytes(M, K) = ceil(M / 128) * (K / 256)
 * * 1024 bytes and the rows past M get the byte 127 (scale 1).  K % 256 == 0.
 * No counterpart in the reference (it has no scaled MFMA kernels). */
int64_t astergemm_mx_lanes128_bytes(int64_t M, int64_t K);
int astergemm_shuffle_scales_e8m0_lanes128(const uint8_t* src, uint8_t* dst, int64_t M, int64_t K);

/* ---- operand quantisers (device to device, on `stream`) -------------------
 * They write the bytes the fp8 / MXFP4 GEMM paths read (dtype_ab
 * ASTERGEMM_FP8_E4M3 / ASTERGEMM_MXFP4), so that a caller holding activations
 * or weights in HBM needs no host round trip.
 *
 * The source is fp32, or the bf16 / f16 a GEMM of this library wrote
 * (src_dtype = ASTERGEMM_F32 / _BF16 / _F16; the 16-bit types widen to fp32
 * exactly, so the result equals quantising the widened values).
 *
 * astergemm_absmax: *dAbsmax = max |dSrc[i]| (0 for n == 0; NaN if any
 * element is NaN).  dSrc 16-byte aligned.
 *
 * astergemm_quantize_fp8_tensor: *dScale = absmax / 448 (1.0 when absmax is
 * zero), dDst[i] = e4m3(dSrc[i] / *dScale) with the rounding of the converter
 * the reference's tests hold (f32_to_fp8_e4m3, fnuz=False:
 * test/integration/test_conversion_pack_e2e.py:91-167): nearest even, carry
 * into the exponent, saturation to 448 = 0x7E, NaN / inf -> S|0x7F, signed
 * zero; the subnormal range rounds to nearest even.  *dScale is what
 * astergemm_operands.dScaleA / dScaleB take.  dDst 4-byte aligned.
 *
 * astergemm_quantize_mxfp4: rows x K elements (row stride ld_src elements,
 * 0 = K) -> dPacked[rows, K/2] (element 2j in the low nibble of byte j) and
 * dScales[rows, K/32] e8m0 bytes, the operand layout of the scaled MFMA
 * (v_mfma_scale_f32_16x16x128_f8f6f4; reference instruction definition
 * include/aster/Dialect/AMDGCN/IR/Instructions/MMA.td:792).  Per 32-element
 * block: scale exponent floor(log2(absmax)) - 2 clamped to [-127, 127] (0 for
 * an all-zero block), elements e2m1 round-to-nearest-even of x / 2^exponent
 * saturated to +-6; a block holding NaN or inf gets scale byte 0xFF.
 * K % 32 == 0, ld_src % 8 == 0, dSrc and dPacked 16-byte aligned.           */
int astergemm_absmax(const void* dSrc, int src_dtype, int64_t n, float* dAbsmax, void* stream);
int astergemm_quantize_fp8_tensor(const void* dSrc, int src_dtype, int64_t n, uint8_t* dDst,
                                  float* dScale, void* stream);
int astergemm_quantize_mxfp4(const void* dSrc, int src_dtype, int64_t rows, int64_t K,
                             int64_t ld_src, uint8_t* dPacked, uint8_t* dScales,
                             void* stream);
/* The same with the scale plane written in `scales_layout` (astergemm_mx_layout):
 * ASTERGEMM_MX_ROWS = astergemm_quantize_mxfp4; ASTERGEMM_MX_LANES128 = dScales
 * holds astergemm_mx_lanes128_bytes(rows, K) bytes in the order of
 * astergemm_shuffle_scales_e8m0_lanes128 (K % 256 == 0; the bytes of rows past
 * `rows` in the last group are left as they are: those rows are never stored).
 * The packed elements are the same bytes either way. */
int astergemm_quantize_mxfp4_ex(const void* dSrc, int src_dtype, int64_t rows, int64_t K,
                                int64_t ld_src, uint8_t* dPacked, uint8_t* dScales,
                                int scales_layout, void* stream);

/* The pre-shuffles above on the device (device to device, on `stream`), for a
 * caller whose weights are already in HBM (e.g. straight out of the quantisers):
 * dSrc[N, K] row-major -> dDst in the order `operand_path` names for
 * `dtype_ab`: DIRECT_B = astergemm_shuffle_weight_16 (16-bit) or
 * astergemm_shuffle_weight_8 (fp8, MXFP4; dMxSrc -> dMxDst in
 * astergemm_shuffle_scales_e8m0 order); DIRECT_B_K8 =
 * astergemm_shuffle_weight_k8_16 (16-bit) or astergemm_shuffle_weight_8 (fp8;
 * MXFP4, with the plane in astergemm_shuffle_scales_e8m0_lanes order);
 * DIRECT_AB (16-bit only) = DIRECT_B's order, one call per operand (A with
 * N = M).  The same
 * size rules as the host functions; source and destination distinct and
 * 16-byte aligned (scale planes 8-byte; ignored unless MXFP4).  The reference
 * shuffles on the host on every call
 * (test_102_gemm_python_multitile_g2s_directb_cdna4.py:446-467).             */
int astergemm_preshuffle(int dtype_ab, int operand_path, int64_t N, int64_t K, const void* dSrc,
                         void* dDst, const uint8_t* dMxSrc, uint8_t* dMxDst, void* stream);
/* astergemm_shuffle_scales_e8m0_lanes128 on the device, for activations that are
 * already quantised: dMxSrc[M, K/32] row-major -> dMxDst (astergemm_mx_lanes128_bytes
 * (M, K) bytes, rows past M get 127).  Distinct, 16-byte aligned planes. */
int astergemm_preshuffle_scales_a(int64_t M, int64_t K, const uint8_t* dMxSrc, uint8_t* dMxDst,
                                  void* stream);

/* ---- weight artefact files (host side) -------------------------------------
 * A weight matrix B[N, K] on disk in the bytes the kernels stream, so that
 * loading is one read + one upload: no conversion, no permutation.  The
 * reference has no file format for this: its execute_fn pre-shuffles B with
 * shuffle_weight on every call
 * (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:440-467,
 * contrib/kittens/test/kittens_helpers.py:90-119) and its fp8 tests convert on
 * the host each time (test/integration/test_conversion_pack_e2e.py:91-167).
 *
 * File = this 128-byte little-endian header, then the payload at
 * payload_offset (N rows; layout ASTERGEMM_OPERAND_LDS = row-major,
 * ASTERGEMM_OPERAND_DIRECT_B = astergemm_shuffle_weight_16 order,
 * ASTERGEMM_OPERAND_DIRECT_B_K8 = astergemm_shuffle_weight_k8_16 order for the
 * 16-bit dtypes; for fp8 and MXFP4 both ASTERGEMM_OPERAND_DIRECT_B and
 * ASTERGEMM_OPERAND_DIRECT_B_K8 = astergemm_shuffle_weight_8 order), then for
 * MXFP4 the e8m0 plane [N, K/32] at scales_offset (layout DIRECT_B: in
 * astergemm_shuffle_scales_e8m0 order, DIRECT_B_K8: in
 * astergemm_shuffle_scales_e8m0_lanes order).
 * Sections start on 256-byte boundaries.  FP8 carries its tensor scale in the
 * header.  Checksums are CRC-32 (the zlib polynomial) of each section.       */
#define ASTERGEMM_WEIGHT_VERSION 1u
typedef struct astergemm_weight_header {
  char magic[8];           /* "ASTGEMW\0"                                   */
  uint32_t version;        /* ASTERGEMM_WEIGHT_VERSION                      */
  uint32_t header_bytes;   /* 128                                           */
  uint32_t dtype;          /* astergemm_dtype of the stored elements        */
  uint32_t layout;         /* astergemm_operand_path                        */
  uint32_t scale_mode;     /* astergemm_scale_mode implied by dtype         */
  float tensor_scale;      /* FP8: the per-tensor scale; else 1.0           */
  int64_t N, K;
  int64_t payload_offset, payload_bytes;
  int64_t scales_offset, scales_bytes; /* 0, 0 unless MXFP4                 */
  uint32_t payload_crc32, scales_crc32;
  uint8_t reserved[40];
} astergemm_weight_header;

uint32_t astergemm_weight_crc32(const void* data, size_t bytes);
/* Fills a header (offsets, sizes, scale mode) for the given matrix; the
 * caller writes the sections and their checksums. */
int astergemm_weight_header_init(astergemm_weight_header* h, int dtype, int layout,
                                 int64_t N, int64_t K, float tensor_scale);
/* Validates the header of a file image (magic, version, sizes against N, K
 * and dtype, sections inside the file) and copies it to *out. */
int astergemm_weight_header_check(const void* file, size_t file_bytes,
                                  astergemm_weight_header* out);
/* header_check + both checksums over the whole file image. */
int astergemm_weight_verify(const void* file, size_t file_bytes);
/* The astergemm_config for C[M, N] = A[M, K] * B^T with this weight. */
int astergemm_weight_config(const astergemm_weight_header* h, int64_t M, int dtype_c,
                            astergemm_config* cfg);

/* ---- diagnostics (not part of the GEMM path; no reference interface) -------
 * The MFMA rate (TFLOP/s) the device reaches on given operand values with
 * nothing else going on: independent MFMAs of dtype_ab's instruction over
 * registers filled once from dSample (operand bytes as a GEMM would read
 * them: at least 4096, a multiple of 16), for about target_ms milliseconds,
 * the first operand held for four instructions in a row as in the GEMM loops.
 * Under the board's power limit the rate depends on the values (zeros run near
 * the published peak, random data well below), so this is a measured
 * reference to read a GEMM's rate against next to the published peak -- not a
 * proven upper bound.  Synchronises the stream and allocates a small buffer.
 * The reference takes its peak from a table (_PEAK_TFLOPS_F16_BY_MCPU,
 * contrib/kittens/test/bench/bench_harness.py:31-41) and measures nothing.   */
int astergemm_diag_mfma_rate(int dtype_ab, const void* dSample, int64_t sample_bytes,
                             int target_ms, double* tflops, void* stream);

/* ---- runtime seam: one function per hip_* function of the reference's
 * nanobind module (RuntimeModule.cpp:140-418).  aster_rt_function_free is a
 * no-op here (the reference frees the heap cell of its handle, :221-226) and
 * aster_rt_module_launch_kernel_ex (:256-300) runs clusters of (1,1,1) as a
 * plain launch and refuses larger ones with ASTERGEMM_ENOTSUP: gfx950 has no
 * cluster launch (the reference uses it for gfx1250 only).                   */
int aster_rt_init(void);
int aster_rt_peek_at_last_error(void);
int aster_rt_clear_last_error(void);
int aster_rt_get_device_count(int* count);
int aster_rt_set_device(int device);
int aster_rt_get_device(int* device);
int aster_rt_device_reset(void);
int aster_rt_device_synchronize(void);
int aster_rt_get_device_props(int device, astergemm_device_props* out);
int aster_rt_malloc(void** dptr, size_t bytes);
int aster_rt_free(void* dptr);
int aster_rt_memcpy_h2d(void* dst, const void* src, size_t bytes);
int aster_rt_memcpy_d2h(void* dst, const void* src, size_t bytes);
int aster_rt_memcpy_d2d(void* dst, const void* src, size_t bytes);
int aster_rt_memset(void* dst, int value, size_t bytes);
int aster_rt_module_load_data(const void* image, size_t bytes, void** module);
int aster_rt_module_get_function(void* module, const char* name, void** fn);
int aster_rt_module_unload(void* module);
/* kernel_params: array of pointers to each argument, kept alive by caller. */
int aster_rt_module_launch_kernel(void* fn, unsigned gx, unsigned gy,
                                  unsigned gz, unsigned bx, unsigned by,
                                  unsigned bz, unsigned shared_bytes,
                                  void* stream, void** kernel_params);
int aster_rt_function_free(void* fn);
int aster_rt_module_launch_kernel_ex(void* fn, unsigned gx, unsigned gy, unsigned gz,
                                     unsigned bx, unsigned by, unsigned bz,
                                     unsigned cluster_x, unsigned cluster_y,
                                     unsigned cluster_z, unsigned shared_bytes,
                                     void* stream, void** kernel_params);
int aster_rt_event_create(void** event);
int aster_rt_event_destroy(void* event);
int aster_rt_event_record(void* event, void* stream);
int aster_rt_event_synchronize(void* event);
int aster_rt_event_elapsed_ms(void* start, void* stop, float* ms);
int aster_rt_stream_create(void** stream);
int aster_rt_stream_destroy(void* stream);
int aster_rt_stream_synchronize(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ASTERGEMM_H_ */
