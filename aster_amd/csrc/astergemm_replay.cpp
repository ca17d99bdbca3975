// astergemm_replay: launch one GEMM configuration N times through the C-ABI and
// print per-launch timing statistics.  A plain executable with no interpreter in
// front of it, so it can sit directly after `rocprofv3 ... --`.
//
// The reference profiles its kernels by replaying a pre-compiled code object
// under rocprofv3 (contrib/kittens/rocprof-kittens-bench.sh:44, 103-112; two
// phases because its compiler cannot run under the profiler).  Nothing is
// compiled at run time here, so the replay is this one program.
//
//   astergemm_replay --m 8192 --n 8192 --k 8192 --ab bf16 --c bf16 --iters 100
//                    [--warmup 20] [--tile 256] [--family tile|skinny|auto]
//                    [--variant ID] [--flush BYTES] [--bias] [--json] [--calib BYTES]
//                    [--direct-b | --direct-b-k8 | --direct-ab]   (B taken as pre-shuffled in the
//                                    reference's order / in K8 order / A and B both in the
//                                    reference's order; timing only, the fill is random)
//                    [--normal]      (operands as the benchmark makes them: N(0,1) sources, for
//                                    bf16 / f16 times 0.02, for fp8 / MXFP4 quantised on the device
//                                    and, with --direct-b-k8, pre-shuffled on the device: valid
//                                    operands, so that counters describe what the benchmark times)
//                    [--same-rows]   (with --normal, 16-bit operands: every row of A and of B a copy of
//                                    its first row: the operand values a kernel sees do not change
//                                    when all its transfers are pointed at one row, so the cost of
//                                    the memory path can be told from the cost of the operand bits)
//                    [--zeros]       (all-zero operands instead of the random fill: what the clock does
//                                    when the operand bits cost nothing)
//                    [--mx-a-lanes]  (MXFP4: A's e8m0 plane in lane order, mx_a_layout LANES128;
//                                    needs --normal and --direct-b-k8)
//   astergemm_replay --quantize fp8|mxfp4 --m ROWS --k K --iters 100
//                    (operand quantiser on a ROWS x K fp32 source instead of a GEMM)
//
// --calib BYTES first copies BYTES device-to-device three times: a copy kernel that
// reads and writes a known number of bytes, against which the counters of a
// hardware-counter run (FETCH_SIZE, WRITE_SIZE) can be scaled.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

#include "astergemm.h"

static int dtype_of(const char* s) {
  if (!strcmp(s, "f16")) return ASTERGEMM_F16;
  if (!strcmp(s, "bf16")) return ASTERGEMM_BF16;
  if (!strcmp(s, "fp8") || !strcmp(s, "fp8_e4m3")) return ASTERGEMM_FP8_E4M3;
  if (!strcmp(s, "mxfp4") || !strcmp(s, "fp4")) return ASTERGEMM_MXFP4;
  if (!strcmp(s, "f32")) return ASTERGEMM_F32;
  fprintf(stderr, "unknown dtype %s\n", s);
  exit(2);
}

#define CHECK(call)                                                          \
  do {                                                                       \
    int _rc = (call);                                                        \
    if (_rc != 0) {                                                          \
      fprintf(stderr, "%s failed: %d %s\n", #call, _rc, astergemm_last_error()); \
      return 1;                                                              \
    }                                                                        \
  } while (0)

// xorshift bytes; for 16-bit floats keep exponents near 1.0 * 2^-6 so nothing
// overflows: sign random, exponent in a narrow band, mantissa random.
static void fill(std::vector<uint8_t>& buf, int dtype, uint64_t seed) {
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + 1;
  auto next = [&]() {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return x;
  };
  if (dtype == ASTERGEMM_BF16 || dtype == ASTERGEMM_F16) {
    uint16_t* p = (uint16_t*)buf.data();
    const size_t n = buf.size() / 2;
    for (size_t i = 0; i < n; ++i) {
      const uint64_t r = next();
      if (dtype == ASTERGEMM_BF16) {
        const uint16_t e = (uint16_t)(118 + (r & 3));  // 2^-9 .. 2^-6
        p[i] = (uint16_t)(((r >> 8) & 1) << 15 | e << 7 | ((r >> 16) & 0x7F));
      } else {
        const uint16_t e = (uint16_t)(6 + (r & 3));
        p[i] = (uint16_t)(((r >> 8) & 1) << 15 | e << 10 | ((r >> 16) & 0x3FF));
      }
    }
  } else if (dtype == ASTERGEMM_FP8_E4M3) {
    for (size_t i = 0; i < buf.size(); ++i) {
      uint8_t b = (uint8_t)next();
      if ((b & 0x7F) == 0x7F) b &= 0xFE;  // no NaN codes
      buf[i] = b;
    }
  } else {
    for (size_t i = 0; i < buf.size(); ++i) buf[i] = (uint8_t)next();
  }
}


// N(0,1) * scale by Box-Muller over xorshift64 (synthetic data, not the benchmark's generator)
static std::vector<float> normal(size_t n, uint64_t seed, float scale) {
  std::vector<float> out(n);
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + 88172645463325252ull;
  auto uni = [&]() {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return ((double)(x >> 11) + 0.5) * (1.0 / 9007199254740992.0);  // (0, 1)
  };
  for (size_t i = 0; i < n; i += 2) {
    const double r = sqrt(-2.0 * log(uni())), t = 6.283185307179586 * uni();
    out[i] = (float)(r * cos(t)) * scale;
    if (i + 1 < n) out[i + 1] = (float)(r * sin(t)) * scale;
  }
  return out;
}

static uint16_t bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// --quantize: time astergemm_quantize_fp8_tensor / astergemm_quantize_mxfp4 on a rows x K
// fp32 source, one event pair per call on the null stream.
static int run_quantize(const char* kind, long long rows, long long K, int iters, int warmup) {
  CHECK(aster_rt_init());
  const size_t n = (size_t)rows * (size_t)K;
  std::vector<float> h(n);
  uint64_t x = 88172645463325252ull;
  for (size_t i = 0; i < n; ++i) {
    x ^= x << 13, x ^= x >> 7, x ^= x << 17;
    h[i] = (float)((double)(int64_t)x * (1.0 / 9223372036854775808.0));  // (-1, 1)
  }
  void *src, *dst, *sc, *e0, *e1;
  CHECK(aster_rt_malloc(&src, n * 4));
  CHECK(aster_rt_malloc(&dst, n));
  CHECK(aster_rt_malloc(&sc, n / 32 + 256));
  CHECK(aster_rt_memcpy_h2d(src, h.data(), n * 4));
  CHECK(aster_rt_event_create(&e0));
  CHECK(aster_rt_event_create(&e1));
  const bool fp8 = !strcmp(kind, "fp8");
  std::vector<double> us;
  for (int i = 0; i < iters; ++i) {
    CHECK(aster_rt_event_record(e0, nullptr));
    if (fp8) CHECK(astergemm_quantize_fp8_tensor(src, ASTERGEMM_F32, (int64_t)n, (uint8_t*)dst, (float*)sc, nullptr));
    else CHECK(astergemm_quantize_mxfp4(src, ASTERGEMM_F32, rows, K, 0, (uint8_t*)dst, (uint8_t*)sc, nullptr));
    CHECK(aster_rt_event_record(e1, nullptr));
    CHECK(aster_rt_event_synchronize(e1));
    float ms = 0;
    CHECK(aster_rt_event_elapsed_ms(e0, e1, &ms));
    if (i >= warmup) us.push_back(ms * 1e3);
  }
  std::sort(us.begin(), us.end());
  const double p50 = us[us.size() / 2];
  // algorithmic bytes: fp8 reads the source twice (absmax, encode) and writes n bytes;
  // mxfp4 reads it once and writes n/2 + n/32 bytes
  const double bytes = fp8 ? (double)n * 9.0 : (double)n * (4.0 + 0.5 + 1.0 / 32.0);
  printf("quantize_%s rows=%lld K=%lld  p50 %.2f us  %.1f GB/s (algorithmic bytes %.0f)\n", kind,
         rows, K, p50, bytes / p50 * 1e-3, bytes);
  return 0;
}

int main(int argc, char** argv) {
  astergemm_config cfg;
  memset(&cfg, 0, sizeof(cfg));
  cfg.M = cfg.N = cfg.K = 8192;
  cfg.dtype_ab = ASTERGEMM_BF16;
  cfg.dtype_c = ASTERGEMM_BF16;
  int iters = 100, warmup = 20, json = 0, use_normal = 0, same_rows = 0, use_zeros = 0;
  long long flush = 0, calib = 0;
  const char* quantize = nullptr;
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i];
    auto val = [&]() -> const char* {
      if (i + 1 >= argc) {
        fprintf(stderr, "%s needs a value\n", a.c_str());
        exit(2);
      }
      return argv[++i];
    };
    if (a == "--m") cfg.M = atoll(val());
    else if (a == "--n") cfg.N = atoll(val());
    else if (a == "--k") cfg.K = atoll(val());
    else if (a == "--ab") cfg.dtype_ab = dtype_of(val());
    else if (a == "--c") cfg.dtype_c = dtype_of(val());
    else if (a == "--iters") iters = atoi(val());
    else if (a == "--warmup") warmup = atoi(val());
    else if (a == "--tile") cfg.wg_tile_m = cfg.wg_tile_n = atoi(val());
    else if (a == "--variant") cfg.variant = atoi(val());
    else if (a == "--flush") flush = atoll(val());
    else if (a == "--calib") calib = atoll(val());
    else if (a == "--direct-b") cfg.operand_path = ASTERGEMM_OPERAND_DIRECT_B;
    else if (a == "--direct-b-k8") cfg.operand_path = ASTERGEMM_OPERAND_DIRECT_B_K8;
    else if (a == "--direct-ab") cfg.operand_path = ASTERGEMM_OPERAND_DIRECT_AB;
    else if (a == "--bias") cfg.has_bias = 1;
    else if (a == "--normal") use_normal = 1;
    else if (a == "--same-rows") same_rows = 1;
    else if (a == "--zeros") use_zeros = 1;
    else if (a == "--mx-a-lanes") cfg.mx_a_layout = ASTERGEMM_MX_LANES128;
    else if (a == "--json") json = 1;
    else if (a == "--quantize") quantize = val();
    else if (a == "--family") {
      const char* f = val();
      cfg.family = !strcmp(f, "tile") ? ASTERGEMM_KERNEL_TILE
                   : !strcmp(f, "skinny") ? ASTERGEMM_KERNEL_SKINNY : ASTERGEMM_KERNEL_AUTO;
    } else {
      fprintf(stderr, "unknown argument %s\n", a.c_str());
      return 2;
    }
  }
  if (cfg.dtype_ab == ASTERGEMM_FP8_E4M3) cfg.scale_mode = ASTERGEMM_SCALE_TENSOR;
  if (cfg.dtype_ab == ASTERGEMM_MXFP4) cfg.scale_mode = ASTERGEMM_SCALE_MX32;
  if (cfg.mx_a_layout == ASTERGEMM_MX_LANES128 &&
      (!use_normal || cfg.operand_path != ASTERGEMM_OPERAND_DIRECT_B_K8 || cfg.dtype_ab != ASTERGEMM_MXFP4)) {
    fprintf(stderr, "--mx-a-lanes needs --ab mxfp4 --normal --direct-b-k8\n");
    return 2;
  }
  if (use_normal && cfg.dtype_ab == ASTERGEMM_F16) {
    fprintf(stderr, "--normal covers bf16, fp8 and mxfp4\n");
    return 2;
  }
  if (iters <= warmup) {
    fprintf(stderr, "--iters must exceed --warmup\n");
    return 2;
  }
  if (quantize) {
    if (strcmp(quantize, "fp8") && strcmp(quantize, "mxfp4")) {
      fprintf(stderr, "--quantize fp8|mxfp4\n");
      return 2;
    }
    return run_quantize(quantize, cfg.M, cfg.K, iters, warmup);
  }

  CHECK(aster_rt_init());
  astergemm_kernel_info info;
  CHECK(astergemm_select(&cfg, &info));

  const int bits = cfg.dtype_ab == ASTERGEMM_MXFP4 ? 4 : cfg.dtype_ab == ASTERGEMM_FP8_E4M3 ? 8 : 16;
  const size_t a_bytes = (size_t)cfg.M * cfg.K * bits / 8, b_bytes = (size_t)cfg.N * cfg.K * bits / 8;
  const size_t c_bytes = (size_t)cfg.M * cfg.N * (cfg.dtype_c == ASTERGEMM_F32 ? 4 : 2);
  astergemm_operands ops;
  memset(&ops, 0, sizeof(ops));
  void *dA, *dB, *dC;
  CHECK(aster_rt_malloc(&dA, a_bytes));
  CHECK(aster_rt_malloc(&dB, b_bytes));
  CHECK(aster_rt_malloc(&dC, c_bytes));
  ops.dA = dA;
  ops.dB = dB;
  ops.dC = dC;
  if (!use_normal) {
    std::vector<uint8_t> ha(a_bytes), hb(b_bytes);
    if (!use_zeros) {  // --zeros: all-zero operands (the vectors are value-initialised)
      fill(ha, cfg.dtype_ab, 42);
      fill(hb, cfg.dtype_ab, 43);
    }
    CHECK(aster_rt_memcpy_h2d(dA, ha.data(), a_bytes));
    CHECK(aster_rt_memcpy_h2d(dB, hb.data(), b_bytes));
    if (cfg.scale_mode == ASTERGEMM_SCALE_TENSOR) {
      const float s[2] = {0.01f, 0.02f};
      void* ds;
      CHECK(aster_rt_malloc(&ds, 256));
      CHECK(aster_rt_memcpy_h2d(ds, s, sizeof(s)));
      ops.dScaleA = (const float*)ds;
      ops.dScaleB = (const float*)ds + 1;
    }
    if (cfg.scale_mode == ASTERGEMM_SCALE_MX32) {
      std::vector<uint8_t> sa((size_t)cfg.M * cfg.K / 32, 122), sb((size_t)cfg.N * cfg.K / 32, 123);
      void *da, *db;
      CHECK(aster_rt_malloc(&da, sa.size()));
      CHECK(aster_rt_malloc(&db, sb.size()));
      CHECK(aster_rt_memcpy_h2d(da, sa.data(), sa.size()));
      CHECK(aster_rt_memcpy_h2d(db, sb.data(), sb.size()));
      ops.dMxA = (const uint8_t*)da;
      ops.dMxB = (const uint8_t*)db;
    }
  } else {
    // the benchmark's operands: N(0,1) sources (16-bit: times 0.02), quantised on the device
    const bool is16 = cfg.dtype_ab == ASTERGEMM_BF16;
    for (int side = 0; side < 2; ++side) {
      const int64_t rows = side == 0 ? cfg.M : cfg.N;
      const size_t n = (size_t)rows * (size_t)cfg.K;
      void* dst = side == 0 ? dA : dB;
      std::vector<float> src = normal(n, 42 + (uint64_t)side, is16 ? 0.02f : 1.0f);
      if (is16) {
        std::vector<uint16_t> h(n);
        for (size_t i = 0; i < n; ++i) h[i] = bf16_rne(src[same_rows ? i % (size_t)cfg.K : i]);
        CHECK(aster_rt_memcpy_h2d(dst, h.data(), n * 2));
        continue;
      }
      void* dsrc;
      CHECK(aster_rt_malloc(&dsrc, n * 4));
      CHECK(aster_rt_memcpy_h2d(dsrc, src.data(), n * 4));
      const bool shuffle = side == 1 && cfg.operand_path != ASTERGEMM_OPERAND_LDS;
      void* payload = dst;
      if (shuffle) CHECK(aster_rt_malloc(&payload, side == 0 ? a_bytes : b_bytes));
      if (cfg.dtype_ab == ASTERGEMM_FP8_E4M3) {
        void* ds;
        CHECK(aster_rt_malloc(&ds, 256));
        CHECK(astergemm_quantize_fp8_tensor(dsrc, ASTERGEMM_F32, (int64_t)n, (uint8_t*)payload, (float*)ds, nullptr));
        (side == 0 ? ops.dScaleA : ops.dScaleB) = (const float*)ds;
        if (shuffle)
          CHECK(astergemm_preshuffle(cfg.dtype_ab, cfg.operand_path, rows, cfg.K, payload, dst, nullptr, nullptr, nullptr));
      } else {
        const bool lanes = side == 0 && cfg.mx_a_layout == ASTERGEMM_MX_LANES128;
        const size_t plane = lanes ? (size_t)astergemm_mx_lanes128_bytes(rows, cfg.K) : n / 32;
        void *sc, *sc2 = nullptr;
        CHECK(aster_rt_malloc(&sc, plane));
        CHECK(astergemm_quantize_mxfp4_ex(dsrc, ASTERGEMM_F32, rows, cfg.K, 0, (uint8_t*)payload, (uint8_t*)sc,
                                          lanes ? ASTERGEMM_MX_LANES128 : ASTERGEMM_MX_ROWS, nullptr));
        if (shuffle) {
          CHECK(aster_rt_malloc(&sc2, plane));
          CHECK(astergemm_preshuffle(cfg.dtype_ab, cfg.operand_path, rows, cfg.K, payload, dst, (const uint8_t*)sc,
                                     (uint8_t*)sc2, nullptr));
        }
        (side == 0 ? ops.dMxA : ops.dMxB) = (const uint8_t*)(shuffle ? sc2 : sc);
      }
      CHECK(aster_rt_device_synchronize());
      CHECK(aster_rt_free(dsrc));
      if (shuffle) CHECK(aster_rt_free(payload));
    }
  }
  if (cfg.has_bias) {
    std::vector<float> hbias((size_t)cfg.N, 0.5f);
    void* dbias;
    CHECK(aster_rt_malloc(&dbias, hbias.size() * 4));
    CHECK(aster_rt_memcpy_h2d(dbias, hbias.data(), hbias.size() * 4));
    ops.dBias = (const float*)dbias;
  }

  if (calib > 0) {
    void *src, *dst;
    CHECK(aster_rt_malloc(&src, (size_t)calib));
    CHECK(aster_rt_malloc(&dst, (size_t)calib));
    CHECK(aster_rt_memset(src, 1, (size_t)calib));
    for (int i = 0; i < 3; ++i) CHECK(aster_rt_memcpy_d2d(dst, src, (size_t)calib));
    CHECK(aster_rt_free(src));
    CHECK(aster_rt_free(dst));
  }

  std::vector<int64_t> t((size_t)iters);
  CHECK(astergemm_bench(&cfg, &ops, iters, t.data(), flush, nullptr));
  std::vector<int64_t> m(t.begin() + warmup, t.end());
  std::sort(m.begin(), m.end());
  auto pct = [&](double p) {
    long idx = lround(p / 100.0 * (double)(m.size() - 1));
    return (double)m[(size_t)std::max(0l, std::min((long)m.size() - 1, idx))];
  };
  double mean = 0;
  for (int64_t v : m) mean += (double)v;
  mean /= (double)m.size();
  const double p50 = pct(50);
  const double tflops = (double)info.flops / p50 * 1e-3, gbps = (double)info.bytes / p50;
  if (json) {
    printf("{\"kernel\": \"%s\", \"M\": %lld, \"N\": %lld, \"K\": %lld, \"grid\": %d, \"block\": %d, "
           "\"lds_bytes\": %d, \"regs\": %d, \"iters\": %d, \"warmup\": %d, \"p0_us\": %.2f, "
           "\"p10_us\": %.2f, \"p50_us\": %.2f, \"p90_us\": %.2f, \"mean_us\": %.2f, "
           "\"tflops_p50\": %.1f, \"gbps_p50\": %.1f, \"flush_bytes\": %lld}\n",
           info.name, (long long)cfg.M, (long long)cfg.N, (long long)cfg.K, info.grid_x, info.block_x,
           info.lds_bytes, info.vgprs, iters, warmup, pct(0) / 1e3, pct(10) / 1e3, p50 / 1e3,
           pct(90) / 1e3, mean / 1e3, tflops, gbps, flush);
  } else {
    printf("%s  M=%lld N=%lld K=%lld grid=%d block=%d lds=%d regs=%d\n", info.name, (long long)cfg.M,
           (long long)cfg.N, (long long)cfg.K, info.grid_x, info.block_x, info.lds_bytes, info.vgprs);
    printf("  p0 %.2f us  p10 %.2f  p50 %.2f  p90 %.2f  mean %.2f   p50: %.1f TFLOP/s  %.1f GB/s\n",
           pct(0) / 1e3, pct(10) / 1e3, p50 / 1e3, pct(90) / 1e3, mean / 1e3, tflops, gbps);
  }
  return 0;
}
