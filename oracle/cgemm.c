/*
 * cgemm.c -- plain-C restatement of the reference's GEMM check.  TEST
 * INFRASTRUCTURE: cross-checks the numpy oracle and serves as a CPU baseline;
 * the product never links it.
 *
 * Formula (reference: contrib/kittens/test/bench/bench_harness.py:821, 1837):
 *     C[m][n] = sum_k float(A[m][k]) * float(B[n][k])        (fp32 accumulate)
 * with B stored N x K (contrib/kittens/gemm_config.py:94, 109).
 * Operand decoders: IEEE binary16, bfloat16, OCP e4m3
 * (test/integration/test_conversion_pack_e2e.py:79-88: gfx950 = OCP, bias 7),
 * OCP e2m1 with e8m0 block scales (32 elements per scale byte).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { DT_F16 = 0, DT_BF16 = 1, DT_FP8 = 2, DT_FP4 = 3, DT_F32 = 4 };

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static float decode_f16(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023;
  if (e == 31) return bits_f32(s | 0x7F800000u | (m << 13));
  if (e == 0) {
    float v = ldexpf((float)m, -24);
    return s ? -v : v;
  }
  return bits_f32(s | ((e + 112) << 23) | (m << 13));
}

static float decode_bf16(uint16_t h) { return bits_f32((uint32_t)h << 16); }

static float decode_e4m3(uint8_t b) {
  int e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) v = NAN;
  else if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return (b & 0x80) ? -v : v;
}

static float decode_e2m1(uint8_t c) {
  static const float t[8] = {0.f, .5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
  float v = t[c & 7];
  return (c & 8) ? -v : v;
}

static float decode_e8m0(uint8_t b) { return b == 0xFF ? NAN : ldexpf(1.0f, (int)b - 127); }

/* Decode `rows` x K elements of one operand into dst (row-major fp32).
 * ld_bytes = row pitch of the storage; mx = e8m0 plane [rows][K/32] or NULL. */
int oracle_decode(const void* src, int dtype, int64_t rows, int64_t K, int64_t ld_bytes,
                  const uint8_t* mx, float* dst) {
  for (int64_t r = 0; r < rows; ++r) {
    const uint8_t* row = (const uint8_t*)src + r * ld_bytes;
    float* o = dst + r * K;
    for (int64_t k = 0; k < K; ++k) {
      switch (dtype) {
        case DT_F16: o[k] = decode_f16(((const uint16_t*)row)[k]); break;
        case DT_BF16: o[k] = decode_bf16(((const uint16_t*)row)[k]); break;
        case DT_FP8: o[k] = decode_e4m3(row[k]); break;
        case DT_FP4: {
          uint8_t byte = row[k >> 1];
          uint8_t code = (k & 1) ? (byte >> 4) : (byte & 15);
          o[k] = decode_e2m1(code) * decode_e8m0(mx[r * (K / 32) + (k >> 5)]);
          break;
        }
        case DT_F32: o[k] = ((const float*)row)[k]; break;
        default: return -1;
      }
    }
  }
  return 0;
}

/* C[M][N] = A[M][K] . B[N][K]^T, fp32 accumulate, OpenMP over row blocks.
 * 4x4 register block of dot products; the k loop is left to the vectoriser. */
int oracle_gemm_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i0 = 0; i0 < M; i0 += 4) {
    for (int64_t j0 = 0; j0 < N; j0 += 4) {
      float acc[4][4] = {{0}};
      const int mi = (M - i0) < 4 ? (int)(M - i0) : 4;
      const int nj = (N - j0) < 4 ? (int)(N - j0) : 4;
      if (mi == 4 && nj == 4) {
        const float *a0 = A + (i0 + 0) * K, *a1 = A + (i0 + 1) * K, *a2 = A + (i0 + 2) * K,
                    *a3 = A + (i0 + 3) * K;
        const float *b0 = B + (j0 + 0) * K, *b1 = B + (j0 + 1) * K, *b2 = B + (j0 + 2) * K,
                    *b3 = B + (j0 + 3) * K;
        float c00 = 0, c01 = 0, c02 = 0, c03 = 0, c10 = 0, c11 = 0, c12 = 0, c13 = 0, c20 = 0,
              c21 = 0, c22 = 0, c23 = 0, c30 = 0, c31 = 0, c32 = 0, c33 = 0;
#pragma omp simd reduction(+ : c00, c01, c02, c03, c10, c11, c12, c13, c20, c21, c22, c23, c30, c31, c32, c33)
        for (int64_t k = 0; k < K; ++k) {
          c00 += a0[k] * b0[k]; c01 += a0[k] * b1[k]; c02 += a0[k] * b2[k]; c03 += a0[k] * b3[k];
          c10 += a1[k] * b0[k]; c11 += a1[k] * b1[k]; c12 += a1[k] * b2[k]; c13 += a1[k] * b3[k];
          c20 += a2[k] * b0[k]; c21 += a2[k] * b1[k]; c22 += a2[k] * b2[k]; c23 += a2[k] * b3[k];
          c30 += a3[k] * b0[k]; c31 += a3[k] * b1[k]; c32 += a3[k] * b2[k]; c33 += a3[k] * b3[k];
        }
        acc[0][0] = c00; acc[0][1] = c01; acc[0][2] = c02; acc[0][3] = c03;
        acc[1][0] = c10; acc[1][1] = c11; acc[1][2] = c12; acc[1][3] = c13;
        acc[2][0] = c20; acc[2][1] = c21; acc[2][2] = c22; acc[2][3] = c23;
        acc[3][0] = c30; acc[3][1] = c31; acc[3][2] = c32; acc[3][3] = c33;
      } else {
        for (int i = 0; i < mi; ++i)
          for (int j = 0; j < nj; ++j) {
            float s = 0;
            for (int64_t k = 0; k < K; ++k) s += A[(i0 + i) * K + k] * B[(j0 + j) * K + k];
            acc[i][j] = s;
          }
      }
      for (int i = 0; i < mi; ++i)
        for (int j = 0; j < nj; ++j) C[(i0 + i) * N + (j0 + j)] = acc[i][j];
    }
  }
  return 0;
}

/* Whole path on raw storage: decode both operands, multiply. C is fp32 [M][N]. */
int oracle_gemm_raw(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t K,
                    int dtype, int64_t lda_bytes, int64_t ldb_bytes, const uint8_t* mx_a,
                    const uint8_t* mx_b) {
  float* a = (float*)malloc(sizeof(float) * (size_t)(M * K));
  float* b = (float*)malloc(sizeof(float) * (size_t)(N * K));
  int rc = -1;
  if (a && b && oracle_decode(A, dtype, M, K, lda_bytes, mx_a, a) == 0 &&
      oracle_decode(B, dtype, N, K, ldb_bytes, mx_b, b) == 0)
    rc = oracle_gemm_f32(a, b, C, M, N, K);
  free(a);
  free(b);
  return rc;
}
