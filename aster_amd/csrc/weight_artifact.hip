// Weight artefact files: a weight matrix B[N, K] stored in exactly the bytes a kernel of this
// library streams (row-major or pre-shuffled 16-bit elements, e4m3 bytes with their tensor
// scale, MXFP4 nibbles with their e8m0 plane), behind a fixed 128-byte little-endian header.
// Host code only: parsing, validation, the checksum and the header -> astergemm_config step.
//
// The pre-shuffled layouts are the reference's shuffle_weight order
// (contrib/kittens/test/kittens_helpers.py:90-119), which its execute_fn applies on every call
// (contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:440-467), read by
// the decode kernels, and the orders read by the stream kernels with direct B (16-bit: the K8
// order of astergemm_shuffle_weight_k8_16; fp8 and MXFP4: step order); a file written once
// replaces that per-call host permutation.
#include <cstring>

#include "astergemm_internal.h"

namespace {

const char kMagic[8] = {'A', 'S', 'T', 'G', 'E', 'M', 'W', '\0'};

// CRC-32 table (reflected polynomial 0xEDB88320), built at compile time
struct CrcTable {
  uint32_t v[256];
  constexpr CrcTable() : v() {
    for (uint32_t i = 0; i < 256; ++i) {
      uint32_t c = i;
      for (int k = 0; k < 8; ++k) c = (c & 1u) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
      v[i] = c;
    }
  }
};
constexpr CrcTable kCrc{};

int fail(const char* why) {
  astergemm::set_error("astergemm_weight: %s", why);
  return ASTERGEMM_EINVAL;
}

}  // namespace

extern "C" uint32_t astergemm_weight_crc32(const void* data, size_t bytes) {
  const uint8_t* p = (const uint8_t*)data;
  uint32_t c = 0xFFFFFFFFu;
  for (size_t i = 0; i < bytes; ++i) c = kCrc.v[(c ^ p[i]) & 0xFFu] ^ (c >> 8);
  return c ^ 0xFFFFFFFFu;
}

extern "C" int astergemm_weight_header_init(astergemm_weight_header* h, int dtype, int layout,
                                            int64_t N, int64_t K, float tensor_scale) {
  if (!h) return fail("null header");
  memset(h, 0, sizeof(*h));
  memcpy(h->magic, kMagic, 8);
  h->version = ASTERGEMM_WEIGHT_VERSION;
  h->header_bytes = (uint32_t)sizeof(*h);
  h->dtype = (uint32_t)dtype;
  h->layout = (uint32_t)layout;
  h->N = N;
  h->K = K;
  h->tensor_scale = 1.0f;
  switch (dtype) {
    case ASTERGEMM_F16:
    case ASTERGEMM_BF16: h->scale_mode = ASTERGEMM_SCALE_NONE; break;
    case ASTERGEMM_FP8_E4M3:
      h->scale_mode = ASTERGEMM_SCALE_TENSOR;
      h->tensor_scale = tensor_scale;
      break;
    case ASTERGEMM_MXFP4: h->scale_mode = ASTERGEMM_SCALE_MX32; break;
    default: return fail("dtype must be F16, BF16, FP8_E4M3 or MXFP4");
  }
  if (N <= 0 || K <= 0) return fail("N and K must be positive");
  if (dtype == ASTERGEMM_MXFP4 && K % 32 != 0) return fail("MXFP4 needs K % 32 == 0");
  if (astergemm::row_bytes(dtype, K) % 16 != 0) return fail("a row must be a multiple of 16 bytes");
  if (layout == ASTERGEMM_OPERAND_DIRECT_B || layout == ASTERGEMM_OPERAND_DIRECT_B_K8) {
    const bool is16 = dtype == ASTERGEMM_F16 || dtype == ASTERGEMM_BF16;
    // MXFP4 for the stream kernel: payload in step order, scale plane in lane order
    // (astergemm_shuffle_scales_e8m0_lanes)
    if (dtype == ASTERGEMM_MXFP4 && layout == ASTERGEMM_OPERAND_DIRECT_B_K8 &&
        (N % 64 != 0 || K % 256 != 0))
      return fail("the stream kernels' pre-shuffled MXFP4 layout needs N % 64 == 0, K % 256 == 0");
    if (is16 && (N % 16 != 0 || K % 32 != 0))
      return fail("the pre-shuffled layouts need N % 16 == 0, K % 32 == 0");
    // fp8 / MXFP4: step order (astergemm_shuffle_weight_8, astergemm_shuffle_scales_e8m0)
    if (!is16 && (N % 16 != 0 || astergemm::row_bytes(dtype, K) % 128 != 0))
      return fail("the pre-shuffled layout of fp8 / MXFP4 needs N % 16 == 0 and rows of whole 128-byte steps");
  } else if (layout != ASTERGEMM_OPERAND_LDS) {
    return fail("unknown layout");
  }
  // sections start on 256-byte boundaries
  h->payload_offset = 256;
  h->payload_bytes = N * astergemm::row_bytes(dtype, K);
  if (h->scale_mode == ASTERGEMM_SCALE_MX32) {
    h->scales_offset = (h->payload_offset + h->payload_bytes + 255) & ~(int64_t)255;
    h->scales_bytes = N * (K / 32);
  }
  return 0;
}

extern "C" int astergemm_weight_header_check(const void* file, size_t file_bytes,
                                             astergemm_weight_header* out) {
  if (!file || file_bytes < sizeof(astergemm_weight_header)) return fail("file shorter than the header");
  astergemm_weight_header h;
  memcpy(&h, file, sizeof(h));
  if (memcmp(h.magic, kMagic, 8) != 0) return fail("bad magic");
  if (h.version != ASTERGEMM_WEIGHT_VERSION) return fail("unsupported version");
  if (h.header_bytes != sizeof(h)) return fail("bad header size");
  astergemm_weight_header want;
  if (int rc = astergemm_weight_header_init(&want, (int)h.dtype, (int)h.layout, h.N, h.K,
                                            h.tensor_scale))
    return rc;
  if (h.scale_mode != want.scale_mode) return fail("scale mode does not match the dtype");
  if (h.payload_bytes != want.payload_bytes || h.scales_bytes != want.scales_bytes)
    return fail("section sizes do not match N, K and the dtype");
  if (h.payload_offset < (int64_t)sizeof(h) || (h.payload_offset & 255) ||
      h.payload_offset + h.payload_bytes > (int64_t)file_bytes)
    return fail("payload section outside the file or misaligned");
  if (h.scales_bytes > 0 &&
      (h.scales_offset < h.payload_offset + h.payload_bytes || (h.scales_offset & 255) ||
       h.scales_offset + h.scales_bytes > (int64_t)file_bytes))
    return fail("scale section outside the file, misaligned or overlapping the payload");
  if (h.scale_mode == ASTERGEMM_SCALE_TENSOR && !(h.tensor_scale > 0.0f && h.tensor_scale < 3.0e38f))
    return fail("tensor scale must be positive and finite");
  if (out) *out = h;
  return 0;
}

extern "C" int astergemm_weight_verify(const void* file, size_t file_bytes) {
  astergemm_weight_header h;
  if (int rc = astergemm_weight_header_check(file, file_bytes, &h)) return rc;
  const uint8_t* p = (const uint8_t*)file;
  if (astergemm_weight_crc32(p + h.payload_offset, (size_t)h.payload_bytes) != h.payload_crc32)
    return fail("payload checksum mismatch");
  if (h.scales_bytes > 0 &&
      astergemm_weight_crc32(p + h.scales_offset, (size_t)h.scales_bytes) != h.scales_crc32)
    return fail("scale plane checksum mismatch");
  return 0;
}

extern "C" int astergemm_weight_config(const astergemm_weight_header* h, int64_t M, int dtype_c,
                                       astergemm_config* cfg) {
  if (!h || !cfg) return fail("null argument");
  memset(cfg, 0, sizeof(*cfg));
  cfg->M = M;
  cfg->N = h->N;
  cfg->K = h->K;
  cfg->dtype_ab = (int32_t)h->dtype;
  cfg->dtype_c = dtype_c;
  cfg->scale_mode = (int32_t)h->scale_mode;
  cfg->operand_path = (int32_t)h->layout;
  return 0;
}
