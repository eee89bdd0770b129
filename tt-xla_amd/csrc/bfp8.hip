// Block-float-8 codec on flat arrays: 16 bfloat16 values <-> 16 element bytes + 1
// shared exponent byte.  One thread owns one group.
#include "common.h"

namespace ttpa {
namespace {

__global__ __launch_bounds__(256) void bfp8_quantize_kernel(const uint16_t *src, uint8_t *elem,
                                                            uint8_t *exps, int64_t groups) {
  int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= groups) return;
  const uint4 *p = reinterpret_cast<const uint4 *>(src + g * 16);
  uint4 lo = p[0], hi = p[1];
  uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  uint32_t bytes[4];
  uint32_t e = bfp8_encode16(w, bytes);
  *reinterpret_cast<uint4 *>(elem + g * 16) = make_uint4(bytes[0], bytes[1], bytes[2], bytes[3]);
  exps[g] = (uint8_t)e;
}

__global__ __launch_bounds__(256) void bfp8_dequantize_kernel(const uint8_t *elem,
                                                              const uint8_t *exps, uint16_t *dst,
                                                              int64_t groups) {
  int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= groups) return;
  uint4 b = *reinterpret_cast<const uint4 *>(elem + g * 16);
  uint32_t bytes[4] = {b.x, b.y, b.z, b.w};
  float sc = bfp8_group_scale(exps[g]);
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 16; i += 2) {
    float f0 = bfp8_decode((bytes[i >> 2] >> (8 * (i & 3))) & 0xffu, sc);
    float f1 = bfp8_decode((bytes[(i + 1) >> 2] >> (8 * ((i + 1) & 3))) & 0xffu, sc);
    // exact: a 7-bit magnitude times a power of two is a bfloat16
    o[i >> 1] = (__builtin_bit_cast(uint32_t, f0) >> 16) | (__builtin_bit_cast(uint32_t, f1) & 0xffff0000u);
  }
  uint4 *q = reinterpret_cast<uint4 *>(dst + g * 16);
  q[0] = make_uint4(o[0], o[1], o[2], o[3]);
  q[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

}  // namespace
}  // namespace ttpa

using namespace ttpa;

extern "C" int ttpa_bfp8_quantize(const void *src_bf16, void *elem_u8, void *exps_u8,
                                  int64_t n_elems, void *stream) {
  TTPA_REQUIRE(src_bf16 && elem_u8 && exps_u8, "null pointer argument");
  TTPA_REQUIRE(n_elems >= 0 && n_elems % 16 == 0, "element count must be a multiple of 16");
  TTPA_REQUIRE(aligned16(src_bf16) && aligned16(elem_u8), "operands must be 16-byte aligned");
  if (n_elems == 0) return TTPA_OK;
  int64_t groups = n_elems / 16;
  bfp8_quantize_kernel<<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
                         static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint16_t *>(src_bf16), static_cast<uint8_t *>(elem_u8),
      static_cast<uint8_t *>(exps_u8), groups);
  return check_launch("bfp8_quantize");
}

extern "C" int ttpa_bfp8_dequantize(const void *elem_u8, const void *exps_u8, void *dst_bf16,
                                    int64_t n_elems, void *stream) {
  TTPA_REQUIRE(elem_u8 && exps_u8 && dst_bf16, "null pointer argument");
  TTPA_REQUIRE(n_elems >= 0 && n_elems % 16 == 0, "element count must be a multiple of 16");
  TTPA_REQUIRE(aligned16(dst_bf16) && aligned16(elem_u8), "operands must be 16-byte aligned");
  if (n_elems == 0) return TTPA_OK;
  int64_t groups = n_elems / 16;
  bfp8_dequantize_kernel<<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint8_t *>(elem_u8), static_cast<const uint8_t *>(exps_u8),
      static_cast<uint16_t *>(dst_bf16), groups);
  return check_launch("bfp8_dequantize");
}
