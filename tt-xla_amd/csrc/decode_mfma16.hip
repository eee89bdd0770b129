// 16x16x32 matrix-core decode kernel: which shapes it is built for, and the dispatch to the
// translation unit of the head size (kernel and launcher: decode_mfma16_kernel.h).
#include "decode_common.h"

namespace ttpa {
namespace decode {

bool launch_mfma16_d64(const DecodeArgs &a, hipStream_t st);
bool launch_mfma16_d128(const DecodeArgs &a, hipStream_t st);
bool launch_mfma16_d256(const DecodeArgs &a, hipStream_t st);

bool mfma16_decode_supported(const DecodeArgs &a, int head_size, int g) {
  const bool bfp8 = a.kv_format == TTPA_KV_BFP8;
  if (head_size != 64 && head_size != 128 && head_size != 256) return false;
  const int rows_per_load = 1024 / (head_size * (bfp8 ? 1 : 2));  // a load covers whole rows of one block
  return g <= 16 && a.users <= kMaxUsers && a.bs % rows_per_load == 0;
}

// With a.k_new set, the launch also performs the cache update of the step.
bool launch_mfma16_main(const DecodeArgs &a, int head_size, hipStream_t st) {
  switch (head_size) {
    case 64: return launch_mfma16_d64(a, st);
    case 128: return launch_mfma16_d128(a, st);
    case 256: return launch_mfma16_d256(a, st);
    default: return false;
  }
}

}  // namespace decode
}  // namespace ttpa
