// 16x16x32 matrix-core decode kernel, head size 256.
#include "decode_mfma16_kernel.h"

namespace ttpa {
namespace decode {

bool launch_mfma16_d256(const DecodeArgs &a, hipStream_t st) {
  return a.kv_format == TTPA_KV_BFP8 ? launch_for_block_size<256, true>(a, st)
                                     : launch_for_block_size<256, false>(a, st);
}

}  // namespace decode
}  // namespace ttpa
