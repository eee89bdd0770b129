// 16x16x32 matrix-core decode kernel, head size 256.
#include "decode_mfma16_kernel.h"

namespace ttpa {
namespace decode {

bool launch_mfma16_d256(const DecodeArgs &a, hipStream_t st) {
  return launch_for_block_size<256, false>(a, st);  // bfloat16 cache only
}

}  // namespace decode
}  // namespace ttpa
