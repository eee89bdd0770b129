// A 64-bit address rebuilt from its two 32-bit words as they come back from a lane broadcast
// (the broadcast intrinsic deals in signed int).  Plain C++, so that a host test can compile it.
#pragma once

#include <stdint.h>

namespace ttpa {

// Each word goes through uint32_t before it is widened: widened as a signed int, a low word with
// bit 31 set would smear ones over the high word and turn a valid address into a wild one.
#if defined(__HIPCC__)
__host__ __device__
#endif
inline uint64_t address_from_words(int low_word, int high_word) {
  return ((uint64_t)(uint32_t)high_word << 32) | (uint64_t)(uint32_t)low_word;
}

}  // namespace ttpa
