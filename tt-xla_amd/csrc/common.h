// Shared host/device helpers for libttpa (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <atomic>

#include "pointer_words.h"
#include "ttpa.h"

namespace ttpa {

// ---- host side -------------------------------------------------------------
// Records a printf-style message for ttpa_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);
int device_cus();

// Events armed by ttpa_profile_next_attention(); take_profile_events() hands them to the
// launcher that times its dominant kernel and disarms them.
void take_profile_events(hipEvent_t &before, hipEvent_t &after);
// Arms events again from inside the library (a call of two launches hands `after` on to its second one).
void arm_profile_events(void *before, void *after);

// Launches a call's dominant kernel.  Armed events ride on the dispatch itself, so they read the
// kernel's own begin and end timestamps (what a profiler reports for the dispatch) and not the
// gaps in front of and behind it, which events recorded around a launch include.
template <typename... Params, typename... Args>
inline void launch_dominant(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds, hipStream_t st,
                            Args... args) {
  hipEvent_t before, after;
  take_profile_events(before, after);
  if (before || after)
    hipExtLaunchKernelGGL(kernel, grid, block, static_cast<uint32_t>(lds), st, before, after, 0u, args...);
  else
    kernel<<<grid, block, lds, st>>>(args...);
}

// Raises the dynamic-LDS limit of `kernel` to `bytes` on the current device, once per device:
// `done_devices` is the call site's own record (one bit per device ordinal; ordinals from 64
// on are set on every call).  Returns false when the runtime refuses.
bool ensure_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done_devices);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define TTPA_REQUIRE(cond, ...)                                            \
  do {                                                                     \
    if (!(cond)) return ::ttpa::fail(TTPA_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

// ---- device side -----------------------------------------------------------
constexpr int kWave = 64;

// DPP controls valid on gfx9: each moves data inside a row of 16 lanes.
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane ^ 7
constexpr int kDppMirror = 0x140;     // lane ^ 15

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) {
  return __builtin_bit_cast(float, w & 0xffff0000u);
}

// two floats -> packed bfloat16 pair (lo in the low half), round to nearest even
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float float_pair __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
  const float_pair f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16_pair));
}

// float -> bfloat16 bits, round to nearest even (NaN stays NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ int64_t load_index(const void *p, int is_i64, int64_t i) {
  return is_i64 ? static_cast<const int64_t *>(p)[i]
                : static_cast<int64_t>(static_cast<const int32_t *>(p)[i]);
}

// ---- block-float-8 ---------------------------------------------------------
// A group of 16 values shares the exponent byte e (largest biased bfloat16 exponent of the
// group); an element byte is 128 + v with the signed mantissa v in [-127, 127] and decodes
// to v * 2^(e - 133).  Offset binary is chosen for the readers: one byte permute makes a
// half-precision number out of an element byte, with no sign handling.
// Encodes 16 bfloat16 values held as 8 packed dwords (element 2j in the low half of
// w[j]).  Returns the shared exponent; out[0..3] receive the 16 element bytes.
__device__ __forceinline__ uint32_t bfp8_encode16(const uint32_t (&w)[8], uint32_t (&out)[4]) {
  uint32_t emax = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t e0 = (w[j] >> 7) & 0xffu, e1 = (w[j] >> 23) & 0xffu;
    emax = max(emax, max(e0, e1));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) out[j] = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t h = (i & 1) ? (w[i >> 1] >> 16) : (w[i >> 1] & 0xffffu);
    const uint32_t ex = (h >> 7) & 0xffu;
    const uint32_t sig = min(ex, 1u) * (0x80u | (h & 0x7fu));  // zero / subnormal: 0
    const uint32_t sh = min(emax - ex + 1u, 16u);  // >= 1
    // round to nearest even without comparisons (they would each cost a scalar mask register):
    // add half an ulp minus one plus the bit that will become the last kept one, then shift
    uint32_t q = (sig + ((1u << (sh - 1u)) - 1u) + ((sig >> sh) & 1u)) >> sh;
    q = min(q, 127u);
    // 128 + q for a positive, 128 - q for a negative element
    const uint32_t neg = (h >> 15) & 1u;
    const uint32_t byte = 128u + q - 2u * q * neg;
    out[i >> 2] |= byte << (8 * (i & 3));
  }
  return emax;
}

// Decodes one element byte with shared exponent e to float: (byte - 128) * 2^(e-133).
__device__ __forceinline__ float bfp8_decode(uint32_t byte, float group_scale) {
  return static_cast<float>(static_cast<int>(byte) - 128) * group_scale;
}
__device__ __forceinline__ float bfp8_group_scale(uint32_t e) {
  return __builtin_ldexpf(1.0f, static_cast<int>(e) - 133);
}

// Byte address inside the workgroup's LDS allocation of a __shared__ object.  LDS-DMA
// destinations are absolute LDS addresses: when a kernel also has static __shared__ arrays the
// dynamic segment does not start at 0.
__device__ __forceinline__ uint32_t lds_address(const void *shared_ptr) {
  return (uint32_t)reinterpret_cast<uintptr_t>(
      (const __attribute__((address_space(3))) unsigned char *)shared_ptr);
}

// 64 lanes x 16 bytes, global memory -> 1 KiB of LDS starting at byte address `lds_addr`
// (wavefront-uniform, passed in M0); lane l's 16 bytes land at lds_addr + 16 l.  Written as
// assembly so that the compiler does not make every later LDS read wait for these loads: the
// kernels wait for them themselves (vmcnt(0)) before the barrier that publishes a tile.  Lanes
// switched off by the execution mask transfer nothing.
__device__ __forceinline__ void dma16(const void *uniform_base, uint32_t lane_bytes, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_bytes), "s"(uniform_base), "s"(lds_addr)
               : "memory", "m0");
}
// The same as a non-temporal load, for data that is read once (a decode pass over the cache): a
// launch that streams a few hundred MB runs 15 % faster with the hint than without.
__device__ __forceinline__ void dma16_streaming(const void *uniform_base, uint32_t lane_bytes, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
               :
               : "v"(lane_bytes), "s"(uniform_base), "s"(lds_addr)
               : "memory", "m0");
}
// Four non-temporal ones at consecutive KiB of LDS behind ONE write of M0: the instruction's immediate
// offset moves the LDS address as well as the global one, so load i (offset 1024 i) reads
// uniform_base + lane_bytes[i] and lands at lds_addr + 1024 i when the caller passes
// uniform_base - 1024 i as its base (bases[i]).  Every write of M0 waits until the load before it
// has been taken by the address unit; this form waits once in four.
__device__ __forceinline__ void dma16_streaming_quad(const void *const (&bases)[4], const uint32_t (&lane_bytes)[4],
                                           uint32_t lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %8\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %4 nt\n\t"
      "global_load_lds_dwordx4 %1, %5 offset:1024 nt\n\t"
      "global_load_lds_dwordx4 %2, %6 offset:2048 nt\n\t"
      "global_load_lds_dwordx4 %3, %7 offset:3072 nt"
      :
      : "v"(lane_bytes[0]), "v"(lane_bytes[1]), "v"(lane_bytes[2]), "v"(lane_bytes[3]), "s"(bases[0]),
        "s"(bases[1]), "s"(bases[2]), "s"(bases[3]), "s"(lds_addr)
      : "memory", "m0");
}
// The same without the non-temporal hint (tiles that other workgroups read again).
__device__ __forceinline__ void dma16_quad(const void *const (&bases)[4], const uint32_t (&lane_bytes)[4], uint32_t lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %8\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %4\n\t"
      "global_load_lds_dwordx4 %1, %5 offset:1024\n\t"
      "global_load_lds_dwordx4 %2, %6 offset:2048\n\t"
      "global_load_lds_dwordx4 %3, %7 offset:3072"
      :
      : "v"(lane_bytes[0]), "v"(lane_bytes[1]), "v"(lane_bytes[2]), "v"(lane_bytes[3]), "s"(bases[0]),
        "s"(bases[1]), "s"(bases[2]), "s"(bases[3]), "s"(lds_addr)
      : "memory", "m0");
}
// The same for callers whose base / LDS address the compiler cannot prove uniform: both are
// read from the first active lane, the address word by word (address_from_words).
__device__ __forceinline__ void dma16_uniform(const void *uniform_base, uint32_t lane_bytes, uint32_t lds_addr) {
  const uint64_t ub = reinterpret_cast<uint64_t>(uniform_base);
  const int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)ub);
  const int hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(ub >> 32));
  dma16(reinterpret_cast<const void *>(address_from_words(lo, hi)), lane_bytes,
        (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr));
}
__device__ __forceinline__ void dma16_lane(const void *lane_ptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(lane_ptr), "s"(lds_addr)
               : "memory", "m0");
}


}  // namespace ttpa
