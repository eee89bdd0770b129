// Pieces shared by the bf16 and block-float-8 paged decode kernels: launch arguments,
// tile-list prefix, wave-level reductions, the partial-merge kernel and workspace sizing.
#pragma once

#include "common.h"

#include <type_traits>

namespace ttpa {
namespace decode {


constexpr int kMaxUsers = 2048;
constexpr int kTile = 64;
constexpr int kWavesPerBlock = 4;

struct DecodeArgs {
  uint16_t *out;
  int64_t out_us, out_hs;
  const uint16_t *q;
  int64_t q_us, q_hs;
  const uint8_t *k, *v;
  const int32_t *pt;
  int64_t pt_rs;
  const void *cur;
  int cur_i64;
  int users, hq, hkv, bs, w, nb;
  float scale_log2e;
  int *ws_seg;   // [users * hkv][2]: first partial slot and number of partials per segment
  float *ws_slots;
  int n_waves;
  int slot_floats;
  int kv_format;
  int window;         // > 0: only the last `window` positions up to cur_pos are attended
  // Units of the flat list that stand in front of the tiles of every non-empty segment and carry
  // no work: they charge the wavefront that opens a segment inside its range for what a change
  // of segment costs (its partial, the search, the next Q rows), so that equal ranges of units
  // take about equal time.  0: the list holds tiles only.
  int seg_units = 0;
  // Partial outputs stored as bfloat16 (16-head latent kernel: a partial there is 16 heads x 512
  // values): a slot is G * D bfloat16 values, then G running maxima and G running sums as floats.
  int partial_bf16 = 0;
  const float *sink;  // [q_heads] extra logit per head in the softmax denominator, or null
  // Fused cache update (16x16x32 kernel only): the token at cur_pos of every user is taken from
  // k_new / v_new [users][>= hkv heads][head_size] instead of the cache, and written to it.
  const uint16_t *k_new, *v_new;
  int64_t new_us, new_hs;
  // Additive mask on the scaled scores (bfloat16, natural-log units), or null: the element for
  // (user, query head, position) is mask[user * mask_us + head * mask_hs + position].  Applied by the
  // dot-product kernel (decode.hip) and by the workgroup-shared latent kernel (decode_wide.hip); the
  // entry points that take a mask launch only those.
  const uint16_t *mask = nullptr;
  int64_t mask_us = 0, mask_hs = 0;
};

// First attended position of a user whose attended range ends at `len` (exclusive).
__device__ __forceinline__ int window_lo(const DecodeArgs &a, int len) {
  return (a.window > 0 && len > a.window) ? len - a.window : 0;
}

// Attended positions of user u are [window_lo(len), len); returns the number of TILE-token tiles
// they touch.
template <int TILE = kTile>
__device__ __forceinline__ int tiles_of_user(const DecodeArgs &a, const void *__restrict__ cur,
                                             int u, int &len) {
  int64_t cp = load_index(cur, a.cur_i64, u);
  int64_t cap = (int64_t)a.w * a.bs;
  int64_t l = cp < 0 ? 0 : (cp + 1 < cap ? cp + 1 : cap);
  len = (int)l;
  return (int)((l + TILE - 1) / TILE) - window_lo(a, len) / TILE;
}

// Exclusive prefix sum of per-user unit counts (tiles, plus `extra` for a user that has any) into
// pref[0..users] and attended lengths into lens[0..users); all 256 threads.  Each position is read
// from global memory once.
template <int TILE = kTile>
__device__ inline void build_prefix(const DecodeArgs &a, const void *__restrict__ cur, int *pref,
                             int *lens, int *wave_sums, int extra = 0) {
  const int tid = threadIdx.x;
  const int per = (a.users + 255) / 256;
  const int beg = tid * per;
  const int end = min(beg + per, a.users);
  int local = 0;
  for (int u = beg; u < end; ++u) {
    int len;
    int nt = tiles_of_user<TILE>(a, cur, u, len);
    if (nt > 0) nt += extra;  // units per segment of this user
    lens[u] = len;
    pref[u + 1] = nt;  // replaced by the running sum below
    local += nt;
  }
  int incl = local;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    int o = __shfl_up(incl, d);
    if ((tid & 63) >= d) incl += o;
  }
  if ((tid & 63) == 63) wave_sums[tid >> 6] = incl;
  __syncthreads();
  int run = incl - local;
  for (int wv = 0; wv < (tid >> 6); ++wv) run += wave_sums[wv];
  if (tid == 0) pref[0] = 0;
  for (int u = beg; u < end; ++u) {
    run += pref[u + 1];
    pref[u + 1] = run;
  }
  __syncthreads();
}

// LDS probabilities are written as 16-bit values and read back as 32-bit pairs
typedef uint16_t __attribute__((may_alias)) lds_u16;
typedef uint32_t __attribute__((may_alias)) lds_u32;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// Largest value of v over the wavefront, as a wavefront-uniform number.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kDppXor1, 0xf, 0xf, true));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kDppXor2, 0xf, 0xf, true));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kDppHalfMirror, 0xf, 0xf, true));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kDppMirror, 0xf, 0xf, true));
  const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
  const uint32_t r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
  const uint32_t r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  return max(max(r0, r1), max(r2, r3));
}

// 4 element bytes (128 + v) -> two half pairs holding v * s, given s2 = (s, s) and
// c2 = (-1152 s, -1152 s) for a power of two s: (1024 + b) * s - 1152 s = (b - 128) * s.
__device__ __forceinline__ void expand4_half(uint32_t w, halfx2 s2, halfx2 c2, uint32_t &p01,
                                             uint32_t &p23) {
  const uint32_t m01 = __builtin_amdgcn_perm(0x64646464u, w, 0x04010400u);
  const uint32_t m23 = __builtin_amdgcn_perm(0x64646464u, w, 0x04030402u);
  p01 = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(halfx2, m01), s2, c2));
  p23 = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(halfx2, m23), s2, c2));
}
// two floats -> packed half pair, round to nearest even
__device__ __forceinline__ uint32_t pack_half2(float lo, float hi) {
  floatx2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, halfx2));
}

// Streaming (non-temporal) load of DW dwords: K/V are read once per launch, so they
// should not displace anything in L2 / MALL.
// `ubase` is wavefront-uniform and `lane_bytes` a 32-bit per-lane offset, which lets the
// load use the scalar-base addressing form: no per-load 64-bit address registers.
template <int DW>
__device__ __forceinline__ void load_stream(const uint16_t *ubase, uint32_t lane_bytes,
                                            uint32_t (&d)[DW]) {
  const char *p = reinterpret_cast<const char *>(ubase) + static_cast<uint64_t>(lane_bytes);
  if constexpr (DW == 4) {
    u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    d[0] = t.x, d[1] = t.y, d[2] = t.z, d[3] = t.w;
  } else {
    u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
    d[0] = t.x, d[1] = t.y;
  }
}
template <int DW>
__device__ __forceinline__ void load_dwords(const uint16_t *p, uint32_t (&d)[DW]) {
  if constexpr (DW == 4) {
    uint4 t = *reinterpret_cast<const uint4 *>(p);
    d[0] = t.x, d[1] = t.y, d[2] = t.z, d[3] = t.w;
  } else {
    uint2 t = *reinterpret_cast<const uint2 *>(p);
    d[0] = t.x, d[1] = t.y;
  }
}

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf2;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, a), __builtin_bit_cast(bf2, b), c,
                                         false);
}

// Level L of the reduce-scatter exchanges along one lane bit inside a row of 16.
// The exchange pattern of a level may flip lane bits that LATER levels partition on,
// never earlier ones: mirror (^15) splits on bit 3, half-mirror (^7) on bit 2, then
// ^2 on bit 1 and ^1 on bit 0.  After four levels lane c holds load bitrev4(c).
template <int LEVEL>
__device__ __forceinline__ float rs_exchange(float v) {
  if constexpr (LEVEL == 1) return dpp_move<kDppMirror>(v);
  if constexpr (LEVEL == 2) return dpp_move<kDppHalfMirror>(v);
  if constexpr (LEVEL == 3) return dpp_move<kDppXor2>(v);
  return dpp_move<kDppXor1>(v);
}

template <int LEVEL, int BASE, int G, int NH, int DW>
__device__ __forceinline__ void qk_reduce_scatter(const uint32_t (&k)[NH][16][DW],
                                                  const uint32_t (&q)[G][NH][DW], int c,
                                                  float (&s)[G]) {
  if constexpr (LEVEL == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float acc = 0.f;
#pragma unroll
      for (int hf = 0; hf < NH; ++hf)
#pragma unroll
        for (int j = 0; j < DW; ++j) acc = dot2(k[hf][BASE][j], q[g][hf][j], acc);
      s[g] = acc;
    }
  } else {
    float lo[G], hi[G];
    qk_reduce_scatter<LEVEL - 1, BASE, G, NH, DW>(k, q, c, lo);
    qk_reduce_scatter<LEVEL - 1, BASE + (1 << (LEVEL - 1)), G, NH, DW>(k, q, c, hi);
    const bool upper = (c >> (4 - LEVEL)) & 1;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float keep = upper ? hi[g] : lo[g];
      float send = upper ? lo[g] : hi[g];
      s[g] = keep + rs_exchange<LEVEL>(send);
    }
  }
}

__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_move<kDppXor1>(v));
  v = fmaxf(v, dpp_move<kDppXor2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppMirror>(v));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppMirror>(v);
  return v;
}

__device__ __forceinline__ int bitrev4(int c) {
  return ((c & 1) << 3) | ((c & 2) << 1) | ((c & 4) >> 1) | ((c & 8) >> 3);
}

template <int D, int G>
struct Shape {
  static constexpr int HD = D > 128 ? 128 : D;  // elements covered by one load pass
  static constexpr int NH = D / HD;
  static constexpr int EPL = HD / 16;  // elements per lane per pass
  static constexpr int DW = EPL / 2;
};

// Position of a wavefront in the flat tile list.
struct Cursor {
  int u, h, t;      // user, kv head, absolute tile index (tile t covers positions TILE t ..)
  int len, lo;      // user u attends positions [lo, len)
  int tiles_left;   // tiles of this segment from t on (including t)
};

// Finds the segment that owns unit `x` of the flat tile list (binary search over the
// per-user prefix in LDS).  Everything is wavefront-uniform.
// With `extra` leading units per segment, a unit among them stands for the segment's first tile;
// `x_tile` receives the unit of the tile found.
template <int TILE = kTile>
__device__ __forceinline__ Cursor locate_unit(const DecodeArgs &a, const int *s_pref,
                                              const int *s_len, int64_t x, int extra = 0,
                                              int64_t *x_tile = nullptr) {
  const int users = a.users, hkv = a.hkv;
  int lo_u = 0, hi_u = users - 1;
  while (lo_u < hi_u) {
    int mid = (lo_u + hi_u + 1) >> 1;
    if ((int64_t)__builtin_amdgcn_readfirstlane(s_pref[mid]) * hkv <= x) lo_u = mid;
    else hi_u = mid - 1;
  }
  Cursor cu;
  cu.u = lo_u;
  const int pref_u = __builtin_amdgcn_readfirstlane(s_pref[lo_u]);
  const int nv = __builtin_amdgcn_readfirstlane(s_pref[lo_u + 1]) - pref_u;  // units per segment
  const int nt = nv - extra;
  const int rem = (int)(x - (int64_t)pref_u * hkv);
  cu.h = rem / nv;
  const int rel = max(rem - cu.h * nv - extra, 0);
  if (x_tile) *x_tile = (int64_t)pref_u * hkv + (int64_t)cu.h * nv + extra + rel;
  cu.tiles_left = nt - rel;
  cu.len = __builtin_amdgcn_readfirstlane(s_len[lo_u]);
  cu.lo = window_lo(a, cu.len);
  cu.t = cu.lo / TILE + rel;
  return cu;
}

// Maximum over the four lanes that share lane%16.  v_permlane16_swap exchanges the odd rows
// of its first operand with the even rows of its second, v_permlane32_swap the upper half of
// the first with the lower half of the second; fed with two copies of a value, the two
// results hold the value of either partner.  Written as assembly: through the builtins the
// compiler takes the two results for equal.
__device__ __forceinline__ float max_over_quads(float v) {
  float x = v, y = v;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
  float m = fmaxf(x, y);
  x = m, y = m;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
  return fmaxf(x, y);
}
__device__ __forceinline__ float sum_over_quads(float v) {
  float x = v, y = v;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
  float m = x + y;
  x = m, y = m;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
  return x + y;
}

// One thread per segment (the first blocks of the grid): publishes which partial slots the
// merge kernel has to read for that segment.
__device__ __forceinline__ void publish_segment_row(const DecodeArgs &a, const int *s_pref,
                                                    int64_t total, int n_eff, int extra = 0) {
  const int seg = blockIdx.x * 256 + threadIdx.x;
  if (seg >= a.users * a.hkv) return;
  const int su = seg / a.hkv, sh = seg - su * a.hkv;
  const int snv = s_pref[su + 1] - s_pref[su];  // units per segment: `extra` in front of the tiles
  int first = 0, count = 0;
  if (snv > 0) {
    const int64_t x0 = (int64_t)s_pref[su] * a.hkv + (int64_t)sh * snv + extra;  // first tile
    const int64_t x1 = x0 + (snv - extra) - 1;                                   // last tile
    // wave owning unit x: largest w with floor(w * total / n_eff) <= x; every wave in
    // [w0, w1] owns at least one unit of the segment because n_eff <= total
    const int w0 = (int)(((x0 + 1) * n_eff + total - 1) / total) - 1;
    const int w1 = (int)(((x1 + 1) * n_eff + total - 1) / total) - 1;
    first = w0 + seg;
    count = w1 - w0 + 1;
  }
  a.ws_seg[2 * seg] = first;
  a.ws_seg[2 * seg + 1] = count;
}

// Merges the row streams of a wavefront (4 rows of 16 lanes) for one head and writes the
// partial (un-normalised output, running max, running sum) of (wave, segment).
template <int D, int NH, int EPL>
__device__ __forceinline__ void write_partial(float *slot, int g, int G, int r, int c, float m,
                                              float l, float (&acc)[NH][EPL]) {
  float lr = row16_sum(l);
  float mall = fmaxf(m, __shfl_xor(m, 16));
  mall = fmaxf(mall, __shfl_xor(mall, 32));
  float wgt = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - mall);
  lr *= wgt;
  lr += __shfl_xor(lr, 16);
  lr += __shfl_xor(lr, 32);
#pragma unroll
  for (int hf = 0; hf < NH; ++hf)
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float v = acc[hf][e] * wgt;
      v += __shfl_xor(v, 16);
      v += __shfl_xor(v, 32);
      acc[hf][e] = v;
    }
  if (r == 0) {
    constexpr int HD = D > 128 ? 128 : D;
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) {
      float *dst = slot + g * D + hf * HD + c * EPL;
#pragma unroll
      for (int e4 = 0; e4 < EPL / 4; ++e4)
        *reinterpret_cast<float4 *>(dst + 4 * e4) = make_float4(
            acc[hf][4 * e4], acc[hf][4 * e4 + 1], acc[hf][4 * e4 + 2], acc[hf][4 * e4 + 3]);
    }
    if (c == 0) {
      slot[G * D + g] = mall;
      slot[G * D + G + g] = lr;
    }
  }
}

// Merges the partials of one (user, kv_head) segment and writes bfloat16 output.
// Partials are read eight at a time so that their loads overlap (with four wavefronts per CU
// and at least one segment per CU, a segment has about five): the kernel is a chain of
// dependent round trips, and this keeps it at two.  G and D are run-time values: the
// matrix-core kernels serve any group width up to 32.  D is a power of two on the attention
// paths (64, 128, 256: split by shift and mask); the latent path also has 384 (divided).
// Grid: x = segment, y = piece of kCombinePiece of the segment's G * D output elements: one
// element per thread, so a thread's loads are one batch in flight (two pieces for the Llama-3-8B
// decode shape, whose step is 0.7 us shorter than with one piece of 512; a latent segment of
// 16 heads x 512 values is 32 pieces, and as one workgroup per segment its merge took as long as
// the attention itself).
constexpr int kCombinePiece = 256;
inline int combine_pieces(int g, int d) { return (g * d + kCombinePiece - 1) / kCombinePiece; }

__global__ inline __launch_bounds__(256) void decode_combine_kernel(DecodeArgs a, int G, int D) {
  const int seg = blockIdx.x;
  const int i_begin = blockIdx.y * kCombinePiece + threadIdx.x;
  const int i_end = min(G * D, (int)(blockIdx.y + 1) * kCombinePiece);
  const int u = seg / a.hkv, h = seg % a.hkv;
  const bool pow2 = (D & (D - 1)) == 0;
  const int dshift = __builtin_ctz(D);
  auto head_of = [&](int i) { return pow2 ? i >> dshift : i / D; };
  auto elem_of = [&](int i) { return pow2 ? i & (D - 1) : i % D; };
  const int first = a.ws_seg[2 * seg], nw = a.ws_seg[2 * seg + 1];
  uint16_t *out = a.out + u * a.out_us;
  if (nw == 0) {  // padded row: no attended position -> NaN like softmax over nothing
    for (int i = i_begin; i < i_end; i += 256)
      out[(int64_t)(h * G + head_of(i)) * a.out_hs + elem_of(i)] = 0x7fc0;
    return;
  }
  constexpr int kBatch = 8;
  const float *base = a.ws_slots + (int64_t)first * a.slot_floats;
  for (int i = i_begin; i < i_end; i += 256) {
    const int g = head_of(i);
    float mall = -INFINITY, num = 0.f, den = 0.f;
    for (int w = 0; w < nw; w += kBatch) {
      float mv[kBatch], lv[kBatch], av[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const float *sl = base + (int64_t)min(w + j, nw - 1) * a.slot_floats;
        mv[j] = (w + j < nw) ? sl[G * D + g] : -INFINITY;
        lv[j] = sl[G * D + G + g];
        av[j] = sl[i];
      }
      float mnew = mall;
#pragma unroll
      for (int j = 0; j < kBatch; ++j) mnew = fmaxf(mnew, mv[j]);
      float resc = __builtin_amdgcn_exp2f(mall - mnew);
      num *= resc;
      den *= resc;
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        float wgt = __builtin_amdgcn_exp2f(mv[j] - mnew);  // 0 for the padding entries
        num = fmaf(wgt, av[j], num);
        den = fmaf(wgt, lv[j], den);
      }
      mall = mnew;
    }
    if (a.sink) {  // the sink logit (natural-log units, not scaled) only enlarges the normaliser
      const float sk = a.sink[h * G + g] * 1.4426950408889634f;
      const float mnew = fmaxf(mall, sk);
      const float resc = __builtin_amdgcn_exp2f(mall - mnew);
      num *= resc;
      den = den * resc + __builtin_amdgcn_exp2f(sk - mnew);
    }
    out[(int64_t)(h * G + g) * a.out_hs + elem_of(i)] = (uint16_t)f32_to_bf16_bits(num / den);
  }
}

// The same merge over partials whose values are bfloat16 (DecodeArgs::partial_bf16).  They lie in
// blocks of 16 heads x 16 elements (element e of head g at
// ((g / 16 * (D / 16) + e / 16) * 16 + g % 16) * 16 + e % 16, the last block of heads padded), the order
// in which the latent kernels hold them: the 64 lanes of a store then write 512 consecutive bytes.  A
// thread owns W consecutive 32-bit words of every partial, in that order, and stores its 2 W
// neighbouring output elements at once: W = 4 (16 bytes per load and store) where output rows start
// on 16-byte boundaries, W = 1 where only on 4-byte ones (the caller checks).
// Grid: x = segment, y = piece of kCombinePiece threads.
template <int W>
__global__ inline __launch_bounds__(256) void decode_combine_bf16_kernel(DecodeArgs a, int G, int D) {
  static_assert(W == 1 || W == 4, "a thread's words stay inside one head's eight");
  typedef uint32_t words_t __attribute__((ext_vector_type(W)));
  const int seg = blockIdx.x;
  const int pairs = (G + 15) / 16 * 16 * D / 2;  // words of values in a partial
  const int p = W * (blockIdx.y * kCombinePiece + threadIdx.x);
  if (p >= pairs) return;
  const int u = seg / a.hkv, h = seg % a.hkv;
  const int blk = p >> 7, in_blk = p & 127;  // a block: 16 heads x 8 words
  const int g = 16 * (blk / (D / 16)) + (in_blk >> 3), e = 16 * (blk % (D / 16)) + 2 * (in_blk & 7);
  if (g >= G) return;
  const int first = a.ws_seg[2 * seg], nw = a.ws_seg[2 * seg + 1];
  words_t *out = reinterpret_cast<words_t *>(a.out + u * a.out_us + (int64_t)(h * G + g) * a.out_hs + e);
  if (nw == 0) {  // padded row: no attended position -> NaN like softmax over nothing
    words_t nan;
#pragma unroll
    for (int k = 0; k < W; ++k) nan[k] = 0x7fc07fc0u;
    *out = nan;
    return;
  }
  const float *base = a.ws_slots + (int64_t)first * a.slot_floats;
  float mall = -INFINITY, den = 0.f, num[2 * W];
#pragma unroll
  for (int k = 0; k < 2 * W; ++k) num[k] = 0.f;
  // partials are read in batches so that their loads overlap; a segment that few ranges share (the
  // 128-head latent form: two or three) takes batches of its size instead of eight mostly repeated loads
  auto merge = [&](auto batch_tag) {
    constexpr int kBatch = decltype(batch_tag)::value;
    for (int w = 0; w < nw; w += kBatch) {
      float mv[kBatch], lv[kBatch];
      words_t av[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const float *sl = base + (int64_t)min(w + j, nw - 1) * a.slot_floats;
        mv[j] = (w + j < nw) ? sl[pairs + g] : -INFINITY;
        lv[j] = sl[pairs + G + g];
        av[j] = *reinterpret_cast<const words_t *>(reinterpret_cast<const uint32_t *>(sl) + p);
      }
      float mnew = mall;
#pragma unroll
      for (int j = 0; j < kBatch; ++j) mnew = fmaxf(mnew, mv[j]);
      const float resc = __builtin_amdgcn_exp2f(mall - mnew);
      den *= resc;
#pragma unroll
      for (int k = 0; k < 2 * W; ++k) num[k] *= resc;
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const float wgt = __builtin_amdgcn_exp2f(mv[j] - mnew);  // 0 for the padding entries
#pragma unroll
        for (int k = 0; k < W; ++k) {
          num[2 * k] = fmaf(wgt, bf16_lo(av[j][k]), num[2 * k]);
          num[2 * k + 1] = fmaf(wgt, bf16_hi(av[j][k]), num[2 * k + 1]);
        }
        den = fmaf(wgt, lv[j], den);
      }
      mall = mnew;
    }
  };
  if (nw <= 2) merge(std::integral_constant<int, 2>{});
  else if (nw <= 4) merge(std::integral_constant<int, 4>{});
  else merge(std::integral_constant<int, 8>{});
  if (a.sink) {
    const float sk = a.sink[h * G + g] * 1.4426950408889634f;
    const float mnew = fmaxf(mall, sk);
    const float resc = __builtin_amdgcn_exp2f(mall - mnew);
#pragma unroll
    for (int k = 0; k < 2 * W; ++k) num[k] *= resc;
    den = den * resc + __builtin_amdgcn_exp2f(sk - mnew);
  }
  const float inv = 1.0f / den;
  words_t res;
#pragma unroll
  for (int k = 0; k < W; ++k) res[k] = f32_to_bf16_bits(num[2 * k] * inv) | (f32_to_bf16_bits(num[2 * k + 1] * inv) << 16);
  *out = res;
}

inline int slot_floats_for(int g, int d) { return ((g * d + 2 * g + 3) / 4) * 4; }
// the same with the values as bfloat16, in blocks of 16 heads (decode_combine_bf16_kernel)
inline int slot_floats_bf16_for(int g, int d) { return (((g + 15) / 16 * 16 * d / 2 + 2 * g + 3) / 4) * 4; }
inline size_t header_bytes(int users, int hkv) { return (((size_t)users * hkv * 8 + 255) / 256) * 256; }


int waves_for_device(double default_per_cu);
// Units in front of every segment of the flat list (TTPA_DECODE_SEG_UNITS overrides, 0 ... 64).
int segment_units(int default_units);
constexpr int kWavesPerBlockHost = kWavesPerBlock;

// Launches the block-float-8 VALU main kernel (decode_bfp8.hip); false = shape not built.
bool launch_bfp8_main(const DecodeArgs &a, int head_size, int g, hipStream_t st);
// Matrix-core main kernel (decode_mfma.hip) for wide head groups and block-float-8.
bool mfma_decode_supported(const DecodeArgs &a, int head_size, int g);
bool launch_mfma_main(const DecodeArgs &a, int head_size, hipStream_t st);
// 16x16x32 matrix-core main kernel (decode_mfma16.hip): up to 16 query heads per KV head, head
// size 128 (either cache format) or 256 (bfloat16 cache).
bool mfma16_decode_supported(const DecodeArgs &a, int head_size, int g);
bool launch_mfma16_main(const DecodeArgs &a, int head_size, hipStream_t st);

}  // namespace decode
}  // namespace ttpa
