// Paged decode attention: split-K over a flattened list of 64-token tiles.
//
// Work decomposition
//   A tile is 64 consecutive cache positions of one (user, kv_head) segment.  All
//   tiles of all segments form one flat list ordered (user, kv_head, tile); the
//   list is cut into n_waves equal ranges and every wavefront streams exactly one
//   range, so ragged context lengths cost no imbalance.  A wavefront emits one
//   partial result (un-normalised output, running max, running sum) per segment
//   its range touches; a second kernel merges the partials of each segment.
//
// Inside a wavefront (lane = 16 * r + c)
//   A K or V tile is read with 16 wide loads; load i gives lane (r, c) the
//   head_size/16 elements c of token 4 i + r, so every load instruction covers 4
//   whole token rows contiguously.  q.k is a per-lane partial dot product
//   (v_dot2_f32_bf16) that must be summed over the 16 lanes c of a row; the 16
//   loads of a tile are summed with a DPP reduce-scatter, after which lane (r, c)
//   holds the score of ONE token for each of the G query heads of the group.
//   The 16 lanes with equal r therefore own every fourth token: each such row of
//   lanes runs its own online softmax and its own accumulators (4 streams per
//   wavefront, merged once per segment).  Probabilities go through a wave-private
//   LDS buffer so that lane (r, c) can read the weight of token 4 i + r when it
//   multiplies its V elements.
//   The G query heads of a group share every K/V load: each element is read once
//   per KV head.
#include <algorithm>
#include "decode_common.h"

#include <cstdlib>
#include <cstring>

namespace ttpa {
namespace decode {

// BIG = block_size is a multiple of 64: a tile lies inside one physical block.
// The grid is one workgroup per CU, so a second resident workgroup is asked of the register
// allocator only where it costs nothing: from five query heads per KV head at head size 128, and
// at head size 256, 256 registers spill (4 ... 864 of them) where 512 hold everything.
template <int D, int G, bool BIG>
__global__ __launch_bounds__(256, (D <= 128 && G <= 4) ? 2 : 1) void paged_decode_kernel(
    DecodeArgs a, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  // page_table / cur_pos are separate restrict parameters so that their wavefront-uniform
  // reads become scalar loads: a vector load + readfirstlane would have to wait for every
  // K/V tile load in flight (one shared counter) and stall the stream between tiles.
  using S = Shape<D, G>;
  constexpr int NH = S::NH, EPL = S::EPL, DW = S::DW;
  constexpr int NOFF = BIG ? 1 : 16;  // distinct row-group bases per tile

  __shared__ int s_pref[kMaxUsers + 1];
  __shared__ int s_len[kMaxUsers];
  __shared__ int s_wsum[kWavesPerBlock];
  // probabilities of one tile as bfloat16: [wave][lane row r][head g][16 loads]
  __shared__ __attribute__((aligned(16))) uint16_t s_p[kWavesPerBlock][4 * G * 16];

  const int seg_units = a.seg_units;
  build_prefix(a, cur_pos, s_pref, s_len, s_wsum, seg_units);
  const int lane = threadIdx.x & 63;
  const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane >> 4, c = lane & 15;
  const int wave = blockIdx.x * kWavesPerBlock + wib;
  // The flat list in units: per segment `seg_units` units that stand for the cost of opening it,
  // then its tiles.  A range of more than seg_units units holds at least one tile.
  const int total_units = __builtin_amdgcn_readfirstlane(s_pref[a.users]);
  const int64_t total = (int64_t)total_units * a.hkv;
  const int64_t max_ranges = total / (seg_units + 1);
  const int n_eff = (int)(max_ranges < a.n_waves ? max_ranges : a.n_waves);  // wavefronts that get work
  if (total == 0 || wave >= n_eff) {  // idle wavefronts still do their share of the table
    publish_segment_row(a, s_pref, total, n_eff, seg_units);
    return;
  }
  const int64_t x_lo = (int64_t)wave * total / n_eff;
  int64_t x = x_lo;  // set below to the unit of the first tile at or behind x_lo
  const int64_t x_hi = (int64_t)(wave + 1) * total / n_eff;
  lds_u16 *plds = s_p[wib];
  const int my_step = bitrev4(c);
  const uint16_t *kb = reinterpret_cast<const uint16_t *>(a.k);
  const uint16_t *vb = reinterpret_cast<const uint16_t *>(a.v);
  const uint32_t lane_bytes = (uint32_t)(r * D + c * EPL) * 2u;

  // ---- helpers (all uniform across the wavefront) ---------------------------------
  auto locate = [&](int64_t xx) { return locate_unit(a, s_pref, s_len, xx, seg_units); };
  // element offset (relative to the cache base) of the first row of each 4-row load
  auto tile_offsets = [&](const Cursor &cu, int64_t (&off)[NOFF]) {
    const int32_t *pt_row = page_table + (int64_t)cu.u * a.pt_rs;
    const int tok0 = cu.t * kTile;
    if constexpr (BIG) {
      int phys = __builtin_amdgcn_readfirstlane(pt_row[tok0 / a.bs]);
      if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
      off[0] = (((int64_t)phys * a.hkv + cu.h) * a.bs + (tok0 % a.bs)) * D;
    } else {
      // block_size is a multiple of 4, so the 4 rows of a load never cross a block: block and
      // row advance without a division, and the table is read only where the block changes
      int col = tok0 / a.bs, row = tok0 - col * a.bs;
      int64_t base = 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (i == 0 || row == 0) {
          int phys = (col < a.w) ? __builtin_amdgcn_readfirstlane(pt_row[col]) : 0;
          if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
          base = ((int64_t)phys * a.hkv + cu.h) * a.bs * D;
        }
        off[i] = base + (int64_t)row * D;
        row += 4;
        if (row >= a.bs) row = 0, ++col;
      }
    }
  };
  // Loads are unconditional: every row of a tile is readable memory (rows past the
  // attended length sit in the same physical block, columns past the table map to block 0).
  auto load_tile = [&](const uint16_t *base, const int64_t (&off)[NOFF],
                       uint32_t (&dst)[NH][16][DW]) {
#pragma unroll
    for (int hf = 0; hf < NH; ++hf)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint16_t *row = BIG ? base + off[0] + i * 4 * D : base + off[BIG ? 0 : i];
        load_stream<DW>(row + hf * S::HD, lane_bytes, dst[hf][i]);
      }
  };
  // Rows that are not attended get weight 0; their V bits are cleared so that stale
  // Inf / NaN in unwritten cache rows cannot turn 0 * x into NaN.
  auto clear_unattended = [&](int nvalid, uint32_t (&dst)[NH][16][DW]) {
#pragma unroll
    for (int hf = 0; hf < NH; ++hf)
#pragma unroll
      for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int j = 0; j < DW; ++j) dst[hf][i][j] = (4 * i + r < nvalid) ? dst[hf][i][j] : 0u;
  };
  auto load_q = [&](const Cursor &cu, uint32_t (&q)[G][NH][DW]) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int hf = 0; hf < NH; ++hf)
        load_dwords<DW>(a.q + cu.u * a.q_us + (int64_t)(cu.h * G + g) * a.q_hs + hf * S::HD + c * EPL,
                        q[g][hf]);
  };

  Cursor cur = locate_unit(a, s_pref, s_len, x_lo, seg_units, &x);
  int64_t off[NOFF];
  uint32_t kreg[NH][16][DW], q[G][NH][DW];
  tile_offsets(cur, off);
  load_tile(kb, off, kreg);
  load_q(cur, q);

  publish_segment_row(a, s_pref, total, n_eff, seg_units);  // hidden behind the first tile's latency

  float m[G], l[G], acc[G][NH][EPL];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int hf = 0; hf < NH; ++hf)
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][hf][e] = 0.f;
  }

  // One tile.  HAS_NEXT is a compile-time property of the call site: the steady-state
  // loop always prefetches the next K tile unconditionally (a conditional prefetch makes
  // the wait-count bookkeeping pessimistic and PV would wait for the prefetch), the last
  // tile of the wavefront's range is peeled off below.
  auto process_tile = [&](auto has_next_tag) {
    constexpr bool has_next = decltype(has_next_tag)::value;
    const int nvalid = cur.len - cur.t * kTile;  // >= 1
    // V of this tile goes in flight behind K (which was requested one iteration ago)
    uint32_t vreg[NH][16][DW];
    if constexpr (NH == 1) load_tile(vb, off, vreg);
    // scheduling fences pin the order "V(t) loads, QK(t), K(t+1) loads, softmax, PV(t)":
    // left alone the scheduler sinks the V loads below the K(t+1) loads, and PV(t) then
    // has to wait for K(t+1) (loads complete in issue order)
    __builtin_amdgcn_sched_barrier(0);

    // ---- scores: lane (r, c) ends with token 4 * bitrev4(c) + r of the tile -----------
    float s[G];
    qk_reduce_scatter<4, 0, G, NH, DW>(kreg, q, c, s);

    __builtin_amdgcn_sched_barrier(0);
    // ---- advance the cursor; K of the next tile goes in flight now --------------------
    const bool same_seg = has_next && cur.tiles_left > 1;
    Cursor nxt = cur;
    int64_t noff[NOFF];
#pragma unroll
    for (int i = 0; i < NOFF; ++i) noff[i] = off[i];
    if constexpr (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate(x + 1);
      }
      tile_offsets(nxt, noff);
      load_tile(kb, noff, kreg);
    }
    if constexpr (NH == 2) load_tile(vb, off, vreg);  // head_size 256: V fetched late
    __builtin_amdgcn_sched_barrier(0);

    // ---- online softmax, one stream per lane row ---------------------------------------
    // positions below the sliding window's lower edge can only occur in a segment's first tile
    const int nbelow = cur.lo - cur.t * kTile;
    const bool valid = 4 * my_step + r < nvalid && 4 * my_step + r >= nbelow;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float sv = valid ? s[g] * a.scale_log2e : -INFINITY;
      if (a.mask != nullptr && valid)
        sv += bf16_lo(a.mask[cur.u * a.mask_us + (int64_t)(cur.h * G + g) * a.mask_hs + cur.t * kTile + 4 * my_step + r]) *
              1.4426950408889634f;
      float mx = fmaxf(m[g], row16_max(sv));
      float msafe = (mx == -INFINITY) ? 0.f : mx;
      float alpha = __builtin_amdgcn_exp2f(m[g] - msafe);
      float p = __builtin_amdgcn_exp2f(sv - msafe);
      // the weight that multiplies V is rounded to bfloat16; the normaliser sums the
      // same rounded values
      uint32_t pb = f32_to_bf16_bits(p);
      l[g] = l[g] * alpha + __builtin_bit_cast(float, pb << 16);
      m[g] = mx;
      plds[(r * G + g) * 16 + my_step] = (uint16_t)pb;
#pragma unroll
      for (int hf = 0; hf < NH; ++hf)
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][hf][e] *= alpha;
    }

    // ---- output accumulation: two tokens per dot2 ----------------------------------------
    if (nvalid < kTile) clear_unattended(nvalid, vreg);
    const lds_u32 *pw = reinterpret_cast<const lds_u32 *>(plds) + r * G * 8;
#pragma unroll
    for (int k2 = 0; k2 < 8; ++k2) {
      uint32_t pk[G];  // weights of loads (2 k2, 2 k2 + 1) as a bf16 pair, per head
#pragma unroll
      for (int g = 0; g < G; ++g) pk[g] = pw[g * 8 + k2];
#pragma unroll
      for (int hf = 0; hf < NH; ++hf)
#pragma unroll
        for (int j = 0; j < DW; ++j) {
          const uint32_t va = vreg[hf][2 * k2][j], vb2 = vreg[hf][2 * k2 + 1][j];
          const uint32_t even = __builtin_amdgcn_perm(vb2, va, 0x05040100u);  // element 2j
          const uint32_t odd = __builtin_amdgcn_perm(vb2, va, 0x07060302u);   // element 2j+1
#pragma unroll
          for (int g = 0; g < G; ++g) {
            acc[g][hf][2 * j] = dot2(even, pk[g], acc[g][hf][2 * j]);
            acc[g][hf][2 * j + 1] = dot2(odd, pk[g], acc[g][hf][2 * j + 1]);
          }
        }
    }

    // ---- close the segment if it ends here ----------------------------------------------
    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wave + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float lr = row16_sum(l[g]);
        float mr = m[g];
        float mall = fmaxf(mr, __shfl_xor(mr, 16));
        mall = fmaxf(mall, __shfl_xor(mall, 32));
        float wgt = (mr == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mr - mall);
        lr *= wgt;
        lr += __shfl_xor(lr, 16);
        lr += __shfl_xor(lr, 32);
#pragma unroll
        for (int hf = 0; hf < NH; ++hf)
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            float v = acc[g][hf][e] * wgt;
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            acc[g][hf][e] = v;
          }
        if (r == 0) {
#pragma unroll
          for (int hf = 0; hf < NH; ++hf) {
            float *dst = slot + g * D + hf * S::HD + c * EPL;
#pragma unroll
            for (int e4 = 0; e4 < EPL / 4; ++e4)
              *reinterpret_cast<float4 *>(dst + 4 * e4) =
                  make_float4(acc[g][hf][4 * e4], acc[g][hf][4 * e4 + 1], acc[g][hf][4 * e4 + 2],
                              acc[g][hf][4 * e4 + 3]);
          }
          if (c == 0) {
            slot[G * D + g] = mall;
            slot[G * D + G + g] = lr;
          }
        }
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int hf = 0; hf < NH; ++hf)
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[g][hf][e] = 0.f;
      }
      if constexpr (has_next) load_q(nxt, q);
    }
    cur = nxt;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) off[i] = noff[i];
    x += same_seg ? 1 : 1 + seg_units;
  };
  // the unit of the tile behind the current one: the next, or behind the next segment's leading units
  auto next_tile_unit = [&]() { return x + (cur.tiles_left > 1 ? 1 : 1 + seg_units); };
  while (next_tile_unit() < x_hi) process_tile(std::true_type{});
  process_tile(std::false_type{});
}

int segment_units(int default_units) {
  const char *e = getenv("TTPA_DECODE_SEG_UNITS");
  const int v = e ? atoi(e) : default_units;
  return v < 0 ? 0 : (v > 64 ? 64 : v);
}

int waves_for_device(double default_per_cu) {
  // TTPA_DECODE_WAVES_PER_CU (read on every call, fractions allowed) overrides the grid size: tests
  // use a small grid to give every wavefront several tiles and segments
  const char *e = getenv("TTPA_DECODE_WAVES_PER_CU");
  const double override_waves = e ? atof(e) : 0.0;
  const double per_cu = override_waves > 0 ? override_waves : default_per_cu;
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  const int waves = (int)(cus * per_cu + 0.5);
  // (whole workgroups, at least one)
  return std::max(kWavesPerBlock, (waves + kWavesPerBlock - 1) / kWavesPerBlock * kWavesPerBlock);
}

template <int D, int G>
bool launch(const DecodeArgs &a, hipStream_t st) {
  if (a.kv_format == TTPA_KV_BFP8) {
    return launch_bfp8_main(a, D, G, st);
  } else {
    // With one workgroup per CU in the grid, a 64 KiB dynamic LDS request (unused) makes two
    // workgroups too large to share a CU, so the dispatcher has to spread them over all CUs.
    const int blocks = a.n_waves / kWavesPerBlock;
    const size_t pad = blocks <= device_cus() ? 65536 : 0;
    if (a.bs % kTile == 0)
      paged_decode_kernel<D, G, true><<<dim3(blocks), dim3(256), pad, st>>>(a, a.pt, a.cur);
    else
      paged_decode_kernel<D, G, false><<<dim3(blocks), dim3(256), pad, st>>>(a, a.pt, a.cur);
  }
  return true;
}

template <int D>
int launch_g(const DecodeArgs &a, int g, hipStream_t st) {
  bool ok = true;
  switch (g) {
    case 1: ok = launch<D, 1>(a, st); break;
    case 2: ok = launch<D, 2>(a, st); break;
    case 3: ok = launch<D, 3>(a, st); break;
    case 4: ok = launch<D, 4>(a, st); break;
    case 5: ok = launch<D, 5>(a, st); break;
    case 6: ok = launch<D, 6>(a, st); break;
    case 7: ok = launch<D, 7>(a, st); break;
    case 8: ok = launch<D, 8>(a, st); break;
    default:
      return fail(TTPA_ERR_UNSUPPORTED,
                  "query heads per KV head = %d: more than 8 (up to 16; up to 32 with head_size 64 / 128 and "
                  "at most 1024 users) need a block_size that is a multiple of 1024 / (bytes of a cache row)",
                  g);
  }
  if (!ok) return fail(TTPA_ERR_UNSUPPORTED, "decode: the dot-product kernel is not built for this head size and cache format");
  return TTPA_OK;
}

}  // namespace decode
}  // namespace ttpa

using namespace ttpa;
using namespace ttpa::decode;

// wavefronts per CU of the largest grid a decode launch uses (the VALU kernel on a block-float-8 cache)
static constexpr double kLargestGrid = 8.0;

extern "C" size_t ttpa_paged_decode_workspace_bytes(int32_t users, int32_t q_heads,
                                                    int32_t kv_heads, int32_t head_size) {
  if (users <= 0 || q_heads <= 0 || kv_heads <= 0 || head_size <= 0 || q_heads % kv_heads) return 0;
  int g = q_heads / kv_heads;
  size_t slots = (size_t)waves_for_device(kLargestGrid) + (size_t)users * kv_heads;  // the larger grid
  return header_bytes(users, kv_heads) + slots * (size_t)slot_floats_for(g, head_size) * sizeof(float);
}

static int decode_impl(void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
                       int64_t q_user_stride, int64_t q_head_stride, const void *k_cache,
                       const void *v_cache, const int32_t *page_table,
                       int64_t page_table_row_stride, const void *cur_pos, int cur_pos_is_i64,
                       int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
                       int32_t block_size, int32_t table_width, int32_t num_blocks, float scale,
                       int32_t kv_format, int32_t sliding_window, const float *attention_sink,
                       void *workspace, size_t workspace_bytes, void *stream,
                       const void *k_new = nullptr, const void *v_new = nullptr,
                       int64_t new_user_stride = 0, int64_t new_head_stride = 0,
                       const void *mask = nullptr, int64_t mask_user_stride = 0, int64_t mask_head_stride = 0) {
  TTPA_REQUIRE(sliding_window >= 0, "decode: sliding_window %d is negative", sliding_window);
  TTPA_REQUIRE(out && q && k_cache && v_cache && page_table && cur_pos, "null pointer argument");
  TTPA_REQUIRE(users > 0 && q_heads > 0 && kv_heads > 0 && head_size > 0 && block_size > 0 &&
                   table_width > 0 && num_blocks > 0,
               "non-positive dimension");
  TTPA_REQUIRE(q_heads % kv_heads == 0, "q_heads %d not divisible by kv_heads %d", q_heads,
               kv_heads);
  if (kv_format != TTPA_KV_BF16 && kv_format != TTPA_KV_BFP8)
    return fail(TTPA_ERR_INVALID_ARGUMENT, "decode: unknown kv_format %d", kv_format);
  if (kv_format == TTPA_KV_BFP8 && block_size % 16)
    return fail(TTPA_ERR_UNSUPPORTED, "decode: a block-float-8 cache needs block_size %% 16 == 0");
  if (kv_format == TTPA_KV_BFP8 && head_size == 256 && (q_heads / kv_heads > 16))
    return fail(TTPA_ERR_UNSUPPORTED,
                "decode: block-float-8 with head_size 256 is built for up to 16 query heads per KV head");
  if (users > kMaxUsers)
    return fail(TTPA_ERR_UNSUPPORTED, "decode: %d users exceeds the limit of %d", users, kMaxUsers);
  if (head_size != 64 && head_size != 128 && head_size != 256)
    return fail(TTPA_ERR_UNSUPPORTED, "decode: head_size %d; supported 64, 128, 256", head_size);
  if (block_size % 4 != 0)
    return fail(TTPA_ERR_UNSUPPORTED, "decode: block_size %d must be a multiple of 4", block_size);
  TTPA_REQUIRE(aligned16(q) && aligned16(k_cache) && aligned16(v_cache) && aligned16(out),
               "decode: q / caches / out must be 16-byte aligned");
  TTPA_REQUIRE(q_user_stride % 8 == 0 && q_head_stride % 8 == 0,
               "decode: q strides must be multiples of 8 elements");
  const size_t need = ttpa_paged_decode_workspace_bytes(users, q_heads, kv_heads, head_size);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return fail(TTPA_ERR_WORKSPACE, "decode: workspace of %zu bytes (256-byte aligned) required, got %zu",
                need, workspace_bytes);

  const int g = q_heads / kv_heads;
  DecodeArgs a;
  a.out = static_cast<uint16_t *>(out);
  a.out_us = out_user_stride, a.out_hs = out_head_stride;
  a.q = static_cast<const uint16_t *>(q);
  a.q_us = q_user_stride, a.q_hs = q_head_stride;
  a.k = static_cast<const uint8_t *>(k_cache);
  a.v = static_cast<const uint8_t *>(v_cache);
  a.pt = page_table, a.pt_rs = page_table_row_stride;
  a.cur = cur_pos, a.cur_i64 = cur_pos_is_i64;
  a.users = users, a.hq = q_heads, a.hkv = kv_heads, a.bs = block_size, a.w = table_width;
  a.nb = num_blocks;
  a.scale_log2e = scale * 1.4426950408889634f;
  a.ws_seg = static_cast<int *>(workspace);
  a.ws_slots = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + header_bytes(users, kv_heads));
  a.slot_floats = slot_floats_for(g, head_size);
  a.kv_format = kv_format;
  a.window = sliding_window;
  a.sink = attention_sink;
  a.k_new = a.v_new = nullptr;
  a.new_us = a.new_hs = 0;
  a.mask = static_cast<const uint16_t *>(mask);
  a.mask_us = mask_user_stride, a.mask_hs = mask_head_stride;

  hipStream_t st = static_cast<hipStream_t>(stream);
  // Kernel choice.  The VALU kernel spends per-head work on every tile; the matrix-core kernels
  // do not (their cost per tile does not depend on the group width).  Measured on bfloat16
  // caches with head size 128: at 1 and 2 query heads per KV head the VALU kernel is 2 - 19 %
  // faster (the larger figure on launches of a few tiles), at 4 the 16x16x32 kernel is 2 - 8 %
  // faster, at 8 the VALU kernel is 2.5 times slower.  With head size 256 the VALU kernel streams
  // at 3.8 TB/s with one head per group and at 1.2 TB/s with eight, the 16x16x32 kernel at 5.3 -
  // 5.6 TB/s with any.  Head size 64 behaves like 128 (block size 32, 4 heads: 47.6 us on the
  // 16x16x32 kernel, 50.0 us on the VALU kernel; block size 64: 47.5 and 46.7).  So: 16x16x32
  // kernel for head sizes 64 / 128 and 4 ... 16 heads per group and for head size 256 (up to 16
  // heads), 32x32x16 kernel for wider groups (up to 32 heads), VALU kernel for the rest.  The block-float-8 cache goes to a matrix-core kernel
  // whenever one applies: there the byte expansion costs one VALU operation per element and the
  // products none, while the VALU kernel pays for both.
  // TTPA_DECODE_KERNEL=valu|mfma|mfma16 overrides the choice.
  // read on every call (a getenv is negligible next to a launch) so that a process can
  // exercise every kernel
  const char *forced_name = getenv("TTPA_DECODE_KERNEL");
  const int forced = !forced_name ? 0
                     : !strcmp(forced_name, "valu") ? 1
                     : !strcmp(forced_name, "mfma") ? 2
                     : !strcmp(forced_name, "mfma16") ? 3 : 0;
  const bool mfma_ok = mfma_decode_supported(a, head_size, g);
  const bool mfma16_ok = mfma16_decode_supported(a, head_size, g);
  // As a step (update + attention) the 16x16x32 kernel with the update inside already wins at 2
  // and 3 heads per group (1 - 6 % and 2 - 11 % per step against update launch + VALU kernel; at
  // 1 head the two are within 2.5 % of each other either way).
  const int g_min16 = k_new ? 2 : 4;
  bool use_mfma16 = mfma16_ok && (g >= g_min16 || kv_format == TTPA_KV_BFP8 || head_size == 256);
  bool use_mfma = !use_mfma16 && mfma_ok && (g >= 5 || kv_format == TTPA_KV_BFP8);
  // a forced kernel that is not built for the shape leaves the default choice in place
  if (forced == 1 && g <= 8 && !(kv_format == TTPA_KV_BFP8 && head_size == 256)) use_mfma = use_mfma16 = false;
  if (forced == 2 && mfma_ok) use_mfma = true, use_mfma16 = false;
  if (forced == 3 && mfma16_ok) use_mfma16 = true, use_mfma = false;
  if (mask) {
    // A mask is applied by the dot-product kernel (bfloat16 caches, up to 8 heads per group) and by
    // the matrix-core kernels (either format; 16x16x32 up to 16 heads, 32x32x16 up to 32); a forced
    // choice holds where it is built.
    const bool valu_ok = g <= 8 && kv_format == TTPA_KV_BF16;
    if (!valu_ok && !mfma16_ok && !mfma_ok)
      return fail(TTPA_ERR_UNSUPPORTED,
                  "masked decode: %d query heads per KV head with this cache format, head size and block size is not "
                  "built (bfloat16 up to 8, or up to 32 on the matrix-core kernels' shapes)", g);
    if (forced == 2 && mfma_ok) use_mfma = true, use_mfma16 = false;
    else if (forced == 3 && mfma16_ok) use_mfma = false, use_mfma16 = true;
    else if (forced == 1 && valu_ok) use_mfma = use_mfma16 = false;
    else {
      use_mfma16 = mfma16_ok && (g >= 4 || !valu_ok);
      use_mfma = !use_mfma16 && !valu_ok;
    }
  }
  // The matrix-core kernels get at most one workgroup per CU whatever the cache format: the 32x32
  // kernel fills the CU's LDS with one, and the 16x16 kernel streams as fast with one as with the
  // two that would fit, while twice the partials cost the merge kernel more.  On a bfloat16 cache
  // the 16x16 kernel is fastest with three quarters of the CUs (measured in one process, grids of
  // 2.5 ... 4 wavefronts per CU: 56.0-56.9 us per step at 2.75 ... 3.75 against 57.3-57.7 at 4 on
  // the 32-user workload, 531 against 544 us on the 128-user one: the streams of 192 workgroups
  // already hold the memory system's latency in bytes, and every further wavefront is one more
  // partial and one more share in the contention); on a block-float-8 cache it wants all of them
  // (50.4 against 43.9 us).
  a.n_waves = waves_for_device(use_mfma16 && kv_format == TTPA_KV_BF16 ? 3.0
                               : (use_mfma || use_mfma16)               ? 4.0
                               : kv_format == TTPA_KV_BFP8              ? kLargestGrid
                                                                        : 4.0);
  // Ranges are equal in units of one tile, with units that carry no work in front of every
  // segment: a change of segment inside a range (partial, search, next Q rows) costs a wavefront
  // about what a tile costs, and the slowest wavefront ends the launch.  Measured in one process,
  // 0 / 1 / 2 units with the 16x16 kernel: 56.4 / 54.9 / 55.1 us per step on the 32-user workload,
  // 44.4 / 42.3 / 42.9 on its block-float-8 form, 534 / 520 / 519 on the 128-user one.  The 32x32
  // kernel wants two (32 users of 64 / 2 heads, contexts 512 ... 4096: 33.3 / 33.2 / 31.6 / 31.5 /
  // 32.0 us at 0 / 1 / 2 / 3 / 4), the VALU kernels none (8 / 8 heads: 52.1 / 53.3 / 53.8 us at
  // 0 / 1 / 2).  TTPA_DECODE_SEG_UNITS (read on every call) overrides.
  a.seg_units = segment_units(use_mfma16 ? 1 : use_mfma ? 2 : 0);
  // one thread of the main grid per segment publishes the segment's partial slots
  if ((int64_t)users * kv_heads > (int64_t)a.n_waves * kWave)
    return fail(TTPA_ERR_UNSUPPORTED, "decode: %d x %d segments need a grid of more than %d wavefronts",
                users, kv_heads, a.n_waves);
  if (k_new) {
    // The step's cache update: inside the 16x16 kernel when that is the kernel of this shape,
    // as a launch of its own in front of the attention otherwise.
    const bool vec_ok = aligned16(k_new) && aligned16(v_new) && new_user_stride % 8 == 0 &&
                        new_head_stride % 8 == 0;
    if (use_mfma16 && vec_ok) {
      a.k_new = static_cast<const uint16_t *>(k_new);
      a.v_new = static_cast<const uint16_t *>(v_new);
      a.new_us = new_user_stride, a.new_hs = new_head_stride;
    } else if (int rc = ttpa_paged_update_cache_kv(
                   const_cast<void *>(k_cache), const_cast<void *>(v_cache), k_new, v_new,
                   new_user_stride, new_head_stride, cur_pos, cur_pos_is_i64, page_table,
                   page_table_row_stride, users, kv_heads, block_size, head_size, table_width,
                   num_blocks, kv_format, stream)) {
      return rc;
    }
  }
  // armed profile events: the 16x16 kernel's launch carries them itself; the other kernels are
  // bracketed here
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  if (!use_mfma16) take_profile_events(ev0, ev1);
  if (ev0) (void)hipEventRecord(ev0, st);
  int rc = TTPA_OK;
  if (use_mfma16) {
    if (!launch_mfma16_main(a, head_size, st))
      rc = fail(TTPA_ERR_LAUNCH, "decode: cannot configure the 16x16 matrix-core kernel");
  } else if (use_mfma) {
    if (!launch_mfma_main(a, head_size, st))
      rc = fail(TTPA_ERR_LAUNCH, "decode: cannot configure the matrix-core kernel");
  } else {
    switch (head_size) {
      case 64: rc = launch_g<64>(a, g, st); break;
      case 128: rc = launch_g<128>(a, g, st); break;
      default: rc = launch_g<256>(a, g, st); break;
    }
  }
  if (ev1) (void)hipEventRecord(ev1, st);
  if (use_mfma16) take_profile_events(ev0, ev1);  // still armed only if the launch did not happen
  if (rc) return rc;
  decode_combine_kernel<<<dim3(users * kv_heads, combine_pieces(g, head_size)), dim3(256), 0, st>>>(a, g, head_size);
  return check_launch("paged_sdpa_decode");
}

extern "C" int ttpa_paged_sdpa_decode(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                      const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                      const void *k_cache, const void *v_cache,
                                      const int32_t *page_table, int64_t page_table_row_stride,
                                      const void *cur_pos, int cur_pos_is_i64, int32_t users,
                                      int32_t q_heads, int32_t kv_heads, int32_t head_size,
                                      int32_t block_size, int32_t table_width, int32_t num_blocks,
                                      float scale, int32_t kv_format, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache,
                     v_cache, page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users,
                     q_heads, kv_heads, head_size, block_size, table_width, num_blocks, scale,
                     kv_format, 0, nullptr, workspace, workspace_bytes, stream);
}

extern "C" int ttpa_paged_sdpa_decode_windowed(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, const void *k_cache, const void *v_cache,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    int32_t sliding_window, const float *attention_sink, void *workspace, size_t workspace_bytes,
    void *stream) {
  return decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache,
                     v_cache, page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users,
                     q_heads, kv_heads, head_size, block_size, table_width, num_blocks, scale,
                     kv_format, sliding_window, attention_sink, workspace, workspace_bytes, stream);
}

extern "C" int ttpa_paged_sdpa_decode_masked(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, const void *k_cache, const void *v_cache,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    const void *mask, int64_t mask_user_stride, int64_t mask_head_stride, void *workspace,
    size_t workspace_bytes, void *stream) {
  TTPA_REQUIRE(mask != nullptr, "masked decode: null mask");
  return decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache,
                     v_cache, page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users,
                     q_heads, kv_heads, head_size, block_size, table_width, num_blocks, scale,
                     kv_format, 0, nullptr, workspace, workspace_bytes, stream, nullptr, nullptr, 0, 0,
                     mask, mask_user_stride, mask_head_stride);
}

// ---- the entry point that allocates nothing ------------------------------------------------
namespace {

constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
// Workspace of ttpa_paged_update_decode_static.  In host code the name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (each GPU holds its own copy).
int static_scratch(void **out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(TTPA_ERR_LAUNCH, "static scratch: no current device (ordinals up to %d)", kMaxDevices - 1);
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return fail(TTPA_ERR_LAUNCH, "static scratch: hipGetSymbolAddress: %s", hipGetErrorString(e));
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing first calls find the same address
  }
  *out = p;
  return TTPA_OK;
}

}  // namespace

extern "C" size_t ttpa_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int ttpa_static_scratch_init(void) {
  void *p = nullptr;
  return static_scratch(&p);
}

extern "C" int ttpa_paged_update_decode_static(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, void *k_cache, void *v_cache, const void *k_new,
    const void *v_new, int64_t new_user_stride, int64_t new_head_stride,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    int32_t sliding_window, const float *attention_sink, void *stream) {
  TTPA_REQUIRE(k_new && v_new, "update + decode: null fresh K / V pointer");
  const size_t need = ttpa_paged_decode_workspace_bytes(users, q_heads, kv_heads, head_size);
  if (need == 0) return fail(TTPA_ERR_INVALID_ARGUMENT, "update + decode: bad users / heads / head_size");
  if (need > kStaticScratchBytes)
    return fail(TTPA_ERR_WORKSPACE,
                "update + decode without a workspace: this shape needs %zu bytes of partial results, the "
                "library's static scratch holds %zu; use ttpa_paged_update_decode with a caller workspace",
                need, kStaticScratchBytes);
  void *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // nothing in the workspace has to start at zero: the segment table and every partial slot that
  // the merge kernel reads are written by the main kernel of the same call
  return decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache,
                     v_cache, page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users,
                     q_heads, kv_heads, head_size, block_size, table_width, num_blocks, scale,
                     kv_format, sliding_window, attention_sink, ws, kStaticScratchBytes, stream,
                     k_new, v_new, new_user_stride, new_head_stride);
}

extern "C" int ttpa_paged_update_decode(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, void *k_cache, void *v_cache, const void *k_new,
    const void *v_new, int64_t new_user_stride, int64_t new_head_stride,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    int32_t sliding_window, const float *attention_sink, void *workspace, size_t workspace_bytes,
    void *stream) {
  TTPA_REQUIRE(k_new && v_new, "update + decode: null fresh K / V pointer");
  return decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache,
                     v_cache, page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users,
                     q_heads, kv_heads, head_size, block_size, table_width, num_blocks, scale,
                     kv_format, sliding_window, attention_sink, workspace, workspace_bytes, stream,
                     k_new, v_new, new_user_stride, new_head_stride);
}
