// Paged decode attention over a block-float-8 KV cache (dequantised inside the kernel).
//
// Same decomposition and lane mapping as the bfloat16 kernel (decode.hip): flat list of
// 64-token tiles cut into equal wavefront ranges, lane (r, c) holds elements c of token
// 4 i + r for load i, reduce-scatter of q.k over the 16 lanes of a row, one online-softmax
// stream per lane row.  What changes is the data: per token row the cache holds head_size
// element bytes (128 + signed 7-bit mantissa) and head_size / 16 shared exponent bytes.
//   * element bytes are expanded to exact bfloat16 integers in registers;
//   * for q.k the group scale 2^(e-133) multiplies the lane's partial dot product (all
//     elements a lane holds for a load belong to one 16-element group);
//   * for p.V the scale is folded into the probability (a power of two times a bfloat16 is
//     still a bfloat16, so nothing is rounded twice).
// 17 bytes are read per 16 elements instead of 32.
#include "decode_common.h"

namespace ttpa {
namespace decode {
namespace {

// 4 element bytes (128 + v) -> two packed bfloat16 pairs holding the integers v exactly.
__device__ __forceinline__ void expand4(uint32_t w, uint32_t &p01, uint32_t &p23) {
  const float f0 = (float)(w & 0xffu) - 128.f, f1 = (float)((w >> 8) & 0xffu) - 128.f;
  const float f2 = (float)((w >> 16) & 0xffu) - 128.f, f3 = (float)(w >> 24) - 128.f;
  // high halves of the floats (an integer of magnitude <= 128 is exact in 8 significand bits)
  p01 = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0),
                              0x07060302u);
  p23 = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2),
                              0x07060302u);
}

// 2^(e - 133) for a shared exponent byte; exponents below 7 (|x| < 2^-120) read as zero.
__device__ __forceinline__ float group_scale(uint32_t e) {
  return e >= 7u ? __builtin_bit_cast(float, (e - 6u) << 23) : 0.f;
}

template <int D, int G, bool BIG>
__global__ __launch_bounds__(256, 2) void paged_decode_bfp8_kernel(
    DecodeArgs a, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  static_assert(D == 64 || D == 128, "block-float-8 decode is built for head sizes 64 and 128");
  constexpr int EPL = D / 16;      // element bytes per lane per load
  constexpr int RW = EPL / 4;      // raw dwords per lane per load
  constexpr int DW = EPL / 2;      // packed bf16 pairs per lane per load
  constexpr int GPR = D / 16;      // exponent bytes per token row
  constexpr int NOFF = BIG ? 1 : 16;

  __shared__ int s_pref[kMaxUsers + 1];
  __shared__ int s_len[kMaxUsers];
  __shared__ int s_wsum[kWavesPerBlock];
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
  if (total == 0 || wave >= n_eff) {
    publish_segment_row(a, s_pref, total, n_eff, seg_units);
    return;
  }
  const int64_t x_lo = (int64_t)wave * total / n_eff;
  int64_t x = x_lo;  // set below to the unit of the first tile at or behind x_lo
  const int64_t x_hi = (int64_t)(wave + 1) * total / n_eff;
  lds_u16 *plds = s_p[wib];
  const int my_step = bitrev4(c);
  const int grp = (c * EPL) / 16;                              // exponent group of this lane
  const uint32_t lane_elem = (uint32_t)(r * D + c * EPL);      // byte offset inside a 4-row load
  const uint32_t lane_exp = (uint32_t)(r * GPR + grp);
  const int64_t slab_bytes = (int64_t)(a.bs + a.bs / 16) * D;  // one (block, head) slab

  auto locate = [&](int64_t xx) { return locate_unit(a, s_pref, s_len, xx, seg_units); };
  // byte offsets of the element rows / exponent rows of each 4-row load of a tile
  auto tile_offsets = [&](const Cursor &cu, int64_t (&eo)[NOFF], int64_t (&xo)[NOFF]) {
    const int32_t *pt_row = page_table + (int64_t)cu.u * a.pt_rs;
    const int tok0 = cu.t * kTile;
    // the 4 rows of a load never cross a block (block_size is a multiple of 16): block and row
    // advance without a division, and the table is read only where the block changes
    int col = tok0 / a.bs, row = tok0 - col * a.bs;
    int64_t slab = 0;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) {
      if (i == 0 || row == 0) {
        int phys = (col < a.w) ? __builtin_amdgcn_readfirstlane(pt_row[col]) : 0;
        if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
        slab = ((int64_t)phys * a.hkv + cu.h) * slab_bytes;
      }
      eo[i] = slab + (int64_t)row * D;
      xo[i] = slab + (int64_t)a.bs * D + (int64_t)row * GPR;
      row += 4;
      if (row >= a.bs) row = 0, ++col;
    }
  };
  auto load_tile = [&](const uint8_t *base, const int64_t (&eo)[NOFF], const int64_t (&xo)[NOFF],
                       uint32_t (&raw)[16][RW], uint32_t (&ex)[16]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint8_t *erow = BIG ? base + eo[0] + i * 4 * D : base + eo[BIG ? 0 : i];
      const uint8_t *xrow = BIG ? base + xo[0] + i * 4 * GPR : base + xo[BIG ? 0 : i];
      const uint8_t *ep = erow + static_cast<uint64_t>(lane_elem);
      if constexpr (RW == 2) {
        u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(ep));
        raw[i][0] = t.x, raw[i][1] = t.y;
      } else {
        raw[i][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(ep));
      }
      ex[i] = __builtin_nontemporal_load(xrow + static_cast<uint64_t>(lane_exp));
    }
  };
  auto load_q = [&](const Cursor &cu, uint32_t (&q)[G][DW]) {
#pragma unroll
    for (int g = 0; g < G; ++g)
      load_dwords<DW>(a.q + cu.u * a.q_us + (int64_t)(cu.h * G + g) * a.q_hs + c * EPL, q[g]);
  };
  auto expand = [&](const uint32_t (&raw)[RW], uint32_t (&out)[DW]) {
#pragma unroll
    for (int w = 0; w < RW; ++w) expand4(raw[w], out[2 * w], out[2 * w + 1]);
  };

  Cursor cur = locate_unit(a, s_pref, s_len, x_lo, seg_units, &x);
  int64_t eo[NOFF], xo[NOFF];
  uint32_t kraw[16][RW], kex[16], q[G][DW];
  tile_offsets(cur, eo, xo);
  load_tile(a.k, eo, xo, kraw, kex);
  load_q(cur, q);
  publish_segment_row(a, s_pref, total, n_eff, seg_units);

  float m[G], l[G], acc[G][1][EPL];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][0][e] = 0.f;
  }

  auto process_tile = [&](auto has_next_tag) {
    constexpr bool has_next = decltype(has_next_tag)::value;
    const int nvalid = cur.len - cur.t * kTile;
    uint32_t vraw[16][RW], vex[16];
    load_tile(a.v, eo, xo, vraw, vex);
    __builtin_amdgcn_sched_barrier(0);

    // ---- scores: scaled partial dot products, reduce-scattered over the 16 lanes of a row --
    float sc[16][G];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      uint32_t kw[DW];
      expand(kraw[i], kw);
      const float gs = group_scale(kex[i]);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < DW; ++j) t = dot2(kw[j], q[g][j], t);
        sc[i][g] = t * gs;
      }
    }
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      // level 1: loads (2b, 2b+1) on lane bit 3; level 2: on bit 2; level 3: bit 1; level 4: bit 0
      float l1[8], l2[4], l3[2];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const bool up = (c >> 3) & 1;
        l1[b] = (up ? sc[2 * b + 1][g] : sc[2 * b][g]) +
                rs_exchange<1>(up ? sc[2 * b][g] : sc[2 * b + 1][g]);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const bool up = (c >> 2) & 1;
        l2[b] = (up ? l1[2 * b + 1] : l1[2 * b]) + rs_exchange<2>(up ? l1[2 * b] : l1[2 * b + 1]);
      }
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const bool up = (c >> 1) & 1;
        l3[b] = (up ? l2[2 * b + 1] : l2[2 * b]) + rs_exchange<3>(up ? l2[2 * b] : l2[2 * b + 1]);
      }
      const bool up = c & 1;
      s[g] = (up ? l3[1] : l3[0]) + rs_exchange<4>(up ? l3[0] : l3[1]);
    }

    __builtin_amdgcn_sched_barrier(0);
    const bool same_seg = has_next && cur.tiles_left > 1;
    Cursor nxt = cur;
    int64_t neo[NOFF], nxo[NOFF];
#pragma unroll
    for (int i = 0; i < NOFF; ++i) neo[i] = eo[i], nxo[i] = xo[i];
    if constexpr (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate(x + 1);
      }
      tile_offsets(nxt, neo, nxo);
      load_tile(a.k, neo, nxo, kraw, kex);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- online softmax, one stream per lane row ------------------------------------------
    const int nbelow = cur.lo - cur.t * kTile;  // sliding window: only in a segment's first tile
    const bool valid = 4 * my_step + r < nvalid && 4 * my_step + r >= nbelow;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float sv = valid ? s[g] * a.scale_log2e : -INFINITY;
      float mx = fmaxf(m[g], row16_max(sv));
      float msafe = (mx == -INFINITY) ? 0.f : mx;
      float alpha = __builtin_amdgcn_exp2f(m[g] - msafe);
      float p = __builtin_amdgcn_exp2f(sv - msafe);
      uint32_t pb = f32_to_bf16_bits(p);
      l[g] = l[g] * alpha + __builtin_bit_cast(float, pb << 16);
      m[g] = mx;
      plds[(r * G + g) * 16 + my_step] = (uint16_t)pb;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][0][e] *= alpha;
    }

    // ---- output accumulation: two tokens per dot2, group scale folded into the weight -------
    const lds_u32 *pw = reinterpret_cast<const lds_u32 *>(plds) + r * G * 8;
#pragma unroll
    for (int k2 = 0; k2 < 8; ++k2) {
      // unattended rows carry weight 0 and must not contribute stale Inf/NaN: the expanded
      // integers are always finite, and a zero weight stays zero after scaling
      const float s0 = (4 * (2 * k2) + r < nvalid) ? group_scale(vex[2 * k2]) : 0.f;
      const float s1 = (4 * (2 * k2 + 1) + r < nvalid) ? group_scale(vex[2 * k2 + 1]) : 0.f;
      uint32_t va[DW], vb[DW];
      expand(vraw[2 * k2], va);
      expand(vraw[2 * k2 + 1], vb);
      uint32_t pk[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const uint32_t pp = pw[g * 8 + k2];
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        bf2 t;
        t[0] = (__bf16)(bf16_lo(pp) * s0);  // exact: bfloat16 times a power of two
        t[1] = (__bf16)(bf16_hi(pp) * s1);
        pk[g] = __builtin_bit_cast(uint32_t, t);
      }
#pragma unroll
      for (int j = 0; j < DW; ++j) {
        const uint32_t even = __builtin_amdgcn_perm(vb[j], va[j], 0x05040100u);
        const uint32_t odd = __builtin_amdgcn_perm(vb[j], va[j], 0x07060302u);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          acc[g][0][2 * j] = dot2(even, pk[g], acc[g][0][2 * j]);
          acc[g][0][2 * j + 1] = dot2(odd, pk[g], acc[g][0][2 * j + 1]);
        }
      }
    }

    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wave + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        write_partial<D, 1, EPL>(slot, g, G, r, c, m[g], l[g], acc[g]);
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][0][e] = 0.f;
      }
      if constexpr (has_next) load_q(nxt, q);
    }
    cur = nxt;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) eo[i] = neo[i], xo[i] = nxo[i];
    x += same_seg ? 1 : 1 + seg_units;
  };
  // the unit of the tile behind the current one: the next, or behind the next segment's leading units
  auto next_tile_unit = [&]() { return x + (cur.tiles_left > 1 ? 1 : 1 + seg_units); };
  while (next_tile_unit() < x_hi) process_tile(std::true_type{});
  process_tile(std::false_type{});
}

template <int D, int G>
void launch(const DecodeArgs &a, hipStream_t st) {
  const int blocks = a.n_waves / kWavesPerBlock;
  const size_t pad = blocks <= device_cus() ? 65536 : 0;  // one workgroup per CU
  if (a.bs % kTile == 0)
    paged_decode_bfp8_kernel<D, G, true><<<dim3(blocks), dim3(256), pad, st>>>(a, a.pt, a.cur);
  else
    paged_decode_bfp8_kernel<D, G, false><<<dim3(blocks), dim3(256), pad, st>>>(a, a.pt, a.cur);
}

template <int D>
bool launch_g(const DecodeArgs &a, int g, hipStream_t st) {
  switch (g) {
    case 1: launch<D, 1>(a, st); return true;
    case 2: launch<D, 2>(a, st); return true;
    case 3: launch<D, 3>(a, st); return true;
    case 4: launch<D, 4>(a, st); return true;
    case 5: launch<D, 5>(a, st); return true;
    case 6: launch<D, 6>(a, st); return true;
    case 7: launch<D, 7>(a, st); return true;
    case 8: launch<D, 8>(a, st); return true;
    default: return false;
  }
}

}  // namespace

bool launch_bfp8_main(const DecodeArgs &a, int head_size, int g, hipStream_t st) {
  if (head_size == 64) return launch_g<64>(a, g, st);
  if (head_size == 128) return launch_g<128>(a, g, st);
  return false;
}

}  // namespace decode
}  // namespace ttpa
