// Paged decode attention, matrix-core formulation for wide head groups and for the
// block-float-8 cache.
//
// The work decomposition is the one of decode.hip (flat list of 64-token tiles cut into
// equal wavefront ranges, one partial per (wavefront, segment), merge kernel afterwards).
// What differs is the arithmetic inside a wavefront.  The VALU kernel spends per-head work
// on every tile (dot products, cross-lane reduction, softmax), which stops hiding behind
// the HBM stream at 8 query heads per KV head, and the block-float-8 cache adds a byte ->
// bfloat16 expansion on top.  Here a tile goes global -> registers -> wave-private LDS
// and the two products run on v_mfma_f32_32x32x16_bf16 with the G query heads of the group as
// the 32-wide N dimension:
//   S^T[key, head] = K[key, :] . Q[head, :]        A = K rows from LDS, B = Q in registers
//   O^T[d, head]  += V^T[d, key] . P^T[key, head]  A = V through the transposing LDS load
// Each lane owns one head column, so softmax statistics are per-lane scalars and the
// probabilities are already the B operand of the second product.  Cost per tile is
// independent of G (up to 32 heads per KV head).
//
// Block-float-8 cache: the tile is expanded to half precision on its way into LDS and the
// products run on v_mfma_f32_32x32x16_f16.  An element byte b = 128 + v becomes the half
// 0x6400 | b = 1024 + b with one byte permute per element pair, and one packed fma per pair
// turns it into v * 2^(e - eref) exactly (e the group's exponent byte, eref the largest
// exponent byte of the tile; groups more than 2^24 below it flush to zero).  The tile's K
// factor 2^(eref - 133) joins the softmax scale.  V tiles are brought to a running largest
// exponent of the segment the way scores are brought to a running maximum: the tile's factor
// multiplies the probabilities, a raised reference rescales the accumulator, and the segment's
// partial is multiplied by 2^(reference - 133) when it is written.  Q is converted to half
// precision once per segment, scaled by a power of two so that its largest element is in [1, 2).
//
// LDS: 37 KiB per wavefront (K rows padded to 68 dwords, V rows to 80), four wavefronts
// per workgroup, one workgroup per CU.
#include "decode_common.h"

namespace ttpa {
namespace decode {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxUsersMfma = 1024;

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

template <bool F16>
__device__ __forceinline__ floatx16 mma(const u32x4 &x, const u32x4 &y, const floatx16 &c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, x),
                                                  __builtin_bit_cast(halfx8, y), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
}

template <int D, bool BFP8, bool BIG>
__global__ __launch_bounds__(256, 1) void paged_decode_mfma_kernel(
    DecodeArgs a, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  static_assert(D == 64 || D == 128, "matrix-core decode is built for head sizes 64 and 128");
  constexpr int KS = D + 8, VS = D + 32;    // LDS row strides in elements
  constexpr int KSTEPS = D / 16, DBLK = D / 32;
  // staging geometry: a load instruction covers RPL whole token rows
  constexpr int BPE = BFP8 ? 1 : 2;         // bytes per cache element
  constexpr int LPR = D * BPE / 16;         // lanes per token row (16 bytes per lane)
  constexpr int RPL = 64 / LPR;             // rows per load
  constexpr int NL = kTile / RPL;           // loads per tile and tensor
  constexpr int GPR = D / 16;               // exponent bytes per row (block-float-8)
  constexpr int NOFF = BIG ? 1 : NL;

  __shared__ int s_pref[kMaxUsersMfma + 1];
  __shared__ int s_len[kMaxUsersMfma];
  __shared__ int s_wsum[kWavesPerBlock];
  extern __shared__ __attribute__((aligned(16))) uint16_t tiles[];

  const int seg_units = a.seg_units;
  build_prefix(a, cur_pos, s_pref, s_len, s_wsum, seg_units);

  const int lane = threadIdx.x & 63;
  const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
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
  uint16_t *ks = tiles + wib * (kTile * (KS + VS));
  uint16_t *vs = ks + kTile * KS;
  const int G = a.hq / a.hkv;

  // staging lane mapping
  const int sr = lane / LPR, sc = lane % LPR;
  const uint32_t lane_bytes = (uint32_t)(sr * D * BPE + sc * 16);
  // block-float-8: one group per lane; its exponent byte is fetched inside its aligned dword
  // and cut out when the tile is staged (a byte load is widened where it is issued, which
  // makes the loop wait for the load at once)
  const uint32_t lane_exp = (uint32_t)((sr * GPR + sc) & ~3);
  const uint32_t exp_shift = (uint32_t)(8 * ((sr * GPR + sc) & 3));
  const int64_t slab = BFP8 ? (int64_t)(a.bs + a.bs / 16) * D : (int64_t)a.bs * D * 2;  // bytes

  auto locate = [&](int64_t xx) { return locate_unit(a, s_pref, s_len, xx, seg_units); };
  auto tile_offsets = [&](const Cursor &cu, int64_t (&eo)[NOFF], int64_t (&xo)[NOFF]) {
    const int32_t *pt_row = page_table + (int64_t)cu.u * a.pt_rs;
    const int tok0 = cu.t * kTile;
    // the rows of a load never cross a block (block_size is a multiple of RPL): block and row
    // advance without a division, and the table is read only where the block changes
    int col = tok0 / a.bs, row = tok0 - col * a.bs;
    int64_t base = 0;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) {
      if (i == 0 || row == 0) {
        int phys = (col < a.w) ? __builtin_amdgcn_readfirstlane(pt_row[col]) : 0;
        if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
        base = ((int64_t)phys * a.hkv + cu.h) * slab;
      }
      eo[i] = base + (int64_t)row * D * BPE;
      xo[i] = base + (int64_t)a.bs * D + (int64_t)row * GPR;
      row += RPL;
      if (row >= a.bs) row = 0, ++col;
    }
  };
  auto fetch = [&](const uint8_t *base, const int64_t (&eo)[NOFF], const int64_t (&xo)[NOFF],
                   u32x4 (&raw)[NL], uint32_t (&ex)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint8_t *erow = BIG ? base + eo[0] + i * (RPL * D * BPE) : base + eo[BIG ? 0 : i];
      raw[i] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4 *>(erow + static_cast<uint64_t>(lane_bytes)));
      if constexpr (BFP8) {
        const uint8_t *xrow = BIG ? base + xo[0] + i * (RPL * GPR) : base + xo[BIG ? 0 : i];
        ex[i] = __builtin_nontemporal_load(
            reinterpret_cast<const uint32_t *>(xrow + static_cast<uint64_t>(lane_exp)));
      }
    }
  };
  // registers -> LDS tile (rows past `nvalid` are cleared when `clear` is set); `eref` is the
  // tile's reference exponent (block-float-8)
  auto stage = [&](uint16_t *dst, int stride, const u32x4 (&raw)[NL], const uint32_t (&ex)[NL],
                   int eref, int nvalid, bool clear) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int row = RPL * i + sr;
      const bool keep = !clear || row < nvalid;
      if constexpr (BFP8) {
        // 2^(e - eref) as a half: through the float with exponent field e - eref + 127; the
        // conversion is exact down to 2^-24 and gives zero below
        const int field = max((int)((ex[i] >> exp_shift) & 0xffu) - (eref - 127), 0);
        const float sf = keep ? __builtin_bit_cast(float, (uint32_t)min(field, 127) << 23) : 0.f;
        const _Float16 sh = (_Float16)sf;
        const halfx2 s2 = {sh, sh};
        const halfx2 c2 = s2 * halfx2{(_Float16)-1152.f, (_Float16)-1152.f};
        uint32_t o[8];
        expand4_half(raw[i].x, s2, c2, o[0], o[1]);
        expand4_half(raw[i].y, s2, c2, o[2], o[3]);
        expand4_half(raw[i].z, s2, c2, o[4], o[5]);
        expand4_half(raw[i].w, s2, c2, o[6], o[7]);
        uint4 *p = reinterpret_cast<uint4 *>(dst + row * stride + sc * 16);
        p[0] = make_uint4(o[0], o[1], o[2], o[3]);
        p[1] = make_uint4(o[4], o[5], o[6], o[7]);
      } else {
        uint4 v = keep ? make_uint4(raw[i].x, raw[i].y, raw[i].z, raw[i].w) : make_uint4(0, 0, 0, 0);
        *reinterpret_cast<uint4 *>(dst + row * stride + sc * 8) = v;
      }
    }
  };
  // largest exponent byte of the tile's attended rows (block-float-8)
  auto tile_exponent = [&](const uint32_t (&ex)[NL], int nvalid, bool partial) {
    uint32_t e = 0;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const bool ok = !partial || RPL * i + sr < nvalid;
      e = max(e, ok ? (ex[i] >> exp_shift) & 0xffu : 0u);
    }
    return (int)wave_max_u32(e);
  };
  // Q fragments: B operand, lane n = head of the group (zero beyond G).  Block-float-8: half
  // precision, scaled by 2^(127 - eq) with eq the largest exponent field of the segment's Q.
  int eq = 0;
  auto load_q = [&](const Cursor &cu, u32x4 (&qf)[KSTEPS]) {
    const uint16_t *qp = a.q + cu.u * a.q_us + (int64_t)(cu.h * G + min(n, G - 1)) * a.q_hs + 8 * h;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      uint4 t = *reinterpret_cast<const uint4 *>(qp + 16 * s);
      if (n >= G) t = make_uint4(0, 0, 0, 0);
      qf[s] = u32x4{t.x, t.y, t.z, t.w};
    }
    if constexpr (BFP8) {
      uint32_t em = 0;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          em = max(em, max((qf[s][j] >> 7) & 0xffu, (qf[s][j] >> 23) & 0xffu));
      eq = (int)min(wave_max_u32(em), 253u);
      const float qs = __builtin_bit_cast(float, (uint32_t)(254 - eq) << 23);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          qf[s][j] = pack_half2(bf16_lo(qf[s][j]) * qs, bf16_hi(qf[s][j]) * qs);
    }
  };

  Cursor cur = locate_unit(a, s_pref, s_len, x_lo, seg_units, &x);
  int64_t eo[NOFF], xo[NOFF];
  u32x4 kraw[NL], vraw[NL];
  uint32_t kex[NL], vex[NL];
  u32x4 qf[KSTEPS];
  tile_offsets(cur, eo, xo);
  fetch(a.k, eo, xo, kraw, kex);
  fetch(a.v, eo, xo, vraw, vex);
  load_q(cur, qf);
  publish_segment_row(a, s_pref, total, n_eff, seg_units);

  floatx16 acc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  int ev_run = 0;  // block-float-8: reference exponent of the V accumulator

  auto process_tile = [&](auto has_next_tag) {
    constexpr bool has_next = decltype(has_next_tag)::value;
    const int nvalid = cur.len - cur.t * kTile;
    const bool partial = nvalid < kTile;
    const int nbelow = cur.lo - cur.t * kTile;  // sliding window: > 0 only in a segment's first tile
    // ---- this tile: registers -> LDS; next tile: global -> registers ----------------------
    const bool same_seg = has_next && cur.tiles_left > 1;
    Cursor nxt = cur;
    auto prefetch_next = [&]() {
      if constexpr (has_next) {
        if (same_seg) {
          nxt.t = cur.t + 1;
          nxt.tiles_left = cur.tiles_left - 1;
        } else {
          nxt = locate(x + 1);
        }
        tile_offsets(nxt, eo, xo);
        fetch(a.k, eo, xo, kraw, kex);
        fetch(a.v, eo, xo, vraw, vex);
      }
    };
    int eref_k = 0, eref_v = 0;
    if constexpr (BFP8) {
      // move the raw tile to a second register set so that the loads of the next tile are in
      // flight while this one is expanded and staged
      u32x4 kcur[NL], vcur[NL];
      uint32_t kexc[NL], vexc[NL];
#pragma unroll
      for (int i = 0; i < NL; ++i) kcur[i] = kraw[i], vcur[i] = vraw[i], kexc[i] = kex[i], vexc[i] = vex[i];
      prefetch_next();
      __builtin_amdgcn_sched_barrier(0);
      eref_k = tile_exponent(kexc, nvalid, partial);
      eref_v = tile_exponent(vexc, nvalid, partial);
      stage(ks, KS, kcur, kexc, eref_k, nvalid, partial);
      stage(vs, VS, vcur, vexc, eref_v, nvalid, partial);
    } else {
      stage(ks, KS, kraw, kex, 0, nvalid, false);
      stage(vs, VS, vraw, vex, 0, nvalid, partial);  // unattended V rows must not carry Inf / NaN
      prefetch_next();
    }

    // ---- S^T = K . Q^T ----------------------------------------------------------------------
    floatx16 st[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[kb][r] = 0.f;
      const uint16_t *krow = ks + (32 * kb + n) * KS + 8 * h;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const uint4 kq = *reinterpret_cast<const uint4 *>(krow + 16 * s);
        st[kb] = mma<BFP8>(u32x4{kq.x, kq.y, kq.z, kq.w}, qf[s], st[kb]);
      }
    }
    // ---- online softmax, one head per lane --------------------------------------------------
    if (partial || nbelow > 0) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = 32 * kb + 8 * (r >> 2) + 4 * h + (r & 3);
          if (key >= nvalid || key < nbelow) st[kb][r] = -INFINITY;
        }
    }
    // > 0 or < 0: the maximum is tracked on scaled scores.  Block-float-8: the factors taken
    // out of the K tile and out of Q come back here.
    const float scale = BFP8 ? __builtin_ldexpf(a.scale_log2e, eref_k + eq - 260) : a.scale_log2e;
    if (a.mask != nullptr) {  // an additive mask row per (user, head), brought to the units of the raw scores
      const float unit = 1.4426950408889634f / scale;
      const uint16_t *mrow = a.mask + cur.u * a.mask_us + (int64_t)(cur.h * G + min(n, G - 1)) * a.mask_hs +
                             cur.t * kTile + 4 * h;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = 32 * kb + 8 * (r >> 2) + (r & 3);
          if (key + 4 * h < nvalid) st[kb][r] += bf16_lo(mrow[key]) * unit;
        }
    }
    float mloc = fmaxf(st[0][0], st[1][0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(st[0][r], st[1][r]));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    mloc *= scale;
    // a negative scale would turn the max into a min; scores are scaled before comparing then
    if (scale < 0.f) {
      mloc = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, st[kb][r] * scale);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    }
    const float m_new = fmaxf(m_run, mloc);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    m_run = m_new;
    float lsum = 0.f;
    u32x4 pf[2][2];
    float alpha_acc = alpha;
    if constexpr (BFP8) {
      // bring this tile's V factor and the accumulator to the larger reference exponent
      const int ev_new = max(ev_run, eref_v);
      const float pscale = __builtin_ldexpf(1.f, eref_v - ev_new);
      alpha_acc = alpha * __builtin_ldexpf(1.f, ev_run - ev_new);
      ev_run = ev_new;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(st[kb][8 * s + e], scale, -m_safe));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(st[kb][8 * s + e + 1], scale, -m_safe));
            lsum += p0 + p1;  // half-precision rounding of the weights is 2^-12: not tracked
            pf[kb][s][e >> 1] = pack_half2(p0 * pscale, p1 * pscale);
          }
    } else {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          bf16x8 pb8;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float p = __builtin_amdgcn_exp2f(fmaf(st[kb][8 * s + e], scale, -m_safe));
            __bf16 pb = (__bf16)p;
            lsum += (float)pb;  // the normaliser sums the weights that multiply V
            pb8[e] = pb;
          }
          pf[kb][s] = __builtin_bit_cast(u32x4, pb8);
        }
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha_acc != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= alpha_acc;
    }
    // ---- O^T += V^T . P^T (V^T fragments through the transposing LDS load) -------------------
    const int grp = lane >> 4, a16 = lane & 15;
    const uint16_t *vbase = vs + (4 * (grp >> 1) + (a16 >> 2)) * VS + 16 * (grp & 1) + 4 * (a16 & 3);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const uint16_t *vk = vbase + (32 * kb + 16 * s) * VS;
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          typedef __attribute__((address_space(3))) shortx4 *lds_v4;
          shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 32 * db));
          shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 8 * VS + 32 * db));
          const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
          acc[db] = mma<BFP8>(u32x4{l2.x, l2.y, h2.x, h2.y}, pf[kb][s], acc[db]);
        }
      }

    // ---- close the segment --------------------------------------------------------------------
    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wave + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
      const float l_tot = l_run + __shfl_xor(l_run, 32);
      if constexpr (BFP8) {
        const float vout = __builtin_ldexpf(1.f, ev_run - 133);
#pragma unroll
        for (int i = 0; i < DBLK; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][r] *= vout;
        ev_run = 0;
      }
      if (n < G) {
        float *dst = slot + n * D + 4 * h;
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            *reinterpret_cast<float4 *>(dst + 32 * db + 8 * j) = make_float4(
                acc[db][4 * j], acc[db][4 * j + 1], acc[db][4 * j + 2], acc[db][4 * j + 3]);
        if (h == 0) {
          slot[G * D + n] = m_run;
          slot[G * D + G + n] = l_tot;
        }
      }
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
      m_run = -INFINITY;
      l_run = 0.f;
      if constexpr (has_next) load_q(nxt, qf);
    }
    cur = nxt;
    x += same_seg ? 1 : 1 + seg_units;
  };
  // the unit of the tile behind the current one: the next, or behind the next segment's leading units
  auto next_tile_unit = [&]() { return x + (cur.tiles_left > 1 ? 1 : 1 + seg_units); };
  while (next_tile_unit() < x_hi) process_tile(std::true_type{});
  process_tile(std::false_type{});
}

template <int D, bool BFP8>
bool launch(const DecodeArgs &a, hipStream_t st) {
  const int blocks = a.n_waves / kWavesPerBlock;
  const size_t lds = (size_t)kWavesPerBlock * kTile * ((D + 8) + (D + 32)) * 2;
  if (a.bs % kTile == 0) {
    static std::atomic<uint64_t> lds_ready{0};
    if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_mfma_kernel<D, BFP8, true>), lds, lds_ready))
      return false;
    paged_decode_mfma_kernel<D, BFP8, true><<<dim3(blocks), dim3(256), lds, st>>>(a, a.pt, a.cur);
  } else {
    static std::atomic<uint64_t> lds_ready{0};
    if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_mfma_kernel<D, BFP8, false>), lds, lds_ready))
      return false;
    paged_decode_mfma_kernel<D, BFP8, false><<<dim3(blocks), dim3(256), lds, st>>>(a, a.pt, a.cur);
  }
  return true;
}

}  // namespace

bool mfma_decode_supported(const DecodeArgs &a, int head_size, int g) {
  if ((head_size != 64 && head_size != 128) || g > 32 || a.users > kMaxUsersMfma) return false;
  // a load instruction covers 1 KiB of whole token rows, which must not straddle a block
  const int row_bytes = head_size * (a.kv_format == TTPA_KV_BFP8 ? 1 : 2);
  return a.bs % (1024 / row_bytes) == 0;
}

bool launch_mfma_main(const DecodeArgs &a, int head_size, hipStream_t st) {
  const bool bfp8 = a.kv_format == TTPA_KV_BFP8;
  if (head_size == 64) return bfp8 ? launch<64, true>(a, st) : launch<64, false>(a, st);
  if (head_size == 128) return bfp8 ? launch<128, true>(a, st) : launch<128, false>(a, st);
  return false;
}

}  // namespace decode
}  // namespace ttpa
