// Paged decode attention on the 16x16x32 matrix-core shape: up to 16 query heads per KV head,
// 80 KiB of LDS per workgroup; head sizes 64, 128 and 256 with a block-float-8 cache (expanded
// to half precision) or a bfloat16 cache.
//
// Work decomposition, partial slots and merge kernel are those of decode.hip, with tiles of
// 16 KiB of 16-bit elements (128, 64 or 32 tokens at head size 64, 128, 256; 8 KiB = 32 tokens
// for a bfloat16 cache with head size 128, see tile_bytes).  Inside a wavefront a tile of K,
// then of V, goes global -> registers -> a wave-private LDS buffer of that size that both
// tensors use in turn:
//   stage K(t) | prefetch K(t+1) | S^T = K Q^T | softmax | stage V(t) | prefetch V(t+1) | O^T += V^T P^T
// so every global load has three quarters of a tile period to arrive.  The byte -> half
// expansion of the block-float-8 cache is the one of decode_mfma.hip (one permute and one
// packed fma per element pair, exponents relative to the tile's largest, running reference
// exponent for the V accumulator).
//
// FUSED: the kernel also performs the decode step's cache update.  The token at cur_pos of a
// user sits in the last tile of each of its segments, and that tile belongs to exactly one
// wavefront: it takes the token's K / V rows from the fresh activations instead of the cache
// (quantising them for a block-float-8 cache) and stores them into the cache, so nobody
// depends on a separate update launch.  The fresh rows of a segment's (user, head) are
// requested where its Q rows are, once per segment (that block has its own waits; a request
// inside the per-tile path would make the wait-count pass drain the tile loads in the
// steady-state loop).  Users whose position is negative (padded rows) attend nothing; their
// write follows the update operator's rule for negative positions and is done by the thread
// that publishes their segment.
//
// v_mfma_f32_16x16x32_{f16,bf16} with the heads as the 16-wide N dimension:
//   S^T block b (16 keys):  A = K rows 16 b + lane%16, 8 elements per lane and k-step
//                           B = Q, lane%16 = head;   C: lane (head, quad) holds keys 16 b + 4 quad + r
//   O^T block db (16 d):    the 32 k slots of a step are the keys lane (., quad) already holds
//                           from blocks 2 s and 2 s + 1, so the probabilities are the B operand
//                           as they are; A = V^T through two transposing LDS loads (4 keys each)
// Compared with the 32x32x16 kernel, a lane carries half the scores and half the
// accumulator, and the matrix pipe is busy half as long per tile.
//
// LDS tile: rows of 2 * head_size bytes, unpadded, 16-byte chunks stored at
// chunk ^ (row & 15) for K (A-operand reads: 16 rows, one chunk column) and at
// chunk ^ (2 y | y & 1), y = row & 7, for V (transposing reads: 32 lanes cover 8 rows x 2
// chunks); both make the staging writes of two neighbouring rows land in different banks too.
// (The exchange stays inside an aligned group of 16 chunks = 256 bytes = every bank once.)
// Head size 64: a row is half a bank period, so two neighbouring rows already differ in their
// banks and the keys are taken from row / 2: (row / 2) & 7 and y = (row / 2) & 3.
//
// Where a tile's rows sit in the cache (RUNS): one run of consecutive rows when a block holds
// whole tiles; two runs of half a tile when block_size is a multiple of half a tile (block size
// 32 with head size 128, the serving default; 64 with 64; 16 with 256); four runs of a quarter
// tile when it is a multiple of a quarter tile (16 with 128; 32 with 64; 8 with 256); otherwise
// one run per load instruction.  A run costs a block-table lookup and a 64-bit base, which are
// scalar registers, the resource this kernel is short of.
//
// This header holds the kernel and its launcher; one translation unit per head size
// instantiates it (decode_mfma16_d64.hip, _d128.hip, _d256.hip).
#pragma once
#include "decode_common.h"

namespace ttpa {
namespace decode {
namespace {

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxUsers16 = kMaxUsers;  // the library-wide limit: 16 KiB of prefix tables
// Bytes of a tile's K (or V) rows as 16-bit elements, i.e. of a wavefront's LDS buffer: 16 KiB
// (128 / 64 / 32 tokens at head size 64 / 128 / 256), except 8 KiB (32 tokens) for a bfloat16
// cache with head size 128.  A wavefront has one tile of K and one of V in flight; the kernel
// ends when the slowest wavefront has drained its last tile, and wavefronts of one launch finish
// several microseconds apart (the XCDs do not get equal shares of the HBM bandwidth), so a
// shorter tile shortens that tail: config 2's step 58.7 -> 57.8 us, config 4's 549 -> 543 us.
// The block-float-8 cache moves half the bytes per token and loses with the shorter tile
// (44.1 -> 46.2 us on config 5).
template <int D, bool BFP8>
constexpr int tile_bytes() {
  return (D == 128 && !BFP8) ? 8192 : 16384;
}

template <bool F16>
__device__ __forceinline__ floatx4 mma16(const u32x4 &x, const u32x4 &y, const floatx4 &c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, x),
                                                  __builtin_bit_cast(halfx8, y), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
}

// The cache write of a user whose position is negative, by one thread per (user, kv head):
// position -k counts from the end of the user's table (the update operator's floor rule:
// column = floor(pos / bs) taken from the end once, row = pos mod bs); positions that still fall
// outside the table and blocks outside the cache are skipped.
template <bool BFP8, int D>
__device__ inline void write_negative_position(const DecodeArgs &a, const int32_t *page_table,
                                               const void *cur_pos, int seg) {
  if (seg >= a.users * a.hkv) return;
  const int u = seg / a.hkv, h = seg - u * a.hkv;
  const int64_t pos = load_index(cur_pos, a.cur_i64, u);
  if (pos >= 0) return;
  int64_t col = pos / a.bs, rem = pos - col * a.bs;
  if (rem < 0) rem += a.bs, col -= 1;
  col += a.w;
  if (col < 0 || col >= a.w) return;
  const int phys = page_table[(int64_t)u * a.pt_rs + col];
  if ((unsigned)phys >= (unsigned)a.nb) return;
  const uint16_t *src[2] = {a.k_new + u * a.new_us + h * a.new_hs, a.v_new + u * a.new_us + h * a.new_hs};
  uint8_t *dst[2] = {const_cast<uint8_t *>(a.k), const_cast<uint8_t *>(a.v)};
  for (int t = 0; t < 2; ++t) {
    if constexpr (BFP8) {
      uint8_t *slab = dst[t] + ((int64_t)phys * a.hkv + h) * (int64_t)(a.bs + a.bs / 16) * D;
      for (int grp = 0; grp < D / 16; ++grp) {
        const uint4 lo = *reinterpret_cast<const uint4 *>(src[t] + 16 * grp);
        const uint4 hi = *reinterpret_cast<const uint4 *>(src[t] + 16 * grp + 8);
        const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        uint32_t bytes[4];
        const uint32_t e = bfp8_encode16(w, bytes);
        *reinterpret_cast<uint4 *>(slab + rem * D + 16 * grp) = make_uint4(bytes[0], bytes[1], bytes[2], bytes[3]);
        slab[(int64_t)a.bs * D + rem * (D / 16) + grp] = (uint8_t)e;
      }
    } else {
      uint16_t *row = reinterpret_cast<uint16_t *>(dst[t]) + (((int64_t)phys * a.hkv + h) * a.bs + rem) * D;
      for (int c = 0; c < D / 8; ++c)
        *reinterpret_cast<uint4 *>(row + 8 * c) = *reinterpret_cast<const uint4 *>(src[t] + 8 * c);
    }
  }
}

// RUNS: 1, 2, 4, or 0 for one run per load.  MASKED: an additive mask row per (user, head) joins the
// scores (a.mask; the form of a pass that is not causal, built with RUNS = 0 and without the update).
template <int D, bool BFP8, int RUNS, bool FUSED, bool MASKED = false>
__global__ __launch_bounds__(256, 1) void paged_decode_mfma16_kernel(
    DecodeArgs a, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  static_assert(D == 64 || D == 128 || D == 256, "shapes built");
  constexpr int kTileBytes = tile_bytes<D, BFP8>();
  constexpr int TILE = kTileBytes / (2 * D);  // tokens per tile
  constexpr int ROWB = 2 * D;                 // bytes of a tile row in LDS
  constexpr int KSTEPS = D / 32, DBLK = D / 16;
  constexpr int KBLK = TILE / 16;     // score blocks (16 keys each) per tile
  constexpr int PSTEPS = TILE / 32;   // k-steps of the second product per tile
  // staging geometry: 16 bytes per lane, so a load instruction covers (head size 128) 8 whole
  // token rows of element bytes or 4 of bfloat16
  constexpr int BPE = BFP8 ? 1 : 2;   // bytes per cache element
  constexpr int LPR = D * BPE / 16;   // lanes per token row
  constexpr int RPL = 64 / LPR;       // rows per load
  constexpr int NL = TILE / RPL;      // loads per tile and tensor
  constexpr int GPR = D / 16;         // exponent bytes per row (block-float-8)
  constexpr int NOFF = RUNS == 0 ? NL : RUNS;  // runs of consecutive cache rows per tile
  constexpr int LPO = NL / NOFF;               // loads per run
  static_assert(NL % NOFF == 0, "a run is a whole number of loads");

  __shared__ int s_pref[kMaxUsers16 + 1];
  __shared__ int s_len[kMaxUsers16];
  __shared__ int s_wsum[kWavesPerBlock];
  extern __shared__ __attribute__((aligned(16))) uint8_t tiles[];

  const int seg_units = a.seg_units;
  build_prefix<TILE>(a, cur_pos, s_pref, s_len, s_wsum, seg_units);

  const int lane = threadIdx.x & 63;
  const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, quad = lane >> 4;
  const int wave = blockIdx.x * kWavesPerBlock + wib;
  // The flat list in units: per segment `seg_units` units that stand for the cost of opening it,
  // then its tiles.  A range of more than seg_units units holds at least one tile.
  const int total_units = __builtin_amdgcn_readfirstlane(s_pref[a.users]);
  const int64_t total = (int64_t)total_units * a.hkv;
  const int64_t max_ranges = total / (seg_units + 1);
  const int n_eff = (int)(max_ranges < a.n_waves ? max_ranges : a.n_waves);
  if constexpr (FUSED) write_negative_position<BFP8, D>(a, page_table, cur_pos, blockIdx.x * 256 + threadIdx.x);
  if (total == 0 || wave >= n_eff) {
    publish_segment_row(a, s_pref, total, n_eff, seg_units);
    return;
  }
  const int64_t x_lo = (int64_t)wave * total / n_eff;
  const int64_t x_hi = (int64_t)(wave + 1) * total / n_eff;
  int64_t x = x_lo;  // set below to the unit of the first tile at or behind x_lo
  uint8_t *tile = tiles + wib * kTileBytes;
  const int G = a.hq / a.hkv;

  // staging lane mapping and swizzled write positions
  const int sr = lane / LPR, sc = lane % LPR;
  const uint32_t lane_bytes = (uint32_t)(sr * D * BPE + sc * 16);
  // block-float-8: the lane's exponent byte (row sr, group sc) is fetched inside its aligned
  // dword and cut out when the tile is staged: a byte load is widened where it is issued, which
  // would make the loop wait for the next tile's exponents at the end of every iteration
  const uint32_t lane_exp = (uint32_t)((sr * GPR + sc) & ~3);
  const uint32_t exp_shift = (uint32_t)(8 * (sc & 3));
  const int64_t slab = BFP8 ? (int64_t)(a.bs + a.bs / 16) * D : (int64_t)a.bs * D * 2;  // bytes
  // A lane stages CPL chunks of 16 bytes (16-bit elements) per load, logical chunks CPL sc ...;
  // load i holds row RPL i + sr, whose swizzle key repeats every 16 / RPL loads for K
  // (row & 15) and every 8 / RPL (at least 1) loads for V (row & 7).
  constexpr int CPL = BFP8 ? 2 : 1;
  // swizzle keys of a tile row (period 16 rows for K, 8 for V)
  auto kkey = [](int row) { return D == 64 ? (row >> 1) & 7 : row & 15; };
  auto vkey = [](int row) {
    const int y = D == 64 ? (row >> 1) & 3 : row & 7;
    return (2 * y) | (y & 1);
  };
  constexpr int KPAT = RPL >= 16 ? 1 : 16 / RPL, VPAT = RPL >= 8 ? 1 : 8 / RPL;
  uint32_t kw[KPAT], vw[VPAT];
#pragma unroll
  for (int j = 0; j < KPAT; ++j)
    kw[j] = (uint32_t)(sr * ROWB + (((CPL * sc) ^ kkey(RPL * j + sr)) << 4));
#pragma unroll
  for (int j = 0; j < VPAT; ++j)
    vw[j] = (uint32_t)(sr * ROWB + (((CPL * sc) ^ vkey(RPL * j + sr)) << 4));
  // A-operand reads of K: row 16 b + n, chunk 4 s + quad
  uint32_t kr[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) kr[s] = (uint32_t)(n * ROWB + (((4 * s + quad) ^ kkey(n)) << 4));
  // transposing reads of V: lane addresses row 4 quad + n / 4 (+ 16 per key block), the 8 bytes
  // at element 16 db + 4 (n & 3)
  uint32_t vr[DBLK];
  {
    const int vrow = 4 * quad + (n >> 2), xx = (n & 3) >> 1;  // key blocks start at multiples of 16
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
      vr[db] = (uint32_t)(vrow * ROWB + (((2 * db + xx) ^ vkey(vrow)) << 4) + 8 * (n & 1));
  }

  auto locate = [&](int64_t xx) { return locate_unit<TILE>(a, s_pref, s_len, xx, seg_units); };
  // `bad`: bit i set where run i's block lies outside the table or the cache (it reads block 0)
  auto tile_offsets = [&](const Cursor &cu, int64_t (&eo)[NOFF], int64_t (&xo)[NOFF], uint32_t &bad) {
    bad = 0;
    bool base_bad = false;
    const int32_t *pt_row = page_table + (int64_t)cu.u * a.pt_rs;
    const int tok0 = cu.t * TILE;
    // a run never crosses a block (block_size is a multiple of the run length), so block and
    // row advance without a division; the table is read again only where the block changes
    int col = tok0 / a.bs, row = tok0 - col * a.bs;
    int64_t base = 0;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) {
      if (i == 0 || row == 0) {
        int phys = (col < a.w) ? __builtin_amdgcn_readfirstlane(pt_row[col]) : -1;
        base_bad = (unsigned)phys >= (unsigned)a.nb;
        if (base_bad) phys = 0;
        base = ((int64_t)phys * a.hkv + cu.h) * slab;
      }
      if (base_bad) bad |= 1u << i;
      eo[i] = base + (int64_t)row * D * BPE;
      xo[i] = base + (int64_t)a.bs * D + (int64_t)row * GPR;
      row += RPL * LPO;
      if (row >= a.bs) row = 0, ++col;
    }
  };
  auto fetch = [&](const uint8_t *base, const int64_t (&eo)[NOFF], const int64_t (&xo)[NOFF],
                   u32x4 (&raw)[NL], uint32_t (&ex)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint8_t *erow = base + eo[i / LPO] + (i % LPO) * (RPL * D * BPE);
      raw[i] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4 *>(erow + static_cast<uint64_t>(lane_bytes)));
      if constexpr (BFP8) {
        const uint8_t *xrow = base + xo[i / LPO] + (i % LPO) * (RPL * GPR);
        ex[i] = __builtin_nontemporal_load(
            reinterpret_cast<const uint32_t *>(xrow + static_cast<uint64_t>(lane_exp)));
      }
    }
  };
  // FUSED: the lane's part of the fresh K or V row of (user, head): the 16 bytes of its chunk
  // for a bfloat16 cache, the 16 bfloat16 elements of its group for block-float-8.
  constexpr int NF = BFP8 ? 2 : 1;
  struct Fresh {
    u32x4 part[NF];
  };
  auto fetch_fresh = [&](const uint16_t *src, const Cursor &cu) {
    const uint16_t *p = src + cu.u * a.new_us + cu.h * a.new_hs + (BFP8 ? 16 : 8) * sc;
    Fresh f;
#pragma unroll
    for (int j = 0; j < NF; ++j) f.part[j] = *reinterpret_cast<const u32x4 *>(p + 8 * j);
    return f;
  };
  // FUSED: puts the fresh row (quantised here for block-float-8) in place of row `r_star` of
  // the fetched tile (registers) and stores it into the cache row `row` of the slab at byte
  // offset `slab_base`.
  auto patch_and_store = [&](uint8_t *cache, u32x4 (&raw)[NL], uint32_t (&ex)[NL], const Fresh &fresh,
                             int r_star, int64_t elem_off, int64_t exp_off) {
    const int i_star = r_star / RPL;
    const bool mine = sr == r_star % RPL;
    u32x4 val = fresh.part[0];
    uint32_t e = 0;
    if constexpr (BFP8) {
      const u32x4 lo = fresh.part[0], hi = fresh.part[NF - 1];
      const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      uint32_t out[4];
      e = bfp8_encode16(w, out);
      val = u32x4{out[0], out[1], out[2], out[3]};
    }
#pragma unroll
    for (int i = 0; i < NL; ++i)
      if (i == i_star && mine) {
        raw[i] = val;
        if constexpr (BFP8) ex[i] = e << exp_shift;
      }
    if (mine) {
      *reinterpret_cast<u32x4 *>(cache + elem_off + 16 * sc) = val;
      if constexpr (BFP8) cache[exp_off + sc] = (uint8_t)e;
    }
  };
  // Cuts the lane's exponent bytes out of the fetched dwords (zero for rows past `nvalid` of a
  // partial tile, which stages them as zeros) and returns the largest of the tile.
  auto tile_exponent = [&](uint32_t (&ex)[NL], int nvalid, bool partial) {
    uint32_t e = 0;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      ex[i] = (ex[i] >> exp_shift) & 0xffu;
      if (partial && RPL * i + sr >= nvalid) ex[i] = 0;
      e = max(e, ex[i]);
    }
    return (int)wave_max_u32(e);
  };
  // registers -> LDS.  Block-float-8: expanded to half precision relative to the exponent
  // `eref`: the group scale 2^(e - eref) is the half with exponent field e - eref + 15; groups
  // more than 2^14 below the tile's largest (field <= 0) are written as zeros.  bfloat16:
  // copied; `clear` writes the rows past `nvalid` as zeros (unattended V rows must not carry
  // Inf / NaN into the product).
  auto stage = [&](bool is_v, const u32x4 (&raw)[NL], const uint32_t (&ex)[NL], int eref, int nvalid,
                   bool clear) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint32_t w0 = (is_v ? vw[i % VPAT] : kw[i % KPAT]) + (uint32_t)(i * RPL * ROWB);
      if constexpr (BFP8) {
        const uint32_t field = (uint32_t)max((int)ex[i] - (eref - 15), 0);
        const uint32_t sbits = field << 10;
        const halfx2 s2 = __builtin_bit_cast(halfx2, sbits | (sbits << 16));
        const halfx2 c2 = s2 * halfx2{(_Float16)-1152.f, (_Float16)-1152.f};
        uint32_t o[8];
        expand4_half(raw[i].x, s2, c2, o[0], o[1]);
        expand4_half(raw[i].y, s2, c2, o[2], o[3]);
        expand4_half(raw[i].z, s2, c2, o[4], o[5]);
        expand4_half(raw[i].w, s2, c2, o[6], o[7]);
        *reinterpret_cast<uint4 *>(tile + w0) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(tile + (w0 ^ 16u)) = make_uint4(o[4], o[5], o[6], o[7]);
      } else {
        const bool keep = !clear || RPL * i + sr < nvalid;
        *reinterpret_cast<uint4 *>(tile + w0) =
            keep ? make_uint4(raw[i].x, raw[i].y, raw[i].z, raw[i].w) : make_uint4(0, 0, 0, 0);
      }
    }
  };
  // Q fragments: B operand, lane%16 = head of the group (zero beyond G): as they are for a
  // bfloat16 cache; half precision, scaled by 2^(127 - eq) with eq the largest exponent field of
  // the segment's Q, for block-float-8.  (Requesting the next segment's Q rows early, ahead of
  // the tile loads and inside the branch that detects the segment change, was measured slower:
  // the wait-count pass then drains the tile loads in the steady-state loop.)
  int eq = 0;
  auto load_q = [&](const Cursor &cu, u32x4 (&qf)[KSTEPS]) {
    const uint16_t *qp =
        a.q + cu.u * a.q_us + (int64_t)(cu.h * G + min(n, G - 1)) * a.q_hs + 8 * quad;
    const uint32_t qmask = n < G ? 0xffffffffu : 0u;  // no branch: a branch would wait for every load in flight
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const uint4 t = *reinterpret_cast<const uint4 *>(qp + 32 * s);
      qf[s] = u32x4{t.x & qmask, t.y & qmask, t.z & qmask, t.w & qmask};
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

  Cursor cur = locate_unit<TILE>(a, s_pref, s_len, x_lo, seg_units, &x);
  int64_t eo[NOFF], xo[NOFF];
  u32x4 kraw[NL], vraw[NL];
  uint32_t kex[NL], vex[NL];
  u32x4 qf[KSTEPS];
  Fresh kfresh = {}, vfresh = {};
  uint32_t bad_cur = 0;  // the current tile's runs that read block 0 in place of a block out of range
  tile_offsets(cur, eo, xo, bad_cur);
  fetch(a.k, eo, xo, kraw, kex);
  fetch(a.v, eo, xo, vraw, vex);
  if constexpr (FUSED) {
    kfresh = fetch_fresh(a.k_new, cur);
    vfresh = fetch_fresh(a.v_new, cur);
  }
  load_q(cur, qf);
  publish_segment_row(a, s_pref, total, n_eff, seg_units);

  floatx4 acc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  int ev_run = 0;  // reference exponent of the V accumulator

  auto process_tile = [&](auto has_next_tag) {
    constexpr bool has_next = decltype(has_next_tag)::value;
    const int nvalid = cur.len - cur.t * TILE;
    const bool partial = nvalid < TILE;
    const int nbelow = cur.lo - cur.t * TILE;  // sliding window: > 0 only in a segment's first tile
    const bool same_seg = has_next && cur.tiles_left > 1;
    Cursor nxt = cur;

    // ---- K: registers -> LDS, then the next tile's K: global -> registers -------------------
    // FUSED: is this the tile that holds the token at cur_pos (the segment's last), and is that
    // position inside the table and its block inside the cache?  The row's place in the cache
    // comes from the tile's own offsets: a second look at the position and the page table would
    // be two round trips to memory in the middle of the tile, each waiting for every load in
    // flight, and the wavefronts that end a segment are the ones a launch ends up waiting for.
    bool fresh_ok = false;
    int64_t fresh_eo = 0, fresh_xo = 0;
    if constexpr (FUSED) {
      if (cur.tiles_left == 1 && nvalid > 0) {
        // a length below the table's capacity is the position + 1; at the capacity it may have
        // been cut short, and only then the position is read again
        const int64_t cap = (int64_t)a.w * a.bs;
        const bool exact = cur.len < cap || load_index(cur_pos, a.cur_i64, cur.u) == cur.len - 1;
        constexpr int RUN_ROWS = RPL * LPO;
        const int i_run = (nvalid - 1) / RUN_ROWS, rr = (nvalid - 1) % RUN_ROWS;
        if (exact && !((bad_cur >> i_run) & 1u)) {
          fresh_ok = true;
#pragma unroll
          for (int i = 0; i < NOFF; ++i)
            if (i == i_run) fresh_eo = eo[i] + (int64_t)rr * D * BPE, fresh_xo = xo[i] + (int64_t)rr * GPR;
        }
      }
      if (fresh_ok) patch_and_store(const_cast<uint8_t *>(a.k), kraw, kex, kfresh, nvalid - 1, fresh_eo, fresh_xo);
    }
    int eref_k = 0, eref_v = 0;
    if constexpr (BFP8) eref_k = tile_exponent(kex, nvalid, partial);
    stage(false, kraw, kex, eref_k, nvalid, false);
    if constexpr (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate(x + 1);
      }
      tile_offsets(nxt, eo, xo, bad_cur);  // (of the next tile: this one's has been used above)
      fetch(a.k, eo, xo, kraw, kex);
    }

    // ---- S^T = K . Q^T ------------------------------------------------------------------------
    floatx4 st[KBLK];
#pragma unroll
    for (int b = 0; b < KBLK; ++b) {
      st[b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const uint4 kq = *reinterpret_cast<const uint4 *>(tile + kr[s] + b * (16 * ROWB));
        st[b] = mma16<BFP8>(u32x4{kq.x, kq.y, kq.z, kq.w}, qf[s], st[b]);
      }
    }
    // ---- online softmax: lane (head, quad) holds keys 16 b + 4 quad + r ------------------------
    if (partial || nbelow > 0) {
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = 16 * b + 4 * quad + r;
          if (key >= nvalid || key < nbelow) st[b][r] = -INFINITY;
        }
    }
    // the factors taken out of the K tile and out of Q come back in the scale
    const float scale = BFP8 ? __builtin_ldexpf(a.scale_log2e, eref_k + eq - 260) : a.scale_log2e;
    if constexpr (MASKED) {  // the mask, brought to the units of the raw scores
      const float unit = 1.4426950408889634f / scale;
      const uint16_t *mrow = a.mask + cur.u * a.mask_us + (int64_t)(cur.h * G + min(n, G - 1)) * a.mask_hs +
                             cur.t * TILE + 4 * quad;
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (16 * b + 4 * quad + r < nvalid) st[b][r] += bf16_lo(mrow[16 * b + r]) * unit;
    }
    float mloc = -INFINITY;
    if (scale >= 0.f) {
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) mloc = fmaxf(mloc, st[b][r]);
      mloc *= scale;
    } else {  // a negative scale turns the maximum into a minimum: compare scaled scores
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) mloc = fmaxf(mloc, st[b][r] * scale);
    }
    mloc = max_over_quads(mloc);
    const float m_new = fmaxf(m_run, mloc);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    m_run = m_new;

    // ---- V: registers -> LDS (the K tile has been consumed), next tile's V -> registers -------
    if constexpr (FUSED) {
      if (fresh_ok) patch_and_store(const_cast<uint8_t *>(a.v), vraw, vex, vfresh, nvalid - 1, fresh_eo, fresh_xo);
    }
    if constexpr (BFP8) eref_v = tile_exponent(vex, nvalid, partial);
    stage(true, vraw, vex, eref_v, nvalid, partial);
    if constexpr (has_next) fetch(a.v, eo, xo, vraw, vex);

    float lsum = 0.f, alpha_acc = alpha;
    u32x4 pf[PSTEPS];
    if constexpr (BFP8) {
      // bring this tile's V factor and the accumulator to the larger reference exponent
      const int ev_new = max(ev_run, eref_v);
      const float pscale = __builtin_ldexpf(1.f, eref_v - ev_new);
      alpha_acc = alpha * __builtin_ldexpf(1.f, ev_run - ev_new);
      ev_run = ev_new;
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(st[b][r], scale, -m_safe));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(st[b][r + 1], scale, -m_safe));
          lsum += p0 + p1;  // half-precision rounding of the weights is 2^-12: not tracked
          pf[b >> 1][2 * (b & 1) + (r >> 1)] = pack_half2(p0 * pscale, p1 * pscale);
        }
    } else {
#pragma unroll
      for (int b = 0; b < KBLK; ++b)
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(st[b][r], scale, -m_safe));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(st[b][r + 1], scale, -m_safe));
          const floatx2 pp = {p0, p1};
          const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(pp, bf16x2));
          lsum += bf16_lo(w) + bf16_hi(w);  // the normaliser sums the weights that multiply V
          pf[b >> 1][2 * (b & 1) + (r >> 1)] = w;
        }
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha_acc != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < DBLK; ++i) acc[i] *= alpha_acc;
    }
    // ---- O^T += V^T . P^T ------------------------------------------------------------------------
#pragma unroll
    for (int s = 0; s < PSTEPS; ++s)
#pragma unroll
      for (int db = 0; db < DBLK; ++db) {
        typedef __attribute__((address_space(3))) shortx4 *lds_v4;
        const uint8_t *vp = tile + vr[db] + s * (32 * ROWB);
        shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vp));
        shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vp + 16 * ROWB));
        const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
        acc[db] = mma16<BFP8>(u32x4{l2.x, l2.y, h2.x, h2.y}, pf[s], acc[db]);
      }

    // ---- close the segment --------------------------------------------------------------------
    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wave + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
      const float l_tot = sum_over_quads(l_run);
      const float vout = BFP8 ? __builtin_ldexpf(1.f, ev_run - 133) : 1.f;
      if (n < G) {
        float *dst = slot + n * D + 4 * quad;
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
          *reinterpret_cast<float4 *>(dst + 16 * db) = make_float4(
              acc[db][0] * vout, acc[db][1] * vout, acc[db][2] * vout, acc[db][3] * vout);
        if (quad == 0) {
          slot[G * D + n] = m_run;
          slot[G * D + G + n] = l_tot;
        }
      }
#pragma unroll
      for (int i = 0; i < DBLK; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
      m_run = -INFINITY;
      l_run = 0.f;
      ev_run = 0;
      if constexpr (has_next) {
        load_q(nxt, qf);
        if constexpr (FUSED) {  // the fresh rows of the new segment, once per segment
          kfresh = fetch_fresh(a.k_new, nxt);
          vfresh = fetch_fresh(a.v_new, nxt);
        }
      }
    }
    cur = nxt;
    x += same_seg ? 1 : 1 + seg_units;
  };
  // the unit of the tile behind the current one: the next, or behind the next segment's leading units
  auto next_tile_unit = [&]() { return x + (cur.tiles_left > 1 ? 1 : 1 + seg_units); };
  while (next_tile_unit() < x_hi) process_tile(std::true_type{});
  process_tile(std::false_type{});
}

template <int D, bool BFP8, int RUNS, bool FUSED, bool MASKED = false>
bool launch(const DecodeArgs &a, hipStream_t st) {
  const int blocks = a.n_waves / kWavesPerBlock;
  const size_t lds = (size_t)kWavesPerBlock * tile_bytes<D, BFP8>();
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_mfma16_kernel<D, BFP8, RUNS, FUSED, MASKED>), lds,
                          lds_ready))
    return false;
  launch_dominant(&paged_decode_mfma16_kernel<D, BFP8, RUNS, FUSED, MASKED>, dim3(blocks), dim3(256), lds, st, a, a.pt, a.cur);
  return true;
}

// Picks the variant for the block size and for a.k_new (set: the launch also performs the
// cache update of the step).
template <int D, bool BFP8>
bool launch_for_block_size(const DecodeArgs &a, hipStream_t st) {
  constexpr int TILE = tile_bytes<D, BFP8>() / (2 * D);
  const bool fused = a.k_new != nullptr;
  if (a.mask != nullptr) return !fused && launch<D, BFP8, 0, false, true>(a, st);
  if (a.bs % TILE == 0) return fused ? launch<D, BFP8, 1, true>(a, st) : launch<D, BFP8, 1, false>(a, st);
  if (a.bs % (TILE / 2) == 0) return fused ? launch<D, BFP8, 2, true>(a, st) : launch<D, BFP8, 2, false>(a, st);
  if (a.bs % (TILE / 4) == 0) return fused ? launch<D, BFP8, 4, true>(a, st) : launch<D, BFP8, 4, false>(a, st);
  return fused ? launch<D, BFP8, 0, true>(a, st) : launch<D, BFP8, 0, false>(a, st);
}

}  // namespace
}  // namespace decode
}  // namespace ttpa
