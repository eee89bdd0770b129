// Paged decode attention for wide, latent-style heads (multi-head latent attention), gfx950.
//
// Shape: few KV heads of DQK features (e.g. one latent head of 576 = 512 + 64 rope
// features), many query heads per KV head, and a value width DV that differs from DQK: V is
// either a separate paged cache or the leading DV features of K itself.
//
// Same split-K scheme as the other decode kernels (flat list of 64-token tiles ordered
// (user, segment, tile), cut into equal ranges, partials merged by decode_combine_kernel),
// with two differences:
//   * a range belongs to a WORKGROUP: its four wavefronts share each K tile in LDS (a 64 x 576
//     tile is 72 KiB; two stages fill the LDS of a CU), and a "segment" is one block of up to
//     32 query heads of one KV head, so a group of 128 heads is four segments per KV head;
//   * every wavefront computes the whole score tile S^T = K Q^T for the segment's heads
//     (redundantly: it costs matrix time, not memory traffic) and then the output columns
//     of its own DVW-wide slice of V, O^T[slice] += V[slice]^T P^T.
// Tiles travel global -> LDS with global_load_lds_dwordx4, one row (or 1 KiB piece of a row)
// per instruction, so LDS rows can carry 16 bytes of padding.
#include "decode_common.h"

#include <cstdlib>
#include <utility>

namespace ttpa {
namespace decode {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxUsersWide = 1024;

struct WideArgs {
  int nkv;         // KV heads of the caches (DecodeArgs::hkv counts segments per user)
  int nhb;         // head blocks (segments) per KV head
  int gseg;        // query heads per segment (<= 32)
  int dv;          // value width
  int n_slices;    // dv / DVW wavefronts take part in the second product
};

template <int DQK, int DVW, bool SHARED_V>
struct WideLds {
  static constexpr int KROW = 2 * DQK + 16;                 // bytes per K row in LDS
  static constexpr int KTILE = kTile * KROW;
  static constexpr int VROW_MAX = 2 * 2 * DVW + 16;         // separate V tile: up to 2 slices
  static constexpr int VTILE = SHARED_V ? 0 : kTile * VROW_MAX;
  static constexpr int STAGE = KTILE + VTILE;
};

template <int DQK, int DVW, bool SHARED_V>
__global__ __launch_bounds__(256, 1) void paged_decode_wide_kernel(
    DecodeArgs a, WideArgs w, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  constexpr int KSTEPS = DQK / 16, DBLK = DVW / 32;
  using L = WideLds<DQK, DVW, SHARED_V>;
  constexpr int ROW_BYTES = 2 * DQK;
  constexpr int ROW_FULL = ROW_BYTES / 1024;          // whole 1 KiB pieces of a K row
  constexpr int ROW_REM_LANES = (ROW_BYTES % 1024) / 16;

  __shared__ int s_pref[kMaxUsersWide + 1];
  __shared__ int s_len[kMaxUsersWide];
  __shared__ int s_wsum[kWavesPerBlock];
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  build_prefix(a, cur_pos, s_pref, s_len, s_wsum);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int wg = blockIdx.x;
  const int total_tiles = __builtin_amdgcn_readfirstlane(s_pref[a.users]);
  const int64_t total = (int64_t)total_tiles * a.hkv;
  const int n_eff = (int)(total < a.n_waves ? total : a.n_waves);  // workgroups that get work
  if (total == 0 || wg >= n_eff) {
    publish_segment_row(a, s_pref, total, n_eff);
    return;
  }
  int64_t x = (int64_t)wg * total / n_eff;
  const int64_t x_hi = (int64_t)(wg + 1) * total / n_eff;
  const int G = w.gseg;
  const int v_row_bytes = 2 * w.dv;                    // separate V cache: bytes per token row
  const int v_lds_row = v_row_bytes + 16;
  const bool pv_wave = wave < w.n_slices;              // this wavefront owns a V slice

  auto locate = [&](int64_t xx) { return locate_unit(a, s_pref, s_len, xx); };

  // ---- tile load: each wavefront moves 16 of the tile's 64 rows, one row per instruction ----
  const uint16_t *kc = reinterpret_cast<const uint16_t *>(a.k);
  const uint16_t *vc = reinterpret_cast<const uint16_t *>(a.v);
  auto issue_tile = [&](const Cursor &cu, int buf) {
    const int32_t *pt_row = page_table + (int64_t)cu.u * a.pt_rs;
    const int kvh = cu.h / w.nhb;
    const int tok0 = cu.t * kTile;
    const uint32_t stage = lds_address(smem) + (uint32_t)(buf * L::STAGE);  // absolute LDS address
    for (int i = 0; i < 16; ++i) {
      const int r = 16 * wave + i;
      const int tk = tok0 + r;
      const int col = tk / a.bs;
      int phys = (col < a.w) ? pt_row[col] : 0;
      if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
      const int64_t row = ((int64_t)phys * w.nkv + kvh) * a.bs + (tk - col * a.bs);
      const char *src = reinterpret_cast<const char *>(kc + row * DQK);
      const uint32_t dst = stage + (uint32_t)(r * L::KROW);
#pragma unroll
      for (int j = 0; j < ROW_FULL; ++j) dma16_uniform(src + 1024 * j, 16u * lane, dst + 1024u * j);
      if constexpr (ROW_REM_LANES > 0) {
        if (lane < ROW_REM_LANES) dma16_uniform(src + 1024 * ROW_FULL, 16u * lane, dst + 1024u * ROW_FULL);
      }
      if constexpr (!SHARED_V) {
        const char *vsrc = reinterpret_cast<const char *>(vc + row * w.dv);
        const uint32_t vdst = stage + (uint32_t)(L::KTILE + r * v_lds_row);
        if (16 * lane < v_row_bytes) dma16_uniform(vsrc, 16u * lane, vdst);  // dv <= 512: one piece
      }
    }
  };
  // Rows past the attended length may be cache rows nobody ever wrote: their scores are
  // masked, but as V rows they would turn 0 * Inf into NaN, so they are cleared in LDS.
  auto clear_unattended_rows = [&](int buf, int nvalid) {
    unsigned char *stage = smem + buf * L::STAGE;
    for (int r = nvalid + wave; r < kTile; r += kWavesPerBlock) {
      uint4 *krow = reinterpret_cast<uint4 *>(stage + r * L::KROW);
      for (int c = lane; c < ROW_BYTES / 16; c += 64) krow[c] = make_uint4(0, 0, 0, 0);
      if constexpr (!SHARED_V) {
        uint4 *vrow = reinterpret_cast<uint4 *>(stage + L::KTILE + r * v_lds_row);
        for (int c = lane; c < v_row_bytes / 16; c += 64) vrow[c] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto load_q = [&](const Cursor &cu, bf16x8 (&qf)[KSTEPS]) {
    const uint16_t *qp = a.q + cu.u * a.q_us + (int64_t)(cu.h * G + min(n, G - 1)) * a.q_hs + 8 * h;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      uint4 t = *reinterpret_cast<const uint4 *>(qp + 16 * s);
      if (n >= G) t = make_uint4(0, 0, 0, 0);
      qf[s] = __builtin_bit_cast(bf16x8, t);
    }
  };

  Cursor cur = locate(x);
  bf16x8 qf[KSTEPS];
  issue_tile(cur, 0);
  load_q(cur, qf);
  publish_segment_row(a, s_pref, total, n_eff);

  floatx16 acc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const int grp = lane >> 4, a16 = lane & 15;

  for (int it = 0; x < x_hi; ++x, ++it) {
    const int buf = it & 1;
    const unsigned char *stage = smem + buf * L::STAGE;
    const int nvalid = cur.len - cur.t * kTile;
    const bool partial = nvalid < kTile;
    const int nbelow = cur.lo - cur.t * kTile;  // sliding window: > 0 only in a segment's first tile
    const bool has_next = x + 1 < x_hi;
    const bool same_seg = has_next && cur.tiles_left > 1;

    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's rows of the tile have landed
    __syncthreads();                     // the tile is complete; everybody has left the other stage
    Cursor nxt = cur;
    if (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate(x + 1);
      }
      issue_tile(nxt, buf ^ 1);
    }
    if (partial) {
      clear_unattended_rows(buf, nvalid);
      __syncthreads();
    }

    // ---- S^T = K . Q^T ----------------------------------------------------------------------
    floatx16 st[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) st[0][r] = 0.f, st[1][r] = 0.f;
    {
      const unsigned char *krow = stage + n * L::KROW + 16 * h;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          bf16x8 kf = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4 *>(krow + 32 * kb * L::KROW + 32 * s));
          st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], st[kb], 0, 0, 0);
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
    if (a.mask != nullptr) {  // additive mask, brought to the units of the raw scores
      const float unit = 1.4426950408889634f / a.scale_log2e;
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
    const float scale = a.scale_log2e;
    float mloc = -INFINITY;  // the maximum is tracked on scaled scores (the scale may be negative)
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, st[kb][r] * scale);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    const float m_new = fmaxf(m_run, mloc);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    m_run = m_new;
    float lsum = 0.f;
    bf16x8 pf[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float p = __builtin_amdgcn_exp2f(fmaf(st[kb][8 * s + e], scale, -m_safe));
          __bf16 pb = (__bf16)p;
          lsum += (float)pb;  // the normaliser sums the weights that multiply V
          pf[kb][s][e] = pb;
        }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= alpha;
    }
    // ---- O^T[slice] += V[slice]^T . P^T (V^T fragments through the transposing LDS load: per
    //      group of 16 lanes, lane i receives element i % 4 of the 8-byte chunks addressed by
    //      lanes 4 j + i / 4) ---------------------------------------------------------------------
    if (pv_wave) {
      const int vstride = SHARED_V ? L::KROW : v_lds_row;
      const unsigned char *vbase = stage + (SHARED_V ? 0 : L::KTILE) +
                                   (4 * (grp >> 1) + (a16 >> 2)) * vstride +
                                   2 * (wave * DVW + 16 * (grp & 1) + 4 * (a16 & 3));
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const unsigned char *vk = vbase + (32 * kb + 16 * s) * vstride;
#pragma unroll
          for (int db = 0; db < DBLK; ++db) {
            typedef __attribute__((address_space(3))) shortx4 *lds_v4;
            shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 64 * db));
            shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 8 * vstride + 64 * db));
            bf16x8 vf;
            bf16x4 l4 = __builtin_bit_cast(bf16x4, lo), h4 = __builtin_bit_cast(bf16x4, hi);
            vf[0] = l4[0], vf[1] = l4[1], vf[2] = l4[2], vf[3] = l4[3];
            vf[4] = h4[0], vf[5] = h4[1], vf[6] = h4[2], vf[7] = h4[3];
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kb][s], acc[db], 0, 0, 0);
          }
        }
    }

    // ---- close the segment: every wavefront writes its slice of the partial ---------------------
    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wg + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
      const float l_tot = l_run + __shfl_xor(l_run, 32);
      if (n < G) {
        if (pv_wave) {
          float *dst = slot + n * w.dv + wave * DVW + 4 * h;
#pragma unroll
          for (int db = 0; db < DBLK; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j)
              *reinterpret_cast<float4 *>(dst + 32 * db + 8 * j) = make_float4(
                  acc[db][4 * j], acc[db][4 * j + 1], acc[db][4 * j + 2], acc[db][4 * j + 3]);
        }
        if (wave == 0 && h == 0) {
          slot[G * w.dv + n] = m_run;
          slot[G * w.dv + G + n] = l_tot;
        }
      }
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
      m_run = -INFINITY;
      l_run = 0.f;
      if (has_next) load_q(nxt, qf);
    }
    cur = nxt;
  }
}


// ---------------------------------------------------------------------------------------------
// Up to 16 query heads per KV head with V taken from K: the latent serving shape (16 heads of
// 576 = 512 + 64 features on a rank, V = the 512 leading ones).  Here nothing is shared between
// wavefronts, and nothing is computed twice: every wavefront streams its own range of 16-token
// tiles, as in the 16x16x32 kernel of the plain decode shapes, with the group's heads as the
// 16-wide N dimension:
//   S^T[key, head]   = K[key, :] . Q[head, :]     v_mfma_f32_16x16x32_bf16, DQK / 32 steps
//   O^T[d, head]    += V^T[d, key] . P^T[key, head]   v_mfma_f32_16x16x16_bf16 per 16 values
// The C layout of the first (lane (head, quad) holds keys 4 quad + r) is the B layout of the
// second.  A tile is 16 consecutive cache rows (block_size is a multiple of 16), so it goes
// global -> LDS as whole 1 KiB LDS-DMA instructions (18 for rows of 1152 bytes; an instruction
// holds the wavefront until the address unit has taken it, and one per row plus one per row tail
// was 32), into one of two wave-private stages; the wavefront waits for its own loads only, there
// is no barrier.  Rows are unpadded in LDS; bank conflicts are avoided by an XOR swizzle of the
// 16-byte chunk position, applied on the global side (which chunk a lane fetches: every lane of
// an LDS-DMA instruction supplies its own source address) and when fragments are read.  Rows of
// 1152 or 384 bytes start 32 banks apart, so chunk ^ ((row >> 1) & 7) inside aligned groups of 8
// chunks gives the sixteen rows of an A-operand read sixteen different bank quads; rows of 256
// bytes start at the same bank and take chunk ^ (row & 15).  The arithmetic of a tile is an
// order of magnitude below what its bytes cost in HBM time, so nothing here is scheduled by hand.
template <int DQK, int DV>
struct Latent16 {
  static constexpr int TILE = 16;
  static constexpr int ROW = 2 * DQK;            // bytes per row, in the cache and in LDS
  static constexpr int CPR = ROW / 16;           // 16-byte chunks per row
  static constexpr int STAGE = TILE * ROW;
  static constexpr int WAVE_LDS = 2 * STAGE;
  static constexpr int NDMA = STAGE / 1024;      // LDS-DMA instructions per tile
  static constexpr bool HALF_PERIOD = (ROW / 4) % 64 == 32;
  static_assert(STAGE % 1024 == 0 && (HALF_PERIOD ? CPR % 8 == 0 : ((ROW / 4) % 64 == 0 && CPR % 16 == 0)),
                "row length the swizzle is not made for");
  // position of chunk c of row r inside the row: c ^ swizzle(r).  Two kinds of reads must find their
  // lanes in different banks (64 banks of 4 bytes), and the LDS of this part serves them in these
  // lane groups (measured with SQ_LDS_BANK_CONFLICT on pairs of active lanes): a 16-byte read in four
  // groups of 16 lanes, {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same plus 32; an 8-byte
  // (transposing) read in two groups of 32 lanes.  The A operand of the score product reads row n,
  // chunk 4 i + quad; the transposing read of the value columns reads rows 4 quad .. 4 quad + 3, an
  // aligned pair of chunks each.  Rows of 1152 or 384 bytes start 32 banks apart, rows of 256 bytes in
  // the same bank; the two swizzles below leave both reads without a conflict (the plain
  // (r >> 1) & 7 and r & 15 gave every transposing read a two-way conflict: twice its LDS time).
  __device__ static constexpr int swizzle(int r) {
    const int m = (r >> 1) & 7;
    return HALF_PERIOD ? ((((m & 3) << 1) | (m >> 2)) ^ ((m >> 2) << 2)) : ((((r & 7) ^ ((r >> 3) << 2)) << 1) | ((r >> 3) & 1));
  }
  __device__ static constexpr int position(int r, int c) { return c ^ swizzle(r & 15); }
};

template <int DQK, int DV>
__global__ __launch_bounds__(256, 1) void paged_decode_latent16_kernel(
    DecodeArgs a, WideArgs w, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  using L = Latent16<DQK, DV>;
  typedef float floatx4 __attribute__((ext_vector_type(4)));
  constexpr int TILE = L::TILE, KSTEPS = DQK / 32, VB = DV / 16;
  constexpr int ROW_BYTES = L::ROW;

  __shared__ int s_pref[kMaxUsersWide + 1];
  __shared__ int s_len[kMaxUsersWide];
  __shared__ int s_wsum[kWavesPerBlock];
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int seg_units = a.seg_units;
  build_prefix<TILE>(a, cur_pos, s_pref, s_len, s_wsum, seg_units);

  const int lane = threadIdx.x & 63;
  const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, quad = lane >> 4;
  // LDS-DMA instruction k fills chunk positions 64 k .. 64 k + 63 of the stage; this lane's is
  // position p of row r, which holds chunk position(r, p): the source offset inside the tile
  uint32_t src_off[L::NDMA];
#pragma unroll
  for (int k = 0; k < L::NDMA; ++k) {
    const int P = 64 * k + lane, r = P / L::CPR, p = P % L::CPR;
    src_off[k] = (uint32_t)(r * ROW_BYTES + 16 * L::position(r, p));
  }
  // Fragment addresses inside a stage: A operand of the score product (row n, chunk 4 s + quad)
  // and the transposing read of the value columns (row 4 quad + n / 4, values 16 vb + 4 (n % 4) ..).
  // The swizzle only touches the chunk index inside its aligned group of GC chunks, so a lane
  // needs one address per chunk offset inside a group; the group itself is an immediate offset.
  constexpr int GC = L::HALF_PERIOD ? 8 : 16;
  constexpr int KB = GC / 4, VBASES = GC / 2;
  uint32_t kbase[KB], vbase[VBASES];
#pragma unroll
  for (int i = 0; i < KB; ++i) kbase[i] = (uint32_t)(n * ROW_BYTES + 16 * L::position(n, 4 * i + quad));
  {
    const int rv = 4 * quad + (n >> 2), q = n & 3;
#pragma unroll
    for (int i = 0; i < VBASES; ++i)
      vbase[i] = (uint32_t)(rv * ROW_BYTES + 16 * L::position(rv, 2 * i + (q >> 1)) + 8 * (q & 1));
  }
  auto read_k = [&](const unsigned char *stage, int s) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(stage + kbase[s % KB] + 16 * GC * (s / KB)));
  };
  auto read_v = [&](const unsigned char *stage, int vb) {
    typedef __attribute__((address_space(3))) shortx4 *lds_v4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(stage + vbase[vb % VBASES] + 16 * GC * (vb / VBASES)));
  };
  constexpr int KPRE = KSTEPS < 8 ? KSTEPS : 8;  // fragments in flight (an LDS read takes a few hundred cycles)
  constexpr int VPRE = VB < 12 ? VB : 12;
  const int wave = blockIdx.x * kWavesPerBlock + wib;
  // The flat list in units: per segment `seg_units` units that stand for the cost of opening it,
  // then its tiles.  A range of more than seg_units units holds at least one tile.
  const int total_units = __builtin_amdgcn_readfirstlane(s_pref[a.users]);
  const int64_t total = (int64_t)total_units * a.hkv;
  const int64_t max_ranges = total / (seg_units + 1);
  const int n_eff = (int)(max_ranges < a.n_waves ? max_ranges : a.n_waves);
  if (total == 0 || wave >= n_eff) {
    publish_segment_row(a, s_pref, total, n_eff, seg_units);
    return;
  }
  const int64_t x_lo = (int64_t)wave * total / n_eff;
  const int64_t x_hi = (int64_t)(wave + 1) * total / n_eff;
  int64_t x = x_lo;  // set below to the unit of the first tile at or behind x_lo
  const int G = w.gseg;
  unsigned char *my_lds = smem + wib * L::WAVE_LDS;

  // ---- tile load: block_size is a multiple of the tile, so a tile is 16 consecutive cache rows ----
  // (the table entry of a block is read once, with the first of the block's tiles: the read is a
  // trip to the L2 in front of the tile's loads)
  int seen_user = -1, seen_col = -1, seen_phys = 0;
  auto issue_tile = [&](const Cursor &cu, int buf) {
    const int tok0 = cu.t * TILE;
    const int col = tok0 / a.bs;
    if (cu.u != seen_user || col != seen_col) {
      int p = (col < a.w) ? page_table[(int64_t)cu.u * a.pt_rs + col] : 0;
      if ((unsigned)p >= (unsigned)a.nb) p = 0;
      seen_user = cu.u, seen_col = col, seen_phys = p;
    }
    const int phys = seen_phys;
    const int64_t row0 = ((int64_t)phys * w.nkv + cu.h) * a.bs + (tok0 - col * a.bs);
    const uint64_t addr = reinterpret_cast<uint64_t>(a.k) + (uint64_t)row0 * ROW_BYTES;
    const char *src = reinterpret_cast<const char *>(address_from_words(
        __builtin_amdgcn_readfirstlane((int)(uint32_t)addr), __builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32))));
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_address(my_lds) + (uint32_t)(buf * L::STAGE)));
    const void *bases[4] = {src, src - 1024, src - 2048, src - 3072};
#pragma unroll
    for (int k = 0; k + 4 <= L::NDMA; k += 4) {
      const uint32_t off[4] = {src_off[k], src_off[k + 1], src_off[k + 2], src_off[k + 3]};
      dma16_streaming_quad(bases, off, dst + 1024u * k);
    }
#pragma unroll
    for (int k = L::NDMA / 4 * 4; k < L::NDMA; ++k) dma16_streaming(src, src_off[k], dst + 1024u * k);
  };
  // Rows past the attended length may be cache rows nobody ever wrote: their scores are masked,
  // but as V rows they would turn 0 * Inf into NaN, so they are cleared in LDS.
  auto clear_unattended_rows = [&](unsigned char *stage, int nvalid) {
    for (int r = nvalid; r < TILE; ++r) {
      uint4 *row = reinterpret_cast<uint4 *>(stage + r * L::ROW);
      for (int c = lane; c < ROW_BYTES / 16; c += 64) row[c] = make_uint4(0, 0, 0, 0);
    }
  };
  // B operand of the score product: lane (head, quad) holds features 32 s + 8 quad .. + 7
  auto load_q = [&](const Cursor &cu, bf16x8 (&qf)[KSTEPS]) {
    const uint16_t *qp = a.q + cu.u * a.q_us + (int64_t)(cu.h * G + min(n, G - 1)) * a.q_hs + 8 * quad;
    const uint32_t qmask = n < G ? 0xffffffffu : 0u;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      uint4 t = *reinterpret_cast<const uint4 *>(qp + 32 * s);
      t.x &= qmask, t.y &= qmask, t.z &= qmask, t.w &= qmask;
      qf[s] = __builtin_bit_cast(bf16x8, t);
    }
  };

  Cursor cur = locate_unit<TILE>(a, s_pref, s_len, x_lo, seg_units, &x);
  bf16x8 qf[KSTEPS];
  issue_tile(cur, 0);
  load_q(cur, qf);
  publish_segment_row(a, s_pref, total, n_eff, seg_units);

  floatx4 acc[VB];
#pragma unroll
  for (int i = 0; i < VB; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  for (int it = 0; x < x_hi; ++it) {
    const int buf = it & 1;
    unsigned char *stage = my_lds + buf * L::STAGE;
    const int nvalid = cur.len - cur.t * TILE;
    const bool partial = nvalid < TILE;
    const int nbelow = cur.lo - cur.t * TILE;
    // the unit of the tile behind this one: the next, or behind the next segment's leading units
    const int64_t x_next = x + (cur.tiles_left > 1 ? 1 : 1 + seg_units);
    const bool has_next = x_next < x_hi;
    const bool same_seg = has_next && cur.tiles_left > 1;

    // The next tile is requested BEFORE this one is waited for (its stage has been idle since the
    // previous iteration), so two tiles are in flight while the wavefront waits: with one, a
    // tile took the memory latency plus its own issue and arithmetic, 3.9 us for 18 KiB.  Vector
    // loads return in order: all but the NDMA newest done means this tile, and the Q rows
    // requested before it, have landed.
    Cursor nxt = cur;
    if (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate_unit<TILE>(a, s_pref, s_len, x + 1, seg_units);
      }
      issue_tile(nxt, buf ^ 1);
      __builtin_amdgcn_s_waitcnt((L::NDMA & 15) | 0x0F70 | ((L::NDMA >> 4) << 14));  // vmcnt(NDMA)
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    }
    if (partial) clear_unattended_rows(stage, max(nvalid, 0));

    // ---- S^T = K . Q^T ----------------------------------------------------------------------
    floatx4 st = {0.f, 0.f, 0.f, 0.f};
    {
      bf16x8 ring[KPRE];
#pragma unroll
      for (int s = 0; s < KPRE; ++s) ring[s] = read_k(stage, s);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[s % KPRE], qf[s], st, 0, 0, 0);
        if (s + KPRE < KSTEPS) ring[s % KPRE] = read_k(stage, s + KPRE);
      }
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {  // pin the order: one fragment read behind every matrix instruction
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (s + KPRE < KSTEPS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    // ---- online softmax: lane (head, quad) holds keys 4 quad + r --------------------------------
    const float scale = a.scale_log2e;
    float sc[4], mloc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = 4 * quad + r;
      sc[r] = (key >= nvalid || key < nbelow) ? -INFINITY : st[r] * scale;
      mloc = fmaxf(mloc, sc[r]);
    }
    mloc = max_over_quads(mloc);
    // the running maximum moves only when a head's maximum grows by more than 2^8: rescaling the
    // 4 VB accumulator registers costs more than the rest of the tile
    const bool move = !(mloc - m_run <= 8.0f);  // also true from -inf
    const float m_new = move ? mloc : m_run;
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = move ? __builtin_amdgcn_exp2f(m_run - m_safe) : 1.0f;
    m_run = m_new;
    float lsum = 0.f;
    shortx4 pf;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = __builtin_amdgcn_exp2f(sc[r] - m_safe);
      const __bf16 pb = (__bf16)p;
      lsum += (float)pb;  // the normaliser sums the weights that multiply V
      pf[r] = __builtin_bit_cast(short, pb);
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < VB; ++i) acc[i] *= alpha;
    }
    // ---- O^T += V^T . P^T: lane (i, quad) of the transposing load addresses row 4 quad + i / 4,
    //      values 16 vb + 4 (i % 4) .. + 3, and receives value 16 vb + i of rows 4 quad .. + 3 ------
    {
      shortx4 vring[VPRE];
#pragma unroll
      for (int vb = 0; vb < VPRE; ++vb) vring[vb] = read_v(stage, vb);
#pragma unroll
      for (int vb = 0; vb < VB; ++vb) {
        acc[vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vring[vb % VPRE], pf, acc[vb], 0, 0, 0);
        if (vb + VPRE < VB) vring[vb % VPRE] = read_v(stage, vb + VPRE);
      }
#pragma unroll
      for (int vb = 0; vb < VB; ++vb) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (vb + VPRE < VB) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    // ---- close the segment ------------------------------------------------------------------------
    if (!same_seg) {
      float *slot = a.ws_slots + ((int64_t)wave + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
      const float l_tot = sum_over_quads(l_run);
      if (n < G) {
        if (a.partial_bf16) {  // wavefront-uniform
          // in blocks of 16 heads x 16 columns (decode_combine_bf16_kernel; here one block of
          // heads): the 64 lanes of a store write 512 consecutive bytes
          uint32_t *dst = reinterpret_cast<uint32_t *>(slot) + 8 * n + 2 * quad;
#pragma unroll
          for (int vb = 0; vb < VB; ++vb)
            *reinterpret_cast<uint2 *>(dst + 128 * vb) =
                make_uint2(pack_bf16x2(acc[vb][0], acc[vb][1]), pack_bf16x2(acc[vb][2], acc[vb][3]));
          if (quad == 0) {
            slot[16 * DV / 2 + n] = m_run;
            slot[16 * DV / 2 + G + n] = l_tot;
          }
        } else {
          float *dst = slot + n * DV + 4 * quad;
#pragma unroll
          for (int vb = 0; vb < VB; ++vb)
            *reinterpret_cast<float4 *>(dst + 16 * vb) = make_float4(acc[vb][0], acc[vb][1], acc[vb][2], acc[vb][3]);
          if (quad == 0) {
            slot[G * DV + n] = m_run;
            slot[G * DV + G + n] = l_tot;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < VB; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
      m_run = -INFINITY;
      l_run = 0.f;
      if (has_next) load_q(nxt, qf);
    }
    cur = nxt;
    x = x_next;
  }
}

template <int DQK, int DV>
bool launch_latent16(const DecodeArgs &a, const WideArgs &w, hipStream_t st) {
  using L = Latent16<DQK, DV>;
  const size_t lds = (size_t)kWavesPerBlock * L::WAVE_LDS;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_latent16_kernel<DQK, DV>), lds, lds_ready))
    return false;
  launch_dominant(&paged_decode_latent16_kernel<DQK, DV>, dim3(a.n_waves / kWavesPerBlock), dim3(256), lds, st, a, w, a.pt, a.cur);
  return true;
}

// ---------------------------------------------------------------------------------------------
// The arithmetic of one wavefront of the two kernels below on one step of 32 keys (two 16-row pieces
// of K in LDS): the Q fragments of its two blocks of 16 rows, the running maxima and sums, and the
// two products as the assembly blocks of build/latent_frag_asm.h (written by gen_latent_frag.py,
// which says why assembly and where everything lives).  The output accumulators are registers that
// no variable stands for: clear, scale, read16 and the second products are all that touches them.
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
#include "build/latent_frag_asm.h"

template <int... Is, class F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}

template <int DQK, int DV>
struct LatentMath {
  using L = Latent16<DQK, DV>;
  using B = LatentBlocks<DQK, DV>;
  static constexpr int RB = 2;  // blocks of 16 rows
  static constexpr int KSTEPS = DQK / 32, VB = DV / 16;
  static constexpr int GC = L::HALF_PERIOD ? 8 : 16;  // chunks per swizzle group
  static constexpr int KB = GC / 4, VBASES = GC / 2;
  static constexpr int NQ16 = KSTEPS / 4, NA = VB / 4;
  static constexpr int REQUESTS = B::REQUESTS;  // LDS-DMA requests of a wavefront per step
  static_assert(VB % 4 == 0 && NQ16 >= 1 && (KSTEPS % 4 == 0 || KSTEPS % 4 == 2), "register blocks of 16");
  u32x16 q16[RB][NQ16];
  u32x8 q8[RB];
  floatx4 ml;                         // running maxima (0, 1) and sums (2, 3) of the two row blocks
  float th[RB];                       // (maximum + 8) / scale: the raw score above which a maximum moves
  uint32_t kfrag[KB], vfrag[VBASES];  // the lane's fragment offsets inside a piece

  // lane (n, quad): A operand of the score product = row n, chunk 4 s + quad; transposing read of
  // the value columns = row 4 quad + n / 4, values 16 vb + 4 (n % 4) ..
  __device__ __forceinline__ void init(int n, int quad) {
#pragma unroll
    for (int i = 0; i < KB; ++i) kfrag[i] = (uint32_t)(n * L::ROW + 16 * L::position(n, 4 * i + quad));
    const int rv = 4 * quad + (n >> 2), q4 = n & 3;
#pragma unroll
    for (int i = 0; i < VBASES; ++i)
      vfrag[i] = (uint32_t)(rv * L::ROW + 16 * L::position(rv, 2 * i + (q4 >> 1)) + 8 * (q4 & 1));
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int r = 0; r < 8; ++r) q8[b][r] = 0;
    restart();
  }
  __device__ __forceinline__ void restart() {
    B::clear();
    ml = floatx4{-INFINITY, -INFINITY, 0.f, 0.f};
    th[0] = th[1] = -INFINITY;
  }
  // B operand of the score product: features 32 s + 8 quad .. + 7 of the lane's row in block b
  __device__ __forceinline__ void set_q(int b, int s, const uint4 &t) {
    if (s < 4 * NQ16) {
      q16[b][s / 4][4 * (s % 4)] = t.x, q16[b][s / 4][4 * (s % 4) + 1] = t.y;
      q16[b][s / 4][4 * (s % 4) + 2] = t.z, q16[b][s / 4][4 * (s % 4) + 3] = t.w;
    } else {
      const int j = 4 * (s - 4 * NQ16);
      q8[b][j] = t.x, q8[b][j + 1] = t.y, q8[b][j + 2] = t.z, q8[b][j + 3] = t.w;
    }
  }
  __device__ __forceinline__ float maximum(int b) const { return ml[b]; }
  __device__ __forceinline__ float sum(int b) const { return ml[RB + b]; }
  // f[4 j + r] = value 16 (4 I + j) + 4 quad + r of the lane's row in block BLK (unnormalised)
  template <int BLK, int I>
  __device__ __forceinline__ void read16(float (&f)[16]) const {
    B::template read16<BLK, I>(f);
  }

  // `step`: LDS byte address of the first of the step's two pieces.  Lane (row, quad) receives in
  // st[b][pc] the scores of keys 16 pc + 4 quad + r of its row in block b.
  __device__ __forceinline__ void scores(uint32_t step, floatx4 (&st)[RB][2]) const { B::scores(step, st, kfrag, q16, q8); }
  // The same with the wavefront's requests for a later step between the matrix instructions:
  // 16 bytes per lane from `from` + off[j] to LDS address dst + 1024 j.  STREAMING: with the
  // non-temporal hint (rows that nobody reads again).
  template <bool STREAMING>
  __device__ __forceinline__ void scores_requesting(uint32_t step, floatx4 (&st)[RB][2], const uint32_t (&off)[REQUESTS],
                                                    const void *from, uint32_t dst) const {
    B::template scores_requesting<STREAMING>(step, st, kfrag, q16, q8, off, static_cast<const char *>(from), dst);
  }
  // Online softmax of a step's scores, in C++, for steps with masked keys: bias(b, pc, e) is added to
  // the scaled score of key 16 pc + 4 quad + e (-inf leaves the key out).  pf[b]: the lane's 8
  // probabilities as bfloat16 pairs; afterwards the accumulators owe the factor of scale_accumulators.
  template <class Bias>
  __device__ __forceinline__ void softmax(floatx4 (&st)[RB][2], u32x4 (&pf)[RB], float (&alpha)[RB], float scale, Bias &&bias) {
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      float sc[8], mloc = -INFINITY;
#pragma unroll
      for (int pc = 0; pc < 2; ++pc)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          sc[4 * pc + e] = st[b][pc][e] * scale + bias(b, pc, e);
          mloc = fmaxf(mloc, sc[4 * pc + e]);
        }
      mloc = max_over_quads(mloc);
      const float m_old = ml[b];
      const bool move = !(mloc - m_old <= 8.0f);  // (lazy: also true from -inf)
      const float m_new = move ? mloc : m_old;
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      alpha[b] = move ? __builtin_amdgcn_exp2f(m_old - m_safe) : 1.0f;
      ml[b] = m_new;
      th[b] = (m_new + 8.0f) * __builtin_amdgcn_rcpf(scale);
      float lsum = 0.f;
      bf16x8 pb8;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(sc[e] - m_safe);
        const __bf16 pb = (__bf16)p;
        lsum += (float)pb;  // the normaliser sums the weights that multiply V
        pb8[e] = pb;
      }
      pf[b] = __builtin_bit_cast(u32x4, pb8);
      ml[RB + b] = ml[RB + b] * alpha[b] + lsum;
    }
  }
  // accumulators *= alpha where a maximum has moved (rare: the maximum moves lazily)
  __device__ __forceinline__ void scale_accumulators(const float (&alpha)[RB]) {
    if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.0f || alpha[1] != 1.0f) != 0) B::scale(alpha[0], alpha[1]);
  }
  // O^T += V^T . P^T of the step at `step` with probabilities pf
  __device__ __forceinline__ void values(uint32_t step, const u32x4 (&pf)[RB]) { B::values(step, pf, vfrag); }
  // A whole step as one block that starts with the workgroup's barrier of the step (the caller has
  // waited for its own requests and does not call __syncthreads): the scores of the step at `step`, the second product of the step at
  // `before` (probabilities pf) and, between the matrix instructions of the latter, the softmax (no
  // masks, scale > 0) of the new scores; pf is replaced by the new probabilities.  The block keeps the
  // running maxima as they are; where a score would move one (rarely: a maximum moves by 8 at least),
  // the softmax above redoes the step.
  __device__ __forceinline__ void whole_step(uint32_t step, uint32_t before, u32x4 (&pf)[RB], floatx4 (&st)[RB][2], float (&alpha)[RB], float scale) {
    u32x4 pn[RB];
    float sum[RB];
    uint64_t moved;
    const float m[RB] = {ml[0], ml[1]};
    B::whole_step(step, before, st, pn, sum, moved, kfrag, vfrag, q16, q8, m, th, pf, scale);
    take(moved, pn, sum, pf, st, alpha, scale);
  }
  // The same with the wavefront's requests between the matrix instructions of the score product
  // (scores_requesting)
  template <bool STREAMING>
  __device__ __forceinline__ void whole_step_requesting(uint32_t step, uint32_t before, u32x4 (&pf)[RB], floatx4 (&st)[RB][2], float (&alpha)[RB],
                                                        float scale, const uint32_t (&off)[REQUESTS], const void *from, uint32_t dst) {
    u32x4 pn[RB];
    float sum[RB];
    uint64_t moved;
    const float m[RB] = {ml[0], ml[1]};
    B::template whole_step_requesting<STREAMING>(step, before, st, pn, sum, moved, kfrag, vfrag, q16, q8, m, th, pf, scale, off,
                                                 static_cast<const char *>(from), dst);
    take(moved, pn, sum, pf, st, alpha, scale);
  }

 private:
  __device__ __forceinline__ void take(uint64_t moved, const u32x4 (&pn)[RB], const float (&sum)[RB], u32x4 (&pf)[RB], floatx4 (&st)[RB][2],
                                       float (&alpha)[RB], float scale) {
    if (moved == 0) {
      pf[0] = pn[0], pf[1] = pn[1];
      ml[RB] += sum[0], ml[RB + 1] += sum[1];
      alpha[0] = alpha[1] = 1.0f;
    } else {
      softmax(st, pf, alpha, scale, [](int, int, int) { return 0.f; });
    }
  }
};

// ---------------------------------------------------------------------------------------------
// More than 16 query heads per KV head with V taken from K (the latent layer with all of its 128
// heads on one GPU): a segment is a block of up to 128 heads, a range of the flat list of 64-token
// tiles belongs to a workgroup of four wavefronts, one per SIMD, and wavefront i computes heads
// 32 i .. 32 i + 31 as two blocks of 16 rows (LatentMath<.., 2>) on K that the four share in LDS:
// a tile is two steps of 32 tokens, a step two 16-row pieces laid out like the 16-head form's stages
// and requested by LDS-DMA, a quarter per wavefront.  Nothing is computed twice and a latent row is
// read from memory once per 128 heads; the workgroup-shared form above re-reads it per block of 32
// heads and computes every score four times.
// The vector unit has no second wavefront to serve while the matrix unit works, so the softmax of a
// step's scores sits between the matrix instructions of the second product of the step before
// (whole_step), and the requests for a later step between those of the score product
// (scores_requesting); steps with masked keys (a sequence's last tile, the first of a sliding
// window) and a segment's first step take the softmax below.  A step's second product thereby runs
// one step late, so K lives in a ring of four stages with one barrier per step: past the barrier of
// step i every wavefront has finished the second product of step i - 2, whose stage the requests for
// step i + 2 overwrite.
template <int DQK, int DV>
__global__ __launch_bounds__(256) void paged_decode_latent128_kernel(
    DecodeArgs a, WideArgs w, const int32_t *__restrict__ page_table, const void *__restrict__ cur_pos) {
  using L = Latent16<DQK, DV>;
  using M = LatentMath<DQK, DV>;
  constexpr int RB = M::RB, SUB = L::TILE, KEYS = 2 * SUB, NWAVES = 4, NSTAGES = 4;
  constexpr int KSTEPS = M::KSTEPS;
  constexpr int PER_WAVE = M::REQUESTS;
  static_assert(kTile == 2 * KEYS && 2 * PER_WAVE == L::NDMA && PER_WAVE < 16, "two wavefronts request each 16-row piece");
  constexpr int STAGE = 2 * L::STAGE, WAVE_HEADS = 16 * RB;

  __shared__ int s_pref[kMaxUsersWide + 1];
  __shared__ int s_len[kMaxUsersWide];
  __shared__ int s_wsum[NWAVES];
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int seg_units = a.seg_units;
  build_prefix(a, cur_pos, s_pref, s_len, s_wsum, seg_units);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, quad = lane >> 4;
  const int wg = blockIdx.x;
  // The flat list in units: per segment `seg_units` units that stand for the cost of closing it (the
  // partial, the next segment's Q), then its tiles.  A range of more than seg_units units holds at
  // least one tile.
  const int total_units = __builtin_amdgcn_readfirstlane(s_pref[a.users]);
  const int64_t total = (int64_t)total_units * a.hkv;
  const int64_t max_ranges = total / (seg_units + 1);
  const int n_eff = (int)(max_ranges < a.n_waves ? max_ranges : a.n_waves);  // workgroups that get work
  if (total == 0 || wg >= n_eff) {
    publish_segment_row(a, s_pref, total, n_eff, seg_units);
    return;
  }
  const int64_t x_lo = (int64_t)wg * total / n_eff;
  const int64_t x_hi = (int64_t)(wg + 1) * total / n_eff;
  int64_t x = x_lo;  // set below to the unit of the first tile at or behind x_lo
  const int G = w.gseg;

  // ---- step requests: wavefronts 2 i and 2 i + 1 fetch piece i of a step (16 consecutive cache rows)
  const int sub_w = wave >> 1;
  uint32_t src_off[PER_WAVE];
#pragma unroll
  for (int j = 0; j < PER_WAVE; ++j) {
    const int kk = (wave & 1) * PER_WAVE + j;
    const int P = 64 * kk + lane, rr = P / L::CPR, p = P % L::CPR;
    src_off[j] = (uint32_t)(rr * L::ROW + 16 * L::position(rr, p));
  }
  const uint32_t lds0 = lds_address(smem);
  // the wavefront's piece of half `half` of tile cu: where its rows lie in the cache, where step i keeps them
  auto piece_source = [&](const Cursor &cu, int half) {
    const int kvh = cu.h / w.nhb;
    const int tok0 = cu.t * kTile + KEYS * half + SUB * sub_w;
    const int col = tok0 / a.bs;
    int phys = (col < a.w) ? page_table[(int64_t)cu.u * a.pt_rs + col] : 0;
    if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
    const int64_t row0 = ((int64_t)phys * w.nkv + kvh) * a.bs + (tok0 - col * a.bs);
    const uint64_t addr = reinterpret_cast<uint64_t>(a.k) + (uint64_t)row0 * L::ROW;
    return reinterpret_cast<const char *>(address_from_words(__builtin_amdgcn_readfirstlane((int)(uint32_t)addr),
                                                             __builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32))));
  };
  auto piece_stage = [&](int i) {
    return (uint32_t)__builtin_amdgcn_readfirstlane(
        (int)(lds0 + (uint32_t)((i % NSTAGES) * STAGE + sub_w * L::STAGE + 1024 * (wave & 1) * PER_WAVE)));
  };
  auto request_step = [&](const Cursor &cu, int half, int i) {
    const char *src = piece_source(cu, half);
    const uint32_t dst = piece_stage(i);
    const void *bases[4] = {src, src - 1024, src - 2048, src - 3072};
#pragma unroll
    for (int j = 0; j + 4 <= PER_WAVE; j += 4) {
      const uint32_t off[4] = {src_off[j], src_off[j + 1], src_off[j + 2], src_off[j + 3]};
      dma16_streaming_quad(bases, off, dst + 1024u * j);
    }
#pragma unroll
    for (int j = PER_WAVE / 4 * 4; j < PER_WAVE; ++j) dma16_streaming(src, src_off[j], dst + 1024u * j);
  };
  // Rows past the attended length may be cache rows nobody ever wrote: their scores are masked,
  // but as V rows they would turn 0 * Inf into NaN, so they are cleared in LDS.
  auto clear_unattended_rows = [&](int i, int nvalid) {
    for (int r = nvalid + wave; r < KEYS; r += NWAVES) {
      uint4 *row = reinterpret_cast<uint4 *>(smem + (i % NSTAGES) * STAGE + (r / SUB) * L::STAGE + (r % SUB) * L::ROW);
      for (int c = lane; c < L::ROW / 16; c += 64) row[c] = make_uint4(0, 0, 0, 0);
    }
  };
  M m;
  m.init(n, quad);
  auto load_q = [&](const Cursor &cu) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int hg = WAVE_HEADS * wave + 16 * rb + n;  // this lane's head inside the segment
      const uint16_t *qp = a.q + cu.u * a.q_us + (int64_t)(cu.h * G + min(hg, G - 1)) * a.q_hs + 8 * quad;
      const uint32_t qmask = hg < G ? 0xffffffffu : 0u;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        uint4 t = *reinterpret_cast<const uint4 *>(qp + 32 * s);
        t.x &= qmask, t.y &= qmask, t.z &= qmask, t.w &= qmask;
        m.set_q(rb, s, t);
      }
    }
  };

  Cursor cur = locate_unit(a, s_pref, s_len, x_lo, seg_units, &x);
  request_step(cur, 0, 0);
  request_step(cur, 1, 1);
  load_q(cur);
  publish_segment_row(a, s_pref, total, n_eff, seg_units);

  const float scale = a.scale_log2e;
  const bool wave_active = WAVE_HEADS * wave < G;
  u32x4 pf[RB];
  uint32_t prev = 0;
  bool have_prev = false;  // a second product is owed: step `prev`, probabilities pf
  bool drain = true;       // loads other than step requests are under way (Q)
  bool landed = false;     // the next step's K and Q have been waited for already
  int i = 0;               // step

  while (x < x_hi) {
    const int nvalid = cur.len - cur.t * kTile;
    const int nbelow = cur.lo - cur.t * kTile;  // sliding window: > 0 only in a segment's first tile
    // the unit of the tile behind this one: the next, or behind the next segment's leading units
    const int64_t x_next = x + (cur.tiles_left > 1 ? 1 : 1 + seg_units);
    const bool has_next = x_next < x_hi;
    const bool same_seg = has_next && cur.tiles_left > 1;
    Cursor nxt = cur;
    if (has_next) {
      if (same_seg) {
        nxt.t = cur.t + 1;
        nxt.tiles_left = cur.tiles_left - 1;
      } else {
        nxt = locate_unit(a, s_pref, s_len, x + 1, seg_units);
      }
    }
#pragma unroll 1
    for (int half = 0; half < 2; ++half, ++i) {
      // this wavefront's share of step i has landed (the requests of step i + 1 may still be under way)
      if (landed) {
        // (waited for while the segment was closed; the partial's stores need not be waited for)
      } else if (!drain && (half == 0 || has_next)) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | PER_WAVE);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      drain = landed = false;
      // ... and behind the workgroup's barrier everybody's has, and nobody reads the stage of step i - 2
      // any more.  A wavefront whose step needs no masks runs it as one block that starts with the barrier.
      const int nv = nvalid - KEYS * half, nb = nbelow - KEYS * half;  // this step attends its keys nb .. nv - 1
      const bool computing = wave_active && nv > 0;
      // (a wavefront that computes sends the requests from inside the score product)
      const bool inside = computing && has_next;
      // Two pieces (32 keys) per step: one softmax for both, and the second product takes them as the
      // 32-deep K dimension of one matrix instruction per block of 16 value columns (k index 8 quad + j
      // stands for key 4 quad + j of the first piece for j < 4, of the second otherwise: the order in
      // which the score tiles hold a lane's keys and the transposing reads their rows).
      const uint32_t step = lds0 + (uint32_t)((i % NSTAGES) * STAGE);
      floatx4 st[RB][2];
      float alpha[RB];
      if (computing && have_prev && nv >= KEYS && nb <= 0 && scale > 0.f) {
        if (inside) m.template whole_step_requesting<true>(step, prev, pf, st, alpha, scale, src_off, piece_source(nxt, half), piece_stage(i + 2));
        else m.whole_step(step, prev, pf, st, alpha, scale);
        m.scale_accumulators(alpha);
        prev = step;
        continue;
      }
      __syncthreads();
      if (has_next && !inside) request_step(nxt, half, i + 2);
      if (nv > 0 && nv < KEYS) {
        clear_unattended_rows(i, nv);
        __syncthreads();
      }
      if (!computing) {
        if (have_prev) m.values(prev, pf), have_prev = false;
        continue;
      }
      {
        if (inside) m.template scores_requesting<true>(step, st, src_off, piece_source(nxt, half), piece_stage(i + 2));
        else m.scores(step, st);
        if (have_prev) m.values(prev, pf);
        // lane (head, quad) holds keys 16 pc + 4 quad + e of the step
        m.softmax(st, pf, alpha, scale, [&](int, int pc, int e) {
          const int key = SUB * pc + 4 * quad + e;
          return (key >= nv || key < nb) ? -INFINITY : 0.f;
        });
      }
      m.scale_accumulators(alpha);
      prev = step, have_prev = true;
    }
    // ---- close the segment: every wavefront writes its heads' part of the partial -----------------
    if (!same_seg) {
      // (the next segment's Q first: its loads run while the partial is written)
      if (has_next) load_q(nxt);
      if (have_prev) m.values(prev, pf), have_prev = false;
      // Everything requested so far (Q, the next two steps) has to land before the next step anyway:
      // waited for here, behind the second product above and in front of the partial's stores, which
      // the next step then does not have to wait for.
      __builtin_amdgcn_s_waitcnt(0x0F70);
      float *slot = a.ws_slots + ((int64_t)wg + (int64_t)cur.u * a.hkv + cur.h) * a.slot_floats;
      // (the lane's place in the slot is worked out here, behind an opaque copy of the lane number:
      // kept across the loop it would not fit the register file)
      int l = lane;
      asm volatile("" : "+v"(l));
      const int quad = l >> 4;
      static_for(std::make_integer_sequence<int, RB>{}, [&](auto rbc) {
        constexpr int rb = decltype(rbc)::value;
        const int hg = WAVE_HEADS * wave + 16 * rb + (l & 15);
        const float l_tot = sum_over_quads(m.sum(rb));
        if (hg < G) {
          if (a.partial_bf16) {  // wavefront-uniform
            // in blocks of 16 heads x 16 columns (decode_combine_bf16_kernel): the 64 lanes of a
            // store write 512 consecutive bytes (head by head they wrote 16 pieces of 32 bytes, and the
            // partial took 7 us of the 10 us that a change of segment cost)
            constexpr int HEADS16 = WAVE_HEADS / 16;
            uint32_t *dst = reinterpret_cast<uint32_t *>(slot) + ((HEADS16 * wave + rb) * (DV / 16) * 16 + (l & 15)) * 8 + 2 * quad;
            static_for(std::make_integer_sequence<int, M::NA>{}, [&](auto ic) {
              constexpr int bi = decltype(ic)::value;
              float f[16];
              m.template read16<rb, bi>(f);
#pragma unroll
              for (int j = 0; j < 4; ++j)
                *reinterpret_cast<uint2 *>(dst + 128 * (4 * bi + j)) =
                    make_uint2(pack_bf16x2(f[4 * j], f[4 * j + 1]), pack_bf16x2(f[4 * j + 2], f[4 * j + 3]));
            });
            const int vals = (G + 15) / 16 * 16 * DV / 2;
            if (quad == 0) {
              slot[vals + hg] = m.maximum(rb);
              slot[vals + G + hg] = l_tot;
            }
          } else {
            float *dst = slot + hg * DV + 4 * quad;
            static_for(std::make_integer_sequence<int, M::NA>{}, [&](auto ic) {
              constexpr int bi = decltype(ic)::value;
              float f[16];
              m.template read16<rb, bi>(f);
#pragma unroll
              for (int j = 0; j < 4; ++j)
                *reinterpret_cast<float4 *>(dst + 16 * (4 * bi + j)) = make_float4(f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]);
            });
            if (quad == 0) {
              slot[G * DV + hg] = m.maximum(rb);
              slot[G * DV + G + hg] = l_tot;
            }
          }
        }
      });
      m.restart();
      landed = true;
    }
    cur = nxt, x = x_next;
  }
}

template <int DQK, int DV>
bool launch_latent128(const DecodeArgs &a, const WideArgs &w, hipStream_t st) {
  using L = Latent16<DQK, DV>;
  const size_t lds = 2 * 4 * (size_t)L::STAGE;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_latent128_kernel<DQK, DV>), lds, lds_ready))
    return false;
  launch_dominant(&paged_decode_latent128_kernel<DQK, DV>, dim3(a.n_waves), dim3(256), lds, st, a, w, a.pt, a.cur);
  return true;
}

// ---------------------------------------------------------------------------------------------
// Prefill over freshly built latent K with V taken from K: the rows of a (batch entry, KV head) are
// its (token, head) pairs, token-major, and a workgroup of eight wavefronts owns 128 consecutive ones
// (eight tokens of a 16-head group, one token of a 128-head group), 16 per wavefront in the N
// dimension of the products of the 16-head decode form above.  The eight wavefronts share every K
// tile of 64 keys in LDS (four 16-row pieces, each laid out and swizzled like a stage of that form,
// requested by LDS-DMA, one eighth per wavefront), so a K row is read from memory once per 128 rows
// and not once per row; two stages, one barrier per tile.  Every lane keeps the causal limit of its
// own row; a wavefront leaves out the 16-key pieces behind the limit of its last row.
struct LatentPrefillArgs {
  uint16_t *out;
  int64_t out_bs, out_hs, out_ts;
  const uint16_t *q;
  int64_t q_bs, q_hs, q_ts;
  const uint16_t *k;
  int64_t k_bs, k_hs, k_ts;
  const uint16_t *mask;  // additive, [batch, 1 or heads, s, s], or null
  int64_t mask_bs, mask_hs, mask_rs;
  int batch, heads, nkv, s, causal;
  float scale_log2e;
};

template <int DQK, int DV>
__global__ __launch_bounds__(256) void latent_prefill_kernel(LatentPrefillArgs a) {
  using L = Latent16<DQK, DV>;
  using M = LatentMath<DQK, DV>;
  constexpr int RB = M::RB, SUB = L::TILE, KEYS = 2 * SUB, NWAVES = 4, WROWS = 16 * RB, ROWS = WROWS * NWAVES, NSTAGES = 4;
  constexpr int KSTEPS = M::KSTEPS;
  constexpr int PER_WAVE = M::REQUESTS;
  static_assert(NWAVES * PER_WAVE == 2 * L::NDMA && PER_WAVE < 16, "a step's requests divide among the wavefronts");
  constexpr int STAGE = 2 * L::STAGE;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, quad = lane >> 4;
  const int G = a.heads / a.nkv;
  const int rows_total = G * a.s;
  const int nblk = (rows_total + ROWS - 1) / ROWS;
  const int groups = a.batch * a.nkv;
  // late (heavy) row blocks first; neighbouring workgroups take the same block of different groups
  const int blk = nblk - 1 - (int)blockIdx.x / groups;
  const int grp = (int)blockIdx.x % groups;
  const int b = grp / a.nkv, kvh = grp - b * a.nkv;

  const int r0 = blk * ROWS + wave * WROWS;
  const bool wave_active = r0 < rows_total;
  // Token and head of the lane's row in block rb (rows past the end repeat the last one and are not
  // stored).  Worked out where it is needed, behind an opaque copy of the lane number: kept across
  // the loop, the rows' tokens, heads and mask addresses would not fit the register file.
  auto row_of = [&](int rb, int &t, int &head) {
    int l = lane;
    asm volatile("" : "+v"(l));
    const int r = min(r0 + 16 * rb + (l & 15), rows_total - 1);
    t = r / G, head = kvh * G + (r - t * G);
  };
  const int first_limit = a.causal ? min(r0, rows_total - 1) / G : a.s - 1;  // the smallest limit among the rows
  const int wave_limit = a.causal ? min(r0 + WROWS - 1, rows_total - 1) / G : a.s - 1;
  const int wg_limit = a.causal ? min(blk * ROWS + ROWS - 1, rows_total - 1) / G : a.s - 1;
  const int nsteps = wg_limit / KEYS + 1;
  const float scale = a.scale_log2e;
  const bool plain = a.mask == nullptr;  // (the scale is positive: the entry point checks)

  // ---- step requests: instruction k = wave * PER_WAVE + j of the step's 2 * NDMA ---------------
  const uint16_t *kbase_g = a.k + b * a.k_bs + kvh * a.k_hs;
  const uint32_t row_bytes = 2u * (uint32_t)a.k_ts;
  // (offsets inside a step whose 32 keys all exist; the last step of a sequence clamps row by row)
  uint32_t req_off[PER_WAVE];
#pragma unroll
  for (int j = 0; j < PER_WAVE; ++j) {
    const int k = wave * PER_WAVE + j, sub = k / L::NDMA, kk = k % L::NDMA;
    const int P = 64 * kk + lane, rr = P / L::CPR, p = P % L::CPR;
    req_off[j] = (uint32_t)(SUB * sub + rr) * row_bytes + 16u * (uint32_t)L::position(rr, p);
  }
  const uint32_t lds0 = lds_address(smem);
  auto request_step = [&](int i) {
    const uint32_t dst0 =
        (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + (uint32_t)((i % NSTAGES) * STAGE + 1024 * wave * PER_WAVE)));
    if ((i + 1) * KEYS <= a.s) {
      const uint16_t *step_base = kbase_g + (int64_t)i * KEYS * a.k_ts;
      // (four requests behind one write of M0: the instruction offset moves the LDS address too)
      const char *tb = reinterpret_cast<const char *>(step_base);
      const void *bases[4] = {tb, tb - 1024, tb - 2048, tb - 3072};
#pragma unroll
      for (int j = 0; j + 4 <= PER_WAVE; j += 4) {
        const uint32_t off[4] = {req_off[j], req_off[j + 1], req_off[j + 2], req_off[j + 3]};
        dma16_quad(bases, off, dst0 + 1024u * j);
      }
#pragma unroll
      for (int j = PER_WAVE / 4 * 4; j < PER_WAVE; ++j) dma16(step_base, req_off[j], dst0 + 1024u * j);
    } else {
#pragma unroll 1
      for (int j = 0; j < PER_WAVE; ++j) {
        const int k = wave * PER_WAVE + j, sub = k / L::NDMA, kk = k % L::NDMA;
        const int P = 64 * kk + lane, rr = P / L::CPR, p = P % L::CPR;
        const int key = min(i * KEYS + SUB * sub + rr, a.s - 1);  // rows past the end repeat the last one
        dma16(kbase_g, (uint32_t)key * row_bytes + 16u * (uint32_t)L::position(rr, p), dst0 + 1024u * (uint32_t)j);
      }
    }
  };

  M m;
  m.init(n, quad);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    int t, head;
    row_of(rb, t, head);
    const uint16_t *qp = a.q + b * a.q_bs + head * a.q_hs + (int64_t)t * a.q_ts + 8 * quad;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) m.set_q(rb, s, *reinterpret_cast<const uint4 *>(qp + 32 * s));
  }
  // (behind the Q loads: the waits below count this wavefront's requests only from here on)
  request_step(0);
  if (nsteps > 1) request_step(1);

  u32x4 pf[RB];
  uint32_t prev = 0;
  bool have_prev = false;  // a second product is owed: step `prev`, probabilities pf

  for (int i = 0; i < nsteps; ++i) {
    // this wavefront's share of step i has landed (the requests of step i + 1 may still be under way)
    if (i + 1 < nsteps) __builtin_amdgcn_s_waitcnt(0x0F70 | PER_WAVE);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    // ... and behind the workgroup's barrier everybody's has, and nobody reads the stage of step i - 2 any
    // more.  A wavefront whose step needs no masks runs the step as one block that starts with the barrier.
    const int key0 = i * KEYS;
    const bool computing = wave_active && key0 <= wave_limit;
    // (a wavefront that computes sends whole steps' requests from inside the score product)
    const bool inside = computing && i + 2 < nsteps && (i + 3) * KEYS <= a.s;
    const uint32_t step = lds0 + (uint32_t)((i % NSTAGES) * STAGE);
    floatx4 st[RB][2];
    float alpha[RB];
    const uint32_t dst0 = (uint32_t)__builtin_amdgcn_readfirstlane(
        (int)(lds0 + (uint32_t)(((i + 2) % NSTAGES) * STAGE + 1024 * wave * PER_WAVE)));
    const uint16_t *from = kbase_g + (int64_t)(i + 2) * KEYS * a.k_ts;
    if (computing && have_prev && plain && key0 + KEYS - 1 <= first_limit && (inside || i + 2 >= nsteps)) {
      if (inside) m.template whole_step_requesting<false>(step, prev, pf, st, alpha, scale, req_off, from, dst0);
      else m.whole_step(step, prev, pf, st, alpha, scale);
      m.scale_accumulators(alpha);
      prev = step;
      continue;
    }
    __syncthreads();
    if (i + 2 < nsteps && !inside) request_step(i + 2);
    if (!computing) {
      if (have_prev) m.values(prev, pf), have_prev = false;
      continue;
    }
    // Two pieces (32 keys) per step: one softmax for both, and the second product takes them as the
    // 32-deep K dimension of one matrix instruction per block of 16 value columns.  k index 8 quad + j
    // of that instruction stands for key 4 quad + j of the first piece (j < 4) or of the second: the
    // order in which the score tiles hold the keys of a lane, and the transposing reads their rows.
    {
      if (inside) m.template scores_requesting<false>(step, st, req_off, from, dst0);
      else m.scores(step, st);
      if (have_prev) m.values(prev, pf);
      // lane (row, quad) holds keys key0 + 16 pc + 4 quad + e of its rows
      int limit[RB], t[RB], head[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        row_of(rb, t[rb], head[rb]);
        limit[rb] = a.causal ? t[rb] : a.s - 1;
      }
      m.softmax(st, pf, alpha, scale, [&](int rb, int pc, int e) {
        const int key = key0 + 16 * pc + 4 * quad + e;
        float add = 0.f;
        if (a.mask) {
          const int kq = min(key0 + 16 * pc + 4 * quad, a.s - 4);
          const uint2 mw = *reinterpret_cast<const uint2 *>(a.mask + b * a.mask_bs + head[rb] * a.mask_hs + (int64_t)t[rb] * a.mask_rs + kq);
          add = (e == 0 ? bf16_lo(mw.x) : e == 1 ? bf16_hi(mw.x) : e == 2 ? bf16_lo(mw.y) : bf16_hi(mw.y)) * 1.4426950408889634f;
        }
        return key > limit[rb] ? -INFINITY : add;
      });
    }
    m.scale_accumulators(alpha);
    prev = step, have_prev = true;
  }
  if (wave_active && have_prev) m.values(prev, pf);
  // ---- normalise and store --------------------------------------------------------------------
  // Lane (row, quad) holds values 16 vb + 4 quad .. + 3 of its rows: stored from there, a store would
  // write 16 pieces of 32 bytes (7.7 us per workgroup, a tenth of its time).  Instead the rows of a row
  // block go through LDS (nobody reads K any more), a wavefront's own 16 rows of 2 DV + 16 bytes (the
  // pitch puts the 16 rows of a 8-byte write into different banks), and come back 16 bytes per lane
  // along the rows: a store writes whole rows.
  __syncthreads();
  if (!wave_active) return;
  constexpr int PITCH = 2 * DV + 16, LPR = DV / 8, RPI = 64 / LPR;  // bytes per staged row, lanes per row, rows per store
  static_assert((PITCH / 4) % 64 == 4 && 64 % LPR == 0 && 16 % RPI == 0 && NWAVES * 16 * PITCH <= NSTAGES * STAGE, "staging area of the output");
  unsigned char *staged = smem + (lds0 - lds_address(smem)) + wave * (16 * PITCH);
  static_for(std::make_integer_sequence<int, RB>{}, [&](auto rbc) {
    constexpr int rb = decltype(rbc)::value;
    const float inv = 1.0f / sum_over_quads(m.sum(rb));
    static_for(std::make_integer_sequence<int, M::NA>{}, [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      float f[16];
      m.template read16<rb, i>(f);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint2 *>(staged + n * PITCH + 32 * (4 * i + j) + 8 * quad) =
            make_uint2(pack_bf16x2(f[4 * j] * inv, f[4 * j + 1] * inv), pack_bf16x2(f[4 * j + 2] * inv, f[4 * j + 3] * inv));
    });
#pragma unroll 4
    for (int r = 0; r < 16; r += RPI) {
      const int rs = r + lane / LPR;  // the lane's row among the 16, 16 bytes of it at chunk lane % LPR
      const int row = r0 + 16 * rb + rs;
      if (row < rows_total) {
        const int t = row / G, head = kvh * G + (row - t * G);
        const uint4 v = *reinterpret_cast<const uint4 *>(staged + rs * PITCH + 16 * (lane % LPR));
        *reinterpret_cast<uint4 *>(a.out + b * a.out_bs + head * a.out_hs + (int64_t)t * a.out_ts + 8 * (lane % LPR)) = v;
      }
    }
  });
}

template <int DQK, int DV>
int launch_latent_prefill(const LatentPrefillArgs &a, hipStream_t st) {
  using L = Latent16<DQK, DV>;
  const size_t lds = 4 * 2 * (size_t)L::STAGE;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&latent_prefill_kernel<DQK, DV>), lds, lds_ready))
    return fail(TTPA_ERR_LAUNCH, "latent prefill: cannot reserve %zu bytes of LDS", lds);
  const int64_t rows = (int64_t)(a.heads / a.nkv) * a.s;
  const int64_t grid = (rows + 127) / 128 * a.batch * a.nkv;
  launch_dominant(&latent_prefill_kernel<DQK, DV>, dim3((unsigned)grid), dim3(256), lds, st, a);
  return check_launch("latent_prefill");
}

template <int DQK, int DVW, bool SHARED_V>
bool launch(const DecodeArgs &a, const WideArgs &w, hipStream_t st) {
  using L = WideLds<DQK, DVW, SHARED_V>;
  const size_t lds = 2 * (size_t)L::STAGE;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&paged_decode_wide_kernel<DQK, DVW, SHARED_V>), lds,
                          lds_ready))
    return false;
  paged_decode_wide_kernel<DQK, DVW, SHARED_V><<<dim3(a.n_waves), dim3(256), lds, st>>>(a, w, a.pt, a.cur);
  return true;
}

}  // namespace
}  // namespace decode
}  // namespace ttpa

using namespace ttpa;
using namespace ttpa::decode;

// Workspace: the segment table followed by (workgroups + segments) partial slots.
// The merge of bfloat16 partials: 16 bytes per thread where the output rows allow it.
static void launch_combine_bf16(const DecodeArgs &a, int segments, int gseg, int head_dim_v, const void *out, int64_t out_user_stride,
                                int64_t out_head_stride, hipStream_t st) {
  const int words = (gseg + 15) / 16 * 16 * head_dim_v / 2;
  if (out_user_stride % 8 == 0 && out_head_stride % 8 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0)
    decode_combine_bf16_kernel<4><<<dim3(segments, combine_pieces(words / 4, 1)), dim3(256), 0, st>>>(a, gseg, head_dim_v);
  else
    decode_combine_bf16_kernel<1><<<dim3(segments, combine_pieces(words, 1)), dim3(256), 0, st>>>(a, gseg, head_dim_v);
}

static int wide_geometry(int32_t q_heads, int32_t kv_heads, int32_t &nhb, int32_t &gseg) {
  const int g = q_heads / kv_heads;
  if (g <= 32) {
    nhb = 1, gseg = g;
  } else if (g % 32 == 0) {
    nhb = g / 32, gseg = 32;
  } else {
    return fail(TTPA_ERR_UNSUPPORTED,
                "latent decode: %d query heads per KV head; supported up to 32 or a multiple of 32", g);
  }
  return TTPA_OK;
}

// The 128-head form: more than 16 heads per KV head in segments of up to 128.
static bool latent128_geometry(int32_t q_heads, int32_t kv_heads, int32_t &nhb, int32_t &gseg) {
  const int g = q_heads / kv_heads;
  if (g <= 16) return false;
  if (g <= 128) {
    nhb = 1, gseg = g;
    return true;
  }
  if (g % 128) return false;
  nhb = g / 128, gseg = 128;
  return true;
}

extern "C" size_t ttpa_paged_mla_decode_workspace_bytes(int32_t users, int32_t q_heads, int32_t kv_heads,
                                                        int32_t head_dim_v) {
  if (users <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim_v <= 0 || q_heads % kv_heads) return 0;
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  size_t need = 0;
  int32_t nhb, gseg;
  // (error text of a geometry the workgroup-shared form refuses is not this function's business)
  if (wide_geometry(q_heads, kv_heads, nhb, gseg) == TTPA_OK) {
    const size_t segs = (size_t)users * kv_heads * nhb;
    // (float partials, or bfloat16 ones in blocks of 16 heads: more when a group has fewer than 8)
    const size_t slot = (size_t)std::max(slot_floats_for(gseg, head_dim_v), slot_floats_bf16_for(gseg, head_dim_v)) * sizeof(float);
    // one slot per range of the largest grid (at most four wavefront ranges per CU in the 16-head form)
    need = header_bytes(users, kv_heads * nhb) + ((size_t)cus * kWavesPerBlockHost + segs) * slot;
  }
  if (latent128_geometry(q_heads, kv_heads, nhb, gseg)) {
    const size_t segs = (size_t)users * kv_heads * nhb;
    const size_t slot = (size_t)slot_floats_for(gseg, head_dim_v) * sizeof(float);
    need = std::max(need, header_bytes(users, kv_heads * nhb) + ((size_t)cus + segs) * slot);  // one range per CU
  }
  return need;
}

static int mla_decode_impl(void *out, int64_t out_user_stride, int64_t out_head_stride,
                           const void *q, int64_t q_user_stride, int64_t q_head_stride,
                           const void *k_cache, const void *v_cache, const int32_t *page_table,
                           int64_t page_table_row_stride, const void *cur_pos,
                           int cur_pos_is_i64, int32_t users, int32_t q_heads,
                           int32_t kv_heads, int32_t head_size, int32_t head_dim_v,
                           int32_t block_size, int32_t table_width, int32_t num_blocks,
                           float scale, const float *attention_sink, void *workspace,
                           size_t workspace_bytes, void *stream, const void *mask,
                           int64_t mask_user_stride, int64_t mask_head_stride) {
  TTPA_REQUIRE(out && q && k_cache && page_table && cur_pos, "null pointer argument");
  TTPA_REQUIRE(users > 0 && q_heads > 0 && kv_heads > 0 && head_size > 0 && head_dim_v > 0 &&
                   block_size > 0 && table_width > 0 && num_blocks > 0,
               "non-positive dimension");
  TTPA_REQUIRE(q_heads % kv_heads == 0, "q_heads %d not divisible by kv_heads %d", q_heads, kv_heads);
  TTPA_REQUIRE(v_cache || head_dim_v <= head_size,
               "head_dim_v %d exceeds head_size %d while V is taken from K", head_dim_v, head_size);
  if (users > kMaxUsersWide)
    return fail(TTPA_ERR_UNSUPPORTED, "latent decode: %d users exceeds the limit of %d", users, kMaxUsersWide);
  int32_t nhb, gseg;
  // The 128-head form: V taken from K, more than 16 heads per KV head, 16-row pieces inside one block,
  // no mask.  TTPA_LATENT_KERNEL=wide (read on every call) keeps such shapes on the workgroup-shared form.
  const char *force = getenv("TTPA_LATENT_KERNEL");
  const bool built128 = (head_size == 576 && (head_dim_v == 512 || head_dim_v == 384)) ||
                        (head_size == 192 && head_dim_v == 128) || (head_size == 128 && head_dim_v == 128);
  const bool want128 = !mask && !v_cache && built128 && block_size % 16 == 0 && !(force && force[0] == 'w') &&
                       latent128_geometry(q_heads, kv_heads, nhb, gseg);
  if (!want128)
    if (int rc = wide_geometry(q_heads, kv_heads, nhb, gseg)) return rc;
  TTPA_REQUIRE(aligned16(q) && aligned16(k_cache) && aligned16(out) && (!v_cache || aligned16(v_cache)),
               "latent decode: q / caches / out must be 16-byte aligned");
  TTPA_REQUIRE(q_user_stride % 8 == 0 && q_head_stride % 8 == 0,
               "latent decode: q strides must be multiples of 8 elements");
  const size_t need = ttpa_paged_mla_decode_workspace_bytes(users, q_heads, kv_heads, head_dim_v);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return fail(TTPA_ERR_WORKSPACE, "latent decode: workspace of %zu bytes (256-byte aligned) required, got %zu",
                need, workspace_bytes);

  // value slices: up to four wavefronts of 64 or 128 columns each
  const int dvw = head_dim_v % 128 == 0 ? 128 : 64;
  if (head_dim_v % dvw || head_dim_v / dvw > (v_cache ? 2 : 4))
    return fail(TTPA_ERR_UNSUPPORTED,
                "latent decode: head_dim_v %d; supported 64, 128, 256 (and 384, 512 when V is taken from K)",
                head_dim_v);

  DecodeArgs a;
  a.out = static_cast<uint16_t *>(out);
  a.out_us = out_user_stride, a.out_hs = out_head_stride;
  a.q = static_cast<const uint16_t *>(q);
  a.q_us = q_user_stride, a.q_hs = q_head_stride;
  a.k = static_cast<const uint8_t *>(k_cache);
  a.v = static_cast<const uint8_t *>(v_cache);
  a.pt = page_table, a.pt_rs = page_table_row_stride;
  a.cur = cur_pos, a.cur_i64 = cur_pos_is_i64;
  a.users = users, a.hq = q_heads, a.hkv = kv_heads * nhb, a.bs = block_size, a.w = table_width;
  a.nb = num_blocks;
  a.scale_log2e = scale * 1.4426950408889634f;
  a.ws_seg = static_cast<int *>(workspace);
  a.ws_slots = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + header_bytes(users, kv_heads * nhb));
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  a.n_waves = cus;  // one range per workgroup, one workgroup per CU
  a.slot_floats = slot_floats_for(gseg, head_dim_v);
  a.kv_format = TTPA_KV_BF16;
  a.window = 0;
  a.sink = attention_sink;
  a.mask = static_cast<const uint16_t *>(mask);
  a.mask_us = mask_user_stride, a.mask_hs = mask_head_stride;
  if (mask) TTPA_REQUIRE(scale != 0.f, "masked latent decode: scale must not be 0");
  WideArgs w;
  w.nkv = kv_heads, w.nhb = nhb, w.gseg = gseg, w.dv = head_dim_v, w.n_slices = head_dim_v / dvw;

  hipStream_t st = static_cast<hipStream_t>(stream);
  // armed profile events: the 16-head kernel's launch carries them itself; the workgroup-shared
  // kernel is bracketed below
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  bool ok = false, built = true;
  const bool shared = v_cache == nullptr;
  if (want128) {
    if ((int64_t)users * kv_heads * nhb > ((int64_t)a.n_waves + 1) * 256)
      return fail(TTPA_ERR_UNSUPPORTED, "latent decode: %d x %d segments need a grid of more than %d workgroups",
                  users, kv_heads * nhb, a.n_waves);
    // partials as bfloat16, as in the 16-head form (TTPA_LATENT_PARTIALS=f32 keeps floats)
    const char *pf = getenv("TTPA_LATENT_PARTIALS");
    a.partial_bf16 = !(pf && pf[0] == 'f') && out_user_stride % 2 == 0 && out_head_stride % 2 == 0 &&
                     reinterpret_cast<uintptr_t>(out) % 4 == 0;
    if (a.partial_bf16) a.slot_floats = slot_floats_bf16_for(gseg, head_dim_v);
    // units in front of every segment of the flat list: what a change of segment costs a range, in tiles
    // (the partial, the next segment's Q and first step; 128 users of 512 ... 8192 tokens: 180 us with none,
    // 167 with two, 163 with three to five)
    a.seg_units = segment_units(4);
    if (head_size == 576 && head_dim_v == 512) ok = launch_latent128<576, 512>(a, w, st);
    else if (head_size == 576 && head_dim_v == 384) ok = launch_latent128<576, 384>(a, w, st);
    else if (head_size == 192 && head_dim_v == 128) ok = launch_latent128<192, 128>(a, w, st);
    else ok = launch_latent128<128, 128>(a, w, st);
    if (!ok) return fail(TTPA_ERR_LAUNCH, "latent decode: cannot configure the kernel");
    if (int rc = check_launch("paged_mla_decode")) return rc;
    if (a.partial_bf16)
      launch_combine_bf16(a, users * kv_heads * nhb, gseg, head_dim_v, out, out_user_stride, out_head_stride, st);
    else
      decode_combine_kernel<<<dim3(users * kv_heads * nhb, combine_pieces(gseg, head_dim_v)), dim3(256), 0, st>>>(a, gseg, head_dim_v);
    return check_launch("paged_mla_decode");
  }
  // The 16-head form: V taken from K, one head block of up to 16 heads, tiles inside one block.
  // (only the workgroup-shared form applies a mask)
  const bool want16 = !mask && shared && nhb == 1 && gseg <= 16 && block_size % 16 == 0 && !(force && force[0] == 'w');
  if (want16) {
    // three wavefront ranges per CU: 131 us per step on the 128-user workload against 134 at four
    // (fewer partials of 32 KiB each), 139 at 2.5 and 159 at two; TTPA_DECODE_WAVES_PER_CU overrides,
    // up to the four per CU that the workspace is sized for
    a.n_waves = std::min(cus * kWavesPerBlockHost, waves_for_device(3.0));
    // one thread of the grid per segment publishes the segment's partial slots
    if ((int64_t)users * kv_heads > (int64_t)a.n_waves * kWave)
      return fail(TTPA_ERR_UNSUPPORTED, "latent decode: %d x %d segments need a grid of more than %d wavefronts",
                  users, kv_heads, a.n_waves);
    // three units in front of every segment of the flat list (a partial here is 32 KiB, a tile
    // 18 KiB): 130 us per step against 131-134 with none
    a.seg_units = segment_units(3);
    // partials as bfloat16 (TTPA_LATENT_PARTIALS=f32, read on every call, keeps floats): half the
    // bytes written here and read by the merge
    const char *pf = getenv("TTPA_LATENT_PARTIALS");
    // (the merge then stores output pairs as words: rows on 4-byte boundaries)
    a.partial_bf16 = !(pf && pf[0] == 'f') && out_user_stride % 2 == 0 && out_head_stride % 2 == 0 &&
                     reinterpret_cast<uintptr_t>(out) % 4 == 0;
    if (a.partial_bf16) a.slot_floats = slot_floats_bf16_for(gseg, head_dim_v);
    bool have = true;
    if (head_size == 576 && head_dim_v == 512) ok = launch_latent16<576, 512>(a, w, st);
    else if (head_size == 576 && head_dim_v == 384) ok = launch_latent16<576, 384>(a, w, st);
    else if (head_size == 192 && head_dim_v == 128) ok = launch_latent16<192, 128>(a, w, st);
    else if (head_size == 128 && head_dim_v == 128) ok = launch_latent16<128, 128>(a, w, st);
    else have = false;
    if (have) {
      take_profile_events(ev0, ev1);  // still armed only if the launch did not happen
      if (!ok) return fail(TTPA_ERR_LAUNCH, "latent decode: cannot configure the kernel");
      if (int rc = check_launch("paged_mla_decode")) return rc;
      if (a.partial_bf16)
        launch_combine_bf16(a, users * kv_heads, gseg, head_dim_v, out, out_user_stride, out_head_stride, st);
      else
        decode_combine_kernel<<<dim3(users * kv_heads, combine_pieces(gseg, head_dim_v)), dim3(256), 0, st>>>(a, gseg, head_dim_v);
      return check_launch("paged_mla_decode");
    }
    a.n_waves = cus;
    a.seg_units = 0;
    a.partial_bf16 = 0;
    a.slot_floats = slot_floats_for(gseg, head_dim_v);
  }
  take_profile_events(ev0, ev1);
  if (ev0) (void)hipEventRecord(ev0, st);
#define TTPA_WIDE_CASE(DQK, DVW)                                                                   \
  if (head_size == DQK && dvw == DVW)                                                              \
    ok = shared ? launch<DQK, DVW, true>(a, w, st) : launch<DQK, DVW, false>(a, w, st);            \
  else
  TTPA_WIDE_CASE(576, 128)
  TTPA_WIDE_CASE(192, 128)
  TTPA_WIDE_CASE(192, 64)
  TTPA_WIDE_CASE(128, 128)
  TTPA_WIDE_CASE(128, 64)
  TTPA_WIDE_CASE(64, 64)
  built = false;
#undef TTPA_WIDE_CASE
  if (!built)
    return fail(TTPA_ERR_UNSUPPORTED, "latent decode: head_size %d with head_dim_v %d is not built", head_size,
                head_dim_v);
  if (!ok) return fail(TTPA_ERR_LAUNCH, "latent decode: cannot configure the kernel");
  if (ev1) (void)hipEventRecord(ev1, st);
  if (int rc = check_launch("paged_mla_decode")) return rc;
  decode_combine_kernel<<<dim3(users * kv_heads * nhb, combine_pieces(gseg, head_dim_v)), dim3(256), 0, st>>>(a, gseg, head_dim_v);
  return check_launch("paged_mla_decode");
}

extern "C" int ttpa_paged_mla_decode(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                     const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                     const void *k_cache, const void *v_cache, const int32_t *page_table,
                                     int64_t page_table_row_stride, const void *cur_pos,
                                     int cur_pos_is_i64, int32_t users, int32_t q_heads,
                                     int32_t kv_heads, int32_t head_size, int32_t head_dim_v,
                                     int32_t block_size, int32_t table_width, int32_t num_blocks,
                                     float scale, const float *attention_sink, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return mla_decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache, v_cache,
                         page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users, q_heads, kv_heads,
                         head_size, head_dim_v, block_size, table_width, num_blocks, scale, attention_sink,
                         workspace, workspace_bytes, stream, nullptr, 0, 0);
}

extern "C" int ttpa_paged_mla_decode_masked(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                            const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                            const void *k_cache, const void *v_cache, const int32_t *page_table,
                                            int64_t page_table_row_stride, const void *cur_pos,
                                            int cur_pos_is_i64, int32_t users, int32_t q_heads,
                                            int32_t kv_heads, int32_t head_size, int32_t head_dim_v,
                                            int32_t block_size, int32_t table_width, int32_t num_blocks,
                                            float scale, const void *mask, int64_t mask_user_stride,
                                            int64_t mask_head_stride, void *workspace, size_t workspace_bytes,
                                            void *stream) {
  TTPA_REQUIRE(mask != nullptr, "masked latent decode: null mask");
  return mla_decode_impl(out, out_user_stride, out_head_stride, q, q_user_stride, q_head_stride, k_cache, v_cache,
                         page_table, page_table_row_stride, cur_pos, cur_pos_is_i64, users, q_heads, kv_heads,
                         head_size, head_dim_v, block_size, table_width, num_blocks, scale, nullptr, workspace,
                         workspace_bytes, stream, mask, mask_user_stride, mask_head_stride);
}

extern "C" int ttpa_latent_prefill(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                                   int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                                   int64_t q_head_stride, int64_t q_token_stride, const void *k,
                                   int64_t k_batch_stride, int64_t k_head_stride, int64_t k_token_stride,
                                   const void *mask, int64_t mask_batch_stride, int64_t mask_head_stride,
                                   int64_t mask_row_stride, int32_t batch, int32_t q_heads, int32_t kv_heads,
                                   int32_t seq_len, int32_t head_size, int32_t head_dim_v, int32_t causal,
                                   float scale, void *stream) {
  TTPA_REQUIRE(out && q && k, "null pointer argument");
  TTPA_REQUIRE(batch > 0 && q_heads > 0 && kv_heads > 0 && seq_len > 0 && head_size > 0 && head_dim_v > 0,
               "non-positive dimension");
  TTPA_REQUIRE(q_heads % kv_heads == 0, "q_heads %d not divisible by kv_heads %d", q_heads, kv_heads);
  TTPA_REQUIRE(head_dim_v <= head_size, "head_dim_v %d exceeds head_size %d while V is taken from K", head_dim_v,
               head_size);
  TTPA_REQUIRE(!(mask && causal), "an additive mask excludes causal masking");
  TTPA_REQUIRE(scale > 0.f, "latent prefill: scale %g must be positive", (double)scale);
  TTPA_REQUIRE(aligned16(q) && aligned16(k) && aligned16(out), "latent prefill: q / k / out must be 16-byte aligned");
  TTPA_REQUIRE(q_batch_stride % 8 == 0 && q_head_stride % 8 == 0 && q_token_stride % 8 == 0 && k_batch_stride % 8 == 0 &&
                   k_head_stride % 8 == 0 && k_token_stride % 8 == 0,
               "latent prefill: q / k strides must be multiples of 8 elements");
  TTPA_REQUIRE(out_batch_stride % 8 == 0 && out_head_stride % 8 == 0 && out_token_stride % 8 == 0,
               "latent prefill: out strides must be multiples of 8 elements");
  TTPA_REQUIRE((int64_t)seq_len * k_token_stride * 2 < (1ll << 32), "latent prefill: a K head must stay below 4 GiB");
  if (mask) {
    TTPA_REQUIRE(seq_len % 4 == 0 && (reinterpret_cast<uintptr_t>(mask) & 7u) == 0 && mask_batch_stride % 4 == 0 &&
                     mask_head_stride % 4 == 0 && mask_row_stride % 4 == 0,
                 "latent prefill: a mask needs seq_len %% 4 == 0, 8-byte alignment and strides that are multiples of 4 elements");
  }
  const int64_t rows = (int64_t)(q_heads / kv_heads) * seq_len;
  TTPA_REQUIRE(rows < (1ll << 31) && (rows + 127) / 128 * batch * kv_heads < (1ll << 31),
               "latent prefill: too many rows for one launch");
  LatentPrefillArgs a;
  a.out = static_cast<uint16_t *>(out);
  a.out_bs = out_batch_stride, a.out_hs = out_head_stride, a.out_ts = out_token_stride;
  a.q = static_cast<const uint16_t *>(q);
  a.q_bs = q_batch_stride, a.q_hs = q_head_stride, a.q_ts = q_token_stride;
  a.k = static_cast<const uint16_t *>(k);
  a.k_bs = k_batch_stride, a.k_hs = k_head_stride, a.k_ts = k_token_stride;
  a.mask = static_cast<const uint16_t *>(mask);
  a.mask_bs = mask_batch_stride, a.mask_hs = mask_head_stride, a.mask_rs = mask_row_stride;
  a.batch = batch, a.heads = q_heads, a.nkv = kv_heads, a.s = seq_len, a.causal = causal ? 1 : 0;
  a.scale_log2e = scale * 1.4426950408889634f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (head_size == 576 && head_dim_v == 512) return launch_latent_prefill<576, 512>(a, st);
  if (head_size == 192 && head_dim_v == 128) return launch_latent_prefill<192, 128>(a, st);
  if (head_size == 128 && head_dim_v == 128) return launch_latent_prefill<128, 128>(a, st);
  return fail(TTPA_ERR_UNSUPPORTED,
              "latent prefill: (head_size, head_dim_v) = (%d, %d); built for (576, 512), (192, 128), (128, 128)",
              head_size, head_dim_v);
}
