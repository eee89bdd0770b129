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

extern "C" size_t ttpa_paged_mla_decode_workspace_bytes(int32_t users, int32_t q_heads, int32_t kv_heads,
                                                        int32_t head_dim_v) {
  if (users <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim_v <= 0 || q_heads % kv_heads) return 0;
  int32_t nhb, gseg;
  if (wide_geometry(q_heads, kv_heads, nhb, gseg) != TTPA_OK) return 0;
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  const size_t segs = (size_t)users * kv_heads * nhb;
  const size_t slot = (size_t)slot_floats_for(gseg, head_dim_v) * sizeof(float);
  return header_bytes(users, kv_heads * nhb) + ((size_t)cus + segs) * slot;
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
  WideArgs w;
  w.nkv = kv_heads, w.nhb = nhb, w.gseg = gseg, w.dv = head_dim_v, w.n_slices = head_dim_v / dvw;

  hipStream_t st = static_cast<hipStream_t>(stream);
  hipEvent_t ev0, ev1;
  take_profile_events(ev0, ev1);
  if (ev0) (void)hipEventRecord(ev0, st);
  bool ok = false, built = true;
  const bool shared = v_cache == nullptr;
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
  decode_combine_kernel<<<dim3(users * kv_heads * nhb), dim3(256), 0, st>>>(a, gseg, head_dim_v);
  return check_launch("paged_mla_decode");
}
