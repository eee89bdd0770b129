// Prefill attention (dense and paged / chunked) on bf16 MFMA tiles, gfx950.
//
// One workgroup = 4 wavefronts that share every K/V tile in LDS.  A wavefront owns a
// block of 32 query rows of one query head; the 4 wavefronts are HPW heads of the same
// KV head times 4 / HPW consecutive row blocks, so with grouped heads a K/V tile is
// fetched once for up to 4 query heads.
//
// Per 64-key tile a wavefront computes, with v_mfma_f32_32x32x16_bf16:
//   S^T[key, row] = K[key, :] . Q[row, :]      A = K tile rows (LDS), B = Q (registers)
//   O^T[d, row]  += V^T[d, key] . P^T[key, row] A = V tile read through the transposing
//                                               LDS load, B = P^T (registers)
// Computing the TRANSPOSED score tile puts one query row in each lane's accumulator
// column: the online-softmax statistics of a row are plain per-lane scalars (one
// exchange between the two lane halves per tile), and the probabilities a lane holds are
// exactly the B-operand fragment the second product needs, so P never moves between
// lanes or through LDS.
//
// Accumulator layout of a 32x32 tile (lane = 32 h + n): register r holds
// element (row 8 (r / 4) + 4 h + r % 4, column n).
#include "common.h"

#include <cstdlib>

namespace ttpa {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kKeysPerTile = 64;
constexpr int kRowsPerWave = 32;

struct PrefillArgs {
  uint16_t *out;
  int64_t out_bs, out_hs, out_ts;
  const uint16_t *q;
  int64_t q_bs, q_hs, q_ts;
  const uint16_t *k, *v;
  int64_t kv_bs, kv_hs, kv_ts;  // dense form
  const int32_t *pt;            // paged form when non-null
  int64_t pt_rs;
  const int32_t *chunk_start;
  const uint16_t *mask;
  int64_t mask_bs, mask_rs;
  int batch, hq, hkv, sq, skv, bs, w, nb, causal;
  float scale_log2e;
};

template <int D>
struct Lds {
  // K rows: 16-byte fragments read by 32 lanes of consecutive rows -> row stride = 4 banks
  // (mod 64); V rows: four consecutive rows read 64 bytes each -> row stride = 16 banks.
  static constexpr int KS = D + 8;    // elements per K row   (D=128: 68 dwords)
  static constexpr int VS = D + 32;   // elements per V row   (D=128: 80 dwords)
  static constexpr int BYTES = kKeysPerTile * (KS + VS) * 2;
};

// Address of the 8-element chunk `c` of key `key` (absolute position) for (batch b, kv head).
__device__ __forceinline__ const uint16_t *kv_chunk(const PrefillArgs &a, const uint16_t *base,
                                                    int b, int hk, int key, int c, int d) {
  if (a.pt) {
    int col = key / a.bs;
    int phys = a.pt[(int64_t)b * a.pt_rs + col];
    if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
    return base + (((int64_t)phys * a.hkv + hk) * a.bs + (key - col * a.bs)) * d + c * 8;
  }
  return base + b * a.kv_bs + hk * a.kv_hs + (int64_t)key * a.kv_ts + c * 8;
}

// MODE 0: dense K/V; 1: paged, block_size a multiple of 64 (a tile lies in one block);
// 2: paged, any block size (per-chunk table lookups).
// R = blocks of 32 query rows per wavefront.  R = 2 reuses every K / V fragment read from
// LDS for two matrix instructions (LDS operand traffic per FLOP halves) and gives the
// scheduler two independent row blocks to overlap: the score product of block 1 runs on the
// matrix pipe while block 0's softmax runs on the VALU.  It needs the 512-register budget
// (one workgroup per CU); R = 1 keeps two workgroups per CU and serves short queries.
template <int D, int HPW, int MODE, int R>
__global__ __launch_bounds__(256, (D <= 128 && R == 1 ? 2 : 1)) void prefill_kernel(PrefillArgs a) {
  constexpr int RPW = 4 / HPW;            // wavefront row slots per workgroup
  constexpr int ROWS = kRowsPerWave * R;  // query rows per wavefront
  constexpr int KSTEPS = D / 16;          // MFMA k-steps over the head dimension
  constexpr int DBLK = D / 32;            // 32-wide output blocks over the head dimension
  constexpr int CPT = D / 32;             // 16-byte chunks per thread per tile and tensor
  using L = Lds<D>;
  constexpr int STAGE = kKeysPerTile * (L::KS + L::VS);  // elements per LDS stage
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int nqt = (a.sq + ROWS * RPW - 1) / (ROWS * RPW);
  const int qt = nqt - 1 - (int)blockIdx.x;  // heavy (late) tiles are scheduled first
  const int groups = a.hq / HPW;
  const int b = blockIdx.y / groups;
  const int hq0 = (blockIdx.y - b * groups) * HPW;
  const int g = a.hq / a.hkv;
  const int hk = hq0 / g;
  const int hq = hq0 + wave % HPW;
  const int row0 = (qt * RPW + wave / HPW) * ROWS;  // first query row of the wavefront
  const int offset = a.causal ? (a.chunk_start ? a.chunk_start[0] : 0) : 0;

  // keys this workgroup / this wavefront can see
  const int wg_last_row = min(a.sq, (qt + 1) * ROWS * RPW) - 1;
  const int kv_end_wg = a.causal ? min(a.skv, offset + wg_last_row + 1) : a.skv;
  const int ntiles = (kv_end_wg + kKeysPerTile - 1) / kKeysPerTile;
  const int wave_last_key = a.causal ? offset + min(a.sq - 1, row0 + ROWS - 1) : a.skv - 1;
  const bool wave_active = row0 < a.sq;

  // ---- Q fragments (B operand: lane n = query row, 8 head-dim elements per k-step) -----
  bf16x8 qf[R][KSTEPS];
#pragma unroll
  for (int rb = 0; rb < R; ++rb) {
    const int qrow = min(row0 + 32 * rb + n, a.sq - 1);
    const uint16_t *qp = a.q + b * a.q_bs + hq * a.q_hs + (int64_t)qrow * a.q_ts + 8 * h;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
      qf[rb][s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 16 * s));
  }

  floatx16 acc[R][DBLK];
  float m_run[R], l_run[R];
#pragma unroll
  for (int rb = 0; rb < R; ++rb) {
    m_run[rb] = -INFINITY;
    l_run[rb] = 0.f;
#pragma unroll
    for (int i = 0; i < DBLK; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][i][r] = 0.f;
  }

  // ---- global -> register staging of one K/V tile -------------------------------------
  // A thread's chunks sit at fixed (key, column) positions of every tile: their offsets are
  // computed once, and per tile only a wavefront-uniform base moves (modes 0 and 1).
  u32x4 kst[CPT], vst[CPT];  // native vectors: struct-typed uint4 arrays end up in scratch memory
  uint32_t chunk_off[CPT];  // element offset of chunk i inside a tile
  int chunk_key[CPT], chunk_col[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int id = tid + 256 * i;
    const int key = id / (D / 8), c = id - key * (D / 8);
    chunk_key[i] = key;
    chunk_col[i] = c;
    chunk_off[i] = (uint32_t)(key * (MODE == 0 ? (int)a.kv_ts : D) + c * 8);
  }
  // Loads are unconditional (a predicated load would make the compiler wait for the prefetch
  // right after issuing it): keys past the end of a dense K/V are clamped to the last row,
  // whose scores are masked and whose V rows therefore carry weight 0.
  auto fetch_tile = [&](int kt) {
    const int key0 = kt * kKeysPerTile;
    int64_t base;  // uniform element offset of the tile
    if constexpr (MODE == 0) {
      base = b * a.kv_bs + hk * a.kv_hs + (int64_t)key0 * a.kv_ts;
    } else if constexpr (MODE == 1) {
      int phys = __builtin_amdgcn_readfirstlane(a.pt[(int64_t)b * a.pt_rs + key0 / a.bs]);
      if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
      base = (((int64_t)phys * a.hkv + hk) * a.bs + (key0 % a.bs)) * D;
    } else {
      base = 0;
    }
    const int last = a.skv - 1 - key0;  // last valid key of this tile, relative (>= 0)
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      if constexpr (MODE == 2) {
        const int key = key0 + min(chunk_key[i], last);
        kst[i] = *reinterpret_cast<const u32x4 *>(kv_chunk(a, a.k, b, hk, key, chunk_col[i], D));
        vst[i] = *reinterpret_cast<const u32x4 *>(kv_chunk(a, a.v, b, hk, key, chunk_col[i], D));
      } else if constexpr (MODE == 1) {  // table_width * block_size is a multiple of the tile
        kst[i] = *reinterpret_cast<const u32x4 *>(a.k + base + chunk_off[i]);
        vst[i] = *reinterpret_cast<const u32x4 *>(a.v + base + chunk_off[i]);
      } else {
        const uint32_t off = (uint32_t)(min(chunk_key[i], last) * (int)a.kv_ts + chunk_col[i] * 8);
        kst[i] = *reinterpret_cast<const u32x4 *>(a.k + base + off);
        vst[i] = *reinterpret_cast<const u32x4 *>(a.v + base + off);
      }
    }
  };
  auto stage_tile = [&](int buf) {
    uint16_t *ks = smem + buf * STAGE;
    uint16_t *vs = ks + kKeysPerTile * L::KS;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      *reinterpret_cast<u32x4 *>(ks + chunk_key[i] * L::KS + chunk_col[i] * 8) = kst[i];
      *reinterpret_cast<u32x4 *>(vs + chunk_key[i] * L::VS + chunk_col[i] * 8) = vst[i];
    }
  };

  // Pipeline: LDS holds two stages.  While tile kt is consumed from stage kt & 1, tile kt + 1
  // (fetched one iteration ago) is written to the other stage and tile kt + 2 is in flight
  // from global memory.  One barrier per tile.  Staging and prefetch are unconditional (past
  // the last tile they repeat it into a stage nobody reads): straight-line code keeps the
  // staged tile in registers and the wait counters exact.  ntiles >= 1 always (row 0 sees
  // key 0).
  const int last_tile = ntiles - 1;
  fetch_tile(0);
  stage_tile(0);
  fetch_tile(min(1, last_tile));
  __syncthreads();
  for (int kt = 0; kt < ntiles; ++kt) {
    stage_tile((kt + 1) & 1);
    fetch_tile(min(kt + 2, last_tile));
    const uint16_t *ks = smem + (kt & 1) * STAGE;
    const uint16_t *vs = ks + kKeysPerTile * L::KS;
    const int key0 = kt * kKeysPerTile;

    if (wave_active && key0 <= wave_last_key) {
      // ---- K fragments: read once, used for every row block ------------------------------
      bf16x8 kf[2][KSTEPS];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const uint16_t *krow = ks + (32 * kb + n) * L::KS + 8 * h;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          kf[kb][s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(krow + 16 * s));
      }
      // ---- S^T = K . Q^T, row block after row block ------------------------------------------
      floatx16 st[R][2];
#pragma unroll
      for (int rb = 0; rb < R; ++rb)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) st[rb][kb][r] = 0.f;
#pragma unroll
          for (int s = 0; s < KSTEPS; ++s)
            st[rb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb][s], qf[rb][s], st[rb][kb], 0, 0, 0);
        }
      bf16x8 pf[R][2][2];
#pragma unroll
      for (int rb = 0; rb < R; ++rb) {
        // ---- mask, online softmax (one query row per lane) -----------------------------------
        // The softmax scale is positive, so the running maximum is tracked on raw scores and
        // the scale is folded into the exponent: p = exp2(s * c - m * c).
        const int rrow0 = row0 + 32 * rb;
        const int qrow = rrow0 + n;
        const bool need_mask = (a.causal && key0 + kKeysPerTile - 1 > offset + rrow0) ||
                               key0 + kKeysPerTile > a.skv || a.mask != nullptr;
        if (need_mask) {  // wavefront-uniform: only diagonal / ragged / explicitly masked tiles
          const int limit = a.causal ? min(offset + qrow, a.skv - 1) : a.skv - 1;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * h + (r & 3);
              float v = st[rb][kb][r];
              if (a.mask) {
                const int kc = min(key, a.skv - 1), qc = min(qrow, a.sq - 1);
                // additive mask is in natural-log units of the scaled score
                v += bf16_lo(a.mask[b * a.mask_bs + (int64_t)qc * a.mask_rs + kc]) *
                     (1.4426950408889634f / a.scale_log2e);
              }
              st[rb][kb][r] = key > limit ? -INFINITY : v;
            }
        }
        float mloc = fmaxf(st[rb][0][0], st[rb][1][0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(st[rb][0][r], st[rb][1][r]));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        // Lazy rescaling: the running maximum only moves when a row's new maximum exceeds it
        // by more than 2^8 in the exponent domain.  Until then probabilities are taken
        // relative to the stale maximum (they may reach 2^8, harmless in bf16 / fp32), the
        // accumulators need no rescale, and the final division by the row sum is unchanged.
        const float kLazy = 8.0f;
        const bool move = !((mloc - m_run[rb]) * a.scale_log2e <= kLazy);  // also true from -inf
        const float m_new = move ? mloc : m_run[rb];
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = move ? __builtin_amdgcn_exp2f((m_run[rb] - m_safe) * a.scale_log2e) : 1.0f;
        const float mc = m_safe * a.scale_log2e;
        m_run[rb] = m_new;
        float lsum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              // B-operand element e of k-step s <-> accumulator register 8 s + e
              float p = __builtin_amdgcn_exp2f(fmaf(st[rb][kb][8 * s + e], a.scale_log2e, -mc));
              lsum += p;
              pf[rb][kb][s][e] = (__bf16)p;
            }
        l_run[rb] = l_run[rb] * alpha + lsum;
        // skip the accumulator rescale when no row of the wavefront moved its maximum
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int i = 0; i < DBLK; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][i][r] *= alpha;
        }
      }
      // ---- O^T += V^T . P^T: V^T fragments come through the transposing LDS load (per group
      //      of 16 lanes, lane i receives element i % 4 of the 8-byte chunks addressed by lanes
      //      4 j + i / 4); each fragment feeds every row block -------------------------------
      {
        const int grp = lane >> 4, a16 = lane & 15;
        const uint16_t *vbase =
            vs + (4 * (grp >> 1) + (a16 >> 2)) * L::VS + 16 * (grp & 1) + 4 * (a16 & 3);
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {
          bf16x8 vf[DBLK];
#pragma unroll
          for (int db = 0; db < DBLK; ++db) {
            typedef __attribute__((address_space(3))) shortx4 *lds_v4;
            const uint16_t *vk = vbase + 16 * k4 * L::VS + 32 * db;
            shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk));
            shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 8 * L::VS));
            bf16x4 l4 = __builtin_bit_cast(bf16x4, lo), h4 = __builtin_bit_cast(bf16x4, hi);
            bf16x8 t;
            t[0] = l4[0], t[1] = l4[1], t[2] = l4[2], t[3] = l4[3];
            t[4] = h4[0], t[5] = h4[1], t[6] = h4[2], t[7] = h4[3];
            vf[db] = t;
          }
#pragma unroll
          for (int rb = 0; rb < R; ++rb)
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
              acc[rb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db], pf[rb][k4 >> 1][k4 & 1],
                                                                    acc[rb][db], 0, 0, 0);
        }
      }
    }
    __syncthreads();  // tile kt + 1 is staged; everyone is done with stage kt & 1
  }

  // ---- normalise and store: lane (n, h) holds head-dim elements 32 db + 8 j + 4 h + i ----
  if (!wave_active) return;
#pragma unroll
  for (int rb = 0; rb < R; ++rb) {
    const float l_tot = l_run[rb] + __shfl_xor(l_run[rb], 32);
    const float inv = 1.0f / l_tot;
    const int qrow = row0 + 32 * rb + n;
    if (qrow >= a.sq) continue;
    uint16_t *op = a.out + b * a.out_bs + hq * a.out_hs + (int64_t)qrow * a.out_ts + 4 * h;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t lo = f32_to_bf16_bits(acc[rb][db][4 * j] * inv) |
                      (f32_to_bf16_bits(acc[rb][db][4 * j + 1] * inv) << 16);
        uint32_t hi = f32_to_bf16_bits(acc[rb][db][4 * j + 2] * inv) |
                      (f32_to_bf16_bits(acc[rb][db][4 * j + 3] * inv) << 16);
        *reinterpret_cast<uint2 *>(op + 32 * db + 8 * j) = make_uint2(lo, hi);
      }
  }
}

template <int D, int HPW, int MODE, int R>
int launch_mode(const PrefillArgs &a, hipStream_t st) {
  constexpr int RPW = 4 / HPW;
  constexpr int ROWS = kRowsPerWave * R;
  const int nqt = (a.sq + ROWS * RPW - 1) / (ROWS * RPW);
  const size_t lds = 2 * Lds<D>::BYTES;  // two stages
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_kernel<D, HPW, MODE, R>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return fail(TTPA_ERR_LAUNCH, "prefill: cannot reserve %zu bytes of LDS", lds);
    attr_set = true;
  }
  hipEvent_t ev0, ev1;
  take_profile_events(ev0, ev1);
  if (ev0) (void)hipEventRecord(ev0, st);
  prefill_kernel<D, HPW, MODE, R><<<dim3(nqt, a.batch * (a.hq / HPW)), dim3(256), lds, st>>>(a);
  if (ev1) (void)hipEventRecord(ev1, st);
  return check_launch("sdpa_prefill");
}

template <int D, int HPW, int MODE>
int launch_rows(const PrefillArgs &a, hipStream_t st) {
  // 64 rows per wavefront once the query is long enough to fill them; head size 256 keeps
  // 32 (its accumulators alone take 128 registers per row block)
  if constexpr (D <= 128) {
    static int forced = -1;
    if (forced < 0) {
      const char *e = getenv("TTPA_PREFILL_ROWS");
      forced = e ? atoi(e) : 0;
    }
    const bool two = forced == 64;  // 64 rows per wavefront is experimental (TTPA_PREFILL_ROWS=64)
    if (two) return launch_mode<D, HPW, MODE, 2>(a, st);
  }
  return launch_mode<D, HPW, MODE, 1>(a, st);
}

template <int D, int HPW>
int launch(const PrefillArgs &a, hipStream_t st) {
  if (!a.pt) return launch_rows<D, HPW, 0>(a, st);
  if (a.bs % kKeysPerTile == 0) return launch_rows<D, HPW, 1>(a, st);
  return launch_rows<D, HPW, 2>(a, st);
}

template <int D>
int launch_d(const PrefillArgs &a, hipStream_t st) {
  const int g = a.hq / a.hkv;
  if (g % 4 == 0) return launch<D, 4>(a, st);
  if (g % 2 == 0) return launch<D, 2>(a, st);
  return launch<D, 1>(a, st);
}

}  // namespace
}  // namespace ttpa

using namespace ttpa;

extern "C" int ttpa_sdpa_prefill(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                                 int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                                 int64_t q_head_stride, int64_t q_token_stride, const void *k,
                                 const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                                 int64_t kv_token_stride, const int32_t *page_table,
                                 int64_t page_table_row_stride, const int32_t *chunk_start,
                                 const void *mask, int64_t mask_batch_stride,
                                 int64_t mask_row_stride, int32_t batch, int32_t q_heads,
                                 int32_t kv_heads, int32_t q_len, int32_t kv_len, int32_t head_size,
                                 int32_t block_size, int32_t table_width, int32_t num_blocks,
                                 int32_t causal, float scale, void *stream) {
  TTPA_REQUIRE(out && q && k && v, "null pointer argument");
  TTPA_REQUIRE(batch > 0 && q_heads > 0 && kv_heads > 0 && q_len > 0 && head_size > 0,
               "non-positive dimension");
  TTPA_REQUIRE(q_heads % kv_heads == 0, "q_heads %d not divisible by kv_heads %d", q_heads,
               kv_heads);
  if (head_size != 64 && head_size != 128 && head_size != 256)
    return fail(TTPA_ERR_UNSUPPORTED, "prefill: head_size %d; supported 64, 128, 256", head_size);
  TTPA_REQUIRE(!(mask && causal), "an additive mask excludes causal masking");
  if (page_table) {
    TTPA_REQUIRE(block_size > 0 && table_width > 0 && num_blocks > 0,
                 "paged form needs block_size, table_width and num_blocks");
    kv_len = table_width * block_size;
  } else {
    TTPA_REQUIRE(kv_len > 0, "dense form needs kv_len > 0");
    TTPA_REQUIRE(kv_batch_stride % 8 == 0 && kv_head_stride % 8 == 0 && kv_token_stride % 8 == 0,
                 "prefill: k / v strides must be multiples of 8 elements");
    TTPA_REQUIRE(chunk_start == nullptr, "chunk_start applies to the paged form only");
  }
  TTPA_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out),
               "prefill: q / k / v / out must be 16-byte aligned");
  TTPA_REQUIRE(q_batch_stride % 8 == 0 && q_head_stride % 8 == 0 && q_token_stride % 8 == 0 &&
                   out_batch_stride % 4 == 0 && out_head_stride % 4 == 0 && out_token_stride % 4 == 0,
               "prefill: q strides must be multiples of 8 elements, out strides of 4");
  TTPA_REQUIRE((int64_t)batch * q_heads < 65536, "prefill: batch * heads too large for one launch");

  PrefillArgs a;
  a.out = static_cast<uint16_t *>(out);
  a.out_bs = out_batch_stride, a.out_hs = out_head_stride, a.out_ts = out_token_stride;
  a.q = static_cast<const uint16_t *>(q);
  a.q_bs = q_batch_stride, a.q_hs = q_head_stride, a.q_ts = q_token_stride;
  a.k = static_cast<const uint16_t *>(k);
  a.v = static_cast<const uint16_t *>(v);
  a.kv_bs = kv_batch_stride, a.kv_hs = kv_head_stride, a.kv_ts = kv_token_stride;
  a.pt = page_table, a.pt_rs = page_table_row_stride;
  a.chunk_start = chunk_start;
  a.mask = static_cast<const uint16_t *>(mask);
  a.mask_bs = mask_batch_stride, a.mask_rs = mask_row_stride;
  a.batch = batch, a.hq = q_heads, a.hkv = kv_heads, a.sq = q_len, a.skv = kv_len;
  a.bs = block_size, a.w = table_width, a.nb = num_blocks, a.causal = causal ? 1 : 0;
  a.scale_log2e = scale * 1.4426950408889634f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (head_size) {
    case 64: return launch_d<64>(a, st);
    case 128: return launch_d<128>(a, st);
    default: return launch_d<256>(a, st);
  }
}
