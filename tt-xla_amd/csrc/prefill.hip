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

namespace ttpa {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

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

template <int D, int HPW>
__global__ __launch_bounds__(256, (D <= 128 ? 2 : 1)) void prefill_kernel(PrefillArgs a) {
  constexpr int RPW = 4 / HPW;            // row blocks per workgroup
  constexpr int KSTEPS = D / 16;          // MFMA k-steps over the head dimension
  constexpr int DBLK = D / 32;            // 32-wide output blocks over the head dimension
  constexpr int CPT = D / 32;             // 16-byte chunks per thread per tile and tensor
  using L = Lds<D>;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t *ks = smem;
  uint16_t *vs = smem + kKeysPerTile * L::KS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int nqt = (a.sq + kRowsPerWave * RPW - 1) / (kRowsPerWave * RPW);
  const int qt = nqt - 1 - (int)blockIdx.x;  // heavy (late) tiles are scheduled first
  const int groups = a.hq / HPW;
  const int b = blockIdx.y / groups;
  const int hq0 = (blockIdx.y - b * groups) * HPW;
  const int g = a.hq / a.hkv;
  const int hk = hq0 / g;
  const int hq = hq0 + wave % HPW;
  const int row0 = (qt * RPW + wave / HPW) * kRowsPerWave;  // first query row of the wave
  const int offset = a.causal ? (a.chunk_start ? a.chunk_start[0] : 0) : 0;

  // keys this workgroup / this wavefront can see
  const int wg_last_row = min(a.sq, (qt + 1) * kRowsPerWave * RPW) - 1;
  const int kv_end_wg = a.causal ? min(a.skv, offset + wg_last_row + 1) : a.skv;
  const int ntiles = (kv_end_wg + kKeysPerTile - 1) / kKeysPerTile;
  const int wave_last_key = a.causal ? offset + min(a.sq - 1, row0 + kRowsPerWave - 1) : a.skv - 1;
  const bool wave_active = row0 < a.sq;

  // ---- Q fragments (B operand: lane n = query row, 8 head-dim elements per k-step) -----
  bf16x8 qf[KSTEPS];
  {
    const int qrow = min(row0 + n, a.sq - 1);
    const uint16_t *qp = a.q + b * a.q_bs + hq * a.q_hs + (int64_t)qrow * a.q_ts + 8 * h;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
      qf[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 16 * s));
  }

  floatx16 acc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- global -> register staging of one K/V tile -------------------------------------
  uint4 kst[CPT], vst[CPT];
  auto fetch_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int id = tid + 256 * i;
      const int key = id / (D / 8), c = id - key * (D / 8);
      const int kabs = kt * kKeysPerTile + key;
      if (kabs < a.skv) {
        kst[i] = *reinterpret_cast<const uint4 *>(kv_chunk(a, a.k, b, hk, kabs, c, D));
        vst[i] = *reinterpret_cast<const uint4 *>(kv_chunk(a, a.v, b, hk, kabs, c, D));
      } else {
        kst[i] = make_uint4(0, 0, 0, 0);
        vst[i] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto stage_tile = [&]() {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int id = tid + 256 * i;
      const int key = id / (D / 8), c = id - key * (D / 8);
      *reinterpret_cast<uint4 *>(ks + key * L::KS + c * 8) = kst[i];
      *reinterpret_cast<uint4 *>(vs + key * L::VS + c * 8) = vst[i];
    }
  };

  if (ntiles > 0) fetch_tile(0);
  for (int kt = 0; kt < ntiles; ++kt) {
    __syncthreads();  // every wavefront is done reading the previous tile
    stage_tile();
    __syncthreads();
    if (kt + 1 < ntiles) fetch_tile(kt + 1);  // in flight while this tile is consumed

    const int key0 = kt * kKeysPerTile;
    if (!wave_active || key0 > wave_last_key) continue;  // nothing visible to this wavefront

    // ---- S^T = K . Q^T for the two 32-key blocks of the tile ----------------------------
    floatx16 st[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) st[kb][r] = 0.f;
      const uint16_t *krow = ks + (32 * kb + n) * L::KS + 8 * h;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(krow + 16 * s));
        st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], st[kb], 0, 0, 0);
      }
    }

    // ---- mask, online softmax (one query row per lane) -----------------------------------
    // The softmax scale is positive, so the running maximum is tracked on raw scores and
    // the scale is folded into the exponent: p = exp2(s * c - m * c).
    const int qrow = row0 + n;
    const bool need_mask = (a.causal && key0 + kKeysPerTile - 1 > offset + row0) ||
                           key0 + kKeysPerTile > a.skv || a.mask != nullptr;
    if (need_mask) {  // wavefront-uniform: only diagonal / ragged / explicitly masked tiles
      const int limit = a.causal ? min(offset + qrow, a.skv - 1) : a.skv - 1;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * h + (r & 3);
          float v = st[kb][r];
          if (a.mask) {
            const int kc = min(key, a.skv - 1), qc = min(qrow, a.sq - 1);
            // additive mask is in natural-log units of the scaled score
            v += bf16_lo(a.mask[b * a.mask_bs + (int64_t)qc * a.mask_rs + kc]) *
                 (1.4426950408889634f / a.scale_log2e);
          }
          st[kb][r] = key > limit ? -INFINITY : v;
        }
    }
    float mloc = fmaxf(st[0][0], st[1][0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(st[0][r], st[1][r]));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    const float m_new = fmaxf(m_run, mloc);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_safe) * a.scale_log2e);
    const float mc = m_safe * a.scale_log2e;
    m_run = m_new;
    float lsum = 0.f;
    bf16x8 pf[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          // B-operand element e of k-step s <-> accumulator register 8 s + e
          float p = __builtin_amdgcn_exp2f(fmaf(st[kb][8 * s + e], a.scale_log2e, -mc));
          lsum += p;
          pf[kb][s][e] = (__bf16)p;
        }
    l_run = l_run * alpha + lsum;
    // skip the accumulator rescale when no row of the wavefront moved its maximum
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= alpha;
    }

    // ---- O^T += V^T . P^T ------------------------------------------------------------------
    // transposing LDS load, per group of 16 lanes: lane i receives element (i % 4) of the
    // 8-byte chunks addressed by lanes 4 j + i / 4 (j = 0..3).  Lane a of a group therefore
    // points at key (a / 4) of the wanted four and at head-dim chunk 4 (a % 4) of the 16
    // columns the group covers.
    const int grp = lane >> 4, a16 = lane & 15;
    const uint16_t *vbase =
        vs + (4 * (grp >> 1) + (a16 >> 2)) * L::VS + 16 * (grp & 1) + 4 * (a16 & 3);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const uint16_t *vk = vbase + (32 * kb + 16 * s) * L::VS;
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          typedef __attribute__((address_space(3))) shortx4 *lds_v4;
          shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 32 * db));
          shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 8 * L::VS + 32 * db));
          bf16x8 vf;
          bf16x4 l4 = __builtin_bit_cast(bf16x4, lo), h4 = __builtin_bit_cast(bf16x4, hi);
          vf[0] = l4[0], vf[1] = l4[1], vf[2] = l4[2], vf[3] = l4[3];
          vf[4] = h4[0], vf[5] = h4[1], vf[6] = h4[2], vf[7] = h4[3];
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kb][s], acc[db], 0, 0, 0);
        }
      }
  }

  // ---- normalise and store: lane (n, h) holds head-dim elements 32 db + 8 j + 4 h + i ----
  if (!wave_active) return;
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  const int qrow = row0 + n;
  if (qrow >= a.sq) return;
  uint16_t *op = a.out + b * a.out_bs + hq * a.out_hs + (int64_t)qrow * a.out_ts + 4 * h;
#pragma unroll
  for (int db = 0; db < DBLK; ++db)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t lo = f32_to_bf16_bits(acc[db][4 * j] * inv) |
                    (f32_to_bf16_bits(acc[db][4 * j + 1] * inv) << 16);
      uint32_t hi = f32_to_bf16_bits(acc[db][4 * j + 2] * inv) |
                    (f32_to_bf16_bits(acc[db][4 * j + 3] * inv) << 16);
      *reinterpret_cast<uint2 *>(op + 32 * db + 8 * j) = make_uint2(lo, hi);
    }
}

template <int D, int HPW>
int launch(const PrefillArgs &a, hipStream_t st) {
  constexpr int RPW = 4 / HPW;
  const int nqt = (a.sq + kRowsPerWave * RPW - 1) / (kRowsPerWave * RPW);
  const size_t lds = Lds<D>::BYTES;
  static bool attr_set = false;
  if (!attr_set && lds > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_kernel<D, HPW>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return fail(TTPA_ERR_LAUNCH, "prefill: cannot reserve %zu bytes of LDS", lds);
    attr_set = true;
  }
  hipEvent_t ev0, ev1;
  take_profile_events(ev0, ev1);
  if (ev0) (void)hipEventRecord(ev0, st);
  prefill_kernel<D, HPW><<<dim3(nqt, a.batch * (a.hq / HPW)), dim3(256), lds, st>>>(a);
  if (ev1) (void)hipEventRecord(ev1, st);
  return check_launch("sdpa_prefill");
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
