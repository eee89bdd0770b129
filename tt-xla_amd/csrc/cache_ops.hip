// Paged KV-cache writes: single-token scatter (decode) and block-wise fill (prefill).
//
// Both are pure data movement and HBM / latency bound.  One thread moves one 16-byte
// chunk (8 bfloat16) of a head row, so a [head_size] row is written by head_size/8
// adjacent lanes as one contiguous burst; the page-table lookup is per row.
// The block-float-8 variants let one thread own one 16-element group: it reads 32
// bytes, encodes, and stores 16 element bytes + 1 exponent byte.
#include "common.h"

namespace ttpa {
namespace {

struct UpdateArgs {
  void *cache;
  const uint16_t *fill;
  void *cache2;           // second (V) cache and fill when both are written in one launch
  const uint16_t *fill2;
  int64_t fill_us, fill_hs;
  const void *idx;
  int idx_i64;
  const int32_t *pt;
  int64_t pt_rs;
  int users, hkv, bs, d, w, nb;
};

// Resolves (user) -> (physical block, row offset); false = skip this user.
__device__ __forceinline__ bool resolve_update(const UpdateArgs &a, int u, int &phys, int &off) {
  int64_t pos = load_index(a.idx, a.idx_i64, u);
  int64_t col = pos / a.bs;
  int64_t rem = pos - col * a.bs;
  if (rem < 0) {  // floor semantics for negative positions
    rem += a.bs;
    col -= 1;
  }
  if (col < 0) col += a.w;  // a negative column indexes from the end, once
  if (col < 0 || col >= a.w) return false;
  phys = a.pt[(int64_t)u * a.pt_rs + col];
  off = (int)rem;
  return (unsigned)phys < (unsigned)a.nb;
}

template <int VEC>  // VEC = 8 (16-byte chunks) or 1 (element-wise, unaligned operands)
__global__ __launch_bounds__(256) void update_bf16_kernel(UpdateArgs a) {
  const int cpr = a.d / VEC;
  int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t row = gid / cpr;
  int chunk = (int)(gid - row * cpr);
  if (row >= (int64_t)a.users * a.hkv) return;
  int u = (int)(row / a.hkv), h = (int)(row % a.hkv);
  int phys, off;
  if (!resolve_update(a, u, phys, off)) return;
  const uint16_t *src = a.fill + u * a.fill_us + h * a.fill_hs + chunk * VEC;
  uint16_t *dst = static_cast<uint16_t *>(a.cache) +
                  (((int64_t)phys * a.hkv + h) * a.bs + off) * a.d + chunk * VEC;
  if constexpr (VEC == 8) {
    *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
  } else {
    *dst = *src;
  }
  if (a.cache2) {
    const int64_t so = src - a.fill, dof = dst - static_cast<uint16_t *>(a.cache);
    if constexpr (VEC == 8) {
      *reinterpret_cast<uint4 *>(static_cast<uint16_t *>(a.cache2) + dof) =
          *reinterpret_cast<const uint4 *>(a.fill2 + so);
    } else {
      static_cast<uint16_t *>(a.cache2)[dof] = a.fill2[so];
    }
  }
}

__device__ __forceinline__ void update_bfp8_row(void *cache, const uint16_t *fill, const UpdateArgs &a,
                                                int u, int h, int grp, int phys, int off) {
  const int gpr = a.d / 16;
  const uint4 *src = reinterpret_cast<const uint4 *>(fill + u * a.fill_us + h * a.fill_hs + grp * 16);
  uint4 lo = src[0], hi = src[1];
  uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  uint32_t bytes[4];
  uint32_t e = bfp8_encode16(w, bytes);
  uint8_t *slab = static_cast<uint8_t *>(cache) +
                  ((int64_t)phys * a.hkv + h) * (int64_t)(a.bs + a.bs / 16) * a.d;
  *reinterpret_cast<uint4 *>(slab + (int64_t)off * a.d + grp * 16) =
      make_uint4(bytes[0], bytes[1], bytes[2], bytes[3]);
  slab[(int64_t)a.bs * a.d + (int64_t)off * gpr + grp] = (uint8_t)e;
}

__global__ __launch_bounds__(256) void update_bfp8_kernel(UpdateArgs a) {
  const int gpr = a.d / 16;  // groups per row
  int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t row = gid / gpr;
  int grp = (int)(gid - row * gpr);
  if (row >= (int64_t)a.users * a.hkv) return;
  int u = (int)(row / a.hkv), h = (int)(row % a.hkv);
  int phys, off;
  if (!resolve_update(a, u, phys, off)) return;
  update_bfp8_row(a.cache, a.fill, a, u, h, grp, phys, off);
  if (a.cache2) update_bfp8_row(a.cache2, a.fill2, a, u, h, grp, phys, off);
}

struct FillArgs {
  void *cache;
  const uint16_t *fill;
  // a second (cache, fill) pair written by the same launch (K and V of a prefill), or null:
  // grid z = fill rows of the first pair, then those of the second
  void *cache2;
  const uint16_t *fill2;
  int64_t fill_us, fill_hs, fill_ts;
  const int32_t *pt;
  int64_t pt_rs;
  const void *bidx;
  int bidx_i64;
  int fill_users, table_rows, hkv, s, bs, d, w, nb;
  // floor(2^32 / divisor) + 1 for the two per-thread divisions (by the threads of a token row
  // and by the block size), or 0 where the multiply-high quotient would not be exact
  uint32_t tpr_magic, bs_magic;
};

// x / d; a thread moves 16 bytes, so a division sequence (about 30 instructions) per quotient
// would make these kernels instruction-bound.
__device__ __forceinline__ int fast_div(int x, int d, uint32_t magic) {
  return magic ? (int)__umulhi((uint32_t)x, magic) : x / d;
}
inline uint32_t magic_for(int64_t max_dividend, int d) {
  return (d >= 2 && max_dividend * d < (1ll << 32)) ? (uint32_t)((1ull << 32) / (uint32_t)d) + 1u : 0u;
}

// Block of token t of fill row i, and the token's row inside it.
__device__ __forceinline__ bool resolve_fill(const FillArgs &a, int i, int t, int &phys, int &off) {
  int64_t b = a.bidx ? load_index(a.bidx, a.bidx_i64, i) : 0;
  if (b < 0 || b >= a.table_rows) return false;
  const int col = fast_div(t, a.bs, a.bs_magic);
  off = t - col * a.bs;
  phys = a.pt[b * a.pt_rs + col];
  return (unsigned)phys < (unsigned)a.nb;
}

// Grid: x over the (token, chunk) pairs of one (user, head), chunk fastest; y = KV head;
// z = fill row.  One (user, head, block) destination slab of bs * D elements is written front
// to back by neighbouring wavefronts while the source is read in whole 2*D-byte rows.
template <int VEC>
__global__ __launch_bounds__(256) void fill_bf16_kernel(FillArgs a) {
  const int cpr = a.d / VEC;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.s * cpr) return;
  const int t = fast_div(idx, cpr, a.tpr_magic), chunk = idx - t * cpr;
  const bool second = (int)blockIdx.z >= a.fill_users;
  const int h = blockIdx.y, i = (int)blockIdx.z - (second ? a.fill_users : 0);
  int phys, off;
  if (!resolve_fill(a, i, t, phys, off)) return;
  const uint16_t *src = (second ? a.fill2 : a.fill) + i * a.fill_us + h * a.fill_hs + t * a.fill_ts + chunk * VEC;
  uint16_t *dst = static_cast<uint16_t *>(second ? a.cache2 : a.cache) +
                  (((int64_t)phys * a.hkv + h) * a.bs + off) * a.d + chunk * VEC;
  if constexpr (VEC == 8) {
    *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
  } else {
    *dst = *src;
  }
}

__global__ __launch_bounds__(256) void fill_bfp8_kernel(FillArgs a) {
  const int gpr = a.d / 16;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.s * gpr) return;
  const int t = fast_div(idx, gpr, a.tpr_magic), grp = idx - t * gpr;
  const bool second = (int)blockIdx.z >= a.fill_users;
  const int h = blockIdx.y, i = (int)blockIdx.z - (second ? a.fill_users : 0);
  int phys, off;
  if (!resolve_fill(a, i, t, phys, off)) return;
  const uint4 *src = reinterpret_cast<const uint4 *>((second ? a.fill2 : a.fill) + i * a.fill_us +
                                                     h * a.fill_hs + t * a.fill_ts + grp * 16);
  uint4 lo = src[0], hi = src[1];
  uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  uint32_t bytes[4];
  uint32_t e = bfp8_encode16(w, bytes);
  uint8_t *slab = static_cast<uint8_t *>(second ? a.cache2 : a.cache) +
                  ((int64_t)phys * a.hkv + h) * (int64_t)(a.bs + a.bs / 16) * a.d;
  *reinterpret_cast<uint4 *>(slab + (int64_t)off * a.d + grp * 16) =
      make_uint4(bytes[0], bytes[1], bytes[2], bytes[3]);
  slab[(int64_t)a.bs * a.d + (int64_t)off * gpr + grp] = (uint8_t)e;
}

int common_checks(const void *cache, const void *fill, const int32_t *pt, int hkv, int bs, int d,
                  int w, int nb, int fmt) {
  TTPA_REQUIRE(cache && fill && pt, "null cache / fill / page_table pointer");
  TTPA_REQUIRE(hkv > 0 && bs > 0 && d > 0 && w > 0 && nb > 0,
               "non-positive dimension (kv_heads=%d block_size=%d head_size=%d width=%d blocks=%d)",
               hkv, bs, d, w, nb);
  TTPA_REQUIRE(fmt == TTPA_KV_BF16 || fmt == TTPA_KV_BFP8, "unknown kv_format %d", fmt);
  if (fmt == TTPA_KV_BFP8) {
    TTPA_REQUIRE(d % 16 == 0 && bs % 16 == 0,
                 "block-float-8 needs head_size and block_size to be multiples of 16");
  }
  return TTPA_OK;
}

}  // namespace
}  // namespace ttpa

using namespace ttpa;

static int launch_update(void *cache, void *cache2, const void *fill, const void *fill2,
                         int64_t fill_user_stride, int64_t fill_head_stride,
                         const void *update_indices, int indices_is_i64, const int32_t *page_table,
                         int64_t page_table_row_stride, int32_t users, int32_t kv_heads,
                         int32_t block_size, int32_t head_size, int32_t table_width,
                         int32_t num_blocks, int32_t kv_format, void *stream) {
  if (int rc = common_checks(cache, fill, page_table, kv_heads, block_size, head_size, table_width,
                             num_blocks, kv_format))
    return rc;
  TTPA_REQUIRE(update_indices, "null update_indices pointer");
  TTPA_REQUIRE(users >= 0, "negative user count");
  if (users == 0) return TTPA_OK;
  UpdateArgs a{cache,      static_cast<const uint16_t *>(fill),
               cache2,     static_cast<const uint16_t *>(fill2),
               fill_user_stride, fill_head_stride,
               update_indices,   indices_is_i64,
               page_table, page_table_row_stride,
               users,      kv_heads,
               block_size, head_size,
               table_width, num_blocks};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = head_size % 8 == 0 && aligned16(cache) && aligned16(fill) &&
                      (!cache2 || (aligned16(cache2) && aligned16(fill2))) &&
                      fill_user_stride % 8 == 0 && fill_head_stride % 8 == 0;
  if (kv_format == TTPA_KV_BFP8) {
    TTPA_REQUIRE(vec_ok, "block-float-8 update needs 16-byte aligned fill rows");
    int64_t threads = (int64_t)users * kv_heads * (head_size / 16);
    update_bfp8_kernel<<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st>>>(a);
  } else if (vec_ok) {
    int64_t threads = (int64_t)users * kv_heads * (head_size / 8);
    update_bf16_kernel<8><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st>>>(a);
  } else {
    int64_t threads = (int64_t)users * kv_heads * head_size;
    update_bf16_kernel<1><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st>>>(a);
  }
  return check_launch("paged_update_cache");
}

extern "C" int ttpa_paged_update_cache(void *cache, const void *fill, int64_t fill_user_stride,
                                       int64_t fill_head_stride, const void *update_indices,
                                       int indices_is_i64, const int32_t *page_table,
                                       int64_t page_table_row_stride, int32_t users,
                                       int32_t kv_heads, int32_t block_size, int32_t head_size,
                                       int32_t table_width, int32_t num_blocks, int32_t kv_format,
                                       void *stream) {
  return launch_update(cache, nullptr, fill, nullptr, fill_user_stride, fill_head_stride,
                       update_indices, indices_is_i64, page_table, page_table_row_stride, users,
                       kv_heads, block_size, head_size, table_width, num_blocks, kv_format, stream);
}

extern "C" int ttpa_paged_update_cache_kv(void *k_cache, void *v_cache, const void *k_fill,
                                          const void *v_fill, int64_t fill_user_stride,
                                          int64_t fill_head_stride, const void *update_indices,
                                          int indices_is_i64, const int32_t *page_table,
                                          int64_t page_table_row_stride, int32_t users,
                                          int32_t kv_heads, int32_t block_size, int32_t head_size,
                                          int32_t table_width, int32_t num_blocks,
                                          int32_t kv_format, void *stream) {
  TTPA_REQUIRE(v_cache && v_fill, "null V cache / fill pointer");
  return launch_update(k_cache, v_cache, k_fill, v_fill, fill_user_stride, fill_head_stride,
                       update_indices, indices_is_i64, page_table, page_table_row_stride, users,
                       kv_heads, block_size, head_size, table_width, num_blocks, kv_format, stream);
}

// cache2 / fill2 non-null: both pairs in one launch.
static int launch_fill(void *cache, void *cache2, const void *fill, const void *fill2,
                       int64_t fill_user_stride, int64_t fill_head_stride, int64_t fill_token_stride,
                       const int32_t *page_table, int64_t page_table_row_stride,
                       const void *batch_idx, int batch_idx_is_i64, int32_t fill_users,
                       int32_t table_rows, int32_t kv_heads, int32_t seq_len, int32_t block_size,
                       int32_t head_size, int32_t table_width, int32_t num_blocks, int32_t kv_format,
                       void *stream) {
  if (int rc = common_checks(cache, fill, page_table, kv_heads, block_size, head_size, table_width,
                             num_blocks, kv_format))
    return rc;
  TTPA_REQUIRE(fill_users >= 0 && seq_len >= 0 && table_rows > 0, "bad fill_users / seq_len / table_rows");
  TTPA_REQUIRE(batch_idx != nullptr || fill_users <= 1,
               "batch_idx may only be omitted for a single-user fill");
  TTPA_REQUIRE((int64_t)seq_len <= (int64_t)table_width * block_size,
               "seq_len %d does not fit %d page-table columns of %d tokens", seq_len, table_width,
               block_size);
  if (fill_users == 0 || seq_len == 0) return TTPA_OK;
  FillArgs a{cache,      static_cast<const uint16_t *>(fill),
             cache2,     static_cast<const uint16_t *>(fill2),
             fill_user_stride, fill_head_stride, fill_token_stride,
             page_table, page_table_row_stride,
             batch_idx,  batch_idx_is_i64,
             fill_users, table_rows, kv_heads, seq_len, block_size, head_size, table_width,
             num_blocks, 0u, 0u};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec_ok = head_size % 8 == 0 && aligned16(cache) && aligned16(fill) &&
                      (!cache2 || (aligned16(cache2) && aligned16(fill2))) &&
                      fill_user_stride % 8 == 0 && fill_head_stride % 8 == 0 &&
                      fill_token_stride % 8 == 0;
  int tpr;  // threads per token row
  if (kv_format == TTPA_KV_BFP8) {
    TTPA_REQUIRE(vec_ok, "block-float-8 fill needs 16-byte aligned fill rows");
    tpr = head_size / 16;
  } else {
    tpr = vec_ok ? head_size / 8 : head_size;
  }
  const int64_t threads = (int64_t)seq_len * tpr;  // per (fill row, head)
  const int pairs = cache2 ? 2 : 1;
  TTPA_REQUIRE(threads < (int64_t)1 << 31 && fill_users * pairs <= 65535 && kv_heads <= 65535,
               "fill too large for one launch");
  a.tpr_magic = magic_for(threads, tpr);
  a.bs_magic = magic_for(seq_len, block_size);
  const dim3 grid((unsigned)((threads + 255) / 256), (unsigned)kv_heads, (unsigned)(fill_users * pairs));
  if (kv_format == TTPA_KV_BFP8) {
    fill_bfp8_kernel<<<grid, dim3(256), 0, st>>>(a);
  } else if (vec_ok) {
    fill_bf16_kernel<8><<<grid, dim3(256), 0, st>>>(a);
  } else {
    fill_bf16_kernel<1><<<grid, dim3(256), 0, st>>>(a);
  }
  return check_launch("paged_fill_cache");
}

extern "C" int ttpa_paged_fill_cache(void *cache, const void *fill, int64_t fill_user_stride,
                                     int64_t fill_head_stride, int64_t fill_token_stride,
                                     const int32_t *page_table, int64_t page_table_row_stride,
                                     const void *batch_idx, int batch_idx_is_i64,
                                     int32_t fill_users, int32_t table_rows, int32_t kv_heads,
                                     int32_t seq_len, int32_t block_size, int32_t head_size,
                                     int32_t table_width, int32_t num_blocks, int32_t kv_format,
                                     void *stream) {
  return launch_fill(cache, nullptr, fill, nullptr, fill_user_stride, fill_head_stride,
                     fill_token_stride, page_table, page_table_row_stride, batch_idx,
                     batch_idx_is_i64, fill_users, table_rows, kv_heads, seq_len, block_size,
                     head_size, table_width, num_blocks, kv_format, stream);
}

extern "C" int ttpa_paged_fill_cache_kv(void *k_cache, void *v_cache, const void *k_fill,
                                        const void *v_fill, int64_t fill_user_stride,
                                        int64_t fill_head_stride, int64_t fill_token_stride,
                                        const int32_t *page_table, int64_t page_table_row_stride,
                                        const void *batch_idx, int batch_idx_is_i64,
                                        int32_t fill_users, int32_t table_rows, int32_t kv_heads,
                                        int32_t seq_len, int32_t block_size, int32_t head_size,
                                        int32_t table_width, int32_t num_blocks, int32_t kv_format,
                                        void *stream) {
  TTPA_REQUIRE(v_cache && v_fill, "null V cache / fill pointer");
  return launch_fill(k_cache, v_cache, k_fill, v_fill, fill_user_stride, fill_head_stride,
                     fill_token_stride, page_table, page_table_row_stride, batch_idx,
                     batch_idx_is_i64, fill_users, table_rows, kv_heads, seq_len, block_size,
                     head_size, table_width, num_blocks, kv_format, stream);
}
