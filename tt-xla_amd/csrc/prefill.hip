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
//
// K/V tiles travel global memory -> LDS directly (global_load_lds_dwordx4: 64 lanes x 16
// bytes land in 1 KiB of consecutive LDS), with no staging registers.  Rows are therefore
// unpadded in LDS; bank conflicts are avoided by an XOR swizzle of the 16-byte chunk
// position inside a row, applied on the global side (which chunk a lane fetches) and again
// when fragments are read.
#include "common.h"
#include "build/prefill_stream_asm.h"

#include <algorithm>
#include <cstdlib>

namespace ttpa {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
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
  uint32_t bs_magic;  // floor(2^32 / bs) + 1: key / bs = mulhi(key, bs_magic) while key * bs < 2^32 (bs >= 2)
  // Dense form with a cache fill in the same launch (fill_kc != null): k / v are also written
  // to the paged caches through fill_pt, by workgroups n_attn ... of the grid.  bs / nb /
  // bs_magic describe the caches; table row of batch entry i = fill_bidx[i] (or i == 0).
  uint16_t *fill_kc, *fill_vc;
  const int32_t *fill_pt;
  int64_t fill_pt_rs;
  const void *fill_bidx;
  int fill_bidx_i64, fill_rows;
  // Grid layout with a fill: fill_groups super-groups of (8 * attn_per_fill attention
  // workgroups, then 8 fill workgroups), then the remaining attention workgroups.  Groups of 8
  // keep an attention workgroup's index congruent to its hardware index modulo 8 (its XCD).
  int fill_groups, attn_per_fill, n_fill;
  int window;  // > 0 (causal only): row i attends keys offset + i - window < j <= offset + i
  float scale_log2e;
  int kv_bfp8;  // paged form: the caches are block-float-8 (mode 4, or expanded into `expand` first)
  void *expand; // scratch for bfloat16 copies of the block-float-8 blocks of this pass, or null
  int stream;   // the hand-scheduled loop serves this launch (head size 128, 4 heads per workgroup, whole blocks)
  int spg;      // ... with this many workgroups per (batch entry, head group), each taking several row blocks
  int spg_even; // > 0: when the row blocks weigh about the same, only this many of them work (equal shares)
};

// key / block_size without a division instruction sequence (about 30 instructions each, and the
// paged tile loads need several per tile).
__device__ __forceinline__ int div_block(const PrefillArgs &a, int key) {
  return a.bs == 1 ? key : (int)__umulhi((uint32_t)key, a.bs_magic);
}

// LDS geometry of one stage: the K tile (64 rows of D elements) followed by the V tile.
// Chunk c (16 bytes) of row r is stored at chunk position c ^ swz(r).
//   K fragments are read by 16 lanes of consecutive rows at one logical chunk: the 16
//   positions must differ (rows of >= 256 bytes) or, for 128-byte rows, differ within each
//   pair of rows that shares a 256-byte bank line.
//   V fragments are read, per 32 lanes, as 4 consecutive rows x 4 consecutive chunks.
template <int D>
struct Tile {
  static constexpr int RB = 2 * D;                 // row bytes
  static constexpr int CPR = D / 8;                // 16-byte chunks per row
  static constexpr int RPI = 1024 / RB;            // rows covered by one wavefront load
  static constexpr int NI = kKeysPerTile / RPI / 4;  // loads per wavefront per tile and tensor
  static constexpr int TILE_BYTES = kKeysPerTile * RB;
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;
  __device__ static constexpr int swz_k(int r) { return RB >= 256 ? (r & 15) : ((r >> 1) & 7); }
  __device__ static constexpr int swz_v(int r) { return RB >= 256 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); }
};

// v_max3_f32 without the input canonicalisation the compiler adds around fmaxf (scores are
// never signalling NaNs).  Callers order it after a compiler-visible read of the matrix
// results, which is where the matrix-to-vector hazard wait states are inserted.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

// The cache fill that rides along with a dense prefill: workgroup f (counted from the end of
// the attention workgroups) copies fill_rows_per_wg(D) token rows (128 KiB) of one (tensor, batch entry, KV head)
// from the dense K / V operand into the paged cache, with the semantics of the fill operator
// (rows whose table row or block is out of range are skipped).  Pure memory work that runs in
// the shadow of the matrix-bound attention workgroups; nothing in this launch reads the caches.
constexpr int kFillPasses = 32;  // 16-byte loads in flight per thread
constexpr int fill_rows_per_wg(int d) { return kFillPasses * (256 / (d / 8)); }

template <int D>
__device__ __forceinline__ void fill_workgroup(const PrefillArgs &a, int f) {
  constexpr int CPR = D / 8;        // 16-byte chunks per row
  constexpr int RPP = 256 / CPR;    // rows per pass of the 256 threads
  constexpr int NP = kFillPasses;
  constexpr int kFillRows = fill_rows_per_wg(D);
  const int chunks = (a.skv + kFillRows - 1) / kFillRows;
  const int c0 = f % chunks;
  int r = f / chunks;
  const int h = r % a.hkv;
  r /= a.hkv;
  const int b = r % a.batch;
  const bool is_v = r / a.batch != 0;
  int64_t row = a.fill_bidx ? load_index(a.fill_bidx, a.fill_bidx_i64, b) : 0;
  if (row < 0 || row >= a.fill_rows) return;
  const uint16_t *src = (is_v ? a.v : a.k) + b * a.kv_bs + h * a.kv_hs;
  uint16_t *cache = is_v ? a.fill_vc : a.fill_kc;
  const int32_t *pt = a.fill_pt + row * a.fill_pt_rs;
  const int t0 = c0 * kFillRows + (int)threadIdx.x / CPR, c = (int)threadIdx.x % CPR;
  // every load (rows and table entries) is requested before the first store: the compiler
  // cannot move a load across a store that might alias it, and a table entry per pass would
  // otherwise cost a round trip each
  u32x4 val[NP];
  int phys[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int t = min(t0 + p * RPP, a.skv - 1);
    val[p] = *reinterpret_cast<const u32x4 *>(src + (int64_t)t * a.kv_ts + 8 * c);
    phys[p] = pt[div_block(a, t)];
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int t = t0 + p * RPP;
    const int off = t - div_block(a, t) * a.bs;
    // (no early exit from the loop: the arrays must stay in registers)
    if (t < a.skv && (unsigned)phys[p] < (unsigned)a.nb)
      __builtin_nontemporal_store(val[p], reinterpret_cast<u32x4 *>(cache + (((int64_t)phys[p] * a.hkv + h) * a.bs + off) * D + 8 * c));
  }
}

// Expansion of the block-float-8 blocks a chunk pass reads into bfloat16 copies, so that the
// hand-scheduled loop (which wants bfloat16 blocks it can request straight into LDS) serves a
// block-float-8 cache too: workgroup (x, y) expands the slab of table entry x = batch entry * width
// + column and of (KV head, K or V) y into block x of a scratch cache, and writes entry x of the
// identity table that goes with it.  Columns behind the last key of the pass are skipped.  Memory
// work (1 byte in, 2 out per element) of about a tenth of the attention's time.
struct ExpandArgs {
  const uint8_t *kc, *vc;  // the block-float-8 caches
  uint16_t *k, *v;         // scratch caches [batch * width][KV heads][block size][D]
  int32_t *table;          // [batch][width]
  const int32_t *pt;
  int64_t pt_rs;
  const int32_t *chunk_start;
  int w, hkv, bs, nb, sq, causal;
};

template <int D>
__global__ __launch_bounds__(256) void bfp8_expand_kernel(ExpandArgs e) {
  const int x = blockIdx.x, b = x / e.w, j = x - b * e.w;
  const int h = blockIdx.y >> 1;
  const bool is_v = blockIdx.y & 1;
  if (blockIdx.y == 0 && threadIdx.x == 0) e.table[x] = x;
  const int skv = e.w * e.bs;
  const int kv_end = e.causal ? min(skv, (e.chunk_start ? e.chunk_start[0] : 0) + e.sq) : skv;
  if (j * e.bs >= kv_end) return;
  int phys = e.pt[(int64_t)b * e.pt_rs + j];
  if ((unsigned)phys >= (unsigned)e.nb) phys = 0;  // (as the attention kernels treat a bad entry)
  const int64_t slab = (int64_t)(e.bs + e.bs / 16) * D;
  const uint8_t *src = (is_v ? e.vc : e.kc) + ((int64_t)phys * e.hkv + h) * slab;
  const uint8_t *exps = src + (int64_t)e.bs * D;
  uint16_t *dst = (is_v ? e.v : e.k) + ((int64_t)x * e.hkv + h) * e.bs * D;
  const int groups = e.bs * D / 16;
  for (int g = threadIdx.x; g < groups; g += 256) {
    const u32x4 bytes = *reinterpret_cast<const u32x4 *>(src + 16 * g);
    const float sc = bfp8_group_scale(exps[g]), off = -128.f * sc;
    u32x4 lo, hi;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t v = bytes[w];
      const float f0 = fmaf((float)(v & 0xffu), sc, off), f1 = fmaf((float)((v >> 8) & 0xffu), sc, off);
      const float f2 = fmaf((float)((v >> 16) & 0xffu), sc, off), f3 = fmaf((float)(v >> 24), sc, off);
      // the products are exact in bfloat16: their upper halves are the elements
      const uint32_t p0 = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
      const uint32_t p1 = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
      if (w < 2) lo[2 * w] = p0, lo[2 * w + 1] = p1;
      else hi[2 * (w - 2)] = p0, hi[2 * (w - 2) + 1] = p1;
    }
    *reinterpret_cast<u32x4 *>(dst + 16 * g) = lo;
    *reinterpret_cast<u32x4 *>(dst + 16 * g + 8) = hi;
  }
}

// ---------------------------------------------------------------------------------------------
// The hand-scheduled loop over whole unmasked tiles (head size 128, 32 rows per wavefront): one
// block of assembly, written by gen_prefill_stream.py, which documents the schedule and the
// state on entry and exit.  Everything the block touches is bound to the registers its text
// names; the compiler moves values in and out around it and keeps its own out of the clobbered
// ones.  Entered with K(0), V(0), K(1) requested and K(0) published; handles tiles 0 .. n - 1.
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

// The requests of a workgroup's first blocks are a block of assembly of their own, issued in front
// of the Q loads so that the two round trips to memory overlap.  (Scalars only: with the per-lane
// offsets in the same struct the compiler keeps the whole of it in vector registers.)
struct StreamRequests {
  uint64_t kbase, vbase;       // dense: block 0 of K / V; paged: the caches (both minus 1024 bytes)
  uint32_t stride;             // dense: bytes from a 32-key block to the next; paged: bytes of a (cache block, head) slab
  uint32_t m0_base;            // LDS address of the wavefront's first segment in K slot 0
  int k_requests, v_requests;  // blocks not requested yet
  uint64_t off0, off1, off2;   // paged: byte offsets of tiles 0, 1, 2 in a cache
};

__device__ __forceinline__ void stream_first_dense(StreamRequests &r, const u32x2 &ldk, const u32x2 &ldv) {
  asm volatile(TTPA_STREAM_FIRST_TEXT_DENSE
               : "+{s[64:65]}"(r.kbase), "+{s[66:67]}"(r.vbase), "+{s71}"(r.k_requests), "+{s73}"(r.v_requests)
               : "{v[188:189]}"(ldk), "{v[190:191]}"(ldv), "{s68}"(r.stride), "{s72}"(r.m0_base)
               : "memory", "scc", "m0");
}

__device__ __forceinline__ void stream_first_paged(StreamRequests &r, const u32x2 &ldk, const u32x2 &ldv) {
  asm volatile(TTPA_STREAM_FIRST_TEXT_PAGED
               : "+{s71}"(r.k_requests), "+{s73}"(r.v_requests)
               : "{v[188:189]}"(ldk), "{v[190:191]}"(ldv), "{s[64:65]}"(r.kbase), "{s[66:67]}"(r.vbase),
                 "{s72}"(r.m0_base), "{s[84:85]}"(r.off1), "{s[86:87]}"(r.off2), "{s[98:99]}"(r.off0)
               : "memory", "scc", "m0", "s90", "s91");
}

// The items of a workgroup (see gen_prefill_stream.py): which row blocks, and what the block needs
// to set one up.
// Values the compiler may hold in vector registers although they are the same in every lane: the
// block binds them to scalar registers.
__device__ __forceinline__ int uni(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ uint32_t uni(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ uint64_t uni(uint64_t x) {
  return address_from_words(__builtin_amdgcn_readfirstlane((int)(uint32_t)x), __builtin_amdgcn_readfirstlane((int)(uint32_t)(x >> 32)));
}

struct StreamItems {
  int k, j, spg, nqt;          // item counter (starts at 0), the workgroup's slot, slots, row blocks
  int sq, skv, offset, causal;
  uint32_t q_row_bytes, out_row_bytes;
  int row0;                    // first query row of item 0
};

#define TTPA_STREAM_COMMON_OUT                                                                        \
  "+{v[64:79]}"(q_lo), "+{v[80:95]}"(q_hi), "+{s[64:65]}"(r.kbase), "+{s[66:67]}"(r.vbase), "+{s70}"(nblk), \
      "+{s71}"(r.k_requests), "+{s73}"(r.v_requests), "+{s40}"(it.k), "+{s57}"(it.row0)
#define TTPA_STREAM_COMMON_IN                                                                       \
  "{v[176:183]}"(koff), "{v[184:187]}"(voff), "{v[188:189]}"(ldk), "{v[190:191]}"(ldv),         \
      "{v[216:217]}"(q_base), "{v[218:219]}"(out_base), "{v220}"(lane_n), "{v221}"(lane_h4),       \
      "{s68}"(r.stride), "{s69}"(c), "{s72}"(r.m0_base), "{s41}"(it.j), "{s42}"(it.spg), "{s43}"(it.nqt), \
      "{s44}"(it.sq), "{s45}"(it.skv), "{s46}"(it.offset), "{s47}"(it.causal), "{s48}"(it.q_row_bytes),  \
      "{s49}"(it.out_row_bytes)

// Everything behind the first requests of item 0, through the stored output rows of the last item.
// q_lo / q_hi: the eight Q fragments of item 0; koff / voff: the lane's LDS addresses of its K and
// V^T fragments in slot 0 of the K and V rings; nblk: the 32-key blocks of item 0; kbase0 / vbase0:
// block 0 of K / V again, for the items that follow.
__device__ __forceinline__ void stream_items_dense(StreamRequests &r, StreamItems &it, u32x16 q_lo, u32x16 q_hi,
                                                   const u32x8 &koff, const u32x4 &voff, const u32x2 &ldk,
                                                   const u32x2 &ldv, uint64_t q_base, uint64_t out_base, int lane_n,
                                                   int lane_h4, float c, int nblk, uint64_t kbase0, uint64_t vbase0) {
  asm volatile(TTPA_STREAM_LOOP_TEXT_DENSE
               : TTPA_STREAM_COMMON_OUT
               : TTPA_STREAM_COMMON_IN, "{s[50:51]}"(kbase0), "{s[52:53]}"(vbase0)
               : "memory", "vcc", "scc", "m0", "v208", TTPA_STREAM_LOOP_CLOBBERS);
}

// Paged: entry is the raw table entry of tile 3, entry_ptr the address of tile 4's.
__device__ __forceinline__ void stream_items_paged(StreamRequests &r, StreamItems &it, u32x16 q_lo, u32x16 q_hi,
                                                   const u32x8 &koff, const u32x4 &voff, const u32x2 &ldk,
                                                   const u32x2 &ldv, uint64_t q_base, uint64_t out_base, int lane_n,
                                                   int lane_h4, float c, int nblk, int kv_heads, int kv_head, int num_blocks, int tiles_per_block,
                                                   int entry, uint64_t entry_ptr) {
  int read_in_block = 3 % tiles_per_block, request_in_block = 4 % tiles_per_block;
  const int read_in_block0 = read_in_block, request_in_block0 = request_in_block, entry0 = entry;
  const uint64_t entry_ptr0 = entry_ptr, off1 = r.off1, off2 = r.off2;
  int entry_requests = max((nblk - 1) / 2 - 3, 0);
  asm volatile(TTPA_STREAM_LOOP_TEXT_PAGED
               : TTPA_STREAM_COMMON_OUT, "+{s80}"(read_in_block), "+{s81}"(request_in_block),
                 "+{s[82:83]}"(entry_ptr), "+{s[84:85]}"(r.off1), "+{s[86:87]}"(r.off2), "+{s96}"(entry_requests),
                 "+{v208}"(entry)
               : TTPA_STREAM_COMMON_IN, "{s76}"(kv_heads), "{s77}"(kv_head), "{s78}"(num_blocks),
                 "{s79}"(tiles_per_block), "{s[98:99]}"(r.off0), "{s[50:51]}"(off1), "{s[52:53]}"(off2),
                 "{s54}"(entry0), "{s55}"(read_in_block0), "{s56}"(request_in_block0), "{s[58:59]}"(entry_ptr0)
               : "memory", "vcc", "scc", "m0", TTPA_STREAM_LOOP_CLOBBERS);
}

// MODE 0: dense K/V; 1: paged, block_size a multiple of 64 (a tile lies in one block);
// 3: paged, block_size a multiple of the rows one wavefront load covers (1 KiB: 8 / 4 / 2 rows
// for head sizes 64 / 128 / 256): one wavefront-uniform table lookup per load; 2: paged, any
// block size (per-lane table lookups); 4: paged block-float-8 caches (block_size a multiple of
// 16).  In mode 4 a tile goes global -> registers -> LDS: a thread fetches groups of 16 element
// bytes with their exponent byte (D / 64 groups per tile and tensor) where the other modes issue
// their LDS-DMA loads, and expands them to bfloat16 (exact: a 7-bit magnitude times a power of
// two) into the same swizzled tile layout at the end of the iteration, one tile period before
// the tile is used.  One workgroup per CU: the staging registers do not fit next to a second one.
//
// Per-tile schedule of a workgroup (LDS holds two K stages and two V stages):
//   S^T = K(t) Q^T | barrier | issue loads of K(t+2) and V(t+1) | softmax | O^T += V(t)^T P^T
// Every load is issued right after a barrier and has to have landed by the next one, one
// whole tile later.  K(t+2) overwrites the stage of K(t), which everybody has finished
// reading at the barrier of tile t; V(t+1) overwrites the stage of V(t-1), read before that
// barrier too.  LDS operand reads run a few fragments ahead of the matrix instructions that
// consume them.
//
// RH: blocks of 32 query rows per wavefront; only 1 is built (a form with two, one workgroup per
// CU and every K / V fragment feeding two matrix instructions, measured slower: with one wavefront
// per SIMD nobody fills the waits for fragments and barriers).
template <int RH>
constexpr int prefill_wgs_per_cu(int d, int mode) { return RH == 1 && d <= 128 ? 2 : 1; }

template <int D, int HPW, int MODE, int RH>
__global__ __launch_bounds__(256, prefill_wgs_per_cu<RH>(D, MODE)) void prefill_kernel(PrefillArgs a) {
  constexpr int RPW = 4 / HPW;            // wavefront row slots per workgroup
  constexpr int ROWS = kRowsPerWave * RH;  // query rows per wavefront
  constexpr int KSTEPS = D / 16;          // MFMA k-steps over the head dimension
  constexpr int DBLK = D / 32;            // 32-wide output blocks over the head dimension
  using T = Tile<D>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  int wg = blockIdx.x;  // index among the attention workgroups
  if constexpr (MODE == 0) {
    if (a.fill_kc != nullptr) {
      const int per = 8 * (a.attn_per_fill + 1);
      const int sg = wg / per, m = wg - sg * per;
      if (sg < a.fill_groups) {
        if (m >= 8 * a.attn_per_fill) {
          const int f = sg * 8 + (m - 8 * a.attn_per_fill);
          if (f < a.n_fill) fill_workgroup<D>(a, f);
          return;
        }
        wg = sg * 8 * a.attn_per_fill + m;
      } else {
        wg -= 8 * a.fill_groups;
      }
    }
  }
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int n_lane = n;
  // Workgroups are dealt to the 8 XCDs round-robin by linear id, and each XCD has its own
  // L2: all query tiles of one (batch, KV-head group) run on the same XCD, one after the
  // other, so that K/V of a group is fetched from HBM by one L2 only and stays resident there
  // while its query tiles stream through.
  const int nqt = (a.sq + ROWS * RPW - 1) / (ROWS * RPW);
  const int groups = a.hq / HPW;
  // (the hand-scheduled loop: a.spg workgroups per group, each taking several row blocks, heavy first)
  constexpr bool kStreams = D == 128 && HPW == 4 && RH == 1 && (MODE == 0 || MODE == 1);
  const bool streamed = kStreams && a.stream != 0;
  const int per_group = streamed ? a.spg : nqt;
  const int xcd = wg & 7, slot = wg >> 3;
  const int yl = slot / per_group;
  const int y = yl * 8 + xcd;
  if (y >= a.batch * groups) return;  // grid is padded to a multiple of 8 groups
  const int qt = nqt - 1 - (slot - yl * per_group);  // heavy (late) tiles are scheduled first
  const int b = y / groups;
  const int hq0 = (y - b * groups) * HPW;
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
  // sliding window: first key any row of the workgroup / of this wavefront can see
  const int wg_first_key = a.window > 0 ? max(0, offset + qt * ROWS * RPW - a.window + 1) : 0;
  const int wave_first_key = a.window > 0 ? max(0, offset + row0 - a.window + 1) : 0;
  const int first_tile = wg_first_key / kKeysPerTile;

  // ---- the hand-scheduled loop: its first requests go out now, in front of the Q loads ----------
  StreamRequests sreq;
  u32x2 stream_ldk = {0, 0}, stream_ldv = {0, 0};
  int stream_entry = 0;
  if constexpr (kStreams) {
    if (streamed) {
      int spg = a.spg;
      if (a.spg_even > 0) {
        const int lightest = a.causal ? min(offset + ROWS, a.skv) : a.skv;
        const int heaviest = a.causal ? min(offset + a.sq, a.skv) : a.skv;
        if (4 * lightest >= 3 * heaviest) {
          spg = a.spg_even;
          if (slot - yl * per_group >= spg) return;
        }
      }
      const uint32_t lds0 = lds_address(smem);
      const uint32_t row_bytes = MODE == 0 ? 2u * (uint32_t)a.kv_ts : (uint32_t)T::RB;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // a block is 8 segments of 1 KiB; wavefront w requests segments 2 w and 2 w + 1
        const int r = (2 * wave + j) * T::RPI + lane / T::CPR, cp = lane % T::CPR;
        stream_ldk[j] = (uint32_t)r * row_bytes + 16u * (uint32_t)(cp ^ T::swz_k(r)) + 1024u - 1024u * j;
        stream_ldv[j] = (uint32_t)r * row_bytes + 16u * (uint32_t)(cp ^ T::swz_v(r)) + 1024u - 1024u * j;
      }
      sreq.m0_base = uni(lds0 + 2048u * (uint32_t)wave);
      sreq.k_requests = sreq.v_requests = __builtin_amdgcn_readfirstlane((kv_end_wg + 31) / 32);
      sreq.off0 = sreq.off1 = sreq.off2 = 0;
      if constexpr (MODE == 0) {
        const int64_t head = b * a.kv_bs + hk * a.kv_hs;
        sreq.kbase = uni(reinterpret_cast<uint64_t>(a.k + head) - 1024u);
        sreq.vbase = uni(reinterpret_cast<uint64_t>(a.v + head) - 1024u);
        sreq.stride = (uint32_t)(64 * a.kv_ts);
        stream_first_dense(sreq, stream_ldk, stream_ldv);
      } else {
        const int tpb = a.bs / kKeysPerTile, last = a.w * tpb - 1;  // (entries exist for every tile of the table)
        sreq.kbase = reinterpret_cast<uint64_t>(a.k) - 1024u;
        sreq.vbase = reinterpret_cast<uint64_t>(a.v) - 1024u;
        sreq.stride = (uint32_t)a.bs * (uint32_t)T::RB;
        int raw[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) raw[t] = a.pt[(int64_t)b * a.pt_rs + min(t, last) / tpb];
        uint64_t off[3];
#pragma unroll
        for (int t = 0; t < 3; ++t) {
          int phys = __builtin_amdgcn_readfirstlane(raw[t]);
          if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
          off[t] = (uint64_t)((int64_t)phys * a.hkv + hk) * sreq.stride + (uint64_t)(min(t, last) % tpb) * T::TILE_BYTES;
        }
        sreq.off0 = uni(off[0]), sreq.off1 = uni(off[1]), sreq.off2 = uni(off[2]);
        stream_entry = raw[3];
        stream_first_paged(sreq, stream_ldk, stream_ldv);
      }
      // Q fragments behind the requests (B operand: lane n = query row, 8 head-dim elements per k-step)
      u32x16 q_lo, q_hi;
      {
        const int qrow = min(row0 + n, a.sq - 1);
        const uint16_t *qp = a.q + b * a.q_bs + hq * a.q_hs + (int64_t)qrow * a.q_ts + 8 * h;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint4 lo = *reinterpret_cast<const uint4 *>(qp + 16 * s), hi = *reinterpret_cast<const uint4 *>(qp + 16 * (s + 4));
          q_lo[4 * s] = lo.x, q_lo[4 * s + 1] = lo.y, q_lo[4 * s + 2] = lo.z, q_lo[4 * s + 3] = lo.w;
          q_hi[4 * s] = hi.x, q_hi[4 * s + 1] = hi.y, q_hi[4 * s + 2] = hi.z, q_hi[4 * s + 3] = hi.w;
        }
      }
      // LDS operand addresses of the lane inside slot 0 of the K ring and of the V ring (the formulas
      // of the plain loop below: K fragment of k-step s, V^T fragment of output block db)
      u32x8 ko;
#pragma unroll
      for (int s = 0; s < 8; ++s) ko[s] = lds0 + (uint32_t)(n * T::RB + 16 * ((2 * s + h) ^ T::swz_k(n)));
      u32x4 vo;
      {
        const int grp = lane >> 4, a16 = lane & 15, vr = 4 * (grp >> 1) + (a16 >> 2);
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int c = 4 * db + 2 * (grp & 1) + ((a16 & 3) >> 1);
          vo[db] = lds0 + TTPA_STREAM_V_RING + (uint32_t)(vr * T::RB + 16 * (c ^ T::swz_v(vr)) + 8 * (a16 & 1));
        }
      }
      StreamItems it;
      it.k = 0, it.j = uni(slot - yl * per_group), it.spg = uni(spg), it.nqt = uni(nqt);
      it.sq = uni(a.sq), it.skv = uni(a.skv), it.offset = uni(offset), it.causal = uni(a.causal);
      it.q_row_bytes = uni(2u * (uint32_t)a.q_ts), it.out_row_bytes = uni(2u * (uint32_t)a.out_ts);
      it.row0 = __builtin_amdgcn_readfirstlane(row0);
      // per lane: row 0 of the lane's head, at the lane's 8 (lane / 32) / 4 (lane / 32) elements
      const uint64_t q_base = reinterpret_cast<uint64_t>(a.q + b * a.q_bs + hq * a.q_hs + 8 * h);
      const uint64_t out_base = reinterpret_cast<uint64_t>(a.out + b * a.out_bs + hq * a.out_hs + 8 * h);
      const int nblk = __builtin_amdgcn_readfirstlane((kv_end_wg + 31) / 32);
      if constexpr (MODE == 0) {
        const int64_t head = b * a.kv_bs + hk * a.kv_hs;
        stream_items_dense(sreq, it, q_lo, q_hi, ko, vo, stream_ldk, stream_ldv, q_base, out_base, n, 4 * h, a.scale_log2e, nblk,
                           uni(reinterpret_cast<uint64_t>(a.k + head) - 1024u), uni(reinterpret_cast<uint64_t>(a.v + head) - 1024u));
      } else {
        const int tpb = a.bs / kKeysPerTile;
        stream_items_paged(sreq, it, q_lo, q_hi, ko, vo, stream_ldk, stream_ldv, q_base, out_base, n, 4 * h, a.scale_log2e, nblk, uni(a.hkv), uni(hk), uni(a.nb), uni(tpb), stream_entry,
                           uni(reinterpret_cast<uint64_t>(a.pt + (int64_t)b * a.pt_rs + 4 / tpb)));
      }
      return;
    }
  }

  // ---- Q fragments (B operand: lane n = query row, 8 head-dim elements per k-step) -----
  static_assert(RH == 1, "one block of 32 query rows per wavefront");
  bf16x8 qf[RH][KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int qrow = min(row0 + n, a.sq - 1);
    const uint16_t *qp = a.q + b * a.q_bs + hq * a.q_hs + (int64_t)qrow * a.q_ts + 8 * h;
    qf[0][s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 16 * s));
  }

  floatx16 acc[RH][DBLK];
  float m_run[RH], l_run[RH];
#pragma unroll
  for (int x = 0; x < RH; ++x) {
    m_run[x] = -INFINITY, l_run[x] = 0.f;
#pragma unroll
    for (int i = 0; i < DBLK; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[x][i][r] = 0.f;
  }

  // ---- global -> LDS tile loads ----------------------------------------------------------
  // Load j of this wavefront fills LDS segment 4 j + wave of a tile: RPI whole rows.  Lane l
  // writes chunk position l % CPR of row seg * RPI + l / CPR, so it fetches logical chunk
  // (l % CPR) ^ swz(row).  The per-lane part of the source address is fixed for all tiles.
  int ld_row[T::NI];       // row inside the tile
  uint32_t ld_k[T::NI], ld_v[T::NI];  // byte offset of the lane's chunk inside a tile (modes 0 and 1)
#pragma unroll
  for (int j = 0; j < T::NI; ++j) {
    const int r = (4 * j + wave) * T::RPI + lane / T::CPR;
    const int cp = lane % T::CPR;
    const uint32_t row_bytes = MODE == 0 ? 2u * (uint32_t)a.kv_ts : (uint32_t)T::RB;
    ld_row[j] = r;
    ld_k[j] = (uint32_t)r * row_bytes + 16u * (uint32_t)(cp ^ T::swz_k(r));
    ld_v[j] = (uint32_t)r * row_bytes + 16u * (uint32_t)(cp ^ T::swz_v(r));
  }
  // Issues the loads of one tile of one tensor.  Keys past the end of K/V are clamped to the
  // last row, whose scores are masked and whose V rows therefore carry weight 0.
  // Modes 1 and 3 look their blocks up one tile ahead of the loads (below): NLK wavefront-
  // uniform table entries per tile, one for the whole tile or one per load of this wavefront.
  constexpr int GPR = D / 16;           // mode 4: 16-element groups (= exponent bytes) per row
  constexpr int NG = D / 64;            // mode 4: groups per thread, tile and tensor
  constexpr int NLK = MODE == 1 ? 1 : (MODE == 3 ? T::NI : (MODE == 4 ? NG : 0));
  struct Blocks {
    int phys[NLK > 0 ? NLK : 1];
  };
  // first key of lookup j of tile kt
  auto lookup_key = [&](int kt, int j) {
    const int key0 = kt * kKeysPerTile;
    if constexpr (MODE == 1) return key0;
    if constexpr (MODE == 4) return key0 + min((tid + 256 * j) / GPR, a.skv - 1 - key0);  // per lane
    // the rows of a load sit in one block; a load wholly past the last key reads the rows that
    // hold the last key again (readable, and masked like any key past the end)
    return key0 + min((4 * j + wave) * T::RPI, (a.skv - 1 - key0) / T::RPI * T::RPI);
  };
  // LDS byte offset of a tile: stages of a K and a V tile each
  auto tile_offset = [&](bool is_v, int buf) { return (uint32_t)(buf * T::STAGE_BYTES + (is_v ? T::TILE_BYTES : 0)); };
  auto issue = [&](const uint16_t *src, const uint32_t (&ld)[T::NI], bool is_v, int kt, int buf,
                   const Blocks &blk) {
    const int key0 = kt * kKeysPerTile;
    const int last = a.skv - 1 - key0;  // last valid key of this tile, relative (>= 0)
    const uint32_t lds_base = lds_address(smem) + tile_offset(is_v, buf);
    const char *base = nullptr;  // uniform address of the tile (modes 0 and 1)
    if constexpr (MODE == 0) {
      base = reinterpret_cast<const char *>(src + b * a.kv_bs + hk * a.kv_hs + (int64_t)key0 * a.kv_ts);
    } else if constexpr (MODE == 1) {
      base = reinterpret_cast<const char *>(
          src + (((int64_t)blk.phys[0] * a.hkv + hk) * a.bs + (key0 - div_block(a, key0) * a.bs)) * D);
    }
    auto lds_dst = [&](int j) { return lds_base + (uint32_t)(4 * j + wave) * 1024u; };
    if constexpr (MODE == 2) {
#pragma unroll
      for (int j = 0; j < T::NI; ++j) {
        const int key = key0 + min(ld_row[j], last);
        const int col = div_block(a, key);
        int phys = a.pt[(int64_t)b * a.pt_rs + col];
        if ((unsigned)phys >= (unsigned)a.nb) phys = 0;
        const int c = (lane % T::CPR) ^ (is_v ? T::swz_v(ld_row[j]) : T::swz_k(ld_row[j]));
        dma16_lane(src + (((int64_t)phys * a.hkv + hk) * a.bs + (key - col * a.bs)) * D + c * 8, lds_dst(j));
      }
    } else if constexpr (MODE == 3) {
#pragma unroll
      for (int j = 0; j < T::NI; ++j) {
        const int key = lookup_key(kt, j);
        const char *seg = reinterpret_cast<const char *>(
            src + (((int64_t)blk.phys[j] * a.hkv + hk) * a.bs + (key - div_block(a, key) * a.bs)) * D);
        dma16(seg, ld[j] - (uint32_t)((4 * j + wave) * T::RPI * T::RB), lds_dst(j));
      }
    } else if (MODE == 0 && last < kKeysPerTile - 1) {  // uniform: dense K/V ending inside the tile
#pragma unroll
      for (int j = 0; j < T::NI; ++j) {
        const int c = (lane % T::CPR) ^ (is_v ? T::swz_v(ld_row[j]) : T::swz_k(ld_row[j]));
        const uint32_t off = (uint32_t)min(ld_row[j], last) * 2u * (uint32_t)a.kv_ts + 16u * (uint32_t)c;
        dma16(base, off, lds_dst(j));
      }
    } else {
#pragma unroll
      for (int j = 0; j < T::NI; ++j) dma16(base, ld[j], lds_dst(j));
    }
  };
  // ---- mode 4: block-float-8 tiles through registers --------------------------------------
  struct Staged {
    u32x4 bytes[MODE == 4 ? NG : 1];
    uint32_t ex[MODE == 4 ? NG : 1];
  };
  // group j of this thread: row (tid + 256 j) / GPR of the tile, 16 elements from 16 ((tid + 256 j) % GPR)
  auto fetch_bfp8 = [&](const uint16_t *cache, int kt, const Blocks &blk) {
    Staged st = {};
    if constexpr (MODE == 4) {
      const uint8_t *base = reinterpret_cast<const uint8_t *>(cache);
      const int64_t slab = (int64_t)(a.bs + a.bs / 16) * D;
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        const int key = lookup_key(kt, j), c16 = (tid + 256 * j) % GPR;
        const int rowin = key - div_block(a, key) * a.bs;
        const uint8_t *sl = base + ((int64_t)blk.phys[j] * a.hkv + hk) * slab;
        st.bytes[j] = *reinterpret_cast<const u32x4 *>(sl + rowin * D + 16 * c16);
        st.ex[j] = sl[(int64_t)a.bs * D + rowin * GPR + c16];
      }
    }
    return st;
  };
  // (b - 128) * 2^(e - 133) for the 16 bytes of a group, as 8 bfloat16 pairs; LDS chunks
  // 2 c16 and 2 c16 + 1 of the row, at their swizzled positions
  auto commit_bfp8 = [&](const Staged &st, bool is_v, int buf) {
    if constexpr (MODE == 4) {
      unsigned char *tile_base = smem + buf * T::STAGE_BYTES + (is_v ? T::TILE_BYTES : 0);
#pragma unroll
      for (int j = 0; j < NG; ++j) {
        const int row = (tid + 256 * j) / GPR, c16 = (tid + 256 * j) % GPR;
        const float sc = bfp8_group_scale(st.ex[j]), off = -128.f * sc;
        uint32_t o[8];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t x = st.bytes[j][w];
          const float f0 = fmaf((float)(x & 0xffu), sc, off), f1 = fmaf((float)((x >> 8) & 0xffu), sc, off);
          const float f2 = fmaf((float)((x >> 16) & 0xffu), sc, off), f3 = fmaf((float)(x >> 24), sc, off);
          // the products are exact in bfloat16: their upper halves are the elements
          o[2 * w] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
          o[2 * w + 1] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
        }
        const int sw = is_v ? T::swz_v(row) : T::swz_k(row);
        unsigned char *rp = tile_base + row * T::RB;
        *reinterpret_cast<uint4 *>(rp + 16 * ((2 * c16) ^ sw)) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4 *>(rp + 16 * ((2 * c16 + 1) ^ sw)) = make_uint4(o[4], o[5], o[6], o[7]);
      }
    }
  };
  auto wait_loads_and_sync = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's tile loads have landed
    __syncthreads();
  };

  // ---- LDS operand addresses of this lane inside a stage (bytes) ------------------------
  uint32_t koff[KSTEPS];  // K fragment of k-step s, key block 0 (key block 1: + 32 rows)
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
    koff[s] = (uint32_t)(n * T::RB + 16 * ((2 * s + h) ^ T::swz_k(n)));
  // V^T fragment: through the transposing LDS load, per group of 16 lanes, lane i receives
  // element i % 4 of the 8-byte chunks addressed by lanes 4 j + i / 4.  This lane addresses
  // row 4 (grp / 2) + a16 / 4 (+ 16 per key step, + 8 for the second half), elements
  // 32 db + 16 (grp % 2) + 4 (a16 % 4).
  const int grp = lane >> 4, a16 = lane & 15;
  uint32_t voff[DBLK];
  {
    const int vr = 4 * (grp >> 1) + (a16 >> 2);
#pragma unroll
    for (int db = 0; db < DBLK; ++db) {
      const int c = 4 * db + 2 * (grp & 1) + ((a16 & 3) >> 1);
      voff[db] = (uint32_t)(vr * T::RB + 16 * (c ^ T::swz_v(vr)) + 8 * (a16 & 1));
    }
  }
  // K fragment i of a tile in issue order: k-step i / 2 of key block i % 2 (the two score
  // blocks alternate so consecutive matrix instructions are independent).
  auto read_k = [&](const unsigned char *st_base, int i) -> bf16x8 {
    const int s = i >> 1, kb = i & 1;
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(st_base + koff[s] + 32 * kb * T::RB));
  };
  // V^T fragment j in issue order: key step j / DBLK, output block j % DBLK (st_base: the V tile).
  auto read_v = [&](const unsigned char *st_base, int j) -> bf16x8 {
    typedef __attribute__((address_space(3))) shortx4 *lds_v4;
    const int k4 = j / DBLK, db = j % DBLK;
    const unsigned char *vk = st_base + voff[db] + 16 * k4 * T::RB;
    shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk));
    shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)(vk + 8 * T::RB));
    bf16x4 l4 = __builtin_bit_cast(bf16x4, lo), h4 = __builtin_bit_cast(bf16x4, hi);
    bf16x8 t;
    t[0] = l4[0], t[1] = l4[1], t[2] = l4[2], t[3] = l4[3];
    t[4] = h4[0], t[5] = h4[1], t[6] = h4[2], t[7] = h4[3];
    return t;
  };

  constexpr int NK = 2 * KSTEPS;  // K fragments per tile
  constexpr int NV = 4 * DBLK;    // V^T fragments per tile
  // Fragments in flight.  Mode 4 holds a K and a V tile's bytes in registers across the iteration
  // and keeps the rings short: with 6 and 4 it spills 17 registers at two workgroups per CU (head
  // size 128), with 4 and 2 none, and the second workgroup is worth 224 -> 136 us on a pass of
  // four 512-token chunks over 2048 cached tokens.
  constexpr int KPRE = MODE == 4 ? 4 : 6;  // K fragments
  constexpr int VPRE = MODE == 4 ? 2 : 4;  // V^T fragments

  // ntiles >= 1 always (row 0 sees key 0).
  const int last_tile = ntiles - 1;
  // Block-table entries are vector loads (the load-to-LDS instruction is opaque to the
  // compiler, so it cannot prove the table unchanged and scalar), and waiting for one means
  // waiting for every tile load in flight.  So the entries of tile t + 3 are requested right
  // behind the loads issued in iteration t and read after the barrier of iteration t + 1, where
  // everything in flight has landed anyway; K(t + 2) and, one iteration later, V(t + 2) use them.
  struct Requested {
    int raw[NLK > 0 ? NLK : 1];
  };
  auto request = [&](int kt) {
    Requested r = {};
    if constexpr (NLK > 0) {
      const int t = min(kt, last_tile);  // past the end: any valid entry, never used
#pragma unroll
      for (int j = 0; j < NLK; ++j) r.raw[j] = a.pt[(int64_t)b * a.pt_rs + div_block(a, lookup_key(t, j))];
    }
    return r;
  };
  auto resolve = [&](const Requested &r) {
    Blocks blk = {};
    if constexpr (NLK > 0) {
#pragma unroll
      for (int j = 0; j < NLK; ++j) {
        const int p = MODE == 4 ? r.raw[j] : __builtin_amdgcn_readfirstlane(r.raw[j]);  // mode 4: per lane
        blk.phys[j] = (unsigned)p >= (unsigned)a.nb ? 0 : p;
      }
    }
    return blk;
  };
  auto kbuf = [&](int t) { return t & 1; };
  auto vbuf = [&](int t) { return t & 1; };
  int kt_begin = first_tile;
  Blocks blk_v = resolve(request(first_tile));     // blocks of the tile whose V is loaded next
  Blocks blk_k = resolve(request(first_tile + 1));  // ... whose K is loaded next
  Requested req = request(first_tile + 2);
  if constexpr (MODE == 4) {
    commit_bfp8(fetch_bfp8(a.k, first_tile, blk_v), false, first_tile & 1);
    commit_bfp8(fetch_bfp8(a.v, first_tile, blk_v), true, first_tile & 1);
    if (last_tile >= first_tile + 1)
      commit_bfp8(fetch_bfp8(a.k, first_tile + 1, blk_k), false, (first_tile + 1) & 1);
  } else {
    issue(a.k, ld_k, false, first_tile, kbuf(first_tile), blk_v);
    issue(a.v, ld_v, true, first_tile, vbuf(first_tile), blk_v);
    if (last_tile >= first_tile + 1) issue(a.k, ld_k, false, first_tile + 1, kbuf(first_tile + 1), blk_k);
  }
  blk_v = blk_k;
  wait_loads_and_sync();
  // The first K fragments of a tile are read one tile ahead (K(t+1) has landed at the barrier
  // of tile t), so the score product starts without waiting for LDS.
  bf16x8 ring[KPRE];
  if (wave_active && kt_begin < ntiles) {
#pragma unroll
    for (int i = 0; i < KPRE; ++i) ring[i] = read_k(smem + (kt_begin & 1) * T::STAGE_BYTES, i);
  }
  for (int kt = kt_begin; kt < ntiles; ++kt) {
    const unsigned char *cur = smem + (kt & 1) * T::STAGE_BYTES;
    const int key0 = kt * kKeysPerTile;
    // wavefront-uniform; with a window, tiles wholly below this wavefront's rows are skipped
    const bool compute = wave_active && key0 <= wave_last_key && key0 + kKeysPerTile > wave_first_key;

    // ---- S^T = K . Q^T -------------------------------------------------------------------
    floatx16 st[RH][2];
    if (compute) {
#pragma unroll
      for (int x = 0; x < RH; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[x][0][r] = 0.f, st[x][1][r] = 0.f;
#pragma unroll
      for (int i = 0; i < NK; ++i) {
#pragma unroll
        for (int x = 0; x < RH; ++x)
          st[x][i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % KPRE], qf[x][i >> 1], st[x][i & 1], 0, 0, 0);
        if (i + KPRE < NK) ring[i % KPRE] = read_k(cur, i + KPRE);
      }
      // pin the order: one fragment read behind the matrix instructions that use a fragment
#pragma unroll
      for (int i = 0; i < NK; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, RH, 0);
        if (i + KPRE < NK) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    // K(kt+1) and V(kt) have landed for everyone; everyone is done with K(kt) and V(kt-1)
    wait_loads_and_sync();
    blk_k = resolve(req);  // blocks of tile kt + 2; blk_v holds those of tile kt + 1
    Staged k_staged = {}, v_staged = {};
    if constexpr (MODE == 4) {
      if (kt + 2 <= last_tile) k_staged = fetch_bfp8(a.k, kt + 2, blk_k);
      if (kt + 1 <= last_tile) v_staged = fetch_bfp8(a.v, kt + 1, blk_v);
    } else {
      if (kt + 2 <= last_tile) issue(a.k, ld_k, false, kt + 2, kt & 1, blk_k);
      if (kt + 1 <= last_tile) issue(a.v, ld_v, true, kt + 1, (kt + 1) & 1, blk_v);
    }
    blk_v = blk_k;
    req = request(kt + 3);

    if (compute) {
      bf16x8 vring[VPRE];
#pragma unroll
      for (int j = 0; j < VPRE; ++j) vring[j] = read_v(cur + T::TILE_BYTES, j);

      // ---- mask, online softmax (one query row per lane and row block) ----------------------
      // The softmax scale is positive, so the running maximum is tracked on raw scores and
      // the scale is folded into the exponent: p = exp2(s * c - m * c).
      const bool need_mask = (a.causal && key0 + kKeysPerTile - 1 > offset + row0) ||
                             key0 + kKeysPerTile > a.skv || a.mask != nullptr ||
                             (a.window > 0 && key0 <= offset + row0 + ROWS - 1 - a.window);
      bf16x8 pf[RH][4];
#pragma unroll
      for (int x = 0; x < RH; ++x) {
        const int qrow = row0 + 32 * x + n;
        if (need_mask) {  // wavefront-uniform: only diagonal / ragged / window-edge / explicitly masked tiles
          const int limit = a.causal ? min(offset + qrow, a.skv - 1) : a.skv - 1;
          const int lowest = a.window > 0 ? offset + qrow - a.window + 1 : 0;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * h + (r & 3);
              float v = st[x][kb][r];
              if (a.mask) {
                const int kc = min(key, a.skv - 1), qc = min(qrow, a.sq - 1);
                // additive mask is in natural-log units of the scaled score
                v += bf16_lo(a.mask[b * a.mask_bs + (int64_t)qc * a.mask_rs + kc]) *
                     (1.4426950408889634f / a.scale_log2e);
              }
              st[x][kb][r] = (key > limit || key < lowest) ? -INFINITY : v;
            }
        }
        // The first maximum is an ordinary compiler-visible read of both score blocks.
        float mloc = fmaxf(st[x][0][0], st[x][1][0]);
#pragma unroll
        for (int r = 1; r < 16; r += 3) {
          mloc = max3(mloc, st[x][0][r], st[x][1][r]);
          mloc = max3(mloc, st[x][0][r + 1], st[x][1][r + 1]);
          mloc = max3(mloc, st[x][0][r + 2], st[x][1][r + 2]);
        }
        {  // The other half of the key rows sits 32 lanes away.  v_permlane32_swap exchanges the
           // upper 32 lanes of its first operand with the lower 32 of its second; with two copies
           // of the value each lane ends up holding its own and its partner's.  Written as
           // assembly: through the builtin the compiler folds the two results into one.
          float ma = mloc, mb = mloc;
          asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(ma), "+v"(mb));
          mloc = max3(ma, mb, mb);
        }
        // Lazy rescaling: the running maximum only moves when a row's new maximum exceeds it
        // by more than 2^8 in the exponent domain.  Until then probabilities are taken
        // relative to the stale maximum (they may reach 2^8, harmless in bf16 / fp32), the
        // accumulators need no rescale, and the final division by the row sum is unchanged.
        const float kLazy = 8.0f;
        const bool move = !((mloc - m_run[x]) * a.scale_log2e <= kLazy);  // also true from -inf
        const float m_new = move ? mloc : m_run[x];
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = move ? __builtin_amdgcn_exp2f((m_run[x] - m_safe) * a.scale_log2e) : 1.0f;
        const float mc = m_safe * a.scale_log2e;
        m_run[x] = m_new;
        // skip the accumulator rescale when no row of the block moved its maximum
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int i = 0; i < DBLK; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[x][i][r] *= alpha;
        }
        // Probabilities as bf16 B-operand fragments: element e of key step k4 = 2 kb + s is
        // accumulator register 8 s + e of score block kb.  The row sum is taken over the rounded
        // values (two per v_dot2_f32_bf16), i.e. over exactly what the second product sees.
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        float lsum = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const int r = 8 * (k4 & 1) + e;
            const float p0 = __builtin_amdgcn_exp2f(fmaf(st[x][k4 >> 1][r], a.scale_log2e, -mc));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(st[x][k4 >> 1][r + 1], a.scale_log2e, -mc));
            const bf16x2 pp = {(__bf16)p0, (__bf16)p1};
            pf[x][k4][e] = pp[0], pf[x][k4][e + 1] = pp[1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(pp, ones, lsum, false);
          }
        l_run[x] = l_run[x] * alpha + lsum;
      }

      // ---- O^T += V^T . P^T -----------------------------------------------------------------
#pragma unroll
      for (int j = 0; j < NV; ++j) {
#pragma unroll
        for (int x = 0; x < RH; ++x)
          acc[x][j % DBLK] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vring[j % VPRE], pf[x][j / DBLK],
                                                                     acc[x][j % DBLK], 0, 0, 0);
        if (j + VPRE < NV) vring[j % VPRE] = read_v(cur + T::TILE_BYTES, j + VPRE);
      }
    }
    if constexpr (MODE == 4) {
      // K(kt+2) takes the place of K(kt), V(kt+1) that of V(kt-1): nobody reads either any more
      // (the barrier above), and the next barrier publishes what is written here
      if (kt + 2 <= last_tile) commit_bfp8(k_staged, false, kt & 1);
      if (kt + 1 <= last_tile) commit_bfp8(v_staged, true, (kt + 1) & 1);
    }
    if (wave_active && kt + 1 < ntiles && key0 + kKeysPerTile <= wave_last_key &&
        key0 + 2 * kKeysPerTile > wave_first_key) {  // this wavefront computes tile kt + 1
      const unsigned char *nxt = smem + ((kt + 1) & 1) * T::STAGE_BYTES;
#pragma unroll
      for (int i = 0; i < KPRE; ++i) ring[i] = read_k(nxt, i);
    }
  }

  // ---- normalise and store: lane (n, h) holds head-dim elements 32 db + 8 j + 4 h + i ----
  if (!wave_active) return;
#pragma unroll
  for (int x = 0; x < RH; ++x) {
    const float l_tot = l_run[x] + __shfl_xor(l_run[x], 32);
    const float inv = 1.0f / l_tot;
    const int qrow = row0 + 32 * x + n;
    if (qrow >= a.sq) continue;
    uint16_t *op = a.out + b * a.out_bs + hq * a.out_hs + (int64_t)qrow * a.out_ts + 4 * h;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t lo = f32_to_bf16_bits(acc[x][db][4 * j] * inv) |
                      (f32_to_bf16_bits(acc[x][db][4 * j + 1] * inv) << 16);
        uint32_t hi = f32_to_bf16_bits(acc[x][db][4 * j + 2] * inv) |
                      (f32_to_bf16_bits(acc[x][db][4 * j + 3] * inv) << 16);
        *reinterpret_cast<uint2 *>(op + 32 * db + 8 * j) = make_uint2(lo, hi);
      }
  }
}

template <int D, int HPW, int MODE, int RH>
int launch_mode(const PrefillArgs &a, hipStream_t st) {
  constexpr int RPW = 4 / HPW;
  constexpr int ROWS = kRowsPerWave * RH;
  const int nqt = (a.sq + ROWS * RPW - 1) / (ROWS * RPW);
  // two stages of a K and a V tile
  // (the hand-scheduled loop keeps two rings of five 8 KiB blocks)
  constexpr bool kStreams = D == 128 && HPW == 4 && RH == 1 && (MODE == 0 || MODE == 1);
  const size_t lds = kStreams ? (size_t)TTPA_STREAM_LDS_BYTES : 2 * Tile<D>::STAGE_BYTES;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_dynamic_lds(reinterpret_cast<const void *>(&prefill_kernel<D, HPW, MODE, RH>), lds, lds_ready))
    return fail(TTPA_ERR_LAUNCH, "prefill: cannot reserve %zu bytes of LDS", lds);
  const int ny8 = (a.batch * (a.hq / HPW) + 7) / 8;
  PrefillArgs b = a;
  // The hand-scheduled loop takes launches of whole 32-key blocks without a window or an explicit mask
  // (a dense K / V that ends inside a 64-key tile goes through the plain loop).  One workgroup per
  // block of 32 query rows and head group, heavy blocks first, and the dispatcher deals them to the CUs
  // as slots free up: the loop can also give a workgroup several row blocks (spg workgroups per group,
  // TTPA_PREFILL_WGS_PER_GROUP), but one round of two workgroups per CU measured 204 us against 150 on
  // the 4 x 2048-token causal workload (a change of row block costs a workgroup about 4 us in which
  // nothing of its own overlaps, and a static deal cannot make up for workgroups that start late).
  b.stream = kStreams && a.stream && a.window == 0 && a.mask == nullptr && (MODE == 1 || a.skv % kKeysPerTile == 0);
  b.spg = b.spg_even = 0;
  int per_group = nqt;
  if (b.stream) {
    b.spg = nqt;
    // Row blocks of nearly one weight (a chunk far into its sequence, or no causal mask) that fill the
    // chip more than once: one round of workgroups with equal shares instead, which saves the later
    // rounds' start-up (267 -> 261 us on 4 x 512-token chunks behind 4096 tokens, 64 heads).  The
    // chunk's start is in device memory, so the kernel decides: the workgroups past the round exit.
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    const int one_round = (2 * cus + ny8 * 8 - 1) / (ny8 * 8);
    b.spg_even = one_round < nqt && nqt % one_round == 0 ? one_round : 0;
    if (const char *e = getenv("TTPA_PREFILL_WGS_PER_GROUP")) {  // (read on every call) an experiment's override
      if (atoi(e) > 0) b.spg = std::min(nqt, atoi(e)), b.spg_even = 0;
    }
    per_group = b.spg;
  }
  int grid = per_group * ny8 * 8;
  if (MODE == 0 && a.fill_kc) {
    // The fill workgroups are spread over the launch in groups of 8, one group behind every
    // attn_per_fill groups of attention workgroups, so that their memory traffic runs while the
    // neighbouring workgroups keep the matrix pipes busy (all of them at the end of the launch
    // cost as much as two separate fills).
    b.n_fill = 2 * a.batch * a.hkv * ((a.skv + fill_rows_per_wg(D) - 1) / fill_rows_per_wg(D));
    const int fg = (b.n_fill + 7) / 8, ag = grid / 8;
    b.fill_groups = fg;
    b.attn_per_fill = ag >= fg ? ag / fg : 1;
    // fewer attention groups than fill groups: one of each per super-group, and the attention
    // slots past the last real one exit at once (the kernel's range check)
    grid = ag >= fg ? grid + 8 * fg : 16 * fg;
  }
  launch_dominant(&prefill_kernel<D, HPW, MODE, RH>, dim3(grid), dim3(256), lds, st, b);
  return check_launch("sdpa_prefill");
}

template <int D, int HPW, int RH>
int launch_rh(const PrefillArgs &a, hipStream_t st) {
  if (!a.pt) return launch_mode<D, HPW, 0, RH>(a, st);
  if (a.bs % kKeysPerTile == 0) return launch_mode<D, HPW, 1, RH>(a, st);
  if (a.bs % Tile<D>::RPI == 0) return launch_mode<D, HPW, 3, RH>(a, st);
  return launch_mode<D, HPW, 2, RH>(a, st);
}

// Bytes of the scratch an expanded block-float-8 pass needs: K and V copies of batch * width blocks
// and their table.
inline int64_t expand_bytes(int batch, int width, int kv_heads, int block_size, int d) {
  const int64_t blocks = (int64_t)batch * width;
  return 2 * blocks * kv_heads * block_size * d * 2 + ((blocks * 4 + 255) & ~int64_t(255));
}

template <int D, int HPW>
int launch(const PrefillArgs &a, hipStream_t st) {
  if (a.pt && a.kv_bfp8) {
    // With scratch from the caller, a pass that the hand-scheduled loop can serve reads bfloat16
    // copies of its blocks (written by one launch in front of it) instead of expanding every
    // tile once per workgroup on its way into LDS.
    constexpr bool kStreams = D == 128 && HPW == 4;
    if (kStreams && a.expand && a.stream && a.window == 0 && a.mask == nullptr && a.bs % kKeysPerTile == 0) {
      const int64_t blocks = (int64_t)a.batch * a.w;
      const int64_t cache_elems = blocks * a.hkv * a.bs * D;
      ExpandArgs e;
      e.kc = reinterpret_cast<const uint8_t *>(a.k), e.vc = reinterpret_cast<const uint8_t *>(a.v);
      e.k = static_cast<uint16_t *>(a.expand), e.v = e.k + cache_elems;
      e.table = reinterpret_cast<int32_t *>(e.v + cache_elems);
      e.pt = a.pt, e.pt_rs = a.pt_rs, e.chunk_start = a.chunk_start;
      e.w = a.w, e.hkv = a.hkv, e.bs = a.bs, e.nb = a.nb, e.sq = a.sq, e.causal = a.causal;
      // armed events: the pair brackets both launches
      hipEvent_t before, after;
      take_profile_events(before, after);
      const dim3 grid((unsigned)blocks, (unsigned)(2 * a.hkv));
      if (before)
        hipExtLaunchKernelGGL(bfp8_expand_kernel<D>, grid, dim3(256), 0u, st, before, nullptr, 0u, e);
      else
        bfp8_expand_kernel<D><<<grid, dim3(256), 0, st>>>(e);
      if (const int rc = check_launch("sdpa_prefill (block-float-8 expansion)")) return rc;
      if (after) arm_profile_events(nullptr, after);
      PrefillArgs b = a;
      b.k = e.k, b.v = e.v, b.pt = e.table, b.pt_rs = a.w, b.nb = (int)blocks, b.kv_bfp8 = 0, b.expand = nullptr;
      return launch_mode<D, HPW, 1, 1>(b, st);
    }
    return launch_mode<D, HPW, 4, 1>(a, st);
  }
  return launch_rh<D, HPW, 1>(a, st);
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

// The cache fill that a dense prefill may carry along (ttpa_sdpa_prefill_fill).
struct FillSpec {
  void *k_cache, *v_cache;
  const int32_t *pt;
  int64_t pt_rs;
  const void *bidx;
  int bidx_i64, table_rows;
};

static int prefill_impl(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                                 int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                                 int64_t q_head_stride, int64_t q_token_stride, const void *k,
                                 const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                                 int64_t kv_token_stride, const int32_t *page_table,
                                 int64_t page_table_row_stride, const int32_t *chunk_start,
                                 const void *mask, int64_t mask_batch_stride,
                                 int64_t mask_row_stride, int32_t batch, int32_t q_heads,
                                 int32_t kv_heads, int32_t q_len, int32_t kv_len, int32_t head_size,
                                 int32_t block_size, int32_t table_width, int32_t num_blocks,
                                 int32_t causal, float scale, int32_t sliding_window, void *stream,
                                 const FillSpec *fill = nullptr, int32_t kv_format = TTPA_KV_BF16,
                                 void *workspace = nullptr, int64_t workspace_bytes = 0) {
  TTPA_REQUIRE(out && q && k && v, "null pointer argument");
  TTPA_REQUIRE(sliding_window >= 0, "prefill: sliding_window %d is negative", sliding_window);
  TTPA_REQUIRE(sliding_window == 0 || causal, "prefill: a sliding window needs causal masking");
  TTPA_REQUIRE(batch > 0 && q_heads > 0 && kv_heads > 0 && q_len > 0 && head_size > 0,
               "non-positive dimension");
  TTPA_REQUIRE(q_heads % kv_heads == 0, "q_heads %d not divisible by kv_heads %d", q_heads,
               kv_heads);
  if (head_size != 64 && head_size != 128 && head_size != 256)
    return fail(TTPA_ERR_UNSUPPORTED, "prefill: head_size %d; supported 64, 128, 256", head_size);
  TTPA_REQUIRE(!(mask && causal), "an additive mask excludes causal masking");
  // the running maximum is tracked on raw scores and the mask is brought to their units by a
  // division: both need a positive scale
  TTPA_REQUIRE(scale > 0.f, "prefill: scale %g must be positive", (double)scale);
  if (page_table) {
    TTPA_REQUIRE(block_size > 0 && table_width > 0 && num_blocks > 0,
                 "paged form needs block_size, table_width and num_blocks");
    kv_len = table_width * block_size;
    TTPA_REQUIRE((int64_t)kv_len * block_size < (1ll << 32), "prefill: table_width * block_size^2 must stay below 2^32");
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
  TTPA_REQUIRE((int64_t)batch * q_heads * ((q_len + 31) / 32) < (1ll << 30),
               "prefill: batch * heads * query tiles too large for one launch");

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
  a.window = sliding_window;
  a.scale_log2e = scale * 1.4426950408889634f;
  if (kv_format != TTPA_KV_BF16 && kv_format != TTPA_KV_BFP8)
    return fail(TTPA_ERR_INVALID_ARGUMENT, "prefill: unknown kv_format %d", kv_format);
  a.kv_bfp8 = kv_format == TTPA_KV_BFP8;
  a.expand = nullptr;
  if (a.kv_bfp8) {
    TTPA_REQUIRE(page_table != nullptr, "prefill: a block-float-8 K / V is a paged cache");
    if (block_size % 16)
      return fail(TTPA_ERR_UNSUPPORTED, "prefill: a block-float-8 cache needs block_size %% 16 == 0");
    TTPA_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0),
                 "prefill: workspace_bytes %lld with a null workspace", (long long)workspace_bytes);
    if (workspace && aligned16(workspace) && (int64_t)batch * table_width < (1ll << 31) &&
        workspace_bytes >= expand_bytes(batch, table_width, kv_heads, block_size, head_size))
      a.expand = workspace;  // (a smaller one is not an error: the pass expands tile by tile instead)
  }
  {
    // (TTPA_PREFILL_STREAM=0, read on every call, sends every shape through the plain loop)
    const char *e = getenv("TTPA_PREFILL_STREAM");
    a.stream = e ? atoi(e) : 1;
  }
  a.bs_magic = block_size >= 2 ? (uint32_t)((1ull << 32) / (uint32_t)block_size) + 1u : 0u;
  a.fill_kc = a.fill_vc = nullptr;
  a.fill_pt = nullptr, a.fill_pt_rs = 0, a.fill_bidx = nullptr, a.fill_bidx_i64 = 0, a.fill_rows = 0;
  a.fill_groups = a.attn_per_fill = a.n_fill = 0;
  if (fill) {
    a.fill_kc = static_cast<uint16_t *>(fill->k_cache), a.fill_vc = static_cast<uint16_t *>(fill->v_cache);
    a.fill_pt = fill->pt, a.fill_pt_rs = fill->pt_rs;
    a.fill_bidx = fill->bidx, a.fill_bidx_i64 = fill->bidx_i64, a.fill_rows = fill->table_rows;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (head_size) {
    case 64: return launch_d<64>(a, st);
    case 128: return launch_d<128>(a, st);
    default: return launch_d<256>(a, st);
  }
}

#define TTPA_PREFILL_PARAMS                                                                        \
  void *out, int64_t out_batch_stride, int64_t out_head_stride, int64_t out_token_stride,          \
      const void *q, int64_t q_batch_stride, int64_t q_head_stride, int64_t q_token_stride,        \
      const void *k, const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,               \
      int64_t kv_token_stride, const int32_t *page_table, int64_t page_table_row_stride,           \
      const int32_t *chunk_start, const void *mask, int64_t mask_batch_stride,                     \
      int64_t mask_row_stride, int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,    \
      int32_t kv_len, int32_t head_size, int32_t block_size, int32_t table_width,                  \
      int32_t num_blocks, int32_t causal, float scale
#define TTPA_PREFILL_ARGS                                                                          \
  out, out_batch_stride, out_head_stride, out_token_stride, q, q_batch_stride, q_head_stride,      \
      q_token_stride, k, v, kv_batch_stride, kv_head_stride, kv_token_stride, page_table,          \
      page_table_row_stride, chunk_start, mask, mask_batch_stride, mask_row_stride, batch,         \
      q_heads, kv_heads, q_len, kv_len, head_size, block_size, table_width, num_blocks, causal,    \
      scale

extern "C" int ttpa_sdpa_prefill(TTPA_PREFILL_PARAMS, void *stream) {
  return prefill_impl(TTPA_PREFILL_ARGS, 0, stream);
}

extern "C" int ttpa_sdpa_prefill_windowed(TTPA_PREFILL_PARAMS, int32_t sliding_window, void *stream) {
  return prefill_impl(TTPA_PREFILL_ARGS, sliding_window, stream);
}

extern "C" int ttpa_sdpa_prefill_format(TTPA_PREFILL_PARAMS, int32_t sliding_window, int32_t kv_format,
                                        void *stream) {
  return prefill_impl(TTPA_PREFILL_ARGS, sliding_window, stream, nullptr, kv_format);
}

extern "C" int ttpa_sdpa_prefill_expanded(TTPA_PREFILL_PARAMS, int32_t sliding_window, int32_t kv_format,
                                          void *workspace, int64_t workspace_bytes, void *stream) {
  return prefill_impl(TTPA_PREFILL_ARGS, sliding_window, stream, nullptr, kv_format, workspace, workspace_bytes);
}

extern "C" int64_t ttpa_sdpa_prefill_workspace_bytes(int32_t batch, int32_t kv_heads, int32_t head_size,
                                                     int32_t block_size, int32_t table_width, int32_t kv_format) {
  if (kv_format != TTPA_KV_BFP8 || batch <= 0 || kv_heads <= 0 || head_size <= 0 || block_size <= 0 || table_width <= 0)
    return 0;
  return expand_bytes(batch, table_width, kv_heads, block_size, head_size);
}

extern "C" int ttpa_sdpa_prefill_fill(
    void *out, int64_t out_batch_stride, int64_t out_head_stride, int64_t out_token_stride,
    const void *q, int64_t q_batch_stride, int64_t q_head_stride, int64_t q_token_stride,
    const void *k, const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
    int64_t kv_token_stride, int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,
    int32_t kv_len, int32_t head_size, int32_t causal, float scale, int32_t sliding_window,
    void *k_cache, void *v_cache, const int32_t *fill_page_table, int64_t fill_page_table_row_stride,
    const void *batch_idx, int batch_idx_is_i64, int32_t table_rows, int32_t block_size,
    int32_t table_width, int32_t num_blocks, void *stream) {
  TTPA_REQUIRE(k_cache && v_cache && fill_page_table, "prefill + fill: null cache / page_table pointer");
  TTPA_REQUIRE(block_size > 0 && table_width > 0 && num_blocks > 0 && table_rows > 0,
               "prefill + fill: non-positive cache geometry");
  TTPA_REQUIRE(batch_idx != nullptr || batch <= 1, "batch_idx may only be omitted for a single-user fill");
  TTPA_REQUIRE((int64_t)kv_len <= (int64_t)table_width * block_size,
               "kv_len %d does not fit %d page-table columns of %d tokens", kv_len, table_width, block_size);
  TTPA_REQUIRE((int64_t)kv_len * block_size < (1ll << 32), "prefill + fill: kv_len * block_size must stay below 2^32");
  TTPA_REQUIRE(aligned16(k_cache) && aligned16(v_cache), "prefill + fill: caches must be 16-byte aligned");
  const FillSpec fill{k_cache, v_cache, fill_page_table, fill_page_table_row_stride, batch_idx,
                      batch_idx_is_i64, table_rows};
  return prefill_impl(out, out_batch_stride, out_head_stride, out_token_stride, q, q_batch_stride,
                      q_head_stride, q_token_stride, k, v, kv_batch_stride, kv_head_stride,
                      kv_token_stride, nullptr, 0, nullptr, nullptr, 0, 0, batch, q_heads, kv_heads,
                      q_len, kv_len, head_size, block_size, table_width, num_blocks, causal, scale,
                      sliding_window, stream, &fill);
}
