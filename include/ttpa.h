/*
 * ttpa — paged KV-cache write and paged attention for MI355X (gfx950).
 *
 * C ABI of libttpa.so.  These entry points are what the device branch of the
 * reference's five custom ops binds to; each comment names the reference
 * interface the function replaces (paths relative to the tt-xla tree).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - activations and bf16 caches are bfloat16, indices int32 unless an
 *     `_is_i64` flag says otherwise; strides are in ELEMENTS, the innermost
 *     (head_size) dimension is always contiguous;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - calls only enqueue work: they never synchronise, never allocate and never
 *     touch the caller's buffers from the host;
 *   - return value: TTPA_OK, or a negative TTPA_ERR_*; ttpa_last_error() returns
 *     a thread-local, human-readable reason for the last failure.
 *
 * Cache layout (reference: TTAttentionBackend.get_kv_cache_shape,
 * integrations/vllm_plugin/vllm_tt/attention_impls/attention.py:104-112):
 *   TTPA_KV_BF16  bfloat16 [num_blocks, kv_heads, block_size, head_size]
 *   TTPA_KV_BFP8  uint8    [num_blocks, kv_heads, block_size + block_size/16, head_size]
 *                 rows 0..block_size-1: one byte b = 128 + v per element, v the signed
 *                 7-bit mantissa in [-127, 127] (offset binary);
 *                 the remaining bytes, read as [block_size][head_size/16], hold one
 *                 shared exponent byte per 16 consecutive head_size elements;
 *                 value = (b - 128) * 2^(e - 133).
 * K and V are two separate tensors of that layout.
 */
#ifndef TTPA_H_
#define TTPA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTPA_ABI_VERSION 1

#define TTPA_OK 0
#define TTPA_ERR_INVALID_ARGUMENT (-1) /* shape / stride / alignment the kernels cannot take */
#define TTPA_ERR_UNSUPPORTED (-2)      /* valid request, no kernel instantiated for it */
#define TTPA_ERR_WORKSPACE (-3)        /* workspace missing or too small */
#define TTPA_ERR_LAUNCH (-4)           /* HIP reported an error at launch */

#define TTPA_KV_BF16 0
#define TTPA_KV_BFP8 1

int ttpa_abi_version(void);
const char *ttpa_last_error(void);

/* Number of compute units of the current device (used to size persistent grids). */
int ttpa_device_compute_units(void);

/*
 * One-token-per-user scatter, IN PLACE on `cache`.
 * Replaces the device branch of tt::paged_update_cache
 * (python_package/tt_torch/custom_ops.py:962-1002; CPU semantics :981-1000):
 *   col = floor(idx[u] / block_size), off = idx[u] mod block_size (floor semantics,
 *   col < 0 wraps once by table_width like a negative Python index);
 *   cache[page_table[u, col], h, off, :] = fill[u, h, :]  for h < kv_heads.
 * fill is the [1, users, >=kv_heads, head_size] operand addressed through
 * fill_user_stride / fill_head_stride.  Users whose column or physical block falls
 * outside the table / the cache are skipped (the reference raises IndexError).
 * With TTPA_KV_BFP8 the bf16 row is encoded on the way in.
 * The functional form of the op (fresh result tensor) is clone + this call.
 */
int ttpa_paged_update_cache(void *cache, const void *fill, int64_t fill_user_stride,
                            int64_t fill_head_stride, const void *update_indices,
                            int indices_is_i64, const int32_t *page_table,
                            int64_t page_table_row_stride, int32_t users, int32_t kv_heads,
                            int32_t block_size, int32_t head_size, int32_t table_width,
                            int32_t num_blocks, int32_t kv_format, void *stream);

/*
 * The decode step's two scatters in one launch: ttpa_paged_update_cache applied to the K cache
 * with k_fill and to the V cache with v_fill (same indices, same page table, same geometry,
 * same fill strides).  The reference issues the op twice
 * (vllm_tt/attention_impls/attention.py:473-484); the result is identical.
 */
int ttpa_paged_update_cache_kv(void *k_cache, void *v_cache, const void *k_fill, const void *v_fill,
                               int64_t fill_user_stride, int64_t fill_head_stride,
                               const void *update_indices, int indices_is_i64,
                               const int32_t *page_table, int64_t page_table_row_stride,
                               int32_t users, int32_t kv_heads, int32_t block_size,
                               int32_t head_size, int32_t table_width, int32_t num_blocks,
                               int32_t kv_format, void *stream);

/*
 * Block-wise prefill write, IN PLACE on `cache`.
 * Replaces the device branch of tt::paged_fill_cache (custom_ops.py:1016-1094; CPU
 * semantics for one user :1037-1092; batched call site
 * vllm_tt/attention_impls/attention.py:486-511):
 *   for i < fill_users, t < seq_len:
 *     cache[page_table[batch_idx[i], t / block_size], h, t % block_size, :] = fill[i, h, t, :]
 * Writing always starts at table column 0; rows of the last block past seq_len keep
 * their contents.  batch_idx may be NULL (= user 0, fill_users must then be 1).
 * seq_len > table_width * block_size is rejected.  batch_idx values outside
 * [0, table_rows) and physical blocks outside the cache are skipped.
 */
int ttpa_paged_fill_cache(void *cache, const void *fill, int64_t fill_user_stride,
                          int64_t fill_head_stride, int64_t fill_token_stride,
                          const int32_t *page_table, int64_t page_table_row_stride,
                          const void *batch_idx, int batch_idx_is_i64, int32_t fill_users,
                          int32_t table_rows, int32_t kv_heads, int32_t seq_len,
                          int32_t block_size, int32_t head_size, int32_t table_width,
                          int32_t num_blocks, int32_t kv_format, void *stream);

/*
 * ttpa_paged_fill_cache on the K cache and on the V cache in one launch: a prefill pass of
 * the backend fills both with the same table and batch_idx (attention.py:500-511).  k_fill
 * and v_fill share their strides.  Same result as the two calls.
 */
int ttpa_paged_fill_cache_kv(void *k_cache, void *v_cache, const void *k_fill, const void *v_fill,
                             int64_t fill_user_stride, int64_t fill_head_stride,
                             int64_t fill_token_stride, const int32_t *page_table,
                             int64_t page_table_row_stride, const void *batch_idx,
                             int batch_idx_is_i64, int32_t fill_users, int32_t table_rows,
                             int32_t kv_heads, int32_t seq_len, int32_t block_size,
                             int32_t head_size, int32_t table_width, int32_t num_blocks,
                             int32_t kv_format, void *stream);

/*
 * Causal paged decode attention, one query token per user.
 * Replaces the device branch of tt::paged_scaled_dot_product_attention_decode
 * (custom_ops.py:1198-1315; CPU semantics :1256-1312, grouped heads as in :551-610):
 *   out[u, hq, :] = softmax_j( scale * q[u, hq, :] . K[u, hq / G, j, :] ) . V[u, hq / G, j, :]
 *   over cache positions j = 0 .. min(cur_pos[u], table_width * block_size - 1),
 *   position j living in block page_table[u, j / block_size], row j % block_size.
 * cur_pos[u] < 0 (padded batch row) gives a NaN output row, as on the reference.
 * (The operator's other form, is_causal = False with an additive attn_mask over all positions
 * of the table, custom_ops.py:1299-1303, needs no entry point of its own: the host side gathers
 * the user's blocks and calls ttpa_sdpa_prefill's masked dense form, see tt_xla_amd/custom_ops.py.)
 * Physical block ids outside [0, num_blocks) are read as block 0.
 * `workspace` holds split-K partial results: at least
 * ttpa_paged_decode_workspace_bytes(...) bytes, 256-byte aligned, private to this
 * call until the stream reaches its end.
 * Built shapes (anything else returns TTPA_ERR_UNSUPPORTED): head_size 64, 128 or 256;
 * block_size a multiple of 4; at most 2048 users; G = q_heads / kv_heads up to 8, and
 * up to 16 (head_size 64 / 128 with at most 1024 users: up to 32) with block_size a multiple
 * of 1024 / (bytes of a cache row) (8 rows for head_size 64, 4 for 128, 2 for 256;
 * block-float-8: 16, 8 and 4).  TTPA_KV_BFP8: block_size a multiple of 16 (head_size 256: G up
 * to 16).
 */
size_t ttpa_paged_decode_workspace_bytes(int32_t users, int32_t q_heads, int32_t kv_heads,
                                         int32_t head_size);

int ttpa_paged_sdpa_decode(void *out, int64_t out_user_stride, int64_t out_head_stride,
                           const void *q, int64_t q_user_stride, int64_t q_head_stride,
                           const void *k_cache, const void *v_cache,
                           const int32_t *page_table, int64_t page_table_row_stride,
                           const void *cur_pos, int cur_pos_is_i64, int32_t users,
                           int32_t q_heads, int32_t kv_heads, int32_t head_size,
                           int32_t block_size, int32_t table_width, int32_t num_blocks,
                           float scale, int32_t kv_format, void *workspace,
                           size_t workspace_bytes, void *stream);

/*
 * The same decode attention with the two arguments of
 * tt::paged_scaled_dot_product_attention_decode that the reference forwards to its device
 * kernel and its CPU branch ignores (custom_ops.py:1207-1209, 1233-1247; the backend passes
 * them at attention.py:646-656):
 *   sliding_window > 0: only positions j > cur_pos[u] - sliding_window are attended
 *                       (the newest `sliding_window` positions, the current one included);
 *                       0 = no window.
 *   attention_sink:     [q_heads] float32 logits on the device, or NULL.  Head hq's sink is
 *                       one more entry of its softmax that contributes no value:
 *                       denominator += exp(attention_sink[hq] - max).  It is in the units of
 *                       the scaled scores (it is not multiplied by `scale`).
 * With sliding_window = 0 and attention_sink = NULL this is ttpa_paged_sdpa_decode.
 */
int ttpa_paged_sdpa_decode_windowed(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                    const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                    const void *k_cache, const void *v_cache,
                                    const int32_t *page_table, int64_t page_table_row_stride,
                                    const void *cur_pos, int cur_pos_is_i64, int32_t users,
                                    int32_t q_heads, int32_t kv_heads, int32_t head_size,
                                    int32_t block_size, int32_t table_width, int32_t num_blocks,
                                    float scale, int32_t kv_format, int32_t sliding_window,
                                    const float *attention_sink, void *workspace,
                                    size_t workspace_bytes, void *stream);

/*
 * Decode with an explicit additive mask in place of the causal rule: the `is_causal=False` form
 * of tt::paged_scaled_dot_product_attention_decode (python_package/tt_torch/custom_ops.py:1296-1311,
 * attn_weight += attn_mask) and of tt::scaled_dot_product_attention_decode on a static cache
 * (custom_ops.py:817-842, where the mask differs between heads:
 * tests/torch/ops/test_custom_ops.py:126-130).  mask is bfloat16, added to the scaled scores;
 * the element for (user, query head, position) is mask[user * mask_user_stride +
 * head * mask_head_stride + position] (a head stride of 0 shares one row between the heads).
 * cur_pos[u] is the last position that is attended at all (the caller passes
 * table_width * block_size - 1 to attend every position of the table).  Built for up to 8 query
 * heads per KV head on bfloat16 caches (dot-product kernel) and up to 32 on either cache format
 * (kv_format as in ttpa_paged_sdpa_decode_windowed) where a matrix-core kernel applies (16x16x32 up
 * to 16 heads, 32x32x16 up to 32 at head sizes 64 / 128); other shapes return TTPA_ERR_UNSUPPORTED.
 * The rest as ttpa_paged_sdpa_decode.
 */
int ttpa_paged_sdpa_decode_masked(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                  const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                  const void *k_cache, const void *v_cache, const int32_t *page_table,
                                  int64_t page_table_row_stride, const void *cur_pos, int cur_pos_is_i64,
                                  int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
                                  int32_t block_size, int32_t table_width, int32_t num_blocks, float scale,
                                  int32_t kv_format, const void *mask, int64_t mask_user_stride,
                                  int64_t mask_head_stride, void *workspace, size_t workspace_bytes,
                                  void *stream);

/*
 * The decode step of the attention backend in one call: the cache update
 * (ttpa_paged_update_cache_kv with update_indices = cur_pos: the new token of user u goes to
 * position cur_pos[u]) followed by ttpa_paged_sdpa_decode_windowed on the updated caches
 * (vllm_tt/attention_impls/attention.py:473-483 followed by :634-668).  Results, in the
 * caches and in `out`, are those of the two calls in that order.  k_new / v_new are the
 * [1, users, >= kv_heads, head_size] bfloat16 operands of the update, addressed through
 * new_user_stride / new_head_stride.  Where the 16x16x32 decode kernel serves the shape
 * (head_size 64 / 128 with 2 ... 16 query heads per KV head or a block-float-8 cache; head_size
 * 256 with up to 16 query heads per KV head) the update runs
 * inside it: the wavefront that owns the tile of position cur_pos[u] takes the token from
 * k_new / v_new and stores it into the cache; otherwise the library issues the two launches.
 * The equivalence assumes that no user attends a cache row which ANOTHER user's token is
 * written to in the same step (rows are owned by one user in a paged cache; the writes of
 * padded rows go to the null block their zero table points to): inside one launch such a
 * read is not ordered after that write.
 * No counterpart as ONE operator in the reference, which issues the ops separately.
 */
int ttpa_paged_update_decode(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, void *k_cache, void *v_cache, const void *k_new,
    const void *v_new, int64_t new_user_stride, int64_t new_head_stride,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    int32_t sliding_window, const float *attention_sink, void *workspace, size_t workspace_bytes,
    void *stream);

/*
 * ttpa_paged_update_decode for callers that cannot hold a workspace: code under HIP graph
 * capture that may not call hipMalloc, tight serving loops, harnesses that forbid allocation.
 * It has no counterpart in the reference.  The split-K partial results go to a static array
 * inside the library's device image (ttpa_static_scratch_bytes() = 16 MiB per GPU the library
 * runs on, held until the process ends) instead of a caller buffer; the call allocates nothing.
 * Shapes whose ttpa_paged_decode_workspace_bytes(...) exceed that size are refused with
 * TTPA_ERR_WORKSPACE (config 2 needs 4.8 MB, config 4 12.8 MB).  The array's device address is
 * looked up once per device, at the first call on that device or by ttpa_static_scratch_init()
 * (call it with the device current, outside graph capture, if the first call would be captured).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
 * host threads) race; calls on one stream run in turn and need nothing cleared between them.
 * Results equal ttpa_paged_update_decode's.
 */
size_t ttpa_static_scratch_bytes(void);
int ttpa_static_scratch_init(void);
int ttpa_paged_update_decode_static(
    void *out, int64_t out_user_stride, int64_t out_head_stride, const void *q,
    int64_t q_user_stride, int64_t q_head_stride, void *k_cache, void *v_cache, const void *k_new,
    const void *v_new, int64_t new_user_stride, int64_t new_head_stride,
    const int32_t *page_table, int64_t page_table_row_stride, const void *cur_pos,
    int cur_pos_is_i64, int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
    int32_t block_size, int32_t table_width, int32_t num_blocks, float scale, int32_t kv_format,
    int32_t sliding_window, const float *attention_sink, void *stream);

/*
 * Paged decode attention for latent-style (multi-head latent attention) caches.
 * Replaces the device branch of tt::paged_flash_mla_decode
 * (python_package/tt_torch/custom_ops.py:381-632; CPU semantics :551-610), causal form:
 *   out[u, hq, :head_dim_v] = softmax_j( scale * q[u, hq, :] . K[u, hq / G, j, :] ) . V[u, hq / G, j, :]
 *   over cache positions j = 0 .. min(cur_pos[u], table_width * block_size - 1).
 * k_cache is [num_blocks, kv_heads, block_size, head_size] bf16.  v_cache is either a cache
 * [num_blocks, kv_heads, block_size, head_dim_v] or NULL: then V is the first head_dim_v
 * features of K (the latent path, custom_ops.py:573-575).  q is [users, q_heads, head_size]
 * by strides, out is [users, q_heads, head_dim_v] by strides.  Built shapes: head_size 64,
 * 128, 192, 576 with head_dim_v a multiple of 64 up to 512 (256 with a separate v_cache);
 * q_heads / kv_heads up to 32 or a multiple of 32.  attention_sink as in
 * ttpa_paged_sdpa_decode_windowed, or NULL.  cur_pos[u] < 0 gives a NaN row.
 * The prefill operator tt::flash_mla_prefill (custom_ops.py:223-378) is served by the same
 * entry point: query row i of a sequence is a user at position i (see tt_xla_amd/custom_ops.py).
 */
size_t ttpa_paged_mla_decode_workspace_bytes(int32_t users, int32_t q_heads, int32_t kv_heads,
                                             int32_t head_dim_v);

int ttpa_paged_mla_decode(void *out, int64_t out_user_stride, int64_t out_head_stride,
                          const void *q, int64_t q_user_stride, int64_t q_head_stride,
                          const void *k_cache, const void *v_cache, const int32_t *page_table,
                          int64_t page_table_row_stride, const void *cur_pos, int cur_pos_is_i64,
                          int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
                          int32_t head_dim_v, int32_t block_size, int32_t table_width,
                          int32_t num_blocks, float scale, const float *attention_sink,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same with an explicit additive mask (tt::paged_flash_mla_decode with is_causal=False,
 * custom_ops.py:590-608: additive_mask = attn_mask; tt::flash_mla_prefill with attn_mask,
 * custom_ops.py:343-357, served with query row i as user i).  mask as in
 * ttpa_paged_sdpa_decode_masked; scale must not be 0.  Runs on the workgroup-shared kernel for
 * every shape.
 */
int ttpa_paged_mla_decode_masked(void *out, int64_t out_user_stride, int64_t out_head_stride,
                                 const void *q, int64_t q_user_stride, int64_t q_head_stride,
                                 const void *k_cache, const void *v_cache, const int32_t *page_table,
                                 int64_t page_table_row_stride, const void *cur_pos, int cur_pos_is_i64,
                                 int32_t users, int32_t q_heads, int32_t kv_heads, int32_t head_size,
                                 int32_t head_dim_v, int32_t block_size, int32_t table_width,
                                 int32_t num_blocks, float scale, const void *mask, int64_t mask_user_stride,
                                 int64_t mask_head_stride, void *workspace, size_t workspace_bytes,
                                 void *stream);

/*
 * Measurement hook, no reference counterpart: the NEXT attention call made by this host
 * thread (decode or prefill) attaches `before` and `after` (hipEvent_t, as void*) to the
 * launch of its dominant kernel (the split-K main kernel for decode, the MFMA kernel for
 * prefill), so that they hold the dispatch's own begin and end timestamps, then forgets
 * them (the VALU, 32x32 and workgroup-shared latent kernels record them on the stream in
 * front of and behind the launch instead).  Pass NULLs to clear.  Used by bench.py to time
 * that kernel alone, the way a profiler's kernel trace does.
 */
int ttpa_profile_next_attention(void *before, void *after);

/*
 * Prefill attention (bf16 MFMA), dense or paged K/V, grouped heads.
 * Replaces the device branches of
 *   tt::scaled_dot_product_attention        (custom_ops.py:635-729; CPU :717-727) and
 *   tt::chunked_scaled_dot_product_attention (custom_ops.py:1334-1431; CPU :1376-1429).
 *   out[b, hq, i, :] = softmax_j( scale * q[b,hq,i,:] . K[b, hq/G, j, :] + mask ) . V[b, hq/G, j, :]
 * Dense form: page_table == NULL, k / v are [batch, kv_heads, kv_len, head_size]
 *   addressed by the kv_* strides.
 * Paged form: page_table != NULL, k / v are caches (bf16 layout above), kv_len is
 *   ignored and the keys of user b are positions 0 .. table_width*block_size-1.
 * Masking: causal != 0 allows key j for query row i iff j <= offset + i, where offset
 *   is *chunk_start (device int32, may be NULL = 0) in the paged form and 0 in the
 *   dense form (the library routine's top-left aligned causal mask).  `mask` (may be
 *   NULL, requires causal == 0) is an additive bf16 mask [batch, 1, q_len, kv_len]
 *   addressed by mask_batch_stride / mask_row_stride.  `scale` must be positive.
 */
int ttpa_sdpa_prefill(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                      int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                      int64_t q_head_stride, int64_t q_token_stride, const void *k,
                      const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                      int64_t kv_token_stride, const int32_t *page_table,
                      int64_t page_table_row_stride, const int32_t *chunk_start,
                      const void *mask, int64_t mask_batch_stride, int64_t mask_row_stride,
                      int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,
                      int32_t kv_len, int32_t head_size, int32_t block_size,
                      int32_t table_width, int32_t num_blocks, int32_t causal, float scale,
                      void *stream);

/*
 * The same prefill attention with the `sliding_window_size` argument of
 * tt::scaled_dot_product_attention, which the reference forwards to its device kernel and
 * its CPU branch ignores (custom_ops.py:645, 704-706; passed by the backend at
 * attention.py:586-587).  sliding_window > 0 needs causal = 1: query row i then attends
 * keys  chunk_start + i - sliding_window < j <= chunk_start + i  (the newest
 * `sliding_window` keys, its own position included).  0 = no window = ttpa_sdpa_prefill.
 */
int ttpa_sdpa_prefill_windowed(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                               int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                               int64_t q_head_stride, int64_t q_token_stride, const void *k,
                               const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                               int64_t kv_token_stride, const int32_t *page_table,
                               int64_t page_table_row_stride, const int32_t *chunk_start,
                               const void *mask, int64_t mask_batch_stride, int64_t mask_row_stride,
                               int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,
                               int32_t kv_len, int32_t head_size, int32_t block_size,
                               int32_t table_width, int32_t num_blocks, int32_t causal, float scale,
                               int32_t sliding_window, void *stream);

/*
 * ttpa_sdpa_prefill_windowed with the cache format as an argument: kv_format = TTPA_KV_BFP8
 * (paged form only; block_size a multiple of 16) reads block-float-8 caches, expanding the
 * element bytes to bfloat16 (exactly) on their way into LDS.  This is what
 * tt::chunked_scaled_dot_product_attention runs when the plugin's
 * experimental_kv_cache_dtype="bfp_bf8" option is on (vllm_tt/platform.py:165, 232-233; the
 * reference's own test of the option is a chunked prefill,
 * tests/integrations/vllm_plugin/generative/test_chunked_prefill.py:86-96).
 * kv_format = TTPA_KV_BF16 is ttpa_sdpa_prefill_windowed.
 */
int ttpa_sdpa_prefill_format(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                             int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                             int64_t q_head_stride, int64_t q_token_stride, const void *k,
                             const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                             int64_t kv_token_stride, const int32_t *page_table,
                             int64_t page_table_row_stride, const int32_t *chunk_start,
                             const void *mask, int64_t mask_batch_stride, int64_t mask_row_stride,
                             int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,
                             int32_t kv_len, int32_t head_size, int32_t block_size,
                             int32_t table_width, int32_t num_blocks, int32_t causal, float scale,
                             int32_t sliding_window, int32_t kv_format, void *stream);

/*
 * ttpa_sdpa_prefill_format with scratch memory from the caller.  With kv_format = TTPA_KV_BFP8 and
 * at least ttpa_sdpa_prefill_workspace_bytes(...) bytes of 16-byte aligned device memory, a pass
 * over head size 128 with a multiple of four query heads per KV head, block_size a multiple of 64,
 * no window and no mask first expands the block-float-8 blocks it will read into bfloat16 copies
 * in the scratch (one launch; the decode is exact, so the result is the same) and then runs the
 * bfloat16 attention kernel over the copies: measured 1.7 times faster than expanding every tile
 * once per workgroup on 4 x 512-token chunks behind 2048 cached tokens.  Every other shape, a null
 * workspace or a smaller one run as ttpa_sdpa_prefill_format.  The scratch holds nothing between
 * calls; calls that overlap on one device need one each.  Serves the same reference operator and
 * option as ttpa_sdpa_prefill_format (vllm_tt/attention.py:762-785 with
 * experimental_kv_cache_dtype="bfp_bf8", vllm_tt/platform.py:165).
 */
int ttpa_sdpa_prefill_expanded(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                               int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                               int64_t q_head_stride, int64_t q_token_stride, const void *k,
                               const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                               int64_t kv_token_stride, const int32_t *page_table,
                               int64_t page_table_row_stride, const int32_t *chunk_start,
                               const void *mask, int64_t mask_batch_stride, int64_t mask_row_stride,
                               int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t q_len,
                               int32_t kv_len, int32_t head_size, int32_t block_size,
                               int32_t table_width, int32_t num_blocks, int32_t causal, float scale,
                               int32_t sliding_window, int32_t kv_format, void *workspace,
                               int64_t workspace_bytes, void *stream);

/* Bytes of scratch ttpa_sdpa_prefill_expanded can use for these dimensions (bfloat16 copies of K and
 * V for batch * table_width blocks plus their table); 0 for kv_format = TTPA_KV_BF16. */
int64_t ttpa_sdpa_prefill_workspace_bytes(int32_t batch, int32_t kv_heads, int32_t head_size,
                                          int32_t block_size, int32_t table_width, int32_t kv_format);

/*
 * The backend's first-chunk prefill pass in one call: ttpa_paged_fill_cache on K and on V
 * (attention.py:486-515: the prompt's keys and values go into the paged caches through the
 * fill page table) and the dense-form ttpa_sdpa_prefill_windowed on the same k / v
 * (attention.py:576-596).  Results, in the caches and in `out`, are those of the three calls;
 * the attention reads the dense k / v and never the caches, so their order does not matter.
 * k / v [batch, kv_heads, kv_len, head_size] by strides are both the attention's operands and
 * the fill operands (batch entry i fills table row batch_idx[i]; batch_idx may be NULL for
 * batch == 1; rows and blocks out of range are skipped, as in the fill).  bfloat16 caches
 * only.  Inside the library this is ONE launch: extra workgroups behind the attention's copy
 * the rows while the matrix pipes are busy.  No counterpart as one operator in the reference.
 */
int ttpa_sdpa_prefill_fill(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                           int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                           int64_t q_head_stride, int64_t q_token_stride, const void *k,
                           const void *v, int64_t kv_batch_stride, int64_t kv_head_stride,
                           int64_t kv_token_stride, int32_t batch, int32_t q_heads,
                           int32_t kv_heads, int32_t q_len, int32_t kv_len, int32_t head_size,
                           int32_t causal, float scale, int32_t sliding_window, void *k_cache,
                           void *v_cache, const int32_t *fill_page_table,
                           int64_t fill_page_table_row_stride, const void *batch_idx,
                           int batch_idx_is_i64, int32_t table_rows, int32_t block_size,
                           int32_t table_width, int32_t num_blocks, void *stream);

/*
 * Block-float-8 codec on flat arrays (n_elems % 16 == 0), for tests and cache
 * conversion.  No reference counterpart: the reference forwards
 * experimental_kv_cache_dtype="bfp_bf8" to an un-vendored compiler
 * (vllm_tt/platform.py:165; pjrt_implementation/src/api/module_builder/module_builder.cc:1050-1063).
 *   quantize:   bf16[n] -> elem uint8[n], exps uint8[n/16]
 *   dequantize: -> bf16[n] (exact: 7-bit magnitudes fit bfloat16)
 */
int ttpa_bfp8_quantize(const void *src_bf16, void *elem_u8, void *exps_u8, int64_t n_elems,
                       void *stream);
int ttpa_bfp8_dequantize(const void *elem_u8, const void *exps_u8, void *dst_bf16,
                         int64_t n_elems, void *stream);

/*
 * tt::flash_mla_prefill with V taken from K (reference python_package/tt_torch/custom_ops.py:223-378,
 * the form the latent backend calls: integrations/vllm_plugin/vllm_tt/attention_impls/
 * attention_mla.py:302-330): out[b, h, i, :] = softmax_j(scale * q[b, h, i] . k[b, h / G, j] + mask)
 * . k[b, h / G, j, :head_dim_v] over the keys j <= i (causal) or over all keys with an additive
 * bfloat16 mask [batch, 1 or q_heads, seq_len, seq_len] (mask_head_stride 0 shares one mask between
 * the heads; causal and mask exclude each other, as in the reference's asserts).  q [batch, q_heads,
 * seq_len, head_size], k [batch, kv_heads, seq_len, head_size], out [batch, q_heads, seq_len,
 * head_dim_v], all bfloat16 with explicit element strides (innermost dimension contiguous).  One
 * launch of a matrix-instruction kernel in which 128 (token, head) rows share every K tile; built
 * for (head_size, head_dim_v) = (576, 512), (192, 128), (128, 128), anything else returns
 * TTPA_ERR_UNSUPPORTED.
 */
int ttpa_latent_prefill(void *out, int64_t out_batch_stride, int64_t out_head_stride,
                        int64_t out_token_stride, const void *q, int64_t q_batch_stride,
                        int64_t q_head_stride, int64_t q_token_stride, const void *k,
                        int64_t k_batch_stride, int64_t k_head_stride, int64_t k_token_stride,
                        const void *mask, int64_t mask_batch_stride, int64_t mask_head_stride,
                        int64_t mask_row_stride, int32_t batch, int32_t q_heads, int32_t kv_heads,
                        int32_t seq_len, int32_t head_size, int32_t head_dim_v, int32_t causal,
                        float scale, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TTPA_H_ */
