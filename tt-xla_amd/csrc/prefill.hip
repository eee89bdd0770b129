// Prefill attention entry point (MFMA kernel under construction).
#include "common.h"
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
  return fail(TTPA_ERR_UNSUPPORTED, "prefill attention kernel not built yet");
}
