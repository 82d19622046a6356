// bfloat16 attention on the matrix cores (placeholder until the MFMA kernels land).
#include "common.h"

int tp_paged_attention_fast(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                            int table_width, const int* cu_seqlens, const int* context_lens,
                            const int* token_req, void* out, int n_tokens, int n_req, int n_heads, int n_kv,
                            int head_dim, int page_size, float scale, int window, int max_q_len, int max_ctx,
                            hipStream_t s) {
  return -1;
}
