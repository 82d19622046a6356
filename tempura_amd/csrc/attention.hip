// Attention over the paged cache, general kernel: any head size up to 512, any number
// of heads and groups, any page size, optional window, float32 or bfloat16.
//
// One wave per (query token, head).  Keys are taken 64 at a time: each lane scores one
// key (a full dot product with the query, which sits in LDS), the tile's maximum and
// sum update the running softmax in float32, then lanes switch to owning output
// elements and add p_j * V[j] for the tile's keys.  The order of keys is ascending and
// does not depend on what else is in the batch or on which pages hold the keys.
//
// Query token t belongs to request r = token_req[t]; its position is
// context_lens[r] - q_len_r + (t - cu_seqlens[r]) and it sees keys lo..pos with
// lo = max(0, pos - window + 1) when window > 0, else 0.
#include <math.h>

#include "common.h"

#define ATT_MAX_ACC 8  // head_dim <= 64 * ATT_MAX_ACC

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, const int* __restrict__ token_req, T* __restrict__ out, int n_heads,
    int n_kv, int head_dim, int page_size, float scale, int window) {
  extern __shared__ float qs[];  // the query row, float32
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = token_req[t];
  const int q_start = cu_seqlens[r];
  const int q_len = cu_seqlens[r + 1] - q_start;
  const int pos = context_lens[r] - q_len + (t - q_start);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int kvh = h / (n_heads / n_kv);
  const T* qrow = q + ((size_t)t * n_heads + h) * head_dim;
  for (int d = lane; d < head_dim; d += TP_WAVE) qs[d] = to_float(qrow[d]);
  __syncthreads();
  const int* table = block_tables + (size_t)r * table_width;

  float m = -INFINITY, l = 0.f;
  float acc[ATT_MAX_ACC];
#pragma unroll
  for (int i = 0; i < ATT_MAX_ACC; ++i) acc[i] = 0.f;

  for (int j0 = lo; j0 <= pos; j0 += TP_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    int row = 0;   // cache row of this lane's key: (page * n_kv + kvh) * page_size + offset
    int vbase = 0; // its value column: values are stored [page, kv_head, head_dim, page_size]
    float s = -INFINITY;
    if (valid) {
      const int page = table[j / page_size];
      row = (page * n_kv + kvh) * page_size + j % page_size;
      vbase = (page * n_kv + kvh);
      const T* kr = k_cache + (size_t)row * head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);  // first tile: exp(-inf) = 0
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < ATT_MAX_ACC; ++i) acc[i] *= alpha;
    const int n_valid = min(TP_WAVE, pos - j0 + 1);
    for (int jj = 0; jj < n_valid; ++jj) {
      const float pj = __shfl(p, jj, TP_WAVE);
      const int vb = __shfl(vbase, jj, TP_WAVE);
      const T* vr = v_cache + (size_t)vb * head_dim * page_size + (j0 + jj) % page_size;
#pragma unroll
      for (int i = 0; i < ATT_MAX_ACC; ++i) {
        const int d = lane + i * TP_WAVE;
        if (d < head_dim) acc[i] = fmaf(pj, to_float(vr[(size_t)d * page_size]), acc[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  T* o = out + ((size_t)t * n_heads + h) * head_dim;
#pragma unroll
  for (int i = 0; i < ATT_MAX_ACC; ++i) {
    const int d = lane + i * TP_WAVE;
    if (d < head_dim) from_float(o + d, acc[i] * inv);
  }
}

// Defined in attention_mfma.hip: takes bfloat16 shapes it is built for, returns -1 otherwise.
int tp_paged_attention_fast(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                            int table_width, const int* cu_seqlens, const int* context_lens, void* out, int n_tokens,
                            int n_req, int n_heads, int n_kv, int head_dim, int page_size, float scale, int window,
                            int max_q_len, int num_single, int num_splits, float* scratch, const int* token_req,
                            int portion_splits, int portion_min_steps, float* portion_scratch, hipStream_t s);

extern "C" int tp_paged_attention(const void* q, int dt, const void* k_cache, const void* v_cache,
                                  const int* block_tables, int table_width, const int* cu_seqlens,
                                  const int* context_lens, const int* token_req, void* out, int n_tokens,
                                  int n_req, int n_heads, int n_kv, int head_dim, int page_size, float scale,
                                  int window, int max_q_len, int max_ctx, int allow_fast, int num_single,
                                  int num_splits, float* scratch, int portion_splits, int portion_min_steps,
                                  float* portion_scratch, hipStream_t s) {
  // num_single: how many requests bring exactly one token (they go to the split decode kernel,
  // which, with more than one split, needs `scratch` of n_req * n_heads * num_splits * (head_dim + 2)
  // floats).  portion_splits > 1: the keys of every longer request are split over that many blocks,
  // which needs `portion_scratch` of n_tokens * n_heads * portion_splits * (head_dim + 4) floats.
  TP_REQUIRE(n_tokens >= 0 && n_req >= 0 && n_heads > 0 && n_kv > 0 && head_dim > 0 && page_size > 0,
             "paged_attention: bad sizes");
  TP_REQUIRE(n_heads % n_kv == 0, "paged_attention: %d heads is not a multiple of %d kv heads", n_heads, n_kv);
  TP_REQUIRE(head_dim <= TP_WAVE * ATT_MAX_ACC, "paged_attention: head_dim %d exceeds %d", head_dim,
             TP_WAVE * ATT_MAX_ACC);
  TP_REQUIRE(window >= 0, "paged_attention: window must be >= 0");
  TP_REQUIRE(n_heads <= 65535, "paged_attention: too many heads");
  if (n_tokens == 0) return 0;
  if (dt == TP_BF16 && allow_fast) {
    const int rc = tp_paged_attention_fast(q, k_cache, v_cache, block_tables, table_width, cu_seqlens,
                                           context_lens, out, n_tokens, n_req, n_heads, n_kv, head_dim,
                                           page_size, scale, window, max_q_len, num_single, num_splits, scratch, token_req,
                                           portion_splits, portion_min_steps, portion_scratch, s);
    if (rc >= 0) return rc;
  }
  const dim3 grid(n_tokens, n_heads);
  const size_t shmem = (size_t)head_dim * sizeof(float);
  if (dt == TP_F32)
    hipLaunchKernelGGL(paged_attention_kernel<float>, grid, dim3(64), shmem, s, (const float*)q,
                       (const float*)k_cache, (const float*)v_cache, block_tables, table_width, cu_seqlens,
                       context_lens, token_req, (float*)out, n_heads, n_kv, head_dim, page_size, scale, window);
  else if (dt == TP_BF16)
    hipLaunchKernelGGL(paged_attention_kernel<bf16_t>, grid, dim3(64), shmem, s, (const bf16_t*)q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, table_width, cu_seqlens,
                       context_lens, token_req, (bf16_t*)out, n_heads, n_kv, head_dim, page_size, scale, window);
  else
    TP_REQUIRE(false, "paged_attention: unknown dtype %d", dt);
  TP_CHECK_LAUNCH("paged_attention");
  return 0;
}
