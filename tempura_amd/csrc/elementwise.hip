// Memory-bound kernels of the step: embedding gather, RMSNorm, rotary + cache
// write, SwiGLU.  Every kernel takes any size (no power-of-two assumptions).
#include <stdarg.h>

#include "common.h"
#include "counter_normal.h"

static thread_local char g_error[512] = "";

void tp_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* tp_last_error() { return g_error; }

// ---- embedding ------------------------------------------------------------------
// out[t, :] = table[token[t], :] widened to float32 (the residual stream).
// grid: (tokens, column blocks of 256); every thread moves one element, so all loads of a
// row are in flight at once.
template <typename T>
__global__ void embed_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                             float* __restrict__ out, int hidden) {
  const int t = blockIdx.x;
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j < hidden) out[(size_t)t * hidden + j] = to_float(table[(size_t)tokens[t] * hidden + j]);
}

extern "C" int tp_embed(const int* tokens, const void* table, int table_dt, float* out, int n,
                        int hidden, hipStream_t s) {
  TP_REQUIRE(n >= 0 && hidden > 0, "embed: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0) return 0;
  const dim3 grid(n, (hidden + 255) / 256);
  TP_REQUIRE(grid.y <= 65535, "embed: hidden size too large");
  if (table_dt == TP_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, dim3(256), 0, s, tokens, (const float*)table, out, hidden);
  else if (table_dt == TP_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, dim3(256), 0, s, tokens, (const bf16_t*)table, out, hidden);
  else
    TP_REQUIRE(false, "embed: unknown dtype %d", table_dt);
  TP_CHECK_LAUNCH("embed");
  return 0;
}

// ---- RMSNorm ---------------------------------------------------------------------
// y = x * (1 / sqrt(mean(x^2) + eps)) * w, all in float32; one block per output row.
// `rows` (optional) picks the input row of each output row.  The row is kept in registers
// between the two passes when it fits (hidden <= 4 * VEC_ITEMS * threads).
#define RMS_ITEMS 4
template <typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               const int* __restrict__ rows, TO* __restrict__ out, int hidden, float eps) {
  __shared__ float scratch[32];
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * hidden;
  TO* o = out + (size_t)r * hidden;
  const bool vec = (hidden % 4 == 0) && hidden <= 4 * RMS_ITEMS * (int)blockDim.x;
  if (vec) {
    float4 v[RMS_ITEMS];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < RMS_ITEMS; ++i) {
      const int j = (threadIdx.x + i * blockDim.x) * 4;
      if (j < hidden) {
        v[i] = *(const float4*)(xr + j);
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
      }
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int i = 0; i < RMS_ITEMS; ++i) {
      const int j = (threadIdx.x + i * blockDim.x) * 4;
      if (j < hidden) {
        const float4 wv = *(const float4*)(w + j);
        from_float4(o + j, v[i].x * scale * wv.x, v[i].y * scale * wv.y, v[i].z * scale * wv.z, v[i].w * scale * wv.w);
      }
    }
    return;
  }
  float ss = 0.f;
  for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
    const float v = xr[j];
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int j = threadIdx.x; j < hidden; j += blockDim.x) from_float(o + j, xr[j] * scale * w[j]);
}

extern "C" int tp_rmsnorm(const float* x, const float* w, const int* rows, void* out, int out_dt,
                          int n_out, int hidden, float eps, hipStream_t s) {
  TP_REQUIRE(n_out >= 0 && hidden > 0, "rmsnorm: bad sizes");
  if (n_out == 0) return 0;
  const int threads = hidden >= 8192 ? 1024 : (hidden >= 1024 ? 256 : 64);
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(n_out), dim3(threads), 0, s, x, w, rows, (float*)out, hidden, eps);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(n_out), dim3(threads), 0, s, x, w, rows, (bf16_t*)out, hidden, eps);
  else
    TP_REQUIRE(false, "rmsnorm: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ---- rotary position encoding + cache write -----------------------------------------
// qkv row: [q heads | k heads | v heads] x head_dim, float32.  The q and k heads come in PAIRED order: the two
// elements that rotate together lie side by side, elements (2 d, 2 d + 1) of a head being elements
// (d, d + rotary_dim / 2) of the reference's split-half order (the attention part lays the rows of its
// projection out so; scores do not change when q and k are permuted alike, so the cache holds keys in this
// order and nothing is ever permuted back).  Pair d of each q and k head turns by the angle
// pos * inv_freq[d]: the product is formed in float64 and reduced to [0, 2 pi) there, sine and cosine of
// the small rest are float32.  q goes to q_out, rotated k and raw v go to the cache place `slots[t]`
// (page * page_size + offset) of the paged pools (qkv may be [splits, n, row] partial sums of the
// projection, added here): keys as [page, kv_head, page_size, head_dim], values TRANSPOSED as
// [page, kv_head, head_dim, page_size] so that the attention kernels read eight consecutive
// keys of one value element with one 16-byte load.  With slots == nullptr only q is produced
// (the row then holds q heads only).
// grid: (tokens, head blocks); a thread owns one pair (or two plain elements) of one head, so
// every load of the row is in flight at once.
// table[t, d] = (cos, sin) of token t's position times inv_freq[d]: long steps compute it once and every
// layer's rotation reads it
__global__ void rope_table_kernel(const int* __restrict__ positions, const double* __restrict__ inv_freq, int half,
                                  float factor, size_t total, float2* __restrict__ table) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float c, sn;
  rope_cos_sin(positions[i / half], inv_freq[i % half], factor, c, sn);
  table[i] = make_float2(c, sn);
}

extern "C" int tp_rope_table(const int* positions, const double* inv_freq, int rotary_dim, float factor, int n,
                             float* table, hipStream_t s) {
  TP_REQUIRE(n >= 0 && rotary_dim > 0 && rotary_dim % 2 == 0 && inv_freq != nullptr, "rope_table: bad sizes");
  const size_t total = (size_t)n * (rotary_dim / 2);
  if (total == 0) return 0;
  TP_REQUIRE((total + 255) / 256 < ((size_t)1 << 31), "rope_table: too many tokens");
  hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, positions, inv_freq,
                     rotary_dim / 2, factor, total, (float2*)table);
  TP_CHECK_LAUNCH("rope_table");
  return 0;
}

template <typename TQ, typename TC>
__global__ void rope_kv_write_kernel(const float* __restrict__ qkv, int row_stride,
                                     const int* __restrict__ positions, const int* __restrict__ slots,
                                     const double* __restrict__ inv_freq, int rotary_dim, float factor,
                                     int n_heads, int n_kv, int head_dim, TQ* __restrict__ q_out,
                                     TC* __restrict__ k_cache, TC* __restrict__ v_cache, int page_size,
                                     int pairs, int heads_per_block, int splits, size_t split_stride,
                                     const float2* __restrict__ cos_sin, int with_values) {
  const int t = blockIdx.x;
  const int hl = threadIdx.x / pairs, d = threadIdx.x % pairs;   // pairs = head_dim / 2
  const int h = blockIdx.y * heads_per_block + hl;
  const int total_heads = n_heads + (slots ? (with_values ? 2 : 1) * n_kv : 0);
  if (hl >= heads_per_block || h >= total_heads) return;
  const int half = rotary_dim / 2;
  const float* row = qkv + (size_t)t * row_stride + (size_t)h * head_dim;
  // the two elements this thread moves: a rotary pair (d < half), or two pass-through elements
  const int i0 = 2 * d, i1 = 2 * d + 1;
  // (splits > 1: the rows are the partial sums of a product whose K was split; added in ascending order)
  float y0 = 0.f, y1 = 0.f;
  {
    float p0[16], p1[16];   // (all loads in flight before the first sum; splits <= 16)
#pragma unroll
    for (int sp = 0; sp < 16; ++sp)
      if (sp < splits) {
        p0[sp] = row[(size_t)sp * split_stride + i0];
        p1[sp] = row[(size_t)sp * split_stride + i1];
      }
#pragma unroll
    for (int sp = 0; sp < 16; ++sp)
      if (sp < splits) {
        y0 += p0[sp];
        y1 += p1[sp];
      }
  }
  size_t page = 0, off = 0;
  if (slots) {
    const int slot = slots[t];
    page = (size_t)(slot / page_size);
    off = (size_t)(slot % page_size);
  }
  if (h < n_heads + n_kv && d < half) {  // q and k heads rotate
    float sn, c;
    if (cos_sin != nullptr) {   // this step's table (rope_table_kernel: the same arithmetic, once for all layers)
      const float2 cs = cos_sin[(size_t)t * half + d];
      c = cs.x;
      sn = cs.y;
    } else {
      rope_cos_sin(positions[t], inv_freq[d], factor, c, sn);
    }
    const float x0 = y0, x1 = y1;
    y0 = x0 * c - x1 * sn;
    y1 = x0 * sn + x1 * c;
  }
  if (h < n_heads) {
    TQ* o = q_out + ((size_t)t * n_heads + h) * head_dim;
    from_float(o + i0, y0);
    from_float(o + i1, y1);
  } else if (h < n_heads + n_kv) {
    TC* o = k_cache + ((page * n_kv + (h - n_heads)) * page_size + off) * head_dim;
    from_float(o + i0, y0);
    from_float(o + i1, y1);
  } else {
    TC* o = v_cache + ((page * n_kv + (h - n_heads - n_kv)) * head_dim) * page_size + off;
    from_float(o + (size_t)i0 * page_size, y0);
    from_float(o + (size_t)i1 * page_size, y1);
  }
}

// The same rotation for the q and k heads of long steps, four pairs (eight consecutive elements) per thread
// (16-byte loads, 8-byte stores of bfloat16): needs head_dim, rotary_dim and the row stride to be multiples of eight.
// grid: (tokens, blocks of 256 threads over heads x head_dim / 8).
template <typename T>
__device__ inline void store4(T* p, const float (&v)[4]) {
  if constexpr (sizeof(T) == 2) {
    union {
      bf16_t h[4];
      uint2 u;
    } pk;
#pragma unroll
    for (int e = 0; e < 4; ++e) pk.h[e] = float_to_bf16(v[e]);
    *(uint2*)p = pk.u;
  } else {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
  }
}

template <typename TQ, typename TC>
__global__ void rope_qk4_kernel(const float* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                                const int* __restrict__ slots, const double* __restrict__ inv_freq, int rotary_dim,
                                float factor, int n_heads, int n_rot_heads, int n_kv, int head_dim,
                                TQ* __restrict__ q_out, TC* __restrict__ k_cache, int page_size, int splits,
                                size_t split_stride, const float2* __restrict__ cos_sin) {
  const int t = blockIdx.x;
  const int tph = head_dim / 8;                       // threads per head
  const int idx = blockIdx.y * blockDim.x + threadIdx.x;
  const int h = idx / tph, j = idx % tph;
  if (h >= n_rot_heads) return;
  const int half = rotary_dim / 2;
  // the eight elements this thread moves: four rotary pairs (side by side), or eight plain elements
  const bool rot = 8 * j < rotary_dim;
  const int i0 = 8 * j, i1 = 8 * j + 4;
  const float* row = qkv + (size_t)t * row_stride + (size_t)h * head_dim;
  float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
  {
    float4 pa[16], pb[16];   // all loads in flight before the first sum; splits <= 16, added in ascending order
#pragma unroll
    for (int sp = 0; sp < 16; ++sp)
      if (sp < splits) {
        pa[sp] = *(const float4*)(row + (size_t)sp * split_stride + i0);
        pb[sp] = *(const float4*)(row + (size_t)sp * split_stride + i1);
      }
#pragma unroll
    for (int sp = 0; sp < 16; ++sp)
      if (sp < splits) {
        a[0] += pa[sp].x; a[1] += pa[sp].y; a[2] += pa[sp].z; a[3] += pa[sp].w;
        b[0] += pb[sp].x; b[1] += pb[sp].y; b[2] += pb[sp].z; b[3] += pb[sp].w;
      }
  }
  if (rot) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {   // pair 4 j + e: elements (a[0], a[1]), (a[2], a[3]), (b[0], b[1]), (b[2], b[3])
      float sn, c;
      if (cos_sin != nullptr) {
        const float2 cs = cos_sin[(size_t)t * half + 4 * j + e];
        c = cs.x;
        sn = cs.y;
      } else {
        rope_cos_sin(positions[t], inv_freq[4 * j + e], factor, c, sn);
      }
      float& r0 = e < 2 ? a[2 * e] : b[2 * e - 4];
      float& r1 = e < 2 ? a[2 * e + 1] : b[2 * e - 3];
      const float x0 = r0, x1 = r1;
      r0 = x0 * c - x1 * sn;
      r1 = x0 * sn + x1 * c;
    }
  }
  if (h < n_heads) {
    TQ* o = q_out + ((size_t)t * n_heads + h) * head_dim;
    store4(o + i0, a);
    store4(o + i1, b);
  } else {
    const int slot = slots[t];
    const size_t page = (size_t)(slot / page_size), off = (size_t)(slot % page_size);
    TC* o = k_cache + ((page * n_kv + (h - n_heads)) * page_size + off) * head_dim;
    store4(o + i0, a);
    store4(o + i1, b);
  }
}

// The values of long steps: a thread takes one element of one kv head for sixteen consecutive tokens and
// stores each run of eight whose cache places follow one another from a multiple of eight (always so inside
// a prompt portion) as one 16-byte piece of the transposed layout, instead of eight scattered elements.
// grid: (ceil(n / 16), kv heads); block: head_dim threads.
template <typename TC>
__global__ void value_write_kernel(const float* __restrict__ qkv, int row_stride, const int* __restrict__ slots,
                                   int n, int v_col0, int n_kv, int head_dim, TC* __restrict__ v_cache,
                                   int page_size, int splits, size_t split_stride) {
  const int t0 = blockIdx.x * 16, kh = blockIdx.y, d = threadIdx.x;
  if (d >= head_dim) return;
  const float* col = qkv + (size_t)v_col0 + (size_t)kh * head_dim + d;
  float y[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) y[i] = 0.f;
  for (int sp = 0; sp < splits; ++sp) {   // ascending order, all sixteen loads of a split in flight
    float p[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) p[i] = t0 + i < n ? col[(size_t)sp * split_stride + (size_t)(t0 + i) * row_stride] : 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) y[i] += p[i];
  }
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int tg = t0 + 8 * g;
    if (tg >= n) break;
    const int s0 = slots[tg];
    bool run = tg + 8 <= n && (s0 & 7) == 0 && page_size % 8 == 0;
    if (run) {
#pragma unroll
      for (int i = 1; i < 8; ++i) run = run && slots[tg + i] == s0 + i;
    }
    if (run) {
      const size_t page = (size_t)(s0 / page_size), off = (size_t)(s0 % page_size);
      TC* o = v_cache + ((page * n_kv + kh) * head_dim + d) * page_size + off;
      if constexpr (sizeof(TC) == 2) {
        union {
          bf16_t h[8];
          uint4 v;
        } pk;
#pragma unroll
        for (int i = 0; i < 8; ++i) pk.h[i] = float_to_bf16(y[8 * g + i]);
        *(uint4*)o = pk.v;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) from_float(o + i, y[8 * g + i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (tg + i >= n) break;
        const int sl = slots[tg + i];
        const size_t page = (size_t)(sl / page_size), off = (size_t)(sl % page_size);
        from_float(v_cache + ((page * n_kv + kh) * head_dim + d) * page_size + off, y[8 * g + i]);
      }
    }
  }
}

extern "C" int tp_rope_kv_write(const float* qkv, int row_stride, const int* positions, const int* slots,
                                const double* inv_freq, int rotary_dim, float factor, int n, int n_heads,
                                int n_kv, int head_dim, void* q_out, int q_dt, void* k_cache, void* v_cache,
                                int cache_dt, int page_size, int splits, const float* cos_sin, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_heads > 0 && n_kv >= 0 && head_dim > 0, "rope_kv_write: bad sizes");
  TP_REQUIRE(splits >= 1 && splits <= 16, "rope_kv_write: bad number of partial sums");
  const size_t split_stride = (size_t)n * row_stride;   // qkv is [splits, n, row_stride]
  TP_REQUIRE(head_dim % 2 == 0 && head_dim <= 1024, "rope_kv_write: head_dim %d must be even and <= 1024", head_dim);
  TP_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= head_dim,
             "rope_kv_write: rotary_dim %d must be even and <= head_dim %d", rotary_dim, head_dim);
  TP_REQUIRE(rotary_dim == 0 || inv_freq != nullptr, "rope_kv_write: no frequency table");
  TP_REQUIRE(slots == nullptr || (k_cache && v_cache && page_size > 0), "rope_kv_write: cache missing");
  TP_REQUIRE(row_stride >= (n_heads + (slots ? 2 * n_kv : 0)) * head_dim, "rope_kv_write: row too short");
  if (n == 0) return 0;
  const int pairs = head_dim / 2;
  const int threads = pairs <= 256 ? 256 : 512;
  const int hpb = threads / pairs;
  // long steps (prompt portions, mostly) write their values sixteen tokens at a time (value_write_kernel);
  // a batch of single decoded tokens has no runs, and a second kernel would only cost it a launch
  const bool grouped_values = slots != nullptr && n >= 256 && n_kv <= 65535;
  const int total_heads = n_heads + (slots ? (grouped_values ? 1 : 2) * n_kv : 0);
  const dim3 grid(n, (total_heads + hpb - 1) / hpb);
  TP_REQUIRE(grid.y <= 65535, "rope_kv_write: too many heads");
  // long steps: q and k four pairs per thread, v sixteen tokens per thread
  if (n >= 256 && head_dim % 8 == 0 && rotary_dim % 8 == 0 && row_stride % 4 == 0 && (slots == nullptr || grouped_values) &&
      ((uintptr_t)qkv % 16) == 0 && (split_stride % 4) == 0) {
    const int n_rot_heads = n_heads + (slots ? n_kv : 0);
    const int work = n_rot_heads * (head_dim / 8);
    const dim3 g4(n, (work + 255) / 256);
    TP_REQUIRE(g4.y <= 65535, "rope_kv_write: too many heads");
#define LAUNCH4(TQ, TC)                                                                                               \
  hipLaunchKernelGGL((rope_qk4_kernel<TQ, TC>), g4, dim3(256), 0, s, qkv, row_stride, positions, slots, inv_freq,      \
                     rotary_dim, factor, n_heads, n_rot_heads, n_kv, head_dim, (TQ*)q_out, (TC*)k_cache, page_size, \
                     splits, split_stride, (const float2*)cos_sin)
    if (q_dt == TP_F32 && cache_dt == TP_F32)
      LAUNCH4(float, float);
    else if (q_dt == TP_BF16 && cache_dt == TP_BF16)
      LAUNCH4(bf16_t, bf16_t);
    else if (q_dt == TP_F32 && cache_dt == TP_BF16)
      LAUNCH4(float, bf16_t);
    else if (q_dt == TP_BF16 && cache_dt == TP_F32)
      LAUNCH4(bf16_t, float);
    else
      TP_REQUIRE(false, "rope_kv_write: unknown dtypes %d %d", q_dt, cache_dt);
#undef LAUNCH4
  } else {
#define LAUNCH(TQ, TC)                                                                                    \
  hipLaunchKernelGGL((rope_kv_write_kernel<TQ, TC>), grid, dim3(threads), 0, s, qkv, row_stride, positions, \
                     slots, inv_freq, rotary_dim, factor, n_heads, n_kv, head_dim, (TQ*)q_out, (TC*)k_cache, \
                     (TC*)v_cache, page_size, pairs, hpb, splits, split_stride, (const float2*)cos_sin, grouped_values ? 0 : 1)
  if (q_dt == TP_F32 && cache_dt == TP_F32)
    LAUNCH(float, float);
  else if (q_dt == TP_BF16 && cache_dt == TP_BF16)
    LAUNCH(bf16_t, bf16_t);
  else if (q_dt == TP_F32 && cache_dt == TP_BF16)
    LAUNCH(float, bf16_t);
  else if (q_dt == TP_BF16 && cache_dt == TP_F32)
    LAUNCH(bf16_t, float);
  else
    TP_REQUIRE(false, "rope_kv_write: unknown dtypes %d %d", q_dt, cache_dt);
#undef LAUNCH
  }
  if (grouped_values) {
    const dim3 vgrid((n + 15) / 16, n_kv);
    const int v_col0 = (n_heads + n_kv) * head_dim;
    if (cache_dt == TP_BF16)
      hipLaunchKernelGGL((value_write_kernel<bf16_t>), vgrid, dim3((head_dim + 63) / 64 * 64), 0, s, qkv, row_stride, slots, n,
                         v_col0, n_kv, head_dim, (bf16_t*)v_cache, page_size, splits, split_stride);
    else
      hipLaunchKernelGGL((value_write_kernel<float>), vgrid, dim3((head_dim + 63) / 64 * 64), 0, s, qkv, row_stride, slots, n,
                         v_col0, n_kv, head_dim, (float*)v_cache, page_size, splits, split_stride);
  }
  TP_CHECK_LAUNCH("rope_kv_write");
  return 0;
}

// ---- SwiGLU --------------------------------------------------------------------------
// out[m, i] = silu(gu[m, i]) * gu[m, I + i], silu(x) = x / (1 + exp(-x)).
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = (int)(idx % inter);
  const float g = to_float(gu[m * 2 * inter + i]);
  const float u = to_float(gu[m * 2 * inter + inter + i]);
  from_float(out + idx, g / (1.0f + expf(-g)) * u);
}

extern "C" int tp_swiglu(const void* gu, int in_dt, void* out, int out_dt, int m, int inter, hipStream_t s) {
  TP_REQUIRE(m >= 0 && inter > 0, "swiglu: bad sizes");
  if (m == 0) return 0;
  const size_t total = (size_t)m * inter;
  const dim3 grid((unsigned)((total + 255) / 256));
#define LAUNCH(TI, TO) \
  hipLaunchKernelGGL((swiglu_kernel<TI, TO>), grid, dim3(256), 0, s, (const TI*)gu, (TO*)out, inter, total)
  if (in_dt == TP_F32 && out_dt == TP_F32)
    LAUNCH(float, float);
  else if (in_dt == TP_BF16 && out_dt == TP_BF16)
    LAUNCH(bf16_t, bf16_t);
  else if (in_dt == TP_F32 && out_dt == TP_BF16)
    LAUNCH(float, bf16_t);
  else
    TP_REQUIRE(false, "swiglu: unsupported dtypes %d -> %d", in_dt, out_dt);
#undef LAUNCH
  TP_CHECK_LAUNCH("swiglu");
  return 0;
}

// ---- rows of 4-byte elements: gather and clear ------------------------------------------------
// out[i, :] = src[rows[i], :] (rows null: out[i, :] = src[i, :]); the element type only has to be four bytes wide
// (float32 logits, int32 token ids).  grid: (rows out, column blocks of 1024); block: 256 threads, four elements each.
__global__ void copy_rows4_kernel(const uint32_t* __restrict__ src, const int* __restrict__ rows, uint32_t* __restrict__ out,
                                  int width) {
  const int i = blockIdx.x;
  const size_t from = (size_t)(rows ? rows[i] : i) * width, to = (size_t)i * width;
  for (int j = blockIdx.y * 1024 + threadIdx.x; j < min(width, (int)(blockIdx.y + 1) * 1024); j += 256) out[to + j] = src[from + j];
}

extern "C" int tp_copy_rows4(const void* src, const int* rows, void* out, int n, int width, hipStream_t s) {
  TP_REQUIRE(n >= 0 && width > 0, "copy_rows: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(copy_rows4_kernel, dim3(n, (width + 1023) / 1024), dim3(256), 0, s, (const uint32_t*)src, rows,
                     (uint32_t*)out, width);
  TP_CHECK_LAUNCH("copy_rows");
  return 0;
}

// t[rows[i], :] = 0 for rows of `width` 4-byte elements.
__global__ void zero_rows4_kernel(uint32_t* __restrict__ t, const int* __restrict__ rows, int width) {
  const size_t at = (size_t)rows[blockIdx.x] * width;
  for (int j = blockIdx.y * 1024 + threadIdx.x; j < min(width, (int)(blockIdx.y + 1) * 1024); j += 256) t[at + j] = 0u;
}

extern "C" int tp_zero_rows4(void* t, const int* rows, int n, int width, hipStream_t s) {
  TP_REQUIRE(n >= 0 && width > 0, "zero_rows: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(zero_rows4_kernel, dim3(n, (width + 1023) / 1024), dim3(256), 0, s, (uint32_t*)t, rows, width);
  TP_CHECK_LAUNCH("zero_rows");
  return 0;
}

// ---- seeded normal fill ------------------------------------------------------------------
// out[i] = mean + std * N(0, 1) where the deviate of element i depends only on (seed, i) and has the same
// bits as the host library's (counter_normal.h): random weights of large models are made directly in device
// memory and can still be regenerated on the host.
template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, size_t n, unsigned long long seed, double mean, double std) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  from_float(out + i, cn_element(seed, i, mean, std));
}

extern "C" int tp_fill_normal(void* out, int dt, size_t n, unsigned long long seed, double mean, double std,
                              hipStream_t s) {
  if (n == 0) return 0;
  const dim3 grid((unsigned)((n + 255) / 256));
  TP_REQUIRE((n + 255) / 256 < ((size_t)1 << 31), "fill_normal: tensor too large");
  if (dt == TP_F32)
    hipLaunchKernelGGL(fill_normal_kernel<float>, grid, dim3(256), 0, s, (float*)out, n, seed, mean, std);
  else if (dt == TP_BF16)
    hipLaunchKernelGGL(fill_normal_kernel<bf16_t>, grid, dim3(256), 0, s, (bf16_t*)out, n, seed, mean, std);
  else
    TP_REQUIRE(false, "fill_normal: unknown dtype %d", dt);
  TP_CHECK_LAUNCH("fill_normal");
  return 0;
}
