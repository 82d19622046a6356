// bfloat16 attention over the paged cache on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16), for head sizes that are multiples of 32 (up to 128) and
// page sizes that are multiples of 8.  Other shapes go to the general kernel.
//
// Everything is computed transposed, so that no operand ever needs a transpose in LDS:
//   S^T[key, query] = K[key, :] . Q[query, :]          (A = K rows, B = Q rows)
//   O^T[d, query]  += V^T[d, keys] . P^T[keys, query]  (A = V^T rows, B = P^T)
// A step covers 32 keys.  The 16x16 result tile of S^T gives lane l the keys 4*(l/16)+r of
// column l%16; the two score tiles of a step take their K rows in the order
// key = 8*(i/4) + 4*t + i%4 (tile t, row i), so that a lane ends up with the eight
// CONSECUTIVE keys 8*(l/16) .. +7 of its column — exactly the B-operand layout of the next
// product, whose A operand is one 16-byte load from the value cache, which is stored
// transposed ([page, kv_head, head_dim, page_size]) for this purpose.
// Softmax statistics (running maximum and sum per query column) are float32, in the
// base-2 domain: scores are multiplied by scale * log2(e) once and exponentials are exp2.
//
// Two kernels share the step:
//  * prefill: a wave owns 16*NQ query rows of one head; the four waves of a block are four
//    heads that share a kv head (their K/V loads hit the same cache lines).  Causal and
//    window masks by absolute position, so a portion after a cached prefix is handled.
//  * decode (requests with one new token): the columns are the query heads that share a kv
//    head; the context is split over blockIdx.z and over the four waves of a block; partial
//    (max, sum, O) go to scratch and a second kernel combines them in a fixed order.
#include <math.h>

#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ inline bf16x8_t frag_of(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

__device__ inline unsigned int pack_bf16(float a, float b) {
  return (unsigned int)float_to_bf16(a).bits | ((unsigned int)float_to_bf16(b).bits << 16);
}

struct AttnArgs {
  const bf16_t* q;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const int* block_tables;
  int table_width;
  const int* cu_seqlens;
  const int* context_lens;
  bf16_t* out;
  float* scratch;
  int n_heads, n_kv, page_size, window, num_splits;
  float scale_log2;
};

// The keys and values of one step of 32 keys, as MFMA operand fragments.
template <int D>
struct KvFrags {
  bf16x8_t k[2][D / 32];
  bf16x8_t v[D / 16];
};

// Fetch the fragments of the step starting at key j0 (kvh: kv head; ctx: keys that exist; keys
// past the end are clamped to the last one and masked later).
template <int D>
__device__ inline void attn_load(const AttnArgs& a, const int* __restrict__ table, int kvh, int ctx, int j0,
                                 KvFrags<D>& f) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4, c = lane & 15;
  const int ps = a.page_size;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key = min(j0 + 8 * (c >> 2) + 4 * t + (c & 3), ctx - 1);
    const int page = table[key / ps];
    const bf16_t* kr = a.k_cache + ((size_t)(page * a.n_kv + kvh) * ps + key % ps) * D + g * 8;
#pragma unroll
    for (int dk = 0; dk < D / 32; ++dk) f.k[t][dk] = frag_of(*(const u32x4_t*)(kr + dk * 32));
  }
  // values: eight consecutive keys of element d per lane
  const int kb = min(j0 + 8 * g, (ctx - 1) & ~7);
  const int vpage = table[kb / ps];
  const bf16_t* vr = a.v_cache + ((size_t)(vpage * a.n_kv + kvh) * D + c) * ps + kb % ps;
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) f.v[dt] = frag_of(*(const u32x4_t*)(vr + (size_t)dt * 16 * ps));
}

// One step of 32 keys starting at j0 for NQ query tiles, on fetched fragments.  qpos[nq] is the
// absolute position of this lane's query column (keys above it are masked).  m/l/o are the
// running statistics and output of each tile.
template <int D, int NQ>
__device__ inline void attn_compute(const AttnArgs& a, int j0, const KvFrags<D>& f, const bf16x8_t (&qf)[NQ][D / 32],
                                    const int (&qpos)[NQ], float (&m)[NQ], float (&l)[NQ], f32x4_t (&o)[NQ][D / 16]) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  // scores: two 16-key tiles
  f32x4_t s[NQ][2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      s[nq][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dk = 0; dk < D / 32; ++dk)
        s[nq][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[t][dk], qf[nq][dk], s[nq][t], 0, 0, 0);
    }
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    // this lane's keys: j0 + 8g + 4t + r
    float v[8];
    float mx = -INFINITY;
    const int hi = qpos[nq];
    const int lo = a.window > 0 ? hi - a.window + 1 : 0;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = j0 + 8 * g + 4 * t + r;
        const float x = (key <= hi && key >= lo) ? s[nq][t][r] * a.scale_log2 : -INFINITY;
        v[t * 4 + r] = x;
        mx = fmaxf(mx, x);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m[nq], mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column with nothing visible yet
    const float alpha = __builtin_amdgcn_exp2f(m[nq] - m_use);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = __builtin_amdgcn_exp2f(v[i] - m_use);
      sum += v[i];
    }
    l[nq] = l[nq] * alpha + sum;  // per-lane partial sum; lanes of a column are added at the end
    m[nq] = m_new;
    u32x4_t pk;
    pk[0] = pack_bf16(v[0], v[1]);
    pk[1] = pack_bf16(v[2], v[3]);
    pk[2] = pack_bf16(v[4], v[5]);
    pk[3] = pack_bf16(v[6], v[7]);
    const bf16x8_t pf = frag_of(pk);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      f32x4_t acc = o[nq][dt];
      acc[0] *= alpha;
      acc[1] *= alpha;
      acc[2] *= alpha;
      acc[3] *= alpha;
      o[nq][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[dt], pf, acc, 0, 0, 0);
    }
  }
}

template <int D, int NQ>
__device__ inline void attn_step(const AttnArgs& a, const int* __restrict__ table, int kvh, int ctx, int j0,
                                 const bf16x8_t (&qf)[NQ][D / 32], const int (&qpos)[NQ], float (&m)[NQ],
                                 float (&l)[NQ], f32x4_t (&o)[NQ][D / 16]) {
  KvFrags<D> f;
  attn_load<D>(a, table, kvh, ctx, j0, f);
  attn_compute<D, NQ>(a, j0, f, qf, qpos, m, l, o);
}

// ---- prefill ----------------------------------------------------------------------------
// grid: (query blocks of 16*NQ rows, kv_heads * ceil(group / 4), requests); block: 4 waves.
template <int D, int NQ>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a, int skip_single) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int r = blockIdx.z;
  const int q_start = a.cu_seqlens[r];
  const int q_len = a.cu_seqlens[r + 1] - q_start;
  if (q_len <= 0 || (skip_single && q_len == 1)) return;
  const int q0 = blockIdx.x * 16 * NQ;
  if (q0 >= q_len) return;
  const int group = a.n_heads / a.n_kv;
  const int hblocks = (group + 3) / 4;
  const int kvh = blockIdx.y / hblocks;
  const int hin = (blockIdx.y % hblocks) * 4 + wave;
  if (hin >= group) return;
  const int head = kvh * group + hin;
  const int ctx = a.context_lens[r];
  const int pos0 = ctx - q_len;  // position of the request's first new token
  const int* table = a.block_tables + (size_t)r * a.table_width;

  bf16x8_t qf[NQ][D / 32];
  int qpos[NQ];
  float m[NQ], l[NQ];
  f32x4_t o[NQ][D / 16];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int qi = min(q0 + nq * 16 + c, q_len - 1);  // rows past the end repeat the last one, never written
    qpos[nq] = pos0 + qi;
    const bf16_t* qr = a.q + ((size_t)(q_start + qi) * a.n_heads + head) * D + g * 8;
#pragma unroll
    for (int dk = 0; dk < D / 32; ++dk) qf[nq][dk] = frag_of(*(const u32x4_t*)(qr + dk * 32));
    m[nq] = -INFINITY;
    l[nq] = 0.f;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) o[nq][dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }
  const int last_pos = pos0 + min(q0 + 16 * NQ, q_len) - 1;
  int first = 0;
  if (a.window > 0) first = max(0, pos0 + q0 - a.window + 1) & ~31;
  for (int j0 = first; j0 <= last_pos; j0 += 32) attn_step<D, NQ>(a, table, kvh, ctx, j0, qf, qpos, m, l, o);

#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    float lt = l[nq];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    const float inv = 1.0f / lt;
    const int qi = q0 + nq * 16 + c;
    if (qi < q_len) {
      bf16_t* orow = a.out + ((size_t)(q_start + qi) * a.n_heads + head) * D;
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) {
        // O^T tile: rows d = dt*16 + 4g + r
        uint2 w;
        w.x = pack_bf16(o[nq][dt][0] * inv, o[nq][dt][1] * inv);
        w.y = pack_bf16(o[nq][dt][2] * inv, o[nq][dt][3] * inv);
        *(uint2*)(orow + dt * 16 + 4 * g) = w;
      }
    }
  }
}

// ---- decode -----------------------------------------------------------------------------
// grid: (requests, kv_heads * ceil(group / 16), splits); block: 4 waves.  Handles requests
// with exactly one new token.  Scratch per (request, head, split): D floats of O, then max, sum.
template <int D>
__global__ __launch_bounds__(256) void attn_decode_kernel(AttnArgs a) {
  __shared__ float red_o[4][D][16];
  __shared__ float red_m[4][16], red_l[4][16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int r = blockIdx.x;
  const int q_start = a.cu_seqlens[r];
  if (a.cu_seqlens[r + 1] - q_start != 1) return;
  const int group = a.n_heads / a.n_kv;
  const int hblocks = (group + 15) / 16;
  const int kvh = blockIdx.y / hblocks;
  const int h0 = (blockIdx.y % hblocks) * 16;            // first head (within the group) of this block
  const int ncols = min(16, group - h0);
  const int head = kvh * group + h0 + min(c, ncols - 1);  // spare columns repeat the last head
  const int ctx = a.context_lens[r];
  const int pos = ctx - 1;
  const int* table = a.block_tables + (size_t)r * a.table_width;

  bf16x8_t qf[1][D / 32];
  int qpos[1] = {pos};
  float m[1] = {-INFINITY}, l[1] = {0.f};
  f32x4_t o[1][D / 16];
  const bf16_t* qr = a.q + ((size_t)q_start * a.n_heads + head) * D + g * 8;
#pragma unroll
  for (int dk = 0; dk < D / 32; ++dk) qf[0][dk] = frag_of(*(const u32x4_t*)(qr + dk * 32));
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) o[0][dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  int first = 0;
  if (a.window > 0) first = max(0, pos - a.window + 1) & ~31;
  const int steps = (ctx - first + 31) / 32;
  const int per_split = (steps + a.num_splits - 1) / a.num_splits;
  const int s_begin = blockIdx.z * per_split, s_end = min(steps, s_begin + per_split);
  // (Fetching the next step's fragments while this one is computed was measured: the doubled
  // fragment registers halve the occupancy and the kernel gets slower, not faster.)
  for (int s = s_begin + wave; s < s_end; s += 4) attn_step<D, 1>(a, table, kvh, ctx, first + s * 32, qf, qpos, m, l, o);

  // merge the four waves (fixed order), then write this split's partial
  float lt = l[0];
  lt += __shfl_xor(lt, 16, 64);
  lt += __shfl_xor(lt, 32, 64);
  if (g == 0) {
    red_m[wave][c] = m[0];
    red_l[wave][c] = lt;
  }
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) red_o[wave][dt * 16 + 4 * g + rr][c] = o[0][dt][rr];
  __syncthreads();
  for (int e = threadIdx.x; e < D * 16; e += 256) {
    const int d = e / 16, col = e % 16;
    if (col >= ncols) continue;
    float mg = red_m[0][col];
#pragma unroll
    for (int w = 1; w < 4; ++w) mg = fmaxf(mg, red_m[w][col]);
    const float mu = (mg == -INFINITY) ? 0.f : mg;
    float acc = 0.f, lsum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __builtin_amdgcn_exp2f(red_m[w][col] - mu);
      acc += f * red_o[w][d][col];
      lsum += f * red_l[w][col];
    }
    if (a.num_splits == 1) {  // nothing to combine: this is the answer
      a.out[((size_t)q_start * a.n_heads + (kvh * group + h0 + col)) * D + d] = float_to_bf16(acc / lsum);
      continue;
    }
    float* part = a.scratch + (((size_t)r * a.n_heads + (kvh * group + h0 + col)) * a.num_splits + blockIdx.z) * (D + 2);
    part[d] = acc;
    if (d == 0) {
      part[D] = mg;
      part[D + 1] = lsum;
    }
  }
}

// out[token, head, :] = sum_s 2^(m_s - m) O_s / sum_s 2^(m_s - m) l_s, splits in ascending order.
// grid: (requests, heads); block: one wave.  Lane s holds split s's statistics (num_splits <= 64).
// (Combining inside the decode kernel by whichever block finishes last was tried and is far
// slower: the L2 caches of the eight XCDs are not coherent with each other, so partial results
// would have to travel through memory with device-scope fences.)
__global__ __launch_bounds__(64) void attn_combine_kernel(const float* __restrict__ scratch,
                                                          const int* __restrict__ cu_seqlens,
                                                          bf16_t* __restrict__ out, int n_heads, int D,
                                                          int num_splits) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int q_start = cu_seqlens[r];
  if (cu_seqlens[r + 1] - q_start != 1) return;
  const float* base = scratch + ((size_t)r * n_heads + h) * num_splits * (D + 2);
  float ms = -INFINITY, ls = 0.f;
  if (lane < num_splits) {
    ms = base[(size_t)lane * (D + 2) + D];
    ls = base[(size_t)lane * (D + 2) + D + 1];
  }
  const float mg = wave_max(ms);
  const float mu = (mg == -INFINITY) ? 0.f : mg;
  const float ws = __builtin_amdgcn_exp2f(ms - mu);  // 0 for lanes without a split
  const float inv = 1.0f / wave_sum(ws * ls);
  for (int d = lane; d < D; d += 64) {
    float acc = 0.f;
    int s = 0;
    for (; s + 8 <= num_splits; s += 8) {   // eight independent loads in flight
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = base[(size_t)(s + u) * (D + 2) + d];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = fmaf(__shfl(ws, s + u, 64), v[u], acc);
    }
    for (; s < num_splits; ++s) acc = fmaf(__shfl(ws, s, 64), base[(size_t)s * (D + 2) + d], acc);
    out[((size_t)q_start * n_heads + h) * D + d] = float_to_bf16(acc * inv);
  }
}

// ---- dispatch ------------------------------------------------------------------------------
template <int D>
static int launch_all(const AttnArgs& a, int n_req, int max_q_len, int num_single, hipStream_t s) {
  const int group = a.n_heads / a.n_kv;
  const bool has_multi = num_single < n_req;
  if (num_single > 0) {
    const dim3 grid(n_req, a.n_kv * ((group + 15) / 16), a.num_splits);
    hipLaunchKernelGGL(attn_decode_kernel<D>, grid, dim3(256), 0, s, a);
    if (a.num_splits > 1) {
      const dim3 cgrid(n_req, a.n_heads);
      hipLaunchKernelGGL(attn_combine_kernel, cgrid, dim3(64), 0, s, a.scratch, a.cu_seqlens, a.out, a.n_heads, D,
                         a.num_splits);
    }
  }
  if (has_multi) {
    constexpr int NQ = (D <= 128) ? 2 : 1;
    const dim3 grid((max_q_len + 16 * NQ - 1) / (16 * NQ), a.n_kv * ((group + 3) / 4), n_req);
    hipLaunchKernelGGL((attn_prefill_kernel<D, NQ>), grid, dim3(256), 0, s, a, num_single > 0 ? 1 : 0);
  }
  return 0;
}

int tp_paged_attention_fast(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                            int table_width, const int* cu_seqlens, const int* context_lens, void* out, int n_tokens,
                            int n_req, int n_heads, int n_kv, int head_dim, int page_size, float scale, int window,
                            int max_q_len, int num_single, int num_splits, float* scratch, hipStream_t s) {
  if (head_dim % 32 != 0 || head_dim > 128 || page_size % 8 != 0) return -1;
  if (n_req > 65535 || n_req <= 0) return -1;
  if (num_single > 0 && (num_splits < 1 || num_splits > 64)) return -1;
  if (num_single > 0 && num_splits > 1 && scratch == nullptr) return -1;
  AttnArgs a;
  a.q = (const bf16_t*)q;
  a.k_cache = (const bf16_t*)k_cache;
  a.v_cache = (const bf16_t*)v_cache;
  a.block_tables = block_tables;
  a.table_width = table_width;
  a.cu_seqlens = cu_seqlens;
  a.context_lens = context_lens;
  a.out = (bf16_t*)out;
  a.scratch = scratch;
  a.n_heads = n_heads;
  a.n_kv = n_kv;
  a.page_size = page_size;
  a.window = window;
  a.num_splits = num_splits;
  a.scale_log2 = scale * 1.4426950408889634f;
  switch (head_dim) {
    case 32: launch_all<32>(a, n_req, max_q_len, num_single, s); break;
    case 64: launch_all<64>(a, n_req, max_q_len, num_single, s); break;
    case 96: launch_all<96>(a, n_req, max_q_len, num_single, s); break;
    case 128: launch_all<128>(a, n_req, max_q_len, num_single, s); break;
    default: return -1;
  }
  TP_CHECK_LAUNCH("paged_attention (mfma)");
  return 0;
}
