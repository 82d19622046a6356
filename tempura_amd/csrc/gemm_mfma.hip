// bfloat16 products on the gfx950 matrix cores: out[M, N] (+)= x[M, K] * w[N, K]^T,
// float32 accumulation (v_mfma_f32_16x16x32_bf16).
//
// Two kernels:
//  * skinny (M <= 64, decode): weight-bandwidth bound.  A block owns 16 output columns
//    (16 weight rows); its waves split K in interleaved 32-wide steps and each lane pulls
//    its 16 bytes of a weight row straight from global memory into the MFMA operand
//    registers (no LDS: a weight is used by exactly one wave).  The activations are the
//    other operand, read through the caches.  Partial tiles are summed through LDS in a
//    fixed order, so results are deterministic and a row's value does not depend on the
//    other rows of the batch.
//  * tiled (M > 64, prefill): 128x128 block tile, 64x64 per wave, K in steps of 64 (or
//    32), operands staged through padded LDS tiles; the next tile is fetched into
//    registers while the current one is multiplied.
// Fragment layout of the 16x16x32 instruction: lane l holds row (l % 16) of its operand
// and 8 consecutive k at (l / 16) * 8; the result lane l holds rows (l / 16) * 4 + r,
// r = 0..3, of column l % 16.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// OUT_SWIGLU: the weight rows alternate eight gate rows and eight up rows; output column
// 8*b + i is silu(row 16*b + i) * (row 16*b + 8 + i), stored as bfloat16 [M, N / 2].
enum { OUT_F32 = 0, OUT_BF16 = 1, OUT_ACC_F32 = 2, OUT_SWIGLU = 3 };

// g * sigmoid(g) * u with the hardware's exp2 and reciprocal (one ulp each; the result is rounded to bfloat16),
// the same arithmetic in every bfloat16 product, whatever the number of rows
__device__ inline float silu_mul(float g, float u) {
  return g * u * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}

__device__ inline bf16x8_t as_frag(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

// A decode product reads every weight once per step and never again before the whole model has streamed through
// the caches: the loads say so (nontemporal), which leaves the cache lines to the activations and measures faster
// on a chain of streaming kernels (5.7 -> 6.4 TB/s on products of these sizes).
#ifndef TP_WEIGHTS_TEMPORAL
#define TP_WLOAD(p) __builtin_nontemporal_load(p)
#else
#define TP_WLOAD(p) (*(p))
#endif

// Layouts of bfloat16 activations of at most 16 rows.  Row-major [M, K], or k-blocked [K / 8, M, 8]:
// eight consecutive k of all rows side by side, so that the operand fragments that the lanes of a
// wave fetch straight from global memory (16 bytes per row and k group) lie next to each other.
// Layout of a weight.  Row-major [N, K], or tiled (N % 16 == 0, K % 64 == 0): [N / 16][K / 32][64][8], the operand
// fragment of the MFMA for 16 weight rows and 32 of k as one run of 1,024 bytes, lane l's eight elements (row l % 16,
// k group l / 16) at l * 16.  A wave's load of a fragment then covers eight whole cache lines instead of 64-byte
// pieces of sixteen rows, which is what the address path of a CU can keep up with when the weights stream from HBM
// (the down projection of 8 rows: 26.0 -> 23.4 us), and a stage of the pipelined kernels is a plain copy.
enum { X_KBLOCKED = 1, OUT_KBLOCKED = 2, W_TILED = 4, XG_KBLOCKED = 8 };

__device__ inline void store_gated(void* out, int layout, int M, int width, int m, int col, float v) {
  const size_t idx = (layout & OUT_KBLOCKED) ? ((size_t)(col >> 3) * M + m) * 8 + (col & 7) : (size_t)m * width + col;
  ((bf16_t*)out)[idx] = float_to_bf16(v);
}

__device__ inline void store_out(void* out, int mode, size_t idx, float v) {
  if (mode == OUT_F32)
    ((float*)out)[idx] = v;
  else if (mode == OUT_BF16)
    ((bf16_t*)out)[idx] = float_to_bf16(v);
  else
    ((float*)out)[idx] += v;
}

// v: this lane's sum of column n of row m; other: the sum of column n ^ 1 (the partner of a rotary pair)
__device__ inline void rope_store(const RopeOut& rp, int m, int n, float v, float other) {
  const int h = n / rp.head_dim, d = n % rp.head_dim;
  float y = v;
  if (h < rp.n_heads + rp.n_kv && d < rp.rotary_dim) {
    float c, sn;
    if (rp.cos_sin != nullptr) {
      const float2 cs = rp.cos_sin[(size_t)m * (rp.rotary_dim >> 1) + (d >> 1)];
      c = cs.x;
      sn = cs.y;
    } else {
      rope_cos_sin(rp.positions[m], rp.inv_freq[d >> 1], rp.factor, c, sn);
    }
    // the pair is (x0, x1) = (even column, odd column): x0 c - x1 s and x0 s + x1 c
    y = (d & 1) ? other * sn + v * c : v * c - other * sn;
  }
  if (h < rp.n_heads) {
    rp.q_out[((size_t)m * rp.n_heads + h) * rp.head_dim + d] = float_to_bf16(y);
    return;
  }
  const int slot = rp.slots[m];
  const size_t page = (size_t)(slot / rp.page_size), off = (size_t)(slot % rp.page_size);
  if (h < rp.n_heads + rp.n_kv)
    rp.k_cache[((page * rp.n_kv + (h - rp.n_heads)) * rp.page_size + off) * rp.head_dim + d] = float_to_bf16(y);
  else
    rp.v_cache[((page * rp.n_kv + (h - rp.n_heads - rp.n_kv)) * rp.head_dim + d) * rp.page_size + off] = float_to_bf16(y);
}

// A root-mean-square norm split over two products (rows of at most 16 tokens).  The product that
// adds into the residual stream h also writes xg = bfloat16(h * norm weight) and, per block and row,
// the sum of squares of the columns it owns (NormPrep).  The product that consumes xg adds those
// partial sums in a fixed order and multiplies its float32 result rows by rsqrt(mean square + eps)
// (RowScale): the norm kernel between the two products is gone, and the scale is applied in float32
// after the sum instead of before the rounding to bfloat16.
struct NormPrep {
  const float* w;    // norm weight [N]; nullptr: no preparation
  bf16_t* xg;        // [M, N]
  float* ss;         // [blocks, 16]
};
struct RowScale {
  const float* ss;   // [count, 16] partial sums of squares; nullptr: no scaling
  int count;
  float inv_k, eps;
};

// RowScale, first half: every thread fetches its share of the partial sums of one row.  The loads are
// issued together, early (before the main loop), and nothing waits for them until the second half.
struct RowScaleLoads {
  float v[8];
};
__device__ inline RowScaleLoads row_scale_begin(const RowScale& pre, int nthreads) {
  RowScaleLoads ld;
#pragma unroll
  for (int i = 0; i < 8; ++i) ld.v[i] = 0.f;
  if (pre.ss == nullptr) return ld;
  const int t = threadIdx.x, nparts = min(nthreads / 16, 32);
  if (t < nparts * 16) {
    const int m = t & 15, p = t >> 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int b = p + i * nparts;
      if (b < pre.count) ld.v[i] = pre.ss[b * 16 + m];
    }
  }
  return ld;
}
// Second half: call after a barrier and follow with one; afterwards rstd[m] is valid for every thread.
__device__ inline void row_scale_finish(const RowScale& pre, const RowScaleLoads& ld, float (*part)[16], float* rstd,
                                        int nthreads) {
  const int t = threadIdx.x, nparts = min(nthreads / 16, 32);
  if (pre.ss == nullptr) {
    if (t < 16) rstd[t] = 1.0f;
    return;
  }
  if (t < nparts * 16) {
    const int m = t & 15, p = t >> 4;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += ld.v[i];
    for (int b = p + 8 * nparts; b < pre.count; b += nparts) sum += pre.ss[b * 16 + m];   // more than 8 each: rare
    part[p][m] = sum;
  }
  __syncthreads();
  if (t < 16) {
    float sum = 0.f;
    for (int p = 0; p < nparts; ++p) sum += part[p][t];
    rstd[t] = rsqrtf(sum * pre.inv_k + pre.eps);
  }
}

// ---- skinny ---------------------------------------------------------------------------
// MT: 16-row tiles of activations; NT: 16-row tiles of weights per block; WAVES: waves that
// split K.  A wave takes K in runs of four consecutive 32-wide steps (256 contiguous bytes of
// each weight row), run r going to wave r % WAVES.
template <int MT, int NT, int WAVES, int DEPTH, bool WT>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_mfma_kernel(const bf16_t* __restrict__ x,
                                                                      const bf16_t* __restrict__ w,
                                                                      void* __restrict__ out, int mode, int M,
                                                                      int N, int K, int layout, RowScale pre,
                                                                      NormPrep post, RopeOut rp) {
  __shared__ float red[WAVES][NT * MT][256];
  __shared__ float rs_part[32][16], rstd[16], ss_lds[NT][4][16];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int n0 = blockIdx.x * 16 * NT;
  const int kofs = (lane >> 4) * 8;
  const u32x4_t* wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int wrow = min(n0 + j * 16 + (lane & 15), N - 1);
    wp[j] = WT ? (const u32x4_t*)(w + (size_t)min(n0 + j * 16, N - 16) * K) + lane
                               : (const u32x4_t*)(w + (size_t)wrow * K + kofs);
  }
  constexpr int wstep = WT ? 64 : 4;   // u32x4 units per 32 of k (a compile-time stride: the four loads of a run share one address)
  // x is [M, K] row-major, or (xblocked, M <= 16) [K / 8, M, 8]: eight consecutive k of all rows side by
  // side, so that the 16 bytes the lanes of a wave fetch lie next to each other
  const u32x4_t* xp[MT];
  const bool xblocked = (layout & X_KBLOCKED) != 0;
  const int xstep = xblocked ? 4 * M : 4;   // u32x4 units per 32 of k
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int xrow = min(t * 16 + (lane & 15), M - 1);
    xp[t] = xblocked ? (const u32x4_t*)(x + ((size_t)(lane >> 4) * M + xrow) * 8) : (const u32x4_t*)(x + (size_t)xrow * K + kofs);
  }
  f32x4_t acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const RowScaleLoads rs_loads = row_scale_begin(pre, WAVES * 64);
  const int steps = K / 32;  // a step is 32 k = 4 u32x4 per row
  // DEPTH runs of four steps are fetched before any of them is multiplied: 4 * DEPTH * NT loads
  // of 16 bytes per lane are in flight, which is what keeps the memory system busy.
  for (int s0 = wave * 4; s0 < steps; s0 += WAVES * 4 * DEPTH) {
    u32x4_t a[DEPTH][NT][4];
    u32x4_t b[DEPTH][MT][4];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // steps past the end repeat the last one; their products are dropped below
        const int sidx = min(s0 + d * WAVES * 4 + u, steps - 1);
#pragma unroll
        for (int j = 0; j < NT; ++j) a[d][j][u] = TP_WLOAD(wp[j] + (size_t)sidx * wstep);
#pragma unroll
        for (int t = 0; t < MT; ++t) b[d][t][u] = xp[t][(size_t)sidx * xstep];
      }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (s0 + d * WAVES * 4 + u < steps) {
#pragma unroll
          for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int j = 0; j < NT; ++j)
              acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(a[d][j][u]), as_frag(b[d][t][u]), acc[j][t], 0, 0, 0);
        }
      }
  }
  // sum the waves' partial tiles in wave order
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][j * MT + t][lane * 4 + r] = acc[j][t][r];
  __syncthreads();
  row_scale_finish(pre, rs_loads, rs_part, rstd, WAVES * 64);
  __syncthreads();
  for (int e = threadIdx.x; e < NT * MT * 256; e += WAVES * 64) {
    const int jt = e / 256, q = e % 256;
    const int j = jt / MT, t = jt % MT;
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) v += red[i][jt][q];
    const int l = q / 4, r = q % 4;
    const int n = n0 + j * 16 + (l >> 4) * 4 + r;   // weight row = output column
    const int m = t * 16 + (l & 15);
    if (MT == 1) v *= rstd[l & 15];
    if (mode == OUT_SWIGLU) {
      if ((l >> 4) < 2 && n + 8 < N && m < M) {       // a gate row: its up row is eight further on
        float u = 0.f;
#pragma unroll
        for (int i = 0; i < WAVES; ++i) u += red[i][jt][q + 128];
        if (MT == 1) u *= rstd[l & 15];
        store_gated(out, layout, M, N / 2, m, (n0 + j * 16) / 2 + (l >> 4) * 4 + r, silu_mul(v, u));
      }
    } else if (MT == 1 && post.w != nullptr) {
      // residual add, and the next norm's preparation (mode is OUT_ACC_F32)
      float sq = 0.f;
      if (n < N && m < M) {
        float* o = (float*)out + (size_t)m * N + n;
        const float h = *o + v;
        *o = h;
        // (k-blocked on request: the product that consumes these rows then reads them straight from memory as operands)
        post.xg[(layout & XG_KBLOCKED) ? ((size_t)(n >> 3) * M + m) * 8 + (n & 7) : (size_t)m * N + n] = float_to_bf16(h * post.w[n]);
        sq = h * h;
      }
      sq += __shfl_xor(sq, 1, 64);      // the four columns r = 0..3 of this row
      sq += __shfl_xor(sq, 2, 64);
      if (r == 0) ss_lds[j][l >> 4][l & 15] = sq;
    } else if (mode == OUT_ROPE) {
      const float other = __shfl_xor(v, 1, 64);   // r and r ^ 1 are neighbouring lanes
      if (n < N && m < M) rope_store(rp, m, n, v, other);
    } else if (n < N && m < M) {
      store_out(out, mode, (size_t)m * N + n, v);
    }
  }
  if (MT == 1 && post.w != nullptr) {
    __syncthreads();
    if (threadIdx.x < 16) {
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) sum += ss_lds[j][c][threadIdx.x];
      post.ss[blockIdx.x * 16 + threadIdx.x] = sum;
    }
  }
}

// ---- skinny, activations through LDS (M <= 16) ------------------------------------------
// With more than one activation row the second operand is a gather of short pieces of several
// rows, and the address path, not HBM, limits the kernel.  Here the block copies the
// activations of one K chunk (1,024 wide) into LDS with wide coalesced loads and every wave
// reads its operand fragments from there; the weight stream is as above, one run of four steps
// per wave and chunk, the next chunk's weights and activations already in flight while this
// chunk is multiplied.  Two LDS buffers, one barrier per chunk.  The LDS row is padded by 8 elements:
// 16-byte reads of 16 rows then hit 64 different banks.
#define LKC 1024            // K elements per chunk with eight waves

// A wave's weights of four chunks (one run per chunk) and the activations of two chunks are requested
// before anything is multiplied, and again as soon as their registers are free, always in the order in
// which they are consumed (loads return in order): a block has 256 bytes per lane in flight from its
// first cycle.  (Measured against one chunk of prefetch: 5-10 % faster at 8 and 16 rows.)
template <int NT, int WAVES, bool WT>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_lds_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                               void* __restrict__ out, int mode, int M, int N, int K,
                                                               int layout, RowScale pre, NormPrep post, RopeOut rp) {
  constexpr int THREADS = WAVES * 64, G = 1;
  constexpr int KC = WAVES * 128;        // K elements per chunk: one run of four steps per wave
  constexpr int LD = KC + 8;             // padded LDS row
  constexpr int TPR = THREADS / 16;      // threads that copy one activation row, 16 bytes each, four passes
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][16 * LD];
  __shared__ float red[WAVES][NT][256];
  __shared__ float rs_part[32][16], rstd[16], ss_lds[NT][4][16];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int kw = wave;
  const int n0 = blockIdx.x * 16 * NT;
  const int kofs = (lane >> 4) * 8;
  const u32x4_t* wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int wrow = min(n0 + j * 16 + (lane & 15), N - 1);
    wp[j] = WT ? (const u32x4_t*)(w + (size_t)min(n0 + j * 16, N - 16) * K) + lane
                               : (const u32x4_t*)(w + (size_t)wrow * K + kofs);
  }
  constexpr int wstep = WT ? 64 : 4;
  const int xrow = tid / TPR, xcol = (tid % TPR) * 8;
  const bool xload = xrow < M;
  const bf16_t* xsrc = x + (size_t)min(xrow, M - 1) * K + xcol;
  f32x4_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const int steps = K / 32;
  const int chunks = (K + KC - 1) / KC;

  u32x4_t a[4][NT][4], xr[2][4];
  auto load_w = [&](int ch, int slot) {
    const int s0 = ch * (KC / 32) + kw * 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int sidx = min(s0 + u, steps - 1);
#pragma unroll
      for (int j = 0; j < NT; ++j) a[slot][j][u] = TP_WLOAD(wp[j] + (size_t)sidx * wstep);
    }
  };
  auto load_x = [&](int ch, int slot) {
    if (xload) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int k = ch * KC + p * TPR * 8 + xcol;
        xr[slot][p] = (k < K) ? *(const u32x4_t*)(xsrc + (size_t)ch * KC + p * TPR * 8) : (u32x4_t){0u, 0u, 0u, 0u};
      }
    }
  };
  load_x(0, 0);
  load_w(0, 0);
  if (chunks > 1) { load_x(1, 1); load_w(1, 1); }
  if (chunks > 2) load_w(2, 2);
  if (chunks > 3) load_w(3, 3);
  const RowScaleLoads rs_loads = row_scale_begin(pre, THREADS);
  for (int ch0 = 0; ch0 < chunks; ch0 += 4) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int ch = ch0 + c;
      if (ch < chunks) {
        const int buf = c & 1;
        if (xload) {
#pragma unroll
          for (int p = 0; p < 4; ++p) *(u32x4_t*)(&xs[buf][xrow * LD + p * TPR * 8 + xcol]) = xr[c & 1][p];
        }
        __syncthreads();
        if (ch + 2 < chunks) load_x(ch + 2, c & 1);
        const int s0 = ch * (KC / 32) + kw * 4;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (s0 + u < steps) {
            const u32x4_t b = *(const u32x4_t*)(&xs[buf][(lane & 15) * LD + (kw * 4 + u) * 32 + kofs]);
#pragma unroll
            for (int j = 0; j < NT; ++j)
              acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(a[c][j][u]), as_frag(b), acc[j], 0, 0, 0);
          }
        }
        if (ch + 4 < chunks) load_w(ch + 4, c);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][j][lane * 4 + r] = acc[j][r];
  __syncthreads();
  row_scale_finish(pre, rs_loads, rs_part, rstd, THREADS);
  __syncthreads();
  for (int e = tid; e < G * NT * 256; e += THREADS) {
    const int gj = e / 256, q = e % 256;
    const int ge = gj / NT, j = gj % NT;            // the group and tile this element belongs to
    const int nt0 = ((blockIdx.x * G + ge) * NT + j) * 16;
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) v += red[ge * WAVES + i][j][q];
    const int l = q / 4, r = q % 4;
    const int n = nt0 + (l >> 4) * 4 + r;
    const int m = l & 15;
    v *= rstd[m];
    if (mode == OUT_SWIGLU) {
      if ((l >> 4) < 2 && n + 8 < N && m < M) {
        float u = 0.f;
#pragma unroll
        for (int i = 0; i < WAVES; ++i) u += red[ge * WAVES + i][j][q + 128];
        u *= rstd[m];
        store_gated(out, layout, M, N / 2, m, nt0 / 2 + (l >> 4) * 4 + r, silu_mul(v, u));
      }
    } else if (post.w != nullptr) {
      float sq = 0.f;
      if (n < N && m < M) {
        float* o = (float*)out + (size_t)m * N + n;
        const float h = *o + v;
        *o = h;
        // (k-blocked on request: the product that consumes these rows then reads them straight from memory as operands)
        post.xg[(layout & XG_KBLOCKED) ? ((size_t)(n >> 3) * M + m) * 8 + (n & 7) : (size_t)m * N + n] = float_to_bf16(h * post.w[n]);
        sq = h * h;
      }
      sq += __shfl_xor(sq, 1, 64);
      sq += __shfl_xor(sq, 2, 64);
      if (r == 0) ss_lds[gj][l >> 4][m] = sq;
    } else if (mode == OUT_ROPE) {
      const float other = __shfl_xor(v, 1, 64);
      if (n < N && m < M) rope_store(rp, m, n, v, other);
    } else if (n < N && m < M) {
      store_out(out, mode, (size_t)m * N + n, v);
    }
  }
  if (post.w != nullptr) {
    __syncthreads();
    if (tid < 16 * G * NT) {
      const int gj = tid / 16, m = tid % 16;
      const int tile = blockIdx.x * G * NT + gj;
      float sum = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) sum += ss_lds[gj][c][m];
      if (tile * 16 < N) post.ss[tile * 16 + m] = sum;
    }
  }
}

// ---- tiled ----------------------------------------------------------------------------
// Block of four waves (2 x 2); a wave owns WMT x WNT result tiles of 16 x 16, so the block
// tile is (32 WMT) x (32 WNT).  blockIdx.z splits K: with more than one split every block
// writes its float32 partial tile to `partial` [split, M, N] and a second kernel adds the
// splits in ascending order and applies the epilogue (so the result does not depend on timing).
// Measured on MI355X: two blocks per CU matter more than a larger tile (a 256 x 128 tile or
// a second set of prefetch registers drops occupancy to one wave per SIMD and loses a third).
template <int BK, int WMT, int WNT>
__global__ __launch_bounds__(256) void gemm_tiled_mfma_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ w, void* __restrict__ out,
                                                              float* __restrict__ partial, int mode, int M, int N,
                                                              int K, int xcd_order) {
  constexpr int BM = 32 * WMT, BN = 32 * WNT;
  constexpr int LD = BK + 8;            // padded row, in bf16 elements (conflict-free 16-byte reads)
  constexpr int CPR = BK / 8;           // 16-byte chunks per tile row
  constexpr int XCPT = BM * CPR / 256;  // chunks per thread, x tile
  constexpr int WCPT = BN * CPR / 256;  // chunks per thread, w tile
  __shared__ __attribute__((aligned(16))) uint16_t xs[BM * LD];
  __shared__ __attribute__((aligned(16))) uint16_t ws[BN * LD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  int bm = blockIdx.y, bn = blockIdx.x;
  if (xcd_order) {
    // Blocks go to the eight XCDs round robin by launch order, and each XCD has an L2 of its own.
    // XCD c takes the column blocks c, c + 8, ...; the blocks it runs at the same time form an
    // 8 x 8 patch of (row block, column block), so that every weight tile and every activation
    // tile it fetches is used by eight blocks while it is still in that L2.
    const int MB = (M + BM - 1) / BM, NB = (N + BN - 1) / BN;
    const int Q = (NB + 7) / 8, MS = (MB + 7) / 8;
    const int c = blockIdx.x % 8, j = blockIdx.x / 8;
    const int t = j / 64, r = j % 64;
    bm = (t % MS) * 8 + r % 8;
    bn = c + 8 * ((t / MS) * 8 + r / 8);
    if (bm >= MB || bn >= NB || (t / MS) * 8 + r / 8 >= Q) return;
  }
  const int m0 = bm * BM, n0 = bn * BN;
  // this block's share of K, in tiles
  const int KT_all = K / BK;
  const int per = (KT_all + gridDim.z - 1) / gridDim.z;
  const int kt_begin = blockIdx.z * per, kt_end = min(KT_all, kt_begin + per);

  f32x4_t acc[WMT][WNT];
#pragma unroll
  for (int i = 0; i < WMT; ++i)
#pragma unroll
    for (int j = 0; j < WNT; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  u32x4_t xr[XCPT], wr[WCPT];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < XCPT; ++i) {
      const int c = tid + 256 * i;
      const int gm = min(m0 + c / CPR, M - 1);
      xr[i] = *(const u32x4_t*)(x + (size_t)gm * K + k0 + (c % CPR) * 8);
    }
#pragma unroll
    for (int i = 0; i < WCPT; ++i) {
      const int c = tid + 256 * i;
      const int gn = min(n0 + c / CPR, N - 1);
      wr[i] = *(const u32x4_t*)(w + (size_t)gn * K + k0 + (c % CPR) * 8);
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < XCPT; ++i) {
      const int c = tid + 256 * i;
      *(u32x4_t*)(&xs[(c / CPR) * LD + (c % CPR) * 8]) = xr[i];
    }
#pragma unroll
    for (int i = 0; i < WCPT; ++i) {
      const int c = tid + 256 * i;
      *(u32x4_t*)(&ws[(c / CPR) * LD + (c % CPR) * 8]) = wr[i];
    }
  };

  // The next tile travels from global memory into registers while this one is multiplied.
  if (kt_begin < kt_end) load_global(kt_begin * BK);
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < kt_end) load_global((kt + 1) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      bf16x8_t b[WNT];
#pragma unroll
      for (int j = 0; j < WNT; ++j)
        b[j] = as_frag(*(const u32x4_t*)(&ws[(wn * 16 * WNT + j * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8]));
#pragma unroll
      for (int i = 0; i < WMT; ++i) {
        const bf16x8_t a =
            as_frag(*(const u32x4_t*)(&xs[(wm * 16 * WMT + i * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8]));
#pragma unroll
        for (int j = 0; j < WNT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[j], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // result lane l: rows (l / 16) * 4 + r of the x tile (m), column l % 16 of the w tile (n)
#pragma unroll
  for (int i = 0; i < WMT; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + wm * 16 * WMT + i * 16 + (lane >> 4) * 4 + r;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < WNT; ++j) {
        const int nt = n0 + wn * 16 * WNT + j * 16;   // first column of this 16-wide tile
        const int n = nt + (lane & 15);
        if (gridDim.z > 1) {
          if (n < N) partial[((size_t)blockIdx.z * M + m) * N + n] = acc[i][j][r];
        } else if (mode == OUT_SWIGLU) {
          const float u = __shfl_xor(acc[i][j][r], 8, 64);   // the up row sits eight columns to the right
          if ((lane & 8) == 0 && n + 8 < N)
            ((bf16_t*)out)[(size_t)m * (N / 2) + nt / 2 + (lane & 7)] = float_to_bf16(silu_mul(acc[i][j][r], u));
        } else if (n < N) {
          store_out(out, mode, (size_t)m * N + n, acc[i][j][r]);
        }
      }
    }
  }
}

// Adds the K splits of `partial` [splits, M, N] in ascending order and applies the epilogue.
__global__ void gemm_splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ out, int mode,
                                          int splits, int M, int N) {
  const size_t total = (size_t)M * N;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (mode == OUT_SWIGLU) {
    // one thread per output element: column 8 b + i pairs rows 16 b + i and 16 b + 8 + i
    const int half = N / 2;
    if (idx >= (size_t)M * half) return;
    const int m = (int)(idx / half), c = (int)(idx % half);
    const int ng = (c / 8) * 16 + (c % 8);
    float g = 0.f, u = 0.f;
    for (int s = 0; s < splits; ++s) {
      g += partial[(size_t)s * total + (size_t)m * N + ng];
      u += partial[(size_t)s * total + (size_t)m * N + ng + 8];
    }
    ((bf16_t*)out)[idx] = float_to_bf16(silu_mul(g, u));
    return;
  }
  if (idx >= total) return;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(size_t)s * total + idx];
  store_out(out, mode, idx, v);
}

// Adds the K splits of `partial` [splits, M, N] (ascending) into the float32 residual rows h [M, N] and
// writes the root-mean-square norm of the updated rows: out = h / sqrt(mean(h^2) + eps) * w.  One block
// per row; takes the place of the reduction kernel and the norm kernel that would follow it.
// Each thread owns four neighbouring columns (N % 4 == 0); all its loads are issued before the first sum.
template <typename TO>
__global__ __launch_bounds__(1024) void splitk_add_rmsnorm_kernel(const float* __restrict__ partial, int splits,
                                                                   float* __restrict__ h, const float* __restrict__ w,
                                                                   float eps, TO* __restrict__ out, int M, int N) {
  __shared__ float red[32];
  const int m = blockIdx.x;
  const size_t total = (size_t)M * N;
  float* hr = h + (size_t)m * N;
  constexpr int MAXC = 4;                       // column groups per thread: N <= 4 * 1024 * MAXC
  f32x4_t acc[MAXC];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int n = (threadIdx.x + i * 1024) * 4;
    acc[i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    if (n < N) {
      f32x4_t p[16];
#pragma unroll
      for (int s = 0; s < 16; ++s)
        if (s < splits) p[s] = *(const f32x4_t*)(partial + (size_t)s * total + (size_t)m * N + n);
      const f32x4_t base = *(const f32x4_t*)(hr + n);
      f32x4_t add = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 16; ++s)
        if (s < splits) add += p[s];
      acc[i] = base + add;
      *(f32x4_t*)(hr + n) = acc[i];
      ss += acc[i][0] * acc[i][0] + acc[i][1] * acc[i][1] + acc[i][2] * acc[i][2] + acc[i][3] * acc[i][3];
    }
  }
  ss = block_sum(ss, red);
  const float scale = rsqrtf(ss / (float)N + eps);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int n = (threadIdx.x + i * 1024) * 4;
    if (n < N) {
      const f32x4_t wv = *(const f32x4_t*)(w + n);
#pragma unroll
      for (int e = 0; e < 4; ++e) from_float(out + (size_t)m * N + n + e, acc[i][e] * scale * wv[e]);
    }
  }
}

extern "C" int tp_splitk_add_rmsnorm(const float* partial, int splits, float* h, const float* w, float eps, void* out,
                                     int out_dt, int M, int N, hipStream_t s) {
  TP_REQUIRE(M > 0 && N > 0 && splits >= 1 && splits <= 16, "splitk_add_rmsnorm: bad sizes");
  TP_REQUIRE(N % 4 == 0 && N <= 16384, "splitk_add_rmsnorm: width %d must be a multiple of 4, at most 16384", N);
  if (out_dt == TP_BF16)
    hipLaunchKernelGGL(splitk_add_rmsnorm_kernel<bf16_t>, dim3(M), dim3(1024), 0, s, partial, splits, h, w, eps, (bf16_t*)out, M, N);
  else if (out_dt == TP_F32)
    hipLaunchKernelGGL(splitk_add_rmsnorm_kernel<float>, dim3(M), dim3(1024), 0, s, partial, splits, h, w, eps, (float*)out, M, N);
  else
    TP_REQUIRE(false, "splitk_add_rmsnorm: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("splitk_add_rmsnorm");
  return 0;
}

// In the skinny kernel x is the second operand, so the result lane holds weight rows
// (l / 16) * 4 + r and activation row l % 16; see the index arithmetic there.

// Tuning knobs of the skinny kernel (0 = choose by shape); set through tp_linear_tune.
static int g_tune_waves = 0, g_tune_nt = 0, g_tune_depth = 0;   // depth 9 selects the LDS kernel
static int g_tune_splits = 0, g_tune_mid = 0;                    // mid = 1: 17..64 rows stay on the skinny kernel
static int g_tune_order = 0;   // large products: 1 tiled kernel, plain block order; 2 tiled, XCD patches; 3 pipelined kernel

// Defined in gemm_pipe.hip; 0 when it took the product, -1 when the sizes are not its own.
int tp_linear_pipe(const bf16_t* x, const bf16_t* w, int w_tiled, void* out, int mode, int M, int N, int K, float* scratch,
                   size_t scratch_floats, int tune_splits, const RopeOut* rope, int defer, int* splits_out, hipStream_t s);

int tp_linear_pipe64(const bf16_t* x, const bf16_t* w, int w_tiled, void* out, int mode, int M, int N, int K, float* scratch,
                     size_t scratch_floats, int tune_splits, int defer, int* splits_out, hipStream_t s);

extern int g_pipe_big;
// order: 1 tiled plain, 2 tiled XCD-aware, 3 pipelined; 5 / 6: pipelined with 256 x 256 tiles always / never;
// 7 / 8: with 256 x 192 tiles wherever N is a multiple of 192 / never
extern "C" void tp_linear_tune_tile(int order) {
  g_pipe_big = order == 5 ? 1 : (order == 6 ? 2 : (order == 7 ? 3 : (order == 8 ? 4 : 0)));
  g_tune_order = order >= 5 ? 0 : order;
}

extern int g_pipe_mid;
// the pipelined product's 128 x 128 blocks: 0 chosen by shape, 1 for every product of more than 128 rows, 2 never
extern "C" void tp_linear_tune_mid_tile(int v) { g_pipe_mid = v; }

extern int g_pipe64_narrow;
// the 64-row pipeline's blocks: 0 chosen by shape, 1 always 64 columns wide, 2 always 128
extern "C" void tp_linear_tune_narrow(int v) { g_pipe64_narrow = v; }

extern "C" void tp_linear_tune_mid(int mid, int splits) {
  g_tune_mid = mid;
  g_tune_splits = splits;
}

extern "C" void tp_linear_tune(int waves, int nt, int depth) {
  g_tune_waves = waves;
  g_tune_nt = nt;
  g_tune_depth = depth;
}

template <int MT, int NT, int WAVES, int DEPTH>
static void launch_skinny4(const bf16_t* x, const bf16_t* w, void* out, int mode, int M, int N, int K, int layout,
                           RowScale pre, NormPrep post, const RopeOut& rp, hipStream_t s) {
  const int blocks = (N + 16 * NT - 1) / (16 * NT);
  if (layout & W_TILED)
    hipLaunchKernelGGL((gemm_skinny_mfma_kernel<MT, NT, WAVES, DEPTH, true>), dim3(blocks), dim3(WAVES * 64), 0, s, x, w, out,
                       mode, M, N, K, layout, pre, post, rp);
  else
    hipLaunchKernelGGL((gemm_skinny_mfma_kernel<MT, NT, WAVES, DEPTH, false>), dim3(blocks), dim3(WAVES * 64), 0, s, x, w, out,
                       mode, M, N, K, layout, pre, post, rp);
}

template <int MT>
static void launch_skinny(const bf16_t* x, const bf16_t* w, void* out, int mode, int M, int N, int K, int layout,
                          RowScale pre, NormPrep post, const RopeOut& rp, hipStream_t s) {
  // every wave should get at least one run of four steps; small N wants many waves per block
  // (one block per 16 columns is all the parallelism there is), large N fewer and two row tiles
  // Measured on MI355X at Llama-8B shapes: eight waves with two runs in flight each stream
  // fastest (5.7-6.3 TB/s with one activation row); wider blocks or two row tiles never won.
  const int runs = K / 128;
  int waves = runs >= 8 ? 8 : (runs >= 4 ? 4 : 2);
  int nt = 1;
  int depth = (runs >= 2 * waves && MT <= 2) ? 2 : 1;
  if (g_tune_waves) waves = g_tune_waves;
  if (g_tune_nt) nt = g_tune_nt;
  if (g_tune_depth) depth = g_tune_depth;
  if (post.w != nullptr) nt = 1;   // the consumer counts one partial sum per 16 columns
  if constexpr (MT == 1) {
    // several activation rows: feed them through LDS, unless K is so long that the barrier per
    // chunk costs more than the gather (measured: K = 14336 is faster without)
    bool lds = M > 1 && K >= 2 * LKC && K <= 8 * LKC && !(layout & X_KBLOCKED);
    if (g_tune_depth && !(layout & X_KBLOCKED)) lds = g_tune_depth == 9;
    if (lds) {
      if (nt > 2) nt = 2;
      const int blocks = (N + 16 * nt - 1) / (16 * nt);
      const bool wt = (layout & W_TILED) != 0;
#define LDS_CASE(NT_, WT_) \
  hipLaunchKernelGGL((gemm_skinny_lds_kernel<NT_, 8, WT_>), dim3(blocks), dim3(512), 0, s, x, w, out, mode, M, N, K, layout, pre, post, rp)
      if (nt == 2 && wt) LDS_CASE(2, true);
      else if (nt == 2) LDS_CASE(2, false);
      else if (wt) LDS_CASE(1, true);
      else LDS_CASE(1, false);
#undef LDS_CASE
      return;
    }
  }
  if (MT > 2 && waves > 8) waves = 8;       // LDS for the partial tiles
  if (MT > 1) nt = 1;
  if (MT > 2 || nt > 2) depth = 1;           // registers
#define CASE(NT_, W_, D_) \
  if (nt == NT_ && waves == W_ && depth == D_) return launch_skinny4<MT, NT_, W_, D_>(x, w, out, mode, M, N, K, layout, pre, post, rp, s)
  CASE(1, 16, 1);
  CASE(1, 8, 1);
  CASE(1, 4, 1);
  CASE(1, 2, 1);
  if constexpr (MT <= 2) {
    CASE(1, 16, 2);
    CASE(1, 8, 2);
    CASE(1, 4, 2);
  }
  if constexpr (MT == 1) {
    CASE(2, 16, 1);
    CASE(2, 8, 1);
    CASE(2, 4, 1);
    CASE(2, 16, 2);
    CASE(2, 8, 2);
    CASE(2, 4, 2);
    CASE(4, 8, 1);
    CASE(4, 4, 1);
  }
#undef CASE
  launch_skinny4<MT, 1, 8, 1>(x, w, out, mode, M, N, K, layout, pre, post, rp, s);
}

// The q/k/v projection of at most 16 rows with rotation and cache write in its epilogue (see RopeOut).
// N = (n_heads + 2 n_kv) * head_dim.  Returns -1 for sizes this path does not take.
int tp_linear_rope_mfma(const void* x, const void* w, int w_tiled, int M, int N, int K, const float* pre_ss, int pre_count,
                        float pre_eps, const int* positions, const int* slots, const double* inv_freq, int rotary_dim,
                        float factor, int n_heads, int n_kv, int head_dim, void* q_out, void* k_cache, void* v_cache,
                        int page_size, const float* cos_sin, hipStream_t s) {
  if (M < 1 || (M > 16 && M <= 128) || K % 32 != 0 || head_dim % 16 != 0 || rotary_dim % 2 != 0 || rotary_dim > head_dim) return -1;
  if (N != (n_heads + 2 * n_kv) * head_dim || page_size < 1) return -1;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return -1;
  // w_tiled: bit 0, the weight is tiled; bit 1 (at most 16 rows), x is k-blocked [K / 8, M, 8]
  if ((w_tiled & 1) && (N % 16 != 0 || K % 64 != 0)) return -1;
  if ((w_tiled & 2) && M > 16) return -1;
  const RowScale pre = {pre_ss, pre_count, 1.0f / (float)K, pre_eps};
  const NormPrep post = {nullptr, nullptr, nullptr};
  const RopeOut rp = {positions, slots, inv_freq, (const float2*)cos_sin, factor, rotary_dim, n_heads, n_kv, head_dim, page_size,
                      0, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache};
  if (M > 16) {
    // long steps: the pipelined kernels, whose wave tiles of 64 columns must each lie inside q, k or v (heads of a
    // multiple of 64; the wider tiles are left out unless the heads are multiples of 128), with the step's table
    // of cosines and sines
    if (head_dim % 64 != 0 || rotary_dim % 8 != 0 || cos_sin == nullptr || pre_ss != nullptr || page_size % 8 != 0) return -1;
    return tp_linear_pipe((const bf16_t*)x, (const bf16_t*)w, w_tiled & 1, nullptr, OUT_ROPE, M, N, K, nullptr, 0, 0, &rp, 0, nullptr, s);
  }
  launch_skinny<1>((const bf16_t*)x, (const bf16_t*)w, nullptr, OUT_ROPE, M, N, K, (w_tiled & 1 ? W_TILED : 0) | (w_tiled & 2 ? X_KBLOCKED : 0),
                   pre, post, rp, s);
  return 0;
}

// accumulate: 0 store, 1 add into the float32 output, 2 gated-SiLU epilogue (see OUT_SWIGLU).
// pre_ss / post_w: the split norm (RowScale / NormPrep above), at most 16 rows; nullptr without.
int tp_linear_mfma(const void* x, const void* w, void* out, int out_dt, int accumulate, int M, int N, int K,
                   float* scratch, size_t scratch_floats, const float* pre_ss, int pre_count, float pre_eps,
                   const void* post_w, void* post_xg, float* post_ss, int layout, int defer_reduce, int* splits_out,
                   hipStream_t s) {
  if (splits_out) *splits_out = 1;
  if (K % 32 != 0) return -1;
  const int w_tiled = (layout & W_TILED) != 0;
  if (w_tiled && (N % 16 != 0 || K % 64 != 0)) return -1;
  if ((layout & (X_KBLOCKED | OUT_KBLOCKED | XG_KBLOCKED)) != 0 && M > 16) return -1;
  if ((layout & XG_KBLOCKED) && (post_w == nullptr || N % 8 != 0)) return -1;
  if ((layout & OUT_KBLOCKED) && accumulate != 2) return -1;
  if ((pre_ss != nullptr || post_w != nullptr) && M > 16) return -1;
  if (post_w != nullptr && accumulate != 1) return -1;
  const RowScale pre = {pre_ss, pre_count, 1.0f / (float)K, pre_eps};
  const NormPrep post = {(const float*)post_w, (bf16_t*)post_xg, post_ss};
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return -1;
  if (accumulate == 2 && (N % 16 != 0 || out_dt != TP_BF16)) return -1;
  const int mode = accumulate == 2 ? OUT_SWIGLU : (accumulate ? OUT_ACC_F32 : (out_dt == TP_F32 ? OUT_F32 : OUT_BF16));
  const bf16_t* xb = (const bf16_t*)x;
  const bf16_t* wb = (const bf16_t*)w;
  const bool mid_ok = scratch != nullptr && g_tune_mid != 1;
  const RopeOut no_rope = {};
  if (M <= 16 || (M <= 64 && !mid_ok)) {
    if (M <= 16)
      launch_skinny<1>(xb, wb, out, mode, M, N, K, layout, pre, post, no_rope, s);
    else if (M <= 32)
      launch_skinny<2>(xb, wb, out, mode, M, N, K, layout, pre, post, no_rope, s);
    else if (M <= 48)
      launch_skinny<3>(xb, wb, out, mode, M, N, K, layout, pre, post, no_rope, s);
    else
      launch_skinny<4>(xb, wb, out, mode, M, N, K, layout, pre, post, no_rope, s);
  } else {
    // large products: 128 x 128 tiles.  Between 17 and 128 rows the weights are still the traffic:
    // 64 x 128 tiles, and K split over blockIdx.z until there are blocks for every CU.
    // the pipelined kernels: from 65 rows on (their 128 x 128 blocks against two 64-row blocks that each fetch
    // the weights: 72 to 128 rows of the 8B shapes 26 -> 17..21 us, 43 -> 31..34 us, 21 -> 16 us, 52 -> 46 us)
    const bool pipe = g_tune_order ? g_tune_order == 3 : M > 64;
    const bool pipe64 = !pipe && M <= 128 && scratch != nullptr && g_tune_mid != 2;
    if (pipe && tp_linear_pipe(xb, wb, w_tiled, out, mode, M, N, K, scratch, scratch_floats, g_tune_splits, nullptr, defer_reduce,
                               splits_out, s) == 0) {
      // taken by the pipelined kernel
    } else if (pipe64 && tp_linear_pipe64(xb, wb, w_tiled, out, mode, M, N, K, scratch, scratch_floats, g_tune_splits,
                                          defer_reduce, splits_out, s) == 0) {
      // taken by the 64-row pipelined kernel
    } else if (w_tiled) {
      return -1;   // the kernels below read row-major weights only
    } else if (M > 128 || scratch == nullptr) {
      dim3 grid((N + 127) / 128, (M + 127) / 128);
      if (grid.y > 65535) return -1;
      const int xcd_order = g_tune_order != 1;
      if (xcd_order) {  // one-dimensional grid: 8 XCDs x patches of 64 blocks
        const int Q = ((int)grid.x + 7) / 8, MS = ((int)grid.y + 7) / 8, QS = (Q + 7) / 8;
        grid = dim3(8 * QS * MS * 64, 1);
      }
      if (K % 64 == 0)
        hipLaunchKernelGGL((gemm_tiled_mfma_kernel<64, 4, 4>), grid, dim3(256), 0, s, xb, wb, out, nullptr, mode, M, N, K,
                           xcd_order);
      else
        hipLaunchKernelGGL((gemm_tiled_mfma_kernel<32, 4, 4>), grid, dim3(256), 0, s, xb, wb, out, nullptr, mode, M, N, K,
                           xcd_order);
    } else {
      const int nb = (N + 127) / 128, mb = (M + 63) / 64;
      int splits = g_tune_splits ? g_tune_splits : (512 + nb * mb - 1) / (nb * mb);
      const int kt = K / (K % 64 == 0 ? 64 : 32);
      splits = max(1, min(splits, min(16, kt / 4)));
      while (splits > 1 && (size_t)splits * M * N > scratch_floats) --splits;
      const dim3 grid(nb, mb, splits);
      if (K % 64 == 0)
        hipLaunchKernelGGL((gemm_tiled_mfma_kernel<64, 2, 4>), grid, dim3(256), 0, s, xb, wb, out, scratch, mode, M, N, K, 0);
      else
        hipLaunchKernelGGL((gemm_tiled_mfma_kernel<32, 2, 4>), grid, dim3(256), 0, s, xb, wb, out, scratch, mode, M, N, K, 0);
      if (splits > 1 && defer_reduce && splits_out != nullptr && mode != OUT_SWIGLU) {
        *splits_out = splits;   // the caller's next kernel adds the partial sums [splits, M, N] in `scratch`
      } else if (splits > 1) {
        const size_t n_out = mode == OUT_SWIGLU ? (size_t)M * (N / 2) : (size_t)M * N;
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s, scratch, out,
                           mode, splits, M, N);
      }
    }
  }
  TP_CHECK_LAUNCH("linear (mfma)");
  return 0;
}
