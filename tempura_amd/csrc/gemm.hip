// out[M, N] (+)= x[M, K] * w[N, K]^T with float32 accumulation.
//
// gemm_tiled_kernel is the general kernel: any M, N, K, float32 or bfloat16 operands,
// plain FMA in float32 (no reduced-precision matrix mode), LDS-tiled 64x64x16 with a
// 4x4 register block per thread.  The k loop runs in ascending order for every output
// element, so a row's result does not depend on how many rows are in the batch.
// bfloat16 products at model sizes go to the MFMA kernels in gemm_mfma.hip.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename TI, typename TO, bool ACC>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TI* __restrict__ x, const TI* __restrict__ w,
                                                         TO* __restrict__ out, int M, int N, int K) {
  __shared__ float xs[BK][BM + 4];
  __shared__ float ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  // loader mapping: 64 rows x 16 k, four consecutive k per thread
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int gm = m0 + lrow;
      const TI* p = x + (size_t)gm * K + k0 + lk;
#pragma unroll
      for (int j = 0; j < 4; ++j) xs[lk + j][lrow] = (gm < M && k0 + lk + j < K) ? to_float(p[j]) : 0.f;
      const int gn = n0 + lrow;
      const TI* q = w + (size_t)gn * K + k0 + lk;
#pragma unroll
      for (int j = 0; j < 4; ++j) ws[lk + j][lrow] = (gn < N && k0 + lk + j < K) ? to_float(q[j]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= N) continue;
      TO* o = out + (size_t)gm * N + gn;
      if (ACC)
        from_float(o, to_float(*o) + acc[i][j]);
      else
        from_float(o, acc[i][j]);
    }
  }
}

// Skinny kernel for a handful of rows (decode): one wave per output column, lanes
// stride over K, float32 FMA, wave reduction.  The x rows are staged in LDS in chunks.
// Result per (row, column) is independent of the other rows in the batch.
#define SK_COLS 16   // output columns per block (4 waves x 4 columns)
#define SK_KC 512    // K chunk staged in LDS
#define SK_MAXM 8

template <typename TI, typename TO, bool ACC>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const TI* __restrict__ x, const TI* __restrict__ w,
                                                          TO* __restrict__ out, int M, int N, int K) {
  __shared__ float xs[SK_MAXM][SK_KC];
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  const int n_base = blockIdx.x * SK_COLS + wave * 4;
  float acc[4][SK_MAXM];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int m = 0; m < SK_MAXM; ++m) acc[c][m] = 0.f;
  for (int k0 = 0; k0 < K; k0 += SK_KC) {
    const int kc = min(SK_KC, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < M * SK_KC; i += blockDim.x) {
      const int m = i / SK_KC, k = i % SK_KC;
      xs[m][k] = (k < kc) ? to_float(x[(size_t)m * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int n = n_base + c;
      if (n >= N) continue;
      const TI* wr = w + (size_t)n * K + k0;
      for (int k = lane; k < kc; k += TP_WAVE) {
        const float wv = to_float(wr[k]);
#pragma unroll
        for (int m = 0; m < SK_MAXM; ++m)
          if (m < M) acc[c][m] = fmaf(wv, xs[m][k], acc[c][m]);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int n = n_base + c;
#pragma unroll
    for (int m = 0; m < SK_MAXM; ++m) {
      const float v = wave_sum(acc[c][m]);
      if (lane == 0 && n < N && m < M) {
        TO* o = out + (size_t)m * N + n;
        if (ACC)
          from_float(o, to_float(*o) + v);
        else
          from_float(o, v);
      }
    }
  }
}

template <typename TI, typename TO, bool ACC>
static void launch_generic(const void* x, const void* w, void* out, int M, int N, int K, hipStream_t s) {
  if (M <= SK_MAXM) {
    dim3 grid((N + SK_COLS - 1) / SK_COLS);
    hipLaunchKernelGGL((gemm_skinny_kernel<TI, TO, ACC>), grid, dim3(256), 0, s, (const TI*)x, (const TI*)w,
                       (TO*)out, M, N, K);
  } else {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    hipLaunchKernelGGL((gemm_tiled_kernel<TI, TO, ACC>), grid, dim3(256), 0, s, (const TI*)x, (const TI*)w,
                       (TO*)out, M, N, K);
  }
}

// Defined in gemm_mfma.hip; returns 0 when it took the product, -1 when the sizes are
// not its own (the general kernel then runs), >0 on error.
int tp_linear_mfma(const void* x, const void* w, void* out, int out_dt, int accumulate, int M, int N, int K,
                   float* scratch, size_t scratch_floats, const float* pre_ss, int pre_count, float pre_eps,
                   const void* post_w, void* post_xg, float* post_ss, int layout, int defer_reduce, int* splits_out,
                   hipStream_t s);

int tp_linear_rope_mfma(const void* x, const void* w, int w_tiled, int M, int N, int K, const float* pre_ss, int pre_count,
                        float pre_eps, const int* positions, const int* slots, const double* inv_freq, int rotary_dim,
                        float factor, int n_heads, int n_kv, int head_dim, void* q_out, void* k_cache, void* v_cache,
                        int page_size, const float* cos_sin, hipStream_t s);

// The q/k/v projection of at most 16 bfloat16 rows that finishes its rows itself: x [M, K] (or the rows of a
// split norm, see below) times w [(n_heads + 2 n_kv) * head_dim, K], the q and k heads in paired order; the
// epilogue rotates q and k (pair d of a head by positions[m] * inv_freq[d]), writes q as bfloat16
// [M, n_heads, head_dim], k into the cache place slots[m] and v into the transposed value cache (both
// bfloat16), as tp_rope_kv_write does for the rows of a plain product.  cos_sin: the step's table from
// tp_rope_table [M, rotary_dim / 2, 2], or nullptr (the epilogue then computes cosines and sines itself).
// w_tiled: the weight is in the tiled layout (see tp_linear_fused).
extern "C" int tp_linear_rope(const void* x, const void* w, int w_tiled, int M, int N, int K, const float* pre_ss, int pre_count,
                              float pre_eps, const int* positions, const int* slots, const double* inv_freq,
                              int rotary_dim, float factor, int n_heads, int n_kv, int head_dim, void* q_out,
                              void* k_cache, void* v_cache, int page_size, const float* cos_sin, hipStream_t s) {
  TP_REQUIRE(x && w && positions && slots && q_out && k_cache && v_cache, "linear_rope: missing operand");
  TP_REQUIRE(rotary_dim == 0 || inv_freq != nullptr, "linear_rope: no frequency table");
  const int r = tp_linear_rope_mfma(x, w, w_tiled, M, N, K, pre_ss, pre_count, pre_eps, positions, slots, inv_freq, rotary_dim,
                                    factor, n_heads, n_kv, head_dim, q_out, k_cache, v_cache, page_size, cos_sin, s);
  TP_REQUIRE(r == 0, "linear_rope: sizes M %d N %d K %d head_dim %d are not this product's (at most 16 rows, "
             "K %% 32 == 0, head_dim %% 16 == 0)", M, N, K, head_dim);
  TP_CHECK_LAUNCH("linear_rope");
  return 0;
}

// `scratch` (optional, `scratch_floats` float32): room for split-K partial sums of mid-sized products.
//
// The split norm (bfloat16, at most 16 rows, K % 32 == 0): with `post_w` (a float32 norm weight [N]; accumulate
// must be 1) the product also writes post_xg [M, N] = bfloat16(out * post_w) and post_ss
// [ceil(N / 16), 16], per block of 16 columns and row the sum of squares of `out`.  With `pre_ss`
// ([pre_count, 16], as written by such a product whose N is this product's K) the result rows are
// multiplied by rsqrt(sum of squares / K + pre_eps): x is then that product's post_xg.
//
// `layout` (bfloat16, at most 16 rows): bit 0, x is k-blocked [K / 8, M, 8] instead of [M, K]; bit 1, the
// gated output (accumulate == 2) is written k-blocked [N / 16, M, 8] for a product that reads it so; bit 3, post_xg
// is written k-blocked [N / 8, M, 8].
// Bit 2 (bfloat16, any number of rows, N % 16 == 0, K % 64 == 0): w is tiled, [N / 16][K / 32][64][8]: the 16 x 32
// block of rows 16 i.. and columns 32 j.. as 1,024 contiguous bytes, element (r, c) of the block at
// ((c / 8) * 16 + r) * 8 + c % 8 (the matrix cores' operand order), blocks of a row group side by side.
//
// `defer_reduce` (products of more than 16 rows whose K is split over blocks): the partial sums stay in `scratch`
// as [*splits_out, M, N] float32 and `out` is not touched; the caller's next kernel adds them (ascending).
// *splits_out == 1 means that the product wrote `out` itself.
extern "C" int tp_linear_fused(const void* x, const void* w, int in_dt, void* out, int out_dt, int accumulate, int M,
                               int N, int K, int allow_mfma, float* scratch, size_t scratch_floats,
                               const float* pre_ss, int pre_count, float pre_eps, const void* post_w, void* post_xg,
                               float* post_ss, int layout, int defer_reduce, int* splits_out, hipStream_t s) {
  if (splits_out) *splits_out = 1;
  TP_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  TP_REQUIRE(accumulate != 1 || out_dt == TP_F32, "linear: accumulating output must be float32");
  const bool split_norm = pre_ss != nullptr || post_w != nullptr || (layout & 3) != 0;
  TP_REQUIRE((layout & ~15) == 0 && (!(layout & 2) || accumulate == 2) && (!(layout & 8) || post_w != nullptr),
             "linear: bad layout flags %d", layout);
  TP_REQUIRE(!(layout & 4) || (in_dt == TP_BF16 && allow_mfma && N % 16 == 0 && K % 64 == 0),
             "linear: tiled weights are bfloat16 with N %% 16 == 0 and K %% 64 == 0 (N=%d K=%d)", N, K);
  if (split_norm) {
    TP_REQUIRE(in_dt == TP_BF16 && allow_mfma && M <= 16 && K % 32 == 0,
               "linear: the split norm and the k-blocked layout need bfloat16 operands, at most 16 rows and K %% 32 == 0 (M=%d K=%d)", M, K);
    TP_REQUIRE(post_w == nullptr || (accumulate == 1 && post_xg != nullptr && post_ss != nullptr),
               "linear: the norm preparation belongs to a product that adds into the residual stream");
    TP_REQUIRE(pre_ss == nullptr || pre_count == (K + 15) / 16, "linear: %d partial sums for K=%d", pre_count, K);
  }
  if (accumulate == 2) {  // gated-SiLU epilogue: only the matrix-core kernels have it
    TP_REQUIRE(in_dt == TP_BF16 && allow_mfma, "linear: the gated epilogue needs bfloat16 operands");
    const int r = tp_linear_mfma(x, w, out, out_dt, 2, M, N, K, scratch, scratch_floats, pre_ss, pre_count, pre_eps,
                                 nullptr, nullptr, nullptr, layout, 0, nullptr, s);
    TP_REQUIRE(r >= 0, "linear: sizes M=%d N=%d K=%d do not fit the gated epilogue", M, N, K);
    return r;
  }
  TP_REQUIRE((size_t)M * N < ((size_t)1 << 40), "linear: output too large");
  if (M == 0) return 0;
  if (in_dt == TP_BF16 && allow_mfma) {
    const int r = tp_linear_mfma(x, w, out, out_dt, accumulate, M, N, K, scratch, scratch_floats, pre_ss, pre_count,
                                 pre_eps, post_w, post_xg, post_ss, layout, defer_reduce, splits_out, s);
    if (r >= 0) return r;
  }
  TP_REQUIRE(!(layout & 4), "linear: no kernel for tiled weights at M=%d N=%d K=%d", M, N, K);
  TP_REQUIRE(!split_norm, "linear: sizes M=%d N=%d K=%d do not fit the split norm or the k-blocked layout", M, N, K);
  if (in_dt == TP_F32 && out_dt == TP_F32) {
    if (accumulate)
      launch_generic<float, float, true>(x, w, out, M, N, K, s);
    else
      launch_generic<float, float, false>(x, w, out, M, N, K, s);
  } else if (in_dt == TP_BF16 && out_dt == TP_F32) {
    if (accumulate)
      launch_generic<bf16_t, float, true>(x, w, out, M, N, K, s);
    else
      launch_generic<bf16_t, float, false>(x, w, out, M, N, K, s);
  } else if (in_dt == TP_BF16 && out_dt == TP_BF16) {
    launch_generic<bf16_t, bf16_t, false>(x, w, out, M, N, K, s);
  } else {
    TP_REQUIRE(false, "linear: unsupported dtypes in=%d out=%d", in_dt, out_dt);
  }
  TP_CHECK_LAUNCH("linear");
  return 0;
}
