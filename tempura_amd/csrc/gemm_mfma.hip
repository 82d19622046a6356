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

enum { OUT_F32 = 0, OUT_BF16 = 1, OUT_ACC_F32 = 2 };

__device__ inline bf16x8_t as_frag(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

__device__ inline void store_out(void* out, int mode, size_t idx, float v) {
  if (mode == OUT_F32)
    ((float*)out)[idx] = v;
  else if (mode == OUT_BF16)
    ((bf16_t*)out)[idx] = float_to_bf16(v);
  else
    ((float*)out)[idx] += v;
}

// ---- skinny ---------------------------------------------------------------------------
template <int MT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_mfma_kernel(const bf16_t* __restrict__ x,
                                                                      const bf16_t* __restrict__ w,
                                                                      void* __restrict__ out, int mode, int M,
                                                                      int N, int K) {
  __shared__ float red[WAVES][MT][256];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int n0 = blockIdx.x * 16;
  const int wrow = min(n0 + (lane & 15), N - 1);
  const int kofs = (lane >> 4) * 8;
  const u32x4_t* wp = (const u32x4_t*)(w + (size_t)wrow * K + kofs);
  const u32x4_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int xrow = min(t * 16 + (lane & 15), M - 1);
    xp[t] = (const u32x4_t*)(x + (size_t)xrow * K + kofs);
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int steps = K / 32;  // a step is 32 k = 4 u32x4_t per row
  int s = wave;
  // four steps in flight per wave
  for (; s + 3 * WAVES < steps; s += 4 * WAVES) {
    u32x4_t a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) a[u] = __builtin_nontemporal_load(wp + (size_t)(s + u * WAVES) * 4);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const u32x4_t b = xp[t][(size_t)(s + u * WAVES) * 4];
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(a[u]), as_frag(b), acc[t], 0, 0, 0);
      }
    }
  }
  for (; s < steps; s += WAVES) {
    const u32x4_t a = __builtin_nontemporal_load(wp + (size_t)s * 4);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const u32x4_t b = xp[t][(size_t)s * 4];
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(a), as_frag(b), acc[t], 0, 0, 0);
    }
  }
  // sum the waves' partial tiles in wave order
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][lane * 4 + r] = acc[t][r];
  __syncthreads();
  for (int e = threadIdx.x; e < MT * 256; e += WAVES * 64) {
    const int t = e / 256, q = e % 256;
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) v += red[i][t][q];
    const int l = q / 4, r = q % 4;
    const int n = n0 + (l >> 4) * 4 + r;   // weight row = output column
    const int m = t * 16 + (l & 15);
    if (n < N && m < M) store_out(out, mode, (size_t)m * N + n, v);
  }
}

// ---- tiled ----------------------------------------------------------------------------
#define TBM 128
#define TBN 128

template <int BK>
__global__ __launch_bounds__(256) void gemm_tiled_mfma_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ w, void* __restrict__ out,
                                                              int mode, int M, int N, int K) {
  constexpr int LD = BK + 8;            // padded row, in bf16 elements (conflict-free 16-byte reads)
  constexpr int CPR = BK / 8;           // 16-byte chunks per tile row
  constexpr int CPT = TBM * CPR / 256;  // chunks per thread per operand
  __shared__ __attribute__((aligned(16))) uint16_t xs[TBM * LD];
  __shared__ __attribute__((aligned(16))) uint16_t ws[TBN * LD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * TBM, n0 = blockIdx.x * TBN;

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  u32x4_t xr[CPT], wr[CPT];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + 256 * i;
      const int row = c / CPR, kc = c % CPR;
      const int gm = min(m0 + row, M - 1), gn = min(n0 + row, N - 1);
      xr[i] = *(const u32x4_t*)(x + (size_t)gm * K + k0 + kc * 8);
      wr[i] = *(const u32x4_t*)(w + (size_t)gn * K + k0 + kc * 8);
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + 256 * i;
      const int row = c / CPR, kc = c % CPR;
      *(u32x4_t*)(&xs[row * LD + kc * 8]) = xr[i];
      *(u32x4_t*)(&ws[row * LD + kc * 8]) = wr[i];
    }
  };

  // The next tile travels from global memory into registers while this one is multiplied.
  const int KT = K / BK;
  load_global(0);
  for (int kt = 0; kt < KT; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < KT) load_global((kt + 1) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      bf16x8_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = as_frag(*(const u32x4_t*)(&xs[(wm * 64 + i * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8]));
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j] = as_frag(*(const u32x4_t*)(&ws[(wn * 64 + j * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8]));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // result lane l: rows (l / 16) * 4 + r of the x tile (m), column l % 16 of the w tile (n)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + wm * 64 + i * 16 + (lane >> 4) * 4 + r;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 64 + j * 16 + (lane & 15);
        if (n < N) store_out(out, mode, (size_t)m * N + n, acc[i][j][r]);
      }
    }
  }
}

// In the skinny kernel x is the second operand, so the result lane holds weight rows
// (l / 16) * 4 + r and activation row l % 16; see the index arithmetic there.

template <int MT>
static void launch_skinny(const bf16_t* x, const bf16_t* w, void* out, int mode, int M, int N, int K, hipStream_t s) {
  const int blocks = (N + 15) / 16;
  // enough waves to keep loads in flight, but every wave should get at least a few steps
  if (K / 32 >= 64 && MT <= 2)
    hipLaunchKernelGGL((gemm_skinny_mfma_kernel<MT, 16>), dim3(blocks), dim3(16 * 64), 0, s, x, w, out, mode, M, N, K);
  else if (K / 32 >= 16)
    hipLaunchKernelGGL((gemm_skinny_mfma_kernel<MT, 8>), dim3(blocks), dim3(8 * 64), 0, s, x, w, out, mode, M, N, K);
  else
    hipLaunchKernelGGL((gemm_skinny_mfma_kernel<MT, 2>), dim3(blocks), dim3(2 * 64), 0, s, x, w, out, mode, M, N, K);
}

int tp_linear_mfma(const void* x, const void* w, void* out, int out_dt, int accumulate, int M, int N, int K,
                   hipStream_t s) {
  if (K % 32 != 0) return -1;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return -1;
  const int mode = accumulate ? OUT_ACC_F32 : (out_dt == TP_F32 ? OUT_F32 : OUT_BF16);
  const bf16_t* xb = (const bf16_t*)x;
  const bf16_t* wb = (const bf16_t*)w;
  if (M <= 64) {
    if (M <= 16)
      launch_skinny<1>(xb, wb, out, mode, M, N, K, s);
    else if (M <= 32)
      launch_skinny<2>(xb, wb, out, mode, M, N, K, s);
    else if (M <= 48)
      launch_skinny<3>(xb, wb, out, mode, M, N, K, s);
    else
      launch_skinny<4>(xb, wb, out, mode, M, N, K, s);
  } else {
    const dim3 grid((N + TBN - 1) / TBN, (M + TBM - 1) / TBM);
    if (grid.y > 65535) return -1;
    if (K % 64 == 0)
      hipLaunchKernelGGL((gemm_tiled_mfma_kernel<64>), grid, dim3(256), 0, s, xb, wb, out, mode, M, N, K);
    else
      hipLaunchKernelGGL((gemm_tiled_mfma_kernel<32>), grid, dim3(256), 0, s, xb, wb, out, mode, M, N, K);
  }
  TP_CHECK_LAUNCH("linear (mfma)");
  return 0;
}
