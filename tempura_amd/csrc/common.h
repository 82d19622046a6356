// Shared helpers of the gfx950 kernels: element types, reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define TP_WAVE 64

// Element type codes of the C interface.
enum TpDtype { TP_F32 = 0, TP_BF16 = 1 };

// bfloat16 as its 16 bits; conversions are explicit so rounding is in one place.
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float bf16_to_float(bf16_t v) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = ((uint32_t)v.bits) << 16;
  return c.f;
}

// Round to nearest, ties to even; NaN stays NaN.
__host__ __device__ inline bf16_t float_to_bf16(float f) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  bf16_t r;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((c.u >> 16) | 0x0040u);
    return r;
  }
  c.u += 0x7fffu + ((c.u >> 16) & 1u);
  r.bits = (uint16_t)(c.u >> 16);
  return r;
}

__device__ inline float to_float(float v) { return v; }
__device__ inline float to_float(bf16_t v) { return bf16_to_float(v); }
__device__ inline void from_float(float* p, float v) { *p = v; }
__device__ inline void from_float(bf16_t* p, float v) { *p = float_to_bf16(v); }
// four neighbouring results as one store (p aligned to four elements)
__device__ inline void from_float4(float* p, float a, float b, float c, float d) { *(float4*)p = make_float4(a, b, c, d); }
__device__ inline void from_float4(bf16_t* p, float a, float b, float c, float d) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16(a).bits | ((uint32_t)float_to_bf16(b).bits << 16);
  u.y = (uint32_t)float_to_bf16(c).bits | ((uint32_t)float_to_bf16(d).bits << 16);
  *(uint2*)p = u;
}

// cosine and sine (times factor) of pos * inv_freq: the product in float64, reduced to [0, 2 pi) there,
// sine and cosine of the small rest in float32 (every kernel that rotates uses this one routine)
__device__ inline void rope_cos_sin(int pos, double inv_freq, float factor, float& c, float& sn) {
  const double turns = (double)pos * inv_freq * 0.15915494309189535;
  const float rest = (float)((turns - floor(turns)) * 6.283185307179586);
  sincosf(rest, &sn, &c);
  c *= factor;
  sn *= factor;
}

// The q/k/v projection can finish its rows itself (mode OUT_ROPE of the bfloat16 products): the q and k heads
// come in paired order (the two elements that rotate together are neighbouring columns), so the epilogue
// rotates what it holds and stores q as bfloat16 [M, heads, head_dim], k into the cache place slots[m] and v
// into the transposed value cache: the rotation and cache-write kernel between the projection and the
// attention is gone.  The arithmetic is that kernel's, on the same float32 sums.
struct RopeOut {
  const int* positions;      // [M]
  const int* slots;          // [M] cache place (page * page_size + offset)
  const double* inv_freq;    // [rotary_dim / 2]
  const float2* cos_sin;     // [M, rotary_dim / 2] this step's table (rope_table_kernel), or nullptr
  float factor;
  int rotary_dim, n_heads, n_kv, head_dim, page_size;
  int col0;                  // first column of this launch (a launch may cover a range of columns)
  bf16_t* q_out;
  bf16_t* k_cache;           // [page, kv_head, page_size, head_dim]
  bf16_t* v_cache;           // [page, kv_head, head_dim, page_size]
};
enum { OUT_ROPE = 4 };

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TP_WAVE);
  return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TP_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` is shared memory of at least 32 floats; safe to call repeatedly.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  const int nwaves = (blockDim.x + TP_WAVE - 1) / TP_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

__device__ inline float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  const int nwaves = (blockDim.x + TP_WAVE - 1) / TP_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nwaves; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// ---- host-side error reporting ------------------------------------------------
// Every entry point returns 0 on success; otherwise tp_last_error() says why.
void tp_set_error(const char* fmt, ...);

#define TP_REQUIRE(cond, ...)    \
  do {                           \
    if (!(cond)) {               \
      tp_set_error(__VA_ARGS__); \
      return 1;                  \
    }                            \
  } while (0)

#define TP_CHECK_LAUNCH(name)                                          \
  do {                                                                 \
    hipError_t e_ = hipGetLastError();                                 \
    if (e_ != hipSuccess) {                                            \
      tp_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                        \
    }                                                                  \
  } while (0)
