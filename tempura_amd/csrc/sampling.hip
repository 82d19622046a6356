// Picking the next token from float32 logits: argmax and (below) filtered sampling.
#include <math.h>

#include "common.h"

// ---- argmax -----------------------------------------------------------------------
// One block per row.  On exact ties the LAST maximum wins, as the reference's greedy
// rule does (/root/reference/engine/src/model.rs:459-473).  NaN never wins.
__device__ inline void argmax_merge(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i > bi)) {
    bv = v;
    bi = i;
  }
}

__global__ void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  float bv = -INFINITY;
  int bi = -1;
  for (int j = threadIdx.x; j < vocab; j += blockDim.x) argmax_merge(bv, bi, row[j], j);
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, TP_WAVE);
    const int oi = __shfl_xor(bi, o, TP_WAVE);
    argmax_merge(bv, bi, ov, oi);
  }
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  if (lane == 0) {
    sv[wave] = bv;
    si[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int nw = (blockDim.x + TP_WAVE - 1) / TP_WAVE;
    for (int i = 1; i < nw; ++i) argmax_merge(bv, bi, sv[i], si[i]);
    out[blockIdx.x] = bi < 0 ? vocab - 1 : bi;  // all -inf / NaN: the last index
  }
}

extern "C" int tp_argmax(const float* logits, int* out, int rows, int vocab, hipStream_t s) {
  TP_REQUIRE(rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, s, logits, out, vocab);
  TP_CHECK_LAUNCH("argmax");
  return 0;
}
