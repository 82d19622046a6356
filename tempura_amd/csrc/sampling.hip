// Picking the next token from float32 logits: argmax and (below) filtered sampling.
#include <math.h>

#include "common.h"
#include "no_alloc.h"

// ---- argmax -----------------------------------------------------------------------
// One block per row.  On exact ties the LAST maximum wins, as the reference's greedy
// rule does (/root/reference/engine/src/model.rs:459-473).  NaN never wins.
__device__ inline void argmax_merge(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i > bi)) {
    bv = v;
    bi = i;
  }
}

// Stage 1: grid (rows, chunks): each block scans its share of the row; stage 2 (chunks == 1 or the
// second launch) merges.  `part` holds (value, index) per (row, chunk).
__global__ void argmax_kernel(const float* __restrict__ logits, int vocab, int chunks, float* __restrict__ part_v,
                              int* __restrict__ part_i, int* __restrict__ out) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int rowi = blockIdx.x, chunk = blockIdx.y;
  const float* row = logits + (size_t)rowi * vocab;
  const int per = (vocab + chunks - 1) / chunks;
  const int lo = chunk * per, hi = min(vocab, lo + per);
  float bv = -INFINITY;
  int bi = -1;
  // four loads in flight per thread (the merge is a pure function of value and index, so the order is free)
  int j = lo + threadIdx.x;
  const int bd = blockDim.x;
  for (; j + 3 * bd < hi; j += 4 * bd) {
    const float v0 = row[j], v1 = row[j + bd], v2 = row[j + 2 * bd], v3 = row[j + 3 * bd];
    argmax_merge(bv, bi, v0, j);
    argmax_merge(bv, bi, v1, j + bd);
    argmax_merge(bv, bi, v2, j + 2 * bd);
    argmax_merge(bv, bi, v3, j + 3 * bd);
  }
  for (; j < hi; j += bd) argmax_merge(bv, bi, row[j], j);
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
    if (chunks == 1) {
      out[rowi] = bi < 0 ? vocab - 1 : bi;  // all -inf / NaN: the last index
    } else {
      part_v[rowi * chunks + chunk] = bv;
      part_i[rowi * chunks + chunk] = bi;
    }
  }
}

__global__ void argmax_merge_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int chunks,
                                    int vocab, int* __restrict__ out) {
  const int rowi = blockIdx.x;
  float bv = -INFINITY;
  int bi = -1;
  for (int c = threadIdx.x; c < chunks; c += TP_WAVE) argmax_merge(bv, bi, part_v[rowi * chunks + c], part_i[rowi * chunks + c]);
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, TP_WAVE);
    const int oi = __shfl_xor(bi, o, TP_WAVE);
    argmax_merge(bv, bi, ov, oi);
  }
  if (threadIdx.x == 0) out[rowi] = bi < 0 ? vocab - 1 : bi;
}

// `part` is scratch of rows * 64 floats followed by rows * 64 ints (may be null for small vocabularies).
extern "C" int tp_argmax(const float* logits, int* out, int rows, int vocab, void* part, hipStream_t s) {
  TP_REQUIRE(rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (rows == 0) return 0;
  int chunks = 1;
  if (part != nullptr && vocab >= 16384) chunks = min(64, max(1, 512 / rows));
  float* pv = (float*)part;
  int* pi = (int*)(pv + (size_t)rows * 64);
  hipLaunchKernelGGL(argmax_kernel, dim3(rows, chunks), dim3(chunks == 1 ? 1024 : 256), 0, s, logits, vocab, chunks, pv,
                     pi, out);
  if (chunks > 1) hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(TP_WAVE), 0, s, pv, pi, chunks, vocab, out);
  TP_CHECK_LAUNCH("argmax");
  return 0;
}

// ---- argmax without a workspace argument (see no_alloc.h) ---------------------------------
// The partial results live in a device array of the library itself.  In host code the array's name is only a
// stand-in for the symbol: its device address is looked up per device, and that pointer is what kernels get.
static __device__ __align__(256) unsigned char argmax_static_scratch[TP_ARGMAX_STATIC_MAX_ROWS * 64 * 8];
#define TP_MAX_DEVICES 64
static void* g_argmax_static_ptr[TP_MAX_DEVICES] = {};

extern "C" int tp_argmax_static_init(void) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TP_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  TP_REQUIRE(dev >= 0 && dev < TP_MAX_DEVICES, "argmax_static: device %d outside the table of %d", dev, TP_MAX_DEVICES);
  if (__atomic_load_n(&g_argmax_static_ptr[dev], __ATOMIC_ACQUIRE) != nullptr) return 0;
  void* ptr = nullptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(argmax_static_scratch));
  TP_REQUIRE(e == hipSuccess && ptr != nullptr, "argmax_static: hipGetSymbolAddress failed on device %d: %s", dev,
             hipGetErrorString(e));
  __atomic_store_n(&g_argmax_static_ptr[dev], ptr, __ATOMIC_RELEASE);   // (two threads racing here store the same address)
  return 0;
}

extern "C" int tp_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t s) {
  TP_REQUIRE(rows >= 0 && vocab > 0, "argmax_static: bad sizes");
  TP_REQUIRE(rows <= TP_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows, the library's scratch array holds %d", rows,
             TP_ARGMAX_STATIC_MAX_ROWS);
  if (rows == 0) return 0;
  if (tp_argmax_static_init() != 0) return 1;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TP_REQUIRE(e == hipSuccess && dev >= 0 && dev < TP_MAX_DEVICES, "argmax_static: hipGetDevice failed");
  return tp_argmax(logits, out, rows, vocab, g_argmax_static_ptr[dev], s);
}

// ---- penalties ----------------------------------------------------------------------
// entries: (row, token, count, in_window).  Presence/frequency penalties subtract
// frequency * count + presence (/root/reference/kernel-api/src/lib.rs:292-308); the
// repetition penalty multiplies non-positive logits and divides positive ones
// (/root/reference/kernels/src/sampler_chain.rs:222-246).  The reference applies
// presence/frequency to the raw logits and the repetition penalty after the temperature;
// dividing by a positive temperature keeps signs, so applying it to the raw logits and
// scaling afterwards gives the same values.
__global__ void penalties_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ rows,
                                 const int* __restrict__ tokens, const int* __restrict__ counts,
                                 const int* __restrict__ in_window, const float* __restrict__ presence,
                                 const float* __restrict__ frequency, const float* __restrict__ repeat, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r = rows[i], tok = tokens[i];
  if (tok < 0 || tok >= vocab) return;
  float* p = logits + (size_t)r * vocab + tok;
  float v = *p;
  if (counts[i] > 0) v -= frequency[r] * (float)counts[i] + presence[r];
  if (in_window[i] && repeat[r] != 1.0f) v = (v <= 0.f) ? v * repeat[r] : v / repeat[r];
  *p = v;
}

extern "C" int tp_apply_penalties(float* logits, int vocab, const int* rows, const int* tokens, const int* counts,
                                  const int* in_window, const float* presence, const float* frequency,
                                  const float* repeat, int n, hipStream_t s) {
  TP_REQUIRE(n >= 0 && vocab > 0, "apply_penalties: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(penalties_kernel, dim3((n + 255) / 256), dim3(256), 0, s, logits, vocab, rows, tokens, counts,
                     in_window, presence, frequency, repeat, n);
  TP_CHECK_LAUNCH("apply_penalties");
  return 0;
}

// ---- filtered sampling ----------------------------------------------------------------
// One block of 1024 threads per row:
//   x = logit / temperature; drop x < max + ln(min_p); typical-p: keep the tokens whose information
//   -ln p lies closest to the entropy, up to a mass above typical_p
//   (/root/reference/kernels/src/sampler_chain.rs:87-141); keep the top_k largest; softmax;
//   keep the shortest prefix (by descending probability) whose mass reaches top_p;
//   renormalise; walk the survivors in INDEX order and return the first index whose
//   cumulative mass exceeds r (/root/reference/kernels/src/sampling.rs:229-333).
// There is no sort: the k-th largest value and the top-p cut are found by radix selection
// over the order-preserving integer image of the floats (4 passes of 8 bits), counting
// elements for top-k and probability mass for top-p.  Mass is summed as 40-bit fixed point
// integers, so every sum is exact and independent of the order of additions: the same row,
// parameters and r always give the same token.  Ties at a cut are admitted in index order.
// temperature == 0 returns the argmax (last maximum wins).
#define SMP_THREADS 1024
#define SMP_WAVES (SMP_THREADS / TP_WAVE)
#define SMP_FIX 1099511627776.0f  // 2^40

__device__ inline unsigned int float_key(float f) {
  const unsigned int u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ inline unsigned long long fix_mass(float x, float maxv) {
  const float d = x - maxv;
  if (d < -27.8f) return 0ull;   // exp(d) * 2^40 < 1 truncates to 0 anyway: the far tail costs no exponential
  return (unsigned long long)(expf(d) * SMP_FIX);
}

// Exclusive prefix sum over the block in thread order; *total gets the block's sum.
__device__ inline unsigned long long block_excl_scan(unsigned long long v, unsigned long long* lds,
                                                     unsigned long long* total) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  unsigned long long inc = v;
#pragma unroll
  for (int o = 1; o < TP_WAVE; o <<= 1) {
    const unsigned long long t = __shfl_up(inc, o, TP_WAVE);
    if (lane >= o) inc += t;
  }
  __syncthreads();
  if (lane == TP_WAVE - 1) lds[wave] = inc;
  __syncthreads();
  unsigned long long base = 0, tot = 0;
  for (int i = 0; i < SMP_WAVES; ++i) {
    const unsigned long long w = lds[i];
    if (i < wave) base += w;
    tot += w;
  }
  *total = tot;
  return base + inc - v;
}

// The key that elements are selected by, largest first: the value itself, or (TYP) how close the element's
// information -ln p is to the entropy H, closest first.  With d = v - max and p = exp(d) / Z:
// -ln p - H = ln Z - d - (ln Z - sum p d) = mean_d - d, the distance of d from its mean under p.
template <bool TYP>
__device__ inline unsigned int select_key(float v, float maxv, float mean_d) {
  if (TYP) return ~float_key(fabsf(mean_d - (v - maxv)));
  return float_key(v);
}

// Radix selection from the top: finds the key K such that weight(key > K) < target <=
// weight(key >= K), where an element's weight is 1 (MASS = false) or its fixed-point mass.
// Only elements whose VALUE key is >= floor_key take part.  Returns K; *gt = weight(key > K),
// *eq_count = number of elements with key == K.
// After the first pass the elements of the chosen bin are copied to `cand` (LDS, SMP_CAND entries) when they fit,
// and the other three passes run over those few instead of the whole row: the k-th largest of 128,256 logits
// shares its first byte (sign and seven exponent bits) with a few thousand others at most.
// Logits crowd into a few bins of the first pass (one binade, one bin), and additions to one LDS address from the lanes
// of a wave go one after the other: every bin therefore has SMP_REP counters side by side, a lane adds to the one of
// its number, and the copies are summed when the pass is over (8 copies, a row of 128,256 logits, timed from the host: top-k 50
// 182 -> 143 us, top-p 0.9 256 -> 199 us, typical-p 623 -> 465 us).
#define SMP_CAND 4096
// f(value) for every element of x[0, n), the block's threads striding over it.  Sixteen loads of a thread are in
// flight at a time: one CU walks a row of 128,256 floats, and with four in flight each walk was a chain of 31 trips
// to memory per thread (about 25 us; a row's top-k sampling has four such walks).  For sums and counts that do not
// depend on the order.
template <typename F>
__device__ inline void walk_row(const float* __restrict__ x, int n, F f) {
  const int bd = blockDim.x;
  int j = threadIdx.x;
  for (; j + 15 * bd < n; j += 16 * bd) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = x[j + u * bd];
#pragma unroll
    for (int u = 0; u < 16; ++u) f(v[u]);
  }
  for (; j + 3 * bd < n; j += 4 * bd) {
    const float v0 = x[j], v1 = x[j + bd], v2 = x[j + 2 * bd], v3 = x[j + 3 * bd];
    f(v0);
    f(v1);
    f(v2);
    f(v3);
  }
  for (; j < n; j += bd) f(x[j]);
}

// One wave looks, in index order over x[lo, hi), for the first element of positive mass whose running mass (from c on)
// exceeds t; every lane returns its index, or -1.  Sixteen groups of 64 elements are loaded before the first is looked
// at (one group at a time, each load waited for, took 60 us for a wave's 8,016 elements), and a group without mass is
// passed over without the prefix sum.
template <typename M>
__device__ inline int wave_find(const float* __restrict__ x, int lo, int hi, unsigned long long c, unsigned long long t,
                                M mass_of, int lane) {
  for (int j0 = lo; j0 < hi; j0 += 16 * TP_WAVE) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u * TP_WAVE + lane;
      v[u] = j < hi ? x[j] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u * TP_WAVE + lane;
      const unsigned long long q = j < hi ? mass_of(v[u]) : 0ull;
      if (__builtin_amdgcn_ballot_w64(q > 0) == 0) continue;
      unsigned long long inc = q;
#pragma unroll
      for (int o = 1; o < TP_WAVE; o <<= 1) {
        const unsigned long long up = __shfl_up(inc, o, TP_WAVE);
        if (lane >= o) inc += up;
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(q > 0 && c + inc > t);
      if (hit != 0) return j0 + u * TP_WAVE + (int)__builtin_ctzll(hit);   // (the first such lane: index order)
      c += __shfl(inc, TP_WAVE - 1, TP_WAVE);
    }
  }
  return -1;
}

#define SMP_REP 8
#define SMP_CHUNKS 32     // pieces of a row that the kernels of many blocks work on
template <bool MASS, bool TYP = false>
__device__ unsigned int radix_select(const float* __restrict__ x, int n, float maxv, unsigned int floor_key,
                                     unsigned long long target, unsigned long long* hist /*256 * SMP_REP*/,
                                     unsigned int* cnt /*256 * SMP_REP*/, unsigned long long* sh /*4*/, float* cand /*SMP_CAND*/,
                                     unsigned long long* gt_out, unsigned int* eq_count, float mean_d = 0.f,
                                     const unsigned int* __restrict__ pre_cnt = nullptr) {
  // pre_cnt (counting only, every finite element takes part): the first pass's counts by bin, SMP_CHUNKS pieces of
  // the row side by side [SMP_CHUNKS, 256], counted by the kernel of many blocks that scaled the row
  unsigned int prefix = 0;
  unsigned long long gt = 0;
  int n_cand = -1;          // >= 0: the passes run over cand[0 .. n_cand)
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    __syncthreads();
    for (int i = threadIdx.x; i < 256 * SMP_REP; i += blockDim.x) {
      hist[i] = 0;
      cnt[i] = 0;
    }
    __syncthreads();
    const bool counted = !MASS && !TYP && pass == 0 && pre_cnt != nullptr;
    if (counted) {
      for (int b = threadIdx.x; b < 256; b += blockDim.x) {
        unsigned int cs = 0;
        for (int c = 0; c < SMP_CHUNKS; ++c) cs += pre_cnt[c * 256 + b];
        cnt[b * SMP_REP] = cs;
      }
    }
    const unsigned int copy = threadIdx.x % SMP_REP;
    auto take = [&](float v) {
      if (float_key(v) < floor_key) return;
      const unsigned int key = select_key<TYP>(v, maxv, mean_d);
      if (pass > 0 && (key >> (shift + 8)) != prefix) return;
      const unsigned int slot = ((key >> shift) & 255u) * SMP_REP + copy;
      atomicAdd(&cnt[slot], 1u);
      if (MASS) atomicAdd(&hist[slot], fix_mass(v, maxv));   // (counting: the weight of a bin is its count)
    };
    if (counted) {
      // (nothing to walk)
    } else if (n_cand >= 0) {
      for (int j = threadIdx.x; j < n_cand; j += blockDim.x) take(cand[j]);
    } else {   // (counts and fixed-point masses do not depend on the order)
      walk_row(x, n, take);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < 256 && !counted; b += blockDim.x) {   // a bin's copies into its first (integers: any order)
      unsigned long long hs = 0;
      unsigned int cs = 0;
#pragma unroll
      for (int r = 0; r < SMP_REP; ++r) {
        hs += hist[b * SMP_REP + r];
        cs += cnt[b * SMP_REP + r];
      }
      hist[b * SMP_REP] = hs;
      cnt[b * SMP_REP] = cs;
    }
    __syncthreads();
    // The bin that holds the target, from the top: the first b in 255 .. 1 with weight(bins above b) + weight(b) >=
    // target, else bin 0.  One wave, four bins a lane, a prefix sum over the lanes (one thread walking the bins took
    // 3 to 6 us a pass).
    if (threadIdx.x < TP_WAVE) {
      const int lane = threadIdx.x;
      unsigned long long w[4], local = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int b = 255 - (4 * lane + i);
        w[i] = MASS ? hist[b * SMP_REP] : (unsigned long long)cnt[b * SMP_REP];
        local += w[i];
      }
      unsigned long long inc = local;
#pragma unroll
      for (int o = 1; o < TP_WAVE; o <<= 1) {
        const unsigned long long up = __shfl_up(inc, o, TP_WAVE);
        if (lane >= o) inc += up;
      }
      unsigned long long run = gt + inc - local;   // the weight above this lane's first bin
      int found = -1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int b = 255 - (4 * lane + i);
        if (found < 0 && b > 0) {
          if (run + w[i] >= target) found = b;
          else run += w[i];
        }
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(found >= 0);
      if (hit != 0) {
        if (lane == (int)__builtin_ctzll(hit)) {
          sh[0] = run;
          sh[1] = (unsigned long long)found;
          sh[2] = (unsigned long long)cnt[found * SMP_REP];
          sh[3] = 0;            // (the candidates' counter)
        }
      } else if (lane == TP_WAVE - 1) {   // bin 0: everything above it is in `run` (the lane's last bin is bin 0)
        sh[0] = run;
        sh[1] = 0;
        sh[2] = (unsigned long long)cnt[0];
        sh[3] = 0;
      }
    }
    __syncthreads();
    gt = sh[0];
    prefix = (prefix << 8) | (unsigned int)sh[1];
    if (n_cand < 0 && pass < 3 && sh[2] <= (unsigned long long)SMP_CAND) {
      // gather the chosen bin's elements (their order does not matter: counts and integer masses): after the first
      // pass, or after the first one whose bin is small enough (logits that are nearly equal, as a model of random
      // weights gives them, share their first byte)
      const unsigned int want = prefix;
      auto gather = [&](float v) {
        if (float_key(v) < floor_key) return;
        if ((select_key<TYP>(v, maxv, mean_d) >> shift) != want) return;
        const unsigned long long at = atomicAdd(&sh[3], 1ull);
        if (at < (unsigned long long)SMP_CAND) cand[at] = v;
      };
      walk_row(x, n, gather);
      __syncthreads();
      n_cand = (int)sh[3];   // (== sh[2], the bin's count)
    }
  }
  *gt_out = gt;
  *eq_count = (unsigned int)sh[2];
  return prefix;
}

// A pass over x[0, n) that gives every element the weight of the ties before it in index order and lets `decide`
// replace the element.  tie_weight(v): 0 for an element that is no tie, else its weight; decide(v, before): the
// new value, `before` being the weight of the ties before this element.  Every wave owns a contiguous part of the
// row (a multiple of 64 elements) and reads it 64 elements at a time, sixteen loads in flight: first the weight of
// its ties, then, from the sum of the parts before it, a prefix sum over the lanes of each group that has a tie.
// (Threads that each own a contiguous run of elements read 64 cache lines per load: 0.1 ms for a row of 128,256.)
template <typename TieW, typename Decide>
__device__ inline void edit_in_index_order(float* __restrict__ x, int n, unsigned long long* scan /*SMP_WAVES*/,
                                           TieW tie_weight, Decide decide) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  const int per_wave = ((n + SMP_WAVES - 1) / SMP_WAVES + TP_WAVE - 1) / TP_WAVE * TP_WAVE;
  const int wlo = min(n, wave * per_wave), whi = min(n, wlo + per_wave);
  unsigned long long mine = 0;
  for (int j0 = wlo; j0 < whi; j0 += 16 * TP_WAVE) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u * TP_WAVE + lane;
      v[u] = j < whi ? x[j] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (j0 + u * TP_WAVE + lane < whi) mine += tie_weight(v[u]);
  }
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, TP_WAVE);
  __syncthreads();
  if (lane == 0) scan[wave] = mine;
  __syncthreads();
  unsigned long long base = 0;
  for (int i = 0; i < wave; ++i) base += scan[i];
  for (int j0 = wlo; j0 < whi; j0 += 16 * TP_WAVE) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u * TP_WAVE + lane;
      v[u] = j < whi ? x[j] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u * TP_WAVE + lane;
      const unsigned long long w = j < whi ? tie_weight(v[u]) : 0ull;
      unsigned long long before = base;
      if (__builtin_amdgcn_ballot_w64(w > 0) != 0) {
        unsigned long long inc = w;
#pragma unroll
        for (int o = 1; o < TP_WAVE; o <<= 1) {
          const unsigned long long up = __shfl_up(inc, o, TP_WAVE);
          if (lane >= o) inc += up;
        }
        before = base + inc - w;
        base += __shfl(inc, TP_WAVE - 1, TP_WAVE);
      }
      if (j < whi) {
        const float nv = decide(v[u], before);
        if (__float_as_uint(nv) != __float_as_uint(v[u])) x[j] = nv;
      }
    }
  }
  __syncthreads();
}

// Keep only the first `quota` elements (index order) among those with key == K: the others become -inf.
__device__ void drop_surplus_ties(float* __restrict__ x, int n, unsigned int K, unsigned long long quota,
                                  unsigned long long* lds) {
  edit_in_index_order(
      x, n, lds, [&](float v) { return float_key(v) == K ? 1ull : 0ull; },
      [&](float v, unsigned long long before) { return (float_key(v) == K && before >= quota) ? -INFINITY : v; });
}

// The typical-p cut: survivors with a selection key above K stay, those below go; the ones at K stay in index
// order for as long as the mass before them is short of `need`.  Survivors without mass go as well (the
// reference only lists tokens of positive probability).
__device__ void typical_cut(float* __restrict__ x, int n, float maxv, unsigned int floor_key, float mean_d,
                            unsigned int K, unsigned long long need, unsigned long long* lds) {
  edit_in_index_order(
      x, n, lds,
      [&](float v) {
        return (float_key(v) >= floor_key && select_key<true>(v, maxv, mean_d) == K) ? fix_mass(v, maxv) : 0ull;
      },
      [&](float v, unsigned long long before) {
        if (float_key(v) < floor_key) return v;
        const unsigned int key = select_key<true>(v, maxv, mean_d);
        const bool keep = key > K || (key == K && before < need);
        return (!keep || fix_mass(v, maxv) == 0) ? -INFINITY : v;
      });
}

// ---- rows cut by a small top_k: selection on many CUs -------------------------------------------------------------
// The k largest of a row all belong to the k largest of their piece of the row.  So each of the SMP_CHUNKS blocks that
// scale a row also hands over the elements of its piece that are at least as large as the piece's k-th largest (value
// and index; ties included), and one block per row then works on those few thousand candidates alone: the k-th
// largest of them, ties at the cut in index order, min_p, top_p and the draw in index order, with the same fixed-point
// masses as sample_kernel, whose result it reproduces bit for bit.  A row that does not qualify (a large
// top_k, typical_p, a report of probabilities asked for, a piece with more than SMP_CCAP candidates, more than 256 ties
// at the cut) is left to sample_kernel (`done` 0).
// A row cut by top_p alone goes the same way with the SMP_KMAX largest of each piece: the candidates hold every element
// of the row that is at least as large as the largest of the pieces' thresholds, so when the prefix that top_p keeps
// (against the mass of the whole row, from sample_mass_kernel) ends above that, it is found among them exactly; when
// it reaches further down, as for a row of nearly equal logits, the row is left to sample_kernel.
#define SMP_KMAX 128        // largest top_k of this path
#define SMP_CCAP 160        // candidates a piece may hand over
#define SMP_PER_MAX 8192    // elements of a piece (vocabularies up to 262,144)

__device__ inline bool topp_fast_row(float T, int k, int vocab, float typ, float tp) {
  return T > 0.f && !(k > 0 && k < vocab) && !(typ < 1.0f) && tp < 1.0f && tp > 0.f && vocab > SMP_KMAX &&
         (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS <= SMP_PER_MAX;
}

__device__ inline bool topk_fast_row(float T, int k, int vocab, float typ) {
  return T > 0.f && k > 0 && k <= SMP_KMAX && k < vocab && !(typ < 1.0f) &&
         (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS <= SMP_PER_MAX;
}

__device__ inline float key_float(unsigned int key) {   // float_key's inverse
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// The target-th largest (counted from 1) of the keys that the threads of the block hold in registers, R each (0: no
// element there): radix selection from the top with 256 counters, as radix_select does for counts.  *gt: how many keys
// are larger, *eq: how many are equal.  With fewer than `target` keys the answer is 0 (nothing is cut).  Called by the
// whole block.
#define SMP_KBINS 256
template <int R>
__device__ inline unsigned int reg_kth_key(const unsigned int (&kreg)[R], unsigned int target, unsigned int* bins /*SMP_KBINS*/,
                                           unsigned int* sh /*4*/, unsigned int* gt_out, unsigned int* eq_out) {
  unsigned int prefix = 0, gt = 0;
  for (int i = threadIdx.x; i < SMP_KBINS; i += blockDim.x) bins[i] = 0;
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const unsigned int key = kreg[u];
      if (key != 0 && (pass == 0 || (key >> (shift + 8)) == prefix)) atomicAdd(&bins[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (threadIdx.x < TP_WAVE) {   // the first bin from the top with count(bins above) + count(bin) >= target, else bin 0
      const int lane = threadIdx.x;
      unsigned int w[4], local = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        w[i] = bins[255 - (4 * lane + i)];
        bins[255 - (4 * lane + i)] = 0;   // (clear for the next pass)
        local += w[i];
      }
      unsigned int inc = local;
#pragma unroll
      for (int o = 1; o < TP_WAVE; o <<= 1) {
        const unsigned int up = __shfl_up(inc, o, TP_WAVE);
        if (lane >= o) inc += up;
      }
      unsigned int run = gt + inc - local, wf = 0;
      int found = -1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int b = 255 - (4 * lane + i);
        if (found < 0 && b > 0) {
          if (run + w[i] >= target) {
            found = b;
            wf = w[i];
          } else {
            run += w[i];
          }
        }
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(found >= 0);
      if (hit != 0) {
        if (lane == (int)__builtin_ctzll(hit)) {
          sh[0] = run;
          sh[1] = (unsigned int)found;
          sh[2] = wf;
        }
      } else if (lane == TP_WAVE - 1) {
        sh[0] = run;
        sh[1] = 0;
        sh[2] = w[3];   // (bin 0)
      }
    }
    __syncthreads();   // (the next write to sh comes after the next pass's barrier)
    gt = sh[0];
    prefix = (prefix << 8) | sh[1];
  }
  *gt_out = gt;
  *eq_out = sh[2];
  return prefix;
}

// The same with a weight per key (0 where there is no element): the largest key K with weight(keys >= K) >= target,
// as radix_select<true> finds it.  *gt: the weight of the larger keys, *eq: how many keys are equal to K.
template <int R>
__device__ inline unsigned int reg_kth_mass(const unsigned int (&kreg)[R], const unsigned long long (&qreg)[R],
                                            unsigned long long target, unsigned long long* hist /*256*/,
                                            unsigned int* cnt /*256*/, unsigned long long* sh /*4*/,
                                            unsigned long long* gt_out, unsigned int* eq_out) {
  unsigned int prefix = 0;
  unsigned long long gt = 0;
  for (int i = threadIdx.x; i < 256; i += blockDim.x) {
    hist[i] = 0;
    cnt[i] = 0;
  }
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const unsigned int key = kreg[u];
      if (key != 0 && (pass == 0 || (key >> (shift + 8)) == prefix)) {
        atomicAdd(&cnt[(key >> shift) & 255u], 1u);
        atomicAdd(&hist[(key >> shift) & 255u], qreg[u]);
      }
    }
    __syncthreads();
    if (threadIdx.x < TP_WAVE) {
      const int lane = threadIdx.x;
      unsigned long long w[4], local = 0;
      unsigned int c[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        w[i] = hist[255 - (4 * lane + i)];
        c[i] = cnt[255 - (4 * lane + i)];
        hist[255 - (4 * lane + i)] = 0;   // (clear for the next pass)
        cnt[255 - (4 * lane + i)] = 0;
        local += w[i];
      }
      unsigned long long inc = local;
#pragma unroll
      for (int o = 1; o < TP_WAVE; o <<= 1) {
        const unsigned long long up = __shfl_up(inc, o, TP_WAVE);
        if (lane >= o) inc += up;
      }
      unsigned long long run = gt + inc - local;
      unsigned int cf = 0;
      int found = -1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int b = 255 - (4 * lane + i);
        if (found < 0 && b > 0) {
          if (run + w[i] >= target) {
            found = b;
            cf = c[i];
          } else {
            run += w[i];
          }
        }
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(found >= 0);
      if (hit != 0) {
        if (lane == (int)__builtin_ctzll(hit)) {
          sh[0] = run;
          sh[1] = (unsigned long long)found;
          sh[2] = cf;
        }
      } else if (lane == TP_WAVE - 1) {
        sh[0] = run;
        sh[1] = 0;
        sh[2] = c[3];   // (bin 0)
      }
    }
    __syncthreads();
    gt = sh[0];
    prefix = (prefix << 8) | (unsigned int)sh[1];
  }
  *gt_out = gt;
  *eq_out = (unsigned int)sh[2];
  return prefix;
}

// Step 1 of sample_kernel for a whole row on many CUs: x = logit / temperature (NaN -> -inf), written to `work`,
// and the maximum of each of SMP_CHUNKS pieces of the row to part_max[row, piece].  grid: (rows, SMP_CHUNKS).
template <int R>   // R * 256: the most elements of a piece whose row takes the way of a small top_k
__global__ __launch_bounds__(256) void sample_scale_kernel(const float* __restrict__ logits, float* __restrict__ work,
                                                           int vocab, const float* __restrict__ temperature,
                                                           float* __restrict__ part_max,
                                                           unsigned int* __restrict__ part_cnt,
                                                           const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                           const float* __restrict__ typical_p,
                                                           float* __restrict__ cand_val, int* __restrict__ cand_idx,
                                                           int* __restrict__ cand_cnt, unsigned int* __restrict__ cand_thr) {
  // part_cnt (may be null): how many finite elements of the piece fall into each of the 256 bins of radix_select's
  // first pass, [rows, SMP_CHUNKS, 256]
  // cand_* (may be null): the piece's candidates for a row cut by a small top_k or by top_p alone (see topk_fast_row,
  // topp_fast_row), [rows, SMP_CHUNKS, SMP_CCAP], their number [rows, SMP_CHUNKS] (more than SMP_CCAP: too many, none
  // usable) and the key from which on the piece has handed over everything [rows, SMP_CHUNKS]
  __shared__ float fscratch[32];
  __shared__ unsigned int bins[256 * 4];
  __shared__ float xs[R * 256];
  __shared__ unsigned int kbins[SMP_KBINS];
  __shared__ unsigned int ksh[4];
  __shared__ int n_out;
  static_assert(R * 256 <= SMP_PER_MAX, "sample_topk_kernel takes rows of pieces up to SMP_PER_MAX");
  const int row = blockIdx.x, chunk = blockIdx.y;
  const bool by_k = cand_cnt != nullptr && topk_fast_row(temperature[row], top_k[row], vocab, typical_p[row]);
  const bool by_p = cand_cnt != nullptr && !by_k &&
                    topp_fast_row(temperature[row], top_k[row], vocab, typical_p[row], top_p[row]);
  const bool local_topk = (by_k || by_p) && (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS <= R * 256;
  if (part_cnt != nullptr) {
    for (int i = threadIdx.x; i < 256 * 4; i += blockDim.x) bins[i] = 0;
    __syncthreads();
  }
  auto count = [&](float v) {
    if (part_cnt != nullptr && v > -INFINITY) atomicAdd(&bins[(float_key(v) >> 24) * 4 + (threadIdx.x & 3)], 1u);
  };
  const float* lg = logits + (size_t)row * vocab;
  float* x = work + (size_t)row * vocab;
  const float T = temperature[row] > 0.f ? temperature[row] : 1.0f;
  const int per = (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS;
  const int lo = min(vocab, chunk * per), hi = min(vocab, lo + per);
  auto scale = [&](float v) {
    if (T != 1.0f) v = v / T;
    if (!(v == v)) v = -INFINITY;  // NaN never survives
    return v;
  };
  float mx = -INFINITY;
  const int bd = blockDim.x;
  int j = lo + threadIdx.x;
  for (; j + 3 * bd < hi; j += 4 * bd) {
    const float v0 = scale(lg[j]), v1 = scale(lg[j + bd]), v2 = scale(lg[j + 2 * bd]), v3 = scale(lg[j + 3 * bd]);
    x[j] = v0;
    x[j + bd] = v1;
    x[j + 2 * bd] = v2;
    x[j + 3 * bd] = v3;
    mx = fmaxf(fmaxf(mx, v0), fmaxf(v1, fmaxf(v2, v3)));
    count(v0);
    count(v1);
    count(v2);
    count(v3);
    if (local_topk) {
      xs[j - lo] = v0;
      xs[j + bd - lo] = v1;
      xs[j + 2 * bd - lo] = v2;
      xs[j + 3 * bd - lo] = v3;
    }
  }
  for (; j < hi; j += bd) {
    const float v = scale(lg[j]);
    x[j] = v;
    mx = fmaxf(mx, v);
    count(v);
    if (local_topk) xs[j - lo] = v;
  }
  mx = block_max(mx, fscratch);
  if (threadIdx.x == 0) part_max[row * SMP_CHUNKS + chunk] = mx;
  if (local_topk) {   // (the same for every thread of the block; xs is whole after block_max's barriers)
    const int np = hi - lo;
    const unsigned int finite = float_key(-INFINITY) + 1u;
    unsigned int kreg[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int i = threadIdx.x + u * 256;
      kreg[u] = 0;
      if (i < np) {
        const unsigned int key = float_key(xs[i]);
        if (key >= finite) kreg[u] = key;
      }
    }
    if (threadIdx.x == 0) n_out = 0;
    unsigned int gt, eq;
    unsigned int K = reg_kth_key(kreg, by_k ? (unsigned int)top_k[row] : (unsigned int)SMP_KMAX, kbins, ksh, &gt,
                                 &eq);   // (barriers: n_out is set)
    if (K < finite) K = finite;
    const size_t base = ((size_t)row * SMP_CHUNKS + chunk) * SMP_CCAP;
#pragma unroll
    for (int u = 0; u < R; ++u) {
      if (kreg[u] >= K) {
        const int at = atomicAdd(&n_out, 1);
        if (at < SMP_CCAP) {
          cand_val[base + at] = key_float(kreg[u]);
          cand_idx[base + at] = lo + threadIdx.x + u * 256;
        }
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      cand_cnt[row * SMP_CHUNKS + chunk] = n_out;
      cand_thr[row * SMP_CHUNKS + chunk] = K;
    }
  }
  if (part_cnt != nullptr) {
    __syncthreads();
    for (int b = threadIdx.x; b < 256; b += blockDim.x)
      part_cnt[((size_t)row * SMP_CHUNKS + chunk) * 256 + b] = bins[b * 4] + bins[b * 4 + 1] + bins[b * 4 + 2] + bins[b * 4 + 3];
  }
}

// For rows that are only scaled (and perhaps cut by min_p) before the draw: the fixed-point mass of each of the
// SMP_CHUNKS pieces, part_mass[row, piece], against the row's maximum from sample_scale_kernel.  The draw then
// looks at one piece only.  grid: (rows, SMP_CHUNKS).
__global__ __launch_bounds__(256) void sample_mass_kernel(const float* __restrict__ work, int vocab,
                                                          const float* __restrict__ min_p,
                                                          const float* __restrict__ part_max,
                                                          unsigned long long* __restrict__ part_mass) {
  __shared__ unsigned long long wsum[4];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float* x = work + (size_t)row * vocab;
  float maxv = part_max[row * SMP_CHUNKS];
  for (int i = 1; i < SMP_CHUNKS; ++i) maxv = fmaxf(maxv, part_max[row * SMP_CHUNKS + i]);
  unsigned int floor_key = float_key(-INFINITY) + 1u;
  const float mp = min_p[row];
  if (mp > 0.f && maxv != -INFINITY) {
    const unsigned int k2 = float_key(maxv + logf(mp));
    if (k2 > floor_key) floor_key = k2;
  }
  const int per = (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS;
  const int lo = min(vocab, chunk * per), hi = min(vocab, lo + per);
  auto mass = [&](int j) {
    if (j >= hi) return 0ull;
    const float v = x[j];
    return float_key(v) >= floor_key ? fix_mass(v, maxv) : 0ull;
  };
  unsigned long long mine = 0;
  const int bd = blockDim.x;
  for (int j = lo + threadIdx.x; j < hi; j += 4 * bd) mine += mass(j) + mass(j + bd) + mass(j + 2 * bd) + mass(j + 3 * bd);
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, TP_WAVE);
  if (threadIdx.x % TP_WAVE == 0) wsum[threadIdx.x / TP_WAVE] = mine;
  __syncthreads();
  if (threadIdx.x == 0) part_mass[row * SMP_CHUNKS + chunk] = wsum[0] + wsum[1] + wsum[2] + wsum[3];
}

// The candidates of a row cut by a small top_k (see above) -> its token.  grid: rows; done[row] = 1 when the row is
// settled here, 0 when sample_kernel has to do it.
#define SMP_TOPK_R (SMP_CHUNKS * SMP_CCAP / 256)
__global__ __launch_bounds__(256) void sample_topk_kernel(const float* __restrict__ cand_val, const int* __restrict__ cand_idx,
                                                          const int* __restrict__ cand_cnt,
                                                          const unsigned int* __restrict__ cand_thr,
                                                          const float* __restrict__ part_max,
                                                          const unsigned long long* __restrict__ part_mass,
                                                          int vocab, const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                          const float* __restrict__ min_p, const float* __restrict__ typical_p,
                                                          const float* __restrict__ rnd, int* __restrict__ out,
                                                          int* __restrict__ done) {
  static_assert(SMP_CHUNKS * SMP_CCAP % 256 == 0, "the candidates are spread evenly over the threads");
  __shared__ int cnts[SMP_CHUNKS];
  __shared__ unsigned int bins[SMP_KBINS];
  __shared__ unsigned int sh[4];
  __shared__ int tl[256];                          // indices of the ties at the cut
  __shared__ unsigned long long sord[SMP_KMAX];    // survivors: key and index as one number that orders them
  __shared__ int si[SMP_KMAX];
  __shared__ unsigned long long sq[SMP_KMAX];      // ... and their masses (0: dropped)
  __shared__ unsigned long long hist[256], sh64[4], pm[SMP_CHUNKS], pl_q[SMP_CCAP], s_Z;   // (rows cut by top_p alone)
  __shared__ int pl_idx[SMP_CCAP];
  __shared__ int s_n, n_tie, s_over, n_pl;
  __shared__ unsigned int s_thr;
  __shared__ float s_max;
  const int row = blockIdx.x, tid = threadIdx.x;
  if (tid == 0) done[row] = 0;
  const int k = top_k[row];
  const bool by_k = topk_fast_row(temperature[row], k, vocab, typical_p[row]);
  const bool by_p = !by_k && part_mass != nullptr && topp_fast_row(temperature[row], k, vocab, typical_p[row], top_p[row]);
  if (!by_k && !by_p) return;
  if (tid < TP_WAVE) {   // how many candidates each piece brings, and the row's maximum
    const int c = tid < SMP_CHUNKS ? cand_cnt[row * SMP_CHUNKS + tid] : 0;
    float mx = tid < SMP_CHUNKS ? part_max[row * SMP_CHUNKS + tid] : -INFINITY;
    unsigned int thr = tid < SMP_CHUNKS ? cand_thr[row * SMP_CHUNKS + tid] : 0u;
    unsigned long long z = (by_p && tid < SMP_CHUNKS) ? part_mass[row * SMP_CHUNKS + tid] : 0ull;
    const bool over = __builtin_amdgcn_ballot_w64(c > SMP_CCAP) != 0;
#pragma unroll
    for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
      mx = fmaxf(mx, __shfl_xor(mx, o, TP_WAVE));
      thr = max(thr, (unsigned int)__shfl_xor((int)thr, o, TP_WAVE));
      z += __shfl_xor(z, o, TP_WAVE);
    }
    if (tid < SMP_CHUNKS) {
      cnts[tid] = c;
      pm[tid] = 0;
    }
    if (tid == 0) {
      s_n = 0;
      n_tie = 0;
      n_pl = 0;
      s_over = over;
      s_max = mx;
      s_thr = thr;
      s_Z = z;
    }
  }
  __syncthreads();
  if (s_over) return;   // some piece had more candidates than it could hand over
  const float maxv = s_max;
  if (maxv == -INFINITY) {   // nothing to choose from: the last index, as sample_kernel answers
    if (tid == 0) {
      out[row] = vocab - 1;
      done[row] = 1;
    }
    return;
  }
  unsigned int floor_key = float_key(-INFINITY) + 1u;
  const float mp = min_p[row];
  if (mp > 0.f) {
    const unsigned int k2 = float_key(maxv + logf(mp));
    if (k2 > floor_key) floor_key = k2;
  }
  // every thread takes its share of the candidates' slots into registers (a slot beyond its piece's count: no element)
  unsigned int kreg[SMP_TOPK_R];
  int ireg[SMP_TOPK_R];
  {
    const size_t base = (size_t)row * SMP_CHUNKS * SMP_CCAP;
    float v[SMP_TOPK_R];
#pragma unroll
    for (int u = 0; u < SMP_TOPK_R; ++u) {
      v[u] = cand_val[base + tid + u * 256];
      ireg[u] = cand_idx[base + tid + u * 256];
    }
#pragma unroll
    for (int u = 0; u < SMP_TOPK_R; ++u) {
      const int e = tid + u * 256, p = e / SMP_CCAP, i = e - p * SMP_CCAP;
      const unsigned int key = float_key(v[u]);
      kreg[u] = (i < cnts[p] && key >= floor_key) ? key : 0u;
    }
  }
  if (by_p) {
    // top_p alone: the prefix by descending value whose mass reaches top_p of the whole row's, then the draw
    const unsigned long long Zrow = s_Z;
    if (Zrow == 0) {   // nothing to draw from: the last index
      if (tid == 0) {
        out[row] = vocab - 1;
        done[row] = 1;
      }
      return;
    }
    unsigned long long qreg[SMP_TOPK_R];
#pragma unroll
    for (int u = 0; u < SMP_TOPK_R; ++u) qreg[u] = kreg[u] != 0 ? fix_mass(key_float(kreg[u]), maxv) : 0ull;
    unsigned long long target = (unsigned long long)((double)top_p[row] * (double)Zrow);
    if (target < 1) target = 1;
    {   // all candidates together short of the target (a row of nearly equal logits): left to sample_kernel at once
      unsigned long long mine = 0;
#pragma unroll
      for (int u = 0; u < SMP_TOPK_R; ++u) mine += qreg[u];
#pragma unroll
      for (int o = TP_WAVE / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, TP_WAVE);
      if (tid % TP_WAVE == 0) sh64[tid / TP_WAVE] = mine;
      __syncthreads();
      const unsigned long long all = sh64[0] + sh64[1] + sh64[2] + sh64[3];
      __syncthreads();   // (sh64 is used again by the selection)
      if (all < target) return;
    }
    unsigned long long gtm;
    unsigned int eqn;
    const unsigned int K2 = reg_kth_mass(kreg, qreg, target, hist, bins, sh64, &gtm, &eqn);
    const unsigned long long q = fix_mass(key_float(K2), maxv);
    // the candidates are all of the row from s_thr upwards: a prefix that ends there is the row's
    if (K2 < s_thr || K2 < floor_key || gtm + (unsigned long long)eqn * q < target) return;
    unsigned long long need = 1;
    if (q > 0 && target > gtm) need = (target - gtm + q - 1) / q;
    if (need < 1) need = 1;
    const bool cut_ties = (unsigned long long)eqn > need;   // each tie has the mass q: as many as the target still needs
    if (cut_ties && eqn > 256u) return;
    if (cut_ties) {
#pragma unroll
      for (int u = 0; u < SMP_TOPK_R; ++u) {
        if (kreg[u] == K2) {
          const int at = atomicAdd(&n_tie, 1);
          if (at < 256) tl[at] = ireg[u];
        }
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < SMP_TOPK_R; ++u) {
        if (kreg[u] == K2) {
          unsigned long long rank = 0;
          for (int j = 0; j < (int)eqn; ++j) rank += tl[j] < ireg[u];
          if (rank >= need) kreg[u] = 0;
        }
      }
    }
    // the survivors' mass piece by piece, the piece that holds the draw, and the survivor there
#pragma unroll
    for (int u = 0; u < SMP_TOPK_R; ++u)
      if (kreg[u] != 0 && kreg[u] >= K2 && qreg[u] != 0) atomicAdd(&pm[(tid + u * 256) / SMP_CCAP], qreg[u]);
    __syncthreads();
    unsigned long long Z = 0;
    for (int i = 0; i < SMP_CHUNKS; ++i) Z += pm[i];
    if (Z == 0) {
      if (tid == 0) {
        out[row] = vocab - 1;
        done[row] = 1;
      }
      return;
    }
    unsigned long long t = (unsigned long long)((double)rnd[row] * (double)Z);
    if (t >= Z) t = Z - 1;
    unsigned long long c = 0;
    int piece = 0;
    for (; piece < SMP_CHUNKS - 1; ++piece) {
      if (t < c + pm[piece]) break;
      c += pm[piece];
    }
#pragma unroll
    for (int u = 0; u < SMP_TOPK_R; ++u) {
      if ((tid + u * 256) / SMP_CCAP == piece && kreg[u] != 0 && kreg[u] >= K2 && qreg[u] != 0) {
        const int at = atomicAdd(&n_pl, 1);   // (a piece brings at most SMP_CCAP)
        pl_idx[at] = ireg[u];
        pl_q[at] = qreg[u];
      }
    }
    __syncthreads();
    if (tid < n_pl) {
      const int mine = pl_idx[tid];
      unsigned long long before = c;
      for (int j = 0; j < n_pl; ++j) before += pl_idx[j] < mine ? pl_q[j] : 0ull;
      if (before <= t && t < before + pl_q[tid]) {
        out[row] = mine;
        done[row] = 1;
      }
    }
    return;
  }
  unsigned int gt, eq;
  const unsigned int K = reg_kth_key(kreg, (unsigned int)k, bins, sh, &gt, &eq);
  // ties at the cut are admitted in index order, as many as k still allows
  const bool cut_ties = gt + eq > (unsigned int)k;
  const unsigned int quota = cut_ties ? (unsigned int)k - gt : eq;
  if (cut_ties && eq > 256u) return;
  auto keep = [&](unsigned int key, int idx) {
    const int at = atomicAdd(&s_n, 1);
    if (at < SMP_KMAX) {   // (at most k by construction)
      sord[at] = ((unsigned long long)key << 32) | (unsigned long long)(0xffffffffu - (unsigned int)idx);
      si[at] = idx;
    }
  };
#pragma unroll
  for (int u = 0; u < SMP_TOPK_R; ++u) {
    const unsigned int key = kreg[u];
    if (key == 0 || key < K) continue;
    if (key > K || !cut_ties) {
      keep(key, ireg[u]);
    } else {
      const int at = atomicAdd(&n_tie, 1);
      if (at < 256) tl[at] = ireg[u];
    }
  }
  __syncthreads();
  if (cut_ties) {
    if (tid < (int)eq) {
      const int mine = tl[tid];
      unsigned int rank = 0;
      for (int j = 0; j < (int)eq; ++j) rank += tl[j] < mine;
      if (rank < quota) keep(K, mine);
    }
    __syncthreads();
  }
  const int S = min(s_n, SMP_KMAX);
  if (tid < SMP_KMAX) sq[tid] = tid < S ? fix_mass(key_float((unsigned int)(sord[tid] >> 32)), maxv) : 0ull;
  __syncthreads();
  // top_p: the survivors in descending order (ties by index) while the mass before one is short of the target
  const float tp = top_p[row];
  if (tp < 1.0f && tp > 0.f) {
    unsigned long long Z = 0;
#pragma unroll 8
    for (int j = 0; j < S; ++j) Z += sq[j];
    unsigned long long target = (unsigned long long)((double)tp * (double)Z);
    if (target < 1) target = 1;
    bool drop = false;
    if (tid < S) {
      const unsigned long long mine = sord[tid];
      unsigned long long before = 0;
#pragma unroll 8
      for (int j = 0; j < S; ++j) before += sord[j] > mine ? sq[j] : 0ull;
      drop = before >= target;
    }
    __syncthreads();
    if (drop) sq[tid] = 0;
    __syncthreads();
  }
  // the draw: the first survivor in index order whose cumulative mass exceeds r * Z
  unsigned long long Z = 0, before = 0;
  const int mine = tid < S ? si[tid] : 0;
#pragma unroll 8
  for (int j = 0; j < S; ++j) {
    const unsigned long long q = sq[j];
    Z += q;
    before += si[j] < mine ? q : 0ull;
  }
  if (Z == 0) {   // nothing left to draw from: the last index
    if (tid == 0) {
      out[row] = vocab - 1;
      done[row] = 1;
    }
    return;
  }
  unsigned long long t = (unsigned long long)((double)rnd[row] * (double)Z);
  if (t >= Z) t = Z - 1;
  if (tid < S && before <= t && t < before + sq[tid]) {
    out[row] = mine;
    done[row] = 1;
  }
}

// The fixed-point mass of the survivors (key >= floor_key) in x[lo, hi), wave by wave: every wave of the block owns
// a contiguous part of the range (a multiple of 64 elements) and sums it with coalesced loads, sixteen in flight;
// scan[w] receives wave w's sum.  Returns the range's total; *wlo, *whi: this wave's part.  Called by the whole block.
__device__ inline unsigned long long range_mass_by_wave(const float* __restrict__ x, int lo, int hi, unsigned int floor_key,
                                                        float maxv, unsigned long long* scan /*SMP_WAVES*/, int* wlo_out,
                                                        int* whi_out) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  const int per_wave = ((hi - lo + SMP_WAVES - 1) / SMP_WAVES + TP_WAVE - 1) / TP_WAVE * TP_WAVE;
  const int wlo = min(hi, lo + wave * per_wave), whi = min(hi, wlo + per_wave);
  unsigned long long mine = 0;
  int j = wlo + lane;
  for (; j + 15 * TP_WAVE < whi; j += 16 * TP_WAVE) {   // sixteen loads in flight (see walk_row)
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = x[j + u * TP_WAVE];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (float_key(v[u]) >= floor_key) mine += fix_mass(v[u], maxv);
  }
  for (; j < whi; j += TP_WAVE) {
    const float v = x[j];
    if (float_key(v) >= floor_key) mine += fix_mass(v, maxv);
  }
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, TP_WAVE);
  __syncthreads();
  if (lane == 0) scan[wave] = mine;
  __syncthreads();
  unsigned long long total = 0;
  for (int i = 0; i < SMP_WAVES; ++i) total += scan[i];
  *wlo_out = wlo;
  *whi_out = whi;
  return total;
}

// After range_mass_by_wave: the first index of the range, in index order, at which the cumulative mass, counted
// from `base` before the range, exceeds t.  The wave whose part holds it walks that part 64 elements at a time;
// its lane 0 gets the index, every other thread -1.
__device__ inline int range_find_by_wave(const float* __restrict__ x, int wlo, int whi, unsigned long long base,
                                         unsigned long long t, unsigned int floor_key, float maxv,
                                         const unsigned long long* scan) {
  const int lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  unsigned long long before = base, mine_base = 0;
  int chosen_wave = -1;
  for (int i = 0; i < SMP_WAVES; ++i) {
    const unsigned long long w = scan[i];
    if (chosen_wave < 0 && t < before + w) {
      chosen_wave = i;
      mine_base = before;
    }
    before += w;
  }
  if (wave != chosen_wave) return -1;
  const int at = wave_find(x, wlo, whi, mine_base, t,
                           [&](float v) { return float_key(v) >= floor_key ? fix_mass(v, maxv) : 0ull; }, lane);
  return lane == 0 ? at : -1;
}

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(
    const float* __restrict__ logits, float* __restrict__ work, int vocab, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
    const float* __restrict__ typical_p, const float* __restrict__ rnd, int* __restrict__ out,
    float* __restrict__ info, const float* __restrict__ part_max, const unsigned long long* __restrict__ part_mass,
    const unsigned int* __restrict__ part_cnt, const int* __restrict__ done) {
  __shared__ unsigned long long hist[256 * SMP_REP];
  __shared__ unsigned int cnt[256 * SMP_REP];
  __shared__ unsigned long long sh[4];
  __shared__ float cand[SMP_CAND];
  __shared__ unsigned long long scan[SMP_WAVES];
  __shared__ float fscratch[32];
  __shared__ int ibest[SMP_WAVES];
  __shared__ float vbest[SMP_WAVES];
  const int row = blockIdx.x;
  if (done != nullptr && done[row]) return;   // settled by sample_topk_kernel
  const float* lg = logits + (size_t)row * vocab;
  float* x = work + (size_t)row * vocab;
  const bool greedy = !(temperature[row] > 0.f);
  const float T = greedy ? 1.0f : temperature[row];   // a greedy row that reports probabilities filters unscaled logits
  float* inf = info == nullptr ? nullptr : info + 4 * row;

  if (greedy) {  // argmax, last maximum wins
    float bv = -INFINITY;
    int bi = -1;
    for (int j = threadIdx.x; j < vocab; j += blockDim.x) argmax_merge(bv, bi, lg[j], j);
    for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, TP_WAVE);
      const int oi = __shfl_xor(bi, o, TP_WAVE);
      argmax_merge(bv, bi, ov, oi);
    }
    if (threadIdx.x % TP_WAVE == 0) {
      vbest[threadIdx.x / TP_WAVE] = bv;
      ibest[threadIdx.x / TP_WAVE] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int i = 1; i < SMP_WAVES; ++i) argmax_merge(bv, bi, vbest[i], ibest[i]);
      out[row] = bi < 0 ? vocab - 1 : bi;
      ibest[0] = bi < 0 ? vocab - 1 : bi;
    }
    if (inf == nullptr) return;
    __syncthreads();
  }
  const int greedy_pick = greedy ? ibest[0] : -1;
  __syncthreads();

  // 1. scale by the temperature, find the maximum
  float mx = -INFINITY;
  if (part_max != nullptr) {   // sample_scale_kernel did this step on many CUs
    if (threadIdx.x < SMP_CHUNKS) mx = part_max[row * SMP_CHUNKS + threadIdx.x];
  } else {
    auto scale = [&](float v) {
      if (T != 1.0f) v = v / T;
      if (!(v == v)) v = -INFINITY;  // NaN never survives
      return v;
    };
    const int bd = blockDim.x;
    int j = threadIdx.x;
    for (; j + 3 * bd < vocab; j += 4 * bd) {   // four loads in flight per thread
      const float v0 = scale(lg[j]), v1 = scale(lg[j + bd]), v2 = scale(lg[j + 2 * bd]), v3 = scale(lg[j + 3 * bd]);
      x[j] = v0;
      x[j + bd] = v1;
      x[j + 2 * bd] = v2;
      x[j + 3 * bd] = v3;
      mx = fmaxf(fmaxf(mx, v0), fmaxf(v1, fmaxf(v2, v3)));
    }
    for (; j < vocab; j += bd) {
      const float v = scale(lg[j]);
      x[j] = v;
      mx = fmaxf(mx, v);
    }
  }
  const float maxv = block_max(mx, fscratch);
  __syncthreads();
  if (maxv == -INFINITY) {  // nothing to choose from: the reference falls through to the last index
    if (threadIdx.x == 0) {
      if (!greedy) out[row] = vocab - 1;
      if (inf != nullptr) {
        inf[0] = 0.f;
        inf[1] = 0.f;
        inf[2] = INFINITY;      // no survivor
        inf[3] = -INFINITY;
      }
    }
    return;
  }

  // 2. min_p: drop x < max + ln(min_p)
  unsigned int floor_key = float_key(-INFINITY) + 1u;  // everything finite
  const float mp = min_p[row];
  if (mp > 0.f) {
    const float thr = maxv + logf(mp);
    const unsigned int k2 = float_key(thr);
    if (k2 > floor_key) floor_key = k2;
  }

  // The short way for a row that is only scaled (and cut by min_p): the masses of its pieces are there already
  // (sample_mass_kernel, same maximum and floor), so the draw finds its piece and walks that one alone.
  {
    const int k0 = top_k[row];
    const float tp0 = top_p[row];
    if (part_mass != nullptr && !greedy && inf == nullptr && !(typical_p[row] < 1.0f) && !(k0 > 0 && k0 < vocab) &&
        !(tp0 < 1.0f && tp0 > 0.f)) {
      const unsigned long long* pm = part_mass + (size_t)row * SMP_CHUNKS;
      unsigned long long Z = 0;
      for (int i = 0; i < SMP_CHUNKS; ++i) Z += pm[i];
      if (Z == 0) {
        if (threadIdx.x == 0) out[row] = vocab - 1;
        return;
      }
      unsigned long long t = (unsigned long long)((double)rnd[row] * (double)Z);
      if (t >= Z) t = Z - 1;
      unsigned long long c = 0;
      int piece = 0;
      for (; piece < SMP_CHUNKS - 1; ++piece) {
        if (t < c + pm[piece]) break;
        c += pm[piece];
      }
      // the piece's mass wave by wave, then one wave walks its sixteenth of the piece, 64 elements at a time
      const int per = (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS;
      const int lo = min(vocab, piece * per), hi = min(vocab, lo + per);
      int wlo, whi;
      range_mass_by_wave(x, lo, hi, floor_key, maxv, scan, &wlo, &whi);
      const int at = range_find_by_wave(x, wlo, whi, c, t, floor_key, maxv, scan);
      if (at >= 0) out[row] = at;
      return;
    }
  }

  // 2b. typical_p: the survivors nearest the entropy, nearest first, until their mass exceeds typical_p
  const float typ = typical_p[row];
  if (typ < 1.0f) {
    unsigned long long part = 0;
    float s1 = 0.f;
    walk_row(x, vocab, [&](float v) {   // (a thread adds its elements in the order of their indices)
      if (float_key(v) >= floor_key) {
        part += fix_mass(v, maxv);
        s1 += expf(v - maxv) * (v - maxv);
      }
    });
    unsigned long long Z0;
    block_excl_scan(part, scan, &Z0);
    const float mean_d = block_sum(s1, fscratch) / ((float)Z0 * (1.0f / SMP_FIX));
    unsigned long long target = (unsigned long long)((double)fmaxf(typ, 0.f) * (double)Z0) + 1;   // mass > typical_p
    if (target > Z0) target = Z0;
    unsigned long long gt;
    unsigned int eq;
    const unsigned int K = radix_select<true, true>(x, vocab, maxv, floor_key, target, hist, cnt, sh, cand, &gt, &eq, mean_d);
    typical_cut(x, vocab, maxv, floor_key, mean_d, K, target - gt, scan);
  }

  // 3. top_k: the k-th largest value among the survivors
  const int k = top_k[row];
  if (k > 0 && k < vocab) {
    unsigned long long gt;
    unsigned int eq;
    // (the first pass is counted already when nothing has been cut from the row so far)
    const bool whole = part_cnt != nullptr && part_max != nullptr && !(mp > 0.f) && !(typ < 1.0f);
    const unsigned int K = radix_select<false>(x, vocab, maxv, floor_key, (unsigned long long)k, hist, cnt, sh, cand, &gt, &eq,
                                               0.f, whole ? part_cnt + (size_t)row * SMP_CHUNKS * 256 : nullptr);
    // fewer than k survivors: K lands on the smallest surviving bin and nothing is cut
    if (gt + eq > (unsigned long long)k) drop_surplus_ties(x, vocab, K, (unsigned long long)k - gt, scan);
    if (K > floor_key) floor_key = K;
  }

  // 4. total mass of the survivors (left to the draw, which sums the same masses wave by wave, when nothing
  // needs it earlier: no top_p and no report)
  const float tp = top_p[row];
  const bool need_mass_now = (tp < 1.0f && tp > 0.f) || inf != nullptr || greedy;
  // (known already when sample_mass_kernel summed the pieces and nothing has been cut since: a row cut by top_p
  // alone that could not be settled from the candidates of its pieces)
  const bool mass_known = part_mass != nullptr && !(typ < 1.0f) && !(k > 0 && k < vocab);
  unsigned long long part = 0;
  if (need_mass_now && !mass_known) {
    walk_row(x, vocab, [&](float v) {   // (integer sums, any order)
      if (float_key(v) >= floor_key) part += fix_mass(v, maxv);
    });
  }
  unsigned long long Z = 0;
  if (need_mass_now && mass_known) {
    for (int i = 0; i < SMP_CHUNKS; ++i) Z += part_mass[(size_t)row * SMP_CHUNKS + i];
  } else if (need_mass_now) {
    block_excl_scan(part, scan, &Z);
  }

  // 5. top_p: the shortest prefix by descending probability whose mass reaches top_p
  if (tp < 1.0f && tp > 0.f) {
    unsigned long long target = (unsigned long long)((double)tp * (double)Z);
    if (target < 1) target = 1;
    unsigned long long gt;
    unsigned int eq;
    const unsigned int K = radix_select<true>(x, vocab, maxv, floor_key, target, hist, cnt, sh, cand, &gt, &eq);
    // each tie at K has the same mass q; take as many as the target still needs
    float kv;
    {
      const unsigned int u = (K & 0x80000000u) ? (K & 0x7fffffffu) : ~K;
      kv = __uint_as_float(u);
    }
    const unsigned long long q = fix_mass(kv, maxv);
    unsigned long long need = 1;
    if (q > 0 && target > gt) need = (target - gt + q - 1) / q;
    if (need < 1) need = 1;
    if ((unsigned long long)eq > need) drop_surplus_ties(x, vocab, K, need, scan);
    if (K > floor_key) floor_key = K;
    Z = gt + (need < (unsigned long long)eq ? need : (unsigned long long)eq) * q;
  }

  // what a caller needs for log-probabilities of the final distribution: ln p(v) = (v - max) - ln Z for v >= floor
  const float lnZ = logf((float)((double)Z * (1.0 / (double)SMP_FIX)));
  if (inf != nullptr && threadIdx.x == 0) {
    const unsigned int u = (floor_key & 0x80000000u) ? (floor_key & 0x7fffffffu) : ~floor_key;
    inf[0] = maxv;
    inf[1] = lnZ;
    inf[2] = __uint_as_float(u);
    if (greedy) {
      const float v = x[greedy_pick];
      inf[3] = (Z > 0 && float_key(v) >= floor_key) ? (v - maxv) - lnZ : -INFINITY;
    } else if (Z == 0) {
      inf[3] = -INFINITY;
    }
  }
  if (greedy) return;

  // 6. draw: first index (index order) whose cumulative mass exceeds r * Z
  // Every wave owns a contiguous range of the row and sums its mass with coalesced loads; the wave whose range
  // holds the target then walks it 64 elements at a time with a prefix sum over its lanes.
  int wlo, whi;
  const unsigned long long total = range_mass_by_wave(x, 0, vocab, floor_key, maxv, scan, &wlo, &whi);
  if (!need_mass_now) Z = total;
  if (total == 0 || Z == 0) {       // nothing left to draw from: the last index
    if (threadIdx.x == 0) out[row] = vocab - 1;
    return;
  }
  const float r = rnd[row];
  unsigned long long t = (unsigned long long)((double)r * (double)Z);
  if (t >= Z) t = Z - 1;
  const int at = range_find_by_wave(x, wlo, whi, 0ull, t, floor_key, maxv, scan);
  if (at >= 0) {
    out[row] = at;
    if (inf != nullptr) inf[3] = (x[at] - maxv) - lnZ;
  }
}

// The n most probable tokens of the distribution a row was drawn from (value descending, ties by index), with their
// log-probabilities (/root/reference/engine/src/model.rs:497-526).  `work` and `info` are what sample_kernel left.
// ids beyond the number of survivors are -1.
__global__ __launch_bounds__(SMP_THREADS) void top_logprobs_kernel(const float* __restrict__ work, const float* __restrict__ info,
                                                                   int vocab, int n, int* __restrict__ ids,
                                                                   float* __restrict__ lps) {
  __shared__ int ibest[SMP_WAVES];
  __shared__ float vbest[SMP_WAVES];
  const int row = blockIdx.x;
  const float* x = work + (size_t)row * vocab;
  const float maxv = info[4 * row], lnZ = info[4 * row + 1], floorv = info[4 * row + 2];
  float last_v = INFINITY;
  int last_i = -1;
  for (int i = 0; i < n; ++i) {
    float bv = -INFINITY;
    int bi = -1;
    auto better = [](float v, int j, float bv, int bi) { return j >= 0 && (bi < 0 || v > bv || (v == bv && j < bi)); };
    for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
      const float v = x[j];
      if (!(v >= floorv) || v == -INFINITY) continue;
      if (!(v < last_v || (v == last_v && j > last_i))) continue;   // taken in an earlier turn
      if (better(v, j, bv, bi)) {
        bv = v;
        bi = j;
      }
    }
    for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, TP_WAVE);
      const int oi = __shfl_xor(bi, o, TP_WAVE);
      if (better(ov, oi, bv, bi)) {
        bv = ov;
        bi = oi;
      }
    }
    __syncthreads();
    if (threadIdx.x % TP_WAVE == 0) {
      vbest[threadIdx.x / TP_WAVE] = bv;
      ibest[threadIdx.x / TP_WAVE] = bi;
    }
    __syncthreads();
    bv = vbest[0];
    bi = ibest[0];
    for (int w = 1; w < SMP_WAVES; ++w)
      if (better(vbest[w], ibest[w], bv, bi)) {
        bv = vbest[w];
        bi = ibest[w];
      }
    if (threadIdx.x == 0) {
      ids[row * n + i] = bi;
      lps[row * n + i] = bi < 0 ? -INFINITY : (bv - maxv) - lnZ;
    }
    if (bi < 0) {
      for (int k = i + 1 + threadIdx.x; k < n; k += blockDim.x) {
        ids[row * n + k] = -1;
        lps[row * n + k] = -INFINITY;
      }
      break;
    }
    last_v = bv;
    last_i = bi;
  }
}

// The sizes that the scratch buffers of tp_sample are laid out by, for the caller that allocates them: pieces of a row,
// candidates a piece may hand over, largest top_k settled from candidates, most elements of a piece, bins of a counting pass.
extern "C" int tp_sample_limits(int* out5) {
  TP_REQUIRE(out5 != nullptr, "sample_limits: no output");
  out5[0] = SMP_CHUNKS;
  out5[1] = SMP_CCAP;
  out5[2] = SMP_KMAX;
  out5[3] = SMP_PER_MAX;
  out5[4] = 256;
  return 0;
}

extern "C" int tp_sample(const float* logits, float* work, int rows, int vocab, const float* temperature,
                         const int* top_k, const float* top_p, const float* min_p, const float* typical_p,
                         const float* rnd, int* out, float* info, float* part_max, unsigned long long* part_mass,
                         unsigned int* part_cnt, float* cand_val, int* cand_idx, int* cand_cnt, unsigned int* cand_thr,
                         int* done, hipStream_t s) {
  // part_max: scratch of rows * 32 floats, or null (the row's first step then runs inside the one block per row);
  // part_mass: scratch of rows * 32 64-bit integers, given when some row is only scaled before the draw;
  // part_cnt: scratch of rows * 32 * 256 32-bit integers, given when some row is cut by top_k;
  // cand_val, cand_idx (rows * 32 * SMP_CCAP each), cand_cnt, cand_thr (rows * 32 each), done (rows): scratch for rows
  // cut by a small top_k or by top_p alone (all five or none; not with `info`; rows cut by top_p alone need part_mass too)
  TP_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes");
  if (rows == 0) return 0;
  const bool fast = part_max != nullptr && vocab >= 4096 && rows <= 65535 && info == nullptr && cand_val != nullptr &&
                    cand_idx != nullptr && cand_cnt != nullptr && cand_thr != nullptr && done != nullptr;
  if (!fast) cand_val = nullptr, cand_idx = nullptr, cand_cnt = nullptr, cand_thr = nullptr, done = nullptr;
  if (part_max != nullptr && vocab >= 4096 && rows <= 65535) {
    if (fast && (vocab + SMP_CHUNKS - 1) / SMP_CHUNKS > 16 * 256)
      hipLaunchKernelGGL(sample_scale_kernel<SMP_PER_MAX / 256>, dim3(rows, SMP_CHUNKS), dim3(256), 0, s, logits, work, vocab,
                         temperature, part_max, part_cnt, top_k, top_p, typical_p, cand_val, cand_idx, cand_cnt, cand_thr);
    else
      hipLaunchKernelGGL(sample_scale_kernel<16>, dim3(rows, SMP_CHUNKS), dim3(256), 0, s, logits, work, vocab, temperature,
                         part_max, part_cnt, top_k, top_p, typical_p, cand_val, cand_idx, cand_cnt, cand_thr);
  } else
    part_max = nullptr, part_cnt = nullptr;
  if (part_max != nullptr && part_mass != nullptr && info == nullptr)
    hipLaunchKernelGGL(sample_mass_kernel, dim3(rows, SMP_CHUNKS), dim3(256), 0, s, work, vocab, min_p, part_max, part_mass);
  else
    part_mass = nullptr;
  if (fast)
    hipLaunchKernelGGL(sample_topk_kernel, dim3(rows), dim3(256), 0, s, cand_val, cand_idx, cand_cnt, cand_thr, part_max,
                       part_mass, vocab, temperature, top_k, top_p, min_p, typical_p, rnd, out, done);
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SMP_THREADS), 0, s, logits, work, vocab, temperature, top_k,
                     top_p, min_p, typical_p, rnd, out, info, part_max, part_mass, part_cnt, done);
  TP_CHECK_LAUNCH("sample");
  return 0;
}

// `info` [rows, 4] and `work` as tp_sample left them; ids and lps are [rows, n].
extern "C" int tp_top_logprobs(const float* work, const float* info, int rows, int vocab, int n, int* ids, float* lps,
                               hipStream_t s) {
  TP_REQUIRE(rows >= 0 && vocab > 0 && n >= 0, "top_logprobs: bad sizes");
  if (rows == 0 || n == 0) return 0;
  hipLaunchKernelGGL(top_logprobs_kernel, dim3(rows), dim3(SMP_THREADS), 0, s, work, info, vocab, n, ids, lps);
  TP_CHECK_LAUNCH("top_logprobs");
  return 0;
}
