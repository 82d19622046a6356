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

typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// two floats to two bfloat16 (round to nearest even) with the hardware's packed conversion
__device__ inline unsigned int pack_bf16(float a, float b) {
  const f32x2_t f = {a, b};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, bf16x2_t));
}

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 with the row-swap instructions of gfx950
// (no trip through LDS): v_permlane16_swap exchanges the odd 16-lane rows of its first operand with
// the even rows of its second, v_permlane32_swap the upper half of the first with the lower half of
// the second; with both operands equal beforehand, the two registers afterwards hold each lane's own
// value and its partner's.  Written as assembly, with the wait states the instruction needs after a
// vector write, because the compiler's builtin folds the following max/add of the two results away.
__device__ inline void rows16_swap(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ inline void rows32_swap(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// (v_max_f32 as assembly: behind the swaps the compiler cannot tell that its operands are no signalling NaNs
// and would quiet each of them with an instruction of its own)
__device__ inline float max_raw(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ inline float quad_rows_max(float x) {
  float y = x;
  rows16_swap(x, y);
  x = max_raw(x, y);
  y = x;
  rows32_swap(x, y);
  return max_raw(x, y);
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
  int page_shift;   // log2(page_size), or -1
  float scale_log2;
  // portions whose keys are split over blocks (few query blocks, long contexts): the largest number of parts
  // (a query block with few steps gets fewer, or stays whole and writes its rows itself) and their partial
  // results, [token, head, part] of PART_STRIDE(D) floats: O (unnormalised), maximum, sum
  int portion_splits;
  int portion_min_steps;   // a query block is split into at most (its steps / this) parts
  float* portion_scratch;
  const int* token_req;
};
#define PART_STRIDE(D) ((D) + 4)

// The keys and values of one step of 32 keys, as MFMA operand fragments.
template <int D>
struct KvFrags {
  bf16x8_t k[2][D / 32];
  bf16x8_t v[D / 16];
};

// A lane's value fragment holds eight consecutive key places of one element.  Places past the last key that
// exists hold whatever the page's previous owner (or a padded row) left there; their probabilities are 0, but
// 0 * NaN and 0 * Inf are NaN, so one request's non-finite values would reach the next owner of the page.
// The mask keeps the first `n` places (n <= 0: none, n >= 8: all) and clears the others to +0.
__device__ inline u32x4_t attn_existing_keys(int n) {
  u32x4_t keep;
#pragma unroll
  for (int w = 0; w < 4; ++w) keep[w] = (2 * w < n ? 0x0000ffffu : 0u) | (2 * w + 1 < n ? 0xffff0000u : 0u);
  return keep;
}

// (per-wave loads of keys and values: a decode step reads a request's cache once, so the loads are nontemporal)
#define ATTN_KV_LOAD(p) __builtin_nontemporal_load(p)

// Fetch the fragments of the step starting at key j0 (kvh: kv head; ctx: keys that exist; keys
// past the end are clamped to the last one and masked later, values past the end are cleared).
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
    for (int dk = 0; dk < D / 32; ++dk) f.k[t][dk] = frag_of(ATTN_KV_LOAD((const u32x4_t*)(kr + dk * 32)));
  }
  // values: eight consecutive keys of element d per lane
  const int kb = min(j0 + 8 * g, (ctx - 1) & ~7);
  const int vpage = table[kb / ps];
  const bf16_t* vr = a.v_cache + ((size_t)(vpage * a.n_kv + kvh) * D + c) * ps + kb % ps;
  if (j0 + 32 > ctx) {   // the step that holds the last key
    const u32x4_t keep = attn_existing_keys(ctx - (j0 + 8 * g));
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) f.v[dt] = frag_of(ATTN_KV_LOAD((const u32x4_t*)(vr + (size_t)dt * 16 * ps)) & keep);
    return;
  }
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) f.v[dt] = frag_of(ATTN_KV_LOAD((const u32x4_t*)(vr + (size_t)dt * 16 * ps)));
}

// One step of 32 keys starting at j0 for NQ query tiles, on fetched fragments.  qpos[nq] is the
// absolute position of this lane's query column (keys above it are masked).  m/l/o are the
// running statistics and output of each tile.  MASK false: the caller knows that every key of the
// step is visible to every query of the wave (no comparison needed).
// The softmax arithmetic, not the matrix core, bounds this step, so it is kept short: the scale is
// folded into the exponent's FMA, and the running output is rescaled only when a maximum moved
// (when none did the factor is exactly 1).
template <int D, int NQ>
__device__ inline void attn_scores(const bf16x8_t (&k)[2][D / 32], const bf16x8_t (&qf)[NQ][D / 32], f32x4_t (&s)[NQ][2]) {
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      s[nq][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dk = 0; dk < D / 32; ++dk)
        s[nq][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k[t][dk], qf[nq][dk], s[nq][t], 0, 0, 0);
    }
}

// Softmax of one step's scores: probabilities as the next product's operand (pf), and the factor by
// which the running sums shrink (alpha; `moved` false when no maximum of the wave moved: alpha is 1).
template <int NQ, bool MASK>
__device__ inline void attn_softmax(const AttnArgs& a, int j0, const f32x4_t (&s)[NQ][2], const int (&qpos)[NQ],
                                    float (&m)[NQ], float (&l)[NQ], bf16x8_t (&pf)[NQ], float (&alpha)[NQ], bool (&moved)[NQ]) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    // this lane's keys: j0 + 8g + 4t + r
    float v[8];
    float mx = -INFINITY;
    if (MASK) {
      const int hi = qpos[nq];
      const int lo = a.window > 0 ? hi - a.window + 1 : 0;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = j0 + 8 * g + 4 * t + r;
          v[t * 4 + r] = (key <= hi && key >= lo) ? s[nq][t][r] : -INFINITY;
        }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) v[t * 4 + r] = s[nq][t][r];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) mx = fmaxf(mx, v[i]);
    mx = quad_rows_max(mx);
    const float m_new = fmaxf(m[nq], mx * a.scale_log2);    // the scale is positive
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column with nothing visible yet
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = __builtin_amdgcn_exp2f(fmaf(v[i], a.scale_log2, -m_use));
      sum += v[i];
    }
    u32x4_t pk;
    pk[0] = pack_bf16(v[0], v[1]);
    pk[1] = pack_bf16(v[2], v[3]);
    pk[2] = pack_bf16(v[4], v[5]);
    pk[3] = pack_bf16(v[6], v[7]);
    pf[nq] = frag_of(pk);
    moved[nq] = __builtin_amdgcn_ballot_w64(m_new != m[nq]) != 0;
    if (moved[nq]) {
      alpha[nq] = __builtin_amdgcn_exp2f(m[nq] - m_use);
      l[nq] = l[nq] * alpha[nq] + sum;  // per-lane partial sum; lanes of a column are added at the end
      m[nq] = m_new;
    } else {
      alpha[nq] = 1.0f;
      l[nq] += sum;
    }
  }
}

// The same arithmetic without a branch, in two halves (each one basic block, so that the scheduler may place
// another instruction stream's MFMAs between these instructions).  The first half needs only the scores: the
// masked values and the new maximum of every column; it runs while the next step's key fragments travel from LDS.
// The second half is the exponentials and the sums: alpha is computed always and chosen afterwards; where no
// maximum moved it is exactly 1 and l * 1 + sum is l + sum.
template <int NQ, bool MASK>
__device__ inline void attn_softmax_max(const AttnArgs& a, int j0, const f32x4_t (&s)[NQ][2], const int (&qpos)[NQ],
                                        const float (&m)[NQ], float (&v)[NQ][8], float (&m_new)[NQ]) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    float mx = -INFINITY;
    if (MASK) {
      const int hi = qpos[nq];
      const int lo = a.window > 0 ? hi - a.window + 1 : 0;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = j0 + 8 * g + 4 * t + r;
          v[nq][t * 4 + r] = (key <= hi && key >= lo) ? s[nq][t][r] : -INFINITY;
        }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) v[nq][t * 4 + r] = s[nq][t][r];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) mx = fmaxf(mx, v[nq][i]);
    mx = quad_rows_max(mx);
    m_new[nq] = fmaxf(m[nq], mx * a.scale_log2);
  }
}

template <int NQ>
__device__ inline void attn_softmax_exp(const AttnArgs& a, float (&v)[NQ][8], const float (&m_new)[NQ], float (&m)[NQ],
                                        float (&l)[NQ], bf16x8_t (&pf)[NQ], float (&alpha)[NQ], bool (&moved)[NQ]) {
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const float m_use = (m_new[nq] == -INFINITY) ? 0.f : m_new[nq];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[nq][i] = __builtin_amdgcn_exp2f(fmaf(v[nq][i], a.scale_log2, -m_use));
      sum += v[nq][i];
    }
    u32x4_t pk;
    pk[0] = pack_bf16(v[nq][0], v[nq][1]);
    pk[1] = pack_bf16(v[nq][2], v[nq][3]);
    pk[2] = pack_bf16(v[nq][4], v[nq][5]);
    pk[3] = pack_bf16(v[nq][6], v[nq][7]);
    pf[nq] = frag_of(pk);
    moved[nq] = __builtin_amdgcn_ballot_w64(m_new[nq] != m[nq]) != 0;
    const float shrink = __builtin_amdgcn_exp2f(m[nq] - m_use);
    alpha[nq] = moved[nq] ? shrink : 1.0f;
    l[nq] = fmaf(l[nq], alpha[nq], sum);
    m[nq] = m_new[nq];     // (where nothing moved, m_new is m)
  }
}

template <int D, int NQ>
__device__ inline void attn_pv(const bf16x8_t (&vf)[D / 16], const bf16x8_t (&pf)[NQ], const float (&alpha)[NQ],
                               const bool (&moved)[NQ], f32x4_t (&o)[NQ][D / 16]) {
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    if (moved[nq]) {
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) {
        o[nq][dt][0] *= alpha[nq];
        o[nq][dt][1] *= alpha[nq];
        o[nq][dt][2] *= alpha[nq];
        o[nq][dt][3] *= alpha[nq];
      }
    }
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) o[nq][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf[nq], o[nq][dt], 0, 0, 0);
  }
}

template <int D, int NQ, bool MASK>
__device__ inline void attn_softmax_pv(const AttnArgs& a, int j0, const f32x4_t (&s)[NQ][2], const bf16x8_t (&vf)[D / 16],
                                       const int (&qpos)[NQ], float (&m)[NQ], float (&l)[NQ], f32x4_t (&o)[NQ][D / 16]) {
  bf16x8_t pf[NQ];
  float alpha[NQ];
  bool moved[NQ];
  attn_softmax<NQ, MASK>(a, j0, s, qpos, m, l, pf, alpha, moved);
  attn_pv<D, NQ>(vf, pf, alpha, moved, o);
}

template <int D, int NQ, bool MASK = true>
__device__ inline void attn_compute(const AttnArgs& a, int j0, const KvFrags<D>& f, const bf16x8_t (&qf)[NQ][D / 32],
                                    const int (&qpos)[NQ], float (&m)[NQ], float (&l)[NQ], f32x4_t (&o)[NQ][D / 16]) {
  f32x4_t s[NQ][2];
  attn_scores<D, NQ>(f.k, qf, s);
  attn_softmax_pv<D, NQ, MASK>(a, j0, s, f.v, qpos, m, l, o);
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

// ---- prefill, keys and values through LDS ---------------------------------------------------
// The four waves of a block (four heads of one kv group) need the same keys and values.  Here a
// step's 32 keys and values are copied once per block into LDS by the direct global-to-LDS load,
// NS - 1 steps ahead of their use (a ring of NS stages, three or four; one barrier per step), and every wave reads
// its operand fragments from there: a quarter of the global load instructions, and none of their
// latency in the way.  Head sizes 32, 64, 128 (a power-of-two number of 16-byte chunks per key row); pages of
// at least 16 keys (a power of two), so that each half of a step lies in one page.
// LDS layout of a stage: the key tile as 32 rows of D elements, chunk c of row r stored at
// (c + f(r)) mod (D / 8) so that the 16 rows a quarter wave reads fall into different banks; the
// value tile in pieces of 1 KB, one per (32 elements, half of the step's keys), the eight keys 8 e.. of
// element d at place 32 e + d % 32 of its piece.
#define GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LPTR(p) ((__attribute__((address_space(3))) void*)(p))
#define ATTN_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

template <int OFF>
__device__ inline u32x4_t attn_lds_read(unsigned addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// Into how many parts the keys of a query block with `steps` steps of 32 keys are split.
__device__ __host__ inline int portion_parts(int steps, int max_parts, int min_steps) {
  return max_parts <= 1 ? 1 : min(max_parts, max(1, steps / min_steps));
}

template <int D, int NQ, int NS = 4, int OCC = 2>
__global__ __launch_bounds__(256, OCC) void attn_prefill_lds_kernel(AttnArgs a, int skip_single) {
  constexpr int C = D / 8;             // 16-byte chunks per key row
  constexpr int SH = C == 16 ? 0 : (C == 8 ? 1 : 2);
  constexpr int KI = D / 16;           // 1 KB loads per key tile (32 rows of 2 D bytes), and per value tile
  constexpr int LP = 2 * KI / 4;       // loads per wave and step
  constexpr int STAGE = 2 * KI * 1024;
  static_assert(D == 32 || D == 64 || D == 128, "head size");
  __shared__ __attribute__((aligned(1024))) unsigned char stages[NS * STAGE];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, c = lane & 15;
  // Blocks go to the eight XCDs in turn, each with an L2 of its own: neighbouring blocks take different
  // kv heads (fastest index), so that one L2 holds the keys and values of few heads, read by all their
  // query blocks; the longest query blocks come first.
  const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const int by = lin % gridDim.y, bx = (lin / gridDim.y) % gridDim.x;
  const int rz = lin / (gridDim.x * gridDim.y);
  const int r = rz / a.portion_splits, part = rz % a.portion_splits;   // (gridDim.z = requests * parts)
  const int q_start = a.cu_seqlens[r];
  const int q_len = a.cu_seqlens[r + 1] - q_start;
  if (q_len <= 0 || (skip_single && q_len == 1)) return;
  const int nqb = (q_len + 16 * NQ - 1) / (16 * NQ);
  if (bx >= nqb) return;
  const int group = a.n_heads / a.n_kv;
  const int kvh = by % a.n_kv;
  const int hin = (by / a.n_kv) * 4 + wave;
  const bool active = hin < group;     // a wave without a head still loads and waits with the others
  const int head = kvh * group + min(hin, group - 1);
  const int ctx = a.context_lens[r];
  const int pos0 = ctx - q_len;
  const int* table = a.block_tables + (size_t)r * a.table_width;
  const int ps = a.page_size;

  const int q0 = (nqb - 1 - bx) * 16 * NQ;
  bf16x8_t qf[NQ][D / 32];
  int qpos[NQ];
  float m[NQ], l[NQ];
  f32x4_t o[NQ][D / 16];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int qi = min(q0 + nq * 16 + c, q_len - 1);
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
  int nsteps = (last_pos - first) / 32 + 1;
  const int my_parts = portion_parts(nsteps, a.portion_splits, a.portion_min_steps);
  if (part >= my_parts) return;
  if (my_parts > 1) {   // this block's share of the steps (never empty: my_parts <= nsteps)
    const int s_begin = (int)((long)part * nsteps / my_parts), s_end = (int)((long)(part + 1) * nsteps / my_parts);
    first += s_begin * 32;
    nsteps = s_end - s_begin;
  }
  const int qpos_min = pos0 + min(q0, q_len - 1);   // the earliest query of this block

  // What this lane fetches in each of its loads of a step: load t = wave + 4 i.  t < KI is a piece of the key tile
  // (64 chunk slots: 64 / C whole rows of one group of eight keys), else a piece of the value tile: the step's keys
  // are two halves of 16 (each inside one page: pages hold at least 16 keys), and value load tv = t - KI covers half
  // tv % 2 for the 32 elements 32 (tv / 2)..: lane L takes the eight keys L / 32 of element L % 32.  So every load
  // has ONE page, and its address is a uniform part (scalar arithmetic, no branches) plus the lane's constant
  // offset.  Page numbers are read with wave-uniform (scalar) loads, one step ahead: a vector load here would have
  // to wait for every outstanding copy into LDS.
  const int psh = a.page_shift, pmask = ps - 1;
  __builtin_assume(wave >= 0 && wave < 4);
  // the block table through the constant address space: uniform loads from it are scalar loads
  const __attribute__((address_space(4))) int* ctab = (const __attribute__((address_space(4))) int*)(uintptr_t)table;
  // (key load t: slot 64 t + lane of the key tile, row = slot / C, chunk slot % C rotated by the row)
  auto key_row = [&](int t) { return (64 * t + lane) / C; };
  auto key_byte = [&](int t) {
    const int row = (64 * t + lane) / C, pc = (64 * t + lane) % C;
    const int f = ((((row >> 3) << 2) | (row & 3)) >> SH);
    return ((pc - f) & (C - 1)) * 16;
  };
  auto value_row = [&](int t) { return 32 * ((t - KI) >> 1) + (lane & 31); };
  unsigned lane_off[LP];   // byte offset of this lane's 16 bytes from the uniform part of a load's address
  bool second[LP];         // the load's keys lie in the second half of the step (keys j0 + 16..)
  unsigned row8[LP];       // key loads: the first key of the load's group of eight, from j0
#pragma unroll
  for (int i = 0; i < LP; ++i) {
    const int t = wave + 4 * i;
    if (t < KI) {
      const int gr = ((64 * t) / C) >> 3;
      lane_off[i] = (unsigned)((key_row(t) - 8 * gr) * D * 2 + key_byte(t));
      second[i] = gr >= 2;
      row8[i] = 8 * gr;
    } else {
      lane_off[i] = (unsigned)((value_row(t) * ps + 8 * (lane >> 5)) * 2);
      second[i] = ((t - KI) & 1) != 0;
      row8[i] = 0;
    }
  }
  const unsigned page_bytes = (unsigned)(a.n_kv * D * ps * 2);   // of a key page, and of a value page
  const unsigned char* kbase = (const unsigned char*)a.k_cache + (size_t)kvh * ps * D * 2;
  const unsigned char* vbase = (const unsigned char*)a.v_cache + (size_t)kvh * D * ps * 2;
  // the pages of the two halves of the step that is issued next (the second clamped to the last key that exists)
  int pp0 = 0, pp1 = 0;
  auto pages_of = [&](int step) {
    const int j0 = first + step * 32;
    pp0 = ctab[j0 >> psh];
    pp1 = ctab[min(j0 + 16, (ctx - 1) & ~7) >> psh];
  };
  auto issue = [&](int step, int stage) {
    const int j0 = first + step * 32;
    unsigned char* buf = stages + stage * STAGE;
    if (j0 + 32 <= ctx) {   // all 32 keys exist
#pragma unroll
      for (int i = 0; i < LP; ++i) {
        const int t = wave + 4 * i;
        const unsigned page = (unsigned)(second[i] ? pp1 : pp0);
        const unsigned char* src;
        if (t < KI)
          src = kbase + (size_t)page * page_bytes + (unsigned)(((j0 + row8[i]) & pmask) * D * 2);
        else
          src = vbase + (size_t)page * page_bytes + (unsigned)(((j0 + (second[i] ? 16 : 0)) & pmask) * 2);
        __builtin_amdgcn_global_load_lds(GPTR(src + lane_off[i]), LPTR(buf + t * 1024), 16, 0, 0);
      }
      return;
    }
    // the step that holds the last key: rows and groups past it are clamped to it (their scores are masked, their
    // values cleared when they are read)
#pragma unroll
    for (int i = 0; i < LP; ++i) {
      const int t = wave + 4 * i;
      const unsigned char* src;
      if (t < KI) {
        const int key = min(j0 + key_row(t), ctx - 1);
        const int page = second[i] ? pp1 : pp0;
        src = (const unsigned char*)(a.k_cache + ((size_t)(page * a.n_kv + kvh) * ps + (key & pmask)) * D) + key_byte(t);
      } else {
        const int kb = min(j0 + (second[i] ? 16 : 0) + 8 * (lane >> 5), (ctx - 1) & ~7);
        const int page = second[i] ? pp1 : pp0;
        src = (const unsigned char*)(a.v_cache + ((size_t)(page * a.n_kv + kvh) * D + value_row(t)) * ps + (kb & pmask));
      }
      __builtin_amdgcn_global_load_lds(GPTR(src), LPTR(buf + t * 1024), 16, 0, 0);
    }
  };
  // this lane's read addresses inside a stage
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)&stages[0];
  unsigned kaddr[2][D / 32];
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) {
    const int row = 8 * (c >> 2) + 4 * t2 + (c & 3);
#pragma unroll
    for (int dk = 0; dk < D / 32; ++dk) kaddr[t2][dk] = (row * C + ((dk * 4 + g + (c >> SH)) & (C - 1))) * 16;
  }
  // value fragment dt of lane (g, c): element 16 dt + c, keys 8 g..: load 2 (dt / 2) + g / 2, place 32 (g % 2) + 16 (dt % 2) + c;
  // eight neighbouring lanes read 128 contiguous bytes
  const unsigned vaddr = KI * 1024 + (g >> 1) * 1024 + (g & 1) * 512 + c * 16;

#pragma unroll
  for (int p = 0; p < NS; ++p)
    if (p < nsteps) {
      pages_of(p);
      issue(p, p);
    }
  if (NS < nsteps) pages_of(NS);
  // The scores of step s + 1 are multiplied while the softmax of step s runs on the vector ALU (two
  // independent instruction streams for the scheduler to interleave); so step s reads the values of
  // stage s and the keys of stage s + 1, and a stage is free again one step later than it would be.
  auto read_keys = [&](unsigned base, bf16x8_t (&kf)[2][D / 32]) {
    u32x4_t kk[2][D / 32];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int dk = 0; dk < D / 32; ++dk) kk[t2][dk] = attn_lds_read<0>(base + kaddr[t2][dk]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int dk = 0; dk < D / 32; ++dk) {
        asm volatile("" : "+v"(kk[t2][dk]));
        kf[t2][dk] = frag_of(kk[t2][dk]);
      }
  };
  f32x4_t sc[NQ][2];
  {
    const int behind = min(NS - 1, nsteps - 1);   // steps in flight behind the first
    if (behind >= 3) ATTN_WAIT_VM(3 * LP); else if (behind == 2) ATTN_WAIT_VM(2 * LP); else if (behind == 1) ATTN_WAIT_VM(LP); else ATTN_WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    bf16x8_t kf[2][D / 32];
    read_keys(lds0, kf);
    attn_scores<D, NQ>(kf, qf, sc);
  }
  int stage = 0;
  // one step: `cur` holds this step's scores, the next step's go to `nxt` (the loop below runs two steps per
  // turn with the two sets swapping roles, so that no register is copied)
  auto step = [&](int s, f32x4_t (&cur)[NQ][2], f32x4_t (&nxt)[NQ][2]) {
    const int nstage = stage + 1 == NS ? 0 : stage + 1;
    // step s + 1 has landed for this wave (later steps may stay in flight), then for all; every wave
    // is done with the stage of step s - 1
    const int ahead = min(NS - 3, nsteps - 2 - s);
    if (ahead >= 1) ATTN_WAIT_VM(LP); else ATTN_WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    if (s >= 1 && s + NS - 1 < nsteps) {
      issue(s + NS - 1, stage == 0 ? NS - 1 : stage - 1);
      if (s + NS < nsteps) pages_of(s + NS);
    }
    const unsigned base = lds0 + stage * STAGE;
    // The keys of the following stage are multiplied into the next step's scores while this step's softmax runs
    // on the vector ALU: its first half (the maxima) while the key fragments travel from LDS, its second (the
    // exponentials) as one block of instructions with the score MFMAs, without a branch, and the scheduler is told
    // to put a few of the softmax's instructions behind each MFMA (a wave issues in order: sixteen MFMAs in a row
    // would hold the softmax back for as long as they take).
    bf16x8_t pf[NQ];
    float alpha[NQ];
    bool moved[NQ];
    u32x4_t vv[D / 16];
    const int j0 = first + s * 32;
    const bool plain_step = j0 + 31 <= qpos_min && (a.window <= 0 || j0 >= last_pos - a.window + 1);
#define ATTN_RV(dt) if constexpr (dt < D / 16) vv[dt] = attn_lds_read<(dt >> 1) * 2048 + (dt & 1) * 256>(base + vaddr)
#define ATTN_BODY(NEXT, MASK)                                                                          \
  {                                                                                                    \
    u32x4_t kk[2][D / 32];                                                                             \
    if (NEXT) {                                                                                        \
      _Pragma("unroll") for (int t2 = 0; t2 < 2; ++t2)                                                 \
        _Pragma("unroll") for (int dk = 0; dk < D / 32; ++dk)                                          \
          kk[t2][dk] = attn_lds_read<0>(lds0 + nstage * STAGE + kaddr[t2][dk]);                        \
    }                                                                                                  \
    ATTN_RV(0); ATTN_RV(1); ATTN_RV(2); ATTN_RV(3); ATTN_RV(4); ATTN_RV(5); ATTN_RV(6); ATTN_RV(7);    \
    float v[NQ][8], m_new[NQ];                                                                         \
    attn_softmax_max<NQ, MASK>(a, j0, cur, qpos, m, v, m_new);                                         \
    __builtin_amdgcn_sched_barrier(0);                                                                 \
    if (NEXT) {                                                                                        \
      /* the key fragments have arrived (the D / 16 value fragments behind them need not) */           \
      static_assert(D / 16 <= 8, "value fragments of a step");                                         \
      if constexpr (D == 128) asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");                       \
      else if constexpr (D == 64) asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory");                   \
      else asm volatile("s_waitcnt lgkmcnt(2)" ::: "memory");                                          \
      bf16x8_t kf[2][D / 32];                                                                          \
      _Pragma("unroll") for (int t2 = 0; t2 < 2; ++t2)                                                 \
        _Pragma("unroll") for (int dk = 0; dk < D / 32; ++dk) {                                        \
          asm volatile("" : "+v"(kk[t2][dk]));                                                         \
          kf[t2][dk] = frag_of(kk[t2][dk]);                                                            \
        }                                                                                              \
      attn_scores<D, NQ>(kf, qf, nxt);                                                                 \
    }                                                                                                  \
    attn_softmax_exp<NQ>(a, v, m_new, m, l, pf, alpha, moved);                                         \
    if (NEXT) {                                                                                        \
      _Pragma("unroll") for (int i = 0; i < 4 * NQ * (D / 32); ++i) {                                  \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                             \
        __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);                                 \
      }                                                                                                \
    }                                                                                                  \
  }
    constexpr int VALU_PER_MFMA = 6;
    if constexpr (NQ == 1) {
      // (one query tile a wave, three blocks a CU: the waves of a SIMD fill one another's gaps, and the interleaved
      // block would cost registers that this variant does not have: 2,048 tokens 68 us either way)
      if (s + 1 < nsteps) {
        bf16x8_t kf[2][D / 32];
        read_keys(lds0 + nstage * STAGE, kf);
        attn_scores<D, NQ>(kf, qf, nxt);
      }
      ATTN_RV(0); ATTN_RV(1); ATTN_RV(2); ATTN_RV(3); ATTN_RV(4); ATTN_RV(5); ATTN_RV(6); ATTN_RV(7);
      if (plain_step)
        attn_softmax<NQ, false>(a, j0, cur, qpos, m, l, pf, alpha, moved);
      else
        attn_softmax<NQ, true>(a, j0, cur, qpos, m, l, pf, alpha, moved);
    } else if (s + 1 < nsteps) {
      if (plain_step) ATTN_BODY(true, false) else ATTN_BODY(true, true)
    } else {
      if (plain_step) ATTN_BODY(false, false) else ATTN_BODY(false, true)
    }
#undef ATTN_BODY
#undef ATTN_RV
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    bf16x8_t vf[D / 16];
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      asm volatile("" : "+v"(vv[dt]));
      vf[dt] = frag_of(vv[dt]);
    }
    if (j0 + 32 > ctx) {   // the step that holds the last key: places past it are cleared (see attn_existing_keys)
      const u32x4_t keep = attn_existing_keys(ctx - (j0 + 8 * g));
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) vf[dt] = frag_of(vv[dt] & keep);
    }
    attn_pv<D, NQ>(vf, pf, alpha, moved, o);
    stage = nstage;
  };
  f32x4_t sd[NQ][2];
  for (int s = 0; s < nsteps; s += 2) {
    step(s, sc, sd);
    if (s + 1 < nsteps) step(s + 1, sd, sc);
  }
  if (active) {
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    float lt = l[nq];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    const float inv = 1.0f / lt;
    const int qi = q0 + nq * 16 + c;
    if (qi < q_len && my_parts > 1) {
      float* pr = a.portion_scratch + (((size_t)(q_start + qi) * a.n_heads + head) * a.portion_splits + part) * PART_STRIDE(D);
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) *(f32x4_t*)(pr + dt * 16 + 4 * g) = o[nq][dt];
      if (g == 0) {
        pr[D] = m[nq];
        pr[D + 1] = lt;
      }
    } else if (qi < q_len) {
      bf16_t* orow = a.out + ((size_t)(q_start + qi) * a.n_heads + head) * D;
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) {
        uint2 w;
        w.x = pack_bf16(o[nq][dt][0] * inv, o[nq][dt][1] * inv);
        w.y = pack_bf16(o[nq][dt][2] * inv, o[nq][dt][3] * inv);
        *(uint2*)(orow + dt * 16 + 4 * g) = w;
      }
    }
  }
  }
}

// ---- decode -----------------------------------------------------------------------------
// grid: (kv_heads * ceil(group / 16), requests, splits); block: 4 waves.  Handles requests
// with exactly one new token.  Scratch per (request, head, split): D floats of O, then max, sum.
// (The kv heads run fastest: consecutive blocks go to the eight XCDs in turn, so the heads of every request are
// spread over all of them and each XCD reads about the same number of bytes however the contexts differ.  With
// the requests fastest, 60 requests of 128 to 2,304 keys took 77 us where 60 of their mean took 54: the XCD
// with the longest requests set the time, and more splits changed nothing, since the splits of a (request, head)
// pair fell to the same XCD.)
template <int D>
__global__ __launch_bounds__(256) void attn_decode_kernel(AttnArgs a) {
  __shared__ float red_o[4][D][16];
  __shared__ float red_m[4][16], red_l[4][16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int r = blockIdx.y;
  const int q_start = a.cu_seqlens[r];
  if (a.cu_seqlens[r + 1] - q_start != 1) return;
  const int group = a.n_heads / a.n_kv;
  const int hblocks = (group + 15) / 16;
  const int kvh = blockIdx.x / hblocks;
  const int h0 = (blockIdx.x % hblocks) * 16;            // first head (within the group) of this block
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
  // (every lane runs every turn of these loops, also where the head size is no multiple of 64: a lane that sat
  // out a turn could not hand its split's weight to the others, and with more than 32 splits of a head size of
  // 32 or 96 the lanes that hold the later splits' weights would sit out)
  for (int d0 = 0; d0 < D; d0 += 64) {
    const int d = min(d0 + lane, D - 1);
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
    if (d0 + lane < D) out[((size_t)q_start * n_heads + h) * D + d] = float_to_bf16(acc * inv);
  }
}

// The same for the rows of portions whose keys were split over blocks: out[token, head, :] from the parts
// [token, head, part] of PART_STRIDE(D) floats, in ascending order.  A row's query block (of 32 rows) may have
// been split into fewer parts than the most, or not at all (then the attention kernel wrote the row itself):
// the count is worked out here as it is there.  grid: (tokens, heads); block: one wave.
__global__ __launch_bounds__(64) void attn_combine_rows_kernel(const float* __restrict__ scratch,
                                                               const int* __restrict__ cu_seqlens,
                                                               const int* __restrict__ context_lens,
                                                               const int* __restrict__ token_req,
                                                               bf16_t* __restrict__ out, int n_heads, int D,
                                                               int max_parts, int min_steps, int window, int skip_single) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = token_req[t];
  const int q_start = cu_seqlens[r], q_len = cu_seqlens[r + 1] - q_start;
  if (skip_single && q_len == 1) return;   // (the decode kernels wrote this row)
  const int pos0 = context_lens[r] - q_len;
  const int q0 = ((t - q_start) / 32) * 32;
  const int last_pos = pos0 + min(q0 + 32, q_len) - 1;
  const int first = window > 0 ? (max(0, pos0 + q0 - window + 1) & ~31) : 0;
  const int parts = portion_parts((last_pos - first) / 32 + 1, max_parts, min_steps);
  if (parts == 1) return;
  const int stride = PART_STRIDE(D);
  const float* base = scratch + ((size_t)t * n_heads + h) * max_parts * stride;
  float ms = -INFINITY, ls = 0.f;
  if (lane < parts) {
    ms = base[(size_t)lane * stride + D];
    ls = base[(size_t)lane * stride + D + 1];
  }
  const float mg = wave_max(ms);
  const float mu = (mg == -INFINITY) ? 0.f : mg;
  const float ws = __builtin_amdgcn_exp2f(ms - mu);  // 0 for lanes without a part
  const float inv = 1.0f / wave_sum(ws * ls);
  for (int d0 = 0; d0 < D; d0 += 64) {      // (every lane runs every turn: see attn_combine_kernel)
    const int d = min(d0 + lane, D - 1);
    float acc = 0.f;
    for (int s = 0; s < parts; ++s) acc = fmaf(__shfl(ws, s, 64), base[(size_t)s * stride + d], acc);
    if (d0 + lane < D) out[((size_t)t * n_heads + h) * D + d] = float_to_bf16(acc * inv);
  }
}

// ---- dispatch ------------------------------------------------------------------------------
static int g_attn_tune = 0;   // 1: portions take the kernel that loads keys and values per wave; 2 / 3: 32 / 16 query rows per wave
extern "C" void tp_attention_tune(int v) { g_attn_tune = v; }

template <int D>
static int launch_all(AttnArgs a, int n_tokens, int n_req, int max_q_len, int num_single, hipStream_t s) {
  const int group = a.n_heads / a.n_kv;
  const bool has_multi = num_single < n_req;
  if (num_single > 0) {
    const dim3 grid(a.n_kv * ((group + 15) / 16), n_req, a.num_splits);
    hipLaunchKernelGGL(attn_decode_kernel<D>, grid, dim3(256), 0, s, a);
    if (a.num_splits > 1) {
      const dim3 cgrid(n_req, a.n_heads);
      hipLaunchKernelGGL(attn_combine_kernel, cgrid, dim3(64), 0, s, a.scratch, a.cu_seqlens, a.out, a.n_heads, D,
                         a.num_splits);
    }
  }
  if (has_multi) {
    // A wave owns 16 query rows, three blocks to a CU, or 32 rows (two tiles: half the key and value reads per
    // product, more registers), two blocks to a CU.  A step's time is set by how many instructions a wave has to
    // issue, so more waves help while there are few blocks: measured with 32 heads of 128 in 8 groups, 16 rows are
    // faster up to about 2,500 query rows (1,024: 31 against 42 us; 2,048: 60 against 78; 3,072: 125 against 118;
    // 8,192: 733 against 674; 32,768: 10.9 against 9.4 ms).  Both give the same bits: a query column never sees
    // another's values.
    const int kv_groups = a.n_kv * ((group + 3) / 4);
    // (blocks of 32 rows that have work: from the rows of the portions, not from the grid, which spans the longest
    // portion for every request; single tokens take the decode kernel)
    const long blocks2 = (long)((n_tokens - num_single + 31) / 32 + (n_req - num_single - 1)) * kv_groups;
    const bool two = g_attn_tune == 2 || (g_attn_tune != 3 && blocks2 >= 768);
    const int rows = two ? 32 : 16;
    const int skip = num_single > 0 ? 1 : 0;
    if constexpr (D == 32 || D == 64 || D == 128) {
      if (a.portion_splits > 1 && g_attn_tune != 1 && a.page_shift >= 4 && a.page_size >= 512 / D) {
        // few query blocks under a long context: the keys of each are split over blocks (of 32 query rows)
        const dim3 sgrid((max_q_len + 31) / 32, kv_groups, n_req * a.portion_splits);
        hipLaunchKernelGGL((attn_prefill_lds_kernel<D, 2>), sgrid, dim3(256), 0, s, a, skip);
        hipLaunchKernelGGL(attn_combine_rows_kernel, dim3(n_tokens, a.n_heads), dim3(64), 0, s, a.portion_scratch,
                           a.cu_seqlens, a.context_lens, a.token_req, a.out, a.n_heads, D, a.portion_splits,
                           a.portion_min_steps, a.window, skip);
        return 0;
      }
    }
    a.portion_splits = 1;   // (the kernels below do not split)
    const dim3 grid((max_q_len + rows - 1) / rows, kv_groups, n_req);
    if constexpr (D == 32 || D == 64 || D == 128) {
      // (a key load covers 512 / D rows, which must lie in one page)
      if (g_attn_tune != 1 && a.page_shift >= 4 && a.page_size >= 512 / D) {
        if (two)
          hipLaunchKernelGGL((attn_prefill_lds_kernel<D, 2>), grid, dim3(256), 0, s, a, skip);
        else
          hipLaunchKernelGGL((attn_prefill_lds_kernel<D, 1, 3, 3>), grid, dim3(256), 0, s, a, skip);
        return 0;
      }
    }
    if (two)
      hipLaunchKernelGGL((attn_prefill_kernel<D, 2>), grid, dim3(256), 0, s, a, skip);
    else
      hipLaunchKernelGGL((attn_prefill_kernel<D, 1>), grid, dim3(256), 0, s, a, skip);
  }
  return 0;
}

int tp_paged_attention_fast(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                            int table_width, const int* cu_seqlens, const int* context_lens, void* out, int n_tokens,
                            int n_req, int n_heads, int n_kv, int head_dim, int page_size, float scale, int window,
                            int max_q_len, int num_single, int num_splits, float* scratch, const int* token_req,
                            int portion_splits, int portion_min_steps, float* portion_scratch, hipStream_t s) {
  if (head_dim % 32 != 0 || head_dim > 128 || page_size % 8 != 0) return -1;
  if (portion_min_steps < 1) return -1;
  if (portion_splits < 1 || portion_splits > 64 || (portion_splits > 1 && (portion_scratch == nullptr || token_req == nullptr))) return -1;
  if ((long)n_req * portion_splits > 65535) return -1;
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
  a.page_shift = -1;
  for (int b = 0; b < 30; ++b)
    if ((1 << b) == page_size) a.page_shift = b;
  a.window = window;
  a.num_splits = num_splits;
  a.portion_splits = portion_splits;
  a.portion_min_steps = portion_min_steps;
  a.portion_scratch = portion_scratch;
  a.token_req = token_req;
  a.scale_log2 = scale * 1.4426950408889634f;
  switch (head_dim) {
    case 32: launch_all<32>(a, n_tokens, n_req, max_q_len, num_single, s); break;
    case 64: launch_all<64>(a, n_tokens, n_req, max_q_len, num_single, s); break;
    case 96: launch_all<96>(a, n_tokens, n_req, max_q_len, num_single, s); break;
    case 128: launch_all<128>(a, n_tokens, n_req, max_q_len, num_single, s); break;
    default: return -1;
  }
  TP_CHECK_LAUNCH("paged_attention (mfma)");
  return 0;
}
