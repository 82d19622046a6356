// Large bfloat16 products (prefill): out[M, N] (+)= x[M, K] * w[N, K]^T on the gfx950 matrix cores,
// software-pipelined by hand.
//
// A block of four waves (2 x 2) owns a 256 x 128 result tile, a wave 128 x 64 of it (8 x 4 tiles of
// v_mfma_f32_16x16x32_bf16, 128 accumulator registers).  K moves in steps of 64.  Three stages of
// (256 + 128) rows x 128 bytes live in LDS (144 KB, one block per CU); global memory is copied into
// them by the direct global-to-LDS load, so the operands never pass through registers on their way
// in.  What the measurements on MI355X asked for, in order of weight:
//  * every instruction that is not an MFMA sits between two MFMAs.  One wave per SIMD issues in
//    order, so a run of address arithmetic, loads or LDS reads is time in which the matrix core
//    idles; spread out one at a time they cost nothing.  The LDS reads of the next half step (32 of
//    K) and the global loads of the stage after next are therefore interleaved with the MFMAs of the
//    current half step, and the operand fragments are double-buffered in registers.
//  * LDS reads are inline assembly: the compiler would otherwise wait for every outstanding
//    global-to-LDS load before each of them.  The waits are written by hand (vmcnt for the stage
//    that must have landed, lgkmcnt for the fragments).
//  * a 128-byte LDS row holds eight 16-byte chunks, chunk c of row r at position c ^ ((r >> 1) & 7):
//    the 16 rows x 16 bytes that a quarter wave reads then fall into 16 different bank groups.
//  * blocks go to the eight XCDs round robin; the blocks that one XCD runs at a time form a patch of
//    (row blocks x column blocks) that share their operand tiles through that XCD's L2.
//  * the result leaves through LDS, so that every store covers whole cache lines (emit_tile).
//  * the weights may come tiled (wt: [N / 16][K / 32][64][8], a 16 x 32 block in the matrix cores' operand order as
//    1,024 contiguous bytes): a load then copies one block to LDS as it is, the fragment read is the lane's own
//    16 bytes of it, and nothing of the above swizzle applies to that operand.
// One barrier per 64 of K.  Sizes: K % 64 == 0; any M and N (loads clamp to the last row, stores are
// masked).  The sum over K runs in ascending order for every output element.
// Further down: the same pipeline on 256 x 256 block tiles (gemm_pipe_big_kernel; the host mixes both tile
// sizes so that whole rounds of tiles fill the CUs) and on 64 x 128 tiles for 17..64 rows (gemm_pipe64_kernel).
#include <algorithm>

#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

// the same codes as in gemm_mfma.hip
enum { OUT_F32 = 0, OUT_BF16 = 1, OUT_ACC_F32 = 2, OUT_SWIGLU = 3 };

#define GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LPTR(p) ((__attribute__((address_space(3))) void*)(p))

namespace {

constexpr int BM = 256, BN = 128, BK = 64, ROWB = 128;
constexpr int STAGE_BYTES = (BM + BN) * ROWB;
constexpr int NS = 3;
constexpr int LPW = 12;        // direct loads per wave and stage: eight of x rows, four of w rows
constexpr int CLD = 64 + 4;    // padded row of a wave's result tile in LDS, in floats

__device__ inline bf16x8_t as_frag(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }
// g * sigmoid(g) * u with the hardware's exp2 and reciprocal (one ulp each; the result is rounded to bfloat16)
__device__ inline float silu_mul(float g, float u) {
  return g * u * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// two floats to two bfloat16 (round to nearest even) in one instruction
__device__ inline unsigned pack_bf16(float a, float b) {
  const f32x2_t f = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2_t));
}

// vmcnt(n) alone: bits [3:0] and [15:14] hold n, the other counters stay at their maxima
#define WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

// One LDS-direct load of 16 bytes a lane from `base` (the same for every lane) + `off` (the lane's own), as a buffer
// load: the base travels in scalar registers and the lane's 32-bit offset goes in as it is, where the flat form
// needs a 64-bit address per lane from the vector unit and holds up the wave's MFMAs for longer (a loop of 32
// MFMAs, 12 LDS reads, a barrier and six such loads, four waves a CU: 1.53 PFLOP/s with flat loads, 1.82 with these,
// 2.1 without loads).  The buffer spans 2 GiB from `base`.
template <int AUX = 0>
__device__ inline void load_lds16(const unsigned char* base, unsigned off, unsigned char* lds) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7fffffff, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LPTR(lds), 16, off, 0, 0, AUX);
}

// load I (0..11) of this wave into stage `buf`: 0..7 are x rows, 8..11 w rows; one load covers 8 rows
template <int I>
__device__ inline void issue_one(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                 const unsigned (&voff)[LPW], int wave) {
  const int t = I < 8 ? wave * 8 + I : 32 + wave * 4 + (I - 8);
  load_lds16(I < 8 ? xk : wk, voff[I], buf + t * 1024);
}

__device__ inline void issue_stage(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                   const unsigned (&voff)[LPW], int wave) {
  issue_one<0>(buf, xk, wk, voff, wave);
  issue_one<1>(buf, xk, wk, voff, wave);
  issue_one<2>(buf, xk, wk, voff, wave);
  issue_one<3>(buf, xk, wk, voff, wave);
  issue_one<4>(buf, xk, wk, voff, wave);
  issue_one<5>(buf, xk, wk, voff, wave);
  issue_one<6>(buf, xk, wk, voff, wave);
  issue_one<7>(buf, xk, wk, voff, wave);
  issue_one<8>(buf, xk, wk, voff, wave);
  issue_one<9>(buf, xk, wk, voff, wave);
  issue_one<10>(buf, xk, wk, voff, wave);
  issue_one<11>(buf, xk, wk, voff, wave);
}

template <int OFF>
__device__ inline u32x4_t lds_read16(unsigned addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// operand fragments of one half step (32 of K): eight 16-row tiles of x, four of w
struct Frags {
  u32x4_t a[8], b[4];
};

__device__ inline void wait_frags(Frags& f) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.a[4]), "+v"(f.a[5]), "+v"(f.a[6]),
                 "+v"(f.a[7]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3]));
}

// read R (0..11) of a half step: b0..b3, then a0..a7
template <int R>
__device__ inline void read_one(Frags& f, unsigned aaddr, unsigned baddr) {
  if constexpr (R < 4)
    f.b[R] = lds_read16<R * 16 * ROWB>(baddr);
  else
    f.a[R - 4] = lds_read16<(R - 4) * 16 * ROWB>(aaddr);
}

template <int I, int J>
__device__ inline void mfma_one(f32x4_t (&acc)[8][4], const Frags& f) {
  acc[I][J] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(f.a[I]), as_frag(f.b[J]), acc[I][J], 0, 0, 0);
}

// The 32 MFMAs of `cur`; between them, one at a time, the LDS reads into `nxt` (READ) and the global
// loads of a stage (LOAD).
template <bool READ, bool LOAD>
__device__ inline void half_step(f32x4_t (&acc)[8][4], const Frags& cur, Frags& nxt, unsigned aaddr, unsigned baddr,
                                 unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                 const unsigned (&voff)[LPW], int wave) {
#define SB() __builtin_amdgcn_sched_barrier(0)
#define RD(R) \
  if (READ) read_one<R>(nxt, aaddr, baddr); \
  SB()
#define LD(I) \
  if (LOAD) issue_one<I>(buf, xk, wk, voff, wave); \
  SB()
#define M1(I, J) \
  mfma_one<I, J>(acc, cur); \
  SB()
  RD(0); M1(0, 0); LD(0); M1(0, 1); RD(1); M1(0, 2); LD(1); M1(0, 3);
  RD(2); M1(1, 0); LD(2); M1(1, 1); RD(3); M1(1, 2); LD(3); M1(1, 3);
  RD(4); M1(2, 0); LD(4); M1(2, 1); RD(5); M1(2, 2); LD(5); M1(2, 3);
  RD(6); M1(3, 0); LD(6); M1(3, 1); RD(7); M1(3, 2); LD(7); M1(3, 3);
  RD(8); M1(4, 0); LD(8); M1(4, 1); RD(9); M1(4, 2); LD(9); M1(4, 3);
  RD(10); M1(5, 0); LD(10); M1(5, 1); RD(11); M1(5, 2); LD(11); M1(5, 3);
  M1(6, 0); M1(6, 1); M1(6, 2); M1(6, 3); M1(7, 0); M1(7, 1); M1(7, 2); M1(7, 3);
#undef RD
#undef LD
#undef M1
#undef SB
}

#define READ_ALL(f, aaddr, baddr)                                                                                  \
  read_one<0>(f, aaddr, baddr); read_one<1>(f, aaddr, baddr); read_one<2>(f, aaddr, baddr); read_one<3>(f, aaddr, baddr); \
  read_one<4>(f, aaddr, baddr); read_one<5>(f, aaddr, baddr); read_one<6>(f, aaddr, baddr); read_one<7>(f, aaddr, baddr); \
  read_one<8>(f, aaddr, baddr); read_one<9>(f, aaddr, baddr); read_one<10>(f, aaddr, baddr); read_one<11>(f, aaddr, baddr)


// The epilogue's fast path, for a wave tile that lies inside the result with rows of `out` aligned to 16 bytes:
// a lane moves 16 bytes per row (eight bfloat16 or four float32 columns), the output pointer steps by a uniform
// stride from pass to pass, and nothing is compared.  (Measured on 256 x 256 tiles: per row and lane a 64-bit
// multiply for the address, a row check and a branch took as long as the store itself, and stores of 8 bytes
// per lane twice as long as stores of 16.)
template <int ROWS, int COLS, int LD>
__device__ inline void emit_tile_fast(const float* ct, int lane, int mrow0, int ncol0, void* out, int mode, int ldo) {
  if (mode == OUT_SWIGLU) {
    // eight outputs per lane: the eight gate columns of a group of sixteen and the eight up columns after them
    constexpr int LPR = COLS / 16, RPP = 64 / LPR, PASSES = ROWS / RPP, B = PASSES < 4 ? PASSES : 4;
    const int o = (lane % LPR) * 8, rr = lane / LPR;
    const float* src = ct + rr * LD + (lane % LPR) * 16;
    bf16_t* dst = (bf16_t*)out + (size_t)(mrow0 + rr) * ldo + ncol0 / 2 + o;
    const size_t step = (size_t)RPP * ldo;
#pragma unroll
    for (int p0 = 0; p0 < PASSES; p0 += B) {
      f32x4_t g0[B], g1[B], u0[B], u1[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const float* r = src + (p0 + u) * RPP * LD;
        g0[u] = *(const f32x4_t*)(r);
        g1[u] = *(const f32x4_t*)(r + 4);
        u0[u] = *(const f32x4_t*)(r + 8);
        u1[u] = *(const f32x4_t*)(r + 12);
      }
#pragma unroll
      for (int u = 0; u < B; ++u) {
        u32x4_t pk;
        pk[0] = pack_bf16(silu_mul(g0[u][0], u0[u][0]), silu_mul(g0[u][1], u0[u][1]));
        pk[1] = pack_bf16(silu_mul(g0[u][2], u0[u][2]), silu_mul(g0[u][3], u0[u][3]));
        pk[2] = pack_bf16(silu_mul(g1[u][0], u1[u][0]), silu_mul(g1[u][1], u1[u][1]));
        pk[3] = pack_bf16(silu_mul(g1[u][2], u1[u][2]), silu_mul(g1[u][3], u1[u][3]));
        *(u32x4_t*)(dst + (p0 + u) * step) = pk;
      }
    }
    return;
  }
  if (mode == OUT_BF16) {
    constexpr int LPR = COLS / 8, RPP = 64 / LPR, PASSES = ROWS / RPP, B = PASSES < 4 ? PASSES : 4;
    const int col = (lane % LPR) * 8, rr = lane / LPR;
    const float* src = ct + rr * LD + col;
    bf16_t* dst = (bf16_t*)out + (size_t)(mrow0 + rr) * ldo + ncol0 + col;
    const size_t step = (size_t)RPP * ldo;
#pragma unroll
    for (int p0 = 0; p0 < PASSES; p0 += B) {
      f32x4_t a[B], b[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        a[u] = *(const f32x4_t*)(src + (p0 + u) * RPP * LD);
        b[u] = *(const f32x4_t*)(src + (p0 + u) * RPP * LD + 4);
      }
#pragma unroll
      for (int u = 0; u < B; ++u) {
        u32x4_t pk;
        pk[0] = pack_bf16(a[u][0], a[u][1]);
        pk[1] = pack_bf16(a[u][2], a[u][3]);
        pk[2] = pack_bf16(b[u][0], b[u][1]);
        pk[3] = pack_bf16(b[u][2], b[u][3]);
        *(u32x4_t*)(dst + (p0 + u) * step) = pk;
      }
    }
    return;
  }
  constexpr int LPR = COLS / 4, RPP = 64 / LPR, PASSES = ROWS / RPP, B = PASSES < 4 ? PASSES : 4;
  const int col = (lane % LPR) * 4, rr = lane / LPR;
  const float* src = ct + rr * LD + col;
  float* dst = (float*)out + (size_t)(mrow0 + rr) * ldo + ncol0 + col;
  const size_t step = (size_t)RPP * ldo;
#pragma unroll
  for (int p0 = 0; p0 < PASSES; p0 += B) {
    f32x4_t v[B], old[B];
#pragma unroll
    for (int u = 0; u < B; ++u) v[u] = *(const f32x4_t*)(src + (p0 + u) * RPP * LD);
    if (mode == OUT_ACC_F32) {
#pragma unroll
      for (int u = 0; u < B; ++u) old[u] = *(const f32x4_t*)(dst + (p0 + u) * step);
#pragma unroll
      for (int u = 0; u < B; ++u) *(f32x4_t*)(dst + (p0 + u) * step) = old[u] + v[u];
    } else {
#pragma unroll
      for (int u = 0; u < B; ++u) *(f32x4_t*)(dst + (p0 + u) * step) = v[u];
    }
  }
}

// The q/k/v projection's epilogue (see RopeOut): the wave tile lies inside one head (head_dim is 128, COLS 64 or
// 128).  q and k: a lane takes eight neighbouring columns (four rotary pairs) of a row, rotates them with the
// step's table of cosines and sines and stores 16 bytes of bfloat16, q into [M, heads, head_dim], k into the row
// of its cache place.  v: a lane takes one column for eight consecutive tokens and stores them as one 16-byte
// piece of the transposed value cache when their cache places follow one another from a multiple of eight
// (inside a prompt portion they do), else one by one.
// What the epilogue needs from global memory (cosines and sines, cache places) is fetched by rope_fetch before
// the accumulators go to LDS, so that the loads travel meanwhile; a tile of eight passes at a time.
template <int ROWS, int COLS>
struct RopeFetch {
  static constexpr int LPR = COLS / 8, RPP = 64 / LPR, PASSES = ROWS / RPP;
  static_assert(PASSES == 8 && COLS * (ROWS / 8) == 8 * 64, "eight passes of q/k rows, eight value items per lane");
  f32x4_t c0[8], c1[8];   // q/k: (cos, sin) of this lane's four pairs in the row of pass p
  int slot[8];            // q/k: the row's cache place; v: the first place of item p's eight tokens, -1 when they
                          // form no run, -2 when the item lies past the last row
};

template <int ROWS, int COLS>
__device__ inline void rope_fetch(RopeFetch<ROWS, COLS>& f, int lane, int mrow0, int ncol0, const RopeOut& rp, int M) {
  using F = RopeFetch<ROWS, COLS>;
  const int n0 = rp.col0 + ncol0;
  const int q_dim = rp.n_heads * rp.head_dim, kv_dim = rp.n_kv * rp.head_dim;
  if (n0 >= q_dim + 2 * kv_dim) return;   // (a wave tile past the last column: N need be no multiple of the block's width)
  if (n0 < q_dim + kv_dim) {
    const int col = (lane % F::LPR) * 8, rr = lane / F::LPR;
    const int d = (n0 + col) % rp.head_dim;
    const bool rotate = d < rp.rotary_dim, is_q = n0 < q_dim;
    const int half = rp.rotary_dim >> 1;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int m = min(mrow0 + p * F::RPP + rr, M - 1);
      if (rotate) {
        const f32x4_t* cs = (const f32x4_t*)(rp.cos_sin + (size_t)m * half + (d >> 1));
        f.c0[p] = cs[0];
        f.c1[p] = cs[1];
      }
      f.slot[p] = is_q ? 0 : rp.slots[m];
    }
    return;
  }
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int rg = (lane + 64 * p) / COLS;
    const int m0 = mrow0 + rg * 8;
    int s0 = -2;
    if (m0 < M) {
      s0 = -1;
      if (m0 + 8 <= M) {
        int sl[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) sl[i] = rp.slots[m0 + i];
        // a run: every place follows the one before, or begins a group of eight where that one ended a group
        // (eight tokens in a row of one request, whose next page may lie anywhere); from a multiple of eight it is
        // one piece of the value cache, otherwise the ends of two
        bool run = true;
#pragma unroll
        for (int i = 1; i < 8; ++i) run = run && (sl[i] == sl[i - 1] + 1 || ((sl[i] & 7) == 0 && (sl[i - 1] & 7) == 7));
        if (run) s0 = sl[0];
      }
    }
    f.slot[p] = s0;
  }
}

template <int ROWS, int COLS, int LD>
__device__ inline void emit_tile_rope(const float* ct, int lane, int mrow0, int ncol0, const RopeOut& rp, int M,
                                      const RopeFetch<ROWS, COLS>& f) {
  using F = RopeFetch<ROWS, COLS>;
  const int n0 = rp.col0 + ncol0;                       // first column of the wave tile in the whole projection
  const int q_dim = rp.n_heads * rp.head_dim, kv_dim = rp.n_kv * rp.head_dim;
  if (n0 >= q_dim + 2 * kv_dim) return;                 // a wave tile past the last column
  if (n0 < q_dim + kv_dim) {
    const int col = (lane % F::LPR) * 8, rr = lane / F::LPR;
    const bool is_q = n0 < q_dim;
    const int d = (n0 + col) % rp.head_dim;             // first of this lane's eight elements within its head
    const int kh = is_q ? 0 : (n0 + col - q_dim) / rp.head_dim;   // (a wave tile may span two heads of 64)
    const bool rotate = d < rp.rotary_dim;
    const float* src = ct + rr * LD + col;
#pragma unroll
    for (int p0 = 0; p0 < 8; p0 += 4) {
      f32x4_t a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = *(const f32x4_t*)(src + (p0 + u) * F::RPP * LD);
        b[u] = *(const f32x4_t*)(src + (p0 + u) * F::RPP * LD + 4);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int p = p0 + u;
        const int m = mrow0 + p * F::RPP + rr;
        if (rotate) {
          const f32x4_t c0 = f.c0[p], c1 = f.c1[p];
          float x0, x1;
          x0 = a[u][0]; x1 = a[u][1]; a[u][0] = x0 * c0[0] - x1 * c0[1]; a[u][1] = x0 * c0[1] + x1 * c0[0];
          x0 = a[u][2]; x1 = a[u][3]; a[u][2] = x0 * c0[2] - x1 * c0[3]; a[u][3] = x0 * c0[3] + x1 * c0[2];
          x0 = b[u][0]; x1 = b[u][1]; b[u][0] = x0 * c1[0] - x1 * c1[1]; b[u][1] = x0 * c1[1] + x1 * c1[0];
          x0 = b[u][2]; x1 = b[u][3]; b[u][2] = x0 * c1[2] - x1 * c1[3]; b[u][3] = x0 * c1[3] + x1 * c1[2];
        }
        u32x4_t pk;
        pk[0] = pack_bf16(a[u][0], a[u][1]);
        pk[1] = pack_bf16(a[u][2], a[u][3]);
        pk[2] = pack_bf16(b[u][0], b[u][1]);
        pk[3] = pack_bf16(b[u][2], b[u][3]);
        if (m >= M) continue;
        bf16_t* dst;
        if (is_q) {
          dst = rp.q_out + (size_t)m * q_dim + n0 + col;
        } else {
          const size_t page = (size_t)(f.slot[p] / rp.page_size), off = (size_t)(f.slot[p] % rp.page_size);
          dst = rp.k_cache + ((page * rp.n_kv + kh) * rp.page_size + off) * rp.head_dim + d;
        }
        *(u32x4_t*)dst = pk;
      }
    }
    return;
  }
  // values: COLS columns x ROWS / 8 groups of eight tokens, one (column, group) per lane and pass
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int it = lane + 64 * p;
    const int colv = it % COLS, rg = it / COLS;
    const int kh = (n0 - q_dim - kv_dim + colv) / rp.head_dim;   // this column's head and its place in it
    const int d0 = (n0 - q_dim - kv_dim + colv) % rp.head_dim - colv;
    const int m0 = mrow0 + rg * 8;
    const int s0 = f.slot[p];
    if (s0 == -2) continue;
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = ct[(rg * 8 + i) * LD + colv];
    if (s0 >= 0 && (s0 & 7) == 0) {
      const size_t page = (size_t)(s0 / rp.page_size), off = (size_t)(s0 % rp.page_size);
      u32x4_t pk;
      pk[0] = pack_bf16(y[0], y[1]);
      pk[1] = pack_bf16(y[2], y[3]);
      pk[2] = pack_bf16(y[4], y[5]);
      pk[3] = pack_bf16(y[6], y[7]);
      *(u32x4_t*)(rp.v_cache + ((page * rp.n_kv + kh) * rp.head_dim + d0 + colv) * rp.page_size + off) = pk;
    } else if (s0 >= 0) {
      // a run that starts inside a group of eight places: the end of that group, then the start of the group that
      // holds the next token (two addresses worked out instead of eight)
      const int n0 = 8 - (s0 & 7);
      const int s1 = rp.slots[m0 + n0];
      const size_t page0 = (size_t)(s0 / rp.page_size), off0 = (size_t)(s0 % rp.page_size);
      const size_t page1 = (size_t)(s1 / rp.page_size), off1 = (size_t)(s1 % rp.page_size);
      bf16_t* p0 = rp.v_cache + ((page0 * rp.n_kv + kh) * rp.head_dim + d0 + colv) * rp.page_size + off0;
      bf16_t* p1 = rp.v_cache + ((page1 * rp.n_kv + kh) * rp.head_dim + d0 + colv) * rp.page_size + off1 - n0;
#pragma unroll
      for (int i = 0; i < 8; ++i) (i < n0 ? p0 : p1)[i] = float_to_bf16(y[i]);
    } else {
      for (int i = 0; i < 8 && m0 + i < M; ++i) {
        const int sl = rp.slots[m0 + i];
        const size_t page = (size_t)(sl / rp.page_size), off = (size_t)(sl % rp.page_size);
        rp.v_cache[((page * rp.n_kv + kh) * rp.head_dim + d0 + colv) * rp.page_size + off] = float_to_bf16(y[i]);
      }
    }
  }
}

// A wave's result rows [0, ROWS) x COLS columns, laid out in LDS with rows of LD floats, to memory: rows mrow0..,
// columns ncol0.. of the launch's N (row stride ldo).  Four rows are read from LDS before the first of them is
// stored, so that the reads (and, when adding into `out`, the loads) overlap.
template <int ROWS, int COLS, int LD>
__device__ inline void emit_tile(const float* ct, int lane, int mrow0, int ncol0, void* out, int mode, int M, int N, int ldo) {
  if (mrow0 + ROWS <= M && ncol0 + COLS <= N && ldo % 8 == 0 && ((uintptr_t)out & 15) == 0) {
    emit_tile_fast<ROWS, COLS, LD>(ct, lane, mrow0, ncol0, out, mode, ldo);
    return;
  }
  if (mode == OUT_SWIGLU) {
    // the weight rows alternate eight gate rows and eight up rows: output column 8 b + i pairs columns
    // 16 b + i and 16 b + 8 + i; COLS / 2 outputs per row, four per lane
    constexpr int LPR = COLS / 8, RPP = 64 / LPR, PASSES = ROWS / RPP, B = PASSES < 4 ? PASSES : 4;
    const int o = (lane % LPR) * 4, rr = lane / LPR;
    const int cg = (o / 8) * 16 + o % 8;
    bf16_t* ob = (bf16_t*)out;
    if (ncol0 + cg >= N) return;   // N is a multiple of 16: the whole group is inside or outside
#pragma unroll
    for (int p0 = 0; p0 < PASSES; p0 += B) {
      f32x4_t gt[B], up[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const int row = (p0 + u) * RPP + rr;
        gt[u] = *(const f32x4_t*)(ct + row * LD + cg);
        up[u] = *(const f32x4_t*)(ct + row * LD + cg + 8);
      }
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const int m = mrow0 + (p0 + u) * RPP + rr;
        u32x2_t pk;
        pk[0] = pack_bf16(silu_mul(gt[u][0], up[u][0]), silu_mul(gt[u][1], up[u][1]));
        pk[1] = pack_bf16(silu_mul(gt[u][2], up[u][2]), silu_mul(gt[u][3], up[u][3]));
        if (m < M) *(u32x2_t*)(ob + (size_t)m * ldo + ncol0 / 2 + o) = pk;
      }
    }
    return;
  }
  constexpr int LPR = COLS / 4, RPP = 64 / LPR, PASSES = ROWS / RPP;
  static_assert(PASSES % 4 == 0, "the loop below takes four passes at a time");
  const int col = (lane % LPR) * 4, rr = lane / LPR;
  if (ldo % 4 == 0 && ncol0 + col + 3 < N) {
#pragma unroll
    for (int p0 = 0; p0 < PASSES; p0 += 4) {
      f32x4_t v[4], old[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *(const f32x4_t*)(ct + ((p0 + u) * RPP + rr) * LD + col);
      if (mode == OUT_ACC_F32) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int m = mrow0 + (p0 + u) * RPP + rr;
          old[u] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
          if (m < M) old[u] = *(const f32x4_t*)((const float*)out + (size_t)m * ldo + ncol0 + col);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int m = mrow0 + (p0 + u) * RPP + rr;
        if (m >= M) continue;
        const size_t idx = (size_t)m * ldo + ncol0 + col;
        if (mode == OUT_BF16) {
          u32x2_t pk;
          pk[0] = pack_bf16(v[u][0], v[u][1]);
          pk[1] = pack_bf16(v[u][2], v[u][3]);
          *(u32x2_t*)((bf16_t*)out + idx) = pk;
        } else if (mode == OUT_F32) {
          *(f32x4_t*)((float*)out + idx) = v[u];
        } else {
          *(f32x4_t*)((float*)out + idx) = old[u] + v[u];
        }
      }
    }
    return;
  }
  // the last columns of an N that is no multiple of four, or a row stride that is none: element by element
  for (int p = 0; p < PASSES; ++p) {
    const int row = p * RPP + rr, m = mrow0 + row;
    if (m >= M) continue;
    const size_t idx = (size_t)m * ldo + ncol0 + col;
    for (int e = 0; e < 4; ++e) {
      if (ncol0 + col + e >= N) break;
      const float v = ct[row * LD + col + e];
      if (mode == OUT_BF16)
        ((bf16_t*)out)[idx + e] = float_to_bf16(v);
      else if (mode == OUT_F32)
        ((float*)out)[idx + e] = v;
      else
        ((float*)out)[idx + e] += v;
    }
  }
}

}  // namespace

// Which tile a block takes.  Blocks go to the 8 XCDs in turn and each XCD has an L2 of its own: XCD j takes the
// j-th eighth of the list of tiles, all eighths equally long (with whole column blocks dealt out instead, 255 tiles
// of three row blocks came to 33 on five XCDs of 32 CUs, a second round for one tile each: 170 us instead of 113),
// and the list has no gaps (a block that finds no tile and leaves at once still held up the ones behind it: a
// product with a fifth of such blocks took twice its time).  The list walks groups of pq column blocks; inside a
// group, strips of pm row blocks; inside a strip, row blocks fastest: the 32 blocks that an XCD runs at a time
// share pm row blocks of x and about 32 / pm column blocks of w.  False for the few blocks past the list's end.
__device__ inline bool tile_of_block(unsigned block, int MB, int NB, int pm, int& bm, int& bn) {
  const int total = MB * NB, per = (total + 7) / 8;
  const int item = (int)(block % 8) * per + (int)(block / 8);
  if ((int)(block / 8) >= per || item >= total) return false;
  const int pq = max(1, 32 / pm);
  const int group = MB * pq;
  const int k = item / group, rem = item - k * group;
  const int wk = min(pq, NB - k * pq);
  const int strip = pm * wk;
  const int sidx = rem / strip, r = rem - sidx * strip;
  const int hs = min(pm, MB - sidx * pm);
  bm = sidx * pm + r % hs;
  bn = k * pq + r / hs;
  return true;
}

// ldo: row stride of `out` in elements (N, or N / 2 for the gated mode, when the launch covers all columns;
// a launch may cover a range of columns with `w` and `out` pointing at its first).
// pm: row blocks of a strip (see tile_of_block).  blockIdx.y splits K:
// with more than one split every block writes its float32 partial tile to `partial` [split, M, N]
// and a second kernel adds the splits in ascending order and applies the epilogue.
__global__ __launch_bounds__(256) void gemm_pipe_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                        void* __restrict__ out, float* __restrict__ partial, int mode,
                                                        int M, int N, int K, int pm, int ldo, RopeOut rp, int wt) {
  __shared__ __attribute__((aligned(1024))) unsigned char stages[NS * STAGE_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int bm, bn;
  {
    const int MB = (M + BM - 1) / BM, NB = (N + BN - 1) / BN;
    if (!tile_of_block(blockIdx.x, MB, NB, pm, bm, bn)) return;
  }
  const int m0 = bm * BM, n0 = bn * BN;
  f32x4_t acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  // this block's share of K, in tiles
  const int kt_per = (K / BK + gridDim.y - 1) / gridDim.y;
  const int kt_first = blockIdx.y * kt_per;
  const int KT = min(K / BK, kt_first + kt_per) - kt_first;
  if (gridDim.y > 1) {
    mode = OUT_F32;
    out = partial + (size_t)blockIdx.y * M * N;
    ldo = N;
  }
  const int g = lane >> 4, c = lane & 15;
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)&stages[0];
  // this lane's byte offset inside a 16-row group of a stage, for the first and second 32 of K
  const unsigned off0 = c * ROWB + (((0 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned off1 = c * ROWB + (((1 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned arow = wm * 128 * ROWB, brow = (BM + wn * 64) * ROWB;
  // this lane's source of each of its loads, relative to the block's first row at the stage's k
  unsigned voff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int row = (i < 8 ? (wave * 8 + i) * 8 : (wave * 4 + i - 8) * 8) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int grow = i < 8 ? min(row, M - 1 - m0) : min(row, N - 1 - n0);
    voff[i] = (unsigned)grow * (unsigned)K * 2u + chunk * 16;
    if (wt && i >= 8) {   // block u of the stage's weights: row group u / 2 of the block tile, first or second 32 of k
      const int u = wave * 4 + i - 8;
      const int grp = min(u / 2, (N - n0) / 16 - 1);
      voff[i] = ((unsigned)grp * (unsigned)(K / 32) + (u & 1)) * 1024u + lane * 16;
    }
  }
  const int wkstep = wt ? 2048 : BK * 2;     // bytes from one stage's weights to the next
  const unsigned boff0 = wt ? lane * 16 : off0, boff1 = wt ? 1024 + lane * 16 : off1;
  const unsigned char* xk = (const unsigned char*)x + ((size_t)m0 * K + (size_t)kt_first * BK) * 2;
  const unsigned char* wk = (const unsigned char*)w + (size_t)n0 * K * 2 + (size_t)kt_first * wkstep;
#pragma unroll
  for (int p = 0; p < NS; ++p)
    if (p < KT) issue_stage(stages + p * STAGE_BYTES, xk + p * BK * 2, wk + p * wkstep, voff, wave);
  xk += NS * BK * 2;  // the next stage to load is that of tile NS
  wk += NS * wkstep;
  Frags fa, fb;
  if (KT > 2) WAIT_VM(2 * LPW); else WAIT_VM(0);
  __builtin_amdgcn_s_barrier();
  READ_ALL(fa, lds0 + arow + off0, lds0 + brow + boff0);
  wait_frags(fa);
  // Tile kt: the first half step multiplies fa and reads the second half's fragments; then tile kt + 1
  // must have landed for every wave (barrier), which also means that every wave is done reading tile
  // kt's stage: the second half step refills it with tile kt + NS while it multiplies fb and reads the
  // first fragments of tile kt + 1.
  int st = 0, kt = 0;
  for (; kt + NS < KT; ++kt) {
    const int sn = st + 1 == NS ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE_BYTES, nxt = lds0 + sn * STAGE_BYTES;
    half_step<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags(fb);
    WAIT_VM(LPW);  // tile kt + 2 may stay in flight
    __builtin_amdgcn_s_barrier();
    half_step<true, true>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, stages + st * STAGE_BYTES, xk, wk, voff, wave);
    wait_frags(fa);
    xk += BK * 2;
    wk += wkstep;
    st = sn;
  }
  for (; kt + 1 < KT; ++kt) {  // nothing left to load
    const int sn = st + 1 == NS ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE_BYTES, nxt = lds0 + sn * STAGE_BYTES;
    half_step<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags(fb);
    WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    half_step<true, false>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, nullptr, nullptr, nullptr, voff, wave);
    wait_frags(fa);
    st = sn;
  }
  {
    const unsigned cur = lds0 + st * STAGE_BYTES;
    half_step<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags(fb);
    half_step<false, false>(acc, fb, fa, 0, 0, nullptr, nullptr, nullptr, voff, wave);
  }

  // ---- the result leaves through LDS: each wave lays its 128 x 64 tile out row by row -----------------
  __syncthreads();  // every wave is done with the stages
  float* ct = (float*)stages + wave * (128 * CLD);
  RopeFetch<64, 64> fetched;   // (the rotating epilogue's loads travel while the tile goes to LDS)
  if (mode == OUT_ROPE) rope_fetch(fetched, lane, m0 + wm * 128, n0 + wn * 64, rp, M);
  // result lane l of tile (i, j): rows i * 16 + (l / 16) * 4 + r, column j * 16 + l % 16
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLD + j * 16 + c] = acc[i][j][r];
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave's LDS writes before its reads
  if (mode == OUT_ROPE) {
    emit_tile_rope<64, 64, CLD>(ct, lane, m0 + wm * 128, n0 + wn * 64, rp, M, fetched);
    rope_fetch(fetched, lane, m0 + wm * 128 + 64, n0 + wn * 64, rp, M);
    emit_tile_rope<64, 64, CLD>(ct + 64 * CLD, lane, m0 + wm * 128 + 64, n0 + wn * 64, rp, M, fetched);
  } else {
    emit_tile<128, 64, CLD>(ct, lane, m0 + wm * 128, n0 + wn * 64, out, mode, M, N, ldo);
  }
}

// ---- 256 x 256 block tiles ---------------------------------------------------------------------------
// What bounds the kernel above is the operand traffic from L2 into LDS (48 KB per 64 of K and CU, three
// quarters of what the path delivers at the full MFMA rate).  A 256 x 256 block tile (a wave owns 128 x 128,
// 256 accumulator registers) needs 64 KB for twice the work.  Two stages of (256 + 256) rows x 128 bytes
// (128 KB); the pipeline is the same: fragments of the next half step and the loads of the tile after next
// between the MFMAs of this half step, one barrier per 64 of K.  Used where whole rounds of such tiles fill
// the CUs; the columns that are left go to the kernel above.
namespace {

constexpr int BNB = 256, NSB = 2;
constexpr int CLDB = 128 + 4;   // padded row of a quarter (32 rows) of a wave's result tile in LDS, in floats
constexpr int CLDS = 32 + 4;    // padded row of a strip (32 columns) of a wave's result tile in LDS, in floats

// Operand fragments of a half step (32 of K): eight 16-row tiles of x, NJ (eight or six) of w.  The w fragments
// are double-buffered, and so are the last two x fragments; x fragments 0..5 are used by one row of MFMAs each,
// so the next half step's takes the register as soon as that row has been issued (the LDS read takes far
// longer than an MFMA needs to fetch its operands).
template <int NJ>
struct FragsBig {
  u32x4_t a[6], a6[2], a7[2], b[2][NJ];
};
template <int NJ, int p>
__device__ inline void tie_frags(FragsBig<NJ>& f) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(f.b[p][0]), "+v"(f.b[p][1]), "+v"(f.b[p][2]), "+v"(f.b[p][3]), "+v"(f.b[p][4]), "+v"(f.b[p][5]),
                 "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.a[4]), "+v"(f.a[5]), "+v"(f.a6[p]),
                 "+v"(f.a7[p]));
  if constexpr (NJ == 8) asm volatile("" : "+v"(f.b[p][6]), "+v"(f.b[p][7]));
}
// load I (0..7 + NJ) of this wave into stage `buf`: 0..7 are x rows, the others w rows; one load covers 8 rows
template <int I, int NJ>
__device__ inline void issue_big(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                 const unsigned (&voff)[8 + NJ], int wave) {
  if constexpr (I < 8 + NJ) {
    const int t = I < 8 ? wave * 8 + I : 32 + wave * NJ + (I - 8);
    load_lds16(I < 8 ? xk : wk, voff[I], buf + t * 1024);
  }
}
template <int NJ>
__device__ inline void issue_stage_big(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                       const unsigned (&voff)[8 + NJ], int wave) {
  issue_big<0, NJ>(buf, xk, wk, voff, wave); issue_big<1, NJ>(buf, xk, wk, voff, wave); issue_big<2, NJ>(buf, xk, wk, voff, wave);
  issue_big<3, NJ>(buf, xk, wk, voff, wave); issue_big<4, NJ>(buf, xk, wk, voff, wave); issue_big<5, NJ>(buf, xk, wk, voff, wave);
  issue_big<6, NJ>(buf, xk, wk, voff, wave); issue_big<7, NJ>(buf, xk, wk, voff, wave); issue_big<8, NJ>(buf, xk, wk, voff, wave);
  issue_big<9, NJ>(buf, xk, wk, voff, wave); issue_big<10, NJ>(buf, xk, wk, voff, wave); issue_big<11, NJ>(buf, xk, wk, voff, wave);
  issue_big<12, NJ>(buf, xk, wk, voff, wave); issue_big<13, NJ>(buf, xk, wk, voff, wave); issue_big<14, NJ>(buf, xk, wk, voff, wave);
  issue_big<15, NJ>(buf, xk, wk, voff, wave);
}
// The 8 x NJ MFMAs of a half step with the fragments of parity P, row by row.  READ: the next half step's
// fragments are requested between them (w and the last two x fragments into the other set, x fragment i into
// a[i] after row i).  LOAD: one global load per group of MFMAs.
template <int P, bool READ, bool LOAD, int NJ>
__device__ inline void half_step_big(f32x4_t (&acc)[8][NJ], FragsBig<NJ>& f, unsigned aaddr, unsigned baddr, unsigned char* buf,
                                     const unsigned char* xk, const unsigned char* wk, const unsigned (&voff)[8 + NJ],
                                     int wave) {
#define SB() __builtin_amdgcn_sched_barrier(0)
#define AF(I) (I < 6 ? f.a[I < 6 ? I : 0] : (I == 6 ? f.a6[P] : f.a7[P]))
// (written as assembly with the accumulator tied to an AGPR: left to itself the register allocator keeps
// part of the accumulator registers in VGPRs and copies them back and forth inside the loop)
#define M1(I, J) \
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[I][J]) : "v"(AF(I)), "v"(f.b[P][J])); \
  SB()
#define RB(J) \
  if (READ) f.b[P ^ 1][J] = lds_read16<(J) * 16 * ROWB>(baddr); \
  SB()
#define RA(I) \
  if (READ) f.a[I] = lds_read16<(I) * 16 * ROWB>(aaddr); \
  SB()
#define R67()                                                  \
  if (READ) f.a6[P ^ 1] = lds_read16<6 * 16 * ROWB>(aaddr);    \
  SB();                                                        \
  if (READ) f.a7[P ^ 1] = lds_read16<7 * 16 * ROWB>(aaddr);    \
  SB()
#define LD(G) \
  if (LOAD) issue_big<G, NJ>(buf, xk, wk, voff, wave); \
  SB()
  if constexpr (NJ == 8) {
#define ROW(I, PRE0, PRE1)                             \
  PRE0;                                                \
  M1(I, 0); M1(I, 1); LD(2 * (I)); M1(I, 2); M1(I, 3); \
  PRE1;                                                \
  M1(I, 4); M1(I, 5); LD(2 * (I) + 1); M1(I, 6); M1(I, 7)
    ROW(0, RB(0), RB(1));
    ROW(1, RB(2); RA(0), RB(3));
    ROW(2, RB(4); RA(1), RB(5));
    ROW(3, RB(6); RA(2), RB(7));
    ROW(4, RA(3), R67());
    ROW(5, RA(4), (void)0);
    ROW(6, RA(5), (void)0);
    ROW(7, (void)0, (void)0);
#undef ROW
  } else {
    static_assert(NJ == 6 || NJ == 8, "w tiles per wave");
#define ROW(I, PRE0, PRE1)                   \
  PRE0;                                      \
  M1(I, 0); M1(I, 1); LD(2 * (I)); M1(I, 2); \
  PRE1;                                      \
  M1(I, 3); M1(I, 4); LD(2 * (I) + 1); M1(I, 5)
    ROW(0, RB(0), RB(1));
    ROW(1, RB(2); RA(0), RB(3));
    ROW(2, RB(4); RA(1), RB(5));
    ROW(3, RA(2), (void)0);
    ROW(4, RA(3), R67());
    ROW(5, RA(4), (void)0);
    ROW(6, RA(5), (void)0);
    ROW(7, (void)0, (void)0);
#undef ROW
  }
  if (READ) {
    tie_frags<NJ, (P ^ 1)>(f);
    SB();
  }
#undef LD
#undef R67
#undef RA
#undef RB
#undef M1
#undef AF
#undef SB
}
template <int NJ>
__device__ inline void read_all_big(FragsBig<NJ>& f, unsigned aaddr, unsigned baddr) {
#define RB0(J) if constexpr (J < NJ) f.b[0][J < NJ ? J : 0] = lds_read16<(J) * 16 * ROWB>(baddr)
#define RA0(I) f.a[I] = lds_read16<(I) * 16 * ROWB>(aaddr)
  RB0(0); RB0(1); RB0(2); RB0(3); RB0(4); RB0(5); RB0(6); RB0(7);
  RA0(0); RA0(1); RA0(2); RA0(3); RA0(4); RA0(5);
  f.a6[0] = lds_read16<6 * 16 * ROWB>(aaddr);
  f.a7[0] = lds_read16<7 * 16 * ROWB>(aaddr);
#undef RB0
#undef RA0
  tie_frags<NJ, 0>(f);
}

}  // namespace

// No split of K here.  A block tile is 256 rows x 32 NJ columns (NJ = 8: 256, a wave owns 128 x 128; NJ = 6: 192, a
// wave owns 128 x 96: for an N where that many more tiles make whole rounds of the CUs).  N: the columns of this
// launch (a multiple of the tile's); ldo as above.
template <int NJ>
__global__ __launch_bounds__(256) void gemm_pipe_big_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                            void* __restrict__ out, int mode, int M, int N, int K,
                                                            int pm, int ldo, RopeOut rp, int wt) {
  constexpr int BNT = 32 * NJ, WN = 16 * NJ, STAGE = (BM + BNT) * ROWB, LPWT = 8 + NJ;
  __shared__ __attribute__((aligned(1024))) unsigned char stages[NSB * STAGE];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int bm, bn;
  {
    const int MB = (M + BM - 1) / BM, NB = N / BNT;
    if (!tile_of_block(blockIdx.x, MB, NB, pm, bm, bn)) return;
  }
  const int m0 = bm * BM, n0 = bn * BNT;
  f32x4_t acc[8][NJ];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const int KT = K / BK;
  const int g = lane >> 4, c = lane & 15;
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)&stages[0];
  const unsigned off0 = c * ROWB + (((0 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned off1 = c * ROWB + (((1 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned arow = wm * 128 * ROWB, brow = (BM + wn * WN) * ROWB;
  unsigned voff[LPWT];
#pragma unroll
  for (int i = 0; i < LPWT; ++i) {
    const int row = (i < 8 ? wave * 8 + i : wave * NJ + (i - 8)) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int grow = i < 8 ? min(row, M - 1 - m0) : row;   // (every w row of the launch exists)
    voff[i] = (unsigned)grow * (unsigned)K * 2u + chunk * 16;
    if (wt && i >= 8) {   // block u of the stage's weights: row group u / 2 of the block tile, first or second 32 of k
      const int u = wave * NJ + (i - 8);
      voff[i] = ((unsigned)(u / 2) * (unsigned)(K / 32) + (u & 1)) * 1024u + lane * 16;
    }
  }
  const int wkstep = wt ? 2048 : BK * 2;
  const unsigned boff0 = wt ? lane * 16 : off0, boff1 = wt ? 1024 + lane * 16 : off1;
  const unsigned char* xk = (const unsigned char*)x + (size_t)m0 * K * 2;
  const unsigned char* wk = (const unsigned char*)w + (size_t)n0 * K * 2;
#pragma unroll
  for (int p = 0; p < NSB; ++p)
    if (p < KT) issue_stage_big<NJ>(stages + p * STAGE, xk + p * BK * 2, wk + p * wkstep, voff, wave);
  xk += NSB * BK * 2;
  wk += NSB * wkstep;
  FragsBig<NJ> f;
  if (KT > 1) WAIT_VM(LPWT); else WAIT_VM(0);
  __builtin_amdgcn_s_barrier();
  read_all_big<NJ>(f, lds0 + arow + off0, lds0 + brow + boff0);
  // Tile kt: the first half step multiplies the fragments of its first 32 of K and reads those of the second;
  // then tile kt + 1 must have landed for every wave (barrier), which also means that every wave is done
  // reading tile kt's stage: the second half step refills it with tile kt + 2 while it multiplies and reads
  // the first fragments of tile kt + 1.
  int st = 0, kt = 0;
  for (; kt + NSB < KT; ++kt) {
    const unsigned cur = lds0 + st * STAGE, nxt = lds0 + (st ^ 1) * STAGE;
    half_step_big<0, true, false, NJ>(acc, f, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    half_step_big<1, true, true, NJ>(acc, f, nxt + arow + off0, nxt + brow + boff0, stages + st * STAGE, xk, wk, voff, wave);
    xk += BK * 2;
    wk += wkstep;
    st ^= 1;
  }
  for (; kt + 1 < KT; ++kt) {  // nothing left to load
    const unsigned cur = lds0 + st * STAGE, nxt = lds0 + (st ^ 1) * STAGE;
    half_step_big<0, true, false, NJ>(acc, f, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    half_step_big<1, true, false, NJ>(acc, f, nxt + arow + off0, nxt + brow + boff0, nullptr, nullptr, nullptr, voff, wave);
    st ^= 1;
  }
  {
    const unsigned cur = lds0 + st * STAGE;
    half_step_big<0, true, false, NJ>(acc, f, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    half_step_big<1, false, false, NJ>(acc, f, 0, 0, nullptr, nullptr, nullptr, voff, wave);
  }
  // The MFMAs are assembly, so the compiler does not know that their results take time: wait out the last ones
  // (eight passes of the matrix core and the write-back).  The wait is tied to their accumulators, or the
  // compiler may read them (a register copy on the way into the epilogue) before it.
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15"
               : "+a"(acc[7][0]), "+a"(acc[7][1]), "+a"(acc[7][2]), "+a"(acc[7][3]), "+a"(acc[7][4]), "+a"(acc[7][5])
               :
               : "memory");
  if constexpr (NJ == 8) asm volatile("" : "+a"(acc[7][6]), "+a"(acc[7][7]));
  // (and every other accumulator passes through an ordered statement after it)
#pragma unroll
  for (int i = 0; i < 7; ++i) {
    asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]), "+a"(acc[i][5]));
    if constexpr (NJ == 8) asm volatile("" : "+a"(acc[i][6]), "+a"(acc[i][7]));
  }

  __syncthreads();
  const int mw = m0 + wm * 128, nw = n0 + wn * WN;
  if constexpr (NJ == 8) {
  // ---- the result leaves through LDS, 32 rows of the wave's 128 x 128 at a time ---------------------------
  float* ct = (float*)stages + wave * (32 * CLDB);
  // (written out four times: were the loop over the quarters not unrolled, the accumulators would be indexed at
  // run time and live in scratch memory)
#define QUARTER(Q)                                                                                              \
  {                                                                                                             \
    RopeFetch<32, 128> fetched;   /* the rotating epilogue's loads travel while the quarter goes to LDS */       \
    if (mode == OUT_ROPE) rope_fetch(fetched, lane, mw + (Q) * 32, nw, rp, M);                                  \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) _Pragma("unroll") for (int j = 0; j < 8; ++j)                 \
        _Pragma("unroll") for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLDB + j * 16 + c] = acc[(Q) * 2 + i][j][r]; \
    /* this wave's LDS writes before its reads, and the reverse below */                                        \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
    if (mode == OUT_ROPE)                                                                                       \
      emit_tile_rope<32, 128, CLDB>(ct, lane, mw + (Q) * 32, nw, rp, M, fetched);                               \
    else                                                                                                        \
      emit_tile<32, 128, CLDB>(ct, lane, mw + (Q) * 32, nw, out, mode, M, N, ldo);                              \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
  }
  QUARTER(0)
  QUARTER(1)
  QUARTER(2)
  QUARTER(3)
#undef QUARTER
  } else {
  // ---- the wave's 128 x 96 leaves as a strip of 64 columns (two halves of 64 rows) and one of 32.  A strip
  // must lie inside one head of the q/k/v projection (heads of 128 begin at multiples of 128): the wave's first
  // column is 0, 32, 64 or 96 past such a multiple, and only from 96 the strip of 32 has to come first.  (Both
  // orders are written out: the accumulators are indexed by constants only.) -----------------------------------
  float* ct = (float*)stages + wave * (128 * CLDS);
#define STRIP32(JB)                                                                                             \
  {                                                                                                             \
    RopeFetch<128, 32> fetched;                                                                                 \
    if (mode == OUT_ROPE) rope_fetch(fetched, lane, mw, nw + (JB) * 16, rp, M);                                 \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) _Pragma("unroll") for (int j = 0; j < 2; ++j)                 \
        _Pragma("unroll") for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLDS + j * 16 + c] = acc[i][(JB) + j][r]; \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
    if (mode == OUT_ROPE)                                                                                       \
      emit_tile_rope<128, 32, CLDS>(ct, lane, mw, nw + (JB) * 16, rp, M, fetched);                              \
    else                                                                                                        \
      emit_tile<128, 32, CLDS>(ct, lane, mw, nw + (JB) * 16, out, mode, M, N, ldo);                             \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
  }
#define STRIP64(JB, H)                                                                                          \
  {                                                                                                             \
    RopeFetch<64, 64> fetched;                                                                                  \
    if (mode == OUT_ROPE) rope_fetch(fetched, lane, mw + (H) * 64, nw + (JB) * 16, rp, M);                      \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) _Pragma("unroll") for (int j = 0; j < 4; ++j)                 \
        _Pragma("unroll") for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLD + j * 16 + c] = acc[(H) * 4 + i][(JB) + j][r]; \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
    if (mode == OUT_ROPE)                                                                                       \
      emit_tile_rope<64, 64, CLD>(ct, lane, mw + (H) * 64, nw + (JB) * 16, rp, M, fetched);                     \
    else                                                                                                        \
      emit_tile<64, 64, CLD>(ct, lane, mw + (H) * 64, nw + (JB) * 16, out, mode, M, N, ldo);                    \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                          \
  }
  static_assert(128 * CLDS >= 64 * CLD, "room for either strip");
  if ((rp.col0 + nw) % 128 == 96) {
    STRIP32(0)
    STRIP64(2, 0)
    STRIP64(2, 1)
  } else {
    STRIP64(0, 0)
    STRIP64(0, 1)
    STRIP32(4)
  }
#undef STRIP64
#undef STRIP32
  }
}

// ---- the same pipeline for 17..64 rows (it takes up to 128) -----------------------------------------------------------
// Here the weights are the traffic and the matrix core has little to do: a block owns 64 x 128 of the
// result (a wave 32 x 64), three stages of (64 + 128) rows (72 KB: two blocks per CU), K split over
// blockIdx.y until there are about two blocks for every CU.  Loads, LDS reads and MFMAs interleave as above.
// NJ = 2 instead of 4: 64 x 64 blocks (a wave 32 x 32, 48 KB of stages), for products whose N gives too few blocks
// of 128 columns to put one on every CU without cutting K into short pieces.
namespace {

constexpr int BM64 = 64;

template <int NJ>
struct Frags64 {
  u32x4_t a[2], b[NJ];
};
template <int NJ>
__device__ inline void wait_frags(Frags64<NJ>& f) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.b[0]), "+v"(f.b[1]));
  if constexpr (NJ == 4) asm volatile("" : "+v"(f.b[2]), "+v"(f.b[3]));
}
// read R of a half step: the NJ w fragments, then the two x fragments
template <int R, int NJ>
__device__ inline void read_one(Frags64<NJ>& f, unsigned aaddr, unsigned baddr) {
  if constexpr (R < NJ)
    f.b[R] = lds_read16<R * 16 * ROWB>(baddr);
  else
    f.a[R - NJ] = lds_read16<(R - NJ) * 16 * ROWB>(aaddr);
}
// load I (0..1 + NJ) of this wave: 0..1 are x rows, the others w rows
template <int I, int NJ>
__device__ inline void issue_one64(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                   const unsigned (&voff)[2 + NJ], int wave) {
  const int t = I < 2 ? wave * 2 + I : 8 + wave * NJ + (I - 2);
  // (the weights are read once per step: nontemporal, aux bit 1; the few activation rows stay cached)
  load_lds16<(I < 2 ? 0 : 2)>(I < 2 ? xk : wk, voff[I], buf + t * 1024);
}
template <bool READ, bool LOAD, int NJ>
__device__ inline void half_step64(f32x4_t (&acc)[2][NJ], const Frags64<NJ>& cur, Frags64<NJ>& nxt, unsigned aaddr, unsigned baddr,
                                   unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                   const unsigned (&voff)[2 + NJ], int wave) {
#define SB() __builtin_amdgcn_sched_barrier(0)
#define RD(R) \
  if (READ) read_one<R, NJ>(nxt, aaddr, baddr); \
  SB()
#define LD(I) \
  if (LOAD) issue_one64<I, NJ>(buf, xk, wk, voff, wave); \
  SB()
#define M1(I, J) \
  acc[I][J] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(cur.a[I]), as_frag(cur.b[J]), acc[I][J], 0, 0, 0); \
  SB()
  if constexpr (NJ == 4) {
    RD(0); M1(0, 0); LD(0); RD(1); M1(0, 1); LD(1); RD(2); M1(0, 2); LD(2); RD(3); M1(0, 3); LD(3);
    RD(4); M1(1, 0); LD(4); RD(5); M1(1, 1); LD(5); M1(1, 2); M1(1, 3);
  } else {
    static_assert(NJ == 2 || NJ == 4, "w tiles per wave");
    RD(0); M1(0, 0); LD(0); RD(1); M1(0, 1); LD(1);
    RD(2); M1(1, 0); LD(2); RD(3); M1(1, 1); LD(3);
  }
#undef RD
#undef LD
#undef M1
#undef SB
}

}  // namespace

template <int NJ>
__global__ __launch_bounds__(256, 2) void gemm_pipe64_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                             void* __restrict__ out, float* __restrict__ partial,
                                                             int mode, int M, int N, int K, int wt) {
  constexpr int BNT = 32 * NJ, STAGE = (BM64 + BNT) * ROWB, LPWT = 2 + NJ;
  __shared__ __attribute__((aligned(1024))) unsigned char stages[NS * STAGE];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int MB = (M + BM64 - 1) / BM64;
  const int bm = blockIdx.x % MB, bn = blockIdx.x / MB;     // the row blocks of a column block run side by side
  const int m0 = bm * BM64, n0 = bn * BNT;
  f32x4_t acc[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const int kt_per = (K / BK + gridDim.y - 1) / gridDim.y;
  const int kt_first = blockIdx.y * kt_per;
  const int KT = min(K / BK, kt_first + kt_per) - kt_first;
  if (partial != nullptr) {   // K is split, or the caller adds the (single) partial sum itself
    mode = OUT_F32;
    out = partial + (size_t)blockIdx.y * M * N;
  }
  const int g = lane >> 4, c = lane & 15;
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)&stages[0];
  const unsigned off0 = c * ROWB + (((0 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned off1 = c * ROWB + (((1 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned arow = wm * 32 * ROWB, brow = (BM64 + wn * 16 * NJ) * ROWB;
  unsigned voff[LPWT];
#pragma unroll
  for (int i = 0; i < LPWT; ++i) {
    const int row = (i < 2 ? (wave * 2 + i) * 8 : (wave * NJ + i - 2) * 8) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int grow = i < 2 ? min(row, M - 1 - m0) : min(row, N - 1 - n0);
    voff[i] = (unsigned)grow * (unsigned)K * 2u + chunk * 16;
    if (wt && i >= 2) {   // block u of the stage's weights: row group u / 2 of the block tile, first or second 32 of k
      const int u = wave * NJ + i - 2;
      const int grp = min(u / 2, (N - n0) / 16 - 1);
      voff[i] = ((unsigned)grp * (unsigned)(K / 32) + (u & 1)) * 1024u + lane * 16;
    }
  }
  const int wkstep = wt ? 2048 : BK * 2;
  const unsigned boff0 = wt ? lane * 16 : off0, boff1 = wt ? 1024 + lane * 16 : off1;
  const unsigned char* xk = (const unsigned char*)x + ((size_t)m0 * K + (size_t)kt_first * BK) * 2;
  const unsigned char* wk = (const unsigned char*)w + (size_t)n0 * K * 2 + (size_t)kt_first * wkstep;
  auto issue_stage64 = [&](unsigned char* buf, const unsigned char* xs, const unsigned char* ws) {
    issue_one64<0, NJ>(buf, xs, ws, voff, wave);
    issue_one64<1, NJ>(buf, xs, ws, voff, wave);
    issue_one64<2, NJ>(buf, xs, ws, voff, wave);
    issue_one64<3, NJ>(buf, xs, ws, voff, wave);
    if constexpr (NJ == 4) {
      issue_one64<4, NJ>(buf, xs, ws, voff, wave);
      issue_one64<5, NJ>(buf, xs, ws, voff, wave);
    }
  };
#pragma unroll
  for (int p = 0; p < NS; ++p)
    if (p < KT) issue_stage64(stages + p * STAGE, xk + p * BK * 2, wk + p * wkstep);
  xk += NS * BK * 2;
  wk += NS * wkstep;
  Frags64<NJ> fa, fb;
  if (KT > 2) WAIT_VM(2 * LPWT); else WAIT_VM(0);
  __builtin_amdgcn_s_barrier();
  auto read_all = [&](Frags64<NJ>& f, unsigned aaddr, unsigned baddr) {
    read_one<0, NJ>(f, aaddr, baddr); read_one<1, NJ>(f, aaddr, baddr); read_one<2, NJ>(f, aaddr, baddr);
    read_one<3, NJ>(f, aaddr, baddr);
    if constexpr (NJ == 4) {
      read_one<4, NJ>(f, aaddr, baddr); read_one<5, NJ>(f, aaddr, baddr);
    }
  };
  read_all(fa, lds0 + arow + off0, lds0 + brow + boff0);
  wait_frags<NJ>(fa);
  int st = 0, kt = 0;
  for (; kt + NS < KT; ++kt) {
    const int sn = st + 1 == NS ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE, nxt = lds0 + sn * STAGE;
    half_step64<true, false, NJ>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags<NJ>(fb);
    WAIT_VM(LPWT);
    __builtin_amdgcn_s_barrier();
    half_step64<true, true, NJ>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, stages + st * STAGE, xk, wk, voff, wave);
    wait_frags<NJ>(fa);
    xk += BK * 2;
    wk += wkstep;
    st = sn;
  }
  for (; kt + 1 < KT; ++kt) {
    const int sn = st + 1 == NS ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE, nxt = lds0 + sn * STAGE;
    half_step64<true, false, NJ>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags<NJ>(fb);
    WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    half_step64<true, false, NJ>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, nullptr, nullptr, nullptr, voff, wave);
    wait_frags<NJ>(fa);
    st = sn;
  }
  {
    const unsigned cur = lds0 + st * STAGE;
    half_step64<true, false, NJ>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags<NJ>(fb);
    half_step64<false, false, NJ>(acc, fb, fa, 0, 0, nullptr, nullptr, nullptr, voff, wave);
  }
  // the result leaves through LDS, as above: 32 x 16 NJ per wave
  __syncthreads();
  float* ct = (float*)stages + wave * (32 * CLD);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLD + j * 16 + c] = acc[i][j][r];
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  emit_tile<32, 16 * NJ, CLD>(ct, lane, m0 + wm * 32, n0 + wn * 16 * NJ, out, mode, M, N, mode == OUT_SWIGLU ? N / 2 : N);
}

// ---- the same pipeline on 128 x 128 blocks ------------------------------------------------------------
// For steps of a few hundred rows (a prompt portion of 512) times a narrow weight: 256 x 128 blocks then make
// fewer than 128 tiles, K has to be split over blocks, and a kernel has to add the partial sums.  Here a block
// owns 128 x 128 (a wave 64 x 64: sixteen MFMAs per eight fragment reads), three stages of (128 + 128) rows
// (96 KB).  The row blocks of a column block run side by side (they share its weights in L2); K is split only when
// even these tiles are too few.  Epilogues as above, the rotating one included (a wave's 64 columns lie in one head).
namespace {

constexpr int BM128 = 128, BN128 = 128, STAGE128 = (BM128 + BN128) * ROWB, LPW128 = 8;
// five stages of 32 KB: a step of 128 x 128 x 64 is short (512 cycles of MFMA a wave), and a load has to be four
// steps ahead to have arrived from L2 when its turn comes
constexpr int NS128 = 5;

struct Frags128 {
  u32x4_t a[4], b[4];
};
__device__ inline void wait_frags128(Frags128& f) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3]));
}
// read R (0..7) of a half step: the four w fragments, then the four x fragments
template <int R>
__device__ inline void read_one128(Frags128& f, unsigned aaddr, unsigned baddr) {
  if constexpr (R < 4)
    f.b[R] = lds_read16<R * 16 * ROWB>(baddr);
  else
    f.a[R - 4] = lds_read16<(R - 4) * 16 * ROWB>(aaddr);
}
// load I (0..7) of this wave: 0..3 are x rows, 4..7 w rows; one load covers 8 rows
template <int I>
__device__ inline void issue_one128(unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                    const unsigned (&voff)[LPW128], int wave) {
  const int t = I < 4 ? wave * 4 + I : 16 + wave * 4 + (I - 4);
  load_lds16(I < 4 ? xk : wk, voff[I], buf + t * 1024);
}
template <bool READ, bool LOAD>
__device__ inline void half_step128(f32x4_t (&acc)[4][4], const Frags128& cur, Frags128& nxt, unsigned aaddr, unsigned baddr,
                                    unsigned char* buf, const unsigned char* xk, const unsigned char* wk,
                                    const unsigned (&voff)[LPW128], int wave) {
#define SB() __builtin_amdgcn_sched_barrier(0)
#define RD(R) \
  if (READ) read_one128<R>(nxt, aaddr, baddr); \
  SB()
#define LD(I) \
  if (LOAD) issue_one128<I>(buf, xk, wk, voff, wave); \
  SB()
// (assembly with the accumulator as an AGPR operand that is read and written in place: left to the compiler,
// the sixteen accumulators were moved between register files around every MFMA)
#define M1(I, J) \
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[I][J]) : "v"(cur.a[I]), "v"(cur.b[J])); \
  SB()
  RD(0); M1(0, 0); LD(0); RD(1); M1(0, 1); LD(1); RD(2); M1(0, 2); LD(2); RD(3); M1(0, 3); LD(3);
  RD(4); M1(1, 0); LD(4); RD(5); M1(1, 1); LD(5); RD(6); M1(1, 2); LD(6); RD(7); M1(1, 3); LD(7);
  M1(2, 0); M1(2, 1); M1(2, 2); M1(2, 3); M1(3, 0); M1(3, 1); M1(3, 2); M1(3, 3);
#undef RD
#undef LD
#undef M1
#undef SB
}

}  // namespace

__global__ __launch_bounds__(256) void gemm_pipe128_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                           void* __restrict__ out, float* __restrict__ partial, int mode,
                                                           int M, int N, int K, int ldo, RopeOut rp, int wt, int splits) {
  __shared__ __attribute__((aligned(1024))) unsigned char stages[NS128 * STAGE128];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  // Blocks go to the 8 XCDs in turn, and each XCD has an L2 of its own: XCD j takes the j-th eighth of the list
  // of (part of K, column block, row block), row blocks fastest, so that what it holds at a time is a few column
  // blocks of the weights and the rows of x over one part of K, and the weights cross the fabric once.
  const int MB = (M + BM128 - 1) / BM128;
  const int tiles = MB * ((N + BN128 - 1) / BN128);
  const int total = tiles * splits;
  const int per_xcd = (total + 7) / 8;
  const int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || item >= total) return;
  const int split = item / tiles, tile = item - split * tiles;
  const int bm = tile % MB, bn = tile / MB;
  const int m0 = bm * BM128, n0 = bn * BN128;
  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const int kt_per = (K / BK + splits - 1) / splits;
  const int kt_first = split * kt_per;
  const int KT = min(K / BK, kt_first + kt_per) - kt_first;
  if (partial != nullptr) {   // K is split: float32 partial sums, added by a kernel of their own
    mode = OUT_F32;
    out = partial + (size_t)split * M * N;
    ldo = N;
  }
  const int g = lane >> 4, c = lane & 15;
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)&stages[0];
  const unsigned off0 = c * ROWB + (((0 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned off1 = c * ROWB + (((1 * 4 + g) ^ ((c >> 1) & 7)) << 4);
  const unsigned arow = wm * 64 * ROWB, brow = (BM128 + wn * 64) * ROWB;
  unsigned voff[LPW128];
#pragma unroll
  for (int i = 0; i < LPW128; ++i) {
    const int row = (wave * 4 + (i & 3)) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int grow = i < 4 ? min(row, M - 1 - m0) : min(row, N - 1 - n0);
    voff[i] = (unsigned)grow * (unsigned)K * 2u + chunk * 16;
    if (wt && i >= 4) {   // block u of the stage's weights: row group u / 2 of the block tile, first or second 32 of k
      const int u = wave * 4 + (i - 4);
      const int grp = min(u / 2, (N - n0) / 16 - 1);
      voff[i] = ((unsigned)grp * (unsigned)(K / 32) + (u & 1)) * 1024u + lane * 16;
    }
  }
  const int wkstep = wt ? 2048 : BK * 2;
  const unsigned boff0 = wt ? lane * 16 : off0, boff1 = wt ? 1024 + lane * 16 : off1;
  const unsigned char* xk = (const unsigned char*)x + ((size_t)m0 * K + (size_t)kt_first * BK) * 2;
  const unsigned char* wk = (const unsigned char*)w + (size_t)n0 * K * 2 + (size_t)kt_first * wkstep;
  auto issue_stage = [&](unsigned char* buf, const unsigned char* xs, const unsigned char* ws) {
    issue_one128<0>(buf, xs, ws, voff, wave); issue_one128<1>(buf, xs, ws, voff, wave);
    issue_one128<2>(buf, xs, ws, voff, wave); issue_one128<3>(buf, xs, ws, voff, wave);
    issue_one128<4>(buf, xs, ws, voff, wave); issue_one128<5>(buf, xs, ws, voff, wave);
    issue_one128<6>(buf, xs, ws, voff, wave); issue_one128<7>(buf, xs, ws, voff, wave);
  };
#pragma unroll
  for (int p = 0; p < NS128; ++p)
    if (p < KT) issue_stage(stages + p * STAGE128, xk + p * BK * 2, wk + p * wkstep);
  xk += NS128 * BK * 2;
  wk += NS128 * wkstep;
  Frags128 fa, fb;
  if (KT >= NS128) WAIT_VM((NS128 - 1) * LPW128); else WAIT_VM(0);
  __builtin_amdgcn_s_barrier();
  auto read_all = [&](Frags128& f, unsigned aaddr, unsigned baddr) {
    read_one128<0>(f, aaddr, baddr); read_one128<1>(f, aaddr, baddr); read_one128<2>(f, aaddr, baddr);
    read_one128<3>(f, aaddr, baddr); read_one128<4>(f, aaddr, baddr); read_one128<5>(f, aaddr, baddr);
    read_one128<6>(f, aaddr, baddr); read_one128<7>(f, aaddr, baddr);
  };
  read_all(fa, lds0 + arow + off0, lds0 + brow + boff0);
  wait_frags128(fa);
  int st = 0, kt = 0;
  for (; kt + NS128 < KT; ++kt) {
    const int sn = st + 1 == NS128 ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE128, nxt = lds0 + sn * STAGE128;
    half_step128<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags128(fb);
    WAIT_VM((NS128 - 2) * LPW128);
    __builtin_amdgcn_s_barrier();
    half_step128<true, true>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, stages + st * STAGE128, xk, wk, voff, wave);
    wait_frags128(fa);
    xk += BK * 2;
    wk += wkstep;
    st = sn;
  }
  for (; kt + 1 < KT; ++kt) {   // nothing left to load
    const int sn = st + 1 == NS128 ? 0 : st + 1;
    const unsigned cur = lds0 + st * STAGE128, nxt = lds0 + sn * STAGE128;
    half_step128<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags128(fb);
    WAIT_VM(0);
    __builtin_amdgcn_s_barrier();
    half_step128<true, false>(acc, fb, fa, nxt + arow + off0, nxt + brow + boff0, nullptr, nullptr, nullptr, voff, wave);
    wait_frags128(fa);
    st = sn;
  }
  {
    const unsigned cur = lds0 + st * STAGE128;
    half_step128<true, false>(acc, fa, fb, cur + arow + off1, cur + brow + boff1, nullptr, nullptr, nullptr, voff, wave);
    wait_frags128(fb);
    half_step128<false, false>(acc, fb, fa, 0, 0, nullptr, nullptr, nullptr, voff, wave);
  }
  // The MFMAs are assembly, so the compiler does not know that their results take time: wait out the last ones,
  // tied to their accumulators, and pass every other accumulator through an ordered statement after the wait.
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15"
               : "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3])
               :
               : "memory");
#pragma unroll
  for (int i = 0; i < 3; ++i) asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]));
  // the result leaves through LDS: 64 x 64 per wave
  __syncthreads();
  float* ct = (float*)stages + wave * (64 * CLD);
  const int mw = m0 + wm * 64, nw = n0 + wn * 64;
  RopeFetch<64, 64> fetched;
  if (mode == OUT_ROPE) rope_fetch(fetched, lane, mw, nw, rp, M);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) ct[(i * 16 + g * 4 + r) * CLD + j * 16 + c] = acc[i][j][r];
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (mode == OUT_ROPE)
    emit_tile_rope<64, 64, CLD>(ct, lane, mw, nw, rp, M, fetched);
  else
    emit_tile<64, 64, CLD>(ct, lane, mw, nw, out, mode, M, N, ldo);
}

// Defined in gemm_mfma.hip.
__global__ void gemm_splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ out, int mode,
                                          int splits, int M, int N);

int g_pipe_mid = 0;   // tuning: 1 = 128 x 128 blocks for every product of more than 128 rows, 2 = never

// What a product costs in microseconds, roughly, as `blocks` blocks that take `steps` steps of K each at
// `step_us` a step, one block on a CU at a time, and a kernel that adds the parts if K is split.  Measured:
// 0.52 us a step for a block of 128 x 128, 0.75 us for one of 256 x 128 (STEP128_US, STEP256_US); the parts are
// written and read again at about 3 TB/s.
constexpr double STEP128_US = 0.52, STEP256_US = 0.75;
static double pipe_cost(long blocks, int steps, double step_us, int splits, int M, int N) {
  const double rounds = (double)((blocks + 255) / 256);
  // (rows counted in whole blocks of 128: a step of 100 rows and the same step padded to 128 rows for a captured
  // graph then cut K alike and give the same bits)
  const double rows = (double)((M + 127) / 128 * 128);
  return rounds * steps * step_us + (splits > 1 ? 3.0 + (splits + 2.0) * rows * N * 4.0 / 3e6 : 0.0);
}

// Into how many parts K (KT steps) is cut for `tiles` result tiles: the cheapest by pipe_cost among whole parts
// of at least sixteen steps that the scratch memory holds and that make no more blocks than there are CUs (96 tiles
// of 256 x 128 and 224 steps: two parts, 192 blocks, not the three that make 288 blocks and a second round; parts
// that fill several rounds measured no better than none).
static int best_splits(long tiles, int KT, double step_us, int M, int N, size_t scratch_floats) {
  int best = 1;
  double best_cost = pipe_cost(tiles, KT, step_us, 1, M, N);
  const int cap = std::min(16, KT / 16);
  for (int sp = 2; sp <= cap && sp * tiles <= 256 && (size_t)sp * M * N <= scratch_floats; ++sp) {
    const int per = (KT + sp - 1) / sp;
    if ((KT + per - 1) / per != sp) continue;   // (no part without a step)
    const double c = pipe_cost(tiles * sp, per, step_us, sp, M, N);
    if (c < best_cost - 1e-9) {
      best_cost = c;
      best = sp;
    }
  }
  return best;
}

// The parts of K for blocks of 128 x 128 (the rotating epilogue takes whole sums: can_split false).
static int splits128(int M, int N, int K, bool can_split, size_t scratch_floats) {
  const long tiles = (long)((M + BM128 - 1) / BM128) * ((N + BN128 - 1) / BN128);
  if (!can_split || tiles >= 256) return 1;
  return best_splits(tiles, K / BK, STEP128_US, M, N, scratch_floats);
}

// The parts of K for blocks of 256 x 128: none with 128 tiles or more.
static int splits256(long tiles, int KT, int M, int N, const float* scratch, size_t scratch_floats, int tune_splits) {
  if (scratch == nullptr) return 1;
  if (tune_splits > 0) {
    int sp = std::max(1, std::min(tune_splits, std::min(16, KT / 16)));
    while (sp > 1 && (size_t)sp * M * N > scratch_floats) --sp;
    const int per = (KT + sp - 1) / sp;
    return (KT + per - 1) / per;
  }
  if (tiles >= 128) return 1;
  return best_splits(tiles, KT, STEP256_US, M, N, scratch_floats);
}

// The 128 x 128 blocks.  Returns 0 when launched.
static int tp_linear_pipe128(const bf16_t* x, const bf16_t* w, int w_tiled, void* out, int mode, int M, int N, int K,
                             float* scratch, size_t scratch_floats, const RopeOut* rope, int defer, int* splits_out,
                             hipStream_t s) {
  const int MB = (M + BM128 - 1) / BM128, NB = (N + BN128 - 1) / BN128;
  const long tiles = (long)MB * NB;
  const int splits = splits128(M, N, K, scratch != nullptr && rope == nullptr, scratch_floats);
  RopeOut rp = {};
  if (rope != nullptr) rp = *rope;
  const int ldo = mode == OUT_SWIGLU ? N / 2 : N;
  const long per_xcd = (tiles * splits + 7) / 8;
  if (8 * per_xcd > 0x7fffffffL) return -1;
  hipLaunchKernelGGL(gemm_pipe128_kernel, dim3((unsigned)(8 * per_xcd)), dim3(256), 0, s, x, w, out,
                     splits > 1 ? scratch : nullptr, mode, M, N, K, ldo, rp, w_tiled, splits);
  if (splits > 1 && defer && splits_out != nullptr && mode != OUT_SWIGLU) {
    *splits_out = splits;   // the parts stay unadded for the caller's next kernel
  } else if (splits > 1) {
    const size_t n_out = mode == OUT_SWIGLU ? (size_t)M * (N / 2) : (size_t)M * N;
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s, scratch, out, mode,
                       splits, M, N);
  }
  return 0;
}

// Returns 0 when launched, -1 when the sizes are not this kernel's.  `scratch` (optional) is room for
// float32 partial sums: with few result tiles K is split over blocks until there is work for every CU.
int g_pipe_big = 0;   // tuning: 1 = 256 x 256 tiles for every whole block of 256 columns, 2 = never; 3 = 256 x 192 wherever N allows, 4 = never
int tp_linear_pipe(const bf16_t* x, const bf16_t* w, int w_tiled, void* out, int mode, int M, int N, int K, float* scratch,
                   size_t scratch_floats, int tune_splits, const RopeOut* rope, int defer, int* splits_out, hipStream_t s) {
  if ((mode == OUT_ROPE) != (rope != nullptr)) return -1;
  if (w_tiled && N % 16 != 0) return -1;
  if (K % BK != 0 || K < BK) return -1;
  if ((size_t)(BM - 1) * K * 2 + 128 >= ((size_t)1 << 31)) return -1;  // a lane's source offset stays inside a buffer of 2 GiB
  if (mode == OUT_SWIGLU && N % 16 != 0) return -1;
  const int MB = (M + BM - 1) / BM, NB = (N + BN - 1) / BN;
  // Steps of 65 to a few hundred rows, with at most one round of 256 x 128 blocks: blocks of 128 x 128 where they
  // are cheaper (more of them, so more CUs at work and K in fewer parts).
  bool mid = g_pipe_mid == 1 || (g_pipe_mid == 0 && M <= 128);   // (one row block either way, of half the height)
  if (g_pipe_mid == 0 && M > 128 && (long)MB * NB <= 256) {
    const int KT = K / BK;
    const bool can_split = scratch != nullptr && rope == nullptr;
    const long tiles = (long)MB * NB, tiles128 = (long)((M + BM128 - 1) / BM128) * ((N + BN128 - 1) / BN128);
    const int s256 = splits256(tiles, KT, M, N, scratch, scratch_floats, tune_splits);
    const int s128 = splits128(M, N, K, can_split, scratch_floats);
    mid = pipe_cost(tiles128 * s128, (KT + s128 - 1) / s128, STEP128_US, s128, M, N) <
          pipe_cost(tiles * s256, (KT + s256 - 1) / s256, STEP256_US, s256, M, N);
  }
  if (mid) return tp_linear_pipe128(x, w, w_tiled, out, mode, M, N, K, scratch, scratch_floats, rope, defer, splits_out, s);
  // (see tile_of_block) strips of at most eight row blocks, all about as tall; a launch of nb column blocks has
  // 8 x ceil(MB x nb / 8) blocks
  const int strips = (MB + 7) / 8;
  const int pm = (MB + strips - 1) / strips;
  auto blocks_for = [&](long nb) { return 8L * (((long)MB * nb + 7) / 8); };
  const long blocks = blocks_for(NB);
  if (blocks > 0x7fffffffL) return -1;
  // parts of K: with few tiles, the cheapest number by the cost model, at least sixteen steps of K each
  const int splits = splits256((long)MB * NB, K / BK, M, N, scratch, scratch_floats, tune_splits);
  const int ldo = mode == OUT_SWIGLU ? N / 2 : N;
  RopeOut rp = {};
  if (rope != nullptr) rp = *rope;
  // Whole rounds of 256 x 256 tiles first (see gemm_pipe_big_kernel), the columns that are left as above.
  // How many blocks of 256 columns take the big tiles: all, none, or whole rounds of 256 tiles, whichever
  // needs the fewest rounds when a big tile is priced at 1.72 small ones (measured: 113 against 65 us at
  // K = 4096).
  int nb_big = 0;
  // (with the rotating epilogue a wave's 128 columns of a big tile have to lie inside one of q, k and v: heads
  // of a multiple of 128; the strips of the 192-column tile are ordered for heads of 128)
  const bool big_ok = rope == nullptr || rope->head_dim % 128 == 0;
  if (splits == 1 && g_pipe_big != 2 && ldo % 4 == 0 && big_ok) {
    const long NB2 = N / BNB;
    auto rounds = [&](long nb) {
      const long rest = (N - nb * BNB + BN - 1) / BN;
      return 1.72 * (double)((MB * nb + 255) / 256) + (double)((MB * rest + 255) / 256);
    };
    const long whole = ((long)MB * NB2 / 256) * 256 / MB;
    double best = rounds(0);
    for (long cand : {NB2, whole})
      if (cand > 0 && rounds(cand) < best - 1e-9) {
        best = rounds(cand);
        nb_big = (int)cand;
      }
    if (g_pipe_big == 1) nb_big = (int)NB2;
    // Tiles of 256 x 192 where N is a multiple of 192 and that many more tiles fill whole rounds: priced at 1.35
    // small tiles (the q/k/v projection of 2,048 rows, N = 6,144: 256 tiles in one round instead of 192 of 256 x 256
    // on three quarters of the CUs, 109 -> 8x us).
    if (N % 192 == 0 && mode != OUT_SWIGLU && g_pipe_big != 4 && (rope == nullptr || rope->head_dim == 128)) {
      const long t192 = (long)MB * (N / 192);
      if (1.35 * (double)((t192 + 255) / 256) < best - 1e-9 || g_pipe_big == 3) {
        const long blocks3 = blocks_for(N / 192);
        hipLaunchKernelGGL(gemm_pipe_big_kernel<6>, dim3((unsigned)blocks3), dim3(256), 0, s, x, w, out, mode, M, N, K, pm, ldo,
                           rp, w_tiled);
        return 0;
      }
    }
  }
  if (nb_big > 0) {
    const long blocks2 = blocks_for(nb_big);
    hipLaunchKernelGGL(gemm_pipe_big_kernel<8>, dim3((unsigned)blocks2), dim3(256), 0, s, x, w, out, mode, M, nb_big * BNB, K,
                       pm, ldo, rp, w_tiled);
    const int n_done = nb_big * BNB;
    if (n_done == N) return 0;
    // the rest of the columns
    const int N2 = N - n_done;
    const int NBr = (N2 + BN - 1) / BN;
    const long blocksr = blocks_for(NBr);
    const size_t esz = mode == OUT_BF16 || mode == OUT_SWIGLU ? 2 : 4;
    void* out2 = out == nullptr ? nullptr : (char*)out + (size_t)(mode == OUT_SWIGLU ? n_done / 2 : n_done) * esz;
    rp.col0 = n_done;
    hipLaunchKernelGGL(gemm_pipe_kernel, dim3((unsigned)blocksr, 1), dim3(256), 0, s, x, w + (size_t)n_done * K, out2, scratch,
                       mode, M, N2, K, pm, ldo, rp, w_tiled);
    return 0;
  }
  hipLaunchKernelGGL(gemm_pipe_kernel, dim3((unsigned)blocks, splits), dim3(256), 0, s, x, w, out, scratch, mode, M, N, K,
                     pm, ldo, rp, w_tiled);
  if (splits > 1 && defer && splits_out != nullptr && mode != OUT_SWIGLU) {
    *splits_out = splits;   // the parts stay unadded for the caller's next kernel
  } else if (splits > 1) {
    const size_t n_out = mode == OUT_SWIGLU ? (size_t)M * (N / 2) : (size_t)M * N;
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s, scratch, out, mode,
                       splits, M, N);
  }
  return 0;
}

int g_pipe64_narrow = 0;   // tuning: 1 = blocks of 64 columns always, 2 = never
// The 64-row pipeline (17..64 rows; up to 128 where the other kernels do not take the sizes).  `defer`: when K is split, leave the partial sums in `scratch` for the
// caller's next kernel and report their number through *splits_out.
int tp_linear_pipe64(const bf16_t* x, const bf16_t* w, int w_tiled, void* out, int mode, int M, int N, int K, float* scratch,
                     size_t scratch_floats, int tune_splits, int defer, int* splits_out, hipStream_t s) {
  if (K % BK != 0 || K < BK || M > 128) return -1;
  if (w_tiled && N % 16 != 0) return -1;
  if ((size_t)(BM64 - 1) * K * 2 + 128 >= ((size_t)1 << 31)) return -1;
  if (mode == OUT_SWIGLU && N % 16 != 0) return -1;
  const int MB = (M + BM64 - 1) / BM64;
  const int KT = K / BK;
  // a block for every CU, at least sixteen tiles of K each (measured at 24, 64 and 128 rows of the 8B
  // shapes: more splits than that cost more in partial sums than they gain)
  auto plan = [&](int bn, long& tiles) {
    tiles = (long)MB * ((N + bn - 1) / bn);
    int splits = 1;
    if (scratch != nullptr) {
      splits = tune_splits > 0 ? tune_splits : (int)(256 / std::max(1L, tiles));
      splits = std::max(1, std::min(splits, std::min(16, KT / 16)));
      while (splits > 1 && (size_t)splits * M * N > scratch_floats) --splits;
      const int per = (KT + splits - 1) / splits;
      splits = (KT + per - 1) / per;
    }
    return splits;
  };
  long tiles = 0, tiles_narrow = 0;
  int splits = plan(BN, tiles);
  const int splits_narrow = plan(64, tiles_narrow);
  if (tiles > 0x7fffffffL || tiles_narrow > 0x7fffffffL) return -1;
  // blocks of 64 columns where those of 128 leave a fifth of the CUs or more without one, or where they give
  // every CU a block without any split of K (measured at 64 rows: 4096 x 4096 15.7 -> 15.0 us with the kernel
  // that adds the partial sums, 5120 x 3072 11.0 -> 9.1, 3072 x 3072 14.1 -> 12.3, 16384 x 3072 gated 25.1 -> 21.1;
  // 6144 x 4096, which has 192 blocks of 128 columns, 12.4 -> 14.9: left as it is)
  const bool narrow = g_pipe64_narrow == 1 ||
                      (g_pipe64_narrow == 0 && tiles_narrow * splits_narrow >= tiles * splits &&
                       ((tiles * splits < 192 && tiles_narrow * splits_narrow > tiles * splits) || (splits > 1 && splits_narrow == 1)));
  if (narrow) {
    tiles = tiles_narrow;
    splits = splits_narrow;
  }
  const bool leave = defer && splits > 1 && splits_out != nullptr && mode != OUT_SWIGLU;
  if (narrow)
    hipLaunchKernelGGL(gemm_pipe64_kernel<2>, dim3((unsigned)tiles, splits), dim3(256), 0, s, x, w, out,
                       splits > 1 ? scratch : nullptr, mode, M, N, K, w_tiled);
  else
    hipLaunchKernelGGL(gemm_pipe64_kernel<4>, dim3((unsigned)tiles, splits), dim3(256), 0, s, x, w, out,
                       splits > 1 ? scratch : nullptr, mode, M, N, K, w_tiled);
  if (leave) {
    *splits_out = splits;
  } else if (splits > 1) {
    const size_t n_out = mode == OUT_SWIGLU ? (size_t)M * (N / 2) : (size_t)M * N;
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s, scratch, out, mode,
                       splits, M, N);
  }
  return 0;
}
