// Attention over the paged cache on the matrix cores (bf16 in, float softmax and accumulation).
//
// One wavefront works on 16 "query columns" against one page of 64 keys at a time:
//   S^T = K Q^T        A = K rows (16 keys x head_dim), B = Q^T; the result leaves lane (kg, c) with
//                       the scores of query column c = lane % 16 for keys kg*4 .. kg*4+3 of each
//                       16-key tile, so the whole softmax of a query lives in the four lanes that
//                       share c, and needs two cross-lane steps.
//   O^T += V^T P^T      A = V^T rows (16 dims x 32 keys), B = P^T.  The probabilities a lane has
//                       just computed are exactly the B fragment it must supply (the order of the
//                       32 keys inside an MFMA is free as long as A and B agree), so P never moves.
//                       V is cached transposed per page ([head_dim][64 tokens]), and the keys of a
//                       page are dealt to the four 16-key tiles so that the eight keys a lane
//                       supplies to one of these instructions are neighbours: the A fragment of V^T
//                       is one 16-byte load (am_key_of).
// No shared memory is needed for the products and nothing is transposed at run time.
//
// Prefill: the 16 query columns are 16 consecutive tokens of one head of one sequence.
// Decode:  they are the query heads that share a key-value head, for one token; the key range is
//          cut into splits that are merged afterwards (float partial results).
// Visibility: query at position p sees keys j <= p of its sequence and, with a window w, p - j < w.
#include <stdlib.h>

#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;

#define AM_WAVES 4
#define AM_PAGE 64
// s_waitcnt vmcnt(0) of gfx9 (vmcnt in bits 3:0 and 15:14; the other counters left at their maxima)
#define AM_WAIT_LOADS() __builtin_amdgcn_s_waitcnt(0x0F70)

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }

// Stores and loads that bypass the per-die caches: what one block writes this way, a block on
// another die reads this way, once the store has completed.
__device__ __forceinline__ void coherent_store(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// keep the first n (0..4) bf16 of an 8-byte group, zero the rest
__device__ __forceinline__ uint2 keep_first(uint2 v, int n) {
  if (n >= 4) return v;
  if (n <= 0) return make_uint2(0u, 0u);
  const unsigned long long m = (1ull << (16 * n)) - 1ull;
  const unsigned long long x = ((unsigned long long)v.y << 32) | v.x;
  const unsigned long long y = x & m;
  return make_uint2((uint32_t)y, (uint32_t)(y >> 32));
}

// keep the first n (0..8) bf16 of a 16-byte group, zero the rest
__device__ __forceinline__ uint4 keep_first(uint4 v, int n) {
  const uint2 lo = keep_first(make_uint2(v.x, v.y), n), hi = keep_first(make_uint2(v.z, v.w), n - 4);
  return make_uint4(lo.x, lo.y, hi.x, hi.y);
}

// Which key of a page row i (0..15) of score tile t (0..3) is: the scores of tile t leave lane group kg
// with rows kg * 4 .. + 3, and the product with the values takes tiles 2 h and 2 h + 1 together, a lane
// supplying its four rows of the one and then of the other.  With this order those are the keys
// h * 32 + kg * 8 .. + 7.  The staged key page holds key am_key_of(t, i) in row t * 16 + i.
__device__ __forceinline__ constexpr int am_key_of(int t, int i) { return (t >> 1) * 32 + (i >> 2) * 8 + (t & 1) * 4 + (i & 3); }
// the staged row of key k of a page (the inverse)
__device__ __forceinline__ constexpr int am_row_of(int k) {
  return ((((k >> 5) << 1) | ((k >> 2) & 1)) << 4) | (((k >> 3) & 3) << 2) | (k & 3);
}

// One page of keys for one wavefront.  qf: B fragments of Q^T.  Lane (kg = lane / 16, c = lane % 16)
// owns query column c.  qpos / lo: highest / lowest key this lane's query may see.  max_key: the last
// key that the cache holds data for (values past it may be garbage and are zeroed; between a query's
// own position and max_key they are other tokens' values, finite, and meet a probability of zero).
// FULL: every key of the page is visible to every query of the tile, so no mask is computed.
// The softmax runs in base 2: scale2 = scale * log2(e), m is the running maximum of s * scale2,
// probabilities are exp2(s * scale2 - m); sums and outputs are the same as in base e.
// PAGE: where the fragments of a staged page lie (one of the two layouts below); the values are read
// after the scores, so they arrive during the softmax and the keys' registers are free by then.

// Rows padded so that the 16-byte fragment reads of 16 rows meet every bank once (any head size):
// keys [64][HD + 8], values [HD][64 + 8] (strides = 16 bytes mod 128).
template <int HD>
struct PaddedPage {
  static constexpr int KSTR = HD + 8, VSTR = AM_PAGE + 8;
  static constexpr int K_ELEMS = AM_PAGE * KSTR, V_ELEMS = HD * VSTR;
  // element offset of the 8 dims ks * 32 + kg * 8 .. of staged key row t * 16 + c
  static __device__ __forceinline__ int k(int t, int ks, int c, int kg) { return (t * 16 + c) * KSTR + ks * 32 + kg * 8; }
  // element offset of the 8 keys h * 32 + kg * 8 .. of value dim dt * 16 + c
  static __device__ __forceinline__ int v(int dt, int h, int c, int kg) { return (dt * 16 + c) * VSTR + h * 32 + kg * 8; }
};
// Rows as they lie in memory (so a page can come straight from global memory, 1 KB per load
// instruction), with the 16-byte pieces of a row permuted: piece J of row r is at place J ^ f(r).  Value
// rows are 128 bytes (8 pieces), f(r) = (r / 2) % 8: the 16 rows of a fragment read then cover the 16
// combinations of (r % 2, place), that is every bank.  Key rows of 64 dims likewise; key rows of 128
// dims are 256 bytes (16 pieces, all banks once per row), f(r) = r % 16.
template <int HD>
struct SwizzledPage {
  static_assert(HD == 64 || HD == 128, "rows of 128 or 256 bytes");
  static constexpr int K_ELEMS = AM_PAGE * HD, V_ELEMS = HD * AM_PAGE;
  static __device__ __forceinline__ int k_twist(int row) { return HD == 64 ? (row >> 1) & 7 : row & 15; }
  static __device__ __forceinline__ int v_twist(int row) { return (row >> 1) & 7; }
  static __device__ __forceinline__ int k(int t, int ks, int c, int kg) {
    return (t * 16 + c) * HD + ((ks * 4 + kg) ^ k_twist(c)) * 8;   // k_twist(t * 16 + c) = k_twist(c)
  }
  static __device__ __forceinline__ int v(int dt, int h, int c, int kg) {
    return (dt * 16 + c) * AM_PAGE + ((h * 4 + kg) ^ v_twist(c)) * 8;
  }
};

// The order of the keys in a staged key page: row r holds key ORDER::key_of(r) of the page, and
// ORDER::row_of is the inverse.
struct TileOrder16 {   // for the 16x16x32 instruction, see am_key_of
  static __device__ __forceinline__ constexpr int key_of(int row) { return am_key_of(row >> 4, row & 15); }
  static __device__ __forceinline__ constexpr int row_of(int key) { return am_row_of(key); }
};

// A page straight from global memory into a SwizzledPage in shared memory, by the four wavefronts of a
// block: wavefront w fills the 1-KB pieces w, w + 4, .. of the key page and of the value page, lane i
// of piece L the place L * 64 + i, with the 16 bytes of global memory that the layout puts there (for
// keys: of the key that belongs in that row).  What a lane adds to the page's address is the same in all
// of a wavefront's pieces up to a term that all lanes share: four pieces further the staged row has
// grown by a multiple of 16, which changes neither the twist nor a key's place among its 16 or 32.
// The loads are invisible to the compiler (blm_dma16_to): the caller waits for them (AM_WAIT_LOADS)
// before the barrier that hands the page over.
template <int HD, class ORDER>
struct DirectStage {
  using PAGE = SwizzledPage<HD>;
  static constexpr int PIECES = AM_PAGE * HD * 2 / 1024, PER_WAVE = PIECES / AM_WAVES;
  static_assert(PIECES % AM_WAVES == 0, "pieces per wavefront");
  static constexpr int K_CPR = HD / 8, V_CPR = AM_PAGE / 8;   // 16-byte pieces per row
  static constexpr int K_RPP = BLM_WAVE / K_CPR;              // staged key rows per 1-KB piece
  uint32_t k_lane, v_lane, k_lds0, v_lds0;
  int wave_u;
  // k_lds, v_lds: the first of the block's page buffers (further ones follow at PAGE::K_ELEMS / V_ELEMS)
  __device__ __forceinline__ void init(const bf16* k_lds, const bf16* v_lds) {
    const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
    wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int k_row = wave * K_RPP + lane / K_CPR;       // staged row that this lane fills in piece w
    const int v_row = (wave * BLM_WAVE + lane) / V_CPR;
    k_lane = (uint32_t)((ORDER::key_of(k_row) * K_CPR + ((lane % K_CPR) ^ PAGE::k_twist(k_row))) * 16);
    v_lane = (uint32_t)((v_row * V_CPR + ((lane % V_CPR) ^ PAGE::v_twist(v_row))) * 16 - wave * 1024);
    k_lds0 = (uint32_t)(uintptr_t)(blm_lds_ptr)k_lds;
    v_lds0 = (uint32_t)(uintptr_t)(blm_lds_ptr)v_lds;
  }
  // base: element offset of the (page, key-value head) in the cache planes (the same in all lanes)
  __device__ __forceinline__ void fetch(const bf16* kcache, const bf16* vcache, size_t base, int buf) const {
    const char* kb = reinterpret_cast<const char*>(kcache + base);
    const char* vb = reinterpret_cast<const char*>(vcache + base);
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
      const int piece = wave_u + i * AM_WAVES;
      const int k_step = (ORDER::key_of(piece * K_RPP) - ORDER::key_of(wave_u * K_RPP)) * HD * 2;
      blm_dma16_to(kb + k_step, k_lane, k_lds0 + (uint32_t)(buf * PAGE::K_ELEMS * 2 + piece * 1024));
      blm_dma16_to(vb + piece * 1024, v_lane, v_lds0 + (uint32_t)(buf * PAGE::V_ELEMS * 2 + piece * 1024));
    }
  }
};

template <int HD, bool FULL, class PAGE>
__device__ __forceinline__ void attn_page(const bf16* __restrict__ kp, const bf16* __restrict__ vp,
                                          const uint4* qf, int key0, int qpos, int lo, int max_key, float scale2,
                                          float& m, f32x4_t& l, f32x4_t* o) {
  constexpr int KS = (HD + 31) / 32;
  constexpr int DT = (HD + 15) / 16;
  const int lane = threadIdx.x & (BLM_WAVE - 1);
  const int c = lane & 15, kg = lane >> 4;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  // issue the loads of the page: keys for S^T, values for O^T
  uint4 kf[4][KS];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + kg * 8;
      kf[t][ks] = (HD % 32 == 0 || d < HD) ? *reinterpret_cast<const uint4*>(kp + PAGE::k(t, ks, c, kg)) : zero;
    }
  // scores, unscaled; the scale (> 0) goes into the exponent's multiply-add
  float s[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kf[t][ks]),
                                                    __builtin_bit_cast(bf16x8_t, qf[ks]), acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (FULL) {
        s[t][r] = acc[r];
      } else {
        const int kj = key0 + am_key_of(t, kg * 4 + r);
        s[t][r] = (kj <= qpos && kj >= lo) ? acc[r] : -INFINITY;
      }
    }
  }
  uint4 vf[DT][2];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h) vf[dt][h] = *reinterpret_cast<const uint4*>(vp + PAGE::v(dt, h, c, kg));
  float mx = blm_max(s[0][0], s[0][1]);
  mx = blm_max(blm_max(mx, s[0][2]), s[0][3]);
#pragma unroll
  for (int t = 1; t < 4; ++t) {
    mx = blm_max(blm_max(mx, s[t][0]), s[t][1]);
    mx = blm_max(blm_max(mx, s[t][2]), s[t][3]);
  }
  mx = rows_max(mx);
  const float m_new = blm_max(m, mx * scale2);
  // m = -inf, m_new finite -> 0;  both -inf (nothing visible yet) -> 1, and every p below is 0
  const float corr = (m == m_new) ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float p;
      if (FULL) p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], scale2, -m_new));
      else p = (s[t][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], scale2, -m_new));
      s[t][r] = p;
    }
  if (__any(m != m_new)) {   // once the running maxima have settled, most pages change none of them
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] *= corr;
#pragma unroll
    for (int r = 0; r < 4; ++r) l[r] *= corr;
  }
  m = m_new;

  // O^T += V^T P^T, 32 keys (two 16-key tiles) per MFMA
  const bool tail = !FULL && key0 + AM_PAGE - 1 > max_key;   // uniform: the page holds places past the data
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint4 pf;
    pf.x = pack_bf16x2(s[2 * h][0], s[2 * h][1]);
    pf.y = pack_bf16x2(s[2 * h][2], s[2 * h][3]);
    pf.z = pack_bf16x2(s[2 * h + 1][0], s[2 * h + 1][1]);
    pf.w = pack_bf16x2(s[2 * h + 1][2], s[2 * h + 1][3]);
    // the softmax's denominator as one more output row: a row of ones for V^T sums the rounded
    // probabilities of every query column over the 32 keys, on the matrix cores instead of 16 adds
    l = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u)),
                                                __builtin_bit_cast(bf16x8_t, pf), l, 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint4 va = vf[dt][h];
      if (tail) va = keep_first(va, max_key - (key0 + h * 32 + kg * 8) + 1);   // 0 * garbage must stay 0
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, va),
                                                      __builtin_bit_cast(bf16x8_t, pf), o[dt], 0, 0, 0);
    }
  }
}

// The page numbers of a stretch of one sequence's block table, 64 at a time in one register (lane i
// holds entry base + i).  A loop over pages then takes the next page's number out of the register
// instead of asking memory for it in front of the loads that need it, once per page.
struct PageNumbers {
  const int* table;
  int width, base, held;
  __device__ __forceinline__ void load(int first) {
    base = first;
    held = table[min(first + (int)(threadIdx.x & (BLM_WAVE - 1)), width - 1)];
  }
  // pi: the same in all lanes, not below the last load's first entry
  __device__ __forceinline__ int at(int pi) {
    if (pi - base >= BLM_WAVE) load(pi);
    return __builtin_amdgcn_readlane(held, __builtin_amdgcn_readfirstlane(pi - base));
  }
};

// A use of loaded fragments that the compiler cannot move or remove: their loads are issued, and
// waited for, in front of it.
template <int N>
__device__ __forceinline__ void am_pin(uint4* f) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i].x), "+v"(f[i].y), "+v"(f[i].z), "+v"(f[i].w));
}

template <int HD>
__device__ __forceinline__ void load_q(const bf16* qrow, uint4* qf) {
  constexpr int KS = (HD + 31) / 32;
  const int kg = (threadIdx.x & (BLM_WAVE - 1)) >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + kg * 8;
    qf[ks] = (HD % 32 == 0 || d < HD) ? *reinterpret_cast<const uint4*>(qrow + d) : make_uint4(0u, 0u, 0u, 0u);
  }
}

// ---------------------------------------------------------------------------------------
// prefill: grid (ceil(G * q_tiles / 4), kv heads, sequences)
//
// The four wavefronts of a block are four (head, 16-query tile) units that share a key-value head
// and, for groups of four or more heads, the same queries.  Every page they need is brought into
// shared memory once per block with coalesced 16-byte loads (the next page travels in registers
// while the current one is used) and each wavefront takes its MFMA fragments from there; rows are
// padded by 16 bytes so that the fragment reads do not collide.
// ---------------------------------------------------------------------------------------
template <int HD>
__global__ void __launch_bounds__(AM_WAVES* BLM_WAVE) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 4 : (HD <= 128 ? 2 : 1), HD <= 64 ? 8 : (HD <= 128 ? 2 : 1))))
    attn_prefill_mfma_kernel(const bf16* __restrict__ q, int q_row_stride, bf16* __restrict__ out,
                             const int* __restrict__ positions, const int* __restrict__ cu_seqlens,
                             const int* __restrict__ block_table, int table_width,
                             const bf16* __restrict__ kcache, const bf16* __restrict__ vcache, int nh, int nkv,
                             float scale, int window) {
  constexpr int KS = (HD + 31) / 32;
  constexpr int DT = (HD + 15) / 16;
  // Head sizes 64 and 128: a page comes straight from global memory into shared memory, its rows'
  // pieces permuted.  Other head sizes: through registers into padded rows.
  constexpr bool DIRECT = HD == 64 || HD == 128;
  using PAGE = std::conditional_t<DIRECT, SwizzledPage<DIRECT ? HD : 64>, PaddedPage<HD>>;
  constexpr int KSTR = PaddedPage<HD>::KSTR, VSTR = PaddedPage<HD>::VSTR;
  constexpr int CHUNKS = AM_PAGE * HD / 8;              // 16-byte pieces of a page (keys and values alike)
  constexpr int PER_THREAD = (CHUNKS + AM_WAVES * BLM_WAVE - 1) / (AM_WAVES * BLM_WAVE);
  // two buffers for head sizes whose pages fit twice: the next page is written while the current
  // one is still being used, and one barrier per page is enough
  constexpr int NBUF = HD <= 128 ? 2 : 1;
  __shared__ __align__(16) bf16 k_lds[NBUF][PAGE::K_ELEMS];
  __shared__ __align__(16) bf16 v_lds[NBUF][PAGE::V_ELEMS];   // a multiple of 16 bytes in either layout
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int c = lane & 15, kg = lane >> 4;
  const int G = nh / nkv;
  const int b = blockIdx.z;
  const int row_begin = cu_seqlens[b];
  const int n_b = cu_seqlens[b + 1] - row_begin;
  // Which (key-value head, query tiles) this block takes.  Blocks are handed out in the order of
  // their linear index, consecutive ones to different dies: the key-value head changes fastest, so
  // a die (with its own L2) mostly sees the pages of one head.  Along the other axis the work of a
  // causal prompt falls from the last query tile (most keys) to the first; every second run of 32
  // is reversed so that compute units that receive one block of each run get equal shares.
  const int lin = blockIdx.x + gridDim.x * blockIdx.y;
  const int kvh = lin % nkv;
  int x = lin / nkv;
  {
    const int seg = x >> 5;
    if ((seg & 1) && seg * 32 + 32 <= (int)gridDim.x) x = seg * 32 + 31 - (x & 31);
  }
  const int u0 = ((int)gridDim.x - 1 - x) * AM_WAVES;
  if ((u0 / G) * 16 >= n_b) return;   // the whole block lies past the sequence's end (uniform)
  const int u = u0 + wave;
  const int g = u % G, qt = u / G;
  const bool active = qt * 16 < n_b;
  const int head = kvh * G + g;
  const int nq = active ? min(16, n_b - qt * 16) : 1;
  const int row = row_begin + (active ? qt * 16 + min(c, nq - 1) : 0);   // columns past the tile's end repeat its last query
  const int qpos = positions[row];
  const int qpos_first = positions[row_begin + (active ? qt * 16 : 0)];
  const int qpos_last = positions[row_begin + (active ? qt * 16 + nq - 1 : 0)];
  const int seq_last = positions[row_begin + n_b - 1];   // the cache holds data up to here: places past it may hold anything
  const int lo = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  const int lo_tile = (window > 0 && qpos_first - window + 1 > 0) ? qpos_first - window + 1 : 0;
  const int lo_last = (window > 0 && qpos_last - window + 1 > 0) ? qpos_last - window + 1 : 0;
  const int my_first = active ? lo_tile / AM_PAGE : 0x7fffffff, my_last = active ? qpos_last / AM_PAGE : -1;
  // page range of the block: from its first unit's first page to its last active unit's last page
  const int qt_lo = u0 / G, qt_hi = min((u0 + AM_WAVES - 1) / G, (n_b - 1) / 16);
  const int blk_qfirst = positions[row_begin + qt_lo * 16];
  const int blk_qlast = positions[row_begin + min(qt_hi * 16 + 15, n_b - 1)];
  const int blk_first = ((window > 0 && blk_qfirst - window + 1 > 0) ? blk_qfirst - window + 1 : 0) / AM_PAGE;
  const int blk_last = blk_qlast / AM_PAGE;

  uint4 qf[KS];
  load_q<HD>(q + (size_t)row * q_row_stride + (size_t)head * HD, qf);
  float m = -INFINITY;
  f32x4_t lsum = {0.f, 0.f, 0.f, 0.f};   // the denominator of query column c, the same in all four places
  f32x4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const float scale2 = scale * 1.4426950408889634f;
  PageNumbers pages{block_table + (size_t)b * table_width, table_width, 0, 0};
  pages.load(blk_first);

  u32x4_t kreg[PER_THREAD], vreg[PER_THREAD];
#define AM_FETCH(pi)                                                                          \
  {                                                                                           \
    const size_t base = ((size_t)pages.at(pi) * nkv + kvh) * AM_PAGE * HD;                    \
    _Pragma("unroll") for (int i = 0; i < PER_THREAD; ++i) {                                  \
      const int j = i * AM_WAVES * BLM_WAVE + threadIdx.x;                                    \
      if (CHUNKS % (AM_WAVES * BLM_WAVE) == 0 || j < CHUNKS) {                                \
        kreg[i] = *reinterpret_cast<const u32x4_t*>(kcache + base + (size_t)j * 8);             \
        vreg[i] = *reinterpret_cast<const u32x4_t*>(vcache + base + (size_t)j * 8);             \
      }                                                                                       \
    }                                                                                         \
  }
#define AM_STAGE(buf)                                                                                         \
  _Pragma("unroll") for (int i = 0; i < PER_THREAD; ++i) {                                                      \
    const int j = i * AM_WAVES * BLM_WAVE + threadIdx.x;                                                        \
    if (CHUNKS % (AM_WAVES * BLM_WAVE) == 0 || j < CHUNKS) {                                                    \
      const int kr = j / (HD / 8), kc = j - kr * (HD / 8);           /* key, 16-byte column */                  \
      *reinterpret_cast<u32x4_t*>(k_lds[buf] + am_row_of(kr) * KSTR + kc * 8) = kreg[i];                        \
      const int vr = j / (AM_PAGE / 8), vc = j - vr * (AM_PAGE / 8); /* value row (a dim), 16-byte column */    \
      *reinterpret_cast<u32x4_t*>(v_lds[buf] + vr * VSTR + vc * 8) = vreg[i];                                   \
    }                                                                                                           \
  }
#define AM_USE(buf)                                                                                           \
  if (pi >= my_first && pi <= my_last) {                                                                        \
    const int key0 = pi * AM_PAGE;                                                                              \
    /* pages wholly inside every query's range need no mask */                                                  \
    if (key0 + AM_PAGE - 1 <= qpos_first && key0 >= lo_last)                                                    \
      attn_page<HD, true, PAGE>(k_lds[buf], v_lds[buf], qf, key0, qpos, lo, seq_last, scale2, m, lsum, o);  \
    else                                                                                                        \
      attn_page<HD, false, PAGE>(k_lds[buf], v_lds[buf], qf, key0, qpos, lo, seq_last, scale2, m, lsum, o); \
  }
  if constexpr (DIRECT) {
    DirectStage<DIRECT ? HD : 64, TileOrder16> stage;
    stage.init(k_lds[0], v_lds[0]);
    auto fetch = [&](int pi, int buf) { stage.fetch(kcache, vcache, ((size_t)pages.at(pi) * nkv + kvh) * AM_PAGE * HD, buf); };
    fetch(blk_first, 0);
    am_pin<KS>(qf);   // see below
    AM_WAIT_LOADS();
    __syncthreads();
    for (int pi = blk_first; pi <= blk_last; ++pi) {
      const int cur = (pi - blk_first) & 1;
      if (pi < blk_last) fetch(pi + 1, cur ^ 1);   // into the other buffer, which nobody reads now
      AM_USE(cur)
      AM_WAIT_LOADS();     // the compiler does not know of these loads: the wait is the program's own
      __syncthreads();     // the next page is in place, and everybody is done with this one
    }
  } else {
  AM_FETCH(blk_first);
  // The query fragments have arrived before the loop starts.  Left alone, the compiler moves their
  // loads down to the loop's entry, and since its count of outstanding loads is merged over the loop's
  // paths, it then waits in front of the first product of every page for all loads, the page it has
  // just asked for included.
  am_pin<KS>(qf);
  if (NBUF == 2) {
    AM_STAGE(0)
    __syncthreads();
    for (int pi = blk_first; pi <= blk_last; ++pi) {
      const int cur = (pi - blk_first) & 1;
      if (pi < blk_last) AM_FETCH(pi + 1);   // travels while this page is used
      AM_USE(cur)
      if (pi < blk_last) { AM_STAGE(cur ^ 1) }   // the other buffer: nobody reads it now
      __syncthreads();   // the next page is in place, and everybody is done with this one
    }
  } else {
    for (int pi = blk_first; pi <= blk_last; ++pi) {
      __syncthreads();   // the page before has been used by every wavefront
      AM_STAGE(0)
      __syncthreads();
      if (pi < blk_last) AM_FETCH(pi + 1);   // travels while this page is used
      AM_USE(0)
    }
  }
  }
#undef AM_STAGE
#undef AM_USE
#undef AM_FETCH
  if (!active) return;
  const float l = lsum[0];
  if (c < nq) {
    const float inv = 1.0f / l;
    bf16* orow = out + (size_t)row * nh * HD + (size_t)head * HD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int d = dt * 16 + kg * 4;
      if (HD % 16 == 0 || d < HD) {
        uint2 w;
        w.x = pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv);
        w.y = pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + d) = w;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// prefill with 32 queries per wavefront (head sizes that are multiples of 32, up to 128)
//
// The same arrangement on the 32x32x16 instruction: a wavefront owns 32 consecutive tokens of one
// head, so every key and value fragment it takes from shared memory serves twice as many queries
// (the shared-memory reads, which bound the 16-query form, are halved per matrix instruction).
//   S^T = K Q^T      A = 32 keys x 16 dims (lane l: key l % 32, dims 8 (l / 32) ..), B = Q^T (lane l:
//                    query l % 32, the same dims); the result leaves lane (j = l % 32, hb = l / 32)
//                    with the scores of query j for keys 8 (v / 4) + 4 hb + v % 4, v < 16, of the tile.
//   O^T += V^T P^T   A = 32 dims x 16 keys, B = P^T.  The 16 keys of instruction n of a 32-key tile are
//                    the ones whose scores sit in accumulator values 8 n .. 8 n + 7: lane hb supplies rows
//                    16 n + 4 hb .. + 3 and 16 n + 8 + 4 hb .. + 3 of the tile, which are exactly those
//                    values, so the probabilities never move.  The staged key page holds its keys in an
//                    order (TileOrder32) in which these eight rows are the neighbouring keys
//                    16 n + 8 hb .. + 7, so the matching V^T fragment is one 16-byte read.
// The softmax of a query lives in the two lanes j and j + 32; the denominator is summed by one
// two-element dot product with ones per pair of rounded probabilities (v_dot2c_f32_bf16).
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

// Key order of the 32-query form: row r of the staged key page holds the key whose number is r with
// bits 2 and 3 exchanged (its own inverse).
struct TileOrder32 {
  static __device__ __forceinline__ constexpr int key_of(int row) { return (row & ~12) | ((row & 4) << 1) | ((row & 8) >> 1); }
  static __device__ __forceinline__ constexpr int row_of(int key) { return key_of(key); }
};
// Element offsets of the 32-query form's fragments in the two page layouts: the 8 dims ks * 16 + hb * 8 ..
// of staged key row `row`, and the 8 keys piece * 8 .. of value dim `dim` (piece: 0..7).
template <int HD>
struct PaddedFragments32 {
  static __device__ __forceinline__ int k(int row, int ks, int hb) { return row * PaddedPage<HD>::KSTR + ks * 16 + hb * 8; }
  static __device__ __forceinline__ int v(int dim, int piece) { return dim * PaddedPage<HD>::VSTR + piece * 8; }
};
template <int HD>
struct SwizzledFragments32 {
  static __device__ __forceinline__ int k(int row, int ks, int hb) { return row * HD + ((ks * 2 + hb) ^ SwizzledPage<HD>::k_twist(row)) * 8; }
  static __device__ __forceinline__ int v(int dim, int piece) { return dim * AM_PAGE + (piece ^ SwizzledPage<HD>::v_twist(dim)) * 8; }
};

// acc + lo + hi of a pair of bf16 in one instruction
__device__ __forceinline__ float am_dot2_ones(uint32_t pair, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 am_bf16x2;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(am_bf16x2, pair), __builtin_bit_cast(am_bf16x2, 0x3f803f80u), acc, false);
}

// Half `half` of a page (32 keys from key0) for one wavefront: the softmax state advances once per 32
// keys, so only 16 scores per lane are alive at a time.  kp, vp: the staged page; FRAG: where its
// fragments lie.  max_key: the last key that the cache holds data for (see attn_page).
template <int HD, bool FULL, class FRAG>
__device__ __forceinline__ void attn_half32(const bf16* __restrict__ kp, const bf16* __restrict__ vp, const uint4* qf,
                                            int half, int key0, int qpos, int lo, int max_key, float scale2, float& m,
                                            float& l, f32x16_t* o) {
  constexpr int KS = HD / 16, RT = HD / 32;
  const int lane = threadIdx.x & (BLM_WAVE - 1);
  const int j = lane & 31, hb = lane >> 5;
  f32x16_t s;
#pragma unroll
  for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const uint4 kf = *reinterpret_cast<const uint4*>(kp + FRAG::k(half * 32 + j, ks, hb));
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf), __builtin_bit_cast(bf16x8_t, qf[ks]), s, 0, 0, 0);
  }
  if (!FULL) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int kj = key0 + TileOrder32::key_of(8 * (v >> 2) + 4 * hb + (v & 3));
      s[v] = (kj <= qpos && kj >= lo) ? s[v] : -INFINITY;
    }
  }
  float mx = blm_max(s[0], s[1]);
#pragma unroll
  for (int v = 2; v < 16; v += 2) mx = blm_max(blm_max(mx, s[v]), s[v + 1]);
  {
    float a, b;
    blm_swap32(mx, a, b);
    mx = blm_max(a, b);
  }
  const float m_new = blm_max(m, mx * scale2);
  const float corr = (m == m_new) ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    if (FULL) s[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], scale2, -m_new));
    else s[v] = (s[v] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], scale2, -m_new));
  }
  if (__any(m != m_new)) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[rt][v] *= corr;
    l *= corr;
  }
  m = m_new;
  const bool tail = !FULL && key0 + 31 > max_key;   // uniform: the half holds places past the data
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    uint4 pf;
    pf.x = pack_bf16x2(s[8 * n + 0], s[8 * n + 1]);
    pf.y = pack_bf16x2(s[8 * n + 2], s[8 * n + 3]);
    pf.z = pack_bf16x2(s[8 * n + 4], s[8 * n + 5]);
    pf.w = pack_bf16x2(s[8 * n + 6], s[8 * n + 7]);
    // the denominator takes the rounded probabilities, two per instruction (a dot product with ones);
    // a lane sums its own keys, the two lanes of a query are added at the end
    l = am_dot2_ones(pf.x, l); l = am_dot2_ones(pf.y, l); l = am_dot2_ones(pf.z, l); l = am_dot2_ones(pf.w, l);
    const int piece = half * 4 + n * 2 + hb;   // this lane's keys of the instruction: piece * 8 .. + 7 of the page
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      uint4 va = *reinterpret_cast<const uint4*>(vp + FRAG::v(rt * 32 + j, piece));
      if (tail) va = keep_first(va, max_key - (key0 + n * 16 + hb * 8) + 1);   // 0 * garbage must stay 0
      o[rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va), __builtin_bit_cast(bf16x8_t, pf), o[rt], 0, 0, 0);
    }
  }
}

// tile_last: the last key that any query of the tile sees
template <int HD, bool FULL, class FRAG>
__device__ __forceinline__ void attn_page32(const bf16* __restrict__ kp, const bf16* __restrict__ vp, const uint4* qf,
                                            int key0, int qpos, int lo, int tile_last, int max_key, float scale2, float& m,
                                            float& l, f32x16_t* o) {
  attn_half32<HD, FULL, FRAG>(kp, vp, qf, 0, key0, qpos, lo, max_key, scale2, m, l, o);
  // the second half of a page on the diagonal may lie wholly behind the tile's last query
  if (FULL || key0 + 32 <= tile_last)
    attn_half32<HD, FULL, FRAG>(kp, vp, qf, 1, key0 + 32, qpos, lo, max_key, scale2, m, l, o);
}

// grid (ceil(G * q_tiles32 / 4), kv heads, sequences); the block order and the page staging are those
// of the 16-query kernel above
template <int HD>
__global__ void __launch_bounds__(AM_WAVES* BLM_WAVE) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 4 : 2, HD <= 64 ? 4 : 2)))
    attn_prefill32_kernel(const bf16* __restrict__ q, int q_row_stride, bf16* __restrict__ out,
                          const int* __restrict__ positions, const int* __restrict__ cu_seqlens,
                          const int* __restrict__ block_table, int table_width,
                          const bf16* __restrict__ kcache, const bf16* __restrict__ vcache, int nh, int nkv,
                          float scale, int window) {
  static_assert(HD % 32 == 0 && HD <= 128, "32-query prefill: head sizes 32, 64, 96, 128");
  constexpr int KS = HD / 16, RT = HD / 32, QT = 32;
  constexpr bool DIRECT = HD == 64 || HD == 128;   // as in the 16-query kernel
  using PAGE = std::conditional_t<DIRECT, SwizzledPage<DIRECT ? HD : 64>, PaddedPage<HD>>;
  using FRAG = std::conditional_t<DIRECT, SwizzledFragments32<DIRECT ? HD : 64>, PaddedFragments32<HD>>;
  constexpr int KSTR = PaddedPage<HD>::KSTR, VSTR = PaddedPage<HD>::VSTR;
  constexpr int CHUNKS = AM_PAGE * HD / 8;
  constexpr int PER_THREAD = (CHUNKS + AM_WAVES * BLM_WAVE - 1) / (AM_WAVES * BLM_WAVE);
  __shared__ __align__(16) bf16 k_lds[2][PAGE::K_ELEMS];
  __shared__ __align__(16) bf16 v_lds[2][PAGE::V_ELEMS];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int j = lane & 31, hb = lane >> 5;
  const int G = nh / nkv;
  const int b = blockIdx.z;
  const int row_begin = cu_seqlens[b];
  const int n_b = cu_seqlens[b + 1] - row_begin;
  const int lin = blockIdx.x + gridDim.x * blockIdx.y;
  const int kvh = lin % nkv;
  int x = lin / nkv;
  {
    const int seg = x >> 5;
    if ((seg & 1) && seg * 32 + 32 <= (int)gridDim.x) x = seg * 32 + 31 - (x & 31);
  }
  const int u0 = ((int)gridDim.x - 1 - x) * AM_WAVES;
  if ((u0 / G) * QT >= n_b) return;   // the whole block lies past the sequence's end (uniform)
  const int u = u0 + wave;
  const int g = u % G, qt = u / G;
  const bool active = qt * QT < n_b;
  const int head = kvh * G + g;
  const int nq = active ? min(QT, n_b - qt * QT) : 1;
  const int row = row_begin + (active ? qt * QT + min(j, nq - 1) : 0);   // columns past the tile's end repeat its last query
  const int qpos = positions[row];
  const int qpos_first = positions[row_begin + (active ? qt * QT : 0)];
  const int qpos_last = positions[row_begin + (active ? qt * QT + nq - 1 : 0)];
  const int seq_last = positions[row_begin + n_b - 1];   // the cache holds data up to here
  const int lo = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  const int lo_tile = (window > 0 && qpos_first - window + 1 > 0) ? qpos_first - window + 1 : 0;
  const int lo_last = (window > 0 && qpos_last - window + 1 > 0) ? qpos_last - window + 1 : 0;
  const int my_first = active ? lo_tile / AM_PAGE : 0x7fffffff, my_last = active ? qpos_last / AM_PAGE : -1;
  const int qt_lo = u0 / G, qt_hi = min((u0 + AM_WAVES - 1) / G, (n_b - 1) / QT);
  const int blk_qfirst = positions[row_begin + qt_lo * QT];
  const int blk_qlast = positions[row_begin + min(qt_hi * QT + QT - 1, n_b - 1)];
  const int blk_first = ((window > 0 && blk_qfirst - window + 1 > 0) ? blk_qfirst - window + 1 : 0) / AM_PAGE;
  const int blk_last = blk_qlast / AM_PAGE;

  uint4 qf[KS];
  {
    const bf16* qrow = q + (size_t)row * q_row_stride + (size_t)head * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const uint4*>(qrow + ks * 16 + hb * 8);
  }
  float m = -INFINITY;
  float lsum = 0.f;
  f32x16_t o[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[rt][v] = 0.f;
  const float scale2 = scale * 1.4426950408889634f;
  PageNumbers pages{block_table + (size_t)b * table_width, table_width, 0, 0};
  pages.load(blk_first);

  u32x4_t kreg[PER_THREAD], vreg[PER_THREAD];
#define AP_FETCH(pi)                                                                          \
  {                                                                                           \
    const size_t base = ((size_t)pages.at(pi) * nkv + kvh) * AM_PAGE * HD;                    \
    _Pragma("unroll") for (int i = 0; i < PER_THREAD; ++i) {                                  \
      const int jj = i * AM_WAVES * BLM_WAVE + threadIdx.x;                                   \
      if (CHUNKS % (AM_WAVES * BLM_WAVE) == 0 || jj < CHUNKS) {                               \
        kreg[i] = *reinterpret_cast<const u32x4_t*>(kcache + base + (size_t)jj * 8);            \
        vreg[i] = *reinterpret_cast<const u32x4_t*>(vcache + base + (size_t)jj * 8);            \
      }                                                                                       \
    }                                                                                         \
  }
#define AP_STAGE(buf)                                                                                         \
  _Pragma("unroll") for (int i = 0; i < PER_THREAD; ++i) {                                                      \
    const int jj = i * AM_WAVES * BLM_WAVE + threadIdx.x;                                                       \
    if (CHUNKS % (AM_WAVES * BLM_WAVE) == 0 || jj < CHUNKS) {                                                   \
      const int kr = jj / (HD / 8), kc = jj - kr * (HD / 8);                                                    \
      *reinterpret_cast<u32x4_t*>(k_lds[buf] + TileOrder32::row_of(kr) * KSTR + kc * 8) = kreg[i];              \
      const int vr = jj / (AM_PAGE / 8), vc = jj - vr * (AM_PAGE / 8);                                          \
      *reinterpret_cast<u32x4_t*>(v_lds[buf] + vr * VSTR + vc * 8) = vreg[i];                                   \
    }                                                                                                           \
  }
#define AP_USE(buf)                                                                                           \
  if (pi >= my_first && pi <= my_last) {                                                                        \
    const int key0 = pi * AM_PAGE;                                                                              \
    if (key0 + AM_PAGE - 1 <= qpos_first && key0 >= lo_last)                                                    \
      attn_page32<HD, true, FRAG>(k_lds[buf], v_lds[buf], qf, key0, qpos, lo, qpos_last, seq_last, scale2, m, lsum, o);  \
    else                                                                                                        \
      attn_page32<HD, false, FRAG>(k_lds[buf], v_lds[buf], qf, key0, qpos, lo, qpos_last, seq_last, scale2, m, lsum, o); \
  }
  if constexpr (DIRECT) {
    DirectStage<DIRECT ? HD : 64, TileOrder32> stage;
    stage.init(k_lds[0], v_lds[0]);
    auto fetch = [&](int pi, int buf) { stage.fetch(kcache, vcache, ((size_t)pages.at(pi) * nkv + kvh) * AM_PAGE * HD, buf); };
    fetch(blk_first, 0);
    am_pin<HD / 16>(qf);   // as in the 16-query kernel
    AM_WAIT_LOADS();
    __syncthreads();
    for (int pi = blk_first; pi <= blk_last; ++pi) {
      const int cur = (pi - blk_first) & 1;
      if (pi < blk_last) fetch(pi + 1, cur ^ 1);   // into the other buffer, which nobody reads now
      AP_USE(cur)
      AM_WAIT_LOADS();
      __syncthreads();     // the next page is in place, and everybody is done with this one
    }
  } else {
    AP_FETCH(blk_first);
    am_pin<HD / 16>(qf);   // as in the 16-query kernel
    AP_STAGE(0)
    __syncthreads();
    for (int pi = blk_first; pi <= blk_last; ++pi) {
      const int cur = (pi - blk_first) & 1;
      if (pi < blk_last) AP_FETCH(pi + 1);   // travels while this page is used
      AP_USE(cur)
      if (pi < blk_last) { AP_STAGE(cur ^ 1) }   // the other buffer: nobody reads it now
      __syncthreads();   // the next page is in place, and everybody is done with this one
    }
  }
#undef AP_STAGE
#undef AP_USE
#undef AP_FETCH
  {   // the two lanes of a query hold the sums over their own keys
    float a, b;
    blm_swap32(lsum, a, b);
    lsum = a + b;
  }
  if (!active || j >= nq) return;
  const float inv = 1.0f / lsum;
  bf16* orow = out + (size_t)row * nh * HD + (size_t)head * HD;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {   // four neighbouring dims per store: rt * 32 + 8 gq + 4 hb ..
      uint2 w;
      w.x = pack_bf16x2(o[rt][4 * gq + 0] * inv, o[rt][4 * gq + 1] * inv);
      w.y = pack_bf16x2(o[rt][4 * gq + 2] * inv, o[rt][4 * gq + 3] * inv);
      *reinterpret_cast<uint2*>(orow + rt * 32 + 8 * gq + 4 * hb) = w;
    }
}

// ---------------------------------------------------------------------------------------
#define AD_MERGE 32   // splits whose partial results are asked for together when they are merged

// decode: grid (splits, kv heads * head tiles, tokens); partial results per split
//   part_o [T, nh, splits, HD] float, part_ml [T, nh, splits, 2] float,
// merged by whichever split of a (token, head tile) finishes last
// ---------------------------------------------------------------------------------------
template <int HD>
__global__ void __launch_bounds__(AM_WAVES* BLM_WAVE)
    attn_decode_mfma_kernel(const bf16* __restrict__ q, int q_row_stride, const int* __restrict__ positions,
                            const int* __restrict__ token_seq, const int* __restrict__ block_table,
                            int table_width, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
                            int nh, int nkv, float scale, int window, int n_splits, float* part_o,
                            float* part_ml, int* arrivals, bf16* out) {
  constexpr int KS = (HD + 31) / 32;
  constexpr int DT = (HD + 15) / 16;
  // Every wavefront brings its pages through a staging area of its own in shared memory: whole
  // pages come in with 16-byte loads that cover complete cache lines and are used once (taking the
  // MFMA fragments straight from global memory touches 16 bytes of 16 lines per instruction, which
  // costs 7 % of a batch-64 step); the fragments are then read from the staged page, whose rows are
  // padded as in the prefill kernel.  Nobody else touches a wavefront's area, so no barrier is
  // needed, and the next page travels in registers while the current one is used.  The areas serve
  // once more at the end, for the wavefronts' partial outputs.
  constexpr int KSTR = PaddedPage<HD>::KSTR, VSTR = PaddedPage<HD>::VSTR;
  constexpr int CHUNKS = AM_PAGE * HD / 8;              // 16-byte pieces of a page (keys and values alike)
  constexpr int PER_LANE = CHUNKS / BLM_WAVE;           // HD is a multiple of 16, so this is exact
  constexpr int STAGE_ELEMS = AM_PAGE * KSTR + HD * VSTR;
  constexpr int AREA_BYTES = STAGE_ELEMS * 2 > 16 * HD * 4 ? STAGE_ELEMS * 2 : 16 * HD * 4;
  static_assert(CHUNKS % BLM_WAVE == 0 && (AM_PAGE * KSTR * 2) % 16 == 0 && AREA_BYTES % 16 == 0, "page staging layout");
  __shared__ float sm_m[AM_WAVES][16], sm_l[AM_WAVES][16];
  __shared__ __align__(16) unsigned char sm_area[AM_WAVES][AREA_BYTES];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  bf16* const k_lds = reinterpret_cast<bf16*>(sm_area[wave]);
  bf16* const v_lds = k_lds + AM_PAGE * KSTR;
  const int c = lane & 15, kg = lane >> 4;
  const int split = blockIdx.x;
  const int G = nh / nkv;
  const int gtiles = (G + 15) / 16;
  const int kvh = blockIdx.y / gtiles, g0 = (blockIdx.y % gtiles) * 16;
  const int t = blockIdx.z;
  const int b = token_seq[t];
  const int head = kvh * G + min(g0 + c, G - 1);   // columns past the group's end repeat its last head

  float m = -INFINITY;
  f32x4_t lsum = {0.f, 0.f, 0.f, 0.f};   // the denominator of query column c, the same in all four places
  f32x4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (b >= 0) {
    const int pos = positions[t];
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int first_page = lo / AM_PAGE, last_page = pos / AM_PAGE;
    const int per_split = (last_page - first_page + 1 + n_splits - 1) / n_splits;
    const int p_begin = first_page + split * per_split;
    const int p_end = min(last_page + 1, p_begin + per_split);
    PageNumbers pages{block_table + (size_t)b * table_width, table_width, 0, 0};
    if (p_begin < p_end) pages.load(p_begin);
    uint4 qf[KS];
    load_q<HD>(q + (size_t)t * q_row_stride + (size_t)head * HD, qf);
    const float scale2 = scale * 1.4426950408889634f;
    u32x4_t kreg[PER_LANE], vreg[PER_LANE];
#define AD_FETCH(pi)                                                                          \
  {                                                                                           \
    const size_t base = ((size_t)pages.at(pi) * nkv + kvh) * AM_PAGE * HD;                    \
    _Pragma("unroll") for (int i = 0; i < PER_LANE; ++i) {                                    \
      const int j = i * BLM_WAVE + lane;                                                      \
      kreg[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kcache + base + (size_t)j * 8));   \
      vreg[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vcache + base + (size_t)j * 8));   \
    }                                                                                         \
  }
#define AD_STAGE()                                                                                            \
  _Pragma("unroll") for (int i = 0; i < PER_LANE; ++i) {                                                        \
    const int j = i * BLM_WAVE + lane;                                                                          \
    const int kr = j / (HD / 8), kc = j - kr * (HD / 8);           /* key, 16-byte column */                    \
    *reinterpret_cast<u32x4_t*>(k_lds + am_row_of(kr) * KSTR + kc * 8) = kreg[i];                               \
    const int vr = j / (AM_PAGE / 8), vc = j - vr * (AM_PAGE / 8); /* value row (a dim), 16-byte column */      \
    *reinterpret_cast<u32x4_t*>(v_lds + vr * VSTR + vc * 8) = vreg[i];                                          \
  }
    int pi = p_begin + wave;
    if (pi < p_end) AD_FETCH(pi);
    am_pin<KS>(qf);   // arrived before the loop, so that no page's first product waits for the page just asked for
    for (; pi < p_end; pi += AM_WAVES) {
      AD_STAGE()
      if (pi + AM_WAVES < p_end) AD_FETCH(pi + AM_WAVES);   // travels while this page is used
      const int key0 = pi * AM_PAGE;
      if (key0 + AM_PAGE - 1 <= pos && key0 >= lo)
        attn_page<HD, true, PaddedPage<HD>>(k_lds, v_lds, qf, key0, pos, lo, pos, scale2, m, lsum, o);
      else
        attn_page<HD, false, PaddedPage<HD>>(k_lds, v_lds, qf, key0, pos, lo, pos, scale2, m, lsum, o);
    }
#undef AD_FETCH
#undef AD_STAGE
  }
  // the staging area is free now: this wavefront's partial output goes there
  float (*const sm_o)[HD] = reinterpret_cast<float (*)[HD]>(sm_area[wave]);
  if (kg == 0) { sm_m[wave][c] = m; sm_l[wave][c] = lsum[0]; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = dt * 16 + kg * 4 + r;
      if (HD % 16 == 0 || d < HD) sm_o[c][d] = o[dt][r];
    }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 16 * HD; idx += blockDim.x) {
    const int cc = idx / HD, d = idx - cc * HD;
    if (g0 + cc >= G) continue;
    float M = sm_m[0][cc];
#pragma unroll
    for (int k = 1; k < AM_WAVES; ++k) M = fmaxf(M, sm_m[k][cc]);
    float L = 0.f, O = 0.f;
#pragma unroll
    for (int k = 0; k < AM_WAVES; ++k) {
      const float f = (sm_m[k][cc] == M) ? 1.f : __builtin_amdgcn_exp2f(sm_m[k][cc] - M);   // maxima are in base 2
      L += sm_l[k][cc] * f;
      O += reinterpret_cast<const float*>(sm_area[k])[cc * HD + d] * f;
    }
    if (n_splits == 1 || b < 0) {   // nothing to merge (a padding token gives zeros)
      out[((size_t)t * nh + kvh * G + g0 + cc) * HD + d] = from_float<bf16>(b < 0 ? 0.f : O / L);
    } else {
      const size_t at = ((size_t)t * nh + kvh * G + g0 + cc) * n_splits + split;
      coherent_store(part_o + at * HD + d, O);
      if (d == 0) { coherent_store(part_ml + at * 2, M); coherent_store(part_ml + at * 2 + 1, L); }
    }
  }
  if (n_splits == 1 || b < 0) return;

  // The block that finishes last among the splits of its (token, head tile) merges them.  Every
  // block writes its partial result with stores that go through to device-coherent memory, waits
  // for them to complete, and then counts itself in; the block that finds all the others counted
  // reads their results with loads that come from device-coherent memory and writes the output.
  // Nobody waits for anybody, and no cache is flushed or invalidated as a whole (a device-wide
  // fence does that on every one of the eight dies, and costs far more than the merge).  The
  // counter goes back to zero for the next launch.
  __shared__ int last;
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's stores have been acknowledged
  __syncthreads();
  int* counter = arrivals + (size_t)t * gridDim.y + blockIdx.y;
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = before == n_splits - 1;
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last) return;
  for (int idx = threadIdx.x; idx < 16 * HD; idx += blockDim.x) {
    const int cc = idx / HD, d = idx - cc * HD;
    if (g0 + cc >= G) continue;
    const size_t head_at = (size_t)t * nh + kvh * G + g0 + cc;
    const size_t base = head_at * n_splits;
    const float* ml = part_ml + base * 2;
    // AD_MERGE splits per memory round trip, merged online (with eight per trip, 64 splits cost 12 us
    // of round trips in a row)
    float M = -INFINITY, L = 0.f, O = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += AD_MERGE) {
      float vm[AD_MERGE], vl[AD_MERGE], po[AD_MERGE];
#pragma unroll
      for (int i = 0; i < AD_MERGE; ++i) {
        const int sp = min(s0 + i, n_splits - 1);
        vm[i] = coherent_load(ml + 2 * sp);
        vl[i] = coherent_load(ml + 2 * sp + 1);
        po[i] = coherent_load(part_o + (base + sp) * HD + d);
      }
      float Mc = M;
#pragma unroll
      for (int i = 0; i < AD_MERGE; ++i) Mc = fmaxf(Mc, vm[i]);
      const float keep = (M == Mc) ? 1.f : __builtin_amdgcn_exp2f(M - Mc);   // maxima are in base 2
      L *= keep;
      O *= keep;
#pragma unroll
      for (int i = 0; i < AD_MERGE; ++i) {
        if (s0 + i < n_splits) {
          const float f = (vm[i] == Mc) ? 1.f : __builtin_amdgcn_exp2f(vm[i] - Mc);
          L += vl[i] * f;
          O += po[i] * f;
        }
      }
      M = Mc;
    }
    out[head_at * HD + d] = from_float<bf16>(O / L);
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
static bool hd_ok(int hd, int max_hd) { return hd >= 16 && hd % 16 == 0 && (hd <= 128 || hd == 256) && hd <= max_hd; }

extern "C" int blm_attn_prefill_mfma_supported(int act_dtype, int hd, int page_size) {
  return (act_dtype == BLM_BF16 && page_size == AM_PAGE && hd_ok(hd, 256)) ? 1 : 0;
}
extern "C" int blm_attn_decode_supported(int act_dtype, int hd, int page_size) {
  return (act_dtype == BLM_BF16 && page_size == AM_PAGE && hd_ok(hd, 128)) ? 1 : 0;
}

// Blocks that the 32-query form would launch (0 if the head size has no such form).
extern "C" long long blm_attn_prefill_blocks32(int n_seqs, int max_new, int nh, int nkv, int hd) {
  if (hd % 32 != 0 || hd > 128 || nkv <= 0 || nh % nkv != 0) return 0;
  const long long units32 = (long long)(nh / nkv) * ((max_new + 31) / 32);
  return (units32 + AM_WAVES - 1) / AM_WAVES * nkv * n_seqs;
}

extern "C" int blm_attn_prefill_mfma(const void* q, int q_row_stride, void* out, int act_dtype,
                                     const int* positions, const int* cu_seqlens, const int* block_table,
                                     int table_width, const void* kcache, const void* vcache, int page_size,
                                     int n_seqs, int max_new, int nh, int nkv, int hd, float scale, int window,
                                     int queries, hipStream_t stream) {
  BLM_REQUIRE(n_seqs > 0 && n_seqs <= 65535 && max_new > 0 && nh > 0 && nkv > 0 && nkv <= 65535 && nh % nkv == 0,
              "attn_prefill_mfma: bad sizes seqs=%d max_new=%d heads=%d kv_heads=%d", n_seqs, max_new, nh, nkv);
  BLM_REQUIRE(blm_attn_prefill_mfma_supported(act_dtype, hd, page_size),
              "attn_prefill_mfma: needs bfloat16, pages of 64 and a head_dim that is a multiple of 16 up to 128, or 256 "
              "(got dtype %d, page %d, head_dim %d)", act_dtype, page_size, hd);
  BLM_REQUIRE(table_width > 0 && window >= 0, "attn_prefill_mfma: bad geometry");
  BLM_REQUIRE(scale > 0.f, "attn_prefill_mfma: the score scale must be positive (got %g)", (double)scale);
  BLM_REQUIRE(q_row_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0,
              "attn_prefill_mfma: q rows must be 16-byte aligned");
  const int G = nh / nkv;
  // queries: 16 or 32 query rows per wavefront.  32 (head sizes 32, 64, 96, 128) halves the shared-memory
  // reads per matrix instruction and is ahead where the work bounds the step (several rounds of blocks); where
  // all blocks run at once the step lasts as long as the block with the most pages, whose pages take longer
  // one after another than those of the 16-query form (measured at 32 heads of 64, 32 against 16 queries:
  // 2,048 tokens 37.6 against 30.5 us, 8,192 tokens 330 against 347, four prompts of 1,024 tokens 48.9 against
  // 37.3, 32 of them 231 against 261; 24 heads of 128: 2,048 tokens 57 against 43, 8,192 tokens 444 against 490).
  // The caller chooses (blm_attn_prefill_blocks32 gives it the number of blocks to compare).
  BLM_REQUIRE(queries == 16 || (queries == 32 && hd % 32 == 0 && hd <= 128),
              "attn_prefill_mfma: %d queries per wavefront with head_dim %d (16, or 32 with head sizes 32, 64, 96, 128)", queries, hd);
  const long long units32 = (long long)G * ((max_new + 31) / 32);
  const bool wide = queries == 32;
  if (hd % 32 == 0 && hd <= 128 && wide) {
    dim3 grid32((unsigned)((units32 + AM_WAVES - 1) / AM_WAVES), nkv, n_seqs), block32(AM_WAVES * BLM_WAVE);
#define BLM_AP32(HD)                                                                                             \
  case HD:                                                                                                       \
    hipLaunchKernelGGL((attn_prefill32_kernel<HD>), grid32, block32, 0, stream, (const bf16*)q, q_row_stride,     \
                       (bf16*)out, positions, cu_seqlens, block_table, table_width, (const bf16*)kcache,          \
                       (const bf16*)vcache, nh, nkv, scale, window);                                              \
    break
    switch (hd) {
      BLM_AP32(32); BLM_AP32(64); BLM_AP32(96); BLM_AP32(128);
    }
#undef BLM_AP32
    BLM_LAUNCH_CHECK("attn_prefill32");
    return 0;
  }
  const long long units = (long long)G * ((max_new + 15) / 16);
  dim3 grid((unsigned)((units + AM_WAVES - 1) / AM_WAVES), nkv, n_seqs), block(AM_WAVES * BLM_WAVE);
#define BLM_AP(HD)                                                                                               \
  case HD:                                                                                                       \
    hipLaunchKernelGGL((attn_prefill_mfma_kernel<HD>), grid, block, 0, stream, (const bf16*)q, q_row_stride,      \
                       (bf16*)out, positions, cu_seqlens, block_table, table_width, (const bf16*)kcache,          \
                       (const bf16*)vcache, nh, nkv, scale, window);                                              \
    break
  switch (hd) {
    BLM_AP(16); BLM_AP(32); BLM_AP(48); BLM_AP(64); BLM_AP(80); BLM_AP(96); BLM_AP(112); BLM_AP(128); BLM_AP(256);
  }
#undef BLM_AP
  BLM_LAUNCH_CHECK("attn_prefill_mfma");
  return 0;
}

// workspace: part_o needs T*nh*n_splits*hd floats, part_ml T*nh*n_splits*2 floats; arrivals needs
// T * kv_heads * ceil(group / 16) ints that are zero before the first call (every call leaves them
// zero again).  Calls that share the arrivals buffer must not overlap in time.
extern "C" int blm_attn_decode(const void* q, int q_row_stride, void* out, int act_dtype, const int* positions,
                               const int* token_seq, const int* block_table, int table_width, const void* kcache,
                               const void* vcache, int page_size, int T, int nh, int nkv, int hd, float scale,
                               int window, int n_splits, float* part_o, float* part_ml, int* arrivals,
                               hipStream_t stream) {
  BLM_REQUIRE(T > 0 && T <= 65535 && nh > 0 && nkv > 0 && nh % nkv == 0,
              "attn_decode: bad sizes T=%d heads=%d kv_heads=%d", T, nh, nkv);
  BLM_REQUIRE(blm_attn_decode_supported(act_dtype, hd, page_size),
              "attn_decode: needs bfloat16, pages of 64 and a head_dim that is a multiple of 16 up to 128 "
              "(got dtype %d, page %d, head_dim %d)", act_dtype, page_size, hd);
  BLM_REQUIRE(table_width > 0 && window >= 0 && n_splits >= 1 && n_splits <= 65535,
              "attn_decode: bad geometry width=%d window=%d splits=%d", table_width, window, n_splits);
  BLM_REQUIRE(q_row_stride % 8 == 0 && ((uintptr_t)q % 16) == 0, "attn_decode: q rows must be 16-byte aligned");
  BLM_REQUIRE(scale > 0.f, "attn_decode: the score scale must be positive (got %g)", (double)scale);
  BLM_REQUIRE(n_splits == 1 || (part_o != nullptr && part_ml != nullptr && arrivals != nullptr),
              "attn_decode: %d splits need the workspaces for partial results and the arrival counters", n_splits);
  const int G = nh / nkv;
  const int gtiles = (G + 15) / 16;
  BLM_REQUIRE((long long)nkv * gtiles <= 65535, "attn_decode: too many heads");
  dim3 grid(n_splits, nkv * gtiles, T), block(AM_WAVES * BLM_WAVE);
#define BLM_AD(HD)                                                                                                 \
  case HD:                                                                                                         \
    hipLaunchKernelGGL((attn_decode_mfma_kernel<HD>), grid, block, 0, stream, (const bf16*)q, q_row_stride,         \
                       positions, token_seq, block_table, table_width, (const bf16*)kcache, (const bf16*)vcache,    \
                       nh, nkv, scale, window, n_splits, part_o, part_ml, arrivals, (bf16*)out);                    \
    break
  switch (hd) { BLM_AD(16); BLM_AD(32); BLM_AD(48); BLM_AD(64); BLM_AD(80); BLM_AD(96); BLM_AD(112); BLM_AD(128); }
#undef BLM_AD
  BLM_LAUNCH_CHECK("attn_decode_mfma");
  return 0;
}
