// Attention over the paged cache, generic form: one wavefront per (query token, head).
// Works for prefill (many query tokens per sequence) and decode (one), any even head size up
// to 256, any head and group counts, float or bf16 storage.  Scores, the running maximum and
// sum and the output accumulator are float.  Keys and values of the step's own tokens are
// already in the cache when this runs.  Key pages are [kv head][token][head_dim], value pages
// [kv head][head_dim][token].
//
// Visibility: the query at position p of its sequence sees keys j of the same sequence with
// j <= p and, if window > 0, p - j < window.
//
// With n_splits > 1 (few query tokens over long key ranges: decode) the key range of every
// (token, head) is cut into that many pieces handled by different wavefronts (blockIdx.y).  Each
// writes its partial maximum, sum and output with stores that reach device-coherent memory, waits
// for them to complete and counts itself in; the wavefront that finds all the others counted reads
// their partial results back and writes the output.  Nobody waits for anybody.
#include "common.h"

template <typename T>
struct Vec8;
template <>
struct Vec8<bf16> {
  uint4 raw;
  __device__ __forceinline__ void load(const bf16* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = (&raw.x)[i >> 1];
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
};
template <>
struct Vec8<float> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? (&a.x)[i] : (&b.x)[i - 4]; }
};

#define ATTN_WAVES 4
#define ATTN_MAX_HD 256
#define ATTN_STAGE_LDS (64 * 1024)       // most shared memory of the form that stages values, as a kernel gets it without asking
#define ATTN_STAGE_LDS_BIG (144 * 1024)  // and after blm_attn_paged_init on the device (head sizes up to 128 in four wavefronts)

// STAGE: the values of a chunk of 64 keys go through shared memory.  A value page keeps a head lane's
// tokens next to each other, so with one lane per key the 64 lanes read 64 neighbouring values per
// head lane (one line), and write them transposed into a tile of the wavefront's own ([key][lane],
// rows padded by one float); the weighted sum then reads the tile with one lane per head lane.
// Without it every lane reads 4 bytes of a line of its own for every key.  The tile is 64 * (hd + 1)
// floats per wavefront.
template <typename TA, bool VEC, bool STAGE, bool SHARE>
__global__ void __launch_bounds__(ATTN_WAVES* BLM_WAVE)
    attn_paged_kernel(const TA* __restrict__ q, int q_row_stride, TA* __restrict__ out,
                      const int* __restrict__ positions, const int* __restrict__ token_seq,
                      const int* __restrict__ block_table, int table_width,
                      const TA* __restrict__ kcache, const TA* __restrict__ vcache, int page_size,
                      int T, int nh, int nkv, int hd, float scale, int window, int n_splits, float* part_o,
                      float* part_ml, int* arrivals) {
  static_assert(STAGE || !SHARE, "shared tiles are staged tiles");
  constexpr bool share = SHARE;
  extern __shared__ float smem[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long w = (long long)blockIdx.x * ATTN_WAVES + wave;
  const bool active = w < (long long)T * nh;
  const int t = active ? (int)(w / nh) : 0;
  const int head = active ? (int)(w - (long long)t * nh) : 0;
  const int b = active ? token_seq[t] : -1;
  float* qs = smem + wave * hd;
  // STAGE: this wavefront's tile of values; with `share` (the block's wavefronts are heads of one group
  // and work on the same token: groups of a multiple of four heads) one tile of keys and one of values
  // for the whole block, filled by all its threads, so the group's keys and values are read once
  float* kt = smem + ATTN_WAVES * hd;
  float* vt = share ? kt + (size_t)BLM_WAVE * (hd + 1) : kt + (size_t)wave * BLM_WAVE * (hd + 1);
  if (active && b >= 0) {
    const TA* qrow = q + (size_t)t * q_row_stride + (size_t)head * hd;
    for (int d = lane; d < hd; d += BLM_WAVE) qs[d] = to_float(qrow[d]);
  }
  __syncthreads();
  if (!active) return;
  TA* orow = out + ((size_t)t * nh + head) * hd;
  if (b < 0) {  // padding token: defined output, no cache access
    for (int d = lane; d < hd; d += BLM_WAVE) orow[d] = from_float<TA>(0.f);
    return;
  }
  const int pos = positions[t];
  const int kvh = head / (nh / nkv);
  const int* bt = block_table + (size_t)b * table_width;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // this wavefront's piece of the key range, in chunks of one wavefront's width
  const int split = blockIdx.y;
  const int n_chunks = (pos - first) / BLM_WAVE + 1;
  const int per_split = (n_chunks + n_splits - 1) / n_splits;
  const int j_begin = first + split * per_split * BLM_WAVE;
  const int j_end = min(pos, j_begin + per_split * BLM_WAVE - 1);   // last key of the piece

  float m = -INFINITY, l = 0.f;
  float acc[ATTN_MAX_HD / BLM_WAVE] = {0.f, 0.f, 0.f, 0.f};

  for (int j0 = j_begin; j0 <= j_end; j0 += BLM_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= j_end;
    float s = -INFINITY;
    if constexpr (SHARE) {
      __syncthreads();   // nobody reads the last chunk's tiles any more
      {   // keys: four threads per key, neighbouring threads neighbouring lanes of the head
        const int key = threadIdx.x >> 2, jk = j0 + key;
        if (jk <= j_end) {
          const int page = bt[jk / page_size];
          const TA* krow = kcache + (((size_t)page * nkv + kvh) * page_size + (jk % page_size)) * hd;
          for (int d = threadIdx.x & 3; d < hd; d += 4) kt[(size_t)key * (hd + 1) + d] = to_float(krow[d]);
        }
      }
      {   // values: a wavefront reads the 64 keys of one head lane, which are neighbours in the page
        const int jk = j0 + lane;
        if (jk <= j_end) {
          const int page = bt[jk / page_size];
          const TA* vcol = vcache + ((size_t)page * nkv + kvh) * page_size * hd + (jk % page_size);
          for (int d = wave; d < hd; d += ATTN_WAVES) vt[(size_t)lane * (hd + 1) + d] = to_float(vcol[(size_t)d * page_size]);
        }
      }
      __syncthreads();
      if (valid) {
        const float* krow = kt + (size_t)lane * (hd + 1);
        float dot = 0.f;
        for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], krow[d], dot);
        s = dot * scale;
      }
    } else if (valid) {
      const int page = bt[j / page_size];
      const TA* krow = kcache + (((size_t)page * nkv + kvh) * page_size + (j % page_size)) * hd;
      float dot = 0.f;
      if (VEC) {
        for (int d = 0; d < hd; d += 8) {
          Vec8<TA> kv;
          kv.load(krow + d);
#pragma unroll
          for (int i = 0; i < 8; ++i) dot = fmaf(qs[d + i], kv.get(i), dot);
        }
      } else {
        for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_float(krow[d]), dot);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // 0 on the first chunk (m = -inf, m_new finite)
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) acc[i] *= corr;
    const int cnt = (j_end - j0 + 1) < BLM_WAVE ? (j_end - j0 + 1) : BLM_WAVE;
    if (STAGE) {
      if (valid && !share) {
        const int page = bt[j / page_size];
        const TA* vcol = vcache + ((size_t)page * nkv + kvh) * page_size * hd + (j % page_size);
        float* mine = vt + (size_t)lane * (hd + 1);
        for (int d = 0; d < hd; ++d) mine[d] = to_float(vcol[(size_t)d * page_size]);
      }
      __builtin_amdgcn_wave_barrier();   // the tile is the wavefront's own: its reads follow its writes in order
      for (int jj = 0; jj < cnt; ++jj) {
        const float pj = __shfl(p, jj, BLM_WAVE);
        const float* vrow = vt + (size_t)jj * (hd + 1);
#pragma unroll
        for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
          const int d = lane + i * BLM_WAVE;
          if (d < hd) acc[i] = fmaf(pj, vrow[d], acc[i]);
        }
      }
      __builtin_amdgcn_wave_barrier();   // the next chunk's writes follow these reads
    } else
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = __shfl(p, jj, BLM_WAVE);
      const int ja = j0 + jj;
      const int page = bt[ja / page_size];
      const TA* vcol = vcache + ((size_t)page * nkv + kvh) * page_size * hd + (ja % page_size);
#pragma unroll
      for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
        const int d = lane + i * BLM_WAVE;
        if (d < hd) acc[i] = fmaf(pj, to_float(vcol[(size_t)d * page_size]), acc[i]);
      }
    }
    m = m_new;
  }
  if (n_splits == 1) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
      const int d = lane + i * BLM_WAVE;
      if (d < hd) orow[d] = from_float<TA>(acc[i] * inv);
    }
    return;
  }
  // publish this piece (an empty piece has m = -inf, l = 0 and counts for nothing)
  const size_t item = (size_t)t * nh + head;
  float* po = part_o + (item * n_splits + split) * hd;
#pragma unroll
  for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
    const int d = lane + i * BLM_WAVE;
    if (d < hd) __hip_atomic_store(po + d, acc[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (lane == 0) {
    __hip_atomic_store(part_ml + (item * n_splits + split) * 2, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(part_ml + (item * n_splits + split) * 2 + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the wavefront's stores have been acknowledged
  int last = 0;
  if (lane == 0) {
    const int before = __hip_atomic_fetch_add(arrivals + item, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = before == n_splits - 1;
    if (last) __hip_atomic_store(arrivals + item, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero again for the next launch
  }
  last = __shfl(last, 0, BLM_WAVE);
  if (!last) return;
  float M = -INFINITY, L = 0.f;
  float O[ATTN_MAX_HD / BLM_WAVE] = {0.f, 0.f, 0.f, 0.f};
  for (int sp = 0; sp < n_splits; ++sp) {
    const float* ml = part_ml + (item * n_splits + sp) * 2;
    const float ms = __hip_atomic_load(ml, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float ls = __hip_atomic_load(ml + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (ls == 0.f) continue;
    const float Mn = fmaxf(M, ms);
    const float keep = expf(M - Mn), take = expf(ms - Mn);   // exp(-inf) = 0 on the first piece
    L = L * keep + ls * take;
    const float* ps = part_o + (item * n_splits + sp) * hd;
#pragma unroll
    for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
      const int d = lane + i * BLM_WAVE;
      if (d < hd) O[i] = O[i] * keep + __hip_atomic_load(ps + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * take;
    }
    M = Mn;
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
    const int d = lane + i * BLM_WAVE;
    if (d < hd) orow[d] = from_float<TA>(O[i] * inv);
  }
}

// Once per device, outside any stream capture: lets the form that stages values ask for more shared
// memory than a kernel gets without asking.  Without it that form serves head sizes up to 62 only.
#define ATTN_DEVICES 64
static bool g_attn_big_lds[ATTN_DEVICES];
extern "C" int blm_attn_paged_init() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  BLM_REQUIRE(e == hipSuccess && dev >= 0, "attn_paged_init: hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev >= ATTN_DEVICES) return 0;   // such a device keeps the small limit
  const void* kernels[] = {(const void*)attn_paged_kernel<float, true, true, false>, (const void*)attn_paged_kernel<float, false, true, false>,
                           (const void*)attn_paged_kernel<bf16, true, true, false>,  (const void*)attn_paged_kernel<bf16, false, true, false>,
                           (const void*)attn_paged_kernel<float, true, true, true>,  (const void*)attn_paged_kernel<float, false, true, true>,
                           (const void*)attn_paged_kernel<bf16, true, true, true>,   (const void*)attn_paged_kernel<bf16, false, true, true>};
  for (const void* k : kernels) {
    e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, ATTN_STAGE_LDS_BIG);
    BLM_REQUIRE(e == hipSuccess, "attn_paged_init: cannot raise the shared memory limit: %s", hipGetErrorString(e));
  }
  g_attn_big_lds[dev] = true;
  return 0;
}

// part_o: T*nh*n_splits*hd floats, part_ml: T*nh*n_splits*2 floats, arrivals: T*nh ints that are
// zero before the first call (every call leaves them zero again); all three may be null when
// n_splits is 1.  Calls that share the arrivals buffer must not overlap in time.
extern "C" int blm_attn_paged(const void* q, int q_row_stride, void* out, int act_dtype,
                              const int* positions, const int* token_seq, const int* block_table,
                              int table_width, const void* kcache, const void* vcache,
                              int page_size, int T, int nh, int nkv, int hd, float scale,
                              int window, int n_splits, float* part_o, float* part_ml, int* arrivals,
                              hipStream_t stream) {
  BLM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && nh % nkv == 0,
              "attn_paged: bad sizes T=%d heads=%d kv_heads=%d (heads must be a multiple of kv_heads)", T, nh, nkv);
  BLM_REQUIRE(hd > 0 && hd % 2 == 0 && hd <= ATTN_MAX_HD,
              "attn_paged: head_dim %d not supported (even, at most %d)", hd, ATTN_MAX_HD);
  BLM_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "attn_paged: bad cache geometry");
  BLM_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || (part_o && part_ml && arrivals)),
              "attn_paged: %d splits need their workspace", n_splits);
  const long long items = (long long)T * nh;
  const long long blocks = (items + ATTN_WAVES - 1) / ATTN_WAVES;
  BLM_REQUIRE(blocks < 2147483647LL, "attn_paged: too many (token, head) pairs: %lld", items);
  dim3 grid((unsigned)blocks, (unsigned)n_splits), block(ATTN_WAVES * BLM_WAVE);
  // the values' tiles fit the shared memory a kernel gets without asking up to a head size of 62, after
  // blm_attn_paged_init up to 139; larger heads take the direct form
  // heads of one group in one block: the group's keys and values are staged once for all of them.  Only
  // where blocks are plentiful (prompts): the block then meets twice per chunk, which a decode step's few
  // blocks cannot hide (float32 at the 1B shape: prefill of 2,048 tokens 120 ms against 164, but a
  // decode step of batch 8 4.7 ms against 4.3).
  const int share = ((nh / nkv) % ATTN_WAVES == 0 && blocks >= 2048) ? 1 : 0;
  const size_t tiles = (size_t)(share ? 2 : ATTN_WAVES) * BLM_WAVE * (hd + 1) * sizeof(float);
  int dev = -1;
  const bool big = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < ATTN_DEVICES && g_attn_big_lds[dev];
  const bool stage = (size_t)ATTN_WAVES * hd * sizeof(float) + tiles <= (size_t)(big ? ATTN_STAGE_LDS_BIG : ATTN_STAGE_LDS);
  const size_t smem = (size_t)ATTN_WAVES * hd * sizeof(float) + (stage ? tiles : 0);
  const bool vec = (hd % 8) == 0 && (q_row_stride % 8) == 0;
#define BLM_ATTN_CASE(TA, V, S, H)                                                                  \
  hipLaunchKernelGGL((attn_paged_kernel<TA, V, S, H>), grid, block, smem, stream, (const TA*)q, q_row_stride, \
                     (TA*)out, positions, token_seq, block_table, table_width, (const TA*)kcache,    \
                     (const TA*)vcache, page_size, T, nh, nkv, hd, scale, window, n_splits, part_o, part_ml, arrivals)
#define BLM_ATTN_PICK(TA)                                                                           \
  do {                                                                                              \
    if (stage && share) { if (vec) BLM_ATTN_CASE(TA, true, true, true); else BLM_ATTN_CASE(TA, false, true, true); } \
    else if (stage) { if (vec) BLM_ATTN_CASE(TA, true, true, false); else BLM_ATTN_CASE(TA, false, true, false); }   \
    else { if (vec) BLM_ATTN_CASE(TA, true, false, false); else BLM_ATTN_CASE(TA, false, false, false); }            \
  } while (0)
  if (act_dtype == BLM_F32) BLM_ATTN_PICK(float);
  else if (act_dtype == BLM_BF16) BLM_ATTN_PICK(bf16);
  else return blm_fail("attn_paged: unsupported dtype %d", act_dtype);
#undef BLM_ATTN_PICK
#undef BLM_ATTN_CASE
  BLM_LAUNCH_CHECK("attn_paged");
  return 0;
}
