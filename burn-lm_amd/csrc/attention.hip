// Attention over the paged cache, generic form: one wavefront per (query token, head).
// Works for prefill (many query tokens per sequence) and decode (one), any even head size up
// to 256, any head and group counts, float or bf16 storage.  Scores, the running maximum and
// sum and the output accumulator are float.  Keys and values of the step's own tokens are
// already in the cache when this runs.  Key pages are [kv head][token][head_dim], value pages
// [kv head][head_dim][token].
//
// Visibility: the query at position p of its sequence sees keys j of the same sequence with
// j <= p and, if window > 0, p - j < window.
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

template <typename TA, bool VEC>
__global__ void __launch_bounds__(ATTN_WAVES* BLM_WAVE)
    attn_paged_kernel(const TA* __restrict__ q, int q_row_stride, TA* __restrict__ out,
                      const int* __restrict__ positions, const int* __restrict__ token_seq,
                      const int* __restrict__ block_table, int table_width,
                      const TA* __restrict__ kcache, const TA* __restrict__ vcache, int page_size,
                      int T, int nh, int nkv, int hd, float scale, int window) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long w = (long long)blockIdx.x * ATTN_WAVES + wave;
  const bool active = w < (long long)T * nh;
  const int t = active ? (int)(w / nh) : 0;
  const int head = active ? (int)(w - (long long)t * nh) : 0;
  const int b = active ? token_seq[t] : -1;
  float* qs = smem + wave * hd;
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

  float m = -INFINITY, l = 0.f;
  float acc[ATTN_MAX_HD / BLM_WAVE] = {0.f, 0.f, 0.f, 0.f};

  for (int j0 = first; j0 <= pos; j0 += BLM_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    if (valid) {
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
    const int cnt = (pos - j0 + 1) < BLM_WAVE ? (pos - j0 + 1) : BLM_WAVE;
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
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ATTN_MAX_HD / BLM_WAVE; ++i) {
    const int d = lane + i * BLM_WAVE;
    if (d < hd) orow[d] = from_float<TA>(acc[i] * inv);
  }
}

extern "C" int blm_attn_paged(const void* q, int q_row_stride, void* out, int act_dtype,
                              const int* positions, const int* token_seq, const int* block_table,
                              int table_width, const void* kcache, const void* vcache,
                              int page_size, int T, int nh, int nkv, int hd, float scale,
                              int window, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && nh % nkv == 0,
              "attn_paged: bad sizes T=%d heads=%d kv_heads=%d (heads must be a multiple of kv_heads)", T, nh, nkv);
  BLM_REQUIRE(hd > 0 && hd % 2 == 0 && hd <= ATTN_MAX_HD,
              "attn_paged: head_dim %d not supported (even, at most %d)", hd, ATTN_MAX_HD);
  BLM_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "attn_paged: bad cache geometry");
  const long long items = (long long)T * nh;
  const long long blocks = (items + ATTN_WAVES - 1) / ATTN_WAVES;
  BLM_REQUIRE(blocks < 2147483647LL, "attn_paged: too many (token, head) pairs: %lld", items);
  dim3 grid((unsigned)blocks), block(ATTN_WAVES * BLM_WAVE);
  const size_t smem = (size_t)ATTN_WAVES * hd * sizeof(float);
  const bool vec = (hd % 8) == 0 && (q_row_stride % 8) == 0;
#define BLM_ATTN_CASE(TA, V)                                                                        \
  hipLaunchKernelGGL((attn_paged_kernel<TA, V>), grid, block, smem, stream, (const TA*)q, q_row_stride, \
                     (TA*)out, positions, token_seq, block_table, table_width, (const TA*)kcache,    \
                     (const TA*)vcache, page_size, T, nh, nkv, hd, scale, window)
  if (act_dtype == BLM_F32) {
    if (vec) BLM_ATTN_CASE(float, true); else BLM_ATTN_CASE(float, false);
  } else if (act_dtype == BLM_BF16) {
    if (vec) BLM_ATTN_CASE(bf16, true); else BLM_ATTN_CASE(bf16, false);
  } else {
    return blm_fail("attn_paged: unsupported dtype %d", act_dtype);
  }
#undef BLM_ATTN_CASE
  BLM_LAUNCH_CHECK("attn_paged");
  return 0;
}
