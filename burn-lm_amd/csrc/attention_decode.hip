// Decode attention over the paged cache: few query tokens, long key ranges.
//
// The key range of every (query token, key-value head) is cut into splits; one block of four
// wavefronts works on one split for all query heads of the group, so each key and value is
// loaded once for the whole group.  A key row is spread over LPK = head_dim / (16 bytes) lanes;
// a wavefront therefore reads 64 / LPK consecutive keys with one 16-byte load per lane, which
// is one contiguous kilobyte of a page.  Every lane keeps an online softmax (running maximum,
// sum, output accumulator, all float) over the keys of its stream; the streams of a wavefront,
// the wavefronts of a block and finally the splits are merged with the usual
// (max, sum, accumulator) rule.  Scores, softmax and accumulation are float.
//
// Head sizes: powers of two from 16 to 256 (other sizes take the generic kernel).
// Query heads per key-value head: any (processed GT at a time).
#include "common.h"

#define AD_WAVES 4

template <typename T>
struct Row16;  // 16 bytes of a row as floats
template <>
struct Row16<bf16> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void load(const bf16* p, float* v) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <>
struct Row16<float> {
  static constexpr int N = 4;
  __device__ static __forceinline__ void load(const float* p, float* v) {
    const float4 r = *reinterpret_cast<const float4*>(p);
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
};

__device__ __forceinline__ void merge_state(float& m, float& l, float* acc, int n, float m2, float l2,
                                            const float* acc2) {
  const float M = fmaxf(m, m2);
  const float f1 = (m == M) ? 1.f : expf(m - M);    // m = -inf, M finite -> 0;  both -inf -> 1 (l = 0 anyway)
  const float f2 = (m2 == M) ? 1.f : expf(m2 - M);
  l = l * f1 + l2 * f2;
#pragma unroll
  for (int i = 0; i < n; ++i) acc[i] = acc[i] * f1 + acc2[i] * f2;
  m = M;
}

// partial results: part_o [T, nh, splits, HD] float, part_ml [T, nh, splits, 2] float
template <typename TA, int HD, int GT>
__global__ void __launch_bounds__(AD_WAVES* BLM_WAVE)
    attn_decode_split_kernel(const TA* __restrict__ q, int q_row_stride, const int* __restrict__ positions,
                             const int* __restrict__ token_seq, const int* __restrict__ block_table,
                             int table_width, const TA* __restrict__ kcache, const TA* __restrict__ vcache,
                             int page_size, int nh, int nkv, float scale, int window, int n_splits,
                             float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int EPL = Row16<TA>::N;       // elements per lane
  constexpr int LPK = HD / EPL;           // lanes per key
  constexpr int KPW = BLM_WAVE / LPK;     // keys per wavefront load
  static_assert(LPK >= 1 && LPK <= BLM_WAVE && (LPK & (LPK - 1)) == 0, "head size must map to a power-of-two lane count");
  const int split = blockIdx.x;
  const int G = nh / nkv;
  const int chunks = (G + GT - 1) / GT;
  const int kvh = blockIdx.y / chunks;
  const int g0 = (blockIdx.y % chunks) * GT;   // first query head of the group handled here
  const int t = blockIdx.z;
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int stream = lane / LPK, sub = lane % LPK;
  const int b = token_seq[t];

  __shared__ float sm_m[AD_WAVES][GT], sm_l[AD_WAVES][GT];
  __shared__ float sm_o[AD_WAVES][GT][HD];

  float m[GT], l[GT], acc[GT][EPL], qv[GT][EPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[g][i] = 0.f;
  }

  if (b >= 0) {
    const int pos = positions[t];
    const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    // page-aligned split of [first_page, last_page]
    const int first_page = first / page_size, last_page = pos / page_size;
    const int n_pages = last_page - first_page + 1;
    const int pages_per_split = (n_pages + n_splits - 1) / n_splits;
    const int p_begin = first_page + split * pages_per_split;
    const int p_end = min(last_page + 1, p_begin + pages_per_split);
    const int* bt = block_table + (size_t)b * table_width;

#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const int head = kvh * G + g0 + g;
      float tmp[EPL];
      if (g0 + g < G) {
        Row16<TA>::load(q + (size_t)t * q_row_stride + (size_t)head * HD + sub * EPL, tmp);
      } else {
#pragma unroll
        for (int i = 0; i < EPL; ++i) tmp[i] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < EPL; ++i) qv[g][i] = tmp[i] * scale;
    }

    for (int pi = p_begin + wave; pi < p_end; pi += AD_WAVES) {
      const int page = bt[pi];
      const size_t base = ((size_t)page * nkv + kvh) * page_size * HD;
      const TA* kp = kcache + base;
      const TA* vp = vcache + base;
      const int j0 = pi * page_size;
      for (int it = 0; it < page_size; it += KPW) {
        const int kidx = it + stream;
        const int j = j0 + kidx;
        const bool valid = kidx < page_size && j >= first && j <= pos;
        float kf[EPL], vf[EPL];
        if (kidx < page_size) {
          Row16<TA>::load(kp + (size_t)kidx * HD + sub * EPL, kf);
          Row16<TA>::load(vp + (size_t)kidx * HD + sub * EPL, vf);
        }
        if (!valid) {
#pragma unroll
          for (int i = 0; i < EPL; ++i) { kf[i] = 0.f; vf[i] = 0.f; }
        }
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          float s = 0.f;
#pragma unroll
          for (int i = 0; i < EPL; ++i) s = fmaf(qv[g][i], kf[i], s);
#pragma unroll
          for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, BLM_WAVE);
          s = valid ? s : -INFINITY;
          const float m_new = fmaxf(m[g], s);
          const float corr = (m[g] == m_new) ? 1.f : expf(m[g] - m_new);
          const float p = valid ? expf(s - m_new) : 0.f;
          l[g] = l[g] * corr + p;
#pragma unroll
          for (int i = 0; i < EPL; ++i) acc[g][i] = fmaf(p, vf[i], acc[g][i] * corr);
          m[g] = m_new;
        }
      }
    }
    // merge the key streams of the wavefront (lanes with equal `sub`)
#pragma unroll
    for (int g = 0; g < GT; ++g) {
#pragma unroll
      for (int o = LPK; o < BLM_WAVE; o <<= 1) {
        const float m2 = __shfl_xor(m[g], o, BLM_WAVE);
        const float l2 = __shfl_xor(l[g], o, BLM_WAVE);
        float a2[EPL];
#pragma unroll
        for (int i = 0; i < EPL; ++i) a2[i] = __shfl_xor(acc[g][i], o, BLM_WAVE);
        merge_state(m[g], l[g], acc[g], EPL, m2, l2, a2);
      }
    }
  }
  // merge the wavefronts of the block through shared memory
  if (stream == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (sub == 0) { sm_m[wave][g] = m[g]; sm_l[wave][g] = l[g]; }
#pragma unroll
      for (int i = 0; i < EPL; ++i) sm_o[wave][g][sub * EPL + i] = acc[g][i];
    }
  }
  __syncthreads();
  for (int w = threadIdx.x; w < GT * HD; w += blockDim.x) {
    const int g = w / HD, d = w - g * HD;
    if (g0 + g >= G) continue;
    float M = sm_m[0][g];
#pragma unroll
    for (int k = 1; k < AD_WAVES; ++k) M = fmaxf(M, sm_m[k][g]);
    float L = 0.f, O = 0.f;
#pragma unroll
    for (int k = 0; k < AD_WAVES; ++k) {
      const float f = (sm_m[k][g] == M) ? 1.f : expf(sm_m[k][g] - M);
      L += sm_l[k][g] * f;
      O += sm_o[k][g][d] * f;
    }
    const int head = kvh * G + g0 + g;
    const size_t idx = ((size_t)t * nh + head) * n_splits + split;
    part_o[idx * HD + d] = O;
    if (d == 0) { part_ml[idx * 2] = M; part_ml[idx * 2 + 1] = L; }
  }
}

template <typename TA, int HD>
__global__ void attn_decode_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                           const int* __restrict__ token_seq, TA* __restrict__ out, int nh,
                                           int n_splits) {
  const int head = blockIdx.x, t = blockIdx.y;
  const int d = threadIdx.x;
  if (d >= HD) return;
  TA* o = out + ((size_t)t * nh + head) * HD;
  if (token_seq[t] < 0) { o[d] = from_float<TA>(0.f); return; }
  const size_t base = ((size_t)t * nh + head) * n_splits;
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, part_ml[(base + s) * 2]);
  float L = 0.f, O = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = part_ml[(base + s) * 2];
    const float f = (ms == M) ? 1.f : expf(ms - M);
    L += part_ml[(base + s) * 2 + 1] * f;
    O += part_o[(base + s) * HD + d] * f;
  }
  o[d] = from_float<TA>(O / L);
}

template <typename TA, int HD, int GT>
static int launch_decode(const void* q, int q_row_stride, void* out, const int* positions, const int* token_seq,
                         const int* block_table, int table_width, const void* kcache, const void* vcache,
                         int page_size, int T, int nh, int nkv, float scale, int window, int n_splits,
                         float* part_o, float* part_ml, hipStream_t stream) {
  const int G = nh / nkv;
  const int chunks = (G + GT - 1) / GT;
  dim3 grid(n_splits, nkv * chunks, T), block(AD_WAVES * BLM_WAVE);
  hipLaunchKernelGGL((attn_decode_split_kernel<TA, HD, GT>), grid, block, 0, stream, (const TA*)q, q_row_stride,
                     positions, token_seq, block_table, table_width, (const TA*)kcache, (const TA*)vcache, page_size,
                     nh, nkv, scale, window, n_splits, part_o, part_ml);
  BLM_LAUNCH_CHECK("attn_decode_split");
  dim3 cgrid(nh, T), cblock(HD < 64 ? 64 : HD);
  hipLaunchKernelGGL((attn_decode_combine_kernel<TA, HD>), cgrid, cblock, 0, stream, part_o, part_ml, token_seq,
                     (TA*)out, nh, n_splits);
  BLM_LAUNCH_CHECK("attn_decode_combine");
  return 0;
}

template <typename TA, int HD>
static int dispatch_g(int G, const void* q, int q_row_stride, void* out, const int* positions, const int* token_seq,
                      const int* block_table, int table_width, const void* kcache, const void* vcache, int page_size,
                      int T, int nh, int nkv, float scale, int window, int n_splits, float* part_o, float* part_ml,
                      hipStream_t stream) {
#define BLM_AD(GT)                                                                                              \
  return launch_decode<TA, HD, GT>(q, q_row_stride, out, positions, token_seq, block_table, table_width, kcache, \
                                   vcache, page_size, T, nh, nkv, scale, window, n_splits, part_o, part_ml, stream)
  if (G == 1) BLM_AD(1);
  if (G == 2) BLM_AD(2);
  if (G <= 4) BLM_AD(4);
  BLM_AD(8);
#undef BLM_AD
}

// 1 if the fast kernel takes this head size and dtype, else 0 (then the generic kernel is used)
extern "C" int blm_attn_decode_supported(int act_dtype, int hd) {
  if (act_dtype != BLM_F32 && act_dtype != BLM_BF16) return 0;
  const int min_hd = act_dtype == BLM_BF16 ? 16 : 8;
  return (hd >= min_hd && hd <= 256 && (hd & (hd - 1)) == 0) ? 1 : 0;
}

// workspace: part_o needs T*nh*n_splits*hd floats, part_ml T*nh*n_splits*2 floats
extern "C" int blm_attn_decode(const void* q, int q_row_stride, void* out, int act_dtype, const int* positions,
                               const int* token_seq, const int* block_table, int table_width, const void* kcache,
                               const void* vcache, int page_size, int T, int nh, int nkv, int hd, float scale,
                               int window, int n_splits, float* part_o, float* part_ml, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && T <= 65535 && nh > 0 && nkv > 0 && nh % nkv == 0,
              "attn_decode: bad sizes T=%d heads=%d kv_heads=%d", T, nh, nkv);
  BLM_REQUIRE(blm_attn_decode_supported(act_dtype, hd), "attn_decode: head_dim %d / dtype %d not supported "
              "(powers of two from 16 to 256)", hd, act_dtype);
  BLM_REQUIRE(page_size > 0 && table_width > 0 && window >= 0 && n_splits >= 1 && n_splits <= 65535,
              "attn_decode: bad geometry page=%d width=%d window=%d splits=%d", page_size, table_width, window, n_splits);
  BLM_REQUIRE(q_row_stride % 8 == 0 && ((uintptr_t)q % 16) == 0, "attn_decode: q rows must be 16-byte aligned");
  const int G = nh / nkv;
#define BLM_AD_HD(TA, HD)                                                                                      \
  case HD: return dispatch_g<TA, HD>(G, q, q_row_stride, out, positions, token_seq, block_table, table_width,   \
                                     kcache, vcache, page_size, T, nh, nkv, scale, window, n_splits, part_o,    \
                                     part_ml, stream)
  if (act_dtype == BLM_BF16) {
    switch (hd) {
      BLM_AD_HD(bf16, 16); BLM_AD_HD(bf16, 32); BLM_AD_HD(bf16, 64); BLM_AD_HD(bf16, 128); BLM_AD_HD(bf16, 256);
    }
  } else {
    switch (hd) {
      BLM_AD_HD(float, 8); BLM_AD_HD(float, 16); BLM_AD_HD(float, 32); BLM_AD_HD(float, 64); BLM_AD_HD(float, 128);
      BLM_AD_HD(float, 256);
    }
  }
#undef BLM_AD_HD
  return blm_fail("attn_decode: head_dim %d not dispatched", hd);
}
