// Token choice from float logits.
//   argmax : first index of the maximum (lowest index wins ties); a row is searched by 32 blocks.
//   sample : softmax(logits / temperature) in float, nucleus (top-p) cut, inverse-CDF pick at a
//            uniform number u given by the caller, walking the kept tokens in index order; one
//            block per row.
// Nucleus rule: a token is kept while the probability mass of the tokens strictly more likely
// than it is below p; so the token that crosses p is kept, and tokens tied with it are too.
//
// The weight of a token is e = 2^((x - max) * log2(e) / temperature), in (0, 1].  The smallest
// kept weight is found by a radix selection over the bit pattern of e (positive floats order like
// their bits): three passes over the row with histograms of 11, 11 and 8 bits, each bin holding
// the mass of its tokens.  Mass is summed as 64-bit integers (e * 2^32, truncated), so the sums do
// not depend on the order in which the shared-memory atomics land and the same logits always give
// the same cut; a token lighter than 2^-32 of the heaviest one counts as no mass.  The pick then
// walks the kept tokens in index order: every wavefront owns a contiguous range of the row.
#include "common.h"

#define SMP_THREADS 1024

// Two stages so that a row of a large vocabulary is searched by many blocks: stage one leaves the
// best (value, index) of each slice of the row, stage two picks among the slices.  Ties go to the
// lower index in both.
#define ARGMAX_SLICES 32

__device__ __forceinline__ void argmax_merge(float& best, int& bi, float ov, int oi) {
  if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
}

__global__ void __launch_bounds__(256)
    argmax_slice_kernel(const float* __restrict__ logits, float* __restrict__ slice_val, int* __restrict__ slice_idx,
                        int V, int ld) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int row = blockIdx.y, slice = blockIdx.x;
  const int per = (V + ARGMAX_SLICES - 1) / ARGMAX_SLICES;
  const int beg = slice * per, end = min(V, beg + per);
  const float* x = logits + (size_t)row * ld;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = beg + threadIdx.x; i < end; i += blockDim.x) argmax_merge(best, bi, x[i], i);
#pragma unroll
  for (int o = BLM_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, BLM_WAVE);
    const int oi = __shfl_xor(bi, o, BLM_WAVE);
    argmax_merge(best, bi, ov, oi);
  }
  const int lane = threadIdx.x & (BLM_WAVE - 1), w = threadIdx.x / BLM_WAVE;
  if (lane == 0) { sv[w] = best; si[w] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; ++k) argmax_merge(best, bi, sv[k], si[k]);
    slice_val[row * ARGMAX_SLICES + slice] = best;
    slice_idx[row * ARGMAX_SLICES + slice] = bi;
  }
}

__global__ void argmax_final_kernel(const float* __restrict__ slice_val, const int* __restrict__ slice_idx,
                                    int* __restrict__ out) {
  const int row = blockIdx.x, lane = threadIdx.x;   // one wavefront per row
  float best = lane < ARGMAX_SLICES ? slice_val[row * ARGMAX_SLICES + lane] : -INFINITY;
  int bi = lane < ARGMAX_SLICES ? slice_idx[row * ARGMAX_SLICES + lane] : 0x7fffffff;
#pragma unroll
  for (int o = BLM_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, BLM_WAVE);
    const int oi = __shfl_xor(bi, o, BLM_WAVE);
    argmax_merge(best, bi, ov, oi);
  }
  if (lane == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}

// scratch: R * 32 floats and R * 32 ints
extern "C" int blm_argmax(const float* logits, int* out, int R, int V, int ld, float* slice_val, int* slice_idx,
                          hipStream_t stream) {
  BLM_REQUIRE(R > 0 && R <= 65535 && V > 0 && ld >= V, "argmax: bad sizes R=%d V=%d ld=%d", R, V, ld);
  hipLaunchKernelGGL(argmax_slice_kernel, dim3(ARGMAX_SLICES, R), dim3(256), 0, stream, logits, slice_val, slice_idx, V, ld);
  BLM_LAUNCH_CHECK("argmax_slice");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(BLM_WAVE), 0, stream, slice_val, slice_idx, out);
  BLM_LAUNCH_CHECK("argmax_final");
  return 0;
}

#define SMP_BINS 2048
#define SMP_MAX_CHUNKS 256   // chunks of 256 elements per wavefront: rows of up to 16 * 256 * 256 elements

// All elements of a row, coalesced: with VEC four consecutive floats per lane, and four such loads
// in flight per lane (a loop that waits for every load in turn spends a memory round trip on each).
// Places past the row's end read as -infinity, which BODY must take as "no token".
#define SMP_FOR_EACH(BODY)                                                                          \
  if (VEC) {                                                                                        \
    const float4* x4 = reinterpret_cast<const float4*>(x);                                          \
    const int n4 = V / 4;                                                                           \
    for (int i4 = tid; i4 < n4; i4 += 4 * SMP_THREADS) {                                            \
      float4 v4[4];                                                                                 \
      _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                               \
        const int j = i4 + u * SMP_THREADS;                                                         \
        v4[u] = j < n4 ? x4[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);           \
      }                                                                                             \
      _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                               \
        { const float xv = v4[u].x; BODY }                                                          \
        { const float xv = v4[u].y; BODY }                                                          \
        { const float xv = v4[u].z; BODY }                                                          \
        { const float xv = v4[u].w; BODY }                                                          \
      }                                                                                             \
    }                                                                                               \
    if (tid < (V & 3)) { const float xv = x[(V & ~3) + tid]; BODY }                                 \
  } else {                                                                                          \
    for (int i = tid; i < V; i += 4 * SMP_THREADS) {                                                \
      float v1[4];                                                                                  \
      _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                               \
        const int j = i + u * SMP_THREADS;                                                          \
        v1[u] = j < V ? x[j] : -INFINITY;                                                           \
      }                                                                                             \
      _Pragma("unroll") for (int u = 0; u < 4; ++u) { const float xv = v1[u]; BODY }                \
    }                                                                                               \
  }

__device__ __forceinline__ unsigned long long shfl_down_u64(unsigned long long v, int d) {
  const uint32_t lo = __shfl_down((uint32_t)v, d, BLM_WAVE), hi = __shfl_down((uint32_t)(v >> 32), d, BLM_WAVE);
  return ((unsigned long long)hi << 32) | lo;
}

// The lowest bin b of hist[0 .. SMP_BINS) with carry + (mass of the bins above b) < target, and
// that sum for it.  Every thread gets both.  Thread t looks after bins 2t and 2t + 1.
__device__ __forceinline__ void lowest_bin_below(const unsigned long long* hist, unsigned long long carry,
                                                 unsigned long long target, unsigned long long* wave_tot, int* found,
                                                 int& bin, unsigned long long& above) {
  const int tid = threadIdx.x, lane = tid & (BLM_WAVE - 1), w = tid / BLM_WAVE;
  const unsigned long long m0 = hist[2 * tid], m1 = hist[2 * tid + 1];
  unsigned long long suf = m0 + m1;   // becomes the mass of this thread's bins and of all higher threads' bins
#pragma unroll
  for (int d = 1; d < BLM_WAVE; d <<= 1) {
    const unsigned long long o = shfl_down_u64(suf, d);
    if (lane + d < BLM_WAVE) suf += o;
  }
  if (tid == 0) *found = 0x7fffffff;
  if (lane == 0) wave_tot[w] = suf;
  __syncthreads();
  for (int k = w + 1; k < SMP_THREADS / BLM_WAVE; ++k) suf += wave_tot[k];
  const unsigned long long above1 = carry + suf - m0 - m1;   // above bin 2t + 1
  const unsigned long long above0 = above1 + m1;             // above bin 2t
  if (above0 < target) atomicMin(found, 2 * tid);
  else if (above1 < target) atomicMin(found, 2 * tid + 1);
  __syncthreads();
  bin = *found;
  // the thread that owns the bin publishes its sum through wave_tot[0] (all reads of it are done)
  if (bin == 2 * tid) wave_tot[0] = above0;
  if (bin == 2 * tid + 1) wave_tot[0] = above1;
  __syncthreads();
  above = wave_tot[0];
  __syncthreads();
}

template <bool VEC>
__global__ void __launch_bounds__(SMP_THREADS)
    sample_kernel(const float* __restrict__ logits, const float* __restrict__ uniforms, int* __restrict__ out, int V,
                  int ld, float k2, float top_p) {
  __shared__ unsigned long long hist[SMP_BINS];
  __shared__ unsigned long long wave_tot[SMP_THREADS / BLM_WAVE];
  __shared__ float red[17];
  __shared__ float wsum[SMP_THREADS / BLM_WAVE];
  __shared__ int found, pick, last_kept;
  const float* x = logits + (size_t)blockIdx.x * ld;
  const int tid = threadIdx.x, lane = tid & (BLM_WAVE - 1), w = tid / BLM_WAVE;

  float mx = -INFINITY;
  SMP_FOR_EACH(mx = fmaxf(mx, xv);)
  mx = block_max(mx, red);

  // smallest kept weight, as a bit pattern; 0 keeps everything
  uint32_t tau = 0u;
  if (top_p < 1.0f) {
    unsigned long long carry = 0ull, target = 0ull;
    uint32_t prefix = 0u;
    // bits 29..19, then 18..8, then 7..0 (e <= 1, so bits 31 and 30 are clear)
    for (int level = 0; level < 3; ++level) {
      const int shift = level == 0 ? 19 : (level == 1 ? 8 : 0);
      const uint32_t mask = level == 2 ? 0xffu : 0x7ffu;
      hist[2 * tid] = 0ull;
      hist[2 * tid + 1] = 0ull;
      __syncthreads();
      SMP_FOR_EACH(
        const float e = __builtin_amdgcn_exp2f((xv - mx) * k2);
        const uint32_t key = __float_as_uint(e);
        // the digits above this level must be the ones already chosen (none at the first level)
        if (level == 0 || (key >> (shift + (level == 1 ? 11 : 8))) == prefix) {
          const unsigned long long q = (unsigned long long)(e * 4294967296.0f);
          if (q) atomicAdd(&hist[(key >> shift) & mask], q);
        }
      )
      __syncthreads();
      if (level == 0) {
        // the whole mass: what every bin holds
        unsigned long long z = hist[2 * tid] + hist[2 * tid + 1];
#pragma unroll
        for (int d = 1; d < BLM_WAVE; d <<= 1) {
          const unsigned long long o = shfl_down_u64(z, d);
          if (lane + d < BLM_WAVE) z += o;
        }
        if (lane == 0) wave_tot[w] = z;
        __syncthreads();
        unsigned long long total = 0ull;
        for (int k = 0; k < SMP_THREADS / BLM_WAVE; ++k) total += wave_tot[k];
        __syncthreads();
        target = (unsigned long long)((double)top_p * (double)total);
        if (target < 1ull) target = 1ull;
      }
      int bin;
      unsigned long long above;
      lowest_bin_below(hist, carry, target, wave_tot, &found, bin, above);
      carry = above;
      prefix = (prefix << (level == 2 ? 8 : 11)) | (uint32_t)bin;
    }
    tau = prefix;
  }

  // The pick, in index order.  Wavefront w owns elements [w * span, (w + 1) * span), span a
  // multiple of 256; it reads them 256 at a time, lane l the four from offset 4 l of each chunk,
  // and remembers the kept mass of every chunk (chunk c in lane c % 64, register c / 64).
  const int span = (((V + SMP_THREADS / BLM_WAVE - 1) / (SMP_THREADS / BLM_WAVE)) + 255) / 256 * 256;
  const int begin = w * span, end = min(V, begin + span);
  const int n_chunks = end > begin ? (end - begin + 255) / 256 : 0;   // at most SMP_MAX_CHUNKS (checked on the host)
  float chunk_mass[SMP_MAX_CHUNKS / BLM_WAVE];
#pragma unroll
  for (int g = 0; g < SMP_MAX_CHUNKS / BLM_WAVE; ++g) chunk_mass[g] = 0.f;
  int my_last = -1;
  // kept weights of the four elements of this lane in chunk ci (0 where there is no kept token)
#define SMP_LOAD_CHUNK(ci, xs)                                                                       \
  {                                                                                                 \
    const int i0_ = begin + (ci) * 256 + lane * 4;                                                  \
    if (VEC && i0_ + 3 < end) {                                                                     \
      const float4 v4_ = *reinterpret_cast<const float4*>(x + i0_);                                 \
      xs[0] = v4_.x; xs[1] = v4_.y; xs[2] = v4_.z; xs[3] = v4_.w;                                   \
    } else {                                                                                        \
      _Pragma("unroll") for (int k = 0; k < 4; ++k) xs[k] = i0_ + k < end ? x[i0_ + k] : -INFINITY; \
    }                                                                                               \
  }
#define SMP_KEPT(xv) ([&](float v_) { const float e_ = __builtin_amdgcn_exp2f((v_ - mx) * k2); \
                                      return (__float_as_uint(e_) >= tau && e_ > 0.f) ? e_ : 0.f; }(xv))
  for (int c0 = 0; c0 < n_chunks; c0 += 4) {
    float xs[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c0 + u < n_chunks) { SMP_LOAD_CHUNK(c0 + u, xs[u]) }
      else { xs[u][0] = xs[u][1] = xs[u][2] = xs[u][3] = -INFINITY; }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int ci = c0 + u;
      float s4 = 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float e = SMP_KEPT(xs[u][k]);
        s4 += e;
        if (e > 0.f) my_last = begin + ci * 256 + lane * 4 + k;
      }
      const float t = wave_sum(s4);
#pragma unroll
      for (int g = 0; g < SMP_MAX_CHUNKS / BLM_WAVE; ++g)
        if (ci < n_chunks && (ci >> 6) == g && (ci & 63) == lane) chunk_mass[g] = t;
    }
  }
  // mass of the wavefront's range: its chunks in order
  float mine = 0.f;
#pragma unroll
  for (int g = 0; g < SMP_MAX_CHUNKS / BLM_WAVE; ++g) {
    float incl = chunk_mass[g];
#pragma unroll
    for (int d = 1; d < BLM_WAVE; d <<= 1) {
      const float o = __shfl_up(incl, d, BLM_WAVE);
      if (lane >= d) incl += o;
    }
    mine += __shfl(incl, BLM_WAVE - 1, BLM_WAVE);
  }
  if (tid == 0) { pick = 0x7fffffff; last_kept = -1; }
  __syncthreads();
  if (lane == 0) wsum[w] = mine;
  if (my_last >= 0) atomicMax(&last_kept, my_last);
  __syncthreads();
  float total = 0.f, before = 0.f;
  for (int k = 0; k < SMP_THREADS / BLM_WAVE; ++k) {
    if (k == w) before = total;
    total += wsum[k];
  }
  const float want = uniforms[blockIdx.x] * total;
  if (mine > 0.f && want >= before && want < before + mine) {   // at most one wavefront
    // which chunk: the first whose running mass passes want
    float acc = before;
    int chunk = -1;
#pragma unroll
    for (int g = 0; g < SMP_MAX_CHUNKS / BLM_WAVE; ++g) {
      if (chunk >= 0) continue;
      float incl = chunk_mass[g];
#pragma unroll
      for (int d = 1; d < BLM_WAVE; d <<= 1) {
        const float o = __shfl_up(incl, d, BLM_WAVE);
        if (lane >= d) incl += o;
      }
      const float group_total = __shfl(incl, BLM_WAVE - 1, BLM_WAVE);
      const unsigned long long hits = __ballot(chunk_mass[g] > 0.f && want < acc + incl);
      if (hits) {
        const int first = __ffsll((long long)hits) - 1;
        chunk = g * 64 + first;
        acc += __shfl(incl - chunk_mass[g], first, BLM_WAVE);
      } else {
        acc += group_total;
      }
    }
    if (chunk >= 0) {
      float xs[4], es[4];
      SMP_LOAD_CHUNK(chunk, xs)
      float s4 = 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) { es[k] = SMP_KEPT(xs[k]); s4 += es[k]; }
      float incl = s4;   // inclusive prefix over the lanes, in lane order
#pragma unroll
      for (int d = 1; d < BLM_WAVE; d <<= 1) {
        const float o = __shfl_up(incl, d, BLM_WAVE);
        if (lane >= d) incl += o;
      }
      unsigned long long hits = __ballot(s4 > 0.f && want < acc + incl);
      const unsigned long long have = __ballot(s4 > 0.f);
      if (!hits && have) hits = 1ull << (63 - __clzll((long long)have));   // rounding: the chunk's last lane with a kept token
      if (hits) {
        const int first = __ffsll((long long)hits) - 1;
        if (lane == first) {
          const int i0 = begin + chunk * 256 + lane * 4;
          float run = acc + incl - s4;
          int chosen = -1, last = -1;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            if (es[k] > 0.f) {
              run += es[k];
              last = i0 + k;
              if (want < run && chosen < 0) chosen = i0 + k;
            }
          }
          atomicMin(&pick, chosen >= 0 ? chosen : last);   // rounding may leave want at the lane's upper edge
        }
      }
    } else {
      // rounding left want at the upper edge of the wavefront's range: its last kept token
      int m = my_last;
#pragma unroll
      for (int d = BLM_WAVE / 2; d > 0; d >>= 1) m = max(m, __shfl_xor(m, d, BLM_WAVE));
      if (lane == 0 && m >= 0) atomicMin(&pick, m);
    }
  }
#undef SMP_LOAD_CHUNK
#undef SMP_KEPT
  __syncthreads();
  if (tid == 0) out[blockIdx.x] = pick != 0x7fffffff ? pick : (last_kept >= 0 ? last_kept : 0);
}

extern "C" int blm_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld,
                          float temperature, float top_p, hipStream_t stream) {
  BLM_REQUIRE(R > 0 && V > 0 && ld >= V, "sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  BLM_REQUIRE(temperature > 0.f, "sample: temperature must be > 0 (got %g); use argmax for 0", (double)temperature);
  BLM_REQUIRE(top_p > 0.f, "sample: top_p must be > 0 (got %g)", (double)top_p);
  BLM_REQUIRE(V <= (SMP_THREADS / BLM_WAVE) * SMP_MAX_CHUNKS * 256, "sample: a vocabulary of %d is more than %d", V,
              (SMP_THREADS / BLM_WAVE) * SMP_MAX_CHUNKS * 256);
  const float k2 = 1.4426950408889634f / temperature;
  const bool vec = ld % 4 == 0 && ((uintptr_t)logits % 16) == 0;
  if (vec)
    hipLaunchKernelGGL(sample_kernel<true>, dim3(R), dim3(SMP_THREADS), 0, stream, logits, uniforms, out, V, ld, k2, top_p);
  else
    hipLaunchKernelGGL(sample_kernel<false>, dim3(R), dim3(SMP_THREADS), 0, stream, logits, uniforms, out, V, ld, k2, top_p);
  BLM_LAUNCH_CHECK("sample");
  return 0;
}
