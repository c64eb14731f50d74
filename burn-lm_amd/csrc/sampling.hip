// Token choice from float logits, one block per row.
//   argmax : first index of the maximum (lowest index wins ties).
//   sample : softmax(logits / temperature) in float, nucleus (top-p) cut, inverse-CDF pick at a
//            uniform number u given by the caller, walking the kept tokens in index order.
// Nucleus rule: a token is kept while the probability mass of the tokens strictly more likely
// than it is below p; so the token that crosses p is kept, and tokens tied with it are too.
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

__global__ void __launch_bounds__(SMP_THREADS)
    sample_kernel(const float* __restrict__ logits, const float* __restrict__ uniforms,
                  int* __restrict__ out, int V, int ld, float inv_temperature, float top_p) {
  __shared__ float red[17];
  __shared__ float seg[SMP_THREADS];
  __shared__ int pick[2];
  const float* x = logits + (size_t)blockIdx.x * ld;
  const int tid = threadIdx.x;

  float mx = -INFINITY;
  for (int i = tid; i < V; i += blockDim.x) mx = fmaxf(mx, x[i]);
  mx = block_max(mx, red);

  float z = 0.f;
  for (int i = tid; i < V; i += blockDim.x) z += expf((x[i] - mx) * inv_temperature);
  z = block_sum(z, red);

  // smallest kept weight tau: the smallest float t with mass{e > t} < top_p * z
  float tau = 0.f;
  if (top_p < 1.0f) {
    const float target = top_p * z;
    uint32_t lo = 0u, hi = 0x3f800000u;  // e <= 1, so mass{e > 1} = 0 < target
    // f(0) >= target unless everything underflowed; then tau collapses to the smallest float
    while (hi - lo > 1u) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      const float t = __uint_as_float(mid);
      float mass = 0.f;
      for (int i = tid; i < V; i += blockDim.x) {
        const float e = expf((x[i] - mx) * inv_temperature);
        mass += e > t ? e : 0.f;
      }
      mass = block_sum(mass, red);
      if (mass < target) hi = mid; else lo = mid;
    }
    tau = __uint_as_float(hi);
  }

  // contiguous segment per thread, so the walk is in index order
  const int per = (V + blockDim.x - 1) / blockDim.x;
  const int beg = tid * per, end = min(V, beg + per);
  float mine = 0.f;
  int last_kept = -1;
  for (int i = beg; i < end; ++i) {
    const float e = expf((x[i] - mx) * inv_temperature);
    if (e >= tau) { mine += e; last_kept = i; }
  }
  seg[tid] = mine;
  if (tid == 0) { pick[0] = 0x7fffffff; pick[1] = -1; }
  __syncthreads();
  if (tid == 0) {  // exclusive prefix over 1024 segment sums, in order
    float run = 0.f;
    for (int k = 0; k < (int)blockDim.x; ++k) { const float s = seg[k]; seg[k] = run; run += s; }
    red[0] = run;
  }
  __syncthreads();
  const float total = red[0];
  const float want = uniforms[blockIdx.x] * total;
  if (last_kept >= 0) atomicMax(&pick[1], last_kept);
  const float before = seg[tid];
  if (mine > 0.f && want >= before && want < before + mine) {
    float run = before;
    int chosen = last_kept;
    for (int i = beg; i < end; ++i) {
      const float e = expf((x[i] - mx) * inv_temperature);
      if (e >= tau) {
        run += e;
        if (want < run) { chosen = i; break; }
      }
    }
    atomicMin(&pick[0], chosen);
  }
  __syncthreads();
  if (tid == 0) out[blockIdx.x] = pick[0] != 0x7fffffff ? pick[0] : (pick[1] >= 0 ? pick[1] : 0);
}

extern "C" int blm_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld,
                          float temperature, float top_p, hipStream_t stream) {
  BLM_REQUIRE(R > 0 && V > 0 && ld >= V, "sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  BLM_REQUIRE(temperature > 0.f, "sample: temperature must be > 0 (got %g); use argmax for 0", (double)temperature);
  BLM_REQUIRE(top_p > 0.f, "sample: top_p must be > 0 (got %g)", (double)top_p);
  hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SMP_THREADS), 0, stream, logits, uniforms, out, V, ld,
                     1.0f / temperature, top_p);
  BLM_LAUNCH_CHECK("sample");
  return 0;
}
