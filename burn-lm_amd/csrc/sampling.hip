// Token choice from float logits.
//   argmax : first index of the maximum (lowest index wins ties); a row is searched by 32 blocks.
//   sample : softmax(logits / temperature) in float, nucleus (top-p) cut, inverse-CDF pick at a
//            uniform number u given by the caller, walking the kept tokens in index order; a row
//            is worked on by 16 blocks, each pass over it a kernel of its own.
// Nucleus rule: a token is kept while the probability mass of the tokens strictly more likely
// than it is below p; so the token that crosses p is kept, and tokens tied with it are too.
//
// The weight of a token is e = 2^((x - max) * log2(e) / temperature), in (0, 1].  The smallest
// kept weight is found by a radix selection over the bit pattern of e (positive floats order like
// their bits): three passes over the row with histograms of 11, 11 and 8 bits, each bin holding
// the mass of its tokens.  Mass is summed as 64-bit integers (e * 2^32, truncated), so the sums do
// not depend on the order in which the atomics land and the same logits always give the same cut;
// a token lighter than 2^-32 of the heaviest one counts as no mass.  The pick then walks the kept
// tokens in index order: every block owns a contiguous slice of the row, cut into chunks of 1024.
//
// One compute unit reads a row of 128K logits in about 10 us, and the five passes (maximum, three
// histograms, pick) each depend on the one before, so a row is cut into up to 16 slices for as
// many blocks and every pass is one kernel: the blocks of a row leave their part (slice maximum,
// histogram bins added to the row's with device-wide atomics, chunk masses) in device-coherent
// memory, count themselves in, and the block that arrives last finishes the pass for the row (the
// row's maximum, the bin of this level, the pick).  No block ever waits for another.
#include <mutex>

#include "common.h"
#include "no_alloc.h"


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

// ---- the same without workspace arguments: see no_alloc.h ------------------------------------
// The array's name is only a stand-in in host code: its address on each device comes from
// hipGetSymbolAddress, asked once per device with that device current, and is what the kernels get.
#define ARGMAX_STATIC_DEVICES 64
static __device__ __align__(256) unsigned char argmax_static_scratch[BLM_ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * 8];
static void* g_argmax_static_ptr[ARGMAX_STATIC_DEVICES];
static std::mutex g_argmax_static_mutex;

static int argmax_static_address(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  BLM_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  BLM_REQUIRE(dev >= 0 && dev < ARGMAX_STATIC_DEVICES, "argmax_static: device %d is beyond the %d this library keeps an address for",
              dev, ARGMAX_STATIC_DEVICES);
  std::lock_guard<std::mutex> hold(g_argmax_static_mutex);
  if (g_argmax_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_static_scratch));
    BLM_REQUIRE(e == hipSuccess && p != nullptr, "argmax_static: hipGetSymbolAddress failed on device %d: %s", dev,
                hipGetErrorString(e));
    g_argmax_static_ptr[dev] = p;
  }
  *ptr = g_argmax_static_ptr[dev];
  return 0;
}

extern "C" int blm_static_scratch_init() {
  void* p = nullptr;
  return argmax_static_address(&p);
}

extern "C" int blm_argmax_static(const float* logits, int* out, int R, int V, int ld, hipStream_t stream) {
  BLM_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: logits and out must be given");
  BLM_REQUIRE(R > 0 && V > 0 && ld >= V, "argmax_static: bad sizes R=%d V=%d ld=%d", R, V, ld);
  BLM_REQUIRE(R <= BLM_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows, the library's own scratch array holds %d (use blm_argmax with workspaces)",
              R, BLM_ARGMAX_STATIC_MAX_ROWS);
  void* base = nullptr;
  if (argmax_static_address(&base)) return 1;
  float* slice_val = reinterpret_cast<float*>(base);
  int* slice_idx = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(base) + (size_t)BLM_ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * 4);
  hipLaunchKernelGGL(argmax_slice_kernel, dim3(ARGMAX_SLICES, R), dim3(256), 0, stream, logits, slice_val, slice_idx, V, ld);
  BLM_LAUNCH_CHECK("argmax_slice");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(BLM_WAVE), 0, stream, slice_val, slice_idx, out);
  BLM_LAUNCH_CHECK("argmax_final");
  return 0;
}

#define SMP_BINS 2048
#define SMP_SLICES 32      // most blocks per row (fewer when there are many rows)
#define SMP_THREADS 256
#define SMP_CHUNK (SMP_THREADS * 4)   // elements per chunk: four neighbours per thread
#define SMP_WAVES (SMP_THREADS / BLM_WAVE)
#define SMP_ROUND 8         // chunks of a slice whose masses are summed behind one barrier

// per row: the maximum, then for the selection the digits found so far, the mass above them and the mass to reach
struct SampleRow {
  float mx;
  uint32_t prefix;
  unsigned long long carry, target;
};

__device__ __forceinline__ void smp_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float smp_load(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned long long smp_load(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Whether this block is the last of its row to get here.  What the block wrote before (coherent
// stores, device-wide atomics) has been acknowledged when it counts itself in; the last one sets
// the counter back to zero.  All threads get the answer.
__device__ __forceinline__ bool smp_arrive_last(int* counter, int* flag, int n_slices) {
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  __syncthreads();
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = before == n_slices - 1;
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last;
  }
  __syncthreads();
  return *flag != 0;
}

// The four elements of thread `tid` in the chunk that starts at element i0 of row x (V elements);
// places past the row's end read as -infinity ("no token").
template <bool VEC>
__device__ __forceinline__ void smp_load4(const float* x, int i0, int V, float xs[4]) {
  if (VEC && i0 + 3 < V) {
    const float4 v = *reinterpret_cast<const float4*>(x + i0);
    xs[0] = v.x; xs[1] = v.y; xs[2] = v.z; xs[3] = v.w;
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) xs[k] = i0 + k < V ? x[i0 + k] : -INFINITY;
  }
}

__device__ __forceinline__ unsigned long long shfl_down_u64(unsigned long long v, int d) {
  const uint32_t lo = __shfl_down((uint32_t)v, d, BLM_WAVE), hi = __shfl_down((uint32_t)(v >> 32), d, BLM_WAVE);
  return ((unsigned long long)hi << 32) | lo;
}

// pass 1: the row's maximum; the last block also clears the row's histograms for the passes to come
template <bool VEC>
__global__ void __launch_bounds__(SMP_THREADS)
    sample_max_kernel(const float* __restrict__ logits, int V, int ld, int slice_len, float* part_max,
                      SampleRow* rows, unsigned long long* hist, int n_rows, int* counters, int with_hist) {
  __shared__ float red[17];
  __shared__ int flag;
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int begin = slice * slice_len, end = min(V, begin + slice_len);
  float mx = -INFINITY;
  for (int c0 = begin; c0 < end; c0 += 4 * SMP_CHUNK) {
    float xs[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) smp_load4<VEC>(x, c0 + u * SMP_CHUNK + tid * 4, end, xs[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int k = 0; k < 4; ++k) mx = fmaxf(mx, xs[u][k]);
  }
  mx = block_max(mx, red);
  if (tid == 0) smp_store(part_max + row * SMP_SLICES + slice, mx);
  if (!smp_arrive_last(counters + row, &flag, gridDim.x)) return;
  float m = tid < (int)gridDim.x ? smp_load(part_max + row * SMP_SLICES + tid) : -INFINITY;
  m = block_max(m, red);
  if (tid == 0) {
    rows[row].mx = m;
    rows[row].prefix = 0u;
    rows[row].carry = 0ull;
    rows[row].target = 0ull;
  }
  if (with_hist)
    for (int level = 0; level < 3; ++level)
      for (int b = tid; b < SMP_BINS; b += SMP_THREADS) hist[((size_t)level * n_rows + row) * SMP_BINS + b] = 0ull;
}

// passes 2 to 4: level 0 takes bits 29..19 of the weights' bit patterns, level 1 bits 18..8, level 2
// bits 7..0 (e <= 1, so bits 31 and 30 are clear); the last block finds the lowest bin above which
// less than the target mass lies
template <bool VEC, int LEVEL>
__global__ void __launch_bounds__(SMP_THREADS)
    sample_level_kernel(const float* __restrict__ logits, int V, int ld, int slice_len, float k2, float top_p,
                        SampleRow* rows, unsigned long long* hist, int n_rows, int* counters) {
  __shared__ unsigned long long bins[SMP_BINS];
  __shared__ unsigned long long wave_tot[SMP_WAVES];
  __shared__ unsigned long long chosen_above;
  __shared__ int flag, found;
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x, lane = tid & (BLM_WAVE - 1), w = tid / BLM_WAVE;
  const float* x = logits + (size_t)row * ld;
  const int begin = slice * slice_len, end = min(V, begin + slice_len);
  const float mx = rows[row].mx;
  const uint32_t prefix = rows[row].prefix;
  constexpr int shift = LEVEL == 0 ? 19 : (LEVEL == 1 ? 8 : 0);
  constexpr uint32_t mask = LEVEL == 2 ? 0xffu : 0x7ffu;
  constexpr int above_bits = LEVEL == 0 ? 0 : (LEVEL == 1 ? 19 : 8);   // the digits above this level start here
  for (int b = tid; b < SMP_BINS; b += SMP_THREADS) bins[b] = 0ull;
  __syncthreads();
  for (int c0 = begin; c0 < end; c0 += 4 * SMP_CHUNK) {
    float xs[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) smp_load4<VEC>(x, c0 + u * SMP_CHUNK + tid * 4, end, xs[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float e = __builtin_amdgcn_exp2f((xs[u][k] - mx) * k2);
        const uint32_t key = __float_as_uint(e);
        // the digits above this level must be the ones already chosen (none at the first level)
        if (LEVEL == 0 || (key >> above_bits) == prefix) {
          const unsigned long long q = (unsigned long long)(e * 4294967296.0f);
          if (q) atomicAdd(&bins[(key >> shift) & mask], q);
        }
      }
  }
  __syncthreads();
  unsigned long long* row_hist = hist + ((size_t)LEVEL * n_rows + row) * SMP_BINS;
  for (int b = tid; b < SMP_BINS; b += SMP_THREADS)
    if (bins[b]) __hip_atomic_fetch_add(row_hist + b, bins[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (!smp_arrive_last(counters + row, &flag, gridDim.x)) return;

  // thread t looks after bins 8 t .. 8 t + 7
  constexpr int PER = SMP_BINS / SMP_THREADS;
  unsigned long long m[PER], tot = 0ull;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    m[j] = smp_load(row_hist + tid * PER + j);
    tot += m[j];
  }
  unsigned long long suf = tot;   // becomes the mass of this thread's bins and of all higher threads' bins
#pragma unroll
  for (int d = 1; d < BLM_WAVE; d <<= 1) {
    const unsigned long long o = shfl_down_u64(suf, d);
    if (lane + d < BLM_WAVE) suf += o;
  }
  if (tid == 0) found = 0x7fffffff;
  if (lane == 0) wave_tot[w] = suf;
  __syncthreads();
  for (int k = w + 1; k < SMP_WAVES; ++k) suf += wave_tot[k];
  unsigned long long carry = rows[row].carry, target = rows[row].target;
  if (LEVEL == 0) {
    // the whole mass: what every bin holds
    unsigned long long total = wave_tot[0];
    for (int k = 1; k < SMP_WAVES; ++k) total += wave_tot[k];
    target = (unsigned long long)((double)top_p * (double)total);
    if (target < 1ull) target = 1ull;
  }
  unsigned long long above = carry + suf - tot;   // above this thread's highest bin
  int mine = -1;
  unsigned long long mine_above = 0ull;
#pragma unroll
  for (int j = PER - 1; j >= 0; --j) {
    if (above < target) { mine = tid * PER + j; mine_above = above; }
    above += m[j];
  }
  if (mine >= 0) atomicMin(&found, mine);
  __syncthreads();
  if (found == mine) chosen_above = mine_above;
  __syncthreads();
  if (tid == 0) {
    rows[row].prefix = (prefix << (LEVEL == 2 ? 8 : 11)) | (uint32_t)found;
    rows[row].carry = chosen_above;
    rows[row].target = target;
  }
}

// inclusive prefix over the block's threads in thread order, and the block's total
__device__ __forceinline__ float smp_block_scan(float v, float* wave_sums, float& total) {
  const int lane = threadIdx.x & (BLM_WAVE - 1), w = threadIdx.x / BLM_WAVE;
  float incl = v;
#pragma unroll
  for (int d = 1; d < BLM_WAVE; d <<= 1) {
    const float o = __shfl_up(incl, d, BLM_WAVE);
    if (lane >= d) incl += o;
  }
  __syncthreads();   // wave_sums may still be read from an earlier call
  if (lane == BLM_WAVE - 1) wave_sums[w] = incl;
  __syncthreads();
  float before = 0.f;
  total = 0.f;
  for (int k = 0; k < SMP_WAVES; ++k) {
    if (k == w) before = total;
    total += wave_sums[k];
  }
  return before + incl;
}

// last pass: the kept mass of every chunk; the last block finds the chunk that holds the pick and
// the token in it.  use_tau 0: no cut, every token with a weight is kept.
template <bool VEC>
__global__ void __launch_bounds__(SMP_THREADS)
    sample_pick_kernel(const float* __restrict__ logits, const float* __restrict__ uniforms, int* __restrict__ out, int V,
                       int ld, int slice_len, float k2, int use_tau, const SampleRow* rows, float* chunk_mass,
                       int* counters) {
  __shared__ float red[17];
  __shared__ float wave_sums[SMP_WAVES];
  __shared__ float round_sums[SMP_ROUND][SMP_WAVES];
  __shared__ int flag, hit, last_with_mass;
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int begin = slice * slice_len, end = min(V, begin + slice_len);
  const int chunks = slice_len / SMP_CHUNK;            // per slice
  const float mx = rows[row].mx;
  const uint32_t tau = use_tau ? rows[row].prefix : 0u;   // smallest kept weight, as a bit pattern
  auto kept = [&](float v) {
    const float e = __builtin_amdgcn_exp2f((v - mx) * k2);
    return (__float_as_uint(e) >= tau && e > 0.f) ? e : 0.f;
  };
  float* row_mass = chunk_mass + (size_t)row * gridDim.x * chunks;
  const float u = uniforms[row];   // asked for early: it may lie in host memory
  // the chunks of the slice, SMP_ROUND at a time: all loads first, one barrier per round
  for (int c0 = 0; c0 < chunks; c0 += SMP_ROUND) {
    float xs[SMP_ROUND][4];
#pragma unroll
    for (int r = 0; r < SMP_ROUND; ++r) smp_load4<VEC>(x, begin + (c0 + r) * SMP_CHUNK + tid * 4, c0 + r < chunks ? end : 0, xs[r]);
    __syncthreads();   // round_sums may still be read from the round before
#pragma unroll
    for (int r = 0; r < SMP_ROUND; ++r) {
      const float s4 = ((kept(xs[r][0]) + kept(xs[r][1])) + kept(xs[r][2])) + kept(xs[r][3]);
      const float ws = wave_sum(s4);
      if ((tid & (BLM_WAVE - 1)) == 0) round_sums[r][tid / BLM_WAVE] = ws;
    }
    __syncthreads();
    if (tid < SMP_ROUND && c0 + tid < chunks) {
      float t = 0.f;
      for (int k = 0; k < SMP_WAVES; ++k) t += round_sums[tid][k];
      smp_store(row_mass + slice * chunks + c0 + tid, t);
    }
  }
  if (!smp_arrive_last(counters + row, &flag, gridDim.x)) return;

  // chunks in index order: slice by slice; first their total, then the chunk in which u * total falls
  const int n = gridDim.x * chunks;
  if (tid == 0) { hit = 0x7fffffff; last_with_mass = -1; }
  int first_idx = 0x7fffffff, last_idx = -1;   // this thread's lowest chunk that passes u * total, its highest with mass
  float first_front = 0.f, last_front = 0.f;   // and the mass in front of each
  float want;
  if (n <= SMP_THREADS) {
    const float mass = tid < n ? smp_load(row_mass + tid) : 0.f;
    float total;
    const float incl = smp_block_scan(mass, wave_sums, total);
    want = u * total;
    if (mass > 0.f) {
      if (want < incl) { first_idx = tid; first_front = incl - mass; }
      last_idx = tid;
      last_front = incl - mass;
    }
  } else {
    float total = 0.f;
    for (int base = 0; base < n; base += SMP_THREADS) {
      float t;
      smp_block_scan(base + tid < n ? smp_load(row_mass + base + tid) : 0.f, wave_sums, t);
      total += t;
    }
    want = u * total;
    float run = 0.f;   // mass in front of this round of chunks
    for (int base = 0; base < n; base += SMP_THREADS) {
      const float mass = base + tid < n ? smp_load(row_mass + base + tid) : 0.f;
      float t;
      const float incl = run + smp_block_scan(mass, wave_sums, t);
      if (mass > 0.f) {
        if (want < incl && first_idx == 0x7fffffff) { first_idx = base + tid; first_front = incl - mass; }
        last_idx = base + tid;
        last_front = incl - mass;
      }
      run += t;
    }
  }
  if (first_idx != 0x7fffffff) atomicMin(&hit, first_idx);
  if (last_idx >= 0) atomicMax(&last_with_mass, last_idx);
  __syncthreads();
  const int chunk = hit != 0x7fffffff ? hit : last_with_mass;   // rounding may leave u * total at the upper edge
  if (chunk < 0) {   // no token has a weight: cannot happen (the maximum has weight 1); answer something valid
    if (tid == 0) out[row] = 0;
    return;
  }
  if (first_idx == chunk) red[0] = first_front;
  else if (last_idx == chunk) red[0] = last_front;
  __syncthreads();
  const float front = red[0];   // mass in front of the chosen chunk
  __syncthreads();
  const int cs = chunk / chunks, cc = chunk % chunks;
  const int i0 = cs * slice_len + cc * SMP_CHUNK + tid * 4;
  float xs[4], es[4];
  smp_load4<VEC>(x, i0, min(V, cs * slice_len + slice_len), xs);
#pragma unroll
  for (int k = 0; k < 4; ++k) es[k] = kept(xs[k]);
  const float s4 = ((es[0] + es[1]) + es[2]) + es[3];
  float t;
  const float incl = front + smp_block_scan(s4, wave_sums, t);
  if (tid == 0) { hit = 0x7fffffff; last_with_mass = -1; }
  __syncthreads();
  if (s4 > 0.f) {
    if (want < incl) atomicMin(&hit, tid);
    atomicMax(&last_with_mass, tid);
  }
  __syncthreads();
  const int owner = hit != 0x7fffffff ? hit : last_with_mass;   // at least one thread has a kept token
  if (tid == owner) {
    float acc = incl - s4;
    int chosen = -1, last = -1;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (es[k] > 0.f) {
        acc += es[k];
        last = i0 + k;
        if (want < acc && chosen < 0) chosen = i0 + k;
      }
    }
    out[row] = chosen >= 0 ? chosen : last;   // rounding may leave want at the thread's upper edge
  }
}

// Blocks per row.  Measured with the nucleus cut at a vocabulary of 128K (one block of 1024 threads per
// row took 77 us whatever the number of rows): 32 blocks 42 us for one row, 16 blocks 45 us; 8 rows
// 51 us with 16 and 55 us with 32; 64 rows 91 us with 16 and 101 us with 4.  Every pass costs
// about 9 us of launch, coherent round trips and the last block's tail, whatever the slice's length.
static int sample_slices(int R) { return R <= 2 ? 32 : 16; }
static int sample_slice_len(int R, int V) {
  const int n = sample_slices(R);
  return ((V + n - 1) / n + SMP_CHUNK - 1) / SMP_CHUNK * SMP_CHUNK;
}

// Bytes of scratch that blm_sample needs for R rows of V logits (see there for the layout).
extern "C" long long blm_sample_scratch_bytes(int R, int V) {
  const long long chunks = (long long)sample_slices(R) * (sample_slice_len(R, V) / SMP_CHUNK);
  return (long long)R * (3 * SMP_BINS * 8 + sizeof(SampleRow) + SMP_SLICES * 4 + chunks * 4);
}

// scratch: blm_sample_scratch_bytes(R, V) bytes, 8-byte aligned: three histograms per row, the rows'
// states, the slices' maxima, the chunks' masses.  counters: R zeroed ints, left zeroed.
extern "C" int blm_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld,
                          float temperature, float top_p, void* scratch, int* counters, hipStream_t stream) {
  BLM_REQUIRE(R > 0 && R <= 65535 && V > 0 && ld >= V, "sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  BLM_REQUIRE(temperature > 0.f, "sample: temperature must be > 0 (got %g); use argmax for 0", (double)temperature);
  BLM_REQUIRE(top_p > 0.f, "sample: top_p must be > 0 (got %g)", (double)top_p);
  BLM_REQUIRE(scratch != nullptr && ((uintptr_t)scratch % 8) == 0 && counters != nullptr, "sample: scratch and counters needed");
  const int slice_len = sample_slice_len(R, V);
  unsigned long long* hist = reinterpret_cast<unsigned long long*>(scratch);
  SampleRow* rows = reinterpret_cast<SampleRow*>(hist + (size_t)3 * R * SMP_BINS);
  float* part_max = reinterpret_cast<float*>(rows + R);
  float* chunk_mass = part_max + (size_t)R * SMP_SLICES;
  const float k2 = 1.4426950408889634f / temperature;
  const bool vec = ld % 4 == 0 && ((uintptr_t)logits % 16) == 0;
  const int cut = top_p < 1.0f ? 1 : 0;
  dim3 grid(sample_slices(R), R), block(SMP_THREADS);
#define SMP_LAUNCH(VEC)                                                                                              \
  do {                                                                                                               \
    hipLaunchKernelGGL(sample_max_kernel<VEC>, grid, block, 0, stream, logits, V, ld, slice_len, part_max, rows,     \
                       hist, R, counters, cut);                                                                      \
    if (cut) {                                                                                                       \
      hipLaunchKernelGGL((sample_level_kernel<VEC, 0>), grid, block, 0, stream, logits, V, ld, slice_len, k2, top_p, \
                         rows, hist, R, counters);                                                                   \
      hipLaunchKernelGGL((sample_level_kernel<VEC, 1>), grid, block, 0, stream, logits, V, ld, slice_len, k2, top_p, \
                         rows, hist, R, counters);                                                                   \
      hipLaunchKernelGGL((sample_level_kernel<VEC, 2>), grid, block, 0, stream, logits, V, ld, slice_len, k2, top_p, \
                         rows, hist, R, counters);                                                                   \
    }                                                                                                                \
    hipLaunchKernelGGL(sample_pick_kernel<VEC>, grid, block, 0, stream, logits, uniforms, out, V, ld, slice_len, k2, \
                       cut, rows, chunk_mass, counters);                                                             \
  } while (0)
  if (vec) SMP_LAUNCH(true);
  else SMP_LAUNCH(false);
#undef SMP_LAUNCH
  BLM_LAUNCH_CHECK("sample");
  return 0;
}
