// Skinny matrix product for decode on the matrix cores: C[M<=64, N] = A[M, K] * W[N, K]^T, bf16
// operands, float accumulation, bf16 or float output.  Up to 16 rows run gemv_mfma_kernel, 17 to 64
// rows gemv_mfma_rows_kernel (two to four row tiles against every weight fragment).
//
// The weight matrix is streamed exactly once, from a copy packed in the order the MFMA wants it:
// for the 16x16x32 instruction the weights are the B operand, lane l of a wavefront holding
// W[n0 + l%16][k0 + (l/16)*8 .. +8].  Read from the checkpoint layout that is 16 bytes from each
// of 16 different rows per quarter-wavefront, which the memory pipeline serves at a fraction of
// its rate; the packed copy (made once when the weights are bound, see pack_weight in ops.py)
// stores the 64 lanes' 16-byte pieces of every (16-column tile, k-step) next to each other, so
// each wavefront load is one contiguous kilobyte:
//     packed[((tile * k_steps + step) * 64 + lane) * 8 + e] = W[tile*16 + lane%16][step*32 + (lane/16)*8 + e]
// with N padded to a multiple of 16 and K to a multiple of 32 by zeros.
//
// A block owns tiles of 16 output columns; its wavefronts split K between them.  The activations
// are the A operand (row m = l%16, rows >= M are zero) and stay in registers for the block's whole
// life, so a block that walks several column tiles reads them once.  The partial tiles of the
// wavefronts are summed through shared memory in a fixed order.  The SwiGLU gating of a
// feed-forward can be fused into the product that computes gate and up (c_mode 1).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ uint4 ld16(const bf16* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint4 ld16_stream(const bf16* p) { return load16_stream(p); }   // the weights: read once

// KSTEPS: k-steps of 32 per wavefront.  MAXT: most threads of a block (sets the register budget).
// KEEP_A: the activations' fragments stay in registers across the block's column tiles.
template <int KSTEPS, int MAXT, bool KEEP_A, typename TC>
__global__ void __launch_bounds__(MAXT)
    gemv_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, TC* __restrict__ C, int M, int N,
                     int K, int lda, int ldc, int n_tiles, int k_steps, int c_mode, int steps_per_group) {
  extern __shared__ float red[];  // [waves][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  // blockIdx.y is the K-group: it covers k-steps [group_begin, group_end) and writes plane blockIdx.y of C
  const int group_begin = blockIdx.y * steps_per_group;
  const int group_end = min(k_steps, group_begin + steps_per_group);
  const int step0 = group_begin + wave * KSTEPS;   // first k-step of this wavefront
  const int kbase = step0 * 32 + kg * 8;
  C += (size_t)blockIdx.y * M * ldc;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  const int arow = row < M ? row : M - 1;   // rows >= M read a real row and are zeroed, so every load is in bounds
  const bf16* ap = A + (size_t)arow * lda;

  // Fragments of A beyond K, beyond M or beyond the block's K-group are zero, so whatever the
  // weights hold there adds nothing; the weight loads are unconditional, with the k-step clamped
  // into the matrix.
  uint4 a[KSTEPS];
  // Every load of the activations, and of the first tile's weights behind them, is asked for before the
  // first fragment is looked at: zeroing the fragments one by one as they are loaded waits for each in
  // turn, and the weights, which come the long way, would start a trip to memory later.  (The weights
  // first is worse: loads come back in order, so the first product would wait for all of them.)
#define GV_LOAD_ACTIVATIONS()                                                         \
  _Pragma("unroll") for (int s = 0; s < KSTEPS; ++s) {                                \
    const int k = kbase + s * 32;                                                     \
    a[s] = ld16(ap + (k < K ? k : K - 8));                                            \
  }
#define GV_ZERO_ACTIVATIONS()                                                         \
  _Pragma("unroll") for (int s = 0; s < KSTEPS; ++s) {                                \
    const int k = kbase + s * 32;                                                     \
    const bool keep = row < M && k < K && step0 + s < group_end;                      \
    a[s] = make_uint4(keep ? a[s].x : 0u, keep ? a[s].y : 0u, keep ? a[s].z : 0u, keep ? a[s].w : 0u); \
  }
  if (KEEP_A) GV_LOAD_ACTIVATIONS()

  // a block takes a run of neighbouring column tiles, so that it streams one contiguous piece of the
  // packed weights (blocks that each read their own region reach a higher memory rate than blocks
  // that all advance through the matrix side by side)
  const int tiles_per_block = (n_tiles + gridDim.x - 1) / gridDim.x;
  const int tile_begin = blockIdx.x * tiles_per_block, tile_end = min(n_tiles, tile_begin + tiles_per_block);
  // 16 k-steps per wavefront: the weights come in two halves of eight fragments, and each half's
  // registers are asked for the next tile's weights as soon as the matrix instructions that read them
  // have been issued, so loads are on their way while the other half is multiplied and while the
  // block sums its tile.  (All blocks start together; without this they also wait together, and
  // the memory idles whenever they multiply and sum: gate/up with 16 rows 14.5 us instead of 15.9,
  // with 8 rows 13.7 instead of 14.3, the head 84-86 instead of 87.5.  No more registers than the
  // sixteen fragments of one tile.)
  constexpr bool PIPE = KSTEPS == 16 && KEEP_A;
  constexpr int HALF = KSTEPS / 2;
  uint4 wa[PIPE ? HALF : 1], wb[PIPE ? HALF : 1];
  int woff[PIPE ? KSTEPS : 1];
  if (PIPE) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) woff[s] = (step0 + s < k_steps ? step0 + s : k_steps - 1) * 512;
    const bf16* wt = Wp + ((size_t)min(tile_begin, n_tiles - 1) * k_steps * 64 + lane) * 8;
#pragma unroll
    for (int s = 0; s < HALF; ++s) wa[s] = ld16_stream(wt + woff[s]);
#pragma unroll
    for (int s = 0; s < HALF; ++s) wb[s] = ld16_stream(wt + woff[HALF + s]);
  }
  __builtin_amdgcn_sched_barrier(0);
  if (KEEP_A) GV_ZERO_ACTIVATIONS()
#undef GV_LOAD_ACTIVATIONS
#undef GV_ZERO_ACTIVATIONS
  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const bf16* wt = Wp + ((size_t)tile * k_steps * 64 + lane) * 8;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int CH = KSTEPS < 16 ? KSTEPS : 16;   // weight loads in flight per wavefront
    if (PIPE) {
      const bool more = tile + 1 < tile_end;
      const bf16* wnext = Wp + ((size_t)(tile + 1) * k_steps * 64 + lane) * 8;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < HALF; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                      __builtin_bit_cast(bf16x8_t, wa[s]), acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (more) {
#pragma unroll
        for (int s = 0; s < HALF; ++s) wa[s] = ld16_stream(wnext + woff[s]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < HALF; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[HALF + s]),
                                                      __builtin_bit_cast(bf16x8_t, wb[s]), acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (more) {
#pragma unroll
        for (int s = 0; s < HALF; ++s) wb[s] = ld16_stream(wnext + woff[HALF + s]);
      }
      __builtin_amdgcn_sched_barrier(0);
    } else
#pragma unroll
    for (int c = 0; c < KSTEPS; c += CH) {
      uint4 w[CH];
#pragma unroll
      for (int s = 0; s < CH; ++s) {
        const int st = step0 + c + s;
        w[s] = ld16_stream(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);
      }
      if (!KEEP_A) {
#pragma unroll
        for (int s = 0; s < CH; ++s) {
          const int k = kbase + (c + s) * 32;
          const uint4 v = ld16(ap + (k < K ? k : K - 8));
          a[c + s] = (row < M && k < K && step0 + c + s < group_end) ? v : zero;
        }
      }
      // All loads of the chunk are issued before its first MFMA: left alone, the scheduler reuses
      // one register for every load and waits for each in turn, which makes the kernel latency-bound.
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < CH; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[c + s]),
                                                      __builtin_bit_cast(bf16x8_t, w[s]), acc, 0, 0, 0);
    }
    // acc[r] is the product for row m = kg*4 + r and column n = tile*16 + row
    if (n_waves == 1 && c_mode == 0) {
      const int n = tile * 16 + row;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = kg * 4 + r;
        if (m < M && n < N) C[(size_t)m * ldc + n] = from_float<TC>(acc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
      __syncthreads();
      for (int idx = threadIdx.x; idx < 256; idx += blockDim.x) {  // a block may have fewer than 256 threads
        const int r = idx >> 6, l2 = idx & 63, col = l2 & 15;
        const int m = (l2 >> 4) * 4 + r;
        if (c_mode == 0) {
          float s = 0.f;
          for (int w2 = 0; w2 < n_waves; ++w2) s += red[w2 * 256 + idx];
          const int nn = tile * 16 + col;
          if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(s);
        } else if (col < 8) {
          // gated pairs: columns 0..7 of the tile are gates, 8..15 the matching ups; one output per pair
          float g = 0.f, u = 0.f;
          for (int w2 = 0; w2 < n_waves; ++w2) {
            g += red[w2 * 256 + idx];
            u += red[w2 * 256 + idx + 8];
          }
          const int nn = tile * 8 + col;
          if (m < M && nn < N / 2) C[(size_t)m * ldc + nn] = from_float<TC>(g / (1.0f + expf(-g)) * u);
        }
      }
      __syncthreads();
    }
  }
}

// 17..64 rows: MT row tiles of 16.  A wavefront keeps the activations of all MT tiles for its
// KSTEPS k-steps in registers (MT * KSTEPS fragments, at most 32) and runs MT MFMAs per weight
// fragment, so the weights still stream once.  Blocks have up to 8 wavefronts, so one K-group
// spans at most 8 * KSTEPS * 32: 2048 with 8 k-steps, and 4096 with 16, which only two row tiles
// leave room for.  PREFETCH: the weights of the block's next column tile are requested before the
// current tile is multiplied and reduced (and the first tile's before the activations), so the
// memory pipeline never idles while the block synchronises; with 16 k-steps the registers do not
// allow it.
template <int MT, int KSTEPS, bool PREFETCH, typename TC>
__global__ void __launch_bounds__(512)
    gemv_mfma_rows_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, TC* __restrict__ C, int M, int N,
                          int K, int lda, int ldc, int n_tiles, int k_steps, int c_mode, int steps_per_group) {
  extern __shared__ float red[];  // [waves][MT][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  const int group_begin = blockIdx.y * steps_per_group;
  const int group_end = min(k_steps, group_begin + steps_per_group);
  const int step0 = group_begin + wave * KSTEPS;
  const int kbase = step0 * 32 + kg * 8;
  C += (size_t)blockIdx.y * M * ldc;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  // weight fragment s of a tile, with the k-step clamped into the matrix (the activations are zero there)
  const bf16* wbase = Wp + (size_t)lane * 8;
  int woff[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) woff[s] = (step0 + s < k_steps ? step0 + s : k_steps - 1) * 512;

  // a block takes a run of neighbouring column tiles: one contiguous piece of the packed weights
  const int tiles_per_block = (n_tiles + gridDim.x - 1) / gridDim.x;
  const int tile_begin = blockIdx.x * tiles_per_block, tile_end = min(n_tiles, tile_begin + tiles_per_block);
  uint4 w[KSTEPS], wn[PREFETCH ? KSTEPS : 1];
  if (PREFETCH) {
    const bf16* wt = wbase + (size_t)min(tile_begin, n_tiles - 1) * k_steps * 512;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) w[s] = ld16_stream(wt + woff[s]);
  }
  uint4 a[MT][KSTEPS];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + row;
    const bf16* ap = A + (size_t)(m < M ? m : M - 1) * lda;   // rows >= M read a real row and are zeroed
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      const uint4 v = ld16(ap + (k < K ? k : K - 8));
      a[mt][s] = (m < M && k < K && step0 + s < group_end) ? v : zero;
    }
  }

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    if (PREFETCH) {
      const int next = tile + 1 < tile_end ? tile + 1 : tile;   // the last round re-reads its own (from the cache)
      const bf16* wt = wbase + (size_t)next * k_steps * 512;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) wn[s] = ld16_stream(wt + woff[s]);
    } else {
      const bf16* wt = wbase + (size_t)tile * k_steps * 512;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) w[s] = ld16_stream(wt + woff[s]);
    }
    __builtin_amdgcn_sched_barrier(0);   // every load is issued before this tile's first MFMA
    f32x4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[mt][s]),
                                                          __builtin_bit_cast(bf16x8_t, w[s]), acc[mt], 0, 0, 0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(wave * MT + mt) * 256 + r * 64 + lane] = acc[mt][r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
      const int mt = idx >> 8, i = idx & 255;
      const int r = i >> 6, l2 = i & 63, col = l2 & 15;
      const int m = mt * 16 + (l2 >> 4) * 4 + r;
      if (c_mode == 0) {
        float s = 0.f;
        for (int w2 = 0; w2 < n_waves; ++w2) s += red[(w2 * MT + mt) * 256 + i];
        const int nn = tile * 16 + col;
        if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(s);
      } else if (col < 8) {
        float g = 0.f, u = 0.f;
        for (int w2 = 0; w2 < n_waves; ++w2) {
          g += red[(w2 * MT + mt) * 256 + i];
          u += red[(w2 * MT + mt) * 256 + i + 8];
        }
        const int nn = tile * 8 + col;
        if (m < M && nn < N / 2) C[(size_t)m * ldc + nn] = from_float<TC>(g / (1.0f + expf(-g)) * u);
      }
    }
    __syncthreads();
    if (PREFETCH) {
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) w[s] = wn[s];
    }
  }
}

// How K is cut: k-steps of 32 per wavefront and wavefronts per block; 0 if K is out of range.
//   K <= 512: 4 steps, <= 4 wavefronts;  K <= 4096: 16 steps, <= 8 wavefronts (512 threads);
//   K <= 8192: 32 steps, <= 8 wavefronts (512 threads);  K <= 16384: 32 steps, <= 16 wavefronts
//   (1024 threads, A fragments re-read per tile)
static int plan_k(int K, int* ksteps) {
  if (K <= 512) { *ksteps = 4; return (K + 127) / 128; }
  if (K <= 4096) { *ksteps = 16; return (K + 511) / 512; }
  if (K <= 16384) { *ksteps = 32; return (K + 1023) / 1024; }
  return 0;
}

// The largest K that one K-group may span for M rows (more rows leave fewer registers per k-step).
extern "C" int blm_gemv_mfma_group_limit(int M) {
  if (M < 1 || M > 64) return 0;
  return M <= 16 ? 16384 : (M <= 32 ? 4096 : 2048);
}

// Whether the product runs with all of K in one group.
extern "C" int blm_gemv_mfma_supported(int M, int N, int K) {
  return (N >= 1 && K >= 8 && K % 8 == 0 && K <= blm_gemv_mfma_group_limit(M)) ? 1 : 0;
}

// The launch geometry of the product for M rows of [N, K] in k_groups groups of K: k-steps per
// wavefront, wavefronts per block, and blocks per group.  A block takes a run of neighbouring column
// tiles; enough blocks to fill the chip, few enough that a block uses its activations more than once,
// and only blocks that have a tile.
struct GemvGeometry {
  int ksteps, waves, blocks;
};
static GemvGeometry gemv_geometry(int M, int N, int K, int k_groups) {
  const int n_tiles = (N + 15) / 16;
  const int k_steps = (K + 31) / 32;
  const int steps_per_group = (k_steps + k_groups - 1) / k_groups;
  GemvGeometry g{0, 0, 0};
  int cap;
  if (M > 16) {
    g.ksteps = steps_per_group > 64 ? 16 : 8;   // more than 2048 of K per group: two row tiles at most
    g.waves = (steps_per_group + g.ksteps - 1) / g.ksteps;   // at most 8 by the group limit
    cap = 256 / k_groups;
  } else {
    g.waves = plan_k(steps_per_group * 32, &g.ksteps);
    cap = (g.waves > 4 ? 256 : 512) / k_groups;
  }
  int blocks = n_tiles < cap ? n_tiles : (cap > 0 ? cap : 1);
  const int tiles_per_block = (n_tiles + blocks - 1) / blocks;
  g.blocks = (n_tiles + tiles_per_block - 1) / tiles_per_block;   // the kernel derives the same tiles per block from it
  return g;
}

// Blocks (over all groups) and wavefronts per block that blm_gemv_mfma launches; 0 if K does not fit.
extern "C" int blm_gemv_mfma_geometry(int M, int N, int K, int k_groups, int* blocks, int* waves) {
  if (M < 1 || M > 64 || N < 1 || K < 8 || k_groups < 1 || k_groups > 64) return 0;
  const int per_group = ((K + 31) / 32 + k_groups - 1) / k_groups * 32;
  if (per_group > blm_gemv_mfma_group_limit(M)) return 0;
  const GemvGeometry g = gemv_geometry(M, N, K, k_groups);
  *blocks = g.blocks * k_groups;
  *waves = g.waves;
  return 1;
}

template <typename TC>
static int launch_mfma(const void* A, const void* Wp, void* C, int M, int N, int K, int lda, int ldc, int c_mode,
                       int k_groups, hipStream_t stream) {
  const int n_tiles = (N + 15) / 16;
  const int k_steps = (K + 31) / 32;
  const int steps_per_group = (k_steps + k_groups - 1) / k_groups;
  const GemvGeometry geo = gemv_geometry(M, N, K, k_groups);
  if (M > 16) {
    const int mt = (M + 15) / 16;
    const int ks = geo.ksteps, waves = geo.waves, blocks = geo.blocks;
    dim3 grid(blocks, k_groups), block(waves * BLM_WAVE);
    const size_t smem = (size_t)waves * mt * 256 * sizeof(float);
#define BLM_GR(MT, KS, PF)                                                                                      \
  hipLaunchKernelGGL((gemv_mfma_rows_kernel<MT, KS, PF, TC>), grid, block, smem, stream, (const bf16*)A,        \
                     (const bf16*)Wp, (TC*)C, M, N, K, lda, ldc, n_tiles, k_steps, c_mode, steps_per_group)
    if (ks == 16) BLM_GR(2, 16, false);
    else if (mt == 2) BLM_GR(2, 8, true);
    else if (mt == 3) BLM_GR(3, 8, true);
    else BLM_GR(4, 8, true);
#undef BLM_GR
    BLM_LAUNCH_CHECK("gemv_mfma_rows");
    return 0;
  }
  const int ksteps = geo.ksteps, waves = geo.waves, blocks = geo.blocks;
  dim3 grid(blocks, k_groups), block(waves * BLM_WAVE);
  const size_t smem = (size_t)waves * 256 * sizeof(float);
#define BLM_GM(KS, MAXT, KEEP)                                                                                  \
  hipLaunchKernelGGL((gemv_mfma_kernel<KS, MAXT, KEEP, TC>), grid, block, smem, stream, (const bf16*)A,         \
                     (const bf16*)Wp, (TC*)C, M, N, K, lda, ldc, n_tiles, k_steps, c_mode, steps_per_group)
  if (ksteps == 4) BLM_GM(4, 256, true);
  else if (ksteps == 16 && waves <= 4) BLM_GM(16, 256, true);
  else if (ksteps == 16) BLM_GM(16, 512, true);
  else if (waves <= 8) BLM_GM(32, 512, true);
  else BLM_GM(32, 1024, false);
#undef BLM_GM
  BLM_LAUNCH_CHECK("gemv_mfma");
  return 0;
}

// Wp: the packed copy of W[N, K] (see the head of this file), ceil(N/16) * ceil(K/32) * 512 elements.
// c_mode 0: C[M, N] = A W^T.
// c_mode 1: the rows of W come in blocks of 8 gate rows followed by their 8 up rows (so every
//           16-column tile holds 8 gated pairs) and C[M, N/2] = silu(gate) * up: the SwiGLU gating
//           fused into the product that feeds it.
// k_groups > 1: K is cut into that many groups handled by different blocks; C is then float
// [k_groups, M, ldc] and holds one partial product per group, to be summed by the reader (the
// residual add in front of the next norm does it), so narrow outputs still occupy the whole chip.
extern "C" int blm_gemv_mfma(const void* A, const void* Wp, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldc, int c_mode, int k_groups, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= 64, "gemv_mfma: M=%d out of range 1..64", M);
  BLM_REQUIRE(N >= 1 && K >= 8 && K % 8 == 0, "gemv_mfma: sizes N=%d K=%d not supported (K a multiple of 8)", N, K);
  BLM_REQUIRE(c_mode == 0 || (c_mode == 1 && N % 16 == 0 && k_groups == 1),
              "gemv_mfma: c_mode %d needs N a multiple of 16 and one K group", c_mode);
  BLM_REQUIRE(k_groups >= 1 && k_groups <= 64 && (k_groups == 1 || c_dtype == BLM_F32),
              "gemv_mfma: k_groups=%d needs 1..64 and a float output when above 1", k_groups);
  {
    const int steps = (K + 31) / 32, per_group = (steps + k_groups - 1) / k_groups;
    BLM_REQUIRE(per_group * 32 <= blm_gemv_mfma_group_limit(M),
                "gemv_mfma: %d rows take at most K=%d per group, got K=%d in %d group(s)", M,
                blm_gemv_mfma_group_limit(M), K, k_groups);
  }
  BLM_REQUIRE(lda % 8 == 0 && lda >= K && ldc >= (c_mode ? N / 2 : N), "gemv_mfma: bad strides lda=%d ldc=%d", lda, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)Wp % 16) == 0, "gemv_mfma: operands must be 16-byte aligned");
  if (c_dtype == BLM_BF16) return launch_mfma<bf16>(A, Wp, C, M, N, K, lda, ldc, c_mode, k_groups, stream);
  if (c_dtype == BLM_F32) return launch_mfma<float>(A, Wp, C, M, N, K, lda, ldc, c_mode, k_groups, stream);
  return blm_fail("gemv_mfma: unsupported output dtype %d", c_dtype);
}
