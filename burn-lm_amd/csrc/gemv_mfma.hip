// Skinny matrix product for decode on the matrix cores: C[M<=16, N] = A[M, K] * W[N, K]^T, bf16
// operands, float accumulation, bf16 or float output.
//
// The weight matrix is streamed exactly once.  A block owns tiles of 16 output columns; its
// wavefronts split K between them.  For the MFMA 16x16x32 the weight tile is the B operand: lane
// l holds W[n0 + l%16][k0 + (l/16)*8 .. +8], which is one 16-byte load from a K-contiguous row.
// The activations are the A operand (row m = l%16, rows >= M are zero) and stay in registers for
// the block's whole life, so a block that walks several column tiles reads them once.  The
// partial tiles of the wavefronts are summed through shared memory in a fixed order.  The SwiGLU
// gating of a feed-forward can be fused into the operand load (a_mode 1).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ uint4 ld16(const bf16* p) { return *reinterpret_cast<const uint4*>(p); }

// A fragment of the activations: 8 consecutive k of row `ap`.  mode 0: the row itself.  mode 1:
// the row holds [gate | up] (2K wide) and the fragment is silu(gate) * up, computed in float and
// rounded once to bf16 (the SwiGLU gating fused into the operand load of the down projection).
__device__ __forceinline__ uint4 load_a(const bf16* ap, int k, int K, int mode) {
  const uint4 g = ld16(ap + k);
  if (mode == 0) return g;
  const uint4 u = ld16(ap + K + k);
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    const float f0 = g0 / (1.0f + expf(-g0)) * u0, f1 = g1 / (1.0f + expf(-g1)) * u1;
    o[i] = (uint32_t)f32_to_bf16_bits(f0) | ((uint32_t)f32_to_bf16_bits(f1) << 16);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// KSTEPS: k-steps of 32 per wavefront (per K-half in HALF mode).  MAXT: most threads of a block
// (sets the register budget).  KEEP_A: the activations' fragments stay in registers across the
// block's column tiles.
// HALF (M <= 8): a tile is 8 output columns.  The 16 MFMA columns are (column n, K-half hb) and
// the 16 MFMA rows (activation row m, K-half ha); the diagonal quadrants ha == hb hold the two
// halves of the wanted dot products and are summed, the others are dropped.  Narrow outputs get
// twice as many tiles this way, enough to occupy every compute unit.
template <int KSTEPS, int MAXT, bool KEEP_A, bool HALF, typename TC>
__global__ void __launch_bounds__(MAXT)
    gemv_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C, int M, int N,
                     int K, int lda, int ldc, int n_tiles, int a_mode) {
  extern __shared__ float red[];  // [waves][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  constexpr int TILE_N = HALF ? 8 : 16;
  constexpr int WAVE_K = HALF ? KSTEPS * 64 : KSTEPS * 32;
  const int half = HALF ? (row >> 3) : 0;        // K-half of this lane's MFMA row / column
  const int rsub = HALF ? (row & 7) : row;       // activation row / column within the tile
  const int kbase = wave * WAVE_K + half * (KSTEPS * 32) + kg * 8;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  const int arow = rsub < M ? rsub : M - 1;   // rows >= M read a real row and are zeroed, so every load is in bounds
  const bf16* ap = A + (size_t)arow * lda;

  // Fragments of A beyond K or beyond M are zero, so whatever W holds there adds nothing; the
  // weight loads can then be unconditional, with their addresses clamped into the matrix.
  uint4 a[KSTEPS];
  if (KEEP_A) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      const uint4 v = load_a(ap, k < K ? k : K - 8, K, a_mode);
      a[s] = (rsub < M && k < K) ? v : zero;
    }
  }

  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int n = tile * TILE_N + rsub;
    const bf16* wrow = W + (size_t)(n < N ? n : N - 1) * K;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int CH = KSTEPS < 16 ? KSTEPS : 16;   // weight loads in flight per wavefront
#pragma unroll
    for (int c = 0; c < KSTEPS; c += CH) {
      uint4 w[CH];
#pragma unroll
      for (int s = 0; s < CH; ++s) {
        const int k = kbase + (c + s) * 32;
        w[s] = ld16(wrow + (k < K ? k : K - 8));
      }
      if (!KEEP_A) {
#pragma unroll
        for (int s = 0; s < CH; ++s) {
          const int k = kbase + (c + s) * 32;
          const uint4 v = load_a(ap, k < K ? k : K - 8, K, a_mode);
          a[c + s] = (rsub < M && k < K) ? v : zero;
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
    // acc[r] is the product of MFMA row kg*4 + r and MFMA column `row`
    if (!HALF && n_waves == 1) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = kg * 4 + r;
        if (m < M && n < N) C[(size_t)m * ldc + n] = from_float<TC>(acc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
      __syncthreads();
      if (!HALF) {
        for (int idx = threadIdx.x; idx < 256; idx += blockDim.x) {  // a block may have fewer than 256 threads
          float s = 0.f;
          for (int w2 = 0; w2 < n_waves; ++w2) s += red[w2 * 256 + idx];
          const int r = idx >> 6, l2 = idx & 63;
          const int m = (l2 >> 4) * 4 + r, nn = tile * 16 + (l2 & 15);
          if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(s);
        }
      } else {
        for (int idx = threadIdx.x; idx < 64; idx += blockDim.x) {   // 8 rows x 8 columns
          const int m = idx >> 3, j = idx & 7;
          float s = 0.f;
          for (int w2 = 0; w2 < n_waves; ++w2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              // MFMA row h*8 + m = kg2*4 + r  ->  kg2 = h*2 + m/4, r = m%4;  MFMA column h*8 + j
              const int l2 = (h * 2 + (m >> 2)) * 16 + h * 8 + j;
              s += red[w2 * 256 + (m & 3) * 64 + l2];
            }
          }
          const int nn = tile * 8 + j;
          if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(s);
        }
      }
      __syncthreads();
    }
  }
}

// How K is cut: k-steps of 32 per wavefront and wavefronts per block; 0 if K is out of range.
//   16-column tiles:  K <= 512: 4 steps, <= 4 wavefronts;  K <= 2048: 16 steps, <= 4 wavefronts (256 threads);
//                     K <= 8192: 32 steps, <= 8 wavefronts (512 threads);  K <= 16384: 32 steps, <= 16 wavefronts
//                     (1024 threads, A fragments re-read per tile)
//   8-column tiles:   a wavefront covers twice as much of K (64 per step)
//                     K <= 512: 4 steps, <= 2;  K <= 4096: 8 steps, <= 8;  K <= 8192: 16 steps, <= 8;
//                     K <= 16384: 32 steps, <= 8 (all 512 threads at most)
static int plan_k(int K, bool half, int* ksteps) {
  if (!half) {
    if (K <= 512) { *ksteps = 4; return (K + 127) / 128; }
    if (K <= 2048) { *ksteps = 16; return (K + 511) / 512; }
    if (K <= 16384) { *ksteps = 32; return (K + 1023) / 1024; }
    return 0;
  }
  if (K <= 512) { *ksteps = 4; return (K + 255) / 256; }
  if (K <= 4096) { *ksteps = 8; return (K + 511) / 512; }
  if (K <= 8192) { *ksteps = 16; return (K + 1023) / 1024; }
  if (K <= 16384) { *ksteps = 32; return (K + 2047) / 2048; }
  return 0;
}

extern "C" int blm_gemv_mfma_supported(int M, int N, int K) {
  int ks;
  return (M >= 1 && M <= 16 && N >= 1 && K >= 8 && K % 8 == 0 && plan_k(K, false, &ks) > 0) ? 1 : 0;
}

template <typename TC>
static int launch_mfma(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldc, int a_mode,
                       hipStream_t stream) {
  // narrow outputs with few rows: 8-column tiles, so that there are tiles for every compute unit
  const bool half = M <= 8 && (N + 15) / 16 < 512;
  int ksteps = 0;
  const int waves = plan_k(K, half, &ksteps);
  const int n_tiles = half ? (N + 7) / 8 : (N + 15) / 16;
  // enough blocks to fill the chip, few enough that a block reuses its activations
  int blocks = n_tiles;
  const int cap = waves > 4 ? 256 : 512;
  if (blocks > cap) blocks = cap;
  dim3 grid(blocks), block(waves * BLM_WAVE);
  const size_t smem = (size_t)waves * 256 * sizeof(float);
#define BLM_GM(KS, MAXT, KEEP, HALF)                                                                            \
  hipLaunchKernelGGL((gemv_mfma_kernel<KS, MAXT, KEEP, HALF, TC>), grid, block, smem, stream, (const bf16*)A,   \
                     (const bf16*)W, (TC*)C, M, N, K, lda, ldc, n_tiles, a_mode)
  if (half) {
    if (ksteps == 4) BLM_GM(4, 128, true, true);
    else if (ksteps == 8) BLM_GM(8, 512, true, true);
    else if (ksteps == 16) BLM_GM(16, 512, true, true);
    else BLM_GM(32, 512, true, true);
  } else {
    if (ksteps == 4) BLM_GM(4, 256, true, false);
    else if (ksteps == 16) BLM_GM(16, 256, true, false);
    else if (waves <= 8) BLM_GM(32, 512, true, false);
    else BLM_GM(32, 1024, false, false);
  }
#undef BLM_GM
  BLM_LAUNCH_CHECK("gemv_mfma");
  return 0;
}

// a_mode 0: A is [M, K].  a_mode 1: A is [M, 2K] = [gate | up] and the product runs on silu(gate) * up.
extern "C" int blm_gemv_mfma(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldc, int a_mode, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= 16, "gemv_mfma: M=%d out of range 1..16", M);
  BLM_REQUIRE(blm_gemv_mfma_supported(M, N, K), "gemv_mfma: sizes N=%d K=%d not supported (K a multiple of 8, at most 16384)", N, K);
  BLM_REQUIRE(a_mode == 0 || a_mode == 1, "gemv_mfma: a_mode %d unknown", a_mode);
  BLM_REQUIRE(lda % 8 == 0 && lda >= (a_mode ? 2 * K : K) && ldc >= N, "gemv_mfma: bad strides lda=%d ldc=%d", lda, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemv_mfma: operands must be 16-byte aligned");
  if (c_dtype == BLM_BF16) return launch_mfma<bf16>(A, W, C, M, N, K, lda, ldc, a_mode, stream);
  if (c_dtype == BLM_F32) return launch_mfma<float>(A, W, C, M, N, K, lda, ldc, a_mode, stream);
  return blm_fail("gemv_mfma: unsupported output dtype %d", c_dtype);
}
