// Skinny matrix product for decode on the matrix cores: C[M<=16, N] = A[M, K] * W[N, K]^T, bf16
// operands, float accumulation, bf16 or float output.
//
// The weight matrix is streamed exactly once.  A block owns tiles of 16 output columns; its
// wavefronts split K between them.  For the MFMA 16x16x32 the weight tile is the B operand: lane
// l holds W[n0 + l%16][k0 + (l/16)*8 .. +8], which is one 16-byte load from a K-contiguous row.
// The activations are the A operand (row m = l%16, rows >= M are zero) and stay in registers for
// the block's whole life, so a block that walks several column tiles reads them once.  The
// partial tiles of the wavefronts are summed through shared memory in a fixed order.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ uint4 ld16(const bf16* p) { return *reinterpret_cast<const uint4*>(p); }

// KSTEPS: k-steps of 32 per wavefront.  MAXT: most threads of a block (sets the register budget).
// KEEP_A: the activations' fragments stay in registers across the block's column tiles.
template <int KSTEPS, int MAXT, bool KEEP_A, typename TC>
__global__ void __launch_bounds__(MAXT)
    gemv_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C, int M, int N,
                     int K, int lda, int ldc, int n_tiles) {
  extern __shared__ float red[];  // [waves][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  const int kbase = wave * (KSTEPS * 32) + kg * 8;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  const int arow = row < M ? row : M - 1;   // rows >= M read a real row and are zeroed, so every load is in bounds
  const bf16* ap = A + (size_t)arow * lda;

  // Fragments of A beyond K or beyond M are zero, so whatever W holds there adds nothing; the
  // weight loads can then be unconditional, with their addresses clamped into the matrix.
  uint4 a[KSTEPS];
  if (KEEP_A) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      const uint4 v = ld16(ap + (k < K ? k : K - 8));
      a[s] = (row < M && k < K) ? v : zero;
    }
  }

  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int n = tile * 16 + row;
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
          const uint4 v = ld16(ap + (k < K ? k : K - 8));
          a[c + s] = (row < M && k < K) ? v : zero;
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
    // acc[r] is C[m = kg*4 + r][n = tile*16 + row]
    if (n_waves == 1) {
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
        float s = 0.f;
        for (int w2 = 0; w2 < n_waves; ++w2) s += red[w2 * 256 + idx];
        const int r = idx >> 6, l2 = idx & 63;
        const int m = (l2 >> 4) * 4 + r, nn = tile * 16 + (l2 & 15);
        if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(s);
      }
      __syncthreads();
    }
  }
}

// How K is cut: k-steps of 32 per wavefront and wavefronts per block; 0 if K is out of range.
//   K <= 512          4 steps, up to 4 wavefronts
//   K <= 2048        16 steps, up to 4 wavefronts   (256 threads: registers are plentiful)
//   K <= 8192        32 steps, up to 8 wavefronts   (512 threads: 256 registers a lane)
//   K <= 16384       32 steps, up to 16 wavefronts  (1024 threads: the A fragments are re-read per tile)
static int plan_k(int K, int* ksteps) {
  if (K <= 512) { *ksteps = 4; return (K + 127) / 128; }
  if (K <= 2048) { *ksteps = 16; return (K + 511) / 512; }
  if (K <= 16384) { *ksteps = 32; return (K + 1023) / 1024; }
  return 0;
}

extern "C" int blm_gemv_mfma_supported(int M, int N, int K) {
  int ks;
  return (M >= 1 && M <= 16 && N >= 1 && K >= 8 && K % 8 == 0 && plan_k(K, &ks) > 0) ? 1 : 0;
}

template <typename TC>
static int launch_mfma(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldc,
                       hipStream_t stream) {
  int ksteps = 0;
  const int waves = plan_k(K, &ksteps);
  const int n_tiles = (N + 15) / 16;
  // enough blocks to fill the chip, few enough that a block reuses its activations
  int blocks = n_tiles;
  const int cap = waves > 4 ? 256 : 512;
  if (blocks > cap) blocks = cap;
  dim3 grid(blocks), block(waves * BLM_WAVE);
  const size_t smem = waves > 1 ? (size_t)waves * 256 * sizeof(float) : 0;
#define BLM_GM(KS, MAXT, KEEP)                                                                                  \
  hipLaunchKernelGGL((gemv_mfma_kernel<KS, MAXT, KEEP, TC>), grid, block, smem, stream, (const bf16*)A,         \
                     (const bf16*)W, (TC*)C, M, N, K, lda, ldc, n_tiles)
  if (ksteps == 4) BLM_GM(4, 256, true);
  else if (ksteps == 16) BLM_GM(16, 256, true);
  else if (waves <= 8) BLM_GM(32, 512, true);
  else BLM_GM(32, 1024, false);
#undef BLM_GM
  BLM_LAUNCH_CHECK("gemv_mfma");
  return 0;
}

extern "C" int blm_gemv_mfma(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldc, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= 16, "gemv_mfma: M=%d out of range 1..16", M);
  BLM_REQUIRE(blm_gemv_mfma_supported(M, N, K), "gemv_mfma: sizes N=%d K=%d not supported (K a multiple of 8, at most 16384)", N, K);
  BLM_REQUIRE(lda % 8 == 0 && lda >= K && ldc >= N, "gemv_mfma: bad strides lda=%d ldc=%d", lda, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemv_mfma: operands must be 16-byte aligned");
  if (c_dtype == BLM_BF16) return launch_mfma<bf16>(A, W, C, M, N, K, lda, ldc, stream);
  if (c_dtype == BLM_F32) return launch_mfma<float>(A, W, C, M, N, K, lda, ldc, stream);
  return blm_fail("gemv_mfma: unsupported output dtype %d", c_dtype);
}
