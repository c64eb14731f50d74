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

template <int KSTEPS, typename TC>
__global__ void __launch_bounds__(1024)
    gemv_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C, int M, int N,
                     int K, int lda, int ldc, int n_tiles) {
  extern __shared__ float red[];  // [waves][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  const int kbase = wave * (KSTEPS * 32) + kg * 8;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  uint4 a[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int k = kbase + s * 32;
    a[s] = (row < M && k < K) ? ld16(A + (size_t)row * lda + k) : zero;
  }

  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int n = tile * 16 + row;
    const bf16* wrow = W + (size_t)n * K;
    uint4 w[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      w[s] = (n < N && k < K) ? ld16(wrow + k) : zero;
    }
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                    __builtin_bit_cast(bf16x8_t, w[s]), acc, 0, 0, 0);
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

// how K is cut: k-steps of 32 per wavefront and wavefronts per block; 0 if K is out of range
static int plan_k(int K, int* ksteps) {
  if (K <= 512) { *ksteps = 4; return (K + 127) / 128; }
  if (K <= 8192) { *ksteps = 16; return (K + 511) / 512; }
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
  const int cap = waves >= 8 ? 256 : 512;
  if (blocks > cap) blocks = cap;
  dim3 grid(blocks), block(waves * BLM_WAVE);
  const size_t smem = waves > 1 ? (size_t)waves * 256 * sizeof(float) : 0;
#define BLM_GM(KS)                                                                                          \
  hipLaunchKernelGGL((gemv_mfma_kernel<KS, TC>), grid, block, smem, stream, (const bf16*)A, (const bf16*)W, \
                     (TC*)C, M, N, K, lda, ldc, n_tiles)
  if (ksteps == 4) BLM_GM(4);
  else if (ksteps == 16) BLM_GM(16);
  else BLM_GM(32);
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
