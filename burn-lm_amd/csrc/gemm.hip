// Matrix products C[M,N] = A[M,K] * W[N,K]^T (W in checkpoint layout, K contiguous).
//   gemm_tiled   : any sizes, any mix of float / bf16 operands, float accumulation with plain
//                  fused multiply-adds.  It is the true 32-bit product of the float path and the
//                  always-right fallback.  From 32 rows and 32 columns on the multiply-adds are
//                  those of the matrix cores' float instruction (v_mfma_f32_32x32x2_f32: float
//                  operands, float products, float sums, nothing narrowed), which does the same
//                  arithmetic about five times as fast.
//   gemv_skinny  : M <= 8 rows (decode).  Streams each weight row once with 16-byte loads;
//                  every wavefront owns output columns and reduces over K across its lanes.
#include "common.h"

// ---------------------------------------------------------------------------------------
// tiled product, 64x64 tile per 256 threads, 4x4 outputs per thread
// ---------------------------------------------------------------------------------------
#define GT_BM 64
#define GT_BN 64
#define GT_BK 16
#define GT_CHUNK 64   // elements of K per first-level sum, a multiple of GT_BK

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
    gemm_tiled_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M,
                      int N, int K, int lda, int ldc) {
  __shared__ float As[GT_BK][GT_BM + 4];
  __shared__ float Ws[GT_BK][GT_BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
  const int tr = tid / 16, tc = tid % 16;  // thread's 4x4 block: rows tr*4.., cols tc*4..
  // sums in two levels (GT_CHUNK elements of K, then the chunks), so that the rounding error does
  // not grow with K additions in a row
  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GT_BK) {
    if (k0 > 0 && k0 % GT_CHUNK == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; k fastest for coalescing
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx / GT_BK, kk = idx % GT_BK;
      const int gk = k0 + kk;
      float a = 0.f, w = 0.f;
      if (gk < K) {
        if (m0 + r < M) a = to_float(A[(size_t)(m0 + r) * lda + gk]);
        if (n0 + r < N) w = to_float(W[(size_t)(n0 + r) * K + gk]);
      }
      As[kk][r] = a;
      Ws[kk][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][tr * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tc * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tr * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tc * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = from_float<TC>(total[i][j] + acc[i][j]);
    }
  }
}

// ---------------------------------------------------------------------------------------
// the same product on the matrix cores' float instruction: 128x128 tile per 512 threads, each
// wavefront 64 rows x 32 columns as two instructions of 32x32, K in steps of 16 through shared memory
// (operands of either type become float there).  Lane l of a 32x32x2 instruction supplies
// A[l % 32][l / 32] and B[l / 32][l % 32] and holds C[8 (v / 4) + 4 (l / 32) + v % 4][l % 32], v < 16.
// ---------------------------------------------------------------------------------------
#define GF_BM 128
#define GF_BN 128
#define GF_BK 16
#define GF_CHUNK 128   // elements of K per first-level sum, a multiple of GF_BK
typedef __attribute__((ext_vector_type(16))) float gf_f32x16;

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(512, 4)   // 128 registers: two blocks per compute unit
    gemm_f32_mfma_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M, int N, int K,
                         int lda, int ldc) {
  __shared__ float As[GF_BK][GF_BM + 4];
  __shared__ float Ws[GF_BK][GF_BN + 4];
  const int tid = threadIdx.x, wave = tid / BLM_WAVE, lane = tid & (BLM_WAVE - 1);
  const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
  const int wm = (wave >> 2) * 64, wn = (wave & 3) * 32;   // eight wavefronts, each 64 rows x 32 columns
  const int li = lane & 31, lk = lane >> 5;
  // Sums in two levels: `acc` takes the products of GF_CHUNK elements of K and is then added to
  // `total`.  One accumulator over all of K would make K/2 additions in a row to a sum that keeps
  // growing, and its rounding error grows with them (measured at K = 8,192 against a 64-bit
  // product: 5e-6 of the largest result, four times a product that is split over K).  The second
  // set of sums is why a wavefront's tile is no larger: with 64 x 64 the two sets take the
  // registers of half the wavefronts.
  gf_f32x16 total[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) total[i][v] = 0.f;
  for (int c0 = 0; c0 < K; c0 += GF_CHUNK) {
    gf_f32x16 acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    const int c1 = c0 + GF_CHUNK < K ? c0 + GF_CHUNK : K;
    for (int k0 = c0; k0 < c1; k0 += GF_BK) {
#pragma unroll
      for (int e = 0; e < GF_BK / 4; ++e) {   // 128 rows x GF_BK k per operand, k fastest
        const int idx = tid + e * 512;
        const int r = idx / GF_BK, kk = idx % GF_BK;
        const int gk = k0 + kk;
        float a = 0.f, w = 0.f;
        if (gk < K) {
          if (m0 + r < M) a = to_float(A[(size_t)(m0 + r) * lda + gk]);
          if (n0 + r < N) w = to_float(W[(size_t)(n0 + r) * K + gk]);
        }
        As[kk][r] = a;
        Ws[kk][r] = w;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < GF_BK; kk += 2) {
        const float b = Ws[kk + lk][wn + li];
#pragma unroll
        for (int i = 0; i < 2; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(As[kk + lk][wm + i * 32 + li], b, acc[i], 0, 0, 0);
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) total[i] += acc[i];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3), n = n0 + wn + li;
      if (m < M && n < N) C[(size_t)m * ldc + n] = from_float<TC>(total[i][v]);
    }
}

template <typename TA, typename TW, typename TC>
static int launch_tiled(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldc,
                        hipStream_t stream) {
  if (M >= 32 && N >= 32) {
    dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM), block(512);
    if (grid.y > 65535) return blm_fail("gemm_tiled: M=%d too large", M);
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)A, (const TW*)W,
                       (TC*)C, M, N, K, lda, ldc);
    BLM_LAUNCH_CHECK("gemm_f32_mfma");
    return 0;
  }
  dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM), block(256);
  if (grid.y > 65535) return blm_fail("gemm_tiled: M=%d too large", M);
  hipLaunchKernelGGL((gemm_tiled_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)A, (const TW*)W,
                     (TC*)C, M, N, K, lda, ldc);
  BLM_LAUNCH_CHECK("gemm_tiled");
  return 0;
}

extern "C" int blm_gemm_tiled(const void* A, int a_dtype, const void* W, int w_dtype, void* C,
                              int c_dtype, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
  BLM_REQUIRE(M > 0 && N > 0 && K > 0 && lda >= K && ldc >= N, "gemm_tiled: bad sizes M=%d N=%d K=%d lda=%d ldc=%d",
              M, N, K, lda, ldc);
  const int code = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (code) {
    case 0: return launch_tiled<float, float, float>(A, W, C, M, N, K, lda, ldc, stream);
    case 1: return launch_tiled<float, float, bf16>(A, W, C, M, N, K, lda, ldc, stream);
    case 2: return launch_tiled<float, bf16, float>(A, W, C, M, N, K, lda, ldc, stream);
    case 3: return launch_tiled<float, bf16, bf16>(A, W, C, M, N, K, lda, ldc, stream);
    case 4: return launch_tiled<bf16, float, float>(A, W, C, M, N, K, lda, ldc, stream);
    case 5: return launch_tiled<bf16, float, bf16>(A, W, C, M, N, K, lda, ldc, stream);
    case 6: return launch_tiled<bf16, bf16, float>(A, W, C, M, N, K, lda, ldc, stream);
    case 7: return launch_tiled<bf16, bf16, bf16>(A, W, C, M, N, K, lda, ldc, stream);
  }
  return blm_fail("gemm_tiled: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
}

// ---------------------------------------------------------------------------------------
// skinny product for decode: MT <= 8 rows of A against all of W
// ---------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v);
template <>
__device__ __forceinline__ void load8<bf16>(const bf16* p, float* v) {
  const uint4 r = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

#define GV_WAVES 4
#define GV_COLS 2  // output columns per wavefront per pass

template <typename TA, typename TW, typename TC, int MT>
__global__ void __launch_bounds__(GV_WAVES* BLM_WAVE)
    gemv_skinny_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int N,
                       int K, int lda, int ldc) {
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_groups = (N + GV_COLS - 1) / GV_COLS;
  for (int g = blockIdx.x * GV_WAVES + wave; g < n_groups; g += gridDim.x * GV_WAVES) {
    const int n0 = g * GV_COLS;
    float acc[GV_COLS][MT];
#pragma unroll
    for (int c = 0; c < GV_COLS; ++c)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[c][m] = 0.f;
    for (int k = lane * 8; k < K; k += BLM_WAVE * 8) {
      float a[MT][8];
#pragma unroll
      for (int m = 0; m < MT; ++m) load8<TA>(A + (size_t)m * lda + k, a[m]);
#pragma unroll
      for (int c = 0; c < GV_COLS; ++c) {
        if (n0 + c < N) {
          float w[8];
          load8<TW>(W + (size_t)(n0 + c) * K + k, w);
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[c][m] = fmaf(a[m][i], w[i], acc[c][m]);
        }
      }
    }
#pragma unroll
    for (int c = 0; c < GV_COLS; ++c)
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float s = wave_sum(acc[c][m]);
        if (lane == 0 && n0 + c < N) C[(size_t)m * ldc + n0 + c] = from_float<TC>(s);
      }
  }
}

template <typename TA, typename TW, typename TC>
static int launch_skinny(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldc,
                         hipStream_t stream) {
  const int n_groups = (N + GV_COLS - 1) / GV_COLS;
  int blocks = (n_groups + GV_WAVES - 1) / GV_WAVES;
  if (blocks > 256 * 16) blocks = 256 * 16;
  dim3 grid(blocks), block(GV_WAVES * BLM_WAVE);
#define BLM_GV(MT)                                                                                  \
  hipLaunchKernelGGL((gemv_skinny_kernel<TA, TW, TC, MT>), grid, block, 0, stream, (const TA*)A,     \
                     (const TW*)W, (TC*)C, N, K, lda, ldc)
  switch (M) {
    case 1: BLM_GV(1); break;
    case 2: BLM_GV(2); break;
    case 3: BLM_GV(3); break;
    case 4: BLM_GV(4); break;
    case 5: BLM_GV(5); break;
    case 6: BLM_GV(6); break;
    case 7: BLM_GV(7); break;
    case 8: BLM_GV(8); break;
    default: return blm_fail("gemv_skinny: M=%d out of range 1..8", M);
  }
#undef BLM_GV
  BLM_LAUNCH_CHECK("gemv_skinny");
  return 0;
}

extern "C" int blm_gemv_skinny(const void* A, int a_dtype, const void* W, int w_dtype, void* C,
                               int c_dtype, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= 8, "gemv_skinny: M=%d out of range 1..8", M);
  BLM_REQUIRE(N > 0 && K > 0, "gemv_skinny: bad sizes N=%d K=%d", N, K);
  BLM_REQUIRE(K % 8 == 0 && lda % 8 == 0, "gemv_skinny: K=%d and lda=%d must be multiples of 8", K, lda);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemv_skinny: operands must be 16-byte aligned");
  BLM_REQUIRE(a_dtype == w_dtype, "gemv_skinny: A and W must share a dtype (got %d, %d)", a_dtype, w_dtype);
  if (a_dtype == BLM_F32 && c_dtype == BLM_F32)
    return launch_skinny<float, float, float>(A, W, C, M, N, K, lda, ldc, stream);
  if (a_dtype == BLM_BF16 && c_dtype == BLM_BF16)
    return launch_skinny<bf16, bf16, bf16>(A, W, C, M, N, K, lda, ldc, stream);
  if (a_dtype == BLM_BF16 && c_dtype == BLM_F32)
    return launch_skinny<bf16, bf16, float>(A, W, C, M, N, K, lda, ldc, stream);
  return blm_fail("gemv_skinny: unsupported dtypes a=%d c=%d", a_dtype, c_dtype);
}
