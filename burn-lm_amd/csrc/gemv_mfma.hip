// Skinny matrix product for decode on the matrix cores: C[M<=16, N] = A[M, K] * W[N, K]^T, bf16
// operands, float accumulation, bf16 or float output.
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
// feed-forward can be fused into the operand load (a_mode 1).
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
    // fast exponential and reciprocal: their error (~1e-7 relative) is far below the bf16 rounding of the result
    const float f0 = g0 * __frcp_rn(1.0f + __expf(-g0)) * u0, f1 = g1 * __frcp_rn(1.0f + __expf(-g1)) * u1;
    o[i] = (uint32_t)f32_to_bf16_bits(f0) | ((uint32_t)f32_to_bf16_bits(f1) << 16);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// KSTEPS: k-steps of 32 per wavefront.  MAXT: most threads of a block (sets the register budget).
// KEEP_A: the activations' fragments stay in registers across the block's column tiles.
template <int KSTEPS, int MAXT, bool KEEP_A, typename TC>
__global__ void __launch_bounds__(MAXT)
    gemv_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, TC* __restrict__ C, int M, int N,
                     int K, int lda, int ldc, int n_tiles, int k_steps, int a_mode, int steps_per_group) {
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
  if (KEEP_A) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      const uint4 v = load_a(ap, k < K ? k : K - 8, K, a_mode);
      a[s] = (row < M && k < K && step0 + s < group_end) ? v : zero;
    }
  }

  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const bf16* wt = Wp + ((size_t)tile * k_steps * 64 + lane) * 8;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int CH = KSTEPS < 16 ? KSTEPS : 16;   // weight loads in flight per wavefront
#pragma unroll
    for (int c = 0; c < KSTEPS; c += CH) {
      uint4 w[CH];
#pragma unroll
      for (int s = 0; s < CH; ++s) {
        const int st = step0 + c + s;
        w[s] = ld16(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);
      }
      if (!KEEP_A) {
#pragma unroll
        for (int s = 0; s < CH; ++s) {
          const int k = kbase + (c + s) * 32;
          const uint4 v = load_a(ap, k < K ? k : K - 8, K, a_mode);
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
    // acc[r] is C[m = kg*4 + r][n = tile*16 + row]
    if (n_waves == 1) {
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

// ---------------------------------------------------------------------------------------
// Variant with the activations staged in shared memory.
//
// A block owns TPB column tiles at a time and one K-group.  It first loads its slice of the
// activations (rows < M, the group's k range) with coalesced 16-byte loads, applies the SwiGLU
// gating if asked (so each gated value is computed once per block), and keeps the slice in LDS with
// a row skew of 16 bytes that makes the fragment reads conflict-free.  Wavefront w works on tile
// w / KW with k-steps (w % KW) * 16 ..; its weight loads are contiguous kilobytes of the packed
// copy and its A fragments come from LDS, so the registers hold weights in flight and little else.
// The KW partial tiles of a column tile are summed through LDS in a fixed order.
// ---------------------------------------------------------------------------------------
#define GL_KSTEPS 16

template <typename TC>
__global__ void __launch_bounds__(1024)
    gemv_mfma_lds_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, TC* __restrict__ C, int M, int N,
                         int K, int lda, int ldc, int n_tiles, int k_steps, int a_mode, int steps_per_group,
                         int kw_count, int tpb) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int row = lane & 15, kg = lane >> 4;
  const int group_begin = blockIdx.y * steps_per_group;
  const int group_end = min(k_steps, group_begin + steps_per_group);
  const int group_k = (group_end - group_begin) * 32;     // elements of k in this group (padded to 32)
  const int lds_stride = group_k + 8;                     // elements; 16 bytes of skew per row
  bf16* a_lds = reinterpret_cast<bf16*>(smem);
  float* red = reinterpret_cast<float*>(smem + (((size_t)M * lds_stride * 2 + 15) & ~(size_t)15));
  C += (size_t)blockIdx.y * M * ldc;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  const int tw = wave / kw_count, kw = wave - tw * kw_count;
  const int step0 = group_begin + kw * GL_KSTEPS;
  const bf16* arow = a_lds + (size_t)(row < M ? row : 0) * lds_stride + (kw * GL_KSTEPS * 32 + kg * 8);

  // The weight loads of the first tile go out before the activations are staged: they do not depend
  // on them, and the two memory round trips then overlap.
  int tile0 = blockIdx.x * tpb;
  uint4 w[GL_KSTEPS];
  {
    const int ltile = min(tile0 + tw, n_tiles - 1);   // wavefronts past the end load a real tile and drop it
    const bf16* wt = Wp + ((size_t)ltile * k_steps * 64 + lane) * 8;
#pragma unroll
    for (int s = 0; s < GL_KSTEPS; ++s) {
      const int st = step0 + s;
      w[s] = ld16(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  // stage the activations: M rows x group_k, 16 bytes per thread and pass
  const int chunks_per_row = group_k / 8;
  for (int idx = threadIdx.x; idx < M * chunks_per_row; idx += blockDim.x) {
    const int m = idx / chunks_per_row, c = idx - m * chunks_per_row;
    const int k = group_begin * 32 + c * 8;
    const uint4 v = k < K ? load_a(A + (size_t)m * lda, k, K, a_mode) : zero;
    *reinterpret_cast<uint4*>(a_lds + (size_t)m * lds_stride + c * 8) = v;
  }
  __syncthreads();

  while (true) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < GL_KSTEPS; ++s) {
      const uint4 af = (row < M && step0 + s < group_end) ? *reinterpret_cast<const uint4*>(arow + s * 32) : zero;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, af),
                                                    __builtin_bit_cast(bf16x8_t, w[s]), acc, 0, 0, 0);
    }
    // the next tile's weights are requested before this tile's sums are formed
    const int next0 = tile0 + gridDim.x * tpb;
    if (next0 < n_tiles) {
      const int ltile = min(next0 + tw, n_tiles - 1);
      const bf16* wt = Wp + ((size_t)ltile * k_steps * 64 + lane) * 8;
#pragma unroll
      for (int s = 0; s < GL_KSTEPS; ++s) {
        const int st = step0 + s;
        w[s] = ld16(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);
      }
    }
    // acc[r] is C[m = kg*4 + r][n = tile*16 + row]
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < tpb * 256; idx += blockDim.x) {
      const int t2 = idx >> 8, e = idx & 255;
      float sum = 0.f;
      for (int k2 = 0; k2 < kw_count; ++k2) sum += red[(t2 * kw_count + k2) * 256 + e];
      const int r = e >> 6, l2 = e & 63;
      const int m = (l2 >> 4) * 4 + r, nn = (tile0 + t2) * 16 + (l2 & 15);
      if (m < M && nn < N) C[(size_t)m * ldc + nn] = from_float<TC>(sum);
    }
    if (next0 >= n_tiles) break;
    tile0 = next0;
    __syncthreads();
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

extern "C" int blm_gemv_mfma_supported(int M, int N, int K) {
  int ks;
  return (M >= 1 && M <= 16 && N >= 1 && K >= 8 && K % 8 == 0 && plan_k(K, &ks) > 0) ? 1 : 0;
}

template <typename TC>
static int launch_mfma(const void* A, const void* Wp, void* C, int M, int N, int K, int lda, int ldc, int a_mode,
                       int k_groups, hipStream_t stream) {
  const int n_tiles = (N + 15) / 16;
  const int k_steps = (K + 31) / 32;
  const int steps_per_group = (k_steps + k_groups - 1) / k_groups;
  if (a_mode == 1) {
    // The shared-memory variant pays off where the operand load is expensive, i.e. with the fused
    // gating (measured: 18 us against 22 us for the down projection of the 1B shape; without gating
    // the register variant below is faster for every shape).  It needs the group's slice of the
    // activations to fit beside the reduction buffer.
    const int kw_count = (steps_per_group + GL_KSTEPS - 1) / GL_KSTEPS;
    const size_t a_bytes = (((size_t)M * (steps_per_group * 32 + 8) * 2) + 15) & ~(size_t)15;
    if (kw_count <= 16) {
      // as many tiles per block as still leave 256 blocks, and as 16 wavefronts hold
      int tpb = 16 / kw_count;
      if (tpb > 4) tpb = 4;
      while (tpb > 1 && (long long)((n_tiles + tpb - 1) / tpb) * k_groups < 256) --tpb;
      const int waves = tpb * kw_count;
      const size_t smem = a_bytes + (size_t)waves * 256 * sizeof(float);
      if (smem <= 64 * 1024) {
        int blocks = (n_tiles + tpb - 1) / tpb;
        const int cap = waves > 8 ? 256 : 512;
        if (blocks * k_groups > cap) blocks = cap / k_groups > 0 ? cap / k_groups : 1;
        hipLaunchKernelGGL((gemv_mfma_lds_kernel<TC>), dim3(blocks, k_groups), dim3(waves * BLM_WAVE), smem, stream,
                           (const bf16*)A, (const bf16*)Wp, (TC*)C, M, N, K, lda, ldc, n_tiles, k_steps, a_mode,
                           steps_per_group, kw_count, tpb);
        BLM_LAUNCH_CHECK("gemv_mfma_lds");
        return 0;
      }
    }
  }
  int ksteps = 0;
  const int waves = plan_k(steps_per_group * 32, &ksteps);
  // enough blocks to fill the chip, few enough that a block reuses its activations
  int blocks = n_tiles;
  const int cap = (waves > 4 ? 256 : 512) / k_groups;
  if (blocks > cap) blocks = cap > 0 ? cap : 1;
  dim3 grid(blocks, k_groups), block(waves * BLM_WAVE);
  const size_t smem = (size_t)waves * 256 * sizeof(float);
#define BLM_GM(KS, MAXT, KEEP)                                                                                  \
  hipLaunchKernelGGL((gemv_mfma_kernel<KS, MAXT, KEEP, TC>), grid, block, smem, stream, (const bf16*)A,         \
                     (const bf16*)Wp, (TC*)C, M, N, K, lda, ldc, n_tiles, k_steps, a_mode, steps_per_group)
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
// a_mode 0: A is [M, K].  a_mode 1: A is [M, 2K] = [gate | up] and the product runs on silu(gate) * up.
// k_groups > 1: K is cut into that many groups handled by different blocks; C is then float
// [k_groups, M, ldc] and holds one partial product per group, to be summed by the reader (the
// residual add in front of the next norm does it), so narrow outputs still occupy the whole chip.
extern "C" int blm_gemv_mfma(const void* A, const void* Wp, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldc, int a_mode, int k_groups, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= 16, "gemv_mfma: M=%d out of range 1..16", M);
  BLM_REQUIRE(blm_gemv_mfma_supported(M, N, K), "gemv_mfma: sizes N=%d K=%d not supported (K a multiple of 8, at most 16384)", N, K);
  BLM_REQUIRE(a_mode == 0 || a_mode == 1, "gemv_mfma: a_mode %d unknown", a_mode);
  BLM_REQUIRE(k_groups >= 1 && k_groups <= 64 && (k_groups == 1 || c_dtype == BLM_F32),
              "gemv_mfma: k_groups=%d needs 1..64 and a float output when above 1", k_groups);
  BLM_REQUIRE(lda % 8 == 0 && lda >= (a_mode ? 2 * K : K) && ldc >= N, "gemv_mfma: bad strides lda=%d ldc=%d", lda, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)Wp % 16) == 0, "gemv_mfma: operands must be 16-byte aligned");
  if (c_dtype == BLM_BF16) return launch_mfma<bf16>(A, Wp, C, M, N, K, lda, ldc, a_mode, k_groups, stream);
  if (c_dtype == BLM_F32) return launch_mfma<float>(A, Wp, C, M, N, K, lda, ldc, a_mode, k_groups, stream);
  return blm_fail("gemv_mfma: unsupported output dtype %d", c_dtype);
}
