// Two measuring kernels for the benchmark: what this machine reaches when a kernel only reads memory,
// and when it only issues matrix instructions.  The benchmark quotes its rates against the published
// peaks and against these.
//   probe_read : every block streams its own contiguous piece of a buffer with 16-byte loads, eight in
//                flight per lane, and keeps an exclusive-or of what it read (stored only if it equals a
//                value it cannot have, so the loads are not optimised away and nothing is written).
//   probe_mfma : every wavefront issues `iters` rounds of four independent 32x32x16 bf16 matrix
//                instructions on registers (4 * 32768 multiply-adds per round per wavefront), either on
//                the same few small values every time, or on random operands that change with every
//                instruction: the rate differs, since the clock follows the power the multipliers
//                draw (measured: 2.2 against 1.8 PFLOP/s), and a product of real data is the second case.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 pb_bf16x8;
typedef __attribute__((ext_vector_type(16))) float pb_f32x16;

__global__ void __launch_bounds__(256) probe_read_kernel(const uint4* __restrict__ x, size_t n16, unsigned* __restrict__ sink) {
  unsigned acc = 0;
  const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t b = (size_t)blockIdx.x * per, e = b + per < n16 ? b + per : n16;
  size_t i = b + threadIdx.x;
  for (; i + 7 * 256 < e; i += 8 * 256) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = x[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < e; i += 256) {
    const uint4 v = x[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x12345678u) sink[0] = acc;
}

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

template <bool RANDOM>
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iters, float* __restrict__ sink) {
  pb_bf16x8 a[4], b[4];
#pragma unroll
  for (int f = 0; f < 4; ++f)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (RANDOM) {
        // uniform in [-2, 2) and in [-0.04, 0.04): activations and weights of a layer, roughly
        const unsigned h = probe_hash(threadIdx.x * 64 + f * 8 + i + blockIdx.x * 7919u), g = probe_hash(h + 1);
        a[f][i] = (__bf16)(((int)(h & 0xffff) - 32768) / 16384.0f);
        b[f][i] = (__bf16)(((int)(g & 0xffff) - 32768) / 16384.0f * 0.02f);
      } else {
        a[f][i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 7));
        b[f][i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
      }
    }
  pb_f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  for (int it = 0; it < iters; it += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[u], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 1) & 3], b[u], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 2) & 3], b[(u + 1) & 3], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 3) & 3], b[(u + 2) & 3], c3, 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 123.456f) sink[0] = s;
}

// Reads `bytes` (a multiple of 16) from x with `blocks` blocks; writes nothing unless the data is a rare one.
extern "C" int blm_probe_read(const void* x, long long bytes, void* sink, int blocks, hipStream_t stream) {
  BLM_REQUIRE(x != nullptr && sink != nullptr && bytes >= 16 && bytes % 16 == 0 && blocks >= 1 && blocks <= 65535,
              "probe_read: bad arguments (bytes=%lld blocks=%d)", bytes, blocks);
  BLM_REQUIRE(((uintptr_t)x % 16) == 0, "probe_read: the buffer must be 16-byte aligned");
  hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(256), 0, stream, (const uint4*)x, (size_t)(bytes / 16), (unsigned*)sink);
  BLM_LAUNCH_CHECK("probe_read");
  return 0;
}

// blocks x 4 wavefronts, `iters` rounds (a multiple of 4) each: flops = blocks * 4 * iters * 4 * 2 * 32 * 32 * 16.
// random_operands: operands that differ from instruction to instruction instead of the same small values.
extern "C" int blm_probe_mfma(int iters, int blocks, int random_operands, void* sink, hipStream_t stream) {
  BLM_REQUIRE(sink != nullptr && iters >= 4 && iters % 4 == 0 && blocks >= 1 && blocks <= 65535,
              "probe_mfma: bad arguments (iters=%d, a multiple of 4; blocks=%d)", iters, blocks);
  if (random_operands) hipLaunchKernelGGL(probe_mfma_kernel<true>, dim3(blocks), dim3(256), 0, stream, iters, (float*)sink);
  else hipLaunchKernelGGL(probe_mfma_kernel<false>, dim3(blocks), dim3(256), 0, stream, iters, (float*)sink);
  BLM_LAUNCH_CHECK("probe_mfma");
  return 0;
}
