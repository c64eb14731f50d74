// Shared device helpers for the gfx950 kernels: storage types, conversions, reductions.
// Every kernel is a template over the storage type (float or bf16) and computes in float.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define BLM_WAVE 64

struct bf16 {
  uint16_t v;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) { return __uint_as_float(((uint32_t)x.v) << 16); }

// round to nearest even; NaN stays NaN (the hardware conversion of gfx950)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

// two floats to a pair of bf16 in one register (lo in the low half), one instruction
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float blm_f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 blm_bf16x2;
  const blm_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, blm_bf16x2));
}

// 16 bytes of a stream that is read once and whole cache lines at a time (packed weights): a load
// that does not displace what the caches hold.  Not for fragments that take 16 bytes of a line
// per instruction (a decode step's key pages): those need the line to stay (measured: 15 % slower).
__device__ __forceinline__ uint4 load16_stream(const void* p) {
  typedef __attribute__((ext_vector_type(4))) unsigned int v4;
  const v4 v = __builtin_nontemporal_load(reinterpret_cast<const v4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) { return f; }
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float f) { return bf16{f32_to_bf16_bits(f)}; }

// Maximum without the copies that quiet signalling NaNs in front of fmaxf (one instruction per operand
// that comes out of a matrix instruction or a load); a NaN operand gives NaN.  Chains of it become
// three-operand instructions.
__device__ __forceinline__ float blm_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// Exchanges across a wavefront without a trip through shared memory.  Inside a row of 16 lanes a
// data-parallel move brings the partner's value; between rows the swap instructions of gfx950 do:
// after blm_swap16(x, a, b), rows 0 and 1 hold a = row 0 of x, b = row 1 of x, rows 2 and 3 hold rows 2
// and 3; after blm_swap32, lanes l and l + 32 both hold a = x of lane l % 32, b = x of lane l % 32 + 32.
// Both partners get the same (a, b), so a + b or max(a, b) has the same bits in both.
template <int CTRL>
__device__ __forceinline__ float blm_dpp(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, 0xf, 0xf, false));
}
#define BLM_DPP_XOR1 0xB1          // quad_perm [1, 0, 3, 2]
#define BLM_DPP_XOR2 0x4E          // quad_perm [2, 3, 0, 1]
#define BLM_DPP_HALF_MIRROR 0x141  // lane i of each 8 takes lane 7 - i: the other quad, once quads are uniform
#define BLM_DPP_MIRROR 0x140       // lane i of each 16 takes lane 15 - i: the other half, once halves are uniform
__device__ __forceinline__ void blm_swap16(float x, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void blm_swap32(float x, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
// over the four lanes l % 16, l % 16 + 16, + 32, + 48
__device__ __forceinline__ float rows_max(float v) {
  float a, b;
  blm_swap16(v, a, b);
  v = blm_max(a, b);
  blm_swap32(v, a, b);
  return blm_max(a, b);
}
__device__ __forceinline__ float rows_sum(float v) {
  float a, b;
  blm_swap16(v, a, b);
  v = a + b;
  blm_swap32(v, a, b);
  return a + b;
}

// Sum and maximum over a whole wavefront (all 64 lanes active); every lane gets the same bits.
__device__ __forceinline__ float wave_sum(float v) {
  v += blm_dpp<BLM_DPP_XOR1>(v);
  v += blm_dpp<BLM_DPP_XOR2>(v);
  v += blm_dpp<BLM_DPP_HALF_MIRROR>(v);
  v += blm_dpp<BLM_DPP_MIRROR>(v);
  return rows_sum(v);
}
__device__ __forceinline__ float wave_max(float v) {
  v = blm_max(v, blm_dpp<BLM_DPP_XOR1>(v));
  v = blm_max(v, blm_dpp<BLM_DPP_XOR2>(v));
  v = blm_max(v, blm_dpp<BLM_DPP_HALF_MIRROR>(v));
  v = blm_max(v, blm_dpp<BLM_DPP_MIRROR>(v));
  return rows_max(v);
}

// Sum over a block of up to 1024 threads (whole wavefronts); every thread gets the result, the
// wavefronts' sums added in the order of the wavefronts.  `red` holds 16 floats.  FRESH: `red` has
// not been used in this kernel before, so nobody can still be reading it.
template <bool FRESH = false>
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (BLM_WAVE - 1), w = threadIdx.x / BLM_WAVE;
  const int nw = (blockDim.x + BLM_WAVE - 1) / BLM_WAVE;
  v = wave_sum(v);
  if (nw == 1) return v;
  if (!FRESH) __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
  for (int k = 1; k < nw; ++k) t += red[k];
  return t;
}
template <bool FRESH = false>
__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x & (BLM_WAVE - 1), w = threadIdx.x / BLM_WAVE;
  const int nw = (blockDim.x + BLM_WAVE - 1) / BLM_WAVE;
  v = wave_max(v);
  if (nw == 1) return v;
  if (!FRESH) __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
  for (int k = 1; k < nw; ++k) t = blm_max(t, red[k]);
  return t;
}

// One direct load of 16 bytes per lane from global memory into shared memory at lds (the same in all
// lanes) + 16 * lane: from a base that is the same in all lanes plus a byte offset per lane, or from a
// full address per lane.  Written as assembly: when the compiler knows of such a load it waits for
// every outstanding one (vmcnt(0)) in front of the next read of shared memory, whatever address that
// read has, so a ring of several stages would never have more than one in flight; with these, the
// waits are the kernel's own (loads complete in order).  m0 holds the address in shared memory and is
// declared as clobbered, so the compiler keeps nothing of its own there across the statement.
typedef __attribute__((address_space(3))) void* blm_lds_ptr;
__device__ __forceinline__ void blm_dma16(const char* base, uint32_t lane_offset, const void* lds) {
  const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(blm_lds_ptr)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_offset), "s"(base) : "memory", "m0");
}
// the same with the address in shared memory given as the number it is (no cast of a generic pointer)
__device__ __forceinline__ void blm_dma16_to(const char* base, uint32_t lane_offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_offset), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void blm_dma16_lanes(const char* address, const void* lds) {
  const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(blm_lds_ptr)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(address) : "memory", "m0");
}

// Error reporting shared by the host entry points (defined in api.hip).
int blm_fail(const char* fmt, ...);
#define BLM_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) return blm_fail(__VA_ARGS__); \
  } while (0)
#define BLM_LAUNCH_CHECK(name)                                                        \
  do {                                                                                \
    hipError_t e__ = hipGetLastError();                                               \
    if (e__ != hipSuccess) return blm_fail("%s: launch failed: %s", name, hipGetErrorString(e__)); \
  } while (0)

// dtype codes of the C ABI
#define BLM_F32 0
#define BLM_BF16 1
