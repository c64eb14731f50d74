// Row-wise kernels: embedding gather, residual add + RMS norm, rotary encoding with the write
// of keys and values into the paged cache, SwiGLU gating.  All arithmetic is in float; inputs
// and outputs are float or bf16.  The residual stream `h` is always float.
#include "common.h"

// ---------------------------------------------------------------------------------------
// embedding: h[t, :] = table[ids[t], :]
// ---------------------------------------------------------------------------------------
template <typename TW>
__global__ void embed_gather_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ h, int D) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const TW* row = table + (size_t)id * D;
  float* out = h + (size_t)t * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) out[d] = to_float(row[d]);
}

extern "C" int blm_embed_gather(const void* table, int table_dtype, const int* ids, float* h,
                                int T, int D, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && D > 0, "embed_gather: bad sizes T=%d D=%d", T, D);
  dim3 grid(T), block(256);
  if (table_dtype == BLM_F32)
    hipLaunchKernelGGL(embed_gather_kernel<float>, grid, block, 0, stream, (const float*)table, ids, h, D);
  else if (table_dtype == BLM_BF16)
    hipLaunchKernelGGL(embed_gather_kernel<bf16>, grid, block, 0, stream, (const bf16*)table, ids, h, D);
  else
    return blm_fail("embed_gather: unsupported table dtype %d", table_dtype);
  BLM_LAUNCH_CHECK("embed_gather");
  return 0;
}

// The same with the token of row t taken on the device where the host does not know it yet:
// id = (*source)[source_rows[t]] if source_rows[t] >= 0, else ids[t].  `source` is a cell in device
// memory that holds the address of an int32 array (what a sampler left), so that a recorded launch
// can read another array at every replay.  An id outside [0, V) gives a row of NaN.
template <typename TW>
__global__ void embed_gather_from_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                                         const int* __restrict__ source_rows, const int* const* __restrict__ source,
                                         float* __restrict__ h, int D, int V) {
  const int t = blockIdx.x;
  const int r = source_rows[t];
  const int id = r >= 0 ? (*source)[r] : ids[t];
  float* out = h + (size_t)t * D;
  if ((unsigned)id >= (unsigned)V) {
    for (int d = threadIdx.x; d < D; d += blockDim.x) out[d] = __builtin_nanf("");
    return;
  }
  const TW* row = table + (size_t)id * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) out[d] = to_float(row[d]);
}

extern "C" int blm_embed_gather_from(const void* table, int table_dtype, const int* ids, const int* source_rows,
                                     const void* source_cell, float* h, int T, int D, int V, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && D > 0 && V > 0, "embed_gather_from: bad sizes T=%d D=%d V=%d", T, D, V);
  BLM_REQUIRE(source_rows && source_cell && ((size_t)source_cell & 7) == 0,
              "embed_gather_from: needs the rows and an 8-byte aligned cell with the tokens' address");
  dim3 grid(T), block(256);
  const int* const* cell = (const int* const*)source_cell;
  if (table_dtype == BLM_F32)
    hipLaunchKernelGGL(embed_gather_from_kernel<float>, grid, block, 0, stream, (const float*)table, ids, source_rows,
                       cell, h, D, V);
  else if (table_dtype == BLM_BF16)
    hipLaunchKernelGGL(embed_gather_from_kernel<bf16>, grid, block, 0, stream, (const bf16*)table, ids, source_rows,
                       cell, h, D, V);
  else
    return blm_fail("embed_gather_from: unsupported table dtype %d", table_dtype);
  BLM_LAUNCH_CHECK("embed_gather_from");
  return 0;
}

// ---------------------------------------------------------------------------------------
// residual add + RMS norm
//   v = h[r] (+ sum over planes p of delta[p][r]);  if write_h: h[r] = v;
//   out[i] = v / sqrt(mean(v^2) + eps) * gamma;     r = rows ? rows[i] : i
//   delta: n_planes planes of [T, D], in the activation dtype or float (partial products of a
//   matrix product whose K was cut over blocks; summed here in plane order).
// ---------------------------------------------------------------------------------------
template <typename TA, typename TG, typename TD>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_planes,
                                   size_t plane_stride, const TG* __restrict__ gamma, TA* __restrict__ out,
                                   const int* __restrict__ rows, int D, float eps, int write_h) {
  __shared__ float red[17];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* hr = h + (size_t)r * D;
  const TD* dr = delta ? delta + (size_t)r * D : nullptr;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = hr[d];
    if (dr) {
      for (int p = 0; p < n_planes; ++p) v += to_float(dr[p * plane_stride + d]);
      if (write_h) hr[d] = v;
    }
    ss += v * v;
  }
  ss = block_sum<true>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  TA* o = out + (size_t)i * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = hr[d];
    if (dr && !write_h)
      for (int p = 0; p < n_planes; ++p) v += to_float(dr[p * plane_stride + d]);
    o[d] = from_float<TA>(v * inv * to_float(gamma[d]));
  }
}

// Fast form for rows that fit the block's registers (D a multiple of 4, at most 4 * 512 * ITERS):
// every load of a row is issued at once with 16-byte accesses, and the normalised row is written
// from registers instead of being read again.
template <typename T>
__device__ __forceinline__ void load4(const T* p, float* v);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float* v) {
  const float4 r = *reinterpret_cast<const float4*>(p);
  v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
}
template <>
__device__ __forceinline__ void load4<bf16>(const bf16* p, float* v) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
  v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
}
// four elements as they lie in memory, and their values
template <typename T>
struct Raw4;
template <>
struct Raw4<float> { typedef float4 type; };
template <>
struct Raw4<bf16> { typedef uint2 type; };
__device__ __forceinline__ void unpack4(float4 r, float* v) { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
__device__ __forceinline__ void unpack4(uint2 r, float* v) {
  v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
  v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
}
template <typename T>
__device__ __forceinline__ void store4(T* p, const float* v);
template <>
__device__ __forceinline__ void store4<float>(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* p, const float* v) {
  uint2 r;
  r.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  r.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = r;
}

template <typename TA, typename TG, typename TD, int ITERS>
__global__ void __launch_bounds__(512)
    add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_planes, size_t plane_stride,
                           const TG* __restrict__ gamma, TA* __restrict__ out, const int* __restrict__ rows, int D,
                           float eps, int write_h) {
  __shared__ float red[17];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* hr = h + (size_t)r * D;
  const TD* dr = delta ? delta + (size_t)r * D : nullptr;
  // The norm's weights are asked for first of all, with the row and its planes, and not behind the
  // barrier: a second trip to memory in a row, where the kernel is nothing but latencies (a decode
  // step's eight rows).  They are unpacked where the row's sum is complete, that is where everything
  // asked for has arrived anyway: behind the barrier a wait for them would also wait for the store of
  // the summed row (stores count with the loads).
  typename Raw4<TG>::type graw[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int d = (it * blockDim.x + threadIdx.x) * 4;
    if (d < D) graw[it] = *reinterpret_cast<const typename Raw4<TG>::type*>(gamma + d);
  }
  float v[ITERS][4];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int d = (it * blockDim.x + threadIdx.x) * 4;
    if (d < D) {
      load4<float>(hr + d, v[it]);
      if (dr) {
        // four planes at a time: their loads are issued together (a loop that loads and adds plane
        // by plane waits for memory once per plane), the adds keep the planes' order
        if (n_planes == 1) {   // the usual case with many rows: one load, not four of the same plane
          float t[4];
          load4<TD>(dr + d, t);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[it][e] += t[e];
        } else {
          // the first four on their own, so that their loads are asked for before the row of h is
          // first used (as the loop's entry it would be waited for in front of the loop: two trips
          // to memory in a row instead of one)
          float t[4][4];
#pragma unroll
          for (int q = 0; q < 4; ++q) load4<TD>(dr + (size_t)min(q, n_planes - 1) * plane_stride + d, t[q]);
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (q < n_planes) {
#pragma unroll
              for (int e = 0; e < 4; ++e) v[it][e] += t[q][e];
            }
          for (int p0 = 4; p0 < n_planes; p0 += 4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) load4<TD>(dr + (size_t)min(p0 + q, n_planes - 1) * plane_stride + d, t[q]);
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (p0 + q < n_planes) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[it][e] += t[q][e];
              }
          }
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += v[it][e] * v[it][e];
    }
  }
  float g[ITERS][4];
#pragma unroll
  for (int it = 0; it < ITERS; ++it)
    if ((it * blockDim.x + threadIdx.x) * 4 < D) {
      unpack4(graw[it], g[it]);
      // a use that cannot move: the unpacking stays in front of the reduction
      asm volatile("" : "+v"(g[it][0]), "+v"(g[it][1]), "+v"(g[it][2]), "+v"(g[it][3]));
    }
  ss = block_sum<true>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  TA* o = out + (size_t)i * D;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int d = (it * blockDim.x + threadIdx.x) * 4;
    if (d < D) {
      if (dr && write_h) store4<float>(hr + d, v[it]);
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = v[it][e] * inv * g[it][e];
      store4<TA>(o + d, y);
    }
  }
}

template <typename TA, typename TG>
static int launch_norm(float* h, const void* delta, int delta_dtype, int n_planes, size_t plane_stride,
                       const void* gamma, void* out, const int* rows, int n_out, int D, float eps, int write_h,
                       hipStream_t stream) {
  dim3 grid(n_out), block(D >= 2048 ? 512 : 256);
  const bool aligned = D % 4 == 0 && plane_stride % 4 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                       ((uintptr_t)gamma % 16) == 0 && ((uintptr_t)delta % 16) == 0;
  if (aligned && D <= 4 * (int)block.x * 4) {
    const int iters = (D + 4 * (int)block.x - 1) / (4 * (int)block.x);
#define BLM_NV(TD, IT)                                                                                             \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TA, TG, TD, IT>), grid, block, 0, stream, h, (const TD*)delta, n_planes, \
                     plane_stride, (const TG*)gamma, (TA*)out, rows, D, eps, write_h)
    if (delta_dtype == BLM_F32) {
      if (iters == 1) BLM_NV(float, 1); else if (iters == 2) BLM_NV(float, 2); else BLM_NV(float, 4);
    } else {
      if (iters == 1) BLM_NV(bf16, 1); else if (iters == 2) BLM_NV(bf16, 2); else BLM_NV(bf16, 4);
    }
#undef BLM_NV
    BLM_LAUNCH_CHECK("add_rmsnorm_vec");
    return 0;
  }
  if (delta_dtype == BLM_F32)
    hipLaunchKernelGGL((add_rmsnorm_kernel<TA, TG, float>), grid, block, 0, stream, h, (const float*)delta, n_planes,
                       plane_stride, (const TG*)gamma, (TA*)out, rows, D, eps, write_h);
  else
    hipLaunchKernelGGL((add_rmsnorm_kernel<TA, TG, bf16>), grid, block, 0, stream, h, (const bf16*)delta, n_planes,
                       plane_stride, (const TG*)gamma, (TA*)out, rows, D, eps, write_h);
  BLM_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

extern "C" int blm_add_rmsnorm(float* h, const void* delta, int delta_dtype, int n_planes, long long plane_stride,
                               const void* gamma, int gamma_dtype, void* out, int act_dtype, const int* rows,
                               int n_out, int D, float eps, int write_h, hipStream_t stream) {
  BLM_REQUIRE(n_out > 0 && D > 0, "add_rmsnorm: bad sizes n=%d D=%d", n_out, D);
  BLM_REQUIRE(delta == nullptr || (n_planes >= 1 && n_planes <= 64 && plane_stride >= 0),
              "add_rmsnorm: bad planes %d", n_planes);
  BLM_REQUIRE(delta == nullptr || delta_dtype == BLM_F32 || delta_dtype == BLM_BF16, "add_rmsnorm: delta dtype %d", delta_dtype);
  if (act_dtype == BLM_F32 && gamma_dtype == BLM_F32)
    return launch_norm<float, float>(h, delta, delta_dtype, n_planes, plane_stride, gamma, out, rows, n_out, D, eps, write_h, stream);
  if (act_dtype == BLM_BF16 && gamma_dtype == BLM_BF16)
    return launch_norm<bf16, bf16>(h, delta, delta_dtype, n_planes, plane_stride, gamma, out, rows, n_out, D, eps, write_h, stream);
  if (act_dtype == BLM_BF16 && gamma_dtype == BLM_F32)
    return launch_norm<bf16, float>(h, delta, delta_dtype, n_planes, plane_stride, gamma, out, rows, n_out, D, eps, write_h, stream);
  if (act_dtype == BLM_F32 && gamma_dtype == BLM_BF16)
    return launch_norm<float, bf16>(h, delta, delta_dtype, n_planes, plane_stride, gamma, out, rows, n_out, D, eps, write_h, stream);
  return blm_fail("add_rmsnorm: unsupported dtypes act=%d gamma=%d", act_dtype, gamma_dtype);
}

// ---------------------------------------------------------------------------------------
// rotary encoding of q (in place) and k, and the write of k, v into the paged cache
//   qkv row layout: [q: nh*hd | k: nkv*hd | v: nkv*hd]
//   key plane layout:   [page][kv head][slot in page][hd]
//   value plane layout: [page][kv head][hd][slot in page]   (transposed, so that the matrix-core
//                        attention kernels find the keys of a page contiguous for every lane)
//   pairing 0: lanes (2i, 2i+1) form a pair; pairing 1: lanes (i, i + hd/2)
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void rope_kv_write_kernel(TA* __restrict__ qkv, const int* __restrict__ positions,
                                     const int* __restrict__ token_seq,
                                     const int* __restrict__ block_table, int table_width,
                                     const float2* __restrict__ cos_sin, TA* __restrict__ kcache,
                                     TA* __restrict__ vcache, int page_size, int nh, int nkv,
                                     int hd, int pairing, int write_kv) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  if (b < 0) return;  // padding token
  const int pos = positions[t];
  const int half = hd >> 1;
  TA* row = qkv + (size_t)t * (size_t)(nh + 2 * nkv) * hd;
  const float2* cs = cos_sin + (size_t)pos * half;
  const int page = block_table[(size_t)b * table_width + pos / page_size];
  const int slot = pos % page_size;
  const bool store = write_kv && page >= 0;

  // rotations: heads 0..nh-1 are queries, nh..nh+nkv-1 keys
  const int n_rot = (nh + nkv) * half;
  for (int w = threadIdx.x; w < n_rot; w += blockDim.x) {
    const int head = w / half, i = w - head * half;
    const int i0 = pairing == 0 ? 2 * i : i;
    const int i1 = pairing == 0 ? 2 * i + 1 : i + half;
    TA* x = row + (size_t)head * hd;
    const float x0 = to_float(x[i0]), x1 = to_float(x[i1]);
    const float2 c = cs[i];
    const TA y0 = from_float<TA>(x0 * c.x - x1 * c.y);
    const TA y1 = from_float<TA>(x0 * c.y + x1 * c.x);
    if (head < nh) {
      x[i0] = y0;
      x[i1] = y1;
    } else if (store) {
      TA* kd = kcache + (((size_t)page * nkv + (head - nh)) * page_size + slot) * hd;
      kd[i0] = y0;
      kd[i1] = y1;
    }
  }
  if (store) {
    const TA* v = row + (size_t)(nh + nkv) * hd;
    for (int w = threadIdx.x; w < nkv * hd; w += blockDim.x) {
      const int head = w / hd, d = w - head * hd;
      vcache[(((size_t)page * nkv + head) * hd + d) * page_size + slot] = v[w];
    }
  }
}

// bf16, head_dim a multiple of 16.  Blocks 0 .. T-1 rotate one token each, eight lanes per thread
// with 16-byte accesses (pairing 1: lanes i..i+7 with i+half..i+half+7; pairing 0: eight neighbouring
// lanes = four pairs).  The blocks after them copy the values: a block takes 16 consecutive tokens of
// one key-value head, reads their rows coalesced into shared memory and writes them transposed, 16
// lanes to the 16 tokens of one head lane, which are neighbours in the page when the tokens are
// neighbours in a sequence (the usual case in a prompt), so that a row of the page is written in
// pieces of 32 bytes and not of 2.
__global__ void __launch_bounds__(256)
    rope_kv_write_vec_kernel(bf16* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ token_seq,
                             const int* __restrict__ block_table, int table_width, const float2* __restrict__ cos_sin,
                             bf16* __restrict__ kcache, bf16* __restrict__ vcache, int page_size, int T, int nh,
                             int nkv, int hd, int pairing, int write_kv) {
  if ((int)blockIdx.x >= T) {   // a tile of values: 16 tokens of one key-value head
    extern __shared__ bf16 vt[];   // [16][hd + 2]
    const int tile = blockIdx.x - T;
    const int head = tile % nkv, t0 = (tile / nkv) * 16;
    const int vstr = hd + 2;
    const size_t row_len = (size_t)(nh + 2 * nkv) * hd;
    for (int e = threadIdx.x; e < 16 * hd / 2; e += blockDim.x) {   // two lanes (4 bytes) per access
      const int j = e / (hd / 2), d2 = e - j * (hd / 2);
      if (t0 + j < T)
        *reinterpret_cast<uint32_t*>(vt + j * vstr + 2 * d2) =
            *reinterpret_cast<const uint32_t*>(qkv + (size_t)(t0 + j) * row_len + (size_t)(nh + nkv + head) * hd + 2 * d2);
    }
    __syncthreads();
    const int j = threadIdx.x & 15;
    if (t0 + j >= T) return;
    const int bj = token_seq[t0 + j];
    if (bj < 0) return;
    const int pj = positions[t0 + j];
    const int pg = block_table[(size_t)bj * table_width + pj / page_size];
    if (pg < 0) return;
    bf16* dst = vcache + ((size_t)pg * nkv + head) * hd * page_size + pj % page_size;
    for (int d = threadIdx.x >> 4; d < hd; d += blockDim.x >> 4) dst[(size_t)d * page_size] = vt[j * vstr + d];
    return;
  }
  const int t = blockIdx.x;
  const int b = token_seq[t];
  if (b < 0) return;  // padding token
  const int pos = positions[t];
  const int half = hd >> 1;
  bf16* row = qkv + (size_t)t * (size_t)(nh + 2 * nkv) * hd;
  const float2* cs = cos_sin + (size_t)pos * half;
  const int page = block_table[(size_t)b * table_width + pos / page_size];
  const int slot = pos % page_size;
  const bool store = write_kv && page >= 0;
  const int per_head = pairing == 1 ? half / 8 : hd / 8;   // threads per head
  const int n_units = (nh + nkv) * per_head;
  for (int w = threadIdx.x; w < n_units; w += blockDim.x) {
    const int head = w / per_head, u = w - head * per_head;
    if (head >= nh && !store) continue;
    bf16* x = row + (size_t)head * hd;
    bf16* dst = head < nh ? x : kcache + (((size_t)page * nkv + (head - nh)) * page_size + slot) * hd;
    if (pairing == 1) {
      const int i = u * 8;
      const uint4 a = *reinterpret_cast<const uint4*>(x + i), c = *reinterpret_cast<const uint4*>(x + i + half);
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, cw[4] = {c.x, c.y, c.z, c.w};
      uint32_t o0[4], o1[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float4 f = *reinterpret_cast<const float4*>(cs + i + 2 * k);   // (cos, sin) of two pairs
        const float x0a = __uint_as_float(aw[k] << 16), x0b = __uint_as_float(aw[k] & 0xffff0000u);
        const float x1a = __uint_as_float(cw[k] << 16), x1b = __uint_as_float(cw[k] & 0xffff0000u);
        o0[k] = f32x2_to_bf16x2_bits(x0a * f.x - x1a * f.y, x0b * f.z - x1b * f.w);
        o1[k] = f32x2_to_bf16x2_bits(x0a * f.y + x1a * f.x, x0b * f.w + x1b * f.z);
      }
      *reinterpret_cast<uint4*>(dst + i) = make_uint4(o0[0], o0[1], o0[2], o0[3]);
      *reinterpret_cast<uint4*>(dst + i + half) = make_uint4(o1[0], o1[1], o1[2], o1[3]);
    } else {
      const int i = u * 8;   // lanes i .. i+7 = pairs i/2 .. i/2+3
      const uint4 a = *reinterpret_cast<const uint4*>(x + i);
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
      uint32_t o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float2 f = cs[i / 2 + k];
        const float x0 = __uint_as_float(aw[k] << 16), x1 = __uint_as_float(aw[k] & 0xffff0000u);
        o[k] = f32x2_to_bf16x2_bits(x0 * f.x - x1 * f.y, x0 * f.y + x1 * f.x);
      }
      *reinterpret_cast<uint4*>(dst + i) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

extern "C" int blm_rope_kv_write(void* qkv, int act_dtype, const int* positions,
                                 const int* token_seq, const int* block_table, int table_width,
                                 const float* cos_sin, void* kcache, void* vcache, int page_size,
                                 int T, int nh, int nkv, int hd, int pairing, int write_kv,
                                 hipStream_t stream) {
  BLM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && hd > 0 && (hd % 2) == 0,
              "rope_kv_write: bad sizes T=%d nh=%d nkv=%d head_dim=%d (head_dim must be even)", T, nh, nkv, hd);
  BLM_REQUIRE(page_size > 0 && table_width > 0, "rope_kv_write: bad cache geometry");
  BLM_REQUIRE(pairing == 0 || pairing == 1, "rope_kv_write: pairing %d unknown", pairing);
  dim3 grid(T), block(256);
  if (act_dtype == BLM_BF16 && hd % 16 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)kcache % 16) == 0 &&
      ((uintptr_t)cos_sin % 16) == 0) {
    const long long v_tiles = write_kv ? (long long)((T + 15) / 16) * nkv : 0;
    BLM_REQUIRE(T + v_tiles < 2147483647LL, "rope_kv_write: too many tokens");
    hipLaunchKernelGGL(rope_kv_write_vec_kernel, dim3((unsigned)(T + v_tiles)), block, (size_t)16 * (hd + 2) * sizeof(bf16),
                       stream, (bf16*)qkv, positions, token_seq, block_table, table_width, (const float2*)cos_sin,
                       (bf16*)kcache, (bf16*)vcache, page_size, T, nh, nkv, hd, pairing, write_kv);
    BLM_LAUNCH_CHECK("rope_kv_write_vec");
    return 0;
  }
  if (act_dtype == BLM_F32)
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, grid, block, 0, stream, (float*)qkv, positions, token_seq,
                       block_table, table_width, (const float2*)cos_sin, (float*)kcache, (float*)vcache,
                       page_size, nh, nkv, hd, pairing, write_kv);
  else if (act_dtype == BLM_BF16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16>, grid, block, 0, stream, (bf16*)qkv, positions, token_seq,
                       block_table, table_width, (const float2*)cos_sin, (bf16*)kcache, (bf16*)vcache,
                       page_size, nh, nkv, hd, pairing, write_kv);
  else
    return blm_fail("rope_kv_write: unsupported dtype %d", act_dtype);
  BLM_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ---------------------------------------------------------------------------------------
// SwiGLU gating: out[t, i] = silu(gu[t, i]) * gu[t, I + i]
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void swiglu_kernel(const TA* __restrict__ gu, TA* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const TA* g = gu + (size_t)t * 2 * I;
  TA* o = out + (size_t)t * I;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < I; i += gridDim.x * blockDim.x) {
    const float z = to_float(g[i]), u = to_float(g[I + i]);
    o[i] = from_float<TA>(z / (1.0f + expf(-z)) * u);
  }
}

// 8 elements per thread with 16-byte accesses (bf16, I a multiple of 8)
__global__ void swiglu_vec_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int I, long long total8) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const int per_row = I / 8;
  const long long t = idx / per_row;
  const int c = (int)(idx - t * per_row) * 8;
  const bf16* g = gu + t * 2 * I + c;
  const uint4 gv = *reinterpret_cast<const uint4*>(g);
  const uint4 uv = *reinterpret_cast<const uint4*>(g + I);
  const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    const float f0 = g0 / (1.0f + expf(-g0)) * u0, f1 = g1 / (1.0f + expf(-g1)) * u1;
    o[i] = (uint32_t)f32_to_bf16_bits(f0) | ((uint32_t)f32_to_bf16_bits(f1) << 16);
  }
  *reinterpret_cast<uint4*>(out + t * I + c) = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int blm_swiglu(const void* gu, void* out, int act_dtype, int T, int I, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && I > 0 && T <= 65535 * 64, "swiglu: bad sizes T=%d I=%d", T, I);
  if (act_dtype == BLM_BF16 && I % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const long long total8 = (long long)T * (I / 8);
    const long long blocks = (total8 + 255) / 256;
    BLM_REQUIRE(blocks < 2147483647LL, "swiglu: too many elements");
    hipLaunchKernelGGL(swiglu_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const bf16*)gu, (bf16*)out, I, total8);
    BLM_LAUNCH_CHECK("swiglu_vec");
    return 0;
  }
  int gx = (I + 255) / 256;
  if (gx > 64) gx = 64;
  for (int t0 = 0; t0 < T; t0 += 65535) {
    int tn = T - t0 < 65535 ? T - t0 : 65535;
    dim3 grid(gx, tn), block(256);
    if (act_dtype == BLM_F32)
      hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream, (const float*)gu + (size_t)t0 * 2 * I,
                         (float*)out + (size_t)t0 * I, I);
    else if (act_dtype == BLM_BF16)
      hipLaunchKernelGGL(swiglu_kernel<bf16>, grid, block, 0, stream, (const bf16*)gu + (size_t)t0 * 2 * I,
                         (bf16*)out + (size_t)t0 * I, I);
    else
      return blm_fail("swiglu: unsupported dtype %d", act_dtype);
  }
  BLM_LAUNCH_CHECK("swiglu");
  return 0;
}
