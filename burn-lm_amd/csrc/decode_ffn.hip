// The feed-forward half of a decode layer as ONE kernel whose blocks stay on their compute units:
//     h += delta;  x = rmsnorm(h) * gamma;  act = silu(x Wg^T) * (x Wu^T);  out[g] = partial act Wd^T
// for up to 16 rows (a decode step's sequences), bfloat16 weights packed for the matrix cores (see
// gemv_mfma.hip), float residual stream.  As three kernels (norm, gate/up product, down product) a
// layer's half costs their memory time plus three times a launch, a first-load latency and a
// drain; here the three stages are phases of one grid of at most one block per compute unit:
//
//   phase 1  every block forms the normalised rows itself, in shared memory (one wavefront per row,
//            so no block-wide reduction), and, right behind the loads of the rows, requests its
//            first tiles of the gate/up weights: they do not depend on the activations and travel
//            while the norm is computed.  Wavefronts without a row request their weights at once.
//   phase 2  gate/up product on the block's run of column tiles (K split over the wavefronts, the
//            activations from shared memory), SwiGLU gating in float; the block's gated values are
//            gathered in shared memory.  Wavefront 0 writes them out with stores that reach
//            device-coherent memory, waits for those stores, and counts the block in at the grid's
//            arrival counter; the other wavefronts have requested their share of the block's first
//            down-projection weights meanwhile and wait at the block's barrier with those loads in
//            flight (the counter of outstanding memory operations is a wavefront's own).
//   phase 3  when all blocks have arrived: down product on (column tile, K-group) items, the gated
//            values read with loads that come from device-coherent memory, the partial products
//            written as float planes that the next norm sums.  One wavefront of each block also
//            writes h + delta back for a share of the rows (only now: nobody reads the old h any more).
//
// Every block waits for all the others, so all blocks must be resident together: the grid is at most
// the number of compute units and a block asks for more than half a unit's shared memory, so two never
// share one.  The wait is bounded: a block that has polled `spin_limit` times without seeing the grid
// complete sets a word in host-visible memory and goes on (its results are then wrong, and the host
// raises an error at its next look at the word); no wave ever waits without end.  The two counters
// return to zero by themselves: the block that leaves last resets them.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define DF_WAVES 8
#define DF_THREADS (DF_WAVES * BLM_WAVE)
#define DF_PAD 8   // bf16 elements of padding per row of the activations in shared memory (16 bytes)

struct DecodeFfnArgs {
  float* h;                 // [M, D] residual stream, updated in place
  const void* delta;        // float planes [n_planes, M, D] or bf16 [M, D] (n_planes 1), or null
  int delta_is_bf16, n_planes;
  long long plane_stride;   // elements between planes
  const void* gamma;        // [D]
  int gamma_is_bf16;
  float eps;
  const bf16* w_gu;         // packed, gated pairs: [2 I, D]
  const bf16* w_down;       // packed: [D, I]
  unsigned* act;            // [M, I] bf16 as 32-bit pairs: scratch between the phases
  float* out;               // [k_groups, M, D] partial products of the down projection
  int M, D, I, k_groups;
  int* sync;                // [0] arrivals, [1] departures; zero between launches
  int* fault;               // host-visible; set to 1 if a wait gave up
  int spin_limit;
};

__device__ __forceinline__ uint4 df_stream16(const bf16* p) { return load16_stream(p); }

__device__ __forceinline__ void df_store_coherent(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long df_load_coherent(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float4 df_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 df_load4(const bf16* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                     __uint_as_float(r.y & 0xffff0000u));
}

// h[row] + delta planes at 4 columns from c, planes added in their order
template <typename TD>
__device__ __forceinline__ float4 df_row_sum4(const DecodeFfnArgs& a, int row, int c) {
  float4 v = df_load4(a.h + (size_t)row * a.D + c);
  if (a.delta) {
    const TD* d = reinterpret_cast<const TD*>(a.delta) + (size_t)row * a.D + c;
    for (int p = 0; p < a.n_planes; ++p) {
      const float4 t = df_load4(d + (size_t)p * a.plane_stride);
      v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
  }
  return v;
}

// One wavefront forms one normalised row in shared memory.  KCH: 256-column chunks a row may have.
// The planes are fetched PB at a time (all loads of a batch issued together) and added in order.
template <int KCH, int PB, typename TD>
__device__ __forceinline__ void df_norm_row(const DecodeFfnArgs& a, int row, bf16* xrow, int lane) {
  const int D = a.D;
  float4 v[KCH];
#pragma unroll
  for (int j = 0; j < KCH; ++j) {
    const int c = j * 256 + lane * 4;
    v[j] = c < D ? df_load4(a.h + (size_t)row * D + c) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if (a.delta) {
    const TD* d = reinterpret_cast<const TD*>(a.delta) + (size_t)row * D;
    for (int p0 = 0; p0 < a.n_planes; p0 += PB) {
      float4 t[PB][KCH];
#pragma unroll
      for (int q = 0; q < PB; ++q)
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
          const int c = j * 256 + lane * 4;
          const int p = p0 + q < a.n_planes ? p0 + q : a.n_planes - 1;
          t[q][j] = c < D ? df_load4(d + (size_t)p * a.plane_stride + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
      for (int q = 0; q < PB; ++q)
        if (p0 + q < a.n_planes) {
#pragma unroll
          for (int j = 0; j < KCH; ++j) { v[j].x += t[q][j].x; v[j].y += t[q][j].y; v[j].z += t[q][j].z; v[j].w += t[q][j].w; }
        }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < KCH; ++j) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)D + a.eps);
#pragma unroll
  for (int j = 0; j < KCH; ++j) {
    const int c = j * 256 + lane * 4;
    if (c < D) {
      const float4 g = a.gamma_is_bf16 ? df_load4(reinterpret_cast<const bf16*>(a.gamma) + c)
                                       : df_load4(reinterpret_cast<const float*>(a.gamma) + c);
      uint2 r;
      r.x = f32x2_to_bf16x2_bits(v[j].x * inv * g.x, v[j].y * inv * g.y);
      r.y = f32x2_to_bf16x2_bits(v[j].z * inv * g.z, v[j].w * inv * g.w);
      *reinterpret_cast<uint2*>(xrow + c) = r;
    }
  }
}

// KS: k-steps of 32 that a wavefront takes of the gate/up product (K = D is split over the 8 wavefronts);
// TPF: column tiles of a round (their weights are in registers together: TPF * KS fragments);
// KCH / PB: see df_norm_row.
template <int KS, int TPF, int KCH, int PB>
__global__ void __launch_bounds__(DF_THREADS) decode_ffn_kernel(const DecodeFfnArgs a) {
  extern __shared__ __align__(16) unsigned char df_smem[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int row = lane & 15, kg = lane >> 4;
  const int M = a.M, D = a.D, I = a.I;
  const int k_steps = (D + 31) / 32;          // of the gate/up product
  const int xstride = k_steps * 32 + DF_PAD;  // elements per row of x in shared memory
  bf16* const x_lds = reinterpret_cast<bf16*>(df_smem);                          // [16][xstride]
  float* const red = reinterpret_cast<float*>(df_smem + (size_t)16 * xstride * 2);   // [DF_WAVES][TPF][256]
  unsigned* const act_s = reinterpret_cast<unsigned*>(red + DF_WAVES * TPF * 256);   // [tiles of the block][16 rows][4 pairs of pairs]

  // ---- the block's share of the gate/up product: a run of neighbouring column tiles ----
  const int n_tiles = I / 8;                  // 16 columns = 8 gated pairs per tile
  const int per_block = (n_tiles + gridDim.x - 1) / gridDim.x;
  const int tile_begin = min(n_tiles, (int)blockIdx.x * per_block), tile_end = min(n_tiles, tile_begin + per_block);
  const int step0 = wave * KS;
  int woff[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) woff[s] = (step0 + s < k_steps ? step0 + s : k_steps - 1) * 512 + lane * 8;
  uint4 w[TPF][KS];
#define DF_LOAD_ROUND(first_tile)                                                                  \
  _Pragma("unroll") for (int j = 0; j < TPF; ++j) {                                                  \
    const int tile = min((first_tile) + j, n_tiles - 1);                                             \
    const bf16* wt = a.w_gu + (size_t)tile * k_steps * 512;                                          \
    _Pragma("unroll") for (int s = 0; s < KS; ++s) w[j][s] = df_stream16(wt + woff[s]);             \
  }

  // ---- phase 1: the normalised rows; the first round's weights travel meanwhile ----
  // rows beyond M and columns beyond D are zero in shared memory
  for (int i = threadIdx.x; i < 16 * xstride / 2; i += DF_THREADS) {
    const int r = (i * 2) / xstride, c = (i * 2) - r * xstride;
    if (r >= M || c >= D) reinterpret_cast<unsigned*>(x_lds)[i] = 0u;
  }
  if (wave >= M) {   // no row of its own: the weights are requested at once
    if (tile_begin < tile_end) { DF_LOAD_ROUND(tile_begin) }
  } else {
    for (int r = wave; r < M; r += DF_WAVES) {
      if (a.delta_is_bf16) df_norm_row<KCH, PB, bf16>(a, r, x_lds + (size_t)r * xstride, lane);
      else df_norm_row<KCH, PB, float>(a, r, x_lds + (size_t)r * xstride, lane);
    }
    if (tile_begin < tile_end) { DF_LOAD_ROUND(tile_begin) }
  }
  __syncthreads();

  // ---- phase 2: gate/up product and gating ----
  uint4 af[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int k = (step0 + s) * 32 + kg * 8;
    af[s] = step0 + s < k_steps ? *reinterpret_cast<const uint4*>(x_lds + (size_t)row * xstride + k) : make_uint4(0u, 0u, 0u, 0u);
  }
  for (int t0 = tile_begin; t0 < tile_end; t0 += TPF) {
    if (t0 != tile_begin) { DF_LOAD_ROUND(t0) }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < TPF; ++j) {
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, af[s]),
                                                      __builtin_bit_cast(bf16x8_t, w[j][s]), acc, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(wave * TPF + j) * 256 + r * 64 + lane] = acc[r];
    }
    __syncthreads();
    // acc[r] of lane l is row m = (l / 16) * 4 + r, column l % 16 of the tile; columns 0..7 are gates,
    // 8..15 their ups.  One thread per (tile of the round, row, pair of pairs).
    for (int idx = threadIdx.x; idx < TPF * 16 * 4; idx += DF_THREADS) {
      const int j = idx / 64, m = (idx >> 2) & 15, pp = idx & 3;   // pairs 2 pp and 2 pp + 1 of the tile
      if (t0 + j < tile_end) {
        float y[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int col = pp * 2 + e;
          const int at = (m & 3) * 64 + (m >> 2) * 16 + col;
          float g = 0.f, u = 0.f;
#pragma unroll
          for (int w2 = 0; w2 < DF_WAVES; ++w2) {
            g += red[(w2 * TPF + j) * 256 + at];
            u += red[(w2 * TPF + j) * 256 + at + 8];
          }
          y[e] = g / (1.0f + expf(-g)) * u;
        }
        act_s[((t0 + j - tile_begin) * 16 + m) * 4 + pp] = f32x2_to_bf16x2_bits(y[0], y[1]);
      }
    }
    __syncthreads();
  }
#undef DF_LOAD_ROUND

  // ---- the block's first item of the down product; its weights are requested before the grid meets ----
  const int n_tiles_d = (D + 15) / 16, k_steps_d = (I + 31) / 32;
  const int per_group = (k_steps_d + a.k_groups - 1) / a.k_groups;      // k-steps of a K-group
  const int per_wave = (per_group + DF_WAVES - 1) / DF_WAVES;           // k-steps of a wavefront in a group
  const int n_items = n_tiles_d * a.k_groups;
  uint4 wd[16];
  // 16 k-steps from c0 of this wavefront's share of the item
#define DF_LOAD_DOWN(item_, c0_)                                                                               \
  {                                                                                                            \
    const int tile_ = (item_) / a.k_groups, g_ = (item_) - tile_ * a.k_groups;                                 \
    const int first_ = g_ * per_group + wave * per_wave + (c0_);                                               \
    const bf16* wt_ = a.w_down + (size_t)tile_ * k_steps_d * 512 + lane * 8;                                   \
    _Pragma("unroll") for (int s = 0; s < 16; ++s) wd[s] = df_stream16(wt_ + (size_t)min(first_ + s, k_steps_d - 1) * 512); \
  }
  if (wave != 0 && (int)blockIdx.x < n_items) DF_LOAD_DOWN(blockIdx.x, 0)

  // ---- the gated values go out; the grid meets ----
  if (wave == 0) {
    const int n_mine = (tile_end - tile_begin) * 16 * 4;
    for (int i = lane; i < n_mine; i += BLM_WAVE) {
      const int t = i / 64, m = (i >> 2) & 15, pp = i & 3;
      if (m < M) df_store_coherent(a.act + ((size_t)m * I + (size_t)(tile_begin + t) * 8 + pp * 2) / 2, act_s[i]);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the stores have been acknowledged
    if ((int)blockIdx.x < n_items) DF_LOAD_DOWN(blockIdx.x, 0)
    if (lane == 0) {
      __hip_atomic_fetch_add(a.sync, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      int polls = 0;
      while (__hip_atomic_load(a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (int)gridDim.x) {
        if (++polls > a.spin_limit) {   // give up: say so where the host sees it, and go on
          __hip_atomic_store(a.fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    }
  }
  __syncthreads();

  // ---- phase 3: down product on (column tile, K-group) items ----
  const unsigned long long* act64 = reinterpret_cast<const unsigned long long*>(a.act);
  for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
    const int tile = item / a.k_groups, g = item - tile * a.k_groups;
    const int group_end = min(k_steps_d, (g + 1) * per_group);
    const int wave_first = g * per_group + wave * per_wave;
    const int wave_end = min(group_end, wave_first + per_wave);
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int c0 = 0; c0 < per_wave; c0 += 16) {
      if (!(item == (int)blockIdx.x && c0 == 0)) DF_LOAD_DOWN(item, c0)
      uint4 ad[16];
#pragma unroll
      for (int s = 0; s < 16; ++s) {
        const int step = wave_first + c0 + s;
        const int k = step * 32 + kg * 8;
        if (row < M && step < wave_end && k < I) {
          const unsigned long long lo = df_load_coherent(act64 + ((size_t)row * I + k) / 4);
          const unsigned long long hi = df_load_coherent(act64 + ((size_t)row * I + k) / 4 + 1);
          ad[s] = make_uint4((unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32));
        } else {
          ad[s] = make_uint4(0u, 0u, 0u, 0u);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 16; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ad[s]),
                                                      __builtin_bit_cast(bf16x8_t, wd[s]), acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
    __syncthreads();
    if (threadIdx.x < 256) {
      const int idx = threadIdx.x, r = idx >> 6, l2 = idx & 63, col = l2 & 15;
      const int m = (l2 >> 4) * 4 + r, n = tile * 16 + col;
      float s = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < DF_WAVES; ++w2) s += red[w2 * 256 + idx];
      if (m < M && n < D) a.out[((size_t)g * M + m) * D + n] = s;
    }
    __syncthreads();
  }

#undef DF_LOAD_DOWN
  // ---- h += delta for this block's share of (row, 256-column chunk) pieces: every block has read the old rows ----
  if (a.delta && wave == DF_WAVES - 1) {
    const int chunks = (D + 255) / 256;
    for (int q = blockIdx.x; q < M * chunks; q += gridDim.x) {
      const int r = q / chunks, c = (q - r * chunks) * 256 + lane * 4;
      if (c < D) {
        const float4 v = a.delta_is_bf16 ? df_row_sum4<bf16>(a, r, c) : df_row_sum4<float>(a, r, c);
        *reinterpret_cast<float4*>(a.h + (size_t)r * D + c) = v;
      }
    }
  }

  // ---- the counters return to zero behind the last block ----
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(a.sync + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before == (int)gridDim.x - 1) {
      __hip_atomic_store(a.sync, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(a.sync + 1, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Shared memory a block needs: the rows of x, the partial tiles of a round, the block's gated values;
// never less than 96 KB, so that two blocks cannot share a compute unit.
static size_t decode_ffn_smem(int D, int I, int blocks, int tpf) {
  const int k_steps = (D + 31) / 32;
  const int n_tiles = I / 8, per_block = (n_tiles + blocks - 1) / blocks;
  size_t s = (size_t)16 * (k_steps * 32 + DF_PAD) * 2 + (size_t)DF_WAVES * tpf * 256 * 4 + (size_t)per_block * 16 * 4 * 4;
  return s < (96u << 10) ? (96u << 10) : s;
}

// The shapes the fused kernel takes: up to 16 rows, width a multiple of 8 up to 4096, inner size a
// multiple of 16 whose gated values of one block fit shared memory.
extern "C" int blm_decode_ffn_supported(int M, int D, int I, int blocks) {
  if (M < 1 || M > 16 || D < 8 || D % 8 || D > 4096 || I < 16 || I % 16 || blocks < 1) return 0;
  const int ks = ((D + 31) / 32 + DF_WAVES - 1) / DF_WAVES;
  const int tpf = ks <= 8 ? 4 : 2;
  return decode_ffn_smem(D, I, blocks, tpf) <= (160u << 10) ? 1 : 0;
}

static int g_decode_ffn_ready[64];

extern "C" int blm_decode_ffn(float* h, const void* delta, int delta_dtype, int n_planes, long long plane_stride,
                              const void* gamma, int gamma_dtype, float eps, const void* w_gu, const void* w_down,
                              void* act, float* out, int M, int D, int I, int k_groups, int blocks, int* sync,
                              int* fault, int spin_limit, hipStream_t stream) {
  BLM_REQUIRE(blm_decode_ffn_supported(M, D, I, blocks), "decode_ffn: M=%d D=%d I=%d with %d blocks is not supported "
              "(up to 16 rows, width a multiple of 8 up to 4096, inner size a multiple of 16)", M, D, I, blocks);
  BLM_REQUIRE(h && gamma && w_gu && w_down && act && out && sync && fault, "decode_ffn: a pointer is missing");
  BLM_REQUIRE(delta == nullptr || (n_planes >= 1 && n_planes <= 64 && plane_stride >= 0 && plane_stride % 4 == 0 &&
                                   (delta_dtype == BLM_F32 || (delta_dtype == BLM_BF16 && n_planes == 1))),
              "decode_ffn: bad delta (dtype %d, %d planes)", delta_dtype, n_planes);
  BLM_REQUIRE(gamma_dtype == BLM_F32 || gamma_dtype == BLM_BF16, "decode_ffn: gamma dtype %d", gamma_dtype);
  BLM_REQUIRE(k_groups >= 1 && k_groups <= 64 && spin_limit > 0, "decode_ffn: bad k_groups %d or spin limit %d", k_groups, spin_limit);
  BLM_REQUIRE(((uintptr_t)h % 16) == 0 && ((uintptr_t)delta % 16) == 0 && ((uintptr_t)gamma % 16) == 0 &&
              ((uintptr_t)w_gu % 16) == 0 && ((uintptr_t)w_down % 16) == 0 && ((uintptr_t)act % 16) == 0 &&
              ((uintptr_t)out % 16) == 0, "decode_ffn: operands must be 16-byte aligned");
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  BLM_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, "decode_ffn: hipGetDevice failed");
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  BLM_REQUIRE(e == hipSuccess && blocks <= cus, "decode_ffn: %d blocks, the device has %d compute units: every block "
              "waits for all the others, so there may be no more blocks than units", blocks, cus);
  const int ks = ((D + 31) / 32 + DF_WAVES - 1) / DF_WAVES;
  const int tpf = ks <= 8 ? 4 : 2;
  const size_t smem = decode_ffn_smem(D, I, blocks, tpf);
  DecodeFfnArgs a;
  a.h = h; a.delta = delta; a.delta_is_bf16 = delta_dtype == BLM_BF16; a.n_planes = n_planes; a.plane_stride = plane_stride;
  a.gamma = gamma; a.gamma_is_bf16 = gamma_dtype == BLM_BF16; a.eps = eps;
  a.w_gu = (const bf16*)w_gu; a.w_down = (const bf16*)w_down; a.act = (unsigned*)act; a.out = out;
  a.M = M; a.D = D; a.I = I; a.k_groups = k_groups; a.sync = sync; a.fault = fault; a.spin_limit = spin_limit;
#define BLM_DF(KS, TPF, KCH, PB)                                                                                  \
  do {                                                                                                            \
    if (!(g_decode_ffn_ready[dev] & (1 << (KS / 4)))) {                                                           \
      e = hipFuncSetAttribute((const void*)decode_ffn_kernel<KS, TPF, KCH, PB>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 << 10); \
      BLM_REQUIRE(e == hipSuccess, "decode_ffn: cannot have %d KB of shared memory: %s", 160, hipGetErrorString(e)); \
      g_decode_ffn_ready[dev] |= 1 << (KS / 4);                                                                   \
    }                                                                                                             \
    hipLaunchKernelGGL((decode_ffn_kernel<KS, TPF, KCH, PB>), dim3(blocks), dim3(DF_THREADS), smem, stream, a);   \
  } while (0)
  if (ks <= 8) BLM_DF(8, 4, 8, 2);
  else if (ks <= 12) BLM_DF(12, 2, 16, 1);
  else BLM_DF(16, 2, 16, 1);
#undef BLM_DF
  BLM_LAUNCH_CHECK("decode_ffn");
  return 0;
}
