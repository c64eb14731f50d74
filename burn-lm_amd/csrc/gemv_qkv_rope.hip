// Decode: the query/key/value projection fused with the rotary encoding and the cache write.
//
//   qkv = x W_qkv^T  (bf16 operands on the matrix cores, packed weights, see gemv_mfma.hip)
//   q, k rotated by each token's position (float, on the float accumulators, rounded once)
//   q -> the activation buffer;  k -> its key page;  v -> its (transposed) value page
//
// A block owns one rotation unit: the two 16-column tiles that hold partner lanes of one head.
// With pairing 1 (lane i with i + head_dim/2) these are tiles j and j + head_dim/32 of the head;
// with pairing 0 (lanes 2i, 2i+1) the partners sit in one tile: see gemv_qkv_rope_tile_kernel, which
// the entry point uses then (this kernel takes both pairings).
// Value heads are not rotated and use the same unit shape.  Wavefronts 0..KW-1 work on the first
// tile, KW..2KW-1 on the second, each on 512 of K; the partial tiles are summed through LDS and
// the epilogue rotates and scatters them.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// QR_KSTEPS: k-steps of 32 per wavefront.  MAXT: most threads of a block (8 or 16 wavefronts).  All
// loads of a block are in flight at once: its time is one memory latency.
template <int QR_KSTEPS, int MAXT>
__global__ void __launch_bounds__(MAXT)
    gemv_qkv_rope_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, bf16* __restrict__ qkv_out,
                         const int* __restrict__ positions, const int* __restrict__ token_seq,
                         const int* __restrict__ block_table, int table_width, const float2* __restrict__ cos_sin,
                         bf16* __restrict__ kcache, bf16* __restrict__ vcache, int page_size, int M, int K, int lda,
                         int ldq, int k_steps, int kw_count, int nh, int nkv, int hd, int pairing, int store) {
  extern __shared__ float red[];   // [2 * kw_count wavefronts][256]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int row = lane & 15, kg = lane >> 4;
  const int units_per_head = hd / 32;
  const int head = blockIdx.x / units_per_head, j = blockIdx.x - head * units_per_head;
  if (!store && head >= nh) return;   // keys and values belong to another layer's cache: only q is needed
  const int tiles_per_head = hd / 16;
  // columns (within the head) of the unit's two tiles
  const int col0 = pairing == 1 ? j * 16 : j * 32;
  const int col1 = pairing == 1 ? j * 16 + hd / 2 : j * 32 + 16;
  const int which = wave / kw_count, kw = wave - which * kw_count;
  const int tile = head * tiles_per_head + (which == 0 ? col0 : col1) / 16;
  const int step0 = kw * QR_KSTEPS;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  const bf16* wt = Wp + ((size_t)tile * k_steps * 64 + lane) * 8;
  uint4 w[QR_KSTEPS];
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s) {
    const int st = step0 + s;
    w[s] = load16_stream(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);   // the weights: read once
  }
  const bf16* ap = A + (size_t)(row < M ? row : M - 1) * lda;
  uint4 a[QR_KSTEPS];
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s) {
    const int k = (step0 + s) * 32 + kg * 8;
    const uint4 v = *reinterpret_cast<const uint4*>(ap + (k < K ? k : K - 8));
    a[s] = (row < M && k < K) ? v : zero;
  }
  __builtin_amdgcn_sched_barrier(0);
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                  __builtin_bit_cast(bf16x8_t, w[s]), acc, 0, 0, 0);
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
  __syncthreads();

  // epilogue: one thread per (token row m, column c of the tiles)
  for (int idx = threadIdx.x; idx < 256; idx += blockDim.x) {
    const int r = idx >> 6, l2 = idx & 63, c = l2 & 15;
    const int m = (l2 >> 4) * 4 + r;
    if (m >= M) continue;
    float x0 = 0.f, x1 = 0.f;
    for (int k2 = 0; k2 < kw_count; ++k2) {
      x0 += red[k2 * 256 + idx];
      x1 += red[(kw_count + k2) * 256 + idx];
    }
    const int b = token_seq[m];
    const int pos = positions[m];
    const int d0 = col0 + c, d1 = col1 + c;      // lanes within the head held by x0 and x1
    float y0 = x0, y1 = x1;     // value heads are stored as they are
    if (head < nh + nkv && pairing == 1) {
      // partners are (d0, d1 = d0 + hd/2): this thread holds both; angle index d0
      const float2 cs = cos_sin[(size_t)pos * (hd / 2) + d0];
      y0 = x0 * cs.x - x1 * cs.y;
      y1 = x0 * cs.y + x1 * cs.x;
    } else if (head < nh + nkv) {
      // partners are neighbours (2i, 2i+1) inside each tile: column c pairs with c ^ 1, whose sums
      // this thread forms as well
      float p0 = 0.f, p1 = 0.f;
      for (int k2 = 0; k2 < kw_count; ++k2) {
        p0 += red[k2 * 256 + (idx ^ 1)];
        p1 += red[(kw_count + k2) * 256 + (idx ^ 1)];
      }
      const float2 c0 = cos_sin[(size_t)pos * (hd / 2) + (d0 >> 1)];
      const float2 c1 = cos_sin[(size_t)pos * (hd / 2) + (d1 >> 1)];
      if ((c & 1) == 0) { y0 = x0 * c0.x - p0 * c0.y; y1 = x1 * c1.x - p1 * c1.y; }
      else              { y0 = p0 * c0.y + x0 * c0.x; y1 = p1 * c1.y + x1 * c1.x; }
    }
    const bf16 o0 = from_float<bf16>(y0), o1 = from_float<bf16>(y1);
    if (head < nh) {
      bf16* qrow = qkv_out + (size_t)m * ldq + (size_t)head * hd;
      qrow[d0] = o0;
      qrow[d1] = o1;
    } else if (b >= 0) {
      const int page = block_table[(size_t)b * table_width + pos / page_size];
      const int slot = pos % page_size;
      if (page < 0) continue;
      if (head < nh + nkv) {
        bf16* kd = kcache + (((size_t)page * nkv + (head - nh)) * page_size + slot) * hd;
        kd[d0] = o0;
        kd[d1] = o1;
      } else {
        bf16* vd = vcache + ((size_t)page * nkv + (head - nh - nkv)) * hd * page_size + slot;
        vd[(size_t)d0 * page_size] = o0;
        vd[(size_t)d1 * page_size] = o1;
      }
    }
  }
}

// Pairing 0 (partners are neighbours 2i, 2i+1): both partners sit in the same 16-column tile, so a
// block owns ONE tile and its wavefronts split K.  That is twice as many blocks as with two-tile
// units, which matters because the whole product is a few blocks per compute unit at most (3072
// columns are 192 tiles).  Value heads are not rotated.  red: [wavefronts][256].
template <int QR_KSTEPS>
__global__ void __launch_bounds__(512)
    gemv_qkv_rope_tile_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, bf16* __restrict__ qkv_out,
                              const int* __restrict__ positions, const int* __restrict__ token_seq,
                              const int* __restrict__ block_table, int table_width,
                              const float2* __restrict__ cos_sin, bf16* __restrict__ kcache,
                              bf16* __restrict__ vcache, int page_size, int M, int K, int lda, int ldq, int k_steps,
                              int nh, int nkv, int hd, int store) {
  extern __shared__ float red[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  const int tiles_per_head = hd / 16;
  const int tile = blockIdx.x;
  const int head = tile / tiles_per_head, col0 = (tile - head * tiles_per_head) * 16;
  if (!store && head >= nh) return;   // keys and values belong to another layer's cache: only q is needed
  const int step0 = wave * QR_KSTEPS;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  const bf16* wt = Wp + ((size_t)tile * k_steps * 64 + lane) * 8;
  uint4 w[QR_KSTEPS];
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s) {
    const int st = step0 + s;
    w[s] = load16_stream(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);   // the weights: read once
  }
  const bf16* ap = A + (size_t)(row < M ? row : M - 1) * lda;
  uint4 a[QR_KSTEPS];
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s) {
    const int k = (step0 + s) * 32 + kg * 8;
    const uint4 v = *reinterpret_cast<const uint4*>(ap + (k < K ? k : K - 8));
    a[s] = (row < M && k < K) ? v : zero;
  }
  __builtin_amdgcn_sched_barrier(0);
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                  __builtin_bit_cast(bf16x8_t, w[s]), acc, 0, 0, 0);
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave * 256 + r * 64 + lane] = acc[r];
  __syncthreads();

  // epilogue: one thread per (token row m, column c of the tile)
  for (int idx = threadIdx.x; idx < 256; idx += blockDim.x) {
    const int r = idx >> 6, l2 = idx & 63, c = l2 & 15;
    const int m = (l2 >> 4) * 4 + r;
    if (m >= M) continue;
    float x = 0.f, partner = 0.f;   // column c and its neighbour c ^ 1
    for (int k2 = 0; k2 < n_waves; ++k2) {
      x += red[k2 * 256 + idx];
      partner += red[k2 * 256 + (idx ^ 1)];
    }
    const int b = token_seq[m];
    const int pos = positions[m];
    const int d = col0 + c;
    float y = x;     // value heads are stored as they are
    if (head < nh + nkv) {
      const float2 cs = cos_sin[(size_t)pos * (hd / 2) + (d >> 1)];
      y = (c & 1) == 0 ? x * cs.x - partner * cs.y : partner * cs.y + x * cs.x;
    }
    const bf16 o = from_float<bf16>(y);
    if (head < nh) {
      qkv_out[(size_t)m * ldq + (size_t)head * hd + d] = o;
    } else if (b >= 0) {
      const int page = block_table[(size_t)b * table_width + pos / page_size];
      const int slot = pos % page_size;
      if (page < 0) continue;
      if (head < nh + nkv) kcache[(((size_t)page * nkv + (head - nh)) * page_size + slot) * hd + d] = o;
      else vcache[((size_t)page * nkv + (head - nh - nkv)) * hd * page_size + (size_t)d * page_size + slot] = o;
    }
  }
}

// 17 to 64 rows, adjacent pairs: as gemv_qkv_rope_tile_kernel, with MT row tiles of 16 against every
// weight fragment (the activations of all row tiles stay in registers, as in gemv_mfma_rows_kernel:
// MT * QR_KSTEPS fragments, at most 32).  One tile per block; red: [wavefronts][MT][256].
template <int MT, int QR_KSTEPS>
__global__ void __launch_bounds__(512)
    gemv_qkv_rope_rows_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wp, bf16* __restrict__ qkv_out,
                              const int* __restrict__ positions, const int* __restrict__ token_seq,
                              const int* __restrict__ block_table, int table_width,
                              const float2* __restrict__ cos_sin, bf16* __restrict__ kcache,
                              bf16* __restrict__ vcache, int page_size, int M, int K, int lda, int ldq, int k_steps,
                              int nh, int nkv, int hd, int store) {
  extern __shared__ float red[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int n_waves = blockDim.x / BLM_WAVE;
  const int row = lane & 15, kg = lane >> 4;
  const int tiles_per_head = hd / 16;
  const int tile = blockIdx.x;
  const int head = tile / tiles_per_head, col0 = (tile - head * tiles_per_head) * 16;
  if (!store && head >= nh) return;   // keys and values belong to another layer's cache: only q is needed
  const int step0 = wave * QR_KSTEPS;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

  const bf16* wt = Wp + ((size_t)tile * k_steps * 64 + lane) * 8;
  uint4 w[QR_KSTEPS];
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s) {
    const int st = step0 + s;
    w[s] = load16_stream(wt + (size_t)(st < k_steps ? st : k_steps - 1) * 512);   // the weights: read once
  }
  uint4 a[MT][QR_KSTEPS];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + row;
    const bf16* ap = A + (size_t)(m < M ? m : M - 1) * lda;   // rows >= M read a real row and are zeroed
#pragma unroll
    for (int s = 0; s < QR_KSTEPS; ++s) {
      const int k = (step0 + s) * 32 + kg * 8;
      const uint4 v = *reinterpret_cast<const uint4*>(ap + (k < K ? k : K - 8));
      a[mt][s] = (m < M && k < K) ? v : zero;
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < QR_KSTEPS; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[mt][s]),
                                                        __builtin_bit_cast(bf16x8_t, w[s]), acc[mt], 0, 0, 0);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[(wave * MT + mt) * 256 + r * 64 + lane] = acc[mt][r];
  __syncthreads();

  // epilogue: one thread per (token row m, column c of the tile)
  for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
    const int mt = idx >> 8, i = idx & 255;
    const int r = i >> 6, l2 = i & 63, c = l2 & 15;
    const int m = mt * 16 + (l2 >> 4) * 4 + r;
    if (m >= M) continue;
    float x = 0.f, partner = 0.f;   // column c and its neighbour c ^ 1
    for (int k2 = 0; k2 < n_waves; ++k2) {
      x += red[(k2 * MT + mt) * 256 + i];
      partner += red[(k2 * MT + mt) * 256 + (i ^ 1)];
    }
    const int b = token_seq[m];
    const int pos = positions[m];
    const int d = col0 + c;
    float y = x;     // value heads are stored as they are
    if (head < nh + nkv) {
      const float2 cs = cos_sin[(size_t)pos * (hd / 2) + (d >> 1)];
      y = (c & 1) == 0 ? x * cs.x - partner * cs.y : partner * cs.y + x * cs.x;
    }
    const bf16 o = from_float<bf16>(y);
    if (head < nh) {
      qkv_out[(size_t)m * ldq + (size_t)head * hd + d] = o;
    } else if (b >= 0) {
      const int page = block_table[(size_t)b * table_width + pos / page_size];
      const int slot = pos % page_size;
      if (page < 0) continue;
      if (head < nh + nkv) kcache[(((size_t)page * nkv + (head - nh)) * page_size + slot) * hd + d] = o;
      else vcache[((size_t)page * nkv + (head - nh - nkv)) * hd * page_size + (size_t)d * page_size + slot] = o;
    }
  }
}

// Up to 16 rows: pairing 0 takes every head size that is a multiple of 16; pairing 1 (partners half a
// head apart, two tiles per block) needs a multiple of 32; K up to 4096.  17 to 64 rows: adjacent
// pairs only; K up to 4096 for at most 32 rows and up to 2048 beyond (the activations' registers).
extern "C" int blm_gemv_qkv_rope_supported(int M, int K, int hd, int pairing) {
  const int step = pairing == 0 ? 16 : 32;
  if (!(M >= 1 && M <= 64 && K >= 8 && K % 8 == 0 && hd >= step && hd % step == 0 && (pairing == 0 || pairing == 1)))
    return 0;
  if (M <= 16) return K <= 4096 ? 1 : 0;
  if (pairing != 0) return 0;
  return K <= (M <= 32 ? 4096 : 2048) ? 1 : 0;
}

// Wp: pack_weight of W_qkv [(nh + 2 nkv) * hd, K].  qkv_out: [M, ldq] bf16; only its first nh*hd
// columns (the rotated queries) are written.  Key plane [pages, nkv, page, hd], value plane
// [pages, nkv, hd, page].  store = 0: keys and values are neither computed nor written.
extern "C" int blm_gemv_qkv_rope(const void* A, const void* Wp, void* qkv_out, const int* positions,
                                 const int* token_seq, const int* block_table, int table_width,
                                 const float* cos_sin, void* kcache, void* vcache, int page_size, int M, int K,
                                 int lda, int ldq, int nh, int nkv, int hd, int pairing, int store,
                                 hipStream_t stream) {
  BLM_REQUIRE(blm_gemv_qkv_rope_supported(M, K, hd, pairing), "gemv_qkv_rope: M=%d K=%d head_dim=%d pairing=%d not "
              "supported (K a multiple of 8 and at most 4096, head_dim a multiple of 16 for adjacent pairs and of "
              "32 for pairs half a head apart; 17 to 64 rows: adjacent pairs, K at most 2048 above 32 rows)",
              M, K, hd, pairing);
  BLM_REQUIRE(nh > 0 && nkv > 0 && page_size > 0 && table_width > 0, "gemv_qkv_rope: bad geometry");
  BLM_REQUIRE(lda % 8 == 0 && lda >= K && ldq >= nh * hd, "gemv_qkv_rope: bad strides lda=%d ldq=%d", lda, ldq);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)Wp % 16) == 0, "gemv_qkv_rope: operands must be 16-byte aligned");
  const int k_steps = (K + 31) / 32;
  const int tiles = (nh + 2 * nkv) * (hd / 16);
  if (M > 16) {
    const int mt = (M + 15) / 16;
    const int ks = k_steps > 64 ? 16 : 8;            // more than 2048 of K: two row tiles at most
    const int waves = (k_steps + ks - 1) / ks;       // at most 8
    const size_t smem = (size_t)waves * mt * 256 * sizeof(float);
#define BLM_QRR(MT, KS)                                                                                            \
  hipLaunchKernelGGL((gemv_qkv_rope_rows_kernel<MT, KS>), dim3(tiles), dim3(waves * BLM_WAVE), smem, stream,       \
                     (const bf16*)A, (const bf16*)Wp, (bf16*)qkv_out, positions, token_seq, block_table,           \
                     table_width, (const float2*)cos_sin, (bf16*)kcache, (bf16*)vcache, page_size, M, K, lda, ldq, \
                     k_steps, nh, nkv, hd, store)
    if (ks == 16) BLM_QRR(2, 16);
    else if (mt == 2) BLM_QRR(2, 8);
    else if (mt == 3) BLM_QRR(3, 8);
    else BLM_QRR(4, 8);
#undef BLM_QRR
    BLM_LAUNCH_CHECK("gemv_qkv_rope_rows");
    return 0;
  }
  // Adjacent pairs: one tile per block while that is one round of blocks on the chip's 256 compute
  // units (or the head size leaves no choice, or K is so wide that two-tile blocks would need 16
  // wavefronts and spill); beyond that, blocks of two tiles (measured at 320 tiles, K = 3072: one
  // tile per block 2.7 % of a step slower).
  if (pairing == 0 && (tiles <= 256 || hd % 32 != 0 || k_steps > 96)) {
    // 16 k-steps per wavefront: up to 8 wavefronts
    const int waves = (k_steps + 15) / 16;
    hipLaunchKernelGGL(gemv_qkv_rope_tile_kernel<16>, dim3(tiles), dim3(waves * BLM_WAVE), (size_t)waves * 256 * sizeof(float),
                       stream, (const bf16*)A, (const bf16*)Wp, (bf16*)qkv_out, positions, token_seq, block_table,
                       table_width, (const float2*)cos_sin, (bf16*)kcache, (bf16*)vcache, page_size, M, K, lda, ldq,
                       k_steps, nh, nkv, hd, store);
    BLM_LAUNCH_CHECK("gemv_qkv_rope_tile");
    return 0;
  }
  // all of a block's loads are in flight at once: 4 wavefronts per tile with 16 k-steps each up to
  // K = 2048, with 24 up to 3072 (their registers still fit), and 8 wavefronts with 16 up to 4096
  const int ksteps = (k_steps > 64 && k_steps <= 96) ? 24 : 16;
  const int kw = (k_steps + ksteps - 1) / ksteps;   // at most 8
  const int units = (nh + 2 * nkv) * (hd / 32);
  const size_t smem = (size_t)2 * kw * 256 * sizeof(float);
#define BLM_QR(KS, MAXT)                                                                                              \
  hipLaunchKernelGGL((gemv_qkv_rope_kernel<KS, MAXT>), dim3(units), dim3(2 * kw * BLM_WAVE), smem, stream, (const bf16*)A, \
                     (const bf16*)Wp, (bf16*)qkv_out, positions, token_seq, block_table, table_width,                 \
                     (const float2*)cos_sin, (bf16*)kcache, (bf16*)vcache, page_size, M, K, lda, ldq, k_steps, kw, nh, \
                     nkv, hd, pairing, store)
  if (ksteps == 24) BLM_QR(24, 512);
  else if (kw <= 4) BLM_QR(16, 512);
  else BLM_QR(16, 1024);
#undef BLM_QR
  BLM_LAUNCH_CHECK("gemv_qkv_rope");
  return 0;
}
