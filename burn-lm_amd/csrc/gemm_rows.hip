// Matrix product for few rows, made for 17 to 64 (decode steps of many sequences), on the matrix
// cores: C[M, N] = A[M, K] * W[N, K]^T, bf16 operands, W as the checkpoint stores it, float accumulation,
// bf16 or float output.  Up to 256 rows it runs as one block for every 32 or 64 rows (blockIdx.z), each a
// product of its own: for narrow products of short prompts and of decode steps of more than 64 sequences.
//
// A block of four wavefronts owns its rows (staged as 32 or 64) and BN columns of C (and one group of
// K).  Its wavefronts take the block's stages of 64 along K in turn (wavefront w: stages w, w + 4, ...), a stage being the
// rows' and the columns' slices of 64, loaded 16 bytes per lane straight from global memory into a ring
// of R slots of shared memory that belongs to the wavefront alone.  A wavefront waits only for its own
// loads (they complete in order), reads its fragments, hands the slot to a later stage and multiplies:
// no wavefront waits for another until the four partial tiles are added at the end, so the loads of a
// compute unit never stop for a barrier.  With so few rows memory, not arithmetic, is the limit, and
// the activations cost as much traffic as the weights (every block reads all rows): they come the same
// way as the weights, which measured faster than keeping them in registers (gemv_mfma_rows_kernel).
// Staged rows are unpadded with their 16-byte pieces XOR-permuted as in gemm_mfma.hip, so that fragment
// reads meet every bank once.
//
// mode 1: W holds gate rows [0, N) and up rows [N, 2N) of a gated feed-forward; a block takes BN / 2
// gate columns and the matching up columns, and C[M, N] = silu(gate) * up.
// k_groups > 1: K is cut into groups, C is float [k_groups, M, ldc] with one partial product each
// (summed by the reader), so that a narrow output still fills the chip.
// mode 2: W is the q/k/v projection; where the partial tiles meet, queries and keys are rotated by
// their positions (partners in adjacent columns), queries go to C, keys and values to their pages
// of the cache, as gemv_qkv_rope.hip does for up to 16 rows.
#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 gr_bf16x8;
typedef __attribute__((ext_vector_type(16))) float gr_f32x16;

__device__ __align__(16) const uint32_t gr_zero_piece[4] = {0u, 0u, 0u, 0u};

#define GR_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#define GR_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

// what mode 2 needs beside the product: positions and sequences of the rows, the pages, the table of
// cosines and sines, the cache planes (keys [pages, nkv, page, hd], values [pages, nkv, hd, page])
struct GrRope {
  const int* positions;
  const int* token_seq;
  const int* block_table;
  const float2* cos_sin;
  bf16* kcache;
  bf16* vcache;
  int table_width, page_size, nh, nkv, hd, store;
};

#define GR_MAX_ROWS 256   // four blocks of 64 rows

template <int BM, int BN, int BK, int R, int MODE, typename TC>
__global__ void __launch_bounds__(256)
    gemm_rows_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C, int M, int N, int K, int lda,
                     int ldw, int ldc, int k_per_group, GrRope rope) {
  constexpr int NW = 4;
  static_assert(BM == 32 || BM == 64, "rows");
  constexpr int TM = BM / 32, TN = BN / 32;
  static_assert(BK == 32 || BK == 64, "stage depth");   // 64: whole cache lines per row (measured: 15 % faster than 32)
  static_assert(BN % 32 == 0, "columns");
  constexpr int P = BK / 8;                 // 16-byte pieces per staged row
  constexpr int RPL = 64 / P;               // rows that one load instruction fills
  constexpr int RPB = 256 / (BK * 2);       // staged rows per pass over the banks
  constexpr int A_LD = BM / RPL, B_LD = BN / RPL, LOADS = A_LD + B_LD;
  constexpr int QN = BK / 16;               // k-steps of the matrix instruction per stage
  constexpr int SLOT = (BM + BN) * BK;      // elements of a slot
  static_assert((R - 1) * LOADS <= 63 && R >= 2, "ring");
  extern __shared__ __align__(16) unsigned char gr_smem[];

  const int tid = threadIdx.x, lane = tid & (BLM_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / BLM_WAVE);   // known to be the same in all lanes
  const int l32 = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.x * (MODE == 1 ? BN / 2 : BN);   // first output column
  if (MODE == 2 && !rope.store && n0 >= rope.nh * rope.hd) return;   // keys and values belong to another layer's cache
  const int k_begin = blockIdx.y * k_per_group, k_end = min(K, k_begin + k_per_group);
  // more rows than one block stages: blockIdx.z counts blocks of BM rows, each a product of its own
  const int m0 = blockIdx.z * BM;
  C += ((size_t)blockIdx.y * M + m0) * ldc;
  A += (size_t)m0 * lda;
  M = min(BM, M - m0);
  if (MODE == 2) {
    rope.positions += m0;
    rope.token_seq += m0;
  }
  bf16* ring = reinterpret_cast<bf16*>(gr_smem) + (size_t)wave * R * SLOT;

  // staging: lane l of a load instruction brings piece (l % P) ^ swizzle of row l / P of its RPL rows
  const int st_row = lane / P, st_slot = lane % P;
  const char* a_base = reinterpret_cast<const char*>(A);
  const char* b_base = reinterpret_cast<const char*>(W + (size_t)n0 * ldw);
  uint32_t a_off[A_LD], b_off[B_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int r = i * RPL + st_row;
    const int piece = st_slot ^ ((r / RPB) % P);
    a_off[i] = (uint32_t)(min(r, M - 1) * lda + piece * 8) * 2u;
  }
#pragma unroll
  for (int i = 0; i < B_LD; ++i) {
    const int r = i * RPL + st_row;
    const int piece = st_slot ^ ((r / RPB) % P);
    int n;
    if (MODE == 1) n = r < BN / 2 ? min(r, N - 1 - n0) : N + min(r - BN / 2, N - 1 - n0);
    else n = min(r, N - 1 - n0);
    b_off[i] = (uint32_t)(n * ldw + piece * 8) * 2u;
  }
  auto fetch = [&](int k0, int slot) {
    bf16* s = ring + slot * SLOT;
    const char* ab = a_base + (size_t)k0 * 2;
    const char* bb = b_base + (size_t)k0 * 2;
    if (k0 + BK <= k_end) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i) blm_dma16(ab, a_off[i], s + i * RPL * BK);
#pragma unroll
      for (int i = 0; i < B_LD; ++i) blm_dma16(bb, b_off[i], s + (BM + i * RPL) * BK);
    } else {
      // the last stage of a K that is no multiple of BK: pieces beyond the end come from a zero constant
      const char* zero_piece = reinterpret_cast<const char*>(gr_zero_piece);
#pragma unroll
      for (int i = 0; i < A_LD; ++i) {
        const int r = i * RPL + st_row;
        const bool in = k0 + (st_slot ^ ((r / RPB) % P)) * 8 < k_end;
        blm_dma16_lanes(in ? ab + a_off[i] : zero_piece, s + i * RPL * BK);
      }
#pragma unroll
      for (int i = 0; i < B_LD; ++i) {
        const int r = i * RPL + st_row;
        const bool in = k0 + (st_slot ^ ((r / RPB) % P)) * 8 < k_end;
        blm_dma16_lanes(in ? bb + b_off[i] : zero_piece, s + (BM + i * RPL) * BK);
      }
    }
  };

  // The weights are the first operand of the matrix instruction, the activations the second:
  // acc[i][j][e] is row 32 i + l32 of C and column 32 j + 8 (e / 4) + 4 lh + e % 4 of the block's columns.
  gr_f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  int a_row[TM], b_row[TN], k_off[QN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_row[i] = (i * 32 + l32) * BK;
#pragma unroll
  for (int j = 0; j < TN; ++j) b_row[j] = (BM + j * 32 + l32) * BK;
#pragma unroll
  for (int q = 0; q < QN; ++q) k_off[q] = ((2 * q + lh) ^ ((l32 / RPB) % P)) * 8;

  // this wavefront's stages: wave, wave + 4, ... of the block's n_stages
  const int n_stages = (k_end - k_begin + BK - 1) / BK;
  const int n_mine = n_stages > wave ? (n_stages - wave + NW - 1) / NW : 0;
  auto stage_k = [&](int i) { return k_begin + (wave + i * NW) * BK; };
#pragma unroll
  for (int s = 0; s < R; ++s)
    if (s < n_mine) fetch(stage_k(s), s);

  auto iteration = [&](int i, int slot, auto steady) {
    if (decltype(steady)::value) GR_WAIT_VM((R - 1) * LOADS);   // stage i has landed; the R - 1 behind it may be under way
    else GR_WAIT_VM(0);
    asm volatile("" ::: "memory");
    const bf16* s = ring + slot * SLOT;
    gr_bf16x8 af[QN][TM], bfr[QN][TN];
#pragma unroll
    for (int q = 0; q < QN; ++q) {
#pragma unroll
      for (int x = 0; x < TM; ++x) af[q][x] = *reinterpret_cast<const gr_bf16x8*>(s + a_row[x] + k_off[q]);
#pragma unroll
      for (int x = 0; x < TN; ++x) bfr[q][x] = *reinterpret_cast<const gr_bf16x8*>(s + b_row[x] + k_off[q]);
    }
    GR_WAIT_LGKM0();   // the fragments are in registers: the slot may take the next stage
    if (i + R < n_mine) fetch(stage_k(i + R), slot);
#pragma unroll
    for (int q = 0; q < QN; ++q)
#pragma unroll
      for (int x = 0; x < TM; ++x)
#pragma unroll
        for (int y = 0; y < TN; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[q][y], af[q][x], acc[x][y], 0, 0, 0);
  };
  int i = 0, slot = 0;
  for (; i + R <= n_mine; ++i, slot = slot + 1 == R ? 0 : slot + 1) iteration(i, slot, std::true_type{});
  for (; i < n_mine; ++i, slot = slot + 1 == R ? 0 : slot + 1) iteration(i, slot, std::false_type{});

  // The four partial tiles meet in shared memory (every wavefront's loads have landed: its last
  // iteration waited for all of them), are added in a fixed order and leave in 16-byte stores.
  __syncthreads();
  constexpr int OSTR = BN + 4;
  float* part = reinterpret_cast<float*>(gr_smem);   // [NW][BM][OSTR]
#pragma unroll
  for (int x = 0; x < TM; ++x)
#pragma unroll
    for (int y = 0; y < TN; ++y)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<float4*>(part + ((wave * BM + x * 32 + l32) * OSTR + y * 32 + 8 * g + 4 * lh)) =
            make_float4(acc[x][y][4 * g], acc[x][y][4 * g + 1], acc[x][y][4 * g + 2], acc[x][y][4 * g + 3]);
  __syncthreads();
  constexpr int ON = MODE == 1 ? BN / 2 : BN;   // output columns of the block
  constexpr int TPR = 256 / BM;                 // threads per row
  constexpr int CPT = ON / TPR;                 // columns per thread
  static_assert(CPT == 4 || CPT == 8 || CPT == 16, "columns per thread");
  const int row = tid / TPR, c0 = (tid % TPR) * CPT;
  if (row < M) {
    float v[CPT];
#pragma unroll
    for (int c = 0; c < CPT; c += 4) {
      float4 s = make_float4(0.f, 0.f, 0.f, 0.f), u = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float4 p = *reinterpret_cast<const float4*>(part + ((w * BM + row) * OSTR + c0 + c));
        s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
        if (MODE == 1) {
          const float4 q = *reinterpret_cast<const float4*>(part + ((w * BM + row) * OSTR + BN / 2 + c0 + c));
          u.x += q.x; u.y += q.y; u.z += q.z; u.w += q.w;
        }
      }
      if (MODE == 1) {
        v[c] = s.x / (1.0f + expf(-s.x)) * u.x;
        v[c + 1] = s.y / (1.0f + expf(-s.y)) * u.y;
        v[c + 2] = s.z / (1.0f + expf(-s.z)) * u.z;
        v[c + 3] = s.w / (1.0f + expf(-s.w)) * u.w;
      } else {
        v[c] = s.x; v[c + 1] = s.y; v[c + 2] = s.z; v[c + 3] = s.w;
      }
    }
    const int n = n0 + c0;
    if constexpr (MODE == 2) {
      const int pos = rope.positions[row], b = rope.token_seq[row];
      int page = -1;
      if (b >= 0 && rope.store) page = rope.block_table[(size_t)b * rope.table_width + pos / rope.page_size];
      const int slot = pos % rope.page_size, hd = rope.hd;
#pragma unroll
      for (int c = 0; c < CPT; c += 2) {
        const int nn = n + c;   // even; its partner nn + 1 is in the same head (head sizes are even)
        if (nn >= N) break;
        const int head = nn / hd, d = nn - head * hd;
        float y0 = v[c], y1 = v[c + 1];   // value heads are stored as they are
        if (head < rope.nh + rope.nkv) {
          const float2 cs = rope.cos_sin[(size_t)pos * (hd / 2) + (d >> 1)];
          y0 = v[c] * cs.x - v[c + 1] * cs.y;
          y1 = v[c] * cs.y + v[c + 1] * cs.x;
        }
        if (head < rope.nh) {
          *reinterpret_cast<uint32_t*>(C + (size_t)row * ldc + nn) = f32x2_to_bf16x2_bits(y0, y1);
        } else if (page >= 0) {
          if (head < rope.nh + rope.nkv) {
            *reinterpret_cast<uint32_t*>(rope.kcache + (((size_t)page * rope.nkv + (head - rope.nh)) * rope.page_size + slot) * hd + d) =
                f32x2_to_bf16x2_bits(y0, y1);
          } else {
            bf16* vp = rope.vcache + ((size_t)page * rope.nkv + (head - rope.nh - rope.nkv)) * hd * rope.page_size +
                       (size_t)d * rope.page_size + slot;
            vp[0] = from_float<bf16>(y0);
            vp[rope.page_size] = from_float<bf16>(y1);
          }
        }
      }
      return;
    }
    TC* dst = C + (size_t)row * ldc + n;
    constexpr int PER = sizeof(TC) == 2 ? 8 : 4;   // elements per 16-byte store
    if constexpr (CPT >= PER) {
#pragma unroll
      for (int c = 0; c < CPT; c += PER) {
        if (n + c + PER <= N && (reinterpret_cast<uintptr_t>(dst + c) & 15) == 0) {
          if constexpr (sizeof(TC) == 2)
            *reinterpret_cast<uint4*>(dst + c) = make_uint4(f32x2_to_bf16x2_bits(v[c], v[c + 1]), f32x2_to_bf16x2_bits(v[c + 2], v[c + 3]),
                                                            f32x2_to_bf16x2_bits(v[c + 4], v[c + 5]), f32x2_to_bf16x2_bits(v[c + 6], v[c + 7]));
          else
            *reinterpret_cast<float4*>(dst + c) = make_float4(v[c], v[c + 1], v[c + 2], v[c + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < PER; ++e)
            if (n + c + e < N) dst[c + e] = from_float<TC>(v[c + e]);
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < CPT; ++e)
        if (n + e < N) dst[e] = from_float<TC>(v[e]);
    }
  }
}

template <int BM, int BN, int BK, int R, int MODE, typename TC>
static int gr_prepare() {
  constexpr size_t smem = (size_t)4 * R * (BM + BN) * BK * sizeof(bf16);
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_rows_kernel<BM, BN, BK, R, MODE, TC>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
    return blm_fail("gemm_rows: %zu bytes of shared memory refused", smem);
  return 0;
}

template <int BM, int BN, int BK, int R, int MODE, typename TC>
static int gr_launch(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc, int k_groups,
                     hipStream_t stream, GrRope rope = GrRope{}) {
  constexpr size_t smem = (size_t)4 * R * (BM + BN) * BK * sizeof(bf16);
  static_assert(smem >= (size_t)4 * BM * (BN + 4) * sizeof(float), "the partial tiles fit where the ring was");
  const int n_tiles = (N + (MODE == 1 ? BN / 2 : BN) - 1) / (MODE == 1 ? BN / 2 : BN);
  const int k_per_group = ((K + k_groups - 1) / k_groups + BK - 1) / BK * BK;
  dim3 grid((unsigned)n_tiles, (unsigned)k_groups, (unsigned)((M + BM - 1) / BM)), block(256);
  hipLaunchKernelGGL((gemm_rows_kernel<BM, BN, BK, R, MODE, TC>), grid, block, smem, stream, (const bf16*)A, (const bf16*)W, (TC*)C, M,
                     N, K, lda, ldw, ldc, k_per_group, rope);
  BLM_LAUNCH_CHECK("gemm_rows");
  return 0;
}

// Lets the kernels use more than 64 KiB of shared memory; to be called once per device before the first
// product (not from inside a stream capture).
extern "C" int blm_gemm_rows_init() {
#define GR_PREP(BM, BN, R, MODE) \
  if (gr_prepare<BM, BN, 64, R, MODE, bf16>() || gr_prepare<BM, BN, 64, R, MODE, float>()) return 1;
  GR_PREP(64, 64, 2, 0) GR_PREP(64, 32, 3, 0) GR_PREP(32, 64, 3, 0) GR_PREP(32, 32, 5, 0)
  GR_PREP(64, 64, 2, 1) GR_PREP(32, 64, 3, 1)
#undef GR_PREP
  if (gr_prepare<64, 32, 64, 3, 2, bf16>() || gr_prepare<32, 32, 64, 5, 2, bf16>() || gr_prepare<64, 64, 64, 2, 2, bf16>()) return 1;
  return 0;
}

// columns: 64 (a ring of two stages per wavefront) or 32 (a ring of three) per block; with mode 1 they
// are gate and up columns together.  Measured at 17 to 64 rows against the packed skinny product: ahead
// for the gated product from 33 rows on and for partial planes (32 columns when that still gives every
// compute unit a block, else 64) at all of them.
extern "C" int blm_gemm_rows(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc,
                             int mode, int k_groups, int columns, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && M <= GR_MAX_ROWS && N >= 1 && K >= 8 && K % 8 == 0,
              "gemm_rows: sizes M=%d N=%d K=%d not supported (M <= %d, K a multiple of 8)", M, N, K, GR_MAX_ROWS);
  BLM_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= N, "gemm_rows: bad strides lda=%d ldw=%d ldc=%d", lda, ldw, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_rows: operands must be 16-byte aligned");
  BLM_REQUIRE(columns == 64 || (columns == 32 && mode == 0), "gemm_rows: %d columns per block: 64, or 32 without gating", columns);
  BLM_REQUIRE(mode == 0 || (mode == 1 && k_groups == 1), "gemm_rows: mode %d needs one K group", mode);
  BLM_REQUIRE(k_groups >= 1 && k_groups <= 64 && (k_groups == 1 || c_dtype == BLM_F32),
              "gemm_rows: k_groups=%d needs 1..64 and a float output when above 1", k_groups);
  BLM_REQUIRE(c_dtype == BLM_BF16 || c_dtype == BLM_F32, "gemm_rows: unsupported output dtype %d", c_dtype);
  BLM_REQUIRE((size_t)64 * lda * 2 < ((size_t)1 << 32) && (size_t)(mode == 1 ? 2 : 1) * N * ldw * 2 < ((size_t)1 << 32),
              "gemm_rows: matrices of 4 GiB and more are not supported (lda=%d, N=%d, ldw=%d)", lda, N, ldw);
#define GR_GO(BM, BN, R, MODE)                                                                                       \
  return c_dtype == BLM_BF16 ? gr_launch<BM, BN, 64, R, MODE, bf16>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream) \
                             : gr_launch<BM, BN, 64, R, MODE, float>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream)
  // up to 32 rows: half the rows staged, and a deeper ring in the room that leaves
  if (mode == 1) {
    if (M > 32) GR_GO(64, 64, 2, 1);
    GR_GO(32, 64, 3, 1);
  }
  if (columns == 64) {
    if (M > 32) GR_GO(64, 64, 2, 0);
    GR_GO(32, 64, 3, 0);
  }
  if (M > 32) GR_GO(64, 32, 3, 0);
  GR_GO(32, 32, 5, 0);
#undef GR_GO
}

// The q/k/v projection of 17 to 256 rows with the rotation and the cache write where the partial tiles meet
// (columns: 32 per block, or 64 with 64 rows staged and a ring of two, for shapes whose blocks of 32 columns
// would not all run at once; rows: 64 staged per block, or 32 with a deeper ring, which up to 32 rows is what
// runs anyway and above makes twice the blocks).  W: W_qkv [(nh + 2 nkv) * hd, K] with rotary partners in adjacent rows; qkv_out:
// [M, ldq] bf16, of which only the first nh * hd columns (the rotated queries) are written; key plane
// [pages, nkv, page, hd], value plane [pages, nkv, hd, page].  store = 0: keys and values are neither
// computed nor written.
extern "C" int blm_gemm_rows_qkv_rope(const void* A, const void* W, void* qkv_out, const int* positions, const int* token_seq,
                                      const int* block_table, int table_width, const float* cos_sin, void* kcache, void* vcache,
                                      int page_size, int M, int K, int lda, int ldw, int ldq, int nh, int nkv, int hd, int store,
                                      int columns, int rows, hipStream_t stream) {
  BLM_REQUIRE(columns == 32 || columns == 64, "gemm_rows_qkv_rope: %d columns per block: 32 or 64", columns);
  BLM_REQUIRE(rows == 64 || (rows == 32 && columns == 32), "gemm_rows_qkv_rope: %d rows per block: 64, or 32 with 32 columns", rows);
  BLM_REQUIRE(M >= 1 && M <= GR_MAX_ROWS && K >= 8 && K % 8 == 0 && hd >= 2 && hd % 2 == 0,
              "gemm_rows_qkv_rope: M=%d K=%d head_dim=%d not supported (M <= %d, K a multiple of 8, an even head size)", M, K, hd,
              GR_MAX_ROWS);
  BLM_REQUIRE(nh > 0 && nkv > 0 && page_size > 0 && table_width > 0, "gemm_rows_qkv_rope: bad geometry");
  BLM_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldq >= nh * hd && ldq % 2 == 0,
              "gemm_rows_qkv_rope: bad strides lda=%d ldw=%d ldq=%d", lda, ldw, ldq);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)qkv_out % 4) == 0 && ((uintptr_t)kcache % 4) == 0,
              "gemm_rows_qkv_rope: operands must be 16-byte aligned (outputs 4-byte)");
  const int N = (nh + 2 * nkv) * hd;
  BLM_REQUIRE((size_t)64 * lda * 2 < ((size_t)1 << 32) && (size_t)N * ldw * 2 < ((size_t)1 << 32),
              "gemm_rows_qkv_rope: matrices of 4 GiB and more are not supported");
  const GrRope rope{positions, token_seq, block_table, (const float2*)cos_sin, (bf16*)kcache, (bf16*)vcache,
                    table_width, page_size, nh, nkv, hd, store};
  if (columns == 64) return gr_launch<64, 64, 64, 2, 2, bf16>(A, W, qkv_out, M, N, K, lda, ldw, ldq, 1, stream, rope);
  if (M > 32 && rows != 32) return gr_launch<64, 32, 64, 3, 2, bf16>(A, W, qkv_out, M, N, K, lda, ldw, ldq, 1, stream, rope);
  return gr_launch<32, 32, 64, 5, 2, bf16>(A, W, qkv_out, M, N, K, lda, ldw, ldq, 1, stream, rope);
}
