// Matrix product for many rows (prefill) on the matrix cores: C[M, N] = A[M, K] * W[N, K]^T, bf16
// operands, float accumulation, bf16 or float output.
//
// A block of four or eight wavefronts owns a BM x BN tile of C and walks K in stages of BK.  Both operands
// are rows of consecutive k (the weight matrix is used as the checkpoint stores it), so their
// tiles are staged the same way: 16 bytes per lane from global memory straight into a ring of NS
// shared-memory buffers (no registers in between), NS - 1 stages ahead of the multiplications: a
// load takes longer than a stage's multiplications, and one or two wavefronts per SIMD have little
// else to hide it behind.  (The loads are inline assembly, see blm_dma16 in common.h.)  The pieces of
// a staged row are permuted so that a fragment read meets every bank once.  A wavefront owns its
// part of the tile as 32x32 accumulators of the 32x32x16 instruction; per k-step of 16 it reads one
// fragment per 32 rows and per 32 columns and multiplies every pair.
//
// mode 1: W holds gate rows [0, I) and up rows [I, 2I) of a gated feed-forward; a block takes
// BN / 2 gate columns and the matching up columns, each wavefront both halves of its pairs, and
// C[M, I] = silu(gate) * up leaves the accumulators directly.
// k_groups > 1: K is cut into groups, C is float [k_groups, M, ldc] with one partial product each
// (summed by the reader), so that a narrow output still fills the chip.
#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;


// 16 zero bytes for the pieces that lie beyond the end of K
__device__ __align__(16) const uint32_t gm_zero_piece[4] = {0u, 0u, 0u, 0u};

// s_waitcnt immediates of gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8
#define GM_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#define GM_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)


// scheduling hints: the next `n` instructions of a kind, in the order the hints are given
#define GM_SCHED_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, n, 0)
#define GM_SCHED_VMEM(n) __builtin_amdgcn_sched_group_barrier(0x020, n, 0)
#define GM_SCHED_DSREAD(n) __builtin_amdgcn_sched_group_barrier(0x100, n, 0)

// x * sigmoid(x) with the hardware's exponential and reciprocal (each within an ulp; the result is
// rounded to bf16 afterwards): 128 of these per lane would otherwise cost as much as 6 % of a tile
__device__ __forceinline__ float gm_silu(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// columns per pass of the epilogue: as many of a wavefront's `on` as the staging of all `waves` leaves room for
constexpr int gm_pass_columns(int on, int waves, size_t bytes) {
  int cw = on;
  while (cw >= 32 && (size_t)waves * 32 * (cw + 4) * sizeof(float) > bytes) cw /= 2;
  return cw;
}

template <int BM, int BN, int BK, int NS, int WGM, int WGN, int MODE, typename TC>
__global__ void __launch_bounds__(WGM* WGN* BLM_WAVE)
    gemm_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C, int M, int N, int K,
                     int lda, int ldw, int ldc, int m_tiles, int n_tiles, int k_per_group) {
  constexpr int NW = WGM * WGN;                   // wavefronts, WGM along M and WGN along N
  constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  static_assert(WM % 32 == 0 && WN % 32 == 0 && (MODE == 0 || TN % 2 == 0), "wavefront tile");
  static_assert(BK == 32 || BK == 64, "stage depth");
  constexpr int P = BK / 8;                       // 16-byte pieces per staged row
  constexpr int RPL = 64 / P;                     // rows that one load instruction of a wavefront fills
  constexpr int RPB = 256 / (BK * 2);             // staged rows per 256 bytes (one pass over the banks)
  constexpr int A_LD = BM / RPL / NW, B_LD = BN / RPL / NW;   // loads per wavefront and stage
  constexpr int LOADS = A_LD + B_LD;
  static_assert(A_LD >= 1 && B_LD >= 1 && (NS - 1) * LOADS <= 63 && NS >= 2, "staging");
  constexpr int QN = BK / 16;                     // k-steps of the matrix instruction per stage
  constexpr int REST = TM * TN - (TM + TN) > 0 ? TM * TN - (TM + TN) : 0;   // multiplications behind a k-step's reads
  constexpr int VM_PER = REST > 0 ? (LOADS + REST - 1) / REST : LOADS;
  extern __shared__ __align__(16) unsigned char gm_smem[];
  bf16* As = reinterpret_cast<bf16*>(gm_smem);    // [NS][BM][BK]
  bf16* Bs = As + NS * BM * BK;                   // [NS][BN][BK]

  const int tid = threadIdx.x, wave = tid / BLM_WAVE, lane = tid & (BLM_WAVE - 1);
  const int l32 = lane & 31, lh = lane >> 5;
  const int wm = wave / WGN, wn = wave % WGN;

  // tile of this block: neighbouring blocks go to different dies, so each die gets a run of tiles
  // of its own (M fastest: the blocks that run together on a die share a few column tiles of W
  // and all of A)
  int t = blockIdx.x;
  const int total = gridDim.x;
  if (total % 8 == 0) t = (t & 7) * (total >> 3) + (t >> 3);
  const int tm = t % m_tiles, tn = t / m_tiles;
  const int m0 = tm * BM;
  const int n0 = tn * (MODE == 1 ? BN / 2 : BN);   // first output column
  const int k_begin = blockIdx.y * k_per_group, k_end = min(K, k_begin + k_per_group);
  C += (size_t)blockIdx.y * M * ldc;

  // Staging: one load instruction moves 16 bytes per lane from global memory straight into shared
  // memory, lane l to base + 16 l, so a wavefront's load fills RPL staged rows.  Staged rows are
  // not padded; instead slot s of row r holds the row's piece s ^ ((r / RPB) % P), which spreads
  // the 16 rows of a fragment read over all banks.  Rows beyond the matrices are clamped into them
  // (their results are dropped), pieces beyond K come from a zero constant.  A load's address is a
  // base that is the same for all lanes and moves with k, plus a per-lane byte offset that never
  // changes.
  const int st_row = lane / P, st_slot = lane % P;
  const char* a_base = reinterpret_cast<const char*>(A + (size_t)m0 * lda);
  const char* b_base = reinterpret_cast<const char*>(W + (size_t)n0 * ldw);
  uint32_t a_off[A_LD], b_off[B_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int r = (wave * A_LD + i) * RPL + st_row;
    const int piece = st_slot ^ ((r / RPB) % P);
    a_off[i] = (uint32_t)(min(r, M - 1 - m0) * lda + piece * 8) * 2u;
  }
#pragma unroll
  for (int i = 0; i < B_LD; ++i) {
    const int r = (wave * B_LD + i) * RPL + st_row;
    const int piece = st_slot ^ ((r / RPB) % P);
    int n;   // row of W relative to n0
    if (MODE == 1) n = r < BN / 2 ? min(r, N - 1 - n0) : N + min(r - BN / 2, N - 1 - n0);
    else n = min(r, N - 1 - n0);
    b_off[i] = (uint32_t)(n * ldw + piece * 8) * 2u;
  }
  auto fetch_whole = [&](int k0, int buf) {
    const char* ab = a_base + (size_t)k0 * 2;
    const char* bb = b_base + (size_t)k0 * 2;
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      blm_dma16(ab, a_off[i], As + (buf * BM + (wave * A_LD + i) * RPL) * BK);
#pragma unroll
    for (int i = 0; i < B_LD; ++i)
      blm_dma16(bb, b_off[i], Bs + (buf * BN + (wave * B_LD + i) * RPL) * BK);
  };
  auto fetch = [&](int k0, int buf) {
    if (k0 + BK <= k_end) {
      fetch_whole(k0, buf);
      return;
    }
    // the last stage of a K that is no multiple of BK
    const char* ab = a_base + (size_t)k0 * 2;
    const char* bb = b_base + (size_t)k0 * 2;
    const char* zero_piece = reinterpret_cast<const char*>(gm_zero_piece);
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int r = (wave * A_LD + i) * RPL + st_row;
      const bool in = k0 + (st_slot ^ ((r / RPB) % P)) * 8 < k_end;
      blm_dma16_lanes(in ? ab + a_off[i] : zero_piece, As + (buf * BM + (wave * A_LD + i) * RPL) * BK);
    }
#pragma unroll
    for (int i = 0; i < B_LD; ++i) {
      const int r = (wave * B_LD + i) * RPL + st_row;
      const bool in = k0 + (st_slot ^ ((r / RPB) % P)) * 8 < k_end;
      blm_dma16_lanes(in ? bb + b_off[i] : zero_piece, Bs + (buf * BN + (wave * B_LD + i) * RPL) * BK);
    }
  };

  // The weights are the first operand of the matrix instruction and the activations the second, so
  // a 32x32 accumulator holds C transposed: acc[i][j][e] is row (of C) l32 and column
  // 8 * (e / 4) + 4 * lh + e % 4 of its tile: four neighbouring columns per lane and e / 4.
  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // fragments: lane (l32, lh) reads row base + l32, k = 16 q + 8 lh .. + 8 of the stage, which is
  // slot (2 q + lh) ^ ((l32 / RPB) % P) of the staged row (every base is a multiple of 32)
  int a_row[TM], b_row[TN], k_off[QN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_row[i] = (wm * WM + i * 32 + l32) * BK;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int r;
    if (MODE == 1) r = (j < TN / 2 ? 0 : BN / 2) + wn * (WN / 2) + (j % (TN / 2)) * 32;
    else r = wn * WN + j * 32;
    b_row[j] = (r + l32) * BK;
  }
#pragma unroll
  for (int q = 0; q < QN; ++q) k_off[q] = ((2 * q + lh) ^ ((l32 / RPB) % P)) * 8;

  bf16x8_t af[2][TM], bfr[2][TN];
  auto fragments = [&](int buf, int q, int set) {
    const bf16* as = As + buf * BM * BK + k_off[q];
    const bf16* bs = Bs + buf * BN * BK + k_off[q];
    // in the order in which multiply() first needs them
#pragma unroll
    for (int x = 0; x < (TM > TN ? TM : TN); ++x) {
      if (x < TM) af[set][x] = *reinterpret_cast<const bf16x8_t*>(as + a_row[x]);
      if (x < TN) bfr[set][x] = *reinterpret_cast<const bf16x8_t*>(bs + b_row[x]);
    }
  };
  // pairs in the order of growing max(i, j), so that the first ones need only the first fragments
  auto multiply = [&](int set) {
#pragma unroll
    for (int d = 0; d < (TM > TN ? TM : TN); ++d) {
#pragma unroll
      for (int j = 0; j < d && j < TN; ++j)
        if (d < TM) acc[d][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[set][j], af[set][d], acc[d][j], 0, 0, 0);
#pragma unroll
      for (int i = 0; i <= d && i < TM; ++i)
        if (d < TN) acc[i][d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[set][d], af[set][i], acc[i][d], 0, 0, 0);
    }
  };

  // Iteration s multiplies stage s out of buffer s % NS.  Its one barrier comes when every wavefront
  // has taken its last fragments of stage s, so the loads of stage s + NS may overwrite that buffer
  // right after it; the same barrier makes stage s + 1 (asked for NS - 1 iterations earlier)
  // visible.  The last k-step of a stage is multiplied after the barrier, over the new loads and
  // the first fragment reads of the next stage.  With one wavefront per SIMD nothing else hides a
  // latency, so the order of issue is prescribed: matrix instructions with the reads and loads
  // spread between them.  (Loads issued in front of the barrier instead, spread over the k-steps of
  // the following iteration, measured 20 % slower.)
  // `steady`: stage s + NS exists and is a whole one, so the part after the barrier has no branch.
  const int n_stages = (k_end - k_begin + BK - 1) / BK;
  auto iteration = [&](int s, int buf, auto steady) {
#pragma unroll
    for (int q = 0; q < QN - 1; ++q) {
      fragments(buf, q + 1, (q + 1) & 1);
      multiply(q & 1);
#pragma unroll
      for (int x = 0; x < (TM + TN < TM * TN ? TM + TN : TM * TN); ++x) {
        GM_SCHED_MFMA(1);
        GM_SCHED_DSREAD((TM + TN + TM * TN - 1) / (TM * TN));
      }
      if (REST > 0) GM_SCHED_MFMA(REST);
    }
    GM_WAIT_LGKM0();   // the last fragments are in registers: the stage may be overwritten
    if (decltype(steady)::value) GM_WAIT_VM((NS - 2) * LOADS);   // this wavefront's part of stage s + 1 has arrived
    else GM_WAIT_VM(0);
    __syncthreads();
    const int next = buf + 1 == NS ? 0 : buf + 1;
    if (decltype(steady)::value) {
      fetch_whole(k_begin + (s + NS) * BK, buf);
      fragments(next, 0, 0);
      multiply((QN - 1) & 1);
#pragma unroll
      for (int x = 0; x < (TM + TN < TM * TN ? TM + TN : TM * TN); ++x) {
        GM_SCHED_MFMA(1);
        GM_SCHED_DSREAD((TM + TN + TM * TN - 1) / (TM * TN));
      }
#pragma unroll
      for (int x = 0; x < REST; ++x) {
        GM_SCHED_MFMA(1);
        GM_SCHED_VMEM(VM_PER);
      }
    } else {
      if (s + NS < n_stages) fetch(k_begin + (s + NS) * BK, buf);
      if (s + 1 < n_stages) fragments(next, 0, 0);
      multiply((QN - 1) & 1);
    }
  };
#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < n_stages) fetch(k_begin + s * BK, s);
  if (NS - 1 < n_stages) {
    fetch(k_begin + (NS - 1) * BK, NS - 1);
    GM_WAIT_VM((NS - 1) * LOADS);
  } else {
    GM_WAIT_VM(0);
  }
  __syncthreads();
  fragments(0, 0, 0);
  const int n_steady = max(0, (k_end - k_begin) / BK - NS);   // whole stages, less those that are ahead
  int s = 0, buf = 0;
  for (; s < n_steady; ++s, buf = buf + 1 == NS ? 0 : buf + 1) iteration(s, buf, std::true_type{});
  for (; s < n_stages; ++s, buf = buf + 1 == NS ? 0 : buf + 1) iteration(s, buf, std::false_type{});

  // Results leave through shared memory, 32 rows and CW columns at a time per wavefront, so that
  // every store writes 16 bytes per lane and runs of whole lines per row.
  __syncthreads();
  constexpr int ON = MODE == 1 ? WN / 2 : WN;           // output columns of a wavefront
  constexpr int CW = gm_pass_columns(ON, NW, (size_t)NS * (BM + BN) * BK * sizeof(bf16));
  static_assert(CW >= 32, "output staging fits");
  constexpr int OSTR = CW + 4;                          // floats per staged row
  float* stage_out = reinterpret_cast<float*>(gm_smem) + wave * 32 * OSTR;
  constexpr int PER = sizeof(TC) == 2 ? 8 : 4;          // elements per 16-byte store
  const int out_n0 = n0 + wn * ON;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int c0 = 0; c0 < ON; c0 += CW) {
#pragma unroll
      for (int jj = 0; jj < CW / 32; ++jj) {
        const int j = c0 / 32 + jj;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float4 v;
          if (MODE == 1) {
            float4 gt = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
            float4 up = make_float4(acc[i][j + TN / 2][4 * g], acc[i][j + TN / 2][4 * g + 1],
                                    acc[i][j + TN / 2][4 * g + 2], acc[i][j + TN / 2][4 * g + 3]);
            v = make_float4(gm_silu(gt.x) * up.x, gm_silu(gt.y) * up.y, gm_silu(gt.z) * up.z, gm_silu(gt.w) * up.w);
          } else {
            v = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
          }
          *reinterpret_cast<float4*>(stage_out + l32 * OSTR + jj * 32 + 8 * g + 4 * lh) = v;
        }
      }
      // the wavefront reads back what it wrote itself: no barrier, the compiler orders the accesses
      const int m_base = m0 + wm * WM + i * 32;
      constexpr int LANES_PER_ROW = CW / PER;
#pragma unroll
      for (int x = 0; x < 32 * LANES_PER_ROW / BLM_WAVE; ++x) {
        const int idx = x * BLM_WAVE + lane;
        const int r = idx / LANES_PER_ROW, c = (idx % LANES_PER_ROW) * PER;
        const int m = m_base + r, n = out_n0 + c0 + c;
        const float* src = stage_out + r * OSTR + c;
        if (m < M && n < N) {
          TC* dst = C + (size_t)m * ldc + n;
          const bool vec = n + PER <= N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
          const float4 lo = *reinterpret_cast<const float4*>(src);
          if (sizeof(TC) == 2) {
            const float4 hi = *reinterpret_cast<const float4*>(src + 4);
            if (vec) {
              *reinterpret_cast<uint4*>(dst) = make_uint4(f32x2_to_bf16x2_bits(lo.x, lo.y), f32x2_to_bf16x2_bits(lo.z, lo.w),
                                                          f32x2_to_bf16x2_bits(hi.x, hi.y), f32x2_to_bf16x2_bits(hi.z, hi.w));
            } else {
              // a row end that is no multiple of 8, or a row that starts off a 16-byte boundary
              dst[0] = from_float<TC>(lo.x);
              if (n + 1 < N) dst[1] = from_float<TC>(lo.y);
              if (n + 2 < N) dst[2] = from_float<TC>(lo.z);
              if (n + 3 < N) dst[3] = from_float<TC>(lo.w);
              if (n + 4 < N) dst[4] = from_float<TC>(hi.x);
              if (n + 5 < N) dst[5] = from_float<TC>(hi.y);
              if (n + 6 < N) dst[6] = from_float<TC>(hi.z);
              if (n + 7 < N) dst[7] = from_float<TC>(hi.w);
            }
          } else {
            if (vec) {
              *reinterpret_cast<float4*>(dst) = lo;
            } else {
              dst[0] = from_float<TC>(lo.x);
              if (n + 1 < N) dst[1] = from_float<TC>(lo.y);
              if (n + 2 < N) dst[2] = from_float<TC>(lo.z);
              if (n + 3 < N) dst[3] = from_float<TC>(lo.w);
            }
          }
        }
      }
    }
  }
}

template <int BM, int BN, int BK, int NS, int WGM, int WGN, int MODE, typename TC>
static int prepare_gemm() {
  constexpr size_t smem = (size_t)NS * (BM + BN) * BK * sizeof(bf16);
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_mfma_kernel<BM, BN, BK, NS, WGM, WGN, MODE, TC>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
    return blm_fail("gemm_mfma: %zu bytes of shared memory refused", smem);
  return 0;
}

template <int BM, int BN, int BK, int NS, int WGM, int WGN, int MODE, typename TC>
static int launch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                       int k_groups, hipStream_t stream) {
  constexpr size_t smem = (size_t)NS * (BM + BN) * BK * sizeof(bf16);
  const int m_tiles = (M + BM - 1) / BM;
  const int n_tiles = (N + (MODE == 1 ? BN / 2 : BN) - 1) / (MODE == 1 ? BN / 2 : BN);
  const int k_per_group = ((K + k_groups - 1) / k_groups + BK - 1) / BK * BK;
  dim3 grid((unsigned)(m_tiles * n_tiles), (unsigned)k_groups), block(WGM * WGN * BLM_WAVE);
  hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, BK, NS, WGM, WGN, MODE, TC>), grid, block, smem, stream, (const bf16*)A,
                     (const bf16*)W, (TC*)C, M, N, K, lda, ldw, ldc, m_tiles, n_tiles, k_per_group);
  BLM_LAUNCH_CHECK("gemm_mfma");
  return 0;
}

#define BLM_GEMM_TILES(X) X(128, 128, 64, 2, 2, 2) X(256, 128, 64, 3, 4, 2) X(256, 256, 64, 2, 4, 2) X(128, 128, 64, 4, 2, 2) X(128, 64, 64, 6, 4, 1)

// Lets every variant use more than 64 KiB of shared memory; to be called once per device before the
// first product (not from inside a stream capture).
extern "C" int blm_gemm_mfma_init() {
#define BLM_PREP(BM, BN, BK, NS, WGM, WGN)                                                                     \
  if (prepare_gemm<BM, BN, BK, NS, WGM, WGN, 0, bf16>() || prepare_gemm<BM, BN, BK, NS, WGM, WGN, 0, float>() ||       \
      prepare_gemm<BM, BN, BK, NS, WGM, WGN, 1, bf16>() || prepare_gemm<BM, BN, BK, NS, WGM, WGN, 1, float>())         \
    return 1;
  BLM_GEMM_TILES(BLM_PREP)
#undef BLM_PREP
  return 0;
}

// tile: rows x columns of C per block: 0 = 128x128 (four wavefronts, several blocks per compute unit),
// 1 = 256x128 and 2 = 256x256 (eight wavefronts: two per SIMD, so that one issues matrix instructions
// while the other issues loads or waits; 10 % faster than four wavefronts with twice the tile each,
// sixteen are no faster; each of the eight owns 64 rows x 128 columns, 2 % faster than 128 x 64).
// 3 = 128x128 with a ring of four stages and 4 = 128x64 with six (four wavefronts, one block per
// compute unit): for products of so few tiles that all run at once, where a block waits for memory
// and not for the matrix cores; a single 128x128 tile walks K = 2048 in 21 us with two stages and
// in 19 us with four, a 128x64 tile in 15 us with six.
// K in stages of 64, two of them in shared memory, three for 256x128;
// stages of 32 in deeper rings were not faster.  Measured at 256 to 4,096 rows: the largest tile
// that still gives every compute unit a block is the fastest.
// mode 0: C[M, N] = A W^T, W [N, K].  mode 1: W [2N, K] = [gate rows; up rows], C[M, N] = silu(gate) * up.
extern "C" int blm_gemm_mfma(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldw, int ldc, int mode, int k_groups, int tile, hipStream_t stream) {
  BLM_REQUIRE(M >= 1 && N >= 1 && K >= 8 && K % 8 == 0, "gemm_mfma: sizes M=%d N=%d K=%d not supported (K a multiple of 8)",
              M, N, K);
  BLM_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= N, "gemm_mfma: bad strides lda=%d ldw=%d ldc=%d",
              lda, ldw, ldc);
  BLM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_mfma: operands must be 16-byte aligned");
  BLM_REQUIRE(mode == 0 || (mode == 1 && k_groups == 1), "gemm_mfma: mode %d needs one K group", mode);
  BLM_REQUIRE(k_groups >= 1 && k_groups <= 64 && (k_groups == 1 || c_dtype == BLM_F32),
              "gemm_mfma: k_groups=%d needs 1..64 and a float output when above 1", k_groups);
  BLM_REQUIRE(c_dtype == BLM_BF16 || c_dtype == BLM_F32, "gemm_mfma: unsupported output dtype %d", c_dtype);
  // per-lane byte offsets into a tile's rows are 32-bit
  BLM_REQUIRE((size_t)256 * lda * 2 < ((size_t)1 << 32) && (size_t)(mode == 1 ? 2 : 1) * N * ldw * 2 < ((size_t)1 << 32),
              "gemm_mfma: matrices of 4 GiB and more are not supported (lda=%d, N=%d, ldw=%d)", lda, N, ldw);
#define BLM_GEMM(BM, BN, BK, NS, WGM, WGN)                                                                           \
  do {                                                                                                               \
    if (mode == 1)                                                                                                   \
      return c_dtype == BLM_BF16                                                                                     \
                 ? launch_gemm<BM, BN, BK, NS, WGM, WGN, 1, bf16>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream) \
                 : launch_gemm<BM, BN, BK, NS, WGM, WGN, 1, float>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream); \
    return c_dtype == BLM_BF16                                                                                       \
               ? launch_gemm<BM, BN, BK, NS, WGM, WGN, 0, bf16>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream)   \
               : launch_gemm<BM, BN, BK, NS, WGM, WGN, 0, float>(A, W, C, M, N, K, lda, ldw, ldc, k_groups, stream); \
  } while (0)
  switch (tile) {
    case 0: BLM_GEMM(128, 128, 64, 2, 2, 2);
    case 1: BLM_GEMM(256, 128, 64, 3, 4, 2);
    case 2: BLM_GEMM(256, 256, 64, 2, 4, 2);
    case 3: BLM_GEMM(128, 128, 64, 4, 2, 2);
    case 4: BLM_GEMM(128, 64, 64, 6, 4, 1);
  }
#undef BLM_GEMM
  return blm_fail("gemm_mfma: tile %d out of range 0..4", tile);
}
