// bf16 matrix products on the matrix cores with float32 accumulation.
//
// stream (below, second): the weight-streaming product for M <= 64 that decode uses.
// skinny (first): an older, simpler form that reads MFMA operands straight from
// memory; kept as the fallback for shapes the streaming kernel refuses.
//
// skinny:  C[M,N] = A[M,K] * W[N,K]^T for few rows M (decode batches, M <= 64).
// The step is bound by reading W once, so the kernel is laid out around the
// weight stream: a block owns 16*NT weight rows; its waves split K between them
// and each wave streams its share of those rows straight from memory into MFMA
// A operands (v_mfma_f32_16x16x32_bf16: lane (r, kb) holds W[row r][k + kb*8 .. +8],
// one 16-byte load), multiplies by the activation fragments (B operands, read
// from L1/L2) and keeps D[weight row][batch row] in registers.  At the end the
// waves' partial sums are added in wave order through LDS (a fixed order, so
// the result is deterministic) and written as bf16 or float32.
#include "common.h"
#include "slots.h"

using namespace tk;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // arrays of HIP's uint4 struct end up in scratch

union Frag8 {
  uint4 u;
  bf16x8 v;
};

template <int NT, int MT, int WAVES, typename TO>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TO* __restrict__ C, int M, int N,
    int K, long lda, long ldw, long ldc) {
  __shared__ float red[(WAVES > 1 ? WAVES - 1 : 1) * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);

  // this wave's share of K, in steps of 32
  const int steps = (K + 31) / 32;
  const int per = (steps + WAVES - 1) / WAVES;
  const int s_begin = wave * per;
  const int s_end = min(steps, s_begin + per);

  // Row pointers are clamped into the matrix: rows past N (or M) are computed from a
  // valid row's data and never stored, so the loads need no predicate.
  const bf16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) wp[t] = W + (size_t)min(n0 + t * 16 + r, N - 1) * ldw + kb * 8;
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) ap[t] = A + (size_t)min(t * 16 + r, M - 1) * lda + kb * 8;

  float4v acc[NT][MT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // whole steps (all 32 k inside K), UNR at a time: every load of a group is issued
  // before the first product, so a wave keeps UNR*(NT+MT) 16-byte loads in flight
  constexpr int UNR = (NT * MT >= 4) ? 2 : 4;
  const int s_whole = min(s_end, K / 32);
  int s = s_begin;
  for (; s + UNR <= s_whole; s += UNR) {
    Frag8 wf[UNR][NT], af[UNR][MT];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
#pragma unroll
      for (int t = 0; t < NT; ++t) wf[u][t].u = *reinterpret_cast<const uint4*>(wp[t] + (s + u) * 32);
#pragma unroll
      for (int t = 0; t < MT; ++t) af[u][t].u = *reinterpret_cast<const uint4*>(ap[t] + (s + u) * 32);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u)
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][i].v, af[u][j].v, acc[i][j], 0, 0, 0);
  }
  // leftover steps, the last of which may reach past K (K is a multiple of 8, so a
  // 16-byte piece is whole or absent; an absent piece is read at k = 0 and zeroed)
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (; s < s_end; ++s) {
    const bool kok = s * 32 + kb * 8 < K;
    const int koff = kok ? s * 32 : -kb * 8;
    Frag8 wf[NT], af[MT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint4 v = *reinterpret_cast<const uint4*>(wp[t] + koff);
      wf[t].u = kok ? v : zero;
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const uint4 v = *reinterpret_cast<const uint4*>(ap[t] + koff);
      af[t].u = kok ? v : zero;
    }
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, af[j].v, acc[i][j], 0, 0, 0);
  }

  // add the waves' partial sums in wave order, one accumulator tile at a time
  if (WAVES > 1) {
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        if (wave > 0)
          *reinterpret_cast<float4*>(red + (size_t)(wave - 1) * 256 + lane * 4) =
              make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
        __syncthreads();
        if (wave == 0) {
          for (int w = 0; w < WAVES - 1; ++w) {
            const float4 v = *reinterpret_cast<const float4*>(red + (size_t)w * 256 + lane * 4);
            acc[i][j][0] += v.x;
            acc[i][j][1] += v.y;
            acc[i][j][2] += v.z;
            acc[i][j][3] += v.w;
          }
        }
        __syncthreads();
      }
    if (wave > 0) return;
  }

  // acc[i][j][e] = C[batch row j*16 + r][weight row n0 + i*16 + kb*4 + e]
  const bool wide = rows_take_wide_stores(C, ldc);
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = j * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int n = n0 + i * 16 + kb * 4;
      store_four<TO>(C + (size_t)m * ldc + n, acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3], N - n, wide);
    }
  }
}

template <int NT, int MT, int WAVES, typename TO>
static int launch_skinny(const void* A, const void* W, void* C, int M, int N, int K, long lda,
                         long ldw, long ldc, hipStream_t stream) {
  const int blocks = (N + 16 * NT - 1) / (16 * NT);
  gemm_skinny_kernel<NT, MT, WAVES, TO><<<blocks, WAVES * 64, 0, stream>>>(
      (const bf16_t*)A, (const bf16_t*)W, (TO*)C, M, N, K, lda, ldw, ldc);
  return launch_status();
}

template <int NT, int MT, typename TO>
static int pick_waves(int waves, const void* A, const void* W, void* C, int M, int N, int K,
                      long lda, long ldw, long ldc, hipStream_t stream) {
  if (waves >= 16) return launch_skinny<NT, MT, 16, TO>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  if (waves >= 8) return launch_skinny<NT, MT, 8, TO>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  if (waves >= 4) return launch_skinny<NT, MT, 4, TO>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  if (waves >= 2) return launch_skinny<NT, MT, 2, TO>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  return launch_skinny<NT, MT, 1, TO>(A, W, C, M, N, K, lda, ldw, ldc, stream);
}

template <typename TO>
static int pick_tiles(int nt, int waves, const void* A, const void* W, void* C, int M, int N, int K,
                      long lda, long ldw, long ldc, hipStream_t stream) {
  const int mt = (M + 15) / 16;
#define TK_GO(NT_, MT_) return pick_waves<NT_, MT_, TO>(waves, A, W, C, M, N, K, lda, ldw, ldc, stream)
  if (nt >= 4) {
    if (mt == 1) TK_GO(4, 1);
    if (mt == 2) TK_GO(4, 2);
    if (mt == 3) TK_GO(4, 3);
    TK_GO(4, 4);
  }
  if (nt >= 2) {
    if (mt == 1) TK_GO(2, 1);
    if (mt == 2) TK_GO(2, 2);
    if (mt == 3) TK_GO(2, 3);
    TK_GO(2, 4);
  }
  if (mt == 1) TK_GO(1, 1);
  if (mt == 2) TK_GO(1, 2);
  if (mt == 3) TK_GO(1, 3);
  TK_GO(1, 4);
#undef TK_GO
}

// out_dtype: 0 float32, 1 bfloat16.  M <= 64, K a multiple of 8, rows 16-byte aligned.
// nt: weight-row tiles (of 16) per block, 1, 2 or 4; waves: how many waves split K.
TK_API int tk_gemm_skinny(int out_dtype, const void* A, const void* W, void* C, int M, int N, int K,
                          long lda, long ldw, long ldc, int nt, int waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0) return -1;
  if (out_dtype == 0) return pick_tiles<float>(nt, waves, A, W, C, M, N, K, lda, ldw, ldc, stream);
  if (out_dtype == 1) return pick_tiles<bf16_t>(nt, waves, A, W, C, M, N, K, lda, ldw, ldc, stream);
  return -1;
}


// ---------------------------------------------------------------------------
// stream:  C[M,N] = A[M,K] * W[N,K]^T, M <= 64, W read exactly once and in long
// contiguous pieces.
//
// A block of 4 waves owns 64 weight rows (16 per wave) and one share of K (split
// s of KS).  K is walked in chunks of 256:
//   * every wave loads its 16 rows x 256 k (8 KB) with 16-byte loads in which 32
//     consecutive lanes cover 512 contiguous bytes of one row, keeps them in
//     registers while the previous chunk is computed, then parks them in its own
//     LDS tile (row stride 264 elements: conflict-free 16-byte reads by row);
//   * the block loads the activations' chunk [16*MT x 256] once into a shared
//     LDS tile (they are small and sit in L2);
//   * each wave then reads MFMA fragments back from LDS: lane (r, kb) takes
//     W[row r][k + kb*8 .. +8] as A operand and X[row r][same k] as B operand of
//     v_mfma_f32_16x16x32_bf16 and accumulates D[weight row][batch row].
// With KS > 1 split s writes float32 partial sums to its own copy of C; the kernel
// that reads C next (residual add + norm, or the q/k norm + rotation kernel) adds
// the copies in split order.  No block waits for, or signals, another.
// ---------------------------------------------------------------------------
constexpr int SBK = 256;        // k per chunk
// Row tiles of activations from which a chunk's operand reads are asked for ahead of the
// products (sched_group_barrier below).  With one row tile the plain loop is kept: the read-ahead
// gains nothing there and cost the two-wave gated product of a 14B-shaped layer 8 % (63 -> 68 us).
constexpr int READ_AHEAD_FROM = 2;
constexpr int SLD = SBK + 8;    // LDS row stride in elements

// GATED: W is [2N, K], gate rows then up rows; the block owns 8*WAVES output columns, the
// first half of its waves their gate rows and the second half the matching up rows, and
// the result is silu(gate) * up [M, N] (the SwiGLU feed-forward's first half in one kernel).
//
// WAVES (4 or 8): waves a block; they share the activations' chunk, so 8 waves read it
// once per 128 weight rows (what pays from 33 rows of activations on: +10 % at 64 rows).
// A second chunk of weights in flight per wave was measured too and gained nothing: at 64
// rows the kernel is held by LDS traffic (seven bytes through LDS per byte of weights),
// at 16 rows and fewer by the launch and drain of blocks that live for a few microseconds.
// Four waves of two row tiles each (the same 128 rows a block, the activations' fragments
// read half as often) were slower than eight waves of one at 40 to 64 rows on every
// projection shape of an 8B model (down at 64 rows 27.4 us against 24.2, gated 52.4 against
// 46.0): one wave a SIMD hides too little of the LDS round trips.
//
// RowScale (up to 16 rows): the activations may be given as bf16(x * gamma) of an RMSNorm whose
// row statistics are not applied yet (what the product that adds into the residual stream
// leaves, gemm_wholek.hip); the product is linear in a row's scale, so the block multiplies
// row m of its sums by rstd[m] = rsqrt(sum_s sumsq[s][m] / K + eps) before it stores them
// (partial sums of a split too: their sum is scaled alike) or gates them.
constexpr int kRowScaleSlabs = 512;  // most slabs of sums of squares: a thread holds kRowScaleSlabs / (threads / 16) of them
struct RowScale {
  const float* sumsq;  // [slabs][M]: sums of squares of the rows over slabs of columns; nullptr: no scaling
  int slabs;
  float eps;
};

template <int MT, typename TO, bool GATED, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_stream_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TO* __restrict__ C, int M, int N,
    int K, long lda, long ldw, long ldc, int chunks_per_split, long split_stride, RowScale scale) {
  constexpr int THREADS = WAVES * 64;
  constexpr int XP = (16 * MT * 32 + THREADS - 1) / THREADS;  // 16-byte pieces of the activations a thread loads per chunk
  constexpr bool XWHOLE = XP * THREADS == 16 * MT * 32;       // else the last piece of some threads lies past the chunk
  static_assert(WAVES % 2 == 0, "waves load the weights' pieces in pairs of rows and the gated form halves them");
  constexpr int HALF = WAVES / 2;
  // XBUF: copies of the activations' chunk.  A wave reads weights from its own tile only, so with
  // two copies written in turn one barrier a chunk is enough (a wave may start to write chunk
  // i + 1 while others still read chunk i): 3-6 % for blocks of eight waves, which have a CU to
  // themselves anyway; nothing at up to 16 rows, and blocks of four would lose a place on the CU.
  constexpr int XBUF = (WAVES >= 6 && MT >= 2 && MT <= 4) ? 2 : 1;  // (five row tiles and more: one copy fits beside the weights)
  __shared__ __attribute__((aligned(16))) bf16_t ws[WAVES][16][SLD];
  __shared__ __attribute__((aligned(16))) bf16_t xs[XBUF][16 * MT][SLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int row_block = blockIdx.x, split = blockIdx.y;
  // n_wave: first output column of this wave; w_first/w_limit: its weight rows
  const bool up_wave = GATED && wave >= HALF;
  const int n_wave = GATED ? row_block * (16 * HALF) + (wave % HALF) * 16 : row_block * (16 * WAVES) + wave * 16;
  const int w_first = up_wave ? N + n_wave : n_wave;
  const int w_limit = up_wave ? 2 * N : N;
  const int total_chunks = (K + SBK - 1) / SBK;
  const int c_begin = split * chunks_per_split;
  const int c_end = min(total_chunks, c_begin + chunks_per_split);

  // loader roles: W piece i of this lane = row 2i + lane/32, 16-byte column lane%32
  const int w_col = (lane & 31) * 8, w_row0 = lane >> 5;
  // X pieces of this thread: piece p = i*THREADS + tid -> row p/32, column p%32
  const int x_col = (tid & 31) * 8, x_row0 = tid >> 5;

  u32x4 wreg[8];
  u32x4 xreg[XP];
  const u32x4 zero = {0u, 0u, 0u, 0u};
  // Rows are clamped into the matrices (rows past N or M are computed from a valid
  // row and never stored).  A piece past K is read at the row's last piece instead and
  // meets zeros: the activations' pieces past K are zeroed on their way into LDS.
  const bf16_t* wrow[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) wrow[i] = W + (size_t)min(w_first + 2 * i + w_row0, w_limit - 1) * ldw;
  const bf16_t* xrow[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) xrow[i] = A + (size_t)min(i * (THREADS / 32) + x_row0, M - 1) * lda;

  float4v acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

  // RowScale: thread (row tid % 16, group tid / 16) adds its share of the row's slab sums;
  // they meet in LDS behind the walk's barriers and are added in group order at the end.
  __shared__ float s_stat[MT == 1 ? THREADS : 1];
  const bool scaled = MT == 1 && scale.sumsq != nullptr;

#define TK_FETCH_W(C_)                                                                              \
  {                                                                                                 \
    const int wo_ = min((C_) * SBK + w_col, K - 8);                                                 \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) /* weights are read once: streaming loads */      \
        wreg[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[i] + wo_));        \
  }
#define TK_FETCH_X(C_)                                                                              \
  {                                                                                                 \
    const int xo_ = min((C_) * SBK + x_col, K - 8);                                                 \
    _Pragma("unroll") for (int i = 0; i < XP; ++i)                                                  \
        xreg[i] = *reinterpret_cast<const u32x4*>(xrow[i] + xo_);                                   \
  }
  // Blocks walk their chunks of K in rotated order (block b starts b chunks in): all blocks
  // start together, and in step they would all read the same 512-byte window of their rows,
  // 8 KB apart, which lands on a few memory channels only.
  const int nchunks = c_end - c_begin;
  const int rot = nchunks > 0 ? (int)(blockIdx.x % (unsigned)nchunks) : 0;
  auto chunk_at = [&](int i) {
    const int j = i + rot;
    return c_begin + (j >= nchunks ? j - nchunks : j);
  };
  // One chunk: park the registers in LDS, start the next chunk's loads into them, multiply.
#define TK_CHUNK(I_)                                                                                \
  {                                                                                                 \
    const int cur_ = chunk_at(I_);                                                                  \
    const int xb_ = XBUF == 2 ? ((I_) & 1) : 0;                                                     \
    if (XBUF == 1) __syncthreads(); /* the previous chunk's fragments have been read */             \
    _Pragma("unroll") for (int i = 0; i < 8; ++i)                                                   \
        *reinterpret_cast<u32x4*>(&ws[wave][2 * i + w_row0][w_col]) = wreg[i];                      \
    {                                                                                               \
      const bool inside_ = cur_ * SBK + x_col < K;                                                  \
      _Pragma("unroll") for (int i = 0; i < XP; ++i)                                                \
        if (XWHOLE || i * (THREADS / 32) + x_row0 < 16 * MT)                                        \
          *reinterpret_cast<u32x4*>(&xs[xb_][i * (THREADS / 32) + x_row0][x_col]) = inside_ ? xreg[i] : zero; \
    }                                                                                               \
    __syncthreads();                                                                                \
    if ((I_) + 1 < nchunks) {                                                                       \
      const int next_ = chunk_at((I_) + 1);                                                         \
      TK_FETCH_W(next_)                                                                             \
      TK_FETCH_X(next_)                                                                             \
    }                                                                                               \
    if constexpr (MT < READ_AHEAD_FROM || MT > 4) { /* (more row tiles: no registers for two steps' fragments) */ \
      _Pragma("unroll") for (int s = 0; s < SBK / 32; ++s) {                                        \
        Frag8 wf, xf[MT];                                                                           \
        wf.u = *reinterpret_cast<const uint4*>(&ws[wave][r][s * 32 + kb * 8]);                      \
        _Pragma("unroll") for (int j = 0; j < MT; ++j)                                              \
            xf[j].u = *reinterpret_cast<const uint4*>(&xs[xb_][j * 16 + r][s * 32 + kb * 8]);       \
        _Pragma("unroll") for (int j = 0; j < MT; ++j)                                              \
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, xf[j].v, acc[j], 0, 0, 0);       \
      }                                                                                             \
    } else {                                                                                        \
      /* the fragments of a step of 32 k are asked for while the step before is multiplied: a    */ \
      /* wave that waits for each fragment in turn spends its time on round trips to LDS         */ \
      Frag8 wf[SBK / 32], xf[SBK / 32][MT];                                                         \
      _Pragma("unroll") for (int s = 0; s < SBK / 32; ++s) {                                        \
        wf[s].u = *reinterpret_cast<const uint4*>(&ws[wave][r][s * 32 + kb * 8]);                   \
        _Pragma("unroll") for (int j = 0; j < MT; ++j)                                              \
            xf[s][j].u = *reinterpret_cast<const uint4*>(&xs[xb_][j * 16 + r][s * 32 + kb * 8]);    \
      }                                                                                             \
      _Pragma("unroll") for (int s = 0; s < SBK / 32; ++s)                                          \
        _Pragma("unroll") for (int j = 0; j < MT; ++j)                                              \
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s].v, xf[s][j].v, acc[j], 0, 0, 0); \
      /* order asked of the scheduler: two steps' reads, then a product and a read in turn */       \
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * (1 + MT), 0);                                 \
      _Pragma("unroll") for (int i = 0; i < (SBK / 32 - 2) * (1 + MT); ++i) {                       \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                          \
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                          \
      }                                                                                             \
      __builtin_amdgcn_sched_group_barrier(0x008, SBK / 32 * MT - (SBK / 32 - 2) * (1 + MT), 0);    \
    }                                                                                               \
  }

  if (nchunks > 0) {
    const int first_ = chunk_at(0);
    TK_FETCH_W(first_)
    TK_FETCH_X(first_)
  }
  // RowScale: the slab sums are asked for now and first looked at after the walk over K (a
  // block that waited for them here would start its walk a memory round trip late).
  constexpr int STAT_STEP = THREADS / 16;
  constexpr int STAT_LOADS = kRowScaleSlabs / STAT_STEP;
  float stat[MT == 1 ? STAT_LOADS : 1];
  if constexpr (MT == 1) {
#pragma unroll
    for (int u = 0; u < STAT_LOADS; ++u) stat[u] = 0.f;
    if (scaled && (tid & 15) < M) {
#pragma unroll
      for (int u = 0; u < STAT_LOADS; ++u) {
        const int sl = (tid >> 4) + u * STAT_STEP;
        if (sl < scale.slabs) stat[u] = scale.sumsq[(size_t)sl * M + (tid & 15)];
      }
    }
  }
  for (int i = 0; i < nchunks; ++i) TK_CHUNK(i)
#undef TK_CHUNK
#undef TK_FETCH_X
#undef TK_FETCH_W

  // With several splits, split s writes its partial sums to C + s * split_stride; whoever
  // reads C next adds the splits (in split order, so the sum is deterministic).
  C += (size_t)split * split_stride;

  if constexpr (MT == 1) {
    if (scaled) {
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < STAT_LOADS; ++u) ss += stat[u];
      s_stat[tid] = ss;
      __syncthreads();
      float total = 0.f;
#pragma unroll
      for (int grp = 0; grp < THREADS / 16; ++grp) total += s_stat[grp * 16 + r];
      acc[0] *= rsqrtf(total / (float)K + scale.eps);
    }
  }

  if (GATED) {
    float* up = reinterpret_cast<float*>(&ws[0][0][0]);  // [HALF up waves][MT][64 lanes][4]
    static_assert(sizeof(ws) >= sizeof(float) * HALF * MT * 64 * 4, "the exchange fits the weights' tiles");
    __syncthreads();                                      // the last chunk's fragments have been read
    if (wave >= HALF) {
#pragma unroll
      for (int j = 0; j < MT; ++j)
        *reinterpret_cast<float4*>(up + ((size_t)((wave - HALF) * MT + j) * 64 + lane) * 4) =
            make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
    }
    __syncthreads();
    if (wave >= HALF) return;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const float4 u = *reinterpret_cast<const float4*>(up + ((size_t)(wave * MT + j) * 64 + lane) * 4);
      acc[j][0] = acc[j][0] / (1.f + __expf(-acc[j][0])) * u.x;
      acc[j][1] = acc[j][1] / (1.f + __expf(-acc[j][1])) * u.y;
      acc[j][2] = acc[j][2] / (1.f + __expf(-acc[j][2])) * u.z;
      acc[j][3] = acc[j][3] / (1.f + __expf(-acc[j][3])) * u.w;
    }
  }

  // acc[j][e] = C[batch row j*16 + r][column n_wave + kb*4 + e]: four columns a store
  const bool wide = rows_take_wide_stores(C, ldc);
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = j * 16 + r;
    if (m >= M) continue;
    const int n = n_wave + kb * 4;
    store_four<TO>(C + (size_t)m * ldc + n, acc[j][0], acc[j][1], acc[j][2], acc[j][3], N - n, wide);
  }
}

template <typename TO, bool GATED, int WAVES>
static int launch_stream_shape(const void* A, const void* W, void* C, int M, int N, int K, long lda,
                               long ldw, long ldc, int chunks_per_split, int KS, long split_stride,
                               RowScale scale, hipStream_t stream) {
  const int cols = GATED ? 8 * WAVES : 16 * WAVES;
  dim3 grid((N + cols - 1) / cols, KS);
  const int mt = (M + 15) / 16;
#define TK_STREAM(MT_)                                                                          \
  gemm_stream_kernel<MT_, TO, GATED, WAVES><<<grid, WAVES * 64, 0, stream>>>(            \
      (const bf16_t*)A, (const bf16_t*)W, (TO*)C, M, N, K, lda, ldw, ldc, chunks_per_split,     \
      split_stride, scale)
  if (mt == 1) TK_STREAM(1);
  else if (mt == 2) TK_STREAM(2);
  else if (mt == 3) TK_STREAM(3);
  else if (mt == 4) TK_STREAM(4);
  else if constexpr (WAVES == 8 && !GATED) {  // 65 to 128 rows: blocks of eight waves, the plain product only
    if (mt == 5) TK_STREAM(5);
    else if (mt == 6) TK_STREAM(6);
    else if (mt == 7) TK_STREAM(7);
    else if (mt == 8) TK_STREAM(8);
    else return -1;
  } else return -1;
#undef TK_STREAM
  return launch_status();
}

// waves: 4, 6 or 8 a block; the gated product also 2.
template <typename TO, bool GATED>
static int launch_stream(int waves, const void* A, const void* W, void* C, int M, int N, int K,
                         long lda, long ldw, long ldc, int cps, int KS, long split_stride, RowScale scale,
                         hipStream_t stream) {
  if (waves >= 8)
    return launch_stream_shape<TO, GATED, 8>(A, W, C, M, N, K, lda, ldw, ldc, cps, KS, split_stride, scale, stream);
  // six waves (96 weight rows a block): for matrices whose rows divide over the CUs that way
  if (waves == 6)
    return launch_stream_shape<TO, GATED, 6>(A, W, C, M, N, K, lda, ldw, ldc, cps, KS, split_stride, scale, stream);
  if constexpr (GATED) {
    // two waves (one gate tile, one up tile: 16 output columns a block): more, smaller blocks
    if (waves == 2)
      return launch_stream_shape<TO, GATED, 2>(A, W, C, M, N, K, lda, ldw, ldc, cps, KS, split_stride, scale, stream);
  }
  return launch_stream_shape<TO, GATED, 4>(A, W, C, M, N, K, lda, ldw, ldc, cps, KS, split_stride, scale, stream);
}

// out_dtype: 0 float32, 1 bfloat16.  M <= 64 (<= 128 with eight waves); K a multiple of 8; rows 16-byte aligned.
// waves: 4 or 8 waves a block.  splits: shares of K.  With splits > 1 the output must be float32 and C holds
// `splits` partial results, split_stride elements apart, that the reader adds.
// sumsq (may be null), slabs, eps: the rows' scale, see RowScale; then M <= 16.
// Returns the number of splits actually used (<= splits; no split is empty), or < 0.
TK_API int tk_gemm_stream(int out_dtype, const void* A, const void* W, void* C, int M, int N, int K,
                          long lda, long ldw, long ldc, int splits, long split_stride, int waves,
                          const float* sumsq, int slabs, float eps, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > (waves >= 8 ? 128 : 64) || K < 8 || K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0 || splits < 1 || splits > 65535) return -1;
  if (sumsq != nullptr && (M > 16 || slabs < 1 || slabs > kRowScaleSlabs || waves >= 6)) return -1;
  const RowScale scale{sumsq, slabs, eps};
  if (splits > 1 && out_dtype != 0) return -1;
  const int total_chunks = (K + SBK - 1) / SBK;
  const int cps = (total_chunks + splits - 1) / splits;
  const int ks = (total_chunks + cps - 1) / cps;
  int status = -1;
  if (out_dtype == 0) status = launch_stream<float, false>(waves, A, W, C, M, N, K, lda, ldw, ldc, cps, ks, split_stride, scale, stream);
  if (out_dtype == 1) status = launch_stream<bf16_t, false>(waves, A, W, C, M, N, K, lda, ldw, ldc, cps, ks, split_stride, scale, stream);
  return status == 0 ? ks : (status > 0 ? -status : status);
}

// C[M, N] = silu(A W_gate^T) * (A W_up^T) with W = [W_gate; W_up] of 2N rows; bfloat16 out.
TK_API int tk_gemm_stream_swiglu(const void* A, const void* W, void* C, int M, int N, int K, long lda,
                                 long ldw, long ldc, int waves, const float* sumsq, int slabs, float eps,
                                 hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K < 8 || K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0) return -1;
  if (sumsq != nullptr && (M > 16 || slabs < 1 || slabs > kRowScaleSlabs || waves >= 6)) return -1;
  const int total_chunks = (K + SBK - 1) / SBK;
  return launch_stream<bf16_t, true>(waves, A, W, C, M, N, K, lda, ldw, ldc, total_chunks, 1, 0,
                                     RowScale{sumsq, slabs, eps}, stream);
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_gemm_stream)
TK_SLOTS(tk_gemm_stream_swiglu)
TK_SLOTS(tk_gemm_skinny)
