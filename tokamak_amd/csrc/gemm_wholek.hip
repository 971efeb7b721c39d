// bf16 products of few rows (M <= 16: decode steps of up to sixteen requests) in which one
// block holds the whole of K for its sixteen output columns.
//
// C[M,N] = A[M,K] W[N,K]^T.  A block of WAVES waves owns 16 weight rows (with GATED also the
// 16 matching rows of the second half of W); its waves split K between them in chunks of
// 256: wave w takes chunks w, w + WAVES, ...  For a chunk a wave loads its 16 rows x 512
// bytes of weights once, with streaming 16-byte loads in which 32 consecutive lanes cover
// 512 contiguous bytes of a row, parks them in its own LDS tile (16-byte pieces xor-swizzled
// by row: no padding, no bank conflicts) and reads them back as MFMA A operands; the
// activations are few and sit in L2, so every lane reads its B operands straight from memory
// (v_mfma_f32_16x16x32_bf16: D[weight row][batch row]).  No barrier is met inside the walk
// over K.  At the end the waves' sums are added in wave order through LDS (a fixed order: the
// result is deterministic), and because a block holds complete sums, no partial sums leave
// the kernel and the epilogue can finish the work of the kernels that used to follow:
//
//   * scaled input: the activations may be given as a = bf16(x * gamma) of an RMSNorm whose
//     row statistics are not applied yet; the product is linear in a row's scale, so the block
//     multiplies row m of its result by rstd[m] = rsqrt(sum_s sumsq[s][m] / K + eps);
//   * GATED: C = silu(A W_gate^T) * (A W_up^T);
//   * ADD: the result is added into the float32 residual stream; the block writes the new
//     stream, bf16(new stream * gamma_next) for the product that follows the next norm, and
//     the sum of squares of its 16 columns of every row (sumsq[block][m]), from which that
//     product takes its rstd.
//
// So a decode layer of few rows runs q/k/v product, attention, o product, gate/up product and
// down product with no kernel in between.
#include "common.h"
#include "slots.h"

using namespace tk;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // arrays of HIP's uint4 struct end up in scratch

union Frag8 {
  u32x4 u;
  bf16x8 v;
};

constexpr int WK = 256;           // k per chunk
constexpr int TILE_BYTES = 16 * WK * 2;

struct RowScale {        // the statistics of the norm before the product; sumsq == nullptr: none
  const float* sumsq;    // [slabs][M]: sums of squares of the rows over slabs of columns
  int slabs;
  float eps;
};

struct StreamSum {       // ADD
  float* resid;          // [M, N] float32, rows ld_resid elements apart
  long ld_resid;
  const float* gamma;    // [N]: weight of the norm that reads the stream next
  bf16_t* scaled;        // [M, N] bf16(resid * gamma), rows ld_scaled apart; or nullptr
  long ld_scaled;
  float* sumsq;          // [gridDim.x][M]
};

enum { EPI_STORE = 0, EPI_GATED = 1, EPI_ADD = 2 };

template <int EPI, typename TO, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_wholek_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TO* __restrict__ C, int M, int N, int K,
    long lda, long ldw, long ldc, RowScale scale, StreamSum sum) {
  constexpr int TILES = EPI == EPI_GATED ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * 16;
  unsigned char* mine = lds + (size_t)wave * (TILES * TILE_BYTES);  // this wave's tiles; later its sums

  const int total_chunks = (K + WK - 1) / WK;
  const int per = (total_chunks + WAVES - 1) / WAVES;   // chunks a wave walks at most
  // Blocks start at different chunks, so that at any moment the blocks in step do not all
  // read the same part of their rows (which would meet a few memory channels only).
  const int rot = per > 0 ? (int)(blockIdx.x % (unsigned)per) : 0;
  auto chunk_at = [&](int i) {
    const int j = i + rot;
    return wave + (j >= per ? j - per : j) * WAVES;     // may be >= total_chunks: skipped
  };

  // loader roles: piece i of this lane = weight row 2i + lane/32, 16-byte column lane%32
  const int w_piece = lane & 31, w_row0 = lane >> 5;
  const bf16_t* wrow[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) wrow[i] = W + (size_t)min(n0 + 2 * i + w_row0, N - 1) * ldw;  // rows past N: a valid row, never stored
  const size_t second = (size_t)N * ldw;  // GATED: from a row of the first half of W to its partner
  const bf16_t* xrow = A + (size_t)min(r, M - 1) * lda;        // rows past M likewise

  u32x4 wreg[TILES][8];
  Frag8 xf[8];
  const u32x4 zero = {0u, 0u, 0u, 0u};
  // A piece past K is read at the row's last piece instead and meets zeros: the
  // activations' pieces past K are zero.
#define TK_FETCH_W(C_)                                                                               \
  {                                                                                                  \
    const int wo_ = min((C_) * WK + w_piece * 8, K - 8);                                             \
    _Pragma("unroll") for (int t = 0; t < TILES; ++t)                                                \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) /* weights are read once: streaming loads */       \
        wreg[t][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[i] + t * second + wo_)); \
  }
#define TK_FETCH_X(C_)                                                                               \
  {                                                                                                  \
    _Pragma("unroll") for (int s = 0; s < 8; ++s) {                                                  \
      const int k_ = (C_) * WK + s * 32 + kb * 8;                                                    \
      const u32x4 v_ = *reinterpret_cast<const u32x4*>(xrow + min(k_, K - 8));                       \
      xf[s].u = k_ < K ? v_ : zero;                                                                  \
    }                                                                                                \
  }

  float4v acc[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};

  int i = 0;
  while (i < per && chunk_at(i) >= total_chunks) ++i;
  if (i < per) {
    TK_FETCH_W(chunk_at(i))
    TK_FETCH_X(chunk_at(i))
  }

  // what only the epilogue needs is asked for now, behind the first chunk's loads
  float4 old = make_float4(0.f, 0.f, 0.f, 0.f), gam = make_float4(0.f, 0.f, 0.f, 0.f);
  const int m = r, n = n0 + kb * 4;  // this lane's part of the block's result: C[m][n .. n+3]
  if constexpr (EPI == EPI_ADD) {
    if (wave == 0 && m < M && n < N) {  // N is a multiple of 4: the four columns are inside together
      old = *reinterpret_cast<const float4*>(sum.resid + (size_t)m * sum.ld_resid + n);
      if (sum.scaled != nullptr) gam = *reinterpret_cast<const float4*>(sum.gamma + n);
    }
  }
  float ss = 0.f;
  if (scale.sumsq != nullptr) {
    // thread -> (row tid%16, group tid/16): the group's share of the row's slab sums
    const int row = tid & 15;
    float part[4] = {0.f, 0.f, 0.f, 0.f};  // four loads in flight at a time
    if (row < M)
      for (int sl = tid >> 4; sl < scale.slabs; sl += 16 * WAVES) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (sl + u * 4 * WAVES < scale.slabs) part[u] += scale.sumsq[(size_t)(sl + u * 4 * WAVES) * M + row];
      }
    ss = (part[0] + part[1]) + (part[2] + part[3]);
  }

  while (i < per) {
    // park the registers in the wave's tile, ask for the next chunk's weights, multiply
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const int row = 2 * p + w_row0;
        *reinterpret_cast<u32x4*>(mine + t * TILE_BYTES + row * (WK * 2) + ((w_piece ^ row) & 31) * 16) = wreg[t][p];
      }
    int nxt = i + 1;
    while (nxt < per && chunk_at(nxt) >= total_chunks) ++nxt;
    if (nxt < per) TK_FETCH_W(chunk_at(nxt))
#pragma unroll
    for (int s = 0; s < 8; ++s) {
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        Frag8 wf;
        wf.u = *reinterpret_cast<const u32x4*>(mine + t * TILE_BYTES + r * (WK * 2) + (((s * 4 + kb) ^ r) & 31) * 16);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, xf[s].v, acc[t], 0, 0, 0);
      }
    }
    // the activations of the next chunk come from L2 and arrive before its weights do
    if (nxt < per) TK_FETCH_X(chunk_at(nxt))
    i = nxt;
  }
#undef TK_FETCH_X
#undef TK_FETCH_W

  // acc[t][e] = sum over this wave's chunks for C[batch row r][column n0 + kb*4 + e].
  // Every wave leaves its sums (and its share of the rows' statistics) in its own tile.
  float* my_sums = reinterpret_cast<float*>(mine);          // [TILES][64 lanes][4]
  float* my_stat = my_sums + TILES * 256;                   // [64 lanes]
#pragma unroll
  for (int t = 0; t < TILES; ++t)
    *reinterpret_cast<float4*>(my_sums + (t * 64 + lane) * 4) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
  my_stat[lane] = ss;
  __syncthreads();
  if (wave != 0) return;

  float4 total[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) total[t] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const float* theirs = reinterpret_cast<const float*>(lds + (size_t)w * (TILES * TILE_BYTES));
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const float4 v = *reinterpret_cast<const float4*>(theirs + (t * 64 + lane) * 4);
      total[t].x += v.x;
      total[t].y += v.y;
      total[t].z += v.z;
      total[t].w += v.w;
    }
  }
  float rstd = 1.f;
  if (scale.sumsq != nullptr) {
    // row r's statistics: groups 0 .. 4*WAVES-1 in order, a quarter of them per lane (r, kb)
    float part = 0.f;
#pragma unroll
    for (int g = 0; g < WAVES; ++g) {
      const int group = kb * WAVES + g;  // thread group*16 + r of the block holds it
      part += reinterpret_cast<const float*>(lds + (size_t)(group >> 2) * (TILES * TILE_BYTES))[TILES * 256 + (group & 3) * 16 + r];
    }
    const float other = __shfl_xor(part, 16, kWave);
    const float pair = kb & 1 ? other + part : part + other;    // (kb 0 + kb 1), (kb 2 + kb 3): in this order
    const float far = __shfl_xor(pair, 32, kWave);
    const float all = kb & 2 ? far + pair : pair + far;
    rstd = rsqrtf(all / (float)K + scale.eps);
  }

  if constexpr (EPI == EPI_ADD) {
    float sq = 0.f;
    if (m < M && n < N) {
      const float4 v = make_float4(old.x + total[0].x, old.y + total[0].y, old.z + total[0].z, old.w + total[0].w);
      *reinterpret_cast<float4*>(sum.resid + (size_t)m * sum.ld_resid + n) = v;
      if (sum.scaled != nullptr)
        *reinterpret_cast<uint2*>(sum.scaled + (size_t)m * sum.ld_scaled + n) =
            make_uint2(pack_bf16x2(v.x * gam.x, v.y * gam.y), pack_bf16x2(v.z * gam.z, v.w * gam.w));
      sq = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    const float other = __shfl_xor(sq, 16, kWave);
    const float pair = kb & 1 ? other + sq : sq + other;
    const float far = __shfl_xor(pair, 32, kWave);
    const float all = kb & 2 ? far + pair : pair + far;
    if (kb == 0 && m < M) sum.sumsq[(size_t)blockIdx.x * M + m] = all;
    return;
  }

  float res[4];
  if constexpr (EPI == EPI_GATED) {
    const float g[4] = {total[0].x * rstd, total[0].y * rstd, total[0].z * rstd, total[0].w * rstd};
    const float u[4] = {total[1].x * rstd, total[1].y * rstd, total[1].z * rstd, total[1].w * rstd};
#pragma unroll
    for (int e = 0; e < 4; ++e) res[e] = g[e] / (1.f + __expf(-g[e])) * u[e];
  } else {
    res[0] = total[0].x * rstd;
    res[1] = total[0].y * rstd;
    res[2] = total[0].z * rstd;
    res[3] = total[0].w * rstd;
  }
  if (m >= M) return;
  store_four<TO>(C + (size_t)m * ldc + n, res[0], res[1], res[2], res[3], N - n, rows_take_wide_stores(C, ldc));
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int EPI, typename TO, int WAVES>
static int launch_wholek(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc,
                         RowScale scale, StreamSum sum, hipStream_t stream) {
  constexpr int TILES = EPI == EPI_GATED ? 2 : 1;
  constexpr int lds = WAVES * TILES * TILE_BYTES;
  static_assert(TILE_BYTES >= (int)sizeof(float) * (2 * 256 + 64), "a wave's sums fit its tile");
  auto kernel = gemm_wholek_kernel<EPI, TO, WAVES>;
  if (lds > 64 * 1024) {
    static bool raised[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
    if (!raised[dev]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return -1;
      raised[dev] = true;
    }
  }
  kernel<<<(N + 15) / 16, WAVES * 64, lds, stream>>>((const bf16_t*)A, (const bf16_t*)W, (TO*)C, M, N, K, lda, ldw, ldc,
                                                    scale, sum);
  return launch_status();
}

static bool operands_fit(const void* A, const void* W, int M, int N, int K, long lda, long ldw) {
  return M <= 16 && K >= 8 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && aligned16(A) && aligned16(W);
}

// C[M, N] = (A W^T) * rstd, rstd[m] = rsqrt(sum_s sumsq[s][m] / K + eps), or 1 with sumsq == nullptr.
// out_dtype: 0 float32, 1 bfloat16.  gated == 1: W = [W_gate; W_up] of 2N rows and
// C = silu(A W_gate^T * rstd) * (A W_up^T * rstd), bfloat16.  M <= 16; K a multiple of 8; rows
// 16-byte aligned.  waves: 4, 8 or 16 a block.
TK_API int tk_gemm_wholek(int out_dtype, int gated, const void* A, const void* W, void* C, int M, int N, int K,
                          long lda, long ldw, long ldc, const float* sumsq, int slabs, float eps, int waves,
                          hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!operands_fit(A, W, M, N, K, lda, ldw) || (sumsq != nullptr && slabs < 1)) return -1;
  if (gated && out_dtype != 1) return -1;
  const RowScale scale{sumsq, slabs, eps};
  const StreamSum none{};
#define TK_GO(EPI_, TO_)                                                                                         \
  {                                                                                                              \
    if (waves >= 16) return launch_wholek<EPI_, TO_, 16>(A, W, C, M, N, K, lda, ldw, ldc, scale, none, stream);  \
    if (waves >= 8) return launch_wholek<EPI_, TO_, 8>(A, W, C, M, N, K, lda, ldw, ldc, scale, none, stream);    \
    return launch_wholek<EPI_, TO_, 4>(A, W, C, M, N, K, lda, ldw, ldc, scale, none, stream);                    \
  }
  if (gated) TK_GO(EPI_GATED, bf16_t)
  if (out_dtype == 0) TK_GO(EPI_STORE, float)
  if (out_dtype == 1) TK_GO(EPI_STORE, bf16_t)
#undef TK_GO
  return -1;
}

// resid[M, N] += A W^T (float32 stream); scaled[M, N] = bf16(resid * gamma) (skipped with
// scaled == nullptr); sumsq[b][m] = sum over columns 16b .. 16b+15 of resid[m][.]^2, for
// b < tk_gemm_wholek_slabs(N).  M <= 16; N a multiple of 4; rows 16-byte aligned.
TK_API int tk_gemm_wholek_slabs(int N) { return (N + 15) / 16; }

TK_API int tk_gemm_wholek_add(const void* A, const void* W, int M, int N, int K, long lda, long ldw, float* resid,
                              long ld_resid, const float* gamma, void* scaled, long ld_scaled, float* sumsq,
                              int waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!operands_fit(A, W, M, N, K, lda, ldw)) return -1;
  if (N % 4 != 0 || ld_resid % 4 != 0 || !aligned16(resid) || resid == nullptr || sumsq == nullptr) return -1;
  if (scaled != nullptr && (gamma == nullptr || !aligned16(gamma) || ld_scaled % 4 != 0 ||
                            (reinterpret_cast<uintptr_t>(scaled) & 7) != 0))
    return -1;
  const StreamSum sum{resid, ld_resid, gamma, (bf16_t*)scaled, ld_scaled, sumsq};
  const RowScale none{};
  if (waves >= 16) return launch_wholek<EPI_ADD, float, 16>(A, W, nullptr, M, N, K, lda, ldw, 0, none, sum, stream);
  if (waves >= 8) return launch_wholek<EPI_ADD, float, 8>(A, W, nullptr, M, N, K, lda, ldw, 0, none, sum, stream);
  return launch_wholek<EPI_ADD, float, 4>(A, W, nullptr, M, N, K, lda, ldw, 0, none, sum, stream);
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_gemm_wholek)
TK_SLOTS(tk_gemm_wholek_add)
