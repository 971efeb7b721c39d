// C[M,N] = A[M,K] * W[N,K]^T with float32 multiply-add and float32 accumulation
// for any M, N, K.  It is the true 32-bit matrix product of the float32 path
// (no reduced-precision matrix mode), and also accepts bf16 inputs.  Every
// output element is summed in one fixed order, whichever kernel below does it, so a row's
// result does not depend on which other rows are in the batch: k ascending within pieces of
// kPiece, whose sums are added to the total one after the other.  The two levels
// keep the rounding error of a sum over K terms near sqrt(kPiece) + sqrt(K / kPiece)
// units instead of sqrt(K) (K is 25,600 in the widest feed-forward).
#include "common.h"
#include "slots.h"

using namespace tk;

constexpr int BK = 16, PAD = 4;
constexpr int kPiece = 256;  // k values summed before they join the total (a multiple of BK)

// A block of 256 threads owns 64H x 64H outputs (H = 1 or 2); thread (ty, tx) of 16 x 16 owns
// rows ty*4.. (and 64 + ty*4..) and columns tx*4.. (and 64 + tx*4..): 4H x 4H outputs, per k
// 2H 16-byte LDS reads for 16 H^2 multiply-adds.  The next 16 k are fetched into registers while
// the current ones are multiplied.  H = 2 is the fast one (65 against 37 TFLOP/s on 2,048 rows);
// H = 1 has four times the blocks, for products too small to fill the GPU otherwise.
template <typename TI, typename TO, int H>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TI* __restrict__ A,
                                                         const TI* __restrict__ W,
                                                         TO* __restrict__ C, int M, int N, int K,
                                                         long lda, long ldw, long ldc) {
  constexpr int BM = 64 * H, BN = 64 * H, R = 4 * H;
  __shared__ __attribute__((aligned(16))) float As[BK][BM + PAD];
  __shared__ __attribute__((aligned(16))) float Ws[BK][BN + PAD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int ty = tid / 16, tx = tid % 16;
  const int lrow = tid / 4, lk = (tid % 4) * 4;   // loader: rows lrow (and lrow + 64), four k from lk

  float acc[R][R], total[R][R];
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int j = 0; j < R; ++j) acc[i][j] = total[i][j] = 0.f;

  float ar[H][4], wr[H][4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const int m = m0 + lrow + 64 * h, n = n0 + lrow + 64 * h;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        ar[h][i] = (m < M && k < K) ? Elem<TI>::load(A + (size_t)m * lda + k) : 0.f;
        wr[h][i] = (n < N && k < K) ? Elem<TI>::load(W + (size_t)n * ldw + k) : 0.f;
      }
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 > 0 && k0 % kPiece == 0) {
#pragma unroll
      for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        As[lk + i][lrow + 64 * h] = ar[h][i];
        Ws[lk + i][lrow + 64 * h] = wr[h][i];
      }
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[R], w[R];
#pragma unroll
      for (int h = 0; h < H; ++h) {
        *reinterpret_cast<float4*>(&a[4 * h]) = *reinterpret_cast<const float4*>(&As[k][64 * h + ty * 4]);
        *reinterpret_cast<float4*>(&w[4 * h]) = *reinterpret_cast<const float4*>(&Ws[k][64 * h + tx * 4]);
      }
#pragma unroll
      for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int m = m0 + (i / 4) * 64 + ty * 4 + i % 4;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int n = n0 + (j / 4) * 64 + tx * 4 + j % 4;
      if (n < N) Elem<TO>::store(C + (size_t)m * ldc + n, total[i][j] + acc[i][j]);
    }
  }
}

// The same product on the matrix cores: v_mfma_f32_32x32x2_f32 multiplies and adds in full
// float32 and, for every output element, gives exactly the bits of fmaf over its two k in
// ascending order (measured against the chain on random operands: every output of every
// step equal), so a walk over k in steps of two is the chain of the kernels above and below,
// bit for bit, and the pieces of kPiece are kept as they are.  A block of four waves owns
// 64H x 64H outputs, a wave 32H x 32H of them (H x H tiles of 32 x 32, each 16 accumulators a
// lane and as many for the total).  The tiles of A and W lie in LDS k-major as above; a lane's
// operand of a step is one float: A[row lane % 32][k + lane / 32].
typedef float float16v __attribute__((ext_vector_type(16)));

template <typename TO, int H>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_tiled_mfma_kernel(const float* __restrict__ A,
                                                              const float* __restrict__ W,
                                                              TO* __restrict__ C, int M, int N, int K,
                                                              long lda, long ldw, long ldc) {
  constexpr int BM = 64 * H, BN = 64 * H;
  __shared__ __attribute__((aligned(16))) float As[BK][BM + PAD];
  __shared__ __attribute__((aligned(16))) float Ws[BK][BN + PAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int wm = (wave & 1) * 32 * H, wn = (wave >> 1) * 32 * H;   // this wave's corner of the block's tile
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lrow = tid / 4, lk = (tid % 4) * 4;   // loader: rows lrow (and lrow + 64), four k from lk
  // rows whose four k are one aligned 16-byte piece are loaded as one
  const bool a_wide = lda % 4 == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0;
  const bool w_wide = ldw % 4 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;

  float16v acc[H][H], total[H][H];
#pragma unroll
  for (int i = 0; i < H; ++i)
#pragma unroll
    for (int j = 0; j < H; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = total[i][j][e] = 0.f;

  float ar[H][4], wr[H][4];
  auto fetch = [&](int k0) {
    const int k = k0 + lk;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const int m = m0 + lrow + 64 * h, n = n0 + lrow + 64 * h;
      if (a_wide && m < M && k + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(A + (size_t)m * lda + k);
        ar[h][0] = v.x; ar[h][1] = v.y; ar[h][2] = v.z; ar[h][3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) ar[h][i] = (m < M && k + i < K) ? A[(size_t)m * lda + k + i] : 0.f;
      }
      if (w_wide && n < N && k + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(W + (size_t)n * ldw + k);
        wr[h][0] = v.x; wr[h][1] = v.y; wr[h][2] = v.z; wr[h][3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) wr[h][i] = (n < N && k + i < K) ? W[(size_t)n * ldw + k + i] : 0.f;
      }
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 > 0 && k0 % kPiece == 0) {
#pragma unroll
      for (int i = 0; i < H; ++i)
#pragma unroll
        for (int j = 0; j < H; ++j) {
          total[i][j] += acc[i][j];
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        }
    }
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        As[lk + i][lrow + 64 * h] = ar[h][i];
        Ws[lk + i][lrow + 64 * h] = wr[h][i];
      }
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float a[H], w[H];
#pragma unroll
      for (int h = 0; h < H; ++h) {
        a[h] = As[kk + g][wm + 32 * h + r];
        w[h] = Ws[kk + g][wn + 32 * h + r];
      }
#pragma unroll
      for (int i = 0; i < H; ++i)
#pragma unroll
        for (int j = 0; j < H; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], w[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // acc[i][j][4 q + e] = C[m0 + wm + 32 i + 8 q + 4 g + e][n0 + wn + 32 j + r]
#pragma unroll
  for (int i = 0; i < H; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + wm + 32 * i + 8 * q + 4 * g + e;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < H; ++j) {
          const int n = n0 + wn + 32 * j + r;
          if (n < N) Elem<TO>::store(C + (size_t)m * ldc + n, total[i][j][4 * q + e] + acc[i][j][4 * q + e]);
        }
      }
}

// Few rows (M <= 16, float32): the tiles above leave most of a block idle.  Here a lane owns
// one weight row and walks it with 16-byte loads, a cache line in eight loads one after the other; the activations are the same for every lane
// (the compiler reads them through the scalar path).  The order of the sum is the one of the
// tiled kernel, bit for bit: k ascending within a piece of kPiece, the pieces' sums added to the
// total one after the other; so a row's result is still the same whatever the batch holds.
// With `partial` a wave sums one piece only and writes it to partial[piece][M][N]; the second
// kernel adds the pieces in order (for matrices of too few rows to fill the GPU otherwise).
template <int MT>
__global__ __launch_bounds__(64) void gemm_fewrows_kernel(const float* __restrict__ A,
                                                          const float* __restrict__ W,
                                                          float* __restrict__ C, float* __restrict__ partial,
                                                          int M, int N, int K, long lda, long ldw, long ldc) {
  const int lane = threadIdx.x;
  const int n = blockIdx.x * 64 + lane;
  const float* wrow = W + (size_t)min(n, N - 1) * ldw;
  const int pieces = (K + kPiece - 1) / kPiece;
  const int p_begin = partial ? blockIdx.y : 0;
  const int p_end = partial ? p_begin + 1 : pieces;
  float total[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) total[m] = 0.f;
  for (int p = p_begin; p < p_end; ++p) {
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.f;
    const int k_end = min(K, (p + 1) * kPiece);
#pragma unroll 8
    for (int k = p * kPiece; k < k_end; k += 4) {
      const float4 w = *reinterpret_cast<const float4*>(wrow + k);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float4 a = *reinterpret_cast<const float4*>(A + (size_t)min(m, M - 1) * lda + k);
        acc[m] = fmaf(a.x, w.x, acc[m]);
        acc[m] = fmaf(a.y, w.y, acc[m]);
        acc[m] = fmaf(a.z, w.z, acc[m]);
        acc[m] = fmaf(a.w, w.w, acc[m]);
      }
    }
    if (partial) {
      if (n < N) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
          if (m < M) partial[((size_t)p * M + m) * N + n] = acc[m];
      }
      return;
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) total[m] += acc[m];
  }
  if (n < N) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (m < M) C[(size_t)m * ldc + n] = total[m];
  }
}

__global__ __launch_bounds__(256) void gemm_fewrows_add_kernel(const float* __restrict__ partial,
                                                               float* __restrict__ C, int M, int N,
                                                               int pieces, long ldc) {
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (n >= N) return;
  float total = 0.f;
  for (int p = 0; p < pieces; ++p) total += partial[((size_t)p * M + m) * N + n];
  C[(size_t)m * ldc + n] = total;
}

// float32 in and out, M <= 16, K and the row strides multiples of 4, 16-byte aligned rows.
// partial: null, or room for ceil(K / 256) * M * N floats: then every piece of K has a wave of its own.
TK_API int tk_gemm_fewrows(const float* A, const float* W, float* C, float* partial, int M, int N, int K,
                           long lda, long ldw, long ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K < 4 || K % 4 != 0 || lda % 4 != 0 || ldw % 4 != 0) return -1;
  if (reinterpret_cast<uintptr_t>(A) % 16 != 0 || reinterpret_cast<uintptr_t>(W) % 16 != 0) return -1;
  const int pieces = (K + kPiece - 1) / kPiece;
  if (pieces > 65535) return -1;
  dim3 grid((N + 63) / 64, partial ? pieces : 1);
#define TK_FEW(MT_) gemm_fewrows_kernel<MT_><<<grid, 64, 0, stream>>>(A, W, C, partial, M, N, K, lda, ldw, ldc)
  if (M == 1) TK_FEW(1);
  else if (M == 2) TK_FEW(2);
  else if (M <= 4) TK_FEW(4);
  else if (M <= 8) TK_FEW(8);
  else TK_FEW(16);
#undef TK_FEW
  if (partial)
    gemm_fewrows_add_kernel<<<dim3((N + 255) / 256, M), 256, 0, stream>>>(partial, C, M, N, pieces, ldc);
  return launch_status();
}

// in_dtype / out_dtype: 0 = float32, 1 = bfloat16
TK_API int tk_gemm_tiled(int in_dtype, int out_dtype, const void* A, const void* W, void* C, int M,
                         int N, int K, long lda, long ldw, long ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K < 0) return -1;
  // tiles of 128 x 128 if they give every CU a block, else of 64 x 64
  const long big = (long)((N + 127) / 128) * ((M + 127) / 128);
  const int H = big >= 256 ? 2 : 1;
  dim3 grid((N + 64 * H - 1) / (64 * H), (M + 64 * H - 1) / (64 * H));
  if (grid.y > 65535) return -1;
#define TK_TILED(TI_, TO_)                                                                         \
  {                                                                                                \
    if (H == 2)                                                                                    \
      gemm_tiled_kernel<TI_, TO_, 2><<<grid, 256, 0, stream>>>((const TI_*)A, (const TI_*)W,       \
                                                               (TO_*)C, M, N, K, lda, ldw, ldc);   \
    else                                                                                           \
      gemm_tiled_kernel<TI_, TO_, 1><<<grid, 256, 0, stream>>>((const TI_*)A, (const TI_*)W,       \
                                                               (TO_*)C, M, N, K, lda, ldw, ldc);   \
  }
  if (in_dtype == 0 && out_dtype == 0) {
    // float32 operands: the matrix-core form (the same bits)
    if (H == 2) gemm_tiled_mfma_kernel<float, 2><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (float*)C, M, N, K, lda, ldw, ldc);
    else gemm_tiled_mfma_kernel<float, 1><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (float*)C, M, N, K, lda, ldw, ldc);
  }
  else if (in_dtype == 1 && out_dtype == 1) TK_TILED(bf16_t, bf16_t)
  else if (in_dtype == 1 && out_dtype == 0) TK_TILED(bf16_t, float)
  else return -1;
#undef TK_TILED
  return launch_status();
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_gemm_tiled)
TK_SLOTS(tk_gemm_fewrows)
