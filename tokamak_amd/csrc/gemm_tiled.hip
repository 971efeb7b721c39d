// C[M,N] = A[M,K] * W[N,K]^T with float32 multiply-add and float32 accumulation
// for any M, N, K.  It is the true 32-bit matrix product of the float32 path
// (no reduced-precision matrix mode), and also accepts bf16 inputs.  Every
// output element is summed by one thread in one fixed order, so a row's result does
// not depend on which other rows are in the batch: k ascending within pieces of
// kPiece, whose sums are added to the total one after the other.  The two levels
// keep the rounding error of a sum over K terms near sqrt(kPiece) + sqrt(K / kPiece)
// units instead of sqrt(K) (K is 25,600 in the widest feed-forward).
#include "common.h"

using namespace tk;

constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;
constexpr int kPiece = 256;  // k values summed before they join the total (a multiple of BK)

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TI* __restrict__ A,
                                                         const TI* __restrict__ W,
                                                         TO* __restrict__ C, int M, int N, int K,
                                                         long lda, long ldw, long ldc) {
  __shared__ float As[BK][BM + PAD];
  __shared__ float Ws[BK][BN + PAD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int ty = tid / 16, tx = tid % 16;
  const int lrow = tid / 4, lk = (tid % 4) * 4;

  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 > 0 && k0 % kPiece == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    {
      const int m = m0 + lrow;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        As[lk + i][lrow] = (m < M && k < K) ? Elem<TI>::load(A + (size_t)m * lda + k) : 0.f;
      }
      const int n = n0 + lrow;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        Ws[lk + i][lrow] = (n < N && k < K) ? Elem<TI>::load(W + (size_t)n * ldw + k) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) Elem<TO>::store(C + (size_t)m * ldc + n, total[i][j] + acc[i][j]);
    }
  }
}

// Few rows (M <= 16, float32): the tiles above leave most of a block idle and read the weights
// in pieces of 64 bytes.  Here a lane owns one weight row and walks it with 16-byte loads, a
// cache line in eight loads one after the other; the activations are the same for every lane
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
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return -1;
  if (in_dtype == 0 && out_dtype == 0)
    gemm_tiled_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W,
                                                             (float*)C, M, N, K, lda, ldw, ldc);
  else if (in_dtype == 1 && out_dtype == 1)
    gemm_tiled_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(
        (const bf16_t*)A, (const bf16_t*)W, (bf16_t*)C, M, N, K, lda, ldw, ldc);
  else if (in_dtype == 1 && out_dtype == 0)
    gemm_tiled_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W,
                                                              (float*)C, M, N, K, lda, ldw, ldc);
  else
    return -1;
  return launch_status();
}
