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
