// bf16 matrix products on the matrix cores with float32 accumulation.
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

using namespace tk;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

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

  const bf16_t* wp[NT];
  bool wok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int row = n0 + t * 16 + r;
    wok[t] = row < N;
    wp[t] = W + (size_t)(wok[t] ? row : 0) * ldw + kb * 8;
  }
  const bf16_t* ap[MT];
  bool aok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = t * 16 + r;
    aok[t] = row < M;
    ap[t] = A + (size_t)(aok[t] ? row : 0) * lda + kb * 8;
  }

  float4v acc[NT][MT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll 4
  for (int s = s_begin; s < s_end; ++s) {
    const int k = s * 32;
    const bool kok = k + kb * 8 < K;  // K is a multiple of 8: a 16-byte piece is whole or absent
    Frag8 wf[NT], af[MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
      wf[t].u = (wok[t] && kok) ? *reinterpret_cast<const uint4*>(wp[t] + k) : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      af[t].u = (aok[t] && kok) ? *reinterpret_cast<const uint4*>(ap[t] + k) : zero;
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
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = j * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int n = n0 + i * 16 + kb * 4;
      TO* cp = C + (size_t)m * ldc + n;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) Elem<TO>::store(cp + e, acc[i][j][e]);
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
// nt: weight-row tiles (of 16) per block, 1 or 2; waves: how many waves split K.
TK_API int tk_gemm_skinny(int out_dtype, const void* A, const void* W, void* C, int M, int N, int K,
                          long lda, long ldw, long ldc, int nt, int waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0) return -1;
  if (out_dtype == 0) return pick_tiles<float>(nt, waves, A, W, C, M, N, K, lda, ldw, ldc, stream);
  if (out_dtype == 1) return pick_tiles<bf16_t>(nt, waves, A, W, C, M, N, K, lda, ldw, ldc, stream);
  return -1;
}
