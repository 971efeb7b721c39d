// Two microbenchmarks that say what this GPU can reach, as denominators beside the
// published peaks: streaming device memory (read only, and copy) and back-to-back
// bf16 MFMA instructions from registers.  The caller times the launches with events.
#include "common.h"

using namespace tk;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Each thread reads 16 bytes at a time, grid-strided, with streaming (non-temporal)
// loads as the decode kernels use for weights; the xor of everything read goes to one
// word per block so that no load can be dropped.
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ src, size_t n16,
                                                          unsigned* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  u32x4 acc = {0u, 0u, 0u, 0u};
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const u32x4 a = __builtin_nontemporal_load(src + i);
    const u32x4 b = __builtin_nontemporal_load(src + i + stride);
    const u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride);
    const u32x4 d = __builtin_nontemporal_load(src + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  const unsigned x = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (x == 0x9e3779b9u) sink[blockIdx.x] = x;  // practically never; keeps the loads alive
}

__global__ __launch_bounds__(256) void stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                          size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// `chains` independent accumulators per wave, `iters` rounds: the matrix cores are fed
// from registers only.  shape 0: 16x16x32 (16,384 flop an instruction); 1: 32x32x16 (32,768).
template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = (__bf16)(0.001f * (float)((threadIdx.x + e) & 7));
    b[e] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + e) & 7));
  }
  float total = 0.f;
  if constexpr (SHAPE == 0) {
    float4v acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = float4v{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int c = 0; c < 8; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
  } else {
    float16v acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[c][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int e = 0; e < 16; ++e) total += acc[c][e];
  }
  if (total == 12345.678f) sink[blockIdx.x] = total;  // keeps the products alive
}

// bytes must be a multiple of 16; sink holds >= `blocks` words.
TK_API int tk_peak_read(const void* src, size_t bytes, void* sink, int blocks, hipStream_t stream) {
  if (bytes == 0 || bytes % 16 != 0 || blocks <= 0 || blocks > 65535) return -1;
  stream_read_kernel<<<blocks, 256, 0, stream>>>((const u32x4*)src, bytes / 16, (unsigned*)sink);
  return launch_status();
}

TK_API int tk_peak_copy(const void* src, void* dst, size_t bytes, int blocks, hipStream_t stream) {
  if (bytes == 0 || bytes % 16 != 0 || blocks <= 0 || blocks > 65535) return -1;
  stream_copy_kernel<<<blocks, 256, 0, stream>>>((const u32x4*)src, (u32x4*)dst, bytes / 16);
  return launch_status();
}

// Returns the flop count of the launch through *flops (blocks * 4 waves * iters * ...).
TK_API int tk_peak_mfma(int shape, int blocks, int iters, void* sink, double* flops, hipStream_t stream) {
  if (blocks <= 0 || blocks > 65535 || iters <= 0 || (shape != 0 && shape != 1)) return -1;
  if (shape == 0) {
    mfma_kernel<0><<<blocks, 256, 0, stream>>>(iters, (float*)sink);
    *flops = (double)blocks * 4 * iters * 8 * 16384.0;
  } else {
    mfma_kernel<1><<<blocks, 256, 0, stream>>>(iters, (float*)sink);
    *flops = (double)blocks * 4 * iters * 4 * 32768.0;
  }
  return launch_status();
}
