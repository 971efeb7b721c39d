// Shared device helpers for the gfx950 kernels: bf16 storage conversions,
// 64-lane wave reductions, launch-error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tk {

typedef uint16_t bf16_t;  // raw bfloat16 bits; arithmetic is always done in float

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// round-to-nearest-even; NaN stays NaN.  gfx950 converts in hardware
// (v_cvt_pk_bf16_f32), which the compiler emits for these casts.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t f = {lo, hi};
  const bf16x2_t v = __builtin_convertvector(f, bf16x2_t);
  return *reinterpret_cast<const uint32_t*>(&v);
}

__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  return static_cast<bf16_t>(pack_bf16x2(f, 0.f) & 0xffffu);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_float(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = float_to_bf16(v); }
};

// Four consecutive elements p[0..3] of which the first `valid` exist.  `wide`: p is 16-byte
// (float32) or 8-byte (bfloat16) aligned, so four that all exist go out as one store: a
// wave's 4-byte stores of an MFMA result tile are sixteen scattered pieces per row of it and
// cost a product of 64 rows a fifth of its time.
template <typename T>
__device__ __forceinline__ void store_four(T* p, float a, float b, float c, float d, int valid, bool wide);
template <>
__device__ __forceinline__ void store_four<float>(float* p, float a, float b, float c, float d, int valid, bool wide) {
  if (wide && valid >= 4) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
    return;
  }
  if (valid > 0) p[0] = a;
  if (valid > 1) p[1] = b;
  if (valid > 2) p[2] = c;
  if (valid > 3) p[3] = d;
}
template <>
__device__ __forceinline__ void store_four<bf16_t>(bf16_t* p, float a, float b, float c, float d, int valid, bool wide) {
  if (wide && valid >= 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
    return;
  }
  if (valid > 0) p[0] = float_to_bf16(a);
  if (valid > 1) p[1] = float_to_bf16(b);
  if (valid > 2) p[2] = float_to_bf16(c);
  if (valid > 3) p[3] = float_to_bf16(d);
}
// Whether rows of `ld` elements starting at p keep every fourth element aligned for store_four.
template <typename T>
__device__ __forceinline__ bool rows_take_wide_stores(const T* p, long ld) {
  return (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0 && ld % 4 == 0;
}

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

// Orders one wave's LDS accesses (a wave's LDS instructions execute in order; this
// keeps the compiler from moving them across the point).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
// Every thread of the block must call it; all get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nwaves; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

}  // namespace tk

#define TK_API extern "C" __attribute__((visibility("default")))
