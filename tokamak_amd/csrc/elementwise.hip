// Memory-bound kernels of one step: embedding gather, residual add + RMSNorm,
// rotary tables, per-head q/k norm + rotation + cache write, SiLU-gate product.
// The residual stream is float32 in both dtypes; norm statistics, rotation
// angles and the residual sum are float32.
#include "common.h"
#include "slots.h"

using namespace tk;

// ---------------------------------------------------------------------------
// embedding: resid[n, :] = float(table[ids[n], :]); an id outside [0, V) gives NaN
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ resid, int H, int V) {
  const int n = blockIdx.x;
  const int id = ids[n];
  float* out = resid + (size_t)n * H;
  if (id < 0 || id >= V) {
    for (int d = threadIdx.x; d < H; d += blockDim.x) out[d] = __uint_as_float(0x7fc00000u);
    return;
  }
  const T* row = table + (size_t)id * H;
  for (int d = threadIdx.x; d < H; d += blockDim.x) out[d] = Elem<T>::load(row + d);
}

TK_API int tk_embed_gather(int dtype, const void* table, const int* ids, float* resid, int N, int H,
                           int V, hipStream_t stream) {
  if (N <= 0) return 0;
  if (dtype == 0)
    embed_gather_kernel<float><<<N, 256, 0, stream>>>((const float*)table, ids, resid, H, V);
  else
    embed_gather_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)table, ids, resid, H, V);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Token ids that are still on the GPU: ids[slots[i]] = sampled[rows[i]].  A step may be
// launched before the host has read the tokens that the step before it sampled; its
// descriptor then names, for such a token, the row of the sampler's output to take it from.
// ---------------------------------------------------------------------------
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ sampled,
                                   const int* __restrict__ slots, const int* __restrict__ rows, int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) ids[slots[i]] = sampled[rows[i]];
}

TK_API int tk_feed_tokens(int* ids, const int* sampled, const int* slots, const int* rows, int count,
                          hipStream_t stream) {
  if (count <= 0) return 0;
  feed_tokens_kernel<<<(count + 255) / 256, 256, 0, stream>>>(ids, sampled, slots, rows, count);
  return launch_status();
}

// ---------------------------------------------------------------------------
// residual add + RMSNorm over rows of width H.
//   x = resid[row] (+ delta[row]);  if write_resid: resid[row] = x
//   out[m] = x * rsqrt(mean(x^2) + eps) * weight
// row = rows ? rows[m] : m.  With `rows`, write_resid must be 0 (a row could be
// named twice).
// ---------------------------------------------------------------------------
// delta may come as `parts` float32 partial sums, part_stride elements apart
// (a split-K product's output): they are added in order.
template <typename TD> struct Load4;
template <> struct Load4<float> {
  static __device__ __forceinline__ float4 at(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <> struct Load4<bf16_t> {
  static __device__ __forceinline__ float4 at(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
};
template <typename T> struct Store4;
template <> struct Store4<float> {
  static __device__ __forceinline__ void at(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Store4<bf16_t> {
  static __device__ __forceinline__ void at(bf16_t* p, float4 v) {
    uint2 u;
    u.x = pack_bf16x2(v.x, v.y);
    u.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

// Vector form: H a multiple of 4 and at most 4 * kNormGroups * blockDim.  A thread
// keeps its elements of the row in registers, and all loads of the partial sums
// are issued before the first add, so a row costs about one memory round trip.
constexpr int kNormGroups = 4;

template <typename T, typename TD>
__global__ __launch_bounds__(1024) void add_rmsnorm_vec_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, int parts, long part_stride,
    const int* __restrict__ rows, const float* __restrict__ weight, T* __restrict__ out, int H,
    float eps, int write_resid) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  const TD* dl = delta ? delta + row * H : nullptr;
  float4 xv[kNormGroups], wv[kNormGroups];
  float ss = 0.f;
  // the norm's weight is asked for with the stream, not after the rows' sums are known (a
  // memory round trip less in a kernel that is little else)
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    wv[g] = d < H ? *reinterpret_cast<const float4*>(weight + d) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    xv[g] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < H) {
      float4 v = *reinterpret_cast<const float4*>(x + d);
      if (dl) {
        int p = 0;
        for (; p + 8 <= parts; p += 8) {   // eight partial sums in flight, added in split order
          float4 q[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) q[u] = Load4<TD>::at(dl + (size_t)(p + u) * part_stride + d);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            v.x += q[u].x;
            v.y += q[u].y;
            v.z += q[u].z;
            v.w += q[u].w;
          }
        }
        for (; p + 4 <= parts; p += 4) {
          const float4 a = Load4<TD>::at(dl + (size_t)p * part_stride + d);
          const float4 b = Load4<TD>::at(dl + (size_t)(p + 1) * part_stride + d);
          const float4 c = Load4<TD>::at(dl + (size_t)(p + 2) * part_stride + d);
          const float4 e = Load4<TD>::at(dl + (size_t)(p + 3) * part_stride + d);
          v.x = (((v.x + a.x) + b.x) + c.x) + e.x;
          v.y = (((v.y + a.y) + b.y) + c.y) + e.y;
          v.z = (((v.z + a.z) + b.z) + c.z) + e.z;
          v.w = (((v.w + a.w) + b.w) + c.w) + e.w;
        }
        for (; p < parts; ++p) {
          const float4 a = Load4<TD>::at(dl + (size_t)p * part_stride + d);
          v.x += a.x;
          v.y += a.y;
          v.z += a.z;
          v.w += a.w;
        }
        if (write_resid) *reinterpret_cast<float4*>(x + d) = v;
      }
      xv[g] = v;
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    if (d < H) {
      const float4 w = wv[g];
      Store4<T>::at(o + d, make_float4(xv[g].x * rstd * w.x, xv[g].y * rstd * w.y,
                                       xv[g].z * rstd * w.z, xv[g].w * rstd * w.w));
    }
  }
}

template <typename T, typename TD>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   int parts, long part_stride, const int* __restrict__ rows,
                                   const float* __restrict__ weight, T* __restrict__ out, int H,
                                   float eps, int write_resid) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  const TD* dl = delta ? delta + row * H : nullptr;
  float ss = 0.f;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (dl) {
      for (int p = 0; p < parts; ++p) v += Elem<TD>::load(dl + (size_t)p * part_stride + d);
      if (write_resid) x[d] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (dl && !write_resid)
      for (int p = 0; p < parts; ++p) v += Elem<TD>::load(dl + (size_t)p * part_stride + d);
    Elem<T>::store(o + d, v * rstd * weight[d]);
  }
}

// delta_f32: delta is float32 (possibly `parts` partial sums) whatever the dtype
TK_API int tk_add_rmsnorm(int dtype, float* resid, const void* delta, int delta_f32, int parts,
                          long part_stride, const int* rows, const float* weight, void* out, int M,
                          int H, float eps, int write_resid, hipStream_t stream) {
  if (M <= 0) return 0;
  if (rows && write_resid) return -1;
  if (parts < 1 || (parts > 1 && !delta_f32 && dtype != 0)) return -1;
  // vector form when the row fits a block's registers and everything is 16-byte aligned
  // one element group per thread when rows are few (short latency chain), four when many
  int threads = 64;
  while (threads < 1024 && threads * 4 * (M >= 512 ? kNormGroups : 1) < H) threads *= 2;
  const bool vec = H % 4 == 0 && H <= threads * 4 * kNormGroups && part_stride % 4 == 0 &&
                   ((uintptr_t)resid % 16 == 0) && ((uintptr_t)delta % 16 == 0) &&
                   ((uintptr_t)weight % 16 == 0) && ((uintptr_t)out % 16 == 0);
#define TK_NORM(KERNEL, T_, TD_)                                                                 \
  KERNEL<T_, TD_><<<M, threads, 0, stream>>>(resid, (const TD_*)delta, parts, part_stride, rows, \
                                             weight, (T_*)out, H, eps, write_resid)
  if (vec) {
    if (dtype == 0) TK_NORM(add_rmsnorm_vec_kernel, float, float);
    else if (delta_f32) TK_NORM(add_rmsnorm_vec_kernel, bf16_t, float);
    else TK_NORM(add_rmsnorm_vec_kernel, bf16_t, bf16_t);
  } else {
    threads = 256;
    if (dtype == 0) TK_NORM(add_rmsnorm_kernel, float, float);
    else if (delta_f32) TK_NORM(add_rmsnorm_kernel, bf16_t, float);
    else TK_NORM(add_rmsnorm_kernel, bf16_t, bf16_t);
  }
#undef TK_NORM
  return launch_status();
}

// ---------------------------------------------------------------------------
// rotary tables: angle = float(pos) * inv_freq[j]  (one float32 product, as the
// formula is written), cos/sin [N, half]
// ---------------------------------------------------------------------------
__global__ void rope_tables_kernel(const int* __restrict__ positions,
                                   const float* __restrict__ inv_freq, float* __restrict__ cos_t,
                                   float* __restrict__ sin_t, int N, int half) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * half) return;
  const int n = i / half, j = i - n * half;
  const float angle = __fmul_rn((float)positions[n], inv_freq[j]);
  cos_t[i] = cosf(angle);
  sin_t[i] = sinf(angle);
}

TK_API int tk_rope_tables(const int* positions, const float* inv_freq, float* cos_t, float* sin_t,
                          int N, int half, hipStream_t stream) {
  const int total = N * half;
  if (total <= 0) return 0;
  rope_tables_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, cos_t, sin_t, N,
                                                               half);
  return launch_status();
}

// ---------------------------------------------------------------------------
// per-head RMSNorm of q and k, half-split rotation of the first `rot` dims,
// q written out, k and v written into the paged cache.
//
// qkv: [N, (nh + 2*nkv) * hd] (q heads, then k heads, then v heads); with
// nkv_in == 0 the input holds q heads only and nothing is stored.
// Cache pages (page_elems = nkv * hd * ps elements each):
//   K page: [nkv][hd/8][ps][8]   (8 consecutive dims of one token are adjacent,
//                                 then tokens, so lanes that hold consecutive
//                                 tokens read consecutive 16-byte pieces)
//   V page: [nkv][hd/16][ps/4][16][4]  (4 consecutive tokens of one dim adjacent,
//                                 then 16 dims, then groups of 4 tokens: the A
//                                 operand of the PV product, lane (dim, quad),
//                                 is 8 contiguous bytes and a wave reads 512
//                                 contiguous bytes)
// One wave per (token, head), four waves a block, each with an LDS row of its own.
// ---------------------------------------------------------------------------
constexpr int kMaxHeadDim = 512;
constexpr int kPairsPerBlock = 4;  // (token, head) pairs per block, one per wave

template <typename T, typename TIN>
__global__ void qknorm_rope_store_kernel(
    const TIN* __restrict__ qkv, int parts, long part_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ block_tables, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int nh, int nkv_in, int nkv, int hd, int rot, int ps, int max_pages,
    float eps, int num_pairs) {
  __shared__ float vecs[kPairsPerBlock][kMaxHeadDim];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int heads = nh + 2 * nkv_in;
  const int pair = blockIdx.x * kPairsPerBlock + wave;
  if (pair >= num_pairs) return;  // nothing below synchronises across waves
  const int n = pair / heads, head = pair - n * heads;
  float* vec = vecs[wave];
  const int row_width = heads * hd;
  const TIN* src = qkv + (size_t)n * row_width + (size_t)head * hd;
  const bool is_q = head < nh;
  const bool is_k = !is_q && head < nh + nkv_in;
  const float* w = is_q ? q_weight : (is_k ? k_weight : nullptr);

  float ss = 0.f;
  for (int d = lane; d < hd; d += kWave) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += Elem<TIN>::load(src + (size_t)p * part_stride + d);
    vec[d] = v;
    ss += v * v;
  }
  if (is_q || is_k) {
    if (w) {
      ss = wave_sum(ss);
      const float rstd = rsqrtf(ss / (float)hd + eps);
      wave_lds_sync();
      for (int d = lane; d < hd; d += kWave) vec[d] = vec[d] * rstd * w[d];
    }
    wave_lds_sync();
    // out[j] = x[j] cos_j - x[j+half] sin_j ; out[j+half] = x[j+half] cos_j + x[j] sin_j
    const int half = rot / 2;
    float lo[kMaxHeadDim / 2 / kWave], hi[kMaxHeadDim / 2 / kWave];
    int cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      const float c = cos_t[(size_t)n * half + j], s = sin_t[(size_t)n * half + j];
      const float a = vec[j], b = vec[j + half];
      lo[cnt] = a * c - b * s;
      hi[cnt] = b * c + a * s;
    }
    wave_lds_sync();
    cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      vec[j] = lo[cnt];
      vec[j + half] = hi[cnt];
    }
  }
  wave_lds_sync();

  if (is_q) {
    T* dst = q_out + ((size_t)n * nh + head) * hd;
    for (int d = lane; d < hd; d += kWave) Elem<T>::store(dst + d, vec[d]);
    return;
  }
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  const size_t page_elems = (size_t)nkv * hd * ps;
  if (is_k) {
    const int kvh = head - nh;
    T* base = k_cache + (size_t)page * page_elems + (size_t)kvh * hd * ps;
    for (int d = lane; d < hd; d += kWave)
      Elem<T>::store(base + ((size_t)(d >> 3) * ps + off) * 8 + (d & 7), vec[d]);
  } else {
    const int kvh = head - nh - nkv_in;
    T* base = v_cache + (size_t)page * page_elems + (size_t)kvh * hd * ps;
    for (int d = lane; d < hd; d += kWave)
      Elem<T>::store(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), vec[d]);
  }
}

// Fast form for head sizes 64 and 128 rotated over their full width (rot == HD):
// a lane owns 8 consecutive dims of one head (one 16-byte piece), so a wave covers
// 64*8/HD (token, head) pairs; the rotation partner (dim +- HD/2) sits HD/16 lanes away, the
// sum of squares is over HD/8 neighbouring lanes.  The query heads come token by token; the
// pairs behind them are the key heads and then the value heads, each head with its tokens in
// order, so that a wave holds consecutive tokens of one head and its cache writes fall next
// to each other in the page: a key piece (8 dims of one token) beside those of the next
// tokens, and the values of four tokens that fill one quad of a page (bfloat16: exchanged
// through LDS inside the wave) as the page's own 16-byte pieces of two dims by four keys,
// where token by token they are 2-byte stores 8 bytes apart.
template <typename T, typename TIN, int HD>
__global__ __launch_bounds__(256) void qknorm_rope_store_vec_kernel(
    const TIN* __restrict__ qkv, int parts, long part_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ block_tables,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int N, int nh, int nkv_in,
    int nkv, int ps, int max_pages, float eps, long num_pairs) {
  constexpr int LPH = HD / 8;  // lanes per head
  __shared__ uint4 s_quad[sizeof(T) == 2 ? 256 : 1];
  const long slot = ((long)blockIdx.x * blockDim.x + threadIdx.x) / LPH;  // (token, head) pair
  if (slot >= num_pairs) return;  // whole LPH-lane groups leave together
  const int sub = threadIdx.x % LPH, d0 = sub * 8;
  const int heads = nh + 2 * nkv_in;
  const long q_pairs = (long)N * nh;
  int n, head;
  if (slot < q_pairs) {
    n = (int)((unsigned)slot / (unsigned)nh);
    head = (int)((unsigned)slot - (unsigned)n * (unsigned)nh);
  } else {
    const unsigned behind = (unsigned)(slot - q_pairs), kv = behind / (unsigned)N;
    n = (int)(behind - kv * (unsigned)N);
    head = nh + (int)kv;
  }
  const bool is_q = head < nh, is_k = !is_q && head < nh + nkv_in;
  const TIN* src = qkv + (size_t)n * heads * HD + (size_t)head * HD + d0;
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = 0.f;
  for (int p = 0; p < parts; ++p) {
    const float4 a = Load4<TIN>::at(src + (size_t)p * part_stride);
    const float4 b = Load4<TIN>::at(src + (size_t)p * part_stride + 4);
    x[0] += a.x; x[1] += a.y; x[2] += a.z; x[3] += a.w;
    x[4] += b.x; x[5] += b.y; x[6] += b.z; x[7] += b.w;
  }
  if (is_q || is_k) {
    const float* w = is_q ? q_weight : k_weight;
    const int j0 = d0 % (HD / 2);  // index into the cos/sin row
    const float4 c0 = *reinterpret_cast<const float4*>(cos_t + (size_t)n * (HD / 2) + j0);
    const float4 c1 = *reinterpret_cast<const float4*>(cos_t + (size_t)n * (HD / 2) + j0 + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sin_t + (size_t)n * (HD / 2) + j0);
    const float4 s1 = *reinterpret_cast<const float4*>(sin_t + (size_t)n * (HD / 2) + j0 + 4);
    const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
      for (int m = LPH / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
      const float rstd = rsqrtf(ss / (float)HD + eps);
      const float4 w0 = *reinterpret_cast<const float4*>(w + d0);
      const float4 w1 = *reinterpret_cast<const float4*>(w + d0 + 4);
      const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = x[e] * rstd * wv[e];
    }
    // first half: x cos - partner sin; second half: x cos + partner sin
    const float sign = (d0 < HD / 2) ? -1.f : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float partner = __shfl_xor(x[e], LPH / 2, kWave);
      x[e] = x[e] * cs[e] + sign * partner * sn[e];
    }
  }
  if (is_q) {
    Store4<T>::at(q_out + ((size_t)n * nh + head) * HD + d0, make_float4(x[0], x[1], x[2], x[3]));
    Store4<T>::at(q_out + ((size_t)n * nh + head) * HD + d0 + 4, make_float4(x[4], x[5], x[6], x[7]));
    return;
  }
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  const size_t page_elems = (size_t)nkv * HD * ps;
  if (is_k) {
    T* base = k_cache + (size_t)page * page_elems + (size_t)(head - nh) * HD * ps;
    T* dst = base + ((size_t)sub * ps + off) * 8;  // dims d0 .. d0+7 of this token: one 8-element piece
    Store4<T>::at(dst, make_float4(x[0], x[1], x[2], x[3]));
    Store4<T>::at(dst + 4, make_float4(x[4], x[5], x[6], x[7]));
  } else {
    T* base = v_cache + (size_t)page * page_elems + (size_t)(head - nh - nkv_in) * HD * ps;
    if constexpr (sizeof(T) == 2) {
      // Four pairs in a row (a "quad" of this wave) that are four consecutive tokens of one
      // request and head and fill one quad of keys in a page?
      constexpr int QL = 4 * LPH;  // lanes of a quad
      const int lane = threadIdx.x & 63, t = (lane / LPH) & 3;
      const int first = lane / QL * QL + sub;  // the lane with these dims in the quad's first pair
      const int req = req_of_token[n];
      const bool fits = n == __shfl(n, first, kWave) + t && pos == __shfl(pos, first, kWave) + t &&
                        req == __shfl(req, first, kWave) && head == __shfl(head, first, kWave) && ((pos - t) & 3) == 0;
      const unsigned long long all = QL == 64 ? ~0ull : ((1ull << (QL & 63)) - 1) << (lane / QL * QL);
      if ((__builtin_amdgcn_ballot_w64(fits) & all) == all) {
        // every lane leaves its four dim pairs; lane t of the quad takes pair t of all four tokens
        s_quad[threadIdx.x] = make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]),
                                         pack_bf16x2(x[6], x[7]));
        wave_lds_sync();
        const unsigned* words = reinterpret_cast<const unsigned*>(s_quad);
        const int quad0 = (int)threadIdx.x / QL * QL + sub;  // thread of the quad's first pair, these dims
        unsigned r[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = words[(quad0 + k * LPH) * 4 + t];  // token k: dims d, d + 1
        const int d = d0 + 2 * t;
        uint4 piece;  // [dim d: keys 0..3][dim d + 1: keys 0..3]
        piece.x = (r[0] & 0xffffu) | (r[1] << 16);
        piece.y = (r[2] & 0xffffu) | (r[3] << 16);
        piece.z = (r[0] >> 16) | (r[1] & 0xffff0000u);
        piece.w = (r[2] >> 16) | (r[3] & 0xffff0000u);
        *reinterpret_cast<uint4*>(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4) = piece;
        return;
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = d0 + e;
      Elem<T>::store(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), x[e]);
    }
  }
}

// in_f32: qkv is float32 (possibly `parts` partial sums, part_stride elements apart)
TK_API int tk_qknorm_rope_store(int dtype, const void* qkv, int in_f32, int parts, long part_stride,
                                const float* q_weight, const float* k_weight, const float* cos_t,
                                const float* sin_t, const int* positions, const int* req_of_token,
                                const int* block_tables, void* q_out, void* k_cache, void* v_cache,
                                int N, int nh, int nkv_in, int nkv, int hd, int rot, int ps,
                                int max_pages, float eps, hipStream_t stream) {
  if (N <= 0) return 0;
  if (hd > kMaxHeadDim || hd % 16 != 0 || ps % 4 != 0 || rot > hd || rot % 2 != 0) return -1;
  if (nkv_in != 0 && nkv_in != nkv) return -1;
  if (parts < 1 || (parts > 1 && !in_f32 && dtype != 0)) return -1;
  const long pairs = (long)N * (nh + 2 * nkv_in);
  if (pairs > 0x7fffffffL) return -1;
  if ((hd == 128 || hd == 64) && rot == hd && part_stride % 4 == 0 && (uintptr_t)qkv % 16 == 0 &&
      (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)cos_t % 16 == 0 &&
      (uintptr_t)sin_t % 16 == 0 && (!q_weight || (uintptr_t)q_weight % 16 == 0) &&
      (!k_weight || (uintptr_t)k_weight % 16 == 0) && (q_weight != nullptr) == (k_weight != nullptr)) {
    const long lanes = pairs * (hd / 8);
    const unsigned vgrid = (unsigned)((lanes + 255) / 256);
#define TK_QKV(T_, TIN_, HD_)                                                                     \
  qknorm_rope_store_vec_kernel<T_, TIN_, HD_><<<vgrid, 256, 0, stream>>>(                         \
      (const TIN_*)qkv, parts, part_stride, q_weight, k_weight, cos_t, sin_t, positions,          \
      req_of_token, block_tables, (T_*)q_out, (T_*)k_cache, (T_*)v_cache, N, nh, nkv_in, nkv, ps, \
      max_pages, eps, pairs)
    if (hd == 128) {
      if (dtype == 0) TK_QKV(float, float, 128);
      else if (in_f32) TK_QKV(bf16_t, float, 128);
      else TK_QKV(bf16_t, bf16_t, 128);
    } else {
      if (dtype == 0) TK_QKV(float, float, 64);
      else if (in_f32) TK_QKV(bf16_t, float, 64);
      else TK_QKV(bf16_t, bf16_t, 64);
    }
#undef TK_QKV
    return launch_status();
  }
  const unsigned grid = (unsigned)((pairs + kPairsPerBlock - 1) / kPairsPerBlock);
#define TK_QK(T_, TIN_)                                                                          \
  qknorm_rope_store_kernel<T_, TIN_><<<grid, kWave * kPairsPerBlock, 0, stream>>>(               \
      (const TIN_*)qkv, parts, part_stride, q_weight, k_weight, cos_t, sin_t, positions,         \
      req_of_token, block_tables, (T_*)q_out, (T_*)k_cache, (T_*)v_cache, nh, nkv_in, nkv, hd,   \
      rot, ps, max_pages, eps, (int)pairs)
  if (dtype == 0) TK_QK(float, float);
  else if (in_f32) TK_QK(bf16_t, float);
  else TK_QK(bf16_t, bf16_t);
#undef TK_QK
  return launch_status();
}

// ---------------------------------------------------------------------------
// out[n, i] = silu(gu[n, i]) * gu[n, I + i],  silu(z) = z / (1 + exp(-z))
// ---------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / I;
  const int i = (int)(idx - n * I);
  const float g = Elem<T>::load(gu + n * 2 * I + i);
  const float u = Elem<T>::load(gu + n * 2 * I + I + i);
  Elem<T>::store(out + idx, g / (1.f + expf(-g)) * u);
}

// 8 elements a thread (16-byte loads): I a multiple of 8, pointers 16-byte aligned
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                       int I, size_t total8) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const int per_row = I / 8;
  const size_t n = idx / per_row;
  const int i = (int)(idx - n * per_row) * 8;
  const uint4 g = *reinterpret_cast<const uint4*>(gu + n * 2 * I + i);
  const uint4 u = *reinterpret_cast<const uint4*>(gu + n * 2 * I + I + i);
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  uint32_t ow[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
    ow[k] = pack_bf16x2(g0 / (1.f + expf(-g0)) * u0, g1 / (1.f + expf(-g1)) * u1);
  }
  *reinterpret_cast<uint4*>(out + n * I + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

TK_API int tk_silu_mul(int dtype, const void* gu, void* out, int N, int I, hipStream_t stream) {
  if (N <= 0 || I <= 0) return 0;
  const size_t total = (size_t)N * I;
  if (dtype == 1 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t total8 = total / 8;
    silu_mul_bf16x8_kernel<<<(unsigned)((total8 + 255) / 256), 256, 0, stream>>>(
        (const bf16_t*)gu, (bf16_t*)out, I, total8);
    return launch_status();
  }
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0)
    silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
  else
    silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
  return launch_status();
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_add_rmsnorm)
TK_SLOTS(tk_rope_tables)
TK_SLOTS(tk_qknorm_rope_store)
TK_SLOTS(tk_silu_mul)
