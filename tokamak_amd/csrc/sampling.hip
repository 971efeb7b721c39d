// Token selection from float32 logits [M, V]: greedy argmax, and temperature /
// top-k / top-p sampling with a per-request counter-based random number.
//
// Filter order and rules follow the reference sampler
// (src/tokamak/sampling/sampler.py:34-39,64-84): divide by temperature; top-k
// keeps every logit >= the k-th largest (ties at the threshold survive); top-p
// sorts descending and drops a token iff the mass ranked before it already
// reaches top_p (the best token always survives); softmax over what is left;
// one draw.  No sort is done here: both thresholds are found by bisection over
// the ordered-integer image of the float values, each probe one pass over the
// row (which sits in L2).
#include "common.h"

using namespace tk;

// ---------------------------------------------------------------------------
// argmax: first maximum wins (lowest index), NaN never wins.  A row is cut into
// kArgmaxSegments pieces, one block each, so that a few rows still fill the chip;
// a second small kernel picks among the pieces' winners.
// ---------------------------------------------------------------------------
constexpr int kArgmaxSegments = 32;
constexpr int kArgmaxThreads = 256;

__device__ __forceinline__ void argmax_take(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) {
    bv = v;
    bi = i;
  }
}

__global__ __launch_bounds__(kArgmaxThreads) void argmax_segments_kernel(
    const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i, int V,
    long ld) {
  __shared__ float best_v[kArgmaxThreads / kWave];
  __shared__ int best_i[kArgmaxThreads / kWave];
  const int seg = blockIdx.x, r = blockIdx.y;
  const float* row = logits + (size_t)r * ld;
  // segment bounds in whole float4s when the row allows it
  const int per = ((V + kArgmaxSegments - 1) / kArgmaxSegments + 3) & ~3;
  const int begin = seg * per, end = min(V, begin + per);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
  if (vec) {
    for (int i = begin + threadIdx.x * 4; i < end; i += kArgmaxThreads * 4) {
      if (i + 4 <= end) {
        const float4 v = *reinterpret_cast<const float4*>(row + i);
        argmax_take(bv, bi, v.x, i);
        argmax_take(bv, bi, v.y, i + 1);
        argmax_take(bv, bi, v.z, i + 2);
        argmax_take(bv, bi, v.w, i + 3);
      } else {
        for (int j = i; j < end; ++j) argmax_take(bv, bi, row[j], j);
      }
    }
  } else {
    for (int i = begin + threadIdx.x; i < end; i += kArgmaxThreads) argmax_take(bv, bi, row[i], i);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(bv, m, kWave);
    const int oi = __shfl_xor(bi, m, kWave);
    argmax_take(bv, bi, ov, oi);
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    best_v[wave] = bv;
    best_i[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxThreads / kWave; ++w) argmax_take(bv, bi, best_v[w], best_i[w]);
    part_v[r * kArgmaxSegments + seg] = bv;
    part_i[r * kArgmaxSegments + seg] = bi;
  }
}

__global__ __launch_bounds__(kWave) void argmax_pick_kernel(const float* __restrict__ part_v,
                                                            const int* __restrict__ part_i,
                                                            int* __restrict__ out) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float bv = lane < kArgmaxSegments ? part_v[r * kArgmaxSegments + lane] : -INFINITY;
  int bi = lane < kArgmaxSegments ? part_i[r * kArgmaxSegments + lane] : 0x7fffffff;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(bv, m, kWave);
    const int oi = __shfl_xor(bi, m, kWave);
    argmax_take(bv, bi, ov, oi);
  }
  if (lane == 0) out[r] = (bi == 0x7fffffff) ? 0 : bi;
}

// part_v, part_i: scratch of M * tk_argmax_segments() floats and ints.
TK_API int tk_argmax_segments() { return kArgmaxSegments; }

TK_API int tk_argmax(const float* logits, int* out, float* part_v, int* part_i, int M, int V, long ld,
                     hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0 || M > 65535) return -1;
  argmax_segments_kernel<<<dim3(kArgmaxSegments, M), kArgmaxThreads, 0, stream>>>(logits, part_v, part_i, V, ld);
  argmax_pick_kernel<<<M, kWave, 0, stream>>>(part_v, part_i, out);
  return launch_status();
}

// ---------------------------------------------------------------------------
// sampling
// ---------------------------------------------------------------------------
// monotone map float -> uint32 (larger float, larger integer)
__device__ __forceinline__ uint32_t ordered(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float unordered(uint32_t o) {
  const uint32_t u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
  return __uint_as_float(u);
}

// splitmix64-style mix of (seed, counter) -> uniform in [0, 1)
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t counter) {
  uint64_t z = seed * 0x9e3779b97f4a7c15ull + (counter + 1) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  z ^= z >> 31;
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nw = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int t = 0;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  return t;
}

// One block per row.  params rows: temperature, top_k, top_p (floats);
// seeds/counters: the request's seed and how many draws it has made.
// probs_out (optional, [M, V]) receives the final distribution, for tests.
__global__ __launch_bounds__(1024) void sample_kernel(
    const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const unsigned long long* __restrict__ seeds, const unsigned long long* __restrict__ counters,
    int* __restrict__ out, float* __restrict__ probs_out) {
  __shared__ float fs[16];
  __shared__ int is[16];
  __shared__ float seg_prefix[1025];
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  if (!(temperature[r] > 0.f)) return;  // greedy row: the argmax pre-pass has written it
  const float* row = logits + (size_t)r * ld;
  const float inv_t = 1.f / temperature[r];
  const int k = top_k[r];
  const float p_keep = top_p[r];

  float mx = -INFINITY;
  for (int i = tid; i < V; i += nt) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, fs);

  // top-k: the k-th largest scaled logit, by bisection on the ordered image:
  // the largest t with count(x >= t) >= k.
  uint32_t kth = 0;  // ordered(-inf) is > 0, so 0 keeps everything
  if (k > 0 && k < V) {
    uint32_t lo = 0, hi = 0xffffffffu;  // invariant: count(>= lo) >= k
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      int c = 0;
      for (int i = tid; i < V; i += nt) c += ordered(row[i] * inv_t) >= mid;
      c = block_sum_int(c, is);
      if (c >= k) lo = mid; else hi = mid - 1;
    }
    kth = lo;
  }

  // softmax normaliser over what top-k kept
  float z = 0.f;
  for (int i = tid; i < V; i += nt) {
    const float x = row[i] * inv_t;
    if (ordered(x) >= kth) z += expf(x - mx);
  }
  z = block_sum(z, fs);

  // top-p: keep x iff mass of kept values strictly greater than x is < top_p.
  // The kept set is {x >= cut}; cut = smallest t with mass(> t) < top_p.
  uint32_t cut = kth;
  if (p_keep < 1.f) {
    uint32_t lo = kth, hi = ordered(mx);  // mass(> hi) = 0 < top_p always
    while (lo < hi) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      float mass = 0.f;
      for (int i = tid; i < V; i += nt) {
        const float x = row[i] * inv_t;
        const uint32_t o = ordered(x);
        if (o >= kth && o > mid) mass += expf(x - mx);
      }
      mass = block_sum(mass, fs) / z;
      if (mass < p_keep) hi = mid; else lo = mid + 1;
    }
    cut = lo;
  }

  // final distribution over {x >= cut}; contiguous segment per thread so the
  // draw walks tokens in index order
  const int seg = (V + nt - 1) / nt;
  const int b = tid * seg, e = (b + seg < V) ? b + seg : V;
  float mine = 0.f;
  for (int i = b; i < e; ++i) {
    const float x = row[i] * inv_t;
    if (ordered(x) >= cut) mine += expf(x - mx);
  }
  __syncthreads();
  seg_prefix[tid + 1] = mine;
  if (tid == 0) seg_prefix[0] = 0.f;
  __syncthreads();
  if (tid == 0)
    for (int i = 1; i <= nt; ++i) seg_prefix[i] += seg_prefix[i - 1];
  __syncthreads();
  const float total = seg_prefix[nt];

  if (probs_out) {
    float* po = probs_out + (size_t)r * V;
    for (int i = tid; i < V; i += nt) {
      const float x = row[i] * inv_t;
      po[i] = (ordered(x) >= cut) ? expf(x - mx) / total : 0.f;
    }
  }

  const float target = uniform01(seeds[r], counters[r]) * total;
  // the segment that holds the target; the last non-empty segment catches rounding
  if (seg_prefix[tid] <= target && (target < seg_prefix[tid + 1] || tid == nt - 1) && b < V) {
    float run = seg_prefix[tid];
    int pick = -1, last_kept = -1;
    for (int i = b; i < e; ++i) {
      const float x = row[i] * inv_t;
      if (ordered(x) >= cut) {
        last_kept = i;
        run += expf(x - mx);
        if (run > target) {
          pick = i;
          break;
        }
      }
    }
    if (pick < 0) pick = last_kept;
    if (pick >= 0) out[r] = pick;
  }
}

// `out` must already hold each row's argmax (tk_argmax): greedy rows keep it, and so
// does a row whose segment search falls through (rounding at a segment edge).
TK_API int tk_sample(const float* logits, long ld, int M, int V, const float* temperature,
                     const int* top_k, const float* top_p, const unsigned long long* seeds,
                     const unsigned long long* counters, int* out, float* probs_out,
                     hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0) return -1;
  sample_kernel<<<M, 1024, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, seeds, counters,
                                        out, probs_out);
  return launch_status();
}
