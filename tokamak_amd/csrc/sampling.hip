// Token selection from float32 logits [M, V]: greedy argmax, and temperature /
// top-k / top-p sampling with a per-request counter-based random number.
//
// Filter order and rules follow the reference sampler
// (src/tokamak/sampling/sampler.py:34-39,64-84): divide by temperature; top-k
// keeps every logit >= the k-th largest (ties at the threshold survive); top-p
// sorts descending and drops a token iff the mass ranked before it already
// reaches top_p (the best token always survives); softmax over what is left;
// one draw.  No sort is done here: both thresholds are found by radix selection
// over the ordered-integer image of the float values, three passes over the row
// each (the row sits in L2).
#include "common.h"
#include "no_alloc.h"

#include <mutex>

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

// temperature, top_k, top_p, part_mass (all or none): for a row with temperature > 0 and no
// threshold the block also leaves the sum of e^((x - its segment's maximum) / temperature) over its segment, from which
// the sampler has the mass of every segment without a pass of its own over the row.
__global__ __launch_bounds__(kArgmaxThreads) void argmax_segments_kernel(
    const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i, int V,
    long ld, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, float* __restrict__ part_mass) {
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
  for (int w = 0; w < kArgmaxThreads / kWave; ++w) argmax_take(bv, bi, best_v[w], best_i[w]);  // every thread: the segment's
  if (threadIdx.x == 0) {
    part_v[r * kArgmaxSegments + seg] = bv;
    part_i[r * kArgmaxSegments + seg] = bi;
  }
  if (part_mass == nullptr || !(temperature[r] > 0.f)) return;
  if ((top_k[r] > 0 && top_k[r] < V) || top_p[r] < 1.f) return;  // a row with a threshold: the sampler sums what it keeps
  // the segment again (it is in the cache): its mass relative to its own maximum
  const float scale = 1.4426950408889634f / temperature[r];  // e^(y / t) = 2^(y log2 e / t)
  float mass = 0.f;
  const auto add = [&](float x) {
    const float y = (x - bv) * scale;
    if (y == y) mass += __builtin_amdgcn_exp2f(y);  // a NaN (also -inf - -inf of a segment without a number) adds nothing
  };
  if (vec) {
    for (int i = begin + threadIdx.x * 4; i < end; i += kArgmaxThreads * 4) {
      if (i + 4 <= end) {
        const float4 v = *reinterpret_cast<const float4*>(row + i);
        add(v.x);
        add(v.y);
        add(v.z);
        add(v.w);
      } else {
        for (int j = i; j < end; ++j) add(row[j]);
      }
    }
  } else {
    for (int i = begin + threadIdx.x; i < end; i += kArgmaxThreads) add(row[i]);
  }
  mass = wave_sum(mass);
  __syncthreads();  // best_v has been read
  if (lane == 0) best_v[wave] = mass;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int w = 0; w < kArgmaxThreads / kWave; ++w) total += best_v[w];
    part_mass[r * kArgmaxSegments + seg] = total;
  }
}

__global__ __launch_bounds__(kWave) void argmax_pick_kernel(const float* __restrict__ part_v,
                                                            const int* __restrict__ part_i,
                                                            int* __restrict__ out,
                                                            float* __restrict__ out_value) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float bv = lane < kArgmaxSegments ? part_v[r * kArgmaxSegments + lane] : -INFINITY;
  int bi = lane < kArgmaxSegments ? part_i[r * kArgmaxSegments + lane] : 0x7fffffff;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(bv, m, kWave);
    const int oi = __shfl_xor(bi, m, kWave);
    argmax_take(bv, bi, ov, oi);
  }
  if (lane == 0) {
    out[r] = (bi == 0x7fffffff) ? 0 : bi;
    if (out_value != nullptr) out_value[r] = bv;
  }
}

// part_v, part_i: scratch of M * tk_argmax_segments() floats and ints.  out_value
// (optional, [M]) receives each row's maximum (-inf if the row holds no number).
TK_API int tk_argmax_segments() { return kArgmaxSegments; }

TK_API int tk_argmax(const float* logits, int* out, float* out_value, float* part_v, int* part_i, int M,
                     int V, long ld, hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0 || M > 65535) return -1;
  argmax_segments_kernel<<<dim3(kArgmaxSegments, M), kArgmaxThreads, 0, stream>>>(logits, part_v, part_i, V, ld,
                                                                                   nullptr, nullptr, nullptr, nullptr);
  argmax_pick_kernel<<<M, kWave, 0, stream>>>(part_v, part_i, out, out_value);
  return launch_status();
}

// The same, and for the rows with temperature[m] > 0 and no threshold the mass of every segment
// relative to its maximum at that temperature (part_mass: M * tk_argmax_segments() floats), for tk_sample.
TK_API int tk_argmax_masses(const float* logits, int* out, float* out_value, float* part_v, int* part_i,
                            const float* temperature, const int* top_k, const float* top_p, float* part_mass,
                            int M, int V, long ld, hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0 || M > 65535 || !temperature || !top_k || !top_p || !part_mass) return -1;
  argmax_segments_kernel<<<dim3(kArgmaxSegments, M), kArgmaxThreads, 0, stream>>>(
      logits, part_v, part_i, V, ld, temperature, top_k, top_p, part_mass);
  argmax_pick_kernel<<<M, kWave, 0, stream>>>(part_v, part_i, out, out_value);
  return launch_status();
}

// The same two kernels with their scratch in a fixed device array (see no_alloc.h).
// `g_argmax_scratch` names the array for the device compiler; in host code the name is
// only a handle, so the address each GPU gave its copy is looked up once per device
// and the kernels get that pointer.
constexpr int kNoAllocRows = TK_ARGMAX_NO_ALLOC_MAX_ROWS;
constexpr int kMaxDevices = 64;
struct ArgmaxScratch {
  float value[kNoAllocRows * kArgmaxSegments];
  int index[kNoAllocRows * kArgmaxSegments];
};
static __device__ __align__(256) ArgmaxScratch g_argmax_scratch;
static ArgmaxScratch* g_argmax_scratch_ptr[kMaxDevices] = {};
static std::mutex g_argmax_scratch_mutex;

static ArgmaxScratch* argmax_scratch_of_current_device() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> guard(g_argmax_scratch_mutex);
  if (g_argmax_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_argmax_scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_argmax_scratch_ptr[device] = static_cast<ArgmaxScratch*>(ptr);
  }
  return g_argmax_scratch_ptr[device];
}

TK_API int tk_argmax_no_alloc_max_rows() { return kNoAllocRows; }

TK_API int tk_argmax_no_alloc(const float* logits, int* out, float* out_value, int M, int V, long ld,
                              hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0 || logits == nullptr || out == nullptr || ld < V) return -1;
  if (M > kNoAllocRows) return -3;
  ArgmaxScratch* scratch = argmax_scratch_of_current_device();
  if (scratch == nullptr) return -4;
  argmax_segments_kernel<<<dim3(kArgmaxSegments, M), kArgmaxThreads, 0, stream>>>(
      logits, scratch->value, scratch->index, V, ld, nullptr, nullptr, nullptr, nullptr);
  argmax_pick_kernel<<<M, kWave, 0, stream>>>(scratch->value, scratch->index, out, out_value);
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

constexpr int kSampleThreads = 1024;
constexpr int kBins = 4096;  // histogram bins of one radix pass (12 bits)

// Prefix sums of one value per thread over the block, threads in index order; `scan`
// holds kSampleThreads entries.  Returns the sum over the threads before this one;
// `inclusive` is that plus the thread's own value as the scan computed it (so the
// ranges [exclusive, inclusive) of the threads tile [0, total) exactly, also in
// floating point); `total` is the sum over all threads.
template <typename T>
__device__ __forceinline__ T block_scan(T v, T* scan, T& inclusive, T& total) {
  const int tid = threadIdx.x;
  __syncthreads();
  scan[tid] = v;
  __syncthreads();
  for (int step = 1; step < kSampleThreads; step <<= 1) {
    const T add = tid >= step ? scan[tid - step] : T(0);
    __syncthreads();
    scan[tid] += add;
    __syncthreads();
  }
  total = scan[kSampleThreads - 1];
  inclusive = scan[tid];
  return tid > 0 ? scan[tid - 1] : T(0);
}

// Walking the bins from the highest down: the bin in which the running sum first
// reaches `target` (sum of higher bins < target <= that sum + the bin), and the sum
// of the higher bins.  Every thread gets the result.  `nbins` is 4096 or 256.
template <typename T>
__device__ __forceinline__ void crossing_bin(const T* hist, int nbins, T target, T* scan, int* found_bin,
                                             T* found_above, int& bin, T& above) {
  const int tid = threadIdx.x;
  const int per = nbins / kSampleThreads > 0 ? nbins / kSampleThreads : 1;
  // thread t owns bins [top - per*t, top - per*t - per + 1], highest first
  T mine = 0;
  const int first = nbins - 1 - tid * per;
  if (first >= 0)
    for (int j = 0; j < per; ++j) mine += hist[first - j];
  T total, upto;
  const T before = block_scan<T>(mine, scan, upto, total);
  if (tid == 0) {  // target beyond everything (rounding): the lowest bin
    *found_bin = 0;
    *found_above = total - hist[0];
  }
  __syncthreads();
  if (first >= 0 && before < target && target <= upto) {
    T run = before;
    for (int j = 0; j < per; ++j) {
      const T h = hist[first - j];
      if (run + h >= target) {
        *found_bin = first - j;
        *found_above = run;
        break;
      }
      run += h;
    }
  }
  __syncthreads();
  bin = *found_bin;
  above = *found_above;
  __syncthreads();
}

// logit / temperature; a NaN is treated as -inf (never kept, never drawn), as the argmax does
__device__ __forceinline__ float scaled(float logit, float inv_t) {
  const float x = logit * inv_t;
  return x == x ? x : -INFINITY;
}

// e^x on the exponential unit (2^(x log2 e)): within some 1e-6 of expf for the exponents that
// count here (0 down to -100), at a tenth of its instructions; a block walks its row alone,
// and 152 k expf a pass were most of a pass's time
__device__ __forceinline__ float exp_unit(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// exp(x - max) as a 32.32 fixed-point number: integer sums do not depend on the
// order of addition, so thresholds found from them are the same on every run
__device__ __forceinline__ unsigned long long fixed_mass(float x, float mx) {
  return (unsigned long long)(exp_unit(x - mx) * 4294967296.f);
}

// f(index, value) for every element of a row, each by one thread of the block.  A block reads
// its row alone, so what counts is the bytes it has in flight: 16-byte loads where the row's
// address allows them (a pass over 152 k logits: 14 us instead of 29 and more).
template <typename F>
__device__ __forceinline__ void for_row(const float* __restrict__ row, int V, F f) {
  const int tid = threadIdx.x;
  const int head = min(V, (int)((16 - (reinterpret_cast<uintptr_t>(row) & 15)) & 15) / 4);  // before the first 16-byte boundary
  if (tid < head) f(tid, row[tid]);
  const float4* row4 = reinterpret_cast<const float4*>(row + head);
  const int n4 = (V - head) / 4;
#pragma unroll 8
  for (int i = tid; i < n4; i += kSampleThreads) {
    const float4 v = row4[i];
    const int at = head + 4 * i;
    f(at, v.x);
    f(at + 1, v.y);
    f(at + 2, v.z);
    f(at + 3, v.w);
  }
  const int done = head + 4 * n4;
  if (tid < V - done) f(done + tid, row[done + tid]);
}

// One block per row.  params rows: temperature, top_k, top_p (floats);
// seeds/counters: the request's seed and how many draws it has made.
// probs_out (optional, [M, V]) receives the final distribution, for tests.
//
// Both thresholds are found by radix selection over the ordered-integer image of the
// scaled logits: three levels (12, 12 and 8 bits), each filling a histogram in LDS (counts
// for top-k, fixed-point probability mass for top-p) in which the bin that holds the
// threshold is found; the next level looks only at the values of that bin.  A pass over the
// row costs 14 us (one CU reads it alone), so the row is walked as rarely as possible: the
// first pass fills the first level's histogram and tells in which of its bins the threshold
// lies; if the values of that bin and the bins above it are few (up to kCandidates; they
// are, unless the logits are nearly all alike), a second pass copies them into LDS, and every
// further level of both searches reads those.  The third pass is the draw's.  (Without the
// copies: seven passes with both thresholds.)
constexpr int kCandidates = 16384;

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const unsigned long long* __restrict__ seeds, const unsigned long long* __restrict__ counters,
    const float* __restrict__ row_max, const float* __restrict__ seg_max, const float* __restrict__ seg_mass,
    int* __restrict__ out, float* __restrict__ probs_out) {
  __shared__ float fs[kArgmaxSegments];  // the masses of the row's chunks (16 of the waves, or the 32 segments of the argmax pass)
  __shared__ unsigned long long hist64[kBins];
  __shared__ uint32_t hist32[kBins];
  __shared__ unsigned long long scan64[kSampleThreads];
  __shared__ uint32_t cand[kCandidates];  // ordered images of the values that may hold a threshold
  __shared__ uint32_t cand_count;
  __shared__ int found_bin;
  __shared__ int last_token;
  __shared__ unsigned long long found_above;
  uint32_t* scan32 = reinterpret_cast<uint32_t*>(scan64);
  float* scanf_ = reinterpret_cast<float*>(scan64);

  const int r = blockIdx.x, tid = threadIdx.x, nt = kSampleThreads;
  if (!(temperature[r] > 0.f)) return;  // greedy row: the argmax pre-pass has written it
  const float* row = logits + (size_t)r * ld;
  const float inv_t = 1.f / temperature[r];
  const int k = top_k[r];
  const float p_keep = top_p[r];
  const bool k_on = k > 0 && k < V, p_on = p_keep < 1.f;

  // the row's maximum comes from the argmax pass that ran before (temperature > 0
  // keeps the order); a row without any number has nothing to draw from
  const float mx = row_max[r] * inv_t;
  if (!(mx > -INFINITY)) return;

  // First pass: the first level's histogram (counts; probability mass too if only top-p is
  // asked for), the bin of the first threshold to be found, and the candidates.
  uint32_t k_prefix = 0, k_remaining = (uint32_t)max(k, 0);
  uint32_t p_prefix = 0;               // only top-p: its first level is found by the first pass
  unsigned long long p_remaining = 0;
  int ncand = -1;                      // >= 0: cand[0 .. ncand) hold every value that can be a threshold
  if (k_on || p_on) {
    for (int i = tid; i < kBins; i += nt) {
      hist32[i] = 0;
      hist64[i] = 0;
    }
    if (tid == 0) cand_count = 0;
    __syncthreads();
    for_row(row, V, [&](int, float logit) {
      const float x = scaled(logit, inv_t);
      const uint32_t bin = ordered(x) >> 20;
      atomicAdd(&hist32[bin], 1u);
      if (!k_on) atomicAdd(&hist64[bin], fixed_mass(x, mx));
    });
    __syncthreads();
    int low_bin;
    if (k_on) {
      uint32_t above;
      crossing_bin<uint32_t>(hist32, kBins, k_remaining, scan32, &found_bin,
                             reinterpret_cast<uint32_t*>(&found_above), low_bin, above);
      k_remaining -= above;
      k_prefix = (uint32_t)low_bin;
    } else {
      // the whole mass, then the share of it that top_p allows (at least one unit)
      unsigned long long mine = 0, upto, whole, above;
      for (int i = tid; i < kBins; i += nt) mine += hist64[i];
      block_scan<unsigned long long>(mine, scan64, upto, whole);
      const double share = (double)p_keep * (double)whole;
      p_remaining = share < 1.0 ? 1ull : (unsigned long long)share;
      crossing_bin<unsigned long long>(hist64, kBins, p_remaining, scan64, &found_bin, &found_above, low_bin, above);
      p_remaining -= above;
      p_prefix = (uint32_t)low_bin;
    }
    // the values in that bin and above it
    uint32_t mine = 0, upto, total;
    for (int i = tid; i < kBins; i += nt) mine += i >= low_bin ? hist32[i] : 0u;
    block_scan<uint32_t>(mine, scan32, upto, total);
    if (total <= (uint32_t)kCandidates) {
      for_row(row, V, [&](int, float logit) {
        const uint32_t o = ordered(scaled(logit, inv_t));
        if ((int)(o >> 20) >= low_bin) cand[atomicAdd(&cand_count, 1u)] = o;  // (in any order: the sums below are of integers)
      });
      ncand = (int)total;
    }
    __syncthreads();
  }
  // f(ordered image, scaled logit) for every value that may still hold a threshold
  const auto each = [&](auto f) {
    if (ncand >= 0) {
      for (int i = tid; i < ncand; i += nt) f(cand[i], unordered(cand[i]));
    } else {
      for_row(row, V, [&](int, float logit) {
        const float x = scaled(logit, inv_t);
        f(ordered(x), x);
      });
    }
  };

  // top-k: kth = the k-th largest scaled logit (everything >= it survives)
  uint32_t kth = 0;  // ordered(-inf) is > 0, so 0 keeps everything
  if (k_on) {
    uint32_t prefix = k_prefix, remaining = k_remaining;
    // (shift, bits): 20/12 (done above), 8/12, 0/8
    for (int level = 1; level < 3; ++level) {
      const int shift = level == 1 ? 8 : 0;
      const int nbins = level == 2 ? 256 : kBins;
      for (int i = tid; i < kBins; i += nt) hist32[i] = 0;
      __syncthreads();
      each([&](uint32_t o, float) {
        if ((o >> (shift + (level == 1 ? 12 : 8))) == prefix) atomicAdd(&hist32[(o >> shift) & (uint32_t)(nbins - 1)], 1u);
      });
      __syncthreads();
      int bin;
      uint32_t above;
      crossing_bin<uint32_t>(hist32, nbins, remaining, scan32, &found_bin,
                             reinterpret_cast<uint32_t*>(&found_above), bin, above);
      remaining -= above;
      prefix = (prefix << (level == 2 ? 8 : 12)) | (uint32_t)bin;
    }
    kth = prefix;
  }

  // top-p: keep x iff the mass of kept values strictly greater than x is < top_p of
  // the whole; the kept set is {x >= cut}
  uint32_t cut = kth;
  if (p_on) {
    uint32_t prefix = p_prefix;
    unsigned long long remaining = p_remaining;
    for (int level = k_on ? 0 : 1; level < 3; ++level) {  // (without top-k the first pass was the first level)
      const int shift = level == 0 ? 20 : level == 1 ? 8 : 0;
      const int nbins = level == 2 ? 256 : kBins;
      for (int i = tid; i < kBins; i += nt) hist64[i] = 0;
      __syncthreads();
      each([&](uint32_t o, float x) {
        const bool in_bin = level == 0 || (o >> (shift + (level == 1 ? 12 : 8))) == prefix;
        if (in_bin && o >= kth) atomicAdd(&hist64[(o >> shift) & (uint32_t)(nbins - 1)], fixed_mass(x, mx));
      });
      __syncthreads();
      if (level == 0) {
        // the whole mass of what top-k keeps (the candidates hold all of it)
        unsigned long long mine = 0, upto, whole;
        for (int i = tid; i < kBins; i += nt) mine += hist64[i];
        block_scan<unsigned long long>(mine, scan64, upto, whole);
        const double share = (double)p_keep * (double)whole;
        remaining = share < 1.0 ? 1ull : (unsigned long long)share;
      }
      int bin;
      unsigned long long above;
      crossing_bin<unsigned long long>(hist64, nbins, remaining, scan64, &found_bin, &found_above, bin, above);
      remaining -= above;
      prefix = (prefix << (level == 2 ? 8 : 12)) | (uint32_t)bin;
    }
    cut = prefix > kth ? prefix : kth;
  }

  // final distribution over {x >= cut}.  The draw walks the tokens in index order: each
  // wave sums a contiguous chunk of the row; the chunk that holds the target is then
  // walked again by the whole block.
  // Without a threshold the chunks are the segments of the argmax pass, which has left their
  // masses (relative to each segment's own maximum): no pass over the row here.
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  constexpr int kWaves = kSampleThreads / kWave;
  static_assert(kWaves <= kArgmaxSegments, "fs holds either kind of chunk");
  const bool by_segments = cut == 0 && seg_mass != nullptr;
  const int nchunks = by_segments ? kArgmaxSegments : kWaves;
  const int chunk = by_segments ? (((V + kArgmaxSegments - 1) / kArgmaxSegments + 3) & ~3)
                                : ((V + kWaves - 1) / kWaves + 4 * kWave - 1) / (4 * kWave) * (4 * kWave);
  const int c_begin = wave * chunk, c_end = min(V, c_begin + chunk);
  float mine = 0.f;
  const auto kept_mass = [&](float logit) {
    const float x = scaled(logit, inv_t);
    return ordered(x) >= cut ? exp_unit(x - mx) : 0.f;
  };
  const int c_len = max(0, c_end - c_begin);
  if (by_segments) {
    __syncthreads();
    if (tid < kArgmaxSegments) {
      const float m = seg_max[r * kArgmaxSegments + tid];
      fs[tid] = m > -INFINITY ? seg_mass[r * kArgmaxSegments + tid] * exp_unit(m * inv_t - mx) : 0.f;
    }
    __syncthreads();
  } else if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {  // (chunks begin at multiples of 256 tokens)
    const int quads = c_len / 4;
#pragma unroll 8
    for (int q = lane; q < quads; q += kWave) {
      const float4 v = *reinterpret_cast<const float4*>(row + c_begin + 4 * q);
      mine += (kept_mass(v.x) + kept_mass(v.y)) + (kept_mass(v.z) + kept_mass(v.w));
    }
    if (lane < c_len - 4 * quads) mine += kept_mass(row[c_begin + 4 * quads + lane]);
  } else {
#pragma unroll 8
    for (int i = lane; i < c_len; i += kWave) mine += kept_mass(row[c_begin + i]);
  }
  if (!by_segments) {
    mine = wave_sum(mine);
    __syncthreads();
    if (lane == 0) fs[wave] = mine;
    __syncthreads();
  }
  float total = 0.f;
  for (int w = 0; w < nchunks; ++w) total += fs[w];

  if (probs_out) {
    float* po = probs_out + (size_t)r * V;
    for_row(row, V, [&](int i, float logit) {
      const float x = scaled(logit, inv_t);
      po[i] = (ordered(x) >= cut) ? exp_unit(x - mx) / total : 0.f;
    });
  }

  const float target = uniform01(seeds[r], counters[r]) * total;
  // The chunk that holds the target (every thread finds the same one; the last chunk of
  // the row catches rounding), then all threads walk that chunk: each sums a contiguous
  // run of it, a prefix sum over the block finds the run, and its thread walks it.
  int sel = (V - 1) / chunk;
  float sel_before = 0.f;
  {
    float run = 0.f;
    bool found = false;
    for (int w = 0; w < nchunks; ++w) {
      const float next = run + fs[w];
      if (!found && (target < next || w == sel)) {
        found = true;
        sel = w;
        sel_before = run;
      }
      run = next;
    }
  }
  const int s_begin = sel * chunk, s_end = min(V, s_begin + chunk);
  const int run_len = ((s_end - s_begin + kSampleThreads - 1) / kSampleThreads + 3) / 4 * 4;
  const int r_begin = min(s_end, s_begin + tid * run_len), r_end = min(s_end, r_begin + run_len);
  float mine_run = 0.f;
  int last_kept = -1;
#pragma unroll 4
  for (int i = r_begin; i < r_end; ++i) {
    const float m = kept_mass(row[i]);
    // (a kept token's mass may round to zero; it is kept all the same)
    if (ordered(scaled(row[i], inv_t)) >= cut) last_kept = i;
    mine_run += m;
  }
  if (tid == 0) {
    found_bin = -1;   // the token that the target falls on
    last_token = -1;  // the chunk's last kept token
  }
  float incl, chunk_total;
  const float excl = block_scan<float>(mine_run, scanf_, incl, chunk_total);  // (its barriers order the two writes above)
  if (last_kept >= 0) atomicMax(&last_token, last_kept);
  if (sel_before + excl <= target && target < sel_before + incl) {
    float run = sel_before + excl;
    int pick = -1;
#pragma unroll 4
    for (int i = r_begin; i < r_end; ++i) {  // (to the run's end, so that its loads can be asked for together)
      const float logit = row[i];
      if (ordered(scaled(logit, inv_t)) >= cut) {
        run += kept_mass(logit);
        if (pick < 0 && run > target) pick = i;
      }
    }
    if (pick < 0) pick = last_kept;  // rounding at the end of the run
    if (pick >= 0) atomicMax(&found_bin, pick);
  }
  __syncthreads();
  // no thread's run held the target (rounding at the chunk's end): the chunk's last kept token
  if (tid == 0) {
    const int chosen = found_bin >= 0 ? found_bin : last_token;
    if (chosen >= 0) out[r] = chosen;
  }
}

// `out` must already hold each row's argmax and `row_max` its maximum (tk_argmax): greedy
// rows keep the argmax, and so does a row whose search falls through (rounding at an edge).
// seg_max, seg_mass (both or neither): what tk_argmax_masses left, [M][tk_argmax_segments()].
TK_API int tk_sample(const float* logits, long ld, int M, int V, const float* temperature,
                     const int* top_k, const float* top_p, const unsigned long long* seeds,
                     const unsigned long long* counters, const float* row_max, const float* seg_max,
                     const float* seg_mass, int* out, float* probs_out, hipStream_t stream) {
  if (M <= 0) return 0;
  if (V <= 0) return -1;
  if (row_max == nullptr || (seg_max == nullptr) != (seg_mass == nullptr)) return -1;
  sample_kernel<<<M, kSampleThreads, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, seeds, counters,
                                                  row_max, seg_max, seg_mass, out, probs_out);
  return launch_status();
}
