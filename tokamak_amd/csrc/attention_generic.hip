// Paged causal attention for any head size (multiple of 16, up to 512), any
// number of heads and groups, any page size that is a multiple of 8, in float32
// or bf16 storage with float32 arithmetic throughout.  It serves prompt portions
// and decode tokens alike: every query token walks its own request's block table
// from the first visible position to its own position.
//
// One block of kWaves waves per (token, query head).  Keys are taken 64 at a time, one
// key per lane; round i of a token's keys goes to wave i % kWaves, which keeps a running
// maximum, a running sum and an output of its own in float32 (online softmax); at the end
// the waves' results are merged in wave order.  Which wave takes which keys follows from
// the token's own position alone, so the result does not depend on how the request was
// cut into steps or what else is in the batch.
//
// Cache pages: K [nkv][hd/8][ps][8], V [nkv][hd/16][ps/4][16][4] (see elementwise.hip).
#include "common.h"

using namespace tk;

constexpr int kMaxHd = 512;
constexpr int kAccPerLane = kMaxHd / kWave;
constexpr int kWaves = 8;  // waves of a block; kWaves * 64 threads cover every dimension of the widest head
static_assert(kWaves * kWave >= kMaxHd, "the merge gives every dimension a thread");

template <typename T>
__global__ __launch_bounds__(kWaves * kWave) void paged_attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, T* __restrict__ out, int nh, int nkv, int hd, int ps,
    int max_pages, float scale, int window) {
  __shared__ float q_s[kMaxHd];
  __shared__ float p_s[kWaves][kWave];
  __shared__ long base_s[kWaves][kWave];
  __shared__ float m_s[kWaves], l_s[kWaves];
  __shared__ float acc_s[kWaves][kMaxHd];

  const int n = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  const int kvh = head / (nh / nkv);
  const int pos = positions[n];
  const int* table = block_tables + (size_t)req_of_token[n] * max_pages;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const size_t page_elems = (size_t)nkv * hd * ps;
  const size_t head_off = (size_t)kvh * hd * ps;

  const T* qrow = q + ((size_t)n * nh + head) * hd;
  for (int d = tid; d < hd; d += kWaves * kWave) q_s[d] = Elem<T>::load(qrow + d) * scale;
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kAccPerLane];
#pragma unroll
  for (int i = 0; i < kAccPerLane; ++i) acc[i] = 0.f;

  // this wave's rounds of 64 keys; every round starts at or before the token's own position
  // and, but for the first, at or after the first visible one: none is empty
  for (int c0 = (first / kWave + wave) * kWave; c0 <= pos; c0 += kWaves * kWave) {
    const int c = c0 + lane;
    const bool valid = c >= first && c <= pos;
    float s = -INFINITY;
    long vbase = -1;
    if (valid) {
      const int page = table[c / ps];
      const int off = c % ps;
      const T* kp = k_cache + (size_t)page * page_elems + head_off;
      float dot = 0.f;
      for (int j = 0; j < hd / 8; ++j) {
        const T* kk = kp + ((size_t)j * ps + off) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) dot = fmaf(q_s[j * 8 + e], Elem<T>::load(kk + e), dot);
      }
      s = dot;
      vbase = (long)((size_t)page * page_elems + head_off + (size_t)(off >> 2) * 64 + (off & 3));
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // m = -inf on the first round: alpha = 0
    l = l * alpha + wave_sum(p);
    m = m_new;
    wave_lds_sync();   // the wave has read its last round's probabilities
    p_s[wave][lane] = p;
    base_s[wave][lane] = vbase;
    wave_lds_sync();
    const int count = (pos - c0 + 1 < kWave) ? pos - c0 + 1 : kWave;
#pragma unroll
    for (int i = 0; i < kAccPerLane; ++i) {
      const int d = lane + i * kWave;
      if (d < hd) {
        const size_t v_dim_off = (size_t)(d >> 4) * (ps >> 2) * 64 + (d & 15) * 4;
        float a = acc[i] * alpha;
        for (int t = 0; t < count; ++t) {
          const long b = base_s[wave][t];
          if (b >= 0) a = fmaf(p_s[wave][t], Elem<T>::load(v_cache + b + v_dim_off), a);
        }
        acc[i] = a;
      }
    }
  }
  // merge: a wave that had no round brings m = -inf, l = 0 and zeros, which weigh nothing
  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
#pragma unroll
  for (int i = 0; i < kAccPerLane; ++i) {
    const int d = lane + i * kWave;
    if (d < hd) acc_s[wave][d] = acc[i];
  }
  __syncthreads();
  if (tid >= hd) return;
  float top = m_s[0];   // wave 0 always has the first round
#pragma unroll
  for (int w = 1; w < kWaves; ++w) top = fmaxf(top, m_s[w]);
  float sum = 0.f, o = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const float e = expf(m_s[w] - top);
    sum = fmaf(l_s[w], e, sum);
    o = fmaf(acc_s[w][tid], e, o);
  }
  Elem<T>::store(out + ((size_t)n * nh + head) * hd + tid, o / sum);
}

TK_API int tk_paged_attention_generic(int dtype, const void* q, const void* k_cache,
                                      const void* v_cache, const int* block_tables,
                                      const int* positions, const int* req_of_token, void* out,
                                      int N, int nh, int nkv, int hd, int ps, int max_pages,
                                      float scale, int window, hipStream_t stream) {
  if (N <= 0) return 0;
  if (hd > kMaxHd || hd % 16 != 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || ps % 4 != 0 || nh > 65535) return -1;
  dim3 grid(N, nh);
  if (dtype == 0)
    paged_attention_generic_kernel<float><<<grid, kWaves * kWave, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, block_tables, positions,
        req_of_token, (float*)out, nh, nkv, hd, ps, max_pages, scale, window);
  else
    paged_attention_generic_kernel<bf16_t><<<grid, kWaves * kWave, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, positions,
        req_of_token, (bf16_t*)out, nh, nkv, hd, ps, max_pages, scale, window);
  return launch_status();
}
