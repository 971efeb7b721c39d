// Paged causal attention on the matrix cores (bf16 in, float32 softmax and
// accumulation) for head sizes 64 and 128 and page sizes 16, 32, 64, ... (powers of two).
//
// Decode tokens (attention_decode_kernel): a block of sixteen waves owns one token, one kv
// head and a range of that request's keys (a split); the waves take contiguous shares
// of the range and merge through LDS.  A wave's 16 "columns" are the query heads of the
// group.  Keys are taken 16 at a time (one MFMA tile, never across a page edge); a tile's
// keys are reloaded for the wave's next tile as soon as the scores are taken, its values
// as soon as they are multiplied:
//   S^T[key][col] = K[key][:] . Q[col][:]      v_mfma_f32_16x16x32_bf16, K rows as A
//   P^T = exp2(S^T * c - m[col])               float32, one column per lane
//   O^T[d][col] += V^T[d][key] * P^T[key][col] v_mfma_f32_16x16x16_bf16, V^T rows as A
// The result layout of the first product is exactly the B operand layout of the
// second, so probabilities never leave registers, and both K and V^T operands
// are loaded straight from the pages (K page [nkv][hd/8][ps][8], V page
// [nkv][hd/16][ps/4][16][4]) in contiguous 16- and 8-byte pieces.
//
// With more than one split the block writes an unnormalised partial (o, m, l) and
// a second kernel merges the splits of each (token, head).
#include "common.h"
#include "slots.h"

using namespace tk;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

union Frag8 {
  uint4 u;
  u32x4 w;
  bf16x8 v;
};
union Frag4 {
  uint2 u;
  u32x2 w;
  short4v v;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int kDecodeWaves = 16;

// The keys of one split of a decode token whose keys are cut in nsplit: the token's own keys
// cut evenly (a whole number of 16 keys for every wave of a block), whatever the longest
// request of the step holds, so that the blocks of a token walk equal shares; splits past the
// token's last key hold nothing.
__device__ __forceinline__ int decode_share(int keys, int nsplit) {
  constexpr int unit = 16 * kDecodeWaves;
  return ((keys + nsplit - 1) / nsplit + unit - 1) / unit * unit;
}

// What the fused form of the decode kernel takes instead of finished queries: the q/k/v
// projection's output as it left the product (`parts` float32 partial sums of a split-K
// product, part_stride elements apart, or one bfloat16 matrix), rows of (nh + 2 nkv_in)
// heads; the per-head norm weights (or null), the rotary tables [N, HD/2] (rot == HD) or
// none (rot == 0).  nkv_in == 0: the call only reads the cache (queries alone are made).
struct DecodeInputs {
  const void* qkv;
  int in_f32, parts;
  long part_stride;
  const float *q_weight, *k_weight, *cos_t, *sin_t;
  int rot, nkv_in;
  float eps;
};

// One head's vector from the projection's output: partial sums added, per-head RMSNorm,
// half-split rotation; lane l ends up with dims 2l and 2l + 1 (HD / 2 lanes take part).
// What the separate kernel of elementwise.hip computes, for one token and head.
template <int HD>
__device__ __forceinline__ void decode_head_vector(const DecodeInputs& in, size_t row_offset, int head_col,
                                                   const float* weight, bool rotate, int token, int lane,
                                                   float& x0, float& x1) {
  const bool active = lane < HD / 2;
  const int d = 2 * (active ? lane : 0);
  x0 = x1 = 0.f;
  if (in.in_f32) {
    const float* src = static_cast<const float*>(in.qkv) + row_offset + (size_t)head_col * HD + d;
    // four partial sums in flight at a time (a chain of dependent loads would cost a memory
    // round trip each); added in split order
    for (int p = 0; p < in.parts; p += 4) {
      float2 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        v[u] = p + u < in.parts ? *reinterpret_cast<const float2*>(src + (size_t)(p + u) * in.part_stride)
                                : make_float2(0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        x0 += v[u].x;
        x1 += v[u].y;
      }
    }
  } else {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(static_cast<const bf16_t*>(in.qkv) + row_offset +
                                                          (size_t)head_col * HD + d);
    x0 = __uint_as_float(v << 16);
    x1 = __uint_as_float(v & 0xffff0000u);
  }
  if (!active) x0 = x1 = 0.f;
  if (weight != nullptr) {
    const float ss = wave_sum(x0 * x0 + x1 * x1);
    const float rstd = rsqrtf(ss / (float)HD + in.eps);
    x0 = x0 * rstd * weight[d];
    x1 = x1 * rstd * weight[d + 1];
  }
  if (rotate) {
    // out[j] = x[j] cos_j - x[j + HD/2] sin_j ; out[j + HD/2] = x[j + HD/2] cos_j + x[j] sin_j
    const float p0 = __shfl_xor(x0, HD / 4, kWave), p1 = __shfl_xor(x1, HD / 4, kWave);
    const int j = d % (HD / 2);
    const float2 c = *reinterpret_cast<const float2*>(in.cos_t + (size_t)token * (HD / 2) + j);
    const float2 sn = *reinterpret_cast<const float2*>(in.sin_t + (size_t)token * (HD / 2) + j);
    const float sign = (d < HD / 2) ? -1.f : 1.f;
    x0 = x0 * c.x + sign * p0 * sn.x;
    x1 = x1 * c.y + sign * p1 * sn.y;
  }
}

// WAVES: waves of a block (they share a split's keys and merge through LDS); D: tiles of
// 16 keys a wave keeps in flight.  FUSED: the block first makes its queries (and, if the
// call stores, the token's own key and value, which the block of the last split writes to
// the page and every wave that meets the token's position takes from LDS) from the
// projection's output: one kernel less a layer than with the separate q/k norm kernel.
template <int HD, int WAVES, int D, bool FUSED>
__global__ __launch_bounds__(WAVES * 64) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache_in,
    const bf16_t* __restrict__ v_cache_in, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ item_token, const int* __restrict__ item_count,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int nsplit,
    int split_keys, int nh, int nkv, int ps, float scale_log2, DecodeInputs in) {
  const bf16_t* __restrict__ k_cache = k_cache_in;
  const bf16_t* __restrict__ v_cache = v_cache_in;
  constexpr int KCH = HD / 32;  // 32-wide chunks of the head dim (QK^T steps)
  constexpr int DBL = HD / 16;  // 16-wide blocks of the head dim (PV outputs)
  // LDS: the waves' accumulators of the group's heads [WAVES][G][HD], then their (m, l) [WAVES][16] each
  extern __shared__ __attribute__((aligned(16))) float s_dyn[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, kb = lane >> 4;
  // splits are the slowest index of the grid: blocks start in the grid's order, so a token's
  // last split (the shortest, or one that holds no key) starts behind every first one
  const int split = blockIdx.z, item = blockIdx.y;
  const int G = nh / nkv;
  const int kvh = blockIdx.x;

  const int n0 = item_token[item];
  const int pos0 = positions[n0];  // the token's position: it sees keys 0 .. pos0
  static_assert(WAVES == kDecodeWaves, "decode_share cuts for blocks of kDecodeWaves waves");
  const int share = nsplit > 1 ? decode_share(pos0 + 1, nsplit) : split_keys;
  const int k_begin = split * share;
  const int k_end = min(pos0 + 1, k_begin + share);
  if (k_begin >= k_end) return;  // the whole block: this split holds no key of the token
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t page_elems = (size_t)nkv * HD * ps;
  const size_t head_off = (size_t)kvh * HD * ps;

  // the split's tiles of 16 keys, in contiguous shares of the waves
  const int tiles = (k_end - k_begin + 15) >> 4;
  const int per = (tiles + WAVES - 1) / WAVES;
  const int t_begin = wave * per, t_end = min(tiles, t_begin + per);

  // this lane's column is query head `col` of the group
  const int c_head = kvh * G + col;
  const bool c_valid = col < G;

  // The wave's first tiles are asked for before anything else: they depend on the block
  // table only, and the queries (which the fused form first has to make) are needed when
  // they arrive.
  Frag8 kreg[D][KCH];
  Frag4 vreg[D][DBL];
#define TK_TILE_ADDR(T_)                                                  \
    const int c0_ = k_begin + (T_) * 16;                                    \
    const int page_ = table[c0_ / ps];                                      \
    const int off_ = c0_ % ps;
#define TK_LOAD_K(SLOT_, T_)                                                                          \
  {                                                                                                   \
    TK_TILE_ADDR(T_)                                                                                  \
    const bf16_t* kp_ = k_cache + (size_t)page_ * page_elems + head_off + (size_t)(off_ + col) * 8;   \
    _Pragma("unroll") for (int c = 0; c < KCH; ++c) kreg[SLOT_][c].w = __builtin_nontemporal_load(    \
        reinterpret_cast<const u32x4*>(kp_ + (size_t)(c * 4 + kb) * ps * 8));                         \
  }
  // V page [hd/16][ps/4][16][4]: lane (dim col, quad kb) of block d reads 8 bytes, the wave 512
  // contiguous bytes
#define TK_LOAD_V(SLOT_, T_)                                                                          \
  {                                                                                                   \
    TK_TILE_ADDR(T_)                                                                                  \
    const bf16_t* vp_ =                                                                               \
        v_cache + (size_t)page_ * page_elems + head_off + (size_t)((off_ >> 2) + kb) * 64 + col * 4;  \
    _Pragma("unroll") for (int d = 0; d < DBL; ++d) vreg[SLOT_][d].w = __builtin_nontemporal_load(    \
        reinterpret_cast<const u32x2*>(vp_ + (size_t)d * (ps >> 2) * 64));                            \
  }

#pragma unroll
  for (int i = 0; i < D; ++i)
    if (t_begin + i < t_end) {
      TK_LOAD_K(i, t_begin + i)
      TK_LOAD_V(i, t_begin + i)
    }

  // Q as B operand: lane (col, kb) holds Q[col][c*32 + kb*8 .. +8]
  bf16x8 qreg[KCH];
  bool stores = false;    // FUSED: this call stores the token's key and value
  bf16_t* s_new = nullptr;  // FUSED: [G + 2][HD] in LDS: the group's queries, then the new key and value
  if constexpr (FUSED) {
    s_new = reinterpret_cast<bf16_t*>(s_dyn + (size_t)WAVES * G * HD + 2 * WAVES * 16);
    stores = in.nkv_in > 0;
    const int heads_in = nh + 2 * in.nkv_in;
    const size_t row_offset = (size_t)n0 * heads_in * HD;
    if (wave < G + (stores ? 2 : 0)) {
      float x0, x1;
      if (wave < G)
        decode_head_vector<HD>(in, row_offset, kvh * G + wave, in.q_weight, in.rot != 0, n0, lane, x0, x1);
      else if (wave == G)
        decode_head_vector<HD>(in, row_offset, nh + kvh, in.k_weight, in.rot != 0, n0, lane, x0, x1);
      else
        decode_head_vector<HD>(in, row_offset, nh + in.nkv_in + kvh, nullptr, false, n0, lane, x0, x1);
      if (lane < HD / 2)
        *reinterpret_cast<uint32_t*>(s_new + (size_t)wave * HD + 2 * lane) = pack_bf16x2(x0, x1);
    }
    __syncthreads();
    // the block that holds the token's position writes its key and value to the page
    if (stores && wave == 0 && lane < HD / 2 && k_begin <= pos0 && pos0 < k_begin + share) {
      const int page = table[pos0 / ps], off = pos0 % ps, d = 2 * lane;
      bf16_t* kp = const_cast<bf16_t*>(k_cache_in) + (size_t)page * page_elems + head_off;
      bf16_t* vp = const_cast<bf16_t*>(v_cache_in) + (size_t)page * page_elems + head_off;
      *reinterpret_cast<uint32_t*>(kp + ((size_t)(d >> 3) * ps + off) * 8 + (d & 7)) =
          *reinterpret_cast<const uint32_t*>(s_new + (size_t)G * HD + d);
      const bf16_t* vn = s_new + (size_t)(G + 1) * HD + d;
      vp[((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3)] = vn[0];
      vp[((size_t)((d + 1) >> 4) * (ps >> 2) + (off >> 2)) * 64 + ((d + 1) & 15) * 4 + (off & 3)] = vn[1];
    }
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      Frag8 f;
      f.u = c_valid ? *reinterpret_cast<const uint4*>(s_new + (size_t)col * HD + c * 32 + kb * 8) : make_uint4(0, 0, 0, 0);
      qreg[c] = f.v;
    }
  } else {
    const bf16_t* qp = q + ((size_t)n0 * nh + c_head) * HD + kb * 8;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      Frag8 f;
      f.u = c_valid ? *reinterpret_cast<const uint4*>(qp + c * 32) : make_uint4(0, 0, 0, 0);
      qreg[c] = f.v;
    }
  }

  float m_run = -INFINITY, l_run = 0.f;
  float4v acc[DBL];
#pragma unroll
  for (int d = 0; d < DBL; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  for (int t0 = t_begin; t0 < t_end; t0 += D) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      const int t = t0 + i;
      if (t >= t_end) break;  // the same for every lane of the wave
      const int c0 = k_begin + t * 16;
      const bool edge = c0 + 15 > pos0;  // some key of this tile lies past the token's position
      if constexpr (FUSED) {
        // the token's own key and value come from LDS (the page's slot is being written, or was not yet)
        if (stores && c0 <= pos0 && pos0 - c0 < 16) {
          if (col == pos0 - c0) {
#pragma unroll
            for (int c = 0; c < KCH; ++c)
              kreg[i][c].u = *reinterpret_cast<const uint4*>(s_new + (size_t)G * HD + c * 32 + kb * 8);
          }
          if (kb == ((pos0 - c0) >> 2)) {
#pragma unroll
            for (int d = 0; d < DBL; ++d) {
              short4v tv = vreg[i][d].v;
              tv[(pos0 - c0) & 3] = (short)s_new[(size_t)(G + 1) * HD + d * 16 + col];
              vreg[i][d].v = tv;
            }
          }
        }
      }
      float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KCH; ++c) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[i][c].v, qreg[c], sc, 0, 0, 0);
      // the slot's keys have been used: its next tile's keys fly while the others are multiplied
      if (t + D < t_end) TK_LOAD_K(i, t + D)
      float sv[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        sv[e] = sc[e] * scale_log2;
        if (edge && c0 + kb * 4 + e > pos0) sv[e] = -INFINITY;
      }
      float tmax = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m_run, tmax);  // finite: a tile's first key is never past the position
      const float alpha = fast_exp2(m_run - m_new);
      m_run = m_new;
      float pr[4];
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pr[e] = fast_exp2(sv[e] - m_new);
        psum += pr[e];
      }
      l_run = l_run * alpha + psum;
      Frag4 pb;
      pb.u = make_uint2(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]));
#pragma unroll
      for (int d = 0; d < DBL; ++d) {
        short4v tv = vreg[i][d].v;
        if (edge) {
          // keys past the request's end may hold anything (NaN included): zero their values
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (c0 + kb * 4 + e > pos0) tv[e] = 0;
        }
        float4v a = acc[d];
        a[0] *= alpha;
        a[1] *= alpha;
        a[2] *= alpha;
        a[3] *= alpha;
        acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tv, pb.v, a, 0, 0, 0);
      }
      if (t + D < t_end) TK_LOAD_V(i, t + D)
    }
  }
#undef TK_LOAD_V
#undef TK_LOAD_K
#undef TK_TILE_ADDR

  // The waves' shares meet in LDS: acc[d][e] = O^T[dim = d*16 + kb*4 + e][col], unnormalised,
  // relative to the wave's own maximum m_run (-inf and zeros for a wave without a tile).
  float* s_acc = s_dyn;                         // [WAVES][G][HD]
  float* s_m = s_dyn + (size_t)WAVES * G * HD;  // [WAVES][16]
  float* s_l = s_m + WAVES * 16;                // [WAVES][16]
  float l = l_run;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (c_valid) {
    float* mine = s_acc + ((size_t)wave * G + col) * HD + kb * 4;
#pragma unroll
    for (int d = 0; d < DBL; ++d)
      *reinterpret_cast<float4*>(mine + d * 16) = make_float4(acc[d][0], acc[d][1], acc[d][2], acc[d][3]);
  }
  if (kb == 0) {
    s_m[wave * 16 + col] = m_run;
    s_l[wave * 16 + col] = l;
  }
  __syncthreads();
  // thread t sums four dims of one head over the waves
  const int t = threadIdx.x;
  if (t >= G * (HD / 4)) return;
  const int head = t / (HD / 4), dim = (t % (HD / 4)) * 4;
  float m_all = s_m[head];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) m_all = fmaxf(m_all, s_m[w * 16 + head]);  // finite: wave 0 has a tile
  float l_all = 0.f;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const float weight = fast_exp2(s_m[w * 16 + head] - m_all);  // exp2(-inf) = 0 for a wave without a tile
    l_all = fmaf(weight, s_l[w * 16 + head], l_all);
    const float4 v = *reinterpret_cast<const float4*>(s_acc + ((size_t)w * G + head) * HD + dim);
    o.x = fmaf(weight, v.x, o.x);
    o.y = fmaf(weight, v.y, o.y);
    o.z = fmaf(weight, v.z, o.z);
    o.w = fmaf(weight, v.w, o.w);
  }
  const size_t row = (size_t)n0 * nh + kvh * G + head;
  const size_t prow = ((size_t)item * nh + kvh * G + head) * nsplit + split;  // partials are indexed by item, not token
  if (nsplit == 1) {
    const float inv = 1.f / l_all;
    *reinterpret_cast<uint2*>(out + row * HD + dim) =
        make_uint2(pack_bf16x2(o.x * inv, o.y * inv), pack_bf16x2(o.z * inv, o.w * inv));
  } else {
    *reinterpret_cast<float4*>(part_o + prow * HD + dim) = o;
    if (dim == 0) {
      part_ml[prow * 2] = m_all;
      part_ml[prow * 2 + 1] = l_all;
    }
  }
}

// Merge the splits of every (token, head): out = sum_s w_s o_s / sum_s w_s l_s,
// w_s = exp2(m_s - max m).  Splits that hold no key of the token are skipped by
// the token's position, so they need not have been written.  Rows: one per decode
// item (item_count == nullptr), or sixteen per tile of a prompt portion, of which
// the tile's first item_count[tile] are tokens.
template <int HD>
__global__ __launch_bounds__(64) void attention_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int* __restrict__ positions, const int* __restrict__ item_token,
    const int* __restrict__ item_count, bf16_t* __restrict__ out, int nsplit, int split_keys, int nh) {
  const int head = blockIdx.y, lane = threadIdx.x;
  int n;
  if (item_count == nullptr) {
    n = item_token[blockIdx.x];
  } else {
    const int tile = blockIdx.x >> 4, t = blockIdx.x & 15;
    if (t >= item_count[tile]) return;
    n = item_token[tile] + t;
  }
  const size_t row = (size_t)blockIdx.x * nh + head;  // partial row
  const size_t orow = (size_t)n * nh + head;          // output row (by token)
  // Where the partials lie follows from the block alone, how many of them count from the
  // token's position: the first splits' partials are asked for before the position is known
  // (one memory round trip instead of three in a row; what a split that does not count left
  // there is not used).
  constexpr int kAhead = 8;
  const float* ml = part_ml + row * nsplit * 2;
  const float* po0 = part_o + row * nsplit * HD;
  float m_first = -INFINITY, l_first = 0.f;
  if (lane < nsplit) {
    m_first = ml[lane * 2];
    l_first = ml[lane * 2 + 1];
  }
  float ahead[kAhead][HD / 64];
#pragma unroll
  for (int t = 0; t < kAhead; ++t)
#pragma unroll
    for (int i = 0; i < HD / 64; ++i) ahead[t][i] = t < nsplit ? po0[(size_t)t * HD + lane + i * 64] : 0.f;
  // splits that hold keys: of a decode token by its own even cut, of a tile by the step's
  const int pos = positions[n];
  const int used = min(nsplit, pos / (item_count == nullptr ? decode_share(pos + 1, nsplit) : split_keys) + 1);
  // lane s holds split s's (m, l): one load each, then the maximum over the wave
  float mx = lane < used ? m_first : -INFINITY;
  for (int s = lane + kWave; s < used; s += kWave) mx = fmaxf(mx, ml[s * 2]);
  mx = wave_max(mx);
  float denom = 0.f;
  float o[HD / 64];
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) o[i] = 0.f;
  for (int s0 = 0; s0 < used; s0 += kWave) {
    const int mine = s0 + lane;
    const float m_mine = s0 == 0 ? m_first : (mine < used ? ml[mine * 2] : 0.f);
    const float l_mine = s0 == 0 ? l_first : (mine < used ? ml[mine * 2 + 1] : 0.f);
    const float w_mine = mine < used ? fast_exp2(m_mine - mx) : 0.f;
    denom += mine < used ? w_mine * l_mine : 0.f;
    const int count = min(kWave, used - s0);
    const float* po = po0 + (size_t)s0 * HD;
    int t = 0;
    if (s0 == 0) {
#pragma unroll
      for (; t < kAhead; ++t) {
        if (t >= count) break;
        const float w = __shfl(w_mine, t, kWave);
#pragma unroll
        for (int i = 0; i < HD / 64; ++i) o[i] = fmaf(w, ahead[t][i], o[i]);
      }
    }
#pragma unroll 4
    for (; t < count; ++t) {
      const float w = __shfl(w_mine, t, kWave);
#pragma unroll
      for (int i = 0; i < HD / 64; ++i) o[i] = fmaf(w, po[(size_t)t * HD + lane + i * 64], o[i]);
    }
  }
  const float inv = 1.f / wave_sum(denom);
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) out[orow * HD + lane + i * 64] = float_to_bf16(o[i] * inv);
}

// ---------------------------------------------------------------------------
// Prompt portions: one block of four waves per (16-token tile, kv head, group of
// HPB query heads); wave w < HPB owns query head w of the group, and all four
// waves load.  The waves share the keys and values: the block copies 64 keys at a
// time from the pages into LDS, the following stages already being in flight into
// registers while the current one is multiplied.  K keeps the page's piece order
// ([dim/8][key][8]); V is regrouped on the way in so that the eight values a lane
// needs for one PV product (four keys of an even 16-key group, four of the odd one
// after it, one dim) lie in one 16-byte piece (pieces xor-swizzled against bank
// conflicts of the 8-byte writes).  Per 64 keys a wave does one softmax
// update: 16 QK^T products (16x16x32), one maximum, one rescale, then 16 PV
// products (16x16x32, the k index running over quads of two 16-key groups, which
// is exactly how the lanes hold the probabilities).
// Every page lookup is wave-uniform (a piece's 16-key group depends on the wave
// only), so a load's address is a scalar base plus a per-lane constant.
// ---------------------------------------------------------------------------
constexpr int kPrefillThreads = 256;

// OCC: waves a SIMD the compiler must leave room for.  Three (what OCC = 2 gives) are best
// when tiles differ in length (a prompt from position zero: the longest tile's walk
// decides); four (a few registers spilled) when every tile walks a long context.
template <int HD, int HPB, int OCC>
__global__ __launch_bounds__(kPrefillThreads) __attribute__((amdgpu_waves_per_eu(OCC)))
void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ item_token, const int* __restrict__ item_count,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int nsplit,
    int split_keys, int num_items, int nh, int nkv, int ps, float scale_log2) {
  constexpr int KCH = HD / 32, DBL = HD / 16;
  constexpr int THREADS = kPrefillThreads;
  constexpr int GROUP_PIECES = 2 * HD;         // 16-byte pieces of K (and of V) per 16-key group
  constexpr int PIECES = 4 * GROUP_PIECES;     // per stage of 64 keys
  constexpr int PPT = PIECES / THREADS;        // pieces of K, and of V, per thread and stage
  constexpr int NBUF = 1;                      // register sets of prefetch
  static_assert(GROUP_PIECES % 64 == 0, "a wave's pieces of one load lie in one 16-key group");
  __shared__ __attribute__((aligned(16))) bf16_t ks[PIECES * 8];
  __shared__ __attribute__((aligned(16))) bf16_t vs[PIECES * 8];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int G = nh / nkv;
  const int groups_per_kv = G / HPB;
  const int kvh = blockIdx.x / groups_per_kv;
  const bool computes = wave < HPB;
  const int head = kvh * G + (blockIdx.x % groups_per_kv) * HPB + (computes ? wave : 0);
  const int item = num_items - 1 - blockIdx.y;  // later tiles have more keys: start them first

  const int n0 = item_token[item];
  const int count = item_count[item];
  const int pos0 = positions[n0];
  const int last_pos = pos0 + count - 1;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t page_elems = (size_t)nkv * HD * ps;
  const size_t head_off = (size_t)kvh * HD * ps;
  const int c_pos = pos0 + col;
  const bool c_valid = col < count;
  // With several splits (few tiles over a long context) this block takes the keys
  // [k_begin, k_begin + split_keys), a multiple of 64, and writes an unnormalised partial.
  const int split = blockIdx.z;
  const int k_begin = split * split_keys;
  if (k_begin > last_pos) return;  // no key of this tile lies in the split (the whole block leaves)
  const int last_key = min(last_pos, k_begin + split_keys - 1);

  bf16x8 qreg[KCH];
  {
    const bf16_t* qp = q + ((size_t)(n0 + (c_valid ? col : 0)) * nh + head) * HD + kb * 8;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      Frag8 f;
      f.u = *reinterpret_cast<const uint4*>(qp + c * 32);
      if (!c_valid) f.u = make_uint4(0, 0, 0, 0);
      qreg[c] = f.v;
    }
  }

  float m_run = -INFINITY, l_run = 0.f;
  float4v acc[DBL];
#pragma unroll
  for (int d = 0; d < DBL; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  // Piece p = i * THREADS + tid of a stage.  K: (group j, dim chunk c8, key) =
  // (p / GROUP_PIECES, (p / 16) % (HD/8), p % 16).  V: (group j, dim block d, quad, dim
  // pair) = (p / GROUP_PIECES, (p / 32) % DBL, (p % 32) / 8, p % 8): two dims x four keys.
  u32x4 kpre[NBUF][PPT], vpre[NBUF][PPT];
  const int ps_shift = __ffs(ps) - 1;  // page sizes are powers of two here
  int grp[PPT];                        // wave-uniform
  unsigned k_in[PPT], v_in[PPT];       // byte offset inside the page's head, for key 0 of a group
  int v_quad[PPT];
  unsigned v_lds[PPT][2];              // element offsets in vs of the piece's two dims
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int p = i * THREADS + tid;
    grp[i] = __builtin_amdgcn_readfirstlane(p / GROUP_PIECES);
    k_in[i] = (unsigned)((((p / 16) % (HD / 8)) * ps + (p % 16)) * 8) * 2u;
    const int d = (p / 32) % DBL, quad = (p % 32) / 8, dp = p % 8;
    v_in[i] = (unsigned)(d * (ps >> 2) * 64 + (p % 32) * 8) * 2u;
    v_quad[i] = quad;
    // vs: [pair of groups h][d][quad][slot = dim col ^ quad][group parity][4 keys]; the
    // xor spreads a wave's 8-byte writes over all banks and keeps the reads contiguous
#pragma unroll
    for (int half = 0; half < 2; ++half)
      v_lds[i][half] = (unsigned)((((((p / GROUP_PIECES) >> 1) * DBL + d) * 4 + quad) * 16 +
                                   ((2 * dp + half) ^ quad)) * 2 + ((p / GROUP_PIECES) & 1)) * 4u;
  }
  // A group past the request's end reads the stage's first group instead (valid
  // memory, masked later), so no load is predicated and all of a stage's loads are
  // in flight together.  The page numbers of a stage are looked up one fetch ahead
  // (scalar loads), so their latency is never waited for.
  int page_next[PPT];  // of the 16-key group of this wave's piece i
#define TK_PAGES(S0)                                                             \
  if ((S0) <= last_key) {                                                        \
    _Pragma("unroll") for (int i = 0; i < PPT; ++i) {                            \
      const int c0 = ((S0) + grp[i] * 16 <= last_pos) ? (S0) + grp[i] * 16 : (S0); \
      page_next[i] = table[c0 >> ps_shift];                                      \
    }                                                                            \
  }
#define TK_FETCH(S0, BUF)                                                                        \
  {                                                                                              \
    _Pragma("unroll") for (int i = 0; i < PPT; ++i) {                                            \
      const int c0 = ((S0) + grp[i] * 16 <= last_pos) ? (S0) + grp[i] * 16 : (S0);               \
      const size_t pg = (size_t)__builtin_amdgcn_readfirstlane(page_next[i]) * page_elems + head_off; \
      const int off = c0 & (ps - 1);                                                             \
      const char* kp = reinterpret_cast<const char*>(k_cache + pg + (size_t)off * 8);            \
      const char* vp = reinterpret_cast<const char*>(v_cache + pg + (size_t)(off >> 2) * 64);    \
      kpre[BUF][i] = *reinterpret_cast<const u32x4*>(kp + k_in[i]);                              \
      vpre[BUF][i] = *reinterpret_cast<const u32x4*>(vp + v_in[i]);                              \
    }                                                                                            \
    TK_PAGES((S0) + 64)                                                                          \
  }

  TK_PAGES(k_begin)
#pragma unroll
  for (int b = 0; b < NBUF; ++b)
    if (b == 0 || k_begin + b * 64 <= last_key) TK_FETCH(k_begin + b * 64, b)
  for (int sp = k_begin; sp <= last_key; sp += 64 * NBUF) {
#pragma unroll
   for (int buf = 0; buf < NBUF; ++buf) {
    const int s0 = sp + buf * 64;
    if (s0 > last_key) break;
    __syncthreads();  // every wave has read the previous stage
    if (s0 + 63 > last_pos) {
      // keys past the request's end may hold anything (their probability is zero, but
      // 0 * NaN is NaN): zero their values on the way into LDS
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int k0 = s0 + grp[i] * 16 + v_quad[i] * 4;
        const unsigned m01 = (k0 + 0 > last_pos ? 0u : 0x0000ffffu) | (k0 + 1 > last_pos ? 0u : 0xffff0000u);
        const unsigned m23 = (k0 + 2 > last_pos ? 0u : 0x0000ffffu) | (k0 + 3 > last_pos ? 0u : 0xffff0000u);
        vpre[buf][i] &= u32x4{m01, m23, m01, m23};
      }
    }
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      *reinterpret_cast<u32x4*>(ks + (size_t)(i * THREADS + tid) * 8) = kpre[buf][i];
      *reinterpret_cast<uint2*>(vs + v_lds[i][0]) = make_uint2(vpre[buf][i][0], vpre[buf][i][1]);
      *reinterpret_cast<uint2*>(vs + v_lds[i][1]) = make_uint2(vpre[buf][i][2], vpre[buf][i][3]);
    }
    __syncthreads();
    if (s0 + 64 * NBUF <= last_key) TK_FETCH(s0 + 64 * NBUF, buf)
    if (!computes) continue;

    // S^T for 4 groups of 16 keys
    float sv[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        Frag8 kf;
        kf.u = *reinterpret_cast<const uint4*>(ks + ((size_t)(j * (HD / 8) + c * 4 + kb) * 16 + col) * 8);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qreg[c], sc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sv[j][i] = sc[i];
    }
    if (s0 + 63 > pos0) {  // some key of this stage is hidden from some column, or is past the end
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = s0 + j * 16 + kb * 4 + i;
          if (key > c_pos || key > last_pos) sv[j][i] = -INFINITY;
        }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, sv[j][i]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    // the running maximum is kept in units of log2: m = max(score) * scale * log2(e)
    const float m_new = fmaxf(m_run, tmax * scale_log2);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float psum = 0.f;
    Frag8 pb[2];  // pb[h]: groups 2h and 2h+1, four probabilities each
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = fast_exp2(fmaf(sv[2 * h][i], scale_log2, -m_safe));
        p[4 + i] = fast_exp2(fmaf(sv[2 * h + 1][i], scale_log2, -m_safe));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) psum += p[i];
      pb[h].u = make_uint4(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                           pack_bf16x2(p[6], p[7]));
    }
    l_run = l_run * alpha + psum;
    // the accumulators need rescaling only when some column's maximum moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int d = 0; d < DBL; ++d) acc[d] *= alpha;
    }
#pragma unroll
    for (int d = 0; d < DBL; ++d) {
      float4v a = acc[d];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // A operand: V^T[dim col][k], k = (group 2h quad kb) then (group 2h+1 quad kb)
        Frag8 vf;
        vf.u = *reinterpret_cast<const uint4*>(vs + ((size_t)((h * DBL + d) * 4 + kb) * 16 + (col ^ kb)) * 8);
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pb[h].v, a, 0, 0, 0);
      }
      acc[d] = a;
    }
   }
  }

  float l = l_run;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (c_valid && computes) {
    if (nsplit == 1) {
      const float inv = 1.f / l;
      bf16_t* op = out + ((size_t)(n0 + col) * nh + head) * HD + kb * 4;
#pragma unroll
      for (int d = 0; d < DBL; ++d) {
        uint2 o;
        o.x = pack_bf16x2(acc[d][0] * inv, acc[d][1] * inv);
        o.y = pack_bf16x2(acc[d][2] * inv, acc[d][3] * inv);
        *reinterpret_cast<uint2*>(op + d * 16) = o;
      }
    } else {
      // partial rows: sixteen per tile, by the token's place in the tile
      const size_t prow = ((size_t)(item * 16 + col) * nh + head) * nsplit + split;
      float* po = part_o + prow * HD + kb * 4;
#pragma unroll
      for (int d = 0; d < DBL; ++d)
        *reinterpret_cast<float4*>(po + d * 16) = make_float4(acc[d][0], acc[d][1], acc[d][2], acc[d][3]);
      if (kb == 0) {
        part_ml[prow * 2] = m_run;
        part_ml[prow * 2 + 1] = l;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Prompt portions, wide form: a tile is up to 32 consecutive tokens of one request, a
// wave owns the tile's 32 queries of one query head, and the products are
// v_mfma_f32_32x32x16_bf16 (twice the work of a 16x16x32 per operand read from LDS, and
// the shape that reaches the matrix cores' full rate).  As in the narrow form above, the
// block of four waves shares 64 keys at a time through LDS, wave w < HPB owns head w of
// the block's group, and every page lookup is wave-uniform.
//   S^T[key][query] = K[key][:] . Q[query][:]   A = K rows (32 keys x 16 dims), B = Q
//   O^T[dim][query] += V^T[dim][key] P^T[key][query]
// A lane holds, of a 32-key block of S^T, the keys 8i + 4g + j (g = lane / 32; i, j < 4)
// of its query: exactly the B operand of the second product if that product's sixteen
// keys are taken in the order (g: four keys of quad 4h+g, then four of quad 4h+2+g).
// V goes into LDS in that order ([16-key group][g][dim][two quads]), so its A operand is
// one 16-byte read, contiguous over the wave's 32 dims.  K keeps the page's piece order.
// No key split here (the narrow form has it for few tiles over long contexts).
// ---------------------------------------------------------------------------
typedef float float16v __attribute__((ext_vector_type(16)));

template <int HD, int HPB>
__global__ __launch_bounds__(kPrefillThreads) __attribute__((amdgpu_waves_per_eu(2)))
void attention_prefill_wide_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ item_token, const int* __restrict__ item_count,
    bf16_t* __restrict__ out, int num_items, int nh, int nkv, int ps, float scale_log2) {
  constexpr int KST = HD / 16;  // 16-wide steps over the head dim (QK^T)
  constexpr int DB = HD / 32;   // 32-wide blocks of the head dim (PV outputs)
  constexpr int DBL = HD / 16;  // 16-dim blocks of a V page
  constexpr int THREADS = kPrefillThreads;
  constexpr int GROUP_PIECES = 2 * HD;      // 16-byte pieces of K (and of V) per 16-key group
  constexpr int PIECES = 4 * GROUP_PIECES;  // per stage of 64 keys
  constexpr int PPT = PIECES / THREADS;     // pieces of K, and of V, per thread and stage
  constexpr int NBUF = 1;
  static_assert(GROUP_PIECES % 64 == 0, "a wave's pieces of one load lie in one 16-key group");
  __shared__ __attribute__((aligned(16))) bf16_t ks[PIECES * 8];
  __shared__ __attribute__((aligned(16))) bf16_t vs[PIECES * 8];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, g = lane >> 5;
  const int G = nh / nkv;
  const int groups_per_kv = G / HPB;
  const int kvh = blockIdx.x / groups_per_kv;
  const bool computes = wave < HPB;
  const int head = kvh * G + (blockIdx.x % groups_per_kv) * HPB + (computes ? wave : 0);
  const int item = num_items - 1 - blockIdx.y;  // later tiles have more keys: start them first

  const int n0 = item_token[item];
  const int count = item_count[item];
  const int pos0 = positions[n0];
  const int last_pos = pos0 + count - 1;
  const int last_key = last_pos;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t page_elems = (size_t)nkv * HD * ps;
  const size_t head_off = (size_t)kvh * HD * ps;
  const int c_pos = pos0 + col;
  const bool c_valid = col < count;

  // Q as B operand: lane (query col, g) holds Q[col][16c + 8g .. +8]
  bf16x8 qreg[KST];
  {
    const bf16_t* qp = q + ((size_t)(n0 + (c_valid ? col : 0)) * nh + head) * HD + g * 8;
#pragma unroll
    for (int c = 0; c < KST; ++c) {
      Frag8 f;
      f.u = *reinterpret_cast<const uint4*>(qp + c * 16);
      if (!c_valid) f.u = make_uint4(0, 0, 0, 0);
      qreg[c] = f.v;
    }
  }

  float m_run = -INFINITY, l_run = 0.f;
  float16v acc[DB];  // acc[db][4i + j] = O^T[dim 32 db + 8i + 4g + j][col]
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[d][e] = 0.f;

  // Piece p = i * THREADS + tid of a stage, as the pages hold it.  K: (group j, dim chunk
  // c8, key) = (p / GROUP_PIECES, (p / 16) % (HD/8), p % 16), kept in that order in LDS.
  // V: (group j, dim block d, quad, dim pair) = (p / GROUP_PIECES, (p / 32) % DBL,
  // (p % 32) / 8, p % 8): two dims x four keys.
  u32x4 kpre[NBUF][PPT], vpre[NBUF][PPT];
  const int ps_shift = __ffs(ps) - 1;  // page sizes are powers of two here
  int grp[PPT];                        // wave-uniform
  unsigned k_in[PPT], v_in[PPT];       // byte offset inside the page's head, for key 0 of a group
  int v_quad[PPT];
  unsigned v_lds[PPT][2];              // element offsets in vs of the piece's two dims
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int p = i * THREADS + tid;
    grp[i] = __builtin_amdgcn_readfirstlane(p / GROUP_PIECES);
    k_in[i] = (unsigned)((((p / 16) % (HD / 8)) * ps + (p % 16)) * 8) * 2u;
    const int d = (p / 32) % DBL, quad = (p % 32) / 8, dp = p % 8;
    v_in[i] = (unsigned)(d * (ps >> 2) * 64 + (p % 32) * 8) * 2u;
    v_quad[i] = quad;
    // vs: [group j][g = quad & 1][dim][quad >> 1][4 keys]
#pragma unroll
    for (int half = 0; half < 2; ++half)
      v_lds[i][half] =
          (unsigned)(((((p / GROUP_PIECES) * 2 + (quad & 1)) * HD + d * 16 + 2 * dp + half) * 2 + (quad >> 1)) * 4);
  }
  int page_next[PPT];

  TK_PAGES(0)
  TK_FETCH(0, 0)
  for (int s0 = 0; s0 <= last_key; s0 += 64) {
    constexpr int buf = 0;
    __syncthreads();  // every wave has read the previous stage
    if (s0 + 63 > last_pos) {
      // keys past the request's end may hold anything (their probability is zero, but
      // 0 * NaN is NaN): zero their values on the way into LDS
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        const int k0 = s0 + grp[i] * 16 + v_quad[i] * 4;
        const unsigned m01 = (k0 + 0 > last_pos ? 0u : 0x0000ffffu) | (k0 + 1 > last_pos ? 0u : 0xffff0000u);
        const unsigned m23 = (k0 + 2 > last_pos ? 0u : 0x0000ffffu) | (k0 + 3 > last_pos ? 0u : 0xffff0000u);
        vpre[buf][i] &= u32x4{m01, m23, m01, m23};
      }
    }
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      *reinterpret_cast<u32x4*>(ks + (size_t)(i * THREADS + tid) * 8) = kpre[buf][i];
      *reinterpret_cast<uint2*>(vs + v_lds[i][0]) = make_uint2(vpre[buf][i][0], vpre[buf][i][1]);
      *reinterpret_cast<uint2*>(vs + v_lds[i][1]) = make_uint2(vpre[buf][i][2], vpre[buf][i][3]);
    }
    __syncthreads();
    if (s0 + 64 <= last_key) TK_FETCH(s0 + 64, buf)
    if (!computes) continue;

    // S^T for two blocks of 32 keys: sc[kb][4i + j] = score of key s0 + 32 kb + 8i + 4g + j
    float16v sc[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int e = 0; e < 16; ++e) sc[kb][e] = 0.f;
#pragma unroll
      for (int c = 0; c < KST; ++c) {
        Frag8 kf;  // K[key 32 kb + col][16c + 8g .. +8]: piece (group 2kb + col/16, chunk 2c + g, key col%16)
        kf.u = *reinterpret_cast<const uint4*>(
            ks + ((size_t)((2 * kb + (col >> 4)) * (HD / 8) + 2 * c + g) * 16 + (col & 15)) * 8);
        sc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qreg[c], sc[kb], 0, 0, 0);
      }
    }
    if (s0 + 63 > pos0) {  // some key of this stage is hidden from some query, or is past the end
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = s0 + 32 * kb + 8 * (e >> 2) + 4 * g + (e & 3);
          if (key > c_pos || key > last_pos) sc[kb][e] = -INFINITY;
        }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, sc[kb][e]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    // the running maximum is kept in units of log2: m = max(score) * scale * log2(e)
    const float m_new = fmaxf(m_run, tmax * scale_log2);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float psum = 0.f;
    Frag8 pb[2][2];  // pb[kb][h]: the sixteen keys 32 kb + 16 h .. of this lane's half
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float pr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pr[e] = fast_exp2(fmaf(sc[kb][8 * h + e], scale_log2, -m_safe));
          psum += pr[e];
        }
        pb[kb][h].u = make_uint4(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]), pack_bf16x2(pr[4], pr[5]),
                                 pack_bf16x2(pr[6], pr[7]));
      }
    l_run = l_run * alpha + psum;
    // the accumulators need rescaling only when some query's maximum moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int d = 0; d < DB; ++d) acc[d] *= alpha;
    }
#pragma unroll
    for (int d = 0; d < DB; ++d) {
      float16v a = acc[d];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          Frag8 vf;  // V^T[dim 32 d + col][the lane half's eight keys of group 2 kb + h]
          vf.u = *reinterpret_cast<const uint4*>(vs + ((size_t)((2 * kb + h) * 2 + g) * HD + 32 * d + col) * 8);
          a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pb[kb][h].v, a, 0, 0, 0);
        }
      acc[d] = a;
    }
  }

  float l = l_run;
  l += __shfl_xor(l, 32, kWave);
  if (c_valid && computes) {
    const float inv = 1.f / l;
    bf16_t* op = out + ((size_t)(n0 + col) * nh + head) * HD + g * 4;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint2 o;
        o.x = pack_bf16x2(acc[d][4 * i] * inv, acc[d][4 * i + 1] * inv);
        o.y = pack_bf16x2(acc[d][4 * i + 2] * inv, acc[d][4 * i + 3] * inv);
        *reinterpret_cast<uint2*>(op + 32 * d + 8 * i) = o;
      }
  }
}

#undef TK_FETCH
#undef TK_PAGES

// ---------------------------------------------------------------------------
// Prompt portions, group form: the wide form's products (tiles of up to 32 tokens,
// v_mfma_f32_32x32x16_bf16) in a block that holds a whole CU: GB query heads of one kv
// head times S shares of the keys, one wave each (GB * S <= 8 waves, two a SIMD with the
// registers the wide form needs).  A stage is 64 * S keys; wave (head hw, share sp) takes
// the stage's keys 64 sp .. 64 sp + 63, and the shares of a head are merged through LDS
// when the tile's keys are done.  Against the wide form with its two independent blocks a
// CU: every kv head's keys and values are copied into LDS once for all its query heads
// (any group size, also 3, 5, 7), and a tile's walk over the keys is S times shorter, so
// that a prompt from position zero, whose tiles differ in length from 32 keys to the whole
// prompt, leaves no CU with one long tile at a quarter of its waves: tiles are started
// longest first, twice as many as there are CUs, and the short ones fill in behind.
// ---------------------------------------------------------------------------
template <int HD, int GB, int S>
__global__ __launch_bounds__(GB * S * 64)
void attention_prefill_group_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ item_token, const int* __restrict__ item_count,
    bf16_t* __restrict__ out, int num_items, int nh, int nkv, int ps, float scale_log2) {
  constexpr int KST = HD / 16;  // 16-wide steps over the head dim (QK^T)
  constexpr int DB = HD / 32;   // 32-wide blocks of the head dim (PV outputs)
  constexpr int DBL = HD / 16;  // 16-dim blocks of a V page
  constexpr int THREADS = GB * S * 64;
  constexpr int STAGE = 64 * S;             // keys a stage
  constexpr int GROUP_PIECES = 2 * HD;      // 16-byte pieces of K (and of V) per 16-key group
  constexpr int SUB_PIECES = 4 * GROUP_PIECES;  // per 64 keys
  constexpr int PIECES = S * SUB_PIECES;    // per stage
  constexpr int PPT = (PIECES + THREADS - 1) / THREADS;
  constexpr bool EVEN = PIECES % THREADS == 0;
  constexpr int ACC = DB * 16;              // accumulator floats a lane
  static_assert(GROUP_PIECES % 64 == 0, "a wave's pieces of one load lie in one 16-key group");
  // two stages in LDS where they fit: the next stage is written while this one is multiplied,
  // and one barrier a stage is enough
  constexpr int NB = (2 * PIECES * 32 <= 160 * 1024) ? 2 : 1;
  constexpr int BUF = 2 * PIECES * 8;       // elements of a stage's K and V
  extern __shared__ __attribute__((aligned(16))) bf16_t smem_group[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, g = lane >> 5;
  const int hw = wave % GB, sp = wave / GB;
  const int G = nh / nkv;
  const int nblk = (G + GB - 1) / GB;
  const int kvh = blockIdx.x / nblk;
  const int hin = (blockIdx.x % nblk) * GB + hw;
  const bool computes = hin < G;
  const int head = kvh * G + (computes ? hin : 0);
  const int item = num_items - 1 - blockIdx.y;  // later tiles have more keys: start them first

  const int n0 = item_token[item];
  const int count = item_count[item];
  const int pos0 = positions[n0];
  const int last_pos = pos0 + count - 1;
  const int last_key = last_pos;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t page_elems = (size_t)nkv * HD * ps;
  const size_t head_off = (size_t)kvh * HD * ps;
  const int c_pos = pos0 + col;
  const bool c_valid = col < count;

  // Q as B operand: lane (query col, g) holds Q[col][16c + 8g .. +8]
  bf16x8 qreg[KST];
  {
    const bf16_t* qp = q + ((size_t)(n0 + (c_valid ? col : 0)) * nh + head) * HD + g * 8;
#pragma unroll
    for (int c = 0; c < KST; ++c) {
      Frag8 f;
      f.u = *reinterpret_cast<const uint4*>(qp + c * 16);
      if (!c_valid) f.u = make_uint4(0, 0, 0, 0);
      qreg[c] = f.v;
    }
  }

  float m_run = -INFINITY, l_run = 0.f;
  float16v acc[DB];  // acc[db][4i + j] = O^T[dim 32 db + 8i + 4g + j][col]
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[d][e] = 0.f;

  // Piece p = i * THREADS + tid of a stage: share p / SUB_PIECES, and within the share's 64
  // keys as the wide form has it.
  u32x4 kpre[PPT], vpre[PPT];
  const int ps_shift = __ffs(ps) - 1;  // page sizes are powers of two here
  int grp[PPT];                        // 16-key group within the stage; wave-uniform
  unsigned k_in[PPT], v_in[PPT];       // byte offset inside the page's head, for key 0 of a group
  int v_quad[PPT];
  unsigned v_lds[PPT][2];              // element offsets in vs of the piece's two dims
  bool piece[PPT];                     // wave-uniform: the piece exists
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int pa = i * THREADS + tid;
    piece[i] = EVEN || pa < PIECES;
    const int share = pa / SUB_PIECES, p = pa % SUB_PIECES;
    grp[i] = __builtin_amdgcn_readfirstlane(piece[i] ? share * 4 + p / GROUP_PIECES : 0);
    k_in[i] = (unsigned)((((p / 16) % (HD / 8)) * ps + (p % 16)) * 8) * 2u;
    const int d = (p / 32) % DBL, quad = (p % 32) / 8, dp = p % 8;
    v_in[i] = (unsigned)(d * (ps >> 2) * 64 + (p % 32) * 8) * 2u;
    v_quad[i] = quad;
    // vs, per share: [group j][g = quad & 1][dim][quad >> 1][4 keys]
#pragma unroll
    for (int half = 0; half < 2; ++half)
      v_lds[i][half] = (unsigned)(share * SUB_PIECES * 8) +
          (unsigned)(((((p / GROUP_PIECES) * 2 + (quad & 1)) * HD + d * 16 + 2 * dp + half) * 2 + (quad >> 1)) * 4);
  }
  int page_next[PPT];
#define TK_GPAGES(S0)                                                              \
  if ((S0) <= last_key) {                                                          \
    _Pragma("unroll") for (int i = 0; i < PPT; ++i) {                              \
      const int c0 = ((S0) + grp[i] * 16 <= last_pos) ? (S0) + grp[i] * 16 : (S0); \
      page_next[i] = table[c0 >> ps_shift];                                        \
    }                                                                              \
  }
#define TK_GFETCH(S0)                                                                              \
  {                                                                                                \
    _Pragma("unroll") for (int i = 0; i < PPT; ++i) if (piece[i]) {                                \
      const int c0 = ((S0) + grp[i] * 16 <= last_pos) ? (S0) + grp[i] * 16 : (S0);                 \
      const size_t pg = (size_t)__builtin_amdgcn_readfirstlane(page_next[i]) * page_elems + head_off; \
      const int off = c0 & (ps - 1);                                                               \
      const char* kp = reinterpret_cast<const char*>(k_cache + pg + (size_t)off * 8);              \
      const char* vp = reinterpret_cast<const char*>(v_cache + pg + (size_t)(off >> 2) * 64);      \
      kpre[i] = *reinterpret_cast<const u32x4*>(kp + k_in[i]);                                     \
      vpre[i] = *reinterpret_cast<const u32x4*>(vp + v_in[i]);                                     \
    }                                                                                              \
    TK_GPAGES((S0) + STAGE)                                                                        \
  }

  // keys past the request's end may hold anything (their probability is zero, but 0 * NaN
  // is NaN): their values are zeroed on the way into LDS
#define TK_GSTORE(S0, KS, VS)                                                                        \
  {                                                                                                  \
    if ((S0) + STAGE - 1 > last_pos) {                                                               \
      _Pragma("unroll") for (int i = 0; i < PPT; ++i) {                                              \
        const int k0 = (S0) + grp[i] * 16 + v_quad[i] * 4;                                           \
        const unsigned m01 = (k0 + 0 > last_pos ? 0u : 0x0000ffffu) | (k0 + 1 > last_pos ? 0u : 0xffff0000u); \
        const unsigned m23 = (k0 + 2 > last_pos ? 0u : 0x0000ffffu) | (k0 + 3 > last_pos ? 0u : 0xffff0000u); \
        vpre[i] &= u32x4{m01, m23, m01, m23};                                                        \
      }                                                                                              \
    }                                                                                                \
    _Pragma("unroll") for (int i = 0; i < PPT; ++i) if (piece[i]) {                                  \
      *reinterpret_cast<u32x4*>((KS) + (size_t)(i * THREADS + tid) * 8) = kpre[i];                   \
      *reinterpret_cast<uint2*>((VS) + v_lds[i][0]) = make_uint2(vpre[i][0], vpre[i][1]);            \
      *reinterpret_cast<uint2*>((VS) + v_lds[i][1]) = make_uint2(vpre[i][2], vpre[i][3]);            \
    }                                                                                                \
  }
  TK_GPAGES(0)
  TK_GFETCH(0)
  if (NB == 2) {
    TK_GSTORE(0, smem_group, smem_group + PIECES * 8)
    if (STAGE <= last_key) TK_GFETCH(STAGE)
    __syncthreads();
  }
  for (int s0 = 0; s0 <= last_key; s0 += STAGE) {
    bf16_t* ks = smem_group;
    if (NB == 2) {
      // this stage lies in buffer (s0 / STAGE) & 1; the next one, on its way in registers since
      // the stage before, goes into the other buffer, which every wave has left behind
      const int b = (s0 / STAGE) & 1;
      ks = smem_group + (size_t)b * BUF;
      if (s0 + STAGE <= last_key) {
        bf16_t* kn = smem_group + (size_t)(b ^ 1) * BUF;
        TK_GSTORE(s0 + STAGE, kn, kn + PIECES * 8)
        if (s0 + 2 * STAGE <= last_key) TK_GFETCH(s0 + 2 * STAGE)
      }
    } else {
      __syncthreads();  // every wave has read the previous stage
      TK_GSTORE(s0, ks, ks + PIECES * 8)
      __syncthreads();
      if (s0 + STAGE <= last_key) TK_GFETCH(s0 + STAGE)
    }
    const bf16_t* const ksw = ks + (size_t)sp * SUB_PIECES * 8;  // this wave's share of the stage
    const bf16_t* const vsw = ksw + PIECES * 8;
    const int w0 = s0 + 64 * sp;  // this wave's 64 keys of the stage
    if (computes && w0 <= last_key) {

    // S^T for two blocks of 32 keys: sc[kb][4i + j] = score of key w0 + 32 kb + 8i + 4g + j.
    // A block's operands are asked for together, and the second block's while the first
    // block's products run: a wave that waits for each operand in turn spends its time on
    // round trips to LDS (some hundred clocks each), not on the products.
    float16v sc[2];
    {
      Frag8 kf[2][KST];  // K[key 32 kb + col][16c + 8g .. +8]: piece (group 2kb + col/16, chunk 2c + g, key col%16)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) sc[kb][e] = 0.f;
#pragma unroll
        for (int c = 0; c < KST; ++c)
          kf[kb][c].u = *reinterpret_cast<const uint4*>(
              ksw + ((size_t)((2 * kb + (col >> 4)) * (HD / 8) + 2 * c + g) * 16 + (col & 15)) * 8);
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int c = 0; c < KST; ++c)
          sc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb][c].v, qreg[c], sc[kb], 0, 0, 0);
      // the order asked of the scheduler: the first block's reads; a product and a read of the
      // second block in turn; the second block's products
      __builtin_amdgcn_sched_group_barrier(0x100, KST, 0);
#pragma unroll
      for (int c = 0; c < KST; ++c) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, KST, 0);
    }
    if (w0 + 63 > pos0) {  // some key of these is hidden from some query, or is past the end
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = w0 + 32 * kb + 8 * (e >> 2) + 4 * g + (e & 3);
          if (key > c_pos || key > last_pos) sc[kb][e] = -INFINITY;
        }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, sc[kb][e]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    // the running maximum is kept in units of log2: m = max(score) * scale * log2(e)
    const float m_new = fmaxf(m_run, tmax * scale_log2);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float psum = 0.f;
    Frag8 pb[2][2];  // pb[kb][h]: the sixteen keys 32 kb + 16 h .. of this lane's half
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float pr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pr[e] = fast_exp2(fmaf(sc[kb][8 * h + e], scale_log2, -m_safe));
          psum += pr[e];
        }
        pb[kb][h].u = make_uint4(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]), pack_bf16x2(pr[4], pr[5]),
                                 pack_bf16x2(pr[6], pr[7]));
      }
    l_run = l_run * alpha + psum;
    // the accumulators need rescaling only when some query's maximum moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int d = 0; d < DB; ++d) acc[d] *= alpha;
    }
    {
      // O^T += V^T P^T, a 32-dim block of the output at a time; operands asked for a block ahead
      Frag8 vf[DB][4];  // V^T[dim 32 d + col][the lane half's eight keys of group 2 kb + h]
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int kh = 0; kh < 4; ++kh)
          vf[d][kh].u = *reinterpret_cast<const uint4*>(vsw + ((size_t)(kh * 2 + g) * HD + 32 * d + col) * 8);
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int kh = 0; kh < 4; ++kh)
          acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[d][kh].v, pb[kh >> 1][kh & 1].v, acc[d], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int i = 0; i < 4 * DB - 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
    }
    }  // computes
    if (NB == 2) __syncthreads();  // the next stage is written, and every wave has read this one
  }
#undef TK_GSTORE
#undef TK_GFETCH
#undef TK_GPAGES

  if (S > 1) {
    // the shares of a head meet in LDS: share sp > 0 leaves its (acc, m, l), share 0 adds them
    // in share order.  Per (share - 1, head): ACC rows of 64 lanes, then m and l.
    float* const ms = reinterpret_cast<float*>(smem_group);
    constexpr int PER = (ACC + 2) * 64;
    __syncthreads();  // every wave has read the last stage
    if (sp > 0) {
      float* mine = ms + (size_t)((sp - 1) * GB + hw) * PER;
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) mine[(d * 16 + e) * 64 + lane] = acc[d][e];
      mine[ACC * 64 + lane] = m_run;
      mine[(ACC + 1) * 64 + lane] = l_run;
    }
    __syncthreads();
    if (sp > 0) return;
#pragma unroll
    for (int s = 1; s < S; ++s) {
      const float* theirs = ms + (size_t)((s - 1) * GB + hw) * PER;
      const float m2 = theirs[ACC * 64 + lane], l2 = theirs[(ACC + 1) * 64 + lane];
      const float m_new = fmaxf(m_run, m2);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float a1 = fast_exp2(m_run - m_safe), a2 = fast_exp2(m2 - m_safe);
      m_run = m_new;
      l_run = l_run * a1 + l2 * a2;
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[d][e] = acc[d][e] * a1 + theirs[(d * 16 + e) * 64 + lane] * a2;
    }
  }

  float l = l_run;
  l += __shfl_xor(l, 32, kWave);
  if (c_valid && computes) {
    const float inv = 1.f / l;
    bf16_t* op = out + ((size_t)(n0 + col) * nh + head) * HD + g * 4;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint2 o;
        o.x = pack_bf16x2(acc[d][4 * i] * inv, acc[d][4 * i + 1] * inv);
        o.y = pack_bf16x2(acc[d][4 * i + 2] * inv, acc[d][4 * i + 3] * inv);
        *reinterpret_cast<uint2*>(op + 32 * d + 8 * i) = o;
      }
  }
}


template <int HD, int HPB, int OCC>
static int launch_prefill(const void* q, const void* k_cache, const void* v_cache,
                          const int* block_tables, int max_pages, const int* positions,
                          const int* req_of_token, const int* item_token, const int* item_count,
                          int num_items, void* out, float* part_o, float* part_ml, int nsplit,
                          int split_keys, int nh, int nkv, int ps, float scale, hipStream_t stream) {
  const int G = nh / nkv;
  dim3 grid(nkv * (G / HPB), num_items, nsplit);
  attention_prefill_kernel<HD, HPB, OCC><<<grid, kPrefillThreads, 0, stream>>>(
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages,
      positions, req_of_token, item_token, item_count, (bf16_t*)out, part_o, part_ml, nsplit,
      split_keys, num_items, nh, nkv, ps, scale * 1.4426950408889634f);
  if (nsplit > 1) {
    dim3 mgrid(num_items * 16, nh);
    attention_merge_kernel<HD><<<mgrid, 64, 0, stream>>>(part_o, part_ml, positions, item_token, item_count,
                                                         (bf16_t*)out, nsplit, split_keys, nh);
  }
  return launch_status();
}

template <int HD, int HPB>
static int launch_prefill_wide(const void* q, const void* k_cache, const void* v_cache,
                               const int* block_tables, int max_pages, const int* positions,
                               const int* req_of_token, const int* item_token, const int* item_count,
                               int num_items, void* out, int nh, int nkv, int ps, float scale,
                               hipStream_t stream) {
  const int G = nh / nkv;
  dim3 grid(nkv * (G / HPB), num_items);
  attention_prefill_wide_kernel<HD, HPB><<<grid, kPrefillThreads, 0, stream>>>(
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages,
      positions, req_of_token, item_token, item_count, (bf16_t*)out, num_items, nh, nkv, ps,
      scale * 1.4426950408889634f);
  return launch_status();
}

template <int HD, int GB, int S>
static int launch_prefill_group(const void* q, const void* k_cache, const void* v_cache,
                                const int* block_tables, int max_pages, const int* positions,
                                const int* req_of_token, const int* item_token, const int* item_count,
                                int num_items, void* out, int nh, int nkv, int ps, float scale,
                                hipStream_t stream) {
  const int G = nh / nkv;
  constexpr size_t one_stage = (size_t)S * 8 * HD * 16 * 2;                       // K and V of a stage
  constexpr size_t stage_bytes = 2 * one_stage <= 160 * 1024 ? 2 * one_stage : one_stage;  // two where they fit
  constexpr size_t merge_bytes = (size_t)(S - 1) * GB * ((HD / 2 + 2) * 64) * 4;  // the shares' results
  constexpr size_t lds = stage_bytes > merge_bytes ? stage_bytes : merge_bytes;
  static_assert(lds <= 160 * 1024, "a stage must fit the CU's LDS");
  if (lds > 48 * 1024) {
    static bool raised = false;  // per template instance
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_group_kernel<HD, GB, S>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
      }
      raised = true;
    }
  }
  dim3 grid(nkv * ((G + GB - 1) / GB), num_items);
  attention_prefill_group_kernel<HD, GB, S><<<grid, GB * S * 64, lds, stream>>>(
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages,
      positions, req_of_token, item_token, item_count, (bf16_t*)out, num_items, nh, nkv, ps,
      scale * 1.4426950408889634f);
  return launch_status();
}

// Heads of a kv head's group that share a block of the group form, and the shares of the
// keys beside them: as many waves as fit two a SIMD (eight), all heads of the group in one
// block where that is possible.
template <int HD>
static int launch_prefill_group_any(const void* q, const void* k_cache, const void* v_cache,
                                    const int* block_tables, int max_pages, const int* positions,
                                    const int* req_of_token, const int* item_token, const int* item_count,
                                    int num_items, void* out, int nh, int nkv, int ps, float scale,
                                    hipStream_t stream) {
#define TK_GARGS                                                                                  \
  q, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, item_token, item_count, \
      num_items, out, nh, nkv, ps, scale, stream
  const int G = nh / nkv;
  const int nblk = (G + 7) / 8;
  const int gb = (G + nblk - 1) / nblk;  // heads a block: G itself up to 8, else an even share
  switch (gb) {
    case 1: return launch_prefill_group<HD, 1, 4>(TK_GARGS);
    case 2: return launch_prefill_group<HD, 2, 4>(TK_GARGS);
    case 3: return launch_prefill_group<HD, 3, 2>(TK_GARGS);
    case 4: return launch_prefill_group<HD, 4, 2>(TK_GARGS);
    case 5: return launch_prefill_group<HD, 5, 1>(TK_GARGS);
    case 6: return launch_prefill_group<HD, 6, 1>(TK_GARGS);
    case 7: return launch_prefill_group<HD, 7, 1>(TK_GARGS);
    case 8: return launch_prefill_group<HD, 8, 1>(TK_GARGS);
  }
#undef TK_GARGS
  return -2;
}

template <int HD, bool FUSED>
static int launch(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                  int max_pages, const int* positions, const int* req_of_token,
                  const int* item_token, const int* item_count, int num_items, void* out,
                  float* part_o, float* part_ml, int nsplit, int split_keys, int nh, int nkv, int ps,
                  float scale, hipStream_t stream, DecodeInputs in = DecodeInputs{}) {
  if (num_items > 65535) return -1;
  dim3 grid(nkv, num_items, nsplit);
  const int G = nh / nkv;
  // sixteen waves a block and one tile a wave in flight measured best at every batch size
  // (four or eight waves with two tiles: 12 % slower at batch 64, 15 % at batch 8)
  const size_t lds = (size_t)(kDecodeWaves * G * HD + 2 * kDecodeWaves * 16) * 4 + (FUSED ? (size_t)(G + 2) * HD * 2 : 0);
  if (lds > 160 * 1024) return -2;
  if (lds > 48 * 1024) {  // beyond the default limit of dynamic LDS (groups of 7 heads and more)
    static bool raised = false;  // per template instance
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_kernel<HD, kDecodeWaves, 1, FUSED>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
      }
      raised = true;
    }
  }
  attention_decode_kernel<HD, kDecodeWaves, 1, FUSED><<<grid, kDecodeWaves * 64, lds, stream>>>(
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages, positions,
      req_of_token, item_token, item_count, (bf16_t*)out, part_o, part_ml, nsplit, split_keys, nh, nkv, ps,
      scale * 1.4426950408889634f, in);
  if (nsplit > 1) {
    dim3 mgrid(num_items, nh);
    attention_merge_kernel<HD><<<mgrid, 64, 0, stream>>>(part_o, part_ml, positions, item_token, nullptr,
                                                         (bf16_t*)out, nsplit, split_keys, nh);
  }
  return launch_status();
}

// mode 0: heads (every item is one decode token; item_count is ignored; split_keys is a multiple of
//         16 * tk_attention_decode_waves(), a tile for every wave of a block, and nsplit of them
//         cover the longest token; with nsplit > 1 every token's own keys are cut evenly in
//         nsplit, see decode_share)
// mode 1: tokens (item = up to 16 consecutive tokens of one request; with nsplit > 1 split_keys
//         is a multiple of 64 and the partial buffers hold 16 rows per item)
// mode 2: tokens, every tile over a long context (same results; the kernel built for four waves a SIMD)
// mode 3: tokens, wide form (item = up to 32 consecutive tokens of one request; nsplit must be 1)
// mode 4: tokens, group form (items as in mode 3; any group size; a block holds a CU)
// Returns -2 if this shape is not instantiated (the caller uses the generic kernel).
TK_API int tk_attention_decode_waves() { return kDecodeWaves; }

TK_API int tk_attention_mfma(int mode, const void* q, const void* k_cache, const void* v_cache,
                             const int* block_tables, int max_pages, const int* positions,
                             const int* req_of_token, const int* item_token, const int* item_count,
                             int num_items, void* out, float* part_o, float* part_ml, int nsplit,
                             int split_keys, int nh, int nkv, int hd, int ps, float scale,
                             hipStream_t stream) {
  if (num_items <= 0) return 0;
  if (mode < 0 || mode > 4) return -1;
  if (nkv <= 0 || nh % nkv != 0 || ps < 16 || (ps & (ps - 1)) != 0 || split_keys % 16 != 0 || nsplit < 1) return -1;
  if (num_items > 65535 || nh > 65535) return -1;
  const int G = nh / nkv;
#define TK_ARGS                                                                                   \
  q, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, item_token, item_count, \
      num_items, out, part_o, part_ml, nsplit, split_keys, nh, nkv, ps, scale, stream
  if (mode == 0) {
    if (G > 16) return -2;
    if (hd == 128) return launch<128, false>(TK_ARGS);
    if (hd == 64) return launch<64, false>(TK_ARGS);
    return -2;
  }
  if (mode == 4) {
    if (nsplit != 1) return -1;
    if (hd == 128) return launch_prefill_group_any<128>(q, k_cache, v_cache, block_tables, max_pages, positions,
                                                        req_of_token, item_token, item_count, num_items, out, nh,
                                                        nkv, ps, scale, stream);
    if (hd == 64) return launch_prefill_group_any<64>(q, k_cache, v_cache, block_tables, max_pages, positions,
                                                      req_of_token, item_token, item_count, num_items, out, nh,
                                                      nkv, ps, scale, stream);
    return -2;
  }
  const int hpb = (G % 4 == 0) ? 4 : (G % 2 == 0) ? 2 : 1;
  if (mode == 3) {
    if (nsplit != 1) return -1;
#define TK_WARGS                                                                                  \
  q, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, item_token, item_count, \
      num_items, out, nh, nkv, ps, scale, stream
    // (groups of three heads and more take the group form; blocks of two heads or one here)
    if (hd == 128) {
      if (G % 2 == 0) return launch_prefill_wide<128, 2>(TK_WARGS);
      return launch_prefill_wide<128, 1>(TK_WARGS);
    }
    if (hd == 64) {
      if (G % 2 == 0) return launch_prefill_wide<64, 2>(TK_WARGS);
      return launch_prefill_wide<64, 1>(TK_WARGS);
    }
#undef TK_WARGS
    return -2;
  }
  // the keys of a tile may be split too: in whole stages of 64 keys, sixteen partial rows a tile
  if (nsplit > 1 && (split_keys % 64 != 0 || (long)num_items * 16 > 65535)) return -1;
#define TK_PARGS                                                                                  \
  q, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, item_token, item_count, \
      num_items, out, part_o, part_ml, nsplit, split_keys, nh, nkv, ps, scale, stream
  const bool dense = mode == 2;
  if (hd == 128) {
    if (hpb == 4) return dense ? launch_prefill<128, 4, 4>(TK_PARGS) : launch_prefill<128, 4, 2>(TK_PARGS);
    if (hpb == 2) return launch_prefill<128, 2, 2>(TK_PARGS);
    return launch_prefill<128, 1, 2>(TK_PARGS);
  }
  if (hd == 64) {
    if (hpb == 4) return launch_prefill<64, 4, 2>(TK_PARGS);
    if (hpb == 2) return launch_prefill<64, 2, 2>(TK_PARGS);
    return launch_prefill<64, 1, 2>(TK_PARGS);
  }
#undef TK_PARGS
#undef TK_ARGS
  return -2;
}

// Decode tokens straight from the q/k/v projection's output: what tk_qknorm_rope_store
// (elementwise.hip) followed by tk_attention_mfma in mode 0 computes, in one kernel (and a
// merge if nsplit > 1).  qkv: rows of (nh + 2 nkv_in) heads of hd, bfloat16 (parts == 1,
// in_f32 == 0) or `parts` float32 partial sums part_stride elements apart; nkv_in is nkv
// (the token's key and value are made and stored) or 0 (the call only reads the cache).
// q_weight/k_weight: per-head norm weights [hd] or null; rot: hd (tables cos_t/sin_t
// [N, hd/2]) or 0.  Groups of up to 14 query heads.  Returns -2 if not instantiated.
TK_API int tk_attention_decode_fused(const void* qkv, int in_f32, int parts, long part_stride,
                                     const float* q_weight, const float* k_weight, const float* cos_t,
                                     const float* sin_t, int rot, float eps, int nkv_in, void* k_cache,
                                     void* v_cache, const int* block_tables, int max_pages,
                                     const int* positions, const int* req_of_token, const int* item_token,
                                     int num_items, void* out, float* part_o, float* part_ml, int nsplit,
                                     int split_keys, int nh, int nkv, int hd, int ps, float scale,
                                     hipStream_t stream) {
  if (num_items <= 0) return 0;
  if (nkv <= 0 || nh % nkv != 0 || ps < 16 || (ps & (ps - 1)) != 0 || split_keys % (16 * kDecodeWaves) != 0 || nsplit < 1)
    return -1;
  if (num_items > 65535 || nh > 65535 || parts < 1 || (parts > 1 && !in_f32)) return -1;
  if ((nkv_in != 0 && nkv_in != nkv) || (rot != 0 && rot != hd) || (rot != 0 && (!cos_t || !sin_t))) return -1;
  if ((q_weight != nullptr) != (k_weight != nullptr) && nkv_in != 0) return -1;
  const int G = nh / nkv;
  if (G + 2 > kDecodeWaves) return -2;
  DecodeInputs in{qkv, in_f32, parts, part_stride, q_weight, k_weight, cos_t, sin_t, rot, nkv_in, eps};
#define TK_FARGS                                                                                       \
  nullptr, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, item_token, nullptr,  \
      num_items, out, part_o, part_ml, nsplit, split_keys, nh, nkv, ps, scale, stream, in
  if (hd == 128) return launch<128, true>(TK_FARGS);
  if (hd == 64) return launch<64, true>(TK_FARGS);
#undef TK_FARGS
  return -2;
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_attention_mfma)
TK_SLOTS(tk_attention_decode_fused)
