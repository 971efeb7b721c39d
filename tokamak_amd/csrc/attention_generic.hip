// Paged causal attention for any head size (multiple of 16, up to 512), any
// number of heads and groups, any page size that is a multiple of 8, in float32
// or bf16 storage with float32 arithmetic throughout.  It serves prompt portions
// and decode tokens alike: every query token walks its own request's block table
// from the first visible position to its own position.
//
// A block of kWaves waves takes up to QT queries that walk the same keys and values and
// share every one they load: consecutive tokens of one request at one query head (a piece
// of a 16-token tile of a prompt portion), or the query heads of one kv head's group at one
// token (a token that runs alone, a decode token).  Keys are taken 64 at a time, one key per lane;
// the round that starts at key 64 i goes to wave i % kWaves, which keeps a running maximum,
// a running sum and an output of its own in float32 for every query (online softmax); at
// the end the waves' results are merged in wave order.  Which wave takes which keys, and
// the order of every sum, follow from the query's own position alone: the result does not
// depend on how the request was cut into steps, on what else is in the batch, or on
// whether the token ran alone or in a tile (equal bits).
//
// Cache pages: K [nkv][hd/8][ps][8], V [nkv][hd/16][ps/4][16][4] (see elementwise.hip).
#include "common.h"
#include "slots.h"

using namespace tk;

constexpr int kMaxHd = 512;
constexpr int kWaves = 8;  // waves of a block; kWaves * 64 threads cover every dimension of the widest head
static_assert(kWaves * kWave >= kMaxHd, "the merge gives every dimension a thread");
constexpr int kTileTokens = 16;  // tokens of a tile in the work list
constexpr int kQueries = 8;      // queries a block of the tile kernel takes

// four consecutive elements (four keys of one dimension in a V page) as one load
__device__ __forceinline__ void load_four(const float* p, float (&v)[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load_four(const bf16_t* p, float (&v)[4]) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
}

// eight consecutive elements (a key's piece of a K page)
__device__ __forceinline__ void load_eight(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load_eight(const bf16_t* p, float (&v)[8]) {
  const uint4 x = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// pieces of a key (8 dimensions each) asked for together: many for a query alone, whose walk
// is a chain of memory round trips; few where eight queries share the key and the
// multiply-adds fill the time (and the registers)
template <int QT> constexpr int key_pieces() { return QT == 1 ? 8 : QT <= 4 ? 4 : 2; }

struct GenericItems {
  const int* single;      // token rows that run alone (null: every token of the step does)
  const int* tile_first;  // first token row of each tile
  const int* tile_count;  // tokens in it (1..kTileTokens), consecutive positions of one request
};

// QT: queries of a block; HEADS: they are heads of one group at one token (blockIdx.y is the kv
// head, blockIdx.z the piece of the group), else tokens of one tile at one head (blockIdx.y).
// SLOTS: dimensions a lane owns (hd <= 64 * SLOTS).
template <typename T, int QT, bool HEADS, int SLOTS>
__global__ __launch_bounds__(kWaves * kWave) void paged_attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, GenericItems items, T* __restrict__ out, int nh, int nkv,
    int hd, int ps, int max_pages, float scale, int window) {
  __shared__ __attribute__((aligned(16))) float q_s[QT][kMaxHd];
  __shared__ __attribute__((aligned(16))) float p_s[kWaves][kWave][QT];
  __shared__ long base_s[kWaves][kWave];  // where a key's values lie (a quad's, for tokens that run alone), or -1
  __shared__ float m_s[kWaves], l_s[kWaves];
  __shared__ float acc_s[kWaves][kMaxHd];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  const int group = nh / nkv;
  int n0, cnt, head0, kvh;
  if (HEADS) {
    n0 = items.single ? items.single[blockIdx.x] : (int)blockIdx.x;
    kvh = blockIdx.y;
    head0 = kvh * group + blockIdx.z * QT;
    cnt = min(QT, group - (int)blockIdx.z * QT);
  } else {
    n0 = items.tile_first[blockIdx.x] + blockIdx.z * QT;
    cnt = min(QT, items.tile_count[blockIdx.x] - (int)blockIdx.z * QT);
    head0 = blockIdx.y;
    kvh = head0 / group;
  }
  if (cnt <= 0) return;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  // query t: its row of q and out, its position and the first key it sees
  size_t row[QT];
  int pos[QT], first[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int u = min(t, cnt - 1);
    row[t] = HEADS ? (size_t)n0 * nh + head0 + u : (size_t)(n0 + u) * nh + head0;
    pos[t] = positions[HEADS ? n0 : n0 + u];
    first[t] = (window > 0 && pos[t] - window + 1 > 0) ? pos[t] - window + 1 : 0;
  }
  const int lo = first[0], hi = pos[QT - 1];  // positions ascend within a tile
  const size_t page_elems = (size_t)nkv * hd * ps;
  const size_t head_off = (size_t)kvh * hd * ps;

#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const T* qrow = q + row[t] * hd;
    for (int d = tid; d < hd; d += kWaves * kWave) q_s[t][d] = Elem<T>::load(qrow + d) * scale;
  }
  __syncthreads();

  float m[QT], l[QT], acc[SLOTS][QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) acc[i][t] = 0.f;
  }

  // this wave's rounds: those whose index is wave modulo kWaves, from the one that holds lo
  const int round0 = lo / kWave;
  for (int rd = round0 + (wave - round0 % kWaves + kWaves) % kWaves; rd * kWave <= hi; rd += kWaves) {
    const int c0 = rd * kWave, c = c0 + lane;
    const bool loaded = c >= lo && c <= hi;
    float dot[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) dot[t] = 0.f;
    // Tokens that run alone (decode) are bound by round trips to memory, not by arithmetic: they
    // ask for eight pieces of a key at once and for the values of four keys in one piece (four
    // such pieces at once).  Tiles of a prompt portion, eight queries to a key, are bound by
    // their multiply-adds and keep the plain loops.  The order of every sum is the same.
    constexpr bool BATCHED = HEADS;
    long vbase = -1;
    if (BATCHED && (lane & 3) == 0 && c <= hi && c + 3 >= lo) {
      // the values of four consecutive keys of a dimension are one piece of a page
      const int page = table[c / ps];
      vbase = (long)((size_t)page * page_elems + head_off + (size_t)((c % ps) >> 2) * 64);
    }
    if (loaded) {
      const int page = table[c / ps];
      const int off = c % ps;
      const T* kp = k_cache + (size_t)page * page_elems + head_off;
      if constexpr (BATCHED) {
        constexpr int kKeyPieces = key_pieces<QT>();
        for (int j0 = 0; j0 < hd / 8; j0 += kKeyPieces) {
          float k8[kKeyPieces][8];
#pragma unroll
          for (int u = 0; u < kKeyPieces; ++u) {
            const int j = min(j0 + u, hd / 8 - 1);      // (a piece past the head is loaded again and not used)
            load_eight(kp + ((size_t)j * ps + off) * 8, k8[u]);
          }
#pragma unroll
          for (int u = 0; u < kKeyPieces; ++u) {
            if (j0 + u < hd / 8) {
#pragma unroll
              for (int t = 0; t < QT; ++t) {
#pragma unroll
                for (int e = 0; e < 8; ++e) dot[t] = fmaf(q_s[t][(j0 + u) * 8 + e], k8[u][e], dot[t]);
              }
            }
          }
        }
      } else {
        for (int j = 0; j < hd / 8; ++j) {
          float k8[8];
          load_eight(kp + ((size_t)j * ps + off) * 8, k8);
#pragma unroll
          for (int t = 0; t < QT; ++t) {
#pragma unroll
            for (int e = 0; e < 8; ++e) dot[t] = fmaf(q_s[t][j * 8 + e], k8[e], dot[t]);
          }
        }
        vbase = (long)((size_t)page * page_elems + head_off + (size_t)(off >> 2) * 64 + (off & 3));
      }
    }
    float alpha[QT], p[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      // a round that holds none of query t's keys leaves its sums as they are
      const bool takes = c0 <= pos[t] && c0 + kWave - 1 >= first[t];
      alpha[t] = 1.f;
      p[t] = 0.f;
      if (takes) {
        const bool valid = c >= first[t] && c <= pos[t];
        const float sc = valid ? dot[t] : -INFINITY;
        const float m_new = fmaxf(m[t], wave_max(sc));
        p[t] = valid ? expf(sc - m_new) : 0.f;
        alpha[t] = expf(m[t] - m_new);  // m = -inf on the first round: alpha = 0
        l[t] = l[t] * alpha[t] + wave_sum(p[t]);
        m[t] = m_new;
      }
    }
    wave_lds_sync();   // the wave has read the probabilities of the 64 keys before
#pragma unroll
    for (int t = 0; t < QT; ++t) p_s[wave][lane][t] = p[t];
    if (!BATCHED) base_s[wave][lane] = vbase;
    else if ((lane & 3) == 0) base_s[wave][lane >> 2] = vbase;
    wave_lds_sync();
    const int count = (hi - c0 + 1 < kWave) ? hi - c0 + 1 : kWave;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      const int d = lane + i * kWave;
      if (d < hd) {
        const size_t v_dim_off = (size_t)(d >> 4) * (ps >> 2) * 64 + (d & 15) * 4;
        float a[QT];
#pragma unroll
        for (int t = 0; t < QT; ++t) a[t] = acc[i][t] * alpha[t];
        if constexpr (BATCHED) {
          // four keys a load (16 bytes of float32) and four such loads asked for together, added
          // key by key in ascending order: the same sums as one key at a time.  A key out of
          // range adds a probability times 0.
          for (int quad0 = 0; quad0 * 4 < count; quad0 += 4) {
            float v4[4][4];
            bool there[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const long b = base_s[wave][quad0 + u];
              there[u] = (quad0 + u) * 4 < count && b >= 0;
              load_four(v_cache + (there[u] ? b : 0) + v_dim_off, v4[u]);   // (absent: the cache's first page, not used)
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int key = (quad0 + u) * 4 + e;
                const bool in = there[u] && c0 + key >= lo && c0 + key <= hi;
                const float v = in ? v4[u][e] : 0.f;   // (the probabilities of such a key are finite: 0 * p adds nothing)
#pragma unroll
                for (int t = 0; t < QT; ++t) a[t] = fmaf(p_s[wave][key][t], v, a[t]);
              }
            }
          }
        } else {
          for (int key = 0; key < count; ++key) {
            const long b = base_s[wave][key];
            if (b >= 0) {
              const float v = Elem<T>::load(v_cache + b + v_dim_off);
#pragma unroll
              for (int t = 0; t < QT; ++t) a[t] = fmaf(p_s[wave][key][t], v, a[t]);
            }
          }
        }
#pragma unroll
        for (int t = 0; t < QT; ++t) acc[i][t] = a[t];
      }
    }
  }
  // merge, one query after the other: a wave that had no round of the query's brings
  // m = -inf, l = 0 and zeros, which weigh nothing
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    if (t >= cnt) break;
    __syncthreads();   // the last query's merge has read the waves' results
    if (lane == 0) {
      m_s[wave] = m[t];
      l_s[wave] = l[t];
    }
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      const int d = lane + i * kWave;
      if (d < hd) acc_s[wave][d] = acc[i][t];
    }
    __syncthreads();
    if (tid < hd) {
      float top = m_s[0];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) top = fmaxf(top, m_s[w]);
      float sum = 0.f, o = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const float e = expf(m_s[w] - top);
        sum = fmaf(l_s[w], e, sum);
        o = fmaf(acc_s[w][tid], e, o);
      }
      Elem<T>::store(out + row[t] * hd + tid, o / sum);
    }
  }
}

template <typename T, int SLOTS>
static void launch_generic(const T* q, const T* k_cache, const T* v_cache, const int* block_tables,
                           const int* positions, const int* req_of_token, GenericItems items,
                           int num_single, int num_tiles, T* out, int nh, int nkv, int hd, int ps,
                           int max_pages, float scale, int window, int share_heads, hipStream_t stream) {
  const int group = nh / nkv;
#define TK_ALONE(QT_)                                                                               \
  paged_attention_generic_kernel<T, QT_, true, SLOTS>                                               \
      <<<dim3(num_single, nkv, (group + QT_ - 1) / QT_), kWaves * kWave, 0, stream>>>(              \
          q, k_cache, v_cache, block_tables, positions, req_of_token, items, out, nh, nkv, hd, ps,  \
          max_pages, scale, window)
  if (num_single > 0) {
    // the heads of a group share a block if that still gives every CU one (the result is the
    // same either way): at batch 64 of an 8B-shaped layer a third faster, at batch 8 slower
    const int qt = group <= 4 ? 4 : kQueries;
    const bool shared = group > 1 && (share_heads < 0 ? (long)num_single * nkv * ((group + qt - 1) / qt) >= 256
                                                      : share_heads > 0);
    if (!shared) TK_ALONE(1);
    else if (qt == 4) TK_ALONE(4);
    else TK_ALONE(kQueries);
  }
#undef TK_ALONE
  if (num_tiles > 0)
    paged_attention_generic_kernel<T, kQueries, false, SLOTS>
        <<<dim3(num_tiles, nh, kTileTokens / kQueries), kWaves * kWave, 0, stream>>>(
            q, k_cache, v_cache, block_tables, positions, req_of_token, items, out, nh, nkv, hd, ps,
            max_pages, scale, window);
}

// tile_first / tile_count (num_tiles of them) and single (num_single token rows): the step's work
// lists, which together name every token once.  With tile_first null every one of the N tokens
// runs alone.  share_heads: whether the query heads of a group share a block for the tokens
// that run alone (1), or not (0), or as fills the GPU (-1); the result is the same.
TK_API int tk_paged_attention_generic(int dtype, const void* q, const void* k_cache,
                                      const void* v_cache, const int* block_tables,
                                      const int* positions, const int* req_of_token, void* out,
                                      int N, int nh, int nkv, int hd, int ps, int max_pages,
                                      float scale, int window, const int* tile_first,
                                      const int* tile_count, int num_tiles, const int* single,
                                      int num_single, int share_heads, hipStream_t stream) {
  if (N <= 0) return 0;
  if (hd > kMaxHd || hd % 16 != 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || ps % 4 != 0 || nh > 65535) return -1;
  if (tile_first == nullptr) {
    num_tiles = 0;
    single = nullptr;
    num_single = N;
  } else if (num_tiles < 0 || num_single < 0 || tile_count == nullptr || (num_single > 0 && single == nullptr)) {
    return -1;
  }
  const GenericItems items{single, tile_first, tile_count};
#define TK_GENERIC(T_, SLOTS_)                                                                      \
  launch_generic<T_, SLOTS_>((const T_*)q, (const T_*)k_cache, (const T_*)v_cache, block_tables,    \
                             positions, req_of_token, items, num_single, num_tiles, (T_*)out, nh,   \
                             nkv, hd, ps, max_pages, scale, window, share_heads, stream)
  if (dtype == 0) {
    if (hd <= 128) TK_GENERIC(float, 2);
    else if (hd <= 256) TK_GENERIC(float, 4);
    else TK_GENERIC(float, 8);
  } else {
    if (hd <= 128) TK_GENERIC(bf16_t, 2);
    else if (hd <= 256) TK_GENERIC(bf16_t, 4);
    else TK_GENERIC(bf16_t, 8);
  }
#undef TK_GENERIC
  return launch_status();
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_paged_attention_generic)
