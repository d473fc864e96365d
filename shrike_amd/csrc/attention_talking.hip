// Attention whose softmax weights are mixed across heads before they meet the
// values ("talking heads" after the softmax), with a logarithmic distance bias
// and an optional sink, over the same paged key/value cache as attention.hip.
//
//   s_g(i, j) = q_g(i) . k(j) * scale - r1_g * ln(1 + r2_g * (i - j))
//   p_g(i, j) = exp(s_g) / (exp(sink) + sum_j exp(s_g))      (no sink: the plain softmax)
//   w_h(i, j) = sum_g talk[h, g] * p_g(i, j)
//   o_h(i)    = sum_j w_h(i, j) * v(j)        with the values of head h's own key/value head
//
// Mixing needs every head's normalised weight of a key, so a query token's heads
// stay together and the keys are walked twice: once for each head's maximum and
// denominator, once more to form the weights, mix them and sum the values.  Keys
// go by in tiles of 64 counted from the query's first key, so the order of every
// sum depends on the query's position alone: prompt portions and single tokens
// give the same bits.
//
// talking_stats_kernel  one workgroup per query token: max and denominator per head
// talking_apply_kernel  one workgroup per (query token, share of its key tiles):
//                       weights, mixing, values; shares are added in order by
//                       talking_merge_kernel where there is more than one
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kTalkThreads = 256;
constexpr int kTalkTile = 64;      // keys a tile
constexpr int kTalkMaxAcc = 16;    // output elements a thread: heads * v_dim <= 16 * 256

// scores of a tile into s[g * 64 + jj] (-inf where masked); q in LDS as float32 [heads, dim]
template <typename T>
__device__ __forceinline__ void tile_scores(float* s, const float* qs, int heads, int kv_heads, int head_dim,
                                            const int32_t* table, const T* k_pool, int page_size, int num_pages,
                                            int j0, int pos, float scale, const float* r1, const float* r2) {
  const int per = heads / kv_heads;
  const int slab = key_slab(head_dim);
  for (int item = threadIdx.x; item < heads * kTalkTile; item += kTalkThreads) {
    const int g = item / kTalkTile, jj = item % kTalkTile;
    const int j = j0 + jj;
    float sc = -INFINITY;
    if (j <= pos) {
      const int page = table[j / page_size];
      if (page >= 0 && page < num_pages) {
        const int kvh = g / per;
        const T* kr = k_pool + static_cast<size_t>(page * kv_heads + kvh) * page_size * head_dim +
                      static_cast<size_t>(j % page_size) * slab;
        const float* qg = qs + g * head_dim;
        float dot = 0.f;
        for (int e0 = 0; e0 < head_dim; e0 += slab) {
          for (int e = 0; e < slab; ++e) dot = fmaf(qg[e0 + e], to_float(kr[e]), dot);
          kr += static_cast<size_t>(page_size) * slab;
        }
        sc = dot * scale;
        if (r1) sc -= r1[g] * log1pf(r2[g] * static_cast<float>(pos - j));
      }
    }
    s[item] = sc;
  }
}

template <typename T>
__global__ void __launch_bounds__(kTalkThreads)
    talking_stats_kernel(const T* __restrict__ q, int q_stride, float* __restrict__ stats, int heads, int kv_heads,
                         int head_dim, const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq,
                         const int32_t* __restrict__ tables, int table_stride, const T* __restrict__ k_pool,
                         int page_size, int num_pages, int window, int chunk, float scale,
                         const float* __restrict__ r1, const float* __restrict__ r2, int has_sink, float sink) {
  extern __shared__ float lds[];
  float* qs = lds;                      // [heads, head_dim]
  float* s = qs + heads * head_dim;     // [heads, 64]
  float* m_run = s + heads * kTalkTile; // [heads]
  float* l_run = m_run + heads;         // [heads]
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int32_t* table = tables + static_cast<size_t>(token_seq[t]) * table_stride;
  const int lo = first_key(pos, window, chunk);
  for (int i = threadIdx.x; i < heads * head_dim; i += kTalkThreads)
    qs[i] = to_float(q[static_cast<size_t>(t) * q_stride + i]);
  for (int g = threadIdx.x; g < heads; g += kTalkThreads) {
    m_run[g] = has_sink ? sink : -INFINITY;
    l_run[g] = has_sink ? 1.f : 0.f;
  }
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  for (int j0 = lo; j0 <= pos; j0 += kTalkTile) {
    tile_scores<T>(s, qs, heads, kv_heads, head_dim, table, k_pool, page_size, num_pages, j0, pos, scale, r1, r2);
    __syncthreads();
    for (int g = wave; g < heads; g += kTalkThreads / kWave) {
      const float sc = s[g * kTalkTile + lane];
      const float m_old = m_run[g];
      const float m_new = fmaxf(m_old, wave_max(sc));
      const float sum = wave_sum(sc > -INFINITY ? expf(sc - m_new) : 0.f);
      if (lane == 0) {
        l_run[g] = l_run[g] * (m_old > -INFINITY ? expf(m_old - m_new) : 0.f) + sum;
        m_run[g] = m_new;
      }
    }
    __syncthreads();
  }
  for (int g = threadIdx.x; g < heads; g += kTalkThreads) {
    stats[(static_cast<size_t>(t) * heads + g) * 2] = m_run[g];
    stats[(static_cast<size_t>(t) * heads + g) * 2 + 1] = l_run[g];
  }
}

// OUT_T: the type of what this kernel writes: T for a token's whole result, float for a share
template <typename T>
__global__ void __launch_bounds__(kTalkThreads)
    talking_apply_kernel(const T* __restrict__ q, int q_stride, const float* __restrict__ stats,
                         const float* __restrict__ talk, T* __restrict__ out, float* __restrict__ shares,
                         int nshare, int heads, int kv_heads, int head_dim, int v_dim,
                         const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq,
                         const int32_t* __restrict__ tables, int table_stride, const T* __restrict__ k_pool,
                         const T* __restrict__ v_pool, int page_size, int num_pages, int window, int chunk,
                         float scale, const float* __restrict__ r1, const float* __restrict__ r2) {
  extern __shared__ float lds[];
  float* qs = lds;                       // [heads, head_dim]
  float* s = qs + heads * head_dim;      // [heads, 64] scores, then weights
  float* w = s + heads * kTalkTile;      // [heads, 64] mixed weights
  float* tk = w + heads * kTalkTile;     // [heads, heads]
  float* m_fin = tk + heads * heads;     // [heads]
  float* l_inv = m_fin + heads;          // [heads]
  __shared__ int32_t vrow[kTalkTile];    // page of each key of the tile, -1 if masked
  const int t = blockIdx.x, share = blockIdx.y;
  const int pos = positions[t];
  const int32_t* table = tables + static_cast<size_t>(token_seq[t]) * table_stride;
  const int lo = first_key(pos, window, chunk);
  const int per = heads / kv_heads;
  for (int i = threadIdx.x; i < heads * head_dim; i += kTalkThreads)
    qs[i] = to_float(q[static_cast<size_t>(t) * q_stride + i]);
  for (int i = threadIdx.x; i < heads * heads; i += kTalkThreads) tk[i] = talk ? talk[i] : (i / heads == i % heads);
  for (int g = threadIdx.x; g < heads; g += kTalkThreads) {
    m_fin[g] = stats[(static_cast<size_t>(t) * heads + g) * 2];
    l_inv[g] = 1.f / stats[(static_cast<size_t>(t) * heads + g) * 2 + 1];
  }
  float acc[kTalkMaxAcc];
#pragma unroll
  for (int a = 0; a < kTalkMaxAcc; ++a) acc[a] = 0.f;
  const int outs = heads * v_dim;
  const int tiles = (pos - lo) / kTalkTile + 1;
  const int per_share = (tiles + nshare - 1) / nshare;
  const int tile_lo = share * per_share, tile_hi = min(tiles, tile_lo + per_share);
  __syncthreads();
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int j0 = lo + tile * kTalkTile;
    tile_scores<T>(s, qs, heads, kv_heads, head_dim, table, k_pool, page_size, num_pages, j0, pos, scale, r1, r2);
    if (threadIdx.x < kTalkTile) {
      const int j = j0 + threadIdx.x;
      int page = -1;
      if (j <= pos) {
        page = table[j / page_size];
        if (page < 0 || page >= num_pages) page = -1;
      }
      vrow[threadIdx.x] = page;
    }
    __syncthreads();
    for (int item = threadIdx.x; item < heads * kTalkTile; item += kTalkThreads) {
      const int g = item / kTalkTile;
      const float sc = s[item];
      s[item] = sc > -INFINITY ? expf(sc - m_fin[g]) * l_inv[g] : 0.f;
    }
    __syncthreads();
    for (int item = threadIdx.x; item < heads * kTalkTile; item += kTalkThreads) {
      const int h = item / kTalkTile, jj = item % kTalkTile;
      float mixed = 0.f;
      for (int g = 0; g < heads; ++g) mixed = fmaf(tk[h * heads + g], s[g * kTalkTile + jj], mixed);
      w[item] = mixed;
    }
    __syncthreads();
    const int count = min(kTalkTile, pos - j0 + 1);
#pragma unroll
    for (int a = 0; a < kTalkMaxAcc; ++a) {
      const int o = threadIdx.x + a * kTalkThreads;
      if (o >= outs) break;
      const int h = o / v_dim, d = o % v_dim;
      const int kvh = h / per;
      float sum = acc[a];
      for (int jj = 0; jj < count; ++jj) {
        const int page = vrow[jj];
        if (page < 0) continue;
        // values are stored [page][kv head][v_dim][page_size]
        const size_t at = (static_cast<size_t>(page * kv_heads + kvh) * v_dim + d) * page_size + (j0 + jj) % page_size;
        sum = fmaf(w[h * kTalkTile + jj], to_float(v_pool[at]), sum);
      }
      acc[a] = sum;
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < kTalkMaxAcc; ++a) {
    const int o = threadIdx.x + a * kTalkThreads;
    if (o >= outs) break;
    if (nshare == 1) out[static_cast<size_t>(t) * outs + o] = from_float<T>(acc[a]);
    else shares[(static_cast<size_t>(t) * nshare + share) * outs + o] = acc[a];
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
    talking_merge_kernel(const float* __restrict__ shares, int nshare, T* __restrict__ out, int outs) {
  const int t = blockIdx.y;
  const int o = blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= outs) return;
  float sum = 0.f;
  for (int z = 0; z < nshare; ++z) sum += shares[(static_cast<size_t>(t) * nshare + z) * outs + o];
  out[static_cast<size_t>(t) * outs + o] = from_float<T>(sum);
}

}  // namespace shk

using namespace shk;

extern "C" long long shk_attention_talking_scratch_floats(int n, int heads, int v_dim, int nshare) {
  return static_cast<long long>(n) * heads * 2 + (nshare > 1 ? static_cast<long long>(n) * nshare * heads * v_dim : 0);
}

extern "C" int shk_attention_talking(const void* q, int q_stride, void* out, int dtype, int n, int heads, int kv_heads,
                                     int head_dim, int v_dim, const int32_t* positions, const int32_t* token_seq,
                                     const int32_t* tables, int table_stride, const void* k_pool, const void* v_pool,
                                     int page_size, int num_pages, int window, int chunk, float scale,
                                     const float* r1, const float* r2, const float* talk, int has_sink, float sink,
                                     float* scratch, int nshare, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "attention_talking: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
              "attention_talking: heads=%d must be a positive multiple of kv_heads=%d", heads, kv_heads);
  SHK_REQUIRE(head_dim > 0 && head_dim <= 256 && v_dim > 0 && v_dim <= 256,
              "attention_talking: head_dim %d or v_dim %d is outside 1..256", head_dim, v_dim);
  SHK_REQUIRE(heads * v_dim <= kTalkMaxAcc * kTalkThreads, "attention_talking: %d heads of %d values are more than %d",
              heads, v_dim, kTalkMaxAcc * kTalkThreads);
  SHK_REQUIRE(q_stride >= heads * head_dim, "attention_talking: q_stride %d < heads*head_dim %d", q_stride,
              heads * head_dim);
  SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0 && nshare >= 1 && nshare <= 64,
              "attention_talking: bad cache sizes or shares");
  SHK_REQUIRE(static_cast<int64_t>(num_pages) * kv_heads * page_size < (1LL << 31),
              "attention_talking: cache pool has too many rows for 32-bit row indices");
  SHK_REQUIRE((r1 == nullptr) == (r2 == nullptr), "attention_talking: the distance bias needs both of its numbers");
  const size_t lds = (static_cast<size_t>(heads) * head_dim + 2 * heads * kTalkTile + heads * heads + 2 * heads) *
                     sizeof(float);
  SHK_REQUIRE(lds <= 60000, "attention_talking: %d heads of %d elements need more LDS than a workgroup has", heads,
              head_dim);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "attention_talking: at most 65535 tokens a call, got %d", n);
  SHK_REQUIRE(q && out && positions && token_seq && tables && k_pool && v_pool && scratch,
              "attention_talking: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // scratch: [n, heads, 2] maxima and denominators, then [n, nshare, heads * v_dim] shares
  float* stats = scratch;
  float* shares = scratch + static_cast<size_t>(n) * heads * 2;
  const int outs = heads * v_dim;
#define SHK_GO(T)                                                                                                      \
  talking_stats_kernel<T><<<n, kTalkThreads, lds, s>>>(static_cast<const T*>(q), q_stride, stats, heads, kv_heads,     \
                                                       head_dim, positions, token_seq, tables, table_stride,           \
                                                       static_cast<const T*>(k_pool), page_size, num_pages, window,    \
                                                       chunk, scale, r1, r2, has_sink, sink);                          \
  talking_apply_kernel<T><<<dim3(n, nshare), kTalkThreads, lds, s>>>(                                                  \
      static_cast<const T*>(q), q_stride, stats, talk, static_cast<T*>(out), shares, nshare, heads, kv_heads,          \
      head_dim, v_dim, positions, token_seq, tables, table_stride, static_cast<const T*>(k_pool),                      \
      static_cast<const T*>(v_pool), page_size, num_pages, window, chunk, scale, r1, r2);                              \
  if (nshare > 1)                                                                                                      \
    talking_merge_kernel<T><<<dim3((outs + 255) / 256, n), 256, 0, s>>>(shares, nshare, static_cast<T*>(out), outs)
  if (dtype == kF32) {
    SHK_GO(float);
  } else {
    SHK_GO(bf16);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("attention_talking");
  return 0;
}
