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

// ---------------------------------------------------------------- bfloat16 on the matrix units
//
// Mixing the weights of a key across heads and then summing the values is the same as summing
// the values with every head's own weights and mixing the sums:
//
//   o_h = sum_j (sum_g talk[h, g] p_g(j)) v_c(j) = sum_g talk[h, g] U[g, c],   c = h's key/value head,
//   U[g, c] = sum_j p_g(j) v_c(j)
//
// so each softmax head g runs as ordinary attention with a running maximum and sum, only
// that its weights meet the values of every key/value head, and a small kernel mixes the
// results.  One pass over the keys, no weights in memory.
//
// A wavefront serves 16 query rows that share a sequence and a key/value head for the keys:
// one single token's heads of a key/value head (talking_mfma_kernel, operands straight from
// memory), or 16 consecutive tokens of a prompt's portion for one head (talking_tiles_lds_kernel,
// tile_seq / tile_q0 list the tiles; a workgroup's four heads share what it stages in LDS).  Keys
// go by in chunks of 32, aligned to 32 in the sequence:
//
//   S^T = K Q^T   [32 keys x 16 rows]  two v_mfma_f32_16x16x32_bf16 per 32 elements of a head;
//                 A = keys straight from their slabs (a lane's 8 elements are 16 bytes), and
//                 the keys are assigned to A's rows so that a lane ends up with the scores of
//                 8 consecutive keys of its query row: P^T is then already a B operand
//   softmax       base 2, float32, running maximum and sum per row (lanes i, i+16, i+32, i+48)
//   O^T += V^T P^T  [16 values x 16 rows] per block of 16 value elements and key/value head;
//                 A = 8 consecutive keys of one value element, 16 bytes of the transposed pool
//
// NB: blocks of 16 value elements that a pass holds (value heads of a pass x blocks a head);
// KS: 32-element steps of a head.  Value heads beyond a pass are other workgroups (grid z),
// which form the scores again.
typedef __bf16 tbf16x8 __attribute__((ext_vector_type(8)));
typedef float tf32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float rows_max(float v) {  // over lanes i, i + 16, i + 32, i + 48
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  return fmaxf(v, __shfl_xor(v, 32, kWave));
}
__device__ __forceinline__ float rows_sum(float v) {
  v += __shfl_xor(v, 16, kWave);
  return v + __shfl_xor(v, 32, kWave);
}

template <int KS, int NB>
__global__ void __launch_bounds__(256)
    talking_mfma_kernel(const bf16* __restrict__ q, int q_stride, float* __restrict__ u_out, int heads, int kv_heads,
                        int head_dim, int v_dim, const int32_t* __restrict__ positions,
                        const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables, int table_stride,
                        const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool, int page_size, int num_pages,
                        int window, int chunk, float scale_l2, const float* __restrict__ r1,
                        const float* __restrict__ r2, int has_sink, float sink_l2, int nsplit,
                        float* __restrict__ partial, int vh_pass) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int group = heads / kv_heads;
  const int unit = blockIdx.y * 4 + wave;
  const int vb = (v_dim + 15) / 16;  // blocks of 16 value elements a head
  const int cv0 = blockIdx.z * vh_pass;
  const int cvn = min(vh_pass, kv_heads - cv0);
  // the lane's query row
  const int subs = (group + 15) / 16;
  if (unit >= kv_heads * subs) return;
  const int t = blockIdx.x / nsplit;
  const int seq = token_seq[t];
  const int ck = unit / subs;
  const int within = (unit % subs) * 16 + i;
  const bool valid = within < group;
  const int head = ck * group + (valid ? within : 0);
  const int pos = valid ? positions[t] : -1;
  const int lo = valid ? first_key(pos, window, chunk) : (1 << 30);
  int pos_max = pos, lo_min = lo;
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) {
    pos_max = max(pos_max, __shfl_xor(pos_max, off, kWave));
    lo_min = min(lo_min, __shfl_xor(lo_min, off, kWave));
  }
  if (pos_max < 0) return;  // (no row of the tile is a token)
  const int32_t* table = tables + static_cast<size_t>(seq) * table_stride;
  const float bias1 = r1 ? r1[head] : 0.f, bias2 = r1 ? r2[head] : 0.f;
  // the queries: B operands, elements ks * 32 + kg * 8 .. + 8 of row i
  tbf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 v = make_uint4(0, 0, 0, 0);
    const int e = ks * 32 + kg * 8;
    if (valid && e < head_dim)
      v = *reinterpret_cast<const uint4*>(q + static_cast<size_t>(t) * q_stride + head * head_dim + e);
    qf[ks] = __builtin_bit_cast(tbf16x8, v);
  }
  tf32x4 o[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) o[b] = tf32x4{0.f, 0.f, 0.f, 0.f};
  // single tokens with many keys: share `share` of nsplit takes a run of the chunks (the sink is the first one's)
  const int share = blockIdx.x % nsplit;
  const int chunk_lo = lo_min / 32, chunk_hi = pos_max / 32;
  const int per_share = (chunk_hi - chunk_lo + nsplit) / nsplit;
  const int j_begin = (chunk_lo + share * per_share) * 32;
  const int j_end = min(pos_max, (chunk_lo + (share + 1) * per_share) * 32 - 1);
  float m_run = has_sink && share == 0 ? sink_l2 : -INFINITY;
  float l_run = has_sink && share == 0 ? 1.f : 0.f;
  const int slab = key_slab(head_dim);
  const size_t k_head = static_cast<size_t>(page_size) * head_dim;  // elements of a page's head
  const size_t v_head = static_cast<size_t>(page_size) * v_dim;
  // the pages of a chunk's keys: this lane's two keys as A rows of the scores, and its 8 keys of the values
  auto pages_of = [&](int j0, int (&kp)[2], int& vp) {
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int jk = j0 + 8 * (i / 4) + 4 * t2 + i % 4;
      kp[t2] = -1;
      if (jk >= lo_min && jk <= pos_max) {
        const int page = table[jk / page_size];
        kp[t2] = page >= 0 && page < num_pages ? page : -1;
      }
    }
    const int jg = j0 + 8 * kg;
    vp = -1;
    if (jg + 7 >= lo_min && jg <= pos_max) {
      const int page = table[jg / page_size];
      vp = page >= 0 && page < num_pages ? page : -1;
    }
  };
  int kpage[2], vpage;
  pages_of(j_begin, kpage, vpage);
  for (int j0 = j_begin; j0 <= j_end; j0 += 32) {
    // All of the chunk's operands are asked for before anything is multiplied, and the next chunk's
    // pages are looked up meanwhile: a chunk waits for memory once.
    // keys: A row m of product t2 is the key j0 + 8 (m / 4) + 4 t2 + m % 4
    uint4 kf[2][KS];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int jk = j0 + 8 * (i / 4) + 4 * t2 + i % 4;
      const bf16* kr = k_pool + (static_cast<size_t>(max(kpage[t2], 0)) * kv_heads + ck) * k_head;
      const int slot = jk % page_size;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        kf[t2][ks] = make_uint4(0, 0, 0, 0);
        const int e = ks * 32 + kg * 8;
        if (kpage[t2] >= 0 && e < head_dim)
          kf[t2][ks] = *reinterpret_cast<const uint4*>(kr + (static_cast<size_t>(e / slab) * page_size + slot) * slab + e % slab);
      }
    }
    // values: A row i of block b is value element (b % vb) * 16 + i of key/value head cv0 + b / vb, keys jg .. + 8
    const int jg = j0 + 8 * kg;
    union VFrag {
      uint4 u;
      uint16_t h[8];
    } vf[NB];
    {
      const int slot = jg % page_size;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const int cvl = b / vb, d = (b % vb) * 16 + i;
        vf[b].u = make_uint4(0, 0, 0, 0);
        if (cvl < cvn && vpage >= 0 && d < v_dim)
          vf[b].u = *reinterpret_cast<const uint4*>(v_pool + (static_cast<size_t>(vpage) * kv_heads + cv0 + cvl) * v_head +
                                                    static_cast<size_t>(d) * page_size + slot);
      }
    }
    const int vpage_now = vpage;
    if (j0 + 32 <= j_end) pages_of(j0 + 32, kpage, vpage);
    tf32x4 s[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      s[t2] = tf32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[t2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tbf16x8, kf[t2][ks]), qf[ks], s[t2], 0, 0, 0);
    }
    // this lane: the scores of keys jg + 4 t2 + r for its row i (8 aligned keys share a page)
    float x[8];
    float mx = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = jg + 4 * t2 + r;
        float v = s[t2][r] * scale_l2;
        if (r1) v -= bias1 * __log2f(1.f + bias2 * static_cast<float>(pos - j));
        const bool seen = vpage_now >= 0 && j >= lo && j <= pos;
        v = seen ? v : -INFINITY;
        x[4 * t2 + r] = v;
        mx = fmaxf(mx, v);
      }
    const float m_new = fmaxf(m_run, rows_max(mx));
    const float alpha = m_run > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_new) : 0.f;
    float psum = 0.f;
    union {
      uint4 u;
      uint16_t h[8];
    } pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = x[e] > -INFINITY ? __builtin_amdgcn_exp2f(x[e] - m_new) : 0.f;
      psum += p;
      const bf16 pb = from_float<bf16>(p);
      pf.h[e] = __builtin_bit_cast(uint16_t, pb);
    }
    l_run = l_run * alpha + rows_sum(psum);
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[b][r] *= alpha;
    }
    const bool ragged = jg < lo_min || jg + 7 > pos_max;  // keys that no row of the tile reads may hold anything
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b / vb < cvn) {
        if (ragged) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (jg + e < lo_min || jg + e > pos_max) vf[b].h[e] = 0;
        }
        o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tbf16x8, vf[b].u),
                                                       __builtin_bit_cast(tbf16x8, pf.u), o[b], 0, 0, 0);
      }
    }
  }
  if (!valid) return;
  // this lane holds value elements (b % vb) * 16 + 4 kg + r of its row
  float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  float* dst = u_out + (static_cast<size_t>(t) * heads + head) * kv_heads * v_dim;
  if (nsplit > 1) {  // the share's sums as they stand, then its maximum and denominator
    const int gv = kv_heads * v_dim;
    dst = partial + ((static_cast<size_t>(t) * heads + head) * nsplit + share) * (gv + 2);
    inv = 1.f;
    if (kg == 0 && blockIdx.z == 0) {
      dst[gv] = m_run;
      dst[gv + 1] = l_run;
    }
  }
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int cvl = b / vb;
    if (cvl >= cvn) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = (b % vb) * 16 + 4 * kg + r;
      if (d < v_dim) dst[static_cast<size_t>(cv0 + cvl) * v_dim + d] = o[b][r] * inv;
    }
  }
}

// Prompt portions with a chunk staged once for four heads: a workgroup serves one tile of 16
// queries, four query heads of one key/value head (a wavefront each) and a pass of key/value heads
// for the values.  A chunk's 32 keys and the 32 values of every value element of the pass's
// key/value heads are fetched once by the workgroup (the next chunk's pieces are on their way into
// registers while this one is multiplied), laid into LDS (key rows 16 bytes longer than a head,
// value rows of 32 keys 80 bytes apart: an operand's sixteen 16-byte reads meet every bank once),
// and every wavefront takes its operands from there.  NB = key/value heads of a pass x blocks of 16
// values, at most 16: with 64 registers of sums two workgroups share a compute unit.
template <int KS, int NB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
    talking_tiles_lds_kernel(const bf16* __restrict__ q, int q_stride, float* __restrict__ u_out, int heads, int kv_heads,
                             int head_dim, int v_dim, const int32_t* __restrict__ positions,
                             const int32_t* __restrict__ tables, int table_stride, const bf16* __restrict__ k_pool,
                             const bf16* __restrict__ v_pool, int page_size, int num_pages, int window, int chunk,
                             float scale_l2, const float* __restrict__ r1, const float* __restrict__ r2, int has_sink,
                             float sink_l2, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ tile_seq,
                             const int32_t* __restrict__ tile_q0, int vh_pass) {
  constexpr int KLD = KS * 32 + 8;      // elements between key rows in LDS
  constexpr int VLD = 40;               // elements between value rows (32 keys and 16 bytes)
  constexpr int KPT = KS >= 2 ? KS / 2 : 1;  // 16-byte pieces of keys a thread stages: 32 keys x 4 KS pieces / 256
  constexpr int VPT = NB >= 4 ? NB / 4 : 1;  // of values: NB x 16 rows x 4 pieces / 256
  extern __shared__ __attribute__((aligned(16))) uint16_t lds_t[];
  uint16_t* sk = lds_t;                      // [32][KLD]
  uint16_t* sv = lds_t + 32 * KLD;           // [NB * 16][VLD]
  __shared__ int group_ok[4];                // whether the chunk's four groups of 8 keys have a page
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int group = heads / kv_heads;
  const int quads = (group + 3) / 4;
  const int ck = blockIdx.y / quads;
  const int within = (blockIdx.y % quads) * 4 + wave;
  const bool has_head = within < group;
  const int head = ck * group + (has_head ? within : 0);
  const int vb = (v_dim + 15) / 16;
  const int cv0 = blockIdx.z * vh_pass;
  const int cvn = min(vh_pass, kv_heads - cv0);
  const int seq = tile_seq[blockIdx.x];
  const int t = cu_q[seq] + tile_q0[blockIdx.x] + i;
  const bool valid = t < cu_q[seq + 1];
  const int pos = valid ? positions[t] : -1;
  const int lo = valid ? first_key(pos, window, chunk) : (1 << 30);
  int pos_max = pos, lo_min = lo;
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) {
    pos_max = max(pos_max, __shfl_xor(pos_max, off, kWave));
    lo_min = min(lo_min, __shfl_xor(lo_min, off, kWave));
  }
  if (pos_max < 0) return;  // (the same for all four wavefronts: they serve the same tokens)
  const int32_t* table = tables + static_cast<size_t>(seq) * table_stride;
  const float bias1 = r1 ? r1[head] : 0.f, bias2 = r1 ? r2[head] : 0.f;
  tbf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 v = make_uint4(0, 0, 0, 0);
    const int e = ks * 32 + kg * 8;
    if (valid && has_head && e < head_dim)
      v = *reinterpret_cast<const uint4*>(q + static_cast<size_t>(t) * q_stride + head * head_dim + e);
    qf[ks] = __builtin_bit_cast(tbf16x8, v);
  }
  tf32x4 o[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) o[b] = tf32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = has_sink ? sink_l2 : -INFINITY;
  float l_run = has_sink ? 1.f : 0.f;
  const int slab = key_slab(head_dim);
  const size_t k_head = static_cast<size_t>(page_size) * head_dim;
  const size_t v_head = static_cast<size_t>(page_size) * v_dim;
  const int kpieces = head_dim / 8;         // 16-byte pieces of a key
  const int vrows = cvn * v_dim;            // value rows of a chunk: (key/value head of the pass, element)
  union Piece {
    uint4 u;
    uint16_t h[8];
  };
  Piece rk[KPT], rv[VPT];
  int rv_ok[VPT];
  auto page_at = [&](int j) {
    const int page = table[j / page_size];
    return page >= 0 && page < num_pages ? page : -1;
  };
  auto fetch = [&](int j0) {
#pragma unroll
    for (int r = 0; r < KPT; ++r) {
      const int p = tid + 256 * r;
      const int key = p / kpieces, e = (p % kpieces) * 8;
      const int j = j0 + key;
      rk[r].u = make_uint4(0, 0, 0, 0);
      if (key < 32 && j >= lo_min && j <= pos_max) {
        const int page = page_at(j);
        if (page >= 0)
          rk[r].u = *reinterpret_cast<const uint4*>(k_pool + (static_cast<size_t>(page) * kv_heads + ck) * k_head +
                                                    (static_cast<size_t>(e / slab) * page_size + j % page_size) * slab +
                                                    e % slab);
      }
    }
#pragma unroll
    for (int r = 0; r < VPT; ++r) {
      const int p = tid + 256 * r;
      const int row = p / 4, jg = j0 + 8 * (p % 4);  // row = key/value head of the pass * v_dim + element
      rv[r].u = make_uint4(0, 0, 0, 0);
      rv_ok[r] = 0;
      if (row < vrows && jg + 7 >= lo_min && jg <= pos_max) {
        const int page = page_at(jg);
        if (page >= 0) {
          rv_ok[r] = 1;
          rv[r].u = *reinterpret_cast<const uint4*>(v_pool + (static_cast<size_t>(page) * kv_heads + cv0 + row / v_dim) * v_head +
                                                    static_cast<size_t>(row % v_dim) * page_size + jg % page_size);
          if (jg < lo_min || jg + 7 > pos_max) {  // keys that no row of the tile reads may hold anything
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (jg + e < lo_min || jg + e > pos_max) rv[r].h[e] = 0;
          }
        }
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int r = 0; r < KPT; ++r) {
      const int p = tid + 256 * r;
      const int key = p / kpieces, e = (p % kpieces) * 8;
      if (key < 32) *reinterpret_cast<uint4*>(&sk[key * KLD + e]) = rk[r].u;
    }
#pragma unroll
    for (int r = 0; r < VPT; ++r) {
      const int p = tid + 256 * r;
      const int row = p / 4, kq = p % 4;
      if (row < vrows) {
        // LDS rows go by blocks of 16 elements of a key/value head: block (cv * vb + d / 16), row d % 16
        const int cv = row / v_dim, d = row % v_dim;
        *reinterpret_cast<uint4*>(&sv[((cv * vb + d / 16) * 16 + d % 16) * VLD + kq * 8]) = rv[r].u;
        if (row == 0) group_ok[kq] = rv_ok[r];
      }
    }
  };
  // (elements of a key beyond head_dim, and value rows beyond v_dim, are never staged: they stay zero from here)
  for (int z = tid; z < (32 * KLD + NB * 16 * VLD) / 2; z += 256) reinterpret_cast<uint32_t*>(lds_t)[z] = 0u;
  const int j_begin = lo_min / 32 * 32;
  fetch(j_begin);
  for (int j0 = j_begin; j0 <= pos_max; j0 += 32) {
    __syncthreads();  // (the chunk before has been read; the first time: the zeros are in place)
    stage();
    __syncthreads();
    if (j0 + 32 <= pos_max) fetch(j0 + 32);
    if (!has_head) continue;
    tf32x4 s[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      s[t2] = tf32x4{0.f, 0.f, 0.f, 0.f};
      const int key = 8 * (i / 4) + 4 * t2 + i % 4;  // A row i of product t2
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint4 kv = *reinterpret_cast<const uint4*>(&sk[key * KLD + ks * 32 + kg * 8]);
        s[t2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tbf16x8, kv), qf[ks], s[t2], 0, 0, 0);
      }
    }
    const int jg = j0 + 8 * kg;
    const bool paged = group_ok[kg] != 0;
    float x[8];
    float mx = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = jg + 4 * t2 + r;
        float v = s[t2][r] * scale_l2;
        if (r1) v -= bias1 * __log2f(1.f + bias2 * static_cast<float>(pos - j));
        const bool seen = paged && j >= lo && j <= pos;
        v = seen ? v : -INFINITY;
        x[4 * t2 + r] = v;
        mx = fmaxf(mx, v);
      }
    const float m_new = fmaxf(m_run, rows_max(mx));
    const float alpha = m_run > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_new) : 0.f;
    float psum = 0.f;
    Piece pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = x[e] > -INFINITY ? __builtin_amdgcn_exp2f(x[e] - m_new) : 0.f;
      psum += p;
      const bf16 pb = from_float<bf16>(p);
      pf.h[e] = __builtin_bit_cast(uint16_t, pb);
    }
    l_run = l_run * alpha + rows_sum(psum);
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[b][r] *= alpha;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b < cvn * vb) {
        const uint4 vv = *reinterpret_cast<const uint4*>(&sv[(b * 16 + i) * VLD + kg * 8]);
        o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tbf16x8, vv), __builtin_bit_cast(tbf16x8, pf.u),
                                                       o[b], 0, 0, 0);
      }
    }
  }
  if (!valid || !has_head) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  float* dst = u_out + (static_cast<size_t>(t) * heads + head) * kv_heads * v_dim;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (b >= cvn * vb) continue;
    const int cv = cv0 + b / vb;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = (b % vb) * 16 + 4 * kg + r;
      if (d < v_dim) dst[static_cast<size_t>(cv) * v_dim + d] = o[b][r] * inv;
    }
  }
}

// u[t, g, :] of single tokens from their shares: sum_z o_z 2^(m_z - m) / sum_z l_z 2^(m_z - m)
__global__ void __launch_bounds__(256)
    talking_join_kernel(const float* __restrict__ partial, float* __restrict__ u_out, int heads, int gv, int nsplit) {
  const int t = blockIdx.y;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= heads * gv) return;
  const int head = idx / gv, rest = idx % gv;
  const float* base = partial + (static_cast<size_t>(t) * heads + head) * nsplit * (gv + 2);
  float m = -INFINITY;
  for (int z = 0; z < nsplit; ++z) m = fmaxf(m, base[static_cast<size_t>(z) * (gv + 2) + gv]);
  float den = 0.f, val = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = base[static_cast<size_t>(z) * (gv + 2) + gv];
    if (mz > -INFINITY) {
      const float w = __builtin_amdgcn_exp2f(mz - m);
      den = fmaf(base[static_cast<size_t>(z) * (gv + 2) + gv + 1], w, den);
      val = fmaf(base[static_cast<size_t>(z) * (gv + 2) + rest], w, val);
    }
  }
  u_out[(static_cast<size_t>(t) * heads + head) * gv + rest] = den > 0.f ? val / den : 0.f;
}

// out[t, h, d] = sum_g talk[h, g] * U[t, g, c(h), d]   (talk null: U[t, h, c(h), d]).  A thread takes one
// value element of one key/value head and forms it for all query heads of that key/value head, eight
// at a time: what it reads of U serves them all.
__global__ void __launch_bounds__(256)
    talking_mix_kernel(const float* __restrict__ u_in, const float* __restrict__ talk, bf16* __restrict__ out, int heads,
                       int kv_heads, int v_dim) {
  const int t = blockIdx.y;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= kv_heads * v_dim) return;
  const int c = idx / v_dim, d = idx % v_dim;
  const int group = heads / kv_heads;
  const size_t gv = static_cast<size_t>(kv_heads) * v_dim;
  const float* ut = u_in + static_cast<size_t>(t) * heads * gv + idx;
  bf16* ot = out + static_cast<size_t>(t) * heads * v_dim + d;
  if (!talk) {
    for (int k = 0; k < group; ++k) {
      const int h = c * group + k;
      ot[static_cast<size_t>(h) * v_dim] = from_float<bf16>(ut[h * gv]);
    }
    return;
  }
  for (int k0 = 0; k0 < group; k0 += 8) {
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = 0.f;
    const float* row = talk + static_cast<size_t>(c * group + k0) * heads;
    for (int g = 0; g < heads; ++g) {
      const float u = ut[g * gv];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (k0 + k < group) acc[k] = fmaf(row[k * heads + g], u, acc[k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (k0 + k < group) ot[static_cast<size_t>(c * group + k0 + k) * v_dim] = from_float<bf16>(acc[k]);
  }
}

// The same a thread per output element, for steps of few tokens (more workgroups than the kernel above has).
__global__ void __launch_bounds__(256)
    talking_mix_each_kernel(const float* __restrict__ u_in, const float* __restrict__ talk, bf16* __restrict__ out,
                            int heads, int kv_heads, int v_dim) {
  const int t = blockIdx.y;
  const int o = blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= heads * v_dim) return;
  const int h = o / v_dim, d = o % v_dim;
  const int c = h / (heads / kv_heads);
  const float* ut = u_in + static_cast<size_t>(t) * heads * kv_heads * v_dim + static_cast<size_t>(c) * v_dim + d;
  float sum = 0.f;
  if (talk) {
    for (int g = 0; g < heads; ++g) sum = fmaf(talk[h * heads + g], ut[static_cast<size_t>(g) * kv_heads * v_dim], sum);
  } else {
    sum = ut[static_cast<size_t>(h) * kv_heads * v_dim];
  }
  out[static_cast<size_t>(t) * heads * v_dim + o] = from_float<bf16>(sum);
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

// bfloat16 on the matrix units.  The step's first `num_single` tokens are single tokens of their
// sequences; the prompt portions that follow are listed in tiles of 16 queries (tile_seq, tile_q0
// from the portion's first query; cu_q[s] is sequence s's first row).  scratch: n * heads *
// kv_heads * v_dim floats.
extern "C" int shk_attention_talking_supports_mfma(int head_dim, int v_dim, int page_size, int q_stride) {
  return head_dim % 8 == 0 && head_dim <= 256 && v_dim >= 1 && v_dim <= 256 && page_size % 8 == 0 && q_stride % 8 == 0;
}

extern "C" long long shk_attention_talking_mfma_scratch_floats(int n, int num_single, int heads, int kv_heads, int v_dim,
                                                               int nsplit) {
  const long long gv = static_cast<long long>(kv_heads) * v_dim;
  return static_cast<long long>(n) * heads * gv + (nsplit > 1 ? static_cast<long long>(num_single) * heads * nsplit * (gv + 2) : 0);
}

namespace shk {

template <int KS, int NB>
static void launch_talking_mfma(dim3 grid, hipStream_t s, const bf16* q, int q_stride, float* u, int heads, int kv_heads,
                                int head_dim, int v_dim, const int32_t* positions, const int32_t* token_seq,
                                const int32_t* tables, int table_stride, const bf16* k_pool, const bf16* v_pool,
                                int page_size, int num_pages, int window, int chunk, float scale_l2, const float* r1,
                                const float* r2, int has_sink, float sink_l2, int nsplit, float* partial, int vh_pass) {
  talking_mfma_kernel<KS, NB><<<grid, 256, 0, s>>>(q, q_stride, u, heads, kv_heads, head_dim, v_dim, positions, token_seq,
                                                   tables, table_stride, k_pool, v_pool, page_size, num_pages, window,
                                                   chunk, scale_l2, r1, r2, has_sink, sink_l2, nsplit, partial, vh_pass);
}

}  // namespace shk

extern "C" int shk_attention_talking_bf16(const void* q, int q_stride, void* out, int n, int num_single, int num_tiles,
                                          int heads, int kv_heads, int head_dim, int v_dim, const int32_t* positions,
                                          const int32_t* token_seq, const int32_t* cu_q, const int32_t* tile_seq,
                                          const int32_t* tile_q0, const int32_t* tables, int table_stride,
                                          const void* k_pool, const void* v_pool, int page_size, int num_pages,
                                          int window, int chunk, float scale, const float* r1, const float* r2,
                                          const float* talk, int has_sink, float sink, float* scratch, int nsplit,
                                          void* stream) {
  SHK_REQUIRE(n >= 0 && num_single >= 0 && num_single <= n && num_tiles >= 0 && heads > 0 && kv_heads > 0 &&
                  heads % kv_heads == 0,
              "attention_talking_bf16: bad sizes n=%d single=%d tiles=%d heads=%d kv_heads=%d", n, num_single, num_tiles,
              heads, kv_heads);
  SHK_REQUIRE(shk_attention_talking_supports_mfma(head_dim, v_dim, page_size, q_stride),
              "attention_talking_bf16: head_dim %d, v_dim %d, page_size %d or q_stride %d is not served", head_dim, v_dim,
              page_size, q_stride);
  SHK_REQUIRE(q_stride >= heads * head_dim && page_size > 0 && num_pages > 0 && table_stride > 0,
              "attention_talking_bf16: bad strides or cache sizes");
  SHK_REQUIRE(static_cast<int64_t>(num_pages) * kv_heads * page_size < (1LL << 31),
              "attention_talking_bf16: cache pool has too many rows for 32-bit row indices");
  SHK_REQUIRE((r1 == nullptr) == (r2 == nullptr), "attention_talking_bf16: the distance bias needs both of its numbers");
  if (n == 0) return 0;
  SHK_REQUIRE(q && out && positions && token_seq && tables && k_pool && v_pool && scratch,
              "attention_talking_bf16: null pointer");
  SHK_REQUIRE(num_tiles == 0 || (cu_q && tile_seq && tile_q0), "attention_talking_bf16: tiles without their lists");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k_pool) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(v_pool) % 16 == 0,
              "attention_talking_bf16: operands must be 16-byte aligned");
  SHK_REQUIRE(n <= 65535 && num_tiles <= 0x7fffffff / 4, "attention_talking_bf16: at most 65535 tokens a call, got %d", n);
  SHK_REQUIRE(nsplit >= 1 && nsplit <= 64, "attention_talking_bf16: 1 to 64 shares of a single token's keys, got %d", nsplit);
  float* partial = scratch + static_cast<size_t>(n) * heads * kv_heads * v_dim;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float log2e = 1.4426950408889634f;
  const int ks = (head_dim + 31) / 32, vb = (v_dim + 15) / 16;
  const int group = heads / kv_heads;
#define SHK_GO(KS, NB)                                                                                                 \
  launch_talking_mfma<KS, NB>(grid, s, static_cast<const bf16*>(q), q_stride, scratch, heads, kv_heads, head_dim, v_dim, \
                              positions, token_seq, tables, table_stride, static_cast<const bf16*>(k_pool),             \
                              static_cast<const bf16*>(v_pool), page_size, num_pages, window, chunk, scale * log2e, r1,  \
                              r2, has_sink, sink * log2e, shares, partial, vh_pass)
#define SHK_NB(KS)                                                                                                     \
  if (nb <= 2) SHK_GO(KS, 2);                                                                                          \
  else if (nb <= 4) SHK_GO(KS, 4);                                                                                     \
  else if (nb <= 8) SHK_GO(KS, 8);                                                                                     \
  else SHK_GO(KS, 16)
#define SHK_KS()                                                                                                       \
  if (ks <= 1) { SHK_NB(1); }                                                                                          \
  else if (ks <= 2) { SHK_NB(2); }                                                                                     \
  else if (ks <= 4) { SHK_NB(4); }                                                                                     \
  else { SHK_NB(8); }
  if (num_single > 0) {
    // single tokens: a key/value head's query heads are a tile's rows; one value head a workgroup
    const int vh_pass = 1, nb = vb, shares = nsplit;
    const int units = kv_heads * ((group + 15) / 16);
    dim3 grid(num_single * nsplit, (units + 3) / 4, kv_heads);
    SHK_KS()
    if (nsplit > 1) {
      const int items = heads * kv_heads * v_dim;
      talking_join_kernel<<<dim3((items + 255) / 256, num_single), 256, 0, s>>>(partial, scratch, heads, kv_heads * v_dim,
                                                                              nsplit);
    }
  }
  if (num_tiles > 0) {
    // a chunk staged once for four heads; 16 blocks of sums a pass where a head's values allow it
    const int vh_pass = max(1, min(kv_heads, 16 / vb));
    const int nb = vh_pass * vb;
    dim3 grid(num_tiles, kv_heads * ((group + 3) / 4), (kv_heads + vh_pass - 1) / vh_pass);
#define SHK_LDS(KS, NB)                                                                                                \
  talking_tiles_lds_kernel<KS, NB><<<grid, 256, (32 * (KS * 32 + 8) + NB * 16 * 40) * sizeof(uint16_t), s>>>(           \
      static_cast<const bf16*>(q), q_stride, scratch, heads, kv_heads, head_dim, v_dim, positions, tables, table_stride, \
      static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), page_size, num_pages, window, chunk,           \
      scale * log2e, r1, r2, has_sink, sink * log2e, cu_q, tile_seq, tile_q0, vh_pass)
#define SHK_LDS_NB(KS)                                                                                                 \
  if (nb <= 4) SHK_LDS(KS, 4);                                                                                         \
  else if (nb <= 8) SHK_LDS(KS, 8);                                                                                    \
  else SHK_LDS(KS, 16)
    if (ks <= 1) { SHK_LDS_NB(1); }
    else if (ks <= 2) { SHK_LDS_NB(2); }
    else if (ks <= 4) { SHK_LDS_NB(4); }
    else { SHK_LDS_NB(8); }
#undef SHK_LDS_NB
#undef SHK_LDS
  }
#undef SHK_KS
#undef SHK_NB
#undef SHK_GO
  if (n >= 64) {
    const int outs = kv_heads * v_dim;
    talking_mix_kernel<<<dim3((outs + 255) / 256, n), 256, 0, s>>>(scratch, talk, static_cast<bf16*>(out), heads,
                                                                  kv_heads, v_dim);
  } else {
    const int outs = heads * v_dim;
    talking_mix_each_kernel<<<dim3((outs + 255) / 256, n), 256, 0, s>>>(scratch, talk, static_cast<bf16*>(out), heads,
                                                                       kv_heads, v_dim);
  }
  SHK_LAUNCH_CHECK("attention_talking_bf16");
  return 0;
}
