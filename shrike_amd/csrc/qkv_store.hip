// Cache write for attention without rotation, whose keys and values may differ in
// size: queries are scaled by a factor that grows slowly with the position, each
// head's value may be brought to unit root mean square, keys and values go to their
// page slots (keys in slabs, values transposed, as the attention kernels read them).
// Queries and keys may be brought to unit root mean square per head first (with or
// without a weight of the head's size that all heads share); a layer that reads
// another layer's keys and values brings rows of queries alone.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kStoreThreads = 256;

template <typename T>
__global__ void __launch_bounds__(kStoreThreads)
    qkv_store_kernel(T* __restrict__ qkv, int heads, int kv_heads, int head_dim, int v_dim, float q_coef,
                     int q_every, float v_eps, float qk_eps, const float* __restrict__ q_weight,
                     const float* __restrict__ k_weight, int has_kv, const int32_t* __restrict__ positions,
                     const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                     int table_stride, T* __restrict__ k_pool, T* __restrict__ v_pool, int page_size,
                     int num_pages, int write_kv) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int q_width = heads * head_dim, k_width = kv_heads * head_dim;
  T* row = qkv + static_cast<size_t>(t) * (q_width + (has_kv ? k_width + kv_heads * v_dim : 0));
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;

  // 1 + coef * ln(floor((p + 1) / every) + 1): 1 for the first `every` - 1 positions
  const float factor = q_every > 0 ? 1.f + q_coef * logf(static_cast<float>((pos + 1) / q_every + 1)) : 1.f;
  if (qk_eps > 0.f) {
    // one wavefront per query head: the head's mean square, then its elements, weighted, times the factor
    for (int h = wave; h < heads; h += kStoreThreads / kWave) {
      T* q = row + h * head_dim;
      float sq = 0.f;
      for (int d = lane; d < head_dim; d += kWave) {
        const float x = to_float(q[d]);
        sq = fmaf(x, x, sq);
      }
      const float inv = 1.f / sqrtf(wave_sum(sq) / static_cast<float>(head_dim) + qk_eps);
      for (int d = lane; d < head_dim; d += kWave) {
        float x = to_float(q[d]) * inv;
        if (q_weight) x *= q_weight[d];
        q[d] = from_float<T>(x * factor);
      }
    }
  } else if (q_every > 0) {
    for (int i = threadIdx.x; i < q_width; i += kStoreThreads) row[i] = from_float<T>(to_float(row[i]) * factor);
  }
  if (!write_kv || !has_kv) return;
  int page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
  if (page < 0 || page >= num_pages) return;  // a host bug; never dereferenced
  const int slot = pos % page_size;
  if (qk_eps > 0.f) {
    for (int g = wave; g < kv_heads; g += kStoreThreads / kWave) {
      const T* k = row + q_width + g * head_dim;
      float sq = 0.f;
      for (int d = lane; d < head_dim; d += kWave) {
        const float x = to_float(k[d]);
        sq = fmaf(x, x, sq);
      }
      const float inv = 1.f / sqrtf(wave_sum(sq) / static_cast<float>(head_dim) + qk_eps);
      T* dst = k_pool + (static_cast<size_t>(page) * kv_heads + g) * page_size * head_dim;
      for (int d = lane; d < head_dim; d += kWave) {
        float x = to_float(k[d]) * inv;
        if (k_weight) x *= k_weight[d];
        dst[key_offset(slot, d, page_size, head_dim)] = from_float<T>(x);
      }
    }
  } else {
    for (int i = threadIdx.x; i < k_width; i += kStoreThreads) {
      const int g = i / head_dim, d = i % head_dim;
      k_pool[(static_cast<size_t>(page) * kv_heads + g) * page_size * head_dim + key_offset(slot, d, page_size, head_dim)] =
          row[q_width + i];
    }
  }
  // one wavefront per key/value head: the head's mean square, then its elements
  for (int g = wave; g < kv_heads; g += kStoreThreads / kWave) {
    const T* v = row + q_width + k_width + g * v_dim;
    float scale = 1.f;
    if (v_eps > 0.f) {
      float sq = 0.f;
      for (int d = lane; d < v_dim; d += kWave) {
        const float x = to_float(v[d]);
        sq = fmaf(x, x, sq);
      }
      scale = 1.f / sqrtf(wave_sum(sq) / static_cast<float>(v_dim) + v_eps);
    }
    T* dst = v_pool + (static_cast<size_t>(page) * kv_heads + g) * v_dim * page_size + slot;
    for (int d = lane; d < v_dim; d += kWave) dst[static_cast<size_t>(d) * page_size] = from_float<T>(to_float(v[d]) * scale);
  }
}

// The same with normed queries and keys, a wavefront per head (of the queries, of the keys, of the
// values): the head is held in registers between its mean square and its write, and a token's heads
// spread over as many workgroups as it takes, so that a step of few tokens is not one long chain.
constexpr int kMaxPerLane = 4;  // head sizes up to 256

template <typename T>
__global__ void __launch_bounds__(kStoreThreads)
    qkv_norm_store_kernel(T* __restrict__ qkv, int heads, int kv_heads, int head_dim, int v_dim, float q_coef,
                          int q_every, float v_eps, float qk_eps, const float* __restrict__ q_weight,
                          const float* __restrict__ k_weight, int has_kv, const int32_t* __restrict__ positions,
                          const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                          int table_stride, T* __restrict__ k_pool, T* __restrict__ v_pool, int page_size,
                          int num_pages, int write_kv) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int unit = blockIdx.y * (kStoreThreads / kWave) + wave;
  const int stored = (write_kv && has_kv) ? 2 * kv_heads : 0;
  if (unit >= heads + stored) return;
  const int pos = positions[t];
  const int q_width = heads * head_dim, k_width = kv_heads * head_dim;
  T* row = qkv + static_cast<size_t>(t) * (q_width + (has_kv ? k_width + kv_heads * v_dim : 0));
  const bool is_q = unit < heads, is_k = !is_q && unit < heads + kv_heads;
  const int g = is_q ? unit : is_k ? unit - heads : unit - heads - kv_heads;
  const int size = (is_q || is_k) ? head_dim : v_dim;
  T* src = row + (is_q ? g * head_dim : is_k ? q_width + g * head_dim : q_width + k_width + g * v_dim);
  float x[kMaxPerLane];
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + i * kWave;
    x[i] = d < size ? to_float(src[d]) : 0.f;
    sq = fmaf(x[i], x[i], sq);
  }
  const float eps = (is_q || is_k) ? qk_eps : v_eps;
  float mult = eps > 0.f ? 1.f / sqrtf(wave_sum(sq) / static_cast<float>(size) + eps) : 1.f;
  const float* weight = is_q ? q_weight : is_k ? k_weight : nullptr;
  if (is_q) {
    // 1 + coef * ln(floor((p + 1) / every) + 1), applied after the norm and its weight
    const float factor = q_every > 0 ? 1.f + q_coef * logf(static_cast<float>((pos + 1) / q_every + 1)) : 1.f;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + i * kWave;
      if (d < size) src[d] = from_float<T>((weight ? x[i] * mult * weight[d] : x[i] * mult) * factor);
    }
    return;
  }
  int page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
  if (page < 0 || page >= num_pages) return;  // a host bug; never dereferenced
  const int slot = pos % page_size;
  if (is_k) {
    T* dst = k_pool + (static_cast<size_t>(page) * kv_heads + g) * page_size * head_dim;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + i * kWave;
      if (d < size) dst[key_offset(slot, d, page_size, head_dim)] = from_float<T>(weight ? x[i] * mult * weight[d] : x[i] * mult);
    }
  } else {
    T* dst = v_pool + (static_cast<size_t>(page) * kv_heads + g) * v_dim * page_size + slot;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + i * kWave;
      if (d < size) dst[static_cast<size_t>(d) * page_size] = eps > 0.f ? from_float<T>(x[i] * mult) : src[d];
    }
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_qkv_store(void* qkv, int dtype, int n, int heads, int kv_heads, int head_dim, int v_dim,
                             float q_coef, int q_every, float v_eps, float qk_eps, const float* q_weight,
                             const float* k_weight, int has_kv, const int32_t* positions,
                             const int32_t* token_seq, const int32_t* tables, int table_stride, void* k_pool,
                             void* v_pool, int page_size, int num_pages, int write_kv, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "qkv_store: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && v_dim > 0,
              "qkv_store: bad sizes n=%d heads=%d kv_heads=%d head_dim=%d v_dim=%d", n, heads, kv_heads, head_dim, v_dim);
  SHK_REQUIRE(q_every >= 0, "qkv_store: q_every must not be negative, got %d", q_every);
  SHK_REQUIRE(qk_eps >= 0.f && (qk_eps > 0.f || (!q_weight && !k_weight)),
              "qkv_store: a norm of queries and keys needs a positive eps (0: no norm, and then no weights)");
  SHK_REQUIRE(has_kv || !write_kv, "qkv_store: rows without keys and values have nothing to write to a cache");
  if (n == 0) return 0;
  SHK_REQUIRE(qkv && positions, "qkv_store: null pointer");
  if (write_kv) {
    SHK_REQUIRE(token_seq && tables && k_pool && v_pool, "qkv_store: null pointer");
    SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
                "qkv_store: bad cache sizes page_size=%d num_pages=%d table_stride=%d", page_size, num_pages, table_stride);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (qk_eps > 0.f && head_dim <= kMaxPerLane * kWave && v_dim <= kMaxPerLane * kWave) {
    const int units = heads + ((write_kv && has_kv) ? 2 * kv_heads : 0);
    const dim3 grid(n, (units + kStoreThreads / kWave - 1) / (kStoreThreads / kWave));
    SHK_REQUIRE(grid.y <= 65535, "qkv_store: too many heads");
    if (dtype == kF32)
      qkv_norm_store_kernel<float><<<grid, kStoreThreads, 0, s>>>(
          static_cast<float*>(qkv), heads, kv_heads, head_dim, v_dim, q_coef, q_every, v_eps, qk_eps, q_weight, k_weight,
          has_kv, positions, token_seq, tables, table_stride, static_cast<float*>(k_pool), static_cast<float*>(v_pool),
          page_size, num_pages, write_kv);
    else
      qkv_norm_store_kernel<bf16><<<grid, kStoreThreads, 0, s>>>(
          static_cast<bf16*>(qkv), heads, kv_heads, head_dim, v_dim, q_coef, q_every, v_eps, qk_eps, q_weight, k_weight,
          has_kv, positions, token_seq, tables, table_stride, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool),
          page_size, num_pages, write_kv);
    SHK_LAUNCH_CHECK("qkv_store");
    return 0;
  }
  if (dtype == kF32)
    qkv_store_kernel<float><<<n, kStoreThreads, 0, s>>>(static_cast<float*>(qkv), heads, kv_heads, head_dim, v_dim,
                                                        q_coef, q_every, v_eps, qk_eps, q_weight, k_weight, has_kv,
                                                        positions, token_seq, tables,
                                                        table_stride, static_cast<float*>(k_pool),
                                                        static_cast<float*>(v_pool), page_size, num_pages, write_kv);
  else
    qkv_store_kernel<bf16><<<n, kStoreThreads, 0, s>>>(static_cast<bf16*>(qkv), heads, kv_heads, head_dim, v_dim,
                                                       q_coef, q_every, v_eps, qk_eps, q_weight, k_weight, has_kv,
                                                       positions, token_seq, tables,
                                                       table_stride, static_cast<bf16*>(k_pool),
                                                       static_cast<bf16*>(v_pool), page_size, num_pages, write_kv);
  SHK_LAUNCH_CHECK("qkv_store");
  return 0;
}
