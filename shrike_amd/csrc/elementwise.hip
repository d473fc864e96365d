// Embedding lookup, residual add + RMSNorm, gate activation times up.
// All arithmetic is float32; storage is float32 or bfloat16.
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

namespace shk {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ------------------------------------------------------------------ embedding

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                             float* __restrict__ out, int hidden, float scale) {
  const int row = blockIdx.x;
  const T* src = table + static_cast<size_t>(ids[row]) * hidden;
  float* dst = out + static_cast<size_t>(row) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

// ------------------------------------------------------------ add + RMSNorm
// One workgroup per row.  add_rmsnorm_vec_kernel holds the row in registers
// (hidden a multiple of 4, at most 8192 elements): all loads are issued
// before the first use, so a row costs one memory round trip.
// add_rmsnorm_kernel takes every other size.

constexpr int kNormThreads = 256;
constexpr int kNormVecs = 2;  // float4 per thread: rows of up to 8192 elements with 1024 threads

__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                     __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  uint2 u;
  u.x = bf16_bits(v.x) | (static_cast<uint32_t>(bf16_bits(v.y)) << 16);
  u.y = bf16_bits(v.z) | (static_cast<uint32_t>(bf16_bits(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// TD is the type of delta: T, or float for the partial sums of a split product
// ([splits][resid_rows][hidden], added in order).  THREADS * 4 * kNormVecs
// elements fit; wide rows get 1024 threads so that few loads follow each other.
template <typename T, typename TD, int THREADS>
__global__ void __launch_bounds__(THREADS)
    add_rmsnorm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                           const float* __restrict__ weight, float eps, T* __restrict__ out,
                           const int32_t* __restrict__ rows, int hidden, int write_resid,
                           int splits, size_t split_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* x = resid + row * hidden;
  const TD* d = delta ? delta + row * hidden : nullptr;
  T* y = out + static_cast<size_t>(r) * hidden;
  const int nvec = hidden / 4;

  float4 v[kNormVecs], dv[kNormVecs], w[kNormVecs];
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    v[i] = dv[i] = w[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < nvec) {
      v[i] = load4(x + c * 4);
      if (d) dv[i] = load4(d + c * 4);
      w[i] = load4(weight + c * 4);
    }
  }
  // further parts, four at a time in flight, added in order
  for (int z0 = 1; z0 < splits; z0 += 4) {
    float4 more[4][kNormVecs];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < kNormVecs; ++i) {
        const int c = threadIdx.x + i * THREADS;
        more[u][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < nvec && z0 + u < splits) more[u][i] = load4(d + (z0 + u) * split_stride + c * 4);
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < kNormVecs; ++i)
        dv[i].x += more[u][i].x, dv[i].y += more[u][i].y, dv[i].z += more[u][i].z,
            dv[i].w += more[u][i].w;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    v[i].x += dv[i].x, v[i].y += dv[i].y, v[i].z += dv[i].z, v[i].w += dv[i].w;
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
    if (d && write_resid) store4(x + c * 4, v[i]);
    store4(y + c * 4, make_float4((v[i].x * inv) * w[i].x, (v[i].y * inv) * w[i].y,
                                  (v[i].z * inv) * w[i].z, (v[i].w * inv) * w[i].w));
  }
}

template <typename T>
__global__ void __launch_bounds__(kNormThreads)
    add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                       const float* __restrict__ weight, float eps, T* __restrict__ out,
                       const int32_t* __restrict__ rows, int hidden, int write_resid) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* x = resid + row * hidden;
  const T* d = delta ? delta + row * hidden : nullptr;
  T* y = out + static_cast<size_t>(r) * hidden;

  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = x[i];
    if (d) {
      v += to_float(d[i]);
      if (write_resid) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = x[i];
    if (d && !write_resid) v += to_float(d[i]);
    y[i] = from_float<T>((v * inv) * weight[i]);
  }
}

// ------------------------------------------------------------ act(gate) * up
// act 1: SiLU, g / (1 + exp(-g)).  act 2: the tanh form of GELU,
// 0.5 g (1 + tanh(u)), u = sqrt(2/pi) (g + 0.044715 g^3), written as g / (1 + exp(-2u)).
// act 3: ReLU.  act 4: g sigmoid(1.702 g).  limit > 0 bounds the gate from above and the
// other factor from both sides before anything else; up_shift is added to that factor.

template <typename T>
__global__ void act_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int act, float limit,
                               float up_shift) {
  const size_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= inter) return;
  float g = to_float(gu[row * 2 * inter + j]);
  float u = to_float(gu[row * 2 * inter + inter + j]);
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  u += up_shift;
  float s;
  if (act == 3) {
    s = fmaxf(g, 0.f);
  } else {
    const float x = act == 2 ? 2.f * 0.7978845608028654f * (g + 0.044715f * g * g * g) : act == 4 ? 1.702f * g : g;
    s = g / (1.f + expf(-x));
  }
  out[row * inter + j] = from_float<T>(s * u);
}

// ------------------------------------------------- rows held in registers
// The kernels below keep one row per workgroup in registers: V elements per access
// (4: whole vectors, for widths that are a multiple of 4 and aligned buffers; 1:
// every other width), S accesses per thread, THREADS threads; V * S * THREADS
// elements fit.  Wide rows get 1024 threads, so that few loads follow each other.

template <int V>
struct RowVec {
  float v[V];
};

template <int V, typename T>
__device__ __forceinline__ RowVec<V> row_load(const T* p) {
  RowVec<V> r;
  if constexpr (V == 4) {
    const float4 f = load4(p);
    r.v[0] = f.x, r.v[1] = f.y, r.v[2] = f.z, r.v[3] = f.w;
  } else {
    r.v[0] = to_float(p[0]);
  }
  return r;
}

template <int V, typename T>
__device__ __forceinline__ void row_store(T* p, const RowVec<V>& r) {
  if constexpr (V == 4) {
    store4(p, make_float4(r.v[0], r.v[1], r.v[2], r.v[3]));
  } else {
    p[0] = from_float<T>(r.v[0]);
  }
}

// The output of a product for one row: a tensor of T (splits 0) or the float32
// partial sums [splits][rows][hidden] of a product split along k, added in order,
// four parts in flight.
template <int V, int THREADS, int S, typename T>
__device__ __forceinline__ void row_gather(const void* delta, int splits, size_t split_stride,
                                           size_t row, int hidden, RowVec<V> (&d)[S]) {
  const int nvec = hidden / V;
#pragma unroll
  for (int i = 0; i < S; ++i)
#pragma unroll
    for (int e = 0; e < V; ++e) d[i].v[e] = 0.f;
  if (splits == 0) {
#pragma unroll
    for (int i = 0; i < S; ++i) {
      const int c = threadIdx.x + i * THREADS;
      if (c < nvec) d[i] = row_load<V>(static_cast<const T*>(delta) + row * hidden + c * V);
    }
    return;
  }
  const float* p = static_cast<const float*>(delta) + row * hidden;
  for (int z0 = 0; z0 < splits; z0 += 4) {
    RowVec<V> more[4][S];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int z = z0 + u < splits ? z0 + u : splits - 1;  // past the last part: the last again, not added
#pragma unroll
      for (int i = 0; i < S; ++i) {
        const int c = threadIdx.x + i * THREADS;
#pragma unroll
        for (int e = 0; e < V; ++e) more[u][i].v[e] = 0.f;
        if (c < nvec) more[u][i] = row_load<V>(p + z * split_stride + c * V);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool have = z0 + u < splits;
#pragma unroll
      for (int i = 0; i < S; ++i)
#pragma unroll
        for (int e = 0; e < V; ++e) d[i].v[e] += have ? more[u][i].v[e] : 0.f;
    }
  }
}

// resid[r] += other[r] + vec: a second stream and a vector that is the same for every row
// (either may be absent).
__global__ void __launch_bounds__(256)
    add_rows_kernel(float* __restrict__ resid, const float* __restrict__ other,
                    const float* __restrict__ vec, int hidden) {
  const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float v = resid[base + i];
    if (other) v += other[base + i];
    if (vec) v += vec[i];
    resid[base + i] = v;
  }
}

// resid[r] += d1[r] + d2[r]; cast[r] = T(resid[r]).  d1 and d2 are outputs of products
// (see row_gather); d2 and cast may be absent.  (d1 + d2) is formed first, then added.
template <typename T, int V, int THREADS, int S>
__global__ void __launch_bounds__(THREADS)
    add_deltas_kernel(float* __restrict__ resid, const void* __restrict__ d1, int splits1,
                      const void* __restrict__ d2, int splits2, T* __restrict__ cast, int hidden,
                      size_t split_stride) {
  const size_t row = blockIdx.x;
  const int nvec = hidden / V;
  RowVec<V> a[S], b[S], x[S];
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const int c = threadIdx.x + i * THREADS;
#pragma unroll
    for (int e = 0; e < V; ++e) x[i].v[e] = b[i].v[e] = 0.f;
    if (c < nvec) x[i] = row_load<V>(resid + row * hidden + c * V);
  }
  row_gather<V, THREADS, S, T>(d1, splits1, split_stride, row, hidden, a);
  if (d2) row_gather<V, THREADS, S, T>(d2, splits2, split_stride, row, hidden, b);
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
#pragma unroll
    for (int e = 0; e < V; ++e) x[i].v[e] += a[i].v[e] + b[i].v[e];
    row_store<V>(resid + row * hidden + c * V, x[i]);
    if (cast) row_store<V>(cast + row * hidden + c * V, x[i]);
  }
}

// x = resid[row] + delta[row] * rsqrt(mean(delta[row]^2) + deps) * dweight: a product's
// output that is normed by itself before it joins the stream.  With write_resid the sum
// is stored back; with `out`, out[r] = x * rsqrt(mean(x^2) + eps) * weight follows in the
// same pass (the next layer's norm).  rows: as in add_rmsnorm.
template <typename T, int V, int THREADS, int S>
__global__ void __launch_bounds__(THREADS)
    add_normed_rmsnorm_kernel(float* __restrict__ resid, const void* __restrict__ delta, int splits,
                              const float* __restrict__ dweight, float deps,
                              const float* __restrict__ weight, float eps, T* __restrict__ out,
                              const int32_t* __restrict__ rows, int hidden, int write_resid,
                              size_t split_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  const int nvec = hidden / V;
  RowVec<V> x[S], d[S], dw[S], w[S];
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const int c = threadIdx.x + i * THREADS;
#pragma unroll
    for (int e = 0; e < V; ++e) x[i].v[e] = dw[i].v[e] = w[i].v[e] = 0.f;
    if (c < nvec) {
      x[i] = row_load<V>(resid + row * hidden + c * V);
      dw[i] = row_load<V>(dweight + c * V);
      if (out) w[i] = row_load<V>(weight + c * V);
    }
  }
  row_gather<V, THREADS, S, T>(delta, splits, split_stride, row, hidden, d);
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < S; ++i)
#pragma unroll
    for (int e = 0; e < V; ++e) ss += d[i].v[e] * d[i].v[e];
  ss = block_sum(ss, scratch);
  const float dinv = rsqrtf(ss / static_cast<float>(hidden) + deps);
  float xx = 0.f;
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      x[i].v[e] += (d[i].v[e] * dinv) * dw[i].v[e];
      xx += x[i].v[e] * x[i].v[e];
    }
    if (write_resid) row_store<V>(resid + row * hidden + c * V, x[i]);
  }
  if (!out) return;
  xx = block_sum(xx, scratch);
  const float inv = rsqrtf(xx / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int i = 0; i < S; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
    RowVec<V> y;
#pragma unroll
    for (int e = 0; e < V; ++e) y.v[e] = (x[i].v[e] * inv) * w[i].v[e];
    row_store<V>(out + static_cast<size_t>(r) * hidden + c * V, y);
  }
}

// out[r, j] = act(a[r, j]) * table[ids[r], offset + j] for j < width: a gate times a slice
// of a table row chosen by the token (table rows are ld elements apart).  act as in
// act_mul.  splits > 0: a is the float32 partial sums [splits][n][width] of a product
// split along k, added in order.
template <typename T>
__global__ void act_mul_rows_kernel(const void* __restrict__ a, int splits, size_t split_stride,
                                    const T* __restrict__ table, const int32_t* __restrict__ ids,
                                    long long ld, int offset, T* __restrict__ out, int width, int act) {
  const size_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= width) return;
  const float u = to_float(table[static_cast<long long>(ids[row]) * ld + offset + j]);
  float g = 0.f;
  if (splits == 0) {
    g = to_float(static_cast<const T*>(a)[row * width + j]);
  } else {
    const float* p = static_cast<const float*>(a) + row * width + j;
    for (int z0 = 0; z0 < splits; z0 += 8) {  // eight parts in flight
      float part[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) part[q] = p[(z0 + q < splits ? z0 + q : splits - 1) * split_stride];
#pragma unroll
      for (int q = 0; q < 8; ++q) g += z0 + q < splits ? part[q] : 0.f;
    }
  }
  const float x = act == 2 ? 2.f * 0.7978845608028654f * (g + 0.044715f * g * g * g) : g;
  const float s = g / (1.f + expf(-x));
  out[row * width + j] = from_float<T>(s * u);
}

// dst[i] = src[i], except dst[patch_at + j] = patch[j] for j < patch_n.  Either side
// may be page-locked host memory: a step's index arrays come to the device, and
// its chosen tokens go back, without the copy engine, whose hand-overs to and from
// the compute queue cost more than these few hundred words.
__global__ void __launch_bounds__(256)
    copy_words_kernel(const int32_t* __restrict__ src, int32_t* __restrict__ dst, int n,
                      const int32_t* __restrict__ patch, int patch_at, int patch_n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int j = i - patch_at;
  dst[i] = (j >= 0 && j < patch_n) ? patch[j] : src[i];
}

// dst[r, :] = src[index[r], :], rows of `width` 32-bit words.
__global__ void __launch_bounds__(256)
    gather_rows_kernel(const int32_t* __restrict__ src, long long ld, const int32_t* __restrict__ index,
                       int32_t* __restrict__ dst, int width) {
  const int32_t* from = src + static_cast<long long>(index[blockIdx.y]) * ld;
  int32_t* to = dst + static_cast<long long>(blockIdx.y) * width;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < width; i += gridDim.x * blockDim.x) to[i] = from[i];
}

// Zeroes `bytes` bytes from dst (4-byte aligned): whole words, then the odd bytes.
__global__ void __launch_bounds__(256) zero_bytes_kernel(uint8_t* __restrict__ dst, long long bytes) {
  const long long words = bytes / 4;
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; i < words; i += stride)
    reinterpret_cast<uint32_t*>(dst)[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x < bytes - words * 4) dst[words * 4 + threadIdx.x] = 0;
}

}  // namespace shk

using namespace shk;

extern "C" const char* shk_last_error(void) { return g_error; }
extern "C" int shk_version(void) { return 1; }

extern "C" int shk_copy_words(const int32_t* src, int32_t* dst, int n, const int32_t* patch,
                              int patch_at, int patch_n, void* stream) {
  SHK_REQUIRE(n >= 0 && patch_n >= 0 && patch_at >= 0 && patch_at + patch_n <= n,
              "copy_words: bad sizes n=%d patch [%d, %d)", n, patch_at, patch_at + patch_n);
  if (n == 0) return 0;
  SHK_REQUIRE(src && dst && (patch || patch_n == 0), "copy_words: null pointer");
  copy_words_kernel<<<(n + 255) / 256, 256, 0, static_cast<hipStream_t>(stream)>>>(src, dst, n, patch,
                                                                                 patch_at, patch_n);
  SHK_LAUNCH_CHECK("copy_words");
  return 0;
}

extern "C" int shk_gather_rows(const int32_t* src, long long ld, int src_rows, const int32_t* index,
                               int32_t* dst, int rows, int width, void* stream) {
  SHK_REQUIRE(rows >= 0 && width > 0 && ld >= width && src_rows >= 0,
              "gather_rows: bad sizes rows=%d width=%d ld=%lld", rows, width, ld);
  if (rows == 0) return 0;
  SHK_REQUIRE(src && index && dst, "gather_rows: null pointer");
  SHK_REQUIRE(rows <= 65535, "gather_rows: at most 65535 rows per call, got %d", rows);
  const int per_row = (width + 255) / 256 < 64 ? (width + 255) / 256 : 64;
  gather_rows_kernel<<<dim3(per_row, rows), 256, 0, static_cast<hipStream_t>(stream)>>>(src, ld, index, dst,
                                                                                       width);
  SHK_LAUNCH_CHECK("gather_rows");
  return 0;
}

extern "C" int shk_zero_bytes(void* dst, long long bytes, void* stream) {
  SHK_REQUIRE(bytes >= 0, "zero_bytes: negative size");
  if (bytes == 0) return 0;
  SHK_REQUIRE(dst && reinterpret_cast<uintptr_t>(dst) % 4 == 0, "zero_bytes: dst must be 4-byte aligned");
  const long long blocks = (bytes / 4 + 255) / 256;
  zero_bytes_kernel<<<static_cast<int>(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks)), 256, 0,
                      static_cast<hipStream_t>(stream)>>>(static_cast<uint8_t*>(dst), bytes);
  SHK_LAUNCH_CHECK("zero_bytes");
  return 0;
}

extern "C" int shk_embed(const void* table, int dtype, const int32_t* ids, float* out, int n,
                         int hidden, int vocab, float scale, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "embed: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes n=%d hidden=%d vocab=%d", n,
              hidden, vocab);
  if (n == 0) return 0;
  SHK_REQUIRE(table && ids && out, "embed: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == kF32)
    embed_kernel<float><<<n, threads, 0, s>>>(static_cast<const float*>(table), ids, out, hidden, scale);
  else
    embed_kernel<bf16><<<n, threads, 0, s>>>(static_cast<const bf16*>(table), ids, out, hidden, scale);
  SHK_LAUNCH_CHECK("embed");
  return 0;
}

extern "C" int shk_add_rmsnorm(float* resid, const void* delta, const float* weight, float eps,
                               void* out, int dtype, const int32_t* rows, int n, int hidden,
                               int write_resid, int delta_splits, int resid_rows, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_rmsnorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
  SHK_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be > 0");
  if (n == 0) return 0;
  SHK_REQUIRE(resid && weight && out, "add_rmsnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = hidden % 4 == 0 && hidden <= 1024 * 4 * kNormVecs && aligned(resid) &&
                   aligned(weight) && aligned(out) && (!delta || aligned(delta));
  SHK_REQUIRE(delta_splits == 0 || (delta && vec && dtype == kBF16 && resid_rows > 0),
              "add_rmsnorm: partial sums need bfloat16 output, hidden %% 4 == 0 and at most 8192");
  const size_t stride = static_cast<size_t>(resid_rows) * hidden;
  const int splits = delta_splits > 0 ? delta_splits : 1;
#define SHK_NORM(T, TD, THREADS)                                                              \
  add_rmsnorm_vec_kernel<T, TD, THREADS><<<n, THREADS, 0, s>>>(                               \
      resid, static_cast<const TD*>(delta), weight, eps, static_cast<T*>(out), rows, hidden,  \
      write_resid, splits, stride)
#define SHK_NORM_T(T, TD)                \
  do {                                   \
    if (hidden <= 256 * 4 * kNormVecs)   \
      SHK_NORM(T, TD, 256);              \
    else                                 \
      SHK_NORM(T, TD, 1024);             \
  } while (0)
  if (delta_splits > 0) {
    SHK_NORM_T(bf16, float);
  } else if (vec && dtype == kF32) {
    SHK_NORM_T(float, float);
  } else if (vec) {
    SHK_NORM_T(bf16, bf16);
  } else if (dtype == kF32) {
    add_rmsnorm_kernel<float><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const float*>(delta), weight, eps, static_cast<float*>(out), rows,
        hidden, write_resid);
  } else {
    add_rmsnorm_kernel<bf16><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const bf16*>(delta), weight, eps, static_cast<bf16*>(out), rows, hidden,
        write_resid);
  }
#undef SHK_NORM_T
#undef SHK_NORM
  SHK_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

extern "C" int shk_act_mul(const void* gu, void* out, int dtype, int n, int inter, int act, float limit,
                           float up_shift, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "act_mul: unknown dtype %d", dtype);
  SHK_REQUIRE(act >= 1 && act <= 4, "act_mul: unknown activation %d", act);
  SHK_REQUIRE(limit >= 0.f, "act_mul: a limit must be positive (0: none), got %g", limit);
  SHK_REQUIRE(n >= 0 && inter > 0, "act_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "act_mul: at most 65535 rows a call, got %d", n);
  SHK_REQUIRE(gu && out, "act_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((inter + 255) / 256, n);
  if (dtype == kF32)
    act_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gu),
                                                static_cast<float*>(out), inter, act, limit, up_shift);
  else
    act_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gu),
                                               static_cast<bf16*>(out), inter, act, limit, up_shift);
  SHK_LAUNCH_CHECK("act_mul");
  return 0;
}

// Which form of the register-held row kernels takes a width: 4 x 256 x 2, 4 x 512 x 2,
// 4 x 1024 x 2 (whole vectors), 1 x 256 x 4 or 1 x 1024 x 8 elements; 0: too wide.
static int row_form(int hidden, bool aligned) {
  if (hidden % 4 == 0 && aligned && hidden <= 4 * 256 * 2) return 1;
  if (hidden % 4 == 0 && aligned && hidden <= 4 * 512 * 2) return 5;
  if (hidden % 4 == 0 && aligned && hidden <= 4 * 1024 * 2) return 2;
  if (hidden <= 256 * 4) return 3;
  if (hidden <= 1024 * 8) return 4;
  return 0;
}
static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// SHK_ROW_FORMS(GO, T): GO(T, V, THREADS, S) for the form that row_form chose
#define SHK_ROW_FORMS(GO, T)        \
  do {                              \
    if (form == 1) GO(T, 4, 256, 2);       \
    else if (form == 5) GO(T, 4, 512, 2);  \
    else if (form == 2) GO(T, 4, 1024, 2); \
    else if (form == 3) GO(T, 1, 256, 4);  \
    else GO(T, 1, 1024, 8);                \
  } while (0)

extern "C" int shk_add_rows(float* resid, const float* other, const float* vec, int n, int hidden,
                            void* stream) {
  SHK_REQUIRE(n >= 0 && hidden > 0, "add_rows: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0 || (!other && !vec)) return 0;
  SHK_REQUIRE(resid, "add_rows: null pointer");
  add_rows_kernel<<<n, 256, 0, static_cast<hipStream_t>(stream)>>>(resid, other, vec, hidden);
  SHK_LAUNCH_CHECK("add_rows");
  return 0;
}

extern "C" int shk_add_deltas(float* resid, const void* d1, int splits1, const void* d2, int splits2,
                              void* cast, int dtype, int n, int hidden, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_deltas: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && splits1 >= 0 && splits2 >= 0, "add_deltas: bad sizes n=%d hidden=%d",
              n, hidden);
  if (n == 0) return 0;
  SHK_REQUIRE(resid && d1, "add_deltas: null pointer");
  const int form = row_form(hidden, aligned16(resid) && aligned16(d1) && aligned16(d2) && aligned16(cast));
  SHK_REQUIRE(form != 0, "add_deltas: rows of %d elements are too wide", hidden);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t stride = static_cast<size_t>(n) * hidden;
#define SHK_GO(T, V, THREADS, S)                                                                 \
  add_deltas_kernel<T, V, THREADS, S><<<n, THREADS, 0, s>>>(resid, d1, splits1, d2, splits2,     \
                                                            static_cast<T*>(cast), hidden, stride)
  if (dtype == kF32) SHK_ROW_FORMS(SHK_GO, float);
  else SHK_ROW_FORMS(SHK_GO, bf16);
#undef SHK_GO
  SHK_LAUNCH_CHECK("add_deltas");
  return 0;
}

extern "C" int shk_add_normed_rmsnorm(float* resid, const void* delta, int delta_splits,
                                      const float* dweight, float deps, const float* weight, float eps,
                                      void* out, int dtype, const int32_t* rows, int n, int hidden,
                                      int write_resid, int resid_rows, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_normed_rmsnorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && delta_splits >= 0 && resid_rows >= 0,
              "add_normed_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
  SHK_REQUIRE(deps > 0.f && (!out || eps > 0.f), "add_normed_rmsnorm: eps must be > 0");
  if (n == 0) return 0;
  SHK_REQUIRE(resid && delta && dweight && (!out || weight), "add_normed_rmsnorm: null pointer");
  SHK_REQUIRE(out || write_resid, "add_normed_rmsnorm: nothing to write");
  const int form = row_form(hidden, aligned16(resid) && aligned16(delta) && aligned16(dweight) &&
                                        aligned16(weight) && aligned16(out));
  SHK_REQUIRE(form != 0, "add_normed_rmsnorm: rows of %d elements are too wide", hidden);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t stride = static_cast<size_t>(resid_rows) * hidden;
#define SHK_GO(T, V, THREADS, S)                                                                      \
  add_normed_rmsnorm_kernel<T, V, THREADS, S><<<n, THREADS, 0, s>>>(                                   \
      resid, delta, delta_splits, dweight, deps, weight, eps, static_cast<T*>(out), rows, hidden,      \
      write_resid, stride)
  if (dtype == kF32) SHK_ROW_FORMS(SHK_GO, float);
  else SHK_ROW_FORMS(SHK_GO, bf16);
#undef SHK_GO
  SHK_LAUNCH_CHECK("add_normed_rmsnorm");
  return 0;
}

extern "C" int shk_act_mul_rows(const void* a, int a_splits, const void* table, int dtype,
                                const int32_t* ids, long long ld, int offset, int table_rows, void* out,
                                int n, int width, int act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "act_mul_rows: unknown dtype %d", dtype);
  SHK_REQUIRE(act == 1 || act == 2, "act_mul_rows: unknown activation %d", act);
  SHK_REQUIRE(n >= 0 && width > 0 && offset >= 0 && ld >= offset + width && table_rows > 0 && a_splits >= 0,
              "act_mul_rows: bad sizes n=%d width=%d offset=%d ld=%lld", n, width, offset, ld);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "act_mul_rows: at most 65535 rows a call, got %d", n);
  SHK_REQUIRE(a && table && ids && out, "act_mul_rows: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = width >= 256 ? 256 : 64;
  const size_t stride = static_cast<size_t>(n) * width;
  dim3 grid((width + threads - 1) / threads, n);
  if (dtype == kF32)
    act_mul_rows_kernel<float><<<grid, threads, 0, s>>>(a, a_splits, stride, static_cast<const float*>(table),
                                                        ids, ld, offset, static_cast<float*>(out), width, act);
  else
    act_mul_rows_kernel<bf16><<<grid, threads, 0, s>>>(a, a_splits, stride, static_cast<const bf16*>(table),
                                                       ids, ld, offset, static_cast<bf16*>(out), width, act);
  SHK_LAUNCH_CHECK("act_mul_rows");
  return 0;
}

// ------------------------------------------------------------------ xIELU
// out = a_pos z^2 + z / 2 for z > 0, a_neg (exp(z) - 1 - z) + z / 2 for z <= 0: an
// activation with a quadratic positive branch and a negative branch that flattens out;
// the two factors are the layer's own (learned), given as they are applied.
namespace shk {
template <typename T>
__global__ void xielu_kernel(const T* __restrict__ x, T* __restrict__ out, long long numel, float a_pos, float a_neg) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= numel) return;
  const float z = to_float(x[i]);
  const float y = z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(a_neg, expm1f(z) - z, 0.5f * z);
  out[i] = from_float<T>(y);
}
}  // namespace shk

namespace shk {
// eight bfloat16 values a thread (16 bytes in, 16 bytes out)
__global__ void xielu_vec_kernel(const uint4* __restrict__ x, uint4* __restrict__ out, long long vecs, float a_pos,
                                 float a_neg) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= vecs) return;
  const uint4 raw = x[i];
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float z[2] = {__uint_as_float(w[e] << 16), __uint_as_float(w[e] & 0xffff0000u)};
#pragma unroll
    for (int h = 0; h < 2; ++h)
      z[h] = z[h] > 0.f ? fmaf(a_pos * z[h], z[h], 0.5f * z[h]) : fmaf(a_neg, expm1f(z[h]) - z[h], 0.5f * z[h]);
    r[e] = bf16_bits(z[0]) | (static_cast<uint32_t>(bf16_bits(z[1])) << 16);
  }
  out[i] = make_uint4(r[0], r[1], r[2], r[3]);
}
}  // namespace shk

extern "C" int shk_xielu(const void* x, void* out, int dtype, long long numel, float a_pos, float a_neg, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "xielu: unknown dtype %d", dtype);
  SHK_REQUIRE(numel >= 0 && numel < (1LL << 31) * 256, "xielu: bad size %lld", numel);
  if (numel == 0) return 0;
  SHK_REQUIRE(x && out, "xielu: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kBF16 && numel % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const long long vecs = numel / 8;
    shk::xielu_vec_kernel<<<static_cast<unsigned>((vecs + 255) / 256), 256, 0, s>>>(
        static_cast<const uint4*>(x), static_cast<uint4*>(out), vecs, a_pos, a_neg);
    SHK_LAUNCH_CHECK("xielu");
    return 0;
  }
  const unsigned grid = static_cast<unsigned>((numel + 255) / 256);
  if (dtype == kF32)
    shk::xielu_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), static_cast<float*>(out), numel, a_pos, a_neg);
  else
    shk::xielu_kernel<shk::bf16><<<grid, 256, 0, s>>>(static_cast<const shk::bf16*>(x), static_cast<shk::bf16*>(out), numel, a_pos, a_neg);
  SHK_LAUNCH_CHECK("xielu");
  return 0;
}
