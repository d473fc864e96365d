// A stream that is normed after every sum, and small row-wise helpers of the sublayers
// around it.
//
// postnorm_kernel        x <- rmsnorm(alpha * x + lscale * delta) * weight, the stream kept in
//                        float32 and left a second time in the compute dtype for the products
//                        that read it next; one workgroup per row, the row held in registers
//                        (rows of up to 8192 elements in multiples of 4) or in LDS
// cast_rows_kernel       the float32 stream in the compute dtype
// activate_kernel        an activation of a plain product, elementwise
// gate_mul_kernel        x * sigmoid(gate), elementwise
// All arithmetic is float32.
#include <initializer_list>

#include "api.h"
#include "common.h"

namespace shk {

namespace {

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16* p, float4 v) {
  uint2 u;
  u.x = bf16_bits(v.x) | (static_cast<uint32_t>(bf16_bits(v.y)) << 16);
  u.y = bf16_bits(v.z) | (static_cast<uint32_t>(bf16_bits(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

constexpr int kPostVecs = 2;  // float4 per thread

// TD: the type of delta, T, or float for the partial sums [splits][n][hidden] of a split product
template <typename T, typename TD, int THREADS>
__global__ void __launch_bounds__(THREADS)
    postnorm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta, int splits, size_t split_stride,
                        float alpha, const float* __restrict__ lscale, const float* __restrict__ weight, float eps,
                        T* __restrict__ cast, int hidden) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  float* x = resid + row * hidden;
  const TD* d = delta ? delta + row * hidden : nullptr;  // (null: nothing is added)
  const int nvec = hidden / 4;
  float4 v[kPostVecs], dv[kPostVecs], w[kPostVecs], ls[kPostVecs];
#pragma unroll
  for (int i = 0; i < kPostVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    v[i] = dv[i] = w[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    ls[i] = make_float4(1.f, 1.f, 1.f, 1.f);
    if (c < nvec) {
      v[i] = ld4(x + c * 4);
      if (d) dv[i] = ld4(d + c * 4);
      w[i] = ld4(weight + c * 4);
      if (lscale) ls[i] = ld4(lscale + c * 4);
    }
  }
  for (int z = 1; z < splits; ++z)  // further parts, added in order
#pragma unroll
    for (int i = 0; i < kPostVecs; ++i) {
      const int c = threadIdx.x + i * THREADS;
      if (c < nvec) {
        const float4 more = ld4(d + z * split_stride + c * 4);
        dv[i].x += more.x, dv[i].y += more.y, dv[i].z += more.z, dv[i].w += more.w;
      }
    }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kPostVecs; ++i) {
    v[i].x = fmaf(alpha, v[i].x, ls[i].x * dv[i].x);
    v[i].y = fmaf(alpha, v[i].y, ls[i].y * dv[i].y);
    v[i].z = fmaf(alpha, v[i].z, ls[i].z * dv[i].z);
    v[i].w = fmaf(alpha, v[i].w, ls[i].w * dv[i].w);
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int i = 0; i < kPostVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
    const float4 y = make_float4((v[i].x * inv) * w[i].x, (v[i].y * inv) * w[i].y, (v[i].z * inv) * w[i].z,
                                 (v[i].w * inv) * w[i].w);
    st4(x + c * 4, y);
    if (cast) st4(cast + row * hidden + c * 4, y);
  }
}

template <typename T, typename TD>
__global__ void __launch_bounds__(256)
    postnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta, int splits, size_t split_stride, float alpha,
                    const float* __restrict__ lscale, const float* __restrict__ weight, float eps, T* __restrict__ cast,
                    int hidden) {
  extern __shared__ float sums[];  // the row's sums before the norm
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  float* x = resid + row * hidden;
  const TD* d = delta ? delta + row * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float add = d ? to_float(d[i]) : 0.f;
    for (int z = 1; z < splits; ++z) add += to_float(d[z * split_stride + i]);
    const float v = fmaf(alpha, x[i], (lscale ? lscale[i] : 1.f) * add);
    sums[i] = v;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float y = (sums[i] * inv) * weight[i];
    x[i] = y;
    if (cast) cast[row * hidden + i] = from_float<T>(y);
  }
}

// eight elements a thread in 16-byte pieces where the arrays allow it (V = 8), else one (V = 1)
template <typename T, int V>
__device__ __forceinline__ void load_run(const T* p, float (&x)[V]) {
  if constexpr (V == 1) {
    x[0] = to_float(p[0]);
  } else {
    const float4 a = ld4(p), b = ld4(p + 4);
    x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
  }
}
template <typename T, int V>
__device__ __forceinline__ void store_run(T* p, const float (&x)[V]) {
  if constexpr (V == 1) {
    p[0] = from_float<T>(x[0]);
  } else {
    st4(p, make_float4(x[0], x[1], x[2], x[3]));
    st4(p + 4, make_float4(x[4], x[5], x[6], x[7]));
  }
}

template <typename T, int V>
__global__ void cast_rows_kernel(const float* __restrict__ src, T* __restrict__ dst, long long numel) {
  const long long i = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= numel) return;
  float x[V];
  load_run<float, V>(src + i, x);
  store_run<T, V>(dst + i, x);
}

// 1: SiLU, 2: GELU (tanh form), 3: ReLU, 4: the square of ReLU
__device__ __forceinline__ float plain_act(float z, int act) {
  if (act == 3) return fmaxf(z, 0.f);
  if (act == 4) {
    const float r = fmaxf(z, 0.f);
    return r * r;
  }
  const float u = act == 2 ? 2.f * 0.7978845608028654f * (z + 0.044715f * z * z * z) : z;
  return z / (1.f + expf(-u));
}

template <typename T, int V>
__global__ void activate_kernel(const T* __restrict__ x, T* __restrict__ out, long long numel, int act) {
  const long long i = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= numel) return;
  float v[V];
  load_run<T, V>(x + i, v);
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = plain_act(v[e], act);
  store_run<T, V>(out + i, v);
}

template <typename T, int V>
__global__ void gate_mul_kernel(const T* __restrict__ x, const T* __restrict__ gate, T* __restrict__ out,
                                long long numel) {
  const long long i = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= numel) return;
  float v[V], g[V];
  load_run<T, V>(x + i, v);
  load_run<T, V>(gate + i, g);
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = v[e] / (1.f + expf(-g[e]));
  store_run<T, V>(out + i, v);
}

inline bool runs_of_eight(long long numel, std::initializer_list<const void*> arrays) {
  if (numel % 8) return false;
  for (const void* p : arrays)
    if (reinterpret_cast<uintptr_t>(p) % 16) return false;
  return true;
}

}  // namespace

}  // namespace shk

using namespace shk;

extern "C" int shk_postnorm(float* resid, const void* delta, int delta_splits, float alpha, const float* lscale,
                            const float* weight, float eps, void* cast, int dtype, int n, int hidden, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "postnorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && delta_splits >= 0, "postnorm: bad sizes n=%d hidden=%d splits=%d", n, hidden,
              delta_splits);
  SHK_REQUIRE(hidden <= 15000, "postnorm: rows of %d elements do not fit a workgroup's LDS", hidden);
  if (n == 0) return 0;
  SHK_REQUIRE(resid && weight && (delta || delta_splits == 0), "postnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t stride = static_cast<size_t>(n) * hidden;
  const bool vec = hidden % 4 == 0 && hidden <= 8192;
  const bool wide = hidden > 2048;
#define SHK_GO(T, TD)                                                                                             \
  do {                                                                                                            \
    if (vec && wide)                                                                                              \
      postnorm_vec_kernel<T, TD, 1024><<<n, 1024, 0, s>>>(resid, static_cast<const TD*>(delta), delta_splits, stride, \
                                                          alpha, lscale, weight, eps, static_cast<T*>(cast), hidden); \
    else if (vec)                                                                                                 \
      postnorm_vec_kernel<T, TD, 256><<<n, 256, 0, s>>>(resid, static_cast<const TD*>(delta), delta_splits, stride,  \
                                                        alpha, lscale, weight, eps, static_cast<T*>(cast), hidden);  \
    else                                                                                                          \
      postnorm_kernel<T, TD><<<n, 256, hidden * sizeof(float), s>>>(resid, static_cast<const TD*>(delta),         \
                                                                    delta_splits, stride, alpha, lscale, weight,  \
                                                                    eps, static_cast<T*>(cast), hidden);          \
  } while (0)
  if (delta_splits > 0) {
    if (dtype == kF32) SHK_GO(float, float); else SHK_GO(bf16, float);
  } else {
    if (dtype == kF32) SHK_GO(float, float); else SHK_GO(bf16, bf16);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("postnorm");
  return 0;
}

extern "C" int shk_cast_rows(const float* src, void* dst, int dtype, long long numel, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "cast_rows: unknown dtype %d", dtype);
  SHK_REQUIRE(numel >= 0 && numel < (1LL << 40), "cast_rows: bad size %lld", numel);
  if (numel == 0) return 0;
  SHK_REQUIRE(src && dst, "cast_rows: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SHK_GO(T, V) \
  cast_rows_kernel<T, V><<<static_cast<unsigned>((numel / V + 255) / 256), 256, 0, s>>>(src, static_cast<T*>(dst), numel)
  const bool eight = runs_of_eight(numel, {src, dst});
  if (dtype == kF32) {
    if (eight) SHK_GO(float, 8); else SHK_GO(float, 1);
  } else {
    if (eight) SHK_GO(bf16, 8); else SHK_GO(bf16, 1);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("cast_rows");
  return 0;
}

extern "C" int shk_activate(const void* x, void* out, int dtype, long long numel, int act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "activate: unknown dtype %d", dtype);
  SHK_REQUIRE(act >= 1 && act <= 4, "activate: unknown activation %d", act);
  SHK_REQUIRE(numel >= 0 && numel < (1LL << 40), "activate: bad size %lld", numel);
  if (numel == 0) return 0;
  SHK_REQUIRE(x && out, "activate: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SHK_GO(T, V)                                                                                     \
  activate_kernel<T, V><<<static_cast<unsigned>((numel / V + 255) / 256), 256, 0, s>>>(static_cast<const T*>(x), \
                                                                                        static_cast<T*>(out), numel, act)
  const bool eight = runs_of_eight(numel, {x, out});
  if (dtype == kF32) {
    if (eight) SHK_GO(float, 8); else SHK_GO(float, 1);
  } else {
    if (eight) SHK_GO(bf16, 8); else SHK_GO(bf16, 1);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("activate");
  return 0;
}

extern "C" int shk_gate_mul(const void* x, const void* gate, void* out, int dtype, long long numel, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "gate_mul: unknown dtype %d", dtype);
  SHK_REQUIRE(numel >= 0 && numel < (1LL << 40), "gate_mul: bad size %lld", numel);
  if (numel == 0) return 0;
  SHK_REQUIRE(x && gate && out, "gate_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SHK_GO(T, V)                                                                                             \
  gate_mul_kernel<T, V><<<static_cast<unsigned>((numel / V + 255) / 256), 256, 0, s>>>(                          \
      static_cast<const T*>(x), static_cast<const T*>(gate), static_cast<T*>(out), numel)
  const bool eight = runs_of_eight(numel, {x, gate, out});
  if (dtype == kF32) {
    if (eight) SHK_GO(float, 8); else SHK_GO(float, 1);
  } else {
    if (eight) SHK_GO(bf16, 8); else SHK_GO(bf16, 1);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("gate_mul");
  return 0;
}
