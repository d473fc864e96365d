// Layer norm with weight and bias around the float32 residual stream, the
// weighted sum of the streams that earlier layers left (a depth average), and
// the scaling and capping of logits.
//
// add_layernorm_kernel: one workgroup per row.  The row is held in LDS as
// float32; mean and variance are formed in two passes (the variance is the mean
// of the squared deviations), each sum in one fixed order, so a row's result
// does not depend on which other rows the call holds.  A product's output that
// is normed by itself before it joins the stream (a norm after the sublayer) is
// added in the same pass, and the norm that follows reads the sum.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kLnThreads = 256;

// (mean, 1 / sqrt(var + eps)) of the `hidden` floats in LDS at `x`
__device__ __forceinline__ void row_moments(const float* x, int hidden, float eps, float* scratch, float& mean,
                                            float& inv) {
  float s = 0.f;
  for (int c = threadIdx.x; c < hidden; c += kLnThreads) s += x[c];
  mean = block_sum(s, scratch) / static_cast<float>(hidden);
  float v = 0.f;
  for (int c = threadIdx.x; c < hidden; c += kLnThreads) {
    const float d = x[c] - mean;
    v = fmaf(d, d, v);
  }
  inv = 1.f / sqrtf(block_sum(v, scratch) / static_cast<float>(hidden) + eps);
}

template <typename T>
__global__ void __launch_bounds__(kLnThreads)
    add_layernorm_kernel(float* __restrict__ resid, const void* __restrict__ delta, int splits, size_t split_stride,
                         const float* __restrict__ dweight, const float* __restrict__ dbias, float deps,
                         const float* __restrict__ weight, const float* __restrict__ bias, float eps,
                         void* __restrict__ out, int out_f32, const int32_t* __restrict__ rows, int hidden,
                         int write_resid) {
  extern __shared__ float lds[];
  float* x = lds;            // the stream's row
  float* d = lds + hidden;   // the addend's row
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  for (int c = threadIdx.x; c < hidden; c += kLnThreads) x[c] = resid[row * hidden + c];
  if (delta) {
    for (int c = threadIdx.x; c < hidden; c += kLnThreads) {
      float v = 0.f;
      if (splits == 0) {
        v = to_float(static_cast<const T*>(delta)[row * hidden + c]);
      } else {
        const float* p = static_cast<const float*>(delta) + row * hidden + c;
        for (int z = 0; z < splits; ++z) v += p[z * split_stride];
      }
      d[c] = v;
    }
    __syncthreads();
    if (dweight) {
      float mean, inv;
      row_moments(d, hidden, deps, scratch, mean, inv);
      for (int c = threadIdx.x; c < hidden; c += kLnThreads)
        x[c] += (d[c] - mean) * inv * dweight[c] + (dbias ? dbias[c] : 0.f);
    } else {
      for (int c = threadIdx.x; c < hidden; c += kLnThreads) x[c] += d[c];
    }
    if (write_resid)
      for (int c = threadIdx.x; c < hidden; c += kLnThreads) resid[row * hidden + c] = x[c];
  }
  if (!out) return;
  __syncthreads();
  float mean, inv;
  row_moments(x, hidden, eps, scratch, mean, inv);
  for (int c = threadIdx.x; c < hidden; c += kLnThreads) {
    const float y = (x[c] - mean) * inv * weight[c] + (bias ? bias[c] : 0.f);
    if (out_f32) static_cast<float*>(out)[static_cast<size_t>(r) * hidden + c] = y;
    else static_cast<T*>(out)[static_cast<size_t>(r) * hidden + c] = from_float<T>(y);
  }
}

// out[r, :] = sum_j coef[j] * history[j][r, :], j < count, added in ascending j.  When a
// product's output is still to join the newest stream (history[count - 1]), normed by itself
// with weight and bias, it is added there first and stored back.
template <typename T>
__global__ void __launch_bounds__(kLnThreads)
    mix_history_kernel(float* __restrict__ history, size_t stride, const float* __restrict__ coef, int count,
                       float* __restrict__ out, int hidden, const void* __restrict__ delta, int splits,
                       size_t split_stride, const float* __restrict__ dweight, const float* __restrict__ dbias,
                       float deps) {
  extern __shared__ float lds[];
  float* d = lds;
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  float mean = 0.f, inv = 0.f;
  if (delta) {
    for (int c = threadIdx.x; c < hidden; c += kLnThreads) {
      float v = 0.f;
      if (splits == 0) {
        v = to_float(static_cast<const T*>(delta)[row * hidden + c]);
      } else {
        const float* p = static_cast<const float*>(delta) + row * hidden + c;
        for (int z = 0; z < splits; ++z) v += p[z * split_stride];
      }
      d[c] = v;
    }
    __syncthreads();
    row_moments(d, hidden, deps, scratch, mean, inv);
  }
  // With few rows a row's columns are shared among gridDim.y workgroups (each forms the addend's
  // moments for itself).  The entries that are only read are fetched four at a time; the sum runs
  // over j in ascending order either way.
  const int per = (hidden + gridDim.y - 1) / gridDim.y;
  const int c_end = min(hidden, static_cast<int>(blockIdx.y + 1) * per);
  const int reads = delta ? count - 1 : count;
  for (int c = blockIdx.y * per + threadIdx.x; c < c_end; c += kLnThreads) {
    const float* base = history + row * hidden + c;
    float acc = 0.f;
    int j = 0;
    for (; j + 4 <= reads; j += 4) {
      const float v0 = base[j * stride], v1 = base[(j + 1) * stride], v2 = base[(j + 2) * stride],
                  v3 = base[(j + 3) * stride];
      acc = fmaf(coef[j], v0, acc);
      acc = fmaf(coef[j + 1], v1, acc);
      acc = fmaf(coef[j + 2], v2, acc);
      acc = fmaf(coef[j + 3], v3, acc);
    }
    for (; j < reads; ++j) acc = fmaf(coef[j], base[j * stride], acc);
    if (delta) {
      float* at = history + (count - 1) * stride + row * hidden + c;
      const float v = *at + ((d[c] - mean) * inv * dweight[c] + (dbias ? dbias[c] : 0.f));
      *at = v;
      acc = fmaf(coef[count - 1], v, acc);
    }
    out[row * hidden + c] = acc;
  }
}

__global__ void __launch_bounds__(256)
    scale_softcap_kernel(float* __restrict__ x, long long numel, float scale, float cap) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= numel) return;
  float v = x[i] * scale;
  if (cap > 0.f) v = cap * tanhf(v / cap);
  x[i] = v;
}

}  // namespace shk

using namespace shk;

extern "C" int shk_add_layernorm(float* resid, const void* delta, int delta_splits, const float* dweight,
                                 const float* dbias, float deps, const float* weight, const float* bias, float eps,
                                 void* out, int dtype, int out_f32, const int32_t* rows, int n, int hidden,
                                 int write_resid, int resid_rows, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_layernorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && hidden <= 16384 && delta_splits >= 0 && resid_rows >= 0,
              "add_layernorm: bad sizes n=%d hidden=%d", n, hidden);
  SHK_REQUIRE((!delta || !dweight || deps > 0.f) && (!out || eps > 0.f), "add_layernorm: eps must be > 0");
  if (n == 0) return 0;
  SHK_REQUIRE(resid && (!out || weight), "add_layernorm: null pointer");
  SHK_REQUIRE(out || (delta && write_resid), "add_layernorm: nothing to write");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t stride = static_cast<size_t>(resid_rows) * hidden;
  const size_t lds = 2 * static_cast<size_t>(hidden) * sizeof(float);
  if (dtype == kF32)
    add_layernorm_kernel<float><<<n, kLnThreads, lds, s>>>(resid, delta, delta_splits, stride, dweight, dbias, deps,
                                                           weight, bias, eps, out, out_f32, rows, hidden, write_resid);
  else
    add_layernorm_kernel<bf16><<<n, kLnThreads, lds, s>>>(resid, delta, delta_splits, stride, dweight, dbias, deps,
                                                          weight, bias, eps, out, out_f32, rows, hidden, write_resid);
  SHK_LAUNCH_CHECK("add_layernorm");
  return 0;
}

extern "C" int shk_mix_history(float* history, long long stride, const float* coef, int count, float* out, int n,
                               int hidden, const void* delta, int delta_splits, const float* dweight,
                               const float* dbias, float deps, int dtype, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "mix_history: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && hidden <= 16384 && count >= 1 && stride >= static_cast<long long>(n) * hidden &&
                  delta_splits >= 0,
              "mix_history: bad sizes n=%d hidden=%d count=%d", n, hidden, count);
  if (n == 0) return 0;
  SHK_REQUIRE(history && coef && out, "mix_history: null pointer");
  SHK_REQUIRE(!delta || (dweight && deps > 0.f), "mix_history: an addend comes with its norm's weight and eps");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = static_cast<size_t>(hidden) * sizeof(float);
  const size_t split_stride = static_cast<size_t>(n) * hidden;
  const dim3 grid(n, n < 64 && hidden >= 8 * kLnThreads ? 8 : 1);
  if (dtype == kF32)
    mix_history_kernel<float><<<grid, kLnThreads, lds, s>>>(history, static_cast<size_t>(stride), coef, count, out, hidden,
                                                         delta, delta_splits, split_stride, dweight, dbias, deps);
  else
    mix_history_kernel<bf16><<<grid, kLnThreads, lds, s>>>(history, static_cast<size_t>(stride), coef, count, out, hidden,
                                                        delta, delta_splits, split_stride, dweight, dbias, deps);
  SHK_LAUNCH_CHECK("mix_history");
  return 0;
}

extern "C" int shk_scale_softcap(float* x, long long numel, float scale, float cap, void* stream) {
  SHK_REQUIRE(numel >= 0 && numel < (1LL << 31) * 256 && cap >= 0.f, "scale_softcap: bad arguments");
  if (numel == 0) return 0;
  SHK_REQUIRE(x, "scale_softcap: null pointer");
  scale_softcap_kernel<<<static_cast<unsigned>((numel + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      x, numel, scale, cap);
  SHK_LAUNCH_CHECK("scale_softcap");
  return 0;
}
