// A routed mixture of gated feed-forward experts.
//
//   scores s = softmax(router logits) over all experts (float32);
//   the `top` experts with the largest s + correction are chosen (the lowest index wins a tie);
//   their weights are their s divided by the chosen experts' sum (+ 1e-20);
//   out = sum over the chosen of weight * W_down_e (act(W_gate_e x) * (W_up_e x))  (+ what a
//   shared expert gave).
//
// moe_route_kernel     a wavefront per token
// moe_gate_up_kernel   a workgroup per (token, chosen expert, block of features): every
//                      (token, expert) pair is a product of its own, summed in one fixed
//                      order, so a token's result does not depend on what else is in the step
// moe_down_kernel      a workgroup per (token, block of columns): the chosen experts'
//                      outputs, weighted and added in the order they were chosen
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kMaxExpertsPerLane = 8;  // experts <= 512

__global__ void __launch_bounds__(256)
    moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction, int experts,
                     int top, int32_t* __restrict__ chosen, float* __restrict__ weights, int n) {
  const int t = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (t >= n) return;
  float s[kMaxExpertsPerLane], c[kMaxExpertsPerLane];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    const int e = lane + i * kWave;
    s[i] = e < experts ? logits[static_cast<size_t>(t) * ld + e] : -INFINITY;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    const int e = lane + i * kWave;
    s[i] = e < experts ? expf(s[i] - mx) : 0.f;
    sum += s[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    const int e = lane + i * kWave;
    s[i] /= sum;
    c[i] = e < experts ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  float picked_sum = 0.f, my_score = 0.f;
  int my_expert = 0;
  for (int k = 0; k < top; ++k) {
    // the largest choice score not yet taken; of equal ones the lowest index
    float best = -INFINITY;
    int best_e = 1 << 30;
#pragma unroll
    for (int i = 0; i < kMaxExpertsPerLane; ++i) {
      const int e = lane + i * kWave;
      if (c[i] > best) {  // ascending e within a lane: the first of equal ones stays
        best = c[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave);
      const int oe = __shfl_xor(best_e, off, kWave);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    if (best_e >= experts) {
      // no score compares (logits that are not numbers): the lowest expert not yet taken, so
      // that what is written is always an expert's index
      best_e = 1 << 30;
#pragma unroll
      for (int i = 0; i < kMaxExpertsPerLane; ++i) {
        const int e = lane + i * kWave;
        if (e < experts && !(c[i] == -INFINITY) && e < best_e) best_e = e;
      }
#pragma unroll
      for (int off = kWave / 2; off > 0; off >>= 1) {
        const int oe = __shfl_xor(best_e, off, kWave);
        best_e = oe < best_e ? oe : best_e;
      }
      if (best_e >= experts) best_e = k;  // (cannot happen while top <= experts)
    }
    float score = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxExpertsPerLane; ++i) {
      if (lane + i * kWave == best_e) {
        score = s[i];
        c[i] = -INFINITY;
      }
    }
    score = wave_sum(score);  // one lane holds it
    picked_sum += score;
    if (lane == k) {  // lane k keeps the k-th choice
      my_expert = best_e;
      my_score = score;
    }
  }
  if (lane < top) {
    chosen[static_cast<size_t>(t) * top + lane] = my_expert;
    weights[static_cast<size_t>(t) * top + lane] = my_score / (picked_sum + 1e-20f);
  }
}

__device__ __forceinline__ float gate_act(float g, int act) {
  const float x = act == 2 ? 2.f * 0.7978845608028654f * (g + 0.044715f * g * g * g) : g;
  return g / (1.f + expf(-x));
}

constexpr int kMoeFeatures = 32;  // features (or columns) a workgroup

template <typename T>
__global__ void __launch_bounds__(256)
    moe_gate_up_kernel(const T* __restrict__ x, const int32_t* __restrict__ chosen, const T* __restrict__ wg,
                       const T* __restrict__ wu, T* __restrict__ act_out, int width, int ff, int top, int act,
                       int experts) {
  extern __shared__ float xs[];
  const int pair = blockIdx.y, t = pair / top;
  const int e = min(max(chosen[pair], 0), experts - 1);  // an index from memory never leaves the stack of experts
  for (int k = threadIdx.x; k < width; k += 256) xs[k] = to_float(x[static_cast<size_t>(t) * width + k]);
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  for (int i = wave; i < kMoeFeatures; i += 256 / kWave) {
    const int f = blockIdx.x * kMoeFeatures + i;
    if (f >= ff) break;
    const T* gr = wg + (static_cast<size_t>(e) * ff + f) * width;
    const T* ur = wu + (static_cast<size_t>(e) * ff + f) * width;
    float g = 0.f, u = 0.f;
    for (int k = lane; k < width; k += kWave) {
      g = fmaf(to_float(gr[k]), xs[k], g);
      u = fmaf(to_float(ur[k]), xs[k], u);
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) act_out[static_cast<size_t>(pair) * ff + f] = from_float<T>(gate_act(g, act) * u);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
    moe_down_kernel(const T* __restrict__ act_in, const int32_t* __restrict__ chosen,
                    const float* __restrict__ weights, const T* __restrict__ wd, const T* __restrict__ add,
                    T* __restrict__ out, int width, int ff, int top, int experts) {
  extern __shared__ float as[];  // [top, ff]
  const int t = blockIdx.y;
  for (int i = threadIdx.x; i < top * ff; i += 256) as[i] = to_float(act_in[static_cast<size_t>(t) * top * ff + i]);
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  for (int i = wave; i < kMoeFeatures; i += 256 / kWave) {
    const int c = blockIdx.x * kMoeFeatures + i;
    if (c >= width) break;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = min(max(chosen[static_cast<size_t>(t) * top + k], 0), experts - 1);
      const T* dr = wd + (static_cast<size_t>(e) * width + c) * ff;
      float d = 0.f;
      for (int f = lane; f < ff; f += kWave) d = fmaf(to_float(dr[f]), as[k * ff + f], d);
      total = fmaf(weights[static_cast<size_t>(t) * top + k], wave_sum(d), total);
    }
    if (lane == 0) {
      if (add) total += to_float(add[static_cast<size_t>(t) * width + c]);
      out[static_cast<size_t>(t) * width + c] = from_float<T>(total);
    }
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_moe_route(const float* logits, int ld, const float* correction, int experts, int top,
                             int32_t* chosen, float* weights, int n, void* stream) {
  SHK_REQUIRE(n >= 0 && experts > 0 && experts <= kMaxExpertsPerLane * kWave && top >= 1 && top <= experts &&
                  top <= kWave && ld >= experts,
              "moe_route: bad sizes n=%d experts=%d top=%d", n, experts, top);
  if (n == 0) return 0;
  SHK_REQUIRE(logits && chosen && weights, "moe_route: null pointer");
  moe_route_kernel<<<(n + 3) / 4, 256, 0, static_cast<hipStream_t>(stream)>>>(logits, ld, correction, experts, top,
                                                                              chosen, weights, n);
  SHK_LAUNCH_CHECK("moe_route");
  return 0;
}

extern "C" int shk_moe_experts(const void* x, const int32_t* chosen, const float* weights, const void* w_gate,
                               const void* w_up, const void* w_down, const void* add, void* act_buf, void* out,
                               int dtype, int n, int width, int ff, int experts, int top, int act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_experts: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && width > 0 && ff > 0 && experts > 0 && top >= 1 && top <= experts,
              "moe_experts: bad sizes n=%d width=%d ff=%d experts=%d top=%d", n, width, ff, experts, top);
  SHK_REQUIRE(act == 1 || act == 2, "moe_experts: unknown activation %d", act);
  SHK_REQUIRE(width <= 15000 && static_cast<long long>(top) * ff <= 15000,
              "moe_experts: rows of %d, or %d chosen experts of %d features, do not fit a workgroup's LDS", width, top,
              ff);
  if (n == 0) return 0;
  SHK_REQUIRE(static_cast<long long>(n) * top <= 65535, "moe_experts: at most 65535 (token, expert) pairs a call");
  SHK_REQUIRE(x && chosen && weights && w_gate && w_up && w_down && act_buf && out, "moe_experts: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 g1((ff + kMoeFeatures - 1) / kMoeFeatures, n * top), g2((width + kMoeFeatures - 1) / kMoeFeatures, n);
#define SHK_GO(T)                                                                                                     \
  moe_gate_up_kernel<T><<<g1, 256, width * sizeof(float), s>>>(static_cast<const T*>(x), chosen,                      \
                                                               static_cast<const T*>(w_gate),                         \
                                                               static_cast<const T*>(w_up), static_cast<T*>(act_buf), \
                                                               width, ff, top, act, experts);                         \
  moe_down_kernel<T><<<g2, 256, static_cast<size_t>(top) * ff * sizeof(float), s>>>(                                  \
      static_cast<const T*>(act_buf), chosen, weights, static_cast<const T*>(w_down), static_cast<const T*>(add),     \
      static_cast<T*>(out), width, ff, top, experts)
  if (dtype == kF32) {
    SHK_GO(float);
  } else {
    SHK_GO(bf16);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("moe_experts");
  return 0;
}
