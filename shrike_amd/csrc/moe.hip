// A routed mixture of gated feed-forward experts.
//
//   scores s = softmax(router logits) over all experts (float32);
//   the `top` experts with the largest s + correction are chosen (the lowest index wins a tie);
//   their weights are their s divided by the chosen experts' sum (+ 1e-20);
//   out = sum over the chosen of weight * W_down_e (act(W_gate_e x) * (W_up_e x))  (+ what a
//   shared expert gave, times sigmoid of a number per token where the design gates it).
//   Experts without a gate whose activation is the square of ReLU are the same with ReLU as act and
//   their one matrix in both places: relu(u) * u; the kernels then form that product once.
//
// moe_route_kernel     a wavefront per token
// moe_gate_up_kernel   a workgroup per (token, chosen expert, block of features): every
//                      (token, expert) pair is a product of its own, summed in one fixed
//                      order, so a token's result does not depend on what else is in the step
// moe_down_kernel      a workgroup per (token, block of columns): the chosen experts'
//                      outputs, weighted and added in the order they were chosen
//
// On the matrix units (bfloat16, many tokens): the (token, expert) pairs are listed per expert
// in the order of the tokens (moe_lists_kernel, a workgroup per expert), and the two products
// run per expert over its list in tiles of 32 pairs (v_mfma_f32_16x16x32_bf16, both operands
// row-major with k innermost and loaded as operands straight from memory).  Workgroups beyond
// an expert's list leave at once, so the grid depends on the step's size alone.  A pair's
// sums run over k in one fixed order wherever the pair stands in its list; the pairs' outputs
// are kept in float32 and joined per token in the order the experts were chosen.
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
  if (act == 3) return fmaxf(g, 0.f);  // ReLU; with the gate's matrix also the other factor's, the square of ReLU
  const float x = act == 2 ? 2.f * 0.7978845608028654f * (g + 0.044715f * g * g * g) : g;
  return g / (1.f + expf(-x));
}

// What multiplies the shared expert's output for token t: sigmoid(add_gate[t * gate_ld]), one number
// per token, or 1 without such a gate.
__device__ __forceinline__ float shared_share(const float* __restrict__ add_gate, int gate_ld, int t) {
  return add_gate ? 1.f / (1.f + expf(-add_gate[static_cast<size_t>(t) * gate_ld])) : 1.f;
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
    if (wg == wu) {  // experts without a gate: the one product is both factors
      for (int k = lane; k < width; k += kWave) g = fmaf(to_float(gr[k]), xs[k], g);
      g = u = wave_sum(g);
    } else {
      for (int k = lane; k < width; k += kWave) {
        g = fmaf(to_float(gr[k]), xs[k], g);
        u = fmaf(to_float(ur[k]), xs[k], u);
      }
      g = wave_sum(g);
      u = wave_sum(u);
    }
    if (lane == 0) act_out[static_cast<size_t>(pair) * ff + f] = from_float<T>(gate_act(g, act) * u);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
    moe_down_kernel(const T* __restrict__ act_in, const int32_t* __restrict__ chosen,
                    const float* __restrict__ weights, const T* __restrict__ wd, const T* __restrict__ add,
                    const float* __restrict__ add_gate, int gate_ld, T* __restrict__ out, int width, int ff, int top,
                    int experts) {
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
      if (add) total += shared_share(add_gate, gate_ld, t) * to_float(add[static_cast<size_t>(t) * width + c]);
      out[static_cast<size_t>(t) * width + c] = from_float<T>(total);
    }
  }
}

typedef __bf16 mbf16x8 __attribute__((ext_vector_type(8)));
typedef float mf32x4 __attribute__((ext_vector_type(4)));

// order[e * n + r] = the r-th pair (token * top + place among the token's choices) of expert e,
// tokens ascending; counts[e] = how many there are
__global__ void __launch_bounds__(256)
    moe_lists_kernel(const int32_t* __restrict__ chosen, int n, int top, int32_t* __restrict__ order,
                     int32_t* __restrict__ counts) {
  __shared__ int wave_total[256 / kWave];
  const int e = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  int base = 0;
  for (int t0 = 0; t0 < n; t0 += 256) {
    const int t = t0 + threadIdx.x;
    int hit = -1;
    if (t < n)
      for (int k = top - 1; k >= 0; --k)
        if (chosen[static_cast<size_t>(t) * top + k] == e) hit = k;
    const unsigned long long votes = __ballot(hit >= 0);
    const int before = __popcll(votes & ((1ull << lane) - 1ull));
    if (lane == 0) wave_total[wave] = __popcll(votes);
    __syncthreads();
    int prefix = 0, total = 0;
    for (int w = 0; w < 256 / kWave; ++w) {
      if (w < wave) prefix += wave_total[w];
      total += wave_total[w];
    }
    if (hit >= 0) order[static_cast<size_t>(e) * n + base + prefix + before] = t * top + hit;
    base += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) counts[e] = base;
}

// act[pair, f] = act(W_gate_e[f] . x_t) * (W_up_e[f] . x_t) for the pairs of expert e's list: a workgroup
// takes 32 pairs and four wavefronts' 32 features each
__global__ void __launch_bounds__(256)
    moe_gate_up_mfma_kernel(const bf16* __restrict__ x, const int32_t* __restrict__ order,
                            const int32_t* __restrict__ counts, const bf16* __restrict__ wg,
                            const bf16* __restrict__ wu, bf16* __restrict__ act_out, int n, int width, int ff, int top,
                            int act) {
  const int e = blockIdx.z;
  const int count = min(counts[e], n);
  const int row0 = blockIdx.y * 32;
  if (row0 >= count) return;
  const bool single = wg == wu;  // experts without a gate: the one product is both factors
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int f0 = (blockIdx.x * 4 + wave) * 32;
  if (f0 >= ff) return;
  int pair[2];
  const bf16* xr[2];
  const bf16* gr[2];
  const bf16* ur[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int r = row0 + a * 16 + i;
    pair[a] = r < count ? order[static_cast<size_t>(e) * n + r] : -1;
    const int t = pair[a] >= 0 ? min(pair[a] / top, n - 1) : 0;
    xr[a] = x + static_cast<size_t>(t) * width + kg * 8;
    const int f = min(f0 + a * 16 + i, ff - 1);
    gr[a] = wg + (static_cast<size_t>(e) * ff + f) * width + kg * 8;
    ur[a] = wu + (static_cast<size_t>(e) * ff + f) * width + kg * 8;
  }
  mf32x4 accg[2][2], accu[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) accg[a][b] = accu[a][b] = mf32x4{0.f, 0.f, 0.f, 0.f};
  if (single) {
    // one matrix: four steps' operands are asked for at once (eight 16-byte pieces of weights a lane in
    // flight: few wavefronts run, and what they have in flight is what the memory delivers); the sums
    // still run over k in ascending order
    constexpr int kAhead = 4;
    for (int k0 = 0; k0 < width; k0 += 32 * kAhead) {
      uint4 av[kAhead][2], gv[kAhead][2];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int kk = k0 + 32 * u;
        const bool have = kk + kg * 8 < width;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          av[u][a] = gv[u][a] = make_uint4(0, 0, 0, 0);
          if (have) {
            gv[u][a] = *reinterpret_cast<const uint4*>(gr[a] + kk);
            if (pair[a] >= 0) av[u][a] = *reinterpret_cast<const uint4*>(xr[a] + kk);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kAhead; ++u)
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b)
            accg[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mbf16x8, gv[u][b]),
                                                                 __builtin_bit_cast(mbf16x8, av[u][a]), accg[a][b], 0, 0, 0);
    }
  } else {
    for (int k0 = 0; k0 < width; k0 += 32) {
      const bool have = k0 + kg * 8 < width;  // (width is a multiple of 8: a piece is whole or absent)
      uint4 av[2], gv[2], uv[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        av[a] = gv[a] = uv[a] = make_uint4(0, 0, 0, 0);
        if (have) {
          if (pair[a] >= 0) av[a] = *reinterpret_cast<const uint4*>(xr[a] + k0);
          gv[a] = *reinterpret_cast<const uint4*>(gr[a] + k0);
          uv[a] = *reinterpret_cast<const uint4*>(ur[a] + k0);
        }
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          accg[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mbf16x8, gv[b]),
                                                               __builtin_bit_cast(mbf16x8, av[a]), accg[a][b], 0, 0, 0);
          accu[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mbf16x8, uv[b]),
                                                               __builtin_bit_cast(mbf16x8, av[a]), accu[a][b], 0, 0, 0);
        }
    }
  }
  // features were the rows of the products: this lane holds features f0 + 16 b + 4 kg + r of pair row a * 16 + i
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    if (pair[a] < 0) continue;
    bf16* dst = act_out + static_cast<size_t>(pair[a]) * ff;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int f = f0 + b * 16 + 4 * kg + r;
        if (f < ff) dst[f] = from_float<bf16>(gate_act(accg[a][b][r], act) * (single ? accg[a][b][r] : accu[a][b][r]));
      }
  }
}

// pair_out[pair, c] = W_down_e[c] . act[pair]: a workgroup takes 32 pairs and four wavefronts' 64 columns each
__global__ void __launch_bounds__(256)
    moe_down_mfma_kernel(const bf16* __restrict__ act_in, const int32_t* __restrict__ order,
                         const int32_t* __restrict__ counts, const bf16* __restrict__ wd,
                         float* __restrict__ pair_out, int n, int width, int ff, int top) {
  const int e = blockIdx.z;
  const int count = min(counts[e], n);
  const int row0 = blockIdx.y * 32;
  if (row0 >= count) return;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int c0 = (blockIdx.x * 4 + wave) * 64;
  if (c0 >= width) return;
  int pair[2];
  const bf16* ar[2];
  const bf16* wr[4];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int r = row0 + a * 16 + i;
    pair[a] = r < count ? order[static_cast<size_t>(e) * n + r] : -1;
    const int p = pair[a] >= 0 ? min(pair[a], n * top - 1) : 0;
    ar[a] = act_in + static_cast<size_t>(p) * ff + kg * 8;
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int c = min(c0 + b * 16 + i, width - 1);
    wr[b] = wd + (static_cast<size_t>(e) * width + c) * ff + kg * 8;
  }
  mf32x4 acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = mf32x4{0.f, 0.f, 0.f, 0.f};
  // two steps' operands are asked for at once (eight 16-byte pieces of weights a lane in flight); the sums
  // run over k in ascending order all the same
  constexpr int kAhead = 2;
  for (int k0 = 0; k0 < ff; k0 += 32 * kAhead) {
    uint4 av[kAhead][2], wv[kAhead][4];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int kk = k0 + 32 * u;
      const bool have = kk + kg * 8 < ff;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        av[u][a] = make_uint4(0, 0, 0, 0);
        if (have && pair[a] >= 0) av[u][a] = *reinterpret_cast<const uint4*>(ar[a] + kk);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        wv[u][b] = make_uint4(0, 0, 0, 0);
        if (have) wv[u][b] = *reinterpret_cast<const uint4*>(wr[b] + kk);
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mbf16x8, wv[u][b]),
                                                              __builtin_bit_cast(mbf16x8, av[u][a]), acc[a][b], 0, 0, 0);
  }
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    if (pair[a] < 0) continue;
    float* dst = pair_out + static_cast<size_t>(pair[a]) * width;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int c = c0 + b * 16 + 4 * kg;
      if (c + 3 < width) {
        *reinterpret_cast<float4*>(dst + c) = make_float4(acc[a][b][0], acc[a][b][1], acc[a][b][2], acc[a][b][3]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (c + r < width) dst[c + r] = acc[a][b][r];
      }
    }
  }
}

// The same two products for lists of many pairs, tiled through LDS: a workgroup forms 128 pairs x 128
// weight rows (gate/up: 64 features of each; down: 128 columns) in steps of 32 along k.  The four
// wavefronts (2 x 2) take 64 x 64 each: four A and four B operands from LDS feed sixteen matrix
// instructions.  Rows of 32 elements lie 80 bytes apart in LDS, so the sixteen 16-byte reads of an
// operand meet every bank once.  The next step's pieces are fetched into registers while this one is
// multiplied.  Sums run over k in the same order as in the kernels above: the same bits.
constexpr int kTileRows = 128;
constexpr int kTileLd = 40;  // elements between rows in LDS (32 and 16 bytes of padding)

// SINGLE (with GATED): the experts have no gate; the tile is 128 features of the one matrix, as in the
// down product, over the tokens' rows, and a feature's product is both factors of its activation.
template <bool GATED, bool SINGLE = false>
__global__ void __launch_bounds__(256)
    moe_tiled_mfma_kernel(const bf16* __restrict__ a, const int32_t* __restrict__ order,
                          const int32_t* __restrict__ counts, const bf16* __restrict__ w0, const bf16* __restrict__ w1,
                          bf16* __restrict__ act_out, float* __restrict__ pair_out, int n, int k, int m, int top, int act) {
  __shared__ __attribute__((aligned(16))) uint16_t sa[2][kTileRows * kTileLd];
  __shared__ __attribute__((aligned(16))) uint16_t sb[2][kTileRows * kTileLd];
  const int e = blockIdx.z;
  const int count = min(counts[e], n);
  const int row0 = blockIdx.y * kTileRows;
  if (row0 >= count) return;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int i = lane % 16, kg = lane / 16;
  const int wm = wave / 2, wn = wave % 2;
  const int lr = tid / 4, lp = tid % 4;  // the row (and the one 64 below) and the 16-byte piece that this thread stages
  const int32_t* list = order + static_cast<size_t>(e) * n;
  const bf16* arow[2];
  const bf16* brow[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = row0 + lr + 64 * h;
    const int pair = r < count ? list[r] : -1;
    // gate/up: a pair's row is its token's; down: its own row of activations
    arow[h] = pair < 0 ? nullptr : a + static_cast<size_t>(GATED ? min(pair / top, n - 1) : min(pair, n * top - 1)) * k + lp * 8;
    if (GATED && !SINGLE) {
      const int f = blockIdx.x * 64 + lr;
      brow[h] = f < m ? (h == 0 ? w0 : w1) + (static_cast<size_t>(e) * m + f) * k + lp * 8 : nullptr;
    } else {
      const int c = blockIdx.x * 128 + lr + 64 * h;
      brow[h] = c < m ? w0 + (static_cast<size_t>(e) * m + c) * k + lp * 8 : nullptr;
    }
  }
  uint4 ra[2], rb[2];
  auto fetch = [&](int k0) {
    const bool have = k0 + lp * 8 < k;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      ra[h] = rb[h] = make_uint4(0, 0, 0, 0);
      if (have && arow[h]) ra[h] = *reinterpret_cast<const uint4*>(arow[h] + k0);
      if (have && brow[h]) rb[h] = *reinterpret_cast<const uint4*>(brow[h] + k0);
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *reinterpret_cast<uint4*>(&sa[buf][(lr + 64 * h) * kTileLd + lp * 8]) = ra[h];
      *reinterpret_cast<uint4*>(&sb[buf][(lr + 64 * h) * kTileLd + lp * 8]) = rb[h];
    }
  };
  constexpr int kOperands = 4;  // B operands a step
  mf32x4 acc[4][4];
#pragma unroll
  for (int am = 0; am < 4; ++am)
#pragma unroll
    for (int bn = 0; bn < 4; ++bn) acc[am][bn] = mf32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < k; k0 += 32, buf ^= 1) {
    const bool more = k0 + 32 < k;
    if (more) fetch(k0 + 32);
    mbf16x8 af[4], bf[4];
#pragma unroll
    for (int am = 0; am < 4; ++am)
      af[am] = __builtin_bit_cast(mbf16x8, *reinterpret_cast<const uint4*>(&sa[buf][(wm * 64 + am * 16 + i) * kTileLd + kg * 8]));
#pragma unroll
    for (int bn = 0; bn < kOperands; ++bn) {
      // gate/up: operands 0, 1 are this wavefront's 32 gate features, 2, 3 the same features of up (rows 64 on)
      const int brw = GATED && !SINGLE ? (bn / 2) * 64 + wn * 32 + (bn % 2) * 16 + i : wn * 64 + bn * 16 + i;
      bf[bn] = __builtin_bit_cast(mbf16x8, *reinterpret_cast<const uint4*>(&sb[buf][brw * kTileLd + kg * 8]));
    }
#pragma unroll
    for (int am = 0; am < 4; ++am)
#pragma unroll
      for (int bn = 0; bn < kOperands; ++bn)
        acc[am][bn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[bn], af[am], acc[am][bn], 0, 0, 0);
    if (more) stage(buf ^ 1);
    __syncthreads();
  }
  // this lane holds weight rows 4 kg + r of operand bn for the pair in row wm * 64 + am * 16 + i of the tile
#pragma unroll
  for (int am = 0; am < 4; ++am) {
    const int r = row0 + wm * 64 + am * 16 + i;
    if (r >= count) continue;
    const int pair = min(max(list[r], 0), n * top - 1);
    if (GATED && SINGLE) {
      bf16* dst = act_out + static_cast<size_t>(pair) * m;
#pragma unroll
      for (int bn = 0; bn < 4; ++bn) {
        const int f = blockIdx.x * 128 + wn * 64 + bn * 16 + 4 * kg;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (f + q < m) dst[f + q] = from_float<bf16>(gate_act(acc[am][bn][q], act) * acc[am][bn][q]);
      }
    } else if (GATED) {
      bf16* dst = act_out + static_cast<size_t>(pair) * m;
#pragma unroll
      for (int bn = 0; bn < 2; ++bn) {
        const int f = blockIdx.x * 64 + wn * 32 + bn * 16 + 4 * kg;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (f + q < m) dst[f + q] = from_float<bf16>(gate_act(acc[am][bn][q], act) * acc[am][bn + 2][q]);
      }
    } else {
      float* dst = pair_out + static_cast<size_t>(pair) * m;
#pragma unroll
      for (int bn = 0; bn < 4; ++bn) {
        const int c = blockIdx.x * 128 + wn * 64 + bn * 16 + 4 * kg;
        if (c + 3 < m) {
          *reinterpret_cast<float4*>(dst + c) = make_float4(acc[am][bn][0], acc[am][bn][1], acc[am][bn][2], acc[am][bn][3]);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (c + q < m) dst[c + q] = acc[am][bn][q];
        }
      }
    }
  }
}

// out[t, c] = add[t, c] + sum_k weights[t, k] * pair_out[t * top + k, c], k in the order chosen
__global__ void __launch_bounds__(256)
    moe_join_kernel(const float* __restrict__ pair_out, const float* __restrict__ weights, const bf16* __restrict__ add,
                    const float* __restrict__ add_gate, int gate_ld, bf16* __restrict__ out, int width, int top) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float total = 0.f;
  for (int k = 0; k < top; ++k)
    total = fmaf(weights[static_cast<size_t>(t) * top + k], pair_out[(static_cast<size_t>(t) * top + k) * width + c], total);
  if (add) total += shared_share(add_gate, gate_ld, t) * to_float(add[static_cast<size_t>(t) * width + c]);
  out[static_cast<size_t>(t) * width + c] = from_float<bf16>(total);
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
                               const void* w_up, const void* w_down, const void* add, const float* add_gate,
                               int gate_ld, void* act_buf, void* out, int dtype, int n, int width, int ff, int experts, int top, int act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_experts: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && width > 0 && ff > 0 && experts > 0 && top >= 1 && top <= experts,
              "moe_experts: bad sizes n=%d width=%d ff=%d experts=%d top=%d", n, width, ff, experts, top);
  SHK_REQUIRE(act >= 1 && act <= 3, "moe_experts: unknown activation %d", act);
  SHK_REQUIRE(!add_gate || (add && gate_ld >= 1), "moe_experts: a gate of the added rows needs those rows and a stride");
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
      add_gate, gate_ld, static_cast<T*>(out), width, ff, top, experts)
  if (dtype == kF32) {
    SHK_GO(float);
  } else {
    SHK_GO(bf16);
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("moe_experts");
  return 0;
}

extern "C" long long shk_moe_grouped_scratch_bytes(int n, int width, int experts, int top) {
  // order [experts, n] and counts [experts] (int32), then the pairs' outputs [n * top, width] (float32)
  const long long ints = static_cast<long long>(experts) * n + experts;
  return ((ints * 4 + 15) / 16) * 16 + static_cast<long long>(n) * top * width * 4;
}

extern "C" int shk_moe_experts_grouped(const void* x, const int32_t* chosen, const float* weights, const void* w_gate,
                                       const void* w_up, const void* w_down, const void* add, const float* add_gate,
                                       int gate_ld, void* act_buf, void* out, void* scratch, int n, int width, int ff, int experts, int top, int act,
                                       void* stream) {
  SHK_REQUIRE(n >= 0 && width > 0 && ff > 0 && experts > 0 && experts <= 65535 && top >= 1 && top <= experts,
              "moe_experts_grouped: bad sizes n=%d width=%d ff=%d experts=%d top=%d", n, width, ff, experts, top);
  SHK_REQUIRE(act >= 1 && act <= 3, "moe_experts_grouped: unknown activation %d", act);
  SHK_REQUIRE(!add_gate || (add && gate_ld >= 1),
              "moe_experts_grouped: a gate of the added rows needs those rows and a stride");
  SHK_REQUIRE(width % 8 == 0 && ff % 8 == 0, "moe_experts_grouped: width %d and ff %d must be multiples of 8", width, ff);
  if (n == 0) return 0;
  SHK_REQUIRE(static_cast<long long>(n) * top < (1LL << 30) && (n + 31) / 32 <= 65535,
              "moe_experts_grouped: too many (token, expert) pairs");
  SHK_REQUIRE(x && chosen && weights && w_gate && w_up && w_down && act_buf && out && scratch,
              "moe_experts_grouped: null pointer");
  for (const void* p : {x, w_gate, w_up, w_down, static_cast<const void*>(act_buf), static_cast<const void*>(scratch)})
    SHK_REQUIRE(reinterpret_cast<uintptr_t>(p) % 16 == 0, "moe_experts_grouped: operands must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* order = static_cast<int32_t*>(scratch);
  int32_t* counts = order + static_cast<size_t>(experts) * n;
  const long long ints = static_cast<long long>(experts) * n + experts;
  float* pair_out = reinterpret_cast<float*>(static_cast<char*>(scratch) + ((ints * 4 + 15) / 16) * 16);
  moe_lists_kernel<<<experts, 256, 0, s>>>(chosen, n, top, order, counts);
  if (static_cast<long long>(n) * top >= 64LL * experts) {
    // lists of 64 pairs and more on average: tiles of 128 pairs through LDS
    const int row_tiles = (n + kTileRows - 1) / kTileRows;
    if (w_gate == w_up)
      moe_tiled_mfma_kernel<true, true><<<dim3((ff + 127) / 128, row_tiles, experts), 256, 0, s>>>(
          static_cast<const bf16*>(x), order, counts, static_cast<const bf16*>(w_gate), static_cast<const bf16*>(w_up),
          static_cast<bf16*>(act_buf), nullptr, n, width, ff, top, act);
    else
      moe_tiled_mfma_kernel<true><<<dim3((ff + 63) / 64, row_tiles, experts), 256, 0, s>>>(
          static_cast<const bf16*>(x), order, counts, static_cast<const bf16*>(w_gate), static_cast<const bf16*>(w_up),
          static_cast<bf16*>(act_buf), nullptr, n, width, ff, top, act);
    moe_tiled_mfma_kernel<false><<<dim3((width + 127) / 128, row_tiles, experts), 256, 0, s>>>(
        static_cast<const bf16*>(act_buf), order, counts, static_cast<const bf16*>(w_down), nullptr, nullptr, pair_out, n,
        ff, width, top, act);
  } else {
    const int row_tiles = (n + 31) / 32;
    moe_gate_up_mfma_kernel<<<dim3((ff + 127) / 128, row_tiles, experts), 256, 0, s>>>(
        static_cast<const bf16*>(x), order, counts, static_cast<const bf16*>(w_gate), static_cast<const bf16*>(w_up),
        static_cast<bf16*>(act_buf), n, width, ff, top, act);
    moe_down_mfma_kernel<<<dim3((width + 255) / 256, row_tiles, experts), 256, 0, s>>>(
        static_cast<const bf16*>(act_buf), order, counts, static_cast<const bf16*>(w_down), pair_out, n, width, ff, top);
  }
  moe_join_kernel<<<dim3((width + 255) / 256, n), 256, 0, s>>>(pair_out, weights, static_cast<const bf16*>(add), add_gate,
                                                               gate_ld, static_cast<bf16*>(out), width, top);
  SHK_LAUNCH_CHECK("moe_experts_grouped");
  return 0;
}
