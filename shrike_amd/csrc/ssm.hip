// Recurrent mixers whose state is a fixed-size tensor per request: the selective
// scan of Mamba (with its short causal convolution) and retention (linear
// attention with a fixed decay per head).  A sequence's tokens of the step are
// walked in order, whether they are a prompt's portion or one decoded token, so
// a position's result does not depend on how the prompt was cut.  All state and
// everything in the recurrences is float32.  A state is taken as zero where the
// sequence's first row of the step is at position 0: a slot that another request
// left full starts from nothing.
//
// Selective scan, per channel c and state n:
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c
// with dt = softplus(W_dt low + b) per channel and A = -exp(A_log).
// A request's slot holds S [inner, state] and then the convolution's last taps - 1
// inputs [(taps - 1), inner], oldest first.
//
// Retention, per head:  S_t = decay S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t.
// A request's slot holds S as [heads, v_dim, dim].
#include "api.h"
#include "common.h"

namespace shk {

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

// Sum over the LANES neighbouring lanes that share a channel or a column (LANES a power of two; every
// lane of the group gets it).  Up to 16 lanes meet by lane permutations of the vector unit: within
// fours [1,0,3,2] and [2,3,0,1], then mirrored halves of 8 and of 16 (all lanes of a four already
// hold the four's sum, so its mirror image holds the other four's).
template <int CTRL>
__device__ __forceinline__ float dpp_moved(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
  if (LANES >= 2) v += dpp_moved<0xB1>(v);
  if (LANES >= 4) v += dpp_moved<0x4E>(v);
  if (LANES >= 8) v += dpp_moved<0x141>(v);
  if (LANES >= 16) v += dpp_moved<0x140>(v);
  if (LANES >= 32) v += __shfl_xor(v, 16, kWave);
  if (LANES >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// y[t, c] = silu(bias[c] + sum_k taps[c, K - 1 - k] * x(t - k, c)): x(t - k) is a row of this
// step where the sequence's portion reaches that far back, else the slot's kept input of
// that position, else (before the sequence's start) zero.
template <typename T>
__global__ void __launch_bounds__(256)
    conv_silu_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ taps, const float* __restrict__ bias,
                     int K, int inner, const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq,
                     const int32_t* __restrict__ cu_q, const int32_t* __restrict__ slots,
                     const float* __restrict__ state, long long slot_stride, long long tail_off,
                     T* __restrict__ y) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= inner) return;
  const int seq = token_seq[t];
  const int pos = positions[t];
  const int first = cu_q[seq];  // the sequence's first row of the step
  const float* tail = state + static_cast<size_t>(slots[seq]) * slot_stride + tail_off;
  float acc = bias[c];
  for (int k = K - 1; k >= 0; --k) {  // oldest input first
    float v = 0.f;
    if (pos - k >= 0) {
      if (t - k >= first) {
        v = to_float(x[static_cast<size_t>(t - k) * ldx + c]);
      } else {
        // the slot keeps the inputs of the K - 1 positions before the step, oldest first:
        // entry e holds position (start - (K - 1) + e), start = the position of row `first`
        const int start = pos - (t - first);
        const int e = (pos - k) - (start - (K - 1));
        v = tail[static_cast<size_t>(e) * inner + c];
      }
    }
    acc = fmaf(taps[c * K + (K - 1 - k)], v, acc);
  }
  y[static_cast<size_t>(t) * inner + c] = from_float<T>(silu_f(acc));
}

constexpr int kDtTokens = 8;  // tokens a workgroup where a step has many: the matrix is read once for all of them

// dt[t, c] = softplus(b[c] + sum_r W[r, c] * low[t, r]) in float32; W is given transposed, [rank, inner], so
// that neighbouring channels' weights are neighbours in memory.  A token's sum runs over r in ascending
// order whatever else is in the step.
template <int kDtTokens>
__global__ void __launch_bounds__(256)
    dt_softplus_kernel(const float* __restrict__ low, int ld, const float* __restrict__ wt, const float* __restrict__ b,
                       int rank, int inner, float* __restrict__ dt, int n) {
  extern __shared__ float lows[];  // [kDtTokens, rank]
  const int t0 = blockIdx.y * kDtTokens;
  const int count = min(kDtTokens, n - t0);
  for (int i = threadIdx.x; i < count * rank; i += blockDim.x)
    lows[i] = low[static_cast<size_t>(t0 + i / rank) * ld + i % rank];
  __syncthreads();
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= inner) return;
  float acc[kDtTokens];
#pragma unroll
  for (int k = 0; k < kDtTokens; ++k) acc[k] = b[c];
  for (int r0 = 0; r0 < rank; r0 += 8) {  // eight rows' weights on their way at once
    float w[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) w[u] = r0 + u < rank ? wt[static_cast<size_t>(r0 + u) * inner + c] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (r0 + u >= rank) break;
#pragma unroll
      for (int k = 0; k < kDtTokens; ++k)
        if (k < count) acc[k] = fmaf(w[u], lows[k * rank + r0 + u], acc[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < kDtTokens; ++k)
    if (k < count) dt[static_cast<size_t>(t0 + k) * inner + c] = softplus_f(acc[k]);
}

constexpr int kStatesPerLane = 4;  // (8 where a channel has more than 256 states)
constexpr int kScanBlock = 16;  // tokens whose inputs are fetched together

// One sequence's tokens for a block of channels.  LANES lanes share a channel's states
// (LANES * 4 >= states); a wavefront holds 64 / LANES channels.
template <typename T, int LANES, int kStatesPerLane>
__global__ void __launch_bounds__(256)
    selective_scan_kernel(const float* __restrict__ dt, const T* __restrict__ x, const float* __restrict__ bc,
                          int ld_bc, int b_off, int c_off, const T* __restrict__ z, int ldz,
                          const float* __restrict__ a_log, const float* __restrict__ dskip, int inner, int states,
                          int K, const T* __restrict__ raw, int ld_raw, const int32_t* __restrict__ positions,
                          const int32_t* __restrict__ cu_q, const int32_t* __restrict__ slots,
                          float* __restrict__ state, long long slot_stride, T* __restrict__ out) {
  // Tokens go by in blocks of kScanBlock: a block's B and C (the same for every channel) are staged in
  // LDS by the workgroup, and a lane fetches its channel's step sizes, inputs and gates of the block at
  // once, so that the walk over the tokens waits for memory once a block and not once a token.
  extern __shared__ float bcs[];  // [kScanBlock][2 * states]
  const int seq = blockIdx.y;
  const int unit = blockIdx.x * (256 / LANES) + threadIdx.x / LANES;  // channel
  const int part = threadIdx.x % LANES;
  const bool active = unit < inner;
  const int c = active ? unit : inner - 1;
  const int first = cu_q[seq], last = cu_q[seq + 1];
  if (last <= first) return;
  float* slot = state + static_cast<size_t>(slots[seq]) * slot_stride;
  float* srow = slot + static_cast<size_t>(c) * states;
  const bool fresh = positions[first] == 0;
  float S[kStatesPerLane], A[kStatesPerLane];
#pragma unroll
  for (int i = 0; i < kStatesPerLane; ++i) {
    const int n = part * kStatesPerLane + i;
    S[i] = (n < states && !fresh) ? srow[n] : 0.f;
    A[i] = n < states ? -expf(a_log[static_cast<size_t>(c) * states + n]) : 0.f;
  }
  const float dc = dskip[c];
  for (int t0 = first; t0 < last; t0 += kScanBlock) {
    const int count = min(kScanBlock, last - t0);
    __syncthreads();  // (the block before has been read)
    for (int i = threadIdx.x; i < count * 2 * states; i += 256) {
      const int tt = i / (2 * states), j = i % (2 * states);
      bcs[i] = bc[static_cast<size_t>(t0 + tt) * ld_bc + (j < states ? b_off + j : c_off + j - states)];
    }
    float stepv[kScanBlock], xs[kScanBlock], gs[kScanBlock];
#pragma unroll
    for (int k = 0; k < kScanBlock; ++k) {
      const int t = t0 + (k < count ? k : 0);
      stepv[k] = dt[static_cast<size_t>(t) * inner + c];
      xs[k] = to_float(x[static_cast<size_t>(t) * inner + c]);
      gs[k] = to_float(z[static_cast<size_t>(t) * ldz + c]);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kScanBlock; ++k) {
      if (k >= count) break;
      const float step = stepv[k], xv = xs[k];
      const float* bt = bcs + k * 2 * states;
      const float* ct = bt + states;
      const float dx = step * xv;
      float y = 0.f;
#pragma unroll
      for (int i = 0; i < kStatesPerLane; ++i) {
        const int n = part * kStatesPerLane + i;
        if (n < states) {
          // (bfloat16 models: the hardware's exponential, float32 all the same; float32 models: the library's)
          const float decay = sizeof(T) == 2 ? __expf(step * A[i]) : expf(step * A[i]);
          S[i] = fmaf(decay, S[i], dx * bt[n]);
          y = fmaf(S[i], ct[n], y);
        }
      }
      y = group_sum<LANES>(y);
      if (part == 0 && active) {
        y = fmaf(dc, xv, y);
        out[static_cast<size_t>(t0 + k) * inner + c] = from_float<T>(y * silu_f(gs[k]));
      }
    }
  }
  if (!active) return;
#pragma unroll
  for (int i = 0; i < kStatesPerLane; ++i) {
    const int n = part * kStatesPerLane + i;
    if (n < states) srow[n] = S[i];
  }
  // the convolution's kept inputs: the K - 1 positions before the next step, oldest first
  if (part == 0 && K > 1) {
    float* tail = slot + static_cast<size_t>(inner) * states;
    const int count = last - first;
    for (int e = 0; e < K - 1; ++e) {
      const int back = (K - 1) - e;  // the input `back` positions before the next step
      float v = 0.f;
      if (back <= count) {
        v = to_float(raw[static_cast<size_t>(last - back) * ld_raw + c]);
      } else if (!fresh) {
        v = tail[static_cast<size_t>(e + count) * inner + c];  // shifts up; e + count <= K - 2
      }
      tail[static_cast<size_t>(e) * inner + c] = v;
    }
  }
}

// Rotation of element pairs (i, i + rot_dim / 2) of every head of float32 rows, in place:
// x[t, off + h * dim + e]; angle position * inv_freq[i]; all of the head is multiplied
// by `mult` afterwards.
__global__ void __launch_bounds__(256)
    rotate_half_rows_kernel(float* __restrict__ x, int ld, int off, int heads, int dim, int rot_dim,
                            const float* __restrict__ inv_freq, const int32_t* __restrict__ positions, float mult,
                            int n) {
  const int half = rot_dim / 2;
  const int per_head = dim - half;  // a thread takes a pair, or one unrotated element
  const long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (item >= static_cast<long long>(n) * heads * per_head) return;
  const int e = static_cast<int>(item % per_head);
  const int h = static_cast<int>((item / per_head) % heads);
  const int t = static_cast<int>(item / (static_cast<long long>(per_head) * heads));
  float* row = x + static_cast<size_t>(t) * ld + off + h * dim;
  if (e < half) {
    const float angle = static_cast<float>(positions[t]) * inv_freq[e];
    const double wide = static_cast<double>(angle);
    const double turns = rint(wide * 0.15915494309189535);
    const float reduced = static_cast<float>(wide - turns * 6.283185307179586);
    float sv, cv;
    sincosf(reduced, &sv, &cv);
    const float u = row[e], v = row[e + half];
    row[e] = (u * cv - v * sv) * mult;
    row[e + half] = (v * cv + u * sv) * mult;
  } else {
    row[e + half] *= mult;  // elements from rot_dim on
  }
}

constexpr int kRowsPerLane = 8;  // (16 where a head has more than 512 elements)
constexpr int kRetBlock = 8;  // tokens whose inputs are fetched together

// the heads that the columns of one workgroup (256 / lanes of them) can belong to
inline int retention_heads_a_workgroup(int lanes, int heads, int v_dim) {
  const int per_wg = 256 / lanes;
  const int most = (per_wg + v_dim - 2) / v_dim + 1;
  return most < heads ? most : heads;
}

// One sequence's tokens for one (head, value column); LANES lanes share the column's rows
// of S (LANES * 8 >= dim).
template <int LANES, int kRowsPerLane>
__global__ void __launch_bounds__(256)
    retention_scan_kernel(const float* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
                          const float* __restrict__ decay, int heads, int dim, int v_dim,
                          const int32_t* __restrict__ positions, const int32_t* __restrict__ cu_q,
                          const int32_t* __restrict__ slots, float* __restrict__ state, long long slot_stride,
                          float* __restrict__ out, int block) {
  // Tokens go by in blocks of `block` (at most kRetBlock): the queries and keys of the heads that this workgroup's columns
  // belong to are staged in LDS by the workgroup ([token][head][q | k]), a lane fetches its column's
  // values of the block at once: the walk waits for memory once a block.
  extern __shared__ float qks[];
  const int seq = blockIdx.y;
  const int per_wg = 256 / LANES;
  const int unit_raw = blockIdx.x * per_wg + threadIdx.x / LANES;  // (head, column)
  const int part = threadIdx.x % LANES;
  const int units = heads * v_dim;
  const bool active = unit_raw < units;
  const int unit = active ? unit_raw : units - 1;
  const int h = unit / v_dim, col = unit % v_dim;
  const int h_lo = blockIdx.x * per_wg / v_dim;
  const int h_hi = min(units - 1, blockIdx.x * per_wg + per_wg - 1) / v_dim;
  const int nh = h_hi - h_lo + 1;
  const int first = cu_q[seq], last = cu_q[seq + 1];
  if (last <= first) return;
  float* srow = state + static_cast<size_t>(slots[seq]) * slot_stride + static_cast<size_t>(unit) * dim;
  const bool fresh = positions[first] == 0;
  float S[kRowsPerLane];
#pragma unroll
  for (int i = 0; i < kRowsPerLane; ++i) {
    const int d = part * kRowsPerLane + i;
    S[i] = (d < dim && !fresh) ? srow[d] : 0.f;
  }
  const float a = decay[h];
  for (int t0 = first; t0 < last; t0 += block) {
    const int count = min(block, last - t0);
    __syncthreads();
    for (int i = threadIdx.x; i < count * nh * 2 * dim; i += 256) {
      const int tt = i / (nh * 2 * dim), rest = i % (nh * 2 * dim);
      const int hh = rest / (2 * dim), j = rest % (2 * dim);
      const float* row = proj + static_cast<size_t>(t0 + tt) * ld;
      qks[i] = j < dim ? row[q_off + (h_lo + hh) * dim + j] : row[k_off + (h_lo + hh) * dim + j - dim];
    }
    float vs[kRetBlock];
#pragma unroll
    for (int k = 0; k < kRetBlock; ++k)
      vs[k] = proj[static_cast<size_t>(t0 + (k < count ? k : 0)) * ld + v_off + h * v_dim + col];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kRetBlock; ++k) {
      if (k >= count) break;
      const float* qt = qks + (static_cast<size_t>(k) * nh + (h - h_lo)) * 2 * dim;
      const float* kt = qt + dim;
      const float vv = vs[k];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < kRowsPerLane; ++i) {
        const int d = part * kRowsPerLane + i;
        if (d < dim) {
          S[i] = fmaf(a, S[i], kt[d] * vv);
          o = fmaf(S[i], qt[d], o);
        }
      }
      o = group_sum<LANES>(o);
      if (part == 0 && active) out[static_cast<size_t>(t0 + k) * heads * v_dim + unit] = o;
    }
  }
  if (!active) return;
#pragma unroll
  for (int i = 0; i < kRowsPerLane; ++i) {
    const int d = part * kRowsPerLane + i;
    if (d < dim) srow[d] = S[i];
  }
}

inline int lanes_for(int items, int per_lane) {
  int lanes = 1;
  while (lanes * per_lane < items) lanes *= 2;
  return lanes;
}

}  // namespace shk

using namespace shk;

extern "C" long long shk_selective_scan_state_floats(int inner, int states, int taps) {
  return static_cast<long long>(inner) * states + static_cast<long long>(taps > 1 ? taps - 1 : 0) * inner;
}

extern "C" int shk_conv_silu(const void* x, int ldx, const float* taps, const float* bias, int num_taps, int inner,
                             const int32_t* positions, const int32_t* token_seq, const int32_t* cu_q,
                             const int32_t* slots, const float* state, long long slot_stride, int states, void* y,
                             int dtype, int n, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "conv_silu: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && inner > 0 && num_taps >= 1 && num_taps <= 64 && ldx >= inner && states > 0,
              "conv_silu: bad sizes n=%d inner=%d taps=%d", n, inner, num_taps);
  SHK_REQUIRE(slot_stride >= shk_selective_scan_state_floats(inner, states, num_taps),
              "conv_silu: a slot of %lld floats does not hold the state", slot_stride);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "conv_silu: at most 65535 tokens a call, got %d", n);
  SHK_REQUIRE(x && taps && bias && positions && token_seq && cu_q && slots && state && y, "conv_silu: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((inner + 255) / 256, n);
  const long long tail_off = static_cast<long long>(inner) * states;
  if (dtype == kF32)
    conv_silu_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), ldx, taps, bias, num_taps, inner,
                                                 positions, token_seq, cu_q, slots, state, slot_stride, tail_off,
                                                 static_cast<float*>(y));
  else
    conv_silu_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(x), ldx, taps, bias, num_taps, inner,
                                                positions, token_seq, cu_q, slots, state, slot_stride, tail_off,
                                                static_cast<bf16*>(y));
  SHK_LAUNCH_CHECK("conv_silu");
  return 0;
}

extern "C" int shk_dt_softplus(const float* low, int ld, const float* w, const float* b, int rank, int inner,
                               float* dt, int n, void* stream) {
  SHK_REQUIRE(n >= 0 && inner > 0 && rank > 0 && rank <= 1024 && ld >= rank, "dt_softplus: bad sizes n=%d inner=%d rank=%d",
              n, inner, rank);
  if (n == 0) return 0;
  SHK_REQUIRE(low && w && b && dt, "dt_softplus: null pointer");
  if (n <= 32) {
    // few tokens: a wavefront per (64 channels, token), so that the launch has workgroups enough
    SHK_REQUIRE(n <= 65535, "dt_softplus: bad n");
    dt_softplus_kernel<1><<<dim3((inner + 63) / 64, n), 64, rank * sizeof(float), static_cast<hipStream_t>(stream)>>>(
        low, ld, w, b, rank, inner, dt, n);
  } else {
    dim3 grid((inner + 255) / 256, (n + kDtTokens - 1) / kDtTokens);
    dt_softplus_kernel<kDtTokens><<<grid, 256, kDtTokens * rank * sizeof(float), static_cast<hipStream_t>(stream)>>>(
        low, ld, w, b, rank, inner, dt, n);
  }
  SHK_LAUNCH_CHECK("dt_softplus");
  return 0;
}

extern "C" int shk_selective_scan(const float* dt, const void* x, const float* bc, int ld_bc, int b_off, int c_off,
                                  const void* z, int ldz, const float* a_log, const float* dskip, int inner,
                                  int states, int num_taps, const void* raw, int ld_raw, const int32_t* positions,
                                  const int32_t* cu_q, const int32_t* slots, float* state, long long slot_stride,
                                  void* out, int dtype, int num_seqs, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "selective_scan: unknown dtype %d", dtype);
  SHK_REQUIRE(num_seqs >= 0 && inner > 0 && states > 0 && states <= 512 && num_taps >= 1,
              "selective_scan: bad sizes seqs=%d inner=%d states=%d", num_seqs, inner, states);
  SHK_REQUIRE(b_off >= 0 && c_off >= 0 && b_off + states <= ld_bc && c_off + states <= ld_bc && ldz >= inner &&
                  ld_raw >= inner,
              "selective_scan: columns do not fit their rows");
  SHK_REQUIRE(slot_stride >= shk_selective_scan_state_floats(inner, states, num_taps),
              "selective_scan: a slot of %lld floats does not hold the state", slot_stride);
  if (num_seqs == 0) return 0;
  SHK_REQUIRE(num_seqs <= 65535, "selective_scan: at most 65535 sequences a call");
  SHK_REQUIRE(dt && x && bc && z && a_log && dskip && raw && positions && cu_q && slots && state && out,
              "selective_scan: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int lanes = states > 64 * kStatesPerLane ? 64 : lanes_for(states, kStatesPerLane);
#define SHK_GO(T, L)                                                                                                 \
  selective_scan_kernel<T, L, (L == 64 ? 8 : kStatesPerLane)>                                                        \
      <<<dim3((inner + 256 / L - 1) / (256 / L), num_seqs), 256, kScanBlock * 2 * states * sizeof(float), s>>>(      \
      dt, static_cast<const T*>(x), bc, ld_bc, b_off, c_off, static_cast<const T*>(z), ldz, a_log, dskip, inner,     \
      states, num_taps, static_cast<const T*>(raw), ld_raw, positions, cu_q, slots, state, slot_stride,              \
      static_cast<T*>(out))
#define SHK_LANES(T)                                                                                                 \
  switch (lanes) {                                                                                                   \
    case 1: SHK_GO(T, 1); break;                                                                                     \
    case 2: SHK_GO(T, 2); break;                                                                                     \
    case 4: SHK_GO(T, 4); break;                                                                                     \
    case 8: SHK_GO(T, 8); break;                                                                                     \
    case 16: SHK_GO(T, 16); break;                                                                                   \
    case 32: SHK_GO(T, 32); break;                                                                                   \
    default: SHK_GO(T, 64); break;                                                                                   \
  }
  if (dtype == kF32) {
    SHK_LANES(float)
  } else {
    SHK_LANES(bf16)
  }
#undef SHK_LANES
#undef SHK_GO
  SHK_LAUNCH_CHECK("selective_scan");
  return 0;
}

extern "C" int shk_rotate_half_rows(float* x, int ld, int off, int heads, int dim, int rot_dim, const float* inv_freq,
                                    const int32_t* positions, float mult, int n, void* stream) {
  SHK_REQUIRE(n >= 0 && heads > 0 && dim > 0 && rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= dim && off >= 0 &&
                  off + heads * dim <= ld,
              "rotate_half_rows: bad sizes heads=%d dim=%d rot_dim=%d", heads, dim, rot_dim);
  if (n == 0) return 0;
  SHK_REQUIRE(x && positions && (rot_dim == 0 || inv_freq), "rotate_half_rows: null pointer");
  const long long items = static_cast<long long>(n) * heads * (dim - rot_dim / 2);
  rotate_half_rows_kernel<<<static_cast<unsigned>((items + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      x, ld, off, heads, dim, rot_dim, inv_freq, positions, mult, n);
  SHK_LAUNCH_CHECK("rotate_half_rows");
  return 0;
}

extern "C" long long shk_retention_state_floats(int heads, int dim, int v_dim) {
  return static_cast<long long>(heads) * v_dim * dim;
}

extern "C" int shk_retention_scan(const float* proj, int ld, int q_off, int k_off, int v_off, const float* decay,
                                  int num_seqs, int heads, int dim, int v_dim, const int32_t* positions,
                                  const int32_t* cu_q, const int32_t* slots, float* state, long long slot_stride,
                                  float* out, void* stream) {
  SHK_REQUIRE(num_seqs >= 0 && heads > 0 && dim > 0 && dim <= 1024 && v_dim > 0,
              "retention_scan: bad sizes seqs=%d heads=%d dim=%d v_dim=%d", num_seqs, heads, dim, v_dim);
  SHK_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= ld && k_off + heads * dim <= ld &&
                  v_off + heads * v_dim <= ld,
              "retention_scan: columns do not fit rows of %d", ld);
  SHK_REQUIRE(slot_stride >= shk_retention_state_floats(heads, dim, v_dim),
              "retention_scan: a slot of %lld floats does not hold the state", slot_stride);
  if (num_seqs == 0) return 0;
  SHK_REQUIRE(num_seqs <= 65535, "retention_scan: at most 65535 sequences a call");
  SHK_REQUIRE(proj && decay && positions && cu_q && slots && state && out, "retention_scan: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int lanes = dim > 64 * kRowsPerLane ? 64 : lanes_for(dim, kRowsPerLane);
  const int units = heads * v_dim;
  const size_t a_token = static_cast<size_t>(retention_heads_a_workgroup(lanes, heads, v_dim)) * 2 * dim * sizeof(float);
  SHK_REQUIRE(a_token <= 64000, "retention_scan: %d heads of %d elements a workgroup do not fit its LDS",
              retention_heads_a_workgroup(lanes, heads, v_dim), dim);
  const int block = static_cast<int>(64000 / a_token) < kRetBlock ? static_cast<int>(64000 / a_token) : kRetBlock;
  const size_t lds = block * a_token;
#define SHK_GO(L)                                                                                              \
  retention_scan_kernel<L, (L == 64 ? 16 : kRowsPerLane)><<<dim3((units + 256 / L - 1) / (256 / L), num_seqs), 256, lds, s>>>(                \
      proj, ld, q_off, k_off, v_off, decay, heads, dim, v_dim, positions, cu_q, slots, state, slot_stride, out, block)
  switch (lanes) {
    case 1: SHK_GO(1); break;
    case 2: SHK_GO(2); break;
    case 4: SHK_GO(4); break;
    case 8: SHK_GO(8); break;
    case 16: SHK_GO(16); break;
    case 32: SHK_GO(32); break;
    default: SHK_GO(64); break;
  }
#undef SHK_GO
  SHK_LAUNCH_CHECK("retention_scan");
  return 0;
}
