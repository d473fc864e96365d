// The matrix memory of an mLSTM layer: per head a matrix S [dim, v_dim], a vector n
// [dim] and a running maximum m, all float32, carried from token to token in the
// request's state slot:
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T       (n_t likewise, with k_t alone)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// with log gates i_t = cap tanh(x / cap) and f_t = logsigmoid(cap tanh(y / cap)) of the
// gates' projections x, y (bias added here).  The state before position 0 is zero (m = 0).
//
// mlstm_scan_kernel: one wavefront per (sequence, head, 4 value columns), eight of them (32
// columns) in a workgroup.  A lane owns one column and a run of dim / 16 rows of S in
// registers; a token costs dim / 16 multiply-adds a lane for S and as many for the readout,
// whose sixteen partial sums meet by four lane exchanges.  Narrow tiles make many wavefronts
// (a head of 512 values: 128), so that every SIMD of the chip has work and the chain from
// token to token is short.  Tokens are staged sixteen at a time through LDS (queries and keys
// once for the workgroup's eight wavefronts, each tile's values, the gates), all loads of a
// stage in flight together, so that the recurrence never waits for global memory.  Every
// wavefront keeps n and m for itself (its own copy in the state), so no two wavefronts share
// anything that one of them writes.  Prompt portions and single tokens take this one path: a
// token's result does not depend on how its sequence was cut into steps.
//
// State of one (slot, layer): [heads][tiles][64 RPT + 16 RPT + 1] floats, tiles = ceil(v_dim /
// 4), RPT = rows per lane (4, 8 or 16 for dim up to 64, 128, 256): S as the lanes hold it,
// [RPT][64 lanes] (lane = 4 * row group + column, row = RPT * row group + i), so that a
// wavefront's loads and stores are whole lines; then n [RPT][16 row groups]; then m.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kCols = 4;        // value columns per wavefront
constexpr int kRowGroups = 16;  // lanes that share a column split the rows among them
constexpr int kStage = 16;      // tokens staged at a time
constexpr int kScanWaves = 8;   // wavefronts (tiles) per workgroup

__host__ __device__ inline int scan_rpt(int dim) { return dim <= 64 ? 4 : dim <= 128 ? 8 : 16; }

// Sum over the sixteen lanes that share a value column (lane = 4 * row group + column): the four
// row groups of a 16-lane row by two rotations on the vector unit, then the four rows by two
// exchanges through the LDS crossbar; every lane gets the sum, always in this order.
template <int CTRL>
__device__ __forceinline__ float scan_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float column_sum(float v) {
  v += scan_dpp<0x124>(v);  // row_ror:4
  v += scan_dpp<0x128>(v);  // row_ror:8
  v += __shfl_xor(v, 16, kWave);
  return v + __shfl_xor(v, 32, kWave);
}

__device__ __forceinline__ float log_sigmoid(float x) {
  return x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
}

template <int RPT>  // rows per lane, a multiple of 4: dim <= 16 * RPT
__global__ void __launch_bounds__(kScanWaves* kWave)
    mlstm_scan_kernel(const float* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int i_off,
                      int f_off, const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                      float q_scale, int heads, int dim, int v_dim, int tiles, const int32_t* __restrict__ positions,
                      const int32_t* __restrict__ cu_q, const int32_t* __restrict__ slots,
                      float* __restrict__ state, long long slot_stride, float* __restrict__ out) {
  constexpr int ROWS = kRowGroups * RPT;
  constexpr int kThreads = kScanWaves * kWave;
  constexpr int kPerTile = kWave * RPT + kRowGroups * RPT + 1;
  constexpr int kLoads = (kStage * ROWS + kThreads - 1) / kThreads;  // staging loads a thread and operand
  __shared__ __attribute__((aligned(16))) float qs[kStage][ROWS];
  __shared__ __attribute__((aligned(16))) float ks[kStage][ROWS];
  __shared__ float vs[kScanWaves][kStage][kCols];
  __shared__ float gi[kStage], gf[kStage];

  const int head = blockIdx.y, seq = blockIdx.z;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int tile = blockIdx.x * kScanWaves + wave;
  const bool live = tile < tiles;  // (a workgroup's last wavefronts may have no tile; they keep the barriers)
  const int col = lane % kCols, rg = lane / kCols;
  const int vcol = tile * kCols + col;
  const int first = cu_q[seq], last = cu_q[seq + 1];
  float* st = state + static_cast<size_t>(slots[seq]) * slot_stride +
              (static_cast<size_t>(head) * tiles + (live ? tile : 0)) * kPerTile;

  float S[RPT], nv[RPT], m = 0.f;
  const bool fresh = positions[first] == 0;  // nothing precedes position 0
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const bool have = !fresh && live;
    S[i] = have ? st[i * kWave + lane] : 0.f;
    nv[i] = have ? st[kWave * RPT + i * kRowGroups + rg] : 0.f;
  }
  if (!fresh && live) m = st[kPerTile - 1];

  for (int t0 = first; t0 < last; t0 += kStage) {
    const int count = last - t0 < kStage ? last - t0 : kStage;
    // the stage's queries and keys: every load issued before the first is used
    float qv[kLoads], kv[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      const int idx = tid + u * kThreads;
      const int tt = idx / ROWS, r = idx % ROWS;
      const bool have = tt < count && r < dim;
      const float* row = proj + static_cast<size_t>(t0 + (tt < count ? tt : 0)) * ld + head * dim + (r < dim ? r : 0);
      qv[u] = have ? row[q_off] : 0.f;
      kv[u] = have ? row[k_off] : 0.f;
    }
    float vv = 0.f;
    {
      const int tt = lane / kCols, c = lane % kCols;  // 16 tokens x 4 columns: one element a lane
      const int vc = tile * kCols + c;
      if (live && tt < count && vc < v_dim)
        vv = proj[static_cast<size_t>(t0 + tt) * ld + v_off + head * v_dim + vc];
    }
    float gx = 0.f, gy = 0.f;
    if (tid < count) {
      const float* row = proj + static_cast<size_t>(t0 + tid) * ld;
      gx = row[i_off + head] + i_bias[head];
      gy = row[f_off + head] + f_bias[head];
    }
    __syncthreads();  // the tokens staged before have been read
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      const int idx = tid + u * kThreads;
      if (idx < kStage * ROWS) {
        qs[idx / ROWS][idx % ROWS] = qv[u] * q_scale;
        ks[idx / ROWS][idx % ROWS] = kv[u];
      }
    }
    vs[wave][lane / kCols][lane % kCols] = vv;
    if (tid < count) {
      gi[tid] = cap * tanhf(gx / cap);
      gf[tid] = log_sigmoid(cap * tanhf(gy / cap));
    }
    __syncthreads();
    if (!live) continue;
    for (int tt = 0; tt < count; ++tt) {
      const float i_log = gi[tt], f_log = gf[tt];
      const float m_new = fmaxf(f_log + m, i_log);
      const float keep = expf(f_log + m - m_new), take = expf(i_log - m_new);
      const float tv = take * vs[wave][tt][col];
      float o = 0.f, nq = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < RPT; i4 += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(&ks[tt][rg * RPT + i4]);
        const float4 q4 = *reinterpret_cast<const float4*>(&qs[tt][rg * RPT + i4]);
        const float kr[4] = {k4.x, k4.y, k4.z, k4.w}, qr[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          S[i4 + u] = fmaf(keep, S[i4 + u], kr[u] * tv);
          nv[i4 + u] = fmaf(keep, nv[i4 + u], take * kr[u]);
          o = fmaf(S[i4 + u], qr[u], o);
          nq = fmaf(nv[i4 + u], qr[u], nq);
        }
      }
      o = column_sum(o);  // over the sixteen lanes of a column, in a fixed order
      nq = column_sum(nq);
      m = m_new;
      const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (rg == 0 && vcol < v_dim) out[static_cast<size_t>(t0 + tt) * heads * v_dim + head * v_dim + vcol] = o / den;
    }
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    st[i * kWave + lane] = S[i];
    if (col == 0) st[kWave * RPT + i * kRowGroups + rg] = nv[i];
  }
  if (lane == 0) st[kPerTile - 1] = m;
}

// out[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * weight[h, :] * sigmoid(gate[t, h, :]): the
// per-head unit norm of a mixer's readout, its weight and its output gate in one pass.
// One wavefront per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
    headnorm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gate, int gate_ld,
                         const float* __restrict__ weight, float eps, T* __restrict__ out, int n, int heads,
                         int v_dim, int gate_act) {
  const int unit = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (unit >= n * heads) return;
  const int t = unit / heads, h = unit % heads;
  const float* x = o + (static_cast<size_t>(t) * heads + h) * v_dim;
  float sq = 0.f;
  for (int d = lane; d < v_dim; d += kWave) sq = fmaf(x[d], x[d], sq);
  const float r = 1.f / sqrtf(wave_sum(sq) / static_cast<float>(v_dim) + eps);
  const float* g = gate + static_cast<size_t>(t) * gate_ld + h * v_dim;
  T* y = out + (static_cast<size_t>(t) * heads + h) * v_dim;
  for (int d = lane; d < v_dim; d += kWave) {
    const float s = (gate_act == 1 ? g[d] : 1.f) / (1.f + expf(-g[d]));
    y[d] = from_float<T>(x[d] * r * (weight ? weight[h * v_dim + d] : 1.f) * s);
  }
}

}  // namespace shk

using namespace shk;

extern "C" long long shk_mlstm_state_floats(int heads, int dim, int v_dim) {
  const int rpt = scan_rpt(dim);
  return static_cast<long long>(heads) * ((v_dim + kCols - 1) / kCols) * (kWave * rpt + kRowGroups * rpt + 1);
}

extern "C" int shk_mlstm_scan(const float* proj, int ld, int q_off, int k_off, int v_off, int i_off, int f_off,
                              const float* i_bias, const float* f_bias, float cap, float q_scale, int num_seqs,
                              int heads, int dim, int v_dim, const int32_t* positions, const int32_t* cu_q,
                              const int32_t* slots, float* state, long long slot_stride, float* out, void* stream) {
  SHK_REQUIRE(num_seqs >= 0 && heads > 0 && dim > 0 && v_dim > 0, "mlstm_scan: bad sizes seqs=%d heads=%d dim=%d v_dim=%d",
              num_seqs, heads, dim, v_dim);
  SHK_REQUIRE(dim <= 256, "mlstm_scan: heads of %d query/key elements are more than the 256 a wavefront holds", dim);
  SHK_REQUIRE(cap > 0.f, "mlstm_scan: the gates' cap must be positive, got %g", cap);
  SHK_REQUIRE(slot_stride >= shk_mlstm_state_floats(heads, dim, v_dim),
              "mlstm_scan: a slot of %lld floats does not hold the state (%lld)", slot_stride,
              shk_mlstm_state_floats(heads, dim, v_dim));
  const int need = heads * v_dim;
  SHK_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && i_off >= 0 && f_off >= 0 && q_off + heads * dim <= ld &&
                  k_off + heads * dim <= ld && v_off + need <= ld && i_off + heads <= ld && f_off + heads <= ld,
              "mlstm_scan: the projections' columns do not fit rows of %d", ld);
  if (num_seqs == 0) return 0;
  SHK_REQUIRE(num_seqs <= 65535 && heads <= 65535, "mlstm_scan: at most 65535 sequences and heads a call");
  SHK_REQUIRE(proj && i_bias && f_bias && positions && cu_q && slots && state && out, "mlstm_scan: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int tiles = (v_dim + kCols - 1) / kCols;
  dim3 grid((tiles + kScanWaves - 1) / kScanWaves, heads, num_seqs);
#define SHK_SCAN(R)                                                                                          \
  mlstm_scan_kernel<R><<<grid, kScanWaves * kWave, 0, s>>>(proj, ld, q_off, k_off, v_off, i_off, f_off, i_bias, \
                                                           f_bias, cap, q_scale, heads, dim, v_dim, tiles,      \
                                                           positions, cu_q, slots, state, slot_stride, out)
  switch (scan_rpt(dim)) {
    case 4: SHK_SCAN(4); break;
    case 8: SHK_SCAN(8); break;
    default: SHK_SCAN(16); break;
  }
#undef SHK_SCAN
  SHK_LAUNCH_CHECK("mlstm_scan");
  return 0;
}

extern "C" int shk_headnorm_gate(const float* o, const float* gate, int gate_ld, const float* weight, float eps,
                                 void* out, int dtype, int n, int heads, int v_dim, int gate_act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "headnorm_gate: unknown dtype %d", dtype);
  SHK_REQUIRE(gate_act == 0 || gate_act == 1, "headnorm_gate: unknown gate %d (0: sigmoid, 1: SiLU)", gate_act);
  SHK_REQUIRE(n >= 0 && heads > 0 && v_dim > 0 && gate_ld >= heads * v_dim, "headnorm_gate: bad sizes n=%d heads=%d v_dim=%d gate_ld=%d",
              n, heads, v_dim, gate_ld);
  if (n == 0) return 0;
  SHK_REQUIRE(o && gate && out, "headnorm_gate: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long units = static_cast<long long>(n) * heads;
  const int grid = static_cast<int>((units + 3) / 4);
  if (dtype == kF32)
    headnorm_gate_kernel<float><<<grid, 256, 0, s>>>(o, gate, gate_ld, weight, eps, static_cast<float*>(out), n, heads, v_dim, gate_act);
  else
    headnorm_gate_kernel<bf16><<<grid, 256, 0, s>>>(o, gate, gate_ld, weight, eps, static_cast<bf16*>(out), n, heads, v_dim, gate_act);
  SHK_LAUNCH_CHECK("headnorm_gate");
  return 0;
}
