// The matrix memory of an mLSTM layer: per head a matrix S [dim, v_dim], a vector n
// [dim] and a running maximum m, all float32, carried from token to token in the
// request's state slot:
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T       (n_t likewise, with k_t alone)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// with log gates i_t = cap tanh(x / cap) and f_t = logsigmoid(cap tanh(y / cap)) of the
// gates' projections x, y (bias added here).  The state before position 0 is zero (m = 0).
//
// mlstm_scan_kernel: one wavefront per (sequence, head, 16 value columns).  A lane owns
// one column and every fourth row of S in registers; a token costs dim / 4 multiply-adds
// a lane for S and as many for the readout, whose four partial sums meet by two lane
// swaps.  Tokens are staged eight at a time through LDS (queries, keys, the 16 values,
// the gates) so that the recurrence never waits for global memory.  Every wavefront
// keeps n and m for itself (its own copy in the state), so no two wavefronts share
// anything that one of them writes.  Prompt portions and single tokens take this one
// path: a token's result does not depend on how its sequence was cut into steps.
//
// State of one (slot, layer): [heads][tiles][dim * 16 + dim + 1] floats, tiles =
// ceil(v_dim / 16): the tile's columns of S row by row, then n, then m.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kCols = 16;      // value columns per wavefront
constexpr int kRowGroups = 4;  // lanes that share a column take every fourth row
constexpr int kStage = 8;      // tokens staged at a time

__device__ __forceinline__ float log_sigmoid(float x) {
  return x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
}

template <int RPT>  // rows per lane: dim <= 4 * RPT
__global__ void __launch_bounds__(kWave)
    mlstm_scan_kernel(const float* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int i_off,
                      int f_off, const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                      float q_scale, int heads, int dim, int v_dim, const int32_t* __restrict__ positions,
                      const int32_t* __restrict__ cu_q, const int32_t* __restrict__ slots,
                      float* __restrict__ state, long long slot_stride, float* __restrict__ out) {
  __shared__ float qs[kStage][4 * RPT];
  __shared__ float ks[kStage][4 * RPT];
  __shared__ float vs[kStage][kCols];
  __shared__ float gi[kStage], gf[kStage];

  const int tile = blockIdx.x, head = blockIdx.y, seq = blockIdx.z;
  const int tiles = gridDim.x;
  const int lane = threadIdx.x, col = lane % kCols, rg = lane / kCols;
  const int vcol = tile * kCols + col;
  const int first = cu_q[seq], last = cu_q[seq + 1];
  const int per_tile = dim * kCols + dim + 1;
  float* st = state + static_cast<size_t>(slots[seq]) * slot_stride +
              (static_cast<size_t>(head) * tiles + tile) * per_tile;

  float S[RPT], nv[RPT], m = 0.f;
  const bool fresh = positions[first] == 0;  // nothing precedes position 0
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg + kRowGroups * i;
    const bool have = !fresh && r < dim;
    S[i] = have ? st[r * kCols + col] : 0.f;
    nv[i] = have ? st[dim * kCols + r] : 0.f;
  }
  if (!fresh) m = st[dim * kCols + dim];

  for (int t0 = first; t0 < last; t0 += kStage) {
    const int count = last - t0 < kStage ? last - t0 : kStage;
    __syncthreads();  // the tokens staged before have been read
    for (int idx = lane; idx < count * 4 * RPT; idx += kWave) {
      const int tt = idx / (4 * RPT), r = idx % (4 * RPT);
      const float* row = proj + static_cast<size_t>(t0 + tt) * ld + head * dim;
      qs[tt][r] = r < dim ? row[q_off + r] * q_scale : 0.f;
      ks[tt][r] = r < dim ? row[k_off + r] : 0.f;
    }
    for (int idx = lane; idx < count * kCols; idx += kWave) {
      const int tt = idx / kCols, c = idx % kCols;
      const int vc = tile * kCols + c;
      vs[tt][c] = vc < v_dim ? proj[static_cast<size_t>(t0 + tt) * ld + v_off + head * v_dim + vc] : 0.f;
    }
    if (lane < count) {
      const float* row = proj + static_cast<size_t>(t0 + lane) * ld;
      const float x = row[i_off + head] + i_bias[head], y = row[f_off + head] + f_bias[head];
      gi[lane] = cap * tanhf(x / cap);
      gf[lane] = log_sigmoid(cap * tanhf(y / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      const float i_log = gi[tt], f_log = gf[tt];
      const float m_new = fmaxf(f_log + m, i_log);
      const float keep = expf(f_log + m - m_new), take = expf(i_log - m_new);
      const float tv = take * vs[tt][col];
      float o = 0.f, nq = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const int r = rg + kRowGroups * i;
        const float kr = ks[tt][r], qr = qs[tt][r];
        S[i] = fmaf(keep, S[i], kr * tv);
        nv[i] = fmaf(keep, nv[i], take * kr);
        o = fmaf(S[i], qr, o);
        nq = fmaf(nv[i], qr, nq);
      }
      o += __shfl_xor(o, 16, kWave);
      o += __shfl_xor(o, 32, kWave);
      nq += __shfl_xor(nq, 16, kWave);
      nq += __shfl_xor(nq, 32, kWave);
      m = m_new;
      const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (rg == 0 && vcol < v_dim) out[static_cast<size_t>(t0 + tt) * heads * v_dim + head * v_dim + vcol] = o / den;
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg + kRowGroups * i;
    if (r < dim) {
      st[r * kCols + col] = S[i];
      if (col == 0) st[dim * kCols + r] = nv[i];
    }
  }
  if (lane == 0) st[dim * kCols + dim] = m;
}

// out[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * weight[h, :] * sigmoid(gate[t, h, :]): the
// per-head unit norm of a mixer's readout, its weight and its output gate in one pass.
// One wavefront per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
    headnorm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gate, int gate_ld,
                         const float* __restrict__ weight, float eps, T* __restrict__ out, int n, int heads,
                         int v_dim) {
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
    const float s = 1.f / (1.f + expf(-g[d]));
    y[d] = from_float<T>(x[d] * r * weight[h * v_dim + d] * s);
  }
}

}  // namespace shk

using namespace shk;

extern "C" long long shk_mlstm_state_floats(int heads, int dim, int v_dim) {
  return static_cast<long long>(heads) * ((v_dim + kCols - 1) / kCols) * (static_cast<long long>(dim) * kCols + dim + 1);
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
  dim3 grid((v_dim + kCols - 1) / kCols, heads, num_seqs);
#define SHK_SCAN(R)                                                                                              \
  mlstm_scan_kernel<R><<<grid, kWave, 0, s>>>(proj, ld, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, \
                                              q_scale, heads, dim, v_dim, positions, cu_q, slots, state,       \
                                              slot_stride, out)
  if (dim <= 32) SHK_SCAN(8);
  else if (dim <= 64) SHK_SCAN(16);
  else if (dim <= 128) SHK_SCAN(32);
  else SHK_SCAN(64);
#undef SHK_SCAN
  SHK_LAUNCH_CHECK("mlstm_scan");
  return 0;
}

extern "C" int shk_headnorm_gate(const float* o, const float* gate, int gate_ld, const float* weight, float eps,
                                 void* out, int dtype, int n, int heads, int v_dim, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "headnorm_gate: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && v_dim > 0 && gate_ld >= heads * v_dim, "headnorm_gate: bad sizes n=%d heads=%d v_dim=%d gate_ld=%d",
              n, heads, v_dim, gate_ld);
  if (n == 0) return 0;
  SHK_REQUIRE(o && gate && weight && out, "headnorm_gate: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long units = static_cast<long long>(n) * heads;
  const int grid = static_cast<int>((units + 3) / 4);
  if (dtype == kF32)
    headnorm_gate_kernel<float><<<grid, 256, 0, s>>>(o, gate, gate_ld, weight, eps, static_cast<float*>(out), n, heads, v_dim);
  else
    headnorm_gate_kernel<bf16><<<grid, 256, 0, s>>>(o, gate, gate_ld, weight, eps, static_cast<bf16*>(out), n, heads, v_dim);
  SHK_LAUNCH_CHECK("headnorm_gate");
  return 0;
}
