// A matrix memory with exponential gates (the mLSTM cell): per head a state S [dk, dv], a normalizer n [dk] and
// a running maximum m of the gates' logarithms, which keeps every exponential at or below one:
//
//   li = cap * tanh((i_lin + i_bias) / cap)                      log of the input gate
//   lf = logsigmoid(cap * tanh((f_lin + f_bias) / cap))          log of the forget gate
//   m' = max(lf + m, li)
//   S' = exp(lf + m - m') S + exp(li - m') k v^T        n' = exp(lf + m - m') n + exp(li - m') k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)               q comes scaled by q_scale
//
// S, n and m start at zero (m at 0, not at minus infinity), are 32-bit and live in the request's state slot.
// A run is walked token by token, in prompts and in decoding.  Two launches.  The first walks what does not depend on
// the values: one wave per (sequence, head) carries n and m along and leaves, per token, the two factors
// exp(lf + m - m'), exp(li - m') and 1 / denominator (the gates' transcendental functions are evaluated there, once per
// token).  The second walks S: a value column j of S needs nothing of another column, so columns are spread over
// lanes and workgroups, the key dimension of a column over G lanes; the per-token vectors (q, k, v of these columns,
// the three factors) are staged through LDS a few tokens at a time, the next tokens' values requested before the
// current ones are computed.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

__device__ __forceinline__ float soft_cap(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

constexpr int kGateTile = 8;
constexpr int kGateMaxPerLane = 4;      // dk up to 256 over 64 lanes

// For steps with long runs the gates' logarithms of all rows are made first, in parallel: coef[row, head] = (li, lf, ., .);
// the walk below then has no transcendental function but its three exponentials a token.
__global__ void __launch_bounds__(256)
    mlstm_gate_logs_kernel(const float* __restrict__ ig, int ldi, const float* __restrict__ fg, int ldf,
                           const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                           float4* __restrict__ coef, long long n, int heads) {
  const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= n) return;
  const long long row = idx / heads;
  const int head = static_cast<int>(idx % heads);
  coef[idx] = float4{soft_cap(ig[row * ldi + head] + i_bias[head], cap), log_sigmoid(soft_cap(fg[row * ldf + head] + f_bias[head], cap)),
                     0.f, 0.f};
}

// one wave per (sequence, head): coef[row, head] = (keep, take, 1 / den, m) for every row of the run.  PER: key entries
// a lane carries (dk <= 64 PER).  The values of the next eight tokens are on their way while the current eight are walked.
template <int PER>
__global__ void __launch_bounds__(kWave)
    mlstm_gates_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk,
                       const float* __restrict__ ig, int ldi, const float* __restrict__ fg, int ldf,
                       const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
                       float4* __restrict__ coef, float* __restrict__ n_state, float* __restrict__ m_state,
                       const int* __restrict__ run_start, const int* __restrict__ seq_start,
                       const int* __restrict__ state_slots, int heads, int dk, int logs_ready) {
  const int head = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
  const int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  if (r1 <= r0) return;
  if (slot < 0) {
    for (int row = r0 + lane; row < r1; row += kWave) coef[size_t(row) * heads + head] = float4{0.f, 0.f, 0.f, 0.f};
    return;
  }
  float* nst = n_state + (size_t(slot) * heads + head) * dk;
  float* mst = m_state + size_t(slot) * heads + head;
  const bool fresh = seq_start[s] == 0;
  float N[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = lane + e * kWave;
    N[e] = (i < dk && !fresh) ? nst[i] : 0.f;
  }
  float m = fresh ? 0.f : *mst;
  const float ib = i_bias[head], fb = f_bias[head];
  float qv[2][kGateTile][PER], kv[2][kGateTile][PER], gi[2][kGateTile], gf[2][kGateTile];
  auto request = [&](int t0, int buf) {      // unconditional loads from clamped places, masked afterwards
#pragma unroll
    for (int t = 0; t < kGateTile; ++t) {
      const int row = t0 + t < r1 ? t0 + t : r1 - 1;
      if (logs_ready) {
        const float4 c = coef[size_t(row) * heads + head];
        gi[buf][t] = c.x;
        gf[buf][t] = c.y;
      } else {
        gi[buf][t] = ig[size_t(row) * ldi + head];
        gf[buf][t] = fg[size_t(row) * ldf + head];
      }
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        const int i = lane + e * kWave;
        const size_t col = size_t(head) * dk + (i < dk ? i : dk - 1);
        const float a = q[size_t(row) * ldq + col], b = k[size_t(row) * ldk + col];
        qv[buf][t][e] = i < dk ? a * q_scale : 0.f;
        kv[buf][t][e] = i < dk ? b : 0.f;
      }
    }
  };
  auto walk = [&](int t0, int buf) {
#pragma unroll
    for (int t = 0; t < kGateTile; ++t) {
      if (t0 + t >= r1) break;
      const float li = logs_ready ? gi[buf][t] : soft_cap(gi[buf][t] + ib, cap);
      const float lf = logs_ready ? gf[buf][t] : log_sigmoid(soft_cap(gf[buf][t] + fb, cap));
      const float m_new = fmaxf(lf + m, li);
      const float keep = expf(lf + m - m_new), take = expf(li - m_new);
      m = m_new;
      float nq = 0.f;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        N[e] = fmaf(keep, N[e], take * kv[buf][t][e]);
        nq = fmaf(N[e], qv[buf][t][e], nq);
      }
      nq = wave_sum(nq);
      const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (lane == 0) coef[size_t(t0 + t) * heads + head] = float4{keep, take, 1.0f / den, m};
    }
  };
  // (a row's own (li, lf) in coef is read before its place is overwritten: the tile that is walked was requested
  // a whole tile earlier, and the one requested meanwhile lies behind it)
  request(r0, 0);
  for (int t0 = r0; t0 < r1; t0 += 2 * kGateTile) {
    if (t0 + kGateTile < r1) request(t0 + kGateTile, 1);
    walk(t0, 0);
    if (t0 + kGateTile >= r1) break;
    if (t0 + 2 * kGateTile < r1) request(t0 + 2 * kGateTile, 0);
    walk(t0 + kGateTile, 1);
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = lane + e * kWave;
    if (i < dk) nst[i] = N[e];
  }
  if (lane == 0) *mst = m;
}

template <int DKP, int G, int TILE>
__global__ void __launch_bounds__(256)
    mlstm_scan_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v,
                      int ldv, const float4* __restrict__ coef, float q_scale, float* __restrict__ o, int ldo,
                      float* __restrict__ s_state, const int* __restrict__ run_start, const int* __restrict__ seq_start,
                      const int* __restrict__ state_slots, int heads, int dk, int dv, int col_blocks) {
  constexpr int IPT = DKP / G, CB = 256 / G, W = 2 * DKP + CB + 3;
  constexpr int PF = (TILE * W + 255) / 256;
  __shared__ __attribute__((aligned(16))) float tile[TILE][W];      // per token: q (scaled), k (zero beyond dk), v of these columns, keep, take, 1/den
  const int s = blockIdx.y, head = blockIdx.x / col_blocks, cb = blockIdx.x % col_blocks;
  const int g = threadIdx.x % G, j = cb * CB + threadIdx.x / G;
  const int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  if (r1 <= r0) return;
  const bool owns = j < dv;
  if (slot < 0) {
    if (owns && g == 0)
      for (int row = r0; row < r1; ++row) o[size_t(row) * ldo + size_t(head) * dv + j] = 0.f;
    return;
  }
  float* st = s_state + ((size_t(slot) * heads + head) * dk) * dv + (owns ? j : 0);      // [slot][head][i][j]
  const bool fresh = seq_start[s] == 0;
  float S[IPT];
#pragma unroll
  for (int il = 0; il < IPT; ++il) {
    const int i = g * IPT + il;
    S[il] = (i < dk && owns && !fresh) ? st[size_t(i) * dv] : 0.f;
  }
  float pf[PF];
  const float* cf = reinterpret_cast<const float*>(coef);
  auto request = [&](int t0) {      // unconditional loads from clamped places, masked afterwards
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int e = threadIdx.x + p * 256;
      const int t = e / W, off = e % W;
      const int row = t0 + t < r1 ? t0 + t : r1 - 1;
      const bool vec = off < 2 * DKP, fac = off >= 2 * DKP + CB;
      const int which = off / DKP, i = off % DKP;
      const int jj = cb * CB + (off - 2 * DKP);
      const bool ok = t < TILE && t0 + t < r1 && (vec ? i < dk : (fac || jj < dv));
      const size_t col = size_t(head) * dk + (i < dk ? i : dk - 1);
      const size_t vcol = size_t(head) * dv + ((jj >= 0 && jj < dv) ? jj : 0);
      const float* src = fac ? cf + (size_t(row) * heads + head) * 4 + (off - 2 * DKP - CB)
                         : !vec ? v + size_t(row) * ldv + vcol
                         : which == 0 ? q + size_t(row) * ldq + col
                                      : k + size_t(row) * ldk + col;
      const float val = *src;
      pf[p] = ok ? (off < DKP ? val * q_scale : val) : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int e = threadIdx.x + p * 256;
      if (e < TILE * W) tile[e / W][e % W] = pf[p];
    }
  };
  request(r0);
  stage();
  __syncthreads();
  for (int t0 = r0; t0 < r1; t0 += TILE) {
    const int nt = r1 - t0 < TILE ? r1 - t0 : TILE;
    const bool more = t0 + TILE < r1;
    if (more) request(t0 + TILE);
    for (int t = 0; t < nt; ++t) {
      const float* tv = tile[t];
      const float keep = tv[2 * DKP + CB], take = tv[2 * DKP + CB + 1], inv_den = tv[2 * DKP + CB + 2];
      const float vj = take * tv[2 * DKP + threadIdx.x / G];
      float acc = 0.f;
#pragma unroll
      for (int il = 0; il < IPT; ++il) {
        const int i = g * IPT + il;
        S[il] = fmaf(keep, S[il], tv[DKP + i] * vj);
        acc = fmaf(S[il], tv[i], acc);
      }
      acc = group_sum<G>(acc);
      if (owns && g == 0) o[size_t(t0 + t) * ldo + size_t(head) * dv + j] = acc * inv_den;
    }
    __syncthreads();
    if (more) stage();
    __syncthreads();
  }
  if (owns) {
#pragma unroll
    for (int il = 0; il < IPT; ++il) {
      const int i = g * IPT + il;
      if (i < dk) st[size_t(i) * dv] = S[il];
    }
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// q, k [T, heads*dk], v [T, heads*dv], ig, fg [T, heads] (the gates' projections without their biases), at their own
// strides; i_bias, f_bias [heads]; coef: scratch of 4 T heads floats (T: the step's rows, max_run: its longest run); o [T, >= heads*dv]; s_state [slots, heads, dk, dv],
// n_state [slots, heads, dk], m_state [slots, heads]; all 32-bit.
int kvcm_mlstm_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* ig, int ldi,
                    const float* fg, int ldf, const float* i_bias, const float* f_bias, float cap, float q_scale, float* coef,
                    float* o, int ldo, float* s_state, float* n_state, float* m_state, const int* run_start,
                    const int* seq_start, const int* state_slots, int S, int heads, int dk, int dv, int T, int max_run,
                    hipStream_t s) {
  if (S == 0) return 0;
  KVCM_REQUIRE(S > 0 && heads > 0 && dk > 0 && dv > 0, "mlstm_scan: bad sizes S=%d heads=%d dk=%d dv=%d", S, heads, dk, dv);
  KVCM_REQUIRE(dk <= kGateMaxPerLane * kWave, "mlstm_scan: a key size of %d is not supported (up to %d)", dk, kGateMaxPerLane * kWave);
  KVCM_REQUIRE(cap > 0.f, "mlstm_scan: the gates' cap must be positive (%g)", cap);
  KVCM_REQUIRE(static_cast<long long>(heads) * ((dv + 15) / 16) < (1ll << 31), "mlstm_scan: too many heads");
  KVCM_REQUIRE(S <= 65535, "mlstm_scan: too many sequences for one launch (%d)", S);
  KVCM_REQUIRE(ldq >= heads * dk && ldk >= heads * dk && ldv >= heads * dv && ldo >= heads * dv && ldi >= heads && ldf >= heads,
               "mlstm_scan: row strides too small");
  KVCM_REQUIRE(coef && reinterpret_cast<uintptr_t>(coef) % 16 == 0, "mlstm_scan: the factors' scratch must be 16-byte aligned");
  float4* cf = reinterpret_cast<float4*>(coef);
  const int logs_first = max_run >= 16 ? 1 : 0;      // long runs: the gates' logarithms of all T rows first, in parallel
  if (logs_first) {
    KVCM_REQUIRE(T > 0, "mlstm_scan: the row count is needed for runs of %d", max_run);
    const long long n = static_cast<long long>(T) * heads;
    mlstm_gate_logs_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(ig, ldi, fg, ldf, i_bias, f_bias, cap, cf, n, heads);
  }
#define KVCM_MLSTM_GATES(PER)                                                                                                 \
  mlstm_gates_kernel<PER><<<dim3(heads, S), kWave, 0, s>>>(q, ldq, k, ldk, ig, ldi, fg, ldf, i_bias, f_bias, cap, q_scale, cf, \
                                                           n_state, m_state, run_start, seq_start, state_slots, heads, dk,    \
                                                           logs_first)
  if (dk <= kWave) KVCM_MLSTM_GATES(1);
  else if (dk <= 2 * kWave) KVCM_MLSTM_GATES(2);
  else KVCM_MLSTM_GATES(4);
#undef KVCM_MLSTM_GATES
#define KVCM_MLSTM(DKP, G, TILE)                                                                                             \
  {                                                                                                                          \
    const int col_blocks = (dv + 256 / G - 1) / (256 / G);                                                                   \
    mlstm_scan_kernel<DKP, G, TILE><<<dim3(heads * col_blocks, S), 256, 0, s>>>(q, ldq, k, ldk, v, ldv, cf, q_scale, o, ldo,  \
                                                                                s_state, run_start, seq_start, state_slots,  \
                                                                                heads, dk, dv, col_blocks);                  \
  }
  if (dk <= 16) KVCM_MLSTM(16, 4, 8)
  else if (dk <= 32) KVCM_MLSTM(32, 8, 8)
  else if (dk <= 64) KVCM_MLSTM(64, 8, 8)
  else if (dk <= 128) KVCM_MLSTM(128, 16, 8)
  else KVCM_MLSTM(256, 16, 4)
#undef KVCM_MLSTM
  return launch_status("mlstm_scan");
}

}  // extern "C"
