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
// A run is walked token by token, in prompts and in decoding.  Only m_t = max(lf_t + m_(t-1), li_t) has to go first, and it
// is a chain of one addition and one maximum a token: a launch with one lane per (sequence, head) walks it and leaves
// (li, lf, m_(t-1), m_t) per row (for runs of 16 rows or more the two logarithms of all rows are made before that, in
// parallel, so that no tanh or log1p sits in the chain).  The main walk needs no transcendental function in its chain: the
// three exponentials of a token are evaluated as its values are staged.  A value column j of S needs nothing of another
// column, so columns are spread over lanes and workgroups, the key dimension of a column over G lanes; every workgroup
// carries n along beside its columns (n is a column of S whose value is always one) and sums n . q like any column's
// output.  The per-token vectors (q, k, v of these columns, the three factors) are staged through LDS a few tokens at a
// time, the next tokens' values requested before the current ones are computed.  All workgroups of a head read the old n
// from the slot; the first one leaves the new n in scratch, and a small launch moves it to the slot afterwards, so that
// no workgroup reads a state that another one of the same launch writes.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

__device__ __forceinline__ float soft_cap(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

constexpr int kGateTile = 8;

// For steps with long runs the gates' logarithms of all rows are made first, in parallel: coef[row, head] = (li, lf, ., .).
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

// one lane per (sequence, head): coef[row, head] = (li, lf, m before the row, m after it) for every row of the run; the
// slot's m is read at the start (a run that starts at position 0 starts from 0) and written at the end.
__global__ void __launch_bounds__(kWave)
    mlstm_max_kernel(const float* __restrict__ ig, int ldi, const float* __restrict__ fg, int ldf,
                     const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float4* __restrict__ coef,
                     float* __restrict__ m_state, const int* __restrict__ run_start, const int* __restrict__ seq_start,
                     const int* __restrict__ state_slots, int S, int heads, int logs_ready) {
  const int idx = blockIdx.x * kWave + threadIdx.x;
  if (idx >= S * heads) return;
  const int s = idx / heads, head = idx % heads;
  const int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  if (r1 <= r0) return;
  if (slot < 0) {
    for (int row = r0; row < r1; ++row) coef[size_t(row) * heads + head] = float4{0.f, 0.f, 0.f, 0.f};
    return;
  }
  float* mst = m_state + size_t(slot) * heads + head;
  float m = seq_start[s] == 0 ? 0.f : *mst;
  const float ib = i_bias[head], fb = f_bias[head];
  for (int t0 = r0; t0 < r1; t0 += kGateTile) {
    float li[kGateTile], lf[kGateTile];
#pragma unroll
    for (int t = 0; t < kGateTile; ++t) {      // the tile's loads first, from clamped places
      const int row = t0 + t < r1 ? t0 + t : r1 - 1;
      if (logs_ready) {
        const float4 c = coef[size_t(row) * heads + head];
        li[t] = c.x;
        lf[t] = c.y;
      } else {
        li[t] = ig[size_t(row) * ldi + head];
        lf[t] = fg[size_t(row) * ldf + head];
      }
    }
#pragma unroll
    for (int t = 0; t < kGateTile; ++t) {
      if (t0 + t >= r1) break;
      const float a = logs_ready ? li[t] : soft_cap(li[t] + ib, cap);
      const float f = logs_ready ? lf[t] : log_sigmoid(soft_cap(lf[t] + fb, cap));
      const float m_new = fmaxf(f + m, a);
      coef[size_t(t0 + t) * heads + head] = float4{a, f, m, m_new};
      m = m_new;
    }
  }
  *mst = m;
}

template <int DKP, int G, int TILE>
__global__ void __launch_bounds__(256)
    mlstm_scan_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v,
                      int ldv, const float4* __restrict__ coef, float q_scale, float* __restrict__ o, int ldo,
                      float* __restrict__ s_state, const float* __restrict__ n_state, float* __restrict__ n_new,
                      const int* __restrict__ run_start, const int* __restrict__ seq_start,
                      const int* __restrict__ state_slots, int heads, int dk, int dv, int col_blocks) {
  constexpr int IPT = DKP / G, CB = 256 / G, W = 2 * DKP + CB + 3;
  constexpr int PF = (TILE * (2 * DKP + CB) + 255) / 256;
  static_assert(TILE <= 256, "one thread stages a token's factors");
  __shared__ __attribute__((aligned(16))) float tile[TILE][W];      // per token: q (scaled), k (zero beyond dk), v of these columns, keep, take, exp(-m)
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
  const float* nst = n_state + (size_t(slot) * heads + head) * dk;
  const bool fresh = seq_start[s] == 0;
  float S[IPT], N[IPT];
#pragma unroll
  for (int il = 0; il < IPT; ++il) {
    const int i = g * IPT + il;
    S[il] = (i < dk && owns && !fresh) ? st[size_t(i) * dv] : 0.f;
    N[il] = (i < dk && !fresh) ? nst[i] : 0.f;
  }
  constexpr int V = 2 * DKP + CB;      // the vectors of a token; its three factors follow
  float pf[PF];
  float4 cf;
  auto request = [&](int t0) {      // unconditional loads from clamped places, masked afterwards
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int e = threadIdx.x + p * 256;
      const int t = e / V, off = e % V;
      const int row = t0 + t < r1 ? t0 + t : r1 - 1;
      const bool vec = off < 2 * DKP;
      const int which = off / DKP, i = off % DKP;
      const int jj = cb * CB + (off - 2 * DKP);
      const bool ok = t < TILE && t0 + t < r1 && (vec ? i < dk : jj < dv);
      const size_t col = size_t(head) * dk + (i < dk ? i : dk - 1);
      const size_t vcol = size_t(head) * dv + ((jj >= 0 && jj < dv) ? jj : 0);
      const float* src = !vec ? v + size_t(row) * ldv + vcol : which == 0 ? q + size_t(row) * ldq + col : k + size_t(row) * ldk + col;
      const float val = *src;
      pf[p] = ok ? (off < DKP ? val * q_scale : val) : 0.f;
    }
    const int t = threadIdx.x < TILE ? threadIdx.x : TILE - 1;
    cf = coef[size_t(t0 + t < r1 ? t0 + t : r1 - 1) * heads + head];
  };
  auto stage = [&]() {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int e = threadIdx.x + p * 256;
      if (e < TILE * V) tile[e / V][e % V] = pf[p];
    }
    if (threadIdx.x < TILE) {      // (li, lf, m before, m after) -> the token's three factors
      tile[threadIdx.x][V] = expf(cf.y + cf.z - cf.w);
      tile[threadIdx.x][V + 1] = expf(cf.x - cf.w);
      tile[threadIdx.x][V + 2] = expf(-cf.w);
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
      const float keep = tv[V], take = tv[V + 1], floor_ = tv[V + 2];
      const float vj = take * tv[2 * DKP + threadIdx.x / G];
      float acc = 0.f, nq = 0.f;
#pragma unroll
      for (int il = 0; il < IPT; ++il) {
        const int i = g * IPT + il;
        const float kd = tv[DKP + i], qd = tv[i];
        S[il] = fmaf(keep, S[il], kd * vj);
        N[il] = fmaf(keep, N[il], take * kd);
        acc = fmaf(S[il], qd, acc);
        nq = fmaf(N[il], qd, nq);
      }
      acc = group_sum<G>(acc);
      nq = group_sum<G>(nq);
      if (owns && g == 0) o[size_t(t0 + t) * ldo + size_t(head) * dv + j] = acc / (fmaxf(fabsf(nq), floor_) + 1e-6f);
    }
    __syncthreads();
    if (more) stage();
    __syncthreads();
  }
#pragma unroll
  for (int il = 0; il < IPT; ++il) {
    const int i = g * IPT + il;
    if (i < dk && owns) st[size_t(i) * dv] = S[il];
    if (i < dk && cb == 0 && threadIdx.x < G) n_new[(size_t(s) * heads + head) * dk + i] = N[il];
  }
}

// n_state[slot of sequence s] = n_new[s] for the sequences that ran
__global__ void __launch_bounds__(256)
    mlstm_keep_n_kernel(const float* __restrict__ n_new, float* __restrict__ n_state, const int* __restrict__ run_start,
                        const int* __restrict__ state_slots, int S, int per_seq) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= S * per_seq) return;
  const int s = idx / per_seq, slot = state_slots[s];
  if (slot < 0 || run_start[s + 1] <= run_start[s]) return;
  n_state[size_t(slot) * per_seq + idx % per_seq] = n_new[idx];
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// q, k [T, heads*dk], v [T, heads*dv], ig, fg [T, heads] (the gates' projections without their biases), at their own
// strides; i_bias, f_bias [heads]; coef: scratch of 4 T heads floats (T: the step's rows, max_run: its longest run); n_new:
// scratch of S heads dk floats; o [T, >= heads*dv]; s_state [slots, heads, dk, dv], n_state [slots, heads, dk],
// m_state [slots, heads]; all 32-bit.
int kvcm_mlstm_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* ig, int ldi,
                    const float* fg, int ldf, const float* i_bias, const float* f_bias, float cap, float q_scale, float* coef,
                    float* n_new, float* o, int ldo, float* s_state, float* n_state, float* m_state, const int* run_start,
                    const int* seq_start, const int* state_slots, int S, int heads, int dk, int dv, int T, int max_run,
                    hipStream_t s) {
  if (S == 0) return 0;
  KVCM_REQUIRE(S > 0 && heads > 0 && dk > 0 && dv > 0, "mlstm_scan: bad sizes S=%d heads=%d dk=%d dv=%d", S, heads, dk, dv);
  KVCM_REQUIRE(dk <= 256, "mlstm_scan: a key size of %d is not supported (up to 256)", dk);
  KVCM_REQUIRE(cap > 0.f, "mlstm_scan: the gates' cap must be positive (%g)", cap);
  KVCM_REQUIRE(static_cast<long long>(heads) * ((dv + 15) / 16) < (1ll << 31), "mlstm_scan: too many heads");
  KVCM_REQUIRE(S <= 65535 && static_cast<long long>(S) * heads * dk < (1ll << 31), "mlstm_scan: too many sequences for one launch (%d)", S);
  KVCM_REQUIRE(ldq >= heads * dk && ldk >= heads * dk && ldv >= heads * dv && ldo >= heads * dv && ldi >= heads && ldf >= heads,
               "mlstm_scan: row strides too small");
  KVCM_REQUIRE(coef && n_new && reinterpret_cast<uintptr_t>(coef) % 16 == 0, "mlstm_scan: the scratch must be there, 16-byte aligned");
  float4* cf = reinterpret_cast<float4*>(coef);
  const int logs_first = max_run >= 16 ? 1 : 0;      // long runs: the gates' logarithms of all T rows first, in parallel
  if (logs_first) {
    KVCM_REQUIRE(T > 0, "mlstm_scan: the row count is needed for runs of %d", max_run);
    const long long n = static_cast<long long>(T) * heads;
    mlstm_gate_logs_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(ig, ldi, fg, ldf, i_bias, f_bias, cap, cf, n, heads);
  }
  mlstm_max_kernel<<<(S * heads + kWave - 1) / kWave, kWave, 0, s>>>(ig, ldi, fg, ldf, i_bias, f_bias, cap, cf, m_state, run_start,
                                                                      seq_start, state_slots, S, heads, logs_first);
#define KVCM_MLSTM(DKP, G, TILE)                                                                                             \
  {                                                                                                                          \
    const int col_blocks = (dv + 256 / G - 1) / (256 / G);                                                                   \
    mlstm_scan_kernel<DKP, G, TILE><<<dim3(heads * col_blocks, S), 256, 0, s>>>(q, ldq, k, ldk, v, ldv, cf, q_scale, o, ldo,  \
                                                                                s_state, n_state, n_new, run_start,          \
                                                                                seq_start, state_slots, heads, dk, dv,       \
                                                                                col_blocks);                                 \
  }
  if (dk <= 16) KVCM_MLSTM(16, 4, 8)
  else if (dk <= 32) KVCM_MLSTM(32, 8, 8)
  else if (dk <= 64) KVCM_MLSTM(64, 8, 8)
  else if (dk <= 128) KVCM_MLSTM(128, 16, 8)
  else KVCM_MLSTM(256, 16, 4)
#undef KVCM_MLSTM
  const int per_seq = heads * dk;
  mlstm_keep_n_kernel<<<(S * per_seq + 255) / 256, 256, 0, s>>>(n_new, n_state, run_start, state_slots, S, per_seq);
  return launch_status("mlstm_scan");
}

}  // extern "C"
