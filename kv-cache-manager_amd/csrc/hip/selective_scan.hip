// Selective scan (a diagonal linear recurrence whose step, input and output maps depend on the token),
// over rows that are packed runs of several sequences, the state of each sequence kept in its slot.
//
//   dt = softplus(dt_lin + dt_bias)                         one step size per channel c
//   S[c, n] <- exp(dt * A[c, n]) * S[c, n] + dt * x_c * B_n,  A = -exp(A_log)
//   y_c = sum_n S[c, n] * C_n + D_c * x_c;   out_c = y_c * silu(z_c)
//
// Everything of the recurrence is 32-bit: the state, the step size with its softplus, the decay's
// exponential, the sums.  The states of a channel are spread over LPC lanes (a power of two, up to a whole
// wave; NPL states a lane beyond that), so that a wave of 64 lanes walks 64 / LPC channels: the run's
// tokens are taken in order, one exponential and two multiply-adds a lane and token, and the sum over a
// channel's states crosses its lanes in a fixed tree.  What a token brings (its step size, input, gate, B
// and C) does not depend on the state: it is requested a few tokens ahead, so that the walk waits for
// arithmetic and not for memory.  A run that starts at position 0 starts from zero without reading its
// slot; the state after the run's last token goes back to the slot.  Tokens are taken one by one in both
// prompts and decoding, so a position's result does not depend on how the prompt was cut.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

// exp of a decay's exponent for a walk whose inputs and outputs are stored as T: exact for float; for bfloat16 the
// hardware's exp2 (about one unit in the last place of a 32-bit value, a tenth of the instructions), which is far
// inside what the storage type keeps of x and of the result.
template <class T> __device__ __forceinline__ float decay_exp(float v);
template <> __device__ __forceinline__ float decay_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float decay_exp<bf16_t>(float v) { return __builtin_amdgcn_exp2f(1.44269504088896341f * v); }

constexpr int kScanAhead = 4;      // tokens whose inputs are on their way while the ones before are computed

template <class T, int LPC, int NPL>
__global__ void __launch_bounds__(kWave)
    selective_scan_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ dt_lin, int lddt,
                          const float* __restrict__ dt_bias, const float* __restrict__ bc, int ldbc, int off_b, int off_c,
                          const float* __restrict__ a_log, const float* __restrict__ dskip, const float* __restrict__ z,
                          int ldz, T* __restrict__ out, int ldo, float* __restrict__ state,
                          const int* __restrict__ run_start, const int* __restrict__ seq_start,
                          const int* __restrict__ state_slots, int C, int N, int prepared, int phase, int chunk_len,
                          float* __restrict__ carry, float* __restrict__ dsum) {
  constexpr int U = kScanAhead;
  const int s = blockIdx.y;
  const int sub = threadIdx.x % LPC;
  const int c_real = blockIdx.x * (kWave / LPC) + threadIdx.x / LPC;
  const bool owns = c_real < C;
  const int c = owns ? c_real : C - 1;      // lanes beyond the last channel walk along (the sums cross lanes) and store nothing
  int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  // phases 1 and 2 walk one piece of chunk_len rows of the run each (blockIdx.z): 1 from zero, leaving the piece's
  // end state and the sum of its step sizes; 2 from the state that enters the piece, writing the outputs
  size_t piece = 0;
  if (phase != 0) {
    piece = size_t(r0 / chunk_len + s) + blockIdx.z;
    r0 += blockIdx.z * chunk_len;
    r1 = r1 < r0 + chunk_len ? r1 : r0 + chunk_len;
  }
  if (r1 <= r0) return;
  if (slot < 0) {      // a padding sequence: its rows carry nothing
    if (owns && sub == 0 && phase != 1)
      for (int r = r0; r < r1; ++r) store_f(out + size_t(r) * ldo + c, 0.f);
    return;
  }
  float* st = phase == 0 ? state + (size_t(slot) * C + c) * N : carry + (piece * C + c) * N;
  const bool fresh = phase == 1 || (phase == 0 && seq_start[s] == 0);
  float S[NPL], A[NPL];
  int nidx[NPL];
  bool has[NPL];
#pragma unroll
  for (int k = 0; k < NPL; ++k) {
    const int n = sub + k * LPC;
    has[k] = n < N;
    nidx[k] = has[k] ? n : N - 1;
    A[k] = has[k] ? -expf(a_log[size_t(c) * N + nidx[k]]) : 0.f;
    S[k] = (has[k] && !fresh) ? st[nidx[k]] : 0.f;
  }
  const float db = dt_bias ? dt_bias[c] : 0.f, dk = dskip[c];

  float dt_total = 0.f;
  float dtv[2][U], xv[2][U], zv[2][U], bv[2][U][NPL], cv[2][U][NPL];
  auto request = [&](int first, int into) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = first + u < r1 ? first + u : r1 - 1;
      dtv[into][u] = dt_lin[size_t(r) * lddt + c];
      xv[into][u] = load_f(x + size_t(r) * ldx + c);
#pragma unroll
      for (int k = 0; k < NPL; ++k) bv[into][u][k] = bc[size_t(r) * ldbc + off_b + nidx[k]];
      if (phase != 1) {      // (the same for every lane) the pass that only wants the state needs neither the gate nor C
        zv[into][u] = z[size_t(r) * ldz + c];
#pragma unroll
        for (int k = 0; k < NPL; ++k) cv[into][u][k] = bc[size_t(r) * ldbc + off_c + nidx[k]];
      }
    }
  };
  auto walk = [&](int first, int from) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = first + u;
      if (r < r1) {
        const float v = dtv[from][u] + db;
        const float dt = prepared ? dtv[from][u] : (v > 20.f ? v : log1pf(expf(v)));
        const float dx = dt * xv[from][u];
        dt_total += dt;
        float y = 0.f;
#pragma unroll
        for (int k = 0; k < NPL; ++k) {
          const float sn = fmaf(decay_exp<T>(dt * A[k]), S[k], dx * bv[from][u][k]);
          S[k] = has[k] ? sn : 0.f;
        }
        if (phase == 1) continue;      // only the state is wanted
#pragma unroll
        for (int k = 0; k < NPL; ++k) y = fmaf(S[k], cv[from][u][k], y);
        y = group_sum<LPC>(y);
        if (owns && sub == 0) {
          y = fmaf(dk, xv[from][u], y);
          const float zz = zv[from][u];
          store_f(out + size_t(r) * ldo + c, y * (prepared ? zz : zz / (1.0f + expf(-zz))));
        }
      }
    }
  };
  request(r0, 0);
  for (int r = r0; r < r1; r += 2 * U) {
    if (r + U < r1) request(r + U, 1);
    walk(r, 0);
    if (r + U < r1) {
      if (r + 2 * U < r1) request(r + 2 * U, 0);
      walk(r + U, 1);
    }
  }
  if (owns && phase != 2) {
#pragma unroll
    for (int k = 0; k < NPL; ++k)
      if (has[k]) st[nidx[k]] = S[k];
    if (phase == 1 && sub == 0) dsum[piece * C + c] = dt_total;
  }
}

// Between the two phases: per (sequence, channel, state) the pieces' end states become the states that enter them,
// S_in[0] = the slot's (zero for a sequence's first portion), S_in[j+1] = exp(A * sum of the piece's step sizes) *
// S_in[j] + end[j]; the last one goes to the slot.
__global__ void __launch_bounds__(256)
    scan_carry_kernel(float* __restrict__ carry, const float* __restrict__ dsum, const float* __restrict__ a_log,
                      float* __restrict__ state, const int* __restrict__ run_start, const int* __restrict__ seq_start,
                      const int* __restrict__ state_slots, int C, int N, int chunk_len) {
  const int s = blockIdx.y;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= C * N) return;
  const int r0 = run_start[s], len = run_start[s + 1] - r0, slot = state_slots[s];
  if (len <= 0 || slot < 0) return;
  const int c = e / N;
  const float A = -expf(a_log[e]);
  float* st = state + size_t(slot) * C * N + e;
  float S = seq_start[s] == 0 ? 0.f : *st;
  const size_t first = size_t(r0 / chunk_len + s);
  const int pieces = (len + chunk_len - 1) / chunk_len;
  for (int j = 0; j < pieces; ++j) {
    float* at = carry + (first + j) * C * N + e;
    const float end = *at;
    *at = S;
    S = fmaf(expf(A * dsum[(first + j) * C + c]), S, end);
  }
  *st = S;
}

// For long runs: the step sizes and the gates of all rows at once, in place (dt <- softplus(dt + bias), z <- silu(z)),
// so that the walk along a run, whose lanes would each repeat them, finds them made.
__global__ void __launch_bounds__(256)
    scan_prepare_kernel(float* __restrict__ dt, int lddt, const float* __restrict__ dt_bias, float* __restrict__ z, int ldz, int C) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const float v = dt[size_t(r) * lddt + c] + (dt_bias ? dt_bias[c] : 0.f);
  dt[size_t(r) * lddt + c] = v > 20.f ? v : log1pf(expf(v));
  const float zz = z[size_t(r) * ldz + c];
  z[size_t(r) * ldz + c] = zz / (1.0f + expf(-zz));
}

template <class T>
int launch_scan(const void* x, int ldx, const float* dt_lin, int lddt, const float* dt_bias, const float* bc, int ldbc,
                int off_b, int off_c, const float* a_log, const float* dskip, const float* z, int ldz, void* out, int ldo,
                float* state, const int* run_start, const int* seq_start, const int* state_slots, int S, int C, int N,
                int prepared, int phase, int chunk_len, int pieces, float* carry, float* dsum, hipStream_t s) {
#define KVCM_SCAN(LPC, NPL)                                                                                             \
  selective_scan_kernel<T, LPC, NPL><<<dim3((C + kWave / LPC - 1) / (kWave / LPC), S, pieces), kWave, 0, s>>>(           \
      static_cast<const T*>(x), ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, off_c, a_log, dskip, z, ldz,               \
      static_cast<T*>(out), ldo, state, run_start, seq_start, state_slots, C, N, prepared, phase, chunk_len, carry, dsum)
  if (N <= 1) KVCM_SCAN(1, 1);
  else if (N <= 2) KVCM_SCAN(2, 1);
  else if (N <= 4) KVCM_SCAN(4, 1);
  else if (N <= 8) KVCM_SCAN(8, 1);
  else if (N <= 16) KVCM_SCAN(16, 1);
  else if (N <= 32) KVCM_SCAN(32, 1);
  else if (N <= 64) KVCM_SCAN(64, 1);
  else if (N <= 128) KVCM_SCAN(64, 2);
  else KVCM_SCAN(64, 4);
#undef KVCM_SCAN
  return launch_status("selective_scan");
}

}  // namespace kvcm

using namespace kvcm;

// x [T, C] (after its convolution and activation) and out [T, C] in the storage type; dt_lin [T, C], bc [T, ldbc]
// (B at off_b, C at off_c, N each), z [T, ldz], a_log [C, N], dt_bias, dskip [C], state [slots, C, N]: 32-bit.
// prepared: dt_lin holds the step sizes and z the gates already (kvcm_scan_prepare).
// chunk_len > 0: runs (of up to max_run rows, T rows in all) are walked in pieces of chunk_len rows, all pieces at once, with
// carry (at least (T / chunk_len + S + 1) * C * (N + 1) floats) between the phases; 0: every run in one walk.
extern "C" int kvcm_selective_scan(const void* x, int dtype, int ldx, const float* dt_lin, int lddt, const float* dt_bias,
                                   const float* bc, int ldbc, int off_b, int off_c, const float* a_log, const float* dskip,
                                   const float* z, int ldz, void* out, int ldo, float* state, const int* run_start,
                                   const int* seq_start, const int* state_slots, int S, int C, int N, int prepared,
                                   int chunk_len, int max_run, float* carry, long long carry_floats, int T, hipStream_t s) {
  if (S == 0) return 0;
  KVCM_REQUIRE(S > 0 && C > 0 && N > 0, "selective_scan: bad sizes S=%d C=%d N=%d", S, C, N);
  KVCM_REQUIRE(N <= 256, "selective_scan: a state of %d per channel is not supported (up to 256)", N);
  KVCM_REQUIRE(S <= 65535, "selective_scan: too many sequences for one launch (%d)", S);
  KVCM_REQUIRE(ldx >= C && lddt >= C && ldz >= C && ldo >= C && off_b >= 0 && off_c >= 0 && ldbc >= off_b + N &&
                   ldbc >= off_c + N, "selective_scan: row strides too small");
  KVCM_REQUIRE(dtype == kF32 || dtype == kBF16, "selective_scan: unknown dtype %d", dtype);
  auto launch = [&](int phase, int pieces, float* cr, float* ds) {
    if (dtype == kF32)
      return launch_scan<float>(x, ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, off_c, a_log, dskip, z, ldz, out, ldo, state,
                                run_start, seq_start, state_slots, S, C, N, prepared, phase, chunk_len, pieces, cr, ds, s);
    return launch_scan<bf16_t>(x, ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, off_c, a_log, dskip, z, ldz, out, ldo, state,
                               run_start, seq_start, state_slots, S, C, N, prepared, phase, chunk_len, pieces, cr, ds, s);
  };
  if (chunk_len <= 0) return launch(0, 1, nullptr, nullptr);
  // long runs in pieces of chunk_len rows: every piece from zero, the states that enter the pieces, every piece again
  KVCM_REQUIRE(prepared, "selective_scan: runs are cut into pieces only with the step sizes made ahead");
  const int pieces = (max_run + chunk_len - 1) / chunk_len;
  const long long slots = static_cast<long long>(T) / chunk_len + S + 1;      // piece j of sequence s: run_start / chunk_len + s + j
  KVCM_REQUIRE(pieces >= 1 && pieces <= 65535 && carry != nullptr && carry_floats >= slots * C * (N + 1),
               "selective_scan: the scratch for %lld pieces is too small", slots);
  float* dsum = carry + slots * C * N;
  if (int rc = launch(1, pieces, carry, dsum)) return rc;
  scan_carry_kernel<<<dim3((C * N + 255) / 256, S), 256, 0, s>>>(carry, dsum, a_log, state, run_start, seq_start, state_slots, C, N,
                                                                 chunk_len);
  if (int rc = launch_status("scan_carry")) return rc;
  return launch(2, pieces, carry, dsum);
  KVCM_REQUIRE(false, "selective_scan: unknown dtype %d", dtype);
}

// dt [T, C] <- softplus(dt + dt_bias), z [T, C] <- silu(z), in place; kvcm_selective_scan then runs with prepared = 1.
extern "C" int kvcm_scan_prepare(float* dt, int lddt, const float* dt_bias, float* z, int ldz, int T, int C, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && C > 0 && lddt >= C && ldz >= C, "scan_prepare: bad sizes T=%d C=%d", T, C);
  KVCM_REQUIRE(T <= 65535, "scan_prepare: too many rows for one launch (%d)", T);
  scan_prepare_kernel<<<dim3((C + 255) / 256, T), 256, 0, s>>>(dt, lddt, dt_bias, z, ldz, C);
  return launch_status("scan_prepare");
}
