// Selective scan (a diagonal linear recurrence whose step, input and output maps depend on the token),
// over rows that are packed runs of several sequences, the state of each sequence kept in its slot.
//
//   dt = softplus(dt_lin + dt_bias)                         one step size per channel c
//   S[c, n] <- exp(dt * A[c, n]) * S[c, n] + dt * x_c * B_n,  A = -exp(A_log)
//   y_c = sum_n S[c, n] * C_n + D_c * x_c;   out_c = y_c * silu(z_c)
//
// Everything of the recurrence is 32-bit: the state, the step size with its softplus, the decay's
// exponential, the sums.  A thread owns one channel of one sequence, keeps that channel's row of the
// state and of A in registers and walks the run's tokens in order; B and C of a token are the same for
// every channel, so a wave's loads of them are broadcasts.  A run that starts at position 0 starts
// from zero without reading its slot; the state after the run's last token goes back to the slot.
// Tokens are taken one by one in both prompts and decoding, so a position's result does not depend on
// how the prompt was cut.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

template <class T, int NP>
__global__ void __launch_bounds__(kWave)
    selective_scan_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ dt_lin, int lddt,
                          const float* __restrict__ dt_bias, const float* __restrict__ bc, int ldbc, int off_b, int off_c,
                          const float* __restrict__ a_log, const float* __restrict__ dskip, const float* __restrict__ z,
                          int ldz, T* __restrict__ out, int ldo, float* __restrict__ state,
                          const int* __restrict__ run_start, const int* __restrict__ seq_start,
                          const int* __restrict__ state_slots, int C, int N) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * kWave + threadIdx.x;
  const int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  if (c >= C || r1 <= r0) return;
  if (slot < 0) {      // a padding sequence: its rows carry nothing
    for (int r = r0; r < r1; ++r) store_f(out + size_t(r) * ldo + c, 0.f);
    return;
  }
  float* st = state + (size_t(slot) * C + c) * N;
  const bool fresh = seq_start[s] == 0;
  float S[NP], A[NP];
#pragma unroll
  for (int n = 0; n < NP; ++n) {
    A[n] = n < N ? -expf(a_log[size_t(c) * N + n]) : 0.f;
    S[n] = (n < N && !fresh) ? st[n] : 0.f;
  }
  const float db = dt_bias ? dt_bias[c] : 0.f, dk = dskip[c];
  for (int r = r0; r < r1; ++r) {
    const float v = dt_lin[size_t(r) * lddt + c] + db;
    const float dt = v > 20.f ? v : log1pf(expf(v));
    const float xv = load_f(x + size_t(r) * ldx + c);
    const float dx = dt * xv;
    const float* brow = bc + size_t(r) * ldbc + off_b;
    const float* crow = bc + size_t(r) * ldbc + off_c;
    float y = 0.f;
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      if (n < N) {
        S[n] = fmaf(expf(dt * A[n]), S[n], dx * brow[n]);
        y = fmaf(S[n], crow[n], y);
      }
    }
    y = fmaf(dk, xv, y);
    const float zv = z[size_t(r) * ldz + c];
    store_f(out + size_t(r) * ldo + c, y * (zv / (1.0f + expf(-zv))));
  }
#pragma unroll
  for (int n = 0; n < NP; ++n)
    if (n < N) st[n] = S[n];
}

template <class T>
int launch_scan(const void* x, int ldx, const float* dt_lin, int lddt, const float* dt_bias, const float* bc, int ldbc,
                int off_b, int off_c, const float* a_log, const float* dskip, const float* z, int ldz, void* out, int ldo,
                float* state, const int* run_start, const int* seq_start, const int* state_slots, int S, int C, int N,
                hipStream_t s) {
  const dim3 grid((C + kWave - 1) / kWave, S);
#define KVCM_SCAN(NP)                                                                                                  \
  selective_scan_kernel<T, NP><<<grid, kWave, 0, s>>>(static_cast<const T*>(x), ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, \
                                                      off_c, a_log, dskip, z, ldz, static_cast<T*>(out), ldo, state,   \
                                                      run_start, seq_start, state_slots, C, N)
  if (N <= 8) KVCM_SCAN(8);
  else if (N <= 16) KVCM_SCAN(16);
  else if (N <= 32) KVCM_SCAN(32);
  else if (N <= 64) KVCM_SCAN(64);
  else KVCM_SCAN(128);
#undef KVCM_SCAN
  return launch_status("selective_scan");
}

}  // namespace kvcm

using namespace kvcm;

// x [T, C] (after its convolution and activation) and out [T, C] in the storage type; dt_lin [T, C], bc [T, ldbc]
// (B at off_b, C at off_c, N each), z [T, ldz], a_log [C, N], dt_bias, dskip [C], state [slots, C, N]: 32-bit.
extern "C" int kvcm_selective_scan(const void* x, int dtype, int ldx, const float* dt_lin, int lddt, const float* dt_bias,
                                   const float* bc, int ldbc, int off_b, int off_c, const float* a_log, const float* dskip,
                                   const float* z, int ldz, void* out, int ldo, float* state, const int* run_start,
                                   const int* seq_start, const int* state_slots, int S, int C, int N, hipStream_t s) {
  if (S == 0) return 0;
  KVCM_REQUIRE(S > 0 && C > 0 && N > 0, "selective_scan: bad sizes S=%d C=%d N=%d", S, C, N);
  KVCM_REQUIRE(N <= 128, "selective_scan: a state of %d per channel is not supported (up to 128)", N);
  KVCM_REQUIRE(S <= 65535, "selective_scan: too many sequences for one launch (%d)", S);
  KVCM_REQUIRE(ldx >= C && lddt >= C && ldz >= C && ldo >= C && off_b >= 0 && off_c >= 0 && ldbc >= off_b + N &&
                   ldbc >= off_c + N, "selective_scan: row strides too small");
  if (dtype == kF32)
    return launch_scan<float>(x, ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, off_c, a_log, dskip, z, ldz, out, ldo, state,
                              run_start, seq_start, state_slots, S, C, N, s);
  if (dtype == kBF16)
    return launch_scan<bf16_t>(x, ldx, dt_lin, lddt, dt_bias, bc, ldbc, off_b, off_c, a_log, dskip, z, ldz, out, ldo, state,
                               run_start, seq_start, state_slots, S, C, N, s);
  KVCM_REQUIRE(false, "selective_scan: unknown dtype %d", dtype);
}
