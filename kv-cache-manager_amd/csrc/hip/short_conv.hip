// A short causal convolution over time on every channel, for rows that are packed runs of several
// sequences, with the last taps-1 inputs of each sequence kept as its state between steps.
//
//   u_t = in_t (+ bias_in)                          the convolution's input at position t (zero before position 0)
//   y_t = sum_j w[c, j] * u_(t - taps + 1 + j)      (+ bias_out), then the activation
//
// A row finds its inputs in the step's own rows where the position lies inside its run, in the
// sequence's state where it lies before the run's start, and takes zero where it lies before the
// sequence's start: a run that starts at position 0 never reads the state, so a slot that another
// request held needs no clearing.  The taps are added in ascending j whatever the run's cut, so a
// position's result does not depend on how its prompt was cut into steps.  The state is written by
// a second launch, after every row has read the old one.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

constexpr int kConvMaxTaps = 8;

template <class TO>
__global__ void __launch_bounds__(256)
    short_conv_kernel(const float* __restrict__ in, int ld_in, const float* __restrict__ bias_in,
                      const float* __restrict__ w, const float* __restrict__ bias_out, float* __restrict__ state,
                      TO* __restrict__ out, int ld_out, const int* __restrict__ row_seq, const int* __restrict__ positions,
                      const int* __restrict__ ctx_lens, const int* __restrict__ run_start, const int* __restrict__ seq_start,
                      const int* __restrict__ state_slots, int C, int taps, int act, int update_state) {
  const int row = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  TO* dst = out + size_t(row) * ld_out + c;
  if (ctx_lens[row] <= 0) {      // a padding row
    store_f(dst, 0.f);
    return;
  }
  const int s = row_seq[row], p = positions[row];
  const int p0 = seq_start[s], r0 = run_start[s], slot = state_slots[s];
  const float bi = bias_in ? bias_in[c] : 0.f;
  float* st = slot >= 0 ? state + (size_t(slot) * (taps - 1)) * C + c : nullptr;
  float y = 0.f;
  float seen[kConvMaxTaps];
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j) {
    seen[j] = 0.f;
    if (j < taps) {
      const int t = p - (taps - 1) + j;
      float u = 0.f;
      if (t >= p0) u = in[size_t(r0 + (t - p0)) * ld_in + c] + bi;
      else if (t >= 0 && st) u = st[size_t(t - (p0 - (taps - 1))) * C];
      seen[j] = u;
      y = fmaf(w[size_t(c) * taps + j], u, y);
    }
  }
  // a step in which every sequence runs one row: nobody else reads this sequence's state, so the row that read it
  // leaves the new one (its inputs but the oldest) and the second launch is not needed
  if (update_state && st) {
#pragma unroll
    for (int j = 1; j < kConvMaxTaps; ++j)
      if (j < taps) st[size_t(j - 1) * C] = seen[j];
  }
  if (bias_out) y += bias_out[c];
  if (act == 1) y = y / (1.0f + expf(-y));
  store_f(dst, y);
}

// state[slot][k][c] <- the input at position end - (taps-1) + k, k = 0 .. taps-2
__global__ void __launch_bounds__(256)
    short_conv_state_kernel(const float* __restrict__ in, int ld_in, const float* __restrict__ bias_in,
                            float* __restrict__ state, const int* __restrict__ run_start, const int* __restrict__ seq_start,
                            const int* __restrict__ seq_end, const int* __restrict__ state_slots, int C, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = state_slots[s];
  const int r0 = run_start[s], n = run_start[s + 1] - r0;
  if (slot < 0 || n <= 0) return;
  const int p0 = seq_start[s], p1 = seq_end[s];
  float* st = state + (size_t(slot) * (taps - 1)) * C + c;
  const float bi = bias_in ? bias_in[c] : 0.f;
  float keep[kConvMaxTaps - 1];
#pragma unroll
  for (int k = 0; k < kConvMaxTaps - 1; ++k) {
    keep[k] = 0.f;
    if (k < taps - 1) {
      const int t = p1 - (taps - 1) + k;
      if (t >= p0) keep[k] = in[size_t(r0 + (t - p0)) * ld_in + c] + bi;
      else if (t >= 0) keep[k] = st[size_t(t - (p0 - (taps - 1))) * C];
    }
  }
#pragma unroll
  for (int k = 0; k < kConvMaxTaps - 1; ++k)
    if (k < taps - 1) st[size_t(k) * C] = keep[k];
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// in [T, >= C] 32-bit; w [C, taps]; state [slots, taps-1, C] 32-bit; out [T, >= C]; act 0: none, 1: silu.
// update_state: only for steps in which every sequence runs exactly one row; the state is then written here.
int kvcm_short_conv(const float* in, int ld_in, const float* bias_in, const float* w, const float* bias_out,
                    float* state, void* out, int out_dtype, int ld_out, const int* row_seq, const int* positions,
                    const int* ctx_lens, const int* run_start, const int* seq_start, const int* state_slots, int T, int C,
                    int taps, int act, int update_state, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && C > 0, "short_conv: bad sizes T=%d C=%d", T, C);
  KVCM_REQUIRE(taps >= 1 && taps <= kConvMaxTaps, "short_conv: %d taps are not supported (1 to %d are)", taps, kConvMaxTaps);
  KVCM_REQUIRE(ld_in >= C && ld_out >= C, "short_conv: row strides too small");
  KVCM_REQUIRE(T <= 65535, "short_conv: too many rows for one launch (%d)", T);
  KVCM_REQUIRE(act == 0 || act == 1, "short_conv: unknown activation %d", act);
  const dim3 grid((C + 255) / 256, T);
  if (out_dtype == kF32)
    short_conv_kernel<float><<<grid, 256, 0, s>>>(in, ld_in, bias_in, w, bias_out, state, static_cast<float*>(out), ld_out,
                                                   row_seq, positions, ctx_lens, run_start, seq_start, state_slots, C, taps, act, update_state);
  else if (out_dtype == kBF16)
    short_conv_kernel<bf16_t><<<grid, 256, 0, s>>>(in, ld_in, bias_in, w, bias_out, state, static_cast<bf16_t*>(out), ld_out,
                                                    row_seq, positions, ctx_lens, run_start, seq_start, state_slots, C, taps, act, update_state);
  else KVCM_REQUIRE(false, "short_conv: unknown output dtype %d", out_dtype);
  return launch_status("short_conv");
}

int kvcm_short_conv_state(const float* in, int ld_in, const float* bias_in, float* state, const int* run_start,
                          const int* seq_start, const int* seq_end, const int* state_slots, int S, int C, int taps,
                          hipStream_t s) {
  if (S == 0 || taps <= 1) return 0;
  KVCM_REQUIRE(S > 0 && C > 0 && taps <= kConvMaxTaps, "short_conv_state: bad sizes S=%d C=%d taps=%d", S, C, taps);
  KVCM_REQUIRE(S <= 65535, "short_conv_state: too many sequences for one launch (%d)", S);
  const dim3 grid((C + 255) / 256, S);
  short_conv_state_kernel<<<grid, 256, 0, s>>>(in, ld_in, bias_in, state, run_start, seq_start, seq_end, state_slots, C, taps);
  return launch_status("short_conv_state");
}

}  // extern "C"
