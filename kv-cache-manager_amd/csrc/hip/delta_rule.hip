// The generalized delta rule: a matrix state per head that decays per key channel, forgets along the
// current unit key and learns the current key-value pair,
//
//   u = k / sqrt(|k|^2 + 1e-6)
//   S <- diag(w) S - (a * u) (u^T S) + k v^T        (both terms read the old S)
//   o = S^T r
//
// with w = exp(-exp(-1/2) * sigmoid(w_lin + w0)) and a = sigmoid(a_lin + a_bias) per head and key channel.
// State, decay, removal rate, unit key and all sums are 32-bit.
//
// Two launches.  The first turns the projections of every row into (w, a * u, u), in parallel over rows
// (the second step of the decay's projection included).
// The second walks each sequence's run token by token: a value column j of S needs u^T S[:, j], updates itself
// and sums o_j, and needs no other column, so columns are spread over lanes and workgroups.  The per-token
// vectors (r, k, w, a*u, u, v) are staged through LDS a few tokens at a time, the next tokens' values
// requested before the current ones are computed.  A run that starts at position 0 starts from zero
// without reading its slot.  Tokens are taken one by one in prompts and in decoding.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

// (tokens staged at once: a template parameter of the walk, fewer for the largest key size so that the values on their way fit the registers)

// one wave per (row, head).  The decay's logit is a two-step projection whose second step runs here in 32-bit:
// w_lin[c] = sum_j w2[c, j] * tanh(low[j]), low = the first step's output (rank values a row); w2 comes transposed,
// [rank, heads*d].
constexpr int kDeltaMaxRank = 256;
__global__ void __launch_bounds__(256)
    delta_prepare_kernel(const float* __restrict__ k, int ldk, const float* __restrict__ a_lin, int lda,
                         const float* __restrict__ a_bias, const float* __restrict__ low, int ldlow,
                         const float* __restrict__ w2t, int rank, const float* __restrict__ w0,
                         float* __restrict__ w_out, float* __restrict__ au_out, float* __restrict__ u_out, long long items,
                         int heads, int d) {
  __shared__ float th[256 / kWave][kDeltaMaxRank];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const long long item = static_cast<long long>(blockIdx.x) * (256 / kWave) + wave;
  const bool active = item < items;
  const int row = active ? static_cast<int>(item / heads) : 0, head = active ? static_cast<int>(item % heads) : 0;
  if (active)
    for (int j = lane; j < rank; j += kWave) th[wave][j] = tanhf(low[size_t(row) * ldlow + j]);
  __syncthreads();
  if (!active) return;
  const size_t col = size_t(head) * d, D = size_t(heads) * d;
  const float* kr = k + size_t(row) * ldk + col;
  float ss = 0.f;
  for (int i = lane; i < d; i += kWave) ss = fmaf(kr[i], kr[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss + 1e-6f);
  const float rate = 0.60653065971263342f;      // exp(-1/2)
  for (int i = lane; i < d; i += kWave) {
    const float u = kr[i] * inv;
    const float a = 1.0f / (1.0f + expf(-(a_lin[size_t(row) * lda + col + i] + a_bias[col + i])));
    float wl = 0.f;
    for (int j = 0; j < rank; ++j) wl = fmaf(w2t[size_t(j) * D + col + i], th[wave][j], wl);      // neighbours read neighbours
    const float g = 1.0f / (1.0f + expf(-(wl + w0[col + i])));
    w_out[size_t(row) * D + col + i] = expf(-rate * g);
    au_out[size_t(row) * D + col + i] = a * u;
    u_out[size_t(row) * D + col + i] = u;
  }
}

// The state of one head is dk x dv.  A workgroup of 256 threads owns 256 / G value columns of one head of one
// sequence; the key dimension of a column is spread over G lanes (IPT = DKP / G entries each, DKP: dk padded
// with zeros), so a token costs a lane IPT multiply-adds for u^T S, a sum across its G lanes, 3 IPT
// multiply-adds for the update, IPT for o and another sum across the lanes.
template <int DKP, int G, int TILE>
__global__ void __launch_bounds__(256)
    delta_scan_kernel(const float* __restrict__ r, int ldr, const float* __restrict__ k, int ldk,
                      const float* __restrict__ v, int ldv, const float* __restrict__ w, const float* __restrict__ au,
                      const float* __restrict__ u, float* __restrict__ o, int ldo, float* __restrict__ state,
                      const int* __restrict__ run_start, const int* __restrict__ seq_start,
                      const int* __restrict__ state_slots, int heads, int dk, int dv, int col_blocks) {
  constexpr int IPT = DKP / G, CB = 256 / G, W = 5 * DKP + CB;
  constexpr int PF = (TILE * W + 255) / 256;
  __shared__ __attribute__((aligned(16))) float tile[TILE][W];      // per token: r, k, w, a*u, u (zero beyond dk), v of these columns
  const int s = blockIdx.y, head = blockIdx.x / col_blocks, cb = blockIdx.x % col_blocks;
  const int g = threadIdx.x % G, j = cb * CB + threadIdx.x / G;
  const int r0 = run_start[s], r1 = run_start[s + 1];
  const int slot = state_slots[s];
  if (r1 <= r0) return;
  const size_t D = size_t(heads) * dk;
  const bool owns = j < dv;
  if (slot < 0) {
    if (owns && g == 0)
      for (int row = r0; row < r1; ++row) o[size_t(row) * ldo + size_t(head) * dv + j] = 0.f;
    return;
  }
  float* st = state + ((size_t(slot) * heads + head) * dk) * dv + (owns ? j : 0);      // [slot][head][i][j]
  const bool fresh = seq_start[s] == 0;
  float S[IPT];
#pragma unroll
  for (int il = 0; il < IPT; ++il) {
    const int i = g * IPT + il;
    S[il] = (i < dk && owns && !fresh) ? st[size_t(i) * dv] : 0.f;
  }
  float pf[PF];
  // (loads are unconditional, from clamped places, and masked afterwards: a branch around a load would make every
  // one of them wait for the one before)
  auto request = [&](int t0) {      // the staged values of the tokens t0 .. t0 + tile - 1, into registers
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      const int e = threadIdx.x + q * 256;
      const int t = e / W, off = e % W;
      const int row = t0 + t < r1 ? t0 + t : r1 - 1;
      const bool vector = off < 5 * DKP;
      const int which = off / DKP, i = off % DKP;
      const int jj = cb * CB + (off - 5 * DKP);
      const bool ok = t < TILE && t0 + t < r1 && (vector ? i < dk : jj < dv);
      const size_t col = size_t(head) * dk + (i < dk ? i : dk - 1);
      const size_t vcol = size_t(head) * dv + ((jj >= 0 && jj < dv) ? jj : 0);
      const float* src = !vector     ? v + size_t(row) * ldv + vcol
                         : which == 0 ? r + size_t(row) * ldr + col
                         : which == 1 ? k + size_t(row) * ldk + col
                         : which == 2 ? w + size_t(row) * D + col
                         : which == 3 ? au + size_t(row) * D + col
                                      : u + size_t(row) * D + col;
      const float val = *src;
      pf[q] = ok ? val : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      const int e = threadIdx.x + q * 256;
      if (e < TILE * W) tile[e / W][e % W] = pf[q];
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
      const float vj = tv[5 * DKP + threadIdx.x / G];
      float sa = 0.f;
#pragma unroll
      for (int il = 0; il < IPT; ++il) sa = fmaf(tv[4 * DKP + g * IPT + il], S[il], sa);
      sa = group_sum<G>(sa);
      float acc = 0.f;
#pragma unroll
      for (int il = 0; il < IPT; ++il) {
        const int i = g * IPT + il;
        float sn = tv[2 * DKP + i] * S[il];
        sn = fmaf(-tv[3 * DKP + i], sa, sn);
        sn = fmaf(tv[DKP + i], vj, sn);
        S[il] = sn;
        acc = fmaf(sn, tv[i], acc);
      }
      acc = group_sum<G>(acc);
      if (owns && g == 0) o[size_t(t0 + t) * ldo + size_t(head) * dv + j] = acc;
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

// k, a_lin: 32-bit rows with heads*d columns each (at their own strides); low: 32-bit rows of `rank` columns;
// w2t [rank, heads*d] (the second step's matrix, transposed), a_bias, w0 [heads*d]; w_out, au_out, u_out [T, heads*d]: all 32-bit.
int kvcm_delta_prepare(const float* k, int ldk, const float* a_lin, int lda, const float* a_bias, const float* low, int ldlow,
                       const float* w2t, int rank, const float* w0, float* w_out, float* au_out, float* u_out, int T, int heads,
                       int d, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && heads > 0 && d > 0, "delta_prepare: bad sizes T=%d heads=%d d=%d", T, heads, d);
  KVCM_REQUIRE(rank > 0 && rank <= kDeltaMaxRank, "delta_prepare: a rank of %d is not supported (1 to %d)", rank, kDeltaMaxRank);
  KVCM_REQUIRE(ldk >= heads * d && lda >= heads * d && ldlow >= rank, "delta_prepare: row strides too small");
  const long long items = static_cast<long long>(T) * heads;
  const long long blocks = (items + 3) / 4;
  KVCM_REQUIRE(blocks < (1ll << 31), "delta_prepare: too many rows");
  delta_prepare_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(k, ldk, a_lin, lda, a_bias, low, ldlow, w2t, rank, w0, w_out,
                                                                     au_out, u_out, items, heads, d);
  return launch_status("delta_prepare");
}

// r, k [T, heads*dk], v [T, heads*dv] at their own strides; w, au, u [T, heads*dk] dense; o [T, >= heads*dv];
// state [slots, heads, dk, dv]; all 32-bit.
int kvcm_delta_scan(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv, const float* w, const float* au,
                    const float* u, float* o, int ldo, float* state, const int* run_start, const int* seq_start,
                    const int* state_slots, int S, int heads, int dk, int dv, hipStream_t s) {
  if (S == 0) return 0;
  KVCM_REQUIRE(S > 0 && heads > 0 && dk > 0 && dv > 0, "delta_scan: bad sizes S=%d heads=%d dk=%d dv=%d", S, heads, dk, dv);
  KVCM_REQUIRE(dk <= 256, "delta_scan: a key size of %d is not supported (up to 256)", dk);
  KVCM_REQUIRE(static_cast<long long>(heads) * ((dv + 31) / 32) < (1ll << 31), "delta_scan: too many heads");
  KVCM_REQUIRE(S <= 65535, "delta_scan: too many sequences for one launch (%d)", S);
  KVCM_REQUIRE(ldr >= heads * dk && ldk >= heads * dk && ldv >= heads * dv && ldo >= heads * dv, "delta_scan: row strides too small");
#define KVCM_DELTA(DKP, G, TILE)                                                                                            \
  {                                                                                                                    \
    const int col_blocks = (dv + 256 / G - 1) / (256 / G);                                                             \
    delta_scan_kernel<DKP, G, TILE><<<dim3(heads * col_blocks, S), 256, 0, s>>>(r, ldr, k, ldk, v, ldv, w, au, u, o, ldo, state, \
                                                                          run_start, seq_start, state_slots, heads, dk, dv, \
                                                                          col_blocks);                                  \
  }
  if (dk <= 16) KVCM_DELTA(16, 2, 8)
  else if (dk <= 32) KVCM_DELTA(32, 4, 8)
  else if (dk <= 64) KVCM_DELTA(64, 8, 8)
  else if (dk <= 128) KVCM_DELTA(128, 8, 8)
  else KVCM_DELTA(256, 16, 2)
#undef KVCM_DELTA
  return launch_status("delta_scan");
}

}  // extern "C"
