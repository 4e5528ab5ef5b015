// Kernels of mixers that keep a state of fixed size per request instead of a cache that grows:
// the inputs of the last few tokens (token shift, short causal convolution) and, per head, a
// matrix S of key channels x value channels that every token decays, writes to and reads from.
//
// A request's state lives in its slot of the runner's state buffer: `state` points at this
// mixer's area inside slot 0 and `state_stride` floats lead from one slot to the next.  All of
// it is float32, and everything that enters a recurrence is float32 arithmetic.  Every kernel
// walks a sequence's tokens of the step in order (cu[s] .. cu[s + 1]) from the state that the
// step before left, whatever else is in the batch; a sequence at position 0 finds zeros (the
// runner clears the slot), which are the zeros in front of a sequence's first token.
//
// The matrix state is walked by one wave per (sequence, head, four value channels): lane i
// holds S[i][j] of each (and i + 64, ... for more than 64 key channels), a token's read-out is
// a sum over the wave, and nothing is shared between waves, so the columns of a head spread
// over the chip.  State layout per head: [value channel][key channel], so a wave's columns are
// contiguous.
#include "common.h"

namespace {

constexpr int kMaxTaps = 16;

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ------------------------------------------------------------------ token shift
// out[m][t][c] = x[t][c] + (prev[t][c] - x[t][c]) * mu[m][c], prev = the row of the token
// before (the tail row of the state for a sequence's first token of the step).
template <typename TX>
__global__ void shift_mix_kernel(TX* __restrict__ out, const TX* __restrict__ x,
                                 const float* __restrict__ mu, const float* __restrict__ state,
                                 long long state_stride, const int* __restrict__ seq_of_token,
                                 const int* __restrict__ cu, const int* __restrict__ slots, int T,
                                 int W, int mixes) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int s = seq_of_token[t];
  const bool first = t == cu[s];
  const float* tail = state + (long long)slots[s] * state_stride;
  // both candidates are asked for, from addresses that always exist, and the value is chosen
  const float cur = ld(x + (long long)t * W + c);
  const float before = ld(x + (long long)(t > 0 ? t - 1 : 0) * W + c);
  const float kept = tail[c];
  const float d = (first ? kept : before) - cur;
  for (int m = 0; m < mixes; ++m)
    st(out + ((long long)m * T + t) * W + c, cur + d * mu[(long long)m * W + c]);
}

// ------------------------------------------------------------------ input tails
// A sequence's tail holds the rows of its last R inputs, oldest first.  After a step of n rows
// it is the last R of (old tail ++ the step's rows).  A thread owns a channel, reads what it
// needs of the old tail and then writes, so a step shorter than the tail shifts it in place.
template <typename TX>
__global__ void tail_update_kernel(float* __restrict__ state, long long state_stride,
                                   const TX* __restrict__ x, long long ldx, int C, int R,
                                   const int* __restrict__ cu, const int* __restrict__ slots) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu[s], n = cu[s + 1] - t0;
  float* tail = state + (long long)slots[s] * state_stride;
  float keep[kMaxTaps];
#pragma unroll
  for (int r = 0; r < kMaxTaps; ++r) {
    if (r < R) {
      const int src = n + r;          // index into (old tail ++ new rows) of the row kept at r
      keep[r] = src < R ? tail[(long long)src * C + c]
                        : ld(x + (long long)(t0 + src - R) * ldx + c);
    }
  }
#pragma unroll
  for (int r = 0; r < kMaxTaps; ++r)
    if (r < R) tail[(long long)r * C + c] = keep[r];
}

// ------------------------------------------- short causal convolution + SiLU (+ unit norm)
// y[t][c] = act(bias[c] + sum_j taps[c][j] * x[t - (K - 1) + j][c]) (bias optional; act is SiLU,
// or nothing with activation 0); channels from blend_from on are then mixed with another
// tensor's rows of the same tokens, y <- (1 - blend_weight) y + blend_weight * blend[t][c -
// blend_from] (blend null: no mixing); rows in front of the step come from
// the tail, rows in front of the sequence are the tail's zeros.  Channels [0, unit_channels)
// are then made unit vectors in groups of unit_group (x / sqrt(sum x^2 + unit_eps)) and those
// below scaled_channels multiplied by `scale`; the other channels are cut into groups of
// rest_group for the grid only.  One wave per (token, group), up to 16 channels per lane; a
// workgroup is four groups of one token.  Both candidates of an input row (the step's, the
// tail's) are asked for from addresses that exist, and the value is chosen.
__device__ __forceinline__ float lanes_sum(float v);

template <typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    TO* __restrict__ out, const float* __restrict__ x, long long ldx,
    const float* __restrict__ taps, const float* __restrict__ bias, int C, int K,
    const float* __restrict__ state, long long state_stride,
    const int* __restrict__ seq_of_token, const int* __restrict__ cu,
    const int* __restrict__ slots, int unit_channels, int unit_group, int scaled_channels,
    float scale, float unit_eps, int rest_group, int groups, int activation,
    const TO* __restrict__ blend, long long ld_blend, int blend_from, float blend_weight) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int g = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (g >= groups) return;
  const int groups_unit = unit_group > 0 ? unit_channels / unit_group : 0;
  int c0, width;
  const bool unit = g < groups_unit;
  if (unit) {
    c0 = g * unit_group;
    width = unit_group;
  } else {
    c0 = unit_channels + (g - groups_unit) * rest_group;
    width = min(rest_group, C - c0);
  }
  const int s = seq_of_token[t];
  const int rel = t - cu[s];                 // rows of the step in front of this one
  const int R = K - 1;
  const float* tail = state + (long long)slots[s] * state_stride;
  constexpr int VPT = 16;
  float y[VPT];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    y[v] = 0.f;
    if (v * kWave < width) {                 // the same for the whole wave
      const int off = lane + v * kWave;
      const int c = c0 + (off < width ? off : width - 1);
      float acc = bias ? bias[c] : 0.f;
      for (int j = 0; j < K; ++j) {
        const int back = R - j;              // how many rows before t
        const bool here = back <= rel;
        const float from_step = x[(long long)(t - (here ? back : 0)) * ldx + c];
        const float from_tail = R > 0 ? tail[(long long)(here ? 0 : R - (back - rel)) * C + c] : 0.f;
        acc += taps[(long long)c * K + j] * (here ? from_step : from_tail);
      }
      if (activation) acc = siluf_(acc);
      if (blend && c >= blend_from)
        acc = (1.0f - blend_weight) * acc +
              blend_weight * ld(blend + (long long)t * ld_blend + (c - blend_from));
      y[v] = off < width ? acc : 0.f;
      ss += y[v] * y[v];
    }
  }
  float mult = 1.0f;
  if (unit) {
    ss = lanes_sum(ss);
    mult = 1.0f / sqrtf(ss + unit_eps);
    if (c0 < scaled_channels) mult *= scale;
  }
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int off = lane + v * kWave;
    if (off < width) st(out + (long long)t * C + c0 + off, y[v] * mult);
  }
}

// ------------------------------------------------------------------ the two scans
// Sum over the 64 lanes of a wave, every lane gets it: four data-parallel-primitive adds inside
// rows of 16 lanes (neighbour, pair, the other quad, the other half-row) and the two half
// swaps; no trip through LDS.  The order of the additions is fixed.
template <int CTRL>
__device__ __forceinline__ float dpp_from(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lanes_sum(float v) {   // (declared above, for the convolution)
  v += dpp_from<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v += dpp_from<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v += dpp_from<0x141>(v);   // row_half_mirror
  v += dpp_from<0x140>(v);   // row_mirror
  v = xor16_sum(v);
  return xor32_sum(v);
}

// Four sums over the wave at once, for values a wave holds per lane for four columns: lanes
// trade columns with their neighbour and their neighbour's neighbour, so that lane l carries on
// with column l % 4 alone, and the steps that follow (4 and 8 lanes round the row, the half
// swaps) keep that class.  Lane l ends with the whole sum of column l % 4: ten adds and moves
// for four sums where four separate sums take twenty-four.  The order of the additions is fixed.
__device__ __forceinline__ float lanes_sum4(const float (&p)[4], int lane) {
  const bool odd = lane & 1, high = lane & 2;
  float a01 = odd ? p[1] : p[0];
  a01 += dpp_from<0xB1>(odd ? p[0] : p[1]);
  float a23 = odd ? p[3] : p[2];
  a23 += dpp_from<0xB1>(odd ? p[2] : p[3]);
  float a = high ? a23 : a01;
  a += dpp_from<0x4E>(high ? a01 : a23);
  a += dpp_from<0x124>(a);   // row_ror 4
  a += dpp_from<0x128>(a);   // row_ror 8
  a = xor16_sum(a);
  return xor32_sum(a);
}

// The same for two columns: lane l ends with the whole sum of column l % 2.
__device__ __forceinline__ float lanes_sum2(const float (&p)[2], int lane) {
  const bool odd = lane & 1;
  float a = odd ? p[1] : p[0];
  a += dpp_from<0xB1>(odd ? p[0] : p[1]);
  a += dpp_from<0x4E>(a);    // two lanes on: the same column
  a += dpp_from<0x124>(a);
  a += dpp_from<0x128>(a);
  a = xor16_sum(a);
  return xor32_sum(a);
}
template <int NC>
__device__ __forceinline__ float lanes_sum_cols(const float (&p)[NC], int lane) {
  if constexpr (NC == 4) return lanes_sum4(p, lane);
  else return lanes_sum2(p, lane);
}

// A wave walks kCols value channels of one (sequence, head): lane i holds S[i][j] of each (and
// i + 64, ... for more than 64 key channels), so what a token brings per key channel is loaded
// once for all of them and their sums over the wave interleave.  What does not depend on the
// state (decays, step sizes, the products of a token's own vectors) is made one token ahead,
// while the token before it waits for its sums.  No load stands under a condition: lanes and
// columns past the end read a clamped address and their values are zeroed or not stored.
constexpr int kCols = 4;

// Gated delta rule.  Per token and head, with one decay g and one step size beta per head:
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
// g = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b), from the raw projections.
// Column j of S is independent of the others.  With d1 = S^T k and d2 = S^T q of the state
// before the token, u_j = beta (v_j - g d1_j) and o_j = g d2_j + (k . q) u_j, so both sums
// are over the old state and wait for nothing but each other.
template <int KR>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    float* __restrict__ out, long long ldo, const float* __restrict__ q, const float* __restrict__ k,
    const float* __restrict__ v, long long ldqkv, const float* __restrict__ b_raw,
    const float* __restrict__ a_raw, long long ldba, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, long long state_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, int heads, int kv_heads, int dk,
    int dv) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int j0 = (blockIdx.x * (blockDim.x / kWave) + wave) * kCols;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  if (j0 >= dv) return;
  const int kh = head / (heads / kv_heads);
  const int t0 = cu[s], t1 = cu[s + 1];
  float* base = state + (long long)slots[s] * state_stride + (long long)head * dv * dk;
  int idx[KR];
  float live[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    idx[r] = i < dk ? i : dk - 1;
    live[r] = i < dk ? 1.f : 0.f;
  }
  int col[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) col[c] = j0 + c < dv ? j0 + c : dv - 1;
  float S[kCols][KR];
#pragma unroll
  for (int c = 0; c < kCols; ++c)
#pragma unroll
    for (int r = 0; r < KR; ++r) S[c][r] = base[(long long)col[c] * dk + idx[r]] * live[r];
  const float neg_a = -expf(a_log[head]);
  const float bias = dt_bias[head];
  // the token ahead: its vectors, and what follows from them alone
  float kn[KR], qn[KR], vn[kCols], gn = 0.f, betan = 0.f, kqn = 0.f;
  auto fetch = [&](int t) {
    const float* kt = k + (long long)t * ldqkv + kh * dk;
    const float* qt = q + (long long)t * ldqkv + kh * dk;
    float kq = 0.f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      kn[r] = kt[idx[r]] * live[r];
      qn[r] = qt[idx[r]] * live[r];
      kq += kn[r] * qn[r];
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) vn[c] = v[(long long)t * ldqkv + head * dv + col[c]];
    betan = sigmoidf_(b_raw[(long long)t * ldba + head]);
    gn = expf(neg_a * softplusf_(a_raw[(long long)t * ldba + head] + bias));
    kqn = lanes_sum(kq);
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float kc[KR], qc[KR], vc[kCols];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) vc[c] = vn[c];
    const float g = gn, beta = betan, kq = kqn;
    fetch(t + 1 < t1 ? t + 1 : t);
    float d1[kCols], d2[kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      d1[c] = 0.f;
      d2[c] = 0.f;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        d1[c] += S[c][r] * kc[r];
        d2[c] += S[c][r] * qc[r];
      }
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      d1[c] = lanes_sum(d1[c]);
      d2[c] = lanes_sum(d2[c]);
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      const float u = beta * (vc[c] - g * d1[c]);
#pragma unroll
      for (int r = 0; r < KR; ++r) S[c][r] = g * S[c][r] + kc[r] * u;
      if (lane == c && j0 + c < dv)
        out[(long long)t * ldo + head * dv + j0 + c] = g * d2[c] + kq * u;
    }
  }
#pragma unroll
  for (int c = 0; c < kCols; ++c)
    if (j0 + c < dv) {
#pragma unroll
      for (int r = 0; r < KR; ++r)
        if (lane + r * kWave < dk) base[(long long)(j0 + c) * dk + lane + r * kWave] = S[c][r];
    }
}

// Decayed state with a bonus for the present.  Per token and head, with a decay per key channel
// w_i = exp(-exp(z_i + w0_i)):
//   o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T.
// Keys, values and receptances have one size `d` here; z is the raw low-rank projection.
// o_j = sum_i r_i S_ij + (sum_i r_i u_i k_i) v_j: the second sum does not depend on the state.
template <int KR>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    float* __restrict__ out, const float* __restrict__ r_in, const float* __restrict__ k_in,
    const float* __restrict__ v_in, const float* __restrict__ z_in, long long ld,
    const float* __restrict__ w0, const float* __restrict__ bonus, float* __restrict__ state,
    long long state_stride, const int* __restrict__ cu, const int* __restrict__ slots, int heads,
    int d) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int j0 = (blockIdx.x * (blockDim.x / kWave) + wave) * kCols;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  if (j0 >= d) return;
  const int t0 = cu[s], t1 = cu[s + 1];
  float* base = state + (long long)slots[s] * state_stride + (long long)head * d * d;
  int idx[KR];
  float live[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    idx[r] = i < d ? i : d - 1;
    live[r] = i < d ? 1.f : 0.f;
  }
  int col[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) col[c] = j0 + c < d ? j0 + c : d - 1;
  float S[kCols][KR], u[KR], w_base[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    u[r] = bonus[head * d + idx[r]];
    w_base[r] = w0[head * d + idx[r]];
#pragma unroll
    for (int c = 0; c < kCols; ++c) S[c][r] = base[(long long)col[c] * d + idx[r]] * live[r];
  }
  float rn[KR], kn[KR], wn[KR], vn[kCols], rukn = 0.f;
  auto fetch = [&](int t) {
    const long long row = (long long)t * ld + head * d;
    float ruk = 0.f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      rn[r] = r_in[row + idx[r]] * live[r];
      kn[r] = k_in[row + idx[r]] * live[r];
      wn[r] = expf(-expf(z_in[row + idx[r]] + w_base[r]));
      ruk += rn[r] * u[r] * kn[r];
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) vn[c] = v_in[row + col[c]];
    rukn = lanes_sum(ruk);
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float rc[KR], kc[KR], wc[KR], vc[kCols];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      rc[r] = rn[r];
      kc[r] = kn[r];
      wc[r] = wn[r];
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) vc[c] = vn[c];
    const float ruk = rukn;
    fetch(t + 1 < t1 ? t + 1 : t);
    float o[kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      o[c] = 0.f;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        o[c] += rc[r] * S[c][r];
        S[c][r] = wc[r] * S[c][r] + kc[r] * vc[c];
      }
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) o[c] = lanes_sum(o[c]);
#pragma unroll
    for (int c = 0; c < kCols; ++c)
      if (lane == c && j0 + c < d) out[(long long)t * ld + head * d + j0 + c] = o[c] + ruk * vc[c];
  }
#pragma unroll
  for (int c = 0; c < kCols; ++c)
    if (j0 + c < d) {
#pragma unroll
      for (int r = 0; r < KR; ++r)
        if (lane + r * kWave < d) base[(long long)(j0 + c) * d + lane + r * kWave] = S[c][r];
    }
}

// ------------------------------------------------------- the scans over long runs of tokens
// The kernels above ask for a token's vectors one token ahead, which hides the arithmetic of one
// token and no more: over a prompt's portion every token would wait out a trip to memory.  The
// forms below are for steps in which some sequence brings many tokens.  A workgroup (four waves,
// sixteen value channels of one head) asks for a whole tile of tokens at once, keeps it in
// registers while its waves walk the tile before from LDS, each over its own columns, and then
// moves it to LDS with everything that follows from a token alone made on the way (decays and
// step sizes; columns and tokens past the end read clamped addresses).  A token's four sums over
// the wave are formed together (lanes_sum4), so a row comes out as above to rounding, not to
// the bit.
template <int KR>
struct ScanTile {
  static constexpr int kTokens = KR == 4 ? 16 : 32;
  static constexpr int kKeys = KR * kWave;
};

#ifndef RLIS_DELTA_GROUP
#define RLIS_DELTA_GROUP 2
#endif
constexpr int kDeltaGroup = RLIS_DELTA_GROUP;   // tokens whose sums run side by side

template <int KR, int NC>
__global__ __launch_bounds__(256) void delta_scan_tiled_kernel(
    float* __restrict__ out, long long ldo, const float* __restrict__ q, const float* __restrict__ k,
    const float* __restrict__ v, long long ldqkv, const float* __restrict__ b_raw,
    const float* __restrict__ a_raw, long long ldba, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, long long state_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, int heads, int kv_heads, int dk,
    int dv) {
  constexpr int TT = ScanTile<KR>::kTokens, DK = ScanTile<KR>::kKeys, CB = 4 * NC, GROUP = kWave / NC;
  constexpr int U = kDeltaGroup;
  __shared__ float tk[TT][DK], tq[TT][DK], tv[TT][CB], tg[TT], tb[TT];
  __shared__ __attribute__((aligned(16))) float tp[TT / U][U * U];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int jb = blockIdx.x * CB;                 // the workgroup's first column
  const int j0 = jb + wave * NC;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  const int kh = head / (heads / kv_heads);
  const int t0 = cu[s], t1 = cu[s + 1];
  float* base = state + (long long)slots[s] * state_stride + (long long)head * dv * dk;
  int idx[KR];
  float live[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    idx[r] = i < dk ? i : dk - 1;
    live[r] = i < dk ? 1.f : 0.f;
  }
  float S[NC][KR];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int col = j0 + c < dv ? j0 + c : dv - 1;
#pragma unroll
    for (int r = 0; r < KR; ++r) S[c][r] = base[(long long)col * dk + idx[r]] * live[r];
  }
  const float neg_a = -expf(a_log[head]);
  const float bias = dt_bias[head];
  // A tile's values wait in registers while the tile before is walked: every load of a tile is
  // asked for at once, and none of them is waited for before the walk in front of it is over.
  constexpr int PER = TT * DK / 256, PERV = (TT * CB + 255) / 256;
  static_assert(TT * DK % 256 == 0 && TT <= 256, "tile sizes");
  float rk[PER], rq[PER], rv[PERV], rb = 0.f, rg = 0.f;
  auto ask = [&](int tile) {
    const int n = min(TT, t1 - tile);
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int e = threadIdx.x + p * 256, tt = e / DK, i = e % DK;
      const long long row = (long long)(tile + (tt < n ? tt : n - 1)) * ldqkv + kh * dk;
      const int ic = i < dk ? i : dk - 1;
      const float keep = (tt < n && i < dk) ? 1.f : 0.f;
      rk[p] = k[row + ic] * keep;
      rq[p] = q[row + ic] * keep;
    }
#pragma unroll
    for (int p = 0; p < PERV; ++p) {
      const int e = min(threadIdx.x + p * 256, TT * CB - 1), tt = e / CB, c = e % CB;
      const int col = jb + c < dv ? jb + c : dv - 1;
      rv[p] = v[(long long)(tile + (tt < n ? tt : n - 1)) * ldqkv + head * dv + col];
    }
    const int tt = threadIdx.x < TT ? threadIdx.x : TT - 1;
    const long long row = (long long)(tile + (tt < n ? tt : n - 1)) * ldba + head;
    rb = b_raw[row];
    rg = a_raw[row];
  };
  if (t0 < t1) ask(t0);
  for (int tile = t0; tile < t1; tile += TT) {
    const int n = min(TT, t1 - tile);
    __syncthreads();                               // the tile before has been walked
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int e = threadIdx.x + p * 256;
      tk[e / DK][e % DK] = rk[p];
      tq[e / DK][e % DK] = rq[p];
    }
#pragma unroll
    for (int p = 0; p < PERV; ++p) {
      const int e = threadIdx.x + p * 256;
      if (e < TT * CB) tv[e / CB][e % CB] = rv[p];
    }
    if (threadIdx.x < TT) {                        // past the end: no step, no decay
      tb[threadIdx.x] = threadIdx.x < n ? sigmoidf_(rb) : 0.f;
      tg[threadIdx.x] = threadIdx.x < n ? expf(neg_a * softplusf_(rg + bias)) : 1.f;
    }
    __syncthreads();
    ask(tile + TT < t1 ? tile + TT : tile);
    // Lane l gathers the read-out of token (l / NC) of a group for column l % NC and stores it
    // when the group is through: one store a group, not NC a token.
    float gathered = 0.f;
    // U tokens at a time.  With S the state in front of the group, G(t) the product of the
    // decays up to token t and G(t, s) that of tokens s + 1 .. t:
    //   u_t = beta_t (v_t - G(t) S^T k_t - sum_{s<t} G(t, s) (k_s . k_t) u_s)
    //   o_t = G(t) S^T q_t + sum_{s<=t} G(t, s) (k_s . q_t) u_s
    //   S  <- G(U-1) S + sum_s G(U-1, s) k_s u_s^T
    // so every sum over the wave is over the state in front of the group or over the tokens'
    // own vectors: all of a group's sums run side by side, and the state waits for them once a
    // group, not once a token.  Tokens past the end carry k = q = 0, beta = 0, g = 1.
    static_assert(TT % U == 0 && GROUP % U == 0 && (TT * U) % 16 == 0, "token groups");
    // The tokens' own products, once a tile for all its groups and all four waves: entry (a, b)
    // of a group is k_b . q_a for b <= a and k_a . k_b for b > a; a wave sums four entries at
    // a time and lanes 0 to 3 put them down.
    {
      float* flat = &tp[0][0];
      for (int f = wave * 4; f < TT * U; f += 16) {
        float four[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const int e = f + m, first = e / (U * U) * U, a2 = e % (U * U) / U, b2 = e % U;
          const float* other = b2 <= a2 ? tq[first + a2] : tk[first + a2];
          float pp = 0.f;
#pragma unroll
          for (int r = 0; r < KR; ++r) pp += tk[first + b2][lane + r * kWave] * other[lane + r * kWave];
          four[m] = pp;
        }
        const float mine = lanes_sum4(four, lane);           // of entry f + lane % 4
        if (lane < 4) flat[f + lane] = mine;
      }
    }
    __syncthreads();
    for (int tb0 = 0; tb0 < n; tb0 += U) {
      float kc[U][KR], qc[U][KR], g[U], beta[U], v_own[U];
#pragma unroll
      for (int t = 0; t < U; ++t) {
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          kc[t][r] = tk[tb0 + t][lane + r * kWave];
          qc[t][r] = tq[tb0 + t][lane + r * kWave];
        }
        g[t] = tg[tb0 + t];
        beta[t] = tb[tb0 + t];
        v_own[t] = tv[tb0 + t][wave * NC + (lane & (NC - 1))];
      }
      float pair[U * U];
#pragma unroll
      for (int f = 0; f < U * U; ++f) pair[f] = tp[tb0 / U][f];
      // the sums over the state in front of the group, for this lane's column
      float s1[U], s2[U];
#pragma unroll
      for (int t = 0; t < U; ++t) {
        float d1[NC], d2[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          d1[c] = 0.f;
          d2[c] = 0.f;
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            d1[c] += S[c][r] * kc[t][r];
            d2[c] += S[c][r] * qc[t][r];
          }
        }
        if constexpr (NC == 2) {       // both sums of both columns in one four-column sum
          const float four[4] = {d1[0], d1[1], d2[0], d2[1]};
          const float mine = lanes_sum4(four, lane);
          s1[t] = dpp_from<0x44>(mine);                      // quad_perm [0, 1, 0, 1]
          s2[t] = dpp_from<0xEE>(mine);                      // quad_perm [2, 3, 2, 3]
        } else {
          s1[t] = lanes_sum_cols<NC>(d1, lane);
          s2[t] = lanes_sum_cols<NC>(d2, lane);
        }
      }
      // the group's recurrence in scalars, for the column lane % NC
      float gam[U][U], upto[U], u_own[U];
#pragma unroll
      for (int t = 0; t < U; ++t) {
        upto[t] = t ? upto[t - 1] * g[t] : g[t];
        gam[t][t] = 1.f;
#pragma unroll
        for (int s0 = 0; s0 < t; ++s0) gam[t][s0] = gam[t - 1][s0] * g[t];
      }
#pragma unroll
      for (int t = 0; t < U; ++t) {
        float inner = upto[t] * s1[t], o = upto[t] * s2[t];
#pragma unroll
        for (int s0 = 0; s0 < t; ++s0) {
          inner += gam[t][s0] * pair[s0 * U + t] * u_own[s0];
          o += gam[t][s0] * pair[t * U + s0] * u_own[s0];
        }
        u_own[t] = beta[t] * (v_own[t] - inner);
        o += pair[t * U + t] * u_own[t];
        if (lane / NC == (tb0 + t) % GROUP) gathered = o;
      }
      // each column's steps to every lane, and the state behind the group
      float coef[U][NC];
#pragma unroll
      for (int t = 0; t < U; ++t) {
        const float scaled = gam[U - 1][t] * u_own[t];
        coef[t][0] = dpp_from<0x00>(scaled);
        coef[t][1] = dpp_from<0x55>(scaled);
        if constexpr (NC == 4) {
          coef[t][2] = dpp_from<0xAA>(scaled);
          coef[t][3] = dpp_from<0xFF>(scaled);
        }
      }
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          float acc = upto[U - 1] * S[c][r];
#pragma unroll
          for (int t = 0; t < U; ++t) acc += kc[t][r] * coef[t][c];
          S[c][r] = acc;
        }
      if ((tb0 + U) % GROUP == 0 || tb0 + U >= n) {
        const int token = tb0 / GROUP * GROUP + lane / NC;
        if (token < n && token < tb0 + U && j0 + (lane & (NC - 1)) < dv)
          out[(long long)(tile + token) * ldo + head * dv + j0 + (lane & (NC - 1))] = gathered;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c)
    if (j0 + c < dv) {
#pragma unroll
      for (int r = 0; r < KR; ++r)
        if (lane + r * kWave < dk) base[(long long)(j0 + c) * dk + lane + r * kWave] = S[c][r];
    }
}

template <int KR, int NC>
__global__ __launch_bounds__(256) void decay_scan_tiled_kernel(
    float* __restrict__ out, const float* __restrict__ r_in, const float* __restrict__ k_in,
    const float* __restrict__ v_in, const float* __restrict__ z_in, long long ld,
    const float* __restrict__ w0, const float* __restrict__ bonus, float* __restrict__ state,
    long long state_stride, const int* __restrict__ cu, const int* __restrict__ slots, int heads,
    int d) {
  constexpr int TT = ScanTile<KR>::kTokens / 2, DK = ScanTile<KR>::kKeys, CB = 4 * NC, GROUP = kWave / NC;
  __shared__ float tr[TT][DK], tk[TT][DK], tw[TT][DK], tv[TT][CB];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int jb = blockIdx.x * CB;
  const int j0 = jb + wave * NC;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  const int t0 = cu[s], t1 = cu[s + 1];
  float* base = state + (long long)slots[s] * state_stride + (long long)head * d * d;
  float S[NC][KR], u[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    const int ic = i < d ? i : d - 1;
    const float keep = i < d ? 1.f : 0.f;
    u[r] = bonus[head * d + ic];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int col = j0 + c < d ? j0 + c : d - 1;
      S[c][r] = base[(long long)col * d + ic] * keep;
    }
  }
  constexpr int PER = TT * DK / 256, PERV = (TT * CB + 255) / 256;
  static_assert(TT * DK % 256 == 0, "tile sizes");
  float rr[PER], rk[PER], rz[PER], rv[PERV];
  auto ask = [&](int tile) {
    const int n = min(TT, t1 - tile);
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int e = threadIdx.x + p * 256, tt = e / DK, i = e % DK;
      const long long row = (long long)(tile + (tt < n ? tt : n - 1)) * ld + head * d;
      const int ic = i < d ? i : d - 1;
      const float keep = (tt < n && i < d) ? 1.f : 0.f;
      rr[p] = r_in[row + ic] * keep;
      rk[p] = k_in[row + ic] * keep;
      rz[p] = z_in[row + ic] + w0[head * d + ic];
    }
#pragma unroll
    for (int p = 0; p < PERV; ++p) {
      const int e = min(threadIdx.x + p * 256, TT * CB - 1), tt = e / CB, c = e % CB;
      const int col = jb + c < d ? jb + c : d - 1;
      rv[p] = v_in[(long long)(tile + (tt < n ? tt : n - 1)) * ld + head * d + col];
    }
  };
  if (t0 < t1) ask(t0);
  for (int tile = t0; tile < t1; tile += TT) {
    const int n = min(TT, t1 - tile);
    __syncthreads();                               // the tile before has been walked
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int e = threadIdx.x + p * 256;
      tr[e / DK][e % DK] = rr[p];
      tk[e / DK][e % DK] = rk[p];
      tw[e / DK][e % DK] = e / DK < n ? expf(-expf(rz[p])) : 1.f;   // no decay past the end
    }
#pragma unroll
    for (int p = 0; p < PERV; ++p) {
      const int e = threadIdx.x + p * 256;
      if (e < TT * CB) tv[e / CB][e % CB] = rv[p];
    }
    __syncthreads();
    ask(tile + TT < t1 ? tile + TT : tile);
    // Four tokens at a time: their read-outs are sums over the state before each of them, and
    // nothing in the state waits for a sum, so the four tokens' sums over the wave are formed
    // side by side (independent chains fill the slots that one chain leaves empty), and
    // four tokens' bonus terms r.u.k in one four-column sum.  Tokens past the end carry r = k = 0
    // and w = 1: they leave the state as it is and are not stored.
    float gathered = 0.f;                          // as in the kernel above
    constexpr int U = 4;                           // eight at a time were no faster
    static_assert(TT % U == 0 && GROUP % U == 0 && U % 4 == 0, "token groups");
    for (int tb = 0; tb < n; tb += U) {
      float o[U][NC], ruk[U], v_own[U];
#pragma unroll
      for (int uu = 0; uu < U; ++uu) {
        const int tt = tb + uu;
        float rc[KR], kc[KR], wc[KR];
        ruk[uu] = 0.f;
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          rc[r] = tr[tt][lane + r * kWave];
          kc[r] = tk[tt][lane + r * kWave];
          wc[r] = tw[tt][lane + r * kWave];
          ruk[uu] += rc[r] * u[r] * kc[r];
        }
        v_own[uu] = tv[tt][wave * NC + (lane & (NC - 1))];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const float vc = tv[tt][wave * NC + c];
          o[uu][c] = 0.f;
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            o[uu][c] += rc[r] * S[c][r];
            S[c][r] = wc[r] * S[c][r] + kc[r] * vc;
          }
        }
      }
      float ruk_all[U];                                      // each token's, to every lane
#pragma unroll
      for (int q4 = 0; q4 < U; q4 += 4) {
        const float four[4] = {ruk[q4], ruk[q4 + 1], ruk[q4 + 2], ruk[q4 + 3]};
        const float mine = lanes_sum4(four, lane);           // of token q4 + lane % 4
        ruk_all[q4] = dpp_from<0x00>(mine);
        ruk_all[q4 + 1] = dpp_from<0x55>(mine);
        ruk_all[q4 + 2] = dpp_from<0xAA>(mine);
        ruk_all[q4 + 3] = dpp_from<0xFF>(mine);
      }
#pragma unroll
      for (int uu = 0; uu < U; ++uu) {
        const float total = lanes_sum_cols<NC>(o[uu], lane);
        if (lane / NC == (tb + uu) % GROUP) gathered = total + ruk_all[uu] * v_own[uu];
      }
      if ((tb + U) % GROUP == 0 || tb + U >= n) {
        const int token = tb / GROUP * GROUP + lane / NC;
        if (token < n && token < tb + U && j0 + (lane & (NC - 1)) < d)
          out[(long long)(tile + token) * ld + head * d + j0 + (lane & (NC - 1))] = gathered;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c)
    if (j0 + c < d) {
#pragma unroll
      for (int r = 0; r < KR; ++r)
        if (lane + r * kWave < d) base[(long long)(j0 + c) * d + lane + r * kWave] = S[c][r];
    }
}

// --------------------------------------------------- per-head RMS norm, weight and gate
// y[t][h][j] = o / sqrt(mean_j o^2 + eps) * weight[h * weight_stride + j] * silu(gate[t][h][j])
// (with sigmoid_gate: * sigmoid(gate[t][h][j])).  One wave per (token, head); one head of
// heads * dv channels is the norm over the heads together.
template <typename TG, typename TO>
__global__ __launch_bounds__(kWave) void head_norm_gate_kernel(
    TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ weight,
    int weight_stride, const TG* __restrict__ gate, long long ldg, int heads, int dv, float eps,
    int sigmoid_gate) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* row = o + ((long long)t * heads + h) * dv;
  float ss = 0.f;
  for (int j = threadIdx.x; j < dv; j += kWave) ss += row[j] * row[j];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int j = threadIdx.x; j < dv; j += kWave) {
    const float g = ld(gate + (long long)t * ldg + h * dv + j);
    st(out + ((long long)t * heads + h) * dv + j,
       row[j] * inv * weight[h * weight_stride + j] *
           (sigmoid_gate ? 1.0f / (1.0f + expf(-g)) : siluf_(g)));
  }
}

// The same for heads of many channels (the norm over all the heads together): a workgroup of
// four waves per (token, head), their sums of squares joined through LDS in a fixed order.
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_wide_kernel(
    TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ weight,
    int weight_stride, const TG* __restrict__ gate, long long ldg, int heads, int dv, float eps,
    int sigmoid_gate) {
  __shared__ float partial[4];
  const int t = blockIdx.x, h = blockIdx.y;
  const float* row = o + ((long long)t * heads + h) * dv;
  float ss = 0.f;
  for (int j = threadIdx.x; j < dv; j += 256) ss += row[j] * row[j];
  ss = wave_sum(ss);
  if (threadIdx.x % kWave == 0) partial[threadIdx.x / kWave] = ss;
  __syncthreads();
  ss = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int j = threadIdx.x; j < dv; j += 256) {
    const float g = ld(gate + (long long)t * ldg + h * dv + j);
    st(out + ((long long)t * heads + h) * dv + j,
       row[j] * inv * weight[h * weight_stride + j] *
           (sigmoid_gate ? 1.0f / (1.0f + expf(-g)) : siluf_(g)));
  }
}

}  // namespace

// ============================================================================ entry points
static int scan_compute_units() {
  static int units = 0;
  if (units == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    units = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
                ? prop.multiProcessorCount : 256;
  }
  return units;
}

RLIS_API int rlis_shift_mix(void* out, const void* x, int dtype, const float* mu,
                            const float* state, long long state_stride, const int* seq_of_token,
                            const int* cu, const int* slots, int T, int W, int mixes,
                            hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && W > 0 && mixes > 0, "shift_mix: bad sizes T=%d W=%d mixes=%d", T, W, mixes);
  RLIS_REQUIRE(state_stride >= W, "shift_mix: the state is shorter than a row");
  RLIS_REQUIRE(ceil_div(W, 256) <= 65535, "shift_mix: W=%d is too wide", W);
  if (T == 0) return 0;
  const dim3 grid(T, ceil_div(W, 256));
  if (dtype == RLIS_F32)
    shift_mix_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (const float*)x, mu, state,
                                                   state_stride, seq_of_token, cu, slots, T, W,
                                                   mixes);
  else if (dtype == RLIS_BF16)
    shift_mix_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, mu, state,
                                                    state_stride, seq_of_token, cu, slots, T, W,
                                                    mixes);
  else
    RLIS_REQUIRE(false, "shift_mix: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("shift_mix");
  return 0;
}

RLIS_API int rlis_tail_update(float* state, long long state_stride, const void* x, int dtype,
                              long long ldx, int C, int R, const int* cu, const int* slots,
                              int num_seqs, hipStream_t stream) {
  RLIS_REQUIRE(C > 0 && R >= 0 && R <= 16, "tail_update: bad sizes C=%d rows=%d (at most 16)", C, R);
  RLIS_REQUIRE(state_stride >= (long long)C * R && ldx >= C, "tail_update: strides too short");
  RLIS_REQUIRE(num_seqs <= 65535, "tail_update: %d sequences, at most 65535", num_seqs);
  if (num_seqs <= 0 || R == 0) return 0;
  const dim3 grid(ceil_div(C, 256), num_seqs);
  if (dtype == RLIS_F32)
    tail_update_kernel<float><<<grid, 256, 0, stream>>>(state, state_stride, (const float*)x, ldx,
                                                        C, R, cu, slots);
  else if (dtype == RLIS_BF16)
    tail_update_kernel<bf16_t><<<grid, 256, 0, stream>>>(state, state_stride, (const bf16_t*)x,
                                                         ldx, C, R, cu, slots);
  else
    RLIS_REQUIRE(false, "tail_update: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("tail_update");
  return 0;
}

RLIS_API int rlis_causal_conv(void* out, int out_dtype, const float* x, long long ldx, const float* taps,
                              const float* bias, int C, int K, const float* state,
                              long long state_stride,
                              const int* seq_of_token, const int* cu, const int* slots, int T,
                              int unit_channels, int unit_group, int scaled_channels, float scale,
                              float unit_eps, int rest_group, int activation, const void* blend,
                              long long ld_blend, int blend_from, float blend_weight,
                              hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && C > 0 && K >= 1 && K <= 16, "causal_conv: bad sizes T=%d C=%d taps=%d", T, C, K);
  RLIS_REQUIRE(!blend || (blend_from >= 0 && blend_from < C && ld_blend >= C - blend_from),
               "causal_conv: the rows to mix in do not cover channels %d to %d", blend_from, C);
  RLIS_REQUIRE(ldx >= C && state_stride >= (long long)C * (K - 1), "causal_conv: strides too short");
  RLIS_REQUIRE(unit_channels >= 0 && unit_channels <= C && scaled_channels <= unit_channels,
               "causal_conv: bad channel ranges");
  RLIS_REQUIRE(unit_channels == 0 || (unit_group > 0 && unit_group <= 1024 &&
                                      unit_channels % unit_group == 0 &&
                                      scaled_channels % unit_group == 0),
               "causal_conv: unit groups of %d do not tile %d channels", unit_group, unit_channels);
  RLIS_REQUIRE(unit_channels == C || (rest_group > 0 && rest_group <= 1024),
               "causal_conv: bad group size %d for the other channels", rest_group);
  if (T == 0) return 0;
  const int groups = (unit_channels ? unit_channels / unit_group : 0) +
                     (unit_channels < C ? ceil_div(C - unit_channels, rest_group) : 0);
  RLIS_REQUIRE(ceil_div(groups, 4) <= 65535, "causal_conv: too many groups");
#define LAUNCH(TO)                                                                           \
  causal_conv_kernel<TO><<<dim3(T, ceil_div(groups, 4)), 256, 0, stream>>>(                    \
      (TO*)out, x, ldx, taps, bias, C, K, state, state_stride, seq_of_token, cu, slots,        \
      unit_channels, unit_group, scaled_channels, scale, unit_eps,                             \
      rest_group > 0 ? rest_group : 1, groups, activation, (const TO*)blend, ld_blend,         \
      blend_from, blend_weight)
  if (out_dtype == RLIS_F32) LAUNCH(float);
  else if (out_dtype == RLIS_BF16) LAUNCH(bf16_t);
  else RLIS_REQUIRE(false, "causal_conv: unknown dtype %d", out_dtype);
#undef LAUNCH
  RLIS_LAUNCH_CHECK("causal_conv");
  return 0;
}

RLIS_API int rlis_delta_scan(float* out, long long ldo, const float* q, const float* k,
                             const float* v, long long ldqkv, const float* b_raw,
                             const float* a_raw, long long ldba, const float* a_log,
                             const float* dt_bias, float* state, long long state_stride,
                             const int* cu, const int* slots, int num_seqs, int heads,
                             int kv_heads, int dk, int dv, int tiled, hipStream_t stream) {
  RLIS_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dk > 0 && dv > 0,
               "delta_scan: bad sizes heads=%d kv_heads=%d dk=%d dv=%d", heads, kv_heads, dk, dv);
  RLIS_REQUIRE(dk <= 256, "delta_scan: %d key channels, at most 256", dk);
  RLIS_REQUIRE(state_stride >= (long long)heads * dk * dv, "delta_scan: the state is too short");
  RLIS_REQUIRE(heads <= 65535 && num_seqs <= 65535, "delta_scan: grid too large");
  if (num_seqs <= 0) return 0;
  const dim3 grid(ceil_div(dv, 4 * kCols), heads, num_seqs);
#define LAUNCH(KR)                                                                            \
  delta_scan_kernel<KR><<<grid, 256, 0, stream>>>(out, ldo, q, k, v, ldqkv, b_raw, a_raw, ldba, \
                                                  a_log, dt_bias, state, state_stride, cu,    \
                                                  slots, heads, kv_heads, dk, dv)
  // Few workgroups (a single prompt): two value channels a wave instead of four, twice the waves.
  // (tiled 2 / 3: four / two channels a wave whatever the grid, for tests)
  const bool narrow = tiled == 3 || (tiled == 1 && (long long)grid.x * heads * num_seqs < 2 * scan_compute_units());
  const dim3 grid2(ceil_div(dv, 4 * 2), heads, num_seqs);
#define LAUNCH_TILED(KR)                                                                      \
  if (narrow)                                                                                 \
    delta_scan_tiled_kernel<KR, 2><<<grid2, 256, 0, stream>>>(                                \
        out, ldo, q, k, v, ldqkv, b_raw, a_raw, ldba, a_log, dt_bias, state, state_stride, cu, \
        slots, heads, kv_heads, dk, dv);                                                      \
  else                                                                                        \
    delta_scan_tiled_kernel<KR, kCols><<<grid, 256, 0, stream>>>(                             \
        out, ldo, q, k, v, ldqkv, b_raw, a_raw, ldba, a_log, dt_bias, state, state_stride, cu, \
        slots, heads, kv_heads, dk, dv)
  // `tiled`: some sequence of the step brings many tokens (the caller knows from the host)
  if (tiled) {
    if (dk <= 64) { LAUNCH_TILED(1); }
    else if (dk <= 128) { LAUNCH_TILED(2); }
    else { LAUNCH_TILED(4); }
  } else if (dk <= 64) LAUNCH(1);
  else if (dk <= 128) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
#undef LAUNCH_TILED
  RLIS_LAUNCH_CHECK("delta_scan");
  return 0;
}

RLIS_API int rlis_decay_scan(float* out, const float* r, const float* k, const float* v,
                             const float* z, long long ld, const float* w0, const float* bonus,
                             float* state, long long state_stride, const int* cu,
                             const int* slots, int num_seqs, int heads, int d, int tiled,
                             hipStream_t stream) {
  RLIS_REQUIRE(heads > 0 && d > 0 && d <= 256, "decay_scan: bad sizes heads=%d d=%d (at most 256)",
               heads, d);
  RLIS_REQUIRE(ld >= (long long)heads * d, "decay_scan: rows shorter than heads x d");
  RLIS_REQUIRE(state_stride >= (long long)heads * d * d, "decay_scan: the state is too short");
  RLIS_REQUIRE(heads <= 65535 && num_seqs <= 65535, "decay_scan: grid too large");
  if (num_seqs <= 0) return 0;
  const dim3 grid(ceil_div(d, 4 * kCols), heads, num_seqs);
#define LAUNCH(KR)                                                                           \
  decay_scan_kernel<KR><<<grid, 256, 0, stream>>>(out, r, k, v, z, ld, w0, bonus, state,     \
                                                  state_stride, cu, slots, heads, d)
  const bool narrow = tiled == 3 || (tiled == 1 && (long long)grid.x * heads * num_seqs < 2 * scan_compute_units());
  const dim3 grid2(ceil_div(d, 4 * 2), heads, num_seqs);
#define LAUNCH_TILED(KR)                                                                     \
  if (narrow)                                                                                \
    decay_scan_tiled_kernel<KR, 2><<<grid2, 256, 0, stream>>>(out, r, k, v, z, ld, w0, bonus, \
                                                              state, state_stride, cu, slots, \
                                                              heads, d);                     \
  else                                                                                       \
    decay_scan_tiled_kernel<KR, kCols><<<grid, 256, 0, stream>>>(out, r, k, v, z, ld, w0,     \
                                                                 bonus, state, state_stride, \
                                                                 cu, slots, heads, d)
  if (tiled) {
    if (d <= 64) { LAUNCH_TILED(1); }
    else if (d <= 128) { LAUNCH_TILED(2); }
    else { LAUNCH_TILED(4); }
  } else if (d <= 64) LAUNCH(1);
  else if (d <= 128) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
#undef LAUNCH_TILED
  RLIS_LAUNCH_CHECK("decay_scan");
  return 0;
}

RLIS_API int rlis_head_norm_gate(void* out, int out_dtype, const float* o, const float* weight,
                                 int weight_stride, const void* gate, int gate_dtype,
                                 long long ldg, int T, int heads, int dv, float eps,
                                 int sigmoid_gate, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && heads > 0 && dv > 0 && heads <= 65535,
               "head_norm_gate: bad sizes T=%d heads=%d dv=%d", T, heads, dv);
  RLIS_REQUIRE(weight_stride == 0 || weight_stride == dv, "head_norm_gate: bad weight stride");
  if (T == 0) return 0;
  const dim3 grid(T, heads);
  const int key = gate_dtype * 2 + out_dtype;
  const bool wide = dv >= 512;       // (by the head's size alone: a row's sums do not depend on the batch)
#define CASE(k_, TG, TO)                                                                     \
  case k_:                                                                                   \
    if (wide)                                                                                \
      head_norm_gate_wide_kernel<TG, TO><<<grid, 256, 0, stream>>>(                          \
          (TO*)out, o, weight, weight_stride, (const TG*)gate, ldg, heads, dv, eps,          \
          sigmoid_gate);                                                                     \
    else                                                                                     \
      head_norm_gate_kernel<TG, TO><<<grid, kWave, 0, stream>>>(                             \
          (TO*)out, o, weight, weight_stride, (const TG*)gate, ldg, heads, dv, eps,          \
          sigmoid_gate);                                                                     \
    break;
  switch (key) {
    CASE(0, float, float)
    CASE(1, float, bf16_t)
    CASE(2, bf16_t, float)
    CASE(3, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "head_norm_gate: unknown dtypes %d %d", gate_dtype, out_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("head_norm_gate");
  return 0;
}


// ------------------------------------------------------------------ selective scan
// A state of N numbers per channel with an input-dependent step: per token and channel c
//   dt = softplus(dt_raw[c] + dt_bias[c]);  S[c][n] <- exp(dt A[c][n]) S[c][n] + dt x[c] B[n];
//   y[c] = sum_n S[c][n] C[n] + D[c] x[c];  out[c] = y[c] * silu(z[c]),
// with A = -exp(A_log).  B and C (N numbers each) are the token's, shared by the channels.
// LPC lanes share a channel, lane `sub` of them holding states n = sub, sub + LPC, ...; a
// token's sum over n ends with log2(LPC) exchanges between those lanes.  A sequence's tokens
// are walked in order from the state its slot holds, which is left as after the last one.
// x (the convolution's output) and the result are in the activation dtype; everything else,
// the state included, is float32.
// Sum over the LPC neighbouring lanes that share a channel (4, 16 or 64, aligned): adds between
// lanes of a row of 16 by data-parallel primitives, no trip through LDS; every lane gets it.
template <int LPC>
__device__ __forceinline__ float channel_sum(float v) {
  if (LPC == 64) return lanes_sum(v);
  v += dpp_from<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  v += dpp_from<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if (LPC == 16) {
    v += dpp_from<0x141>(v);   // row_half_mirror
    v += dpp_from<0x140>(v);   // row_mirror
  }
  return v;
}

// PASS 0: a workgroup row per sequence, from the slot's state to the slot's state.  The chunked
// form for long prompts cuts every sequence into chunks of chunk_len tokens (a workgroup row
// per chunk) and runs three launches: PASS 1 walks every chunk from a zero state and leaves the
// chunk's end state and the sum of its steps (the product of a chunk's decays is
// exp(A * that sum)); selective_scan_join walks a sequence's chunks in order,
// S <- exp(A sum) S + end, from the slot's state, leaves every chunk's true start state where
// its end state was and the sequence's last state in the slot; PASS 2 walks every chunk again
// from its start state and makes the outputs.  The recurrence is linear in the state, so this
// is the sequential walk up to the order of a few additions.
template <typename TO, int NPL, int LPC, int PASS>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    TO* __restrict__ out, long long ldo, const TO* __restrict__ x, long long ldx,
    const float* __restrict__ dt_raw, long long lddt, const float* __restrict__ dt_bias,
    const float* __restrict__ bmat, const float* __restrict__ cmat, long long ldbc,
    const float* __restrict__ z, long long ldz, const float* __restrict__ a_log,
    const float* __restrict__ dskip, float* __restrict__ state, long long state_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, int C, int N, int num_seqs,
    int chunk_len, float* __restrict__ chunk_state, float* __restrict__ chunk_dt) {
  int s = blockIdx.y;
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  const int c = gid / LPC, sub = gid % LPC;
  if (c >= C) return;                 // (LPC divides the wave: a channel's lanes stay together)
  int t0, t1;
  if (PASS == 0) {
    t0 = cu[s];
    t1 = cu[s + 1];
  } else {                            // blockIdx.y counts chunks over all sequences
    int k = blockIdx.y;
    for (s = 0; s < num_seqs; ++s) {
      const int chunks = (cu[s + 1] - cu[s] + chunk_len - 1) / chunk_len;
      if (k < chunks) break;
      k -= chunks;
    }
    if (s == num_seqs) return;
    t0 = cu[s] + k * chunk_len;
    t1 = min(t0 + chunk_len, cu[s + 1]);
  }
  float* S = PASS == 0 ? state + (long long)slots[s] * state_stride + (long long)c * N
                       : chunk_state + ((long long)blockIdx.y * C + c) * N;
  float st_[NPL], a[NPL];
#pragma unroll
  for (int j = 0; j < NPL; ++j) {
    const int n = sub + j * LPC;
    st_[j] = (PASS != 1 && n < N) ? S[n] : 0.f;
    a[j] = n < N ? -expf(a_log[(long long)c * N + n]) : 0.f;
  }
  float dt_sum = 0.f;
  const float bias = dt_bias[c], dsk = dskip[c];
  // Tokens are walked in groups of kScanGroup: everything that does not depend on the state
  // (a token's step, input, gate, B and C, and the decays exp(dt A)) is asked for and made for
  // the whole group first, so that the walk itself waits for no load; tokens past the
  // sequence's end take the last token's addresses and are not stored.
  constexpr int G = NPL <= 8 ? 8 : 4;
  if (PASS == 0 && t1 - t0 == 1) {             // a decoded token: nothing to group
    const int t = t0;
    const float raw = dt_raw[(long long)t * lddt + c] + bias;
    const float dt = raw > 20.f ? raw : log1pf(expf(raw));
    const float xs = ld(x + (long long)t * ldx + c), dx = dt * xs;
    float y = 0.f;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
      const int n = sub + j * LPC;
      const int nn = n < N ? n : 0;
      const float v = expf(dt * a[j]) * st_[j] + dx * bmat[(long long)t * ldbc + nn];
      st_[j] = n < N ? v : 0.f;
      y = fmaf(st_[j], cmat[(long long)t * ldbc + nn], y);
    }
    y = channel_sum<LPC>(y);
    if (sub == 0) {
      const float zs = z[(long long)t * ldz + c];
      st(out + (long long)t * ldo + c, (y + dsk * xs) * (zs / (1.0f + expf(-zs))));
    }
  } else
  for (int tg = t0; tg < t1; tg += G) {
    float dtv[G], xv[G], zv[G], bn[G][NPL], cn[G][NPL];
#pragma unroll
    for (int u = 0; u < G; ++u) {
      const int t = min(tg + u, t1 - 1);
      dtv[u] = dt_raw[(long long)t * lddt + c];
      xv[u] = ld(x + (long long)t * ldx + c);
      zv[u] = z[(long long)t * ldz + c];
#pragma unroll
      for (int j = 0; j < NPL; ++j) {
        const int n = sub + j * LPC;
        const int nn = n < N ? n : 0;
        bn[u][j] = bmat[(long long)t * ldbc + nn];
        cn[u][j] = cmat[(long long)t * ldbc + nn];
      }
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
      const float raw = dtv[u] + bias;
      dtv[u] = raw > 20.f ? raw : log1pf(expf(raw));
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
      if (tg + u < t1) {                       // (the same for all lanes of a sequence)
        const float dt = dtv[u], dx = dt * xv[u];
        dt_sum += dt;
        float y = 0.f;
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
          const int n = sub + j * LPC;
          const float v = expf(dt * a[j]) * st_[j] + dx * bn[u][j];
          st_[j] = n < N ? v : 0.f;
          y = fmaf(st_[j], cn[u][j], y);
        }
        if (PASS != 1) {
          y = channel_sum<LPC>(y);
          if (sub == 0)
            st(out + (long long)(tg + u) * ldo + c,
               (y + dsk * xv[u]) * (zv[u] / (1.0f + expf(-zv[u]))));
        }
      }
    }
  }
  if (PASS == 2) return;               // (the join has left the sequence's last state in the slot)
#pragma unroll
  for (int j = 0; j < NPL; ++j) {
    const int n = sub + j * LPC;
    if (n < N) S[n] = st_[j];
  }
  if (PASS == 1 && sub == 0) chunk_dt[(long long)blockIdx.y * C + c] = dt_sum;
}

// One thread per (sequence, channel, state): the sequence's chunks in order.
__global__ void selective_scan_join_kernel(float* __restrict__ state, long long state_stride,
                                           const float* __restrict__ a_log,
                                           float* __restrict__ chunk_state,
                                           const float* __restrict__ chunk_dt,
                                           const int* __restrict__ cu,
                                           const int* __restrict__ slots, int C, int N,
                                           int chunk_len) {
  const int s = blockIdx.y;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)C * N) return;
  const int c = (int)(i / N);
  int first = 0;
  for (int q = 0; q < s; ++q) first += (cu[q + 1] - cu[q] + chunk_len - 1) / chunk_len;
  const int chunks = (cu[s + 1] - cu[s] + chunk_len - 1) / chunk_len;
  float* slot = state + (long long)slots[s] * state_stride + i;
  const float a = -expf(a_log[i]);
  float S = *slot;
  for (int k = 0; k < chunks; ++k) {
    float* at = chunk_state + (long long)(first + k) * C * N + i;
    const float end = *at;
    *at = S;
    S = expf(a * chunk_dt[(long long)(first + k) * C + c]) * S + end;
  }
  *slot = S;
}

RLIS_API int rlis_selective_scan(void* out, int out_dtype, long long ldo, const void* x,
                                 long long ldx, const float* dt_raw, long long lddt,
                                 const float* dt_bias, const float* bmat, const float* cmat,
                                 long long ldbc, const float* z, long long ldz,
                                 const float* a_log, const float* dskip, float* state,
                                 long long state_stride, const int* cu, const int* slots,
                                 int num_seqs, int C, int N, int long_runs, int chunk_len,
                                 int max_chunks, float* chunk_state, float* chunk_dt,
                                 hipStream_t stream) {
  RLIS_REQUIRE(num_seqs >= 0 && C > 0 && N > 0, "selective_scan: bad sizes C=%d N=%d", C, N);
  RLIS_REQUIRE(N <= 1024, "selective_scan: a state of %d numbers per channel is too large", N);
  RLIS_REQUIRE(ldo >= C && ldx >= C && lddt >= C && ldz >= C && ldbc >= N &&
                   state_stride >= (long long)C * N,
               "selective_scan: strides shorter than rows");
  RLIS_REQUIRE(num_seqs <= 65535, "selective_scan: too many sequences");
  if (num_seqs == 0) return 0;
  RLIS_REQUIRE(chunk_len == 0 || (chunk_len > 0 && max_chunks > 0 && max_chunks <= 65535 &&
                                  chunk_state && chunk_dt),
               "selective_scan: the chunked form needs its scratch and at most 65,535 chunks");
#define LAUNCH_PASS(TO, NPL, LPC, PASS, ROWS)                                                 \
  selective_scan_kernel<TO, NPL, LPC, PASS>                                                   \
      <<<dim3(ceil_div(C * LPC, 256), ROWS), 256, 0, stream>>>(                               \
          (TO*)out, ldo, (const TO*)x, ldx, dt_raw, lddt, dt_bias, bmat, cmat, ldbc, z, ldz,  \
          a_log, dskip, state, state_stride, cu, slots, C, N, num_seqs, chunk_len,            \
          chunk_state, chunk_dt)
#define LAUNCH(TO, NPL, LPC)                                                                  \
  do {                                                                                        \
    if (chunk_len > 0) {                                                                      \
      LAUNCH_PASS(TO, NPL, LPC, 1, max_chunks);                                               \
      selective_scan_join_kernel<<<dim3(ceil_div(C * N, 256), num_seqs), 256, 0, stream>>>(   \
          state, state_stride, a_log, chunk_state, chunk_dt, cu, slots, C, N, chunk_len);     \
      LAUNCH_PASS(TO, NPL, LPC, 2, max_chunks);                                               \
    } else {                                                                                  \
      LAUNCH_PASS(TO, NPL, LPC, 0, num_seqs);                                                 \
    }                                                                                         \
  } while (0)
  // long_runs: sequences bring many tokens each and there are few of them, so a channel's states
  // are spread over more lanes (more waves on a chip that the walk leaves mostly idle); the sum
  // over the states is then added up in another order
#define BY_N(TO)                                  \
  do {                                            \
    if (N <= 16 && long_runs) LAUNCH(TO, 1, 16);  \
    else if (N <= 16) LAUNCH(TO, 4, 4);           \
    else if (N <= 64 && long_runs) LAUNCH(TO, 4, 16); \
    else if (N <= 32) LAUNCH(TO, 8, 4);           \
    else if (N <= 64) LAUNCH(TO, 16, 4);          \
    else if (N <= 256) LAUNCH(TO, 16, 16);        \
    else LAUNCH(TO, 16, 64);                      \
  } while (0)
  if (out_dtype == RLIS_F32) BY_N(float);
  else if (out_dtype == RLIS_BF16) BY_N(bf16_t);
  else RLIS_REQUIRE(false, "selective_scan: unknown dtype %d", out_dtype);
#undef BY_N
#undef LAUNCH
#undef LAUNCH_PASS
  RLIS_LAUNCH_CHECK("selective_scan");
  return 0;
}
