// Linear attention with one fixed decay per head: per (sequence, head) a matrix state S (key
// channel x value channel, float32, kept in the request's state slot) with
//
//     S_t = decay_h * S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t
//
// (the token's own key and value are in what its query reads; no other scale).  q, k and v come
// as the raw projections and pass `activation` (1: SiLU, 0: nothing) in float32 on the way in.
// State layout per head: [value channel][key channel], so that the wave that owns a value
// channel reads its column contiguously.  Everything but the stored inputs is float32.
//
//  * decay_attention_scan: token by token.  A wave owns four value channels of one (sequence,
//    head), lane i holds S[.][i + 64 r]; the next token's inputs are asked for before the
//    current token's sums.  Decode steps and short portions.
//  * decay_attention_chunks: long portions in chunks of 64 tokens on the matrix cores (float32
//    products): a chunk's own contribution to the state, a sequential pass over the chunks that
//    leaves every chunk's start state, and the chunk's read-outs
//    O = (Q K^T . D) V + diag(decay^(t+1)) Q S_start with D[t][s] = decay^(t-s) for s <= t.
#include "common.h"
#include "tile_mma.h"

#include <math.h>

namespace {

__device__ __forceinline__ float act_in(float x, int activation) {
  return activation ? x / (1.0f + expf(-x)) : x;
}

template <typename TX, int KR>
__global__ __launch_bounds__(256) void decay_attention_scan_kernel(
    float* __restrict__ out, const TX* __restrict__ q, long long ldq, const TX* __restrict__ k,
    long long ldk, const TX* __restrict__ v, long long ldv, const float* __restrict__ decay,
    float* __restrict__ state, long long state_stride, const int* __restrict__ cu,
    const int* __restrict__ slots, int H, int d, int dv, int activation) {
  constexpr int VC = 4;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int h = blockIdx.y, s = blockIdx.z;
  const int j0 = (blockIdx.x * 4 + wave) * VC;
  if (j0 >= dv) return;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  const float lam = decay[h];
  float* base = state + (long long)slots[s] * state_stride + ((long long)h * dv + j0) * d;
  int jc[VC];              // value channels past the head's end work on the last one, unstored
#pragma unroll
  for (int c = 0; c < VC; ++c) jc[c] = min(j0 + c, dv - 1);
  float S[VC][KR];
#pragma unroll
  for (int c = 0; c < VC; ++c)
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = lane + r * kWave;
      S[c][r] = i < d ? base[(long long)(jc[c] - j0) * d + i] : 0.f;
    }
  float qn[KR], kn[KR], vn[VC];
  auto load = [&](int t) {
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = min(lane + r * kWave, d - 1);
      qn[r] = ld(q + (long long)t * ldq + h * d + i);
      kn[r] = ld(k + (long long)t * ldk + h * d + i);
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) vn[c] = ld(v + (long long)t * ldv + h * dv + jc[c]);
  };
  load(t0);
  for (int t = t0; t < t1; ++t) {
    float qv[KR], kv[KR], vv[VC];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const bool live = lane + r * kWave < d;
      qv[r] = live ? act_in(qn[r], activation) : 0.f;
      kv[r] = live ? act_in(kn[r], activation) : 0.f;
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) vv[c] = act_in(vn[c], activation);
    load(t + 1 < t1 ? t + 1 : t);
    float p[VC];
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      float a = 0.f;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        S[c][r] = fmaf(lam, S[c][r], kv[r] * vv[c]);
        a = fmaf(S[c][r], qv[r], a);
      }
      p[c] = a;
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) p[c] = wave_sum(p[c]);
    if (lane < VC && j0 + lane < dv) {
      const float o = lane == 0 ? p[0] : (lane == 1 ? p[1] : (lane == 2 ? p[2] : p[3]));
      out[(long long)t * H * dv + h * dv + j0 + lane] = o;
    }
  }
#pragma unroll
  for (int c = 0; c < VC; ++c)
    if (j0 + c < dv) {
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const int i = lane + r * kWave;
        if (i < d) base[(long long)c * d + i] = S[c][r];
      }
    }
}

}  // namespace

// out (T, H * dv) float32; q, k (T, >= H * d) and v (T, >= H * dv) with row strides, float32 or
// bfloat16 alike; decay (H) float32; state: per slot H * dv * d floats from `state` on, slots
// state_stride floats apart; cu (S + 1) and slots (S) as every scan takes them.
RLIS_API int rlis_decay_attention_scan(float* out, const void* q, long long ldq, const void* k,
                                       long long ldk, const void* v, long long ldv, int dtype,
                                       const float* decay, float* state, long long state_stride,
                                       const int* cu, const int* slots, int S, int T, int H, int d,
                                       int dv, int activation, hipStream_t stream) {
  RLIS_REQUIRE(S >= 0 && T >= 0 && H > 0 && d > 0 && dv > 0,
               "decay_attention_scan: bad sizes S=%d T=%d H=%d d=%d dv=%d", S, T, H, d, dv);
  RLIS_REQUIRE(d <= 256, "decay_attention_scan: %d key channels a head, at most 256", d);
  RLIS_REQUIRE(H <= 65535 && S <= 65535, "decay_attention_scan: too many heads or sequences");
  RLIS_REQUIRE(ldq >= (long long)H * d && ldk >= (long long)H * d && ldv >= (long long)H * dv,
               "decay_attention_scan: row strides shorter than the heads");
  RLIS_REQUIRE(state_stride >= (long long)H * dv * d, "decay_attention_scan: state too short");
  if (S == 0 || T == 0) return 0;
  const dim3 grid(ceil_div(dv, 16), H, S);
  const int kr = ceil_div(d, kWave);
#define LAUNCH(TX, KR)                                                                          \
  decay_attention_scan_kernel<TX, KR><<<grid, 256, 0, stream>>>(                                \
      out, (const TX*)q, ldq, (const TX*)k, ldk, (const TX*)v, ldv, decay, state, state_stride, \
      cu, slots, H, d, dv, activation)
#define BY_KR(TX)                 \
  do {                            \
    if (kr <= 1) LAUNCH(TX, 1);   \
    else if (kr <= 2) LAUNCH(TX, 2); \
    else LAUNCH(TX, 4);           \
  } while (0)
  if (dtype == RLIS_F32) BY_KR(float);
  else if (dtype == RLIS_BF16) BY_KR(bf16_t);
  else RLIS_REQUIRE(false, "decay_attention_scan: unknown dtype %d", dtype);
#undef BY_KR
#undef LAUNCH
  RLIS_LAUNCH_CHECK("decay_attention_scan");
  return 0;
}
