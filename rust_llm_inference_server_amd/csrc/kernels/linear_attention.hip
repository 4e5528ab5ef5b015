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
//    products, v_mfma_f32_16x16x4_f32): a chunk's own contribution to the state, a pass over
//    each sequence's chunks in order that leaves every chunk's start state, and the chunk's
//    read-outs O = (Q K^T . D) V + diag(decay^(t+1)) Q S_start with D[t][s] = decay^(t-s) for
//    s <= t.  Chunks and heads run side by side; only the join is sequential, and it is one
//    multiply-add per state element and chunk.
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


// ---------------------------------------------------------------------------- chunked form
constexpr int kChunk = 64;           // tokens a chunk
constexpr int kTokStride = kChunk + 4;   // floats between rows that run along the tokens

__device__ __forceinline__ int round16(int n) { return (n + 15) / 16 * 16; }

// The b-th chunk of the step, counting every sequence's chunks of kChunk tokens in order:
// its sequence, its number inside it, its first token and how many it holds.  False: the step
// has fewer chunks.
struct ChunkAt {
  int seq, index, first, count, chunks_before_seq;
};

__device__ __forceinline__ bool find_chunk(const int* __restrict__ cu, int S, int b, ChunkAt& at) {
  int seen = 0;
  for (int s = 0; s < S; ++s) {
    const int t0 = cu[s], len = cu[s + 1] - t0;
    const int nc = (len + kChunk - 1) / kChunk;
    if (b < seen + nc) {
      at.seq = s;
      at.index = b - seen;
      at.first = t0 + at.index * kChunk;
      at.count = min(kChunk, t0 + len - at.first);
      at.chunks_before_seq = seen;
      return true;
    }
    seen += nc;
  }
  return false;
}

// A wave's tile of a product on the float32 matrix cores for operands that lie in LDS with any
// stride along k: C[i][n] = sum_k A[i][k] B[n][k] for 16 rows of A and NB blocks of 16 rows of
// B.  Every lane hands in the address of element k = 0 of the row it serves (row lane % 16 of A
// and of each block of B) and the distance between consecutive k.  The result's layout is that
// of wave_tile_product; K is a multiple of 4.
template <int NB>
__device__ __forceinline__ void wave_tile_product_strided(const float* a_lane, int a_kstride,
                                                          const float* const (&b_lane)[NB],
                                                          int b_kstride, int K,
                                                          mma_f32x4 (&acc)[NB]) {
  const int g = (threadIdx.x % kWave) / 16;
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = mma_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 4) {
    const float av = a_lane[(k0 + g) * a_kstride];
    float bv[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) bv[b] = b_lane[b][(k0 + g) * b_kstride];
#pragma unroll
    for (int b = 0; b < NB; ++b)
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv[b], acc[b], 0, 0, 0);
  }
}

// Rows first .. first + n - 1 of a projection (columns col0 .. col0 + width - 1, through the
// activation) into LDS as [token][channel], four channels a thread; rows from n on and
// channels from width to width16 are zeros.  VEC: 16-byte loads (width a multiple of 4, rows
// aligned).  l2 != 0 or weigh: row s is multiplied by 2^(l2 * (n - 1 - s)).
template <bool VEC>
__device__ __forceinline__ void fill_rows(float* dst, int dst_stride, const float* __restrict__ src,
                                          long long ld, int col0, int width, int width16,
                                          int first, int n, int activation, bool weigh, float l2) {
  const int groups = width16 / 4;
  for (int idx = threadIdx.x; idx < kChunk * groups; idx += blockDim.x) {
    const int s = idx / groups, i = (idx - s * groups) * 4;
    float val[4] = {0.f, 0.f, 0.f, 0.f};
    if (s < n && i < width) {
      const float* p = src + (long long)(first + s) * ld + col0 + i;
      if (VEC) {
        const mma_f32x4 v = *reinterpret_cast<const mma_f32x4*>(p);
#pragma unroll
        for (int c = 0; c < 4; ++c) val[c] = v[c];
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) val[c] = i + c < width ? p[c] : 0.f;
      }
      const float w = weigh ? exp2f(l2 * (float)(n - 1 - s)) : 1.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) val[c] = i + c < width ? act_in(val[c], activation) * w : 0.f;
    }
    *reinterpret_cast<mma_f32x4*>(dst + s * dst_stride + i) =
        mma_f32x4{val[0], val[1], val[2], val[3]};
  }
}

// What a chunk of n tokens adds to the state, from a zero state: A[j][i] = sum_s decay^(n-1-s)
// k_s[i] v_s[j], the product over the tokens of V and of K with the decays folded in, both in
// LDS as they come ([token][channel]).  grid (chunks, heads); ws holds (chunk, head, value
// channel, key channel).
template <bool VEC>
__global__ __launch_bounds__(256) void decay_chunk_states_kernel(
    float* __restrict__ ws, const float* __restrict__ k, long long ldk,
    const float* __restrict__ v, long long ldv, const float* __restrict__ decay,
    const int* __restrict__ cu, int S, int H, int d, int dv, int activation) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  ChunkAt at;
  if (!find_chunk(cu, S, blockIdx.x, at)) return;
  const int h = blockIdx.y, n = at.count;
  const int d16 = round16(d), dv16 = round16(dv), DS = d16 + 4, DVS = dv16 + 4;
  float* Ks = lds;                          // [kChunk][DS]
  float* Vs = lds + kChunk * DS;            // [kChunk][DVS]
  fill_rows<VEC>(Ks, DS, k, ldk, h * d, d, d16, at.first, n, activation, true, log2f(decay[h]));
  fill_rows<VEC>(Vs, DVS, v, ldv, h * dv, dv, dv16, at.first, n, activation, false, 0.f);
  __syncthreads();
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int l16 = lane % 16, lg = lane / 16;
  float* out = ws + ((long long)blockIdx.x * H + h) * dv * d;
  const int iblocks = d16 / 16;
  for (int jb = wave; jb < dv16 / 16; jb += 4) {
    const float* a_lane = Vs + jb * 16 + l16;
    for (int ib0 = 0; ib0 < iblocks; ib0 += 4) {
      const float* b_lane[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) b_lane[b] = Ks + min(ib0 + b, iblocks - 1) * 16 + l16;
      mma_f32x4 acc[4];
      wave_tile_product_strided<4>(a_lane, DVS, b_lane, DS, kChunk, acc);
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int i = (ib0 + b) * 16 + l16;
        if (ib0 + b < iblocks && i < d) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int j = jb * 16 + 4 * lg + r;
            if (j < dv) out[(long long)j * d + i] = acc[b][r];
          }
        }
      }
    }
  }
}

// Every sequence's chunks in order: the chunk's entry in ws becomes the state in front of it,
// the state moves on by S <- decay^n S + A, and the slot keeps what the last chunk leaves.  A
// thread per state element; grid (elements / 256, sequences).
__global__ __launch_bounds__(256) void decay_chunk_join_kernel(
    float* __restrict__ ws, float* __restrict__ state, long long state_stride,
    const float* __restrict__ decay, const int* __restrict__ cu, const int* __restrict__ slots,
    int H, int d, int dv) {
  const int s = blockIdx.y;
  const long long per_head = (long long)dv * d, all = per_head * H;
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= all) return;
  const int len = cu[s + 1] - cu[s];
  if (len <= 0) return;
  int first = 0;
  for (int p = 0; p < s; ++p) first += (cu[p + 1] - cu[p] + kChunk - 1) / kChunk;
  const float l2 = log2f(decay[(int)(e / per_head)]);
  const float whole = exp2f(l2 * (float)kChunk);
  float* st = state + (long long)slots[s] * state_stride + e;
  float cur = *st;
  const int nc = (len + kChunk - 1) / kChunk;
  for (int c = 0; c < nc; ++c) {
    float* slot = ws + (long long)(first + c) * all + e;
    const float add = *slot;
    *slot = cur;
    const int n = min(kChunk, len - c * kChunk);
    cur = fmaf(n == kChunk ? whole : exp2f(l2 * (float)n), cur, add);
  }
  *st = cur;
}

// A chunk's read-outs from the state in front of it (ws) and from its own tokens:
// O = (Q K^T . D) V + diag(decay^(t+1)) Q S^T with D[t][s] = decay^(t-s) for s <= t, else 0.
// grid (chunks, heads); a wave owns 16 tokens.  VEC: 16-byte loads of the inputs;
// STATE_ALIGNED: the state's rows take 16-byte loads (d a multiple of 4).
template <bool VEC, bool STATE_ALIGNED>
__global__ __launch_bounds__(256) void decay_chunk_outputs_kernel(
    float* __restrict__ out, const float* __restrict__ q, long long ldq,
    const float* __restrict__ k, long long ldk, const float* __restrict__ v, long long ldv,
    const float* __restrict__ decay, const float* __restrict__ ws, const int* __restrict__ cu,
    int S, int H, int d, int dv, int activation) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  ChunkAt at;
  if (!find_chunk(cu, S, blockIdx.x, at)) return;
  const int h = blockIdx.y, n = at.count;
  const int d16 = round16(d), dv16 = round16(dv), DS = d16 + 4, DVS = dv16 + 4;
  float* Qs = lds;                              // [kChunk][DS]
  float* Ks = Qs + kChunk * DS;                 // [kChunk][DS]
  float* Vs = Ks + kChunk * DS;                 // [kChunk][DVS]
  float* Ps = Vs + kChunk * DVS;                // [kChunk][kTokStride]
  const float l2 = log2f(decay[h]);
  fill_rows<VEC>(Qs, DS, q, ldq, h * d, d, d16, at.first, n, activation, false, 0.f);
  fill_rows<VEC>(Ks, DS, k, ldk, h * d, d, d16, at.first, n, activation, false, 0.f);
  fill_rows<VEC>(Vs, DVS, v, ldv, h * dv, dv, dv16, at.first, n, activation, false, 0.f);
  __syncthreads();
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int l16 = lane % 16, lg = lane / 16;
  const float* q_row = Qs + (wave * 16 + l16) * DS;
  {
    const float* b_row[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) b_row[b] = Ks + (b * 16 + l16) * DS;
    mma_f32x4 acc[4];
    wave_tile_product<float, 4, true>(q_row, b_row, d16, acc);
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = wave * 16 + 4 * lg + r, s = b * 16 + l16;
        Ps[t * kTokStride + s] = s <= t ? acc[b][r] * exp2f(l2 * (float)(t - s)) : 0.f;
      }
  }
  __syncthreads();
  const float* p_row = Ps + (wave * 16 + l16) * kTokStride;
  const float* s0 = ws + ((long long)blockIdx.x * H + h) * dv * d;
  const int jblocks = dv16 / 16;
  float grown[4];                               // decay^(t + 1) of the lane's four tokens
#pragma unroll
  for (int r = 0; r < 4; ++r) grown[r] = exp2f(l2 * (float)(wave * 16 + 4 * lg + r + 1));
  for (int jb0 = 0; jb0 < jblocks; jb0 += 4) {
    const float* v_lane[4];
    const float* s_row[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int jb = min(jb0 + b, jblocks - 1);
      v_lane[b] = Vs + jb * 16 + l16;
      s_row[b] = s0 + (long long)min(jb * 16 + l16, dv - 1) * d;
    }
    mma_f32x4 own[4], carried[4];
    // (a wave's tokens see the keys up to its own last one)
    wave_tile_product_strided<4>(p_row, 1, v_lane, DVS, (wave + 1) * 16, own);
    wave_tile_product<float, 4, STATE_ALIGNED>(q_row, s_row, d, carried);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int j = (jb0 + b) * 16 + l16;
      if (jb0 + b < jblocks && j < dv) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = wave * 16 + 4 * lg + r;
          if (t < n)
            out[(long long)(at.first + t) * H * dv + h * dv + j] =
                fmaf(grown[r], carried[b][r], own[b][r]);
        }
      }
    }
  }
}

// More dynamic LDS than a kernel gets unasked, asked for once on every device.
static int grant_lds(const void* kernel, size_t bytes, bool* granted) {
  constexpr int kDevices = 64;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return 1;
  if (dev >= 0 && dev < kDevices && granted[dev]) return 0;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return 1;
  if (dev >= 0 && dev < kDevices) granted[dev] = true;
  return 0;
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

// The same result as rlis_decay_attention_scan (to rounding) for steps of long portions, in
// three launches: every chunk of 64 tokens from a zero state, the chunks of a sequence joined in
// order, every chunk's read-outs.  q, k, v float32; d and dv at most 128; ws: (max_chunks, H,
// dv, d) floats with max_chunks at least the step's chunks (T / 64 + S bounds them).
RLIS_API int rlis_decay_attention_chunks(float* out, const float* q, long long ldq,
                                         const float* k, long long ldk, const float* v,
                                         long long ldv, const float* decay, float* state,
                                         long long state_stride, const int* cu, const int* slots,
                                         int S, int T, int H, int d, int dv, int activation,
                                         float* ws, int max_chunks, hipStream_t stream) {
  RLIS_REQUIRE(S >= 0 && T >= 0 && H > 0 && d > 0 && dv > 0,
               "decay_attention_chunks: bad sizes S=%d T=%d H=%d d=%d dv=%d", S, T, H, d, dv);
  RLIS_REQUIRE(d <= 128 && dv <= 128,
               "decay_attention_chunks: heads of %d and %d channels, at most 128", d, dv);
  RLIS_REQUIRE(H <= 65535 && S <= 65535, "decay_attention_chunks: too many heads or sequences");
  RLIS_REQUIRE(ldq >= (long long)H * d && ldk >= (long long)H * d && ldv >= (long long)H * dv,
               "decay_attention_chunks: row strides shorter than the heads");
  RLIS_REQUIRE(state_stride >= (long long)H * dv * d, "decay_attention_chunks: state too short");
  RLIS_REQUIRE(ws && max_chunks >= T / kChunk + S,
               "decay_attention_chunks: workspace of %d chunks for %d tokens of %d sequences",
               max_chunks, T, S);
  if (S == 0 || T == 0) return 0;
  const int d16 = (d + 15) / 16 * 16, dv16 = (dv + 15) / 16 * 16;
  const size_t lds_states = (size_t)kChunk * (d16 + dv16 + 8) * sizeof(float);
  const size_t lds_outputs =
      (size_t)kChunk * (2 * (d16 + 4) + dv16 + 4 + kTokStride) * sizeof(float);
  constexpr size_t kMostLds = 160 * 1024;
  RLIS_REQUIRE(lds_outputs <= kMostLds, "decay_attention_chunks: %zu bytes of LDS", lds_outputs);
  const bool vec = d % 4 == 0 && dv % 4 == 0 && ldq % 4 == 0 && ldk % 4 == 0 && ldv % 4 == 0 &&
                   (uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0;
  const bool aligned = d % 4 == 0 && ((uintptr_t)ws % 16 == 0);
  static bool granted[6][64];
  const void* kernels[6] = {
      reinterpret_cast<const void*>(&decay_chunk_states_kernel<true>),
      reinterpret_cast<const void*>(&decay_chunk_states_kernel<false>),
      reinterpret_cast<const void*>(&decay_chunk_outputs_kernel<true, true>),
      reinterpret_cast<const void*>(&decay_chunk_outputs_kernel<false, true>),
      reinterpret_cast<const void*>(&decay_chunk_outputs_kernel<true, false>),
      reinterpret_cast<const void*>(&decay_chunk_outputs_kernel<false, false>)};
  for (int i = 0; i < 6; ++i)
    RLIS_REQUIRE(grant_lds(kernels[i], kMostLds, granted[i]) == 0,
                 "decay_attention_chunks: the device grants no %zu bytes of LDS", kMostLds);
  const dim3 grid(max_chunks, H);
  if (vec)
    decay_chunk_states_kernel<true><<<grid, 256, lds_states, stream>>>(ws, k, ldk, v, ldv, decay,
                                                                      cu, S, H, d, dv, activation);
  else
    decay_chunk_states_kernel<false><<<grid, 256, lds_states, stream>>>(ws, k, ldk, v, ldv, decay,
                                                                       cu, S, H, d, dv, activation);
  RLIS_LAUNCH_CHECK("decay_attention_chunks (states)");
  const long long elements = (long long)H * dv * d;
  decay_chunk_join_kernel<<<dim3((unsigned)((elements + 255) / 256), S), 256, 0, stream>>>(
      ws, state, state_stride, decay, cu, slots, H, d, dv);
  RLIS_LAUNCH_CHECK("decay_attention_chunks (join)");
#define OUTPUTS(V_, A_)                                                          \
  decay_chunk_outputs_kernel<V_, A_><<<grid, 256, lds_outputs, stream>>>(        \
      out, q, ldq, k, ldk, v, ldv, decay, ws, cu, S, H, d, dv, activation)
  if (vec && aligned) OUTPUTS(true, true);
  else if (vec) OUTPUTS(true, false);
  else if (aligned) OUTPUTS(false, true);
  else OUTPUTS(false, false);
#undef OUTPUTS
  RLIS_LAUNCH_CHECK("decay_attention_chunks (outputs)");
  return 0;
}
