// Several residual streams side by side (hyper-connections), and what a projected row of
// heads may need before attention reads it and after attention has written it.
//
//  * lanes_step: S float32 streams `lanes[s][t][:]`.  A sublayer reads u = sum_s a[s] lanes[s]
//    through a norm, and its result y comes back into all streams at once,
//    lanes'[t] = sum_s M[s][t] lanes[s] + b[t] y.  One kernel does the update that the sublayer
//    in front left behind and the read of the sublayer that follows, in one pass over the
//    streams: every sum is float32, added in the order of s.
//  * head_prepare: on the rows of a fused q/k/v product, in place: a bias per column, an RMS
//    norm over every query and key head with a weight per dim that all heads share, and a
//    factor on the queries that depends on the token's position.
//  * head_gate: every head of attention's result times the sigmoid of a number per head.
//  * gelu_erf: the erf form of GELU.
#include "common.h"

#include <math.h>

constexpr int kMaxLanes = 16;

// Grid: one workgroup of 256 per row.  `rows` (or null: every row) picks the tokens; with
// rows the streams are not written.  `y` null: nothing is mixed in.  `read` null: no read-out.
// `norm_w` null: the read-out is stored as it is (float32 or bfloat16 by TO).
template <typename TY, typename TW, typename TO>
__global__ __launch_bounds__(256) void lanes_step_kernel(
    const float* __restrict__ src, long long src_stride, float* __restrict__ dst,
    long long dst_stride, const TY* __restrict__ y, int y_parts, long long y_part_stride,
    int round16, const float* __restrict__ mix, const float* __restrict__ back,
    const float* __restrict__ read, const TW* __restrict__ norm_w, float eps,
    TO* __restrict__ out, const int* __restrict__ rows, int H, int S, int store) {
  extern __shared__ float u_s[];          // H
  __shared__ float red[4];
  __shared__ float coef[kMaxLanes * kMaxLanes + 2 * kMaxLanes];
  float* mix_s = coef;
  float* back_s = coef + kMaxLanes * kMaxLanes;
  float* read_s = back_s + kMaxLanes;
  const int r = blockIdx.x, tid = threadIdx.x;
  const long long t = rows ? rows[r] : r;
  for (int i = tid; i < S * S; i += 256) mix_s[i] = y ? mix[i] : 0.f;
  for (int i = tid; i < S; i += 256) {
    back_s[i] = y ? back[i] : 0.f;
    read_s[i] = read ? read[i] : 1.f;
  }
  __syncthreads();
  float ss = 0.f;
  for (int j = tid; j < H; j += 256) {
    float v[kMaxLanes];
#pragma unroll
    for (int s = 0; s < kMaxLanes; ++s)
      if (s < S) v[s] = src[s * src_stride + t * H + j];
    if (y) {
      const float yy = delta_sum(y + t * H + j, y_parts, y_part_stride, round16);
      float nv[kMaxLanes];
#pragma unroll
      for (int to = 0; to < kMaxLanes; ++to) {
        if (to < S) {
          float a = 0.f;
#pragma unroll
          for (int s = 0; s < kMaxLanes; ++s)
            if (s < S) a += mix_s[s * S + to] * v[s];
          nv[to] = a + back_s[to] * yy;
        }
      }
#pragma unroll
      for (int s = 0; s < kMaxLanes; ++s)
        if (s < S) {
          v[s] = nv[s];
          if (store) dst[s * dst_stride + t * H + j] = nv[s];
        }
    }
    if (out) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < kMaxLanes; ++s)
        if (s < S) u += read_s[s] * v[s];
      u_s[j] = u;
      ss += u * u;
    }
  }
  if (!out) return;
  float inv = 1.0f;
  if (norm_w) {
    const float total = block_sum<256>(ss, red);
    inv = 1.0f / sqrtf(total / (float)H + eps);
  } else {
    __syncthreads();
  }
  for (int j = tid; j < H; j += 256) {
    const float u = u_s[j];
    st(out + (long long)r * H + j, norm_w ? u * inv * widen(norm_w[j]) : u);
  }
}

// The same step for one to four streams whose rows are a multiple of four wide (what models
// have): the stream count is a constant of the kernel, so the sums over streams are straight
// code with every stream's load in flight at once, and a thread moves four columns at a time.
__device__ __forceinline__ void load4(const float* p, float* o) {
  const float4 v = *(const float4*)p;
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* o) {
  const uint2 v = *(const uint2*)p;
  o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
  o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float* v) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float* v) {
  uint2 o;
  o.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
  o.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
  *(uint2*)p = o;
}

template <int S, typename TY, typename TW, typename TO>
__global__ __launch_bounds__(256) void lanes_step4_kernel(
    const float* __restrict__ src, long long src_stride, float* __restrict__ dst,
    long long dst_stride, const TY* __restrict__ y, int y_parts, long long y_part_stride,
    int round16, const float* __restrict__ mix, const float* __restrict__ back,
    const float* __restrict__ read, const TW* __restrict__ norm_w, float eps,
    TO* __restrict__ out, const int* __restrict__ rows, int H, int store) {
  extern __shared__ float u_s[];          // H
  __shared__ float red[4];
  const int r = blockIdx.x, tid = threadIdx.x;
  const long long t = rows ? rows[r] : r;
  float m[S][S], b[S], a[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    b[s] = y ? back[s] : 0.f;
    a[s] = read ? read[s] : 1.f;
#pragma unroll
    for (int to = 0; to < S; ++to) m[s][to] = y ? mix[s * S + to] : 0.f;
  }
  float ss = 0.f;
  for (int j = tid * 4; j < H; j += 1024) {
    float v[S][4];
#pragma unroll
    for (int s = 0; s < S; ++s) load4(src + s * src_stride + t * H + j, v[s]);
    if (y) {
      float yy[4];
      load4(y + t * H + j, yy);
      // further parts four at a time, asked for together (one past the last reads the last
      // again and is dropped), added in their order
      for (int p = 1; p < y_parts; p += 4) {
        float more[4][4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          load4(y + (long long)min(p + q, y_parts - 1) * y_part_stride + t * H + j, more[q]);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (p + q < y_parts) {
#pragma unroll
            for (int e = 0; e < 4; ++e) yy[e] += more[q][e];
          }
      }
      if (round16) {
#pragma unroll
        for (int e = 0; e < 4; ++e) yy[e] = bf16_to_f32(f32_to_bf16(yy[e]));
      }
      float nv[S][4];
#pragma unroll
      for (int to = 0; to < S; ++to)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < S; ++s) acc += m[s][to] * v[s][e];
          nv[to][e] = acc + b[to] * yy[e];
        }
#pragma unroll
      for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[s][e] = nv[s][e];
        if (store) store4(dst + s * dst_stride + t * H + j, nv[s]);
      }
    }
    if (out) {
      float u[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) acc += a[s] * v[s][e];
        u[e] = acc;
        ss += acc * acc;
      }
      store4(u_s + j, u);
    }
  }
  if (!out) return;
  float inv = 1.0f;
  if (norm_w) inv = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)H + eps);
  // (a thread reads back the columns it wrote itself: no barrier is needed for them)
  for (int j = tid * 4; j < H; j += 1024) {
    float u[4], w[4];
    load4(u_s + j, u);
    if (norm_w) {
      load4(norm_w + j, w);
#pragma unroll
      for (int e = 0; e < 4; ++e) u[e] = u[e] * inv * w[e];
    }
    store4(out + (long long)r * H + j, u);
  }
}

RLIS_API int rlis_lanes_step(const float* src, long long src_stride, float* dst,
                             long long dst_stride, const void* y, int y_dtype, int y_parts,
                             long long y_part_stride, int round16, const float* mix,
                             const float* back, const float* read, const void* norm_w,
                             int w_dtype, float eps, void* out, int out_dtype, const int* rows,
                             int R, int H, int S, int store, hipStream_t stream) {
  RLIS_REQUIRE(R >= 0 && H > 0 && S >= 1 && S <= kMaxLanes, "lanes_step: bad sizes R=%d H=%d S=%d",
               R, H, S);
  RLIS_REQUIRE(H <= 16384, "lanes_step: rows of %d are above 16384", H);
  RLIS_REQUIRE(!y || (mix && back), "lanes_step: an update needs its coefficients");
  RLIS_REQUIRE(!(y && store) || dst, "lanes_step: an update that is kept needs a place");
  RLIS_REQUIRE(!(rows && store && y), "lanes_step: picked rows leave the streams as they are");
  if (R == 0) return 0;
  const size_t smem = (size_t)H * 4;
  const bool by4 = S <= 4 && H % 4 == 0 && ((uintptr_t)src % 16) == 0 &&
                   ((uintptr_t)dst % 16) == 0 && src_stride % 4 == 0 && dst_stride % 4 == 0 &&
                   ((uintptr_t)y % 16) == 0 && y_part_stride % 4 == 0 &&
                   ((uintptr_t)norm_w % 16) == 0 && ((uintptr_t)out % 16) == 0;
#define LAUNCH4(SC, TY, TW, TO)                                                               \
  lanes_step4_kernel<SC, TY, TW, TO><<<R, 256, smem, stream>>>(                               \
      src, src_stride, dst, dst_stride, (const TY*)y, y_parts, y_part_stride, round16, mix,   \
      back, read, (const TW*)norm_w, eps, (TO*)out, rows, H, store)
#define LAUNCH(TY, TW, TO)                                                                    \
  do {                                                                                        \
    if (by4 && S == 1) LAUNCH4(1, TY, TW, TO);                                                \
    else if (by4 && S == 2) LAUNCH4(2, TY, TW, TO);                                           \
    else if (by4 && S == 3) LAUNCH4(3, TY, TW, TO);                                           \
    else if (by4 && S == 4) LAUNCH4(4, TY, TW, TO);                                           \
    else                                                                                      \
      lanes_step_kernel<TY, TW, TO><<<R, 256, smem, stream>>>(                                \
          src, src_stride, dst, dst_stride, (const TY*)y, y_parts, y_part_stride, round16,    \
          mix, back, read, (const TW*)norm_w, eps, (TO*)out, rows, H, S, store);              \
  } while (0)
#define BY_OUT(TY, TW)                                     \
  do {                                                     \
    if (out_dtype == RLIS_BF16) LAUNCH(TY, TW, bf16_t);    \
    else LAUNCH(TY, TW, float);                            \
  } while (0)
#define BY_W(TY)                                           \
  do {                                                     \
    if (w_dtype == RLIS_BF16) BY_OUT(TY, bf16_t);          \
    else BY_OUT(TY, float);                                \
  } while (0)
  if (y_dtype == RLIS_BF16) BY_W(bf16_t); else BY_W(float);
#undef BY_W
#undef BY_OUT
#undef LAUNCH
#undef LAUNCH4
  RLIS_LAUNCH_CHECK("lanes_step");
  return 0;
}

// ------------------------------------------------------------------ head_prepare
// Grid (token, head of the row): one wave per head.  Heads 0 .. nh - 1 are queries, the next
// nkv keys, the next nkv values; every head is D wide, of which the first `dim` numbers are the
// head itself (the rest is padding: zero, and stays zero).  bias (or null): one float per column
// of the row.  q_w / k_w (or null): the norm's weight over a head's `dim` numbers.
// temp_every > 0: queries times 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1).
template <typename TX, int DPL>
__global__ __launch_bounds__(64) void head_prepare_kernel(
    TX* __restrict__ qkv, long long stride, int nh, int nkv, int D, int dim,
    const float* __restrict__ bias, const float* __restrict__ q_w, const float* __restrict__ k_w,
    float eps, const int* __restrict__ positions, float temp_coef, int temp_every) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < nh, is_v = h >= nh + nkv;
  const float* w = is_q ? q_w : (is_v ? nullptr : k_w);
  const bool scaled = is_q && temp_every > 0;
  if (!bias && !w && !scaled) return;
  TX* row = qkv + (long long)t * stride + (long long)h * D;
  float x[DPL];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int j = lane + 64 * i;
    x[i] = 0.f;
    if (j < D) {
      x[i] = ld(row + j) + (bias ? bias[(long long)h * D + j] : 0.f);
      if (j < dim) ss += x[i] * x[i];
    }
  }
  float f = 1.0f;
  if (w) f = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
  float g = 1.0f;
  if (scaled) g = 1.0f + temp_coef * logf((float)((positions[t] + 1) / temp_every) + 1.0f);
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int j = lane + 64 * i;
    if (j < D) {
      float v = x[i];
      if (w) v = j < dim ? v * f * w[j] : 0.f;
      st(row + j, v * g);
    }
  }
}

// bfloat16 rows in steps of 8: LPH lanes share a head, eight numbers each (16-byte accesses), so
// that a wave takes 64 / LPH heads at once; the sum of squares runs over the head's lanes.
// Whether there is a bias and a norm is known to the compiler, so that no load sits under a
// condition and all of a lane's loads are on their way before the first is used.
__device__ __forceinline__ void load8f_at(const float* p, float* o) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

template <int LPH, bool BIAS, bool NORM>
__global__ __launch_bounds__(256) void head_prepare_bf16x8_kernel(
    bf16_t* __restrict__ qkv, long long stride, int nh, int nkv, int D, int dim,
    const float* __restrict__ bias, const float* __restrict__ q_w, const float* __restrict__ k_w,
    float eps, const int* __restrict__ positions, float temp_coef, int temp_every,
    long long pairs) {
  // (32-bit arithmetic: the host sees to it that the pairs fit)
  const unsigned pair = (blockIdx.x * 256u + threadIdx.x) / LPH;
  const int sub = threadIdx.x % LPH;
  const unsigned heads = nh + 2 * nkv;
  // (lanes past the last pair, and lanes past the head's width, work on a place that is there
  // and drop the result: the shuffles below want every lane of the wave)
  const bool live = pair < pairs && sub * 8 < D;
  const int j0 = sub * 8 < D ? sub * 8 : 0;
  const unsigned pr = pair < pairs ? pair : (unsigned)pairs - 1;
  const int t = (int)(pr / heads), h = (int)(pr - (unsigned)t * heads);
  const bool is_q = h < nh, is_v = h >= nh + nkv;
  const bool normed = NORM && !is_v && (is_q || k_w != nullptr);
  const bool scaled = is_q && temp_every > 0;
  bf16_t* row = qkv + (long long)t * stride + (long long)h * D + j0;
  const uint4 raw = *(const uint4*)row;
  float bv[8], wv[8];
  if constexpr (BIAS) load8f_at(bias + (long long)h * D + j0, bv);
  if constexpr (NORM) load8f_at(((is_q || !k_w) ? q_w : k_w) + min(j0, dim - 8), wv);
  const int pos = temp_every > 0 ? positions[t] : 0;
  float x[8];
  const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = __uint_as_float(u[i] << 16);
    x[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if constexpr (BIAS) x[e] += bv[e];
    if (j0 + e < dim && live) ss += x[e] * x[e];
  }
  float f = 1.0f;
  if constexpr (NORM) {
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
    f = 1.0f / sqrtf(ss / (float)dim + eps);
  }
  const float g = scaled ? 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f) : 1.0f;
  if (!live || (!BIAS && !normed && !scaled)) return;
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float r[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      float v = x[2 * i + e];
      if constexpr (NORM) {
        if (normed) v = j0 + 2 * i + e < dim ? v * f * wv[2 * i + e] : 0.f;
      }
      r[e] = v * g;
    }
    o[i] = (uint32_t)f32_to_bf16(r[0]) | ((uint32_t)f32_to_bf16(r[1]) << 16);
  }
  *(uint4*)row = make_uint4(o[0], o[1], o[2], o[3]);
}

RLIS_API int rlis_head_prepare(void* qkv, int dtype, long long stride, int T, int nh, int nkv,
                               int D, int dim, const float* bias, const float* q_w,
                               const float* k_w, float eps, const int* positions,
                               float temp_coef, int temp_every, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && nkv >= 0 && D > 0 && dim > 0 && dim <= D,
               "head_prepare: bad sizes");
  RLIS_REQUIRE(D <= 512, "head_prepare: heads of %d are above 512", D);
  RLIS_REQUIRE(nh + 2 * nkv <= 65535, "head_prepare: too many heads");
  RLIS_REQUIRE(temp_every <= 0 || positions, "head_prepare: the queries' factor needs positions");
  if (T == 0) return 0;
  if (dtype == RLIS_BF16 && D % 8 == 0 && dim % 8 == 0 && stride % 8 == 0 &&
      ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)bias % 16) == 0 && ((uintptr_t)q_w % 16) == 0 &&
      ((uintptr_t)k_w % 16) == 0 && (q_w || !k_w)) {
    const long long pairs = (long long)T * (nh + 2 * nkv);
    int lph = 1;
    while (lph * 8 < D) lph *= 2;
    const long long blocks = ceil_div_ll(pairs * lph, 256);
    RLIS_REQUIRE(blocks * 256 < (1ll << 31), "head_prepare: too many rows");
#define LAUNCH8(LPH, BIAS, NORM)                                                             \
  head_prepare_bf16x8_kernel<LPH, BIAS, NORM><<<(unsigned)blocks, 256, 0, stream>>>(         \
      (bf16_t*)qkv, stride, nh, nkv, D, dim, bias, q_w, k_w, eps, positions, temp_coef,      \
      temp_every, pairs)
#define BY_FORM(LPH)                                          \
  do {                                                        \
    if (bias && q_w) LAUNCH8(LPH, true, true);                \
    else if (bias) LAUNCH8(LPH, true, false);                 \
    else if (q_w) LAUNCH8(LPH, false, true);                  \
    else LAUNCH8(LPH, false, false);                          \
  } while (0)
    if (lph <= 1) BY_FORM(1);
    else if (lph == 2) BY_FORM(2);
    else if (lph == 4) BY_FORM(4);
    else if (lph == 8) BY_FORM(8);
    else if (lph == 16) BY_FORM(16);
    else if (lph == 32) BY_FORM(32);
    else BY_FORM(64);
#undef BY_FORM
#undef LAUNCH8
    RLIS_LAUNCH_CHECK("head_prepare");
    return 0;
  }
  dim3 grid(T, nh + 2 * nkv);
  const int dpl = ceil_div(D, 64);
#define LAUNCH(TX, DPL)                                                                     \
  head_prepare_kernel<TX, DPL><<<grid, 64, 0, stream>>>((TX*)qkv, stride, nh, nkv, D, dim,  \
                                                        bias, q_w, k_w, eps, positions,     \
                                                        temp_coef, temp_every)
#define BY_DPL(TX)                       \
  do {                                   \
    if (dpl <= 1) LAUNCH(TX, 1);         \
    else if (dpl <= 2) LAUNCH(TX, 2);    \
    else if (dpl <= 4) LAUNCH(TX, 4);    \
    else LAUNCH(TX, 8);                  \
  } while (0)
  if (dtype == RLIS_F32) BY_DPL(float);
  else if (dtype == RLIS_BF16) BY_DPL(bf16_t);
  else RLIS_REQUIRE(false, "head_prepare: unknown dtype %d", dtype);
#undef BY_DPL
#undef LAUNCH
  RLIS_LAUNCH_CHECK("head_prepare");
  return 0;
}

// --------------------------------------------------------------------- head_gate
// x[t][h][:] *= 1 / (1 + exp(-gate[t][h])), float32 arithmetic, in place.
template <typename TX>
__global__ void head_gate_kernel(TX* __restrict__ x, long long x_stride,
                                 const TX* __restrict__ gate, long long gate_stride, int nh,
                                 int D, long long total) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long step = (long long)gridDim.x * blockDim.x;
  const int width = nh * D;
  for (; i < total; i += step) {
    const long long t = i / width;
    const int c = (int)(i % width);
    const float g = ld(gate + t * gate_stride + c / D);
    TX* p = x + t * x_stride + c;
    st(p, ld(p) / (1.0f + expf(-g)));
  }
}

// bfloat16 heads in steps of 8: eight numbers a thread, all of one head.
__global__ void head_gate_bf16x8_kernel(bf16_t* __restrict__ x, long long x_stride,
                                        const bf16_t* __restrict__ gate, long long gate_stride,
                                        int nh, int D, long long total8) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long step = (long long)gridDim.x * blockDim.x;
  const unsigned width8 = nh * D / 8;
  for (; i < total8; i += step) {
    // (the host keeps total8 below 2^31: 32-bit division)
    const unsigned t = (unsigned)i / width8;
    const int c = (int)((unsigned)i - t * width8) * 8;
    const float g = 1.0f / (1.0f + expf(-bf16_to_f32(gate[(long long)t * gate_stride + c / D])));
    bf16_t* p = x + (long long)t * x_stride + c;
    const uint4 v = *(const uint4*)p;
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      o[k] = (uint32_t)f32_to_bf16(__uint_as_float(u[k] << 16) * g) |
             ((uint32_t)f32_to_bf16(__uint_as_float(u[k] & 0xffff0000u) * g) << 16);
    *(uint4*)p = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

RLIS_API int rlis_head_gate(void* x, int dtype, long long x_stride, const void* gate,
                            long long gate_stride, int T, int nh, int D, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && D > 0, "head_gate: bad sizes");
  const long long total = (long long)T * nh * D;
  if (total == 0) return 0;
  if (dtype == RLIS_BF16 && D % 8 == 0 && x_stride % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
      total / 8 < (1ll << 31)) {
    const long long total8 = total / 8;
    const int blocks8 = (int)(ceil_div_ll(total8, 256) < 16384 ? ceil_div_ll(total8, 256) : 16384);
    head_gate_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)x, x_stride, (const bf16_t*)gate,
                                                        gate_stride, nh, D, total8);
    RLIS_LAUNCH_CHECK("head_gate");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(total, 256) < 16384 ? ceil_div_ll(total, 256) : 16384);
  if (dtype == RLIS_F32)
    head_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, x_stride, (const float*)gate,
                                                        gate_stride, nh, D, total);
  else if (dtype == RLIS_BF16)
    head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, x_stride,
                                                         (const bf16_t*)gate, gate_stride, nh, D,
                                                         total);
  else
    RLIS_REQUIRE(false, "head_gate: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("head_gate");
  return 0;
}

// ---------------------------------------------------------------------- gelu_erf
// y = 0.5 x (1 + erf(x / sqrt 2)), float32 arithmetic, one rounding.
template <typename TX>
__global__ void gelu_erf_kernel(TX* __restrict__ out, const TX* __restrict__ x, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const float v = ld(x + i);
    st(out + i, 0.5f * v * (1.0f + erff(v * 0.7071067811865476f)));
  }
}

// bfloat16, eight values a thread (16-byte accesses).  erf by the rational form
// 1 - (a1 t + ... + a5 t^5) exp(-z^2), t = 1 / (1 + p |z|), whose error stays below 2e-7 (a
// thousandth of a bfloat16's last digit), with the hardware's exponential and reciprocal: the
// library's erff costs more instructions than this kernel has time for per value.
__device__ __forceinline__ float gelu_erf_fast(float v) {
  const float z = fabsf(v) * 0.7071067811865476f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
  float poly = fmaf(1.061405429f, t, -1.453152027f);
  poly = fmaf(poly, t, 1.421413741f);
  poly = fmaf(poly, t, -0.284496736f);
  poly = fmaf(poly, t, 0.254829592f);
  const float tail = poly * t * __builtin_amdgcn_exp2f(-z * z * 1.4426950408889634f);
  const float erf_abs = 1.0f - tail;
  return 0.5f * v * (1.0f + (v < 0.f ? -erf_abs : erf_abs));
}

__global__ void gelu_erf_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x,
                                       long long n8) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n8; i += stride) {
    const uint4 v = *(const uint4*)(x + i * 8);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = gelu_erf_fast(__uint_as_float(w[j] << 16));
      const float hi = gelu_erf_fast(__uint_as_float(w[j] & 0xffff0000u));
      o[j] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
    }
    *(uint4*)(out + i * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

RLIS_API int rlis_gelu_erf(void* out, const void* x, int dtype, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  if (dtype == RLIS_BF16 && n % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)x % 16) == 0) {
    const long long n8 = n / 8;
    const int blocks8 = (int)(ceil_div_ll(n8, 256) < 16384 ? ceil_div_ll(n8, 256) : 16384);
    gelu_erf_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, n8);
    RLIS_LAUNCH_CHECK("gelu_erf");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(n, 256) < 16384 ? ceil_div_ll(n, 256) : 16384);
  if (dtype == RLIS_F32)
    gelu_erf_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)x, n);
  else if (dtype == RLIS_BF16)
    gelu_erf_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, n);
  else
    RLIS_REQUIRE(false, "gelu_erf: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("gelu_erf");
  return 0;
}
