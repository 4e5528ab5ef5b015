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
#define LAUNCH(TY, TW, TO)                                                                    \
  lanes_step_kernel<TY, TW, TO><<<R, 256, smem, stream>>>(                                    \
      src, src_stride, dst, dst_stride, (const TY*)y, y_parts, y_part_stride, round16, mix,   \
      back, read, (const TW*)norm_w, eps, (TO*)out, rows, H, S, store)
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

RLIS_API int rlis_head_gate(void* x, int dtype, long long x_stride, const void* gate,
                            long long gate_stride, int T, int nh, int D, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && D > 0, "head_gate: bad sizes");
  const long long total = (long long)T * nh * D;
  if (total == 0) return 0;
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

RLIS_API int rlis_gelu_erf(void* out, const void* x, int dtype, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
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
