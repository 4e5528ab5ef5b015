// Row-wise and element-wise kernels of the decoder step: embedding gather, residual add fused
// with RMSNorm, SwiGLU, rotary position encoding fused with the write of K and V into cache
// pages, and page copies.  All arithmetic is float32; storage is float32 or bfloat16.
//
// Formulas follow the reference: RMSNorm y = x * rsqrt(mean(x^2) + eps) * w
// (crates/model/src/layers.rs:141-146), SwiGLU silu(gate) * up (layers.rs:179-186), rotate-half
// rotation with per-position cos/sin rows (crates/model/src/rope.rs:111-117), K and V written
// at slot = table[pos / page] * page + pos % page before attention reads them
// (crates/model/src/paged.rs:258-263, 324-337).
#include "common.h"

static thread_local char g_err[512] = "";

void rlis_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

RLIS_API const char* rlis_last_error() { return g_err; }

// ------------------------------------------------------------------------ embedding
// out[t] = table[ids[t]] * scale (+ learned[positions[t]] when a table of learned position
// vectors is given: added as it is, in float32).
template <typename TW>
__global__ void embed_kernel(float* __restrict__ out, const TW* __restrict__ table,
                             const int* __restrict__ ids, int H, float scale,
                             const TW* __restrict__ learned, const int* __restrict__ positions) {
  const int t = blockIdx.x;
  const long long row = ids[t];
  const TW* src = table + row * H;
  float* dst = out + (long long)t * H;
  if (learned) {
    const TW* add = learned + (long long)positions[t] * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = ld(src + j) * scale + ld(add + j);
  } else {
    for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = ld(src + j) * scale;
  }
}

// out (T,H) f32 <- table[ids] * scale (+ learned[positions]); ids and positions are checked
// against the tables' rows on the host before the call.
RLIS_API int rlis_embed(float* out, const void* table, int table_dtype, const int* ids, int T,
                        int H, float scale, const void* learned, const int* positions,
                        hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && H > 0, "embed: bad sizes T=%d H=%d", T, H);
  RLIS_REQUIRE(!learned || positions, "embed: learned position vectors need positions");
  if (T == 0) return 0;
  if (table_dtype == RLIS_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(out, (const float*)table, ids, H, scale,
                                               (const float*)learned, positions);
  else if (table_dtype == RLIS_BF16)
    embed_kernel<bf16_t><<<T, 256, 0, stream>>>(out, (const bf16_t*)table, ids, H, scale,
                                                (const bf16_t*)learned, positions);
  else
    RLIS_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
  RLIS_LAUNCH_CHECK("embed");
  return 0;
}

// ------------------------------------------------------------------- residual add
// delta may come as `parts` partial sums of n elements each, one after the other; they are
// added in order (and their sum rounded to bfloat16 first when round_parts is set).
template <typename TD>
__global__ void add_residual_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                    long long n, int parts, int round_parts,
                                    float delta_scale) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    resid[i] += delta_scale * delta_sum(delta + i, parts, n, round_parts);
  }
}

// resid += delta_scale * delta (the multiplier of a block's output, in float32).
RLIS_API int rlis_add_residual(float* resid, const void* delta, int delta_dtype, long long n,
                               int parts, int round_parts, float delta_scale,
                               hipStream_t stream) {
  RLIS_REQUIRE(parts >= 1, "add_residual: parts=%d", parts);
  if (n <= 0) return 0;
  const int blocks = (int)(ceil_div_ll(n, 256) < 4096 ? ceil_div_ll(n, 256) : 4096);
  if (delta_dtype == RLIS_F32)
    add_residual_kernel<float><<<blocks, 256, 0, stream>>>(resid, (const float*)delta, n, parts,
                                                           round_parts, delta_scale);
  else if (delta_dtype == RLIS_BF16)
    add_residual_kernel<bf16_t><<<blocks, 256, 0, stream>>>(resid, (const bf16_t*)delta, n, parts,
                                                            round_parts, delta_scale);
  else
    RLIS_REQUIRE(false, "add_residual: unknown dtype %d", delta_dtype);
  RLIS_LAUNCH_CHECK("add_residual");
  return 0;
}

// ------------------------------------------------------- residual add + RMSNorm
// One block per output row r; the source row is rows[r] when rows is given.  The residual is
// float32; delta (may be null) is added first and, when write_resid is set, the sum is stored
// back.  delta may come as `parts` partial sums, part_stride elements apart, added in order
// (their sum rounded to bfloat16 first when round_parts is set).
// Sum of squares, rsqrt and both multiplies are float32; one rounding at the store.
template <typename TD, typename TW, typename TO, int NT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   const TW* __restrict__ weight, TO* __restrict__ out,
                                   const int* __restrict__ rows, int H, float eps,
                                   int write_resid, int parts, long long part_stride,
                                   int round_parts, float delta_scale) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const TD* d = delta ? delta + src * H : nullptr;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += NT) {
    float v = x[j];
    if (d) {
      v += delta_scale * delta_sum(d + j, parts, part_stride, round_parts);
      if (write_resid) x[j] = v;
    }
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
  const bool reread_sum = d && !write_resid;
  for (int j = threadIdx.x; j < H; j += NT) {
    float v = x[j];
    if (reread_sum) v += delta_scale * delta_sum(d + j, parts, part_stride, round_parts);
    st(o + j, v * inv * ld(weight + j));
  }
}

// The same for rows of at most NT * VPT elements, which stay in registers between the sum
// of squares and the store: one read of every input, no second pass.
template <typename TD, typename TW, typename TO, int NT, int VPT>
__global__ __launch_bounds__(NT) void add_rmsnorm_small_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid,
    int parts, long long part_stride, int round_parts, float delta_scale) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const TD* d = delta ? delta + src * H : nullptr;
  float v[VPT], w[VPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int j = threadIdx.x + i * NT;
    v[i] = 0.f;
    w[i] = 0.f;
    if (j < H) {
      v[i] = x[j];
      if (d) v[i] += delta_scale * delta_sum(d + j, parts, part_stride, round_parts);
      w[i] = ld(weight + j);
    }
    ss += v[i] * v[i];
  }
  if (d && write_resid) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int j = threadIdx.x + i * NT;
      if (j < H) x[j] = v[i];
    }
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int j = threadIdx.x + i * NT;
    if (j < H) st(o + j, v[i] * inv * w[i]);
  }
}

// The all-bfloat16 case with rows of a multiple of 8 and at most 256 * 8 * CH elements: eight
// elements per thread and chunk, 16- and 32-byte accesses.
template <int CH>
__global__ __launch_bounds__(256) void add_rmsnorm_bf16x8_kernel(
    float* __restrict__ resid, const bf16_t* __restrict__ delta, const bf16_t* __restrict__ weight,
    bf16_t* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid) {
  __shared__ float red[256 / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const bf16_t* d = delta ? delta + src * H : nullptr;
  float v[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * 256) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[ch][e] = 0.f;
    if (j < H) {
      const float4 a = *(const float4*)(x + j), b = *(const float4*)(x + j + 4);
      v[ch][0] = a.x; v[ch][1] = a.y; v[ch][2] = a.z; v[ch][3] = a.w;
      v[ch][4] = b.x; v[ch][5] = b.y; v[ch][6] = b.z; v[ch][7] = b.w;
      if (d) {
        const uint4 dv = *(const uint4*)(d + j);
        const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[ch][2 * e] += __uint_as_float(dw[e] << 16);
          v[ch][2 * e + 1] += __uint_as_float(dw[e] & 0xffff0000u);
        }
        if (write_resid) {
          *(float4*)(x + j) = make_float4(v[ch][0], v[ch][1], v[ch][2], v[ch][3]);
          *(float4*)(x + j + 4) = make_float4(v[ch][4], v[ch][5], v[ch][6], v[ch][7]);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[ch][e] * v[ch][e];
    }
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  bf16_t* o = out + (long long)r * H;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * 256) * 8;
    if (j < H) {
      const uint4 wv = *(const uint4*)(weight + j);
      const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
      uint32_t ow[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float r0 = v[ch][2 * e] * inv * __uint_as_float(ww[e] << 16);
        const float r1 = v[ch][2 * e + 1] * inv * __uint_as_float(ww[e] & 0xffff0000u);
        ow[e] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
      }
      *(uint4*)(o + j) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
}

// True when the vectorised kernel took the call.
static bool launch_add_rmsnorm_bf16x8(float* resid, const void* delta, const void* weight, void* out,
                                      const int* rows, int R, int H, float eps, int write_resid,
                                      int parts, hipStream_t stream) {
  if (H % 8 != 0 || H > 256 * 8 * 4 || parts != 1) return false;
  if (((uintptr_t)resid | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out) % 16) return false;
#define LAUNCH(CH)                                                                               \
  add_rmsnorm_bf16x8_kernel<CH><<<R, 256, 0, stream>>>(resid, (const bf16_t*)delta,              \
                                                       (const bf16_t*)weight, (bf16_t*)out, rows, \
                                                       H, eps, write_resid)
  if (H <= 256 * 8) LAUNCH(1);
  else if (H <= 256 * 16) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
  return true;
}

// The delta as a stack of float32 partial sums (what the split-k and the streaming products
// leave for their consumer), rows of a multiple of 4 and at most NT * 4 * CH elements: four
// elements per thread and chunk, 16-byte accesses.  Such stacks come with few rows (64 at most)
// and up to dozens of parts, so a row gets a wide workgroup (NT threads, as many as the row has
// groups of four, up to 1024) and every thread keeps eight parts of its chunk in flight (four
// of each where it has several chunks); the parts are added in order and their sum rounded to
// bfloat16 when round_parts is set.
template <typename TW, typename TO, int CH, int NT>
__global__ __launch_bounds__(NT) void add_rmsnorm_stack_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid,
    int parts, long long part_stride, int round_parts) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const float* d = delta + src * H;
  // A chunk past the row reads the row's first elements instead (and stores nothing).
  int col[CH];
  bool live[CH];
  float4 xr[CH], s[CH];
  // The norm's weight is asked for with the first loads, long before it is needed.
  TW wt[CH][4];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * NT) * 4;
    live[ch] = j < H;
    col[ch] = live[ch] ? j : 0;
    xr[ch] = *(const float4*)(x + col[ch]);
#pragma unroll
    for (int e = 0; e < 4; ++e) wt[ch][e] = weight[col[ch] + e];
  }
  // The parts in batches of AHEAD, every batch's loads issued together and none under a
  // condition (a part past the last reads the last again and adds nothing): a stack of eight
  // parts is one trip to memory, and no part waits for the one before it.  They are added in
  // order, the first one as it is.
  constexpr int AHEAD = CH == 1 ? 8 : 4;
  for (int p = 0; p < parts; p += AHEAD) {
    float4 a[CH][AHEAD];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
#pragma unroll
      for (int q = 0; q < AHEAD; ++q)
        a[ch][q] = *(const float4*)(d + (long long)min(p + q, parts - 1) * part_stride + col[ch]);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
#pragma unroll
      for (int q = 0; q < AHEAD; ++q) {
        if (p == 0 && q == 0) {
          s[ch] = a[ch][0];
        } else if (p + q < parts) {
          s[ch].x += a[ch][q].x; s[ch].y += a[ch][q].y; s[ch].z += a[ch][q].z; s[ch].w += a[ch][q].w;
        }
      }
  }
  float v[CH][4];
  float ss = 0.f;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (round_parts) {
      s[ch].x = bf16_to_f32(f32_to_bf16(s[ch].x)); s[ch].y = bf16_to_f32(f32_to_bf16(s[ch].y));
      s[ch].z = bf16_to_f32(f32_to_bf16(s[ch].z)); s[ch].w = bf16_to_f32(f32_to_bf16(s[ch].w));
    }
    v[ch][0] = xr[ch].x + s[ch].x; v[ch][1] = xr[ch].y + s[ch].y;
    v[ch][2] = xr[ch].z + s[ch].z; v[ch][3] = xr[ch].w + s[ch].w;
    if (live[ch]) {
      if (write_resid)
        *(float4*)(x + col[ch]) = make_float4(v[ch][0], v[ch][1], v[ch][2], v[ch][3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += v[ch][e] * v[ch][e];
    }
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (live[ch]) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        st(o + col[ch] + e, v[ch][e] * inv * widen(wt[ch][e]));
    }
  }
}

// True when the kernel for stacks of float32 partial sums took the call.
template <typename TW, typename TO>
static bool launch_add_rmsnorm_stack(float* resid, const void* delta, const void* weight,
                                     void* out, const int* rows, int R, int H, float eps,
                                     int write_resid, int parts, long long part_stride,
                                     int round_parts, hipStream_t stream) {
  if (H % 4 != 0 || H > 1024 * 4 * 4 || part_stride % 4 != 0) return false;
  if (((uintptr_t)resid | (uintptr_t)delta) % 16) return false;
#define LAUNCH(CH, NT)                                                                        \
  add_rmsnorm_stack_kernel<TW, TO, CH, NT><<<R, NT, 0, stream>>>(                             \
      resid, (const float*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid,     \
      parts, part_stride, round_parts)
  if (H <= 256 * 4) LAUNCH(1, 256);
  else if (H <= 512 * 4) LAUNCH(1, 512);
  else if (H <= 1024 * 4) LAUNCH(1, 1024);
  else if (H <= 1024 * 8) LAUNCH(2, 1024);
  else LAUNCH(4, 1024);
#undef LAUNCH
  return true;
}

template <typename TD, typename TW, typename TO>
static void launch_add_rmsnorm(float* resid, const void* delta, const void* weight, void* out,
                               const int* rows, int R, int H, float eps, int write_resid,
                               int parts, long long part_stride, int round_parts,
                               float delta_scale, hipStream_t stream) {
  if (H <= 256 * 4)
    add_rmsnorm_small_kernel<TD, TW, TO, 256, 4><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts, delta_scale);
  else if (H <= 256 * 16)
    add_rmsnorm_small_kernel<TD, TW, TO, 256, 16><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts, delta_scale);
  else
    add_rmsnorm_kernel<TD, TW, TO, 256><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts, delta_scale);
}

RLIS_API int rlis_add_rmsnorm(float* resid, const void* delta, int delta_dtype,
                              const void* weight, int weight_dtype, void* out, int out_dtype,
                              const int* rows, int R, int H, float eps, int write_resid,
                              int parts, long long part_stride, int round_parts,
                              float delta_scale, hipStream_t stream) {
  RLIS_REQUIRE(R >= 0 && H > 0, "add_rmsnorm: bad sizes R=%d H=%d", R, H);
  RLIS_REQUIRE(parts >= 1, "add_rmsnorm: parts=%d", parts);
  RLIS_REQUIRE(!(rows && write_resid && delta),
               "add_rmsnorm: writing the residual back needs all rows, not a selection");
  if (R == 0) return 0;
  // (the forms below for special layouts add the delta as it is; a delta that comes with a
  // multiplier takes the general kernels)
  const bool plain_delta = !delta || delta_scale == 1.0f;
  if (plain_delta && (!delta || delta_dtype == RLIS_BF16) && weight_dtype == RLIS_BF16 &&
      out_dtype == RLIS_BF16 &&
      launch_add_rmsnorm_bf16x8(resid, delta, weight, out, rows, R, H, eps, write_resid, parts,
                                stream)) {
    RLIS_LAUNCH_CHECK("add_rmsnorm");
    return 0;
  }
  if (plain_delta && delta && delta_dtype == RLIS_F32 && parts > 1) {
    bool took = false;
    if (weight_dtype == RLIS_BF16 && out_dtype == RLIS_BF16)
      took = launch_add_rmsnorm_stack<bf16_t, bf16_t>(resid, delta, weight, out, rows, R, H, eps,
                                                      write_resid, parts, part_stride, round_parts,
                                                      stream);
    else if (weight_dtype == RLIS_F32 && out_dtype == RLIS_BF16)
      took = launch_add_rmsnorm_stack<float, bf16_t>(resid, delta, weight, out, rows, R, H, eps,
                                                     write_resid, parts, part_stride, round_parts,
                                                     stream);
    else if (weight_dtype == RLIS_F32 && out_dtype == RLIS_F32)
      took = launch_add_rmsnorm_stack<float, float>(resid, delta, weight, out, rows, R, H, eps,
                                                    write_resid, parts, part_stride, round_parts,
                                                    stream);
    if (took) {
      RLIS_LAUNCH_CHECK("add_rmsnorm");
      return 0;
    }
  }
  const int key = (delta ? delta_dtype : out_dtype) * 4 + weight_dtype * 2 + out_dtype;
#define CASE(k, TD, TW, TO)                                                                  \
  case k:                                                                                    \
    launch_add_rmsnorm<TD, TW, TO>(resid, delta, weight, out, rows, R, H, eps, write_resid,  \
                                   parts, part_stride, round_parts, delta_scale, stream);    \
    break;
  switch (key) {
    CASE(0, float, float, float)
    CASE(1, float, float, bf16_t)
    CASE(2, float, bf16_t, float)
    CASE(3, float, bf16_t, bf16_t)
    CASE(4, bf16_t, float, float)
    CASE(5, bf16_t, float, bf16_t)
    CASE(6, bf16_t, bf16_t, float)
    CASE(7, bf16_t, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "add_rmsnorm: unknown dtypes %d %d %d", delta_dtype, weight_dtype,
                   out_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// -------------------------------------------------------------------------- SwiGLU
// gu (T, 2I): columns [0, I) are the gate projection, [I, 2I) the up projection.
template <typename TX>
__global__ void swiglu_kernel(TX* __restrict__ out, const TX* __restrict__ gu, int I,
                              long long total) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const long long t = i / I;
    const int c = (int)(i - t * I);
    const float g = ld(gu + t * 2 * I + c);
    const float u = ld(gu + t * 2 * I + I + c);
    const float s = g / (1.0f + expf(-g));
    st(out + i, s * u);
  }
}

// bfloat16 rows whose width is a multiple of 8: eight columns per thread, 16-byte accesses.
__global__ void swiglu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu,
                                     int I8 /* I / 8 */, long long total8) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total8; i += stride) {
    const long long t = i / I8;
    const int c = (int)(i - t * I8);
    const uint4 gv = *(const uint4*)(gu + (t * 2 * I8 + c) * 8);
    const uint4 uv = *(const uint4*)(gu + (t * 2 * I8 + I8 + c) * 8);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
      // silu(g) * u with the hardware's exponential and reciprocal (an ulp each, far inside
      // what the rounding to bfloat16 leaves): the library functions made this kernel spend as
      // long on arithmetic as on its bytes.
      const float e0 = __builtin_amdgcn_exp2f(g0 * -1.4426950408889634f);
      const float e1 = __builtin_amdgcn_exp2f(g1 * -1.4426950408889634f);
      const float r0 = g0 * __builtin_amdgcn_rcpf(1.0f + e0) * u0;
      const float r1 = g1 * __builtin_amdgcn_rcpf(1.0f + e1) * u1;
      ow[j] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
    }
    *(uint4*)(out + i * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

RLIS_API int rlis_swiglu(void* out, const void* gu, int dtype, int T, int I, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  const long long total = (long long)T * I;
  if (total == 0) return 0;
  if (dtype == RLIS_BF16 && I % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gu % 16) == 0) {
    const long long total8 = total / 8;
    const int blocks8 = (int)(ceil_div_ll(total8, 256) < 16384 ? ceil_div_ll(total8, 256) : 16384);
    swiglu_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I / 8, total8);
    RLIS_LAUNCH_CHECK("swiglu");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(total, 256) < 8192 ? ceil_div_ll(total, 256) : 8192);
  if (dtype == RLIS_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, I, total);
  else if (dtype == RLIS_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I, total);
  else
    RLIS_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("swiglu");
  return 0;
}

// ------------------------------------------------------------- clamped gated unit
// gu (T, 2I) as above.  g = min(gate, limit), u = clamp(up, -limit, limit),
// y = g * sigmoid(alpha * g) * (u + 1): a gated unit whose two branches are bounded before
// they meet.  float32 arithmetic, one rounding at the store.
template <typename TX>
__global__ void clamped_glu_kernel(TX* __restrict__ out, const TX* __restrict__ gu, int I,
                                   long long total, float limit, float alpha) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const long long t = i / I;
    const int c = (int)(i - t * I);
    const float g = fminf(ld(gu + t * 2 * I + c), limit);
    const float u = fminf(fmaxf(ld(gu + t * 2 * I + I + c), -limit), limit);
    st(out + i, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

// bfloat16 rows whose width is a multiple of 8: eight columns per thread, 16-byte accesses, the
// hardware's exponential and reciprocal (as the SwiGLU kernel above).
__global__ void clamped_glu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu,
                                          int I8 /* I / 8 */, long long total8, float limit,
                                          float neg_alpha_log2e) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total8; i += stride) {
    const long long t = i / I8;
    const int c = (int)(i - t * I8);
    const uint4 gv = *(const uint4*)(gu + (t * 2 * I8 + c) * 8);
    const uint4 uv = *(const uint4*)(gu + (t * 2 * I8 + I8 + c) * 8);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g0 = fminf(__uint_as_float(gw[j] << 16), limit);
      const float g1 = fminf(__uint_as_float(gw[j] & 0xffff0000u), limit);
      const float u0 = fminf(fmaxf(__uint_as_float(uw[j] << 16), -limit), limit);
      const float u1 = fminf(fmaxf(__uint_as_float(uw[j] & 0xffff0000u), -limit), limit);
      const float e0 = __builtin_amdgcn_exp2f(g0 * neg_alpha_log2e);
      const float e1 = __builtin_amdgcn_exp2f(g1 * neg_alpha_log2e);
      const float r0 = g0 * __builtin_amdgcn_rcpf(1.0f + e0) * (u0 + 1.0f);
      const float r1 = g1 * __builtin_amdgcn_rcpf(1.0f + e1) * (u1 + 1.0f);
      ow[j] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
    }
    *(uint4*)(out + i * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

RLIS_API int rlis_clamped_glu(void* out, const void* gu, int dtype, int T, int I, float limit,
                              float alpha, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && I > 0, "clamped_glu: bad sizes T=%d I=%d", T, I);
  const long long total = (long long)T * I;
  if (total == 0) return 0;
  if (dtype == RLIS_BF16 && I % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gu % 16) == 0) {
    const long long total8 = total / 8;
    const int blocks8 = (int)(ceil_div_ll(total8, 256) < 16384 ? ceil_div_ll(total8, 256) : 16384);
    clamped_glu_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I / 8,
                                                          total8, limit,
                                                          -alpha * 1.4426950408889634f);
    RLIS_LAUNCH_CHECK("clamped_glu");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(total, 256) < 8192 ? ceil_div_ll(total, 256) : 8192);
  if (dtype == RLIS_F32)
    clamped_glu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, I, total,
                                                          limit, alpha);
  else if (dtype == RLIS_BF16)
    clamped_glu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I,
                                                           total, limit, alpha);
  else
    RLIS_REQUIRE(false, "clamped_glu: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("clamped_glu");
  return 0;
}

// ------------------------------------------------------------- weighted sum of two
// out (float32) = a * x + b * y, element by element: two branches that read the same input
// meet here on their way into the residual stream.  Either operand may come as a stack of
// float32 partial sums, n elements apart, which are added in order first (and, with round16,
// rounded to bfloat16 as a result that arrives whole in bfloat16 was); y may be absent.
template <typename TX, typename TY>
__global__ void weighted_sum_kernel(float* __restrict__ out, const TX* __restrict__ x, float a,
                                    int x_parts, const TY* __restrict__ y, float b, int y_parts,
                                    long long n, int round16) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = a * delta_sum(x + i, x_parts, n, round16 && x_parts > 1);
    if (y) v += b * delta_sum(y + i, y_parts, n, round16 && y_parts > 1);
    out[i] = v;
  }
}

RLIS_API int rlis_weighted_sum(float* out, const void* x, int x_dtype, float a, int x_parts,
                               const void* y, int y_dtype, float b, int y_parts, long long n,
                               int round16, hipStream_t stream) {
  RLIS_REQUIRE(x && x_parts >= 1 && (!y || y_parts >= 1), "weighted_sum: bad operands");
  RLIS_REQUIRE((x_parts == 1 || x_dtype == RLIS_F32) && (!y || y_parts == 1 || y_dtype == RLIS_F32),
               "weighted_sum: partial sums are float32");
  if (n <= 0) return 0;
  const int blocks = (int)(ceil_div_ll(n, 256) < 8192 ? ceil_div_ll(n, 256) : 8192);
  const int key = x_dtype * 2 + (y ? y_dtype : 0);
#define CASE(k, TX, TY)                                                                        \
  case k:                                                                                      \
    weighted_sum_kernel<TX, TY><<<blocks, 256, 0, stream>>>(out, (const TX*)x, a, x_parts,     \
                                                            (const TY*)y, b, y_parts, n, round16); \
    break;
  switch (key) {
    CASE(0, float, float)
    CASE(1, float, bf16_t)
    CASE(2, bf16_t, float)
    CASE(3, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "weighted_sum: unknown dtypes %d %d", x_dtype, y_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("weighted_sum");
  return 0;
}

// ------------------------------------------------------------- tanh form of GELU
// y = 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))), float32 arithmetic, one rounding.
__device__ __forceinline__ float gelu_tanh_f(float x) {
  const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(inner));
}

template <typename TX>
__global__ void gelu_tanh_kernel(TX* __restrict__ out, const TX* __restrict__ x, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) st(out + i, gelu_tanh_f(ld(x + i)));
}

// bfloat16, eight values a thread (16-byte accesses); tanh(z) = 1 - 2 / (exp(2 z) + 1) with the
// hardware's exponential and reciprocal.
__global__ void gelu_tanh_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x,
                                        long long n8) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n8; i += stride) {
    const uint4 v = *(const uint4*)(x + i * 8);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float r[2];
      const float a[2] = {__uint_as_float(w[j] << 16), __uint_as_float(w[j] & 0xffff0000u)};
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float z = 0.7978845608028654f * (a[e] + 0.044715f * a[e] * a[e] * a[e]);
        // 0.5 (1 + tanh z) = 1 / (1 + exp(-2 z))
        const float ex = __builtin_amdgcn_exp2f(-2.0f * 1.4426950408889634f * z);
        r[e] = a[e] * __builtin_amdgcn_rcpf(1.0f + ex);
      }
      o[j] = (uint32_t)f32_to_bf16(r[0]) | ((uint32_t)f32_to_bf16(r[1]) << 16);
    }
    *(uint4*)(out + i * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

RLIS_API int rlis_gelu_tanh(void* out, const void* x, int dtype, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  if (dtype == RLIS_BF16 && n % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)x % 16) == 0) {
    const long long n8 = n / 8;
    const int blocks8 = (int)(ceil_div_ll(n8, 256) < 16384 ? ceil_div_ll(n8, 256) : 16384);
    gelu_tanh_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, n8);
    RLIS_LAUNCH_CHECK("gelu_tanh");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(n, 256) < 8192 ? ceil_div_ll(n, 256) : 8192);
  if (dtype == RLIS_F32)
    gelu_tanh_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)x, n);
  else if (dtype == RLIS_BF16)
    gelu_tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, n);
  else
    RLIS_REQUIRE(false, "gelu_tanh: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("gelu_tanh");
  return 0;
}

// ------------------------------------------------- a learned mix of the layers' results
// The stream that the next layer reads is a weighted sum of the embedding output and of every
// layer's result so far.  `hist` holds them, one (T, W) float32 slab per source, `n` elements
// apart.  This layer's result y = x + delta becomes source `count - 1`; x then becomes
// sum_j weights[j] * source j over the `count` sources, added in order, all in float32.  With
// save_input, x itself is stored as source 0 first (the first layer: its input is the embedding
// output as it is).
template <typename TW>
__global__ void depth_mix_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                 float* __restrict__ hist, long long n, int count,
                                 const TW* __restrict__ weights, int save_input) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const float in = x[i];
    const float y = in + delta[i];
    if (save_input) hist[i] = in;
    hist[(long long)(count - 1) * n + i] = y;
    float acc = ld(weights) * (save_input ? in : hist[i]);
    for (int j = 1; j < count - 1; ++j) acc += ld(weights + j) * hist[(long long)j * n + i];
    acc += ld(weights + count - 1) * y;
    x[i] = acc;
  }
}

RLIS_API int rlis_depth_mix(float* x, const float* delta, float* hist, long long n, int count,
                            const void* weights, int weights_dtype, int save_input,
                            hipStream_t stream) {
  RLIS_REQUIRE(count >= 2, "depth_mix: %d sources, at least the input and one result", count);
  RLIS_REQUIRE(!save_input || count == 2, "depth_mix: only the first layer stores its input");
  if (n <= 0) return 0;
  const int blocks = (int)(ceil_div_ll(n, 256) < 8192 ? ceil_div_ll(n, 256) : 8192);
  if (weights_dtype == RLIS_F32)
    depth_mix_kernel<float><<<blocks, 256, 0, stream>>>(x, delta, hist, n, count,
                                                        (const float*)weights, save_input);
  else if (weights_dtype == RLIS_BF16)
    depth_mix_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, delta, hist, n, count,
                                                         (const bf16_t*)weights, save_input);
  else
    RLIS_REQUIRE(false, "depth_mix: unknown dtype %d", weights_dtype);
  RLIS_LAUNCH_CHECK("depth_mix");
  return 0;
}

// ------------------------------------------------------------- tanh, in place
// x <- cap * tanh(x / cap) (cap 1: the plain function): the bound on the logits, and the
// activation between the two thin products of a low-rank projection.
template <typename TX>
__global__ void soft_cap_kernel(TX* __restrict__ x, long long n, float cap, float inv_cap) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) st(x + i, cap * tanhf(ld(x + i) * inv_cap));
}

RLIS_API int rlis_soft_cap(void* x, int dtype, long long n, float cap, hipStream_t stream) {
  RLIS_REQUIRE(cap > 0.f, "soft_cap: the cap must be positive");
  if (n <= 0) return 0;
  const int blocks = (int)(ceil_div_ll(n, 256) < 8192 ? ceil_div_ll(n, 256) : 8192);
  if (dtype == RLIS_F32)
    soft_cap_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n, cap, 1.0f / cap);
  else if (dtype == RLIS_BF16)
    soft_cap_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n, cap, 1.0f / cap);
  else
    RLIS_REQUIRE(false, "soft_cap: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("soft_cap");
  return 0;
}

// ------------------------------------------------ rotary encoding + K/V page write
// qkv (T, row_stride): q heads at columns [0, nh*d), k heads at [k_off, k_off + nkv*d), v heads
// at [v_off, v_off + nkv*d).  The first rot_dim dims of every q and k head are rotated
// (rotate-half: dim j pairs with j + rot_dim/2; or, `interleaved`, dim 2j pairs with 2j + 1;
// either way with the j-th angle of the position's row), the rest pass through.  q is rotated in
// place (not at all without rotate_q: the consumer turns it as it loads it).  When write_kv is
// set, rotated k goes to k_pages[page][kv head][offset][d] and v to
// v_pages[page][kv head][d][offset] (v is stored transposed inside a page), with
// page = slot / page_size, offset = slot % page_size; rotated k is not stored back to qkv.
template <typename TX>
__global__ void rope_kv_write_kernel(TX* __restrict__ qkv, long long row_stride, int k_off,
                                     int v_off, int nh, int nkv, int d, int rot_dim,
                                     const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ slots, TX* __restrict__ k_pages,
                                     TX* __restrict__ v_pages, int page_size, int write_kv,
                                     int interleaved, int rotate_q) {
  const int t = blockIdx.x;
  TX* row = qkv + (long long)t * row_stride;
  const int pos = positions[t];
  const int half = rot_dim / 2;
  const float* c = cos_t + (long long)pos * half;
  const float* s = sin_t + (long long)pos * half;
  // q heads: rotate in place.
  for (int i = threadIdx.x; i < (rotate_q ? nh * half : 0); i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    TX* p = row + h * d;
    const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
    const float x1 = ld(p + a), x2 = ld(p + b);
    const float cc = c[j], sn = s[j];
    st(p + a, x1 * cc - x2 * sn);
    st(p + b, x2 * cc + x1 * sn);
  }
  if (!write_kv) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const long long page = slot / page_size;
  const int off = slot - (int)page * page_size;
  // k heads: rotate and store to the page.
  for (int i = threadIdx.x; i < nkv * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    const TX* p = row + k_off + h * d;
    const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
    const float x1 = ld(p + a), x2 = ld(p + b);
    const float cc = c[j], sn = s[j];
    TX* dst = k_pages + ((page * nkv + h) * page_size + off) * d;
    st(dst + a, x1 * cc - x2 * sn);
    st(dst + b, x2 * cc + x1 * sn);
  }
  const int tail = d - rot_dim;
  for (int i = threadIdx.x; i < nkv * tail; i += blockDim.x) {
    const int h = i / tail, j = rot_dim + (i - h * tail);
    TX* dst = k_pages + ((page * nkv + h) * page_size + off) * d;
    dst[j] = row[k_off + h * d + j];
  }
  // v heads: store transposed.
  for (int i = threadIdx.x; i < nkv * d; i += blockDim.x) {
    const int h = i / d, j = i - h * d;
    v_pages[((page * nkv + h) * d + j) * page_size + off] = row[v_off + h * d + j];
  }
}

// bfloat16 with every head segment a multiple of 8 wide: 16-byte accesses.  The first
// `qk_blocks` workgroups rotate q in place and k into its page, tok_qk tokens each (heads from
// first_head on: nh when q is left alone); the others take kRopeTokV tokens times kRopeVCols value columns each and turn them through LDS, so
// that lanes which are neighbours in a page's (d, offset) layout store neighbouring offsets
// (tokens with adjacent slots fill whole 32-byte runs, whatever their alignment).
constexpr int kRopeTokV = 16;
constexpr int kRopeVCols = 256;                // v columns per workgroup
constexpr int kRopeVRow = kRopeVCols + 8;      // padded: rows stay 16-byte aligned, banks spread

__device__ __forceinline__ void unpack8(const uint4 u, float (&v)[8]) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(256) void rope_kv_write_bf16x8_kernel(
    bf16_t* __restrict__ qkv, long long row_stride, int k_off, int v_off, int T, int nh, int nkv,
    int d, int rot_dim, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slots,
    bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, int page_size, int write_kv,
    int qk_blocks, int tok_qk, int first_head) {
  const int tid = threadIdx.x;
  const int half = rot_dim / 2;
  if ((int)blockIdx.x < qk_blocks) {
    const int t0 = blockIdx.x * tok_qk;
    const int hc = half / 8;                             // chunks of 8 pairs per head
    const int heads = nh + (write_kv ? nkv : 0) - first_head;
    const int per_tok = heads * hc;
    for (int i = tid; i < tok_qk * per_tok; i += blockDim.x) {
      const int tt = i / per_tok, r = i - tt * per_tok, t = t0 + tt;
      if (t >= T) break;
      const int h = first_head + r / hc, j = (r - (h - first_head) * hc) * 8;
      const bool is_k = h >= nh;
      const int slot = is_k ? slots[t] : 0;
      if (slot < 0) continue;
      bf16_t* src = qkv + (long long)t * row_stride + (is_k ? k_off + (h - nh) * d : h * d);
      bf16_t* dst = src;
      if (is_k) {
        const long long page = slot / page_size;
        const int off = slot - (int)page * page_size;
        dst = k_pages + ((page * nkv + (h - nh)) * page_size + off) * d;
      }
      const long long cs = (long long)positions[t] * half + j;
      float x1[8], x2[8], c[8], s[8], o1[8], o2[8];
      unpack8(*(const uint4*)(src + j), x1);
      unpack8(*(const uint4*)(src + j + half), x2);
      *(float4*)&c[0] = *(const float4*)(cos_t + cs);
      *(float4*)&c[4] = *(const float4*)(cos_t + cs + 4);
      *(float4*)&s[0] = *(const float4*)(sin_t + cs);
      *(float4*)&s[4] = *(const float4*)(sin_t + cs + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        o1[e] = x1[e] * c[e] - x2[e] * s[e];
        o2[e] = x2[e] * c[e] + x1[e] * s[e];
      }
      *(uint4*)(dst + j) = pack8(o1);
      *(uint4*)(dst + j + half) = pack8(o2);
    }
    if (write_kv && d > rot_dim) {                       // the dims of k that are not rotated
      const int tc = (d - rot_dim) / 8, per = nkv * tc;
      for (int i = tid; i < tok_qk * per; i += blockDim.x) {
        const int tt = i / per, r = i - tt * per, t = t0 + tt;
        if (t >= T) break;
        const int h = r / tc, j = rot_dim + (r - h * tc) * 8;
        const int slot = slots[t];
        if (slot < 0) continue;
        const long long page = slot / page_size;
        const int off = slot - (int)page * page_size;
        *(uint4*)(k_pages + ((page * nkv + h) * page_size + off) * d + j) =
            *(const uint4*)(qkv + (long long)t * row_stride + k_off + h * d + j);
      }
    }
    return;
  }
  // Values: a tile of kRopeTokV tokens times kRopeVCols columns per workgroup.
  __shared__ __attribute__((aligned(16))) bf16_t v_s[kRopeTokV * kRopeVRow];
  __shared__ long long page_s[kRopeTokV];                // -1: the token is not stored
  __shared__ int off_s[kRopeTokV];
  const int cols = nkv * d;
  const int chunks = (cols + kRopeVCols - 1) / kRopeVCols;
  const int vb = (int)blockIdx.x - qk_blocks;
  const int t0 = (vb / chunks) * kRopeTokV, c0 = (vb % chunks) * kRopeVCols;
  if (tid < kRopeTokV) {
    const int slot = t0 + tid < T ? slots[t0 + tid] : -1;
    const int page = slot < 0 ? -1 : slot / page_size;
    page_s[tid] = page;
    off_s[tid] = slot < 0 ? 0 : slot - page * page_size;
  }
  const int nc = min(kRopeVCols, cols - c0), nc8 = nc / 8;
  for (int i = tid; i < kRopeTokV * nc8; i += blockDim.x) {
    const int tt = i / nc8, c = (i - tt * nc8) * 8;
    if (t0 + tt < T)
      *(uint4*)(v_s + tt * kRopeVRow + c) =
          *(const uint4*)(qkv + (long long)(t0 + tt) * row_stride + v_off + c0 + c);
  }
  __syncthreads();
  for (int i = tid; i < kRopeTokV * nc; i += blockDim.x) {
    const int tt = i % kRopeTokV, c = i / kRopeTokV;
    const long long page = page_s[tt];
    if (page < 0) continue;
    const int col = c0 + c, h = col / d, j = col - h * d;
    v_pages[((page * nkv + h) * d + j) * page_size + off_s[tt]] = v_s[tt * kRopeVRow + c];
  }
}

RLIS_API int rlis_rope_kv_write(void* qkv, int dtype, long long row_stride, int k_off, int v_off,
                                int T, int nh, int nkv, int d, int rot_dim, const float* cos_t,
                                const float* sin_t, const int* positions, const int* slots,
                                void* k_pages, void* v_pages, int page_size, int write_kv,
                                int interleaved, int rotate_q, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && nkv >= 0 && (nkv > 0 || !write_kv) && d > 0,
               "rope_kv_write: bad sizes");
  RLIS_REQUIRE(rot_dim >= 0 && rot_dim <= d && rot_dim % 2 == 0,
               "rope_kv_write: rot_dim %d must be even and at most head_dim %d", rot_dim, d);
  RLIS_REQUIRE(!write_kv || (page_size > 0 && k_pages && v_pages && slots),
               "rope_kv_write: cache write asked for without pages");
  if (T == 0 || (!rotate_q && !write_kv)) return 0;
  const bool by8 = !interleaved && dtype == RLIS_BF16 && d % 8 == 0 && rot_dim % 16 == 0 && row_stride % 8 == 0 &&
                   k_off % 8 == 0 && v_off % 8 == 0 && ((uintptr_t)qkv % 16) == 0 &&
                   ((uintptr_t)cos_t % 16) == 0 && ((uintptr_t)sin_t % 16) == 0 &&
                   (!write_kv || (((uintptr_t)k_pages % 16) == 0 && T <= (1 << 30)));
  if (by8) {
    // about 64 chunks of 8 pairs or more to a workgroup of the first kind
    const int first_head = rotate_q ? 0 : nh;
    const int per_tok = (nh + (write_kv ? nkv : 0) - first_head) * (rot_dim / 16);
    int tok_qk = 2;
    while (tok_qk < 16 && tok_qk * per_tok < 256) tok_qk *= 2;
    const int qk_blocks = (per_tok > 0 || (write_kv && d > rot_dim)) ? ceil_div(T, tok_qk) : 0;
    const int v_blocks = write_kv ? ceil_div(T, kRopeTokV) * ceil_div(nkv * d, kRopeVCols) : 0;
    if (qk_blocks + v_blocks == 0) return 0;             // nothing is rotated, nothing stored
    rope_kv_write_bf16x8_kernel<<<qk_blocks + v_blocks, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, k_off, v_off, T, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, write_kv, qk_blocks, tok_qk,
        first_head);
    RLIS_LAUNCH_CHECK("rope_kv_write");
    return 0;
  }
  if (dtype == RLIS_F32)
    rope_kv_write_kernel<float><<<T, 256, 0, stream>>>(
        (float*)qkv, row_stride, k_off, v_off, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (float*)k_pages, (float*)v_pages, page_size, write_kv, interleaved, rotate_q);
  else if (dtype == RLIS_BF16)
    rope_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, k_off, v_off, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, write_kv, interleaved, rotate_q);
  else
    RLIS_REQUIRE(false, "rope_kv_write: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ---------------------------------------------------------------------- page copies
// pages (num_layers, num_pages, page_elems): copy page src[i] to dst[i] in every layer.
template <typename TX>
__global__ void copy_pages_kernel(TX* __restrict__ pages, long long layer_stride,
                                  long long page_elems, const int* __restrict__ src,
                                  const int* __restrict__ dst) {
  const int pair = blockIdx.x, layer = blockIdx.y;
  const TX* s = pages + layer * layer_stride + (long long)src[pair] * page_elems;
  TX* d = pages + layer * layer_stride + (long long)dst[pair] * page_elems;
  for (long long i = threadIdx.x; i < page_elems; i += blockDim.x) d[i] = s[i];
}

RLIS_API int rlis_copy_pages(void* pages, int dtype, int num_layers, long long num_pages,
                             long long page_elems, const int* src, const int* dst, int num_pairs,
                             hipStream_t stream) {
  RLIS_REQUIRE(num_layers > 0 && num_pages > 0 && page_elems > 0, "copy_pages: bad sizes");
  if (num_pairs <= 0) return 0;
  dim3 grid(num_pairs, num_layers);
  if (dtype == RLIS_F32)
    copy_pages_kernel<float><<<grid, 256, 0, stream>>>((float*)pages, num_pages * page_elems,
                                                       page_elems, src, dst);
  else if (dtype == RLIS_BF16)
    copy_pages_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)pages, num_pages * page_elems,
                                                        page_elems, src, dst);
  else
    RLIS_REQUIRE(false, "copy_pages: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("copy_pages");
  return 0;
}

// ------------------------------------------------------------- seeded random weights
// The generator of runtime/random_fill.cpp on the device: value i of a tensor is a function of
// (seed, tensor index, i) alone: two splitmix64 hashes of the pair index give two uniforms,
// Box-Muller in double precision turns them into the pair's two normals, rounded once to
// float32 (and, for a bfloat16 destination, once more).  The host's and the device's log, cos
// and sin may differ in the last digit of a double, which the rounding to float32 hides but for
// a value in a few hundred million.
__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

template <typename TO>
__global__ void fill_normal_kernel(TO* __restrict__ out, long long n, uint64_t key, double mean,
                                   double std_dev) {
  const long long pairs = (n + 1) / 2;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long j = (long long)blockIdx.x * blockDim.x + threadIdx.x; j < pairs; j += stride) {
    const uint64_t a = splitmix64(key + 2 * (uint64_t)j), b = splitmix64(key + 2 * (uint64_t)j + 1);
    const double u1 = ((double)(a >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    const double u2 = ((double)(b >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    const double r = sqrt(-2.0 * log(u1));
    const double angle = 6.283185307179586476925286766559 * u2;
    st(out + 2 * j, (float)(mean + std_dev * (r * cos(angle))));
    if (2 * j + 1 < n) st(out + 2 * j + 1, (float)(mean + std_dev * (r * sin(angle))));
  }
}

// out[0 .. n) = mean + std * N(0, 1) keyed by (seed, tensor); out is float32 or bfloat16.
RLIS_API int rlis_fill_normal_device(void* out, int out_dtype, long long n, unsigned long long seed,
                                     unsigned long long tensor, double mean, double std_dev,
                                     hipStream_t stream) {
  RLIS_REQUIRE(n >= 0 && out, "fill_normal: bad arguments");
  if (n == 0) return 0;
  // host side of the same hash
  auto mix = [](uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
  };
  const uint64_t key = mix((uint64_t)seed ^ mix((uint64_t)tensor));
  const long long pairs = (n + 1) / 2;
  const int blocks = (int)(ceil_div_ll(pairs, 256) < 8192 ? ceil_div_ll(pairs, 256) : 8192);
  if (out_dtype == RLIS_F32)
    fill_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, key, mean, std_dev);
  else if (out_dtype == RLIS_BF16)
    fill_normal_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, n, key, mean, std_dev);
  else
    RLIS_REQUIRE(false, "fill_normal: unknown dtype %d", out_dtype);
  RLIS_LAUNCH_CHECK("fill_normal");
  return 0;
}

// ------------------------------------------------------------------ layer norm
// out = (x - mean) / sqrt(var + eps) * weight + bias over a row of x = resid + scale * delta
// (delta optional; a stack of float32 partial sums is added in order, and with round_parts
// rounded to bfloat16 first), var the mean of the squared deviations from the mean.  The
// sum is stored back into the residual when write_resid is set; with `rows` only those rows
// are made and the residual stays.  Sum, statistics and both multiplies are float32; the row
// waits in LDS between the passes (one read of the operands).
template <typename TD, typename TW, typename TO>
__global__ __launch_bounds__(256) void add_layernorm_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, const TW* __restrict__ weight,
    const TW* __restrict__ bias, TO* __restrict__ out, const int* __restrict__ rows, int H,
    float eps, int write_resid, int parts, long long part_stride, int round_parts,
    float delta_scale) {
  extern __shared__ float row_s[];
  __shared__ float red[4];
  const int r = blockIdx.x;
  const long long src = rows ? rows[r] : r;
  float* xr = resid + src * H;
  float sum = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = xr[j];
    if (delta) v += delta_scale * delta_sum(delta + src * H + j, parts, part_stride, round_parts);
    row_s[j] = v;
    if (write_resid) xr[j] = v;
    sum += v;
  }
  const float mean = block_sum<256>(sum, red) / (float)H;
  float sq = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) {
    const float d = row_s[j] - mean;
    sq += d * d;
  }
  const float mult = 1.0f / sqrtf(block_sum<256>(sq, red) / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256)
    st(out + (long long)r * H + j, (row_s[j] - mean) * mult * widen(weight[j]) + widen(bias[j]));
}

RLIS_API int rlis_add_layernorm(float* resid, const void* delta, int delta_dtype,
                                const void* weight, const void* bias, int weight_dtype, void* out,
                                int out_dtype, const int* rows, int R, int H, float eps,
                                int write_resid, int parts, long long part_stride,
                                int round_parts, float delta_scale, hipStream_t stream) {
  RLIS_REQUIRE(R >= 0 && H > 0 && H <= 16000, "add_layernorm: bad sizes R=%d H=%d", R, H);
  RLIS_REQUIRE(parts >= 1, "add_layernorm: parts=%d", parts);
  RLIS_REQUIRE(!(rows && write_resid && delta),
               "add_layernorm: writing the residual back needs all rows, not a selection");
  if (R == 0) return 0;
  const int key = (delta ? delta_dtype : RLIS_F32) * 4 + weight_dtype * 2 + out_dtype;
#define CASE(k, TD, TW, TO)                                                                  \
  case k:                                                                                    \
    add_layernorm_kernel<TD, TW, TO><<<R, 256, (size_t)H * 4, stream>>>(                     \
        resid, (const TD*)delta, (const TW*)weight, (const TW*)bias, (TO*)out, rows, H, eps, \
        write_resid && delta, parts, part_stride, round_parts, delta_scale);                 \
    break;
  switch (key) {
    CASE(0, float, float, float)
    CASE(1, float, float, bf16_t)
    CASE(2, float, bf16_t, float)
    CASE(3, float, bf16_t, bf16_t)
    CASE(4, bf16_t, float, float)
    CASE(5, bf16_t, float, bf16_t)
    CASE(6, bf16_t, bf16_t, float)
    CASE(7, bf16_t, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "add_layernorm: unknown dtypes");
  }
#undef CASE
  RLIS_LAUNCH_CHECK("add_layernorm");
  return 0;
}

// x <- x * factor in place (float32 product, one rounding).
template <typename TX>
__global__ void scale_kernel(TX* __restrict__ x, long long n, float factor) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) st(x + i, ld(x + i) * factor);
}

RLIS_API int rlis_scale(void* x, int dtype, long long n, float factor, hipStream_t stream) {
  RLIS_REQUIRE(n >= 0, "scale: bad size");
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)ceil_div_ll(n, 256);
  if (dtype == RLIS_F32) scale_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n, factor);
  else if (dtype == RLIS_BF16) scale_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n, factor);
  else RLIS_REQUIRE(false, "scale: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("scale");
  return 0;
}
