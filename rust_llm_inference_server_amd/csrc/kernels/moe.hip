// A routed feed-forward: every token goes through `top` of E small gated units.
//
//  * moe_route: from the router's float32 logits z: s = sigmoid(z); choice = s + correction;
//    experts stand in G equal groups of neighbours, a group's score is the sum of its two
//    largest choice scores, only experts of the `keep` best groups can be chosen (the others
//    count as minus infinity); the `top` largest choice scores win (the lower index on a tie);
//    an expert's weight is its s times `scale`, not renormalised.  One wave per token.
//    Switches: s = softmax(z) over all experts; a group's score the largest choice score in it;
//    the chosen experts' weights divided by their sum; a bias per expert added to the logits in
//    front of everything (softmax scores over all experts, divided by the chosen ones' sum, are
//    the softmax over the chosen logits alone).  A unit's bounded form: see gated_unit; units
//    without a gate (one projection, the square of its ReLU, the down projection): plain_unit.
//  * moe_sort: the step's (token, choice) pairs ordered by expert, every expert's run padded to
//    whole tiles of rows, so that a tile has one expert.  Decided on the device: nothing waits
//    for the host.  Which row of its expert's run a pair gets does not move its result: rows of a
//    tile do not see each other.
//  * moe_gate_up / moe_down: the units' products on the matrix cores, tile by tile
//    (tile_mma.h), rows gathered through the sorted list; silu(gate) * up in the epilogue of the
//    first, the pair's weight in the epilogue of the second.
//    Steps of thousands of pairs take tiles of 128 rows staged through LDS (moe_tiles128).
//  * moe_combine: a token's pairs added in the order of its choices, plus an optional addend
//    (a shared unit that every token takes), float32.
#include "common.h"
#include "tile_mma.h"

#include <math.h>

// ------------------------------------------------------------------ router logits
// z[t][e] = w_router[e] . ln(x[t]) with ln the layer norm of the float32 residual row
// ((x - mean) / sqrt(var + eps) * weight + bias), all in float32: the router then decides on
// the unrounded normalised input, whatever dtype the other consumers of the norm take.  One
// workgroup per token and eight experts; the normalised row waits in LDS.
template <typename TW>
__global__ __launch_bounds__(256) void moe_router_logits_kernel(
    const float* __restrict__ resid, const TW* __restrict__ ln_w, const TW* __restrict__ ln_b,
    float eps, const TW* __restrict__ w_router, float* __restrict__ z, int W, int E) {
  extern __shared__ float row_s[];
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* xr = resid + (long long)t * W;
  float sum = 0.f;
  for (int j = threadIdx.x; j < W; j += 256) {
    const float v = xr[j];
    row_s[j] = v;
    sum += v;
  }
  const float mean = block_sum<256>(sum, red) / (float)W;
  float sq = 0.f;
  for (int j = threadIdx.x; j < W; j += 256) {
    const float d = row_s[j] - mean;
    sq += d * d;
  }
  const float mult = 1.0f / sqrtf(block_sum<256>(sq, red) / (float)W + eps);
  for (int j = threadIdx.x; j < W; j += 256)
    row_s[j] = (row_s[j] - mean) * mult * widen(ln_w[j]) + widen(ln_b[j]);
  __syncthreads();
  // a workgroup takes eight experts (grid.y of them cover all), a wave two of them in turn; a
  // lane's products of a row are asked for eight at a time
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int e_end = min(E, (int)(blockIdx.y + 1) * 8);
  for (int e = blockIdx.y * 8 + wave; e < e_end; e += 4) {
    const TW* w = w_router + (long long)e * W;
    float part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = 0.f;
    for (int j0 = 0; j0 < W; j0 += 8 * kWave) {
      TW wv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = j0 + u * kWave + lane;
        wv[u] = w[j < W ? j : 0];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = j0 + u * kWave + lane;
        part[u] = fmaf(j < W ? row_s[j] : 0.f, widen(wv[u]), part[u]);
      }
    }
    float dot = ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
    dot = wave_sum(dot);
    if (lane == 0) z[(long long)t * E + e] = dot;
  }
}

RLIS_API int rlis_moe_router_logits(const float* resid, const void* ln_w, const void* ln_b,
                                    float eps, const void* w_router, int dtype, float* z, int T,
                                    int W, int E, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && W > 0 && W <= 16000 && E > 0 && E <= 8 * 65535,
               "moe_router_logits: bad sizes");
  if (T == 0) return 0;
  if (dtype == RLIS_F32)
    moe_router_logits_kernel<float><<<dim3(T, ceil_div(E, 8)), 256, (size_t)W * 4, stream>>>(
        resid, (const float*)ln_w, (const float*)ln_b, eps, (const float*)w_router, z, W, E);
  else if (dtype == RLIS_BF16)
    moe_router_logits_kernel<bf16_t><<<dim3(T, ceil_div(E, 8)), 256, (size_t)W * 4, stream>>>(
        resid, (const bf16_t*)ln_w, (const bf16_t*)ln_b, eps, (const bf16_t*)w_router, z, W, E);
  else
    RLIS_REQUIRE(false, "moe_router_logits: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("moe_router_logits");
  return 0;
}

// What a unit makes of its gate and up products: silu(g) * u, or with limit > 0 the bounded
// form g' * sigmoid(alpha * g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit).
// With alpha < 0 the unit is not gated at all: the two products are two halves of one
// projection's columns and each goes through the squared ReLU by itself (see plain_unit).
__device__ __forceinline__ float plain_unit(float z) {
  const float r = fmaxf(z, 0.f);
  return r * r;
}

__device__ __forceinline__ float gated_unit(float g, float u, float limit, float alpha) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
  }
  return g / (1.0f + expf(-g)) * u;
}

// ------------------------------------------------------------------------ route
// Scores: sigmoid of the logits, or (softmax_scores) their softmax over all experts.  A group's
// score: the sum of its two largest choice scores, or (group_max) the largest.  Weights: the
// chosen experts' scores times `scale`, or (renormalise) divided by their sum + 1e-20 first.
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, kWave);
    const int oi = __shfl_xor(idx, o, kWave);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
}

__global__ __launch_bounds__(64) void moe_route_kernel(
    const float* __restrict__ z, long long ldz, const float* __restrict__ correction, int E,
    int G, int keep, int top, float scale, int* __restrict__ chosen, float* __restrict__ weights,
    int softmax_scores, int group_max, int renormalise, const float* __restrict__ bias) {
  extern __shared__ float sm[];
  float* choice = sm;            // E
  float* gscore = sm + E;        // G
  float* score = sm + E + G;     // E
  const int t = blockIdx.x, lane = threadIdx.x;
  const int per = E / G;
  float zmax = -INFINITY, zsum = 1.f;
  if (softmax_scores) {
    for (int e = lane; e < E; e += 64)
      zmax = fmaxf(zmax, z[(long long)t * ldz + e] + (bias ? bias[e] : 0.f));
    zmax = wave_max(zmax);
    float part = 0.f;
    for (int e = lane; e < E; e += 64)
      part += expf(z[(long long)t * ldz + e] + (bias ? bias[e] : 0.f) - zmax);
    zsum = wave_sum(part);
  }
  for (int e = lane; e < E; e += 64) {
    const float zv = z[(long long)t * ldz + e] + (bias ? bias[e] : 0.f);
    const float s = softmax_scores ? expf(zv - zmax) / zsum : 1.0f / (1.0f + expf(-zv));
    score[e] = s;
    choice[e] = s + (correction ? correction[e] : 0.f);
  }
  __syncthreads();
  for (int g = lane; g < G; g += 64) {
    float a = -INFINITY, b = -INFINITY;       // the group's two largest
    for (int i = 0; i < per; ++i) {
      const float c = choice[g * per + i];
      if (c > a) { b = a; a = c; } else if (c > b) { b = c; }
    }
    gscore[g] = (per > 1 && !group_max) ? a + b : a;
  }
  __syncthreads();
  // the groups that stay: `keep` rounds of the largest score, lower index on a tie
  for (int round = 0; round < keep; ++round) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int g = lane; g < G; g += 64) {
      const float c = gscore[g];
      if (c == c && (c > v || (c == v && g < idx)) && c != INFINITY) { v = c; idx = g; }
    }
    wave_argmax(v, idx);
    if (lane == 0 && idx != 0x7fffffff) gscore[idx] = INFINITY;     // marks a kept group
    __syncthreads();
  }
  for (int e = lane; e < E; e += 64)
    if (gscore[e / per] != INFINITY) choice[e] = -INFINITY;
  __syncthreads();
  for (int round = 0; round < top; ++round) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c > v || (c == v && e < idx && c != -INFINITY)) { v = c; idx = e; }
    }
    wave_argmax(v, idx);
    if (idx == 0x7fffffff) idx = 0;            // fewer experts allowed than asked for
    if (lane == 0) {
      chosen[(long long)t * top + round] = idx;
      weights[(long long)t * top + round] = v == -INFINITY ? 0.f : score[idx] * scale;
      choice[idx] = -INFINITY;
    }
    __syncthreads();
  }
  if (renormalise && lane == 0) {
    float total = 0.f;
    for (int r = 0; r < top; ++r) total += weights[(long long)t * top + r];
    const float inv = 1.0f / (total + 1e-20f);
    for (int r = 0; r < top; ++r) weights[(long long)t * top + r] *= inv;
  }
}

RLIS_API int rlis_moe_route(const float* z, long long ldz, const float* correction, int T, int E,
                            int G, int keep, int top, float scale, int* chosen, float* weights,
                            int softmax_scores, int group_max, int renormalise,
                            const float* bias, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && E > 0 && G > 0 && E % G == 0 && keep >= 1 && keep <= G && top >= 1,
               "moe_route: bad sizes E=%d groups=%d keep=%d top=%d", E, G, keep, top);
  RLIS_REQUIRE(top <= keep * (E / G), "moe_route: %d experts asked of %d allowed", top,
               keep * (E / G));
  RLIS_REQUIRE(E <= 64 * 1024 / 16, "moe_route: too many experts");
  if (T == 0) return 0;
  moe_route_kernel<<<T, 64, (size_t)(2 * E + G) * 4, stream>>>(
      z, ldz, correction, E, G, keep, top, scale, chosen, weights, softmax_scores, group_max,
      renormalise, bias);
  RLIS_LAUNCH_CHECK("moe_route");
  return 0;
}

// ------------------------------------------------------------------------- sort
// sorted[row] = pair (or -1 for padding), tile_expert[tile] = expert (or -1: tile unused).
// One workgroup.  `tile_rows` rows a tile; `max_tiles` tiles are laid out.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ chosen, int P,
                                                        int E, int tile_rows, int max_tiles,
                                                        int* __restrict__ sorted,
                                                        int* __restrict__ tile_expert) {
  extern __shared__ int si[];
  int* count = si;          // E
  int* start = si + E;      // E
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int i = threadIdx.x; i < max_tiles * tile_rows; i += blockDim.x) sorted[i] = -1;
  for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = tile * tile_rows;
      const int tiles = (count[e] + tile_rows - 1) / tile_rows;
      for (int i = 0; i < tiles && tile + i < max_tiles; ++i) tile_expert[tile + i] = e;
      tile += tiles;
      count[e] = 0;
    }
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = chosen[p];
    sorted[start[e] + atomicAdd(&count[e], 1)] = p;
  }
}

RLIS_API int rlis_moe_sort(const int* chosen, int P, int E, int tile_rows, int max_tiles,
                           int* sorted, int* tile_expert, hipStream_t stream) {
  RLIS_REQUIRE(P >= 0 && E > 0 && tile_rows > 0 && max_tiles >= 0, "moe_sort: bad sizes");
  RLIS_REQUIRE((long long)max_tiles * tile_rows >= P + (long long)E * (tile_rows - 1) ||
                   max_tiles >= P,
               "moe_sort: %d tiles of %d rows may not hold %d pairs of %d experts", max_tiles,
               tile_rows, P, E);
  RLIS_REQUIRE(E <= 8192, "moe_sort: too many experts");
  if (P == 0) return 0;
  moe_sort_kernel<<<1, 1024, (size_t)E * 8, stream>>>(chosen, P, E, tile_rows, max_tiles, sorted,
                                                     tile_expert);
  RLIS_LAUNCH_CHECK("moe_sort");
  return 0;
}

// ---------------------------------------------------------------- gate/up product
// hidden[row][f] = silu(Wg[e][f] . x[token]) * (Wu[e][f] . x[token]) for the sorted rows of a
// tile; w_gu is (E, 2 F, K) with an expert's gate rows in front of its up rows.  A workgroup of
// WAVES waves takes 16 * WAVES rows x 32 columns.
template <typename T, int WAVES, bool ALIGNED>
__global__ __launch_bounds__(64 * WAVES) void moe_gate_up_kernel(
    const T* __restrict__ x, long long ldx, const T* __restrict__ w_gu,
    const int* __restrict__ sorted, const int* __restrict__ tile_expert, int top, int F, int K,
    T* __restrict__ hidden, float limit, float alpha) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int row0 = (blockIdx.x * WAVES + wave) * 16;
  const int f0 = blockIdx.y * 32;
  const int pair = sorted[row0 + lane % 16];
  const T* a_row = x + (long long)(pair < 0 ? 0 : pair / top) * ldx;
  const T* b_row[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int f = min(f0 + (b & 1) * 16 + lane % 16, F - 1);
    b_row[b] = w_gu + (((long long)e * 2 + (b >> 1)) * F + f) * K;      // 0, 1: gate; 2, 3: up
  }
  mma_f32x4 acc[4];
  wave_tile_product<T, 4, ALIGNED>(a_row, b_row, K, acc);
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int f = f0 + b * 16 + lane % 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = row0 + (lane / 16) * 4 + i;
      const float g = acc[b][i], u = acc[b + 2][i];
      if (f < F) {
        if (alpha < 0.f) {
          st(hidden + (long long)row * 2 * F + f, plain_unit(g));
          st(hidden + (long long)row * 2 * F + F + f, plain_unit(u));
        } else {
          st(hidden + (long long)row * F + f, gated_unit(g, u, limit, alpha));
        }
      }
    }
  }
}

// y[pair][n] = weight[pair] * (Wd[e][n] . hidden[row]); w_d is (E, N, F).  16 * WAVES rows x 64
// columns a workgroup.
template <typename T, int WAVES, bool ALIGNED>
__global__ __launch_bounds__(64 * WAVES) void moe_down_kernel(
    const T* __restrict__ hidden, const T* __restrict__ w_d, const int* __restrict__ sorted,
    const int* __restrict__ tile_expert, const float* __restrict__ weights, int N, int F,
    float* __restrict__ y) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int row0 = (blockIdx.x * WAVES + wave) * 16;
  const int n0 = blockIdx.y * 64;
  const T* a_row = hidden + (long long)(row0 + lane % 16) * F;
  const T* b_row[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int n = min(n0 + b * 16 + lane % 16, N - 1);
    b_row[b] = w_d + ((long long)e * N + n) * F;
  }
  mma_f32x4 acc[4];
  wave_tile_product<T, 4, ALIGNED>(a_row, b_row, F, acc);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int pair = sorted[row0 + (lane / 16) * 4 + i];
    if (pair < 0) continue;
    const float wt = weights[pair];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int n = n0 + b * 16 + lane % 16;
      if (n < N) y[(long long)pair * N + n] = acc[b][i] * wt;
    }
  }
}


// The same two products for tiles of 64 rows (steps of many pairs): a wave takes all 64 rows of
// the tile against columns of its own (gate/up: 32 of each, down: 64), so that every weight
// fragment it loads serves four blocks of rows; the four waves of a workgroup take four
// neighbouring column blocks of the same tile.  A row's sums are those of the small tiles.
template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256) void moe_gate_up_rows_kernel(
    const T* __restrict__ x, long long ldx, const T* __restrict__ w_gu,
    const int* __restrict__ sorted, const int* __restrict__ tile_expert, int top, int F, int K,
    T* __restrict__ hidden, float limit, float alpha) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int row0 = blockIdx.x * 64;
  const int f0 = (blockIdx.y * 4 + wave) * 32;
  if (f0 >= F) return;
  const T* a_row[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int pair = sorted[row0 + a * 16 + lane % 16];
    a_row[a] = x + (long long)(pair < 0 ? 0 : pair / top) * ldx;
  }
  const T* b_row[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int f = min(f0 + (b & 1) * 16 + lane % 16, F - 1);
    b_row[b] = w_gu + (((long long)e * 2 + (b >> 1)) * F + f) * K;
  }
  mma_f32x4 acc[4][4];
  wave_tile_product_rows<T, 4, 4, ALIGNED>(a_row, b_row, K, acc);
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int f = f0 + b * 16 + lane % 16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = row0 + a * 16 + (lane / 16) * 4 + i;
        const float g = acc[a][b][i], u = acc[a][b + 2][i];
        if (f < F) {
          if (alpha < 0.f) {
            st(hidden + (long long)row * 2 * F + f, plain_unit(g));
            st(hidden + (long long)row * 2 * F + F + f, plain_unit(u));
          } else {
            st(hidden + (long long)row * F + f, gated_unit(g, u, limit, alpha));
          }
        }
      }
    }
}

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256) void moe_down_rows_kernel(
    const T* __restrict__ hidden, const T* __restrict__ w_d, const int* __restrict__ sorted,
    const int* __restrict__ tile_expert, const float* __restrict__ weights, int N, int F,
    float* __restrict__ y) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int row0 = blockIdx.x * 64;
  const int n0 = (blockIdx.y * 4 + wave) * 64;
  if (n0 >= N) return;
  const T* a_row[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) a_row[a] = hidden + (long long)(row0 + a * 16 + lane % 16) * F;
  const T* b_row[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int n = min(n0 + b * 16 + lane % 16, N - 1);
    b_row[b] = w_d + ((long long)e * N + n) * F;
  }
  mma_f32x4 acc[4][4];
  wave_tile_product_rows<T, 4, 4, ALIGNED>(a_row, b_row, F, acc);
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int pair = sorted[row0 + a * 16 + (lane / 16) * 4 + i];
      if (pair < 0) continue;
      const float wt = weights[pair];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int n = n0 + b * 16 + lane % 16;
        if (n < N) y[(long long)pair * N + n] = acc[a][b][i] * wt;
      }
    }
}

// ------------------------------------------------- tiles of 128 rows through LDS (bfloat16)
// For steps of thousands of pairs: the dense matrix-core product's cut (tile 128 x 128 x 64,
// both operands staged through LDS with the next k slab in registers meanwhile, four waves of
// 64 x 64 as 2 x 2 blocks of v_mfma_f32_32x32x16_bf16) with a tile's rows gathered through the
// sorted list and its weights taken from the tile's expert.  GATE_UP: the 128 weight rows of a
// tile are [gate f..f+31 | up f..f+31 | gate f+32..f+63 | up f+32..f+63], so that a wave holds
// gate and up of the same 32 columns and stores silu(gate) * up; otherwise the result times
// the pair's weight goes to the pair's row of y.
typedef float moe_f32x16 __attribute__((ext_vector_type(16)));

template <bool GATE_UP>
__global__ __launch_bounds__(256) void moe_tiles128_kernel(
    const bf16_t* __restrict__ A, long long lda, const bf16_t* __restrict__ W,
    const int* __restrict__ sorted, const int* __restrict__ tile_expert,
    const float* __restrict__ weights, int top, int N, int K, bf16_t* __restrict__ hidden,
    float* __restrict__ y, float limit, float alpha) {
  constexpr int BM = 128, BK = 64, LDS_STRIDE = BK + 8;
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BM * LDS_STRIDE];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int row0 = blockIdx.x * BM;
  const int n0 = blockIdx.y * (GATE_UP ? 64 : 128);
  // the rows this thread moves: chunk c = tid + 256 i covers tile row c / 8, k offset (c % 8) * 8
  const bf16_t* a_src[4];
  const bf16_t* b_src[4];
  bool b_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (tid + i * 256) / 8;
    if (GATE_UP) {
      const int pair = sorted[row0 + r];
      a_src[i] = A + (long long)(pair < 0 ? 0 : pair / top) * lda;
      const int f = n0 + (r / 64) * 32 + r % 32;
      b_ok[i] = f < N;
      b_src[i] = W + (((long long)e * 2 + (r / 32) % 2) * N + (b_ok[i] ? f : 0)) * K;
    } else {
      a_src[i] = A + (long long)(row0 + r) * lda;
      const int n = n0 + r;
      b_ok[i] = n < N;
      b_src[i] = W + ((long long)e * N + (b_ok[i] ? n : 0)) * K;
    }
  }
  moe_f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  mma_u32x4 ra[4], rb[4];
  const mma_u32x4 zero = {0u, 0u, 0u, 0u};
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int gk = k0 + ((tid + i * 256) % 8) * 8;
      const mma_u32x4 va = *reinterpret_cast<const mma_u32x4*>(a_src[i] + (gk < K ? gk : 0));
      const mma_u32x4 vb = *reinterpret_cast<const mma_u32x4*>(b_src[i] + (gk < K ? gk : 0));
      ra[i] = gk < K ? va : zero;
      rb[i] = (gk < K && b_ok[i]) ? vb : zero;
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * 256;
      *reinterpret_cast<mma_u32x4*>(As + (c / 8) * LDS_STRIDE + (c % 8) * 8) = ra[i];
      *reinterpret_cast<mma_u32x4*>(Bs + (c / 8) * LDS_STRIDE + (c % 8) * 8) = rb[i];
    }
  };
  const int num_k = (K + BK - 1) / BK;
  load_global(0);
  store_lds();
  __syncthreads();
  for (int kt = 0; kt < num_k; ++kt) {
    if (kt + 1 < num_k) load_global((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      mma_bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = *reinterpret_cast<const mma_bf16x8*>(
            As + (wm * 64 + i * 32 + lane % 32) * LDS_STRIDE + ks * 16 + (lane / 32) * 8);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        b[j] = *reinterpret_cast<const mma_bf16x8*>(
            Bs + (wn * 64 + j * 32 + lane % 32) * LDS_STRIDE + ks * 16 + (lane / 32) * 8);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (kt + 1 < num_k) {
      store_lds();
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row0 + wm * 64 + i * 32 + (r / 4) * 8 + (lane / 32) * 4 + r % 4;
      if (GATE_UP) {
        const int f = n0 + wn * 32 + lane % 32;
        const float g = acc[i][0][r], u = acc[i][1][r];
        if (f < N) {
          if (alpha < 0.f) {
            hidden[(long long)row * 2 * N + f] = f32_to_bf16(plain_unit(g));
            hidden[(long long)row * 2 * N + N + f] = f32_to_bf16(plain_unit(u));
          } else {
            hidden[(long long)row * N + f] = f32_to_bf16(gated_unit(g, u, limit, alpha));
          }
        }
      } else {
        const int pair = sorted[row];
        if (pair < 0) continue;
        const float wt = weights[pair];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + wn * 64 + j * 32 + lane % 32;
          if (n < N) y[(long long)pair * N + n] = acc[i][j][r] * wt;
        }
      }
    }
}

RLIS_API int rlis_moe_experts(const void* x, int dtype, long long ldx, const void* w_gu,
                              const void* w_d, const int* sorted, const int* tile_expert,
                              const float* weights, int tile_rows, int max_tiles, int top, int F,
                              int K, void* hidden, float* y, float limit, float alpha,
                              hipStream_t stream) {
  RLIS_REQUIRE((tile_rows == 16 || tile_rows == 64 || tile_rows == 128) && max_tiles >= 0 &&
                   top > 0 && F > 0 && K > 0,
               "moe_experts: bad sizes");
  RLIS_REQUIRE(ldx >= K, "moe_experts: row stride shorter than a row");
  if (max_tiles == 0) return 0;
  // plain units (alpha < 0): the up projection's 2 F columns are the hidden row, F "gate"
  // columns in front of F "up" columns, and the down product runs over all of them
  const int FD = alpha < 0.f ? 2 * F : F;
  if (tile_rows == 128) {
    RLIS_REQUIRE(dtype == RLIS_BF16 && mma_rows_aligned<bf16_t>(x, ldx, 0, K) &&
                     mma_rows_aligned<bf16_t>(w_gu, K, 0, K) &&
                     mma_rows_aligned<bf16_t>(hidden, FD, 0, FD) &&
                     mma_rows_aligned<bf16_t>(w_d, FD, 0, FD),
                 "moe_experts: tiles of 128 rows take bfloat16 rows on 16-byte boundaries");
    RLIS_REQUIRE(ceil_div(F, 64) <= 65535 && ceil_div(K, 128) <= 65535, "moe_experts: too wide");
    moe_tiles128_kernel<true><<<dim3(max_tiles, ceil_div(F, 64)), 256, 0, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w_gu, sorted, tile_expert, weights, top, F, K,
        (bf16_t*)hidden, nullptr, limit, alpha);
    moe_tiles128_kernel<false><<<dim3(max_tiles, ceil_div(K, 128)), 256, 0, stream>>>(
        (const bf16_t*)hidden, FD, (const bf16_t*)w_d, sorted, tile_expert, weights, top, K, FD,
        nullptr, y, 0.f, 0.f);
    RLIS_LAUNCH_CHECK("moe_experts");
    return 0;
  }
  RLIS_REQUIRE(ceil_div(F, 32) <= 65535 && ceil_div(K, 64) <= 65535, "moe_experts: too wide");
  dim3 g1(max_tiles, ceil_div(F, 32)), g2(max_tiles, ceil_div(K, 64));
#define LAUNCH(T, WAVES, AL1, AL2)                                                             \
  do {                                                                                         \
    if (WAVES == 4) {                                                                          \
      moe_gate_up_rows_kernel<T, AL1><<<dim3(max_tiles, ceil_div(F, 128)), 256, 0, stream>>>(  \
          (const T*)x, ldx, (const T*)w_gu, sorted, tile_expert, top, F, K, (T*)hidden, limit, \
          alpha);                                                                              \
      moe_down_rows_kernel<T, AL2><<<dim3(max_tiles, ceil_div(K, 256)), 256, 0, stream>>>(     \
          (const T*)hidden, (const T*)w_d, sorted, tile_expert, weights, K, FD, y);            \
    } else {                                                                                   \
      moe_gate_up_kernel<T, WAVES, AL1><<<g1, 64 * WAVES, 0, stream>>>(                        \
          (const T*)x, ldx, (const T*)w_gu, sorted, tile_expert, top, F, K, (T*)hidden, limit, \
          alpha);                                                                              \
      moe_down_kernel<T, WAVES, AL2><<<g2, 64 * WAVES, 0, stream>>>(                           \
          (const T*)hidden, (const T*)w_d, sorted, tile_expert, weights, K, FD, y);            \
    }                                                                                          \
  } while (0)
#define BY_ALIGN(T, WAVES)                                                                    \
  do {                                                                                        \
    const bool a1 = mma_rows_aligned<T>(x, ldx, 0, K) && mma_rows_aligned<T>(w_gu, K, 0, K);  \
    const bool a2 = mma_rows_aligned<T>(hidden, FD, 0, FD) && mma_rows_aligned<T>(w_d, FD, 0, FD); \
    if (a1 && a2) LAUNCH(T, WAVES, true, true);                                               \
    else if (a1) LAUNCH(T, WAVES, true, false);                                               \
    else if (a2) LAUNCH(T, WAVES, false, true);                                               \
    else LAUNCH(T, WAVES, false, false);                                                      \
  } while (0)
  if (dtype == RLIS_BF16) {
    if (tile_rows == 16) BY_ALIGN(bf16_t, 1); else BY_ALIGN(bf16_t, 4);
  } else if (dtype == RLIS_F32) {
    if (tile_rows == 16) BY_ALIGN(float, 1); else BY_ALIGN(float, 4);
  } else {
    RLIS_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  }
#undef BY_ALIGN
#undef LAUNCH
  RLIS_LAUNCH_CHECK("moe_experts");
  return 0;
}

// ---------------------------------------------------------------------- combine
// out[t][n] = sum over the token's `top` pairs of y[t * top + k][n], in the order of k, plus
// addend[t][n] when there is one.
template <typename TA>
__global__ void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y,
                                   const TA* __restrict__ addend, int top, int N, long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long t = i / N;
  const int n = (int)(i % N);
  float s = 0.f;
  for (int k = 0; k < top; ++k) s += y[(t * top + k) * N + n];
  if (addend) s += ld(addend + i);
  out[i] = s;
}

RLIS_API int rlis_moe_combine(float* out, const float* y, const void* addend, int addend_dtype,
                              int T, int top, int N, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && top > 0 && N > 0, "moe_combine: bad sizes");
  const long long total = (long long)T * N;
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)ceil_div_ll(total, 256);
  if (!addend || addend_dtype == RLIS_F32)
    moe_combine_kernel<float><<<blocks, 256, 0, stream>>>(out, y, (const float*)addend, top, N, total);
  else if (addend_dtype == RLIS_BF16)
    moe_combine_kernel<bf16_t><<<blocks, 256, 0, stream>>>(out, y, (const bf16_t*)addend, top, N, total);
  else
    RLIS_REQUIRE(false, "moe_combine: unknown dtype %d", addend_dtype);
  RLIS_LAUNCH_CHECK("moe_combine");
  return 0;
}
