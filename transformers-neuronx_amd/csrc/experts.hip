// A mixture of gated experts: the router's choice, the step's (token, choice) pairs put in the order of their
// experts, and the two products of every expert over its own pairs,
//     inner = act(w g) * (w u)  with [g | u] = W_gate_up[e] h      (the weight w on the expert's input; on its
//     y = W_down[e] inner                                           output it multiplies y instead)
// summed over a token's choices onto the residual in float32. Nothing is read back by the host: the launches are
// sized by the most tiles the pairs can make, and a block that finds no tile ends at once.
#include "common.h"

TNX_DEFINE_ERROR_API

#define TNX_ACT_SILU 4
#define TNX_ACT_CLAMPED_SWIGLU 6

namespace {

__device__ __forceinline__ float gate_act(float x, int act) {
  if (act == TNX_ACT_SILU) return x / (1.f + expf(-x));
  return apply_act(x, act);
}

// What a gated expert makes of the two halves of its first product: act(g) * u; the clamped form, with
// g' = min(g, limit) and u' = clamp(u, -limit, limit): g' sigmoid(1.702 g') (u' + 1).
__device__ __forceinline__ float gated(float g, float u, int act, float limit) {
  if (act == TNX_ACT_CLAMPED_SWIGLU) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + expf(-1.702f * g)) * (u + 1.f);
  }
  return gate_act(g, act) * u;
}

// ---------------------------------------------------------------- the router's choice
// A wave a token: `top` rounds of the largest logit (the lower number where two are equal), whose score sigmoid(z)
// or softmax(z) is the weight. The ranking is by the logits, which both scores grow with: two large logits that
// float32 still tells apart can have scores that it does not. With `correction` (a number an expert) the ranking is
// by score + correction, and the weight is the score without it; `scale` multiplies every weight.
__global__ void __launch_bounds__(256) route_kernel(const float* __restrict__ z, int tokens, int experts, int top,
                                                    int softmax, int renormalize, int* __restrict__ chosen,
                                                    float* __restrict__ weights, const float* __restrict__ correction,
                                                    float scale) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= tokens) return;
  const float* row = z + (size_t)t * experts;
  float peak = -INFINITY, total = 1.f;
  if (softmax) {
    for (int e = lane; e < experts; e += 64) peak = fmaxf(peak, row[e]);
    peak = wave_max(peak);
    float s = 0.f;
    for (int e = lane; e < experts; e += 64) s += expf(row[e] - peak);
    total = wave_sum(s);
  }
  auto score = [&](float z) { return softmax ? expf(z - peak) / total : 1.f / (1.f + expf(-z)); };
  auto rank = [&](int e) { return correction ? score(row[e]) + correction[e] : row[e]; };
  float sum = 0.f;
  unsigned long long taken = 0;        // bit i: expert lane + 64 i is chosen already (a lane's own experts)
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY;
    int at = experts;
    for (int e = lane, i = 0; e < experts; e += 64, ++i) {
      const float z = rank(e);
      if (!((taken >> i) & 1) && (z > best || at == experts)) best = z, at = e;   // ascending e: the lower number stays where two are equal
    }
    const float high = wave_max(best);
    const int first = -(int)wave_max((float)-((best == high && at < experts) ? at : experts));
    if ((first & 63) == lane) taken |= 1ull << (first >> 6);
    const float s = correction ? score(row[first]) : score(high);
    if (lane == 0) {
      chosen[(size_t)t * top + c] = first;
      weights[(size_t)t * top + c] = renormalize ? 0.f : s * scale;
    }
    sum += s;
  }
  if (renormalize) {
    // the same rounds again, now that the sum is known: each weight is written once
    taken = 0;
    for (int c = 0; c < top; ++c) {
      float best = -INFINITY;
      int at = experts;
      for (int e = lane, i = 0; e < experts; e += 64, ++i) {
        const float z = rank(e);
        if (!((taken >> i) & 1) && (z > best || at == experts)) best = z, at = e;
      }
      const float high = wave_max(best);
      const int first = -(int)wave_max((float)-((best == high && at < experts) ? at : experts));
      if ((first & 63) == lane) taken |= 1ull << (first >> 6);
      if (lane == 0) weights[(size_t)t * top + c] = (correction ? score(row[first]) : score(high)) / sum * scale;
    }
  }
}

// ---------------------------------------------------------------- pairs in the order of their experts
// One block: counts an expert, where each expert's pairs begin (`first[E + 1]`), and the pairs (t * top + c)
// put there (`order`). The order within an expert changes no result: every pair's row is computed alone.
__global__ void __launch_bounds__(1024) order_kernel(const int* __restrict__ chosen, int pairs, int experts,
                                                     int* __restrict__ first, int* __restrict__ order,
                                                     int* __restrict__ place, int* __restrict__ token, int top,
                                                     const float* __restrict__ weights, float* __restrict__ sorted_weights) {
  extern __shared__ int counts[];      // [experts] counts, then [experts] cursors
  int* cursor = counts + experts;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      cursor[e] = at;
      at += counts[e];
    }
    first[experts] = at;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= 0 && e < experts) {
      const int at = atomicAdd(&cursor[e], 1);
      order[at] = i;
      if (place) place[i] = at;                       // where the pair's row lies among the sorted ones
      if (token) token[at] = i / top;                 // the token whose row the sorted row reads
      if (sorted_weights) sorted_weights[at] = weights[i];
    }
  }
}

// ---------------------------------------------------------------- an expert's product over its pairs
// out[pair, j] = sum_k A[row(pair), k] W[e][j][k] for the pairs of expert e, a tile of 16 pairs by 64 columns a
// block, float32 sums from tiles staged in LDS. GATED: W holds F gate rows and then F up rows, column j of the
// result is act(w g_j) * (w u_j) and the A row of a pair is its token's (pair / top). Otherwise the A row is the
// pair's own, and the result goes to `out` (pair rows, float32) or, where a token has one choice, straight onto
// the residual into the token's row.
struct ProductArgs {
  const void* a;            // GATED: h [T, K]; else inner [pairs, K]
  const void* w;            // [E, N(, 2), K]
  const int* first;         // [E + 1]
  const int* order;         // [pairs]
  const float* weights;     // [pairs]
  const float* residual;    // [T, N] or null (not GATED, one choice a token)
  void* out;
  int experts, top, n, k, act, weight_on_input, pairs;
  float limit;              // of the clamped activation
};

template <typename T, bool GATED>
__global__ void __launch_bounds__(256) expert_product_kernel(ProductArgs p) {
  constexpr int TM = 16, TN = 64, TK = 32;
  __shared__ float As[TM][TK + 1];
  __shared__ float Ws[GATED ? 2 : 1][TN][TK + 1];
  __shared__ int rows[TM];
  // which expert and which of its tiles of 16 pairs this block is
  int tile = blockIdx.y, e = 0, begin = 0, end = 0;
  for (; e < p.experts; ++e) {
    begin = p.first[e];
    end = p.first[e + 1];
    const int tiles = (end - begin + TM - 1) / TM;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (e >= p.experts) return;
  begin += tile * TM;
  const int count = min(TM, end - begin);
  const int col0 = blockIdx.x * TN;
  if (threadIdx.x < TM) rows[threadIdx.x] = threadIdx.x < count ? p.order[begin + threadIdx.x] : -1;
  __syncthreads();
  const T* A = (const T*)p.a;
  const T* W = (const T*)p.w + (size_t)e * (GATED ? 2 : 1) * p.n * p.k;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;        // column, and rows 4 ty .. 4 ty + 3
  float acc[GATED ? 2 : 1][4] = {};
  for (int k0 = 0; k0 < p.k; k0 += TK) {
    // the tile of A: 16 rows of 32, two elements a thread
    for (int i = threadIdx.x; i < TM * TK; i += 256) {
      const int r = i / TK, c = i - r * TK;
      const int pair = rows[r];
      float v = 0.f;
      if (pair >= 0 && k0 + c < p.k) v = to_f32(A[(size_t)(GATED ? pair / p.top : pair) * p.k + k0 + c]);
      As[r][c] = v;
    }
    // the tile of W: 64 (or twice 64) rows of 32
    for (int i = threadIdx.x; i < (GATED ? 2 : 1) * TN * TK; i += 256) {
      const int half = i / (TN * TK), j = (i - half * TN * TK) / TK, c = i % TK;
      float v = 0.f;
      if (col0 + j < p.n && k0 + c < p.k) v = to_f32(W[((size_t)half * p.n + col0 + j) * p.k + k0 + c]);
      Ws[half][j][c] = v;
    }
    __syncthreads();
#pragma unroll 8
    for (int c = 0; c < TK; ++c) {
      const float w0 = Ws[0][tx][c];
      const float w1 = GATED ? Ws[GATED ? 1 : 0][tx][c] : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float x = As[4 * ty + r][c];
        acc[0][r] += x * w0;
        if (GATED) acc[GATED ? 1 : 0][r] += x * w1;
      }
    }
    __syncthreads();
  }
  const int col = col0 + tx;
  if (col >= p.n) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int pair = rows[4 * ty + r];
    if (pair < 0) continue;
    const float w = p.weights[pair];
    if (GATED) {
      float g = acc[0][r], u = acc[GATED ? 1 : 0][r];
      if (p.weight_on_input) g *= w, u *= w;
      ((T*)p.out)[(size_t)pair * p.n + col] = from_f32<T>(gated(g, u, p.act, p.limit));
    } else {
      float y = acc[0][r];
      if (!p.weight_on_input) y *= w;
      if (p.top == 1)
        ((float*)p.out)[(size_t)pair * p.n + col] = y + (p.residual ? p.residual[(size_t)pair * p.n + col] : 0.f);
      else
        ((float*)p.out)[(size_t)pair * p.n + col] = y;
    }
  }
}


// The same tile on the matrix unit, bfloat16 with an inner size in 8s: a wave takes 16 columns (and with GATED the
// 16 up rows that go with its 16 gate rows) for the tile's 16 pairs and makes out^T[column][pair] with MFMA
// 16x16x32, the matrix's rows as the A operand, the pairs' rows as the B operand. An expert's matrix is read once
// for every 16 of its pairs, which in a decode step is once, so what counts is how the matrix streams: a wave
// brings KC elements of each of its rows into a piece of LDS of its own with loads that cover a row's bytes side
// by side (512 bytes or more a row and instruction, marked as read once), all of a chunk's loads under way
// together, and takes the operands from there; the pairs' rows come from the caches. The waves of a block never
// wait for one another.
template <bool GATED>
__global__ void __launch_bounds__(256) expert_product_mfma_kernel(ProductArgs p) {
  constexpr int TM = 16;
  constexpr int ROWS = GATED ? 32 : 16;                   // rows of the matrix a wave holds
  constexpr int KC = 256;                                 // elements of a row a chunk
  constexpr int LD = KC + 8;                              // a row in LDS: 16 bytes more, so that rows lie in different banks
  constexpr int LPR = KC / 8, RPI = 64 / LPR;             // lanes a row, rows an instruction
  constexpr int LOADS = ROWS / RPI;
  __shared__ __attribute__((aligned(16))) bf16_t staged[4][ROWS * LD];
  int tile = blockIdx.y, e = 0, begin = 0, end = 0;
  for (; e < p.experts; ++e) {
    begin = p.first[e];
    end = p.first[e + 1];
    const int tiles = (end - begin + TM - 1) / TM;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (e >= p.experts) return;
  begin += tile * TM;
  const int count = min(TM, end - begin);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int col0 = (blockIdx.x * 4 + wave) * 16;
  if (col0 >= p.n) return;
  const int pair = r < count ? p.order[begin + r] : -1;
  const bf16_t* xrow = (const bf16_t*)p.a + (size_t)(pair < 0 ? 0 : (GATED ? pair / p.top : pair)) * p.k;
  const bf16_t* W = (const bf16_t*)p.w + (size_t)e * (GATED ? 2 : 1) * p.n * p.k;
  bf16_t* mine = staged[wave];
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // load i of a chunk: row RPI i + lane / LPR of the wave's rows (the up rows behind the gate rows), elements 8 (lane % LPR) on
  const int lrow = lane / LPR, lcol = 8 * (lane % LPR);
  const bf16_t* src[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int row = RPI * i + lrow;                       // 0 .. 15 gate (or plain) rows, 16 .. 31 up rows
    const int n = col0 + (row & 15);
    src[i] = n < p.n ? W + ((size_t)(row >> 4) * p.n + n) * p.k + lcol : nullptr;
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc_up = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < p.k; k0 += KC) {
    bf16x8 got[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) got[i] = (src[i] != nullptr && k0 + lcol < p.k) ? load_once(src[i] + k0) : zero8;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) *(bf16x8*)(mine + (RPI * i + lrow) * LD + lcol) = got[i];
    const int steps = min(KC, p.k - k0);
    for (int kk = 0; kk < steps; kk += 32) {
      const int d0 = kk + 8 * g;
      const bool in = k0 + d0 < p.k;
      const bf16x8 b = (in && pair >= 0) ? *(const bf16x8*)(xrow + k0 + d0) : zero8;
      const bf16x8 a = *(const bf16x8*)(mine + r * LD + d0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
      if (GATED) {
        const bf16x8 u = *(const bf16x8*)(mine + (16 + r) * LD + d0);
        acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u, b, acc_up, 0, 0, 0);
      }
    }
  }
  if (pair < 0) return;
  const float w = p.weights[pair];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = col0 + 4 * g + i;        // the lane holds columns 4 g .. 4 g + 3 of pair r
    if (col >= p.n) continue;
    if (GATED) {
      float gt = acc[i], up = acc_up[i];
      if (p.weight_on_input) gt *= w, up *= w;
      ((bf16_t*)p.out)[(size_t)pair * p.n + col] = (bf16_t)gated(gt, up, p.act, p.limit);
    } else {
      float y = acc[i];
      if (!p.weight_on_input) y *= w;
      if (p.top == 1 && p.residual) y += p.residual[(size_t)pair * p.n + col];
      ((float*)p.out)[(size_t)pair * p.n + col] = y;
    }
  }
}

// (`place`: the row of y that holds pair t * top + c, where the rows lie in another order; `scale`: a factor a pair)
__global__ void combine_kernel(const float* __restrict__ y, const float* __restrict__ residual, float* __restrict__ out,
                               int top, size_t n, size_t total, const int* __restrict__ place,
                               const float* __restrict__ scale) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const size_t t = i / n, col = i - t * n;
    float s = residual ? residual[i] : 0.f;
    for (int c = 0; c < top; ++c) {
      const size_t pair = t * top + c;
      const float v = y[(place ? (size_t)place[pair] : pair) * n + col];
      s += scale ? scale[pair] * v : v;
    }
    out[i] = s;
  }
}

// act(g) * u from rows [g | u] of float32
// (`row_weights`: a factor a row on both g and u, the weight on an expert's input)
template <typename T>
__global__ void gated_activation_kernel(const float* __restrict__ gu, T* __restrict__ out, int f, int act, size_t total,
                                        const float* __restrict__ row_weights, float limit) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const size_t t = i / f, j = i - t * f;
    const float w = row_weights ? row_weights[t] : 1.f;
    out[i] = from_f32<T>(gated(w * gu[t * 2 * f + j], w * gu[t * 2 * f + f + j], act, limit));
  }
}

int blocks_for(size_t total) {
  size_t b = (total + 255) / 256;
  return (int)(b > 16384 ? 16384 : (b ? b : 1));
}

}  // namespace

extern "C" int tnx_route(const float* z, int tokens, int experts, int top, int softmax, int renormalize, int* chosen,
                         float* weights, const float* correction, float scale, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && experts > 0 && top > 0 && top <= experts, "route: %d of %d experts", top, experts);
  if (tokens == 0) return 0;
  route_kernel<<<(tokens + 3) / 4, 256, 0, stream>>>(z, tokens, experts, top, softmax, renormalize, chosen, weights,
                                                     correction, scale);
  TNX_CHECK_LAUNCH("route");
  return 0;
}

extern "C" int tnx_expert_mixture(const void* h, const int* chosen, const float* weights, const void* w_gate_up,
                                  const void* w_down, int* first, int* order, void* inner, float* pair_rows,
                                  const float* residual, float* out, int dtype, int tokens, int experts, int top,
                                  int width, int f, int act, int weight_on_input, int plain, float limit,
                                  hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && experts > 0 && top > 0 && width > 0 && f > 0, "expert_mixture: bad sizes");
  TNX_REQUIRE(experts <= 4096, "expert_mixture: up to 4096 experts, got %d", experts);
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "expert_mixture: dtype %d", dtype);
  TNX_REQUIRE(top == 1 || pair_rows != nullptr, "expert_mixture: several choices a token need room for their rows");
  if (tokens == 0) return 0;
  const int pairs = tokens * top;
  order_kernel<<<1, 1024, 2 * experts * sizeof(int), stream>>>(chosen, pairs, experts, first, order, nullptr, nullptr,
                                                               top, nullptr, nullptr);
  TNX_CHECK_LAUNCH("expert order");
  const int tiles = pairs / 16 + experts;       // the most tiles of 16 pairs: every expert may end in a part of one
  ProductArgs up{h, w_gate_up, first, order, weights, nullptr, inner, experts, top, f, width, act, weight_on_input, pairs,
                 limit};
  ProductArgs down{inner, w_down, first, order, weights, residual, top == 1 ? out : pair_rows, experts, top, width, f,
                   act, weight_on_input, pairs, limit};
  const dim3 grid_up((f + 63) / 64, tiles), grid_down((width + 63) / 64, tiles);
  if (dtype == TNX_F32) {
    expert_product_kernel<float, true><<<grid_up, 256, 0, stream>>>(up);
    expert_product_kernel<float, false><<<grid_down, 256, 0, stream>>>(down);
  } else if (width % 8 == 0 && f % 8 == 0 && !plain) {
    expert_product_mfma_kernel<true><<<grid_up, 256, 0, stream>>>(up);
    expert_product_mfma_kernel<false><<<grid_down, 256, 0, stream>>>(down);
  } else {
    expert_product_kernel<bf16_t, true><<<grid_up, 256, 0, stream>>>(up);
    expert_product_kernel<bf16_t, false><<<grid_down, 256, 0, stream>>>(down);
  }
  TNX_CHECK_LAUNCH("expert products");
  if (top > 1) {
    const size_t total = (size_t)tokens * width;
    combine_kernel<<<blocks_for(total), 256, 0, stream>>>(pair_rows, residual, out, top, (size_t)width, total, nullptr,
                                                          nullptr);
    TNX_CHECK_LAUNCH("expert combine");
  }
  return 0;
}

extern "C" int tnx_gated_activation(const float* gate_up, void* out, int dtype, int tokens, int f, int act,
                                    const float* row_weights, float limit, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && f > 0, "gated_activation: bad sizes");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "gated_activation: dtype %d", dtype);
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * f;
  if (dtype == TNX_F32)
    gated_activation_kernel<float><<<blocks_for(total), 256, 0, stream>>>(gate_up, (float*)out, f, act, total, row_weights, limit);
  else
    gated_activation_kernel<bf16_t><<<blocks_for(total), 256, 0, stream>>>(gate_up, (bf16_t*)out, f, act, total,
                                                                            row_weights, limit);
  TNX_CHECK_LAUNCH("gated_activation");
  return 0;
}

// The pairs in the order of their experts, for a caller that runs the experts' products itself: `first[E + 1]`,
// `order[pairs]`, `place[pairs]` (where a pair went), `token[pairs]` (the token of each sorted row) and the weights in
// sorted order.
extern "C" int tnx_expert_order(const int* chosen, const float* weights, int tokens, int experts, int top, int* first,
                                int* order, int* place, int* token, float* sorted_weights, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && experts > 0 && experts <= 4096 && top > 0, "expert_order: bad sizes");
  if (tokens == 0) return 0;
  order_kernel<<<1, 1024, 2 * experts * sizeof(int), stream>>>(chosen, tokens * top, experts, first, order, place, token,
                                                               top, weights, sorted_weights);
  TNX_CHECK_LAUNCH("expert order");
  return 0;
}

// out[t] = residual[t] + sum_c scale[t, c] y[place[t * top + c]]
extern "C" int tnx_expert_combine(const float* y, const int* place, const float* scale, const float* residual, float* out,
                                  int tokens, int top, int width, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && top > 0 && width > 0, "expert_combine: bad sizes");
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * width;
  combine_kernel<<<blocks_for(total), 256, 0, stream>>>(y, residual, out, top, (size_t)width, total, place, scale);
  TNX_CHECK_LAUNCH("expert combine");
  return 0;
}
