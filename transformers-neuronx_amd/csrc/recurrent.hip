// Recurrences that carry a state of fixed size from token to token, element by element.
//   min_gru                  S <- (1 - z) S + z c, the result S silu(g)
//   channel_conv             a causal convolution of a few taps on every channel, with a bias and per-request state
//   gated_linear_recurrence  S <- a S + sqrt(1 - a^2) i u with a = exp(rate sigmoid(r')), the result S gelu_tanh(y)
// Gates, decays and state are float32 with full-precision exponentials. In a step of single tokens a thread owns
// one channel of one run; what does not depend on the state (loads, gates) is made eight tokens at a time ahead of
// the chain. In a step with longer runs a run's tokens are cut into parts that a block's sixteen waves walk side by
// side (`*_by_segments`): both recurrences are S <- a S + b, so a part taken from S = 0 leaves (A, B) = (the product
// of its a, its last S), the parts' (A, B) meet in LDS, each part works out the S it begins with from those before
// it (S <- A S + B), and walks its tokens again from there, now writing. A token's S is made by the same chain of
// operations as by one thread alone from its part's first S on. State lies by position: the token at position p reads place (p - 1) & 1 of two and writes place p & 1, so
// a step of single tokens that is recorded and run again reads what it read the first time.
#include "common.h"

TNX_DEFINE_ERROR_API

namespace {

__device__ __forceinline__ float sigmoid_full(float x) { return 1.f / (1.f + expf(-x)); }

constexpr int AHEAD = 8;

template <typename T>
__global__ void __launch_bounds__(256)
min_gru_kernel(const float* __restrict__ proj, int ld, int inner, const int* __restrict__ positions,
               const int* __restrict__ run_start, const int* __restrict__ slots, float* __restrict__ carried,
               T* __restrict__ out, long long out_ld, float out_scale) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const int first = run_start[r], n = run_start[r + 1] - first;
  if (c >= inner || n <= 0) return;
  const int p0 = positions[first];
  float* mine = carried + (size_t)slots[r] * 2 * inner;
  float s = p0 > 0 ? mine[(size_t)((p0 - 1) & 1) * inner + c] : 0.f;
  for (int i0 = 0; i0 < n; i0 += AHEAD) {
    float z[AHEAD], cand[AHEAD], g[AHEAD];
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      const float* row = proj + (size_t)(first + i0 + k) * ld;
      z[k] = row[c];
      cand[k] = row[inner + c];
      g[k] = row[2 * inner + c];
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      z[k] = sigmoid_full(z[k]);
      cand[k] = cand[k] >= 0.f ? cand[k] + 0.5f : sigmoid_full(cand[k]);
      g[k] = g[k] * sigmoid_full(g[k]) * out_scale;
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      s = (1.f - z[k]) * s + z[k] * cand[k];
      out[(size_t)(first + i0 + k) * out_ld + c] = from_f32<T>(s * g[k]);
    }
  }
  mine[(size_t)((p0 + n - 1) & 1) * inner + c] = s;
}

// u[t, c] = bias[c] + sum_j w[j, c] x[t - taps + 1 + j, c] over the tokens of t's own request (zeros before its
// start); inputs from before the step's run come from the request's state `[taps, channels]`, the input at
// position p at place p mod taps. Weights tap by tap, `[taps, channels]`.
template <typename T>
__global__ void __launch_bounds__(256)
channel_conv_kernel(const float* __restrict__ x, long long ld, const float* __restrict__ w, const float* __restrict__ bias,
                    const float* __restrict__ state, int taps, const int* __restrict__ positions,
                    const int* __restrict__ token_request, const int* __restrict__ run_start,
                    const int* __restrict__ slots, float* __restrict__ out, T* __restrict__ out_cd, int channels) {
  const int t = blockIdx.x;
  const int r = token_request[t];
  const int i = t - run_start[r], p = positions[t];
  const float* mine = state ? state + (size_t)slots[r] * taps * channels : nullptr;
  for (int c = threadIdx.x; c < channels; c += 256) {
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float v = 0.f;
      if (back <= i)
        v = x[(size_t)(t - back) * ld + c];
      else if (back <= p && mine)
        v = mine[(size_t)((p - back) % taps) * channels + c];
      acc = fmaf(w[(size_t)j * channels + c], v, acc);
    }
    out[(size_t)t * channels + c] = acc;
    if (out_cd) out_cd[(size_t)t * channels + c] = from_f32<T>(acc);
  }
}

__global__ void __launch_bounds__(256)
channel_state_kernel(const float* __restrict__ x, long long ld, float* __restrict__ state, int taps,
                     const int* __restrict__ positions, const int* __restrict__ run_start,
                     const int* __restrict__ slots, int channels) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int first = run_start[r], n = run_start[r + 1] - first;
  if (c >= channels || n == 0) return;
  float* mine = state + (size_t)slots[r] * taps * channels;
  for (int i = max(0, n - (taps - 1)); i < n; ++i)
    mine[(size_t)(positions[first + i] % taps) * channels + c] = x[(size_t)(first + i) * ld + c];
}

struct RecurrenceArgs {
  const float* gates;       // [T, blocks, 2 w]
  const float* gate_bias;   // [blocks, 2 w]
  const float* u;           // [T, channels]
  const float* y;           // [T, y_ld]
  long long y_ld;
  const float* rate;        // [channels]
  const int* positions;
  const int* run_start;
  const int* slots;
  float* carried;           // [slots, 2, channels]
  void* out;
  long long out_ld;
  float out_scale;
  int channels, w;
};

template <typename T>
__global__ void __launch_bounds__(256) gated_linear_recurrence_kernel(RecurrenceArgs a) {
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const int first = a.run_start[r], n = a.run_start[r + 1] - first;
  if (c >= a.channels || n <= 0) return;
  const int b = c / a.w, j = c - b * a.w;
  const int at_r = b * 2 * a.w + j, at_i = at_r + a.w;            // within a token's gates
  const float bias_r = a.gate_bias[at_r], bias_i = a.gate_bias[at_i], rate = a.rate[c];
  const int p0 = a.positions[first];
  float* mine = a.carried + (size_t)a.slots[r] * 2 * a.channels;
  float s = p0 > 0 ? mine[(size_t)((p0 - 1) & 1) * a.channels + c] : 0.f;
  T* out = (T*)a.out;
  const size_t gates_ld = (size_t)2 * a.channels;
  for (int i0 = 0; i0 < n; i0 += AHEAD) {
    float decay[AHEAD], inp[AHEAD], y[AHEAD];
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      const size_t t = (size_t)(first + i0 + k);
      decay[k] = a.gates[t * gates_ld + at_r];
      inp[k] = a.gates[t * gates_ld + at_i];
      y[k] = a.y[t * a.y_ld + c];
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      const float uv = a.u[(size_t)(first + i0 + k) * a.channels + c];
      const float log_a = rate * sigmoid_full(decay[k] + bias_r);
      decay[k] = expf(log_a);
      // sqrt(1 - a^2) as sqrt(-expm1(2 log a)): no cancellation where a is close to 1
      inp[k] = sqrtf(-expm1f(2.f * log_a)) * sigmoid_full(inp[k] + bias_i) * uv;
      y[k] = apply_act(y[k], TNX_ACT_GELU_NEW) * a.out_scale;
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= n) break;
      s = decay[k] * s + inp[k];
      out[(size_t)(first + i0 + k) * a.out_ld + c] = from_f32<T>(s * y[k]);
    }
  }
  mine[(size_t)((p0 + n - 1) & 1) * a.channels + c] = s;
}

// ------------------------------------------------------------------------------------------ runs cut into parts

constexpr int SEGMENTS = 16;          // waves a block
constexpr int SEG_MIN = 4;            // tokens a part at least: shorter runs use fewer parts
// A block takes CH = 16 channels of a run and cuts its tokens into 1024 / CH = 64 parts, four a wave (a lane's
// neighbours in memory are 16 channels, 64 bytes): 2,048 channels of one prompt make 128 blocks.

// What a recurrence S <- a S + b with a result S * f needs of a token: `Gate::ab(t, a, b)`, `Gate::factor(t)`.
struct MinGruGate {
  const float* proj;
  int ld, inner, c;
  float out_scale;
  __device__ __forceinline__ void ab(size_t t, float& a, float& b) const {
    const float* row = proj + t * ld;
    const float z = sigmoid_full(row[c]);
    const float u = row[inner + c];
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_full(u);
    a = 1.f - z;
    b = z * cand;
  }
  __device__ __forceinline__ float factor(size_t t) const {
    const float g = proj[t * ld + 2 * inner + c];
    return g * sigmoid_full(g) * out_scale;
  }
};

struct LinearGate {
  const float* gates;
  const float* u;
  const float* y;
  long long y_ld;
  size_t gates_ld;
  int channels, c, at_r, at_i;
  float bias_r, bias_i, rate, out_scale;
  __device__ __forceinline__ void ab(size_t t, float& a, float& b) const {
    const float log_a = rate * sigmoid_full(gates[t * gates_ld + at_r] + bias_r);
    a = expf(log_a);
    b = sqrtf(-expm1f(2.f * log_a)) * sigmoid_full(gates[t * gates_ld + at_i] + bias_i) * u[t * channels + c];
  }
  __device__ __forceinline__ float factor(size_t t) const {
    return apply_act(y[t * y_ld + c], TNX_ACT_GELU_NEW) * out_scale;
  }
};

// Tokens [from, to) of the step from state `s`; `prod` gathers the product of the a. WRITE: the results go out.
template <bool WRITE, typename T, typename Gate>
__device__ __forceinline__ void walk_part(const Gate& gate, int from, int to, float& s, float& prod, T* out,
                                          long long out_ld, int c) {
  for (int i0 = from; i0 < to; i0 += AHEAD) {
    float a[AHEAD], b[AHEAD], f[AHEAD];
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= to) break;
      gate.ab((size_t)(i0 + k), a[k], b[k]);
      if (WRITE) f[k] = gate.factor((size_t)(i0 + k));
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      if (i0 + k >= to) break;
      s = a[k] * s + b[k];
      if (WRITE)
        out[(size_t)(i0 + k) * out_ld + c] = from_f32<T>(s * f[k]);
      else
        prod *= a[k];
    }
  }
}

// A block: 64 channels of one run, wave w the w-th part of its tokens. `carried` as above.
template <int CH, typename T, typename Gate>
__device__ __forceinline__ void recurrence_by_segments(const Gate& gate, bool live, int c, int channels, int first, int n,
                                                       int p0, float* mine, T* out, long long out_ld) {
  constexpr int NSEG = 64 * SEGMENTS / CH;
  __shared__ float part_a[NSEG][CH], part_b[NSEG][CH];
  const int lane = threadIdx.x % CH, seg = threadIdx.x / CH;
  const int parts = min(NSEG, max(1, n / SEG_MIN));
  const int len = (n + parts - 1) / parts;
  const int from = first + min(n, seg * len), to = first + min(n, (seg + 1) * len);
  const float s0 = live && p0 > 0 ? mine[(size_t)((p0 - 1) & 1) * channels + c] : 0.f;
  float s = 0.f, prod = 1.f;
  if (live && seg < parts - 1) walk_part<false, T>(gate, from, to, s, prod, out, out_ld, c);   // the last part's is not needed
  part_a[seg][lane] = prod;
  part_b[seg][lane] = s;
  __syncthreads();
  if (!live || from >= to) return;
  s = s0;
  for (int k = 0; k < seg; ++k) s = part_a[k][lane] * s + part_b[k][lane];
  walk_part<true, T>(gate, from, to, s, prod, out, out_ld, c);
  if (to == first + n) mine[(size_t)((p0 + n - 1) & 1) * channels + c] = s;
}

template <int CH, typename T>
__global__ void __launch_bounds__(64 * SEGMENTS)
min_gru_by_segments_kernel(const float* __restrict__ proj, int ld, int inner, const int* __restrict__ positions,
                           const int* __restrict__ run_start, const int* __restrict__ slots, float* __restrict__ carried,
                           T* __restrict__ out, long long out_ld, float out_scale) {
  const int r = blockIdx.y, c = blockIdx.x * CH + threadIdx.x % CH;
  const int first = run_start[r], n = run_start[r + 1] - first;
  if (n <= 0) return;
  const bool live = c < inner;
  const MinGruGate gate{proj, ld, inner, live ? c : 0, out_scale};
  recurrence_by_segments<CH, T>(gate, live, c, inner, first, n, positions[first], carried + (size_t)slots[r] * 2 * inner, out,
                            out_ld);
}

template <int CH, typename T>
__global__ void __launch_bounds__(64 * SEGMENTS) gated_linear_recurrence_by_segments_kernel(RecurrenceArgs a) {
  const int r = blockIdx.y, c = blockIdx.x * CH + threadIdx.x % CH;
  const int first = a.run_start[r], n = a.run_start[r + 1] - first;
  if (n <= 0) return;
  const bool live = c < a.channels;
  const int cc = live ? c : 0;
  const int b = cc / a.w, j = cc - b * a.w;
  const int at_r = b * 2 * a.w + j, at_i = at_r + a.w;
  const LinearGate gate{a.gates, a.u, a.y, a.y_ld, (size_t)2 * a.channels, a.channels, cc, at_r, at_i,
                        a.gate_bias[at_r], a.gate_bias[at_i], a.rate[cc], a.out_scale};
  recurrence_by_segments<CH, T>(gate, live, c, a.channels, first, n, a.positions[first],
                            a.carried + (size_t)a.slots[r] * 2 * a.channels, (T*)a.out, a.out_ld);
}

}  // namespace

extern "C" int tnx_min_gru(const float* proj, int ld, int inner, const int* positions, const int* run_start,
                           const int* slots, float* carried, void* out, long long out_ld, int out_dtype, float out_scale,
                           int tokens, int runs, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && runs >= 0 && inner > 0 && ld >= 3 * inner && out_ld >= inner, "min_gru: bad sizes");
  TNX_REQUIRE(out_dtype == TNX_F32 || out_dtype == TNX_BF16, "min_gru: dtype %d", out_dtype);
  if (tokens == 0 || runs == 0) return 0;
  if (tokens > runs) {      // some run has several tokens
    const dim3 by_parts((inner + 15) / 16, runs);
#define LAUNCH_MIN_GRU(CH, T)                                                                                          \
  min_gru_by_segments_kernel<CH, T><<<by_parts, 64 * SEGMENTS, 0, stream>>>(proj, ld, inner, positions, run_start, slots, \
                                                                            carried, (T*)out, out_ld, out_scale)
    if (out_dtype == TNX_F32) {
      LAUNCH_MIN_GRU(16, float);
    } else {
      LAUNCH_MIN_GRU(16, bf16_t);
    }
#undef LAUNCH_MIN_GRU
    TNX_CHECK_LAUNCH("min_gru_by_segments");
    return 0;
  }
  const dim3 grid((inner + 255) / 256, runs);
  if (out_dtype == TNX_F32)
    min_gru_kernel<float><<<grid, 256, 0, stream>>>(proj, ld, inner, positions, run_start, slots, carried, (float*)out,
                                                    out_ld, out_scale);
  else
    min_gru_kernel<bf16_t><<<grid, 256, 0, stream>>>(proj, ld, inner, positions, run_start, slots, carried, (bf16_t*)out,
                                                     out_ld, out_scale);
  TNX_CHECK_LAUNCH("min_gru");
  return 0;
}

extern "C" int tnx_channel_conv(const float* x, long long ld, const float* w, const float* bias, float* state, int taps,
                                const int* positions, const int* token_request, const int* run_start, const int* slots,
                                float* out, void* out_cd, int cd_dtype, int tokens, int channels, int runs,
                                hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && channels > 0 && taps >= 1 && runs >= 0 && ld >= channels, "channel_conv: bad sizes");
  TNX_REQUIRE(taps == 1 || state, "channel_conv: %d taps need the requests' state", taps);
  if (tokens == 0) return 0;
  if (out_cd && cd_dtype == TNX_BF16)
    channel_conv_kernel<bf16_t><<<tokens, 256, 0, stream>>>(x, ld, w, bias, taps > 1 ? state : nullptr, taps, positions,
                                                            token_request, run_start, slots, out, (bf16_t*)out_cd, channels);
  else
    channel_conv_kernel<float><<<tokens, 256, 0, stream>>>(x, ld, w, bias, taps > 1 ? state : nullptr, taps, positions,
                                                           token_request, run_start, slots, out, nullptr, channels);
  TNX_CHECK_LAUNCH("channel_conv");
  if (taps > 1) {
    channel_state_kernel<<<dim3((channels + 255) / 256, runs), 256, 0, stream>>>(x, ld, state, taps, positions, run_start,
                                                                                slots, channels);
    TNX_CHECK_LAUNCH("channel_state");
  }
  return 0;
}

extern "C" int tnx_gated_linear_recurrence(const float* gates, const float* gate_bias, const float* u, const float* y,
                                           long long y_ld, const float* rate, const int* positions, const int* run_start,
                                           const int* slots, float* carried, void* out, long long out_ld, int out_dtype,
                                           float out_scale, int tokens, int runs, int blocks, int w, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && runs >= 0 && blocks > 0 && w > 0, "gated_linear_recurrence: bad sizes");
  const int channels = blocks * w;
  TNX_REQUIRE(y_ld >= channels && out_ld >= channels, "gated_linear_recurrence: rows shorter than %d", channels);
  TNX_REQUIRE(out_dtype == TNX_F32 || out_dtype == TNX_BF16, "gated_linear_recurrence: dtype %d", out_dtype);
  if (tokens == 0 || runs == 0) return 0;
  RecurrenceArgs a{gates, gate_bias, u, y, y_ld, rate, positions, run_start, slots, carried, out, out_ld, out_scale,
                   channels, w};
  if (tokens > runs) {      // some run has several tokens
    const dim3 by_parts((channels + 15) / 16, runs);
    if (out_dtype == TNX_F32)
      gated_linear_recurrence_by_segments_kernel<16, float><<<by_parts, 64 * SEGMENTS, 0, stream>>>(a);
    else
      gated_linear_recurrence_by_segments_kernel<16, bf16_t><<<by_parts, 64 * SEGMENTS, 0, stream>>>(a);
    TNX_CHECK_LAUNCH("gated_linear_recurrence_by_segments");
    return 0;
  }
  const dim3 grid((channels + 255) / 256, runs);
  if (out_dtype == TNX_F32)
    gated_linear_recurrence_kernel<float><<<grid, 256, 0, stream>>>(a);
  else
    gated_linear_recurrence_kernel<bf16_t><<<grid, 256, 0, stream>>>(a);
  TNX_CHECK_LAUNCH("gated_linear_recurrence");
  return 0;
}
