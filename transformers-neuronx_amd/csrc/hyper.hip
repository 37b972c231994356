// Several copies of the residual stream (hyper-connections), and the sines and cosines that start the stream.
//   add_sinusoid   out = src * scale + (sin, cos)(position * freqs[i]) at elements 2i, 2i + 1; float32 angles
//   hyper_step     joins a sublayer's result to the copies, x_b <- sum_a mix[a, b] x_a + out[b] y, then makes the
//                  next sublayer's input, norm(sum_a in[a] x_a), and / or the sum of the copies: one launch
// Copies, sums and norms are float32. One block a token; a token's elements of all copies pass through the
// block's registers once.
#include "common.h"

TNX_DEFINE_ERROR_API

namespace {

constexpr int MAX_COPIES = 8;

__global__ void __launch_bounds__(256)
add_sinusoid_kernel(const void* __restrict__ src, int src_dtype, const int* __restrict__ positions,
                    const float* __restrict__ freqs, float* __restrict__ out, void* __restrict__ out_cd, int cd_dtype,
                    int width, float scale) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const size_t base = (size_t)t * width;
  for (int i = threadIdx.x; i < width / 2; i += 256) {
    float s, c;
    sincosf(pos * freqs[i], &s, &c);
    const float a = load_any(src, src_dtype, base + 2 * i) * scale + s;
    const float b = load_any(src, src_dtype, base + 2 * i + 1) * scale + c;
    out[base + 2 * i] = a;
    out[base + 2 * i + 1] = b;
    if (out_cd) {
      store_any(out_cd, cd_dtype, base + 2 * i, a);
      store_any(out_cd, cd_dtype, base + 2 * i + 1, b);
    }
  }
}

struct HyperArgs {
  float* copies;            // [s, T, width]
  const float* y;           // [T, width] or null: nothing to join
  const float* mix;         // [s, s], indexed [from, to]
  const float* out_w;       // [s]
  const float* read;        // [s] or null: no input is made
  const float* norm_w;      // [width]
  float eps;
  float* h32;               // [T, width] or null
  void* hcd;                // [T, width] or null
  int cd_dtype;
  float* sum;               // [T, width] or null: the sum of the copies
  int s, tokens, width;
};

// PER elements a thread (width <= 256 * PER): the weighted sum u stays in registers between the pass that makes
// it and the pass that scales it.
template <int PER>
__global__ void __launch_bounds__(256) hyper_step_kernel(HyperArgs a) {
  __shared__ float scratch[4];
  __shared__ float w_mix[MAX_COPIES * MAX_COPIES], w_out[MAX_COPIES], w_read[MAX_COPIES];
  const int t = blockIdx.x, s = a.s;
  if (threadIdx.x < s * s && a.y) w_mix[threadIdx.x] = a.mix[threadIdx.x];
  if (threadIdx.x < s) {
    if (a.y) w_out[threadIdx.x] = a.out_w[threadIdx.x];
    if (a.read) w_read[threadIdx.x] = a.read[threadIdx.x];
  }
  __syncthreads();
  const size_t row = (size_t)t * a.width, plane = (size_t)a.tokens * a.width;
  float u[PER];
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int d = threadIdx.x + 256 * k;
    u[k] = 0.f;
    if (d >= a.width) continue;
    float x[MAX_COPIES];
    for (int c = 0; c < s; ++c) x[c] = a.copies[c * plane + row + d];
    if (a.y) {
      const float yv = a.y[row + d];
      float nx[MAX_COPIES];
      for (int b = 0; b < s; ++b) {
        float v = 0.f;
        for (int c = 0; c < s; ++c) v = fmaf(w_mix[c * s + b], x[c], v);
        nx[b] = fmaf(w_out[b], yv, v);
      }
      for (int b = 0; b < s; ++b) {
        x[b] = nx[b];
        a.copies[b * plane + row + d] = nx[b];
      }
    }
    if (a.sum) {
      float v = 0.f;
      for (int c = 0; c < s; ++c) v += x[c];
      a.sum[row + d] = v;
    }
    if (a.read) {
      float v = 0.f;
      for (int c = 0; c < s; ++c) v = fmaf(w_read[c], x[c], v);
      u[k] = v;
      sq = fmaf(v, v, sq);
    }
  }
  if (!a.read) return;
  const float r = 1.f / sqrtf(block_sum<4>(sq, scratch) / (float)a.width + a.eps);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int d = threadIdx.x + 256 * k;
    if (d >= a.width) continue;
    const float h = u[k] * r * a.norm_w[d];
    if (a.h32) a.h32[row + d] = h;
    if (a.hcd) store_any(a.hcd, a.cd_dtype, row + d, h);
  }
}

}  // namespace

extern "C" int tnx_add_sinusoid(const void* src, int src_dtype, const int* positions, const float* freqs, float* out,
                                void* out_cd, int cd_dtype, int tokens, int width, float scale, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && width % 2 == 0, "add_sinusoid: the width must be even, got %d", width);
  if (tokens == 0) return 0;
  add_sinusoid_kernel<<<tokens, 256, 0, stream>>>(src, src_dtype, positions, freqs, out, out_cd, cd_dtype, width, scale);
  TNX_CHECK_LAUNCH("add_sinusoid");
  return 0;
}

extern "C" int tnx_hyper_step(float* copies, const float* y, const float* mix, const float* out_w, const float* read,
                              const float* norm_w, float eps, float* h32, void* hcd, int cd_dtype, float* sum, int s,
                              int tokens, int width, hipStream_t stream) {
  TNX_REQUIRE(s >= 1 && s <= MAX_COPIES, "hyper_step: %d copies of the stream, at most %d", s, MAX_COPIES);
  TNX_REQUIRE(tokens >= 0 && width > 0 && width <= 256 * 64, "hyper_step: width %d", width);
  TNX_REQUIRE(!y || (mix && out_w), "hyper_step: a result to join needs its weights");
  TNX_REQUIRE(!read || (norm_w && (h32 || hcd)), "hyper_step: an input needs its norm and a place");
  if (tokens == 0) return 0;
  HyperArgs a{copies, y, mix, out_w, read, norm_w, eps, h32, hcd, cd_dtype, sum, s, tokens, width};
  const int per = (width + 255) / 256;
  if (per <= 2)
    hyper_step_kernel<2><<<tokens, 256, 0, stream>>>(a);
  else if (per <= 8)
    hyper_step_kernel<8><<<tokens, 256, 0, stream>>>(a);
  else if (per <= 32)
    hyper_step_kernel<32><<<tokens, 256, 0, stream>>>(a);
  else
    hyper_step_kernel<64><<<tokens, 256, 0, stream>>>(a);
  TNX_CHECK_LAUNCH("hyper_step");
  return 0;
}
