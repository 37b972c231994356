// Several copies of the residual stream (hyper-connections), and the sines and cosines that start the stream.
//   add_sinusoid   out = src * scale + (sin, cos)(position * freqs[i]) at elements 2i, 2i + 1; float32 angles
//   hyper_step     joins a sublayer's result to the copies, x_b <- sum_a mix[a, b] x_a + out[b] y, then makes the
//                  next sublayer's input, norm(sum_a in[a] x_a), and / or the sum of the copies: one launch
// Copies, sums and norms are float32. One block a token; a token's elements of all copies pass through the
// block's registers once. The number of copies is a template parameter (1 to 8).
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

// S copies, PER groups of VEC consecutive elements a thread (width <= 256 * PER * VEC): every loop over the copies
// is unrolled, so that a token's elements and the weighted sum u stay in registers between the pass that makes
// them and the pass that scales them. VEC = 4 reads and writes 16 bytes at a time (widths that are multiples of 4).
template <int S, int PER, int VEC>
__global__ void __launch_bounds__(256) hyper_step_kernel(HyperArgs a) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  float w_mix[S][S], w_out[S], w_read[S];
#pragma unroll
  for (int c = 0; c < S; ++c) {
    w_out[c] = a.y ? a.out_w[c] : 0.f;
    w_read[c] = a.read ? a.read[c] : 0.f;
#pragma unroll
    for (int b = 0; b < S; ++b) w_mix[c][b] = a.y ? a.mix[c * S + b] : 0.f;
  }
  const size_t row = (size_t)t * a.width, plane = (size_t)a.tokens * a.width;
  float u[PER][VEC];
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int d = (threadIdx.x + 256 * k) * VEC;
#pragma unroll
    for (int e = 0; e < VEC; ++e) u[k][e] = 0.f;
    if (d >= a.width) continue;
    float x[S][VEC], yv[VEC];
#pragma unroll
    for (int c = 0; c < S; ++c) {
      if (VEC == 4) {
        const f32x4 v = *(const f32x4*)(a.copies + c * plane + row + d);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[c][e] = v[e];
      } else {
        x[c][0] = a.copies[c * plane + row + d];
      }
    }
    if (a.y) {
      if (VEC == 4) {
        const f32x4 v = *(const f32x4*)(a.y + row + d);
#pragma unroll
        for (int e = 0; e < VEC; ++e) yv[e] = v[e];
      } else {
        yv[0] = a.y[row + d];
      }
      float nx[S][VEC];
#pragma unroll
      for (int b = 0; b < S; ++b)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float v = 0.f;
#pragma unroll
          for (int c = 0; c < S; ++c) v = fmaf(w_mix[c][b], x[c][e], v);
          nx[b][e] = fmaf(w_out[b], yv[e], v);
        }
#pragma unroll
      for (int b = 0; b < S; ++b) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[b][e] = nx[b][e];
        if (VEC == 4)
          *(f32x4*)(a.copies + b * plane + row + d) = (f32x4){nx[b][0], nx[b][VEC > 1 ? 1 : 0], nx[b][VEC > 2 ? 2 : 0], nx[b][VEC > 3 ? 3 : 0]};
        else
          a.copies[b * plane + row + d] = nx[b][0];
      }
    }
    if (a.sum) {
      float v[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        v[e] = 0.f;
#pragma unroll
        for (int c = 0; c < S; ++c) v[e] += x[c][e];
      }
      if (VEC == 4)
        *(f32x4*)(a.sum + row + d) = (f32x4){v[0], v[VEC > 1 ? 1 : 0], v[VEC > 2 ? 2 : 0], v[VEC > 3 ? 3 : 0]};
      else
        a.sum[row + d] = v[0];
    }
    if (a.read) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float v = 0.f;
#pragma unroll
        for (int c = 0; c < S; ++c) v = fmaf(w_read[c], x[c][e], v);
        u[k][e] = v;
        sq = fmaf(v, v, sq);
      }
    }
  }
  if (!a.read) return;
  const float r = 1.f / sqrtf(block_sum<4>(sq, scratch) / (float)a.width + a.eps);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int d = (threadIdx.x + 256 * k) * VEC;
    if (d >= a.width) continue;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float h = u[k][e] * r * a.norm_w[d + e];
      if (a.h32) a.h32[row + d + e] = h;
      if (a.hcd) store_any(a.hcd, a.cd_dtype, row + d + e, h);
    }
  }
}

template <int S>
void launch_hyper_step(const HyperArgs& a, hipStream_t stream) {
  const bool aligned = (((uintptr_t)a.copies | (uintptr_t)a.y | (uintptr_t)a.sum) & 15) == 0;
  const bool by_four = aligned && a.width % 4 == 0 && a.width <= 256 * 16 * 4;
  const int per = by_four ? (a.width / 4 + 255) / 256 : (a.width + 255) / 256;
  if (by_four) {
    if (per <= 1)
      hyper_step_kernel<S, 1, 4><<<a.tokens, 256, 0, stream>>>(a);
    else if (per <= 4)
      hyper_step_kernel<S, 4, 4><<<a.tokens, 256, 0, stream>>>(a);
    else
      hyper_step_kernel<S, 16, 4><<<a.tokens, 256, 0, stream>>>(a);
  } else if (per <= 4) {
    hyper_step_kernel<S, 4, 1><<<a.tokens, 256, 0, stream>>>(a);
  } else if (per <= 16) {
    hyper_step_kernel<S, 16, 1><<<a.tokens, 256, 0, stream>>>(a);
  } else {
    hyper_step_kernel<S, 64, 1><<<a.tokens, 256, 0, stream>>>(a);
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
  switch (s) {
    case 1: launch_hyper_step<1>(a, stream); break;
    case 2: launch_hyper_step<2>(a, stream); break;
    case 3: launch_hyper_step<3>(a, stream); break;
    case 4: launch_hyper_step<4>(a, stream); break;
    case 5: launch_hyper_step<5>(a, stream); break;
    case 6: launch_hyper_step<6>(a, stream); break;
    case 7: launch_hyper_step<7>(a, stream); break;
    default: launch_hyper_step<8>(a, stream); break;
  }
  TNX_CHECK_LAUNCH("hyper_step");
  return 0;
}
