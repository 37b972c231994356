// Between the query/key/value projection and attention, for mixers whose queries and keys are normed over the
// whole projection, turned by halves, or whose values are blended or of a size of their own: one launch takes the
// float32 projections of a step's tokens to the queries (compute dtype) and to the tokens' places in the cache.
// Everything is float32 until the one rounding at the store.
#include "common.h"

TNX_DEFINE_ERROR_API

namespace {

struct PrepareArgs {
  const float* proj;        // [T, ld]: queries, keys, values side by side, bias added
  int ld;
  const float* q_weight;    // [H n] or null: no norm
  const float* k_weight;    // [G n]
  float eps;
  const float* freqs;       // [half] or null: no turning
  int half;
  int interleaved;
  const int* positions;     // [T]
  float scale;
  const float* mix_weight;  // [1] or null
  const float* first;       // [T, first_ld] or null: no blending
  long long first_ld;
  const int* token_page;    // [T]
  const int* token_offset;  // [T]
  void* q_out;              // [T, H D]
  void* k_pages;            // [pages, G, page, D]
  void* v_pages;            // [pages, G, D, page]
  long long page_stride;    // elements from one page to the next
  int num_pages, page_size;
  int heads, groups, n, v, d;
  int per_head;             // every head is normed by itself (the weights, if any, still one a projection element)
  int values_at;            // the column of a row where the values begin (behind the keys, or the keys' own)
  const float* head_scale;  // [H] or null: a query head's elements times its number, beside `scale`
};

// Element `e` of head `head` of a normed projection, turned by the token's position. `x` points at the
// projection's first head, `w` at its norm weight (or null), `r` is the factor of the norm.
__device__ __forceinline__ float turned(const float* x, const float* w, float r, int head, int e, const PrepareArgs& a,
                                        const float* cosines, const float* sines) {
  const int at = head * a.n + e;
  const float own = x[at] * r * (w ? w[at] : 1.f);
  if (a.freqs == nullptr || e >= 2 * a.half) return own;
  int i, other;
  bool first;
  if (a.interleaved) {
    i = e >> 1;
    first = (e & 1) == 0;
    other = first ? e + 1 : e - 1;
  } else {
    first = e < a.half;
    i = first ? e : e - a.half;
    other = first ? e + a.half : e - a.half;
  }
  const int oat = head * a.n + other;
  const float mate = x[oat] * r * (w ? w[oat] : 1.f);
  const float s = sines[i], c = cosines[i];
  // the pair (u, v) becomes (u c - v s, v c + u s)
  return first ? own * c - mate * s : own * c + mate * s;
}

// grid: (tokens, 3): a block takes a token's queries, its keys or its values; each of the three needs nothing of
// the other two.
template <typename T>
__global__ void __launch_bounds__(256) qkv_prepare_kernel(PrepareArgs a) {
  __shared__ float scratch[4];
  __shared__ float cosines[128], sines[128];       // of the token's angles, once for all heads
  const int t = blockIdx.x, part = blockIdx.y;
  const float* row = a.proj + (size_t)t * a.ld;
  const int nq = a.heads * a.n, nk = a.groups * a.n;
  const int page = a.token_page[t], off = a.token_offset[t];
  if (part > 0 && (page < 0 || page >= a.num_pages)) return;       // the host checks that every token has a page
  if (part == 2) {
    const float* xv = row + a.values_at;
    T* vp = (T*)a.v_pages + (size_t)page * a.page_stride;
    const float lam = a.first != nullptr ? a.mix_weight[0] : 0.f;
    const float* first = a.first != nullptr ? a.first + (size_t)t * a.first_ld : nullptr;
    for (int i = threadIdx.x; i < a.groups * a.d; i += 256) {
      const int g = i / a.d, e = i - g * a.d;
      float val = 0.f;
      if (e < a.v) {
        val = xv[g * a.v + e];
        if (first != nullptr) val = (1.f - lam) * val + lam * first[g * a.v + e];
      }
      vp[((size_t)g * a.d + e) * a.page_size + off] = from_f32<T>(val);
    }
    return;
  }
  if (a.freqs != nullptr) {
    const float pos = (float)a.positions[t];
    for (int i = threadIdx.x; i < a.half; i += 256) sincosf(pos * a.freqs[i], &sines[i], &cosines[i]);
  }
  // queries (part 0) or keys (part 1): the norm over the whole projection, then head by head
  const float* x = part == 0 ? row : row + nq;
  const float* w = part == 0 ? a.q_weight : a.k_weight;
  const int count = part == 0 ? nq : nk, heads = part == 0 ? a.heads : a.groups;
  if (a.per_head) {
    // a wave a head: the head's sum of squares over its lanes, then its elements
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();       // the token's sines and cosines are there
    T* kp = part == 1 ? (T*)a.k_pages + (size_t)page * a.page_stride : nullptr;
    T* q_out = part == 0 ? (T*)a.q_out + (size_t)t * a.heads * a.d : nullptr;
    for (int head = wave; head < heads; head += 4) {
      float s = 0.f;
      for (int e = lane; e < a.n; e += 64) s += x[head * a.n + e] * x[head * a.n + e];
      const float r = 1.f / sqrtf(wave_sum(s) / (float)a.n + a.eps);
      for (int e = lane; e < a.d; e += 64) {
        const float val = e < a.n ? turned(x, w, r, head, e, a, cosines, sines) : 0.f;
        if (part == 0)
          q_out[head * a.d + e] = from_f32<T>(val * (a.head_scale ? a.scale * a.head_scale[head] : a.scale));
        else
          kp[((size_t)head * a.page_size + off) * a.d + e] = from_f32<T>(val);
      }
    }
    return;
  }
  float norm = 1.f;
  if (w != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < count; i += 256) s += x[i] * x[i];
    s = block_sum<4>(s, scratch);
    norm = 1.f / sqrtf(s / (float)count + a.eps);
  }
  __syncthreads();
  if (part == 0) {
    T* q_out = (T*)a.q_out + (size_t)t * a.heads * a.d;
    for (int i = threadIdx.x; i < heads * a.d; i += 256) {
      const int head = i / a.d, e = i - head * a.d;
      q_out[i] = from_f32<T>(e < a.n ? turned(x, w, norm, head, e, a, cosines, sines) *
                                           (a.head_scale ? a.scale * a.head_scale[head] : a.scale)
                                     : 0.f);
    }
  } else {
    T* kp = (T*)a.k_pages + (size_t)page * a.page_stride;
    for (int i = threadIdx.x; i < heads * a.d; i += 256) {
      const int g = i / a.d, e = i - g * a.d;
      kp[((size_t)g * a.page_size + off) * a.d + e] = from_f32<T>(e < a.n ? turned(x, w, norm, g, e, a, cosines, sines) : 0.f);
    }
  }
}

}  // namespace

extern "C" int tnx_qkv_prepare(const float* proj, int ld, const float* q_weight, const float* k_weight, float eps,
                               const float* freqs, int half, int interleaved, const int* positions, float scale,
                               const float* mix_weight, const float* first, long long first_ld, const int* token_page,
                               const int* token_offset, void* q_out, void* k_pages, void* v_pages, long long page_stride,
                               int num_pages, int page_size, int dtype, int tokens, int heads, int groups, int n, int v,
                               int d, int per_head, int values_at, const float* head_scale, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && heads > 0 && groups > 0 && n > 0 && v > 0, "qkv_prepare: bad sizes");
  TNX_REQUIRE(d >= n && d >= v, "qkv_prepare: cached heads of %d elements do not hold %d and %d", d, n, v);
  if (values_at < 0) values_at = heads * n + groups * n;
  TNX_REQUIRE(ld >= heads * n + groups * n && ld >= values_at + groups * v,
              "qkv_prepare: rows of %d elements do not hold the keys and the values at column %d", ld, values_at);
  TNX_REQUIRE(freqs == nullptr || (2 * half <= n && half <= 128), "qkv_prepare: %d turned elements in heads of %d", 2 * half, n);
  TNX_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qkv_prepare: both norm weights or none");
  TNX_REQUIRE((first == nullptr) || (mix_weight != nullptr && first_ld >= groups * v), "qkv_prepare: blending needs its weight");
  TNX_REQUIRE(page_stride >= (long long)groups * d * page_size, "qkv_prepare: pages closer than a page's elements");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "qkv_prepare: dtype %d", dtype);
  if (tokens == 0) return 0;
  PrepareArgs a{proj, ld, q_weight, k_weight, eps, freqs, half, interleaved, positions, scale, mix_weight, first, first_ld,
                token_page, token_offset, q_out, k_pages, v_pages, page_stride, num_pages, page_size, heads, groups, n, v, d,
                per_head, values_at, head_scale};
  if (dtype == TNX_F32)
    qkv_prepare_kernel<float><<<dim3(tokens, 3), 256, 0, stream>>>(a);
  else
    qkv_prepare_kernel<bf16_t><<<dim3(tokens, 3), 256, 0, stream>>>(a);
  TNX_CHECK_LAUNCH("qkv_prepare");
  return 0;
}
