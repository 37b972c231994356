// Attention whose scores or mask are not the plain ones: a cap on the scores (c tanh(s / c)), a learned bias by
// the distance between query and key, visibility inside chunks of the sequence, and a gate on the result.
//   attention_scored_any   one wave per (token, head), any dtype, any head size in steps of 16: the float32 path,
//                          decoding, and whatever the matrix-unit kernel does not take
// Scores, the cap, the bias and the softmax are float32. The bias comes as a table by distance, `[heads, D + 1]`,
// read at min(i - j, D): the buckets of the distances are worked out on the host, once a model.
#include "common.h"

TNX_DEFINE_ERROR_API

namespace {

struct ScoredArgs {
  const void* q;            // [T, H d], scaled
  const void* k_pages;      // [pages, G, page, d]
  const void* v_pages;      // [pages, G, d, page]
  const int* positions;
  const int* token_request;
  const int* table;
  int table_width, page_size, num_pages;
  void* out;                // [T, out_ld]
  long long out_ld;
  float out_scale;
  const float* gate;        // [T, gate_ld] or null: pre-activations of the gate, H * value_size a token
  long long gate_ld;
  const float* bias;        // [H, far + 1] or null
  int far;
  float softcap;            // 0: none
  int window, chunk;        // 0: none
  int tokens, num_heads, num_kv, head_size, value_size, page_pad;
};

__device__ __forceinline__ float exp_for(float x, float) { return expf(x); }
__device__ __forceinline__ float exp_for(float x, bf16_t) { return __expf(x); }

// Keys are taken 64 at a time, one a lane; the softmax is the running kind (maximum and sum carried in float32,
// earlier sums rescaled); the value sum is kept per lane for the head's elements lane, lane + 64, ... Keys
// before the first visible one are not read.
template <typename T>
__global__ void __launch_bounds__(256) attention_scored_any_kernel(ScoredArgs a) {
  __shared__ float qs[4][256];
  const T* q = (const T*)a.q;
  const T* k_pages = (const T*)a.k_pages;
  const T* v_pages = (const T*)a.v_pages;
  const int head_size = a.head_size, page_size = a.page_size;
  const size_t page_stride = (size_t)a.num_kv * page_size * head_size + a.page_pad;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long idx = (long long)blockIdx.x * 4 + wave;
  const bool active = idx < (long long)a.tokens * a.num_heads;
  const int t = active ? (int)(idx / a.num_heads) : 0;
  const int h = active ? (int)(idx % a.num_heads) : 0;
  const int kvh = h / (a.num_heads / a.num_kv);
  const int nq = a.num_heads * head_size;
  for (int d = lane; d < head_size; d += 64) qs[wave][d] = to_f32(q[(size_t)t * nq + h * head_size + d]);
  __syncthreads();
  if (!active) return;

  const int pos = a.positions[t];
  const int* tab = a.table + (size_t)a.token_request[t] * a.table_width;
  int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  if (a.chunk > 0) lo = max(lo, pos - pos % a.chunk);
  const float* bias = a.bias ? a.bias + (size_t)h * (a.far + 1) : nullptr;
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};

  for (int c = (lo / 64) * 64; c <= pos; c += 64) {
    const int key = c + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = tab[key / page_size];
      if (page >= 0 && page < a.num_pages) {
        const T* kp = k_pages + (size_t)page * page_stride + ((size_t)kvh * page_size + key % page_size) * head_size;
        float dot = 0.f;
        for (int d = 0; d < head_size; d += 4) {
          dot = fmaf(qs[wave][d], to_f32(kp[d]), dot);
          dot = fmaf(qs[wave][d + 1], to_f32(kp[d + 1]), dot);
          dot = fmaf(qs[wave][d + 2], to_f32(kp[d + 2]), dot);
          dot = fmaf(qs[wave][d + 3], to_f32(kp[d + 3]), dot);
        }
        if (cap > 0.f) dot = cap * tanhf(dot * inv_cap);
        if (bias) dot += bias[min(pos - key, a.far)];
        s = dot;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid && s > -INFINITY ? exp_for(s - m_new, T()) : 0.f;
    const float alpha = m_new > -INFINITY ? exp_for(m - m_new, T()) : 1.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] *= alpha;
    // values: 16 keys at a time lie in one page (page sizes are multiples of 16)
#pragma unroll
    for (int grp = 0; grp < 4; ++grp) {
      const int key0 = c + 16 * grp;
      if (key0 > pos || key0 + 15 < lo) continue;
      const int page = tab[key0 / page_size];
      if (page < 0 || page >= a.num_pages) continue;
      const int off0 = key0 % page_size;
      const T* vbase = v_pages + (size_t)page * page_stride + (size_t)kvh * head_size * page_size + off0;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float pj = __shfl(p, 16 * grp + j, 64);
        const int kj = key0 + j;
        if (kj < lo || kj > pos) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int d = lane + 64 * e;
          if (d < head_size) acc[e] = fmaf(pj, to_f32(vbase[(size_t)d * page_size + j]), acc[e]);
        }
      }
    }
  }
  const float inv = a.out_scale / l;
  T* out = (T*)a.out + (size_t)t * a.out_ld + (size_t)h * head_size;
  const float* gate = a.gate ? a.gate + (size_t)t * a.gate_ld + (size_t)h * a.value_size : nullptr;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int d = lane + 64 * e;
    if (d >= head_size) continue;
    float v = acc[e] * inv;
    if (gate && d < a.value_size) v *= 1.f / (1.f + expf(-gate[d]));
    out[d] = from_f32<T>(v);
  }
}

}  // namespace

extern "C" int tnx_attention_scored(const void* q, int dtype, const void* k_pages, const void* v_pages,
                                    const int* positions, const int* token_request, const int* table, int table_width,
                                    int page_size, int num_pages, void* out, long long out_ld, float out_scale,
                                    const float* gate, long long gate_ld, const float* bias, int far, float softcap,
                                    int window, int chunk, int tokens, int num_heads, int num_kv, int head_size,
                                    int value_size, int page_pad, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention_scored: bad head counts");
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention_scored: bad distance between pages");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention_scored: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(value_size > 0 && value_size <= head_size, "attention_scored: values of %d in heads of %d", value_size, head_size);
  TNX_REQUIRE(page_size % 16 == 0 && page_size > 0, "attention_scored: page size %d is not a multiple of 16", page_size);
  TNX_REQUIRE(out_ld >= (long long)num_heads * head_size, "attention_scored: result rows of %lld elements", out_ld);
  TNX_REQUIRE(!gate || gate_ld >= (long long)num_heads * value_size, "attention_scored: gate rows of %lld elements", gate_ld);
  TNX_REQUIRE(!bias || far >= 0, "attention_scored: a bias table needs its last distance");
  TNX_REQUIRE(window >= 0 && chunk >= 0 && softcap >= 0.f, "attention_scored: bad window, chunk or cap");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "attention_scored: dtype %d", dtype);
  if (tokens == 0) return 0;
  const long long waves = (long long)tokens * num_heads;
  const long long blocks = (waves + 3) / 4;
  TNX_REQUIRE(blocks < (1ll << 31), "attention_scored: too many (token, head) pairs");
  ScoredArgs a{q, k_pages, v_pages, positions, token_request, table, table_width, page_size, num_pages, out, out_ld,
               out_scale, gate, gate_ld, bias, far, softcap, window, chunk, tokens, num_heads, num_kv, head_size,
               value_size, page_pad};
  if (dtype == TNX_F32)
    attention_scored_any_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(a);
  else
    attention_scored_any_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(a);
  TNX_CHECK_LAUNCH("attention_scored_any");
  return 0;
}
