// Attention whose scores or mask are not the plain ones: a cap on the scores (c tanh(s / c)), a learned bias by
// the distance between query and key, visibility inside chunks of the sequence, and a gate on the result.
//   attention_scored_any   one wave per (token, head), any dtype, any head size in steps of 16: the float32 path
//                          and whatever the matrix-unit kernels do not take
//   attention_scored_tiles bfloat16 on MFMA 16x16x32: a block takes 128 queries of a run of several tokens for
//                          one head, each of its four waves 32 of them
//   attention_scored_single bfloat16 on MFMA: a block takes a run of one token and one key/value head; the
//                          columns are the query heads that share it, the four waves share out the keys
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
  const float* gate;        // [T, gate_ld] or null: pre-activations of the gate, H * gate_head a token
  long long gate_ld;
  int gate_head;            // the gate's numbers a head: value_size (one an element) or 1 (one for the whole head)
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
  const float* gate = a.gate ? a.gate + (size_t)t * a.gate_ld + (size_t)h * a.gate_head : nullptr;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int d = lane + 64 * e;
    if (d >= head_size) continue;
    float v = acc[e] * inv;
    if (gate && d < a.value_size) v *= 1.f / (1.f + expf(-gate[a.gate_head == 1 ? 0 : d]));
    out[d] = from_f32<T>(v);
  }
}

// ------------------------------------------------------------------------------------------ bfloat16, on the matrix unit

// tanh from one exponential and one reciprocal: 1 - 2 / (1 + e^(2x)); +-1 where the exponential leaves the range.
__device__ __forceinline__ float tanh_quick(float x) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * x));
}

// The first key a query at `pos` sees.
__device__ __forceinline__ int first_visible(int pos, int window, int chunk) {
  int lo = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) lo = max(lo, pos - pos % chunk);
  return lo;
}

// A wave's walk over key tiles of 64: the transposed scores S^T = K Q^T of NQB blocks of 16 query columns, so
// that the accumulators (lane = column, four consecutive keys a register group) are at once the B operand of
// O^T += V^T P^T. A column has its own position (`qpos`), first visible key (`qlo`) and bias row (`bias`, by
// distance, in LDS or global memory): the columns are 32 queries of one head, or the heads of one query.
// Tiles `tile_begin`, `tile_begin + tile_step`, ... up to the key `stop` (at most `last_q`, the last position among
// the columns);
// `first_q` the first and `lo_last` the first visible key of the last: a tile between them needs no mask.
template <int NDB, int NQB>
__device__ __forceinline__ void scored_walk(const ScoredArgs& a, const int* __restrict__ tab, size_t page_stride,
                                            int kvh, const bf16x8 (&qf)[NQB][(NDB + 1) / 2], const int (&qpos)[NQB],
                                            const int (&qlo)[NQB], const float* const (&bias)[NQB], int first_q,
                                            int last_q, int stop, int lo_last, int total, int tile_begin, int tile_step,
                                            float (&m)[NQB], float (&l)[NQB], f32x4 (&o)[NDB][NQB]) {
  constexpr int NKS = (NDB + 1) / 2;
  const bf16_t* k_pages = (const bf16_t*)a.k_pages;
  const bf16_t* v_pages = (const bf16_t*)a.v_pages;
  const int head_size = a.head_size, page_size = a.page_size, num_pages = a.num_pages;
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int ndb = head_size / 16;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const bool biased = a.bias != nullptr;

  // A tile's keys as the A operand of the scores (row r of block kb is key 16 kb + r) and its values as that
  // of the result (row r of block db is element 16 db + r; keys 16 tb + 4 g .. + 3), zeros for what has no page,
  // lies beyond the head's size or beyond the request.
  bf16x8 kf[4][NKS];
  bf16x4 vf[NDB][4];
  auto load_keys = [&](int tile0) {
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int key0 = tile0 + 16 * kb;
      int page = -1;
      if (key0 <= last_q) page = tab[key0 / page_size];
      const bool ok = page >= 0 && page < num_pages;
      const bf16_t* kbase = k_pages + (size_t)(ok ? page : 0) * page_stride +
                            ((size_t)kvh * page_size + key0 % page_size + r) * head_size;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        kf[kb][ks] = (ok && d0 < head_size) ? *(const bf16x8*)(kbase + d0) : zero8;
      }
    }
  };
  auto load_values = [&](int tile0) {
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
      const int key0 = tile0 + 16 * tb;
      int page = -1;
      if (key0 <= last_q) page = tab[key0 / page_size];
      const bool ok = page >= 0 && page < num_pages;
      const bf16_t* vbase = v_pages + (size_t)(ok ? page : 0) * page_stride + (size_t)kvh * head_size * page_size +
                            key0 % page_size + 4 * g;
      const bool tail = key0 + 16 > total;      // some keys of this block lie beyond the request
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        bf16x4 v4 = {0, 0, 0, 0};
        if (ok && db < ndb) v4 = *(const bf16x4*)(vbase + (size_t)(16 * db + r) * page_size);
        if (tail) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (key0 + 4 * g + i >= total) v4[i] = 0;
        }
        vf[db][tb] = v4;
      }
    }
  };
  // Where the registers hold both (heads of up to 128 elements), a tile's values are asked for before its
  // scores are made and the next tile's keys as soon as they are: both arrive while the scores are capped,
  // biased and turned into weights.
  constexpr bool AHEAD = NDB <= 8;
  if (AHEAD && tile_begin <= stop) load_keys(tile_begin);

  for (int tile0 = tile_begin; tile0 <= stop; tile0 += tile_step) {
    f32x4 s[4][NQB];
    if (!AHEAD) load_keys(tile0);
    if (AHEAD) load_values(tile0);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) s[kb][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb)
          s[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb][ks], qf[qb][ks], s[kb][qb], 0, 0, 0);
    }
    if (AHEAD && tile0 + tile_step <= stop) load_keys(tile0 + tile_step);
    // the cap, the bias by distance, and -inf for what a query may not see
    const bool full_tile = tile0 + 63 <= first_q && tile0 >= lo_last;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = tile0 + 16 * kb + 4 * g + i;
          float x = s[kb][qb][i];
          if (cap > 0.f) x = cap * tanh_quick(x * inv_cap);
          if (biased) x += bias[qb][min(max(qpos[qb] - key, 0), a.far)];
          if (!full_tile && !(key <= qpos[qb] && key >= qlo[qb])) x = -INFINITY;
          s[kb][qb][i] = x;
        }
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][qb][i]);
      mx = rows_max(mx);
      const float m_new = fmaxf(m[qb], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __expf(m[qb] - m_safe);
      float sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __expf(s[kb][qb][i] - m_safe);
          s[kb][qb][i] = p;
          sum += p;
        }
      sum = rows_sum(sum);
      l[qb] = l[qb] * alpha + sum;
      m[qb] = m_new;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][qb][i] *= alpha;
    }
    if (!AHEAD) load_values(tile0);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (tile0 + 32 * t > last_q) continue;
      bf16x8 pb[NQB];
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int j = 0; j < 8; ++j) pb[qb][j] = (bf16_t)s[2 * t + (j >> 2)][qb][j & 3];
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        if (db >= ndb) continue;
        bf16x8 v8;
#pragma unroll
        for (int j = 0; j < 8; ++j) v8[j] = vf[db][2 * t + (j >> 2)][j & 3];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) o[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v8, pb[qb], o[db][qb], 0, 0, 0);
      }
    }
  }
}

// A column's four elements d0 .. d0 + 3 of one head: times `scale`, through the gate, to the result.
__device__ __forceinline__ void store_four(const ScoredArgs& a, int token, int head, int d0, f32x4 v, float scale,
                                           bool vector_store) {
  bf16_t* orow = (bf16_t*)a.out + (size_t)token * a.out_ld + (size_t)head * a.head_size + d0;
  const float* gate = a.gate ? a.gate + (size_t)token * a.gate_ld + (size_t)head * a.gate_head : nullptr;
  bf16x4 v4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float x = v[i] * scale;
    if (gate && d0 + i < a.value_size) x *= __builtin_amdgcn_rcpf(1.f + __expf(-gate[a.gate_head == 1 ? 0 : d0 + i]));
    v4[i] = (bf16_t)x;
  }
  if (vector_store) {
    *(bf16x4*)orow = v4;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) orow[i] = v4[i];
  }
}

// 128 queries of a run for one head. Dynamic LDS: the head's bias row, where `bias_in_lds`.
template <int NDB>
__global__ void __launch_bounds__(256)
attention_scored_tiles_kernel(ScoredArgs a, const int* __restrict__ run_start, const int* __restrict__ cached_lens,
                              const int* __restrict__ tile_run, const int* __restrict__ tile_q0, int bias_in_lds,
                              int vector_store) {
  extern __shared__ float lds[];
  constexpr int NKS = (NDB + 1) / 2;
  const bf16_t* q = (const bf16_t*)a.q;
  const int head_size = a.head_size;
  const size_t page_stride = (size_t)a.num_kv * a.page_size * head_size + a.page_pad;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x / a.num_heads, h = blockIdx.x % a.num_heads;
  const int run = tile_run[tile];
  const int kvh = h / (a.num_heads / a.num_kv);
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const float* bias_row = a.bias ? a.bias + (size_t)h * (a.far + 1) : nullptr;
  if (bias_row && bias_in_lds) {
#pragma unroll 4
    for (int i = threadIdx.x; i <= a.far; i += 256) lds[i] = bias_row[i];
    __syncthreads();
    bias_row = lds;
  }
  const int qw0 = tile_q0[tile] + 32 * wave;
  if (qw0 >= qlen) return;
  const int nq = a.num_heads * head_size;
  const int* tab = a.table + (size_t)run * a.table_width;
  const int total = cached + qlen;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int ndb = head_size / 16;

  bf16x8 qf[2][NKS];
  int qpos[2], qlo[2];
  const float* bias[2] = {bias_row, bias_row};
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    qpos[qb] = cached + qi;
    qlo[qb] = first_visible(qpos[qb], a.window, a.chunk);
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      const int d0 = 32 * s + 8 * g;
      qf[qb][s] = (qi < qlen && d0 < head_size) ? *(const bf16x8*)(q + (size_t)(t0 + qi) * nq + h * head_size + d0)
                                                : zero8;
    }
  }
  const int first_q = cached + qw0, last_q = cached + min(qw0 + 31, qlen - 1);
  const int lo = first_visible(first_q, a.window, a.chunk);          // no query of the wave reads before this
  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  f32x4 o[NDB][2];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) o[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  scored_walk<NDB, 2>(a, tab, page_stride, kvh, qf, qpos, qlo, bias, first_q, last_q, last_q,
                      first_visible(last_q, a.window, a.chunk), total, (lo / 64) * 64, 64, m, l, o);
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = a.out_scale / l[qb];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (db >= ndb) continue;
      store_four(a, t0 + qi, h, 16 * db + 4 * g, o[db][qb], inv, vector_store != 0);
    }
  }
}

// A run of one token and one key/value head: column c is query head `kvh * pack + width * blockIdx.z + c` of the
// `pack` that share the keys, `width` (up to 16) of them a block. `splits` blocks share the request's key tiles
// (a block's waves take its share's tiles in turn) and leave what they have in `partial`. Wave w of SINGLE_WAVES takes the tiles w, w + SINGLE_WAVES, ...; all but the first
// leave their maxima, sums and weighted values (float32) in LDS and the first joins them. Dynamic LDS:
// (SINGLE_WAVES - 1) * 16 * (16 NDB + 4) floats, then the bias rows of the block's heads, where `bias_in_lds`.
constexpr int SINGLE_WAVES = 8;

template <int NDB>
__global__ void __launch_bounds__(64 * SINGLE_WAVES)
attention_scored_single_kernel(ScoredArgs a, const int* __restrict__ run_start, const int* __restrict__ cached_lens,
                               const int* __restrict__ single_runs, int width, int splits, float* __restrict__ partial,
                               int bias_in_lds, int vector_store) {
  extern __shared__ float lds[];
  constexpr int NKS = (NDB + 1) / 2;
  constexpr int PART = 16 * NDB + 4;      // maximum, sum, two unused, the values (16-byte rows)
  const bf16_t* q = (const bf16_t*)a.q;
  const int head_size = a.head_size;
  const size_t page_stride = (size_t)a.num_kv * a.page_size * head_size + a.page_pad;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int single = blockIdx.x / splits, split = blockIdx.x - single * splits;
  const int run = single_runs[single], kvh = blockIdx.y;
  const int pack = a.num_heads / a.num_kv;
  const int col0 = width * blockIdx.z;
  const int cols = min(width, pack - col0);
  const int head = kvh * pack + col0 + min(r, cols - 1);
  const bool live = r < cols;
  const int token = run_start[run], pos = cached_lens[run];
  float* bias_lds = lds + (SINGLE_WAVES - 1) * 16 * PART;
  if (a.bias && bias_in_lds) {
    const float* rows = a.bias + (size_t)(kvh * pack + col0) * (a.far + 1);
#pragma unroll 4
    for (int i = threadIdx.x; i < cols * (a.far + 1); i += 64 * SINGLE_WAVES) bias_lds[i] = rows[i];
    __syncthreads();
  }
  const int nq = a.num_heads * head_size;
  const int* tab = a.table + (size_t)run * a.table_width;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int ndb = head_size / 16;

  bf16x8 qf[1][NKS];
#pragma unroll
  for (int s = 0; s < NKS; ++s) {
    const int d0 = 32 * s + 8 * g;
    qf[0][s] = (live && d0 < head_size) ? *(const bf16x8*)(q + (size_t)token * nq + head * head_size + d0) : zero8;
  }
  const int lo = first_visible(pos, a.window, a.chunk);
  const int qpos[1] = {pos}, qlo[1] = {lo};
  const float* bias[1] = {nullptr};
  if (a.bias)
    bias[0] = bias_in_lds ? bias_lds + (size_t)min(r, cols - 1) * (a.far + 1) : a.bias + (size_t)head * (a.far + 1);
  float m[1] = {-INFINITY}, l[1] = {0.f};
  f32x4 o[NDB][1];
#pragma unroll
  for (int db = 0; db < NDB; ++db) o[db][0] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // this block's share of the request's key tiles
  const int tile_lo = (lo / 64) * 64;
  const int tiles = (pos - tile_lo) / 64 + 1, share = (tiles + splits - 1) / splits;
  const int begin = tile_lo + 64 * split * share;
  const int stop = min(pos, begin + 64 * share - 1);
  scored_walk<NDB, 1>(a, tab, page_stride, kvh, qf, qpos, qlo, bias, pos, pos, stop, lo, pos + 1, begin + 64 * wave,
                      64 * SINGLE_WAVES, m, l, o);
  if (wave > 0) {
    float* part = lds + ((wave - 1) * 16 + r) * PART;
    if (g == 0) {
      part[0] = m[0];
      part[1] = l[0];
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db)
      if (db < ndb) *(f32x4*)(part + 4 + 16 * db + 4 * g) = o[db][0];
  }
  __syncthreads();
  if (wave > 0 || !live) return;
#pragma unroll
  for (int w = 0; w < SINGLE_WAVES - 1; ++w) {
    const float* part = lds + (w * 16 + r) * PART;
    const float m2 = part[0], l2 = part[1];
    const float m_new = fmaxf(m[0], m2);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float mine = __expf(m[0] - m_safe), other = __expf(m2 - m_safe);
    l[0] = l[0] * mine + l2 * other;
    m[0] = m_new;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
      if (db < ndb) {
        const f32x4 o2 = *(const f32x4*)(part + 4 + 16 * db + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][0][i] = o[db][0][i] * mine + o2[i] * other;
      }
  }
  if (splits > 1) {       // the blocks of a request meet in `attention_scored_join_kernel`
    float* mine = partial + (((size_t)single * a.num_heads + head) * splits + split) * (head_size + 4);
    if (g == 0) {
      mine[0] = m[0];
      mine[1] = l[0];
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db)
      if (db < ndb) *(f32x4*)(mine + 4 + 16 * db + 4 * g) = o[db][0];
    return;
  }
  const float inv = a.out_scale / l[0];
#pragma unroll
  for (int db = 0; db < NDB; ++db) {
    if (db >= ndb) continue;
    store_four(a, token, head, 16 * db + 4 * g, o[db][0], inv, vector_store != 0);
  }
}

// What the `splits` blocks of a decoded token's (request, head) left (maximum, sum, weighted values): joined,
// times the factor, through the gate, to the result. A block of 64 threads a (token, head).
__global__ void __launch_bounds__(64)
attention_scored_join_kernel(ScoredArgs a, const int* __restrict__ run_start, const int* __restrict__ single_runs,
                             int splits, const float* __restrict__ partial) {
  const int single = blockIdx.x, head = blockIdx.y;
  const int token = run_start[single_runs[single]];
  const int stride = a.head_size + 4;
  const float* mine = partial + ((size_t)single * a.num_heads + head) * splits * stride;
  float mm = -INFINITY;
  for (int s = 0; s < splits; ++s) mm = fmaxf(mm, mine[s * stride]);
  float ll = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float ms = mine[s * stride];
    ll += ms == -INFINITY ? 0.f : mine[s * stride + 1] * __expf(ms - mm);
  }
  bf16_t* orow = (bf16_t*)a.out + (size_t)token * a.out_ld + (size_t)head * a.head_size;
  const float* gate = a.gate ? a.gate + (size_t)token * a.gate_ld + (size_t)head * a.gate_head : nullptr;
  for (int d = threadIdx.x; d < a.head_size; d += 64) {
    float oo = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = mine[s * stride];
      if (ms != -INFINITY) oo += mine[s * stride + 4 + d] * __expf(ms - mm);
    }
    float x = oo * a.out_scale / ll;
    if (gate && d < a.value_size) x *= 1.f / (1.f + __expf(-gate[a.gate_head == 1 ? 0 : d]));
    orow[d] = (bf16_t)x;
  }
}

}  // namespace

extern "C" int tnx_attention_scored(const void* q, int dtype, const void* k_pages, const void* v_pages,
                                    const int* positions, const int* token_request, const int* table, int table_width,
                                    int page_size, int num_pages, void* out, long long out_ld, float out_scale,
                                    const float* gate, long long gate_ld, const float* bias, int far, float softcap,
                                    int window, int chunk, int tokens, int num_heads, int num_kv, int head_size,
                                    int value_size, int page_pad, int gate_head, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention_scored: bad head counts");
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention_scored: bad distance between pages");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention_scored: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(value_size > 0 && value_size <= head_size, "attention_scored: values of %d in heads of %d", value_size, head_size);
  TNX_REQUIRE(page_size % 16 == 0 && page_size > 0, "attention_scored: page size %d is not a multiple of 16", page_size);
  TNX_REQUIRE(out_ld >= (long long)num_heads * head_size, "attention_scored: result rows of %lld elements", out_ld);
  TNX_REQUIRE(!gate || ((gate_head == 1 || gate_head == value_size) && gate_ld >= (long long)num_heads * gate_head),
              "attention_scored: gate rows of %lld elements, %d a head", gate_ld, gate_head);
  TNX_REQUIRE(!bias || far >= 0, "attention_scored: a bias table needs its last distance");
  TNX_REQUIRE(window >= 0 && chunk >= 0 && softcap >= 0.f, "attention_scored: bad window, chunk or cap");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "attention_scored: dtype %d", dtype);
  if (tokens == 0) return 0;
  const long long waves = (long long)tokens * num_heads;
  const long long blocks = (waves + 3) / 4;
  TNX_REQUIRE(blocks < (1ll << 31), "attention_scored: too many (token, head) pairs");
  ScoredArgs a{q, k_pages, v_pages, positions, token_request, table, table_width, page_size, num_pages, out, out_ld,
               out_scale, gate, gate_ld, gate_head, bias, far, softcap, window, chunk, tokens, num_heads, num_kv, head_size,
               value_size, page_pad};
  if (dtype == TNX_F32)
    attention_scored_any_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(a);
  else
    attention_scored_any_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(a);
  TNX_CHECK_LAUNCH("attention_scored_any");
  return 0;
}

// The same on the matrix unit, bfloat16: `tile_run` and `tile_q0` name the tiles of 128 queries of the runs of
// several tokens, `single_runs` the runs of one token (either may be empty).
extern "C" int tnx_attention_scored_mfma(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                                         const int* cached_lens, const int* table, int table_width, int page_size,
                                         int num_pages, const int* tile_run, const int* tile_q0, int num_tiles,
                                         int query_tile, const int* single_runs, int num_single, void* out,
                                         long long out_ld, float out_scale, const float* gate, long long gate_ld,
                                         const float* bias, int far, float softcap, int window, int chunk,
                                         int num_heads, int num_kv, int head_size, int value_size, int page_pad,
                                         int splits, float* partial, int gate_head, hipStream_t stream) {
  TNX_REQUIRE(num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention_scored_mfma: bad head counts");
  TNX_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || partial),
              "attention_scored_mfma: %d blocks a decoded token need a workspace", splits);
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention_scored_mfma: bad distance between pages");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention_scored_mfma: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(value_size > 0 && value_size <= head_size, "attention_scored_mfma: values of %d in heads of %d", value_size, head_size);
  TNX_REQUIRE(page_size % 16 == 0 && page_size > 0, "attention_scored_mfma: page size %d is not a multiple of 16", page_size);
  TNX_REQUIRE(out_ld >= (long long)num_heads * head_size, "attention_scored_mfma: result rows of %lld elements", out_ld);
  TNX_REQUIRE(!gate || ((gate_head == 1 || gate_head == value_size) && gate_ld >= (long long)num_heads * gate_head),
              "attention_scored_mfma: gate rows of %lld elements, %d a head", gate_ld, gate_head);
  TNX_REQUIRE(!bias || far >= 0, "attention_scored_mfma: a bias table needs its last distance");
  TNX_REQUIRE(window >= 0 && chunk >= 0 && softcap >= 0.f, "attention_scored_mfma: bad window, chunk or cap");
  TNX_REQUIRE(num_tiles <= 0 || query_tile == 128, "attention_scored_mfma: tiles of %d queries, the kernel takes 128", query_tile);
  TNX_REQUIRE((long long)(num_tiles > 0 ? num_tiles : 0) * num_heads < (1ll << 31), "attention_scored_mfma: too many tiles");
  TNX_REQUIRE(num_single < 65536 * 1024 && num_kv < 65536, "attention_scored_mfma: too many runs or heads");
  ScoredArgs a{q, k_pages, v_pages, nullptr, nullptr, table, table_width, page_size, num_pages, out, out_ld,
               out_scale, gate, gate_ld, gate_head, bias, far, softcap, window, chunk, 0, num_heads, num_kv, head_size,
               value_size, page_pad};
  const int vector_store = out_ld % 4 == 0 && ((uintptr_t)out & 7) == 0;
  const int pack = num_heads / num_kv;
  const size_t budget = 64 * 1024;
  if (num_tiles > 0) {
    const size_t row = bias ? (size_t)(far + 1) * sizeof(float) : 0;
    const int in_lds = bias && row <= budget;
    const size_t lds = in_lds ? row : 0;
    dim3 grid((unsigned)num_tiles * num_heads);
#define LAUNCH_TILES(NDB)                                                                                     \
  attention_scored_tiles_kernel<NDB><<<grid, 256, lds, stream>>>(a, run_start, cached_lens, tile_run, tile_q0, \
                                                                 in_lds, vector_store)
    if (head_size <= 64)
      LAUNCH_TILES(4);
    else if (head_size <= 128)
      LAUNCH_TILES(8);
    else
      LAUNCH_TILES(16);
#undef LAUNCH_TILES
    TNX_CHECK_LAUNCH("attention_scored_tiles");
  }
  if (num_single > 0) {
    const int ndb = head_size <= 64 ? 4 : head_size <= 128 ? 8 : 16;
    const size_t parts = (size_t)(SINGLE_WAVES - 1) * 16 * (16 * ndb + 4) * sizeof(float);
    const int width = pack < 16 ? pack : 16;      // query heads a block
    const size_t rows = bias ? (size_t)width * (far + 1) * sizeof(float) : 0;
    const size_t most = 160 * 1024;
    const int in_lds = bias && parts + rows <= most;
    const size_t lds = parts + (in_lds ? rows : 0);
    dim3 grid((unsigned)num_single * splits, (unsigned)num_kv, (unsigned)((pack + width - 1) / width));
#define LAUNCH_SINGLE(NDB)                                                                                       \
  {                                                                                                              \
    static bool configured = false;                                                                              \
    if (!configured) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)attention_scored_single_kernel<NDB>,                       \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);                 \
      TNX_REQUIRE(e == hipSuccess, "attention_scored_single: cannot reserve LDS: %s", hipGetErrorString(e));     \
      configured = true;                                                                                         \
    }                                                                                                            \
    attention_scored_single_kernel<NDB><<<grid, 64 * SINGLE_WAVES, lds, stream>>>(a, run_start, cached_lens,     \
                                                                                   single_runs, width, splits, partial, in_lds, vector_store); \
  }
    if (ndb == 4) {
      LAUNCH_SINGLE(4)
    } else if (ndb == 8) {
      LAUNCH_SINGLE(8)
    } else {
      LAUNCH_SINGLE(16)
    }
#undef LAUNCH_SINGLE
    TNX_CHECK_LAUNCH("attention_scored_single");
    if (splits > 1) {
      attention_scored_join_kernel<<<dim3((unsigned)num_single, (unsigned)num_heads), 64, 0, stream>>>(a, run_start, single_runs,
                                                                                                       splits, partial);
      TNX_CHECK_LAUNCH("attention_scored_join");
    }
  }
  return 0;
}
