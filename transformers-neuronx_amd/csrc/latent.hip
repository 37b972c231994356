// Latent attention: a token's keys and values are made from one small cached vector c (R elements) and a
// rotated key part k_r (r elements) that all heads share. The products with the key and value matrices are
// moved to the query's side, so the kernels read the cache as it lies:
//   score(i, j, head) = scale * (q_lat[i, head] . c[j] + turn(q_r[i, head]) . k_r[j]),   out[i, head] = sum_j p_j c[j].
// Here: the norms of the two latents with the store into pages, a product per head (batched), and attention.
#include "common.h"

TNX_DEFINE_ERROR_API

// the pair (u, v) at position p, frequency f: angle, sine and cosine in float32
__device__ __forceinline__ void turn_pair(float u, float v, int position, float f, float& a, float& b) {
  const float angle = (float)position * f;
  const float c = cosf(angle), s = sinf(angle);
  a = u * c - v * s;
  b = v * c + u * s;
}

// ------------------------------------------------------------------------------------------------ latents

// One block a token. `down[t]` = [Q | R | r] float32 (rows `ld` elements apart, which may hold more): the first Q, scaled to unit root mean square and
// weighted, go to `c_q`; the next R likewise to the token's place in the latent pages; the last r, pairs
// (2i, 2i + 1) turned for i < pairs, to its place in the rotated pages. R = 0: a mixer without a latent of its own.
__global__ void __launch_bounds__(256)
latent_norms_kernel(const float* __restrict__ down, int ld, int q_rank, int kv_rank, int rot, const float* __restrict__ q_w,
                    const float* __restrict__ kv_w, float eps, const float* __restrict__ freqs, int pairs,
                    const int* __restrict__ positions, const int* __restrict__ token_page,
                    const int* __restrict__ token_offset, void* __restrict__ c_q, int dtype,
                    void* __restrict__ latent_pages, void* __restrict__ rotated_pages, size_t latent_stride,
                    size_t rotated_stride, int num_pages, void* __restrict__ across_pages, size_t across_stride,
                    int page_size) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* row = down + (size_t)t * ld;
  float s = 0.f;
  if (q_rank > 0) {      // (0: a mixer without a query latent)
    for (int i = threadIdx.x; i < q_rank; i += 256) s += row[i] * row[i];
    const float rq = 1.f / sqrtf(block_sum<4>(s, scratch) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += 256) store_any(c_q, dtype, (size_t)t * q_rank + i, row[i] * rq * q_w[i]);
  }
  if (kv_rank == 0) return;
  const int page = token_page[t];
  if (page < 0 || page >= num_pages) return;  // the host checks that every token has a page
  const int off = token_offset[t];
  const float* lat = row + q_rank;
  s = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += 256) s += lat[i] * lat[i];
  const float rk = 1.f / sqrtf(block_sum<4>(s, scratch) / (float)kv_rank + eps);
  const size_t at = (size_t)page * latent_stride + (size_t)off * kv_rank;
  for (int i = threadIdx.x; i < kv_rank; i += 256) {
    const float v = lat[i] * rk * kv_w[i];
    store_any(latent_pages, dtype, at + i, v);
    // the same latent once more with the page's tokens side by side: what the weighted sum contracts over
    if (across_pages) store_any(across_pages, dtype, (size_t)page * across_stride + (size_t)i * page_size + off, v);
  }
  const float* kr = lat + kv_rank;
  const size_t rat = (size_t)page * rotated_stride + (size_t)off * rot;
  for (int i = threadIdx.x; i < rot / 2; i += 256) {
    float a = kr[2 * i], b = kr[2 * i + 1];
    if (i < pairs) turn_pair(kr[2 * i], kr[2 * i + 1], positions[t], freqs[i], a, b);
    store_any(rotated_pages, dtype, rat + 2 * i, a);
    store_any(rotated_pages, dtype, rat + 2 * i + 1, b);
  }
}

extern "C" int tnx_latent_norms(const float* down, int ld, int q_rank, int kv_rank, int rot, const float* q_w,
                                const float* kv_w, float eps, const float* freqs, int pairs, const int* positions,
                                const int* token_page, const int* token_offset, void* c_q, int dtype,
                                void* latent_pages, void* rotated_pages, long long latent_stride,
                                long long rotated_stride, int num_pages, int page_size, void* across_pages,
                                long long across_stride, int tokens, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && q_rank >= 0 && kv_rank >= 0 && q_rank + kv_rank > 0 && rot >= 0 && rot % 2 == 0 &&
                  (kv_rank == 0 || 2 * pairs <= rot) && (q_rank == 0 || (q_w && c_q)),
              "latent_norms: bad sizes q=%d kv=%d rot=%d pairs=%d", q_rank, kv_rank, rot, pairs);
  TNX_REQUIRE(ld >= q_rank + kv_rank + (kv_rank ? rot : 0), "latent_norms: rows of %d elements", ld);
  TNX_REQUIRE(kv_rank == 0 || (latent_pages && rotated_pages && kv_w && latent_stride >= (long long)page_size * kv_rank &&
                               rotated_stride >= (long long)page_size * rot),
              "latent_norms: pages too small for their tokens");
  if (tokens == 0) return 0;
  latent_norms_kernel<<<tokens, 256, 0, stream>>>(down, ld, q_rank, kv_rank, kv_rank ? rot : 0, q_w, kv_w, eps, freqs, pairs,
                                                  positions, token_page, token_offset, c_q, dtype, latent_pages,
                                                  rotated_pages, (size_t)latent_stride, (size_t)rotated_stride,
                                                  num_pages, kv_rank ? across_pages : nullptr, (size_t)across_stride,
                                                  page_size);
  TNX_CHECK_LAUNCH("latent_norms");
  return 0;
}

// ------------------------------------------------------------------------------------------------ a product per head

// out[t, h, n] = alpha * sum_k x[t, h, k] w[h, n, k]. Plain multiply-adds in float32 on tiles of 64 x 64 held in
// LDS, sixteen values of K at a time; each thread makes 4 x 4 results. x is a view: `x_row`, `x_head` are the
// distances, in elements, between tokens and heads.
#define BL_TILE 64
#define BL_K 16
template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(256)
batched_linear_kernel(const TX* __restrict__ x, size_t x_row, size_t x_head, const TW* __restrict__ w,
                      TO* __restrict__ out, float alpha, int tokens, int heads, int n_out, int k_in) {
  __shared__ float xs[BL_K][BL_TILE + 1];
  __shared__ float ws[BL_K][BL_TILE + 1];
  const int h = blockIdx.z;
  const int t0 = blockIdx.y * BL_TILE, n0 = blockIdx.x * BL_TILE;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  const TW* wh = w + (size_t)h * n_out * k_in;
  for (int k0 = 0; k0 < k_in; k0 += BL_K) {
    for (int e = threadIdx.x; e < BL_TILE * BL_K; e += 256) {
      const int row = e / BL_K, kk = e % BL_K;
      const int t = t0 + row, n = n0 + row, k = k0 + kk;
      xs[kk][row] = (t < tokens && k < k_in) ? to_f32(x[(size_t)t * x_row + (size_t)h * x_head + k]) : 0.f;
      ws[kk][row] = (n < n_out && k < k_in) ? to_f32(wh[(size_t)n * k_in + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BL_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = xs[kk][ty * 4 + i];
        b[i] = ws[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= tokens) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < n_out) out[((size_t)t * heads + h) * n_out + n] = from_f32<TO>(alpha * acc[i][j]);
    }
  }
}

// The same for few tokens in bfloat16, on the matrix unit: a wave takes one head and 16 of its outputs and makes
// out^T[n][t] = W[n][:] . x[t][:] for 16 tokens at a time (MFMA 16x16x32: the matrix's rows are the A operand,
// 16 bytes a lane as they lie, the tokens the B operand). The matrix is read once for every 16 tokens.
__global__ void __launch_bounds__(256)
batched_linear_few_kernel(const bf16_t* __restrict__ x, size_t x_row, size_t x_head, const bf16_t* __restrict__ w,
                          bf16_t* __restrict__ out, float alpha, int tokens, int heads, int n_out, int k_in) {
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int n_blocks = (n_out + 15) / 16;
  const int id = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (id >= heads * n_blocks) return;
  const int h = id / n_blocks, nb = id % n_blocks;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int n = 16 * nb + r;
  const bf16_t* wrow = w + ((size_t)h * n_out + min(n, n_out - 1)) * k_in;
  for (int t0 = 0; t0 < tokens; t0 += 16) {
    const int t = t0 + r;
    const bf16_t* xrow = x + (size_t)min(t, tokens - 1) * x_row + (size_t)h * x_head;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < k_in; k0 += 32) {
      const int d0 = k0 + 8 * g;
      const bool in = d0 < k_in;
      const bf16x8 a = (in && n < n_out) ? *(const bf16x8*)(wrow + d0) : zero8;
      const bf16x8 b = (in && t < tokens) ? *(const bf16x8*)(xrow + d0) : zero8;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
    if (t < tokens) {
      bf16_t* orow = out + ((size_t)t * heads + h) * n_out;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int no = 16 * nb + 4 * g + i;
        if (no < n_out) orow[no] = (bf16_t)(alpha * acc[i]);
      }
    }
  }
}

extern "C" int tnx_batched_linear(const void* x, int x_dtype, long long x_row, long long x_head, const void* w,
                                  int w_dtype, void* out, int out_dtype, float alpha, int tokens, int heads, int n_out,
                                  int k_in, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && heads > 0 && n_out > 0 && k_in > 0, "batched_linear: bad sizes");
  TNX_REQUIRE(heads <= 65535 && (tokens + BL_TILE - 1) / BL_TILE <= 65535, "batched_linear: too many heads or tokens");
  if (tokens == 0) return 0;
  if (x_dtype == TNX_BF16 && w_dtype == TNX_BF16 && out_dtype == TNX_BF16 && tokens <= 64 && k_in % 8 == 0 &&
      x_row % 8 == 0 && x_head % 8 == 0 && ((size_t)x % 16) == 0 && ((size_t)w % 16) == 0) {
    const int waves = heads * ((n_out + 15) / 16);
    batched_linear_few_kernel<<<(waves + 3) / 4, 256, 0, stream>>>((const bf16_t*)x, (size_t)x_row, (size_t)x_head,
                                                                   (const bf16_t*)w, (bf16_t*)out, alpha, tokens, heads,
                                                                   n_out, k_in);
    TNX_CHECK_LAUNCH("batched_linear_few");
    return 0;
  }
  const dim3 grid((n_out + BL_TILE - 1) / BL_TILE, (tokens + BL_TILE - 1) / BL_TILE, heads);
#define BL_LAUNCH(TX, TW, TO)                                                                                      \
  batched_linear_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (size_t)x_row, (size_t)x_head,         \
                                                              (const TW*)w, (TO*)out, alpha, tokens, heads, n_out, k_in)
  const int key = x_dtype * 4 + w_dtype * 2 + out_dtype;
  switch (key) {
    case 0: BL_LAUNCH(float, float, float); break;
    case 1: BL_LAUNCH(float, float, bf16_t); break;
    case 2: BL_LAUNCH(float, bf16_t, float); break;
    case 3: BL_LAUNCH(float, bf16_t, bf16_t); break;
    case 4: BL_LAUNCH(bf16_t, float, float); break;
    case 5: BL_LAUNCH(bf16_t, float, bf16_t); break;
    case 6: BL_LAUNCH(bf16_t, bf16_t, float); break;
    default: BL_LAUNCH(bf16_t, bf16_t, bf16_t); break;
  }
#undef BL_LAUNCH
  TNX_CHECK_LAUNCH("batched_linear");
  return 0;
}

// What ends a (query, head)'s softmax beside the division by its sum (`softmax_finish`): a number a head that
// joins the denominator as exp(sink), and a gate a (token, head) whose sigmoid multiplies the result; either may
// be absent.
struct LatentFinish {
  const float* sink;     // [H] or null
  const float* gate;     // [T, gate_ld], a number a head, or null
  long long gate_ld;
};
__device__ __forceinline__ float latent_finish(const LatentFinish& f, float m, float l, size_t token, int head) {
  return softmax_finish(m, l, f.sink ? f.sink + head : nullptr, f.gate ? f.gate + token * f.gate_ld + head : nullptr);
}

// ------------------------------------------------------------------------------------------------ attention, any sizes

// One block of 256 threads a (token, head). The query's two parts lie in LDS as float32 (q_r turned by the
// token's position and scaled here). Keys are taken 256 at a time, one a thread: its score, then the running
// maximum and sum of the softmax, then every thread adds the tile's weighted latents for the elements it owns
// (element d of c is owned by thread d mod 256; up to LA_OWN elements a thread).
#define LA_OWN 8
template <typename T>
__global__ void __launch_bounds__(256)
latent_attention_any_kernel(const T* __restrict__ q, const T* __restrict__ q_lat, T* __restrict__ out,
                            const int* __restrict__ positions, const int* __restrict__ token_request,
                            const int* __restrict__ block_table, int table_width, int page_size, int num_pages,
                            const T* __restrict__ latent_pages, const T* __restrict__ rotated_pages,
                            size_t latent_stride, size_t rotated_stride, const float* __restrict__ freqs, int pairs,
                            float scale, int heads, int head_size, int rot, int kv_rank, int window, LatentFinish fin) {
  extern __shared__ float lds[];
  float* ql = lds;                 // [kv_rank]
  float* qr = ql + kv_rank;        // [rot]
  float* prob = qr + rot;          // [256]
  int* where = (int*)(prob + 256); // [256] page of each key of the tile
  __shared__ float scratch[4];
  const int t = blockIdx.x, h = blockIdx.y;
  const int p = positions[t];
  const int* table = block_table + (size_t)token_request[t] * table_width;
  const T* qrow = q + ((size_t)t * heads + h) * (head_size + rot) + head_size;
  for (int i = threadIdx.x; i < kv_rank; i += 256) ql[i] = scale * to_f32(q_lat[((size_t)t * heads + h) * kv_rank + i]);
  for (int i = threadIdx.x; i < rot / 2; i += 256) {
    float a = to_f32(qrow[2 * i]), b = to_f32(qrow[2 * i + 1]);
    if (i < pairs) turn_pair(to_f32(qrow[2 * i]), to_f32(qrow[2 * i + 1]), p, freqs[i], a, b);
    qr[2 * i] = a * scale;
    qr[2 * i + 1] = b * scale;
  }
  __syncthreads();
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[LA_OWN];
#pragma unroll
  for (int i = 0; i < LA_OWN; ++i) acc[i] = 0.f;
  for (int j0 = lo; j0 <= p; j0 += 256) {
    const int j = j0 + threadIdx.x;
    float s = -INFINITY;
    int page = -1;
    if (j <= p) {
      const int b = j / page_size;
      page = b < table_width ? table[b] : -1;
      if (page >= 0 && page < num_pages) {
        const T* c = latent_pages + (size_t)page * latent_stride + (size_t)(j % page_size) * kv_rank;
        const T* kr = rotated_pages + (size_t)page * rotated_stride + (size_t)(j % page_size) * rot;
        float dot = 0.f;
        for (int d = 0; d < kv_rank; ++d) dot += ql[d] * to_f32(c[d]);
        for (int d = 0; d < rot; ++d) dot += qr[d] * to_f32(kr[d]);
        s = dot;
      } else {
        page = -1;
      }
    }
    // the tile's maximum, through LDS
    float tile_max = wave_max(s);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = tile_max;
    __syncthreads();
    tile_max = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
    const float m_new = fmaxf(m, tile_max);
    const float w = (page >= 0 && m_new > -INFINITY) ? expf(s - m_new) : 0.f;
    const float fade = m > -INFINITY ? expf(m - m_new) : 0.f;
    prob[threadIdx.x] = w;
    where[threadIdx.x] = page;
    l = l * fade + block_sum<4>(w, scratch);   // (its barriers also make `prob` and `where` visible)
    m = m_new;
    const int count = min(256, p - j0 + 1);
#pragma unroll
    for (int i = 0; i < LA_OWN; ++i) {
      const int d = threadIdx.x + i * 256;
      if (d < kv_rank) {
        float a = acc[i] * fade;
        for (int k = 0; k < count; ++k) {
          const int pg = where[k];
          if (pg >= 0)
            a += prob[k] * to_f32(latent_pages[(size_t)pg * latent_stride + (size_t)((j0 + k) % page_size) * kv_rank + d]);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  const float inv = latent_finish(fin, m, l, t, h);
#pragma unroll
  for (int i = 0; i < LA_OWN; ++i) {
    const int d = threadIdx.x + i * 256;
    if (d < kv_rank) out[((size_t)t * heads + h) * kv_rank + d] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int tnx_latent_attention_any(const void* q, int dtype, const void* q_lat, void* out, const int* positions,
                                        const int* token_request, const int* block_table, int table_width,
                                        int page_size, int num_pages, const void* latent_pages,
                                        const void* rotated_pages, long long latent_stride, long long rotated_stride,
                                        const float* freqs, int pairs, float scale, int heads, int head_size, int rot,
                                        int kv_rank, int window, int tokens, const float* sink, const float* gate,
                                        long long gate_ld, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && heads > 0 && heads <= 65535 && kv_rank > 0 && rot >= 0 && rot % 2 == 0 && 2 * pairs <= rot,
              "latent_attention: bad sizes heads=%d kv_rank=%d rot=%d", heads, kv_rank, rot);
  TNX_REQUIRE(kv_rank <= 256 * LA_OWN, "latent_attention: a latent of %d elements is more than %d", kv_rank, 256 * LA_OWN);
  TNX_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0 && window >= 0, "latent_attention: bad page sizes");
  if (tokens == 0) return 0;
  TNX_REQUIRE(!gate || gate_ld >= heads, "latent_attention: gate rows of %lld elements", gate_ld);
  const size_t lds = (size_t)(kv_rank + rot + 512) * sizeof(float);
  const dim3 grid(tokens, heads);
  const LatentFinish fin{sink, gate, gate_ld};
  if (dtype == TNX_F32)
    latent_attention_any_kernel<float><<<grid, 256, lds, stream>>>(
        (const float*)q, (const float*)q_lat, (float*)out, positions, token_request, block_table, table_width, page_size,
        num_pages, (const float*)latent_pages, (const float*)rotated_pages, (size_t)latent_stride, (size_t)rotated_stride,
        freqs, pairs, scale, heads, head_size, rot, kv_rank, window, fin);
  else
    latent_attention_any_kernel<bf16_t><<<grid, 256, lds, stream>>>(
        (const bf16_t*)q, (const bf16_t*)q_lat, (bf16_t*)out, positions, token_request, block_table, table_width,
        page_size, num_pages, (const bf16_t*)latent_pages, (const bf16_t*)rotated_pages, (size_t)latent_stride,
        (size_t)rotated_stride, freqs, pairs, scale, heads, head_size, rot, kv_rank, window, fin);
  TNX_CHECK_LAUNCH("latent_attention_any");
  return 0;
}

// ------------------------------------------------------------------------------------------------ attention, bfloat16

// On the matrix unit (MFMA 16x16x32), for latents of a multiple of 16 elements up to 16 * NDB and a rotated part
// of a multiple of 8 up to LM_ROT. A key is the row [c | k_r] (its two parts lie in pages of their own); the
// values are the c once more, kept with a page's tokens side by side (`across`: [pages, R, page_size]), since
// the weighted sum contracts over tokens. As in the attention kernels of the other designs the transposed
// scores S^T = K Q^T are computed, so that the accumulators (lane = column, four consecutive keys a register
// group) are at once the B operand of O^T += C^T P^T. A column is a (query, head): in a prompt's run the 16
// columns of a block of columns are 16 consecutive queries of one head, in decoding 16 heads of the one query,
// which read the request's keys once between them. q_r is turned by the query's position as it is loaded;
// the scale meets the float32 scores.
#define LM_ROT 64

struct LatentPages {
  const bf16_t* latent;   // [pages, page_size, R]
  const bf16_t* rotated;  // [pages, page_size, rot]
  const bf16_t* across;   // [pages, R, page_size]
  size_t latent_stride, rotated_stride, across_stride;
  int page_size, num_pages, kv_rank, rot;
};

// the query operand of one column: chunk `d0 .. d0 + 7` of [q_lat | turn(q_r)]
__device__ __forceinline__ bf16x8 latent_query_chunk(const bf16_t* q_lat_row, const bf16_t* q_rot_row, int d0, int kv_rank,
                                                     int rot, int position, const float* freqs, int pairs) {
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  if (d0 < kv_rank) return *(const bf16x8*)(q_lat_row + d0);
  if (d0 >= kv_rank + rot) return zero8;
  const bf16x8 raw = *(const bf16x8*)(q_rot_row + (d0 - kv_rank));
  bf16x8 out;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int pair = (d0 - kv_rank) / 2 + j;
    float a = (float)raw[2 * j], b = (float)raw[2 * j + 1];
    if (pair < pairs) turn_pair((float)raw[2 * j], (float)raw[2 * j + 1], position, freqs[pair], a, b);
    out[2 * j] = (bf16_t)a;
    out[2 * j + 1] = (bf16_t)b;
  }
  return out;
}

// S^T of 64 keys from `tile0` on against QB blocks of 16 columns: s[kb][qb][i] = key tile0 + 16 kb + 4 g + i
template <int NKS, int QB>
__device__ __forceinline__ void latent_scores(const LatentPages& pg, const int* tab, int tile0, int last_key, int r, int g,
                                              const bf16x8 (&qf)[QB][NKS], f32x4 (&s)[4][QB]) {
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    const int key0 = tile0 + 16 * kb;
    f32x4 a[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) a[qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    int page = -1;
    if (key0 <= last_key) page = tab[key0 / pg.page_size];
    if (page >= 0 && page < pg.num_pages) {
      const int off = key0 % pg.page_size + r;
      const bf16_t* crow = pg.latent + (size_t)page * pg.latent_stride + (size_t)off * pg.kv_rank;
      const bf16_t* rrow = pg.rotated + (size_t)page * pg.rotated_stride + (size_t)off * pg.rot;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        bf16x8 kf = zero8;
        if (d0 < pg.kv_rank) kf = *(const bf16x8*)(crow + d0);
        else if (d0 < pg.kv_rank + pg.rot) kf = *(const bf16x8*)(rrow + (d0 - pg.kv_rank));
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) a[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qb][ks], a[qb], 0, 0, 0);
      }
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) s[kb][qb] = a[qb];
  }
}

// the running softmax of one block of columns over a tile's masked scores; leaves the probabilities in `s`
template <int NDB, int QB>
__device__ __forceinline__ void latent_softmax(f32x4 (&s)[4][QB], int qb, float& m, float& l, f32x4 (&o)[NDB][QB]) {
  float mx = -INFINITY;
#pragma unroll
  for (int kb = 0; kb < 4; ++kb)
#pragma unroll
    for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][qb][i]);
  mx = rows_max(mx);
  const float m_new = fmaxf(m, mx);
  const float m_safe = m_new == -INFINITY ? 0.f : m_new;
  const float alpha = __expf(m - m_safe);
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
  l = l * alpha + sum;
  m = m_new;
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) o[db][qb][i] *= alpha;
}

// O^T += C^T P^T for the tile's 64 keys
template <int NDB, int QB>
__device__ __forceinline__ void latent_weighted_sum(const LatentPages& pg, const int* tab, int tile0, int last_key, int total,
                                                    int r, int g, const f32x4 (&s)[4][QB], f32x4 (&o)[NDB][QB]) {
  const int ndb = pg.kv_rank / 16;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (tile0 + 32 * t > last_key) continue;
    bf16x8 pb[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int j = 0; j < 8; ++j) pb[qb][j] = (bf16_t)s[2 * t + (j >> 2)][qb][j & 3];
    const bf16_t* vbase[2];
    bool vok[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int key0 = tile0 + 32 * t + 16 * b;
      int page = -1;
      if (key0 <= last_key) page = tab[key0 / pg.page_size];
      vok[b] = page >= 0 && page < pg.num_pages;
      vbase[b] = pg.across + (size_t)(vok[b] ? page : 0) * pg.across_stride + key0 % pg.page_size + 4 * g;
    }
    const bool tail = tile0 + 32 * t + 32 > total;   // some keys of this step lie beyond the request
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (db >= ndb) continue;
      const int d = 16 * db + r;
      bf16x8 vf;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        bf16x4 v4 = {0, 0, 0, 0};
        if (vok[b]) v4 = *(const bf16x4*)(vbase[b] + (size_t)d * pg.page_size);
        if (tail) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (tile0 + 32 * t + 16 * b + 4 * g + i >= total) v4[i] = 0;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) vf[4 * b + i] = v4[i];
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) o[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[qb], o[db][qb], 0, 0, 0);
    }
  }
}

// A prompt's run: a block of four waves takes 64 QB consecutive queries of one head, a wave 16 QB of them.
template <int NDB, int QB>
__global__ void __launch_bounds__(256)
latent_attention_prompt_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ q_lat, bf16_t* __restrict__ out,
                               const int* __restrict__ run_start, const int* __restrict__ cached_lens,
                               const int* __restrict__ table, int table_width, const int* __restrict__ tile_run,
                               const int* __restrict__ tile_q0, int tile_tokens, LatentPages pg,
                               const float* __restrict__ freqs, int pairs, float scale, int heads, int head_size,
                               int window, LatentFinish fin) {
  constexpr int NKS = (16 * NDB + LM_ROT) / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int parts = tile_tokens / (64 * QB);       // blocks a tile of the plan is cut into
  const int h = blockIdx.x % heads;
  const int part = (blockIdx.x / heads) % parts, tile = blockIdx.x / heads / parts;
  const int run = tile_run[tile];
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int qw0 = tile_q0[tile] + 64 * QB * part + 16 * QB * wave;
  if (qw0 >= qlen) return;
  const int* tab = table + (size_t)run * table_width;
  const int total = cached + qlen;
  const int R = pg.kv_rank, rot = pg.rot;

  bf16x8 qf[QB][NKS];
  int qpos[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    qpos[qb] = cached + qi;
    const size_t th = (size_t)(t0 + min(qi, qlen - 1)) * heads + h;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      qf[qb][ks] = latent_query_chunk(q_lat + th * R, q + th * (head_size + rot) + head_size, 32 * ks + 8 * g, R, rot,
                                      qpos[qb], freqs, pairs);
  }
  const int last_q = cached + min(qw0 + 16 * QB - 1, qlen - 1);
  const int first_q = cached + qw0;
  const int lo = window > 0 ? max(0, first_q - window + 1) : 0;

  float m[QB], l[QB];
  f32x4 o[NDB][QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = -INFINITY;
    l[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  for (int tile0 = (lo / 64) * 64; tile0 <= last_q; tile0 += 64) {
    f32x4 s[4][QB];
    latent_scores<NKS, QB>(pg, tab, tile0, last_q, r, g, qf, s);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = tile0 + 16 * kb + 4 * g + i;
          const bool ok = key <= qpos[qb] && (window <= 0 || key > qpos[qb] - window);
          s[kb][qb][i] = ok ? s[kb][qb][i] * scale : -INFINITY;
        }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) latent_softmax<NDB, QB>(s, qb, m[qb], l[qb], o);
    latent_weighted_sum<NDB, QB>(pg, tab, tile0, last_q, total, r, g, s, o);
  }
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = latent_finish(fin, m[qb], l[qb], t0 + qi, h);
    bf16_t* orow = out + ((size_t)(t0 + qi) * heads + h) * R;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (16 * db >= R) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[db][qb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

// Decoding: a block takes 16 heads of one request's query (the 16 columns) and a share of its keys, 64 at a
// time. Its four waves work on the same tile: each makes the scores of 16 of the keys, the maxima and sums meet
// in LDS, the probabilities go to LDS as the B operand of the second product, and there each wave owns a
// quarter of the latent's blocks of 16 elements, over all 64 keys. So a wave holds a quarter of the result, the
// keys are read once a block, and the second product reads 8 consecutive tokens of `across`, 16 bytes a lane.
// With `splits` > 1 the partial results (maximum, sum, weighted latents, float32) go to `part` and a second
// kernel joins them.
template <int NDB>
__global__ void __launch_bounds__(256)
latent_attention_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ q_lat, bf16_t* __restrict__ out,
                               const int* __restrict__ run_start, const int* __restrict__ cached_lens,
                               const int* __restrict__ table, int table_width, const int* __restrict__ decode_runs,
                               LatentPages pg, const float* __restrict__ freqs, int pairs, float scale, int heads,
                               int head_size, int window, float* __restrict__ part, int splits, int tiles_per_split,
                               LatentFinish fin) {
  constexpr int NKS = (16 * NDB + LM_ROT) / 32;
  constexpr int OWN = (NDB + 3) / 4;           // blocks of 16 latent elements a wave owns: wave, wave + 4, ...
  __shared__ float tile_max[4][16], tile_sum[4][16];
  __shared__ __attribute__((aligned(16))) bf16_t prob[16][64 + 8];   // [column][key of the tile]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int run = decode_runs[blockIdx.x];
  const int t = run_start[run], p = cached_lens[run];
  const int h = 16 * blockIdx.y + r;
  const int* tab = table + (size_t)run * table_width;
  const int R = pg.kv_rank, rot = pg.rot;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8 qf[NKS];
  {
    const size_t th = (size_t)t * heads + min(h, heads - 1);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      qf[ks] = h < heads ? latent_query_chunk(q_lat + th * R, q + th * (head_size + rot) + head_size, 32 * ks + 8 * g, R,
                                              rot, p, freqs, pairs)
                         : zero8;
  }
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int first = (lo / 64) * 64 + 64 * tiles_per_split * (int)blockIdx.z;
  const int end = min(p, first + 64 * tiles_per_split - 1);       // the last key this block may read
  float m = -INFINITY, l = 0.f;
  f32x4 o[OWN];
#pragma unroll
  for (int j = 0; j < OWN; ++j) o[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int tile0 = first; tile0 <= end; tile0 += 64) {
    // this wave's 16 keys against the 16 columns
    const int key0 = tile0 + 16 * wave;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    int page = -1;
    if (key0 <= p) page = tab[key0 / pg.page_size];
    if (page >= 0 && page < pg.num_pages) {
      const int off = key0 % pg.page_size + r;
      const bf16_t* crow = pg.latent + (size_t)page * pg.latent_stride + (size_t)off * R;
      const bf16_t* rrow = pg.rotated + (size_t)page * pg.rotated_stride + (size_t)off * rot;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        bf16x8 kf = zero8;
        if (d0 < R) kf = *(const bf16x8*)(crow + d0);
        else if (d0 < R + rot) kf = *(const bf16x8*)(rrow + (d0 - R));
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], a, 0, 0, 0);
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + 4 * g + i;
      a[i] = (key <= p && key >= lo && page >= 0) ? a[i] * scale : -INFINITY;
      mx = fmaxf(mx, a[i]);
    }
    mx = rows_max(mx);
    if (g == 0) tile_max[wave][r] = mx;
    __syncthreads();
    const float m_new = fmaxf(m, fmaxf(fmaxf(tile_max[0][r], tile_max[1][r]), fmaxf(tile_max[2][r], tile_max[3][r])));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(m - m_safe);
    float sum = 0.f;
    bf16x4 p4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float pr = __expf(a[i] - m_safe);
      sum += pr;
      p4[i] = (bf16_t)pr;
    }
    sum = rows_sum(sum);
    *(bf16x4*)&prob[r][16 * wave + 4 * g] = p4;
    if (g == 0) tile_sum[wave][r] = sum;
    __syncthreads();
    l = l * alpha + ((tile_sum[0][r] + tile_sum[1][r]) + (tile_sum[2][r] + tile_sum[3][r]));
    m = m_new;
    // the weighted latents of the blocks this wave owns, over the tile's 64 keys
    bf16x8 pb[2];
    const bf16_t* vbase[2];
    bool vok[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      pb[s2] = *(const bf16x8*)&prob[r][32 * s2 + 8 * g];
      const int k0 = tile0 + 32 * s2 + 8 * g;         // this lane's 8 consecutive keys
      int pgn = -1;
      if (k0 <= p) pgn = tab[k0 / pg.page_size];
      vok[s2] = pgn >= 0 && pgn < pg.num_pages;
      vbase[s2] = pg.across + (size_t)(vok[s2] ? pgn : 0) * pg.across_stride + k0 % pg.page_size;
    }
    const bool tail = tile0 + 63 > p;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= R) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[j][i] *= alpha;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        bf16x8 vf = zero8;
        if (vok[s2]) vf = *(const bf16x8*)(vbase[s2] + (size_t)(16 * db + r) * pg.page_size);
        if (tail) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (tile0 + 32 * s2 + 8 * g + e > p) vf[e] = 0;
        }
        o[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[s2], o[j], 0, 0, 0);
      }
    }
    __syncthreads();       // before the next tile's probabilities are written
  }
  if (h >= heads) return;
  if (splits == 1) {
    const float inv = latent_finish(fin, m, l, t, h);
    bf16_t* orow = out + ((size_t)t * heads + h) * R;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= R) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[j][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
    return;
  }
  // [decode run][head][split][R + 2]: the weighted latents, then the maximum and the sum
  float* mine = part + (((size_t)blockIdx.x * heads + h) * splits + blockIdx.z) * (R + 2);
#pragma unroll
  for (int j = 0; j < OWN; ++j) {
    const int db = wave + 4 * j;
    if (16 * db >= R) continue;
    *(f32x4*)(mine + 16 * db + 4 * g) = o[j];
  }
  if (wave == 0 && g == 0) {
    mine[R] = m;
    mine[R + 1] = l;
  }
}

// A prompt's run with the waves of a block on one tile, as in decoding: the columns are 16 consecutive queries
// of HB heads (HB blocks of 16 columns, which see the same keys), each wave makes the scores of 16 of a tile's 64
// keys for all of them and owns a quarter of the latent's blocks in the second product. Against a wave that walks
// the keys alone for its own 16 queries, the keys are read once a block and not once a wave, and every operand
// that is loaded meets HB products.
template <int NDB, int HB>
__global__ void __launch_bounds__(256)
latent_attention_prompt_shared_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ q_lat,
                                      bf16_t* __restrict__ out, const int* __restrict__ run_start,
                                      const int* __restrict__ cached_lens, const int* __restrict__ table,
                                      int table_width, const int* __restrict__ tile_run,
                                      const int* __restrict__ tile_q0, int tile_tokens, LatentPages pg,
                                      const float* __restrict__ freqs, int pairs, float scale, int heads,
                                      int head_size, int window, LatentFinish fin) {
  constexpr int NKS = (16 * NDB + LM_ROT) / 32;
  constexpr int OWN = (NDB + 3) / 4;
  __shared__ float tile_max[4][HB][16], tile_sum[4][HB][16];
  __shared__ __attribute__((aligned(16))) bf16_t prob[HB][16][64 + 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int head_groups = (heads + HB - 1) / HB, parts = tile_tokens / 16;
  const int hg = blockIdx.x % head_groups;
  const int part = (blockIdx.x / head_groups) % parts, tile = blockIdx.x / head_groups / parts;
  const int run = tile_run[tile];
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int q0 = tile_q0[tile] + 16 * part;
  if (q0 >= qlen) return;
  const int* tab = table + (size_t)run * table_width;
  const int total = cached + qlen;
  const int R = pg.kv_rank, rot = pg.rot;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int qi = q0 + r, qpos = cached + qi;

  bf16x8 qf[HB][NKS];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    const int h = HB * hg + hb;
    const size_t th = (size_t)(t0 + min(qi, qlen - 1)) * heads + min(h, heads - 1);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      qf[hb][ks] = h < heads ? latent_query_chunk(q_lat + th * R, q + th * (head_size + rot) + head_size, 32 * ks + 8 * g, R,
                                                  rot, qpos, freqs, pairs)
                             : zero8;
  }
  const int first_q = cached + q0, last_q = cached + min(q0 + 15, qlen - 1);
  const int lo = window > 0 ? max(0, first_q - window + 1) : 0;
  float m[HB], l[HB];
  f32x4 o[OWN][HB];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    m[hb] = -INFINITY;
    l[hb] = 0.f;
#pragma unroll
    for (int j = 0; j < OWN; ++j) o[j][hb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  for (int tile0 = (lo / 64) * 64; tile0 <= last_q; tile0 += 64) {
    const int key0 = tile0 + 16 * wave;
    f32x4 a[HB];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) a[hb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    int page = -1;
    if (key0 <= last_q) page = tab[key0 / pg.page_size];
    if (page >= 0 && page < pg.num_pages) {
      const int off = key0 % pg.page_size + r;
      const bf16_t* crow = pg.latent + (size_t)page * pg.latent_stride + (size_t)off * R;
      const bf16_t* rrow = pg.rotated + (size_t)page * pg.rotated_stride + (size_t)off * rot;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        bf16x8 kf = zero8;
        if (d0 < R) kf = *(const bf16x8*)(crow + d0);
        else if (d0 < R + rot) kf = *(const bf16x8*)(rrow + (d0 - R));
#pragma unroll
        for (int hb = 0; hb < HB; ++hb) a[hb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[hb][ks], a[hb], 0, 0, 0);
      }
    }
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 4 * g + i;
        const bool ok = page >= 0 && key <= qpos && (window <= 0 || key > qpos - window);
        a[hb][i] = ok ? a[hb][i] * scale : -INFINITY;
        mx = fmaxf(mx, a[hb][i]);
      }
      mx = rows_max(mx);
      if (g == 0) tile_max[wave][hb][r] = mx;
    }
    __syncthreads();
    float alpha[HB];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      const float m_new = fmaxf(m[hb], fmaxf(fmaxf(tile_max[0][hb][r], tile_max[1][hb][r]),
                                             fmaxf(tile_max[2][hb][r], tile_max[3][hb][r])));
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[hb] = __expf(m[hb] - m_safe);
      m[hb] = m_new;
      float sum = 0.f;
      bf16x4 p4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = __expf(a[hb][i] - m_safe);
        sum += pr;
        p4[i] = (bf16_t)pr;
      }
      sum = rows_sum(sum);
      *(bf16x4*)&prob[hb][r][16 * wave + 4 * g] = p4;
      if (g == 0) tile_sum[wave][hb][r] = sum;
    }
    __syncthreads();
    bf16x8 pb[HB][2];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      l[hb] = l[hb] * alpha[hb] + ((tile_sum[0][hb][r] + tile_sum[1][hb][r]) + (tile_sum[2][hb][r] + tile_sum[3][hb][r]));
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) pb[hb][s2] = *(const bf16x8*)&prob[hb][r][32 * s2 + 8 * g];
    }
    const bf16_t* vbase[2];
    bool vok[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const int k0 = tile0 + 32 * s2 + 8 * g;
      int pgn = -1;
      if (k0 <= last_q) pgn = tab[k0 / pg.page_size];
      vok[s2] = pgn >= 0 && pgn < pg.num_pages;
      vbase[s2] = pg.across + (size_t)(vok[s2] ? pgn : 0) * pg.across_stride + k0 % pg.page_size;
    }
    const bool tail = tile0 + 64 > total;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= R) continue;
#pragma unroll
      for (int hb = 0; hb < HB; ++hb)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[j][hb][i] *= alpha[hb];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        bf16x8 vf = zero8;
        if (vok[s2]) vf = *(const bf16x8*)(vbase[s2] + (size_t)(16 * db + r) * pg.page_size);
        if (tail) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (tile0 + 32 * s2 + 8 * g + e >= total) vf[e] = 0;
        }
#pragma unroll
        for (int hb = 0; hb < HB; ++hb) o[j][hb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[hb][s2], o[j][hb], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (qi >= qlen) return;
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    const int h = HB * hg + hb;
    if (h >= heads) continue;
    const float inv = latent_finish(fin, m[hb], l[hb], t0 + qi, h);
    bf16_t* orow = out + ((size_t)(t0 + qi) * heads + h) * R;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= R) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[j][hb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

// joins the partial results of the splits of one (decode run, head): one block each
__global__ void __launch_bounds__(256)
latent_attention_join_kernel(const float* __restrict__ part, bf16_t* __restrict__ out, const int* __restrict__ run_start,
                             const int* __restrict__ decode_runs, int heads, int kv_rank, int splits, LatentFinish fin) {
  const int h = blockIdx.y;
  const int t = run_start[decode_runs[blockIdx.x]];
  const float* mine = part + ((size_t)blockIdx.x * heads + h) * splits * (kv_rank + 2);
  float m = -INFINITY;
  for (int s = 0; s < splits; ++s) m = fmaxf(m, mine[(size_t)s * (kv_rank + 2) + kv_rank]);
  const float m_safe = m == -INFINITY ? 0.f : m;
  float l = 0.f;
  for (int s = 0; s < splits; ++s)
    l += mine[(size_t)s * (kv_rank + 2) + kv_rank + 1] * __expf(mine[(size_t)s * (kv_rank + 2) + kv_rank] - m_safe);
  const float inv = latent_finish(fin, m, l, t, h);
  for (int d = threadIdx.x; d < kv_rank; d += 256) {
    float acc = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float f = __expf(mine[(size_t)s * (kv_rank + 2) + kv_rank] - m_safe);
      if (f > 0.f) acc += mine[(size_t)s * (kv_rank + 2) + d] * f;
    }
    out[((size_t)t * heads + h) * kv_rank + d] = (bf16_t)(acc * inv);
  }
}

// `tiles` runs of several tokens cut into tiles of `tile_tokens` queries (`tile_run`, `tile_q0`), and `decodes`
// runs of one token (`decode_runs`); either may be none. The keys of a decoding request are shared out over
// `splits` blocks of `tiles_per_split` tiles of 64 keys each; beyond one split `part` holds
// decodes * heads * splits * (kv_rank + 2) floats. `prompt_kind` 0: the prompt kernel whose waves share a tile;
// 1: the one whose waves walk the keys each for its own queries.
extern "C" int tnx_latent_attention_mfma(const void* q, const void* q_lat, void* out, const int* run_start,
                                         const int* cached_lens, const int* block_table, int table_width, int page_size,
                                         int num_pages, const int* tile_run, const int* tile_q0, int tiles,
                                         int tile_tokens, const int* decode_runs, int decodes, const void* latent_pages,
                                         const void* rotated_pages, const void* across_pages, long long latent_stride,
                                         long long rotated_stride, long long across_stride, const float* freqs, int pairs,
                                         float scale, int heads, int head_size, int rot, int kv_rank, int window,
                                         float* part, int splits, int tiles_per_split, int prompt_kind,
                                         const float* sink, const float* gate, long long gate_ld, hipStream_t stream) {
  TNX_REQUIRE(kv_rank > 0 && kv_rank % 16 == 0 && kv_rank <= 512, "latent_attention_mfma: a latent of %d elements", kv_rank);
  TNX_REQUIRE(rot >= 0 && rot % 8 == 0 && rot <= LM_ROT && 2 * pairs <= rot, "latent_attention_mfma: a rotated part of %d", rot);
  TNX_REQUIRE(page_size > 0 && page_size % 16 == 0 && table_width > 0 && num_pages > 0 && window >= 0 && heads > 0,
              "latent_attention_mfma: bad page sizes");
  TNX_REQUIRE(kv_rank % 8 == 0 && (head_size + rot) % 8 == 0 && head_size % 8 == 0,
              "latent_attention_mfma: query rows of %d + %d elements are not read 16 bytes at a time", head_size, rot);
  TNX_REQUIRE(tile_tokens == 128 || tiles == 0, "latent_attention_mfma: tiles of %d queries", tile_tokens);
  TNX_REQUIRE(decodes == 0 || (splits >= 1 && splits <= 65535 && tiles_per_split >= 1 && (splits == 1 || part)),
              "latent_attention_mfma: %d splits of %d tiles", splits, tiles_per_split);
  TNX_REQUIRE(latent_stride % 8 == 0 && rotated_stride % 8 == 0 && across_stride % 8 == 0,
              "latent_attention_mfma: pages that are not aligned");
  TNX_REQUIRE(!gate || gate_ld >= heads, "latent_attention_mfma: gate rows of %lld elements", gate_ld);
  const LatentFinish fin{sink, gate, gate_ld};
  LatentPages pg = {(const bf16_t*)latent_pages, (const bf16_t*)rotated_pages, (const bf16_t*)across_pages,
                    (size_t)latent_stride, (size_t)rotated_stride, (size_t)across_stride, page_size, num_pages, kv_rank, rot};
#define LM_PROMPT(NDB, QB)                                                                                             \
  latent_attention_prompt_kernel<NDB, QB><<<tiles * (tile_tokens / (64 * QB)) * heads, 256, 0, stream>>>(              \
      (const bf16_t*)q, (const bf16_t*)q_lat, (bf16_t*)out, run_start, cached_lens, block_table, table_width, tile_run, \
      tile_q0, tile_tokens, pg, freqs, pairs, scale, heads, head_size, window, fin)
#define LM_DECODE(NDB)                                                                                          \
  latent_attention_decode_kernel<NDB><<<dim3(decodes, (heads + 15) / 16, splits), 256, 0, stream>>>(            \
      (const bf16_t*)q, (const bf16_t*)q_lat, (bf16_t*)out, run_start, cached_lens, block_table, table_width,   \
      decode_runs, pg, freqs, pairs, scale, heads, head_size, window, part, splits, tiles_per_split, fin)
#define LM_SHARED(NDB, HB)                                                                                            \
  latent_attention_prompt_shared_kernel<NDB, HB><<<tiles * (tile_tokens / 16) * ((heads + HB - 1) / HB), 256, 0, stream>>>( \
      (const bf16_t*)q, (const bf16_t*)q_lat, (bf16_t*)out, run_start, cached_lens, block_table, table_width, tile_run,   \
      tile_q0, tile_tokens, pg, freqs, pairs, scale, heads, head_size, window, fin)
  if (tiles > 0 && prompt_kind == 0) {
    if (kv_rank <= 64) { if (heads >= 4) LM_SHARED(4, 4); else LM_SHARED(4, 1); }
    else if (kv_rank <= 128) { if (heads >= 4) LM_SHARED(8, 4); else LM_SHARED(8, 1); }
    else if (kv_rank <= 256) { if (heads >= 2) LM_SHARED(16, 2); else LM_SHARED(16, 1); }
    else { if (heads >= 2) LM_SHARED(32, 2); else LM_SHARED(32, 1); }
    TNX_CHECK_LAUNCH("latent_attention_prompt_shared");
  } else if (tiles > 0) {
    if (kv_rank <= 64) LM_PROMPT(4, 2);
    else if (kv_rank <= 128) LM_PROMPT(8, 2);
    else if (kv_rank <= 256) LM_PROMPT(16, 1);
    else LM_PROMPT(32, 1);
    TNX_CHECK_LAUNCH("latent_attention_prompt");
  }
#undef LM_SHARED
  if (decodes > 0) {
    if (kv_rank <= 64) LM_DECODE(4);
    else if (kv_rank <= 128) LM_DECODE(8);
    else if (kv_rank <= 256) LM_DECODE(16);
    else LM_DECODE(32);
    TNX_CHECK_LAUNCH("latent_attention_decode");
    if (splits > 1) {
      latent_attention_join_kernel<<<dim3(decodes, heads), 256, 0, stream>>>(part, (bf16_t*)out, run_start, decode_runs,
                                                                            heads, kv_rank, splits, fin);
      TNX_CHECK_LAUNCH("latent_attention_join");
    }
  }
#undef LM_PROMPT
#undef LM_DECODE
  return 0;
}

// ------------------------------------------------------------------------------------------------ prompts, keys expanded

// For steps that are prompts' runs only, the other order of the products pays: the keys W_uk c and the values
// W_uv c of the tokens a run can see are made once a step by library products (from the latents gathered out of
// the pages into dense rows), and attention runs on them as on ordinary keys and values: a (query, key) pair
// then costs 2 (n + r + v) multiply-adds a head instead of 2 (2 R + r).

// row i of the dense latents: the token at `row_pos[i]` of run `row_run[i]` (zeros for a row that pads a run)
__global__ void __launch_bounds__(256)
latent_gather_kernel(const bf16_t* __restrict__ latent_pages, const bf16_t* __restrict__ rotated_pages,
                     size_t latent_stride, size_t rotated_stride, int page_size, int num_pages,
                     const int* __restrict__ table, int table_width, const int* __restrict__ row_run,
                     const int* __restrict__ row_pos, bf16_t* __restrict__ c_dense, bf16_t* __restrict__ r_dense,
                     int kv_rank, int rot) {
  const int i = blockIdx.x;
  const int pos = row_pos[i];
  int page = -1;
  if (pos >= 0) {
    const int b = pos / page_size;
    page = b < table_width ? table[(size_t)row_run[i] * table_width + b] : -1;
    if (page >= num_pages) page = -1;
  }
  const bf16_t* c = page >= 0 ? latent_pages + (size_t)page * latent_stride + (size_t)(pos % page_size) * kv_rank : nullptr;
  const bf16_t* kr = page >= 0 ? rotated_pages + (size_t)page * rotated_stride + (size_t)(pos % page_size) * rot : nullptr;
  for (int d = threadIdx.x; d < kv_rank; d += 256) c_dense[(size_t)i * kv_rank + d] = c ? c[d] : (bf16_t)0.f;
  for (int d = threadIdx.x; d < rot; d += 256) r_dense[(size_t)i * rot + d] = kr ? kr[d] : (bf16_t)0.f;
}

// One block: 64 consecutive queries of one head of one run (QB = 4 blocks of 16 columns). Its four waves work on
// the same 64-key tile: each the scores of 16 keys for all columns, then each a quarter of the value's blocks of
// 16 elements over all 64 keys. `k_n` `[rows, heads * n]`, `k_r` `[rows, rot]` (turned already), `v_t`
// `[heads * v, rows]` (a head's values with the tokens side by side); a run's rows begin at `ctx_start[run]`
// with the token at position `ctx_base[run]` (both multiples of 64).
template <int NKS, int NDV>
__global__ void __launch_bounds__(256)
expanded_attention_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_n, const bf16_t* __restrict__ k_r,
                          const bf16_t* __restrict__ v_t, bf16_t* __restrict__ out, const int* __restrict__ run_start,
                          const int* __restrict__ cached_lens, const int* __restrict__ ctx_start,
                          const int* __restrict__ ctx_base, const int* __restrict__ tile_run,
                          const int* __restrict__ tile_q0, int tile_tokens, size_t rows, const float* __restrict__ freqs,
                          int pairs, float scale, int heads, int head_size, int rot, int value_size, int window,
                          LatentFinish fin) {
  constexpr int QB = 4;
  constexpr int OWN = (NDV + 3) / 4;
  __shared__ float tile_max[4][QB][16], tile_sum[4][QB][16];
  __shared__ __attribute__((aligned(16))) bf16_t prob[QB][16][64 + 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int parts = tile_tokens / (16 * QB);
  const int h = blockIdx.x % heads;
  const int part = (blockIdx.x / heads) % parts, tile = blockIdx.x / heads / parts;
  const int run = tile_run[tile];
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int q0 = tile_q0[tile] + 16 * QB * part;
  if (q0 >= qlen) return;
  const int total = cached + qlen;
  const int base = ctx_base[run];
  const size_t first_row = (size_t)ctx_start[run];
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int qk = head_size + rot;

  bf16x8 qf[QB][NKS];
  int qpos[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = q0 + 16 * qb + r;
    qpos[qb] = cached + qi;
    const bf16_t* qrow = q + ((size_t)(t0 + min(qi, qlen - 1)) * heads + h) * qk;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      qf[qb][ks] = latent_query_chunk(qrow, qrow + head_size, 32 * ks + 8 * g, head_size, rot, qpos[qb], freqs, pairs);
  }
  const int first_q = cached + q0, last_q = cached + min(q0 + 16 * QB - 1, qlen - 1);
  const int lo = max(base, window > 0 ? max(0, first_q - window + 1) : 0);
  float m[QB], l[QB];
  f32x4 o[OWN][QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = -INFINITY;
    l[qb] = 0.f;
#pragma unroll
    for (int j = 0; j < OWN; ++j) o[j][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  for (int tile0 = (lo / 64) * 64; tile0 <= last_q; tile0 += 64) {
    const int key0 = tile0 + 16 * wave;
    f32x4 a[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) a[qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bool live = key0 <= last_q;
    if (live) {
      const size_t row = first_row + (size_t)(key0 - base + r);
      const bf16_t* krow = k_n + (row * heads + h) * head_size;
      const bf16_t* rrow = k_r + row * rot;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = 32 * ks + 8 * g;
        bf16x8 kf = zero8;
        if (d0 < head_size) kf = *(const bf16x8*)(krow + d0);
        else if (d0 < qk) kf = *(const bf16x8*)(rrow + (d0 - head_size));
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) a[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qb][ks], a[qb], 0, 0, 0);
      }
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 4 * g + i;
        const bool ok = live && key <= qpos[qb] && (window <= 0 || key > qpos[qb] - window);
        a[qb][i] = ok ? a[qb][i] * scale : -INFINITY;
        mx = fmaxf(mx, a[qb][i]);
      }
      mx = rows_max(mx);
      if (g == 0) tile_max[wave][qb][r] = mx;
    }
    __syncthreads();
    float alpha[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float m_new = fmaxf(m[qb], fmaxf(fmaxf(tile_max[0][qb][r], tile_max[1][qb][r]),
                                             fmaxf(tile_max[2][qb][r], tile_max[3][qb][r])));
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[qb] = __expf(m[qb] - m_safe);
      m[qb] = m_new;
      float sum = 0.f;
      bf16x4 p4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = __expf(a[qb][i] - m_safe);
        sum += pr;
        p4[i] = (bf16_t)pr;
      }
      sum = rows_sum(sum);
      *(bf16x4*)&prob[qb][r][16 * wave + 4 * g] = p4;
      if (g == 0) tile_sum[wave][qb][r] = sum;
    }
    __syncthreads();
    bf16x8 pb[QB][2];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      l[qb] = l[qb] * alpha[qb] + ((tile_sum[0][qb][r] + tile_sum[1][qb][r]) + (tile_sum[2][qb][r] + tile_sum[3][qb][r]));
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) pb[qb][s2] = *(const bf16x8*)&prob[qb][r][32 * s2 + 8 * g];
    }
    const bool tail = tile0 + 64 > total;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= value_size) continue;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[j][qb][i] *= alpha[qb];
      const bf16_t* vrow = v_t + ((size_t)h * value_size + 16 * db + r) * rows + first_row + (size_t)(tile0 - base);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        bf16x8 vf = zero8;
        if (tile0 + 32 * s2 <= last_q) vf = *(const bf16x8*)(vrow + 32 * s2 + 8 * g);
        if (tail) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (tile0 + 32 * s2 + 8 * g + e >= total) vf[e] = 0;
        }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o[j][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[qb][s2], o[j][qb], 0, 0, 0);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = q0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = latent_finish(fin, m[qb], l[qb], t0 + qi, h);
    bf16_t* orow = out + ((size_t)(t0 + qi) * heads + h) * value_size;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int db = wave + 4 * j;
      if (16 * db >= value_size) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[j][qb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

extern "C" int tnx_latent_gather(const void* latent_pages, const void* rotated_pages, long long latent_stride,
                                 long long rotated_stride, int page_size, int num_pages, const int* block_table,
                                 int table_width, const int* row_run, const int* row_pos, void* c_dense, void* r_dense,
                                 int kv_rank, int rot, int rows, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && kv_rank > 0 && rot >= 0 && page_size > 0 && table_width > 0 && num_pages > 0,
              "latent_gather: bad sizes");
  if (rows == 0) return 0;
  latent_gather_kernel<<<rows, 256, 0, stream>>>((const bf16_t*)latent_pages, (const bf16_t*)rotated_pages,
                                                 (size_t)latent_stride, (size_t)rotated_stride, page_size, num_pages,
                                                 block_table, table_width, row_run, row_pos, (bf16_t*)c_dense,
                                                 (bf16_t*)r_dense, kv_rank, rot);
  TNX_CHECK_LAUNCH("latent_gather");
  return 0;
}

extern "C" int tnx_expanded_attention(const void* q, const void* k_n, const void* k_r, const void* v_t, void* out,
                                      const int* run_start, const int* cached_lens, const int* ctx_start,
                                      const int* ctx_base, const int* tile_run, const int* tile_q0, int tiles,
                                      int tile_tokens, long long rows, const float* freqs, int pairs, float scale,
                                      int heads, int head_size, int rot, int value_size, int window, const float* sink,
                                      const float* gate, long long gate_ld, hipStream_t stream) {
  TNX_REQUIRE(tiles >= 0 && heads > 0 && head_size > 0 && head_size % 8 == 0 && rot >= 0 && rot % 8 == 0 &&
                  head_size + rot <= 256 && 2 * pairs <= rot,
              "expanded_attention: query/key sizes %d + %d", head_size, rot);
  TNX_REQUIRE(value_size > 0 && value_size % 16 == 0 && value_size <= 256, "expanded_attention: a value of %d elements", value_size);
  TNX_REQUIRE(tile_tokens == 128 && rows % 64 == 0 && window >= 0, "expanded_attention: tiles of %d queries, %lld rows",
              tile_tokens, rows);
  TNX_REQUIRE(!gate || gate_ld >= heads, "expanded_attention: gate rows of %lld elements", gate_ld);
  if (tiles == 0) return 0;
  const LatentFinish fin{sink, gate, gate_ld};
  const int grid = tiles * (tile_tokens / 64) * heads;
  const int nks = (head_size + rot + 31) / 32, ndv = value_size / 16;
#define EA_LAUNCH(NKS, NDV)                                                                                          \
  expanded_attention_kernel<NKS, NDV><<<grid, 256, 0, stream>>>(                                                     \
      (const bf16_t*)q, (const bf16_t*)k_n, (const bf16_t*)k_r, (const bf16_t*)v_t, (bf16_t*)out, run_start,          \
      cached_lens, ctx_start, ctx_base, tile_run, tile_q0, tile_tokens, (size_t)rows, freqs, pairs, scale, heads,     \
      head_size, rot, value_size, window, fin)
#define EA_VALUES(NKS)                        \
  if (ndv <= 4) { EA_LAUNCH(NKS, 4); }        \
  else if (ndv <= 8) { EA_LAUNCH(NKS, 8); }   \
  else { EA_LAUNCH(NKS, 16); }
  if (nks <= 2) { EA_VALUES(2) }
  else if (nks <= 4) { EA_VALUES(4) }
  else if (nks <= 6) { EA_VALUES(6) }
  else { EA_VALUES(8) }
#undef EA_VALUES
#undef EA_LAUNCH
  TNX_CHECK_LAUNCH("expanded_attention");
  return 0;
}
