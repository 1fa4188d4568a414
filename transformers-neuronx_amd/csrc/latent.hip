// Latent attention: a token's keys and values are made from one small cached vector c (R elements) and a
// rotated key part k_r (r elements) that all heads share. The products with the key and value matrices are
// moved to the query's side, so the kernels read the cache as it lies:
//   score(i, j, head) = q_lat[i, head] . c[j] + scale * turn(q_r[i, head]) . k_r[j],   out[i, head] = sum_j p_j c[j].
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

// One block a token. `down[t]` = [Q | R | r] float32: the first Q, scaled to unit root mean square and
// weighted, go to `c_q`; the next R likewise to the token's place in the latent pages; the last r, pairs
// (2i, 2i + 1) turned for i < pairs, to its place in the rotated pages. R = 0: a mixer without a latent of its own.
__global__ void __launch_bounds__(256)
latent_norms_kernel(const float* __restrict__ down, int q_rank, int kv_rank, int rot, const float* __restrict__ q_w,
                    const float* __restrict__ kv_w, float eps, const float* __restrict__ freqs, int pairs,
                    const int* __restrict__ positions, const int* __restrict__ token_page,
                    const int* __restrict__ token_offset, void* __restrict__ c_q, int dtype,
                    void* __restrict__ latent_pages, void* __restrict__ rotated_pages, size_t latent_stride,
                    size_t rotated_stride, int num_pages) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* row = down + (size_t)t * (q_rank + kv_rank + rot);
  float s = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += 256) s += row[i] * row[i];
  const float rq = 1.f / sqrtf(block_sum<4>(s, scratch) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += 256) store_any(c_q, dtype, (size_t)t * q_rank + i, row[i] * rq * q_w[i]);
  if (kv_rank == 0) return;
  const int page = token_page[t];
  if (page < 0 || page >= num_pages) return;  // the host checks that every token has a page
  const int off = token_offset[t];
  const float* lat = row + q_rank;
  s = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += 256) s += lat[i] * lat[i];
  const float rk = 1.f / sqrtf(block_sum<4>(s, scratch) / (float)kv_rank + eps);
  const size_t at = (size_t)page * latent_stride + (size_t)off * kv_rank;
  for (int i = threadIdx.x; i < kv_rank; i += 256) store_any(latent_pages, dtype, at + i, lat[i] * rk * kv_w[i]);
  const float* kr = lat + kv_rank;
  const size_t rat = (size_t)page * rotated_stride + (size_t)off * rot;
  for (int i = threadIdx.x; i < rot / 2; i += 256) {
    float a = kr[2 * i], b = kr[2 * i + 1];
    if (i < pairs) turn_pair(kr[2 * i], kr[2 * i + 1], positions[t], freqs[i], a, b);
    store_any(rotated_pages, dtype, rat + 2 * i, a);
    store_any(rotated_pages, dtype, rat + 2 * i + 1, b);
  }
}

extern "C" int tnx_latent_norms(const float* down, int q_rank, int kv_rank, int rot, const float* q_w,
                                const float* kv_w, float eps, const float* freqs, int pairs, const int* positions,
                                const int* token_page, const int* token_offset, void* c_q, int dtype,
                                void* latent_pages, void* rotated_pages, long long latent_stride,
                                long long rotated_stride, int num_pages, int page_size, int tokens,
                                hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && q_rank > 0 && kv_rank >= 0 && rot >= 0 && rot % 2 == 0 && (kv_rank == 0 || 2 * pairs <= rot),
              "latent_norms: bad sizes q=%d kv=%d rot=%d pairs=%d", q_rank, kv_rank, rot, pairs);
  TNX_REQUIRE(kv_rank == 0 || (latent_pages && rotated_pages && kv_w && latent_stride >= (long long)page_size * kv_rank &&
                               rotated_stride >= (long long)page_size * rot),
              "latent_norms: pages too small for their tokens");
  if (tokens == 0) return 0;
  latent_norms_kernel<<<tokens, 256, 0, stream>>>(down, q_rank, kv_rank, kv_rank ? rot : 0, q_w, kv_w, eps, freqs, pairs,
                                                  positions, token_page, token_offset, c_q, dtype, latent_pages,
                                                  rotated_pages, (size_t)latent_stride, (size_t)rotated_stride,
                                                  num_pages);
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

extern "C" int tnx_batched_linear(const void* x, int x_dtype, long long x_row, long long x_head, const void* w,
                                  int w_dtype, void* out, int out_dtype, float alpha, int tokens, int heads, int n_out,
                                  int k_in, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && heads > 0 && n_out > 0 && k_in > 0, "batched_linear: bad sizes");
  TNX_REQUIRE(heads <= 65535 && (tokens + BL_TILE - 1) / BL_TILE <= 65535, "batched_linear: too many heads or tokens");
  if (tokens == 0) return 0;
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
                            float scale, int heads, int head_size, int rot, int kv_rank, int window) {
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
  for (int i = threadIdx.x; i < kv_rank; i += 256) ql[i] = to_f32(q_lat[((size_t)t * heads + h) * kv_rank + i]);
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
  const float inv = l > 0.f ? 1.f / l : 0.f;
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
                                        int kv_rank, int window, int tokens, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && heads > 0 && heads <= 65535 && kv_rank > 0 && rot >= 0 && rot % 2 == 0 && 2 * pairs <= rot,
              "latent_attention: bad sizes heads=%d kv_rank=%d rot=%d", heads, kv_rank, rot);
  TNX_REQUIRE(kv_rank <= 256 * LA_OWN, "latent_attention: a latent of %d elements is more than %d", kv_rank, 256 * LA_OWN);
  TNX_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0 && window >= 0, "latent_attention: bad page sizes");
  if (tokens == 0) return 0;
  const size_t lds = (size_t)(kv_rank + rot + 512) * sizeof(float);
  const dim3 grid(tokens, heads);
  if (dtype == TNX_F32)
    latent_attention_any_kernel<float><<<grid, 256, lds, stream>>>(
        (const float*)q, (const float*)q_lat, (float*)out, positions, token_request, block_table, table_width, page_size,
        num_pages, (const float*)latent_pages, (const float*)rotated_pages, (size_t)latent_stride, (size_t)rotated_stride,
        freqs, pairs, scale, heads, head_size, rot, kv_rank, window);
  else
    latent_attention_any_kernel<bf16_t><<<grid, 256, lds, stream>>>(
        (const bf16_t*)q, (const bf16_t*)q_lat, (bf16_t*)out, positions, token_request, block_table, table_width,
        page_size, num_pages, (const bf16_t*)latent_pages, (const bf16_t*)rotated_pages, (size_t)latent_stride,
        (size_t)rotated_stride, freqs, pairs, scale, heads, head_size, rot, kv_rank, window);
  TNX_CHECK_LAUNCH("latent_attention_any");
  return 0;
}
