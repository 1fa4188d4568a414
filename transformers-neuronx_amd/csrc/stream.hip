// Kernels around the residual stream that are no matrix products: a token table with a row for the pair of a
// token and the one before it, the norm that follows a part and joins its result to the stream, the short
// causal convolution before a part with its per-request state, the activation made of normed powers, a
// product with columns of a table's rows, and the weighted sum over what earlier layers left.
// Statistics, sums and state are float32.
#include "common.h"

TNX_DEFINE_ERROR_API

// ------------------------------------------------------------------------------------------------ pair table

__device__ __forceinline__ int resolve_token(const int* ids, int t, const int* kept, int kept_size) {
  int v = ids[t];
  if (v < 0 && kept && -1 - v < kept_size) v = kept[-1 - v];
  return v;
}

// out[t, :] = table[token, :] + pairs[row, :] in float32; row = (previous * mul_prev + token * mul_cur) mod
// buckets, `buckets` for a request's first token. A request keeps its last token in `last_token[slot, p & 1]`, p
// the token's position: the token before a run's first is read from the other place than the run's last is
// written to, so a step of single tokens that is run twice (recorded once, then replayed) reads the same.
__global__ void __launch_bounds__(256)
embed_pairs_kernel(const int* __restrict__ ids, const int* __restrict__ kept, int kept_size,
                   const void* __restrict__ table, const void* __restrict__ pairs, int dtype, int vocab, int buckets,
                   long long mul_prev, long long mul_cur, const int* __restrict__ positions,
                   const int* __restrict__ token_request, const int* __restrict__ run_start,
                   const int* __restrict__ slots, const int* __restrict__ last_token, float* __restrict__ out,
                   int width) {
  const int t = blockIdx.x;
  const int tok = resolve_token(ids, t, kept, kept_size);
  if (tok < 0 || tok >= vocab) return;  // the host checks ids
  int row = buckets;
  if (positions[t] != 0) {
    const int r = token_request[t];
    const long long before = t == run_start[r] ? (long long)last_token[2 * slots[r] + ((positions[t] - 1) & 1)]
                                               : (long long)resolve_token(ids, t - 1, kept, kept_size);
    long long v = (before * mul_prev + (long long)tok * mul_cur) % (long long)buckets;
    if (v < 0) v += buckets;
    row = (int)v;
  }
  const size_t a = (size_t)tok * width, b = (size_t)row * width, o = (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += 256) out[o + i] = load_any(table, dtype, a + i) + load_any(pairs, dtype, b + i);
}

// the run's last token goes to its place, after every run has read what was there
__global__ void keep_last_token_kernel(const int* __restrict__ ids, const int* __restrict__ kept, int kept_size,
                                       const int* __restrict__ positions, const int* __restrict__ run_start,
                                       const int* __restrict__ slots, int* __restrict__ last_token, int runs) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= runs || run_start[r + 1] == run_start[r]) return;
  const int t = run_start[r + 1] - 1;
  last_token[2 * slots[r] + (positions[t] & 1)] = resolve_token(ids, t, kept, kept_size);
}

extern "C" int tnx_embed_pairs(const int* ids, const int* kept, int kept_size, const void* table, const void* pairs,
                               int dtype, int vocab, int buckets, long long mul_prev, long long mul_cur,
                               const int* positions, const int* token_request, const int* run_start, const int* slots,
                               int* last_token, float* out, int tokens, int width, int runs, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && buckets > 0 && runs >= 0, "embed_pairs: bad sizes");
  if (tokens == 0) return 0;
  embed_pairs_kernel<<<tokens, 256, 0, stream>>>(ids, kept, kept ? kept_size : 0, table, pairs, dtype, vocab, buckets,
                                                 mul_prev, mul_cur, positions, token_request, run_start, slots,
                                                 last_token, out, width);
  TNX_CHECK_LAUNCH("embed_pairs");
  keep_last_token_kernel<<<(runs + 255) / 256, 256, 0, stream>>>(ids, kept, kept ? kept_size : 0, positions, run_start,
                                                                 slots, last_token, runs);
  TNX_CHECK_LAUNCH("keep_last_token");
  return 0;
}

// ------------------------------------------------------------------------------------------------ norm, then the sum

// out = residual + mult * ((y - mean) * rstd * weight + bias), the row's statistics in float32 (the variance
// about the mean; `center` 0: the mean taken as 0). One block a row, the row read three times (it is in cache).
__global__ void __launch_bounds__(256)
norm_add_kernel(const float* __restrict__ y, const float* __restrict__ weight, const float* __restrict__ bias,
                float eps, int center, const float* residual, float mult, float* out, int width) {
  __shared__ float scratch[4];
  const size_t base = (size_t)blockIdx.x * width;
  const float* row = y + base;
  float s = 0.f;
  if (center)
    for (int i = threadIdx.x; i < width; i += 256) s += row[i];
  const float mean = center ? block_sum<4>(s, scratch) / (float)width : 0.f;
  float q = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float d = row[i] - mean;
    q += d * d;
  }
  const float rstd = 1.f / sqrtf(block_sum<4>(q, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += 256) {
    float v = (row[i] - mean) * rstd;
    if (weight) v *= weight[i];
    if (bias) v += bias[i];
    out[base + i] = residual[base + i] + mult * v;
  }
}

extern "C" int tnx_norm_add(const float* y, const float* weight, const float* bias, float eps, int center,
                            const float* residual, float mult, float* out, int tokens, int width, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && eps > 0.f, "norm_add: bad sizes tokens=%d width=%d", tokens, width);
  TNX_REQUIRE(y && residual && out && out != y, "norm_add: the result may not lie where the normed rows do");
  if (tokens == 0) return 0;
  norm_add_kernel<<<tokens, 256, 0, stream>>>(y, weight, bias, eps, center, residual, mult, out, width);
  TNX_CHECK_LAUNCH("norm_add");
  return 0;
}

// ------------------------------------------------------------------------------------------------ input convolution

// out[t, d] = h[t, d] + sum_j w[d, j] * h[t - taps + 1 + j, d] over the tokens of t's own request (zeros before
// its start). Inputs from before the step's run come from the request's state, `[taps, width]`: the input at
// position p lies at place p mod taps. A run's last taps - 1 inputs are written behind the kernel that reads, by
// another launch; with one place more than is kept, a step of single tokens writes where it does not read, so
// that running it twice (recorded once, then replayed) reads the same.
__global__ void __launch_bounds__(256)
input_conv_kernel(const float* __restrict__ h, const float* __restrict__ w, const float* __restrict__ state,
                  size_t slot_stride, int taps, const int* __restrict__ positions,
                  const int* __restrict__ token_request, const int* __restrict__ run_start,
                  const int* __restrict__ slots, void* __restrict__ out, int out_dtype, int width) {
  const int t = blockIdx.x;
  const int r = token_request[t];
  const int first = run_start[r];
  const int i = t - first, p = positions[t];
  const float* mine = state ? state + (size_t)slots[r] * slot_stride : nullptr;
  for (int d = threadIdx.x; d < width; d += 256) {
    float acc = h[(size_t)t * width + d];
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;           // the input `back` tokens before this one
      float x = 0.f;
      if (back <= i)
        x = h[(size_t)(t - back) * width + d];
      else if (back <= p && mine)
        x = mine[(size_t)((p - back) % taps) * width + d];
      acc += w[(size_t)d * taps + j] * x;
    }
    store_any(out, out_dtype, (size_t)t * width + d, acc);
  }
}

__global__ void __launch_bounds__(256)
conv_state_kernel(const float* __restrict__ h, float* __restrict__ state, size_t slot_stride, int taps,
                  const int* __restrict__ positions, const int* __restrict__ run_start,
                  const int* __restrict__ slots, int width) {
  const int r = blockIdx.y;
  const int d = blockIdx.x * 256 + threadIdx.x;
  const int first = run_start[r], n = run_start[r + 1] - first;
  if (d >= width || n == 0) return;
  float* mine = state + (size_t)slots[r] * slot_stride;
  for (int i = max(0, n - (taps - 1)); i < n; ++i)
    mine[(size_t)(positions[first + i] % taps) * width + d] = h[(size_t)(first + i) * width + d];
}

// `state` is `[slots, slot_stride]` floats with this convolution's `[taps, width]` at the pointer given
// (null for taps of 1, which keep nothing).
extern "C" int tnx_input_conv(const float* h, const float* w, float* state, long long slot_stride, int taps,
                              const int* positions, const int* token_request, const int* run_start, const int* slots,
                              void* out, int out_dtype, int tokens, int width, int runs, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && taps >= 1 && runs >= 0, "input_conv: bad sizes");
  TNX_REQUIRE(taps == 1 || state, "input_conv: %d taps need the requests' state", taps);
  TNX_REQUIRE((const void*)h != out, "input_conv: the result may not lie where the inputs do");
  if (tokens == 0) return 0;
  input_conv_kernel<<<tokens, 256, 0, stream>>>(h, w, taps > 1 ? state : nullptr, (size_t)slot_stride, taps, positions,
                                                token_request, run_start, slots, out, out_dtype, width);
  TNX_CHECK_LAUNCH("input_conv");
  if (taps > 1) {
    conv_state_kernel<<<dim3((width + 255) / 256, runs), 256, 0, stream>>>(h, state, (size_t)slot_stride, taps,
                                                                          positions, run_start, slots, width);
    TNX_CHECK_LAUNCH("conv_state");
  }
  return 0;
}

// ------------------------------------------------------------------------------------------------ normed powers

// out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row.
__global__ void __launch_bounds__(256)
poly_norm_kernel(const float* __restrict__ z, const float* __restrict__ coeffs, float eps, void* __restrict__ out,
                 int out_dtype, int width) {
  __shared__ float scratch[4];
  const size_t base = (size_t)blockIdx.x * width;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = z[base + i], v2 = v * v, v3 = v2 * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v3 * v3;
  }
  const float r1 = 1.f / sqrtf(block_sum<4>(s2, scratch) / (float)width + eps);
  const float r2 = 1.f / sqrtf(block_sum<4>(s4, scratch) / (float)width + eps);
  const float r3 = 1.f / sqrtf(block_sum<4>(s6, scratch) / (float)width + eps);
  const float a = coeffs[0] * r1, b = coeffs[1] * r2, c = coeffs[2] * r3, e = coeffs[3];
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = z[base + i], v2 = v * v;
    store_any(out, out_dtype, base + i, a * v + b * v2 + c * (v2 * v) + e);
  }
}

extern "C" int tnx_poly_norm(const float* z, const float* coeffs, float eps, void* out, int out_dtype, int tokens,
                             int width, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && eps > 0.f, "poly_norm: bad sizes tokens=%d width=%d", tokens, width);
  if (tokens == 0) return 0;
  poly_norm_kernel<<<tokens, 256, 0, stream>>>(z, coeffs, eps, out, out_dtype, width);
  TNX_CHECK_LAUNCH("poly_norm");
  return 0;
}

// ------------------------------------------------------------------------------------------------ small ones

// out[t, i] = g[t, i] * rows[t, offset + i]
__global__ void mul_columns_kernel(const void* __restrict__ g, const void* __restrict__ rows, int dtype, int offset,
                                   int dim, int columns, void* __restrict__ out, size_t n) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const size_t t = e / dim;
  const int i = (int)(e % dim);
  store_any(out, dtype, e, load_any(g, dtype, e) * load_any(rows, dtype, t * columns + offset + i));
}

extern "C" int tnx_mul_columns(const void* g, const void* rows, int dtype, int offset, int dim, int columns, void* out,
                               int tokens, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && dim > 0 && offset >= 0 && offset + dim <= columns, "mul_columns: columns %d..%d of %d",
              offset, offset + dim, columns);
  if (tokens == 0) return 0;
  const size_t n = (size_t)tokens * dim;
  mul_columns_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(g, rows, dtype, offset, dim, columns, out, n);
  TNX_CHECK_LAUNCH("mul_columns");
  return 0;
}

// out[e] = sum_j weights[j] * history[j * slot_stride + e], j < count, added in the order of j
__global__ void weighted_sum_kernel(const float* __restrict__ history, const float* __restrict__ weights, int count,
                                    size_t slot_stride, float* __restrict__ out, size_t n) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  float acc = 0.f;
  for (int j = 0; j < count; ++j) acc += weights[j] * history[(size_t)j * slot_stride + e];
  out[e] = acc;
}

extern "C" int tnx_weighted_sum(const float* history, const float* weights, int count, long long slot_stride,
                                float* out, long long n, hipStream_t stream) {
  TNX_REQUIRE(count >= 1 && n >= 0 && slot_stride >= n, "weighted_sum: bad sizes");
  if (n == 0) return 0;
  weighted_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(history, weights, count, (size_t)slot_stride,
                                                                       out, (size_t)n);
  TNX_CHECK_LAUNCH("weighted_sum");
  return 0;
}
