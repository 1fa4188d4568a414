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


// ------------------------------------------------------------------------------------------------ rows in registers

__global__ void conv_state_kernel(const float* __restrict__ h, float* __restrict__ state, size_t slot_stride, int taps,
                                  const int* __restrict__ positions, const int* __restrict__ run_start,
                                  const int* __restrict__ slots, int width);

// The same row kernels for widths that are multiples of 4 up to 1024 * PER: a thread holds PER chunks of four
// floats of the row (chunk c at element 4 * (threadIdx.x + 256 * c)), so a row is read once.
typedef __attribute__((ext_vector_type(4))) float rf4;
typedef __attribute__((ext_vector_type(4))) __bf16 rb4;

template <int PER>
__device__ __forceinline__ void row_load(const float* row, int w4, rf4 (&v)[PER]) {
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int i = threadIdx.x + 256 * c;
    v[c] = i < w4 ? ((const rf4*)row)[i] : (rf4){0.f, 0.f, 0.f, 0.f};
  }
}

// v <- (v - mean) * rstd * weight + bias (the mean taken as 0 without `center`), statistics over the block
template <int PER>
__device__ __forceinline__ void row_norm(rf4 (&v)[PER], int w4, int width, const float* weight, const float* bias,
                                         float eps, int center, float* scratch) {
  float s = 0.f;
  if (center) {
#pragma unroll
    for (int c = 0; c < PER; ++c) s += (v[c].x + v[c].y) + (v[c].z + v[c].w);
  }
  const float mean = center ? block_sum<4>(s, scratch) / (float)width : 0.f;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    if (threadIdx.x + 256 * c < w4) {
      const rf4 d = v[c] - mean;
      q += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
    }
  }
  const float rstd = 1.f / sqrtf(block_sum<4>(q, scratch) / (float)width + eps);
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int i = threadIdx.x + 256 * c;
    if (i < w4) {
      rf4 y = (v[c] - mean) * rstd;
      if (weight) y = y * ((const rf4*)weight)[i];
      if (bias) y = y + ((const rf4*)bias)[i];
      v[c] = y;
    }
  }
}

// a vector's chunks as `row_load` lays a row out; zeros for a vector that is not there
template <int PER>
__device__ __forceinline__ void vector_load(const float* vec, int w4, float fill, rf4 (&v)[PER]) {
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int i = threadIdx.x + 256 * c;
    v[c] = (vec && i < w4) ? ((const rf4*)vec)[i] : (rf4){fill, fill, fill, fill};
  }
}

// `row_norm` with the weight and the bias in registers already (ones and zeros where there is none)
template <int PER>
__device__ __forceinline__ void row_norm_held(rf4 (&v)[PER], int w4, int width, const rf4 (&weight)[PER],
                                              const rf4 (&bias)[PER], float eps, int center, float* scratch) {
  float s = 0.f;
  if (center) {
#pragma unroll
    for (int c = 0; c < PER; ++c) s += (v[c].x + v[c].y) + (v[c].z + v[c].w);
  }
  const float mean = center ? block_sum<4>(s, scratch) / (float)width : 0.f;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    if (threadIdx.x + 256 * c < w4) {
      const rf4 d = v[c] - mean;
      q += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
    }
  }
  const float rstd = 1.f / sqrtf(block_sum<4>(q, scratch) / (float)width + eps);
#pragma unroll
  for (int c = 0; c < PER; ++c)
    if (threadIdx.x + 256 * c < w4) v[c] = (v[c] - mean) * rstd * weight[c] + bias[c];   // (chunks beyond the row stay zero)
}

__device__ __forceinline__ void store_chunk(void* out, int dtype, size_t chunk, rf4 y) {
  if (dtype == TNX_F32) {
    ((rf4*)out)[chunk] = y;
  } else {
    rb4 o;
    o.x = (bf16_t)y.x; o.y = (bf16_t)y.y; o.z = (bf16_t)y.z; o.w = (bf16_t)y.w;
    ((rb4*)out)[chunk] = o;
  }
}

// out = residual + mult * norm(y), and a copy in another dtype beside it if asked for
template <int PER>
__global__ void __launch_bounds__(256)
norm_add_rows_kernel(const float* __restrict__ y, const float* __restrict__ weight, const float* __restrict__ bias,
                     float eps, int center, const float* residual, float mult, float* out, void* __restrict__ copy,
                     int copy_dtype, int width) {
  __shared__ float scratch[4];
  const int w4 = width >> 2;
  const size_t base = (size_t)blockIdx.x * w4;
  rf4 v[PER];
  row_load<PER>(y + (size_t)blockIdx.x * width, w4, v);
  row_norm<PER>(v, w4, width, weight, bias, eps, center, scratch);
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int i = threadIdx.x + 256 * c;
    if (i < w4) {
      const rf4 r = ((const rf4*)residual)[base + i] + mult * v[c];
      ((rf4*)out)[base + i] = r;
      if (copy) store_chunk(copy, copy_dtype, base + i, r);
    }
  }
}

// What a part reads, in one launch: for a token t of a run, h_t = pre_norm(x'_t), out_t = h_t + conv(h)_t, where
// x' = x, or with `y`, x' = x + mult * post_norm(y) (the part before, joined to the stream here; x'_t is written
// to `x_out`). The rows of the taps - 1 tokens before t are made again by this block where they lie in the
// step's run, and come from the request's state otherwise (`[taps, width]`, position p at place p mod taps).
// `h_keep`: where a run's last taps - 1 tokens leave their h for the launch that writes the state afterwards;
// with `write_state` (every run of the step is one token) this kernel writes the state itself.
// TAPS: the number of taps where it is 1 to 4 (what is read from the state and the weights are then asked for
// before the first reduction, and nothing waits for them afterwards); 0: any number, taken as it comes.
template <int PER, int TAPS>
__global__ void __launch_bounds__(256)
join_norm_conv_kernel(const float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ post_w,
                      const float* __restrict__ post_b, int post_center, float mult, float* __restrict__ x_out,
                      const float* __restrict__ pre_w, const float* __restrict__ pre_b, int pre_center, float eps,
                      const float* __restrict__ conv_w, float* state, size_t slot_stride, int taps_given,
                      const int* __restrict__ positions, const int* __restrict__ token_request,
                      const int* __restrict__ run_start, const int* __restrict__ slots, void* __restrict__ out,
                      int out_dtype, float* __restrict__ h_keep, int write_state, int width) {
  __shared__ float scratch[4];
  const int taps = TAPS > 0 ? TAPS : taps_given;
  constexpr int KEPT = TAPS > 1 ? TAPS - 1 : 1;
  const int w4 = width >> 2;
  const int t = blockIdx.x;
  const int r = token_request[t];
  const int first = run_start[r], n = run_start[r + 1] - first;
  const int i = t - first, p = positions[t];
  float* mine = state ? state + (size_t)slots[r] * slot_stride : nullptr;
  rf4 acc[PER], v[PER];
#pragma unroll
  for (int c = 0; c < PER; ++c) acc[c] = (rf4){0.f, 0.f, 0.f, 0.f};
  // the norms' vectors, the taps' weights and what comes from the state, all asked for at once
  rf4 pw[PER], pb[PER], qw[PER], qb[PER];
  vector_load<PER>(pre_w, w4, 1.f, pw);
  vector_load<PER>(pre_b, w4, 0.f, pb);
  vector_load<PER>(y ? post_w : nullptr, w4, 1.f, qw);
  vector_load<PER>(y ? post_b : nullptr, w4, 0.f, qb);
  rf4 taps_w[TAPS > 0 ? TAPS : 1][PER];
  if (TAPS > 0) {
#pragma unroll
    for (int j = 0; j < (TAPS > 0 ? TAPS : 1); ++j)
#pragma unroll
      for (int c = 0; c < PER; ++c) {
        const int k = threadIdx.x + 256 * c;
        taps_w[j][c] = ((const rf4*)(conv_w + (size_t)j * width))[min(k, w4 - 1)];
      }
  }
  rf4 kept[KEPT][PER];
  if (TAPS > 1) {
#pragma unroll
    for (int back = 1; back < (TAPS > 1 ? TAPS : 1); ++back) {
      if (back > i && back <= p && mine) {
        row_load<PER>(mine + (size_t)((p - back) % taps) * width, w4, kept[back - 1]);
      } else {
#pragma unroll
        for (int c = 0; c < PER; ++c) kept[back - 1][c] = (rf4){0.f, 0.f, 0.f, 0.f};
      }
    }
  }
#pragma unroll 1
  for (int back = taps - 1; back >= 0; --back) {
    if (back <= i) {
      const size_t row = (size_t)(t - back) * width;
      row_load<PER>(x + row, w4, v);
      if (y) {
        rf4 u[PER];
        row_load<PER>(y + row, w4, u);
        row_norm_held<PER>(u, w4, width, qw, qb, eps, post_center, scratch);
#pragma unroll
        for (int c = 0; c < PER; ++c) {
          v[c] = v[c] + mult * u[c];
          const int k = threadIdx.x + 256 * c;
          if (back == 0 && k < w4) ((rf4*)(x_out + row))[k] = v[c];
        }
      }
      row_norm_held<PER>(v, w4, width, pw, pb, eps, pre_center, scratch);
    } else if (TAPS > 1) {
      if (back > p) continue;
#pragma unroll
      for (int b = 1; b < (TAPS > 1 ? TAPS : 1); ++b)
        if (b == back) {
#pragma unroll
          for (int c = 0; c < PER; ++c) v[c] = kept[b - 1][c];
        }
    } else if (back <= p && mine) {
      row_load<PER>(mine + (size_t)((p - back) % taps) * width, w4, v);
    } else {
      continue;      // before the request's start: zeros
    }
    const int j = taps - 1 - back;
#pragma unroll
    for (int c = 0; c < PER; ++c) {
      const int k = threadIdx.x + 256 * c;
      if (k < w4) {
        rf4 wj;
        if (TAPS > 0) {
          wj = taps_w[0][c];
#pragma unroll
          for (int jj = 1; jj < (TAPS > 0 ? TAPS : 1); ++jj)
            if (jj == j) wj = taps_w[jj][c];
        } else {
          wj = ((const rf4*)(conv_w + (size_t)j * width))[k];
        }
        acc[c] = acc[c] + wj * v[c];
        if (back == 0) acc[c] = acc[c] + v[c];
      }
    }
  }
  // (v holds h_t now)
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int k = threadIdx.x + 256 * c;
    if (k < w4) {
      store_chunk(out, out_dtype, (size_t)t * w4 + k, acc[c]);
      if (taps > 1 && i >= n - (taps - 1)) {
        if (write_state) ((rf4*)(mine + (size_t)(p % taps) * width))[k] = v[c];
        else ((rf4*)(h_keep + (size_t)t * width))[k] = v[c];
      }
    }
  }
}

template <int PER>
__global__ void __launch_bounds__(256)
poly_norm_rows_kernel(const float* __restrict__ z, const float* __restrict__ coeffs, float eps, void* __restrict__ out,
                      int out_dtype, int width) {
  __shared__ float scratch[4];
  const int w4 = width >> 2;
  rf4 v[PER];
  row_load<PER>(z + (size_t)blockIdx.x * width, w4, v);
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const rf4 a = v[c] * v[c], b = a * a, d = b * a;
    s2 += (a.x + a.y) + (a.z + a.w);
    s4 += (b.x + b.y) + (b.z + b.w);
    s6 += (d.x + d.y) + (d.z + d.w);
  }
  const float r1 = 1.f / sqrtf(block_sum<4>(s2, scratch) / (float)width + eps);
  const float r2 = 1.f / sqrtf(block_sum<4>(s4, scratch) / (float)width + eps);
  const float r3 = 1.f / sqrtf(block_sum<4>(s6, scratch) / (float)width + eps);
  const float a = coeffs[0] * r1, b = coeffs[1] * r2, c3 = coeffs[2] * r3, e = coeffs[3];
#pragma unroll
  for (int c = 0; c < PER; ++c) {
    const int k = threadIdx.x + 256 * c;
    if (k < w4) {
      const rf4 x1 = v[c], x2 = x1 * x1;
      store_chunk(out, out_dtype, (size_t)blockIdx.x * w4 + k, a * x1 + b * x2 + c3 * (x2 * x1) + e);
    }
  }
}

#define ROWS_DISPATCH(width, LAUNCH)      \
  if (width <= 1024) { LAUNCH(1); }       \
  else if (width <= 2048) { LAUNCH(2); }  \
  else if (width <= 4096) { LAUNCH(4); }  \
  else if (width <= 8192) { LAUNCH(8); }  \
  else { LAUNCH(16); }

static inline bool rows_fit(int width) { return width % 4 == 0 && width <= 16384; }

// `copy` (optional): the result once more, in `copy_dtype`; widths that the rows-in-registers kernel takes only.
extern "C" int tnx_norm_add(const float* y, const float* weight, const float* bias, float eps, int center,
                            const float* residual, float mult, float* out, void* copy, int copy_dtype, int tokens,
                            int width, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0 && eps > 0.f, "norm_add: bad sizes tokens=%d width=%d", tokens, width);
  TNX_REQUIRE(y && residual && out && out != y, "norm_add: the result may not lie where the normed rows do");
  TNX_REQUIRE(!copy || rows_fit(width), "norm_add: no copy beside a row of %d", width);
  if (tokens == 0) return 0;
  if (rows_fit(width)) {
#define NA_LAUNCH(PER) \
  norm_add_rows_kernel<PER><<<tokens, 256, 0, stream>>>(y, weight, bias, eps, center, residual, mult, out, copy, copy_dtype, width)
    ROWS_DISPATCH(width, NA_LAUNCH)
#undef NA_LAUNCH
  } else {
    norm_add_kernel<<<tokens, 256, 0, stream>>>(y, weight, bias, eps, center, residual, mult, out, width);
  }
  TNX_CHECK_LAUNCH("norm_add");
  return 0;
}

// See `join_norm_conv_kernel`. `h_keep` `[tokens, width]` floats is needed unless every run is one token
// (`single_runs`); widths that `tnx_rows_fit` takes only.
extern "C" int tnx_rows_fit(int width) { return rows_fit(width) ? 1 : 0; }

extern "C" int tnx_join_norm_conv(const float* x, const float* y, const float* post_w, const float* post_b,
                                  int post_center, float mult, float* x_out, const float* pre_w, const float* pre_b,
                                  int pre_center, float eps, const float* conv_w, float* state, long long slot_stride,
                                  int taps, const int* positions, const int* token_request, const int* run_start,
                                  const int* slots, void* out, int out_dtype, float* h_keep, int single_runs, int tokens,
                                  int width, int runs, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && rows_fit(width) && taps >= 1 && runs >= 0 && eps > 0.f, "join_norm_conv: bad sizes");
  TNX_REQUIRE(taps == 1 || state, "join_norm_conv: %d taps need the requests' state", taps);
  TNX_REQUIRE(taps == 1 || single_runs || h_keep, "join_norm_conv: nowhere to leave the inputs that the state takes");
  TNX_REQUIRE(!y || (x_out && x_out != x), "join_norm_conv: the joined stream needs a place of its own");
  if (tokens == 0) return 0;
#define JN_ARGS                                                                                                       \
  x, y, post_w, post_b, post_center, mult, x_out, pre_w, pre_b, pre_center, eps, conv_w, taps > 1 ? state : nullptr,  \
      (size_t)slot_stride, taps, positions, token_request, run_start, slots, out, out_dtype, h_keep, single_runs, width
#define JN_LAUNCH(PER)                                                                       \
  switch (taps) {                                                                            \
    case 2: join_norm_conv_kernel<PER, 2><<<tokens, 256, 0, stream>>>(JN_ARGS); break;       \
    case 3: join_norm_conv_kernel<PER, 3><<<tokens, 256, 0, stream>>>(JN_ARGS); break;       \
    case 4: join_norm_conv_kernel<PER, 4><<<tokens, 256, 0, stream>>>(JN_ARGS); break;       \
    default: join_norm_conv_kernel<PER, 0><<<tokens, 256, 0, stream>>>(JN_ARGS); break;      \
  }
  ROWS_DISPATCH(width, JN_LAUNCH)
#undef JN_LAUNCH
#undef JN_ARGS
  TNX_CHECK_LAUNCH("join_norm_conv");
  if (taps > 1 && !single_runs) {
    conv_state_kernel<<<dim3((width + 255) / 256, runs), 256, 0, stream>>>(h_keep, state, (size_t)slot_stride, taps,
                                                                          positions, run_start, slots, width);
    TNX_CHECK_LAUNCH("conv_state");
  }
  return 0;
}

// ------------------------------------------------------------------------------------------------ input convolution

// out[t, d] = h[t, d] + sum_j w[j, d] * h[t - taps + 1 + j, d] over the tokens of t's own request (zeros before
// its start); the weights come tap by tap, `[taps, width]`, so that a tap's weights of neighbouring channels are
// neighbours. Inputs from before the step's run come from the request's state, `[taps, width]`: the input at
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
      acc += w[(size_t)j * width + d] * x;
    }
    store_any(out, out_dtype, (size_t)t * width + d, acc);
  }
}

// the same, four channels a thread (widths that are multiples of 4): 16-byte loads and stores
__global__ void __launch_bounds__(256)
input_conv4_kernel(const float* __restrict__ h, const float* __restrict__ w, const float* __restrict__ state,
                   size_t slot_stride, int taps, const int* __restrict__ positions,
                   const int* __restrict__ token_request, const int* __restrict__ run_start,
                   const int* __restrict__ slots, void* __restrict__ out, int out_dtype, int width) {
  const int t = blockIdx.x;
  const int r = token_request[t];
  const int i = t - run_start[r], p = positions[t];
  const int w4 = width >> 2;
  const float* mine = state ? state + (size_t)slots[r] * slot_stride : nullptr;
  for (int k = threadIdx.x; k < w4; k += 256) {
    rf4 acc = ((const rf4*)(h + (size_t)t * width))[k];
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      rf4 x;
      if (back <= i)
        x = ((const rf4*)(h + (size_t)(t - back) * width))[k];
      else if (back <= p && mine)
        x = ((const rf4*)(mine + (size_t)((p - back) % taps) * width))[k];
      else
        continue;
      acc = acc + ((const rf4*)(w + (size_t)j * width))[k] * x;
    }
    store_chunk(out, out_dtype, (size_t)t * w4 + k, acc);
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
  if (width % 4 == 0)
    input_conv4_kernel<<<tokens, 256, 0, stream>>>(h, w, taps > 1 ? state : nullptr, (size_t)slot_stride, taps, positions,
                                                   token_request, run_start, slots, out, out_dtype, width);
  else
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
  if (rows_fit(width)) {
#define PN_LAUNCH(PER) poly_norm_rows_kernel<PER><<<tokens, 256, 0, stream>>>(z, coeffs, eps, out, out_dtype, width)
    ROWS_DISPATCH(width, PN_LAUNCH)
#undef PN_LAUNCH
  } else
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
