// The matrix memory (mLSTM cell): a state S [n, v] a head that is carried from token to token,
//     m' = max(f + m, i),  S' = exp(f + m - m') S + exp(i - m') k val^T,  nrm' likewise with k alone,
//     o = S'^T q / (max(|nrm' . q|, exp(-m')) + 1e-6),
// with i = cap tanh(x_i / cap) and f = logsigmoid(cap tanh(x_f / cap)) from a head's two pre-activations.
// Everything is float32. The state lies in two places by the parity of the position: the token at position p
// reads place (p - 1) & 1 (nothing at p = 0) and writes place p & 1, so a step of single tokens that is run
// twice reads the same both times.
#include "common.h"

TNX_DEFINE_ERROR_API

namespace {

struct CellArgs {
  const float* proj;      // [T, ld]: q [H n] | k [H n] | val [H v] | gate [H v] | x_i [H] | x_f [H]
  int ld;
  const int* run_start;   // [R + 1]
  const int* cached;      // [R]
  const int* slots;       // [R]
  float* memory;          // [slots, 2, H, n, v]
  float* normalizer;      // [slots, 2, H, n]
  float* peak;            // [slots, 2, H]
  float* out;             // [T, H v], before the norm
  int heads, n, v;
  float cap, q_scale;
};

__device__ __forceinline__ float log_sigmoid(float z) {
  // min(z, 0) - log(1 + exp(-|z|)): neither side overflows
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

// One block a (request, head): wave w holds the columns 16 (w C + c) + (lane & 15), c < C, of S, and of these the
// rows NR (lane >> 4) + j, j < NR: a lane's share of a column is a quarter of its rows, and the four quarters meet
// through the wave's row exchanges (`rows_sum`). A run is taken `chunk` tokens at a time: the block brings their
// queries (scaled), keys and values into LDS with loads that lie side by side, one thread walks the chunk's gates
// (the running maximum and the two factors of every token, a chain of its own that needs nothing of S), and then
// every wave runs the chunk's tokens from LDS with nothing but multiply-adds between one token and the next.
template <int NR, int C>
__global__ void __launch_bounds__(512) memory_cell_kernel(CellArgs a, int chunk) {
  extern __shared__ float lds[];
  const int r = blockIdx.x / a.heads, head = blockIdx.x - r * a.heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int quarter = lane >> 4;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
  const int np = 4 * NR;                                  // a token's queries (and keys) in LDS, zeros behind n
  const int vp = 16 * C * (blockDim.x >> 6);              // and its values, zeros behind v
  float* qs = lds;                                        // [chunk][np]
  float* ks = qs + (size_t)chunk * np;                    // [chunk][np]
  float* vs = ks + (size_t)chunk * np;                    // [chunk][vp]
  float* keeps = vs + (size_t)chunk * vp;                 // [chunk] exp(f + m - m')
  float* takes = keeps + chunk;                           // [chunk] exp(i - m')
  float* floors = takes + chunk;                          // [chunk] exp(-m')
  float* gis = floors + chunk;                            // [chunk] log of the input gate
  float* gfs = gis + chunk;                               // [chunk] log of the forget gate
  float* ms = gfs + chunk;                                // [chunk + 1] the running maximum
  int col[C];
  bool col_ok[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    col[c] = 16 * (wave * C + c) + (lane & 15);
    col_ok[c] = col[c] < a.v;
  }
  float S[C][NR], nrm[NR], m = 0.f;
  const int from = (have - 1) & 1, to = (have + count - 1) & 1;
  const size_t head_at = (size_t)slot * 2 * a.heads + head;        // + place * heads
  {
    const float* Sp = a.memory + (head_at + (size_t)from * a.heads) * a.n * a.v;
    const float* np_ = a.normalizer + (head_at + (size_t)from * a.heads) * a.n;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int d = quarter * NR + j;
      const bool ok = have > 0 && d < a.n;
      nrm[j] = ok ? np_[d] : 0.f;
#pragma unroll
      for (int c = 0; c < C; ++c) S[c][j] = (ok && col_ok[c]) ? Sp[(size_t)d * a.v + col[c]] : 0.f;
    }
    if (have > 0) m = a.peak[head_at + (size_t)from * a.heads];       // thread 0 alone carries it on
  }
  // every wave has read the state before any wave writes it: the two places coincide for runs of even length
  __syncthreads();
  for (int t0 = 0; t0 < count; t0 += chunk) {
    const int len = min(chunk, count - t0);
    for (int i = threadIdx.x; i < len * np; i += blockDim.x) {
      const int t = i / np, d = i - t * np;
      const float* row = a.proj + (size_t)(start + t0 + t) * a.ld;
      qs[i] = d < a.n ? row[head * a.n + d] * a.q_scale : 0.f;
      ks[i] = d < a.n ? row[hn + head * a.n + d] : 0.f;
    }
    for (int i = threadIdx.x; i < len * vp; i += blockDim.x) {
      const int t = i / vp, c = i - t * vp;
      vs[i] = c < a.v ? a.proj[(size_t)(start + t0 + t) * a.ld + 2 * hn + head * a.v + c] : 0.f;
    }
    // the gates: each token's two logarithms side by side, the running maximum as a chain of one thread (an add
    // and a maximum a token), and each token's factors side by side again
    if (threadIdx.x < len) {
      const float* row = a.proj + (size_t)(start + t0 + threadIdx.x) * a.ld + 2 * hn + 2 * hv;
      gis[threadIdx.x] = a.cap * tanhf(row[head] / a.cap);
      gfs[threadIdx.x] = log_sigmoid(a.cap * tanhf(row[a.heads + head] / a.cap));
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      ms[0] = m;                                   // ms[t + 1]: the maximum after token t
      for (int t = 0; t < len; ++t) ms[t + 1] = m = fmaxf(gfs[t] + m, gis[t]);
    }
    __syncthreads();
    if (threadIdx.x < len) {
      const int t = threadIdx.x;
      keeps[t] = expf(gfs[t] + ms[t] - ms[t + 1]);
      takes[t] = expf(gis[t] - ms[t + 1]);
      floors[t] = expf(-ms[t + 1]);
    }
    __syncthreads();
    for (int t = 0; t < len; ++t) {
      const float keep = keeps[t], take = takes[t];
      const float* q = qs + (size_t)t * np + quarter * NR;
      const float* k = ks + (size_t)t * np + quarter * NR;
      float val[C], top[C], nq = 0.f;
#pragma unroll
      for (int c = 0; c < C; ++c) val[c] = vs[(size_t)t * vp + 16 * (wave * C + c) + (lane & 15)], top[c] = 0.f;
#pragma unroll
      for (int j = 0; j < NR; ++j) {
        const float tk = take * k[j], qj = q[j];
        nrm[j] = keep * nrm[j] + tk;
        nq += nrm[j] * qj;
#pragma unroll
        for (int c = 0; c < C; ++c) {
          S[c][j] = keep * S[c][j] + tk * val[c];
          top[c] += S[c][j] * qj;
        }
      }
      nq = rows_sum(nq);
      const float below = fmaxf(fabsf(nq), floors[t]) + 1e-6f;
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const float o = rows_sum(top[c]) / below;
        if (quarter == 0 && col_ok[c]) a.out[(size_t)(start + t0 + t) * hv + head * a.v + col[c]] = o;
      }
    }
    __syncthreads();        // before the next chunk overwrites what this one read
  }
  if (count <= 0) return;
  float* Sp = a.memory + (head_at + (size_t)to * a.heads) * a.n * a.v;
  float* np_ = a.normalizer + (head_at + (size_t)to * a.heads) * a.n;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int d = quarter * NR + j;
    if (d >= a.n) continue;
#pragma unroll
    for (int c = 0; c < C; ++c)
      if (col_ok[c]) Sp[(size_t)d * a.v + col[c]] = S[c][j];
    if (wave == 0 && (lane & 15) == 0) np_[d] = nrm[j];
  }
  if (threadIdx.x == 0) a.peak[head_at + (size_t)to * a.heads] = m;
}

// What follows the cell up to the output projection: each head's o at unit root mean square, weighted, times
// sigmoid(gate); a wave a (token, head).
template <typename T>
__global__ void __launch_bounds__(256) memory_output_kernel(const float* __restrict__ o, const float* __restrict__ proj,
                                                            int ld, int gate_at, const float* __restrict__ weight,
                                                            float eps, T* __restrict__ out, int pairs, int heads, int v) {
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (pair >= pairs) return;
  const int t = pair / heads, head = pair - t * heads;
  const float* mine = o + (size_t)t * heads * v + head * v;
  float s = 0.f;
  for (int i = lane; i < v; i += 64) s += mine[i] * mine[i];
  s = wave_sum(s);
  const float r = 1.f / sqrtf(s / (float)v + eps);
  const float* gate = proj + (size_t)t * ld + gate_at + head * v;
  for (int i = lane; i < v; i += 64) {
    const float g = 1.f / (1.f + expf(-gate[i]));
    out[(size_t)t * heads * v + head * v + i] = from_f32<T>(mine[i] * r * weight[head * v + i] * g);
  }
}

template <int NR>
int launch_cell(const CellArgs& a, int requests, int columns16, int longest, hipStream_t stream) {
  // waves of a block: one for every 16 columns up to 8 waves; beyond that a wave takes 2, 4 or 8 groups of 16
  const int per = columns16 <= 8 ? 1 : (columns16 <= 16 ? 2 : (columns16 <= 32 ? 4 : 8));
  const int waves = (columns16 + per - 1) / per;
  const dim3 grid(requests * a.heads), block(64 * waves);
  // tokens a chunk: up to 32, as many as 60 KB of LDS hold (a token's queries, keys, values and three numbers)
  const int token_floats = 2 * 4 * NR + 16 * per * waves + 6;
  int chunk = (60 << 10) / (4 * token_floats);
  chunk = chunk > 32 ? 32 : (chunk < 1 ? 1 : chunk);
  if (chunk > longest) chunk = longest < 1 ? 1 : longest;
  const size_t lds = ((size_t)chunk * token_floats + 1) * sizeof(float);
  if (per == 1)
    memory_cell_kernel<NR, 1><<<grid, block, lds, stream>>>(a, chunk);
  else if (per == 2)
    memory_cell_kernel<NR, 2><<<grid, block, lds, stream>>>(a, chunk);
  else if (per == 4)
    memory_cell_kernel<NR, 4><<<grid, block, lds, stream>>>(a, chunk);
  else
    memory_cell_kernel<NR, 8><<<grid, block, lds, stream>>>(a, chunk);
  return 0;
}

}  // namespace

extern "C" int tnx_matrix_memory(const float* proj, int ld, const int* run_start, const int* cached, const int* slots,
                                 float* memory, float* normalizer, float* peak, int num_slots, float* raw,
                                 const float* weight, float eps, void* out, int dtype, int tokens, int requests, int heads,
                                 int n, int v, float cap, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && n > 0 && v > 0, "matrix_memory: bad sizes");
  TNX_REQUIRE(n <= 256, "matrix_memory: query/key heads of up to 256 elements, got %d", n);
  TNX_REQUIRE(v <= 1024, "matrix_memory: value heads of up to 1024 elements, got %d", v);
  TNX_REQUIRE(ld >= 2 * heads * n + 2 * heads * v + 2 * heads, "matrix_memory: rows of %d elements, %d needed", ld,
              2 * heads * n + 2 * heads * v + 2 * heads);
  TNX_REQUIRE(cap > 0.f, "matrix_memory: the gates' cap must be positive");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "matrix_memory: dtype %d", dtype);
  if (tokens == 0 || requests == 0) return 0;
  CellArgs a{proj, ld, run_start, cached, slots, memory, normalizer, peak, raw, heads, n, v, cap, 1.f / sqrtf((float)n)};
  const int quarter_rows = (n + 3) / 4, columns16 = (v + 15) / 16;
  if (quarter_rows <= 8)
    launch_cell<8>(a, requests, columns16, tokens, stream);
  else if (quarter_rows <= 16)
    launch_cell<16>(a, requests, columns16, tokens, stream);
  else if (quarter_rows <= 32)
    launch_cell<32>(a, requests, columns16, tokens, stream);
  else
    launch_cell<64>(a, requests, columns16, tokens, stream);
  TNX_CHECK_LAUNCH("matrix_memory");
  const int pairs = tokens * heads;
  const int gate_at = 2 * heads * n + heads * v;
  if (dtype == TNX_F32)
    memory_output_kernel<float><<<(pairs + 3) / 4, 256, 0, stream>>>(raw, proj, ld, gate_at, weight, eps, (float*)out,
                                                                      pairs, heads, v);
  else
    memory_output_kernel<bf16_t><<<(pairs + 3) / 4, 256, 0, stream>>>(raw, proj, ld, gate_at, weight, eps, (bf16_t*)out,
                                                                       pairs, heads, v);
  TNX_CHECK_LAUNCH("matrix_memory output");
  return 0;
}
