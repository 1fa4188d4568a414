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
// rows (lane >> 4) + 4 j, j < NR: a lane's share of a column is a quarter of its rows, and the four quarters meet
// through the wave's row exchanges (`rows_sum`). The waves of a block do not wait for one another inside the
// loop over the run's tokens. The next token's inputs are loaded while this token's are worked on.
template <int NR, int C>
__global__ void __launch_bounds__(512) memory_cell_kernel(CellArgs a) {
  const int r = blockIdx.x / a.heads, head = blockIdx.x - r * a.heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int quarter = lane >> 4;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
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
    const float* np = a.normalizer + (head_at + (size_t)from * a.heads) * a.n;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int d = quarter + 4 * j;
      const bool ok = have > 0 && d < a.n;
      nrm[j] = ok ? np[d] : 0.f;
#pragma unroll
      for (int c = 0; c < C; ++c) S[c][j] = (ok && col_ok[c]) ? Sp[(size_t)d * a.v + col[c]] : 0.f;
    }
    if (have > 0) m = a.peak[head_at + (size_t)from * a.heads];
  }
  // every wave has read the state before any wave writes it: the two places coincide for runs of even length
  __syncthreads();
  if (count <= 0) return;

  float q[NR], k[NR], val[C], xi, xf;
  auto fetch = [&](int t) {
    const float* row = a.proj + (size_t)t * a.ld;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int d = quarter + 4 * j;
      const bool ok = d < a.n;
      q[j] = ok ? row[head * a.n + d] : 0.f;
      k[j] = ok ? row[hn + head * a.n + d] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < C; ++c) val[c] = col_ok[c] ? row[2 * hn + head * a.v + col[c]] : 0.f;
    xi = row[2 * hn + 2 * hv + head];
    xf = row[2 * hn + 2 * hv + a.heads + head];
  };
  fetch(start);
  for (int t = start; t < start + count; ++t) {
    float cq[NR], ck[NR], cval[C];
#pragma unroll
    for (int j = 0; j < NR; ++j) cq[j] = q[j] * a.q_scale, ck[j] = k[j];
#pragma unroll
    for (int c = 0; c < C; ++c) cval[c] = val[c];
    const float gi = a.cap * tanhf(xi / a.cap);
    const float gf = log_sigmoid(a.cap * tanhf(xf / a.cap));
    if (t + 1 < start + count) fetch(t + 1);
    const float m_new = fmaxf(gf + m, gi);
    const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
    m = m_new;
    float top[C], nq = 0.f;
#pragma unroll
    for (int c = 0; c < C; ++c) top[c] = 0.f;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const float tk = take * ck[j];
      nrm[j] = keep * nrm[j] + tk;
      nq += nrm[j] * cq[j];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        S[c][j] = keep * S[c][j] + tk * cval[c];
        top[c] += S[c][j] * cq[j];
      }
    }
    nq = rows_sum(nq);
    const float below = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const float o = rows_sum(top[c]) / below;
      if (quarter == 0 && col_ok[c]) a.out[(size_t)t * hv + head * a.v + col[c]] = o;
    }
  }
  float* Sp = a.memory + (head_at + (size_t)to * a.heads) * a.n * a.v;
  float* np = a.normalizer + (head_at + (size_t)to * a.heads) * a.n;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int d = quarter + 4 * j;
    if (d >= a.n) continue;
#pragma unroll
    for (int c = 0; c < C; ++c)
      if (col_ok[c]) Sp[(size_t)d * a.v + col[c]] = S[c][j];
    if (wave == 0 && (lane & 15) == 0) np[d] = nrm[j];
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
int launch_cell(const CellArgs& a, int requests, int columns16, hipStream_t stream) {
  // waves of a block: one for every 16 columns up to 8 waves; beyond that a wave takes 2, 4 or 8 groups of 16
  const int per = columns16 <= 8 ? 1 : (columns16 <= 16 ? 2 : (columns16 <= 32 ? 4 : 8));
  const int waves = (columns16 + per - 1) / per;
  const dim3 grid(requests * a.heads), block(64 * waves);
  if (per == 1)
    memory_cell_kernel<NR, 1><<<grid, block, 0, stream>>>(a);
  else if (per == 2)
    memory_cell_kernel<NR, 2><<<grid, block, 0, stream>>>(a);
  else if (per == 4)
    memory_cell_kernel<NR, 4><<<grid, block, 0, stream>>>(a);
  else
    memory_cell_kernel<NR, 8><<<grid, block, 0, stream>>>(a);
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
    launch_cell<8>(a, requests, columns16, stream);
  else if (quarter_rows <= 16)
    launch_cell<16>(a, requests, columns16, stream);
  else if (quarter_rows <= 32)
    launch_cell<32>(a, requests, columns16, stream);
  else
    launch_cell<64>(a, requests, columns16, stream);
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
