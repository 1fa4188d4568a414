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

// The recurrence is taken apart. Its gates and its normalizer need nothing of S: one block a (request, head) walks
// the run's tokens (`memory_gates_kernel`), leaves every token's two factors exp(f + m - m'), exp(i - m') and the
// reciprocal of the denominator max(|nrm' . q|, exp(-m')) + 1e-6 in memory, and carries nrm and m on. The blocks
// that hold S (`memory_cell_kernel`, 64 columns each) then have nothing but multiply-adds between one token and
// the next, and no two blocks share state that either writes.
//
// Both take a run a chunk of tokens at a time through LDS. A token's queries, keys and values lie far from the
// next token's (a row of all heads' projections apart), so what counts is how many loads are under way: every
// thread loads 16 bytes at a time into registers, the next chunk's while this chunk is worked on, and the
// registers go to LDS afterwards. ALIGNED: rows and heads begin at multiples of 16 bytes; otherwise the same with
// loads of one element.

template <bool ALIGNED>
__device__ __forceinline__ f32x4 load4(const float* p, int valid) {      // the first `valid` of four elements, zeros behind
  f32x4 r = {0.f, 0.f, 0.f, 0.f};
  if (valid <= 0) return r;
  if (ALIGNED) return *(const f32x4*)p;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (e < valid) r[e] = p[e];
  return r;
}

// grid: requests * heads blocks of four waves. All threads load; the first wave walks the chain, a row of the
// normalizer a lane (and up to four). LDS: [CHG][np + 1] queries (scaled) and keys, 8 numbers a token.
constexpr int CHG = 32;      // the most tokens a chunk; `chg` of them where LDS holds no more
template <bool ALIGNED>
__global__ void __launch_bounds__(256) memory_gates_kernel(CellArgs a, float* __restrict__ keeps, float* __restrict__ takes,
                                                           float* __restrict__ belows, int np, int chg) {
  extern __shared__ float lds[];
  const int r = blockIdx.x / a.heads, head = blockIdx.x - r * a.heads;
  const int lane = threadIdx.x;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
  if (count <= 0) return;
  const int ldq = np + 1;                           // a token's row in LDS: one more, so that tokens lie in different banks
  float* qs = lds;                                  // [CHG][ldq]
  float* ks = qs + chg * ldq;                       // [CHG][ldq]
  float* gis = ks + chg * ldq;                      // [CHG] log of the input gate
  float* gfs = gis + chg;                           // [CHG] log of the forget gate
  float* ms = gfs + chg;                            // [CHG + 1] the running maximum
  float* kp = ms + chg + 1;                         // [CHG] exp(f + m - m')
  float* tk = kp + chg;                             // [CHG] exp(i - m')
  float* fl = tk + chg;                             // [CHG] exp(-m')
  const int from = (have - 1) & 1, to = (have + count - 1) & 1;
  const size_t head_at = (size_t)slot * 2 * a.heads + head;
  float nrm[4] = {0.f, 0.f, 0.f, 0.f}, m = 0.f;     // lane l of the first wave holds rows l, l + 64, l + 128, l + 192
  if (lane < 64) {
    const float* np_ = a.normalizer + (head_at + (size_t)from * a.heads) * a.n;
#pragma unroll
    for (int j = 0; j < 4; ++j) nrm[j] = (have > 0 && lane + 64 * j < a.n) ? np_[lane + 64 * j] : 0.f;
    if (have > 0) m = a.peak[head_at + (size_t)from * a.heads];
  }
  const int fours = np >> 2;                        // 16-byte pieces of a token's queries: up to 64
  f32x4 rq[8], rk[8];                               // CHG * fours / 256 <= 8 pieces a thread
  float ri = 0.f, rf = 0.f;
  auto fetch = [&](int t0) {
    const int len = min(chg, count - t0);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int f = lane + 256 * u, t = f / fours, d = 4 * (f - t * fours);
      const bool in = f < chg * fours && t < len;
      const float* row = a.proj + (size_t)(start + t0 + (in ? t : 0)) * a.ld + head * a.n + d;
      rq[u] = load4<ALIGNED>(row, in ? a.n - d : 0);
      rk[u] = load4<ALIGNED>(row + hn, in ? a.n - d : 0);
    }
    if (lane < len) {
      const float* row = a.proj + (size_t)(start + t0 + lane) * a.ld + 2 * hn + 2 * hv;
      ri = row[head];
      rf = row[a.heads + head];
    }
  };
  auto stash = [&](int t0) {
    const int len = min(chg, count - t0);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int f = lane + 256 * u, t = f / fours, d = 4 * (f - t * fours);
      if (f < chg * fours) {
#pragma unroll
        for (int e = 0; e < 4; ++e) qs[t * ldq + d + e] = rq[u][e] * a.q_scale, ks[t * ldq + d + e] = rk[u][e];
      }
    }
    if (lane < len) {
      gis[lane] = a.cap * tanhf(ri / a.cap);
      gfs[lane] = log_sigmoid(a.cap * tanhf(rf / a.cap));
    }
  };
  fetch(0);
  stash(0);
  __syncthreads();
  for (int t0 = 0; t0 < count; t0 += chg) {
    const int len = min(chg, count - t0);
    const bool more = t0 + chg < count;
    if (more) fetch(t0 + chg);                      // under way while this chunk is worked on
    if (lane == 0) {
      ms[0] = m;                                    // ms[t + 1]: the maximum after token t
      for (int t = 0; t < len; ++t) ms[t + 1] = m = fmaxf(gfs[t] + m, gis[t]);
    }
    __syncthreads();
    if (lane < len) {
      const size_t at = (size_t)(start + t0 + lane) * a.heads + head;
      keeps[at] = kp[lane] = expf(gfs[lane] + ms[lane] - ms[lane + 1]);
      takes[at] = tk[lane] = expf(gis[lane] - ms[lane + 1]);
      fl[lane] = expf(-ms[lane + 1]);
    }
    __syncthreads();
    // the normalizer's chain, a row a lane: its products with the queries take the queries' places, and the
    // tokens' sums over the rows are then made side by side, a token a lane
    if (lane < 64) {
#pragma unroll 4
      for (int t = 0; t < len; ++t) {
        const float keep = kp[t], take = tk[t];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = lane + 64 * j;
          if (d < np) {
            nrm[j] = keep * nrm[j] + take * ks[t * ldq + d];
            qs[t * ldq + d] *= nrm[j];
          }
        }
      }
    }
    __syncthreads();
    if (lane < len) {
      float dot = 0.f;
      for (int d = 0; d < np; ++d) dot += qs[lane * ldq + d];
      belows[(size_t)(start + t0 + lane) * a.heads + head] = 1.f / (fmaxf(fabsf(dot), fl[lane]) + 1e-6f);
    }
    __syncthreads();
    if (more) {
      stash(t0 + chg);
      __syncthreads();
    }
  }
  if (lane < 64) {
    float* np_ = a.normalizer + (head_at + (size_t)to * a.heads) * a.n;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (lane + 64 * j < a.n) np_[lane + 64 * j] = nrm[j];
  }
  if (lane == 0) a.peak[head_at + (size_t)to * a.heads] = m;
}

// grid: requests * heads * column blocks; a block is four waves and 64 columns of S: wave w holds the columns
// 64 b + 16 w + (lane & 15), and of these the rows NR (lane >> 4) + j, j < NR: a lane's share of a column is a
// quarter of its rows, and the four quarters meet through the wave's row exchanges (`rows_sum`).
template <int NR, bool ALIGNED>
__global__ void __launch_bounds__(256) memory_cell_kernel(CellArgs a, const float* __restrict__ keeps,
                                                          const float* __restrict__ takes,
                                                          const float* __restrict__ belows, int column_blocks) {
  constexpr int CH = NR == 64 ? 16 : 32;                  // tokens a chunk
  constexpr int np = 4 * NR;                              // a token's queries (and keys) in LDS, zeros behind n
  constexpr int QN = CH * NR / 256;                       // 16-byte pieces of queries (and keys) a thread and chunk
  constexpr int VN = CH * 16 / 256;                       // and of values
  __shared__ __attribute__((aligned(16))) float qs[CH * np];      // queries, scaled
  __shared__ __attribute__((aligned(16))) float ks[CH * np];      // keys times exp(i - m')
  __shared__ __attribute__((aligned(16))) float vs[CH * 64];
  __shared__ float kp[CH], bl[CH];                        // exp(f + m - m'), one over the denominators
  const int cb = blockIdx.x % column_blocks, rh = blockIdx.x / column_blocks;
  const int r = rh / a.heads, head = rh - r * a.heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int quarter = lane >> 4;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
  if (count <= 0) return;
  const int col = 64 * cb + 16 * wave + (lane & 15);
  const bool col_ok = col < a.v;
  float S[NR];
  const int from = (have - 1) & 1, to = (have + count - 1) & 1;
  const size_t head_at = (size_t)slot * 2 * a.heads + head;        // + place * heads
  {
    const float* Sp = a.memory + (head_at + (size_t)from * a.heads) * a.n * a.v;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int d = quarter * NR + j;
      S[j] = (have > 0 && d < a.n && col_ok) ? Sp[(size_t)d * a.v + col] : 0.f;
    }
  }
  f32x4 rq[QN], rk[QN], rv[VN];
  float rt[QN], rkeep = 0.f, rbl = 0.f;
  auto fetch = [&](int t0) {
    const int len = min(CH, count - t0);
#pragma unroll
    for (int u = 0; u < QN; ++u) {
      const int f = threadIdx.x + 256 * u, t = f / NR, d = 4 * (f - t * NR);
      const bool in = t < len;
      const float* row = a.proj + (size_t)(start + t0 + (in ? t : 0)) * a.ld + head * a.n + d;
      rq[u] = load4<ALIGNED>(row, in ? a.n - d : 0);
      rk[u] = load4<ALIGNED>(row + hn, in ? a.n - d : 0);
      rt[u] = in ? takes[(size_t)(start + t0 + t) * a.heads + head] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < VN; ++u) {
      const int f = threadIdx.x + 256 * u, t = f >> 4, c = 64 * cb + 4 * (f & 15);
      const bool in = t < len;
      rv[u] = load4<ALIGNED>(a.proj + (size_t)(start + t0 + (in ? t : 0)) * a.ld + 2 * hn + head * a.v + c, in ? a.v - c : 0);
    }
    if (threadIdx.x < len) {
      rkeep = keeps[(size_t)(start + t0 + threadIdx.x) * a.heads + head];
      rbl = belows[(size_t)(start + t0 + threadIdx.x) * a.heads + head];
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int u = 0; u < QN; ++u) {
      const int f = threadIdx.x + 256 * u;
      *(f32x4*)(qs + 4 * f) = rq[u] * a.q_scale;          // piece f of the chunk: token f / NR, elements 4 (f % NR) on
      *(f32x4*)(ks + 4 * f) = rk[u] * rt[u];
    }
#pragma unroll
    for (int u = 0; u < VN; ++u) *(f32x4*)(vs + 4 * (threadIdx.x + 256 * u)) = rv[u];
    if (threadIdx.x < CH) kp[threadIdx.x] = rkeep, bl[threadIdx.x] = rbl;
  };
  fetch(0);
  stash();
  __syncthreads();
  for (int t0 = 0; t0 < count; t0 += CH) {
    const int len = min(CH, count - t0);
    const bool more = t0 + CH < count;
    if (more) fetch(t0 + CH);                             // under way while this chunk is worked on
#pragma unroll 4
    for (int t = 0; t < len; ++t) {
      const float keep = kp[t];
      const float* q = qs + t * np + quarter * NR;
      const float* k = ks + t * np + quarter * NR;
      const float val = vs[t * 64 + 16 * wave + (lane & 15)];
      float top = 0.f, top2 = 0.f;
#pragma unroll
      for (int j = 0; j < NR; j += 2) {
        S[j] = keep * S[j] + k[j] * val;
        S[j + 1] = keep * S[j + 1] + k[j + 1] * val;
        top += S[j] * q[j];
        top2 += S[j + 1] * q[j + 1];
      }
      const float o = rows_sum(top + top2) * bl[t];
      if (quarter == 0 && col_ok) a.out[(size_t)(start + t0 + t) * hv + head * a.v + col] = o;
    }
    __syncthreads();        // before the next chunk takes the place of what this one read
    if (more) {
      stash();
      __syncthreads();
    }
  }
  float* Sp = a.memory + (head_at + (size_t)to * a.heads) * a.n * a.v;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int d = quarter * NR + j;
    if (d < a.n && col_ok) Sp[(size_t)d * a.v + col] = S[j];
  }
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
void launch_cell(const CellArgs& a, const float* keeps, const float* takes, const float* belows, int requests, bool aligned,
                 hipStream_t stream) {
  const int column_blocks = (a.v + 63) / 64;
  const dim3 grid(requests * a.heads * column_blocks);
  if (aligned)
    memory_cell_kernel<NR, true><<<grid, 256, 0, stream>>>(a, keeps, takes, belows, column_blocks);
  else
    memory_cell_kernel<NR, false><<<grid, 256, 0, stream>>>(a, keeps, takes, belows, column_blocks);
}

}  // namespace

extern "C" int tnx_matrix_memory(const float* proj, int ld, const int* run_start, const int* cached, const int* slots,
                                 float* memory, float* normalizer, float* peak, int num_slots, float* raw, float* gates,
                                 const float* weight, float eps, void* out, int dtype, int tokens, int requests, int heads,
                                 int n, int v, float cap, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && n > 0 && v > 0, "matrix_memory: bad sizes");
  TNX_REQUIRE(n <= 256, "matrix_memory: query/key heads of up to 256 elements, got %d", n);
  TNX_REQUIRE(ld >= 2 * heads * n + 2 * heads * v + 2 * heads, "matrix_memory: rows of %d elements, %d needed", ld,
              2 * heads * n + 2 * heads * v + 2 * heads);
  TNX_REQUIRE(cap > 0.f, "matrix_memory: the gates' cap must be positive");
  TNX_REQUIRE(dtype == TNX_F32 || dtype == TNX_BF16, "matrix_memory: dtype %d", dtype);
  if (tokens == 0 || requests == 0) return 0;
  CellArgs a{proj, ld, run_start, cached, slots, memory, normalizer, peak, raw, heads, n, v, cap, 1.f / sqrtf((float)n)};
  float* keeps = gates;                             // [T, H] each
  float* takes = gates + (size_t)tokens * heads;
  float* belows = gates + 2 * (size_t)tokens * heads;
  // rows and heads that begin at multiples of 16 bytes are loaded 16 bytes at a time
  const bool aligned = n % 4 == 0 && v % 4 == 0 && ld % 4 == 0 && (uintptr_t)proj % 16 == 0;
  {
    const int np = (n + 3) / 4 * 4;
    const int chg = np > 240 ? CHG / 2 : CHG;          // 64 KB of LDS hold 32 tokens of up to 240 elements
    const size_t lds = ((size_t)chg * (2 * (np + 1) + 6) + 1) * sizeof(float);
    if (aligned)
      memory_gates_kernel<true><<<requests * heads, 256, lds, stream>>>(a, keeps, takes, belows, np, chg);
    else
      memory_gates_kernel<false><<<requests * heads, 256, lds, stream>>>(a, keeps, takes, belows, np, chg);
    TNX_CHECK_LAUNCH("matrix_memory gates");
  }
  const int quarter_rows = (n + 3) / 4;
  if (quarter_rows <= 8)
    launch_cell<8>(a, keeps, takes, belows, requests, aligned, stream);
  else if (quarter_rows <= 16)
    launch_cell<16>(a, keeps, takes, belows, requests, aligned, stream);
  else if (quarter_rows <= 32)
    launch_cell<32>(a, keeps, takes, belows, requests, aligned, stream);
  else
    launch_cell<64>(a, keeps, takes, belows, requests, aligned, stream);
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
