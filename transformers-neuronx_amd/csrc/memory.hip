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
  float* memory;          // [slots, 2, H, v, n]
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

// The recurrence is taken apart. The gates need nothing of S: one wave a (request, head) walks the run's tokens
// (`memory_gates_kernel`), leaves every token's two factors exp(f + m - m'), exp(i - m') and the floor exp(-m') of
// its denominator in memory, carries m on, and sets the normalizer the run begins with aside. The blocks that hold
// S (`memory_cell_kernel`, 16 columns each) each carry the normalizer along as one more column, so that between
// one token and the next there is nothing but multiply-adds and sums within 16 lanes, and no block reads state
// that another writes: they read the normalizer from where the first kernel set it aside, and the block of a
// head's first columns alone writes it back.
//
// The state lies with a column's rows side by side (`memory` [slots, 2, H, v, n]): a lane's rows of a column are
// neighbours in memory.
//
// A run goes a chunk of tokens at a time through LDS. A token's queries, keys and values lie far from the next
// token's (a row of all heads' projections apart), so what counts is how many loads are under way: every thread
// loads 16 bytes at a time into registers, the next chunk's while this chunk is worked on, and the registers go to
// LDS afterwards. ALIGNED: rows and heads begin at multiples of 16 bytes; otherwise the same with loads of one
// element.

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

// grid: requests * heads blocks of one wave; 64 tokens a round, a token a lane, the running maximum a chain of
// lane 0 between two rounds of side-by-side work.
__global__ void __launch_bounds__(64) memory_gates_kernel(CellArgs a, float* __restrict__ keeps, float* __restrict__ takes,
                                                          float* __restrict__ floors, float* __restrict__ aside) {
  __shared__ float gis[64], gfs[64], ms[65];
  const int r = blockIdx.x / a.heads, head = blockIdx.x - r * a.heads;
  const int lane = threadIdx.x;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
  if (count <= 0) return;
  const int from = (have - 1) & 1, to = (have + count - 1) & 1;
  const size_t head_at = (size_t)slot * 2 * a.heads + head;
  {
    const float* np_ = a.normalizer + (head_at + (size_t)from * a.heads) * a.n;
    float* out = aside + (size_t)blockIdx.x * a.n;
    for (int d = lane; d < a.n; d += 64) out[d] = have > 0 ? np_[d] : 0.f;
  }
  float m = have > 0 ? a.peak[head_at + (size_t)from * a.heads] : 0.f;
  for (int t0 = 0; t0 < count; t0 += 64) {
    const int len = min(64, count - t0);
    if (lane < len) {
      const float* row = a.proj + (size_t)(start + t0 + lane) * a.ld + 2 * hn + 2 * hv;
      gis[lane] = a.cap * tanhf(row[head] / a.cap);
      gfs[lane] = log_sigmoid(a.cap * tanhf(row[a.heads + head] / a.cap));
    }
    __syncthreads();
    if (lane == 0) {
      // (what the chain reads from LDS is read before it begins: a store into LDS between two loads would keep the
      // second load from being under way with the first)
      float gi_r[64], gf_r[64], after[64], peak = m;
#pragma unroll
      for (int t = 0; t < 64; ++t) gi_r[t] = t < len ? gis[t] : 0.f, gf_r[t] = t < len ? gfs[t] : 0.f;
#pragma unroll
      for (int t = 0; t < 64; ++t) after[t] = peak = t < len ? fmaxf(gf_r[t] + peak, gi_r[t]) : peak;
      ms[0] = m;                                    // ms[t + 1]: the maximum after token t
#pragma unroll
      for (int t = 0; t < 64; ++t)
        if (t < len) ms[t + 1] = after[t];
    }
    __syncthreads();
    if (lane < len) {
      const size_t at = (size_t)(start + t0 + lane) * a.heads + head;
      keeps[at] = expf(gfs[lane] + ms[lane] - ms[lane + 1]);
      takes[at] = expf(gis[lane] - ms[lane + 1]);
      floors[at] = expf(-ms[lane + 1]);
    }
    m = ms[len];
    __syncthreads();
  }
  if (lane == 0) a.peak[head_at + (size_t)to * a.heads] = m;
}

// grid: requests * heads * column blocks; a block is four waves and 16 columns of S. In a wave the 16 lanes of a
// row of lanes share a column (column 16 b + 4 w + lane / 16): lane % 16 holds its rows NR (lane % 16) + j, j < NR,
// and the same rows of the normalizer; a column's sum over the rows is a sum over the 16 lanes of a row of lanes.
template <int NR, bool ALIGNED>
__global__ void __launch_bounds__(256) memory_cell_kernel(CellArgs a, const float* __restrict__ keeps,
                                                          const float* __restrict__ takes,
                                                          const float* __restrict__ floors,
                                                          const float* __restrict__ aside, int column_blocks) {
  constexpr int CH = NR == 16 ? 16 : 32;                  // tokens a chunk
  constexpr int np = 16 * NR;                             // a token's queries (and keys) in LDS, zeros behind n
  constexpr int PT = np / 4;                              // 16-byte pieces of a token's queries
  constexpr int QN = (CH * PT + 255) / 256;               // pieces of queries (and keys) a thread and chunk
  __shared__ __attribute__((aligned(16))) float qs[CH * np];      // queries, scaled
  __shared__ __attribute__((aligned(16))) float ks[CH * np];      // keys times exp(i - m')
  __shared__ __attribute__((aligned(16))) float vs[CH * 16];
  __shared__ float kp[CH], fl[CH];                        // exp(f + m - m'), exp(-m')
  const int cb = blockIdx.x % column_blocks, rh = blockIdx.x / column_blocks;
  const int r = rh / a.heads, head = rh - r * a.heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane & 15;
  const int start = a.run_start[r], count = a.run_start[r + 1] - start;
  const int have = a.cached[r], slot = a.slots[r];
  const int hn = a.heads * a.n, hv = a.heads * a.v;
  if (count <= 0) return;
  const int col = 16 * cb + 4 * wave + (lane >> 4);
  const bool col_ok = col < a.v;
  float S[NR], nrm[NR];
  const int from = (have - 1) & 1, to = (have + count - 1) & 1;
  const size_t head_at = (size_t)slot * 2 * a.heads + head;        // + place * heads
  {
    const float* Sp = a.memory + ((head_at + (size_t)from * a.heads) * a.v + (col_ok ? col : 0)) * a.n;
    const float* np_ = aside + (size_t)rh * a.n;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int d = grp * NR + j;
      S[j] = (have > 0 && d < a.n && col_ok) ? Sp[d] : 0.f;
      nrm[j] = d < a.n ? np_[d] : 0.f;
    }
  }
  f32x4 rq[QN], rk[QN], rv = {0.f, 0.f, 0.f, 0.f};
  float rt[QN], rkeep = 1.f, rfl = 0.f;
  auto fetch = [&](int t0) {
    const int len = min(CH, count - t0);
#pragma unroll
    for (int u = 0; u < QN; ++u) {
      const int f = threadIdx.x + 256 * u, t = f / PT, d = 4 * (f - t * PT);
      const bool in = f < CH * PT && t < len;
      const float* row = a.proj + (size_t)(start + t0 + (in ? t : 0)) * a.ld + head * a.n + d;
      rq[u] = load4<ALIGNED>(row, in ? a.n - d : 0);
      rk[u] = load4<ALIGNED>(row + hn, in ? a.n - d : 0);
      rt[u] = in ? takes[(size_t)(start + t0 + t) * a.heads + head] : 0.f;
    }
    if (threadIdx.x < CH * 4) {                            // a token's 16 values: four pieces
      const int t = threadIdx.x >> 2, c = 16 * cb + 4 * (threadIdx.x & 3);
      const bool in = t < len;
      rv = load4<ALIGNED>(a.proj + (size_t)(start + t0 + (in ? t : 0)) * a.ld + 2 * hn + head * a.v + c, in ? a.v - c : 0);
    }
    if (threadIdx.x < CH) {
      const bool in = threadIdx.x < len;
      rkeep = in ? keeps[(size_t)(start + t0 + threadIdx.x) * a.heads + head] : 1.f;
      rfl = in ? floors[(size_t)(start + t0 + threadIdx.x) * a.heads + head] : 1.f;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int u = 0; u < QN; ++u) {
      const int f = threadIdx.x + 256 * u;                // piece f of the chunk: token f / PT, elements 4 (f % PT) on
      if (f < CH * PT) {
        *(f32x4*)(qs + 4 * f) = rq[u] * a.q_scale;
        *(f32x4*)(ks + 4 * f) = rk[u] * rt[u];
      }
    }
    if (threadIdx.x < CH * 4) *(f32x4*)(vs + 4 * threadIdx.x) = rv;
    if (threadIdx.x < CH) kp[threadIdx.x] = rkeep, fl[threadIdx.x] = rfl;
  };
  fetch(0);
  stash();
  __syncthreads();
  for (int t0 = 0; t0 < count; t0 += CH) {
    const int len = min(CH, count - t0);
    const bool more = t0 + CH < count;
    if (more) fetch(t0 + CH);                             // under way while this chunk is worked on
    // a token's operands are read from LDS while the token before it is worked on
    float q_n[NR], k_n[NR], val_n, keep_n, fl_n;
    auto read = [&](int t) {
      const float* q = qs + t * np + grp * NR;
      const float* k = ks + t * np + grp * NR;
#pragma unroll
      for (int j = 0; j < NR; ++j) q_n[j] = q[j], k_n[j] = k[j];
      val_n = vs[t * 16 + 4 * wave + (lane >> 4)];
      keep_n = kp[t];
      fl_n = fl[t];
    };
    auto token = [&](int t, bool last) {
      float q[NR], k[NR];
#pragma unroll
      for (int j = 0; j < NR; ++j) q[j] = q_n[j], k[j] = k_n[j];
      const float val = val_n, keep = keep_n, floor_ = fl_n;
      if (!last) read(t + 1);
      float top = 0.f, dot = 0.f;
#pragma unroll
      for (int j = 0; j < NR; ++j) {
        S[j] = keep * S[j] + k[j] * val;
        nrm[j] = keep * nrm[j] + k[j];
        top += S[j] * q[j];
        dot += nrm[j] * q[j];
      }
      // sums over the 16 lanes of a row of lanes
      top += lane_dpp<TNX_DPP_XOR1>(top), dot += lane_dpp<TNX_DPP_XOR1>(dot);
      top += lane_dpp<TNX_DPP_XOR2>(top), dot += lane_dpp<TNX_DPP_XOR2>(dot);
      top += lane_dpp<TNX_DPP_HALF_MIRROR>(top), dot += lane_dpp<TNX_DPP_HALF_MIRROR>(dot);
      top += lane_dpp<TNX_DPP_MIRROR>(top), dot += lane_dpp<TNX_DPP_MIRROR>(dot);
      // (the denominator is 1e-6 at least: its reciprocal, right to a unit in the last place, is no subnormal)
      const float o = top * __builtin_amdgcn_rcpf(fmaxf(fabsf(dot), floor_) + 1e-6f);
      if (grp == 0 && col_ok) a.out[(size_t)(start + t0 + t) * hv + head * a.v + col] = o;
    };
    read(0);
    if (len == CH) {        // a whole chunk: a count the compiler knows
#pragma unroll 4
      for (int t = 0; t < CH; ++t) token(t, t == CH - 1);
    } else {
      for (int t = 0; t < len; ++t) token(t, t == len - 1);
    }
    __syncthreads();        // before the next chunk takes the place of what this one read
    if (more) {
      stash();
      __syncthreads();
    }
  }
  if (col_ok) {
    float* Sp = a.memory + ((head_at + (size_t)to * a.heads) * a.v + col) * a.n;
#pragma unroll
    for (int j = 0; j < NR; ++j)
      if (grp * NR + j < a.n) Sp[grp * NR + j] = S[j];
  }
  if (cb == 0 && wave == 0 && lane < 16) {                 // the normalizer, once a head
    float* np_ = a.normalizer + (head_at + (size_t)to * a.heads) * a.n;
#pragma unroll
    for (int j = 0; j < NR; ++j)
      if (grp * NR + j < a.n) np_[grp * NR + j] = nrm[j];
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
void launch_cell(const CellArgs& a, const float* keeps, const float* takes, const float* floors, const float* aside,
                 int requests, bool aligned, hipStream_t stream) {
  const int column_blocks = (a.v + 15) / 16;
  const dim3 grid(requests * a.heads * column_blocks);
  if (aligned)
    memory_cell_kernel<NR, true><<<grid, 256, 0, stream>>>(a, keeps, takes, floors, aside, column_blocks);
  else
    memory_cell_kernel<NR, false><<<grid, 256, 0, stream>>>(a, keeps, takes, floors, aside, column_blocks);
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
  float* floors = gates + 2 * (size_t)tokens * heads;
  float* aside = gates + 3 * (size_t)tokens * heads;      // [R, H, n]: the normalizers the runs begin with
  // rows and heads that begin at multiples of 16 bytes are loaded 16 bytes at a time
  const bool aligned = n % 4 == 0 && v % 4 == 0 && ld % 4 == 0 && (uintptr_t)proj % 16 == 0;
  memory_gates_kernel<<<requests * heads, 64, 0, stream>>>(a, keeps, takes, floors, aside);
  TNX_CHECK_LAUNCH("matrix_memory gates");
  const int rows16 = (n + 15) / 16;
  if (rows16 <= 2)
    launch_cell<2>(a, keeps, takes, floors, aside, requests, aligned, stream);
  else if (rows16 <= 4)
    launch_cell<4>(a, keeps, takes, floors, aside, requests, aligned, stream);
  else if (rows16 <= 8)
    launch_cell<8>(a, keeps, takes, floors, aside, requests, aligned, stream);
  else
    launch_cell<16>(a, keeps, takes, floors, aside, requests, aligned, stream);
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
