// Gated linear attention: per head a float32 matrix state S [dk, dv] that every token decays
// row by row and adds an outer product to, read by the token's query:
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,      o_t = qscale * S_t^T q_t,      a_t = exp(ld_t), ld_t <= 0
//
// gla_prepare  finishes the input product of a step (partial sums) into float32 rows
//              [q | k | ld | v | g] and makes the logarithm of the decay from a low-rank product:
//              z = A2 (A1 h) + b,  ld = log(sigmoid(z)) / tau  (so that a = sigmoid(z)^(1/tau)).
// gla_scan     walks the tokens of every request of the step in their order from the state that
//              earlier steps left in the request's slot, and leaves the new state there.
// gla_chunks   the same for requests that bring many tokens, sixteen tokens at a time on the matrix cores.
// gla_finish   divides every head's output by its root mean square, times a gain over dv that the
//              heads share, times silu(g) and a scale; writes the rows that the output product reads.
//
// Decays, their logarithms, the state and the unit norm are float32 whatever the model's type.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;
constexpr int kMaxRank = 512;

__global__ __launch_bounds__(kThreads) void gla_prepare_kernel(
    const void* __restrict__ proj, int proj_dt, int n_partials, size_t partial_stride, int ld, int col0,
    const void* __restrict__ a2, int a2_dt, const void* __restrict__ a2_bias, int bias_dt, float inv_tau,
    float* __restrict__ x, int heads, int dk, int dv, int rank) {
  __shared__ float a1s[kMaxRank];
  const int n = blockIdx.x, tid = threadIdx.x;
  const size_t in_row = static_cast<size_t>(n) * ld + col0;
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv;
  float* xr = x + static_cast<size_t>(n) * width;
  auto value = [&](int col) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_float(proj, proj_dt, p * partial_stride + in_row + col);
    return v;
  };
  // the product's columns: q, k (hk each), v, g (hv each), the low-rank input (rank)
  for (int r = tid; r < rank; r += kThreads) a1s[r] = value(2 * hk + 2 * hv + r);
  for (int i = tid; i < 2 * hk; i += kThreads) xr[i] = value(i);
  for (int i = tid; i < 2 * hv; i += kThreads) xr[3 * hk + i] = value(2 * hk + i);
  __syncthreads();
  for (int c = tid; c < hk; c += kThreads) {
    float z = 0.f;
    for (int r = 0; r < rank; ++r) z = fmaf(load_as_float(a2, a2_dt, static_cast<size_t>(c) * rank + r), a1s[r], z);
    if (a2_bias) z += load_as_float(a2_bias, bias_dt, c);
    // log(sigmoid(z)) without overflow on either side
    const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
    xr[2 * hk + c] = ls * inv_tau;
  }
}

// The same with four columns to a load and an element's partial sums asked for together (all widths,
// the first column and the partial sums' stride are multiples of four).
template <typename TP, typename TA>
__global__ __launch_bounds__(kThreads) void gla_prepare_vec_kernel(
    const TP* __restrict__ proj, int n_partials, size_t partial_stride, int ld, int col0, const TA* __restrict__ a2,
    const void* __restrict__ a2_bias, int bias_dt, float inv_tau, float* __restrict__ x, int heads, int dk,
    int dv, int rank) {
  __shared__ float a1s[kMaxRank];
  const int n = blockIdx.x, tid = threadIdx.x;
  const TP* in = proj + static_cast<size_t>(n) * ld + col0;
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv;
  float* xr = x + static_cast<size_t>(n) * width;
  for (int r = tid; r < rank; r += kThreads) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += to_float(in[p * partial_stride + 2 * hk + 2 * hv + r]);
    a1s[r] = v;
  }
  for (int i = 4 * tid; i < 2 * hk; i += 4 * kThreads) Vec4<float>::store(xr + i, sum_partials4(in + i, partial_stride, n_partials));
  for (int i = 4 * tid; i < 2 * hv; i += 4 * kThreads)
    Vec4<float>::store(xr + 3 * hk + i, sum_partials4(in + 2 * hk + i, partial_stride, n_partials));
  __syncthreads();
  for (int c = tid; c < hk; c += kThreads) {
    float z = 0.f;
    const TA* row = a2 + static_cast<size_t>(c) * rank;
#pragma unroll 8
    for (int r = 0; r < rank; ++r) z = fmaf(to_float(row[r]), a1s[r], z);  // typed loads: eight of them on their way together
    if (a2_bias) z += load_as_float(a2_bias, bias_dt, c);
    const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
    xr[2 * hk + c] = ls * inv_tau;
  }
}

// A block: one request, one head, 64 columns of the state (a lane a column); wave w keeps the rows
// w, w + 4, ... in registers, DR of them. A token's four partial outputs are joined through LDS.
template <int DR>
__global__ __launch_bounds__(kThreads) void gla_scan_kernel(
    const float* __restrict__ x, float* __restrict__ state, float* __restrict__ o, const int* __restrict__ q_start,
    const int* __restrict__ state_slots, int heads, int dk, int dv, float qscale, const float* __restrict__ decay) {
  __shared__ float red[2][4][kWave];
  const int s = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  const int col = blockIdx.z * kWave + lane;
  const bool has_col = col < dv;
  const int t_begin = q_start[s], t_end = q_start[s + 1];
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv;
  float* st = state + (static_cast<size_t>(state_slots[s]) * heads + hd) * dk * dv;
  float S[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = w + 4 * r;
    S[r] = has_col && row < dk ? st[static_cast<size_t>(row) * dv + col] : 0.f;
  }
  const float fixed = decay ? decay[hd] : 0.f;  // one decay for the whole head, given as it is: no exponential
  for (int t = t_begin; t < t_end; ++t) {
    const float* xr = x + static_cast<size_t>(t) * width;
    const float* qr = xr + hd * dk;
    const float* kr = qr + hk;
    const float* lr = kr + hk;
    const float v = has_col ? xr[3 * hk + hd * dv + col] : 0.f;
    float part = 0.f;
#pragma unroll
    for (int r = 0; r < DR; ++r) {
      const int row = w + 4 * r;
      if (row < dk) {
        S[r] = (decay ? fixed : expf(lr[row])) * S[r] + kr[row] * v;
        part = fmaf(S[r], qr[row], part);
      }
    }
    const int buf = (t - t_begin) & 1;
    red[buf][w][lane] = part;
    __syncthreads();
    if (w == 0 && has_col)
      o[static_cast<size_t>(t) * hv + hd * dv + col] =
          (((red[buf][0][lane] + red[buf][1][lane]) + red[buf][2][lane]) + red[buf][3][lane]) * qscale;
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = w + 4 * r;
    if (has_col && row < dk) st[static_cast<size_t>(row) * dv + col] = S[r];
  }
}

// The same recurrence for requests that bring many tokens: chunks of 16 tokens on the matrix cores'
// float32 instruction, so that the chain of dependent steps is a sixteenth as long. With b_t the sum
// of the chunk's log decays up to and including token t (per key channel) and B = b of its last token:
//
//   o_t = qscale * ( (q_t * exp(b_t))^T S_prev + sum_{s <= t} A[t][s] v_s ),   A[t][s] = sum_d q_td k_sd exp(b_td - b_sd)
//   S   = diag(exp(B)) S_prev + sum_s (k_s * exp(B - b_s)) v_s^T
//
// Every exponent is <= 0 (a decay never grows), whatever the decays are: the pair (t, s) gets its own
// exponentials instead of a product of two factors that could overflow. Nothing but S_prev depends on
// the chunks before, so one kernel prepares all chunks of the step at once (gla_chunk_prep: a block per
// chunk and head makes A, q * exp(b), k * exp(B - b), exp(B) and v in the layouts of the matrix
// instruction's operands) and the kernel that walks the chunks (gla_chunk_walk: a wave per request,
// head and 16 columns of the state, nothing shared between waves) is left with three small matrix
// products per chunk, whose operands it asks for one chunk ahead.
// Chunks are counted from the first token that the request brings in this step. A chunk's operands
// lie at "slots": token t of request s of the step has slot t + 16 s, so that the 16 slots of a
// request's last, shorter chunk do not reach into the next request's.
constexpr int kChunk = 16;
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct ChunkScratch {
  float* qd;     // [slot][head][dkp]:                 q * exp(b)
  float* kdt;    // per chunk [head][dkp][16 tokens]:  k * exp(B - b)
  float* vt;     // per chunk [head][dvp][16 tokens]:  v
  float* pairs;  // [slot][head][16]:                  row of A
  float* eb;     // per chunk [head][256]:             exp(B)
};
__host__ __device__ inline size_t chunk_scratch_floats(size_t slots, int heads, int dkp, int dvp) {
  return slots * heads * (2 * static_cast<size_t>(dkp) + dvp + 2 * kChunk);
}
__host__ __device__ inline ChunkScratch carve(float* base, size_t slots, int heads, int dkp, int dvp) {
  ChunkScratch c;
  c.qd = base;
  c.kdt = c.qd + slots * heads * dkp;
  c.vt = c.kdt + slots * heads * dkp;
  c.pairs = c.vt + slots * heads * dvp;
  c.eb = c.pairs + slots * heads * kChunk;
  return c;
}

__global__ __launch_bounds__(kThreads) void gla_chunk_prep_kernel(
    const float* __restrict__ x, ChunkScratch sc, const int* __restrict__ q_start, int heads, int dk, int dv, int dkp,
    int dvp) {
  extern __shared__ float prep_lds[];
  float* qs = prep_lds;
  float* ks = qs + kChunk * dk;
  float* bs = ks + kChunk * dk;
  const int s = blockIdx.z, hd = blockIdx.y, tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  const int t0 = q_start[s] + blockIdx.x * kChunk, t_end = q_start[s + 1];
  if (t0 >= t_end) return;
  const int nc = min(kChunk, t_end - t0);
  const size_t slot0 = static_cast<size_t>(t0) + kChunk * s;
  const size_t region = slot0 * heads + static_cast<size_t>(hd) * kChunk;  // of this chunk and head, in slots
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv;
  for (int i = tid; i < nc * dk; i += kThreads) {
    const int t = i / dk, d = i % dk;
    const float* xr = x + static_cast<size_t>(t0 + t) * width + hd * dk + d;
    qs[i] = xr[0];
    ks[i] = xr[hk];
    bs[i] = xr[2 * hk];
  }
  for (int i = tid; i < dvp * kChunk; i += kThreads) {
    const int cc = i / kChunk, t = i % kChunk;
    sc.vt[region * dvp + i] = t < nc && cc < dv ? x[static_cast<size_t>(t0 + t) * width + 3 * hk + hd * dv + cc] : 0.f;
  }
  __syncthreads();
  for (int d = tid; d < dk; d += kThreads)
    for (int t = 1; t < nc; ++t) bs[t * dk + d] += bs[(t - 1) * dk + d];
  __syncthreads();
  for (int p = w; p < kChunk * kChunk; p += 4) {  // a wave a pair, its lanes over the key channels
    const int t = p / kChunk, sidx = p % kChunk;
    float a = 0.f;
    if (sidx <= t && t < nc) {
      for (int d = lane; d < dk; d += kWave)
        a = fmaf(qs[t * dk + d] * ks[sidx * dk + d], expf(bs[t * dk + d] - bs[sidx * dk + d]), a);
      a = wave_sum(a);
    }
    if (lane == 0) sc.pairs[((slot0 + t) * heads + hd) * kChunk + sidx] = a;
  }
  for (int i = tid; i < kChunk * dkp; i += kThreads) {
    const int t = i / dkp, d = i % dkp;
    const bool there = t < nc && d < dk;
    sc.qd[((slot0 + t) * heads + hd) * dkp + d] = there ? qs[t * dk + d] * expf(bs[t * dk + d]) : 0.f;
  }
  for (int i = tid; i < kChunk * dkp; i += kThreads) {
    const int d = i / kChunk, t = i % kChunk;
    const bool there = t < nc && d < dk;
    sc.kdt[region * dkp + i] = there ? ks[t * dk + d] * expf(bs[(nc - 1) * dk + d] - bs[t * dk + d]) : 0.f;
  }
  for (int d = tid; d < dkp; d += kThreads) sc.eb[region * kChunk + d] = d < dk ? expf(bs[(nc - 1) * dk + d]) : 0.f;
}

// DT: tiles of 16 rows of the state (dk <= 16 DT; the rows beyond dk are zeros and stay so). The wave
// keeps its 16 columns' rows in the layout of the instruction's result: lane (g = lane / 16,
// c = lane % 16) holds rows 16 j + 4 g + i (i < 4) of column c in S[j][i]. The sums over the rows take
// them in the order i, then g, so that a lane's own S[j][i] is the operand it has to supply; the sums
// over the chunk's tokens take token 4 g + i in step i.
template <int DT>
struct ChunkOperands {
  f32x4 q[DT], k[DT], e[DT], v, a;
};

template <int DT>
__global__ __launch_bounds__(kWave) void gla_chunk_walk_kernel(
    ChunkScratch sc, float* __restrict__ state, float* __restrict__ o, const int* __restrict__ q_start,
    const int* __restrict__ state_slots, int heads, int dk, int dv, int dvp, float qscale) {
  constexpr int dkp = 16 * DT;
  const int s = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x, g = lane >> 4, c = lane & 15;
  const int col = blockIdx.z * 16 + c;
  const bool has_col = col < dv;
  const int t_begin = q_start[s], t_end = q_start[s + 1], hv = heads * dv;
  float* st = state + (static_cast<size_t>(state_slots[s]) * heads + hd) * dk * dv;
  f32x4 S[DT];
#pragma unroll
  for (int j = 0; j < DT; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * j + 4 * g + i;
      S[j][i] = has_col && row < dk ? st[static_cast<size_t>(row) * dv + col] : 0.f;
    }
  auto fetch = [&](int t0, ChunkOperands<DT>& r) {
    const size_t slot0 = static_cast<size_t>(t0) + kChunk * s;
    const size_t region = slot0 * heads + static_cast<size_t>(hd) * kChunk;
    const float* qp = sc.qd + ((slot0 + c) * heads + hd) * dkp + 4 * g;
    const float* kp = sc.kdt + region * dkp + c * kChunk + 4 * g;
    const float* ep = sc.eb + region * kChunk + 4 * g;
#pragma unroll
    for (int j = 0; j < DT; ++j) {
      r.q[j] = *reinterpret_cast<const f32x4*>(qp + 16 * j);
      r.k[j] = *reinterpret_cast<const f32x4*>(kp + 16 * j * kChunk);
      r.e[j] = *reinterpret_cast<const f32x4*>(ep + 16 * j);
    }
    r.v = *reinterpret_cast<const f32x4*>(sc.vt + region * dvp + static_cast<size_t>(min(col, dvp - 1)) * kChunk + 4 * g);
    if (!has_col) r.v = f32x4{0.f, 0.f, 0.f, 0.f};
    r.a = *reinterpret_cast<const f32x4*>(sc.pairs + ((slot0 + c) * heads + hd) * kChunk + 4 * g);
  };
  ChunkOperands<DT> now, next;
  if (t_begin < t_end) fetch(t_begin, now);
  for (int t0 = t_begin; t0 < t_end; t0 += kChunk) {
    const int nc = min(kChunk, t_end - t0);
    const bool more = t0 + kChunk < t_end;
    if (more) fetch(t0 + kChunk, next);
    f32x4 out = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < DT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) out = __builtin_amdgcn_mfma_f32_16x16x4f32(now.q[j][i], S[j][i], out, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) out = __builtin_amdgcn_mfma_f32_16x16x4f32(now.a[i], now.v[i], out, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 4 * g + i;
      if (t < nc && has_col) o[static_cast<size_t>(t0 + t) * hv + hd * dv + col] = out[i] * qscale;
    }
#pragma unroll
    for (int j = 0; j < DT; ++j) {
#pragma unroll
      for (int i = 0; i < 4; ++i) S[j][i] *= now.e[j][i];
#pragma unroll
      for (int i = 0; i < 4; ++i) S[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(now.k[j][i], now.v[i], S[j], 0, 0, 0);
    }
    if (more) now = next;
  }
#pragma unroll
  for (int j = 0; j < DT; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * j + 4 * g + i;
      if (has_col && row < dk) st[static_cast<size_t>(row) * dv + col] = S[j][i];
    }
}

__global__ __launch_bounds__(kThreads) void gla_finish_kernel(
    const float* __restrict__ o, const float* __restrict__ x, const void* __restrict__ gain, int gain_dt, float eps,
    float out_scale, void* __restrict__ out, int out_dt, int out_ld, int heads, int dk, int dv) {
  const int n = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv;
  const float* g = x + static_cast<size_t>(n) * width + 3 * hk + hv;
  for (int hd = wave; hd < heads; hd += kThreads / kWave) {
    float v[4], ss = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = lane + 64 * u;
      v[u] = e < dv ? o[static_cast<size_t>(n) * hv + hd * dv + e] : 0.f;
      ss += v[u] * v[u];
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dv) + eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = lane + 64 * u;
      if (e >= dv) continue;
      const float gg = g[hd * dv + e];
      const float y = v[u] * inv * (gain ? load_as_float(gain, gain_dt, e) : 1.f) * (gg / (1.f + expf(-gg))) * out_scale;
      store_from_float(out, out_dt, static_cast<size_t>(n) * out_ld + hd * dv + e, y);
    }
  }
}

// The rows [q | k | ld | v | g] for a recurrence whose decay is one fixed number per head: the first `rot` elements of
// every query and key head are turned by position (pairs (e, e + rot / 2), or neighbours (2e, 2e + 1)), the keys then
// scaled; ld of every key channel of head h is log_decay[h]. One block a token, a thread a pair (or an element).
__global__ __launch_bounds__(kThreads) void retention_prepare_kernel(
    const void* __restrict__ proj, int proj_dt, int n_partials, size_t partial_stride, int ld, int col0,
    const float* __restrict__ log_decay, const float* __restrict__ cos, const float* __restrict__ sin, int rot,
    int neighbours, const int* __restrict__ positions, float kscale, float* __restrict__ x, int heads, int dk, int dv) {
  const int n = blockIdx.x, tid = threadIdx.x;
  const size_t in_row = static_cast<size_t>(n) * ld + col0;
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv, half = rot / 2;
  float* xr = x + static_cast<size_t>(n) * width;
  auto value = [&](int col) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_float(proj, proj_dt, p * partial_stride + in_row + col);
    return v;
  };
  const size_t trig = static_cast<size_t>(positions[n]) * half;
  // queries (columns 0 .. hk) and keys (hk .. 2 hk): the turned pairs of every head, then the elements that pass
  for (int i = tid; i < 2 * heads * half; i += kThreads) {
    const int head = i / half, e = i % half;  // head counts query heads, then key heads
    const int e1 = neighbours ? 2 * e : e, e2 = neighbours ? 2 * e + 1 : e + half;
    const int base = head * dk;
    float a, b;
    rotate_pair(value(base + e1), value(base + e2), cos[trig + e], sin[trig + e], a, b);
    const float f = head >= heads ? kscale : 1.f;
    xr[base + e1] = a * f;
    xr[base + e2] = b * f;
  }
  const int rest = dk - rot;
  for (int i = tid; i < 2 * heads * rest; i += kThreads) {
    const int head = i / rest, col = head * dk + rot + i % rest;
    xr[col] = value(col) * (head >= heads ? kscale : 1.f);
  }
  for (int c = tid; c < hk; c += kThreads) xr[2 * hk + c] = log_decay[c / dk];
  for (int i = tid; i < 2 * hv; i += kThreads) xr[3 * hk + i] = value(2 * hk + i);
}

// The same with a wave per block and four columns a lane: blocks 0 .. 2 heads - 1 of a token take a query or key head
// each (the partners of a rotation exchanged through LDS), the blocks behind them 256 columns of [ld | v | g] each. The
// head sizes, the product's width, first column and stride are multiples of four.
template <typename TP>
__global__ __launch_bounds__(kWave) void retention_prepare_vec_kernel(
    const TP* __restrict__ proj, int n_partials, size_t partial_stride, int ld, int col0,
    const float* __restrict__ log_decay, const float* __restrict__ cos, const float* __restrict__ sin, int rot,
    int neighbours, const int* __restrict__ positions, float kscale, float* __restrict__ x, int heads, int dk, int dv) {
  __shared__ __attribute__((aligned(16))) float xs[256];
  const int n = blockIdx.x, lane = threadIdx.x;
  const TP* in = proj + static_cast<size_t>(n) * ld + col0;
  const int hk = heads * dk, hv = heads * dv, width = 3 * hk + 2 * hv, half = rot / 2;
  float* xr = x + static_cast<size_t>(n) * width;
  if (static_cast<int>(blockIdx.y) >= 2 * heads) {
    const int i = (static_cast<int>(blockIdx.y) - 2 * heads) * 4 * kWave + 4 * lane;  // a column of [ld | v | g]
    if (i < hk) {
      const float l = log_decay[i / dk];  // four neighbours share a head: dk is a multiple of four
      *reinterpret_cast<float4*>(xr + 2 * hk + i) = float4{l, l, l, l};
    } else if (i < hk + 2 * hv) {
      *reinterpret_cast<float4*>(xr + 2 * hk + i) = sum_partials4(in + 2 * hk + (i - hk), partial_stride, n_partials);
    }
    return;
  }
  const int head = blockIdx.y, e = 4 * lane;  // head counts query heads, then key heads
  const bool mine = e < dk;
  float4 v = {0.f, 0.f, 0.f, 0.f};
  if (mine) {
    v = sum_partials4(in + head * dk + e, partial_stride, n_partials);
    *reinterpret_cast<float4*>(xs + e) = v;
  }
  __syncthreads();
  if (!mine) return;
  float y[4] = {v.x, v.y, v.z, v.w};
  const size_t trig = static_cast<size_t>(positions[n]) * half;
  const float f = head >= heads ? kscale : 1.f;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int el = e + u;
    if (el < rot) {
      const int pair = neighbours ? el >> 1 : (el < half ? el : el - half);
      const bool first = neighbours ? !(el & 1) : el < half;
      const int partner = neighbours ? el ^ 1 : (first ? el + half : el - half);
      float a, b;
      if (first) rotate_pair(y[u], xs[partner], cos[trig + pair], sin[trig + pair], a, b);
      else rotate_pair(xs[partner], y[u], cos[trig + pair], sin[trig + pair], a, b);
      y[u] = first ? a : b;
    }
    y[u] *= f;
  }
  *reinterpret_cast<float4*>(xr + head * dk + e) = float4{y[0], y[1], y[2], y[3]};
}

}  // namespace

extern "C" int pyre_gla_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                const void* a2, int a2_dt, const void* a2_bias, int bias_dt, float tau, float* x,
                                int n, int heads, int dk, int dv, int rank, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(a2_dt) && (!a2_bias || known_dtype(bias_dt)) && n_partials >= 1,
               "gla_prepare: bad dtypes");
  PYRE_REQUIRE(heads > 0 && dk > 0 && dv > 0 && rank > 0 && rank <= kMaxRank, "gla_prepare: bad sizes (rank %d of at most %d)", rank, kMaxRank);
  PYRE_REQUIRE(tau > 0.f, "gla_prepare: tau must be positive");
  if (n <= 0) return 0;
  const int hk = heads * dk, hv = heads * dv;
  if (hk % 4 == 0 && hv % 4 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 &&
      reinterpret_cast<uintptr_t>(proj) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(a2_dt, TA,
        hipLaunchKernelGGL((gla_prepare_vec_kernel<TP, TA>), dim3(n), dim3(kThreads), 0, stream,
                           static_cast<const TP*>(proj), n_partials, static_cast<size_t>(partial_stride), ld, col0,
                           static_cast<const TA*>(a2), a2_bias, bias_dt, 1.f / tau, x, heads, dk, dv, rank)));
    return check_launch("gla_prepare");
  }
  hipLaunchKernelGGL(gla_prepare_kernel, dim3(n), dim3(kThreads), 0, stream, proj, proj_dt, n_partials,
                     static_cast<size_t>(partial_stride), ld, col0, a2, a2_dt, a2_bias, bias_dt, 1.f / tau, x, heads, dk,
                     dv, rank);
  return check_launch("gla_prepare");
}

extern "C" int pyre_gla_scan(const float* x, float* state, float* o, const int* q_start, const int* state_slots,
                             int n_seqs, int heads, int dk, int dv, float qscale, const float* decay, hipStream_t stream) {
  PYRE_REQUIRE(heads > 0 && heads <= 65535 && dk > 0 && dk <= 256 && dv > 0, "gla_scan: heads %d, sizes %d / %d are not taken", heads, dk, dv);
  if (n_seqs <= 0) return 0;
  const dim3 grid(n_seqs, heads, (dv + kWave - 1) / kWave);
#define PYRE_SCAN(DR)                                                                                            \
  hipLaunchKernelGGL(gla_scan_kernel<DR>, grid, dim3(kThreads), 0, stream, x, state, o, q_start, state_slots, heads, \
                     dk, dv, qscale, decay)
  if (dk <= 32) PYRE_SCAN(8);
  else if (dk <= 64) PYRE_SCAN(16);
  else if (dk <= 128) PYRE_SCAN(32);
  else PYRE_SCAN(64);
#undef PYRE_SCAN
  return check_launch("gla_scan");
}

static int chunk_tiles(int dk) { return dk <= 32 ? 2 : dk <= 64 ? 4 : dk <= 128 ? 8 : 16; }

// Floats of scratch that pyre_gla_chunks needs for a step of n_tokens tokens of n_seqs requests.
extern "C" long pyre_gla_chunks_scratch(int n_tokens, int n_seqs, int heads, int dk, int dv) {
  const size_t slots = static_cast<size_t>(n_tokens) + static_cast<size_t>(kChunk) * n_seqs;
  return static_cast<long>(chunk_scratch_floats(slots, heads, 16 * chunk_tiles(dk), (dv + 3) / 4 * 4));
}

extern "C" int pyre_gla_chunks(const float* x, float* scratch, float* state, float* o, const int* q_start,
                               const int* state_slots, int n_tokens, int n_seqs, int max_tokens, int heads, int dk, int dv,
                               float qscale, hipStream_t stream) {
  PYRE_REQUIRE(heads > 0 && heads <= 65535 && dk > 0 && dk <= 256 && dv > 0, "gla_chunks: heads %d, sizes %d / %d are not taken", heads, dk, dv);
  PYRE_REQUIRE(n_seqs <= 65535 && max_tokens >= 0 && n_tokens >= 0, "gla_chunks: %d requests are more than a launch takes", n_seqs);
  PYRE_REQUIRE(reinterpret_cast<uintptr_t>(scratch) % 16 == 0, "gla_chunks: the scratch memory must start on 16 bytes");
  if (n_seqs <= 0 || max_tokens == 0) return 0;
  const int DTs = chunk_tiles(dk), dkp = 16 * DTs, dvp = (dv + 3) / 4 * 4;
  const ChunkScratch sc = carve(scratch, static_cast<size_t>(n_tokens) + static_cast<size_t>(kChunk) * n_seqs, heads, dkp, dvp);
  hipLaunchKernelGGL(gla_chunk_prep_kernel, dim3((max_tokens + kChunk - 1) / kChunk, heads, n_seqs), dim3(kThreads),
                     sizeof(float) * 3 * kChunk * dk, stream, x, sc, q_start, heads, dk, dv, dkp, dvp);
  if (check_launch("gla_chunk_prep")) return 1;
  const dim3 grid(n_seqs, heads, (dv + 15) / 16);
#define PYRE_WALK(DT)                                                                                                  \
  hipLaunchKernelGGL(gla_chunk_walk_kernel<DT>, grid, dim3(kWave), 0, stream, sc, state, o, q_start, state_slots, heads, \
                     dk, dv, dvp, qscale)
  switch (DTs) {
    case 2: PYRE_WALK(2); break;
    case 4: PYRE_WALK(4); break;
    case 8: PYRE_WALK(8); break;
    default: PYRE_WALK(16); break;
  }
#undef PYRE_WALK
  return check_launch("gla_chunks");
}

extern "C" int pyre_gla_finish(const float* o, const float* x, const void* gain, int gain_dt, float eps, float out_scale,
                               void* out, int out_dt, int out_ld, int n, int heads, int dk, int dv, hipStream_t stream) {
  PYRE_REQUIRE((!gain || known_dtype(gain_dt)) && known_dtype(out_dt), "gla_finish: bad dtypes");
  PYRE_REQUIRE(heads > 0 && dk > 0 && dv > 0 && dv <= 256 && eps > 0.f, "gla_finish: sizes %d / %d are not taken", dk, dv);
  if (n <= 0) return 0;
  hipLaunchKernelGGL(gla_finish_kernel, dim3(n), dim3(kThreads), 0, stream, o, x, gain, gain_dt, eps, out_scale, out,
                     out_dt, out_ld, heads, dk, dv);
  return check_launch("gla_finish");
}

extern "C" int pyre_retention_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                      const float* log_decay, const float* cos, const float* sin, int rot, int neighbours,
                                      const int* positions, float kscale, float* x, int n, int heads, int dk, int dv,
                                      hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && n_partials >= 1, "retention_prepare: bad dtypes");
  PYRE_REQUIRE(heads > 0 && dk > 0 && dv > 0 && log_decay && positions, "retention_prepare: bad sizes");
  PYRE_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || (cos && sin)),
               "retention_prepare: %d turned elements of a head of %d need tables and an even number", rot, dk);
  if (n <= 0) return 0;
  const int tail_blocks = (heads * dk + 2 * heads * dv + 4 * kWave - 1) / (4 * kWave);
  if (dk % 4 == 0 && dv % 4 == 0 && dk <= 256 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 &&
      2 * heads + tail_blocks <= 65535 && reinterpret_cast<uintptr_t>(proj) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    PYRE_DISPATCH(proj_dt, TP,
        hipLaunchKernelGGL(retention_prepare_vec_kernel<TP>, dim3(n, 2 * heads + tail_blocks), dim3(kWave), 0, stream,
                           static_cast<const TP*>(proj), n_partials, static_cast<size_t>(partial_stride), ld, col0,
                           log_decay, cos, sin, rot, neighbours, positions, kscale, x, heads, dk, dv));
    return check_launch("retention_prepare");
  }
  hipLaunchKernelGGL(retention_prepare_kernel, dim3(n), dim3(kThreads), 0, stream, proj, proj_dt, n_partials,
                     static_cast<size_t>(partial_stride), ld, col0, log_decay, cos, sin, rot, neighbours, positions, kscale,
                     x, heads, dk, dv);
  return check_launch("retention_prepare");
}
