// The gated delta rule: per request and head a float32 state S [dk][dv] (kept column by column, [dv][dk], so that the
// rows of a column lie together) that every token first decays per key channel,
// then corrects towards its value along its key, then reads with its query:
//
//   S <- diag(a_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
//
// H value heads of dv; G query/key heads of dk, value head h reading query/key head h / (H / G).
//
// gdr_prepare   finishes a step's input product from col0 on, columns [q: G dk | k: G dk | v: H dv | beta: H |
//               low: rank_a | low': rank_g], into float32 rows x = [q | k | a: H dk | v | gate: H dv | beta: H]:
//               q, k, v go through a short causal convolution over the request's tokens (taps [T][channels], inputs before
//               the step's first token from the request's state, which is then brought up to date) and SiLU; q and k
//               are made unit vectors per head, x / sqrt(sum x^2 + unit_eps), q also times dk^-1/2;
//               beta = sigmoid(.); a = exp(rate_h softplus(A2 low + dt_bias)) per head and key channel, rate_h < 0;
//               gate = sigmoid(G2 low').
// gdr_scan      the recurrence over each request's tokens of the step, from and into the state. The columns of S never
//               meet, so a token costs two sums over the rows (S^T k, then S^T q). Key heads of a multiple of 16 elements up
//               to 128: a wave for one request, one head and 8 or 16 columns; eight or four neighbouring lanes share a
//               column, a part of its rows each in registers, and join their sums by exchanges among themselves; a second
//               wave of the block fetches the tokens' rows sixteen tokens ahead and hands them over through LDS, so that
//               the chain from token to token is arithmetic alone. Other sizes: a block of four waves for 64 columns (a
//               lane a column), wave w keeping the rows w, w + 4, .., the sums joined through LDS.
// gdr_finish    out = o / sqrt(mean(o^2 over dv) + eps) * gain * gate * out_scale, rounded to the output's type.
//
// All arithmetic float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_conv.h"

using namespace pyre;

namespace {

constexpr int kThreads = kConvThreads;
constexpr int kMaxHead = 256;
constexpr int kMaxTaps = 16;
constexpr int kMaxRank = 512;

struct Geometry {
  int H, G, dk, dv;
  __host__ __device__ int q0() const { return 0; }
  __host__ __device__ int k0() const { return G * dk; }
  __host__ __device__ int a0() const { return 2 * G * dk; }
  __host__ __device__ int v0() const { return 2 * G * dk + H * dk; }
  __host__ __device__ int g0() const { return v0() + H * dv; }
  __host__ __device__ int b0() const { return g0() + H * dv; }
  __host__ __device__ int width() const { return (b0() + H + 3) / 4 * 4; }  // rows start on 16 bytes
};

__device__ inline float sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float silu(float z) { return z / (1.f + expf(-z)); }
__device__ inline float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// Row `row` of w [rows][rank] against `low`: the sum in ascending order, the row's elements eight (bfloat16) or four
// (float32) to a load where the rank allows it.
__device__ inline float dot_row(const void* w, int dt, size_t row, int rank, const float* low) {
  float z = 0.f;
  if (dt == kBF16 && rank % 8 == 0) {
    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const bf16*>(w) + row * rank);
    for (int r = 0; r < rank / 8; ++r) {
      const uint4 u = p[r];
      const uint32_t words[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        z = fmaf(__uint_as_float(words[i] << 16), low[8 * r + 2 * i], z);
        z = fmaf(__uint_as_float(words[i] & 0xffff0000u), low[8 * r + 2 * i + 1], z);
      }
    }
    return z;
  }
  if (dt == kF32 && rank % 4 == 0) {
    const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(w) + row * rank);
    for (int r = 0; r < rank / 4; ++r) {
      const float4 u = p[r];
      z = fmaf(u.x, low[4 * r], z), z = fmaf(u.y, low[4 * r + 1], z), z = fmaf(u.z, low[4 * r + 2], z), z = fmaf(u.w, low[4 * r + 3], z);
    }
    return z;
  }
  for (int r = 0; r < rank; ++r) z = fmaf(load_as_float(w, dt, row * rank + r), low[r], z);
  return z;
}

__global__ __launch_bounds__(kThreads) void gdr_prepare_kernel(
    ConvIn in, const int* __restrict__ state_slots, const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
    const void* __restrict__ a2, int a2_dt, const float* __restrict__ dt_bias, const float* __restrict__ rate,
    const void* __restrict__ g2, int g2_dt, float unit_eps, float* __restrict__ x, Geometry s, int rank_a, int rank_g) {
  __shared__ float low[2 * kMaxRank];
  const int n = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int seq = seq_of_token[n], run = n - q_start[seq], st = state_slots[seq];
  float* xr = x + static_cast<size_t>(n) * s.width();
  const int vcol = 2 * s.G * s.dk, bcol = vcol + s.H * s.dv, lcol = bcol + s.H;  // columns of the product
  for (int i = tid; i < rank_a + rank_g; i += kThreads) low[i < rank_a ? i : kMaxRank + i - rank_a] = product_value(in, n, lcol + i);

  // queries and keys: a wave a head
  const float qscale = 1.f / sqrtf(static_cast<float>(s.dk));
  for (int head = wave; head < 2 * s.G; head += kThreads / kWave) {
    float y[kMaxHead / kWave], ss = 0.f;
#pragma unroll
    for (int u = 0; u < kMaxHead / kWave; ++u) {
      const int e = lane + kWave * u;
      y[u] = e < s.dk ? silu(conv_value(in, n, run, st, head * s.dk + e)) : 0.f;
      ss = fmaf(y[u], y[u], ss);
    }
    const float inv = (head < s.G ? qscale : 1.f) / sqrtf(wave_sum(ss) + unit_eps);
#pragma unroll
    for (int u = 0; u < kMaxHead / kWave; ++u) {
      const int e = lane + kWave * u;
      if (e < s.dk) xr[head * s.dk + e] = y[u] * inv;
    }
  }
  for (int i = tid; i < s.H * s.dv; i += kThreads) xr[s.v0() + i] = silu(conv_value(in, n, run, st, vcol + i));
  for (int i = tid; i < s.H; i += kThreads) xr[s.b0() + i] = sigmoid(product_value(in, n, bcol + i));
  __syncthreads();
  for (int i = tid; i < s.H * s.dk; i += kThreads) {
    const float z = dot_row(a2, a2_dt, i, rank_a, low);
    xr[s.a0() + i] = expf(rate[i / s.dk] * softplus(z + dt_bias[i]));
  }
  for (int i = tid; i < s.H * s.dv; i += kThreads) {
    xr[s.g0() + i] = sigmoid(dot_row(g2, g2_dt, i, rank_g, low + kMaxRank));
  }
}

// The same with four elements a lane and the work of a token dealt to the blocks y = 0 .. P - 1 of its row of the grid
// (steps of few tokens fill more of the chip that way): a wave takes a query or key head at a time, the threads four
// value channels each; every block loads the low-rank inputs. Head sizes, the product's width, first column and stride
// are multiples of four. The sums run in the order of the kernel above but for the heads' sums of squares (a lane's four
// neighbours here, elements 64 apart there): a difference of rounding, and which of the two runs depends on sizes alone.
template <typename TP>
__global__ __launch_bounds__(kThreads) void gdr_prepare_vec_kernel(
    ConvIn in, const int* __restrict__ state_slots, const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
    const void* __restrict__ a2, int a2_dt, const float* __restrict__ dt_bias, const float* __restrict__ rate,
    const void* __restrict__ g2, int g2_dt, float unit_eps, float* __restrict__ x, Geometry s, int rank_a, int rank_g) {
  __shared__ float low[2 * kMaxRank];
  const int n = blockIdx.x, y = blockIdx.y, P = gridDim.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int seq = seq_of_token[n], run = n - q_start[seq], st = state_slots[seq];
  float* xr = x + static_cast<size_t>(n) * s.width();
  const TP* proj = static_cast<const TP*>(in.proj);
  const int vcol = 2 * s.G * s.dk, bcol = vcol + s.H * s.dv, lcol = bcol + s.H;
  for (int i = tid; i < rank_a + rank_g; i += kThreads) low[i < rank_a ? i : kMaxRank + i - rank_a] = product_value(in, n, lcol + i);
  const float qscale = 1.f / sqrtf(static_cast<float>(s.dk));
  for (int head = y * (kThreads / kWave) + wave; head < 2 * s.G; head += P * (kThreads / kWave)) {
    const int e = 4 * lane;
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (e < s.dk) {
      v = conv_value4(in, proj, n, run, st, head * s.dk + e);
      v = float4{silu(v.x), silu(v.y), silu(v.z), silu(v.w)};
    }
    const float inv = (head < s.G ? qscale : 1.f) / sqrtf(wave_sum(fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, v.x * v.x)))) + unit_eps);
    if (e < s.dk) *reinterpret_cast<float4*>(xr + head * s.dk + e) = float4{v.x * inv, v.y * inv, v.z * inv, v.w * inv};
  }
  for (int i = 4 * (y * kThreads + tid); i < s.H * s.dv; i += 4 * kThreads * P) {
    const float4 v = conv_value4(in, proj, n, run, st, vcol + i);
    *reinterpret_cast<float4*>(xr + s.v0() + i) = float4{silu(v.x), silu(v.y), silu(v.z), silu(v.w)};
  }
  if (y == 0)
    for (int i = tid; i < s.H; i += kThreads) xr[s.b0() + i] = sigmoid(product_value(in, n, bcol + i));
  __syncthreads();
  for (int i = y * kThreads + tid; i < s.H * s.dk; i += kThreads * P) {
    const float z = dot_row(a2, a2_dt, i, rank_a, low);
    xr[s.a0() + i] = expf(rate[i / s.dk] * softplus(z + dt_bias[i]));
  }
  for (int i = y * kThreads + tid; i < s.H * s.dv; i += kThreads * P) {
    xr[s.g0() + i] = sigmoid(dot_row(g2, g2_dt, i, rank_g, low + kMaxRank));
  }
}

template <int DR>
__global__ __launch_bounds__(kThreads) void gdr_scan_kernel(const float* __restrict__ x, float* __restrict__ state,
                                                            float* __restrict__ o, const int* __restrict__ q_start,
                                                            const int* __restrict__ state_slots, Geometry s) {
  __shared__ float red[2][4][kWave];
  const int seq = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  const int col = blockIdx.z * kWave + lane, g = hd / (s.H / s.G);
  const bool has_col = col < s.dv;
  const int t_begin = q_start[seq], t_end = q_start[seq + 1], width = s.width();
  float* st = state + (static_cast<size_t>(state_slots[seq]) * s.H + hd) * s.dk * s.dv;
  float S[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = w + 4 * r;
    S[r] = has_col && row < s.dk ? st[static_cast<size_t>(col) * s.dk + row] : 0.f;
  }
  for (int t = t_begin; t < t_end; ++t) {
    const float* xr = x + static_cast<size_t>(t) * width;
    const float* qr = xr + s.q0() + g * s.dk;
    const float* kr = xr + s.k0() + g * s.dk;
    const float* ar = xr + s.a0() + hd * s.dk;
    const float v = has_col ? xr[s.v0() + hd * s.dv + col] : 0.f;
    const float beta = xr[s.b0() + hd];
    float part = 0.f;
#pragma unroll
    for (int r = 0; r < DR; ++r) {
      const int row = w + 4 * r;
      if (row < s.dk) {
        S[r] *= ar[row];
        part = fmaf(S[r], kr[row], part);
      }
    }
    red[0][w][lane] = part;
    __syncthreads();
    const float u = beta * (v - (((red[0][0][lane] + red[0][1][lane]) + red[0][2][lane]) + red[0][3][lane]));
    part = 0.f;
#pragma unroll
    for (int r = 0; r < DR; ++r) {
      const int row = w + 4 * r;
      if (row < s.dk) {
        S[r] = fmaf(kr[row], u, S[r]);
        part = fmaf(S[r], qr[row], part);
      }
    }
    red[1][w][lane] = part;
    __syncthreads();
    if (w == 0 && has_col)
      o[static_cast<size_t>(t) * s.H * s.dv + hd * s.dv + col] =
          ((red[1][0][lane] + red[1][1][lane]) + red[1][2][lane]) + red[1][3][lane];
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = w + 4 * r;
    if (has_col && row < s.dk) st[static_cast<size_t>(col) * s.dk + row] = S[r];
  }
}

// A block of two waves: one request, one head, 64 / LPC columns of the state. The first wave walks the tokens: LPC
// neighbouring lanes share a column, lane part p keeping the rows p * DR .. p * DR + DR - 1 in registers (dk = LPC * DR);
// the sums over the rows are joined within each group of LPC lanes by exchanges of neighbours, whatever else the step
// holds. The second wave only fetches: the rows of q, k and decay, the values of the block's columns and beta come
// through a ring of two slots in LDS, kGroup tokens to a slot (sixteen; two for steps of single tokens, whose blocks
// then need little LDS), and while the first wave works on one slot the second asks for the next group's rows (all its lanes together, 16 bytes each), waits for them and fills the other
// slot. The two meet at a barrier per slot that waits for LDS alone, so the walking wave never waits for memory: its
// chain from token to token is arithmetic and LDS reads, and it reads a token's rows while it works on the one before.

// The sum over a group of four or eight neighbouring lanes, in every lane of the group, by exchanges through the data
// path of the vector unit itself (no LDS): neighbours at distance one, then two, then the other quad of the eight
// (a mirror within the half row: all lanes of a quad hold the quad's sum by then, so any lane of the other quad will do).
template <int CTRL>
__device__ inline float lane_exchange(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int LPC>
__device__ inline float lanes_sum(float v) {
  v += lane_exchange<0xB1>(v);               // quad_perm [1, 0, 3, 2]
  v += lane_exchange<0x4E>(v);               // quad_perm [2, 3, 0, 1]
  if (LPC == 8) v += lane_exchange<0x141>(v);  // row_half_mirror
  return v;
}
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int DR, int LPC, int kGroup>
__global__ __launch_bounds__(2 * kWave) void gdr_scan_lanes_kernel(const float* __restrict__ x, float* __restrict__ state,
                                                                   float* __restrict__ o, const int* __restrict__ q_start,
                                                                   const int* __restrict__ state_slots, Geometry s) {
  constexpr int kCols = kWave / LPC, kDk = DR * LPC;
  constexpr int kPieces = (3 * kDk + kCols) / 4;     // 16-byte pieces of a token: its q, k and decay rows, its kCols values
  constexpr int kTok = 4 * kPieces + 4;              // floats of a token in the ring: these and beta (and padding)
  constexpr int kItems = kGroup * kPieces;
  constexpr int kMine = (kItems + kWave - 1) / kWave;
  __shared__ __attribute__((aligned(16))) float ring[2][kGroup * kTok];
  const int seq = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x & (kWave - 1);
  const bool fetches = threadIdx.x >= kWave;
  const int col0 = blockIdx.z * kCols, g = hd / (s.H / s.G);
  const int t_begin = q_start[seq], t_end = q_start[seq + 1], width = s.width();
  const int groups = (t_end - t_begin + kGroup - 1) / kGroup;
  if (groups <= 0) return;

  if (fetches) {
    const int qo = s.q0() + g * kDk, ko = s.k0() + g * kDk, ao = s.a0() + hd * kDk, vo = s.v0() + hd * s.dv + col0, bo = s.b0() + hd;
    // Where this lane's pieces of a group lie in a token's row and in the ring: piece j of the lane is piece
    // (lane + 64 j) % kPieces of token (lane + 64 j) / kPieces of the group. A piece that is not there (behind the
    // group's pieces, or values of columns past dv, which is a multiple of four) has the offset -1.
    int from[kMine], to[kMine], tok_of[kMine];
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
      const int i = lane + kWave * j, piece = i % kPieces, e = 4 * piece;
      tok_of[j] = i / kPieces;
      to[j] = tok_of[j] * kTok + e;
      from[j] = e < kDk ? qo + e : e < 2 * kDk ? ko + e - kDk : e < 3 * kDk ? ao + e - 2 * kDk : vo + e - 3 * kDk;
      if (i >= kItems || (e >= 3 * kDk && col0 + e - 3 * kDk >= s.dv)) from[j] = -1;
    }
    for (int grp = 0; grp < groups; ++grp) {
      const int first = t_begin + grp * kGroup;
      float4 in_flight[kMine];
      float beta = 0.f;
#pragma unroll
      for (int j = 0; j < kMine; ++j) {
        const int t = first + tok_of[j];
        in_flight[j] = float4{0.f, 0.f, 0.f, 0.f};
        if (from[j] >= 0 && t < t_end) in_flight[j] = *reinterpret_cast<const float4*>(x + static_cast<size_t>(t) * width + from[j]);
      }
      if (lane < kGroup && first + lane < t_end) beta = x[static_cast<size_t>(first + lane) * width + bo];
      float* slot = ring[grp & 1];   // the walking wave left it at the barrier before this group
#pragma unroll
      for (int j = 0; j < kMine; ++j)
        if (lane + kWave * j < kItems) *reinterpret_cast<float4*>(slot + to[j]) = in_flight[j];
      if (lane < kGroup) slot[lane * kTok + 4 * kPieces] = beta;
      lds_barrier();   // the slot is full; the walking wave has finished the slot before it
    }
    lds_barrier();
    return;
  }

  const int part = lane % LPC, col = col0 + lane / LPC, row0 = part * DR;
  const bool has_col = col < s.dv;
  float* st = state + (static_cast<size_t>(state_slots[seq]) * s.H + hd) * s.dk * s.dv;
  float S[DR];
#pragma unroll
  for (int r = 0; r < DR; r += 4) {
    const float4 v4 = has_col ? *reinterpret_cast<const float4*>(st + static_cast<size_t>(col) * kDk + row0 + r) : float4{0.f, 0.f, 0.f, 0.f};
    S[r] = v4.x, S[r + 1] = v4.y, S[r + 2] = v4.z, S[r + 3] = v4.w;
  }
  lds_barrier();   // the first slot is full
  for (int grp = 0; grp < groups; ++grp) {
    const int first = t_begin + grp * kGroup;
    const int count = t_end - first < kGroup ? t_end - first : kGroup;
    const float* slot = ring[grp & 1];
    float4 a[DR / 4], k[DR / 4], q[DR / 4];
    float v, beta;
    auto read = [&](int i, float4* ra, float4* rk, float4* rq, float& rv, float& rb) {
      const float* tk = slot + i * kTok;
#pragma unroll
      for (int r = 0; r < DR / 4; ++r) {
        ra[r] = *reinterpret_cast<const float4*>(tk + 2 * kDk + row0 + 4 * r);
        rk[r] = *reinterpret_cast<const float4*>(tk + kDk + row0 + 4 * r);
        rq[r] = *reinterpret_cast<const float4*>(tk + row0 + 4 * r);
      }
      rv = tk[3 * kDk + lane / LPC];
      rb = tk[4 * kPieces];
    };
    // one token: decay, the sum S^T k, the correction along k, the sum S^T q
    auto step = [&](int i, const float4* ta, const float4* tk, const float4* tq, float tv, float tb) {
      float4 pk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < DR / 4; ++r) {
        S[4 * r] *= ta[r].x, S[4 * r + 1] *= ta[r].y, S[4 * r + 2] *= ta[r].z, S[4 * r + 3] *= ta[r].w;
        pk.x = fmaf(S[4 * r], tk[r].x, pk.x), pk.y = fmaf(S[4 * r + 1], tk[r].y, pk.y);
        pk.z = fmaf(S[4 * r + 2], tk[r].z, pk.z), pk.w = fmaf(S[4 * r + 3], tk[r].w, pk.w);
      }
      const float u = tb * (tv - lanes_sum<LPC>((pk.x + pk.y) + (pk.z + pk.w)));
      float4 pq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < DR / 4; ++r) {
        S[4 * r] = fmaf(tk[r].x, u, S[4 * r]), S[4 * r + 1] = fmaf(tk[r].y, u, S[4 * r + 1]);
        S[4 * r + 2] = fmaf(tk[r].z, u, S[4 * r + 2]), S[4 * r + 3] = fmaf(tk[r].w, u, S[4 * r + 3]);
        pq.x = fmaf(S[4 * r], tq[r].x, pq.x), pq.y = fmaf(S[4 * r + 1], tq[r].y, pq.y);
        pq.z = fmaf(S[4 * r + 2], tq[r].z, pq.z), pq.w = fmaf(S[4 * r + 3], tq[r].w, pq.w);
      }
      const float out = lanes_sum<LPC>((pq.x + pq.y) + (pq.z + pq.w));
      if (part == 0 && has_col) o[static_cast<size_t>(first + i) * s.H * s.dv + hd * s.dv + col] = out;
    };
    // two sets of registers take turns: a token's rows are read while the token before it is worked on, and nothing
    // is moved from one set to the other
    float4 a2[DR / 4], k2[DR / 4], q2[DR / 4];
    float v2, beta2;
    read(0, a, k, q, v, beta);
    for (int i = 0; i < count; i += 2) {
      read(i + 1 < count ? i + 1 : i, a2, k2, q2, v2, beta2);
      step(i, a, k, q, v, beta);
      if (i + 1 < count) {
        read(i + 2 < count ? i + 2 : i + 1, a, k, q, v, beta);
        step(i + 1, a2, k2, q2, v2, beta2);
      }
    }
    lds_barrier();   // done with this slot; the one after it is full
  }
  if (has_col) {
#pragma unroll
    for (int r = 0; r < DR; r += 4)
      *reinterpret_cast<float4*>(st + static_cast<size_t>(col) * kDk + row0 + r) = float4{S[r], S[r + 1], S[r + 2], S[r + 3]};
  }
}

__global__ __launch_bounds__(kThreads) void gdr_finish_kernel(const float* __restrict__ o, const float* __restrict__ x,
                                                              const void* __restrict__ gain, int gain_dt, float eps,
                                                              float out_scale, void* __restrict__ out, int out_dt,
                                                              size_t out_ld, Geometry s) {
  const int n = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* gate = x + static_cast<size_t>(n) * s.width() + s.g0();
  for (int hd = wave; hd < s.H; hd += kThreads / kWave) {
    const float* row = o + (static_cast<size_t>(n) * s.H + hd) * s.dv;
    float y[kMaxHead / kWave], ss = 0.f;
#pragma unroll
    for (int u = 0; u < kMaxHead / kWave; ++u) {
      const int e = lane + kWave * u;
      y[u] = e < s.dv ? row[e] : 0.f;
      ss = fmaf(y[u], y[u], ss);
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(s.dv) + eps);
#pragma unroll
    for (int u = 0; u < kMaxHead / kWave; ++u) {
      const int e = lane + kWave * u;
      if (e < s.dv)
        store_from_float(out, out_dt, n * out_ld + hd * s.dv + e,
                         y[u] * inv * load_as_float(gain, gain_dt, e) * gate[hd * s.dv + e] * out_scale);
    }
  }
}

bool good(const Geometry& s) {
  return s.H > 0 && s.G > 0 && s.H % s.G == 0 && s.dk > 0 && s.dk <= kMaxHead && s.dv > 0 && s.dv <= kMaxHead;
}

}  // namespace

extern "C" long pyre_gdr_row_width(int H, int G, int dk, int dv) { return Geometry{H, G, dk, dv}.width(); }

extern "C" int pyre_gdr_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                const float* bias, const float* taps_w, int taps, float* conv_state, const int* state_slots,
                                const int* seq_of_token, const int* q_start, int n_seqs, const void* a2, int a2_dt,
                                const float* dt_bias, const float* rate, const void* g2, int g2_dt, float unit_eps,
                                float* x, int n, int H, int G, int dk, int dv, int rank_a, int rank_g, hipStream_t stream) {
  const Geometry s{H, G, dk, dv};
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(a2_dt) && known_dtype(g2_dt) && n_partials >= 1, "gdr_prepare: bad dtypes");
  PYRE_REQUIRE(good(s), "gdr_prepare: heads %d / %d of %d / %d elements are not taken (heads a multiple of the key heads, sizes up to %d)",
               H, G, dk, dv, kMaxHead);
  PYRE_REQUIRE(rank_a > 0 && rank_a <= kMaxRank && rank_g > 0 && rank_g <= kMaxRank && a2 && g2 && dt_bias && rate,
               "gdr_prepare: low-rank inputs of %d and %d columns (up to %d) and their matrices are needed", rank_a, rank_g, kMaxRank);
  PYRE_REQUIRE(taps_w ? (taps >= 1 && taps <= kMaxTaps && (taps == 1 || conv_state)) : taps == 0,
               "gdr_prepare: %d taps (of at most %d) need their weights and, beyond one, the state", taps, kMaxTaps);
  PYRE_REQUIRE(state_slots && seq_of_token && q_start && x && n_seqs >= 0 && n_seqs <= 65535 && unit_eps > 0.f,
               "gdr_prepare: the step's arrays are needed");
  if (n <= 0) return 0;
  ConvIn in{proj, proj_dt, n_partials, static_cast<size_t>(partial_stride), ld, col0, taps_w, taps, conv_state,
            2 * G * dk + H * dv};
  in.bias = bias;
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (taps <= kConvVecTaps && dk % 4 == 0 && dv % 4 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 &&
      a16(proj) && a16(bias) && a16(taps_w) && a16(conv_state) && a16(x)) {
    const int parts = n >= 512 ? 1 : n >= 64 ? 2 : 8;  // a step of few tokens: more blocks a token
    PYRE_DISPATCH(proj_dt, TP,
        hipLaunchKernelGGL(gdr_prepare_vec_kernel<TP>, dim3(n, parts), dim3(kThreads), 0, stream, in, state_slots,
                           seq_of_token, q_start, a2, a2_dt, dt_bias, rate, g2, g2_dt, unit_eps, x, s, rank_a, rank_g));
  } else {
    hipLaunchKernelGGL(gdr_prepare_kernel, dim3(n), dim3(kThreads), 0, stream, in, state_slots, seq_of_token, q_start, a2,
                       a2_dt, dt_bias, rate, g2, g2_dt, unit_eps, x, s, rank_a, rank_g);
  }
  if (check_launch("gdr_prepare")) return 1;
  if (taps > 1 && n_seqs > 0) {
    const int cols = (in.channels + kThreads - 1) / kThreads;
    hipLaunchKernelGGL(conv_state_update_kernel, dim3(n_seqs, cols < 64 ? cols : 64), dim3(kThreads), 0, stream, in,
                       conv_state, state_slots, q_start);
    return check_launch("gdr_conv_state_update");
  }
  return 0;
}

extern "C" int pyre_gdr_scan(const float* x, float* state, float* o, const int* q_start, const int* state_slots, int n_seqs,
                             int max_tokens, int H, int G, int dk, int dv, hipStream_t stream) {
  const Geometry s{H, G, dk, dv};
  PYRE_REQUIRE(good(s) && H <= 65535, "gdr_scan: heads %d / %d of %d / %d elements are not taken", H, G, dk, dv);
  PYRE_REQUIRE(x && state && o && q_start && state_slots, "gdr_scan: rows, state and the step's arrays are needed");
  if (n_seqs <= 0) return 0;
  if (dk % 16 == 0 && dk <= 128 && dv % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    // eight lanes a column where that leaves each a multiple of four rows, else four
#define PYRE_LANES(DR, LPC)                                                                                             \
  do {                                                                                                                  \
    const dim3 lanes_grid(n_seqs, H, (dv + kWave / LPC - 1) / (kWave / LPC));                                           \
    if (max_tokens > 0 && max_tokens <= 2)                                                                              \
      hipLaunchKernelGGL((gdr_scan_lanes_kernel<DR, LPC, 2>), lanes_grid, dim3(2 * kWave), 0, stream, x, state, o, q_start, \
                         state_slots, s);                                                                               \
    else                                                                                                                \
      hipLaunchKernelGGL((gdr_scan_lanes_kernel<DR, LPC, 16>), lanes_grid, dim3(2 * kWave), 0, stream, x, state, o, q_start, \
                         state_slots, s);                                                                               \
  } while (0)
    switch (dk) {
      case 16: PYRE_LANES(4, 4); break;
      case 32: PYRE_LANES(4, 8); break;
      case 48: PYRE_LANES(12, 4); break;
      case 64: PYRE_LANES(8, 8); break;
      case 80: PYRE_LANES(20, 4); break;
      case 96: PYRE_LANES(12, 8); break;
      case 112: PYRE_LANES(28, 4); break;
      default: PYRE_LANES(16, 8); break;
    }
#undef PYRE_LANES
    return check_launch("gdr_scan");
  }
  const dim3 grid(n_seqs, H, (dv + kWave - 1) / kWave);
#define PYRE_SCAN(DR) \
  hipLaunchKernelGGL(gdr_scan_kernel<DR>, grid, dim3(kThreads), 0, stream, x, state, o, q_start, state_slots, s)
  if (dk <= 32) PYRE_SCAN(8);
  else if (dk <= 64) PYRE_SCAN(16);
  else if (dk <= 128) PYRE_SCAN(32);
  else PYRE_SCAN(64);
#undef PYRE_SCAN
  return check_launch("gdr_scan");
}

extern "C" int pyre_gdr_finish(const float* o, const float* x, const void* gain, int gain_dt, float eps, float out_scale,
                               void* out, int out_dt, long out_ld, int n, int H, int G, int dk, int dv, hipStream_t stream) {
  const Geometry s{H, G, dk, dv};
  PYRE_REQUIRE(known_dtype(gain_dt) && known_dtype(out_dt) && gain, "gdr_finish: bad dtypes");
  PYRE_REQUIRE(good(s) && eps > 0.f && out_ld >= static_cast<long>(H) * dv, "gdr_finish: sizes %d x %d are not taken", H, dv);
  if (n <= 0) return 0;
  hipLaunchKernelGGL(gdr_finish_kernel, dim3(n), dim3(kThreads), 0, stream, o, x, gain, gain_dt, eps, out_scale, out,
                     out_dt, static_cast<size_t>(out_ld), s);
  return check_launch("gdr_finish");
}
