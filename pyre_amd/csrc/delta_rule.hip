// The gated delta rule: per request and head a float32 state S [dk][dv] that every token first decays per key channel,
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
// gdr_scan      the recurrence over each request's tokens of the step, from and into the state. A block: one request,
//               one head, 64 columns of the state (a lane a column); wave w keeps the rows w, w + 4, .. in registers.
//               The columns of S never meet, so a token costs two sums over the rows (S^T k, then S^T q), each joined
//               over the four waves through LDS in a fixed order.
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
  __host__ __device__ int width() const { return b0() + H; }
};

__device__ inline float sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float silu(float z) { return z / (1.f + expf(-z)); }
__device__ inline float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

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
    float z = 0.f;
    for (int r = 0; r < rank_a; ++r) z = fmaf(load_as_float(a2, a2_dt, static_cast<size_t>(i) * rank_a + r), low[r], z);
    xr[s.a0() + i] = expf(rate[i / s.dk] * softplus(z + dt_bias[i]));
  }
  for (int i = tid; i < s.H * s.dv; i += kThreads) {
    float z = 0.f;
    for (int r = 0; r < rank_g; ++r) z = fmaf(load_as_float(g2, g2_dt, static_cast<size_t>(i) * rank_g + r), low[kMaxRank + r], z);
    xr[s.g0() + i] = sigmoid(z);
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
    S[r] = has_col && row < s.dk ? st[static_cast<size_t>(row) * s.dv + col] : 0.f;
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
    if (has_col && row < s.dk) st[static_cast<size_t>(row) * s.dv + col] = S[r];
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
  hipLaunchKernelGGL(gdr_prepare_kernel, dim3(n), dim3(kThreads), 0, stream, in, state_slots, seq_of_token, q_start, a2,
                     a2_dt, dt_bias, rate, g2, g2_dt, unit_eps, x, s, rank_a, rank_g);
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
                             int H, int G, int dk, int dv, hipStream_t stream) {
  const Geometry s{H, G, dk, dv};
  PYRE_REQUIRE(good(s) && H <= 65535, "gdr_scan: heads %d / %d of %d / %d elements are not taken", H, G, dk, dv);
  PYRE_REQUIRE(x && state && o && q_start && state_slots, "gdr_scan: rows, state and the step's arrays are needed");
  if (n_seqs <= 0) return 0;
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
