// The step between the input product and the attention kernels for an attention whose projected queries, keys and
// values first go through a short causal convolution over time:
//
//   u_t      = the product's columns of token t (sum of its partial sums): nq query heads and nkv key heads of dk,
//              nkv value heads of dv, then nq * dv gate columns
//   y_t[c]   = sum_j taps[j][c] * u_(t - (T - 1) + j)[c],  j = 0 .. T - 1, for the query, key and value channels c
//              (the taps as float32 [T][channels]: a tap's weights of neighbouring channels lie together);
//              rows before the request's first token are zero, rows before the step's first token of the request come
//              from the request's state, which holds its last T - 1 rows u (float32 [T - 1][channels], oldest first)
//   q, k     = per head: y / sqrt(mean(y^2) + eps) * gain   (gains over dk, shared by the heads; or not normed)
//   q, k     = their first `rot` elements turned by position: pairs (e, e + rot/2) or neighbours (2e, 2e + 1)
//   gate     = sigmoid(u_t[gate columns])                   (float32, one per element of the heads' outputs)
//
// conv_qkv_write       a wave per token and head (four neighbouring elements a lane, dk <= 256): it norms the head,
//                      leaves it in LDS, turns the pairs and stores queries (rows) and keys (pages); further waves take
//                      256 columns of values and gates each. A form for any sizes and element types has one block a
//                      token, whose waves take a head at a time.
// conv_state_update    one block a request, after every token has read the old state: the last T - 1 rows u of the
//                      request, taken from the step's rows and, for a step shorter than that, from the old state.
//
// A sum over the taps runs in the order j = 0 .. T - 1 wherever its inputs come from, so a token's result does not
// depend on where a step begins. All arithmetic float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_conv.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = kConvThreads;
constexpr int kMaxHead = 256;
constexpr int kMaxTaps = 16;

template <typename TC>
__global__ __launch_bounds__(kThreads) void conv_qkv_write_kernel(
    ConvIn in, const int* __restrict__ state_slots, const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps, const float* __restrict__ cos,
    const float* __restrict__ sin, int rot, int neighbours, const int* __restrict__ positions, void* __restrict__ q_out,
    int q_dt, TC* __restrict__ k_cache, TC* __restrict__ v_cache, float* __restrict__ gate_out,
    const int* __restrict__ slots, int nq, int nkv, int dk, int dv, int page_size, int write_kv) {
  __shared__ float head_s[kThreads / kWave][kMaxHead];
  const int n = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int seq = seq_of_token[n], run = n - q_start[seq], st = state_slots[seq];
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const int half = rot / 2;
  const size_t trig = static_cast<size_t>(positions[n]) * half;

  for (int base = 0; base < nq + nkv; base += kThreads / kWave) {  // the same number of rounds for every wave
    const int head = base + wave;
    const bool there = head < nq + nkv;
    if (there) {
      float x[4], ss = 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = lane + 64 * u;
        x[u] = e < dk ? conv_value(in, n, run, st, head * dk + e) : 0.f;
        ss += x[u] * x[u];
      }
      const float* gain = head < nq ? q_gain : k_gain;
      const float inv = gain ? 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps) : 1.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = lane + 64 * u;
        if (e < dk) head_s[wave][e] = gain ? x[u] * inv * gain[e] : x[u];
      }
    }
    __syncthreads();
    if (there) {
      const float* hs = head_s[wave];
      auto put = [&](int e, float v) {
        if (head < nq) store_from_float(q_out, q_dt, (static_cast<size_t>(n) * nq + head) * dk + e, v);
        else if (slot >= 0) k_cache[((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * dk + e] = from_float<TC>(v);
      };
      for (int i = lane; i < half; i += kWave) {
        const int e1 = neighbours ? 2 * i : i, e2 = neighbours ? 2 * i + 1 : i + half;
        float a, b;
        rotate_pair(hs[e1], hs[e2], cos[trig + i], sin[trig + i], a, b);
        put(e1, a), put(e2, b);
      }
      for (int e = rot + lane; e < dk; e += kWave) put(e, hs[e]);
    }
    __syncthreads();
  }
  const int v0 = (nq + nkv) * dk;
  if (slot >= 0)
    for (int i = tid; i < nkv * dv; i += kThreads) {
      const int g = i / dv, e = i % dv;
      v_cache[((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e] = from_float<TC>(conv_value(in, n, run, st, v0 + i));
    }
  if (gate_out)
    for (int i = tid; i < nq * dv; i += kThreads)
      gate_out[static_cast<size_t>(n) * nq * dv + i] = 1.f / (1.f + expf(-product_value(in, n, in.channels + i)));
}


// The same with a wave per block, four elements a lane and an element's partial sums asked for together: blocks
// 0 .. nq + nkv - 1 of a token take a head each, the blocks behind them 256 value or gate columns each. Head sizes, the
// product's width, first column and stride are multiples of four; queries and caches share one element type. The sums
// run in the order of the kernel above: the same bits.
template <typename TP, typename TC>
__global__ __launch_bounds__(kWave) void conv_qkv_write_vec_kernel(
    ConvIn in, const int* __restrict__ state_slots, const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps, const float* __restrict__ cos,
    const float* __restrict__ sin, int rot, int neighbours, const int* __restrict__ positions, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, float* __restrict__ gate_out, const int* __restrict__ slots,
    int nq, int nkv, int dk, int dv, int page_size, int write_kv) {
  __shared__ __attribute__((aligned(16))) float xs[kMaxHead];
  const int n = blockIdx.x, lane = threadIdx.x;
  const int seq = seq_of_token[n], run = n - q_start[seq], st = state_slots[seq];
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const TP* proj = static_cast<const TP*>(in.proj);
  if (static_cast<int>(blockIdx.y) >= nq + nkv) {
    // 256 columns of the values, then of the gates
    const int i = (static_cast<int>(blockIdx.y) - nq - nkv) * 4 * kWave + 4 * lane, nv = nkv * dv;
    if (i < nv) {
      if (slot >= 0) {
        const int g = i / dv, e = i % dv;
        Vec4<TC>::store(v_cache + ((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e,
                        conv_value4(in, proj, n, run, st, (nq + nkv) * dk + i));
      }
    } else if (gate_out && i - nv < nq * dv) {
      const float4 z = sum_partials4(proj + static_cast<size_t>(n) * in.ld + in.col0 + in.channels + (i - nv), in.partial_stride, in.n_partials);
      *reinterpret_cast<float4*>(gate_out + static_cast<size_t>(n) * nq * dv + (i - nv)) =
          float4{1.f / (1.f + expf(-z.x)), 1.f / (1.f + expf(-z.y)), 1.f / (1.f + expf(-z.z)), 1.f / (1.f + expf(-z.w))};
    }
    return;
  }
  const int head = blockIdx.y, e = 4 * lane, half = rot / 2;
  const bool mine = e < dk;
  float4 x = {0.f, 0.f, 0.f, 0.f};
  if (mine) x = conv_value4(in, proj, n, run, st, head * dk + e);
  const float* gain = head < nq ? q_gain : k_gain;
  if (gain) {
    // the sum of squares in the order of the kernel above: a lane's elements e, e + 64, .. there, four neighbours here;
    // both are wave sums of per-lane sums, a difference of rounding
    const float inv = 1.f / sqrtf(wave_sum((x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w)) / static_cast<float>(dk) + eps);
    if (mine) {
      const float4 g = *reinterpret_cast<const float4*>(gain + e);
      x = float4{x.x * inv * g.x, x.y * inv * g.y, x.z * inv * g.z, x.w * inv * g.w};
    }
  }
  if (mine) *reinterpret_cast<float4*>(xs + e) = x;
  __syncthreads();
  if (!mine) return;
  float y[4] = {x.x, x.y, x.z, x.w};
  const size_t trig = static_cast<size_t>(positions[n]) * half;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int el = e + u;
    if (el >= rot) continue;
    // the pair's index, and whether this element is its first or its second
    const int pair = neighbours ? el >> 1 : (el < half ? el : el - half);
    const bool first = neighbours ? !(el & 1) : el < half;
    const int partner = neighbours ? el ^ 1 : (first ? el + half : el - half);
    float a, b;
    if (first) rotate_pair(y[u], xs[partner], cos[trig + pair], sin[trig + pair], a, b);
    else rotate_pair(xs[partner], y[u], cos[trig + pair], sin[trig + pair], a, b);
    y[u] = first ? a : b;
  }
  const float4 out = {y[0], y[1], y[2], y[3]};
  if (head < nq) Vec4<TC>::store(q_out + (static_cast<size_t>(n) * nq + head) * dk + e, out);
  else if (slot >= 0) Vec4<TC>::store(k_cache + ((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * dk + e, out);
}

}  // namespace

extern "C" int pyre_conv_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                   const float* taps_w, int taps, float* conv_state, const int* state_slots,
                                   const int* seq_of_token, const int* q_start, int n_seqs, const float* q_gain,
                                   const float* k_gain, float eps, const float* cos, const float* sin, int rot,
                                   int neighbours, const int* positions, void* q_out, int q_dt, void* k_cache,
                                   void* v_cache, int cache_dt, float* gate_out, const int* slots, int n, int nq, int nkv,
                                   int dk, int dv, int page_size, int write_kv, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(q_dt) && known_dtype(cache_dt) && n_partials >= 1, "conv_qkv_write: bad dtypes");
  PYRE_REQUIRE(nq > 0 && nkv > 0 && dk > 0 && dk <= kMaxHead && dv > 0 && page_size > 0,
               "conv_qkv_write: head sizes %d / %d are outside what the kernel takes (keys up to %d)", dk, dv, kMaxHead);
  PYRE_REQUIRE(!write_kv || (k_cache && v_cache && slots), "conv_qkv_write: a cache write needs caches and slots");
  PYRE_REQUIRE((!q_gain && !k_gain) || (q_gain && k_gain && eps > 0.f), "conv_qkv_write: both gains and a positive eps, or no norm");
  PYRE_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || (cos && sin)),
               "conv_qkv_write: %d turned elements of a head of %d need tables and an even number", rot, dk);
  PYRE_REQUIRE(taps_w ? (taps >= 1 && taps <= kMaxTaps && (taps == 1 || conv_state)) : taps == 0,
               "conv_qkv_write: %d taps (of at most %d) need their weights and, beyond one, the state", taps, kMaxTaps);
  PYRE_REQUIRE(state_slots && seq_of_token && q_start && positions && n_seqs >= 0 && n_seqs <= 65535, "conv_qkv_write: the step's arrays are needed");
  if (n <= 0) return 0;
  const ConvIn in{proj, proj_dt, n_partials, static_cast<size_t>(partial_stride), ld, col0, taps_w, taps, conv_state,
                  (nq + nkv) * dk + nkv * dv};
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const int tail_blocks = (nkv * dv + (gate_out ? nq * dv : 0) + 4 * kWave - 1) / (4 * kWave);
  if (taps <= kConvVecTaps && dk % 4 == 0 && dv % 4 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 && q_dt == cache_dt &&
      nq + nkv + tail_blocks <= 65535 && a16(proj) && a16(q_out) && a16(k_cache) && a16(v_cache) && a16(gate_out) &&
      a16(taps_w) && a16(conv_state) && a16(q_gain) && a16(k_gain)) {
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL((conv_qkv_write_vec_kernel<TP, TC>), dim3(n, nq + nkv + tail_blocks), dim3(kWave), 0, stream, in,
                           state_slots, seq_of_token, q_start, q_gain, k_gain, eps, cos, sin, rot, neighbours, positions,
                           static_cast<TC*>(q_out), static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), gate_out, slots,
                           nq, nkv, dk, dv, page_size, write_kv)));
  } else {
    PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL(conv_qkv_write_kernel<TC>, dim3(n), dim3(kThreads), 0, stream, in, state_slots, seq_of_token,
                           q_start, q_gain, k_gain, eps, cos, sin, rot, neighbours, positions, q_out, q_dt,
                           static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), gate_out, slots, nq, nkv, dk, dv,
                           page_size, write_kv));
  }
  if (check_launch("conv_qkv_write")) return 1;
  if (taps > 1 && n_seqs > 0) {
    const int cols = (in.channels + kThreads - 1) / kThreads;
    hipLaunchKernelGGL(conv_state_update_kernel, dim3(n_seqs, cols < 64 ? cols : 64), dim3(kThreads), 0, stream, in,
                       conv_state, state_slots, q_start);
    return check_launch("conv_state_update");
  }
  return 0;
}
