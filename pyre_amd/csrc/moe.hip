// A mixture of small feed-forward layers whose router squashes its logits one by one.
//
//   route_topk   z = the router product's partial sums, s = sigmoid(z); per token the `top` experts of largest
//                s (the lower index among equals), each weighted s / (sum of the chosen s + 1e-20); written as a
//                dense row gates[n, experts] (0 for an expert that is not chosen), float32. The experts are compared
//                by z, which orders them as s does and still tells two apart where both their s round to one.
//                In its softmax form the chosen experts' weights are the softmax over their logits alone. Columns of
//                the product behind the experts' (`extra`) are gates of their own: their sigmoid is written behind
//                the experts' weights (a shared expert's gate per token).
//   expert_act   the experts' way up is one product over [W_0; W_1; ...; W_shared]; its result becomes
//                act[n, e ff + j] = gates[n, e] f(up[n, e ff + j]) for the routed experts and f(up) for the columns
//                of the shared expert behind them, f(u) = max(u, 0)^2. One product over
//                [W'_0 | W'_1 | ... | W'_shared] then gives the weighted sum of the chosen experts' results and the
//                shared expert's in one go.
//
//   route_grouped   s = softmax(z) over all experts; the choice goes by c = s + correction: the experts form `groups`
//                equal groups of neighbours, a group is worth its largest c, and only the experts of the `keep` best
//                groups can be chosen (the lower index among equals, of groups as of experts); the `top` chosen
//                experts get their s itself as weight (no renormalisation), the others 0.
//   expert_glu_act  experts that are gated units: one product over [G_0; ..; G_E-1; U_0; ..; U_E-1], then
//                act[n, e ff + j] = gates[n, e] silu(g) u.
//   add_weighted_rows  experts that hand their input back: p[n, :] += (sum of their weights) h[n, :].
//
// All arithmetic is float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kMaxPerLane = 8;  // experts a lane keeps: up to 512 experts

__global__ __launch_bounds__(kWave) void route_topk_kernel(const void* __restrict__ z, int z_dt, int n_partials,
                                                           size_t partial_stride, const void* __restrict__ bias,
                                                           int bias_dt, float* __restrict__ gates, int experts, int top,
                                                           int softmax, int extra) {
  const int n = blockIdx.x, lane = threadIdx.x, width = experts + extra;
  float s[kMaxPerLane], w[kMaxPerLane];  // s: the logits still to choose from
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    s[u] = -INFINITY, w[u] = 0.f;
    if (e < experts) {
      float v = 0.f;
      for (int p = 0; p < n_partials; ++p) v += load_as_float(z, z_dt, p * partial_stride + static_cast<size_t>(n) * width + e);
      if (bias) v += load_as_float(bias, bias_dt, e);
      s[u] = fmaxf(v, -3.0e38f);  // finite, so that it beats the mark of an expert that is taken or not there
    }
  }
  // the columns behind the experts: gates of their own, sigmoid of the logit
  for (int e = experts + lane; e < width; e += kWave) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_float(z, z_dt, p * partial_stride + static_cast<size_t>(n) * width + e);
    if (bias) v += load_as_float(bias, bias_dt, e);
    gates[static_cast<size_t>(n) * width + e] = 1.f / (1.f + expf(-v));
  }
  float total = 0.f, first = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = experts;
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (s[u] > best) best = s[u], at = lane + kWave * u;  // ascending index within the lane: the first of equals stays
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    if (k == 0) first = best;  // the largest logit: the softmax over the chosen ones is taken relative to it
    const float score = softmax ? expf(best - first) : 1.f / (1.f + expf(-best));
    total += score;
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (at == lane + kWave * u) w[u] = score, s[u] = -INFINITY;
  }
  const float inv = 1.f / (softmax ? total : total + 1e-20f);
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    if (e < experts) gates[static_cast<size_t>(n) * width + e] = w[u] * inv;
  }
}

__global__ __launch_bounds__(256) void expert_act_kernel(const void* __restrict__ up, int up_dt, int n_partials,
                                                         size_t partial_stride, const float* __restrict__ gates,
                                                         void* __restrict__ out, int out_dt, size_t total, int experts,
                                                         int ff, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / width;
  const int c = static_cast<int>(i % width), e = c / ff;
  const float g = e < experts ? gates[n * experts + e] : 1.f;
  float y = 0.f;
  if (g != 0.f) {
    float u = 0.f;
    for (int p = 0; p < n_partials; ++p) u += load_as_float(up, up_dt, p * partial_stride + i);
    u = fmaxf(u, 0.f);
    y = g * (u * u);
  }
  store_from_float(out, out_dt, i, y);
}

// Four columns a thread (the experts' sizes, the shared expert's and the partial sums' stride are multiples of four,
// so the four share an expert); columns of an expert that the token does not take are not read.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void expert_act_vec_kernel(const TI* __restrict__ up, int n_partials, size_t partial_stride,
                                                             const float* __restrict__ gates, TO* __restrict__ out,
                                                             size_t total4, int experts, int ff, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int per_row = width / 4;
  const size_t n = i / per_row;
  const int c = 4 * static_cast<int>(i % per_row), e = c / ff;
  const float g = e < experts ? gates[n * experts + e] : 1.f;
  float4 y = {0.f, 0.f, 0.f, 0.f};
  if (g != 0.f) {
    const float4 u = sum_partials4(up + n * width + c, partial_stride, n_partials);
    const float a = fmaxf(u.x, 0.f), b = fmaxf(u.y, 0.f), cc = fmaxf(u.z, 0.f), d = fmaxf(u.w, 0.f);
    y = float4{g * (a * a), g * (b * b), g * (cc * cc), g * (d * d)};
  }
  Vec4<TO>::store(out + n * width + c, y);
}

// A wave a token; lane l keeps experts l, l + 64, ... The scores are kept to the end; `c` is what is still to choose from.
__global__ __launch_bounds__(kWave) void route_grouped_kernel(const void* __restrict__ z, int z_dt, int n_partials,
                                                              size_t partial_stride, const void* __restrict__ bias,
                                                              int bias_dt, const float* __restrict__ correction,
                                                              float* __restrict__ gates, int experts, int top, int groups,
                                                              int keep) {
  __shared__ float group_best[kWave * kMaxPerLane];
  const int n = blockIdx.x, lane = threadIdx.x, size = experts / groups;
  float s[kMaxPerLane], c[kMaxPerLane], w[kMaxPerLane];
  float mx = -INFINITY;
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    s[u] = -INFINITY, w[u] = 0.f;
    if (e < experts) {
      float v = 0.f;
      for (int p = 0; p < n_partials; ++p) v += load_as_float(z, z_dt, p * partial_stride + static_cast<size_t>(n) * experts + e);
      if (bias) v += load_as_float(bias, bias_dt, e);
      s[u] = v;
      mx = fmaxf(mx, v);
    }
  }
  mx = wave_max(mx);
  float total = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    s[u] = lane + kWave * u < experts ? expf(s[u] - mx) : 0.f;
    total += s[u];
  }
  const float inv = 1.f / wave_sum(total);
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    s[u] *= inv;
    c[u] = e < experts ? fmaxf(s[u] + (correction ? correction[e] : 0.f), -3.0e38f) : -INFINITY;
  }
  if (groups > 1) {
    // every group's largest c, then the `keep` best groups: an expert outside them cannot be chosen
    for (int g = lane; g < groups; g += kWave) group_best[g] = -INFINITY;
    __syncthreads();
    for (int g = 0; g < groups; ++g) {
      float best = -INFINITY;
#pragma unroll
      for (int u = 0; u < kMaxPerLane; ++u) {
        const int e = lane + kWave * u;
        if (e < experts && e / size == g) best = fmaxf(best, c[u]);
      }
      best = wave_max(best);
      if (lane == 0) group_best[g] = best;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u) {
      const int e = lane + kWave * u;
      if (e >= experts) continue;
      const int g = e / size;
      const float mine = group_best[g];
      int ahead = 0;  // groups that come before this one: a larger best, or the same with a lower index
      for (int o = 0; o < groups; ++o) ahead += group_best[o] > mine || (group_best[o] == mine && o < g);
      if (ahead >= keep) c[u] = -INFINITY;
    }
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = experts;
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (c[u] > best) best = c[u], at = lane + kWave * u;
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (at == lane + kWave * u) w[u] = s[u], c[u] = -INFINITY;
  }
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    if (e < experts) gates[static_cast<size_t>(n) * experts + e] = w[u];
  }
}

// act[n, e ff + j] = gates[n, e] * silu(g) * u, g and u the columns e ff + j and width + e ff + j of the product
// (width = experts ff + shared_ff: the columns behind the routed experts' are a shared expert's, of a size of its own,
// whose weight is gates[n, shared_gate], or one if shared_gate < 0).
__device__ inline float expert_weight(const float* gates, int e, int experts, int shared_gate) {
  if (e < experts) return gates[e];
  return shared_gate >= 0 ? gates[shared_gate] : 1.f;
}

__global__ __launch_bounds__(256) void expert_glu_act_kernel(const void* __restrict__ gu, int gu_dt, int n_partials,
                                                             size_t partial_stride, const float* __restrict__ gates,
                                                             size_t gates_stride, void* __restrict__ out, int out_dt,
                                                             size_t total, int ff, int width, int experts,
                                                             int shared_gate) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / width;
  const int c = static_cast<int>(i % width);
  const float w = expert_weight(gates + n * gates_stride, c / ff, experts, shared_gate);
  float y = 0.f;
  if (w != 0.f) {
    float g = 0.f, u = 0.f;
    for (int p = 0; p < n_partials; ++p) {
      g += load_as_float(gu, gu_dt, p * partial_stride + n * 2 * width + c);
      u += load_as_float(gu, gu_dt, p * partial_stride + n * 2 * width + width + c);
    }
    y = w * (g / (1.f + expf(-g))) * u;
  }
  store_from_float(out, out_dt, i, y);
}

// Four columns a thread (the experts' size and the partial sums' stride are multiples of four).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void expert_glu_act_vec_kernel(const TI* __restrict__ gu, int n_partials, size_t partial_stride,
                                                                 const float* __restrict__ gates, size_t gates_stride,
                                                                 TO* __restrict__ out, size_t total4, int ff, int width,
                                                                 int experts, int shared_gate) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int per_row = width / 4;
  const size_t n = i / per_row;
  const int c = 4 * static_cast<int>(i % per_row);
  const float w = expert_weight(gates + n * gates_stride, c / ff, experts, shared_gate);
  float4 y = {0.f, 0.f, 0.f, 0.f};
  if (w != 0.f) {
    const float4 g = sum_partials4(gu + n * 2 * width + c, partial_stride, n_partials);
    const float4 u = sum_partials4(gu + n * 2 * width + width + c, partial_stride, n_partials);
    y = float4{w * (g.x / (1.f + expf(-g.x))) * u.x, w * (g.y / (1.f + expf(-g.y))) * u.y,
               w * (g.z / (1.f + expf(-g.z))) * u.z, w * (g.w / (1.f + expf(-g.w))) * u.w};
  }
  Vec4<TO>::store(out + n * width + c, y);
}

__global__ __launch_bounds__(256) void add_weighted_rows_kernel(float* __restrict__ p, const void* __restrict__ h, int h_dt,
                                                                size_t h_stride, const float* __restrict__ gates,
                                                                size_t gates_stride, int first, int count, size_t total,
                                                                int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / width;
  const int c = static_cast<int>(i % width);
  float w = 0.f;
  for (int e = 0; e < count; ++e) w += gates[n * gates_stride + first + e];
  if (w != 0.f) p[i] = fmaf(w, load_as_float(h, h_dt, n * h_stride + c), p[i]);
}

}  // namespace

extern "C" int pyre_route_topk(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                               float* gates, int n, int experts, int top, int softmax, int extra, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(z_dt) && n_partials >= 1 && (!bias || known_dtype(bias_dt)), "route_topk: bad dtypes");
  PYRE_REQUIRE(experts > 0 && experts <= kWave * kMaxPerLane && top > 0 && top <= experts && extra >= 0,
               "route_topk: %d of %d experts is not a choice this kernel makes", top, experts);
  if (n <= 0) return 0;
  hipLaunchKernelGGL(route_topk_kernel, dim3(n), dim3(kWave), 0, stream, z, z_dt, n_partials,
                     static_cast<size_t>(partial_stride), bias, bias_dt, gates, experts, top, softmax, extra);
  return check_launch("route_topk");
}

extern "C" int pyre_expert_act(const void* up, int up_dt, int n_partials, long partial_stride, const float* gates, void* out,
                               int out_dt, int n, int experts, int ff, int shared_ff, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(up_dt) && known_dtype(out_dt) && n_partials >= 1, "expert_act: bad dtypes");
  PYRE_REQUIRE(experts >= 0 && ff > 0 && shared_ff >= 0 && (gates || experts == 0), "expert_act: bad sizes");
  if (n <= 0) return 0;
  const int width = experts * ff + shared_ff;
  const size_t total = static_cast<size_t>(n) * width;
  if (ff % 4 == 0 && shared_ff % 4 == 0 && partial_stride % 4 == 0 && reinterpret_cast<uintptr_t>(up) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    PYRE_DISPATCH(up_dt, TI, PYRE_DISPATCH(out_dt, TO,
        hipLaunchKernelGGL((expert_act_vec_kernel<TI, TO>), dim3((total / 4 + 255) / 256), dim3(256), 0, stream,
                           static_cast<const TI*>(up), n_partials, static_cast<size_t>(partial_stride), gates,
                           static_cast<TO*>(out), total / 4, experts, ff, width)));
    return check_launch("expert_act");
  }
  hipLaunchKernelGGL(expert_act_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, up, up_dt, n_partials,
                     static_cast<size_t>(partial_stride), gates, out, out_dt, total, experts, ff, width);
  return check_launch("expert_act");
}

extern "C" int pyre_route_grouped(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                                  const float* correction, float* gates, int n, int experts, int top, int groups,
                                  int keep_groups, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(z_dt) && n_partials >= 1 && (!bias || known_dtype(bias_dt)), "route_grouped: bad dtypes");
  PYRE_REQUIRE(experts > 0 && experts <= kWave * kMaxPerLane && groups > 0 && experts % groups == 0 && keep_groups > 0 &&
                   keep_groups <= groups && top > 0 && top <= keep_groups * (experts / groups),
               "route_grouped: %d of %d experts in %d of %d groups is not a choice this kernel makes", top, experts,
               keep_groups, groups);
  if (n <= 0) return 0;
  hipLaunchKernelGGL(route_grouped_kernel, dim3(n), dim3(kWave), 0, stream, z, z_dt, n_partials,
                     static_cast<size_t>(partial_stride), bias, bias_dt, correction, gates, experts, top, groups, keep_groups);
  return check_launch("route_grouped");
}

extern "C" int pyre_expert_glu_act(const void* gu, int gu_dt, int n_partials, long partial_stride, const float* gates,
                                   long gates_stride, void* out, int out_dt, int n, int experts, int ff, int shared_ff,
                                   int shared_gate, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(gu_dt) && known_dtype(out_dt) && n_partials >= 1, "expert_glu_act: bad dtypes");
  PYRE_REQUIRE(experts > 0 && ff > 0 && shared_ff >= 0 && gates && gates_stride >= experts && shared_gate < gates_stride,
               "expert_glu_act: bad sizes");
  if (n <= 0) return 0;
  const int width = experts * ff + shared_ff;
  const size_t total = static_cast<size_t>(n) * width;
  if (ff % 4 == 0 && shared_ff % 4 == 0 && partial_stride % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    PYRE_DISPATCH(gu_dt, TI, PYRE_DISPATCH(out_dt, TO,
        hipLaunchKernelGGL((expert_glu_act_vec_kernel<TI, TO>), dim3((total / 4 + 255) / 256), dim3(256), 0, stream,
                           static_cast<const TI*>(gu), n_partials, static_cast<size_t>(partial_stride), gates,
                           static_cast<size_t>(gates_stride), static_cast<TO*>(out), total / 4, ff, width, experts, shared_gate)));
    return check_launch("expert_glu_act");
  }
  hipLaunchKernelGGL(expert_glu_act_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, gu, gu_dt, n_partials,
                     static_cast<size_t>(partial_stride), gates, static_cast<size_t>(gates_stride), out, out_dt, total, ff,
                     width, experts, shared_gate);
  return check_launch("expert_glu_act");
}

extern "C" int pyre_add_weighted_rows(float* p, const void* h, int h_dt, long h_stride, const float* gates,
                                      long gates_stride, int first, int count, int n, int width, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(h_dt) && p && h && gates, "add_weighted_rows: bad arguments");
  PYRE_REQUIRE(first >= 0 && count > 0 && width > 0 && gates_stride >= first + count, "add_weighted_rows: bad sizes");
  if (n <= 0) return 0;
  const size_t total = static_cast<size_t>(n) * width;
  hipLaunchKernelGGL(add_weighted_rows_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, p, h, h_dt,
                     static_cast<size_t>(h_stride), gates, static_cast<size_t>(gates_stride), first, count, total, width);
  return check_launch("add_weighted_rows");
}
