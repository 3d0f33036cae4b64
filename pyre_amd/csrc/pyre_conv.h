// A short causal convolution over time on the columns of a step's input product, for the kernels that finish such a
// product: what a column of a token is (the sum of the product's partial sums, plus a bias if there is one), what it is
// after the convolution, and the kernel that brings a request's state (its last taps - 1 projected rows) up to date.
#pragma once

#include "pyre_common.h"
#include "pyre_vec4.h"

namespace pyre {

constexpr int kConvThreads = 256;

struct ConvIn {
  const void* proj;
  int proj_dt, n_partials;
  size_t partial_stride;
  int ld, col0;
  const float* taps_w;   // [taps][channels] or null
  int taps;
  const float* state;    // [slots][taps - 1][channels] or null
  int channels;
  const float* bias = nullptr;  // over the product's columns (col0 is column 0 of its own), or null
};

// Column `col` of the step's row `n` of the product.
__device__ inline float product_value(const ConvIn& in, int n, int col) {
  const size_t at = static_cast<size_t>(n) * in.ld + in.col0 + col;
  float v = 0.f;
  for (int p = 0; p < in.n_partials; ++p) v += load_as_float(in.proj, in.proj_dt, p * in.partial_stride + at);
  return in.bias ? v + in.bias[in.col0 + col] : v;
}

// Channel `ch` of token n after the convolution; `run` is the token's index among its request's tokens of the step.
__device__ inline float conv_value(const ConvIn& in, int n, int run, int slot, int ch) {
  if (!in.taps_w) return product_value(in, n, ch);
  float y = 0.f;
  for (int j = 0; j < in.taps; ++j) {
    const int back = in.taps - 1 - j;  // this tap's input lies `back` tokens before n
    float u;
    if (run - back >= 0) u = product_value(in, n - back, ch);
    else u = in.state[(static_cast<size_t>(slot) * (in.taps - 1) + (in.taps - 1 + run - back)) * in.channels + ch];
    y = fmaf(in.taps_w[static_cast<size_t>(j) * in.channels + ch], u, y);
  }
  return y;
}

// Four neighbouring channels at a time (the product's width, first column and stride, the channels and `ch` are multiples
// of four, the pointers on 16 bytes): every tap's input asked for before the first is used; the same sums in the same
// order as conv_value.
constexpr int kConvVecTaps = 8;  // the most taps of this form
template <typename TP>
__device__ inline float4 conv_value4(const ConvIn& in, const TP* proj, int n, int run, int slot, int ch) {
  const TP* row = proj + static_cast<size_t>(n) * in.ld + in.col0 + ch;
  const float4 b = in.bias ? *reinterpret_cast<const float4*>(in.bias + in.col0 + ch) : float4{0.f, 0.f, 0.f, 0.f};
  if (!in.taps_w) return in.bias ? add4(sum_partials4(row, in.partial_stride, in.n_partials), b) : sum_partials4(row, in.partial_stride, in.n_partials);
  float4 u[kConvVecTaps];
#pragma unroll
  for (int j = 0; j < kConvVecTaps; ++j) {  // every tap's input asked for before the first is used
    if (j >= in.taps) break;
    const int back = in.taps - 1 - j;
    if (run - back >= 0) {
      u[j] = sum_partials4(row - static_cast<size_t>(back) * in.ld, in.partial_stride, in.n_partials);
      if (in.bias) u[j] = add4(u[j], b);
    } else u[j] = *reinterpret_cast<const float4*>(in.state + (static_cast<size_t>(slot) * (in.taps - 1) + (in.taps - 1 + run - back)) * in.channels + ch);
  }
  float4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < kConvVecTaps; ++j) {
    if (j >= in.taps) break;
    const float4 w = *reinterpret_cast<const float4*>(in.taps_w + static_cast<size_t>(j) * in.channels + ch);
    y = float4{fmaf(w.x, u[j].x, y.x), fmaf(w.y, u[j].y, y.y), fmaf(w.z, u[j].z, y.z), fmaf(w.w, u[j].w, y.w)};
  }
  return y;
}

// A thread a channel, the rows of the new state in ascending order: row i takes the step's row len - (T - 1) + i of the
// request or, where the step is shorter than that, the old state's row i + len, which lies further on and is still old.
static __global__ __launch_bounds__(kConvThreads) void conv_state_update_kernel(ConvIn in, float* __restrict__ state,
                                                                     const int* __restrict__ state_slots,
                                                                     const int* __restrict__ q_start) {
  const int s = blockIdx.x, first = q_start[s], len = q_start[s + 1] - first, keep = in.taps - 1;
  float* st = state + static_cast<size_t>(state_slots[s]) * keep * in.channels;
  for (int ch = blockIdx.y * kConvThreads + threadIdx.x; ch < in.channels; ch += gridDim.y * kConvThreads)
    for (int i = 0; i < keep; ++i) {
      const int r = len - keep + i;
      st[static_cast<size_t>(i) * in.channels + ch] = r >= 0 ? product_value(in, first + r, ch)
                                                              : st[static_cast<size_t>(i + len) * in.channels + ch];
    }
}


}  // namespace pyre
