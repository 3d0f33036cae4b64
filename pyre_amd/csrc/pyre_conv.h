// A short causal convolution over time on the columns of a step's input product, for the kernels that finish such a
// product: what a column of a token is (the sum of the product's partial sums, plus a bias if there is one), what it is
// after the convolution, and the kernel that brings a request's state (its last taps - 1 projected rows) up to date.
#pragma once

#include "pyre_common.h"

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
