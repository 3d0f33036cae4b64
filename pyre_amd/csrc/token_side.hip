// A layer's input from the token itself: a slice of a second token table, gated by a narrow product of the stream.
//
//   out[n, j] = gelu_tanh(z[n, j]) * table[ids[n], first + j],   j < dim
//
// z is the product's partial sums (plus a bias if there is one); gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
// Float32 arithmetic; the result is rounded to the output's type.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

__global__ __launch_bounds__(256) void token_side_gate_kernel(const void* __restrict__ z, int z_dt, int n_partials,
                                                              size_t partial_stride, const void* __restrict__ bias,
                                                              int bias_dt, const void* __restrict__ table, int table_dt,
                                                              int table_width, int first, const int* __restrict__ ids,
                                                              void* __restrict__ out, int out_dt, size_t total, int dim) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / dim;
  const int j = static_cast<int>(i % dim);
  float v = 0.f;
  for (int p = 0; p < n_partials; ++p) v += load_as_float(z, z_dt, p * partial_stride + i);
  if (bias) v += load_as_float(bias, bias_dt, j);
  const float g = 0.5f * v * (1.f + tanhf(0.7978845608028654f * fmaf(0.044715f * v, v * v, v)));
  store_from_float(out, out_dt, i, g * load_as_float(table, table_dt, static_cast<size_t>(ids[n]) * table_width + first + j));
}

}  // namespace

extern "C" int pyre_token_side_gate(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias,
                                    int bias_dt, const void* table, int table_dt, int table_width, int first,
                                    const int* ids, void* out, int out_dt, int n, int dim, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(z_dt) && known_dtype(table_dt) && known_dtype(out_dt) && (!bias || known_dtype(bias_dt)) &&
                   n_partials >= 1, "token_side_gate: bad dtypes");
  PYRE_REQUIRE(dim > 0 && first >= 0 && first + dim <= table_width && table && ids && out,
               "token_side_gate: columns %d..%d lie outside the table's %d", first, first + dim, table_width);
  if (n <= 0) return 0;
  const size_t total = static_cast<size_t>(n) * dim;
  hipLaunchKernelGGL(token_side_gate_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, z, z_dt, n_partials,
                     static_cast<size_t>(partial_stride), bias, bias_dt, table, table_dt, table_width, first, ids, out,
                     out_dt, total, dim);
  return check_launch("token_side_gate");
}
