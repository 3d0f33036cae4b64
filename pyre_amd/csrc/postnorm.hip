// The residual sum of blocks that norm what a sublayer returns and not what it reads, with RMS norms:
//
//   t_i    = sum of the partial sums of pending term i                          (i = 0, 1; the second may be absent)
//   u_i    = term i has a gain ? scale_i * RMS(t_i; inner_eps) * gain_i : scale_i * t_i
//   y      = u_0 + u_1;   y <- outer gain ? RMS(y; outer_eps) * outer_gain : y
//   resid += y
//   out    = out gain ? RMS(resid; out_eps) * out_gain : resid                    (rounded to out's element type)
//   RMS(x; e) = x / sqrt(mean(x^2) + e)
//
// One block per row; a thread keeps its elements of both terms in registers, so every row is read once.
// A row's sums of squares are block sums of per-thread sums, in an order that the row's width fixes.
// With `rows` only the listed rows are handled, into out[0 .. n), and resid is left as it was.
// All arithmetic float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;

struct Term {
  const void* data;
  int dt, n_partials;
  size_t stride;
  const void* gain;
  int gain_dt;
  float scale;
};

template <int ITEMS>
__global__ __launch_bounds__(kThreads) void add_rms_terms_kernel(
    float* __restrict__ resid, Term a, Term b, float inner_eps, const void* __restrict__ outer_gain, int outer_dt,
    float outer_eps, const void* __restrict__ out_gain, int out_gain_dt, float out_eps, void* __restrict__ out, int out_dt,
    const int* __restrict__ rows, int hidden) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out, tid = threadIdx.x;
  const size_t row = static_cast<size_t>(r_in) * hidden;
  const float inv_n = 1.f / static_cast<float>(hidden);
  float y[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) y[k] = 0.f;

  auto inv_rms = [&](const float (&v)[ITEMS], float e) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (tid + k * kThreads < hidden) ss += v[k] * v[k];
    return 1.f / sqrtf(block_sum(ss, scratch) * inv_n + e);
  };
  auto take = [&](const Term& t) {
    float v[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      float d = 0.f;
      if (i < hidden)
        for (int p = 0; p < t.n_partials; ++p) d += load_as_float(t.data, t.dt, p * t.stride + row + i);
      v[k] = d;
    }
    const float f = t.gain ? inv_rms(v, inner_eps) * t.scale : t.scale;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      if (i < hidden) y[k] += t.gain ? v[k] * f * load_as_float(t.gain, t.gain_dt, i) : v[k] * f;
    }
  };
  if (a.data) take(a);
  if (b.data) take(b);
  if (outer_gain) {
    const float f = inv_rms(y, outer_eps);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      if (i < hidden) y[k] = y[k] * f * load_as_float(outer_gain, outer_dt, i);
    }
  }
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = tid + k * kThreads;
    if (i < hidden) {
      y[k] += resid[row + i];
      if (!rows && a.data) resid[row + i] = y[k];
    } else {
      y[k] = 0.f;
    }
  }
  if (!out) return;
  const float f = out_gain ? inv_rms(y, out_eps) : 1.f;
  const size_t orow = static_cast<size_t>(r_out) * hidden;
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = tid + k * kThreads;
    if (i < hidden) store_from_float(out, out_dt, orow + i, out_gain ? y[k] * f * load_as_float(out_gain, out_gain_dt, i) : y[k]);
  }
}

// The same with four elements to a load: the row's width and the partial sums' strides are multiples of four, all
// gains share one element type, every pointer lies on 16 bytes. THREADS x ITEMS float4 hold a row.
template <typename TA, typename TG, typename TO, int THREADS, int ITEMS>
__global__ __launch_bounds__(THREADS) void add_rms_terms_vec_kernel(
    float* __restrict__ resid, Term a, Term b, float inner_eps, const TG* __restrict__ outer_gain, float outer_eps,
    const TG* __restrict__ out_gain, float out_eps, TO* __restrict__ out, const int* __restrict__ rows, int hidden) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out, tid = threadIdx.x;
  const size_t row = static_cast<size_t>(r_in) * hidden;
  const float inv_n = 1.f / static_cast<float>(hidden);
  float4 y[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) y[k] = float4{0.f, 0.f, 0.f, 0.f};

  auto inv_rms = [&](const float4 (&v)[ITEMS], float e) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (4 * (tid + k * THREADS) < hidden) ss += (v[k].x * v[k].x + v[k].y * v[k].y) + (v[k].z * v[k].z + v[k].w * v[k].w);
    return 1.f / sqrtf(block_sum(ss, scratch) * inv_n + e);
  };
  auto take = [&](const Term& t) {
    float4 v[ITEMS];
    const TA* src = static_cast<const TA*>(t.data) + row;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      v[k] = i < hidden ? sum_partials4(src + i, t.stride, t.n_partials) : float4{0.f, 0.f, 0.f, 0.f};
    }
    const float f = t.gain ? inv_rms(v, inner_eps) * t.scale : t.scale;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      if (i >= hidden) continue;
      float4 g = {1.f, 1.f, 1.f, 1.f};
      if (t.gain) g = Vec4<TG>::load(static_cast<const TG*>(t.gain) + i);
      y[k] = float4{y[k].x + v[k].x * f * g.x, y[k].y + v[k].y * f * g.y, y[k].z + v[k].z * f * g.z, y[k].w + v[k].w * f * g.w};
    }
  };
  if (a.data) take(a);
  if (b.data) take(b);
  if (outer_gain) {
    const float f = inv_rms(y, outer_eps);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      if (i >= hidden) continue;
      const float4 g = Vec4<TG>::load(outer_gain + i);
      y[k] = float4{y[k].x * f * g.x, y[k].y * f * g.y, y[k].z * f * g.z, y[k].w * f * g.w};
    }
  }
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = 4 * (tid + k * THREADS);
    if (i < hidden) {
      y[k] = add4(y[k], Vec4<float>::load(resid + row + i));
      if (!rows && a.data) Vec4<float>::store(resid + row + i, y[k]);
    }
  }
  if (!out) return;
  const float f = out_gain ? inv_rms(y, out_eps) : 1.f;
  const size_t orow = static_cast<size_t>(r_out) * hidden;
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = 4 * (tid + k * THREADS);
    if (i >= hidden) continue;
    float4 g = {1.f, 1.f, 1.f, 1.f};
    if (out_gain) g = Vec4<TG>::load(out_gain + i);
    Vec4<TO>::store(out + orow + i, float4{y[k].x * f * g.x, y[k].y * f * g.y, y[k].z * f * g.z, y[k].w * f * g.w});
  }
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

}  // namespace

extern "C" int pyre_add_rms_terms(float* resid, const void* a, int a_dt, int a_partials, long a_stride, const void* a_gain,
                                  int a_gain_dt, float a_scale, const void* b, int b_dt, int b_partials, long b_stride,
                                  const void* b_gain, int b_gain_dt, float b_scale, float inner_eps,
                                  const void* outer_gain, int outer_dt, float outer_eps, const void* out_gain,
                                  int out_gain_dt, float out_eps, void* out, int out_dt, const int* rows, int n, int hidden,
                                  hipStream_t stream) {
  PYRE_REQUIRE(!a || (known_dtype(a_dt) && a_partials >= 1), "add_rms_terms: bad first term");
  PYRE_REQUIRE(!b || (a && known_dtype(b_dt) && b_partials >= 1), "add_rms_terms: a second term without a first, or a bad one");
  PYRE_REQUIRE((!a_gain || (a && known_dtype(a_gain_dt))) && (!b_gain || (b && known_dtype(b_gain_dt))),
               "add_rms_terms: a term's gain without the term");
  PYRE_REQUIRE(!(a_gain || b_gain) || inner_eps > 0.f, "add_rms_terms: the terms' own norm needs a positive eps");
  PYRE_REQUIRE(!outer_gain || (a && known_dtype(outer_dt) && outer_eps > 0.f), "add_rms_terms: a norm of the sum needs a term and a positive eps");
  PYRE_REQUIRE(!out_gain || (out && known_dtype(out_gain_dt) && out_eps > 0.f), "add_rms_terms: bad output norm");
  PYRE_REQUIRE(!out || known_dtype(out_dt), "add_rms_terms: unknown output dtype");
  PYRE_REQUIRE(n >= 0 && hidden > 0 && hidden <= 64 * kThreads, "add_rms_terms: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0) return 0;
  const Term ta{a, a_dt, a_partials, static_cast<size_t>(a_stride), a_gain, a_gain_dt, a_scale};
  const Term tb{b, b_dt, b_partials, static_cast<size_t>(b_stride), b_gain, b_gain_dt, b_scale};
  // one element type among the gains that are there, and among the terms
  const void* gains[4] = {a_gain, b_gain, outer_gain, out_gain};
  const int gain_dts[4] = {a_gain_dt, b_gain_dt, outer_dt, out_gain_dt};
  int gdt = -1;
  bool one_gain_type = true;
  for (int i = 0; i < 4; ++i)
    if (gains[i]) {
      if (gdt < 0) gdt = gain_dts[i];
      one_gain_type = one_gain_type && gain_dts[i] == gdt;
    }
  if (gdt < 0) gdt = kF32;
  const bool vec = hidden % 4 == 0 && hidden <= 4 * 256 * 16 && one_gain_type && (!a || a_stride % 4 == 0) &&
                   (!b || (b_stride % 4 == 0 && b_dt == a_dt)) && aligned16(a) && aligned16(b) && aligned16(a_gain) &&
                   aligned16(b_gain) && aligned16(outer_gain) && aligned16(out_gain) && aligned16(out) && aligned16(resid);
  if (vec) {
    const int quads = hidden / 4;
    const bool few = n <= 128 && quads > 256;  // a decode step: spread each row over more threads
#define PYRE_RTV(THREADS, ITEMS)                                                                                          \
  hipLaunchKernelGGL((add_rms_terms_vec_kernel<TA, TG, TO, THREADS, ITEMS>), dim3(n), dim3(THREADS), 0, stream, resid, ta, \
                     tb, inner_eps, static_cast<const TG*>(outer_gain), outer_eps, static_cast<const TG*>(out_gain),      \
                     out_eps, static_cast<TO*>(out), rows, hidden)
    PYRE_DISPATCH(a ? a_dt : kF32, TA, PYRE_DISPATCH(gdt, TG, PYRE_DISPATCH(out ? out_dt : kF32, TO, {
      if (few && quads <= 1024) PYRE_RTV(1024, 1);
      else if (few) PYRE_RTV(1024, 4);
      else if (quads <= 256) PYRE_RTV(256, 1);
      else if (quads <= 1024) PYRE_RTV(256, 4);
      else PYRE_RTV(256, 16);
    })));
#undef PYRE_RTV
    return check_launch("add_rms_terms");
  }
#define PYRE_RT(ITEMS)                                                                                                  \
  hipLaunchKernelGGL(add_rms_terms_kernel<ITEMS>, dim3(n), dim3(kThreads), 0, stream, resid, ta, tb, inner_eps, outer_gain, \
                     outer_dt, outer_eps, out_gain, out_gain_dt, out_eps, out, out_dt, rows, hidden)
  if (hidden <= 4 * kThreads) PYRE_RT(4);
  else if (hidden <= 16 * kThreads) PYRE_RT(16);
  else PYRE_RT(64);
#undef PYRE_RT
  return check_launch("add_rms_terms");
}
