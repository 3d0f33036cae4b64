// The step between the input product and the attention kernels for an attention whose queries and keys are normed over
// their whole projection (all heads of a token at once) before they are turned by position:
//
//   u        = the product's columns of the token from col0 on (sum of its partial sums, plus the bias): nq query heads
//              of dk, then nkv key heads of dk and nkv value heads of dv (nkv = 0: a layer that reads another's keys
//              and values has queries alone)
//   q        = u_q / sqrt(mean(u_q^2 over all nq * dk columns) + eps) * q_gain     (q_gain over nq * dk; null: as it is)
//   k        = the same over the nkv * dk key columns with k_gain
//   q, k     = the first `rot` elements of every head turned by position, element e with e + rot / 2, by the tables
//              cos, sin [positions][rot / 2] (whatever frequencies and factor they were made with)
//
// Queries go to q_out [N, nq * dk], keys and values to their pages [pages][nkv][page][dk | dv] at `slots`.
// One block a token. The form for rows of up to 48 KB whose sizes are multiples of four (turned elements: of eight) sums
// the token's columns once into LDS, four to a thread with an element's partial sums asked for together, and norms,
// turns and stores from there, four elements a store. The general form makes a column's value again wherever it is
// needed (the rows are in the caches), so no size is bounded by what a block keeps. The two sums of squares are block
// sums whose order the thread layout fixes: a token's result depends on nothing but its own row, and which form runs
// on sizes and alignment alone. All arithmetic float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;

struct Product {
  const void* data;
  int dt, n_partials;
  size_t partial_stride;
  int ld, col0;
  const float* bias;  // over the product's columns, or null
};

__device__ inline float column(const Product& p, int n, int col) {
  const size_t at = static_cast<size_t>(n) * p.ld + p.col0 + col;
  float v = 0.f;
  for (int i = 0; i < p.n_partials; ++i) v += load_as_float(p.data, p.dt, i * p.partial_stride + at);
  return p.bias ? v + p.bias[p.col0 + col] : v;
}

template <typename TC>
__global__ __launch_bounds__(kThreads) void wide_norm_qkv_write_kernel(
    Product p, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps, const float* __restrict__ cos,
    const float* __restrict__ sin, int rot, const int* __restrict__ positions, void* __restrict__ q_out, int q_dt,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, const int* __restrict__ slots, int nq, int nkv, int dk, int dv,
    int page_size, int write_kv) {
  __shared__ float scratch[16];
  const int n = blockIdx.x, tid = threadIdx.x;
  const int qw = nq * dk, kw = nkv * dk;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const int half = rot / 2;
  const size_t trig = static_cast<size_t>(positions[n]) * half;

  float inv_q = 1.f, inv_k = 1.f;
  if (q_gain) {
    float ss = 0.f;
    for (int i = tid; i < qw; i += kThreads) {
      const float v = column(p, n, i);
      ss = fmaf(v, v, ss);
    }
    inv_q = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(qw) + eps);
  }
  if (k_gain && kw > 0 && slot >= 0) {
    float ss = 0.f;
    for (int i = tid; i < kw; i += kThreads) {
      const float v = column(p, n, qw + i);
      ss = fmaf(v, v, ss);
    }
    inv_k = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(kw) + eps);
  }

  // element i of the query (first = 0) or key (first = qw) columns, normed
  auto normed = [&](int first, int i, const float* gain, float inv) {
    const float v = column(p, n, first + i);
    return gain ? v * inv * gain[i] : v;
  };
  auto turned = [&](int first, int i, const float* gain, float inv) {
    const int e = i % dk;
    const float x = normed(first, i, gain, inv);
    if (e >= rot) return x;
    const bool lower = e < half;
    const int pair = lower ? e : e - half;
    const float other = normed(first, lower ? i + half : i - half, gain, inv);
    float a, b;
    if (lower) rotate_pair(x, other, cos[trig + pair], sin[trig + pair], a, b);
    else rotate_pair(other, x, cos[trig + pair], sin[trig + pair], a, b);
    return lower ? a : b;
  };
  for (int i = tid; i < qw; i += kThreads)
    store_from_float(q_out, q_dt, static_cast<size_t>(n) * qw + i, turned(0, i, q_gain, inv_q));
  if (slot < 0) return;
  for (int i = tid; i < kw; i += kThreads) {
    const int g = i / dk, e = i % dk;
    k_cache[((static_cast<size_t>(page) * nkv + g) * page_size + off) * dk + e] = from_float<TC>(turned(qw, i, k_gain, inv_k));
  }
  for (int i = tid; i < nkv * dv; i += kThreads) {
    const int g = i / dv, e = i % dv;
    v_cache[((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e] = from_float<TC>(column(p, n, qw + kw + i));
  }
}

template <typename TP, typename TC>
__global__ __launch_bounds__(kThreads) void wide_norm_qkv_write_row_kernel(
    Product p, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps, const float* __restrict__ cos,
    const float* __restrict__ sin, int rot, const int* __restrict__ positions, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, const int* __restrict__ slots, int nq, int nkv, int dk, int dv,
    int page_size, int write_kv) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float scratch[16];
  const int n = blockIdx.x, tid = threadIdx.x;
  const int qw = nq * dk, kw = nkv * dk, W = qw + kw + nkv * dv;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const int half = rot / 2;
  const size_t trig = static_cast<size_t>(positions[n]) * half;
  const TP* src = static_cast<const TP*>(p.data) + static_cast<size_t>(n) * p.ld + p.col0;
  for (int i = 4 * tid; i < W; i += 4 * kThreads) {
    float4 v = sum_partials4(src + i, p.partial_stride, p.n_partials);
    if (p.bias) v = add4(v, *reinterpret_cast<const float4*>(p.bias + p.col0 + i));
    *reinterpret_cast<float4*>(row + i) = v;
  }
  __syncthreads();
  auto inverse_rms = [&](int first, int width) {
    float ss = 0.f;
    for (int i = 4 * tid; i < width; i += 4 * kThreads) {
      const float4 v = *reinterpret_cast<const float4*>(row + first + i);
      ss = fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, fmaf(v.x, v.x, ss))));
    }
    return 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
  };
  const float inv_q = q_gain ? inverse_rms(0, qw) : 1.f;
  const float inv_k = k_gain && kw > 0 && slot >= 0 ? inverse_rms(qw, kw) : 1.f;
  auto normed = [&](int first, int i, const float* gain, float inv) {
    const float4 v = *reinterpret_cast<const float4*>(row + first + i);
    if (!gain) return v;
    const float4 g = *reinterpret_cast<const float4*>(gain + i);
    return float4{v.x * inv * g.x, v.y * inv * g.y, v.z * inv * g.z, v.w * inv * g.w};
  };
  // (the turned elements are a multiple of eight: four neighbours lie in one half, their partners likewise)
  auto turned = [&](int first, int i, const float* gain, float inv) {
    const int e = i % dk;
    const float4 x = normed(first, i, gain, inv);
    if (e >= rot) return x;
    const bool lower = e < half;
    const int pair = lower ? e : e - half;
    const float4 other = normed(first, lower ? i + half : i - half, gain, inv);
    const float4 c = *reinterpret_cast<const float4*>(cos + trig + pair), sn = *reinterpret_cast<const float4*>(sin + trig + pair);
    float4 a, b;
    if (lower) {
      rotate_pair(x.x, other.x, c.x, sn.x, a.x, b.x), rotate_pair(x.y, other.y, c.y, sn.y, a.y, b.y);
      rotate_pair(x.z, other.z, c.z, sn.z, a.z, b.z), rotate_pair(x.w, other.w, c.w, sn.w, a.w, b.w);
      return a;
    }
    rotate_pair(other.x, x.x, c.x, sn.x, a.x, b.x), rotate_pair(other.y, x.y, c.y, sn.y, a.y, b.y);
    rotate_pair(other.z, x.z, c.z, sn.z, a.z, b.z), rotate_pair(other.w, x.w, c.w, sn.w, a.w, b.w);
    return b;
  };
  for (int i = 4 * tid; i < qw; i += 4 * kThreads) Vec4<TC>::store(q_out + static_cast<size_t>(n) * qw + i, turned(0, i, q_gain, inv_q));
  if (slot < 0) return;
  for (int i = 4 * tid; i < kw; i += 4 * kThreads) {
    const int g = i / dk, e = i % dk;
    Vec4<TC>::store(k_cache + ((static_cast<size_t>(page) * nkv + g) * page_size + off) * dk + e, turned(qw, i, k_gain, inv_k));
  }
  for (int i = 4 * tid; i < nkv * dv; i += 4 * kThreads) {
    const int g = i / dv, e = i % dv;
    Vec4<TC>::store(v_cache + ((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e,
                    *reinterpret_cast<const float4*>(row + qw + kw + i));
  }
}

}  // namespace

extern "C" int pyre_wide_norm_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                        const float* bias, const float* q_gain, const float* k_gain, float eps,
                                        const float* cos, const float* sin, int rot, const int* positions, void* q_out,
                                        int q_dt, void* k_cache, void* v_cache, int cache_dt, const int* slots, int n,
                                        int nq, int nkv, int dk, int dv, int page_size, int write_kv, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(q_dt) && known_dtype(cache_dt) && n_partials >= 1, "wide_norm_qkv_write: bad dtypes");
  PYRE_REQUIRE(nq > 0 && nkv >= 0 && dk > 0 && dv > 0 && page_size > 0, "wide_norm_qkv_write: bad head geometry");
  PYRE_REQUIRE(!write_kv || (nkv > 0 && k_cache && v_cache && slots), "wide_norm_qkv_write: a cache write needs key heads, caches and slots");
  PYRE_REQUIRE((!q_gain && !k_gain) || eps > 0.f, "wide_norm_qkv_write: a norm needs a positive eps");
  PYRE_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || (cos && sin)),
               "wide_norm_qkv_write: %d turned elements of a head of %d need tables and an even number", rot, dk);
  PYRE_REQUIRE(positions && q_out, "wide_norm_qkv_write: positions and an output are needed");
  if (n <= 0) return 0;
  const Product p{proj, proj_dt, n_partials, static_cast<size_t>(partial_stride), ld, col0, bias};
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const size_t row_bytes = sizeof(float) * (static_cast<size_t>(nq + nkv) * dk + static_cast<size_t>(nkv) * dv);
  if (dk % 4 == 0 && dv % 4 == 0 && rot % 8 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 && q_dt == cache_dt &&
      row_bytes <= 48 * 1024 && a16(proj) && a16(bias) && a16(q_gain) && a16(k_gain) && a16(cos) && a16(sin) && a16(q_out) &&
      a16(k_cache) && a16(v_cache)) {
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL((wide_norm_qkv_write_row_kernel<TP, TC>), dim3(n), dim3(kThreads), row_bytes, stream, p, q_gain, k_gain,
                           eps, cos, sin, rot, positions, static_cast<TC*>(q_out), static_cast<TC*>(k_cache),
                           static_cast<TC*>(v_cache), slots, nq, nkv, dk, dv, page_size, write_kv)));
    return check_launch("wide_norm_qkv_write");
  }
  PYRE_DISPATCH(cache_dt, TC,
      hipLaunchKernelGGL(wide_norm_qkv_write_kernel<TC>, dim3(n), dim3(kThreads), 0, stream, p, q_gain, k_gain, eps, cos, sin,
                         rot, positions, q_out, q_dt, static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), slots, nq, nkv,
                         dk, dv, page_size, write_kv));
  return check_launch("wide_norm_qkv_write");
}
