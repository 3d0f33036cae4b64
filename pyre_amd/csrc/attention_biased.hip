// Softmax attention without rotation whose positions enter through the scores: unit-norm
// queries and keys, a cap on the scores, a learned bias by distance, a window that also keeps
// the first tokens of the sequence, key and value heads of different sizes, and one gate per
// head on the output. Three kernels over the paged cache k [pages, nkv, page, dk] and
// v [pages, nkv, page, dv] (both one record per token), float32 or bfloat16 storage, all
// arithmetic float32:
//
//   s(i, j) = (q_i . k_j) * scale;   s <- cap * tanh(s / cap)  (cap > 0);   s <- s + bias[head][min(i - j, far)]
//   i sees j  iff  j <= i and (window == 0 or i - j < window or j < keep_first)
//                 and (chunk == 0 or i / chunk == j / chunk)      (chunks of positions counted from 0)
//   out_i = gate_i * out_scale * sum_j softmax_j(s(i, .)) v_j
//
// `bias` is the table by distance that the host made of the model's buckets: [nq][far + 1] float32,
// or null. `gate` is float32 [n][nq] (already squashed; gate_dim = 1) or [n][nq * dv] (a gate per element of the
// output; gate_dim = dv), or null. `sink` is float32 [nq] or null: exp(sink[head]) joins the softmax's denominator,
// a key that has no value (it is neither scaled nor capped nor biased).
//
// unit_qkv_write  finishes the input product of a step (partial sums), divides every query and key
//                 head by its root mean square, stores queries, keys and values and the squashed gates.
// attn_biased_tile    prompt portions: tiles of up to 32 consecutive tokens of a request, four query
//                 heads of a key/value head per block, chunks of 32 keys through LDS, both products on
//                 the matrix cores' float32 instruction (scores and weights stay float32).
// attn_biased_single  single tokens: a block per (token, up to eight query heads of a key/value head), the keys in
//                 spans of 128 that the block's heads read together.
//
// Chunks start at multiples of 32 keys and spans at the token's first visible key, so the order of
// every sum of a token depends on its own bounds alone.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------------
template <typename TC>
__global__ __launch_bounds__(kThreads) void unit_qkv_write_kernel(
    const void* __restrict__ proj, int proj_dt, int n_partials, size_t partial_stride, int ld, int col0,
    void* __restrict__ q_out, int q_dt, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    float* __restrict__ gate_out, const int* __restrict__ slots, int nq, int nkv, int dk, int dv, int page_size,
    int unit_norm, float eps, int gated, int write_kv) {
  const int n = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const size_t in_row = static_cast<size_t>(n) * ld + col0;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

  auto value = [&](int col) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_float(proj, proj_dt, p * partial_stride + in_row + col);
    return v;
  };

  // query heads 0..nq-1, then key heads: one wave a head, four elements a lane (dk <= 256)
  for (int head = wave; head < nq + nkv; head += kThreads / kWave) {
    float x[4], ss = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = lane + 64 * u;
      x[u] = e < dk ? value(head * dk + e) : 0.f;
      ss += x[u] * x[u];
    }
    float inv = 1.f;
    if (unit_norm) inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = lane + 64 * u;
      if (e >= dk) continue;
      if (head < nq) {
        store_from_float(q_out, q_dt, (static_cast<size_t>(n) * nq + head) * dk + e, x[u] * inv);
      } else if (slot >= 0) {
        k_cache[((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * dk + e] = from_float<TC>(x[u] * inv);
      }
    }
  }
  const int v0 = (nq + nkv) * dk;
  if (slot >= 0)
    for (int i = tid; i < nkv * dv; i += kThreads) {
      const int g = i / dv, e = i % dv;
      v_cache[((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e] = from_float<TC>(value(v0 + i));
    }
  if (gated)
    for (int h = tid; h < nq; h += kThreads) gate_out[static_cast<size_t>(n) * nq + h] = 1.f / (1.f + expf(-value(v0 + nkv * dv + h)));
}

// The same with four elements to a load and an element's partial sums asked for together (head sizes,
// the product's width, first column and stride are multiples of four; queries stored as the cache's type).
template <typename TP, typename TC>
__global__ __launch_bounds__(kThreads) void unit_qkv_write_vec_kernel(
    const TP* __restrict__ proj, int n_partials, size_t partial_stride, int ld, int col0, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, float* __restrict__ gate_out, const int* __restrict__ slots,
    int nq, int nkv, int dk, int dv, int page_size, int unit_norm, float eps, int gated, int write_kv) {
  const int n = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const TP* in = proj + static_cast<size_t>(n) * ld + col0;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  for (int head = wave; head < nq + nkv; head += kThreads / kWave) {  // a wave a head, four elements a lane
    const int e = 4 * lane;
    float4 x = {0.f, 0.f, 0.f, 0.f};
    if (e < dk) x = sum_partials4(in + head * dk + e, partial_stride, n_partials);
    float inv = 1.f;
    if (unit_norm) inv = 1.f / sqrtf(wave_sum((x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w)) / static_cast<float>(dk) + eps);
    if (e >= dk) continue;
    const float4 y = {x.x * inv, x.y * inv, x.z * inv, x.w * inv};
    if (head < nq) Vec4<TC>::store(q_out + (static_cast<size_t>(n) * nq + head) * dk + e, y);
    else if (slot >= 0) Vec4<TC>::store(k_cache + ((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * dk + e, y);
  }
  const int v0 = (nq + nkv) * dk;
  if (slot >= 0)
    for (int i = 4 * tid; i < nkv * dv; i += 4 * kThreads) {
      const int g = i / dv, e = i % dv;
      Vec4<TC>::store(v_cache + ((static_cast<size_t>(page) * nkv + g) * page_size + off) * dv + e,
                      sum_partials4(in + v0 + i, partial_stride, n_partials));
    }
  if (gated)
    for (int h = tid; h < nq; h += kThreads) {
      float v = 0.f;
      for (int p = 0; p < n_partials; ++p) v += to_float(in[p * partial_stride + v0 + nkv * dv + h]);
      gate_out[static_cast<size_t>(n) * nq + h] = 1.f / (1.f + expf(-v));
    }
}

// ---------------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(16))) float f32x16;
constexpr int kKeys = 32;
constexpr int kTileMaxKeyHead = 128;  // the queries of a block's four heads lie in LDS
constexpr int kVtLd = kKeys + 4;      // a row of transposed values: 16-byte reads of four keys
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Eight consecutive elements as floats in one or two 16-byte loads; p is aligned to 16 bytes.
__device__ inline void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}
__device__ inline void load8(const bf16* p, float (&v)[8]) {
  const uint4 r = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    v[2 * u] = __uint_as_float(w[u] << 16);
    v[2 * u + 1] = __uint_as_float(w[u] & 0xffff0000u);
  }
}

// tanh(x) = sign(x) (1 - e) / (1 + e) with e = exp(-2 |x|) <= 1: one exponential and one division, no
// branches; its absolute error is a few 1e-8 everywhere (the library's branches cost a tile of scores
// more than both of its matrix products).
__device__ inline float tanh_by_exp(float x) {
  const float e = expf(-2.f * fabsf(x));
  return copysignf((1.f - e) / (1.f + e), x);
}

// The first key that a query at `pos` sees, the kept first tokens aside.
__device__ inline int first_seen(int pos, int window, int chunk) {
  int lo = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) lo = max(lo, pos - pos % chunk);
  return lo;
}

// The softmax's last factor with a sink in the denominator: the output sums were made against the maximum m and the
// sum l; with M = max(m, sink) they are worth e^(m - M) / (l e^(m - M) + e^(sink - M)).
__device__ inline float softmax_factor(float m, float l, const float* sink, int head) {
  if (!sink) return l > 0.f ? 1.f / l : 0.f;
  const float sk = sink[head], M = fmaxf(m, sk);
  const float a = m == -INFINITY ? 0.f : expf(m - M);
  return a / (l * a + expf(sk - M));
}

__device__ inline float shaped_score(float raw, float scale, float cap, const float* bias_row, int dist, int far) {
  float s = raw * scale;
  if (cap > 0.f) s = cap * tanh_by_exp(s / cap);
  if (bias_row) s += bias_row[min(dist, far)];
  return s;
}

// NV: the value head's size in tiles of 32 (the rest of the last tile is zeros); the key head's
// size is a run-time number of up to 128, padded to a multiple of 32 in LDS. Layout as in attention_f32_mfma.hip:
// the transposed problem, S^T[key, token] and O^T[d, token], so that a lane's sixteen scores are
// the operands of the second product as they are.
// VEC: both head sizes are multiples of eight and the caches start on 16 bytes, so that keys and
// values come eight elements to a load.
template <typename T, int NV, bool VEC>
__global__ __launch_bounds__(kThreads) void attn_biased_tile_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    int out_ld, const float* __restrict__ gate, float out_scale, const int* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, int nq, int nkv, int dk, int dkp, int dv, int page_size, float scale, float cap,
    const float* __restrict__ bias, int far, int window, int keep_first, int chunk, int tab_lds, int bias_lds,
    const float* __restrict__ sink, int gate_dim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // rows of keys and queries hold the even elements first, then the odd ones: a lane's operands of four
  // steps of the first product are then one 16-byte read
  float* Ks = lds;                              // [kKeys][dkp + 4]
  float* Qs = Ks + kKeys * (dkp + 4);           // [4 waves][32 tokens][dkp + 4]
  float* Vt = Qs + 4 * 32 * (dkp + 4);          // [32 NV][kVtLd]
  int* tab_s = reinterpret_cast<int*>(Vt + 32 * NV * kVtLd);  // [tab_lds]: the request's block table, if it fits
  float* bias_s = reinterpret_cast<float*>(tab_s + tab_lds);  // [4][far + 1]: the four heads' biases, if they fit
  __shared__ int page_s[2][kKeys];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int n_rep = nq / nkv, hgroups = (n_rep + 3) / 4;
  const int kvh = blockIdx.y / hgroups, hin = (blockIdx.y % hgroups) * 4 + wave;
  const bool active = hin < n_rep;  // a wave without a head still helps loading
  const int head = kvh * n_rep + (active ? hin : 0);
  const int t0 = tiles[2 * blockIdx.x], ntok = tiles[2 * blockIdx.x + 1];
  if (ntok <= 0) return;
  const int pos0 = positions[t0];
  const int* table = block_table + static_cast<size_t>(seq_of_token[t0]) * table_stride;
  const int ldk = dkp + 4, half = dkp / 2;

  const bool live = active && c < ntok;
  const int hi = c < ntok ? pos0 + c : pos0;
  const int lo = first_seen(hi, window, chunk);
  const int keep = window > 0 ? keep_first : 0;
  const float* bias_row = bias ? bias + static_cast<size_t>(head) * (far + 1) : nullptr;
  for (int i = tid; i < tab_lds; i += kThreads) tab_s[i] = table[i];
  if (bias && bias_lds) {  // from here on the biases are read from LDS: no load that a wait for them would queue behind
    for (int i = lane; i <= far; i += 64) bias_s[wave * (far + 1) + i] = bias_row[i];
    bias_row = bias_s + wave * (far + 1);
  }
  {  // this wave's queries: Qs[wave][token][d], zeros where there is no token or no element
    float* mine = Qs + wave * 32 * ldk;
    if (VEC) {
      for (int i = lane; i < 32 * (dkp / 8); i += 64) {
        const int t = i / (dkp / 8), d = 8 * (i % (dkp / 8));
        float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (active && t < ntok && d < dk) load8(q + (static_cast<size_t>(t0 + t) * nq + head) * dk + d, v);
#pragma unroll
        for (int u = 0; u < 8; ++u) mine[t * ldk + (u & 1) * half + ((d + u) >> 1)] = v[u];
      }
    } else {
      for (int i = lane; i < 32 * dkp; i += 64) {
        const int t = i / dkp, d = i % dkp;
        mine[t * ldk + (d & 1) * half + (d >> 1)] = active && t < ntok && d < dk ? to_float(q[(static_cast<size_t>(t0 + t) * nq + head) * dk + d]) : 0.f;
      }
    }
  }
  const float* myq = Qs + wave * 32 * ldk + c * ldk + h * half;
  f32x16 o[NV];
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // the chunks that hold the kept first tokens which the window has passed, then the window's
  const int lo_all = first_seen(pos0, window, chunk);  // rises with the position: the tile's first token sees furthest back
  const int hi_all = pos0 + ntok - 1;
  const int kept_end = min(keep, lo_all);                        // keys 0 .. kept_end - 1 lie before every window
  const int n_first = kept_end > 0 ? (kept_end - 1) / kKeys + 1 : 0;
  const int chunk_b = max(lo_all / kKeys, n_first);
  const int n_chunks = n_first + (hi_all / kKeys - chunk_b + 1);
  // VEC: the next chunk's keys and values are asked for (into registers) before the current chunk is
  // multiplied, and go to LDS when every wave is done with it
  constexpr int KI = kKeys * (kTileMaxKeyHead / 8) / kThreads, VI = (kKeys * 4 * NV + kThreads - 1) / kThreads;
  float kreg[KI][8], vreg[VI][8];
  auto chunk_key0 = [&](int it) { return (it < n_first ? it : chunk_b + (it - n_first)) * kKeys; };
  auto page_of = [&](int key) {
    const int entry = key / page_size;
    if (key > hi_all || entry >= table_stride) return -1;
    return entry < tab_lds ? tab_s[entry] : table[entry];
  };
  auto ask = [&](int it) {
    const int key0 = chunk_key0(it), kg = dkp / 8;
    if (tid < kKeys) page_s[it & 1][tid] = page_of(key0 + tid);
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      const int i = tid + k * kThreads, key = key0 + i / kg, d = 8 * (i % kg);
      const int page = i < kKeys * kg ? page_of(key) : -1;
#pragma unroll
      for (int u = 0; u < 8; ++u) kreg[k][u] = 0.f;
      if (page >= 0 && d < dk) load8(k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + key % page_size) * dk + d, kreg[k]);
    }
#pragma unroll
    for (int k = 0; k < VI; ++k) {
      const int i = tid + k * kThreads, key = key0 + i / (4 * NV), d = 8 * (i % (4 * NV));
      const int page = i < kKeys * 4 * NV ? page_of(key) : -1;
#pragma unroll
      for (int u = 0; u < 8; ++u) vreg[k][u] = 0.f;
      if (page >= 0 && d < dv) load8(v_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + key % page_size) * dv + d, vreg[k]);
    }
  };
  auto stash = [&]() {
    const int kg = dkp / 8;
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      const int i = tid + k * kThreads, key = i / kg, d = 8 * (i % kg);
      if (i < kKeys * kg)
#pragma unroll
        for (int u = 0; u < 8; ++u) Ks[key * ldk + (u & 1) * half + ((d + u) >> 1)] = kreg[k][u];
    }
#pragma unroll
    for (int k = 0; k < VI; ++k) {
      const int i = tid + k * kThreads, key = i / (4 * NV), d = 8 * (i % (4 * NV));
      if (i < kKeys * 4 * NV)
#pragma unroll
        for (int u = 0; u < 8; ++u) Vt[(d + u) * kVtLd + key] = vreg[k][u];
    }
  };
  __syncthreads();  // the table and the biases are in LDS
  if (VEC) ask(0);
  for (int it = 0; it < n_chunks; ++it) {
    const int key0 = chunk_key0(it);
    const int* pages = page_s[it & 1];
    __syncthreads();  // the previous chunk has been read by every wave (and the queries are written)
    if (VEC) {
      stash();
    } else {
      if (tid < kKeys) page_s[it & 1][tid] = page_of(key0 + tid);
      __syncthreads();
      for (int i = tid; i < kKeys * dkp; i += kThreads) {
        const int key = i / dkp, d = i % dkp, page = pages[key];
        float v = 0.f;
        if (page >= 0 && d < dk)
          v = to_float(k_cache[((static_cast<size_t>(page) * nkv + kvh) * page_size + (key0 + key) % page_size) * dk + d]);
        Ks[key * ldk + (d & 1) * half + (d >> 1)] = v;
      }
      for (int i = tid; i < kKeys * 32 * NV; i += kThreads) {
        const int key = i / (32 * NV), d = i % (32 * NV), page = pages[key];
        float v = 0.f;
        if (page >= 0 && d < dv)
          v = to_float(v_cache[((static_cast<size_t>(page) * nkv + kvh) * page_size + (key0 + key) % page_size) * dv + d]);
        Vt[d * kVtLd + key] = v;
      }
    }
    __syncthreads();
    if (VEC && it + 1 < n_chunks) ask(it + 1);
    if (!active) continue;

    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    const float* krow = Ks + c * ldk + h * half;
#pragma unroll 4
    for (int st = 0; st < half; st += 4) {  // elements 2 st + h, ..., 2 (st + 3) + h of the key and the query
      const f32x4 k4 = *reinterpret_cast<const f32x4*>(krow + st), q4 = *reinterpret_cast<const f32x4*>(myq + st);
#pragma unroll
      for (int u = 0; u < 4; ++u) s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[u], q4[u], s, 0, 0, 0);
    }

    // element i of s: key key0 + 8 (i / 4) + 4 h + i % 4, token c
    // the biases of the lane's sixteen distances, asked for together (a key that is not seen reads a distance that is there)
    float bv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = key0 + 8 * (i >> 2) + 4 * h + (i & 3);
      bv[i] = bias_row ? bias_row[min(max(hi - key, 0), far)] : 0.f;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kk = 8 * (i >> 2) + 4 * h + (i & 3), key = key0 + kk;
      const bool seen = key <= hi && (key >= lo || key < keep) && pages[kk] >= 0;
      const float shaped = shaped_score(s[i], scale, cap, nullptr, 0, 0) + bv[i];
      s[i] = seen ? shaped : -INFINITY;
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = expf(m - m_use);
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = expf(s[i] - m_use);
      sum += s[i];
    }
    l = l * alpha + sum;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(&Vt[(32 * dt + c) * kVtLd + 8 * a + 4 * h]);
#pragma unroll
        for (int u = 0; u < 4; ++u) o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(v4[u], s[4 * a + u], o[dt], 0, 0, 0);
      }
  }

  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  if (!live) return;
  float f = softmax_factor(m, l, sink, head) * out_scale;
  const float* grow = gate ? gate + (static_cast<size_t>(t0 + c) * nq + head) * gate_dim : nullptr;
  if (gate && gate_dim == 1) f *= grow[0];
  T* dst = out + static_cast<size_t>(t0 + c) * out_ld + head * dv;
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * dt + 8 * (i >> 2) + 4 * h + (i & 3);
      if (d < dv) dst[d] = from_float<T>(o[dt][i] * (gate_dim > 1 && gate ? f * grow[d] : f));
    }
}

// The tile kernel for bfloat16 queries and caches, on the matrix cores' 16-bit instruction with nothing rounded that
// the float32 form keeps: a product of two bfloat16 values is exact in float32, so S^T = K Q^T is what the float32
// instruction gives (sums in float32 either way); and a float32 weight p is split into three bfloat16 pieces
// p = p1 + p2 + p3 (p1 = bf16(p), p2 = bf16(p - p1), p3 = p - p1 - p2, which has eight bits left: exact), each
// multiplied with the values and added in float32: scores and weights stay 32-bit. 32 such instructions a chunk and
// head of 128 where the float32 form has 128, keys, queries and values as bfloat16 in LDS (a third of the space, so
// that three blocks share a compute unit). Head sizes are multiples of eight; the caches start on 16 bytes.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
constexpr int kPad16 = 8;            // bfloat16 elements of padding behind a row of keys, queries or transposed values

// Where key kk of a chunk lies in a row of transposed values: the eight keys that a lane multiplies in one
// instruction (kk = 16 a + 4 h + u and 16 a + 8 + 4 h + u, u < 4) side by side, one 16-byte read.
__device__ inline int vt_slot(int kk) { return (kk & 16) + 8 * ((kk >> 2) & 1) + 4 * ((kk >> 3) & 1) + (kk & 3); }

template <int NV>
__global__ __launch_bounds__(kThreads) void attn_biased_tile16_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache, bf16* __restrict__ out,
    int out_ld, const float* __restrict__ gate, float out_scale, const int* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, int nq, int nkv, int dk, int dkp, int dv, int page_size, float scale, float cap,
    const float* __restrict__ bias, int far, int window, int keep_first, int chunk, int tab_lds, int bias_lds,
    const float* __restrict__ sink, int gate_dim) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int ldk = dkp + kPad16, ldv = kKeys + kPad16;
  bf16* Ks = reinterpret_cast<bf16*>(lds_raw);                 // [kKeys][ldk]
  bf16* Qs = Ks + kKeys * ldk;                                 // [4 waves][32 tokens][ldk]
  bf16* Vt = Qs + 4 * 32 * ldk;                                // [32 NV][ldv], keys in the order of vt_slot
  int* tab_s = reinterpret_cast<int*>(Vt + 32 * NV * ldv);     // [tab_lds]: the request's block table, if it fits
  float* bias_s = reinterpret_cast<float*>(tab_s + tab_lds);   // [4][far + 1]: the four heads' biases, if they fit
  __shared__ int page_s[2][kKeys];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int n_rep = nq / nkv, hgroups = (n_rep + 3) / 4;
  const int kvh = blockIdx.y / hgroups, hin = (blockIdx.y % hgroups) * 4 + wave;
  const bool active = hin < n_rep;  // a wave without a head still helps loading
  const int head = kvh * n_rep + (active ? hin : 0);
  const int t0 = tiles[2 * blockIdx.x], ntok = tiles[2 * blockIdx.x + 1];
  if (ntok <= 0) return;
  const int pos0 = positions[t0];
  const int* table = block_table + static_cast<size_t>(seq_of_token[t0]) * table_stride;

  const bool live = active && c < ntok;
  const int hi = c < ntok ? pos0 + c : pos0;
  const int lo = first_seen(hi, window, chunk);
  const int keep = window > 0 ? keep_first : 0;
  const float* bias_row = bias ? bias + static_cast<size_t>(head) * (far + 1) : nullptr;
  for (int i = tid; i < tab_lds; i += kThreads) tab_s[i] = table[i];
  if (bias && bias_lds) {
    for (int i = lane; i <= far; i += 64) bias_s[wave * (far + 1) + i] = bias_row[i];
    bias_row = bias_s + wave * (far + 1);
  }
  const uint4 zero4 = {0u, 0u, 0u, 0u};
  {  // this wave's queries: Qs[wave][token][d], zeros where there is no token or no element
    bf16* mine = Qs + wave * 32 * ldk;
    for (int i = lane; i < 32 * (dkp / 8); i += 64) {
      const int t = i / (dkp / 8), d = 8 * (i % (dkp / 8));
      uint4 v = zero4;
      if (active && t < ntok && d < dk) v = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(t0 + t) * nq + head) * dk + d);
      *reinterpret_cast<uint4*>(mine + t * ldk + d) = v;
    }
  }
  const bf16* myq = Qs + wave * 32 * ldk + c * ldk + 8 * h;
  f32x16 o[NV];
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int lo_all = first_seen(pos0, window, chunk);
  const int hi_all = pos0 + ntok - 1;
  const int kept_end = min(keep, lo_all);
  const int n_first = kept_end > 0 ? (kept_end - 1) / kKeys + 1 : 0;
  const int chunk_b = max(lo_all / kKeys, n_first);
  const int n_chunks = n_first + (hi_all / kKeys - chunk_b + 1);
  // the next chunk's keys and values are asked for (into registers) before the current chunk is multiplied, and go
  // to LDS when every wave is done with it
  constexpr int KI = kKeys * (kTileMaxKeyHead / 8) / kThreads, VI = (kKeys * 4 * NV + kThreads - 1) / kThreads;
  uint4 kreg[KI], vreg[VI];
  auto chunk_key0 = [&](int it) { return (it < n_first ? it : chunk_b + (it - n_first)) * kKeys; };
  auto page_of = [&](int key) {
    const int entry = key / page_size;
    if (key > hi_all || entry >= table_stride) return -1;
    return entry < tab_lds ? tab_s[entry] : table[entry];
  };
  auto ask = [&](int it) {
    const int key0 = chunk_key0(it), kg = dkp / 8;
    if (tid < kKeys) page_s[it & 1][tid] = page_of(key0 + tid);
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      const int i = tid + k * kThreads, key = key0 + i / kg, d = 8 * (i % kg);
      const int page = i < kKeys * kg ? page_of(key) : -1;
      kreg[k] = zero4;
      if (page >= 0 && d < dk)
        kreg[k] = *reinterpret_cast<const uint4*>(k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + key % page_size) * dk + d);
    }
#pragma unroll
    for (int k = 0; k < VI; ++k) {
      const int i = tid + k * kThreads, key = key0 + i / (4 * NV), d = 8 * (i % (4 * NV));
      const int page = i < kKeys * 4 * NV ? page_of(key) : -1;
      vreg[k] = zero4;
      if (page >= 0 && d < dv)
        vreg[k] = *reinterpret_cast<const uint4*>(v_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + key % page_size) * dv + d);
    }
  };
  auto stash = [&]() {
    const int kg = dkp / 8;
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      const int i = tid + k * kThreads, key = i / kg, d = 8 * (i % kg);
      if (i < kKeys * kg) *reinterpret_cast<uint4*>(Ks + key * ldk + d) = kreg[k];
    }
#pragma unroll
    for (int k = 0; k < VI; ++k) {
      const int i = tid + k * kThreads, key = i / (4 * NV), d = 8 * (i % (4 * NV));
      if (i < kKeys * 4 * NV) {
        const uint32_t w[4] = {vreg[k].x, vreg[k].y, vreg[k].z, vreg[k].w};
        const int slot = vt_slot(key);
#pragma unroll
        for (int u = 0; u < 8; ++u) Vt[(d + u) * ldv + slot].bits = static_cast<uint16_t>(u & 1 ? w[u >> 1] >> 16 : w[u >> 1] & 0xffffu);
      }
    }
  };
  __syncthreads();  // the table and the biases are in LDS
  ask(0);
  for (int it = 0; it < n_chunks; ++it) {
    const int key0 = chunk_key0(it);
    const int* pages = page_s[it & 1];
    __syncthreads();  // the previous chunk has been read by every wave (and the queries are written)
    stash();
    __syncthreads();
    if (it + 1 < n_chunks) ask(it + 1);
    if (!active) continue;

    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    const bf16* krow = Ks + c * ldk + 8 * h;
#pragma unroll 4
    for (int st = 0; st < dkp; st += 16) {  // elements st + 8 h .. st + 8 h + 7 of the key and the query
      const bf16x8 k8 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow + st));
      const bf16x8 q8 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(myq + st));
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k8, q8, s, 0, 0, 0);
    }

    // element i of s: key key0 + 8 (i / 4) + 4 h + i % 4, token c
    float bv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = key0 + 8 * (i >> 2) + 4 * h + (i & 3);
      bv[i] = bias_row ? bias_row[min(max(hi - key, 0), far)] : 0.f;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kk = 8 * (i >> 2) + 4 * h + (i & 3), key = key0 + kk;
      const bool seen = key <= hi && (key >= lo || key < keep) && pages[kk] >= 0;
      const float shaped = shaped_score(s[i], scale, cap, nullptr, 0, 0) + bv[i];
      s[i] = seen ? shaped : -INFINITY;
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = expf(m - m_use);
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = expf(s[i] - m_use);
      sum += s[i];
    }
    l = l * alpha + sum;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
    // the weights in three bfloat16 pieces each; piece[a]: the lane's eight keys of instruction a (s[8 a .. 8 a + 7])
    uint4 piece[3][2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      uint32_t w1[4], w2[4], w3[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float p0 = s[8 * a + 2 * u], p1 = s[8 * a + 2 * u + 1];
        w1[u] = pack_bf16x2(p0, p1);
        const float r0 = p0 - __uint_as_float(w1[u] << 16), r1 = p1 - __uint_as_float(w1[u] & 0xffff0000u);
        w2[u] = pack_bf16x2(r0, r1);
        w3[u] = pack_bf16x2(r0 - __uint_as_float(w2[u] << 16), r1 - __uint_as_float(w2[u] & 0xffff0000u));
      }
      piece[0][a] = uint4{w1[0], w1[1], w1[2], w1[3]};
      piece[1][a] = uint4{w2[0], w2[1], w2[2], w2[3]};
      piece[2][a] = uint4{w3[0], w3[1], w3[2], w3[3]};
    }
#pragma unroll
    for (int dt = 0; dt < NV; ++dt)
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const bf16x8 v8 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(Vt + (32 * dt + c) * ldv + 16 * a + 8 * h));
#pragma unroll
        for (int pc = 2; pc >= 0; --pc)  // the smallest pieces first
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v8, __builtin_bit_cast(bf16x8, piece[pc][a]), o[dt], 0, 0, 0);
      }
  }

  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  if (!live) return;
  float f = softmax_factor(m, l, sink, head) * out_scale;
  const float* grow = gate ? gate + (static_cast<size_t>(t0 + c) * nq + head) * gate_dim : nullptr;
  if (gate && gate_dim == 1) f *= grow[0];
  bf16* dst = out + static_cast<size_t>(t0 + c) * out_ld + head * dv;
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * dt + 8 * (i >> 2) + 4 * h + (i & 3);
      if (d < dv) dst[d] = from_float<bf16>(o[dt][i] * (gate_dim > 1 && gate ? f * grow[d] : f));
    }
}

// ---------------------------------------------------------------------------------------------
constexpr int kSpan = 128;
constexpr int kMaxHead = 256;

// A block: one token, up to kGroup query heads of one key/value head, the keys in spans of 128. The heads share what
// the block reads: a thread takes a key's row once for its heads' scores (two threads a key, each with every second
// head), and a value once for all heads' sums. VEC: the key head is a multiple of eight elements and the cache starts
// on 16 bytes (a key in 16-byte loads).
constexpr int kGroup = 8;
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void attn_biased_single_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    int out_ld, const float* __restrict__ gate, float out_scale, const int* __restrict__ tokens,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, int nq, int nkv, int dk, int dv, int page_size, float scale, float cap,
    const float* __restrict__ bias, int far, int window, int keep_first, int chunk, int hg, float* __restrict__ part,
    const float* __restrict__ sink, int gate_dim) {
  __shared__ __attribute__((aligned(16))) float qs[kGroup][kMaxHead];
  __shared__ float sc[kGroup][kSpan];
  __shared__ int row_s[kSpan];
  __shared__ float accs[kGroup][kThreads];
  __shared__ float m_s[kGroup], l_s[kGroup], alpha_s[kGroup];
  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int rep = nq / nkv, hgroups = (rep + hg - 1) / hg;
  const int kvh = blockIdx.y / hgroups, first = (blockIdx.y % hgroups) * hg, nh = min(hg, rep - first);
  const int h0 = kvh * rep + first;  // the block's heads are h0 .. h0 + nh - 1
  const int pos = positions[n];
  const int* table = block_table + static_cast<size_t>(seq_of_token[n]) * table_stride;
  const int lo = first_seen(pos, window, chunk);
  const int kept_end = window > 0 ? min(keep_first, lo) : 0;  // keys 0 .. kept_end - 1, then lo .. pos
  const int spans_first = (kept_end + kSpan - 1) / kSpan, spans_all = spans_first + (pos - lo) / kSpan + 1;
  // with scratch for partial results a block takes one span (grid.z of them), else all of them in turn
  const int span_lo = part ? static_cast<int>(blockIdx.z) : 0, span_hi = part ? min(span_lo + 1, spans_all) : spans_all;
  if (span_lo >= span_hi) return;
  for (int i = tid; i < nh * dk; i += kThreads) qs[i / dk][i % dk] = to_float(q[(static_cast<size_t>(n) * nq + h0 + i / dk) * dk + i % dk]);
  if (tid < kGroup) m_s[tid] = -INFINITY, l_s[tid] = 0.f;
  __syncthreads();

  const int groups = kThreads / dv;  // >= 1: dv <= 256
  const int g = tid / dv, d = tid % dv;
  const bool active = g < groups;
  float acc[kGroup];
#pragma unroll
  for (int a = 0; a < kGroup; ++a) acc[a] = 0.f;
  const int j = tid & (kSpan - 1), side = tid / kSpan;  // this thread's key of a span; it scores heads side, side + 2, ...
  for (int span = span_lo; span < span_hi; ++span) {
    const int base = span < spans_first ? span * kSpan : lo + (span - spans_first) * kSpan;
    const int cnt = min(kSpan, (span < spans_first ? kept_end : pos + 1) - base);
    if (side < nh) {
      const int key = base + j;
      const int page = j < cnt ? table[key / page_size] : -1, off = key % page_size;
      float s[kGroup / 2];
#pragma unroll
      for (int a = 0; a < kGroup / 2; ++a) s[a] = 0.f;
      if (side == 0) row_s[j] = page >= 0 ? page * page_size + off : -1;  // the key's row in the cache, for the second product
      if (page >= 0) {
        const T* kp = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * dk;
        if (VEC) {
#pragma unroll 2
          for (int e = 0; e < dk; e += 8) {
            float kv[8];
            load8(kp + e, kv);
#pragma unroll
            for (int a = 0; a < kGroup / 2; ++a)
              if (side + 2 * a < nh)
#pragma unroll
                for (int u = 0; u < 8; ++u) s[a] = fmaf(qs[side + 2 * a][e + u], kv[u], s[a]);
          }
        } else {
          for (int e = 0; e < dk; ++e) {
            const float kv = to_float(kp[e]);
#pragma unroll
            for (int a = 0; a < kGroup / 2; ++a)
              if (side + 2 * a < nh) s[a] = fmaf(qs[side + 2 * a][e], kv, s[a]);
          }
        }
      }
#pragma unroll
      for (int a = 0; a < kGroup / 2; ++a)
        if (side + 2 * a < nh) {
          const float* bias_row = bias ? bias + static_cast<size_t>(h0 + side + 2 * a) * (far + 1) : nullptr;
          sc[side + 2 * a][j] = page >= 0 ? shaped_score(s[a], scale, cap, bias_row, pos - key, far) : -INFINITY;
        }
    }
    __syncthreads();
    // a wave a head: the running maximum and sum, the scores turned into weights
    for (int a = wave; a < nh; a += kThreads / kWave) {
      const float s0 = sc[a][lane], s1 = sc[a][lane + kWave];
      const float m_old = m_s[a], m_new = fmaxf(m_old, wave_max(fmaxf(s0, s1)));
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float p0 = expf(s0 - m_use), p1 = expf(s1 - m_use), alpha = expf(m_old - m_use);
      sc[a][lane] = p0, sc[a][lane + kWave] = p1;
      const float sum = wave_sum(p0 + p1);
      if (lane == 0) m_s[a] = m_new, l_s[a] = l_s[a] * alpha + sum, alpha_s[a] = alpha;
    }
    __syncthreads();
    if (active) {
#pragma unroll
      for (int a = 0; a < kGroup; ++a)
        if (a < nh) acc[a] *= alpha_s[a];
      // eight keys at a time, so that their values are on their way together
      for (int j0 = g; j0 < cnt; j0 += 8 * groups) {
        float vv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int jj = j0 + u * groups;
          const int row = jj < cnt ? row_s[jj] : -1;
          vv[u] = row >= 0 ? to_float(v_cache[((static_cast<size_t>(row / page_size) * nkv + kvh) * page_size + row % page_size) * dv + d]) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int jj = j0 + u * groups;
          if (jj < cnt)
#pragma unroll
            for (int a = 0; a < kGroup; ++a)
              if (a < nh) acc[a] = fmaf(sc[a][jj], vv[u], acc[a]);
        }
      }
    }
    __syncthreads();  // sc[] and row_s[] are read; the next span may write them
  }
#pragma unroll
  for (int a = 0; a < kGroup; ++a) accs[a][tid] = active && a < nh ? acc[a] : 0.f;
  __syncthreads();
  for (int i = tid; i < nh * dv; i += kThreads) {
    const int a = i / dv, dd = i % dv, h = h0 + a;
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += accs[a][gg * dv + dd];
    if (part) {  // [token of the list][head][span][dv + 2]: unnormalised output, max, sum
      float* dst = part + ((static_cast<size_t>(blockIdx.x) * nq + h) * gridDim.z + blockIdx.z) * (dv + 2);
      dst[dd] = total;
      if (dd == 0) dst[dv] = m_s[a], dst[dv + 1] = l_s[a];
      continue;
    }
    float f = softmax_factor(m_s[a], l_s[a], sink, h) * out_scale;
    if (gate) f *= gate[(static_cast<size_t>(n) * nq + h) * gate_dim + (gate_dim > 1 ? dd : 0)];
    out[static_cast<size_t>(n) * out_ld + h * dv + dd] = from_float<T>(total * f);
  }
}

// out = gate * out_scale * sum_s acc_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the token's spans, in their order.
template <typename T>
__global__ __launch_bounds__(kThreads) void attn_biased_join_kernel(
    const float* __restrict__ part, T* __restrict__ out, int out_ld, const float* __restrict__ gate, float out_scale,
    const int* __restrict__ tokens, const int* __restrict__ positions, int nq, int dv, int window, int keep_first,
    int chunk, int max_spans, const float* __restrict__ sink, int gate_dim) {
  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[n];
  const int lo = first_seen(pos, window, chunk);
  const int kept_end = window > 0 ? min(keep_first, lo) : 0;
  const int spans = min(max_spans, (kept_end + kSpan - 1) / kSpan + (pos - lo) / kSpan + 1);
  const float* src = part + (static_cast<size_t>(blockIdx.x) * nq + h) * max_spans * (dv + 2);
  float M = -INFINITY;
  for (int s = 0; s < spans; ++s) M = fmaxf(M, src[s * (dv + 2) + dv]);
  if (sink) M = fmaxf(M, sink[h]);
  const float m_use = M == -INFINITY ? 0.f : M;
  if (tid < dv) {
    float total = 0.f, l = 0.f;
    for (int s = 0; s < spans; ++s) {
      const float w = expf(src[s * (dv + 2) + dv] - m_use);
      total = fmaf(src[s * (dv + 2) + tid], w, total);
      l = fmaf(src[s * (dv + 2) + dv + 1], w, l);
    }
    if (sink) l += expf(sink[h] - m_use);
    float f = (l > 0.f ? 1.f / l : 0.f) * out_scale;
    if (gate) f *= gate[(static_cast<size_t>(n) * nq + h) * gate_dim + (gate_dim > 1 ? tid : 0)];
    out[static_cast<size_t>(n) * out_ld + h * dv + tid] = from_float<T>(total * f);
  }
}

int check_geometry(const char* what, int nq, int nkv, int dk, int dv, int page_size) {
  PYRE_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "%s: %d query heads do not divide over %d key/value heads", what, nq, nkv);
  PYRE_REQUIRE(dk > 0 && dk <= kMaxHead && dv > 0 && dv <= kMaxHead, "%s: head sizes %d / %d are outside 1..%d", what, dk, dv, kMaxHead);
  PYRE_REQUIRE(page_size > 0 && nq <= 65535, "%s: bad page size or too many heads", what);
  return 0;
}

}  // namespace

extern "C" int pyre_unit_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                   void* q_out, int q_dt, void* k_cache, void* v_cache, int cache_dt, float* gate_out,
                                   const int* slots, int n, int nq, int nkv, int dk, int dv, int page_size,
                                   int unit_norm, float eps, int write_kv, hipStream_t stream) {
  if (check_geometry("unit_qkv_write", nq, nkv, dk, dv, page_size)) return 1;
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(q_dt) && known_dtype(cache_dt) && n_partials >= 1, "unit_qkv_write: bad dtypes");
  PYRE_REQUIRE(!write_kv || (k_cache && v_cache && slots), "unit_qkv_write: a cache write needs caches and slots");
  PYRE_REQUIRE(!unit_norm || eps > 0.f, "unit_qkv_write: eps must be positive");
  if (n <= 0) return 0;
  if (dk % 4 == 0 && dv % 4 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 && q_dt == cache_dt &&
      reinterpret_cast<uintptr_t>(proj) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0) {
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL((unit_qkv_write_vec_kernel<TP, TC>), dim3(n), dim3(kThreads), 0, stream,
                           static_cast<const TP*>(proj), n_partials, static_cast<size_t>(partial_stride), ld, col0,
                           static_cast<TC*>(q_out), static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), gate_out, slots,
                           nq, nkv, dk, dv, page_size, unit_norm, eps, gate_out ? 1 : 0, write_kv)));
    return check_launch("unit_qkv_write");
  }
  PYRE_DISPATCH(cache_dt, TC,
      hipLaunchKernelGGL(unit_qkv_write_kernel<TC>, dim3(n), dim3(kThreads), 0, stream, proj, proj_dt, n_partials,
                         static_cast<size_t>(partial_stride), ld, col0, q_out, q_dt, static_cast<TC*>(k_cache),
                         static_cast<TC*>(v_cache), gate_out, slots, nq, nkv, dk, dv, page_size, unit_norm, eps,
                         gate_out ? 1 : 0, write_kv));
  return check_launch("unit_qkv_write");
}

extern "C" int pyre_attn_biased_tile(const void* q, void* out, int out_ld, int dt, const void* k_cache, const void* v_cache,
                                     const float* gate, float out_scale, const int* tiles, int n_tiles,
                                     const int* positions, const int* seq_of_token, const int* block_table,
                                     int table_stride, int nq, int nkv, int dk, int dv, int page_size, float scale,
                                     float cap, const float* bias, int far, int window, int keep_first, int chunk,
                                     const float* sink, int gate_dim, hipStream_t stream) {
  if (check_geometry("attn_biased_tile", nq, nkv, dk, dv, page_size)) return 1;
  PYRE_REQUIRE(gate_dim == 1 || gate_dim == dv, "attn_biased_tile: a gate per head or per element, not per %d", gate_dim);
  PYRE_REQUIRE(known_dtype(dt) && table_stride > 0 && window >= 0 && keep_first >= 0 && far >= 0 && chunk >= 0, "attn_biased_tile: bad arguments");
  PYRE_REQUIRE(dk <= kTileMaxKeyHead, "attn_biased_tile: key heads of %d elements are more than %d", dk, kTileMaxKeyHead);
  if (n_tiles <= 0) return 0;
  const int hgroups = (nq / nkv + 3) / 4;
  PYRE_REQUIRE(nkv * hgroups <= 65535, "attn_biased_tile: grid too large");
  const int dkp = (dk + 31) / 32 * 32, nv = (dv + 31) / 32;
  const int nvp = nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : 8;
  size_t lds = sizeof(float) * (static_cast<size_t>(kKeys + 4 * 32) * (dkp + 4) + 32 * nvp * kVtLd);
  // what is left of a compute unit's LDS takes the request's block table and the four heads' biases
  const size_t budget = 158 * 1024;
  const int tab_lds = lds + sizeof(int) * table_stride <= budget ? table_stride : 0;
  lds += sizeof(int) * tab_lds;
  const int bias_lds = bias && lds + sizeof(float) * 4 * (far + 1) <= budget ? 1 : 0;
  lds += bias_lds ? sizeof(float) * 4 * (far + 1) : 0;
  const dim3 grid(n_tiles, nkv * hgroups);
#define PYRE_TILE(T, NV, VEC)                                                                                           \
  do {                                                                                                               \
    static size_t raised = 64 * 1024;                                                                                \
    if (lds > raised) {                                                                                              \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_biased_tile_kernel<T, NV, VEC>),                        \
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)      \
        return fail("attn_biased_tile: the device refuses %zu bytes of LDS", lds);                                   \
      raised = lds;                                                                                                  \
    }                                                                                                                \
    hipLaunchKernelGGL((attn_biased_tile_kernel<T, NV, VEC>), grid, dim3(kThreads), lds, stream, static_cast<const T*>(q), \
                       static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), static_cast<T*>(out), out_ld, \
                       gate, out_scale, tiles, positions, seq_of_token, block_table, table_stride, nq, nkv, dk, dkp,  \
                       dv, page_size, scale, cap, bias, far, window, keep_first, chunk, tab_lds, bias_lds, sink, gate_dim); \
  } while (0)
#define PYRE_TILE_NV(T, VEC)                \
  switch (nvp) {                            \
    case 1: PYRE_TILE(T, 1, VEC); break;    \
    case 2: PYRE_TILE(T, 2, VEC); break;    \
    case 4: PYRE_TILE(T, 4, VEC); break;    \
    default: PYRE_TILE(T, 8, VEC); break;   \
  }
  const bool vec = dk % 8 == 0 && dv % 8 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(v_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0;
  if (dt == kBF16 && vec) {  // the 16-bit instruction, scores and weights in 32 bits all the same
    const int ldk = dkp + kPad16, ldv = kKeys + kPad16;
    size_t lds16 = sizeof(bf16) * (static_cast<size_t>(kKeys + 4 * 32) * ldk + 32 * nvp * ldv);
    lds16 = (lds16 + 15) / 16 * 16;
    const int tab16 = lds16 + sizeof(int) * table_stride <= 48 * 1024 ? table_stride : 0;
    lds16 += sizeof(int) * tab16;
    const int bias16 = bias && lds16 + sizeof(float) * 4 * (far + 1) <= 52 * 1024 ? 1 : 0;
    lds16 += bias16 ? sizeof(float) * 4 * (far + 1) : 0;
#define PYRE_TILE16(NV)                                                                                                  \
  do {                                                                                                                   \
    static size_t raised = 64 * 1024;                                                                                    \
    if (lds16 > raised) {                                                                                                \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_biased_tile16_kernel<NV>),                             \
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds16)) != hipSuccess)        \
        return fail("attn_biased_tile: the device refuses %zu bytes of LDS", lds16);                                     \
      raised = lds16;                                                                                                    \
    }                                                                                                                    \
    hipLaunchKernelGGL((attn_biased_tile16_kernel<NV>), grid, dim3(kThreads), lds16, stream, static_cast<const bf16*>(q), \
                       static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache), static_cast<bf16*>(out),    \
                       out_ld, gate, out_scale, tiles, positions, seq_of_token, block_table, table_stride, nq, nkv, dk,  \
                       dkp, dv, page_size, scale, cap, bias, far, window, keep_first, chunk, tab16, bias16, sink,         \
                       gate_dim);                                                                                        \
  } while (0)
    switch (nvp) {
      case 1: PYRE_TILE16(1); break;
      case 2: PYRE_TILE16(2); break;
      case 4: PYRE_TILE16(4); break;
      default: PYRE_TILE16(8); break;
    }
#undef PYRE_TILE16
    return check_launch("attn_biased_tile");
  }
  if (dt == kF32) {
    if (vec) { PYRE_TILE_NV(float, true) } else { PYRE_TILE_NV(float, false) }
  } else {
    if (vec) { PYRE_TILE_NV(bf16, true) } else { PYRE_TILE_NV(bf16, false) }
  }
#undef PYRE_TILE_NV
#undef PYRE_TILE
  return check_launch("attn_biased_tile");
}

// Spans of 128 keys that a token of such a launch can have: those of the kept first tokens and those
// of the window (or of all `max_keys` keys that a block table holds).
extern "C" int pyre_attn_biased_spans(int max_keys, int window, int keep_first, int chunk) {
  int seen = window > 0 ? min(window, max_keys) : max_keys;
  if (chunk > 0) seen = min(seen, chunk);
  return (window > 0 ? (min(keep_first, max_keys) + kSpan - 1) / kSpan : 0) + (max(seen, 1) - 1) / kSpan + 1;
}

extern "C" int pyre_attn_biased_single(const void* q, void* out, int out_ld, int dt, const void* k_cache,
                                       const void* v_cache, const float* gate, float out_scale, const int* tokens,
                                       int n, const int* positions, const int* seq_of_token, const int* block_table,
                                       int table_stride, int nq, int nkv, int dk, int dv, int page_size, float scale,
                                       float cap, const float* bias, int far, int window, int keep_first, int chunk,
                                       float* part, int max_spans, const float* sink, int gate_dim,
                                       hipStream_t stream) {
  if (check_geometry("attn_biased_single", nq, nkv, dk, dv, page_size)) return 1;
  PYRE_REQUIRE(gate_dim == 1 || gate_dim == dv, "attn_biased_single: a gate per head or per element, not per %d", gate_dim);
  PYRE_REQUIRE(known_dtype(dt) && table_stride > 0 && window >= 0 && keep_first >= 0 && far >= 0 && chunk >= 0, "attn_biased_single: bad arguments");
  PYRE_REQUIRE(!part || (max_spans >= 1 && max_spans <= 65535), "attn_biased_single: %d spans are not a launch", max_spans);
  if (n <= 0) return 0;
  // the query heads of a key/value head in blocks of up to kGroup heads, which read the keys and values once for all of
  // them: as many heads a block as still leave two blocks for every compute unit (a head's sums do not depend on its
  // block-mates), equally many in each
  const int rep = nq / nkv, want = 2 * compute_units();
  int hgroups = rep;
  for (int g = (rep + kGroup - 1) / kGroup; g < rep; ++g)
    if (static_cast<long>(n) * nkv * g * (part ? max_spans : 1) >= want) {
      hgroups = g;
      break;
    }
  const int hg = (rep + hgroups - 1) / hgroups;
  hgroups = (rep + hg - 1) / hg;  // as the kernel counts them: blocks of hg heads may be fewer than were asked for
  PYRE_REQUIRE(hg >= 1 && hg <= kGroup && hgroups * hg >= rep && (hgroups - 1) * hg < rep && static_cast<long>(nkv) * hgroups <= 65535,
               "attn_biased_single: %d heads a key/value head do not go into %d blocks of %d", rep, hgroups, hg);
  const dim3 grid(n, nkv * hgroups, part ? max_spans : 1);
#define PYRE_SINGLE(VEC)                                                                                                 \
  PYRE_DISPATCH(dt, T,                                                                                                    \
      hipLaunchKernelGGL((attn_biased_single_kernel<T, VEC>), grid, dim3(kThreads), 0, stream,                            \
                         static_cast<const T*>(q), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache),        \
                         static_cast<T*>(out), out_ld, gate, out_scale, tokens, positions, seq_of_token, block_table,     \
                         table_stride, nq, nkv, dk, dv, page_size, scale, cap, bias, far, window, keep_first, chunk, hg, part, \
                         sink, gate_dim))
  if (dk % 8 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0) {
    PYRE_SINGLE(true);
  } else {
    PYRE_SINGLE(false);
  }
#undef PYRE_SINGLE
  if (part)
    PYRE_DISPATCH(dt, T,
        hipLaunchKernelGGL(attn_biased_join_kernel<T>, dim3(n, nq), dim3(kThreads), 0, stream, part, static_cast<T*>(out),
                           out_ld, gate, out_scale, tokens, positions, nq, dv, window, keep_first, chunk, max_spans, sink,
                           gate_dim));
  return check_launch("attn_biased_single");
}
