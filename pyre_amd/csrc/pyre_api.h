// C entry points of the gfx950 kernel library. Pointers are device pointers
// unless a comment says otherwise; `stream` is the HIP stream the work is put on.
// Every function returns 0, or non-zero after storing a message that
// pyre_last_error() returns. Element type codes: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

const char* pyre_last_error();
int pyre_abi_version();
// Compute units of the current device (256 where there is no device to ask): the kernels whose
// blocks are meant to fill the chip in one round shape their launches by it, and so must
// whoever plans work for them on the host.
int pyre_compute_units();
// A digest of the sources this library was compiled from, as the build wrote it in.
const char* pyre_sources_digest();

// Streams `bytes` of device memory through the chip and writes (almost) nothing:
// a measurement of achievable read bandwidth.
int pyre_read_probe(const void* p, size_t bytes, int blocks, unsigned* sink, hipStream_t stream);

// out[n] = table[ids[n]] * scale, float32.
int pyre_embed(const void* table, int table_dt, const int* ids, float* out, int n, int hidden, float scale,
               hipStream_t stream);

int pyre_add_rmsnorm(float* resid, const void* delta, int delta_dt, int n_partials,
                     long partial_stride, const void* bias, int bias_dt, const void* gain,
                     int gain_dt, void* out, int out_dt, const int* rows, int n, int hidden,
                     float eps, hipStream_t stream);

// Finishes the q/k/v product (partial sums, bias), rotates queries and keys by position, stores
// the queries and, with write_kv, keys and values at slots[n] = page * page_size + offset
// (-1: not stored) of caches k [pages, nkv, page_size, hd] and v [pages, nkv, hd, page_size]. The
// tokens that one call writes into one page are neighbours in the batch and take consecutive
// slots in rising order (a request's next positions); the last of them zeroes the values of the
// slots behind it, so that nothing of the page's previous owner stays behind a request's last key.
int pyre_rope_kv_write(const void* qkv, int qkv_dt, int n_partials, long partial_stride,
                       const void* bias, int bias_dt, void* q_out, int q_dt, void* k_cache,
                       void* v_cache, int cache_dt, const float* cos_t, const float* sin_t,
                       int rotary_dim, const int* positions, const int* slots, int n, int nq,
                       int nkv, int hd, int page_size, int write_kv, hipStream_t stream);

int pyre_silu_mul(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out,
                  int out_dt, int n, int inter, hipStream_t stream);

int pyre_reduce_partials(const void* in, int in_dt, int n_partials, long partial_stride,
                         const void* bias, int bias_dt, void* out, int out_dt, int n, int width,
                         hipStream_t stream);

int pyre_gemm_generic(const void* A, int a_dt, long lda, const int* a_rows, const void* W,
                      int w_dt, long ldw, const void* bias, int bias_dt, void* out, int out_dt,
                      long ldo, int M, int N, int K, hipStream_t stream);

// base[o][ids[i]][0 .. row_elems) = pattern for every o < n_outer: rows of a contiguous
// [n_outer, n_rows, row_elems] tensor of 2- or 4-byte elements (outer_stride in elements).
// ids_host is HOST memory. Zeroes state slots; poisons freed pages in the debug mode.
int pyre_fill_rows(void* base, int elem_bytes, long outer_stride, int n_outer, int n_rows, long row_elems,
                   const int* ids_host, int n_ids, unsigned pattern, hipStream_t stream);

// The same for float32 operands and results only, on the matrix cores' float32 instruction:
// the product of the true 32-bit path. The order of an element's additions depends on k alone.
// ksplit > 1: partial sums out[s] (part_stride elements apart) over ksplit parts of k, the bias
// in part 0; the consumer adds them in the order 0..ksplit-1.
int pyre_gemm_f32(const float* A, long lda, const float* W, long ldw, const void* bias, int bias_dt,
                  float* out, long ldo, long part_stride, int M, int N, int K, int ksplit,
                  hipStream_t stream);

// bfloat16 products with 1..64 rows (decode): 1 if the kernel takes the shape.
int pyre_gemm_skinny_supports(int M, int N, int K, long ldx, long ldw);

// out: float32 [ksplit][M][N] partial sums of X[M, K] W[N, K]^T over ksplit parts of k.
int pyre_gemm_skinny_bf16(const void* X, long ldx, const void* W, long ldw, float* out, int M, int N,
                          int K, int ksplit, hipStream_t stream);

// W = [gate rows; up rows] (two_i x K); out: bfloat16 [M][two_i / 2] = silu(X gate^T) * (X up^T).
int pyre_gemm_skinny_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M,
                               int two_i, int K, hipStream_t stream);

// The first of them for up to 256 rows (a decode step of many requests), for products with few
// output columns: a block keeps all rows of X against 64 rows of W (128 with `wide`), and ksplit
// blocks share them. out: float32 [ksplit][M][N].
int pyre_gemm_mid_supports(int M, int N, int K, long ldx, long ldw);
int pyre_gemm_mid_bf16(const void* X, long ldx, const void* W, long ldw, float* out, int M, int N, int K,
                       int ksplit, int wide, hipStream_t stream);
// The second of them for up to 256 rows: a block takes 64 or 96 features (pyre_gemm_mid_silu_blocks
// blocks in all) against all rows of X; it pays where one round of blocks holds them.
int pyre_gemm_mid_silu_blocks(int M, int two_i);
int pyre_gemm_mid_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M, int two_i,
                            int K, hipStream_t stream);

// tokens: the n tokens of the flat batch to attend for, or null for tokens 0..n-1. max_keys: a
// bound on the keys that any of them sees (the block table's width in tokens will do); part:
// n * nq * pyre_attn_generic_spans(max_keys) * (hd + 2) floats of scratch when that is more than one span.
// matrix_cores: float32 queries and caches with a head size of 16, 32, ..., 128 and pages of a multiple
// of 16 tokens go to the kernel that reads a span's keys and values once for all query heads of a
// key/value head and multiplies on the float32 matrix instruction (its sums run in another order than
// those of one block per head, which 0 asks for: a difference of rounding). Which kernel runs depends
// on these sizes alone, never on the tokens of the call.
int pyre_attn_generic_spans(int max_keys);
int pyre_attn_generic(const void* q, void* out, int q_dt, const void* k_cache,
                      const void* v_cache, int cache_dt, const int* tokens, const int* positions,
                      const int* seq_of_token, const int* block_table, int table_stride, int n,
                      int nq, int nkv, int hd, int page_size, float scale, int window, int max_keys,
                      float* part, int matrix_cores, hipStream_t stream);

// Prompt portions in true float32 on the matrix cores' float32 instruction: tiles as for
// pyre_attn_prefill_bf16, float32 queries, caches and output, any head size up to 256, any
// page size. The order of a token's sums depends on its own bounds alone.
int pyre_attn_prefill_f32(const float* q, float* out, const float* k_cache, const float* v_cache,
                          const int* tiles, int n_tiles, const int* positions, const int* seq_of_token,
                          const int* block_table, int table_stride, int nq, int nkv, int hd, int page_size,
                          float scale, int window, hipStream_t stream);

// 1 if the MFMA attention kernels take this geometry (else use pyre_attn_generic).
int pyre_attn_mfma_supports(int hd, int page_size, int nq, int nkv);

// One new token per request, from a work list that deals every request's keys to blocks of
// four waves:
// rows of eight ints: work[0] = (blocks in the list, 0, ...), work[1 + i] = (token in the flat batch,
// block b of its request + 65536 * blocks nb of its request (<= 64), chunks `per` of 32 keys that a
// wave of this request takes, the request's first partial slot, the token's position, its request's
// row of the block table, 0, 0: the kernel takes position and row from the list, `positions` and
// `seq_of_token` are not read); block b takes chunks 4 b per ..
// 4 (b + 1) per - 1 of its request, counted from the first chunk that the token sees, and the
// nb blocks of a request cover all of them. The slots of the requests are disjoint runs of nb
// within 0..capacity-1. `alone`: a compute unit runs one block at a time (for steps of so few
// requests that a block per unit covers them); else two. The launch has
// `capacity` blocks per key/value head (and group of 16 query heads); blocks past the list's
// end exit. Scratch: part_acc [capacity, items, 16, hd] and part_ml [capacity, items, 16, 2]
// floats, counters [capacity, items] ints that are zero before the first call and are left
// at zero, items = nkv * ceil(nq / nkv / 16).
int pyre_attn_decode_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                               const int* work, int capacity, const int* positions,
                               const int* seq_of_token, const int* block_table, int table_stride,
                               float* part_acc, float* part_ml, int* counters, int alone, int nq, int nkv,
                               int hd, int page_size, float scale, int window, hipStream_t stream);

// The same for a step of single tokens straight from the step's q/k/v product (float32 partial sums
// [n_partials][n_rows][(nq + 2 nkv) hd], partial_stride elements apart, with its bias or null): every
// block sums, biases and rotates its heads' queries itself, and for every token and key/value head one
// wave writes the token's rotated key and its value into the cache (slots[token], -1: not stored;
// write_kv 0: a layer that keeps none) and zeroes the values behind it in its page, all with the
// arithmetic of pyre_rope_kv_write (the same bits in the cache and in the result), so that no kernel
// runs between the product and the attention. Full-head rotation (cos_t, sin_t: [positions][hd / 2]),
// heads of up to 128 elements, up to 16 query heads per key/value head.
int pyre_attn_decode_work_rope_supports(int hd, int page_size, int nq, int nkv, long partial_stride);
int pyre_attn_decode_work_rope_bf16(const float* qkv, int n_partials, long partial_stride, const void* bias,
                                    int bias_dt, const float* cos_t, const float* sin_t, const int* slots,
                                    int n_rows, int write_kv, void* out, void* k_cache, void* v_cache,
                                    const int* work, int capacity, const int* positions, const int* seq_of_token,
                                    const int* block_table, int table_stride, float* part_acc, float* part_ml,
                                    int* counters, int alone, int nq, int nkv, int hd, int page_size, float scale,
                                    int window, hipStream_t stream);


// Prompt portions. tiles[i] = (first token in the flat batch, token count <= 32),
// all tokens of a tile from one request at consecutive positions. Every wave reads the
// cache directly (any head size that pyre_attn_mfma_supports takes).
int pyre_attn_prefill_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                           const int* tiles, int n_tiles, const int* positions,
                           const int* seq_of_token, const int* block_table, int table_stride,
                           int nq, int nkv, int hd, int page_size, float scale, int window,
                           hipStream_t stream);

// The same for heads of up to 128 elements from a work list: K and V go straight into LDS in
// chunks of 64 keys for 32x32 MFMA tiles, and the chunks of a tile may be dealt to several blocks.
// work[2 i] = (first token of the tile, tokens <= 32, first chunk, last chunk), work[2 i + 1] =
// (first partial slot of the tile, this block's number among the tile's blocks, their number
// nb, 0); the nb blocks of a tile cover the chunks lo / 64 .. hi / 64 of the keys lo .. hi that
// its tokens see, each chunk once. A block has pyre_attn_prefill_waves(nq, nkv) waves, one per
// query head of a key/value head (groups of that many heads: `groups`). Scratch for tiles
// of more than one block: partials [slots, nkv * groups, waves, hd / 32 * 1024 + 128] floats
// and counters [slots, nkv * groups, waves] ints that are zero before the first call and are
// left at zero.
int pyre_attn_prefill_waves(int nq, int nkv);
int pyre_attn_prefill_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                                const int* work, int n_items, float* partials, int* counters,
                                int n_slots, const int* positions, const int* seq_of_token, const int* block_table,
                                int table_stride, int nq, int nkv, int hd, int page_size, float scale,
                                int window, hipStream_t stream);

// scratch: m * 64 floats followed by m * 64 ints of device memory.
int pyre_argmax(const float* logits, long row_stride, int* out, void* scratch, int m, int vocab,
                hipStream_t stream);

// pyre_argmax without a scratch argument and without any allocation. It has no counterpart in
// the reference; it is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc. The slices' partial results
// go to an array that is part of the library's device image (128 KB on every GPU the library
// runs on, until the process ends), so m is at most PYRE_ARGMAX_STATIC_MAX_ROWS; more rows are
// refused with an error. The caller makes the GPU of `stream`, `logits` and `out` the current
// device. Same kernels and same results as pyre_argmax. All calls on one GPU share that GPU's
// array: calls that may overlap there (two streams, two threads) race; put them on one stream
// or use pyre_argmax with scratch of their own. The first call on a device looks the array's
// address up (hipGetSymbolAddress), which must not happen while a stream is capturing: a caller
// that captures calls pyre_argmax_static_init() on that device beforehand (it launches nothing
// and may be called any number of times).
#define PYRE_ARGMAX_STATIC_MAX_ROWS 256
int pyre_argmax_static_init();
int pyre_argmax_static(const float* logits, long row_stride, int* out, int m, int vocab,
                       hipStream_t stream);

// tokens[i] = ids[src[i]] where src[i] >= 0: a step's token that is the previous step's
// sampled id, taken on the device so that the host need not wait for it.
int pyre_feed_tokens(int* tokens, const int* src, const int* ids, int n, hipStream_t stream);

int pyre_sample(const float* logits, long row_stride, const float* temperature,
                const float* uniform, int* out, int m, int vocab, hipStream_t stream);

// The gate/up products with another gated unit in the epilogue: out = g sigmoid(slope (g + cubic g^3)) (u + shift) with
// g = min(X gate^T, limit), u = clamp(X up^T, -limit, limit) (limit <= 0: no clipping); shapes as the _silu_ forms.
int pyre_gemm_skinny_glu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M, int two_i, int K,
                              float limit, float slope, float shift, float cubic, hipStream_t stream);
int pyre_gemm_mid_glu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M, int two_i, int K,
                           float limit, float slope, float shift, float cubic, hipStream_t stream);

// ---- layer norm around the residual stream, clipped gated activation, scaling (layernorm.hip) ----
// resid += y, out = LN(resid) * gain, where y is the pending term (partial sums, bias) or, with
// post_gain, LN(term; post_eps) * post_gain (* post_scale). rows: only these rows, resid untouched.
int pyre_add_layernorm(float* resid, const void* delta, int delta_dt, int n_partials, long partial_stride,
                       const void* bias, int bias_dt, const void* post_gain, int post_gain_dt,
                       const void* post_scale, int post_scale_dt, float post_eps, const void* gain,
                       int gain_dt, void* out, int out_dt, const int* rows, int n, int hidden, float eps,
                       hipStream_t stream);
// out[n, i] = g sigmoid(slope (g + cubic g^3)) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit); gu = [gate | up].
int pyre_clipped_glu(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out, int out_dt,
                     int n, int inter, float limit, float slope, float shift, float cubic, hipStream_t stream);
int pyre_scale(float* x, long total, float s, hipStream_t stream);

// ---- attention with capped scores, a bias by distance and kept first tokens (attention_biased.hip) ----
// proj columns from col0 on: nq query heads and nkv key heads of dk, nkv value heads of dv, then (gate_out
// given) nq gates. Caches: k [pages, nkv, page, dk], v [pages, nkv, page, dv].
int pyre_unit_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                        void* q_out, int q_dt, void* k_cache, void* v_cache, int cache_dt, float* gate_out,
                        const int* slots, int n, int nq, int nkv, int dk, int dv, int page_size,
                        int unit_norm, float eps, int write_kv, hipStream_t stream);
// chunk > 0: a query sees only the keys of its own run of `chunk` positions (runs counted from position 0).
// tiles: [n_tiles][2] = (first token, count <= 32). bias: float32 [nq][far + 1] by distance, or null.
// gate: float32 [tokens][nq] or null. out rows are out_ld elements apart; head h writes columns h dv ...
int pyre_attn_biased_tile(const void* q, void* out, int out_ld, int dt, const void* k_cache, const void* v_cache,
                          const float* gate, float out_scale, const int* tiles, int n_tiles,
                          const int* positions, const int* seq_of_token, const int* block_table,
                          int table_stride, int nq, int nkv, int dk, int dv, int page_size, float scale,
                          float cap, const float* bias, int far, int window, int keep_first, int chunk,
                          const float* sink, int gate_dim, hipStream_t stream);
// tokens: the n tokens of the flat batch to attend for (null: 0..n-1), a block per token and head.
int pyre_attn_biased_single(const void* q, void* out, int out_ld, int dt, const void* k_cache,
                            const void* v_cache, const float* gate, float out_scale, const int* tokens,
                            int n, const int* positions, const int* seq_of_token, const int* block_table,
                            int table_stride, int nq, int nkv, int dk, int dv, int page_size, float scale,
                            float cap, const float* bias, int far, int window, int keep_first, int chunk,
                            float* part, int max_spans, const float* sink, int gate_dim, hipStream_t stream);
// part: scratch of n * nq * max_spans * (dv + 2) floats, max_spans = pyre_attn_biased_spans(the most keys a
// block table holds, window, keep_first): a block then takes one span of 128 keys and a second kernel joins
// them in their order; null: a block takes all spans of its token and head in turn.
int pyre_attn_biased_spans(int max_keys, int window, int keep_first, int chunk);

// ---- gated linear attention (linear_attention.hip) ----
// proj columns from col0 on: q, k (heads dk each), v, g (heads dv each), the low-rank input (rank).
// x: float32 [n][3 heads dk + 2 heads dv] = [q | k | log decay | v | g].
int pyre_gla_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                     const void* a2, int a2_dt, const void* a2_bias, int bias_dt, float tau, float* x,
                     int n, int heads, int dk, int dv, int rank, hipStream_t stream);
// state: float32 [slots][heads][dk][dv]; o: float32 [tokens][heads dv]; request s owns the tokens
// q_start[s] .. q_start[s + 1] - 1 and the slot state_slots[s].
int pyre_gla_scan(const float* x, float* state, float* o, const int* q_start, const int* state_slots,
                  int n_seqs, int heads, int dk, int dv, float qscale, const float* decay,
                  hipStream_t stream);
// The same recurrence in chunks of 16 tokens (steps that carry prompt portions); differs from the scan by rounding.
// scratch: pyre_gla_chunks_scratch(...) floats, starting on 16 bytes; max_tokens: the most tokens that one request brings.
long pyre_gla_chunks_scratch(int n_tokens, int n_seqs, int heads, int dk, int dv);
int pyre_gla_chunks(const float* x, float* scratch, float* state, float* o, const int* q_start, const int* state_slots,
                    int n_tokens, int n_seqs, int max_tokens, int heads, int dk, int dv, float qscale, hipStream_t stream);
int pyre_gla_finish(const float* o, const float* x, const void* gain, int gain_dt, float eps, float out_scale,
                    void* out, int out_dt, int out_ld, int n, int heads, int dk, int dv, hipStream_t stream);

// ---- a norm without statistics and the squashing of logits (tanh_norm.hip) ----
// resid += a_scale (sum of a's partial sums + a_bias) + b_scale (the same of b); out = tanh(alpha resid) gain + shift.
// a, b: pending terms or null (b only with a); alpha: one element; shift may be null; alpha, gain and shift share
// param_dt. rows: only these rows, into a dense output, resid untouched.
int pyre_add_tanhnorm(float* resid, const void* a, int a_dt, int a_count, long a_stride, const void* a_bias,
                      int a_bias_dt, float a_scale, const void* b, int b_dt, int b_count, long b_stride,
                      const void* b_bias, int b_bias_dt, float b_scale, const void* alpha, const void* gain,
                      const void* shift, int param_dt, void* out, int out_dt, const int* rows, int n, int hidden,
                      hipStream_t stream);
// x <- cap tanh(x / cap), float32 in place.
int pyre_softcap(float* x, long total, float cap, hipStream_t stream);

// ---- between the input product and the attention kernels (latent.hip) ----
// proj columns from col0 on: nq query heads and nkv key heads of d; bias over these columns or null. The first rot
// elements of every head are turned by position (cos_t, sin_t: float32 [positions][rot / 2]); queries to
// q_out [n, nq d], turned keys to k_cache and the keys as they were to v_cache (both [pages, nkv, page, d]).
int pyre_rope_tied_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                         const void* bias, int bias_dt, void* q_out, int q_dt, void* k_cache, void* v_cache,
                         int cache_dt, const float* cos_t, const float* sin_t, int rot, const int* positions,
                         const int* slots, int n, int nq, int nkv, int d, int page_size, int write_kv,
                         hipStream_t stream);
// proj columns from col0 on: q_width of queries, then (write) rank of the compressed row, which is stored divided
// by its root mean square and times gain in c_cache [pages, 1, page, rank].
int pyre_latent_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                      void* q_out, int q_dt, void* c_cache, int cache_dt, const void* gain, int gain_dt, float eps,
                      const int* slots, int n, int q_width, int rank, int page_size, int write, hipStream_t stream);
// out[n, h, :] = x[n, h, :] w[h], w [heads, din, dout]; rows of x and out are x_ld and out_ld elements apart; one
// element type for all three.
int pyre_head_matmul(const void* x, int x_ld, const void* w, void* out, int out_ld, int dt, int n, int heads, int din,
                     int dout, hipStream_t stream);

// ---- a mixture of experts with a sigmoid router (moe.hip) ----
// gates[n, experts + extra] float32: for the `top` experts of largest logit z, s / (sum of the chosen s + 1e-20) with
// s = sigmoid(z), or (softmax) the softmax over the chosen logits alone; 0 for the others; sigmoid(z) for the `extra`
// columns behind the experts, which are gates of their own.
int pyre_route_topk(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                    float* gates, int n, int experts, int top, int softmax, int extra, hipStream_t stream);
// out[n, e ff + j] = gates[n, e] max(up, 0)^2 for e < experts, max(up, 0)^2 for the shared_ff columns behind them.
int pyre_expert_act(const void* up, int up_dt, int n_partials, long partial_stride, const float* gates, void* out,
                    int out_dt, int n, int experts, int ff, int shared_ff, hipStream_t stream);

// resid += y, out = (out_gain ? RMS(resid) * out_gain : resid): y the sum of up to two pending terms, each with an RMS
// norm and gain of its own (or none) and a factor, the sum normed again if outer_gain is given (postnorm.hip).
int pyre_add_rms_terms(float* resid, const void* a, int a_dt, int a_partials, long a_stride, const void* a_gain,
                       int a_gain_dt, float a_scale, const void* b, int b_dt, int b_partials, long b_stride,
                       const void* b_gain, int b_gain_dt, float b_scale, float inner_eps, const void* outer_gain,
                       int outer_dt, float outer_eps, const void* out_gain, int out_gain_dt, float out_eps, void* out,
                       int out_dt, const int* rows, int n, int hidden, hipStream_t stream);

// out[n] = table[ids[n]] + pairs[row of (previous token, token)]; state [slots][1] float32 holds a request's last token.
int pyre_bigram_embed(const void* table, const void* pairs, int dt, const int* ids, const int* positions,
                      const int* seq_of_token, const int* q_start, float* state, const int* state_slots, float* out, int n,
                      int hidden, int buckets, int mul_prev, int mul_cur, hipStream_t stream);

// The input product of an attention whose projections go through a short causal convolution (conv_attention.hip).
int pyre_conv_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                        const float* taps_w, int taps, float* conv_state, const int* state_slots, const int* seq_of_token,
                        const int* q_start, int n_seqs, const float* q_gain, const float* k_gain, float eps,
                        const float* cos, const float* sin, int rot, int neighbours, const int* positions, void* q_out,
                        int q_dt, void* k_cache, void* v_cache, int cache_dt, float* gate_out, const int* slots, int n,
                        int nq, int nkv, int dk, int dv, int page_size, int write_kv, hipStream_t stream);

// The rows [q | k | log decay | v | g] of the recurrent kernels for a fixed decay per head, queries and keys turned.
int pyre_retention_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                           const float* log_decay, const float* cos, const float* sin, int rot, int neighbours,
                           const int* positions, float kscale, float* x, int n, int heads, int dk, int dv,
                           hipStream_t stream);

int pyre_route_grouped(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                       const float* correction, float* gates, int n, int experts, int top, int groups, int keep_groups,
                       hipStream_t stream);
// The experts' gated units, weighted; behind them shared_ff columns of a shared expert, weighted by gates[n, shared_gate]
// (shared_gate < 0: by one).
int pyre_expert_glu_act(const void* gu, int gu_dt, int n_partials, long partial_stride, const float* gates,
                        long gates_stride, void* out, int out_dt, int n, int experts, int ff, int shared_ff,
                        int shared_gate, hipStream_t stream);
int pyre_add_weighted_rows(float* p, const void* h, int h_dt, long h_stride, const float* gates, long gates_stride,
                           int first, int count, int n, int width, hipStream_t stream);

// The input product of an attention whose queries and keys are normed over their whole projection (wide_norm_qkv.hip).
int pyre_wide_norm_qkv_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                             const float* bias, const float* q_gain, const float* k_gain, float eps, const float* cos,
                             const float* sin, int rot, const int* positions, void* q_out, int q_dt, void* k_cache,
                             void* v_cache, int cache_dt, const int* slots, int n, int nq, int nkv, int dk, int dv,
                             int page_size, int write_kv, hipStream_t stream);

// ---- the gated delta rule (delta_rule.hip) ----
// Columns of the float32 rows [q | k | decay | v | gate | beta] that its kernels share.
long pyre_gdr_row_width(int H, int G, int dk, int dv);
int pyre_gdr_prepare(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                     const float* bias, const float* taps_w, int taps, float* conv_state, const int* state_slots,
                     const int* seq_of_token, const int* q_start, int n_seqs, const void* a2, int a2_dt,
                     const float* dt_bias, const float* rate, const void* g2, int g2_dt, float unit_eps, float* x, int n,
                     int H, int G, int dk, int dv, int rank_a, int rank_g, hipStream_t stream);
// state [slots][H][dv][dk]: a column's rows lie together; max_tokens: the most tokens that one request brings (0: unknown)
int pyre_gdr_scan(const float* x, float* state, float* o, const int* q_start, const int* state_slots, int n_seqs,
                  int max_tokens, int H, int G, int dk, int dv, hipStream_t stream);
int pyre_gdr_finish(const float* o, const float* x, const void* gain, int gain_dt, float eps, float out_scale, void* out,
                    int out_dt, long out_ld, int n, int H, int G, int dk, int dv, hipStream_t stream);

// out[n, j] = gelu_tanh(z[n, j]) * table[ids[n], first + j], z the partial sums of a product [n, dim] (token_side.hip).
int pyre_token_side_gate(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                         const void* table, int table_dt, int table_width, int first, const int* ids, void* out,
                         int out_dt, int n, int dim, hipStream_t stream);
}  // extern "C"
