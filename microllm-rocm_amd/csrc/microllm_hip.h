// C interface of libmicrollm_hip: every function launches on `stream`, returns 0 or a
// non-zero code, and leaves a text for mll_last_error() when it refuses its arguments.
// Pointers are device pointers unless a comment says otherwise. `dtype` is 0 for float32 and
// 1 for bfloat16 and names the element type of activations, cache pages and, where stated,
// weights. Statistics, softmax and accumulators are float32 in every kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* mll_last_error();
int mll_version();

// out[t, :] = table[ids[t], :] widened to float32, times scale. An id outside [0, vocab) gives a row of NaN.
int mll_embedding(const void* table, int table_dtype, const int32_t* ids, float* out,
                  int n_tokens, int width, int vocab, float scale, hipStream_t stream);

// out[i] = act(in[i]) for count values; in is float32 (n_parts partial sums part_stride elements apart, added in
// order first) or of the output's type. act: 0 SiLU, 1 the exact gelu 0.5 z (1 + erf(z / sqrt 2)), 2 the tanh form.
int mll_activation(const void* in, int in_dtype, int n_parts, int64_t part_stride, void* out, int dtype, int64_t count, int act,
                   hipStream_t stream);

// For i < n_rows, r = rows ? rows[i] : i:  v = h[r] + (delta ? delta[r] : 0);
// if write_h, h[r] = v;  out[i] = v * rsqrt(mean(v^2) + eps) * weight.
// h is the float32 residual stream; out has element type `dtype`, delta `delta_dtype`
// (float32, or the same as out). delta may come in n_partials parts, partial_stride elements apart, which
// are added in order (the partial sums of a matrix product that was split over k).
int mll_rms_norm(float* h, const void* delta, int delta_dtype, int n_partials, int64_t partial_stride,
                 const int32_t* rows, const float* weight, float eps,
                 void* out, int dtype, int n_rows, int width, int write_h, hipStream_t stream);

// d = the delta's parts added in order; v = h[r] + mult * d * rsqrt(mean(d^2) + after_eps) * after_weight; if write_h,
// h[r] = v; out[i] = v * rsqrt(mean(v^2) + eps) * weight (weight null: no output). A sublayer's result that is normed
// itself before it joins the stream, fused with the norm that follows (csrc/norm_after.hip). extra (null: none): float32
// rows like h's, added to v after the delta (what a model adds to its stream between two layers).
int mll_rms_norm_after(float* h, const void* delta, int delta_dtype, int n_partials, int64_t partial_stride,
                       const int32_t* rows, const float* after_weight, float after_eps, float mult, const float* extra,
                       const float* weight, float eps, void* out, int dtype, int n_rows, int width, int write_h, hipStream_t stream);

// values[r][c] += bias[c] for n_rows rows of `width` float32 values, in place.
int mll_add_bias(float* values, const float* bias, int64_t n_rows, int width, hipStream_t stream);

// values[i] = cap * tanh(values[i] / cap), in place, float32.
int mll_softcap(float* values, int64_t count, float cap, hipStream_t stream);

// Adds a pending delta into the residual stream: h[r] += delta[r] for all rows.
int mll_residual_add(float* h, const void* delta, int dtype, int n_rows, int width, hipStream_t stream);

// out[t][i] = (cos, sin) of positions[t] * inv_freq[i], the angle in float64: float32 [n_tokens][n_freq][2].
int mll_rope_table(const int32_t* positions, const double* inv_freq, int n_freq, int n_tokens, float* out,
                   hipStream_t stream);

// Splits fused projections qkv[t] = [q (H*hd) | k (KVH*hd) | v (KVH*hd)], adds `bias` (nullable),
// rotates q and k by the split-half rule with angle position * inv_freq[i] in float64, or with the cos and sin
// of mll_rope_table's `cos_sin` if that is given (both null: no rotation; rotary_dim = 2 * n_freq <= hd), writes q to q_out[t] and k, v into the pages (laid out as
// cache_layout.h says): slot = slot_mapping[t] (negative: not stored), page = slot / page_size,
// offset = slot % page_size. k_cache / v_cache nullable together with slot_mapping. qkv has element type
// `in_dtype` (float32, or the same as `dtype`) and may come in n_partials parts, partial_stride elements
// apart, which are added in order; q_out and the pages have `dtype`. With pair_order the query and key heads
// of qkv hold dims p and p + n_freq side by side (columns 2p, 2p + 1), as a weight in rotary pair order gives
// them (see MllQkvStore); bias and outputs are in the ordinary order.
int mll_qkv_rope_store(const void* qkv, int in_dtype, int n_partials, int64_t partial_stride, int dtype,
                       const float* bias, const int32_t* positions,
                       const int32_t* slot_mapping, const double* inv_freq, const void* cos_sin, int n_freq,
                       void* q_out, void* k_cache, void* v_cache,
                       int n_tokens, int heads, int kv_heads, int head_dim, int page_size, int pair_order,
                       hipStream_t stream);

// Attention of every query token over its request's pages, for any dtype and head size.
// Key j is visible to a query at position p iff j <= p and (window <= 0 or p - j < window).
// block_table[seq, j / page_size] gives the page of key j. Reduction order depends only on
// (p, window), so the result does not depend on how tokens were cut into steps, to the last bit.
// A token whose seq_of_token is negative is skipped and its output row left as it is (a row that pads a step to
// a fixed shape).
// max_chunks 0: one wave per (token, head). max_chunks > 0: one wave per (token, head, chunk of
// mll_paged_attention_rowwise_chunk() keys) and a second kernel that merges the chunks in the same order with
// the same arithmetic (the same bits), for steps with few rows; no row's visible keys may then span more than
// max_chunks chunks (chunks lie at absolute positions), and part_o [n_tokens * heads * max_chunks * head_dim]
// and part_ml [n_tokens * heads * max_chunks * 2] floats are the workspace.
// usual_chunks (0: max_chunks): how many chunks the rows have in this step, where max_chunks leaves room for later
// steps of the same shape; it only decides how many heads a wave takes.
int mll_paged_attention_rowwise_chunk();
// In float32 with head sizes up to 128 a wave takes several query heads of a kv head (their keys and values read
// once) where the step still has waves enough for the GPU that way. This forces the count (1 to 8; 0: the launch
// chooses again) and returns the value before. The same bits whatever the count.
int mll_rowwise_heads_a_wave(int count);
int mll_paged_attention_rowwise(const void* q, int dtype, const void* k_cache, const void* v_cache,
                                const int32_t* block_table, int table_width,
                                const int32_t* seq_of_token, const int32_t* positions, void* out,
                                float* part_o, float* part_ml, int max_chunks, int usual_chunks, float scale, int window,
                                int n_tokens, int heads, int kv_heads, int head_dim, int page_size,
                                hipStream_t stream);

// The same attention for bfloat16 portions of prompts with MFMA: one workgroup per (two tiles of up to
// mll_paged_attention_prefill_tile() consecutive tokens of one request, query head). `tiles` holds, for each
// workgroup, (request index; first token in the flat list and number of tokens of the first tile; the same of the
// second, whose number may be 0); a tile never spans two requests and its tokens have consecutive positions.
// Workgroups take as long as the keys of both tiles together: pair a tile late in a prompt with an early one.
// An entry whose tiles are both empty is skipped (padding of the list to a fixed length).
int mll_paged_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                const int32_t* block_table, int table_width, const int32_t* tiles,
                                int n_tiles, const int32_t* positions, void* out, float scale, int window,
                                int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream);
int mll_paged_attention_prefill_tile();

// out[t, c] = silu(gate[t, c]) * up[t, c]; gate and up rows are `in_stride` elements apart.
int mll_silu_mul(const void* gate, const void* up, int64_t in_stride, void* out, int dtype,
                 int n_tokens, int width, hipStream_t stream);

// C[m, n] = sum_k A[m, k] * W[n, k] (+ bias[n]), all float32, k summed in ascending order by one
// thread per output element, so a row's result does not depend on the other rows. With splits > 1
// (only the number mll_gemm_f32_splits gives for the weight's shape) C is [splits, m, n]: sums over
// consecutive ranges of k, the bias in the first, for the reader to add in order.
int mll_gemm_f32_splits(int n, int k);
// Which kernel takes a product of at most 16 rows: 0 gives the choice back to the launch; 1 (an element a thread), 2
// (two rows and two columns) and 4 (one row and four columns; at most 8 rows) force one, for measurements and tests. Returns the value before. The same bits whichever.
int mll_gemm_f32_small_variant(int variant);
int mll_gemm_f32(const float* a, const float* w, const float* bias, float* c,
                 int m, int n, int k, int splits, hipStream_t stream);

// C = A . W^T for bfloat16 A [m <= 64, k] and a weight packed as [n/16][k/32][4][16][8] (zero padded):
// element (row, col) of W sits at piece (row / 16, col / 32), position ((col % 32) / 8, row % 16, col % 8).
// epilogue 0: float32 [m, n]; 1: bfloat16 [m, n]; 2: bfloat16 [m, n / 2] = silu(even weight rows' results) *
// (odd rows' results). The order of additions is fixed by (n, k): the same in every run and whatever the
// other rows of A.
// With `scale` (may be null; at most 16 rows) row r of the product is first multiplied by
// 1 / sqrt(sum_{g < groups} sumsq[r][g] / width + eps): the factor of an RMS norm whose input came without it.
struct MllRowScale {
    const float* sumsq;   // [m][stride], 16-byte aligned; the first `groups` of a row count
    int groups;
    int stride;           // a multiple of 4
    int width;
    float eps;
};
int mll_gemm_skinny(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                    const MllRowScale* scale, hipStream_t stream);

// What the q/k/v projection's product does with its result instead of writing it out: the work of
// mll_qkv_rope_store. The packed weight's rows must be in rotary pair order: in every query and key head, row
// 2p holds dim p and row 2p + 1 dim p + n_freq for p < n_freq, the other dims follow in place; value heads are
// as they are. bias (float32, may be null) and the outputs are in the ordinary order.
struct MllQkvStore {
    const float* bias;
    const int32_t* slot_mapping;   // [m] page * page_size + offset, or null: keys and values are not kept
    const float* cos_sin;          // [m][n_freq][2]: mll_rope_table's
    int n_freq;
    void* q_out;                   // bfloat16 [m, heads * head_dim]
    void* k_cache;                 // bfloat16 pages
    void* v_cache;
    int heads, kv_heads, head_dim, page_size;
};
// Queries, keys and values of at most 16 rows: A [m, k] . W^T with n = (heads + 2 kv_heads) * head_dim, finished
// as `store` says.
int mll_gemm_skinny_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store,
                        const MllRowScale* scale, hipStream_t stream);

// The product of at most 16 rows added to the residual stream, and the next RMS norm begun: h += A . W^T;
// x_out = h * norm_weight (the norm's input without the rows' factors); sumsq_out[r][g] = the sum of h[r]^2 over
// columns 16 g .. 16 g + 15, g < ceil(n / 16): what MllRowScale takes.
struct MllResidualNorm {
    float* h;                  // [m][n]
    const float* norm_weight;  // [n]
    void* x_out;               // bfloat16 [m][n]
    float* sumsq_out;          // [m][sumsq_stride]; the first ceil(n / 16) of a row are written
    int sumsq_stride;
};
int mll_gemm_skinny_residual(const void* a, const void* w_packed, int m, int n, int k, const MllResidualNorm* residual,
                             const MllRowScale* scale, hipStream_t stream);

// What the kernel takes beside the product's operands (internal to the library's launches).
struct MllSkinnyExtras {
    MllQkvStore store;
    MllRowScale scale;
    MllResidualNorm residual;
};

// The same product for up to 64 rows with the activations shared through LDS by the waves of a workgroup
// (faster than mll_gemm_skinny from 17 rows on). A wave takes tiles_per_wave (1 or 2) tiles of W. With
// splits > 1 (epilogue 0 only) k is cut into that many ranges and out is [splits][m][n]: partial sums that the
// caller adds in order. The order of additions is fixed by (n, k, splits).
int mll_gemm_medium(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                    int tiles_per_wave, int waves, int splits, hipStream_t stream);

// The same product for many rows: 256 x 256 tiles of C per workgroup, pieces of A and W brought into LDS by
// direct global-to-LDS loads. A is row-major [m, k] with k a multiple of 32; epilogues 0, 1 and 2 of
// mll_gemm_skinny. With epilogue 0, `splits` > 1 deals the stages of 64 of k to that many workgroups per tile:
// out is then [splits, m, n] partial sums for the caller to add in order. For weights that are kept in the packed
// order alone.
// tile_rows: the rows of a workgroup's tile of the result, 256, 192, 160 or 128, or 0 for mll_tiled_tile_rows's
// choice; the result's bits do not depend on it.
int mll_gemm_tiled(const void* a, const void* w_packed, void* out, int epilogue, int m, int n, int k,
                   int splits, int tile_rows, hipStream_t stream);
int mll_tiled_tile_rows(int m, int n, int splits);
// Queries, keys and values of many rows: the tiled product finished as mll_gemm_skinny_qkv finishes its own (the
// same MllQkvStore, the weight in rotary pair order). k a multiple of 32, store->n_freq even, no rows' factors; a
// workgroup owns a whole tile of the result and the reduction is never taken in parts.
int mll_gemm_tiled_qkv(const void* a, const void* w_packed, int m, int k, const MllQkvStore* store, int tile_rows,
                       hipStream_t stream);

// Calibration: a kernel that reads `bytes` of memory once with `blocks` workgroups, and one in which every wave of
// `blocks` workgroups of 4 issues iterations * 16 independent v_mfma_f32_16x16x32_bf16 (16384 flops each). The caller
// times them. `sink` is 4 bytes of device memory that are never written with ordinary data.
int mll_measure_read(const void* data, int64_t bytes, void* sink, int blocks, hipStream_t stream);
int mll_measure_mfma(int iterations, void* sink, int blocks, hipStream_t stream);

// Index of the first maximum of each row; a row that holds a non-finite value gives -1.
// `parts` is device scratch of n_rows * mll_argmax_slices(vocab) * 16 bytes (contents need not be cleared).
int mll_argmax(const float* logits, int32_t* out, void* parts, int n_rows, int vocab, hipStream_t stream);
int mll_argmax_slices(int vocab);

// mll_argmax for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc). It has no counterpart in the reference. The slices' scratch is a static
// array in device memory of MLL_ARGMAX_STATIC_MAX_PARTS * 16 bytes (1 MiB), one per GPU, held until the process
// ends; the call allocates and frees nothing. It refuses n_rows * mll_argmax_slices(vocab) beyond
// MLL_ARGMAX_STATIC_MAX_PARTS (at 64 slices, vocabularies from 129 025 tokens on: 1024 rows). The GPU whose
// scratch is used is the current one, which must be the stream's; the first call on a GPU looks the array's
// address up (make that call outside a graph capture). All calls on one GPU share the array: calls that overlap
// on one GPU (two streams, two threads) race; calls on one stream do not. The array keeps the last call's
// contents and needs no clearing: each call writes every entry it reads.
#define MLL_ARGMAX_STATIC_MAX_PARTS 65536
int mll_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, hipStream_t stream);

// Draws one token per row from softmax(logits / temperature) restricted to the top_k largest
// logits (top_k <= 0: all; ties at the k-th value go to the lower token ids), by inverse CDF in
// token order with the given uniform in [0, 1). temperature == 0 or top_k == 1 gives the
// argmax. A non-finite logit gives -1. top_k may be null (no row is restricted: the search for the
// k-th value is left out). `workspace`: mll_sample_workspace(n_rows, vocab) bytes of device scratch,
// 4-byte aligned; its contents need not be cleared.
int mll_sample(const float* logits, const float* temperature, const int32_t* top_k,
               const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab,
               hipStream_t stream);
int64_t mll_sample_workspace(int n_rows, int vocab);

// What the MFMA attention kernels take beyond scale and window (the *_extra entry points; null: nothing of it):
// bias: float32 [longest + 1][heads], added to the scaled score of key j for a query at p as
// bias[min(p - j, longest)][head] (null: none); sink: float32 [heads], exp(sink[head]) is one more term of the
// softmax's denominator, without key or value (null: none); the result is multiplied by out_scale, and its rows
// lie out_stride elements apart (at least heads * head_dim: it may be columns of a wider buffer).
typedef struct MllAttentionExtras {
    const float* bias;
    int longest;
    const float* sink;
    float out_scale;
    int64_t out_stride;
    int chunk;              // > 0 (and no window): a query at p sees the keys from floor(p / chunk) * chunk on
    const float* gate;      // null, or float32 rows gate_stride apart, one number a head: the head's result times sigmoid(gate[t][head])
    int64_t gate_stride;
} MllAttentionExtras;

int mll_paged_attention_decode_extra(const void* q, const void* k_cache, const void* v_cache,
                                     const int32_t* block_table, int table_width, const int32_t* seq_of_token,
                                     const int32_t* positions, const int32_t* token_ids, void* out, float* part_o,
                                     float* part_ml, float scale, int window, int n_tokens, int heads, int kv_heads,
                                     int head_dim, int page_size, int n_splits, const MllAttentionExtras* extras,
                                     hipStream_t stream);
int mll_paged_attention_prefill_extra(const void* q, const void* k_cache, const void* v_cache,
                                      const int32_t* block_table, int table_width, const int32_t* tiles,
                                      int n_tiles, const int32_t* positions, void* out, float scale, int window,
                                      int heads, int kv_heads, int head_dim, int page_size, const MllAttentionExtras* extras,
                                      hipStream_t stream);

// ---- several copies of the residual stream, a norm with a mean, a sinusoidal position vector ----------------

// out[t, :] = table[ids[t], :] + wave(positions[t]) in float32, where entry 2i of the wave is
// sin(p * rates[i]) and entry 2i + 1 the cosine of the same angle (the angle in float64; rates: (width + 1) / 2 doubles).
int mll_embedding_sinusoid(const void* table, int table_dtype, const int32_t* ids, const int32_t* positions,
                           const double* rates, float* out, int n_tokens, int width, int vocab, hipStream_t stream);

// out[t, c, :] = in[t, :] for every copy c: float32 [n_tokens][copies][width].
int mll_stream_copies(const float* in, float* out, int n_tokens, int width, int copies, hipStream_t stream);

// x is float32 [rows][streams][width]. For i < n_rows, r = rows ? rows[i] : i:
//   if y:  d = sum of y's n_parts parts at row r (float32 [width], parts part_stride elements apart);
//          x'_t = sum_s mix[s * streams + t] * x_s + give[t] * d  for every t (mix null: x'_t = x_t + give[t] * d;
//          give null: ones); with write_x the new rows replace the old ones;
//   u = sum_t take[t] * x'_t  (take null: ones);
//   out[i] = (u - mean(u)) / sqrt(var(u) + eps) * weight, or with rms: u / sqrt(mean(u^2) + eps) * weight.
// out null: only the streams are written. out has element type `dtype`; mix, give, take and weight are float32.
int mll_stream_norm(float* x, const float* y, int n_parts, int64_t part_stride, const float* mix, const float* give,
                    const float* take, const int32_t* rows, const float* weight, float eps, int rms, void* out, int dtype,
                    int n_rows, int streams, int width, int write_x, hipStream_t stream);

// gate_up[t] = [gate (width) | up (width)] in float32: g = min(gate, limit), u = clamp(up, -limit, limit),
// out[t] = g * sigmoid(slope * g) * (u + 1) in `dtype`.
int mll_clamped_glu(const float* gate_up, void* out, int dtype, int n_tokens, int width, float limit, float slope,
                    hipStream_t stream);

// ---- attention with a bias by distance and a sink, keys and values of different widths in plain pages --------

// qkv[t] = [q (heads * key_dim) | k (kv_heads * key_dim) | v (kv_heads * value_dim)] in float32, perhaps in
// n_parts parts that are added in order. Queries and keys are divided by their root mean square over their head
// (+ eps inside the root) if `normed`, and multiplied by q_weight / k_weight [key_dim] (both null: no weight); `bias`
// (nullable, one number a column of a row) is added first; with queries_only a row holds queries alone and nothing
// is stored; queries are then
// multiplied by 1 + temp_coef * ln((p + 1) / temp_every + 1) (whole-number division) at position p
// (temp_coef 0: not). Queries go to q_out [t][heads][key_dim]; keys and values into the pages
// [slot][kv_head][dim] at slot_mapping[t] (negative: not stored), or, with tiled_page_size > 0 (the positions of a
// page; key_dim == value_dim), into pages in the MFMA kernels' order (cache_layout.h).
// Rows of qkv lie row_stride floats apart (they may hold further columns after the values). With cos_sin (float32
// [n_tokens][rot_dims / 2][cos, sin]) queries and keys are turned after their norm: channel i < rot_dims / 2 of a head
// with channel i + rot_dims / 2, (u, v) -> (u cos - v sin, v cos + u sin); the other channels pass.
int mll_qk_norm_store(const float* qkv, int n_parts, int64_t part_stride, const float* q_weight, const float* k_weight,
                      float eps, const int32_t* positions, const int32_t* slot_mapping, float temp_coef, int temp_every,
                      void* q_out, void* k_pages, void* v_pages, int dtype, int n_tokens, int heads, int kv_heads, int key_dim,
                      int value_dim, int tiled_page_size, const float* bias, int normed, int queries_only, int64_t row_stride,
                      const float* cos_sin, int rot_dims, hipStream_t stream);

// Causal attention of every token over its request's pages: score_j = (q . k_j) * scale + bias[min(p - j, longest)][head]
// (bias null: none; float32 [longest + 1][heads]) - slopes[head] * (p - j) (slopes null: none); softmax over j <= p
// (with window > 0: p - window < j <= p) with exp(sink[head]) added to the denominator
// (sink null: not); out[t][head] = out_scale * sum_j weight_j v_j, rows out_stride elements apart.
// A token whose seq_of_token is negative is skipped. The order of every sum depends on p alone.
// With chunk > 0 (and no window) a query at p sees the keys from floor(p / chunk) * chunk on. With gate (float32, rows
// gate_stride apart, one number a head) the head's result is multiplied by sigmoid(gate[t][head]).
int mll_bias_attention(const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table, int table_width,
                       const int32_t* seq_of_token, const int32_t* positions, const float* bias, int longest,
                       const float* sink, void* out, int64_t out_stride, int dtype, int n_tokens, int heads, int kv_heads,
                       int key_dim, int value_dim, int page_size, float scale, float out_scale, const float* slopes, int window,
                       int chunk, const float* gate, int64_t gate_stride, hipStream_t stream);

// ---- gated linear attention --------------------------------------------------------------------------------

// decay[t][c] = sigmoid(z)^(1 / tau), z = bias[c] + sum_r a2[c][r] * proj[t][low_offset + r]; float32 but a2.
int mll_gla_decay(const float* proj, int64_t proj_stride, int low_offset, int rank, const void* a2, int a2_dtype,
                  const float* bias, float tau, float* decay, int n_tokens, int channels, hipStream_t stream);

// For every request i of the step, its tokens cu_tokens[i] .. cu_tokens[i + 1] - 1 in order, per head:
//   S = diag(decay_t) S + k_t v_t^T;  out[t][head] = S^T (q_t * q_scale)
// with S = state[slots[i]][head] (float32 [key_dim][value_dim]) read at the start and written at the end.
// q, k, v are float32 columns of proj's rows at the given offsets. A request without tokens is passed over.
// long_portions: the kernel that brings tiles of tokens through LDS (for steps with portions of many tokens); the
// same operations per token in the same order either way, so the same bits.
// decay: float32, token t's heads * key_dim numbers at decay + t * decay_stride (0: one row for every token).
int mll_gla_scan(const float* proj, int64_t proj_stride, int q_offset, int k_offset, int v_offset, const float* decay,
                 float* state, const int32_t* cu_tokens, const int32_t* slots, float* out, int n_seqs, int heads, int key_dim,
                 int value_dim, float q_scale, int long_portions, int64_t decay_stride, hipStream_t stream);

// out[t][head] = o[t][head] / rms(o[t][head]) * weight * silu(gate[t][head]) * out_scale, gate at gate_offset of
// proj's rows (weight null: none); out in `dtype`, rows out_stride elements apart.
int mll_gla_gate(const float* o, const float* proj, int64_t proj_stride, int gate_offset, const float* weight, float eps,
                 void* out, int64_t out_stride, int dtype, int n_tokens, int heads, int value_dim, float out_scale,
                 hipStream_t stream);

// ---- attention through latents (csrc/latent_attention.hip) ----------------------------------------------------

// proj[t] holds, in float32, the queries' down projection at q_at (q_rank wide; 0: the queries have no latent) and the keys' and values' at kv_at
// (kv_rank, then rot_dim). q_latent[t] = proj / rms * q_weight in `dtype`. With slot_mapping (null: the layer stores
// nothing): the first kv_rank entries / rms * kv_weight and the last rot_dim turned by the split-half rule with
// cos_sin [t][rot_dim / 2][2] go to slot slot_mapping[t] (negative: not stored) of `pages` [slot][kv_rank + rot_dim],
// or, with tiled_page_size > 0, of k_pages and v_pages (one kv head of kv_rank + rot_dim dims, cache_layout.h): the
// same row as key and as value.
int mll_latent_prepare(const float* proj, int64_t proj_stride, int q_at, int q_rank, const float* q_weight, int kv_at,
                       int kv_rank, int rot_dim, const float* kv_weight, float eps, const float* cos_sin,
                       const int32_t* slot_mapping, void* q_latent, void* pages, void* k_pages, void* v_pages,
                       int tiled_page_size, int dtype, int n_tokens, hipStream_t stream);

// q: float32 [t][head][dim | rot_dim], rows q_stride elements apart. q_full [t][head][kv_rank | rot_dim] in `dtype` gets the rotated part turned;
// `folded` ([head][t][kv_rank], nullable) is copied in front of it; `flat_out` ([head][t][dim], nullable) receives
// the unrotated part.
int mll_latent_query(const float* q, int64_t q_stride, int n_tokens, int heads, int dim, int rot_dim, int kv_rank, const float* cos_sin,
                     const void* folded, void* flat_out, void* q_full, int dtype, hipStream_t stream);

// out[t][h][o] = sum_i x[t][h][i] * w[h][i][o] (* sigmoid(gate[t][h * n_out + o]) with gate, float32 rows gate_stride
// apart; with gate_a_head one gate a head: gate[t][h]), sums float32 in ascending i. Strides in elements. Built for (x, w, out) = (f32, f32, f32), (f32, bf16, bf16),
// (bf16, bf16, bf16), (f32, bf16, f32).
int mll_head_product(const void* x, int x_dtype, int64_t x_token_stride, int64_t x_head_stride, const void* w, int w_dtype,
                     void* out, int out_dtype, int64_t out_token_stride, int64_t out_head_stride, const float* gate,
                     int64_t gate_stride, int gate_a_head, int n_tokens, int heads, int n_in, int n_out, hipStream_t stream);

// out[t][h * n + c] = in[h][t][c] (* sigmoid(gate[t][h * n + c]) with gate, float32 rows gate_stride apart; with
// gate_a_head sigmoid(gate[t][h])); in and out in `dtype`.
int mll_gate_heads(const void* in, const float* gate, int64_t gate_stride, int gate_a_head, void* out, int dtype, int n_tokens,
                   int heads, int n, hipStream_t stream);

// For every token and head: softmax over the keys j in (p - window, p] (window <= 0: all j <= p) of
// (q_full[t][h] . pages[slot_j]) * scale, out[t][h] = sum_j weight_j pages[slot_j][:kv_rank]. A token whose
// seq_of_token is negative is skipped. The order of every sum depends on p and the window alone.
int mll_latent_attention(const void* q_full, const void* pages, const int32_t* block_table, int table_width,
                         const int32_t* seq_of_token, const int32_t* positions, void* out, int64_t out_token_stride,
                         int64_t out_head_stride, int dtype, int n_tokens, int heads, int kv_rank, int rot_dim, int page_size,
                         int window, float scale, hipStream_t stream);

// ---- the gated delta rule (csrc/delta_rule.hip) ------------------------------------------------------------------

// Channels: key_heads query heads of key_dim, key_heads key heads of key_dim, heads value heads of value_dim, in this
// order, at conv_at of proj's rows. u[t][c] = silu(sum_j taps[c][j] * input(t - (n_taps - 1 - j), c)), the input being
// proj's for the step's tokens of the same request and the request's kept inputs (kept [slot][n_taps - 1][channels],
// newest last) before them; query and key heads are then divided by sqrt(sum of squares + unit_eps), queries also
// multiplied by q_factor. gates[t][2 h] = sigmoid(proj[t][beta_at + h]), gates[t][2 h + 1] = exp(-exp(a_log[h]) *
// softplus(proj[t][step_at + h] + dt_bias[h])). All float32.
int mll_delta_prepare(const float* proj, int64_t proj_stride, int conv_at, const float* taps, const float* kept,
                      const int32_t* seq_of_token, const int32_t* cu_tokens, const int32_t* slots, int beta_at, int step_at,
                      const float* a_log, const float* dt_bias, float* u, float* gates, int n_tokens, int key_heads, int heads,
                      int key_dim, int value_dim, int n_taps, float q_factor, float unit_eps, hipStream_t stream);

// kept[slot] <- the newest n_taps - 1 rows of proj[.][conv_at ..] of every request, older kept rows before them where
// the step brought fewer.
int mll_conv_keep(const float* proj, int64_t proj_stride, int conv_at, float* kept, const int32_t* cu_tokens,
                  const int32_t* slots, int n_seqs, int channels, int n_taps, hipStream_t stream);

// Per request and head, over the request's tokens in order, with S = state[slot][head] ([key_dim][value_dim], read
// first, written last): S *= g; c = beta * (v - S^T k); S += k c^T; out[t][head] = S^T q. u and gates as above.
// long_portions: the kernel that stages tiles of tokens through LDS, for steps whose requests bring many tokens (the
// same bits).
int mll_delta_scan(const float* u, const float* gates, float* state, const int32_t* cu_tokens, const int32_t* slots, float* out,
                   int n_seqs, int key_heads, int heads, int key_dim, int value_dim, int long_portions, hipStream_t stream);

// ---- a recurrent block with a gated linear recurrence (csrc/recurrent.hip) ----------------------------------------

// u[t][c] = conv_bias[c] + sum_j taps[c][j] * input(t - (n_taps - 1 - j), c), input = proj[.][x_at + c] + x_bias[c] for
// the step's tokens of the same request, the request's kept inputs (kept [slot][n_taps - 1][width], newest last)
// before them. Biases nullable. taps in taps_dtype.
int mll_rglru_conv(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, const void* taps, int taps_dtype,
                   const float* conv_bias, const float* kept, const int32_t* seq_of_token, const int32_t* cu_tokens,
                   const int32_t* slots, float* u, int n_tokens, int width, int n_taps, hipStream_t stream);

// Per request and channel, over the request's tokens in order: r = sigmoid(gates[t][b][c'] + r_bias), i =
// sigmoid(gates[t][b][size + c'] + i_bias) (gates: float32 [t][blocks][2 * size]), a = exp(-decay_scale * r *
// softplus(lam)), S = a S + sqrt(1 - a^2) * i * u; out[t][c] = S * gelu_tanh(proj[t][y_at + c] + y_bias[c]) in `dtype`.
// S = state[slot][c] is read first and written last, and `kept` receives the convolution's newest inputs.
int mll_rglru_scan(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, int y_at, const float* y_bias,
                   const float* u, const float* gates, const float* r_bias, const float* i_bias, const float* lam,
                   float decay_scale, float* state, float* kept, const int32_t* cu_tokens, const int32_t* slots, void* out,
                   int dtype, int n_seqs, int width, int blocks, int n_taps, hipStream_t stream);

// ---- a mixture of experts (csrc/moe.hip) ------------------------------------------------------------------------

// ids[t][n], weights[t][n] for n < top: the experts with the largest scores (sigmoid, or softmax over the experts)
// of z[t][0 .. experts), ties to the lower index; weights are the scores, divided by their sum with renormalize.
// shared_at >= 0: shared_gate[t] = sigmoid(z[t][shared_at]).
// groups > 0: the experts form that many equal groups of neighbours; a group's score is its largest, and only experts of
// the `keep` best groups (ties: the lower) are chosen.
int mll_moe_route(const float* z, int64_t z_stride, int n_tokens, int experts, int top, int softmax_scores, int renormalize,
                  int shared_at, int32_t* ids, float* weights, float* shared_gate, int groups, int keep, hipStream_t stream);

// act[t * top + n] = silu(Wg_e xs) * (Wu_e xs), e = ids[t][n], xs = x[t] * weights[t][n] rounded to `dtype`
// (weight_on_input) or x[t]; gate_up [experts][2 * ff][width] with the gate rows first.
// gated 0: gate_up is [experts][ff][width] and act = activation(Wu_e xs). activation: 0 SiLU, 1 gelu (erf), 2 gelu (tanh).
int mll_moe_gate_up(const void* x, const int32_t* ids, const float* weights, int top, const void* gate_up, void* act,
                    int dtype, int n_tokens, int width, int ff, int weight_on_input, int gated, int activation,
                    hipStream_t stream);

// out[n][t] = Wd_e act[t * top + n] (* weights[t][n] unless weight_on_input): float32 [top][n_tokens][width].
int mll_moe_down(const void* act, const int32_t* ids, const float* weights, int top, const void* down, float* out, int dtype,
                 int n_tokens, int width, int ff, int weight_on_input, hipStream_t stream);

// The same for n_tokens tokens of an output whose parts hold part_tokens rows each (a launch for some of a step's tokens).
int mll_moe_down_rows(const void* act, const int32_t* ids, const float* weights, int top, const void* down, float* out, int dtype,
                      int n_tokens, int part_tokens, int width, int ff, int weight_on_input, hipStream_t stream);

// out[t] = factor[t] * (in[0][t] + in[1][t] + ...), float32; parts part_stride elements apart.
int mll_scale_rows(const float* in, int n_parts, int64_t part_stride, const float* factor, float* out, int n_tokens, int width,
                   hipStream_t stream);

// The same as mll_moe_gate_up and mll_moe_down together for many bfloat16 pairs: the pairs are sorted by expert (counts
// [experts], offsets [experts + 1], order [n_tokens * top]: int32 scratch), their inputs gathered into `sorted`
// ([pairs][width]), and every expert multiplies its rows in tiles on the matrix units; `act` is [pairs][ff] scratch.
// width and ff are multiples of 8.
int mll_moe_grouped(const void* x, const int32_t* ids, const float* weights, int top, const void* gate_up, const void* down,
                    int32_t* counts, int32_t* offsets, int32_t* order, void* sorted, void* act, float* out, int n_tokens,
                    int experts, int width, int ff, int weight_on_input, int gated, int activation, hipStream_t stream);

// mll_rglru_scan for steps with long portions: the recurrence in chunks of 64 tokens (every chunk walked from zero,
// the state carried from chunk to chunk, every chunk walked again from its start), the same result but for the
// rounding of the chunks' products. `scratch`: mll_rglru_scan_scratch(n_tokens, n_seqs, width) floats.
int mll_rglru_scan_chunked(const float* proj, int64_t proj_stride, int x_at, const float* x_bias, int y_at, const float* y_bias,
                           const float* u, const float* gates, const float* r_bias, const float* i_bias, const float* lam,
                           float decay_scale, float* state, float* kept, const int32_t* cu_tokens, const int32_t* slots, void* out,
                           float* scratch, int dtype, int n_tokens, int n_seqs, int width, int blocks, int n_taps, hipStream_t stream);
int64_t mll_rglru_scan_scratch(int n_tokens, int n_seqs, int width);

// z[t][e] = w[e] . x[t] in float32: x in `dtype`, w float32 [n_out][width] (a router's logits).
int mll_router_logits(const void* x, int dtype, const float* w, float* z, int n_tokens, int n_out, int width, hipStream_t stream);

}  // extern "C"
