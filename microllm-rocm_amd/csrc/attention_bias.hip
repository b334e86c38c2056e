// Causal attention whose scores carry a bias by distance and whose softmax may have a sink, over keys and values
// of different widths in plain pages.
//
// Pages: keys [page, position, kv_head, key_dim], values [page, position, kv_head, value_dim]. A score is
// (q . k_j) * scale + bias[min(p - j, longest), head]; the bias table has one row per distance up to `longest`,
// which stands for every longer one. A sink is one more term exp(sink[head]) in the softmax's denominator, with
// no key and no value: the running maximum starts at the sink and the running sum at 1.
//
// One wave takes a (token, head). Keys are walked in tiles of 64 at absolute positions: each lane forms the score
// of one key, the tile's maximum and weights follow, and then the lanes turn to the value's channels and add the
// 64 weighted values in key order. The order of every sum depends on the query's position alone, so a row does
// not change with the step's cut, the batch or the pages. Scores, weights and sums are float32.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kBiasKeyTile = 64;
constexpr int kMaxValueChannelsALane = 4;     // value_dim up to 256

template <typename T> __device__ inline float dot_row(const T* key, const float* q, int dim);

template <> __device__ inline float dot_row<float>(const float* key, const float* q, int dim) {
    float sum = 0.0f;
    int c = 0;
    if ((dim & 3) == 0 && (reinterpret_cast<uintptr_t>(key) & 15) == 0) {
        for (; c < dim; c += 4) {
            const float4 k = *reinterpret_cast<const float4*>(key + c);
            sum = fmaf(k.x, q[c], sum);
            sum = fmaf(k.y, q[c + 1], sum);
            sum = fmaf(k.z, q[c + 2], sum);
            sum = fmaf(k.w, q[c + 3], sum);
        }
        return sum;
    }
    for (; c < dim; ++c) sum = fmaf(key[c], q[c], sum);
    return sum;
}

template <> __device__ inline float dot_row<bf16>(const bf16* key, const float* q, int dim) {
    float sum = 0.0f;
    int c = 0;
    if ((dim & 7) == 0 && (reinterpret_cast<uintptr_t>(key) & 15) == 0) {
        for (; c < dim; c += 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(key + c);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float low = __builtin_bit_cast(float, words[w] << 16);
                const float high = __builtin_bit_cast(float, words[w] & 0xffff0000u);
                sum = fmaf(low, q[c + 2 * w], sum);
                sum = fmaf(high, q[c + 2 * w + 1], sum);
            }
        }
        return sum;
    }
    for (; c < dim; ++c) sum = fmaf(to_float(key[c]), q[c], sum);
    return sum;
}

template <typename T>
__global__ void __launch_bounds__(kWave)
bias_attention_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                      const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ seq_of_token,
                      const int32_t* __restrict__ positions, const float* __restrict__ bias, int longest,
                      const float* __restrict__ sink, T* __restrict__ out, int64_t out_stride, int heads, int kv_heads,
                      int key_dim, int value_dim, int page_size, float scale, float out_scale,
                      const float* __restrict__ slopes, int window, int chunk, const float* __restrict__ gate,
                      int64_t gate_stride) {
    extern __shared__ float q_row[];
    const int token = blockIdx.x / heads;
    const int head = blockIdx.x % heads;
    const int seq = seq_of_token[token];
    if (seq < 0) return;       // a row that pads the step
    const int lane = threadIdx.x;
    const int position = positions[token];
    const int kv_head = head / (heads / kv_heads);
    const T* query = q + (static_cast<int64_t>(token) * heads + head) * key_dim;
    for (int c = lane; c < key_dim; c += kWave) q_row[c] = to_float(query[c]);
    __syncthreads();
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    float running_max = sink ? sink[head] : -INFINITY;
    float running_sum = sink ? 1.0f : 0.0f;
    float acc[kMaxValueChannelsALane] = {0.0f, 0.0f, 0.0f, 0.0f};
    const int64_t key_row = static_cast<int64_t>(kv_heads) * key_dim;
    const int64_t value_row = static_cast<int64_t>(kv_heads) * value_dim;
    const float slope = slopes ? slopes[head] : 0.0f;
    // the oldest key seen: the first of the query's chunk of positions, or what the window reaches back to
    const int low = chunk > 0 ? position / chunk * chunk : (window > 0 ? max(0, position - window + 1) : 0);
    for (int first = low / kBiasKeyTile * kBiasKeyTile; first <= position; first += kBiasKeyTile) {
        const int j = first + lane;
        float score = -INFINITY;
        int64_t place = 0;
        const bool seen = j >= low && j <= position;
        if (seen) {
            place = static_cast<int64_t>(table[j / page_size]) * page_size + j % page_size;
            const T* key = k_pages + place * key_row + static_cast<int64_t>(kv_head) * key_dim;
            score = dot_row<T>(key, q_row, key_dim) * scale;
            if (bias) score += bias[static_cast<int64_t>(min(position - j, longest)) * heads + head];
            if (slopes) score -= slope * static_cast<float>(position - j);
        }
        const float tile_max = wave_max(score);
        const float new_max = fmaxf(running_max, tile_max);
        const float keep = running_max == -INFINITY ? 0.0f : expf(running_max - new_max);
        const float weight = seen ? expf(score - new_max) : 0.0f;
        running_sum = running_sum * keep + wave_sum(weight);
        running_max = new_max;
#pragma unroll
        for (int m = 0; m < kMaxValueChannelsALane; ++m) acc[m] *= keep;
        const int in_tile = min(kBiasKeyTile, position - first + 1);
        for (int n = max(0, low - first); n < in_tile; ++n) {
            const float w = __shfl(weight, n, kWave);
            const int64_t at = __shfl(place, n, kWave);
            const T* value = v_pages + at * value_row + static_cast<int64_t>(kv_head) * value_dim;
#pragma unroll
            for (int m = 0; m < kMaxValueChannelsALane; ++m) {
                const int c = lane + m * kWave;
                if (c < value_dim) acc[m] = fmaf(w, to_float(value[c]), acc[m]);
            }
        }
    }
    float factor = out_scale / running_sum;
    if (gate) factor *= 1.0f / (1.0f + expf(-gate[static_cast<int64_t>(token) * gate_stride + head]));
    T* to = out + static_cast<int64_t>(token) * out_stride + static_cast<int64_t>(head) * value_dim;
#pragma unroll
    for (int m = 0; m < kMaxValueChannelsALane; ++m) {
        const int c = lane + m * kWave;
        if (c < value_dim) to[c] = from_float<T>(acc[m] * factor);
    }
}

// One wave a (token, head of q, k or v): the norm of queries and keys over their head, the queries' factor by
// position, and the write of keys and values into their pages.
template <typename T>
__global__ void __launch_bounds__(kWave)
qk_norm_store_kernel(const float* __restrict__ qkv, int n_parts, int64_t part_stride, const float* __restrict__ q_weight,
                     const float* __restrict__ k_weight, float eps, const int32_t* __restrict__ positions,
                     const int32_t* __restrict__ slot_mapping, float temp_coef, int temp_every, T* __restrict__ q_out,
                     T* __restrict__ k_pages, T* __restrict__ v_pages, int heads, int kv_heads, int key_dim, int value_dim,
                     int tiled_page_size, const float* __restrict__ bias, int normed, int queries_only, int64_t row_stride,
                     const float* __restrict__ cos_sin, int rot_dims) {
    const int vectors = queries_only ? heads : heads + 2 * kv_heads;
    const int token = blockIdx.x / vectors;
    const int which = blockIdx.x % vectors;
    const int lane = threadIdx.x;
    const float* row = qkv + static_cast<int64_t>(token) * row_stride;
    const bool is_q = which < heads, is_k = !is_q && which < heads + kv_heads;
    const int head = is_q ? which : (is_k ? which - heads : which - heads - kv_heads);
    const int dim = (is_q || is_k) ? key_dim : value_dim;
    const int offset = is_q ? head * key_dim : (is_k ? (heads + head) * key_dim : (heads + kv_heads) * key_dim + head * value_dim);
    const int slot = is_q ? 0 : slot_mapping[token];
    if (!is_q && slot < 0) return;
    float squares = 0.0f;
    for (int c = lane; c < dim; c += kWave) {
        float value = row[offset + c];
        for (int part = 1; part < n_parts; ++part) value += row[part * part_stride + offset + c];
        if (bias) value += bias[offset + c];
        squares += value * value;
    }
    const float* weight = is_q ? q_weight : (is_k ? k_weight : nullptr);
    const bool norm = normed && (is_q || is_k);
    float factor = 1.0f;
    if (norm) factor = 1.0f / sqrtf(wave_sum(squares) / static_cast<float>(dim) + eps);
    if (is_q && temp_coef != 0.0f) {
        const int steps = (positions[token] + 1) / temp_every;
        factor *= 1.0f + temp_coef * static_cast<float>(log(static_cast<double>(steps) + 1.0));
    }
    T* to = is_q ? q_out + (static_cast<int64_t>(token) * heads + head) * key_dim
                 : (is_k ? k_pages + (static_cast<int64_t>(slot) * kv_heads + head) * key_dim
                         : v_pages + (static_cast<int64_t>(slot) * kv_heads + head) * value_dim);
    // tiled_page_size > 0: the pages are in the order the MFMA kernels read them (cache_layout.h; both widths equal)
    const bool tiled = tiled_page_size > 0 && !is_q;
    const CacheLayout layout(kv_heads, tiled ? tiled_page_size : 16, key_dim);
    const int64_t page = tiled ? slot / tiled_page_size : 0;
    const int in_page = tiled ? slot % tiled_page_size : 0;
    // what the vector holds at channel c before it is turned: the sums, the bias, the norm
    auto prepared = [&](int c) {
        float value = row[offset + c];
        for (int part = 1; part < n_parts; ++part) value += row[part * part_stride + offset + c];
        if (bias) value += bias[offset + c];
        return norm ? (weight ? value * factor * weight[c] : value * factor) : value;
    };
    // queries and keys turn by the token's position in their first rot_dims channels, channel i with i + rot_dims / 2
    const bool turns = cos_sin != nullptr && (is_q || is_k);
    const int half = rot_dims / 2;
    const float* angles = cos_sin + static_cast<int64_t>(token) * rot_dims;     // [rot_dims / 2][cos, sin]
    for (int c = lane; c < dim; c += kWave) {
        float value = prepared(c);
        if (turns && c < rot_dims) {
            const int pair = c < half ? c : c - half;
            const float other = prepared(c < half ? c + half : c - half);
            const float cosine = angles[2 * pair], sine = angles[2 * pair + 1];
            value = c < half ? value * cosine - other * sine : value * cosine + other * sine;
        }
        const T rounded = from_float<T>(value);
        if (tiled) {
            if (is_k) k_pages[layout.k_at(page, head, in_page, c)] = rounded;
            else v_pages[layout.v_at(page, head, in_page, c)] = rounded;
        } else {
            to[c] = rounded;
        }
    }
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_qk_norm_store(const float* qkv, int n_parts, int64_t part_stride, const float* q_weight, const float* k_weight,
                      float eps, const int32_t* positions, const int32_t* slot_mapping, float temp_coef, int temp_every,
                      void* q_out, void* k_pages, void* v_pages, int dtype, int n_tokens, int heads, int kv_heads, int key_dim,
                      int value_dim, int tiled_page_size, const float* bias, int normed, int queries_only, int64_t row_stride,
                      const float* cos_sin, int rot_dims, hipStream_t stream) {
    MLL_REQUIRE(tiled_page_size == 0 || (tiled_page_size > 0 && tiled_page_size % 16 == 0 && key_dim == value_dim),
                "qk_norm_store: tiled pages hold a multiple of 16 positions and keys and values of one width");
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0, "qk_norm_store: sizes must be positive");
    MLL_REQUIRE(n_parts >= 1, "qk_norm_store: at least one part");
    MLL_REQUIRE(row_stride >= (queries_only ? heads * key_dim : (heads + kv_heads) * key_dim + kv_heads * value_dim),
                "qk_norm_store: the rows are narrower than their queries, keys and values");
    MLL_REQUIRE(cos_sin == nullptr || (rot_dims > 0 && rot_dims % 2 == 0 && rot_dims <= key_dim),
                "qk_norm_store: an even number of turned channels, at most the head's");
    MLL_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qk_norm_store: norm weights for queries and keys, or for neither");
    MLL_REQUIRE(!normed || eps > 0.0f, "qk_norm_store: eps must be positive");
    MLL_REQUIRE(normed || q_weight == nullptr, "qk_norm_store: norm weights without a norm");
    MLL_REQUIRE(queries_only || (slot_mapping != nullptr && k_pages != nullptr && v_pages != nullptr), "qk_norm_store: keys and values need pages and slots");
    MLL_REQUIRE(temp_coef == 0.0f || temp_every > 0, "qk_norm_store: the factor by position needs a positive step");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * (queries_only ? heads : heads + 2 * kv_heads);
    MLL_REQUIRE(blocks < (1ll << 31), "qk_norm_store: too many rows for one launch");
    if (dtype == kF32) {
        qk_norm_store_kernel<float><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(
            qkv, n_parts, part_stride, q_weight, k_weight, eps, positions, slot_mapping, temp_coef, temp_every,
            static_cast<float*>(q_out), static_cast<float*>(k_pages), static_cast<float*>(v_pages), heads, kv_heads, key_dim, value_dim,
            tiled_page_size, bias, normed, queries_only, row_stride, cos_sin, rot_dims);
    } else if (dtype == kBF16) {
        qk_norm_store_kernel<bf16><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(
            qkv, n_parts, part_stride, q_weight, k_weight, eps, positions, slot_mapping, temp_coef, temp_every,
            static_cast<bf16*>(q_out), static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), heads, kv_heads, key_dim, value_dim,
            tiled_page_size, bias, normed, queries_only, row_stride, cos_sin, rot_dims);
    } else {
        return fail("qk_norm_store: unknown dtype");
    }
    return check_launch("qk_norm_store");
}

int mll_bias_attention(const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table, int table_width,
                       const int32_t* seq_of_token, const int32_t* positions, const float* bias, int longest,
                       const float* sink, void* out, int64_t out_stride, int dtype, int n_tokens, int heads, int kv_heads,
                       int key_dim, int value_dim, int page_size, float scale, float out_scale, const float* slopes, int window,
                       int chunk, const float* gate, int64_t gate_stride, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0 && page_size > 0 && table_width > 0,
                "bias_attention: sizes must be positive");
    MLL_REQUIRE(heads % kv_heads == 0, "bias_attention: heads must divide into kv heads");
    MLL_REQUIRE(value_dim <= kMaxValueChannelsALane * kWave, "bias_attention: value heads wider than 256 are not supported");
    MLL_REQUIRE(bias == nullptr || longest >= 0, "bias_attention: the bias table needs at least one row");
    MLL_REQUIRE(out_stride >= static_cast<int64_t>(heads) * value_dim, "bias_attention: the output rows overlap");
    MLL_REQUIRE(window >= 0 && chunk >= 0 && !(window > 0 && chunk > 0), "bias_attention: a window or chunks of positions, not both");
    MLL_REQUIRE(gate == nullptr || gate_stride >= heads, "bias_attention: one gate a head in every row");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * heads;
    MLL_REQUIRE(blocks < (1ll << 31), "bias_attention: too many rows for one launch");
    const size_t lds = static_cast<size_t>(key_dim) * sizeof(float);
    MLL_REQUIRE(lds <= 64 * 1024, "bias_attention: key heads wider than 16384 are not supported");
    if (dtype == kF32) {
        bias_attention_kernel<float><<<static_cast<unsigned>(blocks), kWave, lds, stream>>>(
            static_cast<const float*>(q), static_cast<const float*>(k_pages), static_cast<const float*>(v_pages), block_table,
            table_width, seq_of_token, positions, bias, longest, sink, static_cast<float*>(out), out_stride, heads, kv_heads,
            key_dim, value_dim, page_size, scale, out_scale, slopes, window, chunk, gate, gate_stride);
    } else if (dtype == kBF16) {
        bias_attention_kernel<bf16><<<static_cast<unsigned>(blocks), kWave, lds, stream>>>(
            static_cast<const bf16*>(q), static_cast<const bf16*>(k_pages), static_cast<const bf16*>(v_pages), block_table,
            table_width, seq_of_token, positions, bias, longest, sink, static_cast<bf16*>(out), out_stride, heads, kv_heads,
            key_dim, value_dim, page_size, scale, out_scale, slopes, window, chunk, gate, gate_stride);
    } else {
        return fail("bias_attention: unknown dtype");
    }
    return check_launch("bias_attention");
}

}  // extern "C"
