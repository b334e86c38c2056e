// Attention through latents: what a token leaves in the cache is one normed latent vector and one rotated key
// part that all heads share; keys and values of a head are projections of the latent. The projections are folded
// into the query and into the result (q' = Wk_h^T q_h, o_h = Wv_h sum_j p_j c_j), so that the attention itself has
// one "kv head" whose key is [latent | rotated part] and whose value is the latent:
//
//   score_j = (q'_h . c_j + qrot_h . krot_j) * scale,   j in (p - window, p],   o'_h = sum_j softmax_j c_j.
//
// Kernels here: the norms of both latents with the rotation and the page write; the queries' rotation and their
// joining with q'; a product per head with weights [head][in][out]; and the attention over plain pages
// [slot][latent + rot] with one wave a (token, head), which serves every dtype and size (bfloat16 with a row of a
// multiple of 16 up to 256 elements goes through the paged attention's own pages and MFMA kernels instead).
// Norm statistics, angles, scores, softmax and every sum are float32.
#include "cache_layout.h"
#include "common.h"
#include "microllm_hip.h"

namespace mll {

// ---- both latents of a token: norm, rotation, page write ---------------------------------------------------------
// One workgroup a (token, which): which 0 is the queries' latent, which 1 the keys' and values'.
constexpr int kPrepareThreads = 256;

template <typename T>
__global__ void __launch_bounds__(kPrepareThreads)
latent_prepare_kernel(const float* __restrict__ proj, int64_t proj_stride, int q_at, int q_rank, const float* __restrict__ q_weight,
                      int kv_at, int kv_rank, int rot_dim, const float* __restrict__ kv_weight, float eps,
                      const float* __restrict__ cos_sin, const int32_t* __restrict__ slot_mapping, T* __restrict__ q_latent,
                      T* __restrict__ pages, T* __restrict__ k_pages, T* __restrict__ v_pages, int tiled_page_size) {
    __shared__ float scratch[16];
    const int token = blockIdx.x / 2, which = blockIdx.x % 2;
    const int thread = threadIdx.x;
    const float* row = proj + static_cast<int64_t>(token) * proj_stride;
    if (which == 0) {
        if (q_rank <= 0) return;        // the queries have no latent of their own
        float squares = 0.0f;
        for (int c = thread; c < q_rank; c += kPrepareThreads) squares = fmaf(row[q_at + c], row[q_at + c], squares);
        const float factor = 1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(q_rank) + eps);
        for (int c = thread; c < q_rank; c += kPrepareThreads)
            q_latent[static_cast<int64_t>(token) * q_rank + c] = from_float<T>(row[q_at + c] * factor * q_weight[c]);
        return;
    }
    if (slot_mapping == nullptr) return;       // a layer that borrows another's latents stores nothing
    const int slot = slot_mapping[token];
    if (slot < 0) return;
    const int width = kv_rank + rot_dim;
    const bool tiled = tiled_page_size > 0;
    const CacheLayout layout(1, tiled ? tiled_page_size : 16, width);
    const int64_t page = tiled ? slot / tiled_page_size : 0;
    const int in_page = tiled ? slot % tiled_page_size : 0;
    auto store = [&](int c, float value) {
        const T rounded = from_float<T>(value);
        if (tiled) {
            k_pages[layout.k_at(page, 0, in_page, c)] = rounded;
            v_pages[layout.v_at(page, 0, in_page, c)] = rounded;
        } else {
            pages[static_cast<int64_t>(slot) * width + c] = rounded;
        }
    };
    float squares = 0.0f;
    for (int c = thread; c < kv_rank; c += kPrepareThreads) squares = fmaf(row[kv_at + c], row[kv_at + c], squares);
    const float factor = 1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(kv_rank) + eps);
    for (int c = thread; c < kv_rank; c += kPrepareThreads) store(c, row[kv_at + c] * factor * kv_weight[c]);
    const int half = rot_dim / 2;
    const float* turn = row + kv_at + kv_rank;
    for (int i = thread; i < half; i += kPrepareThreads) {
        const float c = cos_sin[(static_cast<int64_t>(token) * half + i) * 2], s = cos_sin[(static_cast<int64_t>(token) * half + i) * 2 + 1];
        store(kv_rank + i, rotate_first(turn[i], turn[i + half], c, s));
        store(kv_rank + i + half, rotate_second(turn[i], turn[i + half], c, s));
    }
}

// ---- queries: q [token][head][dim | rot] float32 -> q_full [token][head][kv_rank | rot] ---------------------------
// One wave a (token, head). The rotated part is turned and written behind the folded part; `folded` (the folded part
// [head][token][kv_rank] from a batched product, nullable) is copied in front of it; `flat_out` (nullable) receives
// the unrotated part as [head][token][dim] for such a product.
template <typename T>
__global__ void __launch_bounds__(kWave)
latent_query_kernel(const float* __restrict__ q, int64_t q_stride, int n_tokens, int heads, int dim, int rot_dim, int kv_rank,
                    const float* __restrict__ cos_sin, const T* __restrict__ folded, T* __restrict__ flat_out,
                    T* __restrict__ q_full) {
    const int token = blockIdx.x / heads, head = blockIdx.x % heads;
    const int lane = threadIdx.x;
    const float* row = q + static_cast<int64_t>(token) * q_stride + static_cast<int64_t>(head) * (dim + rot_dim);
    T* to = q_full + (static_cast<int64_t>(token) * heads + head) * (kv_rank + rot_dim);
    const int half = rot_dim / 2;
    for (int i = lane; i < half; i += kWave) {
        const float c = cos_sin[(static_cast<int64_t>(token) * half + i) * 2], s = cos_sin[(static_cast<int64_t>(token) * half + i) * 2 + 1];
        to[kv_rank + i] = from_float<T>(rotate_first(row[dim + i], row[dim + i + half], c, s));
        to[kv_rank + i + half] = from_float<T>(rotate_second(row[dim + i], row[dim + i + half], c, s));
    }
    if (folded != nullptr) {
        const T* from = folded + (static_cast<int64_t>(head) * n_tokens + token) * kv_rank;
        for (int c = lane; c < kv_rank; c += kWave) to[c] = from[c];
    }
    if (flat_out != nullptr) {
        T* flat = flat_out + (static_cast<int64_t>(head) * n_tokens + token) * dim;
        for (int c = lane; c < dim; c += kWave) flat[c] = from_float<T>(row[c]);
    }
}

// ---- a product per head: out[t][h][o] = sum_i x[t][h][i] * w[h][i][o] ----------------------------------------------
// A workgroup of four waves takes 64 outputs of one head for kHeadProductRows tokens. The tokens' inputs lie in LDS as
// float32, a tile of up to 1024 inputs at a time; wave s walks the s-th quarter of each tile (the bounds follow n_in
// alone) in ascending order and the four partial sums meet in wave order through LDS: a row's sums do not depend on
// its neighbours. The weight is stored [head][in][out]: the lanes of a wave read neighbouring outputs. Optionally the
// result is multiplied by sigmoid(gate[t][h * n_out + o]) (float32 rows, gate_stride apart).
constexpr int kHeadProductRows = 8;
constexpr int kHeadProductSlices = 4;
constexpr int kHeadProductTile = 1024;

// SLICES 4: four waves, one a quarter (steps of few rows: more loads on their way). SLICES 1: one wave walks the four
// quarters one after the other into sums of their own (steps of many rows: no exchange, less staging). The same
// terms are added in the same order either way, so a row's bits do not depend on the step it is in.
template <typename X, typename W, typename O, int SLICES>
__global__ void __launch_bounds__(SLICES * kWave)
head_product_kernel(const X* __restrict__ x, int64_t x_token_stride, int64_t x_head_stride, const W* __restrict__ w,
                    O* __restrict__ out, int64_t out_token_stride, int64_t out_head_stride, const float* __restrict__ gate,
                    int64_t gate_stride, int gate_a_head, int n_tokens, int heads, int n_in, int n_out) {
    extern __shared__ float x_rows[];      // [kHeadProductRows][tile], then [slices - 1][kHeadProductRows][64] partial sums
    constexpr int kOwn = kHeadProductSlices / SLICES;       // quarters a thread walks
    constexpr int kAhead = 16;                              // weight loads a thread of the four-wave kernel has on their way
    const int head = blockIdx.y;
    const int first = blockIdx.z * kHeadProductRows;
    const int rows = min(kHeadProductRows, n_tokens - first);
    const int lane = threadIdx.x % kWave, slice = threadIdx.x / kWave;
    const int o = blockIdx.x * kWave + lane;
    const int tile = min(n_in, kHeadProductTile);      // the inputs pass through LDS a tile at a time
    float acc[kOwn][kHeadProductRows];
#pragma unroll
    for (int q = 0; q < kOwn; ++q)
#pragma unroll
        for (int r = 0; r < kHeadProductRows; ++r) acc[q][r] = 0.0f;
    const W* column = w + static_cast<int64_t>(head) * n_in * n_out + min(o, n_out - 1);
    for (int i0 = 0; i0 < n_in; i0 += tile) {
        const int length = min(tile, n_in - i0);
        __syncthreads();        // the tile before has been read
        for (int r = 0; r < kHeadProductRows; ++r) {
            const X* from = x + static_cast<int64_t>(first + min(r, rows - 1)) * x_token_stride + static_cast<int64_t>(head) * x_head_stride + i0;
            for (int i = threadIdx.x; i < length; i += blockDim.x) x_rows[r * tile + i] = r < rows ? to_float(from[i]) : 0.0f;
        }
        __syncthreads();
        const int per_slice = (length + kHeadProductSlices - 1) / kHeadProductSlices;
#pragma unroll
        for (int q = 0; q < kOwn; ++q) {
            const int quarter = SLICES == 1 ? q : slice;
            const int begin = quarter * per_slice, end = min(begin + per_slice, length);
            if constexpr (SLICES == 1) {
#pragma unroll 4
                for (int i = begin; i < end; ++i) {
                    const float weight = to_float(column[static_cast<int64_t>(i0 + i) * n_out]);
#pragma unroll
                    for (int r = 0; r < kHeadProductRows; ++r) acc[q][r] = fmaf(x_rows[r * tile + i], weight, acc[q][r]);
                }
                continue;
            }
            for (int i = begin; i < end; i += kAhead) {      // few rows: kAhead loads of the weight are asked for before the first is used
                W ahead[kAhead];
#pragma unroll
                for (int n = 0; n < kAhead; ++n) ahead[n] = column[static_cast<int64_t>(i0 + min(i + n, end - 1)) * n_out];
#pragma unroll
                for (int n = 0; n < kAhead; ++n) {
                    const float weight = i + n < end ? to_float(ahead[n]) : 0.0f;      // past the end: a term of exactly zero
                    const int at = min(i + n, end - 1);
#pragma unroll
                    for (int r = 0; r < kHeadProductRows; ++r) acc[q][r] = fmaf(x_rows[r * tile + at], weight, acc[q][r]);
                }
            }
        }
    }
    float* partial = x_rows + kHeadProductRows * tile;
    if (SLICES > 1) {
        if (slice > 0) {
#pragma unroll
            for (int r = 0; r < kHeadProductRows; ++r) partial[((slice - 1) * kHeadProductRows + r) * kWave + lane] = acc[0][r];
        }
        __syncthreads();
    }
    if (slice > 0 || o >= n_out) return;
#pragma unroll
    for (int r = 0; r < kHeadProductRows; ++r) {
        if (r >= rows) break;
        float value = acc[0][r];
#pragma unroll
        for (int other = 1; other < kHeadProductSlices; ++other)
            value += SLICES == 1 ? acc[other % kOwn][r] : partial[((other - 1) * kHeadProductRows + r) * kWave + lane];
        if (gate != nullptr) {
            const float g = gate[static_cast<int64_t>(first + r) * gate_stride + (gate_a_head ? head : static_cast<int64_t>(head) * n_out + o)];
            value *= 1.0f / (1.0f + expf(-g));
        }
        out[static_cast<int64_t>(first + r) * out_token_stride + static_cast<int64_t>(head) * out_head_stride + o] = from_float<O>(value);
    }
}

// out[t][h * n + c] = in[h][t][c] * sigmoid(gate[t][h * n + c]): the heads of a batched product side by side, gated.
template <typename T>
__global__ void __launch_bounds__(256)
gate_heads_kernel(const T* __restrict__ in, const float* __restrict__ gate, int64_t gate_stride, int gate_a_head,
                  T* __restrict__ out, int n_tokens, int heads, int n) {
    const int token = blockIdx.x;
    for (int column = threadIdx.x; column < heads * n; column += blockDim.x) {
        const int head = column / n, c = column % n;
        float value = to_float(in[(static_cast<int64_t>(head) * n_tokens + token) * n + c]);
        if (gate != nullptr) value *= 1.0f / (1.0f + expf(-gate[static_cast<int64_t>(token) * gate_stride + (gate_a_head ? head : column)]));
        out[static_cast<int64_t>(token) * heads * n + column] = from_float<T>(value);
    }
}

// ---- the attention over plain pages --------------------------------------------------------------------------------
constexpr int kLatentKeyTile = 64;
constexpr int kLatentChannelsALane = 16;      // latents up to 1024 wide

template <typename T> __device__ inline float latent_dot(const T* key, const float* q, int dim);

template <> __device__ inline float latent_dot<float>(const float* key, const float* q, int dim) {
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

template <> __device__ inline float latent_dot<bf16>(const bf16* key, const float* q, int dim) {
    float sum = 0.0f;
    int c = 0;
    if ((dim & 7) == 0 && (reinterpret_cast<uintptr_t>(key) & 15) == 0) {
        for (; c < dim; c += 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(key + c);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                sum = fmaf(__builtin_bit_cast(float, words[w] << 16), q[c + 2 * w], sum);
                sum = fmaf(__builtin_bit_cast(float, words[w] & 0xffff0000u), q[c + 2 * w + 1], sum);
            }
        }
        return sum;
    }
    for (; c < dim; ++c) sum = fmaf(to_float(key[c]), q[c], sum);
    return sum;
}

// One wave a (token, head). Keys are walked in tiles of 64 at absolute positions from the tile that holds the
// oldest visible key: a lane forms the score of one key (over latent and rotated part), then the lanes turn to
// the latent's channels and add the tile's weighted latents in key order. The order of every sum depends on the
// query's position and the window alone.
template <typename T>
__global__ void __launch_bounds__(kWave)
latent_attention_kernel(const T* __restrict__ q_full, const T* __restrict__ pages, const int32_t* __restrict__ block_table,
                        int table_width, const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                        T* __restrict__ out, int64_t out_token_stride, int64_t out_head_stride, int heads, int kv_rank,
                        int rot_dim, int page_size, int window, float scale) {
    extern __shared__ float q_row[];
    const int token = blockIdx.x / heads, head = blockIdx.x % heads;
    const int seq = seq_of_token[token];
    if (seq < 0) return;       // a row that pads the step
    const int lane = threadIdx.x;
    const int position = positions[token];
    const int width = kv_rank + rot_dim;
    const T* query = q_full + (static_cast<int64_t>(token) * heads + head) * width;
    for (int c = lane; c < width; c += kWave) q_row[c] = to_float(query[c]);
    __syncthreads();
    const int32_t* table = block_table + static_cast<int64_t>(seq) * table_width;
    const int oldest = window > 0 ? max(0, position - window + 1) : 0;
    float running_max = -INFINITY, running_sum = 0.0f;
    float acc[kLatentChannelsALane];
#pragma unroll
    for (int m = 0; m < kLatentChannelsALane; ++m) acc[m] = 0.0f;
    for (int first = oldest / kLatentKeyTile * kLatentKeyTile; first <= position; first += kLatentKeyTile) {
        const int j = first + lane;
        const bool seen = j >= oldest && j <= position;
        float score = -INFINITY;
        int64_t place = 0;
        if (seen) {
            place = static_cast<int64_t>(table[j / page_size]) * page_size + j % page_size;
            score = latent_dot<T>(pages + place * width, q_row, width) * scale;
        }
        const float new_max = fmaxf(running_max, wave_max(score));
        const float keep = running_max == -INFINITY ? 0.0f : expf(running_max - new_max);
        const float weight = seen ? expf(score - new_max) : 0.0f;
        running_sum = running_sum * keep + wave_sum(weight);
        running_max = new_max;
#pragma unroll
        for (int m = 0; m < kLatentChannelsALane; ++m) acc[m] *= keep;
        const int from = max(oldest - first, 0), to = min(kLatentKeyTile, position - first + 1);
        for (int n = from; n < to; ++n) {
            const float w = __shfl(weight, n, kWave);
            const T* value = pages + __shfl(place, n, kWave) * width;
#pragma unroll
            for (int m = 0; m < kLatentChannelsALane; ++m) {
                const int c = lane + m * kWave;
                if (c < kv_rank) acc[m] = fmaf(w, to_float(value[c]), acc[m]);
            }
        }
    }
    const float factor = 1.0f / running_sum;
    T* to = out + static_cast<int64_t>(token) * out_token_stride + static_cast<int64_t>(head) * out_head_stride;
#pragma unroll
    for (int m = 0; m < kLatentChannelsALane; ++m) {
        const int c = lane + m * kWave;
        if (c < kv_rank) to[c] = from_float<T>(acc[m] * factor);
    }
}

constexpr int kHeadProductFewRows = 64;     // up to this many tokens a step, four waves share a workgroup's reduction

template <typename X, typename W, typename O>
int launch_head_product(const void* x, int64_t x_token_stride, int64_t x_head_stride, const void* w, void* out,
                        int64_t out_token_stride, int64_t out_head_stride, const float* gate, int64_t gate_stride, int gate_a_head,
                        int n_tokens, int heads, int n_in, int n_out, hipStream_t stream) {
    const dim3 grid((n_out + kWave - 1) / kWave, heads, (n_tokens + kHeadProductRows - 1) / kHeadProductRows);
    const size_t staged = static_cast<size_t>(kHeadProductRows) * (n_in < kHeadProductTile ? n_in : kHeadProductTile);
    if (n_tokens <= kHeadProductFewRows) {
        const size_t lds = (staged + (kHeadProductSlices - 1) * kHeadProductRows * kWave) * sizeof(float);
        head_product_kernel<X, W, O, kHeadProductSlices><<<grid, kHeadProductSlices * kWave, lds, stream>>>(
            static_cast<const X*>(x), x_token_stride, x_head_stride, static_cast<const W*>(w), static_cast<O*>(out),
            out_token_stride, out_head_stride, gate, gate_stride, gate_a_head, n_tokens, heads, n_in, n_out);
    } else {
        head_product_kernel<X, W, O, 1><<<grid, kWave, staged * sizeof(float), stream>>>(
            static_cast<const X*>(x), x_token_stride, x_head_stride, static_cast<const W*>(w), static_cast<O*>(out),
            out_token_stride, out_head_stride, gate, gate_stride, gate_a_head, n_tokens, heads, n_in, n_out);
    }
    return check_launch("head_product");
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_latent_prepare(const float* proj, int64_t proj_stride, int q_at, int q_rank, const float* q_weight, int kv_at,
                       int kv_rank, int rot_dim, const float* kv_weight, float eps, const float* cos_sin,
                       const int32_t* slot_mapping, void* q_latent, void* pages, void* k_pages, void* v_pages,
                       int tiled_page_size, int dtype, int n_tokens, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && eps > 0.0f && (q_rank == 0 || (q_rank > 0 && q_weight != nullptr && q_latent != nullptr)),
                "latent_prepare: the queries' latent needs a size, a weight and a place (size 0: there is none)");
    if (slot_mapping != nullptr) {
        MLL_REQUIRE(kv_rank > 0 && rot_dim > 0 && rot_dim % 2 == 0 && kv_weight != nullptr && cos_sin != nullptr,
                    "latent_prepare: the keys' latent needs its sizes (an even rotated part), a weight and cos/sin");
        MLL_REQUIRE(tiled_page_size == 0 ? pages != nullptr : (tiled_page_size % 16 == 0 && k_pages != nullptr && v_pages != nullptr),
                    "latent_prepare: plain pages, or tiled pages of a multiple of 16 positions for keys and values");
    }
    if (n_tokens == 0) return 0;
    MLL_REQUIRE(n_tokens < (1 << 30), "latent_prepare: too many rows for one launch");
    const unsigned blocks = static_cast<unsigned>(n_tokens) * 2;
    if (dtype == kF32) {
        latent_prepare_kernel<float><<<blocks, kPrepareThreads, 0, stream>>>(
            proj, proj_stride, q_at, q_rank, q_weight, kv_at, kv_rank, rot_dim, kv_weight, eps, cos_sin, slot_mapping,
            static_cast<float*>(q_latent), static_cast<float*>(pages), static_cast<float*>(k_pages), static_cast<float*>(v_pages), tiled_page_size);
    } else if (dtype == kBF16) {
        latent_prepare_kernel<bf16><<<blocks, kPrepareThreads, 0, stream>>>(
            proj, proj_stride, q_at, q_rank, q_weight, kv_at, kv_rank, rot_dim, kv_weight, eps, cos_sin, slot_mapping,
            static_cast<bf16*>(q_latent), static_cast<bf16*>(pages), static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), tiled_page_size);
    } else {
        return fail("latent_prepare: unknown dtype");
    }
    return check_launch("latent_prepare");
}

int mll_latent_query(const float* q, int64_t q_stride, int n_tokens, int heads, int dim, int rot_dim, int kv_rank, const float* cos_sin,
                     const void* folded, void* flat_out, void* q_full, int dtype, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && dim > 0 && rot_dim > 0 && rot_dim % 2 == 0 && kv_rank > 0 && cos_sin != nullptr,
                "latent_query: sizes must be positive, the rotated part even");
    MLL_REQUIRE(q_stride >= static_cast<int64_t>(heads) * (dim + rot_dim), "latent_query: the queries' rows overlap");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * heads;
    MLL_REQUIRE(blocks < (1ll << 31), "latent_query: too many rows for one launch");
    if (dtype == kF32) {
        latent_query_kernel<float><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(
            q, q_stride, n_tokens, heads, dim, rot_dim, kv_rank, cos_sin, static_cast<const float*>(folded), static_cast<float*>(flat_out),
            static_cast<float*>(q_full));
    } else if (dtype == kBF16) {
        latent_query_kernel<bf16><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(
            q, q_stride, n_tokens, heads, dim, rot_dim, kv_rank, cos_sin, static_cast<const bf16*>(folded), static_cast<bf16*>(flat_out),
            static_cast<bf16*>(q_full));
    } else {
        return fail("latent_query: unknown dtype");
    }
    return check_launch("latent_query");
}

int mll_head_product(const void* x, int x_dtype, int64_t x_token_stride, int64_t x_head_stride, const void* w, int w_dtype,
                     void* out, int out_dtype, int64_t out_token_stride, int64_t out_head_stride, const float* gate,
                     int64_t gate_stride, int gate_a_head, int n_tokens, int heads, int n_in, int n_out, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && n_in > 0 && n_out > 0, "head_product: sizes must be positive");
    MLL_REQUIRE(heads < 65536 && (n_tokens + kHeadProductRows - 1) / kHeadProductRows < 65536, "head_product: too many heads or rows for one launch");
    if (n_tokens == 0) return 0;
#define MLL_HEAD_PRODUCT(X, W, O)                                                                                          \
    return launch_head_product<X, W, O>(x, x_token_stride, x_head_stride, w, out, out_token_stride, out_head_stride, gate, \
                                        gate_stride, gate_a_head, n_tokens, heads, n_in, n_out, stream)
    if (x_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) MLL_HEAD_PRODUCT(float, float, float);
    if (x_dtype == kF32 && w_dtype == kBF16 && out_dtype == kBF16) MLL_HEAD_PRODUCT(float, bf16, bf16);
    if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) MLL_HEAD_PRODUCT(bf16, bf16, bf16);
    if (x_dtype == kF32 && w_dtype == kBF16 && out_dtype == kF32) MLL_HEAD_PRODUCT(float, bf16, float);
#undef MLL_HEAD_PRODUCT
    return fail("head_product: this combination of element types is not built");
}

int mll_latent_attention(const void* q_full, const void* pages, const int32_t* block_table, int table_width,
                         const int32_t* seq_of_token, const int32_t* positions, void* out, int64_t out_token_stride,
                         int64_t out_head_stride, int dtype, int n_tokens, int heads, int kv_rank, int rot_dim, int page_size,
                         int window, float scale, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && kv_rank > 0 && rot_dim >= 0 && page_size > 0 && table_width > 0,
                "latent_attention: sizes must be positive");
    MLL_REQUIRE(kv_rank <= kLatentChannelsALane * kWave, "latent_attention: latents wider than 1024 are not supported");
    MLL_REQUIRE(out_head_stride >= kv_rank && out_token_stride >= static_cast<int64_t>(heads) * kv_rank, "latent_attention: the output rows overlap");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * heads;
    MLL_REQUIRE(blocks < (1ll << 31), "latent_attention: too many rows for one launch");
    const size_t lds = static_cast<size_t>(kv_rank + rot_dim) * sizeof(float);
    if (dtype == kF32) {
        latent_attention_kernel<float><<<static_cast<unsigned>(blocks), kWave, lds, stream>>>(
            static_cast<const float*>(q_full), static_cast<const float*>(pages), block_table, table_width, seq_of_token, positions,
            static_cast<float*>(out), out_token_stride, out_head_stride, heads, kv_rank, rot_dim, page_size, window, scale);
    } else if (dtype == kBF16) {
        latent_attention_kernel<bf16><<<static_cast<unsigned>(blocks), kWave, lds, stream>>>(
            static_cast<const bf16*>(q_full), static_cast<const bf16*>(pages), block_table, table_width, seq_of_token, positions,
            static_cast<bf16*>(out), out_token_stride, out_head_stride, heads, kv_rank, rot_dim, page_size, window, scale);
    } else {
        return fail("latent_attention: unknown dtype");
    }
    return check_launch("latent_attention");
}

int mll_gate_heads(const void* in, const float* gate, int64_t gate_stride, int gate_a_head, void* out, int dtype, int n_tokens,
                   int heads, int n, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && n > 0, "gate_heads: sizes must be positive");
    if (n_tokens == 0) return 0;
    if (dtype == kF32) {
        gate_heads_kernel<float><<<n_tokens, 256, 0, stream>>>(static_cast<const float*>(in), gate, gate_stride, gate_a_head, static_cast<float*>(out), n_tokens, heads, n);
    } else if (dtype == kBF16) {
        gate_heads_kernel<bf16><<<n_tokens, 256, 0, stream>>>(static_cast<const bf16*>(in), gate, gate_stride, gate_a_head, static_cast<bf16*>(out), n_tokens, heads, n);
    } else {
        return fail("gate_heads: unknown dtype");
    }
    return check_launch("gate_heads");
}

}  // extern "C"
