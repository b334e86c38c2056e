// The gated delta rule: a matrix of state per head and request that forgets by one factor a head and is corrected
// towards the new value along the new key.
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t        (S: [key_dim, value_dim])
//
// so the read-out sees the token's own write. q, k and v come from a short causal convolution per channel over the
// projections and SiLU; q and k are then made unit vectors per head (x / sqrt(sum(x^2) + unit_eps)) and q multiplied
// by a factor; beta = sigmoid(.) and g = exp(-exp(A_log) * softplus(. + dt_bias)) are one number a head and token.
// Three kernels: the convolution with its activation, the unit vectors and the two gates for all tokens of a step at
// once; the newest inputs of the convolution into the request's slot; and the walk over each request's tokens in
// order (in two forms: operands straight from memory for steps of few tokens a request, tiles of tokens staged through
// LDS for portions of prompts). The columns of S are independent, so a head is spread over waves by value channel.
// Everything is float32.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

__device__ inline float delta_softplus(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }
__device__ inline float delta_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// One wave a (token, vector): vectors 0 .. key_heads - 1 are the queries' heads, the next key_heads the keys', the last
// `heads` the values'. Channel c of the convolution reads proj[.][conv_at + c]; the step's tokens of the same request
// come from proj, what lies before the step from the request's kept inputs (kept [slot][n_taps - 1][channels], newest
// last; a fresh slot is zero). The wave of a value head also writes the head's two gates: gates[t][2 h] = beta,
// gates[t][2 h + 1] = g.
__global__ void __launch_bounds__(kWave)
delta_prepare_kernel(const float* __restrict__ proj, int64_t proj_stride, int conv_at, const float* __restrict__ taps,
                     const float* __restrict__ kept, const int32_t* __restrict__ seq_of_token,
                     const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ slots, int beta_at, int step_at,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ u,
                     float* __restrict__ gates, int key_heads, int heads, int key_dim, int value_dim, int n_taps,
                     float q_factor, float unit_eps) {
    const int vectors = 2 * key_heads + heads;
    const int token = blockIdx.x / vectors, which = blockIdx.x % vectors;
    const int lane = threadIdx.x;
    const int channels = 2 * key_heads * key_dim + heads * value_dim;
    const bool is_value = which >= 2 * key_heads;
    const int dim = is_value ? value_dim : key_dim;
    const int first_channel = is_value ? 2 * key_heads * key_dim + (which - 2 * key_heads) * value_dim : which * key_dim;
    float* to = u + static_cast<int64_t>(token) * channels + first_channel;
    const int seq = seq_of_token[token];
    if (seq < 0) {      // a row that pads the step
        for (int c = lane; c < dim; c += kWave) to[c] = 0.0f;
        if (is_value && lane < 2) gates[static_cast<int64_t>(token) * 2 * heads + 2 * (which - 2 * key_heads) + lane] = 0.0f;
        return;
    }
    const int local = token - cu_tokens[seq];
    const int before = n_taps - 1;
    const float* tail = kept + static_cast<int64_t>(slots[seq]) * before * channels;
    float squares = 0.0f;
    for (int c = lane; c < dim; c += kWave) {
        const int channel = first_channel + c;
        float sum = 0.0f;
        for (int j = 0; j < n_taps; ++j) {
            const int back = before - j;        // how many tokens before this one
            const float value = back <= local ? proj[static_cast<int64_t>(token - back) * proj_stride + conv_at + channel]
                                              : tail[static_cast<int64_t>(before - (back - local)) * channels + channel];
            sum = fmaf(taps[static_cast<int64_t>(channel) * n_taps + j], value, sum);
        }
        const float activated = sum * delta_sigmoid(sum);
        to[c] = activated;
        squares = fmaf(activated, activated, squares);
    }
    if (!is_value) {
        float factor = 1.0f / sqrtf(wave_sum(squares) + unit_eps);
        if (which < key_heads) factor *= q_factor;
        for (int c = lane; c < dim; c += kWave) to[c] *= factor;     // a lane scales what it wrote itself
        return;
    }
    if (lane == 0) {
        const int head = which - 2 * key_heads;
        const float* row = proj + static_cast<int64_t>(token) * proj_stride;
        float* gate = gates + static_cast<int64_t>(token) * 2 * heads + 2 * head;
        gate[0] = delta_sigmoid(row[beta_at + head]);
        gate[1] = expf(-expf(a_log[head]) * delta_softplus(row[step_at + head] + dt_bias[head]));
    }
}

// kept[slot] <- the newest n_taps - 1 inputs of the request: the step's own where it brought enough, older kept
// ones before them. One thread a (request, channel) reads all it needs before it writes.
constexpr int kMaxTaps = 32;

__global__ void __launch_bounds__(256)
conv_keep_kernel(const float* __restrict__ proj, int64_t proj_stride, int conv_at, float* __restrict__ kept,
                 const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ slots, int channels, int n_taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    const int count = last - first, before = n_taps - 1;
    if (count <= 0 || before <= 0) return;
    float* tail = kept + static_cast<int64_t>(slots[seq]) * before * channels + c;
    float newest[kMaxTaps];
    for (int j = 0; j < before; ++j) {      // j counts from the oldest kept place
        const int back = before - 1 - j;    // tokens before the step's last one
        newest[j] = back < count ? proj[static_cast<int64_t>(last - 1 - back) * proj_stride + conv_at + c]
                                 : tail[static_cast<int64_t>(j + count) * channels];
    }
    for (int j = 0; j < before; ++j) tail[static_cast<int64_t>(j) * channels] = newest[j];
}

// The sum of `value` over the 16 lanes of a row of the wave, in every one of them: exchanges on the vector unit
// (within fours, within eights by the half mirror, within the row by the mirror). The additions pair up the same
// operands in every lane, so all lanes hold the same bits.
template <int CONTROL>
__device__ inline float lanes_exchanged(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CONTROL, 0xf, 0xf, false));
}
__device__ inline float sum_row_of_16(float value) {
    value += lanes_exchanged<0xB1>(value);      // lanes 1, 0, 3, 2 of every four
    value += lanes_exchanged<0x4E>(value);      // lanes 2, 3, 0, 1 of every four
    value += lanes_exchanged<0x141>(value);     // every eight mirrored
    value += lanes_exchanged<0x140>(value);     // the row of 16 mirrored
    return value;
}

// One wave a (request, head, four value channels): lane = 16 * column + r, and lane r of a column keeps the key
// channels ROWS r .. ROWS r + ROWS - 1 of that column of S. A token's two sums over key channels run over a lane's
// channels in order and then over the column's 16 lanes by exchanges, the same way whatever the step holds: a
// request's state and results are the same bits however its tokens are cut into steps.
constexpr int kDeltaLanesAColumn = 16;
constexpr int kDeltaColumnsAWave = kWave / kDeltaLanesAColumn;

template <int ROWS>
__global__ void __launch_bounds__(kWave)
delta_scan_kernel(const float* __restrict__ u, const float* __restrict__ gates, float* __restrict__ state,
                  const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ slots, float* __restrict__ out,
                  int key_heads, int heads, int key_dim, int value_dim) {
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;       // a request that pads the step brings no tokens
    const int lane = threadIdx.x;
    const int r = lane % kDeltaLanesAColumn;
    const int column = blockIdx.z * kDeltaColumnsAWave + lane / kDeltaLanesAColumn;
    const bool live = column < value_dim;
    const int safe_column = live ? column : 0;
    const int key_head = head / (heads / key_heads);
    const int channels = 2 * key_heads * key_dim + heads * value_dim;
    const int q_at = key_head * key_dim, k_at = (key_heads + key_head) * key_dim;
    const int v_at = 2 * key_heads * key_dim + head * value_dim + safe_column;
    float* mine = state + ((static_cast<int64_t>(slots[seq]) * heads + head) * key_dim) * value_dim + safe_column;
    float s[ROWS];
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        s[m] = i < key_dim ? mine[static_cast<int64_t>(i) * value_dim] : 0.0f;
    }
    float k_next[ROWS], q_next[ROWS], v_next, beta_next, g_next;
    auto fetch = [&](int token) {
        const float* row = u + static_cast<int64_t>(token) * channels;
#pragma unroll
        for (int m = 0; m < ROWS; ++m) {
            const int i = ROWS * r + m;
            const bool in = i < key_dim;
            k_next[m] = in ? row[k_at + i] : 0.0f;
            q_next[m] = in ? row[q_at + i] : 0.0f;
        }
        v_next = row[v_at];
        beta_next = gates[static_cast<int64_t>(token) * 2 * heads + 2 * head];
        g_next = gates[static_cast<int64_t>(token) * 2 * heads + 2 * head + 1];
    };
    fetch(first);
    for (int token = first; token < last; ++token) {
        float k[ROWS], q[ROWS];
#pragma unroll
        for (int m = 0; m < ROWS; ++m) k[m] = k_next[m], q[m] = q_next[m];
        const float v = v_next, beta = beta_next, g = g_next;
        if (token + 1 < last) fetch(token + 1);
        float seen = 0.0f;
#pragma unroll
        for (int m = 0; m < ROWS; ++m) {
            s[m] *= g;
            seen = fmaf(s[m], k[m], seen);
        }
        const float correction = beta * (v - sum_row_of_16(seen));
        float read = 0.0f;
#pragma unroll
        for (int m = 0; m < ROWS; ++m) {
            s[m] = fmaf(k[m], correction, s[m]);
            read = fmaf(s[m], q[m], read);
        }
        read = sum_row_of_16(read);
        if (live && r == 0) out[(static_cast<int64_t>(token) * heads + head) * value_dim + column] = read;
    }
    if (!live) return;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        if (i < key_dim) mine[static_cast<int64_t>(i) * value_dim] = s[m];
    }
}


// The same walk for portions of many tokens: a wave brings tiles of tokens (keys and queries of its key head, the
// values of its columns, the head's two gates) from memory straight into LDS, the next tile on its way while it
// walks this one, so that a token waits for LDS and not for memory. The operations per token and their order are
// those of the kernel above: the same bits, only where the operands come from differs.
// WIDE: rows of key channels and their places in memory are multiples of 16 bytes, and a lane's load brings 16.
constexpr int kDeltaTileFloats = 2048;      // of each of keys and queries in a tile
constexpr int kDeltaTileTokens = 64;        // at most
constexpr int kDeltaBufferFloats = 2 * kDeltaTileFloats + kDeltaTileTokens * (kDeltaColumnsAWave + 2);

template <bool WIDE, int ROWS>
__global__ void __launch_bounds__(kWave)
delta_scan_tiled_kernel(const float* __restrict__ u, const float* __restrict__ gates, float* __restrict__ state,
                        const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ slots, float* __restrict__ out,
                        int key_heads, int heads, int key_dim, int value_dim) {
    __shared__ __align__(16) float buffer_even[kDeltaBufferFloats];
    __shared__ __align__(16) float buffer_odd[kDeltaBufferFloats];
    constexpr int kRowFloats = ROWS * kDeltaLanesAColumn;                                      // a token's row of key channels in LDS
    constexpr int kTileTokens = kDeltaTileFloats / kRowFloats < kDeltaTileTokens ? kDeltaTileFloats / kRowFloats : kDeltaTileTokens;
    constexpr int kValuesAt = 2 * kDeltaTileFloats, kGatesAt = kValuesAt + kDeltaTileTokens * kDeltaColumnsAWave;
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;
    const int lane = threadIdx.x;
    const int r = lane % kDeltaLanesAColumn;
    const int column_in_wave = lane / kDeltaLanesAColumn;
    const int column = blockIdx.z * kDeltaColumnsAWave + column_in_wave;
    const bool live = column < value_dim;
    const int safe_column = live ? column : 0;
    const int key_head = head / (heads / key_heads);
    const int channels = 2 * key_heads * key_dim + heads * value_dim;
    const int q_at = key_head * key_dim, k_at = (key_heads + key_head) * key_dim;
    const int v_at = 2 * key_heads * key_dim + head * value_dim;
    float* mine = state + ((static_cast<int64_t>(slots[seq]) * heads + head) * key_dim) * value_dim + safe_column;
    float s[ROWS];
    bool valid[ROWS];
    bool all_valid = true;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        valid[m] = i < key_dim;
        all_valid = all_valid && valid[m];
        s[m] = valid[m] ? mine[static_cast<int64_t>(i) * value_dim] : 0.0f;
    }
    all_valid = __all(all_valid);
    // Nothing that is read from LDS may be a stray bit pattern: places that no load fills are read beside others.
    for (int index = lane; index < kDeltaBufferFloats; index += kWave) buffer_even[index] = buffer_odd[index] = 0.0f;
    __syncthreads();
    // Which token of a tile and which channel each of this lane's loads brings (the same for every tile). A row's
    // places beyond key_dim bring a channel of the row again; the walk never lets them count.
    constexpr int kPiece = WIDE ? 4 : 1;                                        // floats a lane's load brings
    constexpr int kCalls = kTileTokens * kRowFloats / (kWave * kPiece);         // loads that bring one of keys, queries
    int token_of[kCalls], channel_of[kCalls];
#pragma unroll
    for (int j = 0; j < kCalls; ++j) {
        const int element = (j * kWave + lane) * kPiece;
        token_of[j] = element / kRowFloats;
        channel_of[j] = min(element % kRowFloats, key_dim - kPiece);
    }
    constexpr int kValueCalls = (kTileTokens * kDeltaColumnsAWave + kWave - 1) / kWave;
    constexpr int kGateCalls = (kTileTokens * 2 + kWave - 1) / kWave;
    auto fetch = [&](int tile_first, float* buffer) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < kCalls; ++j) {
            const int64_t token = min(tile_first + token_of[j], last - 1);
            const float* row = u + token * channels + channel_of[j];
            float* place = buffer + j * kWave * kPiece;
            if constexpr (WIDE) {
                __builtin_amdgcn_global_load_lds(row + k_at, place, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(row + q_at, place + kDeltaTileFloats, 16, 0, 0);
            } else {
                __builtin_amdgcn_global_load_lds(row + k_at, place, 4, 0, 0);
                __builtin_amdgcn_global_load_lds(row + q_at, place + kDeltaTileFloats, 4, 0, 0);
            }
        }
#pragma unroll
        for (int j = 0; j < kValueCalls; ++j) {
            const int element = j * kWave + lane;
            const int64_t token = min(tile_first + element / kDeltaColumnsAWave, last - 1);
            const int wanted = min(static_cast<int>(blockIdx.z) * kDeltaColumnsAWave + element % kDeltaColumnsAWave, value_dim - 1);
            __builtin_amdgcn_global_load_lds(u + token * channels + v_at + wanted, buffer + kValuesAt + j * kWave, 4, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < kGateCalls; ++j) {
            const int element = j * kWave + lane;
            const int64_t token = min(tile_first + element / 2, last - 1);
            __builtin_amdgcn_global_load_lds(gates + token * 2 * heads + 2 * head + element % 2, buffer + kGatesAt + j * kWave, 4, 0, 0);
        }
    };
    auto walk_tokens = [&](auto every_channel, int tile_first, int count, const float* buffer) __attribute__((always_inline)) {
        // Two sets of a token's operands take turns: while one token is worked, the next one's leave LDS.
        float k_a[ROWS], q_a[ROWS], k_b[ROWS], q_b[ROWS];
        float few_a[3], few_b[3];       // value, beta, g
        auto read_token = [&](int t, float* k, float* q, float* few) __attribute__((always_inline)) {
            const float* row = buffer + t * kRowFloats + ROWS * r;
            if constexpr (ROWS % 4 == 0) {
#pragma unroll
                for (int piece = 0; piece < ROWS; piece += 4) {
                    *reinterpret_cast<float4*>(k + piece) = *reinterpret_cast<const float4*>(row + piece);
                    *reinterpret_cast<float4*>(q + piece) = *reinterpret_cast<const float4*>(row + kDeltaTileFloats + piece);
                }
            } else {
#pragma unroll
                for (int m = 0; m < ROWS; ++m) k[m] = row[m], q[m] = row[kDeltaTileFloats + m];
            }
            if constexpr (!decltype(every_channel)::value) {
#pragma unroll
                for (int m = 0; m < ROWS; ++m) {
                    k[m] = valid[m] ? k[m] : 0.0f;
                    q[m] = valid[m] ? q[m] : 0.0f;
                }
            }
            few[0] = buffer[kValuesAt + t * kDeltaColumnsAWave + column_in_wave];
            few[1] = buffer[kGatesAt + 2 * t];
            few[2] = buffer[kGatesAt + 2 * t + 1];
        };
        float* to = out + (static_cast<int64_t>(tile_first) * heads + head) * value_dim + column;
        const int64_t to_stride = static_cast<int64_t>(heads) * value_dim;
        const bool writes = live && r == 0;
        auto work = [&](const float* k, const float* q, const float* few) __attribute__((always_inline)) {
            const float v = few[0], beta = few[1], g = few[2];
            float seen = 0.0f;
#pragma unroll
            for (int m = 0; m < ROWS; ++m) {
                s[m] *= g;
                seen = fmaf(s[m], k[m], seen);
            }
            const float correction = beta * (v - sum_row_of_16(seen));
            float read = 0.0f;
#pragma unroll
            for (int m = 0; m < ROWS; ++m) {
                s[m] = fmaf(k[m], correction, s[m]);
                read = fmaf(s[m], q[m], read);
            }
            read = sum_row_of_16(read);
            if (writes) *to = read;
            to += to_stride;
        };
        read_token(0, k_a, q_a, few_a);
        int t = 0;
        for (; t + 1 < count; t += 2) {
            read_token(t + 1, k_b, q_b, few_b);
            work(k_a, q_a, few_a);
            read_token(min(t + 2, count - 1), k_a, q_a, few_a);
            work(k_b, q_b, few_b);
        }
        if (t < count) work(k_a, q_a, few_a);
    };
    auto walk = [&](int tile_first, const float* buffer) __attribute__((always_inline)) {
        const int count = min(kTileTokens, last - tile_first);
        if (all_valid) walk_tokens(std::true_type{}, tile_first, count, buffer);
        else walk_tokens(std::false_type{}, tile_first, count, buffer);
    };
    fetch(first, buffer_even);
    for (int tile_first = first; tile_first < last;) {
        wait_for_loads();
        __syncthreads();
        if (tile_first + kTileTokens < last) fetch(tile_first + kTileTokens, buffer_odd);
        walk(tile_first, buffer_even);
        tile_first += kTileTokens;
        if (tile_first >= last) break;
        wait_for_loads();
        __syncthreads();
        if (tile_first + kTileTokens < last) fetch(tile_first + kTileTokens, buffer_even);
        walk(tile_first, buffer_odd);
        tile_first += kTileTokens;
    }
    if (!live) return;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        if (i < key_dim) mine[static_cast<int64_t>(i) * value_dim] = s[m];
    }
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_delta_prepare(const float* proj, int64_t proj_stride, int conv_at, const float* taps, const float* kept,
                      const int32_t* seq_of_token, const int32_t* cu_tokens, const int32_t* slots, int beta_at, int step_at,
                      const float* a_log, const float* dt_bias, float* u, float* gates, int n_tokens, int key_heads, int heads,
                      int key_dim, int value_dim, int n_taps, float q_factor, float unit_eps, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && key_heads > 0 && heads > 0 && key_dim > 0 && value_dim > 0, "delta_prepare: sizes must be positive");
    MLL_REQUIRE(heads % key_heads == 0, "delta_prepare: the value heads must divide into the key heads");
    MLL_REQUIRE(n_taps >= 1 && n_taps <= kMaxTaps, "delta_prepare: 1 to 32 taps");
    MLL_REQUIRE(n_taps == 1 || kept != nullptr, "delta_prepare: a convolution over several tokens needs the kept inputs");
    MLL_REQUIRE(unit_eps > 0.0f, "delta_prepare: the unit vectors' eps must be positive");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * (2 * key_heads + heads);
    MLL_REQUIRE(blocks < (1ll << 31), "delta_prepare: too many rows for one launch");
    delta_prepare_kernel<<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(
        proj, proj_stride, conv_at, taps, kept, seq_of_token, cu_tokens, slots, beta_at, step_at, a_log, dt_bias, u, gates,
        key_heads, heads, key_dim, value_dim, n_taps, q_factor, unit_eps);
    return check_launch("delta_prepare");
}

int mll_conv_keep(const float* proj, int64_t proj_stride, int conv_at, float* kept, const int32_t* cu_tokens,
                  const int32_t* slots, int n_seqs, int channels, int n_taps, hipStream_t stream) {
    MLL_REQUIRE(n_seqs >= 0 && channels > 0, "conv_keep: sizes must be positive");
    MLL_REQUIRE(n_taps >= 1 && n_taps <= kMaxTaps, "conv_keep: 1 to 32 taps");
    if (n_seqs == 0 || n_taps == 1) return 0;
    MLL_REQUIRE(n_seqs < 65536, "conv_keep: too many requests for one launch");
    conv_keep_kernel<<<dim3((channels + 255) / 256, n_seqs), 256, 0, stream>>>(proj, proj_stride, conv_at, kept, cu_tokens,
                                                                               slots, channels, n_taps);
    return check_launch("conv_keep");
}

int mll_delta_scan(const float* u, const float* gates, float* state, const int32_t* cu_tokens, const int32_t* slots, float* out,
                   int n_seqs, int key_heads, int heads, int key_dim, int value_dim, int long_portions, hipStream_t stream) {
    MLL_REQUIRE(n_seqs >= 0 && key_heads > 0 && heads > 0 && key_dim > 0 && value_dim > 0, "delta_scan: sizes must be positive");
    MLL_REQUIRE(heads % key_heads == 0, "delta_scan: the value heads must divide into the key heads");
    MLL_REQUIRE(key_dim <= 16 * kDeltaLanesAColumn, "delta_scan: key heads wider than 256 are not supported");
    if (n_seqs == 0) return 0;
    const int groups = (value_dim + kDeltaColumnsAWave - 1) / kDeltaColumnsAWave;
    MLL_REQUIRE(heads < 65536 && groups < 65536, "delta_scan: too many heads or value channels for one launch");
    const dim3 grid(n_seqs, heads, groups);
    const int rows = (key_dim + kDeltaLanesAColumn - 1) / kDeltaLanesAColumn;
    if (long_portions) {
        const int channels = 2 * key_heads * key_dim + heads * value_dim;
        const bool wide = key_dim % 4 == 0 && channels % 4 == 0 && reinterpret_cast<uintptr_t>(u) % 16 == 0;
#define MLL_DELTA_TILED(WIDE, ROWS) \
    delta_scan_tiled_kernel<WIDE, ROWS><<<grid, kWave, 0, stream>>>(u, gates, state, cu_tokens, slots, out, key_heads, heads, key_dim, value_dim)
#define MLL_DELTA_TILED_ROWS(ROWS) \
    do { if (wide) MLL_DELTA_TILED(true, ROWS); else MLL_DELTA_TILED(false, ROWS); } while (0)
        if (rows <= 1) MLL_DELTA_TILED(false, 1);
        else if (rows <= 2) MLL_DELTA_TILED(false, 2);
        else if (rows <= 4) MLL_DELTA_TILED_ROWS(4);
        else if (rows <= 8) MLL_DELTA_TILED_ROWS(8);
        else MLL_DELTA_TILED_ROWS(16);
#undef MLL_DELTA_TILED_ROWS
#undef MLL_DELTA_TILED
        return check_launch("delta_scan_tiled");
    }
#define MLL_DELTA_SCAN(ROWS) \
    delta_scan_kernel<ROWS><<<grid, kWave, 0, stream>>>(u, gates, state, cu_tokens, slots, out, key_heads, heads, key_dim, value_dim)
    if (rows <= 1) MLL_DELTA_SCAN(1);
    else if (rows <= 2) MLL_DELTA_SCAN(2);
    else if (rows <= 4) MLL_DELTA_SCAN(4);
    else if (rows <= 8) MLL_DELTA_SCAN(8);
    else MLL_DELTA_SCAN(16);
#undef MLL_DELTA_SCAN
    return check_launch("delta_scan");
}

}  // extern "C"
