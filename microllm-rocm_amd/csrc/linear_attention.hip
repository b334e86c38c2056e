// Gated linear attention: a matrix of state per head and request, decayed per key channel and carried from token
// to token.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T        (S: [key_dim, value_dim], a_t in (0, 1) per key channel)
//   o_t = S_t^T q_t
//
// with a_t = sigmoid(z_t)^(1 / tau), z_t = A2 (low-rank input) + b. Three kernels: the decays of a step's tokens
// (all tokens at once), the walk over each request's tokens in order (the state's columns are independent, so a
// request's head is spread over workgroups by value channel), and the norm and gate of the results. State, decays
// and everything the walk touches are float32, whatever the engine's element type.
#include <type_traits>

#include "common.h"
#include "microllm_hip.h"

namespace mll {

// Key channels a lane keeps of its column of the state (ROWS below): 4 for key heads up to 256 channels, so that a
// column is spread over more lanes and a token costs each fewer operations, 8 beyond. The choice follows the head
// size alone, so both walk kernels make it alike.
constexpr int kWideHeadRows = 8;
constexpr int kUsualRows = 4;

// decay[t, c] = exp(log_sigmoid(z) / tau), z = bias[c] + sum_r a2[c, r] * low[t, r]
template <typename W>
__global__ void gla_decay_kernel(const float* __restrict__ proj, int64_t proj_stride, int low_offset, int rank,
                                 const W* __restrict__ a2, const float* __restrict__ bias, float inv_tau,
                                 float* __restrict__ decay, int channels) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const float* low = proj + static_cast<int64_t>(token) * proj_stride + low_offset;
    float z = bias ? bias[c] : 0.0f;
    for (int r = 0; r < rank; ++r) z = fmaf(to_float(a2[static_cast<int64_t>(c) * rank + r]), low[r], z);
    // log(sigmoid(z)) = -(max(-z, 0) + log1p(exp(-|z|)))
    const float log_sigmoid = -(fmaxf(-z, 0.0f) + log1pf(expf(-fabsf(z))));
    decay[static_cast<int64_t>(token) * channels + c] = expf(log_sigmoid * inv_tau);
}

// One wave a (request, head, group of value channels). lane = column_in_group * lanes_a_column + r; lane r of a
// column keeps the key channels ROWS r .. ROWS r + ROWS - 1. A token's result is the sum over a lane's channels in order, then
// over the column's lanes in order (the lanes leave their sums in LDS and one adds them up): both kernels below add
// in this order, so a request gives the same bits whichever of them walks its tokens.
template <int ROWS>
__global__ void __launch_bounds__(kWave)
gla_scan_kernel(const float* __restrict__ proj, int64_t proj_stride, int q_offset, int k_offset, int v_offset,
                const float* __restrict__ decay, float* __restrict__ state, const int32_t* __restrict__ cu_tokens,
                const int32_t* __restrict__ slots, float* __restrict__ out, int heads, int key_dim, int value_dim,
                int lanes_a_column, float q_scale, int64_t decay_stride) {
    __shared__ float lane_sums[kWave];
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;       // a request that pads the step brings no tokens
    const int lane = threadIdx.x;
    const int r = lane % lanes_a_column;
    const int column = blockIdx.z * (kWave / lanes_a_column) + lane / lanes_a_column;
    const bool live = column < value_dim;
    const int safe_column = live ? column : 0;
    const int slot = slots[seq];
    float* mine = state + ((static_cast<int64_t>(slot) * heads + head) * key_dim) * value_dim + safe_column;
    float s[ROWS];
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        s[m] = i < key_dim ? mine[static_cast<int64_t>(i) * value_dim] : 0.0f;
    }
    float a_next[ROWS], k_next[ROWS], q_next[ROWS], v_next;
    auto fetch = [&](int token) {
        const float* row = proj + static_cast<int64_t>(token) * proj_stride;
        const float* decays = decay + static_cast<int64_t>(token) * decay_stride + head * key_dim;
#pragma unroll
        for (int m = 0; m < ROWS; ++m) {
            const int i = ROWS * r + m;
            const bool in = i < key_dim;
            a_next[m] = in ? decays[i] : 0.0f;
            k_next[m] = in ? row[k_offset + head * key_dim + i] : 0.0f;
            q_next[m] = in ? row[q_offset + head * key_dim + i] : 0.0f;
        }
        v_next = row[v_offset + head * value_dim + safe_column];
    };
    fetch(first);
    for (int token = first; token < last; ++token) {
        float a[ROWS], k[ROWS], q[ROWS];
#pragma unroll
        for (int m = 0; m < ROWS; ++m) a[m] = a_next[m], k[m] = k_next[m], q[m] = q_next[m];
        const float v = v_next;
        if (token + 1 < last) fetch(token + 1);
        float partial = 0.0f;
#pragma unroll
        for (int m = 0; m < ROWS; ++m) {
            s[m] = fmaf(a[m], s[m], k[m] * v);
            partial = fmaf(s[m], q[m], partial);
        }
        __syncthreads();      // the sums of the token before have been read
        lane_sums[lane] = partial;
        __syncthreads();
        if (live && r == 0) {
            float total = 0.0f;
            for (int other = 0; other < lanes_a_column; ++other) total += lane_sums[lane + other];
            out[(static_cast<int64_t>(token) * heads + head) * value_dim + column] = total * q_scale;
        }
    }
    if (!live) return;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        if (i < key_dim) mine[static_cast<int64_t>(i) * value_dim] = s[m];
    }
}

// The same walk for portions of many tokens: a wave brings tiles of tokens (decays, keys, queries of its head, the
// values of its columns) from memory straight into LDS, the next tile on its way while it walks this one, and reads
// its key channels of a token in pieces of 16 bytes. The walk over a request's tokens stays in order, with the
// same operations per token in the same order as above; only where the operands come from differs.
// WIDE: rows of key channels and their places in memory are multiples of 16 bytes, and a lane's load brings 16.
constexpr int kScanTileFloats = 2048;                    // of each of decays, keys, queries (and at most of values) in a tile
constexpr int kScanBufferFloats = 4 * kScanTileFloats;

template <bool WIDE, int ROWS>
__global__ void __launch_bounds__(kWave)
gla_scan_tiled_kernel(const float* __restrict__ proj, int64_t proj_stride, int q_offset, int k_offset, int v_offset,
                      const float* __restrict__ decay, float* __restrict__ state, const int32_t* __restrict__ cu_tokens,
                      const int32_t* __restrict__ slots, float* __restrict__ out, int heads, int key_dim, int value_dim,
                      int lanes_a_column, int tile_tokens, float q_scale, int64_t decay_stride) {
    __shared__ __align__(16) float buffer_even[kScanBufferFloats];
    __shared__ __align__(16) float buffer_odd[kScanBufferFloats];
    __shared__ __align__(16) float lane_sums[64 * kWave];    // of a tile's tokens (at most 64), added up after its walk
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    if (last <= first) return;
    const int lane = threadIdx.x;
    const int r = lane % lanes_a_column;
    const int columns = kWave / lanes_a_column;              // of this wave
    const int column_in_group = lane / lanes_a_column;
    const int column = blockIdx.z * columns + column_in_group;
    const bool live = column < value_dim;
    const int safe_column = live ? column : 0;
    const int row_floats = (key_dim + 7) / 8 * 8;            // a token's row of key channels in LDS
    const int slot = slots[seq];
    float* mine = state + ((static_cast<int64_t>(slot) * heads + head) * key_dim) * value_dim + safe_column;
    float s[ROWS];
    bool valid[ROWS];
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        valid[m] = i < key_dim;
        s[m] = valid[m] ? mine[static_cast<int64_t>(i) * value_dim] : 0.0f;
    }
    // Nothing that is read from LDS may be a stray bit pattern: places that no load fills are read beside others.
    for (int index = lane; index < kScanBufferFloats; index += kWave) buffer_even[index] = buffer_odd[index] = 0.0f;
    __syncthreads();
    // Which token of a tile and which channel each of this lane's loads brings (the same for every tile).
    constexpr int kPiece = WIDE ? 4 : 1;                                  // floats a lane's load brings
    constexpr int kScanCalls = kScanTileFloats / (kWave * kPiece);       // loads that bring one of decays, keys, queries
    int token_of[kScanCalls], channel_of[kScanCalls];
#pragma unroll
    for (int j = 0; j < kScanCalls; ++j) {
        const int element = (j * kWave + lane) * kPiece;
        token_of[j] = element / row_floats;
        channel_of[j] = min(element % row_floats, key_dim - kPiece);
    }
    bool all_valid = true;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) all_valid = all_valid && valid[m];
    all_valid = __all(all_valid);
    const int value_calls = (tile_tokens * columns + kWave - 1) / kWave;
    auto fetch = [&](int tile_first, float* buffer) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < kScanCalls; ++j) {
            if (j * kWave * (WIDE ? 4 : 1) >= tile_tokens * row_floats) break;
            const int64_t token = min(tile_first + token_of[j], last - 1);
            constexpr int kPiece = WIDE ? 4 : 1;
            const float* row = proj + token * proj_stride + head * key_dim + channel_of[j];
            const float* decays = decay + token * decay_stride + head * key_dim + channel_of[j];
            float* place = buffer + j * kWave * kPiece;
            if constexpr (WIDE) {
                __builtin_amdgcn_global_load_lds(decays, place, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(row + k_offset, place + kScanTileFloats, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(row + q_offset, place + 2 * kScanTileFloats, 16, 0, 0);
            } else {
                __builtin_amdgcn_global_load_lds(decays, place, 4, 0, 0);
                __builtin_amdgcn_global_load_lds(row + k_offset, place + kScanTileFloats, 4, 0, 0);
                __builtin_amdgcn_global_load_lds(row + q_offset, place + 2 * kScanTileFloats, 4, 0, 0);
            }
        }
        for (int j = 0; j < value_calls; ++j) {
            const int element = j * kWave + lane;
            const int64_t token = min(tile_first + element / columns, last - 1);
            const int wanted = min(static_cast<int>(blockIdx.z) * columns + element % columns, value_dim - 1);
            __builtin_amdgcn_global_load_lds(proj + token * proj_stride + v_offset + head * value_dim + wanted,
                                             buffer + 3 * kScanTileFloats + j * kWave, 4, 0, 0);
        }
    };
    auto walk_tokens = [&](auto every_channel, int count, const float* buffer) __attribute__((always_inline)) {
#pragma unroll 4
        for (int t = 0; t < count; ++t) {
            const float* row = buffer + t * row_floats + ROWS * r;
            float a[ROWS], k[ROWS], q[ROWS];
#pragma unroll
            for (int piece = 0; piece < ROWS; piece += 4) {
                *reinterpret_cast<float4*>(a + piece) = *reinterpret_cast<const float4*>(row + piece);
                *reinterpret_cast<float4*>(k + piece) = *reinterpret_cast<const float4*>(row + kScanTileFloats + piece);
                *reinterpret_cast<float4*>(q + piece) = *reinterpret_cast<const float4*>(row + 2 * kScanTileFloats + piece);
            }
            const float v = buffer[3 * kScanTileFloats + t * columns + column_in_group];
            float partial = 0.0f;
#pragma unroll
            for (int m = 0; m < ROWS; ++m) {
                s[m] = fmaf(a[m], s[m], ((decltype(every_channel)::value || valid[m]) ? k[m] : 0.0f) * v);
                partial = fmaf(s[m], q[m], partial);
            }
            lane_sums[t * kWave + lane] = partial;
        }
    };
    auto walk = [&](int tile_first, const float* buffer) __attribute__((always_inline)) {
        const int count = min(tile_tokens, last - tile_first);
        if (all_valid) walk_tokens(std::true_type{}, count, buffer);
        else walk_tokens(std::false_type{}, count, buffer);
        __syncthreads();
        // The tile's results: a column's lanes' sums added in lane order, a result a lane, neighbours' columns by neighbours.
        for (int result = lane; result < count * columns; result += kWave) {
            const int t = result / columns, in_group = result % columns;
            const int wanted = blockIdx.z * columns + in_group;
            const float* sums = lane_sums + t * kWave + in_group * lanes_a_column;
            float total = 0.0f;
            if (lanes_a_column % 4 == 0) {
                for (int other = 0; other < lanes_a_column; other += 4) {
                    const float4 four = *reinterpret_cast<const float4*>(sums + other);
                    total = (((total + four.x) + four.y) + four.z) + four.w;
                }
            } else {
                for (int other = 0; other < lanes_a_column; ++other) total += sums[other];
            }
            if (wanted < value_dim) out[(static_cast<int64_t>(tile_first + t) * heads + head) * value_dim + wanted] = total * q_scale;
        }
        __syncthreads();      // before the next tile's sums are written
    };
    fetch(first, buffer_even);
    for (int tile_first = first; tile_first < last;) {
        wait_for_loads();
        __syncthreads();
        if (tile_first + tile_tokens < last) fetch(tile_first + tile_tokens, buffer_odd);
        walk(tile_first, buffer_even);
        tile_first += tile_tokens;
        if (tile_first >= last) break;
        wait_for_loads();
        __syncthreads();
        if (tile_first + tile_tokens < last) fetch(tile_first + tile_tokens, buffer_even);
        walk(tile_first, buffer_odd);
        tile_first += tile_tokens;
    }
    if (!live) return;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
        const int i = ROWS * r + m;
        if (i < key_dim) mine[static_cast<int64_t>(i) * value_dim] = s[m];
    }
}

// out[t, head, :] = rms_norm(o[t, head, :]) * weight * silu(gate[t, head, :]) * out_scale (weight null: none); one wave a (token, head).
template <typename T>
__global__ void __launch_bounds__(kWave)
gla_gate_kernel(const float* __restrict__ o, const float* __restrict__ proj, int64_t proj_stride, int gate_offset,
                const float* __restrict__ weight, float eps, T* __restrict__ out, int64_t out_stride, int heads,
                int value_dim, float out_scale) {
    const int token = blockIdx.x / heads;
    const int head = blockIdx.x % heads;
    const int lane = threadIdx.x;
    const float* row = o + (static_cast<int64_t>(token) * heads + head) * value_dim;
    const float* gate = proj + static_cast<int64_t>(token) * proj_stride + gate_offset + head * value_dim;
    float squares = 0.0f;
    for (int c = lane; c < value_dim; c += kWave) squares += row[c] * row[c];
    const float factor = 1.0f / sqrtf(wave_sum(squares) / static_cast<float>(value_dim) + eps);
    T* to = out + static_cast<int64_t>(token) * out_stride + head * value_dim;
    for (int c = lane; c < value_dim; c += kWave) {
        const float g = gate[c];
        const float silu = g / (1.0f + expf(-g));
        to[c] = from_float<T>((weight ? row[c] * factor * weight[c] : row[c] * factor) * silu * out_scale);
    }
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_gla_decay(const float* proj, int64_t proj_stride, int low_offset, int rank, const void* a2, int a2_dtype,
                  const float* bias, float tau, float* decay, int n_tokens, int channels, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && channels > 0 && rank > 0 && tau > 0.0f, "gla_decay: sizes and tau must be positive");
    MLL_REQUIRE(low_offset >= 0 && low_offset + rank <= proj_stride, "gla_decay: the low-rank input lies outside its row");
    if (n_tokens == 0) return 0;
    MLL_REQUIRE(n_tokens <= 65535, "gla_decay: more than 65535 tokens in one call");
    const dim3 grid((channels + 127) / 128, n_tokens);
    if (a2_dtype == kF32) {
        gla_decay_kernel<float><<<grid, 128, 0, stream>>>(proj, proj_stride, low_offset, rank, static_cast<const float*>(a2), bias,
                                                         1.0f / tau, decay, channels);
    } else if (a2_dtype == kBF16) {
        gla_decay_kernel<bf16><<<grid, 128, 0, stream>>>(proj, proj_stride, low_offset, rank, static_cast<const bf16*>(a2), bias,
                                                        1.0f / tau, decay, channels);
    } else {
        return fail("gla_decay: unknown weight dtype");
    }
    return check_launch("gla_decay");
}

int mll_gla_scan(const float* proj, int64_t proj_stride, int q_offset, int k_offset, int v_offset, const float* decay,
                 float* state, const int32_t* cu_tokens, const int32_t* slots, float* out, int n_seqs, int heads, int key_dim,
                 int value_dim, float q_scale, int long_portions, int64_t decay_stride, hipStream_t stream) {
    MLL_REQUIRE(n_seqs >= 0 && heads > 0 && key_dim > 0 && value_dim > 0, "gla_scan: sizes must be positive");
    MLL_REQUIRE(key_dim <= kWideHeadRows * kWave, "gla_scan: key heads wider than 512 are not supported");
    MLL_REQUIRE(q_offset >= 0 && k_offset >= 0 && v_offset >= 0 && q_offset + heads * key_dim <= proj_stride &&
                    k_offset + heads * key_dim <= proj_stride && v_offset + heads * value_dim <= proj_stride,
                "gla_scan: a projection lies outside its row");
    MLL_REQUIRE(decay_stride == 0 || decay_stride >= static_cast<int64_t>(heads) * key_dim,
                "gla_scan: the decays of a token are heads * key_dim numbers; a stride of 0 gives every token the same");
    if (n_seqs == 0) return 0;
    const int rows = key_dim <= kUsualRows * kWave ? kUsualRows : kWideHeadRows;
    int lanes_a_column = 1;
    while (lanes_a_column * rows < key_dim) lanes_a_column <<= 1;
    const int columns_a_wave = kWave / lanes_a_column;
    MLL_REQUIRE(n_seqs <= 65535 * 32 && heads <= 65535, "gla_scan: too many requests or heads for one launch");
    const dim3 grid(n_seqs, heads, (value_dim + columns_a_wave - 1) / columns_a_wave);
    if (long_portions) {
        const int row_floats = (key_dim + 7) / 8 * 8;
        int tile_tokens = kScanTileFloats / row_floats;
        if (tile_tokens * columns_a_wave > kScanTileFloats) tile_tokens = kScanTileFloats / columns_a_wave;
        if (tile_tokens > 64) tile_tokens = 64;
        const bool wide = key_dim % 8 == 0 && proj_stride % 4 == 0 && q_offset % 4 == 0 && k_offset % 4 == 0 &&
                          reinterpret_cast<uintptr_t>(proj) % 16 == 0 && reinterpret_cast<uintptr_t>(decay) % 16 == 0 &&
                          decay_stride % 4 == 0;
#define MLL_SCAN_TILED(WIDE, ROWS)                                                                                         \
    gla_scan_tiled_kernel<WIDE, ROWS><<<grid, kWave, 0, stream>>>(proj, proj_stride, q_offset, k_offset, v_offset, decay, state, \
                                                                 cu_tokens, slots, out, heads, key_dim, value_dim,              \
                                                                 lanes_a_column, tile_tokens, q_scale, decay_stride)
        if (wide && rows == kUsualRows) MLL_SCAN_TILED(true, kUsualRows);
        else if (wide) MLL_SCAN_TILED(true, kWideHeadRows);
        else if (rows == kUsualRows) MLL_SCAN_TILED(false, kUsualRows);
        else MLL_SCAN_TILED(false, kWideHeadRows);
#undef MLL_SCAN_TILED
        return check_launch("gla_scan_tiled");
    }
    if (rows == kUsualRows) {
        gla_scan_kernel<kUsualRows><<<grid, kWave, 0, stream>>>(proj, proj_stride, q_offset, k_offset, v_offset, decay, state, cu_tokens,
                                                               slots, out, heads, key_dim, value_dim, lanes_a_column, q_scale, decay_stride);
    } else {
        gla_scan_kernel<kWideHeadRows><<<grid, kWave, 0, stream>>>(proj, proj_stride, q_offset, k_offset, v_offset, decay, state, cu_tokens,
                                                                  slots, out, heads, key_dim, value_dim, lanes_a_column, q_scale, decay_stride);
    }
    return check_launch("gla_scan");
}

int mll_gla_gate(const float* o, const float* proj, int64_t proj_stride, int gate_offset, const float* weight, float eps,
                 void* out, int64_t out_stride, int dtype, int n_tokens, int heads, int value_dim, float out_scale,
                 hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && heads > 0 && value_dim > 0 && eps > 0.0f, "gla_gate: sizes and eps must be positive");
    MLL_REQUIRE(gate_offset >= 0 && gate_offset + heads * value_dim <= proj_stride, "gla_gate: the gate lies outside its row");
    MLL_REQUIRE(out_stride >= static_cast<int64_t>(heads) * value_dim, "gla_gate: the output rows overlap");
    if (n_tokens == 0) return 0;
    const int64_t blocks = static_cast<int64_t>(n_tokens) * heads;
    MLL_REQUIRE(blocks < (1ll << 31), "gla_gate: too many rows for one launch");
    if (dtype == kF32) {
        gla_gate_kernel<float><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(o, proj, proj_stride, gate_offset, weight, eps,
                                                                                   static_cast<float*>(out), out_stride, heads, value_dim, out_scale);
    } else if (dtype == kBF16) {
        gla_gate_kernel<bf16><<<static_cast<unsigned>(blocks), kWave, 0, stream>>>(o, proj, proj_stride, gate_offset, weight, eps,
                                                                                  static_cast<bf16*>(out), out_stride, heads, value_dim, out_scale);
    } else {
        return fail("gla_gate: unknown dtype");
    }
    return check_launch("gla_gate");
}

}  // extern "C"
