// A mixture of experts: the choice of every token's experts from router logits, and the experts' gated
// feed-forwards for (token, choice) pairs whose expert is only known on the device. An expert is gated,
// Wd (act(Wg x) * (Wu x)), or has one inner weight, Wd act(Wu x); act is chosen by number (common.h).
//
// Choice: scores are sigmoid(z) or softmax(z) over the experts, the `top` largest are taken (ties: the lower
// index), their weights are the scores, optionally divided by their sum. Everything float32.
//
// Experts, plain kernels: a workgroup takes one (token, choice) pair and a stretch of the expert's output rows; a
// wave forms one output at a time with its lanes along the reduction (16-byte loads of the weight's row), so a
// pair's sums never depend on the other pairs. These serve every dtype and number of tokens; their cost per pair is
// one reading of the expert's weights, which is what decoding a few tokens costs anyway.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kMaxTop = 16;

// One thread a token (taken beyond 256 experts; fewer go to the kernel below, a wave a token). z: float32 rows, z_stride apart, experts first; a further column `shared_at` (negative: none)
// holds the logit of the shared expert's gate, whose sigmoid goes to shared_gate[t].
__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ z, int64_t z_stride, int n_tokens, int experts, int top, int softmax_scores,
                 int renormalize, int shared_at, int32_t* __restrict__ ids, float* __restrict__ weights,
                 float* __restrict__ shared_gate, int groups, int keep) {
    const int token = blockIdx.x * blockDim.x + threadIdx.x;
    if (token >= n_tokens) return;
    const float* row = z + static_cast<int64_t>(token) * z_stride;
    float peak = -INFINITY, total = 1.0f;
    if (softmax_scores) {
        for (int e = 0; e < experts; ++e) peak = fmaxf(peak, row[e]);
        total = 0.0f;
        for (int e = 0; e < experts; ++e) total += expf(row[e] - peak);
    }
    // Groups of neighbouring experts: a group counts as much as its best expert, and only the experts of the `keep`
    // best groups (ties: the lower group) can be chosen. A bit a group (at most 64).
    unsigned long long open_groups = ~0ull;
    const int group_size = groups > 0 ? experts / groups : experts;
    if (groups > 0 && keep < groups) {
        open_groups = 0ull;
        for (int n = 0; n < keep; ++n) {
            int best_group = -1;
            float best_logit = 0.0f;
            for (int g = 0; g < groups; ++g) {
                if ((open_groups >> g) & 1ull) continue;
                float top_logit = row[g * group_size];
                for (int e = 1; e < group_size; ++e) top_logit = fmaxf(top_logit, row[g * group_size + e]);
                if (best_group < 0 || top_logit > best_logit) {
                    best_group = g;
                    best_logit = top_logit;
                }
            }
            open_groups |= 1ull << best_group;
        }
    }
    int chosen[kMaxTop];
    float taken[kMaxTop];
    float sum = 0.0f;
    for (int n = 0; n < top; ++n) {
        int best = -1;
        float best_logit = 0.0f;
        for (int e = 0; e < experts; ++e) {
            bool used = false;
            for (int m = 0; m < n; ++m) used = used || chosen[m] == e;
            if (used || (groups > 0 && !((open_groups >> (e / group_size)) & 1ull))) continue;
            // the scores rise with the logits, so the largest logit is the largest score; a logit that is no number is never larger
            if (best < 0 || row[e] > best_logit) {
                best = e;
                best_logit = row[e];
            }
        }
        chosen[n] = best;
        taken[n] = softmax_scores ? expf(best_logit - peak) / total : 1.0f / (1.0f + expf(-best_logit));
        sum += taken[n];
    }
    for (int n = 0; n < top; ++n) {
        ids[static_cast<int64_t>(token) * top + n] = chosen[n];
        weights[static_cast<int64_t>(token) * top + n] = renormalize ? taken[n] / sum : taken[n];
    }
    if (shared_at >= 0 && shared_gate != nullptr) shared_gate[token] = 1.0f / (1.0f + expf(-row[shared_at]));
}

// The same choice by one wave a token, for up to 64 * PER experts: lane l holds the experts l, l + 64, ...; maxima,
// sums and every "largest of what is left" are taken across the wave, ties to the lower index. The scores' sum is
// added in the wave's order, not in the experts'; everything else is the arithmetic of the kernel above, and a token's
// result depends on its own row alone.
struct Candidate {
    float value;
    int index;
};

__device__ inline Candidate wave_best(Candidate mine) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        const float value = __shfl_xor(mine.value, offset, kWave);
        const int index = __shfl_xor(mine.index, offset, kWave);
        const bool better = index >= 0 && (mine.index < 0 || value > mine.value || (value == mine.value && index < mine.index));
        if (better) {
            mine.value = value;
            mine.index = index;
        }
    }
    return mine;
}

template <int PER>
__global__ void __launch_bounds__(kWave)
moe_route_wave_kernel(const float* __restrict__ z, int64_t z_stride, int experts, int top, int softmax_scores, int renormalize,
                      int shared_at, int32_t* __restrict__ ids, float* __restrict__ weights, float* __restrict__ shared_gate,
                      int groups, int keep) {
    const int token = blockIdx.x, lane = threadIdx.x;
    const float* row = z + static_cast<int64_t>(token) * z_stride;
    float logit[PER];
    bool free_to_take[PER];
    float peak = -INFINITY;
#pragma unroll
    for (int n = 0; n < PER; ++n) {
        const int e = lane + n * kWave;
        const float value = e < experts ? row[e] : -INFINITY;
        logit[n] = value != value ? -INFINITY : value;       // a logit that is no number is never the largest
        free_to_take[n] = e < experts;
        peak = fmaxf(peak, logit[n]);
    }
    float total = 1.0f;
    if (softmax_scores) {
        peak = wave_max(peak);
        float part = 0.0f;
#pragma unroll
        for (int n = 0; n < PER; ++n)
            if (lane + n * kWave < experts) part += expf(logit[n] - peak);
        total = wave_sum(part);
    }
    if (groups > 0 && keep < groups) {
        // lane g learns group g's largest logit; then the best `keep` groups are opened, one after the other
        const int group_size = experts / groups;
        float group_top = -INFINITY;
        for (int g = 0; g < groups; ++g) {
            float inside = -INFINITY;
#pragma unroll
            for (int n = 0; n < PER; ++n) {
                const int e = lane + n * kWave;
                if (e < experts && e / group_size == g) inside = fmaxf(inside, logit[n]);
            }
            inside = wave_max(inside);
            if (lane == g) group_top = inside;
        }
        unsigned long long open_groups = 0ull;
        for (int n = 0; n < keep; ++n) {
            Candidate mine = {group_top, (lane < groups && !((open_groups >> lane) & 1ull)) ? lane : -1};
            open_groups |= 1ull << wave_best(mine).index;
        }
#pragma unroll
        for (int n = 0; n < PER; ++n) {
            const int e = lane + n * kWave;
            free_to_take[n] = free_to_take[n] && ((open_groups >> (e / group_size)) & 1ull);
        }
    }
    float sum = 0.0f, my_weight = 0.0f;
    int my_id = 0;
    for (int choice = 0; choice < top; ++choice) {
        Candidate mine = {-INFINITY, -1};
#pragma unroll
        for (int n = 0; n < PER; ++n)       // ascending index: of equal logits the lower stays
            if (free_to_take[n] && (mine.index < 0 || logit[n] > mine.value)) mine = {logit[n], lane + n * kWave};
        const Candidate best = wave_best(mine);
#pragma unroll
        for (int n = 0; n < PER; ++n)
            if (lane + n * kWave == best.index) free_to_take[n] = false;
        const float taken = softmax_scores ? expf(best.value - peak) / total : 1.0f / (1.0f + expf(-best.value));
        sum += taken;
        if (lane == choice) {
            my_weight = taken;
            my_id = best.index;
        }
    }
    if (lane < top) {
        ids[static_cast<int64_t>(token) * top + lane] = my_id;
        weights[static_cast<int64_t>(token) * top + lane] = renormalize ? my_weight / sum : my_weight;
    }
    if (lane == 0 && shared_at >= 0 && shared_gate != nullptr) shared_gate[token] = 1.0f / (1.0f + expf(-row[shared_at]));
}

template <typename T> __device__ inline float row_dot(const T* __restrict__ w, const float* __restrict__ x, int k, int lane);

template <> __device__ inline float row_dot<float>(const float* __restrict__ w, const float* __restrict__ x, int k, int lane) {
    float sum = 0.0f;
    if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        for (int c = lane * 4; c < k; c += kWave * 4) {
            const float4 v = *reinterpret_cast<const float4*>(w + c);
            sum = fmaf(v.x, x[c], sum);
            sum = fmaf(v.y, x[c + 1], sum);
            sum = fmaf(v.z, x[c + 2], sum);
            sum = fmaf(v.w, x[c + 3], sum);
        }
    } else {
        for (int c = lane; c < k; c += kWave) sum = fmaf(w[c], x[c], sum);
    }
    return wave_sum(sum);
}

template <> __device__ inline float row_dot<bf16>(const bf16* __restrict__ w, const float* __restrict__ x, int k, int lane) {
    float sum = 0.0f;
    if ((k & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        for (int c = lane * 8; c < k; c += kWave * 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(w + c);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sum = fmaf(__builtin_bit_cast(float, words[i] << 16), x[c + 2 * i], sum);
                sum = fmaf(__builtin_bit_cast(float, words[i] & 0xffff0000u), x[c + 2 * i + 1], sum);
            }
        }
    } else {
        for (int c = lane; c < k; c += kWave) sum = fmaf(to_float(w[c]), x[c], sum);
    }
    return wave_sum(sum);
}

// Four rows against the same x at once: four loads on their way a lane instead of one. Each row's sum is formed
// exactly as row_dot forms it (the same terms in the same order), so a pair's result does not depend on which rows
// happen to go together.
template <typename T> __device__ inline void rows_dot4(const T* const (&w)[4], const float* __restrict__ x, int k, int lane, float (&out)[4]);

template <> __device__ inline void rows_dot4<float>(const float* const (&w)[4], const float* __restrict__ x, int k, int lane, float (&out)[4]) {
#pragma unroll
    for (int n = 0; n < 4; ++n) out[n] = row_dot<float>(w[n], x, k, lane);
}

template <> __device__ inline void rows_dot4<bf16>(const bf16* const (&w)[4], const float* __restrict__ x, int k, int lane, float (&out)[4]) {
    bool fast = (k & 7) == 0;
#pragma unroll
    for (int n = 0; n < 4; ++n) fast = fast && (reinterpret_cast<uintptr_t>(w[n]) & 15) == 0;
    if (!fast) {
#pragma unroll
        for (int n = 0; n < 4; ++n) out[n] = row_dot<bf16>(w[n], x, k, lane);
        return;
    }
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = lane * 8; c < k; c += kWave * 8) {
        typedef unsigned int uintx4_t __attribute__((ext_vector_type(4)));
        uintx4_t raw[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) raw[n] = __builtin_nontemporal_load(reinterpret_cast<const uintx4_t*>(w[n] + c));
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const uint32_t words[4] = {raw[n][0], raw[n][1], raw[n][2], raw[n][3]};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sum[n] = fmaf(__builtin_bit_cast(float, words[i] << 16), x[c + 2 * i], sum[n]);
                sum[n] = fmaf(__builtin_bit_cast(float, words[i] & 0xffff0000u), x[c + 2 * i + 1], sum[n]);
            }
        }
    }
#pragma unroll
    for (int n = 0; n < 4; ++n) out[n] = wave_sum(sum[n]);
}

// z[t][e] = w[e] . x[t], float32 sums: a workgroup takes a token and four rows of w, a wave a row.
template <typename T>
__global__ void __launch_bounds__(256)
router_logits_kernel(const T* __restrict__ x, const float* __restrict__ w, float* __restrict__ z, int n_out, int width) {
    extern __shared__ float xs[];
    const int token = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) xs[c] = to_float(x[static_cast<int64_t>(token) * width + c]);
    __syncthreads();
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int e = blockIdx.y * (blockDim.x / kWave) + wave;     // a wave a row of w
    if (e >= n_out) return;
    const float value = row_dot<float>(w + static_cast<int64_t>(e) * width, xs, width, lane);
    if (lane == 0) z[static_cast<int64_t>(token) * n_out + e] = value;
}

constexpr int kExpertWaves = 4;
constexpr int kExpertRowsAWave = 8;     // outputs a wave forms one after the other
constexpr int kExpertRowsABlock = kExpertWaves * kExpertRowsAWave;

// act[pair][f] = silu(Wg_e[f] . xs) * (Wu_e[f] . xs), xs = x[token] * weight[pair] rounded to T (the weight
// multiplies the expert's input) or x[token] (weight_on_input 0). gate_up: [experts][2 * ff][width], gate rows first.
template <typename T>
__global__ void __launch_bounds__(kExpertWaves * kWave)
moe_gate_up_kernel(const T* __restrict__ x, const int32_t* __restrict__ ids, const float* __restrict__ weights, int top,
                   const T* __restrict__ gate_up, T* __restrict__ act, int width, int ff, int weight_on_input, int gated,
                   int activation) {
    extern __shared__ float xs[];
    const int pair = blockIdx.y;
    const int token = pair / top;
    const int expert = ids[pair];
    const float factor = weight_on_input ? weights[pair] : 1.0f;
    for (int c = threadIdx.x; c < width; c += blockDim.x)
        xs[c] = to_float(from_float<T>(to_float(x[static_cast<int64_t>(token) * width + c]) * factor));
    __syncthreads();
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    if (!gated) {       // act[pair][f] = activation(Wu_e[f] . xs); gate_up is [experts][ff][width]
        const T* up = gate_up + static_cast<int64_t>(expert) * ff * width;
        for (int n = 0; n < kExpertRowsAWave; n += 4) {
            const int f = blockIdx.x * kExpertRowsABlock + wave * kExpertRowsAWave + n;
            if (f >= ff) break;
            const T* const rows[4] = {up + static_cast<int64_t>(f) * width, up + static_cast<int64_t>(min(f + 1, ff - 1)) * width,
                                      up + static_cast<int64_t>(min(f + 2, ff - 1)) * width, up + static_cast<int64_t>(min(f + 3, ff - 1)) * width};
            float sums[4];
            rows_dot4<T>(rows, xs, width, lane, sums);
            if (lane == 0) {
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    if (f + m < ff) act[static_cast<int64_t>(pair) * ff + f + m] = from_float<T>(activate(sums[m], activation));
            }
        }
        return;
    }
    const T* base = gate_up + static_cast<int64_t>(expert) * 2 * ff * width;
    for (int n = 0; n < kExpertRowsAWave; n += 2) {      // two outputs at a time: their gate and up rows are four rows
        const int f = blockIdx.x * kExpertRowsABlock + wave * kExpertRowsAWave + n;
        if (f >= ff) break;
        const int second = min(f + 1, ff - 1);
        const T* const rows[4] = {base + static_cast<int64_t>(f) * width, base + static_cast<int64_t>(ff + f) * width,
                                  base + static_cast<int64_t>(second) * width, base + static_cast<int64_t>(ff + second) * width};
        float sums[4];
        rows_dot4<T>(rows, xs, width, lane, sums);
        if (lane == 0) {
            act[static_cast<int64_t>(pair) * ff + f] = from_float<T>(activate(sums[0], activation) * sums[1]);
            if (f + 1 < ff) act[static_cast<int64_t>(pair) * ff + f + 1] = from_float<T>(activate(sums[2], activation) * sums[3]);
        }
    }
}

// out[choice][token][c] = (Wd_e[c] . act[pair]) (* weight[pair] with weight_on_input 0): float32 [top][tokens][width],
// partial sums that the reader adds in order. down: [experts][width][ff].
template <typename T>
__global__ void __launch_bounds__(kExpertWaves * kWave)
moe_down_kernel(const T* __restrict__ act, const int32_t* __restrict__ ids, const float* __restrict__ weights, int top,
                const T* __restrict__ down, float* __restrict__ out, int n_tokens, int width, int ff, int weight_on_input) {
    extern __shared__ float as[];
    const int pair = blockIdx.y;
    const int token = pair / top, choice = pair % top;
    const int expert = ids[pair];
    for (int c = threadIdx.x; c < ff; c += blockDim.x) as[c] = to_float(act[static_cast<int64_t>(pair) * ff + c]);
    __syncthreads();
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const T* base = down + static_cast<int64_t>(expert) * width * ff;
    const float factor = weight_on_input ? 1.0f : weights[pair];
    for (int n = 0; n < kExpertRowsAWave; n += 4) {
        const int c = blockIdx.x * kExpertRowsABlock + wave * kExpertRowsAWave + n;
        if (c >= width) break;
        const T* rows[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) rows[m] = base + static_cast<int64_t>(min(c + m, width - 1)) * ff;
        const T* const fixed[4] = {rows[0], rows[1], rows[2], rows[3]};
        float sums[4];
        rows_dot4<T>(fixed, as, ff, lane, sums);
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < 4; ++m)
                if (c + m < width) out[(static_cast<int64_t>(choice) * n_tokens + token) * width + c + m] = sums[m] * factor;
        }
    }
}

// out[t][c] = factor[t] * sum over parts of in[part][t][c], float32.
__global__ void __launch_bounds__(256)
scale_rows_kernel(const float* __restrict__ in, int n_parts, int64_t part_stride, const float* __restrict__ factor,
                  float* __restrict__ out, int width) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int64_t at = static_cast<int64_t>(token) * width + c;
    float value = in[at];
    for (int part = 1; part < n_parts; ++part) value += in[part * part_stride + at];
    out[at] = value * factor[token];
}

// ---- many pairs: rows sorted by expert and tiled MFMA products ---------------------------------------------------
// With many (token, choice) pairs the pairs are put in the order of their experts (stable: a pair keeps its place
// among its expert's), their inputs are gathered (and multiplied by their weights) into that order, and every expert
// multiplies its own stretch of rows: a workgroup takes a tile of up to 128 rows of one expert and 128 of its weight's
// rows, stages both through LDS in steps of 64 of the reduction and forms the products with
// v_mfma_f32_16x16x32_bf16 (four waves, 64 x 64 each). Which expert a tile belongs to is read from the device-side
// offsets; the grid has a tile for every case (pairs / 128 + experts), and tiles beyond the last expert's leave at once.
// A row's sums do not depend on the other rows of its tile.

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(kWave)
moe_count_kernel(const int32_t* __restrict__ ids, int n_pairs, int32_t* __restrict__ counts) {
    const int expert = blockIdx.x, lane = threadIdx.x;
    int count = 0;
    for (int p = lane; p < n_pairs; p += kWave) count += ids[p] == expert ? 1 : 0;
    for (int offset = kWave / 2; offset > 0; offset >>= 1) count += __shfl_xor(count, offset, kWave);
    if (lane == 0) counts[expert] = count;
}

// offsets[e] = pairs of the experts before e; order[offsets[e] + n] = the n-th pair (ascending) that chose e.
__global__ void __launch_bounds__(kWave)
moe_order_kernel(const int32_t* __restrict__ ids, int n_pairs, int experts, const int32_t* __restrict__ counts,
                 int32_t* __restrict__ offsets, int32_t* __restrict__ order) {
    const int expert = blockIdx.x, lane = threadIdx.x;
    int base = 0;
    for (int e = 0; e < expert; ++e) base += counts[e];
    if (lane == 0) {
        offsets[expert] = base;
        if (expert == experts - 1) offsets[experts] = base + counts[expert];
    }
    int running = 0;
    for (int first = 0; first < n_pairs; first += kWave) {
        const int p = first + lane;
        const bool mine = p < n_pairs && ids[p] == expert;
        const unsigned long long mask = __ballot(mine);
        if (mine) order[base + running + __popcll(mask & ((1ull << lane) - 1ull))] = p;
        running += __popcll(mask);
    }
}

// sorted[row] = x[token of order[row]] (* weight of the pair), rounded to bfloat16.
__global__ void __launch_bounds__(256)
moe_gather_kernel(const bf16* __restrict__ x, const int32_t* __restrict__ order, const float* __restrict__ weights, int top,
                  bf16* __restrict__ sorted, int width, int weight_on_input) {
    const int row = blockIdx.x;
    const int pair = order[row];
    const float factor = weight_on_input ? weights[pair] : 1.0f;
    const bf16* from = x + static_cast<int64_t>(pair / top) * width;
    bf16* to = sorted + static_cast<int64_t>(row) * width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) to[c] = from_float<bf16>(to_float(from[c]) * factor);
}

constexpr int kGroupRows = 128, kGroupCols = 128, kGroupStep = 64, kGroupPad = 72;     // rows of a tile lie 144 bytes apart in LDS: 16-byte reads of 16 rows meet no bank twice

// FORM 2: w is [experts][n_out][k] and out (bfloat16 [pairs][n_out], sorted order) gets activation(product).
// FORM 1 (GATED): w is [experts][2 * n_half][k] (gate rows, then up rows); a tile holds 64 gate rows and the 64 up rows that
// belong to them, and out (bfloat16 [pairs][n_half], sorted order) gets silu(gate) * up. Otherwise w is
// [experts][n_out][k] and out (float32 [top][n_tokens][n_out]) gets the product at the pair's token and choice,
// times the pair's weight unless that multiplied the input.
template <int FORM>
__global__ void __launch_bounds__(256)
moe_grouped_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w, const int32_t* __restrict__ offsets,
                   const int32_t* __restrict__ order, const float* __restrict__ weights, int experts, int n_out, int k,
                   void* __restrict__ out, int top, int n_tokens, int weight_on_input, int activation) {
    constexpr bool GATED = FORM == 1;
    __shared__ __attribute__((aligned(16))) bf16 a_tile[kGroupRows * kGroupPad];
    __shared__ __attribute__((aligned(16))) bf16 w_tile[kGroupCols * kGroupPad];
    int expert = 0, first_row = 0, rows = 0, before = 0;
    for (; expert < experts; ++expert) {
        const int begin = offsets[expert], end = offsets[expert + 1];
        const int tiles = (end - begin + kGroupRows - 1) / kGroupRows;
        if (static_cast<int>(blockIdx.y) < before + tiles) {
            first_row = begin + (blockIdx.y - before) * kGroupRows;
            rows = min(kGroupRows, end - first_row);
            break;
        }
        before += tiles;
    }
    if (rows == 0) return;      // a tile beyond the last expert's (the same for every thread of the workgroup)
    const int w_rows = GATED ? 2 * n_out : n_out;
    const bf16* w_expert = w + static_cast<int64_t>(expert) * w_rows * k;
    const int col0 = blockIdx.x * (GATED ? 64 : kGroupCols);
    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int wm = wave / 2, wn = wave % 2, r = lane % 16, quad = lane / 16;

    // what this thread brings into LDS each step: four 16-byte pieces of the rows' tile and four of the weight's
    constexpr int kPieces = kGroupRows * (kGroupStep / 8) / 256;
    const bf16* a_from[kPieces];
    const bf16* w_from[kPieces];
    int lds_at[kPieces];
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
        const int piece = t + i * 256, row = piece / (kGroupStep / 8), segment = piece % (kGroupStep / 8);
        lds_at[i] = row * kGroupPad + segment * 8;
        a_from[i] = row < rows ? a + static_cast<int64_t>(first_row + row) * k + segment * 8 : nullptr;
        int w_row;
        bool live;
        if (GATED) {
            const int column = col0 + row % 64;
            live = column < n_out;
            w_row = row < 64 ? column : n_out + column;
        } else {
            w_row = col0 + row;
            live = w_row < n_out;
        }
        w_from[i] = live ? w_expert + static_cast<int64_t>(w_row) * k + segment * 8 : nullptr;
    }
    floatx4_t acc[4][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
    int w_base[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) w_base[nt] = GATED ? (nt < 2 ? wn * 32 + nt * 16 : 64 + wn * 32 + (nt - 2) * 16) : wn * 64 + nt * 16;

    uint4 a_next[kPieces], w_next[kPieces];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int segment = (t + i * 256) % (kGroupStep / 8);
            const bool in_k = k0 + segment * 8 < k;        // k is a multiple of 8: a piece is whole or absent
            a_next[i] = (a_from[i] != nullptr && in_k) ? *reinterpret_cast<const uint4*>(a_from[i] + k0) : make_uint4(0u, 0u, 0u, 0u);
            w_next[i] = (w_from[i] != nullptr && in_k) ? *reinterpret_cast<const uint4*>(w_from[i] + k0) : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < k; k0 += kGroupStep) {
        __syncthreads();        // the step before has read its tiles
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            *reinterpret_cast<uint4*>(a_tile + lds_at[i]) = a_next[i];
            *reinterpret_cast<uint4*>(w_tile + lds_at[i]) = w_next[i];
        }
        __syncthreads();
        if (k0 + kGroupStep < k) fetch(k0 + kGroupStep);      // on its way while this step's products run
#pragma unroll
        for (int half = 0; half < kGroupStep / 32; ++half) {
            bf16x8_t a_piece[4], w_piece[4];
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
                a_piece[mt] = *reinterpret_cast<const bf16x8_t*>(a_tile + (wm * 64 + mt * 16 + r) * kGroupPad + half * 32 + quad * 8);
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
                w_piece[nt] = *reinterpret_cast<const bf16x8_t*>(w_tile + (w_base[nt] + r) * kGroupPad + half * 32 + quad * 8);
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int nt = 0; nt < 4; ++nt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_piece[nt], a_piece[mt], acc[mt][nt], 0, 0, 0);
        }
    }
    // acc[mt][nt][i] of lane (r, quad): row wm * 64 + mt * 16 + r of the tile, weight row w_base[nt] + quad * 4 + i
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int row = wm * 64 + mt * 16 + r;
        if (row >= rows) continue;
        if (GATED) {
            bf16* to = static_cast<bf16*>(out) + static_cast<int64_t>(first_row + row) * n_out;
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = col0 + wn * 32 + nt * 16 + quad * 4 + i;
                    const float g = acc[mt][nt][i], u = acc[mt][nt + 2][i];
                    if (column < n_out) to[column] = from_float<bf16>(activate(g, activation) * u);
                }
        } else if (FORM == 2) {
            bf16* to = static_cast<bf16*>(out) + static_cast<int64_t>(first_row + row) * n_out;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = col0 + w_base[nt] + quad * 4 + i;
                    if (column < n_out) to[column] = from_float<bf16>(activate(acc[mt][nt][i], activation));
                }
        } else {
            const int pair = order[first_row + row];
            const float factor = weight_on_input ? 1.0f : weights[pair];
            float* to = static_cast<float*>(out) + (static_cast<int64_t>(pair % top) * n_tokens + pair / top) * n_out;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int column = col0 + w_base[nt] + quad * 4 + i;
                    if (column < n_out) to[column] = acc[mt][nt][i] * factor;
                }
        }
    }
}

}  // namespace mll

using namespace mll;

extern "C" {

int mll_moe_route(const float* z, int64_t z_stride, int n_tokens, int experts, int top, int softmax_scores, int renormalize,
                  int shared_at, int32_t* ids, float* weights, float* shared_gate, int groups, int keep, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && experts > 0 && top > 0 && top <= experts, "moe_route: 1 <= top <= experts");
    MLL_REQUIRE(top <= (experts <= 4 * kWave ? kWave : kMaxTop),
                "moe_route: at most 64 experts a token (16 where there are more than 256 experts)");
    MLL_REQUIRE(shared_at < 0 || shared_gate != nullptr, "moe_route: the shared expert's gate needs a place");
    MLL_REQUIRE(groups == 0 || (groups > 0 && groups <= 64 && experts % groups == 0 && keep >= 1 && keep <= groups &&
                                keep * (experts / groups) >= top),
                "moe_route: at most 64 equal groups, of which the kept ones hold at least `top` experts");
    if (n_tokens == 0) return 0;
#define MLL_ROUTE_WAVE(PER)                                                                                                  \
    moe_route_wave_kernel<PER><<<n_tokens, kWave, 0, stream>>>(z, z_stride, experts, top, softmax_scores, renormalize, shared_at, \
                                                              ids, weights, shared_gate, groups, keep)
    if (experts <= kWave) MLL_ROUTE_WAVE(1);
    else if (experts <= 2 * kWave) MLL_ROUTE_WAVE(2);
    else if (experts <= 4 * kWave) MLL_ROUTE_WAVE(4);
    else
        moe_route_kernel<<<(n_tokens + 63) / 64, 64, 0, stream>>>(z, z_stride, n_tokens, experts, top, softmax_scores, renormalize,
                                                                shared_at, ids, weights, shared_gate, groups, keep);
#undef MLL_ROUTE_WAVE
    return check_launch("moe_route");
}

int mll_moe_gate_up(const void* x, const int32_t* ids, const float* weights, int top, const void* gate_up, void* act,
                    int dtype, int n_tokens, int width, int ff, int weight_on_input, int gated, int activation,
                    hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && top > 0 && width > 0 && ff > 0, "moe_gate_up: sizes must be positive");
    MLL_REQUIRE(activation >= 0 && activation <= 2, "moe_gate_up: 0 SiLU, 1 gelu (erf), 2 gelu (tanh)");
    MLL_REQUIRE(static_cast<int64_t>(n_tokens) * top < 65536, "moe_gate_up: too many (token, expert) pairs for one launch");
    MLL_REQUIRE(static_cast<size_t>(width) * sizeof(float) <= 64 * 1024, "moe_gate_up: rows wider than 16384 are not supported");
    if (n_tokens == 0) return 0;
    const dim3 grid((ff + kExpertRowsABlock - 1) / kExpertRowsABlock, n_tokens * top);
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (dtype == kF32) {
        moe_gate_up_kernel<float><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const float*>(x), ids, weights, top, static_cast<const float*>(gate_up), static_cast<float*>(act), width, ff, weight_on_input, gated, activation);
    } else if (dtype == kBF16) {
        moe_gate_up_kernel<bf16><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const bf16*>(x), ids, weights, top, static_cast<const bf16*>(gate_up), static_cast<bf16*>(act), width, ff, weight_on_input, gated, activation);
    } else {
        return fail("moe_gate_up: unknown dtype");
    }
    return check_launch("moe_gate_up");
}

int mll_moe_down(const void* act, const int32_t* ids, const float* weights, int top, const void* down, float* out, int dtype,
                 int n_tokens, int width, int ff, int weight_on_input, hipStream_t stream) {
    return mll_moe_down_rows(act, ids, weights, top, down, out, dtype, n_tokens, n_tokens, width, ff, weight_on_input, stream);
}

int mll_moe_down_rows(const void* act, const int32_t* ids, const float* weights, int top, const void* down, float* out, int dtype,
                      int n_tokens, int part_tokens, int width, int ff, int weight_on_input, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && top > 0 && width > 0 && ff > 0 && part_tokens >= n_tokens, "moe_down: sizes must be positive");
    MLL_REQUIRE(static_cast<int64_t>(n_tokens) * top < 65536, "moe_down: too many (token, expert) pairs for one launch");
    MLL_REQUIRE(static_cast<size_t>(ff) * sizeof(float) <= 64 * 1024, "moe_down: experts wider than 16384 are not supported");
    if (n_tokens == 0) return 0;
    const dim3 grid((width + kExpertRowsABlock - 1) / kExpertRowsABlock, n_tokens * top);
    const size_t lds = static_cast<size_t>(ff) * sizeof(float);
    if (dtype == kF32) {
        moe_down_kernel<float><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const float*>(act), ids, weights, top, static_cast<const float*>(down), out, part_tokens, width, ff, weight_on_input);
    } else if (dtype == kBF16) {
        moe_down_kernel<bf16><<<grid, kExpertWaves * kWave, lds, stream>>>(
            static_cast<const bf16*>(act), ids, weights, top, static_cast<const bf16*>(down), out, part_tokens, width, ff, weight_on_input);
    } else {
        return fail("moe_down: unknown dtype");
    }
    return check_launch("moe_down");
}

int mll_scale_rows(const float* in, int n_parts, int64_t part_stride, const float* factor, float* out, int n_tokens, int width,
                   hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && width > 0 && n_parts >= 1, "scale_rows: sizes must be positive");
    MLL_REQUIRE(n_tokens < 65536, "scale_rows: too many rows for one launch");
    if (n_tokens == 0) return 0;
    scale_rows_kernel<<<dim3((width + 255) / 256, n_tokens), 256, 0, stream>>>(in, n_parts, part_stride, factor, out, width);
    return check_launch("scale_rows");
}

int mll_moe_grouped(const void* x, const int32_t* ids, const float* weights, int top, const void* gate_up, const void* down,
                    int32_t* counts, int32_t* offsets, int32_t* order, void* sorted, void* act, float* out, int n_tokens,
                    int experts, int width, int ff, int weight_on_input, int gated, int activation, hipStream_t stream) {
    MLL_REQUIRE(n_tokens > 0 && top > 0 && experts > 0 && width > 0 && ff > 0, "moe_grouped: sizes must be positive");
    MLL_REQUIRE(activation >= 0 && activation <= 2, "moe_grouped: 0 SiLU, 1 gelu (erf), 2 gelu (tanh)");
    MLL_REQUIRE(width % 8 == 0 && ff % 8 == 0, "moe_grouped: widths must be multiples of 8");
    const int64_t pairs = static_cast<int64_t>(n_tokens) * top;
    MLL_REQUIRE(pairs < (1 << 30), "moe_grouped: too many (token, expert) pairs");
    const int n_pairs = static_cast<int>(pairs);
    moe_count_kernel<<<experts, kWave, 0, stream>>>(ids, n_pairs, counts);
    moe_order_kernel<<<experts, kWave, 0, stream>>>(ids, n_pairs, experts, counts, offsets, order);
    moe_gather_kernel<<<n_pairs, 256, 0, stream>>>(static_cast<const bf16*>(x), order, weights, top, static_cast<bf16*>(sorted), width,
                                                  weight_on_input);
    const int tiles = (n_pairs + kGroupRows - 1) / kGroupRows + experts;
    MLL_REQUIRE(tiles < 65536, "moe_grouped: too many tiles of rows for one launch");
    if (gated) {
        moe_grouped_kernel<1><<<dim3((ff + 63) / 64, tiles), 256, 0, stream>>>(
            static_cast<const bf16*>(sorted), static_cast<const bf16*>(gate_up), offsets, order, weights, experts, ff, width, act, top,
            n_tokens, weight_on_input, activation);
    } else {
        moe_grouped_kernel<2><<<dim3((ff + kGroupCols - 1) / kGroupCols, tiles), 256, 0, stream>>>(
            static_cast<const bf16*>(sorted), static_cast<const bf16*>(gate_up), offsets, order, weights, experts, ff, width, act, top,
            n_tokens, weight_on_input, activation);
    }
    moe_grouped_kernel<0><<<dim3((width + kGroupCols - 1) / kGroupCols, tiles), 256, 0, stream>>>(
        static_cast<const bf16*>(act), static_cast<const bf16*>(down), offsets, order, weights, experts, width, ff, out, top, n_tokens,
        weight_on_input, activation);
    return check_launch("moe_grouped");
}

int mll_router_logits(const void* x, int dtype, const float* w, float* z, int n_tokens, int n_out, int width, hipStream_t stream) {
    MLL_REQUIRE(n_tokens >= 0 && n_out > 0 && width > 0, "router_logits: sizes must be positive");
    MLL_REQUIRE(static_cast<size_t>(width) * sizeof(float) <= 64 * 1024, "router_logits: rows wider than 16384 are not supported");
    MLL_REQUIRE(n_out <= 4 * 65535, "router_logits: too many rows of w for one launch");
    if (n_tokens == 0) return 0;
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (dtype == kF32) {
        router_logits_kernel<float><<<dim3(n_tokens, (n_out + 3) / 4), 256, lds, stream>>>(static_cast<const float*>(x), w, z, n_out, width);
    } else if (dtype == kBF16) {
        router_logits_kernel<bf16><<<dim3(n_tokens, (n_out + 3) / 4), 256, lds, stream>>>(static_cast<const bf16*>(x), w, z, n_out, width);
    } else {
        return fail("router_logits: unknown dtype");
    }
    return check_launch("router_logits");
}

}  // extern "C"
