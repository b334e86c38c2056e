// A sublayer's result that is RMS-normed itself before it joins the residual stream, and the norm that follows:
//
//   d = sum of the delta's parts, in order          (the partial sums of a product cut along its reduction)
//   v = h + mult * d * rsqrt(mean(d^2) + after_eps) * after_weight (+ extra, a further float32 row for every row of h)
//   out = v * rsqrt(mean(v^2) + eps) * weight       (weight null: no output, the sum alone)
//
// One workgroup a row; the row stays in registers between the two sums of squares. Both sums are float32 and
// added in an order that follows the width alone, so a row's bits do not depend on the step it is in.
#include "common.h"
#include "microllm_hip.h"

namespace mll {

constexpr int kAfterThreads = 256;

template <typename T, typename D, int CHUNKS>
__global__ void __launch_bounds__(kAfterThreads)
rms_norm_after_kernel(float* __restrict__ h, const D* __restrict__ delta, int n_partials, int64_t partial_stride,
                      const int32_t* __restrict__ rows, const float* __restrict__ after_weight, float after_eps, float mult,
                      const float* __restrict__ extra, const float* __restrict__ weight, float eps, T* __restrict__ out, int width, int write_h) {
    __shared__ float scratch[16];
    const int index = blockIdx.x;
    const int64_t source = rows ? rows[index] : index;
    float* h_row = h + source * width;
    const D* delta_row = delta + source * width;
    float d[CHUNKS];
    float squares = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int column = threadIdx.x + c * kAfterThreads;
        d[c] = 0.0f;
        if (column < width) {
            float sum = to_float(delta_row[column]);
            for (int part = 1; part < n_partials; ++part) sum += to_float(delta_row[part * partial_stride + column]);
            d[c] = sum;
            squares = fmaf(sum, sum, squares);
        }
    }
    const float after = mult * (1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(width) + after_eps));
    squares = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int column = threadIdx.x + c * kAfterThreads;
        if (column < width) {
            float value = h_row[column] + d[c] * after * after_weight[column];
            if (extra) value += extra[source * width + column];
            d[c] = value;
            if (write_h) h_row[column] = value;
            squares = fmaf(value, value, squares);
        }
    }
    if (weight == nullptr) return;
    const float factor = 1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(width) + eps);
    T* out_row = out + static_cast<int64_t>(index) * width;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int column = threadIdx.x + c * kAfterThreads;
        if (column < width) out_row[column] = from_float<T>(d[c] * factor * weight[column]);
    }
}

// The same for rows of float4, taken when the width is a multiple of 4 and at most 4 * CHUNKS * blockDim.x and
// every operand lies on 16 bytes: a thread keeps CHUNKS pieces of four columns. Which kernel runs follows the width
// and the operands' places alone, never the number of rows.
__device__ inline float4 after_load_four(const float* source) { return *reinterpret_cast<const float4*>(source); }
__device__ inline float4 after_load_four(const bf16* source) {
    return make_float4(to_float(source[0]), to_float(source[1]), to_float(source[2]), to_float(source[3]));
}

template <typename T, typename D, int CHUNKS>
__global__ void rms_norm_after_vec4_kernel(float* __restrict__ h, const D* __restrict__ delta, int n_partials, int64_t partial_stride,
                                           const int32_t* __restrict__ rows, const float* __restrict__ after_weight, float after_eps,
                                           float mult, const float* __restrict__ extra, const float* __restrict__ weight, float eps, T* __restrict__ out, int width,
                                           int write_h) {
    __shared__ float scratch[16];
    const int index = blockIdx.x;
    const int64_t source = rows ? rows[index] : index;
    float* h_row = h + source * width;
    const D* delta_row = delta + source * width;
    const int quads = width / 4;
    float4 d[CHUNKS], stream[CHUNKS];
    float squares = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int q = threadIdx.x + c * blockDim.x;
        d[c] = stream[c] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (q < quads) {
            stream[c] = reinterpret_cast<const float4*>(h_row)[q];
            float4 sum = after_load_four(delta_row + 4 * q);
            constexpr int kAtATime = 8;      // parts asked for at a time, then added in order
            for (int base = 1; base < n_partials; base += kAtATime) {
                float4 more[kAtATime];
#pragma unroll
                for (int j = 0; j < kAtATime; ++j)
                    if (base + j < n_partials) more[j] = after_load_four(delta_row + (base + j) * partial_stride + 4 * q);
#pragma unroll
                for (int j = 0; j < kAtATime; ++j)
                    if (base + j < n_partials) {
                        sum.x += more[j].x;
                        sum.y += more[j].y;
                        sum.z += more[j].z;
                        sum.w += more[j].w;
                    }
            }
            d[c] = sum;
            squares = fmaf(sum.x, sum.x, squares);
            squares = fmaf(sum.y, sum.y, squares);
            squares = fmaf(sum.z, sum.z, squares);
            squares = fmaf(sum.w, sum.w, squares);
        }
    }
    const float after = mult * (1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(width) + after_eps));
    squares = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int q = threadIdx.x + c * blockDim.x;
        if (q < quads) {
            const float4 w = reinterpret_cast<const float4*>(after_weight)[q];
            float4 value;
            value.x = stream[c].x + d[c].x * after * w.x;
            value.y = stream[c].y + d[c].y * after * w.y;
            value.z = stream[c].z + d[c].z * after * w.z;
            value.w = stream[c].w + d[c].w * after * w.w;
            if (extra) {
                const float4 more = reinterpret_cast<const float4*>(extra + source * width)[q];
                value.x += more.x;
                value.y += more.y;
                value.z += more.z;
                value.w += more.w;
            }
            d[c] = value;
            if (write_h) reinterpret_cast<float4*>(h_row)[q] = value;
            squares = fmaf(value.x, value.x, squares);
            squares = fmaf(value.y, value.y, squares);
            squares = fmaf(value.z, value.z, squares);
            squares = fmaf(value.w, value.w, squares);
        }
    }
    if (weight == nullptr) return;
    const float factor = 1.0f / sqrtf(block_sum(squares, scratch) / static_cast<float>(width) + eps);
    T* out_row = out + static_cast<int64_t>(index) * width;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int q = threadIdx.x + c * blockDim.x;
        if (q < quads) {
            const float4 w = reinterpret_cast<const float4*>(weight)[q];
            out_row[4 * q + 0] = from_float<T>(d[c].x * factor * w.x);
            out_row[4 * q + 1] = from_float<T>(d[c].y * factor * w.y);
            out_row[4 * q + 2] = from_float<T>(d[c].z * factor * w.z);
            out_row[4 * q + 3] = from_float<T>(d[c].w * factor * w.w);
        }
    }
}

template <typename T, typename D>
static int launch_after(float* h, const D* delta, int n_partials, int64_t partial_stride, const int32_t* rows,
                        const float* after_weight, float after_eps, float mult, const float* extra, const float* weight, float eps, T* out,
                        int n_rows, int width, int write_h, hipStream_t stream) {
#define MLL_AFTER(CHUNKS)                                                                                                \
    rms_norm_after_kernel<T, D, CHUNKS><<<n_rows, kAfterThreads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, \
                                                                              after_weight, after_eps, mult, extra, weight, eps, \
                                                                              out, width, write_h)
    const bool delta_aligned = sizeof(D) != sizeof(float) ||
                               (reinterpret_cast<uintptr_t>(delta) % 16 == 0 && (n_partials == 1 || partial_stride % 4 == 0));
    const bool aligned = width % 4 == 0 && delta_aligned && reinterpret_cast<uintptr_t>(h) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(after_weight) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(extra) % 16 == 0;
    const int quads = width / 4;
    if (aligned && quads <= 1024) {
        const int threads = quads <= 64 ? 64 : (quads + 63) / 64 * 64;
        rms_norm_after_vec4_kernel<T, D, 1><<<n_rows, threads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, after_weight,
                                                                           after_eps, mult, extra, weight, eps, out, width, write_h);
        return check_launch("rms_norm_after");
    }
    if (aligned && quads <= 4096) {
        rms_norm_after_vec4_kernel<T, D, 4><<<n_rows, 1024, 0, stream>>>(h, delta, n_partials, partial_stride, rows, after_weight,
                                                                        after_eps, mult, extra, weight, eps, out, width, write_h);
        return check_launch("rms_norm_after");
    }
    const int chunks = (width + kAfterThreads - 1) / kAfterThreads;
    if (chunks <= 1) MLL_AFTER(1);
    else if (chunks <= 2) MLL_AFTER(2);
    else if (chunks <= 4) MLL_AFTER(4);
    else if (chunks <= 8) MLL_AFTER(8);
    else if (chunks <= 16) MLL_AFTER(16);
    else if (chunks <= 32) MLL_AFTER(32);
    else return fail("rms_norm_after: rows wider than 8192 are not supported");
#undef MLL_AFTER
    return check_launch("rms_norm_after");
}

}  // namespace mll

using namespace mll;

extern "C" int mll_rms_norm_after(float* h, const void* delta, int delta_dtype, int n_partials, int64_t partial_stride,
                                  const int32_t* rows, const float* after_weight, float after_eps, float mult,
                                  const float* extra, const float* weight, float eps, void* out, int dtype, int n_rows, int width, int write_h,
                                  hipStream_t stream) {
    MLL_REQUIRE(h != nullptr && delta != nullptr && after_weight != nullptr, "rms_norm_after: a stream, a delta and its norm's weight");
    MLL_REQUIRE(n_partials >= 1, "rms_norm_after: the delta needs at least one part");
    MLL_REQUIRE(n_rows >= 0 && width > 0, "rms_norm_after: sizes must be positive");
    MLL_REQUIRE(after_eps > 0.0f && (weight == nullptr || eps > 0.0f), "rms_norm_after: eps must be positive");
    MLL_REQUIRE(!(write_h && rows), "rms_norm_after: cannot write h through a row selection");
    MLL_REQUIRE(weight == nullptr || out != nullptr, "rms_norm_after: a second norm needs an output");
    if (n_rows == 0) return 0;
    if (dtype == kF32 && delta_dtype == kF32)
        return launch_after<float, float>(h, static_cast<const float*>(delta), n_partials, partial_stride, rows, after_weight,
                                          after_eps, mult, extra, weight, eps, static_cast<float*>(out), n_rows, width, write_h, stream);
    if (dtype == kBF16 && delta_dtype == kF32)
        return launch_after<bf16, float>(h, static_cast<const float*>(delta), n_partials, partial_stride, rows, after_weight,
                                         after_eps, mult, extra, weight, eps, static_cast<bf16*>(out), n_rows, width, write_h, stream);
    if (dtype == kBF16 && delta_dtype == kBF16)
        return launch_after<bf16, bf16>(h, static_cast<const bf16*>(delta), n_partials, partial_stride, rows, after_weight,
                                        after_eps, mult, extra, weight, eps, static_cast<bf16*>(out), n_rows, width, write_h, stream);
    return fail("rms_norm_after: the delta is float32 or has the output's type");
}
