// A sublayer's result that is RMS-normed itself before it joins the residual stream, and the norm that follows:
//
//   d = sum of the delta's parts, in order          (the partial sums of a product cut along its reduction)
//   v = h + mult * d * rsqrt(mean(d^2) + after_eps) * after_weight
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
                      const float* __restrict__ weight, float eps, T* __restrict__ out, int width, int write_h) {
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
            const float value = h_row[column] + d[c] * after * after_weight[column];
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

template <typename T, typename D>
static int launch_after(float* h, const D* delta, int n_partials, int64_t partial_stride, const int32_t* rows,
                        const float* after_weight, float after_eps, float mult, const float* weight, float eps, T* out,
                        int n_rows, int width, int write_h, hipStream_t stream) {
#define MLL_AFTER(CHUNKS)                                                                                                \
    rms_norm_after_kernel<T, D, CHUNKS><<<n_rows, kAfterThreads, 0, stream>>>(h, delta, n_partials, partial_stride, rows, \
                                                                              after_weight, after_eps, mult, weight, eps, \
                                                                              out, width, write_h)
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
                                  const float* weight, float eps, void* out, int dtype, int n_rows, int width, int write_h,
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
                                          after_eps, mult, weight, eps, static_cast<float*>(out), n_rows, width, write_h, stream);
    if (dtype == kBF16 && delta_dtype == kF32)
        return launch_after<bf16, float>(h, static_cast<const float*>(delta), n_partials, partial_stride, rows, after_weight,
                                         after_eps, mult, weight, eps, static_cast<bf16*>(out), n_rows, width, write_h, stream);
    if (dtype == kBF16 && delta_dtype == kBF16)
        return launch_after<bf16, bf16>(h, static_cast<const bf16*>(delta), n_partials, partial_stride, rows, after_weight,
                                        after_eps, mult, weight, eps, static_cast<bf16*>(out), n_rows, width, write_h, stream);
    return fail("rms_norm_after: the delta is float32 or has the output's type");
}
