// Residual sums with a factor, and a stream that is a weighted sum of every earlier layer's result.
//
//   residual_norm  x += scale * delta (delta float [n, hidden] or planes [p, n, hidden] whose sum, in order, is meant),
//                  then y = x / sqrt(mean(x^2) + eps) * gain in y's type.  With `rows` only those rows come out and x
//                  is left as it was.  Either half may be absent (no delta: only the norm; no gain: only the sum).
//   depth_mix      X = x + scale * delta is a layer's own result: it is kept as history[count - 1], and the stream that
//                  goes on is x <- sum_{j < count} weight[j] * history[j] (history[0] the embedding's output, history[j]
//                  the result of layer j - 1), summed in the order of j.
//
// One workgroup a row; sums of squares and all sums are float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kDepthThreads = 256;

template <typename TY>
__global__ void __launch_bounds__(kDepthThreads)
residual_norm_kernel(float* __restrict__ x, const float* __restrict__ delta, int planes, long plane, float scale, AnyVec gain,
                     float eps, TY* __restrict__ y, const int* __restrict__ rows, int hidden) {
    __shared__ float scratch[kDepthThreads / kWave];
    const int out_row = blockIdx.x;
    const long in_row = rows ? rows[out_row] : out_row;
    float* xr = x + in_row * hidden;
    const float* dr = delta ? delta + in_row * hidden : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < hidden; c += kDepthThreads) {
        float v = xr[c];
        if (dr) {
            float d = 0.f;
            for (int p = 0; p < planes; ++p) d += dr[p * plane + c];
            v = fmaf(scale, d, v);
            if (!rows) xr[c] = v;
        }
        ss = fmaf(v, v, ss);
    }
    if (!y) return;
    const float inv = 1.0f / sqrtf(block_sum<kDepthThreads>(ss, scratch) / static_cast<float>(hidden) + eps);
    TY* yr = y + static_cast<long>(out_row) * hidden;
    for (int c = threadIdx.x; c < hidden; c += kDepthThreads) {
        float v = xr[c];
        if (dr && rows) {
            float d = 0.f;
            for (int p = 0; p < planes; ++p) d += dr[p * plane + c];
            v = fmaf(scale, d, v);
        }
        yr[c] = from_float<TY>(v * inv * load_any(gain, c));
    }
}

__global__ void __launch_bounds__(kDepthThreads)
depth_mix_kernel(float* __restrict__ x, const float* __restrict__ delta, int planes, long plane, float scale,
                 float* __restrict__ history, long slot_stride, int count, AnyVec weight, long total) {
    const long at = static_cast<long>(blockIdx.x) * kDepthThreads + threadIdx.x;
    if (at >= total) return;
    float own = x[at];
    if (delta) {
        float d = 0.f;
        for (int p = 0; p < planes; ++p) d += delta[p * plane + at];
        own = fmaf(scale, d, own);
    }
    history[static_cast<long>(count - 1) * slot_stride + at] = own;
    float sum = 0.f;
    for (int j = 0; j + 1 < count; ++j) sum = fmaf(load_any(weight, j), history[j * slot_stride + at], sum);
    x[at] = fmaf(load_any(weight, count - 1), own, sum);
}

}  // namespace leone

using namespace leone;

extern "C" int leone_residual_norm(float* x, const float* delta, int planes, long plane, float scale, const void* gain,
                                   int gain_dtype, float eps, void* y, int y_dtype, const int* rows, int n_rows, int hidden,
                                   hipStream_t stream) {
    LEONE_REQUIRE(x && n_rows > 0 && hidden > 0 && (delta || y), "residual_norm: null pointer or nothing to do");
    LEONE_REQUIRE(!delta || (planes >= 1 && planes <= 16), "residual_norm: %d planes of what is to be added", planes);
    LEONE_REQUIRE(!y || (gain && eps > 0.f && (gain_dtype == kF32 || gain_dtype == kBF16) && (y_dtype == kF32 || y_dtype == kBF16)),
                  "residual_norm: a norm needs a gain, eps and known types");
    LEONE_REQUIRE(!rows || y, "residual_norm: picked rows come with a norm");
    if (y_dtype == kBF16 && y)
        residual_norm_kernel<bf16_t><<<n_rows, kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, AnyVec{gain, gain_dtype},
                                                                         eps, static_cast<bf16_t*>(y), rows, hidden);
    else
        residual_norm_kernel<float><<<n_rows, kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, AnyVec{gain, gain_dtype},
                                                                        eps, static_cast<float*>(y), rows, hidden);
    LEONE_LAUNCH_CHECK("residual_norm");
    return 0;
}

extern "C" int leone_depth_mix(float* x, const float* delta, int planes, long plane, float scale, float* history,
                               long slot_stride, int count, const void* weight, int weight_dtype, long total,
                               hipStream_t stream) {
    LEONE_REQUIRE(x && history && weight && total > 0 && count >= 1 && slot_stride >= total, "depth_mix: null pointer or empty sizes");
    LEONE_REQUIRE(weight_dtype == kF32 || weight_dtype == kBF16, "depth_mix: unknown type of the weights");
    LEONE_REQUIRE(!delta || (planes >= 1 && planes <= 16), "depth_mix: %d planes of what is to be added", planes);
    const long blocks = (total + kDepthThreads - 1) / kDepthThreads;
    LEONE_REQUIRE(blocks <= 0x7fffffffL, "depth_mix: %ld elements are too many", total);
    depth_mix_kernel<<<static_cast<unsigned>(blocks), kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, history,
                                                                                 slot_stride, count, AnyVec{weight, weight_dtype}, total);
    LEONE_LAUNCH_CHECK("depth_mix");
    return 0;
}
