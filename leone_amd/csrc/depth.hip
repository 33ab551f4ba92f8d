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

// A thread holds up to kHold runs of kRun elements of its row in registers between the two passes (rows of up to
// 256 * kHold * kRun elements; longer rows read the stream a second time): every read of the first pass is asked for
// before any is used, so a row is one trip to memory.
template <typename TY, int kRun>
__global__ void __launch_bounds__(kDepthThreads)
residual_norm_kernel(float* __restrict__ x, const float* __restrict__ delta, int planes, long plane, float scale, AnyVec gain,
                     float eps, TY* __restrict__ y, const int* __restrict__ rows, int hidden) {
    constexpr int kHold = 4;
    __shared__ float scratch[kDepthThreads / kWave];
    const int out_row = blockIdx.x;
    const long in_row = rows ? rows[out_row] : out_row;
    float* xr = x + in_row * hidden;
    const float* dr = delta ? delta + in_row * hidden : nullptr;
    auto load = [](const float* p, float* to) {
        if constexpr (kRun == 4) {
            const float4 v = *reinterpret_cast<const float4*>(p);
            to[0] = v.x, to[1] = v.y, to[2] = v.z, to[3] = v.w;
        } else {
            to[0] = *p;
        }
    };
    auto sum_of = [&](int c, float* v) {           // the stream's elements from c on with the delta added
        load(xr + c, v);
        if (dr) {
            float d[kRun], part[kRun];
#pragma unroll
            for (int i = 0; i < kRun; ++i) d[i] = 0.f;
            for (int p = 0; p < planes; ++p) {
                load(dr + p * plane + c, part);
#pragma unroll
                for (int i = 0; i < kRun; ++i) d[i] += part[i];
            }
#pragma unroll
            for (int i = 0; i < kRun; ++i) v[i] = fmaf(scale, d[i], v[i]);
        }
    };
    const int step = kDepthThreads * kRun;
    float held[kHold][kRun];
    float ss = 0.f;
#pragma unroll
    for (int h = 0; h < kHold; ++h) {
        const int c = threadIdx.x * kRun + h * step;
        if (c < hidden) sum_of(c, held[h]);
    }
#pragma unroll
    for (int h = 0; h < kHold; ++h) {
        const int c = threadIdx.x * kRun + h * step;
        if (c < hidden) {
#pragma unroll
            for (int i = 0; i < kRun; ++i) {
                ss = fmaf(held[h][i], held[h][i], ss);
                if (dr && !rows) xr[c + i] = held[h][i];
            }
        }
    }
    for (int c = threadIdx.x * kRun + kHold * step; c < hidden; c += step) {
        float v[kRun];
        sum_of(c, v);
#pragma unroll
        for (int i = 0; i < kRun; ++i) {
            ss = fmaf(v[i], v[i], ss);
            if (dr && !rows) xr[c + i] = v[i];
        }
    }
    if (!y) return;
    const float inv = 1.0f / sqrtf(block_sum<kDepthThreads>(ss, scratch) / static_cast<float>(hidden) + eps);
    TY* yr = y + static_cast<long>(out_row) * hidden;
#pragma unroll
    for (int h = 0; h < kHold; ++h) {
        const int c = threadIdx.x * kRun + h * step;
        if (c < hidden) {
#pragma unroll
            for (int i = 0; i < kRun; ++i) yr[c + i] = from_float<TY>(held[h][i] * inv * load_any(gain, c + i));
        }
    }
    for (int c = threadIdx.x * kRun + kHold * step; c < hidden; c += step) {
        float v[kRun];
        if (dr && rows) {
            sum_of(c, v);
        } else {
#pragma unroll
            for (int i = 0; i < kRun; ++i) v[i] = xr[c + i];
        }
#pragma unroll
        for (int i = 0; i < kRun; ++i) yr[c + i] = from_float<TY>(v[i] * inv * load_any(gain, c + i));
    }
}

// kRun elements a thread (4 where the sizes allow 16-byte accesses, else 1).
template <int kRun>
__global__ void __launch_bounds__(kDepthThreads)
depth_mix_kernel(float* __restrict__ x, const float* __restrict__ delta, int planes, long plane, float scale,
                 float* __restrict__ history, long slot_stride, int count, AnyVec weight, long total) {
    const long at = (static_cast<long>(blockIdx.x) * kDepthThreads + threadIdx.x) * kRun;
    if (at >= total) return;
    float own[kRun], sum[kRun];
    auto load = [](const float* p, float* to) {
        if constexpr (kRun == 4) {
            const float4 v = *reinterpret_cast<const float4*>(p);
            to[0] = v.x, to[1] = v.y, to[2] = v.z, to[3] = v.w;
        } else {
            to[0] = *p;
        }
    };
    auto store = [](float* p, const float* from) {
        if constexpr (kRun == 4) *reinterpret_cast<float4*>(p) = float4{from[0], from[1], from[2], from[3]};
        else *p = from[0];
    };
    load(x + at, own);
    if (delta) {
        float d[kRun], part[kRun];
#pragma unroll
        for (int i = 0; i < kRun; ++i) d[i] = 0.f;
        for (int p = 0; p < planes; ++p) {
            load(delta + p * plane + at, part);
#pragma unroll
            for (int i = 0; i < kRun; ++i) d[i] += part[i];
        }
#pragma unroll
        for (int i = 0; i < kRun; ++i) own[i] = fmaf(scale, d[i], own[i]);
    }
    store(history + static_cast<long>(count - 1) * slot_stride + at, own);
#pragma unroll
    for (int i = 0; i < kRun; ++i) sum[i] = 0.f;
    for (int j = 0; j + 1 < count; ++j) {
        float kept[kRun];
        load(history + j * slot_stride + at, kept);
        const float w = load_any(weight, j);
#pragma unroll
        for (int i = 0; i < kRun; ++i) sum[i] = fmaf(w, kept[i], sum[i]);
    }
    const float last = load_any(weight, count - 1);
#pragma unroll
    for (int i = 0; i < kRun; ++i) sum[i] = fmaf(last, own[i], sum[i]);
    store(x + at, sum);
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
    const bool runs = hidden % 4 == 0 && plane % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(delta) % 16 == 0;
#define LEONE_RESIDUAL_NORM(TY, R)                                                                                      \
    residual_norm_kernel<TY, R><<<n_rows, kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, AnyVec{gain, gain_dtype}, \
                                                                    eps, static_cast<TY*>(y), rows, hidden)
    if (y_dtype == kBF16 && y) {
        if (runs) LEONE_RESIDUAL_NORM(bf16_t, 4);
        else LEONE_RESIDUAL_NORM(bf16_t, 1);
    } else {
        if (runs) LEONE_RESIDUAL_NORM(float, 4);
        else LEONE_RESIDUAL_NORM(float, 1);
    }
#undef LEONE_RESIDUAL_NORM
    LEONE_LAUNCH_CHECK("residual_norm");
    return 0;
}

extern "C" int leone_depth_mix(float* x, const float* delta, int planes, long plane, float scale, float* history,
                               long slot_stride, int count, const void* weight, int weight_dtype, long total,
                               hipStream_t stream) {
    LEONE_REQUIRE(x && history && weight && total > 0 && count >= 1 && slot_stride >= total, "depth_mix: null pointer or empty sizes");
    LEONE_REQUIRE(weight_dtype == kF32 || weight_dtype == kBF16, "depth_mix: unknown type of the weights");
    LEONE_REQUIRE(!delta || (planes >= 1 && planes <= 16), "depth_mix: %d planes of what is to be added", planes);
    const bool runs = total % 4 == 0 && slot_stride % 4 == 0 && plane % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(history) % 16 == 0 && reinterpret_cast<uintptr_t>(delta) % 16 == 0;
    const long threads = runs ? total / 4 : total;
    const long blocks = (threads + kDepthThreads - 1) / kDepthThreads;
    LEONE_REQUIRE(blocks <= 0x7fffffffL, "depth_mix: %ld elements are too many", total);
    if (runs)
        depth_mix_kernel<4><<<static_cast<unsigned>(blocks), kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, history,
                                                                                        slot_stride, count, AnyVec{weight, weight_dtype}, total);
    else
        depth_mix_kernel<1><<<static_cast<unsigned>(blocks), kDepthThreads, 0, stream>>>(x, delta, planes, plane, scale, history,
                                                                                        slot_stride, count, AnyVec{weight, weight_dtype}, total);
    LEONE_LAUNCH_CHECK("depth_mix");
    return 0;
}
