// Row-wise kernels of projections that carry a bias:
//
//   bias_span_norm   in place on float rows: the first `biased` columns get their bias (and, for an engine that keeps
//                    products in bfloat16, that type's rounding); then every named span of columns is divided by its
//                    root mean square over the whole span (all heads of a projection at once) and multiplied by a gain
//                    of the span's size
//   bias_glu         act(gate + b_gate) * (up + b_up) from rows [gate | up]
//   add_bias         x[r, c] += b[c] in place
//
// Sums and means are float whatever the storage type.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

// Threads a row: many for steps of few rows (a row is then a handful of trips to memory), fewer from kSpanManyRows rows
// on, so that many rows are in flight on a compute unit.
constexpr int kSpanThreadsFew = 1024;
constexpr int kSpanThreadsMany = 256;
constexpr int kSpanManyRows = 512;
constexpr int kMaxSpans = 4;

struct NormSpans {
    int offset[kMaxSpans], width[kMaxSpans], count[kMaxSpans];   // count: the elements the mean is taken over
    AnyVec gain[kMaxSpans];
};

template <int kSpanThreads>
__global__ void __launch_bounds__(kSpanThreads)
bias_span_norm_kernel(float* __restrict__ rows, long stride, AnyVec bias, int biased, int round_bf16, NormSpans spans,
                      int n_spans, float eps) {
    __shared__ float scratch[kSpanThreads / kWave];
    float* r = rows + static_cast<long>(blockIdx.x) * stride;
    if (bias.ptr || round_bf16) {
        for (int c = threadIdx.x; c < biased; c += kSpanThreads) {
            float v = r[c] + (bias.ptr ? load_any(bias, c) : 0.f);
            if (round_bf16) v = to_float(from_float<bf16_t>(v));
            r[c] = v;
        }
        __syncthreads();
    }
    for (int s = 0; s < n_spans; ++s) {
        float* at = r + spans.offset[s];
        const int width = spans.width[s];
        float ss = 0.f;
        for (int c = threadIdx.x; c < width; c += kSpanThreads) ss = fmaf(at[c], at[c], ss);
        const float inv = 1.0f / sqrtf(block_sum<kSpanThreads>(ss, scratch) / static_cast<float>(spans.count[s]) + eps);
        for (int c = threadIdx.x; c < width; c += kSpanThreads) at[c] = at[c] * inv * load_any(spans.gain[s], c);
    }
}

template <typename TIn, typename TOut>
__global__ void bias_glu_kernel(const TIn* __restrict__ in, AnyVec bias, TOut* __restrict__ out, long rows, int ffn, int act) {
    const long n = rows * ffn;
    for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
        const long r = i / ffn;
        const int c = static_cast<int>(i % ffn);
        float g = to_float(in[r * 2 * ffn + c]), u = to_float(in[r * 2 * ffn + ffn + c]);
        if (bias.ptr) {
            g += load_any(bias, c);
            u += load_any(bias, ffn + c);
        }
        out[i] = from_float<TOut>(gate_act(g, act) * u);
    }
}

__global__ void add_bias_kernel(float* __restrict__ x, AnyVec bias, long rows, int width) {
    const long n = rows * width;
    for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x)
        x[i] += load_any(bias, i % width);
}

static bool known_type(int dtype) { return dtype == kF32 || dtype == kBF16; }
static int blocks_for(long n) { return static_cast<int>((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192); }

}  // namespace leone

using namespace leone;

extern "C" int leone_bias_span_norm(float* rows_at, long stride, int rows, const void* bias, int bias_dtype, int biased,
                                    int round_bf16, const int* offsets, const int* widths, const int* counts,
                                    const void* const* gains, int gain_dtype, int n_spans, float eps, hipStream_t stream) {
    LEONE_REQUIRE(rows_at && rows > 0 && biased >= 0 && stride >= biased, "bias_span_norm: %d rows of %ld with %d biased columns",
                  rows, stride, biased);
    LEONE_REQUIRE(n_spans >= 0 && n_spans <= kMaxSpans && (n_spans == 0 || (offsets && widths && gains)),
                  "bias_span_norm: %d spans, the kernel takes up to %d", n_spans, kMaxSpans);
    LEONE_REQUIRE((!bias || known_type(bias_dtype)) && (n_spans == 0 || known_type(gain_dtype)) && eps > 0.f,
                  "bias_span_norm: unknown element type or eps");
    NormSpans spans{};
    for (int s = 0; s < n_spans; ++s) {
        LEONE_REQUIRE(gains[s] && offsets[s] >= 0 && widths[s] > 0 && offsets[s] + static_cast<long>(widths[s]) <= stride,
                      "bias_span_norm: span %d (%d + %d) does not fit rows of %ld", s, offsets[s], widths[s], stride);
        for (int t = 0; t < s; ++t)
            LEONE_REQUIRE(offsets[s] >= offsets[t] + widths[t] || offsets[t] >= offsets[s] + widths[s],
                          "bias_span_norm: spans %d and %d overlap", t, s);
        spans.offset[s] = offsets[s];
        spans.width[s] = widths[s];
        spans.count[s] = counts ? counts[s] : widths[s];
        LEONE_REQUIRE(spans.count[s] > 0 && spans.count[s] <= widths[s], "bias_span_norm: span %d of %d elements cannot count %d",
                      s, widths[s], spans.count[s]);
        spans.gain[s] = AnyVec{gains[s], gain_dtype};
    }
    if (rows >= kSpanManyRows)
        bias_span_norm_kernel<kSpanThreadsMany><<<rows, kSpanThreadsMany, 0, stream>>>(rows_at, stride, AnyVec{bias, bias_dtype}, biased,
                                                                                      round_bf16, spans, n_spans, eps);
    else
        bias_span_norm_kernel<kSpanThreadsFew><<<rows, kSpanThreadsFew, 0, stream>>>(rows_at, stride, AnyVec{bias, bias_dtype}, biased,
                                                                                    round_bf16, spans, n_spans, eps);
    LEONE_LAUNCH_CHECK("bias_span_norm");
    return 0;
}

extern "C" int leone_bias_glu(const void* gate_up, int in_dtype, const void* bias, int bias_dtype, void* out, int out_dtype,
                              int rows, int ffn, int act, hipStream_t stream) {
    LEONE_REQUIRE(gate_up && out && rows > 0 && ffn > 0, "bias_glu: needs rows [gate | up] and positive sizes");
    LEONE_REQUIRE(known_type(in_dtype) && known_type(out_dtype) && (!bias || known_type(bias_dtype)), "bias_glu: unknown element type");
    LEONE_REQUIRE(act == kGateSilu || act == kGateGeluTanh, "bias_glu: unknown activation %d", act);
    const long n = static_cast<long>(rows) * ffn;
    const AnyVec vb{bias, bias_dtype};
#define LEONE_GLU(TIN, TOUT)                                                                                             \
    bias_glu_kernel<TIN, TOUT><<<blocks_for(n), 256, 0, stream>>>(static_cast<const TIN*>(gate_up), vb, static_cast<TOUT*>(out), \
                                                                  rows, ffn, act)
    if (in_dtype == kF32 && out_dtype == kF32) LEONE_GLU(float, float);
    else if (in_dtype == kF32) LEONE_GLU(float, bf16_t);
    else if (out_dtype == kF32) LEONE_GLU(bf16_t, float);
    else LEONE_GLU(bf16_t, bf16_t);
#undef LEONE_GLU
    LEONE_LAUNCH_CHECK("bias_glu");
    return 0;
}

extern "C" int leone_add_bias(float* x, const void* bias, int bias_dtype, int rows, int width, hipStream_t stream) {
    LEONE_REQUIRE(x && bias && rows > 0 && width > 0 && known_type(bias_dtype), "add_bias: needs rows, a bias and positive sizes");
    add_bias_kernel<<<blocks_for(static_cast<long>(rows) * width), 256, 0, stream>>>(x, AnyVec{bias, bias_dtype}, rows, width);
    LEONE_LAUNCH_CHECK("add_bias");
    return 0;
}
