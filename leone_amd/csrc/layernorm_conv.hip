// Row-wise kernels of layers that keep a short history of their own inputs:
//
//   add_layernorm     x += LayerNorm_a(delta) (if a delta comes), y = LayerNorm_b(x): the norm after one
//                     sublayer, the residual sum and the norm before the next in one pass over the row
//   entry_spans       first row and end of every entry of a step, and its state slot, from the row -> entry map
//   causal_conv       out[t] = (in[t] if asked) + sum_j w[c, j] * in[t - (taps - 1) + j], per channel, the
//                     rows before a portion taken from the request's state (its last taps - 1 inputs)
//   causal_conv_state leaves the last taps - 1 inputs of every entry behind as the new state
//   head_norm_gate    per head: (read-out / denominator) / rms * gain * act(gate)
//   rms_mix           scale * sum_b rms(branch_b) * gain_b over the model width
//   relu_squared      max(x, 0)^2
//
// Sums, means and variances are float whatever the storage type.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

// Threads a row.  Few rows (decode steps): 1,024, so that a thread has few elements and a row is a handful of trips to
// memory, not one per element.  Many rows (prompt portions): 256, so that many rows are in flight on a compute unit.
constexpr int kNormThreadsFew = 1024;
constexpr int kNormThreadsMany = 256;
constexpr int kNormManyRows = 512;
constexpr int kMaxTaps = 16;

// Mean and inverse deviation of n values read through f(i); every thread gets both.
template <int kNormThreads, typename F>
__device__ inline void mean_rstd(F value, int n, float eps, float* scratch, float& mean, float& rstd) {
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) s += value(i);
    mean = block_sum<kNormThreads>(s, scratch) / static_cast<float>(n);
    float q = 0.f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) {
        const float d = value(i) - mean;
        q = fmaf(d, d, q);
    }
    const float var = block_sum<kNormThreads>(q, scratch) / static_cast<float>(n);
    rstd = 1.0f / sqrtf(var + eps);
}

// One workgroup a row; the row lies in shared memory between the passes.
template <typename TOut, int kNormThreads>
__global__ void __launch_bounds__(kNormThreads)
add_layernorm_kernel(float* __restrict__ x, const float* __restrict__ delta, AnyVec dw, AnyVec db, float deps,
                     AnyVec w, AnyVec b, float eps, TOut* __restrict__ y, const int* __restrict__ rows, int hidden,
                     AnyVec conv, int taps, float* __restrict__ conv_state, int write_state,
                     const int* __restrict__ positions, const int* __restrict__ row_entry, const int* __restrict__ entry_slots,
                     int stage_delta) {
    extern __shared__ float row_buf[];          // the row; behind it, if there is room, the delta's row
    __shared__ float scratch[kNormThreads / kWave];
    const long src = rows ? rows[blockIdx.x] : blockIdx.x;
    float* xr = x + src * hidden;
    if (delta) {
        const float* dr = delta + src * hidden;
        // both rows are fetched once, side by side; the passes after that read shared memory
        float* staged = stage_delta ? row_buf + hidden : nullptr;
        for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
            row_buf[i] = xr[i];
            if (staged) staged[i] = dr[i];
        }
        __syncthreads();
        float mean = 0.f, rstd = 1.f;
        if (dw.ptr) {
            if (staged) mean_rstd<kNormThreads>([&](int i) { return staged[i]; }, hidden, deps, scratch, mean, rstd);
            else mean_rstd<kNormThreads>([&](int i) { return dr[i]; }, hidden, deps, scratch, mean, rstd);
        }
        for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
            float d = staged ? staged[i] : dr[i];
            if (dw.ptr) d = (d - mean) * rstd * load_any(dw, i) + load_any(db, i);
            const float t = row_buf[i] + d;
            row_buf[i] = t;
            if (!rows) xr[i] = t;
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += kNormThreads) row_buf[i] = xr[i];
    }
    if (!y) return;
    __syncthreads();
    float mean, rstd;
    mean_rstd<kNormThreads>([&](int i) { return row_buf[i]; }, hidden, eps, scratch, mean, rstd);
    TOut* yr = y + static_cast<long>(blockIdx.x) * hidden;
    if (!conv.ptr) {
        for (int i = threadIdx.x; i < hidden; i += kNormThreads)
            yr[i] = from_float<TOut>((row_buf[i] - mean) * rstd * load_any(w, i) + load_any(b, i));
        return;
    }
    // A step of single rows, every row another request: the input convolution of the sublayer that reads this
    // norm is done here, h + conv(h) over the request's last inputs, and its state moved on by this row.
    const int pos = positions[blockIdx.x];
    float* keep = conv_state + static_cast<long>(entry_slots[row_entry[blockIdx.x]]) * (taps - 1) * hidden;
    for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
        const float h = (row_buf[i] - mean) * rstd * load_any(w, i) + load_any(b, i);
        float acc = 0.f;
        for (int j = 0; j + 1 < taps; ++j) {                 // oldest input first
            const float old = pos - (taps - 1 - j) < 0 ? 0.f : keep[static_cast<long>(j) * hidden + i];
            acc = fmaf(load_any(conv, static_cast<long>(i) * taps + j), old, acc);
            if (write_state && j > 0) keep[static_cast<long>(j - 1) * hidden + i] = old;
        }
        acc = fmaf(load_any(conv, static_cast<long>(i) * taps + taps - 1), h, acc);
        if (write_state) keep[static_cast<long>(taps - 2) * hidden + i] = h;
        yr[i] = from_float<TOut>(h + acc);
    }
}

__global__ void entry_spans_kernel(const int* __restrict__ row_entry, const int* __restrict__ positions,
                                   const int* __restrict__ entry_slots, int rows, int* __restrict__ spans) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const int e = row_entry[r];
    if (r == 0 || row_entry[r - 1] != e) {
        spans[4 * e] = r;
        spans[4 * e + 2] = positions[r] == 0 ? -1 : entry_slots[e];     // a sequence's start: from zeros
        spans[4 * e + 3] = entry_slots[e];
    }
    if (r == rows - 1 || row_entry[r + 1] != e) spans[4 * e + 1] = r + 1;
}

enum Activation : int { kActNone = 0, kActSigmoid = 1, kActSilu = 2 };

__device__ inline float activate(float v, int act) {
    if (act == kActNone) return v;
    const float s = 1.0f / (1.0f + expf(-v));
    return act == kActSigmoid ? s : v * s;
}

constexpr int kConvRows = 8;     // consecutive rows a workgroup takes in a step of many rows: what it must know of a row is
                                 // fetched once for all of them; a step of few rows has a workgroup a row

template <typename TIn, typename TOut>
__global__ void causal_conv_kernel(const TIn* __restrict__ in, long in_stride, TOut* __restrict__ out, long out_stride,
                                   AnyVec w, AnyVec bias, const float* __restrict__ state, const int* __restrict__ positions,
                                   const int* __restrict__ row_entry, const int* __restrict__ entry_slots, int rows,
                                   int channels, int taps, int add_input, int act, float* __restrict__ own_state, int per_block) {
    __shared__ int s_inside[kConvRows], s_pos[kConvRows], s_slot[kConvRows];
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int r0 = blockIdx.x * per_block;
    if (threadIdx.x < per_block && r0 + threadIdx.x < rows) {
        const int r = r0 + threadIdx.x;
        const int e = row_entry[r];
        int inside = 0;      // rows of this request that stand before row r in this step, as far as the taps reach
        while (inside < taps - 1 && r - inside - 1 >= 0 && row_entry[r - inside - 1] == e) ++inside;
        s_inside[threadIdx.x] = inside;
        s_pos[threadIdx.x] = positions[r];
        s_slot[threadIdx.x] = entry_slots[e];
    }
    __syncthreads();
    if (c >= channels) return;
    for (int k = 0; k < per_block && r0 + k < rows; ++k) {
        const int r = r0 + k;
        const int pos = s_pos[k], inside = s_inside[k];
        const float* mine = state + (static_cast<long>(s_slot[k]) * (taps - 1)) * channels + c;
        float acc = 0.f;
        for (int back = taps - 1; back >= 0; --back) {          // oldest input first
            float h;
            if (pos - back < 0) h = 0.f;                          // before the sequence's start
            else if (back <= inside) h = to_float(in[static_cast<long>(r - back) * in_stride + c]);
            else h = mine[static_cast<long>(taps - 1 - (back - inside)) * channels];
            acc = fmaf(load_any(w, static_cast<long>(c) * taps + (taps - 1 - back)), h, acc);
        }
        const float now = to_float(in[static_cast<long>(r) * in_stride + c]);
        if (add_input) acc += now;
        if (bias.ptr) acc += load_any(bias, c);
        out[static_cast<long>(r) * out_stride + c] = from_float<TOut>(activate(acc, act));
        if (own_state) {      // a step of single rows, every row another request: this thread alone touches (slot, channel)
            float* keep = own_state + (static_cast<long>(s_slot[k]) * (taps - 1)) * channels + c;
            for (int j = 0; j + 2 < taps; ++j)
                keep[static_cast<long>(j) * channels] = pos - (taps - 2 - j) < 0 ? 0.f : keep[static_cast<long>(j + 1) * channels];
            keep[static_cast<long>(taps - 2) * channels] = now;
        }
    }
}

template <typename TIn>
__global__ void causal_conv_state_kernel(const TIn* __restrict__ in, long in_stride, float* __restrict__ state,
                                         const int* __restrict__ spans, const int* __restrict__ entry_slots,
                                         const int* __restrict__ positions, int channels, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int e = blockIdx.y;
    if (c >= channels) return;
    const int first = spans[4 * e], n = spans[4 * e + 1] - first;
    const int start = positions[first];
    float* mine = state + (static_cast<long>(entry_slots[e]) * (taps - 1)) * channels + c;
    float keep[kMaxTaps - 1];
    for (int j = 0; j < taps - 1; ++j) {
        const int back = taps - 1 - j;                        // how far before the end of the portion
        if (back <= n) keep[j] = to_float(in[static_cast<long>(first + n - back) * in_stride + c]);
        else if (start + n - back < 0) keep[j] = 0.f;
        else keep[j] = mine[static_cast<long>(taps - 1 - (back - n)) * channels];
    }
    for (int j = 0; j < taps - 1; ++j) mine[static_cast<long>(j) * channels] = keep[j];
}

// One wave per (row, head).
template <typename TOut>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ dot, const float* __restrict__ top,
                                      AnyVec gain, int gain_per_head, const float* __restrict__ gate, long gate_stride,
                                      int act, float eps, TOut* __restrict__ out, int heads, int vdim, int gate_first) {
    const int row = blockIdx.x;
    const int head = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    if (head >= heads) return;
    const long at = static_cast<long>(row) * heads + head;
    const float* src = o + at * vdim;
    float under = 1.f;
    if (dot) under = fmaxf(fabsf(dot[at]), expf(-top[at])) + 1e-6f;
    const float* gate_row = gate ? gate + static_cast<long>(row) * gate_stride + static_cast<long>(head) * vdim : nullptr;
    // with gate_first the gate multiplies ahead of the norm, and the root mean square is that of the gated values
    auto fetch = [&](int j) {
        const float v = src[j] / under;
        return (gate_first && gate_row) ? v * activate(gate_row[j], act) : v;
    };
    constexpr int kKept = 8;                                   // values a lane keeps between the two passes
    float kept[kKept];
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < kKept; ++n) {
        const int j = lane + n * kWave;
        kept[n] = j < vdim ? fetch(j) : 0.f;
        ss = fmaf(kept[n], kept[n], ss);
    }
    for (int j = lane + kKept * kWave; j < vdim; j += kWave) {
        const float v = fetch(j);
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
    TOut* dst = out + at * vdim;
    auto finish = [&](int j, float v) {
        v *= inv;
        if (gain.ptr) v *= load_any(gain, gain_per_head ? static_cast<long>(head) * vdim + j : j);
        if (gate_row && !gate_first) v *= activate(gate_row[j], act);
        dst[j] = from_float<TOut>(v);
    };
#pragma unroll
    for (int n = 0; n < kKept; ++n)
        if (lane + n * kWave < vdim) finish(lane + n * kWave, kept[n]);
    for (int j = lane + kKept * kWave; j < vdim; j += kWave) finish(j, fetch(j));
}

constexpr int kMaxBranches = 4;
struct Branches {
    const float* rows[kMaxBranches];
    AnyVec gain[kMaxBranches];
};

template <int kNormThreads>
__global__ void __launch_bounds__(kNormThreads)
rms_mix_kernel(Branches in, int branches, float eps, float scale, float* __restrict__ out, int hidden) {
    __shared__ float scratch[kNormThreads / kWave];
    const long row = blockIdx.x;
    float inv[kMaxBranches];
    for (int b = 0; b < branches; ++b) {
        const float* src = in.rows[b] + row * hidden;
        float ss = 0.f;
        for (int i = threadIdx.x; i < hidden; i += kNormThreads) ss = fmaf(src[i], src[i], ss);
        inv[b] = 1.0f / sqrtf(block_sum<kNormThreads>(ss, scratch) / static_cast<float>(hidden) + eps);
    }
    for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
        float total = 0.f;
        for (int b = 0; b < branches; ++b) total += in.rows[b][row * hidden + i] * inv[b] * load_any(in.gain[b], i);
        out[row * hidden + i] = total * scale;
    }
}

// out = sum_b weight_b * branch_b, nothing normed.
__global__ void weighted_mix_kernel(Branches in, int branches, float w0, float w1, float w2, float w3, float* __restrict__ out, long n) {
    const float weight[kMaxBranches] = {w0, w1, w2, w3};
    for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
        float total = 0.f;
        for (int b = 0; b < branches; ++b) total = fmaf(weight[b], in.rows[b][i], total);
        out[i] = total;
    }
}

template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ in, T* __restrict__ out, long n) {
    for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
        const float v = fmaxf(to_float(in[i]), 0.f);
        out[i] = from_float<T>(v * v);
    }
}

// Per-head sigmoid gates on attention's output: out[r, h, :] *= sigmoid(gate[r * stride + h]).
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ out, const float* __restrict__ gate, long gate_stride, int heads, int vdim, long n) {
    const long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
    if (i >= n) return;
    const long row = i / (static_cast<long>(heads) * vdim);
    const int head = static_cast<int>((i / vdim) % heads);
    out[i] = from_float<T>(to_float(out[i]) * activate(gate[row * gate_stride + head], kActSigmoid));
}

static bool known(int dtype) { return dtype == kF32 || dtype == kBF16; }

}  // namespace leone

using namespace leone;

extern "C" int leone_add_layernorm(float* x, const float* delta, const void* dw, const void* db, float deps,
                                   const void* w, const void* b, int w_dtype, float eps, void* y, int y_dtype,
                                   const int* rows, int n_out, int hidden, const void* conv, int conv_dtype, int taps,
                                   float* conv_state, int write_state, const int* positions, const int* row_entry,
                                   const int* entry_slots, hipStream_t stream) {
    LEONE_REQUIRE(!conv || (y && !rows && conv_state && positions && row_entry && entry_slots && taps >= 2 && taps <= kMaxTaps &&
                            known(conv_dtype)), "add_layernorm: a folded convolution needs its state, the rows' places and 2..%d taps", kMaxTaps);
    const AnyVec vconv{conv, conv_dtype};
    LEONE_REQUIRE(x && n_out > 0 && hidden > 0, "add_layernorm: needs a stream and positive sizes");
    LEONE_REQUIRE(known(w_dtype) && known(y_dtype), "add_layernorm: unknown element type");
    LEONE_REQUIRE((dw == nullptr) == (db == nullptr), "add_layernorm: the delta's gain and bias come together");
    LEONE_REQUIRE(!dw || (delta && deps > 0.f), "add_layernorm: a norm of the delta needs a delta and an eps");
    LEONE_REQUIRE(!y || (w && b && eps > 0.f), "add_layernorm: the output norm needs gain, bias and eps");
    LEONE_REQUIRE(y || (delta && !rows), "add_layernorm: nothing to do");
    LEONE_REQUIRE(static_cast<size_t>(hidden) * sizeof(float) <= 64 * 1024, "add_layernorm: rows of %d elements are too long", hidden);
    const AnyVec vdw{dw, w_dtype}, vdb{db, w_dtype}, vw{w, w_dtype}, vb{b, w_dtype};
    const int stage_delta = (delta && static_cast<size_t>(hidden) * 2 * sizeof(float) <= 64 * 1024) ? 1 : 0;
    const size_t shared = static_cast<size_t>(hidden) * sizeof(float) * (stage_delta ? 2 : 1);
#define LEONE_LAYERNORM(T, THREADS)                                                                                        \
    add_layernorm_kernel<T, THREADS><<<n_out, THREADS, shared, stream>>>(x, delta, vdw, vdb, deps, vw, vb, eps, static_cast<T*>(y), \
                                                                         rows, hidden, vconv, taps, conv_state, write_state,   \
                                                                         positions, row_entry, entry_slots, stage_delta)
    const bool many = n_out >= kNormManyRows;
    if (y_dtype == kF32) {
        if (many) LEONE_LAYERNORM(float, kNormThreadsMany);
        else LEONE_LAYERNORM(float, kNormThreadsFew);
    } else {
        if (many) LEONE_LAYERNORM(bf16_t, kNormThreadsMany);
        else LEONE_LAYERNORM(bf16_t, kNormThreadsFew);
    }
#undef LEONE_LAYERNORM
    LEONE_LAUNCH_CHECK("add_layernorm");
    return 0;
}

extern "C" int leone_entry_spans(const int* row_entry, const int* positions, const int* entry_slots, int rows, int* spans,
                                 hipStream_t stream) {
    LEONE_REQUIRE(row_entry && positions && entry_slots && spans && rows > 0, "entry_spans: needs a row map");
    entry_spans_kernel<<<ceil_div(rows, 256), 256, 0, stream>>>(row_entry, positions, entry_slots, rows, spans);
    LEONE_LAUNCH_CHECK("entry_spans");
    return 0;
}

extern "C" int leone_causal_conv(const void* in, int in_dtype, long in_stride, void* out, int out_dtype, long out_stride,
                                 const void* w, int w_dtype, float* state, int write_state, const int* spans, int entries,
                                 const int* positions, const int* row_entry, const int* entry_slots, int rows,
                                 int channels, int taps, int add_input, int act, int single_rows, hipStream_t stream) {
    return leone_causal_conv_biased(in, in_dtype, in_stride, out, out_dtype, out_stride, w, nullptr, w_dtype, state, write_state,
                                    spans, entries, positions, row_entry, entry_slots, rows, channels, taps, add_input, act,
                                    single_rows, stream);
}

// bias: one value a channel ([channels], of the filters' type) added to the filter's sum ahead of the activation; may be null.
extern "C" int leone_causal_conv_biased(const void* in, int in_dtype, long in_stride, void* out, int out_dtype, long out_stride,
                                        const void* w, const void* bias, int w_dtype, float* state, int write_state,
                                        const int* spans, int entries, const int* positions, const int* row_entry,
                                        const int* entry_slots, int rows, int channels, int taps, int add_input, int act,
                                        int single_rows, hipStream_t stream) {
    LEONE_REQUIRE(in && out && w && state && positions && row_entry && entry_slots, "causal_conv: null pointer");
    LEONE_REQUIRE(known(in_dtype) && known(out_dtype) && known(w_dtype), "causal_conv: unknown element type");
    LEONE_REQUIRE(rows > 0 && channels > 0 && ceil_div(channels, 256) <= 65535 && in_stride >= channels && out_stride >= channels,
                  "causal_conv: %d rows of %d channels", rows, channels);
    LEONE_REQUIRE(taps >= 2 && taps <= kMaxTaps, "causal_conv: %d taps, the kernel takes 2..%d", taps, kMaxTaps);
    LEONE_REQUIRE(act >= kActNone && act <= kActSilu, "causal_conv: unknown activation %d", act);
    LEONE_REQUIRE(!write_state || single_rows || (spans && entries > 0 && entries <= 65535),
                  "causal_conv: the state's update needs the entries' spans");
    const AnyVec vw{w, w_dtype};
    const AnyVec vbias{bias, w_dtype};
    const int per_block = rows >= kNormManyRows ? kConvRows : 1;
    const dim3 grid(ceil_div(rows, per_block), ceil_div(channels, 256));
#define LEONE_CONV(TIN, TOUT)                                                                                         \
    causal_conv_kernel<TIN, TOUT><<<grid, 256, 0, stream>>>(static_cast<const TIN*>(in), in_stride, static_cast<TOUT*>(out), \
                                                            out_stride, vw, vbias, state, positions, row_entry, entry_slots, \
                                                            rows, channels, taps, add_input, act,                    \
                                                            (write_state && single_rows) ? state : nullptr, per_block)
    if (in_dtype == kF32 && out_dtype == kF32) LEONE_CONV(float, float);
    else if (in_dtype == kF32) LEONE_CONV(float, bf16_t);
    else if (out_dtype == kF32) LEONE_CONV(bf16_t, float);
    else LEONE_CONV(bf16_t, bf16_t);
#undef LEONE_CONV
    LEONE_LAUNCH_CHECK("causal_conv");
    if (write_state && !single_rows) {
        const dim3 sgrid(ceil_div(channels, 256), entries);
        if (in_dtype == kF32)
            causal_conv_state_kernel<float><<<sgrid, 256, 0, stream>>>(static_cast<const float*>(in), in_stride, state, spans,
                                                                       entry_slots, positions, channels, taps);
        else
            causal_conv_state_kernel<bf16_t><<<sgrid, 256, 0, stream>>>(static_cast<const bf16_t*>(in), in_stride, state, spans,
                                                                        entry_slots, positions, channels, taps);
        LEONE_LAUNCH_CHECK("causal_conv_state");
    }
    return 0;
}

extern "C" int leone_head_norm_gate(const float* o, const float* dot, const float* top, const void* gain, int gain_dtype,
                                    int gain_per_head, const float* gate, long gate_stride, int act, float eps, void* out,
                                    int out_dtype, int rows, int heads, int vdim, hipStream_t stream) {
    return leone_head_norm_gate_ordered(o, dot, top, gain, gain_dtype, gain_per_head, gate, gate_stride, act, 0, eps, out,
                                        out_dtype, rows, heads, vdim, stream);
}

// gate_first: the gate multiplies ahead of the norm (the root mean square is taken of the gated values) instead of behind it.
extern "C" int leone_head_norm_gate_ordered(const float* o, const float* dot, const float* top, const void* gain, int gain_dtype,
                                            int gain_per_head, const float* gate, long gate_stride, int act, int gate_first,
                                            float eps, void* out, int out_dtype, int rows, int heads, int vdim,
                                            hipStream_t stream) {
    LEONE_REQUIRE(o && out && rows > 0 && heads > 0 && vdim > 0, "head_norm_gate: needs read-outs and positive sizes");
    LEONE_REQUIRE(known(out_dtype) && (!gain || known(gain_dtype)), "head_norm_gate: unknown element type");
    LEONE_REQUIRE((dot == nullptr) == (top == nullptr), "head_norm_gate: the denominator's two parts come together");
    LEONE_REQUIRE(act >= kActNone && act <= kActSilu && eps > 0.f, "head_norm_gate: activation %d, eps %g", act, eps);
    LEONE_REQUIRE(rows <= 0x7fffffff && ceil_div(heads, 4) <= 65535, "head_norm_gate: too many heads");
    const AnyVec vg{gain, gain_dtype};
    const dim3 grid(rows, ceil_div(heads, 4));
    if (out_dtype == kF32)
        head_norm_gate_kernel<float><<<grid, 4 * kWave, 0, stream>>>(o, dot, top, vg, gain_per_head, gate, gate_stride, act, eps,
                                                                     static_cast<float*>(out), heads, vdim, gate_first);
    else
        head_norm_gate_kernel<bf16_t><<<grid, 4 * kWave, 0, stream>>>(o, dot, top, vg, gain_per_head, gate, gate_stride, act, eps,
                                                                      static_cast<bf16_t*>(out), heads, vdim, gate_first);
    LEONE_LAUNCH_CHECK("head_norm_gate");
    return 0;
}

extern "C" int leone_rms_mix(const float* const* branch_rows, const void* const* gains, int gain_dtype, int branches,
                             float eps, float scale, float* out, int rows, int hidden, hipStream_t stream) {
    LEONE_REQUIRE(branch_rows && gains && out && rows > 0 && hidden > 0, "rms_mix: needs branches and positive sizes");
    LEONE_REQUIRE(branches >= 1 && branches <= kMaxBranches, "rms_mix: %d branches, the kernel takes 1..%d", branches, kMaxBranches);
    LEONE_REQUIRE(known(gain_dtype) && eps > 0.f, "rms_mix: unknown gain type or eps");
    Branches in{};
    for (int b = 0; b < branches; ++b) {
        LEONE_REQUIRE(branch_rows[b] && gains[b], "rms_mix: branch %d is missing", b);
        in.rows[b] = branch_rows[b];
        in.gain[b] = AnyVec{gains[b], gain_dtype};
    }
    if (rows >= kNormManyRows) rms_mix_kernel<kNormThreadsMany><<<rows, kNormThreadsMany, 0, stream>>>(in, branches, eps, scale, out, hidden);
    else rms_mix_kernel<kNormThreadsFew><<<rows, kNormThreadsFew, 0, stream>>>(in, branches, eps, scale, out, hidden);
    LEONE_LAUNCH_CHECK("rms_mix");
    return 0;
}

extern "C" int leone_weighted_mix(const float* const* branch_rows, const float* weights, int branches, float* out, long n,
                                  hipStream_t stream) {
    LEONE_REQUIRE(branch_rows && weights && out && n > 0, "weighted_mix: needs branches and a positive size");
    LEONE_REQUIRE(branches >= 1 && branches <= kMaxBranches, "weighted_mix: %d branches, the kernel takes 1..%d", branches, kMaxBranches);
    Branches in{};
    float w[kMaxBranches] = {0.f, 0.f, 0.f, 0.f};
    for (int b = 0; b < branches; ++b) {
        LEONE_REQUIRE(branch_rows[b], "weighted_mix: branch %d is missing", b);
        in.rows[b] = branch_rows[b];
        w[b] = weights[b];
    }
    const long blocks = (n + 255) / 256;
    weighted_mix_kernel<<<static_cast<int>(blocks < 4096 ? blocks : 4096), 256, 0, stream>>>(in, branches, w[0], w[1], w[2], w[3], out, n);
    LEONE_LAUNCH_CHECK("weighted_mix");
    return 0;
}

extern "C" int leone_relu_squared(const void* in, void* out, int dtype, long n, hipStream_t stream) {
    LEONE_REQUIRE(in && out && n > 0 && known(dtype), "relu_squared: needs values of a known type");
    const long blocks = (n + 255) / 256;
    const int grid = static_cast<int>(blocks < 8192 ? blocks : 8192);
    if (dtype == kF32) relu_squared_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(in), static_cast<float*>(out), n);
    else relu_squared_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), n);
    LEONE_LAUNCH_CHECK("relu_squared");
    return 0;
}

extern "C" int leone_head_gate(void* out, int dtype, const float* gate, long gate_stride, int rows, int heads, int vdim,
                               hipStream_t stream) {
    LEONE_REQUIRE(out && gate && known(dtype) && rows > 0 && heads > 0 && vdim > 0, "head_gate: needs values and gates");
    const long n = static_cast<long>(rows) * heads * vdim;
    LEONE_REQUIRE((n + 255) / 256 <= 0x7fffffffL, "head_gate: too many values");
    const int grid = static_cast<int>((n + 255) / 256);
    if (dtype == kF32) head_gate_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), gate, gate_stride, heads, vdim, n);
    else head_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), gate, gate_stride, heads, vdim, n);
    LEONE_LAUNCH_CHECK("head_gate");
    return 0;
}
