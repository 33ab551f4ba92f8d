// A matrix memory whose forget gate, one per head and key channel, also says what is written:
//
//   gated_scan    f_t = lower + (1 - lower) * sigmoid(pre_t + bias)          per head and key channel
//                 S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,   o_t = S_t^T q_t,   q_t = act(q_pre_t)
//                 (1 - f_t is taken as (1 - lower) * sigmoid(-(pre_t + bias)), which keeps its digits where f_t
//                 is close to 1)
//   state_space_scan   the same walk for a state-space layer whose decay is one number a head and row:
//                 dt_t = softplus(pre_t + bias),  f_t = exp(-exp(rate_log) * dt_t)  for every key channel of the head,
//                 S_t = f_t S_(t-1) + (dt_t B_t) x_t^T,   o_t = S_t^T C_t + skip * x_t
//                 with B and C shared by the heads of a group (head h reads group h / (heads / groups))
//   gated_chain   chains the end states of chunks that were walked side by side (see below).
//
// The layout is that of the other matrix-memory recurrences: a workgroup of four waves owns a run of columns of one
// head of one segment (a request's rows in the step, or a chunk of them) and walks the rows in order, so a single
// decoded token and a prompt portion are the same kernel.  A column's key channels are spread over 1, 2, 4 or 8
// lanes, 32 to a lane in registers, two columns a lane; q, f and 1 - f of 16 rows at a time are made in shared
// memory by all threads; the lanes of a column add their parts of a read-out by shuffles.
//
// A long portion is cut into chunks that are walked side by side, three launches instead of one: every chunk from
// zeros (what its own rows write and what they read of it; the walk also leaves, per key channel, the product of the
// chunk's gates), then the chunks' end states chained into the state every chunk starts from (gated_chain: S <- product
// * S + end state, row by row of S), then every chunk once more from that state with nothing written into it
// (`no_input`), added to the first walk's read-outs.  Everything here is float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kGsTokens = 16;
constexpr int kGsLaneRows = 32;      // key channels a lane holds
constexpr int kGsThreads = 256;
constexpr int kGsLaneCols = 2;       // columns a lane holds: every q and gate it reads serves both
constexpr int kGsMaxDim = 256;

inline int gs_lane_groups(int dim) { return dim <= 32 ? 1 : dim <= 64 ? 2 : dim <= 128 ? 4 : 8; }

struct GsSegment {
    int first, end, in, out;        // rows [first, end); state read (negative: zeros) and written (negative: nowhere)
};

struct GatedScanArgs {
    const float* proj;              // [rows, stride]
    long stride;
    int q_off, f_off, v_off;        // columns of head 0; head h of q and f at + h * dim, of v at + h * vdim
    AnyVec f_bias, lower;           // [heads * dim]
    int q_silu;                     // q = silu(q_pre) instead of q_pre
    int no_input;                   // nothing is written: the state is only carried through the rows and read
    int accumulate;                 // read-outs are added to what out holds
    const GsSegment* segments;
    const float* state_in;          // [index, heads, dim * vdim]
    long in_stride;
    float* state_out;
    long out_stride;
    float* gate_product;            // [segments, heads, dim]: the product of f_t over the segment's rows, or null
    float* out;                     // [rows, heads, vdim]
    int heads, dim, vdim;
    // the state-space form: q (the read vector C) and the write vector B come in qk_heads groups of dim columns
    // (B's group 0 at k_off), the step size's pre-activation at step[row * step_stride + step_off + head]
    int qk_heads, k_off;
    const float* step;
    long step_stride;
    int step_off;
    AnyVec step_bias, rate_log, skip;   // [heads] each
};

enum GsKind : int { kGsGated = 0, kGsStateSpace = 1 };

template <bool kTrack, int kKind>
__global__ void __launch_bounds__(kGsThreads) gated_scan_kernel(GatedScanArgs p, int groups) {
    extern __shared__ __align__(16) float gs_lds[];
    const int dkp = groups * kGsLaneRows;
    float* sq = gs_lds;                          // [kGsTokens][dkp]
    float* sf = sq + kGsTokens * dkp;            // f_t
    float* sk = sf + kGsTokens * dkp;            // 1 - f_t
    const int head = blockIdx.y, tid = threadIdx.x, lane = tid % kWave;
    const GsSegment seg = p.segments[blockIdx.x];
    const int per_wave = kWave / groups;
    const int part = lane / per_wave;
    int col[kGsLaneCols];
#pragma unroll
    for (int c = 0; c < kGsLaneCols; ++c)
        col[c] = ((blockIdx.z * (blockDim.x / kWave) + tid / kWave) * kGsLaneCols + c) * per_wave + lane % per_wave;
    const int first = seg.first, n = seg.end - seg.first;
    const int ch0 = part * kGsLaneRows;
    const int shared_head = kKind == kGsStateSpace ? head / (p.heads / p.qk_heads) : head;
    const float skip = kKind == kGsStateSpace ? load_any(p.skip, head) : 0.f;
    const float rate = kKind == kGsStateSpace ? expf(load_any(p.rate_log, head)) : 0.f;
    const float* from = seg.in < 0 ? nullptr : p.state_in + seg.in * p.in_stride + static_cast<long>(head) * p.dim * p.vdim;

    float S[kGsLaneCols][kGsLaneRows];
    float carried[kTrack ? kGsLaneRows : 1];
#pragma unroll
    for (int c = 0; c < kGsLaneCols; ++c)
#pragma unroll
        for (int i = 0; i < kGsLaneRows; ++i)
            S[c][i] = (from && ch0 + i < p.dim && col[c] < p.vdim) ? from[static_cast<long>(ch0 + i) * p.vdim + col[c]] : 0.f;
    if constexpr (kTrack) {
#pragma unroll
        for (int i = 0; i < kGsLaneRows; ++i) carried[i] = 1.f;
    }

    __shared__ float s_dt[kGsTokens], s_decay[kGsTokens];   // the state-space form: a row's step size and decay, made once
    for (int t0 = 0; t0 < n; t0 += kGsTokens) {
        const int here = min(kGsTokens, n - t0);
        if (kKind == kGsStateSpace) {
            if (tid < here) {
                const float z = p.step[static_cast<long>(first + t0 + tid) * p.step_stride + p.step_off + head] + load_any(p.step_bias, head);
                const float dt = z > 20.f ? z : log1pf(expf(z));
                s_dt[tid] = dt;
                s_decay[tid] = expf(-rate * dt);
            }
            __syncthreads();
        }
        for (int idx = tid; idx < here * dkp; idx += blockDim.x) {
            const int t = idx / dkp, i = idx % dkp;
            float qv = 0.f, fv = 1.f, kv = 0.f;
            if (kKind == kGsStateSpace) {
                if (i < p.dim) {
                    const long r = first + t0 + t;
                    const float* base = p.proj + r * p.stride;
                    qv = base[p.q_off + shared_head * p.dim + i];
                    fv = s_decay[t];
                    kv = p.no_input ? 0.f : s_dt[t] * base[p.k_off + shared_head * p.dim + i];
                }
            } else if (i < p.dim) {
                const float* base = p.proj + static_cast<long>(first + t0 + t) * p.stride;
                const float qp = base[p.q_off + head * p.dim + i];
                qv = p.q_silu ? qp / (1.0f + expf(-qp)) : qp;
                const int ch = head * p.dim + i;
                const float z = base[p.f_off + ch] + load_any(p.f_bias, ch);
                const float low = load_any(p.lower, ch);
                fv = low + (1.0f - low) / (1.0f + expf(-z));
                kv = p.no_input ? 0.f : (1.0f - low) / (1.0f + expf(z));
            }
            sq[idx] = qv;
            sf[idx] = fv;
            sk[idx] = kv;
        }
        __syncthreads();
        if (col[0] < p.vdim) {                                  // the lanes of a column are in or out together
            for (int t = 0; t < here; ++t) {
                const long row = first + t0 + t;
                const float* ft = sf + t * dkp + ch0;
                const float* kt = sk + t * dkp + ch0;
                const float* qt = sq + t * dkp + ch0;
                float acc[kGsLaneCols], v[kGsLaneCols];
#pragma unroll
                for (int c = 0; c < kGsLaneCols; ++c) {
                    acc[c] = 0.f;
                    v[c] = (!p.no_input && col[c] < p.vdim) ? p.proj[row * p.stride + p.v_off + head * p.vdim + col[c]] : 0.f;
                }
#pragma unroll
                for (int i = 0; i < kGsLaneRows; ++i) {
                    const float f = ft[i], k = kt[i], q = qt[i];
#pragma unroll
                    for (int c = 0; c < kGsLaneCols; ++c) {
                        S[c][i] = fmaf(f, S[c][i], k * v[c]);
                        acc[c] = fmaf(S[c][i], q, acc[c]);
                    }
                    if constexpr (kTrack) carried[i] *= f;
                }
#pragma unroll
                for (int c = 0; c < kGsLaneCols; ++c) {
                    for (int off = per_wave; off < kWave; off <<= 1) acc[c] += __shfl_xor(acc[c], off, kWave);
                    if (part == 0 && col[c] < p.vdim) {
                        float* dst = p.out + (row * p.heads + head) * p.vdim + col[c];
                        const float read = kKind == kGsStateSpace ? fmaf(skip, v[c], acc[c]) : acc[c];
                        *dst = p.accumulate ? *dst + read : read;
                    }
                }
            }
        }
        __syncthreads();
    }
    if constexpr (kTrack) {
        if (p.gate_product && blockIdx.z == 0 && tid < kWave && lane % per_wave == 0) {
            float* to = p.gate_product + (static_cast<long>(blockIdx.x) * p.heads + head) * p.dim;
#pragma unroll
            for (int i = 0; i < kGsLaneRows; ++i)
                if (ch0 + i < p.dim) to[ch0 + i] = carried[i];
        }
    }
    if (!p.state_out || seg.out < 0) return;
    float* to = p.state_out + seg.out * p.out_stride + static_cast<long>(head) * p.dim * p.vdim;
#pragma unroll
    for (int c = 0; c < kGsLaneCols; ++c) {
        if (col[c] >= p.vdim) continue;
#pragma unroll
        for (int i = 0; i < kGsLaneRows; ++i)
            if (ch0 + i < p.dim) to[static_cast<long>(ch0 + i) * p.vdim + col[c]] = S[c][i];
    }
}

// links[l] = (slot, fresh, g0, g1): for a long portion whose chunks are [g0, g1) of `work` (each holding what its own
// rows wrote, from zeros), S = the request's state (zeros at a sequence's start); for every chunk in order what the
// chunk holds is replaced by S (the state it starts from), and S <- product[chunk][channel] * S + what it held.  The
// last S is the request's new state.
__global__ void gated_chain_kernel(const int* __restrict__ links, float* __restrict__ work, long work_stride,
                                   const float* __restrict__ product, float* __restrict__ state, long slot_stride,
                                   int heads, int dim, int vdim, int write_state) {
    const int l = blockIdx.x, head = blockIdx.y;
    const int el = blockIdx.z * blockDim.x + threadIdx.x;
    if (el >= dim * vdim) return;
    const int channel = el / vdim;
    const int slot = links[4 * l], fresh = links[4 * l + 1], g0 = links[4 * l + 2], g1 = links[4 * l + 3];
    const long at_head = static_cast<long>(head) * dim * vdim + el;
    float* mine = state + slot * slot_stride + at_head;
    float S = fresh ? 0.f : *mine;
    for (int g = g0; g < g1; ++g) {
        float* at = work + g * work_stride + at_head;
        const float wrote = *at;
        *at = S;
        S = fmaf(product[(static_cast<long>(g) * heads + head) * dim + channel], S, wrote);
    }
    if (write_state) *mine = S;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_gated_scan(const float* proj, long stride, int q_off, int f_off, int v_off, const void* f_bias,
                                const void* lower, int vec_dtype, int q_silu, int no_input, int accumulate,
                                const int* segments, int n_segments, const float* state_in, long in_stride, float* state_out,
                                long out_stride, float* gate_product, float* out, int heads, int dim, int vdim,
                                hipStream_t stream) {
    LEONE_REQUIRE(proj && f_bias && lower && segments && out, "gated_scan: null pointer");
    LEONE_REQUIRE(vec_dtype == kF32 || vec_dtype == kBF16, "gated_scan: unknown element type");
    LEONE_REQUIRE(n_segments > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0, "gated_scan: %d segments, %d heads of %d x %d",
                  n_segments, heads, dim, vdim);
    LEONE_REQUIRE(dim <= kGsMaxDim, "gated_scan: heads of %d key channels, the kernel takes up to %d", dim, kGsMaxDim);
    const long per_slot = static_cast<long>(heads) * dim * vdim;
    LEONE_REQUIRE((!state_in || in_stride >= per_slot) && (!state_out || out_stride >= per_slot),
                  "gated_scan: states of %ld floats do not fit", per_slot);
    LEONE_REQUIRE(q_off >= 0 && f_off >= 0 && v_off >= 0 && stride >= q_off + heads * dim && stride >= f_off + heads * dim &&
                  stride >= v_off + heads * vdim, "gated_scan: the projection's rows of %ld do not hold the named columns", stride);
    GatedScanArgs a{proj, stride, q_off, f_off, v_off, AnyVec{f_bias, vec_dtype}, AnyVec{lower, vec_dtype}, q_silu, no_input,
                    accumulate, reinterpret_cast<const GsSegment*>(segments), state_in, in_stride, state_out, out_stride,
                    gate_product, out, heads, dim, vdim, heads, 0, nullptr, 0, 0, AnyVec{nullptr, vec_dtype},
                    AnyVec{nullptr, vec_dtype}, AnyVec{nullptr, vec_dtype}};
    const int groups = gs_lane_groups(dim);
    const int per_block = (kGsThreads / kWave) * (kWave / groups) * kGsLaneCols;
    const dim3 grid(n_segments, heads, ceil_div(vdim, per_block));
    const size_t shared = 3 * kGsTokens * groups * kGsLaneRows * sizeof(float);
    if (gate_product) gated_scan_kernel<true, kGsGated><<<grid, kGsThreads, shared, stream>>>(a, groups);
    else gated_scan_kernel<false, kGsGated><<<grid, kGsThreads, shared, stream>>>(a, groups);
    LEONE_LAUNCH_CHECK("gated_scan");
    return 0;
}

// The state-space form.  xbc float [rows, stride] holds x (heads * vdim columns from x_off), B and C (groups * dim columns
// each from b_off and c_off); step float [rows, step_stride] the step sizes' pre-activations (heads columns from step_off);
// step_bias, rate_log, skip [heads] of vec_dtype.  States, segments, products and out as for leone_gated_scan (dim is the
// state size a head, the rows of S).
extern "C" int leone_state_space_scan(const float* xbc, long stride, int x_off, int b_off, int c_off, int groups_bc,
                                      const float* step, long step_stride, int step_off, const void* step_bias,
                                      const void* rate_log, const void* skip, int vec_dtype, int no_input, int accumulate,
                                      const int* segments, int n_segments, const float* state_in, long in_stride,
                                      float* state_out, long out_stride, float* gate_product, float* out, int heads, int dim,
                                      int vdim, hipStream_t stream) {
    LEONE_REQUIRE(xbc && step && step_bias && rate_log && skip && segments && out, "state_space_scan: null pointer");
    LEONE_REQUIRE(vec_dtype == kF32 || vec_dtype == kBF16, "state_space_scan: unknown element type");
    LEONE_REQUIRE(n_segments > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0, "state_space_scan: %d segments, %d heads of %d x %d",
                  n_segments, heads, dim, vdim);
    LEONE_REQUIRE(groups_bc > 0 && heads % groups_bc == 0, "state_space_scan: %d heads do not share %d groups evenly", heads, groups_bc);
    LEONE_REQUIRE(dim <= kGsMaxDim, "state_space_scan: states of %d rows a head, the kernel takes up to %d", dim, kGsMaxDim);
    const long per_slot = static_cast<long>(heads) * dim * vdim;
    LEONE_REQUIRE((!state_in || in_stride >= per_slot) && (!state_out || out_stride >= per_slot),
                  "state_space_scan: states of %ld floats do not fit", per_slot);
    LEONE_REQUIRE(x_off >= 0 && b_off >= 0 && c_off >= 0 && stride >= x_off + heads * vdim && stride >= b_off + groups_bc * dim &&
                  stride >= c_off + groups_bc * dim, "state_space_scan: rows of %ld do not hold the named columns", stride);
    LEONE_REQUIRE(step_off >= 0 && step_stride >= step_off + heads, "state_space_scan: rows of %ld do not hold %d step sizes",
                  step_stride, heads);
    GatedScanArgs a{xbc, stride, c_off, 0, x_off, AnyVec{nullptr, vec_dtype}, AnyVec{nullptr, vec_dtype}, 0, no_input,
                    accumulate, reinterpret_cast<const GsSegment*>(segments), state_in, in_stride, state_out, out_stride,
                    gate_product, out, heads, dim, vdim, groups_bc, b_off, step, step_stride, step_off,
                    AnyVec{step_bias, vec_dtype}, AnyVec{rate_log, vec_dtype}, AnyVec{skip, vec_dtype}};
    const int groups = gs_lane_groups(dim);
    // heads of few columns: a workgroup of as many waves as hold them (a wave holds 2 * 64 / groups columns), so that no
    // wave stands idle beside the others
    const int per_wave = (kWave / groups) * kGsLaneCols;
    const int waves = ceil_div(vdim, per_wave) < kGsThreads / kWave ? ceil_div(vdim, per_wave) : kGsThreads / kWave;
    const int per_block = waves * per_wave;
    const dim3 grid(n_segments, heads, ceil_div(vdim, per_block));
    const size_t shared = 3 * kGsTokens * groups * kGsLaneRows * sizeof(float);
    if (gate_product) gated_scan_kernel<true, kGsStateSpace><<<grid, waves * kWave, shared, stream>>>(a, groups);
    else gated_scan_kernel<false, kGsStateSpace><<<grid, waves * kWave, shared, stream>>>(a, groups);
    LEONE_LAUNCH_CHECK("state_space_scan");
    return 0;
}

extern "C" int leone_gated_chain(const int* links, int n_links, float* work, long work_stride, const float* product,
                                 float* state, long slot_stride, int heads, int dim, int vdim, int write_state,
                                 hipStream_t stream) {
    LEONE_REQUIRE(links && work && product && state && n_links > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0,
                  "gated_chain: null pointer or empty sizes");
    const long per_slot = static_cast<long>(heads) * dim * vdim;
    LEONE_REQUIRE(work_stride >= per_slot && slot_stride >= per_slot && ceil_div(static_cast<long>(dim) * vdim, 256) <= 65535,
                  "gated_chain: states of %ld floats do not fit", per_slot);
    gated_chain_kernel<<<dim3(n_links, heads, ceil_div(static_cast<long>(dim) * vdim, 256)), 256, 0, stream>>>(
        links, work, work_stride, product, state, slot_stride, heads, dim, vdim, write_state);
    LEONE_LAUNCH_CHECK("gated_chain");
    return 0;
}
