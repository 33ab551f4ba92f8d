// A feed-forward of routed experts: the router's choice, the rows sorted by expert, the experts' products.
//
//   route_topk   scores s = softmax(z) over all router outputs (float); choice scores s + correction; experts in
//                equal groups of neighbours, a group's score its best choice score, only the best `keep` groups
//                stay open (the others count as minus infinity); the `top` best open choice scores win; the
//                weights are the winners' s over their sum (+ 1e-20).
//   moe_plan     the (row, place) pairs of every expert gathered into tiles of pairs of one expert.
//   route_plan   both in one launch of one workgroup, for steps of few rows; experts that every row takes with
//                weight 1 (a shared expert cut to the experts' size) may stand behind the routed ones.
//   moe_product  gated: act(W_gate x) * (W_up x) of every pair, by its expert's matrices; else W_down of that, times
//                the pair's weight, float.  Three kernels: any type and size (float sums of 8-element runs a lane);
//                bfloat16 on the matrix cores from registers (tiles of 16 or 64 pairs); bfloat16 on the matrix cores
//                through shared memory (tiles of 128 pairs x 128 rows).
//   moe_combine  a row's pairs summed in the order of its places; a router output beyond the experts with
//                matrices hands the row itself on (times its weight); a delta that comes along is added.
//
// Every grid is fixed by the step's row count alone (tiles that turn out unused end at once), so a step that is
// recorded once can be replayed with other choices.  Products accumulate in float from operands of the engine's
// type; the router, its softmax and the weights are float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kRouteSlots = 8;                 // router outputs a lane holds: up to 512 experts
constexpr int kTilePairs = 8;                  // pairs of one expert a workgroup of the products takes
constexpr int kMoeThreads = 256;
constexpr int kMoeWaves = kMoeThreads / kWave;
constexpr int kColsPerWave = 4;
constexpr int kMoeCols = kMoeWaves * kColsPerWave;

// The better of two (value, index): the larger value, the lower index among equals.
__device__ inline void wave_best(float& v, int& at) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float v2 = __shfl_xor(v, off, kWave);
        const int at2 = __shfl_xor(at, off, kWave);
        if (v2 > v || (v2 == v && at2 < at)) {
            v = v2;
            at = at2;
        }
    }
}

// One wave a row; a lane holds kSlots router outputs (kSlots * 64 >= total).
// How a router scores and weighs: `score` 0 softmax over all outputs, 1 a sigmoid of each; `group_best` how many of a
// group's best choice scores make the group's score (their sum; 1: the best alone); `renorm` 1: the winners' scores over
// their sum, 0: the scores themselves; `scale` multiplies the weights either way.
struct RouteRule {
    int score, group_best, renorm;
    float scale;
};

template <int kSlots>
__device__ inline void route_row(int row, int lane, const float* __restrict__ logits, const AnyVec& correction,
                                 int* __restrict__ chosen, float* __restrict__ weight, int total, int top, int group_count,
                                 int group_keep, const RouteRule rule, int shift_from = 0x7fffffff, int always = 0) {
    // `always` experts that every row takes with weight 1 stand behind the routed ones in the matrices (indices
    // shift_from .. shift_from + always - 1): a row's places are its `top` choices and then these; a chosen router
    // output from shift_from on (one that hands the row on) is numbered behind them.
    const int places = top + always;
    const float* z = logits + static_cast<long>(row) * total;
    float s[kSlots], choice[kSlots];
    bool taken[kSlots];
    float top_z = -INFINITY;
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
        const int e = lane + i * kWave;
        s[i] = e < total ? z[e] : -INFINITY;
        top_z = fmaxf(top_z, s[i]);
    }
    top_z = wave_max(top_z);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
        const int e = lane + i * kWave;
        if (rule.score == 1) s[i] = e < total ? 1.0f / (1.0f + expf(-s[i])) : 0.f;
        else s[i] = e < total ? expf(s[i] - top_z) : 0.f;
        sum += s[i];
    }
    sum = rule.score == 1 ? 1.0f : wave_sum(sum);
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
        const int e = lane + i * kWave;
        s[i] = s[i] / sum;
        choice[i] = e < total ? s[i] + (correction.ptr ? load_any(correction, e) : 0.f) : -INFINITY;
        taken[i] = e >= total;
    }
    if (group_count > 1) {
        // a group's score: lane g % 64 keeps group g's in its place g / 64 (there are no more groups than outputs)
        const int size = total / group_count;
        int group_of[kSlots];
#pragma unroll
        for (int i = 0; i < kSlots; ++i) group_of[i] = (lane + i * kWave) / size;
        float mine[kSlots];
        bool mine_taken[kSlots];
#pragma unroll
        for (int i = 0; i < kSlots; ++i) {
            mine[i] = -INFINITY;
            mine_taken[i] = lane + i * kWave >= group_count;
        }
        for (int g = 0; g < group_count; ++g) {
            float best = 0.f;
            int used[kSlots];                              // the group's outputs already counted into its score
#pragma unroll
            for (int i = 0; i < kSlots; ++i) used[i] = 0;
            for (int n = 0; n < rule.group_best && n < size; ++n) {
                float v = -INFINITY;
                int at = 0x7fffffff;
#pragma unroll
                for (int i = 0; i < kSlots; ++i) {
                    const int e = lane + i * kWave;
                    if (e < total && group_of[i] == g && !used[i] && (at == 0x7fffffff || choice[i] > v)) {
                        v = choice[i];
                        at = e;
                    }
                }
                wave_best(v, at);
#pragma unroll
                for (int i = 0; i < kSlots; ++i)
                    if (lane + i * kWave == at) used[i] = 1;
                best = n == 0 ? v : best + v;
            }
#pragma unroll
            for (int i = 0; i < kSlots; ++i)
                if (lane + i * kWave == g) mine[i] = best;
        }
        unsigned open = 0u;                                   // bit i: group lane + 64 i stays open
        for (int n = 0; n < group_keep; ++n) {
            float v = -INFINITY;
            int at = 0x7fffffff;
#pragma unroll
            for (int i = 0; i < kSlots; ++i)
                if (!mine_taken[i] && (at == 0x7fffffff || mine[i] > v)) {
                    v = mine[i];
                    at = lane + i * kWave;
                }
            wave_best(v, at);
            if (at == 0x7fffffff) break;
#pragma unroll
            for (int i = 0; i < kSlots; ++i)
                if (lane + i * kWave == at) {
                    mine_taken[i] = true;
                    open |= 1u << i;
                }
        }
#pragma unroll
        for (int i = 0; i < kSlots; ++i) {
            const int e = lane + i * kWave;
            const int g = e < total ? group_of[i] : 0;
            const unsigned theirs = __shfl(open, g % kWave, kWave);
            if (e < total && !((theirs >> (g / kWave)) & 1u)) choice[i] = -INFINITY;
        }
    }
    float picked_sum = 0.f;
    float my_s = 0.f;
    int my_e = 0;
    for (int n = 0; n < top; ++n) {
        float v = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < kSlots; ++i) {
            const int e = lane + i * kWave;
            if (!taken[i] && (at == 0x7fffffff || choice[i] > v)) {
                v = choice[i];
                at = e;
            }
        }
        wave_best(v, at);
        float got = 0.f;
#pragma unroll
        for (int i = 0; i < kSlots; ++i) {
            const int e = lane + i * kWave;
            if (e == at) {
                taken[i] = true;
                got = s[i];
            }
        }
        got = wave_sum(got);               // one lane held it
        picked_sum += got;
        if (lane == n % kWave && n < kWave) {
            my_s = got;
            my_e = at;
        }
        if (n >= kWave && lane == 0) {       // more than 64 places: written as they come, scaled below
            chosen[static_cast<long>(row) * places + n] = at >= shift_from ? at + always : at;
            weight[static_cast<long>(row) * places + n] = got;
        }
    }
    const float denom = rule.renorm ? picked_sum + 1e-20f : 1.0f;
    if (lane < top && lane < kWave) {
        chosen[static_cast<long>(row) * places + lane] = my_e >= shift_from ? my_e + always : my_e;
        weight[static_cast<long>(row) * places + lane] = my_s / denom * rule.scale;
    }
    if (top > kWave && lane == 0)
        for (int n = kWave; n < top; ++n)
            weight[static_cast<long>(row) * places + n] = weight[static_cast<long>(row) * places + n] / denom * rule.scale;
    for (int i = lane; i < always; i += kWave) {
        chosen[static_cast<long>(row) * places + top + i] = shift_from + i;
        weight[static_cast<long>(row) * places + top + i] = 1.0f;
    }
}

__global__ void __launch_bounds__(kWave)
route_topk_kernel(const float* __restrict__ logits, AnyVec correction, int* __restrict__ chosen, float* __restrict__ weight,
                  int total, int top, int group_count, int group_keep, RouteRule rule) {
    if (total <= kWave) route_row<1>(blockIdx.x, threadIdx.x, logits, correction, chosen, weight, total, top, group_count, group_keep, rule);
    else if (total <= 2 * kWave) route_row<2>(blockIdx.x, threadIdx.x, logits, correction, chosen, weight, total, top, group_count, group_keep, rule);
    else route_row<kRouteSlots>(blockIdx.x, threadIdx.x, logits, correction, chosen, weight, total, top, group_count, group_keep, rule);
}

// One workgroup.  counts and places live in shared memory (experts <= 1024).
__device__ inline void plan_tiles(const int* __restrict__ chosen, int pairs, int experts, int* __restrict__ tile_expert,
                                  int* __restrict__ tile_pairs, int max_tiles, int tile, int* count, int* first_tile) {
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
    for (int t = threadIdx.x; t < max_tiles; t += blockDim.x) tile_expert[t] = -1;
    for (long i = threadIdx.x; i < static_cast<long>(max_tiles) * tile; i += blockDim.x) tile_pairs[i] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            first_tile[e] = at;
            const int tiles = (count[e] + tile - 1) / tile;
            for (int t = 0; t < tiles && at + t < max_tiles; ++t) tile_expert[at + t] = e;
            at += tiles;
            count[e] = 0;
        }
    }
    __syncthreads();
    // Which place of its expert's tiles a pair gets does not matter to its result: every pair is worked out by itself.
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) {
            const int at = atomicAdd(&count[e], 1);
            const long place = static_cast<long>(first_tile[e]) * tile + at;
            if (place < static_cast<long>(max_tiles) * tile) tile_pairs[place] = p;
        }
    }
}

__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int* __restrict__ chosen, int pairs, int experts, int* __restrict__ tile_expert,
                int* __restrict__ tile_pairs, int max_tiles, int tile) {
    __shared__ int count[1024];
    __shared__ int first_tile[1024];
    plan_tiles(chosen, pairs, experts, tile_expert, tile_pairs, max_tiles, tile, count, first_tile);
}

// The router's choice and the tiles in one launch, for steps of few rows (a wave a row, 16 waves in turn).
__global__ void __launch_bounds__(1024)
route_plan_kernel(const float* __restrict__ logits, AnyVec correction, int* __restrict__ chosen, float* __restrict__ weight,
                  int rows, int total, int top, int group_count, int group_keep, int experts, int* __restrict__ tile_expert,
                  int* __restrict__ tile_pairs, int max_tiles, int tile, int always, RouteRule rule) {
    const int routed = experts - always;               // experts the router chooses among; the others every row takes
    __shared__ int count[1024];
    __shared__ int first_tile[1024];
    for (int row = threadIdx.x / kWave; row < rows; row += 1024 / kWave) {
        const int lane = threadIdx.x % kWave;
        if (total <= kWave) route_row<1>(row, lane, logits, correction, chosen, weight, total, top, group_count, group_keep, rule, routed, always);
        else if (total <= 2 * kWave) route_row<2>(row, lane, logits, correction, chosen, weight, total, top, group_count, group_keep, rule, routed, always);
        else route_row<kRouteSlots>(row, lane, logits, correction, chosen, weight, total, top, group_count, group_keep, rule, routed, always);
    }
    __syncthreads();                                   // the choices are written; the same workgroup reads them
    plan_tiles(chosen, rows * (top + always), experts, tile_expert, tile_pairs, max_tiles, tile, count, first_tile);
}

template <typename T>
__device__ inline void load8f(const T* __restrict__ p, int k, int limit, bool runs, float out[8]);

template <>
__device__ inline void load8f<float>(const float* __restrict__ p, int k, int limit, bool runs, float out[8]) {
    if (runs && k + 8 <= limit) {
        const float4 a = *reinterpret_cast<const float4*>(p + k);
        const float4 b = *reinterpret_cast<const float4*>(p + k + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = k + i < limit ? p[k + i] : 0.f;
}

template <>
__device__ inline void load8f<bf16_t>(const bf16_t* __restrict__ p, int k, int limit, bool runs, float out[8]) {
    if (runs && k + 8 <= limit) {
        const uint4 t = *reinterpret_cast<const uint4*>(p + k);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = k + i < limit ? to_float(p[k + i]) : 0.f;
}

// A tile's pairs against kMoeCols rows of its expert's matrices: a wave takes kColsPerWave rows, its lanes runs of
// eight elements of the inner size; sums over the lanes at the end.
//   kGated: w = [experts][2][n][k] (gate rows, then up rows), y[pair][col] = act(gate) * up in T
//   else:   w = [experts][n][k], y[pair][col] = weight[pair] * product in float
// x: kGated: row pair / top of [rows][k]; else row pair of [pairs][k].
template <typename T, bool kGated>
__global__ void __launch_bounds__(kMoeThreads)
moe_product_kernel(const T* __restrict__ x, const T* __restrict__ w, void* __restrict__ y, const float* __restrict__ pair_weight,
                   const int* __restrict__ tile_expert, const int* __restrict__ tile_pairs, int top, int n, int k, int act,
                   float limit, int runs) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int col0 = blockIdx.y * kMoeCols + wave * kColsPerWave;
    if (col0 >= n) return;
    int pair[kTilePairs];
#pragma unroll
    for (int p = 0; p < kTilePairs; ++p) pair[p] = tile_pairs[static_cast<long>(tile) * kTilePairs + p];
    float acc[kColsPerWave][kTilePairs], acc2[kGated ? kColsPerWave : 1][kTilePairs];
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c)
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            acc[c][p] = 0.f;
            if constexpr (kGated) acc2[c][p] = 0.f;
        }
    const long matrix = static_cast<long>(n) * k;
    const T* w_first = w + static_cast<long>(e) * (kGated ? 2 : 1) * matrix;
    for (int at = 8 * lane; at < k; at += 8 * kWave) {
        float xv[kTilePairs][8];
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            if (pair[p] >= 0) {
                load8f<T>(x + static_cast<long>(kGated ? pair[p] / top : pair[p]) * k, at, k, runs != 0, xv[p]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[p][i] = 0.f;
            }
        }
#pragma unroll
        for (int c = 0; c < kColsPerWave; ++c) {
            const int col = col0 + c;
            if (col >= n) continue;
            float wv[8], wv2[8];
            load8f<T>(w_first + static_cast<long>(col) * k, at, k, runs != 0, wv);
            if constexpr (kGated) load8f<T>(w_first + matrix + static_cast<long>(col) * k, at, k, runs != 0, wv2);
#pragma unroll
            for (int p = 0; p < kTilePairs; ++p)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc[c][p] = fmaf(wv[i], xv[p][i], acc[c][p]);
                    if constexpr (kGated) acc2[c][p] = fmaf(wv2[i], xv[p][i], acc2[c][p]);
                }
        }
    }
    // lane c * kTilePairs + p writes (column c, pair p)
    float mine = 0.f, mine2 = 0.f;
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c)
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            const float total = wave_sum(acc[c][p]);
            float total2 = 0.f;
            if constexpr (kGated) total2 = wave_sum(acc2[c][p]);
            if (lane == c * kTilePairs + p) {
                mine = total;
                mine2 = total2;
            }
        }
    if (lane < kColsPerWave * kTilePairs) {
        const int c = lane / kTilePairs, p = lane % kTilePairs;
        const int col = col0 + c;
        // the pair of this lane, without indexing the register array by a lane's value
        int which = -1;
#pragma unroll
        for (int q = 0; q < kTilePairs; ++q)
            if (q == p) which = pair[q];
        if (col < n && which >= 0) {
            if constexpr (kGated)
                static_cast<T*>(y)[static_cast<long>(which) * n + col] = from_float<T>(glu_value(mine, mine2, act, limit));
            else
                static_cast<float*>(y)[static_cast<long>(which) * n + col] = mine * pair_weight[which];
        }
    }
}


// The same products on the matrix cores, bfloat16: a workgroup takes a tile of 16 * kPB pairs of one expert and 64
// rows of its matrix, a wave 16 of those rows against all the tile's pairs (v_mfma_f32_16x16x32_bf16: the rows are
// one operand, 16 pairs the other; lane (c, g) holds elements 8 g .. 8 g + 7 of a step of 32 of row c and of pair c,
// and gets rows 4 g .. 4 g + 3 of pair c).  Inner sizes are multiples of 8; a step's lanes beyond the inner size
// bring zeros.
typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_floatx4 __attribute__((ext_vector_type(4)));

__device__ inline moe_bf16x8 moe_load8(const bf16_t* p) {
    return __builtin_bit_cast(moe_bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline moe_bf16x8 moe_zero8() {
    const uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(moe_bf16x8, z);
}

template <int kPB, int kRT, bool kGated>
__global__ void __launch_bounds__(kMoeThreads)
moe_product_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ y,
                        const float* __restrict__ pair_weight, const int* __restrict__ tile_expert,
                        const int* __restrict__ tile_pairs, int top, int n, int k, int act, float limit) {
    // kPB blocks of 16 pairs a tile; kRT blocks of 16 rows a wave (a workgroup takes 64 * kRT rows): the more of
    // both, the fewer times the rows of the matrix and of x are fetched again by other workgroups.
    constexpr int kTile = 16 * kPB;
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int c = lane & 15, g = lane >> 4;
    const int row0 = (blockIdx.y * kMoeWaves + wave) * 16 * kRT;
    if (row0 >= n) return;
    int pair[kPB];
    const bf16_t* xrow[kPB];
#pragma unroll
    for (int b = 0; b < kPB; ++b) {
        pair[b] = tile_pairs[static_cast<long>(tile) * kTile + 16 * b + c];
        xrow[b] = x + static_cast<long>(pair[b] < 0 ? 0 : (kGated ? pair[b] / top : pair[b])) * k;
    }
    const long matrix = static_cast<long>(n) * k;
    bool row_ok[kRT];
    const bf16_t* wa[kRT];
#pragma unroll
    for (int t = 0; t < kRT; ++t) {
        row_ok[t] = row0 + 16 * t + c < n;
        wa[t] = w + static_cast<long>(e) * (kGated ? 2 : 1) * matrix + static_cast<long>(row_ok[t] ? row0 + 16 * t + c : 0) * k;
    }
    moe_floatx4 acc[kRT][kPB], acc2[kGated ? kRT : 1][kPB];
#pragma unroll
    for (int t = 0; t < kRT; ++t)
#pragma unroll
        for (int b = 0; b < kPB; ++b) {
            acc[t][b] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
            if constexpr (kGated) acc2[t][b] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
        }
    // A ring of kDepth steps of 32: a step's operands are asked for kDepth steps before the matrix instructions
    // that use them run, so that a wave that has its SIMD to itself still keeps loads on their way.
    constexpr int kDepth = kPB * kRT >= 16 ? 4 : kPB >= 4 ? 4 : 8;
    moe_bf16x8 a[kDepth][kRT], a2[kDepth][kGated ? kRT : 1], xb[kDepth][kPB];
#define LEONE_MOE_FETCH(D, K0)                                                                                  \
    {                                                                                                           \
        const int at = (K0) + 8 * g;                                                                            \
        const bool in = at < k;                                                                                 \
        _Pragma("unroll") for (int t = 0; t < kRT; ++t) {                                                       \
            a[D][t] = (row_ok[t] && in) ? moe_load8(wa[t] + at) : moe_zero8();                                  \
            if constexpr (kGated) a2[D][t] = (row_ok[t] && in) ? moe_load8(wa[t] + matrix + at) : moe_zero8();  \
        }                                                                                                       \
        _Pragma("unroll") for (int b = 0; b < kPB; ++b)                                                         \
            xb[D][b] = (pair[b] >= 0 && in) ? moe_load8(xrow[b] + at) : moe_zero8();                            \
    }
#pragma unroll
    for (int d = 0; d < kDepth; ++d) LEONE_MOE_FETCH(d, 32 * d)
    for (int k0 = 0; k0 < k; k0 += 32 * kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (k0 + 32 * d < k) {                                   // the same for the whole workgroup
#pragma unroll
                for (int t = 0; t < kRT; ++t) {
#pragma unroll
                    for (int b = 0; b < kPB; ++b) {
                        acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[d][t], xb[d][b], acc[t][b], 0, 0, 0);
                        if constexpr (kGated)
                            acc2[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[d][t], xb[d][b], acc2[t][b], 0, 0, 0);
                    }
                }
            }
            LEONE_MOE_FETCH(d, k0 + 32 * (kDepth + d))
        }
    }
#undef LEONE_MOE_FETCH
#pragma unroll
    for (int b = 0; b < kPB; ++b) {
        if (pair[b] < 0) continue;
        const float scale = kGated ? 1.f : pair_weight[pair[b]];
#pragma unroll
        for (int t = 0; t < kRT; ++t) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = row0 + 16 * t + 4 * g + j;
                if (r >= n) continue;
                if constexpr (kGated)
                    static_cast<bf16_t*>(y)[static_cast<long>(pair[b]) * n + r] =
                        from_float<bf16_t>(glu_value(acc[t][b][j], acc2[t][b][j], act, limit));
                else
                    static_cast<float*>(y)[static_cast<long>(pair[b]) * n + r] = acc[t][b][j] * scale;
            }
        }
    }
}

// Tiles of 128 pairs, bfloat16: a workgroup takes a tile and 128 rows of its expert's matrix (gated: 128 gate rows and
// their up rows), in chunks of 64 of the inner size that go through shared memory: a row's chunk is one line of 128
// bytes, fetched whole by eight neighbouring threads (rows of a matrix lie a power of two apart, so lines that are
// only half used at a time push one another out of the caches before their other half is asked for).  While the
// waves work on a chunk the next is on its way from memory into registers.  In shared memory a chunk lies as two
// halves of 32 elements, rows one after the other within a half: the 16 rows of an operand are one kilobyte that the
// 64 lanes read in one piece.  The four waves take 64 rows x 64 pairs each: 4 + 4 operands for 16 matrix instructions.
constexpr int kBigPairs = 128;
constexpr int kBigRows = 128;
constexpr int kBigChunk = 64;

template <bool kGated>
__global__ void __launch_bounds__(kMoeThreads, 2)
moe_product_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ y,
                         const float* __restrict__ pair_weight, const int* __restrict__ tile_expert,
                         const int* __restrict__ tile_pairs, int top, int n, int k, int act, float limit, int n_tiles, int n_blocks) {
    constexpr int kWRows = kGated ? 2 * kBigRows : kBigRows;          // rows of the matrix in a chunk
    constexpr int kXPieces = kBigPairs * 8 / kMoeThreads;             // 16-byte pieces of x a thread brings per chunk
    constexpr int kWPieces = kWRows * 8 / kMoeThreads;
    __shared__ uint4 sx[2 * kBigPairs * 4];                           // [half][row][4 pieces]
    __shared__ uint4 sw[2 * kWRows * 4];
    // Workgroups go to the eight dies in turn, and each die has a cache of its own: the work is numbered so that a
    // die gets a run of neighbouring (row block, tile) places, tiles fastest: the tiles of one expert, which read the
    // same rows of its matrix, then lie on one die.
    const int per_die = (n_tiles * n_blocks + 7) / 8;
    const int place = static_cast<int>(blockIdx.x % 8) * per_die + static_cast<int>(blockIdx.x / 8);
    if (place >= n_tiles * n_blocks) return;
    const int tile = place % n_tiles;
    const int row_block = place / n_tiles;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int c = lane & 15, g = lane >> 4;
    const int wr = wave >> 1, wp = wave & 1;
    const int row_base = row_block * kBigRows;
    const long matrix = static_cast<long>(n) * k;
    const int* my_pairs = tile_pairs + static_cast<long>(tile) * kBigPairs;

    // what this thread brings: piece p = tid + 256 i is part p % 8 of row p / 8 (row tid / 8 + 32 i)
    const int part = tid & 7;
    const int half = part >> 2, quarter = part & 3;
    const bf16_t* x_from[kXPieces];
    const bf16_t* w_from[kWPieces];
#pragma unroll
    for (int i = 0; i < kXPieces; ++i) {
        const int pair = my_pairs[tid / 8 + 32 * i];
        x_from[i] = pair < 0 ? nullptr : x + static_cast<long>(kGated ? pair / top : pair) * k + 8 * part;
    }
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) {
        const int local = tid / 8 + 32 * i;                           // gated: rows 0..127 gate, 128..255 up
        const int row = row_base + (local % kBigRows);
        w_from[i] = row >= n ? nullptr
                             : w + static_cast<long>(e) * (kGated ? 2 : 1) * matrix + (local >= kBigRows ? matrix : 0) +
                                   static_cast<long>(row) * k + 8 * part;
    }
    uint4 hx[kXPieces], hw[kWPieces];

    moe_floatx4 acc[4][4], acc2[kGated ? 4 : 1][4];
#pragma unroll
    for (int ta = 0; ta < 4; ++ta)
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) {
            acc[ta][tb] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
            if constexpr (kGated) acc2[ta][tb] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
        }
    const int chunks = (k + kBigChunk - 1) / kBigChunk;
#define LEONE_MOE_BRING(K0)                                                                                              \
    {                                                                                                                    \
        const bool in = (K0) + 8 * part < k;                                                                             \
        _Pragma("unroll") for (int i = 0; i < kXPieces; ++i) {                                                           \
            hx[i] = uint4{0u, 0u, 0u, 0u};                                                                               \
            if (x_from[i] && in) hx[i] = *reinterpret_cast<const uint4*>(x_from[i] + (K0));                              \
        }                                                                                                                \
        _Pragma("unroll") for (int i = 0; i < kWPieces; ++i) {                                                           \
            hw[i] = uint4{0u, 0u, 0u, 0u};                                                                               \
            if (w_from[i] && in) hw[i] = *reinterpret_cast<const uint4*>(w_from[i] + (K0));                              \
        }                                                                                                                \
    }
    LEONE_MOE_BRING(0)
    for (int ck = 0; ck < chunks; ++ck) {
#pragma unroll
        for (int i = 0; i < kXPieces; ++i) sx[(half * kBigPairs + tid / 8 + 32 * i) * 4 + quarter] = hx[i];
#pragma unroll
        for (int i = 0; i < kWPieces; ++i) sw[(half * kWRows + tid / 8 + 32 * i) * 4 + quarter] = hw[i];
        __syncthreads();
        if (ck + 1 < chunks) LEONE_MOE_BRING((ck + 1) * kBigChunk)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            moe_bf16x8 a[4], a2[kGated ? 4 : 1], b[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                a[t] = __builtin_bit_cast(moe_bf16x8, sw[(h * kWRows + 64 * wr + 16 * t + c) * 4 + g]);
                if constexpr (kGated) a2[t] = __builtin_bit_cast(moe_bf16x8, sw[(h * kWRows + kBigRows + 64 * wr + 16 * t + c) * 4 + g]);
                b[t] = __builtin_bit_cast(moe_bf16x8, sx[(h * kBigPairs + 64 * wp + 16 * t + c) * 4 + g]);
            }
#pragma unroll
            for (int ta = 0; ta < 4; ++ta)
#pragma unroll
                for (int tb = 0; tb < 4; ++tb) {
                    acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ta], b[tb], acc[ta][tb], 0, 0, 0);
                    if constexpr (kGated) acc2[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[ta], b[tb], acc2[ta][tb], 0, 0, 0);
                }
        }
        __syncthreads();                               // everyone has read the chunk before the next is put down
    }
#undef LEONE_MOE_BRING
    // lane (c, g) holds rows 4 g .. 4 g + 3 of pair c of every (ta, tb)
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int pair = my_pairs[64 * wp + 16 * tb + c];
        if (pair < 0) continue;
        const float scale = kGated ? 1.f : pair_weight[pair];
#pragma unroll
        for (int ta = 0; ta < 4; ++ta) {
            const int r = row_base + 64 * wr + 16 * ta + 4 * g;
            if (r >= n) continue;
            float v0, v1, v2, v3;
            if constexpr (kGated) {
                v0 = glu_value(acc[ta][tb][0], acc2[ta][tb][0], act, limit);
                v1 = glu_value(acc[ta][tb][1], acc2[ta][tb][1], act, limit);
                v2 = glu_value(acc[ta][tb][2], acc2[ta][tb][2], act, limit);
                v3 = glu_value(acc[ta][tb][3], acc2[ta][tb][3], act, limit);
                bf16_t* to = static_cast<bf16_t*>(y) + static_cast<long>(pair) * n + r;
                if (r + 3 < n && n % 4 == 0) {
                    uint2 packed;
                    packed.x = bf16_bits_from_float(v0) | (static_cast<uint32_t>(bf16_bits_from_float(v1)) << 16);
                    packed.y = bf16_bits_from_float(v2) | (static_cast<uint32_t>(bf16_bits_from_float(v3)) << 16);
                    *reinterpret_cast<uint2*>(to) = packed;
                } else {
                    to[0] = from_float<bf16_t>(v0);
                    if (r + 1 < n) to[1] = from_float<bf16_t>(v1);
                    if (r + 2 < n) to[2] = from_float<bf16_t>(v2);
                    if (r + 3 < n) to[3] = from_float<bf16_t>(v3);
                }
            } else {
                v0 = acc[ta][tb][0] * scale;
                v1 = acc[ta][tb][1] * scale;
                v2 = acc[ta][tb][2] * scale;
                v3 = acc[ta][tb][3] * scale;
                float* to = static_cast<float*>(y) + static_cast<long>(pair) * n + r;
                if (r + 3 < n && n % 4 == 0) {
                    *reinterpret_cast<float4*>(to) = float4{v0, v1, v2, v3};
                } else {
                    to[0] = v0;
                    if (r + 1 < n) to[1] = v1;
                    if (r + 2 < n) to[2] = v2;
                    if (r + 3 < n) to[3] = v3;
                }
            }
        }
    }
}

// A workgroup takes 256 columns of a row; a thread one column.
template <typename T>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ pair_out, const int* __restrict__ chosen, const float* __restrict__ weight,
                   const T* __restrict__ x, const float* __restrict__ extra, float* __restrict__ out, int top, int experts,
                   int hidden) {
    const int row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= hidden) return;
    const int* ch = chosen + static_cast<long>(row) * top;
    const float* wt = weight + static_cast<long>(row) * top;
    const long at = static_cast<long>(row) * hidden + c;
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {                       // in the order of the row's places, whatever the tiles were
        const int e = ch[j];
        if (e >= experts)
            sum += wt[j] * to_float(x[at]);               // hands the row on as it came
        else if (e >= 0)
            sum += pair_out[(static_cast<long>(row) * top + j) * hidden + c];
    }
    if (extra != nullptr) sum += extra[at];
    out[at] = sum;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_moe_tile_pairs() { return kTilePairs; }
extern "C" int leone_route_max_outputs() { return kRouteSlots * kWave; }

extern "C" int leone_route_topk(const float* logits, const void* correction, int correction_dtype, int* chosen, float* weight,
                                int rows, int total, int top, int group_count, int group_keep, int score, int group_best,
                                int renorm, float weight_scale, hipStream_t stream) {
    LEONE_REQUIRE(logits && chosen && weight, "route_topk: null pointer");
    LEONE_REQUIRE((score == 0 || score == 1) && group_best >= 1 && (renorm == 0 || renorm == 1),
                  "route_topk: score kind %d, %d best of a group, renorm %d", score, group_best, renorm);
    LEONE_REQUIRE(rows > 0 && total > 0 && total <= kRouteSlots * kWave, "route_topk: rows %d, %d router outputs (at most %d)",
                  rows, total, kRouteSlots * kWave);
    LEONE_REQUIRE(top > 0 && top <= total, "route_topk: %d of %d outputs", top, total);
    LEONE_REQUIRE(!correction || correction_dtype == kF32 || correction_dtype == kBF16, "route_topk: unknown type of the correction");
    LEONE_REQUIRE(group_count >= 1 && total % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
                  "route_topk: %d groups (dividing %d outputs), %d kept", group_count, total, group_keep);
    route_topk_kernel<<<rows, kWave, 0, stream>>>(logits, AnyVec{correction, correction_dtype}, chosen, weight, total, top,
                                                  group_count, group_keep, RouteRule{score, group_best, renorm, weight_scale});
    LEONE_LAUNCH_CHECK("route_topk");
    return 0;
}

// leone_route_topk and leone_moe_plan in one launch (one workgroup: for steps of few rows).  `always`: the last so many
// of the `experts` are taken by every row with weight 1 (a shared expert cut to the experts' size): chosen and weight are
// [rows, top + always], a row's choices and then these; a chosen router output that stands for no matrix (from
// experts - always on in the router's numbering) is numbered from `experts` on.
extern "C" int leone_route_plan(const float* logits, const void* correction, int correction_dtype, int* chosen, float* weight,
                                int rows, int total, int top, int group_count, int group_keep, int experts, int* tile_expert,
                                int* tile_pairs, int max_tiles, int tile, int always, int score, int group_best, int renorm,
                                float weight_scale, hipStream_t stream) {
    LEONE_REQUIRE((score == 0 || score == 1) && group_best >= 1 && (renorm == 0 || renorm == 1),
                  "route_plan: score kind %d, %d best of a group, renorm %d", score, group_best, renorm);
    LEONE_REQUIRE(always >= 0 && always < experts, "route_plan: %d of %d experts for every row", always, experts);
    LEONE_REQUIRE(logits && chosen && weight && tile_expert && tile_pairs, "route_plan: null pointer");
    LEONE_REQUIRE(rows > 0 && rows <= 256 && total > 0 && total <= kRouteSlots * kWave, "route_plan: rows %d (at most 256), %d router outputs",
                  rows, total);
    LEONE_REQUIRE(top > 0 && top <= total, "route_plan: %d of %d outputs", top, total);
    LEONE_REQUIRE(!correction || correction_dtype == kF32 || correction_dtype == kBF16, "route_plan: unknown type of the correction");
    LEONE_REQUIRE(group_count >= 1 && total % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
                  "route_plan: %d groups (dividing %d outputs), %d kept", group_count, total, group_keep);
    LEONE_REQUIRE(experts > 0 && experts <= 1024, "route_plan: %d experts (at most 1024)", experts);
    LEONE_REQUIRE(tile == kTilePairs || tile == 16 || tile == 64 || tile == 128, "route_plan: tiles of %d pairs", tile);
    const long pairs = static_cast<long>(rows) * (top + always);
    const long needed = pairs / tile + experts;
    LEONE_REQUIRE(max_tiles >= (needed < pairs ? needed : pairs), "route_plan: %d tiles cannot hold %ld pairs of %d experts", max_tiles,
                  pairs, experts);
    route_plan_kernel<<<1, 1024, 0, stream>>>(logits, AnyVec{correction, correction_dtype}, chosen, weight, rows, total, top,
                                              group_count, group_keep, experts, tile_expert, tile_pairs, max_tiles, tile, always,
                                              RouteRule{score, group_best, renorm, weight_scale});
    LEONE_LAUNCH_CHECK("route_plan");
    return 0;
}

extern "C" int leone_moe_plan(const int* chosen, int pairs, int experts, int* tile_expert, int* tile_pairs, int max_tiles,
                              int tile, hipStream_t stream) {
    LEONE_REQUIRE(tile == kTilePairs || tile == 16 || tile == 64 || tile == 128, "moe_plan: tiles of %d pairs", tile);
    LEONE_REQUIRE(chosen && tile_expert && tile_pairs, "moe_plan: null pointer");
    LEONE_REQUIRE(pairs > 0 && experts > 0 && experts <= 1024, "moe_plan: %d pairs, %d experts (at most 1024)", pairs, experts);
    const long needed = static_cast<long>(pairs) / tile + experts;
    LEONE_REQUIRE(max_tiles >= (needed < pairs ? needed : pairs), "moe_plan: %d tiles cannot hold %d pairs of %d experts", max_tiles,
                  pairs, experts);
    moe_plan_kernel<<<1, 1024, 0, stream>>>(chosen, pairs, experts, tile_expert, tile_pairs, max_tiles, tile);
    LEONE_LAUNCH_CHECK("moe_plan");
    return 0;
}

// gated != 0: x [rows, k], w [experts, 2, n, k], y [pairs, n] of dtype = act(gate) * up (act: GateAct).
// gated == 0: x [pairs, k], w [experts, n, k], y float32 [pairs, n] = pair_weight[pair] * product.
// tile: pairs a tile holds, as leone_moe_plan was told: leone_moe_tile_pairs() for the kernel that takes any type and
// size; 16 or 64 for the matrix-core kernel (bfloat16, n and k multiples of 8).
extern "C" int leone_moe_product(const void* x, const void* w, void* y, const float* pair_weight, int dtype, int gated,
                                 const int* tile_expert, const int* tile_pairs, int max_tiles, int tile, int top, int n, int k,
                                 int act, float limit, hipStream_t stream) {
    if (tile != kTilePairs) {
        LEONE_REQUIRE(tile == 16 || tile == 64 || tile == 128, "moe_product: tiles of %d pairs", tile);
        LEONE_REQUIRE(dtype == kBF16 && k % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                      "moe_product: the matrix-core kernel takes bfloat16 with an inner size that is a multiple of 8, not %d", k);
        LEONE_REQUIRE(x && w && y && tile_expert && tile_pairs && (gated || pair_weight), "moe_product: null pointer");
        LEONE_REQUIRE(max_tiles > 0 && top > 0 && n > 0 && k > 0, "moe_product: %d tiles, sizes %d x %d", max_tiles, n, k);
        LEONE_REQUIRE(act == kGateSilu || act == kGateGeluTanh || (act == kGateClampedSwish && limit > 0.f), "moe_product: unknown activation %d (limit %g)", act, limit);
        const dim3 cores(max_tiles, ceil_div(n, tile == 128 ? 128 : 64));
        LEONE_REQUIRE(cores.y <= 65535, "moe_product: %d rows of a matrix are too many", n);
#define LEONE_MOE_CORES(PB, RT, G)                                                                                      \
    moe_product_mfma_kernel<PB, RT, G><<<cores, kMoeThreads, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), \
                                                                          y, pair_weight, tile_expert, tile_pairs, top, n, k, act, limit)
        if (tile == 16) {
            if (gated) LEONE_MOE_CORES(1, 1, true);
            else LEONE_MOE_CORES(1, 1, false);
        } else if (tile == 64) {
            if (gated) LEONE_MOE_CORES(4, 1, true);
            else LEONE_MOE_CORES(4, 1, false);
        } else {
            const long places = static_cast<long>(cores.x) * cores.y;
            LEONE_REQUIRE(places + 7 <= 0x7fffffffL, "moe_product: too many tiles");
            const int grid = static_cast<int>((places + 7) / 8 * 8);
            if (gated)
                moe_product_tiled_kernel<true><<<grid, kMoeThreads, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w),
                                                                                 y, pair_weight, tile_expert, tile_pairs, top, n, k, act, limit,
                                                                                 static_cast<int>(cores.x), static_cast<int>(cores.y));
            else
                moe_product_tiled_kernel<false><<<grid, kMoeThreads, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w),
                                                                                  y, pair_weight, tile_expert, tile_pairs, top, n, k, act, limit,
                                                                                  static_cast<int>(cores.x), static_cast<int>(cores.y));
        }
#undef LEONE_MOE_CORES
        LEONE_LAUNCH_CHECK("moe_product");
        return 0;
    }
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_product: unknown element type %d", dtype);
    LEONE_REQUIRE(x && w && y && tile_expert && tile_pairs && (gated || pair_weight), "moe_product: null pointer");
    LEONE_REQUIRE(max_tiles > 0 && top > 0 && n > 0 && k > 0, "moe_product: %d tiles, sizes %d x %d", max_tiles, n, k);
    LEONE_REQUIRE(act == kGateSilu || act == kGateGeluTanh || (act == kGateClampedSwish && limit > 0.f), "moe_product: unknown activation %d (limit %g)", act, limit);
    const uintptr_t run = 8 * (dtype == kF32 ? sizeof(float) : sizeof(bf16_t));
    const int runs = k % 8 == 0 && reinterpret_cast<uintptr_t>(x) % run == 0 && reinterpret_cast<uintptr_t>(w) % run == 0;
    const dim3 grid(max_tiles, ceil_div(n, kMoeCols));
    LEONE_REQUIRE(grid.y <= 65535, "moe_product: %d rows of a matrix are too many", n);
#define LEONE_MOE(T, G)                                                                                                   \
    moe_product_kernel<T, G><<<grid, kMoeThreads, 0, stream>>>(static_cast<const T*>(x), static_cast<const T*>(w), y, pair_weight, \
                                                               tile_expert, tile_pairs, top, n, k, act, limit, runs)
    if (dtype == kF32) {
        if (gated) LEONE_MOE(float, true);
        else LEONE_MOE(float, false);
    } else {
        if (gated) LEONE_MOE(bf16_t, true);
        else LEONE_MOE(bf16_t, false);
    }
#undef LEONE_MOE
    LEONE_LAUNCH_CHECK("moe_product");
    return 0;
}

extern "C" int leone_moe_combine(const float* pair_out, const int* chosen, const float* weight, const void* x, int dtype,
                                 const float* extra, float* out, int rows, int top, int experts, int hidden, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_combine: unknown element type %d", dtype);
    LEONE_REQUIRE(pair_out && chosen && weight && x && out, "moe_combine: null pointer");
    LEONE_REQUIRE(rows > 0 && top > 0 && experts >= 0 && hidden > 0, "moe_combine: rows %d, top %d, hidden %d", rows, top, hidden);
    const dim3 grid(rows, ceil_div(hidden, 256));
    LEONE_REQUIRE(grid.y <= 65535, "moe_combine: rows of %d are too wide", hidden);
    if (dtype == kF32)
        moe_combine_kernel<float><<<grid, 256, 0, stream>>>(pair_out, chosen, weight, static_cast<const float*>(x), extra, out, top,
                                                            experts, hidden);
    else
        moe_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(pair_out, chosen, weight, static_cast<const bf16_t*>(x), extra, out, top,
                                                             experts, hidden);
    LEONE_LAUNCH_CHECK("moe_combine");
    return 0;
}
