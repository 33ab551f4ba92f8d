// Attention through a latent: what a token leaves in the cache is one vector for all heads, a normed latent c of
// `rank` elements followed by a rotated key part of `rot` elements that every head shares.  Head h's key is
// (W_uk[h] c, rotated part), its value W_uv[h] c.  The kernels here never make those: the up-projections are taken
// to the query's and the result's side,
//
//     score_h(j) = (q_plain_h . W_uk[h] c_j + q_rot_h . r_j) * scale = ((W_uk[h]^T q_plain_h) . c_j + q_rot_h . r_j) * scale
//     out_h      = W_uv[h] (sum_j p_j c_j)
//
// so attention runs with one shared "key" (c_j, r_j) of rank + rot elements and one shared "value" c_j for all
// heads, straight from the cache:
//
//   latent_prepare    one row: the query latent RMS-normed (times its gain) for the product that follows; the key/value
//                     latent RMS-normed (times its gain), the shared key part rotated, both written into the cache
//                     page of the row's position.
//   head_product      y[r, h, :] = x[r, h, :] W[h] for W[h] [inner, outer] (a product a head, rows in tiles of 8);
//                     optionally the `tail` elements behind x's inner ones are rotated by the row's position and put
//                     behind y's outer ones: W_uk^T on the queries with the rotated query part, and W_uv on the result.
//   latent_attention  softmax attention of every (row, head) over the latents of its request inside the window.
//                     A workgroup takes one row and a few heads; its four waves take the keys in turn (so every
//                     cached vector is read once for all of the workgroup's heads), lanes split the elements; the
//                     waves' partial results are merged in a fixed order.
//
// The cache of one layer: [page][token in page][rank + rot] in the engine's type.  Norms, angles, scores, softmax and
// all sums are float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kLatThreads = 256;
constexpr int kLatWaves = kLatThreads / kWave;

// Rotation of the pair (2i, 2i + 1) of `src` by the row's angle i (tables already hold any growth of cos and sin);
// elements from 2 * rot_half on are handed through.
__device__ inline float rotated_adjacent(const float* src, int i, const float* cos_row, const float* sin_row, int rot_half) {
    if (!cos_row || i >= 2 * rot_half) return src[i];
    const int pair = i >> 1;
    const float u = src[i & ~1], v = src[i | 1];
    return (i & 1) ? v * cos_row[pair] + u * sin_row[pair] : u * cos_row[pair] - v * sin_row[pair];
}

template <typename T>
__global__ void __launch_bounds__(kLatThreads)
latent_prepare_kernel(const float* __restrict__ proj, long stride, int q_off, int q_rank, AnyVec q_gain, T* __restrict__ q_out,
                      int kv_off, int rank, int rot, AnyVec kv_gain, float eps, const float* __restrict__ cos_table,
                      const float* __restrict__ sin_table, int rot_half, int table_positions,
                      const int* __restrict__ positions, const int* __restrict__ row_entry,
                      const int* __restrict__ block_table, int max_blocks, int page_tokens, T* __restrict__ pool) {
    __shared__ float scratch[kLatWaves];
    const int row = blockIdx.x;
    const float* base = proj + static_cast<long>(row) * stride;
    if (q_off >= 0) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < q_rank; c += kLatThreads) ss = fmaf(base[q_off + c], base[q_off + c], ss);
        const float inv = 1.0f / sqrtf(block_sum<kLatThreads>(ss, scratch) / static_cast<float>(q_rank) + eps);
        for (int c = threadIdx.x; c < q_rank; c += kLatThreads)
            q_out[static_cast<long>(row) * q_rank + c] = from_float<T>(base[q_off + c] * inv * load_any(q_gain, c));
    }
    if (kv_off < 0) return;
    const int pos = positions[row];
    const int page = block_table[static_cast<long>(row_entry[row]) * max_blocks + pos / page_tokens];
    if (page < 0) return;                                       // no page mapped: nothing is written outside the pool
    T* to = pool + (static_cast<long>(page) * page_tokens + pos % page_tokens) * (rank + rot);
    const float* kv = base + kv_off;
    float ss = 0.f;
    for (int c = threadIdx.x; c < rank; c += kLatThreads) ss = fmaf(kv[c], kv[c], ss);
    const float inv = 1.0f / sqrtf(block_sum<kLatThreads>(ss, scratch) / static_cast<float>(rank) + eps);
    for (int c = threadIdx.x; c < rank; c += kLatThreads) to[c] = from_float<T>(kv[c] * inv * load_any(kv_gain, c));
    const int at = min(pos, table_positions - 1);
    const float* cos_row = cos_table ? cos_table + static_cast<long>(at) * rot_half : nullptr;
    const float* sin_row = cos_table ? sin_table + static_cast<long>(at) * rot_half : nullptr;
    for (int c = threadIdx.x; c < rot; c += kLatThreads)
        to[rank + c] = from_float<T>(rotated_adjacent(kv + rank, c, cos_row, sin_row, rot_half));
}

constexpr int kHpRows = 8;

// x: [rows] rows of x_row_stride floats or TX, head h's `inner` elements at h * x_head_stride; w: [heads][inner][outer];
// y: rows of y_row_stride, head h's results at h * y_head_stride.  A thread owns one output column for 8 rows.
template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(kLatThreads)
head_product_kernel(const TX* __restrict__ x, long x_row_stride, long x_head_stride, const TW* __restrict__ w,
                    TY* __restrict__ y, long y_row_stride, long y_head_stride, int rows, int inner, int outer, int tail,
                    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_half,
                    int table_positions, const int* __restrict__ positions) {
    extern __shared__ __align__(16) float hp_lds[];            // [kHpRows][inner + tail]
    const int head = blockIdx.y, row0 = blockIdx.x * kHpRows;
    const int here = min(kHpRows, rows - row0);
    const int width = inner + tail;
    for (int idx = threadIdx.x; idx < kHpRows * width; idx += kLatThreads) {
        const int r = idx / width, k = idx % width;
        hp_lds[idx] = r < here ? to_float(x[(row0 + r) * x_row_stride + head * x_head_stride + k]) : 0.f;
    }
    __syncthreads();
    const TW* wh = w + static_cast<long>(head) * inner * outer;
    for (int n = threadIdx.x; n < outer; n += kLatThreads) {
        float acc[kHpRows];
#pragma unroll
        for (int r = 0; r < kHpRows; ++r) acc[r] = 0.f;
        for (int k = 0; k < inner; ++k) {
            const float wv = to_float(wh[static_cast<long>(k) * outer + n]);
#pragma unroll
            for (int r = 0; r < kHpRows; ++r) acc[r] = fmaf(hp_lds[r * width + k], wv, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < kHpRows; ++r)
            if (r < here) y[(row0 + r) * y_row_stride + head * y_head_stride + n] = from_float<TY>(acc[r]);
    }
    for (int idx = threadIdx.x; idx < here * tail; idx += kLatThreads) {
        const int r = idx / tail, c = idx % tail;
        const int at = min(positions[row0 + r], table_positions - 1);
        const float* cos_row = cos_table ? cos_table + static_cast<long>(at) * rot_half : nullptr;
        const float* sin_row = cos_table ? sin_table + static_cast<long>(at) * rot_half : nullptr;
        y[(row0 + r) * y_row_stride + head * y_head_stride + outer + c] =
            from_float<TY>(rotated_adjacent(hp_lds + r * width + inner, c, cos_row, sin_row, rot_half));
    }
}

// One workgroup: one row, kHeads heads.  q: float [rows][heads][rank + rot]; out: float [rows][heads][rank].
// kChunks * 64 >= rank + rot.
template <typename T, int kChunks, int kHeads>
__global__ void __launch_bounds__(kLatThreads)
latent_attention_kernel(const float* __restrict__ q, float* __restrict__ out, const T* __restrict__ pool,
                        const int* __restrict__ positions, const int* __restrict__ row_entry,
                        const int* __restrict__ block_table, int max_blocks, int heads, int rank, int rot, int page_tokens,
                        float scale, int window) {
    extern __shared__ __align__(16) float la_lds[];            // [waves][kHeads][2] maxima and sums, then [waves][kHeads][rank]
    float* sm_ml = la_lds;
    float* sm_acc = la_lds + kLatWaves * kHeads * 2;
    const int row = blockIdx.x, head0 = blockIdx.y * kHeads;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int width = rank + rot;
    const int pos = positions[row];
    const int* table = block_table + static_cast<long>(row_entry[row]) * max_blocks;
    const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    float qv[kHeads][kChunks], acc[kHeads][kChunks], m[kHeads], l[kHeads];
#pragma unroll
    for (int h = 0; h < kHeads; ++h) {
        const bool live = head0 + h < heads;
        const float* qr = q + (static_cast<long>(row) * heads + (live ? head0 + h : head0)) * width;
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int d = lane + i * kWave;
            qv[h][i] = (live && d < width) ? qr[d] * scale : 0.f;
            acc[h][i] = 0.f;
        }
        m[h] = -INFINITY;
        l[h] = 0.f;
    }
    for (int j = first + wave; j <= pos; j += kLatWaves) {
        const int page = table[j / page_tokens];
        if (page < 0) {                                        // an unmapped block: poison the result instead of reading outside the pool
#pragma unroll
            for (int h = 0; h < kHeads; ++h) l[h] = __builtin_nanf("");
            continue;
        }
        const T* kr = pool + (static_cast<long>(page) * page_tokens + j % page_tokens) * width;
        float kv[kChunks];
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int d = lane + i * kWave;
            kv[i] = d < width ? to_float(kr[d]) : 0.f;
        }
#pragma unroll
        for (int h = 0; h < kHeads; ++h) {
            float partial = 0.f;
#pragma unroll
            for (int i = 0; i < kChunks; ++i) partial = fmaf(qv[h][i], kv[i], partial);
            const float s = wave_sum(partial);
            const float m_new = fmaxf(m[h], s);
            const float alpha = expf(m[h] - m_new), beta = expf(s - m_new);
            l[h] = l[h] * alpha + beta;
#pragma unroll
            for (int i = 0; i < kChunks; ++i) acc[h][i] = acc[h][i] * alpha + beta * kv[i];
            m[h] = m_new;
        }
    }
#pragma unroll
    for (int h = 0; h < kHeads; ++h) {
        if (lane == 0) {
            sm_ml[(wave * kHeads + h) * 2] = m[h];
            sm_ml[(wave * kHeads + h) * 2 + 1] = l[h];
        }
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int d = lane + i * kWave;
            if (d < rank) sm_acc[(static_cast<long>(wave) * kHeads + h) * rank + d] = acc[h][i];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < kHeads * rank; idx += kLatThreads) {
        const int h = idx / rank, d = idx % rank;
        if (head0 + h >= heads) continue;
        float top = -INFINITY;
#pragma unroll
        for (int w = 0; w < kLatWaves; ++w) top = fmaxf(top, sm_ml[(w * kHeads + h) * 2]);
        float denom = 0.f, num = 0.f;
#pragma unroll
        for (int w = 0; w < kLatWaves; ++w) {
            const float mw = sm_ml[(w * kHeads + h) * 2];
            const float wgt = mw == -INFINITY ? 0.f : expf(mw - top);         // a wave that saw no key adds nothing
            denom += sm_ml[(w * kHeads + h) * 2 + 1] * wgt;
            num += sm_acc[(static_cast<long>(w) * kHeads + h) * rank + d] * wgt;
        }
        out[(static_cast<long>(row) * heads + head0 + h) * rank + d] = num / denom;
    }
}

template <typename T, int kChunks, int kHeads>
static int launch_latent_attention(const float* q, float* out, const void* pool, const int* positions, const int* row_entry,
                                   const int* block_table, int max_blocks, int rows, int heads, int rank, int rot,
                                   int page_tokens, float scale, int window, hipStream_t stream) {
    const size_t shared = (static_cast<size_t>(kLatWaves) * kHeads * 2 + static_cast<size_t>(kLatWaves) * kHeads * rank) * sizeof(float);
    LEONE_REQUIRE(shared <= 64 * 1024, "latent_attention: %zu bytes of shared memory for a latent of %d", shared, rank);
    latent_attention_kernel<T, kChunks, kHeads><<<dim3(rows, ceil_div(heads, kHeads)), kLatThreads, shared, stream>>>(
        q, out, static_cast<const T*>(pool), positions, row_entry, block_table, max_blocks, heads, rank, rot, page_tokens, scale,
        window);
    LEONE_LAUNCH_CHECK("latent_attention");
    return 0;
}

template <typename T>
static int pick_latent_attention(const float* q, float* out, const void* pool, const int* positions, const int* row_entry,
                                 const int* block_table, int max_blocks, int rows, int heads, int rank, int rot,
                                 int page_tokens, float scale, int window, hipStream_t stream) {
    const int width = rank + rot;
#define LEONE_LATENT(C, H)                                                                                              \
    return launch_latent_attention<T, C, H>(q, out, pool, positions, row_entry, block_table, max_blocks, rows, heads, rank, \
                                            rot, page_tokens, scale, window, stream)
    if (width <= 128) LEONE_LATENT(2, 4);
    if (width <= 256) LEONE_LATENT(4, 4);
    if (width <= 640) LEONE_LATENT(10, 4);
    LEONE_LATENT(18, 2);
#undef LEONE_LATENT
}

}  // namespace leone

using namespace leone;

extern "C" int leone_latent_max_width() { return 18 * kWave; }

// proj float32 [rows, stride].  q_off >= 0: the query latent's q_rank columns from there, RMS-normed times q_gain, go
// to q_out [rows, q_rank] of `dtype`.  kv_off >= 0: the key/value latent's `rank` columns and the shared key part's
// `rot` columns from there go, normed (times kv_gain) and rotated (tables [table_positions, rot_half], pairs (2i, 2i+1)
// of the part's first 2 * rot_half elements), into pool [pages, page_tokens, rank + rot] of `dtype`.
extern "C" int leone_latent_prepare(const float* proj, long stride, int rows, int q_off, int q_rank, const void* q_gain,
                                    void* q_out, int kv_off, int rank, int rot, const void* kv_gain, int gain_dtype, float eps,
                                    const float* cos_table, const float* sin_table, int rot_half, int table_positions,
                                    const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                                    int page_tokens, void* pool, int dtype, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_prepare: unknown element type %d", dtype);
    LEONE_REQUIRE(gain_dtype == kF32 || gain_dtype == kBF16, "latent_prepare: unknown type of the gains");
    LEONE_REQUIRE(proj && rows > 0 && eps > 0.f && (q_off >= 0 || kv_off >= 0), "latent_prepare: null pointer, no rows or nothing to do");
    LEONE_REQUIRE(q_off < 0 || (q_gain && q_out && q_rank > 0 && stride >= q_off + q_rank), "latent_prepare: the query latent does not fit rows of %ld", stride);
    if (kv_off >= 0) {
        LEONE_REQUIRE(kv_gain && pool && positions && row_entry && block_table, "latent_prepare: a cache write needs a pool, positions, a row map and a block table");
        LEONE_REQUIRE(rank > 0 && rot >= 0 && stride >= kv_off + rank + rot && max_blocks > 0 && page_tokens > 0,
                      "latent_prepare: a latent of %d + %d does not fit rows of %ld", rank, rot, stride);
        LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr) && (!cos_table || (rot_half > 0 && 2 * rot_half <= rot && table_positions > 0)),
                      "latent_prepare: tables for %d pairs of a part of %d", rot_half, rot);
    }
    if (dtype == kF32)
        latent_prepare_kernel<float><<<rows, kLatThreads, 0, stream>>>(
            proj, stride, q_off, q_rank, AnyVec{q_gain, gain_dtype}, static_cast<float*>(q_out), kv_off, rank, rot,
            AnyVec{kv_gain, gain_dtype}, eps, cos_table, sin_table, cos_table ? rot_half : 0, table_positions, positions, row_entry,
            block_table, max_blocks, page_tokens, static_cast<float*>(pool));
    else
        latent_prepare_kernel<bf16_t><<<rows, kLatThreads, 0, stream>>>(
            proj, stride, q_off, q_rank, AnyVec{q_gain, gain_dtype}, static_cast<bf16_t*>(q_out), kv_off, rank, rot,
            AnyVec{kv_gain, gain_dtype}, eps, cos_table, sin_table, cos_table ? rot_half : 0, table_positions, positions, row_entry,
            block_table, max_blocks, page_tokens, static_cast<bf16_t*>(pool));
    LEONE_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// y[r, h, n] = sum_k x[r, h, k] w[h, k, n]; x float32, w of w_dtype, y of y_dtype (strides in elements).  tail > 0: the
// `tail` elements behind x's inner ones, rotated by the row's position, go behind y's outer ones.
extern "C" int leone_head_product(const float* x, long x_row_stride, long x_head_stride, const void* w, int w_dtype, void* y,
                                  int y_dtype, long y_row_stride, long y_head_stride, int rows, int heads, int inner, int outer,
                                  int tail, const float* cos_table, const float* sin_table, int rot_half, int table_positions,
                                  const int* positions, hipStream_t stream) {
    LEONE_REQUIRE((w_dtype == kF32 || w_dtype == kBF16) && (y_dtype == kF32 || y_dtype == kBF16), "head_product: unknown element type");
    LEONE_REQUIRE(x && w && y && rows > 0 && heads > 0 && heads <= 65535 && inner > 0 && outer > 0 && tail >= 0,
                  "head_product: null pointer or empty sizes");
    LEONE_REQUIRE(x_head_stride >= inner + tail && x_row_stride >= (heads - 1) * x_head_stride + inner + tail &&
                  y_head_stride >= outer + tail && y_row_stride >= (heads - 1) * y_head_stride + outer + tail,
                  "head_product: rows too short for %d heads of %d + %d in, %d + %d out", heads, inner, tail, outer, tail);
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr) && (!cos_table || (rot_half > 0 && 2 * rot_half <= tail && table_positions > 0 && positions)),
                  "head_product: tables for %d pairs of a tail of %d", rot_half, tail);
    const size_t shared = static_cast<size_t>(kHpRows) * (inner + tail) * sizeof(float);
    LEONE_REQUIRE(shared <= 64 * 1024, "head_product: %d + %d elements a head are too many", inner, tail);
    const dim3 grid(ceil_div(rows, kHpRows), heads);
    const int half = cos_table ? rot_half : 0;
#define LEONE_HP(TW, TY)                                                                                               \
    head_product_kernel<float, TW, TY><<<grid, kLatThreads, shared, stream>>>(                                         \
        x, x_row_stride, x_head_stride, static_cast<const TW*>(w), static_cast<TY*>(y), y_row_stride, y_head_stride, rows, inner, \
        outer, tail, cos_table, sin_table, half, table_positions, positions)
    if (w_dtype == kF32) {
        if (y_dtype == kF32) LEONE_HP(float, float);
        else LEONE_HP(float, bf16_t);
    } else {
        if (y_dtype == kF32) LEONE_HP(bf16_t, float);
        else LEONE_HP(bf16_t, bf16_t);
    }
#undef LEONE_HP
    LEONE_LAUNCH_CHECK("head_product");
    return 0;
}

// q float32 [rows, heads, rank + rot] (up-projection already taken to the query's side, shared key part rotated);
// out float32 [rows, heads, rank]: sum_j p_j c_j over the keys j of the row's request with pos - window < j <= pos
// (window 0: all j <= pos); pool [pages, page_tokens, rank + rot] of `dtype`.
extern "C" int leone_latent_attention(const float* q, float* out, const void* pool, int dtype, const int* positions,
                                      const int* row_entry, const int* block_table, int max_blocks, int rows, int heads,
                                      int rank, int rot, int page_tokens, float scale, int window, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_attention: unknown element type %d", dtype);
    LEONE_REQUIRE(q && out && pool && positions && row_entry && block_table, "latent_attention: null pointer");
    LEONE_REQUIRE(rows > 0 && heads > 0 && heads <= 65535 * 2 && rank > 0 && rot >= 0 && rank + rot <= leone_latent_max_width(),
                  "latent_attention: rows %d, %d heads, a latent of %d + %d (at most %d)", rows, heads, rank, rot, leone_latent_max_width());
    LEONE_REQUIRE(page_tokens > 0 && max_blocks > 0 && window >= 0, "latent_attention: page_tokens %d, max_blocks %d, window %d",
                  page_tokens, max_blocks, window);
    if (dtype == kF32)
        return pick_latent_attention<float>(q, out, pool, positions, row_entry, block_table, max_blocks, rows, heads, rank, rot,
                                            page_tokens, scale, window, stream);
    return pick_latent_attention<bf16_t>(q, out, pool, positions, row_entry, block_table, max_blocks, rows, heads, rank, rot,
                                         page_tokens, scale, window, stream);
}
