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
//   latent_attention_cores  the same on the matrix cores (bfloat16): a workgroup takes 16 (row, head) pairs, its four
//                     waves take 32-key tiles in turn; S^T = K Q^T and O^T += V^T P^T with v_mfma_f32_16x16x32_bf16,
//                     both operands straight from the cache in 16-byte runs.
//
// The cache of one layer holds a token's vector twice, each time in the order one of the two products reads it:
// as a key, [page][element / 8][token in page][8] over the rank + rot elements (filled up to a multiple of 8), and
// as a value, [page][token in page / 8][element][8] over the first `rank` elements.  Norms, angles, scores, softmax
// and all sums are float.
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
                      const int* __restrict__ block_table, int max_blocks, int page_tokens, T* __restrict__ k_pool,
                      T* __restrict__ v_pool) {
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
    const int tok = pos % page_tokens, runs = (rank + rot + 7) / 8;
    T* as_key = k_pool + static_cast<long>(page) * runs * page_tokens * 8;
    T* as_value = v_pool + (static_cast<long>(page) * (page_tokens / 8) + tok / 8) * rank * 8 + tok % 8;
    auto put = [&](int e, T v) { as_key[(static_cast<long>(e / 8) * page_tokens + tok) * 8 + e % 8] = v; };
    const float* kv = base + kv_off;
    float ss = 0.f;
    for (int c = threadIdx.x; c < rank; c += kLatThreads) ss = fmaf(kv[c], kv[c], ss);
    const float inv = 1.0f / sqrtf(block_sum<kLatThreads>(ss, scratch) / static_cast<float>(rank) + eps);
    for (int c = threadIdx.x; c < rank; c += kLatThreads) {
        const T v = from_float<T>(kv[c] * inv * load_any(kv_gain, c));
        put(c, v);
        as_value[static_cast<long>(c) * 8] = v;
    }
    const int at = min(pos, table_positions - 1);
    const float* cos_row = cos_table ? cos_table + static_cast<long>(at) * rot_half : nullptr;
    const float* sin_row = cos_table ? sin_table + static_cast<long>(at) * rot_half : nullptr;
    for (int c = threadIdx.x; c < rot; c += kLatThreads)
        put(rank + c, from_float<T>(rotated_adjacent(kv + rank, c, cos_row, sin_row, rot_half)));
    for (int c = rank + rot + threadIdx.x; c < runs * 8; c += kLatThreads) put(c, from_float<T>(0.f));
}

constexpr int kHpRows = 8;

// Eight neighbouring weights of one inner element as floats: one 16- or 32-byte read where `runs` says the rows of the
// matrix allow it, element by element (zeros beyond `valid`) otherwise.
template <typename TW>
__device__ inline void load_weights8(const TW* p, int valid, bool runs, float* to) {
    if (runs && valid >= 8) {
        if constexpr (sizeof(TW) == 2) {
            const uint4 raw = *reinterpret_cast<const uint4*>(p);
            const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                to[2 * i] = __uint_as_float(w[i] << 16);
                to[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
            }
        } else {
            const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
            to[0] = a.x, to[1] = a.y, to[2] = a.z, to[3] = a.w, to[4] = b.x, to[5] = b.y, to[6] = b.z, to[7] = b.w;
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) to[j] = j < valid ? to_float(p[j]) : 0.f;
}

// x: [rows] rows of x_row_stride floats or TX, head h's `inner` elements at h * x_head_stride; w: [heads][inner][outer]
// (null: only the tail is handed on); y: rows of y_row_stride, head h's results at h * y_head_stride.  A workgroup takes
// 8 rows, one head and 8 * kGroups columns.  A thread owns 8 neighbouring columns and every (256 / kGroups)th inner
// element, so that a wave reads whole runs of the matrix and a thread's reads are on their way together: the first
// four are asked for before the rows are staged (they do not depend on them; a step of few rows is a chain of a few
// trips to memory and nothing else).  The partial sums of a result are added over a wave's lanes by shuffles and over
// the waves, in their order, in shared memory.  Deep products (W_uv on the weighted sums) take kGroups = 2, flat ones 8.
template <typename TX, typename TW, typename TY, int kGroups>
__global__ void __launch_bounds__(kLatThreads)
head_product_kernel(const TX* __restrict__ x, long x_row_stride, long x_head_stride, const TW* __restrict__ w,
                    TY* __restrict__ y, long y_row_stride, long y_head_stride, int rows, int inner, int outer, int tail,
                    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_half,
                    int table_positions, const int* __restrict__ positions, int runs) {
    constexpr int kCols = 8 * kGroups, kSlices = kLatThreads / kGroups, kAhead = 4;
    extern __shared__ __align__(16) float hp_lds[];            // [kHpRows][inner + tail], then [waves][kHpRows][kCols]
    const int head = blockIdx.y, row0 = blockIdx.x * kHpRows;
    const int here = min(kHpRows, rows - row0);
    const int width = inner + tail;
    float* partial = hp_lds + kHpRows * width;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int group = threadIdx.x % kGroups, slice = threadIdx.x / kGroups;
    const int n0 = blockIdx.z * kCols + group * 8;
    const int valid = w ? min(8, outer - n0) : 0;
    const TW* wh = w ? w + static_cast<long>(head) * inner * outer + n0 : nullptr;
    float ahead[kAhead][8];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
        const int k = slice + i * kSlices;
        if (valid > 0 && k < inner) {
            load_weights8(wh + static_cast<long>(k) * outer, valid, runs != 0, ahead[i]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) ahead[i][j] = 0.f;
        }
    }
    // eight elements a thread are asked for before the first is put away: a read a trip would be a trip to memory each
    constexpr int kStage = 8;
    for (int base = threadIdx.x; base < kHpRows * width; base += kLatThreads * kStage) {
        float staged[kStage];
#pragma unroll
        for (int i = 0; i < kStage; ++i) {
            const int idx = base + i * kLatThreads;
            const int r = idx / width, k = idx % width;
            staged[i] = (idx < kHpRows * width && r < here) ? to_float(x[(row0 + r) * x_row_stride + head * x_head_stride + k]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < kStage; ++i)
            if (base + i * kLatThreads < kHpRows * width) hp_lds[base + i * kLatThreads] = staged[i];
    }
    __syncthreads();
    if (w) {
        float acc[kHpRows][8];
#pragma unroll
        for (int r = 0; r < kHpRows; ++r)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[r][j] = 0.f;
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const int k = min(slice + i * kSlices, inner - 1);     // beyond the inner size the weights are zeros
#pragma unroll
            for (int r = 0; r < kHpRows; ++r) {
                const float xv = hp_lds[r * width + k];
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[r][j] = fmaf(xv, ahead[i][j], acc[r][j]);
            }
        }
        if (valid > 0) {
#pragma unroll 4
            for (int k = slice + kAhead * kSlices; k < inner; k += kSlices) {
                float wv[8];
                load_weights8(wh + static_cast<long>(k) * outer, valid, runs != 0, wv);
#pragma unroll
                for (int r = 0; r < kHpRows; ++r) {
                    const float xv = hp_lds[r * width + k];
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[r][j] = fmaf(xv, wv[j], acc[r][j]);
                }
            }
        }
        // one step of the sum over lanes for all 64 sums before the next: the exchanges of a step do not wait for each other
#pragma unroll
        for (int off = kGroups; off < kWave; off <<= 1) {
            float other[kHpRows][8];
#pragma unroll
            for (int r = 0; r < kHpRows; ++r)
#pragma unroll
                for (int j = 0; j < 8; ++j) other[r][j] = __shfl_xor(acc[r][j], off, kWave);
#pragma unroll
            for (int r = 0; r < kHpRows; ++r)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[r][j] += other[r][j];
        }
        if (lane < kGroups) {
#pragma unroll
            for (int r = 0; r < kHpRows; ++r)
#pragma unroll
                for (int j = 0; j < 8; ++j) partial[(wave * kHpRows + r) * kCols + group * 8 + j] = acc[r][j];
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < here * kCols; idx += kLatThreads) {
            const int r = idx / kCols, col = idx % kCols;
            if (blockIdx.z * kCols + col >= outer) continue;
            float sum = 0.f;
#pragma unroll
            for (int p = 0; p < kLatWaves; ++p) sum += partial[(p * kHpRows + r) * kCols + col];
            y[(row0 + r) * y_row_stride + head * y_head_stride + blockIdx.z * kCols + col] = from_float<TY>(sum);
        }
    }
    if (blockIdx.z != 0) return;
    for (int idx = threadIdx.x; idx < here * tail; idx += kLatThreads) {
        const int r = idx / tail, c = idx % tail;
        const int at = cos_table ? min(positions[row0 + r], table_positions - 1) : 0;
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
        const T* kr = pool + (static_cast<long>(page) * ((width + 7) / 8) * page_tokens + j % page_tokens) * 8;
        float kv[kChunks];
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int d = lane + i * kWave;
            kv[i] = d < width ? to_float(kr[static_cast<long>(d / 8) * page_tokens * 8 + d % 8]) : 0.f;
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


// ---- the same on the matrix cores ------------------------------------------------------------------------------
//
// Operand layouts of v_mfma_f32_16x16x32_bf16 (lane l, c = l % 16, g = l / 16): A: row c, k-slots 8g .. 8g+7; B: column
// c, k-slots 8g .. 8g+7; C/D: column c, rows 4g .. 4g+3.  A workgroup's 16 columns are 16 consecutive (row, head)
// pairs of the step; they may belong to several requests (single decoded tokens of a model with few heads), which
// are then taken one after the other with the other requests' columns masked.  For S^T the two 16-key halves of a
// 32-key tile are laid out so that lane (g, c) ends up with the scores of keys 8g .. 8g+7 of the tile: the k-slots it
// supplies as P^T to the second product.  Each wave keeps a running maximum and sum per column; the waves' partial
// results are merged in shared memory in the waves' order.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 lat_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float lat_floatx4;

constexpr int kCoreTile = 32;        // keys of a tile

__device__ inline lat_bf16x8 lat_load8(const bf16_t* p) {
    return __builtin_bit_cast(lat_bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline lat_bf16x8 lat_zero8() {
    return __builtin_bit_cast(lat_bf16x8, uint4{0u, 0u, 0u, 0u});
}

// kSteps * 32 >= rank + rot, kDT * 16 >= rank; `steps` and `dts` are the counts in use.
template <int kSteps, int kDT>
__global__ void __launch_bounds__(kLatThreads)
latent_attention_cores_kernel(const bf16_t* __restrict__ q, float* __restrict__ out, const bf16_t* __restrict__ k_pool,
                              const bf16_t* __restrict__ v_pool, const int* __restrict__ positions,
                              const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
                              int total, int heads, int rank, int width, int page_tokens, float to_log2, int window,
                              int splits, float* __restrict__ part_acc, float* __restrict__ part_ml) {
    extern __shared__ __align__(16) float lc_lds[];               // [16][rank + 4] sums, then [waves][16] maxima, [waves][16] sums
    const int pitch = rank + 4;
    float* sm_acc = lc_lds;
    float* sm_m = lc_lds + 16 * pitch;
    float* sm_l = sm_m + kLatWaves * 16;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int c = lane % 16, g = lane / 16;
    const int steps = width / 32, dts = rank / 16;
    // (Numbering the workgroups so that each of the chip's dies gets a run of neighbouring tiles was measured: a prompt's
    // attention took a sixth longer, 2.0 against 1.7 ms for six layers of 2,048 rows.)
    const int tile = blockIdx.x;
    const long pair = static_cast<long>(tile) * 16 + c;           // this lane's column: (row, head) pair of the step
    const bool valid = pair < total;
    const int row = valid ? static_cast<int>(pair / heads) : 0;
    const int pos = valid ? positions[row] : -1;
    const int entry = valid ? row_entry[row] : -1;
    const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    lat_bf16x8 qreg[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
        qreg[s] = (valid && s < steps) ? lat_load8(q + pair * width + 32 * s + 8 * g) : lat_zero8();
    lat_floatx4 acc[kDT];
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) acc[dt] = lat_floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    bool unmapped = false;
    const long key_page = static_cast<long>(width / 8) * page_tokens * 8;      // elements of a page, as keys
    const long value_page = static_cast<long>(page_tokens / 8) * rank * 8;      // and as values

    int at = 0;                                                   // first column of the request that is walked next
    while (at < 16) {
        const int walked = __shfl(entry, at, kWave);              // lanes 0..15 are the columns with g = 0
        if (walked < 0) break;                                    // columns beyond the step's last pair
        const bool mine = valid && entry == walked;
        at += __popcll(__ballot(mine) & 0xffffull);               // a request's columns stand side by side
        int hi = mine ? pos : -1, lo = mine ? first : 0x7fffffff;
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            hi = max(hi, __shfl_xor(hi, off, kWave));
            lo = min(lo, __shfl_xor(lo, off, kWave));
        }
        const int* table = block_table + static_cast<long>(walked) * max_blocks;
        // the tiles go round the waves of all the workgroups that share these columns (blockIdx.y: one of `splits`)
        for (int t = lo / kCoreTile + blockIdx.y * kLatWaves + wave; t <= hi / kCoreTile; t += kLatWaves * splits) {
            const int key0 = t * kCoreTile;
            const int page = table[key0 / page_tokens];
            const int tok0 = key0 % page_tokens;
            if (page < 0) {                                       // a key in reach without a page: say so in the result
                unmapped = true;
                continue;
            }
            const bool inner = key0 >= lo && key0 + kCoreTile - 1 <= hi;     // every key of the tile belongs to the request's range
            // ---- S^T = K Q^T for the two 16-key halves ----
            const int ka = 8 * (c >> 2) + (c & 3);                // this lane's key of the first half; the second's is 4 further
            const bf16_t* kp = k_pool + page * key_page + static_cast<long>(tok0 + ka) * 8;
            // All of a tile's keys are asked for before the first product waits for any (no branch stands between the
            // loads): steps beyond the latent's width read a step that exists and meet zero queries.
            lat_bf16x8 xa[kSteps], xb[kSteps];
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                const bf16_t* from = kp + static_cast<long>(4 * min(s, steps - 1) + g) * page_tokens * 8;
                xa[s] = lat_load8(from);
                xb[s] = lat_load8(from + 32);
            }
            if (!inner) {                                         // what lies outside the range may hold anything
                const bool drop_a = key0 + ka < lo || key0 + ka > hi, drop_b = key0 + ka + 4 < lo || key0 + ka + 4 > hi;
#pragma unroll
                for (int s = 0; s < kSteps; ++s) {
                    if (drop_a) xa[s] = lat_zero8();
                    if (drop_b) xb[s] = lat_zero8();
                }
            }
            lat_floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[s], qreg[s], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xb[s], qreg[s], sb, 0, 0, 0);
            }
            // The tile's values are asked for now, all of them, into the registers the keys have left: they arrive while
            // the softmax is worked out.  Runs beyond the latent read one that exists, into sums that nobody reads.
            const int run0 = key0 + 8 * g;
            const bf16_t* vp = v_pool + page * value_page + (static_cast<long>((tok0 + 8 * g) / 8) * rank + c) * 8;
            uint4 raw[kDT];
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt)
                raw[dt] = *reinterpret_cast<const uint4*>(vp + static_cast<long>(16 * min(dt, dts - 1)) * 8);
            if (!inner) {                                         // slots outside the range may hold anything, even NaN
                unsigned keep[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e0 = run0 + 2 * i, e1 = e0 + 1;
                    keep[i] = ((e0 >= lo && e0 <= hi) ? 0x0000ffffu : 0u) | ((e1 >= lo && e1 <= hi) ? 0xffff0000u : 0u);
                }
#pragma unroll
                for (int dt = 0; dt < kDT; ++dt) {
                    raw[dt].x &= keep[0];
                    raw[dt].y &= keep[1];
                    raw[dt].z &= keep[2];
                    raw[dt].w &= keep[3];
                }
            }
            // lane (g, c) holds, for column c, the scores of keys key0 + 8g + j, j = 0 .. 7
            float sc[8], tile_max = -INFINITY;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int key = run0 + j;
                const float score = j < 4 ? sa[j & 3] : sb[j & 3];
                sc[j] = (mine && key >= first && key <= pos) ? score * to_log2 : -INFINITY;
                tile_max = fmaxf(tile_max, sc[j]);
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, kWave));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
            const float m_new = fmaxf(m_run, tile_max);
            const bool none = m_new == -INFINITY;                 // a column that has seen no key yet
            const float alpha = none ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
            float psum = 0.f;
            lat_bf16x8 pt;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                pt[j] = static_cast<__bf16>(none ? 0.f : __builtin_amdgcn_exp2f(sc[j] - m_new));
                psum += static_cast<float>(pt[j]);
            }
            psum += __shfl_xor(psum, 16, kWave);
            psum += __shfl_xor(psum, 32, kWave);
            l_run = l_run * alpha + psum;
            m_run = m_new;
            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[dt][r] *= alpha;
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lat_bf16x8, raw[dt]), pt, acc[dt], 0, 0, 0);
            }
        }
    }

    // ---- merge the four waves, in their order ----
    if (__any(unmapped)) l_run = __builtin_nanf("");
    if (g == 0) {
        sm_m[wave * 16 + c] = m_run;
        sm_l[wave * 16 + c] = l_run;
    }
    __syncthreads();
    float top = -INFINITY;
#pragma unroll
    for (int w = 0; w < kLatWaves; ++w) top = fmaxf(top, sm_m[w * 16 + c]);
    float denom = 0.f;
#pragma unroll
    for (int w = 0; w < kLatWaves; ++w) {
        const float mw = sm_m[w * 16 + c];
        denom += sm_l[w * 16 + c] * (mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - top));
    }
    // one workgroup a tile of columns: the result itself; several: sums against the workgroup's maximum, for the merge
    const float weight = (m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - top)) / (splits == 1 ? denom : 1.f);
    for (int w = 0; w < kLatWaves; ++w) {
        if (wave == w) {
            // what the waves before left is read in one go, then added to and written in one go
            float4 sum[kDT];
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt) {
                const float4* from = reinterpret_cast<const float4*>(sm_acc + c * pitch + 16 * min(dt, dts - 1) + 4 * g);
                sum[dt] = w == 0 ? float4{0.f, 0.f, 0.f, 0.f} : *from;
            }
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt) {
                if (dt < dts) {
                    sum[dt].x += acc[dt][0] * weight;
                    sum[dt].y += acc[dt][1] * weight;
                    sum[dt].z += acc[dt][2] * weight;
                    sum[dt].w += acc[dt][3] * weight;
                    *reinterpret_cast<float4*>(sm_acc + c * pitch + 16 * dt + 4 * g) = sum[dt];
                }
            }
        }
        __syncthreads();
    }
    const long pair0 = static_cast<long>(tile) * 16;
    if (splits == 1) {
        for (int i = threadIdx.x; i < 16 * rank; i += kLatThreads) {
            const int col = i / rank, e = i % rank;
            if (pair0 + col < total) out[(pair0 + col) * rank + e] = sm_acc[col * pitch + e];
        }
        return;
    }
    const long mine_at = (static_cast<long>(tile) * splits + blockIdx.y) * 16;
    for (int i = threadIdx.x; i < 16 * rank; i += kLatThreads) {
        const int col = i / rank, e = i % rank;
        part_acc[(mine_at + col) * rank + e] = sm_acc[col * pitch + e];
    }
    if (wave == 0 && g == 0) {
        part_ml[(mine_at + c) * 2] = top;
        part_ml[(mine_at + c) * 2 + 1] = denom;
    }
}

// The partial results of the workgroups that shared a tile of columns, in their order; one workgroup a column.
__global__ void __launch_bounds__(kLatThreads)
latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, float* __restrict__ out, int total,
                    int rank, int splits) {
    const int col = blockIdx.y;
    const long pair = static_cast<long>(blockIdx.x) * 16 + col;
    if (pair >= total) return;
    const long first = static_cast<long>(blockIdx.x) * splits * 16 + col;       // + 16 a split
    // every split's figures are asked for at once (a loop of as many turns as there are splits would wait for each)
    constexpr int kMost = 16;
    float m[kMost], f[kMost], l[kMost];
#pragma unroll
    for (int sp = 0; sp < kMost; ++sp) {
        const bool there = sp < splits;
        m[sp] = there ? part_ml[(first + 16L * sp) * 2] : -INFINITY;
        l[sp] = there ? part_ml[(first + 16L * sp) * 2 + 1] : 0.f;
    }
    float top = -INFINITY;
#pragma unroll
    for (int sp = 0; sp < kMost; ++sp) top = fmaxf(top, m[sp]);
    float den = 0.f;
#pragma unroll
    for (int sp = 0; sp < kMost; ++sp) {
        f[sp] = m[sp] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[sp] - top);
        if (sp < splits) den += l[sp] * f[sp];            // NaN: a key in reach had no page
    }
    for (int e = threadIdx.x; e < rank; e += kLatThreads) {
        float part[kMost];
#pragma unroll
        for (int sp = 0; sp < kMost; ++sp) part[sp] = sp < splits ? part_acc[(first + 16L * sp) * rank + e] : 0.f;
        float num = 0.f;
#pragma unroll
        for (int sp = 0; sp < kMost; ++sp) num += part[sp] * f[sp];
        out[pair * rank + e] = num / den;
    }
}

template <int kSteps, int kDT>
static int launch_latent_cores(const void* q, float* out, const void* k_pool, const void* v_pool, const int* positions,
                               const int* row_entry, const int* block_table, int max_blocks, int rows, int heads, int rank,
                               int rot, int page_tokens, float scale, int window, int splits, float* part_acc, float* part_ml,
                               hipStream_t stream) {
    const long total = static_cast<long>(rows) * heads;
    const size_t shared = (static_cast<size_t>(16) * (rank + 4) + 2 * kLatWaves * 16) * sizeof(float);
    LEONE_REQUIRE(shared <= 64 * 1024 && (total + 15) / 16 <= 0x7fffffffL, "latent_attention_cores: %ld pairs, a latent of %d", total, rank);
    const unsigned tiles = static_cast<unsigned>((total + 15) / 16);
    latent_attention_cores_kernel<kSteps, kDT><<<dim3(tiles, splits), kLatThreads, shared, stream>>>(
        static_cast<const bf16_t*>(q), out, static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool), positions,
        row_entry, block_table, max_blocks, static_cast<int>(total), heads, rank, rank + rot, page_tokens,
        scale * 1.4426950408889634f, window, splits, part_acc, part_ml);
    LEONE_LAUNCH_CHECK("latent_attention_cores");
    if (splits > 1) {
        latent_merge_kernel<<<dim3(tiles, 16), kLatThreads, 0, stream>>>(part_acc, part_ml, out, static_cast<int>(total), rank, splits);
        LEONE_LAUNCH_CHECK("latent_merge");
    }
    return 0;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_latent_max_width() { return 18 * kWave; }

// proj float32 [rows, stride].  q_off >= 0: the query latent's q_rank columns from there, RMS-normed times q_gain, go
// to q_out [rows, q_rank] of `dtype`.  kv_off >= 0: the key/value latent's `rank` columns and the shared key part's
// `rot` columns from there go, normed (times kv_gain) and rotated (tables [table_positions, rot_half], pairs (2i, 2i+1)
// of the part's first 2 * rot_half elements), into the two pools of `dtype` (the layouts at the top).
extern "C" int leone_latent_prepare(const float* proj, long stride, int rows, int q_off, int q_rank, const void* q_gain,
                                    void* q_out, int kv_off, int rank, int rot, const void* kv_gain, int gain_dtype, float eps,
                                    const float* cos_table, const float* sin_table, int rot_half, int table_positions,
                                    const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                                    int page_tokens, void* k_pool, void* v_pool, int dtype, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_prepare: unknown element type %d", dtype);
    LEONE_REQUIRE(gain_dtype == kF32 || gain_dtype == kBF16, "latent_prepare: unknown type of the gains");
    LEONE_REQUIRE(proj && rows > 0 && eps > 0.f && (q_off >= 0 || kv_off >= 0), "latent_prepare: null pointer, no rows or nothing to do");
    LEONE_REQUIRE(q_off < 0 || (q_gain && q_out && q_rank > 0 && stride >= q_off + q_rank), "latent_prepare: the query latent does not fit rows of %ld", stride);
    if (kv_off >= 0) {
        LEONE_REQUIRE(kv_gain && k_pool && v_pool && positions && row_entry && block_table, "latent_prepare: a cache write needs both pools, positions, a row map and a block table");
        LEONE_REQUIRE(rank > 0 && rot >= 0 && stride >= kv_off + rank + rot && max_blocks > 0 && page_tokens > 0 && page_tokens % 8 == 0,
                      "latent_prepare: a latent of %d + %d does not fit rows of %ld", rank, rot, stride);
        LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr) && (!cos_table || (rot_half > 0 && 2 * rot_half <= rot && table_positions > 0)),
                      "latent_prepare: tables for %d pairs of a part of %d", rot_half, rot);
    }
    if (dtype == kF32)
        latent_prepare_kernel<float><<<rows, kLatThreads, 0, stream>>>(
            proj, stride, q_off, q_rank, AnyVec{q_gain, gain_dtype}, static_cast<float*>(q_out), kv_off, rank, rot,
            AnyVec{kv_gain, gain_dtype}, eps, cos_table, sin_table, cos_table ? rot_half : 0, table_positions, positions, row_entry,
            block_table, max_blocks, page_tokens, static_cast<float*>(k_pool), static_cast<float*>(v_pool));
    else
        latent_prepare_kernel<bf16_t><<<rows, kLatThreads, 0, stream>>>(
            proj, stride, q_off, q_rank, AnyVec{q_gain, gain_dtype}, static_cast<bf16_t*>(q_out), kv_off, rank, rot,
            AnyVec{kv_gain, gain_dtype}, eps, cos_table, sin_table, cos_table ? rot_half : 0, table_positions, positions, row_entry,
            block_table, max_blocks, page_tokens, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool));
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
    LEONE_REQUIRE(x && y && rows > 0 && heads > 0 && heads <= 65535 && inner > 0 && outer > 0 && tail >= 0 && (w || tail > 0),
                  "head_product: null pointer or empty sizes");
    LEONE_REQUIRE(x_head_stride >= inner + tail && x_row_stride >= (heads - 1) * x_head_stride + inner + tail &&
                  y_head_stride >= outer + tail && y_row_stride >= (heads - 1) * y_head_stride + outer + tail,
                  "head_product: rows too short for %d heads of %d + %d in, %d + %d out", heads, inner, tail, outer, tail);
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr) && (!cos_table || (rot_half > 0 && 2 * rot_half <= tail && table_positions > 0 && positions)),
                  "head_product: tables for %d pairs of a tail of %d", rot_half, tail);
    const int groups = inner >= 256 ? 2 : 8;            // deep products: fewer columns and more of the inner size a workgroup
    const size_t shared = (static_cast<size_t>(kHpRows) * (inner + tail) + kLatWaves * kHpRows * 8 * groups) * sizeof(float);
    LEONE_REQUIRE(shared <= 64 * 1024 && ceil_div(outer, 8 * groups) <= 65535, "head_product: %d + %d elements a head are too many", inner, tail);
    const dim3 grid(ceil_div(rows, kHpRows), heads, w ? ceil_div(outer, 8 * groups) : 1);
    const int half = cos_table ? rot_half : 0;
    // rows of the matrices that begin on 16-byte borders (32 for float) are read in whole runs
    const int runs = outer % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 32 == 0;
#define LEONE_HP_G(TW, TY, G)                                                                                          \
    head_product_kernel<float, TW, TY, G><<<grid, kLatThreads, shared, stream>>>(                                      \
        x, x_row_stride, x_head_stride, static_cast<const TW*>(w), static_cast<TY*>(y), y_row_stride, y_head_stride, rows, inner, \
        outer, tail, cos_table, sin_table, half, table_positions, positions, runs)
#define LEONE_HP(TW, TY)                                                                                               \
    do {                                                                                                               \
        if (groups == 2) LEONE_HP_G(TW, TY, 2);                                                                        \
        else LEONE_HP_G(TW, TY, 8);                                                                                    \
    } while (0)
    if (w_dtype == kF32) {
        if (y_dtype == kF32) LEONE_HP(float, float);
        else LEONE_HP(float, bf16_t);
    } else {
        if (y_dtype == kF32) LEONE_HP(bf16_t, float);
        else LEONE_HP(bf16_t, bf16_t);
    }
#undef LEONE_HP
#undef LEONE_HP_G
    LEONE_LAUNCH_CHECK("head_product");
    return 0;
}

// q float32 [rows, heads, rank + rot] (up-projection already taken to the query's side, shared key part rotated);
// out float32 [rows, heads, rank]: sum_j p_j c_j over the keys j of the row's request with pos - window < j <= pos
// (window 0: all j <= pos); pool: the keys' form of the cache, of `dtype`.
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

// The same on the matrix cores: bfloat16 queries [rows, heads, rank + rot] and both forms of the cache; rank + rot a
// multiple of 32 up to leone_latent_cores_max_width(), rank a multiple of 16, pages of a multiple of 32 tokens.  splits
// > 1: so many workgroups share the keys of every 16 (row, head) pairs; their partial results go through part_acc float32
// [tiles of 16 pairs, splits, 16, rank] and part_ml [tiles, splits, 16, 2] and a merge.
extern "C" int leone_latent_cores_max_width() { return 576; }

extern "C" int leone_latent_attention_cores(const void* q, float* out, const void* k_pool, const void* v_pool, const int* positions,
                                            const int* row_entry, const int* block_table, int max_blocks, int rows, int heads,
                                            int rank, int rot, int page_tokens, float scale, int window, int splits, float* part_acc,
                                            float* part_ml, hipStream_t stream) {
    LEONE_REQUIRE(q && out && k_pool && v_pool && positions && row_entry && block_table, "latent_attention_cores: null pointer");
    LEONE_REQUIRE(splits >= 1 && splits <= 16 && (splits == 1 || (part_acc && part_ml)), "latent_attention_cores: %d workgroups a tile of columns need a workspace", splits);
    LEONE_REQUIRE(rows > 0 && heads > 0 && rank > 0 && rot >= 0 && (rank + rot) % 32 == 0 && rank % 16 == 0 &&
                  rank + rot <= leone_latent_cores_max_width(),
                  "latent_attention_cores: rows %d, %d heads, a latent of %d + %d", rows, heads, rank, rot);
    LEONE_REQUIRE(page_tokens > 0 && page_tokens % 32 == 0 && max_blocks > 0 && window >= 0 && scale > 0.f,
                  "latent_attention_cores: page_tokens %d, max_blocks %d, window %d", page_tokens, max_blocks, window);
    LEONE_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k_pool) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(v_pool) % 16 == 0, "latent_attention_cores: operands must lie on 16-byte borders");
    const int width = rank + rot;
#define LEONE_LATENT_CORES(S, D)                                                                                          \
    return launch_latent_cores<S, D>(q, out, k_pool, v_pool, positions, row_entry, block_table, max_blocks, rows, heads, rank, \
                                     rot, page_tokens, scale, window, splits, part_acc, part_ml, stream)
    if (width <= 128) LEONE_LATENT_CORES(4, 8);
    if (width <= 256) LEONE_LATENT_CORES(8, 16);
    LEONE_LATENT_CORES(18, 32);
#undef LEONE_LATENT_CORES
}
