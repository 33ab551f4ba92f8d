// C entry points of the gfx950 kernel library.  Every function returns 0 on
// success; otherwise leone_last_error() describes what was refused.  Pointers
// are device pointers unless said otherwise; `dtype` arguments are 0 for
// float and 1 for bfloat16.  All work is queued on `stream`.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

const char* leone_last_error();
int leone_library_version();

// out[r, :] = table[tokens[r], :] widened to float, times scale (1 for none).
int leone_embed(const void* table, int dtype, const int* tokens, float* out, int rows, int hidden, int vocab,
                float scale, hipStream_t stream);

// x = cap * tanh(x / cap) in place, n floats.
int leone_soft_cap(float* x, long n, float cap, hipStream_t stream);

// x += delta (delta may be null); y = rmsnorm(x) * gain.  With `rows` given,
// y[r] is computed from row rows[r] and x is not written.  delta may be delta_planes (1..16) planes,
// delta_plane elements apart, whose sum in order is what is added.  With squares_out (float32 [n_rows,
// ceil(hidden / 16)]) the norm is only prepared for leone_gemm_fused_bf16's in_mode 2: y = x * gain, not yet
// scaled, and the row's sum of squares in squares_out[r][0], zeros behind it.
int leone_add_rmsnorm(float* x, const void* delta, int delta_dtype, int delta_planes, long delta_plane, const void* gain,
                      int gain_dtype, float eps, void* y, int y_dtype, const int* rows, int n_rows, int hidden,
                      float* squares_out, hipStream_t stream);

// out[r, c] = silu(gate) * up, where gate_up[r] holds, in every block of 16 columns, 8 gate values
// and then the 8 up values that belong to them; ffn is a multiple of 8.
int leone_swiglu(const void* gate_up, void* out, int dtype, int rows, int ffn, hipStream_t stream);

// cos/sin[pos, i] of pos * theta^(-2i/rotary_dim), for pos < positions.
int leone_rope_table(float* cos_out, float* sin_out, double theta, int rotary_dim, int positions,
                     hipStream_t stream);

// Per-head RMSNorm (gains may be null), rotation (tables may be null), q to q_out, k and v into the paged
// cache.  The input is of the outputs' type, or float32 in qkv_planes planes (qkv_plane elements apart) that are
// added up in order: a product cut along K.  The tables are [table_positions, rotary_dim / 2]; the first
// rotary_dim elements of a head are rotated (rotary_dim even, at most head_dim), in pairs (i, i + rotary_dim / 2)
// for pairing 0 (half split) or (2 i, 2 i + 1) for pairing 1 (adjacent); the rest is only normalised.
// Value heads may have a size of their own (v_dim; 0: head_dim) and a row more columns than the heads
// (row_width elements from row to row; 0: exactly the heads), which are left alone.
int leone_qk_norm_rope_write(const void* qkv, int qkv_dtype, int qkv_planes, long qkv_plane, void* q_out,
                             void* k_pool, void* v_pool, int dtype,
                             const void* q_gain, const void* k_gain, int gain_dtype, float eps,
                             const float* cos_table, const float* sin_table, int table_positions,
                             int rotary_dim, int pairing, const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                             int rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int write_cache,
                             int v_dim, long row_width, hipStream_t stream);

// Attention of each query row over its request's cached keys [first, pos].  Values have v_dim elements a head
// (the output's width); with `gate` (float, gate_stride elements from row to row, one a query head) a head's
// result is multiplied by sigmoid(gate[row, head]).
int leone_attention_rows(const void* q, void* out, const void* k_pool, const void* v_pool, int dtype,
                         const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                         int rows, int q_heads, int kv_heads, int head_dim, int v_dim, int page_tokens, float scale,
                         int window, const float* gate, long gate_stride, hipStream_t stream);

// The same on the matrix cores for bfloat16, the keys of a row cut into `splits` parts whose
// partial results (part_acc: rows*q_heads*splits*head_dim floats, part_ml: rows*q_heads*splits*2)
// are merged by a second kernel.  head_dim a multiple of 16 up to 256, page_tokens a power of two >= 16.
int leone_attention_decode(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                           const int* row_entry, const int* block_table, int max_blocks, float* part_acc,
                           float* part_ml, int rows, int q_heads, int kv_heads, int head_dim, int page_tokens,
                           float scale, int window, int splits, hipStream_t stream);

// The same for a step in which every row is another request, from the fused q/k/v projection instead of finished
// queries: the kernel normalises and rotates the query heads itself and, with write_cache, makes the new key,
// and writes it and the new value into the cache before the keys are read (what leone_qk_norm_rope_write does,
// without its launch).  qkv: bfloat16, or float32 in qkv_planes planes added up in order.  head_dim a multiple
// of 64.  A row's keys must not be another row's new key: one row a request.  The rotation it is built for is
// the half-split one over the whole head (rotary_dim == head_dim, pairing 0); any other is refused.
int leone_attention_decode_projected(const void* qkv, int qkv_dtype, int qkv_planes, long qkv_plane, const void* q_gain,
                                     const void* k_gain, int gain_dtype, float eps, const float* cos_table,
                                     const float* sin_table, int table_positions, int rotary_dim, int pairing, void* out, void* k_pool, void* v_pool,
                                     int write_cache, const int* positions, const int* row_entry, const int* block_table,
                                     int max_blocks, float* part_acc, float* part_ml, int rows, int q_heads, int kv_heads,
                                     int head_dim, int page_tokens, float scale, int window, int splits,
                                     hipStream_t stream);

// Causal attention of prompt portions on the matrix cores for bfloat16.  `tiles` lists (entry, first
// row, rows) for runs of at most leone_attention_prefill_tile_rows() consecutive rows of one request;
// the rows of a tile sit at consecutive positions; leone_attention_prefill_group_tiles() tiles of one
// request make a group (a workgroup), unused places have 0 rows.  head_dim a multiple of 16 up to 128.
// splits > 1 (at most leone_attention_prefill_max_splits()) cuts each group's keys into that many ranges,
// one workgroup each, merged by a second kernel; it needs part_acc (rows * q_heads * splits * head_dim
// floats) and part_ml (rows * q_heads * splits * 2), rows being one more than the last row a tile names.
int leone_attention_prefill_tile_rows();
int leone_attention_prefill_group_tiles();
int leone_attention_prefill_max_splits();
int leone_attention_prefill(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                            const int* tiles, int n_groups, const int* block_table, int max_blocks, int q_heads,
                            int kv_heads, int head_dim, int page_tokens, float scale, int window, float* part_acc,
                            float* part_ml, int splits, hipStream_t stream);

// C[M,N] = A[M,K] . B[N,K]^T in float.
int leone_gemm_f32(const float* a, const float* b, float* c, int m, int n, int k, hipStream_t stream);

// Tiled weights.  The two weight-streaming products below read W either row by row ([N,K]) or, with w_tiled, from
// a copy laid out in the order in which their waves ask for it, for K a multiple of 64: rows in tiles of 16
// (the last tile filled up with zero rows), K in steps of 64, a step in two halves; element e (0..7) of the 16
// bytes that lane L = 16 g + c takes in half h of step s of tile t is W[16 t + c][64 s + 16 g + 8 h + e] and
// lies at ((((t * K / 64 + s) * 2 + h) * 64 + L) * 8 + e.  Every load of a wave is then 1 KB in one piece, which
// alone may carry the non-temporal hint (row by row an instruction covers half a line of each of 16 rows, and
// a line that is not kept is fetched twice); measured as a pure read 5.9 against 5.2 TB/s.  The results are
// the same bit for bit.
//
// Y[M,N] = X[M,K] . W[N,K]^T for bfloat16 W, M <= 16, K a multiple of 8, with row-wise neighbours folded in.
// in_mode 0: x is bfloat16 [M,K]; 1: x is the float32 stream (row r reads rows[r] if rows is given), the
// operand is x * gain and the result is scaled by 1/sqrt(mean(x^2) + eps); 2: x is bfloat16 [M,K] = bf16(stream *
// gain) and squares_in float32 [M, ceil(K / 16)] partial sums of stream^2, as a call with out_mode 3 leaves
// them; the result is scaled as for 1.  out_mode 0: y[M,N] of out_dtype; 1: y float32 [M,N] += product; 2: W
// interleaves 8 gate rows with their 8 up rows, y bfloat16 [M,N/2] = silu(gate) * up; 3: as 1, and from the new
// y: operand_out bfloat16 [M,N] = bf16(y * next_gain), squares_out float32 [M, ceil(N / 16)] sums of y^2 over
// 16 columns each.
int leone_gemm_fused_bf16(const void* x, int in_mode, const int* rows, const void* gain, int gain_dtype, float eps,
                          const void* w, int w_tiled, void* y, int out_mode, int out_dtype, int m, int n, int k,
                          const float* squares_in, void* operand_out, float* squares_out, const void* next_gain,
                          int next_gain_dtype, hipStream_t stream);

// Y[M,N] = X[M,K] . W[N,K]^T for bfloat16 X and W, M in 1..leone_gemm_rows_max_rows(), K a multiple of 8: W is
// streamed once, X goes through shared memory.  out_mode 0: y[M,N] of out_dtype; 1: y float32 [M,N] += product;
// 2: W interleaves 8 gate rows with their 8 up rows, y bfloat16 [M,N/2] = silu(gate) * up; 3: y float32
// [splits][M,N], planes `plane` elements apart, plane s holding the product over the s-th range of K (whole
// chunks of leone_gemm_rows_chunk(M) elements, ceil(chunks / splits) a range, no range empty).  splits > 1 only
// with out_mode 3.  waves (4, 6 or 8 tiles of 16 rows of W a workgroup) and ways (1 or 2 waves that share a
// tile's units of K; leone_gemm_rows_shape_built says which combinations exist for M rows) are tuning choices:
// they change the result only through the order of the sum over K.
int leone_gemm_rows_max_rows();
int leone_gemm_rows_chunk(int m);
int leone_gemm_rows_shape_built(int m, int waves, int ways);
int leone_gemm_rows_bf16(const void* x, const void* w, int w_tiled, void* y, int out_mode, int out_dtype, int m, int n, int k,
                         int splits, long plane, int waves, int ways, hipStream_t stream);

// The vendor library's product for more rows than the kernels above take, Y[M,N] = X[M,K] . W[N,K]^T (or Y +=
// with `accumulate`, Y float32), X and W bfloat16, Y of out_dtype, float accumulation, with the library's
// algorithm chosen by measurement.  leone_library_product_tune times up to max_candidates of the algorithms the
// library's heuristic lists for the problem, with every_algorithm also all others the library has for it (some
// thousands, a few seconds), on the caller's operands (x, the n_ws weights of that shape in turn, y as
// scratch: it is overwritten) and keeps the fastest for this device and exactly this (m, n, k, out_dtype,
// accumulate); it reports the time of the library's own first choice and of the winner in microseconds.
// leone_library_product runs a problem that was tuned and refuses any other: the caller keeps its ordinary
// call of the library for those.  _available: 1 if hipBLASLt could be found in the process or on the loader's
// path (it is looked up at run time and only then), 2 if its list of all algorithms is there as well, else 0; _tuned: 1 if the problem was tuned on the current device.
int leone_library_product_available();
int leone_library_product_tuned(int m, int n, int k, int out_dtype, int accumulate);
int leone_library_product_forget(int m, int n, int k, int out_dtype, int accumulate);
int leone_library_product(const void* x, const void* w, void* y, int m, int n, int k, int out_dtype, int accumulate,
                          hipStream_t stream);
int leone_library_product_tune(const void* x, const void* const* ws, int n_ws, void* y, int m, int n, int k,
                               int out_dtype, int accumulate, int max_candidates, int every_algorithm, float* first_us,
                               float* best_us, int* candidates_timed, hipStream_t stream);

// What the memory and the matrix cores give with nothing else going on: one read of `bytes` (a multiple of
// 16), one copy, and blocks x 4 waves x iterations x 8 v_mfma_f32_16x16x32_bf16, or with `wide` x 4
// v_mfma_f32_32x32x16_bf16, the same work (leone_peak_mfma_flops in all).
// The caller times them.  sink: four bytes of device memory that are practically never written.
int leone_peak_read(const void* src, long bytes, void* sink, int blocks, hipStream_t stream);
int leone_peak_copy(const void* src, void* dst, long bytes, int blocks, hipStream_t stream);
double leone_peak_mfma_flops(int blocks, int iterations);
int leone_peak_mfma(int blocks, int iterations, int wide, void* sink, hipStream_t stream);

// Highest finite logit of each row, lowest index on ties, -1 if none.  Workspace: part_value and
// part_index with rows * ceil(vocab / leone_argmax_chunk()) entries each.
int leone_argmax_chunk();
int leone_argmax(const float* logits, int* out, float* part_value, int* part_index, int rows, int vocab,
                 hipStream_t stream);
// leone_argmax with its workspace in a fixed device array of the library instead of an argument.  It has no
// counterpart in the reference; it is for callers that cannot allocate device memory (under graph capture, in
// a tight serving loop, in a harness that forbids it): the call allocates and frees nothing.  rows *
// ceil(vocab / leone_argmax_chunk()) may be at most leone_argmax_static_max_entries() (128 KiB of device
// memory that every GPU the library runs on holds until the process ends); larger calls are refused.  Calls
// on one GPU share that array: calls that overlap in time on one GPU race.
int leone_argmax_static_max_entries();
int leone_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream);
// The token whose share of the weights exp(l / t - max / t), walked in id order, holds uniform[row]; -1 for a
// row without a finite logit.  Workspace: part_value and part_index as for leone_argmax, best with one
// entry a row, sums with rows * ceil(vocab / leone_argmax_chunk()) doubles.
int leone_sample_temperature(const float* logits, const double* temperature, const double* uniform, int* out,
                             float* part_value, int* part_index, int* best, double* sums, int rows, int vocab,
                             hipStream_t stream);

// The `wanted` best finite logits of each row (higher first, lower id on a tie), best first, for a sampler
// that truncates to the k best before anything else.  out_values and out_ids have
// leone_top_candidates_max() places a row; out_count[row] is the number filled (fewer than wanted only if the
// row has fewer finite logits).
int leone_top_candidates_max();
int leone_top_candidates(const float* logits, float* out_values, int* out_ids, int* out_count, int rows, int vocab,
                         int wanted, hipStream_t stream);

// One token a row by temperature sampling with truncation stages, the first of which keeps the k best logits
// (k at most leone_top_candidates_max()): selection, stages and draw in one launch, in double, by the host
// sampler's rules.  `params` holds leone_sample_truncated_params() doubles a row: temperature, uniform value,
// number of stages (1..leone_sample_truncated_stages(); 0: the row is skipped and gets -1), then (kind, value)
// for each stage, kind 0 top-k, 1 top-p, 2 min-p.  out[row] is -1 for a row without a finite logit.
int leone_sample_truncated_stages();
int leone_sample_truncated_params();
int leone_sample_truncated(const float* logits, const double* params, int* out, int rows, int vocab,
                           hipStream_t stream);

// ---- layers that keep state of their own per request (layernorm_conv.hip, recurrent.hip) ----------------------
// x += LayerNorm(delta; dw, db, deps) if delta comes (dw null: added as it is), then y = LayerNorm(x; w, b, eps)
// if y is wanted.  With `rows` (indices) row i of y comes from row rows[i] and x is not written.  With `conv`
// ([hidden, taps]; a step of single rows, every row another request) y is h + conv(h) over the request's last
// inputs in conv_state [slots, taps - 1, hidden], which this row then joins (see leone_causal_conv).
int leone_add_layernorm(float* x, const float* delta, const void* dw, const void* db, float deps, const void* w,
                        const void* b, int w_dtype, float eps, void* y, int y_dtype, const int* rows, int n_out,
                        int hidden, const void* conv, int conv_dtype, int taps, float* conv_state, int write_state,
                        const int* positions, const int* row_entry, const int* entry_slots, hipStream_t stream);
// spans[4e .. 4e + 3]: first row and end of entry e (an entry's rows are consecutive), the state slot it reads
// (-1 at a sequence's start: zeros) and the one it writes.
int leone_entry_spans(const int* row_entry, const int* positions, const int* entry_slots, int rows, int* spans,
                      hipStream_t stream);
// A causal convolution over time per channel, w [channels, taps] with the last tap on the current row; the
// rows before a portion come from state [slots, taps - 1, channels] (float), which is brought up to date if asked.
// act: 0 none, 1 sigmoid, 2 silu.  single_rows: every entry brings one row, and the kernel that convolves moves the
// state on as well (otherwise a second launch does, from the entries' spans).
int leone_causal_conv(const void* in, int in_dtype, long in_stride, void* out, int out_dtype, long out_stride,
                      const void* w, int w_dtype, float* state, int write_state, const int* spans, int entries,
                      const int* positions, const int* row_entry, const int* entry_slots, int rows, int channels,
                      int taps, int add_input, int act, int single_rows, hipStream_t stream);
// out = (o / (max(|dot|, exp(-top)) + 1e-6) if dot comes) / rms over vdim * gain * act(gate), head by head.
int leone_head_norm_gate(const float* o, const float* dot, const float* top, const void* gain, int gain_dtype,
                         int gain_per_head, const float* gate, long gate_stride, int act, float eps, void* out,
                         int out_dtype, int rows, int heads, int vdim, hipStream_t stream);
// Projections with biases (see biased.hip).  bias_span_norm, in place on float rows [rows, stride]: the first `biased` columns
// get bias[c] (may be null) and, with round_bf16, bfloat16's rounding; then span s (columns offsets[s] .. + widths[s]) is
// divided by its root mean square over the whole span and multiplied by gains[s] ([widths[s]]); the mean is taken over
// counts[s] elements (null: widths[s]; fewer where a span holds columns of zeros that do not count).  offsets, widths,
// counts and gains are host arrays.
int leone_bias_span_norm(float* rows_at, long stride, int rows, const void* bias, int bias_dtype, int biased, int round_bf16,
                         const int* offsets, const int* widths, const int* counts, const void* const* gains, int gain_dtype,
                         int n_spans, float eps, hipStream_t stream);
// out[r, c] = act(gate_up[r, c] + bias[c]) * (gate_up[r, ffn + c] + bias[ffn + c]); act 0 silu, 1 the tanh form of gelu.
int leone_bias_glu(const void* gate_up, int in_dtype, const void* bias, int bias_dtype, void* out, int out_dtype, int rows,
                   int ffn, int act, hipStream_t stream);
// x[r, c] += bias[c] in place, x float [rows, width].
int leone_add_bias(float* x, const void* bias, int bias_dtype, int rows, int width, hipStream_t stream);
// leone_causal_conv with a bias a channel (of the filters' type, may be null) added ahead of the activation.
int leone_causal_conv_biased(const void* in, int in_dtype, long in_stride, void* out, int out_dtype, long out_stride,
                             const void* w, const void* bias, int w_dtype, float* state, int write_state, const int* spans,
                             int entries, const int* positions, const int* row_entry, const int* entry_slots, int rows,
                             int channels, int taps, int add_input, int act, int single_rows, hipStream_t stream);
// leone_head_norm_gate with the gate ahead of the norm if gate_first.
int leone_head_norm_gate_ordered(const float* o, const float* dot, const float* top, const void* gain, int gain_dtype,
                                 int gain_per_head, const float* gate, long gate_stride, int act, int gate_first, float eps,
                                 void* out, int out_dtype, int rows, int heads, int vdim, hipStream_t stream);
// out = sum over branches of weights[b] * branch (host floats; n elements each), nothing normed.
int leone_weighted_mix(const float* const* branch_rows, const float* weights, int branches, float* out, long n,
                       hipStream_t stream);
// out = scale * sum over branches of rms(branch) * gain.
int leone_rms_mix(const float* const* branch_rows, const void* const* gains, int gain_dtype, int branches, float eps,
                  float scale, float* out, int rows, int hidden, hipStream_t stream);
int leone_relu_squared(const void* in, void* out, int dtype, long n, hipStream_t stream);
int leone_head_gate(void* out, int dtype, const float* gate, long gate_stride, int rows, int heads, int vdim,
                    hipStream_t stream);
// The matrix-memory recurrences (see recurrent.hip); key sizes up to leone_scan_max_dim().
int leone_scan_max_dim();
// segments: n x (first row, end, index of the state read or -1 for zeros, index of the state written or -1).
int leone_exp_gates(const float* proj, long stride, int i_off, int f_off, const void* i_bias, const void* f_bias,
                    int bias_dtype, float cap, const int* spans, int entries, float* state, long slot_stride,
                    long head_stride, long top_at, int write_state, float* coef, float* top, int heads, hipStream_t stream);
int leone_outer_scan(const float* proj, long stride, int q_off, int k_off, int v_off, const float* coef,
                     const float* decay, int no_input, int accumulate, int norm_column, float q_scale, float k_scale,
                     const float* cos_table, const float* sin_table, int rotary_dim, int table_positions,
                     const int* positions, const int* segments, int n_segments, const float* state_in, long in_stride,
                     float* state_out, long out_stride, long head_stride, float* decay_product, float* out, float* dot,
                     int heads, int dim, int vdim, hipStream_t stream);
int leone_outer_chain(const int* links, int n_links, float* work, long work_stride, const float* product, float* state,
                      long slot_stride, long head_stride, int per_head, int heads, int write_state, hipStream_t stream);
int leone_delta_scan(const float* qkv, long stride, int q_off, int k_off, int v_off, const float* beta,
                     long beta_stride, const float* step, long step_stride, const void* rate_log,
                     const void* step_bias, int vec_dtype, float q_scale, float unit_eps, int no_input, int accumulate,
                     const int* segments, int n_segments, const float* state_in, long in_stride, float* state_out,
                     long out_stride, float* transition, float* out, int heads, int kv_heads, int dim, int vdim,
                     hipStream_t stream);
int leone_delta_chain(const int* links, int n_links, float* work, long work_stride, const float* transition, float* state,
                      long slot_stride, int heads, int dim, int vdim, int write_state, hipStream_t stream);

// ---- a token table with a learned position table added, norms behind sublayers, kept first keys, routed experts ----
// leone_embed, and place_table[positions[r], :] (of the table's type, [places, hidden]) added unscaled.
int leone_embed_placed(const void* table, int dtype, const int* tokens, float* out, int rows, int hidden, int vocab,
                       float scale, const void* place_table, const int* positions, int places, hipStream_t stream);
// gate_up as for leone_swiglu; act: 0 silu, 1 the tanh form of gelu on the gate.
int leone_glu(const void* gate_up, void* out, int dtype, int rows, int ffn, int act, hipStream_t stream);
// x[r] += rmsnorm(sum of the delta's planes)[r] * gain (delta float32, may be null); then y[r] = x[r] in y_dtype
// (y may be null), or, with gain2, y[i] = rmsnorm(x[rows ? rows[i] : i]) * gain2 (with rows, x is not written).
int leone_add_normed(float* x, const float* delta, int delta_planes, long delta_plane, const void* gain, int gain_dtype,
                     float eps, void* y, int y_dtype, const void* gain2, int gain2_dtype, float eps2, const int* rows,
                     int n_rows, int hidden, hipStream_t stream);
// leone_attention_rows with the keys below keep_first kept in sight of a windowed layer, and with gate_each a
// gate value for every element of every head ([rows, q_heads * v_dim] within rows of gate_stride).
int leone_attention_rows_kept(const void* q, void* out, const void* k_pool, const void* v_pool, int dtype,
                              const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                              int rows, int q_heads, int kv_heads, int head_dim, int v_dim, int page_tokens,
                              float scale, int window, const float* gate, long gate_stride, int keep_first,
                              int gate_each, hipStream_t stream);
// leone_attention_rows_kept with a distance bias (slopes float [q_heads] or null: head h's score at distance d is lowered by
// slopes[h] * d) and a query factor that grows with the position (temp_every > 0: 1 + temp_coef * ln(floor((pos + 1) /
// temp_every) + 1)).
int leone_attention_rows_biased(const void* q, void* out, const void* k_pool, const void* v_pool, int dtype,
                                const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                                int rows, int q_heads, int kv_heads, int head_dim, int v_dim, int page_tokens,
                                float scale, int window, const float* gate, long gate_stride, int keep_first,
                                int gate_each, const float* slopes, float temp_coef, int temp_every, hipStream_t stream);
// The matrix-core kernels with the same distance bias and query factor as leone_attention_rows_biased.
int leone_attention_decode_biased(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                                  const int* row_entry, const int* block_table, int max_blocks, float* part_acc,
                                  float* part_ml, int rows, int q_heads, int kv_heads, int head_dim, int page_tokens,
                                  float scale, int window, int splits, int keep_first, const float* slopes,
                                  float temp_coef, int temp_every, hipStream_t stream);
int leone_attention_prefill_biased(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                                   const int* tiles, int n_groups, const int* block_table, int max_blocks, int q_heads,
                                   int kv_heads, int head_dim, int page_tokens, float scale, int window, float* part_acc,
                                   float* part_ml, int splits, int keep_first, const float* slopes, float temp_coef,
                                   int temp_every, hipStream_t stream);
// leone_attention_decode with the keys at positions below keep_first kept in sight of a windowed layer.
int leone_attention_decode_kept(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                                const int* row_entry, const int* block_table, int max_blocks, float* part_acc,
                                float* part_ml, int rows, int q_heads, int kv_heads, int head_dim, int page_tokens,
                                float scale, int window, int splits, int keep_first, hipStream_t stream);
// leone_attention_prefill with the keys at positions below keep_first kept in sight of a windowed layer (splits 1).
int leone_attention_prefill_kept(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                                 const int* tiles, int n_groups, const int* block_table, int max_blocks, int q_heads,
                                 int kv_heads, int head_dim, int page_tokens, float scale, int window, float* part_acc,
                                 float* part_ml, int splits, int keep_first, hipStream_t stream);
// Router: chosen int32 [rows, top], weight float32 [rows, top] from logits float32 [rows, total] (see routed.hip).
// score: 0 softmax over the outputs, 1 a sigmoid of each; group_best: how many of a group's best choice scores are summed
// into the group's score; renorm: the winners' scores over their sum (1) or as they are (0); weight_scale multiplies them.
int leone_route_max_outputs();
int leone_route_topk(const float* logits, const void* correction, int correction_dtype, int* chosen, float* weight,
                     int rows, int total, int top, int group_count, int group_keep, int score, int group_best, int renorm,
                     float weight_scale, hipStream_t stream);
// Pairs (row, place) of the experts below `experts` gathered in tiles of `tile` pairs of one expert (leone_moe_tile_pairs(),
// 16, 64 or 128): tile_expert int32 [max_tiles] (-1: unused), tile_pairs int32 [max_tiles, tile] (-1: empty);
// max_tiles >= min(pairs, pairs / tile + experts).
int leone_moe_tile_pairs();
// leone_route_topk and leone_moe_plan in one launch of one workgroup, for steps of at most 256 rows.  always: the last
// so many of the experts are taken by every row with weight 1 (chosen and weight are [rows, top + always] then).
int leone_route_plan(const float* logits, const void* correction, int correction_dtype, int* chosen, float* weight, int rows,
                     int total, int top, int group_count, int group_keep, int experts, int* tile_expert, int* tile_pairs,
                     int max_tiles, int tile, int always, int score, int group_best, int renorm, float weight_scale,
                     hipStream_t stream);
int leone_moe_plan(const int* chosen, int pairs, int experts, int* tile_expert, int* tile_pairs, int max_tiles, int tile,
                   hipStream_t stream);
// tile: leone_moe_tile_pairs() (any type and size), or 16, 64 or 128 (matrix cores: bfloat16, n and k multiples of 8).
int leone_moe_product(const void* x, const void* w, void* y, const float* pair_weight, int dtype, int gated,
                      const int* tile_expert, const int* tile_pairs, int max_tiles, int tile, int top, int n, int k, int act,
                      float limit, hipStream_t stream);
int leone_moe_combine(const float* pair_out, const int* chosen, const float* weight, const void* x, int dtype,
                      const float* extra, float* out, int rows, int top, int experts, int hidden, hipStream_t stream);
// A matrix memory whose forget gate per head and key channel also says what is written (see gated_scan.hip).
int leone_gated_scan(const float* proj, long stride, int q_off, int f_off, int v_off, const void* f_bias, const void* lower,
                     int vec_dtype, int q_silu, int no_input, int accumulate, const int* segments, int n_segments,
                     const float* state_in, long in_stride, float* state_out, long out_stride, float* gate_product, float* out,
                     int heads, int dim, int vdim, hipStream_t stream);
// The same walk for a state-space layer: S <- exp(-exp(rate_log) dt) S + (dt B) x^T, o = S^T C + skip x, dt =
// softplus(step + step_bias); B and C in groups_bc groups shared by neighbouring heads.  Chunks chain through leone_gated_chain.
int leone_state_space_scan(const float* xbc, long stride, int x_off, int b_off, int c_off, int groups_bc, const float* step,
                           long step_stride, int step_off, const void* step_bias, const void* rate_log, const void* skip,
                           int vec_dtype, int no_input, int accumulate, const int* segments, int n_segments,
                           const float* state_in, long in_stride, float* state_out, long out_stride, float* gate_product,
                           float* out, int heads, int dim, int vdim, hipStream_t stream);
int leone_gated_chain(const int* links, int n_links, float* work, long work_stride, const float* product, float* state,
                      long slot_stride, int heads, int dim, int vdim, int write_state, hipStream_t stream);
// Attention through a latent that all heads share (see latent.hip).
int leone_latent_max_width();
int leone_latent_prepare(const float* proj, long stride, int rows, int q_off, int q_rank, const void* q_gain, void* q_out,
                         int kv_off, int rank, int rot, const void* kv_gain, int gain_dtype, float eps, const float* cos_table,
                         const float* sin_table, int rot_half, int table_positions, const int* positions, const int* row_entry,
                         const int* block_table, int max_blocks, int page_tokens, void* k_pool, void* v_pool, int dtype,
                         hipStream_t stream);
int leone_head_product(const float* x, long x_row_stride, long x_head_stride, const void* w, int w_dtype, void* y, int y_dtype,
                       long y_row_stride, long y_head_stride, int rows, int heads, int inner, int outer, int tail,
                       const float* cos_table, const float* sin_table, int rot_half, int table_positions, const int* positions,
                       hipStream_t stream);
int leone_latent_attention(const float* q, float* out, const void* pool, int dtype, const int* positions, const int* row_entry,
                           const int* block_table, int max_blocks, int rows, int heads, int rank, int rot, int page_tokens,
                           float scale, int window, hipStream_t stream);
int leone_latent_cores_max_width();
int leone_latent_attention_cores(const void* q, float* out, const void* k_pool, const void* v_pool, const int* positions,
                                 const int* row_entry, const int* block_table, int max_blocks, int rows, int heads, int rank,
                                 int rot, int page_tokens, float scale, int window, int splits, float* part_acc, float* part_ml,
                                 hipStream_t stream);
// Residual sums with a factor; the stream as a weighted sum of every earlier layer's result (see depth.hip).
int leone_residual_norm(float* x, const float* delta, int planes, long plane, float scale, const void* gain, int gain_dtype,
                        float eps, void* y, int y_dtype, const int* rows, int n_rows, int hidden, hipStream_t stream);
int leone_depth_mix(float* x, const float* delta, int planes, long plane, float scale, float* history, long slot_stride,
                    int count, const void* weight, int weight_dtype, long total, hipStream_t stream);
}
