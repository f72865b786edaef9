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
int leone_qk_norm_rope_write(const void* qkv, int qkv_dtype, int qkv_planes, long qkv_plane, void* q_out,
                             void* k_pool, void* v_pool, int dtype,
                             const void* q_gain, const void* k_gain, int gain_dtype, float eps,
                             const float* cos_table, const float* sin_table, int table_positions,
                             int rotary_dim, int pairing, const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                             int rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int write_cache,
                             hipStream_t stream);

// Attention of each query row over its request's cached keys [first, pos].
int leone_attention_rows(const void* q, void* out, const void* k_pool, const void* v_pool, int dtype,
                         const int* positions, const int* row_entry, const int* block_table, int max_blocks,
                         int rows, int q_heads, int kv_heads, int head_dim, int page_tokens, float scale,
                         int window, hipStream_t stream);

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
}
