// C ABI of the kernel library.  Every function launches on `stream`, returns 0 on success or a
// negative value after recording a message for fllm_last_error(), and never allocates device
// memory.  Element type codes: 0 = float32, 1 = bfloat16.  All tensors are dense row-major
// unless a stride is given.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *fllm_last_error(void);
int fllm_abi_version(void);
// 0: bfloat16 calls use the plain kernels only (for comparing them with the MFMA kernels); default 1
void fllm_set_fast_kernels(int on);
// Switches a kernel variant (for measurements and tests): "attention.tile32" 0/1; "linear.slices" n
// (0: chosen by shape); "linear.dual_k" 0/1; "linear.x_direct" 0/1; "attention.fused_merge" 0/1;
// "attention.prefill_parts" 0/1; "linear.slab" 0/1/2; "linear.wide_waves" 0 (planned)/4/7/8; "linear.resident_tiles" 0/1;
// "attention.tile32_rows" 0 (chosen by the launch)/128/256.  0 on success.
int fllm_set_option(const char *name, int value);

// out[r, :] = scale * table[ids[r], :]            out: float32 [rows, width]
int fllm_embed(const int32_t *ids, const void *table, float *out, int rows, int width, int vocab, int table_dtype,
               float scale, hipStream_t stream);

// out[i, :] = x[row(i), :] * (rsqrt(mean(x[row(i)]^2) + eps) * weight),  row(i) = rows ? rows[i] : i
int fllm_rmsnorm(const float *x, const int32_t *rows, const float *weight, void *out, int count, int width, float eps,
                 int out_dtype, hipStream_t stream);

// x[r, :] += branch[r, :] (float32 sum, written back), then out[r, :] = rmsnorm(x[r, :]) as above
int fllm_add_rmsnorm(float *x, const void *branch, int branch_dtype, const float *weight, void *out, int count, int width,
                     float eps, int out_dtype, hipStream_t stream);

// y[m, n] = sum_k x[m, k] * w[n, k] (+ bias[n]);   x: [M, K] (row stride ldx), w: [N, K]
// out_mode 0: store as `dtype`; 1: store float32; 2: add to float32 `out` (row stride ldo)
int fllm_linear(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N, int K,
                int dtype, int out_mode, hipStream_t stream);

// Device memory for kernels that meet across workgroups: the decode-shaped products (1..16 rows), whose K
// dimension is cut into slices over workgroups when the activations of all of K do not fit into LDS, and
// decode attention over split contexts, and prompt attention of few rows over long contexts (the keys of a row
// tile go to several workgroups: 66 KiB a part for heads of 128).  Its first 64 KiB are counters, which must be zero when it is handed
// over and are zero again after every launch; partial sums follow.  One per device (the current one);
// work that would need more than it holds runs another way.  Launches on different streams of one device
// must not overlap while it is set.  nullptr takes it away.
int fllm_set_device_workspace(void *workspace, size_t bytes);

// Fused forms for decode steps in bfloat16 (1..64 rows, K a multiple of 8; fllm_fused_decode_supported).
// x is the float32 residual stream [M, K]; each computes rmsnorm(x; norm_w, eps) @ w^T (+ bias) and
//   fllm_norm_linear          stores it as bfloat16 [M, N]
//   fllm_norm_gate_up_swiglu  w = [gate; up] ([2 I, K]): stores silu(gate) * up as bfloat16 [M, I]
//   fllm_norm_qkv_rope_store  w = [q; k; v]: rotates query and key lanes in pairs (2l, 2l+1), stores the
//                             queries as bfloat16 [M, heads * head_dim] and keys and values into the pages
//                             (layouts and row/segment/table arguments as fllm_rope_kv_store)
int fllm_fused_decode_supported(int M, int K);
// out = silu(x gate^T) * (x up^T) for bfloat16 rows x [M, K] (1..64 rows, row stride ldx; fllm_gate_up_swiglu_tiled: to 128), w = [gate; up] ([2 I, K])
int fllm_gate_up_swiglu(const void *x, int ldx, const void *w_gate_up, const float *bias, void *out, int M, int inter,
                        int K, hipStream_t stream);
// The gated products with the activation's constants as arguments: a(g') * (u' + offset), a(g) = g * sigmoid(alpha g),
// g' = min(gate, limit), u' = clamp(up, -limit, limit) (limit <= 0: nothing is clamped).  fllm_norm_gate_up_glu folds the
// RMSNorm of float32 rows in (1..64 rows); fllm_gate_up_glu takes bfloat16 rows (1..64, or 17..128 with `w_tiles`).
int fllm_norm_gate_up_glu(const float *x, const float *norm_w, float eps, const void *w_gate_up, const float *bias, void *out,
                          int M, int inter, int K, float limit, float alpha, float offset, hipStream_t stream);
int fllm_gate_up_glu(const void *x, int ldx, const void *w_gate_up, const void *w_tiles, const float *bias, void *out, int M,
                     int inter, int K, float limit, float alpha, float offset, hipStream_t stream);
int fllm_norm_linear(const float *x, const float *norm_w, float eps, const void *w, const float *bias, void *out, int M,
                     int N, int K, hipStream_t stream);
int fllm_norm_gate_up_swiglu(const float *x, const float *norm_w, float eps, const void *w_gate_up, const float *bias,
                             void *out, int M, int inter, int K, hipStream_t stream);
int fllm_norm_qkv_rope_store(const float *x, const float *norm_w, float eps, const void *w_qkv, const float *bias,
                             void *q_out, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                             int table_stride, const float *cos_table, const float *sin_table, int rope_dims, void *k_pages,
                             void *v_pages, int M, int heads, int kv_heads, int head_dim, int K, int page_size,
                             int store_kv, hipStream_t stream);

// A norm prepared by the product before it, for steps of up to 64 rows (the sum itself: up to 128).  fllm_linear_add_normed: out += x w^T
// (float32 out [M, N], N a multiple of 16) and, for the RMSNorm that reads out next, next_x = out * next_w as
// bfloat16 [M, N] and next_ssq [M, *tiles_out]: the sums of squares of out over the outputs of each tile (room for
// M * N / 8 floats; *tiles_out, host memory, is set at the call).  The scaled forms are the norm forms above with
// that pair in place of the float32 rows and the norm's weight.
// w_tiles (may be null up to 16 rows): the tile-major copy of w, see below; the scaled forms of 17 to 64 rows need it, and K
// in steps of 256.
int fllm_linear_add_normed(const void *x, int ldx, const void *w, const float *bias, float *out, int M, int N, int K,
                           const float *next_w, void *next_x, float *next_ssq, int *tiles_out, const void *w_tiles,
                           hipStream_t stream);

// Tile-major weights for the products of decode steps that add into the residual stream (output and down
// projections).  A decode-shaped product feeds 16 weight rows x 32 columns to a matrix-core instruction, 16 bytes a
// lane: from a row-major matrix that is 64 bytes of each of 16 rows a load, and the memory pipeline of a compute unit
// looks up 64 cache lines for it; from the tile-major copy it is 1 KiB in a row, 8 lines, and the product of 8 or 16 rows
// takes no longer than that of one (down projection of the 8B sizes: 29 -> 24 us at 8 rows).  The copy costs the
// matrix's memory a second time, which a GPU with 288 GB affords; row-major stays for the GEMM library's products.
// Steps of 17 to 64 rows read the copies too (four to eight weight tiles a workgroup, the activations through LDS in chunks;
// the two products of the feed-forward up to 128 rows):
// the feed-forward and q/k/v products with their fused prologues and epilogues then beat the library's products and
// the separate norm, rotary and SwiGLU kernels.
//   fllm_weight_tiles_supported  1 where the kernels take tiles: N >= 16, K a multiple of 1,024
//   fllm_weight_tiles_elements   bfloat16 elements of the copy: N rounded up to 16, times K
//   fllm_tile_weights            writes the copy: [tile of 16 rows][block of 128 columns][k-step of 32][lane][8]
//   fllm_linear_add_tiled        out += x w^T (+ bias), float32 out, 1..128 rows (beyond 64: w_tiles required, K in steps of 256)
//   fllm_linear_f32_tiled        out = x w^T (+ bias), float32 out, 1..64 rows (the vocabulary projection); with w_tiles where it can
//   fllm_tile_weights_gate_up    the copy of [gate; up] ([2 inter][K]) for the SwiGLU epilogue of 17 to 64 rows: tile T holds
//                                gate rows 8 T .. 8 T + 7 and then the same up rows; fllm_weight_tiles_elements_gate_up elements
//   fllm_gate_up_swiglu_tiled    fllm_gate_up_swiglu for 17..128 rows with that copy (null: row-major, up to 64 rows)
int fllm_weight_tiles_supported(int N, int K);
size_t fllm_weight_tiles_elements(int N, int K);
int fllm_tile_weights(const void *w, void *tiles, int N, int K, hipStream_t stream);
int fllm_linear_add_tiled(const void *x, int ldx, const void *w, const void *w_tiles, const float *bias, float *out, int ldo,
                          int M, int N, int K, hipStream_t stream);
int fllm_linear_f32_tiled(const void *x, int ldx, const void *w, const void *w_tiles, const float *bias, float *out, int ldo,
                          int M, int N, int K, hipStream_t stream);
size_t fllm_weight_tiles_elements_gate_up(int inter, int K);
int fllm_tile_weights_gate_up(const void *w, void *tiles, int inter, int K, hipStream_t stream);
int fllm_gate_up_swiglu_tiled(const void *x, int ldx, const void *w_gate_up, const void *w_tiles, const float *bias, void *out, int M,
                              int inter, int K, hipStream_t stream);
int fllm_scaled_gate_up_swiglu(const void *xn, const float *ssq, int ssq_count, float eps, const void *w_gate_up,
                               const float *bias, void *out, int M, int inter, int K, const void *w_tiles, hipStream_t stream);
int fllm_scaled_qkv_rope_store(const void *xn, const float *ssq, int ssq_count, float eps, const void *w_qkv, const float *bias,
                               void *q_out, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                               int table_stride, const float *cos_table, const float *sin_table, int rope_dims, void *k_pages,
                               void *v_pages, int M, int heads, int kv_heads, int head_dim, int K, int page_size, int store_kv,
                               const void *w_tiles, hipStream_t stream);

// The pair that fllm_linear_add_normed leaves, from float32 rows that no such product wrote: xn = x * weight as bfloat16
// [rows, width] and ssq [rows] (one part a row).
int fllm_prepare_norm(const float *x, const float *weight, void *xn, float *ssq, int rows, int width, hipStream_t stream);

// residual[r, :] += branch[r, :]   (residual float32 [rows, width], branch of type `dtype`)
int fllm_add_residual(float *residual, const void *branch, int rows, int width, int dtype, hipStream_t stream);

// out[r, j] = silu(gu[r, j]) * gu[r, I + j]
int fllm_swiglu(const void *gate_up, void *out, int rows, int inter, int dtype, hipStream_t stream);

// Rotates the query and key heads of qkv rows in place and stores keys and values in pages.
// qkv: [rows, (heads + kv_heads) * head_dim + kv_heads * v_dim] (values may have a width of their own); row r belongs to
// segment row_seg[r] at position row_pos[r]; its page is tables[row_seg[r] * table_stride + row_pos[r] / page_size].
// K pages: [page][kv_head][head_dim / 8][token][8]; V pages: [page][kv_head][v_dim][token].
// pairing 0: lanes (l, l + rope_dims/2); 1: lanes (2l, 2l + 1).  store_kv 0 leaves the pages alone.
int fllm_rope_kv_store(void *qkv, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                       int table_stride, const float *cos_table, const float *sin_table, int table_positions,
                       void *k_pages, void *v_pages, int num_pages, int rows, int heads, int kv_heads, int head_dim,
                       int v_dim, int rope_dims, int pairing, int page_size, int key_chunk, int dtype, int store_kv,
                       hipStream_t stream);

// Causal attention of each row over the pages of its segment: keys at positions
// [max(0, pos - window + 1), pos] (window <= 0: from 0), and with chunk > 0 none before pos - pos % chunk (the start of
// the row's own chunk of positions).  q: rows of `q_stride` elements, head h at h * head_dim.  Values have `v_dim` lanes
// a head; out: [rows, heads * v_dim].  Keys lie in chunks of `key_chunk` values inside a page (8, or 1 for head sizes
// that are no multiple of 8).  The matrix-core kernels take v_dim == head_dim and chunks of 8; the rest runs the plain kernel.  Rows of a segment are consecutive in the batch, at
// consecutive positions; seg_start[s] is the first row of segment s (seg_start[num_segs] = rows).
// `max_context` bounds pos + 1.  The segments from `single_from` on have one row each (0: every segment, a decode
// step; num_segs: none is known to): rows of long contexts among them are split over workgroups, which portions
// of prompts are not.  `workspace` holds partial results of split contexts (fllm_attention_workspace_bytes() of
// the number of single rows).
int fllm_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                   int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                   int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int v_dim, int page_size,
                   int num_pages, float scale, int window, int chunk, int key_chunk, const float *sinks, int dtype, int max_context,
                   int single_from, void *workspace, size_t workspace_bytes, hipStream_t stream);
size_t fllm_attention_workspace_bytes(int rows, int heads, int kv_heads, int head_dim, int max_context);
// The same attention with a bias on every score that depends on the distance alone: score(row, key) = q . k * scale +
// head_slopes[head] * (key position - row position), float32 `head_slopes[heads]` (for position encodings that bias
// scores instead of, or beside, rotating q and k).  Runs the plain kernel (one workgroup a row and head) in both
// precisions: the MFMA kernels know no bias.
int fllm_attention_sloped(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                          int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                          int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int page_size,
                          int num_pages, float scale, int window, int dtype, int max_context, const float *head_slopes,
                          hipStream_t stream);

// ids[r] = previous[source[r]] where source[r] >= 0: token ids that an earlier step chose and that have not left
// the device yet become the input of this step
int fllm_carry_ids(int32_t *ids, const int32_t *source, const int32_t *previous, int rows, int previous_rows,
                   hipStream_t stream);

// Probes for measurements: a kernel that only reads `bytes` from `src` (`sink`: 4 bytes a workgroup, left alone),
// and one that only multiplies (32x32x16 bfloat16 MFMA, `blocks` workgroups of 8 waves; `sink`: 2 KiB a workgroup;
// returns the floating-point operations of the launch, negative on error).  The caller times them.
// out[i] = element i of the random tensor with key (key_lo, key_hi): kind 0 a normal number of deviation 0.02, kind 1
// a norm weight 1 + U(-0.1, 0.1); the generator that fllm_amd/weights/random_init.py specifies, bit for bit what
// that module computes on the host.  `dtype` 0 float32, 1 bfloat16 (rounded to nearest even).
int fllm_random_fill(void *out, uint64_t count, uint32_t key_lo, uint32_t key_hi, int kind, int dtype, hipStream_t stream);

int fllm_probe_read(const void *src, size_t bytes, void *sink, int blocks, hipStream_t stream);
double fllm_probe_mfma_bf16(void *sink, int blocks, int iters, hipStream_t stream);

// out[r] = first index of the largest finite value of logits[r, :]
int fllm_argmax(const float *logits, int32_t *out, int rows, int vocab, hipStream_t stream);

// fllm_argmax for callers that cannot allocate device memory and have no workspace to hand over (code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
// The workgroups of a row meet in a static device array of 132,096 bytes that every GPU the library runs on holds
// until the process ends; the call allocates nothing and needs no fllm_set_device_workspace.  At most 256 rows
// (more are refused; any vocabulary).  Same result as fllm_argmax.  All calls on one GPU share that GPU's array:
// calls that overlap on one GPU (different streams, different threads) race; calls in stream order do not.  The
// entry point takes any stream and checks nothing of this: keeping one call in flight a device is the caller's duty.  The
// first call on a device looks up the array's address (once per device); make it outside a graph capture.
int fllm_argmax_static(const float *logits, int32_t *out, int rows, int vocab, hipStream_t stream);

struct FllmSampleRow {
    float temperature;   // <= 1e-5: greedy
    float top_p;         // nucleus; outside (0, 1): off
    int32_t top_k;       // <= 0: off
    float min_p;         // drops what weighs less than min_p times the likeliest token; <= 0: off
    uint64_t seed;       // Philox key
    uint64_t draw;       // number of the draw of this request
};
// What is done to a row of logits before a token is chosen (rust/engine/src/sampling.rs:220-229, :252-274).  The
// lists live in arrays shared by all rows: seen_ids / seen_counts [seen_off .. + seen_len) are the distinct tokens of
// the request's history (within its window) and how often each occurs; bias_ids / bias_values; blocked_ids (to -inf);
// allowed_ids (rising; when a row has any, every other token goes to -inf); if_last / then_blocked (pairs: the second
// goes to -inf when the newest token is the first).
// last_row >= 0: last_tokens[last_row] (device memory, written by an earlier launch) is the newest token of the
// history and not in the lists yet: it counts once more, and the pairs are judged by it.  A row whose lists are empty
// and last_row < 0 is left alone.
struct FllmAdjustRow {
    float repetition_penalty;   // 1: off
    float presence_penalty;
    float frequency_penalty;
    int32_t seen_off, seen_len;
    int32_t bias_off, bias_len;
    int32_t blocked_off, blocked_len;
    int32_t last_row;           // -1: none
    int32_t allowed_off, allowed_len;
    int32_t pairs_off, pairs_len;
};
// Device arrays that the rows' offsets point into; any may be null when no row uses it.  The struct itself is read
// on the host, at the call.
struct FllmAdjustLists {
    const int32_t *seen_ids, *seen_counts;
    const int32_t *bias_ids;
    const float *bias_values;
    const int32_t *blocked_ids;
    const int32_t *allowed_ids;
    const int32_t *if_last, *then_blocked;
};
// logits: float32 [rows, vocab], changed in place; one record a row (device memory)
int fllm_adjust_logits(float *logits, int rows, int vocab, const struct FllmAdjustRow *row_records,
                       const struct FllmAdjustLists *lists, const int32_t *last_tokens, hipStream_t stream);

// Log-probabilities in the softmax of logits [rows, vocab] as they are: for each of the `wanted` rows named in
// wanted_rows, values[(1 + top) * w] is that of tokens[row], the `top` (at most 20) values behind it those of the
// likeliest tokens, whose ids stand at the same places of `ids` (ids[(1 + top) * w] repeats the chosen token).
// wanted_rows are checked by the caller: they are read on the device.
int fllm_logprobs(const float *logits, int rows, int vocab, const int32_t *wanted_rows, int wanted, const int32_t *tokens,
                  int top, float *values, int32_t *ids, hipStream_t stream);

// The same for the distribution a token was drawn from: logits as the sampler saw them (penalties and biases applied),
// divided by the temperature, over the tokens that top-k, min-p and top-p leave (params: the records fllm_sample got,
// one a row); a greedy row is a point mass.  A chosen token that the filters leave out has -inf; where fewer than `top`
// tokens are left the rest of ids is -1.
int fllm_logprobs_processed(const float *logits, int rows, int vocab, const int32_t *wanted_rows, int wanted, const int32_t *tokens,
                            const struct FllmSampleRow *params, int top, float *values, int32_t *ids, hipStream_t stream);

// work: float32 [rows, vocab] scratch.  kinds: what the caller knows of the rows, a sum of 1 (some have a temperature
// and no filter: their draw looks at every token, and several workgroups share such a row), 2 (some are of another
// kind) and 4 (some of those have a top-k of at most 64: several workgroups share such a row as well).
int fllm_sample(const float *logits, float *work, const struct FllmSampleRow *params, int32_t *out, int rows, int vocab,
                int kinds, hipStream_t stream);

// ---- parts of other layer designs -------------------------------------------------------------------------------
// Two RMSNorms of the same float32 rows in one pass: out1 = x * rsqrt(mean(x^2) + eps1) * w1, out2 likewise with w2
// and eps2 (w2 and out2 null: one norm).  For blocks whose branches read the same residual stream.
int fllm_rmsnorm_pair(const float *x, const float *w1, const float *w2, void *out1, void *out2, int rows, int width,
                      float eps1, float eps2, int out_dtype, hipStream_t stream);
// out[r, j] = g * sigmoid(alpha * g) * (u + up_offset), g = min(gu[r, j], limit), u = clamp(gu[r, I + j], -limit, limit)
// (limit <= 0: nothing is clamped)
int fllm_glu_clamped(const void *gate_up, void *out, int rows, int inter, float limit, float alpha, float up_offset, int dtype,
                     hipStream_t stream);
// x[i] *= scale
int fllm_scale_f32(float *x, size_t total, float scale, hipStream_t stream);
// x[r, :] = (x[r, :] + scale * table[ids[r], :]) + vec[:]; table (with ids) or vec may be null
int fllm_stream_add(float *x, const int32_t *ids, const void *table, int table_dtype, int vocab, float scale, const float *vec,
                    int rows, int width, hipStream_t stream);

// Rows of a joint q/k/v product (row stride ld; queries first, then keys, then values): RMSNorm over the whole query
// projection with q_weight [heads * k_dim] and over the whole key projection with k_weight [kv_heads * k_dim], rotary on
// the first rope_dims lanes of every query and key head (lane i with lane i + rope_dims / 2; float32 tables [positions,
// rope_dims / 2]); queries to q_out [rows, heads * k_dim], keys and values into the pages of the row's request.
// K pages: [page][kv_head][k_dim / key_chunk][token][key_chunk]; V pages: [page][kv_head][v_dim][token].
int fllm_qk_norm_rope_store(const void *qkv, int ld, const float *q_weight, const float *k_weight, float eps, void *q_out,
                            const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables, int table_stride,
                            const float *cos_table, const float *sin_table, int table_positions, void *k_pages, void *v_pages,
                            int rows, int heads, int kv_heads, int k_dim, int v_dim, int rope_dims, int page_size, int key_chunk,
                            int dtype, int store_kv, hipStream_t stream);
// Attention whose scores are mixed across heads before the softmax: score[h] = sum_g talk[h, g] * (q_g . k * scale *
// temp[g]) over the keys lo .. pos of the row's request, lo = pos - pos % chunk (chunk 0: lo = 0); out[h] = gate *
// softmax(score[h]) v, gate = sigmoid(gate[row * gate_stride + h]) (gate null: 1).  q: [rows, heads * k_dim]; out:
// [rows, heads * v_dim]; talk float32 [heads, heads], temp float32 [heads].  Rows, segments and tables as fllm_attention.
int fllm_talking_attention(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                           const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                           const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out, int rows,
                           int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale, int chunk, int key_chunk,
                           int dtype, int max_context, int splits, float *ws, size_t ws_floats, int single_rows, hipStream_t stream);
// `splits` > 1 (bfloat16, the matrix-core kernel): that many workgroups share the keys of a tile of 16 rows and meet in
// `ws`, float32, at least fllm_talking_attention_workspace(...) floats; the plain kernels ignore both.  `single_rows`: the
// caller knows that every segment has one row (a decode step), which has a matrix-core kernel of its own.
size_t fllm_talking_attention_workspace(int rows, int num_segs, int heads, int v_dim, int splits);

// A branch that is normed on its way into the float32 residual stream: v = the sum of the row's `parts` partial branches
// (branch: [rows, parts, width] of `branch_dtype`), x[r] += v * rsqrt(mean(v^2) + eps) * gain (normalize 0: x[r] += v * gain).
// With next_w, next_out[r] = rmsnorm(x[r]) * next_w with next_eps (of `next_dtype`) as well.
// part_weights (float32 [rows * parts], or null): partial row k of a token is multiplied by its weight as it is summed.
int fllm_postnorm_add(float *x, const void *branch, int branch_dtype, int parts, const float *part_weights, const float *gain, float eps,
                      int normalize,
                      const float *next_w, float next_eps, void *next_out, int next_dtype, int rows, int width, hipStream_t stream);

// Routed experts, plain kernels.  fllm_route_topk: score = sigmoid(w_router h) in float32 ([E, K] beside rows [rows, K] of
// `dtype`, row stride ldh); ids[r, k] / weights[r, k] = the expert with the k-th largest score of row r (the lower index
// among equals) and that score.  fllm_experts_gate_up: for every (row, pick) pair, act[pair] = a(g) * (u + up_offset) with
// g, u = the gate and up rows of the picked expert times (h[row] * weight), clamped as in fllm_glu_clamped;
// w_gate_up = [E][2 inter][K].  fllm_experts_down: out[pair] = w_down[e] act[pair], float32; w_down = [E][N][inter].
// score_mode 1: the score is the softmax of the logits over all experts; renormalize: the picks' weights are divided by their
// sum (+ 1e-20); route_scale multiplies them.
int fllm_route_topk(const void *h, int ldh, const void *w_router, int rows, int K, int E, int top, int32_t *ids, float *weights,
                    int score_mode, int renormalize, float route_scale, int dtype, hipStream_t stream);
int fllm_experts_gate_up(const void *h, int ldh, const int32_t *ids, const float *weights, int rows, int top, const void *w_gate_up,
                         int E, int inter, int K, void *act, float limit, float alpha, float up_offset, int dtype, hipStream_t stream);
int fllm_experts_down(const void *act, const int32_t *ids, int pairs, const void *w_down, int E, int N, int inter, float *out, int dtype,
                      hipStream_t stream);
// The same products on the matrix cores (bfloat16): the pairs are grouped by expert on the device and multiplied as tiles of
// 64 or 128 rows.  0: launched; 1: shape declined (the caller runs the plain kernels).  act and xs: scratch, bfloat16
// [rows * top, inter] and [rows * top, K]; out: float32 [rows * top, N]; work: fllm_experts_grouped_work_ints(rows * top, E)
// int32 of scratch.
size_t fllm_experts_grouped_work_ints(int pairs, int E);
size_t fllm_experts_grouped_plane_floats(int pairs, int E, int N, int inter);   // `planes`: float32 scratch of that many (0: none)
int fllm_experts_grouped(const void *h, int ldh, const int32_t *ids, const float *weights, int rows, int top, const void *w_gate_up,
                         const void *w_down, int E, int inter, int K, int N, void *act, void *xs, float *out, int32_t *work,
                         float *planes, float limit, float alpha, float up_offset, hipStream_t stream);

// ---- mechanisms that carry something from token to token outside the pages (sequence_ops.hip) --------------------------------
// Rows, segments and slots as in fllm_attention: rows of a segment are consecutive, seg_start[s] is its first row, slots[s] the
// state slot of its request; rows with row_seg < 0 are padding (outputs zero, no state touched).  A segment's rows continue
// the state that the request's slot holds.
// fllm_short_conv: out[t] = x[t] + sum_j w[c][j] x[t - taps + 1 + j] on every channel c (w float32 [width][taps]); the inputs
// before a step's first row come from state [slots][taps - 1][width] (of `dtype`, zeros at a sequence's start), which
// afterwards holds the last taps - 1 inputs of the sequence.
int fllm_short_conv(const void *x, const float *w, void *state, const int32_t *row_seg, const int32_t *seg_start,
                    const int32_t *slots, int num_segs, void *out, int rows, int width, int taps, int dtype, hipStream_t stream);
// The same behind a norm with one weight vector, for steps of one row a segment: h = x * rsqrt(mean x^2 + eps) * norm_w is
// computed from the float32 stream x, convolved with the state's inputs, and h takes its place in the state.
int fllm_norm_short_conv(const float *x, const float *norm_w, float eps, const float *w, void *state, const int32_t *row_seg,
                         const int32_t *slots, void *out, int rows, int width, int taps, int dtype, hipStream_t stream);
// fllm_linear_attention: per head S <- decay_h S + k_t v_t^T, o_t = S^T q_t, token after token; S float32
// state[slots][heads][dim][vdim].  q, k (heads * dim) and v (heads * vdim) are columns of rows of `ld` elements of `dtype`;
// activation 1 applies silu to all three on the way in (0: none).  decay_h = decay_hi[h] + decay_lo[h] (a float pair, so that
// the power over many tokens is that of the number itself and not of its rounding).  out float32 [rows, heads * vdim].
// form 0: steps with more rows than segments (portions of prompts) run chunks of 32 tokens on the matrix cores in float32 where
// the sizes allow (dim a multiple of 16 up to 128, vdim a multiple of 16), all others token after token; 1: token after token;
// 2: chunks, an error where the sizes do not allow them.  `carried` (null, or fllm_linear_attention_carried_floats floats):
// with it, the chunked form cuts the segments of a step of 512 rows or more into parts of 256 tokens that run side by side,
// each from zeros, and a second kernel hands the states from part to part and adds what the tokens of a part lack.
int fllm_linear_attention(const void *q, const void *k, const void *v, int ld, const float *decay_hi, const float *decay_lo,
                          float *state, const int32_t *row_seg, const int32_t *seg_start, const int32_t *slots, int num_segs,
                          float *out, int rows, int heads, int dim, int vdim, int activation, int form, int dtype,
                          float *carried, hipStream_t stream);
size_t fllm_linear_attention_carried_floats(int rows, int num_segs, int heads, int dim, int vdim);
// out = x * rsqrt(mean x^2 + eps) * w * sigmoid(gate) over rows of `width` (w null: out = x * sigmoid(gate)); x float32 or of
// `dtype`, gate rows of gate_ld elements and out of `dtype`.
int fllm_gated_norm(const void *x, int x_dtype, const float *w, float eps, const void *gate, int gate_ld, void *out, int rows,
                    int width, int dtype, hipStream_t stream);
// out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, powers lane by lane, N the division of a row by its root mean square (eps inside
// the root); coeffs float32 [4] on the device.
int fllm_polynorm(const void *z, int ld, const float *coeffs, float eps, void *out, int rows, int width, int dtype, hipStream_t stream);
// Rows [q | k | v | ..] of `ld` elements: every head of q and k is divided by its root mean square over `norm_dim` lanes (heads
// widened with zero lanes keep the mean of their own lanes), in place for q; k and v go into the pages of the row's request
// (store_kv 0: q alone is normed, nothing is stored).
int fllm_head_norm_kv_store(void *qkv, int ld, float eps, int norm_dim, const int32_t *row_pos, const int32_t *row_seg,
                            const int32_t *tables, int table_stride, void *k_pages, void *v_pages, int rows, int heads, int kv_heads,
                            int head_dim, int v_dim, int page_size, int key_chunk, int dtype, int store_kv, hipStream_t stream);

// ---- mixers beside the softmax attention over all keys (mixer_variants.hip) ----
// Rows of a joint product [q | k | v | ..]: norm_mode 0 none, 1 an RMS norm of every head of q and of k over its own lanes with
// one weight vector [k_dim] for all heads, 2 an RMS norm over the whole query projection and over the whole key projection
// with weights of those sizes; rotary on the first rope_dims lanes of every head (lane i with lane i + rope_dims / 2);
// queries to q_out, keys and values into the pages.  values_from_keys: the values are the keys as projected and the rows
// hold no value columns.
int fllm_normed_rope_store(const void *qkv, int ld, int norm_mode, const float *q_weight, const float *k_weight, float eps, void *q_out,
                           const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables, int table_stride,
                           const float *cos_table, const float *sin_table, int table_positions, void *k_pages, void *v_pages, int rows,
                           int heads, int kv_heads, int k_dim, int v_dim, int rope_dims, int page_size, int key_chunk, int dtype,
                           int store_kv, int values_from_keys, hipStream_t stream);
// For every row whose position ends a block of `pool` positions: the float32 means of the block's keys and values, read from
// the pages, into pool_k / pool_v [page][kv_head][ceil(page_size / pool)][k_dim or v_dim] at the page of the block's last token,
// slot (that token's place in the page) / pool.
int fllm_pool_blocks(const void *k_pages, const void *v_pages, float *pool_k, float *pool_v, const int32_t *tables, int table_stride,
                     const int32_t *row_pos, const int32_t *row_seg, int rows, int kv_heads, int k_dim, int v_dim, int page_size,
                     int key_chunk, int pool, int dtype, hipStream_t stream);
// A row at position p sees the tokens max(0, p - window + 1) .. p and one mean key and value for every block b of `pool`
// positions with b * pool + pool - 1 <= p - window; one softmax over both.
int fllm_pooled_window_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const float *pool_k,
                                 const float *pool_v, const int32_t *tables, int table_stride, const int32_t *row_pos,
                                 const int32_t *row_seg, const int32_t *seg_start, int num_segs, void *out, int rows, int heads,
                                 int kv_heads, int head_dim, int v_dim, int page_size, float scale, int window, int pool, int key_chunk,
                                 int dtype, int max_context, hipStream_t stream);
// out[h] = sum over the keys j <= p of sigmoid(cap * tanh(s / cap) - r1[h] * ln(1 + r2[h] * (p - j)) + pb[h]) * v_j with
// s = q . k_j * scale * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)).  max_context bounds position + 1 over the rows (0:
// unknown); steps of single rows with long contexts share a row's keys among workgroups by it.
int fllm_sigmoid_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables, int table_stride,
                           const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start, int num_segs, void *out, int rows,
                           int heads, int kv_heads, int head_dim,
                           int v_dim, int page_size, float scale, float softcap, const float *r1, const float *r2, const float *pb,
                           float temp_coef, int temp_every, int key_chunk, int dtype, int max_context, hipStream_t stream);
// Rows [q | k | v | ..] (heads * dim, heads * dim, heads * vdim) -> float32 rows [q | k | v]: q and k rotated on the first
// rope_dims lanes of every head at the row's position, k times key_scale, v as it is.
int fllm_rotate_scale(const void *qkv, int ld, float *out, const int32_t *row_pos, const float *cos_table, const float *sin_table,
                      int table_positions, int rows, int heads, int dim, int vdim, int rope_dims, float key_scale, int dtype,
                      hipStream_t stream);
// out = x / rms(x over each group of `group` lanes) * act(gate), act silu or sigmoid; x float32 or of `dtype`.
int fllm_group_norm_gate(const void *x, int x_dtype, float eps, int group, const void *gate, int gate_ld, void *out, int rows, int width,
                         int silu, int dtype, hipStream_t stream);
// out = a x + b y (accumulate: out += a x + b y), float32.
int fllm_weighted_sum(float *out, const float *x, float a, const float *y, float b, size_t total, int accumulate, hipStream_t stream);
// out[r] = [x[r] | table[ids[r]] * scale] in `dtype` (x float32, table of `dtype`), rows of 2 * width.
int fllm_stream_concat(const float *x, const int32_t *ids, const void *table, int vocab, float scale, void *out, int rows, int width,
                       int dtype, hipStream_t stream);
// out = relu(x)^2, element by element (out may be x).
int fllm_relu_squared(const void *x, void *out, size_t total, int dtype, hipStream_t stream);
// Router with corrections and groups, and the up product of experts without a gate (routed_experts.hip).
int fllm_route_grouped(const void *h, int ldh, const void *w_router, const float *correction, int rows, int K, int E, int top, int groups,
                       int kept, int32_t *ids, float *weights, float route_scale, int dtype, hipStream_t stream);
int fllm_experts_up(const void *h, int ldh, const int32_t *ids, int rows, int top, const void *w_up, int E, int inter, int K, void *act,
                    int dtype, hipStream_t stream);
// Experts without a gate on the matrix cores: pairs grouped by expert, act = relu(W_up[e] h)^2, out = W_down[e] act (float32
// [rows * top, N]); scratch as for fllm_experts_grouped (no scaled rows).  1: shape declined.
int fllm_experts_grouped_ungated(const void *h, int ldh, const int32_t *ids, int rows, int top, const void *w_up, const void *w_down,
                                 int E, int inter, int K, int N, void *act, float *out, int32_t *work, float *planes,
                                 hipStream_t stream);

#ifdef __cplusplus
}
#endif
