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
// qkv: [rows, (heads + 2 kv_heads) * head_dim]; row r belongs to segment row_seg[r] at position
// row_pos[r]; its page is tables[row_seg[r] * table_stride + row_pos[r] / page_size].
// K pages: [page][kv_head][token][head_dim]; V pages: [page][kv_head][head_dim][token].
// pairing 0: lanes (l, l + rope_dims/2); 1: lanes (2l, 2l + 1).  store_kv 0 leaves the pages alone.
int fllm_rope_kv_store(void *qkv, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                       int table_stride, const float *cos_table, const float *sin_table, int table_positions,
                       void *k_pages, void *v_pages, int num_pages, int rows, int heads, int kv_heads, int head_dim,
                       int rope_dims, int pairing, int page_size, int dtype, int store_kv, hipStream_t stream);

// Causal attention of each row over the pages of its segment: keys at positions
// [max(0, pos - window + 1), pos] (window <= 0: from 0).  q: rows of `q_stride` elements, head h at
// h * head_dim.  out: [rows, heads * head_dim].  Rows of a segment are consecutive in the batch, at
// consecutive positions; seg_start[s] is the first row of segment s (seg_start[num_segs] = rows).
// `max_context` bounds pos + 1.  The segments from `single_from` on have one row each (0: every segment, a decode
// step; num_segs: none is known to): rows of long contexts among them are split over workgroups, which portions
// of prompts are not.  `workspace` holds partial results of split contexts (fllm_attention_workspace_bytes() of
// the number of single rows).
int fllm_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                   int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                   int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int page_size,
                   int num_pages, float scale, int window, int dtype, int max_context, int single_from,
                   void *workspace, size_t workspace_bytes, hipStream_t stream);
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

#ifdef __cplusplus
}
#endif
