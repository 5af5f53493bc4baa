// The C interface of the kernel library.  Every function launches on the given
// stream, returns 0 on success and otherwise leaves a message for
// hal_last_error().  Pointers are device pointers unless a comment says otherwise;
// dtype codes are HAL_F32 = 0 and HAL_BF16 = 1.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* hal_last_error();
int hal_version();

int hal_embedding(const int* ids, const void* table, int table_dtype, float* out, int n_tokens,
                  int d, int vocab, hipStream_t stream);

// hal_embedding with every row multiplied by `scale` in float32.
int hal_embedding_scaled(const int* ids, const void* table, int table_dtype, float* out,
                         int n_tokens, int d, int vocab, float scale, hipStream_t stream);

int hal_take_tokens(const int* src, int n_src, int* tokens, int n, hipStream_t stream);

int hal_rmsnorm(float* h, const void* delta, const int* rows, const void* w, int w_dtype,
                float eps, void* out, int dtype, int n_rows, int d, int update_h,
                hipStream_t stream);

int hal_residual_add(float* h, const void* delta, int dtype, long long n, hipStream_t stream);

int hal_silu_mul(const void* gu, void* out, int dtype, int n_tokens, int F, hipStream_t stream);

// out [m, d] = bf16(x * rsqrt(sum_p ss[p][row] / d + eps)): the rows of an RMSNorm whose
// scaling was left to the reader (x = bf16(w * bf16(h)), ss [n_parts, row_width] partial
// sums of h^2), for a reader that does not scale by itself.
int hal_scale_normed_rows(const void* x, int ldx, const float* ss, int n_parts, int row_width,
                          float eps, void* out, int m, int d, hipStream_t stream);

int hal_rope_append(void* qkv, int dtype, int row_stride, const int* positions,
                    const int* token_seg, const int* block_table, int bt_stride,
                    const float* cos_t, const float* sin_t, int table_len, void* k_pages,
                    void* v_pages, int n_tokens, int H, int K, int D, int rot, int interleaved,
                    int page_size, int n_pages, int tiled, hipStream_t stream);

// `max_kv_len`: no request of the step has more keys (an upper bound will do); `min_q_len`:
// none has fewer tokens in the step (a lower bound will do, 1 if not known).  They decide how
// the step is cut, never a result.  `hal_attention_simple_plan` says how; if `split`, `part`
// must bring `part_floats` floats for the pieces' partial sums.
int hal_attention_simple_plan(int n_tokens, int H, int K, int D, int max_kv_len, int min_q_len, int* tq,
                              int* split, int* rows_per_wave, int* max_pieces, long long* part_floats);
int hal_attention_simple(const void* q, int q_row_stride, void* out, int out_row_stride,
                         int dtype, const int* positions, const int* token_seg,
                         const int* block_table, int bt_stride, const void* k_pages,
                         const void* v_pages, float* part, int n_tokens, int H, int K, int D,
                         int page_size, int n_pages, float scale, int window, int max_kv_len,
                         int min_q_len, hipStream_t stream);

// hal_attention_simple with a rule for the scores: `chunk` > 0: a query sees no key before
// the start of its own chunk of that many positions; `bias` (or null): float32
// [H][bias_len], added to the scaled score of the key n tokens back at
// [head][min(n, bias_len - 1)]; `sink`: one more term of score 0 and no value in the softmax
// (`sink_value`, or null: float32 [H], that term's score per head instead of 0); `softcap` > 0:
// the scaled score s becomes softcap * tanh(s / softcap) before the bias.
int hal_attention_simple_ruled(const void* q, int q_row_stride, void* out, int out_row_stride,
                               int dtype, const int* positions, const int* token_seg,
                               const int* block_table, int bt_stride, const void* k_pages,
                               const void* v_pages, float* part, int n_tokens, int H, int K, int D,
                               int page_size, int n_pages, float scale, int window, int chunk,
                               const float* bias, int bias_len, int sink, float softcap,
                               const float* sink_value, int max_kv_len, int min_q_len,
                               hipStream_t stream);

int hal_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M,
                 int N, int K, hipStream_t stream);

// X [M <= 64, K] bf16, W [N, K] bf16, optional W2 [N, K] (gated: up * silu(gate), W the gate).
// out_mode: 0 bf16, 1 float32, 2 add into float32, 3 bf16 of the square of relu of the result.
int hal_gemm_bf16_skinny(const void* X, int ldx, const void* W, const void* W2, int ldw, void* C,
                         int ldc, int out_mode, int M, int N, int K, hipStream_t stream);

// The packed q, k, v projection of M <= 32 tokens with the rotation of q and k (pairs
// (j, j + D/2), whole head) and the append of k and v to the pages in its epilogue.  W:
// the weight's rows reordered per head to [8j .. 8j+7, D/2 + 8j .. D/2 + 8j+7] for
// j = 0 .. D/16 - 1, then tiled as for ldw == 0 above.  q_out [M, H * D] bf16.  ss_in (or
// null), n_parts, eps: the norm before the projection, as for hal_gemm_bf16_skinny_norm.
int hal_qkv_rope_append(const void* X, int ldx, const void* W, void* q_out, int M, int K_in,
                        const int* positions, const int* token_seg, const int* block_table,
                        int bt_stride, const float* cos_t, const float* sin_t, int table_len,
                        void* k_pages, void* v_pages, int H, int K, int D, int page_size,
                        int n_pages, int tiled, const float* ss_in, int n_parts, float eps,
                        hipStream_t stream);

// The product for M <= 32 rows with the RMSNorm before it (ss_in: partial sums of squares
// [n_parts, 16] (32 for more than 16 rows) left by the product before; X holds
// bf16(w * bf16(h))) or after it (norm_w: C is the float32 stream h, added into; xw_out [M, N]
// and ss_out [ceil(N/16), 16 or 32] are left for the product after) folded in.
int hal_gemm_bf16_skinny_norm(const void* X, int ldx, const void* W, const void* W2, int ldw,
                              void* C, int ldc, int M, int N, int K, const float* ss_in,
                              int n_parts, float eps, const void* norm_w, int norm_w_dtype,
                              void* xw_out, float* ss_out, hipStream_t stream);

int hal_sample(const float* logits, int ld, int n_rows, int V, const float* temperature,
               const int* top_k, const float* top_p, const float* min_p, const uint64_t* seeds,
               const int* draw_index, int* out_token, float* out_logprob, uint32_t* key_rows,
               hipStream_t stream);

// Greedy decoding of every row, each row spread over 32 blocks.  `parts`: n_rows * 32 * 4 floats.
int hal_sample_greedy(const float* logits, int ld, int n_rows, int V, float* parts,
                      int* out_token, float* out_logprob, hipStream_t stream);

// hal_sample_greedy without any allocation.  This entry point has no counterpart in the
// reference.  It is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  The partial results go
// to an array that the library holds on every GPU it runs on (512 KiB, there until the
// process ends) instead of to `parts`; at most hal_sample_greedy_static_max_rows() (1024)
// rows, more are refused.  It calls no hipMalloc, hipFree or allocating routine.  All calls
// on one GPU share that array: calls that may overlap there (other streams, other host
// threads) race; calls on one stream do not.
int hal_sample_greedy_static_max_rows();
int hal_sample_greedy_static(const float* logits, int ld, int n_rows, int V, int* out_token,
                             float* out_logprob, hipStream_t stream);

// Rows without filters, greedy or drawn from the whole temperature-scaled distribution; each
// row is spread over 32 blocks.  `parts`: room for n_rows * 32 * 4 floats.
int hal_sample_unfiltered(const float* logits, int ld, int n_rows, int V, const float* temperature,
                          const int* top_k, const uint64_t* seeds, const int* draw_index,
                          float* parts, int* out_token, float* out_logprob, hipStream_t stream);

// Rows with filters spread over 32 blocks a pass.  any_late: some row has top-k, top-p and
// min-p all at once (searched twice).  parts: n_rows * 32 * 4 floats; kept: n_rows * 32
// floats; state: n_rows * 20 words; hist: n_rows * 2 * 2048 64-bit words.
int hal_sample_spread(const float* logits, int ld, int n_rows, int V, const float* temperature,
                      const int* top_k, const float* top_p, const float* min_p,
                      const uint64_t* seeds, const int* draw_index, float* parts, float* kept,
                      void* state, void* hist, int any_late, int* out_token, float* out_logprob,
                      hipStream_t stream);

// ---- products in groups (grouped_gemm.hip) ---------------------------------------------
// Y_g = X_g * W_g^T for G groups in one launch, float32 accumulation; operands of `dtype`.
// Group g reads the columns from g * x_group_cols + x_col0 of X's rows (row length ldx) and
// W + g * w_group_stride ([N, K], row length ldw), and writes the columns from
// g * y_group_cols + y_col0 of Y's rows (row length ldy, element type y_dtype; y_add: added
// into a float32 Y).  group_offsets == null: every group has the rows 0 .. M-1.  Otherwise
// group g has the rows group_offsets[g] .. group_offsets[g + 1] - 1 of a list of M rows in
// all (tile_offsets: the same counted in tiles of 128 rows, each group rounded up; both
// [G + 1] on the device): row i of the list reads row row_src[i] / src_div of X (i if null)
// and writes row row_dst[i] of Y (i if null).  W2 != null: two products and the clamped
// gated activation g = min(x W^T, limit), u = clamp(x W2^T, -limit, limit),
// y = g * sigmoid(alpha * g) * (u + 1).  gate != null (float32 rows of length ldg): the
// result is multiplied by sigmoid(gate[row, g * y_group_cols + n]).  act (W2 null): 0 the
// product as it is, 1 the square of its positive part.
int hal_grouped_gemm(const void* X, int ldx, int x_group_cols, int x_col0, const void* W,
                     const void* W2, long long w_group_stride, int ldw, int dtype, void* Y, int ldy,
                     int y_group_cols, int y_col0, int y_dtype, int y_add, int M, int N, int K,
                     int G, const int* group_offsets, const int* tile_offsets, const int* row_src,
                     int src_div, const int* row_dst, const float* gate, int ldg, int gate_per_group,
                     float limit, float up_shift, float alpha, int act, int allow_mfma,
                     hipStream_t stream);

// ---- around a latent attention and a mixture of experts (latent_moe.hip) -----------------
// RMSNorm of rows of the float32 stream (rows[r] or r) with one or two weights, x * rstd * w
// in float32, rounded once.
int hal_norm_pair(const float* h, const int* rows, const void* w1, const void* w2, int w_dtype,
                  float eps, void* out1, void* out2, int dtype, int n_rows, int d,
                  hipStream_t stream);
// From the float32 down projections of a latent attention (a [T, lda]: query latent of q_rank
// columns from q_col0, none if q_rank == 0; key/value latent of kv_rank columns from kv_col0
// followed by `rot` shared rotated-key columns): cq [T, q_rank] = the normed query latent,
// and in the packed rows qkv (row length row_stride) the key row [rot | normed latent | 0]
// at column k_col0 and the value row [0 | normed latent | 0] at k_col0 + D, D columns each.
int hal_latent_prep(const float* a, int lda, int q_col0, int q_rank, int kv_col0, int kv_rank,
                    int rot, int D, const void* wq, const void* wkv, int w_dtype, float eps,
                    void* cq, void* qkv, int row_stride, int k_col0, int dtype, int n_tokens,
                    hipStream_t stream);
// y[t, h * ys + y0 + j] = x[t, h * xs + x0 + j] (j < n) and zero in the n_zero columns from
// h * ys + z0, for H heads.
int hal_head_cols(const void* x, int ldx, int xs, int x0, void* y, int ldy, int ys, int y0, int n,
                  int z0, int n_zero, int H, int dtype, int n_tokens, hipStream_t stream);
int hal_scale_f32(float* x, long long n, float s, hipStream_t stream);
// Router of a mixture of experts on float32 logits z [T, E]: scores by sigmoid (softmax over
// the experts if `softmax`), the `top` largest (lower index on a tie) to idx [T, top], their
// scores (divided by their sum + norm_eps if `normalize`) to wgt [T, top].
int hal_moe_route(const float* z, int ldz, int E, int top, int softmax, int normalize, float norm_eps,
                  int* idx, float* wgt, int n_tokens, hipStream_t stream);
// Counting sort of the n (token, choice) pairs by expert (idx [n]); offsets, tile_offsets
// [E + 1] and sorted [n] as hal_grouped_gemm takes them (tiles of `tile` rows).
int hal_moe_sort(const int* idx, int n, int E, int tile, int* offsets, int* tile_offsets,
                 int* sorted, hipStream_t stream);
// h[t] += sum_j wgt[t, j] * y[t * top + j] (+ extra[t] if given, times sigmoid(extra_gate[t *
// ld_gate]) if that is given)  (h, extra [T, d] and y [T * top, d] float32); overwrite: h[t] = the sum
int hal_moe_combine(float* h, const float* y, const float* wgt, const float* extra,
                    const float* extra_gate, int ld_gate, int top, int d, int n_tokens, int overwrite,
                    hipStream_t stream);
// hal_moe_route and hal_moe_sort in one workgroup (for steps of few tokens)
int hal_moe_route_sort(const float* z, int ldz, int E, int top, int softmax, int normalize, float norm_eps,
                       int* idx, float* wgt, int n_tokens, int tile, int* offsets, int* tile_offsets,
                       int* sorted, hipStream_t stream);

// out [T, F] = g * sigmoid(alpha * g) * (u + up_shift), g = min(gu[t, f], limit), u = clamp(gu[t, F + f],
// -limit, limit), for rows gu [T, 2F] that hold a gate projection and an up projection.
int hal_clamped_gate_mul(const void* gu, void* out, int dtype, int n_tokens, int F, float limit,
                         float alpha, float up_shift, hipStream_t stream);

// ---- rows of the stream and of projections (stream_ops.hip) -------------------------------
// out = T(h), n elements
int hal_cast_rows(const float* h, void* out, int dtype, long long n, hipStream_t stream);
// h[r] += x * rsqrt(mean(x^2) + eps) * w with x = s1 * a[r] (+ s2 * a2[r] if a2 is given);
// float32 h, a and a2, [n_rows, d]; cast (or null) receives the new rows of h rounded to `dtype`.
int hal_post_norm_add(float* h, const float* a, const float* a2, float s1, float s2, const void* w,
                      int w_dtype, float eps, void* cast, int dtype, int n_rows, int d,
                      hipStream_t stream);
int hal_relu_squared(const void* x, void* out, int dtype, long long n, hipStream_t stream);
// y = alpha * y + beta * x
int hal_scaled_sum_f32(float* y, float alpha, const float* x, float beta, long long n,
                       hipStream_t stream);
// From float32 projections q [T, H * dq], k [T, K * dq] and v [T, K * dv] (null: the values
// are the rows of k as they are; row lengths ldq, ldk, ldv): q and k each divided by the root
// mean square of their whole row and multiplied by wq, wk; q further by
// 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1) if temp_every > 0; written as
// packed rows [H heads | K key heads | K value heads] of D entries a head (the rest zero).
// With k_pages (not null): keys and values are appended to the pages as well, as
// hal_rope_append does it (for an attention that does not rotate).
int hal_qk_norm_pack(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                     const void* wq, const void* wk, int w_dtype, float eps, const int* positions,
                     float temp_coef, int temp_every, void* out, int row_stride, int dtype,
                     int n_tokens, int H, int K, int dq, int dv, int D, const int* token_seg,
                     const int* block_table, int bt_stride, void* k_pages, void* v_pages,
                     int page_size, int n_pages, int tiled, hipStream_t stream);

// ---- mixers with a carried state (recurrent.hip) -----------------------------------------
// y[t, c] = act(bias[c] + sum_j w[c, j] * u[t - taps + 1 + j, c]) over the tokens of each
// request, the inputs before a step's first token taken from state [slots][taps - 1][C]
// (float32; zero for a new request).  act: 0 none, 1 silu.  w [C, taps], bias [C] or null.
// in_bias (or null; here and in the two entry points below): [C], added to every input u[t, c]
// where it is read (not to the zeros before a request's first token)
int hal_short_conv(const float* u, int ldu, const void* w, const void* bias, int w_dtype,
                   const void* in_bias, int ib_dtype, int taps,
                   const float* state, const int* token_seg, const int* seg_q_start,
                   const int* token_slot, void* y, int ldy, int y_dtype, int act, int n_tokens,
                   int C, hipStream_t stream);
// Both in one kernel for a step in which every request brings one token (token t belongs to
// slot token_slot[t], no two tokens to the same): y as above, and the state moved one on.
int hal_short_conv_step(const float* u, int ldu, const void* w, const void* bias, int w_dtype,
                        const void* in_bias, int ib_dtype, int taps, float* state, const int* token_slot, void* y, int ldy,
                        int y_dtype, int act, int n_tokens, int C, hipStream_t stream);
// The state after the step: the last taps - 1 of (the state, then the step's inputs).
int hal_short_conv_carry(const float* u, int ldu, const void* in_bias, int ib_dtype, float* state, int taps,
                         const int* seg_q_start,
                         const int* seg_q_len, const int* token_slot, int n_segs, int C,
                         hipStream_t stream);
// xbc [T, ldx]: x (heads * P), then B and C (groups * N each).  state [slots][heads][N][P].
// y [T, heads * P] float32 = S_t^T C_t + D x_t.  chunks [n_chunks][4] (first token, tokens,
// segment, 0), seg_chunks [segments][2] (first chunk, chunks), sums (n_chunks * heads * N * P
// floats) and decays (n_chunks * heads floats): the segments cut into chunks that are walked
// side by side, or all null: a wave walks a whole segment.  fixed_decay (or null): float32
// [heads], one constant decay a head with step sizes of 1 and no D: S <- decay S + B x^T.
// in_silu: x, B and C are SiLU of what xbc holds.
int hal_ssd_scan(const void* xbc, int ldx, int dtype, const float* dt_raw, int ld_dt,
                 const void* dt_bias, const void* a_log, const void* d_skip, int w_dtype,
                 float* state, const int* seg_q_start, const int* seg_q_len, const int* token_slot,
                 float* y, int n_segs, int heads, int P, int N, int groups, const int* chunks,
                 const int* seg_chunks, int n_chunks, float* sums, float* decays,
                 const float* fixed_decay, int in_silu, hipStream_t stream);
// out = (y * silu(z)) / rms over each of `parts` equal parts of the row * w
int hal_gated_part_norm(const float* y, const float* z, int ldz, const void* w, int w_dtype,
                        float eps, void* out, int dtype, int n_tokens, int inner, int parts,
                        hipStream_t stream);

// ---- the generalized delta rule (delta_rule.hip) ------------------------------------------
// S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t per head,
// with w = exp(-decay_rate * sigmoid(w0 + W2 tanh(x1))), a = sigmoid(a_raw + a_bias) and
// u = k / sqrt(sum(k^2) + unit_eps).  r, k, v, a_raw: float32 [T, H * D] (row lengths given),
// x1 float32 [T, lora]; w2 [H * D, lora], w0 and a_bias [H * D] of element type w_dtype; state
// float32 [slots][H][D][D], read and left as the step's last state; pre: scratch of
// T * H * 5 * DP floats (DP: D rounded up to 16, 32, 64, 128 or 256); o float32 [T, H * D].
int hal_delta_rule(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv,
                   const float* a_raw, int lda, const float* x1, int ldx1, const void* w2,
                   const void* w0, const void* a_bias, int w_dtype, int lora, float decay_rate,
                   float unit_eps, float* pre, float* state, const int* seg_q_start,
                   const int* seg_q_len, const int* token_slot, float* o, int n_tokens, int n_segs,
                   int H, int D, hipStream_t stream);
// out = y / rms(y over each head of D) * w * sigmoid(z)  (w, z: null for none)
int hal_head_norm_gate(const float* y, const float* z, int ldz, const void* w, int w_dtype, float eps,
                       void* out, int dtype, int n_tokens, int H, int D, hipStream_t stream);

// ---- several copies of the residual stream, per-head norms, per-head gates (stream_ops.hip) --
// x float32 [S][rows][W] (copy_stride elements between copies).  With y (float32 [rows][W]):
// x_t <- sum_s mix[s][t] x_s + m * out[t] * y for every copy t, from the old copies.  With
// read: u = sum_s in[s] x_s (in null: ones) of the new copies, written to result as it is
// (norm_w null, float32) or as u / sqrt(mean(u^2) + eps) * (offset + norm_w).  rows (or null;
// only without y): the rows to take, results in that order.
int hal_streams_step(float* x, long long copy_stride, int S, const float* y, const void* mix,
                     const void* outw, float m, const void* inw, int c_dtype, int read,
                     const void* norm_w, int norm_dtype, float offset, float eps, void* result,
                     int result_dtype, const int* rows, int n_rows, int W, hipStream_t stream);
// Every head of float32 q [T, H * dq], k [T, K * dq], v [T, K * dv] divided by its own root
// mean square, packed as hal_qk_norm_pack packs (and appended to the pages, if given).
// w_q, w_k (or null): a weight [dq] for every normed head of q / k; norm_v 0: the values are not
// divided; v_other (or null): the values become (1 - v_mix) v + v_mix v_other.
int hal_head_norm_pack(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, float eps,
                       const void* w_q, const void* w_k, int w_dtype, int norm_v, const float* v_other,
                       int ldvo, float v_mix, const int* positions, void* out, int row_stride, int dtype, int n_tokens, int H,
                       int K, int dq, int dv, int D, const int* token_seg, const int* block_table,
                       int bt_stride, void* k_pages, void* v_pages, int page_size, int n_pages, int tiled,
                       hipStream_t stream);
// a[t, c] += bias[c] (float32 rows, in place)
int hal_bias_rows(float* a, int lda, const void* bias, int b_dtype, int n_rows, int n_cols, hipStream_t stream);
// out[t, c] = silu(a[t, c]) for the first n_cols columns of float32 rows
int hal_silu_rows(const float* a, int lda, void* out, int dtype, int n_rows, int n_cols, hipStream_t stream);
// out[t, j] = gelu_tanh(g[t, j]) * table[tokens[t]][col0 + j], j < dim (a token out of range: NaN)
int hal_token_gate(const float* g, int ldg, const void* table, int t_dtype, int ld_table, int col0,
                   const int* tokens, int vocab, void* out, int dtype, int n_rows, int dim, hipStream_t stream);
// y[t, h * n + j] = x[t, h * x_head + j] * sigmoid(g[t, h]), j < n
int hal_head_gate_cols(const void* x, int ldx, int x_head, const float* g, int ldg, void* y, int n, int H,
                       int dtype, int n_tokens, hipStream_t stream);

// ---- the head-size-specific library (attention_mfma.hip) ---------------------------------
int hal_attention_mfma_head_dim();
int hal_attention_mfma_rows_per_big_item();
// merge_parts: the most partial results that any merge item joins, or 0 if not known (the
// kernel for many partials is taken then).  Items of both lists come in runs of four, a
// workgroup's waves (max_items and max_big are multiples of four): the one-tile items of a
// run are four pieces of one piece of a tile's key range (the last may be empty), whose sums
// the kernel joins itself, into the output or the run's partial slot.  counters: zeroed
// ints (left zeroed), one per (partial slot, kv head), for the one-tile items that ask the
// kernel to merge their tile's partial results itself; null if none does.
int hal_attention_mfma(const void* q, int q_row_stride, void* out, int out_row_stride,
                       const int* items, int max_items, const int* big_items, int max_big,
                       const int* merges, int max_merges, const int* counts,
                       const int* seg_q_start, const int* seg_q_len, const int* seg_kv_len,
                       const int* block_table, int bt_stride, const void* k_pages,
                       const void* v_pages, float* part_o, float* part_ml, int* counters,
                       int n_counters, int H, int K, int head_dim, int page_size, int tiled,
                       float scale, int window, int merge_parts, hipStream_t stream);

// hal_attention_mfma with a rule for the scores (see hal_attention_simple_ruled); the bias
// table and the sinks' values come multiplied by log2 e, and the work lists are cut for the chunk.
int hal_attention_mfma_ruled(const void* q, int q_row_stride, void* out, int out_row_stride,
                             const int* items, int max_items, const int* big_items, int max_big,
                             const int* merges, int max_merges, const int* counts,
                             const int* seg_q_start, const int* seg_q_len, const int* seg_kv_len,
                             const int* block_table, int bt_stride, const void* k_pages,
                             const void* v_pages, float* part_o, float* part_ml, int* counters,
                             int n_counters, int H, int K, int head_dim, int page_size, int tiled,
                             float scale, int window, int chunk, const float* bias_log2,
                             int bias_len, int sink, float softcap, const float* sink_log2,
                             int merge_parts, hipStream_t stream);

}  // extern "C"
