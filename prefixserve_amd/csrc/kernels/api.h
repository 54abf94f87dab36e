// C interface of the kernel library (libpsamd_kernels.so). Every function launches on the
// given HIP stream, takes raw device pointers, returns 0 on success and otherwise leaves a
// message for psamd_last_error(). dtype codes: 0 = float32, 1 = bfloat16. Shapes are checked
// on the host before a launch; a shape a kernel does not take is an error, never a wrong
// result.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* psamd_last_error(void);

// out[t, :] = float(table[ids[t], :]); table is [vocab, hidden]; an id outside [0, vocab) reads the nearest row.
int psamd_embed(void* stream, const int32_t* ids, const void* table, int table_dtype, float* out, int64_t tokens,
                int hidden, int vocab);

// x = residual + delta, where delta is [rows, hidden] (delta_dtype) or n_partials float32 slices of that
// shape, partial_stride elements apart (the partial sums of a K-split product).
// rows == NULL: residual[r] = x[r], out[r] = weight * rmsnorm(x[r]) for r < out_rows.
// rows != NULL: out[i] = weight * rmsnorm(x[rows[i]]); residual untouched.
int psamd_add_rmsnorm(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                      int64_t partial_stride, const int32_t* rows, const void* weight, int weight_dtype, float eps,
                      void* out, int act_dtype, int64_t out_rows, int hidden);

// out[t, c] = act(gate_up[t, c]) * gate_up[t, inter + c]; gate: 0 = SiLU, 1 = ReLU, 2 = GELU (tanh form).
int psamd_swiglu(void* stream, const void* gate_up, void* out, int act_dtype, int64_t tokens, int inter, int gate);

// Rotates the q and k heads of qkv[t] in place by table[positions[t]] (NULL table: no rotation) and, if kv
// is given, writes k and v of token t to page slot write_slot[t] (= page * 16 + offset).
int psamd_rope_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                         const int32_t* positions, const float* table, void* kv, const int32_t* write_slot);

// The norm behind the sum: x = alpha * residual + delta (delta as for psamd_add_rmsnorm, or NULL),
// y = weight * rmsnorm(x) in float; residual[r] = y[r] and, if out is given, out[r] = y[r] in act_dtype.
int psamd_scaled_add_rmsnorm(void* stream, float* residual, float alpha, const void* delta, int delta_dtype,
                             int n_partials, int64_t partial_stride, const void* weight, int weight_dtype, float eps,
                             void* out, int act_dtype, int64_t rows, int hidden);

// out[i] = in[i] in act_dtype.
int psamd_to_activation(void* stream, const float* in, void* out, int act_dtype, int64_t n);

// psamd_rope_kv_append with a unit norm behind the rotation: every q and k head is divided by
// sqrt(sum of its squares / norm_dim + eps) (norm_dim 0: no norm; norm_dim < head_dim: the rest of
// the head's slots hold zeros). hkv may be 0: rows of queries alone.
int psamd_rope_norm_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                              const int32_t* positions, const float* table, int norm_dim, float eps, void* kv,
                              const int32_t* write_slot);

// The general form of psamd_rope_norm_kv_append. bias (float [(hq + hkv) * head_dim] or NULL) is added to
// the q and k heads first; q_weight / k_weight (float [head_dim] or NULL) multiply the heads behind the
// division by the root mean square; v_from_k: rows are [q heads | k heads] only and the value written
// to the pages is the k head as projected (with its bias, before rotation and norm).
int psamd_qk_prepare_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                               const int32_t* positions, const float* table, int norm_dim, float eps, const float* bias,
                               const float* q_weight, const float* k_weight, int v_from_k, void* kv,
                               const int32_t* write_slot, int q_weight_per_head);

// residual[r] += delta[r]; delta as for psamd_add_rmsnorm (one tensor in delta_dtype, or n_partials float32 slices).
int psamd_residual_add(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                       int64_t partial_stride, int64_t rows, int hidden);
// x[r, c] = x[r, c] * factor + row[c] (row may be NULL) on a float32 tensor [rows, hidden].
int psamd_stream_affine(void* stream, float* x, int64_t rows, int hidden, float factor, const float* row);
// out[r] = [a[r], b[r]] in act_dtype, a and b float32 [rows, hidden].
int psamd_concat_to_activation(void* stream, const float* a, const float* b, void* out, int act_dtype, int64_t rows,
                               int hidden);

// One small product per head: out[t, h, n] = sum_k x[t, h, k] * w[h, n, k], float accumulation. Row t of
// x starts at x + t * x_row, its head h at + h * x_head (elements), likewise out; w is [H, N, K], dense.
int psamd_heads_linear(void* stream, const void* x, int x_dtype, int64_t x_row, int x_head, const void* w, int w_dtype,
                       void* out, int out_dtype, int64_t out_row, int out_head, int64_t M, int H, int N, int K);

// Latent attention, one compressed vector per token. Row t of `in` is [hq heads x (dim + rot) | rank | rot]:
// the compressed part is divided by its root mean square (eps inside the root) and multiplied by norm_w
// (float [rank]), the shared key part and every head's last `rot` query dimensions are rotated pair by
// pair, (2i, 2i + 1) by table[positions[t]][i] = (cos, sin). The page of kv ([blocks, 2, 1, 16 * slots])
// gets the key [compressed | rotated part | zeros] and, transposed, the value [compressed | zeros];
// q_lat[t, h] (slots wide) gets the rotated query part at [rank, rank + rot) and zeros behind it, and
// is left alone in front: that is where the product of the head's other dimensions goes.
int psamd_latent_kv_append(void* stream, const void* in, int64_t in_row, void* q_lat, int act_dtype, int64_t tokens,
                           int hq, int dim, int rot, int rank, int slots, const int32_t* positions, const float* table,
                           const float* norm_w, float eps, void* kv, const int32_t* write_slot);

// A causal convolution per channel over each item's tokens, continued from the item's state:
// u[t, c] = conv_b[c] + sum_j conv_w[c, j] * v(t - (taps - 1) + j, c) with v(s, c) = in[s, c] + in_bias[c]
// for tokens of this step and the state's saved inputs (state[slot, (taps - 1) x width], oldest first)
// in front of the item's first token. `in` rows are in_row apart. u is float32. The state is only read.
int psamd_causal_conv(void* stream, const void* in, int act_dtype, int64_t in_row, const float* in_bias,
                      const float* conv_w, const float* conv_b, float* u, const float* state, int64_t state_row,
                      const int32_t* tok_item, const int32_t* item_start, const int32_t* slots, int64_t tokens,
                      int width, int taps);

// The gated linear recurrence over each item's tokens, state in 32-bit: with r = sigmoid(gates[t, b, c'] +
// gate_b), i = sigmoid(gates[t, b, bw + c'] + gate_b) (gates [tokens, blocks, 2 * bw], c = b * bw + c'),
// log a = decay[c] * r: S = a S + sqrt(1 - a^2) i u[t, c]; out[t, c] = S * gelu_tanh(y[t, c] + y_bias[c]).
// S lives in state[slot, (taps - 1) * width + c]; behind the scan the state's saved inputs become the
// item's last taps - 1 values of x[t, c] + x_bias[c]. tiles == NULL: every item token after token.
// Otherwise the step packer's lists: tiles[k] = (item, first token) of the n_tiles tiles of `tile` tokens
// that the items of more than one token are cut into (summed up tile by tile, then run side by side;
// carry: 3 * n_tiles * width floats), and singles: the n_singles items of one token.
int psamd_gated_scan(void* stream, const float* gates, const float* gate_b, const float* u, const float* decay,
                     const void* y, const void* x, int act_dtype, int64_t in_row, const float* y_bias,
                     const float* x_bias, void* out, float* state, int64_t state_row, const int32_t* item_start,
                     const int32_t* slots, int items, const int32_t* tiles, int n_tiles, int tile,
                     const int32_t* singles, int n_singles, float* carry, int width, int blocks, int taps);

// Mixture of experts. Router: z = x w_router^T in float (x in x_dtype, w_router float [E, K]), score =
// sigmoid(z); chosen[t, :] = the top largest scores' experts (lower index among equals, largest
// first), weight[t, :] = those scores. bias (float [experts] or NULL) is added to z first. mode 1: the
// choice is by z itself and the weights are the softmax over the chosen z alone.
int psamd_moe_route(void* stream, const void* x, int x_dtype, const float* w_router, int32_t* chosen, float* weight,
                    int64_t tokens, int K, int experts, int top, const float* bias, int mode);
// The same choice from logits that a product has written (float [tokens, experts]).
int psamd_moe_topk(void* stream, const float* logits, int32_t* chosen, float* weight, int64_t tokens, int experts,
                   int top, const float* bias, int mode);
// Experts, one (token, choice) pair at a time: h = weight[t, j] * x[t]; g = min(gate h, limit), u =
// clamp(up h, -limit, limit); act[t * top + j] = g * sigmoid(gate_alpha * g) * (u + up_shift);
// out[j][t] = down act (float). w_gate_up is [E, 2F, K] (gate rows, then up rows), w_down [E, K, F].
// weight_on_output: h = x[t] and out[j][t] = weight[t, j] * down act instead.
int psamd_moe_experts_rows(void* stream, const void* x, const int32_t* chosen, const float* weight,
                           const void* w_gate_up, const void* w_down, void* act, float* out, int dtype,
                           int64_t tokens, int K, int F, int experts, int top, float gate_alpha, float limit,
                           float up_shift, int weight_on_output);

// The same for bfloat16 with the pairs sorted by expert and every expert's pairs run through its
// matrices in tiles on the matrix cores. ints: scratch of pairs + 3 * psamd_moe_grouped_max_tiles(pairs,
// experts) integers (pairs = tokens * top). K and F multiples of 8.
int psamd_moe_grouped_tile_rows(int64_t pairs, int experts);
int psamd_moe_grouped_max_tiles(int64_t pairs, int experts);
int psamd_moe_experts_grouped(void* stream, const void* x, const int32_t* chosen, const float* weight,
                              const void* w_gate_up, const void* w_down, void* act, float* out, int32_t* ints,
                              int64_t tokens, int K, int F, int experts, int top, float gate_alpha, float limit,
                              float up_shift, int grouped_already, int weight_on_output);
// psamd_moe_topk and the sorting of the pairs into `ints` in one workgroup, for up to 64 tokens;
// psamd_moe_experts_grouped is then called with grouped_already = 1 and the same `ints`.
int psamd_moe_topk_group(void* stream, const float* logits, int32_t* chosen, float* weight, int32_t* ints, int64_t tokens,
                         int experts, int top, const float* bias, int mode);
// out[t, :] *= sigmoid(x[t] . w) for float out [tokens, out_hidden], x [tokens, hidden] in act_dtype, w float [hidden].
int psamd_row_gate(void* stream, float* out, const void* x, int act_dtype, const float* w, int64_t tokens, int out_hidden,
                   int hidden);

// Layer norm with weight and bias (float [hidden] each) around the float32 residual stream:
// if delta: residual[r] += LN_post(delta[r]) (delta as for psamd_add_rmsnorm); if out: out[r] = LN_pre(residual[r])
// in out_dtype. rows (NULL or int32 [n_rows], without a delta): out[i] = LN_pre(residual[rows[i]]).
int psamd_layernorm_step(void* stream, float* residual, const int32_t* rows, const void* delta, int delta_dtype,
                         int n_partials, int64_t partial_stride, const float* post_w, const float* post_b, float post_eps,
                         const float* pre_w, const float* pre_b, float pre_eps, void* out, int out_dtype, int64_t n_rows,
                         int hidden);
// x[t, e] += sin (e even) / cos (e odd) of positions[t] * freq[e / 2]; x float [tokens, hidden], freq double [(hidden + 1) / 2].
int psamd_add_sinusoid(void* stream, float* x, const int32_t* positions, const double* freq, int64_t tokens, int hidden);

// Short causal convolution per channel over each item's tokens: out[t, c] = act(sum_j taps_w[c, j] in[t - (taps - 1) + j, c]),
// continued in front of an item's first token from the inputs its state slot saved (state[slot, j * channels + c],
// oldest first), which are replaced by the item's last taps - 1 inputs. act 1 = SiLU, 0 = none. out is float.
int psamd_short_conv(void* stream, const void* in, int act_dtype, int64_t in_row, const float* taps_w, float* out,
                     int64_t out_row, float* state, int64_t state_row, const int32_t* tok_item, const int32_t* item_start,
                     const int32_t* slots, int64_t tokens, int items, int channels, int taps, int act);
// The same with a bias per channel (or NULL) added to the sum, an input of either type (in_dtype) whatever the output's,
// and the output in out_dtype.
int psamd_short_conv_to(void* stream, const void* in, int in_dtype, int64_t in_row, const float* taps_w, const float* bias,
                        void* out, int out_dtype, int64_t out_row, float* state, int64_t state_row, const int32_t* tok_item,
                        const int32_t* item_start, const int32_t* slots, int64_t tokens, int items, int channels, int taps,
                        int act);
// Operands of the gated delta rule: u row [q: groups x dim | k: groups x dim | ...] float, q and k made unit
// vectors in place (q times q_scale); gates row [strength logits | decay inputs] (heads each) -> coef row
// [g | -b | b]: b = sigmoid(.), g = exp(-exp(a_log[h]) softplus(. + dt_bias[h])).
int psamd_gated_delta_prepare(void* stream, float* u, int64_t u_row, int groups, int dim, const float* gates,
                              const float* a_log, const float* dt_bias, float* coef, int64_t tokens, int heads,
                              float q_scale, float unit_eps);
// Operands of the generalized delta rule from rows in act_dtype (r, k, v, removal logits: heads x dim at their
// columns; the decay's low-rank inner values: rank at l_col) -> ops row [r | k | v | w | p | c] float.
int psamd_general_delta_prepare(void* stream, const void* rows, int act_dtype, int64_t in_row, int r_col, int k_col,
                                int v_col, int a_col, int l_col, const float* a_bias, const float* w2, const float* w0,
                                float* ops, int64_t tokens, int heads, int dim, int rank, float decay_floor, float unit_eps);
// The delta-rule recurrence over each item's tokens from its state slot (state[slot, (h * vdim + j) * dim + i]):
// S' = d S; S = S' + (ps p)(c^T S*) + k (xs x)^T, S* = S' if reads_decayed else S; out = S^T r. k, c, p, r: float
// vectors of `dim` per (token, key group), rows key_row apart; dvec (or NULL) per (token, head), dscal / pscal /
// xscal (or NULL = 1) per (token, head), rows scal_row apart; x [.., heads x vdim] rows x_row apart; out likewise.
// reads_decayed 2 (with c = p = k and no dvec): the caller says that pscal is zero throughout, S = d S + k (xs x)^T.
int psamd_delta_scan(void* stream, const float* kvec, const float* cvec, const float* pvec, const float* rvec, int64_t key_row,
                     int key_groups, const float* dvec, int64_t dvec_row, const float* dscal, const float* pscal,
                     const float* xscal, int64_t scal_row, const float* x, int64_t x_row, float* out, int64_t out_row,
                     float* state, int64_t state_row, const int32_t* item_start, const int32_t* slots, int items, int heads,
                     int dim, int vdim, int reads_decayed);
// out[t, h, :] = o[t, h, :] / sqrt(mean(o^2) + eps) * weight * act(gate[t, h, :]); o float, weight float [vdim]
// (or [heads * vdim] with weight_per_head), gate rows gate_row apart in act_dtype, act 0 = SiLU, 1 = sigmoid.
int psamd_heads_norm_gate(void* stream, const float* o, int64_t tokens, int heads, int vdim, const float* weight,
                          int weight_per_head, float eps, const void* gate, int act_dtype, int64_t gate_row, int gate_act,
                          void* out);

// ---- several residual streams, side-by-side mixers, recurrences through the delta scan (streams.hip) ----
// x[r, :] <- weight * x[r, :] / sqrt(mean(x[r, :]^2) + eps), float, in place.
int psamd_stream_rms_norm(void* stream, float* x, const float* weight, float eps, int64_t rows, int hidden);
// out[t, :] = u / sqrt(mean(u^2) + eps) * weight (* factor), u = sum_s read[s] streams[s, t, :]; streams float
// [count, tokens, hidden], out in out_dtype.
int psamd_hyper_read(void* stream, const float* streams, int count, const float* read, const float* weight, float eps,
                     const float* factor, void* out, int out_dtype, int64_t tokens, int hidden);
// streams[t', t, :] <- sum_s mix[s, t'] streams[s, t, :] + write[t'] y[t, :], every copy from the old ones; y = a_scale a
// (+ b_scale b, b may be NULL), each one tensor in its dtype or float slices a stride apart.
int psamd_hyper_write(void* stream, float* streams, int count, const float* mix, const float* write, const void* a,
                      int a_dtype, int a_slices, int64_t a_stride, float a_scale, const void* b, int b_dtype, int b_slices,
                      int64_t b_stride, float b_scale, int64_t tokens, int hidden);
// out = a_scale * a + b_scale * b (float, n entries); a and b as the delta of psamd_hyper_write.
int psamd_weighted_sum(void* stream, const void* a, int a_dtype, int a_slices, int64_t a_stride, float a_scale, const void* b,
                       int b_dtype, int b_slices, int64_t b_stride, float b_scale, float* out, int64_t n);
// x <- f(x) in place; kind 0 = GELU (erf), 1 = GELU (tanh form), 2 = SiLU, 3 = ReLU.
int psamd_activation(void* stream, void* x, int act_dtype, int64_t n, int kind);
// out = v / sqrt(mean(v^2) + eps) * weight over each of `parts` equal parts of the row, v = (y + skip[head] x) silu(gate).
int psamd_gated_group_norm(void* stream, const float* y, const float* x, int64_t x_row, const float* skip, int heads,
                           const void* gate, int act_dtype, int64_t gate_row, const float* weight, int parts, float eps,
                           void* out, int64_t tokens, int inner);
// coef row [decay | 0 | step] (heads each): step = softplus(dt + dt_bias[h]), decay = exp(-exp(a_log[h]) step).
int psamd_state_space_prepare(void* stream, const float* dt, const float* dt_bias, const float* a_log, float* coef,
                              int64_t tokens, int heads);
// The exponential gates of a matrix memory with their running maximum (state[slot, h], read and left behind), item
// by item and token by token: coef row [keep | 0 | write | exp(-m)] (heads each).
int psamd_matrix_memory_gates(void* stream, const float* gates, const float* bias, float cap, float* coef, float* state,
                              int64_t state_row, const int32_t* item_start, const int32_t* slots, int items, int heads);
// u row [q * q_scale | k] float, vals row per head [v | 1] float, from rows in act_dtype.
int psamd_matrix_memory_operands(void* stream, const void* rows, int act_dtype, int64_t in_row, int q_col, int k_col, int v_col,
                                 int heads, int dim, int vdim, float q_scale, float* u, float* vals, int64_t tokens);
// raw row per head [S^T q | n . q]: o = S^T q / (max(|n . q|, floor[t, h]) + read_eps), then as psamd_heads_norm_gate
// with a weight over all heads and a sigmoid gate.
int psamd_memory_read_norm_gate(void* stream, const float* raw, const float* floor_, int64_t floor_row, int heads, int vdim,
                                float read_eps, const float* weight, float eps, const void* gate, int act_dtype,
                                int64_t gate_row, void* out, int64_t tokens);
// For every token whose pool_slot is >= 0: the mean key and value of the `block` tokens that end with it, from the
// token pages to place pool_slot of the pool's pages (both [blocks][2][kv_heads][16 * head_dim]).
int psamd_pool_kv_append(void* stream, const void* kv, void* pool, int act_dtype, const int32_t* positions,
                         const int32_t* tok_item, const int32_t* table_off, const int32_t* block_ids, const int32_t* pool_slot,
                         int64_t tokens, int hkv, int head_dim, int block);
// Attention in a sliding window that also sees the first keep_first positions and, with pool != NULL, one mean key
// and value per block of tokens wholly in front of the window; gate (float [tokens, hq] or NULL): output times sigmoid.
int psamd_attention_masked(void* stream, const void* qkv, int q_stride, void* out, const void* kv, int act_dtype,
                           int64_t tokens, const int32_t* positions, const int32_t* tok_item, const int32_t* table_off,
                           const int32_t* block_ids, int hq, int hkv, int head_dim, float scale, int window, int keep_first,
                           const void* pool, const int32_t* pool_table_off, const int32_t* pool_block_ids, int block,
                           const float* gate);
// The same on the matrix cores (bfloat16; shapes psamd_attention_mfma_supports takes, head sizes up to 192): the step's portions as tiles
// of 32 queries (pf_tiles) and its single tokens as tiles of one (dec_items).
int psamd_attention_masked_mfma(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                                const int32_t* pf_tiles, int n_tiles, const int32_t* dec_items, int n_dec, int max_kv_len,
                                const int32_t* item_start, const int32_t* item_pos0, const int32_t* table_off,
                                const int32_t* block_ids, int hq, int hkv, int head_dim, float scale, int window,
                                int keep_first, const void* pool, const int32_t* pool_table_off,
                                const int32_t* pool_block_ids, int block, const float* gate, int exact_weights);

// out[M, N] = x[M, K] * w[N, K]^T with float accumulation (LDS-tiled FMA; exact path and fallback).
int psamd_linear(void* stream, const void* x, int x_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                 int64_t M, int N, int K);

// Library product (hipBLASLt, looked up at run time) for large bfloat16 steps, with the
// descriptors and the chosen algorithm kept per shape. psamd_gemm_lt_available(): 1 if the
// library is ready on the current device; its first call per device allocates the workspace.
// use_workspace = 0: only algorithms that need none (for calls under stream capture).
// psamd_gemm_lt returns 2, not an error, if the library has no algorithm for the shape.
int psamd_gemm_lt_available();
int psamd_gemm_lt(void* stream, const void* x, const void* w, void* out, int out_dtype, int64_t M, int N, int K,
                  int use_workspace, int accumulate);


// bfloat16 product for M <= 64 on the matrix cores. epilogue 1: w = [gate; up], out = silu(gate) * up;
// 2 and 3: the same with ReLU and with GELU (tanh form) on the gate.
// ksplit > 1: out receives ksplit float32 partial sums [ksplit][M, n_out] (plain epilogue only).
int psamd_linear_skinny_ksplit(int M, int n_out, int K);
int psamd_linear_skinny(void* stream, const void* x, const void* w, void* out, int out_dtype, int M, int n_out, int K,
                        int epilogue, int ksplit);

// The q/k/v projection of a step of at most 64 tokens fused with the rotation of q and k and the write of k
// and v into their cache pages (see psamd_rope_kv_append for the meaning of table, kv and write_slot).
int psamd_qkv_rope_append(void* stream, const void* x, const void* w, void* qkv_out, int M, int K, int hq, int hkv,
                          int head_dim, const int32_t* positions, const float* table, void* kv,
                          const int32_t* write_slot);

// Small steps without a norm kernel and without partial slices to add up (bfloat16, M <= 16):
// the products that feed the residual stream add into it (psamd_linear_skinny_add: float atomics,
// K split over workgroups; the order of the additions differs from run to run), and the products
// that read the normalized stream (q/k/v, gate/up, the output matrix) take rows of the float32
// residual and apply the RMS norm themselves (weight norm_w, bfloat16 or float32; statistics in
// 32-bit, eps inside the root). psamd_normed_supports: whether they take M tokens of width K.
int psamd_normed_supports(int M, int K);
int psamd_linear_skinny_add(void* stream, const void* x, const void* w, float* out, int M, int n_out, int K);
int psamd_linear_normed(void* stream, const float* resid, const int32_t* rows, const void* norm_w, int norm_w_dtype,
                        float eps, const void* w, void* out, int out_dtype, int M, int n_out, int K, int epilogue);
int psamd_qkv_rope_append_normed(void* stream, const float* resid, const void* norm_w, int norm_w_dtype, float eps,
                                 const void* w, void* qkv_out, int M, int K, int hq, int hkv, int head_dim,
                                 const int32_t* positions, const float* table, void* kv, const int32_t* write_slot);

// sink (float [hq] or NULL): exp(sink[h]) is added to the softmax's denominator. dist_bias (float
// [hq, n_dist] or NULL): dist_bias[h, min(i - j, n_dist - 1)] is added to the scaled score of query i and key j.
int psamd_attention_generic(void* stream, const void* qkv, int q_stride, void* out, const void* kv, int act_dtype,
                            int64_t tokens, const int32_t* positions, const int32_t* tok_item,
                            const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                            float scale, int window, const float* sink, const float* dist_bias, int n_dist);

int psamd_attention_mfma_supports(int hq, int hkv, int head_dim);

// Few query tiles on long contexts: their keys are cut into nsplit runs (what
// psamd_attention_prefill_nsplit allows for the step's sizes, or fewer; 1: no cut) that
// part_o [32 * n_tiles * hq * nsplit * head_dim] and part_ml [32 * n_tiles * hq * nsplit * 2] carry
// to a merge kernel.
int psamd_attention_prefill_nsplit(int n_tiles, int max_kv_len, int hq, int hkv, int head_dim);
// exact_weights (here and in psamd_attention_decode): the softmax weights enter the second product
// as three bfloat16 terms whose sum is the float32 weight exactly, instead of rounded to bfloat16.
// pf_tiles: (item, first query) of every tile of 32 queries; pf_blocks: the first tile of every run
// of up to four consecutive tiles of one item, in the order of the tiles (n_blocks = 0: no such
// list; steps with one or two query heads per kv head then run a slower form).
// The most rows (32 * n_tiles * nsplit) of part_o / part_ml any step of this shape needs.
int psamd_attention_prefill_part_rows(int hq, int hkv, int head_dim);
int psamd_attention_prefill(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                            const int32_t* pf_tiles, int n_tiles, const int32_t* pf_blocks, int n_blocks, int max_kv_len,
                            const int32_t* item_start, const int32_t* item_pos0,
                            const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                            float scale, int window, float* part_o, float* part_ml, int nsplit, int exact_weights);

// The plan for a decode step's keys: whether its context lengths count as skewed (one far longer
// than the rest), into how many runs of at least how many keys each request's keys are cut, and
// the most (requests x runs) any plan gives (part_o: that many x hq x head_dim floats).
int psamd_attention_decode_skewed(int n_dec, int longest, int64_t total);
int psamd_attention_decode_plan(int n_dec, int kv_len, int skewed, int hkv, int window, int* nsplit, int* min_run);
int psamd_attention_decode_max_parts(int max_requests);

int psamd_attention_decode(void* stream, const void* qkv, int q_stride, void* out, const void* kv, float* part_o,
                           float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start,
                           const int32_t* item_end, const int32_t* table_off, const int32_t* block_ids, int hq,
                           int hkv, int head_dim, int nsplit, float scale, int window, int min_split_keys,
                           int exact_weights);

// psamd_attention_prefill and psamd_attention_decode with a sink and a bias by distance (see
// psamd_attention_generic for both; either may be NULL).
int psamd_attention_prefill_extras(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                                   const int32_t* pf_tiles, int n_tiles, const int32_t* pf_blocks, int n_blocks,
                                   int max_kv_len, const int32_t* item_start, const int32_t* item_pos0,
                                   const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                                   float scale, int window, float* part_o, float* part_ml, int nsplit, int exact_weights,
                                   const float* sink, const float* dist_bias, int n_dist);
int psamd_attention_decode_extras(void* stream, const void* qkv, int q_stride, void* out, const void* kv, float* part_o,
                                  float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start,
                                  const int32_t* item_end, const int32_t* table_off, const int32_t* block_ids, int hq,
                                  int hkv, int head_dim, int nsplit, float scale, int window, int min_split_keys,
                                  int exact_weights, const float* sink, const float* dist_bias, int n_dist);

// out[r] = argmax (temperature[r] <= 0) or the inverse-CDF draw with uniform[r] in [0, 1).
int64_t psamd_sample_scratch_floats(int rows);
int psamd_sample(void* stream, const float* logits, const float* temperature, const float* uniform, int32_t* out,
                 float* scratch, int rows, int vocab);

// psamd_sample for callers that cannot allocate or bring a scratch buffer (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc). It has no counterpart in the
// reference. The run statistics live in a 128 KiB array inside the library that every GPU holds
// until the process ends, so rows is limited to psamd_sample_static_max_rows() (256); more is an
// error. The call allocates nothing and calls no library routine that does; the caller passes
// inputs and outputs as for psamd_sample, with the stream's device current. All calls on one GPU
// share the array: two calls that overlap there (different streams, or two threads) race, and
// the caller has to order them. Same kernels and the same result as psamd_sample. The first
// call on a device asks the runtime for the array's address there (hipGetSymbolAddress, under
// a mutex): make it once at set-up, outside any graph capture; later calls only launch.
int psamd_sample_static_max_rows(void);
int psamd_sample_static(void* stream, const float* logits, const float* temperature, const float* uniform,
                        int32_t* out, int rows, int vocab);

#ifdef __cplusplus
}
#endif
