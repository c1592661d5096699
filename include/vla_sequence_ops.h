/* C-ABI of libvla_seq_gfx950.so: the layers of decoder stacks that keep their residual stream in
 * fp32 and mix tokens with a paged sliding-window attention and / or a gated linear recurrence.
 *
 * Conventions are those of vla_paged_attention.h: raw device pointers, element strides, VLA_F16 /
 * VLA_BF16 / VLA_F32 codes for the activation dtype, a hipStream_t, VLA_OK or a VLA_ERR_* code
 * back; nothing is allocated, every launch goes to the caller's stream and can be captured.
 *
 * A step is a packed batch of `num_tokens` rows that belong to `num_seqs` sequences: sequence b
 * owns rows query_start_loc[b] .. query_start_loc[b + 1] - 1, its tokens continue
 * context_lens[b] tokens that earlier steps left in the cache / state.  A decode step is the
 * case of one row per sequence; a prompt (or any portion of one) is the case of several.  The
 * same kernels serve both, so a position's result does not depend on how its sequence was cut.
 */
#ifndef VLA_SEQUENCE_OPS_H
#define VLA_SEQUENCE_OPS_H

#include <stdint.h>

#include "vla_paged_attention.h"

#ifdef __cplusplus
extern "C" {
#endif

int vla_seq_last_hip_error(void);

/* out[t, :] = table[ids[t], :] + pe(positions[t]) in fp32, pe[2i] = sin(p * inv_freq[i]),
 * pe[2i + 1] = cos(p * inv_freq[i]).  table is `dtype`, inv_freq fp32 [(width + 1) / 2]
 * (null: no position term). */
int vla_seq_embed_positions(float* out, const void* table, const int64_t* ids,
                            const int64_t* positions, const float* inv_freq, int num_tokens,
                            int width, int vocab, int dtype, void* stream);

/* RMS norm of an fp32 stream with a single gain: first x += add_rows + add_row (either may be
 * null; add_rows [T, width] fp32, add_row [width] fp32; x is written back when one is given),
 * then out = dtype(x / sqrt(mean(x^2) + eps) * gain[0]). */
int vla_seq_scalar_rms_norm(void* out, float* x, const float* add_rows, const float* add_row,
                            const float* gain, float eps, int num_tokens, int width, int dtype,
                            void* stream);

/* x[fp32] += y[dtype], elementwise over n values. */
int vla_seq_residual_add(float* x, const void* y, int64_t n, int dtype, void* stream);

/* PolyNorm: out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 per row of `features` values,
 * N(u) = u / sqrt(mean(u^2) + eps); coef fp32 [4] on the device; fp32 arithmetic. */
int vla_seq_poly_norm(void* out, int64_t out_stride, const void* z, int64_t z_stride,
                      const float* coef, float eps, int num_tokens, int features, int dtype,
                      void* stream);

/* Per (token, head): out = dtype(o / sqrt(mean_v(o^2) + eps) * weight[v] * silu(gate) * scale);
 * o fp32 [T, heads, vdim] contiguous, weight fp32 [vdim], gate / out `dtype` rows of
 * heads * vdim with their own strides. */
int vla_seq_gated_head_rms_norm(void* out, int64_t out_stride, const float* o,
                                const float* weight, const void* gate, int64_t gate_stride,
                                float eps, float scale, int num_tokens, int heads, int vdim,
                                int dtype, void* stream);

/* Keys of a step into the paged key cache [num_blocks, block_size, kv_heads, dim] (`dtype`);
 * slot = block * block_size + offset, negative = skip. */
int vla_seq_key_cache_write(void* cache, const void* k, int64_t k_stride,
                            const int64_t* slot_mapping, int num_tokens, int kv_heads, int dim,
                            int block_size, int num_blocks, int dtype, void* stream);

/* Sliding-window attention over the paged key cache whose values are its keys.
 * For the token at position p of sequence b and query head h (KV head h / (heads / kv_heads)):
 *   s_j = (q . k_j) * scale * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1))
 *         - slopes[h] * (p - j)            for max(0, p - window + 1) <= j <= p
 *   out = sum_j softmax(s)_j k_j, then * sigmoid(gate) (gate null: no gate) * out_scale.
 * All of it fp32; the step's own keys must be in the cache already.  slopes null = no bias,
 * temp_coef 0 = no temperature, window <= 0 = everything before p.  token_seq [T] names each
 * row's sequence; positions int64 [T]; block_tables int32 [num_seqs, max_blocks]. */
int vla_seq_window_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                             const void* gate, int64_t gate_stride, const void* cache,
                             const int* block_tables, int max_blocks, const int* token_seq,
                             const int64_t* positions, const float* slopes, int num_tokens,
                             int heads, int kv_heads, int dim, int block_size, int num_blocks,
                             int window, float scale, float temp_coef, float temp_every,
                             float out_scale, int dtype, void* stream);

/* Log-decays of a gated linear recurrence from a low-rank projection:
 * out[t, c] = -softplus(-(sum_r w2[c, r] y[t, r] + bias[c])) * inv_tau   (= ln sigmoid(z)^(1/tau)),
 * fp32; y `dtype` [T, rank] with stride, w2 `dtype` [channels, rank], bias fp32 [channels]. */
int vla_seq_gla_log_decay(float* out, const void* y, int64_t y_stride, const void* w2,
                          const float* bias, float inv_tau, int num_tokens, int channels,
                          int rank, int dtype, void* stream);

/* Gated linear attention with a per-key-channel decay, state carried in fp32 slots:
 *   S_t = diag(exp(g_t)) S_(t-1) + k_t v_t^T,   o_t = S_t^T (q_t * q_scale)
 * per head, S [dim, vdim].  Sequence b starts from zero when context_lens[b] == 0 and from
 * state[state_slots[b]] otherwise, and leaves its state there.  q, k [T, heads * dim] and
 * v [T, heads * vdim] `dtype` with strides, log_decay fp32 [T, heads * dim], o fp32
 * [T, heads, vdim], state fp32 [num_slots, heads, dim, vdim].  max_query_len: the longest run of
 * rows of one sequence in the step, or 0 if unknown (a hint that sizes the staging buffers). */
int vla_seq_gla_scan(float* o, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                     const void* v, int64_t v_stride, const float* log_decay, float* state,
                     const int* query_start_loc, const int* context_lens, const int* state_slots,
                     float q_scale, int num_seqs, int num_slots, int max_query_len, int heads,
                     int dim, int vdim, int dtype, void* stream);

/* A long run of rows cut into pieces that are walked at once (each from a zero state, through
 * vla_seq_gla_scan with one entry per piece): with c_t the sum of the log decays from a piece's
 * first row to row t, vla_seq_gla_piece_prefix writes q_decayed[t] = q[t] * q_scale * exp(c_t)
 * (fp32 [T, channels], channels = heads * dim) and totals[piece] = exp(c_last) for the pieces
 * piece_start_loc[i] .. piece_start_loc[i + 1] - 1; the caller adds q_decayed S_start to the
 * outputs of each piece (a matrix product).  vla_seq_gla_combine_states walks one sequence's
 * pieces: state[slots[i]] <- totals[pieces[i]] (per key channel) * state[slots[i - 1]] +
 * state[slots[i]] for i = 1 .. count - 1, then state[final_slot] <- state[slots[count - 1]]. */
int vla_seq_gla_piece_prefix(float* q_decayed, float* totals, const void* q, int64_t q_stride,
                             const float* log_decay, const int* piece_start_loc, float q_scale,
                             int num_pieces, int channels, int dtype, void* stream);
int vla_seq_gla_combine_states(float* state, const int* slots, const int* pieces,
                               const float* totals, int count, int final_slot, int num_slots,
                               int heads, int dim, int vdim, void* stream);

/* The same attention for 16-bit activations, tiled over runs of 32 query rows of a sequence on
 * the matrix cores: rows query_start_loc[b] .. query_start_loc[b + 1] - 1 of sequence b sit at
 * positions context_lens[b] ...  dim must be a multiple of 32, at most 128
 * (vla_seq_window_attention_tiles_supported); query rows and cache rows must be 8-byte aligned. */
int vla_seq_window_attention_tiles_supported(int dim, int dtype);
int vla_seq_window_attention_tiles(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                   const void* gate, int64_t gate_stride, const void* cache,
                                   const int* block_tables, int max_blocks,
                                   const int* query_start_loc, const int* context_lens,
                                   const float* slopes, int num_seqs, int max_query_len, int heads,
                                   int kv_heads, int dim, int block_size, int num_blocks,
                                   int window, float scale, float temp_coef, float temp_every,
                                   float out_scale, int dtype, void* stream);

/* ---- layers that norm a sublayer's input and its output -------------------------------------- */

/* Activation codes of vla_seq_gated_act / vla_seq_grouped_linear. */
#define VLA_ACT_NONE 0
#define VLA_ACT_RELU 1
#define VLA_ACT_RELU2 2      /* relu(z)^2 */
#define VLA_ACT_SILU 3
#define VLA_ACT_GELU_TANH 4  /* 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) */

/* One launch around a sublayer, on the fp32 stream x [T, width] (in place):
 *   y given:        y' = y + y_bias (null: none);
 *                   x += y' / sqrt(mean(y'^2) + eps) * post_weight * layer_scale (layer_scale null: 1)
 *   add_row given:  x += add_row
 *   out given:      out = out_dtype(x / sqrt(mean(x^2) + eps) * pre_weight), or out_dtype(x) when
 *                   pre_weight is null
 * y is `y_dtype` rows of `width` values with stride y_stride; weights, layer_scale, add_row fp32
 * [width].  All of it fp32. */
int vla_seq_residual_norms(float* x, const void* y, int64_t y_stride, int y_dtype,
                           const float* y_bias, const float* post_weight, const float* layer_scale,
                           const float* add_row, void* out, const float* pre_weight, float eps,
                           int num_tokens, int width, int out_dtype, void* stream);

/* Causal convolution over time on each channel, added to its input:
 *   out[t] = dtype(h[t] + sum_j weight[:, j] h[t - taps + 1 + j]),  zeros before a sequence's start,
 * h fp32 [T, width], weight fp32 [width, taps].  The last taps - 1 inputs of a sequence live in
 * state fp32 [num_slots, taps - 1, width] (oldest first): rows of earlier steps are read from
 * there, and the step leaves its own last inputs there.  taps <= 32. */
int vla_seq_causal_conv(void* out, const float* h, const float* weight, float* state,
                        const int* query_start_loc, const int* context_lens,
                        const int* state_slots, const int* token_seq, int num_tokens, int num_seqs,
                        int num_slots, int width, int taps, int dtype, void* stream);

/* out[t] = dtype([a[t]; b[t]]), a and b fp32 [T, width], out [T, 2 width]. */
int vla_seq_concat_cast(void* out, const float* a, const float* b, int num_tokens, int width,
                        int dtype, void* stream);

/* out = act(gate) * up (up null: act(gate)); rows of `features` values with their own strides. */
int vla_seq_gated_act(void* out, int64_t out_stride, const void* gate, int64_t gate_stride,
                      const void* up, int64_t up_stride, int num_tokens, int features, int act,
                      int dtype, void* stream);

/* out = g * sigmoid(alpha g) * (u + shift) with g = min(gate, limit), u = clamp(up, -limit, limit);
 * rows of `features` values with their own strides, fp32 arithmetic. */
int vla_seq_clamped_glu(void* out, int64_t out_stride, const void* gate, int64_t gate_stride,
                        const void* up, int64_t up_stride, int num_tokens, int features, float limit,
                        float alpha, float shift, int dtype, void* stream);

/* out[t] (fp32 [T, width]) = table[ids[t]] + pair_table[r], r = (prev * mul_prev + ids[t] * mul_cur)
 * mod buckets with prev the token before t in its sequence, r = buckets for a sequence's first
 * token (pair_table has buckets + 1 rows).  The token before a step's first row is read from
 * last_token[state_slots[b]] (int64 [num_slots]) when context_lens[b] > 0; afterwards every
 * sequence's slot receives its last token of the step. */
int vla_seq_pair_hash_embed(float* out, const void* table, const void* pair_table,
                            const int64_t* ids, int64_t* last_token, const int* query_start_loc,
                            const int* context_lens, const int* state_slots, const int* token_seq,
                            int num_tokens, int num_seqs, int num_slots, int width, int vocab,
                            int64_t buckets, int64_t mul_prev, int64_t mul_cur, int dtype,
                            void* stream);

/* ---- attention over paged key and value caches with rotary positions ------------------------- */

/* Rotates the step's queries in place and writes its rotated keys and values to the caches
 * (keys [num_blocks, block_size, kv_heads, dim], values [.., kv_heads, vdim], `dtype`).  Pair i of
 * the first rot_dims elements of a query / key head -- elements (2i, 2i + 1) when interleaved,
 * (i, i + rot_dims / 2) otherwise -- turns by positions[t] * inv_freq[i]: (a, b) ->
 * (a cos - b sin, b cos + a sin).  value_inv_freq [vdim / 2] (null: values are cached as they
 * are) turns the pairs of a value head over all vdim elements the same way.  Angles are fp32
 * products.  slot_mapping < 0 skips the caches.  q_norm [heads * dim] / k_norm [kv_heads * dim]
 * (fp32, null: none): the whole query / key row is divided by its root mean square (norm_eps inside
 * the root) and multiplied by these weights before it is rotated.  v_other (null: none; rows of
 * kv_heads * vdim values, not together with value_inv_freq): the cached value is
 * (1 - v_blend[0]) v + v_blend[0] v_other, v_blend one fp32 number on the device. */
int vla_seq_rotary_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride,
                            const void* v, int64_t v_stride, void* key_cache, void* value_cache,
                            const int64_t* positions, const int64_t* slot_mapping,
                            const float* inv_freq, const float* value_inv_freq, int num_tokens,
                            int heads, int kv_heads, int dim, int vdim, int rot_dims,
                            int interleaved, int block_size, int num_blocks, int dtype,
                            const float* q_norm, const float* k_norm, float norm_eps,
                            const void* v_other, int64_t v_other_stride, const float* v_blend,
                            void* stream);

/* For the token at position p of sequence b and query head h (KV head h / (heads / kv_heads)):
 *   s_j = (q . k_j) * scale  for max(0, p - window + 1) <= j <= p  (window <= 0: all j <= p)
 *         and, with a window, for j < keep_first as well (a sequence's first tokens stay visible)
 *   s_j <- softcap * tanh(s_j / softcap)                      (softcap 0: no cap)
 *   o = sum_j softmax(s)_j v_j;  out_inv_freq given: pair m of o turns by -p * out_inv_freq[m]
 *   out = dtype(o * sigmoid(gate[t, h]))                      (gate null: no gate)
 * in fp32; the step's own keys and values must be in the caches already.  gate holds one number
 * per (token, head) with row stride gate_stride. */
int vla_seq_kv_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                         const void* gate, int64_t gate_stride, const void* key_cache,
                         const void* value_cache, const int* block_tables, int max_blocks,
                         const int* token_seq, const int64_t* positions, const float* out_inv_freq,
                         int interleaved, int num_tokens, int heads, int kv_heads, int dim, int vdim,
                         int block_size, int num_blocks, int window, float scale, int dtype,
                         int keep_first, float softcap, void* stream);

/* The same attention for 16-bit activations, tiled over runs of 32 query rows of a sequence on
 * the matrix cores: rows query_start_loc[b] .. query_start_loc[b + 1] - 1 of sequence b sit at
 * positions context_lens[b] ...  dim and vdim must be multiples of 32, at most 128
 * (vla_seq_kv_attention_tiles_supported); query rows and cache rows must be 8-byte aligned.
 * vla_seq_kv_attention takes single rows of such shapes to the matrix cores by itself;
 * vla_seq_set_kv_attention_kernel(1) keeps both off them (tests run both), 0 is the default. */
int vla_seq_kv_attention_tiles_supported(int dim, int vdim, int dtype);
int vla_seq_kv_attention_tiles(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                               const void* gate, int64_t gate_stride, const void* key_cache,
                               const void* value_cache, const int* block_tables, int max_blocks,
                               const int* query_start_loc, const int* context_lens,
                               const float* out_inv_freq, int interleaved, int num_seqs,
                               int max_query_len, int heads, int kv_heads, int dim, int vdim,
                               int block_size, int num_blocks, int window, float scale, int dtype,
                               int keep_first, float softcap, void* stream);
int vla_seq_set_kv_attention_kernel(int mode);

/* ---- element-wise gated recurrence (minGRU) ---------------------------------------------------- */

/* S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, z = sigmoid(zp), c = up + 1/2 where up >= 0 and
 * sigmoid(up) below; out = dtype(S_t * silu(gp)).  zp, up, gp, out: `dtype` rows of `channels`
 * values with their own strides; state fp32 [num_slots, channels]; a sequence with context 0
 * starts from zero.  Runs of 256 rows and more are cut into pieces that are walked at once when
 * scratch (fp32, vla_seq_mingru_scratch_floats values) is given. */
int64_t vla_seq_mingru_scratch_floats(int num_seqs, int max_query_len, int channels);
int vla_seq_mingru_scan(void* out, int64_t out_stride, const void* zp, int64_t z_stride,
                        const void* up, int64_t u_stride, const void* gp, int64_t g_stride,
                        float* state, const int* query_start_loc, const int* context_lens,
                        const int* state_slots, int num_seqs, int num_slots, int max_query_len,
                        int channels, float* scratch, int64_t scratch_floats, int dtype,
                        void* stream);

/* ---- mixture of experts in the activation dtype -------------------------------------------------- */

/* Router of one token over `routed` experts (at most 512): z = router h + bias in fp32 (router
 * fp32 [routed, width], bias fp32 [routed] or null), s = softmax(z), the `top` largest s +
 * correction (null: s) are chosen, weights = their s / (sum + 1e-20) -- without a correction that
 * is the softmax over the chosen logits.  experts int32 / weights fp32 [T, top].  shared_gate given:
 * shared_gate[t] = sigmoid(shared_gate_weight . h), shared_gate_weight fp32 [width].  logits given
 * (fp32 rows of routed (+ 1 with a shared gate, its logit last) values, stride logits_stride): the
 * products are the caller's and h, router, shared_gate_weight are not read. */
int vla_seq_moe_route(const void* h, int64_t h_stride, const float* router, const float* logits,
                      int64_t logits_stride, const float* bias, const float* correction,
                      const float* shared_gate_weight, int* experts, float* weights,
                      float* shared_gate, int num_tokens, int width, int routed, int top, int dtype,
                      void* stream);

/* Groups the pairs (token, choice) whose expert is below num_experts by expert, every group padded
 * to whole tiles of vla_seq_moe_tile_rows() rows: pair_row int32 [T * top] (-1: the pair's expert
 * has no weights), row_token int32 [max_tiles * tile rows] (-1: padding), tile_expert int32
 * [max_tiles] (-1: unused).  max_tiles >= (T * top + (tile rows - 1) * min(num_experts, T * top))
 * / tile rows, rounded up, holds every case. */
int vla_seq_moe_tile_rows(void);
int vla_seq_moe_plan(const int* experts, int num_tokens, int top, int num_experts, int* pair_row,
                     int* row_token, int* tile_expert, int max_tiles, void* stream);

/* out[row, :] = out_dtype(act(weight[e] a[src(row)])) for the rows of every tile, e =
 * tile_expert[tile] (tiles with -1 are skipped), src(row) = row_token[row] (null: row; -1: a zero
 * row).  weight `dtype` [experts, n_out, k_in], a `dtype` rows of k_in values. */
int vla_seq_grouped_linear(void* out, int64_t out_stride, int out_dtype, const void* a,
                           int64_t a_stride, const int* row_token, const void* weight,
                           const int* tile_expert, int max_tiles, int n_out, int k_in, int act,
                           int dtype, void* stream);

/* Form of the 16-bit product for tests: 0 = per shape, 1 = one-wave workgroups (decode steps),
 * 2 = runs of tiles per workgroup (prompts). */
int vla_seq_set_grouped_linear_form(int mode);

/* out[t] (fp32 [T, width]) = sum_k weights[t, k] * (y[pair_row[t, k]] or, where pair_row is -1,
 * h[t]) + shared_gate[t] * shared_y[t] (shared_y null: none; shared_gate null: 1).  y, shared_y
 * fp32 rows of `width`. */
int vla_seq_moe_combine(float* out, const float* y, const int* pair_row, const float* weights,
                        const void* h, int64_t h_stride, const float* shared_y,
                        const float* shared_gate, int num_tokens, int width, int top, int dtype,
                        void* stream);

/* ---- layers that norm the stream itself after every sublayer --------------------------------------- */

/* x (fp32 [T, width], in place) <- (alpha x + y) / sqrt(mean((alpha x + y)^2) + eps) * weight;
 * out (null: none) = out_dtype(new x).  y: `y_dtype` rows of `width` values with stride y_stride. */
int vla_seq_post_norm(float* x, float alpha, const void* y, int64_t y_stride, int y_dtype,
                      const float* weight, float eps, void* out, int out_dtype, int num_tokens,
                      int width, void* stream);

/* out = out_dtype(in / sqrt(mean(in^2) + eps) * weight) per row of n values; fp32 arithmetic. */
int vla_seq_rms_norm_rows(void* out, int64_t out_stride, int out_dtype, const void* in,
                          int64_t in_stride, int in_dtype, const float* weight, float eps,
                          int num_tokens, int n, void* stream);

/* Causal convolution over time on each channel:
 *   out[t] = out_dtype(act(bias + sum_j weight[:, j] u[t - taps + 1 + j])),  zeros before a
 * sequence's start; weight fp32 [channels, taps], bias fp32 [channels] or null, act a VLA_ACT_*
 * code.  The last taps - 1 inputs of a sequence live in state fp32 [num_slots, taps - 1, channels]
 * (oldest first): rows of earlier steps are read from there, and the step leaves its own last
 * inputs there.  taps <= 32. */
int vla_seq_short_conv(void* out, int64_t out_stride, int out_dtype, const void* u, int64_t u_stride,
                       int u_dtype, const float* weight, const float* bias, float* state,
                       const int* query_start_loc, const int* context_lens, const int* state_slots,
                       const int* token_seq, int num_tokens, int num_seqs, int num_slots,
                       int channels, int taps, int act, void* stream);

/* out[t, c] = out_dtype(act(gate[t, c]) * table[ids[t], first_col + c]), c < features. */
int vla_seq_gated_act_lookup(void* out, int64_t out_stride, int out_dtype, const void* gate,
                             int64_t gate_stride, int gate_dtype, const void* table,
                             int64_t table_stride, int table_dtype, const int64_t* ids, int rows,
                             int first_col, int num_tokens, int features, int act, void* stream);

/* out[t, :] (fp32) = table[ids[t], :] * scale. */
int vla_seq_embed_scaled(float* out, const void* table, const int64_t* ids, float scale,
                         int num_tokens, int width, int vocab, int dtype, void* stream);

/* z <- cap * tanh(z / cap) over n fp32 values. */
int vla_seq_softcap(float* z, int64_t n, float cap, void* stream);

/* ---- gated delta rule ----------------------------------------------------------------------------- */

/* Per head, with a state S fp32 [dim, vdim] per sequence (stored [num_slots, heads, vdim, dim]):
 *   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
 * k, q of the head's key head (heads / kv_heads value heads share one) divided by
 * sqrt(sum of squares + 1e-6), q also times dim^-1/2; beta = sigmoid(beta row); g = exp(-exp(a_log)
 * softplus(dt row + dt_bias)); out = out_dtype(o / sqrt(mean_v(o^2) + eps) * norm_weight *
 * silu(gate)).  q, k [T, kv_heads * dim], v, gate, out [T, heads * vdim], beta, dt [T, heads]:
 * rows with their own strides, inputs fp32 (in_dtype VLA_F32).  A sequence with context 0 starts
 * from zero.  scratch: fp32, vla_seq_delta_rule_scratch_floats values (the heads' outputs between
 * the walk and their norm).  max_query_len: the longest run of the step (0: unknown).  dim up to
 * 1024. */
int64_t vla_seq_delta_rule_scratch_floats(int num_tokens, int heads, int vdim);
/* Kernel choice for tests: 0 = per step (runs of at most four rows skip the LDS staging), 1 = always
 * without staging, 2 = never. */
int vla_seq_set_delta_kernel(int mode);
int vla_seq_delta_rule_scan(void* out, int64_t out_stride, int out_dtype, const void* q,
                            int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                            int64_t v_stride, const void* gate, int64_t gate_stride,
                            const void* beta, int64_t beta_stride, const void* dt, int64_t dt_stride,
                            int in_dtype, const float* a_log, const float* dt_bias,
                            const float* norm_weight, float* state, const int* query_start_loc,
                            const int* context_lens, const int* state_slots, int num_tokens,
                            int num_seqs, int max_query_len, int num_slots, int heads, int kv_heads,
                            int dim, int vdim, float eps, float* scratch, void* stream);

/* ---- real-gated linear recurrent unit ------------------------------------------------------------- */

/* S_t = a S_(t-1) + sqrt(1 - a^2) sigmoid(i) u per channel, a = exp(-rate sigmoid(r));
 * out = out_dtype(S_t * gelu_tanh(y)).  u, y fp32 rows of `channels` values with their own
 * strides; the gates' rows r, i come in blocks of gate_block channels, channel c of token t at
 * t * stride + (c / gate_block) * gate_block_stride + c % gate_block (the blocks of a batched
 * product; plain rows: gate_block = channels); rate fp32 [channels], state fp32 [num_slots,
 * channels]; scratch as for
 * vla_seq_mingru_scan (vla_seq_mingru_scratch_floats values). */
int vla_seq_rglru_scan(void* out, int64_t out_stride, int out_dtype, const float* r, int64_t r_stride,
                       const float* i, int64_t i_stride, int gate_block, int64_t gate_block_stride,
                       const float* u, int64_t u_stride,
                       const float* y, int64_t y_stride, const float* rate, float* state,
                       const int* query_start_loc, const int* context_lens, const int* state_slots,
                       int num_seqs, int num_slots, int max_query_len, int channels, float* scratch,
                       int64_t scratch_floats, void* stream);

/* ---- attention over a cached latent ----------------------------------------------------------------- */

/* cache [num_blocks, block_size, rank + rot] (`dtype`): per token the normed latent and the rotated
 * key part every head shares.  Rotates the rot_dims first elements of every head's rotated query
 * part in place (head h's part starts at q + t q_stride + h q_head_stride + q_first; pairs
 * (2i, 2i + 1) when interleaved, (i, i + rot_dims / 2) otherwise, turn by positions[t] * inv_freq[i],
 * sine and cosine times `magnitude`) and
 * writes the rows [kv[:rank] / sqrt(mean^2 + eps) * norm_weight | kv[rank:] rotated the same way].
 * slot_mapping < 0 skips the cache. */
int vla_seq_latent_rotary_write(void* q, int64_t q_stride, int q_head_stride, int q_first,
                                const void* kv, int64_t kv_stride, const float* norm_weight,
                                float eps, void* cache, const int64_t* positions,
                                const int64_t* slot_mapping, const float* inv_freq, float magnitude,
                                int num_tokens, int heads, int rank, int rot, int rot_dims,
                                int block_size, int num_blocks, int dtype, int interleaved,
                                void* stream);

/* out[t, h, :rank] = sum_j p_j c_j over the keys j <= position of the row's sequence, p = softmax
 * of (q_lat[t, h] . c_j + q_rot[t, h] . k_rot_j) * scale; q_lat, q_rot and out are addressed by a
 * token stride and a head stride each.  window > 0 keeps the keys with position - j < window only;
 * gate (null: none; one number per (token, head), row stride gate_stride) multiplies a head's sums
 * by its sigmoid.  Any dtype, rank and rot up to 1024. */
int vla_seq_latent_attention(void* out, int64_t out_token_stride, int64_t out_head_stride,
                             const void* q_lat, int64_t lat_token_stride, int64_t lat_head_stride,
                             const void* q_rot, int64_t rot_token_stride, int64_t rot_head_stride,
                             const void* cache, const int* block_tables, int max_blocks,
                             const int* token_seq, const int64_t* positions, int num_tokens,
                             int heads, int rank, int rot, int block_size, int num_blocks,
                             float scale, int dtype, int window, const void* gate,
                             int64_t gate_stride, void* stream);

/* The same attention on the matrix cores for 16-bit models: 32 query rows that are (token, head)
 * pairs of one sequence per workgroup, tiles of 32 keys.  rank a multiple of 32 up to 512, rot a
 * multiple of 16 (vla_seq_latent_attention_tiles_supported); query and cache rows must be 16-byte
 * aligned.  Rows query_start_loc[b] .. of sequence b sit at positions context_lens[b] ...
 * key_splits > 1 shares the keys of every row tile out to that many workgroups and merges their
 * sums in a second launch (few rows over long contexts); scratch then holds
 * vla_seq_latent_attention_scratch_floats fp32 values and num_tokens is the step's row count.
 * vla_seq_set_latent_attention_kernel(1) keeps it off (tests run both), 0 is the default. */
int vla_seq_latent_attention_tiles_supported(int rank, int rot, int dtype);
int64_t vla_seq_latent_attention_scratch_floats(int key_splits, int num_tokens, int heads, int rank);
int vla_seq_latent_attention_tiles(void* out, int64_t out_token_stride, int64_t out_head_stride,
                                   const void* q_lat, int64_t lat_token_stride,
                                   int64_t lat_head_stride, const void* q_rot,
                                   int64_t rot_token_stride, int64_t rot_head_stride,
                                   const void* cache, const int* block_tables, int max_blocks,
                                   const int* query_start_loc, const int* context_lens,
                                   int num_seqs, int max_query_len, int heads, int rank, int rot,
                                   int block_size, int num_blocks, float scale, int key_splits,
                                   float* scratch, int num_tokens, int dtype, int window,
                                   const void* gate, int64_t gate_stride, void* stream);
int vla_seq_set_latent_attention_kernel(int mode);

/* Kernel choice for tests: window attention 0 = per shape, 1 = one wave per (row, head);
 * scan 0 = per shape, 1 = token by token. */
int vla_seq_set_window_kernel(int mode);
int vla_seq_set_scan_kernel(int mode);

#ifdef __cplusplus
}
#endif
#endif
